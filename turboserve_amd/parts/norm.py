"""RMSNorm (src/turboserve/engine/model/layers.py:178-211)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import Norm, ResidualStream, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    """``weight * round(x * rsqrt(mean(x^2) + eps))``: statistics in 32-bit, the normalised
    value rounded to the run dtype before the gain (layers.py:202-208).  The fused form also
    carries the residual sum, kept in 32-bit.

    With ``one_rounding`` the whole norm is 32-bit arithmetic that is rounded once, at the end:
    ``round(x * rsqrt(mean(x^2) + eps) * (gain_offset + weight))``; ``gain_offset = 1`` is a gain
    that is stored around zero.  ``weight_name``: the tensor's name under the part's prefix
    (empty: the prefix itself is the tensor's name)."""

    def __init__(self, prefix: str, runtime: Runtime, *, size: int, eps: float, gain_offset: float = 0.0,
                 one_rounding: bool = False, weight_name: str = "weight") -> None:
        super().__init__(prefix, runtime)
        self.size = int(size)
        self.eps = float(eps)
        self.gain_offset = float(gain_offset)
        self.one_rounding = bool(one_rounding)
        if self.gain_offset != 0.0 and not self.one_rounding:
            raise ValueError("a gain offset is applied in 32-bit: it needs one_rounding")
        self.weight_name = weight_name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name(self.weight_name): TensorSpec((self.size,), init="zeros" if self.gain_offset == 1.0 else "ones")}

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        return tokens * self.size * itemsize

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name(self.weight_name)].contiguous()

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.runtime.ops.rmsnorm(x, self.weight, self.eps, gain_offset=self.gain_offset, one_rounding=self.one_rounding)

    def forward_residual(self, stream: ResidualStream, rows: torch.Tensor | None = None) -> torch.Tensor:
        y = self.runtime.ops.add_rmsnorm(stream.residual, stream.pending, self.weight, self.eps, rows,
                                         gain_offset=self.gain_offset, one_rounding=self.one_rounding, also=stream.also,
                                         pending_norm=stream.pending_norm)
        if rows is None:
            stream.pending = stream.also = stream.pending_norm = None
        return y

    def pending_rule(self, scale: float) -> tuple:
        if self.gain_offset != 0.0:
            raise ValueError(f"{self.prefix}: a norm on a pending output takes its gain as stored (no offset)")
        return (self.weight, self.eps, float(scale))
