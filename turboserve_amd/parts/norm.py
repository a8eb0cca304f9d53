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


@register_norm("tanh_norm")
class TanhNorm(Norm):
    """A norm that computes no mean or variance: ``tanh(alpha x) * weight + bias`` with a learned scalar
    ``alpha`` and vectors ``weight``, ``bias`` of the row's size, in 32-bit with one rounding.  The fused form
    also carries the residual sum, kept in 32-bit.  ``weight_name``: the weight's name under the part's
    prefix (empty: the prefix itself); ``alpha_name`` and ``bias_name`` are appended to the weight's name."""

    def __init__(self, prefix: str, runtime: Runtime, *, size: int, weight_name: str = "weight", alpha_name: str = "alpha",
                 bias_name: str = "b", initial_alpha: float = 0.5) -> None:
        super().__init__(prefix, runtime)
        self.size = int(size)
        self.weight_name, self.alpha_name, self.bias_name = weight_name, alpha_name, bias_name
        self.initial_alpha = float(initial_alpha)
        self.weight: torch.Tensor | None = None
        self.bias: torch.Tensor | None = None
        self.alpha = self.initial_alpha

    def _beside(self, suffix: str) -> str:
        return f"{self.name(self.weight_name)}.{suffix}"

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {
            self.name(self.weight_name): TensorSpec((self.size,), init="ones"),
            self._beside(self.bias_name): TensorSpec((self.size,), init="zeros"),
            self._beside(self.alpha_name): TensorSpec((), init=f"constant:{self.initial_alpha}"),
        }

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        return tokens * self.size * itemsize

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name(self.weight_name)].contiguous()
        self.bias = tensors[self._beside(self.bias_name)].contiguous()
        self.alpha = float(tensors[self._beside(self.alpha_name)].float().item())

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError(f"{self.prefix}: this norm runs where it carries the residual sum")

    def forward_residual(self, stream: ResidualStream, rows: torch.Tensor | None = None) -> torch.Tensor:
        if stream.pending_norm is not None:
            raise ValueError(f"{self.prefix}: a pending output with a norm of its own is added by a norm with statistics")
        y = self.runtime.ops.add_tanh_norm(stream.residual, stream.pending, self.weight, self.bias, self.alpha, rows,
                                           also=stream.also)
        if rows is None:
            stream.pending = stream.also = None
        return y
