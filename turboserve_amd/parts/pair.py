"""Two mixers side by side: both read the same input, and what the stream gets is a weighted sum of
their outputs."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import CacheNeed, Mixer, PartSpec, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_mixer


def _flat(need: CacheNeed) -> tuple:
    if need is None:
        return ()
    return tuple(need) if isinstance(need, (tuple, list)) else (need,)


@register_mixer("mixer_pair")
class MixerPair(Mixer):
    """``left_scale * left(x) + right_scale * right(x)``, ``left`` and ``right`` any two registered mixers
    (their tensors under ``<prefix>.<left_name>`` and ``<prefix>.<right_name>``).  The pair's cache need is
    the two mixers' needs one after the other; each gets its own views back.

    Where both mixers end in an output matrix and can scale and place what that matrix multiplies (``heads_out(...,
    scale, out)``, ``scales_its_heads()``), the two output matrices are held side by side as one, ``[hidden, K_left
    + K_right]``: each side writes its heads' output, times its weight, into its columns of one buffer, and one
    product makes the weighted sum (a bias is multiplied by its side's weight at load).  Otherwise the sum is
    formed in 32-bit from whatever the two leave (tensors of the run dtype or 32-bit partial sums,
    ``ops.scaled_pair``) and handed on as one 32-bit partial sum for the residual stream."""

    def __init__(self, prefix: str, runtime: Runtime, *, left: PartSpec, right: PartSpec, left_scale: float = 1.0,
                 right_scale: float = 1.0, left_name: str = "left", right_name: str = "right") -> None:
        super().__init__(prefix, runtime)
        self.left = build_part("mixer", left, self.name(left_name), runtime)
        self.right = build_part("mixer", right, self.name(right_name), runtime)
        self.left_scale = float(left_scale)
        self.right_scale = float(right_scale)
        self._left_needs = len(_flat(self.left.cache_need()))
        self._right_needs = len(_flat(self.right.cache_need()))
        self.fused = all(getattr(side, "scales_its_heads", lambda: False)() for side in (self.left, self.right))
        self.o_weight: torch.Tensor | None = None  # [hidden, K_left + K_right] where the two are run as one
        self.o_bias: torch.Tensor | None = None

    def cache_need(self) -> CacheNeed:
        needs = _flat(self.left.cache_need()) + _flat(self.right.cache_need())
        return None if not needs else needs[0] if len(needs) == 1 else needs

    def is_capturable(self) -> bool:
        return self.capturable and self.left.is_capturable() and self.right.is_capturable()

    def step_fields(self) -> tuple:
        return (*self.left.step_fields(), *self.right.step_fields())

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The first mixer's output is held while the second runs."""
        hidden = max(self.left.activation_bytes(tokens, itemsize), self.right.activation_bytes(tokens, itemsize))
        return hidden + 2 * tokens * getattr(self.left, "hidden_size", 0) * 4

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {**self.left.tensor_specs(), **self.right.tensor_specs()}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.left.load(tensors)
        self.right.load(tensors)
        if not self.fused:
            return
        self.o_weight = torch.cat([self.left.o_weight, self.right.o_weight], dim=1).contiguous()
        biases = [(side.o_bias_tensor, scale) for side, scale in ((self.left, self.left_scale), (self.right, self.right_scale))
                  if side.o_bias_tensor is not None]
        if biases:
            total = sum(bias.float() * scale for bias, scale in biases)
            self.o_bias = total.to(self.o_weight.dtype).contiguous()
        # The sides' own copies are not read again.
        self.left.o_weight = self.right.o_weight = None
        self.left.o_bias_tensor = self.right.o_bias_tensor = None

    @staticmethod
    def _views(views: tuple, count: int):
        return None if count == 0 else views[0] if count == 1 else tuple(views)

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        views = () if cache is None else tuple(cache) if isinstance(cache, (tuple, list)) else (cache,)
        if len(views) != self._left_needs + self._right_needs:
            raise ValueError(f"{self.prefix}: {len(views)} cache views for {self._left_needs} + {self._right_needs} needs")
        left_views = self._views(views[: self._left_needs], self._left_needs)
        right_views = self._views(views[self._left_needs:], self._right_needs)
        ops = self.runtime.ops
        if self.fused:
            wide = self.left.out_features
            heads = ops.rows_buffer(ctx.num_tokens, wide + self.right.out_features, self.runtime.dtype, x.device)
            self.left.heads_out(x, ctx, left_views, scale=self.left_scale, out=(heads, 0))
            self.right.heads_out(x, ctx, right_views, scale=self.right_scale, out=(heads, wide))
            return ops.linear(heads, self.o_weight, self.o_bias, for_residual=True)
        left = self.left.forward(x, ctx, left_views)
        right = self.right.forward(x, ctx, right_views)
        return ops.scaled_pair(left, self.left_scale, right, self.right_scale, self.runtime.dtype)
