"""SwiGLU feed-forward (src/turboserve/engine/model/layers.py:394-440)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import FeedForward, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(FeedForward):
    """``down(silu(gate(x)) * up(x))`` (layers.py:437-440).  Gate and up are held as one
    ``[2 I, H]`` matrix whose rows alternate gate, up (interleaved at load; the checkpoint keeps
    them apart): a step does one product for both, and the product's kernel has each gate
    value next to its up value, so it can apply the activation itself.

    ``rule = (steepness, limit, up_shift)`` makes it another gated unit: with ``g = min(gate(x),
    limit)`` and ``u = clamp(up(x), -limit, limit)`` where ``limit > 0``, ``down(g * sigmoid(steepness
    * g) * (u + up_shift))``; the default ``(1, 0, 0)`` is SwiGLU.  A fourth number ``cubic`` makes the
    gate ``g * sigmoid(steepness * (g + cubic * g^3))``; ``ops.GELU_TANH_RULE`` is the tanh form of GELU
    on the gate.  ``names``: the three matrices' tensor names under the part's prefix."""

    def __init__(self, prefix: str, runtime: Runtime, *, hidden_size: int, intermediate_size: int,
                 rule: tuple[float, float, float] = (1.0, 0.0, 0.0),
                 names: tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.rule = tuple(float(v) for v in rule)
        self.gate_name, self.up_name, self.down_name = names
        self.gate_up_weight: torch.Tensor | None = None
        self.down_weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {
            self.name(self.gate_name): TensorSpec((self.intermediate_size, self.hidden_size)),
            self.name(self.up_name): TensorSpec((self.intermediate_size, self.hidden_size)),
            self.name(self.down_name): TensorSpec((self.hidden_size, self.intermediate_size)),
        }

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The gate|up projection, the activated product and the down projection (32-bit: it is
        added to the residual stream) of a step."""
        return tokens * (3 * self.intermediate_size * itemsize + self.hidden_size * 4)

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        gate, up = tensors[self.name(self.gate_name)], tensors[self.name(self.up_name)]
        self.gate_up_weight = torch.stack([gate, up], dim=1).reshape(2 * gate.shape[0], gate.shape[1]).contiguous()
        self.down_weight = tensors[self.name(self.down_name)].contiguous()

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.runtime.ops
        return ops.linear(ops.linear_swiglu(x, self.gate_up_weight, self.rule), self.down_weight, for_residual=True)


@register_feed_forward("mlp")
class ActivatedMLP(FeedForward):
    """``down(act(up(x)))``: a feed-forward without a gate.  ``activation`` is one of
    ``ops.ACTIVATIONS`` (``relu_squared``: ``max(z, 0)^2``; ``relu``; ``silu``; ``gelu_tanh``), applied in
    32-bit to the first product's sums and rounded once.  ``names``: the two matrices' tensor names
    under the part's prefix."""

    def __init__(self, prefix: str, runtime: Runtime, *, hidden_size: int, intermediate_size: int, activation: str,
                 names: tuple[str, str] = ("up_proj.weight", "down_proj.weight")) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.intermediate_size = int(intermediate_size)
        self.activation = str(activation)
        self.up_name, self.down_name = names
        self.up_weight: torch.Tensor | None = None
        self.down_weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {
            self.name(self.up_name): TensorSpec((self.intermediate_size, self.hidden_size)),
            self.name(self.down_name): TensorSpec((self.hidden_size, self.intermediate_size)),
        }

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The up projection, its activation and the down projection (32-bit: it is added to the
        residual stream) of a step."""
        return tokens * (2 * self.intermediate_size * itemsize + self.hidden_size * 4)

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.up_weight = tensors[self.name(self.up_name)].contiguous()
        self.down_weight = tensors[self.name(self.down_name)].contiguous()

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.runtime.ops
        hidden = ops.activate(ops.linear(x, self.up_weight), self.activation, x.dtype)
        return ops.linear(hidden, self.down_weight, for_residual=True)
