"""A routed feed-forward: many small gated feed-forwards ("experts"), of which each token takes a
few, chosen by a router; optionally one more that every token takes."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import FeedForward, PartSpec, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_feed_forward


@register_feed_forward("routed_experts")
class RoutedExperts(FeedForward):
    """``sum_j w_j * expert_{e_j}(x)  (+ gate(x) * shared(x))``.

    Router, in 32-bit: ``s = sigmoid(router x)``.  The ``experts`` form ``groups`` equal groups
    of neighbours; a group's mark is the sum of its two largest ``s``; only experts of the
    ``keep`` groups with the largest marks can be taken; the ``top`` of them with the largest
    ``s`` are, with weights ``s / (sum of the taken s + 1e-20) * route_scale`` (``groups = keep
    = 1`` is plain top-k).  An expert is ``down(g * sigmoid(steepness g) * (u + up_shift))`` by
    ``rule`` as in the ``swiglu`` part.  ``shared``: the ``PartSpec`` of a feed-forward every
    token runs through, under ``<prefix>.<shared_name>``; with ``shared_gate_name`` its output
    is multiplied by ``sigmoid(v . x)``, one number per token, ``v`` the tensor of that name.

    Other routers, each a parameter: ``router_scores = "softmax"`` (``s`` is the softmax over all the
    router's outputs); ``correction_name`` (a vector ``[outputs]`` under the part's prefix that is
    added to ``s`` where experts are chosen, while the weights use ``s`` alone); ``normalise =
    False`` (weights ``s * route_scale``, not divided by their sum); ``identity = n`` (the router
    has ``experts + n`` outputs, and the last ``n`` stand for the token itself: such a pair
    contributes ``w * x`` and has no matrices); ``group_mark = "max"`` (a group's mark is its largest
    score alone, not the sum of its two largest).

    The experts' matrices are stacked at load: ``[E, 2 I, H]`` with rows alternating gate, up,
    and ``[E, H, I]``.  A step routes on the device, runs every (token, taken expert) pair
    against its expert's matrices (pair by pair in steps of few tokens, grouped by expert on the
    matrix cores in bfloat16 steps of many) and sums with the weights, so nothing depends on data
    the host has not seen and single-token steps can be recorded.
    """

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        hidden_size: int,
        expert_size: int,
        experts: int,
        top: int,
        groups: int = 1,
        keep: int = 1,
        route_scale: float = 1.0,
        rule: tuple[float, float, float] = (1.0, 0.0, 0.0),
        shared: PartSpec | None = None,
        shared_name: str = "shared",
        shared_gate_name: str | None = None,
        router_name: str = "router",
        expert_names: tuple[str, str, str, str] = ("e{index}", "gate", "up", "down"),
        router_scores: str = "sigmoid",
        correction_name: str | None = None,
        normalise: bool = True,
        identity: int = 0,
        group_mark: str = "top2_sum",
    ) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.expert_size = int(expert_size)
        self.experts = int(experts)
        self.top = int(top)
        self.groups = int(groups)
        self.keep = int(keep)
        self.route_scale = float(route_scale)
        self.rule = tuple(float(v) for v in rule)
        self.identity = int(identity)
        if self.identity < 0:
            raise ValueError(f"{prefix}: {self.identity} identity experts")
        #: What the router chooses among: the experts with matrices, then the identity ones.
        self.outputs = self.experts + self.identity
        if self.experts < 1 or self.groups < 1 or self.outputs % self.groups != 0:
            raise ValueError(f"{prefix}: {self.outputs} router outputs do not form {self.groups} equal groups")
        if not 1 <= self.keep <= self.groups:
            raise ValueError(f"{prefix}: {self.keep} of {self.groups} groups cannot be kept")
        if not 1 <= self.top <= (self.outputs // self.groups) * self.keep:
            raise ValueError(f"{prefix}: {self.top} experts cannot be taken from {self.keep} groups of {self.outputs // self.groups}")
        if self.outputs > 1024 or self.top > 32:
            raise ValueError(f"{prefix}: the router's kernel takes up to 1,024 outputs and 32 per token")
        if router_scores not in ("sigmoid", "softmax"):
            raise ValueError(f"{prefix}: router scores {router_scores!r} are neither 'sigmoid' nor 'softmax'")
        if group_mark not in ("top2_sum", "max"):
            raise ValueError(f"{prefix}: a group's mark {group_mark!r} is neither 'top2_sum' nor 'max'")
        self.mark_top = 2 if group_mark == "top2_sum" else 1
        self.softmax = router_scores == "softmax"
        self.correction_name = correction_name or None
        self.normalise = bool(normalise)
        self.correction: torch.Tensor | None = None
        self.router_name = router_name
        self.expert_names = tuple(expert_names)
        self.shared = None if shared is None else build_part("feed_forward", shared, self.name(shared_name), runtime)
        self.shared_gate_name = None if shared is None or not shared_gate_name else self.shared.name(shared_gate_name)
        self.router: torch.Tensor | None = None
        self.gate_up: torch.Tensor | None = None   # [E, 2 I, H], rows alternate gate, up
        self.down: torch.Tensor | None = None      # [E, H, I]

    def _expert(self, index: int, which: int) -> str:
        return self.name(f"{self.expert_names[0].format(index=index)}.{self.expert_names[which]}")

    def is_capturable(self) -> bool:
        return self.capturable and (self.shared is None or self.shared.is_capturable())

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs = {self.name(self.router_name): TensorSpec((self.outputs, self.hidden_size))}
        if self.correction_name:
            specs[self.name(self.correction_name)] = TensorSpec((self.outputs,), init="zeros")
        for index in range(self.experts):
            specs[self._expert(index, 1)] = TensorSpec((self.expert_size, self.hidden_size))
            specs[self._expert(index, 2)] = TensorSpec((self.expert_size, self.hidden_size))
            specs[self._expert(index, 3)] = TensorSpec((self.hidden_size, self.expert_size))
        if self.shared is not None:
            specs.update(self.shared.tensor_specs())
        if self.shared_gate_name:
            specs[self.shared_gate_name] = TensorSpec((1, self.hidden_size))
        return specs

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """Per pair the gated units and the 32-bit output; per token the 32-bit sum; the shared
        feed-forward runs while the pairs' outputs are held."""
        pairs = tokens * self.top
        own = pairs * (self.expert_size * itemsize + self.hidden_size * 4) + tokens * self.hidden_size * 4
        return own + (self.shared.activation_bytes(tokens, itemsize) if self.shared is not None else 0)

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.router = tensors[self.name(self.router_name)].contiguous()
        if self.correction_name:
            self.correction = tensors[self.name(self.correction_name)].to(torch.float32).contiguous()
        if self.shared_gate_name:
            # The shared expert's gate is one more row of the router's matrix: one product for both.
            self.router = torch.cat([self.router, tensors[self.shared_gate_name].reshape(1, -1)], dim=0).contiguous()
        first = tensors[self._expert(0, 1)]
        self.gate_up = torch.empty((self.experts, 2 * self.expert_size, self.hidden_size), dtype=first.dtype, device=first.device)
        self.down = torch.empty((self.experts, self.hidden_size, self.expert_size), dtype=first.dtype, device=first.device)
        for index in range(self.experts):
            self.gate_up[index, 0::2] = first if index == 0 else tensors[self._expert(index, 1)]
            self.gate_up[index, 1::2] = tensors[self._expert(index, 2)]
            self.down[index] = tensors[self._expert(index, 3)]
        del first
        if self.shared is not None:
            self.shared.load(tensors)

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        ops = self.runtime.ops
        taken, weights, gate = ops.moe_route(x, self.router, top=self.top, groups=self.groups, keep=self.keep,
                                             scale=self.route_scale, experts=self.outputs, softmax=self.softmax,
                                             correction=self.correction, normalise=self.normalise, mark_top=self.mark_top)
        grouping = ops.moe_grouping(taken, self.experts, x.dtype, self.hidden_size, self.expert_size)
        units = ops.moe_expert_units(x, self.gate_up, taken, self.rule, grouping)
        outputs = ops.moe_expert_outputs(units, self.down, taken, grouping)
        extra = self.shared.forward(x, ctx) if self.shared is not None else None
        if self.identity:
            return ops.moe_combine(outputs, weights, extra, gate, x.dtype, taken=taken, experts=self.experts, rows=x)
        return ops.moe_combine(outputs, weights, extra, gate, x.dtype)
