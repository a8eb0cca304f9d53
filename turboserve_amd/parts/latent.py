"""Latent attention: keys and values of all heads are made from one small vector per token, and
only that vector and a rotated key part that the heads share are cached."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.kernels.ops import ATTENTION_MAX_ROW
from turboserve_amd.parts.attention import tiled_attention
from turboserve_amd.parts.base import CacheNeed, Mixer, PagedKV, PagedKVView, PartSpec, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_mixer


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """Per token ``c = norm(Wd x)[:C]`` (the latent, ``C = rank``) and ``r = rot(Wd x[C:])`` (``R =
    rot_dim`` elements, turned by the position); head ``h`` has the key ``[Uk_h c | r]`` and the
    value ``Uv_h c``; its query is ``[q_h plain (D) | rot(q_h rotated (R))]``; scores ``scale (q . k)``
    over all keys up to the token's own, softmax, output matrix.

    Computed with the up-projections carried to the query's side: ``q_h . (Uk_h c) = (Uk_h^T q_h) . c``
    and ``sum_j p_j Uv_h c_j = Uv_h (sum_j p_j c_j)``, so a step attends over the cached rows ``[c |
    r]`` themselves, as one key head of ``C + R`` elements whose first ``C`` are also its value, and
    nothing per head is ever made for a cached token.  The page holds what the layer needs
    cached and no more: ``PagedKV(1, C + R, value_dim=0)``.

    The query matrix and the down-projection are held as one matrix (one product a step); the two
    up-projections are stacks over the heads, ``[H, C, D]`` (transposed at load) and ``[H, Dv, C]``,
    run by ``ops.per_head_rows``.  ``rotation`` is the ``PartSpec`` of a rotary encoding (its tables
    are what this part reads; ``turned <= R`` elements are turned, the rest pass; pairs in halves or,
    if the encoding says ``neighbours``, ``(2i, 2i + 1)``).  ``window``: a token sees itself and the
    ``window - 1`` tokens before it.  ``gate_name``: a matrix ``[H, hidden]`` of that name makes one
    number per head from the mixer's input, and the head's output is multiplied by its sigmoid
    before the output matrix (its rows ride behind the fused matrix's).  ``names``: tensor
    names under the part's prefix of ``q, down, down_norm, up_k, up_v, o``."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        hidden_size: int,
        num_heads: int,
        head_dim: int,
        rot_dim: int,
        value_dim: int,
        rank: int,
        scale: float,
        norm_eps: float,
        rotation: PartSpec,
        names: Mapping[str, str] | None = None,
        window: int | None = None,
        gate_name: str | None = None,
    ) -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.head_dim = int(head_dim)
        self.rot_dim = int(rot_dim)
        self.value_dim = int(value_dim)
        self.rank = int(rank)
        self.scale = float(scale)
        self.norm_eps = float(norm_eps)
        self.wide = self.rank + self.rot_dim
        self.window = None if window is None else int(window)
        if self.window is not None and self.window < 1:
            raise ValueError(f"{prefix or 'latent attention'}: a window of {self.window} tokens")
        self.gate_name = gate_name
        if min(self.num_heads, self.head_dim, self.rot_dim, self.value_dim, self.rank) < 1 or self.num_heads > 1024:
            raise ValueError(f"{prefix or 'latent attention'}: sizes must be positive and the heads at most 1,024")
        if self.wide > ATTENTION_MAX_ROW:
            raise ValueError(f"{prefix or 'latent attention'}: a cached row of {self.wide} elements is above the "
                             f"{ATTENTION_MAX_ROW} the attention kernel takes")
        self.rotation = build_part("position_encoding", rotation, prefix, runtime)
        if not 2 <= self.rotation.head_dim <= self.rot_dim:
            raise ValueError(f"{prefix or 'latent attention'}: {self.rotation.head_dim} turned elements do not fit {self.rot_dim}")
        self.names = {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_k": "uk", "up_v": "uv", "o": "o", **(names or {})}
        self.q_size = self.num_heads * (self.head_dim + self.rot_dim)
        self.fused: torch.Tensor | None = None       # [H (D + R) + C + R, hidden]
        self.down_gain: torch.Tensor | None = None   # [C]
        self.up_k: torch.Tensor | None = None        # [H, C, D]: head h's matrix transposed
        self.up_v: torch.Tensor | None = None        # [H, Dv, C]
        self.o_weight: torch.Tensor | None = None    # [hidden, H Dv]

    def cache_need(self) -> CacheNeed:
        return PagedKV(1, self.wide, self.window, 0)

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        per_token = (self.q_size + self.wide + self.num_heads * (self.head_dim + 2 * self.wide + self.value_dim)) * itemsize
        return tokens * (per_token + self.num_heads * (self.rank + self.value_dim) * 4 + self.hidden_size * 4)

    def tensor_specs(self) -> dict[str, TensorSpec]:
        n = self.names
        gate = {} if self.gate_name is None else {self.name(self.gate_name): TensorSpec((self.num_heads, self.hidden_size))}
        return {
            **gate,
            self.name(n["q"]): TensorSpec((self.q_size, self.hidden_size)),
            self.name(n["down"]): TensorSpec((self.wide, self.hidden_size)),
            self.name(n["down_norm"]): TensorSpec((self.rank,), init="ones"),
            self.name(n["up_k"]): TensorSpec((self.num_heads * self.head_dim, self.rank)),
            self.name(n["up_v"]): TensorSpec((self.num_heads * self.value_dim, self.rank)),
            self.name(n["o"]): TensorSpec((self.hidden_size, self.num_heads * self.value_dim)),
        }

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.names
        rows = [tensors[self.name(n["q"])], tensors[self.name(n["down"])]]
        if self.gate_name is not None:
            rows.append(tensors[self.name(self.gate_name)])
        self.fused = torch.cat(rows, dim=0).contiguous()
        self.down_gain = tensors[self.name(n["down_norm"])].contiguous()
        up_k = tensors[self.name(n["up_k"])].view(self.num_heads, self.head_dim, self.rank)
        self.up_k = up_k.transpose(1, 2).contiguous()
        self.up_v = tensors[self.name(n["up_v"])].view(self.num_heads, self.value_dim, self.rank).contiguous()
        self.o_weight = tensors[self.name(n["o"])].contiguous()

    def forward(self, x: torch.Tensor, ctx, cache: PagedKVView) -> torch.Tensor:
        ops, dtype = self.runtime.ops, self.runtime.dtype
        tokens = ctx.num_tokens
        proj = ops.linear(x, self.fused)
        self.rotation.ensure_capacity(ctx.max_context_len)
        slots = ctx.slot_mapping[cache.group] if cache.writable else None
        q_plain, q_wide = ops.latent_store(
            proj, cache.k, self.down_gain, self.norm_eps, self.rotation.cos, self.rotation.sin, ctx.positions, slots,
            self.num_heads, self.head_dim, self.rot_dim, self.rank, cache.block_size, ctx.max_context_len - 1, dtype,
            neighbours=self.rotation.neighbours, tail=0 if self.gate_name is None else self.num_heads)
        # The plain query parts through the keys' up-projection: what they are against the latent itself.
        carried = ops.per_head_rows(q_plain, self.up_k)
        q_wide[:, :, : self.rank].copy_(carried.view(tokens, self.num_heads, self.rank))
        stride = self.num_heads * self.wide
        if ops.tiled_attention_supported(dtype, self.wide, self.rank, cache.block_size, stride, True):
            attended = tiled_attention(ops, q_wide.view(tokens, stride), stride, cache.k, None, ctx.block_tables[cache.group],
                                       ctx, heads=self.num_heads, scale=self.scale, value_dim=self.rank, window=self.window)
        else:
            attended = ops.paged_attention_generic(
                q_wide.view(tokens, stride), stride, cache.k, None, ctx.block_tables[cache.group], ctx.token_seq,
                ctx.positions, self.num_heads, self.scale, self.window, value_dim=self.rank)
        values = ops.per_head_rows(attended.view(tokens * self.num_heads, self.rank), self.up_v)
        heads_out = values.view(tokens, self.num_heads * self.value_dim)
        if self.gate_name is not None:
            # Every head's output times the sigmoid of its gate (the projection's last columns), rounded once.
            heads_out = ops.head_gate(heads_out, proj, self.q_size + self.wide, self.num_heads, dtype)
        elif dtype != torch.float32:  # the products' 32-bit results, rounded once for the output matrix
            rounded = ops.rows_buffer(tokens, self.num_heads * self.value_dim, dtype, x.device)
            rounded.copy_(heads_out)
            heads_out = rounded
        return ops.linear(heads_out, self.o_weight, for_residual=True)
