"""Rotary position encoding (src/turboserve/engine/model/layers.py:214-308)."""

from __future__ import annotations

import math
from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import PagedKVView, PositionEncoding, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_position_encoding


def rotary_tables(capacity: int, head_dim: int, theta: float, factor: float) -> tuple[torch.Tensor, torch.Tensor]:
    """32-bit ``cos, sin [capacity, D/2]`` of the angles ``(pos / factor) * theta^(-2i/D)``.

    Computed on the CPU with the reference's expressions (layers.py:258-262 for the inverse
    frequencies, :281-286 for the outer product; its tables repeat the ``D/2`` columns twice,
    which is not stored here)."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float32) / head_dim))
    positions = torch.arange(capacity, dtype=torch.float32)
    if factor != 1.0:
        positions = positions / factor
    angles = torch.outer(positions, inv_freq)
    return angles.cos().contiguous(), angles.sin().contiguous()


def interpolated_frequencies(head_dim: int, theta: float, scaling: Mapping | None) -> tuple[torch.Tensor, float]:
    """64-bit ``f [D/2]`` and the factor on cosine and sine of a rotary encoding whose frequencies are
    stretched where they are slow (YaRN; Peng et al., "YaRN: Efficient Context Window Extension of Large
    Language Models").  ``f_i = theta^(-2i/D)``; with ``scaling = {factor, original, fast, slow}``: the
    dimension at which a frequency turns ``t`` times within ``original`` positions is ``d(t) = D ln(original
    / (2 pi t)) / (2 ln theta)``; ``lo = max(floor(d(fast)), 0)``, ``hi = min(ceil(d(slow)), D - 1)``;
    ``r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)``; ``f_i <- f_i / factor * r_i + f_i (1 - r_i)``,
    and cosine and sine are multiplied by ``0.1 ln(factor) + 1``.  Without ``scaling``: ``f`` and 1."""
    index = torch.arange(head_dim // 2, dtype=torch.float64)
    freq = float(theta) ** (-2.0 * index / head_dim)
    if scaling is None:
        return freq, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turns_at(turns: float) -> float:
        return head_dim * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(float(theta)))

    low = max(math.floor(turns_at(float(scaling["fast"]))), 0)
    high = min(math.ceil(turns_at(float(scaling["slow"]))), head_dim - 1)
    ramp = ((index - low) / max(high - low, 0.001)).clamp(0.0, 1.0)
    return freq / factor * ramp + freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def exact_rotary_tables(capacity: int, freq: torch.Tensor, magnitude: float) -> tuple[torch.Tensor, torch.Tensor]:
    """32-bit ``cos, sin [capacity, D/2]`` times ``magnitude`` from 64-bit angles ``pos * freq``, rounded once."""
    angles = torch.outer(torch.arange(capacity, dtype=torch.float64), freq)
    return (angles.cos() * magnitude).float().contiguous(), (angles.sin() * magnitude).float().contiguous()


def normed_store(runtime: Runtime, qkv, num_heads, num_kv_heads, head_dim, value_dim, ctx, cache: PagedKVView, slots,
                 head_norm: tuple | None, cos, sin, span_norm: tuple | None = None, values: Mapping | None = None,
                 shape: Mapping | None = None):
    """The store of a mixer that asked for more than an encoding alone does: a norm per q and k
    head (``head_norm = (q_gain, k_gain, eps, gain_offset)``) and values of a width of their own,
    with the rotation by ``cos``/``sin`` where given, all in one pass (``ops.head_norm_store``); or
    a norm over all q heads at once and all k heads at once (``span_norm``, the same four with
    gains of the projections' full sizes; ``ops.span_norm_store``, which rotates nothing).  ``values =
    {"keep": tensor}`` and/or ``{"blend": (tensor, weight)}``: the step's values as projected are left in
    ``keep``, and what is stored is mixed with ``blend`` (``ops.head_norm_store``).  ``shape``: what else the
    per-head store takes (``normed``, ``norm_after``, ``values_are_keys``, ``query_temperature``, ``tail``)."""
    if span_norm is not None:
        if values or shape:
            raise ValueError("values are kept or mixed by the per-head store only")
        if head_norm is not None or cos is not None:
            raise ValueError("a norm over the whole projection goes with no per-head norm and no rotation")
        q_gain, k_gain, eps, gain_offset = span_norm
        return runtime.ops.span_norm_store(
            qkv, cache.k, cache.v, q_gain, k_gain, eps, slots, ctx.num_tokens, num_heads, num_kv_heads, head_dim, value_dim,
            cache.block_size, runtime.dtype, gain_offset=gain_offset)
    q_gain, k_gain, eps, gain_offset = head_norm if head_norm is not None else (None, None, 0.0, 0.0)
    return runtime.ops.head_norm_store(
        qkv, cache.k, cache.v, q_gain, k_gain, eps, ctx.positions, slots, num_heads, num_kv_heads, head_dim, value_dim,
        cache.block_size, runtime.dtype, gain_offset=gain_offset, cos=cos, sin=sin, max_position=ctx.max_context_len - 1,
        keep_values=(values or {}).get("keep"), blend_values=(values or {}).get("blend"), **dict(shape or {}),
    )


@register_position_encoding("rope")
class RotaryEncoding(PositionEncoding):
    """Half-split rotary encoding: the pair ``(i, i + D/2)`` of every query and key head is
    turned by the angle of the token's position (layers.py:214-222, 298-302).  The rotation is
    computed in 32-bit from 32-bit tables and rounded once.  It has no weights, so layers with
    the same constants share one instance and one pair of tables.

    The tables are made once, at the first step, for ``max_positions`` (the model's
    ``max_position_embeddings``) or ``initial_positions`` when given; a step that reaches
    further makes them grow by doubling, driven by the host-known largest position
    (layers.py:272-288).  A recorded step (a HIP graph) holds the addresses of the tables it was
    recorded with, so tables that growth has superseded are kept, never freed: they cover every
    position such a recording can bring, because the recording's widest context was inside them
    when it was made.

    ``interpolation = {factor, original, fast, slow}`` stretches the slow frequencies
    (:func:`interpolated_frequencies`); ``exact`` (implied by it) makes the tables from 64-bit angles
    rounded once.  ``neighbours``: the pairs turned together are ``(2i, 2i + 1)``; only a part that
    reads the tables itself (the latent layer's store) takes that.  ``head_dim`` may be smaller than the
    heads it is applied to: their first ``head_dim`` elements are turned, the rest pass."""

    shareable = True

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        head_dim: int,
        theta: float,
        scaling_factor: float = 1.0,
        max_positions: int = 2048,
        initial_positions: int | None = None,
        interpolation: Mapping | None = None,
        exact: bool = False,
        neighbours: bool = False,
    ) -> None:
        super().__init__(prefix, runtime)
        if head_dim % 2 != 0:
            raise ValueError(f"head_dim must be even for rotary encoding, got {head_dim}")
        self.head_dim = int(head_dim)
        self.theta = float(theta)
        self.scaling_factor = float(scaling_factor)
        self.interpolation = None if interpolation is None else dict(interpolation)
        self.exact = bool(exact) or interpolation is not None
        self.neighbours = bool(neighbours)
        if self.exact and self.scaling_factor != 1.0:
            raise ValueError("positions divided by a factor and exact or interpolated tables exclude each other")
        self.cos: torch.Tensor | None = None
        self.sin: torch.Tensor | None = None
        self.capacity = 0
        #: First table size; the tables themselves are made at the first step.  The reference
        #: starts at ``min(max_positions, 1024)`` (layers.py:265); here the whole of
        #: ``max_positions`` is made at once (7B: 32,768 x 64 x 4 bytes x 2 = 16.8 MB), so that
        #: growth is the exception.
        self.initial_capacity = int(max_positions if initial_positions is None else initial_positions)
        #: Tables that growth has replaced; recorded steps may still read them.
        self.superseded: list[tuple[torch.Tensor, torch.Tensor]] = []

    def ensure_capacity(self, num_positions: int) -> None:
        if num_positions <= self.capacity:
            return
        target = max(num_positions, 2 * self.capacity, self.initial_capacity, 16)
        if self.exact:
            cos, sin = exact_rotary_tables(target, *interpolated_frequencies(self.head_dim, self.theta, self.interpolation))
        else:
            cos, sin = rotary_tables(target, self.head_dim, self.theta, self.scaling_factor)
        if self.cos is not None:
            self.superseded.append((self.cos, self.sin))
        self.cos = cos.to(self.runtime.device)
        self.sin = sin.to(self.runtime.device)
        self.capacity = target

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache: PagedKVView, *,
                         value_dim: int | None = None, head_norm: tuple | None = None, span_norm: tuple | None = None,
                         values: Mapping | None = None, shape: Mapping | None = None):
        if self.neighbours:
            raise ValueError("the stores of whole heads turn the pairs (i, i + D/2) only")
        if self.head_dim > head_dim:
            raise ValueError(f"{self.head_dim} turned elements do not fit heads of {head_dim}")
        self.ensure_capacity(ctx.max_context_len)
        slots = ctx.slot_mapping[cache.group] if cache.writable else None
        # (Tables narrower than the heads turn the heads' first elements only: the per-head store takes that.)
        if (head_norm is not None or span_norm is not None or values or shape or self.head_dim != head_dim
                or (value_dim is not None and value_dim != head_dim)):
            return normed_store(self.runtime, qkv, num_heads, num_kv_heads, head_dim, value_dim or head_dim, ctx, cache,
                                slots, head_norm, self.cos, self.sin, span_norm, values, shape)
        return self.runtime.ops.rope_store(
            qkv, cache.k, cache.v, self.cos, self.sin, ctx.positions, slots,
            num_heads, num_kv_heads, head_dim, cache.block_size, ctx.max_context_len - 1, self.runtime.dtype,
        )


@register_position_encoding("none")
class NoPositionEncoding(PositionEncoding):
    """No encoding: queries and keys stay as projected; keys and values are stored."""

    shareable = True

    def __init__(self, prefix: str, runtime: Runtime) -> None:
        super().__init__(prefix, runtime)

    def encode_and_store(self, qkv, num_heads, num_kv_heads, head_dim, ctx, cache: PagedKVView, *,
                         value_dim: int | None = None, head_norm: tuple | None = None, span_norm: tuple | None = None,
                         values: Mapping | None = None, shape: Mapping | None = None):
        slots = ctx.slot_mapping[cache.group] if cache.writable else None
        if head_norm is not None or span_norm is not None or values or shape or (value_dim is not None and value_dim != head_dim):
            return normed_store(self.runtime, qkv, num_heads, num_kv_heads, head_dim, value_dim or head_dim, ctx, cache,
                                slots, head_norm, None, None, span_norm, values, shape)
        return self.runtime.ops.rope_store(
            qkv, cache.k, cache.v, None, None, ctx.positions, slots,
            num_heads, num_kv_heads, head_dim, cache.block_size, ctx.max_context_len - 1, self.runtime.dtype,
        )


@register_position_encoding("distance_slopes")
class DistanceSlopes(NoPositionEncoding):
    """Positions enter the scores only: the score of key ``j`` for the query at ``i`` of head ``h`` (of
    ``H``) loses ``m_h (i - j)``, ``m_h = 2^(-exponent (h + 1) / H)``.  Queries and keys are stored as
    projected."""

    shareable = True

    def __init__(self, prefix: str, runtime: Runtime, *, exponent: float = 8.0) -> None:
        super().__init__(prefix, runtime)
        self.exponent = float(exponent)
        self._slopes: dict[int, torch.Tensor] = {}

    def score_slopes(self, num_heads: int) -> torch.Tensor:
        if num_heads not in self._slopes:
            values = [2.0 ** (-self.exponent * (h + 1) / num_heads) for h in range(num_heads)]
            self._slopes[num_heads] = torch.tensor(values, dtype=torch.float32, device=self.runtime.device)
        return self._slopes[num_heads]


def distance_bucket(distance: int, buckets: int, max_distance: float) -> int:
    """The row of a table of ``buckets`` learned biases for a key ``distance`` positions back: the
    first ``buckets // 2`` distances have a row each; beyond, rows are spaced evenly in the logarithm of
    the distance up to ``max_distance``, and everything further shares the last row."""
    exact = buckets // 2
    if distance < exact:
        return distance
    spread = math.log(distance / exact) / math.log(max_distance / exact) * (buckets - exact)
    return min(buckets - 1, exact + int(math.floor(spread)))


@register_position_encoding("distance_buckets")
class DistanceBuckets(NoPositionEncoding):
    """Positions enter the scores only, through a learned table ``[B, H]`` (``table_name`` under the
    part's prefix): the score of the key ``n`` positions back gets ``table[bucket(n), h]`` added, after
    the scale (:func:`distance_bucket`).  Queries and keys are stored as projected.  ``B`` is the
    table's own (``buckets``, or from the tensor).  At load the table is spread out by distance,
    ``[H, L]`` 32-bit with ``L`` the first distance of the last bucket plus one (or the layer's
    ``reach``, if that is shorter): the attention kernels read it by ``min(n, L - 1)``."""

    shareable = False

    def __init__(self, prefix: str, runtime: Runtime, *, num_heads: int, max_distance: float, buckets: int | None = None,
                 reach: int | None = None, table_name: str = "rel") -> None:
        super().__init__(prefix, runtime)
        self.prefix = prefix
        self.num_heads = int(num_heads)
        self.max_distance = float(max_distance)
        self.buckets = None if buckets is None else int(buckets)
        self.reach = None if reach is None else int(reach)
        self.table_name = table_name
        self.by_distance: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name(self.table_name): TensorSpec((-1 if self.buckets is None else self.buckets, self.num_heads))}

    def load(self, tensors) -> None:
        table = tensors[self.name(self.table_name)].float()
        buckets = table.shape[0]
        if buckets < 2 or self.max_distance <= buckets // 2:
            raise ValueError(f"{self.name(self.table_name)}: {buckets} rows need distances beyond {buckets // 2}, "
                             f"not a largest distance of {self.max_distance}")
        rows = []
        distance = 0
        while True:
            rows.append(distance_bucket(distance, buckets, self.max_distance))
            if rows[-1] == buckets - 1 or (self.reach is not None and len(rows) >= self.reach):
                break
            distance += 1
        index = torch.tensor(rows, dtype=torch.long, device=table.device)
        self.by_distance = table[index].t().contiguous()  # [H, L]

    def score_bias_table(self, num_heads: int) -> torch.Tensor:
        if num_heads != self.num_heads:
            raise ValueError(f"{self.prefix}: a table for {self.num_heads} heads asked for {num_heads}")
        return self.by_distance
