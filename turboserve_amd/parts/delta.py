"""The gated delta rule: a mixer whose memory is one matrix per head and request, which every token
decays channel by channel, corrects by what its key reads there, and reads with its query."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import CacheNeed, FixedState, Mixer, Runtime, TensorSpec
from turboserve_amd.parts.registry import register_mixer


@register_mixer("gated_delta_rule")
class GatedDeltaRule(Mixer):
    """Per head a state ``S [D, Dv]`` (32-bit, zero when the request starts).  With ``q = Wq x``, ``k = Wk x``
    (``kv_heads`` heads of ``D``; head ``h`` uses key head ``h // (heads / kv_heads)``) and ``v = Wv x`` (``heads``
    heads of ``Dv``), each through a causal convolution over time of ``taps`` taps per channel and ``silu``, then
    ``q`` and ``k`` made unit vectors per head (``x / sqrt(sum x^2 + 1e-6)``, ``q`` also times ``D^-1/2``):

        g = exp(-exp(A_h) softplus(A2 (A1 x) + dt))      a decay per head and key channel
        beta = sigmoid(Wb x)                             one number per head
        S <- diag(g) S;  w = beta (v - S^T k);  S <- S + k w^T;  o = S^T q

    so the read-out sees the token's own write.  Each head's ``o`` is divided by its root mean square,
    multiplied by one gain ``[Dv]`` and by ``sigmoid(G2 (G1 x))``, and the heads side by side go through the
    output matrix.  Everything that enters the recurrence behind the convolution is 32-bit.

    ``Wq, Wk, Wv, Wb, A1, G1`` are held as one matrix (one product a step).  The state and the convolution's
    last ``taps - 1`` inputs are ``FixedState``s of the cache: the request's slot holds them between steps.
    ``decay_rank`` / ``gate_rank``: the widths of ``A1 x`` and ``G1 x`` (``None``: from the checkpoint's tensors).
    ``names``: tensor names under the part's prefix of ``q, k, v, beta, a1, a2, dt, a_log, g1, g2, norm, o``; the
    convolutions' weights ``[channels, taps]`` are ``<q|k|v name>.<conv_suffix>``."""

    def __init__(self, prefix: str, runtime: Runtime, *, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int,
                 value_dim: int, taps: int, norm_eps: float, decay_rank: int | None = None, gate_rank: int | None = None,
                 names: Mapping[str, str] | None = None, conv_suffix: str = "conv") -> None:
        super().__init__(prefix, runtime)
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.value_dim = int(value_dim)
        self.taps = int(taps)
        self.norm_eps = float(norm_eps)
        self.decay_rank = None if decay_rank is None else int(decay_rank)
        self.gate_rank = None if gate_rank is None else int(gate_rank)
        where = prefix or "gated delta rule"
        if min(self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim) < 1 or self.num_heads % self.num_kv_heads != 0:
            raise ValueError(f"{where}: sizes must be positive and the heads a multiple of the key heads")
        if self.head_dim > 256 or self.num_heads > 65535:
            raise ValueError(f"{where}: the kernel takes up to 256 key channels a head")
        if not 1 <= self.taps <= 8:
            raise ValueError(f"{where}: a convolution of {self.taps} taps is outside 1..8")
        for rank in (self.decay_rank, self.gate_rank):
            if rank is not None and not 1 <= rank <= 256:
                raise ValueError(f"{where}: a low-rank input of {rank} is outside 1..256")
        self.names = {"q": "q", "k": "k", "v": "v", "beta": "b", "a1": "a1", "a2": "a2", "dt": "dt_bias", "a_log": "A_log",
                      "g1": "g1", "g2": "g2", "norm": "norm", "o": "o", **(names or {})}
        self.conv_suffix = conv_suffix
        self.key_size = self.num_kv_heads * self.head_dim
        self.value_size = self.num_heads * self.value_dim
        self.channels = 2 * self.key_size + self.value_size
        self.fused: torch.Tensor | None = None        # [2 G D + H Dv + H + Ra + Rg, hidden]
        self.conv_weight: torch.Tensor | None = None  # [2 G D + H Dv, taps]
        self.a2: torch.Tensor | None = None           # [H D, Ra]
        self.dt: torch.Tensor | None = None           # [H D]
        self.a_log: torch.Tensor | None = None        # [H] 32-bit
        self.g2: torch.Tensor | None = None           # [H Dv, Rg]
        self.gain: torch.Tensor | None = None         # [Dv]
        self.o_weight: torch.Tensor | None = None     # [hidden, H Dv]

    def cache_need(self) -> CacheNeed:
        return (FixedState((self.num_heads, self.head_dim, self.value_dim), torch.float32),
                FixedState((max(self.taps - 1, 1), self.channels), torch.float32))

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        per_token = (self.channels + self.num_heads + 256) * itemsize + self.value_size * itemsize + self.hidden_size * 4
        return tokens * (per_token + (self.channels + 2 * self.key_size + self.num_heads * (self.head_dim + 1) + self.value_size) * 4)

    def tensor_specs(self) -> dict[str, TensorSpec]:
        n = self.names
        low_a = -1 if self.decay_rank is None else self.decay_rank
        low_g = -1 if self.gate_rank is None else self.gate_rank
        sizes = {"q": self.key_size, "k": self.key_size, "v": self.value_size}
        specs = {self.name(n[p]): TensorSpec((sizes[p], self.hidden_size)) for p in ("q", "k", "v")}
        for p in ("q", "k", "v"):
            specs[self.name(f"{n[p]}.{self.conv_suffix}")] = TensorSpec((sizes[p], self.taps))
        specs.update({
            self.name(n["beta"]): TensorSpec((self.num_heads, self.hidden_size)),
            self.name(n["a_log"]): TensorSpec((self.num_heads,), init="zeros"),
            self.name(n["norm"]): TensorSpec((self.value_dim,), init="ones"),
            self.name(n["a1"]): TensorSpec((low_a, self.hidden_size)),
            self.name(n["a2"]): TensorSpec((self.num_heads * self.head_dim, low_a)),
            self.name(n["dt"]): TensorSpec((self.num_heads * self.head_dim,), init="zeros"),
            self.name(n["g1"]): TensorSpec((low_g, self.hidden_size)),
            self.name(n["g2"]): TensorSpec((self.value_size, low_g)),
            self.name(n["o"]): TensorSpec((self.hidden_size, self.value_size)),
        })
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        n = self.names
        a1, g1 = tensors[self.name(n["a1"])], tensors[self.name(n["g1"])]
        self.a2 = tensors[self.name(n["a2"])].contiguous()
        self.g2 = tensors[self.name(n["g2"])].contiguous()
        for low, high, what in ((a1, self.a2, "decay"), (g1, self.g2, "gate")):
            if low.shape[0] != high.shape[1] or not 1 <= low.shape[0] <= 256:
                raise ValueError(f"{self.prefix}: the {what}'s two matrices meet at {low.shape[0]} and {high.shape[1]} "
                                 "elements; they must agree and be 1..256")
        self.beta_at = self.channels
        self.decay_at = self.beta_at + self.num_heads
        self.gate_at = self.decay_at + int(a1.shape[0])
        self.fused = torch.cat([tensors[self.name(n[key])] for key in ("q", "k", "v", "beta")] + [a1, g1], dim=0).contiguous()
        del a1, g1
        self.conv_weight = torch.cat([tensors[self.name(f"{n[p]}.{self.conv_suffix}")] for p in ("q", "k", "v")], dim=0).contiguous()
        self.dt = tensors[self.name(n["dt"])].contiguous()
        self.a_log = tensors[self.name(n["a_log"])].float().contiguous()
        self.gain = tensors[self.name(n["norm"])].contiguous()
        self.o_weight = tensors[self.name(n["o"])].contiguous()

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        return self.runtime.ops.linear(self.heads_out(x, ctx, cache), self.o_weight, for_residual=True)

    o_bias_tensor = None

    @property
    def out_features(self) -> int:
        """The width of what the output matrix multiplies."""
        return self.value_size

    def scales_its_heads(self) -> bool:
        return True

    def heads_out(self, x: torch.Tensor, ctx, cache, *, scale: float = 1.0, out: tuple | None = None) -> torch.Tensor:
        """Everything but the output matrix: ``[T, H Dv]`` of the run dtype times ``scale``, optionally written into
        columns of a wider buffer (``out = (buffer, col0)``)."""
        ops, dtype = self.runtime.ops, self.runtime.dtype
        memory, held = cache
        proj = ops.linear(x, self.fused)
        u = ops.short_conv(proj, 0, self.conv_weight, held.state, ctx.state_slots, ctx.token_seq, ctx.query_start_loc,
                           tokens=ctx.num_tokens, num_seqs=ctx.num_seqs, dtype=dtype, silu=True, out_float32=True)
        return ops.delta_rule(u, proj, beta_at=self.beta_at, decay_at=self.decay_at, gate_at=self.gate_at, a2=self.a2,
                              dt_bias=self.dt, a_log=self.a_log, g2=self.g2, gain=self.gain, eps=self.norm_eps,
                              state=memory.state, state_slots=ctx.state_slots, query_start_loc=ctx.query_start_loc,
                              tokens=ctx.num_tokens, num_seqs=ctx.num_seqs, heads=self.num_heads, kv_heads=self.num_kv_heads,
                              head_dim=self.head_dim, value_dim=self.value_dim, dtype=dtype,
                              num_long_seqs=0 if ctx.recorded else ctx.num_prefill_seqs, scale=scale, out=out)
