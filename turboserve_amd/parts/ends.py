"""The two ends of a decoder: the token table its residual stream starts from, and the head
that turns the stream into scores over the vocabulary (src/turboserve/engine/model/model.py:
64-72 and :105-108, :139-142 for the tie)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import Embedding, Head, PartSpec, ResidualStream, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_embedding, register_head


@register_embedding("token_table")
class TokenTable(Embedding):
    """One row of ``[V, H]`` per token id, into the 32-bit residual stream.  ``weight_name``: the
    table's name under the part's prefix (empty: the prefix itself)."""

    def __init__(self, prefix: str, runtime: Runtime, *, vocab_size: int, hidden_size: int,
                 weight_name: str = "weight") -> None:
        super().__init__(prefix, runtime)
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.weight_name = weight_name
        self.weight: torch.Tensor | None = None

    def tensor_specs(self) -> dict[str, TensorSpec]:
        return {self.name(self.weight_name): TensorSpec((self.vocab_size, self.hidden_size))}

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.weight = tensors[self.name(self.weight_name)].contiguous()

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        return self.runtime.ops.embed(self.weight, token_ids)


def sinusoid_table(capacity: int, width: int, base: float) -> torch.Tensor:
    """32-bit ``[capacity, width]``: entry ``2i`` of row ``p`` is ``sin(p * base^(-2i/width))``, entry
    ``2i + 1`` the cosine of the same angle.  Angles are formed in 64-bit on the CPU and the
    results rounded once, so a row does not depend on how far the table reaches."""
    pairs = (width + 1) // 2
    rates = torch.tensor(base, dtype=torch.float64) ** (-2.0 * torch.arange(pairs, dtype=torch.float64) / width)
    angles = torch.outer(torch.arange(capacity, dtype=torch.float64), rates)
    table = torch.stack([angles.sin(), angles.cos()], dim=2).reshape(capacity, 2 * pairs)[:, :width]
    return table.to(torch.float32).contiguous()


@register_embedding("token_table_sinusoid")
class SinusoidTokenTable(TokenTable):
    """A token's row of the table plus the sinusoidal vector of its position
    (:func:`sinusoid_table`), summed in 32-bit.  The position table is made at the first step for
    ``max_positions`` rows and grows by doubling when a step reaches further; a recorded step
    holds the address of the table it was recorded with, so superseded tables are kept (they
    cover every position such a recording can bring)."""

    def __init__(self, prefix: str, runtime: Runtime, *, vocab_size: int, hidden_size: int, base: float = 10000.0,
                 max_positions: int = 4096, weight_name: str = "weight") -> None:
        super().__init__(prefix, runtime, vocab_size=vocab_size, hidden_size=hidden_size, weight_name=weight_name)
        self.base = float(base)
        self.initial_capacity = int(max_positions)
        self.capacity = 0
        self.at: torch.Tensor | None = None
        self.superseded: list[torch.Tensor] = []

    def ensure_capacity(self, num_positions: int) -> None:
        if num_positions <= self.capacity:
            return
        target = max(num_positions, 2 * self.capacity, self.initial_capacity, 16)
        if self.at is not None:
            self.superseded.append(self.at)
        self.at = sinusoid_table(target, self.hidden_size, self.base).to(self.runtime.device)
        self.capacity = target

    def forward(self, token_ids: torch.Tensor, ctx) -> torch.Tensor:
        self.ensure_capacity(ctx.max_context_len)
        return self.runtime.ops.embed_positions(self.weight, token_ids, ctx.positions, self.at)


@register_head("norm_linear")
class NormLinearHead(Head):
    """A norm over the summed stream, then ``[V, H]`` without bias, at the wanted rows only
    (model.py:108, :237-244).  ``tied_to`` names the tensor of another part (the token table)
    that serves as the matrix; the checkpoint's own copy under this part's prefix is then not
    read (the reference shares one parameter, model.py:139-142).  ``softcap = c``: the scores ``z`` leave as
    ``c tanh(z / c)``."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        vocab_size: int,
        hidden_size: int,
        norm: PartSpec,
        norm_prefix: str,
        tied_to: str | None,
        weight_name: str = "weight",
        softcap: float = 0.0,
    ) -> None:
        super().__init__(prefix, runtime)
        self.softcap = float(softcap)
        if self.softcap < 0.0:
            raise ValueError(f"a cap of {self.softcap} on the scores")
        self.own_weight_name = weight_name
        self.vocab_size = int(vocab_size)
        self.hidden_size = int(hidden_size)
        self.norm = build_part("norm", norm, norm_prefix, runtime)
        self.tied_to = tied_to
        self.weight: torch.Tensor | None = None

    @property
    def weight_name(self) -> str:
        return self.tied_to or self.name(self.own_weight_name)

    def is_capturable(self) -> bool:
        return self.capturable and self.norm.is_capturable()

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs = dict(self.norm.tensor_specs())
        specs[self.weight_name] = TensorSpec((self.vocab_size, self.hidden_size))
        return specs

    def ignorable_names(self) -> set[str]:
        return {self.name(self.own_weight_name)} if self.tied_to else set()

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        self.norm.load(tensors)
        self.weight = tensors[self.weight_name].contiguous()

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        return self.norm.activation_bytes(tokens, itemsize)

    def forward(self, stream: ResidualStream, rows: torch.Tensor) -> torch.Tensor:
        hidden = self.norm.forward_residual(stream, rows)
        scores = self.runtime.ops.linear_float32_out(hidden, self.weight)
        if self.softcap > 0.0:
            scores = self.runtime.ops.tanh_cap(scores.contiguous(), self.softcap)
        return scores


def standard_ends(vocab_size: int, hidden_size: int, norm: PartSpec, *, tie_head: bool,
                  embedding_prefix: str = "model.embed_tokens", norm_prefix: str = "model.norm") -> dict:
    """The ``embedding`` and ``head`` entries of a plan for the usual pair: a token table, and a
    final norm followed by a matrix that is the table itself (``tie_head``) or the head's own."""
    return {
        "embedding": PartSpec("token_table", {"vocab_size": vocab_size, "hidden_size": hidden_size}),
        "head": PartSpec("norm_linear", {
            "vocab_size": vocab_size, "hidden_size": hidden_size, "norm": norm, "norm_prefix": norm_prefix,
            "tied_to": f"{embedding_prefix}.weight" if tie_head else None,
        }),
        "embedding_prefix": embedding_prefix,
    }
