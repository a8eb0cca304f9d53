"""Block arrangements (src/turboserve/engine/model/layers.py:443-487)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.parts.base import Block, CacheView, Part, PartSpec, ResidualStream, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_block


@register_block("prenorm")
class PreNormBlock(Block):
    """``h += mixer(norm_a(h)); h += feed_forward(norm_b(h))`` (layers.py:479-487).

    The sums are carried in the 32-bit residual stream; each part's output waits in
    ``stream.pending`` until the next norm adds it, in the same pass that normalises.
    ``mixer_norm_name`` / ``ff_norm_name`` / ``mixer_name`` / ``ff_name`` are the checkpoint
    names of the four parts under the block's prefix.  A block without a feed-forward
    (``feed_forward=None``) is its first half alone and has no second norm."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        mixer: PartSpec,
        feed_forward: PartSpec | None,
        mixer_norm: PartSpec,
        ff_norm: PartSpec | None,
        mixer_name: str = "self_attn",
        ff_name: str = "mlp",
        mixer_norm_name: str = "input_layernorm",
        ff_norm_name: str = "post_attention_layernorm",
    ) -> None:
        super().__init__(prefix, runtime)
        self.mixer_norm = build_part("norm", mixer_norm, self.name(mixer_norm_name), runtime)
        self.mixer = build_part("mixer", mixer, self.name(mixer_name), runtime)
        self.ff_norm = self.feed_forward = None
        if feed_forward is not None:
            if ff_norm is None:
                raise ValueError(f"{prefix}: a feed-forward needs its norm")
            self.ff_norm = build_part("norm", ff_norm, self.name(ff_norm_name), runtime)
            self.feed_forward = build_part("feed_forward", feed_forward, self.name(ff_name), runtime)

    def parts(self) -> list[Part]:
        if self.feed_forward is None:
            return [self.mixer_norm, self.mixer]
        return [self.mixer_norm, self.mixer, self.ff_norm, self.feed_forward]

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """A norm's output stays alive while the part it feeds runs."""
        first = self.mixer_norm.activation_bytes(tokens, itemsize) + self.mixer.activation_bytes(tokens, itemsize)
        if self.feed_forward is None:
            return first
        return max(first, self.ff_norm.activation_bytes(tokens, itemsize) + self.feed_forward.activation_bytes(tokens, itemsize))

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs: dict[str, TensorSpec] = {}
        for part in self.parts():
            specs.update(part.tensor_specs())
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.load(tensors)

    def forward(self, stream: ResidualStream, ctx, cache: CacheView) -> ResidualStream:
        x = self.mixer_norm.forward_residual(stream)
        stream.pending = self.mixer.forward(x, ctx, cache)
        if self.feed_forward is None:
            return stream
        x = self.ff_norm.forward_residual(stream)
        stream.pending = self.feed_forward.forward(x, ctx)
        return stream


@register_block("parallel")
class ParallelBlock(Block):
    """``h += mixer(n) + feed_forward(n)`` with one ``n = norm(h)`` that both parts read.

    The feed-forward's output waits in ``stream.pending`` for the next norm, as in the pre-norm
    block; the mixer's waits beside it in ``stream.also`` where it is 32-bit partial sums (steps of
    few tokens), and is otherwise added into the 32-bit residual stream by a pass of its own
    (``ops.stream_fold``).  A block without a feed-forward (``feed_forward=None``) leaves the mixer's
    output pending instead.  ``norm_name`` / ``mixer_name`` / ``ff_name`` are the checkpoint names
    of the parts under the block's prefix."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        mixer: PartSpec,
        feed_forward: PartSpec | None,
        norm: PartSpec,
        mixer_name: str = "mix",
        ff_name: str = "mlp",
        norm_name: str = "norm1",
    ) -> None:
        super().__init__(prefix, runtime)
        self.norm = build_part("norm", norm, self.name(norm_name), runtime)
        self.mixer = build_part("mixer", mixer, self.name(mixer_name), runtime)
        self.feed_forward = None
        if feed_forward is not None:
            self.feed_forward = build_part("feed_forward", feed_forward, self.name(ff_name), runtime)

    def parts(self) -> list[Part]:
        return [self.norm, self.mixer] if self.feed_forward is None else [self.norm, self.mixer, self.feed_forward]

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The norm's output stays alive while both parts run, one after the other."""
        largest = max(part.activation_bytes(tokens, itemsize) for part in self.parts()[1:])
        return self.norm.activation_bytes(tokens, itemsize) + largest

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs: dict[str, TensorSpec] = {}
        for part in self.parts():
            specs.update(part.tensor_specs())
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.load(tensors)

    def forward(self, stream: ResidualStream, ctx, cache: CacheView) -> ResidualStream:
        x = self.norm.forward_residual(stream)
        mixed = self.mixer.forward(x, ctx, cache)
        if self.feed_forward is None:
            stream.pending = mixed
            return stream
        if mixed.dim() == 3:  # 32-bit partial sums (steps of few tokens): the next norm adds them with the feed-forward's
            stream.also = mixed
        else:
            self.runtime.ops.stream_fold(stream.residual, mixed, self.runtime.dtype)
        stream.pending = self.feed_forward.forward(x, ctx)
        return stream


@register_block("sandwich")
class SandwichBlock(Block):
    """``h += m * norm_a2(mixer(norm_a(h))); h += m * norm_b2(feed_forward(norm_b(h)))``: a norm before
    and one behind each part, and a multiplier ``m`` (``residual_scale``) on what is added.

    The norm behind a part is not a pass of its own: the part's output waits in ``stream.pending``
    with the norm's rule beside it (``stream.pending_norm``), and the next norm that carries the
    residual sum (this block's, the next block's or the head's) normalises it, scales it and adds it,
    all in 32-bit, before it normalises the sum.  A block without a feed-forward
    (``feed_forward=None``) is its first half alone.  The four norms' checkpoint names under the
    block's prefix are ``mixer_norm_name``, ``mixer_post_name``, ``ff_norm_name``, ``ff_post_name``."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        mixer: PartSpec,
        feed_forward: PartSpec | None,
        norm: PartSpec,
        residual_scale: float = 1.0,
        mixer_name: str = "mix",
        ff_name: str = "mlp",
        mixer_norm_name: str = "norm1",
        mixer_post_name: str = "norm1b",
        ff_norm_name: str = "norm2",
        ff_post_name: str = "norm2b",
    ) -> None:
        super().__init__(prefix, runtime)
        self.residual_scale = float(residual_scale)
        self.mixer_norm = build_part("norm", norm, self.name(mixer_norm_name), runtime)
        self.mixer = build_part("mixer", mixer, self.name(mixer_name), runtime)
        self.mixer_post = build_part("norm", norm, self.name(mixer_post_name), runtime)
        self.ff_norm = self.feed_forward = self.ff_post = None
        if feed_forward is not None:
            self.ff_norm = build_part("norm", norm, self.name(ff_norm_name), runtime)
            self.feed_forward = build_part("feed_forward", feed_forward, self.name(ff_name), runtime)
            self.ff_post = build_part("norm", norm, self.name(ff_post_name), runtime)

    def parts(self) -> list[Part]:
        first = [self.mixer_norm, self.mixer, self.mixer_post]
        return first if self.feed_forward is None else [*first, self.ff_norm, self.feed_forward, self.ff_post]

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """A norm's output stays alive while the part it feeds runs."""
        first = self.mixer_norm.activation_bytes(tokens, itemsize) + self.mixer.activation_bytes(tokens, itemsize)
        if self.feed_forward is None:
            return first
        return max(first, self.ff_norm.activation_bytes(tokens, itemsize) + self.feed_forward.activation_bytes(tokens, itemsize))

    def tensor_specs(self) -> dict[str, TensorSpec]:
        specs: dict[str, TensorSpec] = {}
        for part in self.parts():
            specs.update(part.tensor_specs())
        return specs

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        for part in self.parts():
            part.load(tensors)

    def forward(self, stream: ResidualStream, ctx, cache: CacheView) -> ResidualStream:
        x = self.mixer_norm.forward_residual(stream)
        stream.pending = self.mixer.forward(x, ctx, cache)
        stream.pending_norm = self.mixer_post.pending_rule(self.residual_scale)
        if self.feed_forward is None:
            return stream
        x = self.ff_norm.forward_residual(stream)
        stream.pending = self.feed_forward.forward(x, ctx)
        stream.pending_norm = self.ff_post.pending_rule(self.residual_scale)
        return stream
