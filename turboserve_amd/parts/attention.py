"""Grouped-query attention over the paged cache (src/turboserve/engine/model/layers.py:311-391,
src/turboserve/engine/model/attention.py:213-295)."""

from __future__ import annotations

from collections.abc import Mapping

import torch

from turboserve_amd.kernels.ops import attention_geometry_error
from turboserve_amd.parts.base import CacheNeed, FixedState, Mixer, PagedKV, PagedKVView, PartSpec, Runtime, TensorSpec
from turboserve_amd.parts.registry import build_part, register_mixer


def tiled_attention(ops, q, q_stride, k_pages, v_pages, table, ctx, **rule) -> torch.Tensor:
    """A step's attention by ``ops.attention_tiles``: the tile list of the requests that bring several
    tokens is made once per step and shared by the layers (a recorded step has none: single tokens)."""
    tiles = None
    if ctx.num_prefill_seqs > 0:
        reach = (rule.get("window"), rule.get("chunk"))
        tiles = ctx.derive(("attention_tiles_64", *reach), lambda step: ops.device_ints(
            ops.attention_tile_list(step.query_lens[:step.num_prefill_seqs], step.context_lens_host[:step.num_prefill_seqs],
                                    window=reach[0], chunk=reach[1])))
    return ops.attention_tiles(
        q, q_stride, k_pages, v_pages, table, ctx.query_start_loc, ctx.context_lens, tokens=ctx.num_tokens,
        prefill_tiles=tiles, num_prefill_seqs=ctx.num_prefill_seqs, num_decode_seqs=ctx.num_decode_seqs,
        max_decode_context=min(ctx.max_decode_context_len, table.shape[1] * k_pages.shape[2]), **rule)


@register_mixer("gqa_attention")
class GroupedQueryAttention(Mixer):
    """q/k/v projections (optionally biased), position encoding, cache write, attention of every
    token over its request's keys up to itself (optionally only the last ``window``), output
    projection.

    The three projections are held as one ``[(Hq + 2 Hkv) D, H]`` matrix (the checkpoint keeps
    them apart; ``load`` concatenates), so a step does one product for them.  Scale is a
    parameter (``head_dim ** -0.5`` for Qwen2, model_config.py:224-227).

    Optional, each a parameter of its own: ``value_dim`` (values of another width than the keys:
    the fused matrix is ``[Hq D + Hkv D + Hkv Dv, H]`` and the output projection reads ``Hq Dv``);
    ``head_norm = {"eps": e, "gain_offset": o}`` (every q and k head is divided by its root mean
    square, eps inside the root, and multiplied by ``o +`` a gain vector ``[D]`` that all heads
    share, one for q and one for k, in 32-bit, before the position encoding); ``softcap = c``
    (a scaled score ``s`` becomes ``c * tanh(s / c)`` before the softmax); ``span_norm = {"eps": e,
    "gain_offset": o}`` (all q heads of a token together are divided by their root mean square and
    multiplied by ``o +`` a gain of their full size ``[Hq D]``, the k heads likewise with a gain ``[Hkv
    D]``, stored under the same names as the per-head gains); ``chunk = C`` (the token at position
    ``i`` sees only keys from ``(i // C) * C`` on: chunks of positions counted from the request's
    start); ``sinks = n`` (the softmax's denominator counts ``n`` more keys of score 0 that have no
    value); ``sink_name``: the sinks' score is learned, one number per query head in the tensor of
    that name ``[Hq]`` (it is not scaled and gets no bias), instead of 0; ``value_mix = {"key": k,
    "source": bool, "name": n}``: the layers of a model that share ``key`` mix their values: the one
    marked ``source`` (the first of them to run) leaves its values as projected for the others of the
    same step, and every other stores and attends over ``(1 - w) v + w v_source`` with its own learned
    scalar ``w`` (tensor ``n``).  ``head_norm`` may also say ``"gain": False`` (the heads are divided by
    their root mean square and nothing else: no gain tensors) and ``"after_position": True`` (the norm
    follows the position encoding instead of preceding it).  ``values_are_keys``: there is no value
    matrix; a token's values are its keys as projected, before norm and encoding.  ``keep_first = n``
    (with a window): the first ``n`` keys of a request stay visible behind the window, at their true
    positions.  ``gate_name``: a matrix ``[Hq, hidden]`` of that name makes one number per head from the
    mixer's input, and the head's output is multiplied by its sigmoid before the output matrix (its rows
    ride behind the fused matrix's).  ``conv = {"taps": K, "suffix": s}``: each channel of q, k and v
    passes a causal convolution over time of ``K`` taps right behind the projection (weights ``[channels,
    K]`` under ``<tensor name>.<s>``, the last column the current token's); the request's last ``K - 1``
    projected rows are state that the cache keeps beside the pages.  ``query_temperature = {"coef": c,
    "every": n}``: the query at position ``p`` is multiplied by ``1 + c ln(floor((p + 1) / n) + 1)`` behind
    norm and encoding.  ``names``: the tensor
    names under the part's prefix of ``q, k, v, o`` (biases: the same with ``weight`` replaced by
    ``bias``) and of the two gains."""

    def __init__(
        self,
        prefix: str,
        runtime: Runtime,
        *,
        hidden_size: int,
        num_heads: int,
        num_kv_heads: int,
        head_dim: int,
        scale: float,
        qkv_bias: bool,
        out_bias: bool,
        window: int | None,
        position: PartSpec,
        value_dim: int | None = None,
        head_norm: Mapping | None = None,
        softcap: float = 0.0,
        names: Mapping[str, str] | None = None,
        span_norm: Mapping | None = None,
        chunk: int | None = None,
        sinks: float = 0.0,
        sink_name: str | None = None,
        value_mix: Mapping | None = None,
        values_are_keys: bool = False,
        keep_first: int = 0,
        gate_name: str | None = None,
        conv: Mapping | None = None,
        query_temperature: Mapping | None = None,
    ) -> None:
        super().__init__(prefix, runtime)
        # Refused here, when the model is put together, not at the first step after the weights
        # have been read: a geometry that no attention kernel takes.
        refusal = attention_geometry_error(int(num_heads), int(num_kv_heads), int(head_dim))
        if refusal is not None:
            raise ValueError(f"{prefix or 'attention'}: {refusal}")
        self.hidden_size = int(hidden_size)
        self.num_heads = int(num_heads)
        self.num_kv_heads = int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.scale = float(scale)
        self.qkv_bias = bool(qkv_bias)
        self.out_bias = bool(out_bias)
        self.window = None if window is None else int(window)
        self.position = build_part("position_encoding", position, prefix, runtime)
        self.value_dim = self.head_dim if value_dim is None else int(value_dim)
        self.values_are_keys = bool(values_are_keys)
        if self.values_are_keys and (self.value_dim != self.head_dim or value_mix is not None):
            raise ValueError(f"{prefix or 'attention'}: values that are the keys have the keys' size and are not mixed")
        self.keep_first = int(keep_first)
        if self.keep_first < 0 or (self.keep_first > 0 and (window is None or chunk is not None)):
            raise ValueError(f"{prefix or 'attention'}: kept first keys go with a window and without chunks")
        self.gate_name = gate_name
        self.conv_taps = None if conv is None else int(conv["taps"])
        self.conv_suffix = "conv" if conv is None else str(conv.get("suffix", "conv"))
        if self.conv_taps is not None and not 1 <= self.conv_taps <= 8:
            raise ValueError(f"{prefix or 'attention'}: a convolution of {self.conv_taps} taps is outside 1..8")
        if self.conv_taps is not None and (self.values_are_keys or value_mix is not None or span_norm is not None):
            raise ValueError(f"{prefix or 'attention'}: the convolution goes with a value matrix of its own and the per-head store")
        self.query_temperature = None
        if query_temperature is not None:
            self.query_temperature = (float(query_temperature["coef"]), int(query_temperature["every"]))
            if self.query_temperature[1] < 1:
                raise ValueError(f"{prefix or 'attention'}: a query temperature every {self.query_temperature[1]} positions")
        if not 1 <= self.value_dim <= 512:
            raise ValueError(f"{prefix or 'attention'}: values of {self.value_dim} elements are outside what the kernels take")
        self.softcap = float(softcap)
        self.head_norm_eps = None if head_norm is None else float(head_norm["eps"])
        self.head_norm_offset = 0.0 if head_norm is None else float(head_norm.get("gain_offset", 0.0))
        self.head_norm_gain = head_norm is not None and bool(head_norm.get("gain", True))
        self.head_norm_after = head_norm is not None and bool(head_norm.get("after_position", False))
        if span_norm is not None and head_norm is not None:
            raise ValueError(f"{prefix or 'attention'}: a norm per head and one over the whole projection exclude each other")
        self.span_norm_eps = None if span_norm is None else float(span_norm["eps"])
        self.span_norm_offset = 0.0 if span_norm is None else float(span_norm.get("gain_offset", 0.0))
        self.chunk = None if chunk is None else int(chunk)
        if self.chunk is not None and self.chunk < 1:
            raise ValueError(f"{prefix or 'attention'}: a chunk of {self.chunk} positions")
        self.sinks = float(sinks)
        if self.sinks < 0:
            raise ValueError(f"{prefix or 'attention'}: {self.sinks} sinks")
        self.sink_name = sink_name
        if sink_name is not None and self.sinks == 0.0:
            raise ValueError(f"{prefix or 'attention'}: learned sink scores need a count of sinks")
        self.sink_scores: torch.Tensor | None = None
        self.value_mix = None if value_mix is None else dict(value_mix)
        if self.value_mix is not None and head_norm is None:
            raise ValueError(f"{prefix or 'attention'}: values are mixed by the store that norms every head")
        self.mix_weight = 0.0
        self.names = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
                      "q_norm": "q_norm.weight", "k_norm": "k_norm.weight", **(names or {})}
        self.q_size = self.num_heads * self.head_dim
        self.kv_size = self.num_kv_heads * self.head_dim
        self.v_size = 0 if self.values_are_keys else self.num_kv_heads * self.value_dim
        self.out_size = self.num_heads * self.value_dim
        self.conv_weight: torch.Tensor | None = None
        self.q_gain: torch.Tensor | None = None
        self.k_gain: torch.Tensor | None = None
        self.qkv_weight: torch.Tensor | None = None
        self.qkv_bias_tensor: torch.Tensor | None = None
        self.o_weight: torch.Tensor | None = None
        self.o_bias_tensor: torch.Tensor | None = None

    def cache_need(self) -> CacheNeed:
        pages = PagedKV(self.num_kv_heads, self.head_dim, self.window,
                        None if self.value_dim == self.head_dim else self.value_dim, self.chunk, self.keep_first)
        if self.conv_taps is None:
            return pages
        # The request's last projected rows, 32-bit, beside its pages.
        return (pages, FixedState((max(self.conv_taps - 1, 1), self.q_size + self.kv_size + self.v_size), torch.float32))

    def _projections(self) -> tuple[str, ...]:
        return ("q", "k") if self.values_are_keys else ("q", "k", "v")

    def is_capturable(self) -> bool:
        return self.capturable and self.position.is_capturable()

    def step_fields(self) -> tuple:
        return self.position.step_fields()

    def activation_bytes(self, tokens: int, itemsize: int) -> int:
        """The fused projection, the attention output and the output projection (32-bit: it is
        added to the residual stream) of a step."""
        fused = (self.q_size + self.kv_size + self.v_size) * (2 if self.conv_taps is not None else 1)
        return tokens * ((fused + self.out_size) * itemsize + self.hidden_size * 4)

    def tensor_specs(self) -> dict[str, TensorSpec]:
        sizes = {"q": self.q_size, "k": self.kv_size, "v": self.v_size}
        specs = {self.name(self.names[p]): TensorSpec((sizes[p], self.hidden_size)) for p in self._projections()}
        specs[self.name(self.names["o"])] = TensorSpec((self.hidden_size, self.out_size))
        if self.qkv_bias:
            for p in self._projections():
                specs[self.name(self._bias(p))] = TensorSpec((sizes[p],))
        if self.out_bias:
            specs[self.name(self._bias("o"))] = TensorSpec((self.hidden_size,))
        if self.conv_taps is not None:
            for p in self._projections():
                specs[self.name(f"{self.names[p]}.{self.conv_suffix}")] = TensorSpec((sizes[p], self.conv_taps))
        if self.gate_name is not None:
            specs[self.name(self.gate_name)] = TensorSpec((self.num_heads, self.hidden_size))
        if self.head_norm_eps is not None and self.head_norm_gain:
            init = "zeros" if self.head_norm_offset == 1.0 else "ones"
            specs[self.name(self.names["q_norm"])] = TensorSpec((self.head_dim,), init=init)
            specs[self.name(self.names["k_norm"])] = TensorSpec((self.head_dim,), init=init)
        if self.span_norm_eps is not None:
            init = "zeros" if self.span_norm_offset == 1.0 else "ones"
            specs[self.name(self.names["q_norm"])] = TensorSpec((self.q_size,), init=init)
            specs[self.name(self.names["k_norm"])] = TensorSpec((self.kv_size,), init=init)
        if self.sink_name is not None:
            specs[self.name(self.sink_name)] = TensorSpec((self.num_heads,), init="zeros")
        if self.value_mix is not None and not self.value_mix.get("source"):
            specs[self.name(self.value_mix["name"])] = TensorSpec(())
        specs.update(self.position.tensor_specs())
        return specs

    def _bias(self, which: str) -> str:
        """The bias beside a matrix: ``weight`` replaced by ``bias`` in its name, or ``.b`` appended to a name
        without ``weight``."""
        name = self.names[which]
        return name.replace("weight", "bias") if "weight" in name else f"{name}.b"

    def load(self, tensors: Mapping[str, torch.Tensor]) -> None:
        rows = [tensors[self.name(self.names[p])] for p in self._projections()]
        if self.gate_name is not None:
            rows.append(tensors[self.name(self.gate_name)])
        self.qkv_weight = torch.cat(rows, dim=0).contiguous()
        del rows
        if self.qkv_bias:
            biases = [tensors[self.name(self._bias(p))] for p in self._projections()]
            if self.gate_name is not None:  # the gate's rows have no bias
                biases.append(torch.zeros((self.num_heads,), dtype=biases[0].dtype, device=biases[0].device))
            self.qkv_bias_tensor = torch.cat(biases, dim=0).contiguous()
        if self.conv_taps is not None:
            self.conv_weight = torch.cat(
                [tensors[self.name(f"{self.names[p]}.{self.conv_suffix}")] for p in self._projections()], dim=0).contiguous()
        self.o_weight = tensors[self.name(self.names["o"])].contiguous()
        if self.out_bias:
            self.o_bias_tensor = tensors[self.name(self._bias("o"))].contiguous()
        if (self.head_norm_eps is not None and self.head_norm_gain) or self.span_norm_eps is not None:
            self.q_gain = tensors[self.name(self.names["q_norm"])].contiguous()
            self.k_gain = tensors[self.name(self.names["k_norm"])].contiguous()
        if self.sink_name is not None:
            self.sink_scores = tensors[self.name(self.sink_name)].float().contiguous()
        if self.value_mix is not None and not self.value_mix.get("source"):
            self.mix_weight = float(tensors[self.name(self.value_mix["name"])].float().item())
        self.position.load(tensors)

    def forward(self, x: torch.Tensor, ctx, cache) -> torch.Tensor:
        return self.runtime.ops.linear(self.heads_out(x, ctx, cache), self.o_weight, self.o_bias_tensor, for_residual=True)

    @property
    def out_features(self) -> int:
        """The width of what the output matrix multiplies."""
        return self.out_size

    def scales_its_heads(self) -> bool:
        """Whether :meth:`heads_out` can apply a scale and write into a wider buffer (the gate's launch does both)."""
        return self.gate_name is not None

    def heads_out(self, x: torch.Tensor, ctx, cache, *, scale: float = 1.0, out: tuple | None = None) -> torch.Tensor:
        """Everything but the output matrix: ``[T, Hq Dv]`` of the run dtype, what that matrix multiplies.  With a gate
        per head the result may be multiplied by ``scale`` and written into columns of a wider buffer (``out =
        (buffer, col0)``): a caller that adds this mixer's output to another's can then run both output matrices as
        one product."""
        ops = self.runtime.ops
        qkv = proj = ops.linear(x, self.qkv_weight, self.qkv_bias_tensor)
        more, shape = {}, {}
        if self.conv_taps is not None:
            cache, held = cache
            # q, k and v of the step through the convolution; the gate's columns stay in `proj`.
            qkv = ops.short_conv(proj, 0, self.conv_weight, held.state, ctx.state_slots, ctx.token_seq, ctx.query_start_loc,
                                 tokens=ctx.num_tokens, num_seqs=ctx.num_seqs, dtype=self.runtime.dtype)
        elif self.gate_name is not None:
            shape["tail"] = self.num_heads
        if self.values_are_keys:
            shape["values_are_keys"] = True
        if self.query_temperature is not None:
            shape["query_temperature"] = self.query_temperature
        if self.value_dim != self.head_dim:
            more["value_dim"] = self.value_dim
        if self.head_norm_eps is not None:
            more["head_norm"] = (self.q_gain, self.k_gain, self.head_norm_eps, self.head_norm_offset)
            if not self.head_norm_gain:
                shape["normed"] = True
            if self.head_norm_after:
                shape["norm_after"] = True
        if shape:
            more["shape"] = shape
        if self.span_norm_eps is not None:
            more["span_norm"] = (self.q_gain, self.k_gain, self.span_norm_eps, self.span_norm_offset)
        if self.value_mix is not None:
            key = ("value_mix", self.value_mix["key"])
            if self.value_mix.get("source"):
                kept = torch.empty((ctx.num_tokens, self.v_size), dtype=torch.float32, device=x.device)
                ctx.carried[key] = kept
                more["values"] = {"keep": kept}
            else:
                more["values"] = {"blend": (ctx.carried[key], self.mix_weight)}
        q, q_stride = self.position.encode_and_store(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, ctx, cache, **more
        )
        attended = self.attend(q, q_stride, ctx, cache)
        if self.gate_name is not None:
            # Every head's output times the sigmoid of its gate (the projection's last columns), rounded once.
            return ops.head_gate(attended, proj, self.q_size + self.kv_size + self.v_size, self.num_heads, self.runtime.dtype,
                                 scale=scale, out=out)
        if scale != 1.0 or out is not None:
            raise ValueError(f"{self.prefix}: without a gate per head nothing scales or places the heads' output")
        return attended

    def attend(self, qkv: torch.Tensor, q_stride: int, ctx, cache: PagedKVView) -> torch.Tensor:
        """``[T, Hq D]`` attention output for the step's encoded queries: the first ``Hq D``
        elements of every ``q_stride``-long row of ``qkv``.

        bfloat16 runs use the matrix-core kernels where the geometry allows: one launch for the
        multi-token requests at the front of the batch, one for the single-token requests
        behind them; a position encoding that biases the scores, a chunk mask, sinks or values of
        another width than the keys go through the tiled matrix-core kernel that takes them; every
        32-bit run and any other geometry goes through the generic kernel."""
        ops = self.runtime.ops
        table = ctx.block_tables[cache.group]
        slopes = self.position.score_slopes(self.num_heads)
        bias = self.position.score_bias_table(self.num_heads)
        fast = (slopes is None and bias is None and self.value_dim == self.head_dim and self.chunk is None and self.sinks == 0.0
                and self.keep_first == 0 and ops.mfma_attention_supported(qkv.dtype, self.head_dim, cache.block_size))
        if fast:
            out = ops.rows_buffer(ctx.num_tokens, self.out_size, qkv.dtype, qkv.device)
            if ctx.num_prefill_seqs > 0:
                # The launch's list of row blocks is the same for every layer with this geometry.
                rows = ops.prefill_block_rows(self.head_dim, self.num_heads, self.num_kv_heads)
                geometry = dict(heads=self.num_heads, kv_heads=self.num_kv_heads, head_dim=self.head_dim,
                                block_size=cache.block_size, window=self.window)
                blocks = ctx.derive(("attention_prefill_blocks", rows, *geometry.values()), lambda step: ops.prefill_blocks(
                    step.query_lens[:step.num_prefill_seqs], step.context_lens_host[:step.num_prefill_seqs], rows, **geometry))
                ops.attention_prefill(
                    out, qkv, q_stride, cache.k, cache.v, table, ctx.query_start_loc, ctx.context_lens,
                    blocks, self.num_heads, self.scale, self.window, ctx.max_prefill_context_len, rows,
                    softcap=self.softcap,
                )
            if ctx.num_decode_seqs > 0:
                ops.attention_decode(
                    out, qkv, q_stride, cache.k, cache.v, table, ctx.query_start_loc, ctx.context_lens,
                    ctx.num_prefill_seqs, ctx.num_decode_seqs, self.num_heads, self.scale, self.window,
                    min(ctx.max_decode_context_len, table.shape[1] * cache.block_size),
                    ctx.max_decode_context_dev, softcap=self.softcap,
                )
            return out
        if ops.tiled_attention_supported(qkv.dtype, self.head_dim, self.value_dim, cache.block_size, q_stride):
            return tiled_attention(ops, qkv, q_stride, cache.k, cache.v, table, ctx, heads=self.num_heads, scale=self.scale,
                                   window=self.window, chunk=self.chunk, sinks=self.sinks, slopes=slopes, softcap=self.softcap,
                                   sink_scores=self.sink_scores, distance_bias=bias, keep_first=self.keep_first)
        return ops.paged_attention_generic(
            qkv, q_stride, cache.k, cache.v, table, ctx.token_seq, ctx.positions,
            self.num_heads, self.scale, self.window, slopes, self.softcap, chunk=self.chunk, sinks=self.sinks,
            sink_scores=self.sink_scores, distance_bias=bias, keep_first=self.keep_first,
        )
