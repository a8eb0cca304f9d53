"""Legavik: from its configuration to a plan of parts.

A pre-norm decoder, ``x += mix(norm1(x))``, ``x += ff(norm2(x))``, whose norms compute no statistics:
``tanh(alpha x) * w + b``.  The stream starts as the token's row of ``embed``; behind ``final.norm`` the output
matrix ``head`` makes the logits, which leave as ``c tanh(z / c)``.  Each layer is described on its own,
with one of two mixers:

* ``attention``: grouped-query attention without a value matrix (a token's values are its keys as
  projected); rotation in halves of a head's first elements with stretched slow frequencies, then every
  query and key head divided by its root mean square; a window behind which the request's first tokens
  stay visible; every head's output times the sigmoid of a gate made from the mixer's input.
* ``parallel``: two mixers that read the same input, their outputs added with a weight each.  ``left`` is
  causal attention with biased projections, a short convolution over time on q, k and v, a norm per q and
  k head with one gain for all heads, a query temperature that grows with the logarithm of the position,
  and the gate per head; ``right`` is the gated delta rule (short convolutions with silu, unit q and k, a
  decay per key channel, a state per head that is corrected and read, a normed and gated read-out).

Feed-forward: routed experts with a softmax router, a group's mark its best expert, weights normalised;
or none.  Tensors are named ``l<i>.norm1``, ``l<i>.mix.q``, ``l<i>.mix.left.q.conv``, ``l<i>.mlp.e<j>.gate`` and so
on, without a ``weight`` suffix; a bias is ``<tensor>.b``.
"""

from __future__ import annotations

from turboserve_amd.config.legavik_config import ConvolvedAttentionSizes, DeltaRuleSizes, KeyedAttentionSizes, LegavikConfig, ParallelSizes
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec

#: Positions the rotary tables are first made for; they grow by doubling.
INITIAL_POSITIONS = 4096

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}
GATE_NAME = "g"


def _keyed_attention(width: int, eps: float, sizes: KeyedAttentionSizes) -> PartSpec:
    position = PartSpec("none", {})
    if sizes.rot_base is not None:
        scaling = None if sizes.rot_scaling is None else sizes.rot_scaling.as_mapping()
        position = PartSpec("rope", {"head_dim": sizes.rot_dims, "theta": sizes.rot_base, "max_positions": INITIAL_POSITIONS,
                                     "interpolation": scaling, "exact": True})
    return PartSpec("gqa_attention", {
        "hidden_size": width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
        "scale": sizes.scale, "qkv_bias": False, "out_bias": False, "window": sizes.window, "keep_first": sizes.keep_first,
        "position": position, "values_are_keys": True, "head_norm": {"eps": eps, "gain": False, "after_position": True},
        "gate_name": GATE_NAME, "names": ATTENTION_NAMES,
    })


def _convolved_attention(width: int, eps: float, sizes: ConvolvedAttentionSizes) -> PartSpec:
    temperature = None if sizes.temp_coef is None else {"coef": sizes.temp_coef, "every": sizes.temp_every}
    return PartSpec("gqa_attention", {
        "hidden_size": width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
        "value_dim": sizes.vdim, "scale": sizes.scale, "qkv_bias": True, "out_bias": True, "window": None,
        "position": PartSpec("none", {}), "head_norm": {"eps": eps, "gain_offset": 0.0},
        "conv": None if sizes.taps is None else {"taps": sizes.taps, "suffix": "conv"},
        "query_temperature": temperature, "gate_name": GATE_NAME, "names": ATTENTION_NAMES,
    })


def _delta_rule(width: int, eps: float, sizes: DeltaRuleSizes) -> PartSpec:
    return PartSpec("gated_delta_rule", {
        "hidden_size": width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
        "value_dim": sizes.vdim, "taps": sizes.taps, "norm_eps": eps, "decay_rank": sizes.decay_rank, "gate_rank": sizes.gate_rank,
    })


def _mixer(width: int, eps: float, sizes) -> PartSpec:
    if isinstance(sizes, KeyedAttentionSizes):
        return _keyed_attention(width, eps, sizes)
    if isinstance(sizes, ParallelSizes):
        return PartSpec("mixer_pair", {
            "left": _convolved_attention(width, eps, sizes.left), "right": _delta_rule(width, eps, sizes.right),
            "left_scale": sizes.left_scale, "right_scale": sizes.right_scale,
        })
    raise TypeError(f"no mixer for {sizes!r}")


def legavik_plan(config: LegavikConfig) -> ModelPlan:
    width = config.hidden_size
    norm = PartSpec("tanh_norm", {"size": width, "weight_name": ""})
    layers = []
    for index, layer in enumerate(config.layers):
        feed_forward = None
        if layer.mlp is not None:
            feed_forward = PartSpec("routed_experts", {
                "hidden_size": width, "expert_size": layer.mlp.ff, "experts": layer.mlp.experts, "top": layer.mlp.top,
                "groups": layer.mlp.groups, "keep": layer.mlp.keep, "router_scores": "softmax", "group_mark": "max",
            })
        block = PartSpec("prenorm", {
            "mixer": _mixer(width, config.norm_eps, layer.mixer), "feed_forward": feed_forward, "mixer_norm": norm,
            "ff_norm": None if feed_forward is None else norm, "mixer_name": "mix", "ff_name": "mlp",
            "mixer_norm_name": "norm1", "ff_norm_name": "norm2",
        })
        layers.append(LayerSpec(prefix=f"l{index}", block=block))
    return ModelPlan(
        vocab_size=config.vocab_size,
        hidden_size=width,
        layers=tuple(layers),
        schedule=tuple(LayerCall(index) for index in range(len(layers))),
        embedding=PartSpec("token_table", {"vocab_size": config.vocab_size, "hidden_size": width, "weight_name": ""}),
        head=PartSpec("norm_linear", {"vocab_size": config.vocab_size, "hidden_size": width, "norm": norm,
                                      "norm_prefix": "final.norm", "tied_to": None, "weight_name": "",
                                      "softcap": config.logit_softcap or 0.0}),
        embedding_prefix="embed",
        head_prefix="head",
    )
