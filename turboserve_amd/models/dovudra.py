"""Dovudra: from its configuration to a plan of parts.

A decoder whose blocks have a norm before and a norm behind each part, and a multiplier on what is
added: ``x += m norm1b(mix(norm1(x)))``, ``x += m norm2b(ff(norm2(x)))``; norms are ``x / sqrt(mean(x^2) +
eps) * g``.  The stream starts as the token's row of ``embed``, and the same table is the output
matrix behind ``final.norm``.  Each layer is described on its own, with one of two mixers:

* ``attention``: grouped-query attention without rotation; a norm per query and key head (one gain
  for all heads); the score of the key ``n`` back is ``scale (q . k)`` plus an entry of a learned
  table ``rel [B, H]`` picked by a bucket of ``n`` (exact below ``B / 2``, logarithmic up to
  ``bias_max``); a window; the softmax's denominator counts one more term ``exp(sink_h)``; the
  layers marked ``v_mix`` behind the first such layer store ``(1 - w) v + w v_first`` as their values.
* ``latent_attention``: keys and values of all heads from one cached latent per token and a rotated
  key part that the heads share; rotation of neighbouring pairs with stretched slow frequencies; a
  window; every head's output times the sigmoid of a gate made from the mixer's input.

Feed-forward: ``down(relu(up(h))^2)``, or none.  Tensors are named ``l<i>.norm1``, ``l<i>.mix.q``,
``l<i>.mlp.up`` and so on, without a ``weight`` suffix.
"""

from __future__ import annotations

from turboserve_amd.config.dovudra_config import BiasedAttentionSizes, DovudraConfig, GatedLatentSizes
from turboserve_amd.models.decoder import LayerCall, LayerSpec, ModelPlan
from turboserve_amd.parts.base import PartSpec

#: Fixed by the design.
ATTENTION_SINKS = 1.0
FEED_FORWARD_ACTIVATION = "relu_squared"
#: Positions the rotary tables are first made for; they grow by doubling.
INITIAL_POSITIONS = 4096

ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm"}


def _mixer(index: int, width: int, eps: float, sizes, source: int | None) -> PartSpec:
    if isinstance(sizes, BiasedAttentionSizes):
        mix = None
        if sizes.v_mix:
            mix = {"key": "v_mix", "source": index == source, "name": "vmix"}
        return PartSpec("gqa_attention", {
            "hidden_size": width, "num_heads": sizes.heads, "num_kv_heads": sizes.kv_heads, "head_dim": sizes.dim,
            "value_dim": sizes.vdim, "scale": sizes.scale, "qkv_bias": False, "out_bias": False, "window": sizes.window,
            "position": PartSpec("distance_buckets", {"num_heads": sizes.heads, "max_distance": sizes.bias_max,
                                                      "buckets": sizes.bias_rows, "reach": sizes.window, "table_name": "rel"}),
            "head_norm": {"eps": eps, "gain_offset": 0.0}, "sinks": ATTENTION_SINKS, "sink_name": "sink",
            "value_mix": mix, "names": ATTENTION_NAMES,
        })
    if isinstance(sizes, GatedLatentSizes):
        scaling = None if sizes.rot_scaling is None else sizes.rot_scaling.as_mapping()
        return PartSpec("latent_attention", {
            "hidden_size": width, "num_heads": sizes.heads, "head_dim": sizes.dim, "rot_dim": sizes.rot_dim,
            "value_dim": sizes.vdim, "rank": sizes.kv_rank, "scale": sizes.scale, "norm_eps": eps, "window": sizes.window,
            "gate_name": "g",
            "rotation": PartSpec("rope", {"head_dim": sizes.rot_dims, "theta": sizes.rot_base, "max_positions": INITIAL_POSITIONS,
                                          "interpolation": scaling, "exact": True, "neighbours": True}),
        })
    raise TypeError(f"no mixer for {sizes!r}")


def dovudra_plan(config: DovudraConfig) -> ModelPlan:
    width = config.hidden_size
    norm = PartSpec("rmsnorm", {"size": width, "eps": config.norm_eps, "one_rounding": True, "weight_name": ""})
    source = config.first_value_mixer()
    layers = []
    for index, layer in enumerate(config.layers):
        feed_forward = None
        if layer.mlp is not None:
            feed_forward = PartSpec("mlp", {"hidden_size": width, "intermediate_size": layer.mlp.ff,
                                            "activation": FEED_FORWARD_ACTIVATION, "names": ("up", "down")})
        block = PartSpec("sandwich", {
            "mixer": _mixer(index, width, config.norm_eps, layer.mixer, source), "feed_forward": feed_forward, "norm": norm,
            "residual_scale": config.residual_mult,
        })
        layers.append(LayerSpec(prefix=f"l{index}", block=block))
    # The first mixing layer's own weight is in the file and is not read.
    unread = () if source is None else (f"l{source}.mix.vmix",)
    return ModelPlan(
        ignorable=unread,
        vocab_size=config.vocab_size,
        hidden_size=width,
        layers=tuple(layers),
        schedule=tuple(LayerCall(index) for index in range(len(layers))),
        embedding=PartSpec("token_table", {"vocab_size": config.vocab_size, "hidden_size": width, "weight_name": ""}),
        head=PartSpec("norm_linear", {"vocab_size": config.vocab_size, "hidden_size": width, "norm": norm,
                                      "norm_prefix": "final.norm", "tied_to": "embed", "weight_name": ""}),
        embedding_prefix="embed",
        head_prefix="head",
    )
