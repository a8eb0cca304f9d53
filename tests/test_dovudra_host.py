"""Dovudra without a GPU: the configuration reader and its refusals, the tensors a model expects,
the cache each layer asks for, and the mechanisms' host-side arithmetic (buckets of distances,
stretched frequencies) in the engine and in the plain implementation against direct formulas."""

from __future__ import annotations

import json
import math

import pytest
import torch

import dovudra_tiny as dt
from plain import dovudra_plain as plain
from turboserve_amd.config.dovudra_config import DovudraConfig
from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.registry import parse_model_config
from turboserve_amd.parts.base import PagedKV
from turboserve_amd.parts.rope import distance_bucket, exact_rotary_tables, interpolated_frequencies
from turboserve_amd.weights.random_init import describe_model


def test_the_reader_takes_every_size_from_the_file():
    config = parse_model_config(dt.CONFIG_A)
    assert isinstance(config, DovudraConfig)
    assert (config.vocab_size, config.hidden_size, config.norm_eps, config.residual_mult) == (211, 64, 1e-5, 0.5)
    assert [layer.type for layer in config.layers] == ["attention", "latent_attention", "attention", "attention"]
    first, latent, third, _ = (layer.mixer for layer in config.layers)
    assert (first.heads, first.kv_heads, first.dim, first.vdim, first.window, first.scale) == (4, 2, 16, 8, 20, 0.3)
    assert (first.bias_max, first.bias_rows, first.v_mix) == (40.0, 8, True)
    assert (third.bias_max, third.window) == (90.0, 120)
    assert (latent.heads, latent.dim, latent.rot_dim, latent.vdim, latent.kv_rank, latent.window) == (3, 16, 8, 12, 24, 50)
    assert (latent.rot_base, latent.rot_dims) == (1000.0, 8)
    assert latent.rot_scaling.as_mapping() == {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0}
    assert config.layers[1].mlp is None and config.layers[0].mlp.ff == 96
    assert config.first_value_mixer() == 0
    other = parse_model_config(dt.CONFIG_B)
    assert other.residual_mult == 1.0 and other.first_value_mixer() is None
    assert other.layers[0].mixer.rot_scaling is None and other.layers[0].mixer.rot_dims == 4
    assert parse_model_config(dt.CONFIG_C).layers[2].mixer.window is None
    assert parse_model_config(dt.without_rows(dt.CONFIG_A)).layers[0].mixer.bias_rows is None


@pytest.mark.parametrize("damage,message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].update(factor=0), "factor"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][0]["mixer"].update(bias_max=-1), "bias_max"),
    (lambda c: c["layers"][0]["mixer"].update(v_mix=1), "v_mix"),
    (lambda c: c["layers"][2]["mixer"].update(vdim=16), "mix their values"),
    (lambda c: c.update(residual_mult=0), "residual_mult"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_the_reader_refuses(damage, message):
    config = json.loads(json.dumps(dt.CONFIG_A))
    damage(config)
    with pytest.raises(UnsupportedModelError, match=message):
        parse_model_config(config)


def test_the_tensors_a_model_expects():
    _, model = describe_model(dt.CONFIG_A)
    specs = {name: spec.shape for name, spec in model.tensor_specs().items()}
    assert specs["embed"] == (211, 64) and specs["final.norm"] == (64,) and "head" not in specs
    for norm in ("norm1", "norm1b", "norm2", "norm2b"):
        assert specs[f"l0.{norm}"] == (64,)
    assert "l1.norm2" not in specs and "l1.norm2b" not in specs and specs["l1.norm1b"] == (64,)
    assert (specs["l0.mix.q"], specs["l0.mix.k"], specs["l0.mix.v"], specs["l0.mix.o"]) == ((64, 64), (32, 64), (16, 64), (64, 32))
    assert (specs["l0.mix.q.norm"], specs["l0.mix.k.norm"], specs["l0.mix.rel"], specs["l0.mix.sink"]) == ((16,), (16,), (8, 4), (4,))
    # The first mixing layer's weight is in a file and is not read; the later ones' are scalars.
    assert "l0.mix.vmix" not in specs and "l0.mix.vmix" in model.ignorable_names()
    assert specs["l2.mix.vmix"] == () and specs["l3.mix.vmix"] == ()
    assert (specs["l0.mlp.up"], specs["l0.mlp.down"]) == ((96, 64), (64, 96))
    assert (specs["l1.mix.q"], specs["l1.mix.dkv"], specs["l1.mix.dkv.norm"], specs["l1.mix.g"]) == ((72, 64), (32, 64), (24,), (3, 64))
    assert (specs["l1.mix.uk"], specs["l1.mix.uv"], specs["l1.mix.o"]) == ((48, 24), (36, 24), (64, 36))
    # A file that does not name the rows of a bias table leaves them to the tensor.
    _, unnamed = describe_model(dt.without_rows(dt.CONFIG_A))
    assert unnamed.tensor_specs()["l0.mix.rel"].shape == (-1, 4)
    # Pages: keys and values of their own widths and a window each; one row per token for a latent layer.
    assert model.cache_needs() == [PagedKV(2, 16, 20, 8), PagedKV(1, 32, 50, 0), PagedKV(2, 24, 120, 8), PagedKV(2, 16, 9, 8)]
    _, open_ended = describe_model(dt.CONFIG_C)
    assert open_ended.cache_needs()[2:] == [PagedKV(1, 64, None, 0), PagedKV(4, 16, None, None)]


def test_the_layers_of_a_plan_say_who_leaves_values_and_who_mixes_them():
    from turboserve_amd.models.dovudra import dovudra_plan

    plan = dovudra_plan(parse_model_config(dt.CONFIG_A))
    mixes = [layer.block.params["mixer"].params.get("value_mix") for layer in plan.layers]
    assert mixes[0]["source"] and mixes[1] is None and not mixes[2]["source"] and not mixes[3]["source"]
    assert plan.ignorable == ("l0.mix.vmix",) and plan.head.params["tied_to"] == "embed"
    alone = dovudra_plan(parse_model_config(dt.CONFIG_B))
    assert alone.ignorable == () and all(layer.block.params["residual_scale"] == 1.0 for layer in alone.layers)


@pytest.mark.parametrize("rows,farthest", [(8, 40), (16, 120), (5, 30), (9, 400.0), (32, 64), (6, 7), (2, 1.5)])
def test_buckets_of_distances(rows, farthest):
    """Engine and plain implementation against the rule spelled out: exact rows below rows // 2, then
    the first distance of every later row from the closed form, the last row for everything beyond."""
    near = rows // 2
    for n in range(0, int(3 * farthest) + 5):
        got = distance_bucket(n, rows, farthest)
        assert got == plain.bucket(n, rows, farthest)
        if n < near:
            assert got == n
        else:
            assert near <= got <= rows - 1
            if got < rows - 1:  # n lies in [near r^(k / m), near r^((k + 1) / m)) with r = farthest / near, m = rows - near
                k, m, r = got - near, rows - near, farthest / near
                assert near * r ** (k / m) <= n * (1 + 1e-12) and n < near * r ** ((k + 1) / m) * (1 + 1e-12)
        if n >= farthest:
            assert got == rows - 1
    ordered = [distance_bucket(n, rows, farthest) for n in range(int(farthest) + 3)]
    assert ordered == sorted(ordered)


def test_a_bias_table_spread_out_by_distance():
    """The table the attention kernels read: row h, column min(n, L - 1) is the learned entry of n's bucket."""
    from turboserve_amd.parts.base import Runtime
    from turboserve_amd.parts.rope import DistanceBuckets

    runtime = Runtime(device=torch.device("cpu"), dtype=torch.float32, ops=None)
    table = torch.randn(16, 3)
    for reach in (None, 10, 500):
        part = DistanceBuckets("m", runtime, num_heads=3, max_distance=120, reach=reach)
        part.load({"m.rel": table})
        spread = part.score_bias_table(3)
        length = spread.shape[1]
        assert spread.shape[0] == 3 and (reach is None or length <= reach)
        for n in range(0, 400):
            if reach is not None and n >= reach:
                break  # a window never asks further
            assert torch.equal(spread[:, min(n, length - 1)], table[plain.bucket(n, 16, 120)]), (reach, n)
    with pytest.raises(ValueError, match="distances beyond"):
        DistanceBuckets("m", runtime, num_heads=3, max_distance=8).load({"m.rel": table})


@pytest.mark.parametrize("rot", [
    {"dims": 16, "base": 200000.0, "scaling": {"factor": 6.0, "original": 128, "fast": 24.0, "slow": 2.0}},
    {"dims": 8, "base": 1000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}},
    {"dims": 4, "base": 300.0, "scaling": {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 0.5}},
    {"dims": 12, "base": 10000.0},
])
def test_stretched_frequencies(rot):
    freq, magnitude = interpolated_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    want, want_magnitude = plain.frequencies(rot)
    assert torch.allclose(freq, want, rtol=1e-14, atol=0) and magnitude == pytest.approx(want_magnitude, rel=1e-15)
    plainly = torch.tensor([rot["base"] ** (-2 * i / rot["dims"]) for i in range(rot["dims"] // 2)], dtype=torch.float64)
    if "scaling" not in rot:
        assert torch.equal(freq, plainly) and magnitude == 1.0
    else:
        factor = rot["scaling"]["factor"]
        assert magnitude == pytest.approx(0.1 * math.log(factor) + 1.0)
        # Every frequency lies between the plain one and the plain one over the factor; the fastest keep theirs.
        assert bool(((freq <= plainly * (1 + 1e-15)) & (freq >= plainly / factor * (1 - 1e-15))).all())
        assert freq[0] == plainly[0]
    cos, sin = exact_rotary_tables(50, freq, magnitude)
    assert cos.dtype == torch.float32 and cos.shape == (50, rot["dims"] // 2)
    assert cos[37, 1].item() == pytest.approx(math.cos(37 * float(freq[1])) * magnitude, abs=1e-7)
    assert sin[49, -1].item() == pytest.approx(math.sin(49 * float(freq[-1])) * magnitude, abs=1e-7)


def test_the_plain_rotation_turns_neighbours_and_keeps_lengths():
    rot = {"dims": 4, "base": 50.0}
    x = torch.randn(6, 3, 8, dtype=torch.float64)
    y = plain.turn(x, rot)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0], x[0])
    pairs = lambda t: t[..., :4].reshape(6, 3, 2, 2).norm(dim=-1)  # noqa: E731
    assert torch.allclose(pairs(y), pairs(x), rtol=1e-12)
    # A dot product of two turned vectors depends on the distance only.
    a, b = torch.randn(1, 8, dtype=torch.float64), torch.randn(1, 8, dtype=torch.float64)
    ya, yb = plain.turn(a.expand(6, 8).clone(), rot), plain.turn(b.expand(6, 8).clone(), rot)
    assert float(ya[5] @ yb[3]) == pytest.approx(float(ya[2] @ yb[0]), rel=1e-10)


def test_the_plain_softmax_with_a_sink():
    scores, sink = torch.tensor([0.3, -1.0, 2.0], dtype=torch.float64), torch.tensor(0.7, dtype=torch.float64)
    weights = plain.sink_softmax_row(scores, sink)
    total = math.exp(0.7) + sum(math.exp(s) for s in (0.3, -1.0, 2.0))
    assert weights.tolist() == pytest.approx([math.exp(s) / total for s in (0.3, -1.0, 2.0)], rel=1e-12)
    assert float(weights.sum()) == pytest.approx(1 - math.exp(0.7) / total, rel=1e-12)


def test_the_plain_model_sees_what_the_design_says():
    """A window's edge, the mixed values and the sink all reach the plain logits: changing a token just
    outside every window leaves the last position alone, one just inside moves it."""
    config = json.loads(json.dumps(dt.CONFIG_A))
    tensors = dt.draw_tensors(config, 5, torch.float64, 0.2)
    tokens = torch.randint(0, config["vocab"], (40,), generator=torch.Generator().manual_seed(1)).tolist()
    base = plain.forward(config, tensors, tokens)[-1]
    # Four layers with windows 20, 50, 120, 9: position 39 reaches back through all of them.
    changed = list(tokens)
    changed[38] = (changed[38] + 1) % config["vocab"]
    assert float((plain.forward(config, tensors, changed)[-1] - base).abs().max()) > 1e-3
    narrow = json.loads(json.dumps(config))
    for entry in narrow["layers"]:
        entry["mixer"]["mask"] = {"size": 3}
    base = plain.forward(narrow, tensors, tokens)[-1]
    # Windows of three over four layers: position 39 sees back to 39 - 4 * 2 = 31 and no further.
    changed = list(tokens)
    changed[30] = (changed[30] + 1) % config["vocab"]
    assert float((plain.forward(narrow, tensors, changed)[-1] - base).abs().max()) == 0.0
    changed = list(tokens)
    changed[31] = (changed[31] + 1) % config["vocab"]
    assert float((plain.forward(narrow, tensors, changed)[-1] - base).abs().max()) > 0.0
    without = dict(tensors)
    for name in tensors:
        if name.endswith(".sink"):
            without[name] = tensors[name] - 30.0
    assert float((plain.forward(config, without, tokens)[-1] - plain.forward(config, tensors, tokens)[-1]).abs().max()) > 1e-3
