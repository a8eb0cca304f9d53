"""Legavik without a GPU: the configuration reader and its refusals, the tensors a model expects, the
cache each layer asks for (pages that keep a request's first keys, state beside pages), and the plain
implementation's own rules against direct formulas."""

from __future__ import annotations

import json
import math

import numpy as np
import pytest
import torch

import legavik_tiny as lt
from plain import legavik_plain as plain
from turboserve_amd.cache.layout import CacheLayout
from turboserve_amd.cache.manager import PAD_PAGE, CacheManager
from turboserve_amd.config.legavik_config import LegavikConfig
from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.registry import parse_model_config
from turboserve_amd.engine.batch import StepEntry, StepLayout, StepLimits, check_packed, pack_step
from turboserve_amd.parts.base import FixedState, PagedKV
from turboserve_amd.weights.random_init import describe_model


def test_the_reader_takes_every_size_from_the_file():
    config = parse_model_config(lt.CONFIG_A)
    assert isinstance(config, LegavikConfig)
    assert (config.vocab_size, config.hidden_size, config.norm_eps, config.logit_softcap) == (211, 64, 1e-5, 12.0)
    assert [layer.type for layer in config.layers] == ["parallel", "attention", "parallel", "attention"]
    pair, keyed = config.layers[0].mixer, config.layers[1].mixer
    assert (pair.left.heads, pair.left.kv_heads, pair.left.dim, pair.left.vdim, pair.left.taps, pair.left.scale) == (4, 2, 16, 24, 3, 0.3)
    assert (pair.left.temp_coef, pair.left.temp_every, pair.left_scale, pair.right_scale) == (0.4, 8, 0.7, 1.2)
    assert (pair.right.heads, pair.right.kv_heads, pair.right.dim, pair.right.vdim, pair.right.taps) == (4, 2, 16, 8, 4)
    assert (pair.right.decay_rank, pair.right.gate_rank) == (6, 5)
    assert (keyed.heads, keyed.kv_heads, keyed.dim, keyed.scale, keyed.window, keyed.keep_first) == (4, 2, 16, 0.5, 20, 5)
    assert (keyed.rot_base, keyed.rot_dims) == (1000.0, 8)
    assert keyed.rot_scaling.as_mapping() == {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0}
    first = config.layers[0].mlp
    assert (first.ff, first.experts, first.top, first.groups, first.keep) == (24, 6, 2, 3, 2)
    assert config.layers[1].mlp is None and (config.layers[2].mlp.groups, config.layers[2].mlp.keep) == (1, 1)
    # What a file leaves out does not exist: cap, mask, kept tokens, rotation, temperature, ranks.
    other = parse_model_config(lt.without_ranks(lt.CONFIG_B))
    assert other.logit_softcap is None
    assert (other.layers[3].mixer.window, other.layers[3].mixer.keep_first, other.layers[3].mixer.rot_base) == (None, 0, None)
    assert (other.layers[2].mixer.window, other.layers[2].mixer.keep_first) == (7, 0)
    assert other.layers[1].mixer.left.temp_coef is None and other.layers[1].mixer.right.decay_rank is None
    assert other.layers[4].mixer.left_scale == -0.8


@pytest.mark.parametrize("damage,message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=8), "values are the keys"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=3), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["rot"]["scaling"].update(factor=0), "factor"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "size"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(keep_first=-1), "keep_first"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "cannot be taken"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "cannot be taken"),
    (lambda c: c["layers"][0]["mixer"]["left"]["q_temp"].update(every=0), "every"),
    (lambda c: c["layers"][0]["mixer"]["right"].pop("conv"), "conv"),
    (lambda c: c["layers"][0]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c.update(logit_softcap=0), "logit_softcap"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_the_reader_refuses(damage, message):
    config = json.loads(json.dumps(lt.CONFIG_A))
    damage(config)
    with pytest.raises(UnsupportedModelError, match=message):
        parse_model_config(config)


def test_the_tensors_a_model_expects():
    _, model = describe_model(lt.CONFIG_A)
    specs = {name: spec.shape for name, spec in model.tensor_specs().items()}
    assert specs["embed"] == (211, 64) and specs["head"] == (211, 64)
    for norm in ("l0.norm1", "l0.norm2", "l1.norm1", "final.norm"):
        assert (specs[norm], specs[norm + ".b"], specs[norm + ".alpha"]) == ((64,), (64,), ())
    assert "l1.norm2" not in specs and not any(name.startswith("l1.mlp") for name in specs)
    # The attention whose values are its keys has no value matrix; its gate has a row per head.
    assert (specs["l1.mix.q"], specs["l1.mix.k"], specs["l1.mix.g"], specs["l1.mix.o"]) == ((64, 64), (32, 64), (4, 64), (64, 64))
    assert "l1.mix.v" not in specs and "l1.mix.q.norm" not in specs
    left = "l0.mix.left."
    assert (specs[left + "q"], specs[left + "k"], specs[left + "v"], specs[left + "o"]) == ((64, 64), (32, 64), (48, 64), (64, 96))
    assert (specs[left + "q.b"], specs[left + "k.b"], specs[left + "v.b"], specs[left + "o.b"]) == ((64,), (32,), (48,), (64,))
    assert (specs[left + "q.conv"], specs[left + "k.conv"], specs[left + "v.conv"]) == ((64, 3), (32, 3), (48, 3))
    assert (specs[left + "q.norm"], specs[left + "k.norm"], specs[left + "g"]) == ((16,), (16,), (4, 64))
    right = "l0.mix.right."
    assert (specs[right + "q"], specs[right + "k"], specs[right + "v"], specs[right + "o"]) == ((32, 64), (32, 64), (32, 64), (64, 32))
    assert (specs[right + "q.conv"], specs[right + "v.conv"], specs[right + "b"], specs[right + "A_log"]) == ((32, 4), (32, 4), (4, 64), (4,))
    assert (specs[right + "a1"], specs[right + "a2"], specs[right + "dt_bias"]) == ((6, 64), (64, 6), (64,))
    assert (specs[right + "g1"], specs[right + "g2"], specs[right + "norm"]) == ((5, 64), (32, 5), (8,))
    assert (specs["l0.mlp.router"], specs["l0.mlp.e5.gate"], specs["l0.mlp.e5.up"], specs["l0.mlp.e0.down"]) == ((6, 64), (24, 64), (24, 64), (64, 24))
    # A file that does not name the low-rank widths leaves them to the tensors.
    _, unnamed = describe_model(lt.without_ranks(lt.CONFIG_A))
    assert unnamed.tensor_specs()[right + "a1"].shape == (-1, 64) and unnamed.tensor_specs()[right + "g2"].shape == (32, -1)


def test_what_each_layer_asks_of_the_cache():
    _, model = describe_model(lt.CONFIG_A)
    needs = model.cache_needs()
    # A parallel layer: the left side's pages and its convolution's last rows, the right side's state and
    # its convolution's last rows, in that order.
    assert needs[0] == (PagedKV(2, 16, None, 24), FixedState((2, 64 + 32 + 48)), FixedState((4, 16, 8)), FixedState((3, 32 + 32 + 32)))
    assert needs[1] == PagedKV(2, 16, 20, None, None, 5)
    assert needs[3] == PagedKV(1, 24, 120, None, None, 17)
    layout = CacheLayout.from_model(model)
    assert layout.kept() == [group.keep_first for group in layout.groups] and sorted(layout.kept()) == [0, 0, 5, 17]
    assert len(layout.state_entries) == 6
    # One tap: nothing to carry, and a state of one row that is never read.
    _, other = describe_model(lt.CONFIG_B)
    assert other.cache_needs()[1][1] == FixedState((1, 60 + 60 + 60)) and other.cache_needs()[4][3] == FixedState((1, 20 + 20 + 12))


def test_pages_of_the_kept_first_keys_stay_while_the_window_moves_on():
    """A window of 6 that keeps the first 5 keys, pages of 4: the two pages that hold keys 0..4 are never
    given back; those between them and the window are."""
    manager = CacheManager([6], [8], 4, 2, kept=[5])
    manager.admit("a")
    manager.append("a", 14)  # positions 0..13
    assert PAD_PAGE not in manager.get("a").tables[0]
    for _ in range(30):
        manager.append("a", 1)
        manager.check_invariants()
    table = manager.get("a").tables[0]
    assert len(table) == 11 and table[0] != PAD_PAGE and table[1] != PAD_PAGE
    assert table[2:9] == [PAD_PAGE] * 7 and PAD_PAGE not in table[9:]
    assert manager.pools[0].num_in_use == 4
    assert manager.peak_pages(0, 1000, 1) == 3 + 2 and manager.peak_pages(0, 7, 64) == 2
    manager.free("a")
    assert manager.pools[0].num_in_use == 0
    # Without kept keys the same run holds the window's pages alone.
    plain_window = CacheManager([6], [8], 4, 2)
    plain_window.admit("a")
    plain_window.append("a", 14)
    for _ in range(30):
        plain_window.append("a", 1)
    assert plain_window.pools[0].num_in_use == 2


def test_a_step_is_refused_when_a_page_of_kept_keys_is_missing():
    limits = StepLimits(num_pages=[16], windows=[6], kept=[5], vocab_size=50, num_state_slots=2)
    tables = [[3, 4, PAD_PAGE, PAD_PAGE, 7, 8]]
    entry = StepEntry("a", [1], 22, tables, [[8 * 4 + 2]])
    layout = StepLayout.make(1, 1, 0, [6])
    data = np.zeros(layout.total, dtype=np.int32)
    pack_step(data, layout, [entry], [])
    check_packed(data, layout, [entry], 4, limits)  # keys 0..4 and 17..22 are there
    gone = StepEntry("a", [1], 22, [[3, PAD_PAGE, PAD_PAGE, PAD_PAGE, 7, 8]], [[8 * 4 + 2]])
    pack_step(data, layout, [gone], [])
    with pytest.raises(ValueError, match="no page at index 1"):
        check_packed(data, layout, [gone], 4, limits)
    check_packed(data, layout, [gone], 4, StepLimits(num_pages=[16], windows=[6], kept=[4], vocab_size=50, num_state_slots=2))


def test_the_plain_convolution_is_causal_and_ends_on_the_current_token():
    u = torch.arange(1.0, 11.0).reshape(5, 2)
    taps = torch.tensor([[100.0, 10.0, 1.0], [0.0, 0.0, 2.0]])
    y = plain.short_conv(u, taps)
    assert y[:, 1].tolist() == (2 * u[:, 1]).tolist()
    assert y[:, 0].tolist() == [1.0, 13.0, 135.0, 357.0, 579.0]


def test_the_plain_rotation_turns_halves_of_the_first_elements_only():
    rot = {"base": 100.0, "dims": 4, "scaling": {"factor": 8.0, "original": 16, "fast": 2.0, "slow": 0.5}}
    f, magnitude = plain.frequencies(rot)
    assert magnitude == pytest.approx(0.1 * math.log(8.0) + 1.0)
    x = torch.randn(6, 2, 7, dtype=torch.float64)
    y = plain.turn_halves(x, rot)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0, :, 0], x[0, :, 0] * magnitude)
    for p in range(6):
        for i in range(2):
            a = p * float(f[i])
            want = x[p, :, i] * math.cos(a) * magnitude - x[p, :, i + 2] * math.sin(a) * magnitude
            assert torch.allclose(y[p, :, i], want)
    lengths = (y[..., :4] ** 2).sum(-1) / (x[..., :4] ** 2).sum(-1)
    assert torch.allclose(lengths, torch.full_like(lengths, magnitude ** 2))
    # The engine's tables hold the same frequencies.
    from turboserve_amd.parts.rope import interpolated_frequencies

    mine, factor = interpolated_frequencies(4, 100.0, rot["scaling"])
    assert torch.allclose(mine, f) and factor == pytest.approx(magnitude)


def test_the_plain_window_keeps_the_first_tokens():
    mask = {"size": 4, "keep_first": 2}
    assert [j for j in range(12) if plain.sees(9, j, mask)] == [0, 1, 6, 7, 8, 9]
    assert [j for j in range(12) if plain.sees(9, j, {"size": 4})] == [6, 7, 8, 9]
    assert [j for j in range(12) if plain.sees(3, j, mask)] == [0, 1, 2, 3]
    assert [j for j in range(5) if plain.sees(3, j, None)] == [0, 1, 2, 3]


def test_the_plain_router_takes_the_best_of_the_best_groups():
    scores = torch.tensor([0.05, 0.30, 0.20, 0.21, 0.02, 0.22])
    rule = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}
    # Groups (0, 1), (2, 3), (4, 5) are marked 0.30, 0.21, 0.22: the middle one is closed.
    assert plain.choose(scores, rule) == [1, 5]
    assert plain.choose(scores, {"experts": 6, "top": 3}) == [1, 5, 3]
    assert plain.choose(torch.tensor([0.25, 0.25, 0.25, 0.25]), {"experts": 4, "top": 2, "groups": {"count": 2, "keep": 1}}) == [0, 1]


def test_the_plain_delta_rule_reads_its_own_write():
    """One head, one token: the state starts at zero, so the read-out is ``beta v (k . q)``, normed and gated."""
    tensors = {"p.q": torch.eye(4), "p.k": torch.eye(4), "p.v": torch.eye(4)[:2], "p.q.conv": torch.ones(4, 1), "p.k.conv": torch.ones(4, 1),
               "p.v.conv": torch.ones(2, 1), "p.b": torch.zeros(1, 4), "p.a1": torch.zeros(1, 4), "p.a2": torch.zeros(4, 1),
               "p.dt_bias": torch.zeros(4), "p.A_log": torch.zeros(1), "p.g1": torch.zeros(1, 4), "p.g2": torch.zeros(2, 1),
               "p.norm": torch.ones(2), "p.o": torch.eye(2)}
    h = torch.tensor([[1.0, 2.0, -1.0, 0.5]])
    out = plain.delta_rule("p", {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 2}, tensors, h, 0.0)
    v = torch.nn.functional.silu(h[0, :2])
    want = v / torch.sqrt((v * v).mean()) * 0.5  # beta, k . q and the norm's scale cancel but for the sign; the gate is a half
    assert torch.allclose(out[0], want, atol=1e-6)


def test_the_plain_model_sees_what_the_design_says():
    """A token outside every window and not among the kept ones cannot reach the last position of a model
    of attention layers; one inside can; the parallel layers carry everything."""
    keyed_only = {"architecture": "Legavik", "vocab": 30, "width": 16, "norm": {"eps": 1e-5},
                  "layers": [lt.layer(lt.keyed(2, 1, 8, window=4, keep=2, rot=4), lt.moe(8, 2, 1))]}
    tensors = lt.draw_tensors(keyed_only, 1, torch.float64, 0.3)
    tokens = [3, 4, 5, 6, 7, 8, 9, 10, 11, 12]
    base = plain.forward(keyed_only, tensors, tokens)[-1]
    for place, reaches in ((0, True), (1, True), (2, False), (5, False), (6, True), (8, True)):
        other = list(tokens)
        other[place] = 20
        moved = float((plain.forward(keyed_only, tensors, other)[-1] - base).abs().max())
        assert (moved > 1e-9) == reaches, (place, moved)
    with_pair = json.loads(json.dumps(keyed_only))
    with_pair["layers"].append(lt.layer(lt.parallel(lt.left(1, 1, 4, 4, 2), lt.right(1, 1, 4, 4, 2, 2, 2), 1.0, 1.0), None))
    tensors = lt.draw_tensors(with_pair, 1, torch.float64, 0.3)
    base = plain.forward(with_pair, tensors, tokens)[-1]
    other = list(tokens)
    other[3] = 20
    assert float((plain.forward(with_pair, tensors, other)[-1] - base).abs().max()) > 1e-9
    capped = dict(keyed_only, logit_softcap=0.5)
    assert float(plain.forward(capped, lt.draw_tensors(capped, 1, torch.float64, 0.3), tokens).abs().max()) < 0.5
