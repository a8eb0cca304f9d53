"""Dovudra on the GPU against the plain implementation (``tests/plain/dovudra_plain.py``): each
mechanism alone (its kernel, and a one-layer model of it), whole prompts, every way of cutting
requests into steps on so few pages that they are used again, keys at the edges of windows and
pages, at a sequence's first positions and far back, and greedy generation through the engine's own
entry point."""

from __future__ import annotations

import json
import random
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import dovudra_tiny as dt
import trace_helpers as th
from plain import dovudra_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROOT = Path(__file__).resolve().parent.parent
#: 32-bit engine against the 32-bit plain implementation, relative to a position's largest logit.
RTOL_F32 = 2e-4
#: bfloat16 engine (weights stored in bfloat16) against the plain implementation in 32-bit on the
#: same weights, for 19 positions in 20; the rest may be off by twice the bound.
RTOL_BF16 = 4e-2
BF16_OUTLIERS = 2.0


@pytest.fixture(scope="module")
def ops():
    from turboserve_amd.kernels.ops import Ops

    return Ops(DEV)


def excess(got: torch.Tensor, want: torch.Tensor, dtype: str) -> float:
    rtol = RTOL_F32 if dtype == "float32" else RTOL_BF16
    bound = rtol * want.abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    rows = ((got - want).abs() / bound).amax(dim=-1)
    if dtype == "float32":
        return float(rows.max())
    ordered = rows.sort().values
    return max(float(ordered[int(0.95 * (len(ordered) - 1))]), float(ordered[-1]) / BF16_OUTLIERS)


def tokens_of(vocab: int, length: int, seed: int) -> list[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=g).tolist()


def stored_as(dtype: str) -> torch.dtype:
    return torch.float32 if dtype == "float32" else torch.bfloat16


def run_trace(folder, dtype: str, page: int, steps: list[dict], max_tokens: int | None = None, max_live: int = 4):
    from turboserve_amd.engine.replay import TraceReplayer

    replayer = TraceReplayer(folder, dtype=dtype, max_tokens=max_tokens or th.peak_tokens(steps, rounding=page),
                             page_size=page, max_live=max_live)
    outputs = {}
    for record in steps:
        logits = replayer.run_step(record)
        if logits.shape[0]:
            outputs[record["step"]] = logits.float().cpu()
    replayer.manager.check_invariants()
    assert all(pool.num_in_use == 0 for pool in replayer.manager.pools), "pages were not given back"
    return outputs


# ---------------------------------------------------------------------------------------------
# mechanisms alone: kernels
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind", ["relu_squared", "relu", "silu", "gelu_tanh"])
@pytest.mark.parametrize("inter", [5, 44, 200])
def test_activations_without_a_gate(ops, dtype, kind, inter):
    g = torch.Generator().manual_seed(inter)
    z = (2 * torch.randn(11, inter, generator=g)).to(dtype)
    z[0, 0], z[0, 1] = -60.0, 60.0
    x = z.float()
    want = {"relu_squared": torch.relu(x) ** 2, "relu": torch.relu(x), "silu": x * torch.sigmoid(x),
            "gelu_tanh": 0.5 * x * (1 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))}[kind]
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(ops.activate(z.to(DEV), kind).float().cpu(), want, **tol)
    # From the 32-bit partial sums of a product that was shared out, rounded once.
    parts = torch.randn(3, 11, inter, generator=g)
    parts[2] = x - parts[0] - parts[1]
    got = ops.activate(parts.to(DEV), kind, dtype).float().cpu()
    exact = parts.sum(0)
    want = {"relu_squared": torch.relu(exact) ** 2, "relu": torch.relu(exact), "silu": exact * torch.sigmoid(exact),
            "gelu_tanh": 0.5 * exact * (1 + torch.tanh(0.7978845608028654 * (exact + 0.044715 * exact ** 3)))}[kind]
    torch.testing.assert_close(got, want.to(dtype).float(), **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim", [(3, 12), (1, 20), (8, 64), (5, 7)])
def test_a_gate_per_head(ops, dtype, heads, vdim):
    g = torch.Generator().manual_seed(heads * vdim)
    tokens, before = 9, 13
    values = torch.randn(tokens, heads * vdim, generator=g)
    proj = (2 * torch.randn(tokens, before + heads + 2, generator=g)).to(dtype)
    want = (values.view(tokens, heads, vdim) * torch.sigmoid(proj.float()[:, before:before + heads, None])).reshape(tokens, -1)
    got = ops.head_gate(values.to(DEV), proj.to(DEV), before, heads, dtype).float().cpu()
    tol = dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got, want, **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,splits", [(52, 0), (64, 3), (320, 0), (1000, 2)])
def test_a_norm_behind_a_part_rides_with_the_next_norm(ops, dtype, hidden, splits):
    """``x += m norm_b(pending)``, then ``norm(x)``: both in one pass, the sum and both norms in 32-bit."""
    g = torch.Generator().manual_seed(hidden)
    tokens, eps_behind, eps, mult = 7, 1e-5, 1e-6, 0.3
    x = torch.randn(tokens, hidden, generator=g)
    behind = (1 + 0.3 * torch.randn(hidden, generator=g)).to(dtype)
    gain = (1 + 0.3 * torch.randn(hidden, generator=g)).to(dtype)
    if splits:
        pending = torch.randn(splits, tokens, hidden, generator=g)
        part = pending.sum(0)
    else:
        pending = (3 * torch.randn(tokens, hidden, generator=g)).to(dtype)
        part = pending.float()
    total = x + mult * plain.rms(part, behind.float(), eps_behind)
    want = plain.rms(total, gain.float(), eps)
    stream = x.clone().to(DEV)
    got = ops.add_rmsnorm(stream, pending.to(DEV), gain.to(DEV), eps, one_rounding=True,
                          pending_norm=(behind.to(DEV), eps_behind, mult)).float().cpu()
    torch.testing.assert_close(stream.cpu(), total, rtol=1e-5, atol=1e-5)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(got, want, **tol)
    # Only some rows (the head's): the stream is left alone.
    rows = torch.tensor([5, 0], dtype=torch.int32, device=DEV)
    stream = x.clone().to(DEV)
    got = ops.add_rmsnorm(stream, pending.to(DEV), gain.to(DEV), eps, rows, one_rounding=True,
                          pending_norm=(behind.to(DEV), eps_behind, mult)).float().cpu()
    torch.testing.assert_close(stream.cpu(), x, rtol=0, atol=0)
    torch.testing.assert_close(got, want[[5, 0]], **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,page", [(4, 2, 16, 8, 16), (5, 5, 12, 12, 8), (1, 1, 20, 36, 8), (8, 2, 64, 64, 16)])
def test_the_store_norms_heads_and_keeps_or_blends_values(ops, dtype, heads, kv_heads, dim, vdim, page):
    g = torch.Generator().manual_seed(dim * vdim)
    tokens, eps, weight = 21, 1e-5, 0.4
    width = (heads + kv_heads) * dim + kv_heads * vdim
    proj = torch.randn(tokens, width, generator=g).to(dtype)
    q_gain, k_gain = ((1 + 0.3 * torch.randn(dim, generator=g)).to(dtype) for _ in range(2))
    pages = 5
    slots = torch.randperm(pages * page, generator=g)[:tokens].to(torch.int32)
    positions = torch.arange(tokens, dtype=torch.int32)
    x = proj.float()
    want_q = plain.rms(x[:, : heads * dim].view(tokens, heads, dim), q_gain.float(), eps)
    want_k = plain.rms(x[:, heads * dim:(heads + kv_heads) * dim].view(tokens, kv_heads, dim), k_gain.float(), eps)
    want_v = x[:, (heads + kv_heads) * dim:].view(tokens, kv_heads, vdim)
    tol = dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    kept = torch.full((tokens, kv_heads * vdim), float("nan"), device=DEV)
    other = torch.randn(tokens, kv_heads * vdim, generator=g)
    for more, values in ((dict(keep_values=kept), want_v),
                         (dict(blend_values=(other.to(DEV), weight)), (1 - weight) * want_v + weight * other.view(tokens, kv_heads, vdim))):
        k_pages = torch.zeros(pages, kv_heads, page, dim, dtype=dtype, device=DEV)
        v_pages = torch.zeros(pages, kv_heads, vdim, page, dtype=dtype, device=DEV)
        q, stride = ops.head_norm_store(proj.clone().to(DEV), k_pages, v_pages, q_gain.to(DEV), k_gain.to(DEV), eps,
                                        positions.to(DEV), slots.to(DEV), heads, kv_heads, dim, vdim, page, dtype, **more)
        got_q = q.view(tokens, -1)[:, : heads * dim].float().cpu().view(tokens, heads, dim)
        torch.testing.assert_close(got_q, want_q, **tol)
        block, offset = (slots // page).long(), (slots % page).long()
        torch.testing.assert_close(k_pages.float().cpu()[block, :, offset], want_k, **tol)
        torch.testing.assert_close(v_pages.float().cpu()[block, :, :, offset], values, **tol)
    torch.testing.assert_close(kept.cpu(), want_v.reshape(tokens, -1), rtol=0, atol=0)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rot_dim,turned,rank,gates", [(3, 16, 8, 8, 24, 3), (1, 12, 12, 4, 10, 0), (2, 6, 4, 4, 18, 2), (8, 64, 32, 32, 96, 8)])
def test_the_latent_store_turns_neighbours(ops, dtype, heads, dim, rot_dim, turned, rank, gates):
    from turboserve_amd.parts.rope import exact_rotary_tables, interpolated_frequencies

    g = torch.Generator().manual_seed(rank)
    tokens, eps, page = 19, 1e-6, 8
    rot = {"dims": turned, "base": 700.0, "scaling": {"factor": 3.0, "original": 32, "fast": 6.0, "slow": 1.5}}
    freq, magnitude = interpolated_frequencies(turned, rot["base"], rot["scaling"])
    positions = torch.randperm(90, generator=g)[:tokens].to(torch.int32)
    cos, sin = exact_rotary_tables(128, freq, magnitude)
    width = heads * (dim + rot_dim) + rank + rot_dim + gates
    proj = torch.randn(tokens, width, generator=g).to(dtype)
    gain = (1 + 0.3 * torch.randn(rank, generator=g)).to(dtype)
    slots = torch.randperm(4 * page, generator=g)[:tokens].to(torch.int32)
    k_pages = torch.zeros(4, 1, page, rank + rot_dim, dtype=dtype, device=DEV)
    q_plain, q_wide = ops.latent_store(proj.to(DEV), k_pages, gain.to(DEV), eps, cos.to(DEV), sin.to(DEV), positions.to(DEV),
                                       slots.to(DEV), heads, dim, rot_dim, rank, page, 127, dtype, neighbours=True, tail=gates)
    x = proj.float()
    q = x[:, : heads * (dim + rot_dim)].view(tokens, heads, dim + rot_dim)
    down = x[:, heads * (dim + rot_dim):heads * (dim + rot_dim) + rank + rot_dim]

    def turned_at(rows: torch.Tensor) -> torch.Tensor:  # the plain rule walks positions 0, 1, ...: place each row at its own
        out = torch.empty_like(rows)
        for t in range(tokens):
            padded = torch.zeros(int(positions[t]) + 1, *rows.shape[1:])
            padded[-1] = rows[t]
            out[t] = plain.turn(padded, rot)[-1]
        return out

    tol = dict(rtol=1e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(q_plain.float().cpu().view(tokens, heads, dim), q[..., :dim], **tol)
    torch.testing.assert_close(q_wide.float().cpu()[..., rank:], turned_at(q[..., dim:]), **tol)
    block, offset = (slots // page).long(), (slots % page).long()
    stored = k_pages.float().cpu()[block, 0, offset]
    torch.testing.assert_close(stored[:, :rank], plain.rms(down[:, :rank], gain.float(), eps), **tol)
    torch.testing.assert_close(stored[:, rank:], turned_at(down[:, rank:]), **tol)


def plain_attention_rows(q, k, v, positions, contexts_of, rel, sink, farthest, scale, window):
    """Row by row from the rules: ``q [T, H, D]`` of tokens at ``positions`` of requests whose keys and
    values are ``k[r] [n, G, D]``, ``v[r] [n, G, Dv]``."""
    tokens, heads, _ = q.shape
    out = torch.zeros(tokens, heads, v[0].shape[-1], dtype=torch.float64)
    for t in range(tokens):
        r, i = contexts_of[t], int(positions[t])
        lo = 0 if window is None else max(0, i - window + 1)
        for h in range(heads):
            kv = h // (heads // k[r].shape[1])
            scores = (k[r][lo:i + 1, kv].double() @ q[t, h].double()) * scale
            if rel is not None:
                scores = scores + torch.tensor([float(rel[plain.bucket(i - j, rel.shape[0], farthest), h]) for j in range(lo, i + 1)],
                                               dtype=torch.float64)
            if sink is None:
                weights = torch.softmax(scores, dim=0)
            else:
                weights = plain.sink_softmax_row(scores, sink[h].double())
            out[t, h] = weights @ v[r][lo:i + 1, kv].double()
    return out.reshape(tokens, -1).float()


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,page,window,rows,farthest", [
    (4, 2, 16, 8, 16, 20, 8, 40), (2, 2, 24, 8, 8, 120, 12, 90.0), (5, 5, 12, 12, 8, 7, 5, 30), (1, 1, 20, 36, 8, 33, 9, 400),
    (8, 4, 16, 16, 32, None, 32, 128), (8, 2, 64, 64, 16, 50, 16, 100), (6, 2, 32, 48, 32, 100, 16, 64)])
def test_scores_with_a_bias_by_distance_a_window_and_a_learned_sink(ops, heads, kv_heads, dim, vdim, page, window, rows, farthest):
    """The attention kernels alone against the rules: 32-bit (one wavefront a row) against plain loops,
    then the matrix-core kernel in bfloat16 against the first on the same pages.  Portions that start
    in the middle of a request beside single tokens; sinks large enough to take much of the weight."""
    from turboserve_amd.parts.base import Runtime
    from turboserve_amd.parts.rope import DistanceBuckets

    g = torch.Generator().manual_seed(heads * 100 + dim)
    query_lens = [70, 9, 2, 1, 1, 1]
    contexts = [160, 9, 301, 210, 1, 65]
    pages_of = [-(-c // page) for c in contexts]
    total_pages = sum(pages_of) + 3
    order = torch.randperm(total_pages, generator=g).tolist()
    table = torch.zeros((len(contexts), max(pages_of)), dtype=torch.int32)
    keys = [torch.randn(c, kv_heads, dim, generator=g) for c in contexts]
    values = [torch.randn(c, kv_heads, vdim, generator=g) for c in contexts]
    k_pages = torch.zeros(total_pages, kv_heads, page, dim)
    v_pages = torch.zeros(total_pages, kv_heads, vdim, page)
    for s, n in enumerate(pages_of):
        table[s, :n] = torch.tensor([order.pop() for _ in range(n)])
        for j in range(contexts[s]):
            k_pages[table[s, j // page], :, j % page] = keys[s][j]
            v_pages[table[s, j // page], :, :, j % page] = values[s][j]
    tokens = sum(query_lens)
    q = 0.7 * torch.randn(tokens, heads * dim, generator=g)
    rel = 1.5 * torch.randn(rows, heads, generator=g)
    sink = 2.0 + torch.randn(heads, generator=g)
    scale = 0.3
    token_seq = torch.repeat_interleave(torch.arange(len(query_lens)), torch.tensor(query_lens)).to(torch.int32)
    positions = torch.cat([torch.arange(c - n, c) for c, n in zip(contexts, query_lens)]).to(torch.int32)
    part = DistanceBuckets("m", Runtime(device=torch.device(DEV), dtype=torch.float32, ops=None), num_heads=heads,
                           max_distance=farthest, reach=window)
    part.load({"m.rel": rel.to(DEV)})
    bias = part.score_bias_table(heads)
    dev = lambda t: t.to(DEV)  # noqa: E731
    got = ops.paged_attention_generic(dev(q), heads * dim, dev(k_pages), dev(v_pages), dev(table), dev(token_seq), dev(positions),
                                      heads, scale, window, sinks=1.0, sink_scores=dev(sink), distance_bias=bias).float().cpu()
    want = plain_attention_rows(q.view(tokens, heads, dim), keys, values, positions, token_seq.tolist(), rel, sink, farthest, scale, window)
    torch.testing.assert_close(got, want, rtol=2e-4, atol=2e-4)
    no_sink = plain_attention_rows(q.view(tokens, heads, dim), keys, values, positions, token_seq.tolist(), rel, None, farthest, scale, window)
    assert float((no_sink - want).abs().max()) > 0.1, "the sinks take too little for the test to see them"
    if not ops.tiled_attention_supported(torch.bfloat16, dim, vdim, page, heads * dim):
        return
    half = lambda t: t.to(torch.bfloat16).to(DEV)  # noqa: E731
    base = ops.paged_attention_generic(half(q), heads * dim, half(k_pages), half(v_pages), dev(table), dev(token_seq), dev(positions),
                                       heads, scale, window, sinks=1.0, sink_scores=dev(sink), distance_bias=bias).float().cpu()
    starts = torch.tensor([0, *torch.tensor(query_lens).cumsum(0).tolist()], dtype=torch.int32)
    tiles = torch.tensor(ops.attention_tile_list(query_lens[:3]), dtype=torch.int32, device=DEV)
    tiled = ops.attention_tiles(half(q), heads * dim, half(k_pages), half(v_pages), dev(table), dev(starts),
                                torch.tensor(contexts, dtype=torch.int32, device=DEV), tokens=tokens, heads=heads, scale=scale,
                                prefill_tiles=tiles, num_prefill_seqs=3, num_decode_seqs=3, max_decode_context=320, window=window,
                                sinks=1.0, sink_scores=dev(sink), distance_bias=bias).float().cpu()
    assert torch.isfinite(tiled).all()
    torch.testing.assert_close(tiled, base, rtol=2e-2, atol=2e-2)


# ---------------------------------------------------------------------------------------------
# mechanisms alone: one-layer models
# ---------------------------------------------------------------------------------------------

ALONE = {
    "biased": dt.layer(dt.attention(4, 2, 16, 24, 13, 8, 30, scale=0.4), None),
    "biased_one_head_no_window": dt.layer(dt.attention(1, 1, 20, 6, None, 6, 50, scale=0.5), None),
    "biased_window_of_one": dt.layer(dt.attention(3, 3, 8, 8, 1, 4, 9, scale=0.5), None),
    "biased_matrix_cores": dt.layer(dt.attention(4, 1, 32, 32, 40, 16, 60), None),
    "latent": dt.layer(dt.latent(3, 16, 8, 12, 24, 21, base=100.0, stretch=(4.0, 32, 8.0, 1.0)), None),
    "latent_part_turned_no_window": dt.layer(dt.latent(2, 8, 12, 20, 9, None, turned=6, base=7.0, scale=0.6), None),
    "latent_matrix_cores": dt.layer(dt.latent(4, 32, 16, 24, 48, 37, base=5000.0, stretch=(2.0, 16, 4.0, 1.0)), None),
    # A cached row (latent and rotated part) longer than any matrix-core attention kernel takes.
    "latent_long_rows": dt.layer(dt.latent(2, 16, 16, 8, 584, 30, base=1000.0), None),
    "dense": dt.layer(dt.latent(1, 8, 4, 8, 8, 4), dt.dense(44)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(ALONE))
@pytest.mark.parametrize("mult", [None, 0.3])
def test_one_layer_models(tmp_path, which, dtype, mult):
    """A model of one layer: whole, token by token from the start, and in portions, against the
    plain implementation."""
    config = {"architecture": "Dovudra", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "layers": [ALONE[which]]}
    if mult is not None:
        config["residual_mult"] = mult
    folder = dt.make_model_dir(tmp_path / "m", config, 31, stored_as(dtype), std=0.2 if dtype == "float32" else 0.1)
    requests = {"a": tokens_of(61, 75, 1), "b": tokens_of(61, 3, 2)}
    want = {rid: dt.plain_logits(folder, tokens) for rid, tokens in requests.items()}
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=74), th.portions(requests, (2, 5, 31, 3))):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps), requests)
        for rid in requests:
            assert excess(got[rid], want[rid], dtype) <= 1.0, (which, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_values_reach_later_layers(tmp_path, dtype):
    """Three mixing layers with a latent layer between: the first one's values go into the others',
    with weights large enough that leaving them out would show."""
    mixing = lambda window, rows: dt.layer(dt.attention(4, 2, 16, 12, window, rows, 50, scale=0.4, v_mix=True), dt.dense(40))  # noqa: E731
    config = {"architecture": "Dovudra", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
              "layers": [mixing(30, 8), dt.layer(dt.latent(2, 8, 4, 8, 12, 9), None), mixing(11, 6),
                         dt.layer(dt.attention(2, 1, 8, 8, 5, 4, 20), None), mixing(None, 10)]}
    tensors = dt.draw_tensors(config, 3, stored_as(dtype), 0.2 if dtype == "float32" else 0.1)
    tensors["l2.mix.vmix"] = torch.tensor(0.7, dtype=stored_as(dtype))
    tensors["l4.mix.vmix"] = torch.tensor(-0.5, dtype=stored_as(dtype))
    tensors["l0.mix.vmix"] = torch.tensor(0.9, dtype=stored_as(dtype))  # the source's own: in the file, never read
    folder = dt.make_model_dir(tmp_path / "m", config, 0, tensors=tensors)
    requests = {"a": tokens_of(61, 90, 5), "b": tokens_of(61, 2, 6), "c": tokens_of(61, 33, 7)}
    raw, loaded = dt.read_model_dir(folder)
    want = {rid: plain.forward(raw, loaded, tokens) for rid, tokens in requests.items()}
    unmixed = dict(loaded)
    unmixed["l2.mix.vmix"] = unmixed["l4.mix.vmix"] = torch.tensor(0.0)
    moved = (plain.forward(raw, unmixed, requests["a"]) - want["a"]).abs().max() / want["a"].abs().max()
    assert float(moved) > 0.1, f"the mixing does not matter enough ({float(moved):.3f})"
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=20), th.portions(requests, (7, 2, 30)),
                  th.mixed(requests, (7, 2, 19), max_live=3, decode_tail=6)):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps), requests)
        for rid in requests:
            assert excess(got[rid], want[rid], dtype) <= 1.0, rid


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windows_on_a_pool_smaller_than_the_request(tmp_path, dtype):
    """Layers that read only a window give the pages below it back while the request runs: 200 tokens
    go through a pool of 96, in portions and token by token, and every position is still right."""
    config = {"architecture": "Dovudra", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 0.6,
              "layers": [dt.layer(dt.attention(4, 2, 16, 16, 19, 8, 30, scale=0.4), dt.dense(44)),
                         dt.layer(dt.latent(2, 8, 4, 8, 12, 30), dt.dense(24))]}
    folder = dt.make_model_dir(tmp_path / "m", config, 77, stored_as(dtype), std=0.2 if dtype == "float32" else 0.1)
    requests = {"long": tokens_of(61, 200, 9)}
    want = dt.plain_logits(folder, requests["long"])
    for steps in (th.portions(requests, (20, 3, 11, 2)), th.prefix_then_single(requests, tail=170)):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps, max_tokens=96), requests)["long"]
        assert excess(got, want, dtype) <= 1.0


# ---------------------------------------------------------------------------------------------
# whole models, every cutting
# ---------------------------------------------------------------------------------------------


@pytest.fixture(scope="module", params=sorted(dt.TINY))
def case(request, tmp_path_factory):
    config, seed, page = dt.TINY[request.param]
    base = tmp_path_factory.mktemp(f"dovudra_{request.param}")
    folders = {"float32": dt.make_model_dir(base / "f32", config, seed, torch.float32, std=0.15),
               "bfloat16": dt.make_model_dir(base / "bf16", config, seed, torch.bfloat16, std=0.08)}
    for folder in folders.values():  # the folder's own file does not name the bias tables' rows: the tensors do
        (folder / "config.json").write_text(json.dumps(dt.without_rows(config)))
    lengths = (1, 2, 37, 150, 70, 9)
    requests = {f"r{i}": tokens_of(config["vocab"], n, 100 * seed + i) for i, n in enumerate(lengths)}
    expected = {dtype: {rid: plain.forward(config, dt.read_model_dir(folder)[1], tokens) for rid, tokens in requests.items()}
                for dtype, folder in folders.items()}
    return {"name": request.param, "page": page, "folders": folders, "requests": requests, "expected": expected}


def check_against_plain(case, dtype: str, steps: list[dict], **more) -> None:
    outputs = run_trace(case["folders"][dtype], dtype, case["page"], steps, **more)
    got = th.collect(steps, outputs, case["requests"])
    for rid, want in case["expected"][dtype].items():
        worst = excess(got[rid], want, dtype)
        assert worst <= 1.0, f"{case['name']} {dtype} {rid}: {worst:.2f} times the bound"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_prompts(case, dtype):
    check_against_plain(case, dtype, th.whole(case["requests"]))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_prefix_then_token_by_token(case, dtype):
    check_against_plain(case, dtype, th.prefix_then_single(case["requests"], tail=40))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("sizes", [(2, 3, 5, 2, 16, 7), (33, 2, 70, 64), (1, 2)])
def test_portions_of_changing_size(case, dtype, sizes):
    check_against_plain(case, dtype, th.portions(case["requests"], sizes))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_batches_on_pages_that_are_used_again(case, dtype):
    """Three requests live at a time out of six, on a pool sized for the peak: every page serves
    several requests, and what one left there must not reach the next."""
    steps = th.mixed(case["requests"], (7, 2, 19, 66, 3), max_live=3, decode_tail=9)
    check_against_plain(case, dtype, steps, max_live=3)


def test_long_decoding(case):
    """One short prompt, then 180 tokens one by one (recorded steps), in 32-bit: every window of the
    model passes wholly over decoded tokens."""
    config = dt.TINY[case["name"]][0]
    tokens = tokens_of(config["vocab"], 186, 4242)
    requests = {"long": tokens}
    steps = th.prefix_then_single(requests, tail=180)
    got = th.collect(steps, run_trace(case["folders"]["float32"], "float32", case["page"], steps), requests)["long"]
    want = plain.forward(config, dt.read_model_dir(case["folders"]["float32"])[1], tokens)
    assert excess(got, want, "float32") <= 1.0, case["name"]


def test_cuttings_agree_in_32_bit(case):
    """The logits of a position do not depend on how its request was cut or batched, beyond rounding."""
    folder, page = case["folders"]["float32"], case["page"]
    ways = {"whole": th.whole(case["requests"]), "single": th.prefix_then_single(case["requests"], tail=40),
            "portions": th.portions(case["requests"], (2, 5, 3, 24)), "mixed": th.mixed(case["requests"], (5, 2, 21, 80), max_live=4)}
    results = {name: th.collect(steps, run_trace(folder, "float32", page, steps), case["requests"]) for name, steps in ways.items()}
    for name, got in results.items():
        for rid, base in results["whole"].items():
            scale = base.abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
            assert float(((got[rid] - base).abs() / scale).max()) <= 5e-5, (name, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_the_replay_program(case, dtype, tmp_path):
    """``bin/trace_run`` itself on a model folder of this design, steps that want nothing included."""
    if case["name"] != "A":
        pytest.skip("one configuration is enough for the subprocess test")
    steps = th.mixed(case["requests"], (7, 2, 19, 66, 3), max_live=3, decode_tail=9)
    for record in steps[1::3]:
        for entry in record["entries"]:
            entry["want"] = []
    out = tmp_path / "out"
    proc = subprocess.run(
        [sys.executable, str(ROOT / "bin" / "trace_run"), "--model", str(case["folders"][dtype]), "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(th.peak_tokens(steps)), "--page-size", str(case["page"])],
        input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600,
    )
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [line for line in proc.stdout.splitlines() if line.startswith("done ")] == [f"done {s['step']}" for s in steps]
    import numpy as np

    vocab = dt.TINY["A"][0]["vocab"]
    position = {rid: 0 for rid in case["requests"]}
    for record in steps:
        wanted = sum(len(e["want"]) for e in record["entries"])
        path = out / f"{record['step']}.f32"
        assert path.exists() == bool(wanted)
        got = torch.from_numpy(np.fromfile(path, dtype="<f4").reshape(wanted, vocab).copy()) if wanted else None
        row = 0
        for entry in record["entries"]:
            for place in entry["want"]:
                want = case["expected"][dtype][entry["id"]][position[entry["id"]] + place]
                assert excess(got[row:row + 1], want[None], dtype) <= (1.0 if dtype == "float32" else BF16_OUTLIERS)
                row += 1
            position[entry["id"]] += len(entry["tokens"])


def random_config(rng: random.Random) -> dict:
    width = rng.choice([40, 52, 64, 72, 96, 100, 128])
    shared_kv, shared_vdim = rng.choice([1, 2, 3]), rng.choice([8, 12, 16, 32])  # what mixing layers must agree on
    layers = []
    for _ in range(rng.randint(1, 5)):
        if rng.random() < 0.5:
            mixing = rng.random() < 0.6
            kv = shared_kv if mixing else rng.choice([1, 1, 2, 3])
            dim = rng.choice([8, 12, 16, 20, 32, 48])
            rows = rng.choice([2, 5, 8, 16, 32])
            mixer = dt.attention(kv * rng.choice([1, 2, 4]), kv, dim, shared_vdim if mixing else rng.choice([dim, 8, 24, 40]),
                                 rng.choice([None, 1, 2, 5, 16, 33, 64, 500]), rows, rows // 2 + rng.choice([1, 7.5, 40, 300]),
                                 scale=rng.choice([dim ** -0.5, 0.2, 0.5]), v_mix=mixing)
        else:
            rot = rng.choice([2, 4, 8, 16])
            stretch = rng.choice([None, (rng.choice([2.0, 8.0, 40.0]), rng.choice([8, 64, 1024]), rng.choice([4.0, 32.0]), rng.choice([0.5, 1.0]))])
            mixer = dt.latent(rng.choice([1, 2, 3, 5]), rng.choice([4, 8, 12, 32]), rot, rng.choice([4, 8, 20, 32]),
                              rng.choice([3, 8, 16, 40]), rng.choice([None, 1, 3, 17, 64, 130]), turned=rng.choice([rot, 2]),
                              base=rng.choice([10.0, 1000.0, 50000.0]), stretch=stretch)
        layers.append(dt.layer(mixer, rng.choice([dt.dense(rng.choice([24, 44, 64, 100])), None])))
    config = {"architecture": "Dovudra", "vocab": rng.choice([50, 97, 256]), "width": width,
              "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        config["residual_mult"] = rng.choice([0.1, 0.3, 0.5, 1.0, 1.5])
    return config


@pytest.mark.parametrize("trial", range(10))
def test_random_configurations_replay_like_plain(trial, tmp_path):
    """Seeded random configurations: one to five layers of either mixer in any order, windows from one
    position to longer than any request or none, tables of two to 32 rows, stretched or plain
    frequencies, mixing layers or none; whole, token by token and mixed; 32-bit (every position
    inside the bound) and bfloat16 (nine positions in ten)."""
    rng = random.Random(7000 + trial)
    config = random_config(rng)
    lengths = [rng.randint(1, 6), rng.randint(10, 60), rng.randint(100, 200), rng.randint(20, 90)]
    requests = {f"r{i}": [rng.randrange(config["vocab"]) for _ in range(n)] for i, n in enumerate(lengths)}
    for dtype, std in (("float32", 0.15), ("bfloat16", 0.06)):
        folder = dt.make_model_dir(tmp_path / dtype, config, trial, stored_as(dtype), std=std)
        raw, tensors = dt.read_model_dir(folder)
        want = {rid: plain.forward(raw, tensors, tokens) for rid, tokens in requests.items()}
        ways = (th.whole(requests), th.prefix_then_single(requests, tail=20),
                th.mixed(requests, (7, 2, 40, 150, 3), max_live=4, decode_tail=5))
        for steps in ways:
            outputs = run_trace(folder, dtype, 16, steps, max_tokens=th.peak_tokens(steps))
            got = th.collect(steps, outputs, requests)
            for rid in requests:
                if dtype == "float32":
                    assert excess(got[rid], want[rid], dtype) <= 1.0, (trial, rid, config)
                else:
                    bound = RTOL_BF16 * want[rid].abs().amax(dim=-1).clamp_min(1.0)
                    rows = (got[rid] - want[rid]).abs().amax(dim=-1) / bound
                    assert float(rows.sort().values[int(0.9 * (len(rows) - 1))]) <= 1.0, (trial, rid, config)


# ---------------------------------------------------------------------------------------------
# one key that a query rests on: far back, at page borders, at the first positions, just inside and
# just outside a window
# ---------------------------------------------------------------------------------------------

MARK, ASKS = 7, 9  # the token that is looked for and the token whose query looks for it
WINDOW = 40


def marked_config(kind: str, window: int | None) -> dict:
    first = {"biased": dt.layer(dt.attention(2, 1, 32, 32, window, 10, 60, scale=0.5), dt.dense(64)),
             "latent": dt.layer(dt.latent(2, 32, 8, 32, 32, window, base=2000.0, scale=0.8, stretch=(4.0, 64, 8.0, 1.0)), dt.dense(64))}[kind]
    return {"architecture": "Dovudra", "vocab": 64, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 0.7, "layers": [first]}


def marked_model(folder, kind: str, dtype: torch.dtype, window: int | None):
    """Weights under which the query of token ASKS rests on the key of token MARK wherever that
    lies, and under which what it finds there matters: the first half of the width is what the
    layer's queries and keys are made of, and there both tokens' rows of the table hold the same
    large vector; the second half is what its values are made of, and there only MARK's row is
    large.  The model has this one layer, so a key that the layer does not see cannot move the
    logits at all."""
    config = marked_config(kind, window)
    tensors = dt.draw_tensors(config, 21, torch.float32, 0.12)
    g = torch.Generator().manual_seed(3)
    address, content = torch.randn(32, generator=g), torch.randn(32, generator=g)
    asking = torch.randn(32, generator=g)  # the latent layer's queries are made from an address of their own
    tensors["embed"][MARK] = torch.cat([5.0 * address, 5.0 * content])
    tensors["l0.norm1"].fill_(1.0)
    if kind == "biased":
        # Queries and keys are normalised per head, so a score is the scale times the head size times
        # the cosine of the two: 16 for the mark (and for the asking token itself), a few for the rest.
        tensors["embed"][ASKS] = torch.cat([5.0 * address, 0.2 * tensors["embed"][ASKS][32:]])
        tensors["l0.mix.q"][:, 32:] = 0
        tensors["l0.mix.k"] = tensors["l0.mix.q"][:32].clone()
        tensors["l0.mix.k.norm"] = tensors["l0.mix.q.norm"].clone()
        tensors["l0.mix.v"][:, :32] = 0
        tensors["l0.mix.rel"] *= 0.3
    else:
        # One latent serves keys and values: it holds the address in its first half and the content
        # in its second (16 + 16 of 32); keys read the first, values the second.  The query matrix
        # first turns the asking token's own address into the marked token's and then does what the
        # latent's first half does, so the asking token finds the mark and not itself.
        tensors["embed"][:, :32] *= 0.05  # every other token's key is small: the marked one stands out among hundreds
        tensors["embed"][MARK] = torch.cat([5.0 * address, 5.0 * content])
        tensors["embed"][ASKS] = torch.cat([5.0 * asking, 5.0 * torch.randn(32, generator=g)])
        down = tensors["l0.mix.dkv"]
        down[:16, 32:] = 0
        down[16:32, :32] = 0
        down[:32] *= 3.0
        up_k = torch.zeros(2, 32, 32)
        up_k[:, :16, :16] = torch.eye(16)
        tensors["l0.mix.uk"] = up_k.reshape(64, 32)
        up_v = torch.zeros(2, 32, 32)
        up_v[:, :16, 16:] = 4.0 * torch.randn(16, 16, generator=g)
        tensors["l0.mix.uv"] = up_v.reshape(64, 32)
        query = torch.zeros(2, 40, 64)
        query[:, :16, :32] = 3.0 * down[:16, :32] @ (address[:, None] * asking[None, :] / (asking @ asking))
        tensors["l0.mix.q"] = query.reshape(80, 64)
        tensors["l0.mix.dkv.norm"].fill_(1.0)
    # The norm in front of the layer takes the table's size away, and the norm behind the layer gives its
    # output a size of its own: with a small table the stream behind the layer is mostly what the layer found.
    tensors["embed"] *= 0.03
    tensors["final.norm"] *= 30.0  # the table is the output matrix too: logits of the usual size
    tensors = {name: t.to(dtype).contiguous() for name, t in tensors.items()}
    return dt.make_model_dir(folder, config, 0, tensors=tensors)


def marked_case(folder, mark_at: int, length: int):
    """``(tokens, plain logits, how far the last position's logits move without the mark)``."""
    config, tensors = dt.read_model_dir(folder)
    filler = [t for t in tokens_of(64, 2 * length + 8, 77) if t not in (MARK, ASKS)][:length]
    tokens = list(filler)
    tokens[mark_at] = MARK
    tokens[-1] = ASKS
    want = plain.forward(config, tensors, tokens)
    without = list(tokens)
    without[mark_at] = filler[mark_at]
    moved = (plain.forward(config, tensors, without)[-1] - want[-1]).abs().max() / want[-1].abs().max()
    return tokens, want, float(moved)


def check_marked(folder, dtype, tokens, want, places=1):
    """The asking token as the last of a whole prompt, decoded alone behind a prefix, and in a portion."""
    requests = {"m": tokens}
    tail = min(30, len(tokens) - 1)
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=tail), th.portions(requests, (17, 2, 64, 5))):
        got = th.collect(steps, run_trace(folder, dtype, 16, steps), requests)["m"]
        assert excess(got[-places:], want[-places:], dtype) <= 1.0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["biased", "latent"])
@pytest.mark.parametrize("mark_at", [0, 1, 15, 16, 17, 128, 230])
def test_a_key_far_back_is_found(tmp_path, kind, dtype, mark_at):
    """No window: a key up to 270 positions back (beyond the last row of the bias table), at a
    sequence's first positions and on both sides of a page border."""
    folder = marked_model(tmp_path / "far", kind, stored_as(dtype), None)
    tokens, want, moved = marked_case(folder, mark_at, 272)
    assert moved > 0.2, f"the far key does not matter enough to this model's last logits ({moved:.3f})"
    check_marked(folder, dtype, tokens, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["biased", "latent"])
@pytest.mark.parametrize("length", [WINDOW - 1, WINDOW, WINDOW + 1, WINDOW + 2, 3 * WINDOW + 9, 129, 128])
@pytest.mark.parametrize("outside", [False, True])
def test_keys_at_a_windows_edge(tmp_path, kind, dtype, length, outside):
    """The mark is the last key the asking token's window holds, or the first it does not (there the
    logits must not move at all, and a kernel that saw it would move them by much).  Sequences so
    short that the window holds their first token, or just loses it; an asking token at a page's
    first and last place."""
    folder = marked_model(tmp_path / "edge", kind, stored_as(dtype), WINDOW)
    mark_at = length - 1 - WINDOW + (0 if outside else 1)
    if mark_at < 0:
        if outside:
            pytest.skip("the sequence is shorter than the window: nothing lies outside")
        mark_at = 0  # the first token, still inside
    tokens, want, moved = marked_case(folder, mark_at, length)
    if outside:
        assert moved == 0.0, f"a key outside the window moves the plain implementation's logits ({moved:.3g})"
    else:
        assert moved > 0.2, f"the key inside the window does not matter enough ({moved:.3f})"
    check_marked(folder, dtype, tokens, want, places=min(3, length))


# ---------------------------------------------------------------------------------------------
# generation through the engine
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(tmp_path, name):
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    config, seed, page = dt.TINY[name]
    folder = dt.make_model_dir(tmp_path / "gen", config, seed + 5, torch.float32, std=0.2)
    raw, tensors = dt.read_model_dir(folder)
    prompts = [tokens_of(config["vocab"], n, 900 + n) for n in (3, 21, 1, 50)]
    new = 40
    want = [dt.greedy(raw, tensors, prompt, new) for prompt in prompts]
    engine = LLMEngine(EngineConfig(
        model=str(folder), dtype="float32",
        scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64, block_size=page, num_blocks=40),
    ))
    outputs = engine.generate(prompts, SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
    assert [out.new_token_ids for out in outputs] == want
    # Once more on the same engine: the pages of the first run are used again.
    again = engine.generate(list(reversed(prompts)), SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
    assert [out.new_token_ids for out in again] == list(reversed(want))


def test_the_command_line_serves_the_design(tmp_path, capsys):
    """``engine random-model`` writes a folder from a config.json of the design, ``engine generate``
    completes prompts given as token ids with the plain implementation's greedy tokens, and
    ``engine kv-size`` sizes a cache with one group per distinct page geometry."""
    import re

    from turboserve_amd import cli

    config, _, page = dt.TINY["A"]
    source = tmp_path / "config.json"
    source.write_text(json.dumps(config))
    folder = tmp_path / "model"
    assert cli.main(["engine", "random-model", "--config", str(source), "--out", str(folder), "--seed", "4", "--dtype", "float32"]) == 0
    raw, tensors = dt.read_model_dir(folder)
    prompts = [tokens_of(config["vocab"], n, 600 + n) for n in (4, 19)]
    capsys.readouterr()
    args = ["engine", "generate", "--model", str(folder), "--dtype", "float32", "--max-tokens", "12", "--ignore-eos",
            "--num-blocks", "24", "--block-size", str(page)]
    assert cli.main(args + [a for p in prompts for a in ("--prompt-ids", ",".join(map(str, p)))]) == 0
    shown = [json.loads(m) for m in re.findall(r"^output \d+: (\[.*\])$", capsys.readouterr().out, flags=re.M)]
    assert len(shown) == len(prompts)
    for prompt, got in zip(prompts, shown):
        tokens = list(prompt)
        for token in got:  # the written model's weights are small: equal logits are allowed for
            logits = plain.forward(raw, tensors, tokens)[-1]
            assert float(logits.max() - logits[token]) <= 1e-4 * float(logits.abs().max().clamp_min(1.0))
            tokens.append(token)
    assert cli.main(["engine", "kv-size", "--model", str(folder), "--dtype", "bfloat16", "--max-model-len", "64",
                     "--block-size", str(page)]) == 0
    sizing = capsys.readouterr().out
    sizing = json.loads(sizing[sizing.index("{"):])
    assert len(sizing["num_blocks"]) >= 2 and sizing["activation_bytes"] > 0
