"""Legavik on the GPU against the plain implementation (``tests/plain/legavik_plain.py``): each mechanism
alone (its kernel, and a one-layer model of it), whole prompts, every way of cutting requests into steps
on so few pages and slots that they are used again, keys at the edges of windows, of the kept first tokens
and of pages, at a sequence's first positions and far back, state that has to last, and greedy generation
through the engine's own entry point."""

from __future__ import annotations

import json
import random
import subprocess
import sys
from pathlib import Path

import pytest
import torch

import legavik_tiny as lt
import trace_helpers as th
from plain import legavik_plain as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
ROOT = Path(__file__).resolve().parent.parent
#: 32-bit engine against the 32-bit plain implementation, relative to a position's largest logit.
RTOL_F32 = 2e-4
#: bfloat16 engine (weights stored in bfloat16) against the plain implementation in 32-bit on the same
#: weights, for 19 positions in 20; the rest may be off by four times the bound (rounding can hand a token
#: to another expert where two router scores are close).
RTOL_BF16 = 4e-2
BF16_OUTLIERS = 4.0


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


def near(got: torch.Tensor, want: torch.Tensor, dtype: torch.dtype, loose: float = 1.0) -> None:
    tol = (2e-5 if dtype == torch.float32 else 1.6e-2) * loose
    scale = float(want.abs().max().clamp_min(1e-3))
    assert float((got.float().cpu() - want).abs().max()) <= tol * scale, float((got.float().cpu() - want).abs().max()) / scale


# ---------------------------------------------------------------------------------------------
# mechanisms alone: kernels
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,splits,also", [(52, 0, 0), (64, 3, 2), (321, 1, 0), (1000, 0, 9)])
def test_the_norm_without_statistics_carries_the_residual_sum(ops, dtype, hidden, splits, also):
    g = torch.Generator().manual_seed(hidden)
    tokens = 7
    residual = torch.randn(tokens, hidden, generator=g)
    pending = torch.randn(max(splits, 1), tokens, hidden, generator=g)
    second = torch.randn(max(also, 1), tokens, hidden, generator=g)
    weight = (1 + 0.3 * torch.randn(hidden, generator=g)).to(dtype)
    bias = (0.2 * torch.randn(hidden, generator=g)).to(dtype)
    alpha = 0.7
    given = pending.to(DEV) if splits else pending[0].to(dtype).to(DEV)
    total = residual + (pending.sum(0) if splits else pending[0].to(dtype).float()) + (second.sum(0) if also else 0)
    want = plain.squash_norm(total, {"n": weight.float(), "n.b": bias.float(), "n.alpha": torch.tensor(alpha)}, "n")
    stream = residual.clone().to(DEV)
    got = ops.add_tanh_norm(stream, given, weight.to(DEV), bias.to(DEV), alpha, also=second.to(DEV) if also else None)
    near(got, want, dtype)
    near(stream, total, torch.float32)
    # At chosen rows only: the stream stays as it is.
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
    stream = residual.clone().to(DEV)
    got = ops.add_tanh_norm(stream, given, weight.to(DEV), bias.to(DEV), alpha, rows, also=second.to(DEV) if also else None)
    near(got, want[[5, 0, 5]], dtype)
    assert torch.equal(stream.cpu(), residual)


def test_the_cap_on_the_logits(ops):
    x = torch.linspace(-90, 90, 1001).reshape(7, 143).contiguous()
    near(ops.tanh_cap(x.clone().to(DEV), 22.0), 22.0 * torch.tanh(x / 22.0), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("taps,channels,silu", [(1, 20, False), (2, 33, True), (3, 64, False), (4, 300, True), (5, 8, False)])
def test_the_short_convolution_carries_its_last_inputs(ops, dtype, taps, channels, silu):
    """Three requests of unequal length through state slots that are not in row order: whole, then cut
    into steps of one to five rows with the requests taking turns, partial sums and plain tensors alike."""
    g = torch.Generator().manual_seed(taps * 100 + channels)
    lengths, slots = [9, 1, 14], [2, 0, 3]
    width, first = channels + 11, 5
    weight = (0.6 * torch.randn(channels, taps, generator=g)).to(dtype)
    rows = [torch.randn(n, width, generator=g).to(dtype).float() for n in lengths]
    want = []
    for u in rows:
        y = plain.short_conv(u[:, first:first + channels], weight.float())
        want.append(torch.nn.functional.silu(y) if silu else y)
    state = torch.full((5, max(taps - 1, 1), channels), float("nan"), device=DEV)
    state[slots] = 0.0
    done = [0] * len(lengths)
    got = [torch.zeros(n, channels) for n in lengths]
    sizes = [1, 3, 2, 5, 1, 1, 4]
    turn = 0
    while any(d < n for d, n in zip(done, lengths)):
        live = [i for i in range(len(lengths)) if done[i] < lengths[i]]
        counts = {}
        for i in live:
            counts[i] = min(sizes[turn % len(sizes)], lengths[i] - done[i])
            turn += 1
        proj = torch.cat([rows[i][done[i]:done[i] + counts[i]] for i in live])
        starts = [0]
        for i in live:
            starts.append(starts[-1] + counts[i])
        seq_of = torch.tensor([j for j, i in enumerate(live) for _ in range(counts[i])], dtype=torch.int32, device=DEV)
        as_sums = turn % 2 == 0
        given = torch.stack([0.25 * proj, 0.75 * proj]).to(DEV) if as_sums else proj.to(dtype).to(DEV)
        out = ops.short_conv(given, first, weight.to(DEV), state, torch.tensor([slots[i] for i in live], dtype=torch.int32, device=DEV),
                             seq_of, torch.tensor(starts, dtype=torch.int32, device=DEV), tokens=proj.shape[0], num_seqs=len(live),
                             dtype=dtype, silu=silu, out_float32=turn % 3 == 0)
        for j, i in enumerate(live):
            got[i][done[i]:done[i] + counts[i]] = out[starts[j]:starts[j + 1]].float().cpu()
            done[i] += counts[i]
    for i in range(len(lengths)):
        near(got[i], want[i], dtype)
    assert torch.isnan(state[[1, 4]]).all() if taps > 1 else True


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_weighted_sum_of_two_outputs(ops, dtype):
    """Two parts' outputs, each a tensor of the run's type or partial sums, as one 32-bit addend."""
    g = torch.Generator().manual_seed(3)
    dense, sums = torch.randn(7, 52, generator=g).to(dtype), torch.randn(3, 7, 52, generator=g)
    other = torch.randn(7, 52, generator=g).to(dtype)
    got = ops.scaled_pair(dense.to(DEV), 0.6, sums.to(DEV), -1.3, dtype)
    assert got.shape == (1, 7, 52) and got.dtype == torch.float32
    near(got[0], 0.6 * dense.float() - 1.3 * sums.sum(0), torch.float32)
    near(ops.scaled_pair(sums.to(DEV), 2.0, sums.to(DEV), 0.5, dtype)[0], 2.5 * sums.sum(0), torch.float32)
    near(ops.scaled_pair(dense.to(DEV), 1.0, other.to(DEV), 1.0, dtype)[0], dense.float() + other.float(), torch.float32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,vdim,col0,scale", [(3, 12, 8, 0.6), (1, 20, 0, -0.8), (8, 64, 16, 1.0), (5, 7, 3, 0.0)])
def test_a_gate_per_head_scales_and_places_its_result(ops, dtype, heads, vdim, col0, scale):
    """The gate's launch multiplies by a weight as well and writes into columns of a wider buffer, whose other
    columns stay as they are; values of the run's own type and 32-bit ones."""
    g = torch.Generator().manual_seed(heads * 10 + vdim)
    tokens, width = 9, heads + 5
    proj = torch.randn(tokens, width, generator=g).to(dtype)
    for values in (torch.randn(tokens, heads * vdim, generator=g), torch.randn(tokens, heads * vdim, generator=g).to(dtype)):
        gate = torch.sigmoid(proj.float()[:, 2:2 + heads]).repeat_interleave(vdim, dim=1)
        want = scale * values.float() * gate
        wide = torch.full((tokens, col0 + heads * vdim + 4), 7.0, dtype=dtype, device=DEV)
        got = ops.head_gate(values.to(DEV), proj.to(DEV), 2, heads, dtype, scale=scale, out=(wide, col0))
        assert got is wide
        near(wide[:, col0:col0 + heads * vdim], want, dtype)
        assert bool((wide[:, :col0] == 7.0).all()) and bool((wide[:, col0 + heads * vdim:] == 7.0).all())
        near(ops.head_gate(values.to(DEV), proj.to(DEV), 2, heads, dtype), values.float() * gate, dtype)


def delta_inputs(g, tokens, heads, kv_heads, dim, vdim, low_a, low_g, dtype):
    keys, values = kv_heads * dim, heads * vdim
    u = torch.randn(tokens, 2 * keys + values, generator=g)
    proj = torch.randn(tokens, heads + low_a + low_g + 3, generator=g).to(dtype).float()
    tensors = {
        "a2": (0.5 * torch.randn(heads * dim, low_a, generator=g)).to(dtype), "dt": (-1 + torch.randn(heads * dim, generator=g)).to(dtype),
        "a_log": -2 + 1.5 * torch.randn(heads, generator=g), "g2": (0.5 * torch.randn(values, low_g, generator=g)).to(dtype),
        "gain": (1 + 0.3 * torch.randn(vdim, generator=g)).to(dtype),
    }
    return u, proj, tensors


def plain_delta(u, proj, t, heads, kv_heads, dim, vdim, low_a, low_g, eps, at):
    """The recurrence of ``plain.delta_rule`` on inputs that are already convolved: the same statements."""
    T, keys = u.shape[0], kv_heads * dim
    q, k, v = u[:, :keys].view(T, kv_heads, dim), u[:, keys:2 * keys].view(T, kv_heads, dim), u[:, 2 * keys:].view(T, heads, vdim)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(proj[:, at:at + heads])
    low = proj[:, at + heads:at + heads + low_a]
    step = torch.nn.functional.softplus(low @ t["a2"].float().T + t["dt"].float())
    decay = torch.exp(-torch.exp(t["a_log"])[:, None] * step.view(T, heads, dim))
    gate = torch.sigmoid(proj[:, at + heads + low_a:at + heads + low_a + low_g] @ t["g2"].float().T).view(T, heads, vdim)
    out = torch.zeros(T, heads, vdim)
    for head in range(heads):
        g = head // (heads // kv_heads)
        S = torch.zeros(dim, vdim)
        for i in range(T):
            S = decay[i, head][:, None] * S
            w = beta[i, head] * (v[i, head] - S.T @ k[i, g])
            S = S + torch.outer(k[i, g], w)
            out[i, head] = S.T @ q[i, g]
    return (plain.unit_rms(out, eps) * t["gain"].float() * gate).reshape(T, heads * vdim)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,low_a,low_g", [(4, 2, 16, 8, 6, 5), (1, 1, 20, 70, 1, 9), (3, 3, 96, 32, 8, 3),
                                                                 (2, 1, 200, 130, 24, 24), (6, 2, 64, 64, 4, 4)])
def test_the_delta_rule_whole_and_in_pieces(ops, dtype, heads, kv_heads, dim, vdim, low_a, low_g):
    """Two requests side by side through slots not in row order: whole, then in pieces of 1, 2, 9 and 30
    tokens, from partial sums and from plain tensors."""
    g = torch.Generator().manual_seed(heads * 1000 + dim)
    lengths, slots, at, eps = [57, 23], [3, 1], 2, 1e-5
    cases = [delta_inputs(g, n, heads, kv_heads, dim, vdim, low_a, low_g, dtype) for n in lengths]
    t = cases[0][2]
    want = [plain_delta(u, proj, t, heads, kv_heads, dim, vdim, low_a, low_g, eps, at) for u, proj, _ in cases]
    on_device = {k: v.to(DEV) for k, v in t.items()}
    for sizes in ([100], [1, 2, 9, 30]):
        state = torch.full((5, heads, dim, vdim), float("nan"), device=DEV)
        state[slots] = 0.0
        done, got, turn = [0, 0], [torch.zeros_like(w) for w in want], 0
        while any(d < n for d, n in zip(done, lengths)):
            live = [i for i in range(2) if done[i] < lengths[i]]
            counts = {i: min(sizes[(turn + i) % len(sizes)], lengths[i] - done[i]) for i in live}
            turn += 1
            u = torch.cat([cases[i][0][done[i]:done[i] + counts[i]] for i in live]).contiguous().to(DEV)
            proj = torch.cat([cases[i][1][done[i]:done[i] + counts[i]] for i in live])
            given = torch.stack([0.5 * proj, 0.5 * proj]).to(DEV) if turn % 2 else proj.to(dtype).to(DEV)
            starts = [0]
            for i in live:
                starts.append(starts[-1] + counts[i])
            y = ops.delta_rule(u, given, beta_at=at, decay_at=at + heads, gate_at=at + heads + low_a, a2=on_device["a2"],
                               dt_bias=on_device["dt"], a_log=on_device["a_log"], g2=on_device["g2"], gain=on_device["gain"], eps=eps,
                               state=state, state_slots=torch.tensor([slots[i] for i in live], dtype=torch.int32, device=DEV),
                               query_start_loc=torch.tensor(starts, dtype=torch.int32, device=DEV), tokens=u.shape[0],
                               num_seqs=len(live), heads=heads, kv_heads=kv_heads, head_dim=dim, value_dim=vdim, dtype=dtype,
                               num_long_seqs=(turn % 3) % (len(live) + 1))
            for j, i in enumerate(live):
                got[i][done[i]:done[i] + counts[i]] = y[starts[j]:starts[j + 1]].float().cpu()
                done[i] += counts[i]
        for i in range(2):
            near(got[i], want[i], dtype, loose=3.0)
        assert torch.isnan(state[[0, 2, 4]]).all()


@pytest.mark.parametrize("experts,top,groups,keep", [(10, 4, 5, 3), (6, 2, 3, 2), (5, 2, 5, 3), (4, 4, 1, 1), (12, 3, 2, 1)])
def test_the_router_marks_a_group_by_its_best_expert(ops, experts, top, groups, keep):
    g = torch.Generator().manual_seed(experts * 10 + top)
    x = torch.randn(50, 24, generator=g)
    router = torch.randn(experts, 24, generator=g)
    taken, weights, _ = ops.moe_route(x.to(DEV), router.to(DEV), top=top, groups=groups, keep=keep, scale=1.0, softmax=True, mark_top=1)
    rule = {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}
    for t in range(x.shape[0]):
        scores = torch.softmax(x[t] @ router.T, dim=0)
        want = plain.choose(scores, rule)
        assert taken[t].tolist() == want
        total = sum(float(scores[e]) for e in want) + 1e-20
        near(weights[t], torch.tensor([float(scores[e]) / total for e in want]), torch.float32, loose=5.0)
    # Where the sum of a group's two best and its best alone disagree, the two rules choose differently.
    z = torch.tensor([[2.0, -9.0, 1.5, 1.4]])
    eye = torch.eye(4)
    best, _, _ = ops.moe_route(z.to(DEV), eye.to(DEV), top=1, groups=2, keep=1, scale=1.0, softmax=True, mark_top=1)
    both, _, _ = ops.moe_route(z.to(DEV), eye.to(DEV), top=1, groups=2, keep=1, scale=1.0, softmax=True, mark_top=2)
    assert best.tolist() == [[0]] and both.tolist() == [[2]]


def plain_rows(q, k, v, contexts, scale, window, keep):
    """``q [S][n, H, D]`` the last ``n`` positions of requests with ``k, v [S][context, G, *]``."""
    out = []
    for qs, ks, vs in zip(q, k, v):
        context, n = ks.shape[0], qs.shape[0]
        H, G = qs.shape[1], ks.shape[1]
        rows = torch.zeros(n, H, vs.shape[2])
        for r in range(n):
            i = context - n + r
            seen = [j for j in range(i + 1) if plain.sees(i, j, None if window is None else {"size": window, "keep_first": keep})]
            for h in range(H):
                scores = (ks[seen, h // (H // G)] @ qs[r, h]) * scale
                rows[r, h] = torch.softmax(scores, dim=0) @ vs[seen, h // (H // G)]
        out.append(rows.reshape(n, -1))
    return torch.cat(out)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,page,window,keep", [
    (4, 2, 16, 16, 16, 20, 5), (3, 1, 24, 8, 8, 1, 3), (6, 2, 32, 32, 32, 70, 40), (8, 1, 64, 128, 16, 33, 1),
    (2, 2, 128, 128, 16, 150, 24), (4, 4, 64, 64, 8, 64, 64), (2, 1, 8, 8, 8, 9, 0), (1, 1, 40, 24, 16, 300, 7)])
def test_a_window_that_keeps_the_first_keys(ops, heads, kv_heads, dim, vdim, page, window, keep):
    """Portions and single tokens in one step, pages scattered and those between the kept keys and the window
    missing: the generic kernel in 32-bit against explicit rows, the tiled kernel in bfloat16 against both."""
    g = torch.Generator().manual_seed(window * 7 + keep)
    contexts, news = [190, 77, 3, 150, 64], [45, 77, 2, 1, 1]
    k = [torch.randn(c, kv_heads, dim, generator=g) for c in contexts]
    v = [torch.randn(c, kv_heads, vdim, generator=g) for c in contexts]
    q = [torch.randn(n, heads, dim, generator=g) for n in news]
    scale = 0.9 * dim ** -0.5
    pages_of = [-(-c // page) for c in contexts]
    order = torch.randperm(sum(pages_of) + 3, generator=g).tolist()
    width = max(pages_of)
    for dtype in (torch.float32, torch.bfloat16):
        as_stored = [[t.to(dtype).float() for t in group] for group in (q, k, v)]
        want = plain_rows(*as_stored, contexts, scale, window, keep)
        # What lies in places no query may read is large, and finite (a masked key's weight is an exact zero).
        k_pages = torch.full((len(order), kv_heads, page, dim), 1e3, dtype=dtype)
        v_pages = torch.full((len(order), kv_heads, vdim, page), -1e3, dtype=dtype)
        table = torch.full((len(contexts), width), -1, dtype=torch.int32)
        at = 0
        for s, c in enumerate(contexts):
            lowest = max(0, c - news[s] - window + 1) // page  # pages below the first query's window ...
            for index in range(pages_of[s]):
                held = index >= lowest or index < -(-keep // page)  # ... are gone, unless they hold kept keys
                if held:
                    table[s, index] = order[at]
                    rows = slice(index * page, min((index + 1) * page, c))
                    count = rows.stop - rows.start
                    k_pages[order[at], :, :count] = as_stored[1][s][rows].transpose(0, 1).to(dtype)
                    v_pages[order[at], :, :, :count] = as_stored[2][s][rows].permute(1, 2, 0).to(dtype)
                at += 1
        flat_q = torch.cat([t.reshape(t.shape[0], -1) for t in as_stored[0]]).to(dtype).contiguous().to(DEV)
        starts = [0]
        for n in news:
            starts.append(starts[-1] + n)
        seq_of = torch.tensor([s for s, n in enumerate(news) for _ in range(n)], dtype=torch.int32, device=DEV)
        positions = torch.tensor([c - n + r for c, n in zip(contexts, news) for r in range(n)], dtype=torch.int32, device=DEV)
        tables = table.clamp_min(0 if dtype == torch.bfloat16 else -1).to(DEV)
        generic = ops.paged_attention_generic(flat_q, heads * dim, k_pages.to(DEV), v_pages.to(DEV), table.clamp_min(0).to(DEV), seq_of, positions,
                                              heads, scale, window, keep_first=keep)
        near(generic, want, dtype, loose=2.0)
        if dtype == torch.bfloat16 and ops.tiled_attention_supported(dtype, dim, vdim, page, heads * dim):
            tiles = ops.device_ints(ops.attention_tile_list(news[:3], contexts[:3], window=window))
            tiled = ops.attention_tiles(flat_q, heads * dim, k_pages.to(DEV), v_pages.to(DEV), tables,
                                        torch.tensor(starts, dtype=torch.int32, device=DEV), torch.tensor(contexts, dtype=torch.int32, device=DEV),
                                        tokens=flat_q.shape[0], heads=heads, scale=scale, prefill_tiles=tiles, num_prefill_seqs=3,
                                        num_decode_seqs=2, max_decode_context=max(contexts[3:]), window=window, keep_first=keep)
            near(tiled, want, dtype, loose=2.0)


# ---------------------------------------------------------------------------------------------
# mechanisms alone: one-layer models
# ---------------------------------------------------------------------------------------------

ALONE = {
    "keyed": lt.layer(lt.keyed(4, 2, 16, scale=0.4, window=13, keep=4, rot=8, base=100.0), None),
    "keyed_one_head_no_window": lt.layer(lt.keyed(1, 1, 20, scale=0.5, rot=20, stretch=(4.0, 32, 8.0, 1.0), base=100.0), None),
    "keyed_window_of_one": lt.layer(lt.keyed(3, 3, 8, scale=0.5, window=1, keep=2, rot=2), None),
    "keyed_no_rotation": lt.layer(lt.keyed(2, 1, 12, window=9), None),
    "keyed_matrix_cores": lt.layer(lt.keyed(4, 1, 32, window=40, keep=17, rot=16, stretch=(2.0, 16, 4.0, 1.0), base=5000.0), None),
    # No kept tokens: keys and values of one size go to the head-size kernels, with and without a window.
    "keyed_head_size_kernels": lt.layer(lt.keyed(4, 2, 32, window=40, rot=16, base=300.0), None),
    "keyed_head_size_kernels_no_window": lt.layer(lt.keyed(4, 1, 64, rot=32, stretch=(4.0, 32, 8.0, 1.0)), None),
    "left_only_matters": lt.layer(lt.parallel(lt.left(4, 2, 16, 24, 3, scale=0.4, temp=(0.5, 4)), lt.right(1, 1, 8, 8, 2, 2, 2), 1.0, 1e-3), None),
    "right_only_matters": lt.layer(lt.parallel(lt.left(1, 1, 8, 8, 2), lt.right(4, 2, 16, 12, 4, 5, 3), 1e-3, 1.0), None),
    "pair_one_tap": lt.layer(lt.parallel(lt.left(2, 2, 8, 16, 1, temp=(1.0, 1)), lt.right(2, 2, 8, 8, 1, 3, 3), 0.5, -0.7), None),
    "pair_matrix_cores": lt.layer(lt.parallel(lt.left(4, 2, 32, 64, 3, temp=(0.3, 16)), lt.right(2, 1, 72, 40, 3, 8, 8), 0.75, 0.5), None),
    "experts": lt.layer(lt.keyed(1, 1, 8, rot=4), lt.moe(20, 9, 4, (3, 2))),
    "experts_plain_top": lt.layer(lt.keyed(1, 1, 8), lt.moe(12, 5, 2)),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", sorted(ALONE))
def test_one_layer_models(tmp_path, which, dtype):
    """A model of one layer: whole, token by token from the start, and in portions, against the plain
    implementation; with and without the cap on the logits."""
    config = {"architecture": "Legavik", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "layers": [ALONE[which]]}
    if "keyed" in which:
        config["logit_softcap"] = 2.0
    folder = lt.make_model_dir(tmp_path / "m", config, 31, stored_as(dtype), std=0.2 if dtype == "float32" else 0.1)
    requests = {"a": tokens_of(61, 75, 1), "b": tokens_of(61, 3, 2)}
    want = {rid: lt.plain_logits(folder, tokens) for rid, tokens in requests.items()}
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=74), th.portions(requests, (2, 5, 31, 3))):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps), requests)
        for rid in requests:
            assert excess(got[rid], want[rid], dtype) <= 1.0, (which, rid)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_windows_on_a_pool_smaller_than_the_request(tmp_path, dtype):
    """A layer that reads a window and the first tokens gives the pages between back while the request
    runs: 200 tokens go through a pool of 96 (the parallel layer's pages are the pool's own and hold
    every token, so that layer is left out here), in portions and token by token."""
    config = {"architecture": "Legavik", "vocab": 61, "width": 40, "norm": {"eps": 1e-5}, "logit_softcap": 9.0,
              "layers": [lt.layer(lt.keyed(4, 2, 16, scale=0.4, window=19, keep=11, rot=8), lt.moe(20, 4, 2, (2, 1))),
                         lt.layer(lt.keyed(2, 2, 16, scale=0.4, window=19, keep=11, rot=16), None)]}
    folder = lt.make_model_dir(tmp_path / "m", config, 77, stored_as(dtype), std=0.2 if dtype == "float32" else 0.1)
    requests = {"long": tokens_of(61, 200, 9)}
    want = lt.plain_logits(folder, requests["long"])
    for steps in (th.portions(requests, (20, 3, 11, 2)), th.prefix_then_single(requests, tail=170)):
        got = th.collect(steps, run_trace(folder, dtype, 8, steps, max_tokens=96), requests)["long"]
        assert excess(got, want, dtype) <= 1.0


# ---------------------------------------------------------------------------------------------
# whole models, every cutting
# ---------------------------------------------------------------------------------------------


@pytest.fixture(scope="module", params=sorted(lt.TINY))
def case(request, tmp_path_factory):
    config, seed, page = lt.TINY[request.param]
    base = tmp_path_factory.mktemp(f"legavik_{request.param}")
    folders = {"float32": lt.make_model_dir(base / "f32", config, seed, torch.float32, std=0.15),
               "bfloat16": lt.make_model_dir(base / "bf16", config, seed, torch.bfloat16, std=0.08)}
    for folder in folders.values():  # the folder's own file does not name the low-rank widths: the tensors do
        (folder / "config.json").write_text(json.dumps(lt.without_ranks(config)))
    lengths = (1, 2, 37, 150, 70, 9)
    requests = {f"r{i}": tokens_of(config["vocab"], n, 100 * seed + i) for i, n in enumerate(lengths)}
    expected = {dtype: {rid: plain.forward(config, lt.read_model_dir(folder)[1], tokens) for rid, tokens in requests.items()}
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
def test_mixed_batches_on_pages_and_slots_that_are_used_again(case, dtype):
    """Three requests live at a time out of six, on a pool sized for the peak and three state slots: every
    page and slot serves several requests, and what one left there must not reach the next."""
    steps = th.mixed(case["requests"], (7, 2, 19, 66, 3), max_live=3, decode_tail=9)
    check_against_plain(case, dtype, steps, max_live=3)


def test_long_decoding(case):
    """One short prompt, then 180 tokens one by one (recorded steps), in 32-bit: every window of the model
    passes wholly over decoded tokens, and the state is carried through every one of them."""
    config = lt.TINY[case["name"]][0]
    tokens = tokens_of(config["vocab"], 186, 4242)
    requests = {"long": tokens}
    steps = th.prefix_then_single(requests, tail=180)
    got = th.collect(steps, run_trace(case["folders"]["float32"], "float32", case["page"], steps), requests)["long"]
    want = plain.forward(config, lt.read_model_dir(case["folders"]["float32"])[1], tokens)
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

    vocab = lt.TINY["A"][0]["vocab"]
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
    layers = []
    for _ in range(rng.randint(1, 5)):
        if rng.random() < 0.5:
            kv = rng.choice([1, 1, 2, 3])
            dim = rng.choice([8, 12, 16, 20, 32, 64])
            window = rng.choice([None, 1, 2, 5, 16, 33, 64, 500])
            keep = None if window is None else rng.choice([None, 0, 1, 3, 16, 20, 70])
            rot = rng.choice([None, 2, dim // 2 // 2 * 2, dim])
            stretch = rng.choice([None, (rng.choice([2.0, 8.0, 40.0]), rng.choice([8, 64, 1024]), rng.choice([4.0, 32.0]), rng.choice([0.5, 1.0]))])
            mixer = lt.keyed(kv * rng.choice([1, 2, 4]), kv, dim, scale=rng.choice([None, 0.2, 0.5]), window=window, keep=keep,
                             rot=rot, stretch=stretch if rot else None, base=rng.choice([10.0, 1000.0, 1e6]))
        else:
            kv, dim = rng.choice([1, 2, 3]), rng.choice([8, 12, 16, 32, 48])
            temp = rng.choice([None, (rng.choice([0.1, 0.5, -0.05]), rng.choice([1, 7, 64, 1000]))])
            one = lt.left(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([dim, 8, 24, 40]), rng.choice([None, 1, 2, 3, 4]),
                          scale=rng.choice([None, 0.2, 0.5]), temp=temp)
            kv = rng.choice([1, 2, 3])
            other = lt.right(kv * rng.choice([1, 2]), kv, rng.choice([4, 8, 20, 64, 100]), rng.choice([4, 8, 20, 32, 66]),
                             rng.choice([1, 2, 4, 5]), rng.choice([1, 3, 8, 24]), rng.choice([1, 4, 24]))
            mixer = lt.parallel(one, other, rng.choice([0.3, 0.6, 1.0, -1.0]), rng.choice([0.3, 0.9, 1.0, 1.7]))
        feed = None
        if rng.random() < 0.7:
            count = rng.choice([1, 2, 3, 4])
            size = rng.choice([1, 2, 3])
            keep = rng.randint(1, count)
            feed = lt.moe(rng.choice([8, 20, 44, 64]), count * size, rng.randint(1, size * keep), rng.choice([None, (count, keep)]) if keep == count else (count, keep))
        layers.append(lt.layer(mixer, feed))
    config = {"architecture": "Legavik", "vocab": rng.choice([50, 97, 256]), "width": width,
              "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.7:
        config["logit_softcap"] = rng.choice([1.5, 10.0, 40.0])
    return config


@pytest.mark.parametrize("trial", range(10))
def test_random_configurations_replay_like_plain(trial, tmp_path):
    """Seeded random configurations: one to five layers of either mixer in any order, windows from one
    position to longer than any request or none, kept first tokens within a page and beyond, rotation of
    two elements, half a head, a whole head or none, convolutions of one to five taps or none, experts in
    groups of one to three or ungrouped; whole, token by token and mixed; 32-bit (every position inside the
    bound) and bfloat16 (nine positions in ten)."""
    rng = random.Random(9000 + trial)
    config = random_config(rng)
    lengths = [rng.randint(1, 6), rng.randint(10, 60), rng.randint(100, 200), rng.randint(20, 90)]
    requests = {f"r{i}": [rng.randrange(config["vocab"]) for _ in range(n)] for i, n in enumerate(lengths)}
    for dtype, std in (("float32", 0.15), ("bfloat16", 0.06)):
        folder = lt.make_model_dir(tmp_path / dtype, config, trial, stored_as(dtype), std=std)
        raw, tensors = lt.read_model_dir(folder)
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
# just outside a window, just inside and just outside the kept first tokens
# ---------------------------------------------------------------------------------------------

MARK, ASKS, OTHER = 7, 9, 11  # the token that is looked for, the token whose query looks for it, one that is neither
WINDOW, KEEP = 40, 6


def marked_model(folder, dtype: torch.dtype, window: int | None, keep: int | None):
    """One attention layer whose query of ``ASKS`` and key of ``MARK`` point the same way in the part of a head
    that is not turned, with a scale under which that one score stands above all others; the key is also
    the value, so what the query finds there reaches the logits.  No other token has anything in the two
    channels that make them."""
    config = {"architecture": "Legavik", "vocab": 40, "width": 32, "norm": {"eps": 1e-5},
              "layers": [lt.layer(lt.keyed(2, 1, 16, scale=1.5, window=window, keep=keep, rot=8, base=100.0), None)]}
    tensors = lt.draw_tensors(config, 5, torch.float32, 0.1)
    embed = tensors["embed"]
    embed[:, :2] = 0.0
    embed[MARK, 0] = 3.0
    embed[ASKS, 1] = 3.0
    tensors["l0.norm1"][:2] = 1.0
    tensors["l0.norm1.b"][:2] = 0.0
    towards = torch.zeros(16)
    towards[8:] = torch.tensor([1.0, -1.0, 1.0, 1.0, -1.0, 1.0, -1.0, -1.0])
    tensors["l0.mix.k"][:, 0] = 4.0 * towards
    tensors["l0.mix.k"][:, 1] = 0.0
    for head in range(2):
        tensors["l0.mix.q"][16 * head:16 * head + 16, 1] = 4.0 * towards
        tensors["l0.mix.q"][16 * head:16 * head + 16, 0] = 0.0
    tensors["l0.mix.g"] *= 0.0
    tensors = {name: t.to(dtype).contiguous() for name, t in tensors.items()}
    return lt.make_model_dir(folder, config, 0, tensors=tensors)


def marked_tokens(length: int, mark_at: int | None, seed: int) -> list[int]:
    """``length`` tokens that end in ``ASKS``; ``MARK`` at ``mark_at`` and nowhere else."""
    g = torch.Generator().manual_seed(seed)
    tokens = [t if t not in (MARK, ASKS) else OTHER for t in torch.randint(0, 40, (length,), generator=g).tolist()]
    tokens[-1] = ASKS
    if mark_at is not None:
        tokens[mark_at] = MARK
    return tokens


def check_marked(folder, dtype: str, tokens: list[int], seen: bool) -> None:
    """The plain implementation says what the mark is worth at the last position; the engine agrees with
    it in every cutting: whole, the last tokens one by one, portions that end at the mark's edge."""
    raw, tensors = lt.read_model_dir(folder)
    want = plain.forward(raw, tensors, tokens)
    without = plain.forward(raw, tensors, [t if t != MARK else OTHER for t in tokens])
    moved = float((want[-1] - without[-1]).abs().max() / want[-1].abs().max())
    assert (moved > 0.3) if seen else (moved < 1e-5), f"the mark moves the last logits by {moved:.3f}"
    requests = {"m": tokens}
    n = len(tokens)
    ways = [th.whole(requests), th.prefix_then_single(requests, tail=min(n - 1, 12)), th.portions(requests, (n - 1, 1)),
            th.portions(requests, (5, 2, 16, 3))]
    for steps in ways:
        got = th.collect(steps, run_trace(folder, dtype, 16, steps), requests)["m"]
        assert excess(got[-1:], want[-1:], dtype) <= (1.0 if dtype == "float32" else BF16_OUTLIERS)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mark_at", [0, 1, 15, 16, 17, 128, 230])
def test_a_key_far_back_is_found(tmp_path, dtype, mark_at):
    folder = marked_model(tmp_path / "m", stored_as(dtype), None, None)
    check_marked(folder, dtype, marked_tokens(260, mark_at, mark_at), seen=True)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("length", [WINDOW + KEEP + 3, 3 * WINDOW + 9, 129, 128])
@pytest.mark.parametrize("where", ["window_in", "window_out", "kept_in", "kept_out"])
def test_keys_at_the_edges_of_the_window_and_of_the_kept_tokens(tmp_path, dtype, length, where):
    """The mark at the oldest position the window still holds and one before it; at the last kept position
    and one behind it."""
    folder = marked_model(tmp_path / "m", stored_as(dtype), WINDOW, KEEP)
    mark_at = {"window_in": length - WINDOW, "window_out": length - WINDOW - 1, "kept_in": KEEP - 1, "kept_out": KEEP}[where]
    check_marked(folder, dtype, marked_tokens(length, mark_at, length), seen=where.endswith("in"))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["left", "right"])
def test_what_a_token_left_hundreds_of_tokens_back_still_counts(tmp_path, dtype, which):
    """A parallel layer in which one side carries the output: a token 250 positions back changes the last
    logits (through the cached keys of the left side, through the slowly decaying state of the right),
    and the engine follows it whole, token by token and in portions."""
    sides = (1.0, 1e-3) if which == "left" else (1e-3, 1.0)
    config = {"architecture": "Legavik", "vocab": 40, "width": 32, "norm": {"eps": 1e-5},
              "layers": [lt.layer(lt.parallel(lt.left(2, 1, 16, 16, 3, scale=1.0, temp=(0.5, 32)), lt.right(2, 1, 16, 16, 4, 4, 4), *sides), None)]}
    tensors = lt.draw_tensors(config, 8, torch.float32, 0.25)
    tensors["l0.mix.right.A_log"][:] = -6.0  # decays close to one: the state lasts
    tensors = {name: t.to(stored_as(dtype)).contiguous() for name, t in tensors.items()}
    folder = lt.make_model_dir(tmp_path / "m", config, 0, tensors=tensors)
    raw, loaded = lt.read_model_dir(folder)
    tokens = tokens_of(40, 260, 77)
    changed = list(tokens)
    changed[9] = (tokens[9] + 1) % 40
    want, other = plain.forward(raw, loaded, tokens), plain.forward(raw, loaded, changed)
    moved = float((want[-1] - other[-1]).abs().max() / want[-1].abs().max())
    assert moved > 0.02, f"the early token moves the last logits by {moved:.4f}"
    requests = {"m": tokens}
    for steps in (th.whole(requests), th.prefix_then_single(requests, tail=200), th.portions(requests, (9, 2, 64, 1, 30))):
        got = th.collect(steps, run_trace(folder, dtype, 16, steps), requests)["m"]
        assert excess(got, want, dtype) <= 1.0


# ---------------------------------------------------------------------------------------------
# generation through the engine's own entry point and the command line
# ---------------------------------------------------------------------------------------------


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_engine(tmp_path, name):
    from turboserve_amd.config.engine_config import EngineConfig, SchedulerConfig
    from turboserve_amd.engine.llm_engine import LLMEngine
    from turboserve_amd.sampling.params import SamplingParams

    config, seed, page = lt.TINY[name]
    folder = lt.make_model_dir(tmp_path / "gen", config, seed + 5, torch.float32, std=0.2)
    raw, tensors = lt.read_model_dir(folder)
    prompts = [tokens_of(config["vocab"], n, 900 + n) for n in (3, 21, 1, 50)]
    new = 40
    want = [lt.greedy(raw, tensors, prompt, new) for prompt in prompts]
    engine = LLMEngine(EngineConfig(
        model=str(folder), dtype="float32",
        scheduler=SchedulerConfig(max_num_seqs=4, max_num_batched_tokens=64, block_size=page, num_blocks=40),
    ))
    outputs = engine.generate(prompts, SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
    assert [out.new_token_ids for out in outputs] == want
    # Once more on the same engine: the pages and slots of the first run are used again.
    again = engine.generate(list(reversed(prompts)), SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True))
    assert [out.new_token_ids for out in again] == list(reversed(want))


def test_the_command_line_serves_the_design(tmp_path, capsys):
    """``engine random-model`` writes a folder from a config.json of the design, ``engine generate``
    completes prompts given as token ids with the plain implementation's greedy tokens, and ``engine
    kv-size`` sizes a cache with one group per distinct page geometry."""
    import re

    from turboserve_amd import cli

    config, _, page = lt.TINY["A"]
    source = tmp_path / "config.json"
    source.write_text(json.dumps(config))
    folder = tmp_path / "model"
    assert cli.main(["engine", "random-model", "--config", str(source), "--out", str(folder), "--seed", "4", "--dtype", "float32"]) == 0
    raw, tensors = lt.read_model_dir(folder)
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
