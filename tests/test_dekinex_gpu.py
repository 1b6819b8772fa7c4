"""Dekinex on the device: each mechanism's kernels against the plain implementation, then whole models under every
way of cutting requests into steps, and generation through the entry points."""
from __future__ import annotations

import json
import math
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import helpers
from plain import dekinex as pd
from dekinex_cases import CASES, folder_of, rounded

pytestmark = pytest.mark.gpu
F64 = torch.float64
DEV = "cuda:0"


def _dev(t, dtype=torch.float32):
    return t.to(dtype).to(DEV).contiguous()


def _i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


def _step_ctx(rows, slots, max_q=None):
    """The tables of a step whose requests bring ``rows`` = [(request, first position, end position)], in that order."""
    lens = [b - a for _, a, b in rows]
    starts = np.cumsum([0] + lens)[:-1]
    tok_seq = [s for s, n in enumerate(lens) for _ in range(n)]
    return SimpleNamespace(q_start=_i32(starts), q_len=_i32(lens), pos0=_i32(a for _, a, _ in rows), tok_seq=_i32(tok_seq),
                           state_slots=_i32(slots[r] for r, _, _ in rows), num_seqs=len(rows),
                           host={"max_q_len": max(lens) if max_q is None else max_q})


# ------------------------------------------------------------------------------------------ embedding
def test_the_pair_table_across_steps_and_slots():
    """Three requests in portions: the row of the pair table follows the token before, also across a step's edge, and a
    request that starts anew in a used slot takes the last row."""
    from glassbox_amd import ops
    torch.manual_seed(0)
    vocab, d, buckets, mp, mc = 40, 24, 11, 7, 3
    table, pairs = torch.randn(vocab, d), torch.randn(buckets + 1, d)
    prev = torch.full((5, 1), 33, dtype=torch.int32, device=DEV)
    toks = {0: helpers.random_tokens(vocab, 9, 1), 1: helpers.random_tokens(vocab, 4, 2), 2: helpers.random_tokens(vocab, 6, 3)}
    slots = {0: 3, 1: 0, 2: 4}
    want = {r: table[t].to(F64) + pairs[pd.pair_rows(t, buckets, mp, mc)].to(F64) for r, t in toks.items()}
    for rows in ([(0, 0, 5), (1, 0, 1)], [(1, 1, 2), (0, 5, 6), (2, 0, 6)], [(0, 6, 9), (1, 2, 4)]):
        ctx = _step_ctx(rows, slots)
        ctx.token_ids = _i32(t for r, a, b in rows for t in toks[r][a:b])
        n = sum(b - a for _, a, b in rows)
        out = torch.empty(2, n, d, device=DEV)
        ops.embed_pairs(_dev(table), _dev(pairs), ctx, out, buckets, mp, mc, prev)
        got = out.cpu().to(F64)
        assert torch.equal(got[0], got[1])
        assert torch.allclose(got[0], torch.cat([want[r][a:b] for r, a, b in rows], 0), atol=1e-6)
    assert prev[:, 0].tolist() == [toks[1][-1], 33, 33, toks[0][-1], toks[2][-1]]


# ------------------------------------------------------------------------------------------ convolution, rotation, norm
@pytest.mark.parametrize("H, G, dk, dv, taps, rot, dtype", [
    (4, 2, 16, 24, 4, 8, torch.float32), (3, 1, 10, 6, 3, 4, torch.float32), (2, 2, 64, 64, 2, 64, torch.bfloat16),
    (2, 1, 136, 40, 5, 32, torch.float32), (1, 1, 32, 48, 1, 0, torch.bfloat16), (2, 2, 8, 8, 0, 2, torch.float32),
    (3, 3, 5, 7, 8, 2, torch.float32),
])
def test_convolved_rotated_normed_heads_in_portions(H, G, dk, dv, taps, rot, dtype):
    """Three requests whose tokens come in three steps of unequal portions (single tokens, portions shorter than the
    convolution, long ones) into slots that hold garbage: queries, keys and values against the plain functions, and the
    pages that the kernel wrote."""
    from glassbox_amd import ops
    from glassbox_amd.parts.attention import cache_head_cols
    torch.manual_seed(dk + dv + taps)
    base, eps, page = 100.0, 1e-5, 16
    C, hc = (H + G) * dk + G * dv, cache_head_cols(dk, dv)
    lens = {0: 23, 1: 3, 2: 9}
    cuts = {0: (1, 20, 1, 1), 1: (1, 1, 0, 1), 2: (1, 2, 1, 5)}   # (the first and third steps bring single tokens only)
    slots = {0: 2, 1: 0, 2: 3}
    wconv = torch.randn(C, taps) if taps else None
    state = torch.full((5, max(taps - 1, 1), C), 55.0, device=DEV) if taps > 1 else None
    data, want = {}, {}
    for r, T in lens.items():
        u = torch.randn(T, C).to(dtype).to(F64)
        data[r] = u
        y = pd.short_convolution(u, wconv.to(F64)) if taps else u
        q, k, v = y[:, :H * dk].view(T, H, dk), y[:, H * dk:(H + G) * dk].view(T, G, dk), y[:, (H + G) * dk:].view(T, G, dv)
        q, k = pd.unit_rms(pd.rotate_neighbours(q, rot, base), eps), pd.unit_rms(pd.rotate_neighbours(k, rot, base), eps)
        want[r] = (q, k, v)
    k_pages = torch.zeros(ops.key_pages_shape(8, G, page, hc), dtype=dtype, device=DEV)
    v_pages = torch.zeros(8, G, hc, page, dtype=dtype, device=DEV)
    page_of = {0: [1, 5], 1: [3], 2: [7]}
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    done = {r: 0 for r in lens}
    for step in range(4):
        rows = [(r, done[r], done[r] + cuts[r][step]) for r in lens if cuts[r][step]]
        rows.sort(key=lambda x: x[2] - x[1] > 1)
        ctx = _step_ctx(rows, slots)
        n = sum(b - a for _, a, b in rows)
        positions = [p for _, a, b in rows for p in range(a, b)]
        ang = torch.tensor(positions, dtype=F64)[:, None] * torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64) \
            if rot else None
        cache_rows = _i32(page_of[r][p // page] * page + p % page for r, a, b in rows for p in range(a, b))
        proj = torch.zeros(n, C + 3, dtype=dtype, device=DEV)   # rows wider than their heads
        proj[:, :C] = _dev(torch.cat([data[r][a:b] for r, a, b in rows], 0), dtype)
        out = torch.full((n, (H + 2 * G) * hc), 9.0, dtype=dtype, device=DEV)
        ops.conv_heads(proj, _dev(wconv) if taps else None, state, ctx, _dev(ang.cos()) if rot else None,
                       _dev(ang.sin()) if rot else None, rot, eps, True, out, hc, cache_rows, k_pages, v_pages, H, G, dk, dv)
        got = out.cpu().to(F64).view(n, H + 2 * G, hc)
        at = 0
        for r, a, b in rows:
            q, k, v = want[r]
            part = got[at:at + b - a]
            assert (part[:, :H, :dk] - q[a:b]).abs().max() < tol, ("queries", step, r)
            assert (part[:, H:H + G, :dk] - k[a:b]).abs().max() < tol, ("keys", step, r)
            assert (part[:, H + G:, :dv] - v[a:b]).abs().max() < tol * max(1.0, float(v.abs().max())), ("values", step, r)
            assert float(part[:, :H + G, dk:].abs().max()) == 0.0 if hc > dk else True
            assert float(part[:, H + G:, dv:].abs().max()) == 0.0 if hc > dv else True
            at += b - a
            done[r] = b
    keys = ops.unpack_keys(k_pages).cpu().to(F64)   # [pages, G, page, hc]
    for r, T in lens.items():
        for p in range(T):
            pg, o = page_of[r][p // page], p % page
            assert (keys[pg, :, o, :dk] - want[r][1][p]).abs().max() < tol
            assert (v_pages[pg, :, :dv, o].cpu().to(F64) - want[r][2][p]).abs().max() < tol * max(1.0, float(want[r][2].abs().max()))
    if state is not None:
        assert torch.all(state[1] == 55.0) and torch.all(state[4] == 55.0)   # nobody else's slot was touched
        for r, T in lens.items():
            kept = state[slots[r]].cpu().to(F64)
            for i in range(taps - 1):
                p = T - (taps - 1) + i
                if p >= 0:
                    assert torch.equal(kept[i], data[r][p])


@pytest.mark.parametrize("H, G, dk, dv, taps, rot, times", [
    (4, 2, 64, 64, 4, 32, 1), (2, 1, 128, 80, 3, 128, 1), (3, 3, 16, 24, 8, 6, 1), (2, 2, 72, 40, 1, 0, 1), (5, 1, 32, 48, 0, 10, 1),
    (1, 1, 24, 8, 2, 24, 1), (32, 32, 64, 64, 4, 8, 14)])   # (the last: enough rows and heads for eight rows a lane)
def test_steps_of_many_rows_take_eight_channels_a_lane(H, G, dk, dv, taps, rot, times):
    """Steps of more than 64 rows in bfloat16 whose heads are whole groups of eight channels, without the cache write:
    two steps, requests that begin, one that goes on from its slot (its first rows read the slot), into slots that held
    garbage; against the plain functions, and the slots after each step."""
    from glassbox_amd import ops
    from glassbox_amd.parts.attention import cache_head_cols
    torch.manual_seed(dk + dv + taps)
    base, eps, dtype = 100.0, 1e-5, torch.bfloat16
    C, hc = (H + G) * dk + G * dv, cache_head_cols(dk, dv)
    m = times
    lens = {0: 110 * m + 3, 1: 30 * m, 2: 50 * m}
    steps = [[(0, 0, 70 * m + 1), (1, 0, 30 * m)], [(0, 70 * m + 1, 110 * m + 3), (2, 0, 50 * m)]]
    slots = {0: 2, 1: 0, 2: 3}
    wconv = torch.randn(C, taps) if taps else None
    state = torch.full((5, max(taps - 1, 1), C), 55.0, device=DEV) if taps > 1 else None
    data, want = {}, {}
    for r, T in lens.items():
        u = torch.randn(T, C).to(dtype).to(F64)
        data[r] = u
        y = pd.short_convolution(u, wconv.to(F64)) if taps else u
        q, k, v = y[:, :H * dk].view(T, H, dk), y[:, H * dk:(H + G) * dk].view(T, G, dk), y[:, (H + G) * dk:].view(T, G, dv)
        want[r] = (pd.unit_rms(pd.rotate_neighbours(q, rot, base), eps), pd.unit_rms(pd.rotate_neighbours(k, rot, base), eps), v)
    for rows in steps:
        ctx = _step_ctx(rows, slots)
        n = sum(b - a for _, a, b in rows)
        assert n > 64
        positions = [p for _, a, b in rows for p in range(a, b)]
        ang = torch.tensor(positions, dtype=F64)[:, None] * torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64) \
            if rot else None
        proj = torch.zeros(n, C + 8, dtype=dtype, device=DEV)   # rows wider than their heads
        proj[:, :C] = _dev(torch.cat([data[r][a:b] for r, a, b in rows], 0), dtype)
        out = torch.full((n, (H + 2 * G) * hc), 9.0, dtype=dtype, device=DEV)
        ops.conv_heads(proj, _dev(wconv) if taps else None, state, ctx, _dev(ang.cos()) if rot else None,
                       _dev(ang.sin()) if rot else None, rot, eps, True, out, hc, None, None, None, H, G, dk, dv)
        got = out.cpu().to(F64).view(n, H + 2 * G, hc)
        at = 0
        for r, a, b in rows:
            q, k, v = want[r]
            part = got[at:at + b - a]
            assert (part[:, :H, :dk] - q[a:b]).abs().max() < 2e-2, ("queries", r, a)
            assert (part[:, H:H + G, :dk] - k[a:b]).abs().max() < 2e-2, ("keys", r, a)
            assert (part[:, H + G:, :dv] - v[a:b]).abs().max() < 2e-2 * max(1.0, float(v.abs().max())), ("values", r, a)
            assert float(part[:, :H + G, dk:].abs().max()) == 0.0 if hc > dk else True
            assert float(part[:, H + G:, dv:].abs().max()) == 0.0 if hc > dv else True
            at += b - a
            if state is not None:
                kept = state[slots[r]].cpu().to(F64)
                assert all(torch.equal(kept[i], data[r][b - (taps - 1) + i]) for i in range(taps - 1))


# ------------------------------------------------------------------------------------------ the matrix memory
def _memory_case(H, dk, dv, lens, seed, vtype=torch.float32, far=False):
    torch.manual_seed(seed)
    out = {}
    for r, T in lens.items():
        q, k = torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dk, dtype=F64)
        v = torch.randn(T, H, dv, dtype=F64)
        zi, zf = torch.randn(T, H, dtype=F64) * 3, torch.randn(T, H, dtype=F64) * 2 + (7.0 if far else 2.0)
        if far:
            zi[3] = 12.0     # one early token that outweighs hundreds after it
        q, k, v, zi, zf = (t.float().to(F64) for t in (q, k, v, zi, zf))
        q, k, v = (t.to(vtype).to(F64) for t in (q, k, v))   # (what the projection's rows hold)
        out[r] = (q, k, v, zi, zf)
    return out


def _run_memory(ops, data, rows, slots, state, H, dk, dv, cap, bias_i, bias_f, vtype, segments_expected=None):
    """One step of gates, operands, recurrence and output division through the kernels; returns y = o / denominator."""
    ctx = _step_ctx(rows, slots)
    n = sum(b - a for _, a, b in rows)
    cat = lambda i: torch.cat([data[r][i][a:b] for r, a, b in rows], 0)
    proj = torch.zeros(n, 2 * H * dk + 2 * H * dv, dtype=vtype, device=DEV)
    proj[:, :H * dk], proj[:, H * dk:2 * H * dk] = _dev(cat(0).reshape(n, -1), vtype), _dev(cat(1).reshape(n, -1), vtype)
    proj[:, 2 * H * dk:2 * H * dk + H * dv] = _dev(cat(2).reshape(n, -1), vtype)
    proj[:, 2 * H * dk + H * dv:] = 50.0     # the gate: sigmoid = 1
    z = _dev(torch.cat([cat(3) - bias_i, cat(4) - bias_f], 1))
    coef = torch.empty(n, H, 3, device=DEV)
    ops.mlstm_gates(z, _dev(bias_i), _dev(bias_f), cap, coef, state, dv + 1, ctx, H)
    q32, k32 = torch.empty(n, H * dk, device=DEV), torch.empty(n, H * dk, device=DEV)
    decay, vext = torch.empty(n, H, device=DEV), torch.empty(n, H * (dv + 1), dtype=vtype, device=DEV)
    ops.mlstm_prep(proj, 0, H * dk, 2 * H * dk, coef, q32, k32, decay, vext, H, dk, dv, 0.5)
    o = torch.empty(n, H * (dv + 1), device=DEV)
    segments = ops.linear_scan_segments(max(b - a for _, a, b in rows))
    if segments_expected is not None:
        assert segments == segments_expected
    ws = torch.full((len(rows) * segments * H * (dv + 2) * dk,), float("nan"), device=DEV) if segments > 1 else None
    ops.linear_scan(q32, k32, vext, o, state, ctx, H, dk, dv + 1, token_decay=decay, segments=segments, workspace=ws)
    gated = torch.empty(n, H * dv, dtype=vtype, device=DEV)
    ops.mlstm_out(o, coef, proj[:, 2 * H * dk + H * dv:], None, gated, H, dv, 1e-6)
    return gated.cpu().to(F64).view(n, H, dv)


@pytest.mark.parametrize("H, dk, dv, cap, vtype", [(2, 24, 40, 10.0, torch.float32), (1, 64, 32, 20.0, torch.bfloat16),
                                                   (5, 6, 10, 3.0, torch.float32), (2, 128, 96, 8.0, torch.float32),
                                                   (3, 8, 16, 5.0, torch.float32)])
def test_the_matrix_memory_in_portions_of_a_batch(H, dk, dv, cap, vtype):
    """Three requests in four steps of unequal portions (the last of single tokens only, which one gate kernel serves),
    slots full of garbage: every head's normed output against the plain recurrence (which the output kernel's norm leaves
    comparable whatever the head's size)."""
    from glassbox_amd import ops
    lens = {0: 71, 1: 4, 2: 30}
    cuts = {0: (1, 64, 5, 1), 1: (1, 1, 1, 1), 2: (27, 1, 1, 1)}
    slots = {0: 2, 1: 0, 2: 3}
    data = _memory_case(H, dk, dv, lens, dk * dv, vtype)
    bias_i, bias_f = torch.linspace(-1, 1, H, dtype=F64), torch.linspace(0.5, 2, H, dtype=F64)
    want = {}
    for r, (q, k, v, zi, zf) in data.items():
        i, f = pd.capped_gates(zi, zf, cap)
        want[r] = pd.unit_rms(pd.matrix_memory_outputs(q * 0.5, k, v, i, f), 1e-6)
    state = torch.full((5, H, dv + 2, dk), 77.0, device=DEV)
    done = {r: 0 for r in lens}
    tol = 3e-5 if vtype == torch.float32 else 2e-2
    for step in range(4):
        rows = [(r, done[r], done[r] + cuts[r][step]) for r in lens]
        got = _run_memory(ops, data, rows, slots, state, H, dk, dv, cap, bias_i, bias_f, vtype)
        at = 0
        for r, a, b in rows:
            err = (got[at:at + b - a] - want[r][a:b]).abs().max().item()
            assert err < tol, (step, r, err)
            at += b - a
            done[r] = b
    assert torch.all(state[1] == 77.0) and torch.all(state[4] == 77.0)


def test_an_early_token_outlives_hundreds_in_the_matrix_memory_and_long_portions_run_as_segments():
    """Forget gates near one and one early token with a huge input gate: the outputs 600 tokens later still rest on it.
    The prompt comes whole (cut into segments that a second kernel joins), then in long portions behind a short one."""
    from glassbox_amd import ops
    H, dk, dv, cap = 2, 32, 48, 15.0
    lens = {0: 640, 1: 300}
    data = _memory_case(H, dk, dv, lens, 5, far=True)
    zero = torch.zeros(H, dtype=F64)
    want = {}
    for r, (q, k, v, zi, zf) in data.items():
        i, f = pd.capped_gates(zi, zf, cap)
        want[r] = pd.unit_rms(pd.matrix_memory_outputs(q * 0.5, k, v, i, f), 1e-6)
        gone = pd.capped_gates(torch.cat([zi[:3], zi[3:4] - 30, zi[4:]]), zf, cap)[0]
        other = pd.unit_rms(pd.matrix_memory_outputs(q * 0.5, k, v, gone, f), 1e-6)
        assert (other[-1] - want[r][-1]).abs().max() > 0.1      # the early token matters at the end
    for cuts in ({0: (640,), 1: (300,)}, {0: (2, 300, 338), 1: (1, 299, 0)}):
        state = torch.full((3, H, dv + 2, dk), -3.0, device=DEV)
        done = {r: 0 for r in lens}
        for step in range(len(cuts[0])):
            rows = [(r, done[r], done[r] + cuts[r][step]) for r in lens if cuts[r][step]]
            got = _run_memory(ops, data, rows, {0: 1, 1: 2}, state, H, dk, dv, cap, zero, zero, torch.float32)
            at = 0
            for r, a, b in rows:
                err = (got[at:at + b - a] - want[r][a:b]).abs().max().item()
                assert err < 1e-4, (cuts[0], step, r, err)
                at += b - a
                done[r] = b
        assert torch.all(state[0] == -3.0)


# ------------------------------------------------------------------------------------------ feed-forwards
def test_the_router_and_the_gated_units():
    from glassbox_amd import ops
    torch.manual_seed(7)
    for E, top, shared, scale in ((6, 2, True, 1.5), (3, 1, False, 1.0), (2, 2, True, 0.7), (70, 4, False, 2.0), (5, 3, True, 2.5)):
        n, ff, sff = 37, 4, 3 if shared else 0
        z = torch.randn(n, E + (1 if shared else 0), dtype=F64) * 2
        z[0, :E] = 0.0                      # equal scores: the lower index wins
        z[1, :E] = torch.arange(E, dtype=F64) * 0.01
        corr = torch.randn(E, dtype=F64) * 0.5
        z, corr = z.float().to(F64), corr.float().to(F64)
        cols = E + (1 if shared else 0)
        combine, ids, wts = torch.empty(n, cols, device=DEV), torch.empty(n, top, dtype=torch.int32, device=DEV), torch.empty(n, top, device=DEV)
        ops.moe_route(_dev(z), E, _dev(corr), top, scale, shared, combine, ids, wts)
        inter = E * ff + sff
        gu = torch.randn(n, 2 * inter, dtype=F64).float()
        act = torch.empty(n, inter, device=DEV)
        ops.moe_gated_units(_dev(gu), combine, act, E, ff)
        gu = gu.to(F64)
        for t in range(n):
            chosen, weights = pd.route(z[t, :E], corr, top, scale)
            if t > 1:   # (rows 0 and 1 are near ties in 32-bit)
                assert ids[t].tolist() == chosen
            assert sorted(ids[t].tolist()) == sorted(chosen) or t <= 1
            if t == 0:
                assert sorted(ids[t].tolist()) == sorted(sorted(range(E), key=lambda e: (-float(corr[e]), e))[:top])
            row = torch.zeros(cols, dtype=F64)
            if t > 1:
                row[chosen] = weights
                if shared:
                    row[E] = torch.sigmoid(z[t, E])
                assert torch.allclose(combine[t].cpu().to(F64), row, atol=1e-6)
                assert torch.allclose(wts[t].cpu().to(F64), weights, atol=1e-6)
                # the experts' gate columns, their up columns, then the shared expert's gate and up columns
                g = torch.cat([gu[t, :E * ff], gu[t, 2 * E * ff:2 * E * ff + sff]])
                u = torch.cat([gu[t, E * ff:2 * E * ff], gu[t, 2 * E * ff + sff:]])
                per = torch.cat([row[:E].repeat_interleave(ff), row[E:].repeat_interleave(sff)]) if shared else row.repeat_interleave(ff)
                assert torch.allclose(act[t].cpu().to(F64), g * torch.sigmoid(g) * u * per, atol=1e-5)


def test_entries_sorted_by_expert_and_cut_into_tiles():
    from glassbox_amd import ops
    gen = torch.Generator().manual_seed(3)
    for n, top, E, tile_rows in ((300, 2, 6, 64), (77, 1, 3, 64), (1000, 4, 9, 128), (130, 3, 70, 64), (64, 2, 2, 128)):
        ids = torch.stack([torch.randperm(E, generator=gen)[:top] for _ in range(n)]).to(torch.int32)
        if E > 4:
            ids[ids == 1] = 0            # an expert that no token chooses
        tiles = ops.moe_sort_tiles(n * top, E, tile_rows)
        counts = torch.empty(E, dtype=torch.int32, device=DEV)
        rows = torch.full((n * top,), -7, dtype=torch.int32, device=DEV)
        pos = torch.full((n, top), -7, dtype=torch.int32, device=DEV)
        tile_map = torch.full((tiles, 3), -7, dtype=torch.int32, device=DEV)
        ops.moe_sort(ids.to(DEV), E, tile_rows, counts, rows, pos, tile_map)
        flat = ids.flatten().tolist()
        order = sorted(range(n * top), key=lambda i: (flat[i], i))      # by expert, entries of one in their own order
        assert rows.tolist() == [i // top for i in order]
        assert [pos.flatten().tolist()[i] for i in order] == list(range(n * top))
        want, at = [], 0
        for e in range(E):
            c = flat.count(e)
            want += [[e, at + j, at + c] for j in range(0, c, tile_rows)]
            at += c
        got = tile_map.tolist()
        assert got[:len(want)] == want and all(t[0] == -1 for t in got[len(want):]) and len(want) <= tiles


@pytest.mark.parametrize("n, d, E, top, ff, sff", [(300, 64, 6, 2, 16, 32), (129, 96, 3, 1, 24, 0), (700, 128, 16, 2, 64, 8),
                                                  (1100, 72, 9, 4, 8, 24)])
def test_experts_on_their_own_tokens_alone(n, d, E, top, ff, sff):
    """A step of many tokens sorts them by expert; the same step through every expert (in two halves of few enough
    tokens) and the plain implementation give the same rows.  One expert's down matrix is a hundred times the others',
    so that a row that went to the wrong expert, or came back to the wrong token, shows."""
    from glassbox_amd.engine.context import Workspace
    from glassbox_amd.parts.moe import RoutedExperts
    gen = torch.Generator().manual_seed(n + E)
    part = RoutedExperts(d, E, top, ff, 1.7, sff)
    w = {}
    for name, spec in part.tensor_specs().items():
        t = torch.randn(spec.shape, generator=gen) * (0.5 if name in ("router", "shared.sg") else d ** -0.5)
        w[name] = t.to(torch.bfloat16) if len(spec.shape) == 2 else t * 0.1
    w["e1.down"] = (w["e1.down"].float() * 100).to(torch.bfloat16)
    part.load({k: v.to(DEV) for k, v in w.items()})
    h = (torch.randn(n, d, generator=gen)).to(torch.bfloat16)
    ctx = SimpleNamespace(dtype=torch.bfloat16, workspace=Workspace(DEV))
    ctx.buffer = ctx.workspace.buffer
    assert part.routed(ctx, n) and not part.routed(ctx, 40)
    out = torch.full((n, d), 3.0, device=DEV)
    part.forward(ctx, h.to(DEV), out, store=True)
    again = torch.full((n, d), 1.0, device=DEV)
    part.forward(ctx, h.to(DEV), again, store=False)
    assert torch.equal(again - 1.0 - out, torch.zeros_like(out)) or float((again - 1.0 - out).abs().max()) < 1e-5 * float(out.abs().max())
    small = torch.empty(n, d, device=DEV)
    for a in range(0, n, 40):
        part.forward(ctx, h[a:a + 40].to(DEV), small[a:a + 40], store=True)
    wp = {"p." + k: v.to(F64) for k, v in w.items()}
    mlp = {"router": {"experts": E, "top": top, "scale": 1.7}, "shared": {"ff": sff} if sff else None}
    ref = pd.routed_experts(wp, "p.", mlp, h.to(F64), r=pd.bf16)
    scale = float(ref.abs().max())
    # a token whose choice hangs on the rounding of the router's sums may differ from the plain choice; both kernels'
    # paths read the same choice
    assert float((out.cpu().to(F64) - small.cpu().to(F64)).abs().max()) < 2e-2 * scale
    close = ((out.cpu().to(F64) - ref).abs().amax(1) < 2e-2 * scale)
    assert int(close.sum()) >= n - max(2, n // 100)


@pytest.mark.parametrize("n, d, ff, limit", [(1, 64, 40, 0.7), (8, 96, 72, 2.0), (37, 128, 1000, 1.5), (65, 64, 40, 0.7), (300, 96, 72, 2.0),
                                            (2048, 64, 3072, 1.0)])
def test_the_clamped_unit_where_the_products_tiles_are_finished(n, d, ff, limit):
    """The unit is applied in the product's kernel: the kernel of few rows, the tiled one, and (the last case) the one
    of the largest tiles; the gate's sums are spread so that many lie beyond the limit on either side."""
    from glassbox_amd import ops
    gen = torch.Generator().manual_seed(n)
    h = torch.randn(n, d, generator=gen).to(torch.bfloat16)
    w = (torch.randn(2 * ff, d, generator=gen) * 2.0 * d ** -0.5).to(torch.bfloat16)
    act = torch.empty(n, ff, dtype=torch.bfloat16, device=DEV)
    ops.gemm_glu(h.to(DEV), w.to(DEV), act, limit, 1.702)
    gu = h.to(F64) @ w.to(F64).t()
    g, u = gu[:, :ff].clamp(max=limit), gu[:, ff:].clamp(-limit, limit)
    want = g * torch.sigmoid(1.702 * g) * (u + 1)
    assert float((gu[:, :ff] > limit).double().mean()) > 0.05 and float((gu[:, ff:] < -limit).double().mean()) > 0.05
    assert float((act.cpu().to(F64) - want).abs().max()) < 1e-2 * float(want.abs().max())


def test_the_clamped_unit_and_the_scaled_add():
    from glassbox_amd import ops
    torch.manual_seed(8)
    n, inter = 19, 30
    gu = (torch.randn(n, 2 * inter) * 2)
    for limit in (0.3, 1.5):
        g, u = gu[:, :inter].to(F64).clamp(max=limit), gu[:, inter:].to(F64).clamp(-limit, limit)
        want = g * torch.sigmoid(1.702 * g) * (u + 1)
        act = torch.empty(n, inter, device=DEV)
        ops.glu_clamped(_dev(gu), act, limit, 1.702)
        assert torch.allclose(act.cpu().to(F64), want, atol=1e-6)
        act16 = torch.empty(n, inter, dtype=torch.bfloat16, device=DEV)
        ops.glu_clamped(_dev(gu), act16, limit, 1.702)
        assert torch.allclose(act16.cpu().to(F64), want, atol=2e-2)
    x, y, b = torch.randn(n, inter), torch.randn(n, inter), torch.randn(inter)
    xd = _dev(x)
    ops.axpy_rows(xd, _dev(y), 0.3)
    ops.axpy_rows(xd, None, 1.0, _dev(b))
    ops.axpy_rows(xd, _dev(y), 1.0, _dev(b))
    assert torch.allclose(xd.cpu(), x + 0.3 * y + b + y + b, atol=1e-6)


# ------------------------------------------------------------------------------------------ whole models
REQUESTS = {"a": 150, "b": 77, "c": 41, "d": 3, "e": 1, "f": 97}


def _requests(vocab: int, seed: int = 0):
    return {r: helpers.random_tokens(vocab, n, seed=seed + n) for r, n in REQUESTS.items()}


_ORACLE: dict = {}


def _want(folder: str, tokens, dtype: str) -> np.ndarray:
    key = (folder, tuple(tokens), dtype)
    if key not in _ORACLE:
        cfg, w = pd.load_folder(folder)
        _ORACLE[key] = pd.forward(rounded(w) if dtype == "bfloat16" else w, cfg, list(tokens)).numpy()
    return _ORACLE[key]


def _moved_by_rounding(folder: str, tokens) -> np.ndarray:
    """How far rounding the activations to bfloat16 moves each position's logits in the plain implementation (root mean
    square over the vocabulary): what a position's sensitivity to rounding is."""
    key = (folder, tuple(tokens), "moved")
    if key not in _ORACLE:
        cfg, w = pd.load_folder(folder)
        coarse = pd.forward(rounded(w), cfg, list(tokens), coarse=True).numpy()
        _ORACLE[key] = np.sqrt(((coarse - _want(folder, tokens, "bfloat16")) ** 2).mean(1))
    return _ORACLE[key]


#: A 32-bit engine is held to helpers.TOL_F32 of the request's largest logit at every position.  A bfloat16 engine is
#: compared with the plain implementation on the weights it holds by the root mean square of a position's logit
#: differences: at most 3 times what rounding the activations moves that position in the plain implementation itself
#: (with random weights the matrix memory's normed heads make some positions ten times as sensitive as others), or
#: 1 % of the request's logits' root mean square where that is more.  One sample of rounding is no sharp bound on
#: another: no position may be beyond one and a half times its limit, and one in fifty beyond the limit itself.
BF16_TIMES, BF16_FLOOR = 3.0, 1e-2


def _check(got, folder, requests, dtype, what):
    for r, toks in requests.items():
        want = _want(folder, toks, dtype)
        if dtype == "float32":
            tol = helpers.TOL_F32 * max(1.0, float(np.abs(want).max()))
            bad = helpers.first_bad(got[r], want, tol)
            assert bad is None, f"{what}, {dtype}, request {r} ({len(toks)} tokens): position {bad[0]} is {bad[1]:.3e} off (limit {tol:.3e})"
            continue
        err = np.sqrt(((got[r] - want) ** 2).mean(1))
        lim = np.maximum(BF16_TIMES * _moved_by_rounding(folder, toks), BF16_FLOOR * float(np.sqrt((want ** 2).mean())))
        over = np.nonzero(err > lim)[0]
        assert over.size <= max(1, len(toks) // 50) and float((err / lim).max()) <= 1.5, (f"{what}, {dtype}, request {r} ({len(toks)} tokens): position {over[0]} is {err[over[0]]:.3e} off "
                                f"(limit {lim[over[0]]:.3e}); {over.size} positions over their limits, worst ratio {(err / lim).max():.2f}")


def _poison(engine) -> None:
    """Garbage in every page and state slot: whatever a request reads, it must have written itself."""
    for lc in engine.layers:
        for t in (lc.k_pages, lc.v_pages, lc.state):
            if t is not None:
                t.fill_(300 if t.dtype == torch.int32 else 300.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
def test_every_way_of_cutting_requests_into_steps(model_dirs, name, dtype):
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, name, steady=dtype == "bfloat16")
    requests = _requests(CASES[name]["vocab"])
    mixed, peak = helpers.schedule_mixed(requests, seed=3, live=3, tail=20)
    eng = Engine(folder, dtype=dtype, max_tokens=max(peak, 192), max_seqs=3)
    _poison(eng)
    for what, steps in (("whole", helpers.schedule_whole(requests)), ("last tokens one by one", helpers.schedule_tail(requests, 60)),
                        ("portions", helpers.schedule_chunks(requests)), ("portions of two", None), ("mixed batches", mixed)):
        if what == "portions of two":
            steps = helpers.schedule_chunks({r: t for r, t in requests.items() if len(t) < 80}, (2,))
        got = helpers.replay(eng, steps)
        _check(got, folder, {r: requests[r] for r in got}, dtype, what)
        assert eng.cache.num_seqs() == 0 and eng.cache.free_state_slots() == 3
        assert all(eng.cache.used_pages(g) == 0 for g in range(len(eng.group_keys)))
        eng.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_whole_and_in_long_portions(model_dirs, dtype):
    """A prompt of 700 tokens: the matrix memory cuts it into segments, attention crosses its window many times."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "A", steady=dtype == "bfloat16")
    requests = {"long": helpers.random_tokens(211, 700, seed=23), "short": helpers.random_tokens(211, 40, seed=22)}
    eng = Engine(folder, dtype=dtype, max_tokens=1024, max_seqs=2)
    _poison(eng)
    for what, steps in (("whole", helpers.schedule_whole(requests)), ("long portions", helpers.schedule_chunks(requests, (300, 1, 399))),
                        ("a long portion beside single tokens", [
                            {"entries": [("short", requests["short"][:39], list(range(39)))], "end": []},
                            {"entries": [("long", requests["long"], list(range(700))), ("short", requests["short"][39:], [0])],
                             "end": ["long", "short"]}])):
        got = helpers.replay(eng, steps)
        _check(got, folder, requests, dtype, what)


def test_the_pool_of_a_windowed_model_holds_windows_not_requests(model_dirs):
    """A request far longer than the pool: every attention layer of the model has a window, whose pages are all it
    holds, and pages that the window has passed are given to the positions after them."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "D")
    toks = helpers.random_tokens(160, 330, seed=9)
    eng = Engine(folder, dtype="float32", max_tokens=160, max_seqs=1)   # ten pages; a window of 50 and a portion of 33 need up to seven
    got = helpers.replay(eng, helpers.schedule_chunks({"long": toks}, (33, 1, 1, 16, 5)))
    _check(got, folder, {"long": toks}, "float32", "a request longer than the pool")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_layers_replayed_from_the_first_of_their_kind(model_dirs, dtype):
    """250 tokens one by one after a prompt of four (windows and pages' edges pass many times over; in bfloat16 the
    steps are replayed from graphs), with the layers of a kind replayed and with every layer walked: the same bits."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "A", steady=dtype == "bfloat16")
    toks = helpers.random_tokens(211, 254, seed=11)
    steps = helpers.schedule_tail({"x": toks}, 250)
    outs = []
    for tapes in (True, False):
        eng = Engine(folder, dtype=dtype, max_tokens=320, max_seqs=2, layer_tapes=tapes)
        outs.append(helpers.replay(eng, steps)["x"])
        if dtype == "bfloat16" and tapes:
            assert eng.decode_graphs is not None and eng.decode_graphs.replays > 200
    _check({"x": outs[0]}, folder, {"x": toks}, dtype, "long decoding")
    assert np.array_equal(outs[0], outs[1])


def test_slots_and_pages_that_are_used_again(model_dirs):
    """Two slots, six requests one after the other in pairs: a request finds the slot (matrix memory, convolution's
    tail, token before) and the pages of one that ended, and must start from nothing."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "A")
    requests = {r: helpers.random_tokens(211, n, seed=70 + n) for r, n in {"p": 50, "q": 31, "r": 18, "s": 64, "t": 2, "u": 45}.items()}
    eng = Engine(folder, dtype="float32", max_tokens=128, max_seqs=2)
    steps, _ = helpers.schedule_mixed(requests, seed=5, live=2, tail=6)
    got = helpers.replay(eng, steps)
    _check(got, folder, requests, "float32", "slots used again")


# ------------------------------------------------------------------------------------------ generation
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_points(model_dirs, name):
    from glassbox_amd.engine import Engine, generate, greedy
    folder = folder_of(model_dirs.base, name, seed=2)
    cfg, w = pd.load_folder(folder)
    vocab = CASES[name]["vocab"]
    prompts = [helpers.random_tokens(vocab, n, seed=50 + n) for n in (5, 44, 1, 23, 70)]
    want = [pd.greedy(w, cfg, p, 12) for p in prompts]
    assert any(len(set(r)) > 2 for r in want), "replies that repeat one token show nothing"
    eng = Engine(folder, dtype="float32", max_tokens=1024, max_seqs=3)
    assert greedy(eng, prompts[1], 12) == want[1]
    # the scheduler: three live requests at most, prompts in portions of at most 16 tokens beside decoding requests
    assert generate(eng, prompts, max_tokens=12, token_budget=16, max_seqs=3) == want
    assert eng.cache.num_seqs() == 0 and eng.cache.free_state_slots() == 3


def test_the_command_line_runs_the_model(model_dirs, tmp_path):
    folder = folder_of(model_dirs.base, "B", seed=2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = lambda *args, stdin=None: subprocess.run([sys.executable, os.path.join(root, "bin", "glassbox"), *args],
                                                   capture_output=True, text=True, timeout=600, input=stdin)
    r = run("generate", "--model", folder, "--prompt", "5,17,3,99,41", "-n", "8", "--dtype", "float32", "--no-prefix-cache")
    assert r.returncode == 0, r.stderr
    cfg, w = pd.load_folder(folder)
    assert [int(t) for t in r.stdout.split()] == pd.greedy(w, cfg, [5, 17, 3, 99, 41], 8)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3, 9], "want": [1, 3]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [8], "want": [0]}, {"id": "b", "tokens": [4, 4], "want": []}], "end": ["a"]}]
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(tmp_path / "o"),
                        "--max-tokens", "128"], capture_output=True, text=True, timeout=600,
                       input="".join(json.dumps(s) + "\n" for s in steps))
    assert r.returncode == 0 and r.stdout.split() == ["done", "0", "done", "1"], r.stderr
    want = pd.forward(w, cfg, [5, 17, 3, 9, 8]).numpy()
    assert np.abs(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1) - want[[1, 3]]).max() < 1e-4
    assert np.abs(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4") - want[4]).max() < 1e-4
