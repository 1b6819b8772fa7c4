"""Sagalorn on the device: each mechanism's kernels against the plain implementation, then whole models under
every way of cutting requests into steps, and generation through the entry points."""
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
from plain import sagalorn as ps
from sagalorn_cases import CASES, folder_of, rounded

pytestmark = pytest.mark.gpu
F64 = torch.float64
DEV = "cuda:0"


def _dev(t, dtype=torch.float32):
    return t.to(dtype).to(DEV).contiguous()


def _i32(values):
    return torch.tensor(list(values), dtype=torch.int32, device=DEV)


# ------------------------------------------------------------------------------------------ the recurrence
@pytest.mark.parametrize("H, dk, dv, gated, vtype", [
    (2, 64, 64, False, torch.float32), (3, 24, 40, True, torch.float32), (1, 128, 33, True, torch.bfloat16),
    (4, 6, 10, False, torch.bfloat16), (2, 200, 70, True, torch.float32), (5, 16, 16, False, torch.float32),
])
def test_the_recurrence_in_portions_of_a_batch(H, dk, dv, gated, vtype):
    """Three requests: their tokens come in two steps of unequal portions (one token, many), in slots that hold
    garbage, rows of the batch in another order than the slots; every output against the plain recurrence."""
    from glassbox_amd import ops
    torch.manual_seed(dk + dv)
    lens = [37, 1, 19]
    cuts = [(20, 17), (1, 0), (1, 18)]
    slots = [2, 0, 3]
    state = torch.full((5, H, dv, dk), 123.0, device=DEV)
    data = []
    for T in lens:
        q, k = torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dk, dtype=F64) / math.sqrt(dk)
        v = torch.randn(T, H, dv, dtype=F64).to(vtype).to(F64)
        decay = torch.rand(T, H, dk, dtype=F64) * 0.3 + 0.7 if gated else (torch.linspace(0.8, 0.999, H, dtype=F64)
                                                                          .view(1, H, 1).expand(T, H, dk))
        q, k, decay = (t.float().to(F64) for t in (q, k, decay))
        data.append((q, k, v, decay, ps.decayed_state_outputs(q, k, v, decay)))
    done = [0, 0, 0]
    for step in range(2):
        rows = [(s, done[s], done[s] + cuts[s][step]) for s in range(3) if cuts[s][step]]
        cat = lambda i: torch.cat([data[s][i][a:b] for s, a, b in rows], 0)
        n = sum(b - a for _, a, b in rows)
        starts = np.cumsum([0] + [b - a for _, a, b in rows])[:-1]
        ctx = SimpleNamespace(q_start=_i32(starts), q_len=_i32(b - a for _, a, b in rows), pos0=_i32(a for _, a, _ in rows),
                              state_slots=_i32(slots[s] for s, _, _ in rows), num_seqs=len(rows))
        wide = torch.zeros(n, H * dv + 8, dtype=vtype, device=DEV)   # the values are a view into wider rows
        wide[:, 8:] = _dev(cat(2).reshape(n, H * dv), vtype)
        out = torch.empty(n, H * dv, device=DEV)
        head_decay = None if gated else _dev(data[0][3][0, :, 0])
        ops.linear_scan(_dev(cat(0).reshape(n, H * dk)), _dev(cat(1).reshape(n, H * dk)), wide[:, 8:], out, state, ctx, H, dk, dv,
                        decay=_dev(cat(3).reshape(n, H * dk)) if gated else None, head_decay=head_decay)
        want = cat(4).reshape(n, H * dv)
        err = (out.cpu().to(F64) - want).abs().max().item()
        assert err <= 2e-5 * max(1.0, want.abs().max().item()), (step, err)
        for s, _, b in rows:
            done[s] = b
    assert torch.all(state[1] == 123.0) and torch.all(state[4] == 123.0)   # nobody else's slot was touched


@pytest.mark.parametrize("H, dk, dv, gated", [(2, 64, 64, False), (3, 24, 40, True), (1, 128, 16, True), (2, 16, 70, False)])
def test_long_portions_run_as_segments(H, dk, dv, gated):
    """Portions beyond 256 rows are cut into segments that run side by side and are joined by a second kernel: three
    requests (one goes on from a state, one is too short to be cut, one brings a single token and then a long portion)
    against the plain recurrence, and the states they leave by going on token after token."""
    from glassbox_amd import ops
    torch.manual_seed(dk * dv)
    lens = [700, 130, 301]
    cuts = [(400, 299, 1), (130, 0, 0), (1, 299, 1)]
    slots = [1, 3, 0]
    state = torch.full((4, H, dv, dk), -7.0, device=DEV)
    data = []
    for T in lens:
        q, k = torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dk, dtype=F64) / math.sqrt(dk)
        v = torch.randn(T, H, dv, dtype=F64)
        decay = torch.rand(T, H, dk, dtype=F64) * 0.1 + 0.9 if gated else (torch.linspace(0.95, 0.999, H, dtype=F64)
                                                                          .view(1, H, 1).expand(T, H, dk))
        q, k, v, decay = (t.float().to(F64) for t in (q, k, v, decay))
        data.append((q, k, v, decay, ps.decayed_state_outputs(q, k, v, decay)))
    done = [0, 0, 0]
    for step in range(3):
        rows = [(s, done[s], done[s] + cuts[s][step]) for s in range(3) if cuts[s][step]]
        cat = lambda i: torch.cat([data[s][i][a:b] for s, a, b in rows], 0)
        n = sum(b - a for _, a, b in rows)
        starts = np.cumsum([0] + [b - a for _, a, b in rows])[:-1]
        ctx = SimpleNamespace(q_start=_i32(starts), q_len=_i32(b - a for _, a, b in rows), pos0=_i32(a for _, a, _ in rows),
                              state_slots=_i32(slots[s] for s, _, _ in rows), num_seqs=len(rows))
        segments = ops.linear_scan_segments(max(b - a for _, a, b in rows))
        assert segments == (4, 3, 1)[step]
        ws = torch.full((len(rows) * segments * H * (dv + 1) * dk,), float("nan"), device=DEV) if segments > 1 else None
        out = torch.empty(n, H * dv, device=DEV)
        ops.linear_scan(_dev(cat(0).reshape(n, -1)), _dev(cat(1).reshape(n, -1)), _dev(cat(2).reshape(n, -1)), out, state, ctx, H, dk,
                        dv, decay=_dev(cat(3).reshape(n, -1)) if gated else None,
                        head_decay=None if gated else _dev(data[0][3][0, :, 0]), segments=segments, workspace=ws)
        want = cat(4).reshape(n, H * dv)
        err = (out.cpu().to(F64) - want).abs().max().item()
        assert err <= 3e-5 * max(1.0, want.abs().max().item()), (step, err)
        for s, _, b in rows:
            done[s] = b
    assert torch.all(state[2] == -7.0)


def test_rotation_of_a_part_of_the_head_and_the_key_scale():
    from glassbox_amd import ops
    torch.manual_seed(3)
    T, H, dk, rot, base = 50, 3, 24, 8, 100.0
    q, k = torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dk, dtype=F64)
    proj = torch.zeros(T, 2 * H * dk + 5, device=DEV)
    proj[:, 5:5 + H * dk], proj[:, 5 + H * dk:] = _dev(q.reshape(T, -1)), _dev(k.reshape(T, -1))
    ang = torch.arange(T, dtype=F64)[:, None] * torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64)
    q32, k32 = torch.empty(T, H * dk, device=DEV), torch.empty(T, H * dk, device=DEV)
    ops.retention_prep(proj, 5, 5 + H * dk, _dev(ang.cos()), _dev(ang.sin()), q32, k32, H, dk, rot, 0.25)
    assert (q32.cpu().to(F64) - ps.rotate_first(q.float().to(F64), rot, base).reshape(T, -1)).abs().max() < 1e-5
    assert (k32.cpu().to(F64) - 0.25 * ps.rotate_first(k.float().to(F64), rot, base).reshape(T, -1)).abs().max() < 1e-5
    ops.retention_prep(proj, 5, 5 + H * dk, None, None, q32, k32, H, dk, 0, 1.0)   # no rotation: the heads pass
    assert torch.equal(q32.cpu(), q.float().reshape(T, -1)) and torch.equal(k32.cpu(), k.float().reshape(T, -1))


def test_decays_of_key_channels_and_the_gated_head_norm():
    from glassbox_amd import ops
    torch.manual_seed(4)
    T, width, rank, tau = 9, 24, 5, 3.0
    low, a2 = torch.randn(T, rank, dtype=F64) * 3, torch.randn(width, rank, dtype=F64)
    bias = torch.randn(width, dtype=F64) * 4
    proj = torch.zeros(T, 2 * width + rank, device=DEV)
    qk = torch.randn(T, 2 * width, dtype=F64)
    proj[:, :2 * width], proj[:, 2 * width:] = _dev(qk), _dev(low)
    q32, k32, decay = (torch.empty(T, width, device=DEV) for _ in range(3))
    ops.gla_prep(proj, 0, width, 2 * width, _dev(a2), _dev(bias), q32, k32, decay, 0.5, tau)
    want = torch.sigmoid(low.float().to(F64) @ a2.float().to(F64).t() + bias.float().to(F64)).pow(1.0 / tau)
    assert (decay.cpu().to(F64) - want).abs().max() < 2e-6 and 0.0 < float(decay.min()) and float(decay.max()) <= 1.0
    assert (q32.cpu().to(F64) - 0.5 * qk[:, :width].float().to(F64)).abs().max() < 1e-6
    assert torch.equal(k32.cpu(), qk[:, width:].float())
    eps = 1e-3
    for T, H, dv in ((9, 3, 20), (70, 3, 20), (70, 2, 72), (65, 1, 7)):   # (few rows and many take different kernels)
        o, gate, wn = torch.randn(T, H, dv, dtype=F64) * 5, torch.randn(T, H * dv, dtype=F64), torch.rand(dv, dtype=F64) + 0.5
        for w in (None, wn):
            out = torch.empty(T, H * dv, device=DEV)
            ops.head_norm_gate(_dev(o.reshape(T, -1)), _dev(gate), None if w is None else _dev(w), out, H, dv, eps)
            want = ps.rms(o.float().to(F64), eps, None if w is None else w.float().to(F64)).reshape(T, -1) * ps.silu(gate.float().to(F64))
            assert (out.cpu().to(F64) - want).abs().max() < 1e-5, (T, H, dv)


# ------------------------------------------------------------------------------------------ streams
def test_streams_kernels():
    from glassbox_amd import ops
    torch.manual_seed(5)
    for S, n, d in ((3, 7, 40), (1, 2, 64), (8, 3, 130)):
        X = torch.randn(S, n, d, dtype=F64)
        w_in, w_out, mix = torch.randn(S, dtype=F64), torch.randn(S, dtype=F64), torch.randn(S, S, dtype=F64)
        gamma, y = torch.rand(d, dtype=F64) + 0.5, torch.randn(n, d, dtype=F64)
        Xd = _dev(X)
        h, total = torch.empty(n, d, device=DEV), torch.empty(n, d, device=DEV)
        ops.streams_norm(Xd, _dev(w_in), _dev(gamma), 1e-5, h, total=total)
        f = lambda t: t.float().to(F64)
        u = sum(f(w_in)[s] * f(X)[s] for s in range(S))
        assert (total.cpu().to(F64) - u).abs().max() < 1e-5 and (h.cpu().to(F64) - ps.rms(u, 1e-5, f(gamma))).abs().max() < 1e-5
        rows = _i32([n - 1, 0])
        picked = torch.empty(2, d, device=DEV)
        ops.streams_norm(Xd, None, _dev(gamma), 1e-5, picked, rows=rows)
        assert (picked.cpu().to(F64) - ps.rms(f(X).sum(0)[[n - 1, 0]], 1e-5, f(gamma))).abs().max() < 1e-5
        again = Xd.clone()
        ops.streams_mix(Xd, _dev(mix), _dev(w_out), _dev(y))
        want = torch.stack([sum(f(mix)[s, t] * f(X)[s] for s in range(S)) + f(w_out)[t] * f(y) for t in range(S)])
        assert (Xd.cpu().to(F64) - want).abs().max() < 1e-5
        # the update and the norm that reads the streams next, in one pass
        h2 = torch.empty(n, d, device=DEV)
        ops.streams_norm(again, _dev(w_in), _dev(gamma), 1e-5, h2, update=(_dev(mix), _dev(w_out), _dev(y)))
        assert (again.cpu().to(F64) - want).abs().max() < 1e-5
        u2 = sum(f(w_in)[s] * want[s] for s in range(S))
        assert (h2.cpu().to(F64) - ps.rms(u2, 1e-5, f(gamma))).abs().max() < 2e-5


# ------------------------------------------------------------------------------------------ attention
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window, keep", [(24, 5), (16, 16), (300, 2), (7, 40), (33, 0)])
def test_window_with_kept_first_keys_at_its_edges(dtype, window, keep):
    """One request of 600 keys in pages of 16.  Every query is built so that four keys would dominate its softmax:
    the oldest key of its window, the key just before it, the last kept key and the key just after that.  Which of
    them the token reads decides its output; keys are stored through the norm-and-store kernel, whose values are
    the keys before the norm."""
    from glassbox_amd import ops
    torch.manual_seed(window * 100 + keep)
    T, H, G, hd, P = 600, 4, 2, 16, 16
    f = lambda t: t.to(dtype).to(F64)
    k_raw = f(torch.randn(T, G, hd, dtype=F64))
    bias_k, wk = f(torch.randn(G * hd, dtype=F64) * 0.2).float().to(F64), torch.rand(hd, dtype=F64).float().to(F64) + 0.5
    v = f(k_raw + bias_k.view(1, G, hd))
    k = f(ps.rms(v, 1e-5, wk))
    q = torch.zeros(T, H, hd, dtype=F64)
    for i in range(T):
        for j in (i - window + 1, i - window, keep - 1, keep):
            if 0 <= j <= i:
                q[i] += 3.0 * k[j, torch.arange(H) // (H // G)]
    q = f(q + 0.3 * torch.randn(T, H, hd, dtype=F64))
    scale = 0.35
    see = torch.tensor([[ps.visible(i, j, {"size": window, "keep_first": keep}) for j in range(T)] for i in range(T)])
    want = torch.zeros(T, H, hd, dtype=F64)
    for h in range(H):
        g = h // (H // G)
        pr = torch.softmax(((q[:, h] @ k[:, g].t()) * scale).masked_fill(~see, -math.inf), 1)
        want[:, h] = pr @ v[:, g]
    # the pages of the request, scattered over the pool
    pages = torch.randperm(T // P + 7)[:-(-T // P)].tolist()
    slots = _i32(pages[i // P] * P + i % P for i in range(T))
    k_pages = torch.zeros(ops.key_pages_shape(T // P + 8, G, P, hd), dtype=dtype, device=DEV)
    v_pages = torch.zeros(T // P + 8, G, hd, P, dtype=dtype, device=DEV)
    qk = torch.cat([q.reshape(T, H * hd), k_raw.reshape(T, G * hd)], 1).to(dtype).to(DEV)
    ops.qk_norm_store(qk, None, _dev(bias_k), None, _dev(wk), 1e-5, slots, k_pages, v_pages, H, G, hd)
    assert torch.equal(qk[:, :H * hd].cpu().to(F64), q.reshape(T, H * hd))   # no weight for the queries: they stay
    out = torch.empty(T, H * hd, dtype=dtype, device=DEV)
    table = _i32(pages).view(1, -1)
    ops.attention_plain(qk[:, :H * hd], out, _i32(range(T)), _i32([0] * T), table, k_pages, v_pages, H, scale, window,
                        keep_first=keep)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    err = (out.cpu().to(F64).view(T, H, hd) - want).abs().amax((1, 2))
    assert float(err.max()) < tol, (int(err.argmax()), float(err.max()))
    # a decode step's form (a workgroup a chunk, merged by a second kernel) gives the same bits
    last = [T - 1, window + keep, max(keep, 1)]
    ws = torch.empty(ops.attention_plain_split_floats(3, H, hd, P, T, keep), device=DEV)
    out2 = torch.empty(3, H * hd, dtype=dtype, device=DEV)
    if ws.numel():
        ops.attention_plain(qk[last, :H * hd].contiguous(), out2, _i32(last), _i32([0] * 3), table, k_pages, v_pages, H, scale,
                            window, workspace=ws, max_context=T, keep_first=keep)
        assert torch.equal(out2, out[last])
    if dtype != torch.bfloat16:
        return
    # the matrix-core kernels: the request as one portion, as a portion behind a cached beginning, and single tokens
    from glassbox_amd.engine.context import Workspace
    from glassbox_amd.parts.base import LayerCache
    ws_all, cache = Workspace(torch.device(DEV)), LayerCache(k_pages, v_pages, group=0)
    for start in (0, 463, T - 2):
        n = T - start
        ctx = SimpleNamespace(host={"n_decode": 0, "max_q_len": n, "max_context": T}, num_seqs=1, q_start=_i32([0]),
                              q_len=_i32([n]), pos0=_i32([start]), tables=[table], buffer=ws_all.buffer)
        got = torch.zeros(n, H * hd, dtype=dtype, device=DEV)
        ops.attention_prefill(qk[start:, :H * hd], got, ctx, cache, H, scale, window, keep)
        err = (got.cpu().to(F64).view(n, H, hd) - want[start:]).abs().amax((1, 2))
        assert float(err.max()) < tol, ("portion from", start, int(err.argmax()), float(err.max()))
    rows = [T - 1, min(T - 1, window + keep), max(keep, 1), 5, 300, min(T - 1, window), 0]
    for chunk_ctx in (T, 2048):   # (the launch's longest context decides how the keys are spread over workgroups)
        ctx = SimpleNamespace(host={"n_decode": len(rows), "max_context": chunk_ctx}, num_seqs=len(rows), positions=_i32(rows),
                              tables=[table.expand(len(rows), -1).contiguous()], buffer=ws_all.buffer)
        got = torch.zeros(len(rows), H * hd, dtype=dtype, device=DEV)
        ops.attention_decode(qk[rows, :H * hd].contiguous(), got, ctx, cache, H, scale, window, keep)
        err = (got.cpu().to(F64).view(len(rows), H, hd) - want[rows]).abs().amax((1, 2))
        assert float(err.max()) < tol, ("single tokens", chunk_ctx, rows[int(err.argmax())], float(err.max()))


# ------------------------------------------------------------------------------------------ whole models
REQUESTS = {"a": 150, "b": 77, "c": 41, "d": 3, "e": 1, "f": 97}


def _requests(vocab: int, seed: int = 0):
    return {r: helpers.random_tokens(vocab, n, seed=seed + n) for r, n in REQUESTS.items()}


_ORACLE: dict = {}


def _want(folder: str, tokens, dtype: str) -> np.ndarray:
    key = (folder, tuple(tokens), dtype)
    if key not in _ORACLE:
        cfg, w = ps.load_folder(folder)
        _ORACLE[key] = ps.forward(rounded(w) if dtype == "bfloat16" else w, cfg, list(tokens)).numpy()
    return _ORACLE[key]


#: how far a bfloat16 engine may be from the plain implementation on the weights it holds, relative to the request's
#: largest logit; 32-bit engines are held to helpers.TOL_F32 times that
TOL_BF16_REL = 3e-2


def _check(got, folder, requests, dtype, what):
    for r, toks in requests.items():
        want = _want(folder, toks, dtype)
        size = max(1.0, float(np.abs(want).max()))
        tol = (helpers.TOL_F32 if dtype == "float32" else TOL_BF16_REL) * size
        bad = helpers.first_bad(got[r], want, tol)
        assert bad is None, f"{what}, {dtype}, request {r} ({len(toks)} tokens): position {bad[0]} is {bad[1]:.3e} off (limit {tol:.3e})"


def _poison(engine) -> None:
    """Garbage in every page and state slot: whatever a request reads, it must have written itself."""
    for lc in engine.layers:
        for t in (lc.k_pages, lc.v_pages, lc.state):
            if t is not None:
                t.fill_(300.0)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(CASES))
def test_every_way_of_cutting_requests_into_steps(model_dirs, name, dtype):
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, name)
    requests = _requests(CASES[name]["vocab"])
    mixed, peak = helpers.schedule_mixed(requests, seed=3, live=3, tail=20)
    eng = Engine(folder, dtype=dtype, max_tokens=max(peak, 192), max_seqs=3)
    _poison(eng)
    for what, steps in (("whole", helpers.schedule_whole(requests)), ("last tokens one by one", helpers.schedule_tail(requests, 60)),
                        ("portions", helpers.schedule_chunks(requests)), ("portions of two", helpers.schedule_chunks(requests, (2,))),
                        ("mixed batches", mixed)):
        if what == "portions of two":
            steps = helpers.schedule_chunks({r: t for r, t in requests.items() if len(t) < 80}, (2,))
        got = helpers.replay(eng, steps)
        _check(got, folder, {r: requests[r] for r in got}, dtype, what)
        assert eng.cache.num_seqs() == 0 and eng.cache.free_state_slots() == 3
        assert all(eng.cache.used_pages(g) == 0 for g in range(len(eng.group_keys)))
        eng.cache.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_prompts_whole_and_in_long_portions(model_dirs, dtype):
    """A prompt of 700 tokens: the recurrent layers cut it into segments, attention crosses its window many times."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "P")
    requests = {"long": helpers.random_tokens(211, 700, seed=21), "short": helpers.random_tokens(211, 40, seed=22)}
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
    """A request far longer than the pool: its window's pages and the pages of its kept first keys are all it holds."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "R")
    toks = helpers.random_tokens(97, 400, seed=9)
    eng = Engine(folder, dtype="float32", max_tokens=160, max_seqs=1)   # ten pages; kept keys 3, a window of 40 up to 4
    got = helpers.replay(eng, helpers.schedule_chunks({"long": toks}, (33, 1, 1, 16, 5)))
    _check(got, folder, {"long": toks}, "float32", "a request longer than the pool")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_layers_replayed_from_the_first_of_their_kind(model_dirs, dtype):
    """250 tokens one by one after a prompt of four (the window, the kept keys and a page's edge pass many times over;
    in bfloat16 the steps are replayed from graphs), with the layers of a kind replayed and with every layer walked:
    the same bits."""
    from glassbox_amd.engine import Engine
    folder = folder_of(model_dirs.base, "P")
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


def test_in_32_bit_the_cutting_changes_no_bit_of_the_recurrent_layers(model_dirs):
    """A model of linear mixers alone (no attention, whose chunks depend on the position only anyway): whole, in
    portions and token by token give the same logits bit for bit, since every sum runs in the order of the tokens."""
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine import Engine
    from glassbox_amd.weights import write_random_model
    raw = dict(CASES["Q"], layers=CASES["Q"]["layers"][:2])
    folder = write_random_model(config_from_dict(raw), os.path.join(model_dirs.base, "sagalorn_linear_only"), 4, std=0.05,
                                norm_init="uniform")
    requests = {"a": helpers.random_tokens(130, 90, seed=1), "b": helpers.random_tokens(130, 33, seed=2)}
    eng = Engine(folder, dtype="float32", max_tokens=256, max_seqs=2)
    whole = helpers.replay(eng, helpers.schedule_whole(requests))
    for steps in (helpers.schedule_chunks(requests), helpers.schedule_tail(requests, 40),
                  helpers.schedule_mixed(requests, seed=1, live=2, tail=10)[0]):
        got = helpers.replay(eng, steps)
        assert all(np.array_equal(got[r], whole[r]) for r in requests)


# ------------------------------------------------------------------------------------------ generation
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_through_the_entry_points(model_dirs, name):
    from glassbox_amd.engine import Engine, generate, greedy
    folder = folder_of(model_dirs.base, name, seed=2)   # (a seed whose replies move on: most echo one token)
    cfg, w = ps.load_folder(folder)
    vocab = CASES[name]["vocab"]
    prompts = [helpers.random_tokens(vocab, n, seed=50 + n) for n in (5, 44, 1, 23, 70)]
    want = [ps.greedy(w, cfg, p, 12) for p in prompts]
    assert all(len(set(r)) > 2 for r in want), "replies that repeat one token show nothing"
    eng = Engine(folder, dtype="float32", max_tokens=1024, max_seqs=3)
    assert greedy(eng, prompts[1], 12) == want[1]
    # the scheduler: three live requests at most, prompts in portions of at most 16 tokens beside decoding requests
    assert generate(eng, prompts, max_tokens=12, token_budget=16, max_seqs=3) == want
    assert eng.cache.num_seqs() == 0 and eng.cache.free_state_slots() == 3


def test_the_command_line_runs_the_model(model_dirs, tmp_path):
    folder = folder_of(model_dirs.base, "Q", seed=2)
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = lambda *args, stdin=None: subprocess.run([sys.executable, os.path.join(root, "bin", "glassbox"), *args],
                                                   capture_output=True, text=True, timeout=600, input=stdin)
    r = run("generate", "--model", folder, "--prompt", "5,17,3,99,41", "-n", "8", "--dtype", "float32", "--no-prefix-cache")
    assert r.returncode == 0, r.stderr
    cfg, w = ps.load_folder(folder)
    assert [int(t) for t in r.stdout.split()] == ps.greedy(w, cfg, [5, 17, 3, 99, 41], 8)
    # the model keeps state and a window: its requests cannot share pages, and asking for that says why
    r = run("generate", "--model", folder, "--prompt", "5", "-n", "1", "--dtype", "float32")
    assert r.returncode != 0 and "state" in r.stderr
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3, 9], "want": [1, 3]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": [8], "want": [0]}, {"id": "b", "tokens": [4, 4], "want": []}], "end": ["a"]}]
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(tmp_path / "o"),
                        "--max-tokens", "128"], capture_output=True, text=True, timeout=600,
                       input="".join(json.dumps(s) + "\n" for s in steps))
    assert r.returncode == 0 and r.stdout.split() == ["done", "0", "done", "1"], r.stderr
    want = ps.forward(w, cfg, [5, 17, 3, 9, 8]).numpy()
    assert np.abs(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(2, -1) - want[[1, 3]]).max() < 1e-4
    assert np.abs(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4") - want[4]).max() < 1e-4
