"""Dekinex without a device: the plain implementation pinned by what fixes it beside its own text, the configuration's
checks, the tensors the model declares, and the order of its layer calls."""
from __future__ import annotations

import math

import pytest
import torch

from plain import dekinex as pd
from dekinex_cases import CASES, folder_of

F64 = torch.float64


# ------------------------------------------------------------------------------------------ the plain implementation
def test_short_convolution_is_a_causal_correlation():
    torch.manual_seed(0)
    u, taps = torch.randn(11, 5, dtype=F64), torch.randn(5, 4, dtype=F64)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(u.t()[None], (3, 0)), taps[:, None, :], groups=5)[0].t()
    assert torch.allclose(pd.short_convolution(u, taps), want, atol=1e-12)
    # the last tap weighs the token itself, the first the oldest
    one = torch.zeros(6, 1, dtype=F64)
    one[2] = 1.0
    got = pd.short_convolution(one, torch.tensor([[1.0, 10.0, 100.0]], dtype=F64))[:, 0].tolist()
    assert got == [0.0, 0.0, 100.0, 10.0, 1.0, 0.0]


def test_rotation_pairs_neighbours_and_scores_depend_on_the_distance_alone():
    x = torch.zeros(3, 1, 6, dtype=F64)
    x[:, 0, 0] = 1.0          # (1, 0) in the first pair
    x[:, 0, 5] = 7.0          # beyond the rotated channels
    out = pd.rotate_neighbours(x, 4, 100.0)
    for t in range(3):
        assert out[t, 0, 0] == pytest.approx(math.cos(t)) and out[t, 0, 1] == pytest.approx(math.sin(t))
        assert out[t, 0, 5] == 7.0 and out[t, 0, 2] == 0.0
    torch.manual_seed(1)
    q, k = torch.randn(1, 2, 8, dtype=F64).expand(9, 2, 8), torch.randn(1, 2, 8, dtype=F64).expand(9, 2, 8)
    rq, rk = pd.rotate_neighbours(q, 8, 50.0), pd.rotate_neighbours(k, 8, 50.0)
    assert torch.allclose((rq[5] * rk[2]).sum(-1), (rq[8] * rk[5]).sum(-1), atol=1e-12)
    assert not torch.allclose((rq[5] * rk[2]).sum(-1), (rq[5] * rk[4]).sum(-1), atol=1e-3)


def test_visibility_at_the_windows_edges():
    assert pd.sees(10, 10, 4) and pd.sees(10, 7, 4) and not pd.sees(10, 6, 4) and not pd.sees(10, 11, 4)
    assert pd.sees(500, 0, 0) and not pd.sees(3, 4, 0)
    assert pd.sees(5, 5, 1) and not pd.sees(5, 4, 1)


def test_the_stabilised_memory_is_the_plain_weighted_sum():
    """Without the running maximum: C_t = sum_s exp(i_s + f_(s+1) + .. + f_t) k_s v_s^T, n likewise, and
    o = C^T q / (max(|n . q|, 1) + 1e-6 exp(m)) once both sides are multiplied by exp(m): checked where the floor is not
    reached and where it is."""
    torch.manual_seed(2)
    T, H, dk, dv = 12, 2, 5, 3
    q, k, v = torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dk, dtype=F64), torch.randn(T, H, dv, dtype=F64)
    i, f = torch.randn(T, H, dtype=F64) * 2, -torch.rand(T, H, dtype=F64)
    got = pd.matrix_memory_outputs(q, k, v, i, f)
    for h in range(H):
        m = 0.0
        for t in range(T):
            m = max(float(f[t, h]) + m, float(i[t, h]))
            wts = [math.exp(float(i[s, h]) + float(f[s + 1:t + 1, h].sum())) for s in range(t + 1)]
            num = sum(a * v[s, h] * float(k[s, h] @ q[t, h]) for s, a in enumerate(wts))
            nq = sum(a * float(k[s, h] @ q[t, h]) for s, a in enumerate(wts))
            want = num * math.exp(-m) / (max(abs(nq) * math.exp(-m), math.exp(-m)) + 1e-6)
            assert torch.allclose(got[t, h], want, atol=1e-10)


def test_capped_gates_stay_inside_their_cap():
    zi = torch.tensor([[-100.0, 0.0, 0.5, 100.0]], dtype=F64)
    i, f = pd.capped_gates(zi, zi, 4.0)
    assert float(i.min()) == pytest.approx(-4.0) and float(i.max()) == pytest.approx(4.0) and float(i[0, 1]) == 0.0
    assert float(f[0, 1]) == pytest.approx(math.log(0.5)) and float(f[0, 3]) == pytest.approx(-math.log1p(math.exp(-4.0)))
    assert float(f[0, 0]) == pytest.approx(-4.0 - math.log1p(math.exp(-4.0)))


def test_the_router_chooses_by_corrected_scores_and_weighs_by_plain_ones():
    z = torch.tensor([2.0, 1.0, 0.0, -1.0], dtype=F64)
    s = torch.sigmoid(z)
    chosen, weights = pd.route(z, torch.zeros(4, dtype=F64), 2, 3.0)
    assert chosen == [0, 1] and torch.allclose(weights, s[:2] / s[:2].sum() * 3.0)
    chosen, weights = pd.route(z, torch.tensor([0.0, 0.0, 0.0, 5.0], dtype=F64), 2, 1.0)
    assert chosen == [3, 0] and torch.allclose(weights, torch.stack([s[3], s[0]]) / (s[3] + s[0]))
    chosen, weights = pd.route(z, torch.zeros(4, dtype=F64), 4, 1.0)
    assert sorted(chosen) == [0, 1, 2, 3] and float(weights.sum()) == pytest.approx(1.0)
    assert pd.route(torch.zeros(3, dtype=F64), torch.zeros(3, dtype=F64), 1, 1.0)[0] == [0]   # of equal ones the lower


def test_pair_rows_and_layer_calls():
    assert pd.pair_rows([4, 9, 9], 7, 3, 1) == [7, (4 * 3 + 9) % 7, (9 * 3 + 9) % 7]
    assert pd.layer_calls(CASES["A"]) == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert pd.layer_calls(CASES["B"]) == [(0, None), (1, None), (2, None)]
    assert pd.layer_calls(CASES["C"]) == [(0, 0), (1, None), (2, None)]
    assert pd.layer_calls(CASES["D"]) == [(0, None), (1, 0), (1, 1), (1, 2), (2, None)]


@pytest.mark.parametrize("name", list(CASES))
def test_the_plain_model_is_causal_and_its_parts_all_matter(model_dirs, name):
    """A later token changes no earlier logits; every tensor of the checkpoint changes the last logits when it is
    disturbed (a part that the forward pass forgot would not)."""
    folder = folder_of(model_dirs.base, name)
    cfg, w = pd.load_folder(folder)
    toks = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3, 2, 3, 8, 4, 6, 2, 6, 4, 3, 3, 8, 3, 2, 7, 9, 5, 0, 2, 8, 8, 4, 1, 9, 7]
    toks = [t % cfg["vocab"] for t in toks]
    base = pd.forward(w, cfg, toks)
    other = pd.forward(w, cfg, toks[:-1] + [(toks[-1] + 1) % cfg["vocab"]])
    assert torch.equal(base[:-1], other[:-1]) and not torch.equal(base[-1], other[-1])
    assert torch.allclose(base[:17], pd.forward(w, cfg, toks[:17]), atol=1e-12)
    used = {n for n in w if not (".mlp.e" in n)}   # (an expert that no token chose is silent)
    for n in sorted(used):
        if n in ("embed", "bigram", "head"):
            continue   # (tables: most rows are not read by forty tokens)
        if n.endswith((".correction", ".router")):
            r = cfg["layers"][int(n.split(".")[0][1:])]["mlp"]["router"]
            if r["top"] == r["experts"] and n.endswith(".correction"):
                continue   # (every expert is chosen whatever the correction)
            if r["top"] == 1 and n.endswith(".router"):
                continue   # (one expert a token weighs the router's scale whatever its score; only a choice that flips shows)
        w2 = dict(w)
        w2[n] = w[n] + 0.9 * torch.cos(1.7 * torch.arange(w[n].numel(), dtype=F64)).view_as(w[n])   # (no constant: one added to all corrections changes no choice)
        assert not torch.allclose(pd.forward(w2, cfg, toks)[-1], base[-1], atol=1e-9), n


# ------------------------------------------------------------------------------------------ configuration and tensors
def test_the_configuration_is_checked_key_by_key():
    from glassbox_amd.config import ConfigError, config_from_dict
    cfg = config_from_dict(CASES["A"])
    assert cfg.architecture == "Dekinex" and cfg.loop == (1, 3, 2) and cfg.bigram == (101, 17, 5)
    assert config_from_dict(cfg.to_dict()) == cfg
    assert config_from_dict(CASES["B"]).loop is None and config_from_dict(CASES["B"]).bigram is None

    def broken(path, value):
        import copy
        raw = copy.deepcopy(CASES["A"])
        at = raw
        for key in path[:-1]:
            at = at[key]
        if value is None:
            at.pop(path[-1])
        else:
            at[path[-1]] = value
        return raw
    for path, value, word in ((("layers", 0, "type"), "conv", "type"), (("layers", 0, "mixer", "kv_heads"), 3, "kv_heads"),
                              (("layers", 0, "mixer", "rot", "dims"), 7, "dims"), (("layers", 1, "mixer", "gate_cap"), None, "gate_cap"),
                              (("layers", 1, "mlp", "router", "top"), 7, "top"), (("layers", 0, "mlp", "limit"), None, "limit"),
                              (("loop", "stop"), 9, "loop"), (("norm",), None, "norm"), (("layers", 1, "mlp", "kind"), "sparse", "kind"),
                              (("embedding", "bigram", "buckets"), 0, "buckets")):
        with pytest.raises(ConfigError, match=word):
            config_from_dict(broken(path, value))


@pytest.mark.parametrize("name", list(CASES))
def test_the_model_declares_the_checkpoints_tensors(model_dirs, name):
    from glassbox_amd.config import config_from_dir
    from glassbox_amd.weights import SafetensorsFile
    from glassbox_amd.weights.loader import build_model, checkpoint_layout
    folder = folder_of(model_dirs.base, name)
    model = build_model(config_from_dir(folder))
    _, shapes = checkpoint_layout(model)
    f = SafetensorsFile(folder + "/model.safetensors")
    assert {n: tuple(f.shape(n)) for n in f.names()} == {n: tuple(s) for n, s in shapes.items()}
    raw = CASES[name]
    assert ("bigram" in shapes) == ("embedding" in raw) and ("loop.step" in shapes) == ("loop" in raw)
    calls = pd.layer_calls(raw)
    assert [(c.block, c.enter) for c in model.schedule] == calls and [c.cache for c in model.schedule] == list(range(len(calls)))
    # a cache layer (pages and state) of its own for every call, and one more for the token before a step
    assert len(model.state_specs()) == len(calls) + (1 if "embedding" in raw else 0)


def test_heads_of_unequal_sizes_share_the_larger_one_in_the_cache():
    from glassbox_amd.parts.attention import ShortConvAttention, cache_head_cols
    assert cache_head_cols(16, 24) == 32 and cache_head_cols(64, 64) == 64 and cache_head_cols(10, 6) == 16
    assert cache_head_cols(136, 40) == 136 and cache_head_cols(40, 130) == 136 and cache_head_cols(128, 8) == 128
    m = ShortConvAttention(64, 4, 2, 16, 24, scale=0.5, window=24, taps=4, rot_dims=8, rot_base=100.0)
    assert m.cache_spec.head_dim == 32 and m.cache_spec.window == 24 and m.state_spec.shape == (3, 4 * 16 + 2 * 16 + 2 * 24)
    assert ShortConvAttention(64, 2, 2, 16, 16, taps=1).state_spec is None and ShortConvAttention(64, 2, 2, 16, 16).wconv is None
    o = torch.arange(8 * 4 * 3, dtype=torch.float32).view(8, 12)
    m = ShortConvAttention(8, 4, 4, 2, 3)
    m.load({"q": torch.zeros(8, 8), "k": torch.zeros(8, 8), "v": torch.zeros(12, 8), "o": o})
    wide = m.wo.view(8, 4, m.head_cols)
    assert torch.equal(wide[:, :, :3].reshape(8, 12), o) and float(wide[:, :, 3:].abs().max()) == 0.0


def test_a_model_with_state_refuses_shared_beginnings():
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.engine.engine import sharing_obstacles
    from glassbox_amd.weights.loader import build_model
    lines = sharing_obstacles(build_model(config_from_dict(CASES["A"])))
    assert any("state" in l for l in lines) and any("window" in l for l in lines)
