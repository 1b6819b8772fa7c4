"""Small Dekinex configurations for the tests, and how their model folders are made.

Each differs from the others in every option: the pair table (present with other multipliers, absent), a repeated run
(two layers twice, one layer three times, the first layer once, none), a short convolution of 1 to 5 taps or none,
rotation (a part of the head, the whole head, two channels, none), windows (shorter than a page, across pages, none),
groups of query heads, key and value sizes that differ either way, heads beyond the matrix-core attention, experts with
and without a shared one, one to four experts a token (also all of them), layers without a feed-forward, sizes that
are no multiple of 8.  Score scales are large enough that single keys carry visible weight, and the forget gates'
biases reach far enough up that old tokens stay in the matrix memory for hundreds of tokens.
"""
from __future__ import annotations

import os
from typing import Dict

import torch

CASES: Dict[str, dict] = {
    # a pair table; layers 1 and 2 run twice; a window across pages; values larger than keys and the other way round
    "A": dict(architecture="Dekinex", vocab=211, width=64, residual_mult=0.5, norm={"eps": 1e-5},
              embedding={"bigram": {"buckets": 101, "mul_prev": 17, "mul_cur": 5}},
              loop={"start": 1, "stop": 3, "times": 2}, layers=[
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "conv": 4, "scale": 0.9,
                                        "rot": {"dims": 8, "base": 100.0}, "mask": {"size": 24}},
         "mlp": {"kind": "dense", "ff": 96, "limit": 0.7}},
        {"type": "mlstm", "mixer": {"heads": 2, "dim": 24, "vdim": 40, "gate_cap": 10.0},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 6, "top": 2, "scale": 1.5}, "shared": {"ff": 32}}},
        {"type": "attention", "mixer": {"heads": 3, "kv_heads": 3, "dim": 32, "vdim": 16, "conv": 2, "scale": 0.5}, "mlp": None},
        {"type": "mlstm", "mixer": {"heads": 3, "dim": 8, "vdim": 16, "gate_cap": 5.0},
         "mlp": {"kind": "dense", "ff": 40, "limit": 2.0}},
    ]),
    # no pair table, every layer once, no convolution / one tap, the whole head rotated / two channels, a window of 17,
    # one expert a token without a shared expert / every expert with one
    "B": dict(architecture="Dekinex", vocab=130, width=96, residual_mult=1.0, norm={"eps": 3e-6}, layers=[
        {"type": "mlstm", "mixer": {"heads": 1, "dim": 64, "vdim": 32, "gate_cap": 20.0},
         "mlp": {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 3, "top": 1, "scale": 1.0}}},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 1, "dim": 48, "vdim": 48, "scale": 0.6,
                                        "rot": {"dims": 48, "base": 10000.0}, "mask": {"size": 17}},
         "mlp": {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 2, "top": 2, "scale": 0.7}, "shared": {"ff": 16}}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 16, "vdim": 64, "conv": 1, "scale": 1.2,
                                        "rot": {"dims": 2, "base": 50.0}},
         "mlp": {"kind": "dense", "ff": 64, "limit": 0.3}},
    ]),
    # sizes that the matrix-core products do not take in bfloat16 (inner sizes that are no multiple of 8); the first layer
    # alone is a run of one pass; a window shorter than a page; three experts of five
    "C": dict(architecture="Dekinex", vocab=53, width=50, residual_mult=0.8, norm={"eps": 1e-5},
              embedding={"bigram": {"buckets": 7, "mul_prev": 3, "mul_cur": 1}},
              loop={"start": 0, "stop": 1, "times": 1}, layers=[
        {"type": "attention", "mixer": {"heads": 3, "kv_heads": 1, "dim": 10, "vdim": 6, "conv": 3, "scale": 1.1,
                                        "rot": {"dims": 4, "base": 20.0}, "mask": {"size": 9}},
         "mlp": {"kind": "moe", "expert": {"ff": 12}, "router": {"experts": 5, "top": 3, "scale": 2.5}, "shared": {"ff": 7}}},
        {"type": "mlstm", "mixer": {"heads": 2, "dim": 12, "vdim": 5, "gate_cap": 15.0}, "mlp": None},
        {"type": "mlstm", "mixer": {"heads": 5, "dim": 6, "vdim": 10, "gate_cap": 3.0},
         "mlp": {"kind": "dense", "ff": 30, "limit": 1.5}},
    ]),
    # a head of 136 channels (the plain attention kernel in bfloat16 too), one layer three times, five taps, a key size of
    # 128 in the matrix memory, four experts of nine
    "D": dict(architecture="Dekinex", vocab=160, width=128, residual_mult=0.25, norm={"eps": 2e-5},
              embedding={"bigram": {"buckets": 64, "mul_prev": 13, "mul_cur": 11}},
              loop={"start": 1, "stop": 2, "times": 3}, layers=[
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 136, "vdim": 40, "conv": 3, "scale": 0.3,
                                        "rot": {"dims": 64, "base": 1000.0}, "mask": {"size": 50}},
         "mlp": {"kind": "dense", "ff": 72, "limit": 1.0}},
        {"type": "attention", "mixer": {"heads": 8, "kv_heads": 2, "dim": 64, "vdim": 64, "conv": 5, "scale": 0.4,
                                        "rot": {"dims": 16, "base": 10000.0}, "mask": {"size": 33}},
         "mlp": {"kind": "moe", "expert": {"ff": 8}, "router": {"experts": 9, "top": 4, "scale": 1.0}, "shared": {"ff": 24}}},
        {"type": "mlstm", "mixer": {"heads": 2, "dim": 128, "vdim": 96, "gate_cap": 8.0},
         "mlp": {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 4, "top": 1, "scale": 2.0}, "shared": {"ff": 8}}},
    ]),
}


def folder_of(base: str, name: str, seed: int = 0, std: float = 0.05, steady: bool = False) -> str:
    """Writes (once) the model folder of a case: random matrices, and vectors of sizes that matter (``_spread``).

    ``steady``: the router's corrections lie 1.5 apart, in another order in every layer, so that a layer chooses the same
    experts for every token (their weights still move with the token).  With random weights a few tokens in a hundred
    have two experts' scores closer than bfloat16 rounding moves them, and an engine that rounds otherwise than the plain
    implementation chooses otherwise there, which is no fault; 32-bit tests use the routers whose choice moves."""
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import write_random_model
    folder = os.path.join(base, f"dekinex_{name}_{seed}" + ("_steady" if steady else ""))
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(config_from_dict(CASES[name]), folder, seed, std=std, norm_init="uniform", dtype=torch.float32)
        _spread(folder, seed, steady)
    return folder


def _spread(folder: str, seed: int, steady: bool = False) -> None:
    """The writer draws vectors as small as matrix entries and leaves 'zeros' tensors zero; here they get sizes at which
    a fault shows: norm weights (stored minus one) a few tenths from zero, convolution taps of the order of one, gate
    biases that spread the gates over their range (forget gates mostly near one), router corrections that change the
    choice, pass vectors as large as the residual."""
    from glassbox_amd.weights import SafetensorsFile, save_file
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    gen = torch.Generator().manual_seed(seed + 1000)
    draw = lambda t, s: torch.randn(t.shape, generator=gen) * s
    for n, t in tensors.items():
        if n.endswith("norm1") or n == "final.norm":
            tensors[n] = draw(t, 0.3)
        elif n.endswith(".conv"):
            tensors[n] = draw(t, 0.6)
        elif n.endswith(".i.b"):
            tensors[n] = draw(t, 2.0)
        elif n.endswith(".f.b"):
            tensors[n] = draw(t, 2.0) + 4.0
        elif n.endswith((".mix.i", ".mix.f")):
            tensors[n] = t * 8.0                     # the gates move with the token
        elif n.endswith(".correction"):
            tensors[n] = torch.randperm(t.numel(), generator=gen).float() * 1.5 if steady else draw(t, 0.15)
        elif n.endswith(".router") or n.endswith(".sg"):
            tensors[n] = t * 10.0                    # scores away from one half
        elif n == "loop.step":
            tensors[n] = draw(t, 0.1)
    save_file(tensors, path)


def rounded(w: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The weights as a bfloat16 engine holds them: matrices rounded, vectors (stored in 32-bit) as they are."""
    keep = (".conv",)
    return {k: (v.to(torch.bfloat16).to(v.dtype) if v.dim() == 2 and not k.endswith(keep) and k != "loop.step" else v)
            for k, v in w.items()}
