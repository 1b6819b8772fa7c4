"""Small Sagalorn configurations for the tests, and how their model folders are made.

Each differs from the others in every option: streams (several, one, none), a repeated run of layers (three times,
once, none), rotation (a part of the head, the whole head, none), windows (with kept first keys, without, none),
groups of query heads, key and value sizes that differ, sizes that are no power of two.  ``sharp`` configurations
have a large score scale and decays close to one, so that single keys and old tokens carry visible weight.
"""
from __future__ import annotations

import os
from typing import Dict, Tuple

import torch

CASES: Dict[str, dict] = {
    # three streams; layers 1 and 2 run three times; a window with kept first keys that ends inside a page
    "P": dict(architecture="Sagalorn", vocab=211, width=64, streams=3, logit_scale=0.5, embedding={"scale": 4.0},
              norm={"eps": 1e-5}, loop={"start": 1, "stop": 3, "times": 3}, layers=[
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 4, "dim": 16, "vdim": 16, "scale": 0.9,
                                        "mask": {"size": 24, "keep_first": 5}}, "mlp": {"kind": "dense", "ff": 96}},
        {"type": "retention", "mixer": {"heads": 2, "dim": 24, "vdim": 40, "decay": [0.9, 0.995],
                                        "rot": {"dims": 8, "base": 100.0}}, "mlp": None},
        {"type": "gla", "mixer": {"heads": 3, "dim": 8, "vdim": 16, "tau": 4.0, "rank": 8}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 6, "kv_heads": 2, "dim": 32, "vdim": 32, "scale": 0.4}, "mlp": None},
    ]),
    # a plain residual, every layer once, no rotation, a window without kept keys, one key head for two query heads
    "Q": dict(architecture="Sagalorn", vocab=130, width=96, logit_scale=2.0, norm={"eps": 3e-6}, layers=[
        {"type": "gla", "mixer": {"heads": 2, "dim": 64, "vdim": 32, "tau": 1.0, "rank": 16}, "mlp": {"kind": "dense", "ff": 64}},
        {"type": "retention", "mixer": {"heads": 4, "dim": 32, "vdim": 32, "decay": [0.5, 0.97, 0.99, 1.0]}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 48, "vdim": 48, "scale": 0.6,
                                        "mask": {"size": 17, "keep_first": 0}}, "mlp": {"kind": "dense", "ff": 128}},
    ]),
    # one stream that still has its weights; a run repeated once; the whole head rotated; more kept keys than two pages
    "R": dict(architecture="Sagalorn", vocab=97, width=128, streams=1, logit_scale=1.0, embedding={"scale": 0.5},
              norm={"eps": 1e-6}, loop={"start": 0, "stop": 2, "times": 1}, layers=[
        {"type": "retention", "mixer": {"heads": 1, "dim": 128, "vdim": 64, "decay": [0.98],
                                        "rot": {"dims": 128, "base": 10000.0}}, "mlp": {"kind": "dense", "ff": 72}},
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.3,
                                        "mask": {"size": 40, "keep_first": 35}}, "mlp": None},
        {"type": "gla", "mixer": {"heads": 1, "dim": 16, "vdim": 128, "tau": 16.0, "rank": 24}, "mlp": {"kind": "dense", "ff": 40}},
    ]),
    # sizes that the matrix-core products do not take in bfloat16 (inner sizes that are no multiple of 8): the plain product
    "O": dict(architecture="Sagalorn", vocab=53, width=50, streams=2, logit_scale=0.7, embedding={"scale": 3.0},
              norm={"eps": 1e-5}, loop={"start": 1, "stop": 2, "times": 2}, layers=[
        {"type": "retention", "mixer": {"heads": 3, "dim": 6, "vdim": 10, "decay": [0.8, 0.9, 0.99],
                                        "rot": {"dims": 4, "base": 50.0}}, "mlp": None},
        {"type": "attention", "mixer": {"heads": 3, "kv_heads": 1, "dim": 10, "vdim": 10, "scale": 1.1,
                                        "mask": {"size": 9, "keep_first": 3}}, "mlp": {"kind": "dense", "ff": 30}},
        {"type": "gla", "mixer": {"heads": 2, "dim": 12, "vdim": 5, "tau": 2.5, "rank": 3}, "mlp": None},
    ]),
    # heads that the matrix-core attention kernels do not take (40 and 24 dimensions: the plain kernel in bfloat16 too),
    # four streams, a decay's middle that is no multiple of 8, a window shorter than a page
    "S": dict(architecture="Sagalorn", vocab=160, width=80, streams=4, logit_scale=1.5, embedding={"scale": 2.0},
              norm={"eps": 2e-5}, loop={"start": 0, "stop": 3, "times": 2}, layers=[
        {"type": "attention", "mixer": {"heads": 2, "kv_heads": 1, "dim": 40, "vdim": 40, "scale": 0.5,
                                        "mask": {"size": 11, "keep_first": 2}}, "mlp": None},
        {"type": "gla", "mixer": {"heads": 2, "dim": 40, "vdim": 24, "tau": 8.0, "rank": 12}, "mlp": {"kind": "dense", "ff": 56}},
        {"type": "attention", "mixer": {"heads": 4, "kv_heads": 4, "dim": 24, "vdim": 24, "scale": 0.7,
                                        "mask": {"size": 50, "keep_first": 17}}, "mlp": None},
        {"type": "retention", "mixer": {"heads": 5, "dim": 16, "vdim": 16, "decay": [0.7, 0.9, 0.95, 0.99, 0.999],
                                        "rot": {"dims": 16, "base": 1000.0}}, "mlp": None},
    ]),
}


def folder_of(base: str, name: str, seed: int = 0, std: float = 0.05) -> str:
    """Writes (once) the model folder of a case: random matrices, norm weights and stream weights away from one,
    biases as large as the projections' outputs."""
    from glassbox_amd.config import config_from_dict
    from glassbox_amd.weights import write_random_model
    folder = os.path.join(base, f"sagalorn_{name}_{seed}")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_random_model(config_from_dict(CASES[name]), folder, seed, std=std, norm_init="uniform", dtype=torch.float32)
        _spread(folder, seed)
    return folder


def _spread(folder: str, seed: int) -> None:
    """Biases and the bias of the decays as random numbers of a size that matters (the writer leaves 'zeros' tensors
    zero and draws biases as small as matrix entries)."""
    from glassbox_amd.weights import SafetensorsFile, save_file
    path = os.path.join(folder, "model.safetensors")
    f = SafetensorsFile(path)
    tensors = {n: f.tensor(n).clone() for n in f.names()}
    f.close()
    gen = torch.Generator().manual_seed(seed + 1000)
    for n, t in tensors.items():
        if n.endswith((".q.b", ".k.b", ".o.b")):
            tensors[n] = torch.randn(t.shape, generator=gen) * 0.3
        elif n.endswith(".a2.b"):
            tensors[n] = torch.randn(t.shape, generator=gen) * 2.0 + 2.0   # decays from 0.5 to nearly 1
        elif n.endswith(".a2"):
            tensors[n] = t * 20.0                                         # and they move with the token
    save_file(tensors, path)


def rounded(w: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """The weights as a bfloat16 engine holds them: matrices rounded, vectors and stream weights as they are."""
    return {k: (v.to(torch.bfloat16).to(v.dtype) if v.dim() == 2 and ".hc" not in k else v) for k, v in w.items()}
