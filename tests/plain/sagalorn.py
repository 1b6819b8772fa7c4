"""Plain, slow implementation of the Sagalorn decoder: whole sequences, no cache, no state carried between calls.

One function per mechanism, float64 throughout, sharing no code with the engine.  ``cfg`` is the parsed
``config.json`` as it stands (nested), ``w`` maps the checkpoint's tensor names to tensors.

Notation: T tokens, positions 0..T-1; H heads; dk key size, dv value size per head; a linear weight W is stored
[out, in] and applied as x W^T.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import torch

from .llama import read_safetensors

F64 = torch.float64


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    w = {k: v.to(F64) for k, v in read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def rms(x: torch.Tensor, eps: float, weight: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension, times the weight if there is one."""
    y = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z / (1.0 + torch.exp(-z))


def rotate_first(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, H, d]: the first ``dims`` dimensions of every head turned by the token's position, dimension i paired
    with i + dims/2, angle = position * base^(-2i/dims); the other dimensions pass."""
    if dims == 0:
        return x
    T, half = x.shape[0], dims // 2
    out = x.clone()
    for t in range(T):
        for i in range(half):
            ang = t * base ** (-2.0 * i / dims)
            c, s = math.cos(ang), math.sin(ang)
            lo, hi = x[t, :, i], x[t, :, i + half]
            out[t, :, i] = lo * c - hi * s
            out[t, :, i + half] = hi * c + lo * s
    return out


def decayed_state_outputs(q, k, v, decay) -> torch.Tensor:
    """The recurrence of both linear mixers, token by token.  q, k [T, H, dk], v [T, H, dv]; ``decay`` [T, H, dk]
    (a factor for every row of the state at every token).  S starts at zero; S <- decay_t (rows) * S + k_t v_t^T;
    o_t = S^T q_t.  Returns [T, H, dv]."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = decay[t, h].unsqueeze(1) * S + torch.outer(k[t, h], v[t, h])
            out[t, h] = S.t() @ q[t, h]
    return out


def retention(w: Dict[str, torch.Tensor], p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T, H, dk, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ w[p + "q"].t()).view(T, H, dk)
    k = (h @ w[p + "k"].t()).view(T, H, dk)
    v = (h @ w[p + "v"].t()).view(T, H, dv)
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rotate_first(q, rot["dims"], rot["base"])
    k = rotate_first(k, rot["dims"], rot["base"]) / math.sqrt(dk)
    decay = torch.tensor(m["decay"], dtype=F64).view(1, H, 1).expand(T, H, dk)
    o = rms(decayed_state_outputs(q, k, v, decay), eps)          # each head by its own root mean square, no weight
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].t())) @ w[p + "o"].t()


def gated_linear_attention(w, p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T, H, dk, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = (h @ w[p + "q"].t()).view(T, H, dk) / math.sqrt(dk)
    k = (h @ w[p + "k"].t()).view(T, H, dk)
    v = (h @ w[p + "v"].t()).view(T, H, dv)
    z = (h @ w[p + "a1"].t()) @ w[p + "a2"].t() + w[p + "a2.b"]
    decay = torch.sigmoid(z).pow(1.0 / m.get("tau", 1.0)).view(T, H, dk)
    o = rms(decayed_state_outputs(q, k, v, decay), eps, w[p + "norm"])
    return (o.reshape(T, H * dv) * silu(h @ w[p + "g"].t())) @ w[p + "o"].t()


def visible(i: int, j: int, mask: Optional[dict]) -> bool:
    """Whether the token at position i reads the key at position j."""
    if j > i:
        return False
    if mask is None:
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def tied_value_attention(w, p: str, m: dict, eps: float, h: torch.Tensor) -> torch.Tensor:
    T, H, d = h.shape[0], m["heads"], m["dim"]
    G = m.get("kv_heads", H)
    q = (h @ w[p + "q"].t() + w[p + "q.b"]).view(T, H, d)
    k = (h @ w[p + "k"].t() + w[p + "k.b"]).view(T, G, d)
    v = k                                                          # the values are the keys before their norm
    q, k = rms(q, eps, w[p + "q.norm"]), rms(k, eps, w[p + "k.norm"])
    scale = m.get("scale", 1.0 / math.sqrt(d))
    see = torch.tensor([[visible(i, j, m.get("mask")) for j in range(T)] for i in range(T)])
    out = torch.zeros(T, H, d, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)                                         # query head hh reads key head floor(hh / (H/G))
        s = (q[:, hh] @ k[:, g].t()) * scale
        pr = torch.softmax(s.masked_fill(~see, -math.inf), dim=1)
        out[:, hh] = pr @ v[:, g]
    return out.reshape(T, H * d) @ w[p + "o"].t() + w[p + "o.b"]


def swiglu(w, p: str, h: torch.Tensor) -> torch.Tensor:
    return (silu(h @ w[p + "gate"].t()) * (h @ w[p + "up"].t())) @ w[p + "down"].t()


MIXERS = {"retention": retention, "gla": gated_linear_attention, "attention": tied_value_attention}


def layer_order(cfg: dict) -> List[int]:
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return list(range(n))
    return list(range(loop["start"])) + list(range(loop["start"], loop["stop"])) * loop["times"] + list(range(loop["stop"], n))


def sublayer_on_streams(w, X: List[torch.Tensor], hc: str, norm_w: torch.Tensor, eps: float, fn) -> List[torch.Tensor]:
    """Streams X_0..X_(S-1): the sublayer reads u = sum_s in[s] X_s through its norm; every new stream t is
    sum_s mix[s, t] X_s + out[t] y, all from the old streams."""
    S = len(X)
    u = sum(w[hc + "in"][s] * X[s] for s in range(S))
    y = fn(rms(u, eps, norm_w))
    return [sum(w[hc + "mix"][s, t] * X[s] for s in range(S)) + w[hc + "out"][t] * y for t in range(S)]


def forward(w, cfg: dict, tokens: List[int], after_layers: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] at every position.  ``after_layers`` collects the residual (the sum of the streams) after
    every layer that runs."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    S = cfg.get("streams")
    X = [x.clone() for _ in range(S)] if S is not None else None
    for i in layer_order(cfg):
        layer = cfg["layers"][i]
        mix = lambda hh, i=i, layer=layer: MIXERS[layer["type"]](w, f"l{i}.mix.", layer["mixer"], eps, hh)
        ffn = (lambda hh, i=i: swiglu(w, f"l{i}.mlp.", hh)) if layer.get("mlp") else None
        if X is not None:
            X = sublayer_on_streams(w, X, f"l{i}.hc1.", w[f"l{i}.norm1"], eps, mix)
            if ffn is not None:
                X = sublayer_on_streams(w, X, f"l{i}.hc2.", w[f"l{i}.norm2"], eps, ffn)
        else:
            x = x + mix(rms(x, eps, w[f"l{i}.norm1"]))
            if ffn is not None:
                x = x + ffn(rms(x, eps, w[f"l{i}.norm2"]))
        if after_layers is not None:
            after_layers.append(sum(X) if X is not None else x.clone())
    if X is not None:
        x = sum(X)
    return (rms(x, eps, w["final.norm"]) @ w["head"].t()) * cfg.get("logit_scale", 1.0)


def greedy(w, cfg: dict, prompt: List[int], n: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(w, cfg, toks)[-1])))
    return toks[len(prompt):]
