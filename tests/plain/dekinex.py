"""Plain, slow implementation of the Dekinex decoder: whole sequences, no cache, no state carried between calls.

One function per mechanism, float64 throughout, sharing no code with the engine.  ``cfg`` is the parsed
``config.json`` as it stands (nested), ``w`` maps the checkpoint's tensor names to tensors.

``forward(..., coarse=True)`` rounds the activations to bfloat16 where a bfloat16 engine may (the normed rows, the
projections, the heads that attention reads, what the output and down projections read): how far that moves a
position's logits says how sensitive the position is to rounding at all, which the device tests use as the scale of
their bfloat16 tolerance.

Notation: T tokens at positions 0..T-1; H query heads, G key/value heads; dk key size, dv value size per head; a
linear weight W is stored [out, in] and applied as x W^T.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Tuple

import torch

from .llama import read_safetensors

F64 = torch.float64


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as fh:
        cfg = json.load(fh)
    w = {k: v.to(F64) for k, v in read_safetensors(os.path.join(folder, "model.safetensors")).items()}
    return cfg, w


def exact(x: torch.Tensor) -> torch.Tensor:
    return x


def bf16(x: torch.Tensor) -> torch.Tensor:
    return x.to(torch.bfloat16).to(F64)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last dimension."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """The layers' norm: the stored weight is the gain minus one."""
    return unit_rms(x, eps) * (1.0 + weight)


# ---------------------------------------------------------------------------------------------- embedding
def pair_rows(tokens: List[int], buckets: int, mul_prev: int, mul_cur: int) -> List[int]:
    """Which row of the pair table each token takes: the last row (number ``buckets``) for the first token, else
    (token before * mul_prev + token * mul_cur) mod buckets."""
    return [buckets if t == 0 else (tokens[t - 1] * mul_prev + tokens[t] * mul_cur) % buckets for t in range(len(tokens))]


def embed(w, cfg: dict, tokens: List[int]) -> torch.Tensor:
    x = w["embed"][torch.tensor(tokens)]
    pairs = (cfg.get("embedding") or {}).get("bigram")
    if pairs:
        x = x + w["bigram"][torch.tensor(pair_rows(tokens, pairs["buckets"], pairs["mul_prev"], pairs["mul_cur"]))]
    return x


# ---------------------------------------------------------------------------------------------- attention
def short_convolution(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """u [T, C], taps [C, K]: y_t = sum_j taps[:, j] * u_(t - (K - 1) + j), with u = 0 before position 0."""
    T, K = u.shape[0], taps.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(K):
            s = t - (K - 1) + j
            if s >= 0:
                y[t] += taps[:, j] * u[s]
    return y


def rotate_neighbours(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, H, d]: channels (2i, 2i + 1), i < dims / 2, of every head turned by the angle t * base^(-2i / dims); the
    channels from ``dims`` on pass."""
    out = x.clone()
    for t in range(x.shape[0]):
        for i in range(dims // 2):
            ang = t * base ** (-2.0 * i / dims)
            c, s = math.cos(ang), math.sin(ang)
            a, b = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            out[t, :, 2 * i] = a * c - b * s
            out[t, :, 2 * i + 1] = b * c + a * s
    return out


def sees(i: int, j: int, window: int) -> bool:
    """Whether the token at position i reads the key at position j: itself and the window - 1 before it (0: all)."""
    return 0 <= i - j and (window == 0 or i - j < window)


def conv_attention(w, p: str, m: dict, eps: float, h: torch.Tensor, r=exact) -> torch.Tensor:
    T, H, G, dk, dv = h.shape[0], m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q, k, v = r(h @ w[p + "q"].t()), r(h @ w[p + "k"].t()), r(h @ w[p + "v"].t())
    if m.get("conv"):
        q, k, v = (short_convolution(u, w[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
    q, k, v = q.view(T, H, dk), k.view(T, G, dk), v.view(T, G, dv)
    rot = m.get("rot")
    if rot and rot["dims"]:
        q, k = rotate_neighbours(q, rot["dims"], rot["base"]), rotate_neighbours(k, rot["dims"], rot["base"])
    q, k, v = r(unit_rms(q, eps)), r(unit_rms(k, eps)), r(v)
    window = (m.get("mask") or {}).get("size", 0)
    see = torch.tensor([[sees(i, j, window) for j in range(T)] for i in range(T)])
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        s = (q[:, hh] @ k[:, g].t()) * m.get("scale", 1.0 / math.sqrt(dk))
        out[:, hh] = torch.softmax(s.masked_fill(~see, -math.inf), dim=1) @ v[:, g]
    return r(out.reshape(T, H * dv)) @ w[p + "o"].t()


# ---------------------------------------------------------------------------------------------- matrix memory
def log_sigmoid(z: float) -> float:
    return -math.log1p(math.exp(-z)) if z >= 0 else z - math.log1p(math.exp(z))


def capped_gates(zi: torch.Tensor, zf: torch.Tensor, cap: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """Log input gate cap * tanh(z / cap) and log forget gate log sigmoid(cap * tanh(z / cap))."""
    i = cap * torch.tanh(zi / cap)
    f = cap * torch.tanh(zf / cap)
    return i, torch.tensor([[log_sigmoid(float(x)) for x in row] for row in f], dtype=F64).view_as(f)


def matrix_memory_outputs(q, k, v, i, f) -> torch.Tensor:
    """q, k [T, H, dk] (q already scaled), v [T, H, dv], log gates i, f [T, H].  Per head, with C [dk, dv], n [dk] and m
    all zero before the first token:  m' = max(f + m, i);  C' = e^(f + m - m') C + e^(i - m') k v^T;  n' likewise with k;
    o = C'^T q / (max(|n' . q|, e^(-m')) + 1e-6)."""
    T, H, dk = q.shape
    dv = v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=F64)
    for h in range(H):
        C, n, m = torch.zeros(dk, dv, dtype=F64), torch.zeros(dk, dtype=F64), 0.0
        for t in range(T):
            ft, it = float(f[t, h]), float(i[t, h])
            m_new = max(ft + m, it)
            keep, take = math.exp(ft + m - m_new), math.exp(it - m_new)
            C = keep * C + take * torch.outer(k[t, h], v[t, h])
            n = keep * n + take * k[t, h]
            m = m_new
            out[t, h] = (C.t() @ q[t, h]) / (max(abs(float(n @ q[t, h])), math.exp(-m)) + 1e-6)
    return out


def mlstm(w, p: str, m: dict, eps: float, h: torch.Tensor, r=exact) -> torch.Tensor:
    T, H, dk, dv = h.shape[0], m["heads"], m["dim"], m.get("vdim", m["dim"])
    q = r(h @ w[p + "q"].t()).view(T, H, dk) / math.sqrt(dk)
    k = r(h @ w[p + "k"].t()).view(T, H, dk)
    v = r(h @ w[p + "v"].t()).view(T, H, dv)
    i, f = capped_gates(h @ w[p + "i"].t() + w[p + "i.b"], h @ w[p + "f"].t() + w[p + "f.b"], m["gate_cap"])
    o = unit_rms(matrix_memory_outputs(q, k, v, i, f), eps).reshape(T, H * dv) * w[p + "norm"]
    return r(o * torch.sigmoid(r(h @ w[p + "g"].t()))) @ w[p + "o"].t()


# ---------------------------------------------------------------------------------------------- feed-forwards
def clamped_unit(w, p: str, limit: float, h: torch.Tensor, r=exact) -> torch.Tensor:
    g = torch.clamp(h @ w[p + "gate"].t(), max=limit)
    u = torch.clamp(h @ w[p + "up"].t(), min=-limit, max=limit)
    return r(g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].t()


def expert(w, p: str, h: torch.Tensor, r=exact) -> torch.Tensor:
    g = h @ w[p + "gate"].t()
    return r(g * torch.sigmoid(g) * (h @ w[p + "up"].t())) @ w[p + "down"].t()


def route(z: torch.Tensor, correction: torch.Tensor, top: int, scale: float) -> Tuple[List[int], torch.Tensor]:
    """One token's logits z [E] -> (chosen experts, their weights): chosen by sigmoid(z) + correction, weighted by
    sigmoid(z) of the chosen over their sum (+ 1e-20), times ``scale``."""
    s = torch.sigmoid(z)
    order = sorted(range(len(z)), key=lambda e: (-float(s[e] + correction[e]), e))[:top]
    picked = s[order]
    return order, picked / (picked.sum() + 1e-20) * scale


def routed_experts(w, p: str, mlp: dict, h: torch.Tensor, r=exact) -> torch.Tensor:
    router = mlp["router"]
    z = h @ w[p + "router"].t()
    correction = w.get(p + "correction", torch.zeros(router["experts"], dtype=F64))
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, weights = route(z[t], correction, router["top"], router.get("scale", 1.0))
        for e, a in zip(chosen, weights):
            y[t] += a * expert(w, f"{p}e{e}.", h[t:t + 1], r)[0]
    if mlp.get("shared"):
        y = y + expert(w, p + "shared.", h, r) * torch.sigmoid(h @ w[p + "shared.sg"].t())
    return y


def feed_forward(w, p: str, mlp: dict, h: torch.Tensor, r=exact) -> torch.Tensor:
    if mlp["kind"] == "dense":
        return clamped_unit(w, p, mlp["limit"], h, r)
    return routed_experts(w, p, mlp, h, r)


# ---------------------------------------------------------------------------------------------- the model
def layer_calls(cfg: dict) -> List[Tuple[int, Optional[int]]]:
    """(layer, number of the pass that begins with this call or None), in the order a step runs them."""
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return [(i, None) for i in range(n)]
    a, b = loop["start"], loop["stop"]
    calls = [(i, None) for i in range(a)]
    for t in range(loop["times"]):
        calls += [(i, t if i == a else None) for i in range(a, b)]
    return calls + [(i, None) for i in range(b, n)]


def forward(w, cfg: dict, tokens: List[int], after_layers: Optional[list] = None, coarse: bool = False) -> torch.Tensor:
    """Logits [T, vocab] at every position.  ``after_layers`` collects the residual after every layer that runs.
    ``coarse``: activations rounded to bfloat16 where a bfloat16 engine may round them (the residual, norms, scores,
    gates and states stay exact)."""
    r = bf16 if coarse else exact
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = embed(w, cfg, tokens)
    first = x.clone()
    for i, begins in layer_calls(cfg):
        if begins is not None:
            if begins > 0:
                x = x + first
            x = x + w["loop.step"][begins]
        layer = cfg["layers"][i]
        h = r(offset_norm(x, w[f"l{i}.norm1"], eps))
        mixer = conv_attention if layer["type"] == "attention" else mlstm
        y = mixer(w, f"l{i}.mix.", layer["mixer"], eps, h, r)
        if layer.get("mlp"):
            y = y + feed_forward(w, f"l{i}.mlp.", layer["mlp"], h, r)
        x = x + mult * y
        if after_layers is not None:
            after_layers.append(x.clone())
    return r(offset_norm(x, w["final.norm"], eps)) @ w["head"].t()


def greedy(w, cfg: dict, prompt: List[int], n: int) -> List[int]:
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(torch.argmax(forward(w, cfg, toks)[-1])))
    return toks[len(prompt):]
