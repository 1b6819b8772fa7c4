"""Mixers that keep a matrix state per request and head instead of keys and values: linear attention without a
softmax or a denominator.

Both compute, per head, S_t = diag(a_t) S_(t-1) + k_t v_t^T and o_t = S_t^T q_t over a request's tokens, S being
[key size, value size], 32-bit, zero before the first token and carried in the request's state slot.  They differ
in the decay a_t and in what is done to q and k first:

``Retention``: a_t is one fixed number a head.  q and k are rotated by the token's position in the first ``rot_dims``
dimensions of each head (rotate-half pairs, frequencies base^(-2i/rot_dims)); k is then divided by sqrt(key size).
Each head's output is divided by its root mean square (no weight).

``GatedLinearAttention``: a_t is a vector over the key channels, sigmoid(z_t)^(1/tau) with z_t = A2 (A1 h_t) + b, a
projection through a narrow middle.  q is divided by sqrt(key size).  Each head's output is RMS-normed over the
value size with a weight that the heads share.

In both, the heads' outputs are multiplied by silu(G h) and projected by O.  Everything that enters the recurrence
after the projections (rotation, scales, decays, the state) is 32-bit in both precisions.
"""
from __future__ import annotations

import math
from typing import Dict, Optional, Sequence

import torch

from .. import ops
from .base import LayerCache, Mixer, StateSpec, TensorSpec, product
from .rotary import Rotary


class _LinearMixer(Mixer):
    """What the two share: the stacked input projection, the state, the gate, the output projection."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, key_dim: int, value_dim: int, eps: float):
        self.width, self.n_heads, self.key_dim, self.value_dim = width, n_heads, key_dim, value_dim
        self.eps = float(eps)
        self.qk_dim, self.v_dim = n_heads * key_dim, n_heads * value_dim
        self.state_spec = StateSpec((n_heads, value_dim, key_dim), torch.float32, 0.0)
        self.w_in: Optional[torch.Tensor] = None
        self.wo: Optional[torch.Tensor] = None

    def _stacked(self) -> Sequence[str]:
        raise NotImplementedError

    def streamed_matrices(self):
        return [self.w_in, self.wo]

    def problems(self, dtype, page_size):
        out = []   # (sizes that the matrix-core products do not take go through the plain product)
        if self.key_dim > ops.LINEAR_MAX_KEY_DIM:
            out.append(("dim", f"{self.key_dim} is above {ops.LINEAR_MAX_KEY_DIM}, the largest key size the recurrence "
                               f"kernel takes"))
        return out

    @staticmethod
    def _stack(parts):
        """The rows of several matrices as one, filled up with rows of zeros to a multiple of 8 (rows of the product's
        result then begin at 16-byte words whatever the sizes)."""
        rows = sum(p.shape[0] for p in parts)
        if rows % 8:
            parts = list(parts) + [torch.zeros((8 - rows % 8, parts[0].shape[1]), dtype=parts[0].dtype, device=parts[0].device)]
        return torch.cat(parts, 0)

    def _project(self, ctx, h, tail: int = 0):
        """The stacked input product.  ``tail``: the last so many rows of the stacked matrix (beyond a multiple of the
        product's tiles they would cost a step of many rows a second round of tiles) go through a product of their own."""
        n = h.shape[0]
        rows = self.w_in.shape[0]
        proj = ctx.buffer("lin_proj", (n, rows), ctx.dtype)
        if tail and n > ops.ROPE_PRODUCT_MAX_ROWS:
            main = rows - tail
            product(ctx, h, self.w_in[:main], proj[:, :main])
            product(ctx, h, self.w_in[main:], proj[:, main:])
        else:
            product(ctx, h, self.w_in, proj)
        return proj

    def _finish(self, ctx, proj, q32, k32, residual, cache, store, norm_weight, decay=None, head_decay=None):
        n = proj.shape[0]
        if cache is None or cache.state is None:
            raise ValueError(f"{type(self).__name__} needs a layer cache with state")
        v_off, g_off = 2 * self.qk_dim, 2 * self.qk_dim + self.v_dim
        o = ctx.buffer("lin_o", (n, self.v_dim), torch.float32)
        # a long portion runs as segments side by side (the step's longest portion decides for the whole launch)
        segments = ops.linear_scan_segments(int(ctx.host["max_q_len"]))
        ws = None
        if segments > 1:
            ws = ctx.buffer("lin_segments", (ctx.num_seqs * segments * self.n_heads * (self.value_dim + 1) * self.key_dim,),
                            torch.float32)
        ops.linear_scan(q32, k32, proj[:, v_off:v_off + self.v_dim], o, cache.state, ctx, self.n_heads, self.key_dim,
                        self.value_dim, decay=decay, head_decay=head_decay, segments=segments, workspace=ws)
        gated = ctx.buffer("lin_gated", (n, self.v_dim), ctx.dtype)
        ops.head_norm_gate(o, proj[:, g_off:g_off + self.v_dim], norm_weight, gated, self.n_heads, self.value_dim, self.eps)
        product(ctx, gated, self.wo, residual, accumulate=not store)


class Retention(_LinearMixer):
    def __init__(self, width: int, n_heads: int, key_dim: int, value_dim: int, decay: Sequence[float], eps: float,
                 rot_dims: int = 0, rot_base: float = 10000.0):
        super().__init__(width, n_heads, key_dim, value_dim, eps)
        if len(decay) != n_heads:
            raise ValueError(f"{len(decay)} decays for {n_heads} heads")
        if rot_dims % 2 or not 0 <= rot_dims <= key_dim:
            raise ValueError(f"{rot_dims} rotated dimensions: an even number up to the key size {key_dim}")
        self.decay = tuple(float(d) for d in decay)
        self.rot_dims = int(rot_dims)
        self.position = Rotary(rot_dims, rot_base) if rot_dims else None
        self.head_decay: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"q": TensorSpec((self.qk_dim, self.width)), "k": TensorSpec((self.qk_dim, self.width)),
                "v": TensorSpec((self.v_dim, self.width)), "g": TensorSpec((self.v_dim, self.width)),
                "o": TensorSpec((self.width, self.v_dim))}

    def load(self, tensors):
        self.w_in = self._stack([tensors[n] for n in ("q", "k", "v", "g")])   # one product computes all four
        self.wo = tensors["o"].contiguous()
        self.head_decay = torch.tensor(self.decay, dtype=torch.float32, device=self.wo.device)

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``, or with ``store`` writes them there (float32 either way)."""
        n = h.shape[0]
        proj = self._project(ctx, h)
        q32 = ctx.buffer("lin_q", (n, self.qk_dim), torch.float32)
        k32 = ctx.buffer("lin_k", (n, self.qk_dim), torch.float32)
        cos, sin = self.position.table(ctx) if self.position is not None else (None, None)
        ops.retention_prep(proj, 0, self.qk_dim, cos, sin, q32, k32, self.n_heads, self.key_dim, self.rot_dims,
                           1.0 / math.sqrt(self.key_dim))
        self._finish(ctx, proj, q32, k32, residual, cache, store, None, head_decay=self.head_decay)


class GatedLinearAttention(_LinearMixer):
    """``rank``: the narrow middle of the decay's projection; None takes it from the checkpoint's tensors."""

    def __init__(self, width: int, n_heads: int, key_dim: int, value_dim: int, tau: float, eps: float,
                 rank: Optional[int] = None):
        super().__init__(width, n_heads, key_dim, value_dim, eps)
        if not tau > 0:
            raise ValueError(f"tau must be positive, got {tau}")
        self.tau = float(tau)
        self.rank = rank
        self.w_a2: Optional[torch.Tensor] = None
        self.a2_bias: Optional[torch.Tensor] = None
        self.norm_weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        r = -1 if self.rank is None else self.rank
        return {"q": TensorSpec((self.qk_dim, self.width)), "k": TensorSpec((self.qk_dim, self.width)),
                "v": TensorSpec((self.v_dim, self.width)), "g": TensorSpec((self.v_dim, self.width)),
                "o": TensorSpec((self.width, self.v_dim)), "norm": TensorSpec((self.value_dim,), kind="f32", init="ones"),
                "a1": TensorSpec((r, self.width)), "a2": TensorSpec((self.qk_dim, r)),
                "a2.b": TensorSpec((self.qk_dim,), kind="f32", init="zeros")}

    def load(self, tensors):
        if tensors["a1"].shape[0] != tensors["a2"].shape[1]:
            raise ValueError(f"a1 has {tensors['a1'].shape[0]} rows, a2 has {tensors['a2'].shape[1]} columns")
        # one product computes q, k, v, the gate and the narrow rows of the decay
        self.w_in = self._stack([tensors[n] for n in ("q", "k", "v", "g", "a1")])
        self.wo = tensors["o"].contiguous()
        self.w_a2 = tensors["a2"].contiguous()
        self.a2_bias = tensors["a2.b"].contiguous()
        self.norm_weight = tensors["norm"].contiguous()

    def streamed_matrices(self):
        return [self.w_in, self.wo, self.w_a2]

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``, or with ``store`` writes them there (float32 either way)."""
        n = h.shape[0]
        main = 2 * self.qk_dim + 2 * self.v_dim
        # (the narrow rows of the decay and the filling rows behind them, where the rest is whole words)
        proj = self._project(ctx, h, tail=self.w_in.shape[0] - main if main % 8 == 0 else 0)
        q32 = ctx.buffer("lin_q", (n, self.qk_dim), torch.float32)
        k32 = ctx.buffer("lin_k", (n, self.qk_dim), torch.float32)
        decay = ctx.buffer("lin_decay", (n, self.qk_dim), torch.float32)
        low_off, rank = 2 * self.qk_dim + 2 * self.v_dim, self.w_a2.shape[1]
        z = None
        if ctx.dtype == torch.float32 or (rank % 8 == 0 and low_off % 8 == 0):
            # the second matrix of the decay's projection as a product of its own (sizes that a bfloat16 product does not
            # take: inside the kernel)
            z = ctx.buffer("lin_z", (n, self.qk_dim), torch.float32)
            product(ctx, proj[:, low_off:low_off + rank], self.w_a2, z)
        ops.gla_prep(proj, 0, self.qk_dim, low_off, self.w_a2, self.a2_bias, q32, k32, decay,
                     1.0 / math.sqrt(self.key_dim), self.tau, z=z)
        self._finish(ctx, proj, q32, k32, residual, cache, store, self.norm_weight, decay=decay)


class MLSTM(Mixer):
    """Matrix memory with exponential gates.  Per head, q = W_q h / sqrt(key size), k = W_k h, v = W_v h, a log input
    gate i = cap tanh((W_i h + b_i) / cap) and a log forget gate f = log sigmoid(cap tanh((W_f h + b_f) / cap)); with a
    running maximum m (0 before the first token): m_t = max(f_t + m_(t-1), i_t),
    S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T, n_t the same with k_t alone,
    o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6).  Every head's o gets a unit-RMS norm, the heads
    side by side are multiplied by ``norm`` (a weight for every channel of every head) and by sigmoid(W_g h), and
    projected by W_o.

    It is the decayed-state recurrence of this module with a decay a token and head, keys scaled by the input gate's
    factor, and n as one more value channel whose v is 1.  The state of a request and head is [value size + 2, key size]
    float32: the columns of S, n, and a row whose first element is m.  Gates, m, the factors, q and k are 32-bit in both
    precisions (the gates' projections are a product of their own with 32-bit results)."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, key_dim: int, value_dim: int, gate_cap: float, eps: float):
        if not gate_cap > 0:
            raise ValueError(f"the gates' cap must be positive, got {gate_cap}")
        self.width, self.n_heads, self.key_dim, self.value_dim = width, n_heads, key_dim, value_dim
        self.gate_cap, self.eps = float(gate_cap), float(eps)
        self.qk_dim, self.v_dim = n_heads * key_dim, n_heads * value_dim
        self.state_spec = StateSpec((n_heads, value_dim + 2, key_dim), torch.float32, 0.0)
        self.w_in = self.w_gates = self.wo = self.bias_i = self.bias_f = self.norm_weight = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H = self.n_heads
        return {"q": TensorSpec((self.qk_dim, self.width)), "k": TensorSpec((self.qk_dim, self.width)),
                "v": TensorSpec((self.v_dim, self.width)), "g": TensorSpec((self.v_dim, self.width)),
                "o": TensorSpec((self.width, self.v_dim)), "norm": TensorSpec((self.v_dim,), kind="f32", init="ones"),
                "i": TensorSpec((H, self.width)), "i.b": TensorSpec((H,), kind="f32", init="normal"),
                "f": TensorSpec((H, self.width)), "f.b": TensorSpec((H,), kind="f32", init="normal")}

    def load(self, tensors):
        self.w_in = _LinearMixer._stack([tensors[n] for n in ("q", "k", "v", "g")])   # one product computes all four
        self.w_gates = torch.cat([tensors["i"], tensors["f"]], 0).contiguous()
        self.wo = tensors["o"].contiguous()
        self.bias_i, self.bias_f = tensors["i.b"].contiguous(), tensors["f.b"].contiguous()
        self.norm_weight = tensors["norm"].contiguous()

    def streamed_matrices(self):
        return [self.w_in, self.w_gates, self.wo]

    def problems(self, dtype, page_size):
        if self.key_dim > ops.LINEAR_MAX_KEY_DIM:
            return [("dim", f"{self.key_dim} is above {ops.LINEAR_MAX_KEY_DIM}, the largest key size the recurrence kernel takes")]
        return []

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``, or with ``store`` writes them there (float32 either way)."""
        if cache is None or cache.state is None:
            raise ValueError("MLSTM needs a layer cache with state")
        n, H, dk, dv = h.shape[0], self.n_heads, self.key_dim, self.value_dim
        proj = ctx.buffer("lin_proj", (n, self.w_in.shape[0]), ctx.dtype)
        product(ctx, h, self.w_in, proj)
        z = ctx.buffer("mlstm_z", (n, 2 * H), torch.float32)
        product(ctx, h, self.w_gates, z)
        coef = ctx.buffer("mlstm_coef", (n, H, 3), torch.float32)
        ops.mlstm_gates(z, self.bias_i, self.bias_f, self.gate_cap, coef, cache.state, dv + 1, ctx, H)
        q32 = ctx.buffer("lin_q", (n, self.qk_dim), torch.float32)
        k32 = ctx.buffer("lin_k", (n, self.qk_dim), torch.float32)
        decay = ctx.buffer("mlstm_decay", (n, H), torch.float32)
        vext = ctx.buffer("mlstm_v", (n, H * (dv + 1)), ctx.dtype)
        ops.mlstm_prep(proj, 0, self.qk_dim, 2 * self.qk_dim, coef, q32, k32, decay, vext, H, dk, dv, 1.0 / math.sqrt(dk))
        o = ctx.buffer("mlstm_o", (n, H * (dv + 1)), torch.float32)
        segments = ops.linear_scan_segments(int(ctx.host["max_q_len"]))
        ws = None
        if segments > 1:
            ws = ctx.buffer("lin_segments", (ctx.num_seqs * segments * H * (dv + 2) * dk,), torch.float32)
        ops.linear_scan(q32, k32, vext, o, cache.state, ctx, H, dk, dv + 1, token_decay=decay, segments=segments, workspace=ws)
        gated = ctx.buffer("lin_gated", (n, self.v_dim), ctx.dtype)
        g_off = 2 * self.qk_dim + self.v_dim
        ops.mlstm_out(o, coef, proj[:, g_off:g_off + self.v_dim], self.norm_weight, gated, H, dv, self.eps)
        product(ctx, gated, self.wo, residual, accumulate=not store)
