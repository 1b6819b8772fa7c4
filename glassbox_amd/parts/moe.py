"""A feed-forward of many small experts of which each token uses a few.

Router logits z = W_router h in 32-bit; scores s = sigmoid(z); the ``top`` experts with the largest s + correction are
chosen (the correction only chooses); their weights are s / (sum of the chosen s + 1e-20) * scale.  An expert is
W_down (silu(W_gate h) * (W_up h)) without biases, and the output is the weighted sum of the chosen experts' outputs.
A shared expert of the same form may run for every token, times sigmoid(W_sg h), one number a token.

The experts' gate and up matrices are stacked by rows and their down matrices side by side, the shared expert's
behind them.  One product gives every expert's gate and up sums; the unit's kernel multiplies each expert's columns by
the token's weight for it, zero for an expert that was not chosen; one product with the down matrices then adds up
exactly the chosen experts' outputs.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import FeedForward, TensorSpec, product


class RoutedExperts(FeedForward):
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_experts: int, top: int, expert_ff: int, router_scale: float = 1.0,
                 shared_ff: int = 0, correction: bool = True):
        if not 1 <= top <= n_experts:
            raise ValueError(f"{top} experts a token out of {n_experts}")
        self.width, self.n_experts, self.top, self.expert_ff = width, int(n_experts), int(top), int(expert_ff)
        self.router_scale, self.shared_ff, self.has_correction = float(router_scale), int(shared_ff), bool(correction)
        self.inter = self.n_experts * self.expert_ff + self.shared_ff
        self.w_router = self.correction = self.w_gate_up = self.w_down = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs: Dict[str, TensorSpec] = {}
        for e in range(self.n_experts):
            specs[f"e{e}.gate"] = TensorSpec((self.expert_ff, self.width))
            specs[f"e{e}.up"] = TensorSpec((self.expert_ff, self.width))
            specs[f"e{e}.down"] = TensorSpec((self.width, self.expert_ff))
        specs["router"] = TensorSpec((self.n_experts, self.width))
        if self.has_correction:
            specs["correction"] = TensorSpec((self.n_experts,), kind="f32", init="normal")
        if self.shared_ff:
            specs["shared.gate"] = TensorSpec((self.shared_ff, self.width))
            specs["shared.up"] = TensorSpec((self.shared_ff, self.width))
            specs["shared.down"] = TensorSpec((self.width, self.shared_ff))
            specs["shared.sg"] = TensorSpec((1, self.width))
        return specs

    def load(self, tensors):
        names = [f"e{e}" for e in range(self.n_experts)] + (["shared"] if self.shared_ff else [])
        self.w_gate_up = torch.cat([tensors[f"{n}.gate"] for n in names] + [tensors[f"{n}.up"] for n in names], 0)
        self.w_down = torch.cat([tensors[f"{n}.down"] for n in names], 1).contiguous()
        router = [tensors["router"]] + ([tensors["shared.sg"]] if self.shared_ff else [])
        self.w_router = torch.cat(router, 0).contiguous()
        self.correction = tensors["correction"].contiguous() if self.has_correction else None

    def streamed_matrices(self):
        return [self.w_router, self.w_gate_up, self.w_down]

    def problems(self, dtype, page_size):
        out = []
        if self.n_experts > ops.MOE_MAX_EXPERTS:
            out.append(("n_experts", f"{self.n_experts} is above {ops.MOE_MAX_EXPERTS}, the most experts the router's kernel takes"))
        if self.top > ops.MOE_MAX_TOP:
            out.append(("top", f"{self.top} is above {ops.MOE_MAX_TOP}, the most experts a token the router's kernel takes"))
        return out

    def forward(self, ctx, h, residual, store: bool = False):
        n, E = h.shape[0], self.n_experts
        cols = E + (1 if self.shared_ff else 0)
        z = ctx.buffer("moe_z", (n, cols), torch.float32)
        product(ctx, h, self.w_router, z)
        combine = ctx.buffer("moe_combine", (n, cols), torch.float32)
        ids = ctx.buffer("moe_ids", (n, self.top), torch.int32)
        weights = ctx.buffer("moe_weights", (n, self.top), torch.float32)
        ops.moe_route(z, E, self.correction, self.top, self.router_scale, bool(self.shared_ff), combine, ids, weights)
        gate_up = ctx.buffer("moe_gate_up", (n, 2 * self.inter), torch.float32)
        product(ctx, h, self.w_gate_up, gate_up)
        act = ctx.buffer("act", (n, self.inter), ctx.dtype)
        ops.moe_gated_units(gate_up, combine, act, E, self.expert_ff)
        product(ctx, act, self.w_down, residual, accumulate=not store)
        return None
