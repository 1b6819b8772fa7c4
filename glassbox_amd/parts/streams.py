"""A residual of several streams (hyper-connections) and the block that works on it.

The model keeps S copies X[0..S-1] of the residual, all equal to the embedding at the start.  A sublayer (mixer or
feed-forward) of a ``StreamsBlock`` reads u = sum_s in[s] X[s] through its norm, and its output y goes back into
all streams at once, from the old ones: X'[t] = sum_s mix[s, t] X[s] + out[t] y (mix is indexed [from, to]).  At the
end ``StreamsSumNorm`` norms sum_s X[s].  The streams and everything added to them are 32-bit.

The sublayers are the ordinary mixers and feed-forwards; what the block needs of them is that they can write their
rows instead of adding them (``forward(..., store=True)``, class attribute ``accepts_store``).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from .base import Block, CacheSpec, FeedForward, LayerCache, Mixer, Normed, Part, StateSpec, TensorSpec
from .norm import RMSNorm


class StreamsSumNorm(RMSNorm):
    """The model's last norm over the sum of the streams; ``x`` is [streams, n, width]."""

    def forward(self, ctx, x, rows=None, out_name="h"):
        m = x.shape[1] if rows is None else rows.numel()
        out = ctx.buffer(out_name, (m, self.width), ctx.dtype)
        ops.streams_norm(x, None, self.weight, self.eps, out, rows)
        return out

    def fuse_spec(self, ctx, n):
        return None

    def emit_spec(self, ctx, n):
        return None


class StreamsBlock(Block):
    replayable = True
    taped = True

    def __init__(self, streams: int, mixer_norm: RMSNorm, mixer: Mixer, ffn_norm: Optional[RMSNorm] = None,
                 ffn: Optional[FeedForward] = None, names=("norm1", "mix", "norm2", "mlp", "hc1", "hc2")):
        if not 1 <= streams <= ops.MAX_STREAMS:
            raise ValueError(f"{streams} streams: between 1 and {ops.MAX_STREAMS}")
        for part in (mixer, ffn):
            if part is not None and not getattr(part, "accepts_store", False):
                raise ValueError(f"{type(part).__name__} cannot write its rows instead of adding them (accepts_store)")
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward and its norm come together")
        self.streams = streams
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn
        self.names = tuple(names)
        self.sublayers = 2 if ffn is not None else 1
        # per sublayer, its weights on the streams: in [S], out [S], mix [S, S]
        self.hc1_in = self.hc1_out = self.hc1_mix = self.hc2_in = self.hc2_out = self.hc2_mix = None

    def children(self) -> Dict[str, Part]:
        out = {self.names[0]: self.mixer_norm, self.names[1]: self.mixer}
        if self.ffn is not None:
            out[self.names[2]] = self.ffn_norm
            out[self.names[3]] = self.ffn
        return out

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        S, specs = self.streams, {}
        for name in self.names[4:4 + self.sublayers]:
            specs[f"{name}.in"] = TensorSpec((S,), kind="f32", init="ones")
            specs[f"{name}.out"] = TensorSpec((S,), kind="f32", init="ones")
            specs[f"{name}.mix"] = TensorSpec((S, S), kind="f32", init="eye")
        return specs

    def load(self, tensors):
        first, second = self.names[4], self.names[5]
        self.hc1_in, self.hc1_out, self.hc1_mix = (tensors[f"{first}.{t}"].contiguous() for t in ("in", "out", "mix"))
        if self.sublayers == 2:
            self.hc2_in, self.hc2_out, self.hc2_mix = (tensors[f"{second}.{t}"].contiguous() for t in ("in", "out", "mix"))

    def cache_spec(self) -> Optional[CacheSpec]:
        return self.mixer.cache_spec

    def state_spec(self) -> Optional[StateSpec]:
        return self.mixer.state_spec

    def entry_norm(self, ctx, n: int):
        """What the block before needs to do this block's first norm in the pass that updates the streams with its
        last sublayer: ``(in weights, gamma, eps)`` (``forward(..., pre=)`` then takes the rows it made)."""
        return (self.hc1_in, self.mixer_norm.weight, self.mixer_norm.eps) if ctx.tuned else None

    def forward(self, ctx, x, cache: Optional[LayerCache], pre=None, emit=None):
        """``x``: the streams, float32 [streams, n, width], updated in place.  ``pre``: a ``Normed`` with the rows of this
        block's first norm, from the block before; ``emit``: the ``entry_norm`` of the block after, whose rows this
        block then returns as a ``Normed``.  An update of the streams and the norm that reads them next are one kernel."""
        n, width = x.shape[1], x.shape[2]
        y = ctx.buffer("streams_y", (n, width), torch.float32)
        h = ctx.buffer("h", (n, width), ctx.dtype)
        if isinstance(pre, Normed):
            h = pre.rows
        else:
            ops.streams_norm(x, self.hc1_in, self.mixer_norm.weight, self.mixer_norm.eps, h)
        self.mixer.forward(ctx, h, y, cache, store=True)
        last = (self.hc1_mix, self.hc1_out, y)
        if self.ffn is not None:
            if ctx.tuned:
                ops.streams_norm(x, self.hc2_in, self.ffn_norm.weight, self.ffn_norm.eps, h, update=last)
            else:
                ops.streams_mix(x, *last)
                ops.streams_norm(x, self.hc2_in, self.ffn_norm.weight, self.ffn_norm.eps, h)
            self.ffn.forward(ctx, h, y, store=True)
            last = (self.hc2_mix, self.hc2_out, y)
        if emit is not None:
            w_in, gamma, eps = emit
            handed = ctx.buffer("h_next", (n, width), ctx.dtype)
            ops.streams_norm(x, w_in, gamma, eps, handed, update=last)
            return Normed(handed)
        ops.streams_mix(x, *last)
        return None
