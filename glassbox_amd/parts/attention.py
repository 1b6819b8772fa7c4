"""Grouped-query attention over the paged cache: the mixer of a Llama layer.

qkv = h . Wqkv^T (query rows, then key rows, then value rows stacked, as the
reference stacks them: crates/glassbox-core/src/model.rs:59-61,260-265);
positions are encoded and keys/values written to the pages
(model.rs:266-276); every token attends to its own request's positions up to
its own through the block table (model.rs:285-312); the output projection is
added into the residual (model.rs:322-325).
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .. import ops
from .base import (FULL, WINDOW, CacheSpec, LayerCache, Mixer, PositionEncoding, PreNormed, StateSpec, TensorSpec, emit_target,
                   needs_multiple_of_8, product, split_workspace)


def paged_attention(ctx, q: torch.Tensor, out: torch.Tensor, cache: LayerCache, n_heads: int, scale: float,
                    window: int, keep_first: int = 0) -> None:
    """Attention of every row of the step over its request's pages.  ``window`` > 0: a token reads the last so many
    keys up to its own, and with ``keep_first`` the request's first so many keys as well, wherever they lie.

    float32 always takes the plain kernel.  bfloat16 takes the tuned kernels where they apply: requests with
    one row go to the split-context decode kernel, longer portions to the matrix-core prefill kernel; a step
    with ``ctx.tuned`` off takes the plain kernel throughout."""
    if (ctx.dtype == torch.float32 or not ctx.tuned
            or not ops.tuned_attention_supports(cache.k_pages, n_heads, window, keep_first)):
        longest = int(ctx.host["max_context"])
        _, _, n_pieces, page_size, piece = cache.k_pages.shape
        tables = ctx.tables[cache.group]

        def rows(a, b, grouped):
            # few tokens with long contexts (a decode step): a workgroup a chunk of the context, merged by a second kernel
            floats = 0 if grouped else ops.attention_plain_split_floats(b - a, n_heads, n_pieces * piece, page_size, longest,
                                                                        keep_first)
            ws = ctx.buffer("attention_plain_parts", (floats,), torch.float32) if floats else None
            ops.attention_plain(q[a:b], out[a:b], ctx.positions[a:b], ctx.tok_seq[a:b], tables, cache.k_pages, cache.v_pages,
                                n_heads, scale, window, workspace=ws, max_context=longest, grouped=grouped,
                                keep_first=keep_first)

        # the rows of requests with one token come first; many rows of prompt portions go eight rows a workgroup
        n, n_decode = q.shape[0], ctx.host["n_decode"]
        if n - n_decode >= ops.PLAIN_GROUP_MIN_ROWS and window == 0:
            if n_decode > 0:
                rows(0, n_decode, False)
            rows(n_decode, n, True)
        else:
            rows(0, n, False)
        return
    n_decode = ctx.host["n_decode"]
    if n_decode > 0:
        ops.attention_decode(q, out, ctx, cache, n_heads, scale, window, keep_first)
    if n_decode < ctx.num_seqs:
        ops.attention_prefill(q, out, ctx, cache, n_heads, scale, window, keep_first)


class PagedAttention(Mixer):
    replayable = True
    taped = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, position: PositionEncoding,
                 window: int = 0, shares_kv: bool = False, scale: Optional[float] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.position = position
        self.window = int(window)
        self.shares_kv = shares_kv          # reads another layer's pages; has no key/value projections
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)  # model.rs:244
        self.q_dim = n_heads * head_dim
        self.kv_dim = n_kv_heads * head_dim
        self.cache_spec = None if shares_kv else CacheSpec(n_kv_heads, head_dim,
                                                           WINDOW if window > 0 else FULL, self.window)
        self.wqkv: Optional[torch.Tensor] = None
        self.wo: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"q_proj.weight": TensorSpec((self.q_dim, self.width))}
        if not self.shares_kv:
            specs["k_proj.weight"] = TensorSpec((self.kv_dim, self.width))
            specs["v_proj.weight"] = TensorSpec((self.kv_dim, self.width))
        specs["o_proj.weight"] = TensorSpec((self.width, self.q_dim))
        return specs

    def children(self):
        return {"": self.position} if self.position.tensor_specs() else {}

    def all_replayable(self) -> bool:
        return self.replayable and self.position.all_replayable()

    def all_taped(self) -> bool:
        return self.taped and self.position.all_taped()

    def load(self, tensors):
        if self.shares_kv:
            self.wqkv = tensors["q_proj.weight"].contiguous()
        else:
            # one product computes all three (model.rs:59-61)
            self.wqkv = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], 0)
        self.wo = tensors["o_proj.weight"].contiguous()

    def streamed_matrices(self):
        return [self.wqkv, self.wo]

    def problems(self, dtype, page_size):
        out = needs_multiple_of_8(dtype, "width", self.width) + needs_multiple_of_8(dtype, "n_heads * head_dim", self.q_dim)
        if self.head_dim > ops.MAX_HEAD_DIM:
            out.append(("head_dim", f"{self.head_dim} is above {ops.MAX_HEAD_DIM}, the largest head the attention kernels take"))
        return out + self.position.problems(dtype, page_size)

    accepts_fused_norm = True
    accepts_emit_norm = True

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], norm=None, emit=None):
        """``norm=(gamma, eps)``: h is the un-normed float32 residual and the first product norms it;
        ``norm=PreNormed``: the product before has done most of that.  ``emit=(gamma, eps)``: the output
        projection may prepare the norm that reads the residual next (returns a PreNormed if it did)."""
        if cache is None or cache.k_pages is None:
            raise ValueError("PagedAttention needs a layer cache with pages")
        n = h.shape[0]
        rows = self.q_dim + (0 if self.shares_kv else 2 * self.kv_dim)
        qkv = ctx.buffer("qkv", (n, rows), ctx.dtype)
        write = cache.writable and not self.shares_kv
        store = (ctx.slots[cache.group], cache.k_pages, cache.v_pages) if write else (None, None, None)
        n_kv = 0 if self.shares_kv else self.n_kv_heads
        pre = isinstance(norm, PreNormed)
        # few rows (decoding): the product's epilogue rotates the heads and writes the cache itself
        tables = None
        if (ctx.dtype == torch.bfloat16 and ctx.fuse_norms and n <= ops.ROPE_PRODUCT_MAX_ROWS
                and self.head_dim % 16 == 0):
            tables = self.position.fuse_spec(ctx, self.head_dim)
        if tables is not None:
            ops.gemm_rope(norm.rows if pre else h, self.wqkv, qkv, self.n_heads, n_kv, self.head_dim, tables[0],
                          tables[1], *store, rms=None if pre else norm, rms_parts=norm.as_gemm_arg() if pre else None)
        else:
            if pre:
                ops.gemm(norm.rows, self.wqkv, qkv, rms_parts=norm.as_gemm_arg())
            else:
                ops.gemm(h, self.wqkv, qkv, rms=norm,
                         workspace=None if norm is not None else split_workspace(ctx, n, rows, self.width))
            self.position.apply_and_store(ctx, qkv, self.n_heads, n_kv, self.head_dim, *store)
        att = ctx.buffer("att", (n, self.q_dim), ctx.dtype)
        paged_attention(ctx, qkv[:, :self.q_dim], att, cache, self.n_heads, self.scale, self.window)
        target, handed_on = emit_target(ctx, n, self.width, self.q_dim, emit, "mixer")
        ops.gemm(att, self.wo, residual, accumulate=True, emit=target,
                 workspace=split_workspace(ctx, n, self.width, self.q_dim))
        return handed_on


class TiedValueAttention(Mixer):
    """Grouped-query attention whose values are its keys: there is no value projection, and a key head as projected
    (bias included, before any norm) is the value head.  Options, each a constructor argument: biases on the query,
    key and output projections; an RMS norm of every query and key head over its dimensions, with a weight for the
    queries and one for the keys that the heads share; the scale of the scores; a window of the last ``window`` keys,
    with the request's first ``keep_first`` keys visible for good.  Positions do not enter the scores.

    Tensors: ``q``, ``k``, ``o`` (and ``q.b``, ``k.b``, ``o.b``; ``q.norm``, ``k.norm``)."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, scale: Optional[float] = None,
                 window: int = 0, keep_first: int = 0, bias: bool = True, qk_norm: bool = True, eps: float = 1e-5):
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        if keep_first and not window:
            raise ValueError("kept first keys go with a window")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.window, self.keep_first = int(window), int(keep_first)
        self.bias, self.qk_norm, self.eps = bool(bias), bool(qk_norm), float(eps)
        self.q_dim, self.kv_dim = n_heads * head_dim, n_kv_heads * head_dim
        self.cache_spec = CacheSpec(n_kv_heads, head_dim, WINDOW if window > 0 else FULL, self.window, self.keep_first)
        self.wqk = self.wo = self.bias_q = self.bias_k = self.bias_o = self.norm_q = self.norm_k = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {"q": TensorSpec((self.q_dim, self.width)), "k": TensorSpec((self.kv_dim, self.width)),
                 "o": TensorSpec((self.width, self.q_dim))}
        if self.bias:
            specs.update({"q.b": TensorSpec((self.q_dim,), kind="f32", init="normal"),
                          "k.b": TensorSpec((self.kv_dim,), kind="f32", init="normal"),
                          "o.b": TensorSpec((self.width,), kind="f32", init="normal")})
        if self.qk_norm:
            specs.update({"q.norm": TensorSpec((self.head_dim,), kind="f32", init="ones"),
                          "k.norm": TensorSpec((self.head_dim,), kind="f32", init="ones")})
        return specs

    def load(self, tensors):
        self.wqk = torch.cat([tensors["q"], tensors["k"]], 0)   # one product computes both
        self.wo = tensors["o"].contiguous()
        if self.bias:
            self.bias_q, self.bias_k, self.bias_o = (tensors[n].contiguous() for n in ("q.b", "k.b", "o.b"))
        if self.qk_norm:
            self.norm_q, self.norm_k = tensors["q.norm"].contiguous(), tensors["k.norm"].contiguous()

    def streamed_matrices(self):
        return [self.wqk, self.wo]

    def problems(self, dtype, page_size):
        out = []   # (sizes that the matrix-core products do not take go through the plain product)
        if self.head_dim > ops.MAX_HEAD_DIM:
            out.append(("dim", f"{self.head_dim} is above {ops.MAX_HEAD_DIM}, the largest head the attention kernels take"))
        return out

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``, or with ``store`` writes them there (float32 either way)."""
        if cache is None or cache.k_pages is None:
            raise ValueError("TiedValueAttention needs a layer cache with pages")
        n = h.shape[0]
        slots = ctx.slots[cache.group] if cache.writable else None
        if n > ops.ROPE_PRODUCT_MAX_ROWS and slots is not None:
            # many rows: values are written into the rows behind the keys, and the kernel that takes a step's keys and
            # values to their pages in whole lines does the cache write (no rotation)
            rows = ctx.buffer("qkv", (n, self.q_dim + 2 * self.kv_dim), ctx.dtype)
            qk = rows[:, :self.q_dim + self.kv_dim]
            product(ctx, h, self.wqk, qk)
            ops.qk_norm_store(rows, self.bias_q, self.bias_k, self.norm_q, self.norm_k, self.eps, None, None, None,
                              self.n_heads, self.n_kv_heads, self.head_dim, values_in_rows=True)
            ops.rope_store(rows, None, None, slots, cache.k_pages, cache.v_pages, self.n_heads, self.n_kv_heads,
                           self.head_dim, rotate=False, portions=ctx.portions())
        else:
            qk = ctx.buffer("qk", (n, self.q_dim + self.kv_dim), ctx.dtype)
            product(ctx, h, self.wqk, qk)
            ops.qk_norm_store(qk, self.bias_q, self.bias_k, self.norm_q, self.norm_k, self.eps, slots,
                              cache.k_pages if slots is not None else None, cache.v_pages if slots is not None else None,
                              self.n_heads, self.n_kv_heads, self.head_dim)
        att = ctx.buffer("att", (n, self.q_dim), ctx.dtype)
        paged_attention(ctx, qk[:, :self.q_dim], att, cache, self.n_heads, self.scale, self.window, self.keep_first)
        product(ctx, att, self.wo, residual, accumulate=not store)
        if self.bias_o is not None:
            ops.add_bias(residual, self.bias_o)


def cache_head_cols(dim: int, vdim: int) -> int:
    """Columns of a head in the pages of a layer whose keys have ``dim`` channels and whose values have ``vdim``: the
    cache and the attention kernels work on heads of one size, so both are filled up with zeros (which change neither a
    score nor a weighted sum) to the larger of the two, and on to a multiple of 16 where the matrix-core kernels then
    take the head, else to a multiple of 8."""
    most = max(dim, vdim)
    cols = -(-most // 16) * 16
    return cols if cols <= 128 else -(-most // 8) * 8


class ShortConvAttention(Mixer):
    """Grouped-query attention whose projections pass a short causal convolution over time before anything else:
    q, k, v = W h; each channel of the three convolved over its request's tokens with ``taps`` weights (``q.conv`` ...,
    [channels, taps], zeros before the first token; ``taps`` 0: no convolution); the first ``rot_dims`` channels of every
    query and key head turned by the position in neighbouring pairs (2i, 2i + 1), frequencies base^(-2i / rot_dims);
    with ``qk_norm`` every query and key head divided by its root mean square; scores q . k * scale over the last
    ``window`` keys (0: all); softmax; output projection.  Key and value heads may differ in size (``dim``, ``vdim``).

    The request's last taps - 1 projections are its state (``state_spec``), beside the pages of keys and values."""
    replayable = True
    taped = True
    accepts_store = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, dim: int, vdim: int, scale: Optional[float] = None,
                 window: int = 0, taps: int = 0, rot_dims: int = 0, rot_base: float = 10000.0, qk_norm: bool = True,
                 eps: float = 1e-5):
        from .rotary import Rotary
        if n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads are not a multiple of {n_kv_heads} key heads")
        if rot_dims % 2 or not 0 <= rot_dims <= dim:
            raise ValueError(f"{rot_dims} rotated channels: an even number up to the key size {dim}")
        self.width, self.n_heads, self.n_kv_heads, self.dim, self.vdim = width, n_heads, n_kv_heads, dim, vdim
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(dim)
        self.window, self.taps, self.rot_dims = int(window), int(taps), int(rot_dims)
        self.qk_norm, self.eps = bool(qk_norm), float(eps)
        self.head_cols = cache_head_cols(dim, vdim)
        self.channels = (n_heads + n_kv_heads) * dim + n_kv_heads * vdim
        self.position = Rotary(rot_dims, rot_base) if rot_dims else None
        self.cache_spec = CacheSpec(n_kv_heads, self.head_cols, WINDOW if window > 0 else FULL, self.window)
        self.state_spec = StateSpec((self.taps - 1, self.channels), torch.float32, 0.0) if self.taps > 1 else None
        self.wqkv = self.wo = self.wconv = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        H, G, D, V = self.n_heads, self.n_kv_heads, self.dim, self.vdim
        specs = {"q": TensorSpec((H * D, self.width)), "k": TensorSpec((G * D, self.width)),
                 "v": TensorSpec((G * V, self.width)), "o": TensorSpec((self.width, H * V))}
        if self.taps:
            specs.update({"q.conv": TensorSpec((H * D, self.taps), kind="f32"), "k.conv": TensorSpec((G * D, self.taps), kind="f32"),
                          "v.conv": TensorSpec((G * V, self.taps), kind="f32")})
        return specs

    def load(self, tensors):
        parts = [tensors["q"], tensors["k"], tensors["v"]]
        if self.channels % 8:   # rows of the product's result then begin at 16-byte words
            parts.append(torch.zeros((8 - self.channels % 8, self.width), dtype=parts[0].dtype, device=parts[0].device))
        self.wqkv = torch.cat(parts, 0)
        # the output projection takes heads of head_cols columns, the columns beyond vdim being zero
        o = tensors["o"]
        wo = torch.zeros((self.width, self.n_heads, self.head_cols), dtype=o.dtype, device=o.device)
        wo[:, :, :self.vdim] = o.view(self.width, self.n_heads, self.vdim)
        self.wo = wo.view(self.width, self.n_heads * self.head_cols)
        if self.taps:
            self.wconv = torch.cat([tensors["q.conv"], tensors["k.conv"], tensors["v.conv"]], 0).float().contiguous()

    def streamed_matrices(self):
        return [self.wqkv, self.wo]

    def problems(self, dtype, page_size):
        out = []
        if self.head_cols > ops.MAX_HEAD_DIM:
            out.append(("dim", f"heads of {max(self.dim, self.vdim)} channels are above {ops.MAX_HEAD_DIM}, the largest head "
                               f"the attention kernels take"))
        if self.taps > ops.CONV_MAX_TAPS:
            out.append(("taps", f"{self.taps} is above {ops.CONV_MAX_TAPS}, the longest convolution the kernel takes"))
        return out

    def forward(self, ctx, h, residual, cache: Optional[LayerCache], store: bool = False):
        """Adds the mixed rows into ``residual``, or with ``store`` writes them there (float32 either way)."""
        if cache is None or cache.k_pages is None or (self.taps > 1 and cache.state is None):
            raise ValueError("ShortConvAttention needs a layer cache with pages (and state, with a convolution)")
        n = h.shape[0]
        H, G, hc = self.n_heads, self.n_kv_heads, self.head_cols
        proj = ctx.buffer("conv_proj", (n, self.wqkv.shape[0]), ctx.dtype)
        product(ctx, h, self.wqkv, proj)
        cos, sin = self.position.table(ctx) if self.position is not None else (None, None)
        heads = ctx.buffer("conv_heads", (n, (H + 2 * G) * hc), ctx.dtype)
        slots = ctx.slots[cache.group] if cache.writable else None
        direct = slots is not None and n <= ops.ROPE_PRODUCT_MAX_ROWS
        ops.conv_heads(proj, self.wconv, cache.state, ctx, cos, sin, self.rot_dims, self.eps, self.qk_norm, heads, hc,
                       slots if direct else None, cache.k_pages, cache.v_pages, H, G, self.dim, self.vdim)
        if slots is not None and not direct:
            # many rows: the kernel that takes a step's keys and values to their pages in whole lines
            ops.rope_store(heads, None, None, slots, cache.k_pages, cache.v_pages, H, G, hc, rotate=False,
                           portions=ctx.portions())
        att = ctx.buffer("att", (n, H * hc), ctx.dtype)
        paged_attention(ctx, heads[:, :H * hc], att, cache, H, self.scale, self.window)
        product(ctx, att, self.wo, residual, accumulate=not store)
