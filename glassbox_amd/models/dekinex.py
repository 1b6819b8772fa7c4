"""The Dekinex decoder assembled from parts.

Every layer is one norm (the file holds its weight minus one) whose rows feed a mixer and, where the configuration gives one,
a feed-forward; their sum, times a constant, goes into the residual (``ParallelBlock``).  The mixers: attention behind a
short convolution (``ShortConvAttention``) and a matrix memory with exponential gates (``MLSTM``); the feed-forwards: a
gated unit with clamped halves (``ClampedGLU``) and routed experts with a shared one (``RoutedExperts``).  A run of
layers may be repeated with the same weights: the schedule names those blocks again, each pass with a cache layer
(pages and state) of its own, and marks the call with which a pass begins (``PassEntry``).  The embedding adds a row
chosen by the token and the one before it (``PairHashEmbedding``).  Tensor names: ``embed``, ``bigram``, ``loop.step``,
``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.dekinex import DekinexConfig
from ..parts.attention import ShortConvAttention
from ..parts.block import ParallelBlock
from ..parts.embedding import Embedding, LMHead, PairHashEmbedding
from ..parts.linear_attention import MLSTM
from ..parts.mlp import ClampedGLU
from ..parts.model import DecoderModel, LayerCall, PassEntry
from ..parts.moe import RoutedExperts
from ..parts.norm import RMSNorm


def _mixer(cfg: DekinexConfig, layer):
    m, d, eps = layer["mixer"], cfg.width, cfg.norm_eps
    if layer["type"] == "attention":
        rot = m.get("rot") or {"dims": 0, "base": 1.0}
        return ShortConvAttention(d, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["scale"],
                                  (m.get("mask") or {"size": 0})["size"], m.get("conv", 0), rot["dims"], rot["base"],
                                  qk_norm=True, eps=eps)
    return MLSTM(d, m["heads"], m["dim"], m["vdim"], m["gate_cap"], eps)


def _ffn(cfg: DekinexConfig, mlp):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return ClampedGLU(cfg.width, mlp["ff"], mlp["limit"])
    r = mlp["router"]
    return RoutedExperts(cfg.width, r["experts"], r["top"], mlp["expert"]["ff"], r["scale"],
                         (mlp.get("shared") or {"ff": 0})["ff"])


def _source(name: str) -> str:
    """The checkpoint names a norm or a table by its place alone."""
    if name.endswith(".weight"):
        name = name[:-len(".weight")]
    return {"embed.pairs": "bigram"}.get(name, name)


def build_dekinex(cfg: DekinexConfig) -> DecoderModel:
    d, eps = cfg.width, cfg.norm_eps
    blocks = [ParallelBlock(RMSNorm(d, eps, offset=1.0), _mixer(cfg, layer), _ffn(cfg, layer["mlp"]), cfg.residual_mult)
              for layer in cfg.layers]
    schedule = [LayerCall(block=b, cache=c, enter=t) for c, (b, t) in enumerate(cfg.layer_order())]
    if cfg.bigram is not None:
        embedding = PairHashEmbedding(cfg.vocab, d, *cfg.bigram)
    else:
        embedding = Embedding(cfg.vocab, d)
    passes = PassEntry(cfg.loop[2], d) if cfg.loop is not None else None
    return DecoderModel(cfg, embedding, blocks, schedule, RMSNorm(d, eps, offset=1.0), LMHead(cfg.vocab, d, any_size=True),
                        names=("embed", "l{}", "final.norm", "head"), sources=_source, passes=passes, passes_name="loop",
                        arg_keys={"width": "width", "dim": "layers[].mixer.dim", "taps": "layers[].mixer.conv",
                                  "n_experts": "layers[].mlp.router.experts", "top": "layers[].mlp.router.top",
                                  "vocab": "vocab"})


register_architecture("Dekinex", DekinexConfig, build_dekinex)
