"""The Sagalorn decoder assembled from parts.

Every layer is one mixer (retention, attention whose values are its keys, or gated linear attention) and, where the
configuration gives one, a SwiGLU feed-forward, each behind an RMS norm.  With ``streams`` the residual is that many
streams and a layer is a ``StreamsBlock``; without, a plain pre-norm block.  A run of layers may be repeated with the
same weights: the schedule names those blocks again, each pass with a cache layer (pages or state) of its own.  The
embedding and the logits are scaled.  Tensor names: ``embed``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.norm2``,
``l<i>.mlp.gate|up|down``, ``l<i>.hc1|hc2.in|out|mix``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from ..config import register_architecture
from ..config.sagalorn import SagalornConfig
from ..parts.attention import TiedValueAttention
from ..parts.block import MixerOnlyBlock, PreNormBlock
from ..parts.embedding import Embedding, LMHead
from ..parts.linear_attention import GatedLinearAttention, Retention
from ..parts.mlp import SwiGLU
from ..parts.model import DecoderModel, LayerCall
from ..parts.norm import RMSNorm
from ..parts.streams import StreamsBlock, StreamsSumNorm


def _mixer(cfg: SagalornConfig, layer):
    m, d, eps = layer["mixer"], cfg.width, cfg.norm_eps
    if layer["type"] == "retention":
        rot = m.get("rot") or {"dims": 0, "base": 1.0}
        return Retention(d, m["heads"], m["dim"], m["vdim"], m["decay"], eps, rot["dims"], rot["base"])
    if layer["type"] == "attention":
        mask = m.get("mask") or {"size": 0, "keep_first": 0}
        return TiedValueAttention(d, m["heads"], m["kv_heads"], m["dim"], m["scale"], mask["size"], mask["keep_first"],
                                  bias=True, qk_norm=True, eps=eps)
    return GatedLinearAttention(d, m["heads"], m["dim"], m["vdim"], m["tau"], eps, m.get("rank"))


def _source(name: str) -> str:
    """The checkpoint names a norm, a table or a projection by its place alone."""
    if name.endswith(".weight"):
        name = name[:-len(".weight")]
    return name.replace("_proj", "")


def build_sagalorn(cfg: SagalornConfig) -> DecoderModel:
    d, eps = cfg.width, cfg.norm_eps
    blocks = []
    for layer in cfg.layers:
        mixer = _mixer(cfg, layer)
        ffn = SwiGLU(d, layer["mlp"]["ff"], any_size=True) if layer["mlp"] is not None else None
        if cfg.streams is not None:
            blocks.append(StreamsBlock(cfg.streams, RMSNorm(d, eps), mixer, RMSNorm(d, eps) if ffn is not None else None, ffn))
        elif ffn is not None:
            blocks.append(PreNormBlock(RMSNorm(d, eps), mixer, RMSNorm(d, eps), ffn, names=("norm1", "mix", "norm2", "mlp")))
        else:
            blocks.append(MixerOnlyBlock(RMSNorm(d, eps), mixer))
    schedule = [LayerCall(block=b, cache=c) for c, b in enumerate(cfg.layer_order())]
    final = StreamsSumNorm(d, eps) if cfg.streams is not None else RMSNorm(d, eps)
    return DecoderModel(cfg, Embedding(cfg.vocab, d, cfg.embedding_scale), blocks, schedule, final,
                        LMHead(cfg.vocab, d, scale=cfg.logit_scale, any_size=True), names=("embed", "l{}", "final.norm", "head"),
                        sources=_source, streams=cfg.streams,
                        arg_keys={"width": "width", "intermediate": "layers[].mlp.ff", "dim": "layers[].mixer.dim",
                                  "heads * dim": "layers[].mixer.heads, dim", "heads * vdim": "layers[].mixer.heads, vdim",
                                  "vocab": "vocab"})


register_architecture("Sagalorn", SagalornConfig, build_sagalorn)
