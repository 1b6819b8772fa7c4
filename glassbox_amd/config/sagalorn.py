"""Configuration of the Sagalorn decoder: a list of layers, each with one of three mixers (retention, attention,
gated linear attention) and an optional dense feed-forward; a run of layers that is repeated with the same weights;
a residual of several streams; a scaled embedding and scaled logits.

``config.json`` is nested, and this class keeps it as it is read (``layers`` as a tuple of mappings), checked key by
key here so that the builder can rely on it:

  architecture, vocab, width, streams (absent: one plain residual), logit_scale, embedding.scale, norm.eps,
  loop {start, stop, times} (absent or null: every layer once),
  layers[i] {type, mixer {...}, mlp {kind: "dense", ff} or null}
    retention: heads, dim, vdim, decay [heads], rot {dims, base} (absent: no rotation)
    attention: heads, kv_heads, dim, vdim (= dim: the values are the keys), scale, mask {size, keep_first} (absent: every
               earlier key)
    gla:       heads, dim, vdim, tau; optionally rank (else the checkpoint's tensors give it)
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig

MIXERS = ("retention", "attention", "gla")


def _int(where: str, raw: Dict[str, Any], key: str, default=None, least: int = 1) -> int:
    v = raw.get(key, default)
    if v is None:
        raise ConfigError(f"{where} lacks the key {key!r}")
    if isinstance(v, float) and v == int(v):
        v = int(v)
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"{where}: {key!r} must be an integer of at least {least}, got {v!r}")
    return v


def _num(where: str, raw: Dict[str, Any], key: str, default=None) -> float:
    v = raw.get(key, default)
    if v is None:
        raise ConfigError(f"{where} lacks the key {key!r}")
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v):
        raise ConfigError(f"{where}: {key!r} must be a number, got {v!r}")
    return float(v)


def _check_layer(i: int, layer: Any) -> Dict[str, Any]:
    where = f"layers[{i}]"
    if not isinstance(layer, dict) or layer.get("type") not in MIXERS or not isinstance(layer.get("mixer"), dict):
        raise ConfigError(f"{where} must have a 'type' out of {', '.join(MIXERS)} and a 'mixer' object")
    kind, m = layer["type"], dict(layer["mixer"])
    mw = f"{where}.mixer"
    out: Dict[str, Any] = {"heads": _int(mw, m, "heads"), "dim": _int(mw, m, "dim")}
    out["vdim"] = _int(mw, m, "vdim", out["dim"])
    if kind == "retention":
        decay = m.get("decay")
        if not isinstance(decay, list) or len(decay) != out["heads"] or any(
                isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(f"{mw}: 'decay' must list one number for each of the {out['heads']} heads")
        out["decay"] = tuple(float(d) for d in decay)
        rot = m.get("rot")
        if rot is not None:
            if not isinstance(rot, dict):
                raise ConfigError(f"{mw}: 'rot' must be an object with 'dims' and 'base'")
            dims = _int(f"{mw}.rot", rot, "dims", least=0)
            if dims % 2 or dims > out["dim"]:
                raise ConfigError(f"{mw}.rot: 'dims' must be even and at most dim, got {dims}")
            out["rot"] = {"dims": dims, "base": _num(f"{mw}.rot", rot, "base")}
            if dims and not out["rot"]["base"] > 0:
                raise ConfigError(f"{mw}.rot: 'base' must be positive")
    elif kind == "attention":
        out["kv_heads"] = _int(mw, m, "kv_heads", out["heads"])
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{mw}: heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
        if out["vdim"] != out["dim"]:
            raise ConfigError(f"{mw}: the values are the keys, so vdim ({out['vdim']}) must equal dim ({out['dim']})")
        out["scale"] = _num(mw, m, "scale", 1.0 / math.sqrt(out["dim"]))
        mask = m.get("mask")
        if mask is not None:
            if not isinstance(mask, dict):
                raise ConfigError(f"{mw}: 'mask' must be an object with 'size' and 'keep_first'")
            out["mask"] = {"size": _int(f"{mw}.mask", mask, "size"),
                           "keep_first": _int(f"{mw}.mask", mask, "keep_first", 0, least=0)}
    else:
        out["tau"] = _num(mw, m, "tau", 1.0)
        if not out["tau"] > 0:
            raise ConfigError(f"{mw}: 'tau' must be positive")
        if m.get("rank") is not None:
            out["rank"] = _int(mw, m, "rank")
    mlp = layer.get("mlp")
    if mlp is not None:
        if not isinstance(mlp, dict) or mlp.get("kind", "dense") != "dense":
            raise ConfigError(f"{where}.mlp must be null or an object of kind 'dense', got {mlp!r}")
        mlp = {"kind": "dense", "ff": _int(f"{where}.mlp", mlp, "ff")}
    return {"type": kind, "mixer": out, "mlp": mlp}


@dataclass(frozen=True)
class SagalornConfig(ModelConfig):
    architecture = "Sagalorn"

    vocab: int
    width: int
    layers: Tuple[Dict[str, Any], ...]
    norm_eps: float
    streams: Optional[int] = None
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    loop: Optional[Tuple[int, int, int]] = None   # (start, stop, times)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "SagalornConfig":
        where = "config.json of Sagalorn"
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where} lacks a non-empty list 'layers'")
        checked = tuple(_check_layer(i, layer) for i, layer in enumerate(layers))
        norm = raw.get("norm")
        if not isinstance(norm, dict):
            raise ConfigError(f"{where} lacks the object 'norm' with 'eps'")
        eps = _num("norm", norm, "eps")
        if not eps > 0:
            raise ConfigError("norm: 'eps' must be positive")
        loop = raw.get("loop")
        if loop is not None:
            if not isinstance(loop, dict):
                raise ConfigError("'loop' must be null or an object with 'start', 'stop' and 'times'")
            start, stop = _int("loop", loop, "start", least=0), _int("loop", loop, "stop", least=0)
            times = _int("loop", loop, "times", 1)
            if not start <= stop <= len(checked):
                raise ConfigError(f"loop: layers {start} to {stop} do not lie among the {len(checked)} layers")
            loop = (start, stop, times)
        emb = raw.get("embedding") or {}
        if not isinstance(emb, dict):
            raise ConfigError("'embedding' must be an object with 'scale'")
        streams = raw.get("streams")
        if streams is not None:
            streams = _int(where, raw, "streams")
        return cls(vocab=_int(where, raw, "vocab"), width=_int(where, raw, "width"), layers=checked, norm_eps=eps,
                   streams=streams, embedding_scale=_num("embedding", emb, "scale", 1.0),
                   logit_scale=_num(where, raw, "logit_scale", 1.0), loop=loop)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "embedding": {"scale": self.embedding_scale}, "norm": {"eps": self.norm_eps},
                               "logit_scale": self.logit_scale,
                               "layers": [{"type": l["type"], "mixer": _plain(l["mixer"]), "mlp": _plain(l["mlp"])}
                                          for l in self.layers]}
        if self.streams is not None:
            out["streams"] = self.streams
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return out

    def layer_order(self) -> Tuple[int, ...]:
        """The layers in the order a step runs them: the looped run so many times in a row, the rest once."""
        n = len(self.layers)
        if self.loop is None:
            return tuple(range(n))
        start, stop, times = self.loop
        return tuple(range(start)) + tuple(range(start, stop)) * times + tuple(range(stop, n))


def _plain(v):
    if isinstance(v, dict):
        return {k: _plain(x) for k, x in v.items()}
    if isinstance(v, tuple):
        return [_plain(x) for x in v]
    return v
