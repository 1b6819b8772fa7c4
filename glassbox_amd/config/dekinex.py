"""Configuration of the Dekinex decoder: a list of layers, each with one of two mixers (attention behind a short
convolution, or a matrix memory with exponential gates) and a feed-forward (a dense gated unit with clamped halves,
routed experts, or none) that reads the same normed rows as the mixer; a run of layers that is repeated with the same
weights, with something added to the residual where each pass begins; an embedding with a hashed table of token pairs.

``config.json`` is nested, and this class keeps it as it is read (``layers`` as a tuple of mappings), checked key by
key here so that the builder can rely on it:

  architecture, vocab, width, residual_mult, norm {eps},
  embedding {bigram {buckets, mul_prev, mul_cur}} (absent: the token's row alone),
  loop {start, stop, times} (absent or null: every layer once),
  layers[i] {type, mixer {...}, mlp {...} or null}
    attention: heads, kv_heads, dim, vdim, scale, conv (taps; absent: no convolution), rot {dims, base} (absent: no
               rotation), mask {size} (absent: every earlier key)
    mlstm:     heads, dim, vdim, gate_cap
    mlp dense: kind "dense", ff, limit
    mlp moe:   kind "moe", expert {ff}, router {experts, top, scale}, shared {ff} (absent: no shared expert)
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Dict, Optional, Tuple

from .base import ConfigError, ModelConfig
from .sagalorn import _int, _num, _plain

MIXERS = ("attention", "mlstm")


def _obj(where: str, raw: Dict[str, Any], key: str, required: bool = False) -> Optional[Dict[str, Any]]:
    v = raw.get(key)
    if v is None:
        if required:
            raise ConfigError(f"{where} lacks the object {key!r}")
        return None
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: {key!r} must be an object, got {v!r}")
    return v


def _check_layer(i: int, layer: Any) -> Dict[str, Any]:
    where = f"layers[{i}]"
    if not isinstance(layer, dict) or layer.get("type") not in MIXERS or not isinstance(layer.get("mixer"), dict):
        raise ConfigError(f"{where} must have a 'type' out of {', '.join(MIXERS)} and a 'mixer' object")
    kind, m = layer["type"], layer["mixer"]
    mw = f"{where}.mixer"
    out: Dict[str, Any] = {"heads": _int(mw, m, "heads"), "dim": _int(mw, m, "dim")}
    out["vdim"] = _int(mw, m, "vdim", out["dim"])
    if kind == "attention":
        out["kv_heads"] = _int(mw, m, "kv_heads", out["heads"])
        if out["heads"] % out["kv_heads"]:
            raise ConfigError(f"{mw}: heads ({out['heads']}) is not a multiple of kv_heads ({out['kv_heads']})")
        out["scale"] = _num(mw, m, "scale", 1.0 / math.sqrt(out["dim"]))
        if m.get("conv") is not None:
            out["conv"] = _int(mw, m, "conv")
        rot = _obj(mw, m, "rot")
        if rot is not None:
            dims = _int(f"{mw}.rot", rot, "dims", least=0)
            if dims % 2 or dims > out["dim"]:
                raise ConfigError(f"{mw}.rot: 'dims' must be even and at most dim, got {dims}")
            out["rot"] = {"dims": dims, "base": _num(f"{mw}.rot", rot, "base")}
            if dims and not out["rot"]["base"] > 0:
                raise ConfigError(f"{mw}.rot: 'base' must be positive")
        mask = _obj(mw, m, "mask")
        if mask is not None:
            out["mask"] = {"size": _int(f"{mw}.mask", mask, "size")}
    else:
        out["gate_cap"] = _num(mw, m, "gate_cap")
        if not out["gate_cap"] > 0:
            raise ConfigError(f"{mw}: 'gate_cap' must be positive")
    mlp = layer.get("mlp")
    if mlp is not None:
        lw = f"{where}.mlp"
        if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
            raise ConfigError(f"{lw} must be null or an object of kind 'dense' or 'moe', got {mlp!r}")
        if mlp["kind"] == "dense":
            mlp = {"kind": "dense", "ff": _int(lw, mlp, "ff"), "limit": _num(lw, mlp, "limit")}
        else:
            expert, router = _obj(lw, mlp, "expert", True), _obj(lw, mlp, "router", True)
            checked = {"kind": "moe", "expert": {"ff": _int(f"{lw}.expert", expert, "ff")},
                       "router": {"experts": _int(f"{lw}.router", router, "experts"), "top": _int(f"{lw}.router", router, "top"),
                                  "scale": _num(f"{lw}.router", router, "scale", 1.0)}}
            if checked["router"]["top"] > checked["router"]["experts"]:
                raise ConfigError(f"{lw}.router: top ({checked['router']['top']}) is above experts ({checked['router']['experts']})")
            shared = _obj(lw, mlp, "shared")
            if shared is not None:
                checked["shared"] = {"ff": _int(f"{lw}.shared", shared, "ff")}
            mlp = checked
    return {"type": kind, "mixer": out, "mlp": mlp}


@dataclass(frozen=True)
class DekinexConfig(ModelConfig):
    architecture = "Dekinex"

    vocab: int
    width: int
    layers: Tuple[Dict[str, Any], ...]
    norm_eps: float
    residual_mult: float = 1.0
    bigram: Optional[Tuple[int, int, int]] = None   # (buckets, mul_prev, mul_cur)
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "DekinexConfig":
        where = "config.json of Dekinex"
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError(f"{where} lacks a non-empty list 'layers'")
        checked = tuple(_check_layer(i, layer) for i, layer in enumerate(layers))
        eps = _num("norm", _obj(where, raw, "norm", True), "eps")
        if not eps > 0:
            raise ConfigError("norm: 'eps' must be positive")
        loop = _obj(where, raw, "loop")
        if loop is not None:
            start, stop = _int("loop", loop, "start", least=0), _int("loop", loop, "stop", least=0)
            times = _int("loop", loop, "times", 1)
            if not start <= stop <= len(checked):
                raise ConfigError(f"loop: layers {start} to {stop} do not lie among the {len(checked)} layers")
            loop = (start, stop, times)
        bigram = _obj("embedding", _obj(where, raw, "embedding") or {}, "bigram")
        if bigram is not None:
            bigram = (_int("embedding.bigram", bigram, "buckets"), _int("embedding.bigram", bigram, "mul_prev", least=0),
                      _int("embedding.bigram", bigram, "mul_cur", least=0))
        return cls(vocab=_int(where, raw, "vocab"), width=_int(where, raw, "width"), layers=checked, norm_eps=eps,
                   residual_mult=_num(where, raw, "residual_mult", 1.0), bigram=bigram, loop=loop)

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width,
                               "residual_mult": self.residual_mult, "norm": {"eps": self.norm_eps},
                               "layers": [{"type": l["type"], "mixer": _plain(l["mixer"]), "mlp": _plain(l["mlp"])}
                                          for l in self.layers]}
        if self.bigram is not None:
            out["embedding"] = {"bigram": dict(zip(("buckets", "mul_prev", "mul_cur"), self.bigram))}
        if self.loop is not None:
            out["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        return out

    def layer_order(self) -> Tuple[Tuple[int, Optional[int]], ...]:
        """The layers in the order a step runs them, each with the number of the pass that begins with it (None where
        none does): the looped run so many times in a row, the rest once."""
        n = len(self.layers)
        if self.loop is None:
            return tuple((i, None) for i in range(n))
        start, stop, times = self.loop
        out = [(i, None) for i in range(start)]
        for t in range(times):
            out += [(i, t if i == start else None) for i in range(start, stop)]
        return tuple(out + [(i, None) for i in range(stop, n)])
