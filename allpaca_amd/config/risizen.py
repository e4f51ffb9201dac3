"""Typed configuration of the Risizen decoder, read from config.json.

Keys: `vocab`, `width`, `streams` (residual streams, 1 if absent), `norm.eps`, `logit_scale` (1 if absent) and
`layers`, a list of {"type", "mixer", "mlp"}.  A mixer of type "attention" names `heads`, `kv_heads`, `dim` (key and
query size of a head), `vdim` (value size), `scale`, `conv` (taps of the short convolution; absent or below 2: none),
`mask` ({"size": n}: chunks of n positions; absent: every earlier position) and `kv_from` (the layer whose keys and
values it reads instead of its own).  `mlp` is null or {"kind": "dense", "ff", "limit"}.  Every size comes from here;
nothing has a silent default that fixes a tensor's shape."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Mapping, Optional, Tuple

from .llama import ConfigError

DEFAULT_MAX_POSITIONS = 1 << 20     # the design has no position tables: a request may be as long as the cache allows


def _int(d: Mapping[str, Any], key: str, where: str, least: int = 1) -> int:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, int) or v < least:
        raise ConfigError(f"config.json: {where}{key!r} must be an integer >= {least}, got {v!r}")
    return v


def _num(d: Mapping[str, Any], key: str, where: str) -> float:
    v = d.get(key)
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: {where}{key!r} must be a number, got {v!r}")
    return float(v)


@dataclass(frozen=True)
class RisizenAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0                       # taps; 0: no convolution
    chunk: Optional[int] = None         # mask.size
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class RisizenMlp:
    ff: int
    limit: float


@dataclass(frozen=True)
class RisizenLayer:
    mixer: RisizenAttention
    mlp: Optional[RisizenMlp]


@dataclass(frozen=True)
class RisizenConfig:
    vocab: int
    width: int
    streams: int
    eps: float
    logit_scale: float
    layers: Tuple[RisizenLayer, ...]
    has_stream_weights: bool = True     # False: `streams` is absent, the residual is the plain sum

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "RisizenConfig":
        vocab, width = _int(d, "vocab", ""), _int(d, "width", "")
        norm = d.get("norm")
        if not isinstance(norm, Mapping):
            raise ConfigError("config.json: 'norm' must be an object with 'eps'")
        eps = _num(norm, "eps", "norm.")
        raw = d.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[RisizenLayer] = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping) or entry.get("type") != "attention":
                kind = entry.get("type") if isinstance(entry, Mapping) else entry
                raise ConfigError(f"config.json: {where}type {kind!r} is not a mixer of this design (known: 'attention')")
            m = entry.get("mixer")
            if not isinstance(m, Mapping):
                raise ConfigError(f"config.json: {where}mixer must be an object")
            mw = where + "mixer."
            mask = m.get("mask")
            if mask is not None and not isinstance(mask, Mapping):
                raise ConfigError(f"config.json: {mw}mask must be an object with 'size' or null")
            conv = m.get("conv")
            att = RisizenAttention(
                heads=_int(m, "heads", mw), kv_heads=_int(m, "kv_heads", mw), dim=_int(m, "dim", mw),
                vdim=_int(m, "vdim", mw), scale=_num(m, "scale", mw),
                conv=0 if conv is None else _int(m, "conv", mw, least=0),
                chunk=None if mask is None else _int(mask, "size", mw + "mask."),
                kv_from=None if m.get("kv_from") is None else _int(m, "kv_from", mw, least=0))
            if att.heads % att.kv_heads:
                raise ConfigError(f"config.json: {mw}heads {att.heads} is no multiple of kv_heads {att.kv_heads}")
            if att.kv_from is not None:
                if att.kv_from >= i:
                    raise ConfigError(f"config.json: {mw}kv_from {att.kv_from} must name an earlier layer")
                src = layers[att.kv_from].mixer
                if src.kv_from is not None:
                    raise ConfigError(f"config.json: {mw}kv_from names layer {att.kv_from}, which has no keys of its own")
                if (src.kv_heads, src.dim, src.vdim) != (att.kv_heads, att.dim, att.vdim):
                    raise ConfigError(f"config.json: {mw}kv_heads, dim and vdim must equal those of layer {att.kv_from}")
            mlp = entry.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "dense":
                    kind = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                    raise ConfigError(f"config.json: {where}mlp.kind {kind!r} is not known (known: 'dense')")
                mlp = RisizenMlp(_int(mlp, "ff", where + "mlp."), _num(mlp, "limit", where + "mlp."))
            layers.append(RisizenLayer(att, mlp))
        return cls(vocab=vocab, width=width, streams=_int(d, "streams", "") if "streams" in d else 1, eps=eps,
                   logit_scale=_num(d, "logit_scale", "") if "logit_scale" in d else 1.0, layers=tuple(layers),
                   has_stream_weights="streams" in d)
