"""Typed configuration of the Gulidra decoder, read from config.json.

Keys: `vocab`, `width`, `max_positions` (rows of the learned position table), `embedding.scale`, `residual_mult`,
`norm.eps` and `layers`, a list of {"type", "mixer", "mlp"}.
  type "attention": `heads`, `kv_heads`, `dim` (size of one map's query and key), `vdim`, `scale`, `diff` (the constant
      of the differential combination), `conv` (taps of the short convolution; absent or 0: none), `kv_from` (the layer
      whose keys and values it reads instead of its own).
  type "lightning": `heads`, `dim`, `vdim`, `decay` (one number a head).
  `mlp`: null, {"kind": "dense", "ff"}, or {"kind": "moe", "expert": {"ff"}, "router": {"experts", "identity", "top"}}.
Every size comes from here; nothing has a silent default that fixes a tensor's shape."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Mapping, Optional, Tuple, Union

from .llama import ConfigError
from .risizen import _int, _num


@dataclass(frozen=True)
class GulidraAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    conv: int = 0                       # taps; 0: no convolution
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class GulidraLightning:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]


@dataclass(frozen=True)
class GulidraDense:
    ff: int


@dataclass(frozen=True)
class GulidraRouted:
    ff: int
    experts: int                        # experts with matrices
    identity: int                       # experts that return their input (the router's last outputs)
    top: int


@dataclass(frozen=True)
class GulidraLayer:
    mixer: Union[GulidraAttention, GulidraLightning]
    mlp: Union[None, GulidraDense, GulidraRouted]


def _obj(d: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    v = d.get(key)
    if not isinstance(v, Mapping):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return v


@dataclass(frozen=True)
class GulidraConfig:
    vocab: int
    width: int
    max_positions: int
    embedding_scale: float
    residual_mult: float
    eps: float
    layers: Tuple[GulidraLayer, ...]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "GulidraConfig":
        vocab, width = _int(d, "vocab", ""), _int(d, "width", "")
        eps = _num(_obj(d, "norm", ""), "eps", "norm.")
        raw = d.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[GulidraLayer] = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            kind = entry.get("type") if isinstance(entry, Mapping) else entry
            if kind not in ("attention", "lightning"):
                raise ConfigError(f"config.json: {where}type {kind!r} is not a mixer of this design "
                                  f"(known: 'attention', 'lightning')")
            m, mw = _obj(entry, "mixer", where), where + "mixer."
            if kind == "attention":
                conv = m.get("conv")
                mixer = GulidraAttention(
                    heads=_int(m, "heads", mw), kv_heads=_int(m, "kv_heads", mw), dim=_int(m, "dim", mw),
                    vdim=_int(m, "vdim", mw), scale=_num(m, "scale", mw), diff=_num(m, "diff", mw),
                    conv=0 if conv is None else _int(m, "conv", mw, least=0),
                    kv_from=None if m.get("kv_from") is None else _int(m, "kv_from", mw, least=0))
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"config.json: {mw}heads {mixer.heads} is no multiple of kv_heads {mixer.kv_heads}")
                if mixer.kv_from is not None:
                    if mixer.kv_from >= i:
                        raise ConfigError(f"config.json: {mw}kv_from {mixer.kv_from} must name an earlier layer")
                    src = layers[mixer.kv_from].mixer
                    if not isinstance(src, GulidraAttention) or src.kv_from is not None:
                        raise ConfigError(f"config.json: {mw}kv_from names layer {mixer.kv_from}, which has no keys "
                                          f"and values of its own")
                    if (src.kv_heads, src.dim, src.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim):
                        raise ConfigError(f"config.json: {mw}kv_heads, dim and vdim must equal those of layer "
                                          f"{mixer.kv_from}")
            else:
                decay = m.get("decay")
                heads = _int(m, "heads", mw)
                if (not isinstance(decay, list) or len(decay) != heads
                        or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in decay)):
                    raise ConfigError(f"config.json: {mw}decay must be a list of {heads} numbers, one a head")
                mixer = GulidraLightning(heads=heads, dim=_int(m, "dim", mw), vdim=_int(m, "vdim", mw),
                                         decay=tuple(float(v) for v in decay))
            mlp = entry.get("mlp")
            if mlp is not None:
                fw = where + "mlp."
                kind = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                if kind == "dense":
                    mlp = GulidraDense(_int(mlp, "ff", fw))
                elif kind == "moe":
                    r = _obj(mlp, "router", fw)
                    mlp = GulidraRouted(
                        ff=_int(_obj(mlp, "expert", fw), "ff", fw + "expert."),
                        experts=_int(r, "experts", fw + "router.", least=0),
                        identity=0 if r.get("identity") is None else _int(r, "identity", fw + "router.", least=0),
                        top=_int(r, "top", fw + "router."))
                    if mlp.experts + mlp.identity < mlp.top:
                        raise ConfigError(f"config.json: {fw}router.top {mlp.top} exceeds the {mlp.experts} + "
                                          f"{mlp.identity} experts")
                else:
                    raise ConfigError(f"config.json: {fw}kind {kind!r} is not known (known: 'dense', 'moe')")
            layers.append(GulidraLayer(mixer, mlp))
        return cls(vocab=vocab, width=width, max_positions=_int(d, "max_positions", ""),
                   embedding_scale=_num(_obj(d, "embedding", ""), "scale", "embedding."),
                   residual_mult=_num(d, "residual_mult", ""), eps=eps, layers=tuple(layers))
