"""Small Gulidra configurations that differ in every size and option, model folders with random weights for them, and
the plain implementation's logits."""
from __future__ import annotations

import functools
import os
from typing import Dict, List, Sequence

import numpy as np
import torch

import plain_gulidra as P
from helpers import tmp_root


def _att(heads, kv_heads, dim, vdim, scale, diff, conv=None, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, diff=diff)
    if conv is not None:
        m["conv"] = conv
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="attention", mixer=m)


def _lin(heads, dim, vdim, decay):
    return dict(type="lightning", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay)))


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(ff, experts, identity, top):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, identity=identity, top=top))


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


# A: odd sizes everywhere (nothing a matrix-core kernel takes): grouped heads 4:2, keys 12 and values 20 wide, 3 taps,
#    a layer that borrows keys and values with 2 taps of its own, two recurrent layers of different shapes (one without
#    feed-forward), experts of which 3 of 5 + 2 are used, one of 4 + 0, an attention without convolution
TINY_GA = dict(
    architecture="Gulidra", vocab=83, width=36, max_positions=300, embedding=dict(scale=2.5), residual_mult=0.7,
    norm=dict(eps=1e-5),
    layers=[_layer(_att(4, 2, 12, 20, 0.35, 0.25, conv=3), _dense(52)),
            _layer(_att(4, 2, 12, 20, 0.2, 0.4, conv=2, kv_from=0), _moe(20, 5, 2, 3)),
            _layer(_lin(2, 20, 12, (0.7, 0.97)), None),
            _layer(_lin(3, 6, 28, (0.5, 0.9, 0.999)), _moe(28, 4, 0, 1)),
            _layer(_att(2, 2, 10, 6, 0.4, 0.1), _dense(44))])
# B: multiples of 16 and 32 everywhere (what the matrix-core kernels take): heads 4:2 and 8:2, 4 taps, borrowed keys,
#    recurrent layers with keys of 64 and of 128, experts 2 of 8 + 1
TINY_GB = dict(
    architecture="Gulidra", vocab=256, width=128, max_positions=600, embedding=dict(scale=1.5), residual_mult=0.5,
    norm=dict(eps=1e-6),
    layers=[_layer(_att(4, 2, 32, 64, 0.18, 0.3, conv=4), _moe(64, 8, 1, 2)),
            _layer(_lin(2, 64, 64, (0.8, 0.995)), _dense(192)),
            _layer(_att(8, 2, 32, 64, 0.2, 0.2, conv=4, kv_from=0), _moe(32, 6, 2, 3)),
            _layer(_lin(2, 128, 32, (0.9, 0.6)), _moe(96, 4, 0, 2)),
            _layer(_att(2, 1, 64, 32, 0.12, 0.45, conv=2), _dense(256))])
# C: the values that make terms vanish: scale and factor 1, one head, one tap, every expert chosen, experts that are
#    all identities beside one, a decay of 1
TINY_GC = dict(
    architecture="Gulidra", vocab=50, width=32, max_positions=128, embedding=dict(scale=1.0), residual_mult=1.0,
    norm=dict(eps=1e-6),
    layers=[_layer(_att(1, 1, 16, 16, 0.25, 0.5, conv=1), _moe(16, 1, 1, 2)),
            _layer(_lin(1, 16, 16, (1.0,)), _moe(24, 3, 0, 3)),
            _layer(_att(1, 1, 16, 16, 0.25, 0.0, conv=0, kv_from=0), None)])

# D: recurrent layers only (no pages at all), the first one without feed-forward
TINY_GD = dict(
    architecture="Gulidra", vocab=70, width=48, max_positions=200, embedding=dict(scale=0.5), residual_mult=1.5,
    norm=dict(eps=1e-5),
    layers=[_layer(_lin(3, 16, 24, (0.9, 0.95, 0.99)), None),
            _layer(_lin(2, 40, 8, (0.6, 0.999)), _moe(40, 2, 3, 2))])
# E: a borrower behind recurrent layers, two owners, experts without any identity key
TINY_GE = dict(
    architecture="Gulidra", vocab=64, width=64, max_positions=200, embedding=dict(scale=4.0), residual_mult=0.25,
    norm=dict(eps=1e-6),
    layers=[_layer(_att(4, 1, 16, 32, 0.25, 0.35, conv=5), _dense(96)),
            _layer(_lin(2, 32, 32, (0.97, 0.9)), dict(kind="moe", expert=dict(ff=48), router=dict(experts=3, top=1))),
            _layer(_att(2, 2, 24, 16, 0.2, 0.15, conv=3), None),
            _layer(_att(4, 1, 16, 32, 0.3, 0.3, conv=2, kv_from=0), _dense(80)),
            _layer(_att(2, 2, 24, 16, 0.2, 0.6, kv_from=2), _moe(64, 2, 1, 3))])

CONFIGS = {"GA": (TINY_GA, 21), "GB": (TINY_GB, 22), "GC": (TINY_GC, 23), "GD": (TINY_GD, 24), "GE": (TINY_GE, 25)}


def planted(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights of a size at which every mechanism shows in the logits: matrices N(0, 1/sqrt(fan-in)) (queries and keys
    larger, so that the softmax is not flat), taps of order 1, norm weights around 1, router corrections that change
    the choice, position vectors as large as the token rows."""
    from allpaca_amd.models import DecoderModel, describe_model
    _, _, spec = describe_model(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, ps in DecoderModel(spec).param_specs().items():
        shape = tuple(ps.shape)
        rnd = torch.randn(shape, generator=g)
        if name.endswith(".conv"):
            t = 0.5 * rnd + 0.3
        elif name.endswith(".correction"):
            t = 0.2 * rnd
        elif name.split(".")[-1] in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.3 * rnd
        elif len(shape) == 1:
            t = 1.0 + 0.2 * rnd
        elif name in ("embed", "pos"):
            t = rnd
        elif name.endswith(".router"):
            t = 2.0 * rnd / shape[1] ** 0.5
        elif name.endswith("mix.q") or name.endswith("mix.k"):
            t = 2.0 * rnd / shape[1] ** 0.5
        else:
            t = rnd / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16).float()     # values that bfloat16 holds, so both runs load the same numbers
    return out


@functools.lru_cache(maxsize=None)
def model_folder(name: str, dtype: str = "float32") -> str:
    from allpaca_amd.weights import write_model_folder
    cfg, seed = CONFIGS[name]
    path = os.path.join(tmp_root(), f"{name}_{dtype}")
    write_model_folder(path, cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16,
                       overrides=planted(cfg, seed))
    return path


@functools.lru_cache(maxsize=None)
def oracle(folder: str) -> P.PlainGulidra:
    return P.PlainGulidra(*P.read_model_folder(folder))


_LOGITS: Dict = {}


def oracle_logits(folder: str, tokens: Sequence[int]) -> np.ndarray:
    key = (folder, tuple(tokens))
    if key not in _LOGITS:
        _LOGITS[key] = oracle(folder).forward(list(tokens))
    return _LOGITS[key]


def tokens_for(name: str, n: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, CONFIGS[name][0]["vocab"], size=n).tolist()
