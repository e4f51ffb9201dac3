"""Small Risizen configurations that differ in every size and option, model folders with random weights for them, and
the plain implementation's logits."""
from __future__ import annotations

import functools
import os
from typing import Dict, List, Sequence

import numpy as np
import torch

import plain_risizen as R
from helpers import tmp_root


def _att(heads, kv_heads, dim, vdim, scale, conv=None, chunk=None, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if conv is not None:
        m["conv"] = conv
    if chunk is not None:
        m["mask"] = dict(size=chunk)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _layer(mixer, ff=None, limit=None):
    return dict(type="attention", mixer=mixer, mlp=None if ff is None else dict(kind="dense", ff=ff, limit=limit))


# A: three streams, grouped heads 4:2, keys 24 and values 16 wide, 3 taps, chunks of 7, a layer that borrows keys and
#    has no feed-forward, a layer without mask and with 2 taps and as many kv heads as heads, and one that borrows those
TINY_RA = dict(
    architecture="Risizen", vocab=97, width=48, streams=3, norm=dict(eps=1e-5), logit_scale=0.75,
    layers=[_layer(_att(4, 2, 24, 16, 0.3, conv=3, chunk=7), ff=80, limit=1.0),
            _layer(_att(4, 2, 24, 16, 0.25, conv=3, chunk=7, kv_from=0)),
            _layer(_att(4, 4, 16, 16, 0.4, conv=2), ff=64, limit=2.0),
            _layer(_att(4, 4, 16, 16, 0.4, conv=4, chunk=20, kv_from=2), ff=72, limit=0.5)])
# B: one stream (with weights), one head, keys wider than the model's rows, no convolution, chunks of 5, no logit scale,
#    widths that are no multiple of 8
TINY_RB = dict(
    architecture="Risizen", vocab=61, width=36, streams=1, norm=dict(eps=1e-6),
    layers=[_layer(_att(1, 1, 40, 12, 0.2, chunk=5), ff=50, limit=1.5),
            _layer(_att(3, 1, 20, 28, 0.35, conv=5, chunk=64), ff=44, limit=3.0)])
# C: two streams, multiples of 16 and 32 everywhere (what the matrix-core kernels take), chunks of 48 that are no
#    multiple of the attention tile, a borrowed layer
TINY_RC = dict(
    architecture="Risizen", vocab=256, width=128, streams=2, norm=dict(eps=1e-6), logit_scale=0.5,
    layers=[_layer(_att(4, 2, 64, 32, 0.15, conv=4, chunk=48), ff=256, limit=1.5),
            _layer(_att(8, 2, 32, 64, 0.2, conv=4, chunk=80), ff=192, limit=1.5),
            _layer(_att(8, 2, 32, 64, 0.2, conv=4, chunk=80, kv_from=1), ff=192, limit=1.5)])
# D: no `streams` key at all (the plain residual sum, no connection tensors), no mask, a convolution of a single tap
TINY_RD = dict(
    architecture="Risizen", vocab=50, width=32, norm=dict(eps=1e-6), logit_scale=2.0,
    layers=[_layer(_att(2, 2, 16, 16, 0.3, conv=1), ff=48, limit=1.0), _layer(_att(2, 1, 16, 8, 0.3, conv=2, kv_from=None))])

CONFIGS = {"RA": (TINY_RA, 11), "RB": (TINY_RB, 12), "RC": (TINY_RC, 13), "RD": (TINY_RD, 14)}


def planted(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights of a size at which every mechanism shows in the logits: matrices N(0, 1/sqrt(fan-in)), biases and
    convolution taps of order 1, norm weights around 1, stream weights well away from 0 and 1."""
    from allpaca_amd.models import DecoderModel, describe_model
    _, _, spec = describe_model(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, ps in DecoderModel(spec).param_specs().items():
        if ps.optional:
            continue
        shape = tuple(ps.shape)
        rnd = torch.randn(shape, generator=g)
        if name.endswith(".conv"):
            t = 0.5 * rnd + 0.3
        elif name.endswith(".b"):
            t = 0.3 * rnd
        elif ".hc" in name and name.endswith(".mix"):
            t = torch.eye(shape[0]) + 0.3 * rnd
        elif ".hc" in name and name.endswith(".in"):
            t = 0.6 + 0.3 * torch.rand(shape, generator=g)
        elif ".hc" in name and name.endswith(".out"):
            t = 0.7 + 0.6 * torch.rand(shape, generator=g)
        elif len(shape) == 1:
            t = 1.0 + 0.2 * rnd
        elif name == "embed":
            t = rnd
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
def oracle(folder: str):
    return R.read_model_folder(folder)


_LOGITS: Dict = {}


def oracle_logits(folder: str, tokens: Sequence[int]) -> np.ndarray:
    key = (folder, tuple(tokens))
    if key not in _LOGITS:
        cfg, w = oracle(folder)
        _LOGITS[key] = R.forward(cfg, w, list(tokens))
    return _LOGITS[key]


def tokens_for(name: str, n: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, CONFIGS[name][0]["vocab"], size=n).tolist()
