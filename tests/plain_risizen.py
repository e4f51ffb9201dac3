"""A plain, slow reading of the Risizen decoder in numpy (float64), one function per mechanism.  It shares no code
with the engine: tests compare the engine's parts and whole steps with it.

Notation: T tokens of one sequence, D the model's width, S residual streams, H query heads, G key/value heads,
dk / dv the key and value sizes of a head, C the chunk of the attention mask, n the taps of the short convolution."""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional

import numpy as np


# ---------------------------------------------------------------------------------------------- single mechanisms
def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return unit_rms(x, eps) * w


def short_conv(u: np.ndarray, w: np.ndarray, before: Optional[np.ndarray] = None) -> np.ndarray:
    """Causal convolution over time on every channel.  u [T, C], w [C, n]: y[t] = sum_j w[:, j] * u[t - (n-1) + j],
    with zeros (or the rows of `before`, the n-1 inputs that came ahead of u) in front of the sequence."""
    T, C = u.shape
    n = w.shape[1]
    pad = np.zeros((n - 1, C)) if before is None else np.asarray(before, dtype=np.float64)
    ext = np.concatenate([pad, u], axis=0)
    y = np.zeros((T, C))
    for t in range(T):
        for j in range(n):
            y[t] += w[:, j] * ext[t + j]
    return y


def visible(i: int, j: int, chunk: Optional[int], window: Optional[int] = None) -> bool:
    """Whether position i sees position j: causal, inside the same chunk (counted from position 0), and among the
    last `window` positions (the design itself has chunks only; the engine's kernel also takes a window)."""
    if j > i:
        return False
    if window is not None and i - j >= window:
        return False
    return chunk is None or (i // chunk) == (j // chunk)


def sink_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, chunk: Optional[int],
                   pos0: int = 0, sink: bool = True, window: Optional[int] = None) -> np.ndarray:
    """q [Tq, H, dk] at positions pos0 + (len(k) - Tq) ..., k [Tk, G, dk], v [Tk, G, dv] at positions pos0 ...
    Query head h reads key/value head h // (H / G).  p_j = exp(s_j) / (1 + sum_j exp(s_j)): the 1 is a sink with
    score 0 and no value.  Returns [Tq, H * dv]."""
    Tq, H, _ = q.shape
    Tk, G, dv = v.shape
    out = np.zeros((Tq, H, dv))
    first_q = pos0 + Tk - Tq
    for a in range(Tq):
        i = first_q + a
        js = [j for j in range(Tk) if visible(i, pos0 + j, chunk, window)]
        for h in range(H):
            g = h // (H // G)
            s = (k[js, g] @ q[a, h]) * scale
            m = max(0.0, s.max()) if len(js) else 0.0
            e = np.exp(s - m)
            den = e.sum() + (math.exp(-m) if sink else 0.0)
            out[a, h] = (e / den) @ v[js, g]
    return out.reshape(Tq, H * dv)


def clamped_glu(h: np.ndarray, w_gate: np.ndarray, w_up: np.ndarray, w_down: np.ndarray, limit: float,
                alpha: float = 1.702) -> np.ndarray:
    """g = min(Wg h, limit), u = clamp(Wu h, -limit, limit), y = g * sigmoid(alpha g) * (u + 1), out = Wd y."""
    g = np.minimum(h @ w_gate.T, limit)
    u = np.clip(h @ w_up.T, -limit, limit)
    y = g / (1.0 + np.exp(-alpha * g)) * (u + 1.0)
    return y @ w_down.T


def hyper_read(xs: np.ndarray, w_in: np.ndarray) -> np.ndarray:
    """xs [S, T, D] -> sum_s w_in[s] xs[s]."""
    return np.tensordot(w_in, xs, axes=(0, 0))


def hyper_write(xs: np.ndarray, y: np.ndarray, w_mix: np.ndarray, w_out: np.ndarray) -> np.ndarray:
    """new[t] = sum_s w_mix[s, t] xs[s] + w_out[t] y, all streams from the old ones."""
    return np.tensordot(w_mix.T, xs, axes=(1, 0)) + w_out[:, None, None] * y[None]


# ---------------------------------------------------------------------------------------------- a model folder
def read_model_folder(path: str):
    """(config dict, name -> float64 array) of a folder with config.json and model.safetensors."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(path, "model.safetensors"), "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        head = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, e in head.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        raw = data[lo:hi]
        if e["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype="<u2").astype(np.uint32) << 16).view(np.float32)
        elif e["dtype"] == "F32":
            a = np.frombuffer(raw, dtype="<f4")
        elif e["dtype"] == "I32":
            a = np.frombuffer(raw, dtype="<i4")
        else:
            raise ValueError(f"{name}: element type {e['dtype']}")
        out[name] = a.astype(np.float64).reshape(e["shape"])
    return cfg, out


# ---------------------------------------------------------------------------------------------- the whole model
class Memory:
    """What a sequence leaves behind for its next tokens: per layer the conv inputs of the last n-1 positions and the
    keys and values of every position."""

    def __init__(self):
        self.length = 0
        self.conv: Dict[str, np.ndarray] = {}
        self.k: Dict[int, np.ndarray] = {}
        self.v: Dict[int, np.ndarray] = {}


def _conv_step(mem: Memory, key: str, u: np.ndarray, w: Optional[np.ndarray]) -> np.ndarray:
    if w is None:
        return u
    n = w.shape[1]
    before = mem.conv.get(key)
    y = short_conv(u, w, before)
    ext = np.concatenate([np.zeros((n - 1, u.shape[1])) if before is None else before, u], axis=0)
    mem.conv[key] = ext[ext.shape[0] - (n - 1):]
    return y


def attention_mixer(cfg: dict, W: Dict[str, np.ndarray], li: int, h: np.ndarray, mem: Memory, eps: float) -> np.ndarray:
    m = cfg["layers"][li]["mixer"]
    p = f"l{li}.mix."
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]

    def proj(name: str, tag: str) -> np.ndarray:
        u = h @ W[p + name].T + W[p + name + ".b"]
        return _conv_step(mem, f"{li}.{tag}", u, W.get(p + name + ".conv"))

    q = unit_rms(proj("q", "q").reshape(T, H, dk), eps)
    src = m.get("kv_from")
    if src is None:
        k = unit_rms(proj("k", "k").reshape(T, G, dk), eps)
        v = proj("v", "v").reshape(T, G, dv)
        mem.k[li] = k if li not in mem.k else np.concatenate([mem.k[li], k], axis=0)
        mem.v[li] = v if li not in mem.v else np.concatenate([mem.v[li], v], axis=0)
        src = li
    chunk = (m.get("mask") or {}).get("size")
    a = sink_attention(q, mem.k[src], mem.v[src], m["scale"], chunk)
    return a @ W[p + "o"].T


def forward(cfg: dict, W: Dict[str, np.ndarray], tokens: List[int], mem: Optional[Memory] = None,
            layers_out: Optional[list] = None) -> np.ndarray:
    """Logits [len(tokens), vocab] of the next `tokens` of a sequence whose earlier tokens are in `mem`."""
    mem = mem if mem is not None else Memory()
    eps = cfg["norm"]["eps"]
    S = int(cfg.get("streams", 1))
    x0 = rms_norm(W["embed"][np.asarray(tokens)], W["embed.norm"], eps)
    xs = np.stack([x0] * S)
    for li, layer in enumerate(cfg["layers"]):
        p = f"l{li}."
        subs = [(1, lambda h: attention_mixer(cfg, W, li, h, mem, eps))]
        if layer.get("mlp") is not None:
            subs.append((2, lambda h: clamped_glu(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"],
                                                  layer["mlp"]["limit"])))
        for qn, fn in subs:
            if p + f"hc{qn}.in" in W:
                u = hyper_read(xs, W[p + f"hc{qn}.in"])
                y = fn(rms_norm(u, W[p + f"norm{qn}"], eps))
                xs = hyper_write(xs, y, W[p + f"hc{qn}.mix"], W[p + f"hc{qn}.out"])
            else:
                xs = xs + fn(rms_norm(xs[0], W[p + f"norm{qn}"], eps))[None]
        if layers_out is not None:
            layers_out.append(xs.sum(axis=0))
    mem.length += len(tokens)
    x = rms_norm(xs.sum(axis=0), W["final.norm"], eps)
    return (x @ W["head"].T) * cfg.get("logit_scale", 1.0)


def greedy(cfg: dict, W: Dict[str, np.ndarray], prompt: List[int], n_new: int) -> List[int]:
    mem = Memory()
    logits = forward(cfg, W, list(prompt), mem)
    out = []
    for _ in range(n_new):
        out.append(int(np.argmax(logits[-1])))
        logits = forward(cfg, W, [out[-1]], mem)
    return out
