"""A plain, slow reading of the Gulidra decoder in numpy (float64), one function per mechanism.  It shares no code
with the engine: tests compare the engine's parts and whole steps with it.

Notation: T tokens of one sequence, D the model's width, H query heads, G key/value heads, dk / dv the key and value
sizes of a head, n the taps of the short convolution, E routed experts, I identity experts, K experts a token uses."""
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


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def embed(table: np.ndarray, positions_table: np.ndarray, tokens, pos0: int, scale: float) -> np.ndarray:
    """Row of the table times `scale`, plus the learned vector of the token's position (not scaled)."""
    tokens = np.asarray(tokens)
    return table[tokens] * scale + positions_table[pos0:pos0 + len(tokens)]


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


def softmax_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float) -> np.ndarray:
    """One map of one head.  q [Tq, dk] are the last Tq of the Tk positions of k [Tk, dk], v [Tk, dv]; a position sees
    itself and everything before it.  Returns [Tq, dv]."""
    Tq, Tk = q.shape[0], k.shape[0]
    out = np.zeros((Tq, v.shape[1]))
    for a in range(Tq):
        last = Tk - Tq + a
        s = (k[:last + 1] @ q[a]) * scale
        e = np.exp(s - s.max())
        out[a] = (e / e.sum()) @ v[:last + 1]
    return out


def diff_lambda(lq1, lk1, lq2, lk2, diff: float) -> float:
    return math.exp(float(np.dot(lq1, lk1))) - math.exp(float(np.dot(lq2, lk2))) + diff


def differential_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, lam: float, diff: float,
                           eps: float) -> np.ndarray:
    """q [Tq, H, 2, dk], k [Tk, G, 2, dk], v [Tk, G, dv].  Two softmax maps a head over the same values; head h reads
    key/value head h // (H / G).  o = a1 - lam * a2, divided by its root mean square over dv, times (1 - diff).
    Returns [Tq, H, dv]."""
    Tq, H = q.shape[0], q.shape[1]
    G, dv = v.shape[1], v.shape[2]
    out = np.zeros((Tq, H, dv))
    for h in range(H):
        g = h // (H // G)
        a1 = softmax_attention(q[:, h, 0], k[:, g, 0], v[:, g], scale)
        a2 = softmax_attention(q[:, h, 1], k[:, g, 1], v[:, g], scale)
        out[:, h] = unit_rms(a1 - lam * a2, eps) * (1.0 - diff)
    return out


def decayed_linear_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, decay: np.ndarray,
                             state: Optional[np.ndarray] = None):
    """q, k [T, H, dk], v [T, H, dv], decay [H].  Per head S <- decay * S + k_t v_t^T (S is [dk, dv], zero at the start
    or `state`), o_t = S^T q_t.  Returns (o [T, H, dv], the state after the last token [H, dk, dv])."""
    T, H, dk = q.shape
    dv = v.shape[2]
    S = np.zeros((H, dk, dv)) if state is None else np.array(state, dtype=np.float64)
    out = np.zeros((T, H, dv))
    for t in range(T):
        for h in range(H):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            out[t, h] = S[h].T @ q[t, h]
    return out, S


def gated_unit(h: np.ndarray, w_gate, w_up, w_down) -> np.ndarray:
    """Wd (silu(Wg h) * (Wu h))"""
    return (silu(h @ w_gate.T) * (h @ w_up.T)) @ w_down.T


def route(h: np.ndarray, w_router: np.ndarray, correction: np.ndarray, top: int):
    """Scores s = softmax(Wr h) over all experts; the `top` largest of s + correction are chosen (the lower index wins
    a tie); the weights are the chosen experts' s.  Returns (ids [T, top], weights [T, top])."""
    z = h @ w_router.T
    e = np.exp(z - z.max(axis=-1, keepdims=True))
    s = e / e.sum(axis=-1, keepdims=True)
    ids = np.argsort(-(s + correction), axis=-1, kind="stable")[:, :top]
    return ids, np.take_along_axis(s, ids, axis=-1)


def routed_experts(h: np.ndarray, w_router, correction, experts: List[tuple], identity: int, top: int) -> np.ndarray:
    """`experts`: (gate, up, down) of every expert with tensors; the last `identity` outputs of the router stand for
    experts that return their input."""
    ids, w = route(h, w_router, correction, top)
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(ids[t], w[t]):
            y = h[t] if e >= len(experts) else gated_unit(h[t:t + 1], *experts[e])[0]
            out[t] += wt * y
    return out


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
    """What a sequence leaves behind for its next tokens: per layer the projected rows of the last n-1 positions, keys
    and values of every position, or the recurrent state."""

    def __init__(self, n_layers: int):
        self.pos = 0
        self.conv: List[Optional[np.ndarray]] = [None] * n_layers
        self.keys: List[Optional[np.ndarray]] = [None] * n_layers
        self.values: List[Optional[np.ndarray]] = [None] * n_layers
        self.state: List[Optional[np.ndarray]] = [None] * n_layers


class PlainGulidra:
    def __init__(self, cfg: dict, w: Dict[str, np.ndarray]):
        self.cfg, self.w = cfg, {k: np.asarray(v, dtype=np.float64) for k, v in w.items()}
        self.eps = float(cfg["norm"]["eps"])
        self.m = float(cfg["residual_mult"])

    def new_memory(self) -> Memory:
        return Memory(len(self.cfg["layers"]))

    def _conv(self, mem: Memory, i: int, u: np.ndarray, names: List[str], taps: int) -> List[np.ndarray]:
        """The projections of layer i in `names` through their convolutions, with the rows the memory holds in front."""
        w = self.w
        if taps <= 1:
            return [u_x * w[f"l{i}.mix.{x}.conv"][:, 0] if taps == 1 else u_x for x, u_x in zip(names, u)]
        width = [a.shape[1] for a in u]
        cat = np.concatenate(u, axis=1)
        wc = np.concatenate([w[f"l{i}.mix.{x}.conv"] for x in names], axis=0)
        y = short_conv(cat, wc, mem.conv[i])
        ext = cat if mem.conv[i] is None else np.concatenate([mem.conv[i], cat], axis=0)
        pad = np.zeros((max(0, taps - 1 - ext.shape[0]), cat.shape[1]))
        mem.conv[i] = np.concatenate([pad, ext], axis=0)[-(taps - 1):]
        return np.split(y, np.cumsum(width)[:-1], axis=1)

    def attention(self, i: int, h: np.ndarray, mem: Memory) -> np.ndarray:
        w, m = self.w, self.cfg["layers"][i]["mixer"]
        p = f"l{i}.mix."
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        T = h.shape[0]
        taps = int(m.get("conv") or 0)
        src = m.get("kv_from")
        names = ["q"] if src is not None else ["q", "k", "v"]
        c = self._conv(mem, i, [h @ w[p + x].T for x in names], names, taps)
        q = rms_norm(c[0].reshape(T, H, 2, dk), w[p + "q.norm"], self.eps)
        if src is None:
            k = rms_norm(c[1].reshape(T, G, 2, dk), w[p + "k.norm"], self.eps)
            v = c[2].reshape(T, G, dv)
            mem.keys[i] = k if mem.keys[i] is None else np.concatenate([mem.keys[i], k], axis=0)
            mem.values[i] = v if mem.values[i] is None else np.concatenate([mem.values[i], v], axis=0)
            src = i
        lam = diff_lambda(w[p + "lq1"], w[p + "lk1"], w[p + "lq2"], w[p + "lk2"], m["diff"])
        o = differential_attention(q, mem.keys[src], mem.values[src], m["scale"], lam, m["diff"], self.eps)
        o = o * sigmoid(h @ w[p + "g"].T)[:, :, None]
        return o.reshape(T, H * dv) @ w[p + "o"].T

    def lightning(self, i: int, h: np.ndarray, mem: Memory) -> np.ndarray:
        w, m = self.w, self.cfg["layers"][i]["mixer"]
        p = f"l{i}.mix."
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        T = h.shape[0]
        q = silu(h @ w[p + "q"].T).reshape(T, H, dk)
        k = silu(h @ w[p + "k"].T).reshape(T, H, dk)
        v = silu(h @ w[p + "v"].T).reshape(T, H, dv)
        o, mem.state[i] = decayed_linear_attention(q, k, v, np.asarray(m["decay"], dtype=np.float64), mem.state[i])
        o = rms_norm(o.reshape(T, H * dv), w[p + "norm"], self.eps) * sigmoid(h @ w[p + "g"].T)
        return o @ w[p + "o"].T

    def feed_forward(self, i: int, h: np.ndarray) -> np.ndarray:
        w, f = self.w, self.cfg["layers"][i]["mlp"]
        p = f"l{i}.mlp."
        if f["kind"] == "dense":
            return gated_unit(h, w[p + "gate"], w[p + "up"], w[p + "down"])
        r = f["router"]
        experts = [(w[f"{p}e{e}.gate"], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"]) for e in range(r["experts"])]
        return routed_experts(h, w[p + "router"], w[p + "correction"], experts, int(r.get("identity") or 0), r["top"])

    def forward(self, tokens, mem: Optional[Memory] = None, layers_out: Optional[list] = None) -> np.ndarray:
        """Logits [T, vocab] of the next T tokens of a sequence whose earlier tokens `mem` has seen."""
        w, cfg = self.w, self.cfg
        mem = mem or self.new_memory()
        x = embed(w["embed"], w["pos"], tokens, mem.pos, cfg["embedding"]["scale"])
        for i, layer in enumerate(cfg["layers"]):
            mix = self.attention if layer["type"] == "attention" else self.lightning
            x = x + self.m * rms_norm(mix(i, x, mem), w[f"l{i}.norm1"], self.eps)
            if layer.get("mlp") is not None:
                x = x + self.m * rms_norm(self.feed_forward(i, x), w[f"l{i}.norm2"], self.eps)
            if layers_out is not None:
                layers_out.append(x.copy())
        mem.pos += len(tokens)
        return rms_norm(x, w["final.norm"], self.eps) @ w["head"].T


def greedy(model: PlainGulidra, prompt, n: int) -> List[int]:
    """The n tokens that follow `prompt` when the largest logit is taken every time (the lowest id wins a tie)."""
    mem = model.new_memory()
    logits = model.forward(list(prompt), mem)[-1]
    out = []
    for _ in range(n):
        out.append(int(np.argmax(logits)))
        logits = model.forward([out[-1]], mem)[-1]
    return out
