"""Attention whose projections pass a short causal convolution over time.

Per row, with h the mixer's input:
  u_q = Wq h + bq, u_k = Wk h + bk, u_v = Wv h + bv                       (biases optional)
  c_x[t] = sum_j conv_x[:, j] * u_x[t - (taps - 1) + j]                   (zeros ahead of the sequence; taps 0: c = u,
                                                                            no tensor; 1 tap is a scale per channel)
  q, k = c_q, c_k divided by their root mean square over a head           (`unit_norm`)
  s = (q . k) * scale over the keys that the mask lets the row see: all earlier ones ("causal"), the last n
      ("window") or those of the row's own chunk of n positions counted from position 0 ("chunk")
  p = exp(s) / (sink + sum exp(s)), sink = 1 or 0;  out = Wo (sum p v)
Keys have `key_dim` and values `value_dim` elements a head; query head j reads kv head j // (H / G).  The cache holds
k after convolution and norm and v after convolution.  With `shares_kv` the mixer has no k and v of its own: it reads
the pages of the plan entry it borrows from (`PlanEntry.cache_of`) with its own q.  The projected rows of the last
taps - 1 positions are per-request state (float32), kept by the mixer itself also when it borrows."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import MIXERS, FixedState, Mixer, PagedKeysValues, Runtime, as_normed, to_device
from .spec import ParamSpec


@MIXERS.register("conv_attention")
class ConvAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int,
                 scale: float, conv_taps: int = 0, unit_norm: bool = True, norm_eps: float = 1e-6, bias: bool = True,
                 mask: str = "causal", mask_size: int = 0, sink: bool = False, shares_kv: bool = False,
                 names: Optional[Mapping[str, str]] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if mask not in ops.MASKS or (mask != "causal" and int(mask_size) <= 0):
            raise ValueError(f"attention mask {mask!r} of size {mask_size}: known masks are {sorted(ops.MASKS)}, "
                             f"and a window or chunk needs a positive size")
        self.D, self.H, self.G = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dk, self.dv = int(key_dim), int(value_dim)
        self.scale, self.taps = float(scale), int(conv_taps)
        self.unit_norm, self.eps, self.bias = bool(unit_norm), float(norm_eps), bool(bias)
        self.mask, self.mask_size, self.sink = mask, int(mask_size), bool(sink)
        self.shares_kv = bool(shares_kv)
        # tensor names: projections q, k, v, o; "<projection><bias>" and "<projection><conv>" beside them
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "bias": ".b", "conv": ".conv", **dict(names or {})}
        self.projections = [("q", self.H * self.dk)]
        if not self.shares_kv:
            self.projections += [("k", self.G * self.dk), ("v", self.G * self.dv)]
        self.width = sum(n for _, n in self.projections)
        self.q_off, self.k_off, self.v_off = 0, self.H * self.dk, (self.H + self.G) * self.dk

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        out: Dict[str, ParamSpec] = {}
        for p, rows in self.projections:
            out[n[p]] = ParamSpec((rows, self.D))
            if self.bias:
                out[n[p] + n["bias"]] = ParamSpec((rows,), store="float32", init="zeros")
            if self.taps >= 1:
                out[n[p] + n["conv"]] = ParamSpec((rows, self.taps), store="float32", init="normal")
        out[n["o"]] = ParamSpec((self.D, self.H * self.dv))
        return out

    def cache_need(self):
        return None if self.shares_kv else PagedKeysValues(self.G, self.dk, self.dv)

    def state_need(self):
        return FixedState((self.taps - 1, self.width)) if self.taps > 1 else None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        mats = [tensors[n[p]] for p, _ in self.projections]
        dt = mats[0].dtype if all(m.dtype == mats[0].dtype for m in mats) else torch.float32
        # one [width, D] matrix: a single product gives q (, k and v) of a row
        self.w_in = ops.prepare_matrix(torch.cat([to_device(m, rt, dt) for m in mats], dim=0), rt.dtype)
        self.w_o = ops.prepare_matrix(to_device(tensors[n["o"]], rt), rt.dtype)
        self.b_in = self.conv_w = None
        if self.bias:
            self.b_in = torch.cat([to_device(tensors[n[p] + n["bias"]], rt, torch.float32)
                                   for p, _ in self.projections]).contiguous()
        if self.taps >= 1:
            self.conv_w = torch.cat([to_device(tensors[n[p] + n["conv"]], rt, torch.float32)
                                     for p, _ in self.projections], dim=0).contiguous()

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden]: the mixer's output.  `cache`: the pages' view, or {"mixer": pages,
        "mixer.state": the convolution's state}."""
        pages, state = (cache.get("mixer"), cache.get("mixer.state")) if isinstance(cache, dict) else (cache, None)
        h = as_normed(h).tensor()
        T, dev, dt = h.shape[0], h.device, self.rt.dtype
        proj = torch.empty((T, self.width), dtype=dt, device=dev)
        ops.linear(h, self.w_in, proj)
        q = torch.empty((T, self.H * self.dk), dtype=dt, device=dev)
        own = not self.shares_kv
        if own and not pages.writes:
            raise ValueError("an attention with keys and values of its own was given another entry's pages")
        ops.conv_heads(proj, self.q_off, self.k_off, self.v_off, self.H, self.G if own else 0, self.dk, self.dv,
                       self.b_in, self.conv_w, state.state if state is not None else None, step,
                       state.slots if state is not None else None, self.unit_norm, self.eps, q,
                       pages.block_table if own else None, pages.kv if own else None, pages.page_tokens)
        attn = torch.empty((T, self.H * self.dv), dtype=dt, device=dev)
        ops.masked_attention(q, attn, self.H, self.G, self.dk, self.dv, pages.kv, pages.page_tokens,
                             pages.block_table, step, self.mask, self.mask_size, self.sink, self.scale)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(attn, self.w_o, out)
        return out
