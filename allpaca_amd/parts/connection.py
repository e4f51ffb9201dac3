"""Residual connections over several streams (hyper-connections).

A row carries S copies x_1 .. x_S of the residual.  A sublayer reads u = sum_a in[a] x_a, and its output y goes back
as x_b <- sum_a mix[a][b] x_a + out[b] y, every copy from the old ones.  S = 1 with in = mix = out = 1 is the plain
residual sum.  All of it in 32-bit."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import CONNECTIONS, Norm, Part, Runtime, to_device
from .spec import ParamSpec


@CONNECTIONS.register("hyper")
class HyperConnection(Part):
    graph_safe = True

    def __init__(self, streams: int, optional_weights: bool = False):
        self.S = int(streams)
        if self.S < 1:
            raise ValueError("a residual connection needs at least one stream")
        self.optional_weights = bool(optional_weights)

    def param_specs(self) -> Dict[str, ParamSpec]:
        S, opt = self.S, self.optional_weights
        return {"in": ParamSpec((S,), store="float32", optional=opt, init=1.0 / S),
                "out": ParamSpec((S,), store="float32", optional=opt, init=1.0),
                "mix": ParamSpec((S, S), store="float32", optional=opt, init="identity_plus_normal")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        S = self.S
        given = [n for n in ("in", "out", "mix") if n in tensors]
        if given and len(given) != 3:
            raise ValueError(f"a residual connection needs all of in, out and mix or none; got {given}")
        ones = torch.ones(S, dtype=torch.float32)
        self.w_in = to_device(tensors.get("in", ones), rt, torch.float32)
        self.w_out = to_device(tensors.get("out", ones), rt, torch.float32)
        self.w_mix = to_device(tensors.get("mix", torch.eye(S, dtype=torch.float32)), rt, torch.float32)

    def read(self, x: torch.Tensor, norm: Norm, h: torch.Tensor) -> None:
        """h = norm(sum_a in[a] x_a)"""
        w, eps = norm.rms_params()
        ops.streams_step(x, self.S, in_w=self.w_in, norm_w=w, eps=eps, h=h)

    def write(self, x: torch.Tensor, y: torch.Tensor, then: Optional["HyperConnection"] = None,
              norm: Optional[Norm] = None, h: Optional[torch.Tensor] = None) -> None:
        """The sublayer's output y into the streams; with `then`, also the next sublayer's read of the new streams
        (one pass over the row)."""
        if then is None:
            ops.streams_step(x, self.S, y=y, mix=self.w_mix, out_w=self.w_out)
            return
        w, eps = norm.rms_params()
        ops.streams_step(x, self.S, y=y, mix=self.w_mix, out_w=self.w_out, in_w=then.w_in, norm_w=w, eps=eps, h=h)


@CONNECTIONS.register("scaled")
class ScaledSum(Part):
    """x <- x + mult * y: a constant of the layer, no tensors."""
    graph_safe = True

    def __init__(self, mult: float = 1.0):
        self.mult = float(mult)
