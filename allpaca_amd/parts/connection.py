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
    """x <- x + mult * y: a constant of the layer, no tensors.  `add` does it in 32-bit; with a norm it also leaves
    h = norm(new x) for the sublayer that reads x next (one pass over the row)."""
    graph_safe = True

    def __init__(self, mult: float = 1.0):
        self.mult = float(mult)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        self._one = torch.ones(1, dtype=torch.float32, device=rt.device)
        self._mult = torch.full((1,), self.mult, dtype=torch.float32, device=rt.device)

    def add(self, x: torch.Tensor, y: torch.Tensor, norm: Optional[Norm] = None, h: Optional[torch.Tensor] = None) -> None:
        if norm is None:
            ops.streams_step(x, 1, y=y, mix=self._one, out_w=self._mult)
            return
        w, eps = norm.rms_params()
        ops.streams_step(x, 1, y=y, mix=self._one, out_w=self._mult, in_w=self._one, norm_w=w, eps=eps, h=h)


@CONNECTIONS.register("reinject")
class InputInjection(Part):
    """A link between plan entries: x <- W [x; x0], x0 the embedding's output of the row and W [width, 2 width] (x's
    columns first).  The two halves of W are two products into the same float32 rows."""
    graph_safe = True

    def __init__(self, hidden_size: int, name: str = "weight"):
        self.D, self.name = int(hidden_size), name

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.name: ParamSpec((self.D, 2 * self.D))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        w = to_device(tensors[self.name], rt)
        self.w_x = ops.prepare_matrix(w[:, :self.D].contiguous(), rt.dtype)
        self.w_x0 = ops.prepare_matrix(w[:, self.D:].contiguous(), rt.dtype)

    def apply(self, x: torch.Tensor, x0: torch.Tensor) -> None:
        """x float32 [rows, width] is replaced; x0 [rows, width] in the run's element type."""
        h = torch.empty(x.shape, dtype=self.rt.dtype, device=x.device)
        ops.cast(x, h)
        ops.linear(h, self.w_x, x)
        ops.linear(x0, self.w_x0, x, accumulate=True)
