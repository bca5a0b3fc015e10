"""RMS norm.  out = x / sqrt(mean(x^2) + eps) * w, the sum and the scale in
32-bit; eps inside the root, the weight applied plainly (no 1 + w)
(crates/allpaca-cpu/src/kernels.rs:492-507).  With `scalar` the weight is a single
number: out = x / sqrt(mean(x^2) + eps) * g."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import NORMS, Norm, Runtime, to_device
from .spec import ParamSpec


@NORMS.register("rmsnorm")
class RMSNorm(Norm):
    graph_safe = True

    def __init__(self, size: int, eps: float, name: str = "weight", scalar: bool = False):
        self.size, self.eps, self.name = int(size), float(eps), name     # `name`: the weight's tensor name
        self.scalar = bool(scalar)     # the weight is one number for all coordinates (a tensor without dimensions)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.name: ParamSpec(() if self.scalar else (self.size,), store="float32")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        w = tensors[self.name].to(torch.float32)
        if self.scalar:                # kept as a row of equal numbers: the kernels and the folded forms are the same
            w = w.reshape(1).expand(self.size)
        self.weight = to_device(w, rt, torch.float32)

    def forward(self, x: torch.Tensor, out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> None:
        ops.rmsnorm_rows(x, self.weight, self.eps, out, rows)

    def rms_params(self):
        return self.weight, self.eps

    def native_desc(self):
        return {"kind": "rmsnorm", "weight": self.weight, "eps": self.eps} if type(self) is RMSNorm else None
