"""SwiGLU feed-forward: a = silu(h Wg^T) * (h Wu^T), residual += a Wd^T, no bias,
silu(z) = z / (1 + exp(-z)) (crates/allpaca-core/src/model.rs:5664-5705,
crates/allpaca-cpu/src/kernels.rs:869-871)."""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, Runtime, as_normed, to_device
from .spec import ParamSpec


@FEED_FORWARDS.register("swiglu")
class SwiGLU(FeedForward):
    graph_safe = True

    takes_normed_input = True
    emits_next_norm = True

    def __init__(self, hidden_size: int, intermediate_size: int, names: Mapping[str, str] | None = None):
        self.D, self.F = int(hidden_size), int(intermediate_size)
        # tensor names of the three matrices
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight",
                      **dict(names or {})}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {
            n["gate"]: ParamSpec((self.F, self.D)),
            n["up"]: ParamSpec((self.F, self.D)),
            n["down"]: ParamSpec((self.D, self.F)),
        }

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        dt = g.dtype if g.dtype == u.dtype else torch.float32
        # one pass over h gives both branches: the pair of tiled matrices for the MFMA kernels, else
        # [2F, D] (gate rows, then up rows)
        wg, wu = ops.prepare_matrix(to_device(g, rt, dt), rt.dtype), ops.prepare_matrix(to_device(u, rt, dt), rt.dtype)
        if isinstance(wg, torch.Tensor):
            self.w_gate_up = torch.cat([wg, wu], dim=0).contiguous()
        else:
            self.w_gate_up = (wg, wu)
        self.w_down = ops.prepare_matrix(to_device(tensors[self.names["down"]], rt), rt.dtype)

    def forward_add(self, h, step, residual: torch.Tensor, emit=None) -> None:
        h = as_normed(h)
        act = torch.empty((h.shape[0], self.F), dtype=self.rt.dtype, device=h.device)
        h.swiglu(self.w_gate_up, act)
        ops.linear(act, self.w_down, residual, accumulate=True, emit=emit)

    def native_desc(self):
        if type(self) is not SwiGLU:
            return None
        return {"kind": "swiglu", "w_gate_up": self.w_gate_up, "w_down": self.w_down, "F": self.F}

    def forward(self, h, step):
        h = as_normed(h)
        act = torch.empty((h.shape[0], self.F), dtype=self.rt.dtype, device=h.device)
        h.swiglu(self.w_gate_up, act)
        out = torch.empty((h.shape[0], self.D), dtype=torch.float32, device=h.device)
        ops.linear(act, self.w_down, out)
        return out


@FEED_FORWARDS.register("clamped_glu")
class ClampedGLU(FeedForward):
    """g = min(h Wg^T, limit), u = clamp(h Wu^T, -limit, limit), a = g * sigmoid(alpha g) * (u + 1), out = a Wd^T,
    no bias."""
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, limit: float, alpha: float = 1.702,
                 names: Mapping[str, str] | None = None):
        self.D, self.F = int(hidden_size), int(intermediate_size)
        self.limit, self.alpha = float(limit), float(alpha)
        self.names = {"gate": "gate", "up": "up", "down": "down", **dict(names or {})}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["gate"]: ParamSpec((self.F, self.D)), n["up"]: ParamSpec((self.F, self.D)),
                n["down"]: ParamSpec((self.D, self.F))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        g, u = tensors[n["gate"]], tensors[n["up"]]
        dt = g.dtype if g.dtype == u.dtype else torch.float32
        # one [2F, D] matrix (gate rows, then up rows): a single product gives both branches of a row
        self.w_gate_up = ops.prepare_matrix(torch.cat([to_device(g, rt, dt), to_device(u, rt, dt)], dim=0), rt.dtype)
        self.w_down = ops.prepare_matrix(to_device(tensors[n["down"]], rt), rt.dtype)

    def forward(self, h, step) -> torch.Tensor:
        h = as_normed(h).tensor()
        act = torch.empty((h.shape[0], self.F), dtype=self.rt.dtype, device=h.device)
        ops.clamped_glu(h, self.w_gate_up, act, self.alpha, self.limit)
        out = torch.empty((h.shape[0], self.D), dtype=torch.float32, device=h.device)
        ops.linear(act, self.w_down, out)
        return out


@FEED_FORWARDS.register("mlp")
class ActMLP(FeedForward):
    """Two matrices and an activation between them, no gate and no bias: out = Wd act(Wu h).  `activation`: "relu2"
    (the square of max(z, 0)), "gelu_tanh" (0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))), "silu"."""
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "relu2",
                 names: Mapping[str, str] | None = None):
        self.D, self.F = int(hidden_size), int(intermediate_size)
        if activation not in ops.ACTIVATIONS or activation == "none":
            raise ValueError(f"mlp: activation {activation!r} is not one of {sorted(set(ops.ACTIVATIONS) - {'none'})}")
        self.activation = activation
        self.names = {"up": "up", "down": "down", **dict(names or {})}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        return {n["up"]: ParamSpec((self.F, self.D)), n["down"]: ParamSpec((self.D, self.F))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.w_up = ops.prepare_matrix(to_device(tensors[n["up"]], rt), rt.dtype)
        self.w_down = ops.prepare_matrix(to_device(tensors[n["down"]], rt), rt.dtype)

    def forward(self, h, step) -> torch.Tensor:
        h = as_normed(h).tensor()
        T, dev = h.shape[0], h.device
        act = torch.empty((T, self.F), dtype=self.rt.dtype, device=dev)
        ops.linear_act(h, self.w_up, act, self.activation)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(act, self.w_down, out)
        return out
