"""A selective state-space mixer (selective scan over time with a state per channel).

Per row, with h the mixer's input, `inner` channels and N states a channel:
  [x | z] = W_in h                                              (inner each)
  x <- silu(conv(x) + conv_bias)                                a short causal convolution over time on every channel,
                                                                zeros ahead of the sequence
  [dt' | B | C] = W_x x                                         (dt_rank, N, N)
  dt = softplus(W_dt dt' + dt_bias)                             one step size a channel
  A = -exp(A_log)                                               [inner, N]
  S[c][n] <- exp(dt_c A[c][n]) S[c][n] + dt_c x_c B_n;   y_c = sum_n S[c][n] C_n + D_c x_c
  out = W_o (y * silu(z))
S is float32 state of the request (a slot, zero when a request starts), and so are the convolution's last taps - 1
inputs.  Step sizes, their softplus, the decays exp(dt A), B, C and the state are 32-bit; x, z and y * silu(z) are held
in the run's element type."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import MIXERS, FixedState, Mixer, Runtime, as_normed, to_device
from .spec import ParamSpec


@MIXERS.register("selective_scan")
class SelectiveScan(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, inner: int, state: int, dt_rank: int, conv_taps: int,
                 names: Optional[Mapping[str, str]] = None):
        self.D, self.C, self.N, self.R, self.taps = int(hidden_size), int(inner), int(state), int(dt_rank), int(conv_taps)
        if min(self.D, self.C, self.N, self.R, self.taps) < 1:
            raise ValueError("selective scan: every size must be positive (a convolution has at least one tap)")
        self.names = {"in": "in", "conv": "conv", "conv_bias": "conv.b", "x": "x", "dt": "dt", "dt_bias": "dt.b",
                      "A_log": "A_log", "D": "D", "o": "o", **dict(names or {})}

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, C, N, R = self.names, self.C, self.N, self.R
        return {n["in"]: ParamSpec((2 * C, self.D)),
                n["conv"]: ParamSpec((C, self.taps), store="float32", init="normal"),
                n["conv_bias"]: ParamSpec((C,), store="float32", init="zeros"),
                n["x"]: ParamSpec((R + 2 * N, C)),
                n["dt"]: ParamSpec((C, R)),
                n["dt_bias"]: ParamSpec((C,), store="float32", init="normal"),
                n["A_log"]: ParamSpec((C, N), store="float32", init="normal"),
                n["D"]: ParamSpec((C,), store="float32", init=1.0),
                n["o"]: ParamSpec((self.D, C))}

    def cache_need(self):
        return FixedState((self.C, self.N), "float32")

    def state_need(self):
        return FixedState((self.taps - 1, self.C), "float32") if self.taps > 1 else None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n, R = self.names, self.R
        self.w_in = ops.prepare_matrix(to_device(tensors[n["in"]], rt), rt.dtype)
        wx = to_device(tensors[n["x"]], rt)
        # two products: the step sizes' low-rank part feeds another product (the run's element type), B and C enter the
        # recurrence as they are (32-bit sums)
        self.w_xdt = ops.prepare_matrix(wx[:R].contiguous(), rt.dtype)
        self.w_xbc = ops.prepare_matrix(wx[R:].contiguous(), rt.dtype)
        self.w_dt = ops.prepare_matrix(to_device(tensors[n["dt"]], rt), rt.dtype)
        self.w_o = ops.prepare_matrix(to_device(tensors[n["o"]], rt), rt.dtype)
        self.conv_w = to_device(tensors[n["conv"]], rt, torch.float32)
        self.conv_b = to_device(tensors[n["conv_bias"]], rt, torch.float32)
        self.dt_b = to_device(tensors[n["dt_bias"]], rt, torch.float32)
        self.A = (-torch.exp(tensors[n["A_log"]].to(torch.float32))).to(rt.device).contiguous()
        self.Dw = to_device(tensors[n["D"]], rt, torch.float32)

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden]: the mixer's output.  `cache`: the state's view, or {"mixer": the state,
        "mixer.state": the convolution's inputs}."""
        state, conv = (cache.get("mixer"), cache.get("mixer.state")) if isinstance(cache, dict) else (cache, None)
        if state is None or not state.writes:
            raise ValueError("a recurrent mixer needs a state of its own")
        h = as_normed(h).tensor()
        T, dev, dt, C, N = h.shape[0], h.device, self.rt.dtype, self.C, self.N
        xz = torch.empty((T, 2 * C), dtype=dt, device=dev)
        ops.linear(h, self.w_in, xz)
        x = torch.empty((T, C), dtype=dt, device=dev)
        ops.conv_channels(xz, C, self.conv_w, self.conv_b, conv.state if conv is not None else None, step,
                          conv.slots if conv is not None else None, "silu", x)
        low = torch.empty((T, self.R), dtype=dt, device=dev)
        ops.linear(x, self.w_xdt, low)
        bc = torch.empty((T, 2 * N), dtype=torch.float32, device=dev)
        ops.linear(x, self.w_xbc, bc)
        steps = torch.empty((T, C), dtype=torch.float32, device=dev)
        ops.linear(low, self.w_dt, steps)
        y = torch.empty((T, C), dtype=dt, device=dev)
        ops.selective_scan(x, steps, self.dt_b, self.A, bc, self.Dw, xz[:, C:], state.state, step, state.slots, y)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(y, self.w_o, out)
        return out
