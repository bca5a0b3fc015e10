"""Linear attention with a decay per head and a matrix of state per request.

Per row, with h the mixer's input and act = silu (or none):
  q = act(Wq h), k = act(Wk h)  (heads x key_dim),  v = act(Wv h)  (heads x value_dim)
  per head:  S <- decay_head * S + k v^T   (S [key_dim, value_dim], float32, zero when a request starts)
             o = S^T q                     (no other scale)
  the concatenated heads through an RMS norm with a weight over the whole row, times sigmoid(Wg h) (`gate`), then Wo.
The state is the mixer's cache: one slot a request, carried from step to step.  Everything behind the projections
(and their activation) is 32-bit.

Options: `rotary_dim` (the first elements of every q and k head are rotated by the position, pairs i, i + rotary_dim/2,
angle p * rope_theta^(-2i/rotary_dim)), `key_scale` (k is multiplied by it behind the rotation), `norm` "heads" (every
head's o is divided by its own root mean square, no weight, no tensor) instead of "row", `gate_act` "silu" (times
silu(Wg h)) instead of "sigmoid"."""
from __future__ import annotations

from typing import Dict, Mapping, Optional, Sequence

import torch

from ..kernels import ops
from .base import MIXERS, FixedState, Mixer, Runtime, as_normed, to_device
from .spec import ParamSpec


@MIXERS.register("decay_linear_attention")
class DecayLinearAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, key_dim: int, value_dim: int, decay: Sequence[float],
                 norm_eps: float = 1e-6, activation: str = "silu", gate: bool = True,
                 names: Optional[Mapping[str, str]] = None, rotary_dim: int = 0, rope_theta: float = 10000.0,
                 key_scale: float = 1.0, norm: str = "row", gate_act: str = "sigmoid"):
        self.D, self.H, self.dk, self.dv = int(hidden_size), int(num_heads), int(key_dim), int(value_dim)
        self.decay = tuple(float(v) for v in decay)
        if len(self.decay) != self.H:
            raise ValueError(f"linear attention: {len(self.decay)} decay rates for {self.H} heads")
        if activation not in ("silu", "none"):
            raise ValueError(f"linear attention: activation {activation!r} is not known (silu, none)")
        self.eps, self.silu, self.gate = float(norm_eps), activation == "silu", bool(gate)
        self.rot, self.theta, self.key_scale = int(rotary_dim), float(rope_theta), float(key_scale)
        if self.rot % 2 or not (0 <= self.rot <= self.dk):
            raise ValueError(f"linear attention: rotary_dim {rotary_dim} must be even and at most key_dim {key_dim}")
        if norm not in ("row", "heads") or gate_act not in ops.GATES:
            raise ValueError(f"linear attention: norm {norm!r} ('row', 'heads'), gate_act {gate_act!r} {sorted(ops.GATES)}")
        self.head_norm, self.gate_act = norm == "heads", gate_act
        self.names = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "norm": "norm", **dict(names or {})}
        self.q_off, self.k_off, self.v_off = 0, self.H * self.dk, 2 * self.H * self.dk
        self.g_off = self.v_off + self.H * self.dv
        self.width = self.g_off + (self.H * self.dv if self.gate else 0)

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, N = self.names, self.H * self.dv
        out = {n["q"]: ParamSpec((self.H * self.dk, self.D)), n["k"]: ParamSpec((self.H * self.dk, self.D)),
               n["v"]: ParamSpec((N, self.D)), n["o"]: ParamSpec((self.D, N))}
        if not self.head_norm:
            out[n["norm"]] = ParamSpec((N,), store="float32")
        if self.gate:
            out[n["gate"]] = ParamSpec((N, self.D))
        return out

    def cache_need(self):
        return FixedState((self.H, self.dk, self.dv), "float32")

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        mats = [tensors[n[x]] for x in (("q", "k", "v", "gate") if self.gate else ("q", "k", "v"))]
        dt = mats[0].dtype if all(m.dtype == mats[0].dtype for m in mats) else torch.float32
        # one [width, D] matrix: a single product gives q, k, v and the gate's logits of a row
        self.w_in = ops.prepare_matrix(torch.cat([to_device(m, rt, dt) for m in mats], dim=0), rt.dtype)
        self.w_o = ops.prepare_matrix(to_device(tensors[n["o"]], rt), rt.dtype)
        self.norm_w = None if self.head_norm else to_device(tensors[n["norm"]], rt, torch.float32)
        self.cos_sin = None
        if self.rot:
            from .rope import rotary_table
            self.cos_sin = rotary_table(self.rot, self.theta, rt)
        self.decay_t = torch.tensor(self.decay, dtype=torch.float32, device=rt.device)
        self.powers = None
        if rt.dtype == torch.bfloat16 and rt.device.type == "cuda":
            from ..kernels import tuned
            # (of the float32 decay, which is what the row-by-row kernel multiplies with)
            self.powers = tuned.decay_powers(self.decay_t.tolist(), rt.device)

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden]: the mixer's output.  `cache`: the state's view."""
        state = cache.get("mixer") if isinstance(cache, dict) else cache
        if not state.writes:
            raise ValueError("a recurrent mixer needs a state of its own")
        h = as_normed(h).tensor()
        T, dev, dt = h.shape[0], h.device, self.rt.dtype
        proj = torch.empty((T, self.width), dtype=dt, device=dev)
        ops.linear(h, self.w_in, proj)
        N = self.H * self.dv
        o = torch.empty((T, N), dtype=torch.float32, device=dev)
        ops.linear_attention(proj, self.q_off, self.k_off, self.v_off, self.H, self.dk, self.dv, self.silu,
                             self.decay_t, state.state, step, state.slots, o, powers=self.powers, rot=self.rot,
                             cos_sin=self.cos_sin, k_scale=self.key_scale)
        a = torch.empty((T, N), dtype=dt, device=dev)
        ops.gated_rmsnorm(o, self.norm_w, self.eps, proj[:, self.g_off:self.g_off + N] if self.gate else None, a,
                          group=self.dv if self.head_norm else 0, gate_act=self.gate_act)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(a, self.w_o, out)
        return out
