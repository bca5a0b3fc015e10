"""A feed-forward of routed experts.

  z = Wr h (32-bit);  s = softmax(z) over all experts;  the `top` experts with the largest s + correction are chosen
  (`correction`: a tensor of one number an expert; it enters the choice only);  the weights are the chosen experts' s
  (divided by their sum with `renormalize`);  out = sum of weight * expert(h).
An expert is a gated unit Wd a(Wg h, Wu h) with tensors "<prefix><i>.gate|up|down"; the last `identity`
outputs of the router stand for experts without tensors that return h itself.  `activation` "silu": a(g, u) =
silu(g) * u; "clamped": g' * sigmoid(alpha g') * (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit).
With `renormalize` and no correction the weights are the softmax over the chosen logits alone.
`score` "sigmoid": s = sigmoid(z), every expert for itself.  `weight_on` "input": the weight multiplies the expert's
input instead of its output, out = sum of expert(weight * h).
The choice is made on the GPU and stays there: nothing is read back, so steps replay in graphs."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import FEED_FORWARDS, FeedForward, Runtime, as_normed, to_device
from .spec import ParamSpec


@FEED_FORWARDS.register("routed_experts")
class RoutedExperts(FeedForward):
    graph_safe = True

    def __init__(self, hidden_size: int, intermediate_size: int, experts: int, top: int, identity: int = 0,
                 correction: bool = True, renormalize: bool = False, names: Optional[Mapping[str, str]] = None,
                 activation: str = "silu", alpha: float = 1.0, limit: float = 0.0, score: str = "softmax",
                 weight_on: str = "output"):
        self.D, self.F, self.E, self.K, self.I = (int(hidden_size), int(intermediate_size), int(experts), int(top),
                                                  int(identity))
        if self.E < 0 or self.I < 0 or not (1 <= self.K <= self.E + self.I):
            raise ValueError(f"routed experts: top {top} of {experts} + {identity} experts")
        self.correction, self.renormalize = bool(correction), bool(renormalize)
        if activation not in ops.EXPERT_ACTIVATIONS or (activation == "clamped" and not float(limit) > 0):
            raise ValueError(f"routed experts: activation {activation!r} (known: {sorted(ops.EXPERT_ACTIVATIONS)}; "
                             f"the clamped unit needs a positive limit)")
        self.activation, self.alpha, self.limit = activation, float(alpha), float(limit)
        if score not in ops.ROUTER_SCORES or weight_on not in ("output", "input"):
            raise ValueError(f"routed experts: score {score!r} (known: {sorted(ops.ROUTER_SCORES)}), weight_on "
                             f"{weight_on!r} ('output', 'input')")
        self.score, self.weight_input = score, weight_on == "input"
        self.names = {"router": "router", "correction": "correction", "expert": "e", "gate": "gate", "up": "up",
                      "down": "down", **dict(names or {})}

    def _expert(self, e: int, x: str) -> str:
        return f"{self.names['expert']}{e}.{self.names[x]}"

    def param_specs(self) -> Dict[str, ParamSpec]:
        n, N = self.names, self.E + self.I
        out = {n["router"]: ParamSpec((N, self.D))}
        if self.correction:
            out[n["correction"]] = ParamSpec((N,), store="float32", init="zeros")
        for e in range(self.E):
            out[self._expert(e, "gate")] = ParamSpec((self.F, self.D))
            out[self._expert(e, "up")] = ParamSpec((self.F, self.D))
            out[self._expert(e, "down")] = ParamSpec((self.D, self.F))
        return out

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.w_router = ops.prepare_matrix(to_device(tensors[n["router"]], rt), rt.dtype)
        self.correction_t = to_device(tensors[n["correction"]], rt, torch.float32) if self.correction else None
        self.w_gate_up = self.w_down = None
        if self.E:
            mats = [tensors[self._expert(e, x)] for e in range(self.E) for x in ("gate", "up", "down")]
            dt = mats[0].dtype if all(m.dtype == mats[0].dtype for m in mats) else torch.float32
            # [experts, 2 ff, width] (an expert's gate rows, then its up rows) and [experts, width, ff]
            gate_up = torch.stack([torch.cat([to_device(tensors[self._expert(e, "gate")], rt, dt),
                                              to_device(tensors[self._expert(e, "up")], rt, dt)], dim=0)
                                   for e in range(self.E)]).contiguous()
            down = torch.stack([to_device(tensors[self._expert(e, "down")], rt, dt) for e in range(self.E)]).contiguous()
            self.w_gate_up, self.w_down = ops.prepare_experts(gate_up, down, rt.dtype)

    def forward(self, h, step) -> torch.Tensor:
        h = as_normed(h).tensor()
        T, dev = h.shape[0], h.device
        N = self.E + self.I
        z = torch.empty((T, N), dtype=torch.float32, device=dev)
        ops.linear(h, self.w_router, z)
        ids = torch.empty((T, self.K), dtype=torch.int32, device=dev)
        weights = torch.empty((T, self.K), dtype=torch.float32, device=dev)
        ops.route_topk(z, self.correction_t, self.K, ids, weights, self.renormalize, score=self.score)
        y = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.routed_experts(h, self.w_gate_up, self.w_down, self.E, self.F, ids, weights, self.K, y,
                           activation=self.activation, alpha=self.alpha, limit=self.limit,
                           weight_input=self.weight_input)
        return y
