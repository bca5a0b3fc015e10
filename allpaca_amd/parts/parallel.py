"""Mixers side by side: every member reads the same input, and the result is the weighted sum of their outputs,
  out = sum_m scale_m * member_m(h).
The members are mixers of any kind (an attention beside a recurrent mixer, say), built from their own descriptions; a
member's tensors stand under "<member's name>." and what it keeps per request under "<role>.<member's name>" (pages or
state that a later layer may read) and "<role>.<member's name>.state" (what it keeps for itself alone)."""
from __future__ import annotations

from typing import Dict, Mapping, Sequence

import torch

from ..kernels import ops
from .base import MIXERS, Mixer, Runtime, build_part
from .spec import ParamSpec, PartSpec


@MIXERS.register("parallel")
class ParallelMixers(Mixer):
    def __init__(self, members: Sequence[Mapping]):
        """`members`: dicts {"name", "kind", "params", "scale"} in the order in which the outputs are added."""
        if len(members) < 2:
            raise ValueError("mixers side by side: at least two members")
        self.names = [str(m["name"]) for m in members]
        if len(set(self.names)) != len(self.names):
            raise ValueError(f"mixers side by side: member names must differ, got {self.names}")
        self.scales = [float(m.get("scale", 1.0)) for m in members]
        self.members = [build_part(MIXERS, PartSpec(m["kind"], dict(m.get("params", {})))) for m in members]

    @property
    def graph_safe(self) -> bool:
        return all(getattr(m, "graph_safe", False) for m in self.members)

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {f"{name}.{n}": ps for name, m in zip(self.names, self.members) for n, ps in m.param_specs().items()}

    def cache_need(self):
        needs = {name: m.cache_need() for name, m in zip(self.names, self.members)}
        return needs if any(n is not None for n in needs.values()) else None

    def state_need(self):
        needs = {name: m.state_need() for name, m in zip(self.names, self.members)}
        return needs if any(n is not None for n in needs.values()) else None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        for name, m in zip(self.names, self.members):
            pre = name + "."
            m.bind({n[len(pre):]: t for n, t in tensors.items() if n.startswith(pre)}, rt)

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden].  `cache`: {"mixer.<member>": view, "mixer.<member>.state": view}."""
        views = cache if isinstance(cache, dict) else {}
        out = None
        for i, (name, m) in enumerate(zip(self.names, self.members)):
            own = {"mixer": views.get(f"mixer.{name}"), "mixer.state": views.get(f"mixer.{name}.state")}
            y = m.forward(h, step, {k: v for k, v in own.items() if v is not None})
            if i == 0:
                out, first = y, self.scales[0]
            else:
                # out <- first * out + scale * y in 32-bit (the first member's factor is applied with the second's sum)
                ops.weighted_pair(out, first, y, self.scales[i], out)
                first = 1.0
        return out
