"""Token embedding (a row copy, no scale: crates/allpaca-core/src/model.rs:8301-8311)
and the output head (logits = h W^T in float32 for the rows that ask,
crates/allpaca-core/src/model.rs:8781-8791)."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import EMBEDDINGS, HEADS, Part, Runtime, to_device
from .spec import ParamSpec


@EMBEDDINGS.register("token_table")
class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, name: str = "weight", scale: float = 1.0):
        self.V, self.D, self.name = int(vocab_size), int(hidden_size), name      # `name`: the table's tensor name
        self.scale = float(scale)                                                # x = table[token] * scale, in 32-bit

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.name: ParamSpec((self.V, self.D))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        self.weight = ops.prepare_matrix(to_device(tensors[self.name], rt), rt.dtype)

    def forward(self, tokens: torch.Tensor, out: torch.Tensor) -> None:
        ops.embed_rows(self.weight, tokens, out)
        if self.scale != 1.0:
            ops.scale_(out, self.scale)

    def native_desc(self):
        if type(self) is not TokenEmbedding or self.scale != 1.0:
            return None
        return {"kind": "token_table", "weight": self.weight}


@EMBEDDINGS.register("token_table_norm")
class NormedTokenEmbedding(Part):
    """A token's row of the table through an RMS norm with a weight of its own (`norm_name`), written into every
    residual stream of the row."""
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, eps: float, streams: int = 1, table_name: str = "weight",
                 norm_name: str = "norm"):
        self.V, self.D, self.eps, self.S = int(vocab_size), int(hidden_size), float(eps), int(streams)
        self.table_name, self.norm_name = table_name, norm_name

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.table_name: ParamSpec((self.V, self.D)), self.norm_name: ParamSpec((self.D,), store="float32")}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        self.weight = to_device(tensors[self.table_name], rt)      # row-major: rows are read whole
        self.norm_weight = to_device(tensors[self.norm_name], rt, torch.float32)

    def forward(self, tokens: torch.Tensor, out: torch.Tensor) -> None:
        ops.embed_streams(self.weight, tokens, self.norm_weight, self.eps, out, self.S)


@EMBEDDINGS.register("token_table_positions")
class PositionedTokenEmbedding(Part):
    """A token's row of the table times `scale`, plus a learned vector of the token's position (not scaled):
    x = table[token] * scale + positions[p].  The position table has `max_positions` rows; a step that reaches
    beyond them is refused."""
    graph_safe = True
    reads_positions = True       # `forward_step(step, out)` instead of `forward(tokens, out)`

    def __init__(self, vocab_size: int, hidden_size: int, max_positions: int, scale: float = 1.0,
                 table_name: str = "weight", positions_name: str = "positions"):
        self.V, self.D, self.P, self.scale = int(vocab_size), int(hidden_size), int(max_positions), float(scale)
        self.table_name, self.positions_name = table_name, positions_name

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.table_name: ParamSpec((self.V, self.D)), self.positions_name: ParamSpec((self.P, self.D))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        self.weight = to_device(tensors[self.table_name], rt)      # row-major: rows are read whole
        self.positions = to_device(tensors[self.positions_name], rt)

    def forward_step(self, step, out: torch.Tensor) -> None:
        if step.max_context > self.P:
            raise ValueError(f"a request reaches position {step.max_context - 1}, the model has position vectors for "
                             f"{self.P} positions")
        ops.embed_positions(self.weight, step.tokens, self.positions, step.positions, self.scale, out)


@HEADS.register("linear")
class LinearHead(Part):
    """`tied`: the head uses the embedding matrix and owns no tensor."""
    graph_safe = True

    def __init__(self, vocab_size: int, hidden_size: int, tied: bool = False, scale: float = 1.0,
                 name: str = "weight"):
        self.V, self.D, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.scale, self.name = float(scale), name     # logits = (h W^T) * scale

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {} if self.tied else {self.name: ParamSpec((self.V, self.D))}

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime, shared: Optional[torch.Tensor] = None) -> None:
        self.rt = rt
        self.weight = shared if self.tied else ops.prepare_matrix(to_device(tensors[self.name], rt), rt.dtype)
        if self.weight is None:
            raise ValueError("a tied head needs the embedding matrix")

    def forward(self, h: torch.Tensor, out: torch.Tensor) -> None:
        ops.linear(h, self.weight, out)
        if self.scale != 1.0:
            ops.scale_(out, self.scale)

    def native_desc(self):
        if type(self) is not LinearHead or self.scale != 1.0:
            return None
        return {"kind": "linear", "weight": self.weight}
