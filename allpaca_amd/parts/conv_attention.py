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
taps - 1 positions are per-request state (float32), kept by the mixer itself also when it borrows.

`key_parts` = M > 1: a head has M softmax maps over the same values.  `key_dim` then counts all M queries (keys) of a
head side by side, the unit norm is taken over each of the M pieces, and `attend` returns the M maps' outputs of every
head side by side in float32 for a subclass to combine (`DifferentialAttention`).  `norm_weights`: the normed pieces of
q and k are multiplied with the tensors "<q>.norm" and "<k>.norm" [key_dim / M], shared by all heads and maps.

`norm_scope` "projection": the root mean square is taken over all heads of q (of k) at once, before they are split into
heads, and the weights "<q>.norm", "<k>.norm" have the projection's size.  `q_temp` = (coef, every): q of the row at
position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).  `distance_bias`: tensors "r1", "r2" [heads];
the score of a key d positions back is lowered by r1[h] * ln(1 + r2[h] * d).  `out_bias`: the output projection has a
bias "<o><bias>"."""
from __future__ import annotations

from typing import Dict, Mapping, Optional, Sequence

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
                 names: Optional[Mapping[str, str]] = None, key_parts: int = 1, norm_weights: bool = False,
                 extra_rows: int = 0, norm_scope: str = "head", q_temp: Optional[Sequence[float]] = None,
                 distance_bias: bool = False, out_bias: bool = False):
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
        self.key_parts, self.norm_weights = int(key_parts), bool(norm_weights)
        if self.key_parts < 1 or self.dk % self.key_parts or (self.norm_weights and not self.unit_norm):
            raise ValueError(f"attention: key_parts {key_parts} must divide key_dim {key_dim}, and norm weights need the norm")
        if norm_scope not in ("head", "projection") or (norm_scope == "projection" and
                                                        (not self.unit_norm or self.key_parts != 1)):
            raise ValueError(f"attention: norm_scope {norm_scope!r} ('head', or 'projection' with the norm and one map a head)")
        self.norm_rows = norm_scope == "projection"
        self.q_temp = None
        if q_temp is not None:
            coef, every = q_temp
            if int(every) != every or int(every) <= 0:
                raise ValueError(f"attention: the query temperature's step {every!r} must be a positive whole number")
            self.q_temp = (float(coef), int(every))
        self.distance_bias, self.out_bias = bool(distance_bias), bool(out_bias)
        self.extra_rows = int(extra_rows)      # rows a subclass adds to the input matrix behind q, k and v
        # tensor names: projections q, k, v, o; "<projection><bias>" and "<projection><conv>" beside them
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "bias": ".b", "conv": ".conv", "norm": ".norm",
                      "r1": "r1", "r2": "r2", **dict(names or {})}
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
        if self.norm_weights:
            for p, rows in self.projections[:2]:
                out[n[p] + n["norm"]] = ParamSpec((rows if self.norm_rows else self.dk // self.key_parts,), store="float32")
        if self.distance_bias:
            out[n["r1"]] = ParamSpec((self.H,), store="float32", init=0.5)
            out[n["r2"]] = ParamSpec((self.H,), store="float32", init=0.5)
        out[n["o"]] = ParamSpec((self.D, self.H * self.dv))
        if self.out_bias:
            out[n["o"] + n["bias"]] = ParamSpec((self.D,), store="float32", init="zeros")
        return out

    def extra_matrices(self, tensors, rt) -> list:
        """Matrices [rows, hidden] of a subclass that go into the one input product behind q, k and v."""
        return []

    def cache_need(self):
        return None if self.shares_kv else PagedKeysValues(self.G, self.dk, self.dv)

    def state_need(self):
        return FixedState((self.taps - 1, self.width)) if self.taps > 1 else None

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        mats = [tensors[n[p]] for p, _ in self.projections] + list(self.extra_matrices(tensors, rt))
        dt = mats[0].dtype if all(m.dtype == mats[0].dtype for m in mats) else torch.float32
        self.q_norm_w = self.k_norm_w = None
        if self.norm_weights:
            self.q_norm_w = to_device(tensors[n["q"] + n["norm"]], rt, torch.float32)
            if not self.shares_kv:
                self.k_norm_w = to_device(tensors[n["k"] + n["norm"]], rt, torch.float32)
        # one [width, D] matrix: a single product gives q (, k and v) of a row
        mats = [to_device(m, rt, dt) for m in mats]
        # (rows of zeros behind a subclass's extra rows, so that a row of the product is a multiple of 16 bytes)
        self.full_width = self.width + (-(-self.extra_rows // 8) * 8 if self.extra_rows else 0)
        if self.full_width > self.width + self.extra_rows:
            mats.append(torch.zeros((self.full_width - self.width - self.extra_rows, self.D), dtype=dt, device=rt.device))
        self.w_in = ops.prepare_matrix(torch.cat(mats, dim=0), rt.dtype)
        self.w_o = ops.prepare_matrix(to_device(tensors[n["o"]], rt), rt.dtype)
        self.b_in = self.conv_w = self.b_o = self.r12 = None
        if self.out_bias:
            self.b_o = to_device(tensors[n["o"] + n["bias"]], rt, torch.float32)
        if self.distance_bias:
            self.r12 = (to_device(tensors[n["r1"]], rt, torch.float32), to_device(tensors[n["r2"]], rt, torch.float32))
        if self.bias:
            self.b_in = torch.cat([to_device(tensors[n[p] + n["bias"]], rt, torch.float32)
                                   for p, _ in self.projections]).contiguous()
        if self.taps >= 1:
            self.conv_w = torch.cat([to_device(tensors[n[p] + n["conv"]], rt, torch.float32)
                                     for p, _ in self.projections], dim=0).contiguous()

    def attend(self, h, step, cache, out_dtype=None):
        """(the input product's rows [rows, width + extra_rows], the attention's output [rows, heads * key_parts *
        value_dim] in `out_dtype`, the run's type if None).  `cache`: the pages' view, or {"mixer": pages,
        "mixer.state": the convolution's state}."""
        pages, state = (cache.get("mixer"), cache.get("mixer.state")) if isinstance(cache, dict) else (cache, None)
        h = as_normed(h).tensor()
        T, dev, dt = h.shape[0], h.device, self.rt.dtype
        full = torch.empty((T, self.full_width), dtype=dt, device=dev)
        ops.linear(h, self.w_in, full)
        proj = full[:, :self.width] if self.extra_rows else full
        q = torch.empty((T, self.H * self.dk), dtype=dt, device=dev)
        own = not self.shares_kv
        if own and not pages.writes:
            raise ValueError("an attention with keys and values of its own was given another entry's pages")
        ops.conv_heads(proj, self.q_off, self.k_off, self.v_off, self.H, self.G if own else 0, self.dk, self.dv,
                       self.b_in, self.conv_w, state.state if state is not None else None, step,
                       state.slots if state is not None else None, self.unit_norm, self.eps, q,
                       pages.block_table if own else None, pages.kv if own else None, pages.page_tokens,
                       norm_dim=self.dk // self.key_parts, q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w,
                       norm_rows=self.norm_rows, q_temp_coef=self.q_temp[0] if self.q_temp else 0.0,
                       q_temp_every=self.q_temp[1] if self.q_temp else 0)
        M = self.key_parts
        attn = torch.empty((T, self.H * M * self.dv), dtype=out_dtype or dt, device=dev)
        ops.masked_attention(q, attn, self.H * M, self.G, self.dk, self.dv, pages.kv, pages.page_tokens,
                             pages.block_table, step, self.mask, self.mask_size, self.sink, self.scale, key_parts=M,
                             distance_bias=self.r12)
        return full, attn

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden]: the mixer's output."""
        if self.key_parts != 1:
            raise ValueError("an attention with several maps a head needs a rule that combines them")
        _, attn = self.attend(h, step, cache)
        T, dev = attn.shape[0], attn.device
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(attn, self.w_o, out)
        if self.b_o is not None:
            ops.bias_rows(out, self.b_o)
        return out


@MIXERS.register("differential_attention")
class DifferentialAttention(ConvAttention):
    """Two softmax maps a head over the same values, a1 and a2:
      lam = exp(lq1 . lk1) - exp(lq2 . lk2) + diff            (one number for the layer)
      o = a1 - lam * a2;  o <- o / sqrt(mean(o^2) + eps) over the head's values, times (1 - diff)
      o <- o * sigmoid(Wg h)[head]  (`head_gate`: one number a head, from the mixer's input);  out = Wo o
    q holds [map 1, map 2] of `key_dim` each per head, k likewise per kv head; convolution, norm (with weights), mask
    and pages are the base class's."""
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 diff: float, conv_taps: int = 0, norm_eps: float = 1e-6, head_gate: bool = True,
                 shares_kv: bool = False, mask: str = "causal", mask_size: int = 0,
                 names: Optional[Mapping[str, str]] = None):
        names = {"lq1": "lq1", "lk1": "lk1", "lq2": "lq2", "lk2": "lk2", "gate": "g", **dict(names or {})}
        super().__init__(hidden_size, num_heads, num_kv_heads, 2 * int(key_dim), value_dim, scale, conv_taps=conv_taps,
                         unit_norm=True, norm_eps=norm_eps, bias=False, mask=mask, mask_size=mask_size, sink=False,
                         shares_kv=shares_kv, names=names, key_parts=2, norm_weights=True,
                         extra_rows=int(num_heads) if head_gate else 0)
        self.diff, self.head_gate, self.map_dim = float(diff), bool(head_gate), int(key_dim)

    def param_specs(self) -> Dict[str, ParamSpec]:
        out = super().param_specs()
        n = self.names
        for x in ("lq1", "lk1", "lq2", "lk2"):
            out[n[x]] = ParamSpec((self.map_dim,), store="float32", init="normal")
        if self.head_gate:
            out[n["gate"]] = ParamSpec((self.H, self.D))
        return out

    def extra_matrices(self, tensors, rt) -> list:
        return [tensors[self.names["gate"]]] if self.head_gate else []

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        super().bind(tensors, rt)
        n = self.names
        lq1, lk1, lq2, lk2 = (tensors[n[x]].to(torch.float32) for x in ("lq1", "lk1", "lq2", "lk2"))
        self.lam = float(torch.exp(torch.dot(lq1, lk1)) - torch.exp(torch.dot(lq2, lk2))) + self.diff

    def forward(self, h, step, cache) -> torch.Tensor:
        full, maps = self.attend(h, step, cache, out_dtype=torch.float32)
        T, dev = maps.shape[0], maps.device
        attn = torch.empty((T, self.H * self.dv), dtype=self.rt.dtype, device=dev)
        gate = full[:, self.width:self.width + self.H] if self.head_gate else None
        ops.diff_combine(maps, self.lam, 1.0 - self.diff, self.eps, gate, attn, self.H, self.dv)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(attn, self.w_o, out)
        return out
