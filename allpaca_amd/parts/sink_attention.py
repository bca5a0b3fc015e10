"""Softmax attention with a learned sink per head, in two forms.

`sink_attention`: grouped heads (query head j reads kv head j // (H / G)).  Per row, with h the mixer's input:
  q = Wq h, k = Wk h, v = Wv h, or v = k as projected when the mixer has no value matrix (`values_are_keys`)
  the first `rotary_dim` elements of every q and k head are rotated by the row's position (pairs i, i + rotary_dim/2);
  v is never rotated
  s = (q . k) * scale over the keys the mask lets the row see ("causal": all earlier ones, "window": the last n)
  p = exp(s) / (exp(sink[head]) + sum exp(s)): the sink is a learned score a head, with no key and no value
  out = Wo (sum p v)
Options: `qk_norm` (every q and k head is divided by its root mean square over the head and multiplied with the
tensors "<q>.norm" / "<k>.norm" [key_dim], shared by all heads, before the rotation; values that are the keys stay as
projected), `softcap` c (s <- c * tanh(s / c)), `rope_scaling` (a frequency rule of `parts/rope.py`).

`latent_attention`: queries, keys and values go through low-rank latents.
  a = [Wdq; Wdkv; Wg] h                                   (one product; 32-bit rows)
  cq = rms_norm(a[:Q]) * dq.norm;  q = Wuq cq             heads of [dim unrotated, rot_dim rotated]
  c = rms_norm(a[Q:Q+R]) * dkv.norm                       the latent of keys and values
  kr = rotate(a[Q+R:Q+R+rot_dim])                         one rotated key part, shared by all heads
  key of head j = [(Wuk c)_j, kr], value of head j = (Wuv c)_j
  attention as above (every head has a key and a value of its own), then head j times sigmoid((Wg h)_j), then Wo.
The pages hold every head's key and value, put together when the row is written: attention over them is the kernel of
any other attention with keys and values of different sizes."""
from __future__ import annotations

from typing import Dict, Mapping, Optional

import torch

from ..kernels import ops
from .base import MIXERS, Mixer, PagedKeysValues, Runtime, as_normed, to_device
from .rope import rotary_table
from .spec import ParamSpec


def _check_mask(mask: str, mask_size: int) -> None:
    if mask not in ("causal", "window") or (mask == "window" and int(mask_size) <= 0):
        raise ValueError(f"attention mask {mask!r} of size {mask_size}: 'causal', or 'window' with a positive size")


@MIXERS.register("sink_attention")
class SinkAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, scale: float,
                 rotary_dim: int = 0, rope_theta: float = 10000.0, mask: str = "causal", mask_size: int = 0,
                 learned_sink: bool = True, values_are_keys: bool = False, names: Optional[Mapping[str, str]] = None,
                 qk_norm: bool = False, norm_eps: float = 1e-6, softcap: float = 0.0,
                 rope_scaling: Optional[Mapping] = None):
        if num_heads % num_kv_heads:
            raise ValueError(f"attention: {num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        _check_mask(mask, mask_size)
        self.D, self.H, self.G = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.dk, self.dv = int(key_dim), int(value_dim)
        if values_are_keys and self.dv != self.dk:
            raise ValueError(f"attention: values that are the keys need value_dim {value_dim} = key_dim {key_dim}")
        self.rot = int(rotary_dim)
        if self.rot % 2 or not (0 <= self.rot <= self.dk):
            raise ValueError(f"attention: rotary_dim {rotary_dim} must be even and at most key_dim {key_dim}")
        self.scale, self.theta = float(scale), float(rope_theta)
        self.mask, self.mask_size = mask, int(mask_size)
        self.learned_sink, self.values_are_keys = bool(learned_sink), bool(values_are_keys)
        self.qk_norm, self.eps, self.softcap = bool(qk_norm), float(norm_eps), float(softcap)
        if self.softcap < 0:
            raise ValueError(f"attention: the soft cap {softcap} must not be negative")
        self.rope_scaling = dict(rope_scaling) if rope_scaling else None
        self.names = {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink", "norm": ".norm", **dict(names or {})}
        self.k_off = self.H * self.dk
        self.v_off = self.k_off if self.values_are_keys else self.k_off + self.G * self.dk
        self.width = self.k_off + self.G * self.dk + (0 if self.values_are_keys else self.G * self.dv)

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        out = {n["q"]: ParamSpec((self.H * self.dk, self.D)), n["k"]: ParamSpec((self.G * self.dk, self.D))}
        if not self.values_are_keys:
            out[n["v"]] = ParamSpec((self.G * self.dv, self.D))
        if self.learned_sink:
            out[n["sink"]] = ParamSpec((self.H,), store="float32", init="normal")
        if self.qk_norm:
            out[n["q"] + n["norm"]] = ParamSpec((self.dk,), store="float32")
            out[n["k"] + n["norm"]] = ParamSpec((self.dk,), store="float32")
        out[n["o"]] = ParamSpec((self.D, self.H * self.dv))
        return out

    def cache_need(self):
        return PagedKeysValues(self.G, self.dk, self.dv, self.mask_size if self.mask == "window" else None)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names
        self.q_norm_w = self.k_norm_w = None
        if self.qk_norm:
            self.q_norm_w = to_device(tensors[n["q"] + n["norm"]], rt, torch.float32)
            self.k_norm_w = to_device(tensors[n["k"] + n["norm"]], rt, torch.float32)
        mats = [tensors[n["q"]], tensors[n["k"]]] + ([] if self.values_are_keys else [tensors[n["v"]]])
        dt = mats[0].dtype if all(m.dtype == mats[0].dtype for m in mats) else torch.float32
        self.w_in = ops.prepare_matrix(torch.cat([to_device(m, rt, dt) for m in mats], dim=0), rt.dtype)
        self.w_o = ops.prepare_matrix(to_device(tensors[n["o"]], rt), rt.dtype)
        self.sinks = to_device(tensors[n["sink"]], rt, torch.float32) if self.learned_sink else None
        self.cos_sin = rotary_table(self.rot, self.theta, rt, self.rope_scaling) if self.rot else None

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden]: the mixer's output."""
        pages = cache.get("mixer") if isinstance(cache, dict) else cache
        if not pages.writes:
            raise ValueError("an attention with keys and values of its own was given another entry's pages")
        h = as_normed(h).tensor()
        T, dev, dt = h.shape[0], h.device, self.rt.dtype
        proj = torch.empty((T, self.width), dtype=dt, device=dev)
        ops.linear(h, self.w_in, proj)
        q = proj[:, :self.k_off]                    # rotated where it lies: a head is read whole before it is written
        ops.rotary_pages(proj, 0, self.H, self.dk, 0, q, proj, self.k_off, self.dk, None, 0, 0, False, 0,
                         proj, self.v_off, self.dv, self.G, self.rot, self.cos_sin, step, pages.block_table, pages.kv,
                         pages.page_tokens, q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w, norm_eps=self.eps)
        attn = torch.empty((T, self.H * self.dv), dtype=dt, device=dev)
        ops.masked_attention(q, attn, self.H, self.G, self.dk, self.dv, pages.kv, pages.page_tokens, pages.block_table,
                             step, self.mask, self.mask_size, self.learned_sink, self.scale, sinks=self.sinks,
                             softcap=self.softcap)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(attn, self.w_o, out)
        return out


@MIXERS.register("latent_attention")
class LatentAttention(Mixer):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, value_dim: int, q_rank: int,
                 kv_rank: int, scale: float, rope_theta: float = 10000.0, norm_eps: float = 1e-6, mask: str = "causal",
                 mask_size: int = 0, learned_sink: bool = True, head_gate: bool = True,
                 names: Optional[Mapping[str, str]] = None):
        _check_mask(mask, mask_size)
        self.D, self.H = int(hidden_size), int(num_heads)
        self.dn, self.dr, self.dv = int(head_dim), int(rot_dim), int(value_dim)
        self.Q, self.R = int(q_rank), int(kv_rank)
        if self.dr % 2 or self.dr < 0 or self.dn < 0 or self.dn + self.dr <= 0:
            raise ValueError(f"latent attention: rot_dim {rot_dim} must be even, and a head needs elements")
        self.dk = self.dn + self.dr
        self.scale, self.theta, self.eps = float(scale), float(rope_theta), float(norm_eps)
        self.mask, self.mask_size = mask, int(mask_size)
        self.learned_sink, self.head_gate = bool(learned_sink), bool(head_gate)
        self.names = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk",
                      "uv": "uv", "sink": "sink", "gate": "g", "o": "o", **dict(names or {})}
        # columns of the first product's rows: query latent, key/value latent, the shared rotated key part, gate logits
        self.c_off, self.kr_off, self.g_off = self.Q, self.Q + self.R, self.Q + self.R + self.dr
        used = self.g_off + (self.H if self.head_gate else 0)
        self.down_width = -(-used // 8) * 8
        self.pad = self.down_width - used

    def param_specs(self) -> Dict[str, ParamSpec]:
        n = self.names
        out = {n["dq"]: ParamSpec((self.Q, self.D)), n["dq_norm"]: ParamSpec((self.Q,), store="float32"),
               n["uq"]: ParamSpec((self.H * self.dk, self.Q)), n["dkv"]: ParamSpec((self.R + self.dr, self.D)),
               n["dkv_norm"]: ParamSpec((self.R,), store="float32"), n["uk"]: ParamSpec((self.H * self.dn, self.R)),
               n["uv"]: ParamSpec((self.H * self.dv, self.R))}
        if self.learned_sink:
            out[n["sink"]] = ParamSpec((self.H,), store="float32", init="normal")
        if self.head_gate:
            out[n["gate"]] = ParamSpec((self.H, self.D))
        out[n["o"]] = ParamSpec((self.D, self.H * self.dv))
        return out

    def cache_need(self):
        return PagedKeysValues(self.H, self.dk, self.dv, self.mask_size if self.mask == "window" else None)

    def bind(self, tensors: Mapping[str, torch.Tensor], rt: Runtime) -> None:
        self.rt = rt
        n = self.names

        def stacked(keys, pad_rows=0):
            mats = [tensors[n[k]] for k in keys]
            dt = mats[0].dtype if all(m.dtype == mats[0].dtype for m in mats) else torch.float32
            mats = [to_device(m, rt, dt) for m in mats]
            if pad_rows:
                mats.append(torch.zeros((pad_rows, mats[0].shape[1]), dtype=dt, device=rt.device))
            return ops.prepare_matrix(torch.cat(mats, dim=0), rt.dtype)

        self.w_down = stacked(["dq", "dkv"] + (["gate"] if self.head_gate else []), self.pad)
        self.w_uq = ops.prepare_matrix(to_device(tensors[n["uq"]], rt), rt.dtype)
        self.w_ukv = stacked(["uk", "uv"])
        self.w_o = ops.prepare_matrix(to_device(tensors[n["o"]], rt), rt.dtype)
        self.q_norm_w = to_device(tensors[n["dq_norm"]], rt, torch.float32)
        self.kv_norm_w = to_device(tensors[n["dkv_norm"]], rt, torch.float32)
        self.sinks = to_device(tensors[n["sink"]], rt, torch.float32) if self.learned_sink else None
        self.cos_sin = rotary_table(self.dr, self.theta, rt) if self.dr else None

    def forward(self, h, step, cache) -> torch.Tensor:
        """float32 [rows, hidden]: the mixer's output."""
        pages = cache.get("mixer") if isinstance(cache, dict) else cache
        if not pages.writes:
            raise ValueError("a latent attention writes its own pages; it was given another entry's")
        h = as_normed(h).tensor()
        T, dev, dt = h.shape[0], h.device, self.rt.dtype
        H, dn, dv, dk = self.H, self.dn, self.dv, self.dk
        a = torch.empty((T, self.down_width), dtype=torch.float32, device=dev)     # the norms read 32-bit rows
        ops.linear(h, self.w_down, a)
        cq = torch.empty((T, self.Q), dtype=dt, device=dev)
        c = torch.empty((T, self.R), dtype=dt, device=dev)
        ops.rmsnorm_rows(a[:, :self.Q], self.q_norm_w, self.eps, cq)
        ops.rmsnorm_rows(a[:, self.c_off:self.kr_off], self.kv_norm_w, self.eps, c)
        q = torch.empty((T, H * dk), dtype=dt, device=dev)
        ops.linear(cq, self.w_uq, q)
        kv = torch.empty((T, H * (dn + dv)), dtype=dt, device=dev)
        ops.linear(c, self.w_ukv, kv)
        ops.rotary_pages(q, 0, H, dk, dn, q, kv, 0, dn, a, self.kr_off, self.dr, True, dn, kv, H * dn, dv, H, self.dr,
                         self.cos_sin, step, pages.block_table, pages.kv, pages.page_tokens)
        attn = torch.empty((T, H * dv), dtype=dt, device=dev)
        gate = a[:, self.g_off:self.g_off + H] if self.head_gate else None
        ops.masked_attention(q, attn, H, H, dk, dv, pages.kv, pages.page_tokens, pages.block_table, step, self.mask,
                             self.mask_size, self.learned_sink, self.scale, sinks=self.sinks, gate=gate)
        out = torch.empty((T, self.D), dtype=torch.float32, device=dev)
        ops.linear(attn, self.w_o, out)
        return out
