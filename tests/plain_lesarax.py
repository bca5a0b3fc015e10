"""A plain, slow reading of the Lesarax decoder in numpy (float64), one function per mechanism.  It shares no code
with the engine: tests compare the engine's parts and whole steps with it.

Notation: T tokens of one sequence at positions 0 .. T-1, D the model's width, H query heads, G key/value heads,
dk / dv key and value sizes of a head, r the rotated elements of a head, E experts of which a token uses K.
`rnd` (where a function takes it) rounds a stored activation: the identity for the exact model, a rounding to
bfloat16 for the estimate of what 16-bit activations cost."""
from __future__ import annotations

import json
import math
import os
from typing import Callable, Dict, List, Optional

import numpy as np


def exact(x):
    return x


def to_bf16(x):
    """Round to the nearest bfloat16 (ties to even), returned as float64."""
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    u = a.view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64).reshape(a.shape)


# ---------------------------------------------------------------------------------------------- single mechanisms
def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def rotate(v: np.ndarray, positions, base: float) -> np.ndarray:
    """v [T, ..., r]: element i and element i + r/2 of the last axis are a pair, turned by position * base^(-2i/r)."""
    r = v.shape[-1]
    half = r // 2
    f = np.power(float(base), -2.0 * np.arange(half) / r)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    shape = (v.shape[0],) + (1,) * (v.ndim - 2) + (half,)
    c, s = np.cos(ang).reshape(shape), np.sin(ang).reshape(shape)
    a, b = v[..., :half], v[..., half:]
    return np.concatenate([a * c - b * s, b * c + a * s], axis=-1)


def rotate_front(v: np.ndarray, positions, base: float, r: int) -> np.ndarray:
    """The first r elements of the last axis are rotated, the others stay."""
    return np.concatenate([rotate(v[..., :r], positions, base), v[..., r:]], axis=-1)


def sink_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, sinks: Optional[np.ndarray],
                   window: Optional[int] = None, q_pos0: Optional[int] = None) -> np.ndarray:
    """q [Tq, H, dk] are the last Tq of the Tk positions of k [Tk, G, dk], v [Tk, G, dv] (or start at `q_pos0`).  The
    row at position p sees the keys j <= p, with a window only those with p - j < window.  The softmax's denominator
    holds one more term, exp(sinks[h]), which has no value.  Head h reads key/value head h // (H / G)."""
    Tq, H = q.shape[0], q.shape[1]
    Tk, G, dv = v.shape
    first = Tk - Tq if q_pos0 is None else q_pos0
    out = np.zeros((Tq, H, dv))
    for h in range(H):
        g = h // (H // G)
        for a in range(Tq):
            p = first + a
            lo = 0 if window is None else max(0, p - window + 1)
            s = (k[lo:p + 1, g] @ q[a, h]) * scale
            m = s.max() if sinks is None else max(s.max(), float(sinks[h]))
            e = np.exp(s - m)
            den = e.sum() + (0.0 if sinks is None else math.exp(float(sinks[h]) - m))
            out[a, h] = (e / den) @ v[lo:p + 1, g]
    return out


def clamped_unit(h: np.ndarray, w_gate, w_up, w_down, limit: float, rnd: Callable = exact) -> np.ndarray:
    g = np.minimum(rnd(h @ w_gate.T), limit)
    u = np.clip(rnd(h @ w_up.T), -limit, limit)
    return rnd(g * sigmoid(1.702 * g) * (u + 1.0)) @ w_down.T


def route(z: np.ndarray, top: int):
    """z [T, E] -> (ids [T, K] by falling logit, weights [T, K]: the softmax over the chosen logits alone)."""
    ids = np.argsort(-z, axis=-1, kind="stable")[:, :top]
    zz = np.take_along_axis(z, ids, axis=-1)
    e = np.exp(zz - zz.max(axis=-1, keepdims=True))
    return ids, e / e.sum(axis=-1, keepdims=True)


def experts(h: np.ndarray, W: Dict[str, np.ndarray], p: str, n_experts: int, top: int, limit: float,
            rnd: Callable = exact) -> np.ndarray:
    ids, wts = route(h @ W[p + "router"].T, top)
    out = np.zeros((h.shape[0], W[p + "e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(ids[t, j])
            out[t] += wts[t, j] * clamped_unit(h[t:t + 1], W[f"{p}e{e}.gate"], W[f"{p}e{e}.up"], W[f"{p}e{e}.down"],
                                               limit, rnd)[0]
    return out


# ---------------------------------------------------------------------------------------------- the two mixers
def attention_mixer(h: np.ndarray, W: Dict[str, np.ndarray], p: str, m: dict, rnd: Callable = exact) -> np.ndarray:
    """Grouped heads whose values are the keys as projected (before the rotation); a window if the mixer names one."""
    T = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    pos = np.arange(T)
    q = rnd(h @ W[p + "q"].T).reshape(T, H, dk)
    k = rnd(h @ W[p + "k"].T).reshape(T, G, dk)
    r, base = m["rot"]["dims"], m["rot"]["base"]
    o = sink_attention(rnd(rotate_front(q, pos, base, r)), rnd(rotate_front(k, pos, base, r)), k, m["scale"],
                       W[p + "sink"], window=(m.get("mask") or {}).get("size"))
    return rnd(o.reshape(T, -1)) @ W[p + "o"].T


def latent_mixer(h: np.ndarray, W: Dict[str, np.ndarray], p: str, m: dict, eps: float,
                 rnd: Callable = exact) -> np.ndarray:
    """Queries, keys and values through low-rank latents; one rotated key part shared by the heads; a window."""
    T = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T)
    base = m["rot"]["base"]
    cq = rnd(rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], eps))
    q = rnd(cq @ W[p + "uq"].T).reshape(T, H, dn + dr)
    q = np.concatenate([q[..., :dn], rnd(rotate(q[..., dn:], pos, base))], axis=-1)
    kv = h @ W[p + "dkv"].T
    c = rnd(rms_norm(kv[:, :R], W[p + "dkv.norm"], eps))
    k_rot = rnd(rotate(kv[:, None, R:], pos, base))                      # [T, 1, dr]
    k_plain = rnd(c @ W[p + "uk"].T).reshape(T, H, dn)
    v = rnd(c @ W[p + "uv"].T).reshape(T, H, dv)
    k = np.concatenate([k_plain, np.broadcast_to(k_rot, (T, H, dr))], axis=-1)
    o = sink_attention(q, k, v, m["scale"], W[p + "sink"], window=(m.get("mask") or {}).get("size"))
    o = o * sigmoid(h @ W[p + "g"].T)[:, :, None]
    return rnd(o.reshape(T, -1)) @ W[p + "o"].T


# ---------------------------------------------------------------------------------------------- the model
def layer_order(cfg: dict) -> List[tuple]:
    """[(layer, starts a pass)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(a)]
    for _ in range(times):
        order += [(i, i == a) for i in range(a, b)]
    return order + [(i, False) for i in range(b, n)]


def forward(cfg: dict, W: Dict[str, np.ndarray], tokens, rnd: Callable = exact, taps: Optional[list] = None):
    """Logits [T, vocab] of a whole sequence; `taps` (a list) receives the residual after every layer that ran."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x0 = W["embed"][np.asarray(tokens)]
    x = x0.copy()
    for i, enters in layer_order(cfg):
        if enters:
            x = np.concatenate([rnd(x), rnd(x0)], axis=-1) @ W["loop.in"].T
        L, p = cfg["layers"][i], f"l{i}."
        h = rnd(rms_norm(x, W[p + "norm1"], eps))
        if L["type"] == "attention":
            y = attention_mixer(h, W, p + "mix.", L["mixer"], rnd)
        elif L["type"] == "latent_attention":
            y = latent_mixer(h, W, p + "mix.", L["mixer"], eps, rnd)
        else:
            raise ValueError(L["type"])
        x = x + mult * y
        f = L.get("mlp")
        if f is not None:
            h = rnd(rms_norm(x, W[p + "norm2"], eps))
            x = x + mult * experts(h, W, p + "mlp.", f["router"]["experts"], f["router"]["top"], f["expert"]["limit"],
                                   rnd)
        if taps is not None:
            taps.append(x.copy())
    return rnd(rms_norm(x, W["final.norm"], eps)) @ W["embed"].T


# ---------------------------------------------------------------------------------------------- tensors of a model
def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    D, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, D), "final.norm": (D,)}
    if cfg.get("loop"):
        out["loop.in"] = (D, 2 * D)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        out[p + "norm1"] = (D,)
        if L["type"] == "attention":
            H, G, dk = m["heads"], m["kv_heads"], m["dim"]
            out.update({p + "mix.q": (H * dk, D), p + "mix.k": (G * dk, D), p + "mix.sink": (H,),
                        p + "mix.o": (D, H * m["vdim"])})
        else:
            H, dn, dr, dv, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            out.update({p + "mix.dq": (Q, D), p + "mix.dq.norm": (Q,), p + "mix.uq": (H * (dn + dr), Q),
                        p + "mix.dkv": (R + dr, D), p + "mix.dkv.norm": (R,), p + "mix.uk": (H * dn, R),
                        p + "mix.uv": (H * dv, R), p + "mix.sink": (H,), p + "mix.g": (H, D),
                        p + "mix.o": (D, H * dv)})
        f = L.get("mlp")
        if f is not None:
            out[p + "norm2"] = (D,)
            F = f["expert"]["ff"]
            out[p + "mlp.router"] = (f["router"]["experts"], D)
            for e in range(f["router"]["experts"]):
                out.update({f"{p}mlp.e{e}.gate": (F, D), f"{p}mlp.e{e}.up": (F, D), f"{p}mlp.e{e}.down": (D, F)})
    return out


def random_weights(cfg: dict, seed: int, sharp: float = 1.0) -> Dict[str, np.ndarray]:
    """Weights that are exact in bfloat16.  Matrices N(0, 1/sqrt(inputs)); the matrices that make queries and keys
    times `sharp`, so that scores spread and a wrong key shows; norm weights near 1; sinks N(0, 1)."""
    rng = np.random.default_rng(seed)
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        last = name.split(".")[-1]
        if name.endswith("norm") or last in ("norm1", "norm2"):
            w = 1.0 + 0.1 * rng.standard_normal(shape)
        elif last == "sink":
            w = rng.standard_normal(shape)
        elif name == "embed":
            w = rng.standard_normal(shape)
        else:
            w = rng.standard_normal(shape) / math.sqrt(shape[-1])
            if last in ("q", "k", "uq", "uk", "dkv"):
                w = w * sharp
            if last == "router":
                w = w * 2.0
        W[name] = to_bf16(w)
    return W


# ---------------------------------------------------------------------------------------------- folders, generation
def read_model_folder(path: str):
    """(config dict, name -> float64 array) of a folder with config.json and model.safetensors: 8 bytes of length,
    that many bytes of JSON (name -> dtype, shape, data_offsets), then the data."""
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    with open(os.path.join(path, "model.safetensors"), "rb") as f:
        n = int.from_bytes(f.read(8), "little")
        head = json.loads(f.read(n))
        data = f.read()
    W = {}
    for name, e in head.items():
        if name == "__metadata__":
            continue
        lo, hi = e["data_offsets"]
        if e["dtype"] == "BF16":
            a = (np.frombuffer(data[lo:hi], dtype="<u2").astype(np.uint32) << 16).view(np.float32)
        elif e["dtype"] == "F32":
            a = np.frombuffer(data[lo:hi], dtype="<f4")
        else:
            raise ValueError(f"{name}: element type {e['dtype']}")
        W[name] = a.astype(np.float64).reshape(e["shape"])
    return cfg, W


def greedy(cfg: dict, W: Dict[str, np.ndarray], prompt, n: int) -> List[int]:
    """The n tokens that follow `prompt` when the largest logit is taken every time (the lowest id wins a tie).  The
    whole sequence is computed anew for every token: this implementation keeps nothing between calls."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(forward(cfg, W, toks)[-1])))
    return toks[len(prompt):]
