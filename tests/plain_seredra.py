"""A plain, slow reading of the Seredra decoder in numpy (float64), one function per mechanism.  It shares no code
with the engine: tests compare the engine's parts and whole steps with it.

Notation: T tokens of one sequence at positions 0 .. T-1, D the model's width, H query heads, G key/value heads,
dk / dv key and value sizes of a head, r the rotated elements of a head, C channels and N states of the selective
scan, E experts of which a token uses K.  `rnd` (where a function takes it) rounds a stored activation: the identity
for the exact model, a rounding to bfloat16 for the estimate of what 16-bit activations cost.

Two forms of the recurrent mechanisms stand side by side: over a whole sequence (`forward`), and token by token with
the state carried in a dict (`Stepper`); the tests hold the one against the other."""
from __future__ import annotations

import json
import math
import os
import struct
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
def unit_rms(x: np.ndarray, eps: float) -> np.ndarray:
    """x over its root mean square along the last axis, eps inside the root."""
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def scalar_norm(x: np.ndarray, g: float, eps: float) -> np.ndarray:
    return unit_rms(x, eps) * float(g)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def relu2(z):
    return np.maximum(z, 0.0) ** 2


def short_conv(u: np.ndarray, w: np.ndarray, before: Optional[np.ndarray] = None) -> np.ndarray:
    """u [T, C], w [C, n]: y[t] = sum_j w[:, j] * u[t - (n - 1) + j], with `before` [n - 1, C] (zeros if None) standing
    in front of the sequence.  The last column of w is the current token's."""
    T, C = u.shape
    n = w.shape[1]
    pad = np.zeros((n - 1, C)) if before is None else np.asarray(before, dtype=np.float64)
    full = np.concatenate([pad, u], axis=0)
    y = np.zeros((T, C))
    for j in range(n):
        y += w[:, j][None, :] * full[j:j + T]
    return y


def frequencies(rot: dict) -> tuple:
    """(frequency of every pair, what cosines and sines are multiplied with) of a rotation {"base", "dims", "scaling"}."""
    r, base = int(rot["dims"]), float(rot["base"])
    i = np.arange(r // 2, dtype=np.float64)
    f = np.power(base, -2.0 * i / r)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def dim_at(turns):
        return r * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_at(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_at(float(sc["slow"]))), r - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_front(v: np.ndarray, positions, rot: dict) -> np.ndarray:
    """v [T, heads, d]: of the first r elements of a head, element i and element i + r/2 are a pair, turned by the angle
    position * frequency_i; the other elements stay."""
    r = int(rot["dims"])
    if r == 0:
        return v
    half = r // 2
    f, mag = frequencies(rot)
    ang = np.asarray(positions, dtype=np.float64)[:, None] * f[None, :]
    c, s = (np.cos(ang) * mag)[:, None, :], (np.sin(ang) * mag)[:, None, :]
    a, b = v[..., :half], v[..., half:r]
    return np.concatenate([a * c - b * s, b * c + a * s, v[..., r:]], axis=-1)


def query_temperature(positions, coef: float, every: int) -> np.ndarray:
    p = np.asarray(positions, dtype=np.float64)
    return 1.0 + coef * np.log(np.floor((p + 1.0) / every) + 1.0)


def softmax_attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float, q_pos0: int = 0,
                      softcap: float = 0.0, r1: Optional[np.ndarray] = None, r2: Optional[np.ndarray] = None) -> np.ndarray:
    """q [Tq, H, dk] stand at positions q_pos0 .. of the keys k [Tk, G, dk] with values v [Tk, G, dv].  The row at
    position p sees the keys j <= p.  Score (q . k) * scale, then c * tanh(score / c) with a soft cap c, then less
    r1[h] * ln(1 + r2[h] * (p - j)) with a distance penalty.  Head h reads key/value head h // (H / G)."""
    Tq, H = q.shape[0], q.shape[1]
    G, dv = v.shape[1], v.shape[2]
    out = np.zeros((Tq, H, dv))
    for h in range(H):
        g = h // (H // G)
        for a in range(Tq):
            p = q_pos0 + a
            s = (k[:p + 1, g] @ q[a, h]) * scale
            if softcap:
                s = softcap * np.tanh(s / softcap)
            if r1 is not None:
                s = s - r1[h] * np.log(1.0 + r2[h] * (p - np.arange(p + 1)))
            e = np.exp(s - s.max())
            out[a, h] = (e / e.sum()) @ v[:p + 1, g]
    return out


def retention(q: np.ndarray, k: np.ndarray, v: np.ndarray, decay, S0: Optional[np.ndarray] = None):
    """q, k [T, H, dk], v [T, H, dv]: S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  Returns (o, last S)."""
    T, H, dk = q.shape
    dv = v.shape[2]
    S = np.zeros((H, dk, dv)) if S0 is None else np.array(S0, dtype=np.float64)
    o = np.zeros((T, H, dv))
    for t in range(T):
        for h in range(H):
            S[h] = decay[h] * S[h] + np.outer(k[t, h], v[t, h])
            o[t, h] = S[h].T @ q[t, h]
    return o, S


def selective_scan(x: np.ndarray, dt: np.ndarray, A: np.ndarray, B: np.ndarray, C: np.ndarray, Dw: np.ndarray,
                   S0: Optional[np.ndarray] = None):
    """x, dt [T, C]; A [C, N]; B, C [T, N]: S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;
    y_c = sum_n S[c, n] C_n + D_c x_c.  Returns (y, last S)."""
    T, ch = x.shape
    S = np.zeros(A.shape) if S0 is None else np.array(S0, dtype=np.float64)
    y = np.zeros((T, ch))
    for t in range(T):
        S = np.exp(dt[t][:, None] * A) * S + (dt[t] * x[t])[:, None] * B[t][None, :]
        y[t] = S @ C[t] + Dw * x[t]
    return y, S


def route(z: np.ndarray, top: int):
    """(the `top` experts with the largest sigmoid(z), lower index first on a tie; their scores, not renormalised)."""
    s = sigmoid(z)
    ids = np.argsort(-s, kind="stable")[:top]
    return ids, s[ids]


# ---------------------------------------------------------------------------------------------- mixers, feed-forwards
def conv_attention_mixer(h, W, p, m, eps, positions, kv=None, before=None, rnd: Callable = exact):
    """The attention whose projections pass a short convolution.  `kv`: (keys, values) of the layer it reads instead of
    its own (then it has no k and v); `before`: {"q": .., "k": .., "v": ..} projected rows in front of `h`'s first.
    Returns (output, (keys, values) as the cache holds them, the projected rows)."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    taps = int(m.get("conv") or 0)
    before = before or {}
    proj = {}

    def through(n):
        u = rnd(h @ W[p + n].T + W[p + n + ".b"])
        proj[n] = u
        return short_conv(u, W[p + n + ".conv"], before.get(n)) if taps else u

    q = unit_rms(through("q"), eps) * W[p + "q.norm"]
    if m.get("q_temp"):
        q = q * query_temperature(positions, m["q_temp"]["coef"], m["q_temp"]["every"])[:, None]
    q = rnd(q).reshape(T, H, dk)
    if kv is None:
        k = rnd(unit_rms(through("k"), eps) * W[p + "k.norm"]).reshape(T, G, dk)
        v = rnd(through("v")).reshape(T, G, dv)
    else:
        k, v = kv
    if before.get("keys") is not None:
        k_all, v_all = np.concatenate([before["keys"], k]), np.concatenate([before["values"], v])
    else:
        k_all, v_all = k, v
    o = softmax_attention(q, k_all, v_all, m["scale"], q_pos0=int(positions[0]), r1=W[p + "r1"], r2=W[p + "r2"])
    return rnd(o).reshape(T, H * dv) @ W[p + "o"].T + W[p + "o.b"], (k, v), proj


def left_mixer(h, W, p, m, eps, positions, before=None, rnd: Callable = exact):
    """The attention of the side-by-side mixer: values are the keys as projected, norm per head, rotation, soft cap."""
    T = h.shape[0]
    H, G, dk = m["heads"], m["kv_heads"], m["dim"]
    q = rnd(h @ W[p + "q"].T).reshape(T, H, dk)
    k = rnd(h @ W[p + "k"].T).reshape(T, G, dk)
    v = k
    q = rnd(rotate_front(unit_rms(q, eps) * W[p + "q.norm"], positions, m["rot"]))
    kn = rnd(rotate_front(unit_rms(k, eps) * W[p + "k.norm"], positions, m["rot"]))
    if before is not None:
        k_all, v_all = np.concatenate([before["keys"], kn]), np.concatenate([before["values"], v])
    else:
        k_all, v_all = kn, v
    o = softmax_attention(q, k_all, v_all, m["scale"], q_pos0=int(positions[0]), softcap=float(m.get("softcap") or 0.0))
    return rnd(o).reshape(T, H * dk) @ W[p + "o"].T, (kn, v)


def right_mixer(h, W, p, m, state=None, rnd: Callable = exact):
    """The selective scan of the side-by-side mixer.  `state`: {"conv": the last inputs, "S": the scan's state}."""
    C, N, R = m["inner"], m["state"], m["dt_rank"]
    state = state or {}
    xz = rnd(h @ W[p + "in"].T)
    x_in, z = xz[:, :C], xz[:, C:]
    x = rnd(silu(short_conv(x_in, W[p + "conv"], state.get("conv")) + W[p + "conv.b"]))
    low = rnd(x @ W[p + "x"][:R].T)
    bc = x @ W[p + "x"][R:].T
    dt = softplus(low @ W[p + "dt"].T + W[p + "dt.b"])
    y, S = selective_scan(x, dt, -np.exp(W[p + "A_log"]), bc[:, :N], bc[:, N:], W[p + "D"], state.get("S"))
    taps = W[p + "conv"].shape[1]
    held = np.concatenate([state.get("conv", np.zeros((taps - 1, C))), x_in])[-(taps - 1):] if taps > 1 else None
    return rnd(y * silu(z)) @ W[p + "o"].T, {"conv": held, "S": S}


def retention_mixer(h, W, p, m, eps, positions, S0=None, rnd: Callable = exact):
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = rnd(h @ W[p + "q"].T).reshape(T, H, dk)
    k = rnd(h @ W[p + "k"].T).reshape(T, H, dk)
    v = rnd(h @ W[p + "v"].T).reshape(T, H, dv)
    q = rotate_front(q, positions, m["rot"])
    k = rotate_front(k, positions, m["rot"]) * dk ** -0.5
    o, S = retention(q, k, v, m["decay"], S0)
    g = rnd(h @ W[p + "g"].T)
    return rnd(unit_rms(o, eps).reshape(T, H * dv) * silu(g)) @ W[p + "o"].T, S


def dense_ff(h, W, p, rnd: Callable = exact):
    return rnd(relu2(h @ W[p + "up"].T)) @ W[p + "down"].T


def expert_ff(h, W, p, f, rnd: Callable = exact):
    """Every token's chosen experts on the token times the expert's score; the outputs are added as they are."""
    E, K = f["router"]["experts"], f["router"]["top"]
    z = h @ W[p + "router"].T
    out = np.zeros_like(h)
    for t in range(h.shape[0]):
        ids, w = route(z[t], K)
        for e, we in zip(ids, w):
            x = we * h[t]
            a = rnd(silu(x @ W[f"{p}e{e}.gate"].T) * (x @ W[f"{p}e{e}.up"].T))
            out[t] += a @ W[f"{p}e{e}.down"].T
    return out


# ---------------------------------------------------------------------------------------------- the model
def forward(cfg: dict, W: Dict[str, np.ndarray], tokens, rnd: Callable = exact, taps: Optional[list] = None):
    """Logits [T, vocab] of one whole sequence; `taps` (a list) receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    T = len(tokens)
    pos = np.arange(T)
    x = W["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
    kv = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        h = rnd(scalar_norm(x, W[f"l{i}.norm1"], eps))
        if layer["type"] == "attention":
            src = m.get("kv_from")
            y, kv[i], _ = conv_attention_mixer(h, W, p, m, eps, pos, kv=None if src is None else kv[src], rnd=rnd)
        elif layer["type"] == "parallel":
            a, _ = left_mixer(h, W, p + "left.", m["left"], eps, pos, rnd=rnd)
            b, _ = right_mixer(h, W, p + "right.", m["right"], rnd=rnd)
            y = m["left_scale"] * a + m["right_scale"] * b
        elif layer["type"] == "retention":
            y, _ = retention_mixer(h, W, p, m, eps, pos, rnd=rnd)
        else:
            raise ValueError(layer["type"])
        x = x + y
        f = layer.get("mlp")
        if f is not None:
            h = rnd(scalar_norm(x, W[f"l{i}.norm2"], eps))
            x = x + (dense_ff(h, W, f"l{i}.mlp.", rnd) if f["kind"] == "dense" else expert_ff(h, W, f"l{i}.mlp.", f, rnd))
        if taps is not None:
            taps.append(x.copy())
    return rnd(scalar_norm(x, W["final.norm"], eps)) @ W["head"].T


class Stepper:
    """The same model fed in portions of any size: keys, values, projected rows, last inputs and states are kept here
    between calls, as a cache would keep them."""

    def __init__(self, cfg: dict, W: Dict[str, np.ndarray]):
        self.cfg, self.W, self.n = cfg, W, 0
        self.kept: Dict[int, dict] = {i: {} for i in range(len(cfg["layers"]))}

    def feed(self, tokens) -> np.ndarray:
        cfg, W = self.cfg, self.W
        eps = cfg["norm"]["eps"]
        T = len(tokens)
        pos = np.arange(self.n, self.n + T)
        x = W["embed"][np.asarray(tokens)] * cfg["embedding"]["scale"]
        fresh = {}
        for i, layer in enumerate(cfg["layers"]):
            p, m, st = f"l{i}.mix.", layer["mixer"], self.kept[i]
            h = scalar_norm(x, W[f"l{i}.norm1"], eps)
            if layer["type"] == "attention":
                taps = int(m.get("conv") or 0)
                src = m.get("kv_from")
                before = {n: st.get("rows_" + n) for n in ("q", "k", "v")}
                owner = self.kept[i if src is None else src]
                before["keys"], before["values"] = owner.get("keys"), owner.get("values")
                y, (k, v), proj = conv_attention_mixer(h, W, p, m, eps, pos, kv=None if src is None else fresh[src],
                                                       before=before, rnd=exact)
                fresh[i] = (k, v)
                for n, u in proj.items():
                    if taps > 1:
                        old = st.get("rows_" + n)
                        old = np.zeros((taps - 1, u.shape[1])) if old is None else old
                        st["rows_" + n] = np.concatenate([old, u])[-(taps - 1):]
            elif layer["type"] == "parallel":
                a, (k, v) = left_mixer(h, W, p + "left.", m["left"], eps, pos,
                                       before=st if st.get("keys") is not None else None)
                fresh[i] = (k, v)
                b, st["right"] = right_mixer(h, W, p + "right.", m["right"], st.get("right"))
                y = m["left_scale"] * a + m["right_scale"] * b
            else:
                y, st["S"] = retention_mixer(h, W, p, m, eps, pos, st.get("S"))
            x = x + y
            f = layer.get("mlp")
            if f is not None:
                h = scalar_norm(x, W[f"l{i}.norm2"], eps)
                x = x + (dense_ff(h, W, f"l{i}.mlp.") if f["kind"] == "dense" else expert_ff(h, W, f"l{i}.mlp.", f))
        for i, (k, v) in fresh.items():          # (after all layers: a borrower of this portion has read the old keys)
            st = self.kept[i]
            if self.cfg["layers"][i]["mixer"].get("kv_from") is None:
                st["keys"] = k if st.get("keys") is None else np.concatenate([st["keys"], k])
                st["values"] = v if st.get("values") is None else np.concatenate([st["values"], v])
        self.n += T
        return scalar_norm(x, W["final.norm"], eps) @ W["head"].T


# ---------------------------------------------------------------------------------------------- tensors and folders
def tensor_shapes(cfg: dict) -> Dict[str, tuple]:
    D, V = cfg["width"], cfg["vocab"]
    out = {"embed": (V, D), "final.norm": (), "head": (V, D)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.mix.", layer["mixer"]
        out[f"l{i}.norm1"] = ()
        if layer["type"] == "attention":
            H, G, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], int(m.get("conv") or 0)
            rows = {"q": H * dk} if m.get("kv_from") is not None else {"q": H * dk, "k": G * dk, "v": G * dv}
            for n, r in rows.items():
                out[p + n], out[p + n + ".b"] = (r, D), (r,)
                if taps:
                    out[p + n + ".conv"] = (r, taps)
                if n != "v":
                    out[p + n + ".norm"] = (r,)
            out[p + "r1"] = out[p + "r2"] = (H,)
            out[p + "o"], out[p + "o.b"] = (D, H * dv), (D,)
        elif layer["type"] == "parallel":
            l, r = m["left"], m["right"]
            out[p + "left.q"], out[p + "left.k"] = (l["heads"] * l["dim"], D), (l["kv_heads"] * l["dim"], D)
            out[p + "left.q.norm"] = out[p + "left.k.norm"] = (l["dim"],)
            out[p + "left.o"] = (D, l["heads"] * l["dim"])
            C, N, R = r["inner"], r["state"], r["dt_rank"]
            out[p + "right.in"], out[p + "right.conv"], out[p + "right.conv.b"] = (2 * C, D), (C, r["conv"]), (C,)
            out[p + "right.x"], out[p + "right.dt"], out[p + "right.dt.b"] = (R + 2 * N, C), (C, R), (C,)
            out[p + "right.A_log"], out[p + "right.D"], out[p + "right.o"] = (C, N), (C,), (D, C)
        else:
            H, dk, dv = m["heads"], m["dim"], m["vdim"]
            out[p + "q"] = out[p + "k"] = (H * dk, D)
            out[p + "v"] = out[p + "g"] = (H * dv, D)
            out[p + "o"] = (D, H * dv)
        f = layer.get("mlp")
        if f is not None:
            out[f"l{i}.norm2"] = ()
            if f["kind"] == "dense":
                out[f"l{i}.mlp.up"], out[f"l{i}.mlp.down"] = (f["ff"], D), (D, f["ff"])
            else:
                out[f"l{i}.mlp.router"] = (f["router"]["experts"], D)
                for e in range(f["router"]["experts"]):
                    out[f"l{i}.mlp.e{e}.gate"] = out[f"l{i}.mlp.e{e}.up"] = (f["expert"]["ff"], D)
                    out[f"l{i}.mlp.e{e}.down"] = (D, f["expert"]["ff"])
    return out


def read_safetensors(path: str) -> Dict[str, np.ndarray]:
    """A reader of its own: 8 bytes of length, that many of JSON, then the data (F32 and BF16)."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        meta = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, e in meta.items():
        if name == "__metadata__":
            continue
        a, b = e["data_offsets"]
        if e["dtype"] == "F32":
            v = np.frombuffer(data[a:b], dtype="<f4").astype(np.float64)
        elif e["dtype"] == "BF16":
            v = (np.frombuffer(data[a:b], dtype="<u2").astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        else:
            raise ValueError(f"{name}: element type {e['dtype']}")
        out[name] = v.reshape(e["shape"])
    return out


def read_model_folder(path: str):
    with open(os.path.join(path, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(path, "model.safetensors"))


def greedy(cfg: dict, W: Dict[str, np.ndarray], prompt, n: int) -> List[int]:
    toks, out = list(prompt), []
    for _ in range(n):
        nxt = int(np.argmax(forward(cfg, W, toks)[-1]))
        out.append(nxt)
        toks.append(nxt)
    return out
