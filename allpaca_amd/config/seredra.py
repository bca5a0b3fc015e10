"""Typed configuration of the Seredra decoder, read from config.json.

Keys: `vocab`, `width`, `embedding.scale`, `norm.eps`, `max_positions` (optional) and `layers`, a list of
{"type", "mixer", "mlp"}.
  type "attention": `heads`, `kv_heads`, `dim` (query and key size of a head), `vdim`, `scale`, `conv` (taps of the
      short convolution on q, k and v; absent or 0: none), `q_temp` ({"coef", "every"}; absent: none), `kv_from` (the
      layer whose keys and values it reads instead of its own).
  type "parallel": `left` (an attention: `heads`, `kv_heads`, `dim`, `vdim` = `dim`, `scale`, `softcap` (absent: none),
      `rot` {"base", "dims", "scaling": {"factor", "original", "fast", "slow"} or absent}), `right` (a selective scan:
      `inner`, `state`, `dt_rank`, `conv`), `left_scale`, `right_scale`.
  type "retention": `heads`, `dim`, `vdim`, `decay` (one number a head), `rot` {"base", "dims"}.
  `mlp`: null, {"kind": "dense", "ff"}, or {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top"}}.
A size that the file leaves out is taken from the shape of the tensor that has it (`sizes_from_tensors`); constants
come from the file alone."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Mapping, Optional, Tuple, Union

from .lesarax import DEFAULT_MAX_POSITIONS, _obj, _rot
from .llama import ConfigError
from .risizen import _int, _num


@dataclass(frozen=True)
class SeredraAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0                                   # taps; 0: no convolution
    q_temp: Optional[Tuple[float, int]] = None      # (coef, every)
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class SeredraYarn:
    factor: float
    original: float
    fast: float
    slow: float


@dataclass(frozen=True)
class SeredraLeft:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float                                  # 0: none
    rot_dims: int
    rot_base: float
    scaling: Optional[SeredraYarn] = None


@dataclass(frozen=True)
class SeredraRight:
    inner: int
    state: int
    dt_rank: int
    conv: int


@dataclass(frozen=True)
class SeredraParallel:
    left: SeredraLeft
    right: SeredraRight
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class SeredraRetention:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class SeredraDense:
    ff: int


@dataclass(frozen=True)
class SeredraExperts:
    ff: int
    experts: int
    top: int


@dataclass(frozen=True)
class SeredraLayer:
    mixer: Union[SeredraAttention, SeredraParallel, SeredraRetention]
    mlp: Union[None, SeredraDense, SeredraExperts]


TYPES = ("attention", "parallel", "retention")


def sizes_from_tensors(d: Mapping[str, Any], shapes: Mapping[str, Tuple[int, ...]]) -> Mapping[str, Any]:
    """config.json with the sizes it leaves out filled in from the shapes of the stored tensors (`embed`,
    `l<i>.mix.*`, `l<i>.mlp.*`).  A size the file names is left as it is: a disagreement shows when the weights load."""
    def dim_of(name: str, axis: int = 0) -> Optional[int]:
        shape = shapes.get(name)
        return int(shape[axis]) if shape is not None and len(shape) > axis else None

    def fill(m: dict, key: str, value) -> None:
        if m.get(key) is None and value is not None:
            m[key] = value

    def over(a: Optional[int], b) -> Optional[int]:
        return a // b if a and isinstance(b, int) and not isinstance(b, bool) and b > 0 and a % b == 0 else None

    out = dict(d)
    if len(shapes.get("embed", ())) == 2:
        fill(out, "vocab", int(shapes["embed"][0]))
        fill(out, "width", int(shapes["embed"][1]))
    layers = d.get("layers")
    if not isinstance(layers, list):
        return out
    out["layers"] = new_layers = []
    for i, entry in enumerate(layers):
        if not isinstance(entry, Mapping) or not isinstance(entry.get("mixer"), Mapping):
            new_layers.append(entry)
            continue
        p, kind = f"l{i}.mix.", entry.get("type")
        m = dict(entry["mixer"])
        if kind == "attention":
            fill(m, "heads", dim_of(p + "r1"))
            fill(m, "dim", over(dim_of(p + "q"), m.get("heads")))
            fill(m, "heads", over(dim_of(p + "q"), m.get("dim")))
            fill(m, "vdim", over(dim_of(p + "o", 1), m.get("heads")))
            src = m.get("kv_from")
            if isinstance(src, int) and not isinstance(src, bool) and 0 <= src < len(new_layers) \
                    and isinstance(new_layers[src], Mapping) and isinstance(new_layers[src].get("mixer"), Mapping):
                fill(m, "kv_heads", new_layers[src]["mixer"].get("kv_heads"))
            else:
                fill(m, "kv_heads", over(dim_of(p + "k"), m.get("dim")))
                fill(m, "vdim", over(dim_of(p + "v"), m.get("kv_heads")))
            if "conv" not in m:
                fill(m, "conv", dim_of(p + "q.conv", 1))
        elif kind == "parallel":
            left = dict(m["left"]) if isinstance(m.get("left"), Mapping) else {}
            right = dict(m["right"]) if isinstance(m.get("right"), Mapping) else {}
            fill(left, "dim", dim_of(p + "left.q.norm"))
            fill(left, "heads", over(dim_of(p + "left.q"), left.get("dim")))
            fill(left, "dim", over(dim_of(p + "left.q"), left.get("heads")))
            fill(left, "kv_heads", over(dim_of(p + "left.k"), left.get("dim")))
            fill(left, "vdim", left.get("dim"))
            fill(right, "inner", dim_of(p + "right.conv"))
            fill(right, "conv", dim_of(p + "right.conv", 1))
            fill(right, "dt_rank", dim_of(p + "right.dt", 1))
            fill(right, "state", dim_of(p + "right.A_log", 1))
            m["left"], m["right"] = left, right
        elif kind == "retention":
            if isinstance(m.get("decay"), list):
                fill(m, "heads", len(m["decay"]))
            fill(m, "dim", over(dim_of(p + "q"), m.get("heads")))
            fill(m, "vdim", over(dim_of(p + "v"), m.get("heads")))
        e = dict(entry, mixer=m)
        f = entry.get("mlp")
        if isinstance(f, Mapping):
            f = dict(f)
            if f.get("kind") == "dense":
                fill(f, "ff", dim_of(f"l{i}.mlp.up"))
            elif f.get("kind") == "moe":
                expert = dict(f["expert"]) if isinstance(f.get("expert"), Mapping) else {}
                router = dict(f["router"]) if isinstance(f.get("router"), Mapping) else {}
                fill(expert, "ff", dim_of(f"l{i}.mlp.e0.gate"))
                fill(router, "experts", dim_of(f"l{i}.mlp.router"))
                f["expert"], f["router"] = expert, router
            e["mlp"] = f
        new_layers.append(e)
    return out


def _heads(m: Mapping[str, Any], where: str) -> Tuple[int, int]:
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of kv_heads {kv}")
    return heads, kv


def _attention(m: Mapping[str, Any], mw: str, i: int, layers: List[SeredraLayer]) -> SeredraAttention:
    heads, kv = _heads(m, mw)
    conv = m.get("conv")
    qt = m.get("q_temp")
    if qt is not None:
        q = dict(_obj(m, "q_temp", mw))
        if isinstance(q.get("every"), float) and q["every"].is_integer():      # (64.0 is 64)
            q["every"] = int(q["every"])
        qt = (_num(q, "coef", mw + "q_temp."), _int(q, "every", mw + "q_temp."))
    mixer = SeredraAttention(heads=heads, kv_heads=kv, dim=_int(m, "dim", mw), vdim=_int(m, "vdim", mw),
                             scale=_num(m, "scale", mw), conv=0 if conv is None else _int(m, "conv", mw, least=0),
                             q_temp=qt, kv_from=None if m.get("kv_from") is None else _int(m, "kv_from", mw, least=0))
    if mixer.kv_from is not None:
        if mixer.kv_from >= i:
            raise ConfigError(f"config.json: {mw}kv_from {mixer.kv_from} must name an earlier layer")
        src = layers[mixer.kv_from].mixer
        if not isinstance(src, SeredraAttention) or src.kv_from is not None:
            raise ConfigError(f"config.json: {mw}kv_from names layer {mixer.kv_from}, which has no keys and values "
                              f"of this kind of its own")
        if (src.kv_heads, src.dim, src.vdim) != (mixer.kv_heads, mixer.dim, mixer.vdim):
            raise ConfigError(f"config.json: {mw}kv_heads, dim and vdim must equal those of layer {mixer.kv_from}")
    return mixer


def _parallel(m: Mapping[str, Any], mw: str) -> SeredraParallel:
    l, lw = dict(_obj(m, "left", mw)), mw + "left."
    if l.get("vdim") is None and l.get("dim") is not None:      # the values are the keys: one size for both
        l["vdim"] = l["dim"]
    heads, kv = _heads(l, lw)
    dims, base = _rot(l, lw)
    sc = l["rot"].get("scaling")
    if sc is not None:
        s, sw = _obj(l["rot"], "scaling", lw + "rot."), lw + "rot.scaling."
        sc = SeredraYarn(_num(s, "factor", sw), _num(s, "original", sw), _num(s, "fast", sw), _num(s, "slow", sw))
        if not (sc.factor > 0 and sc.original > 0 and sc.fast > 0 and sc.slow > 0):
            raise ConfigError(f"config.json: {sw}factor, original, fast and slow must be positive")
    cap = l.get("softcap")
    left = SeredraLeft(heads=heads, kv_heads=kv, dim=_int(l, "dim", lw), vdim=_int(l, "vdim", lw),
                       scale=_num(l, "scale", lw), softcap=0.0 if cap is None else _num(l, "softcap", lw),
                       rot_dims=dims, rot_base=base, scaling=sc)
    if left.vdim != left.dim:
        raise ConfigError(f"config.json: {lw}vdim {left.vdim} must equal dim {left.dim}: the values are the keys as projected")
    if dims > left.dim:
        raise ConfigError(f"config.json: {lw}rot.dims {dims} exceeds dim {left.dim}")
    if left.softcap < 0:
        raise ConfigError(f"config.json: {lw}softcap must not be negative")
    r, rw = _obj(m, "right", mw), mw + "right."
    right = SeredraRight(inner=_int(r, "inner", rw), state=_int(r, "state", rw), dt_rank=_int(r, "dt_rank", rw),
                         conv=_int(r, "conv", rw))
    return SeredraParallel(left, right, _num(m, "left_scale", mw), _num(m, "right_scale", mw))


def _retention(m: Mapping[str, Any], mw: str) -> SeredraRetention:
    heads = _int(m, "heads", mw)
    decay = m.get("decay")
    if (not isinstance(decay, list) or len(decay) != heads
            or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in decay)):
        raise ConfigError(f"config.json: {mw}decay must be a list of {heads} numbers, one a head")
    dims, base = _rot(m, mw)
    mixer = SeredraRetention(heads=heads, dim=_int(m, "dim", mw), vdim=_int(m, "vdim", mw),
                             decay=tuple(float(v) for v in decay), rot_dims=dims, rot_base=base)
    if dims > mixer.dim:
        raise ConfigError(f"config.json: {mw}rot.dims {dims} exceeds dim {mixer.dim}")
    return mixer


@dataclass(frozen=True)
class SeredraConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    layers: Tuple[SeredraLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "SeredraConfig":
        vocab, width = _int(d, "vocab", ""), _int(d, "width", "")
        eps = _num(_obj(d, "norm", ""), "eps", "norm.")
        raw = d.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[SeredraLayer] = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            kind = entry.get("type") if isinstance(entry, Mapping) else entry
            if kind not in TYPES:
                raise ConfigError(f"config.json: {where}type {kind!r} is not a mixer of this design (known: "
                                  + ", ".join(repr(t) for t in TYPES) + ")")
            m, mw = _obj(entry, "mixer", where), where + "mixer."
            mixer = (_attention(m, mw, i, layers) if kind == "attention" else _parallel(m, mw) if kind == "parallel"
                     else _retention(m, mw))
            mlp = entry.get("mlp")
            if mlp is not None:
                fw = where + "mlp."
                fk = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                if fk == "dense":
                    mlp = SeredraDense(_int(mlp, "ff", fw))
                elif fk == "moe":
                    r = _obj(mlp, "router", fw)
                    mlp = SeredraExperts(ff=_int(_obj(mlp, "expert", fw), "ff", fw + "expert."),
                                         experts=_int(r, "experts", fw + "router."), top=_int(r, "top", fw + "router."))
                    if mlp.top > mlp.experts:
                        raise ConfigError(f"config.json: {fw}router.top {mlp.top} exceeds the {mlp.experts} experts")
                else:
                    raise ConfigError(f"config.json: {fw}kind {fk!r} is not known (known: 'dense', 'moe')")
            layers.append(SeredraLayer(mixer, mlp))
        mp = d.get("max_positions")
        return cls(vocab=vocab, width=width, embedding_scale=_num(_obj(d, "embedding", ""), "scale", "embedding."),
                   eps=eps, layers=tuple(layers),
                   max_positions=DEFAULT_MAX_POSITIONS if mp is None else _int(d, "max_positions", ""))
