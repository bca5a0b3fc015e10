"""Typed configuration of the Lesarax decoder, read from config.json.

Keys: `vocab`, `width`, `residual_mult`, `norm.eps`, `loop` ({"start", "stop", "times"}: layers start .. stop-1 run
`times` times in a row with the same weights; absent or null: every layer once) and `layers`, a list of
{"type", "mixer", "mlp"}.
  type "attention": `heads`, `kv_heads`, `dim` (query and key size of a head), `vdim` (equal to `dim`: the values are
      the keys as projected), `scale`, `rot` ({"base", "dims"}: the rotation on a head's first `dims` elements), `mask`
      as below (absent: every earlier position).
  type "latent_attention": `heads`, `dim` (unrotated elements of a head's query and key), `rot_dim` (rotated ones),
      `vdim`, `q_rank`, `kv_rank` (sizes of the latents), `scale`, `rot` ({"base", "dims"}, dims = rot_dim), `mask`
      ({"size": n}: a row sees itself and the n - 1 positions before it; absent: every earlier position).
  `mlp`: null or {"kind": "moe", "expert": {"ff", "limit"}, "router": {"experts", "top"}}.
Every size and constant comes from here; nothing has a silent default that fixes a tensor's shape."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, List, Mapping, Optional, Tuple, Union

from .llama import ConfigError
from .risizen import _int, _num

DEFAULT_MAX_POSITIONS = 1 << 17     # the design names no limit: what the rotation tables are made for at most


@dataclass(frozen=True)
class LesaraxAttention:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float
    window: Optional[int] = None


@dataclass(frozen=True)
class LesaraxLatent:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    rot_base: float
    window: Optional[int] = None


@dataclass(frozen=True)
class LesaraxExperts:
    ff: int
    limit: float
    experts: int
    top: int


@dataclass(frozen=True)
class LesaraxLayer:
    mixer: Union[LesaraxAttention, LesaraxLatent]
    mlp: Optional[LesaraxExperts]


@dataclass(frozen=True)
class LesaraxLoop:
    start: int
    stop: int
    times: int


def _obj(d: Mapping[str, Any], key: str, where: str) -> Mapping[str, Any]:
    v = d.get(key) if isinstance(d, Mapping) else None
    if not isinstance(v, Mapping):
        raise ConfigError(f"config.json: {where}{key!r} must be an object")
    return v


def _rot(m: Mapping[str, Any], where: str) -> Tuple[int, float]:
    r = _obj(m, "rot", where)
    dims = _int(r, "dims", where + "rot.", least=0)
    if dims % 2:
        raise ConfigError(f"config.json: {where}rot.dims {dims} must be even")
    base = _num(r, "base", where + "rot.")
    if not base > 0:
        raise ConfigError(f"config.json: {where}rot.base must be positive")
    return dims, base


def sizes_from_tensors(d: Mapping[str, Any], shapes: Mapping[str, Tuple[int, ...]]) -> Mapping[str, Any]:
    """config.json with the sizes it leaves out filled in from the shapes of the stored tensors (`embed`,
    `l<i>.mix.*`, `l<i>.mlp.*`).  A size the file names is left as it is: a disagreement shows when the weights load."""
    def rows(name: str) -> Optional[int]:
        shape = shapes.get(name)
        return int(shape[0]) if shape else None

    def fill(m: dict, key: str, value) -> None:
        if key not in m and value is not None:
            m[key] = value

    out = dict(d)
    if "embed" in shapes and len(shapes["embed"]) == 2:
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
        p = f"l{i}.mix."
        m = dict(entry["mixer"])
        fill(m, "heads", rows(p + "sink"))
        H = m.get("heads")
        if entry.get("type") == "attention" and isinstance(H, int) and H > 0:
            q, k = rows(p + "q"), rows(p + "k")
            fill(m, "dim", q // H if q else None)
            dim = m.get("dim")
            fill(m, "kv_heads", k // dim if k and isinstance(dim, int) and dim > 0 else None)
            fill(m, "vdim", dim)
        elif entry.get("type") == "latent_attention" and isinstance(H, int) and H > 0:
            fill(m, "q_rank", rows(p + "dq"))
            fill(m, "kv_rank", rows(p + "dkv.norm"))
            dkv, uk, uv = rows(p + "dkv"), rows(p + "uk"), rows(p + "uv")
            if dkv and isinstance(m.get("kv_rank"), int):
                fill(m, "rot_dim", dkv - m["kv_rank"])
            fill(m, "dim", uk // H if uk else None)
            fill(m, "vdim", uv // H if uv else None)
        e = dict(entry, mixer=m)
        f = entry.get("mlp")
        if isinstance(f, Mapping):
            f = dict(f)
            expert = dict(f["expert"]) if isinstance(f.get("expert"), Mapping) else {}
            router = dict(f["router"]) if isinstance(f.get("router"), Mapping) else {}
            fill(expert, "ff", rows(f"l{i}.mlp.e0.gate"))
            fill(router, "experts", rows(f"l{i}.mlp.router"))
            f["expert"], f["router"] = expert, router
            e["mlp"] = f
        new_layers.append(e)
    return out


@dataclass(frozen=True)
class LesaraxConfig:
    vocab: int
    width: int
    residual_mult: float
    eps: float
    layers: Tuple[LesaraxLayer, ...]
    loop: Optional[LesaraxLoop] = None
    max_positions: int = DEFAULT_MAX_POSITIONS

    def order(self) -> List[Tuple[int, bool]]:
        """[(layer, a pass of the loop starts here)] in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        a, b, times = self.loop.start, self.loop.stop, self.loop.times
        out = [(i, False) for i in range(a)]
        for _ in range(times):
            out += [(i, i == a) for i in range(a, b)]
        return out + [(i, False) for i in range(b, n)]

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "LesaraxConfig":
        vocab, width = _int(d, "vocab", ""), _int(d, "width", "")
        eps = _num(_obj(d, "norm", ""), "eps", "norm.")
        raw = d.get("layers")
        if not isinstance(raw, list) or not raw:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        layers: List[LesaraxLayer] = []
        for i, entry in enumerate(raw):
            where = f"layers[{i}]."
            kind = entry.get("type") if isinstance(entry, Mapping) else entry
            if kind not in ("attention", "latent_attention"):
                raise ConfigError(f"config.json: {where}type {kind!r} is not a mixer of this design "
                                  f"(known: 'attention', 'latent_attention')")
            m, mw = _obj(entry, "mixer", where), where + "mixer."
            dims, base = _rot(m, mw)
            mask = m.get("mask")
            window = None if mask is None else _int(_obj(m, "mask", mw), "size", mw + "mask.")
            if kind == "attention":
                mixer = LesaraxAttention(heads=_int(m, "heads", mw), kv_heads=_int(m, "kv_heads", mw),
                                         dim=_int(m, "dim", mw), vdim=_int(m, "vdim", mw), scale=_num(m, "scale", mw),
                                         rot_dims=dims, rot_base=base, window=window)
                if mixer.heads % mixer.kv_heads:
                    raise ConfigError(f"config.json: {mw}heads {mixer.heads} is no multiple of kv_heads {mixer.kv_heads}")
                if mixer.vdim != mixer.dim:
                    raise ConfigError(f"config.json: {mw}vdim {mixer.vdim} must equal dim {mixer.dim}: the values "
                                      f"are the keys as projected")
                if dims > mixer.dim:
                    raise ConfigError(f"config.json: {mw}rot.dims {dims} exceeds dim {mixer.dim}")
            else:
                mixer = LesaraxLatent(heads=_int(m, "heads", mw), dim=_int(m, "dim", mw),
                                      rot_dim=_int(m, "rot_dim", mw, least=0), vdim=_int(m, "vdim", mw),
                                      q_rank=_int(m, "q_rank", mw), kv_rank=_int(m, "kv_rank", mw),
                                      scale=_num(m, "scale", mw), rot_base=base, window=window)
                if dims != mixer.rot_dim:
                    raise ConfigError(f"config.json: {mw}rot.dims {dims} must equal rot_dim {mixer.rot_dim}")
            mlp = entry.get("mlp")
            if mlp is not None:
                fw = where + "mlp."
                fk = mlp.get("kind") if isinstance(mlp, Mapping) else mlp
                if fk != "moe":
                    raise ConfigError(f"config.json: {fw}kind {fk!r} is not known (known: 'moe')")
                e, r = _obj(mlp, "expert", fw), _obj(mlp, "router", fw)
                mlp = LesaraxExperts(ff=_int(e, "ff", fw + "expert."), limit=_num(e, "limit", fw + "expert."),
                                     experts=_int(r, "experts", fw + "router."), top=_int(r, "top", fw + "router."))
                if mlp.top > mlp.experts:
                    raise ConfigError(f"config.json: {fw}router.top {mlp.top} exceeds the {mlp.experts} experts")
                if not mlp.limit > 0:
                    raise ConfigError(f"config.json: {fw}expert.limit must be positive")
            layers.append(LesaraxLayer(mixer, mlp))
        loop = d.get("loop")
        if loop is not None:
            lp = _obj(d, "loop", "")
            loop = LesaraxLoop(_int(lp, "start", "loop.", least=0), _int(lp, "stop", "loop.", least=0),
                               _int(lp, "times", "loop.", least=0))
            if not (loop.start <= loop.stop <= len(layers)):
                raise ConfigError(f"config.json: loop.start {loop.start} .. loop.stop {loop.stop} must lie within the "
                                  f"{len(layers)} layers")
        mp = d.get("max_positions")
        return cls(vocab=vocab, width=width, residual_mult=_num(d, "residual_mult", ""), eps=eps, layers=tuple(layers),
                   loop=loop, max_positions=DEFAULT_MAX_POSITIONS if mp is None else _int(d, "max_positions", ""))
