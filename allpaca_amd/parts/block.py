"""Arrangements: how the parts of one layer are wired on the residual stream.
The residual stream x is float32 [T, D]; parts read a normalised copy in the
run's element type and add their output into x in 32-bit."""
from __future__ import annotations

from typing import Dict, Mapping

import torch

from .base import ARRANGEMENTS, CONNECTIONS, FEED_FORWARDS, MIXERS, NORMS, NormEmit, NormedInput, Part, build_part
from .spec import BlockSpec


class Block:
    """The built parts of one layer and the function that runs them."""

    def __init__(self, spec: BlockSpec):
        self.spec = spec
        arrangement = ARRANGEMENTS.get(spec.arrangement)
        self.parts: Dict[str, Part] = {}
        for role, pspec in spec.parts.items():
            self.parts[role] = build_part(arrangement.registries[role], pspec)
        self.arrangement = arrangement
        self.chains_norms = bool(getattr(arrangement, "chains_norms", False))

    def run(self, x: torch.Tensor, step, cache, pre=None, next_norm=None):
        """Runs the layer on the residual stream x.  `pre`: what the layer before left for this layer's first norm
        (a filled `NormEmit`) or None; `next_norm`: the norm that reads x after this layer.  Returns what this
        layer left for `next_norm`, or None.  Only arrangements with `chains_norms` take part in that."""
        if self.chains_norms:
            return self.arrangement.run(self.parts, x, step, cache, pre=pre, next_norm=next_norm)
        self.arrangement.run(self.parts, x, step, cache)
        return None

    def first_norm(self):
        """The norm that reads the residual stream first in this layer, if the layer can use what the product
        before it leaves for that norm."""
        return self.arrangement.first_norm(self.parts) if self.chains_norms else None

    @property
    def mixer(self):
        return self.parts["mixer"]

    def cache_needs(self, borrows: bool = False) -> Dict[str, object]:
        """role -> what that part needs of the cache manager, for every part of the layer that keeps something per
        request (`cache_need()` answering other than None): attention heads beside recurrent heads are two roles with
        a need each.  What a part keeps for itself alone (`state_need()`) stands under "<role>.state".  `borrows`: the
        layer runs against another plan entry's cache, and only what its parts keep for themselves is asked for."""
        out = {}
        for role, part in self.parts.items():
            for name, key in (("cache_need", role), ("state_need", role + ".state")):
                ask = getattr(part, name, None)
                need = ask() if callable(ask) and not (borrows and name == "cache_need") else None
                if isinstance(need, dict):
                    # a part made of several (mixers side by side): its members' needs stand under "<role>.<member>"
                    for member, n in need.items():
                        if n is not None:
                            out[f"{role}.{member}" + (".state" if name == "state_need" else "")] = n
                elif need is not None:
                    out[key] = need
        return out

    def native_desc(self):
        describe = getattr(self.arrangement, "native_desc", None)
        return describe(self.parts) if describe is not None else None

    def param_specs(self):
        out = {}
        for role, part in self.parts.items():
            prefix = self.spec.weight_prefix + self.spec.parts[role].weight_prefix
            for name, ps in part.param_specs().items():
                out[prefix + name] = ps
        return out

    def bind(self, tensors: Mapping[str, torch.Tensor], rt) -> None:
        for role, part in self.parts.items():
            prefix = self.spec.weight_prefix + self.spec.parts[role].weight_prefix
            local = {name: tensors[prefix + name] for name in part.param_specs() if prefix + name in tensors}
            part.bind(local, rt)


class NormedLeft:
    """What a pre-norm layer with a scaled sum leaves for the next one: the next layer's first input, already
    normalised (the sum of this layer's last output and that norm are one pass over the row)."""

    def __init__(self, norm, h: torch.Tensor):
        self.norm, self.h = norm, h


class ScaledFirst:
    """What such a layer shows the layer before it: the norm of its first read."""

    def __init__(self, norm):
        self.norm = norm

    def rms_params(self):       # to an arrangement that folds norms into products this is no norm it can fold
        return None


@ARRANGEMENTS.register("pre_norm")
class PreNorm:
    """x += mixer(norm(x)); x += ffn(norm(x))  (crates/allpaca-core/src/model.rs:8447-8455, 8667-8696).
    With the role "scale" (a `scaled` connection) the sums are x += mult * mixer(norm(x)) and x += mult * ffn(norm(x)),
    made in 32-bit by a kernel that also normalises the new x for whoever reads it next; such a layer may have no
    feed-forward."""
    registries = {"mixer_norm": NORMS, "mixer": MIXERS, "ffn_norm": NORMS, "ffn": FEED_FORWARDS, "scale": CONNECTIONS}
    chains_norms = True

    @staticmethod
    def first_norm(parts):
        if "scale" in parts:
            return ScaledFirst(parts["mixer_norm"]) if parts["mixer_norm"].rms_params() is not None else None
        return parts["mixer_norm"] if parts["mixer"].takes_normed_input else None

    @staticmethod
    def run_scaled(parts, x: torch.Tensor, step, cache, pre, next_norm):
        mixer, ffn, link = parts["mixer"], parts.get("ffn"), parts["scale"]
        rt = mixer.rt

        def buffer():
            return torch.empty(x.shape, dtype=rt.dtype, device=x.device)

        def fusable(norm):
            return norm is not None and norm.rms_params() is not None

        if isinstance(pre, NormedLeft) and pre.norm is parts["mixer_norm"]:
            h = pre.h
        else:
            h = buffer()
            parts["mixer_norm"].forward(x, h)
        y = mixer.forward(h, step, cache)
        wanted = next_norm.norm if isinstance(next_norm, ScaledFirst) else None
        if ffn is not None:
            norm2 = parts["ffn_norm"]
            h = buffer()
            if fusable(norm2):
                link.add(x, y, norm2, h)
            else:
                link.add(x, y)
                norm2.forward(x, h)
            y = ffn.forward(h, step)
        if fusable(wanted):
            h = buffer()
            link.add(x, y, wanted, h)
            return NormedLeft(wanted, h)
        link.add(x, y)
        return None

    @staticmethod
    def native_desc(parts):
        """The layer for the compiled executor, if it knows all four parts: a dict role -> the part's own description."""
        if "scale" in parts or "ffn" not in parts:
            return None
        out = {role: parts[role].native_desc() for role in ("mixer_norm", "mixer", "ffn_norm", "ffn")}
        kinds = {"mixer_norm": "rmsnorm", "mixer": "attention", "ffn_norm": "rmsnorm", "ffn": "swiglu"}
        if any(d is None or d.get("kind") != kinds[role] for role, d in out.items()):
            return None
        return {"kind": "pre_norm", **out}

    @staticmethod
    def run(parts, x: torch.Tensor, step, cache, pre=None, next_norm=None):
        if "scale" in parts:
            return PreNorm.run_scaled(parts, x, step, cache, pre, next_norm)
        mixer, ffn = parts["mixer"], parts["ffn"]
        if isinstance(cache, dict):      # a layer with several parts that keep a cache: each gets its own
            cache = cache.get("mixer")
        rt = mixer.rt
        h = NormedInput(x, parts["mixer_norm"], rt.dtype, pre)
        emit = NormEmit.of(parts["ffn_norm"]) if mixer.emits_next_norm and ffn.takes_normed_input else None
        if mixer.emits_next_norm:
            mixer.forward_add(h if mixer.takes_normed_input else h.tensor(), step, cache, x, emit=emit)
        else:
            mixer.forward_add(h if mixer.takes_normed_input else h.tensor(), step, cache, x)
        h = NormedInput(x, parts["ffn_norm"], rt.dtype, emit)
        emit = NormEmit.of(next_norm) if ffn.emits_next_norm else None
        if ffn.emits_next_norm:
            ffn.forward_add(h if ffn.takes_normed_input else h.tensor(), step, x, emit=emit)
        else:
            ffn.forward_add(h if ffn.takes_normed_input else h.tensor(), step, x)
        return emit if emit is not None and emit.filled else None


class StreamsLeft:
    """What a layer over residual streams leaves for the next one: the next layer's first input, already read from
    the streams and normalised (the write of this layer's last output and that read are one pass over the row)."""

    def __init__(self, connection, norm, h: torch.Tensor):
        self.connection, self.norm, self.h = connection, norm, h


class StreamsFirst:
    """What a layer over residual streams shows the layer before it: the connection and the norm of its first read."""

    def __init__(self, connection, norm):
        self.connection, self.norm = connection, norm

    def rms_params(self):       # to an arrangement that folds norms into products this is no norm it can fold
        return None


@ARRANGEMENTS.register("hyper_pre_norm")
class HyperPreNorm:
    """Over S residual streams x_1 .. x_S of a row (x is [rows, S * hidden] float32):
       u = sum_a in1[a] x_a;  y = mixer(norm1(u));  x_b <- sum_a mix1[a][b] x_a + out1[b] y
    and the same with the feed-forward and the second connection, if the layer has one."""
    registries = {"mixer_norm": NORMS, "mixer": MIXERS, "mixer_link": CONNECTIONS,
                  "ffn_norm": NORMS, "ffn": FEED_FORWARDS, "ffn_link": CONNECTIONS}
    chains_norms = True

    @staticmethod
    def first_norm(parts):
        return StreamsFirst(parts["mixer_link"], parts["mixer_norm"])

    @staticmethod
    def run(parts, x: torch.Tensor, step, cache, pre=None, next_norm=None):
        mixer, link1, norm1 = parts["mixer"], parts["mixer_link"], parts["mixer_norm"]
        ffn = parts.get("ffn")
        rt = mixer.rt
        T, D = x.shape[0], x.shape[1] // link1.S

        def buffer():
            return torch.empty((T, D), dtype=rt.dtype, device=x.device)

        if isinstance(pre, StreamsLeft) and pre.connection is link1 and pre.norm is norm1:
            h = pre.h
        else:
            h = buffer()
            link1.read(x, norm1, h)
        y = mixer.forward(h, step, cache)
        last = link1
        if ffn is not None:
            link2, norm2 = parts["ffn_link"], parts["ffn_norm"]
            h = buffer()
            link1.write(x, y, then=link2, norm=norm2, h=h)
            y = ffn.forward(h, step)
            last = link2
        if isinstance(next_norm, StreamsFirst) and next_norm.connection.S == last.S:
            h = buffer()
            last.write(x, y, then=next_norm.connection, norm=next_norm.norm, h=h)
            return StreamsLeft(next_norm.connection, next_norm.norm, h)
        last.write(x, y)
        return None


class RowsLeft:
    """What a layer whose sublayers read the residual itself leaves for the next one: the residual in the run's
    element type (the kernel that adds the last sublayer's output writes it on the way)."""

    def __init__(self, h: torch.Tensor):
        self.h = h


class ReadsResidual:
    """What such a layer shows the layer before it: its first sublayer reads the residual as it is."""

    def rms_params(self):       # to an arrangement that folds norms into products this is no norm it can fold
        return None


@ARRANGEMENTS.register("sublayer_norm")
class SublayerNorm:
    """The norm stands on the sublayer's output only, and the sum is scaled:
       x <- x + mult * norm1(mixer(x));  x <- x + mult * norm2(ffn(x))      (a layer may have no feed-forward)
    The sublayers read x itself (in the run's element type).  Norm and sum are one kernel in 32-bit, which also
    leaves the new x in the run's element type for the next sublayer."""
    registries = {"mixer": MIXERS, "mixer_norm": NORMS, "ffn": FEED_FORWARDS, "ffn_norm": NORMS, "scale": CONNECTIONS}
    chains_norms = True

    @staticmethod
    def first_norm(parts):
        return ReadsResidual()

    @staticmethod
    def run(parts, x: torch.Tensor, step, cache, pre=None, next_norm=None):
        from ..kernels import ops
        mixer, ffn = parts["mixer"], parts.get("ffn")
        rt = mixer.rt
        mult = parts["scale"].mult
        narrow = rt.dtype != torch.float32       # a 32-bit run reads x as it is: no copy

        def copy():
            return torch.empty(x.shape, dtype=rt.dtype, device=x.device) if narrow else None

        if not narrow:
            h = x
        elif isinstance(pre, RowsLeft):
            h = pre.h
        else:
            h = copy()
            ops.cast(x, h)
        y = mixer.forward(h, step, cache)
        w, eps = parts["mixer_norm"].rms_params()
        last = ffn is None
        wants = isinstance(next_norm, ReadsResidual)
        h = copy() if (not last or wants) else None
        ops.rmsnorm_add(y, w, eps, mult, x, h)
        if not last:
            y = ffn.forward(h if narrow else x, step)
            w, eps = parts["ffn_norm"].rms_params()
            h = copy() if wants else None
            ops.rmsnorm_add(y, w, eps, mult, x, h)
        return RowsLeft(h) if (wants and narrow) else None
