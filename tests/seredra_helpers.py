"""Small Seredra configurations that differ in every size and option, model folders with planted weights for them, and
the plain implementation's logits."""
from __future__ import annotations

import functools
import os
from typing import Dict, List, Sequence

import numpy as np
import torch

import plain_seredra as P
from helpers import tmp_root


def _att(heads, kv_heads, dim, vdim, scale, conv=None, q_temp=None, kv_from=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
    if conv is not None:
        m["conv"] = conv
    if q_temp is not None:
        m["q_temp"] = dict(coef=q_temp[0], every=q_temp[1])
    if kv_from is not None:
        m["kv_from"] = kv_from
    return dict(type="attention", mixer=m)


def _par(left, right, left_scale, right_scale):
    heads, kv_heads, dim, scale, rot, base, softcap, scaling = left
    l = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale, rot=dict(base=base, dims=rot))
    if softcap is not None:
        l["softcap"] = softcap
    if scaling is not None:
        l["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    inner, state, dt_rank, conv = right
    return dict(type="parallel", mixer=dict(left=l, right=dict(inner=inner, state=state, dt_rank=dt_rank, conv=conv),
                                            left_scale=left_scale, right_scale=right_scale))


def _ret(heads, dim, vdim, decay, rot, base):
    return dict(type="retention", mixer=dict(heads=heads, dim=dim, vdim=vdim, decay=list(decay),
                                             rot=dict(base=base, dims=rot)))


def _dense(ff):
    return dict(kind="dense", ff=ff)


def _moe(ff, experts, top):
    return dict(kind="moe", expert=dict(ff=ff), router=dict(experts=experts, top=top))


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


def _model(vocab, width, scale, eps, layers):
    return dict(architecture="Seredra", vocab=vocab, width=width, embedding=dict(scale=scale), norm=dict(eps=eps),
                layers=layers)


# A: odd sizes everywhere (nothing a matrix-core kernel takes): three retention heads of 10 / 6 with 6 rotated elements;
#    attention 4:2 with keys of 6 and values of 10, 2 taps, a temperature that steps every 3 positions; a side-by-side
#    mixer with 4 of 12 elements rotated under a frequency rule, 20 channels of 5 states and 4 taps; a borrower of the
#    attention's keys and values; 2 of 5 and 3 of 4 experts, a layer without feed-forward
TINY_SA = _model(83, 36, 1.7, 1e-5, [
    _layer(_ret(3, 10, 6, (0.9, 0.99, 0.5), 6, 300.0), _moe(20, 5, 2)),
    _layer(_att(4, 2, 6, 10, 0.4, conv=2, q_temp=(0.7, 3)), _dense(28)),
    _layer(_par((4, 2, 12, 0.3, 4, 50.0, 3.0, (3.0, 16, 8.0, 1.0)), (20, 5, 3, 4), 1.3, 0.6), None),
    _layer(_att(4, 2, 6, 10, 0.5, conv=3, q_temp=(0.2, 7), kv_from=1), _moe(12, 4, 3))])
# B: multiples of 16 and 32 everywhere (what the matrix-core kernels take); the side-by-side mixer first; 2 of 8 experts
TINY_SB = _model(256, 128, 4.0, 1e-6, [
    _layer(_par((8, 2, 64, 0.11, 32, 20000.0, 20.0, (4.0, 64, 16.0, 2.0)), (256, 16, 8, 4), 0.7, 0.9), _moe(64, 8, 2)),
    _layer(_att(8, 4, 32, 64, 0.17, conv=4, q_temp=(0.5, 16)), _dense(256)),
    _layer(_ret(4, 64, 64, (0.97, 0.99, 0.999, 0.9), 32, 10000.0), _dense(128)),
    _layer(_att(8, 4, 32, 64, 0.2, conv=2, kv_from=1), _moe(32, 6, 3)),
    _layer(_ret(2, 32, 128, (0.95, 0.995), 32, 500.0), None)])
# C: the values that make terms vanish or coincide: scale 1, one head, one kv head a head, every expert chosen, one
#    expert alone, no convolution and one of a single tap, no temperature, no soft cap, no frequency rule, nothing
#    rotated, a decay of 1, factors of 1, one state, a step size of rank 1, one tap in the scan
TINY_SC = _model(50, 32, 1.0, 1e-6, [
    _layer(_att(1, 1, 16, 16, 0.25), _moe(16, 3, 3)),
    _layer(_par((1, 1, 16, 0.25, 0, 10000.0, None, None), (8, 1, 1, 1), 1.0, 1.0), _moe(24, 1, 1)),
    _layer(_ret(1, 16, 16, (1.0,), 0, 10000.0), None),
    _layer(_att(3, 3, 8, 8, 0.3, conv=1, kv_from=None), _dense(8)),
    _layer(_par((2, 2, 8, 0.3, 8, 7.0, 2.0, None), (16, 3, 2, 2), 1.0, 0.5), _dense(16))])
# D: multiples of 8 that are no multiples of 16 or 32 (keys of 24 and 40, values of 40 and 24, 72 channels), 4 of 10
#    experts, two borrowers of one owner, whole heads rotated
TINY_SD = _model(300, 96, 9.0, 1e-6, [
    _layer(_att(6, 2, 24, 40, 0.2, conv=3, q_temp=(0.3, 5)), _moe(72, 10, 4)),
    _layer(_ret(3, 40, 24, (0.97, 0.9, 0.99), 40, 1000.0), _dense(200)),
    _layer(_att(6, 2, 24, 40, 0.15, conv=5, kv_from=0), None),
    _layer(_par((6, 3, 40, 0.15, 40, 5000.0, 10.0, (2.0, 32, 4.0, 0.5)), (72, 8, 6, 3), 0.9, 0.4), _dense(104)),
    _layer(_att(6, 2, 24, 40, 0.25, kv_from=0), _moe(24, 3, 1))])

CONFIGS = {"SA": (TINY_SA, 51), "SB": (TINY_SB, 52), "SC": (TINY_SC, 53), "SD": (TINY_SD, 54)}


def planted(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights of a size at which every mechanism shows in the logits: matrices N(0, 1/sqrt(fan-in)), those that make
    queries and keys larger (so that the softmax is not flat and one key more or less moves the logits), norm weights
    around 1, distance penalties and step sizes of order 1, routers that separate the experts."""
    from allpaca_amd.models import DecoderModel, describe_model
    _, _, spec = describe_model(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, ps in DecoderModel(spec).param_specs().items():
        shape = tuple(ps.shape)
        rnd = torch.randn(shape, generator=g)
        parts = name.split(".")
        last = parts[-1]
        if shape == ():
            t = 1.0 + 0.2 * rnd
        elif last in ("r1", "r2"):
            t = 0.2 + 0.5 * rnd.abs()
        elif last == "conv":
            t = rnd / shape[1] ** 0.5 + (torch.arange(shape[1]) == shape[1] - 1).float()
        elif last == "b":
            t = (rnd - 1.0) if parts[-2] == "dt" else 0.2 * rnd
        elif last == "A_log":
            t = 0.7 * rnd - 1.0
        elif len(shape) == 1:
            t = 1.0 + 0.2 * rnd
        elif name == "embed":
            t = rnd
        elif last == "router":
            t = 2.0 * rnd / shape[1] ** 0.5
        elif last in ("q", "k"):
            t = 2.0 * rnd / shape[1] ** 0.5
        elif last in ("gate", "up"):
            t = 1.5 * rnd / shape[1] ** 0.5
        else:
            t = rnd / shape[1] ** 0.5
        out[name] = t.to(torch.bfloat16).float()     # values that bfloat16 holds, so both runs load the same numbers
    return out


def write_folder(path: str, cfg: dict, seed: int, dtype: str = "float32") -> str:
    from allpaca_amd.weights import write_model_folder
    write_model_folder(path, cfg, seed, torch.float32 if dtype == "float32" else torch.bfloat16,
                       overrides=planted(cfg, seed))
    return path


@functools.lru_cache(maxsize=None)
def model_folder(name: str, dtype: str = "float32") -> str:
    cfg, seed = CONFIGS[name]
    return write_folder(os.path.join(tmp_root(), f"seredra_{name}_{dtype}"), cfg, seed, dtype)


@functools.lru_cache(maxsize=None)
def oracle(folder: str):
    return P.read_model_folder(folder)


_LOGITS: Dict = {}


def oracle_logits(folder: str, tokens: Sequence[int]) -> np.ndarray:
    key = (folder, tuple(tokens))
    if key not in _LOGITS:
        _LOGITS[key] = P.forward(*oracle(folder), list(tokens))
    return _LOGITS[key]


def oracle_noise(folder: str, tokens: Sequence[int]):
    """What rounding every stored activation to bfloat16 costs the plain implementation itself (exact arithmetic
    otherwise), relative to the size of the logits: (root mean square over all rows, the row that 9 in 10 stay under)."""
    key = (folder, tuple(tokens), "bf16")
    if key not in _LOGITS:
        want = oracle_logits(folder, tokens)
        err = P.forward(*oracle(folder), list(tokens), rnd=P.to_bf16) - want
        size = float(np.sqrt(np.mean(want ** 2)))
        _LOGITS[key] = (float(np.sqrt(np.mean(err ** 2))) / size,
                        float(np.quantile(np.sqrt(np.mean(err ** 2, axis=1)), 0.9)) / size)
    return _LOGITS[key]


def tokens_for(name: str, n: int, seed: int) -> List[int]:
    return np.random.default_rng(seed).integers(0, CONFIGS[name][0]["vocab"], size=n).tolist()
