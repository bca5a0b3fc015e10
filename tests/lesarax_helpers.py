"""Small Lesarax configurations that differ in every size and option, model folders with random weights for them, and
the plain implementation's logits."""
from __future__ import annotations

import functools
import os
from typing import Dict, List, Sequence

import numpy as np
import torch

import plain_lesarax as P
from helpers import tmp_root


def _att(heads, kv_heads, dim, scale, rot, base, window=None):
    m = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale, rot=dict(base=base, dims=rot))
    if window is not None:
        m["mask"] = dict(size=window)
    return dict(type="attention", mixer=m)


def _lat(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, window=None):
    m = dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale,
             rot=dict(base=base, dims=rot_dim))
    if window is not None:
        m["mask"] = dict(size=window)
    return dict(type="latent_attention", mixer=m)


def _moe(ff, limit, experts, top):
    return dict(kind="moe", expert=dict(ff=ff, limit=limit), router=dict(experts=experts, top=top))


def _layer(mixer, mlp):
    return dict(mixer, mlp=mlp)


# A: odd sizes everywhere (nothing a matrix-core kernel takes): three latent heads with 10 + 6 key elements and
#    values of 14, a window of 5; grouped heads 4:2 of 12 with 4 rotated elements; 3 of 5 experts, a layer without
#    feed-forward; the loop starts at the first layer and runs three times
TINY_LA = dict(
    architecture="Lesarax", vocab=83, width=36, residual_mult=0.7, norm=dict(eps=1e-5),
    loop=dict(start=0, stop=2, times=3),
    layers=[_layer(_lat(3, 10, 6, 14, 20, 12, 0.3, 300.0, window=5), _moe(20, 0.8, 5, 3)),
            _layer(_att(4, 2, 12, 0.35, 4, 50.0), None),
            _layer(_lat(2, 6, 2, 10, 9, 7, 0.4, 10000.0, window=11), _moe(28, 1.5, 4, 1))])
# B: multiples of 16 and 32 everywhere (what the matrix-core kernels take): latent heads with 32 + 32 and 16 + 16
#    key elements, windows of 24 and of 40, grouped heads 8:2 of 64 (32 rotated) and 4:4 of 32 (all rotated), 2 of 8 and
#    3 of 6 experts; the loop holds the two middle layers, twice
TINY_LB = dict(
    architecture="Lesarax", vocab=256, width=128, residual_mult=0.4, norm=dict(eps=1e-6),
    loop=dict(start=1, stop=3, times=2),
    layers=[_layer(_lat(4, 32, 32, 64, 64, 32, 0.12, 10000.0, window=24), _moe(64, 1.0, 8, 2)),
            _layer(_att(8, 2, 64, 0.11, 32, 20000.0), _moe(32, 2.0, 6, 3)),
            _layer(_lat(8, 16, 16, 32, 96, 64, 0.17, 500.0, window=40), None),
            _layer(_att(4, 4, 32, 0.2, 32, 1000.0), _moe(96, 0.5, 4, 2))])
# C: the values that make terms vanish or coincide: factor 1, one head, one kv head a head, every expert chosen, one
#    expert alone, a window of 1 (a row sees itself only) and one no sequence of the tests reaches, nothing rotated in
#    an attention, a loop that runs once
TINY_LC = dict(
    architecture="Lesarax", vocab=50, width=32, residual_mult=1.0, norm=dict(eps=1e-6),
    loop=dict(start=1, stop=2, times=1),
    layers=[_layer(_lat(1, 16, 16, 16, 16, 16, 0.2, 10000.0, window=1), _moe(16, 3.0, 3, 3)),
            _layer(_att(1, 1, 16, 0.25, 0, 10000.0), _moe(24, 1.0, 1, 1)),
            _layer(_lat(2, 16, 8, 8, 24, 8, 0.2, 100.0, window=4096), None),
            _layer(_att(3, 3, 8, 0.3, 8, 7.0), _moe(8, 0.25, 2, 1))])
# D: no loop at all, a latent attention without a window, attention first
TINY_LD = dict(
    architecture="Lesarax", vocab=70, width=48, residual_mult=1.5, norm=dict(eps=1e-5),
    layers=[_layer(_att(6, 3, 16, 0.25, 8, 100.0), _moe(40, 1.0, 3, 2)),
            _layer(_lat(3, 8, 8, 24, 40, 16, 0.25, 10000.0), _moe(16, 1.0, 7, 2))])
# E: the loop is the whole model, four times; the window is a multiple of the page sizes the tests use
TINY_LE = dict(
    architecture="Lesarax", vocab=64, width=64, residual_mult=0.25, norm=dict(eps=1e-6),
    loop=dict(start=0, stop=2, times=4),
    layers=[_layer(_lat(4, 16, 16, 16, 32, 48, 0.18, 10000.0, window=16), _moe(48, 1.0, 3, 1)),
            _layer(_att(2, 1, 32, 0.18, 16, 10000.0), _moe(32, 1.0, 2, 2))])
# F: a width, heads and latents that are multiples of nothing, one layer alone in the loop, a window of 2, and a window
#    on the grouped attention as well
TINY_LF = dict(
    architecture="Lesarax", vocab=37, width=50, residual_mult=0.9, norm=dict(eps=1e-6),
    loop=dict(start=1, stop=2, times=3),
    layers=[_layer(_att(5, 1, 6, 0.4, 6, 31.0, window=7), _moe(7, 0.6, 3, 2)),
            _layer(_lat(2, 5, 2, 3, 7, 5, 0.45, 13.0, window=2), _moe(9, 1.1, 2, 1))])
# G: multiples of 8 that are no multiples of 16 or 32 (keys of 80 and 48, values of 40, latents of 72 and 56, experts
#    72 wide, a window of 50 that is no multiple of a page), 4 of 10 experts
TINY_LG = dict(
    architecture="Lesarax", vocab=300, width=192, residual_mult=0.35, norm=dict(eps=1e-6),
    loop=dict(start=0, stop=2, times=3),
    layers=[_layer(_lat(6, 48, 32, 40, 72, 56, 0.11, 10000.0, window=50), _moe(72, 1.0, 10, 4)),
            _layer(_att(8, 4, 48, 0.14, 32, 20000.0), _moe(72, 1.0, 10, 4)),
            _layer(_lat(3, 24, 8, 24, 40, 24, 0.17, 10000.0, window=23), None)])

CONFIGS = {"LA": (TINY_LA, 31), "LB": (TINY_LB, 32), "LC": (TINY_LC, 33), "LD": (TINY_LD, 34), "LE": (TINY_LE, 35),
           "LF": (TINY_LF, 36), "LG": (TINY_LG, 37)}


def planted(cfg: dict, seed: int) -> Dict[str, torch.Tensor]:
    """Weights of a size at which every mechanism shows in the logits: matrices N(0, 1/sqrt(fan-in)), those that make
    queries and keys larger (so that the softmax is not flat and one key more or less moves the logits), norm weights
    around 1, sinks of order 1, routers that separate the experts, experts large enough for the clamps to act."""
    from allpaca_amd.models import DecoderModel, describe_model
    _, _, spec = describe_model(cfg)
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, ps in DecoderModel(spec).param_specs().items():
        shape = tuple(ps.shape)
        rnd = torch.randn(shape, generator=g)
        last = name.split(".")[-1]
        if last == "sink":
            t = rnd
        elif len(shape) == 1:
            t = 1.0 + 0.2 * rnd
        elif name == "embed":
            t = rnd
        elif last == "router":
            t = 2.0 * rnd / shape[1] ** 0.5
        elif last in ("q", "k", "uq", "uk", "dkv"):
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
    return write_folder(os.path.join(tmp_root(), f"{name}_{dtype}"), cfg, seed, dtype)


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
