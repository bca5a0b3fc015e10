"""The plain implementation of the Seredra decoder (tests/plain_seredra.py) pinned by hand, its two forms held against
each other, and the parts of the engine that need no GPU: configuration, tensor names, sizes from shapes, cache needs."""
import copy
import math

import numpy as np
import pytest

import plain_seredra as P
from seredra_helpers import CONFIGS, _att, _dense, _layer, _model, _moe, _par, _ret, planted


def weights(cfg, seed):
    return {k: v.double().numpy() for k, v in planted(cfg, seed).items()}


def test_short_convolution_by_hand():
    u = np.array([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0]])
    w = np.array([[0.5, 1.0, 2.0], [0.0, 0.0, 1.0]])
    y = P.short_conv(u, w)
    assert np.allclose(y[:, 0], [2.0, 1.0 + 4.0, 0.5 + 2.0 + 6.0]) and np.allclose(y[:, 1], u[:, 1])
    y2 = P.short_conv(u[1:], w, before=np.array([[0.0, 0.0], [1.0, 10.0]]))
    assert np.allclose(y2, y[1:])


def test_rotation_by_hand_and_the_frequency_rule():
    rot = dict(base=100.0, dims=4)
    v = np.array([[[1.0, 2.0, 3.0, 4.0, 5.0]]])
    out = P.rotate_front(v, [3], rot)[0, 0]
    a0, a1 = 3.0, 3.0 * 100.0 ** -0.5
    assert np.allclose(out, [math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
                             3 * math.cos(a0) + math.sin(a0), 4 * math.cos(a1) + 2 * math.sin(a1), 5.0])
    # the rule: dimensions faster than `fast` turns in the original length keep their frequency, slower than `slow` are
    # divided by the factor, and the magnitude grows with the logarithm of the factor
    rot = dict(base=10000.0, dims=32, scaling=dict(factor=4.0, original=64, fast=16.0, slow=2.0))
    f, mag = P.frequencies(rot)
    plain = 10000.0 ** (-2.0 * np.arange(16) / 32)
    assert np.isclose(mag, 0.1 * math.log(4.0) + 1.0)
    assert np.allclose(f[0], plain[0]) and np.allclose(f[-1], plain[-1] / 4.0)
    assert (np.diff(f / plain) <= 1e-12).all() and 0.25 < (f / plain)[1] < 1.0 and 0.25 < (f / plain)[2] < 1.0


def test_distance_penalty_soft_cap_and_temperature_by_hand():
    q = np.array([[[2.0]], [[2.0]], [[2.0]]])
    k = np.array([[[1.0]], [[1.0]], [[1.0]]])
    v = np.array([[[1.0]], [[2.0]], [[4.0]]])
    o = P.softmax_attention(q, k, v, 0.5, r1=np.array([1.0]), r2=np.array([1.0]))
    # scores 1 - ln(1 + d): weights proportional to e / (1 + d)
    w = np.array([1 / 3, 1 / 2, 1.0])
    assert np.allclose(o[2, 0, 0], (w * np.array([1.0, 2.0, 4.0])).sum() / w.sum())
    o = P.softmax_attention(q * 100, k, v, 0.5, softcap=1.0)
    assert np.allclose(o[2, 0, 0], 7.0 / 3.0)                       # every score is capped at 1: equal weights
    t = P.query_temperature([0, 1, 2, 5], 0.5, 3)
    assert np.allclose(t, [1.0, 1.0, 1.0 + 0.5 * math.log(2.0), 1.0 + 0.5 * math.log(3.0)])


def test_retention_and_scan_by_hand():
    q = np.ones((2, 1, 1)); k = np.array([[[1.0]], [[2.0]]]); v = np.array([[[3.0]], [[5.0]]])
    o, S = P.retention(q, k, v, [0.5])
    assert np.allclose(o[:, 0, 0], [3.0, 0.5 * 3.0 + 10.0]) and np.allclose(S, [[[11.5]]])
    x = np.array([[1.0], [2.0]]); dt = np.array([[0.5], [1.0]])
    A = np.array([[-1.0]]); B = np.array([[1.0], [1.0]]); C = np.array([[2.0], [3.0]])
    y, S = P.selective_scan(x, dt, A, B, C, np.array([10.0]))
    s0 = 0.5
    s1 = math.exp(-1.0) * s0 + 2.0
    assert np.allclose(y[:, 0], [2.0 * s0 + 10.0, 3.0 * s1 + 20.0]) and np.allclose(S, [[s1]])


def test_experts_take_the_weighted_input():
    ids, w = P.route(np.array([0.0, 2.0, 2.0, -1.0]), 2)
    assert list(ids) == [1, 2] and np.allclose(w, [P.sigmoid(2.0)] * 2)
    rng = np.random.default_rng(0)
    W = {"m.router": np.array([[5.0, 0.0], [-5.0, 0.0]]), "m.e0.gate": rng.normal(size=(3, 2)),
         "m.e0.up": rng.normal(size=(3, 2)), "m.e0.down": rng.normal(size=(2, 3)),
         "m.e1.gate": rng.normal(size=(3, 2)), "m.e1.up": rng.normal(size=(3, 2)), "m.e1.down": rng.normal(size=(2, 3))}
    h = np.array([[1.0, 0.3]])
    s = P.sigmoid(5.0)
    x = s * h[0]
    want = (P.silu(W["m.e0.gate"] @ x) * (W["m.e0.up"] @ x)) @ W["m.e0.down"].T
    got = P.expert_ff(h, W, "m.", dict(router=dict(experts=2, top=1)))
    assert np.allclose(got[0], want)
    # the weight on the output would give another number: the unit is not linear
    other = s * ((P.silu(W["m.e0.gate"] @ h[0]) * (W["m.e0.up"] @ h[0])) @ W["m.e0.down"].T)
    assert not np.allclose(got[0], other, rtol=1e-3)


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_portions_and_single_tokens_give_the_whole_sequence_s_logits(name):
    cfg, seed = CONFIGS[name]
    W = weights(cfg, seed)
    toks = np.random.default_rng(seed).integers(0, cfg["vocab"], size=23).tolist()
    want = P.forward(cfg, W, toks)
    for cuts in ([1], [2], [5, 1, 9, 3]):
        st, got, at, i = P.Stepper(cfg, W), [], 0, 0
        while at < len(toks):
            n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
            got.append(st.feed(toks[at:at + n]))
            at, i = at + n, i + 1
        assert np.allclose(np.concatenate(got), want, atol=1e-9), (name, cuts)


def test_every_mechanism_moves_the_logits():
    """What the tests' weights would hide could be wrong unseen: every constant of the design, changed a little, moves
    the logits by far more than any tolerance."""
    cfg, seed = CONFIGS["SA"]
    W = weights(cfg, seed)
    toks = np.random.default_rng(1).integers(0, cfg["vocab"], size=30).tolist()
    want = P.forward(cfg, W, toks)
    size = float(np.sqrt(np.mean(want ** 2)))

    def moved(change, weights_change=None):
        c, w = copy.deepcopy(cfg), dict(W)
        change(c["layers"])
        if weights_change:
            weights_change(w)
        return float(np.sqrt(np.mean((P.forward(c, w, toks) - want) ** 2))) / size

    assert moved(lambda L: L[1]["mixer"]["q_temp"].update(every=4)) > 1e-3
    assert moved(lambda L: L[1]["mixer"]["q_temp"].update(coef=0.0)) > 1e-3
    assert moved(lambda L: L[2]["mixer"]["left"].update(softcap=30.0)) > 1e-3
    assert moved(lambda L: L[2]["mixer"]["left"]["rot"].pop("scaling")) > 1e-3
    assert moved(lambda L: L[2]["mixer"].update(right_scale=0.0)) > 1e-2
    assert moved(lambda L: L[2]["mixer"].update(left_scale=0.0)) > 1e-2
    assert moved(lambda L: L[0]["mixer"].update(decay=[0.9, 0.99, 0.6])) > 1e-3
    assert moved(lambda L: L[0]["mixer"]["rot"].update(dims=4)) > 1e-3
    assert moved(lambda L: L[3]["mixer"].update(kv_from=1), lambda w: w.update({"l1.mix.r1": w["l1.mix.r1"] * 0})) > 1e-3
    assert moved(lambda L: None, lambda w: w.update({"l3.mix.r2": w["l3.mix.r2"] * 2})) > 1e-3
    assert moved(lambda L: L[0]["mlp"]["router"].update(top=3)) > 1e-3
    assert moved(lambda L: None, lambda w: w.update({"l1.norm1": w["l1.norm1"] * 1.1})) > 1e-3


# ---------------------------------------------------------------------------------------------- the engine's side, no GPU
def test_tensor_names_and_shapes_are_the_plain_implementation_s():
    from allpaca_amd.models import DecoderModel, describe_model
    for name, (cfg, _) in CONFIGS.items():
        _, typed, spec = describe_model(cfg)
        got = {n: tuple(ps.shape) for n, ps in DecoderModel(spec).param_specs().items()}
        assert got == P.tensor_shapes(cfg), name


def bare(cfg):
    """The configuration without the sizes that the tensors' shapes give."""
    c = copy.deepcopy(cfg)
    c.pop("vocab"), c.pop("width")
    for layer in c["layers"]:
        m = layer["mixer"]
        if layer["type"] == "parallel":
            for k in ("heads", "kv_heads", "dim", "vdim"):
                m["left"].pop(k)
            for k in ("inner", "state", "dt_rank", "conv"):
                m["right"].pop(k)
        else:
            for k in ("heads", "kv_heads", "dim", "vdim", "conv"):
                m.pop(k, None)
        f = layer.get("mlp")
        if f and f["kind"] == "dense":
            f.pop("ff")
        elif f:
            f["expert"].pop("ff"), f["router"].pop("experts")
    return c


def test_sizes_that_the_file_leaves_out_come_from_the_shapes():
    from allpaca_amd.models import describe_model
    for name, (cfg, _) in CONFIGS.items():
        _, full, _ = describe_model(cfg)
        _, filled, _ = describe_model(bare(cfg), P.tensor_shapes(cfg))
        assert filled == full, name


def test_configuration_errors_name_the_key():
    from allpaca_amd.config import ConfigError
    from allpaca_amd.models import describe_model
    cfg = CONFIGS["SA"][0]

    def broken(change, word):
        c = copy.deepcopy(cfg)
        change(c)
        with pytest.raises(ConfigError) as e:
            describe_model(c)
        assert word in str(e.value), str(e.value)

    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from")
    broken(lambda c: c["layers"][3]["mixer"].update(kv_from=0), "kv_from")
    broken(lambda c: c["layers"][3]["mixer"].update(vdim=8), "vdim")
    broken(lambda c: c["layers"][0]["mixer"].update(decay=[0.5]), "decay")
    broken(lambda c: c["layers"][2]["mixer"]["left"].update(vdim=10), "vdim")
    broken(lambda c: c["layers"][2]["mixer"]["left"]["rot"].update(dims=5), "dims")
    broken(lambda c: c["layers"][1].update(type="mamba"), "type")
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=9), "top")
    broken(lambda c: c["layers"][1]["mixer"]["q_temp"].update(every=0), "every")
    broken(lambda c: c.pop("embedding"), "embedding")


def test_cache_needs_of_owners_borrowers_and_recurrent_layers():
    from allpaca_amd.models import DecoderModel, describe_model
    from allpaca_amd.parts import FixedState, PagedKeysValues
    _, _, spec = describe_model(CONFIGS["SA"][0])
    needs = DecoderModel(spec).cache_needs()
    assert needs[0] == FixedState((3, 10, 6), "float32")
    assert needs[1] == {"mixer": PagedKeysValues(2, 6, 10), "mixer.state": FixedState((1, 4 * 6 + 2 * 6 + 2 * 10))}
    assert needs[2] == {"mixer.left": PagedKeysValues(2, 12, 12), "mixer.right": FixedState((20, 5), "float32"),
                        "mixer.right.state": FixedState((3, 20), "float32")}
    assert needs[3] == {"mixer.state": FixedState((2, 4 * 6))} and spec.plan[3].cache_of == 1
    from allpaca_amd.cache import CacheManager
    cm = CacheManager(needs, 4, 16, 2)
    assert len(cm.paged_groups) == 2 and len(cm.state_groups) == 5
    # a single tap keeps no rows, no convolution none either
    _, _, spec = describe_model(CONFIGS["SC"][0])
    needs = DecoderModel(spec).cache_needs()
    assert needs[0] == PagedKeysValues(1, 16, 16) and needs[3] == PagedKeysValues(3, 8, 8)
    assert needs[1] == {"mixer.left": PagedKeysValues(1, 16, 16), "mixer.right": FixedState((8, 1), "float32")}


def test_a_preset_of_the_design():
    from allpaca_amd.config import preset
    from allpaca_amd.models import describe_model
    arch, cfg, spec = describe_model(preset("seredra-tiny"))
    assert arch.name == "seredra" and len(spec.plan) == len(cfg.layers) and any(e.cache_of is not None for e in spec.plan)
