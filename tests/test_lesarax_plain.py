"""The plain implementation of the Lesarax decoder pinned by values worked out by hand, and what needs no GPU of the
design's place in the framework: configuration, tensor names, the order of the layers, cache needs."""
import math

import numpy as np
import pytest

import plain_lesarax as P
from lesarax_helpers import CONFIGS, TINY_LA, TINY_LB, TINY_LC, TINY_LD, planted


def test_rotation_pairs_an_element_with_the_one_half_the_range_further_on():
    """Four rotated elements, base 100: pairs (0, 2) and (1, 3), angles p and p / 10; the rest of the head stays."""
    v = np.array([[[1.0, 2.0, 3.0, 4.0, 5.0, 6.0]]])
    got = P.rotate_front(v, [3], 100.0, 4)[0, 0]
    c0, s0, c1, s1 = math.cos(3.0), math.sin(3.0), math.cos(0.3), math.sin(0.3)
    assert np.allclose(got, [1 * c0 - 3 * s0, 2 * c1 - 4 * s1, 3 * c0 + 1 * s0, 4 * c1 + 2 * s1, 5.0, 6.0])
    assert np.allclose(P.rotate_front(v, [0], 100.0, 4), v)
    # a rotation keeps the product of a query and a key a function of the distance alone
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(1, 8)), rng.normal(size=(1, 8))
    a = P.rotate(q, [17], 50.0) @ P.rotate(k, [12], 50.0).T
    b = P.rotate(q, [1005], 50.0) @ P.rotate(k, [1000], 50.0).T
    assert np.allclose(a, b)


def test_sink_takes_weight_and_gives_nothing():
    """Two keys with equal scores and a sink with the same score: each key gets a third."""
    q = np.array([[[1.0, 0.0]]])
    k = np.array([[[2.0, 5.0]], [[2.0, -1.0]]])
    v = np.array([[[3.0]], [[9.0]]])
    out = P.sink_attention(q, k, v, 0.5, np.array([1.0]))
    assert np.allclose(out, (3.0 + 9.0) / 3)
    assert np.allclose(P.sink_attention(q, k, v, 0.5, None), 6.0)
    # a sink far below the scores changes nothing, one far above takes everything
    assert np.allclose(P.sink_attention(q, k, v, 0.5, np.array([-60.0])), 6.0)
    assert np.allclose(P.sink_attention(q, k, v, 0.5, np.array([60.0])), 0.0)


def test_window_counts_the_row_itself():
    """Values 1, 2, 4, 8 at positions 0 .. 3 and flat scores: a window of 2 averages a row with the one before."""
    q, k = np.zeros((4, 1, 1)), np.zeros((4, 1, 1))
    v = np.array([1.0, 2.0, 4.0, 8.0]).reshape(4, 1, 1)
    assert np.allclose(P.sink_attention(q, k, v, 1.0, None, window=2).ravel(), [1.0, 1.5, 3.0, 6.0])
    assert np.allclose(P.sink_attention(q, k, v, 1.0, None, window=1).ravel(), [1.0, 2.0, 4.0, 8.0])
    assert np.allclose(P.sink_attention(q, k, v, 1.0, None, window=9).ravel(), [1.0, 1.5, 7 / 3, 15 / 4])
    # the last row alone, as a decoded token sees it
    assert np.allclose(P.sink_attention(q[3:], k, v, 1.0, None, window=3).ravel(), [14 / 3])


def test_grouped_heads_read_the_kv_head_of_their_group():
    q = np.zeros((1, 4, 1))
    k = np.zeros((1, 2, 1))
    v = np.array([[[5.0], [7.0]]])
    assert P.sink_attention(q, k, v, 1.0, None).ravel().tolist() == [5.0, 5.0, 7.0, 7.0]


def test_clamped_unit_by_hand():
    """gate 3 -> 2 (only from above), gate -5 stays; up 4 -> 2, up -4 -> -2; y = g sigmoid(1.702 g) (u + 1)."""
    h = np.array([[1.0, 1.0]])
    w_gate, w_up = np.array([[3.0, 0.0], [0.0, -5.0]]), np.array([[4.0, 0.0], [0.0, -4.0]])
    w_down = np.array([[1.0, 0.0], [0.0, 1.0]])
    got = P.clamped_unit(h, w_gate, w_up, w_down, 2.0)[0]
    want = [2.0 / (1 + math.exp(-1.702 * 2.0)) * 3.0, -5.0 / (1 + math.exp(1.702 * 5.0)) * (-1.0)]
    assert np.allclose(got, want)


def test_router_weights_are_the_softmax_over_the_chosen_logits():
    z = np.array([[0.0, math.log(6.0), -3.0, math.log(2.0)]])
    ids, w = P.route(z, 2)
    assert ids.tolist() == [[1, 3]] and np.allclose(w, [[0.75, 0.25]])
    ids, w = P.route(z, 1)
    assert ids.tolist() == [[1]] and np.allclose(w, [[1.0]])
    ids, w = P.route(z, 4)
    assert sorted(ids[0].tolist()) == [0, 1, 2, 3] and math.isclose(w.sum(), 1.0)


def test_latent_mixer_equals_attention_over_the_keys_it_stands_for():
    """With identity-like up projections the latent attention is an attention whose keys are [latent, shared rotated
    part] and whose values are the latent: worked out with the single mechanisms."""
    rng = np.random.default_rng(2)
    T, D, H, dn, dr, dv, Q, R = 7, 12, 2, 3, 2, 4, 5, 6
    m = dict(heads=H, dim=dn, rot_dim=dr, vdim=dv, q_rank=Q, kv_rank=R, scale=0.4, rot=dict(base=30.0, dims=dr),
             mask=dict(size=3))
    W = {"dq": rng.normal(size=(Q, D)), "dq.norm": rng.normal(size=Q), "uq": rng.normal(size=(H * (dn + dr), Q)),
         "dkv": rng.normal(size=(R + dr, D)), "dkv.norm": rng.normal(size=R), "uk": rng.normal(size=(H * dn, R)),
         "uv": rng.normal(size=(H * dv, R)), "sink": rng.normal(size=H), "g": rng.normal(size=(H, D)),
         "o": rng.normal(size=(D, H * dv))}
    h = rng.normal(size=(T, D))
    got = P.latent_mixer(h, W, "", m, 1e-5)
    pos = np.arange(T)
    q = (P.rms_norm(h @ W["dq"].T, W["dq.norm"], 1e-5) @ W["uq"].T).reshape(T, H, dn + dr)
    a = h @ W["dkv"].T
    c = P.rms_norm(a[:, :R], W["dkv.norm"], 1e-5)
    shared = P.rotate(a[:, R:], pos, 30.0)
    heads = []
    for j in range(H):
        qj = np.concatenate([q[:, j, :dn], P.rotate(q[:, j, dn:], pos, 30.0)], axis=-1)[:, None]
        kj = np.concatenate([c @ W["uk"][j * dn:(j + 1) * dn].T, shared], axis=-1)[:, None]
        vj = (c @ W["uv"][j * dv:(j + 1) * dv].T)[:, None]
        o = P.sink_attention(qj, kj, vj, 0.4, W["sink"][j:j + 1], window=3)[:, 0]
        heads.append(o * P.sigmoid(h @ W["g"][j])[:, None])
    assert np.allclose(got, np.concatenate(heads, axis=-1) @ W["o"].T)


def test_order_of_the_layers_and_where_a_pass_starts():
    assert P.layer_order(dict(layers=[0] * 4, loop=dict(start=1, stop=3, times=2))) == \
        [(0, False), (1, True), (2, False), (1, True), (2, False), (3, False)]
    assert P.layer_order(dict(layers=[0] * 2)) == [(0, False), (1, False)]
    from allpaca_amd.models import describe_model
    for name, (cfg, _) in CONFIGS.items():
        _, c, spec = describe_model(cfg)
        want = P.layer_order(cfg)
        assert [(e.block, e.enter is not None) for e in spec.plan] == want, name
        assert c.order() == want
        assert all(e.cache_of is None for e in spec.plan)        # every run of a layer has pages of its own


def test_configuration_and_tensor_names():
    from allpaca_amd.config import ConfigError
    from allpaca_amd.models import DecoderModel, describe_model
    arch, cfg, spec = describe_model(TINY_LA)
    assert arch.name == "lesarax" and cfg.residual_mult == 0.7 and cfg.loop.times == 3 and cfg.eps == 1e-5
    assert cfg.layers[0].mixer.window == 5 and cfg.layers[1].mlp is None and cfg.layers[0].mlp.limit == 0.8
    names = DecoderModel(spec).param_specs()
    assert {n: tuple(ps.shape) for n, ps in names.items()} == P.tensor_shapes(TINY_LA)
    assert names["loop.in"].shape == (36, 72) and names["l0.mix.dkv"].shape == (12 + 6, 36)
    assert names["l0.mix.uq"].shape == (3 * 16, 20) and names["l1.mix.k"].shape == (24, 36) and "l1.mix.v" not in names
    assert "l1.norm2" not in names and "l1.mlp.router" not in names and names["l2.mlp.e3.down"].shape == (36, 28)
    for name, (c, _) in CONFIGS.items():
        got = {n: tuple(ps.shape) for n, ps in DecoderModel(describe_model(c)[2]).param_specs().items()}
        assert got == P.tensor_shapes(c), name
    assert "loop.in" not in DecoderModel(describe_model(TINY_LD)[2]).param_specs()
    assert describe_model(TINY_LD)[1].layers[1].mixer.window is None

    def changed(layer, **mixer):
        layers = list(TINY_LB["layers"])
        layers[layer] = dict(layers[layer], mixer=dict(layers[layer]["mixer"], **mixer))
        return dict(TINY_LB, layers=layers)

    for bad, text in [({**TINY_LA, "residual_mult": None}, "residual_mult"), ({**TINY_LA, "norm": {}}, "eps"),
                      ({**TINY_LA, "loop": dict(start=2, stop=1, times=1)}, "loop"),
                      ({**TINY_LA, "loop": dict(start=0, stop=4, times=1)}, "loop"),
                      (changed(1, kv_heads=3), "kv_heads"), (changed(1, vdim=32), "vdim"),
                      (changed(1, rot=dict(base=10.0, dims=66)), "rot.dims"),
                      (changed(1, rot=dict(base=10.0, dims=7)), "even"),
                      (changed(0, rot=dict(base=10.0, dims=16)), "rot_dim"),
                      (changed(0, mask=dict(size=0)), "size"),
                      ({**TINY_LA, "layers": [dict(TINY_LA["layers"][0], type="lightning")]}, "not a mixer"),
                      ({**TINY_LA, "layers": [dict(TINY_LA["layers"][0], mlp=dict(kind="dense"))]}, "kind"),
                      ({**TINY_LA, "layers": [dict(TINY_LA["layers"][0],
                                                   mlp=dict(kind="moe", expert=dict(ff=8, limit=1.0),
                                                            router=dict(experts=2, top=3)))]}, "top")]:
        with pytest.raises(ConfigError, match=text):
            describe_model(bad)


def test_cache_needs_every_run_of_a_layer_has_pages_and_a_window_where_the_mixer_has_one():
    from allpaca_amd.models import DecoderModel, describe_model
    from allpaca_amd.parts import PagedKeysValues
    needs = DecoderModel(describe_model(TINY_LA)[2]).cache_needs()
    latent, grouped = PagedKeysValues(3, 16, 14, 5), PagedKeysValues(2, 12, 12, None)
    assert needs == [latent, grouped] * 3 + [PagedKeysValues(2, 8, 10, 11)]
    needs = DecoderModel(describe_model(TINY_LC)[2]).cache_needs()
    assert needs[0].window == 1 and needs[1] == PagedKeysValues(1, 16, 16, None) and needs[2].window == 4096


def test_planted_weights_make_the_mechanisms_show():
    """With the tests' weights a key more or less in a window, the sink and the clamps all move the logits by far more
    than any tolerance: a model that leaves one out cannot pass the comparisons."""
    cfg, seed = CONFIGS["LB"]
    W = {k: v.double().numpy() for k, v in planted(cfg, seed).items()}
    toks = np.random.default_rng(5).integers(0, cfg["vocab"], size=60).tolist()
    base = P.forward(cfg, W, toks)

    def moved(other_cfg=None, other_w=None):
        return float(np.abs(P.forward(other_cfg or cfg, other_w or W, toks) - base)[30:].max())

    wider = dict(cfg, layers=[dict(L, mixer=dict(L["mixer"], mask=dict(size=L["mixer"]["mask"]["size"] + 1)))
                              if "mask" in L["mixer"] else L for L in cfg["layers"]])
    assert moved(wider) > 1e-2
    assert moved(other_w={k: (v - 30.0 if k.endswith(".sink") else v) for k, v in W.items()}) > 1e-2
    loose = dict(cfg, layers=[dict(L, mlp=dict(L["mlp"], expert=dict(L["mlp"]["expert"], limit=100.0)))
                              if L["mlp"] else L for L in cfg["layers"]])
    assert moved(loose) > 1e-2
    assert moved(dict(cfg, loop=dict(cfg["loop"], times=1))) > 1e-2
    assert moved(other_w={**W, "loop.in": np.concatenate([W["loop.in"][:, :128], 0 * W["loop.in"][:, 128:]], axis=1)}) > 1e-2


def bare(cfg):
    """The configuration without the sizes that the shapes of the tensors give."""
    import copy
    out = copy.deepcopy(cfg)
    out.pop("vocab")
    out.pop("width")
    for L in out["layers"]:
        for k in ("heads", "kv_heads", "dim", "vdim", "q_rank", "kv_rank", "rot_dim"):
            L["mixer"].pop(k, None)
        if L["mlp"]:
            L["mlp"]["expert"].pop("ff")
            L["mlp"]["router"].pop("experts")
    return out


def test_sizes_that_config_json_leaves_out_come_from_the_tensors_shapes():
    from allpaca_amd.config import ConfigError
    from allpaca_amd.config.lesarax import sizes_from_tensors
    from allpaca_amd.models import describe_model
    for name, (cfg, _) in CONFIGS.items():
        shapes = P.tensor_shapes(cfg)
        assert describe_model(bare(cfg), shapes)[1] == describe_model(cfg)[1], name
        assert sizes_from_tensors(cfg, shapes) == cfg                 # what the file names stays
    with pytest.raises(ConfigError, match="vocab"):
        describe_model(bare(TINY_LA))                                  # no shapes at hand: the sizes are missing
