"""The Lesarax decoder on the GPU against the plain implementation (tests/plain_lesarax.py): every new kernel alone,
then whole models of several shapes through the step function, the cache manager and the engine."""
import os

import numpy as np
import pytest
import torch

import plain_lesarax as P
from lesarax_helpers import (CONFIGS, _att, _lat, _layer, model_folder, oracle, oracle_logits, oracle_noise, tokens_for,
                             write_folder)

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.asarray(a), dtype=dtype).to(DEV).contiguous()


def bf(a):
    """The values bfloat16 holds of `a`, as float64."""
    return torch.as_tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).double().numpy()


def close(got, want, dtype="float32", what="", rel=0.04, rel_rows=None):
    """float32: 3e-5 of the largest value.  bfloat16: the root mean square of the difference over that of the values, of
    the whole without its worst row in twenty (`rel`) and of nine rows in ten (`rel_rows`): where two router logits
    are nearly equal the choice of experts falls the other way in 16 bits, which is rounding and moves that row a lot;
    a key too many or too few moves every row behind it, and the float32 runs are exact about both."""
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert np.isfinite(got).all(), (what, "not finite")
    if dtype == "float32":
        tol = 3e-5 * max(1.0, float(np.abs(want).max()))
        err = np.abs(got - want)
        rows = np.argwhere(err.reshape(err.shape[0], -1).max(axis=1) > tol).ravel()[:6] if err.ndim > 1 else []
        assert float(err.max()) <= tol, (what, float(err.max()), tol, "first rows", list(rows))
    else:
        size = max(1e-9, float(np.sqrt(np.mean(want ** 2))))
        if got.ndim == 2 and got.shape[0] >= 10:
            per_row = np.sort(np.sqrt(np.mean((got - want) ** 2, axis=1)) / size)
            kept = per_row[:len(per_row) - -(-len(per_row) // 20)]            # without the worst row in twenty
            assert float(np.sqrt(np.mean(kept ** 2))) <= rel, (what, float(np.sqrt(np.mean(kept ** 2))))
            lim = rel if rel_rows is None else rel_rows
            assert float(np.quantile(per_row, 0.9)) <= lim, (what, "rows", float(np.quantile(per_row, 0.9)))
            assert float(per_row[-1]) <= 1.0, (what, "a row is off by its own size", float(per_row[-1]))
        else:
            rms = float(np.sqrt(np.mean((got - want) ** 2))) / size
            assert rms <= rel, (what, rms)


def check(got, name, toks, dtype, what=""):
    """Logits of a whole model against the plain implementation's.  bfloat16: at most one and a half times what rounding
    the stored activations to bfloat16 costs the plain implementation itself (and 1% of the logits' size)."""
    folder = folder_of(name)
    want = oracle_logits(folder, toks)
    if dtype == "float32":
        close(got, want, "float32", what)
    else:
        rms, rows = oracle_noise(folder, toks)
        close(got, want, "bfloat16", what, rel=max(0.01, 1.5 * rms), rel_rows=max(0.01, 1.5 * rows))


def near(got, want, dtype, what=""):
    """Element by element: float32 as `close`; bfloat16 within one step of bfloat16 of the exact value."""
    if dtype == "float32":
        return close(got, want, "float32", what)
    err = np.abs(np.asarray(got, dtype=np.float64) - want)
    assert (err <= 2.0 ** -8 * np.abs(want) + 1e-30).all(), (what, float(err.max()))


def make_step(segments, tables):
    """segments: [(pos0, rows)]; a step description on the device through the Python packer."""
    from allpaca_amd.engine.batch import Entry, pack_step
    entries = [Entry(i, [0] * n) for i, (_, n) in enumerate(segments)]
    return pack_step(entries, [p for p, _ in segments], list(range(len(segments))), [tables], torch.device(DEV), [0])


def scattered_tables(rng, lens, P_):
    n_pages = sum(-(-L // P_) for L in lens) + 3
    perm = (rng.permutation(n_pages - 1) + 1).tolist()
    tables = []
    for L in lens:
        n = -(-L // P_)
        tables.append(perm[:n])
        perm = perm[n:]
    return n_pages, tables


def fill_pages(pages, tables, keys, vals, P_):
    """pages [n + 1, G, P (dk + dv)]: a head's keys slot by slot, then its values with the slot as the fast axis."""
    dk = keys[0].shape[-1]
    for tb, k_, v_ in zip(tables, keys, vals):
        for pos in range(k_.shape[0]):
            page, slot = tb[pos // P_], pos % P_
            pages[page, :, slot * dk:(slot + 1) * dk] = k_[pos]
            pages[page, :, P_ * dk + slot::P_] = v_[pos]


# =========================================================================================== kernels alone
@pytest.mark.parametrize("H, G, dk, rot, P_", [(4, 2, 12, 4, 3), (10, 2, 64, 32, 16), (3, 3, 16, 16, 8), (2, 1, 40, 0, 4),
                                               (8, 2, 128, 64, 16)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rotation_of_the_front_of_a_head_and_values_that_are_the_unrotated_keys(H, G, dk, rot, P_, dtype):
    """One projected row holds q and k.  q is rotated where it lies, k goes rotated into the pages and unrotated into
    the values, at scattered pages, for a portion that starts inside a page beside two single rows."""
    from allpaca_amd.kernels import ops
    from allpaca_amd.parts.rope import rotary_table
    from allpaca_amd.parts.base import Runtime
    rng = np.random.default_rng(H * dk + rot)
    tdt = DTYPES[dtype]
    segs, lens = [(P_ + 1, 2 * P_ + 3), (0, 1), (5 * P_ - 1, 1)], [3 * P_ + 4, 1, 5 * P_]
    n_pages, tables = scattered_tables(rng, lens, P_)
    T = sum(n for _, n in segs)
    rows = bf(rng.normal(size=(T, (H + G) * dk)))
    proj = dev(rows, tdt)
    cache = torch.full((n_pages + 1, G, P_ * 2 * dk), float("nan"), dtype=tdt, device=DEV)
    step = make_step(segs, tables)
    base = 70.0
    table = rotary_table(rot, base, Runtime(torch.device(DEV), tdt, 6 * P_)) if rot else None
    ops.rotary_pages(proj, 0, H, dk, 0, proj[:, :H * dk], proj, H * dk, dk, None, 0, 0, False, 0, proj, H * dk, dk, G,
                     rot, table, step, step.block_tables[0], cache, P_)
    got_rows, got_pages = proj.float().cpu().numpy(), cache.float().cpu().numpy()
    r = 0
    for (p0, n), tb in zip(segs, tables):
        pos = np.arange(p0, p0 + n)
        q = rows[r:r + n, :H * dk].reshape(n, H, dk)
        k = rows[r:r + n, H * dk:].reshape(n, G, dk)
        want_q = P.rotate_front(q, pos, base, rot) if rot else q
        want_k = P.rotate_front(k, pos, base, rot) if rot else k
        near(got_rows[r:r + n, :H * dk], want_q.reshape(n, -1), dtype, "q")
        assert np.array_equal(got_rows[r:r + n, H * dk:], rows[r:r + n, H * dk:])       # k's columns stay as projected
        for a, p in enumerate(pos):
            page, slot = tb[p // P_], p % P_
            near(got_pages[page, :, slot * dk:(slot + 1) * dk], want_k[a], dtype, f"key at {p}")
            assert np.array_equal(got_pages[page, :, P_ * dk + slot::P_], k[a]), f"value at {p}"
        r += n
    written = sum(n for _, n in segs) * G * 2 * dk
    assert int(np.isfinite(got_pages).sum()) == written          # nothing beside the rows' own slots was touched


@pytest.mark.parametrize("H, dn, dr, dv, P_, pad", [(3, 10, 6, 14, 3, 2), (4, 32, 16, 64, 16, 0), (4, 16, 32, 64, 8, 4),
                                                    (2, 64, 64, 128, 16, 0), (1, 6, 2, 10, 4, 1)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_keys_put_together_from_a_head_s_own_part_and_a_rotated_part_all_heads_share(H, dn, dr, dv, P_, pad, dtype):
    """q rows of heads [dn plain, dr rotated]; keys [a head's dn, the dr shared ones rotated] from two tensors, the
    shared part in float32 rows at a column offset; values a third range."""
    from allpaca_amd.kernels import ops
    from allpaca_amd.parts.rope import rotary_table
    from allpaca_amd.parts.base import Runtime
    rng = np.random.default_rng(H * dn + dr)
    tdt = DTYPES[dtype]
    dk = dn + dr
    segs, lens = [(2 * P_ - 1, 3 * P_ + 2), (7, 1)], [5 * P_ + 1, 8]
    n_pages, tables = scattered_tables(rng, lens, P_)
    T = sum(n for _, n in segs)
    q = bf(rng.normal(size=(T, H, dk)))
    kv = bf(rng.normal(size=(T, H * (dn + dv))))
    off = 8 + pad
    a = np.float32(rng.normal(size=(T, off + dr + (8 if pad == 0 else 3))))     # a row stride of 8s, or any
    q_dev = dev(q.reshape(T, -1), tdt)
    cache = torch.full((n_pages + 1, H, P_ * (dk + dv)), float("nan"), dtype=tdt, device=DEV)
    step = make_step(segs, tables)
    base = 900.0
    table = rotary_table(dr, base, Runtime(torch.device(DEV), tdt, 6 * P_))
    ops.rotary_pages(q_dev, 0, H, dk, dn, q_dev, dev(kv, tdt), 0, dn, dev(a), off, dr, True, dn, dev(kv, tdt), H * dn, dv,
                     H, dr, table, step, step.block_tables[0], cache, P_)
    got_q, got_pages = q_dev.float().cpu().numpy().reshape(T, H, dk), cache.float().cpu().numpy()
    r = 0
    for (p0, n), tb in zip(segs, tables):
        pos = np.arange(p0, p0 + n)
        assert np.array_equal(got_q[r:r + n, :, :dn], q[r:r + n, :, :dn])
        near(got_q[r:r + n, :, dn:], P.rotate(q[r:r + n, :, dn:], pos, base), dtype, "q")
        shared = P.rotate(a[r:r + n, off:off + dr].astype(np.float64), pos, base)
        for i, p in enumerate(pos):
            page, slot = tb[p // P_], p % P_
            keys = got_pages[page, :, slot * dk:(slot + 1) * dk]
            assert np.array_equal(keys[:, :dn], kv[r + i, :H * dn].reshape(H, dn))
            near(keys[:, dn:], np.broadcast_to(shared[i], (H, dr)), dtype, f"shared part at {p}")
            assert np.array_equal(got_pages[page, :, P_ * dk + slot::P_], kv[r + i, H * dn:].reshape(H, dv))
        r += n
    assert int(np.isfinite(got_pages).sum()) == T * H * (dk + dv)


@pytest.mark.parametrize("H, G, dk, dv, P_, W", [(4, 2, 12, 12, 4, 0), (3, 3, 16, 14, 3, 37), (10, 2, 64, 64, 16, 0),
                                                 (4, 4, 48, 32, 16, 88), (4, 4, 32, 64, 8, 64), (2, 1, 128, 128, 16, 100),
                                                 (16, 2, 64, 64, 16, 0), (5, 5, 80, 40, 16, 50), (6, 3, 24, 24, 16, 0),
                                                 (2, 2, 200, 72, 16, 130), (12, 4, 96, 96, 16, 0), (7, 7, 160, 96, 16, 200),
                                                 (4, 1, 256, 256, 16, 0)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_sink_window_and_head_gate_over_pages_with_one_key_that_stands_out(H, G, dk, dv, P_, W, dtype):
    """Attention with a learned sink a head, a window (W > 0) or none, and a gate a head, on scattered pages whose
    unwritten slots hold NaN: a portion of 70 rows that starts at position 200 beside decoded rows at positions 300
    and 64.  Head 0 of the last row of the portion and of the first decoded row asks, with a large query, for one key:
    far back, at a page's border, the first one the window still holds, the one just in front of it, the row itself.
    A key the mask hides must not show, however loudly it is asked for."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(H + dk + W)
    tdt = DTYPES[dtype]
    lens, segs = [270, 301, 65], [(200, 70), (300, 1), (64, 1)]
    n_pages, tables = scattered_tables(rng, lens, P_)
    keys = [bf(rng.normal(size=(L, G, dk))) * 0.5 for L in lens]
    vals = [bf(rng.normal(size=(L, G, dv))) for L in lens]
    sinks = np.float32(rng.normal(size=H))
    sinks[-1] = 4.0                                   # a sink that takes most of a head's weight
    last = (269, 300)                                 # the asking rows' own positions in segments 0 and 1
    border = (200 // P_) * P_
    if W:
        targets = [tuple(p - W + 1 for p in last), tuple(p - W for p in last), tuple(p - W // 2 for p in last), last]
    else:
        targets = [(1, 1), (border - 1, border - 1), (border, border), last]
    for t0, t1 in targets:
        if t0 >= 0:
            keys[0][t0, 0] *= 4.0
        if t1 >= 0:
            keys[1][t1, 0] *= 4.0
    pages = np.full((n_pages + 1, G, P_ * (dk + dv)), np.nan, dtype=np.float32)
    fill_pages(pages, tables, keys, vals, P_)
    cache = dev(pages, tdt)
    step = make_step(segs, tables)
    T = 72
    win = W if W else None
    for t0, t1 in targets:
        q = bf(rng.normal(size=(T, H, dk))) * 0.5
        q[69, 0] = bf(keys[0][t0, 0] / np.linalg.norm(keys[0][t0, 0]) * 8.0)
        q[70, 0] = bf(keys[1][t1, 0] / np.linalg.norm(keys[1][t1, 0]) * 8.0)
        gate = np.float32(rng.normal(size=(T, H + 3)))
        for out_dt in (torch.float32, tdt):
            out = torch.empty((T, H * dv), dtype=out_dt, device=DEV)
            ops.masked_attention(dev(q.reshape(T, -1), tdt), out, H, G, dk, dv, cache, P_, step.block_tables[0], step,
                                 "window" if W else "causal", W, True, 0.8, sinks=dev(sinks), gate=dev(gate))
            got = out.float().cpu().numpy().reshape(T, H, dv)
            r = 0
            for (p0, n), k_, v_ in zip(segs, keys, vals):
                want = P.sink_attention(q[r:r + n], k_[:p0 + n], v_[:p0 + n], 0.8, sinks, window=win, q_pos0=p0)
                want = want * P.sigmoid(gate[r:r + n, :H].astype(np.float64))[:, :, None]
                if dtype == "float32":
                    close(got[r:r + n], want, "float32", f"targets {t0, t1} segment at {p0}")
                else:
                    close(got[r:r + n].reshape(n, -1), want.reshape(n, -1), "bfloat16", f"targets {t0, t1} at {p0}", rel=0.02)
                r += n
        # where the planted key may be seen it carries the row, almost alone; where not, the plain result above has
        # no trace of it and the comparison has shown that the kernel's has none either
        for row, seg, t_, p in ((69, 0, t0, 269), (70, 1, t1, 300)):
            w = P.sink_attention(q[row:row + 1, :1], keys[seg][:p + 1, :1], np.eye(p + 1)[:, None, :], 0.8, sinks[:1],
                                 window=win)[0, 0]
            if W and p - t_ >= W:
                assert w[t_] == 0.0
            else:
                assert w[t_] > 0.5, (t_, w[t_])


@pytest.mark.parametrize("N, K", [(5, 3), (11, 3), (4, 4), (70, 5), (2, 1), (1, 1)])
def test_router_takes_the_largest_logits_and_the_softmax_over_them_alone(N, K):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(N * 7 + K)
    T = 41
    z = np.float32(2 * rng.normal(size=(T, N)))
    ids = torch.empty((T, K), dtype=torch.int32, device=DEV)
    w = torch.empty((T, K), dtype=torch.float32, device=DEV)
    ops.route_topk(dev(z), None, K, ids, w, True)
    want_ids, want_w = P.route(z.astype(np.float64), K)
    assert np.array_equal(ids.cpu().numpy(), want_ids)
    close(w.cpu(), want_w, "float32", "weights")
    assert np.allclose(w.cpu().numpy().sum(axis=1), 1.0, atol=1e-5)


@pytest.mark.parametrize("D, F, E, K, T, limit", [(36, 20, 5, 3, 19, 0.8), (128, 64, 8, 2, 150, 1.0), (64, 32, 3, 3, 40, 0.5),
                                                  (32, 16, 1, 1, 7, 2.0), (256, 96, 4, 2, 700, 1.0), (192, 80, 10, 3, 1, 1.0),
                                                  (64, 48, 6, 2, 2, 7.0), (72, 40, 6, 2, 30, 1.0), (200, 136, 5, 4, 500, 1.0)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_routed_experts_with_clamped_units(D, F, E, K, T, limit, dtype):
    """Few rows and many, an expert nobody chooses, every expert chosen; inputs large enough that both clamps act on
    a good part of the elements (and a limit of 7 that hardly ever does)."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(D + T)
    tdt = DTYPES[dtype]
    h = bf(rng.normal(size=(T, D)))
    gate, up = bf(1.5 * rng.normal(size=(E, F, D)) / D ** 0.5), bf(1.5 * rng.normal(size=(E, F, D)) / D ** 0.5)
    down = bf(rng.normal(size=(E, D, F)) / F ** 0.5)
    pool = [e for e in range(E) if not (e == 1 and E - 1 >= K and E > 2)]
    ids = np.stack([rng.permutation(pool)[:K] for _ in range(T)]).astype(np.int32)
    w = np.float32(rng.random(size=(T, K)))
    gu, dn = ops.prepare_experts(dev(np.concatenate([gate, up], axis=1), tdt), dev(down, tdt), tdt)
    y = torch.empty((T, D), dtype=torch.float32, device=DEV)
    ops.routed_experts(dev(h, tdt), gu, dn, E, F, dev(ids, torch.int32), dev(w), K, y, activation="clamped", alpha=1.702,
                       limit=limit)
    rnd = P.to_bf16 if dtype == "bfloat16" else P.exact
    want = np.zeros((T, D))
    clamped = 0
    for t in range(T):
        for e, wt in zip(ids[t], w[t]):
            want[t] += wt * P.clamped_unit(h[t:t + 1], gate[e], up[e], down[e], limit, rnd)[0]
            clamped += int((np.abs(h[t] @ up[e].T) > limit).sum())
    assert limit > 5 or clamped > 0.05 * T * K * F
    close(y.cpu(), want, dtype, "experts", rel=6e-3)


@pytest.mark.parametrize("D", [36, 256, 1030])
def test_scaled_sum_in_32_bit_with_the_next_norm(D):
    """x += m y in float32, and h = rms_norm(new x) * w for whoever reads x next, also in the run's 16-bit type."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(D)
    T = 21
    x, y, w = np.float32(rng.normal(size=(T, D))), np.float32(rng.normal(size=(T, D))), np.float32(1 + 0.2 * rng.normal(size=D))
    one = torch.ones(1, dtype=torch.float32, device=DEV)
    mult = torch.full((1,), 0.3, dtype=torch.float32, device=DEV)
    for tdt in (torch.float32, torch.bfloat16):
        xd = dev(x)
        h = torch.empty((T, D), dtype=tdt, device=DEV)
        ops.streams_step(xd, 1, y=dev(y), mix=one, out_w=mult, in_w=one, norm_w=dev(w), eps=1e-5, h=h)
        want_x = x.astype(np.float64) + np.float64(np.float32(0.3)) * y
        close(xd.cpu(), want_x, "float32", "sum")
        want_h = P.rms_norm(want_x, w.astype(np.float64), 1e-5)
        if tdt == torch.float32:
            close(h.cpu(), want_h, "float32", "norm")
        else:
            assert float(np.abs(h.float().cpu().numpy() - want_h).max()) <= 2.0 ** -8 * float(np.abs(want_h).max())
        xd = dev(x)
        ops.streams_step(xd, 1, y=dev(y), mix=one, out_w=mult)
        close(xd.cpu(), want_x, "float32", "sum alone")


# =========================================================================================== whole models
# a mixer alone: one layer without feed-forward and without a loop
ONE_GROUPED = dict(architecture="Lesarax", vocab=40, width=24, residual_mult=0.5, norm=dict(eps=1e-5),
                   layers=[_layer(_att(6, 2, 8, 0.5, 4, 25.0), None)])
ONE_LATENT = dict(architecture="Lesarax", vocab=40, width=24, residual_mult=2.0, norm=dict(eps=1e-5),
                  layers=[_layer(_lat(3, 4, 4, 6, 7, 5, 0.6, 40.0, window=3), None)])
ALONE = {"grouped": (ONE_GROUPED, 41), "latent": (ONE_LATENT, 42)}


def folder_of(name):
    if name in ALONE:
        from helpers import tmp_root
        path = os.path.join(tmp_root(), "lesarax_" + name)
        if not os.path.isdir(path):
            write_folder(path, *ALONE[name])
        return path
    return model_folder(name)


def make_runner(name, dtype, page_tokens=4, num_pages=160, max_requests=3, poison=False, use_graphs=False):
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    _, model = load_model(folder_of(name), DTYPES[dtype], DEV)
    return ModelRunner(model, page_tokens, num_pages, max_requests=max_requests, poison_free_pages=poison,
                       use_graphs=use_graphs)


def run_cut(runner, toks, cuts, seq="s"):
    """All logits of `toks` fed in portions of the sizes `cuts` (the last size repeats)."""
    from allpaca_amd.engine.batch import Entry
    runner.admit(seq)
    out, at, i = [], 0, 0
    while at < len(toks):
        n = min(cuts[min(i, len(cuts) - 1)], len(toks) - at)
        out.append(runner.step([Entry(seq, toks[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
        i += 1
    runner.release(seq)
    return np.concatenate(out)


@pytest.mark.parametrize("name", ["grouped", "latent"])
def test_a_mixer_alone(name):
    cfg, _ = ALONE[name]
    toks = np.random.default_rng(3).integers(0, cfg["vocab"], size=23).tolist()
    want = P.forward(*oracle(folder_of(name)), toks)
    for P_ in (1, 4):
        runner = make_runner(name, "float32", page_tokens=P_, num_pages=64)
        close(run_cut(runner, toks, [23]), want, "float32", "whole")
        close(run_cut(runner, toks, [1]), want, "float32", "token by token")
        close(run_cut(runner, toks, [2, 5, 3]), want, "float32", "portions")


def test_a_folder_whose_config_leaves_sizes_to_the_tensors_shapes():
    import json
    import shutil
    from helpers import tmp_root
    from test_lesarax_plain import bare
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    src = model_folder("LA")
    path = os.path.join(tmp_root(), "LA_bare")
    shutil.copytree(src, path, dirs_exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(bare(CONFIGS["LA"][0]), f)
    cfg, model = load_model(path, torch.float32, DEV)
    assert cfg.vocab == 83 and cfg.layers[0].mixer.q_rank == 20 and cfg.layers[2].mlp.ff == 28
    toks = tokens_for("LA", 19, 4)
    close(run_cut(ModelRunner(model, 4, 64, max_requests=2), toks, [19]), oracle_logits(src, toks), "float32", "bare")


def test_ten_layers_with_ten_different_windows():
    """Every layer's pages are a group of their own (ten block tables a request), and every window gives pages back at
    its own pace."""
    from helpers import tmp_root
    cfg = dict(architecture="Lesarax", vocab=30, width=16, residual_mult=0.5, norm=dict(eps=1e-5),
               loop=dict(start=2, stop=5, times=2),
               layers=[_layer(_lat(2, 4, 4, 4, 8, 6, 0.4, 50.0, window=2 + 3 * i), None) for i in range(10)])
    path = write_folder(os.path.join(tmp_root(), "lesarax_windows"), cfg, 44)
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    _, model = load_model(path, torch.float32, DEV)
    runner = ModelRunner(model, 4, 24, max_requests=2, poison_free_pages=True)
    assert len(runner.cache.paged_groups) == 10
    toks = np.random.default_rng(6).integers(0, 30, size=60).tolist()
    want = P.forward(*P.read_model_folder(path), toks)
    close(run_cut(runner, toks, [60]), want, "float32", "whole")
    close(run_cut(runner, toks, [7, 1, 1, 30, 2, 1]), want, "float32", "portions")
    runner.cache.check()


def test_layers_one_by_one_in_32_bit():
    """The residual after every run of a layer (a looped layer counts each time) against the plain implementation's,
    for a prompt and for its last token alone."""
    for name in CONFIGS:
        toks = tokens_for(name, 37, 3)
        want = []
        P.forward(*oracle(model_folder(name)), toks, taps=want)
        assert len(want) == len(P.layer_order(CONFIGS[name][0]))
        runner = make_runner(name, "float32")
        got = []
        runner.model.layer_tap = lambda i, x: got.append(x.detach().cpu().numpy().copy())
        run_cut(runner, toks, [36, 1])
        n = len(want)
        assert len(got) == 2 * n
        for i in range(n):
            close(np.concatenate([got[i], got[n + i]]), want[i], "float32", f"{name} layer run {i}")


@pytest.mark.parametrize("name", ["LA", "LB", "LC", "LD", "LE", "LF", "LG"])
@pytest.mark.parametrize("dtype, page_tokens", [("float32", 4), ("bfloat16", 4), ("bfloat16", 16)])
def test_whole_prompts_decoding_and_portions(name, dtype, page_tokens):
    """(Pages of 16 positions: the bfloat16 run's attention on the matrix-core kernels where they take the sizes; of
    4: on the plain one.)  101 tokens: every window of the configurations but one passes over prompt rows and over
    decoded rows, and portions start and end inside windows and pages."""
    toks = tokens_for(name, 101, 1)
    runner = make_runner(name, dtype, page_tokens=page_tokens)
    check(run_cut(runner, toks, [101]), name, toks, dtype, "whole")
    check(run_cut(runner, toks, [1]), name, toks, dtype, "token by token")
    check(run_cut(runner, toks, [40, 1]), name, toks, dtype, "prompt, then decoding")
    for cuts in ([2], [3, 2, 7, 1, 5], [6, 13, 2, 2, 66], [65, 1, 1, 2, 19, 3]):
        check(run_cut(runner, toks, cuts), name, toks, dtype, f"portions {cuts}")
    runner.cache.check()


def test_cuttings_agree_to_the_bit_in_32_bit():
    toks = tokens_for("LA", 50, 8)
    runner = make_runner("LA", "float32")
    whole = run_cut(runner, toks, [50])
    for cuts in ([1], [2], [7, 3, 1]):
        assert np.array_equal(whole, run_cut(runner, toks, cuts)), cuts


@pytest.mark.parametrize("name", ["LA", "LB"])
def test_first_tokens_and_page_sizes(name):
    for P_ in (1, 3, 16):
        runner = make_runner(name, "float32", page_tokens=P_, num_pages=200 if P_ == 1 else 80)
        for n in (1, 2, 3, 5, 7):
            toks = tokens_for(name, n, 40 + n)
            close(run_cut(runner, toks, [n]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens")
            close(run_cut(runner, toks, [1]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens, singly")


@pytest.mark.parametrize("name, dtype, page_tokens", [("LA", "float32", 4), ("LB", "float32", 4), ("LB", "bfloat16", 16),
                                                     ("LB", "bfloat16", 8), ("LC", "float32", 4), ("LE", "float32", 16),
                                                     ("LE", "bfloat16", 16), ("LG", "bfloat16", 16)])
def test_mixed_batches_with_pages_used_again(name, dtype, page_tokens):
    """Five requests of unequal lengths through three places and a pool that cannot hold them all at once: portions of
    some beside single tokens of others, free pages filled with a huge number, some requests left out of some steps.
    Pages behind a window go back to the pool while their request still runs, and come out again for another."""
    from allpaca_amd.engine.batch import Entry
    rng = np.random.default_rng(9)
    lens = [37, 5, 90, 21, 70]
    reqs = {f"r{i}": tokens_for(name, n, 70 + i) for i, n in enumerate(lens)}
    P_ = page_tokens
    total = 50 * 4 // P_
    runner = make_runner(name, dtype, page_tokens=P_, num_pages=total, max_requests=3, poison=True)
    groups = range(len(runner.cache.paged_groups))

    def room(s, n, taken):
        need = runner.cache.pages_needed(s, n)
        return all(need[g] <= runner.cache.free_pages(g) - 2 * taken for g in groups)

    waiting, live, at, got = list(reqs), [], {}, {k: [] for k in reqs}
    while waiting or live:
        while waiting and len(live) < 3 and all(runner.cache.free_pages(g) >= -(-len(reqs[waiting[0]]) // P_) + 2
                                                for g in groups):
            s = waiting.pop(0)
            runner.admit(s)
            live.append(s)
            at[s] = 0
        entries = []
        for s in live:
            if rng.random() < 0.2 and len(live) > 1:
                continue                                   # left out of this step
            left = len(reqs[s]) - at[s]
            n = min(left, int(rng.choice([1, 1, 2, 3, 9, 16, 40])))
            if not room(s, n, len(entries)):
                n = 1
            entries.append(Entry(s, reqs[s][at[s]:at[s] + n], list(range(n))))
        if not entries:
            continue
        logits = runner.step(entries).cpu().numpy()
        r = 0
        for e in entries:
            n = len(e.tokens)
            got[e.seq].append(logits[r:r + n])
            r += n
            at[e.seq] += n
            if at[e.seq] == len(reqs[e.seq]):
                runner.release(e.seq)
                live.remove(e.seq)
    assert any(g.pool.allocations > total for g in runner.cache.paged_groups)      # pages came back and went out again
    for s, toks in reqs.items():
        check(np.concatenate(got[s]), name, toks, dtype, s)
    runner.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A short prompt, then 280 tokens one by one: the windows pass over decoded tokens only, the decode attention's
    passes of 256 keys and many pages go by."""
    toks = tokens_for("LB", 300, 2)
    check(run_cut(make_runner("LB", dtype, page_tokens=16, num_pages=160), toks, [20, 1]), "LB", toks, dtype,
          "long decoding")


def test_greedy_generation_through_the_engine():
    """Requests of unequal lengths through the engine's scheduler, sampler and decode graphs, in float32: the tokens
    are the plain implementation's."""
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    for name in ("LA", "LB"):
        folder = model_folder(name)
        prompts = [tokens_for(name, n, 90 + n) for n in (1, 9, 30, 4, 17)]
        want = [P.greedy(*oracle(folder), p, 10) for p in prompts]
        for graphs in (True, False):
            engine = Engine(folder, dtype="float32", max_tokens=512, page_tokens=4, max_active_requests=3,
                            chunk_tokens=8, max_batch_tokens=16, use_graphs=graphs)
            outs = engine.generate(prompts, GenerationParams(max_tokens=10, temperature=0.0))
            assert [o.token_ids for o in outs] == want, (name, graphs)


def test_graphs_replay_decode_steps_in_bfloat16():
    """Decode steps recorded as graphs and replayed give the tokens of the same engine without graphs."""
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    folder = model_folder("LB", "bfloat16")
    prompts = [tokens_for("LB", n, 50 + n) for n in (3, 40, 11)]
    outs = []
    for graphs in (True, False):
        engine = Engine(folder, dtype="bfloat16", max_tokens=1024, page_tokens=16, max_active_requests=3,
                        use_graphs=graphs)
        outs.append([o.token_ids for o in engine.generate(prompts, GenerationParams(max_tokens=20, temperature=0.0))])
    assert outs[0] == outs[1]


def test_command_line_and_replay_program(tmp_path):
    """The command line on a model folder of the design (float32, greedy: the plain implementation's tokens), and the
    replay program: three requests through a pool that holds two of them."""
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = model_folder("LA")
    prompts = [tokens_for("LA", 7, 5), tokens_for("LA", 19, 6)]
    spec = ";".join(",".join(str(t) for t in p) for p in prompts)
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--model", folder, "--dtype", "fp32",
           "--prompt-tokens", spec, "--max-tokens", "6", "--temperature", "0", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert [o["token_ids"] for o in outs] == [P.greedy(*oracle(folder), p, 6) for p in prompts]
    # the design's preset with random weights, sampled with temperature, top-k and top-p in bfloat16
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--synthetic", "lesarax-tiny",
           "--prompt-tokens", "1,2,3;4,5", "--max-tokens", "5", "--temperature", "0.8", "--top-k", "20", "--top-p",
           "0.9", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert len(outs) == 2 and all(len(o["token_ids"]) == 5 for o in outs)

    name = "LB"
    folder = model_folder(name)
    a, b, c = tokens_for(name, 70, 31), tokens_for(name, 9, 32), tokens_for(name, 50, 33)
    steps = [
        dict(step=0, entries=[dict(id="a", tokens=a[:33], want=list(range(33))), dict(id="b", tokens=b[:1], want=[0])], end=[]),
        dict(step=1, entries=[dict(id="b", tokens=b[1:3], want=[0, 1])], end=[]),
        dict(step=2, entries=[dict(id="a", tokens=a[33:69], want=list(range(36))), dict(id="b", tokens=b[3:], want=list(range(6)))],
             end=["b"]),
        dict(step=3, entries=[dict(id="a", tokens=a[69:], want=[0]), dict(id="c", tokens=c[:2], want=[0, 1])], end=["a"]),
        dict(step=4, entries=[dict(id="c", tokens=c[2:], want=list(range(48)))], end=["c"]),
    ]
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / f"replay_{dtype}")
        cmd = [sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
               "--max-tokens", "192", "--max-live", "2", "--poison-free-pages"]
        r = subprocess.run(cmd, input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True,
                           timeout=280)
        assert r.returncode == 0, r.stderr[-3000:]
        assert [ln for ln in r.stdout.split("\n") if ln.startswith("done")] == [f"done {i}" for i in range(5)]
        V = CONFIGS[name][0]["vocab"]
        got = {k: [] for k in "abc"}
        for s in steps:
            rows = np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4").reshape(-1, V)
            at = 0
            for e in s["entries"]:
                got[e["id"]].append(rows[at:at + len(e["want"])])
                at += len(e["want"])
            assert at == rows.shape[0]
        for k, toks in zip("abc", (a, b, c)):
            check(np.concatenate(got[k]), name, toks, dtype, f"replay {k}")
