"""The Seredra decoder on the GPU against the plain implementation (tests/plain_seredra.py): every new kernel alone,
then whole models of several shapes through the step function, the cache manager and the engine."""
import os

import numpy as np
import pytest
import torch

import plain_seredra as P
from seredra_helpers import (CONFIGS, _att, _dense, _layer, _model, _par, _ret, model_folder, oracle, oracle_logits,
                             oracle_noise, tokens_for, write_folder)

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
    the whole without its worst row in twenty (`rel`) and of nine rows in ten (`rel_rows`): where two router scores
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


def make_step(segments, tables, slots=None):
    """segments: [(pos0, rows)]; a step description on the device through the Python packer."""
    from allpaca_amd.engine.batch import Entry, pack_step
    entries = [Entry(i, [0] * n) for i, (_, n) in enumerate(segments)]
    return pack_step(entries, [p for p, _ in segments], slots or list(range(len(segments))), [tables],
                     torch.device(DEV), [0])


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


def read_pages(cache, table, n, G, dk, dv, P_):
    """(keys [n, G, dk], values [n, G, dv]) of positions 0 .. n-1 as the pages hold them."""
    pages = cache.float().cpu().numpy()
    keys, vals = np.zeros((n, G, dk)), np.zeros((n, G, dv))
    for pos in range(n):
        page, slot = table[pos // P_], pos % P_
        keys[pos] = pages[page, :, slot * dk:(slot + 1) * dk]
        vals[pos] = pages[page, :, P_ * dk + slot::P_][:, :dv]
    return keys, vals


# =========================================================================================== kernels alone
@pytest.mark.parametrize("H, G, dk, dv, taps, P_, qt", [(4, 2, 6, 10, 2, 3, (0.7, 3)), (8, 2, 64, 64, 4, 16, (0.5, 16)),
                                                        (6, 3, 40, 24, 5, 8, None), (3, 0, 16, 16, 3, 4, (0.3, 1)),
                                                        (2, 1, 32, 32, 1, 16, (1.5, 40)), (5, 5, 8, 8, 0, 4, None)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_convolution_norm_over_the_whole_projection_and_query_temperature(H, G, dk, dv, taps, P_, qt, dtype):
    """Two steps of three requests: the second step's portions (one of a single row, one shorter than the taps) look
    back into the rows the first step left.  q and k are normed over all their heads at once with weights of the
    projection's size, q is multiplied by the temperature of its position, v passes the convolution only."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(H * 100 + dk + taps)
    tdt = DTYPES[dtype]
    width = H * dk + G * (dk + dv)
    eps = 1e-5
    lens1, lens2 = [37, 2, 1], [9, 1, 2]
    total = [a + b for a, b in zip(lens1, lens2)]
    n_pages, tables = scattered_tables(rng, total, P_)
    rows = [bf(rng.normal(size=(L, width))) for L in total]
    bias = np.float32(rng.normal(size=width) * 0.3)
    conv = np.float32(rng.normal(size=(width, max(taps, 1)))) if taps else None
    qw, kw = np.float32(1 + 0.3 * rng.normal(size=H * dk)), np.float32(1 + 0.3 * rng.normal(size=max(G, 1) * dk))
    state = torch.zeros((4, max(taps, 1) - 1, width), dtype=torch.float32, device=DEV) if taps > 1 else None
    cache = torch.full((n_pages + 1, max(G, 1), P_ * (dk + dv)), float("nan"), dtype=tdt, device=DEV) if G else None
    got_q = [[], [], []]
    for first, lens in ((True, lens1), (False, lens2)):
        segs = [(0 if first else a, n) for a, n in zip(lens1, lens)]
        step = make_step(segs, tables)
        x = np.concatenate([r[p0:p0 + n] for r, (p0, n) in zip(rows, segs)])
        T = x.shape[0]
        q_out = torch.empty((T, H * dk), dtype=tdt, device=DEV)
        ops.conv_heads(dev(x, tdt), 0, H * dk, (H + G) * dk, H, G, dk, dv, dev(bias), dev(conv) if taps else None,
                       state, step, step.state_slots if taps > 1 else None, True, eps, q_out,
                       step.block_tables[0] if G else None, cache, P_, norm_dim=dk, q_norm_w=dev(qw),
                       k_norm_w=dev(kw) if G else None, norm_rows=True, q_temp_coef=qt[0] if qt else 0.0,
                       q_temp_every=qt[1] if qt else 0)
        r = 0
        for i, (_, n) in enumerate(segs):
            got_q[i].append(q_out[r:r + n].float().cpu().numpy())
            r += n
    for i, L in enumerate(total):
        u = rows[i] + bias
        y = P.short_conv(u, conv.astype(np.float64)) if taps else u
        q = P.unit_rms(y[:, :H * dk], eps) * qw
        if qt:
            q = q * P.query_temperature(np.arange(L), *qt)[:, None]
        tol = dict(dtype=dtype, rel=0.01)
        close(np.concatenate(got_q[i]), q, what=f"q of request {i}", **tol)
        if G:
            keys, vals = read_pages(cache, tables[i], L, G, dk, dv, P_)
            k = P.unit_rms(y[:, H * dk:(H + G) * dk], eps) * kw
            close(keys.reshape(L, -1), k, what=f"keys of request {i}", **tol)
            close(vals.reshape(L, -1), y[:, (H + G) * dk:], what=f"values of request {i}", **tol)


@pytest.mark.parametrize("H, G, dk, dv, P_, cap, bias", [(4, 2, 12, 12, 4, 0.0, True), (3, 3, 16, 14, 3, 2.5, False),
                                                         (8, 2, 64, 64, 16, 0.0, True), (8, 4, 32, 64, 16, 0.0, True),
                                                         (12, 4, 96, 96, 16, 6.0, False), (4, 1, 128, 128, 16, 3.0, True),
                                                         (6, 2, 40, 24, 8, 0.0, True)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_distance_penalty_and_soft_cap_over_pages_with_one_key_that_stands_out(H, G, dk, dv, P_, cap, bias, dtype):
    """Attention with a penalty r1 ln(1 + r2 d) on a key d positions back and / or a soft cap on the scores, on
    scattered pages whose unwritten slots hold NaN: a portion of 70 rows that starts at position 200 beside decoded
    rows at positions 300 and 64.  Head 0 of the last row of the portion and of the first decoded row asks, with a
    large query, for one key: far back, on either side of a page's border, the row itself."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(H + dk + int(cap * 10))
    tdt = DTYPES[dtype]
    lens, segs = [270, 301, 65], [(200, 70), (300, 1), (64, 1)]
    n_pages, tables = scattered_tables(rng, lens, P_)
    keys = [bf(rng.normal(size=(L, G, dk))) * 0.5 for L in lens]
    vals = [bf(rng.normal(size=(L, G, dv))) for L in lens]
    r1 = np.float32(0.2 + 0.6 * rng.random(size=H)) if bias else None
    r2 = np.float32(0.1 + 2.0 * rng.random(size=H)) if bias else None
    last = (269, 300)
    border = (200 // P_) * P_
    targets = [(1, 1), (border - 1, border - 1), (border, border), last]
    for t0, t1 in targets:
        keys[0][t0, 0] *= 4.0
        keys[1][t1, 0] *= 4.0
    pages = np.full((n_pages + 1, G, P_ * (dk + dv)), np.nan, dtype=np.float32)
    fill_pages(pages, tables, keys, vals, P_)
    cache = dev(pages, tdt)
    step = make_step(segs, tables)
    T = 72
    for t0, t1 in targets:
        q = bf(rng.normal(size=(T, H, dk))) * 0.5
        q[69, 0] = bf(keys[0][t0, 0] / np.linalg.norm(keys[0][t0, 0]) * 8.0)
        q[70, 0] = bf(keys[1][t1, 0] / np.linalg.norm(keys[1][t1, 0]) * 8.0)
        out = torch.empty((T, H * dv), dtype=tdt, device=DEV)
        ops.masked_attention(dev(q.reshape(T, -1), tdt), out, H, G, dk, dv, cache, P_, step.block_tables[0], step,
                             "causal", 0, False, 0.8, softcap=cap,
                             distance_bias=(dev(r1), dev(r2)) if bias else None)
        got = out.float().cpu().numpy().reshape(T, H, dv)
        r = 0
        for (p0, n), k_, v_ in zip(segs, keys, vals):
            want = P.softmax_attention(q[r:r + n], k_[:p0 + n], v_[:p0 + n], 0.8, q_pos0=p0, softcap=cap, r1=r1, r2=r2)
            if dtype == "float32":
                close(got[r:r + n], want, "float32", f"targets {t0, t1} segment at {p0}")
            else:
                close(got[r:r + n].reshape(n, -1), want.reshape(n, -1), "bfloat16", f"targets {t0, t1} at {p0}", rel=0.02)
            r += n
        if not cap:          # without a cap the planted key carries its row, also from far back under the penalty
            for row, seg, t_, p in ((69, 0, t0, 269), (70, 1, t1, 300)):
                w = P.softmax_attention(q[row:row + 1, :1], keys[seg][:p + 1, :1], np.eye(p + 1)[:, None, :], 0.8,
                                        q_pos0=p, r1=r1, r2=r2)[0, 0]
                assert w[t_] > 0.3, (t_, w[t_])


@pytest.mark.parametrize("H, G, dk, rot, P_, scaling", [(4, 2, 12, 4, 3, (3.0, 16, 8.0, 1.0)), (8, 2, 64, 32, 16, (4.0, 64, 16.0, 2.0)),
                                                        (3, 3, 16, 16, 8, None), (2, 1, 40, 0, 4, None),
                                                        (12, 4, 96, 64, 16, (5.0, 128, 16.0, 2.0)), (4, 4, 128, 64, 16, None)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_head_norms_rotation_under_a_frequency_rule_and_values_that_stay_as_projected(H, G, dk, rot, P_, scaling, dtype):
    """One projected row holds q and k.  Every head is normed with weights all heads share, then rotated; k goes into
    the pages normed and rotated, and as projected into the values; a portion that starts inside a page beside two
    single rows."""
    from allpaca_amd.kernels import ops
    from allpaca_amd.parts.base import Runtime
    from allpaca_amd.parts.rope import rotary_table
    rng = np.random.default_rng(H * dk + rot)
    tdt = DTYPES[dtype]
    eps = 1e-5
    segs, lens = [(P_ + 1, 2 * P_ + 3), (0, 1), (5 * P_ - 1, 1)], [3 * P_ + 4, 1, 5 * P_]
    n_pages, tables = scattered_tables(rng, lens, P_)
    T = sum(n for _, n in segs)
    rows = bf(rng.normal(size=(T, (H + G) * dk)))
    proj = dev(rows, tdt)
    qw, kw = np.float32(1 + 0.3 * rng.normal(size=dk)), np.float32(1 + 0.3 * rng.normal(size=dk))
    cache = torch.full((n_pages + 1, G, P_ * 2 * dk), float("nan"), dtype=tdt, device=DEV)
    step = make_step(segs, tables)
    rule = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    table = None
    if rot:
        table = rotary_table(rot, 700.0, Runtime(torch.device(DEV), tdt, 8 * P_),
                             dict(rule, rope_type="yarn") if rule else None)
    q = proj[:, :H * dk]
    ops.rotary_pages(proj, 0, H, dk, 0, q, proj, H * dk, dk, None, 0, 0, False, 0, proj, H * dk, dk, G, rot, table, step,
                     step.block_tables[0], cache, P_, q_norm_w=dev(qw), k_norm_w=dev(kw), norm_eps=eps)
    pos = np.concatenate([np.arange(p0, p0 + n) for p0, n in segs])
    spec = dict(base=700.0, dims=rot, scaling=rule)
    want_q = P.rotate_front(P.unit_rms(rows[:, :H * dk].reshape(T, H, dk), eps) * qw, pos, spec)
    want_k = P.rotate_front(P.unit_rms(rows[:, H * dk:].reshape(T, G, dk), eps) * kw, pos, spec)
    close(q.float().cpu().numpy(), want_q.reshape(T, -1), dtype, "q", rel=0.01)
    pages = cache.float().cpu().numpy()
    r = 0
    for (p0, n), tb in zip(segs, tables):
        for a in range(n):
            page, slot = tb[(p0 + a) // P_], (p0 + a) % P_
            close(pages[page, :, slot * dk:(slot + 1) * dk], want_k[r + a], dtype, "keys", rel=0.01)
            close(pages[page, :, P_ * dk + slot::P_], rows[r + a, H * dk:].reshape(G, dk), dtype, "values", rel=0.004)
        r += n


@pytest.mark.parametrize("H, dk, dv, rot", [(3, 10, 6, 6), (4, 64, 64, 32), (2, 32, 128, 32), (1, 16, 16, 0), (2, 128, 64, 128)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_retention_with_rotation_over_two_steps_and_the_norm_of_every_head(H, dk, dv, rot, dtype):
    """Rotated q and k, k scaled behind the rotation, a decay a head (one of them 1), the state carried from a step of
    portions of 70, 3 and 1 rows into a step of 1, 2 and 22 rows; then every head's output over its own root mean
    square, times silu of a gate."""
    from allpaca_amd.kernels import ops
    from allpaca_amd.parts.base import Runtime
    from allpaca_amd.parts.rope import rotary_table
    rng = np.random.default_rng(dk + dv + rot)
    tdt = DTYPES[dtype]
    decay = [1.0, 0.9, 0.99, 0.5][:H]
    lens1, lens2 = [70, 3, 1], [1, 2, 22]
    width = H * (2 * dk + 2 * dv)
    rows = [bf(rng.normal(size=(a + b, width)) * 0.5) for a, b in zip(lens1, lens2)]
    state = torch.zeros((4, H, dk, dv), dtype=torch.float32, device=DEV)
    table = rotary_table(rot, 300.0, Runtime(torch.device(DEV), tdt, 128)) if rot else None
    scale = dk ** -0.5
    outs = [[], [], []]
    for first, lens in ((True, lens1), (False, lens2)):
        segs = [(0 if first else a, n) for a, n in zip(lens1, lens)]
        step = make_step(segs, [[0]] * 3)
        x = np.concatenate([r[p0:p0 + n] for r, (p0, n) in zip(rows, segs)])
        T = x.shape[0]
        o = torch.empty((T, H * dv), dtype=torch.float32, device=DEV)
        xd = dev(x, tdt)
        ops.linear_attention(xd, 0, H * dk, 2 * H * dk, H, dk, dv, False, dev(np.float32(decay)), state, step,
                             step.state_slots, o, rot=rot, cos_sin=table, k_scale=scale)
        a = torch.empty((T, H * dv), dtype=tdt, device=DEV)
        ops.gated_rmsnorm(o, None, 1e-5, xd[:, H * (2 * dk + dv):], a, group=dv, gate_act="silu")
        r = 0
        for i, (_, n) in enumerate(segs):
            outs[i].append(a[r:r + n].float().cpu().numpy())
            r += n
    spec = dict(base=300.0, dims=rot)
    for i, r in enumerate(rows):
        L = r.shape[0]
        q = P.rotate_front(r[:, :H * dk].reshape(L, H, dk), np.arange(L), spec)
        k = P.rotate_front(r[:, H * dk:2 * H * dk].reshape(L, H, dk), np.arange(L), spec) * scale
        o, S = P.retention(q, k, r[:, 2 * H * dk:H * (2 * dk + dv)].reshape(L, H, dv), decay)
        want = P.unit_rms(o, 1e-5).reshape(L, -1) * P.silu(r[:, H * (2 * dk + dv):])
        close(np.concatenate(outs[i]), want, dtype, f"request {i}", rel=0.01)
        close(state[i].cpu().numpy(), S, "float32" if dtype == "float32" else "bfloat16", f"state {i}", rel=0.01)


@pytest.mark.parametrize("C, N, taps, lens1, lens2", [
    (20, 5, 4, [70, 3, 1], [1, 2, 22]), (256, 16, 4, [70, 3, 1], [1, 2, 22]), (72, 8, 3, [70, 3, 1], [1, 2, 22]),
    (8, 1, 1, [70, 3, 1], [1, 2, 22]), (40, 100, 2, [70, 3, 1], [1, 2, 22]), (130, 64, 5, [70, 3, 1], [1, 2, 22]),
    (96, 16, 4, [333, 64, 128], [65, 1, 200]), (50, 33, 3, [129, 1, 5], [1, 1, 1]),
    (64, 16, 4, [601, 3, 70], [70, 519, 1]), (24, 4, 2, [515, 2, 1], [3, 2, 600])])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_selective_scan_and_its_convolution_over_two_steps(C, N, taps, lens1, lens2, dtype):
    """The convolution with its bias and silu, then the scan, with the last inputs and the state carried from one step
    of three portions into the next: portions of a row, of fewer rows than taps, of more rows than a chunk of the
    kernel that takes the chunks of a portion side by side, ending on a chunk's edge and one row behind it; a step of
    single rows only."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(C + N + taps)
    tdt = DTYPES[dtype]
    total = [a + b for a, b in zip(lens1, lens2)]
    xz = [bf(rng.normal(size=(L, 2 * C))) for L in total]
    dt = [np.float32(rng.normal(size=(L, C))) for L in total]
    bc = [np.float32(rng.normal(size=(L, 2 * N)) * 0.5) for L in total]
    w = np.float32(rng.normal(size=(C, taps)) * 0.5)
    b = np.float32(rng.normal(size=C) * 0.2)
    dtb = np.float32(rng.normal(size=C) - 1.0)
    A = np.float32(-np.exp(rng.normal(size=(C, N)) * 0.7 - 1.0))
    Dw = np.float32(1 + 0.2 * rng.normal(size=C))
    conv_state = torch.zeros((4, taps - 1, C), dtype=torch.float32, device=DEV) if taps > 1 else None
    state = torch.zeros((4, C, N), dtype=torch.float32, device=DEV)
    outs, xs = [[], [], []], [[], [], []]
    for first, lens in ((True, lens1), (False, lens2)):
        segs = [(0 if first else a, n) for a, n in zip(lens1, lens)]
        step = make_step(segs, [[0]] * 3)
        cat = lambda parts: np.concatenate([r[p0:p0 + n] for r, (p0, n) in zip(parts, segs)])
        xzd = dev(cat(xz), tdt)
        T = xzd.shape[0]
        x = torch.empty((T, C), dtype=tdt, device=DEV)
        ops.conv_channels(xzd, C, dev(w), dev(b), conv_state, step, step.state_slots if taps > 1 else None, "silu", x)
        y = torch.empty((T, C), dtype=tdt, device=DEV)
        ops.selective_scan(x, dev(cat(dt)), dev(dtb), dev(A), dev(cat(bc)), dev(Dw), xzd[:, C:], state, step,
                           step.state_slots, y)
        r = 0
        for i, (_, n) in enumerate(segs):
            outs[i].append(y[r:r + n].float().cpu().numpy())
            xs[i].append(x[r:r + n].float().cpu().numpy())
            r += n
    for i, L in enumerate(total):
        x = P.silu(P.short_conv(xz[i][:, :C], w.astype(np.float64)) + b)
        close(np.concatenate(xs[i]), x, dtype, f"convolution of request {i}", rel=0.01)
        x = x if dtype == "float32" else np.concatenate(xs[i]).astype(np.float64)      # the scan reads the stored x
        y, S = P.selective_scan(x, P.softplus(dt[i].astype(np.float64) + dtb), A.astype(np.float64), bc[i][:, :N],
                                bc[i][:, N:], Dw.astype(np.float64))
        close(np.concatenate(outs[i]), y * P.silu(xz[i][:, C:]), dtype, f"request {i}", rel=0.01)
        close(state[i].cpu().numpy(), S, "float32", f"state {i}")


@pytest.mark.parametrize("N, K", [(5, 3), (11, 3), (4, 4), (70, 5), (2, 1), (1, 1)])
def test_router_takes_the_largest_sigmoids_as_they_are(N, K):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(N + K)
    z = np.float32(rng.normal(size=(33, N)) * 2)
    z[3, :] = z[3, 0]                                        # a row of equal scores: the lower indices win
    ids = torch.empty((33, K), dtype=torch.int32, device=DEV)
    w = torch.empty((33, K), dtype=torch.float32, device=DEV)
    ops.route_topk(dev(z), None, K, ids, w, False, score="sigmoid")
    for t in range(33):
        want_ids, want_w = P.route(z[t].astype(np.float64), K)
        assert ids[t].cpu().tolist() == list(want_ids), t
        assert np.allclose(w[t].cpu().numpy(), want_w, rtol=1e-6)


@pytest.mark.parametrize("D, F, E, K, T", [(36, 20, 5, 2, 19), (128, 64, 8, 2, 150), (64, 32, 3, 3, 40), (128, 32, 2, 1, 300),
                                           (96, 72, 10, 4, 7), (256, 128, 4, 2, 700)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_experts_on_their_weighted_input(D, F, E, K, T, dtype):
    """Every pair's weight multiplies the expert's input; few and many rows an expert (tiles of 16, 64 and 128 rows on
    the matrix cores), an expert nobody chose."""
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(D + F + E + T)
    tdt = DTYPES[dtype]
    h = bf(rng.normal(size=(T, D)))
    W = {"m.router": np.zeros((E, D))}
    for e in range(E):
        W[f"m.e{e}.gate"], W[f"m.e{e}.up"] = bf(rng.normal(size=(F, D)) / D ** 0.5 * 1.5), bf(rng.normal(size=(F, D)) / D ** 0.5 * 1.5)
        W[f"m.e{e}.down"] = bf(rng.normal(size=(D, F)) / F ** 0.5)
    ids = np.stack([rng.permutation(E - 1 if E - 1 >= K else E)[:K] for _ in range(T)]).astype(np.int32)   # the last one idle
    weights = np.float32(0.2 + 0.8 * rng.random(size=(T, K)))
    gate_up = torch.stack([torch.cat([dev(W[f"m.e{e}.gate"], tdt), dev(W[f"m.e{e}.up"], tdt)]) for e in range(E)])
    down = torch.stack([dev(W[f"m.e{e}.down"], tdt) for e in range(E)])
    wgu, wd = ops.prepare_experts(gate_up.contiguous(), down.contiguous(), tdt)
    y = torch.empty((T, D), dtype=torch.float32, device=DEV)
    ops.routed_experts(dev(h, tdt), wgu, wd, E, F, dev(ids, torch.int32), dev(weights), K, y, activation="silu",
                       weight_input=True)
    want = np.zeros((T, D))
    for t in range(T):
        for e, we in zip(ids[t], weights[t].astype(np.float64)):
            x = we * h[t]
            want[t] += (P.silu(W[f"m.e{e}.gate"] @ x) * (W[f"m.e{e}.up"] @ x)) @ W[f"m.e{e}.down"].T
    close(y.cpu().numpy(), want, dtype, "experts", rel=0.012)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_activations_biases_and_the_sum_of_two_mixers(dtype):
    from allpaca_amd.kernels import ops
    rng = np.random.default_rng(5)
    tdt = DTYPES[dtype]
    for T, D, F in ((7, 36, 28), (150, 128, 256), (3, 96, 200)):
        h, w = bf(rng.normal(size=(T, D))), bf(rng.normal(size=(F, D)) / D ** 0.5)
        z = h @ w.T
        for name, fn in (("relu2", P.relu2), ("silu", P.silu),
                         ("gelu_tanh", lambda v: 0.5 * v * (1 + np.tanh(np.sqrt(2 / np.pi) * (v + 0.044715 * v ** 3))))):
            out = torch.empty((T, F), dtype=tdt, device=DEV)
            ops.linear_act(dev(h, tdt), ops.prepare_matrix(dev(w, tdt), tdt), out, name)
            close(out.float().cpu().numpy(), fn(z), dtype, name, rel=0.006)
        x, b = np.float32(rng.normal(size=(T, D))), np.float32(rng.normal(size=D))
        xd = dev(x)
        ops.bias_rows(xd, dev(b))
        close(xd.cpu().numpy(), x.astype(np.float64) + b, "float32", "bias")
        u, v = np.float32(rng.normal(size=(T, D))), np.float32(rng.normal(size=(T, D)))
        ud = dev(u)
        ops.weighted_pair(ud, 0.8, dev(v), 0.5, ud)
        close(ud.cpu().numpy(), 0.8 * u.astype(np.float64) + 0.5 * v, "float32", "weighted sum")


# =========================================================================================== whole models
# a mixer alone: one layer without feed-forward
ALONE = {
    "attention": (_model(40, 24, 2.0, 1e-5, [_layer(_att(6, 2, 4, 8, 0.5, conv=3, q_temp=(0.6, 2)), None)]), 61),
    "side_by_side": (_model(40, 24, 0.5, 1e-5, [_layer(_par((3, 1, 8, 0.4, 6, 25.0, 2.0, (2.0, 8, 4.0, 1.0)),
                                                           (12, 3, 2, 3), 0.8, 1.2), None)]), 62),
    "retention": (_model(40, 24, 1.5, 1e-5, [_layer(_ret(2, 6, 10, (0.8, 0.97), 4, 40.0), None)]), 63),
}


def folder_of(name, dtype="float32"):
    """The model's folder; with "bfloat16" the one whose matrices are stored in 16 bits (the same values: the planted
    weights are numbers that bfloat16 holds), which a bfloat16 run keeps in the matrix-core kernels' layout."""
    if name in ALONE:
        from helpers import tmp_root
        path = os.path.join(tmp_root(), "seredra_" + name)
        if not os.path.isdir(path):
            write_folder(path, *ALONE[name])
        return path
    return model_folder(name, dtype)


def make_runner(name, dtype, page_tokens=4, num_pages=160, max_requests=3, poison=False, use_graphs=False):
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    _, model = load_model(folder_of(name, dtype), DTYPES[dtype], DEV)
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


@pytest.mark.parametrize("name", sorted(ALONE))
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
    from test_seredra_plain import bare
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    src = model_folder("SA")
    path = os.path.join(tmp_root(), "seredra_SA_bare")
    shutil.copytree(src, path, dirs_exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(bare(CONFIGS["SA"][0]), f)
    cfg, model = load_model(path, torch.float32, DEV)
    assert cfg.vocab == 83 and cfg.layers[2].mixer.right.state == 5 and cfg.layers[3].mlp.ff == 12
    toks = tokens_for("SA", 19, 4)
    close(run_cut(ModelRunner(model, 4, 64, max_requests=2), toks, [19]), oracle_logits(src, toks), "float32", "bare")


def test_layers_one_by_one_in_32_bit():
    """The residual stream after every layer, for a prompt and for its last token alone."""
    for name in CONFIGS:
        toks = tokens_for(name, 37, 3)
        want = []
        P.forward(*oracle(model_folder(name)), toks, taps=want)
        runner = make_runner(name, "float32")
        got = []
        runner.model.layer_tap = lambda i, x: got.append(x.detach().cpu().numpy().copy())
        run_cut(runner, toks, [36, 1])
        n = len(want)
        assert len(got) == 2 * n
        for i in range(n):
            close(np.concatenate([got[i], got[n + i]]), want[i], "float32", f"{name} layer {i}")


@pytest.mark.parametrize("name", sorted(CONFIGS))
@pytest.mark.parametrize("dtype, page_tokens", [("float32", 4), ("bfloat16", 4), ("bfloat16", 16)])
def test_whole_prompts_decoding_and_portions(name, dtype, page_tokens):
    """(Pages of 16 positions: the bfloat16 run's attention on the matrix-core kernels where they take the sizes; of
    4: on the plain one.)  101 tokens: the temperatures step several times, portions start and end inside pages and
    inside the convolutions' reach."""
    toks = tokens_for(name, 101, 1)
    runner = make_runner(name, dtype, page_tokens=page_tokens)
    check(run_cut(runner, toks, [101]), name, toks, dtype, "whole")
    check(run_cut(runner, toks, [1]), name, toks, dtype, "token by token")
    check(run_cut(runner, toks, [40, 1]), name, toks, dtype, "prompt, then decoding")
    for cuts in ([2], [3, 2, 7, 1, 5], [6, 13, 2, 2, 66], [65, 1, 1, 2, 19, 3]):
        check(run_cut(runner, toks, cuts), name, toks, dtype, f"portions {cuts}")
    runner.cache.check()


def test_a_bfloat16_run_is_on_the_matrix_core_kernels():
    """A prompt portion and a decoded row of a model whose sizes the bfloat16 kernels take: the new mechanisms run on
    them and not on the plain kernels they would otherwise fall back to."""
    from allpaca_amd.engine.batch import Entry
    from allpaca_amd.kernels import lib as klib
    toks = tokens_for("SB", 70, 5)
    runner = make_runner("SB", "bfloat16", page_tokens=16)
    runner.admit("s")
    with klib.timing() as t:
        runner.step([Entry("s", toks[:69], [68])])
        runner.step([Entry("s", toks[69:], [0])])
    used = set(t.totals())
    runner.release("s")
    for name in ("apc_conv_heads_bf16", "apc_attention_masked_prefill_bf16", "apc_attention_masked_decode_bf16",
                 "apc_rotary_pages_bf16", "apc_linear_rotate_bf16", "apc_linear_attention_bf16",
                 "apc_selective_scan_bf16", "apc_routed_experts_bf16", "apc_gemm_bf16"):
        assert name in used, (name, sorted(used))
    for name in ("apc_conv_heads", "apc_masked_attention_plain", "apc_rotary_pages", "apc_routed_glu", "apc_gemm_plain"):
        assert name not in used, (name, sorted(used))


def test_cuttings_agree_to_the_bit_in_32_bit():
    for name in ("SA", "SC"):
        toks = tokens_for(name, 50, 8)
        runner = make_runner(name, "float32")
        whole = run_cut(runner, toks, [50])
        for cuts in ([1], [2], [7, 3, 1]):
            assert np.array_equal(whole, run_cut(runner, toks, cuts)), (name, cuts)


@pytest.mark.parametrize("name", ["SA", "SB"])
def test_first_tokens_and_page_sizes(name):
    for P_ in (1, 3, 16):
        runner = make_runner(name, "float32", page_tokens=P_, num_pages=200 if P_ == 1 else 80)
        for n in (1, 2, 3, 5, 7):
            toks = tokens_for(name, n, 40 + n)
            close(run_cut(runner, toks, [n]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens")
            close(run_cut(runner, toks, [1]), oracle_logits(model_folder(name), toks), "float32", f"{n} tokens, singly")


@pytest.mark.parametrize("name, dtype, page_tokens", [("SA", "float32", 4), ("SB", "float32", 4), ("SB", "bfloat16", 16),
                                                     ("SB", "bfloat16", 8), ("SC", "float32", 4), ("SD", "float32", 16),
                                                     ("SD", "bfloat16", 16)])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype, page_tokens):
    """Five requests of unequal lengths through three places and a pool that cannot hold them all at once: portions of
    some beside single tokens of others, free pages filled with a huge number, some requests left out of some steps.
    A request that comes later takes the pages and the state slot of one that has ended: a state that was not cleared,
    or a row of the convolutions left behind, would show."""
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
    """A short prompt, then 280 tokens one by one: the decode attention's passes of 256 keys and many pages go by, the
    states run through hundreds of single steps, the temperature steps many times."""
    toks = tokens_for("SB", 300, 2)
    check(run_cut(make_runner("SB", dtype, page_tokens=16, num_pages=160), toks, [20, 1]), "SB", toks, dtype,
          "long decoding")


def test_a_key_far_back_under_the_penalty_and_the_cap_in_a_whole_model():
    """One layer of each attention; the embedding of one token is made large, so that its key, hundreds of positions
    back, stands out for the rows that follow: in a prompt, in portions, in decoded rows."""
    from helpers import tmp_root
    from seredra_helpers import planted
    cfg = _model(60, 32, 3.0, 1e-6, [_layer(_att(4, 2, 8, 8, 0.6, conv=2, q_temp=(0.4, 50)), _dense(40)),
                                     _layer(_par((4, 2, 8, 0.6, 8, 100.0, 4.0, (2.0, 64, 8.0, 1.0)), (16, 4, 2, 3), 1.0, 0.7), None)])
    w = planted(cfg, 77)
    w["embed"][7] *= 6.0
    path = os.path.join(tmp_root(), "seredra_far_key")
    if not os.path.isdir(path):
        from allpaca_amd.weights import write_model_folder
        write_model_folder(path, cfg, 77, torch.float32, overrides=w)
    rng = np.random.default_rng(4)
    toks = [int(t) if t != 7 else 8 for t in rng.integers(0, 60, size=420)]
    toks[5] = 7
    want = P.forward(*P.read_model_folder(path), toks)
    plain = list(toks)
    plain[5] = 8
    moved = np.abs(P.forward(*P.read_model_folder(path), plain)[400:] - want[400:]).max()
    assert moved > 1e-2, moved                     # the far token does reach the last rows
    from allpaca_amd.engine.runner import ModelRunner
    from allpaca_amd.models import load_model
    _, model = load_model(path, torch.float32, DEV)
    runner = ModelRunner(model, 16, 64, max_requests=2, poison_free_pages=True)
    close(run_cut(runner, toks, [420]), want, "float32", "whole")
    close(run_cut(runner, toks, [390, 1]), want, "float32", "decoded")
    close(run_cut(runner, toks, [100, 3, 100, 43, 2]), want, "float32", "portions")


def test_greedy_generation_through_the_engine():
    """Requests of unequal lengths through the engine's scheduler, sampler and decode graphs, in float32: the tokens
    are the plain implementation's."""
    from allpaca_amd.engine import Engine
    from allpaca_amd.sampling import GenerationParams
    for name in ("SA", "SB"):
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
    folder = model_folder("SB", "bfloat16")
    prompts = [tokens_for("SB", n, 50 + n) for n in (3, 40, 11)]
    outs = []
    for graphs in (True, False):
        engine = Engine(folder, dtype="bfloat16", max_tokens=1024, page_tokens=16, max_active_requests=3,
                        use_graphs=graphs)
        assert engine.runner.use_graphs == graphs
        outs.append([o.token_ids for o in engine.generate(prompts, GenerationParams(max_tokens=20, temperature=0.0))])
    assert outs[0] == outs[1]


def test_command_line_and_replay_program(tmp_path):
    """The command line on a model folder of the design (float32, greedy: the plain implementation's tokens), and the
    replay program: three requests through a pool that holds two of them."""
    import json
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = model_folder("SA")
    prompts = [tokens_for("SA", 7, 5), tokens_for("SA", 19, 6)]
    spec = ";".join(",".join(str(t) for t in p) for p in prompts)
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--model", folder, "--dtype", "fp32",
           "--prompt-tokens", spec, "--max-tokens", "6", "--temperature", "0", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert [o["token_ids"] for o in outs] == [P.greedy(*oracle(folder), p, 6) for p in prompts]
    # the design's preset with random weights, sampled with temperature, top-k and top-p in bfloat16
    cmd = [sys.executable, os.path.join(root, "bin", "allpaca-amd"), "generate", "--synthetic", "seredra-tiny",
           "--prompt-tokens", "1,2,3;4,5", "--max-tokens", "5", "--temperature", "0.8", "--top-k", "20", "--top-p",
           "0.9", "--json"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    outs = [json.loads(ln) for ln in r.stdout.strip().splitlines() if ln.startswith("{")]
    assert len(outs) == 2 and all(len(o["token_ids"]) == 5 for o in outs)

    name = "SB"
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
