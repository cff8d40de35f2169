"""Every mechanism of the Suripel parts alone: the kernel against the plain function of
``plain_suripel``, with rows cut into requests and steps the way an engine cuts them, and with
inputs made so that a fault shows (one key that stands out just inside or just outside a window
or a block's edge, far away, at a page's border; state rows that start as NaN)."""
import math

import numpy as np
import pytest
import torch

import plain_suripel as S

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from xyntetik_runner_amd.csrc.ops import load_ops
    return load_ops()


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def step_ctx(starts, q_lens, slots, tables=()):
    """A step's context as the engine makes it: rows of the requests one after another.
    ``tables``: per cache group, one list of pages per request."""
    from xyntetik_runner_amd.cache import RequestCache
    from xyntetik_runner_amd.csrc.ops import load_ops
    from xyntetik_runner_amd.engine.batch import StepContext, StepEntry
    entries = [StepEntry(b, [0] * n, []) for b, n in enumerate(q_lens)]
    rcs = [RequestCache(b, int(slots[b]), int(starts[b]), [list(g[b]) for g in tables], fresh=False) for b in range(len(q_lens))]
    return StepContext(load_ops(), torch.device(DEV), entries, rcs, len(tables))


def cuts(total, sizes):
    out, i, k = [], 0, 0
    while i < total:
        n = min(sizes[k % len(sizes)], total - i)
        out.append((i, n))
        i += n
        k += 1
    return out


def close(got, want, tol, what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert np.isfinite(got).all(), f"{what}: not finite"
    err = np.abs(got - want).max() / max(1e-30, np.abs(want).max())
    assert err <= tol, f"{what}: {err:.3g} > {tol}"


# ----------------------------------------------------------------------------- row-wise
@pytest.mark.parametrize("E", [5, 48, 256, 1030])
def test_layernorm(ops, E):
    rng = np.random.default_rng(E)
    x = rng.normal(size=(7, E)) * 3 + 1.5
    w = rng.normal(size=E)
    got = ops.layernorm(dev(x), dev(w), 1e-5, torch.float32)
    close(got.cpu(), S.layer_norm(x, w, 1e-5), 2e-6, "layernorm")
    rows = dev([5, 0, 5], torch.int32)
    got = ops.layernorm(dev(x), dev(w), 1e-5, torch.bfloat16, rows=rows)
    close(got.float().cpu(), S.layer_norm(x[[5, 0, 5]], w, 1e-5), 1e-2, "layernorm rows bf16")


@pytest.mark.parametrize("F", [6, 72, 1000])
def test_polynorm(ops, F):
    rng = np.random.default_rng(F)
    z = rng.normal(size=(5, F)) * 2
    coef = [0.7, -1.3, 0.45, 0.2]
    got = ops.polynorm(dev(z), dev(coef), 1e-5, torch.float32)
    close(got.cpu(), S.polynorm(z, coef, 1e-5), 3e-6, "polynorm")
    # a view with a wider row stride, as a part of a wider product
    wide = dev(np.concatenate([z, z], axis=1))
    close(ops.polynorm(wide[:, :F], dev(coef), 1e-5, torch.float32).cpu(), S.polynorm(z, coef, 1e-5), 3e-6, "polynorm view")


@pytest.mark.parametrize("D,rot", [(16, 16), (16, 8), (10, 6), (12, 0)])
def test_rotation_in_place(ops, D, rot):
    rng = np.random.default_rng(D + rot)
    H, T = 3, 9
    x = rng.normal(size=(T, H, D))
    pos = np.array([0, 1, 2, 700, 701, 5, 6, 7, 2000])
    want = S.rotate_half(x, pos, rot, 1e4) if rot else x.copy()
    want = want * 0.25
    inv = dev((1e4 ** (-2.0 * np.arange(rot // 2) / rot))) if rot else None
    buf = dev(np.concatenate([x.reshape(T, H * D), np.zeros((T, 5))], axis=1))      # a view into a wider row
    ops.rotate_rows_(buf[:, :H * D], dev(pos, torch.int32), inv, H, D, rot, 0.25)
    close(buf[:, :H * D].cpu().reshape(T, H, D), want, 3e-6, "rotation")
    assert float(buf[:, H * D:].abs().max()) == 0.0


@pytest.mark.parametrize("H,Dv,weight", [(3, 20, True), (2, 64, False), (1, 130, True)])
def test_gated_norm_of_a_read_out(ops, H, Dv, weight):
    rng = np.random.default_rng(Dv)
    o = rng.normal(size=(6, H, Dv)) * 4
    g = rng.normal(size=(6, H, Dv))
    w = rng.normal(size=Dv) if weight else None
    want = S.rms_div(o, 1e-5) * (w if weight else 1.0) * S.silu(g)
    got = ops.gated_rmsnorm(dev(o.reshape(6, -1)), dev(g.reshape(6, -1)), dev(w) if weight else None, H, Dv, 1e-5, torch.float32)
    close(got.cpu().reshape(6, H, Dv), want, 3e-6, "gated norm")


# ----------------------------------------------------------------------------- convolution over time
@pytest.mark.parametrize("taps", [1, 2, 4, 7])
@pytest.mark.parametrize("residual,act", [(True, None), (False, "silu"), (False, None)])
def test_causal_conv_in_portions_and_batches(ops, taps, residual, act):
    """Three requests of unequal length, cut into portions (down to one and two tokens: shorter
    than the taps), run as batches of whatever each still has; state rows start as NaN except the
    rows of the requests, which are zeroed as the engine zeroes a new request's."""
    rng = np.random.default_rng(taps)
    C = 37
    lens = [23, 5, 40]
    us = [rng.normal(size=(n, C)) for n in lens]
    w = rng.normal(size=(C, taps))
    want = []
    for u in us:
        y = S.causal_conv(u, w) + (u if residual else 0)
        want.append(S.silu(y) if act else y)
    state = torch.full((4, max(taps - 1, 1), C), float("nan"), device=DEV) if taps > 1 else None
    slots = [2, 0, 1]
    if state is not None:
        state[:3] = 0
    plans = [cuts(lens[0], [1, 2, 5, 1, 9]), cuts(lens[1], [2, 1]), cuts(lens[2], [13, 1, 1, 2, 30])]
    got = [np.zeros((n, C)) for n in lens]
    k = 0
    while any(plans):
        live = [b for b in range(3) if plans[b]]
        if k % 3 == 1 and len(live) > 1:
            live = live[1:]                     # a request left out of a step goes on later
        k += 1
        parts = [plans[b].pop(0) for b in live]
        ctx = step_ctx([p[0] for p in parts], [p[1] for p in parts], [slots[b] for b in live])
        u = dev(np.concatenate([us[b][i:i + n] for b, (i, n) in zip(live, parts)]))
        y = ops.causal_conv(u, dev(w), state, ctx, torch.float32,
                            residual=residual, activation=act).cpu().numpy()
        r = 0
        for b, (i, n) in zip(live, parts):
            got[b][i:i + n] = y[r:r + n]
            r += n
    for b in range(3):
        close(got[b], want[b], 3e-6, f"conv request {b}")


@pytest.mark.parametrize("E,taps", [(48, 3), (1100, 4), (64, 1)])
def test_norm_and_convolution_in_one_kernel_for_steps_of_one_row(ops, E, taps):
    """Five requests decode 9 tokens each, one row a request and step: the fused kernel against
    the plain layer norm and convolution over each request's whole sequence, and bit for bit
    against the two kernels it stands for."""
    rng = np.random.default_rng(E)
    B, n = 5, 9
    xs = rng.normal(size=(B, n, E)) * 2 + 0.3
    w, cw = rng.normal(size=E), rng.normal(size=(E, taps))
    want = []
    for b in range(B):
        h = S.layer_norm(xs[b], w, 1e-5)
        want.append(h + S.causal_conv(h, cw))
    mk = lambda: torch.zeros((B + 1, taps - 1, E), device=DEV) if taps > 1 else None
    st_a, st_b = mk(), mk()
    slots = [3, 0, 4, 1, 2]
    for t in range(n):
        ctx = step_ctx([t] * B, [1] * B, slots)
        x = dev(xs[:, t])
        got = ops.layernorm_conv(x, dev(w), 1e-5, dev(cw), st_a, ctx, torch.float32)
        two = ops.causal_conv(ops.layernorm(x, dev(w), 1e-5, torch.float32), dev(cw), st_b, ctx, torch.float32, residual=True)
        assert torch.equal(got, two)
        if taps > 1:
            assert torch.equal(st_a, st_b)
        close(got.cpu(), np.stack([want[b][t] for b in range(B)]), 3e-6, f"token {t}")


# ----------------------------------------------------------------------------- recurrences
def run_recurrence(ops, kind, qs, ks, vs, extra, H, G, D, Dv, plans, slots, n_slots):
    """Requests (lists of per-token arrays) through ``linear_recurrence`` in the given portions."""
    state = torch.full((n_slots + 1,) + tuple(ops.recurrence_state_shape(H, D, Dv)), float("nan"), device=DEV)
    state[torch.tensor(slots, device=DEV)] = 0
    got = [np.zeros((len(q), H, Dv)) for q in qs]
    plans = [list(p) for p in plans]
    while any(plans):
        live = [b for b in range(len(qs)) if plans[b]]
        parts = [plans[b].pop(0) for b in live]
        ctx = step_ctx([p[0] for p in parts], [p[1] for p in parts], [slots[b] for b in live])
        cat = lambda xs: np.concatenate([xs[b][i:i + n].reshape(n, -1) for b, (i, n) in zip(live, parts)])
        # one wide row as a projection would bring it: q | k | v | pad, and the gates in rows of their own
        row = dev(np.concatenate([cat(qs), cat(ks), cat(vs), np.zeros((ctx.T, 3))], axis=1))
        q, k, v = row[:, :G * D], row[:, G * D:2 * G * D], row[:, 2 * G * D:2 * G * D + H * Dv]
        if kind == "delta":
            gates = dev(np.concatenate([cat(extra[0]), cat(extra[1])], axis=1))
            o = ops.linear_recurrence("delta", q, k, v, state, ctx, H, G, D, Dv, beta=gates[:, :H], gate=gates[:, H:])
        else:
            o = ops.linear_recurrence("retention", q, k, v, state, ctx, H, G, D, Dv, decay=dev(extra))
        o = o.cpu().numpy()
        r = 0
        for b, (i, n) in zip(live, parts):
            got[b][i:i + n] = o[r:r + n].reshape(n, H, Dv)
            r += n
    assert torch.isnan(state[n_slots]).all(), "the row that is nobody's was written"
    return got


@pytest.mark.parametrize("H,G,D,Dv", [(2, 2, 16, 16), (4, 2, 7, 9), (3, 1, 33, 70), (2, 1, 64, 130), (1, 1, 130, 8)])
def test_gated_delta_rule(ops, H, G, D, Dv):
    rng = np.random.default_rng(D * Dv)
    lens = [41, 3, 18]
    qs = [S.unit(rng.normal(size=(n, G, D))) * D ** -0.5 for n in lens]
    ks = [S.unit(rng.normal(size=(n, G, D))) for n in lens]
    vs = [rng.normal(size=(n, H, Dv)) for n in lens]
    beta = [S.sigmoid(rng.normal(size=(n, H)) * 2) for n in lens]
    g = [np.exp(-rng.uniform(0, 0.3, size=(n, H))) for n in lens]
    rep = H // G
    want = [S.gated_delta_rule(np.repeat(q, rep, 1), np.repeat(k, rep, 1), v, b, gg) for q, k, v, b, gg in zip(qs, ks, vs, beta, g)]
    plans = [cuts(41, [1, 9, 2, 17, 1]), cuts(3, [2, 1]), cuts(18, [18])]
    got = run_recurrence(ops, "delta", qs, ks, vs, (beta, g), H, G, D, Dv, plans, [1, 3, 0], 4)
    for b in range(3):
        close(got[b], want[b], 5e-6, f"delta request {b}")


def test_delta_rule_keeps_a_far_write(ops):
    """One token writes a value under a key nothing else uses; 500 tokens later a query along that
    key reads it back, decayed by the product of 500 gates: a state that is lost, reset or
    mixed up between slots on the way changes the answer by orders of magnitude."""
    rng = np.random.default_rng(1)
    H, D, Dv, n = 1, 8, 4, 520
    k = np.zeros((n, 1, D)); k[:, 0, 1:] = S.unit(rng.normal(size=(n, D - 1)))
    q = np.zeros((n, 1, D)); q[:, 0, 1:] = rng.normal(size=(n, D - 1)) * 0.01
    v = rng.normal(size=(n, 1, Dv))
    k[7, 0] = 0; k[7, 0, 0] = 1.0; v[7, 0] = [100.0, -50.0, 25.0, 5.0]
    q[510, 0] = 0; q[510, 0, 0] = 1.0
    beta = np.full((n, 1), 0.9); g = np.full((n, 1), 0.999)
    want = S.gated_delta_rule(q, k, v, beta, g)
    assert abs(want[510, 0, 0]) > 30          # the far write dominates that read-out
    got = run_recurrence(ops, "delta", [q], [k], [v], ([beta], [g]), H, 1, D, Dv, [cuts(n, [100, 1, 1, 63, 2])], [2], 3)
    close(got[0], want, 3e-5, "far write")        # 500 roundings of the decayed state, 6e-8 each


@pytest.mark.parametrize("H,D,Dv", [(2, 16, 8), (3, 6, 5), (1, 64, 100), (4, 10, 24)])
def test_retention(ops, H, D, Dv):
    rng = np.random.default_rng(D + Dv)
    lens = [37, 2, 64]
    qs = [rng.normal(size=(n, H, D)) for n in lens]
    ks = [rng.normal(size=(n, H, D)) * D ** -0.5 for n in lens]
    vs = [rng.normal(size=(n, H, Dv)) for n in lens]
    decay = list(rng.uniform(0.5, 0.999, size=H))
    want = [S.retention(q, k, v, decay) for q, k, v in zip(qs, ks, vs)]
    plans = [cuts(37, [5, 1, 1, 30]), cuts(2, [1]), cuts(64, [8, 9, 47])]
    got = run_recurrence(ops, "retention", qs, ks, vs, decay, H, H, D, Dv, plans, [0, 1, 2], 3)
    for b in range(3):
        close(got[b], want[b], 5e-6, f"retention request {b}")


@pytest.mark.parametrize("H,D,Dv", [(2, 64, 48), (1, 20, 70)])
def test_retention_in_chunks_side_by_side(ops, H, D, Dv):
    """A portion long enough to be cut into chunks that run side by side (1,300 rows: five chunks and a
    rest), in one step with a short request and one that ends on a chunk's edge; then the state each
    left is carried on token by token."""
    rng = np.random.default_rng(D)
    lens = [1300 + 9, 40 + 9, 1024 + 9]
    qs = [rng.normal(size=(n, H, D)) for n in lens]
    ks = [rng.normal(size=(n, H, D)) * D ** -0.5 for n in lens]
    vs = [rng.normal(size=(n, H, Dv)) for n in lens]
    decay = [0.97, 0.9995][:H]
    want = [S.retention(q, k, v, decay) for q, k, v in zip(qs, ks, vs)]
    assert max(lens) - 9 >= ops.RETENTION_CHUNKED_FROM
    plans = [[(0, n - 9)] + [(i, 1) for i in range(n - 9, n)] for n in lens]
    got = run_recurrence(ops, "retention", qs, ks, vs, decay, H, H, D, Dv, plans, [2, 0, 1], 3)
    for b in range(3):
        close(got[b], want[b], 2e-5, f"chunked retention request {b}")


def test_delta_prepare(ops):
    rng = np.random.default_rng(3)
    T, G, H, D = 5, 2, 4, 12
    q, k = rng.normal(size=(T, G, D)) * 3, rng.normal(size=(T, G, D)) * 1e-3
    b, a = rng.normal(size=(T, H)) * 3, rng.normal(size=(T, H)) * 4
    a[0, 0] = 40.0                                   # softplus far up its straight part
    a_log, dt = rng.normal(size=H), rng.normal(size=H)
    qk = dev(np.concatenate([q.reshape(T, -1), k.reshape(T, -1)], axis=1))
    ba = dev(np.concatenate([np.zeros((T, 2)), b, a], axis=1))
    ops.delta_prepare_(qk[:, :G * D], qk[:, G * D:], ba[:, 2:2 + H], ba[:, 2 + H:], dev(a_log), dev(dt), G, H, D, D ** -0.5, 1e-6)
    close(qk[:, :G * D].cpu().reshape(T, G, D), S.unit(q) * D ** -0.5, 3e-6, "unit q")
    close(qk[:, G * D:].cpu().reshape(T, G, D), S.unit(k), 3e-6, "unit k")      # tiny keys: the 1e-6 matters
    close(ba[:, 2:2 + H].cpu(), S.sigmoid(b), 3e-6, "beta")
    close(ba[:, 2 + H:].cpu(), np.exp(-np.exp(a_log) * S.softplus(a + dt)), 3e-6, "decay")


# ----------------------------------------------------------------------------- windowed attention with block means
def paged_attention_case(ops, dtype, H, G, D, Dv, size, P, page, lens, plans, q, k, v, scale, shuffle=0):
    """Requests through ``qkv_store`` / ``pool_blocks`` / ``attention_pooled`` in the given portions,
    with pages handed out in a shuffled order, as a pool that has been in use hands them out."""
    rng = np.random.default_rng(shuffle)
    n_pages = sum(-(-n // page) for n in lens) + 1
    pool_pages = sum(-(-max(1, n // P) // page) for n in lens) + 1 if P else 1
    free = list(rng.permutation(np.arange(1, n_pages)))
    pfree = list(rng.permutation(np.arange(1, pool_pages + len(lens))))
    fill = float("nan")
    kc = torch.full((n_pages, G, page, D), fill, dtype=dtype, device=DEV)
    vc = torch.full((n_pages, G, Dv, page), fill, dtype=dtype, device=DEV)
    pk = torch.full((pool_pages + len(lens), G, page, D), fill, dtype=dtype, device=DEV) if P else None
    pv = torch.full((pool_pages + len(lens), G, Dv, page), fill, dtype=dtype, device=DEV) if P else None
    tables = [[] for _ in lens]
    ptables = [[] for _ in lens]
    got = [np.zeros((n, H, Dv)) for n in lens]
    plans = [list(p) for p in plans]
    while any(plans):
        live = [b for b in range(len(lens)) if plans[b]]
        parts = [plans[b].pop(0) for b in live]
        for b, (i, n) in zip(live, parts):
            while len(tables[b]) < -(-(i + n) // page):
                tables[b].append(int(free.pop()))
            while P and len(ptables[b]) < -(-((i + n) // P) // page):
                ptables[b].append(int(pfree.pop()))
        ctx = step_ctx([p[0] for p in parts], [p[1] for p in parts], list(range(len(live))),
                       tables=([tables[b] for b in live], [ptables[b] for b in live]))
        cat = lambda xs: np.concatenate([xs[b][i:i + n].reshape(n, -1) for b, (i, n) in zip(live, parts)])
        row = dev(np.concatenate([cat(q), cat(k), cat(v)], axis=1))
        Q, K = H * D, G * D
        qd = ops.qkv_store(row[:, :Q], row[:, Q:Q + K], row[:, Q + K:], kc, vc, ctx, 0, H, G, D, Dv, page, dtype)
        if P:
            ops.pool_blocks(pk, pv, kc, vc, ctx, 0, 1, G, D, Dv, P, page)
        o = ops.attention_pooled(qd, kc, vc, pk, pv, ctx, 0, 1 if P else None, H, G, D, Dv, page, scale, size, P)
        o = o.float().cpu().numpy()
        r = 0
        for b, (i, n) in zip(live, parts):
            got[b][i:i + n] = o[r:r + n].reshape(n, H, Dv)
            r += n
    return got


def bf16_round(a):
    return torch.tensor(np.asarray(a), dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()


@pytest.mark.parametrize("H,G,D,Dv,size,P,page", [
    (4, 2, 16, 24, 9, 5, 8),        # blocks that divide no page, value size unlike key size
    (2, 2, 10, 6, 4, 8, 4),         # a block longer than the window (positions seen by nobody for a while)
    (3, 1, 8, 8, 11, 0, 16),        # no blocks
    (2, 1, 32, 32, 40, 16, 64),     # blocks of a quarter page
    (2, 2, 5, 3, 1, 1, 2),          # a window of one, blocks of one: every older token is a block
    (1, 1, 12, 12, 200, 3, 8),      # a window longer than any request: plain causal attention
])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_random_in_portions(ops, H, G, D, Dv, size, P, page, dtype):
    rng = np.random.default_rng(size * 31 + P)
    lens = [77, 1, 30]
    q = [rng.normal(size=(n, H, D)) for n in lens]
    k = [rng.normal(size=(n, G, D)) for n in lens]
    v = [rng.normal(size=(n, G, Dv)) for n in lens]
    plans = [cuts(77, [13, 1, 2, 1, 30, 1]), [(0, 1)], cuts(30, [2, 28])]
    rnd = bf16_round if dtype == torch.bfloat16 else None
    want = [S.pooled_window_attention(rnd(qq) if rnd else qq, kk, vv, 0.3, size, P, cache_round=rnd) for qq, kk, vv in zip(q, k, v)]
    got = paged_attention_case(ops, dtype, H, G, D, Dv, size, P, page, lens, plans, q, k, v, 0.3, shuffle=P)
    for b in range(3):
        close(got[b], want[b], 5e-6 if dtype == torch.float32 else 1.5e-2, f"attention request {b}")


@pytest.mark.parametrize("H,G,D,size,P,page", [(4, 2, 64, 100, 16, 16), (8, 2, 128, 70, 32, 64), (2, 2, 32, 33, 5, 32),
                                                 (4, 1, 16, 150, 0, 64)])
def test_attention_on_the_matrix_cores_in_long_portions(ops, H, G, D, size, P, page):
    """bfloat16 with head sizes the matrix-core kernels take: the window's keys go through them (row
    blocks of a whole workgroup for the long portions, key ranges for the decoded tokens), the block
    means through a kernel of their own, and the merge adds them."""
    rng = np.random.default_rng(D + size)
    lens = [420, 1, 90]
    q = [rng.normal(size=(n, H, D)) for n in lens]
    k = [rng.normal(size=(n, G, D)) for n in lens]
    v = [rng.normal(size=(n, G, D)) for n in lens]
    plans = [[(0, 300), (300, 100)] + [(i, 1) for i in range(400, 420)], [(0, 1)], cuts(90, [64, 2, 24])]
    scale = D ** -0.5
    want = [S.pooled_window_attention(bf16_round(qq), kk, vv, scale, size, P, cache_round=bf16_round) for qq, kk, vv in zip(q, k, v)]
    got = paged_attention_case(ops, torch.bfloat16, H, G, D, D, size, P, page, lens, plans, q, k, v, scale, shuffle=size)
    for b in range(3):
        close(got[b], want[b], 1.5e-2, f"attention request {b}")


@pytest.mark.parametrize("size,P,page", [(9, 5, 8), (12, 4, 4), (6, 16, 8), (33, 8, 16)])
@pytest.mark.parametrize("decode_from", [None, 40])
def test_one_key_that_stands_out_at_every_distance(ops, size, P, page, decode_from):
    """One key (position j*) lies along every query with a score far above the rest, and carries a
    value of its own.  A query sees it alone, as one of the P members of a block's mean, or not
    at all, depending on its distance: the read-out's first channel is then about 1, about 1/P
    (the block's mean key scores 1/P of it, but still far above the rest) or about 0.  Every
    distance from 0 to 70 is checked against the plain function, in a prompt's portions and with
    the last positions decoded one by one."""
    D, Dv, n = 8, 4, 120
    rng = np.random.default_rng(size + P)
    for jstar in (3, 29, 47):
        k = np.zeros((n, 1, D)); k[:, 0, 1:] = rng.normal(size=(n, D - 1)) * 0.05
        q = np.zeros((n, 1, D)); q[:, 0, 0] = 1.0; q[:, 0, 1:] = rng.normal(size=(n, D - 1)) * 0.05
        v = np.zeros((n, 1, Dv)); v[:, 0, 1:] = rng.normal(size=(n, Dv - 1))
        k[jstar, 0, 0] = 40.0 * P
        v[jstar, 0, 0] = 1.0
        want = S.pooled_window_attention(q, k, v, 1.0, size, P)
        seen = want[:, 0, 0]
        assert seen[jstar] > 0.99 and seen[jstar + size - 1] > 0.99 and seen[jstar + size] < 0.6      # the window's edge
        plans = [cuts(n, [17, 2, 40, 3])] if decode_from is None else [[(0, decode_from)] + [(i, 1) for i in range(decode_from, n)]]
        got = paged_attention_case(ops, torch.float32, 1, 1, D, Dv, size, P, page, [n], plans, [q], [k], [v], 1.0, shuffle=jstar)
        close(got[0], want, 5e-6, f"key {jstar}")


def test_block_means_are_of_the_cached_values(ops):
    """In bfloat16 the mean of a block is the mean of what the cache holds (rounded keys), rounded
    once more when it is stored."""
    rng = np.random.default_rng(8)
    n, P, page, D, Dv = 40, 4, 8, 8, 8
    q = [rng.normal(size=(n, 2, D))]; k = [rng.normal(size=(n, 1, D)) * 3]; v = [rng.normal(size=(n, 1, Dv)) * 3]
    want = S.pooled_window_attention(bf16_round(q[0]), k[0], v[0], 0.5, 3, P, cache_round=bf16_round)
    got = paged_attention_case(ops, torch.bfloat16, 2, 1, D, Dv, 3, P, page, [n], [cuts(n, [7, 1])], q, k, v, 0.5)
    close(got[0], want, 1.2e-2, "bf16 means")
