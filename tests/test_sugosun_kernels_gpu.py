"""Every mechanism of the Sugosun parts alone: the kernel, or a one-layer model around it, against
the plain function of ``plain_sugosun``, with rows cut into requests and steps the way an engine
cuts them, and with inputs made so that a fault shows (a connection matrix that is not symmetric,
experts whose scores tie, one key that stands out just inside or just outside a window, far away,
at a page's border; state that starts as garbage)."""
import io

import numpy as np
import pytest
import torch

import plain_sugosun as G
import traces

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from xyntetik_runner_amd.csrc.ops import load_ops
    return load_ops()


def dev(a, dtype=torch.float32):
    return torch.tensor(np.asarray(a), dtype=dtype, device=DEV)


def step_ctx(starts, q_lens, slots, tables=()):
    """A step's context as the engine makes it: rows of the requests one after another."""
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


# ----------------------------------------------------------------------------- embedding
@pytest.mark.parametrize("buckets,mp,mc", [(53, 17, 5), (7, 3, 3), (1, 1, 0), (100003, 2147483647, 2147483629), (1009, 10 ** 15 + 37, 2 ** 40 + 1), (0, 0, 0)])
def test_pair_hash_embedding_in_portions(ops, buckets, mp, mc):
    """Three requests cut into portions (down to one token), one of them left out of some steps, in
    slots whose last-token entries start as garbage: a portion's first token hashes with the last
    token of the step before, a sequence's first token reads the extra row."""
    rng = np.random.default_rng(buckets + 1)
    V, E = 300, 24
    table, pairs = rng.normal(size=(V, E)), rng.normal(size=(buckets + 1, E)) if buckets else None
    w = rng.normal(size=E) + 1.0
    seqs = [list(rng.integers(0, V, size=n)) for n in (1, 19, 40)]
    want = [G.embed(s, table, pairs, w, 1e-5, buckets, mp, mc) for s in seqs]
    plans = [cuts(1, [1]), cuts(19, [1, 1, 5, 2, 10]), cuts(40, [7, 1, 2, 30])]
    last = torch.full((5,), 77, dtype=torch.int32, device=DEV)
    slots = [3, 0, 2]
    got = [np.zeros((len(s), E)) for s in seqs]
    turn = 0
    while any(plans):
        live = [b for b in range(3) if plans[b] and not (b == 1 and turn % 3 == 1)]
        turn += 1
        if not live:
            continue
        parts = [plans[b].pop(0) for b in live]
        ctx = step_ctx([p[0] for p in parts], [p[1] for p in parts], [slots[b] for b in live])
        ids = dev(np.concatenate([seqs[b][i:i + n] for b, (i, n) in zip(live, parts)]), torch.int32)
        x = ops.embedding_pairs(dev(table), dev(pairs) if buckets else None, dev(w), ids, ctx, last if buckets else None,
                                buckets, mp, mc, 1e-5).cpu().numpy()
        r = 0
        for b, (i, n) in zip(live, parts):
            got[b][i:i + n] = x[r:r + n]
            r += n
    for b in range(3):
        close(got[b], want[b], 3e-6, f"request {b}")
    if buckets:
        assert [int(last[s]) for s in slots] == [int(s[-1]) for s in seqs] and int(last[1]) == 77 and int(last[4]) == 77


# ----------------------------------------------------------------------------- residual streams
@pytest.mark.parametrize("S", [1, 2, 3, 8])
@pytest.mark.parametrize("E", [5, 64, 1030])
def test_streams_write_and_read(ops, S, E):
    rng = np.random.default_rng(S * 100 + E)
    T = 6
    xs = rng.normal(size=(S, T, E)) * 2
    y = rng.normal(size=(T, E))
    mix, out_w, in_w, nw = rng.normal(size=(S, S)), rng.normal(size=S), rng.normal(size=S), rng.normal(size=E)
    new = np.stack([sum(mix[s, t] * xs[s] for s in range(S)) + out_w[t] * y for t in range(S)])     # [from, to]
    u_old, u_new = np.tensordot(in_w, xs, 1), np.tensordot(in_w, new, 1)
    # read alone, with and without the norm
    d = dev(xs)
    close(ops.streams_step(d, in_w=dev(in_w)).cpu(), u_old, 3e-6, "read")
    close(ops.streams_step(d, in_w=dev(in_w), norm_w=dev(nw), eps=1e-5).cpu(), G.rms_norm(u_old, nw, 1e-5), 5e-6, "read + norm")
    assert np.array_equal(d.cpu().numpy(), xs.astype(np.float32))
    # write alone
    assert ops.streams_step(d, y=dev(y), mix=dev(mix), out_w=dev(out_w)) is None
    close(d.cpu(), new, 3e-6, "write")
    # write and the next read in one pass
    d = dev(xs)
    h = ops.streams_step(d, y=dev(y), mix=dev(mix), out_w=dev(out_w), in_w=dev(in_w), norm_w=dev(nw), eps=1e-5,
                         h_dtype=torch.bfloat16)
    close(d.cpu(), new, 3e-6, "write (fused)")
    close(h.float().cpu(), G.rms_norm(u_new, nw, 1e-5), 1e-2, "read after write")
    close(ops.streams_sum(d).cpu(), new.sum(0), 3e-6, "sum")
    close(ops.streams_expand(dev(y), S).cpu(), np.stack([y] * S), 1e-7, "copies")


# ----------------------------------------------------------------------------- row-wise
@pytest.mark.parametrize("H,Dv", [(3, 20), (1, 130), (6, 64)])
def test_read_outs_normed_together_with_a_sigmoid_gate(ops, H, Dv):
    rng = np.random.default_rng(Dv)
    o = rng.normal(size=(6, H * Dv)) * 4
    g = rng.normal(size=(6, H * Dv)) * 2
    w = rng.normal(size=H * Dv)
    got = ops.gated_rmsnorm(dev(o), dev(g), dev(w), 1, H * Dv, 1e-5, torch.float32, gate_activation="sigmoid")
    close(got.cpu(), G.rms_norm(o, w, 1e-5) * G.sigmoid(g), 3e-6, "row norm")
    # head by head with a weight a channel of the row
    got = ops.gated_rmsnorm(dev(o), dev(g), dev(w), H, Dv, 1e-5, torch.float32, gate_activation="sigmoid")
    want = (G.rms_div(o.reshape(6, H, Dv), 1e-5)).reshape(6, -1) * w * G.sigmoid(g)
    close(got.cpu(), want, 3e-6, "head norm, full weight")


def test_silu_in_place_on_a_view(ops):
    rng = np.random.default_rng(4)
    x = rng.normal(size=(9, 37)) * 3
    buf = dev(x)
    ops.act_rows_(buf[:, :30])
    close(buf[:, :30].cpu(), G.silu(x[:, :30]), 3e-6, "silu")
    assert np.array_equal(buf[:, 30:].cpu().numpy(), x[:, 30:].astype(np.float32))


@pytest.mark.parametrize("limit", [0.3, 1.5, 50.0])
def test_clamped_gate(ops, limit):
    rng = np.random.default_rng(int(limit * 10))
    F = 45
    gu = rng.normal(size=(7, 2 * F)) * 2
    gu[0, :4] = [limit, limit * 1.01, -limit * 3, 9.0]
    gu[0, F:F + 4] = [limit * 1.5, -limit * 1.5, limit, -limit]
    g, u = np.minimum(gu[:, :F], limit), np.clip(gu[:, F:], -limit, limit)
    want = g * G.sigmoid(1.702 * g) * (u + 1.0)
    close(ops.gate_mul(dev(gu), "clamped_swish", limit).cpu(), want, 3e-6, "clamped gate")
    got = ops.gate_mul(dev(gu), "clamped_swish", limit, out_dtype=torch.bfloat16)
    close(got.float().cpu(), want, 1e-2, "clamped gate to bfloat16")


@pytest.mark.parametrize("T", [3, 40, 700])
@pytest.mark.parametrize("E,F", [(64, 96), (128, 1024), (40, 20)])
def test_clamped_gate_in_the_products_epilogue(ops, T, E, F):
    """The gate-and-up product with the clamped gate, by the skinny, the split and the tile kernels (and,
    for sizes the matrix cores do not take, the 32-bit product with the gate's own kernel)."""
    rng = np.random.default_rng(T + F)
    b16 = lambda x: torch.tensor(x, dtype=torch.float32).to(torch.bfloat16)
    h, w = b16(rng.normal(size=(T, E))), b16(rng.normal(size=(2 * F, E)) * 0.4)
    limit = 1.3
    z = h.double().numpy() @ w.double().numpy().T
    g, u = np.minimum(z[:, :F], limit), np.clip(z[:, F:], -limit, limit)
    want = g * G.sigmoid(1.702 * g) * (u + 1.0)
    assert (z[:, :F] > limit).any() and (np.abs(z[:, F:]) > limit).any()
    for packed in (False, True):
        wd = w.to(DEV)
        got = ops.linear_gated(h.to(DEV), ops.pack_weight(wd, gated=True) if packed else wd, activation="clamped_swish", param=limit)
        close(got.float().cpu(), want, 1.5e-2, f"packed {packed}")
    got = ops.linear_gated(h.float().to(DEV), w.float().to(DEV), activation="clamped_swish", param=limit)
    close(got.cpu(), want, 5e-6, "float32")


# ----------------------------------------------------------------------------- experts
@pytest.mark.parametrize("n,top,E", [(6, 2, 40), (3, 1, 17), (4, 4, 64), (70, 5, 33), (40, 33, 24)])
def test_routing(ops, n, top, E):
    rng = np.random.default_rng(n * 10 + top)
    T = 50
    h = rng.normal(size=(T, E))
    router = rng.normal(size=(n, E)) * 0.4
    corr = rng.normal(size=n) * 0.3             # as large as the scores: the choice is not the largest scores
    # rows whose scores tie exactly: all logits equal (the lower index wins), and two equal experts
    h[0] = 0.0
    router[1] = router[0]
    corr[1] = corr[0]
    chosen, weights = G.route(h, router, corr, top)
    plain_top, _ = G.route(h, router, np.zeros(n), top)
    assert n == top or (np.sort(chosen, -1) != np.sort(plain_top, -1)).any(), "the correction decides nothing in this case"
    idx, wts = ops.moe_route(dev(h), dev(router), dev(corr), top)
    assert np.array_equal(idx.cpu().numpy(), chosen), "choice"
    close(wts.cpu(), weights, 5e-6, "weights")
    close(wts.sum(-1).cpu(), np.ones(T), 1e-6, "weights add up to one")
    # scores that are no numbers (the row of no request) still name experts that exist
    idx, wts = ops.route_logits(torch.full((3, n), float("nan"), device=DEV), dev(corr), top)
    assert int(idx.min()) >= 0 and int(idx.max()) < n


@pytest.mark.parametrize("T,G,N,K,aw,ow", [(5, 3, 24, 16, 16, 40), (40, 2, 48, 32, 48, 48), (150, 4, 16, 64, 72, 16), (7, 2, 5, 6, 6, 9)])
def test_products_head_by_head_in_one_launch(ops, T, G, N, K, aw, ow):
    """Column ranges of wider rows through a matrix a head into column ranges of wider rows; what lies
    between the ranges stays as it is.  The last case has sizes the matrix cores do not take."""
    rng = np.random.default_rng(T + G)
    b16 = lambda x: torch.tensor(x, dtype=torch.float32).to(torch.bfloat16)
    a = b16(rng.normal(size=(T, (G - 1) * aw + K + 8)))
    w = b16(rng.normal(size=(G, N, K)) * 0.3)
    out = torch.full((T, (G - 1) * ow + N + 3), 7.0, dtype=torch.bfloat16, device=DEV)
    ops.heads_linear(a.to(DEV), w.to(DEV), out, G, aw, ow)
    got = out.float().cpu().numpy()
    covered = np.zeros(got.shape[1], dtype=bool)
    for g in range(G):
        want = a[:, g * aw:g * aw + K].double().numpy() @ w[g].double().numpy().T
        close(got[:, g * ow:g * ow + N], want, 1e-2, f"head {g}")
        covered[g * ow:g * ow + N] = True
    assert (got[:, ~covered] == 7.0).all()


@pytest.mark.parametrize("n,top,E,F,T", [(6, 2, 64, 24, 70), (16, 3, 128, 80, 300), (4, 4, 32, 8, 33), (4, 2, 192, 136, 300), (3, 1, 256, 128, 700)])
def test_experts_over_many_rows_on_the_matrix_cores(ops, n, top, E, F, T):
    rng = np.random.default_rng(n + T)
    r16 = (lambda a: torch.tensor(a, dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy())
    h, router, corr = r16(rng.normal(size=(T, E))), r16(rng.normal(size=(n, E)) * 0.4), rng.normal(size=n) * 0.2
    router[n - 1] = 0.0
    corr[n - 1] = -100.0                       # an expert that nobody takes (unless every expert is taken)
    w = {"router": router, "correction": corr}
    for e in range(n):
        w[f"e{e}.up"], w[f"e{e}.down"] = r16(rng.normal(size=(F, E)) * 0.3), r16(rng.normal(size=(E, F)) * 0.3)
    want = G.moe_ff(h, w, n, top)
    up = dev(np.stack([w[f"e{e}.up"] for e in range(n)]), torch.bfloat16)
    down = dev(np.stack([w[f"e{e}.down"] for e in range(n)]), torch.bfloat16)
    assert T * top >= ops.GROUPED_EXPERTS_FROM
    idx, wts = ops.moe_route(dev(h, torch.bfloat16), dev(router, torch.bfloat16), dev(corr), top)
    assert np.array_equal(idx.cpu().numpy(), G.route(h, router, corr, top)[0])
    y = ops.moe_experts(dev(h, torch.bfloat16), up, down, idx, wts)
    close(y.cpu(), want, 2e-2, "experts, sorted")
    base = rng.normal(size=(T, E))
    acc = dev(base)
    ops.moe_experts(dev(h, torch.bfloat16), up, down, idx, wts, out=acc, accumulate=True)
    close(acc.cpu(), base + want, 2e-2, "experts added to rows")


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 5e-6), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("n,top,E,F", [(6, 2, 40, 24), (3, 1, 17, 5), (4, 4, 64, 96)])
def test_experts(ops, n, top, E, F, dtype, tol):
    rng = np.random.default_rng(n + E)
    T = 21
    r16 = (lambda a: torch.tensor(a, dtype=torch.float32).to(dtype).to(torch.float64).numpy())
    h, router, corr = r16(rng.normal(size=(T, E))), r16(rng.normal(size=(n, E)) * 0.4), rng.normal(size=n) * 0.2
    w = {"router": router, "correction": corr}
    for e in range(n):
        w[f"e{e}.up"], w[f"e{e}.down"] = r16(rng.normal(size=(F, E)) * 0.3), r16(rng.normal(size=(E, F)) * 0.3)
    want = G.moe_ff(h, w, n, top)
    up = dev(np.stack([w[f"e{e}.up"] for e in range(n)]), dtype)
    down = dev(np.stack([w[f"e{e}.down"] for e in range(n)]), dtype)
    idx, wts = ops.moe_route(dev(h, dtype), dev(router, dtype), dev(corr), top)
    y = ops.moe_experts(dev(h, dtype), up, down, idx, wts)
    close(y.cpu(), want, tol, "experts")
    base = rng.normal(size=(T, E))
    acc = dev(base)
    ops.moe_experts(dev(h, dtype), up, down, idx, wts, out=acc, accumulate=True)
    close(acc.cpu(), base + want, tol, "experts added to rows")


# ----------------------------------------------------------------------------- lightning attention's recurrence
def test_a_far_write_is_kept_by_a_head_that_does_not_decay(ops):
    """Token 2 writes a value of its own along a key that every later query reads; 500 tokens later
    the head with decay 1 still returns it whole, the head with decay 0.5 has lost it.  In portions
    and single tokens, from a state row that starts as garbage but for the request's own."""
    from xyntetik_runner_amd.csrc.ops import Ops
    H, D, Dv, n = 2, 12, 5, 520
    rng = np.random.default_rng(8)
    q = np.zeros((n, H, D)); k = rng.normal(size=(n, H, D)) * 0.01; v = rng.normal(size=(n, H, Dv))
    q[:, :, 0] = 1.0
    k[:, :, 0] = 0.0
    k[2, :, 0] = 1.0
    v[2] = 100.0
    decay = [1.0, 0.5]
    want = np.zeros((n, H, Dv))
    for hd in range(H):
        Sm = np.zeros((D, Dv))
        for t in range(n):
            Sm = decay[hd] * Sm + np.outer(k[t, hd], v[t, hd])
            want[t, hd] = Sm.T @ q[t, hd]
    assert want[-1, 0, 0] > 99 and abs(want[-1, 1, 0]) < 1
    state = torch.full((3,) + Ops.recurrence_state_shape(H, D, Dv), float("nan"), device=DEV)
    state[1] = 0.0
    got = np.zeros((n, H, Dv))
    for i, m in cuts(n, [40, 1, 1, 300, 2, 1]):
        ctx = step_ctx([i], [m], [1])
        row = dev(np.concatenate([q[i:i + m].reshape(m, -1), k[i:i + m].reshape(m, -1), v[i:i + m].reshape(m, -1)], axis=1))
        o = ops.linear_recurrence("retention", row[:, :H * D], row[:, H * D:2 * H * D], row[:, 2 * H * D:], state, ctx, H, H, D, Dv,
                                  decay=dev(decay))
        got[i:i + m] = o.cpu().numpy().reshape(m, H, Dv)
    close(got, want, 5e-6, "far write")


@pytest.mark.parametrize("H,D,Dv", [(2, 12, 5), (3, 64, 32)])
def test_recurrence_applies_silu_as_it_reads(ops, H, D, Dv):
    """q, k and v through SiLU inside the recurrence kernel: the same read-outs as from rows that passed it before."""
    from xyntetik_runner_amd.csrc.ops import Ops
    rng = np.random.default_rng(D)
    n = 45
    row = rng.normal(size=(n, 2 * H * D + H * Dv)) * 1.5
    decay = dev(rng.uniform(0.5, 1.0, size=H))
    outs = []
    for fused in (True, False):
        state = torch.zeros((2,) + Ops.recurrence_state_shape(H, D, Dv), device=DEV)
        got = []
        for i, m in cuts(n, [20, 1, 1, 17, 2, 4]):
            ctx = step_ctx([i], [m], [0])
            r = dev(row[i:i + m])
            if not fused:
                ops.act_rows_(r)
            got.append(ops.linear_recurrence("retention", r[:, :H * D], r[:, H * D:2 * H * D], r[:, 2 * H * D:], state, ctx, H, H, D, Dv,
                                             decay=decay, activation="silu" if fused else None).cpu().numpy())
        outs.append(np.concatenate(got))
    close(outs[0], outs[1], 2e-6, "silu in the recurrence")


# ----------------------------------------------------------------------------- one-layer models with made weights
def needle_model(window, rot_dim=4, heads=2):
    """A latent-attention layer whose token 1 (the needle) has a key along every query, with a score
    far above the fillers' (token 0), and a value that lands in logit 2; the rotated parts are small."""
    E, Q, C, D, Dv, V = 8, 6, 6, 4, 3, 4
    rng = np.random.default_rng(window or 999)
    m = {"heads": heads, "dim": D, "rot_dim": rot_dim, "vdim": Dv, "q_rank": Q, "kv_rank": C, "scale": 1.0,
         "rot": {"dims": rot_dim, "base": 100.0}}
    if window:
        m["mask"] = {"size": window}
    cfg = {"architecture": "Sugosun", "vocab": V, "width": E, "norm": {"eps": 1e-6},
           "layers": [{"type": "latent_attention", "mixer": m, "mlp": None}]}
    w = {}
    emb = np.zeros((V, E)); emb[0, 1] = 1.0; emb[1, 0] = 1.0; emb[2, 2] = 1.0; emb[3, 3] = 1.0
    w["embed"], w["embed.norm"] = emb, np.ones(E)
    w["l0.norm1"], w["final.norm"] = np.ones(E), np.ones(E)
    dq = rng.normal(size=(Q, E)) * 0.01; dq[0, :] += 0.5             # every token's query latent has channel 0
    dkv = rng.normal(size=(C + rot_dim, E)) * 0.01
    dkv[0, 0] = 1.0                                                   # the needle's latent lies along channel 0
    dkv[1, 1] = 1.0                                                   # a filler's along channel 1
    dkv[C:] *= 0.1
    uq = rng.normal(size=(heads * (D + rot_dim), Q)) * 0.01
    uk = rng.normal(size=(heads * D, C)) * 0.01
    uv = rng.normal(size=(heads * Dv, C)) * 0.01
    for hd in range(heads):
        uq[hd * (D + rot_dim), 0] = 6.0                               # query channel 0 of every head is large
        uk[hd * D, 0] = 3.0                                           # and reads latent channel 0
        uv[hd * Dv, 0] = 1.0                                          # the needle's value: channel 0 of the head
    o = rng.normal(size=(E, heads * Dv)) * 0.01
    o[4, 0] = 2.0
    head = rng.normal(size=(V, E)) * 0.01
    head[2, 4] = 1.0
    w.update({"l0.mix.dq": dq, "l0.mix.dq.norm": np.ones(Q), "l0.mix.uq": uq, "l0.mix.dkv": dkv, "l0.mix.dkv.norm": np.ones(C),
              "l0.mix.uk": uk, "l0.mix.uv": uv, "l0.mix.o": o, "head": head})
    return cfg, w


def engine_logits(cfg, w, steps, dtype, page, max_tokens, tmp_path):
    from xyntetik_runner_amd.config import config_from_dict
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    arch, typed = config_from_dict(cfg)
    tensors = {k: torch.tensor(v, dtype=torch.float32) for k, v in w.items()}
    runner = ModelRunner(arch.build_spec(typed), tensors, dtype, max_tokens=max_tokens, page_size=page, max_requests=2)
    for lc in runner.storage.layers:
        if lc.owns and lc.k is not None:
            lc.k.fill_(float("nan")); lc.v.fill_(float("nan"))
    out = str(tmp_path / "out")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    return traces.collect(steps, out, cfg["vocab"])


@pytest.mark.parametrize("window,page", [(9, 8), (16, 16), (33, 8), (64, 64), (65, 64), (1, 4), (None, 16)])
@pytest.mark.parametrize("decode_from", [None, 30])
def test_one_latent_that_stands_out_at_every_distance(tmp_path, window, page, decode_from):
    """The needle at position j*: every later query sees it (logit 2 is high) up to distance
    window - 1 and not at distance window; without a window, 600 tokens later among hundreds of
    fillers.  In a prompt's portions and with the last positions decoded one by one."""
    cfg, w = needle_model(window)
    n = 150 if window else 640
    for jstar in (3, 29):
        toks = [0] * n
        toks[jstar] = 1
        want = G.forward(cfg, w, toks)
        seen = want[:, 2] - want[:, 3]
        if window:
            assert seen[jstar + window - 1] > 1.0 and seen[jstar + window] < 0.3, "the made weights do not show the window's edge"
        else:
            assert seen[-1] > 1.0
        if decode_from is None:
            steps = traces.portions({"a": toks}, sizes=(17, 2, 40, 3))
        else:
            steps = traces.tail_one_by_one({"a": toks}, tail=n - decode_from)
        got = engine_logits(cfg, w, steps, "float32", page, -(-n // 64) * 64 + 64, tmp_path / f"{jstar}")
        close(got["a"], want, 1e-5, f"needle at {jstar}")


def test_first_tokens_of_a_sequence(tmp_path):
    """Sequences of one, two and three tokens, and the first rows of a longer one: the extra row of
    the pair table, a window that is not full yet, a state that starts at zero."""
    from sugosun_tiny import TINY_G1
    from plain_llama import load_folder
    from xyntetik_runner_amd.weights import write_random_model
    d = write_random_model(TINY_G1, str(tmp_path / "m"), seed=5, std=0.12, norm_jitter=0.1)
    cfg, w = load_folder(d)
    reqs = {f"r{n}": [int(t) for t in np.random.default_rng(n).integers(0, cfg["vocab"], size=n)] for n in (1, 2, 3, 30)}
    steps = traces.mixed(reqs, {k: min(2, len(v)) for k, v in reqs.items()}, max_live=4, seed=1)
    from xyntetik_runner_amd.engine.runner import ModelRunner
    from xyntetik_runner_amd.trace import replay
    runner = ModelRunner.from_folder(d, dtype="float32", max_tokens=256, page_size=16, max_requests=4)
    out = str(tmp_path / "out")
    replay(runner, traces.to_lines(steps), out, report=io.StringIO())
    got = traces.collect(steps, out, cfg["vocab"])
    for rid, toks in reqs.items():
        close(got[rid], G.forward(cfg, w, toks), 2e-5, rid)
