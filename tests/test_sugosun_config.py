"""Sugosun without a GPU: the config's refusals by key, the spec it builds, the cache groups and
pool sizes of its layers, and the plain mechanisms against closed forms."""
import copy

import numpy as np
import pytest

import plain_sugosun as G
from sugosun_tiny import TINY_G1, TINY_G2, TINY_G3


def parse(raw):
    from xyntetik_runner_amd.config import config_from_dict
    arch, cfg = config_from_dict(raw)
    return arch, cfg


def test_config_reads_every_size_and_constant():
    arch, cfg = parse(TINY_G1)
    assert arch.name == "Sugosun" and cfg.vocab == 200 and cfg.width == 64 and cfg.eps == 1e-5 and cfg.streams == 3
    assert (cfg.bigram.buckets, cfg.bigram.mul_prev, cfg.bigram.mul_cur) == (53, 17, 5)
    assert cfg.loop == (1, 3, 3) and cfg.run_order() == (0, 1, 2, 1, 2, 1, 2, 3)
    a, l = cfg.layers[0].mixer, cfg.layers[1].mixer
    assert (a.kind, a.heads, a.dim, a.rot_dim, a.vdim, a.q_rank, a.kv_rank, a.scale, a.window, a.rot_dims, a.rot_base) == \
        ("latent_attention", 4, 16, 16, 24, 40, 48, 0.2, 21, 16, 1000.0)
    assert (l.kind, l.heads, l.dim, l.vdim, l.decay) == ("lightning", 2, 32, 16, (0.9, 0.995))
    assert cfg.layers[2].mlp is None and cfg.layers[2].mixer.rot_dims == 8
    m = cfg.layers[0].mlp
    assert (m.kind, m.ff, m.experts, m.top) == ("moe", 40, 6, 2)
    d = cfg.layers[1].mlp
    assert (d.kind, d.ff, d.limit) == ("dense", 72, 0.8)
    _, c2 = parse(TINY_G2)
    assert c2.streams is None and c2.bigram is None and c2.loop is None and c2.run_order() == (0, 1, 2, 3)
    assert c2.layers[1].mixer.window is None
    _, c3 = parse(TINY_G3)
    assert c3.run_order() == (0, 1, 2, 0, 1, 2) and c3.streams == 1


@pytest.mark.parametrize("path,value,word", [
    (("layers", 0, "type"), "attention", "type"),
    (("layers", 0, "mixer", "heads"), 0, "heads"),
    (("layers", 0, "mixer", "rot", "dims"), 7, "rot.dims"),
    (("layers", 0, "mixer", "rot", "dims"), 18, "rot.dims"),
    (("layers", 0, "mixer", "scale"), "big", "scale"),
    (("layers", 1, "mixer", "decay"), [0.5], "decay"),
    (("layers", 1, "mixer", "decay"), [0.5, 1.5], "decay"),
    (("layers", 0, "mlp", "router", "top"), 7, "top"),
    (("layers", 0, "mlp", "kind"), "sparse", "kind"),
    (("layers", 1, "mlp", "limit"), 0.0, "limit"),
    (("loop", "stop"), 0, "stop"),
    (("loop", "stop"), 5, "stop"),
    (("loop", "times"), 0, "times"),
    (("streams",), 0, "streams"),
    (("embedding", "bigram", "buckets"), 0, "buckets"),
    (("norm", "eps"), -1.0, "eps"),
    (("vocab",), None, "vocab"),
])
def test_config_refuses_by_key(path, value, word):
    from xyntetik_runner_amd.config import ConfigError
    raw = copy.deepcopy(TINY_G1)
    at = raw
    for p in path[:-1]:
        at = at[p]
    at[path[-1]] = value
    with pytest.raises(ConfigError) as e:
        parse(raw)
    assert word in str(e.value)


def test_spec_cache_groups_and_pools():
    from xyntetik_runner_amd.cache import cache_groups, size_pools
    from xyntetik_runner_amd.engine.model import Model
    arch, cfg = parse(TINY_G1)
    spec = arch.build_spec(cfg)
    assert spec.streams == 3 and len(spec.order) == 8 and all(st.cache_of is None for st in spec.order)
    model = Model(spec)
    kv, st, of = model.cache_needs()
    # both attention layers cache one row of 64 channels a token behind a window of 21: one group, four owners
    specs, owners = cache_groups(kv, of)
    assert len(specs) == 1 and specs[0].num_kv_heads == 1 and specs[0].head_dim == 64 and specs[0].window == 21
    sizes = size_pools(specs, owners, 16, 2, 3, 40, max_tokens=512)
    assert sizes[0] == 3 * (-(-21 // 16) + 2) + -(-40 // 16)          # a window's pages a request, not the requests' lengths
    exp = model.expected()
    assert exp["bigram"].shape == (54, 64) and exp["l0.hc1.mix"].shape == (3, 3) and exp["l0.mlp.e5.down"].shape == (64, 40)
    assert exp["l0.mix.dkv"].shape == (64, 64) and exp["l0.mix.uq"].shape == (4 * 32, 40) and exp["l1.mix.norm"].shape == (32,)


def test_plain_mechanisms_against_closed_forms():
    rng = np.random.default_rng(0)
    # pair rows: the first token reads the extra row, the others the hash of (before, token)
    assert list(G.bigram_rows([5, 7, 7], 11, 3, 2)) == [11, (5 * 3 + 7 * 2) % 11, (7 * 3 + 7 * 2) % 11]
    # rotation: lengths are kept, position 0 is the identity, pairs are (2i, 2i + 1)
    x = rng.normal(size=(4, 3, 8))
    r = G.rotate_pairs(x, [0, 1, 2, 50], 6, 100.0)
    assert np.allclose(r[0], x[0]) and np.allclose(r[..., 6:], x[..., 6:])
    assert np.allclose(np.hypot(r[..., 0], r[..., 1]), np.hypot(x[..., 0], x[..., 1]))
    a = 2 * 100.0 ** (-2.0 / 6)
    assert np.allclose(r[2, 0, 2], x[2, 0, 2] * np.cos(a) - x[2, 0, 3] * np.sin(a), atol=1e-6)
    # lightning with decay 1 and one head: the read-out is a causal sum of (q . k_j) v_j
    E, D, Dv, T = 6, 4, 3, 5
    w = {"q": rng.normal(size=(D, E)), "k": rng.normal(size=(D, E)), "v": rng.normal(size=(Dv, E)), "g": rng.normal(size=(Dv, E)),
         "o": np.eye(E, Dv), "norm": np.ones(Dv)}
    h = rng.normal(size=(T, E))
    q, k, v = G.silu(h @ w["q"].T), G.silu(h @ w["k"].T), G.silu(h @ w["v"].T)
    o = np.stack([sum((q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(T)])
    want = (G.rms_norm(o, 1.0, 1e-6) * G.sigmoid(h @ w["g"].T)) @ w["o"].T
    assert np.allclose(G.lightning(h, w, {"heads": 1, "dim": D, "vdim": Dv, "decay": [1.0]}, 1e-6), want)
    # routing: weights of the chosen add up to one; with every expert chosen they are the softmax itself
    hh, router = rng.normal(size=(7, E)), rng.normal(size=(4, E))
    idx, wt = G.route(hh, router, np.zeros(4), 4)
    assert np.allclose(wt.sum(-1), 1) and np.allclose(np.take_along_axis(G.softmax(hh @ router.T), idx, -1), wt)
    idx, wt = G.route(hh, router, np.array([0, 0, 0, 100.0]), 1)
    assert (idx == 3).all() and np.allclose(wt, 1)
    # the clamped gate at its corners
    one = np.ones((1, 1))
    f = lambda g, u, L: G.dense_ff(np.array([[g, u]]), {"gate": np.array([[1.0, 0]]), "up": np.array([[0, 1.0]]), "down": one}, L)[0, 0]
    assert np.isclose(f(5.0, 9.0, 2.0), 2.0 * G.sigmoid(3.404) * 3.0) and np.isclose(f(-5.0, -9.0, 2.0), -5.0 * G.sigmoid(-8.51) * -1.0)
    # streams: with in = out = 1 and mix = identity, one stream is the plain residual sum
    cfg = copy.deepcopy(TINY_G2)
    cfg["layers"] = cfg["layers"][:1]
    from xyntetik_runner_amd.weights.random_init import random_state
    from xyntetik_runner_amd.engine.model import Model
    arch, typed = parse(cfg)
    wts = {k: v.double().numpy() for k, v in random_state(Model.expected_tensors(arch.build_spec(typed)), 3, std=0.1, dtype="float32").items()}
    toks = [3, 9, 9, 50, 1]
    base = G.forward(cfg, wts, toks)
    cfg1 = dict(cfg, streams=1)
    for q in (1, 2):
        wts[f"l0.hc{q}.in"], wts[f"l0.hc{q}.out"], wts[f"l0.hc{q}.mix"] = np.ones(1), np.ones(1), np.ones((1, 1))
    assert np.allclose(G.forward(cfg1, wts, toks), base)
