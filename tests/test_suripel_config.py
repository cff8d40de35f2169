"""Host logic of the Suripel design, no GPU: the typed configuration and its refusals, the model
as data (parts, run order, expected tensors, what the cache must keep), cache groups with a
stride in the manager and in the sizing, and the plain implementation's own mechanisms against
closed forms."""
import copy

import numpy as np
import pytest

import plain_suripel as S
from suripel_tiny import TINY_S1, TINY_S2, TINY_S3


def build(raw):
    from xyntetik_runner_amd.config import config_from_dict
    arch, cfg = config_from_dict(raw)
    return arch, cfg, arch.build_spec(cfg)


def test_config_is_read_key_by_key():
    arch, cfg, spec = build(TINY_S1)
    assert arch.name == "Suripel" and cfg.vocab == 131 and cfg.width == 48 and cfg.canon_taps == 3 and cfg.eps == 1e-5
    kinds = [l.mixer.kind for l in cfg.layers]
    assert kinds == ["delta", "attention", "retention", "attention", "retention"]
    a = cfg.layers[1].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.pool, a.conv, a.scale) == (4, 2, 16, 24, 9, 5, 3, 0.31)
    assert cfg.layers[3].mixer.kv_from == 1 and cfg.layers[2].ff is None and cfg.layers[0].ff == 72
    r = cfg.layers[2].mixer
    assert r.decay == (0.9, 0.97, 0.995) and (r.rot_dims, r.rot_base) == (8, 500.0)
    assert cfg.layers[4].mixer.rot_dims == 0
    assert [st.cache_of for st in spec.order] == [None, None, None, 1, None]


def test_parts_get_their_constants_from_the_config():
    _, cfg, spec = build(TINY_S2)
    m = spec.layers[0].mixer
    assert m.kind == "pooled_window_attention" and m.params["window"] == 4 and m.params["pool"] == 8 and m.params["keep"] == 8
    assert spec.layers[2].mixer.params["pool"] == 0 and spec.layers[2].mixer.params["conv_taps"] == 0
    assert spec.layers[0].mixer.params["conv_taps"] == 1 and spec.layers[4].mixer.params["conv_taps"] == 0
    assert spec.layers[1].mixer.kind == "gated_delta" and spec.layers[1].mixer.params["num_kv_heads"] == 1
    assert spec.layers[3].mixer.params["position"].params == {"head_dim": 6, "theta": 10000.0, "rotary_dim": 6}
    assert spec.layers[0].filters["mixer_filter"].params["taps"] == 2
    assert spec.layers[0].feed_forward.params["eps"] == 1e-6 and spec.final_norm.params["eps"] == 1e-6


def test_an_owners_cache_reaches_as_far_as_its_readers():
    _, cfg, spec = build(TINY_S3)
    # layer 0 (window 40, blocks of 16) is read by layers 2 (24, 8) and 5 (52, 16)
    assert [spec.layers[i].mixer.params["keep"] for i in (0, 2, 5)] == [52, 52, 52]
    assert spec.layers[4].mixer.params["keep"] == 70


@pytest.mark.parametrize("edit,word", [
    (lambda c: c["layers"][0].update(type="mamba"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(heads=3), "kv_heads"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=0), "kv_from"),          # names a delta layer
    (lambda c: c["layers"][3]["mixer"].update(dim=8), "differ"),
    (lambda c: c["layers"][2]["mixer"].update(decay=[0.9, 0.9]), "decay"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mlp"].update(kind="experts"), "kind"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "mask"),
    (lambda c: c["canon"].update(taps=0), "taps"),
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c.update(layers=[]), "layers"),
])
def test_a_config_that_cannot_be_built_is_refused_by_name(edit, word):
    from xyntetik_runner_amd.config import ConfigError
    raw = copy.deepcopy(TINY_S1)
    edit(raw)
    with pytest.raises(ConfigError) as e:
        build(raw)
    assert word in str(e.value)


def test_expected_tensors_and_cache_needs():
    from xyntetik_runner_amd.engine.model import Model
    _, cfg, spec = build(TINY_S3)
    exp = Model.expected_tensors(spec)
    assert exp["l0.mix.q"].shape == (128, 64) and exp["l0.mix.k.conv"].shape == (64, 4) and exp["l0.canon2"].shape == (64, 4)
    assert exp["l3.mix.A_log"].shape == (2,) and exp["l3.mix.norm"].shape == (64,) and exp["l3.mix.b"].shape == (2, 64)
    assert exp["l1.mix.g"].shape == (32, 64) and exp["l0.mlp.act"].shape == (4,) and exp["head"].shape == (256, 64)
    assert "l2.mix.v" not in exp and "l5.mix.k.conv" not in exp
    kv, st, of = Model(spec).cache_needs()
    from xyntetik_runner_amd.cache import cache_groups
    specs, owners = cache_groups(kv, of)
    # layers 0 and 4 own keys and values; each has a group for its block means; reader 2's blocks
    # (8) differ from its owner's (16), so it keeps means of its own; reader 5 uses the owner's
    assert [(s.window, s.pooled, s.stride) for s in specs] == [(52, 16, 1), (None, None, 16), (None, None, 8), (70, 32, 1), (None, None, 32)]
    assert owners == [1, 1, 1, 1, 1]


def test_a_layer_without_a_feed_forward_loads_with_or_without_its_second_norm():
    import torch
    from xyntetik_runner_amd.engine.model import Model
    from xyntetik_runner_amd.weights.loader import WeightError, check_against
    _, cfg, spec = build(TINY_S1)
    exp = Model.expected_tensors(spec)
    names = [n for n in exp if n not in ("l2.norm2", "l2.canon2")]
    shape, dtype = (lambda n: exp[n].shape), (lambda n: torch.bfloat16)
    check_against(exp, names, shape, dtype)
    check_against(exp, list(exp), shape, dtype)
    with pytest.raises(WeightError):
        check_against(exp, [n for n in names if n != "l1.norm2"], shape, dtype)
    with pytest.raises(WeightError):
        check_against(exp, names + ["l2.mlp.up"], shape, dtype)


def test_manager_with_a_group_of_stride():
    from xyntetik_runner_amd.cache import CacheManager
    from xyntetik_runner_amd.parts import KVSpec
    main = KVSpec(2, 8, window=12, pooled=5)
    mgr = CacheManager([main, main.pooled_spec()], page_size=4, pages_per_group=[9, 3], n_slots=2)
    mgr.admit("a")
    assert mgr.pages_needed_new(23) == [6, 1]                   # 23 positions; 4 complete blocks of 5
    mgr.reserve("a", 23); mgr.advance("a", 23); mgr.check()
    rc = mgr.get("a")
    assert len(rc.tables[0]) == 6 and len(rc.tables[1]) == 1
    assert rc.tables[0][:3] == [-1, -1, -1]                      # positions below 23 - 12 + 1 = 12 are given back
    assert all(p > 0 for p in rc.tables[1])                      # block means are kept while the request lives
    mgr.reserve("a", 25); mgr.advance("a", 25); mgr.check()      # the fifth block completes: a second page of means
    assert len(rc.tables[1]) == 2
    mgr.reserve("a", 41)                                         # a step that reserves and then does not run
    assert len(rc.tables[0]) == 11 and len(rc.tables[1]) == 2
    mgr.trim("a"); mgr.check()
    assert len(rc.tables[0]) == 7 and len(rc.tables[1]) == 2     # what 25 tokens hold
    mgr.release("a")
    assert mgr.all_free()
    assert mgr.capacity_tokens() == 3 * 4 * 5                    # the windowed group sets no limit, the means do


def test_pools_for_a_number_of_tokens():
    from xyntetik_runner_amd.cache import size_pools
    from xyntetik_runner_amd.parts import KVSpec
    main = KVSpec(2, 8, window=40, pooled=16)
    sizes = size_pools([main, main.pooled_spec()], [1, 1], 64, 2, 4, None, max_tokens=1024)
    assert sizes == [16, 1 + 4]                                  # 16 pages of tokens; a 16th of them, and one begun page a request


def test_plain_mechanisms_against_closed_forms():
    # retention of constant inputs is a geometric sum
    T, d = 12, 0.5
    q = np.ones((T, 1, 1)); k = np.ones((T, 1, 1)); v = np.ones((T, 1, 1))
    o = S.retention(q, k, v, [d])[:, 0, 0]
    assert np.allclose(o, [(1 - d ** (t + 1)) / (1 - d) for t in range(T)])
    # the delta rule with beta = 1 and g = 1 stores v under a unit key exactly, and overwrites it
    D = 4
    kk = np.zeros((3, 1, D)); kk[:, 0, 0] = 1.0
    vv = np.array([[[2.0]], [[5.0]], [[-1.0]]])
    o = S.gated_delta_rule(kk, kk, vv, np.ones((3, 1)), np.ones((3, 1)))[:, 0, 0]
    assert np.allclose(o, [2.0, 5.0, -1.0])
    # what a query sees: the window, then blocks that end at least `size` back
    assert S.visible(20, 6, 4) == ([15, 16, 17, 18, 19, 20], [0, 1, 2])        # block 3 = 12..15 ends at 15 > 14
    assert S.visible(21, 6, 4) == ([16, 17, 18, 19, 20, 21], [0, 1, 2, 3])
    assert S.visible(5, 6, 4) == ([0, 1, 2, 3, 4, 5], [])
    assert S.visible(9, 2, 8) == ([8, 9], [0])                                   # 7 <= 9 - 2
    assert S.visible(8, 2, 8) == ([7, 8], [])                                    # positions 0..6 are seen by nobody
    # the convolution's last column is the current token's
    u = np.arange(5.0)[:, None]
    assert np.allclose(S.causal_conv(u, np.array([[0.0, 0.0, 1.0]]))[:, 0], u[:, 0])
    assert np.allclose(S.causal_conv(u, np.array([[1.0, 0.0, 0.0]]))[:, 0], [0, 0, 0, 1, 2])
    # PolyNorm of a constant row: every N is 1 up to eps
    assert np.allclose(S.polynorm(np.full((1, 8), 2.0), [1.0, 10.0, 100.0, 0.5], 0.0), 111.5)
