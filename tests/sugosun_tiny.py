"""Small Sugosun configurations for the tests, each with sizes and constants of its own.

Between them they differ in everything config.json gives: width, vocabulary, the order of the
mixers, heads, key and value sizes (multiples of 8 and 16 and not), latent sizes, the rotated part
(whole, a part of it, two channels), windows (longer than a page, one, none), residual streams
(three, two, one, none), the pair table (present with equal and unequal multipliers, absent), the
looped span (a part, the whole model, once, none), feed-forwards (dense with a limit that clamps
and one that does not, experts with one, some and all chosen, none), eps.
"""


def lightning(heads, dim, vdim, decay):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, size=None, dims=None, base=10000.0):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
         "rot": {"dims": rot_dim if dims is None else dims, "base": base}}
    if size is not None:
        m["mask"] = {"size": size}
    return {"type": "latent_attention", "mixer": m}


def dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def moe(ff, experts, top):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def with_ff(layer, mlp):
    out = dict(layer)
    out["mlp"] = mlp
    return out


# three streams, a pair table, the middle two layers three times; sizes the matrix kernels take in
# bfloat16; a window that is no multiple of anything; a layer without a feed-forward
TINY_G1 = {
    "architecture": "Sugosun", "vocab": 200, "width": 64, "norm": {"eps": 1e-5}, "streams": 3,
    "embedding": {"bigram": {"buckets": 53, "mul_prev": 17, "mul_cur": 5}},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        with_ff(latent(4, 16, 16, 24, 40, 48, 0.2, size=21, base=1000.0), moe(40, 6, 2)),
        with_ff(lightning(2, 32, 16, [0.9, 0.995]), dense(72, 0.8)),
        with_ff(latent(2, 32, 16, 16, 48, 48, 0.15, size=21, dims=8), None),
        with_ff(lightning(4, 16, 16, [0.5, 0.8, 0.95, 1.0]), moe(24, 5, 3)),
    ],
}

# the plain residual sum, no pair table, no loop, no window; sizes that are multiples of nothing;
# a part of the rotated channels turns; one expert a token; a limit that never clamps
TINY_G2 = {
    "architecture": "Sugosun", "vocab": 97, "width": 40, "norm": {"eps": 1e-6},
    "layers": [
        with_ff(lightning(3, 10, 6, [0.7, 0.9, 0.97]), moe(20, 3, 1)),
        with_ff(latent(2, 6, 6, 5, 12, 10, 0.4, dims=4, base=50.0), dense(56, 30.0)),
        with_ff(latent(3, 5, 2, 7, 9, 13, 0.3, size=9), None),
        with_ff(lightning(1, 12, 20, [0.96]), dense(24, 0.3)),
    ],
}

# one stream with connection weights; equal multipliers; the whole model looped twice; a window of
# one and a window of a page; all experts chosen; rows of 64 and 80 channels for the matrix-core attention
TINY_G3 = {
    "architecture": "Sugosun", "vocab": 256, "width": 96, "norm": {"eps": 1e-5}, "streams": 1,
    "embedding": {"bigram": {"buckets": 31, "mul_prev": 3, "mul_cur": 3}},
    "loop": {"start": 0, "stop": 3, "times": 2},
    "layers": [
        with_ff(latent(4, 32, 16, 32, 64, 64, 0.12, size=64, base=250000.0), moe(48, 4, 4)),
        with_ff(latent(2, 16, 32, 48, 32, 32, 0.2, size=1), dense(128, 1.2)),
        with_ff(lightning(2, 64, 32, [0.97, 0.999]), moe(32, 8, 2)),
    ],
}

# two streams, a span looped once (as good as none), windows over pages of 64 in a deep run order
TINY_G4 = {
    "architecture": "Sugosun", "vocab": 128, "width": 64, "norm": {"eps": 1e-6}, "streams": 2,
    "embedding": {"bigram": {"buckets": 127, "mul_prev": 1000003, "mul_cur": 999983}},
    "loop": {"start": 2, "stop": 3, "times": 1},
    "layers": [
        with_ff(lightning(2, 32, 32, [0.9, 0.99]), dense(96, 1.0)),
        with_ff(latent(4, 16, 16, 16, 32, 64, 0.25, size=70), moe(32, 4, 2)),
        with_ff(latent(4, 16, 16, 16, 32, 64, 0.25, size=130), moe(32, 4, 2)),
    ],
}

# a cached row longer than the matrix-core attention takes (272 + 32 channels): the 32-bit attention kernel
# on bfloat16 storage; one expert in all; a single head
TINY_G5 = {
    "architecture": "Sugosun", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "streams": 2,
    "layers": [
        with_ff(latent(1, 24, 32, 40, 24, 272, 0.1, size=40), moe(16, 1, 1)),
        with_ff(lightning(2, 8, 24, [0.9, 0.8]), None),
    ],
}

# the plain residual sum with a pair table; attention without a rotated part, and with two rotated channels
# of which none turns; a single expert chosen of two
TINY_G6 = {
    "architecture": "Sugosun", "vocab": 50, "width": 32, "norm": {"eps": 1e-6},
    "embedding": {"bigram": {"buckets": 11, "mul_prev": 0, "mul_cur": 1}},
    "layers": [
        with_ff(latent(2, 8, 0, 8, 16, 24, 0.3, size=5), moe(8, 2, 1)),
        with_ff(lightning(2, 4, 4, [0.0, 1.0]), dense(16, 1.0)),
        with_ff(latent(1, 8, 2, 4, 8, 6, 0.5, dims=0), None),
    ],
}

CONFIGS = {"G1": (TINY_G1, 21), "G2": (TINY_G2, 22), "G3": (TINY_G3, 23), "G4": (TINY_G4, 24), "G5": (TINY_G5, 25),
           "G6": (TINY_G6, 26)}


def make_model(which: str, folder: str, std: float = 0.12) -> str:
    from xyntetik_runner_amd.weights import write_random_model
    config, seed = CONFIGS[which]
    return write_random_model(config, folder, seed=seed, std=std, norm_jitter=0.1, dtype="bfloat16")
