"""Small Suripel configurations for the tests, each with sizes and constants of its own.

Between them they differ in everything config.json gives: width, vocabulary, feed-forward width
(and a layer without one), the order of the mixers, heads and key heads, key and value sizes
(equal and unequal, multiples of 4 and not), windows and block lengths (a block longer than the
window, a block that does not divide a page, no blocks at all), a reader whose mask differs from
the owner's, taps of the input convolution and of the mixers' convolutions (different from each
other, and 1), rotation over the whole head and over a part of it and none, eps.
"""
import os


def attention(heads, kv_heads, dim, vdim, size, pool, conv, scale, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale,
         "mask": {"size": size, "pool": pool}}
    if not pool:
        del m["mask"]["pool"]
    if not conv:
        del m["conv"]               # no convolution of the projections, and no tensors of one
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def delta(heads, kv_heads, dim, vdim, conv):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}
    if not conv:
        del m["conv"]
    return {"type": "delta", "mixer": m}


def retention(heads, dim, vdim, decay, rot=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}
    if rot:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "retention", "mixer": m}


def with_ff(layer, ff):
    out = dict(layer)
    out["mlp"] = {"kind": "dense", "ff": ff} if ff else None
    return out


# delta first, grouped key heads; attention with unequal key and value sizes and blocks of 5 (no
# divisor of any page); a reader with a shorter window and longer blocks than its owner;
# retention rotating half of each head; a layer without a feed-forward
TINY_S1 = {
    "architecture": "Suripel", "vocab": 131, "width": 48, "norm": {"eps": 1e-5}, "canon": {"taps": 3},
    "layers": [
        with_ff(delta(4, 2, 12, 20, 2), 72),
        with_ff(attention(4, 2, 16, 24, 9, 5, 3, 0.31), 56),
        with_ff(retention(3, 16, 8, [0.9, 0.97, 0.995], rot=(8, 500.0)), None),
        with_ff(attention(4, 2, 16, 24, 6, 7, 2, 0.2, kv_from=1), 72),
        with_ff(retention(2, 10, 24, [0.8, 0.99]), 40),
    ],
}

# attention first; a block longer than the window; attention without blocks; convolutions of one
# tap and mixers without any; key sizes that are no multiples of 4; heads = key heads in attention, one key head in delta
TINY_S2 = {
    "architecture": "Suripel", "vocab": 97, "width": 40, "norm": {"eps": 1e-6}, "canon": {"taps": 2},
    "layers": [
        with_ff(attention(2, 2, 10, 10, 4, 8, 1, 0.4), 64),
        with_ff(delta(3, 1, 7, 9, 4), 48),
        with_ff(attention(3, 1, 8, 6, 11, 0, 0, 0.25), 64),
        with_ff(retention(2, 6, 5, [0.5, 0.9375], rot=(6, 10000.0)), 32),
        with_ff(delta(2, 2, 16, 16, 0), 48),
    ],
}

# sizes the matrix kernels take in bfloat16 (multiples of 8 and 16), pages of 64, blocks of 16
# with a window that is no multiple of them, two owners of which one has two readers
TINY_S3 = {
    "architecture": "Suripel", "vocab": 256, "width": 64, "norm": {"eps": 1e-5}, "canon": {"taps": 4},
    "layers": [
        with_ff(attention(4, 2, 32, 32, 40, 16, 4, 0.18), 96),
        with_ff(retention(2, 32, 16, [0.95, 0.998], rot=(32, 250000.0)), 96),
        with_ff(attention(4, 2, 32, 32, 24, 8, 3, 0.18, kv_from=0), 96),
        with_ff(delta(2, 2, 32, 64, 4), 96),
        with_ff(attention(2, 1, 16, 48, 70, 32, 2, 0.25), 96),
        with_ff(attention(4, 2, 32, 32, 52, 16, 2, 0.1, kv_from=0), 96),
    ],
}

# no attention at all (no cache group, state only), a width that is no multiple of 8, one layer
TINY_S4 = {
    "architecture": "Suripel", "vocab": 61, "width": 50, "norm": {"eps": 1e-5}, "canon": {"taps": 1},
    "layers": [with_ff(retention(1, 40, 72, [0.9], rot=(2, 100.0)), 30), with_ff(delta(1, 1, 36, 3, 5), None)],
}

# attention alone: one layer, one head, a window of one with blocks of two
TINY_S5 = {
    "architecture": "Suripel", "vocab": 80, "width": 32, "norm": {"eps": 1e-3}, "canon": {"taps": 5},
    "layers": [with_ff(attention(1, 1, 16, 16, 1, 2, 2, 1.0), 48)],
}

CONFIGS = {"S1": (TINY_S1, 11), "S2": (TINY_S2, 12), "S3": (TINY_S3, 13), "S4": (TINY_S4, 14), "S5": (TINY_S5, 15)}


def make_model(which: str, folder: str, std: float = 0.12) -> str:
    from xyntetik_runner_amd.weights import write_random_model
    config, seed = CONFIGS[which]
    return write_random_model(config, folder, seed=seed, std=std, norm_jitter=0.1, dtype="bfloat16")
