"""A plain, slow Sugosun decoder in numpy float64: whole sequences, no cache, no state.

One function per mechanism, each written from its equation; nothing here knows of pages,
slots, batches or kernels, and nothing is shared with the engine.  The tests compare what the
engine does, however its work is cut, with these functions run over the whole sequence.

Notation: ``T`` tokens, ``E`` width, ``S`` residual streams; a mixer has ``H`` heads, key size
``D`` (latent attention: ``D`` unrotated + ``R`` rotated channels a head), value size ``Dv``, latent
size ``C``.  Weights are ``[out, in]`` and applied as ``W x``.
"""
from __future__ import annotations

import math

import numpy as np


# ----------------------------------------------------------------------------- small pieces
def rms_div(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, w, eps):
    return rms_div(x, eps) * w


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softmax(z):
    z = z - z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return e / e.sum(axis=-1, keepdims=True)


# ----------------------------------------------------------------------------- embedding
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the bigram table for every token: a hash of (token before, token) into ``buckets``
    rows; the first token of a sequence, which has none before it, takes the extra last row."""
    rows = []
    for t, tok in enumerate(tokens):
        rows.append(buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets)
    return np.asarray(rows, dtype=np.int64)


def embed(tokens, table, bigram, norm_w, eps, buckets, mul_prev, mul_cur):
    x = table[np.asarray(tokens, dtype=np.int64)]
    if bigram is not None:
        x = x + bigram[bigram_rows(tokens, buckets, mul_prev, mul_cur)]
    return rms_norm(x, norm_w, eps)


# ----------------------------------------------------------------------------- rotation
def rotate_pairs(x, positions, dims, base):
    """Rotate the first ``dims`` channels of the last axis of ``x [T, ..., D]``: channel 2i pairs with
    channel 2i + 1, angle = position * base^(-2i/dims), formed as the 32-bit product of a 32-bit
    position and a 32-bit frequency (as an engine would form it)."""
    out = x.copy()
    half = dims // 2
    f = (float(base) ** (-2.0 * np.arange(half) / dims)).astype(np.float32)
    a = (np.asarray(positions, dtype=np.float32)[:, None] * f[None, :]).astype(np.float64)      # [T, half]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (half,)
    c, s = np.cos(a).reshape(shape), np.sin(a).reshape(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


# ----------------------------------------------------------------------------- mixers
def lightning(h, w, m, eps):
    """Linear attention with one fixed decay a head: q, k, v through SiLU; S <- decay S + k v^T,
    read out as S^T q after the update; all heads' read-outs normed together (RMS, a weight),
    times sigmoid(Wg h), then Wo."""
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).reshape(T, H, D)
    k = silu(h @ w["k"].T).reshape(T, H, D)
    v = silu(h @ w["v"].T).reshape(T, H, Dv)
    o = np.zeros((T, H, Dv))
    for hd in range(H):
        S = np.zeros((D, Dv))
        for t in range(T):
            S = m["decay"][hd] * S + np.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    y = rms_norm(o.reshape(T, H * Dv), w["norm"], eps) * sigmoid(h @ w["g"].T)
    return y @ w["o"].T


def latent_attention(h, w, m, eps, positions=None):
    """Attention whose keys and values are made from one small latent a token.  Queries come
    through a latent of their own.  A head's score has two terms: unrotated query channels with
    keys made from the latent, and rotated query channels with one rotated key part that all
    heads share.  A token sees itself and the ``window - 1`` before it (all, without a window)."""
    T = h.shape[0]
    H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T) if positions is None else np.asarray(positions)
    cq = rms_norm(h @ w["dq"].T, w["dq.norm"], eps)
    q = (cq @ w["uq"].T).reshape(T, H, D + R)
    kv = h @ w["dkv"].T
    c = rms_norm(kv[:, :C], w["dkv.norm"], eps)
    rot = m.get("rot") or {}
    dims, base = rot.get("dims", 0), rot.get("base", 10000.0)
    kr = kv[:, C:]
    qn, qr = q[..., :D], q[..., D:]
    if dims:
        kr = rotate_pairs(kr, pos, dims, base)
        qr = rotate_pairs(qr, pos, dims, base)
    kn = (c @ w["uk"].T).reshape(T, H, D)
    val = (c @ w["uv"].T).reshape(T, H, Dv)
    window = (m.get("mask") or {}).get("size")
    out = np.zeros((T, H, Dv))
    for i in range(T):
        lo = 0 if not window else max(0, i - window + 1)
        for hd in range(H):
            s = (kn[lo:i + 1, hd] @ qn[i, hd] + kr[lo:i + 1] @ qr[i, hd]) * m["scale"]
            out[i, hd] = softmax(s) @ val[lo:i + 1, hd]
    return out.reshape(T, H * Dv) @ w["o"].T


# ----------------------------------------------------------------------------- feed-forward
def dense_ff(h, w, limit):
    """A gated feed-forward with both branches clamped: the gate from above, the other branch
    from both sides; the gate passes x sigmoid(1.702 x), the other branch has one added."""
    g = np.minimum(h @ w["gate"].T, limit)
    u = np.clip(h @ w["up"].T, -limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ w["down"].T


def route(h, router, correction, top):
    """(chosen experts [T, top], their weights [T, top]): softmax over all experts; the choice adds
    a correction to the scores, the weights do not; the weights are the chosen scores over their sum."""
    s = softmax(h @ router.T)
    pick = s + correction
    chosen = np.argsort(-pick, axis=-1, kind="stable")[:, :top]
    sc = np.take_along_axis(s, chosen, axis=-1)
    return chosen, sc / (sc.sum(axis=-1, keepdims=True) + 1e-20)


def expert(h, up, down):
    z = np.maximum(h @ up.T, 0.0)
    return (z * z) @ down.T


def moe_ff(h, w, n_experts, top):
    chosen, weights = route(h, w["router"], w["correction"], top)
    y = np.zeros((h.shape[0], w["e0.down"].shape[0]))
    for t in range(h.shape[0]):
        for e, g in zip(chosen[t], weights[t]):
            y[t] += g * expert(h[t], w[f"e{e}.up"], w[f"e{e}.down"])
    return y


# ----------------------------------------------------------------------------- the model
def sub(weights, prefix):
    """The tensors below ``prefix``, by the rest of their names."""
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def run_order(cfg):
    """Layer indices in the order they run: the looped span repeated in place."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def mixer_of(layer, h, w, eps):
    if layer["type"] == "lightning":
        return lightning(h, w, layer["mixer"], eps)
    if layer["type"] == "latent_attention":
        return latent_attention(h, w, layer["mixer"], eps)
    raise ValueError(layer["type"])


def ff_of(layer, h, w):
    mlp = layer["mlp"]
    if mlp["kind"] == "dense":
        return dense_ff(h, w, mlp["limit"])
    return moe_ff(h, w, mlp["router"]["experts"], mlp["router"]["top"])


def forward(cfg, weights, tokens, keep_layers=False):
    """Logits ``[T, vocab]`` of one sequence (and the residual stream after every layer run)."""
    eps = cfg["norm"]["eps"]
    big = (cfg.get("embedding") or {}).get("bigram")
    x = embed(tokens, weights["embed"], weights["bigram"] if big else None, weights["embed.norm"], eps,
              big["buckets"] if big else 0, big["mul_prev"] if big else 0, big["mul_cur"] if big else 0)
    S = cfg.get("streams")
    xs = [x.copy() for _ in range(S)] if S else None
    after = []
    for i in run_order(cfg):
        layer = cfg["layers"][i]
        w = sub(weights, f"l{i}.")
        subs = [(1, lambda h: mixer_of(layer, h, sub(w, "mix."), eps))]
        if layer.get("mlp"):
            subs.append((2, lambda h: ff_of(layer, h, sub(w, "mlp."))))
        for q, fn in subs:
            if xs is None:
                x = x + fn(rms_norm(x, w[f"norm{q}"], eps))
                continue
            u = sum(w[f"hc{q}.in"][s] * xs[s] for s in range(S))
            y = fn(rms_norm(u, w[f"norm{q}"], eps))
            xs = [sum(w[f"hc{q}.mix"][s, t] * xs[s] for s in range(S)) + w[f"hc{q}.out"][t] * y for t in range(S)]
        if xs is not None:
            x = sum(xs)
        after.append(x.copy())
    logits = rms_norm(x, weights["final.norm"], eps) @ weights["head"].T
    return (logits, np.stack(after)) if keep_layers else logits
