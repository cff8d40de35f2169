"""A plain, slow Suripel decoder in numpy float64: whole sequences, no cache, no state.

One function per mechanism, each written from its equation; nothing here knows of pages,
slots, batches or kernels, and nothing is shared with the engine.  The tests compare what the
engine does, however its work is cut, with these functions run over the whole sequence.

Notation: ``T`` tokens, ``E`` width; a mixer has ``H`` heads (``G`` key heads where they are
grouped), key size ``D`` and value size ``Dv``.  Weights are ``[out, in]`` and applied as ``W x``.
"""
from __future__ import annotations

import math

import numpy as np

from plain_llama import load_folder    # noqa: F401  (config.json + safetensors as float64 arrays)


# ----------------------------------------------------------------------------- small pieces
def layer_norm(x, w, eps):
    """(x - mean) / sqrt(var + eps) * w over the last axis, var = mean of squared deviations; no bias."""
    m = x.mean(axis=-1, keepdims=True)
    d = x - m
    return d / np.sqrt((d * d).mean(axis=-1, keepdims=True) + eps) * w


def rms_div(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def causal_conv(u, w):
    """y_t = sum_j w[:, j] * u_(t - taps + 1 + j) per channel, zeros before the start.
    ``u [T, C]``, ``w [C, taps]`` (the last column is the current token's)."""
    T, C = u.shape
    taps = w.shape[1]
    y = np.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def silu(z):
    return z / (1.0 + np.exp(-z))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.where(z > 30.0, z, np.log1p(np.exp(np.minimum(z, 30.0))))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotate_half(x, positions, dims, base):
    """Rotate the first ``dims`` channels of every head of ``x [T, H, D]``: channel i pairs with
    i + dims/2, angle = position * base^(-2i/dims), formed as a 32-bit product of a 32-bit
    position and a 32-bit frequency (as an engine would form it)."""
    out = x.copy()
    half = dims // 2
    f = (float(base) ** (-2.0 * np.arange(half) / dims)).astype(np.float32)
    a = (np.asarray(positions, dtype=np.float32)[:, None] * f[None, :]).astype(np.float64)      # [T, half]
    c, s = np.cos(a)[:, None, :], np.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    out[..., :half] = u * c - v * s
    out[..., half:dims] = v * c + u * s
    return out


# ----------------------------------------------------------------------------- feed-forward
def polynorm(z, act, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N = division by the row's
    root mean square."""
    a, b, c, e = act
    return a * rms_div(z, eps) + b * rms_div(z * z, eps) + c * rms_div(z * z * z, eps) + e


def dense_ff(h, w_up, w_down, act, eps):
    return polynorm(h @ w_up.T, act, eps) @ w_down.T


# ----------------------------------------------------------------------------- windowed attention with pooled blocks
def visible(i, size, pool):
    """(the positions query ``i`` sees one by one, the pooled blocks it sees)."""
    lo = max(0, i - size + 1)
    blocks = []
    if pool:
        b = 0
        while b * pool + pool - 1 <= i - size:
            blocks.append(b)
            b += 1
    return list(range(lo, i + 1)), blocks


def pooled_window_attention(q, k, v, scale, size, pool, cache_round=None):
    """``q [T, H, D]``, ``k [T, G, D]``, ``v [T, G, Dv]`` -> ``[T, H, Dv]``.  One softmax per query i over
    the keys j, i - size < j <= i, and the mean key (with the mean value) of every block of ``pool``
    positions that ``visible`` lists.  ``cache_round``: what a cache does to the keys and values it
    stores (the means are of the stored ones and are stored themselves)."""
    T, H, D = q.shape
    G = k.shape[1]
    per = H // G
    if cache_round is not None:
        k, v = cache_round(k), cache_round(v)
    out = np.zeros((T, H, v.shape[2]))
    for i in range(T):
        toks, blocks = visible(i, size, pool)
        for h in range(H):
            g = h // per
            ks = [k[j, g] for j in toks]
            vs = [v[j, g] for j in toks]
            for b in blocks:
                mk, mv = k[b * pool:(b + 1) * pool, g].mean(axis=0), v[b * pool:(b + 1) * pool, g].mean(axis=0)
                if cache_round is not None:
                    mk, mv = cache_round(mk), cache_round(mv)
                ks.append(mk)
                vs.append(mv)
            s = np.array([q[i, h] @ kk for kk in ks]) * scale
            p = np.exp(s - s.max())
            p /= p.sum()
            out[i, h] = sum(pp * vv for pp, vv in zip(p, vs))
    return out


def attention_mixer(h, w, p, m, kv=None):
    """``m``: the mixer's config entry; ``kv``: another layer's (keys, values) for a layer that
    has none of its own.  Returns (output, (keys, values) as a cache would hold them)."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    conv = (lambda u, name: causal_conv(u, w[p + name + ".conv"])) if m.get("conv") else (lambda u, name: u)
    q = conv(h @ w[p + "q"].T, "q").reshape(T, H, D)
    if kv is None:
        k = conv(h @ w[p + "k"].T, "k").reshape(T, G, D)
        v = conv(h @ w[p + "v"].T, "v").reshape(T, G, Dv)
    else:
        k, v = kv
    o = pooled_window_attention(q, k, v, m["scale"], m["mask"]["size"], m["mask"].get("pool", 0))
    return o.reshape(T, H * Dv) @ w[p + "o"].T, (k, v)


# ----------------------------------------------------------------------------- gated delta rule
def unit(x):
    return x / np.sqrt((x * x).sum(axis=-1, keepdims=True) + 1e-6)


def gated_delta_rule(q, k, v, beta, g):
    """Per head, token by token: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    ``q, k [T, H, D]``, ``v [T, H, Dv]``, ``beta, g [T, H]`` -> ``[T, H, Dv]``."""
    T, H, D = q.shape
    Dv = v.shape[2]
    out = np.zeros((T, H, Dv))
    for h in range(H):
        S = np.zeros((D, Dv))
        for t in range(T):
            S = g[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + np.outer(k[t, h], u)
            out[t, h] = S.T @ q[t, h]
    return out


def delta_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    conv = (lambda u, name: causal_conv(u, w[p + name + ".conv"])) if m.get("conv") else (lambda u, name: u)
    q = silu(conv(h @ w[p + "q"].T, "q")).reshape(T, G, D)
    k = silu(conv(h @ w[p + "k"].T, "k")).reshape(T, G, D)
    v = silu(conv(h @ w[p + "v"].T, "v")).reshape(T, H, Dv)
    q = unit(q) * D ** -0.5
    k = unit(k)
    per = H // G
    q = np.repeat(q, per, axis=1)       # head h uses q/k head h // per
    k = np.repeat(k, per, axis=1)
    beta = sigmoid(h @ w[p + "b"].T)
    g = np.exp(-np.exp(w[p + "A_log"]) * softplus(h @ w[p + "a"].T + w[p + "dt_bias"]))
    o = gated_delta_rule(q, k, v, beta, g)
    o = rms_div(o, eps) * w[p + "norm"] * silu(h @ w[p + "g"].T).reshape(T, H, Dv)
    return o.reshape(T, H * Dv) @ w[p + "o"].T


# ----------------------------------------------------------------------------- retention
def retention(q, k, v, decay):
    """Per head: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T, H, D = q.shape
    out = np.zeros((T, H, v.shape[2]))
    for h in range(H):
        S = np.zeros((D, v.shape[2]))
        for t in range(T):
            S = decay[h] * S + np.outer(k[t, h], v[t, h])
            out[t, h] = S.T @ q[t, h]
    return out


def retention_mixer(h, w, p, m, eps):
    T = h.shape[0]
    H, D, Dv = m["heads"], m["dim"], m["vdim"]
    pos = np.arange(T)
    q = (h @ w[p + "q"].T).reshape(T, H, D)
    k = (h @ w[p + "k"].T).reshape(T, H, D)
    v = (h @ w[p + "v"].T).reshape(T, H, Dv)
    rot = m.get("rot")
    if rot:
        q = rotate_half(q, pos, rot["dims"], rot["base"])
        k = rotate_half(k, pos, rot["dims"], rot["base"])
    k = k * D ** -0.5
    o = rms_div(retention(q, k, v, m["decay"]), eps).reshape(T, H * Dv)
    return (o * silu(h @ w[p + "g"].T)) @ w[p + "o"].T


# ----------------------------------------------------------------------------- the model
def forward(cfg, w, tokens, layers_out=None):
    """Logits ``[T, vocab]`` of a whole sequence; ``layers_out`` (a list) receives the residual
    stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][np.asarray(tokens)].copy()
    kvs = {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = layer["mixer"]
        h = layer_norm(x, w[p + "norm1"], eps)
        h = h + causal_conv(h, w[p + "canon1"])
        if layer["type"] == "attention":
            src = m.get("kv_from")
            y, kvs[i] = attention_mixer(h, w, p + "mix.", m, kv=kvs[src] if src is not None else None)
        elif layer["type"] == "delta":
            y = delta_mixer(h, w, p + "mix.", m, eps)
        elif layer["type"] == "retention":
            y = retention_mixer(h, w, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + y
        if layer.get("mlp") is not None:
            h = layer_norm(x, w[p + "norm2"], eps)
            h = h + causal_conv(h, w[p + "canon2"])
            x = x + dense_ff(h, w[p + "mlp.up"], w[p + "mlp.down"], w[p + "mlp.act"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return layer_norm(x, w["final.norm"], eps) @ w["head"].T


def greedy(cfg, w, prompt, n_new):
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        t = int(np.argmax(forward(cfg, w, toks)[-1]))
        out.append(t)
        toks.append(t)
    return out
