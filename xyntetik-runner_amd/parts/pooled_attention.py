"""Sliding-window attention with pooled blocks over the paged cache.

Per token: ``q = Wq h``, ``k = Wk h``, ``v = Wv h`` (no biases), each channel then through a
short causal convolution over time (no activation); keys and values go to the cache as they
leave the convolution, no rotation.  Query head ``h`` reads key/value head ``h // (H / G)``.
The query at position ``i`` attends, in a single softmax over ``(q . k) * scale``, to the cached keys
at positions ``j`` with ``i - window < j <= i`` and to one summary per block of ``pool`` positions whose
last position ``b pool + pool - 1`` is at most ``i - window``: the means of that block's cached keys and
values.  Older positions whose block does not qualify yet contribute nothing.  Key and value
sizes may differ.

The block means are kept in a cache of their own (``KVSpec.pooled``): the layer writes the mean of
every block a step completes, so a request cut into steps anywhere reads what a whole prompt reads.
A layer with ``kv_shared`` has no key or value projection: it reads the cache of the layer the run
order names, with its own queries, window and blocks.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from .base import KVSpec, Mixer, ParamSpec, StateSpec, register_mixer

MAX_HEAD_DIM = 256


class PooledWindowAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, window: int,
                 v_head_dim: Optional[int] = None, pool: int = 0, scale: Optional[float] = None, conv_taps: int = 1,
                 keep: Optional[int] = None, kv_shared: bool = False,
                 q_name: str = "q", k_name: str = "k", v_name: str = "v", o_name: str = "o", conv_suffix: str = ".conv"):
        """``keep``: how many positions back the cache must reach (at least ``window`` and ``pool``, the
        default; more where a layer with a longer reach reads this layer's cache)."""
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are not a multiple of {num_kv_heads} key/value heads")
        if window < 1 or pool < 0:
            raise ValueError(f"attention window {window} must be at least 1 and blocks of {pool} at least 0")
        self.hidden_size, self.num_heads, self.num_kv_heads = int(hidden_size), int(num_heads), int(num_kv_heads)
        self.head_dim = int(head_dim)
        self.v_head_dim = int(v_head_dim) if v_head_dim is not None else self.head_dim
        if not (1 <= self.head_dim <= MAX_HEAD_DIM and 1 <= self.v_head_dim <= MAX_HEAD_DIM):
            raise ValueError(f"attention head sizes {self.head_dim}/{self.v_head_dim} are outside what the kernels take (1 to {MAX_HEAD_DIM})")
        self.window, self.pool = int(window), int(pool)
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(self.head_dim)
        self.conv_taps = int(conv_taps)      # 0: no convolution, and no tensors of one
        if not (0 <= self.conv_taps <= 16):
            raise ValueError(f"attention: {conv_taps} convolution taps (0 to 16)")
        need = max(self.window, self.pool)
        self.keep = max(int(keep), need) if keep is not None else need
        self.kv_shared = bool(kv_shared)
        self.names = (q_name, k_name, v_name, o_name)
        self.conv_suffix = conv_suffix
        self.q_size = self.num_heads * self.head_dim
        self.k_size = self.num_kv_heads * self.head_dim
        self.v_size = self.num_kv_heads * self.v_head_dim
        self.in_size = self.q_size + (0 if self.kv_shared else self.k_size + self.v_size)
        self.w_in = self.w_out = self.w_conv = None

    def kv_spec(self) -> Optional[KVSpec]:
        return KVSpec(self.num_kv_heads, self.head_dim, self.keep, self.v_head_dim if self.v_head_dim != self.head_dim else None,
                      self.pool or None)

    def state_spec(self):
        if self.conv_taps <= 1:
            return None
        return {"conv": StateSpec((self.conv_taps - 1, self.in_size), torch.float32)}

    def _projections(self):
        q, k, v, _ = self.names
        out = [(q, self.q_size)]
        if not self.kv_shared:
            out += [(k, self.k_size), (v, self.v_size)]
        return out

    def param_specs(self) -> Dict[str, ParamSpec]:
        E = self.hidden_size
        specs = {}
        for name, rows in self._projections():
            specs[name] = ParamSpec((rows, E))
            if self.conv_taps:
                specs[name + self.conv_suffix] = ParamSpec((rows, self.conv_taps), role="vector", init="normal:0.6")
        specs[self.names[3]] = ParamSpec((E, self.num_heads * self.v_head_dim))
        return specs

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        mats = [tensors[name] for name, _ in self._projections()]
        self.w_in = rt.ops.pack_weight(torch.cat(mats, dim=0).contiguous() if len(mats) > 1 else mats[0])
        self.w_conv = (torch.cat([tensors[name + self.conv_suffix].float() for name, _ in self._projections()], dim=0).contiguous()
                       if self.conv_taps else None)
        self.w_out = rt.ops.pack_weight(tensors[self.names[3]])

    def _attend(self, ctx, cache, h):
        ops = self.rt.ops
        H, G, D, Dv, P = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, self.pool
        Q, K = self.q_size, self.k_size
        writes = not self.kv_shared and cache.owns
        if writes == self.kv_shared:
            raise ValueError("pooled attention: a layer stores its keys and values exactly when it projects them")
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        y = ops.causal_conv(proj, self.w_conv, cache.states.get("mixer.conv"), ctx, torch.float32) if self.conv_taps else proj
        q = ops.qkv_store(y[:, :Q], y[:, Q:Q + K] if writes else None, y[:, Q + K:] if writes else None,
                          cache.k, cache.v, ctx, cache.group, H, G, D, Dv, cache.page_size, self.rt.dtype)
        if P and cache.pool_owns:
            ops.pool_blocks(cache.pool_k, cache.pool_v, cache.k, cache.v, ctx, cache.group, cache.pool_group, G, D, Dv, P,
                            cache.page_size)
        return ops.attention_pooled(q, cache.k, cache.v, cache.pool_k, cache.pool_v, ctx, cache.group,
                                    cache.pool_group if P else None, H, G, D, Dv, cache.page_size, self.scale,
                                    self.window, P)

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, out=residual, accumulate=True)


register_mixer("pooled_window_attention", PooledWindowAttention)
