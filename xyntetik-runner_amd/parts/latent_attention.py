"""Attention whose keys and values are made from one small latent a token.

Per token: ``c_q = rmsnorm(W_dq h)``, ``q = W_uq c_q`` (H heads, each ``D`` unrotated channels followed
by ``R`` rotated ones); ``W_dkv h`` has ``C + R`` rows: the first ``C``, RMS-normed, are the latent ``c``, the
last ``R`` are one key part that all heads share.  The rotation turns the first ``rot_dims`` of the ``R``
channels (of every query head and of the shared key part) in pairs ``(2i, 2i + 1)`` by
``position x base^(-2i / rot_dims)``.  A head's key is ``[W_uk c | shared part]``, its value ``W_uv c``; the
score is ``(q . k) * scale``; a token sees itself and the ``window - 1`` before it (all, without a
window); softmax in 32-bit; ``W_o`` on the concatenated heads.

Only ``[c | shared part]`` is cached, one row a token, as the one key/value head of a paged cache
that all query heads share.  The queries are brought into the latent's space instead of the keys
out of it: ``q_abs = W_uk_h^T q_unrotated`` gives ``q_abs . c = q_unrotated . (W_uk_h c)``; attention then
runs over the cached rows with value ``c``, and ``W_uv_h`` is applied to its output
(``W_uv_h sum_j p_j c_j = sum_j p_j W_uv_h c_j``).  The value pages hold the row transposed, as
every attention cache here does; where the matrix-core attention serves (bfloat16, a row length
that is a multiple of 16 up to 256) they hold all ``C + R`` channels, because that kernel wants values
as long as keys, and the output's last ``R`` channels are not read.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import KVSpec, Mixer, ParamSpec, register_mixer
from .rotary import rotary_inv_freq

MAX_ROW = 512       # the 32-bit attention kernel keeps a cached row in registers up to this size (the matrix-core kernels: 256)


class LatentAttention(Mixer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, rot_dim: int, v_head_dim: int, q_rank: int,
                 kv_rank: int, scale: float, eps: float, rot_dims: Optional[int] = None, rot_base: float = 10000.0,
                 window: Optional[int] = None, dq_name: str = "dq", dq_norm_name: str = "dq.norm", uq_name: str = "uq",
                 dkv_name: str = "dkv", dkv_norm_name: str = "dkv.norm", uk_name: str = "uk", uv_name: str = "uv",
                 o_name: str = "o"):
        self.hidden_size, self.num_heads = int(hidden_size), int(num_heads)
        self.head_dim, self.rot_dim, self.v_head_dim = int(head_dim), int(rot_dim), int(v_head_dim)
        self.q_rank, self.kv_rank = int(q_rank), int(kv_rank)
        self.row = self.kv_rank + self.rot_dim          # what is cached a token
        if not (1 <= self.row <= MAX_ROW):
            raise ValueError(f"latent attention: a cached row of {self.kv_rank} + {self.rot_dim} channels is outside what the "
                             f"attention kernels take (1 to {MAX_ROW})")
        self.rot_dims = self.rot_dim if rot_dims is None else int(rot_dims)
        if self.rot_dims % 2 or not (0 <= self.rot_dims <= self.rot_dim):
            raise ValueError(f"latent attention: {self.rot_dims} rotated channels must be even and at most {self.rot_dim}")
        if window is not None and window < 1:
            raise ValueError(f"attention window {window} must be at least 1")
        self.rot_base, self.scale, self.eps = float(rot_base), float(scale), float(eps)
        self.window = int(window) if window is not None else None
        self.names = dict(dq=dq_name, dq_norm=dq_norm_name, uq=uq_name, dkv=dkv_name, dkv_norm=dkv_norm_name, uk=uk_name,
                          uv=uv_name, o=o_name)
        self.rt = None

    def _matrix_cores(self) -> bool:
        """Whether the matrix-core attention kernels take this layer's cached rows."""
        if self.rt is None or self.rt.dtype != torch.bfloat16 or not getattr(self.rt.ops, "use_mfma", False):
            return False
        return self.row % 16 == 0 and 16 <= self.row <= 256

    def kv_spec(self) -> Optional[KVSpec]:
        return KVSpec(1, self.row, self.window, None if self._matrix_cores() else self.kv_rank)

    def param_specs(self) -> Dict[str, ParamSpec]:
        E, H, D, R, Dv, n = self.hidden_size, self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.names
        return {
            n["dq"]: ParamSpec((self.q_rank, E)), n["dq_norm"]: ParamSpec((self.q_rank,), role="vector", init="ones_jitter"),
            n["uq"]: ParamSpec((H * (D + R), self.q_rank)),
            n["dkv"]: ParamSpec((self.row, E)), n["dkv_norm"]: ParamSpec((self.kv_rank,), role="vector", init="ones_jitter"),
            n["uk"]: ParamSpec((H * D, self.kv_rank)), n["uv"]: ParamSpec((H * Dv, self.kv_rank)),
            n["o"]: ParamSpec((E, H * Dv)),
        }

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        ops, n = rt.ops, self.names
        H, D, R, Dv, C = self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank
        # both down projections in one product
        self.w_down = ops.pack_weight(torch.cat([tensors[n["dq"]], tensors[n["dkv"]]], dim=0).contiguous())
        self.w_dq_norm = tensors[n["dq_norm"]]
        self.w_c_norm = tensors[n["dkv_norm"]].float().contiguous()
        self.w_uq = ops.pack_weight(tensors[n["uq"]])
        # Per head: W_uk_h^T [C, D] takes the unrotated query channels into the latent's space,
        # W_uv_h [Dv, C] the attention's output out of it; each is one launch over all heads.
        self.w_absorb = tensors[n["uk"]].view(H, D, C).transpose(1, 2).contiguous()      # [H, C, D]
        self.w_expand = tensors[n["uv"]].view(H, Dv, C).contiguous()                     # [H, Dv, C]
        self.w_out = ops.pack_weight(tensors[n["o"]])
        self.inv_freq = (rotary_inv_freq(self.rot_dims, self.rot_base).to(torch.float32).to(rt.device)
                         if self.rot_dims else None)

    def _attend(self, ctx, cache, h):
        ops, rt = self.rt.ops, self.rt
        H, D, R, Dv, C, DK = self.num_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank, self.row
        T = h.shape[0]
        if not cache.owns:
            raise ValueError("latent attention: every layer stores its own latents")
        down = ops.linear(h, self.w_down, out_dtype=torch.float32)                       # [T, q_rank + C + R]
        cq = ops.rmsnorm(down[:, :self.q_rank], self.w_dq_norm, self.eps, rt.dtype)
        q_in = ops.linear(cq, self.w_uq, out_dtype=torch.float32)                        # [T, H * (D + R)]
        q = torch.empty((T, H * DK), dtype=rt.dtype, device=h.device)
        qn = ops.latent_prepare(q_in, down[:, self.q_rank:], self.w_c_norm, self.eps, q, cache.k, cache.v, ctx, cache.group,
                                self.inv_freq, H, D, R, C, self.rot_dims, cache.page_size)
        ops.heads_linear(qn, self.w_absorb, q, H, D, DK)
        Dvc = cache.v.shape[2]
        if Dvc == DK and self._matrix_cores():
            o = ops.attention(q, cache.k, cache.v, ctx, cache.group, H, 1, DK, cache.page_size, self.scale, self.window)
        else:
            o = ops.attention_pooled(q, cache.k, cache.v, None, None, ctx, cache.group, None, H, 1, DK, Dvc,
                                     cache.page_size, self.scale, self.window or (1 << 30), 0, matrix_cores=False)
        ov = torch.empty((T, H * Dv), dtype=rt.dtype, device=h.device)
        ops.heads_linear(o, self.w_expand, ov, H, Dvc, Dv)
        return ov

    def forward(self, ctx, cache, h):
        return self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out)

    def forward_f32(self, ctx, cache, h):
        return self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, out_dtype=torch.float32)

    def forward_add(self, ctx, cache, h, residual) -> None:
        self.rt.ops.linear(self._attend(ctx, cache, h), self.w_out, out=residual, accumulate=True)


register_mixer("latent_attention", LatentAttention)
