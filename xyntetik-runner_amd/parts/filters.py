"""Sequence filters: what a sublayer reads passes through one on its way from the norm.

``CausalConv``: a short convolution over time on every channel,
``y_t = sum_j w[:, j] u_(t - taps + 1 + j)`` with zeros before a request's first token, added to
its input (``residual``) or in its place, then an optional activation.  The last ``taps - 1``
inputs of every request are its state, so a request may be cut into steps anywhere.
The same part serves a mixer's convolutions of its projections.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import ParamSpec, SequenceFilter, StateSpec, register_filter


class CausalConv(SequenceFilter):
    def __init__(self, channels: int, taps: int, residual: bool = True, activation: Optional[str] = None,
                 weight_name: str = "weight", optional: bool = False):
        from ..csrc.ops import CONV_ACTIVATIONS
        if activation not in CONV_ACTIVATIONS:
            raise ValueError(f"causal convolution: activation {activation!r} is not built into the kernels (none, silu)")
        if not (1 <= int(taps) <= 16):
            raise ValueError(f"causal convolution: {taps} taps (the kernel takes 1 to 16)")
        self.channels, self.taps = int(channels), int(taps)
        self.residual, self.activation = bool(residual), activation
        self.weight_name, self.optional = weight_name, bool(optional)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.weight_name: ParamSpec((self.channels, self.taps), role="vector", init="normal:0.4", optional=self.optional)}

    def state_spec(self) -> Optional[StateSpec]:
        if self.taps <= 1:
            return None
        return StateSpec((self.taps - 1, self.channels), torch.float32)

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        w = tensors.get(self.weight_name)
        self.weight = w.float().contiguous() if w is not None else None

    def forward(self, ctx, state, h, out_dtype=None):
        """``h``: 32-bit rows ``[T, channels]``; the result is in the compute dtype unless told otherwise."""
        return self.rt.ops.causal_conv(h, self.weight, state, ctx, out_dtype or self.rt.dtype, residual=self.residual,
                                       activation=self.activation)


    def forward_normed(self, ctx, state, x, norm):
        """``forward(ctx, state, norm.forward(ctx, x))`` in one kernel where there is one: a step of one
        row a request, a layer norm in front, the input added, no activation.  None: the caller
        runs the two one after the other."""
        from .norm import LayerNorm
        if (ctx.max_q_len != 1 or not isinstance(norm, LayerNorm) or not self.residual or self.activation is not None
                or self.weight is None):
            return None
        return self.rt.ops.layernorm_conv(x, norm.weight, norm.eps, self.weight, state, ctx, self.rt.dtype)


register_filter("causal_conv", CausalConv)
