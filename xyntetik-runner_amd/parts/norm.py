"""Norms of the residual stream, in 32-bit.

RMSNorm: ``y = x / sqrt(mean(x^2) + eps) * w``
(src/model.c:3386-3392; kernel src/kernels.cu:32-48).
LayerNorm: ``y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * w``, a weight and no bias.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import Norm, ParamSpec, register_norm


class RMSNorm(Norm):
    def __init__(self, size: int, eps: float, weight_name: str = "weight", has_weight: bool = True, optional: bool = False):
        self.size, self.eps = int(size), float(eps)
        self.weight_name, self.has_weight, self.optional = weight_name, has_weight, bool(optional)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if not self.has_weight:
            return {}
        return {self.weight_name: ParamSpec((self.size,), role="vector", init="ones_jitter", optional=self.optional)}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.weight = tensors.get(self.weight_name)

    def forward(self, ctx, x, rows=None):
        return self.rt.ops.rmsnorm(x, self.weight, self.eps, self.rt.dtype, rows=rows)

    def fold(self):
        return (self.weight, self.eps) if self.weight is not None else None


class LayerNorm(Norm):
    """``out_dtype``: "compute" (the engine's dtype) or "float32", for a reader that wants the
    rows unrounded (a filter that carries them from token to token)."""

    def __init__(self, size: int, eps: float, weight_name: str = "weight", has_weight: bool = True,
                 out_dtype: str = "compute", optional: bool = False):
        if out_dtype not in ("compute", "float32"):
            raise ValueError(f"layer norm: out_dtype {out_dtype!r} (compute or float32)")
        self.size, self.eps = int(size), float(eps)
        self.weight_name, self.has_weight, self.out_dtype, self.optional = weight_name, has_weight, out_dtype, bool(optional)
        self.weight: Optional[torch.Tensor] = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        if not self.has_weight:
            return {}
        return {self.weight_name: ParamSpec((self.size,), role="vector", init="ones_jitter", optional=self.optional)}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        w = tensors.get(self.weight_name)
        self.weight = w.float().contiguous() if w is not None else None

    def forward(self, ctx, x, rows=None):
        dt = torch.float32 if self.out_dtype == "float32" else self.rt.dtype
        return self.rt.ops.layernorm(x, self.weight, self.eps, dt, rows=rows)


register_norm("rmsnorm", RMSNorm)
register_norm("layernorm", LayerNorm)
