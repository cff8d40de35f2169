"""``SuripelConfig``: the hyper-parameters of a Suripel decoder, typed.

config.json of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``canon.taps`` and a list
``layers`` whose entries name their mixer (``type``: "attention", "delta" or "retention"), the
mixer's sizes (``mixer``) and the feed-forward (``mlp``: ``{"kind": "dense", "ff": F}``, or null for a
layer without one).  Every size and constant that can differ between models is read here and
nowhere else; what the design fixes (the unit vectors' 1e-6, the powers of PolyNorm) lives in the parts.

====================  =====================================================================
mixer                 keys of ``mixer``
====================  =====================================================================
attention             heads, kv_heads, dim, vdim, conv (taps), scale, mask.size, mask.pool
                      (absent or 0: no pooled blocks), kv_from (the layer whose keys and values it reads)
delta                 heads, kv_heads, dim, vdim, conv (taps)
retention             heads, dim, vdim, decay (one a head), rot.dims and rot.base (absent: no rotation)
====================  =====================================================================
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, Fields

MIXERS = ("attention", "delta", "retention")


@dataclass(frozen=True)
class SuripelMixer:
    kind: str
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int = 0                       # taps of the convolutions of q, k and v (attention, delta); 0: none
    scale: Optional[float] = None       # attention
    window: Optional[int] = None        # attention: mask.size
    pool: int = 0                       # attention: mask.pool
    kv_from: Optional[int] = None       # attention
    decay: Tuple[float, ...] = ()       # retention
    rot_dims: int = 0                   # retention
    rot_base: float = 10000.0


@dataclass(frozen=True)
class SuripelLayer:
    mixer: SuripelMixer
    ff: Optional[int]                   # the feed-forward's inner width; None: the layer has none


@dataclass(frozen=True)
class SuripelConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    canon_taps: int
    layers: Tuple[SuripelLayer, ...]
    max_position: int

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "SuripelConfig":
        f = Fields(raw)
        norm = f.mapping("norm")
        canon = f.mapping("canon")
        if norm is None or canon is None:
            raise ConfigError("config.json: 'norm' and 'canon' are required objects")
        layers = []
        entries = f.mappings("layers")
        for i, lf in enumerate(entries):
            kind = lf.string("type", choices=MIXERS)
            mf = lf.mapping("mixer")
            if mf is None:
                raise ConfigError(f"{lf.where}: 'mixer' is required")
            layers.append(SuripelLayer(_mixer(kind, mf, i, entries), _ff(lf)))
        return SuripelConfig(
            architecture="Suripel", vocab=f.integer("vocab"), width=f.integer("width"),
            eps=norm.number("eps", lo=0.0), canon_taps=canon.integer("taps", lo=1, hi=16), layers=tuple(layers),
            max_position=f.integer("max_position", default=1 << 20, hi=1 << 30))


def _ff(lf: Fields) -> Optional[int]:
    mlp = lf.mapping("mlp")
    if mlp is None:
        return None
    mlp.string("kind", choices=("dense",))
    return mlp.integer("ff")


def _mixer(kind: str, mf: Fields, index: int, entries) -> SuripelMixer:
    heads = mf.integer("heads")
    dim, vdim = mf.integer("dim"), mf.integer("vdim")
    if kind == "retention":
        rot = mf.mapping("rot")
        dims = rot.integer("dims", lo=2) if rot is not None else 0
        if dims % 2 or dims > dim:
            raise ConfigError(f"{mf.where}: rot.dims = {dims} must be even and at most dim = {dim}")
        return SuripelMixer(kind, heads, heads, dim, vdim, decay=mf.numbers("decay", count=heads, lo=0.0, hi=1.0),
                            rot_dims=dims, rot_base=rot.number("base", lo=0.0, lo_open=True) if rot is not None else 10000.0)
    kv_heads = mf.integer("kv_heads", default=heads)
    if heads % kv_heads:
        raise ConfigError(f"{mf.where}: heads = {heads} is no multiple of kv_heads = {kv_heads}")
    conv = mf.integer("conv", default=0, hi=16)     # absent: the projections go on as they are, and no taps are stored
    if kind == "delta":
        return SuripelMixer(kind, heads, kv_heads, dim, vdim, conv=conv)
    mask = mf.mapping("mask")
    if mask is None:
        raise ConfigError(f"{mf.where}: 'mask' is required")
    kv_from = mf.integer("kv_from", default=None, lo=0, hi=max(0, index - 1)) if index > 0 else None
    if index == 0 and mf.raw.get("kv_from") is not None:
        raise ConfigError(f"{mf.where}: the first layer has no layer before it to read keys and values from")
    if kv_from is not None:
        src = entries[kv_from]
        sm = src.mapping("mixer")
        if src.raw.get("type") != "attention" or sm is None or sm.raw.get("kv_from") is not None:
            raise ConfigError(f"{mf.where}: kv_from = {kv_from} must name an attention layer with keys and values of its own")
        if (sm.raw.get("kv_heads", sm.raw.get("heads")), sm.raw.get("dim"), sm.raw.get("vdim")) != (kv_heads, dim, vdim):
            raise ConfigError(f"{mf.where}: layer {kv_from}'s key/value heads and sizes differ from this layer's")
    return SuripelMixer(kind, heads, kv_heads, dim, vdim, conv=conv, scale=mf.number("scale", default=None),
                        window=mask.integer("size", hi=1 << 30), pool=mask.integer("pool", default=0, lo=0, hi=1 << 30),
                        kv_from=kv_from)
