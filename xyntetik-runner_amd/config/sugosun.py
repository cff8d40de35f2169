"""``SugosunConfig``: the hyper-parameters of a Sugosun decoder, typed.

config.json of this design is nested: ``vocab``, ``width``, ``norm.eps``, ``embedding.bigram`` (the
hashed table added to the token embedding: ``buckets``, ``mul_prev``, ``mul_cur``; absent: none),
``streams`` (copies of the residual stream that the layers mix; absent: the plain sum), ``loop``
(``start``, ``stop``, ``times``: a span of layers that runs several times in a row) and a list
``layers`` whose entries name their mixer (``type``), the mixer's sizes (``mixer``) and the
feed-forward (``mlp``, or null for a layer without one).  Every size and constant that can differ
between models is read here and nowhere else; what the design fixes lives in the parts.

====================  =====================================================================
mixer                 keys of ``mixer``
====================  =====================================================================
lightning             heads, dim, vdim, decay (one a head)
latent_attention      heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, rot.dims, rot.base,
                      mask.size (absent: every earlier token is seen)
====================  =====================================================================

====================  =====================================================================
mlp.kind              keys of ``mlp``
====================  =====================================================================
dense                 ff, limit
moe                   expert.ff, router.experts, router.top
====================  =====================================================================
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Mapping, Optional, Tuple

from .base import ConfigError, Fields

MIXERS = ("lightning", "latent_attention")
MLPS = ("dense", "moe")


@dataclass(frozen=True)
class SugosunMixer:
    kind: str
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...] = ()       # lightning
    rot_dim: int = 0                    # latent attention: rotated channels a head
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    rot_dims: int = 0                   # how many of the rotated part's channels turn
    rot_base: float = 10000.0
    window: Optional[int] = None


@dataclass(frozen=True)
class SugosunMLP:
    kind: str
    ff: int
    limit: float = 0.0                  # dense
    experts: int = 0                    # moe
    top: int = 0


@dataclass(frozen=True)
class SugosunLayer:
    mixer: SugosunMixer
    mlp: Optional[SugosunMLP]


@dataclass(frozen=True)
class SugosunBigram:
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass(frozen=True)
class SugosunConfig:
    architecture: str
    vocab: int
    width: int
    eps: float
    bigram: Optional[SugosunBigram]
    streams: Optional[int]
    layers: Tuple[SugosunLayer, ...]
    loop: Optional[Tuple[int, int, int]]        # (start, stop, times)
    max_position: int

    def run_order(self) -> Tuple[int, ...]:
        """Layer indices in the order they run."""
        n = len(self.layers)
        if self.loop is None:
            return tuple(range(n))
        a, b, times = self.loop
        return tuple(range(a)) + tuple(range(a, b)) * times + tuple(range(b, n))

    @staticmethod
    def from_dict(raw: Mapping[str, Any]) -> "SugosunConfig":
        f = Fields(raw)
        norm = f.mapping("norm")
        if norm is None:
            raise ConfigError("config.json: 'norm' is a required object")
        layers = []
        for lf in f.mappings("layers"):
            kind = lf.string("type", choices=MIXERS)
            mf = lf.mapping("mixer")
            if mf is None:
                raise ConfigError(f"{lf.where}: 'mixer' is required")
            layers.append(SugosunLayer(_mixer(kind, mf), _mlp(lf)))
        bigram = None
        emb = f.mapping("embedding")
        bf = emb.mapping("bigram") if emb is not None else None
        if bf is not None:
            # the hash is formed in 64-bit integers from the multipliers' remainders: token ids below 2^20 times
            # remainders below 2^30
            bigram = SugosunBigram(bf.integer("buckets", hi=1 << 30), bf.integer("mul_prev", lo=0, hi=1 << 62),
                                   bf.integer("mul_cur", lo=0, hi=1 << 62))
        loop = None
        lp = f.mapping("loop")
        if lp is not None:
            start = lp.integer("start", lo=0, hi=len(layers))
            stop = lp.integer("stop", lo=start, hi=len(layers))
            loop = (start, stop, lp.integer("times", lo=1, hi=1 << 10))
        return SugosunConfig(
            architecture="Sugosun", vocab=f.integer("vocab"), width=f.integer("width"), eps=norm.number("eps", lo=0.0),
            bigram=bigram, streams=f.integer("streams", default=None, hi=64), layers=tuple(layers), loop=loop,
            max_position=f.integer("max_position", default=1 << 20, hi=1 << 30))


def _mlp(lf: Fields) -> Optional[SugosunMLP]:
    mlp = lf.mapping("mlp")
    if mlp is None:
        return None
    kind = mlp.string("kind", choices=MLPS)
    if kind == "dense":
        return SugosunMLP(kind, mlp.integer("ff"), limit=mlp.number("limit", lo=0.0, lo_open=True))
    ef, rf = mlp.mapping("expert"), mlp.mapping("router")
    if ef is None or rf is None:
        raise ConfigError(f"{mlp.where}: 'expert' and 'router' are required objects")
    experts = rf.integer("experts", hi=1 << 12)
    return SugosunMLP(kind, ef.integer("ff"), experts=experts, top=rf.integer("top", hi=experts))


def _mixer(kind: str, mf: Fields) -> SugosunMixer:
    heads, dim, vdim = mf.integer("heads"), mf.integer("dim"), mf.integer("vdim")
    if kind == "lightning":
        return SugosunMixer(kind, heads, dim, vdim, decay=mf.numbers("decay", count=heads, lo=0.0, hi=1.0))
    rot_dim = mf.integer("rot_dim", lo=0)
    rot = mf.mapping("rot")
    dims = rot.integer("dims", lo=0) if rot is not None else 0
    if dims % 2 or dims > rot_dim:
        raise ConfigError(f"{mf.where}: rot.dims = {dims} must be even and at most rot_dim = {rot_dim}")
    mask = mf.mapping("mask")
    return SugosunMixer(
        kind, heads, dim, vdim, rot_dim=rot_dim, q_rank=mf.integer("q_rank"), kv_rank=mf.integer("kv_rank"),
        scale=mf.number("scale"), rot_dims=dims,
        rot_base=rot.number("base", lo=0.0, lo_open=True) if rot is not None else 10000.0,
        window=mask.integer("size", default=None, hi=1 << 30) if mask is not None else None)
