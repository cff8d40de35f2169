"""Token embedding: one row of the table per token, as 32-bit rows of the residual
stream; an id outside the vocabulary reads row 0 (src/model.c:6148-6162).

``PairHashEmbedding`` adds a row of a second table that is found by a hash of the token and the
token before it, ``(prev * mul_prev + token * mul_cur) mod buckets`` (a sequence's first token, which
has none before it, reads the extra last row), and norms the sum (RMS, a weight).  The token before a
portion's first one is state of the request: one int32 a slot, kept by the cache storage.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import Part, ParamSpec, StateSpec, register_embedding


class TokenEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int, scale: float = 1.0, weight_name: str = "weight"):
        self.vocab_size, self.hidden_size, self.scale = int(vocab_size), int(hidden_size), float(scale)
        self.weight_name = weight_name
        self.weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        return {self.weight_name: ParamSpec((self.vocab_size, self.hidden_size), role="matrix")}

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        self.weight = tensors[self.weight_name]

    def share_table(self, table) -> None:
        """Gather from ``table`` from now on: the same values in another layout (a tied output
        head's packed copy), so that the model keeps the table once."""
        if tuple(table.shape) != (self.vocab_size, self.hidden_size):
            raise ValueError(f"a table of {tuple(table.shape)} cannot stand for one of {(self.vocab_size, self.hidden_size)}")
        self.weight = table

    def forward(self, ctx, token_ids):
        return self.rt.ops.embedding(self.weight, token_ids, self.scale)


class PairHashEmbedding(Part):
    def __init__(self, vocab_size: int, hidden_size: int, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0,
                 eps: float = 1e-6, weight_name: str = "weight", pairs_name: str = "pairs", norm_name: str = "norm",
                 has_norm: bool = True):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.buckets, self.mul_prev, self.mul_cur = int(buckets), int(mul_prev), int(mul_cur)   # buckets 0: no pair table
        self.eps, self.has_norm = float(eps), bool(has_norm)
        self.names = (weight_name, pairs_name, norm_name)
        self.weight = self.pairs = self.norm_weight = None

    def param_specs(self) -> Dict[str, ParamSpec]:
        w, p, n = self.names
        specs = {w: ParamSpec((self.vocab_size, self.hidden_size), role="matrix")}
        if self.buckets:
            # as large as the token's own row: a pair's row that is missing or wrong must show
            specs[p] = ParamSpec((self.buckets + 1, self.hidden_size), role="matrix")
        if self.has_norm:
            specs[n] = ParamSpec((self.hidden_size,), role="vector", init="ones_jitter")
        return specs

    def state_spec(self):
        """One int32 a request: the last token of the step before."""
        return StateSpec((), torch.int32) if self.buckets else None

    def bind(self, tensors, rt) -> None:
        self.rt = rt
        w, p, n = self.names
        self.weight = tensors[w]
        self.pairs = tensors[p] if self.buckets else None
        self.norm_weight = tensors[n].float().contiguous() if self.has_norm else None

    def forward(self, ctx, token_ids, state=None):
        if self.buckets and state is None:
            raise ValueError("an embedding that hashes token pairs needs the requests' last tokens")
        return self.rt.ops.embedding_pairs(self.weight, self.pairs, self.norm_weight, token_ids, ctx, state, self.buckets,
                                           self.mul_prev, self.mul_cur, self.eps)


register_embedding("token_embedding", TokenEmbedding)
register_embedding("pair_hash_embedding", PairHashEmbedding)
