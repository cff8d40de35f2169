"""The device memory behind the cache manager.

For every entry of the run order that owns a cache: keys ``[pages, Hk, page_size, D]``
and values ``[pages, Hk, D, page_size]`` (values transposed inside a page so that
attention reads several positions of one channel with one load), in the engine's
dtype.  A layer that keeps block means (``KVSpec.pooled``) has a second pair of tensors of the
same layout in the group of its blocks.  For every tensor of fixed-size state a layer names:
``[slots + 1, *shape]``; row ``null_slot`` (the last) belongs to no request.
Page 0 is the null page.  Nothing is zeroed when a page changes hands: reads are
bounded by a request's length, so a page's old contents are never seen.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Union

import torch

from ..parts.base import KVSpec, StateSpec


@dataclass
class LayerCache:
    """What one entry of the run order sees of the cache."""
    group: int                 # which block table of a request applies
    page_size: int
    owns: bool                 # this entry writes keys and values (False: it reads another entry's)
    k: Optional[torch.Tensor]
    v: Optional[torch.Tensor]
    state: Optional[torch.Tensor] = None    # [slots + 1, *shape]; the last row is nobody's (the mixer's own, if it has one)
    states: Dict[str, torch.Tensor] = field(default_factory=dict)     # every state tensor of the layer by name
    pool_group: int = -1                    # the block table of the block means, for a layer that keeps them
    pool_k: Optional[torch.Tensor] = None   # [pages, Hk, page_size, D]: entry b of a request is block b's mean key
    pool_v: Optional[torch.Tensor] = None   # [pages, Hk, Dv, page_size]
    pool_owns: bool = False                 # this entry writes the block means (False: another entry's are the same)


class CacheStorage:
    def __init__(self, kv_specs: List[Optional[KVSpec]], state_specs: List[Optional[StateSpec]],
                 cache_of: List[Optional[int]], page_size: int,
                 pages_per_group: Union[int, Callable[[KVSpec], int]], n_slots: int,
                 dtype: torch.dtype, device: torch.device, model_states: Optional[Dict[str, StateSpec]] = None):
        """``kv_specs[i]``/``state_specs[i]``/``cache_of[i]`` describe entry ``i`` of the run order.
        ``pages_per_group``: one number for every group, or a function of a group's ``KVSpec``
        (a group that keeps a window of keys needs fewer pages than one that keeps them all)."""
        self.page_size, self.n_slots = page_size, n_slots
        sized = pages_per_group if callable(pages_per_group) else (lambda spec: pages_per_group)
        self.null_slot = n_slots
        self.group_specs: List[KVSpec] = []
        self.group_pages: List[int] = []        # usable pages of each group (the null page comes on top)
        self.layers: List[LayerCache] = []

        def group_of(spec: KVSpec) -> int:
            if spec not in self.group_specs:
                self.group_specs.append(spec)
                self.group_pages.append(max(1, int(sized(spec))))
            return self.group_specs.index(spec)

        def pages_of(spec: KVSpec):
            n_pages = self.group_pages[group_of(spec)] + 1
            return (torch.zeros((n_pages, spec.num_kv_heads, page_size, spec.head_dim), dtype=dtype, device=device),
                    torch.zeros((n_pages, spec.num_kv_heads, spec.value_dim, page_size), dtype=dtype, device=device))

        def states_of(st) -> Dict[str, torch.Tensor]:
            # one row more than requests: the last is nobody's (rows that pad a recorded step use it)
            named = {} if st is None else ({"mixer": st} if isinstance(st, StateSpec) else dict(st))
            return {name: torch.zeros((n_slots + 1,) + tuple(s.shape), dtype=s.dtype or dtype, device=device)
                    for name, s in named.items()}

        # per-request state that belongs to no layer (an embedding's, say), by name
        self.model_states: Dict[str, torch.Tensor] = states_of(dict(model_states) if model_states else None)

        for i, (kv, st) in enumerate(zip(kv_specs, state_specs)):
            owner = cache_of[i]
            states = states_of(st)
            if owner is not None:
                src = self.layers[owner]
                if kv is not None and src.k is not None:
                    okv = kv_specs[owner]
                    if (okv.num_kv_heads, okv.head_dim, okv.value_dim) != (kv.num_kv_heads, kv.head_dim, kv.value_dim):
                        raise ValueError(f"run order entry {i} reads the cache of entry {owner}, "
                                         f"whose heads or head size differ")
                    # the owner's window decides which pages exist: a reader that looks further
                    # back would look up pages that were given back
                    if okv.window is not None and (kv.window is None or kv.window > okv.window):
                        raise ValueError(f"run order entry {i} (window {kv.window}) reads the cache of entry {owner}, "
                                         f"which keeps only the last {okv.window} keys")
                lc = LayerCache(src.group, page_size, False, src.k, src.v, states.get("mixer"), states)
                if kv is not None and kv.pooled:
                    # block means of the owner's keys: the owner's own where its blocks are as long,
                    # else a cache of this entry's making
                    if src.pool_k is not None and kv_specs[owner].pooled == kv.pooled:
                        lc.pool_group, lc.pool_k, lc.pool_v = src.pool_group, src.pool_k, src.pool_v
                    else:
                        ps = kv.pooled_spec()
                        lc.pool_group, lc.pool_owns = group_of(ps), True
                        lc.pool_k, lc.pool_v = pages_of(ps)
                self.layers.append(lc)
                continue
            group, k, v = -1, None, None
            if kv is not None:
                group = group_of(kv)
                k, v = pages_of(kv)
            lc = LayerCache(group, page_size, True, k, v, states.get("mixer"), states)
            if kv is not None and kv.pooled:
                ps = kv.pooled_spec()
                lc.pool_group, lc.pool_owns = group_of(ps), True
                lc.pool_k, lc.pool_v = pages_of(ps)
            self.layers.append(lc)

    def bytes_per_token(self) -> int:
        total = 0
        for lc in self.layers:
            if lc.owns and lc.k is not None:
                total += lc.k.shape[1] * (lc.k.shape[3] + lc.v.shape[2]) * lc.k.element_size()
        return total
