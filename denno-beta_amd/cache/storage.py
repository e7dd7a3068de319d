"""CacheStorage: the device memory behind the cache manager, and its grouping.

Each cache that the model's run order names has a need (PagedKV or FixedState, from its
mixer).  Caches with the same need form a group: a paged group has one pool of pages,
[caches, n_pages, Hkv, page_size, dh] for keys and [caches, n_pages, Hkv, dv, page_size] for
values (a page's values transposed, as attention's second product reads them; dv is dh unless
the need names a width of its own for values), and one block table per request, shared by the group's caches; a state group has [caches, slots, *shape] and is
indexed by the request's slot.  Groups with different needs (all keys, a window of them)
draw from pools of their own.
"""
from __future__ import annotations

from typing import List, Sequence

import torch

from ..parts.base import FixedState, PagedKV
from ..parts.model import CacheView
from .manager import PAGED, STATE, CacheManager, GroupLayout

_TORCH = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class CacheStorage:
    def __init__(self, cache_specs: Sequence, *, kv_dtype: torch.dtype, page_size: int, cache_tokens: int,
                 max_live: int, device, allocate: bool = True):
        """cache_specs[i]: the need of cache i (PagedKV, FixedState or None).  kv_dtype: what pages hold
        whose PagedKV names no dtype of its own."""
        self.page_size, self.max_live, self.device, self.kv_dtype = page_size, max_live, device, kv_dtype
        self.group_specs: List = []
        self.members: List[List[int]] = []
        self.where = []                       # cache index -> (group, index in group)
        for i, cs in enumerate(cache_specs):
            if cs is None:
                self.where.append((-1, 0))
                continue
            if cs not in self.group_specs:
                self.group_specs.append(cs)
                self.members.append([])
            g = self.group_specs.index(cs)
            self.where.append((g, len(self.members[g])))
            self.members[g].append(i)
        n_pages = max(1, -(-cache_tokens // page_size))
        layouts = []
        for cs in self.group_specs:
            if isinstance(cs, PagedKV):
                layouts.append(GroupLayout(PAGED, n_pages, page_size, cs.window))
            elif isinstance(cs, FixedState):
                layouts.append(GroupLayout(STATE))
            else:
                raise TypeError(f"unknown cache need {cs!r}")
        self.layouts = layouts
        self.manager = CacheManager(layouts, max_live)
        self.k, self.v, self.state = [], [], []
        for g, cs in enumerate(self.group_specs):
            n = len(self.members[g])
            if isinstance(cs, PagedKV):
                shape = (n, n_pages, cs.n_kv_heads, page_size, cs.head_dim)
                vshape = (n, n_pages, cs.n_kv_heads, cs.v_dim, page_size)   # a page's values transposed
                dt = _TORCH[cs.dtype] if cs.dtype is not None else kv_dtype
                if allocate:
                    # zeros, not empty: a page's unwritten tail is read (masked) by attention,
                    # and must hold numbers, not whatever bits the allocator left
                    self.k.append(torch.zeros(shape, dtype=dt, device=device))
                    self.v.append(torch.zeros(vshape, dtype=dt, device=device))
                else:
                    self.k.append(None), self.v.append(None)
                self.state.append(None)
            else:
                self.k.append(None), self.v.append(None)
                self.state.append(torch.zeros((n, max_live) + tuple(cs.shape), dtype=_TORCH[cs.dtype],
                                              device=device) if allocate else None)

    @property
    def n_groups(self):
        return len(self.group_specs)

    def paged_groups(self):
        return [g for g, cs in enumerate(self.group_specs) if isinstance(cs, PagedKV)]

    def view(self, cache_index: int, writes: bool) -> CacheView:
        g, j = self.where[cache_index]
        if g < 0:
            return CacheView(group=-1, writes=writes)
        if isinstance(self.group_specs[g], PagedKV):
            return CacheView(group=g, writes=writes, k=self.k[g][j], v=self.v[g][j])
        return CacheView(group=g, writes=writes, state=self.state[g][j])

    def start_request(self, rid: int) -> int:
        """A slot for the request; its fixed-size states start at zero."""
        slot = self.manager.add(rid)
        for st in self.state:
            if st is not None:
                st[:, slot].zero_()
        return slot

    def reset_states(self, slot: int):
        for st in self.state:
            if st is not None:
                st[:, slot].zero_()

    def bytes_per_token(self) -> int:
        total = 0
        for g, cs in enumerate(self.group_specs):
            if isinstance(cs, PagedKV):
                dt = _TORCH[cs.dtype] if cs.dtype is not None else self.kv_dtype
                total += len(self.members[g]) * cs.n_kv_heads * (cs.head_dim + cs.v_dim) * torch.empty((), dtype=dt).element_size()
        return total
