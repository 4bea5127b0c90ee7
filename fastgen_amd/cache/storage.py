"""Device tensors behind the cache manager's pages and slots.

Per cache group one K pool ``[n_layers, n_pages, KV, P, hd]`` and one V pool
``[n_layers, n_pages, KV, hd_v, P]`` (``hd_v`` = ``hd`` unless the group's need says otherwise): a page of one layer's keys is ``P`` rows of
``hd`` contiguous elements per head; a page of values is stored transposed so
that the keys of a page are contiguous for one head dimension.  (The
reference keeps per layer ``[n_pages*P, KV, hd]`` for both,
``fastgen/cache.py:66-78``.)  Pages are not cleared when they change hands:
what a page holds beyond a request's length is never read.

Per-request state of fixed size lives in ``[n_slots + 1, *shape]`` tensors, one
per run entry that asked for it, cleared when a slot is handed out (the last
row is nobody's: stand-in sequences of a captured step use it).
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..parts.base import LayerStore, PagedNeed, StateNeed


@dataclass(frozen=True)
class CacheGroup:
    need: PagedNeed
    entries: Tuple[int, ...]  # run-order indices that own pages in this group


def group_entries(needs: Sequence[Optional[PagedNeed]]) -> List[CacheGroup]:
    """Run entries with equal needs share a group (and so a block table)."""
    by_need: Dict[PagedNeed, List[int]] = {}
    for i, n in enumerate(needs):
        if n is not None:
            by_need.setdefault(n, []).append(i)
    return [CacheGroup(n, tuple(e)) for n, e in by_need.items()]


def bytes_per_token(groups: Sequence[CacheGroup], dtype: torch.dtype) -> int:
    """Cache bytes one token takes over all layers of all groups."""
    esize = torch.empty((), dtype=dtype).element_size()
    return sum(len(g.entries) * g.need.n_kv_heads * (g.need.head_dim + g.need.value_dim) * esize for g in groups)


def state_bytes(state_needs: Dict[int, StateNeed], n_slots: int) -> int:
    """Bytes of the per-request state tensors for ``n_slots`` slots (and the one row that is nobody's)."""
    total = 0
    for need in state_needs.values():
        n = 1
        for d in need.shape:
            n *= int(d)
        total += (n_slots + 1) * n * torch.empty((), dtype=need.dtype).element_size()
    return total


def tokens_that_fit(free_bytes: int, groups: Sequence[CacheGroup], page_size: int, dtype: torch.dtype,
                    reserve_bytes: int, state_needs: Optional[Dict[int, StateNeed]] = None, n_slots: int = 0,
                    at_most: Optional[int] = None) -> int:
    """Tokens of cache, a whole number of pages, that ``free_bytes`` hold beside ``reserve_bytes`` and the
    state tensors of ``n_slots`` requests (0: less than one page fits)."""
    per_token = max(1, bytes_per_token(groups, dtype))
    left = free_bytes - reserve_bytes - state_bytes(state_needs or {}, n_slots)
    tokens = max(0, int(left // per_token))
    if at_most is not None:
        tokens = min(tokens, at_most)
    return tokens // page_size * page_size


def tokens_for_free_memory(groups: Sequence[CacheGroup], page_size: int, dtype: torch.dtype,
                           device: torch.device | str, reserve_bytes: int, at_most: Optional[int] = None,
                           state_needs: Optional[Dict[int, StateNeed]] = None, n_slots: int = 0) -> int:
    """The cache that the device's free memory holds beside ``reserve_bytes`` (activations of the
    largest step, captured steps, the libraries' work space) and beside the per-request state of
    ``n_slots`` requests, in tokens, a whole number of pages.
    The reference sizes its cache from a memory budget the same way (``fastgen/utils/tune.py:68-84``,
    ``fastgen/generate.py:224-238``); here the budget is what the device reports as free now, after
    the weights are in place.  ``at_most``: no more than this many tokens are ever needed."""
    free, _total = torch.cuda.mem_get_info(torch.device(device))
    # what torch's allocator holds but does not use is free for the pools as well
    free += torch.cuda.memory_reserved(device) - torch.cuda.memory_allocated(device)
    tokens = tokens_that_fit(free, groups, page_size, dtype, reserve_bytes, state_needs, n_slots, at_most)
    if tokens < page_size:
        per_token = max(1, bytes_per_token(groups, dtype))
        raise RuntimeError(
            f"no room for one cache page: {free / 1e9:.2f} GB are free on {device}, {reserve_bytes / 1e9:.2f} GB"
            f" are kept for the steps' activations, {state_bytes(state_needs or {}, n_slots) / 1e9:.2f} GB for the"
            f" requests' state, a page of {page_size} tokens takes {per_token * page_size / 1e6:.2f} MB"
        )
    return tokens


class CacheStorage:
    def __init__(self, groups: Sequence[CacheGroup], pages_per_group: Sequence[int], page_size: int,
                 state_needs: Dict[int, StateNeed], n_slots: int, dtype: torch.dtype,
                 device: torch.device | str) -> None:
        self.groups = list(groups)
        self.page_size = page_size
        self.k: List[torch.Tensor] = []
        self.v: List[torch.Tensor] = []
        self._where: Dict[int, Tuple[int, int]] = {}  # run entry -> (group, layer index in group)
        for g, (grp, n_pages) in enumerate(zip(self.groups, pages_per_group)):
            kv, hd = grp.need.n_kv_heads, grp.need.head_dim
            n = len(grp.entries)
            self.k.append(torch.empty((n, n_pages, kv, page_size, hd), dtype=dtype, device=device))
            self.v.append(torch.empty((n, n_pages, kv, grp.need.value_dim, page_size), dtype=dtype, device=device))
            for j, e in enumerate(grp.entries):
                self._where[e] = (g, j)
        # one row more than there are slots: row ``n_slots`` belongs to nobody.  The stand-in sequences that
        # fill a captured step up to its capacity keep their state there, so that no request's state moves.
        self.scratch_slot = n_slots
        self.state: Dict[int, torch.Tensor] = {
            e: torch.zeros((n_slots + 1, *need.shape), dtype=need.dtype, device=device)
            for e, need in state_needs.items()
        }

    def store_for(self, entry: int, owner: Optional[int] = None) -> LayerStore:
        """Storage of run entry ``entry``; with ``owner`` the storage of that
        earlier entry, read only."""
        src = entry if owner is None else owner
        st = LayerStore(owns=owner is None)
        if src in self._where:
            g, j = self._where[src]
            st.group, st.k_pages, st.v_pages = g, self.k[g][j], self.v[g][j]
        st.state = self.state.get(src)
        return st

    def reset_slot(self, slot: int) -> None:
        for t in self.state.values():
            t[slot].zero_()

    def bytes_per_token(self) -> int:
        """Cache bytes one token takes over all layers (``fastgen/cache.py`` ``bytes_per_token``)."""
        return bytes_per_token(self.groups, self.k[0].dtype) if self.k else 0
