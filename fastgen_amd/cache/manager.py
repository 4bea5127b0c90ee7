"""Host-side bookkeeping of the cache: pages, block tables, state slots.

The reference keeps one free-page set and one ordered page list per lane and
frees a lane's pages all at once (``fastgen/generate.py:291, 505, 591-595,
898-932``; ``fastgen/utils/iset.py``).  Here layers with the same storage need
form a *group*; each group has pages of its own and a block table per
request.  A group with a window gives a page back as soon as every key in it
is behind the window of all tokens still to come.  Freed pages go on top of a
stack, so the page freed last is the first to be used again.  Beside the
pages, every live request holds one *state slot* for per-request state of
fixed size.

Nothing here touches a device: the device tensors that the pages and slots
index live in ``storage.py``.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Hashable, List, Optional, Sequence

import numpy as np

RELEASED = -1  # block-table entry of a page that a window has passed


class OutOfPages(RuntimeError):
    """A reservation needs more free pages than a group has."""


class OutOfSlots(RuntimeError):
    """Every state slot is held by a live request."""


@dataclass
class _RequestCache:
    slot: int
    length: int = 0  # tokens whose keys are in the cache
    pages: List[List[int]] = field(default_factory=list)  # [group][logical page] -> page or RELEASED


class CacheManager:
    def __init__(self, page_size: int, pages_per_group: Sequence[int],
                 windows: Sequence[Optional[int]], n_slots: int) -> None:
        if page_size <= 0 or page_size % 8:
            raise ValueError(f"page_size={page_size} must be a positive multiple of 8")
        if len(pages_per_group) != len(windows):
            raise ValueError("one page count and one window per group are needed")
        self.page_size = page_size
        self.n_groups = len(windows)
        self.windows = [w if w else None for w in windows]
        self.n_pages = list(pages_per_group)
        # stacks: pop() takes the page freed last; initially page 0 is on top
        self._free: List[List[int]] = [list(range(n - 1, -1, -1)) for n in self.n_pages]
        self.n_slots = n_slots
        self._free_slots: List[int] = list(range(n_slots - 1, -1, -1))
        self._live: Dict[Hashable, _RequestCache] = {}

    # ------------------------------------------------------------ requests
    def admit(self, rid: Hashable) -> int:
        """Give ``rid`` a state slot and empty block tables; returns the slot."""
        if rid in self._live:
            raise KeyError(f"request {rid!r} is already live")
        if not self._free_slots:
            raise OutOfSlots(f"all {self.n_slots} state slots are in use")
        rc = _RequestCache(slot=self._free_slots.pop(), pages=[[] for _ in range(self.n_groups)])
        self._live[rid] = rc
        return rc.slot

    def is_live(self, rid: Hashable) -> bool:
        return rid in self._live

    def live_requests(self) -> List[Hashable]:
        return list(self._live)

    def length(self, rid: Hashable) -> int:
        return self._live[rid].length

    def slot(self, rid: Hashable) -> int:
        return self._live[rid].slot

    def free_pages(self, group: int = 0) -> int:
        return len(self._free[group])

    def free_slots(self) -> int:
        return len(self._free_slots)

    # ------------------------------------------------------------ pages
    def _first_needed_page(self, group: int, first_query_pos: int) -> int:
        """Lowest logical page that a query at ``first_query_pos`` still reads."""
        w = self.windows[group]
        if w is None:
            return 0
        return max(0, first_query_pos - w + 1) // self.page_size

    def pages_needed(self, rid: Hashable, n_new: int) -> List[int]:
        """Pages each group would have to take from its free stack to hold
        ``n_new`` more tokens of ``rid``."""
        rc = self._live[rid]
        total = -(-(rc.length + n_new) // self.page_size)
        return [max(0, total - len(rc.pages[g])) for g in range(self.n_groups)]

    def pages_needed_fresh(self, n_tokens: int, group: int = 0) -> int:
        """Pages a request holds in ``group`` right after a step has brought it
        from nothing to ``n_tokens`` tokens (the whole prompt in one step needs
        them all at once, window or not)."""
        return -(-n_tokens // self.page_size)

    def can_reserve(self, rid: Hashable, n_new: int) -> bool:
        need = self.pages_needed(rid, n_new)
        return all(need[g] <= len(self._free[g]) for g in range(self.n_groups))

    def reserve(self, rid: Hashable, n_new: int) -> None:
        """Make sure pages exist for positions ``length .. length+n_new-1`` in
        every group; takes all of them or none."""
        need = self.pages_needed(rid, n_new)
        for g in range(self.n_groups):
            if need[g] > len(self._free[g]):
                raise OutOfPages(
                    f"request {rid!r} needs {need[g]} more pages in cache group {g},"
                    f" {len(self._free[g])} are free"
                )
        rc = self._live[rid]
        for g in range(self.n_groups):
            for _ in range(need[g]):
                rc.pages[g].append(self._free[g].pop())

    def advance(self, rid: Hashable, n_new: int) -> None:
        """``n_new`` tokens were written; pages a window has passed go back."""
        rc = self._live[rid]
        room = min((len(p) for p in rc.pages), default=None)
        if room is not None and rc.length + n_new > room * self.page_size:
            raise RuntimeError(f"request {rid!r}: {n_new} tokens written without reserved pages")
        rc.length += n_new
        for g in range(self.n_groups):
            if self.windows[g] is None:
                continue
            keep_from = self._first_needed_page(g, rc.length)
            pages = rc.pages[g]
            for j in range(min(keep_from, len(pages))):
                if pages[j] != RELEASED:
                    self._free[g].append(pages[j])
                    pages[j] = RELEASED

    def release(self, rid: Hashable) -> None:
        """The request ends (or is preempted): everything it holds goes back."""
        rc = self._live.pop(rid)
        for g in range(self.n_groups):
            for p in rc.pages[g]:
                if p != RELEASED:
                    self._free[g].append(p)
        self._free_slots.append(rc.slot)

    # ------------------------------------------------------------ tables
    def block_table(self, rid: Hashable, group: int = 0) -> List[int]:
        return list(self._live[rid].pages[group])

    def n_table_entries(self, rid: Hashable, group: int = 0) -> int:
        return len(self._live[rid].pages[group])

    def pages_of(self, rid: Hashable, group: int = 0) -> List[int]:
        """The request's own page list (not a copy; do not change it)."""
        return self._live[rid].pages[group]

    def write_slot(self, rid: Hashable, group: int, pos: int) -> int:
        """:meth:`write_slots` for one position."""
        page = self._live[rid].pages[group][pos // self.page_size]
        if page < 0:
            raise RuntimeError(f"request {rid!r}: position in a released page of group {group}")
        return page * self.page_size + pos % self.page_size

    def write_slots(self, rid: Hashable, group: int, start: int, n: int) -> np.ndarray:
        """Flat token slots ``page*page_size + offset`` of positions
        ``start .. start+n-1`` (which must be reserved)."""
        pages = np.asarray(self._live[rid].pages[group], dtype=np.int64)
        pos = np.arange(start, start + n, dtype=np.int64)
        page = pages[pos // self.page_size]
        if (page < 0).any():
            raise RuntimeError(f"request {rid!r}: position in a released page of group {group}")
        return (page * self.page_size + pos % self.page_size).astype(np.int32)

    # ------------------------------------------------------------ checks
    def check(self) -> None:
        """Every page and slot is either free or held by exactly one request."""
        for g in range(self.n_groups):
            held = [p for rc in self._live.values() for p in rc.pages[g] if p != RELEASED]
            seen = held + self._free[g]
            if len(seen) != len(set(seen)):
                raise AssertionError(f"group {g}: a page is held or free twice")
            if set(seen) != set(range(self.n_pages[g])):
                raise AssertionError(f"group {g}: pages lost: {set(range(self.n_pages[g])) - set(seen)}")
            for rid, rc in self._live.items():
                pages = rc.pages[g]
                if len(pages) < -(-rc.length // self.page_size):
                    raise AssertionError(f"{rid!r} holds too few pages in group {g}")
                lo = self._first_needed_page(g, rc.length)
                if any(p == RELEASED for p in pages[lo:]):
                    raise AssertionError(f"{rid!r}: a page still inside the window was released")
        slots = [rc.slot for rc in self._live.values()] + self._free_slots
        if len(slots) != len(set(slots)) or set(slots) != set(range(self.n_slots)):
            raise AssertionError("a state slot is lost or held twice")
