"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.

One call runs only the tokens it is given, as one batch, against the cache
that earlier calls left: portions of prompts beside single decoded tokens,
cut anywhere.  The reference has two entry points for this, ``prefill`` and
``decode`` (``fastgen/forward.py:518-606``), over one ``_forward``; here there
is one, because a decoded token is a portion of length one.
"""

from __future__ import annotations

from typing import Dict, Hashable, List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage, group_entries
from .context import StepContext, StepEntry, build_context
from .model import Model


class ModelRunner:
    """A model with its cache: admits requests, steps them, lets them go.

    ``max_tokens`` is the number of tokens the pages of one group can hold
    (each live request's length counts rounded up to whole pages);
    ``max_requests`` is the number of state slots.
    """

    def __init__(self, model: Model, page_size: int = 64, max_tokens: int = 4096, max_requests: int = 64,
                 pages_per_group: Optional[Sequence[int]] = None) -> None:
        self.model = model
        self.page_size = page_size
        self.groups = group_entries(model.paged_needs())
        n_pages = -(-max_tokens // page_size)
        pages = list(pages_per_group) if pages_per_group is not None else [n_pages] * len(self.groups)
        self.cache = CacheManager(page_size, pages, [g.need.window for g in self.groups], max_requests)
        self.storage = CacheStorage(self.groups, pages, page_size, model.state_needs(), max_requests,
                                    model.dtype, model.device)
        self.stores = [
            self.storage.store_for(i, e.reads_cache_of) for i, e in enumerate(model.layout.order)
        ]
        self.last_context: Optional[StepContext] = None

    # ------------------------------------------------------------ requests
    def admit(self, rid: Hashable) -> int:
        slot = self.cache.admit(rid)
        self.storage.reset_slot(slot)
        return slot

    def release(self, rid: Hashable) -> None:
        self.cache.release(rid)

    def length(self, rid: Hashable) -> int:
        return self.cache.length(rid)

    # ---------------------------------------------------------------- step
    def prepare(self, entries: Sequence[StepEntry]) -> StepContext:
        """Admit new requests, reserve the pages of this step, build its context."""
        seen = set()
        for e in entries:
            if e.rid in seen:
                raise ValueError(f"request {e.rid!r} appears twice in one step")
            seen.add(e.rid)
            if not self.cache.is_live(e.rid):
                self.admit(e.rid)
        for e in entries:
            self.cache.reserve(e.rid, len(e.tokens))
        return build_context(entries, self.cache, self.model.dtype, self.model.device, self.model.vocab_size)

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """fp32 logits ``[n_wanted, vocab]`` in the order of the entries and
        of their ``want`` lists; None if nothing is wanted."""
        ctx = self.prepare(entries)
        self.last_context = ctx
        logits = self.model.forward(ctx, self.stores)
        for e in entries:
            self.cache.advance(e.rid, len(e.tokens))
        return logits
