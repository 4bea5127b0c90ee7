"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.

One call runs only the tokens it is given, as one batch, against the cache
that earlier calls left: portions of prompts beside single decoded tokens,
cut anywhere.  The reference has two entry points for this, ``prefill`` and
``decode`` (``fastgen/forward.py:518-606``), over one ``_forward``; here there
is one, because a decoded token is a portion of length one.
"""

from __future__ import annotations

import logging
import os
from typing import Dict, Hashable, Optional, Sequence, Tuple

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage, group_entries, tokens_for_free_memory
from ..kernels.ops import upload
from .context import StepContext, StepEntry, build_context, context_from_packed, pack_context
from .model import Model


def graph_capacity_for(n: int) -> int:
    """The number of sequences of the captured step that serves a decode batch
    of ``n``: every size up to 16, then steps of 8, 16 and 32, so that a few
    dozen captures cover hundreds of batch sizes (the reference spaces its 16
    graphs likewise and pads, ``fastgen/generate.py:296-352``)."""
    if n <= 16:
        return n
    step = 8 if n <= 64 else 16 if n <= 128 else 32
    return -(-n // step) * step


def graph_table_width_for(n_pages: int, limit: int) -> int:
    """The block-table width of the captured step that serves requests holding
    up to ``n_pages`` pages: powers of two from 16 on, at most ``limit`` (the
    widest a request can get).  The step's vectors are copied to the device at
    every replay: tables as wide as the cache would make that copy as large as
    the cache's page count times the batch."""
    w = 16
    while w < n_pages:
        w *= 2
    return max(1, min(w, limit))


logger = logging.getLogger("fastgen_amd")


class _DecodeGraph:
    """One captured decode step for a fixed number of sequences and a fixed
    width of their block tables.

    The step's int32 vectors live in a device buffer of fixed layout; a replay
    copies the new values in and runs the captured kernels, which read lengths
    and pages from that buffer.  A smaller batch is filled up with stand-in
    sequences that write nothing; a graph is captured when a batch of its
    capacity and table width first occurs.
    """

    def __init__(self, runner: "ModelRunner", entries: Sequence[StepEntry], table_width: int) -> None:
        model, cache = runner.model, runner.cache
        self.capacity = runner.graph_capacity(len(entries))
        self.table_width = table_width
        packed, offs, shapes, host = pack_context(entries, cache, model.vocab_size, table_width, self.capacity)
        self.layout = (tuple(int(o) for o in offs), tuple(shapes))
        # a ring of pinned staging buffers: the host may run several steps ahead of the device
        self.staging = [torch.empty(packed.size, dtype=torch.int32, pin_memory=True) for _ in range(runner.run_ahead)]
        self.copied = [torch.cuda.Event() for _ in range(runner.run_ahead)]
        self.turn = 0
        self.staging[0].numpy()[:] = packed
        self.packed = self.staging[0].to(model.device)
        self.ctx = context_from_packed(self.packed, offs, shapes, host, cache.page_size, model.dtype)
        self.ctx.graph_capacity = table_width * cache.page_size  # the longest sequence this step may meet
        # warm up outside the capture (libraries load, the matrix library picks its kernels), then capture.
        # The warm-up is a step of its own: keys and values that it writes are the ones the replay writes
        # again, but state of fixed size would move twice, so the rows of this step's slots are put back.
        rows = self.ctx.slot_ids.long()
        kept = {e: t.index_select(0, rows) for e, t in runner.storage.state.items()}
        side = torch.cuda.Stream(device=model.device)
        side.wait_stream(torch.cuda.current_stream(model.device))
        with torch.cuda.stream(side):
            model.forward(self.ctx, runner.stores)
        torch.cuda.current_stream(model.device).wait_stream(side)
        for e, t in runner.storage.state.items():
            t.index_copy_(0, rows, kept[e])
        torch.cuda.synchronize(model.device)
        # what the warm-up derived from this step's values (tables of sines, ...) is derived again
        # inside the capture, so that a replay derives it from its own values
        self.ctx.scratch.clear()
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, pool=runner.graph_pool):
            self.logits = model.forward(self.ctx, runner.stores)
        runner.graph_pool = runner.graph_pool or self.graph.pool()

    def replay(self, runner: "ModelRunner", entries: Sequence[StepEntry],
               tokens_on_device: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Copy the step's vectors in and run the captured step.  With
        ``tokens_on_device`` (int32 ``[B]``) the tokens come from there, not from
        ``entries``: the step before sampled them and the host has not seen them."""
        n = len(entries)
        packed, offs, shapes, host = pack_context(entries, runner.cache, None if tokens_on_device is not None
                                                  else runner.model.vocab_size, self.table_width, self.capacity)
        if (tuple(int(o) for o in offs), tuple(shapes)) != self.layout:
            raise RuntimeError("decode graph: the step's layout differs from the captured one")
        i = self.turn = (self.turn + 1) % len(self.staging)
        self.copied[i].synchronize()  # this staging buffer is free again
        self.staging[i].numpy()[:] = packed
        self.packed.copy_(self.staging[i], non_blocking=True)
        self.copied[i].record()
        if tokens_on_device is not None:
            self.ctx.tokens[:n].copy_(tokens_on_device)
        self.graph.replay()
        return self.logits[:n]


class ModelRunner:
    """A model with its cache: admits requests, steps them, lets them go.

    ``max_tokens`` is the number of tokens the pages of one group can hold
    (each live request's length counts rounded up to whole pages); None: as
    many as the device's free memory holds beside ``reserve_bytes``, at most
    ``at_most_tokens``.  ``max_requests`` is the number of state slots.
    """

    def __init__(self, model: Model, page_size: int = 64, max_tokens: Optional[int] = 4096, max_requests: int = 64,
                 pages_per_group: Optional[Sequence[int]] = None, reserve_bytes: int = 2 << 30,
                 at_most_tokens: Optional[int] = None) -> None:
        self.model = model
        self.page_size = page_size
        self.groups = group_entries(model.paged_needs())
        if max_tokens is None and pages_per_group is None:
            max_tokens = tokens_for_free_memory(self.groups, page_size, model.dtype, model.device, reserve_bytes,
                                                at_most_tokens, model.state_needs(), max_requests
                                                ) if self.groups else page_size
        n_pages = -(-max_tokens // page_size)
        pages = list(pages_per_group) if pages_per_group is not None else [n_pages] * len(self.groups)
        self.cache = CacheManager(page_size, pages, [g.need.window for g in self.groups], max_requests)
        self.storage = CacheStorage(self.groups, pages, page_size, model.state_needs(), max_requests,
                                    model.dtype, model.device)
        self.stores = [
            self.storage.store_for(i, e.reads_cache_of) for i, e in enumerate(model.layout.order)
        ]
        self.last_context: Optional[StepContext] = None
        # decode graphs: FG_NO_GRAPHS=1 switches them off (the reference: FG_NO_CUDA_GRAPHS); a model with a
        # part that cannot be recorded is stepped eagerly
        self.use_graphs = os.environ.get("FG_NO_GRAPHS", "0") in ("", "0") and model.capturable()
        self.table_width = max(1, max(pages, default=1))
        self.graphs: Dict[Tuple[int, int], _DecodeGraph] = {}  # (capacity, table width) -> step, oldest use first
        self.graph_pool = None
        self.graph_capacity = graph_capacity_for  # batch size -> sequences of the recorded step that serves it
        self.max_graphs = 64
        logger.info("weights %.2f GB%s; cache %s pages of %d tokens (%.2f GB), %d request slots; decode steps are %s",
                    model.weight_bytes() / 1e9, " (the matrices twice: rows and packed)" if model.packed() else "",
                    pages, page_size,
                    sum(t.numel() * t.element_size() for t in self.storage.k + self.storage.v) / 1e9, max_requests,
                    "recorded as graphs" if self.use_graphs else "run eagerly")
        self.run_ahead = 16  # steps the host may prepare before the device has run them

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

    def step(self, entries: Sequence[StepEntry], prev_tokens: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
        """fp32 logits ``[n_wanted, vocab]`` in the order of the entries and
        of their ``want`` lists; None if nothing is wanted.  The tensor may be
        the buffer of a captured step: it holds these logits until the next
        step; copy what is to be kept.  ``prev_tokens``: int32 tokens on the
        device that entries with ``from_row`` take their token from."""
        fill = self._token_fill(entries, prev_tokens)
        if self.use_graphs and self._is_plain_decode(entries):
            logits = self._graph_step(entries, fill)
        else:
            ctx = self.prepare(entries)
            self.last_context = ctx
            if fill is not None:
                ctx.tokens.index_copy_(0, fill[0], fill[1])
            logits = self.model.forward(ctx, self.stores)
        for e in entries:
            self.cache.advance(e.rid, len(e.tokens))
        return logits

    def _token_fill(self, entries: Sequence[StepEntry], prev_tokens: Optional[torch.Tensor]):
        """(flat token indices, their tokens) on the device for the entries whose token is still
        there, or None."""
        dst, src, at = [], [], 0
        for e in entries:
            if e.from_row is not None:
                if len(e.tokens) != 1:
                    raise ValueError(f"request {e.rid!r}: only a single token can come from the step before")
                dst.append(at)
                src.append(e.from_row)
            at += len(e.tokens)
        if not dst:
            return None
        if prev_tokens is None or prev_tokens.dtype != torch.int32:
            raise ValueError("entries name rows of the last step's tokens: give them as an int32 tensor")
        if max(src) >= prev_tokens.numel():
            raise ValueError("an entry names a row beyond the last step's tokens")
        idx = upload([dst, src], torch.int64, self.model.device)
        return idx[0], prev_tokens.index_select(0, idx[1])

    # ------------------------------------------------------- decode graphs
    def _is_plain_decode(self, entries: Sequence[StepEntry]) -> bool:
        """One token a request, its logits wanted, every request already live."""
        return bool(entries) and all(
            len(e.tokens) == 1 and list(e.want) == [0] and self.cache.is_live(e.rid) for e in entries
        ) and self.can_graph(len(entries))

    def can_graph(self, n: int) -> bool:
        """Whether decode batches run from captured steps."""
        return self.use_graphs and self.max_graphs > 0

    def _graph_for(self, entries: Sequence[StepEntry]) -> _DecodeGraph:
        """The captured step for these entries (whose pages are reserved): by batch capacity and
        block-table width.  At most ``max_graphs`` are kept; the one unused longest gives way."""
        held = max(self.cache.n_table_entries(e.rid, g) for e in entries for g in range(self.cache.n_groups))
        key = (self.graph_capacity(len(entries)), graph_table_width_for(held, self.table_width))
        g = self.graphs.pop(key, None)
        if g is None:
            while len(self.graphs) >= self.max_graphs:
                torch.cuda.synchronize(self.model.device)  # its last replay may still be running
                self.graphs.pop(next(iter(self.graphs)))
            g = _DecodeGraph(self, entries, key[1])
            logger.info("recorded a decode step for %d sequences, block tables %d pages wide (%d recorded steps)",
                        key[0], key[1], len(self.graphs) + 1)
        self.graphs[key] = g  # most recently used last
        return g

    def decode_run(self, entries: Sequence[StepEntry], n_steps: int, sample) -> torch.Tensor:
        """``n_steps`` decode steps of the same requests without the host seeing
        a token in between (``fastgen/generate.py:690-736``: ``sync_freq`` steps
        between host checks): each step's sampled tokens feed the next on the
        device.  ``entries`` bring each request's pending token; pages for all
        steps must be reservable.  ``sample(logits, step, out)`` writes the
        step's int32 tokens into ``out``.  Returns int32 ``[n_steps, B]`` on
        the device; the caller reads it once."""
        if not (self.use_graphs and self._is_plain_decode(entries)):
            raise RuntimeError("decode_run needs a plain decode step and decode graphs")
        n_steps = min(n_steps, self.run_ahead - 1)
        for e in entries:
            self.cache.reserve(e.rid, n_steps)
        g = self._graph_for(entries)
        out = torch.empty((n_steps, len(entries)), dtype=torch.int32, device=self.model.device)
        for s in range(n_steps):
            logits = g.replay(self, entries, out[s - 1] if s else None)
            sample(logits, s, out[s])
            for e in entries:
                self.cache.advance(e.rid, 1)
        return out

    def _graph_step(self, entries: Sequence[StepEntry], fill=None) -> torch.Tensor:
        if len({e.rid for e in entries}) != len(entries):
            raise ValueError("a request appears twice in one step")
        for e in entries:
            self.cache.reserve(e.rid, 1)
        tokens = None
        if fill is not None:  # some tokens are on the device: the replay takes all of them from there
            tokens = upload([e.tokens[0] for e in entries], torch.int32, self.model.device)
            tokens.index_copy_(0, fill[0], fill[1])
        # (a capture runs the step's kernels only as a recording: the replay gives this step's result)
        return self._graph_for(entries).replay(self, entries, tokens)
