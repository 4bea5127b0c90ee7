"""The ragged description of one step, on the host and on the device.

A step holds ``B`` sequences; sequence ``b`` has ``n_cached[b]`` tokens in the
cache and brings ``q_len[b] >= 1`` new ones, a prompt portion or one decoded
token alike (``fastgen/forward.py:518-573``: ``seq_info = [(n0, n1), ...]``).
The per-token vectors the kernels read (position, sequence, cache slot) are
built once on the host with numpy and reach the device in one copy.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager
from ..kernels.ops import upload


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places among
    them whose logits are wanted."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()
    # the entry's one token is row ``from_row`` of the tokens that the step before sampled and the
    # host has not seen (the step function is given that tensor); ``tokens`` then holds a stand-in
    from_row: Optional[int] = None


@dataclass
class GroupContext:
    page_size: int
    block_table: torch.Tensor  # int32 [B, max_pages]
    slots: torch.Tensor  # int32 [T]: page*P + offset where each token's k, v go


@dataclass
class StepContext:
    n_tokens: int
    n_seqs: int
    act_dtype: torch.dtype
    tokens: torch.Tensor  # int32 [T]
    positions: torch.Tensor  # int32 [T]
    seq_of_token: torch.Tensor  # int32 [T]
    q_start: torch.Tensor  # int32 [B+1]
    kv_len: torch.Tensor  # int32 [B]: keys of each sequence after this step
    slot_ids: torch.Tensor  # int32 [B]: state slot of each sequence
    out_rows: torch.Tensor  # int32 [n_out]: flat token rows whose logits are wanted
    groups: List[GroupContext]
    seq_records: Optional[torch.Tensor] = None  # int32 [B, 4]: sequence, first flat token, tokens, first position
    # host copies, for decisions about grids and kernels
    q_lens: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    n_cached: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    slot_ids_host: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    q_start_host: np.ndarray = field(default_factory=lambda: np.zeros(1, np.int32))
    n_out: int = 0
    # > 0: the context is the static one of a captured graph, replayed for requests of up to
    # this many tokens; sizes derived from it must not depend on this step's lengths
    graph_capacity: int = 0
    # per-step derived data that kernels' dispatchers compute once and share between layers
    scratch: dict = field(default_factory=dict)

    @property
    def max_q_len(self) -> int:
        return int(self.q_lens.max()) if self.n_seqs else 0

    @property
    def max_kv_len(self) -> int:
        return int((self.q_lens + self.n_cached).max()) if self.n_seqs else 0


def pack_context(entries: Sequence[StepEntry], cache: CacheManager, vocab_size: Optional[int] = None,
                 table_width: Optional[int] = None, pad_to: Optional[int] = None):
    """Host side of :func:`build_context`: every int32 vector of the step in
    one numpy buffer, and where each lies in it.  With ``table_width`` the block
    tables have that many columns whatever the requests hold, so that steps of
    the same batch shape have the same layout.  With ``pad_to`` the batch is
    filled up to that many sequences with stand-ins of one token at position 0
    that write nothing to the cache (slot -1), own no page (their block
    table rows name page 0, which they only read) and have the state row
    behind the last slot, which is nobody's: a captured step of
    ``pad_to`` sequences then serves any smaller batch; the stand-ins' logits
    are the last rows and mean nothing."""
    n_real = len(entries)
    q_lens = np.array([len(e.tokens) for e in entries], dtype=np.int32)
    if n_real == 0 or (q_lens <= 0).any():
        raise ValueError("a step needs at least one entry and every entry at least one token")
    n_pad = max(0, (pad_to or 0) - n_real)
    B = n_real + n_pad
    q_lens = np.concatenate([q_lens, np.ones(n_pad, dtype=np.int32)])
    n_cached = np.array([cache.length(e.rid) for e in entries] + [0] * n_pad, dtype=np.int32)
    q_start = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(q_lens, out=q_start[1:])
    T = int(q_start[-1])
    tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries] + [np.zeros(n_pad, dtype=np.int64)])
    if (tokens < 0).any() or (vocab_size is not None and (tokens >= vocab_size).any()):
        raise ValueError(f"token id outside [0, {vocab_size})")
    seq_of_token = np.repeat(np.arange(B, dtype=np.int32), q_lens)
    positions = (np.arange(T, dtype=np.int32) - q_start[seq_of_token] + n_cached[seq_of_token]).astype(np.int32)
    out_rows: List[int] = []
    for b, e in enumerate(entries):
        for w in e.want:
            if not 0 <= w < q_lens[b]:
                raise ValueError(f"request {e.rid!r}: wanted place {w} is outside its {q_lens[b]} tokens")
            out_rows.append(int(q_start[b]) + int(w))
    out_rows += [int(q_start[b]) for b in range(n_real, B)]
    # stand-ins keep their state in the row behind the last slot, which belongs to no request
    slot_ids = np.array([cache.slot(e.rid) for e in entries] + [cache.n_slots] * n_pad, dtype=np.int32)

    # one record per sequence (sequence, first flat token, tokens, first position): the items of the
    # attention kernels when every sequence brings so few tokens that it is one item; first in the
    # buffer, so 16-byte aligned
    records = np.stack([np.arange(B, dtype=np.int32), q_start[:-1], q_lens, n_cached], axis=1).astype(np.int32)
    pieces = [records.reshape(-1), tokens.astype(np.int32), positions, seq_of_token, q_start,
              (n_cached + q_lens).astype(np.int32), slot_ids, np.asarray(out_rows, dtype=np.int32)]
    table_shapes = []
    for g in range(cache.n_groups):
        width = max(len(cache.pages_of(e.rid, g)) for e in entries)
        if table_width is not None:
            if width > table_width:
                raise ValueError(f"a request holds {width} pages, the fixed table width is {table_width}")
            width = table_width
        tbl = np.zeros((B, max(1, width)), dtype=np.int32)
        slots = np.full(T, -1, dtype=np.int32)
        for b, e in enumerate(entries):
            row = cache.pages_of(e.rid, g)
            tbl[b, : len(row)] = row
            if q_lens[b] == 1:
                slots[q_start[b]] = cache.write_slot(e.rid, g, int(n_cached[b]))
            else:
                slots[q_start[b] : q_start[b + 1]] = cache.write_slots(e.rid, g, int(n_cached[b]), int(q_lens[b]))
        table_shapes.append(tbl.shape)
        pieces += [tbl.reshape(-1), slots]
    offs = np.cumsum([0] + [p.size for p in pieces])
    host = dict(q_lens=q_lens, n_cached=n_cached, slot_ids=slot_ids, q_start=q_start, n_out=len(out_rows))
    return np.concatenate(pieces), offs, table_shapes, host


def context_from_packed(packed: torch.Tensor, offs, table_shapes, host, page_size: int,
                        act_dtype: torch.dtype) -> StepContext:
    """Views into the device copy of a packed buffer."""
    part = [packed[offs[i] : offs[i + 1]] for i in range(len(offs) - 1)]
    groups = [
        GroupContext(page_size, part[8 + 2 * g].view(table_shapes[g]), part[9 + 2 * g])
        for g in range(len(table_shapes))
    ]
    return StepContext(
        n_tokens=int(host["q_start"][-1]), n_seqs=len(host["q_lens"]), act_dtype=act_dtype,
        seq_records=part[0].view(-1, 4), tokens=part[1],
        positions=part[2], seq_of_token=part[3], q_start=part[4], kv_len=part[5], slot_ids=part[6],
        out_rows=part[7], groups=groups, q_lens=host["q_lens"], n_cached=host["n_cached"],
        slot_ids_host=host["slot_ids"], q_start_host=host["q_start"], n_out=host["n_out"],
    )


def build_context(entries: Sequence[StepEntry], cache: CacheManager, act_dtype: torch.dtype,
                  device: torch.device | str, vocab_size: Optional[int] = None) -> StepContext:
    """Host vectors for ``entries`` (whose pages are already reserved), packed
    into one int32 buffer and copied to the device once."""
    packed, offs, table_shapes, host = pack_context(entries, cache, vocab_size)
    return context_from_packed(upload(packed, torch.int32, device), offs, table_shapes, host, cache.page_size,
                               act_dtype)
