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


@dataclass
class StepEntry:
    """One request's share of a step: its next tokens and the places among
    them whose logits are wanted."""

    rid: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()


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
    # host copies, for decisions about grids and kernels
    q_lens: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    n_cached: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    slot_ids_host: np.ndarray = field(default_factory=lambda: np.zeros(0, np.int32))
    n_out: int = 0

    @property
    def max_q_len(self) -> int:
        return int(self.q_lens.max()) if self.n_seqs else 0

    @property
    def max_kv_len(self) -> int:
        return int((self.q_lens + self.n_cached).max()) if self.n_seqs else 0


def build_context(entries: Sequence[StepEntry], cache: CacheManager, act_dtype: torch.dtype,
                  device: torch.device | str, vocab_size: Optional[int] = None) -> StepContext:
    """Host vectors for ``entries`` (whose pages are already reserved), packed
    into one int32 buffer and copied to the device once."""
    B = len(entries)
    q_lens = np.array([len(e.tokens) for e in entries], dtype=np.int32)
    if B == 0 or (q_lens <= 0).any():
        raise ValueError("a step needs at least one entry and every entry at least one token")
    n_cached = np.array([cache.length(e.rid) for e in entries], dtype=np.int32)
    q_start = np.zeros(B + 1, dtype=np.int32)
    np.cumsum(q_lens, out=q_start[1:])
    T = int(q_start[-1])
    tokens = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries])
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
    slot_ids = np.array([cache.slot(e.rid) for e in entries], dtype=np.int32)

    pieces = [tokens.astype(np.int32), positions, seq_of_token, q_start, (n_cached + q_lens).astype(np.int32),
              slot_ids, np.asarray(out_rows, dtype=np.int32)]
    tables = []
    for g in range(cache.n_groups):
        width = max(cache.n_table_entries(e.rid, g) for e in entries)
        tbl = np.zeros((B, max(1, width)), dtype=np.int32)
        slots = np.empty(T, dtype=np.int32)
        for b, e in enumerate(entries):
            row = cache.block_table(e.rid, g)
            tbl[b, : len(row)] = row
            slots[q_start[b] : q_start[b + 1]] = cache.write_slots(e.rid, g, int(n_cached[b]), int(q_lens[b]))
        tables.append(tbl.shape)
        pieces += [tbl.reshape(-1), slots]
    packed = torch.from_numpy(np.concatenate(pieces)).to(device)
    offs = np.cumsum([0] + [p.size for p in pieces])
    part = [packed[offs[i] : offs[i + 1]] for i in range(len(pieces))]
    groups = [
        GroupContext(cache.page_size, part[7 + 2 * g].view(tables[g]), part[8 + 2 * g])
        for g in range(cache.n_groups)
    ]
    return StepContext(
        n_tokens=T, n_seqs=B, act_dtype=act_dtype, tokens=part[0], positions=part[1], seq_of_token=part[2],
        q_start=part[3], kv_len=part[4], slot_ids=part[5], out_rows=part[6], groups=groups, q_lens=q_lens,
        n_cached=n_cached, slot_ids_host=slot_ids, n_out=len(out_rows),
    )
