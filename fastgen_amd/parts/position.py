"""Position encodings.

``Rope`` is the rotary encoding of ``fastgen/kernels/rope.py:56-89`` with the
frequency table of ``fastgen/forward.py:609-635`` (optionally the llama3
piecewise scaling).  The kernel rotates interleaved pairs ``(2i, 2i+1)``;
checkpoints store q/k projections for the half-split pairing ``(i, i+hd/2)``,
so their rows are permuted once at load (``fastgen/utils/loading.py:296-305``).
"""

from __future__ import annotations

import math
from typing import Optional

import torch

from .base import PositionEncoding, register_part


class Rope(PositionEncoding):
    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.head_dim = int(o["head_dim"])
        self.rotary_dim = int(o.get("rotary_dim", self.head_dim))
        if self.rotary_dim % 2 or not 0 <= self.rotary_dim <= self.head_dim:
            raise ValueError(f"rotary_dim={self.rotary_dim} must be even and at most head_dim={self.head_dim}")
        self.theta = float(o["theta"])
        self.scaled = bool(o.get("scaled", False))
        self.original_context = int(o.get("original_context", 0))
        self.factor = float(o.get("factor", 1.0))
        self.low_freq_factor = float(o.get("low_freq_factor", 1.0))
        self.high_freq_factor = float(o.get("high_freq_factor", 1.0))

    def frequencies(self) -> Optional[torch.Tensor]:
        """fp32 ``[rotary_dim/2]``: ``1/theta^(2i/rotary_dim)``, then per
        frequency by wavelength ``2 pi / f``: longer than
        ``ctx/low_freq_factor`` divided by ``factor``; between that and
        ``ctx/high_freq_factor`` blended; shorter unchanged."""
        if self.rotary_dim == 0:
            return None
        exponents = torch.arange(0, self.rotary_dim, 2, dtype=torch.float32) / self.rotary_dim
        freqs = 1.0 / (self.theta ** exponents)
        if not self.scaled:
            return freqs
        long_edge = self.original_context / self.low_freq_factor
        short_edge = self.original_context / self.high_freq_factor
        out = freqs.clone()
        for i in range(freqs.numel()):
            f = freqs[i]
            wavelength = 2 * math.pi / f
            if wavelength > long_edge:
                out[i] = f / self.factor
            elif wavelength >= short_edge:
                blend = (self.original_context / wavelength - self.low_freq_factor) / (
                    self.high_freq_factor - self.low_freq_factor
                )
                out[i] = (1 - blend) * f / self.factor + blend * f
        return out

    def arrange_rows(self, w: torch.Tensor, n_heads: int) -> torch.Tensor:
        """Rows of a q/k projection ``[n_heads*head_dim, in]`` from the
        checkpoint's half-split order to interleaved pairs: within the rotary
        part of a head, stored row ``j`` (first half) goes to ``2j`` and row
        ``j + rotary_dim/2`` to ``2j+1``; rows past the rotary part stay."""
        hd, rd = self.head_dim, self.rotary_dim
        if rd == 0:
            return w
        idx = torch.arange(hd)
        # new row r of a head takes old row src[r]
        src = idx.clone()
        src[0:rd:2] = idx[: rd // 2]
        src[1:rd:2] = idx[rd // 2 : rd]
        full = (torch.arange(n_heads)[:, None] * hd + src[None, :]).reshape(-1)
        return w.index_select(0, full.to(w.device))


class NoPosition(PositionEncoding):
    """Positions do not enter the mixer (nothing is rotated)."""


register_part("position", "rope", Rope)
register_part("position", "none", NoPosition)
