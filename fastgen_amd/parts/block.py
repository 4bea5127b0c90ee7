"""Arrangements: how a layer's mixer, feed-forward and norms are wired to
the residual stream."""

from __future__ import annotations

from typing import Any, Optional

import torch

from ..kernels.ops import ScaledRows
from .base import FeedForward, LayerStore, Mixer, Norm, register_part


class PreNormBlock:
    """``h += mixer(norm(h)); h += ffn(norm(h))`` (``fastgen/forward.py:419-499``).

    The residual stream ``h`` is fp32.  Each addition is done by the norm
    that follows it, so a block takes the previous block's output as
    ``pending`` and returns its feed-forward's output un-added.

    For few rows the norms need no kernels of their own: a part that says so (``folds_norms``) is
    handed the norm that follows it (``then``) and may add its output to ``h`` and half-do that norm
    in its last product; it then returns ``ScaledRows`` instead of rows to be added, and the part
    after it finishes the norm in its first product.  ``next_norm`` is the norm that follows this
    block (the next block's first); a ``pending`` that is ``ScaledRows`` was made for this block's
    first norm.  Every step of this is optional: what a part does not fold, the norm's kernel does.
    """

    folds_norms = True

    def __init__(self, mixer: Mixer, ffn: FeedForward, mixer_norm: Norm, ffn_norm: Norm) -> None:
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    @staticmethod
    def _run(part, x, then, *args):
        """``part.forward`` with what it understands: ScaledRows and ``then`` only if it folds norms."""
        if getattr(part, "folds_norms", False):
            return part.forward(x, *args, then=then)
        return part.forward(x.materialize() if isinstance(x, ScaledRows) else x, *args)

    def forward(self, h: torch.Tensor, pending, ctx: Any, store: LayerStore, next_norm: Optional[Norm] = None):
        x = pending if isinstance(pending, ScaledRows) else self.mixer_norm.forward(h, pending, ctx.act_dtype)
        then = self.ffn_norm.fold_request(h) if hasattr(self.ffn_norm, "fold_request") else None
        mixed = self._run(self.mixer, x, then, ctx, store)
        x = mixed if isinstance(mixed, ScaledRows) else self.ffn_norm.forward(h, mixed, ctx.act_dtype)
        then = next_norm.fold_request(h) if next_norm is not None and hasattr(next_norm, "fold_request") else None
        return self._run(self.ffn, x, then)


register_part("arrangement", "pre_norm", lambda spec, *parts: PreNormBlock(*parts))
