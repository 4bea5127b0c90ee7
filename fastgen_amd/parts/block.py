"""Arrangements: how a layer's mixer, feed-forward and norms are wired to
the residual stream."""

from __future__ import annotations

from typing import Any, Optional, Tuple

import torch

from .base import FeedForward, LayerStore, Mixer, Norm, register_part


class PreNormBlock:
    """``h += mixer(norm(h)); h += ffn(norm(h))`` (``fastgen/forward.py:419-499``).

    The residual stream ``h`` is fp32.  Each addition is done by the norm
    that follows it, so a block takes the previous block's output as
    ``pending`` and returns its feed-forward's output un-added.
    """

    def __init__(self, mixer: Mixer, ffn: FeedForward, mixer_norm: Norm, ffn_norm: Norm) -> None:
        self.mixer, self.ffn, self.mixer_norm, self.ffn_norm = mixer, ffn, mixer_norm, ffn_norm

    def forward(self, h: torch.Tensor, pending: Optional[torch.Tensor], ctx: Any,
                store: LayerStore) -> torch.Tensor:
        x = self.mixer_norm.forward(h, pending, ctx.act_dtype)
        mixed = self.mixer.forward(x, ctx, store)
        x = self.ffn_norm.forward(h, mixed, ctx.act_dtype)
        return self.ffn.forward(x)


register_part("arrangement", "pre_norm", lambda spec, *parts: PreNormBlock(*parts))
