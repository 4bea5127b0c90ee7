"""The two ends of the model: token embedding and the output head."""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, Part, TensorSpec, place, register_part


class Embedding(Part):
    """``h[t] = table[token[t]]`` into the fp32 residual stream, no scaling
    (``fastgen/forward.py:406-409``)."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.vocab_size = int(spec.options["vocab_size"])
        self.dim = int(spec.options["dim"])
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self._name("weight"), (self.vocab_size, self.dim))]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        self.weight = place(tensors[self._name("weight")], MATRIX, dtype, device)

    def forward(self, tokens: torch.Tensor, ctx: Any = None) -> torch.Tensor:
        """``ctx`` is the step's context: an embedding that adds something per position (learned or
        computed absolute positions) finds ``ctx.positions`` there; this one does not look at it."""
        h = torch.empty((tokens.numel(), self.dim), dtype=torch.float32, device=tokens.device)
        return ops.embed(self.weight, tokens, h)


class LMHead(Part):
    """fp32 logits ``x W^T``; ``W`` is the head's own matrix or, when tied,
    the embedding table (``fastgen/forward.py:507-515``)."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.vocab_size = int(spec.options["vocab_size"])
        self.dim = int(spec.options["dim"])
        self.tied_to: Optional[str] = spec.options.get("tied_to")
        self.weight: Optional[StreamedMatrix] = None

    def tensor_specs(self) -> List[TensorSpec]:
        if self.tied_to:
            return []
        return [TensorSpec(self._name("weight"), (self.vocab_size, self.dim))]

    def duplicates(self) -> Mapping[str, str]:
        """Tensors a checkpoint may carry although they repeat another one."""
        return {self._name("weight"): f"{self.tied_to}.weight"} if self.tied_to else {}

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        if not self.tied_to:
            self.weight = streamed(place(tensors[self._name("weight")], MATRIX, dtype, device))

    def tie(self, table: torch.Tensor) -> None:
        self.weight = streamed(table)  # the table itself row by row; a packed copy of it if copies are made

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear(x, self.weight, out_dtype=torch.float32)


register_part("embedding", "embedding", Embedding)
register_part("head", "lm_head", LMHead)
