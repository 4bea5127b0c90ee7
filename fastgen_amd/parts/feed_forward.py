"""Dense gated feed-forward (``fastgen/forward.py:483-499``):
``down(silu(gate(x)) * up(x))``.  Gate and up are one matrix with their rows
interleaved in groups of 8, so one product gives both and a tile of it holds
both halves of a channel: for few rows ``silu(gate) * up`` is applied where the
product is stored."""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, streamed
from .base import MATRIX, FeedForward, TensorSpec, place, register_part


class SwiGLU(FeedForward):
    folds_norms = True  # takes ScaledRows and the ``then`` request (see parts.block)

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.options["dim"])
        self.hidden_dim = int(spec.options["hidden_dim"])
        self.w_gate_up: Optional[StreamedMatrix] = None
        self.w_down: Optional[StreamedMatrix] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [
            TensorSpec(self._name("gate_proj.weight"), (self.hidden_dim, self.dim)),
            TensorSpec(self._name("up_proj.weight"), (self.hidden_dim, self.dim)),
            TensorSpec(self._name("down_proj.weight"), (self.dim, self.hidden_dim)),
        ]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        gate, up = tensors[self._name("gate_proj.weight")], tensors[self._name("up_proj.weight")]
        down = tensors[self._name("down_proj.weight")]
        pad = -self.hidden_dim % 8
        if pad:
            # the kernels work on groups of 8 channels: channels of zero weights are added, whose
            # activation silu(0) * 0 = 0 meets zero columns of the down projection
            gate = torch.cat([gate, gate.new_zeros(pad, self.dim)])
            up = torch.cat([up, up.new_zeros(pad, self.dim)])
            down = torch.cat([down, down.new_zeros(self.dim, pad)], dim=1)
        self.w_gate_up = streamed(place(ops.interleave_gate_up(gate, up), MATRIX, dtype, device))
        self.w_down = streamed(place(down, MATRIX, dtype, device))

    def forward(self, x, then=None):
        """``x``: the normed rows, or ``ScaledRows`` (the gate/up product finishes the norm).  ``then``:
        a norm's ``fold_request`` for the down projection (see ``Attention.forward``)."""
        act = linear(x, self.w_gate_up, epilogue="silu_mul")
        return linear(act, self.w_down, partials_ok=True, residual=then)


register_part("feed_forward", "swiglu", SwiGLU)
