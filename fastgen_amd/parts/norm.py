"""RMSNorm on the residual stream (``fastgen/kernels/rmsnorm.py:33-60``)."""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from .base import VECTOR, Norm, TensorSpec, place, register_part


class RMSNorm(Norm):
    """``y = x * rsqrt(mean(x^2) + eps) * weight`` in fp32, one rounding."""

    def __init__(self, spec) -> None:
        super().__init__(spec)
        self.dim = int(spec.options["dim"])
        self.eps = float(spec.options["eps"])
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        return [TensorSpec(self._name("weight"), (self.dim,), VECTOR, ("one_plus_normal", 0.01))]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        self.weight = place(tensors[self._name("weight")], VECTOR, dtype, device)

    def fold_request(self, h: torch.Tensor):
        """(h, weight, eps): what a matrix product needs to fold the addition to the residual stream
        and this norm into its kernel (``fastgen_amd.kernels.linear.linear(residual=...)``)."""
        return (h, self.weight, self.eps)

    def forward(self, h, delta, dtype, rows=None):
        n = h.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, self.dim), dtype=dtype, device=h.device)
        return ops.add_rmsnorm(h, delta, self.weight, self.eps, out, rows)


register_part("norm", "rmsnorm", RMSNorm)
