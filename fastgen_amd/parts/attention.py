"""Grouped-query causal attention over the paged cache.

Per step (``fastgen/forward.py:421-472``): one product for q, k and v (the
three projections are stored as one matrix), rotation of q and k and the
write of k, v into the pages in one launch, attention of every new token
over all cached keys of its request, output projection.
"""

from __future__ import annotations

from typing import Any, List, Mapping, Optional

import torch

from ..kernels import ops
from ..kernels.linear import StreamedMatrix, linear, skinny_ok, streamed
from .base import LayerStore, Mixer, PagedNeed, TensorSpec, build_part, place, register_part, MATRIX


class Attention(Mixer):
    folds_norms = True  # takes ScaledRows and the ``then`` request (see parts.block)

    def __init__(self, spec) -> None:
        super().__init__(spec)
        o = spec.options
        self.dim = int(o["dim"])
        self.n_heads = int(o["n_heads"])
        self.n_kv_heads = int(o["n_kv_heads"])
        self.head_dim = int(o["head_dim"])
        self.scale = float(o.get("scale", self.head_dim**-0.5))
        self.window: Optional[int] = o.get("window") or None
        if self.n_heads % self.n_kv_heads:
            raise ValueError(f"n_heads={self.n_heads} is not a multiple of n_kv_heads={self.n_kv_heads}")
        if self.head_dim % 8 or self.head_dim > 512:
            raise ValueError(
                f"{self.prefix}: head size {self.head_dim} is not supported: the cache and the attention"
                " kernels work in chunks of 8 head dimensions, up to 512"
            )
        self.position = build_part("position", o["position"])
        self.wqkv: Optional[StreamedMatrix] = None
        self.wo: Optional[StreamedMatrix] = None
        self.freqs: Optional[torch.Tensor] = None

    def tensor_specs(self) -> List[TensorSpec]:
        q, kv = self.n_heads * self.head_dim, self.n_kv_heads * self.head_dim
        return [
            TensorSpec(self._name("q_proj.weight"), (q, self.dim)),
            TensorSpec(self._name("k_proj.weight"), (kv, self.dim)),
            TensorSpec(self._name("v_proj.weight"), (kv, self.dim)),
            TensorSpec(self._name("o_proj.weight"), (self.dim, q)),
        ]

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: Any) -> None:
        wq = self.position.arrange_rows(tensors[self._name("q_proj.weight")], self.n_heads)
        wk = self.position.arrange_rows(tensors[self._name("k_proj.weight")], self.n_kv_heads)
        wv = tensors[self._name("v_proj.weight")]
        self.wqkv = streamed(place(torch.cat([wq, wk, wv], dim=0), MATRIX, dtype, device))
        self.wo = streamed(place(tensors[self._name("o_proj.weight")], MATRIX, dtype, device))
        self.freqs = self.position.frequencies_on(device)

    def paged_need(self) -> PagedNeed:
        return PagedNeed(self.n_kv_heads, self.head_dim, self.window)

    def forward(self, x, ctx: Any, store: LayerStore, then=None):
        """``x``: the normed rows, or ``ScaledRows`` (a norm not yet finished, which the q/k/v product
        finishes).  ``then``: a norm's ``fold_request``; the output projection may fold the addition
        to the residual stream and that norm into its kernel and return ``ScaledRows``."""
        group = ctx.groups[store.group]
        q_width = self.n_heads * self.head_dim
        table = None
        if self.freqs is not None:
            # sin and cos of the step's positions: computed by the first layer, shared by all layers
            # that rotate with the same frequencies
            key = ("rope_table", self.freqs.data_ptr())
            table = ctx.scratch.get(key)
            if table is None:
                table = ctx.scratch[key] = ops.rope_table(ctx.positions, self.freqs)
        rows = x.rows if isinstance(x, ops.ScaledRows) else x
        if not (store.owns and self.head_dim % 16 == 0 and skinny_ok(rows, self.wqkv)) and rows is not x:
            x = x.materialize()
        if store.owns and self.head_dim % 16 == 0 and skinny_ok(rows, self.wqkv):
            # few rows (decode): rotation and cache write happen where the product is stored
            qkv = ops.gemm_skinny_qkv(x, self.wqkv.streaming, table, group.slots, store.k_pages, store.v_pages, self.n_heads,
                                      self.n_kv_heads, self.head_dim, self.position.rotary_dim)
        else:
            # an entry that reads another entry's cache needs its queries only
            qkv = linear(x, self.wqkv if store.owns else self.wqkv.first_rows(q_width))
            ops.rope_kv_write(
                qkv, ctx.positions, self.freqs, group.slots, store.k_pages, store.v_pages,
                self.n_heads, self.n_kv_heads, self.head_dim, self.position.rotary_dim, write_kv=store.owns,
                table=table,
            )
        out = torch.empty((rows.shape[0], q_width), dtype=rows.dtype, device=rows.device)
        ops.paged_attention(qkv, out, store.k_pages, store.v_pages, group, ctx, self.n_heads, self.scale,
                            self.window or 0)
        return linear(out, self.wo, partials_ok=True, residual=then)


register_part("mixer", "attention", Attention)
