"""``y = x W^T`` for the two precisions of the engine.

float32: the engine's own fused-multiply-add kernel (``gemm.hip``), a true
32-bit product whose rows do not depend on one another.  bfloat16: up to 16
rows (decode) the engine's weight-streaming MFMA kernel (``gemm_skinny.hip``);
up to 64 rows (128 where the k range is cut) its wider sibling where that beats
the library; otherwise the vendor library's matrix product through ``torch`` (the
reference uses cuBLAS through ``F.linear`` for all of them,
``fastgen/forward.py:433-513``), with fp32 accumulation; logits are asked for in
fp32 directly.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import ops

_mm_out_dtype_ok: Optional[bool] = None


def _library_mm_f32_out(x: torch.Tensor, w: torch.Tensor) -> Optional[torch.Tensor]:
    """bf16 x bf16 -> fp32 through the library if this torch build offers it."""
    global _mm_out_dtype_ok
    if _mm_out_dtype_ok is False:
        return None
    try:
        y = torch.mm(x, w.t(), out_dtype=torch.float32)
        _mm_out_dtype_ok = True
        return y
    except (TypeError, RuntimeError):
        if _mm_out_dtype_ok is None:
            _mm_out_dtype_ok = False
            return None
        raise


# up to this many rows the weight-streaming kernels are used (more: the library's product)
SKINNY_ROWS = 16  # one 16-row block of x, 16 output columns a workgroup
FUSED_GATE_UP_ROWS = 80
LOGITS_SKINNY_ROWS = 8
TALL_ROWS = 128   # with k splits (few output columns, long k) the same kernel with up to eight blocks of x


def _aligned(x: torch.Tensor, w: torch.Tensor) -> bool:
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0
            and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Few rows (decode): the engine's own weight-streaming kernel takes the product."""
    return x.shape[0] <= SKINNY_ROWS and _aligned(x, w)


def fused_gate_up_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """The gate/up product with ``silu(gate) * up`` in its epilogue, where that beats the library's product plus
    an activation kernel: up to 80 rows (8B shape at 80 rows: 63 us against 64 + 8; at 96 rows 66 against 54 + 8).
    Above 16 rows only for k below 8,192: the wide kernel streams 4.4 to 4.7 TB/s whatever the size, the library
    reaches 5.4 on the 70B shape's 939 MB (17 / 64 rows: 174 / 184 us with the activation kernel against 199 / 209)
    and 3.7 on the 8B shape's 235 MB (65 / 65 us against 48 / 59; 3B shape 42 / 35 against 28 / 32)."""
    rows = x.shape[0]
    return (rows <= SKINNY_ROWS or (rows <= FUSED_GATE_UP_ROWS and w.shape[1] < 8192)) and _aligned(x, w)


def tall_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Up to 128 rows, for a product whose k range is cut (the o and down projections: the library runs them as
    32 tiles of 128 columns without a cut, 76 / 24 us at 128 rows of the 8B shape against 46 / 18).  Not for 8,192
    and more output columns with a k range no longer than that (the 70B shape's o projection: the library's 64
    tiles take 30 / 33 us at 17 / 64 rows against 35 / 39; its down projection, k = 28,672, stays here: 86 / 111
    against 91 / 141)."""
    N, K = w.shape
    return x.shape[0] <= TALL_ROWS and _aligned(x, w) and (N < 8192 or K > N)


_n_cus: Optional[int] = None


def _compute_units() -> int:
    global _n_cus
    if _n_cus is None:
        _n_cus = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _n_cus


def k_splits_for(n_out: int, k: int, rows: int = 0) -> int:
    """Splits of the k range that give the wide kernel (64 output columns a workgroup) about two
    workgroups per compute unit, at most 8; with many rows a split keeps at least 1,024 of k (the
    partial sums it writes grow with the rows), else 512.  1: the output is wide enough by itself."""
    blocks = -(-n_out // 64)
    return max(1, min(8, 2 * _compute_units() // blocks, k // (1024 if rows > 48 else 512)))


def fold_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Few rows of bfloat16: the norms around a product can be folded into the products
    (:class:`~fastgen_amd.kernels.ops.ScaledRows`)."""
    return skinny_ok(x, w)


def linear(x, w: torch.Tensor, out_dtype: Optional[torch.dtype] = None,
           partials_ok: bool = False, residual: Optional[Tuple[torch.Tensor, torch.Tensor, float]] = None):
    """``x @ w.T``.  With ``partials_ok`` the result may come as fp32 ``[S, M, N]``
    partial sums whose sum over ``S`` is the product (the caller hands it to a
    norm, which adds them in order).

    ``x`` may be :class:`~fastgen_amd.kernels.ops.ScaledRows`.  ``residual`` = (h, norm weight,
    eps) asks for more than the product: add it to the fp32 residual stream ``h`` and prepare the
    RMSNorm that follows.  Where that can be folded into the product's kernel (few rows, bfloat16)
    the result is ``ScaledRows`` and ``h`` is updated; where not, the plain product comes back and
    adding and norming are the caller's."""
    scaled = x if isinstance(x, ops.ScaledRows) else None
    if scaled is not None:
        if not fold_ok(scaled.rows, w):
            x, scaled = scaled.materialize(), None
        else:
            x = scaled.rows
    if residual is not None and x.is_cuda and fold_ok(x, w) and out_dtype in (None, torch.bfloat16):
        h, norm_w, eps = residual
        if h.dtype == torch.float32 and h.is_contiguous() and h.shape == (x.shape[0], w.shape[0]):
            return ops.gemm_skinny_residual(scaled or x, w, h, norm_w, eps)
    if scaled is not None:
        if out_dtype in (None, torch.bfloat16):
            return ops.gemm_skinny(scaled, w, torch.bfloat16, wide=False)
        x = scaled.materialize()
    if not x.is_cuda:
        raise ops.KernelArgumentError("fastgen_amd runs on the GPU only; got a tensor on " + str(x.device))
    out_dtype = out_dtype or x.dtype
    if x.dtype == torch.float32:
        if out_dtype != torch.float32:
            raise ops.KernelArgumentError("a float32 product has float32 output")
        return ops.gemm_nt(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ops.KernelArgumentError(f"linear: unsupported dtypes {x.dtype}, {w.dtype}")
    if partials_ok and x.shape[0] > 2 and tall_ok(x, w):
        splits = k_splits_for(w.shape[0], w.shape[1], x.shape[0])
        if splits > 3:  # (fewer: the output's own workgroups nearly fill the GPU, partial sums only cost)
            return ops.gemm_skinny(x, w, k_splits=splits, wide=True)
    # (the product for the logits, fp32 out over a whole vocabulary: from 9 rows on the library's is the faster one,
    # 8B shape at 12 / 16 rows 189 / 192 us against 204 / 220)
    if skinny_ok(x, w) and not (out_dtype == torch.float32 and x.shape[0] > LOGITS_SKINNY_ROWS):
        return ops.gemm_skinny(x, w, out_dtype, wide=False)
    if out_dtype == torch.bfloat16:
        return torch.nn.functional.linear(x, w)
    y = _library_mm_f32_out(x, w)
    return y if y is not None else ops.gemm_nt(x, w, out_dtype=torch.float32)
