"""``y = x W^T`` for the two precisions of the engine.

float32: the engine's own fused-multiply-add kernel (``gemm.hip``), a true
32-bit product whose rows do not depend on one another.  bfloat16: several
kernels can take a product (the engine's weight-streaming MFMA kernels of
``gemm_skinny.hip``, narrow and wide, with or without a cut of the k range, and
the vendor library's product through ``torch``, which the reference uses for
all of them: cuBLAS through ``F.linear``, ``fastgen/forward.py:433-513``).
Which one is the fastest depends on the matrix and on the number of rows, so
it is measured: the first time a product of some shape ``(N, K)`` meets some
number of rows, the kernels that can take it are timed on the operands at hand
(the caches emptied before each run) and the winner is kept in one table (``choices``) for every later product of
that shape and row bucket.  No size of any model stands here or in the parts.

A part hands ``linear`` its matrix as a :class:`StreamedMatrix` (made by :func:`streamed` when the part
loads): the matrix row by row and, where a model's weights fit the GPU twice over, a second copy in the order
in which the streaming kernels read it, which those kernels take.
"""

from __future__ import annotations

import os
from contextlib import contextmanager
from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Tuple

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


# what the kernels take (their limits, not a model's sizes)
SKINNY_ROWS = 16  # one 16-row block of x: the narrow kernel (16 output columns a workgroup) and every folded epilogue
WIDE_ROWS = ops.SKINNY_MAX_ROWS  # the wide kernel (64 columns a workgroup): up to eight blocks of x
# the tiled kernel takes any number of rows; it is offered where it has been seen to win or come close (from the
# wide kernel's range up to a few hundred rows; beyond, the library's large tiles are twice as fast)
TILED_MIN_ROWS, TILED_MAX_ROWS = 65, 512


# ------------------------------------------------------- a weight, stored for its readers
@dataclass
class StreamedMatrix:
    """A weight matrix ``[N, K]`` as its products read it: ``rows`` is the matrix row by row (what the
    library's and the tiled product take, and the 32-bit path); ``packed``, where there is memory for
    a second copy, the same matrix in the order in which the streaming kernels' waves read it
    (:class:`~fastgen_amd.kernels.ops.PackedWeight`): the products of up to 128 rows then ask the
    memory for whole cache lines and take 8 to 13 % less time."""

    rows: torch.Tensor
    packed: Optional[ops.PackedWeight] = None

    @property
    def shape(self):
        return self.rows.shape

    @property
    def dtype(self) -> torch.dtype:
        return self.rows.dtype

    @property
    def streaming(self):
        """What the streaming kernels are given: the packed copy if there is one."""
        return self.packed if self.packed is not None else self.rows

    def first_rows(self, n: int) -> "StreamedMatrix":
        """The matrix of the first ``n`` rows (views; the packed copy only if ``n`` is a multiple of 16)."""
        keep = self.packed is not None and (n % 16 == 0 or n == self.rows.shape[0])
        return StreamedMatrix(self.rows[:n], self.packed.first_rows(n) if keep else None)

    def nbytes(self) -> int:
        return self.rows.numel() * self.rows.element_size() + (
            self.packed.data.numel() * self.packed.data.element_size() if self.packed is not None else 0)


# whether `streamed` makes the second copy: set for the time a model loads (`packing`)
_pack_now = False


@contextmanager
def packing(on: bool):
    """While a model's parts load: whether their matrices get the second, packed copy."""
    global _pack_now
    before, _pack_now = _pack_now, bool(on)
    try:
        yield
    finally:
        _pack_now = before


def packing_fits(matrix_bytes: int, device, budget_bytes: Optional[int] = None) -> bool:
    """The rule for the second copy when nobody says otherwise (``FG_PACKED_WEIGHTS=0`` / ``1`` does): the
    weights twice take at most half of the memory that the model and its cache may use (``budget_bytes``;
    default: all of the GPU's), so that at least half stays for the cache."""
    forced = os.environ.get("FG_PACKED_WEIGHTS", "")
    if forced in ("0", "1"):
        return forced == "1"
    dev = torch.device(device)
    if dev.type != "cuda":
        return False
    if budget_bytes is None:
        budget_bytes = torch.cuda.get_device_properties(dev).total_memory
    return 2 * matrix_bytes <= budget_bytes // 2


def streamed(w: torch.Tensor) -> StreamedMatrix:
    """A part's weight matrix, placed on the device, as the products take it."""
    if _pack_now and w.is_cuda and w.dtype == torch.bfloat16 and w.dim() == 2:
        return StreamedMatrix(w, ops.pack_weight(w))
    return StreamedMatrix(w)


def _rows_of(w) -> torch.Tensor:
    return w.rows if isinstance(w, StreamedMatrix) else w


def _aligned(x: torch.Tensor, w) -> bool:
    w = _rows_of(w)
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.shape[1] % 8 == 0
            and x.stride(1) == 1 and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def skinny_ok(x: torch.Tensor, w) -> bool:
    """Few rows (decode): the engine's own weight-streaming kernels take the product, with the
    epilogues that are folded into them."""
    return x.shape[0] <= SKINNY_ROWS and _aligned(x, w)


def fold_ok(x: torch.Tensor, w) -> bool:
    """Few rows of bfloat16: the norms around a product can be folded into the products
    (:class:`~fastgen_amd.kernels.ops.ScaledRows`)."""
    return skinny_ok(x, w)


def k_splits_for(n_out: int, k: int, rows: int = 0) -> int:
    """Splits of the k range that give the wide kernel (64 output columns a workgroup) about two
    workgroups per compute unit, at most 8; with many rows a split keeps at least 1,024 of k (the
    partial sums it writes grow with the rows), else 512.  1: the output is wide enough by itself."""
    blocks = -(-n_out // 64)
    return max(1, min(8, 2 * ops.compute_units() // blocks, k // (1024 if rows > 48 else 512)))


# ------------------------------------------------------------------ the table
# (what is asked for, N, K, row bucket) -> name of the kernel that measured fastest
choices: Dict[Tuple[str, int, int, int], str] = {}
# the same keys -> what each candidate took when it was measured (milliseconds, the consumer's cost included)
timings: Dict[Tuple[str, int, int, int], Dict[str, float]] = {}
# set to a candidate's name to take that kernel wherever it is among the candidates (tests run the
# engine once under each name, so that every kernel that may be chosen is compared with the plain run)
force: Optional[str] = None
_TIMED_RUNS = 4
# Before each timed run this many bytes are read, so that a candidate finds the weights where a model's step
# finds them: in memory, not in the caches (a memory-side cache of 256 MB and the L2s; a decode step streams
# gigabytes of other weights between two uses of a matrix).  Timed warm, the wide kernel looks faster than the
# narrow one on matrices that fit the cache and is the slower one in the model.  (Read, not written: modified
# lines would be written back while the candidate runs, which costs the candidates unequally.)
_FLUSH_BYTES = 384 << 20


def row_bucket(rows: int) -> int:
    """Products of up to 16 rows are measured per number of rows, above that per block of 16 rows
    (the kernels work on such blocks) up to 256, per block of 64 up to the last size at which an own
    kernel is offered, and as one beyond."""
    if rows <= SKINNY_ROWS:
        return rows
    if rows <= 256:
        return -(-rows // 16) * 16
    return min(-(-rows // 64) * 64, TILED_MAX_ROWS + 64)


def tiled_splits(n_out: int, k: int, rows: int, tile_rows: int) -> int:
    """Splits of the k range that give the tiled kernel about two workgroups a compute unit, at most 16,
    each with at least 512 of k."""
    tiles = -(-rows // tile_rows) * -(-n_out // 128)
    return max(1, min(16, 2 * ops.compute_units() // tiles, k // 512))


def _capturing() -> bool:
    return torch.cuda.is_current_stream_capturing()


def _choose(what: str, n: int, k: int, rows: int, candidates: List[Tuple[str, Callable[[], torch.Tensor]]],
            handicap: Optional[Dict[str, float]] = None) -> str:
    """The candidate to run: the forced one, the one the table holds, or the one that is fastest now.
    Timing needs the device to itself (events and a wait for them), so a product that is first met while
    a step is being recorded runs the first candidate, unrecorded in the table; the engine runs every
    step once, unrecorded, before it records it.  The candidates are timed in turn on the same
    operands, each run behind a sweep of memory that empties the caches.  ``handicap``: milliseconds added to a candidate's time
    for what its result costs the consumer (partial sums that are still to be added)."""
    names = [c[0] for c in candidates]
    if force in names:
        return force
    if len(candidates) == 1:
        return names[0]
    key = (what, n, k, row_bucket(rows))
    got = choices.get(key)
    if got in names:
        return got
    if _capturing():
        return names[0]
    best: Dict[str, float] = {}
    for fn in (c[1] for c in candidates):  # once each, unmeasured: libraries load, the library picks its kernel
        fn()
    try:
        flush = torch.zeros(_FLUSH_BYTES // 4, dtype=torch.int32, device=torch.cuda.current_device())
        torch.cuda.current_stream().synchronize()  # (its zeros are in memory before anything is timed)
    except RuntimeError:  # no memory to spare: the candidates are timed on what the caches hold
        flush = None
    events = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
               for _ in range(_TIMED_RUNS)] for _ in candidates]
    for r in range(_TIMED_RUNS):
        for ev, (_, fn) in zip(events, candidates):
            if flush is not None:
                flush.amax()
            ev[r][0].record()
            fn()
            ev[r][1].record()
    torch.cuda.current_stream().synchronize()
    del flush
    for ev, name in zip(events, names):
        best[name] = min(a.elapsed_time(b) for a, b in ev) + (handicap or {}).get(name, 0.0)
    winner = min(names, key=lambda nm: best[nm])
    choices[key] = winner
    timings[key] = best
    return winner


def linear(x, w, out_dtype: Optional[torch.dtype] = None,
           partials_ok: bool = False, residual: Optional[Tuple[torch.Tensor, torch.Tensor, float]] = None,
           epilogue: Optional[str] = None):
    """``x @ w.T`` for ``w`` a matrix or a :class:`StreamedMatrix` (whose packed copy, if it has one, the
    streaming kernels read).  With ``partials_ok`` the result may come as fp32 ``[S, M, N]``
    partial sums whose sum over ``S`` is the product (the caller hands it to a
    norm, which adds them in order).

    ``epilogue="silu_mul"``: ``w`` is a gate and an up matrix interleaved by
    :func:`~fastgen_amd.kernels.ops.interleave_gate_up` and the result is
    ``silu(gate) * up`` ``[M, N/2]``, in the product's kernel where one that does so is the fastest.

    ``x`` may be :class:`~fastgen_amd.kernels.ops.ScaledRows`.  ``residual`` = (h, norm weight,
    eps) asks for more than the product: add it to the fp32 residual stream ``h`` and prepare the
    RMSNorm that follows.  Where that can be folded into the product's kernel (few rows, bfloat16)
    the result is ``ScaledRows`` and ``h`` is updated; where not, the plain product comes back and
    adding and norming are the caller's."""
    silu = epilogue == "silu_mul"
    if epilogue not in (None, "silu_mul"):
        raise ops.KernelArgumentError(f"linear: unknown epilogue {epilogue!r}")
    sw = w.streaming if isinstance(w, StreamedMatrix) else w  # what the streaming kernels read
    w = _rows_of(w)
    scaled = x if isinstance(x, ops.ScaledRows) else None
    if scaled is not None:
        if not fold_ok(scaled.rows, w) or out_dtype not in (None, torch.bfloat16):
            x, scaled = scaled.materialize(), None
        else:
            x = scaled.rows
    if not x.is_cuda:
        raise ops.KernelArgumentError("fastgen_amd runs on the GPU only; got a tensor on " + str(x.device))
    if x.dtype == torch.float32:
        if out_dtype not in (None, torch.float32):
            raise ops.KernelArgumentError("a float32 product has float32 output")
        y = ops.gemm_nt(x, w)
        return ops.silu_mul(y) if silu else y
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        raise ops.KernelArgumentError(f"linear: unsupported dtypes {x.dtype}, {w.dtype}")
    out_dtype = out_dtype or torch.bfloat16
    rows, (N, K) = x.shape[0], w.shape
    own = _aligned(x, w)
    src = scaled or x  # what the own kernels are given: they finish a norm that is still open

    if residual is not None and own and rows <= SKINNY_ROWS and out_dtype == torch.bfloat16 and not silu:
        h, norm_w, eps = residual
        if h.dtype == torch.float32 and h.is_contiguous() and h.shape == (rows, N):
            return ops.gemm_skinny_residual(src, sw, h, norm_w, eps)

    def library() -> torch.Tensor:
        xin = scaled.materialize() if scaled is not None else x
        if out_dtype == torch.bfloat16:
            y = torch.nn.functional.linear(xin, w)
        else:
            y = _library_mm_f32_out(xin, w)
            if y is None:
                y = ops.gemm_nt(xin, w, out_dtype=torch.float32)
        return ops.silu_mul(y) if silu else y

    candidates: List[Tuple[str, Callable[[], torch.Tensor]]] = []
    handicap: Dict[str, float] = {}
    tiled_ok = own and TILED_MIN_ROWS <= rows <= TILED_MAX_ROWS

    def sums_cost(splits: int) -> float:
        """Milliseconds the consumer takes to read the partial sums beyond the first (at 4 TB/s)."""
        return (splits - 1) * rows * N * 4 / 4e9

    if own and silu and out_dtype == torch.bfloat16 and N % 16 == 0:
        if rows <= SKINNY_ROWS:
            candidates.append(("narrow", lambda: ops.gemm_skinny(src, sw, silu_mul_epilogue=True, wide=False)))
        if rows <= WIDE_ROWS:
            candidates.append(("wide", lambda: ops.gemm_skinny(src, sw, silu_mul_epilogue=True, wide=True)))
        if tiled_ok:
            candidates.append(("tiled256", lambda: ops.gemm_tiled(x, sw, silu_mul_epilogue=True, tile_rows=256)))
    elif own and not silu:
        if rows <= SKINNY_ROWS:
            candidates.append(("narrow", lambda: ops.gemm_skinny(src, sw, out_dtype, wide=False)))
        elif rows <= WIDE_ROWS and partials_ok:
            splits = k_splits_for(N, K, rows)
            candidates.append(("wide", lambda: ops.gemm_skinny(x, sw, out_dtype, k_splits=splits, wide=True)))
            handicap["wide"] = sums_cost(splits)
        elif rows <= 64:
            candidates.append(("wide", lambda: ops.gemm_skinny(x, sw, out_dtype, wide=True)))
        if tiled_ok and partials_ok and out_dtype == torch.bfloat16:
            for name, tile_rows in zip(("tiled", "tiled256"), ops.TILED_TILE_ROWS):
                s_t = tiled_splits(N, K, rows, tile_rows)
                candidates.append((name, lambda tile_rows=tile_rows, s_t=s_t: ops.gemm_tiled(
                    x, sw, out_dtype, k_splits=s_t, tile_rows=tile_rows)))
                handicap[name] = sums_cost(s_t)
    if scaled is None or not candidates:
        candidates.append(("library", library))
    what = ("silu_mul" if silu else "store") + ("+partials" if partials_ok and rows > SKINNY_ROWS else "") + (
        "+f32" if out_dtype == torch.float32 else "") + ("+scaled" if scaled is not None else "") + (
        "+packed" if sw is not w else "")
    name = _choose(what, N, K, rows, candidates, handicap)
    return dict(candidates)[name]()
