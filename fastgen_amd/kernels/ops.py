"""Python faces of the HIP kernels.

Every function checks on the host that the operands have the shapes, dtypes
and strides the kernel and its grid assume, then launches on the current
stream of the tensors' device.  Nothing here runs on the CPU: a tensor that
is not on a GPU is refused.
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
import os
from typing import Dict, Optional, Tuple

import numpy as np

import torch

from . import _lib

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelArgumentError(ValueError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _DTYPE_CODE[t.dtype]
    except KeyError:
        raise KernelArgumentError(f"dtype {t.dtype} is not supported (float32 or bfloat16)") from None


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelArgumentError(msg)


def _gpu(*tensors: Optional[torch.Tensor]) -> None:
    dev = None
    for t in tensors:
        if t is None:
            continue
        _need(t.is_cuda, "fastgen_amd kernels run on the GPU only; got a tensor on " + str(t.device))
        dev = dev or t.device
        _need(t.device == dev, "operands live on different devices")


def _ptr(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)  # the stream's handle without a Stream object


def _stream(t: torch.Tensor) -> ctypes.c_void_p:
    """The device's current stream (a few hundred launches a step ask for it)."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def upload(values, dtype: torch.dtype, device: torch.device | str) -> torch.Tensor:
    """``values`` (a numpy array or nested lists) on the device, through pinned host memory and a
    copy that does not make the host wait for the work already queued on the stream: a step can be
    prepared while the step before it runs.  (The pinned block goes back to torch's host allocator,
    which hands it out again only after the copy has happened.)"""
    src = torch.from_numpy(values) if isinstance(values, np.ndarray) else torch.tensor(values, dtype=dtype)
    if src.dtype != dtype:
        src = src.to(dtype)
    staged = torch.empty(src.shape, dtype=dtype, pin_memory=True)
    staged.copy_(src)
    return staged.to(device, non_blocking=True)


def _check(status: int, what: str) -> None:
    if status == 1:
        raise KernelArgumentError(f"{what}: the kernel refuses these sizes or dtypes")
    if status != 0:
        raise RuntimeError(f"{what}: launch failed (status {status})")


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32")
    if n is not None:
        _need(t.numel() >= n, f"{name} holds {t.numel()} entries, {n} are needed")


# --------------------------------------------------------------------- rows
def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = table[tokens[t]] as fp32 (``fastgen/forward.py:406-409``)."""
    _gpu(table, tokens, out)
    n = tokens.numel()
    _need(table.dim() == 2 and table.is_contiguous(), "table must be contiguous [vocab, dim]")
    _i32(tokens, "tokens")
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (n, table.shape[1]),
          "out must be contiguous float32 [n_tokens, dim]")
    st = _lib.load("rows").fg_embed(
        _ptr(table), _code(table), _ptr(tokens), _ptr(out), n, table.shape[1], table.shape[0], _stream(out))
    _check(st, "embed")
    return out


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += delta`` (fp32 residual stream), ``out = rmsnorm(h) * weight``.

    ``delta`` is ``[T, dim]`` of ``out``'s dtype, or fp32 ``[S, T, dim]``: partial
    sums of a matrix product whose k range was cut, added in order.  With
    ``rows`` only those rows of ``h`` are normed, into consecutive rows of
    ``out``, and ``h`` is left unchanged.  Norm as in
    ``fastgen/kernels/rmsnorm.py:33-60``.
    """
    _gpu(h, delta, weight, out, rows)
    _need(h.dtype == torch.float32 and h.dim() == 2 and h.is_contiguous(), "h must be contiguous float32 [T, dim]")
    T, dim = h.shape
    n_rows = T if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, "rows")
    _need(weight.shape == (dim,) and weight.is_contiguous(), "weight must be [dim]")
    _need(out.is_contiguous() and out.shape == (n_rows, dim), "out must be contiguous [rows, dim]")
    parts, n_parts, part_stride = None, 0, 0
    if delta is not None and delta.dim() == 3:
        _need(delta.dtype == torch.float32 and delta.shape[1:] == h.shape and delta.stride(2) == 1
              and delta.stride(1) == dim, "partial sums must be float32 [S, T, dim] with contiguous rows")
        parts, n_parts, part_stride, delta = delta, delta.shape[0], delta.stride(0), None
    elif delta is not None:
        _need(delta.shape == h.shape and delta.is_contiguous() and delta.dtype == out.dtype,
              "delta must be contiguous, shaped like h, of out's dtype")
    st = _lib.load("rows").fg_add_rmsnorm(
        _ptr(h), _ptr(delta), _ptr(parts), n_parts, ctypes.c_longlong(part_stride), _ptr(weight), _ptr(out),
        _ptr(rows), n_rows, dim, ctypes.c_float(eps), _code(out), _code(weight), _stream(out))
    _check(st, "add_rmsnorm")
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMSNorm over the last dimension of a contiguous tensor."""
    _gpu(x, weight, out)
    _need(x.is_contiguous(), "x must be contiguous")
    dim = x.shape[-1]
    out = torch.empty_like(x) if out is None else out
    _need(out.shape == x.shape and out.dtype == x.dtype and out.is_contiguous(), "out must match x")
    _need(weight.shape == (dim,) and weight.is_contiguous(), "weight must be [dim]")
    st = _lib.load("rows").fg_rmsnorm(
        _ptr(x), _ptr(weight), _ptr(out), x.numel() // dim, dim, ctypes.c_float(eps), _code(x),
        _code(weight), _stream(out))
    _check(st, "rmsnorm")
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of a gate and an up matrix ``[hidden, dim]`` as one matrix
    ``[2*hidden, dim]`` in groups of 8: rows ``16k..16k+7`` are gate rows
    ``8k..8k+7``, rows ``16k+8..16k+15`` the up rows of the same channels.  One
    16-row tile of a product with it holds both halves of 8 channels, so
    ``silu(gate) * up`` can be applied where the tile is stored."""
    hidden, dim = gate.shape
    _need(up.shape == gate.shape and hidden % 8 == 0,
          f"gate and up must have the same shape and a row count that is a multiple of 8 (got {hidden})")
    return torch.stack([gate.reshape(hidden // 8, 8, dim), up.reshape(hidden // 8, 8, dim)], dim=1).reshape(
        2 * hidden, dim)


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of ``[T, 2*hidden]`` whose columns are interleaved as
    :func:`interleave_gate_up` orders the matrix rows; fp32 inside."""
    _gpu(gate_up, out)
    _need(gate_up.dim() == 2 and gate_up.is_contiguous() and gate_up.shape[1] % 16 == 0,
          "gate_up must be contiguous [T, 2*hidden] with hidden a multiple of 8")
    T, hidden = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((T, hidden), dtype=gate_up.dtype, device=gate_up.device) if out is None else out
    _need(out.shape == (T, hidden) and out.dtype == gate_up.dtype and out.is_contiguous(), "out must be [T, hidden]")
    st = _lib.load("rows").fg_silu_mul(_ptr(gate_up), _ptr(out), T, hidden, _code(out), _stream(out))
    _check(st, "silu_mul")
    return out


# ------------------------------------------------------------ rope + kv write
def rope_table(positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """``[T, n_freqs, 2]`` fp32: cos and sin of ``float(pos) * freqs[i]``, for all
    layers of a step that rotate with the same frequencies."""
    _gpu(positions, freqs)
    _i32(positions, "positions")
    _need(freqs.dtype == torch.float32 and freqs.is_contiguous(), "freqs must be contiguous float32")
    T, n = positions.numel(), freqs.numel()
    table = torch.empty((T, n, 2), dtype=torch.float32, device=positions.device)
    st = _lib.load("rope_kv").fg_rope_table(_ptr(positions), _ptr(freqs), _ptr(table), T, n, _stream(table))
    _check(st, "rope_table")
    return table


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, freqs: Optional[torch.Tensor],
                  slots: Optional[torch.Tensor], k_pages: Optional[torch.Tensor],
                  v_pages: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
                  rotary_dim: int, write_kv: bool = True, table: Optional[torch.Tensor] = None) -> None:
    """Rotate q and k of ``qkv [T, (H+2KV)*hd]`` in place and store k, v at
    ``slots`` of the paged cache (K pages ``[n_pages, KV, P, hd]``, V pages
    ``[n_pages, KV, hd, P]``).  ``kernels/rope.py:56-89``, ``forward.py:449-460``.
    """
    _gpu(qkv, positions, freqs, slots, k_pages, v_pages)
    _need(qkv.dim() == 2 and qkv.stride(1) == 1, "qkv must be [T, width] with unit column stride")
    T = qkv.shape[0]
    width = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    _need(qkv.shape[1] >= width, f"qkv rows hold {qkv.shape[1]} elements, {width} are needed")
    _i32(positions, "positions", T)
    _need(head_dim % 2 == 0 and 0 <= rotary_dim <= head_dim and rotary_dim % 2 == 0,
          "head_dim and rotary_dim must be even and rotary_dim <= head_dim")
    if rotary_dim and table is None:
        _need(freqs is not None and freqs.dtype == torch.float32 and freqs.is_contiguous()
              and freqs.numel() >= rotary_dim // 2, "freqs must be float32 [rotary_dim/2]")
    if rotary_dim and table is not None:
        _need(table.dtype == torch.float32 and table.is_contiguous() and table.shape == (T, rotary_dim // 2, 2),
              "table must be float32 [T, rotary_dim/2, 2]")
    page_size = 1
    if write_kv:
        _need(slots is not None and k_pages is not None and v_pages is not None, "cache operands missing")
        _i32(slots, "slots", T)
        _need(k_pages.dim() == 4 and k_pages.is_contiguous() and k_pages.dtype == qkv.dtype
              and k_pages.shape[1] == n_kv and k_pages.shape[3] == head_dim,
              "k_pages must be contiguous [n_pages, KV, P, hd] of qkv's dtype")
        page_size = k_pages.shape[2]
        _need(v_pages.is_contiguous() and v_pages.dtype == qkv.dtype
              and v_pages.shape == (k_pages.shape[0], n_kv, head_dim, page_size),
              "v_pages must be contiguous [n_pages, KV, hd, P] of qkv's dtype")
    st = _lib.load("rope_kv").fg_rope_kv_write(
        _ptr(qkv), qkv.stride(0), _ptr(positions), _ptr(freqs), _ptr(table if rotary_dim else None), _ptr(slots),
        _ptr(k_pages), _ptr(v_pages),
        T, n_heads, n_kv, head_dim, rotary_dim, page_size, int(write_kv), _code(qkv), _stream(qkv))
    _check(st, "rope_kv_write")


# ------------------------------------------------------------------ attention
def paged_attention_general(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                            block_table: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                            n_heads: int, scale: float, window: int = 0) -> torch.Tensor:
    """Causal attention of every token over its sequence's cached keys.

    ``q`` is ``[T, >= H*hd]`` (the first ``H*hd`` columns are the query heads;
    it may be a qkv buffer), ``out`` is ``[T, H*hd]``.  ``forward.py:176-258``.
    """
    _gpu(q, out, k_pages, v_pages, block_table, seq_of_token, positions)
    T = q.shape[0]
    _need(k_pages.dim() == 4 and k_pages.is_contiguous(), "k_pages must be contiguous [n_pages, KV, P, hd]")
    n_pages, n_kv, page_size, hd = k_pages.shape
    _need(v_pages.shape == (n_pages, n_kv, hd, page_size) and v_pages.is_contiguous(),
          "v_pages must be contiguous [n_pages, KV, hd, P]")
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * hd, "q must be [T, >= H*hd]")
    _need(out.dim() == 2 and out.stride(1) == 1 and out.shape == (T, n_heads * hd), "out must be [T, H*hd]")
    _need(q.dtype == out.dtype == k_pages.dtype == v_pages.dtype, "q, out and the cache must share a dtype")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1,
          "block_table must be int32 [B, max_pages]")
    _i32(seq_of_token, "seq_of_token", T)
    _i32(positions, "positions", T)
    _need(n_heads % n_kv == 0, "the number of heads must be a multiple of the number of kv heads")
    _need(hd % 8 == 0 and hd <= 512, f"head size {hd} is not supported (multiple of 8, at most 512)")
    _need(page_size % 8 == 0, f"page size {page_size} is not supported (multiple of 8)")
    st = _lib.load("attention").fg_paged_attention_general(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
        block_table.stride(0), _ptr(seq_of_token), _ptr(positions), T, n_heads, n_kv, hd, page_size,
        ctypes.c_float(scale), int(window or 0), _code(q), _stream(q))
    _check(st, "paged_attention_general")
    return out


MFMA_MAX_HEAD_DIM = 256

_n_cus: Optional[int] = None


def compute_units() -> int:
    """Compute units of the current device (asked once)."""
    global _n_cus
    if _n_cus is None:
        _n_cus = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _n_cus


def _split_target_blocks() -> int:
    """Workgroups wanted for the decode attention kernel: one per compute unit measured best (half as many
    to eight times as many tried at batch 1, 8 and 64).  The splits' partial results are merged by a second
    kernel: merging them in the split that finishes last needs device-scope fences, which on a GPU of
    several dies cost more than the launch they save (measured)."""
    env = os.environ.get("FG_SPLIT_TARGET")
    return int(env) if env else compute_units()


# a chunk of the decode attention's key ranges is a multiple of this many 64-key tiles (one a wave)
_SPLIT_MIN_TILES = int(os.environ.get("FG_SPLIT_MIN_TILES", 4))


def attention_tile_rows(head_dim: int, small: bool = False) -> int:
    """Query rows of one item of the tile kernel for this head size: of its larger form (128 rows up to
    head size 128), or of the form with ``small`` items (64 rows, more and lighter workgroups)."""
    return int(_lib.load(f"attention_mfma@{head_dim}").fg_attn_tile_rows(int(small)))


def attention_items(q_lens, q_start, n_cached, group_size: int, tile_rows: int = 64):
    """Cut the step's sequences into items for the MFMA kernels.

    Returns two int32 arrays ``[n, 4]`` of (sequence, first flat token, tokens,
    position of the first token): items of at most 16 rows for the split
    kernel (decoded tokens and very short portions) and items of at most
    ``tile_rows`` rows for the tile kernel, those with the most keys first (the
    kernel's workgroups start in that order, so short items fill in behind long
    ones).
    """
    small, big = [], []
    per_tile = max(1, tile_rows // group_size)
    for b, n in enumerate(q_lens):
        n, s, c = int(n), int(q_start[b]), int(n_cached[b])
        if n * group_size <= 16:
            small.append((b, s, n, c))
        else:
            big.extend((b, s + i, min(per_tile, n - i), c + i) for i in range(0, n, per_tile))
    big.sort(key=lambda it: -(it[3] + it[2]))  # the longest key ranges start first
    as_arr = lambda x: np.asarray(x, dtype=np.int32).reshape(-1, 4)
    return as_arr(small), as_arr(big)


def attention_chunks_for(n_items: int, n_kv: int) -> int:
    """Length of the split kernel's chunk list for ``n_items`` items: enough chunks for a few
    workgroups per compute unit, and at least two an item so that a long sequence among short
    ones can be cut."""
    return max(-(-_split_target_blocks() // n_kv) + n_items, 2 * n_items)


def _plan_ints(lib, max_chunks: int) -> int:
    lib.fg_attn_plan_ints.restype = ctypes.c_longlong
    return int(lib.fg_attn_plan_ints(max_chunks))


def attention_plan(items: torch.Tensor, n_items: int, max_chunks: int, head_dim: int, window: int = 0,
                   min_tiles: int = 4) -> torch.Tensor:
    """Cuts the key ranges of ``items`` (device int32 ``[n_items, 4]``, 16-byte aligned) into chunks of
    the same number of 64-key tiles, a multiple of ``min_tiles``, on the device: a captured step cuts
    anew for the lengths of every replay.  The int32 plan that :func:`paged_attention_mfma` takes."""
    _gpu(items)
    _i32(items, "items")
    _need(items.data_ptr() % 16 == 0 and items.numel() >= 4 * n_items > 0, "items must be [n, 4], 16-byte aligned")
    _need(max_chunks >= 2 * n_items and min_tiles >= 1, "max_chunks must be at least twice the number of items")
    lib = _lib.load(f"attention_mfma@{head_dim}")  # the plan is the same for every head size
    plan = torch.empty(_plan_ints(lib, max_chunks), dtype=torch.int32, device=items.device)
    _check(lib.fg_attn_plan(_ptr(items), n_items, int(window or 0), max_chunks, min_tiles, _ptr(plan),
                            _stream(items)), "attn_plan")
    return plan


_ONE_STREAM = bool(os.environ.get("FG_ONE_STREAM"))  # no kernel runs beside another
_second: Dict[int, "torch.cuda.Stream"] = {}


def _second_stream(device) -> "torch.cuda.Stream":
    """A stream of the default priority beside the current one, one a device, made at first use."""
    index = torch.device(device).index
    index = torch.cuda.current_device() if index is None else index
    if index not in _second:
        _second[index] = torch.cuda.Stream(device)
    return _second[index]


def paged_attention_mfma(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                         block_table: torch.Tensor, small_items: Optional[torch.Tensor],
                         big_items: Optional[torch.Tensor], n_heads: int, scale: float, window: int = 0,
                         plan: Optional[torch.Tensor] = None, max_chunks: Optional[int] = None,
                         min_tiles: int = 4, max_rows: int = 16, tile_rows: Optional[int] = None) -> torch.Tensor:
    """bf16 attention on the matrix cores.  ``small_items`` / ``big_items`` are
    device int32 ``[n, 4]`` lists from :func:`attention_items` (16-byte aligned);
    every query token of the step must be covered by exactly one item.
    ``plan``: :func:`attention_plan` of the small items with this ``max_chunks``
    and ``window`` (made here if not given).  ``max_rows``: no small item has
    more rows (tokens times query heads per kv head) than this.  ``tile_rows``: the
    rows the big items were cut for (:func:`attention_tile_rows`; default: the larger form's).
    With items of both kinds the tile kernel runs on a second stream beside the split kernel and
    the current stream waits for it before this returns (not while a graph is captured, not with
    ``FG_ONE_STREAM=1``)."""
    _gpu(q, out, k_pages, v_pages, block_table, small_items, big_items, plan)
    n_pages, n_kv, page_size, hd = k_pages.shape
    _need(q.dtype == torch.bfloat16 and out.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16
          and v_pages.dtype == torch.bfloat16, "the MFMA attention kernels take bfloat16")
    _need(hd % 16 == 0 and hd <= MFMA_MAX_HEAD_DIM, f"head size {hd}: multiples of 16 up to {MFMA_MAX_HEAD_DIM}")
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and v_pages.shape == (n_pages, n_kv, hd, page_size),
          "k_pages [n_pages, KV, P, hd] and v_pages [n_pages, KV, hd, P] must be contiguous")
    _need(n_heads % n_kv == 0 and page_size % 8 == 0, "heads must be a multiple of kv heads, pages of 8 tokens")
    _need(scale > 0, "the score scale must be positive")
    T = q.shape[0]
    _need(q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= n_heads * hd and q.stride(0) % 8 == 0
          and q.data_ptr() % 16 == 0, "q must be [T, >= H*hd], rows 16-byte aligned")
    _need(out.shape == (T, n_heads * hd) and out.stride(1) == 1 and out.stride(0) % 4 == 0, "out must be [T, H*hd]")
    _need(block_table.dim() == 2 and block_table.dtype == torch.int32 and block_table.stride(1) == 1,
          "block_table must be int32 [B, max_pages]")
    lib = _lib.load(f"attention_mfma@{hd}")
    G = n_heads // n_kv
    beside = None
    if (small_items is not None and small_items.numel() and big_items is not None and big_items.numel()
            and not _ONE_STREAM and not torch.cuda.is_current_stream_capturing()):
        # a step with both kinds of items (prompt portions beside decoded tokens): the two kernels write
        # different rows of `out`, one is bound by the matrix cores and one by memory, so the tile kernel
        # runs on a second stream beside the split kernel (3 % of a continuous-batching run)
        beside = _second_stream(q.device)
        beside.wait_event(torch.cuda.current_stream(q.device).record_event())
    if small_items is not None and small_items.numel():
        _need(G <= 16 and 1 <= max_rows <= 16, "the split kernel takes at most 16 rows an item")
        _i32(small_items, "small_items")
        _need(small_items.data_ptr() % 16 == 0, "items must be 16-byte aligned")
        n = small_items.numel() // 4
        if max_chunks is None:
            max_chunks = attention_chunks_for(n, n_kv)
        _need(2 * n <= max_chunks <= 65535, "the chunk list holds at least two chunks an item and at most 65535")
        if plan is None:
            plan = attention_plan(small_items, n, max_chunks, hd, window, min_tiles)
        _need(plan.dtype == torch.int32 and plan.numel() == _plan_ints(lib, max_chunks),
              "the plan does not fit the items and max_chunks")
        part_o = torch.empty((max_chunks * n_kv * 16, hd), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((max_chunks * n_kv * 16, 2), dtype=torch.float32, device=q.device)
        st = lib.fg_attn_split(
            _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            block_table.stride(0), _ptr(plan), n, max_chunks, max_rows, _ptr(part_o), _ptr(part_ml), n_heads, n_kv, hd,
            page_size, ctypes.c_float(scale), int(window or 0), _stream(q))
        _check(st, "attn_split")
    if big_items is not None and big_items.numel():
        tile_rows = attention_tile_rows(hd) if tile_rows is None else int(tile_rows)
        _need(tile_rows in (attention_tile_rows(hd), attention_tile_rows(hd, True)), "tile_rows is no form of the tile kernel")
        _need(G <= tile_rows, "too many query heads per kv head for the tile kernel")
        _i32(big_items, "big_items")
        _need(big_items.data_ptr() % 16 == 0, "items must be 16-byte aligned")
        st = lib.fg_attn_tile(
            _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
            block_table.stride(0), _ptr(big_items), big_items.numel() // 4, tile_rows, n_heads, n_kv, hd, page_size,
            ctypes.c_float(scale), int(window or 0), ctypes.c_void_p(beside.cuda_stream) if beside else _stream(q))
        _check(st, "attn_tile")
        if beside is not None:
            torch.cuda.current_stream(q.device).wait_event(beside.record_event())
    return out


def paged_attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                    group, ctx, n_heads: int, scale: float, window: int = 0) -> torch.Tensor:
    """Attention for one step: picks the kernel for the step's dtype and shape.

    ``group`` carries the block table of the layer's cache group, ``ctx`` the
    step's per-token vectors (``fastgen_amd.engine.context``).  bfloat16 with a
    head size in steps of 16 up to 256 and at most 16 query heads per kv head
    runs on the matrix cores; everything else (float32 always) runs the general
    kernel.
    """
    n_kv, hd = k_pages.shape[1], k_pages.shape[3]
    G = n_heads // n_kv
    if q.dtype != torch.bfloat16 or hd % 16 or hd > MFMA_MAX_HEAD_DIM or G > 16:
        return paged_attention_general(q, out, k_pages, v_pages, group.block_table, ctx.seq_of_token,
                                       ctx.positions, n_heads, scale, window)
    items_key = ("attention_items", G, hd, n_kv)  # (how a step is cut into items depends on all three)
    plan = ctx.scratch.get(items_key)
    if plan is None:
        if ctx.seq_records is not None and int(ctx.q_lens.max()) * G <= 16:
            # every sequence is one item of the split kernel: its records are in the step's buffer
            # already (and are refreshed with it when the step is a replayed graph)
            plan = (ctx.seq_records, None, ctx.n_seqs, None)
        else:
            tile_rows = attention_tile_rows(hd)
            small, big = attention_items(ctx.q_lens, ctx.q_start_host, ctx.n_cached, G, tile_rows)
            if 0 < len(big) * n_kv <= compute_units() // 2 and attention_tile_rows(hd, True) < tile_rows:
                # so few items that half the compute units would stand idle: items of half the rows, whose
                # lighter workgroups share a unit (prompt portions of up to 512 tokens: 11.6 / 17.6 us
                # against 14.1 / 19.5 at 256 / 512 tokens; equal at 1,024, slower beyond)
                tile_rows = attention_tile_rows(hd, True)
                small, big = attention_items(ctx.q_lens, ctx.q_start_host, ctx.n_cached, G, tile_rows)
            both = upload(np.concatenate([small, big]).reshape(-1), torch.int32, q.device)
            plan = (both[: small.size] if small.size else None, both[small.size:] if big.size else None, len(small),
                    tile_rows)
        ctx.scratch[items_key] = plan
    small_d, big_d, n_small, tile_rows = plan
    chunks = split_plan = None
    if n_small:
        # how the items' key ranges are cut depends on the window: layers with the same one share the cut
        chunks = attention_chunks_for(n_small, n_kv)
        key = ("attention_plan", G, int(window or 0), chunks)
        split_plan = ctx.scratch.get(key)
        if split_plan is None:
            split_plan = ctx.scratch[key] = attention_plan(small_d, n_small, chunks, hd, window, _SPLIT_MIN_TILES)
    # rows of the largest small item: one token a sequence in a decode step (also a captured one)
    rows = G * int(ctx.q_lens.max()) if big_d is None else 16
    return paged_attention_mfma(q, out, k_pages, v_pages, group.block_table, small_d, big_d, n_heads, scale,
                                window, split_plan, chunks, max_rows=min(16, rows), tile_rows=tile_rows)


# ----------------------------------------------------------------------- gemm
def gemm_nt(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
            out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ w.T`` with ``w [N, K]``, by the engine's own fp32-FMA kernel (sum
    over k in ascending order; a row's result does not depend on the others)."""
    _gpu(x, w, out)
    _need(x.dim() == 2 and w.dim() == 2 and x.shape[1] == w.shape[1], "x [M,K] and w [N,K] must share K")
    _need(x.stride(1) == 1 and w.stride(1) == 1, "x and w need unit column stride")
    _need(x.dtype == w.dtype, "x and w must share a dtype")
    M, K = x.shape
    N = w.shape[0]
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "out must be [M, N]")
    for m0 in range(0, M, 65535 * 64):  # grid.y limit
        m1 = min(M, m0 + 65535 * 64)
        st = _lib.load("gemm").fg_gemm_nt(
            _ptr(x[m0:m1]), _ptr(w), _ptr(out[m0:m1]), m1 - m0, N, K, x.stride(0), w.stride(0), out.stride(0),
            _code(x), _code(out), _stream(out))
        _check(st, "gemm_nt")
    return out


SKINNY_MAX_ROWS = 128


@dataclass
class PackedWeight:
    """A bfloat16 weight matrix ``[n, k]`` in the order in which the streaming products read it
    (:func:`pack_weight`): ``data [ceil(n / 16), ceil(k / 32), 64, 8]``, a block of 16 rows x 32 k as
    the 1 KB that a wave holds as one MFMA operand (lane ``16 g + r``: row ``r``, k ``8 g .. 8 g + 7``),
    rows and k padded with zeros.  A wave's load is then whole cache lines in a row; from a matrix
    stored row by row it is 16 pieces of half a line."""

    data: torch.Tensor
    n: int
    k: int

    @property
    def shape(self) -> Tuple[int, int]:
        return (self.n, self.k)

    @property
    def dtype(self) -> torch.dtype:
        return self.data.dtype

    def first_rows(self, n: int) -> "PackedWeight":
        """The matrix of the first ``n`` rows (a multiple of 16, or all): a view."""
        _need(0 < n <= self.n and (n % 16 == 0 or n == self.n), "a packed matrix is cut at multiples of 16 rows")
        return PackedWeight(self.data[: -(-n // 16)], n, self.k)


def pack_weight(w: torch.Tensor) -> PackedWeight:
    """``w [n, k]`` (bfloat16) as :class:`PackedWeight`: a copy, on the device of ``w``."""
    _need(w.dim() == 2 and w.dtype == torch.bfloat16, "pack_weight takes a bfloat16 matrix")
    n, k = w.shape
    nb, ks = -(-n // 16), -(-k // 32)
    if (nb * 16, ks * 32) != (n, k):
        padded = w.new_zeros((nb * 16, ks * 32))
        padded[:n, :k] = w
        w = padded
    # [nb, r, ks, g, 8] -> [nb, ks, g, r, 8]
    data = w.view(nb, 16, ks, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(nb, ks, 64, 8)
    return PackedWeight(data, n, k)


def unpack_weight(p: PackedWeight) -> torch.Tensor:
    """The matrix ``[n, k]`` that :func:`pack_weight` was given."""
    nb, ks = p.data.shape[:2]
    w = p.data.view(nb, ks, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(nb * 16, ks * 32)
    return w[: p.n, : p.k].contiguous()


def _weight_args(w, K: int, what: str):
    """C arguments (pointer, ldw) for the weight of a streaming product, a matrix or :class:`PackedWeight`
    (ldw = 0), checked against the k of x."""
    if isinstance(w, PackedWeight):
        _gpu(w.data)
        _need(w.data.dtype == torch.bfloat16 and w.data.is_contiguous() and w.k == K
              and w.data.shape == (-(-w.n // 16), -(-w.k // 32), 64, 8) and w.data.data_ptr() % 16 == 0,
              f"{what}: the packed weight does not fit x [M, {K}]")
        return _ptr(w.data), 0
    _gpu(w)
    _need(w.dim() == 2 and w.dtype == torch.bfloat16 and w.shape[1] == K, f"{what}: w must be bfloat16 [N, {K}]")
    _need(w.stride(1) == 1 and w.stride(0) % 8 == 0 and w.data_ptr() % 16 == 0, f"{what}: w needs 16-byte aligned rows")
    return _ptr(w), w.stride(0)


@dataclass
class ScaledRows:
    """Rows that are not yet divided by their root mean square: the true row ``t`` is
    ``rows[t] * rsqrt(sum(ssq[t]) / dim + eps)``.  For few rows the norm before a matrix product
    is folded into the products around it: the one before stores ``rows`` and the sums of squares
    of its workgroups' columns (:func:`gemm_skinny_residual`), the one after scales its result
    rows (``x @ w.T`` is linear in a row's scale)."""

    rows: torch.Tensor  # [T, dim] bfloat16
    ssq: torch.Tensor  # [T, n_parts] float32
    dim: int
    eps: float

    @property
    def shape(self):
        return self.rows.shape

    def materialize(self) -> torch.Tensor:
        """The rows themselves (a kernel of its own: for a consumer that does not take the pair)."""
        return scale_rows(self.rows, self.ssq, self.dim, self.eps)


def _row_scale_args(x, M: int):
    """C arguments (ssq, n_parts, dim, eps) for ``x`` a tensor or :class:`ScaledRows`."""
    if not isinstance(x, ScaledRows):
        return ctypes.c_void_p(0), 0, 0, ctypes.c_float(0.0)
    ssq = x.ssq
    _need(ssq.dtype == torch.float32 and ssq.is_contiguous() and ssq.dim() == 2 and ssq.shape[0] == M
          and ssq.is_cuda, "ssq must be contiguous float32 [M, n_parts] on the GPU")
    _need(x.dim > 0 and x.eps >= 0, "ScaledRows needs dim > 0 and eps >= 0")
    return _ptr(ssq), ssq.shape[1], int(x.dim), ctypes.c_float(x.eps)


def scale_rows(rows: torch.Tensor, ssq: torch.Tensor, dim: int, eps: float) -> torch.Tensor:
    """``rows[t] * rsqrt(sum(ssq[t]) / dim + eps)`` in the dtype of ``rows``."""
    _gpu(rows, ssq)
    _need(rows.dim() == 2 and rows.is_contiguous() and ssq.dim() == 2 and ssq.is_contiguous()
          and ssq.dtype == torch.float32 and ssq.shape[0] == rows.shape[0], "rows [T, D], ssq float32 [T, n_parts]")
    out = torch.empty_like(rows)
    st = _lib.load("rows").fg_scale_rows(_ptr(rows), _ptr(ssq), _ptr(out), rows.shape[0], rows.shape[1],
                                         ssq.shape[1], int(dim), ctypes.c_float(eps), _code(rows), _stream(rows))
    _check(st, "scale_rows")
    return out


def gemm_skinny_residual(x: torch.Tensor, w, h: torch.Tensor, norm_weight: torch.Tensor,
                         eps: float) -> ScaledRows:
    """For at most 16 rows: ``h += x @ w.T`` on the fp32 residual stream ``h [M, N]`` and, in the same
    kernel, what the RMSNorm that follows needs: ``h * norm_weight`` in bfloat16 and a sum of squares
    of ``h`` per row and workgroup (16 columns).  ``x`` may itself be :class:`ScaledRows`, ``w`` a
    matrix or :class:`PackedWeight`."""
    rows = x.rows if isinstance(x, ScaledRows) else x
    _gpu(rows, h, norm_weight)
    M, K = rows.shape
    N = w.shape[0]
    _need(rows.dtype == torch.bfloat16 and 0 < M <= 16, "gemm_skinny_residual takes bfloat16 x [M<=16, K] and w [N, K]")
    _need(K % 8 == 0 and rows.stride(1) == 1 and rows.stride(0) % 8 == 0 and rows.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    w_ptr, ldw = _weight_args(w, K, "gemm_skinny_residual")
    _need(h.dtype == torch.float32 and h.shape == (M, N) and h.stride(1) == 1, "h must be float32 [M, N]")
    _need(norm_weight.shape == (N,) and norm_weight.is_contiguous()
          and norm_weight.dtype in (torch.float32, torch.bfloat16), "norm_weight must be [N], float32 or bfloat16")
    n_parts = -(-N // 16)
    x_out = torch.empty((M, N), dtype=torch.bfloat16, device=rows.device)
    ssq_out = torch.empty((M, n_parts), dtype=torch.float32, device=rows.device)
    sc = _row_scale_args(x, M)
    st = _lib.load("gemm_skinny").fg_gemm_skinny_fused(
        _ptr(rows), rows.stride(0), w_ptr, ldw, ctypes.c_void_p(0), 0, M, N, K, 3, *sc,
        _ptr(h), h.stride(0), _ptr(norm_weight), _code(norm_weight), _ptr(x_out), x_out.stride(0), _ptr(ssq_out),
        _stream(rows))
    _check(st, "gemm_skinny_residual")
    return ScaledRows(x_out, ssq_out, N, float(eps))


def gemm_skinny(x, w, out_dtype: Optional[torch.dtype] = None,
                silu_mul_epilogue: bool = False, k_splits: int = 1, wide: Optional[bool] = None) -> torch.Tensor:
    """``x @ w.T`` for at most 128 rows of bf16 ``x`` on the matrix cores, built to
    stream ``w [N, K]`` (a matrix or :class:`PackedWeight`) once.  ``x`` may be :class:`ScaledRows` (at most 16 rows, bfloat16 out): the
    result rows are scaled.  With ``silu_mul_epilogue`` ``w`` is a gate/up matrix
    ordered by :func:`interleave_gate_up` and the result is ``silu(gate) * up``
    ``[M, N/2]``.  With ``k_splits > 1`` the k range is cut over workgroups and the
    result is fp32 ``[k_splits, M, N]`` partial sums (for few output columns,
    where one workgroup per 64 columns would leave most of the GPU idle).
    ``wide`` picks the kernel for 17..128 rows (64 columns a workgroup, x shared
    through LDS; it takes fewer rows and ``ScaledRows`` too); default: by the number of rows."""
    scaled = x if isinstance(x, ScaledRows) else None
    if scaled is not None:
        x = scaled.rows
    _gpu(x)
    _need(x.dtype == torch.bfloat16 and x.dim() == 2, "gemm_skinny takes bfloat16 x [M, K]")
    M, K = x.shape
    N = w.shape[0]
    _need(0 < M <= SKINNY_MAX_ROWS, f"gemm_skinny takes 1..{SKINNY_MAX_ROWS} rows, got {M}")
    _need(K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    w_ptr, ldw = _weight_args(w, K, "gemm_skinny")
    out_dtype = out_dtype or torch.bfloat16
    if silu_mul_epilogue:
        _need(N % 16 == 0 and out_dtype == torch.bfloat16, "the gate/up epilogue needs N % 16 == 0 and bf16 output")
    wide = (M > 16 or k_splits > 1) if wide is None else wide
    _need(M <= 64 or wide, "more than 64 rows take the wide kernel")
    _need(k_splits >= 1 and (k_splits == 1 or (wide and not silu_mul_epilogue)), "k_splits needs the wide kernel")
    if k_splits > 1:
        out_dtype = torch.float32
    cols = N // 2 if silu_mul_epilogue else N
    y = torch.empty((k_splits, M, cols) if k_splits > 1 else (M, cols), dtype=out_dtype, device=x.device)
    lib = _lib.load("gemm_skinny")
    if scaled is not None and wide:
        _need(M <= 16 and k_splits == 1 and out_dtype == torch.bfloat16, "scaled rows: at most 16 rows, bfloat16 out")
        st = lib.fg_gemm_skinny64(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), cols, ctypes.c_longlong(M * cols), 1, M, N,
            K, _code(y), 1 if silu_mul_epilogue else 0, *_row_scale_args(scaled, M), _stream(x))
    elif scaled is not None:
        _need(M <= 16 and out_dtype == torch.bfloat16, "scaled rows: at most 16 rows, bfloat16 out")
        st = lib.fg_gemm_skinny_fused(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), y.stride(0), M, N, K, 1 if silu_mul_epilogue else 0,
            *_row_scale_args(scaled, M), ctypes.c_void_p(0), 0, ctypes.c_void_p(0), 0, ctypes.c_void_p(0), 0,
            ctypes.c_void_p(0), _stream(x))
    elif wide:
        st = lib.fg_gemm_skinny64(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), cols, ctypes.c_longlong(M * cols), k_splits, M, N,
            K, _code(y), 1 if silu_mul_epilogue else 0, *_row_scale_args(None, M), _stream(x))
    else:
        st = lib.fg_gemm_skinny(
            _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), y.stride(0), M, N, K, _code(y),
            1 if silu_mul_epilogue else 0, _stream(x))
    _check(st, "gemm_skinny")
    return y


TILED_TILE_ROWS = (128, 256)  # rows of x a workgroup of the tiled kernel takes (by 128 columns)


def gemm_tiled(x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None,
               silu_mul_epilogue: bool = False, k_splits: int = 1, tile_rows: int = 128) -> torch.Tensor:
    """``x @ w.T`` for many rows of bf16 ``x`` by the engine's tiled MFMA kernel (both operands through a
    ring of LDS stages), with the k range cut over workgroups if ``k_splits > 1``: the result is then
    fp32 ``[k_splits, M, N]`` partial sums.  ``tile_rows``: 128 or 256 rows of x a workgroup (by 128
    columns).  With ``silu_mul_epilogue`` as :func:`gemm_skinny`; ``w`` a matrix or :class:`PackedWeight`."""
    _gpu(x)
    _need(x.dtype == torch.bfloat16 and x.dim() == 2, "gemm_tiled takes bfloat16 x [M, K]")
    M, K = x.shape
    N = w.shape[0]
    _need(M > 0 and K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    w_ptr, ldw = _weight_args(w, K, "gemm_tiled")
    _need(tile_rows in TILED_TILE_ROWS, f"tile_rows must be one of {TILED_TILE_ROWS}")
    out_dtype = out_dtype or torch.bfloat16
    if silu_mul_epilogue:
        _need(N % 16 == 0 and out_dtype == torch.bfloat16 and k_splits == 1,
              "the gate/up epilogue needs N % 16 == 0, bf16 output and one split")
    _need(1 <= k_splits <= 65535, "k_splits must be 1..65535")
    if k_splits > 1:
        out_dtype = torch.float32
    cols = N // 2 if silu_mul_epilogue else N
    y = torch.empty((k_splits, M, cols) if k_splits > 1 else (M, cols), dtype=out_dtype, device=x.device)
    st = _lib.load("gemm_tiled").fg_gemm_tiled(
        _ptr(x), x.stride(0), w_ptr, ldw, _ptr(y), cols, ctypes.c_longlong(M * cols), k_splits, M, N, K,
        _code(y), 1 if silu_mul_epilogue else 0, int(tile_rows), _stream(x))
    _check(st, "gemm_tiled")
    return y


def gemm_skinny_qkv(x, wqkv, table: Optional[torch.Tensor], slots: torch.Tensor,
                    k_pages: torch.Tensor, v_pages: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                    rotary_dim: int) -> torch.Tensor:
    """The q, k, v projections of at most 16 rows with :func:`rope_kv_write` in
    the product's epilogue: returns the rotated queries ``[M, H*hd]``; the rotated
    keys and the values go straight into their cache pages.  ``x`` may be :class:`ScaledRows`, ``wqkv`` a
    matrix or :class:`PackedWeight`."""
    scaled = x if isinstance(x, ScaledRows) else None
    if scaled is not None:
        x = scaled.rows
    _gpu(x, table, slots, k_pages, v_pages)
    _need(x.dim() == 2 and k_pages.dim() == 4, "x [M, K], wqkv [N, K], k_pages [n, KV, P, hd]")
    M, K = x.shape
    _need(x.dtype == torch.bfloat16 and k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16,
          "gemm_skinny_qkv takes bfloat16")
    w_ptr, ldw = _weight_args(wqkv, K, "gemm_skinny_qkv")
    _need(0 < M <= 16 and tuple(wqkv.shape) == ((n_heads + 2 * n_kv) * head_dim, K), "x [M<=16, K], wqkv [(H+2KV)*hd, K]")
    _need(K % 8 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0,
          "K must be a multiple of 8, rows 16-byte aligned")
    _need(head_dim % 16 == 0, "head size must be a multiple of 16")
    page_size = k_pages.shape[2]
    _need(k_pages.is_contiguous() and v_pages.is_contiguous() and k_pages.shape[1:] == (n_kv, page_size, head_dim)
          and v_pages.shape == (k_pages.shape[0], n_kv, head_dim, page_size), "pages do not fit the heads")
    _i32(slots, "slots", M)
    if rotary_dim:
        _need(table is not None and table.dtype == torch.float32 and table.is_contiguous()
              and table.shape == (M, rotary_dim // 2, 2), "table must be float32 [M, rotary_dim/2, 2]")
    q = torch.empty((M, n_heads * head_dim), dtype=torch.bfloat16, device=x.device)
    st = _lib.load("gemm_skinny").fg_gemm_skinny_qkv(
        _ptr(x), x.stride(0), w_ptr, ldw, _ptr(q), q.stride(0), M, K,
        _ptr(table if rotary_dim else None), _ptr(slots), _ptr(k_pages), _ptr(v_pages), n_heads, n_kv, head_dim,
        rotary_dim, page_size, *_row_scale_args(scaled, M), _stream(x))
    _check(st, "gemm_skinny_qkv")
    return q


# ------------------------------------------------------------------- sampling
def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None,
           top_p: Optional[torch.Tensor] = None, seeds: Optional[torch.Tensor] = None,
           counters: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token id per row of fp32 ``logits [n, V]``: argmax where the row's
    temperature is 0 (or none is given), else a draw from
    ``softmax(logits / temperature)`` cut to the ``top_p`` nucleus, with the
    uniform number taken from ``(seeds[row], counters[row])``.
    ``fastgen/generate.py:887-896``, ``utils/sampling.py:6-31``.
    """
    _gpu(logits, temperature, top_p, seeds, counters, out)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "logits must be float32 [n, V]")
    n, V = logits.shape
    out = torch.empty((n,), dtype=torch.int32, device=logits.device) if out is None else out
    _i32(out, "out", n)
    for name, t in (("temperature", temperature), ("top_p", top_p)):
        if t is not None:
            _need(t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= n, f"{name} must be float32 [n]")
    for name, t in (("seeds", seeds), ("counters", counters)):
        if t is not None:
            _need(t.dtype == torch.int64 and t.is_contiguous() and t.numel() >= n, f"{name} must be int64 [n]")
    if temperature is not None:
        _need(seeds is not None and counters is not None, "sampling needs seeds and counters")
    st = _lib.load("sampling").fg_sample(
        _ptr(logits), logits.stride(0), n, V, _ptr(temperature), _ptr(top_p), _ptr(seeds), _ptr(counters),
        _ptr(out), _stream(logits))
    _check(st, "sample")
    return out


def logprob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """``log_softmax(logits)[row, tokens[row]]`` (``fastgen/generate.py:725-730``)."""
    _gpu(logits, tokens)
    _need(logits.dim() == 2 and logits.dtype == torch.float32 and logits.stride(1) == 1,
          "logits must be float32 [n, V]")
    n, V = logits.shape
    _i32(tokens, "tokens", n)
    out = torch.empty((n,), dtype=torch.float32, device=logits.device)
    st = _lib.load("sampling").fg_logprob(_ptr(logits), logits.stride(0), n, V, _ptr(tokens), _ptr(out), _stream(logits))
    _check(st, "logprob")
    return out
