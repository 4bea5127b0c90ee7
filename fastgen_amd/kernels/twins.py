"""A plain PyTorch function beside every kernel of ``ops``: the same name, the
same arguments, the same effect on the same tensors, written as the formula
and not as the kernel works.  They say what each kernel computes and are what
the kernels are held to in ``tests/test_twins.py``; nothing of the engine
calls them (the engine has no execution path but its kernels), and they work
on CPU tensors as well as on GPU ones.

All arithmetic between a load and a store is fp32, as in the kernels; a result
is rounded once, to the dtype of the tensor it goes to.  Formulas:
``fastgen/forward.py:406-515``, ``fastgen/kernels/{rmsnorm,rope,paged_memcpy}.py``,
``fastgen/utils/sampling.py``.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.layout import store_k, store_v, unpack_k, unpack_v
from .ops import PackedWeight, ScaledRows


def embed(table: torch.Tensor, tokens: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """``out[t] = table[tokens[t]]`` as fp32."""
    out.copy_(table[tokens.long()].float())
    return out


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``h += delta`` (a ``[T, dim]`` tensor, or fp32 ``[S, T, dim]`` partial sums added in order), then
    ``out = h * rsqrt(mean(h^2) + eps) * weight``; with ``rows`` only those rows, and ``h`` stays as it was."""
    total = h.clone()
    if delta is not None and delta.dim() == 3:
        for s in range(delta.shape[0]):
            total += delta[s]
    elif delta is not None:
        total += delta.float()
    if rows is None:
        h.copy_(total)
    else:
        total = total[rows.long()]
    rstd = torch.rsqrt((total * total).sum(-1, keepdim=True) / total.shape[-1] + eps)
    out.copy_((total * rstd * weight.float()).to(out.dtype))
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    xf = x.float()
    y = (xf * torch.rsqrt((xf * xf).sum(-1, keepdim=True) / x.shape[-1] + eps) * weight.float()).to(x.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of the gate and the up matrix in turns of 8: gate rows 8j..8j+7, then up rows 8j..8j+7."""
    F, K = gate.shape
    return torch.stack([gate.view(F // 8, 8, K), up.view(F // 8, 8, K)], dim=1).reshape(2 * F, K)


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``silu(gate) * up`` of ``[T, 2F]`` whose columns are interleaved in turns of 8 as above."""
    T, F2 = gate_up.shape
    gu = gate_up.float().view(T, F2 // 16, 2, 8)
    g, u = gu[:, :, 0].reshape(T, F2 // 2), gu[:, :, 1].reshape(T, F2 // 2)
    y = (g * torch.sigmoid(g) * u).to(gate_up.dtype)
    if out is None:
        return y
    out.copy_(y)
    return out


def rope_table(positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """fp32 ``[T, len(freqs), 2]``: cos and sin of ``position * frequency``."""
    ang = positions.to(torch.float32)[:, None] * freqs.float()[None, :]
    return torch.stack([torch.cos(ang), torch.sin(ang)], dim=-1)


def _rotate(x: torch.Tensor, table: torch.Tensor, rotary_dim: int) -> torch.Tensor:
    """Interleaved pairs ``(2i, 2i+1)`` of the first ``rotary_dim`` head dims of ``x [T, heads, hd]`` (fp32)."""
    out = x.clone()
    if rotary_dim:
        cos, sin = table[:, None, :, 0], table[:, None, :, 1]
        a, b = x[..., 0:rotary_dim:2], x[..., 1:rotary_dim:2]
        out[..., 0:rotary_dim:2] = a * cos - b * sin
        out[..., 1:rotary_dim:2] = b * cos + a * sin
    return out


def _write_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, slots: torch.Tensor, k: torch.Tensor,
                 v: torch.Tensor) -> None:
    """Rows ``k, v [T, KV, hd]`` into the pages at ``slots`` (page * P + offset; negative: not written)."""
    P = k_pages.shape[2]
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        page, off = divmod(s, P)
        for kvh in range(k_pages.shape[1]):
            store_k(k_pages, page, kvh, off, k[t, kvh].to(k_pages.dtype))
            store_v(v_pages, page, kvh, off, v[t, kvh].to(v_pages.dtype))


def rope_kv_write(qkv: torch.Tensor, positions: torch.Tensor, freqs: Optional[torch.Tensor], slots: torch.Tensor,
                  k_pages: torch.Tensor, v_pages: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                  rotary_dim: int, write_kv: bool = True, table: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``qkv [T, >= H*hd (+ 2*KV*hd)]``: q is rotated in place; k is rotated and, with v, written into the
    pages (``fastgen/kernels/rope.py:56-89``, ``paged_memcpy.py:57-76``)."""
    T = qkv.shape[0]
    if rotary_dim and table is None:
        table = rope_table(positions, freqs)
    q_cols, kv_cols = n_heads * head_dim, n_kv * head_dim
    q = _rotate(qkv[:, :q_cols].float().view(T, n_heads, head_dim), table, rotary_dim)
    qkv[:, :q_cols] = q.reshape(T, q_cols).to(qkv.dtype)
    if write_kv:
        k = _rotate(qkv[:, q_cols : q_cols + kv_cols].float().view(T, n_kv, head_dim), table, rotary_dim)
        v = qkv[:, q_cols + kv_cols : q_cols + 2 * kv_cols].float().view(T, n_kv, head_dim)
        _write_pages(k_pages, v_pages, slots, k, v)
    return qkv


def _gather_kv(pages: torch.Tensor, unpack, table_row: torch.Tensor, n: int) -> torch.Tensor:
    """The first ``n`` keys (or values) of a sequence in natural order ``[n, KV, hd]``, fp32."""
    P = pages.shape[2] if unpack is unpack_k else pages.shape[3]
    natural = unpack(pages[table_row[: -(-n // P)].long()])  # [n_pages, KV, P, hd]
    return natural.permute(0, 2, 1, 3).reshape(-1, natural.shape[1], natural.shape[3])[:n].float()


def paged_attention_general(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                            block_table: torch.Tensor, seq_of_token: torch.Tensor, positions: torch.Tensor,
                            n_heads: int, scale: float, window: int = 0) -> torch.Tensor:
    """Token ``t`` of sequence ``b`` at position ``p`` attends keys ``0..p`` (``p-window+1..p`` with a window)
    of its sequence, read through ``block_table[b]``; query head ``h`` reads kv head ``h // (H / KV)``;
    softmax of ``scale * q.k`` in fp32 (``fastgen/forward.py:176-258``)."""
    n_kv, P, hd = k_pages.shape[1], k_pages.shape[2], k_pages.shape[3]
    G = n_heads // n_kv
    for t in range(q.shape[0]):
        b, p = int(seq_of_token[t]), int(positions[t])
        k = _gather_kv(k_pages, unpack_k, block_table[b], p + 1)
        v = _gather_kv(v_pages, unpack_v, block_table[b], p + 1)
        lo = max(0, p - window + 1) if window else 0
        qt = q[t, : n_heads * hd].float().view(n_heads, hd)
        for h in range(n_heads):
            s = (k[lo:, h // G] @ qt[h]) * scale
            out[t, h * hd : (h + 1) * hd] = (torch.softmax(s, 0) @ v[lo:, h // G]).to(out.dtype)
    return out


def paged_attention_mfma(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                         block_table: torch.Tensor, small_items: Optional[torch.Tensor],
                         big_items: Optional[torch.Tensor], n_heads: int, scale: float, window: int = 0,
                         plan=None, max_chunks=None, min_tiles: int = 4, max_rows: int = 16,
                         tile_rows=None) -> torch.Tensor:
    """The same attention for tokens listed as items (sequence, first flat token, tokens, position of the
    first token).  How the kernels cut the work (``plan`` and what follows it) does not change the result."""
    seq_of_token = torch.zeros(q.shape[0], dtype=torch.int32)
    positions = torch.zeros(q.shape[0], dtype=torch.int32)
    for items in (small_items, big_items):
        if items is None:
            continue
        for b, first, n, pos in items.reshape(-1, 4).tolist():
            seq_of_token[first : first + n] = b
            positions[first : first + n] = torch.arange(pos, pos + n, dtype=torch.int32)
    return paged_attention_general(q, out, k_pages, v_pages, block_table, seq_of_token, positions, n_heads, scale,
                                   window)


def paged_attention(q: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor,
                    group, ctx, n_heads: int, scale: float, window: int = 0) -> torch.Tensor:
    """Attention of one step: the block table from the layer's cache group, sequences and positions of the
    tokens from the step's context."""
    return paged_attention_general(q, out, k_pages, v_pages, group.block_table, ctx.seq_of_token, ctx.positions,
                                   n_heads, scale, window)


def gemm_nt(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None,
            out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``x @ w.T`` with fp32 accumulation."""
    y = (x.float() @ w.float().T).to(out_dtype or (out.dtype if out is not None else x.dtype))
    if out is None:
        return y
    out.copy_(y)
    return out


def _rows(x) -> torch.Tensor:
    """The true rows of ``x``, a tensor or :class:`ScaledRows`, in fp32."""
    if isinstance(x, ScaledRows):
        return x.rows.float() * torch.rsqrt(x.ssq.sum(1, keepdim=True) / x.dim + x.eps)
    return x.float()


def _matrix(w) -> torch.Tensor:
    """The weight matrix ``[N, K]`` in fp32, from a matrix or from :class:`PackedWeight` (the inverse of the
    packing, written out: block ``[nb, ks]`` holds rows ``16 nb + r`` and k ``32 ks + 8 g + e`` at lane
    ``16 g + r``, element ``e``)."""
    if not isinstance(w, PackedWeight):
        return w.float()
    nb, ks = w.data.shape[:2]
    out = torch.zeros((nb * 16, ks * 32), dtype=torch.float32, device=w.data.device)
    for g in range(4):
        for r in range(16):
            out[r::16].view(nb, ks, 32)[:, :, 8 * g : 8 * g + 8] = w.data[:, :, 16 * g + r, :].float()
    return out[: w.n, : w.k]


def scale_rows(rows: torch.Tensor, ssq: torch.Tensor, dim: int, eps: float) -> torch.Tensor:
    return (rows.float() * torch.rsqrt(ssq.sum(1, keepdim=True) / dim + eps)).to(rows.dtype)


def gemm_skinny(x, w, out_dtype: Optional[torch.dtype] = None, silu_mul_epilogue: bool = False,
                k_splits: int = 1, wide: Optional[bool] = None) -> torch.Tensor:
    """``x @ w.T`` (``x`` may be :class:`ScaledRows`, ``w`` :class:`PackedWeight`: so in all three); with ``silu_mul_epilogue`` ``silu(gate) * up`` of a gate/up
    matrix interleaved in turns of 8; with ``k_splits > 1`` fp32 ``[S, M, N]`` partial sums over the k ranges
    ``[s * ceil(K / S / 256) * 256, ...)``.  ``wide`` only picks a kernel."""
    xf, wf = _rows(x), _matrix(w)
    if k_splits > 1:
        K = wf.shape[1]
        step = -(-K // (k_splits * 256)) * 256
        return torch.stack([xf[:, s * step : (s + 1) * step] @ wf[:, s * step : (s + 1) * step].T
                            for s in range(k_splits)])
    y = xf @ wf.T
    if silu_mul_epilogue:
        M, N = y.shape
        gu = y.view(M, N // 16, 2, 8)
        g, u = gu[:, :, 0].reshape(M, N // 2), gu[:, :, 1].reshape(M, N // 2)
        y = g * torch.sigmoid(g) * u
    return y.to(out_dtype or torch.bfloat16)


def gemm_tiled(x: torch.Tensor, w, out_dtype: Optional[torch.dtype] = None,
               silu_mul_epilogue: bool = False, k_splits: int = 1, tile_rows: int = 128) -> torch.Tensor:
    """``x @ w.T``; with ``silu_mul_epilogue`` as :func:`gemm_skinny`; with ``k_splits > 1`` fp32 ``[S, M, N]``
    partial sums over the k ranges ``[s * ceil(K / S / 32) * 32, ...)``.  ``tile_rows`` only picks a tile."""
    xf, wf = x.float(), _matrix(w)
    if k_splits > 1:
        K = wf.shape[1]
        step = -(-K // (k_splits * 32)) * 32
        return torch.stack([xf[:, s * step : (s + 1) * step] @ wf[:, s * step : (s + 1) * step].T
                            for s in range(k_splits)])
    y = xf @ wf.T
    if silu_mul_epilogue:
        M, N = y.shape
        gu = y.view(M, N // 16, 2, 8)
        g, u = gu[:, :, 0].reshape(M, N // 2), gu[:, :, 1].reshape(M, N // 2)
        y = g * torch.sigmoid(g) * u
    return y.to(out_dtype or torch.bfloat16)


def gemm_skinny_residual(x, w, h: torch.Tensor, norm_weight: torch.Tensor, eps: float) -> ScaledRows:
    """``h += x @ w.T``; returns what the RMSNorm after it needs: ``h * norm_weight`` in bfloat16 and the sums of
    squares of ``h`` over each block of 16 columns."""
    h += _rows(x) @ _matrix(w).T
    M, N = h.shape
    sq = torch.nn.functional.pad(h * h, (0, -N % 16)).view(M, -1, 16).sum(-1)
    return ScaledRows((h * norm_weight.float()).to(torch.bfloat16), sq, N, float(eps))


def gemm_skinny_qkv(x, wqkv, table: Optional[torch.Tensor], slots: torch.Tensor, k_pages: torch.Tensor,
                    v_pages: torch.Tensor, n_heads: int, n_kv: int, head_dim: int, rotary_dim: int) -> torch.Tensor:
    """The q, k, v projections with :func:`rope_kv_write` on the fp32 sums: returns the rotated queries in
    bfloat16; the rotated keys and the values go into the pages."""
    qkv = _rows(x) @ _matrix(wqkv).T
    T, q_cols, kv_cols = qkv.shape[0], n_heads * head_dim, n_kv * head_dim
    q = _rotate(qkv[:, :q_cols].view(T, n_heads, head_dim), table, rotary_dim)
    k = _rotate(qkv[:, q_cols : q_cols + kv_cols].view(T, n_kv, head_dim), table, rotary_dim)
    v = qkv[:, q_cols + kv_cols :].view(T, n_kv, head_dim)
    _write_pages(k_pages, v_pages, slots, k, v)
    return q.reshape(T, q_cols).to(torch.bfloat16)


def sample(logits: torch.Tensor, temperature: Optional[torch.Tensor] = None, top_p: Optional[torch.Tensor] = None,
           seeds: Optional[torch.Tensor] = None, counters: Optional[torch.Tensor] = None,
           out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Greedy rows (no temperature, or temperature 0): the lowest index among the largest logits.  For rows with
    a temperature the kernel draws with a generator of its own keyed by (seed, counter); this function gives
    the set a draw must come from instead: -1 for such a row (see :func:`sample_support`)."""
    tok = torch.argmax(logits, dim=-1).to(torch.int32)  # torch.argmax returns the first of equal maxima
    if temperature is not None:
        tok = torch.where(temperature[: logits.shape[0]] > 0, torch.full_like(tok, -1), tok)
    if out is None:
        return tok
    out.copy_(tok)
    return out


def sample_support(logits: torch.Tensor, temperature: float, top_p: float) -> torch.Tensor:
    """bool ``[V]``: the tokens a draw with this temperature and nucleus can give, that is, those whose
    preceding mass in descending order of probability does not exceed ``top_p`` (``fastgen/utils/sampling.py:26-28``)."""
    probs = torch.softmax(logits.float() / temperature, -1)
    sort, idx = torch.sort(probs, descending=True)
    keep_sorted = ~(torch.cumsum(sort, -1) - sort > top_p)
    keep = torch.zeros_like(keep_sorted)
    keep[idx] = keep_sorted
    return keep


def logprob(logits: torch.Tensor, tokens: torch.Tensor) -> torch.Tensor:
    """``log_softmax(logits)[row, tokens[row]]`` (``fastgen/generate.py:725-730``)."""
    return torch.log_softmax(logits.float(), -1)[torch.arange(logits.shape[0], device=logits.device), tokens.long()]
