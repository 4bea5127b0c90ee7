"""The order of elements inside a cache page, for code that fills or reads
pages outside the kernels (tests, tools).  The kernels' own statement of the
layout is ``csrc/kv_layout.h``; this file says the same in index tensors.

Per kv head a page holds ``P*hd`` key elements and ``P*hd`` value elements.
``k_index(P, hd)[kappa, d]`` is the flat offset of key ``kappa``'s head
dimension ``d``; ``v_index(P, hd)[kappa, d]`` the same for values.
"""

from __future__ import annotations

from functools import lru_cache

import torch


@lru_cache(maxsize=None)
def k_index(page_size: int, head_dim: int) -> torch.Tensor:
    kb = 16 if page_size % 16 == 0 else 8
    kappa = torch.arange(page_size)[:, None]
    d = torch.arange(head_dim)[None, :]
    return (((kappa // kb) * (head_dim // 8) + d // 8) * kb + kappa % kb) * 8 + d % 8


@lru_cache(maxsize=None)
def v_index(page_size: int, head_dim: int) -> torch.Tensor:
    db = 16 if head_dim % 16 == 0 else 8
    kappa = torch.arange(page_size)
    if page_size % 32 == 0:
        k = kappa % 32
        slot = kappa - k + 8 * ((k % 16) // 4) + 4 * (k // 16) + k % 4
    else:
        slot = kappa
    slot = slot[:, None]
    d = torch.arange(head_dim)[None, :]
    return (((d // db) * (page_size // 8) + slot // 8) * db + d % db) * 8 + slot % 8


def store_k(pages: torch.Tensor, page: int, kv_head: int, kappa: int, k: torch.Tensor) -> None:
    """Write one key ``[hd]`` into ``pages [n_pages, KV, P, hd]``."""
    P, hd = pages.shape[2], pages.shape[3]
    pages[page, kv_head].view(-1)[k_index(P, hd)[kappa].to(pages.device)] = k


def store_v(pages: torch.Tensor, page: int, kv_head: int, kappa: int, v: torch.Tensor) -> None:
    """Write one value ``[hd]`` into ``pages [n_pages, KV, hd, P]``."""
    hd, P = pages.shape[2], pages.shape[3]
    pages[page, kv_head].view(-1)[v_index(P, hd)[kappa].to(pages.device)] = v


def pack_k(natural: torch.Tensor) -> torch.Tensor:
    """``[..., P, hd]`` keys in natural order -> the same shape in storage order."""
    P, hd = natural.shape[-2:]
    out = torch.empty_like(natural).reshape(*natural.shape[:-2], P * hd)
    out[..., k_index(P, hd).reshape(-1).to(natural.device)] = natural.reshape(*natural.shape[:-2], P * hd)
    return out.reshape(natural.shape)


def pack_v(natural: torch.Tensor) -> torch.Tensor:
    """``[..., P, hd]`` values in natural order -> ``[..., hd, P]`` storage."""
    P, hd = natural.shape[-2:]
    out = torch.empty_like(natural).reshape(*natural.shape[:-2], P * hd)
    out[..., v_index(P, hd).reshape(-1).to(natural.device)] = natural.reshape(*natural.shape[:-2], P * hd)
    return out.reshape(*natural.shape[:-2], hd, P)


def unpack_k(stored: torch.Tensor) -> torch.Tensor:
    """Storage order ``[..., P, hd]`` -> natural ``[..., P, hd]``."""
    P, hd = stored.shape[-2:]
    flat = stored.reshape(*stored.shape[:-2], P * hd)
    return flat[..., k_index(P, hd).reshape(-1).to(stored.device)].reshape(stored.shape)


def unpack_v(stored: torch.Tensor) -> torch.Tensor:
    """Storage ``[..., hd, P]`` -> natural ``[..., P, hd]``."""
    hd, P = stored.shape[-2:]
    flat = stored.reshape(*stored.shape[:-2], P * hd)
    return flat[..., v_index(P, hd).reshape(-1).to(stored.device)].reshape(*stored.shape[:-2], P, hd)
