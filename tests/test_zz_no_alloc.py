"""The decode attention entry point that allocates nothing (``fg_attn_decode_static``,
``csrc/attention_static.h``), called through ``ctypes`` as a caller without an allocator would:
its output against the existing entry points' (``fg_attn_plan`` + ``fg_attn_split`` with buffers
from the caller) on two calls in a row, the second with a smaller input, so that what the first
call left in the static array is there when the second runs."""

import ctypes

import numpy as np
import pytest
import torch

from test_gpu_kernels import DEV, _paged_case, _plain_rows

pytestmark = pytest.mark.gpu


def _static_call(lib, case, items, n_items, max_chunks, min_tiles, max_rows, H, KV, hd, P, out, window=0):
    from fastgen_amd.kernels.ops import _ptr, _stream

    q = case["q"]
    return lib.fg_attn_decode_static(
        _ptr(q), q.stride(0), _ptr(out), out.stride(0), _ptr(case["kp"]), _ptr(case["vp"]), _ptr(case["table"]),
        case["table"].stride(0), _ptr(items), n_items, max_chunks, min_tiles, max_rows, H, KV, hd, P,
        ctypes.c_float(hd ** -0.5), window, _stream(q))


@pytest.mark.parametrize("H,KV,hd,P,window,n_new", [(32, 8, 128, 64, 0, 1), (5, 1, 48, 32, 0, 1),
                                                    (32, 8, 128, 64, 100, 1), (32, 8, 128, 64, 0, 2),
                                                    (5, 1, 48, 32, 100, 2)])
def test_decode_attention_without_allocation(H, KV, hd, P, window, n_new):
    """``window``: keys further back than that are not seen (the plan then starts behind key 0);
    ``n_new``: tokens an item brings (two tokens of a group of at most 8 heads are one item of at most 16 rows)."""
    from fastgen_amd.kernels import _lib, ops

    lib = _lib.load(f"attention_mfma@{hd}")
    lib.fg_attn_decode_static_error.restype = ctypes.c_char_p
    G = H // KV
    assert G * n_new <= 16
    # the first call: many sequences, some long (several chunks each); the second: fewer and shorter
    calls = [
        [(n, n_new) for n in (700, 64, 1500, 3, 255, 256, 1023, 90, 2100, 17, 333, 640)],
        [(n, n_new) for n in (300, 5, 129)],
    ]
    n_calls = 0
    for min_tiles in (4, 1):
        for seqs in calls:
            case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=31 + len(seqs))
            q_lens = [b for _, b in seqs]
            q_start = np.concatenate([[0], np.cumsum(q_lens)])
            small, big = ops.attention_items(q_lens, q_start, [a for a, _ in seqs], G, ops.attention_tile_rows(hd))
            assert len(small) == len(seqs) and not len(big)
            items = torch.from_numpy(small.reshape(-1)).to(DEV)
            n = len(seqs)
            max_chunks = ops.attention_chunks_for(n, KV)
            assert max_chunks <= lib.fg_attn_decode_static_max_chunks(KV)
            # the existing entry points, with buffers that torch allocates
            want = torch.full_like(case["q"], float("nan"))
            ops.paged_attention_mfma(case["q"], want, case["kp"], case["vp"], case["table"], items, None, H,
                                     hd ** -0.5, window, None, max_chunks, min_tiles, max_rows=G * n_new)
            got = torch.full_like(case["q"], float("nan"))
            torch.cuda.synchronize()
            before = torch.cuda.memory_stats()["allocation.all.allocated"]
            free_before = torch.cuda.mem_get_info()[0]
            st = _static_call(lib, case, items, n, max_chunks, min_tiles, G * n_new, H, KV, hd, P, got, window)
            assert st == 0, lib.fg_attn_decode_static_error().decode()
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == before  # torch was asked for nothing
            torch.cuda.synchronize()
            if n_calls:  # (the library's code and its array reach the device with its first launch)
                assert torch.cuda.mem_get_info()[0] == free_before  # and the device for nothing either
            n_calls += 1
            assert torch.isfinite(got).all()
            assert torch.equal(got, want)  # the same kernels with the same cut: the same bits
            assert torch.allclose(got.cpu().float(), _plain_rows(case, seqs, window or None), atol=1.5e-2, rtol=2e-2)


def test_sizes_beyond_the_static_array_are_refused():
    from fastgen_amd.kernels import _lib

    H, KV, hd, P = 32, 8, 128, 64
    lib = _lib.load(f"attention_mfma@{hd}")
    lib.fg_attn_decode_static_error.restype = ctypes.c_char_p
    most = lib.fg_attn_decode_static_max_chunks(KV)
    assert 100 < most < 65535
    seqs = [(10, 1)]
    case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=3)
    items = torch.tensor([0, 0, 1, 10], dtype=torch.int32, device=DEV)
    out = torch.full_like(case["q"], 7.0)
    st = _static_call(lib, case, items, 1, most + 1, 4, H // KV, H, KV, hd, P, out)
    torch.cuda.synchronize()
    assert st == 3 and b"static array holds" in lib.fg_attn_decode_static_error()
    assert (out == 7.0).all()  # nothing ran
    st = _static_call(lib, case, items, 1, most, 4, H // KV, H, KV, hd, P, out)
    torch.cuda.synchronize()
    assert st == 0 and lib.fg_attn_decode_static_error() == b""
    assert torch.allclose(out.cpu().float(), _plain_rows(case, seqs), atol=1.5e-2, rtol=2e-2)
