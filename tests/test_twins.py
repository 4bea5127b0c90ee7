"""The plain PyTorch twin beside each kernel (``fastgen_amd/kernels/twins.py``).

Without a GPU: every kernel of ``ops`` has a twin with the same parameters, and the twins
themselves give what the plain functions of ``tests/plain_llama.py`` give (which share no code with
them).  With a GPU: each kernel against its twin, on the same tensors, at two sizes that differ from
the engine's.
"""

from __future__ import annotations

import inspect
import math

import pytest
import torch

from fastgen_amd.kernels import ops as kernel_ops
from fastgen_amd.kernels import twins
from fastgen_amd.cache.layout import pack_k, pack_v

from plain_llama import plain_attention, plain_rmsnorm, plain_rope_interleaved, plain_top_p_keep

# functions of ops that launch a kernel (the others plan work, build arguments or pick a kernel)
KERNEL_OPS = ["embed", "add_rmsnorm", "rmsnorm", "silu_mul", "rope_table", "rope_kv_write", "paged_attention_general",
              "paged_attention_mfma", "paged_attention", "gemm_nt", "scale_rows", "gemm_skinny_residual", "gemm_skinny",
              "gemm_skinny_qkv", "gemm_tiled", "sample", "logprob"]


@pytest.mark.parametrize("name", KERNEL_OPS + ["interleave_gate_up"])
def test_every_kernel_has_a_twin_with_the_same_parameters(name):
    kernel, twin = getattr(kernel_ops, name), getattr(twins, name)
    assert list(inspect.signature(kernel).parameters) == list(inspect.signature(twin).parameters)


def test_no_kernel_without_a_twin():
    """A function of ``ops`` that loads a library is a kernel's entry: it is on the list above."""
    for name, fn in inspect.getmembers(kernel_ops, inspect.isfunction):
        if fn.__module__ != kernel_ops.__name__ or name.startswith("_"):
            continue
        launches = "_lib.load(" in inspect.getsource(fn) and "_check(" in inspect.getsource(fn)
        if launches and name != "attention_plan":  # the plan is how the work is cut, not a result
            assert name in KERNEL_OPS, f"{name} launches a kernel and has no twin"


def test_twins_are_not_on_the_product_path():
    import pathlib
    root = pathlib.Path(kernel_ops.__file__).resolve().parents[1]
    for path in root.rglob("*.py"):
        if path.name != "twins.py":
            assert "twins" not in path.read_text(), f"{path} names the twins"


# ------------------------------------------------------------ the twins against the plain functions
def _pages(k, v, P, n_pages, table):
    """Natural ``k, v [n, KV, hd]`` of one sequence into pages at ``table``."""
    n, KV, hd = k.shape
    kp = torch.zeros(n_pages, KV, P, hd)
    vp = torch.zeros(n_pages, KV, hd, P)
    pad = -n % P
    kn = torch.nn.functional.pad(k, (0, 0, 0, 0, 0, pad)).view(-1, P, KV, hd).permute(0, 2, 1, 3)
    vn = torch.nn.functional.pad(v, (0, 0, 0, 0, 0, pad)).view(-1, P, KV, hd).permute(0, 2, 1, 3)
    for i, page in enumerate(table[: kn.shape[0]]):
        kp[page], vp[page] = pack_k(kn[i]), pack_v(vn[i])
    return kp, vp


@pytest.mark.parametrize("H,KV,hd,P,n,window", [(6, 2, 24, 8, 37, 0), (5, 5, 16, 16, 50, 11), (4, 1, 40, 32, 70, 0)])
def test_attention_twin_is_plain_attention(H, KV, hd, P, n, window):
    torch.manual_seed(H * 100 + n)
    q, k, v = torch.randn(n, H, hd), torch.randn(n, KV, hd), torch.randn(n, KV, hd)
    table = torch.randperm(16)[: -(-n // P)].tolist()
    kp, vp = _pages(k, v, P, 16, table)
    bt = torch.full((2, 16), -1, dtype=torch.int32)
    bt[1, : len(table)] = torch.tensor(table, dtype=torch.int32)
    out = torch.zeros(n, H * hd)
    twins.paged_attention_general(q.reshape(n, -1), out, kp, vp, bt, torch.ones(n, dtype=torch.int32),
                                  torch.arange(n, dtype=torch.int32), H, 1 / math.sqrt(hd), window)
    want = plain_attention(q, k, v, window or None)
    torch.testing.assert_close(out.view(n, H, hd), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("H,KV,hd,rot,P", [(4, 2, 16, 16, 8), (3, 1, 24, 8, 16)])
def test_rope_kv_write_twin_is_the_plain_rotation(H, KV, hd, rot, P):
    torch.manual_seed(3)
    T = 9
    qkv = torch.randn(T, (H + 2 * KV) * hd)
    before = qkv.clone()
    pos = torch.tensor([3, 4, 5, 0, 1, 100, 101, 7, 8], dtype=torch.int32)
    freqs = 1.0 / 10000.0 ** (torch.arange(0, rot, 2).float() / rot)
    kp, vp = torch.zeros(4, KV, P, hd), torch.zeros(4, KV, hd, P)
    slots = torch.tensor([2 * P + 1, 2 * P + 2, 2 * P + 3, 0, 1, 3 * P + P - 1, 1 * P, -1, 5], dtype=torch.int32)
    twins.rope_kv_write(qkv, pos, freqs, slots, kp, vp, H, KV, hd, rot)
    q0 = before[:, : H * hd].view(T, H, hd)
    want_q = torch.cat([plain_rope_interleaved(q0[..., :rot], pos, freqs), q0[..., rot:]], -1)
    torch.testing.assert_close(qkv[:, : H * hd].view(T, H, hd), want_q, rtol=1e-5, atol=1e-5)
    k0 = before[:, H * hd : (H + KV) * hd].view(T, KV, hd)
    want_k = torch.cat([plain_rope_interleaved(k0[..., :rot], pos, freqs), k0[..., rot:]], -1)
    from fastgen_amd.cache.layout import unpack_k, unpack_v
    kn, vn = unpack_k(kp), unpack_v(vp)  # [pages, KV, P, hd]
    for t, s in enumerate(slots.tolist()):
        if s < 0:
            continue
        torch.testing.assert_close(kn[s // P, :, s % P], want_k[t], rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(vn[s // P, :, s % P], before[t, (H + KV) * hd :].view(KV, hd))
    assert int((kn.abs().sum((1, 3)) > 0).sum()) == 8  # the token with slot -1 is written nowhere


@pytest.mark.parametrize("N,K", [(16, 32), (37, 72), (515, 240), (64, 8)])
def test_packed_weight_layout(N, K):
    """``pack_weight`` against the layout written out element by element (the order the kernels' comment
    gives: block ``[n / 16, k / 32]``, lane ``16 g + r`` holds row ``r`` and k ``8 g .. 8 g + 7``; rows and k
    padded with zeros), its inverse, the twins' reading of it, and the cut at a multiple of 16 rows."""
    torch.manual_seed(N)
    w = torch.randn(N, K).to(torch.bfloat16)
    p = kernel_ops.pack_weight(w)
    nb, ks = -(-N // 16), -(-K // 32)
    assert p.shape == (N, K) and p.data.shape == (nb, ks, 64, 8)
    want = torch.zeros(nb, ks, 64, 8, dtype=torch.bfloat16)
    for n in range(N):
        for k in range(K):
            want[n // 16, k // 32, 16 * ((k % 32) // 8) + n % 16, k % 8] = w[n, k]
    assert torch.equal(p.data, want)
    assert torch.equal(kernel_ops.unpack_weight(p), w)
    assert torch.equal(twins._matrix(p), w.float())
    x = torch.randn(3, K).to(torch.bfloat16)
    assert torch.equal(twins.gemm_skinny(x, p), twins.gemm_skinny(x, w))
    if N > 16:
        assert torch.equal(kernel_ops.unpack_weight(p.first_rows(16)), w[:16])
        with pytest.raises(kernel_ops.KernelArgumentError, match="multiples of 16"):
            p.first_rows(17)


def test_norm_twins_are_the_plain_norm():
    torch.manual_seed(5)
    h, d, w = torch.randn(7, 52), torch.randn(7, 52), torch.rand(52) + 0.5
    out = torch.zeros(7, 52)
    h2 = h.clone()
    twins.add_rmsnorm(h2, d, w, 3e-4, out)
    torch.testing.assert_close(h2, h + d)
    torch.testing.assert_close(out, plain_rmsnorm(h + d, w, 3e-4), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(twins.rmsnorm(h, w, 1e-6), plain_rmsnorm(h, w, 1e-6), rtol=1e-5, atol=1e-5)
    # the folded norm: what gemm_skinny_residual returns, scaled, is the norm of the new residual stream
    x, wt = torch.randn(7, 24), torch.randn(52, 24)
    h3 = h.clone()
    folded = twins.gemm_skinny_residual(x.bfloat16(), wt.bfloat16(), h3, w, 3e-4)
    want = plain_rmsnorm(h + x.bfloat16().float() @ wt.bfloat16().float().T, w, 3e-4)
    torch.testing.assert_close(twins.scale_rows(folded.rows, folded.ssq, folded.dim, folded.eps).float(), want,
                               rtol=2e-2, atol=2e-2)


def test_sample_support_twin_is_the_plain_nucleus():
    torch.manual_seed(9)
    logits = torch.randn(300) * 3
    for p, temp in ((0.3, 1.0), (0.9, 0.7), (1.0, 2.0)):
        keep = twins.sample_support(logits, temp, p)
        assert torch.equal(keep, plain_top_p_keep(torch.softmax(logits / temp, -1), p))


# ----------------------------------------------------------------- the kernels against the twins
gpu = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    return kernel_ops


def _both(fn_name, make, compare, ops):
    """Run the kernel on GPU copies and the twin on CPU copies of what ``make`` returns."""
    args = make()
    dev = [a.cuda() if isinstance(a, torch.Tensor) else a for a in args]
    cpu = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
    got = getattr(ops, fn_name)(*dev)
    want = getattr(twins, fn_name)(*cpu)
    compare(got, want, dev, cpu)


def _close(a, b, dtype):
    tol = dict(rtol=2e-2, atol=2e-2) if dtype == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), **tol)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,D,T", [(37, 24, 5), (1000, 1032, 70)])
def test_embed_twin(ops, dtype, V, D, T):
    torch.manual_seed(V)
    make = lambda: (torch.randn(V, D).to(dtype), torch.randint(0, V, (T,), dtype=torch.int32), torch.zeros(T, D))
    _both("embed", make, lambda g, w, *_: torch.testing.assert_close(g.cpu(), w), ops)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D,S", [(3, 40, 0), (70, 1032, 0), (5, 520, 3)])
def test_add_rmsnorm_twin(ops, dtype, T, D, S):
    torch.manual_seed(D)
    delta = torch.randn(S, T, D) if S else torch.randn(T, D).to(dtype)
    make = lambda: (torch.randn(T, D), delta, (torch.rand(D) + 0.5).to(dtype), 2e-5, torch.zeros(T, D).to(dtype))

    def compare(got, want, dev, cpu):
        _close(got, want, dtype)
        torch.testing.assert_close(dev[0].cpu(), cpu[0], rtol=1e-6, atol=1e-6)  # the residual stream itself
    _both("add_rmsnorm", make, compare, ops)
    rows = torch.tensor([T - 1, 0], dtype=torch.int32)
    make_rows = lambda: (torch.randn(T, D), None, (torch.rand(D) + 0.5).to(dtype), 2e-5, torch.zeros(2, D).to(dtype), rows)
    _both("add_rmsnorm", make_rows, compare, ops)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rmsnorm_silu_scale_rows_twins(ops, dtype):
    torch.manual_seed(11)
    for T, D in ((5, 48), (33, 1040)):
        _both("rmsnorm", lambda: (torch.randn(T, D).to(dtype), (torch.rand(D) + 0.5).to(dtype), 1e-6),
              lambda g, w, *_: _close(g, w, dtype), ops)
        _both("silu_mul", lambda: (torch.randn(T, 2 * D).to(dtype),), lambda g, w, *_: _close(g, w, dtype), ops)
        _both("scale_rows", lambda: (torch.randn(T, D).to(dtype), torch.rand(T, 7) * D, D, 1e-5),
              lambda g, w, *_: _close(g, w, dtype), ops)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KV,hd,rot,P", [(6, 2, 48, 48, 16), (5, 1, 80, 32, 64)])
def test_rope_kv_write_twin(ops, dtype, H, KV, hd, rot, P):
    torch.manual_seed(hd)
    T = 21
    pos = torch.randint(0, 5000, (T,), dtype=torch.int32)
    slots = torch.randperm(6 * P)[:T].to(torch.int32)
    slots[4] = -1
    freqs = 1.0 / 500000.0 ** (torch.arange(0, rot, 2).float() / rot)
    _both("rope_table", lambda: (pos, freqs), lambda g, w, *_: torch.testing.assert_close(g.cpu(), w, rtol=1e-4, atol=1e-4),
          ops)
    make = lambda: (torch.randn(T, (H + 2 * KV) * hd).to(dtype), pos, freqs, slots, torch.zeros(6, KV, P, hd).to(dtype),
                    torch.zeros(6, KV, hd, P).to(dtype), H, KV, hd, rot)

    def compare(got, want, dev, cpu):
        for i in (0, 4, 5):  # q (and the untouched k, v columns), the K pages, the V pages
            _close(dev[i], cpu[i], dtype)
    _both("rope_kv_write", make, compare, ops)


def _attention_case(dtype, H, KV, hd, P, lens, seed):
    """Pages filled for sequences of ``lens`` keys, a query for the last ``n_q`` positions of each."""
    torch.manual_seed(seed)
    n_pages = sum(-(-n // P) for n, _ in lens) + 3
    order = torch.randperm(n_pages).tolist()
    kp, vp = torch.randn(n_pages, KV, P, hd).to(dtype), torch.randn(n_pages, KV, hd, P).to(dtype)
    bt = torch.zeros(len(lens), max(-(-n // P) for n, _ in lens), dtype=torch.int32)
    seq, posn, items, first = [], [], [], 0
    for b, (n, n_q) in enumerate(lens):
        need = -(-n // P)
        bt[b, :need] = torch.tensor([order.pop() for _ in range(need)], dtype=torch.int32)
        seq += [b] * n_q
        posn += list(range(n - n_q, n))
        items.append((b, first, n_q, n - n_q))
        first += n_q
    T = len(seq)
    q = torch.randn(T, H * hd).to(dtype)
    return q, kp, vp, bt, torch.tensor(seq, dtype=torch.int32), torch.tensor(posn, dtype=torch.int32), items


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,KV,hd,P,window", [(6, 2, 48, 16, 0), (5, 5, 24, 8, 13), (8, 1, 80, 64, 0)])
def test_paged_attention_general_twin(ops, dtype, H, KV, hd, P, window):
    q, kp, vp, bt, seq, posn, _ = _attention_case(dtype, H, KV, hd, P, [(70, 9), (5, 5), (131, 1)], hd)
    make = lambda: (q, torch.zeros(q.shape[0], H * hd).to(dtype), kp, vp, bt, seq, posn, H, 1 / math.sqrt(hd), window)
    _both("paged_attention_general", make, lambda g, w, *_: _close(g, w, dtype), ops)


@gpu
@pytest.mark.parametrize("H,KV,hd,P,window", [(6, 2, 48, 16, 0), (16, 2, 80, 64, 70), (4, 4, 128, 32, 0)])
def test_paged_attention_mfma_twin(ops, H, KV, hd, P, window):
    dtype = torch.bfloat16
    G = H // KV
    lens = [(300, 1), (70, 40), (5, 5), (700, 2 if 2 * G <= 16 else 1), (129, 129)]
    q, kp, vp, bt, seq, posn, items = _attention_case(dtype, H, KV, hd, P, lens, hd + 1)
    small = [it for it in items if it[2] * G <= 16]
    big = []
    per_tile = max(1, ops.attention_tile_rows(hd) // G)
    for b, first, n, pos in items:
        if n * G > 16:
            big += [(b, first + i, min(per_tile, n - i), pos + i) for i in range(0, n, per_tile)]
    out_g = torch.zeros(q.shape[0], H * hd, dtype=dtype, device="cuda")
    both = torch.tensor(small + big, dtype=torch.int32).cuda()
    ops.paged_attention_mfma(q.cuda(), out_g, kp.cuda(), vp.cuda(), bt.cuda(), both[: len(small)], both[len(small):],
                             H, 1 / math.sqrt(hd), window)
    out_c = torch.zeros(q.shape[0], H * hd, dtype=dtype)
    twins.paged_attention_mfma(q, out_c, kp, vp, bt, torch.tensor(small, dtype=torch.int32),
                               torch.tensor(big, dtype=torch.int32), H, 1 / math.sqrt(hd), window)
    _close(out_g, out_c, dtype)


@gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(3, 50, 72), (130, 264, 1032)])
def test_gemm_nt_twin(ops, dtype, M, N, K):
    torch.manual_seed(K)
    make = lambda: ((torch.randn(M, K) / 4).to(dtype), (torch.randn(N, K) / 4).to(dtype))
    _both("gemm_nt", make, lambda g, w, *_: _close(g, w, dtype), ops)


@gpu
@pytest.mark.parametrize("M,N,K", [(1, 48, 72), (7, 528, 1032), (16, 104, 520)])
def test_gemm_skinny_twins(ops, M, N, K):
    torch.manual_seed(N)
    bf = torch.bfloat16
    x, w = (torch.randn(M, K) / 4).to(bf), (torch.randn(N, K) / 4).to(bf)
    _both("gemm_skinny", lambda: (x, w), lambda g, t, *_: _close(g, t, bf), ops)
    _both("gemm_skinny", lambda: (x, w, torch.float32), lambda g, t, *_: _close(g, t, bf), ops)
    if N % 16 == 0:
        _both("gemm_skinny", lambda: (x, w, None, True), lambda g, t, *_: _close(g, t, bf), ops)
    _both("gemm_skinny", lambda: (x, w, None, False, 3), lambda g, t, *_: _close(g.sum(0), t.sum(0), bf), ops)
    # the norm folded into the products around it
    norm_w = (torch.rand(N) + 0.5).to(bf)
    h = torch.randn(M, N)

    def compare(got, want, dev, cpu):
        torch.testing.assert_close(dev[2].cpu(), cpu[2], rtol=1e-4, atol=1e-4)  # the residual stream
        _close(got.rows, want.rows, bf)
        torch.testing.assert_close(got.ssq.cpu().sum(1), want.ssq.sum(1), rtol=1e-4, atol=1e-4)
        torch.testing.assert_close(got.ssq.cpu(), want.ssq, rtol=1e-3, atol=1e-3)
    _both("gemm_skinny_residual", lambda: (x, w, h, norm_w, 1e-5), compare, ops)
    if M <= 16:
        folded_c = twins.gemm_skinny_residual(x, w, h.clone(), norm_w, 1e-5)
        folded_g = kernel_ops.ScaledRows(folded_c.rows.cuda(), folded_c.ssq.cuda(), folded_c.dim, folded_c.eps)
        w2 = (torch.randn(48, N) / 4).to(bf)
        _close(ops.gemm_skinny(folded_g, w2.cuda()), twins.gemm_skinny(folded_c, w2), bf)
        for wide in (False, True):  # the norm's factor in either kernel, with and without the gate/up epilogue
            _close(ops.gemm_skinny(folded_g, w2.cuda(), wide=wide), twins.gemm_skinny(folded_c, w2, wide=wide), bf)
            _close(ops.gemm_skinny(folded_g, w2.cuda(), None, True, 1, wide),
                   twins.gemm_skinny(folded_c, w2, None, True, 1, wide), bf)


@gpu
@pytest.mark.parametrize("M,N,K", [(130, 48, 72), (300, 528, 1032), (70, 272, 520)])
def test_gemm_tiled_twins(ops, M, N, K):
    torch.manual_seed(N)
    bf = torch.bfloat16
    x, w = (torch.randn(M, K) / 4).to(bf), (torch.randn(N, K) / 4).to(bf)
    for tile_rows in kernel_ops.TILED_TILE_ROWS:
        _both("gemm_tiled", lambda: (x, w, None, False, 1, tile_rows), lambda g, t, *_: _close(g, t, bf), ops)
        _both("gemm_tiled", lambda: (x, w, torch.float32, False, 1, tile_rows), lambda g, t, *_: _close(g, t, bf), ops)
        _both("gemm_tiled", lambda: (x, w, None, True, 1, tile_rows), lambda g, t, *_: _close(g, t, bf), ops)
        _both("gemm_tiled", lambda: (x, w, None, False, 3, tile_rows),
              lambda g, t, *_: (_close(g.sum(0), t.sum(0), bf), torch.testing.assert_close(g.cpu(), t, rtol=2e-3, atol=2e-3)), ops)


@gpu
@pytest.mark.parametrize("M,H,KV,hd,rot,P,K", [(5, 6, 2, 48, 48, 16, 72), (16, 5, 1, 80, 32, 64, 520)])
def test_gemm_skinny_qkv_twin(ops, M, H, KV, hd, rot, P, K):
    torch.manual_seed(K)
    bf = torch.bfloat16
    x, w = (torch.randn(M, K) / 4).to(bf), (torch.randn((H + 2 * KV) * hd, K) / 4).to(bf)
    pos = torch.randint(0, 3000, (M,), dtype=torch.int32)
    freqs = 1.0 / 10000.0 ** (torch.arange(0, rot, 2).float() / rot)
    table = twins.rope_table(pos, freqs)
    slots = torch.randperm(4 * P)[:M].to(torch.int32)
    make = lambda: (x, w, table, slots, torch.zeros(4, KV, P, hd).to(bf), torch.zeros(4, KV, hd, P).to(bf), H, KV, hd, rot)

    def compare(got, want, dev, cpu):
        _close(got, want, bf)
        _close(dev[4], cpu[4], bf)
        _close(dev[5], cpu[5], bf)
    _both("gemm_skinny_qkv", make, compare, ops)


@gpu
def test_sample_and_logprob_twins(ops):
    torch.manual_seed(2)
    logits = torch.randn(6, 1003) * 2
    logits[2, 17] = logits[2, 900] = 50.0  # equal maxima: the lowest index
    _both("sample", lambda: (logits,), lambda g, w, *_: torch.testing.assert_close(g.cpu(), w), ops)
    temp = torch.tensor([0.0, 0.8, 0.0, 1.5, 0.0, 0.3])
    top_p = torch.tensor([1.0, 0.5, 1.0, 0.9, 1.0, 0.2])
    seeds, counters = torch.arange(6, dtype=torch.int64) + 5, torch.zeros(6, dtype=torch.int64)
    want = twins.sample(logits, temp, top_p, seeds, counters)
    for c in range(20):
        got = ops.sample(logits.cuda(), temp.cuda(), top_p.cuda(), seeds.cuda(), (counters + c).cuda()).cpu()
        for r in range(6):
            if want[r] >= 0:
                assert got[r] == want[r]
            else:  # a draw: from the set the twin names
                assert twins.sample_support(logits[r], float(temp[r]), float(top_p[r]))[got[r]]
    tokens = torch.randint(0, 1003, (6,), dtype=torch.int32)
    _both("logprob", lambda: (logits, tokens), lambda g, w, *_: torch.testing.assert_close(g.cpu(), w, rtol=1e-5, atol=1e-5),
          ops)
