"""Each HIP kernel alone against its plain reference, at sizes other than the
engine tests' (head sizes in steps of 16, odd numbers of heads and groups,
widths and vocabularies that are no power of two)."""

import math

import pytest
import torch

from plain_llama import (
    plain_attention,
    plain_rmsnorm,
    plain_rope_frequencies,
    plain_rope_interleaved,
    plain_top_p_keep,
)

from fastgen_amd.cache.layout import pack_k, pack_v, unpack_k, unpack_v

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(scope="module")
def ops():
    from fastgen_amd.kernels import ops as _ops

    return _ops


def tol(dtype):
    return dict(atol=1e-5, rtol=1e-5) if dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)


# ------------------------------------------------------------------- rows
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,D,T", [(515, 240, 7), (1000, 4096, 3), (33, 24, 300)])
def test_embed(ops, dtype, V, D, T):
    torch.manual_seed(0)
    table = torch.randn(V, D).to(dtype)
    tok = torch.randint(0, V, (T,), dtype=torch.int32)
    tok[0], tok[-1] = 0, V - 1
    out = torch.empty(T, D, dtype=torch.float32, device=DEV)
    ops.embed(table.to(DEV), tok.to(DEV), out)
    assert torch.equal(out.cpu(), table[tok.long()].float())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("wdtype", DTYPES)
@pytest.mark.parametrize("T,D,eps", [(1, 4096, 1e-5), (5, 240, 3e-6), (300, 72, 1e-2), (3, 8200, 1e-6)])
def test_add_rmsnorm(ops, dtype, wdtype, T, D, eps):
    torch.manual_seed(1)
    h = torch.randn(T, D) * 3
    delta = torch.randn(T, D).to(dtype)
    w = (1 + 0.1 * torch.randn(D)).to(wdtype)
    hd, out = h.to(DEV), torch.empty(T, D, dtype=dtype, device=DEV)
    ops.add_rmsnorm(hd, delta.to(DEV), w.to(DEV), eps, out)
    hsum = h + delta.float()
    assert torch.equal(hd.cpu(), hsum)  # the residual sum is exact fp32
    want = (hsum * torch.rsqrt((hsum * hsum).mean(-1, keepdim=True) + eps) * w.float()).to(dtype)
    assert torch.allclose(out.cpu().float(), want.float(), **tol(dtype))
    # without delta, and gathered rows (h untouched, a row may be named twice)
    rows = torch.tensor([T - 1, 0, T - 1], dtype=torch.int32)
    h2 = h.to(DEV)
    out2 = torch.empty(3, D, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h2, delta.to(DEV), w.to(DEV), eps, out2, rows.to(DEV))
    assert torch.equal(h2.cpu(), h)
    assert torch.allclose(out2.cpu().float(), want[rows.long()].float(), **tol(dtype))
    out3 = torch.empty(T, D, dtype=dtype, device=DEV)
    ops.add_rmsnorm(h2, None, w.to(DEV), eps, out3)
    assert torch.allclose(out3.cpu().float(), plain_rmsnorm(h, w.float(), eps).to(dtype).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_per_head_rows(ops, dtype):
    torch.manual_seed(2)
    x = torch.randn(6, 5, 48).to(dtype)  # a norm over head_dim, applied per head
    w = torch.rand(48).to(dtype)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), 1e-6).cpu()
    assert torch.allclose(got.float(), plain_rmsnorm(x, w, 1e-6).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,F", [(1, 14336), (9, 328), (70, 1000), (3, 8)])
def test_silu_mul(ops, dtype, T, F):
    torch.manual_seed(3)
    g, u = (torch.randn(T, F) * 4).to(dtype), (torch.randn(T, F) * 4).to(dtype)
    # columns in groups of 8: 8 gate values, then the 8 up values of the same channels
    gu = torch.stack([g.view(T, F // 8, 8), u.view(T, F // 8, 8)], dim=2).reshape(T, 2 * F).contiguous()
    got = ops.silu_mul(gu.to(DEV)).cpu()
    want = (g.float() * torch.sigmoid(g.float()) * u.float()).to(dtype)
    assert torch.allclose(got.float(), want.float(), **tol(dtype))
    # the same order for the rows of the weight matrix
    wg, wu = torch.arange(F * 3.0).view(F, 3), -torch.arange(F * 3.0).view(F, 3)
    w = ops.interleave_gate_up(wg, wu)
    assert torch.equal(w[16:24], wg[8:16]) and torch.equal(w[24:32], wu[8:16])


# ------------------------------------------------------------- rope + write
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,rot,P", [(4, 2, 16, 16, 16), (5, 1, 48, 48, 32), (8, 8, 128, 128, 64),
                                           (6, 3, 64, 32, 8), (3, 3, 80, 0, 16)])
@pytest.mark.parametrize("with_table", [False, True])
def test_rope_kv_write(ops, dtype, H, KV, hd, rot, P, with_table):
    torch.manual_seed(4)
    T, n_pages = 37, 9
    width = (H + 2 * KV) * hd
    qkv = torch.randn(T, width).to(dtype)
    pos = torch.randint(0, 5000, (T,), dtype=torch.int32)
    freqs = plain_rope_frequencies(rot, 10000.0) if rot else None
    slots = torch.randperm(n_pages * P)[:T].to(torch.int32)
    slots[5] = -1  # a token whose k, v are not to be written
    kp = torch.full((n_pages, KV, P, hd), 7.0, dtype=dtype)
    vp = torch.full((n_pages, KV, hd, P), 7.0, dtype=dtype)
    qkv_d, kp_d, vp_d = qkv.to(DEV), kp.to(DEV), vp.to(DEV)
    table = None
    if with_table and rot:  # sines and cosines computed once for the step, as the engine does
        table = ops.rope_table(pos.to(DEV), freqs.to(DEV))
        ang = pos.float()[:, None] * freqs[None, :]
        assert torch.allclose(table.cpu(), torch.stack([torch.cos(ang), torch.sin(ang)], -1), atol=1e-6)
    ops.rope_kv_write(qkv_d, pos.to(DEV), None if freqs is None else freqs.to(DEV), slots.to(DEV), kp_d, vp_d,
                      H, KV, hd, rot, table=table)
    q = qkv[:, : H * hd].view(T, H, hd)
    k = qkv[:, H * hd : (H + KV) * hd].view(T, KV, hd)
    v = qkv[:, (H + KV) * hd :].view(T, KV, hd)

    def rotate(x):
        if not rot:
            return x
        out = x.clone()
        out[..., :rot] = plain_rope_interleaved(x[..., :rot], pos, freqs)
        return out

    got = qkv_d.cpu()
    assert torch.allclose(got[:, : H * hd].float(), rotate(q).reshape(T, -1).float(), **tol(dtype))
    assert torch.equal(got[:, (H + KV) * hd :], qkv[:, (H + KV) * hd :])  # v untouched in place
    want_k, want_v = torch.full((n_pages, KV, P, hd), 7.0, dtype=dtype), torch.full((n_pages, KV, P, hd), 7.0, dtype=dtype)
    rk = rotate(k)
    for t in range(T):
        s = int(slots[t])
        if s < 0:
            continue
        want_k[s // P, :, s % P, :] = rk[t]
        want_v[s // P, :, s % P, :] = v[t]
    # the pool in natural order: key p of a page at [p, :], whatever the storage order inside the page
    assert torch.allclose(unpack_k(kp_d.cpu()).float(), want_k.float(), **tol(dtype))
    assert torch.equal(unpack_v(vp_d.cpu()), want_v)  # nothing else in the pool changed either


@pytest.mark.parametrize("M", [1, 7, 16])
@pytest.mark.parametrize("H,KV,hd,rot,P,K", [(4, 2, 16, 16, 16, 64), (5, 1, 48, 48, 32, 240), (8, 2, 128, 128, 64, 1024),
                                             (6, 3, 64, 32, 8, 328), (3, 3, 80, 0, 16, 72)])
def test_gemm_skinny_qkv_rotates_and_writes_the_cache(ops, M, H, KV, hd, rot, P, K):
    """The decode step's fused product: the same result as the product, the
    rotation and the cache write as three steps (plain fp32 arithmetic here)."""
    torch.manual_seed(M + hd)
    n_pages = 5
    x = (torch.randn(M, K) * 0.5).to(torch.bfloat16)
    w = (torch.randn((H + 2 * KV) * hd, K) * K**-0.5).to(torch.bfloat16)
    pos = torch.randint(0, 5000, (M,), dtype=torch.int32)
    freqs = plain_rope_frequencies(rot, 10000.0) if rot else None
    slots = torch.randperm(n_pages * P)[:M].to(torch.int32)
    if M > 2:
        slots[2] = -1
    kp_d = torch.full((n_pages, KV, P, hd), 7.0, dtype=torch.bfloat16, device=DEV)
    vp_d = torch.full((n_pages, KV, hd, P), 7.0, dtype=torch.bfloat16, device=DEV)
    table = ops.rope_table(pos.to(DEV), freqs.to(DEV)) if rot else None
    got_q = ops.gemm_skinny_qkv(x.to(DEV), w.to(DEV), table, slots.to(DEV), kp_d, vp_d, H, KV, hd, rot).cpu()
    qkv = x.float() @ w.float().T
    q = qkv[:, : H * hd].view(M, H, hd)
    k = qkv[:, H * hd : (H + KV) * hd].view(M, KV, hd)
    v = qkv[:, (H + KV) * hd :].view(M, KV, hd)

    def rotate(t):
        if not rot:
            return t
        out = t.clone()
        out[..., :rot] = plain_rope_interleaved(t[..., :rot], pos, freqs)
        return out

    assert torch.allclose(got_q.float(), rotate(q).reshape(M, -1), **tol(torch.bfloat16))
    want_k, want_v = torch.full((n_pages, KV, P, hd), 7.0), torch.full((n_pages, KV, P, hd), 7.0)
    rk = rotate(k)
    for t in range(M):
        s = int(slots[t])
        if s >= 0:
            want_k[s // P, :, s % P, :] = rk[t]
            want_v[s // P, :, s % P, :] = v[t]
    assert torch.allclose(unpack_k(kp_d.cpu()).float(), want_k, **tol(torch.bfloat16))
    assert torch.allclose(unpack_v(vp_d.cpu()).float(), want_v, **tol(torch.bfloat16))


# ---------------------------------------------------------------- attention
def _paged_case(dtype, seqs, H, KV, hd, P, seed, poison=True, peak=None):
    """``seqs``: list of (n_cached, n_new).  Returns device operands and the
    per-sequence whole q, k, v on the CPU."""
    g = torch.Generator().manual_seed(seed)
    B = len(seqs)
    pages_of = [-(-(a + b) // P) for a, b in seqs]
    n_pages = sum(pages_of) + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    fill = float("nan") if poison else 0.0
    kp = torch.full((n_pages, KV, P, hd), fill, dtype=dtype)
    vp = torch.full((n_pages, KV, hd, P), fill, dtype=dtype)
    table = torch.zeros(B, max(pages_of), dtype=torch.int32)
    qs, ks, vs, q_rows, seq_of, posv = [], [], [], [], [], []
    for b, (n0, n1) in enumerate(seqs):
        n = n0 + n1
        q = torch.randn(n, H, hd, generator=g).to(dtype)
        k = torch.randn(n, KV, hd, generator=g).to(dtype)
        v = torch.randn(n, KV, hd, generator=g).to(dtype)
        if peak is not None and b == peak[0]:
            _, qpos, qh, kpos = peak  # one score made to stand out
            k[kpos, qh // (H // KV)] = 0
            k[kpos, qh // (H // KV), 0] = 12.0
            q[qpos, qh] = 0
            q[qpos, qh, 0] = 12.0 * math.sqrt(hd)
        pages = [perm.pop() for _ in range(pages_of[b])]
        table[b, : len(pages)] = torch.tensor(pages, dtype=torch.int32)
        for j, pg in enumerate(pages):  # natural [KV, P, hd] per page, then into storage order
            nk = torch.full((KV, P, hd), fill, dtype=dtype)
            nv = torch.full((KV, P, hd), fill, dtype=dtype)
            cnt = min(P, n - j * P)
            nk[:, :cnt] = k[j * P : j * P + cnt].transpose(0, 1)
            nv[:, :cnt] = v[j * P : j * P + cnt].transpose(0, 1)
            kp[pg], vp[pg] = pack_k(nk), pack_v(nv)
        qs.append(q), ks.append(k), vs.append(v)
        q_rows.append(q[n0:].reshape(n1, H * hd))
        seq_of += [b] * n1
        posv += list(range(n0, n))
    q_flat = torch.cat(q_rows)
    dev = lambda t: t.to(DEV)
    return dict(
        q=dev(q_flat), kp=dev(kp), vp=dev(vp), table=dev(table),
        seq_of=dev(torch.tensor(seq_of, dtype=torch.int32)), pos=dev(torch.tensor(posv, dtype=torch.int32)),
        whole=(qs, ks, vs),
    )


def _plain_rows(case, seqs, window=None):
    qs, ks, vs = case["whole"]
    out = []
    for (n0, n1), q, k, v in zip(seqs, qs, ks, vs):
        o = plain_attention(q.float(), k.float(), v.float(), window)
        out.append(o[n0:].reshape(n1, -1))
    return torch.cat(out)


ATT_SHAPES = [
    # H, KV, hd, P
    (4, 2, 16, 16),
    (5, 1, 48, 32),
    (6, 3, 32, 8),
    (8, 2, 128, 64),
    (3, 3, 80, 128),
    (16, 2, 64, 16),
    (2, 1, 256, 32),
]
ATT_SEQS = [(0, 1), (0, 70), (131, 1), (60, 9), (17, 2), (255, 1), (0, 129)]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,KV,hd,P", ATT_SHAPES)
@pytest.mark.parametrize("window", [0, 37])
def test_paged_attention_general(ops, dtype, H, KV, hd, P, window):
    case = _paged_case(dtype, ATT_SEQS, H, KV, hd, P, seed=5)
    out = torch.empty_like(case["q"])
    ops.paged_attention_general(case["q"], out, case["kp"], case["vp"], case["table"], case["seq_of"],
                                case["pos"], H, hd**-0.5, window)
    want = _plain_rows(case, ATT_SEQS, window or None)
    assert torch.isfinite(out).all()  # poison in unwritten slots never reaches the output
    assert torch.allclose(out.cpu().float(), want, **(dict(atol=2e-5, rtol=1e-5) if dtype == torch.float32
                                                       else dict(atol=1.5e-2, rtol=2e-2)))


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_far_key_stands_out(ops, dtype):
    """One key among hundreds, in an early page, gets nearly all the weight:
    the output is that key's value, which a kernel that drops a page, a tile
    or a tile's edge would miss."""
    H, KV, hd, P = 4, 2, 64, 16
    for kpos in (0, 15, 16, 63, 64, 300):
        seqs = [(0, 3), (400, 1), (10, 2)]
        case = _paged_case(dtype, seqs, H, KV, hd, P, seed=6, peak=(1, 400, 3, kpos))
        out = torch.empty_like(case["q"])
        ops.paged_attention_general(case["q"], out, case["kp"], case["vp"], case["table"], case["seq_of"],
                                    case["pos"], H, hd**-0.5, 0)
        v = case["whole"][2][1]
        got = out.cpu().float()[3].view(H, hd)[3]
        assert torch.allclose(got, v[kpos, 1].float(), atol=2e-2), kpos


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_window_edge(ops, dtype):
    """The key just outside the window is made to stand out and must not be
    seen; the key just inside must."""
    H, KV, hd, P, w = 2, 1, 32, 16, 40
    for kpos, seen in ((100 - w, False), (100 - w + 1, True)):
        seqs = [(100, 1)]
        case = _paged_case(dtype, seqs, H, KV, hd, P, seed=7, peak=(0, 100, 1, kpos))
        out = torch.empty_like(case["q"])
        ops.paged_attention_general(case["q"], out, case["kp"], case["vp"], case["table"], case["seq_of"],
                                    case["pos"], H, hd**-0.5, w)
        v = case["whole"][2][0]
        got = out.cpu().float()[0].view(H, hd)[1]
        assert torch.allclose(got, v[kpos, 0].float(), atol=2e-2) == seen
        assert torch.allclose(out.cpu().float(), _plain_rows(case, seqs, w), atol=2e-2)


# --------------------------------------------------------------------- gemm
@pytest.mark.parametrize("dtype,odtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                          (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(1, 515, 240), (7, 64, 64), (65, 130, 17), (300, 33, 1000), (2, 4096, 328)])
def test_gemm_nt(ops, dtype, odtype, M, N, K):
    torch.manual_seed(8)
    x, w = torch.randn(M, K).to(dtype), torch.randn(N, K).to(dtype)
    got = ops.gemm_nt(x.to(DEV), w.to(DEV), out_dtype=odtype).cpu()
    want = (x.double() @ w.double().T)
    assert got.dtype == odtype
    err = (got.double() - want).abs().max() / want.abs().max()
    assert err < (2e-6 if odtype == torch.float32 else 1e-2)


def test_gemm_rows_do_not_depend_on_the_batch(ops):
    torch.manual_seed(9)
    x, w = torch.randn(70, 333), torch.randn(129, 333)
    full = ops.gemm_nt(x.to(DEV), w.to(DEV)).cpu()
    for rows in ([0], [69], list(range(3, 68))):
        part = ops.gemm_nt(x[rows].to(DEV), w.to(DEV)).cpu()
        assert torch.equal(part, full[rows])  # bit for bit


@pytest.mark.parametrize("M", [1, 2, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(515, 240), (4096, 4096), (6144, 64), (48, 8), (1000, 14336), (16, 328)])
@pytest.mark.parametrize("odtype", [torch.bfloat16, torch.float32])
def test_gemm_skinny(ops, M, N, K, odtype):
    torch.manual_seed(14)
    x, w = torch.randn(M, K).bfloat16(), (torch.randn(N, K) * 0.1).bfloat16()
    got = ops.gemm_skinny(x.to(DEV), w.to(DEV), out_dtype=odtype).cpu()
    want = x.double() @ w.double().T
    assert got.dtype == odtype and got.shape == (M, N)
    err = (got.double() - want).abs().max() / want.abs().max()
    assert err < (1e-5 if odtype == torch.float32 else 6e-3), float(err)


@pytest.mark.parametrize("M", [1, 8, 17, 40, 64, 65, 83, 128])
@pytest.mark.parametrize("N,K,S", [(515, 240, 1), (4096, 4096, 4), (4096, 14336, 8), (100, 264, 3), (6144, 64, 1)])
def test_gemm_skinny_wide_and_k_splits(ops, M, N, K, S):
    torch.manual_seed(17)
    x, w = torch.randn(M, K).bfloat16(), (torch.randn(N, K) * 0.1).bfloat16()
    got = ops.gemm_skinny(x.to(DEV), w.to(DEV), k_splits=S, wide=True)
    want = x.double() @ w.double().T
    if S > 1:
        assert got.dtype == torch.float32 and got.shape == (S, M, N)
        total = got.cpu().double().sum(0)
        assert (total - want).abs().max() / want.abs().max() < 1e-5
        # the norm that follows adds the partial sums itself
        h = torch.randn(M, N)
        wn = 1 + 0.1 * torch.randn(N)
        hd, out = h.to(DEV), torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
        ops.add_rmsnorm(hd, got, wn.to(DEV), 1e-5, out)
        hs = h + got.cpu().sum(0)
        assert torch.allclose(hd.cpu(), hs, atol=1e-4 * float(hs.abs().max()))
        ref = (hs * torch.rsqrt((hs * hs).mean(-1, keepdim=True) + 1e-5) * wn).bfloat16()
        assert torch.allclose(out.cpu().float(), ref.float(), atol=2e-2, rtol=2e-2)
    else:
        assert got.dtype == torch.bfloat16 and got.shape == (M, N)
        assert (got.cpu().double() - want).abs().max() / want.abs().max() < 6e-3


@pytest.mark.parametrize("M", [17, 64, 65, 80, 128])
def test_gemm_skinny_wide_gate_up(ops, M):
    torch.manual_seed(18)
    F, K = 1000, 328
    x = torch.randn(M, K).bfloat16()
    wg, wu = (torch.randn(F, K) * 0.05).bfloat16(), (torch.randn(F, K) * 0.05).bfloat16()
    got = ops.gemm_skinny(x.to(DEV), ops.interleave_gate_up(wg, wu).contiguous().to(DEV), silu_mul_epilogue=True).cpu()
    g, u = x.float() @ wg.float().T, x.float() @ wu.float().T
    want = g * torch.sigmoid(g) * u
    assert got.shape == (M, F) and (got.float() - want).abs().max() <= 1e-2 * want.abs().max() + 1e-3


@pytest.mark.parametrize("tile_rows", [128, 256])
@pytest.mark.parametrize("M,N,K,S", [(129, 515, 240, 1), (192, 4096, 4096, 8), (256, 4096, 14336, 16), (1, 16, 8, 1),
                                     (300, 100, 264, 3), (2048, 256, 1000, 2), (65, 6144, 64, 2)])
def test_gemm_tiled_and_k_splits(ops, tile_rows, M, N, K, S):
    """The tiled product (both operands through a ring of LDS stages) at both tile shapes: sizes that are no
    multiple of a tile, of a stage (32 k) or of anything but 8; one row; k splits whose ranges are not equal;
    each split's partial sums against the product over its own k range."""
    torch.manual_seed(M + N)
    x = torch.randn(M, K).bfloat16()
    w = (torch.randn(N, K) * K**-0.5).bfloat16()
    want = x.double() @ w.double().T
    got = ops.gemm_tiled(x.to(DEV), w.to(DEV), k_splits=S, tile_rows=tile_rows)
    if S > 1:
        assert got.dtype == torch.float32 and got.shape == (S, M, N)
        step = -(-K // (S * 32)) * 32
        for s in range(S):
            part = x[:, s * step:(s + 1) * step].double() @ w[:, s * step:(s + 1) * step].double().T
            assert (got[s].cpu().double() - part).abs().max() <= 1e-4 * want.abs().max() + 1e-6
        got = got.sum(0)
    else:
        assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    assert (got.cpu().double() - want).abs().max() <= (1e-4 if S > 1 else 1e-2) * want.abs().max() + 1e-6
    y32 = ops.gemm_tiled(x.to(DEV), w.to(DEV), torch.float32, tile_rows=tile_rows)
    assert y32.dtype == torch.float32 and (y32.cpu().double() - want).abs().max() <= 1e-4 * want.abs().max() + 1e-6
    # the weight packed in the kernels' blocks: the same bits
    pw = ops.pack_weight(w.to(DEV))
    assert torch.equal(ops.gemm_tiled(x.to(DEV), pw, torch.float32, tile_rows=tile_rows), y32)
    assert torch.equal(ops.gemm_tiled(x.to(DEV), pw, k_splits=S, tile_rows=tile_rows),
                       ops.gemm_tiled(x.to(DEV), w.to(DEV), k_splits=S, tile_rows=tile_rows))


@pytest.mark.parametrize("M,F,K", [(129, 328, 240), (256, 14336, 4096), (70, 8, 64)])
def test_gemm_tiled_gate_up_epilogue(ops, M, F, K):
    torch.manual_seed(F)
    x = torch.randn(M, K).bfloat16()
    wg, wu = (torch.randn(F, K) * 0.05).bfloat16(), (torch.randn(F, K) * 0.05).bfloat16()
    w = ops.interleave_gate_up(wg, wu).contiguous().to(DEV)
    g, u = x.float() @ wg.float().T, x.float() @ wu.float().T
    want = g * torch.sigmoid(g) * u
    for tile_rows in (128, 256):
        got = ops.gemm_tiled(x.to(DEV), w, silu_mul_epilogue=True, tile_rows=tile_rows).cpu().float()
        assert got.shape == (M, F) and (got - want).abs().max() <= 1.5e-2 * want.abs().max() + 1e-3


def test_gemm_skinny_takes_views_and_refuses_the_rest(ops):
    from fastgen_amd.kernels import KernelArgumentError

    torch.manual_seed(15)
    big = torch.randn(8, 3 * 256).bfloat16().to(DEV)
    w = torch.randn(40, 256).bfloat16().to(DEV)
    x = big[:, 256:512]  # a column slice: row stride 768
    got = ops.gemm_skinny(x, w).cpu().float()
    assert torch.allclose(got, x.cpu().float() @ w.cpu().float().T, atol=0.3, rtol=2e-2)
    with pytest.raises(KernelArgumentError, match="rows"):
        ops.gemm_skinny(torch.zeros(129, 64, dtype=torch.bfloat16, device=DEV), w[:, :64].contiguous())
    with pytest.raises(KernelArgumentError, match="wide"):
        ops.gemm_skinny(torch.zeros(65, 64, dtype=torch.bfloat16, device=DEV), w[:, :64].contiguous(), wide=False)
    with pytest.raises(KernelArgumentError, match="multiple of 8"):
        ops.gemm_skinny(torch.zeros(4, 12, dtype=torch.bfloat16, device=DEV),
                        torch.zeros(8, 12, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("M", [1, 3, 16, 17, 40, 64, 100, 128])
@pytest.mark.parametrize("N,K", [(515, 240), (4096, 4096), (48, 8), (1008, 14336), (16, 328), (200, 72)])
def test_streaming_products_read_a_packed_weight(ops, M, N, K):
    """The weight in the order of the kernels' reads (``pack_weight``: blocks of 16 rows x 32 k, padded with
    zeros) instead of row by row: only where a lane finds its bytes differs, so every product gives the same
    bits.  Sizes that are no multiples of the blocks; every entry point that streams a weight."""
    torch.manual_seed(M + N + K)
    x = torch.randn(M, K).bfloat16().to(DEV)
    w = (torch.randn(N, K) * K**-0.5).bfloat16().to(DEV)
    pw = ops.pack_weight(w)
    assert pw.data.shape == (-(-N // 16), -(-K // 32), 64, 8) and torch.equal(ops.unpack_weight(pw), w)
    both = lambda fn: (fn(w), fn(pw))
    if M <= 64:
        for odtype in (torch.bfloat16, torch.float32):
            a, b = both(lambda m: ops.gemm_skinny(x, m, out_dtype=odtype, wide=False))
            assert torch.equal(a, b)
        want = x.double() @ w.double().T
        assert (b.double() - want).abs().max() / want.abs().max() < 1e-5
    a, b = both(lambda m: ops.gemm_skinny(x, m, wide=True))
    assert torch.equal(a, b)
    for S in (2, 5):
        a, b = both(lambda m: ops.gemm_skinny(x, m, k_splits=S, wide=True))
        assert torch.equal(a, b)
    if N % 16 == 0:
        for wide in ([False] if M <= 64 else []) + [True]:
            a, b = both(lambda m: ops.gemm_skinny(x, m, silu_mul_epilogue=True, wide=wide))
            assert torch.equal(a, b)
    if M <= 16:
        nw = (1 + 0.1 * torch.randn(N)).to(DEV)
        h0 = torch.randn(M, N, device=DEV)
        ha, hb = h0.clone(), h0.clone()
        sa, sb = ops.gemm_skinny_residual(x, w, ha, nw, 1e-5), ops.gemm_skinny_residual(x, pw, hb, nw, 1e-5)
        assert torch.equal(ha, hb) and torch.equal(sa.rows, sb.rows) and torch.equal(sa.ssq, sb.ssq)
        # a consumer of rows whose norm is still open (K of the next product = this N)
        if N % 8 == 0:
            w2 = (torch.randn(104, N) * N**-0.5).bfloat16().to(DEV)
            pw2 = ops.pack_weight(w2)
            for wide in (False, True):
                assert torch.equal(ops.gemm_skinny(sa, w2, wide=wide), ops.gemm_skinny(sa, pw2, wide=wide))
        # the first rows of a packed matrix, as an entry that reads another's cache takes its queries' rows
        if N > 32:
            assert torch.equal(ops.gemm_skinny(x, w[:32], wide=False), ops.gemm_skinny(x, pw.first_rows(32), wide=False))


@pytest.mark.parametrize("M", [1, 7, 16])
def test_gemm_skinny_qkv_reads_a_packed_weight(ops, M):
    H, KV, hd, rot, P, K = 5, 1, 48, 48, 32, 240
    torch.manual_seed(M)
    x = (torch.randn(M, K) * 0.5).bfloat16().to(DEV)
    w = (torch.randn((H + 2 * KV) * hd, K) * K**-0.5).bfloat16().to(DEV)
    pos = torch.randint(0, 5000, (M,), dtype=torch.int32, device=DEV)
    table = ops.rope_table(pos, plain_rope_frequencies(rot, 10000.0).to(DEV))
    slots = torch.randperm(5 * P)[:M].to(torch.int32).to(DEV)
    got = []
    for m in (w, ops.pack_weight(w)):
        kp = torch.full((5, KV, P, hd), 7.0, dtype=torch.bfloat16, device=DEV)
        vp = torch.full((5, KV, hd, P), 7.0, dtype=torch.bfloat16, device=DEV)
        got.append((ops.gemm_skinny_qkv(x, m, table, slots, kp, vp, H, KV, hd, rot), kp, vp))
    for a, b in zip(*got):
        assert torch.equal(a, b)


@pytest.mark.parametrize("M", [1, 8, 40])
@pytest.mark.parametrize("F,K", [(328, 240), (14336, 4096), (8, 64)])
def test_gemm_skinny_gate_up_epilogue(ops, M, F, K):
    torch.manual_seed(16)
    x = torch.randn(M, K).bfloat16()
    wg, wu = (torch.randn(F, K) * 0.05).bfloat16(), (torch.randn(F, K) * 0.05).bfloat16()
    w = ops.interleave_gate_up(wg, wu).contiguous().to(DEV)
    got = ops.gemm_skinny(x.to(DEV), w, silu_mul_epilogue=True).cpu().float()
    g, u = x.float() @ wg.float().T, x.float() @ wu.float().T
    want = g * torch.sigmoid(g) * u
    assert got.shape == (M, F)
    assert (got - want).abs().max() <= 1e-2 * want.abs().max() + 1e-3


@pytest.mark.parametrize("M", [1, 2, 8, 11, 16])
@pytest.mark.parametrize("N,K,F", [(240, 328, 200), (4096, 14336, 1000), (104, 64, 24), (520, 240, 328)])
@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
def test_norms_folded_into_the_products(ops, M, N, K, F, w_dtype):
    """For few rows: ``h += x W^T`` with what the RMSNorm after it needs made in the same kernel
    (h times the norm's weight, sums of squares per workgroup), and the products that take such
    rows and scale their results: plain store, the gate/up product, and a second residual product;
    each against the plain formulas ``h + x W^T`` and ``rmsnorm(h) W2^T``."""
    torch.manual_seed(M + N)
    eps = 1e-5
    x = torch.randn(M, K).bfloat16()
    w = (torch.randn(N, K) * K**-0.5).bfloat16()
    h = torch.randn(M, N) * 3
    nw = (1 + 0.2 * torch.randn(N)).to(w_dtype)
    h_d = h.to(DEV)
    sr = ops.gemm_skinny_residual(x.to(DEV), w.to(DEV), h_d, nw.to(DEV), eps)
    h_new = h.double() + x.double() @ w.double().T
    assert torch.allclose(h_d.cpu().double(), h_new, atol=1e-4 * float(h_new.abs().max()))
    assert sr.rows.shape == (M, N) and sr.ssq.shape == (M, -(-N // 16)) and sr.dim == N
    assert torch.allclose(sr.ssq.cpu().double().sum(1), (h_new * h_new).sum(1), rtol=1e-5)
    normed = plain_rmsnorm(h_new.float(), nw.float(), eps)  # what the norm's own kernel would hand on
    got = sr.materialize().cpu().float()
    assert torch.allclose(got, normed, atol=2e-2 * float(normed.abs().max()), rtol=2e-2)
    # consumers: a plain product, the gate/up product, a residual product on scaled rows
    w2 = (torch.randn(F, N) * N**-0.5).bfloat16()
    y = ops.gemm_skinny(sr, w2.to(DEV)).cpu().float()
    want = normed @ w2.float().T
    assert (y - want).abs().max() <= 1.5e-2 * want.abs().max() + 1e-3
    if F % 8 == 0:
        wg, wu = (torch.randn(F, N) * N**-0.5).bfloat16(), (torch.randn(F, N) * N**-0.5).bfloat16()
        act = ops.gemm_skinny(sr, ops.interleave_gate_up(wg, wu).contiguous().to(DEV), silu_mul_epilogue=True).cpu().float()
        g, u = normed @ wg.float().T, normed @ wu.float().T
        want = g * torch.sigmoid(g) * u
        assert (act - want).abs().max() <= 1.5e-2 * want.abs().max() + 1e-3
    # the same consumers through the wide kernel (64 columns a workgroup), which takes such rows too
    y = ops.gemm_skinny(sr, w2.to(DEV), wide=True).cpu().float()
    assert (y - normed @ w2.float().T).abs().max() <= 1.5e-2 * (normed @ w2.float().T).abs().max() + 1e-3
    if F % 8 == 0:
        act = ops.gemm_skinny(sr, ops.interleave_gate_up(wg, wu).contiguous().to(DEV), silu_mul_epilogue=True,
                              wide=True).cpu().float()
        assert (act - want).abs().max() <= 1.5e-2 * want.abs().max() + 1e-3
    h2 = torch.randn(M, F)
    h2_d = h2.to(DEV)
    nw2 = 1 + 0.1 * torch.randn(F)
    sr2 = ops.gemm_skinny_residual(sr, w2.to(DEV), h2_d, nw2.to(DEV), eps)
    want_h2 = h2 + normed @ w2.float().T
    assert torch.allclose(h2_d.cpu(), want_h2, atol=1.5e-2 * float(want_h2.abs().max()))
    assert sr2.ssq.shape == (M, -(-F // 16))


@pytest.mark.parametrize("M", [1, 8, 9, 16, 17, 64, 200])
def test_logits_product_at_a_whole_vocabulary(ops, M):
    """``linear(x, w, out_dtype=float32)`` as the head calls it, at the size of a real vocabulary (128,256 rows
    of 4,096): every kernel that takes it, by the number of rows, against a float64 product of the same bfloat16
    operands."""
    from fastgen_amd.kernels.linear import linear

    torch.manual_seed(M)
    N, K = 128256, 4096
    x = torch.randn(M, K).bfloat16().to(DEV)
    w = (torch.randn(N, K, device=DEV) * K**-0.5).bfloat16()
    y = linear(x, w, out_dtype=torch.float32)
    assert y.dtype == torch.float32 and y.shape == (M, N)
    want = x.double() @ w.double().T
    assert float((y.double() - want).abs().max()) <= 1e-4 * float(want.abs().max())


@pytest.mark.parametrize("M", [1, 5, 16])
def test_gemm_skinny_qkv_on_rows_with_a_norm_to_finish(ops, M):
    """The q/k/v product on rows that still lack their division by the root mean square: the same
    queries and cache contents as on the normed rows."""
    H, KV, hd, P, K = 6, 2, 32, 16, 200
    torch.manual_seed(M)
    x = (torch.randn(M, K) * 2).bfloat16()
    ssq = torch.rand(M, 13) * 50
    eps = 1e-6
    w = (torch.randn((H + 2 * KV) * hd, K) * K**-0.5).to(torch.bfloat16)
    pos = torch.randint(0, 300, (M,), dtype=torch.int32)
    freqs = plain_rope_frequencies(hd, 10000.0)
    slots = torch.randperm(4 * P)[:M].to(torch.int32)
    table = ops.rope_table(pos.to(DEV), freqs.to(DEV))
    pools = [[torch.zeros((4, KV, P, hd), dtype=torch.bfloat16, device=DEV),
              torch.zeros((4, KV, hd, P), dtype=torch.bfloat16, device=DEV)] for _ in range(2)]
    sr = ops.ScaledRows(x.to(DEV), ssq.to(DEV), K, eps)
    q1 = ops.gemm_skinny_qkv(sr, w.to(DEV), table, slots.to(DEV), *pools[0], H, KV, hd, hd).cpu().float()
    rstd = torch.rsqrt(ssq.sum(1, keepdim=True) / K + eps)
    # the reference: the rows scaled in fp32 (the kernel scales the sums, which is the same product)
    qkv = (x.float() * rstd) @ w.float().T
    q = plain_rope_interleaved(qkv[:, : H * hd].view(M, H, hd), pos, freqs).reshape(M, -1)
    assert torch.allclose(q1, q, **tol(torch.bfloat16))
    k = plain_rope_interleaved(qkv[:, H * hd : (H + KV) * hd].view(M, KV, hd), pos, freqs)
    v = qkv[:, (H + KV) * hd :].view(M, KV, hd)
    got_k, got_v = unpack_k(pools[0][0].cpu()).float(), unpack_v(pools[0][1].cpu()).float()
    for t in range(M):
        s = int(slots[t])
        assert torch.allclose(got_k[s // P, :, s % P], k[t], **tol(torch.bfloat16))
        assert torch.allclose(got_v[s // P, :, s % P], v[t], **tol(torch.bfloat16))


# ----------------------------------------------------------------- sampling
def test_argmax_lowest_index_wins(ops):
    torch.manual_seed(10)
    logits = torch.randn(5, 128256)
    logits[0, 77] = logits[0, 100000] = 50.0
    logits[1, -1] = 60.0
    logits[2, 0] = 60.0
    got = ops.sample(logits.to(DEV)).cpu()
    assert got.tolist() == [77, 128255, 0, int(logits[3].argmax()), int(logits[4].argmax())]


def test_sampling_follows_the_distribution(ops):
    V, n = 37, 20000
    torch.manual_seed(11)
    row = torch.randn(V) * 2
    temp = 0.8
    logits = row[None].expand(n, V).contiguous().to(DEV)
    t = torch.full((n,), temp, device=DEV)
    seeds = torch.full((n,), 1234, dtype=torch.int64, device=DEV)
    counters = torch.arange(n, dtype=torch.int64, device=DEV)
    got = ops.sample(logits, t, None, seeds, counters).cpu()
    probs = torch.softmax(row / temp, -1)
    counts = torch.bincount(got.long(), minlength=V).float()
    chi2 = ((counts - n * probs) ** 2 / (n * probs)).sum()
    assert chi2 < 80, chi2  # 36 degrees of freedom: 80 is beyond the 99.99th percentile
    # the same (seed, counter) gives the same token whatever else is in the batch
    again = ops.sample(logits[100:103].contiguous(), t[:3], None, seeds[:3], counters[100:103].contiguous()).cpu()
    assert torch.equal(again, got[100:103])
    # temperature 0 rows are greedy inside a sampling batch
    t2 = t.clone()
    t2[:5] = 0
    assert (ops.sample(logits, t2, None, seeds, counters).cpu()[:5] == int(row.argmax())).all()


def test_top_p_keeps_the_reference_set(ops):
    V, n = 515, 4000
    torch.manual_seed(12)
    row = torch.randn(V) * 3
    for p in (0.3, 0.9):
        probs = torch.softmax(row, -1)
        keep = plain_top_p_keep(probs[None], p)[0]
        logits = row[None].expand(n, V).contiguous().to(DEV)
        got = ops.sample(logits, torch.ones(n, device=DEV), torch.full((n,), p, device=DEV),
                         torch.full((n,), 7, dtype=torch.int64, device=DEV),
                         torch.arange(n, dtype=torch.int64, device=DEV)).cpu().long()
        assert keep[got].all()  # never a dropped token
        seen = torch.zeros(V, dtype=torch.bool)
        seen[got] = True
        likely = keep & (probs * n > 20)
        assert seen[likely].all()  # every kept token that should show up does


@pytest.mark.parametrize("p", [0.04, 0.3, 0.9])
def test_top_p_draws_follow_the_kept_distribution(ops, p):
    """The draws are distributed as the kept tokens' probabilities, renormalised
    (the reference draws with multinomial from the un-renormalised rest).  The
    smallest p makes most first draws miss the kept set, so that the exact
    search for the kept set's edge is taken as well."""
    V, n = 1031, 30000
    torch.manual_seed(14)
    row = torch.randn(V) * 2
    probs = torch.softmax(row / 0.9, -1)
    keep = plain_top_p_keep(probs[None], p)[0]
    logits = row[None].expand(n, V).contiguous().to(DEV)
    got = ops.sample(logits, torch.full((n,), 0.9, device=DEV), torch.full((n,), p, device=DEV),
                     torch.full((n,), 99, dtype=torch.int64, device=DEV),
                     torch.arange(n, dtype=torch.int64, device=DEV)).cpu().long()
    assert keep[got].all()
    want = probs * keep / (probs * keep).sum()
    counts = torch.bincount(got, minlength=V).float()
    big = n * want >= 10  # cells with enough expected draws; the others as one cell
    obs = torch.cat([counts[big], counts[~big].sum()[None]])
    exp = torch.cat([n * want[big], (n * want[~big]).sum()[None]])
    ok = exp > 0
    chi2 = float(((obs[ok] - exp[ok]) ** 2 / exp[ok]).sum())
    dof = int(ok.sum()) - 1
    assert chi2 < dof + 6 * math.sqrt(2 * max(dof, 1)) + 10, (chi2, dof)


def test_logprob(ops):
    torch.manual_seed(13)
    logits = torch.randn(4, 1000) * 5
    tok = torch.tensor([0, 999, 5, 17], dtype=torch.int32)
    got = ops.logprob(logits.to(DEV), tok.to(DEV)).cpu()
    want = torch.log_softmax(logits, -1)[torch.arange(4), tok.long()]
    assert torch.allclose(got, want, atol=1e-5)


# ------------------------------------------------------------ refused sizes
def test_kernels_refuse_what_they_cannot_take(ops):
    from fastgen_amd.kernels import KernelArgumentError

    q = torch.zeros(1, 2 * 20, device=DEV)
    kp = torch.zeros(2, 1, 16, 20, device=DEV)
    vp = torch.zeros(2, 1, 20, 16, device=DEV)
    i = torch.zeros(1, dtype=torch.int32, device=DEV)
    with pytest.raises(KernelArgumentError, match="head size"):
        ops.paged_attention_general(q, torch.empty_like(q), kp, vp, i.view(1, 1), i, i, 2, 1.0)
    with pytest.raises(KernelArgumentError, match="GPU only"):
        ops.silu_mul(torch.zeros(2, 4))


# ------------------------------------------------------- attention on MFMA
# how the split kernel's key ranges are cut: (max_chunks, min_tiles); max_chunks None: the engine's
# choice, "least": twice the items (the fewest chunks), a large number with min_tiles 1: one tile a chunk
CUTS = {"auto": (None, 4), "coarse": ("least", 4), "fine": (4096, 1), "pairs": (4096, 2)}


def _run_mfma(ops, case, seqs, H, KV, window=0, cut="auto", max_rows=16, small_tiles=False):
    import numpy as np

    q_lens = [b for _, b in seqs]
    q_start = np.concatenate([[0], np.cumsum(q_lens)])
    tile_rows = ops.attention_tile_rows(case["kp"].shape[3], small_tiles)
    small, big = ops.attention_items(q_lens, q_start, [a for a, _ in seqs], H // KV, tile_rows)
    dev = lambda a: torch.from_numpy(a.reshape(-1)).to(DEV) if a.size else None
    out = torch.full_like(case["q"], float("nan"))
    max_chunks, min_tiles = CUTS[cut]
    if max_chunks == "least":
        max_chunks = 2 * len(small)
    ops.paged_attention_mfma(case["q"], out, case["kp"], case["vp"], case["table"], dev(small), dev(big), H,
                             case["kp"].shape[3] ** -0.5, window, None, max_chunks, min_tiles, max_rows, tile_rows)
    return out, len(small), len(big)


MFMA_SHAPES = [
    # H, KV, hd, P
    (4, 2, 16, 16),
    (5, 1, 48, 32),
    (6, 3, 32, 8),
    (32, 8, 128, 64),
    (3, 3, 80, 128),
    (16, 1, 64, 16),
    (2, 1, 256, 32),
    (7, 7, 112, 24),
]
MFMA_SEQS = [(0, 1), (0, 70), (131, 1), (60, 9), (17, 2), (255, 1), (0, 129), (300, 3), (63, 66)]


@pytest.mark.parametrize("H,KV,hd,P", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 37, 150])
@pytest.mark.parametrize("cut", ["coarse", "fine", "small tiles"])
def test_paged_attention_mfma(ops, H, KV, hd, P, window, cut):
    """``small tiles``: the prompt portions as items of 64 rows (the tile kernel's lighter form, which head sizes
    above 128 always take) instead of 128."""
    case = _paged_case(torch.bfloat16, MFMA_SEQS, H, KV, hd, P, seed=21)
    small_tiles = cut == "small tiles"
    out, n_small, n_big = _run_mfma(ops, case, MFMA_SEQS, H, KV, window, "coarse" if small_tiles else cut,
                                    small_tiles=small_tiles)
    assert n_small and n_big  # both kernels run
    want = _plain_rows(case, MFMA_SEQS, window or None)
    assert torch.isfinite(out).all()  # every row written, no poison read
    assert torch.allclose(out.cpu().float(), want, atol=1.5e-2, rtol=2e-2)


def test_paged_attention_mfma_two_streams(ops, monkeypatch):
    """Prompt portions beside decoded tokens: the tile kernel runs on a second stream beside the
    split kernel.  The result is there when the caller's stream goes on (work queued behind the
    call, on a stream that is not the default one, sees every row), equals the one-stream result
    bit for bit, and a call while a graph is captured stays on the capturing stream."""
    import numpy as np

    H, KV, hd, P = 32, 8, 128, 64
    seqs = [(900, 1), (0, 700), (2000, 1), (300, 260), (64, 1)]
    case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=26)
    q_lens = [b for _, b in seqs]
    small, big = ops.attention_items(q_lens, np.concatenate([[0], np.cumsum(q_lens)]), [a for a, _ in seqs], H // KV,
                                     ops.attention_tile_rows(hd))
    assert small.size and big.size
    small, big = (torch.from_numpy(a.reshape(-1)).to(DEV) for a in (small, big))

    def run(out):
        return ops.paged_attention_mfma(case["q"], out, case["kp"], case["vp"], case["table"], small, big, H,
                                        hd ** -0.5)

    monkeypatch.setattr(ops, "_ONE_STREAM", True)
    one = run(torch.full_like(case["q"], float("nan")))
    assert torch.allclose(one.cpu().float(), _plain_rows(case, seqs), atol=1.5e-2, rtol=2e-2)
    monkeypatch.setattr(ops, "_ONE_STREAM", False)
    mine = torch.cuda.Stream(DEV)
    mine.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(mine):
        for _ in range(3):
            two = run(torch.full_like(case["q"], float("nan")))
            copy = two.clone()  # queued on the caller's stream right behind the call
            mine.synchronize()
            assert torch.equal(copy, one)
    held = torch.empty_like(case["q"])
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        run(held)
    for _ in range(2):
        held.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(held, one)


@pytest.mark.parametrize("cut", ["coarse", "pairs", "fine"])
def test_paged_attention_mfma_far_key_and_edges(ops, cut):
    """A key that gets nearly all the weight, at the edges of tiles, pages and
    chunks, for a decoded token (split kernel) and inside a portion (tile
    kernel)."""
    H, KV, hd, P = 8, 2, 64, 16
    for kpos in (0, 15, 16, 63, 64, 127, 128, 300, 399, 400):
        for seqs, qpos, row in (([(0, 3), (400, 1), (10, 2)], 400, 3), ([(0, 2), (380, 40)], 400, 2 + 20)):
            case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=22, peak=(1, qpos, 5, kpos))
            out, _, _ = _run_mfma(ops, case, seqs, H, KV, 0, cut)
            v = case["whole"][2][1]
            got = out.cpu().float()[row].view(H, hd)[5]
            assert torch.allclose(got, v[kpos, 1].float(), atol=2e-2), (kpos, seqs)
            assert torch.allclose(out.cpu().float(), _plain_rows(case, seqs), atol=1.5e-2, rtol=2e-2)


def test_paged_attention_mfma_window_edge(ops):
    H, KV, hd, P, w = 4, 1, 32, 16, 40
    for seqs, row in (([(100, 1)], 0), ([(90, 30)], 10)):
        for kpos, seen in ((100 - w, False), (100 - w + 1, True)):
            case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=23, peak=(0, 100, 1, kpos))
            out, _, _ = _run_mfma(ops, case, seqs, H, KV, w, "fine")
            v = case["whole"][2][0]
            got = out.cpu().float()[row].view(H, hd)[1]
            assert torch.allclose(got, v[kpos, 0].float(), atol=2e-2) == seen
            assert torch.allclose(out.cpu().float(), _plain_rows(case, seqs, w), atol=1.5e-2, rtol=2e-2)


@pytest.mark.parametrize("cut,longest", [("auto", 5000), ("fine", 5000), ("fine", 17000), ("coarse", 5000)])
def test_paged_attention_mfma_long_context(ops, cut, longest):
    """Llama-3.1-8B's attention shape at a context of several thousand keys,
    one decoded token and one long portion, beside a short sequence that has
    one chunk; with more chunks an item than one wave of the combine has
    lanes, and (17,000 keys, one tile a chunk asked for) more tiles than an
    item may have chunks."""
    H, KV, hd, P = 32, 8, 128, 64
    seqs = [(longest, 1), (3000, 200), (70, 1)]
    case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=24, poison=True)
    out, _, _ = _run_mfma(ops, case, seqs, H, KV, 0, cut)
    assert torch.allclose(out.cpu().float(), _plain_rows(case, seqs), atol=1.5e-2, rtol=2e-2)


@pytest.mark.parametrize("n_items", [24, 64, 300])
@pytest.mark.parametrize("cut", ["coarse", "fine"])
def test_paged_attention_mfma_many_decoding_sequences(ops, n_items, cut):
    """A decode step of dozens and hundreds of sequences of very different lengths, one token
    each, at Llama-3.1-8B's attention shape: the chunk list is long, items have from one chunk to
    dozens, and the partial results are merged by the combine kernel that takes a workgroup a row
    (few chunks: 24 and 64 sequences cut coarsely) or by the one that takes a workgroup a kv head."""
    import numpy as np

    H, KV, hd, P = 32, 8, 128, 64
    rng = np.random.default_rng(n_items)
    lens = rng.integers(0, 2500 if n_items < 100 else 700, n_items)
    lens[0], lens[1], lens[2] = 0, 63, 4000  # a first token, the last of a tile, one far longer than the rest
    seqs = [(int(n), 1) for n in lens]
    case = _paged_case(torch.bfloat16, seqs, H, KV, hd, P, seed=25)
    max_chunks = 2 * n_items if cut == "coarse" else 4096
    by_rows = max_chunks * KV * (H // KV) <= 8192  # COMBINE_ROWS_MAX_GROUPS in attention_mfma.hip
    assert by_rows == (cut == "coarse" and n_items <= 64)
    out, n_small, n_big = _run_mfma(ops, case, seqs, H, KV, 0, cut, max_rows=H // KV)  # as a decode step has it
    assert n_small == n_items and not n_big
    assert torch.isfinite(out).all()
    assert torch.allclose(out.cpu().float(), _plain_rows(case, seqs), atol=1.5e-2, rtol=2e-2)


@pytest.mark.parametrize("n_items,window,max_chunks,min_tiles", [
    (1, 0, 2, 4), (7, 0, 128, 4), (7, 100, 14, 1), (300, 0, 600, 4), (300, 777, 1024, 1), (513, 0, 4096, 2),
    (8, 0, 40, 4), (12, 0, 44, 4), (40, 0, 81, 2),
])
def test_attention_plan_cuts_every_item_into_equal_chunks(ops, n_items, window, max_chunks, min_tiles):
    """The plan that the split kernel works from: every item's tiles are covered once, in order, by
    chunks of the plan's size (the last may be shorter), the items' chunks one after the other; no
    more chunks than the list holds, none in use beyond the count, at most 256 an item."""
    import numpy as np

    rng = np.random.default_rng(n_items + window)
    n_tok = rng.integers(1, 4, n_items)
    pos0 = rng.integers(0, 40000 if n_items < 10 else 6000, n_items)
    items = np.stack([np.arange(n_items), np.cumsum(n_tok) - n_tok, n_tok, pos0], axis=1).astype(np.int32)
    plan = ops.attention_plan(torch.from_numpy(items.reshape(-1)).to(DEV), n_items, max_chunks, 128, window,
                              min_tiles).cpu().numpy()
    ts, used = int(plan[0]), int(plan[1])
    chunks = plan[4: 4 + 8 * max_chunks].reshape(max_chunks, 8)
    assert ts % min_tiles == 0 and 0 < used <= max_chunks
    assert (chunks[used:, 6] == 0).all() and (chunks[:used, 6] > 0).all()
    nxt = 0
    for i in range(n_items):
        last = pos0[i] + n_tok[i] - 1
        first_key = max(0, pos0[i] - window + 1) if window else 0
        t_lo, t_hi = first_key // 64, last // 64
        count = -(-(t_hi - t_lo + 1) // ts)
        assert count <= 256
        for c in range(count):
            rec = chunks[nxt + c]
            assert tuple(rec[:4]) == tuple(items[i]) and rec[6] == count and rec[7] == c
            assert rec[4] == t_lo + c * ts and rec[5] == min(t_hi + 1, t_lo + (c + 1) * ts)
        nxt += count
    assert nxt == used
    # the size that fits whatever the lengths are; with the longest item's number of chunks at that size, as even
    # as they can be, if all items' chunks still fit
    tiles = np.array([(pos0[i] + n_tok[i] - 1) // 64 - ((max(0, pos0[i] - window + 1) if window else 0) // 64) + 1
                      for i in range(n_items)])
    up = lambda v: max(1, -(-v // min_tiles)) * min_tiles
    longest = int(tiles.max())
    want = up(max(-(-int(tiles.sum()) // (max_chunks - n_items)), -(-longest // 256)))
    even = up(-(-longest // -(-longest // want)))
    if even < want and int((-(-tiles // even)).sum()) <= max_chunks:
        want = even
    assert ts == want
