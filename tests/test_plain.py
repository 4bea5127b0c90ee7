"""The plain implementation pinned by what fixes it beside the reference's
text: library special cases, invariants, and the input vectors of the
reference's own scripts.  Each check is chosen so that a plausible mistake
(a wrong sign or pairing, a norm in the wrong place) fails it."""

import math

import pytest
import torch
import torch.nn.functional as F

from plain_llama import (
    TINY_A,
    TINY_B,
    TINY_C,
    plain_attention,
    plain_forward,
    plain_random_weights,
    plain_rmsnorm,
    plain_rope_frequencies,
    plain_rope_interleaved,
    plain_rope_shuffle,
    plain_swiglu,
    plain_top_p_keep,
)


# ------------------------------------------------------------------ rmsnorm
def test_rmsnorm_is_the_library_routine():
    torch.manual_seed(0)
    x, w = torch.randn(7, 96), torch.randn(96)
    assert torch.allclose(plain_rmsnorm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), atol=1e-6)


def test_rmsnorm_invariants():
    torch.manual_seed(1)
    x = torch.randn(5, 64)
    y = plain_rmsnorm(x, torch.ones(64), 0.0)
    assert torch.allclose((y * y).mean(-1), torch.ones(5), atol=1e-5)  # unit mean square
    assert torch.allclose(plain_rmsnorm(3.7 * x, torch.ones(64), 0.0), y, atol=1e-5)  # scale free
    # eps sits inside the square root, added to the mean (not to the sum, not outside)
    x1 = torch.full((1, 4), 2.0)
    assert torch.allclose(plain_rmsnorm(x1, torch.ones(4), 5.0), x1 / 3.0)


# --------------------------------------------------------------------- rope
def test_rope_is_complex_multiplication():
    torch.manual_seed(2)
    x = torch.randn(6, 3, 32)
    pos = torch.tensor([0, 1, 5, 17, 100, 4000])
    freqs = torch.rand(16)
    want = torch.view_as_real(
        torch.view_as_complex(x.view(6, 3, 16, 2).contiguous())
        * torch.polar(torch.ones(6, 16), pos[:, None].float() * freqs)[:, None]
    ).reshape(6, 3, 32)
    assert torch.allclose(plain_rope_interleaved(x, pos, freqs), want, atol=1e-5)


@pytest.mark.parametrize("N", [1, 3, 4, 5, 8])
@pytest.mark.parametrize("H", [1, 8, 12])
@pytest.mark.parametrize("D", [128, 192])
def test_rope_on_the_reference_scripts_vectors(N, H, D):
    """scripts/rope.py:56-71: x[n,h,:] = arange(D) in bf16, pos = arange(N),
    random fp32 freqs under seed 24, atol 5e-4 against the formulation there
    (cos/sin of the outer product, even lanes real, odd lanes imaginary)."""
    torch.manual_seed(24)
    x = torch.arange(D, dtype=torch.bfloat16)[None, None].expand(N, H, -1).contiguous()
    pos = torch.arange(N, dtype=torch.int)
    freqs = torch.rand(D // 2, dtype=torch.float32)
    cos = torch.cos(pos.float().outer(freqs))[:, None]
    sin = torch.sin(pos.float().outer(freqs))[:, None]
    res, ims = x[:, :, ::2], x[:, :, 1::2]
    want = torch.cat(((res * cos - ims * sin).unsqueeze(-1), (ims * cos + res * sin).unsqueeze(-1)), -1)
    want = want.reshape(x.shape).to(x.dtype)
    assert torch.allclose(plain_rope_interleaved(x, pos, freqs).float(), want.float(), atol=5e-4)


def test_rope_invariants():
    torch.manual_seed(3)
    q, k = torch.randn(1, 2, 48), torch.randn(1, 2, 48)
    f = plain_rope_frequencies(48, 10000.0)
    at = lambda x, p: plain_rope_interleaved(x, torch.tensor([p]), f)
    assert torch.equal(at(q, 0), q)  # position 0 is the identity
    assert torch.allclose(at(at(q, 3), 9), at(q, 12), atol=1e-5)  # rotations add
    assert torch.allclose(at(q, 7).norm(), q.norm(), atol=1e-5)
    # only distances count: a shift of both positions leaves q.k unchanged ...
    d0 = (at(q, 11) * at(k, 4)).sum(-1)
    d1 = (at(q, 511) * at(k, 504)).sum(-1)
    assert torch.allclose(d0, d1, atol=1e-4)
    # ... and a wrong sign of the angle on one side would not
    d2 = (at(q, 11) * at(k, -4)).sum(-1)
    assert not torch.allclose(d0, d2, atol=1e-3)


def test_shuffle_plus_interleaved_is_rotate_half_on_checkpoint_rows():
    """The checkpoint convention rotates pairs (i, i + hd/2):
    out = x*cos + rotate_half(x)*sin with rotate_half(x) = cat(-x2, x1).  With
    the rows permuted as in loading.py:296-305 the interleaved rotation gives
    the same scores q.k, though q and k themselves come out permuted."""
    torch.manual_seed(4)
    H, hd, D, T = 3, 16, 40, 9
    wq, wk = torch.randn(H * hd, D), torch.randn(H * hd, D)
    x = torch.randn(T, D)
    pos = torch.arange(T) + 3
    f = plain_rope_frequencies(hd, 10000.0)

    def rotate_half_rope(v):  # v [T, H, hd]
        ang = pos[:, None].float() * f[None, :]
        cos = torch.cat([torch.cos(ang), torch.cos(ang)], -1)[:, None]
        sin = torch.cat([torch.sin(ang), torch.sin(ang)], -1)[:, None]
        v1, v2 = v[..., : hd // 2], v[..., hd // 2 :]
        return v * cos + torch.cat([-v2, v1], -1) * sin

    q_hf = rotate_half_rope((x @ wq.T).view(T, H, hd))
    k_hf = rotate_half_rope((x @ wk.T).view(T, H, hd))
    q_il = plain_rope_interleaved((x @ plain_rope_shuffle(wq, H).T).view(T, H, hd), pos, f)
    k_il = plain_rope_interleaved((x @ plain_rope_shuffle(wk, H).T).view(T, H, hd), pos, f)
    s_hf = torch.einsum("thd,shd->hts", q_hf, k_hf)
    s_il = torch.einsum("thd,shd->hts", q_il, k_il)
    assert torch.allclose(s_hf, s_il, atol=1e-3)
    # the shuffle is a permutation of rows
    assert torch.equal(plain_rope_shuffle(wq, H).sort(0).values, wq.sort(0).values)
    # without it the scores differ: the test can fail
    q_bad = plain_rope_interleaved((x @ wq.T).view(T, H, hd), pos, f)
    k_bad = plain_rope_interleaved((x @ wk.T).view(T, H, hd), pos, f)
    assert not torch.allclose(torch.einsum("thd,shd->hts", q_bad, k_bad), s_hf, atol=1e-2)


def test_llama3_frequencies():
    sc = TINY_B["rope_scaling"]
    base = plain_rope_frequencies(32, 500000.0)
    f = plain_rope_frequencies(32, 500000.0, sc)
    assert torch.equal(base, 1.0 / (500000.0 ** (torch.arange(0, 32, 2).float() / 32)))
    wl = 2 * math.pi / base
    ctx = sc["original_max_position_embeddings"]
    hi, lo = ctx / sc["high_freq_factor"], ctx / sc["low_freq_factor"]
    # all three branches occur at this size
    assert (wl < hi).any() and ((wl >= hi) & (wl <= lo)).any() and (wl > lo).any()
    assert torch.equal(f[wl < hi], base[wl < hi])  # short waves untouched, bit for bit
    assert torch.allclose(f[wl > lo], base[wl > lo] / sc["factor"])
    mid = (wl >= hi) & (wl <= lo)
    assert ((f[mid] > base[mid] / sc["factor"]) & (f[mid] < base[mid])).all()
    assert (f[1:] < f[:-1]).all()  # still decreasing
    # factor 1 is no scaling; continuity at both edges of the blend
    one = dict(sc, factor=1.0)
    assert torch.allclose(plain_rope_frequencies(32, 500000.0, one), base)
    for edge, expect_div in ((lo, sc["factor"]), (hi, 1.0)):
        # a frequency whose wavelength is exactly an edge: theta chosen so that f_1 = 2 pi / edge
        fr = 2 * math.pi / edge
        theta = (1 / fr) ** (4 / 2)  # head_dim 4: f_1 = theta^(-2/4)
        got = plain_rope_frequencies(4, theta, sc)[1]
        assert math.isclose(float(got), fr / expect_div, rel_tol=1e-4)


@pytest.mark.parametrize("head_dim,theta,sc", [
    (128, 500000.0, dict(factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)),
    (128, 500000.0, dict(factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)),
    (256, 10000.0, dict(factor=3.0, low_freq_factor=2.0, high_freq_factor=16.0, original_max_position_embeddings=96)),
])
def test_llama3_blend_is_affine_in_the_frequency(head_dim, theta, sc):
    """What fixes the middle band beside the reference's text (fastgen/forward.py:630-633): the blend's
    variable is ``ctx / wavelength = ctx * f / (2 pi)``, so ``f' / f = (1 - x) / factor + x`` is affine in the
    frequency ``f``, with the values 1 / factor and 1 at the band's two edges.  An affine function with those
    two values is one function: a blend that is linear in the wavelength (or in the index, or in log f) equals
    it at the edges and nowhere between, and fails here."""
    base = plain_rope_frequencies(head_dim, theta).double()
    f = plain_rope_frequencies(head_dim, theta, sc).double()
    ctx, lo_f, hi_f, factor = (sc["original_max_position_embeddings"], sc["low_freq_factor"], sc["high_freq_factor"],
                               sc["factor"])
    f_lo, f_hi = 2 * math.pi * lo_f / ctx, 2 * math.pi * hi_f / ctx  # frequencies of the band's edges
    mid = (base > f_lo * 1.001) & (base < f_hi * 0.999)
    assert int(mid.sum()) >= 3, "the test needs three frequencies inside the band"
    ratio = f[mid] / base[mid]
    # the affine function through (f_lo, 1 / factor) and (f_hi, 1)
    want = 1 / factor + (base[mid] - f_lo) / (f_hi - f_lo) * (1 - 1 / factor)
    assert torch.allclose(ratio, want, rtol=2e-5, atol=0), (ratio, want)
    # equal slopes between neighbours (affine), and the plausible mistakes are far from it
    slopes = (ratio[1:] - ratio[:-1]) / (base[mid][1:] - base[mid][:-1])
    assert torch.allclose(slopes, slopes[0].expand_as(slopes), rtol=1e-3)
    wl, wl_lo, wl_hi = 2 * math.pi / base[mid], ctx / lo_f, ctx / hi_f
    in_wavelength = 1 / factor + (wl_lo - wl) / (wl_lo - wl_hi) * (1 - 1 / factor)
    assert float((in_wavelength - want).abs().max()) > 0.05
    in_log = 1 / factor + (base[mid].log() - math.log(f_lo)) / (math.log(f_hi) - math.log(f_lo)) * (1 - 1 / factor)
    assert float((in_log - want).abs().max()) > 0.05


# ---------------------------------------------------------------- attention
@pytest.mark.parametrize("H,KV", [(4, 4), (4, 2), (6, 1), (1, 1)])
def test_attention_is_the_library_routine(H, KV):
    torch.manual_seed(5)
    T, hd = 11, 16
    q, k, v = torch.randn(T, H, hd), torch.randn(T, KV, hd), torch.randn(T, KV, hd)
    G = H // KV
    want = F.scaled_dot_product_attention(
        q.transpose(0, 1)[None], k.repeat_interleave(G, 1).transpose(0, 1)[None],
        v.repeat_interleave(G, 1).transpose(0, 1)[None], is_causal=True,
    )[0].transpose(0, 1)
    assert torch.allclose(plain_attention(q, k, v), want, atol=1e-5)


def test_attention_invariants():
    torch.manual_seed(6)
    T, H, KV, hd = 9, 4, 2, 8
    q, k, v = torch.randn(T, H, hd), torch.randn(T, KV, hd), torch.randn(T, KV, hd)
    o = plain_attention(q, k, v)
    assert torch.allclose(o[0], v[0].repeat_interleave(2, 0), atol=1e-6)  # first token sees itself only
    # causal: changing a later key changes no earlier output
    k2, v2 = k.clone(), v.clone()
    k2[6:], v2[6:] = 9.0, -9.0
    assert torch.allclose(plain_attention(q, k2, v2)[:6], o[:6], atol=1e-6)
    # one score made to stand out: the output is that key's value
    qq, kk = q.clone(), k.clone()
    kk[3, 0] = 0
    kk[3, 0, 0] = 50.0
    qq[8, 1] = 0
    qq[8, 1, 0] = 50.0
    assert torch.allclose(plain_attention(qq, kk, v)[8, 1], v[3, 0], atol=1e-4)
    # window w: token p sees keys p-w+1 .. p
    ow = plain_attention(q, k, v, window=3)
    assert torch.allclose(ow[:3], o[:3], atol=1e-6)
    assert torch.allclose(ow[8], plain_attention(q[6:], k[6:], v[6:])[2], atol=1e-5)


def test_swiglu_special_cases():
    torch.manual_seed(7)
    x = torch.randn(4, 12)
    w1, w3, w2 = torch.randn(20, 12), torch.randn(20, 12), torch.randn(12, 20)
    assert torch.allclose(plain_swiglu(x, w1, w3, w2), (F.silu(x @ w1.T) * (x @ w3.T)) @ w2.T, atol=1e-5)
    assert torch.equal(plain_swiglu(x, torch.zeros_like(w1), w3, w2), torch.zeros(4, 12))  # zero gate
    # gate and up are not interchangeable
    assert not torch.allclose(plain_swiglu(x, w1, w3, w2), plain_swiglu(x, w3, w1, w2), atol=1e-3)


# -------------------------------------------------------------- whole model
@pytest.mark.parametrize("cfg,seed", [(TINY_A, 0), (TINY_B, 1), (TINY_C, 2)])
def test_model_is_causal_and_deterministic(cfg, seed):
    w = plain_random_weights(cfg, seed)
    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(0, cfg["vocab_size"], (21,), generator=g).tolist()
    full = plain_forward(w, cfg, toks)
    assert full.shape == (21, cfg["vocab_size"]) and full.dtype == torch.float32
    # a prefix gives the same logits: no token looks ahead
    assert torch.allclose(plain_forward(w, cfg, toks[:9]), full[:9], atol=1e-5)


def test_model_one_layer_by_hand():
    """One layer, one head, no rotation effect at position 0: the first
    token's logits follow from the formulas with nothing but matrix products,
    which pins the order norm -> attention -> residual -> norm -> mlp."""
    cfg = dict(TINY_A, num_hidden_layers=1, num_attention_heads=1, num_key_value_heads=1,
               hidden_size=16, intermediate_size=24, vocab_size=32)
    w = plain_random_weights(cfg, 3)
    w = {k: v * 10 if "proj" in k else v for k, v in w.items()}
    tok = 5
    h = w["model.embed_tokens.weight"][tok]
    p = "model.layers.0."
    x = F.rms_norm(h, (16,), w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
    a = w[p + "self_attn.o_proj.weight"] @ (w[p + "self_attn.v_proj.weight"] @ x)  # softmax over one key = 1
    h = h + a
    x = F.rms_norm(h, (16,), w[p + "post_attention_layernorm.weight"], cfg["rms_norm_eps"])
    m = w[p + "mlp.down_proj.weight"] @ (F.silu(w[p + "mlp.gate_proj.weight"] @ x) * (w[p + "mlp.up_proj.weight"] @ x))
    h = F.rms_norm(h + m, (16,), w["model.norm.weight"], cfg["rms_norm_eps"])
    want = w["model.embed_tokens.weight"] @ h  # tied
    got = plain_forward(w, cfg, [tok])[0]
    assert torch.allclose(got, want, atol=1e-4)


def test_top_p_keep_mask():
    probs = torch.tensor([[0.5, 0.3, 0.15, 0.05]])
    assert plain_top_p_keep(probs, 0.6).tolist() == [[True, True, False, False]]
    assert plain_top_p_keep(probs, 0.45).tolist() == [[True, False, False, False]]
    assert plain_top_p_keep(probs[:, [2, 0, 3, 1]], 0.85).tolist() == [[True, True, False, True]]
