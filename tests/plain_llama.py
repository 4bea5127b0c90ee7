"""A plain, slow Llama: whole sequences, no cache, no batching, one function
per part, written from the reference's formulas and sharing no code with
``fastgen_amd``.  It is what the engine is compared with.

Citations are ``file:line`` of facebookresearch/fastgen.  Weights are taken
under their checkpoint names and, as the reference does, the q/k projection
rows are permuted at load so that the rotation acts on interleaved pairs.
"""

from __future__ import annotations

import math
from typing import Dict, Mapping, Optional

import torch


def _up(x: torch.Tensor) -> torch.Tensor:
    """To the precision of the fp32 islands: float32, or float64 when the whole
    run is in float64 (used to judge float32 runs of wide layers)."""
    return x if x.dtype == torch.float64 else x.float()


def plain_rope_frequencies(head_dim: int, theta: float, scaling: Optional[Mapping] = None) -> torch.Tensor:
    """fastgen/forward.py:609-635.  ``scaling`` holds the config.json keys
    ``factor``, ``low_freq_factor``, ``high_freq_factor``,
    ``original_max_position_embeddings`` (fastgen/utils/loading.py:75-82)."""
    pows = torch.arange(0, head_dim, 2).float() / head_dim
    freqs = 1.0 / (theta**pows)
    if not scaling:
        return freqs
    low, high = scaling["low_freq_factor"], scaling["high_freq_factor"]
    ctx, factor = scaling["original_max_position_embeddings"], scaling["factor"]
    low_freq_wavelen = ctx / low
    high_freq_wavelen = ctx / high
    result = freqs.clone()
    for idx in range(len(freqs)):
        freq = freqs[idx]
        wavelen = 2 * math.pi / freq
        if wavelen > low_freq_wavelen:
            result[idx] = freq / factor
        if high_freq_wavelen <= wavelen <= low_freq_wavelen:
            x = ctx / wavelen - low
            x = x / (high - low)
            result[idx] = (1 - x) * freq / factor + x * freq
    return result


def plain_rope_interleaved(x: torch.Tensor, pos: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """fastgen/kernels/rope.py:56-89 (and the formulation of scripts/rope.py:10-20):
    x ``[T, heads, hd]``; pair (x[2i], x[2i+1]) rotated by pos * freqs[i]."""
    angles = pos.to(torch.float32)[:, None] * freqs[None, :]  # [T, hd/2]
    cos, sin = torch.cos(angles)[:, None, :], torch.sin(angles)[:, None, :]
    re, im = _up(x[..., 0::2]), _up(x[..., 1::2])
    out = torch.empty_like(x, dtype=re.dtype)
    out[..., 0::2] = re * cos - im * sin
    out[..., 1::2] = im * cos + re * sin
    return out.to(x.dtype)


def plain_rope_shuffle(w: torch.Tensor, n_heads: int) -> torch.Tensor:
    """fastgen/utils/loading.py:296-305: rows of a checkpoint's q/k projection
    (per head: first half "real", second half "imaginary") to interleaved."""
    out_dim, in_dim = w.shape
    hd = out_dim // n_heads
    return w.reshape(n_heads, 2, hd // 2, in_dim).transpose(1, 2).reshape(out_dim, in_dim)


def plain_rmsnorm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """fastgen/kernels/rmsnorm.py:33-60: fp32 mean of squares, a * rstd * w."""
    xf = _up(x)
    rstd = torch.rsqrt((xf * xf).sum(-1, keepdim=True) / x.shape[-1] + eps)
    return (xf * rstd * _up(w)).to(x.dtype)


def plain_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, window: Optional[int] = None) -> torch.Tensor:
    """fastgen/forward.py:176-258 for one whole sequence: q ``[T, H, hd]``,
    k, v ``[T, KV, hd]``; causal; scale hd^-0.5 (225, 249); query head h reads
    kv head h // (H // KV).  ``window``: keys p-window+1 .. p only."""
    T, H, hd = q.shape
    KV = k.shape[1]
    G = H // KV
    out = torch.empty_like(q)
    scale = hd**-0.5
    idx = torch.arange(T, device=q.device)
    mask = idx[None, :] <= idx[:, None]
    if window:
        mask &= idx[None, :] > idx[:, None] - window
    for h in range(H):
        kh, vh = _up(k[:, h // G]), _up(v[:, h // G])
        s = (_up(q[:, h]) @ kh.T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, dim=-1)
        out[:, h] = (p @ vh).to(q.dtype)
    return out


def plain_swiglu(x: torch.Tensor, w1: torch.Tensor, w3: torch.Tensor, w2: torch.Tensor) -> torch.Tensor:
    """fastgen/forward.py:488-496: w2(silu(w1 x) * w3 x); w1 = gate, w3 = up
    (fastgen/utils/loading.py:100-111)."""
    g = x @ w1.T
    u = x @ w3.T
    return ((g * torch.sigmoid(g)) * u) @ w2.T


def plain_forward(weights: Mapping[str, torch.Tensor], config: Mapping, tokens, dtype=torch.float32,
                  window: Optional[int] = None) -> torch.Tensor:
    """Logits ``[T, vocab]`` (fp32) of one whole sequence, fastgen/forward.py:347-515.

    ``dtype`` is the precision of weights and activations between the fp32
    islands; the residual stream is added in ``dtype`` as the reference does
    (forward.py:472, 499)."""
    D = config["hidden_size"]
    H = config["num_attention_heads"]
    KV = config.get("num_key_value_heads", H)
    hd = D // H  # fastgen/forward.py:364
    eps = config["rms_norm_eps"]
    L = config["num_hidden_layers"]
    dev = next(iter(weights.values())).device  # where the weights are is where it runs (the CPU, in most tests)
    freqs = plain_rope_frequencies(hd, config["rope_theta"], config.get("rope_scaling")).to(dev)
    W = {k: v.to(dtype) for k, v in weights.items()}
    tok = torch.as_tensor(tokens, dtype=torch.long, device=dev)
    T = tok.numel()
    pos = torch.arange(T, device=dev)
    h = W["model.embed_tokens.weight"][tok]  # forward.py:406-409
    for i in range(L):
        p = f"model.layers.{i}."
        x = plain_rmsnorm(h, W[p + "input_layernorm.weight"], eps)  # forward.py:419
        wq = plain_rope_shuffle(W[p + "self_attn.q_proj.weight"], H)
        wk = plain_rope_shuffle(W[p + "self_attn.k_proj.weight"], KV)
        xq = (x @ wq.T).view(T, H, hd)  # forward.py:438-445
        xk = (x @ wk.T).view(T, KV, hd)
        xv = (x @ W[p + "self_attn.v_proj.weight"].T).view(T, KV, hd)
        xq = plain_rope_interleaved(xq, pos, freqs)  # forward.py:449-450
        xk = plain_rope_interleaved(xk, pos, freqs)
        a = plain_attention(xq, xk, xv, window).reshape(T, H * hd)  # forward.py:468
        h = h + a @ W[p + "self_attn.o_proj.weight"].T  # forward.py:470-472
        x = plain_rmsnorm(h, W[p + "post_attention_layernorm.weight"], eps)  # forward.py:474
        h = h + plain_swiglu(x, W[p + "mlp.gate_proj.weight"], W[p + "mlp.up_proj.weight"],
                             W[p + "mlp.down_proj.weight"])  # forward.py:483-499
    h = plain_rmsnorm(h, W["model.norm.weight"], eps)  # forward.py:501
    head = W["model.embed_tokens.weight"] if config.get("tie_word_embeddings") else W["lm_head.weight"]
    return _up(h @ head.T)  # forward.py:507-515


def plain_greedy(weights, config, prompt, n_new: int, dtype=torch.float32):
    """Greedy continuation by re-running the whole sequence for every token
    (argmax of the last row: fastgen/generate.py:892-896)."""
    toks = list(prompt)
    for _ in range(n_new):
        logits = plain_forward(weights, config, toks, dtype)
        toks.append(int(torch.argmax(logits[-1])))
    return toks[len(prompt):]


def plain_top_p_keep(probs: torch.Tensor, p: float) -> torch.Tensor:
    """fastgen/utils/sampling.py:26-28: the mask of tokens that stay, i.e.
    whose preceding mass in descending order does not exceed p."""
    sort, idx = torch.sort(probs, dim=-1, descending=True)
    csum = torch.cumsum(sort, dim=-1)
    keep_sorted = ~(csum - sort > p)
    keep = torch.zeros_like(keep_sorted)
    keep.scatter_(-1, idx, keep_sorted)
    return keep


# ---------------------------------------------------------------- test models
TINY_A = dict(
    architectures=["LlamaForCausalLM"], hidden_size=64, intermediate_size=192, num_hidden_layers=2,
    num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-6, vocab_size=256, rope_theta=10000.0,
    rope_scaling=None, tie_word_embeddings=True, max_position_embeddings=128,
)
TINY_B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=192, intermediate_size=512, num_hidden_layers=3,
    num_attention_heads=6, num_key_value_heads=3, rms_norm_eps=1e-5, vocab_size=384, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=64),
    tie_word_embeddings=False, max_position_embeddings=256,
)
# a third one with sizes that are no power of two anywhere, one kv head and a wide group
TINY_C = dict(
    architectures=["LlamaForCausalLM"], hidden_size=240, intermediate_size=328, num_hidden_layers=2,
    num_attention_heads=5, num_key_value_heads=1, rms_norm_eps=3e-6, vocab_size=515, rope_theta=31000.0,
    rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=2.0,
                      original_max_position_embeddings=32),
    tie_word_embeddings=False, max_position_embeddings=512,
)


def plain_random_weights(config: Mapping, seed: int) -> Dict[str, torch.Tensor]:
    """Random fp32 weights under checkpoint names: linears and embedding
    N(0, 0.02), norm weights 1 + N(0, 0.01)."""
    g = torch.Generator().manual_seed(seed)
    D, F, V = config["hidden_size"], config["intermediate_size"], config["vocab_size"]
    H = config["num_attention_heads"]
    KV = config.get("num_key_value_heads", H)
    hd = D // H

    def lin(o, i):
        return torch.randn(o, i, generator=g) * 0.02

    def nrm():
        return 1 + torch.randn(D, generator=g) * 0.01

    w = {"model.embed_tokens.weight": lin(V, D), "model.norm.weight": nrm()}
    if not config.get("tie_word_embeddings"):
        w["lm_head.weight"] = lin(V, D)
    for i in range(config["num_hidden_layers"]):
        p = f"model.layers.{i}."
        w[p + "self_attn.q_proj.weight"] = lin(H * hd, D)
        w[p + "self_attn.k_proj.weight"] = lin(KV * hd, D)
        w[p + "self_attn.v_proj.weight"] = lin(KV * hd, D)
        w[p + "self_attn.o_proj.weight"] = lin(D, H * hd)
        w[p + "mlp.gate_proj.weight"] = lin(F, D)
        w[p + "mlp.up_proj.weight"] = lin(F, D)
        w[p + "mlp.down_proj.weight"] = lin(D, F)
        w[p + "input_layernorm.weight"] = nrm()
        w[p + "post_attention_layernorm.weight"] = nrm()
    return w
