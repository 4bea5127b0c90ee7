#!/usr/bin/python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L]
    python bench.py --workload serve        # continuous batching, see serve_workload()
    python bench.py --workload readme       # the load of the reference's README, see readme_workload()
    python bench.py --workload readme --shape 70b   # the same load at the 70B sizes, cache = the memory left

The model has the layer sizes of Llama 3.1 8B (32 layers, hidden 4096, 32
heads, 8 kv heads, head size 128, feed-forward 14336, vocabulary 128256,
llama3 rope scaling) with random bfloat16 weights.  A "step" is one decode
step of a batch whose requests each hold a 2,048-token prompt; ``value`` is
decoded tokens a second.  The same line carries the time of a 2,048-token
prefill, the decode step's fraction of the HBM roofline, and decode at batch
1 and 64.  Token ids are uniform random (synthetic); nothing is read from disk.
"""

from __future__ import annotations

import argparse
import json
import sys
import time

PEAK_HBM = 8.0e12  # bytes/s, MI355X published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

LLAMA_8B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=4096, intermediate_size=14336, num_hidden_layers=32,
    num_attention_heads=32, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=131072,
)
PROMPT_LEN = 2048
CONTEXT_LEN = 8192  # capacity per request
PAGE = 64


LLAMA_3B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=3072, intermediate_size=8192, num_hidden_layers=28,
    num_attention_heads=24, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=True, max_position_embeddings=131072,
)


LLAMA_70B = dict(
    architectures=["LlamaForCausalLM"], hidden_size=8192, intermediate_size=28672, num_hidden_layers=80,
    num_attention_heads=64, num_key_value_heads=8, rms_norm_eps=1e-5, vocab_size=128256, rope_theta=500000.0,
    rope_scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                      original_max_position_embeddings=8192),
    tie_word_embeddings=False, max_position_embeddings=131072,
)
SHAPES = {"3b": ("llama-3.2-3b-shape-random", LLAMA_3B), "8b": ("llama-3.1-8b-shape-random", LLAMA_8B),
          "70b": ("llama-3.1-70b-shape-random", LLAMA_70B)}


def workload_roofline(engine, cfg: dict, seconds: float) -> dict:
    """Where a whole run stands against the two rooflines: the bytes its steps had to read (every weight once
    a step, and the cache of every request in the step) over the time and the HBM peak; the flops of its matrix
    products and attention over the time and the bf16 MFMA peak.  A run is bound by neither alone (its prompt
    steps by the matrix cores, its decode steps by memory), so the two fractions together say how much of the
    GPU it used."""
    D, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    H, KV, L = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["num_hidden_layers"]
    hd = D // H
    layer_params = D * (H + 2 * KV) * hd + H * hd * D + 3 * D * F
    w = engine.work
    weight_bytes = (L * layer_params + D * V) * 2
    nbytes = w.steps * weight_bytes + w.cache_reads * 2 * KV * hd * 2 * L
    flops = 2 * w.tokens * L * layer_params + 4 * H * hd * L * w.keys_attended
    return {"hbm_frac": round(nbytes / seconds / PEAK_HBM, 4), "mfma_frac": round(flops / seconds / PEAK_FLOPS["bf16"], 4),
            "gbytes": round(nbytes / 1e9, 1), "tflop": round(flops / 1e12, 1), "steps": w.steps, "tokens": w.tokens}


def serve_workload(n_requests: int = 256, step_budget: int = 2048, shape: str = "3b") -> int:
    """Continuous batching at the Llama 3.2 3B shape (random bfloat16 weights): ``n_requests`` requests
    arrive at once, prompts of 128..4096 uniform random ids, 32..512 greedy tokens each, at most 256 live,
    a budget of ``step_budget`` tokens a step (prompt portions beside decoded tokens).  One JSON line: generated
    tokens a second over the whole run, prompt processing included."""
    import random

    import torch

    from fastgen_amd.engine import Engine
    from fastgen_amd.sampling import SamplingParams

    rng = random.Random(3)
    plens = [rng.randint(128, 4096) for _ in range(n_requests)]
    olens = [rng.randint(32, 512) for _ in range(n_requests)]
    max_batch = min(256, n_requests)
    model_name, cfg = SHAPES[shape]
    engine = Engine.from_config(cfg, seed=3, dtype=torch.bfloat16, page_size=PAGE, max_tokens=max_batch * 4672,
                                max_batch=max_batch, max_step_tokens=step_budget)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg["vocab_size"], (n,), generator=g).tolist() for n in plens]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for p, o in zip(prompts, olens):
        engine.add_request(p, SamplingParams(temperature=0.0, max_new_tokens=o))
    n_done, last = 0, t0
    while engine.has_work():
        n_done += len(engine.step())
        if time.perf_counter() - last > 20:
            last = time.perf_counter()
            print(f"[bench] {n_done}/{n_requests} requests done", file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    print(json.dumps({
        "metric": "generated tok/s, continuous batching", "value": round(sum(olens) / dt, 1), "unit": "tokens/s",
        "n_gpus": 1, "seconds": round(dt, 3), "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
        "roofline": workload_roofline(engine, cfg, dt),
        "config": {"model": model_name, "requests": n_requests, "prompt_tokens": sum(plens),
                   "generated_tokens": sum(olens), "max_batch": max_batch, "step_budget": step_budget, "page_size": PAGE,
                   "engine_steps": engine.n_steps, "preemptions": engine.scheduler.n_preemptions,
                   "weight_copies": 2 if engine.model.packed() else 1},
    }), flush=True)
    return 0


def readme_workload(shape: str = "8b") -> int:
    """The load behind the numbers of the reference's README (``README.md:22-28``, ``scripts/bench.py:104-106``:
    512 prompts of 1,024 tokens, 128 decode steps each, generated tokens over the wall-clock time of the whole
    batch), with random bfloat16 weights and uniform random ids, at the Llama 3.1 8B shape or, ``--shape 70b``, at
    the 70B shape (141 GB of weights).  The cache is what the GPU has free once the weights are in place
    (``fastgen/utils/tune.py:68-84`` sizes it from a budget): at 8B it holds all 512 requests, at 70B it does not
    and requests are preempted and recomputed.  The reference publishes 3,430 tok/s for Mistral 7B on one H100 and
    2,260 tok/s for Llama 70B on eight, through its server: other models and other hardware, so the ratio in
    ``vs_published`` is context, not a like-for-like comparison."""
    import torch

    from fastgen_amd.engine import Engine, Model
    from fastgen_amd.sampling import SamplingParams

    n, p_len, n_gen, max_batch = 512, 1024, 128, 512
    model_name, cfg = SHAPES[shape]
    published = {"8b": (3430.0, "3430 tok/s, Mistral 7B, 1x H100 (reference README)"),
                 "70b": (2260.0, "2260 tok/s, Llama 70B, 8x H100 (reference README)")}.get(shape)
    t0 = time.perf_counter()
    model = Model.random(cfg, 4 if shape == "70b" else 2, torch.bfloat16, "cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.perf_counter() - t0:.1f} s", file=sys.stderr, flush=True)
    # no request is longer than prompt + generated: the cache never needs more than that for each
    engine = Engine(model, page_size=PAGE, max_tokens=None, max_batch=max_batch, max_step_tokens=8192,
                    max_seq=-(-(p_len + n_gen) // PAGE) * PAGE)
    pool = engine.scheduler.pool_tokens
    print(f"[bench] cache of {pool} tokens ({pool * engine.runner.storage.bytes_per_token() / 1e9:.1f} GB)",
          file=sys.stderr, flush=True)
    g = torch.Generator().manual_seed(0)
    prompts = [torch.randint(0, cfg["vocab_size"], (p_len,), generator=g).tolist() for _ in range(n)]
    params = SamplingParams(temperature=0.0, max_new_tokens=n_gen)
    torch.cuda.synchronize()
    t0 = last = time.perf_counter()
    for p in prompts:
        engine.add_request(p, params)
    generated = n_done = 0
    while engine.has_work():
        for r in engine.step():
            generated += len(r.generated)
            n_done += 1
        if time.perf_counter() - last > 20:
            last = time.perf_counter()
            print(f"[bench] {n_done}/{n} requests done, {engine.scheduler.n_preemptions} preemptions",
                  file=sys.stderr, flush=True)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    print(json.dumps({
        "metric": "generated tok/s, 512 prompts x 1024 tokens, 128 decode steps", "value": round(generated / dt, 1),
        "unit": "tokens/s", "n_gpus": 1, "seconds": round(dt, 3), "higher_is_better": True, "dtype": "bf16",
        "data": "synthetic", "vs_published": round(generated / dt / published[0], 3) if published else None,
        "roofline": workload_roofline(engine, cfg, dt),
        "config": {"model": model_name, "requests": n, "prompt_len": p_len, "generated": n_gen,
                   "max_batch": max_batch, "step_budget": 8192, "page_size": PAGE, "engine_steps": engine.n_steps,
                   "cache_tokens": pool, "cache": "free memory after the weights",
                   "preemptions": engine.scheduler.n_preemptions,
                   "weight_copies": 2 if engine.model.packed() else 1,
                   "published": published[1] if published else None},
    }), flush=True)
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the shape has (both numbers are reported)")
    ap.add_argument("--shape", choices=sorted(SHAPES), default=None,
                    help="layer sizes: Llama 3.1 8B (the benchmark's configuration; default but for serve), 70B"
                         " (141 GB of weights) or Llama 3.2 3B (the default of serve)")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT_LEN,
                    help="tokens of the timed prefill step (default: the benchmark's 2,048)")
    ap.add_argument("--context", type=int, default=None,
                    help="cached tokens of each request when the timed decode steps begin (default: the prompt's"
                         " 2,048); more are fed untimed, in portions")
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--no-points", action="store_true", help="skip decode at batch 1 and 64")
    ap.add_argument("--workload", choices=["decode", "serve", "readme"], default="decode",
                    help="decode (default): the step benchmark; serve: continuous batching of 256 requests; "
                         "readme: the load of the reference's README")
    ap.add_argument("--step-budget", type=int, default=2048, help="tokens a step of the serve workload")
    ap.add_argument("--show-choices", action="store_true",
                    help="print (stderr) which kernel the run's measurements chose for each matrix product")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported", flush=True)
        return 2
    if a.workload == "serve":
        return serve_workload(step_budget=a.step_budget, shape=a.shape or "3b")
    if a.workload == "readme":
        return readme_workload(a.shape or "8b")
    a.shape = a.shape or "8b"

    import torch

    from fastgen_amd.engine import Engine

    dtype = {"bf16": torch.bfloat16, "fp32": torch.float32}[a.dtype]
    model_name, shape = SHAPES[a.shape]
    full_layers = shape["num_hidden_layers"]
    a.layers = a.layers or full_layers
    cfg = dict(shape, num_hidden_layers=a.layers)
    batches = sorted({a.batch} | (set() if a.no_points else {1, 64}))
    max_b = max(batches)
    t0 = time.time()
    # The cache holds CONTEXT_LEN tokens for every request of the largest batch (68.7 GB at batch 64 of the 8B
    # shape in bfloat16), or what the GPU has free beside the weights if that is less (the 70B shape); with
    # --context, as many as the requests reach: the first requests of a batch decode while the prompts of the
    # later ones are still fed in portions, so they are longer than --context by the number of those steps.
    from fastgen_amd.engine import Model

    ctx_len = a.context or PROMPT_LEN
    feed_steps = -(-max_b * ctx_len // max(1, PROMPT_LEN - max_b)) + max_b
    capacity = max(CONTEXT_LEN, -(-(ctx_len + feed_steps + a.warmup + a.steps + 72) // PAGE) * PAGE,
                   -(-a.prefill_tokens // PAGE) * PAGE)
    if capacity > cfg["max_position_embeddings"]:
        print(f"bench.py: --context {ctx_len} and the steps after it pass the model's {cfg['max_position_embeddings']}"
              " positions", flush=True)
        return 2
    model = Model.random(cfg, 2, dtype, "cuda:0")
    engine = Engine(model, page_size=PAGE, max_tokens=None, max_batch=max_b, max_step_tokens=PROMPT_LEN,
                    max_seq=capacity)
    torch.cuda.synchronize()
    print(f"[bench] model built in {time.time() - t0:.1f} s", file=sys.stderr, flush=True)
    model = engine.model
    D, F, V = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    H, KV = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd, L = D // H, a.layers
    esize = 2 if a.dtype == "bf16" else 4
    layer_params = D * (H + 2 * KV) * hd + H * hd * D + 3 * D * F
    kv_bytes_per_token = 2 * KV * hd * esize * L

    g = torch.Generator().manual_seed(0)

    def prompt(n):
        return torch.randint(0, V, (n,), generator=g).tolist()

    # ------------------------------------------------------------ prefill
    times = engine.time_prefill(prompt(a.prefill_tokens), repeats=5)
    pre = sum(times) / len(times)  # the mean of the repeats after one warm-up; the best is reported beside it
    T = a.prefill_tokens
    flops = 2 * T * L * layer_params + L * 4 * H * hd * (T * (T + 1) // 2) + 2 * D * V
    prefill = {"value": round(T / pre, 1), "tokens": T, "ms": round(pre * 1e3, 3),
               "frac": round(flops / pre / PEAK_FLOPS[a.dtype], 4), "repeats": len(times),
               "best_ms": round(min(times) * 1e3, 3)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)

    # ------------------------------------------------------------- decode
    results = {}
    for b in batches:
        steps, warm = (a.steps, a.warmup)
        dt = engine.time_decode([prompt(ctx_len) for _ in range(b)], steps=steps, warmup=warm)
        ctx = engine.last_mean_context  # mean cached tokens of a request during the timed steps
        nbytes = (L * layer_params + D * V) * esize + b * ctx * kv_bytes_per_token
        results[b] = dict(tok_s=b * steps / dt, ms=dt / steps * 1e3, gbs=nbytes / (dt / steps) / 1e9, ctx=ctx)
        print(f"[bench] decode batch {b}: {results[b]}", file=sys.stderr, flush=True)

    r = results[a.batch]
    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2048 tokens; % of roofline",
        "value": round(r["tok_s"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(r["ms"], 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": a.dtype, "data": "synthetic",
        "config": {
            "model": model_name, "global_batch": a.batch, "seq_len": capacity, "mean_context": round(r["ctx"], 1),
            "prompt_len": ctx_len, "cache_tokens": engine.scheduler.pool_tokens, "parallelism": "none", "layers": L, "layers_full": full_layers,
            "hidden": D, "heads": H, "kv_heads": KV, "head_dim": hd, "ffn": F, "vocab": V, "page_size": PAGE,
            "rope_theta": cfg["rope_theta"], "rope_factor": cfg["rope_scaling"]["factor"], "norm_eps": cfg["rms_norm_eps"],
            # 2: every matrix is also held in the order the decode products read it (the roofline's bytes count one)
            "weight_copies": 2 if model.packed() else 1,
        },
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(r["gbs"], 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(r["gbs"] * 1e9 / PEAK_HBM, 4)},
        "points": {f"decode_b{b}": round(v["tok_s"], 1) for b, v in results.items() if b != a.batch},
    }
    print(json.dumps(line), flush=True)
    if a.show_choices:
        from fastgen_amd.kernels import linear

        for (what, n, k, rows), name in sorted(linear.choices.items(), key=lambda kv: (kv[0][1], kv[0][2], kv[0][0], kv[0][3])):
            took = ", ".join(f"{c} {1e3 * t:.1f} us" for c, t in sorted(linear.timings.get((what, n, k, rows), {}).items()))
            print(f"[bench] product {what} N={n} K={k} rows<={rows}: {name} ({took})", file=sys.stderr)
    return 0


if __name__ == "__main__":
    sys.exit(main())
