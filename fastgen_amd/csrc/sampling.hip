// Next-token choice from fp32 logits, one workgroup per row.
//
// Reference semantics (fastgen/generate.py:887-896, utils/sampling.py:6-31):
// greedy = argmax(logits); else probs = softmax(logits / temperature) in fp32
// and, with top_p < 1, the tokens are ranked by probability and a token is
// dropped when the mass ranked before it exceeds top_p; the draw is from the
// rest, un-renormalised weights.  Here the kept set is found without a sort:
// with M(x) = sum of weights > x, a token is kept iff M(its weight) <= top_p,
// and the smallest such weight is found by bisection over float bit patterns.
// The draw is an inverse CDF in token-id order with one uniform number from a
// counter-based generator keyed by (seed, counter) of the row's request, so a
// request's tokens do not depend on what else is in the batch.
#include "common.h"

#define SMP_THREADS 1024
#define SMP_WAVES (SMP_THREADS / FG_WAVE)

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ULL;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ULL;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBULL;
  return x ^ (x >> 31);
}

// uniform in [0, 1) with 24 random bits
__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t counter) {
  const uint64_t z = splitmix64(splitmix64(seed) ^ (counter * 0xD1342543DE82EF95ULL + 1));
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// f(i, x[i]) for this thread's share of a row (i = tid, tid + threads, ... in ascending order), with
// eight loads in flight at a time: a row is read by one workgroup, so latency is what it costs.
template <class F>
__device__ __forceinline__ void for_each_logit(const float* __restrict__ x, int vocab, F f) {
  int i = threadIdx.x;
  for (; i + 7 * SMP_THREADS < vocab; i += 8 * SMP_THREADS) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = x[i + u * SMP_THREADS];
#pragma unroll
    for (int u = 0; u < 8; ++u) f(i + u * SMP_THREADS, v[u]);
  }
  for (; i < vocab; i += SMP_THREADS) f(i, x[i]);
}

// (value, index) maximum with the lowest index winning ties; every thread
// gets the result.
__device__ __forceinline__ void block_argmax(float& v, int& idx, float* lds_v, int* lds_i) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
#pragma unroll
  for (int m = FG_WAVE / 2; m > 0; m >>= 1) {
    const float ov = __shfl_xor(v, m, FG_WAVE);
    const int oi = __shfl_xor(idx, m, FG_WAVE);
    if (ov > v || (ov == v && oi < idx)) {
      v = ov;
      idx = oi;
    }
  }
  __syncthreads();
  if (lane == 0) {
    lds_v[wave] = v;
    lds_i[wave] = idx;
  }
  __syncthreads();
  v = lds_v[0];
  idx = lds_i[0];
  for (int i = 1; i < SMP_WAVES; ++i) {
    if (lds_v[i] > v || (lds_v[i] == v && lds_i[i] < idx)) {
      v = lds_v[i];
      idx = lds_i[i];
    }
  }
}

__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
    const float* __restrict__ top_p, const unsigned long long* __restrict__ seeds,
    const unsigned long long* __restrict__ counters, int* __restrict__ out) {
  __shared__ float red_v[SMP_WAVES];
  __shared__ int red_i[SMP_WAVES];
  __shared__ float part[SMP_THREADS];
  __shared__ int owner_s;
  __shared__ float owner_base_s;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)r * ld;

  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for_each_logit(x, vocab, [&](int i, float v) {
    if (v > best) {  // ascending i: the first maximum is kept
      best = v;
      best_i = i;
    }
  });
  block_argmax(best, best_i, red_v, red_i);
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = best_i == 0x7fffffff ? 0 : best_i;
    return;
  }
  const float inv_t = 1.f / temp;
  const float mx = best;
  float z = 0.f;
  for_each_logit(x, vocab, [&](int, float v) { z += expf((v - mx) * inv_t); });
  z = block_sum(z, red_v);

  // ---- nucleus: smallest weight that is kept
  const float p = top_p ? top_p[r] : 1.f;
  float thresh = 0.f;
  if (p < 1.f) {
    const float budget = p * z;
    unsigned lo = 0u, hi = __float_as_uint(1.0f);  // M(lo) > budget >= M(hi)
    while (hi - lo > 1u) {
      const unsigned mid = lo + (hi - lo) / 2u;
      const float xm = __uint_as_float(mid);
      float mass = 0.f;
      for_each_logit(x, vocab, [&](int, float v) {
        const float w = expf((v - mx) * inv_t);
        if (w > xm) mass += w;
      });
      mass = block_sum(mass, red_v);
      if (mass <= budget) hi = mid; else lo = mid;
    }
    thresh = __uint_as_float(hi);
  }

  // ---- inverse CDF over the kept tokens in id order
  const int chunk = (vocab + SMP_THREADS - 1) / SMP_THREADS;
  const int i0 = tid * chunk, i1 = min(vocab, i0 + chunk);
  float mine = 0.f;
  for (int i = i0; i < i1; ++i) {
    const float w = expf((x[i] - mx) * inv_t);
    if (w >= thresh) mine += w;
  }
  part[tid] = mine;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int i = 0; i < SMP_THREADS; ++i) total += part[i];
    const float u = uniform01(seeds[r], counters[r]) * total;
    float cum = 0.f;
    int owner = -1, last_nonempty = 0;
    float base = 0.f, last_base = 0.f;
    for (int i = 0; i < SMP_THREADS; ++i) {
      if (part[i] > 0.f) {
        last_nonempty = i;
        last_base = cum;
        if (u < cum + part[i]) {
          owner = i;
          base = cum;
          break;
        }
      }
      cum += part[i];
    }
    if (owner < 0) {  // rounding put u at or past the total
      owner = last_nonempty;
      base = last_base;
    }
    owner_s = owner;
    owner_base_s = base;
    // u is recomputed by the owner from the same inputs
    part[0] = u;
  }
  __syncthreads();
  if (tid == owner_s) {
    const float u = part[0];
    float cum = owner_base_s;
    int pick = -1, last_kept = best_i;
    for (int i = i0; i < i1; ++i) {
      const float w = expf((x[i] - mx) * inv_t);
      if (w >= thresh) {
        last_kept = i;
        cum += w;
        if (u < cum) {
          pick = i;
          break;
        }
      }
    }
    out[r] = pick >= 0 ? pick : last_kept;
  }
}

// temperature / top_p may be null (greedy / no nucleus); a row whose
// temperature is <= 0 is greedy.
extern "C" int fg_sample(const float* logits, int ld, int n_rows, int vocab,
                         const float* temperature, const float* top_p,
                         const unsigned long long* seeds, const unsigned long long* counters,
                         int* out, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (vocab <= 0 || ld < vocab) return FG_ERR_ARG;
  if (temperature && (!seeds || !counters)) return FG_ERR_ARG;
  sample_kernel<<<n_rows, SMP_THREADS, 0, stream>>>(logits, ld, vocab, temperature, top_p,
                                                    seeds, counters, out);
  return fg_launch_status();
}

// log softmax of the raw logits at one token per row (the reference's
// logprobs: fastgen/generate.py:725-730 uses the un-tempered logits).
__global__ __launch_bounds__(SMP_THREADS) void logprob_kernel(
    const float* __restrict__ logits, int ld, int vocab, const int* __restrict__ tokens,
    float* __restrict__ out) {
  __shared__ float red[SMP_WAVES];
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)r * ld;
  float mx = -INFINITY;
  for_each_logit(x, vocab, [&](int, float v) { mx = fmaxf(mx, v); });
  mx = block_max(mx, red);
  float z = 0.f;
  for_each_logit(x, vocab, [&](int, float v) { z += expf(v - mx); });
  z = block_sum(z, red);
  if (tid == 0) {
    int tok = tokens[r];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    out[r] = x[tok] - mx - logf(z);
  }
}

extern "C" int fg_logprob(const float* logits, int ld, int n_rows, int vocab, const int* tokens,
                          float* out, hipStream_t stream) {
  if (n_rows <= 0) return FG_OK;
  if (vocab <= 0 || ld < vocab) return FG_ERR_ARG;
  logprob_kernel<<<n_rows, SMP_THREADS, 0, stream>>>(logits, ld, vocab, tokens, out);
  return fg_launch_status();
}
