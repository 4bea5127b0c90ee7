// Next-token choice from fp32 logits, one workgroup per row.
//
// Reference semantics (fastgen/generate.py:887-896, utils/sampling.py:6-31):
// greedy = argmax(logits); else probs = softmax(logits / temperature) in fp32
// and, with top_p < 1, the tokens are ranked by probability and a token is
// dropped when the mass ranked before it exceeds top_p; the draw is from the
// rest, un-renormalised weights.  Here nothing is sorted.  With M(x) = sum of
// weights > x, a token is kept iff M(its weight) <= top_p * sum of all weights.
// A draw from the kept tokens is made by rejection: draw from all tokens, take
// the token if it is a kept one (one pass for M of its weight), else draw
// again; the kept tokens hold at least top_p of the mass, so few draws are
// needed.  After FG_SAMPLE_ATTEMPTS rejections the smallest kept weight is
// found by bisection over float bit patterns and the draw is made among the
// kept tokens only.  A draw is an inverse CDF with one uniform number from a
// counter-based generator keyed by (seed, counter, attempt) of the row's
// request, so a request's tokens do not depend on what else is in the batch.
// The CDF runs over the tokens in the order the threads hold them (thread t:
// tokens t, t + 1024, ...), which lets every pass read the row coalesced.
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
__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t counter, uint64_t attempt) {
  const uint64_t z = splitmix64(splitmix64(seed) ^ (counter * 0xD1342543DE82EF95ULL + 1) ^
                                (attempt * 0xA24BAED4963EE407ULL));
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

// Exclusive prefix sum of v over the block's threads in thread order; `total` gets the sum of all.
// The order of additions is fixed by the block size alone.
__device__ __forceinline__ float block_exclusive_scan(float v, float* lds /* SMP_WAVES floats */, float& total) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  float x = v;
#pragma unroll
  for (int d = 1; d < FG_WAVE; d <<= 1) {
    const float o = __shfl_up(x, d, FG_WAVE);
    if (lane >= d) x += o;
  }
  __syncthreads();
  if (lane == FG_WAVE - 1) lds[wave] = x;
  __syncthreads();
  float base = 0.f, all = 0.f;
  for (int i = 0; i < SMP_WAVES; ++i) {
    if (i == wave) base = all;
    all += lds[i];
  }
  total = all;
  return base + x - v;
}

#define FG_SAMPLE_ATTEMPTS 12

__global__ __launch_bounds__(SMP_THREADS) void sample_kernel(
    const float* __restrict__ logits, int ld, int vocab, const float* __restrict__ temperature,
    const float* __restrict__ top_p, const unsigned long long* __restrict__ seeds,
    const unsigned long long* __restrict__ counters, int* __restrict__ out) {
  __shared__ float red_v[SMP_WAVES];
  __shared__ int red_i[SMP_WAVES];
  __shared__ int owner_s, pick_s;
  __shared__ float pick_w_s;
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid % FG_WAVE;
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
  auto weight = [&](float v) { return expf((v - mx) * inv_t); };  // the same bits wherever a token's weight is needed

  // One draw among the tokens of weight >= thresh, given this thread's sum of them, its place in
  // the running sum over the threads, and the sum of all: the thread in whose stretch u falls hands
  // its tokens (t, t + 1024, ...) to its wave, which finds the token.  Every thread gets the token
  // and its weight.
  auto draw = [&](float mine, float before, float total, float thresh, float u01, int& pick, float& pick_w) {
    const float u = u01 * total;
    // the last thread that holds something and starts at or before u (one exists: the first that
    // holds something starts at 0)
    int cand = (mine > 0.f && before <= u) ? tid : -1;
#pragma unroll
    for (int m = FG_WAVE / 2; m > 0; m >>= 1) cand = max(cand, __shfl_xor(cand, m, FG_WAVE));
    __syncthreads();
    if (lane == 0) red_i[tid / FG_WAVE] = cand;
    __syncthreads();
    int owner = -1;
    for (int i = 0; i < SMP_WAVES; ++i) owner = max(owner, red_i[i]);
    if (owner < 0) {  // no thread holds anything (weights that are not numbers): the largest logit
      pick = best_i == 0x7fffffff ? 0 : best_i;
      pick_w = 1.f;
      return;
    }
    if (tid / FG_WAVE == owner / FG_WAVE) {  // the owner's wave, all lanes
      const float start = __shfl(before, owner % FG_WAVE, FG_WAVE);
      float carry = start;
      int found = -1, last_kept = -1;
      float found_w = 0.f, last_w = 0.f;
      for (int k0 = 0; (long long)k0 * SMP_THREADS + owner < vocab && found < 0; k0 += FG_WAVE) {
        const long long i = (long long)(k0 + lane) * SMP_THREADS + owner;
        float w = 0.f;
        if (i < vocab) {
          w = weight(x[i]);
          if (!(w >= thresh)) w = 0.f;
        }
        float inc = w;
#pragma unroll
        for (int d = 1; d < FG_WAVE; d <<= 1) {
          const float o = __shfl_up(inc, d, FG_WAVE);
          if (lane >= d) inc += o;
        }
        const unsigned long long hit = __ballot(w > 0.f && u < carry + inc);
        const unsigned long long kept = __ballot(w > 0.f);
        if (hit) {
          const int l = __ffsll((long long)hit) - 1;
          found = (int)((long long)(k0 + l) * SMP_THREADS + owner);
          found_w = __shfl(w, l, FG_WAVE);
        }
        if (kept) {
          const int l = 63 - __clzll((long long)kept);
          last_kept = (int)((long long)(k0 + l) * SMP_THREADS + owner);
          last_w = __shfl(w, l, FG_WAVE);
        }
        carry += __shfl(inc, FG_WAVE - 1, FG_WAVE);
      }
      if (lane == 0) {  // rounding may put u past the owner's last token: that token then
        pick_s = found >= 0 ? found : last_kept;
        pick_w_s = found >= 0 ? found_w : last_w;
      }
    }
    __syncthreads();
    pick = pick_s;
    pick_w = pick_w_s;
  };

  float mine = 0.f;
  for_each_logit(x, vocab, [&](int, float v) { mine += weight(v); });
  float z;
  const float before = block_exclusive_scan(mine, red_v, z);
  const float p = top_p ? top_p[r] : 1.f;
  const uint64_t seed = seeds[r], counter = counters[r];
  int pick;
  float pick_w;
  if (!(p < 1.f)) {
    draw(mine, before, z, 0.f, uniform01(seed, counter, 0), pick, pick_w);
    if (tid == 0) out[r] = pick;
    return;
  }
  const float budget = p * z;
  for (int attempt = 0; attempt < FG_SAMPLE_ATTEMPTS; ++attempt) {
    draw(mine, before, z, 0.f, uniform01(seed, counter, attempt), pick, pick_w);
    float above = 0.f;  // M(weight of the drawn token)
    for_each_logit(x, vocab, [&](int, float v) {
      const float w = weight(v);
      if (w > pick_w) above += w;
    });
    above = block_sum(above, red_v);
    if (above <= budget) {  // a kept token (uniform over the block)
      if (tid == 0) out[r] = pick;
      return;
    }
  }
  // ---- the smallest kept weight by bisection, then one draw among the kept tokens
  unsigned lo = 0u, hi = __float_as_uint(1.0f);  // M(lo) > budget >= M(hi)
  while (hi - lo > 1u) {
    const unsigned mid = lo + (hi - lo) / 2u;
    const float xm = __uint_as_float(mid);
    float mass = 0.f;
    for_each_logit(x, vocab, [&](int, float v) {
      const float w = weight(v);
      if (w > xm) mass += w;
    });
    mass = block_sum(mass, red_v);
    if (mass <= budget) hi = mid; else lo = mid;
  }
  const float thresh = __uint_as_float(hi);
  float mine_kept = 0.f;
  for_each_logit(x, vocab, [&](int, float v) {
    const float w = weight(v);
    if (w >= thresh) mine_kept += w;
  });
  float total_kept;
  const float before_kept = block_exclusive_scan(mine_kept, red_v, total_kept);
  draw(mine_kept, before_kept, total_kept, thresh, uniform01(seed, counter, FG_SAMPLE_ATTEMPTS), pick, pick_w);
  if (tid == 0) out[r] = pick;
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
