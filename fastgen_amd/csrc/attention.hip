// Paged causal attention over the cache, general form: any element type,
// any head size that is a multiple of 8 up to 512, any number of heads and
// groups, any page size that is a multiple of 8.  One wavefront computes one
// (query token, query head) from key 0 (or the window's first key) to the
// token's own position, in tiles of 64 keys that start at multiples of 64.
// The arithmetic for a (token, head) therefore depends on nothing but that
// token's keys: not on the batch, on how the prompt was cut, or on which
// pages hold the keys.  This is the kernel of the 32-bit path and the
// fallback of the bf16 path for shapes the MFMA kernel refuses.
//
// Semantics (fastgen/forward.py:176-258): query at position p of sequence b
// sees keys 0..p of b through block_table[b]; scores (q.k)*scale, softmax in
// fp32, o = P.V; query head h reads kv head h / (H/KV).  With window > 0 only
// keys p-window+1..p are seen.
#include "common.h"
#include "kv_layout.h"

#define ATT_WAVES 4
#define ATT_TILE 64
#define ATT_MAX_HD 512

template <class T> struct Vec8;
template <> struct Vec8<float> {
  float v[8];
  __device__ __forceinline__ void load(const float* p) {
    const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
};
template <> struct Vec8<bf16_t> {
  float v[8];
  __device__ __forceinline__ void load(const bf16_t* p) {
    const uint4 raw = *(const uint4*)p;
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

template <class T>
__global__ __launch_bounds__(ATT_WAVES* FG_WAVE) void paged_attention_general_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages,
    const int* __restrict__ block_table, int bt_stride, const int* __restrict__ seq_of_token,
    const int* __restrict__ positions, int n_tokens, int n_heads, int n_kv, int hd,
    int page_size, float scale, int window) {
  __shared__ float q_s[ATT_WAVES][ATT_MAX_HD];
  __shared__ float p_s[ATT_WAVES][ATT_TILE];
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const long long item = (long long)blockIdx.x * ATT_WAVES + wave;
  if (item >= (long long)n_tokens * n_heads) return;  // whole wave leaves; no block barrier below
  const int t = (int)(item / n_heads), h = (int)(item % n_heads);
  const int kvh = h / (n_heads / n_kv);
  const int seq = seq_of_token[t];
  const int pos = positions[t];
  const int* table = block_table + (size_t)seq * bt_stride;
  const int first = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
  const KvLayout lay(page_size, hd);
  const size_t head_elems = (size_t)page_size * hd;

  const T* qrow = q + (size_t)t * q_stride + (size_t)h * hd;
  float* qs = q_s[wave];
  float* ps = p_s[wave];
  for (int d = lane; d < hd; d += FG_WAVE) qs[d] = to_f<T>(qrow[d]);
  __builtin_amdgcn_wave_barrier();

  constexpr int MAXD = ATT_MAX_HD / FG_WAVE;  // head dims owned by a lane
  float o[MAXD];
#pragma unroll
  for (int i = 0; i < MAXD; ++i) o[i] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int kb = (first / ATT_TILE) * ATT_TILE; kb <= pos; kb += ATT_TILE) {
    // ---- scores: lane j owns key kb + j
    const int key = kb + lane;
    const bool valid = key >= first && key <= pos;
    float s = -INFINITY;
    if (valid) {
      const int page = table[key / page_size];
      const T* khead = k_pages + ((size_t)page * n_kv + kvh) * head_elems;
      const int kappa = key % page_size;
      float acc = 0.f;
      for (int d = 0; d < hd; d += 8) {
        Vec8<T> kv;
        kv.load(khead + lay.k_off(kappa, d));
#pragma unroll
        for (int e = 0; e < 8; ++e) acc += qs[d + e] * kv.v[e];
      }
      s = acc * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // m = -inf on the first tile: alpha = 0
    l = l * alpha + wave_sum(p);
    m = m_new;
    __builtin_amdgcn_wave_barrier();
    ps[lane] = p;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < MAXD; ++i) o[i] *= alpha;
    // ---- o += P.V: lane owns head dims lane, lane+64, ...; one stored chunk
    // of eight key slots at a time (one page; with the permuted order the
    // slots of chunk g of a 32-key group are keys 4g..4g+3 and 16+4g..16+4g+3)
    for (int q = 0; q < ATT_TILE / 8; ++q) {
      const int base = lay.permuted ? kb + 32 * (q / 4) + 4 * (q % 4) : kb + 8 * q;  // lowest key of the chunk
      const int stride_hi = lay.permuted ? 12 : 0;  // slots 4..7 are 16 keys on (4 + 12)
      if (base > pos) { if (lay.permuted) continue; else break; }
      if (base + 7 + stride_hi < first) continue;
      const int page = table[base / page_size];
      const T* vhead = v_pages + ((size_t)page * n_kv + kvh) * head_elems;
      const int kc = lay.v_slot(base % page_size) / 8;
#pragma unroll
      for (int i = 0; i < MAXD; ++i) {
        const int d = lane + i * FG_WAVE;
        if (d < hd) {
          Vec8<T> vv;
          vv.load(vhead + lay.v_chunk_off(kc, d));
          float acc = o[i];
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int kk = base + e + (e >= 4 ? stride_hi : 0);
            // select, not multiply: a slot never written may hold NaN
            if (kk >= first && kk <= pos) acc += ps[kk - kb] * vv.v[e];
          }
          o[i] = acc;
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  T* orow = out + (size_t)t * out_stride + (size_t)h * hd;
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < MAXD; ++i) {
    const int d = lane + i * FG_WAVE;
    if (d < hd) orow[d] = from_f<T>(o[i] * inv);
  }
}

extern "C" int fg_paged_attention_general(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pages,
    const void* v_pages, const int* block_table, int bt_stride, const int* seq_of_token,
    const int* positions, int n_tokens, int n_heads, int n_kv, int hd, int page_size,
    float scale, int window, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (hd <= 0 || hd % 8 || hd > ATT_MAX_HD || page_size <= 0 || page_size % 8 || n_kv <= 0 ||
      n_heads <= 0 || n_heads % n_kv || window < 0)
    return FG_ERR_ARG;
  const long long items = (long long)n_tokens * n_heads;
  const long long blocks = (items + ATT_WAVES - 1) / ATT_WAVES;
  if (blocks > 2147483647LL) return FG_ERR_ARG;
  dim3 grid((unsigned)blocks);
  if (dtype == FG_F32)
    paged_attention_general_kernel<float><<<grid, ATT_WAVES * FG_WAVE, 0, stream>>>(
        (const float*)q, q_stride, (float*)out, out_stride, (const float*)k_pages,
        (const float*)v_pages, block_table, bt_stride, seq_of_token, positions, n_tokens,
        n_heads, n_kv, hd, page_size, scale, window);
  else if (dtype == FG_BF16)
    paged_attention_general_kernel<bf16_t><<<grid, ATT_WAVES * FG_WAVE, 0, stream>>>(
        (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pages,
        (const bf16_t*)v_pages, block_table, bt_stride, seq_of_token, positions, n_tokens,
        n_heads, n_kv, hd, page_size, scale, window);
  else
    return FG_ERR_ARG;
  return fg_launch_status();
}
