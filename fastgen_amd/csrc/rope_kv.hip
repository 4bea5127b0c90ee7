// Rotary position encoding of q and k and the write of k, v into the paged
// cache, in one launch (the reference issues four: fastgen/forward.py:449-460
// with kernels/rope.py and kernels/paged_memcpy.py).
//
// Rotation (kernels/rope.py:56-89): pair (x[2i], x[2i+1]) of a head, angle =
// float(pos) * freqs[i] in fp32, precise sin/cos,
//   x[2i] = a cos - b sin,  x[2i+1] = b cos + a sin,
// rounded once at the store.  Pairs beyond rotary_dim are left as they are.
//
// Cache layout, per cache layer: K pages [n_pages, KV, P*hd], V pages
// [n_pages, KV, hd*P], the elements inside a page ordered as kv_layout.h
// says (16-byte chunks placed for the matrix-core kernels; V transposed).  A
// token's place is slot = page*P + offset; a negative slot means "write
// nothing".
#include "common.h"
#include "kv_layout.h"

#define ROPE_THREADS 256

// cos and sin of float(pos) * freqs[i] for every token of the step, computed
// once and shared by all layers: table[(t * n_freqs + i) * 2 + {0, 1}].
__global__ __launch_bounds__(ROPE_THREADS) void rope_table_kernel(
    const int* __restrict__ positions, const float* __restrict__ freqs, float* __restrict__ table,
    int n_tokens, int n_freqs) {
  const int e = blockIdx.x * ROPE_THREADS + threadIdx.x;
  if (e >= n_tokens * n_freqs) return;
  const float ang = (float)positions[e / n_freqs] * freqs[e % n_freqs];
  table[2 * e] = cosf(ang);
  table[2 * e + 1] = sinf(ang);
}

extern "C" int fg_rope_table(const int* positions, const float* freqs, float* table, int n_tokens,
                             int n_freqs, hipStream_t stream) {
  if (n_tokens <= 0 || n_freqs <= 0) return FG_OK;
  const long long n = (long long)n_tokens * n_freqs;
  if (n > 2147483647LL) return FG_ERR_ARG;
  rope_table_kernel<<<(unsigned)((n + ROPE_THREADS - 1) / ROPE_THREADS), ROPE_THREADS, 0, stream>>>(
      positions, freqs, table, n_tokens, n_freqs);
  return fg_launch_status();
}

template <class T>
__global__ __launch_bounds__(ROPE_THREADS) void rope_kv_write_kernel(
    T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
    const float* __restrict__ freqs, const float* __restrict__ table, const int* __restrict__ slots,
    T* __restrict__ k_pages,
    T* __restrict__ v_pages, int n_heads, int n_kv, int hd, int rotary_dim, int page_size,
    int write_kv) {
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * row_stride;
  const float pos = (float)positions[t];
  const int half = hd / 2;
  const int slot = write_kv ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const KvLayout lay(page_size, hd);
  const size_t head_elems = (size_t)page_size * hd;

  // q heads then k heads: (n_heads + n_kv) * hd/2 pairs
  const int n_rot_heads = n_heads + (write_kv ? n_kv : 0);
  const int n_pairs = n_rot_heads * half;
  for (int p = threadIdx.x; p < n_pairs; p += ROPE_THREADS) {
    const int head = p / half, i = p % half;
    T* x = row + (size_t)head * hd + 2 * i;
    float a = to_f<T>(x[0]), b = to_f<T>(x[1]);
    if (2 * i < rotary_dim) {
      float s, c;
      if (table) {
        c = table[((size_t)t * (rotary_dim / 2) + i) * 2];
        s = table[((size_t)t * (rotary_dim / 2) + i) * 2 + 1];
      } else {
        const float ang = pos * freqs[i];
        s = sinf(ang);
        c = cosf(ang);
      }
      const float ra = a * c - b * s;
      const float rb = b * c + a * s;
      a = ra;
      b = rb;
    }
    if (head < n_heads) {
      x[0] = from_f<T>(a);
      x[1] = from_f<T>(b);
    } else if (slot >= 0) {
      const int kvh = head - n_heads;
      T* dst = k_pages + ((size_t)page * n_kv + kvh) * head_elems + lay.k_off(off, 2 * i);
      dst[0] = from_f<T>(a);
      dst[1] = from_f<T>(b);
    }
  }
  if (slot >= 0) {
    const T* v = row + (size_t)(n_heads + n_kv) * hd;
    for (int e = threadIdx.x; e < n_kv * hd; e += ROPE_THREADS) {
      const int kvh = e / hd, d = e % hd;
      v_pages[((size_t)page * n_kv + kvh) * head_elems + lay.v_off(off, d)] = v[e];
    }
  }
}

// The same with eight consecutive elements (four pairs) a thread; for
// hd % 8 == 0, rotary_dim % 8 == 0 and rows 16-byte aligned.
template <class T>
__global__ __launch_bounds__(ROPE_THREADS) void rope_kv_write_vec_kernel(
    T* __restrict__ qkv, int row_stride, const int* __restrict__ positions,
    const float* __restrict__ freqs, const float* __restrict__ table, const int* __restrict__ slots,
    T* __restrict__ k_pages,
    T* __restrict__ v_pages, int n_heads, int n_kv, int hd, int rotary_dim, int page_size,
    int write_kv) {
  const int t = blockIdx.x;
  T* row = qkv + (size_t)t * row_stride;
  const float pos = (float)positions[t];
  const int slot = write_kv ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0;
  const int off = slot >= 0 ? slot % page_size : 0;
  const KvLayout lay(page_size, hd);
  const size_t head_elems = (size_t)page_size * hd;
  const int cph = hd / 8;  // chunks per head
  const int n_rot = (n_heads + (write_kv ? n_kv : 0)) * cph;
  for (int w = threadIdx.x; w < n_rot; w += ROPE_THREADS) {
    {
      const int head = w / cph, c = w % cph;
      if (head >= n_heads && slot < 0) continue;
      T* x = row + (size_t)head * hd + 8 * c;
      float v[8];
      load8<T>(x, v);
      if (8 * c < rotary_dim) {
        float cs4[8];  // cos, sin of the chunk's four pairs
        if (table) {
          load8<float>(table + ((size_t)t * (rotary_dim / 2) + 4 * c) * 2, cs4);
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float ang = pos * freqs[4 * c + j];
            cs4[2 * j] = cosf(ang);
            cs4[2 * j + 1] = sinf(ang);
          }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float cs = cs4[2 * j], sn = cs4[2 * j + 1];
          const float a = v[2 * j], b = v[2 * j + 1];
          v[2 * j] = a * cs - b * sn;
          v[2 * j + 1] = b * cs + a * sn;
        }
      }
      if (head < n_heads)
        store8<T>(x, v);
      else
        store8<T>(k_pages + ((size_t)page * n_kv + (head - n_heads)) * head_elems + lay.k_off(off, 8 * c), v);
    }
  }
  if (slot >= 0) {
    // v: one element a thread, consecutive threads consecutive head dims: in the transposed page
    // these lie 16 bytes apart, so a wave's store stays within a few cache lines
    const T* v = row + (size_t)(n_heads + n_kv) * hd;
    for (int e = threadIdx.x; e < n_kv * hd; e += ROPE_THREADS) {
      const int kvh = e / hd, d = e % hd;
      v_pages[((size_t)page * n_kv + kvh) * head_elems + lay.v_off(off, d)] = v[e];
    }
  }
}

// qkv: [n_tokens, row_stride] with q heads, then k heads, then v heads in a
// row.  With write_kv == 0 only q is rotated (a mixer that reads another
// layer's cache).
// `table` (from fg_rope_table, for the same positions) replaces the sin/cos
// of `freqs` when given.
extern "C" int fg_rope_kv_write(void* qkv, int row_stride, const int* positions,
                                const float* freqs, const float* table, const int* slots, void* k_pages,
                                void* v_pages, int n_tokens, int n_heads, int n_kv, int hd,
                                int rotary_dim, int page_size, int write_kv, int dtype,
                                hipStream_t stream) {
  if (n_tokens <= 0) return FG_OK;
  if (hd <= 0 || hd % 2 || rotary_dim < 0 || rotary_dim > hd || rotary_dim % 2 ||
      page_size <= 0 || n_heads <= 0 || n_kv < 0)
    return FG_ERR_ARG;
  if (write_kv && (hd % 8 || page_size % 8)) return FG_ERR_ARG;  // the page layout is in chunks of 8
  if (row_stride < (n_heads + (write_kv ? 2 * n_kv : 0)) * hd) return FG_ERR_ARG;
  const bool vec = hd % 8 == 0 && rotary_dim % 8 == 0 && row_stride % 8 == 0;
#define LAUNCH(T, KERNEL)                                                                         \
  KERNEL<T><<<n_tokens, ROPE_THREADS, 0, stream>>>((T*)qkv, row_stride, positions, freqs, table,  \
                                                   slots, (T*)k_pages, (T*)v_pages, n_heads, n_kv, \
                                                   hd, rotary_dim, page_size, write_kv)
  if (dtype == FG_F32) {
    if (vec) LAUNCH(float, rope_kv_write_vec_kernel); else LAUNCH(float, rope_kv_write_kernel);
  } else if (dtype == FG_BF16) {
    if (vec) LAUNCH(bf16_t, rope_kv_write_vec_kernel); else LAUNCH(bf16_t, rope_kv_write_kernel);
  } else {
    return FG_ERR_ARG;
  }
#undef LAUNCH
  return fg_launch_status();
}
