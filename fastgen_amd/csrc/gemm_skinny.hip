// y = x W^T for few rows of x (decode: M <= 128), bf16 operands, fp32
// accumulation on the matrix cores.  The work is streaming W once from HBM,
// so the kernel is built around keeping many 16-byte loads of W in flight:
//
//  * a workgroup owns 16 rows of W (16 output columns); its waves split K,
//    each wave walks its K range with v_mfma_f32_16x16x32_bf16 taking W as
//    the A operand (16 rows x 32 k) and x^T as B (32 k x 16 rows of x), eight
//    k steps unrolled so that 8 loads of W per lane are in flight; x (a few
//    KB per k range) comes from the caches;
//  * the waves' partial 16x16 tiles are added in LDS in wave order, so a
//    result does not depend on timing;
//  * the epilogue stores bf16 or fp32, or, for a gate/up matrix whose rows are
//    interleaved in groups of 8 (8 gate rows, then their 8 up rows), stores
//    silu(gate) * up directly: the gate/up activations never reach memory.
//
// Replaces the library product of fastgen/forward.py:433-513 where M is small.
//
// W comes row by row (ldw = elements between rows), or packed (ldw = 0): in blocks of 16 rows x 32 k
// of 1 KB, each in the order in which a wave's lanes hold an MFMA operand (lane 16 g + r: row r, k
// 8 g .. 8 g + 7), the blocks of 16 rows one after the other along k, rows and k padded with zeros to
// whole blocks: [ceil(N / 16)][ceil(K / 32)][64][8].  A wave's load of an operand is then 1 KB of
// whole cache lines, and its eight loads of a pass 8 KB in a row; from rows it is 16 pieces of 64
// bytes, half a cache line each, whose other halves the next load asks for again: the kernels here
// are bound by the number of such requests, not by the bytes.
#include "common.h"
#include "kv_layout.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// Where a lane finds its 16 bytes of W for the 16 rows from n0 on: at base + (k / 32) * step for the
// k step of 32 that begins at k (a multiple of 32).  A lane whose chunk lies beyond the k range loads
// `safe` instead (every load is issued, none is conditional) and zeroes what it got.
struct WSrc {
  const bf16_t* base;
  const bf16_t* safe;
  int step;
  __device__ __forceinline__ const bf16x8* at(int k, bool in) const {
    return (const bf16x8*)(in ? base + (size_t)(k >> 5) * step : safe);
  }
};
__device__ __forceinline__ WSrc w_src(const bf16_t* w, int ldw, int n0, int N, int K, int lane) {
  if (ldw) {  // rows are clamped, not skipped: what they give is not stored
    const bf16_t* row = w + (size_t)min(n0 + (lane & 15), N - 1) * ldw;
    return WSrc{row + 8 * (lane >> 4), row, 32};
  }
  const bf16_t* block = w + ((size_t)min(n0 >> 4, (N - 1) >> 4) * ((K + 31) >> 5) * 64 + lane) * 8;
  return WSrc{block, block, 512};
}

#define EPI_STORE 0
#define EPI_SILU_MUL 1
#define EPI_ROPE_KV 2  // w = [q; k; v] projections: rotate q and k, q to y, k and v into their cache pages
#define EPI_RESIDUAL 3  // the product is added to the fp32 residual stream; see Residual

// For at most 16 rows the two RMSNorms of a layer need no kernels of their own.  The product that
// feeds the residual stream (EPI_RESIDUAL) adds its result to h, stores h * norm_w (not yet divided by
// the row's root mean square) as the next product's x, and one sum of squares of h per row and
// workgroup.  The next product (RowScale) adds those sums up, in a fixed order, and multiplies its
// result rows by rsqrt(mean + eps): W (x' * r) = r * (W x').  x' is rounded to bfloat16 as the normed
// row would be, to the same relative error.
struct RowScale {
  const float* ssq;  // [M, n_parts] sums of squares whose sum over n_parts is the row's; null: rows are taken as they are
  int n_parts;
  float inv_dim, eps;
};
struct Residual {
  float* h;             // [M, N] fp32 residual stream, updated in place
  int ldh;
  const void* norm_w;   // [N] weight of the norm that follows
  int norm_w_f32;       // its dtype: fp32 or bf16
  bf16_t* x_out;        // [M, N] h * norm_w
  int ldxo;
  float* ssq_out;       // [M, gridDim.x]
};

// The sum of a row's partial sums of squares is taken by 1/16 of the workgroup's threads: each adds up
// a strided share early (eight loads in flight at a time, issued before the product's own, so that
// their latency passes during the product), the shares are added in the end.
template <int THREADS>
__device__ __forceinline__ float row_scale_begin(const RowScale& sc, int M) {
  constexpr int TPR = THREADS / 16;
  const int m = min((int)threadIdx.x / TPR, M - 1), sub = threadIdx.x % TPR;
  float s = 0.f;
  if (sc.ssq) {  // uniform
    const float* row = sc.ssq + (size_t)m * sc.n_parts;
    for (int p0 = 0; p0 < sc.n_parts; p0 += 8 * TPR) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = row[min(p0 + sub + j * TPR, sc.n_parts - 1)];  // never conditional
#pragma unroll
      for (int j = 0; j < 8; ++j) s += p0 + sub + j * TPR < sc.n_parts ? v[j] : 0.f;
    }
  }
  return s;
}
template <int THREADS>
__device__ __forceinline__ void row_scale_end(const RowScale& sc, float part, float* rscale /* LDS [16] */) {
  constexpr int TPR = THREADS / 16;  // 16 or 32: the threads of a row are neighbours in one wave
#pragma unroll
  for (int w = TPR / 2; w > 0; w >>= 1) part += __shfl_xor(part, w, FG_WAVE);
  if (threadIdx.x % TPR == 0) rscale[threadIdx.x / TPR] = sc.ssq ? rsqrtf(part * sc.inv_dim + sc.eps) : 1.f;
}

// EPI_RESIDUAL for one 16 x 16 tile whose waves' partial sums lie in red[WAVES][256] (row m, column c at
// m * 16 + c): the first 256 threads take an element each.  What they need from memory (h and the
// norm's weight at their element) is asked for before the product (residual_begin), so that the
// epilogue does not wait for it.
struct ResidualRegs { float h, w; };
__device__ __forceinline__ ResidualRegs residual_begin(const Residual& rs, int n0, int M, int N) {
  ResidualRegs r{0.f, 0.f};
  const int e = threadIdx.x;
  if (e < 256) {  // whole waves
    const int m = min(e >> 4, M - 1), n = min(n0 + (e & 15), N - 1);
    r.h = rs.h[(size_t)m * rs.ldh + n];
    r.w = rs.norm_w_f32 ? ((const float*)rs.norm_w)[n] : (float)((const bf16_t*)rs.norm_w)[n];
  }
  return r;
}
template <int WAVES>
__device__ __forceinline__ void residual_epilogue(const float (*red)[256], const float* rscale, const Residual& rs,
                                                  const ResidualRegs& pre, int n0, int M, int N) {
  const int e = threadIdx.x;
  if (e >= 256) return;  // (whole waves)
  const int m = e >> 4, c = e & 15, n = n0 + c;
  float s = 0.f;
#pragma unroll
  for (int wv = 0; wv < WAVES; ++wv) s += red[wv][e];
  float sq = 0.f;
  if (m < M && n < N) {
    const float hv = pre.h + s * rscale[m];
    rs.h[(size_t)m * rs.ldh + n] = hv;
    rs.x_out[(size_t)m * rs.ldxo + n] = (bf16_t)(hv * pre.w);
    sq = hv * hv;
  }
  // the 16 columns of a row are 16 neighbouring lanes
#pragma unroll
  for (int w = 8; w > 0; w >>= 1) sq += __shfl_xor(sq, w, FG_WAVE);
  if (c == 0 && m < M) rs.ssq_out[(size_t)m * gridDim.x + blockIdx.x] = sq;
}

// What the EPI_ROPE_KV epilogue needs beside the product (rope_kv.hip does the same as a kernel of
// its own for steps with more rows).
struct RopeKv {
  const float* table;  // [M, rotary_dim/2, 2] cos, sin of each row's position; null: no rotation
  const int* slots;    // [M] page * page_size + offset of each row's token; < 0: keep k, v out of the cache
  bf16_t* k_pages;
  bf16_t* v_pages;
  int n_heads, n_kv, hd, rotary_dim, page_size;
};

__device__ __forceinline__ bf16x8 gs_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

template <int MB, int WAVES, int EPI, class TY>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(
    const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw, TY* __restrict__ y,
    int ldy, int M, int N, int K, RowScale sc, Residual rs) {
  constexpr int U = MB <= 2 ? 8 : 4;  // k steps in flight
  __shared__ float red[WAVES][MB * 256];
  __shared__ float rscale[16];
  static_assert(EPI != EPI_RESIDUAL || MB == 1, "the residual epilogue is for at most 16 rows");
  const float sc_part = MB == 1 ? row_scale_begin<WAVES * 64>(sc, M) : 0.f;
  ResidualRegs pre{0.f, 0.f};
  if (EPI == EPI_RESIDUAL) pre = residual_begin(rs, blockIdx.x * 16, M, N);
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const WSrc ws = w_src(w, ldw, n0, N, K, lane);
  const bf16_t* xrow[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) xrow[mb] = x + (size_t)min(16 * mb + r16, M - 1) * ldx;

  const int kw = ((K + WAVES * 32 - 1) / (WAVES * 32)) * 32;  // k per wave
  const int k_begin = min(K, wave * kw), k_end = min(K, k_begin + kw);
  f32x4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kk = k_begin; kk < k_end; kk += 32 * U) {
    bf16x8 a[U], b[U][MB];
    // all loads first, unconditional (addresses clamped), so that they are issued together
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = kk + 32 * u + 8 * g;
      const bool in = k < k_end;  // K % 8 == 0: a chunk is inside or outside as a whole
      const int kc = in ? k : k_begin;
      const bf16x8 av = *ws.at(kk + 32 * u, in);
      a[u] = in ? av : gs_zero8();
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) b[u][mb] = *(const bf16x8*)(xrow[mb] + kc);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mb], acc[mb], 0, 0, 0);
  }
  // acc[mb][i] = C[n = 4g + i][m = 16 mb + r16]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) *(f32x4*)(&red[wave][(mb * 16 + r16) * 16 + 4 * g]) = acc[mb];
  if (MB == 1) row_scale_end<WAVES * 64>(sc, sc_part, rscale);
  __syncthreads();
  if (EPI == EPI_RESIDUAL) {
    if constexpr (MB == 1) residual_epilogue<WAVES>(red, rscale, rs, pre, n0, M, N);
  } else if (EPI == EPI_STORE) {
    for (int e = threadIdx.x; e < MB * 256; e += WAVES * 64) {
      float s = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) s += red[wv][e];
      const int m = e >> 4, n = n0 + (e & 15);
      if (MB == 1) s *= rscale[m];
      if (m < M && n < N) y[(size_t)m * ldy + n] = from_f<TY>(s);
    }
  } else {
    // rows n0 .. n0+7 are gate rows j0 .. j0+7, rows n0+8 .. n0+15 their up rows; j0 = n0 / 2
    for (int e = threadIdx.x; e < MB * 128; e += WAVES * 64) {
      const int m = e >> 3, j = e & 7;
      float gate = 0.f, up = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) {
        gate += red[wv][m * 16 + j];
        up += red[wv][m * 16 + 8 + j];
      }
      if (MB == 1) {
        gate *= rscale[m];
        up *= rscale[m];
      }
      const int col = n0 / 2 + j;
      if (m < M && n0 + 8 + j < N) y[(size_t)m * ldy + col] = from_f<TY>(gate / (1.f + __expf(-gate)) * up);
    }
  }
}

// The same for at most 16 rows of x with x going through LDS: a lane of an
// MFMA operand row group reads 16 different rows of x, which from memory is 16
// cache lines for 256 bytes; instead the wave copies its 16 x 256 slice of x
// for the next 8 k steps with whole-row loads into LDS, chunk-major, and reads
// the operands from there (the 16 lanes then read 256 contiguous bytes).  Row r
// of chunk c sits in slot r ^ (c & 15) of the chunk: the 16 lanes that store one
// row's consecutive chunks would otherwise all hit the same banks (a chunk is
// 256 bytes, the width of all banks).
template <int WAVES, int EPI, class TY>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny16_kernel(
    const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw, TY* __restrict__ y,
    int ldy, int M, int N, int K, RopeKv rk, RowScale sc, Residual rs) {
  constexpr int U = 8;
  __shared__ float red[WAVES][256];
  __shared__ float rscale[16];
  const float sc_part = row_scale_begin<WAVES * 64>(sc, M);
  ResidualRegs pre{0.f, 0.f};
  if (EPI == EPI_RESIDUAL) pre = residual_begin(rs, blockIdx.x * 16, M, N);
  __shared__ __attribute__((aligned(16))) bf16_t xs[WAVES][4 * U * 16 * 8];  // [k chunk][row][8]
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const WSrc ws = w_src(w, ldw, n0, N, K, lane);
  const int kw = ((K + WAVES * 32 - 1) / (WAVES * 32)) * 32;
  const int k_begin = min(K, wave * kw), k_end = min(K, k_begin + kw);
  // copying x: a row's 256 k of one iteration are 32 chunks = 32 lanes; a load covers 2 rows
  const int c_row = lane >> 5, c_chunk = lane & 31;
  const int x_loads = (M + 1) / 2;
  bf16_t* my_xs = xs[wave];
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int kk = k_begin; kk < k_end; kk += 32 * U) {
    bf16x8 a[U], xv[8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = kk + 32 * u + 8 * g;
      const bool in = k < k_end;
      const bf16x8 av = *ws.at(kk + 32 * u, in);
      a[u] = in ? av : gs_zero8();
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j < x_loads) {  // uniform
        const int row = min(2 * j + c_row, M - 1), k = kk + 8 * c_chunk;
        xv[j] = *(const bf16x8*)(x + (size_t)row * ldx + (k < k_end ? k : k_begin));
      }
    }
    __builtin_amdgcn_wave_barrier();  // the reads of the previous iteration are done (same wave, in order)
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (j < x_loads) *(bf16x8*)(my_xs + (c_chunk * 16 + ((2 * j + c_row) ^ (c_chunk & 15))) * 8) = xv[j];
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bf16x8 b = *(const bf16x8*)(my_xs + ((4 * u + g) * 16 + (r16 ^ ((4 * u + g) & 15))) * 8);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b, acc, 0, 0, 0);
    }
  }
  *(f32x4*)(&red[wave][r16 * 16 + 4 * g]) = acc;
  row_scale_end<WAVES * 64>(sc, sc_part, rscale);
  __syncthreads();
  if (EPI == EPI_RESIDUAL) {
    residual_epilogue<WAVES>(red, rscale, rs, pre, n0, M, N);
  } else if (EPI == EPI_ROPE_KV) {
    // 16 columns = 8 pairs of one head of q, k or v (head sizes are multiples of 16)
    for (int e = threadIdx.x; e < 128; e += WAVES * 64) {
      const int m = e >> 3, p = e & 7, n = n0 + 2 * p;
      if (m >= M || n >= N) continue;
      float a = 0.f, b = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) {
        a += red[wv][m * 16 + 2 * p];
        b += red[wv][m * 16 + 2 * p + 1];
      }
      a *= rscale[m];
      b *= rscale[m];
      const int q_cols = rk.n_heads * rk.hd, k_cols = rk.n_kv * rk.hd;
      const int d = n % rk.hd;
      if (n < q_cols + k_cols && rk.table && d < rk.rotary_dim) {
        const float cs = rk.table[((size_t)m * (rk.rotary_dim / 2) + d / 2) * 2];
        const float sn = rk.table[((size_t)m * (rk.rotary_dim / 2) + d / 2) * 2 + 1];
        const float ra = a * cs - b * sn, rb = b * cs + a * sn;
        a = ra;
        b = rb;
      }
      typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
      if (n < q_cols) {
        bf16x2_t v2 = {(__bf16)a, (__bf16)b};
        *(bf16x2_t*)((bf16_t*)y + (size_t)m * ldy + n) = v2;
        continue;
      }
      const int slot = rk.slots[m];
      if (slot < 0) continue;
      const KvLayout lay(rk.page_size, rk.hd);
      const int page = slot / rk.page_size, off = slot % rk.page_size;
      const size_t head_elems = (size_t)rk.page_size * rk.hd;
      if (n < q_cols + k_cols) {
        const int kvh = (n - q_cols) / rk.hd;
        bf16x2_t v2 = {(__bf16)a, (__bf16)b};
        *(bf16x2_t*)(rk.k_pages + ((size_t)page * rk.n_kv + kvh) * head_elems + lay.k_off(off, d)) = v2;
      } else {
        const int kvh = (n - q_cols - k_cols) / rk.hd;
        bf16_t* vh = rk.v_pages + ((size_t)page * rk.n_kv + kvh) * head_elems;
        vh[lay.v_off(off, d)] = (bf16_t)a;
        vh[lay.v_off(off, d + 1)] = (bf16_t)b;
      }
    }
  } else if (EPI == EPI_STORE) {
    for (int e = threadIdx.x; e < 256; e += WAVES * 64) {
      float s = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) s += red[wv][e];
      const int m = e >> 4, n = n0 + (e & 15);
      s *= rscale[m];
      if (m < M && n < N) y[(size_t)m * ldy + n] = from_f<TY>(s);
    }
  } else {
    for (int e = threadIdx.x; e < 128; e += WAVES * 64) {
      const int m = e >> 3, j = e & 7;
      float gate = 0.f, up = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) {
        gate += red[wv][m * 16 + j];
        up += red[wv][m * 16 + 8 + j];
      }
      gate *= rscale[m];
      up *= rscale[m];
      if (m < M && n0 + 8 + j < N) y[(size_t)m * ldy + n0 / 2 + j] = from_f<TY>(gate / (1.f + __expf(-gate)) * up);
    }
  }
}

// More rows of x (17..128): a workgroup owns 64 rows of W, one 16-row block a
// wave over the whole k range of the workgroup, so nothing is reduced across
// waves; the workgroup's slice of x for the next 8 k steps (MB*16 rows x 256)
// goes through LDS once for all four waves.  blockIdx.y cuts K: split s adds
// rows k in [s*k_per_split, ...) and stores its partial sums at y + s *
// part_stride (fp32); the consumer adds the partials in split order.
// U: k steps of 32 a pass of the loop (8; 4 halves the x slice in LDS, which measured no faster at 64 rows).
// The x slice has one buffer in LDS (two barriers a pass) and the kernel is held to 170 registers, so that a
// compute unit holds three workgroups and their loads of W in flight: the gate/up product at 64 rows measured
// 58.5 us so against 63.5 with two buffers and two workgroups (four workgroups would need 128 registers: spills).
// Above 64 rows (five to eight blocks of x: two workgroups a compute unit) every wave reads eight blocks of x from
// LDS for each 16 rows of W, which bounds it: worth it where the k range is cut (down and o projections at 128
// rows of the 8B shape 46 / 18 us against the library's 76 / 24), not for wide outputs (gate/up 75 against 55).
template <int MB, int U, int EPI, class TY>
__global__ __launch_bounds__(256, MB <= 4 ? 3 : 2) void gemm_skinny64_kernel(
    const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw, TY* __restrict__ y,
    int ldy, size_t part_stride, int M, int N, int K, int k_per_split, RowScale sc) {
  // [k chunk][row][8]; row r of chunk c in slot r ^ (c & 15) of its block of 16 (bank conflicts, as above)
  __shared__ __attribute__((aligned(16))) bf16_t xs[4 * U * MB * 16 * 8];
  __shared__ float rscale[16];  // with sc (one block of x only): the rows' factors of a norm folded into this product
  const float sc_part = MB == 1 ? row_scale_begin<256>(sc, M) : 0.f;
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * 64 + wave * 16;
  const WSrc ws = w_src(w, ldw, n0, N, K, lane);
  const int k_begin = min(K, (int)blockIdx.y * k_per_split), k_end = min(K, k_begin + k_per_split);
  f32x4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // copying x: 4 U chunks a row and pass; thread t copies chunk t % (4 U) of rows t / (4 U) + RP j
  constexpr int RP = 256 / (4 * U);  // rows the workgroup copies at a time
  const int c_chunk = threadIdx.x & (4 * U - 1), c_row = threadIdx.x / (4 * U);
  constexpr int XL = MB * 16 / RP;  // loads a thread issues for the x slice
  // The loads of the next 8 k steps (W and the x slice) are in flight while the current ones are
  // multiplied: they are issued right after the barrier that publishes the current x slice.
  bf16x8 a_next[U], xv[XL];
  auto fetch = [&](int kk) {
#pragma unroll
    for (int j = 0; j < XL; ++j) {
      const int row = min(c_row + RP * j, M - 1), k = kk + 8 * c_chunk;
      xv[j] = *(const bf16x8*)(x + (size_t)row * ldx + (k < k_end ? k : k_begin));
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = kk + 32 * u + 8 * g;
      const bool in = k < k_end;
      const bf16x8 av = *ws.at(kk + 32 * u, in);
      a_next[u] = in ? av : gs_zero8();
    }
  };
  if (k_begin < k_end) fetch(k_begin);
  for (int kk = k_begin; kk < k_end; kk += 32 * U) {
    bf16_t* my = xs;
    __syncthreads();  // the slice of the pass before is no longer read
#pragma unroll
    for (int j = 0; j < XL; ++j) *(bf16x8*)(my + (c_chunk * (MB * 16) + ((c_row + RP * j) ^ (c_chunk & 15))) * 8) = xv[j];
    bf16x8 a[U];
#pragma unroll
    for (int u = 0; u < U; ++u) a[u] = a_next[u];
    __syncthreads();  // the slice is complete
    if (kk + 32 * U < k_end) fetch(kk + 32 * U);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const bf16x8 b = *(const bf16x8*)(my + ((4 * u + g) * (MB * 16) + 16 * mb + (r16 ^ ((4 * u + g) & 15))) * 8);
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b, acc[mb], 0, 0, 0);
      }
  }
  // acc[mb][i] = C[n = n0 + 4g + i][m = 16 mb + r16]
  TY* yp = y + (size_t)blockIdx.y * part_stride;
  if (MB == 1 && sc.ssq) {  // uniform
    row_scale_end<256>(sc, sc_part, rscale);
    __syncthreads();
    acc[0] *= rscale[r16];
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = 16 * mb + r16;
    if (EPI == EPI_STORE) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + 4 * g + i;
        if (m < M && n < N) yp[(size_t)m * ldy + n] = from_f<TY>(acc[mb][i]);
      }
    } else {
      // lane groups 0,1 hold gate rows 4g+i of 8 channels, groups 2,3 the up rows of the same channels
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float other = __shfl_xor(acc[mb][i], 32, FG_WAVE);
        const float gate = acc[mb][i], up = other;
        const int col = n0 / 2 + 4 * g + i;
        if (g < 2 && m < M && n0 + 8 + 4 * g + i < N) yp[(size_t)m * ldy + col] = from_f<TY>(gate / (1.f + __expf(-gate)) * up);
      }
    }
  }
}

template <int MB, int EPI, class TY>
static void launch_skinny(const void* x, int ldx, const void* w, int ldw, void* y, int ldy, int M, int N,
                          int K, const RowScale& sc, const Residual& rs, hipStream_t stream) {
  const int blocks = (N + 15) / 16;
  if (MB == 1 && M > 1) {  // one row of x is a broadcast already
    if (blocks >= 1024)
      gemm_skinny16_kernel<4, EPI, TY><<<blocks, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw,
                                                                   (TY*)y, ldy, M, N, K, RopeKv{}, sc, rs);
    else
      gemm_skinny16_kernel<8, EPI, TY><<<blocks, 512, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw,
                                                                   (TY*)y, ldy, M, N, K, RopeKv{}, sc, rs);
    return;
  }
  // few blocks: more waves a block, so that enough loads are in flight on every CU
  if (blocks >= 1024)
    gemm_skinny_kernel<MB, 4, EPI, TY><<<blocks, 256, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw,
                                                                   (TY*)y, ldy, M, N, K, sc, rs);
  else
    gemm_skinny_kernel<MB, 8, EPI, TY><<<blocks, 512, 0, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw,
                                                                   (TY*)y, ldy, M, N, K, sc, rs);
}

// x [M, K] bf16 (M <= 64), w [N, K] bf16, K % 8 == 0, rows 16-byte aligned; ldw = 0: w is packed (see the top;
// so in every entry point of this file).
// epilogue 0: y [M, N] of out_dtype; epilogue 1: w's rows interleaved gate/up in
// groups of 8 (N % 16 == 0), y [M, N/2] = silu(gate) * up of out_dtype.
extern "C" int fg_gemm_skinny(const void* x, int ldx, const void* w, int ldw, void* y, int ldy, int M, int N,
                              int K, int out_dtype, int epilogue, hipStream_t stream) {
  if (M <= 0 || N <= 0) return FG_OK;
  if (M > 64 || K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || (ldw && ldw < K)) return FG_ERR_ARG;
  if (epilogue == EPI_SILU_MUL && (N % 16 || ldy < N / 2)) return FG_ERR_ARG;
  if (epilogue == EPI_STORE && ldy < N) return FG_ERR_ARG;
  if (epilogue != EPI_STORE && epilogue != EPI_SILU_MUL) return FG_ERR_ARG;
  const int mb = (M + 15) / 16;
  const RowScale sc{nullptr, 0, 0.f, 0.f};
  const Residual rs{};
#define GO(MB)                                                                                        \
  do {                                                                                                \
    if (epilogue == EPI_STORE && out_dtype == FG_BF16)                                                \
      launch_skinny<MB, EPI_STORE, bf16_t>(x, ldx, w, ldw, y, ldy, M, N, K, sc, rs, stream);          \
    else if (epilogue == EPI_STORE && out_dtype == FG_F32)                                            \
      launch_skinny<MB, EPI_STORE, float>(x, ldx, w, ldw, y, ldy, M, N, K, sc, rs, stream);           \
    else if (epilogue == EPI_SILU_MUL && out_dtype == FG_BF16)                                        \
      launch_skinny<MB, EPI_SILU_MUL, bf16_t>(x, ldx, w, ldw, y, ldy, M, N, K, sc, rs, stream);       \
    else                                                                                              \
      return FG_ERR_ARG;                                                                              \
  } while (0)
  if (mb == 1) GO(1);
  else if (mb == 2) GO(2);
  else if (mb == 3) GO(3);
  else GO(4);
#undef GO
  return fg_launch_status();
}

// The same for at most 16 rows with the layer's norms folded into the products (see RowScale and
// Residual above).  ssq [M, n_parts] (null: x is taken as it is), dim = the width that the sums of
// squares run over.  epilogue 0 and 1 as above (y bf16); epilogue 3: y is not written; h [M, N] fp32
// += the product, x_out [M, N] bf16 = h * norm_w, ssq_out [M, ceil(N / 16)] = the sums of squares of
// h over each workgroup's 16 columns.
extern "C" int fg_gemm_skinny_fused(const void* x, int ldx, const void* w, int ldw, void* y, int ldy, int M, int N,
                                    int K, int epilogue, const float* ssq, int n_parts, int dim, float eps,
                                    float* h, int ldh, const void* norm_w, int norm_w_dtype, void* x_out, int ldxo,
                                    float* ssq_out, hipStream_t stream) {
  if (M <= 0 || N <= 0) return FG_OK;
  if (M > 16 || K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || (ldw && ldw < K)) return FG_ERR_ARG;
  if (ssq && (n_parts < 1 || dim < 1 || !(eps >= 0.f))) return FG_ERR_ARG;
  if (epilogue == EPI_SILU_MUL && (N % 16 || ldy < N / 2 || !y)) return FG_ERR_ARG;
  if (epilogue == EPI_STORE && (ldy < N || !y)) return FG_ERR_ARG;
  if (epilogue == EPI_RESIDUAL && (!h || !norm_w || !x_out || !ssq_out || ldh < N || ldxo < N ||
                                   (norm_w_dtype != FG_F32 && norm_w_dtype != FG_BF16)))
    return FG_ERR_ARG;
  const RowScale sc{ssq, n_parts, ssq ? 1.f / (float)dim : 0.f, eps};
  const Residual rs{h, ldh, norm_w, norm_w_dtype == FG_F32, (bf16_t*)x_out, ldxo, ssq_out};
  if (epilogue == EPI_STORE) launch_skinny<1, EPI_STORE, bf16_t>(x, ldx, w, ldw, y, ldy, M, N, K, sc, rs, stream);
  else if (epilogue == EPI_SILU_MUL) launch_skinny<1, EPI_SILU_MUL, bf16_t>(x, ldx, w, ldw, y, ldy, M, N, K, sc, rs, stream);
  else if (epilogue == EPI_RESIDUAL) launch_skinny<1, EPI_RESIDUAL, bf16_t>(x, ldx, w, ldw, y, ldy, M, N, K, sc, rs, stream);
  else return FG_ERR_ARG;
  return fg_launch_status();
}

// x [M, K] bf16 with 16 < M <= 128 (fewer rows work too).  k_splits > 1: y is fp32 [k_splits, M, N]
// (part_stride elements apart), partial sums over K to be added by the consumer in split order;
// only with epilogue 0.
// ssq [M, n_parts] (null: x is taken as it is; else M <= 16 and one split): the rows' sums of squares for a norm
// folded into this product, dim = the width that they run over.
extern "C" int fg_gemm_skinny64(const void* x, int ldx, const void* w, int ldw, void* y, int ldy,
                                long long part_stride, int k_splits, int M, int N, int K, int out_dtype,
                                int epilogue, const float* ssq, int n_parts, int dim, float eps,
                                hipStream_t stream) {
  if (M <= 0 || N <= 0) return FG_OK;
  if (ssq && (M > 16 || k_splits != 1 || n_parts < 1 || dim < 1 || !(eps >= 0.f))) return FG_ERR_ARG;
  const RowScale sc{ssq, n_parts, ssq ? 1.f / (float)dim : 0.f, eps};
  if (M > 128 || K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || (ldw && ldw < K) || k_splits < 1 || k_splits > 65535)
    return FG_ERR_ARG;
  if (epilogue == EPI_SILU_MUL && (N % 16 || ldy < N / 2 || k_splits != 1 || out_dtype != FG_BF16)) return FG_ERR_ARG;
  if (epilogue == EPI_STORE && (ldy < N || (k_splits > 1 && out_dtype != FG_F32))) return FG_ERR_ARG;
  if (epilogue != EPI_STORE && epilogue != EPI_SILU_MUL) return FG_ERR_ARG;
  const int k_per_split = ((K + k_splits * 256 - 1) / (k_splits * 256)) * 256;
  const dim3 grid((N + 63) / 64, k_splits);
  const int mb = (M + 15) / 16;
#define GO64(MB, EPI, TY)                                                                                    \
  gemm_skinny64_kernel<MB, 8, EPI, TY><<<grid, 256, 0, stream>>>(                                             \
      (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (TY*)y, ldy, (size_t)part_stride, M, N, K, k_per_split, sc)
#define PICK(MB)                                                                   \
  do {                                                                             \
    if (epilogue == EPI_SILU_MUL) GO64(MB, EPI_SILU_MUL, bf16_t);                  \
    else if (out_dtype == FG_BF16) GO64(MB, EPI_STORE, bf16_t);                    \
    else if (out_dtype == FG_F32) GO64(MB, EPI_STORE, float);                      \
    else return FG_ERR_ARG;                                                        \
  } while (0)
  if (mb == 1) PICK(1);
  else if (mb == 2) PICK(2);
  else if (mb == 3) PICK(3);
  else if (mb == 4) PICK(4);
  else if (mb == 5) PICK(5);
  else if (mb == 6) PICK(6);
  else if (mb == 7) PICK(7);
  else PICK(8);
#undef PICK
#undef GO64
  return fg_launch_status();
}

// q, k, v projections of at most 16 rows with the rotation and the cache write in the epilogue:
// w = [q rows; k rows; v rows] ([(H + 2 KV) * hd, K]); y = rotated q [M, H * hd]; rotated k and v go
// to slots[m] of the pages.  table: cos/sin of the rows' positions (null: no rotation).
// ssq [M, n_parts] (null: x is taken as it is): the rows' sums of squares for the norm folded into this product.
extern "C" int fg_gemm_skinny_qkv(const void* x, int ldx, const void* w, int ldw, void* y, int ldy, int M, int K,
                                  const float* table, const int* slots, void* k_pages, void* v_pages,
                                  int n_heads, int n_kv, int hd, int rotary_dim, int page_size,
                                  const float* ssq, int n_parts, int dim, float eps, hipStream_t stream) {
  if (M <= 0) return FG_OK;
  const int N = (n_heads + 2 * n_kv) * hd;
  if (M > 16 || K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || (ldw && ldw < K) || hd % 16 || n_heads <= 0 ||
      n_kv <= 0 || rotary_dim < 0 || rotary_dim > hd || rotary_dim % 2 || page_size <= 0 || page_size % 8 ||
      ldy < n_heads * hd || ldy % 2 || !slots || !k_pages || !v_pages || (rotary_dim && !table) ||
      (ssq && (n_parts < 1 || dim < 1 || !(eps >= 0.f))))
    return FG_ERR_ARG;
  const RowScale sc{ssq, n_parts, ssq ? 1.f / (float)dim : 0.f, eps};
  const Residual rs{};
  const RopeKv rk{rotary_dim ? table : nullptr, slots, (bf16_t*)k_pages, (bf16_t*)v_pages,
                  n_heads, n_kv, hd, rotary_dim, page_size};
  const int blocks = N / 16;
  if (blocks >= 1024)
    gemm_skinny16_kernel<4, EPI_ROPE_KV, bf16_t><<<blocks, 256, 0, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (bf16_t*)y, ldy, M, N, K, rk, sc, rs);
  else
    gemm_skinny16_kernel<8, EPI_ROPE_KV, bf16_t><<<blocks, 512, 0, stream>>>(
        (const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (bf16_t*)y, ldy, M, N, K, rk, sc, rs);
  return fg_launch_status();
}
