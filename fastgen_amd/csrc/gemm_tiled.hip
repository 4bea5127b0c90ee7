// y = x W^T for many rows of x (batches of more than a hundred decoding sequences, prompt portions of
// a few hundred tokens), bf16 operands, fp32 accumulation on the matrix cores, where the output is
// narrow (few columns, long k): the output projection and the down projection of a decoder layer.
// The vendor library runs such a product as a few dozen tiles without cutting k and leaves most of
// the GPU idle (forward.py:470-472, 497-499 of the reference go through it); here the k range is cut
// over workgroups (blockIdx.z) until there are workgroups for every compute unit, and the fp32
// partial sums are added, in split order, by the norm kernel that consumes them.
//
//  * A workgroup owns 64 WM rows of x and 64 WN columns of the output, its WM x WN waves 64 x 64
//    each.  v_mfma_f32_16x16x32_bf16 with W as the A operand (16 columns x 32 k) and x^T as B, so
//    that a lane holds 4 consecutive columns of one row of y.
//  * Both operands go from memory straight into LDS (global_load_lds: no registers, no store
//    instructions) through a ring of NST stages of 32 k.  A stage is 4 WN blocks of W and 4 WM
//    blocks of x, each block 16 rows x 32 k = 1 KB in the order a wave's lanes read an MFMA operand
//    (lane = 16 * (k chunk of 8) + row): a wave's load of a block lands in that order (the hardware
//    puts lane i's 16 bytes at base + 16 i), its operand read is one contiguous KB, and in memory it
//    covers 64 contiguous bytes of 16 rows.
//  * One barrier a stage: it publishes the stage that has landed and frees the one read before it,
//    into which the loads of the stage NST - 1 ahead are issued right away.  Every wave issues the
//    same number of loads per stage, so "my loads of this stage have landed" is a count (s_waitcnt
//    vmcnt); the barrier is the bare instruction (__syncthreads() would wait for every load in
//    flight, which would make the ring one stage deep).
//  * Epilogues: store bf16 or fp32 (partial sums: fp32), or, for a gate/up matrix whose rows are
//    interleaved in groups of 8 (gemm_skinny.hip), silu(gate) * up.
// Sums over k run in ascending order within a split whatever the batch holds: a row's result does
// not depend on the other rows.
#include "common.h"

#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define EPI_STORE 0
#define EPI_SILU_MUL 1

__device__ __forceinline__ bf16x8 gt_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// s_waitcnt for the vector memory counter alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

template <int WM, int WN, int NST, int EPI, class TY>
__global__ __launch_bounds__(64 * WM * WN) void gemm_tiled_kernel(
    const bf16_t* __restrict__ x, int ldx, const bf16_t* __restrict__ w, int ldw, TY* __restrict__ y, int ldy,
    size_t part_stride, int M, int N, int K, int k_per_split) {
  constexpr int NW = WM * WN;            // waves
  constexpr int WB = 4 * WN, XB = 4 * WM;  // blocks of 16 rows of W and of x in a stage
  constexpr int NB = WB + XB;            // blocks a stage holds
  constexpr int LPW = NB / NW;           // loads a wave issues per stage
  static_assert(NB % NW == 0, "blocks must divide over the waves");
  constexpr int BLOCK = 16 * 32;         // elements of a block
  static_assert(NST >= 3 && LPW * (NST - 2) < 64, "the ring's loads must fit the counter");
  extern __shared__ __attribute__((aligned(16))) bf16_t ring[];  // [NST][NB][BLOCK]

  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int r16 = lane & 15, g = lane >> 4;
  const int wm = wave / WN, wn = wave % WN;
  const int n_base = blockIdx.x * (64 * WN), m_base = blockIdx.y * (64 * WM);
  const int k_begin = min(K, (int)blockIdx.z * k_per_split), k_end = min(K, k_begin + k_per_split);
  const int n_stages = (k_end - k_begin + 31) / 32;

  // this lane's 16 bytes of the blocks its wave loads: block b = wave + NW j; rows beyond the matrix are
  // a copy of its last row (their results are not stored)
  const bf16_t* src[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int b = wave + NW * j;
    if (b >= WB) src[j] = x + (size_t)min(m_base + 16 * (b - WB) + r16, M - 1) * ldx + 8 * g;
    else if (ldw) src[j] = w + (size_t)min(n_base + 16 * b + r16, N - 1) * ldw + 8 * g;
    else src[j] = w + ((size_t)min((n_base >> 4) + b, (N - 1) >> 4) * ((K + 31) >> 5) * 64 + lane) * 8;  // packed
  }
  // elements from one k step of 32 to the next: 32 along a row, 512 (a block) in a packed W
  int step[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) step[j] = (wave + NW * j < WB && !ldw) ? 16 : 1;
  // stage s into slot s % NST; beyond the last stage the last one again, which nobody reads (every
  // wave issues LPW loads a stage to the end, so the count it waits for stays the same)
  auto issue = [&](int s) {
    const int k = k_begin + 32 * min(s, n_stages - 1);
    const int koff = k + 8 * g < k_end ? k : k_begin;  // a chunk beyond the k range: any readable one, zeroed at use
    bf16_t* slot = ring + (size_t)(s % NST) * NB * BLOCK;
#pragma unroll
    for (int j = 0; j < LPW; ++j)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src[j] + (size_t)koff * step[j]),
                                       (__attribute__((address_space(3))) void*)(slot + (wave + NW * j) * BLOCK), 16, 0, 0);
  };

  f32x4 acc[4][4];  // [row block mb][column block nb]
#pragma unroll
  for (int mb = 0; mb < 4; ++mb)
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) acc[mb][nb] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (n_stages > 0) {
#pragma unroll
    for (int s = 0; s < NST - 1; ++s) issue(s);
    // MASKED: the stage's last chunks of 8 k may lie beyond the k range (only the last stage of a range
    // whose length is no multiple of 32): their W operand is zeroed
    auto stage = [&](int i, auto masked) {
      wait_vmcnt<LPW*(NST - 2)>();  // this wave's loads of stage i have landed
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();  // everybody's have, and nobody reads stage i - 1 any more
      asm volatile("" ::: "memory");
      issue(i + NST - 1);            // into the slot of stage i - 1
      const bf16_t* st = ring + (size_t)(i % NST) * NB * BLOCK;
      bf16x8 a[4], b[4];
#pragma unroll
      for (int nb = 0; nb < 4; ++nb) {
        a[nb] = *(const bf16x8*)(st + (wn * 4 + nb) * BLOCK + lane * 8);
        if (decltype(masked)::value) a[nb] = k_begin + 32 * i + 8 * g < k_end ? a[nb] : gt_zero8();
      }
#pragma unroll
      for (int mb = 0; mb < 4; ++mb) b[mb] = *(const bf16x8*)(st + (WB + wm * 4 + mb) * BLOCK + lane * 8);
#pragma unroll
      for (int nb = 0; nb < 4; ++nb)
#pragma unroll
        for (int mb = 0; mb < 4; ++mb) acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[nb], b[mb], acc[mb][nb], 0, 0, 0);
    };
    const int n_full = (k_end - k_begin) / 32;
    for (int i = 0; i < n_full; ++i) stage(i, std::false_type{});
    if (n_full < n_stages) stage(n_full, std::true_type{});
    wait_vmcnt<0>();  // the loads issued past the end have to land before the workgroup's LDS is given up
  }

  // acc[mb][nb][i] = y[m = m_base + 64 wm + 16 mb + r16][n = n_base + 64 wn + 16 nb + 4 g + i]
  TY* yp = y + (size_t)blockIdx.z * part_stride;
#pragma unroll
  for (int mb = 0; mb < 4; ++mb) {
    const int m = m_base + 64 * wm + 16 * mb + r16;
#pragma unroll
    for (int nb = 0; nb < 4; ++nb) {
      const int n0 = n_base + 64 * wn + 16 * nb;
      if (EPI == EPI_STORE) {
        const int n = n0 + 4 * g;
        if (m >= M) continue;
        if (n + 3 < N && (ldy & 3) == 0) {
          if (sizeof(TY) == 4) {
            *(f32x4*)((float*)yp + (size_t)m * ldy + n) = acc[mb][nb];
          } else {
            bf16x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (__bf16)acc[mb][nb][i];
            *(bf16x4*)((bf16_t*)yp + (size_t)m * ldy + n) = v;
          }
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (n + i < N) yp[(size_t)m * ldy + n + i] = from_f<TY>(acc[mb][nb][i]);
        }
      } else {
        // lane groups 0, 1 hold the gate rows 4 g + i of 8 channels, groups 2, 3 the up rows of the same channels
        float act[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float up = __shfl_xor(acc[mb][nb][i], 32, FG_WAVE);
          const float gate = acc[mb][nb][i];
          act[i] = gate / (1.f + __expf(-gate)) * up;
        }
        const int col = n0 / 2 + 4 * g;  // n0 is a multiple of 16: 8 channels a block
        if (g < 2 && m < M && n0 + 8 + 4 * g + 3 < N) {
          if ((ldy & 3) == 0 && sizeof(TY) == 2) {
            bf16x4 v;
#pragma unroll
            for (int i = 0; i < 4; ++i) v[i] = (__bf16)act[i];
            *(bf16x4*)((bf16_t*)yp + (size_t)m * ldy + col) = v;
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) yp[(size_t)m * ldy + col + i] = from_f<TY>(act[i]);
          }
        }
      }
    }
  }
}

// Tile shapes (waves as rows x columns of 64 x 64 each), both with a ring of 4 stages:
//   tile_rows 128: 2 x 2 waves, 128 rows x 128 columns (64 KB of LDS: two workgroups a compute unit)
//   tile_rows 256: 4 x 2 waves, 256 rows x 128 columns (96 KB)
// (Measured and dropped: rings of 6 and 8 stages, and 128 rows x 256 columns: never faster than these two.)
template <int WM, int WN, int NST, int EPI, class TY>
static int launch_tiled(const void* x, int ldx, const void* w, int ldw, void* y, int ldy, long long part_stride,
                        int k_splits, int M, int N, int K, int k_per_split, hipStream_t stream) {
  constexpr int lds = NST * 4 * (WM + WN) * 1024;
  static bool raised = false;  // more than 64 KB of dynamic LDS has to be asked for once
  auto kernel = gemm_tiled_kernel<WM, WN, NST, EPI, TY>;
  if (lds > 65536 && !raised) {
    if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess)
      return FG_ERR_LAUNCH;
    raised = true;
  }
  const dim3 grid((N + 64 * WN - 1) / (64 * WN), (M + 64 * WM - 1) / (64 * WM), k_splits);
  kernel<<<grid, 64 * WM * WN, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)w, ldw, (TY*)y, ldy,
                                              (size_t)part_stride, M, N, K, k_per_split);
  return fg_launch_status();
}

// x [M, K] bf16, w [N, K] bf16, K % 8 == 0, rows 16-byte aligned; ldw = 0: w is packed in blocks of 16 rows x 32 k
// (gemm_skinny.hip), each of which is one block of a stage here and one contiguous KB in memory.
// epilogue 0: y [M, N] of out_dtype (k_splits > 1: fp32 [k_splits, M, N], part_stride elements apart,
// partial sums over K for the consumer to add in split order; a split's k range is a multiple of 32);
// epilogue 1: w's rows are gate/up interleaved in groups of 8 (N % 16 == 0), y [M, N / 2] bf16 =
// silu(gate) * up; k_splits must be 1.
extern "C" int fg_gemm_tiled(const void* x, int ldx, const void* w, int ldw, void* y, int ldy, long long part_stride,
                             int k_splits, int M, int N, int K, int out_dtype, int epilogue, int tile_rows,
                             hipStream_t stream) {
  if (M <= 0 || N <= 0) return FG_OK;
  if (K <= 0 || K % 8 || ldx % 8 || ldw % 8 || ldx < K || (ldw && ldw < K) || k_splits < 1 || k_splits > 65535 ||
      (tile_rows != 128 && tile_rows != 256))
    return FG_ERR_ARG;
  if (epilogue == EPI_SILU_MUL && (N % 16 || ldy < N / 2 || k_splits != 1 || out_dtype != FG_BF16)) return FG_ERR_ARG;
  if (epilogue == EPI_STORE && (ldy < N || (k_splits > 1 && out_dtype != FG_F32))) return FG_ERR_ARG;
  if (epilogue != EPI_STORE && epilogue != EPI_SILU_MUL) return FG_ERR_ARG;
  if (out_dtype != FG_BF16 && out_dtype != FG_F32) return FG_ERR_ARG;
  if (((long long)M + 127) / 128 > 65535) return FG_ERR_ARG;
  const int k_per_split = ((K + k_splits * 32 - 1) / (k_splits * 32)) * 32;
#define GO(WM, WN, NST, EPI, TY) \
  return launch_tiled<WM, WN, NST, EPI, TY>(x, ldx, w, ldw, y, ldy, part_stride, k_splits, M, N, K, k_per_split, stream)
#define PICK(WM, WN, NST)                                                   \
  do {                                                                      \
    if (epilogue == EPI_SILU_MUL) GO(WM, WN, NST, EPI_SILU_MUL, bf16_t);    \
    else if (out_dtype == FG_BF16) GO(WM, WN, NST, EPI_STORE, bf16_t);      \
    else GO(WM, WN, NST, EPI_STORE, float);                                 \
  } while (0)
  if (tile_rows == 128) PICK(2, 2, 4);
  PICK(4, 2, 4);
#undef PICK
#undef GO
}
