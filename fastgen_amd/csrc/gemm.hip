// y = x W^T with W stored [out, in] row-major (fastgen/forward.py:433-440,
// 470, 488-496, 513: F.linear).  This is the engine's own matrix product for
// the true 32-bit path: plain fp32 fused multiply-adds, no matrix-core mode of
// reduced precision.  Every output element is one dot product summed by one
// thread in an order fixed by K alone (16 products into a partial sum, 16
// partial sums into a second one, those into the total: rounding grows with
// K/256 + 32, not with K), so a row's result does not depend on how many other
// rows the call holds.  It also takes bf16 operands (fp32
// accumulate) so that any shape has a product when the tuned ones refuse it.
#include "common.h"

#define GT_M 64
#define GT_N 64
#define GT_K 16
#define GT_THREADS 256

template <class TX, class TW, class TY>
__global__ __launch_bounds__(GT_THREADS) void gemm_nt_kernel(
    const TX* __restrict__ x, const TW* __restrict__ w, TY* __restrict__ y, int M, int N,
    int K, int ldx, int ldw, int ldy) {
  // tiles stored k-major so that the inner product reads consecutive floats
  __shared__ float xs[GT_K][GT_M + 4];
  __shared__ float ws[GT_K][GT_N + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GT_M, n0 = blockIdx.x * GT_N;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4], mid[4][4];  // total; sum of up to 16 tiles' partial sums
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = mid[i][j] = 0.f;
  int tiles_in_mid = 0;

  // each thread loads 4 elements of each tile: row = tid / 4, k = (tid % 4) * 4 ..
  const int lr = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += GT_K) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int m = m0 + lr, n = n0 + lr;
      xs[lk + e][lr] = (m < M && k < K) ? to_f<TX>(x[(size_t)m * ldx + k]) : 0.f;
      ws[lk + e][lr] = (n < N && k < K) ? to_f<TW>(w[(size_t)n * ldw + k]) : 0.f;
    }
    __syncthreads();
    float part[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
    for (int k = 0; k < GT_K; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[k][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
    }
    const bool fold = ++tiles_in_mid == 16;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        mid[i][j] += part[i][j];
        if (fold) {
          acc[i][j] += mid[i][j];
          mid[i][j] = 0.f;
        }
      }
    if (fold) tiles_in_mid = 0;
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] += mid[i][j];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + tm + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tn + j;
      if (n < N) y[(size_t)m * ldy + n] = from_f<TY>(acc[i][j]);
    }
  }
}

// dtypes: x and w share `in_dtype`; y is `out_dtype` (fp32 output of bf16
// operands serves the LM head).
extern "C" int fg_gemm_nt(const void* x, const void* w, void* y, int M, int N, int K, int ldx,
                          int ldw, int ldy, int in_dtype, int out_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return FG_OK;
  if (K <= 0 || ldx < K || ldw < K || ldy < N) return FG_ERR_ARG;
  dim3 grid((N + GT_N - 1) / GT_N, (M + GT_M - 1) / GT_M);
  if (grid.y > 65535) return FG_ERR_ARG;
#define LAUNCH(TX, TY)                                                                      \
  gemm_nt_kernel<TX, TX, TY><<<grid, GT_THREADS, 0, stream>>>((const TX*)x, (const TX*)w,   \
                                                              (TY*)y, M, N, K, ldx, ldw, ldy)
  if (in_dtype == FG_F32 && out_dtype == FG_F32) LAUNCH(float, float);
  else if (in_dtype == FG_BF16 && out_dtype == FG_BF16) LAUNCH(bf16_t, bf16_t);
  else if (in_dtype == FG_BF16 && out_dtype == FG_F32) LAUNCH(bf16_t, float);
  else return FG_ERR_ARG;
#undef LAUNCH
  return fg_launch_status();
}
