// Shared device helpers for the gfx950 kernels of this engine.
//
// Every kernel file is compiled on its own into one shared library with a
// plain C interface; the Python side passes raw device pointers and the HIP
// stream.  Element types are `float` (the true 32-bit path) and `bf16_t`
// (the serving path); all arithmetic between a load and a store is fp32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define FG_WAVE 64

// Error codes returned by every extern "C" entry point.
#define FG_OK 0
#define FG_ERR_ARG 1     // an argument the kernel cannot take (size, dtype)
#define FG_ERR_LAUNCH 2  // hipGetLastError() after the launch was not hipSuccess

// dtype codes shared with fastgen_amd/kernels/_lib.py
#define FG_F32 0
#define FG_BF16 1

template <class T> __device__ __forceinline__ float to_f(T x);
template <> __device__ __forceinline__ float to_f<float>(float x) { return x; }
template <> __device__ __forceinline__ float to_f<bf16_t>(bf16_t x) { return (float)x; }

template <class T> __device__ __forceinline__ T from_f(float x);
template <> __device__ __forceinline__ float from_f<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_f<bf16_t>(float x) { return (bf16_t)x; }

// Eight consecutive elements as floats; p must be 16-byte aligned (32 for float).
template <class T> __device__ __forceinline__ void load8(const T* p, float (&v)[8]);
template <> __device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <> __device__ __forceinline__ void load8<bf16_t>(const bf16_t* p, float (&v)[8]) {
  const uint4 raw = *(const uint4*)p;
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[2 * i] = __uint_as_float(w[i] << 16);
    v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
  }
}
template <class T> __device__ __forceinline__ void store8(T* p, const float (&v)[8]);
template <> __device__ __forceinline__ void store8<float>(float* p, const float (&v)[8]) {
  *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
  *(float4*)(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
template <> __device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float (&v)[8]) {
  typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
  bf16x8_t o;
#pragma unroll
  for (int i = 0; i < 8; ++i) o[i] = (__bf16)v[i];
  *(bf16x8_t*)p = o;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = FG_WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, FG_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = FG_WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, FG_WAVE));
  return v;
}

// Sum over a block of up to 16 waves; every thread gets the result.  The
// order of additions is fixed by the block size alone.
__device__ __forceinline__ float block_sum(float v, float* lds /* >= 16 floats */) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int nwaves = (blockDim.x + FG_WAVE - 1) / FG_WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; ++i) total += lds[i];
  return total;
}

__device__ __forceinline__ float block_max(float v, float* lds) {
  const int lane = threadIdx.x % FG_WAVE, wave = threadIdx.x / FG_WAVE;
  const int nwaves = (blockDim.x + FG_WAVE - 1) / FG_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) lds[wave] = v;
  __syncthreads();
  float total = lds[0];
  for (int i = 1; i < nwaves; ++i) total = fmaxf(total, lds[i]);
  return total;
}

static inline int fg_launch_status() {
  return hipGetLastError() == hipSuccess ? FG_OK : FG_ERR_LAUNCH;
}
