// Shared device helpers for the gfx950 kernels: element conversion, wave64
// reductions, error codes.  Everything is written for wave64 (CDNA4) only.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define TL_WAVE 64

// Status codes returned by every extern "C" entry point (0 = launched).
#define TL_OK 0
#define TL_ERR_ARG 1      // a size or pointer the kernel cannot take
#define TL_ERR_LAUNCH 2   // the runtime refused the launch

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }  // round to nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = TL_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, TL_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = TL_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, TL_WAVE));
  return v;
}

// Sum over a workgroup of `NW` waves; `red` is LDS of at least NW floats.
// Every thread gets the total.  The order of additions is fixed.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x / TL_WAVE, lane = threadIdx.x % TL_WAVE;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) t += red[i];
  return t;
}

static inline int tl_launch_status() {
  return hipGetLastError() == hipSuccess ? TL_OK : TL_ERR_LAUNCH;
}

static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
