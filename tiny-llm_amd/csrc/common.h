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

// Exchanges between the lanes of a wave64 without the LDS crossbar (ds_bpermute, which costs a
// round trip to LDS per step and sits in the dependent chains of the softmax and the norms):
// gfx950's lane swaps for the steps over 32 and 16 lanes, DPP moves inside a row of 16 lanes.
typedef unsigned int tl_u32x2 __attribute__((ext_vector_type(2)));
constexpr int TL_DPP_XOR1 = 0xB1, TL_DPP_XOR2 = 0x4E;              // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int TL_DPP_MIRROR = 0x140, TL_DPP_HALF_MIRROR = 0x141;   // lane 15 - i of the row, 7 - i of the half row
constexpr int TL_DPP_ROR1 = 0x121, TL_DPP_ROR2 = 0x122, TL_DPP_ROR4 = 0x124, TL_DPP_ROR8 = 0x128;   // rotate the row
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false); }
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) { return __int_as_float(dpp_i32<CTRL>(__float_as_int(v))); }
// a = v of lane (l & ~16), b = v of lane (l | 16): this lane's value and its partner's over 16 lanes
__device__ __forceinline__ void pair16(float v, float& a, float& b) {
  const tl_u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
// the same over 32 lanes
__device__ __forceinline__ void pair32(float v, float& a, float& b) {
  const tl_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  a = __uint_as_float(r[0]);
  b = __uint_as_float(r[1]);
}
// v + v of lane l ^ 16, then the same over 32: the sum over the four rows of 16 lanes
__device__ __forceinline__ float sum_over_rows(float v) {
  float a, b;
  pair16(v, a, b);
  v = a + b;
  pair32(v, a, b);
  return a + b;
}
__device__ __forceinline__ float max_over_rows(float v) {
  float a, b;
  pair16(v, a, b);
  v = fmaxf(a, b);
  pair32(v, a, b);
  return fmaxf(a, b);
}

// Butterfly over 32, 16, 8, 4, 2, 1 lanes; every lane gets the result.  Inside a row the partner
// over n lanes is reached by rotating the row by n: lanes that differ only in the higher bits hold
// the same value by then, so the result is that of the exchange with lane l ^ n, to the bit.
__device__ __forceinline__ float wave_sum(float v) {
  float a, b;
  pair32(v, a, b);
  v = a + b;
  pair16(v, a, b);
  v = a + b;
  v += dpp_f32<TL_DPP_ROR8>(v);
  v += dpp_f32<TL_DPP_ROR4>(v);
  v += dpp_f32<TL_DPP_ROR2>(v);
  v += dpp_f32<TL_DPP_ROR1>(v);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
  float a, b;
  pair32(v, a, b);
  v = fmaxf(a, b);
  pair16(v, a, b);
  v = fmaxf(a, b);
  v = fmaxf(v, dpp_f32<TL_DPP_ROR8>(v));
  v = fmaxf(v, dpp_f32<TL_DPP_ROR4>(v));
  v = fmaxf(v, dpp_f32<TL_DPP_ROR2>(v));
  v = fmaxf(v, dpp_f32<TL_DPP_ROR1>(v));
  return v;
}

// Maximum and minimum over a row of 16 lanes (integers); every lane of the row gets the result.
__device__ __forceinline__ int row_max_i32(int v) {
  v = max(v, dpp_i32<TL_DPP_ROR8>(v));
  v = max(v, dpp_i32<TL_DPP_ROR4>(v));
  v = max(v, dpp_i32<TL_DPP_ROR2>(v));
  return max(v, dpp_i32<TL_DPP_ROR1>(v));
}
__device__ __forceinline__ int row_min_i32(int v) {
  v = min(v, dpp_i32<TL_DPP_ROR8>(v));
  v = min(v, dpp_i32<TL_DPP_ROR4>(v));
  v = min(v, dpp_i32<TL_DPP_ROR2>(v));
  return min(v, dpp_i32<TL_DPP_ROR1>(v));
}
// Sum over aligned groups of 8 or 16 lanes, as the butterfly over 1, 2, 4 (, 8) lanes gives it.
template <int GROUP>
__device__ __forceinline__ float group_sum(float v) {
  static_assert(GROUP == 8 || GROUP == 16, "groups of 8 or 16 lanes");
  v += dpp_f32<TL_DPP_XOR1>(v);
  v += dpp_f32<TL_DPP_XOR2>(v);
  v += dpp_f32<TL_DPP_HALF_MIRROR>(v);      // the quads of a half row hold one value each by now
  if constexpr (GROUP == 16) v += dpp_f32<TL_DPP_MIRROR>(v);
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
