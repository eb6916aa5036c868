// What the machine gives when nothing else is in the way: kernels for the measurement program to
// time, so that a step's rate can be set against a measured peak beside the published one.
//   * peak_read_kernel / peak_copy_kernel: streaming reads (and writes) of a large buffer;
//   * peak_mfma_bf16_kernel / peak_mfma_f32_kernel: a loop of independent matrix instructions on
//     registers (v_mfma_f32_32x32x16_bf16, v_mfma_f32_16x16x4_f32), no memory traffic;
//   * peak_handover_kernel: what it costs to hand data from every workgroup to every other INSIDE one
//     launch (write-through stores, a flag per workgroup, loads that go past the caches): the time a
//     decode step would pay per dependent phase if its kernels were fused into one persistent kernel,
//     to be set against the time between two dependent launches of a graph.
#include "common.h"

namespace {

constexpr int P_THREADS = 256;

__global__ __launch_bounds__(P_THREADS) void peak_read_kernel(const f32x4* __restrict__ src, float* __restrict__ sink,
                                                              int64_t n16) {
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const int64_t stride = (int64_t)gridDim.x * P_THREADS;
  int64_t i = (int64_t)blockIdx.x * P_THREADS + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {      // four loads in flight per thread
    const f32x4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc += a + b + c + d;
  }
  for (; i < n16; i += stride) acc += src[i];
  const float s = acc[0] + acc[1] + acc[2] + acc[3];
  if (s == 123456.789f) sink[0] = s;      // never true for the buffers used: keeps the loads alive
}

__global__ __launch_bounds__(P_THREADS) void peak_copy_kernel(const f32x4* __restrict__ src, f32x4* __restrict__ dst,
                                                              int64_t n16) {
  const int64_t stride = (int64_t)gridDim.x * P_THREADS;
  int64_t i = (int64_t)blockIdx.x * P_THREADS + threadIdx.x;
  for (; i + 3 * stride < n16; i += 4 * stride) {
    const f32x4 a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    dst[i] = a;
    dst[i + stride] = b;
    dst[i + 2 * stride] = c;
    dst[i + 3 * stride] = d;
  }
  for (; i < n16; i += stride) dst[i] = src[i];
}

// Each wave keeps four independent 32x32 accumulators busy: 4 * 2 * 32 * 32 * 16 flops per trip.
__global__ __launch_bounds__(P_THREADS) void peak_mfma_bf16_kernel(float* __restrict__ sink, int iters) {
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = (bf16_t)(0.001f * (float)(threadIdx.x % 7 + e));
    b[e] = (bf16_t)(0.002f * (float)(threadIdx.x % 5 + e));
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int i = 0; i < iters; ++i) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  const f32x16 c = c0 + c1 + c2 + c3;
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 16; ++e) s += c[e];
  if (s == 123456.789f) sink[0] = s;
}

// Four independent 16x16 accumulators: 4 * 2 * 16 * 16 * 4 flops per trip.
__global__ __launch_bounds__(P_THREADS) void peak_mfma_f32_kernel(float* __restrict__ sink, int iters) {
  const float a = 0.001f * (float)(threadIdx.x % 7 + 1), b = 0.002f * (float)(threadIdx.x % 5 + 1);
  f32x4 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int i = 0; i < iters; ++i) {
    c0 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c3, 0, 0, 0);
  }
  const f32x4 c = c0 + c1 + c2 + c3;
  const float s = c[0] + c[1] + c[2] + c[3];
  if (s == 123456.789f) sink[0] = s;
}

// One round: every workgroup writes `payload` floats with stores that go through to memory, waits
// until they are acknowledged, raises its flag; one wave per workgroup reads all flags until all are
// up; every workgroup then reads another workgroup's floats with loads that go past the caches and
// checks them.  No read-modify-write, no shared counter: the round's cost is the few trips to the
// point where the caches of the eight dies meet.  Waits are bounded: after `spin_limit` polls a
// workgroup gives up, says so in *err and everybody leaves.
constexpr int H_THREADS = 512, H_MAX_WG = 256;
__global__ __launch_bounds__(H_THREADS) void peak_handover_kernel(unsigned* __restrict__ flags, float* __restrict__ data,
                                                                   int rounds, int payload, unsigned spin_limit,
                                                                   int* __restrict__ err, unsigned* __restrict__ wrong) {
  __shared__ int ok_s;
  const int nwg = gridDim.x, wg = blockIdx.x;
  unsigned bad = 0;
  for (int it = 0; it < rounds; ++it) {
    float* mine = data + ((size_t)(it & 1) * nwg + wg) * payload;
    for (int i = threadIdx.x; i < payload; i += H_THREADS)
      __hip_atomic_store(&mine[i], (float)(it * 7 + wg * 3 + i), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_s_waitcnt(0);          // this wave's stores have been acknowledged
    __builtin_amdgcn_s_barrier();
    if (threadIdx.x < TL_WAVE) {
      const int lane = threadIdx.x;
      if (lane == 0) __hip_atomic_store(&flags[wg], (unsigned)(it + 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      bool ok = true;
      unsigned spins = 0;
      while (true) {
        bool up = true;
#pragma unroll
        for (int j = 0; j < H_MAX_WG / TL_WAVE; ++j) {
          const int i = lane * (H_MAX_WG / TL_WAVE) + j;
          if (i < nwg) up &= __hip_atomic_load(&flags[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= (unsigned)(it + 1);
        }
        if (__all(up)) break;
        if (++spins > spin_limit || __hip_atomic_load(err, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
          ok = false;
          break;
        }
      }
      if (lane == 0) {
        if (!ok) __hip_atomic_store(err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok_s = ok;
      }
    }
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (!*(volatile int*)&ok_s) return;
    const int other = (wg + 77 + it) % nwg;
    const float* theirs = data + ((size_t)(it & 1) * nwg + other) * payload;
    for (int i = threadIdx.x; i < payload; i += H_THREADS)
      if (__hip_atomic_load(&theirs[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != (float)(it * 7 + other * 3 + i)) ++bad;
  }
  if (bad) atomicAdd(wrong, bad);
}

}  // namespace

extern "C" {

// `rounds` hand-overs of `payload` floats a workgroup among `workgroups` (at most 256, one per compute
// unit at most: all must be resident at once).  flags: `workgroups` zeroed words; data: 2 * workgroups *
// payload floats; err, wrong: zeroed words (after the launch: 1 if a wait ran out; values read wrong).
int tl_peak_handover(unsigned* flags, float* data, int workgroups, int rounds, int payload, unsigned spin_limit, int* err,
                     unsigned* wrong, hipStream_t stream) {
  if (!flags || !data || !err || !wrong || workgroups <= 0 || workgroups > H_MAX_WG || rounds <= 0 || payload <= 0 ||
      spin_limit == 0)
    return TL_ERR_ARG;
  hipLaunchKernelGGL(peak_handover_kernel, dim3(workgroups), dim3(H_THREADS), 0, stream, flags, data, rounds, payload,
                     spin_limit, err, wrong);
  return tl_launch_status();
}

// mode 0: read `bytes` of src; mode 1: copy them to dst.  Both 16-byte aligned, bytes a multiple of 16.
int tl_peak_stream(const void* src, void* dst, float* sink, int64_t bytes, int mode, int blocks, hipStream_t stream) {
  if (bytes <= 0 || bytes % 16 || blocks <= 0 || blocks > 65535 * 16 || !sink || !src) return TL_ERR_ARG;
  if (mode == 0)
    hipLaunchKernelGGL(peak_read_kernel, dim3(blocks), dim3(P_THREADS), 0, stream, (const f32x4*)src, sink, bytes / 16);
  else if (mode == 1 && dst)
    hipLaunchKernelGGL(peak_copy_kernel, dim3(blocks), dim3(P_THREADS), 0, stream, (const f32x4*)src, (f32x4*)dst,
                       bytes / 16);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

// dtype 1: bfloat16 32x32x16, dtype 0: float32 16x16x4.  Returns the flops of the launch through *flops.
int tl_peak_mfma(float* sink, int dtype, int iters, int blocks, double* flops, hipStream_t stream) {
  if (!sink || iters <= 0 || blocks <= 0 || blocks > 65535 * 16) return TL_ERR_ARG;
  const double waves = (double)blocks * (P_THREADS / TL_WAVE);
  if (dtype == 1) {
    hipLaunchKernelGGL(peak_mfma_bf16_kernel, dim3(blocks), dim3(P_THREADS), 0, stream, sink, iters);
    if (flops) *flops = waves * iters * 4.0 * 2.0 * 32 * 32 * 16;
  } else if (dtype == 0) {
    hipLaunchKernelGGL(peak_mfma_f32_kernel, dim3(blocks), dim3(P_THREADS), 0, stream, sink, iters);
    if (flops) *flops = waves * iters * 4.0 * 2.0 * 16 * 16 * 4;
  } else {
    return TL_ERR_ARG;
  }
  return tl_launch_status();
}

}  // extern "C"
