// Causal attention over the paged cache, for any mix of prompt portions and
// single decoded tokens in one launch.
//
// The math is the reference's online softmax (tiny_llm/ops/cuda/
// flash_attention.cu:50-117, 374-405): scores q.k * hd^-0.5, running maximum m and
// denominator l, output rescaled by exp(m - m') when the maximum moves.  Two
// things differ on purpose.  The mask compares absolute positions (key position
// <= query position, and > query position - window when a window is set) instead
// of indices relative to the launch, which is only right for a prompt that
// starts at position 0; and the division by l happens once at the end instead of
// after every tile.
//
// paged_attention_kernel: one wave64 per (token, query head); lanes split the
// keys of a 64-key tile for the scores and the head dimension for the output.
// All arithmetic is float32 whatever the cache's element type.  It takes any head
// size up to 256, any page size, any grouping of query heads.
#include "common.h"

namespace {

constexpr int kMaxHd = 256;
constexpr int kDPL = kMaxHd / TL_WAVE;  // output dims per lane

template <typename T>
__global__ __launch_bounds__(TL_WAVE) void paged_attention_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ req_of_token, const int32_t* __restrict__ positions,
    T* __restrict__ out, int64_t out_stride, int nq, int nkv, int hd, int block_size, float scale,
    int window) {
  __shared__ float qs[kMaxHd];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int r = req_of_token[t];
  const int pos = positions[t];
  const int kv_end = pos + 1;
  const int kv_begin = (window > 0 && kv_end > window) ? kv_end - window : 0;
  const int kvh = h / (nq / nkv);
  const int32_t* bt = block_tables + (int64_t)r * max_blocks;

  const T* qrow = q + (int64_t)t * q_stride + (int64_t)h * hd;
  for (int d = lane; d < hd; d += TL_WAVE) qs[d] = to_f32(qrow[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float o[kDPL];
#pragma unroll
  for (int i = 0; i < kDPL; ++i) o[i] = 0.f;

  for (int base = kv_begin; base < kv_end; base += TL_WAVE) {
    const int j = base + lane;
    const bool valid = j < kv_end;
    float s = -INFINITY;
    int64_t row_off = 0;  // element offset of key/value row j in its cache
    if (valid) {
      const int64_t blk = bt[j / block_size];
      row_off = ((blk * nkv + kvh) * block_size + (j % block_size)) * hd;
      const T* kp = k_cache + row_off;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(qs[d], to_f32(kp[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // lane 0 of every tile is valid, so m_new is finite
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < kDPL; ++i) o[i] *= alpha;
    const int n_keys = min(TL_WAVE, kv_end - base);
    const int lo = (int)(row_off & 0xffffffff), hi = (int)(row_off >> 32);
    for (int jj = 0; jj < n_keys; ++jj) {
      const float pj = __shfl(p, jj, TL_WAVE);
      const int64_t off = ((int64_t)__shfl(hi, jj, TL_WAVE) << 32) | (uint32_t)__shfl(lo, jj, TL_WAVE);
      const T* vp = v_cache + off;
#pragma unroll
      for (int i = 0; i < kDPL; ++i) {
        const int d = lane + i * TL_WAVE;
        if (d < hd) o[i] = fmaf(pj, to_f32(vp[d]), o[i]);
      }
    }
    m = m_new;
  }
  T* orow = out + (int64_t)t * out_stride + (int64_t)h * hd;
#pragma unroll
  for (int i = 0; i < kDPL; ++i) {
    const int d = lane + i * TL_WAVE;
    if (d < hd) orow[d] = from_f32<T>(o[i] / l);
  }
}

}  // namespace

extern "C" {

// q: [n_tokens, nq*hd] with row stride q_stride (elements); out likewise.
// caches: [num_blocks, nkv, block_size, hd].  block_tables: [n_requests, max_blocks].
int tl_paged_attention(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                       const int32_t* block_tables, int max_blocks, const int32_t* req_of_token,
                       const int32_t* positions, void* out, int64_t out_stride, int n_tokens, int nq,
                       int nkv, int hd, int block_size, float scale, int window, int dtype,
                       hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (nq <= 0 || nkv <= 0 || nq % nkv || hd <= 0 || hd > kMaxHd || block_size <= 0 || max_blocks <= 0 ||
      window < 0 || nq > 65535)
    return TL_ERR_ARG;
  dim3 g(n_tokens, nq), b(TL_WAVE);
  if (dtype == 0)
    hipLaunchKernelGGL(paged_attention_kernel<float>, g, b, 0, stream, (const float*)q, q_stride,
                       (const float*)k_cache, (const float*)v_cache, block_tables, max_blocks, req_of_token,
                       positions, (float*)out, out_stride, nq, nkv, hd, block_size, scale, window);
  else if (dtype == 1)
    hipLaunchKernelGGL(paged_attention_kernel<bf16_t>, g, b, 0, stream, (const bf16_t*)q, q_stride,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_tables, max_blocks, req_of_token,
                       positions, (bf16_t*)out, out_stride, nq, nkv, hd, block_size, scale, window);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

}  // extern "C"
