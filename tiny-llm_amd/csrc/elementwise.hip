// Memory-bound kernels of the step: embedding gather, RMSNorm (with optional
// row gather), SiLU-gate, residual add, and rotary position encoding fused with
// the write of keys and values into the paged cache.
//
// Formulas follow the reference's kernels: tiny_llm/ops/cuda/embedding.cu:10-29,
// norm.cu:29-48, silu.cu:10, arithmetic.cu:13, rope.cu:46-54 and 73-93.
// The residual stream is float32 in both precisions; T is the element type of
// weights, activations and cache (float or bf16).
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / TL_WAVE;

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embedding_kernel(const int32_t* __restrict__ tokens, const T* __restrict__ table,
                                 float* __restrict__ out, int hidden, int vocab) {
  const int t = blockIdx.x;
  const int tok = tokens[t];
  float* dst = out + (int64_t)t * hidden;
  if (tok < 0 || tok >= vocab) {  // ids are checked on the host; poison instead of reading outside
    for (int j = threadIdx.x; j < hidden; j += kThreads) dst[j] = __builtin_nanf("");
    return;
  }
  const T* src = table + (int64_t)tok * hidden;
  for (int j = threadIdx.x; j < hidden; j += kThreads) dst[j] = to_f32(src[j]);
}

// -------------------------------------------------------------------- RMSNorm
// y = w * x / sqrt(mean(x^2) + eps), statistics in float32.  One workgroup per
// output row; `rows` (optional) selects the input row of each output row.
template <typename TW, typename TO>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                               const int32_t* __restrict__ rows, TO* __restrict__ out, int hidden,
                               float eps) {
  __shared__ float red[kWaves];
  const int64_t in_row = rows ? rows[blockIdx.x] : blockIdx.x;
  const float* src = x + in_row * hidden;
  float ss = 0.f;
  for (int j = threadIdx.x; j < hidden; j += kThreads) {
    const float v = src[j];
    ss += v * v;
  }
  ss = block_sum<kWaves>(ss, red);
  const float r = sqrtf(ss / (float)hidden + eps);
  TO* dst = out + (int64_t)blockIdx.x * hidden;
  for (int j = threadIdx.x; j < hidden; j += kThreads) dst[j] = from_f32<TO>(to_f32(w[j]) * src[j] / r);
}

// --------------------------------------------------- RMSNorm, scale left out
// out = bf16(w * x) and inv_rms = 1 / sqrt(mean(x^2) + eps) per row: the operand of a product that
// applies the row factor to its result (the few-row product does the same inside its kernel).
template <typename TW>
__global__ void norm_prescale_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                                     const int32_t* __restrict__ rows, bf16_t* __restrict__ out,
                                     float* __restrict__ inv_rms, int hidden, float eps) {
  __shared__ float red[kWaves];
  const int64_t in_row = rows ? rows[blockIdx.x] : blockIdx.x;
  const float* src = x + in_row * hidden;
  bf16_t* dst = out + (int64_t)blockIdx.x * hidden;
  float ss = 0.f;
  const bool aligned = (((uintptr_t)x | (uintptr_t)out) & 15) == 0 && ((uintptr_t)w & (4 * sizeof(TW) - 1)) == 0;
  if (hidden % 4 == 0 && aligned) {       // four elements per access
    for (int j = threadIdx.x * 4; j < hidden; j += kThreads * 4) {
      const f32x4 v = *(const f32x4*)(src + j);
      float wv[4];
      if constexpr (sizeof(TW) == 4) {
        const f32x4 w4 = *(const f32x4*)(w + j);
        wv[0] = w4[0]; wv[1] = w4[1]; wv[2] = w4[2]; wv[3] = w4[3];
      } else {
        const bf16x4 w4 = *(const bf16x4*)(w + j);
        wv[0] = (float)w4[0]; wv[1] = (float)w4[1]; wv[2] = (float)w4[2]; wv[3] = (float)w4[3];
      }
      ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
      bf16x4 o = {(bf16_t)(wv[0] * v[0]), (bf16_t)(wv[1] * v[1]), (bf16_t)(wv[2] * v[2]), (bf16_t)(wv[3] * v[3])};
      *(bf16x4*)(dst + j) = o;
    }
  } else {
    for (int j = threadIdx.x; j < hidden; j += kThreads) {
      const float v = src[j];
      ss += v * v;
      dst[j] = (bf16_t)(to_f32(w[j]) * v);
    }
  }
  ss = block_sum<kWaves>(ss, red);
  if (threadIdx.x == 0) inv_rms[blockIdx.x] = 1.f / sqrtf(ss / (float)hidden + eps);
}

// ------------------------------------------------------------------ SiLU-gate
// z[t, j] = silu(gate_up[t, j]) * gate_up[t, I + j]
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ z, int64_t total, int inter) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / inter;
  const int j = (int)(i - t * inter);
  const float g = to_f32(gate_up[t * 2 * inter + j]);
  const float u = to_f32(gate_up[t * 2 * inter + inter + j]);
  z[i] = from_f32<T>(g / (1.f + expf(-g)) * u);
}

// --------------------------------------------------------------- residual add
template <typename T>
__global__ void add_residual_kernel(float* __restrict__ x, const T* __restrict__ y, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < total) x[i] += to_f32(y[i]);
}

// ------------------------------------------------------ rotary + cache write
// qkv row t = [q heads | k heads | v heads], each head `hd` wide.  The first
// `rot` dims of every q and k head are rotated by the angle table row positions[t]:
// pair i is the dims (i, i + rot/2) (rotate-half pairing, interleaved == 0) or the
// dims (2i, 2i + 1) (interleaved pairing); q is rewritten in place,
// k (rotated) and v go to the cache slot slot_mapping[t] (a negative slot
// stores nothing).  Cache layout: [block, kv_head, slot_in_block, hd].
template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, const int32_t* __restrict__ positions,
                                  const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                  const int32_t* __restrict__ slot_mapping, T* __restrict__ k_cache,
                                  T* __restrict__ v_cache, int nq, int nkv, int hd, int rot,
                                  int block_size, int64_t row_stride, int interleaved, int heads_wg) {
  // blockIdx.y: a run of `heads_wg` of the token's q and k heads (a k head brings its v head along), so
  // that a step of few tokens still is a launch of many workgroups
  const int t = blockIdx.x;
  const int head0 = blockIdx.y * heads_wg, head1 = min(nq + nkv, head0 + heads_wg);
  const int kv0 = max(head0, nq) - nq, kv1 = max(head1, nq) - nq;        // the kv heads among them
  const int pos = positions[t];
  const int half = rot / 2;
  const int slot = slot_mapping ? slot_mapping[t] : -1;
  T* row = qkv + (int64_t)t * row_stride;
  const float* cs = cos_t + (int64_t)pos * half;
  const float* sn = sin_t + (int64_t)pos * half;
  const int64_t blk = slot >= 0 ? slot / block_size : 0;
  const int in_blk = slot >= 0 ? slot % block_size : 0;

  if constexpr (sizeof(T) == 2) {
    // bfloat16, whole heads rotated, halves that are multiples of 8 and 16-byte aligned rows:
    // eight pairs per thread and 16-byte accesses throughout
    const bool aligned = (((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache | (uintptr_t)cos_t |
                           (uintptr_t)sin_t) & 15) == 0;
    if (rot == hd && half % 8 == 0 && row_stride % 8 == 0 && aligned && !interleaved) {
      const int chunks = half / 8;
      for (int i = threadIdx.x; i < (head1 - head0) * chunks; i += kThreads) {
        const int head = head0 + i / chunks, j = (i % chunks) * 8;
        bf16_t* h = (bf16_t*)row + (int64_t)head * hd;
        const bf16x8 a8 = *(const bf16x8*)(h + j), b8 = *(const bf16x8*)(h + j + half);
        const f32x4 c0 = *(const f32x4*)(cs + j), c1 = *(const f32x4*)(cs + j + 4);
        const f32x4 s0 = *(const f32x4*)(sn + j), s1 = *(const f32x4*)(sn + j + 4);
        bf16x8 ra, rb;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = e < 4 ? c0[e] : c1[e - 4], sv = e < 4 ? s0[e] : s1[e - 4];
          const float a = (float)a8[e], b = (float)b8[e];
          ra[e] = (bf16_t)(c * a - sv * b);
          rb[e] = (bf16_t)(sv * a + c * b);
        }
        if (head < nq) {
          *(bf16x8*)(h + j) = ra;
          *(bf16x8*)(h + j + half) = rb;
        } else if (slot >= 0) {
          bf16_t* dst = (bf16_t*)k_cache + ((blk * nkv + (head - nq)) * block_size + in_blk) * hd;
          *(bf16x8*)(dst + j) = ra;
          *(bf16x8*)(dst + j + half) = rb;
        }
      }
      if (slot < 0) return;
      for (int i = threadIdx.x; i < (kv1 - kv0) * (hd / 8); i += kThreads) {
        const int head = kv0 + i / (hd / 8), j = (i % (hd / 8)) * 8;
        *(bf16x8*)((bf16_t*)v_cache + ((blk * nkv + head) * block_size + in_blk) * hd + j) =
            *(const bf16x8*)((const bf16_t*)row + (int64_t)(nq + nkv + head) * hd + j);
      }
      return;
    }
  }
  // rotated pairs of q and k heads
  const int pairs = (head1 - head0) * half;
  for (int i = threadIdx.x; i < pairs; i += kThreads) {
    const int head = head0 + i / half, j = i % half;
    const int ia = interleaved ? 2 * j : j, ib = interleaved ? 2 * j + 1 : j + half;
    T* h = row + (int64_t)head * hd;
    const float a = to_f32(h[ia]), b = to_f32(h[ib]);
    const float c = cs[j], s = sn[j];
    const T ra = from_f32<T>(c * a - s * b);
    const T rb = from_f32<T>(s * a + c * b);
    if (head < nq) {
      h[ia] = ra;
      h[ib] = rb;
    } else if (slot >= 0) {
      T* dst = k_cache + ((blk * nkv + (head - nq)) * block_size + in_blk) * hd;
      dst[ia] = ra;
      dst[ib] = rb;
    }
  }
  if (slot < 0) return;
  // dims of k beyond the rotated part, and all of v, are copied as they are
  const int tail = hd - rot;
  for (int i = threadIdx.x; i < (kv1 - kv0) * tail; i += kThreads) {
    const int head = kv0 + i / tail, j = rot + i % tail;
    k_cache[((blk * nkv + head) * block_size + in_blk) * hd + j] = row[(int64_t)(nq + head) * hd + j];
  }
  for (int i = threadIdx.x; i < (kv1 - kv0) * hd; i += kThreads) {
    const int head = kv0 + i / hd, j = i % hd;
    v_cache[((blk * nkv + head) * block_size + in_blk) * hd + j] = row[(int64_t)(nq + nkv + head) * hd + j];
  }
}

// ------------------------------------------------------- seeded normal numbers
// out[i] = shift + scale * table[splitmix64(key + (i + 1) * golden) >> (64 - table_bits)]: a pure
// function of (key, i).  The product and the sum are rounded to float32 one after the other (no
// fused multiply-add), so a host that does the same two operations gets the same bits.
template <typename T>
__global__ void random_normal_kernel(T* __restrict__ out, int64_t n, uint64_t key, const float* __restrict__ table,
                                     int table_bits, float scale, float shift) {
  for (int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (int64_t)gridDim.x * kThreads) {
    uint64_t x = key + ((uint64_t)i + 1ull) * 0x9E3779B97F4A7C15ull;
    x ^= x >> 30;
    x *= 0xBF58476D1CE4E5B9ull;
    x ^= x >> 27;
    x *= 0x94D049BB133111EBull;
    x ^= x >> 31;
    const float z = table[x >> (64 - table_bits)];
    float v;
    {
#pragma clang fp contract(off)      // two roundings, as on the host: never one fused multiply-add
      const float p = scale * z;
      v = p + shift;
    }
    out[i] = from_f32<T>(v);
  }
}

// ------------------------------------------------- a decode step feeds the next
// After a decode step's sampler: the chosen token of every request becomes its next input, its
// position, cached length and sampling counter go up by one, and its cache slot is looked up in
// the block table for the new position.  A run of decode steps can then be replayed back to back
// without the host in between; `history` [history_steps, R] keeps what each step chose.
constexpr int TL_MAX_CACHE_GROUPS = 16;     // cache groups a model may have and still chain decode steps on the device
struct AdvanceArgs {
  int32_t* tokens;
  int32_t* positions;
  int32_t* seq_lens;
  int32_t* counters;
  const int32_t* sampled;
  int32_t* history;
  int32_t* step;           // how many steps have run since the host last wrote the metadata
  int R, G, MB, block_size, history_steps;
  int32_t* slots[TL_MAX_CACHE_GROUPS];
  const int32_t* tables[TL_MAX_CACHE_GROUPS];
};

__global__ void decode_advance_kernel(const AdvanceArgs a) {
  const int s = *a.step;
  __syncthreads();          // every thread has read the step before thread 0 moves it on
  for (int r = threadIdx.x; r < a.R; r += blockDim.x) {
    const int tok = a.sampled[r];
    if (s < a.history_steps) a.history[(int64_t)s * a.R + r] = tok;
    a.tokens[r] = tok;
    const int p = a.positions[r] + 1;
    a.positions[r] = p;
    a.seq_lens[r] += 1;
    a.counters[r] += 1;
    for (int g = 0; g < a.G; ++g) {
      const int blk = max(a.tables[g][(int64_t)r * a.MB + min(p / a.block_size, a.MB - 1)], 0);
      a.slots[g][r] = blk * a.block_size + p % a.block_size;
    }
  }
  if (threadIdx.x == 0) *a.step = s + 1;
}

}  // namespace

#define TL_DISPATCH_T(dtype, ...)                 \
  if ((dtype) == 0) { using T = float; __VA_ARGS__ } \
  else if ((dtype) == 1) { using T = bf16_t; __VA_ARGS__ } \
  else return TL_ERR_ARG;

extern "C" {

int tl_embedding(const int32_t* tokens, const void* table, float* out, int n_tokens, int hidden,
                 int vocab, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (hidden <= 0 || vocab <= 0) return TL_ERR_ARG;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(embedding_kernel<T>, dim3(n_tokens), dim3(kThreads), 0, stream,
                                          tokens, (const T*)table, out, hidden, vocab);)
  return tl_launch_status();
}

// w_dtype / out_dtype: 0 float32, 1 bfloat16.  rows may be null.
int tl_rmsnorm(const float* x, const void* w, const int32_t* rows, void* out, int n_rows, int hidden,
               float eps, int w_dtype, int out_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (hidden <= 0) return TL_ERR_ARG;
  dim3 g(n_rows), b(kThreads);
  if (w_dtype == 0 && out_dtype == 0)
    hipLaunchKernelGGL((rmsnorm_kernel<float, float>), g, b, 0, stream, x, (const float*)w, rows, (float*)out, hidden, eps);
  else if (w_dtype == 1 && out_dtype == 0)
    hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, float>), g, b, 0, stream, x, (const bf16_t*)w, rows, (float*)out, hidden, eps);
  else if (w_dtype == 0 && out_dtype == 1)
    hipLaunchKernelGGL((rmsnorm_kernel<float, bf16_t>), g, b, 0, stream, x, (const float*)w, rows, (bf16_t*)out, hidden, eps);
  else if (w_dtype == 1 && out_dtype == 1)
    hipLaunchKernelGGL((rmsnorm_kernel<bf16_t, bf16_t>), g, b, 0, stream, x, (const bf16_t*)w, rows, (bf16_t*)out, hidden, eps);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_norm_prescale(const float* x, const void* w, const int32_t* rows, void* out, float* inv_rms, int n_rows,
                      int hidden, float eps, int w_dtype, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (hidden <= 0) return TL_ERR_ARG;
  dim3 g(n_rows), b(kThreads);
  if (w_dtype == 0)
    hipLaunchKernelGGL(norm_prescale_kernel<float>, g, b, 0, stream, x, (const float*)w, rows, (bf16_t*)out, inv_rms,
                       hidden, eps);
  else if (w_dtype == 1)
    hipLaunchKernelGGL(norm_prescale_kernel<bf16_t>, g, b, 0, stream, x, (const bf16_t*)w, rows, (bf16_t*)out,
                       inv_rms, hidden, eps);
  else
    return TL_ERR_ARG;
  return tl_launch_status();
}

int tl_silu_mul(const void* gate_up, void* z, int n_tokens, int inter, int dtype, hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (inter <= 0) return TL_ERR_ARG;
  const int64_t total = (int64_t)n_tokens * inter;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(silu_mul_kernel<T>, dim3((unsigned)ceil_div64(total, kThreads)),
                                          dim3(kThreads), 0, stream, (const T*)gate_up, (T*)z, total, inter);)
  return tl_launch_status();
}

int tl_add_residual(float* x, const void* y, int64_t total, int dtype, hipStream_t stream) {
  if (total <= 0) return TL_OK;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(add_residual_kernel<T>, dim3((unsigned)ceil_div64(total, kThreads)),
                                          dim3(kThreads), 0, stream, x, (const T*)y, total);)
  return tl_launch_status();
}

int tl_rope_store(void* qkv, const int32_t* positions, const float* cos_t, const float* sin_t,
                  const int32_t* slot_mapping, void* k_cache, void* v_cache, int n_tokens, int nq,
                  int nkv, int hd, int rot, int block_size, int64_t row_stride, int dtype, int interleaved,
                  hipStream_t stream) {
  if (n_tokens <= 0) return TL_OK;
  if (nq < 0 || nkv < 0 || hd <= 0 || rot < 0 || rot > hd || (rot & 1) || block_size <= 0) return TL_ERR_ARG;
  if (interleaved != 0 && interleaved != 1) return TL_ERR_ARG;
  if (rot > 0 && (!cos_t || !sin_t)) return TL_ERR_ARG;
  if (slot_mapping && (!k_cache || !v_cache)) return TL_ERR_ARG;
  // about 256 workgroups where the tokens alone are fewer: the heads of a token shared out
  const int heads = nq + nkv;
  int groups = n_tokens >= 256 ? 1 : (256 + n_tokens - 1) / n_tokens;
  if (groups > heads) groups = heads;
  const int heads_wg = (heads + groups - 1) / groups;
  groups = (heads + heads_wg - 1) / heads_wg;
  TL_DISPATCH_T(dtype, hipLaunchKernelGGL(rope_store_kernel<T>, dim3(n_tokens, groups), dim3(kThreads), 0, stream,
                                          (T*)qkv, positions, cos_t, sin_t, slot_mapping, (T*)k_cache,
                                          (T*)v_cache, nq, nkv, hd, rot, block_size, row_stride, interleaved,
                                          heads_wg);)
  return tl_launch_status();
}

// Seeded normal numbers (random-weights mode).  table: 2^table_bits float32 quantiles of N(0, 1).
int tl_random_normal(void* out, int64_t n, uint64_t key, const float* table, int table_bits, float scale,
                     float shift, int dtype, hipStream_t stream) {
  if (n <= 0) return TL_OK;
  if (table_bits < 1 || table_bits > 30 || (dtype != 0 && dtype != 1)) return TL_ERR_ARG;
  const int blocks = (int)(ceil_div64(n, kThreads) < 65536 ? ceil_div64(n, kThreads) : 65536);
  if (dtype == 0)
    hipLaunchKernelGGL(random_normal_kernel<float>, dim3(blocks), dim3(kThreads), 0, stream, (float*)out, n, key,
                       table, table_bits, scale, shift);
  else
    hipLaunchKernelGGL(random_normal_kernel<bf16_t>, dim3(blocks), dim3(kThreads), 0, stream, (bf16_t*)out, n, key,
                       table, table_bits, scale, shift);
  return tl_launch_status();
}

// One workgroup: R requests, G <= 16 cache groups with block tables [R, MB].
int tl_decode_advance(int32_t* tokens, int32_t* positions, int32_t* seq_lens, int32_t* counters,
                      const int32_t* sampled, int32_t* history, int32_t* step, int R, int G, int MB, int block_size,
                      int history_steps, int32_t* const* slots, const int32_t* const* tables, hipStream_t stream) {
  if (R <= 0) return TL_OK;
  if (G < 0 || G > TL_MAX_CACHE_GROUPS || MB <= 0 || block_size <= 0 || history_steps < 0 || !tokens || !positions || !seq_lens ||
      !counters || !sampled || !history || !step)
    return TL_ERR_ARG;
  AdvanceArgs a{tokens, positions, seq_lens, counters, sampled, history, step, R, G, MB, block_size, history_steps, {}, {}};
  for (int g = 0; g < G; ++g) {
    if (!slots[g] || !tables[g]) return TL_ERR_ARG;
    a.slots[g] = slots[g];
    a.tables[g] = tables[g];
  }
  hipLaunchKernelGGL(decode_advance_kernel, dim3(1), dim3(kThreads), 0, stream, a);
  return tl_launch_status();
}

}  // extern "C"
