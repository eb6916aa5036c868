// Token selection on the device: greedy argmax, or the reference's processor
// chain temperature -> top-k -> top-p -> multinomial
// (tiny_llm/pipeline/pipeline.cpp:156-164) without sorting the vocabulary.
//
// What the chain computes, written for a row sorted by descending logit
// (tiny_llm/logit_processors/sort_processors.cpp:54-142, sample_processors.cpp:7-54,
// temperature_processor.hpp:12-19, argmax_processor.cpp:6-35):
//   x_i = logit_i * (1/T);  keep the k largest;  prob_i = exp(x_i - x_0) / Z over the kept ones;
//   keep the shortest prefix whose probability reaches p (at least one token);
//   renormalise and take the first token at which the running sum exceeds u in [0,1).
// All three cuts are "the first place in the sorted order where a running measure
// (a count, or probability mass) reaches a target".  That place is found by radix
// descent over the bits of the logit: four passes, each a 256-bin histogram of the
// measure over the keys that share the prefix found so far.  Ties (equal logits)
// are ordered by token id.  Mass is kept as 64-bit fixed point (2^-40 units) and
// added with integer atomics, so the result does not depend on the order in which
// threads arrive and a (seed, position) pair always gives the same token.
//
// One workgroup per row.  u comes from a counter-based generator keyed by the
// row's seed and the row's position counter.
#include "common.h"

namespace {

constexpr int S_THREADS = 1024;
constexpr int S_WAVES = S_THREADS / TL_WAVE;
constexpr double kFix = 1099511627776.0;  // 2^40

__device__ __forceinline__ uint32_t order_key(float x) {
  if (x != x) return 0u;  // NaN sorts last
  const uint32_t b = __float_as_uint(x);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t k) {
  const uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(b);
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

struct Shared {
  unsigned long long hmass[256];
  unsigned int hcnt[256];
  unsigned long long red64[S_WAVES];
  unsigned int red32[S_WAVES];
  // result of one histogram scan
  unsigned int bin;
  unsigned long long above_mass;
  unsigned int above_cnt;
  unsigned long long bin_mass;
  unsigned int bin_cnt;
  int token;
};

struct Row {
  const float* logits;
  int vocab;
  float inv_t;
  float xmax;
};

__device__ __forceinline__ float scaled(const Row& r, int i) { return r.logits[i] * r.inv_t; }

__device__ __forceinline__ unsigned long long mass_of(const Row& r, float x) {
  return (unsigned long long)((double)expf(x - r.xmax) * kFix);
}

// Finds the key K* at which the running measure, taken over keys in descending
// order, first reaches `target` (>= 1).  by_mass selects the measure.  On return
// (in sh): above_mass / above_cnt = mass and count of keys > K*; bin_mass / bin_cnt
// = mass and count of keys == K*.  Returns K*.
__device__ uint32_t descend(const Row& r, Shared& sh, bool by_mass, unsigned long long target) {
  uint32_t prefix = 0;
  unsigned long long above_mass = 0;
  unsigned int above_cnt = 0;
  for (int shift = 24; shift >= 0; shift -= 8) {
    for (int b = threadIdx.x; b < 256; b += S_THREADS) {
      sh.hmass[b] = 0;
      sh.hcnt[b] = 0;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < r.vocab; i += S_THREADS) {
      const float x = scaled(r, i);
      const uint32_t key = order_key(x);
      const bool match = (shift == 24) || ((key >> (shift + 8)) == (prefix >> (shift + 8)));
      if (match) {
        const int bin = (key >> shift) & 255;
        atomicAdd(&sh.hmass[bin], mass_of(r, x));
        atomicAdd(&sh.hcnt[bin], 1u);
      }
    }
    __syncthreads();
    if (threadIdx.x < TL_WAVE) {
      // lane L owns bins 255-4L .. 252-4L, i.e. the scan runs from the largest keys down
      const int lane = threadIdx.x;
      unsigned long long lm[4], tm = 0;
      unsigned int lc[4], tc = 0;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        lm[i] = sh.hmass[255 - 4 * lane - i];
        lc[i] = sh.hcnt[255 - 4 * lane - i];
        tm += lm[i];
        tc += lc[i];
      }
      unsigned long long im = tm;  // inclusive scan over lanes
      unsigned int ic = tc;
#pragma unroll
      for (int off = 1; off < TL_WAVE; off <<= 1) {
        const unsigned long long um = __shfl_up(im, off, TL_WAVE);
        const unsigned int uc = __shfl_up(ic, off, TL_WAVE);
        if (lane >= off) {
          im += um;
          ic += uc;
        }
      }
      unsigned long long run_m = above_mass + (im - tm);
      unsigned int run_c = above_cnt + (ic - tc);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const unsigned long long before = by_mass ? run_m : (unsigned long long)run_c;
        const unsigned long long after = by_mass ? run_m + lm[i] : (unsigned long long)(run_c + lc[i]);
        if (before < target && after >= target) {
          sh.bin = 255 - 4 * lane - i;
          sh.above_mass = run_m;
          sh.above_cnt = run_c;
          sh.bin_mass = lm[i];
          sh.bin_cnt = lc[i];
        }
        run_m += lm[i];
        run_c += lc[i];
      }
    }
    __syncthreads();
    prefix |= (uint32_t)sh.bin << shift;
    above_mass = sh.above_mass;
    above_cnt = sh.above_cnt;
    __syncthreads();
  }
  return prefix;
}

// Token id of the n-th (1-based) element, in ascending id order, whose key equals `key`.
__device__ int nth_with_key(const Row& r, Shared& sh, uint32_t key, unsigned int n) {
  const int chunk = (r.vocab + S_THREADS - 1) / S_THREADS;
  const int begin = min(r.vocab, (int)threadIdx.x * chunk), end = min(r.vocab, begin + chunk);
  unsigned int cnt = 0;
  for (int i = begin; i < end; ++i) cnt += order_key(scaled(r, i)) == key;
  // exclusive scan of cnt over the workgroup: within the wave, then over wave totals
  const int lane = threadIdx.x % TL_WAVE, wave = threadIdx.x / TL_WAVE;
  unsigned int inc = cnt;
#pragma unroll
  for (int off = 1; off < TL_WAVE; off <<= 1) {
    const unsigned int up = __shfl_up(inc, off, TL_WAVE);
    if (lane >= off) inc += up;
  }
  if (lane == TL_WAVE - 1) sh.red32[wave] = inc;
  if (threadIdx.x == 0) sh.token = -1;
  __syncthreads();
  unsigned int base = 0;
  for (int wv = 0; wv < wave; ++wv) base += sh.red32[wv];
  const unsigned int before = base + inc - cnt;
  if (before < n && before + cnt >= n) {
    unsigned int seen = before;
    for (int i = begin; i < end; ++i)
      if (order_key(scaled(r, i)) == key && ++seen == n) {
        sh.token = i;
        break;
      }
  }
  __syncthreads();
  const int tok = sh.token;
  __syncthreads();
  return tok;
}

__global__ __launch_bounds__(S_THREADS) void sample_kernel(
    const float* __restrict__ logits, int64_t row_stride, int vocab, const float* __restrict__ temperature,
    const int32_t* __restrict__ top_k, const float* __restrict__ top_p, const int64_t* __restrict__ seeds,
    const int32_t* __restrict__ counters, int32_t* __restrict__ out) {
  __shared__ Shared sh;
  const int row = blockIdx.x;
  Row r;
  r.logits = logits + (int64_t)row * row_stride;
  r.vocab = vocab;
  const float temp = temperature ? temperature[row] : 0.f;
  const bool greedy = !(temp > 0.f);
  r.inv_t = greedy ? 1.f : 1.f / temp;
  r.xmax = 0.f;

  if (greedy) {
    // One pass: the largest (key, lowest index) pair.  The index is stored inverted in the low
    // half, so the maximum of the pairs is the first maximum of the row.
    unsigned long long best = 0;
    const bool vec = (vocab % 4 == 0) && (((uintptr_t)r.logits & 15) == 0);
    if (vec) {
      for (int i = threadIdx.x * 4; i < vocab; i += S_THREADS * 4) {
        const f32x4 x = *(const f32x4*)(r.logits + i);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          best = max(best, ((unsigned long long)order_key(x[e]) << 32) | (uint32_t)(0xffffffffu - (uint32_t)(i + e)));
      }
    } else {
      for (int i = threadIdx.x; i < vocab; i += S_THREADS)
        best = max(best, ((unsigned long long)order_key(r.logits[i]) << 32) | (uint32_t)(0xffffffffu - (uint32_t)i));
    }
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) {
      const uint32_t hi = (uint32_t)__shfl_xor((int)(best >> 32), off, TL_WAVE);
      const uint32_t lo = (uint32_t)__shfl_xor((int)(best & 0xffffffffu), off, TL_WAVE);
      best = max(best, ((unsigned long long)hi << 32) | lo);
    }
    if (threadIdx.x % TL_WAVE == 0) sh.red64[threadIdx.x / TL_WAVE] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
      for (int wv = 0; wv < S_WAVES; ++wv) best = max(best, sh.red64[wv]);
      out[row] = (int32_t)(0xffffffffu - (uint32_t)(best & 0xffffffffu));
    }
    return;
  }

  // maximum key of the row
  uint32_t kmax = 0;
  for (int i = threadIdx.x; i < vocab; i += S_THREADS) kmax = max(kmax, order_key(scaled(r, i)));
#pragma unroll
  for (int off = TL_WAVE / 2; off > 0; off >>= 1) kmax = max(kmax, (uint32_t)__shfl_xor((int)kmax, off, TL_WAVE));
  if (threadIdx.x % TL_WAVE == 0) sh.red32[threadIdx.x / TL_WAVE] = kmax;
  __syncthreads();
  kmax = 0;
  for (int wv = 0; wv < S_WAVES; ++wv) kmax = max(kmax, sh.red32[wv]);
  __syncthreads();

  r.xmax = key_value(kmax);

  // top-k: mass of the k largest
  unsigned long long z;
  const int k = top_k ? top_k[row] : 0;
  if (k > 0 && k < vocab) {
    descend(r, sh, false, (unsigned long long)k);
    const unsigned int ties = (unsigned int)k - sh.above_cnt;
    const unsigned long long w = sh.bin_mass / sh.bin_cnt;
    z = sh.above_mass + (unsigned long long)ties * w;
    __syncthreads();
  } else {
    unsigned long long part = 0;
    for (int i = threadIdx.x; i < vocab; i += S_THREADS) part += mass_of(r, scaled(r, i));
#pragma unroll
    for (int off = TL_WAVE / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, TL_WAVE);
    if (threadIdx.x % TL_WAVE == 0) sh.red64[threadIdx.x / TL_WAVE] = part;
    __syncthreads();
    z = 0;
    for (int wv = 0; wv < S_WAVES; ++wv) z += sh.red64[wv];
    __syncthreads();
  }

  // top-p: shortest prefix whose mass reaches p * z
  const float p = top_p ? top_p[row] : 1.f;
  if (p < 1.f) {
    unsigned long long target = (unsigned long long)((double)fmaxf(p, 0.f) * (double)z);
    target = min(max(target, 1ull), z);
    descend(r, sh, true, target);
    const unsigned long long w = max(sh.bin_mass / sh.bin_cnt, 1ull);
    unsigned long long ties = (target - sh.above_mass + w - 1) / w;
    ties = min(max(ties, 1ull), (unsigned long long)sh.bin_cnt);
    z = sh.above_mass + ties * w;
    __syncthreads();
  }

  // multinomial: first token at which the running mass exceeds u * z
  const uint64_t seed = seeds ? (uint64_t)seeds[row] : 0ull;
  const uint64_t ctr = counters ? (uint64_t)(uint32_t)counters[row] : 0ull;
  const uint64_t bits = splitmix64(splitmix64(seed) ^ (ctr * 0xD1B54A32D192ED03ull));
  const double u = (double)(bits >> 40) * (1.0 / 16777216.0);  // 24 bits, [0, 1)
  unsigned long long target = (unsigned long long)(u * (double)z) + 1ull;
  target = min(target, z);
  const uint32_t key = descend(r, sh, true, target);
  const unsigned long long w = max(sh.bin_mass / sh.bin_cnt, 1ull);
  unsigned long long nth = (target - sh.above_mass + w - 1) / w;
  nth = min(max(nth, 1ull), (unsigned long long)sh.bin_cnt);
  __syncthreads();
  const int tok = nth_with_key(r, sh, key, (unsigned int)nth);
  if (threadIdx.x == 0) out[row] = tok;
}

}  // namespace

extern "C" {

// temperature[row] <= 0 (or a null pointer) selects greedy argmax for that row.
// top_k[row] <= 0 or >= vocab keeps every token; top_p[row] >= 1 keeps every token.
int tl_sample(const float* logits, int64_t row_stride, int n_rows, int vocab, const float* temperature,
              const int32_t* top_k, const float* top_p, const int64_t* seeds, const int32_t* counters,
              int32_t* out, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (vocab <= 0 || row_stride < vocab) return TL_ERR_ARG;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(S_THREADS), 0, stream, logits, row_stride, vocab,
                     temperature, top_k, top_p, seeds, counters, out);
  return tl_launch_status();
}

}  // extern "C"
