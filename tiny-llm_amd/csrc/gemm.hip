// Linear layers: out[m, n] = sum_k a[m, k] * w[n, k] (+ residual[m, n]).
// Weights are [out, in] row-major as in the checkpoint, the contraction the
// reference's GEMM family computes (tiny_llm/ops/cuda/gemm.cu:86-100); the
// residual add that the reference runs as a separate kernel
// (tiny_llm/ops/cuda/arithmetic.cu:13) is folded into the epilogue.
//
//  * gemm_f32_kernel (tiles of 128 x 128 or 64 x 64), and gemm_f32_rows_kernel for at most 64 rows:
//    true float32 on the matrix cores (v_mfma_f32_16x16x4_f32), no reduced-precision mode.  Both add
//    in ONE order, so a row gives the same bits whether it is computed alone or in a batch, by
//    either kernel.
//  * gemm_bf16_kernel: bf16 inputs on the matrix cores (v_mfma_f32_32x32x16_bf16), float32
//    accumulation, 256 x 256, 256 x 128, 128 x 128 or 64 x 128 tiles with k steps of 64 staged through
//    double-buffered LDS; optionally over a share of the inner size (split k).
//  * gemm_oneshot_bf16_kernel: the split product for few rows, operands streamed through a ring of
//    LDS slabs filled straight from memory; splitk_reduce_kernel adds the parts and applies the epilogue.
//  * gemm_skinny_bf16_kernel: at most 64 rows (decode steps), weights streamed once into registers.
#include <type_traits>

#include "common.h"

namespace {

// ===================================================================== float32
// True float32 on the matrix cores: v_mfma_f32_16x16x4_f32 takes float32 operands and keeps float32
// sums (no reduced-precision mode).  Both kernels below add the terms of an output element in ONE
// order, so that a row gives the same bits alone and in any batch, by either kernel:
//   * k runs in blocks of 256, each block summed from zero, the block sums added in ascending order;
//   * inside a block, groups of 16 k in ascending order; a group is four matrix instructions, the
//     e-th of which takes k = 16 group + {0, 4, 8, 12} + e (a lane holds four consecutive k of its row,
//     one for each of the four instructions);
//   * operands beyond K are zero.
constexpr int F_KBLOCK = 256;     // the k block of the order of addition
constexpr int F_BK = 16, F_THREADS = 256;
constexpr int F_LD = F_BK + 4;    // LDS row stride in floats (80 bytes: 16-byte aligned rows)

// silu(g) * u of an interleaved gate|up pair of output columns, as the reference computes it
// (tiny_llm/ops/cuda/silu.cu:10, arithmetic.cu:13), from the float32 accumulators.
__device__ __forceinline__ float swiglu_pair(float g, float u) { return g / (1.f + expf(-g)) * u; }
// The same for the bfloat16 kernels, whose result is rounded to 8 bits anyway: hardware exp2 and
// reciprocal (about 1 ulp of float32 each) instead of the library's exp and a full division, which
// were a tenth of the gate/up product's time.
__device__ __forceinline__ float swiglu_pair_fast(float g, float u) {
  return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.44269504088896341f * g)) * u;
}

// Four consecutive k of one row, zero beyond K; VEC: 16-byte aligned rows and K a multiple of 4.
template <bool VEC>
__device__ __forceinline__ f32x4 load_k4(const float* __restrict__ row, int k, int K) {
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  if constexpr (VEC) {
    if (k < K) v = *(const f32x4*)(row + k);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (k + e < K) v[e] = row[k + e];
  }
  return v;
}

// The factor of a row's RMSNorm from the sum of its squares: ONE expression for every kernel that
// takes part in a float32 norm, so that they agree to the bit.
__device__ __forceinline__ float f32_norm_factor(float sumsq, int K, float eps) {
  return 1.f / sqrtf(sumsq / (float)K + eps);
}

// The norm in front of a float32 product for any number of rows, as two kernels: this one writes
// h = norm_w * x (float32) and a row's factor 1 / rms; the product then multiplies its sums by the
// factor (row_scale).  The squares of a row are added up in the order of gemm_f32_rows_kernel<NORM>:
// per k block of 256 four chains (chain q takes k = 16 g + 4 q + e for g = 0..15, e = 0..3, in that
// order, by fused multiply-adds from zero), the chains as (c0 + c1) + (c2 + c3), the blocks in
// ascending order.  So a row's result has the same bits whether the norm rode in the few-row product
// or went through here: a row's logits do not depend on how many rows its step had.
constexpr int FN_THREADS = 256;
template <bool VEC>
__global__ __launch_bounds__(FN_THREADS) void norm_prescale_f32_kernel(const float* __restrict__ x,
                                                                       const float* __restrict__ norm_w,
                                                                       const int32_t* __restrict__ rows,
                                                                       float* __restrict__ h,
                                                                       float* __restrict__ inv_rms, int K,
                                                                       int64_t lda, float eps) {
  extern __shared__ float chain_sums[];     // [k blocks][4]
  const int m = blockIdx.x;
  const float* row = x + (int64_t)(rows ? rows[m] : m) * lda;
  float* dst = h + (int64_t)m * K;
  const int nkb = (K + F_KBLOCK - 1) / F_KBLOCK;
  for (int c = threadIdx.x; c < nkb * 4; c += FN_THREADS) {
    const int kb = (c >> 2) * F_KBLOCK, q = c & 3;
    // all sixteen pieces of the chain are requested before the first is used: one round trip, not sixteen
    f32x4 v[16], nw[16];
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      v[g] = load_k4<VEC>(row, kb + g * 16 + q * 4, K);
      nw[g] = load_k4<VEC>(norm_w, kb + g * 16 + q * 4, K);
    }
    float ss = 0.f;
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      const int k = kb + g * 16 + q * 4;
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ss = __builtin_fmaf(v[g][e], v[g][e], ss);
        o[e] = v[g][e] * nw[g][e];
      }
      if constexpr (VEC) {
        if (k < K) *(f32x4*)(dst + k) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (k + e < K) dst[k + e] = o[e];
      }
    }
    chain_sums[c] = ss;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int b = 0; b < nkb; ++b)
      total += (chain_sums[4 * b] + chain_sums[4 * b + 1]) + (chain_sums[4 * b + 2] + chain_sums[4 * b + 3]);
    inv_rms[m] = f32_norm_factor(total, K, eps);
  }
}

// Tiles of 32 T rows x 32 T columns, four waves of 16 T x 16 T (T x T matrix tiles of 16 x 16), k in
// steps of 16 through double-buffered LDS.  T = 4 (128 x 128) where that gives the chip enough
// tiles, T = 2 (64 x 64) where it does not (a portion of 512 tokens times 2048 columns is 64 tiles
// of 128 x 128 for 256 compute units); the order in which an output element is added up is the
// same for every T.  The matrix instruction's rows are the output COLUMNS (weights are its first
// operand), so a lane ends up with four consecutive columns of one row.
template <bool SWIGLU, bool VEC, int T>
__global__ __launch_bounds__(F_THREADS) void gemm_f32_kernel(const float* __restrict__ a,
                                                             const float* __restrict__ w,
                                                             float* __restrict__ out,
                                                             const float* __restrict__ residual, int M,
                                                             int N, int K, int64_t lda, int64_t ldo,
                                                             const float* __restrict__ row_scale) {
  constexpr int BT = 32 * T;        // rows and columns of the workgroup's tile
  constexpr int PIECES = BT / 64;   // 16-byte pieces of each operand per thread and k step
  static_assert(T == 2 || T == 4, "tiles of 64 x 64 or 128 x 128");
  __shared__ __attribute__((aligned(16))) float As[2][BT * F_LD];
  __shared__ __attribute__((aligned(16))) float Ws[2][BT * F_LD];
  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * BT, n0 = blockIdx.x * BT;
  const int l16 = lane % 16, kk = lane / 16;
  // staging: piece h of a thread is row (h * 256 + tid) / 4 of the tile, four k from 4 * (tid % 4)
  const int sr = tid / 4, sk = (tid % 4) * 4;
  const float *arow[PIECES], *wrow[PIECES];
#pragma unroll
  for (int h = 0; h < PIECES; ++h) {
    arow[h] = a + (int64_t)min(m0 + h * 64 + sr, M - 1) * lda;
    wrow[h] = w + (int64_t)min(n0 + h * 64 + sr, N - 1) * K;
  }
  f32x4 acc[T][T], tot[T][T];
#pragma unroll
  for (int nt = 0; nt < T; ++nt)
#pragma unroll
    for (int mt = 0; mt < T; ++mt) {
      acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      tot[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
  f32x4 ga[PIECES], gw[PIECES];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int h = 0; h < PIECES; ++h) {
      ga[h] = load_k4<VEC>(arow[h], k0 + sk, K);
      gw[h] = load_k4<VEC>(wrow[h], k0 + sk, K);
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int h = 0; h < PIECES; ++h) {
      *(f32x4*)(&As[buf][(h * 64 + sr) * F_LD + sk]) = ga[h];
      *(f32x4*)(&Ws[buf][(h * 64 + sr) * F_LD + sk]) = gw[h];
    }
  };
  fetch(0);
  stage(0);
  __syncthreads();
  const int steps = (K + F_BK - 1) / F_BK;
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) fetch((s + 1) * F_BK);
    f32x4 wv[T], av[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
      wv[t] = *(const f32x4*)(&Ws[buf][(wn * 16 * T + t * 16 + l16) * F_LD + kk * 4]);
      av[t] = *(const f32x4*)(&As[buf][(wm * 16 * T + t * 16 + l16) * F_LD + kk * 4]);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
#pragma unroll
      for (int nt = 0; nt < T; ++nt)
#pragma unroll
        for (int mt = 0; mt < T; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[nt][e], av[mt][e], acc[nt][mt], 0, 0, 0);
    if (((s + 1) * F_BK) % F_KBLOCK == 0 || s + 1 == steps) {     // a block of the order of addition ends
#pragma unroll
      for (int nt = 0; nt < T; ++nt)
#pragma unroll
        for (int mt = 0; mt < T; ++mt) {
          tot[nt][mt] += acc[nt][mt];
          acc[nt][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    if (s + 1 < steps) stage(buf ^ 1);
    __syncthreads();
  }
  // lane (l16, kk) of tile (nt, mt) holds row m = mt*16 + l16, columns n = nt*16 + 4 kk + r
#pragma unroll
  for (int mt = 0; mt < T; ++mt) {
    const int m = m0 + wm * 16 * T + mt * 16 + l16;
    if (m >= M) continue;
#pragma unroll
    for (int nt = 0; nt < T; ++nt) {
      const int n = n0 + wn * 16 * T + nt * 16 + kk * 4;
      f32x4 v = tot[nt][mt];
      if (row_scale) {      // the factor of a norm in front (norm_prescale_f32_kernel)
        const float f = row_scale[m];
#pragma unroll
        for (int r = 0; r < 4; ++r) v[r] *= f;
      }
      if constexpr (SWIGLU) {   // columns (2j, 2j+1) = (gate_j, up_j); N is even
#pragma unroll
        for (int r = 0; r < 4; r += 2)
          if (n + r < N) out[(int64_t)m * ldo + (n + r) / 2] = swiglu_pair(v[r], v[r + 1]);
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < N) {
            const int64_t at = (int64_t)m * ldo + n + r;
            out[at] = residual ? v[r] + residual[at] : v[r];
          }
      }
    }
  }
}

// The same product for few rows (decode steps): the weights stream once, straight from memory
// into the matrix instruction's operand registers.  A workgroup owns 16 output columns (8 where
// 16 would leave compute units without work: the matrix tile's other 8 rows then repeat them and
// are dropped); its eight waves deal the k blocks of 256 out among themselves, a wave requests a
// whole block (16 KB) at once and the next one before it multiplies; the block sums meet in LDS and
// are added in ascending order: the order of gemm_f32_kernel, to the bit.  Rows come in tiles of
// 16 (up to four).
constexpr int FR_WAVES = 8, FR_THREADS = FR_WAVES * TL_WAVE, FR_MAX_MT = 4;

//
// NORM: `a` is the float32 residual stream and the product is that of its RMSNorm,
// ((norm_w * a) @ w.T) / sqrt(mean(a^2) + eps): the rows are multiplied by the norm's weight as they
// are loaded, their squares are added up on the way (per k block and row in a fixed order, the
// blocks in ascending order, so a row's factor depends on nothing but the row), and the factor is
// applied to the block sums' total.  That saves the norm's kernel in front of the product.
//
// CT (one row tile only): a workgroup owns CT column tiles side by side.  The activations of a k block,
// which weigh as much as one tile's weights, are fetched once for all of them, and a wide product
// (gate and up, the output head) becomes one or two rounds of workgroups instead of three to eight.
// The weights come as a chain of pieces, the block's tiles and then the wave's next block, each
// requested while the piece before it is multiplied.  A tile's block sums are what they are with one
// tile a workgroup, bit for bit.
//
// PAIR (8 columns, at most 8 rows, no norm): the matrix tile of 16 x 16 then holds two k blocks at
// once.  Operand rows 0 to 7 are the 8 columns (and the 8 activation rows) at the k of one block, rows
// 8 to 15 the same columns and rows at the k of the next; the two diagonal 8 x 8 blocks of the result
// are the two block sums, each accumulated from zero in the order it has everywhere else, and the
// rest of the tile is dropped.  Without it the second half of the tile repeats the first: every load
// instruction then fetches half of what it could, and 8 columns are what bounds these products,
// since a workgroup is as fast as its loads.  A wave takes pairs of blocks instead of blocks.
template <bool SWIGLU, int COLS, bool NORM = false, bool WIDE = false, int CT = 1, bool PAIR = false>
__global__ __launch_bounds__(FR_THREADS) void gemm_f32_rows_kernel(const float* __restrict__ a,
                                                                   const float* __restrict__ w,
                                                                   float* __restrict__ out,
                                                                   const float* __restrict__ residual, int M,
                                                                   int N, int K, int64_t lda, int64_t ldo,
                                                                   const float* __restrict__ norm_w = nullptr,
                                                                   float eps = 0.f,
                                                                   const float* __restrict__ row_scale = nullptr,
                                                                   int tiles_wg = FR_MAX_MT, int cols_wg = 0) {
  // cols_wg (even, with CT column tiles of which the last is partly used): the columns a workgroup owns
  // where whole tiles would not make whole rounds of 256 workgroups; the tile's other columns repeat
  // the last one and are dropped.
  // WIDE (more than 16 rows): blockIdx.y picks a group of `tiles_wg` row tiles, so that a product with
  // few column tiles still gives every compute unit a workgroup with whole matrix tiles (16 columns)
  // instead of half-used ones (8 columns); the activations of the next row tile are requested before
  // this one is multiplied, and the registers that takes are those of the next block's weights, which
  // are requested behind the block's last row tile instead.
  static_assert(!(NORM && WIDE), "the norm rides in the product of one row tile");
  static_assert(CT >= 1 && CT <= 3 && !(WIDE && CT > 1) && !(NORM && CT > 1), "several column tiles go with one row tile and no norm");
  static_assert(!PAIR || (COLS == 8 && !NORM && !WIDE && CT == 1), "pairs of k blocks: 8 columns, one row tile of at most 8 rows");
  extern __shared__ float rows_smem[];      // [m tiles][CT][k blocks][16 rows][COLS columns], NORM: + [m tiles][k blocks][16]
  const int nkb = (K + F_KBLOCK - 1) / F_KBLOCK;
  const int mt0 = WIDE ? blockIdx.y * tiles_wg : 0;                       // first row tile of this workgroup
  const int mts = WIDE ? min(tiles_wg, (M + 15) / 16 - mt0) : (M + 15) / 16;   // and how many it owns
  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int l16 = lane % 16, kk = lane / 16;
  // a wave's unit of work: a k block, or a pair of them, of which this lane feeds the first or the second
  constexpr int UNIT = PAIR ? 2 : 1;
  const int second = PAIR ? l16 / 8 : 0;
  const int units = (nkb + UNIT - 1) / UNIT;
  const int cw = cols_wg > 0 ? cols_wg : COLS * CT;
  const int n0 = blockIdx.x * cw;
  auto wrow_of = [&](int ct) { return w + (int64_t)min(n0 + min(ct * COLS + l16 % COLS, cw - 1), N - 1) * K; };
  const float* wrow = wrow_of(0);
  // A k block that lies wholly inside K is loaded without a predicate per load (each would be a
  // branch of its own, and the waits around branches are placed for the worst case); only the last,
  // partial block of an inner size that is no multiple of 256 takes the predicated loads.  The loop
  // body exists once per case (this block whole or not, the next block whole or not).
  auto load16 = [&](auto whole, f32x4 (&dst)[16], const float* row, int k0) {
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      if constexpr (decltype(whole)::value) dst[g] = *(const f32x4*)(row + k0 + g * 16 + kk * 4);
      else dst[g] = load_k4<true>(row, k0 + g * 16 + kk * 4, K);
    }
  };
  auto a_row = [&](int mt) { return a + (int64_t)min((mt0 + mt) * 16 + (PAIR ? l16 % 8 : l16), M - 1) * lda; };
  f32x4 wv[16], wnext[WIDE ? 1 : 16];
  if (wave < units) {
    if ((wave + 1) * UNIT * F_KBLOCK <= K) load16(std::true_type{}, wv, wrow, (wave * UNIT + second) * F_KBLOCK);
    else load16(std::false_type{}, wv, wrow, (wave * UNIT + second) * F_KBLOCK);
  }
  float* ss_smem = rows_smem + mts * CT * nkb * 16 * COLS;
  // one row tile and column tile of one k block: the block sum of 16 rows x COLS columns goes to LDS
  auto multiply = [&](f32x4 (&av)[16], int mt, int b, int ct = 0) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int g = 0; g < 16; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(wv[g][e], av[g][e], acc, 0, 0, 0);
    // lane (l16, kk): row m = l16, columns 4 kk + r
    if constexpr (PAIR) {     // rows 0..7 x columns 0..7: this lane's block is the first; 8..15 x 8..15: the second
      if ((l16 < 8) == (kk < 2) && b < nkb) *(f32x4*)(&rows_smem[(b * 16 + l16 % 8) * COLS + (kk % 2) * 4]) = acc;
    } else {
      if (kk * 4 < COLS) *(f32x4*)(&rows_smem[(((mt * CT + ct) * nkb + b) * 16 + l16) * COLS + kk * 4]) = acc;
    }
  };
  // NORM: the rows times the norm's weights, their squares added up on the way (one row tile of one k block)
  auto scale_rows = [&](auto whole, f32x4 (&av)[16], int mt, int b) {
    f32x4 nw[16];
    load16(whole, nw, norm_w, b * F_KBLOCK);      // 4 * K bytes, from the caches
    float ss = 0.f;
#pragma unroll
    for (int g = 0; g < 16; ++g)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        ss = __builtin_fmaf(av[g][e], av[g][e], ss);
        av[g][e] *= nw[g][e];
      }
    // the four lanes of a row (one per k quarter): every lane gets (s0 + s1) + (s2 + s3)
    ss += __shfl_xor(ss, 16, TL_WAVE);
    ss += __shfl_xor(ss, 32, TL_WAVE);
    if (kk == 0) ss_smem[(mt * nkb + b) * 16 + l16] = ss;
  };
  constexpr int AHEAD = FR_WAVES * UNIT * F_KBLOCK;        // from a wave's unit to its next
  auto block = [&](auto whole, auto next_whole, int u) {
    const int b = u * UNIT + second;          // this lane's k block
    const int kb = b * F_KBLOCK;
    // (NORM keeps the norm's weights in registers beside the rows instead of the next block's
    // weights; those are requested once this block is done.  The norm's products have the hidden
    // size as their inner size: one block a wave up to 2048, two at 4096.)
    // The first row tile's activations are requested BEFORE the next block's weights: loads come
    // back in the order they were asked for, and the matrix instructions below wait for the
    // activations; asked for behind the weights they would wait for those as well, and the block
    // ahead would hide nothing.
    f32x4 av[16];
    load16(whole, av, a_row(0), kb);
    if constexpr (WIDE) {
      f32x4 av2[16];
      for (int mt = 0; mt < mts; mt += 2) {
        if (mt + 1 < mts) load16(whole, av2, a_row(mt + 1), kb);
        multiply(av, mt, b);
        if (mt + 1 < mts) {
          if (mt + 2 < mts) load16(whole, av, a_row(mt + 2), kb);
          multiply(av2, mt + 1, b);
        }
      }
      if (u + FR_WAVES < units) load16(next_whole, wv, wrow, kb + AHEAD);
    } else if constexpr (CT > 1) {
      // one row tile, no norm
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const bool more = ct + 1 < CT || u + FR_WAVES < units;
        if (ct + 1 < CT) load16(whole, wnext, wrow_of(ct + 1), kb);
        else if (u + FR_WAVES < units) load16(next_whole, wnext, wrow, kb + AHEAD);
        multiply(av, 0, b, ct);
        if (more) {
#pragma unroll
          for (int g = 0; g < 16; ++g) wv[g] = wnext[g];
        }
      }
    } else {
      if (!NORM && u + FR_WAVES < units) load16(next_whole, wnext, wrow, kb + AHEAD);
      for (int mt = 0; mt < mts; ++mt) {
        if (mt > 0) load16(whole, av, a_row(mt), kb);
        if constexpr (NORM) scale_rows(whole, av, mt, b);
        multiply(av, mt, b);
      }
      if constexpr (NORM) {
        if (u + FR_WAVES < units) load16(next_whole, wv, wrow, kb + AHEAD);
      } else {
#pragma unroll
        for (int g = 0; g < 16; ++g) wv[g] = wnext[g];
      }
    }
  };
  for (int u = wave; u < units; u += FR_WAVES) {
    const bool whole = (u + 1) * UNIT * F_KBLOCK <= K, next_whole = (u + FR_WAVES + 1) * UNIT * F_KBLOCK <= K;
    if (whole && next_whole) block(std::true_type{}, std::true_type{}, u);
    else if (whole) block(std::true_type{}, std::false_type{}, u);
    else block(std::false_type{}, std::false_type{}, u);
  }
  __syncthreads();
  for (int e = tid; e < mts * CT * 16 * COLS; e += FR_THREADS) {
    const int tile = e / (16 * COLS), mt = tile / CT, ct = tile % CT, r = (e % (16 * COLS)) / COLS, c = e % COLS;
    float t = 0.f;
    for (int b = 0; b < nkb; ++b) t += rows_smem[((tile * nkb + b) * 16 + r) * COLS + c];
    if constexpr (NORM) {
      float q = 0.f;
      for (int b = 0; b < nkb; ++b) q += ss_smem[(mt * nkb + b) * 16 + r];
      t *= f32_norm_factor(q, K, eps);
    }
    const int m = (mt0 + mt) * 16 + r, n = n0 + ct * COLS + c;
    if constexpr (!NORM) {
      if (row_scale && m < M) t *= row_scale[m];    // the factor of a norm in front (norm_prescale_f32_kernel)
    }
    if constexpr (SWIGLU) {   // columns (2j, 2j+1) = (gate_j, up_j); N and n0 are even
      const float u = __shfl_down(t, 1, TL_WAVE);
      if (m < M && n < N && ct * COLS + c < cw && (c & 1) == 0) out[(int64_t)m * ldo + n / 2] = swiglu_pair(t, u);
    } else {
      if (m < M && n < N && ct * COLS + c < cw) {
        const int64_t at = (int64_t)m * ldo + n;
        out[at] = residual ? t + residual[at] : t;
      }
    }
  }
}

// ==================================================================== bfloat16
// Tiles of BM x BN outputs, k in steps of 64, WM x WN wave64, each owning (BM/WM) x (BN/WN)
// outputs as 32x32x16 MFMA tiles.  Operand tiles go global -> registers -> LDS; LDS is
// double-buffered so an iteration needs one barrier, and the global loads of the next k step are
// in flight while the current one is multiplied.
//
// Tile shapes: 256 x 256 (eight waves of 128 x 64), 256 x 128, 128 x 128 and 64 x 128.  The larger
// the tile, the fewer operand bytes and LDS reads per flop and the higher the rate on a full chip;
// small products take small tiles all the same, because 256 compute units want at least that many
// workgroups (launch_gemm_bf16_any estimates the time of each shape and takes the best).
//
// Workgroups are handed to the eight XCDs in turn, each with an L2 of its own.  The tile index is
// therefore remapped so that an XCD owns a contiguous run of tiles in column-major order: it then
// reads only its own share of the weight matrix (plus the activations), instead of all of it.
constexpr int B_BK = 64;
constexpr int B_LD = B_BK + 8;  // LDS row stride in elements: 144 bytes, keeps 16-byte alignment
constexpr int B_XCDS = 8;

// What the epilogue of the tiled kernel does to a row besides the product: a factor per row
// (`row_scale`), or a norm handed from product to product as the few-row kernel does it (see
// SkinnyArgs).  The producer (float32 output, no SiLU-gate, N a multiple of 64, ldo of 4) also writes
// emit_operand[m, n] = bf16(emit_w[n] * out[m, n]) and, for every 64 columns, the sum of out^2 into
// emit_sumsq[m, n / 64] (rows of `emit_parts` parts).  The consumer takes such an operand as `a`
// and in_sumsq [rows, in_parts], and its row factor is 1 / sqrt(sum / in_width + in_eps).
struct TileNorm {
  const float* row_scale = nullptr;
  const void* emit_w = nullptr;
  int emit_w_is_f32 = 0;
  bf16_t* emit_operand = nullptr;
  int64_t emit_ld = 0;                // row stride of the operand
  float* emit_sumsq = nullptr;
  int emit_parts = 0;
  const float* in_sumsq = nullptr;
  int in_parts = 0, in_width = 0;
  float in_eps = 0.f;
  TileNorm() = default;
  TileNorm(const float* rs) : row_scale(rs) {}
};

template <int BM, int BN, int WM, int WN>
struct GemmShape {
  static constexpr int THREADS = WM * WN * TL_WAVE;
  static constexpr int TM = BM / WM, TN = BN / WN;        // a wave's outputs
  static constexpr int MI = TM / 32, NJ = TN / 32;        // as 32 x 32 MFMA tiles
  static constexpr int AC = BM * (B_BK / 8) / THREADS, WC = BN * (B_BK / 8) / THREADS;
  static constexpr size_t SMEM = (size_t)2 * (BM + BN) * B_LD * sizeof(bf16_t);      // the operand tiles
  static constexpr size_t SMEM_ALL = SMEM + BM * sizeof(float);                      // and a factor per row behind them
  static_assert(TM % 32 == 0 && TN % 32 == 0 && AC >= 1 && WC >= 1, "tile does not divide");
};

// K must be a multiple of 8 (16-byte chunks of bf16 never straddle the end).
template <int BM, int BN, int WM, int WN, typename TO, bool SWIGLU, bool FULL>
__global__ __launch_bounds__(WM * WN * TL_WAVE) void gemm_bf16_kernel(const bf16_t* __restrict__ a,
                                                                      const bf16_t* __restrict__ w,
                                                                      TO* __restrict__ out,
                                                                      const float* __restrict__ residual,
                                                                      const TileNorm nm, int M, int N, int K,
                                                                      int64_t lda, int64_t ldo, int k_per_split) {
  using S = GemmShape<BM, BN, WM, WN>;
  constexpr int MI = S::MI, NJ = S::NJ, THREADS = S::THREADS;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* As = (bf16_t*)smem_raw;                       // [2][BM][B_LD]
  bf16_t* Ws = As + 2 * BM * B_LD;                      // [2][BN][B_LD]
  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int wm = wave / WN, wn = wave % WN;
  // k_per_split > 0 (a multiple of the k step): the inner size is split over workgroups, each
  // writing its float32 partial product [M, N] behind `out` (no epilogue); a second kernel adds
  // them up.  That is how products with few output tiles still fill the chip.
  const int splits = k_per_split > 0 ? (K + k_per_split - 1) / k_per_split : 1;
  const int tiles_m = (M + BM - 1) / BM, tiles = tiles_m * ((N + BN - 1) / BN), total = tiles * splits;
  const int per_xcd = (total + B_XCDS - 1) / B_XCDS;
  const int t_all = (blockIdx.x % B_XCDS) * per_xcd + blockIdx.x / B_XCDS;
  if (t_all >= total) return;                           // the grid is padded to a multiple of 8
  const int split = t_all / tiles, t = t_all % tiles;
  const int m0 = (t % tiles_m) * BM, n0 = (t / tiles_m) * BN;
  const int kbase = split * k_per_split;
  const int kend = k_per_split > 0 ? min(K, kbase + k_per_split) : K;
  if (k_per_split > 0) out += (int64_t)split * M * ldo;

  f32x16 acc[MI][NJ];
#pragma unroll
  for (int i = 0; i < MI; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // A norm handed over: the factors of this tile's rows are worked out once, here, where the loads
  // hide behind the main loop (16 threads share a row's parts out), and wait in LDS for the
  // epilogue; the barriers of the main loop lie in between.
  float* row_factor = (float*)(smem_raw + S::SMEM);      // [BM]
  if (nm.in_sumsq) {      // uniform
    for (int r = tid / 16; r < BM; r += THREADS / 16) {
      const int64_t at = (int64_t)min(m0 + r, M - 1) * nm.in_parts;
      float t = 0.f;
      for (int q = tid % 16; q < nm.in_parts; q += 16) t += nm.in_sumsq[at + q];
      t = group_sum<16>(t);
      if (tid % 16 == 0) row_factor[r] = 1.f / sqrtf(t / (float)nm.in_width + nm.in_eps);
    }
  }

  // One k step of both operand tiles is AC + WC 16-byte pieces per thread, fetched with buffer
  // loads: the address is the tile's first row (the buffer's base, per workgroup) + an offset per
  // piece that never changes + the k offset, which is one scalar for all lanes, so a k step costs
  // no address arithmetic; and the buffer ends with the matrix, so rows beyond it read as zero
  // without a branch.  (A piece beyond K within a row is zeroed when it is written to LDS.)
  constexpr int PIECES = S::AC + S::WC;
  bf16x8 stage[PIECES];
  const int prow = tid / 8, pk = (tid % 8) * 8;            // this thread's row within a pass, k offset
  constexpr int PASS = THREADS / 8;                        // rows per pass
  auto tile_buffer = [](const bf16_t* first_row, int rows, int64_t ld, int K_) {
    const int64_t bytes = rows > 0 ? ((int64_t)(rows - 1) * ld + K_) * 2 : 0;
    return __builtin_amdgcn_make_buffer_rsrc((void*)first_row, 0, (int)(bytes < 0x7fffffff ? bytes : 0x7fffffff), 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t buf_a = tile_buffer(a + (int64_t)m0 * lda, min(M - m0, BM), lda, K);
  const __amdgpu_buffer_rsrc_t buf_w = tile_buffer(w + (int64_t)n0 * K, min(N - n0, BN), K, K);
  int piece_off[PIECES];                                   // bytes from the tile's first row
#pragma unroll
  for (int p = 0; p < PIECES; ++p) {
    const bool is_a = p < S::AC;
    const int r = (is_a ? p : p - S::AC) * PASS + prow;
    piece_off[p] = (int)(((int64_t)r * (is_a ? lda : (int64_t)K) + pk) * 2);
  }
  typedef int tl_i32x4 __attribute__((ext_vector_type(4)));
  auto gload1 = [&](int k0, int p) {
    const tl_i32x4 v = __builtin_bit_cast(
        tl_i32x4, __builtin_amdgcn_raw_buffer_load_b128(p < S::AC ? buf_a : buf_w, piece_off[p], k0 * 2, 0));
    stage[p] = __builtin_bit_cast(bf16x8, v);
  };
  // FULL: K is a multiple of the k step (and M, N of the tile), so nothing is zeroed
  auto lds_write1 = [&](int buf, int k0, int p) {
    const bool is_a = p < S::AC;
    const int r = (is_a ? p : p - S::AC) * PASS + prow;
    const bool ok = FULL || k0 + pk < K;
    bf16x8 z = {};
    bf16_t* dst = is_a ? As + (buf * BM + r) * B_LD + pk : Ws + (buf * BN + r) * B_LD + pk;
    *(bf16x8*)dst = ok ? stage[p] : z;
  };
  // MFMA operands of one k16 step: NJ weight pieces, then MI activation pieces, in the order of use
  struct Frag {
    bf16x8 w[NJ], a[MI];
  };
  constexpr int FRAG = NJ + MI;
  const bf16_t* ra = As + (wm * S::TM + lane % 32) * B_LD + (lane / 32) * 8;
  const bf16_t* rw = Ws + (wn * S::TN + lane % 32) * B_LD + (lane / 32) * 8;
  auto lds_read1 = [&](Frag& f, int buf, int ks, int p) {
    if (p < NJ) f.w[p] = *(const bf16x8*)(rw + (buf * BN + p * 32) * B_LD + ks * 16);
    else f.a[p - NJ] = *(const bf16x8*)(ra + (buf * BM + (p - NJ) * 32) * B_LD + ks * 16);
  };
  // The MFMAs of one k16 step, with memory operations issued between them: slot(n) comes after the
  // n-th MFMA.  The result tile is transposed (rows = n, columns = m) so that a lane holds four
  // consecutive n of one output row and can store them as one vector.  The scheduling barriers
  // keep the compiler from gathering the memory operations back into one place.
  constexpr int SLOTS = MI * NJ;
  auto group = [&](const Frag& f, auto&& slot) {
#pragma unroll
    for (int n = 0; n < SLOTS; ++n) {
      acc[n / NJ][n % NJ] =
          __builtin_amdgcn_mfma_f32_32x32x16_bf16(f.w[n % NJ], f.a[n / NJ], acc[n / NJ][n % NJ], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      slot(n);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // pieces [n * per, (n + 1) * per) of `total`, for spreading `total` operations over slots
  auto spread = [](int n, int total, int slots, auto&& op) {
    const int per = (total + slots - 1) / slots;
#pragma unroll
    for (int p = n * per; p < (n + 1) * per; ++p)
      if (p < total) op(p);
  };

  // The loop is software-pipelined by hand, because all waves of a workgroup meet at the barrier
  // of every k step and so cannot cover for each other: while the MFMAs of one k16 step run, the
  // fragments of the next are read; the tile of step kt + 1 (loaded into registers during step
  // kt - 1) is written to the other LDS buffer in the middle of step kt, and the loads of tile
  // kt + 2 are issued right after; the last k16 step of a tile is multiplied after the barrier,
  // while the first fragments of the next tile are on their way.
  const int nk = (kend - kbase + B_BK - 1) / B_BK;
#pragma unroll
  for (int p = 0; p < PIECES; ++p) gload1(kbase, p);
#pragma unroll
  for (int p = 0; p < PIECES; ++p) lds_write1(0, kbase, p);
  if (nk > 1) {
#pragma unroll
    for (int p = 0; p < PIECES; ++p) gload1(kbase + B_BK, p);
  }
  __syncthreads();
  Frag f0, f1;
#pragma unroll
  for (int p = 0; p < FRAG; ++p) lds_read1(f0, 0, 0, p);
  static_assert(SLOTS >= 2, "a wave owns at least two MFMA tiles");
  constexpr int HALF = SLOTS / 2;
  auto step = [&](auto has_next, auto has_next2, int kt) {
    constexpr bool NX = decltype(has_next)::value, NX2 = decltype(has_next2)::value;
    const int cur = kt & 1, nxt = cur ^ 1, k1 = kbase + (kt + 1) * B_BK, k2 = kbase + (kt + 2) * B_BK;
    group(f0, [&](int n) { spread(n, FRAG, SLOTS, [&](int p) { lds_read1(f1, cur, 1, p); }); });
    group(f1, [&](int n) {
      spread(n, FRAG, SLOTS, [&](int p) { lds_read1(f0, cur, 2, p); });
      if constexpr (NX)
        if (n >= SLOTS - HALF) spread(n - (SLOTS - HALF), PIECES / 2, HALF, [&](int p) { lds_write1(nxt, k1, p); });
    });
    group(f0, [&](int n) {
      spread(n, FRAG, SLOTS, [&](int p) { lds_read1(f1, cur, 3, p); });
      if constexpr (NX)
        if (n < HALF) spread(n, PIECES - PIECES / 2, HALF, [&](int p) { lds_write1(nxt, k1, PIECES / 2 + p); });
      if constexpr (NX2)
        if (n >= SLOTS - HALF) spread(n - (SLOTS - HALF), PIECES, HALF, [&](int p) { gload1(k2, p); });
    });
    __syncthreads();
    group(f1, [&](int n) {
      if constexpr (NX) spread(n, FRAG, SLOTS, [&](int p) { lds_read1(f0, nxt, 0, p); });
    });
  };
  {
    int kt = 0;
    for (; kt + 2 < nk; ++kt) step(std::true_type{}, std::true_type{}, kt);
    if (kt + 1 < nk) {
      step(std::true_type{}, std::false_type{}, kt);
      ++kt;
    }
    step(std::false_type{}, std::false_type{}, kt);
  }

  // Epilogue.  A lane's accumulators hold four consecutive n of 32 different rows, so stored from
  // there a row would go out in 16-byte pieces.  Each wave therefore passes its result, 32 rows x
  // 64 columns at a time, through an LDS area of its own (the operand tiles are no longer read:
  // the last fragments were fetched before the loop's last barrier) and reads it back row by
  // row: 16 lanes then cover 256 contiguous bytes of one row, and so do the residual reads.
  static_assert(S::TN == 64, "the epilogue stages 64 columns per wave");
  constexpr int E_LD = 68;                 // floats per staged row: 16-byte aligned, conflict-free
  static_assert((size_t)WM * WN * 32 * E_LD * sizeof(float) <= S::SMEM, "staging areas fit the tile buffers");
  float* cstage = (float*)smem_raw + wave * (32 * E_LD);
  const bool vec_ok = (N % 4 == 0) && (ldo % 4 == 0);
#pragma unroll
  for (int i = 0; i < MI; ++i) {
#pragma unroll
    for (int j = 0; j < NJ; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        f32x4 v4 = {acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2], acc[i][j][q * 4 + 3]};
        *(f32x4*)(cstage + (lane % 32) * E_LD + j * 32 + q * 8 + (lane / 32) * 4) = v4;
      }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int c8 = 0; c8 < 8; ++c8) {
      const int c = c8 * TL_WAVE + lane;
      const int r = c / 16, col = (c % 16) * 4;
      const int m = m0 + wm * S::TM + i * 32 + r, n = n0 + wn * S::TN + col;
      if (m >= M || n >= N) continue;
      // the row's factor (1 / rms of a norm left out of the operand): given, or that of a norm handed over
      float rs = 1.f;
      if (nm.in_sumsq) rs = row_factor[m - m0];
      else if (nm.row_scale) rs = nm.row_scale[m];
      const f32x4 s4 = *(const f32x4*)(cstage + r * E_LD + col);
      float v[4] = {s4[0] * rs, s4[1] * rs, s4[2] * rs, s4[3] * rs};
      if constexpr (SWIGLU) {   // (gate, up, gate, up) -> two outputs; N is even and n a multiple of 4
        const int64_t oz = (int64_t)m * ldo + n / 2;
        if (n + 2 < N) {
          typedef TO to2 __attribute__((ext_vector_type(2)));
          to2 sv = {from_f32<TO>(swiglu_pair_fast(v[0], v[1])), from_f32<TO>(swiglu_pair_fast(v[2], v[3]))};
          if (ldo % 2 == 0) {
            *(to2*)(out + oz) = sv;
          } else {
            out[oz] = sv[0];
            out[oz + 1] = sv[1];
          }
        } else {
          out[oz] = from_f32<TO>(swiglu_pair_fast(v[0], v[1]));
        }
        continue;
      }
      const int64_t o = (int64_t)m * ldo + n;
      if (vec_ok) {  // n + 3 < N because n and N are both multiples of 4
        if (residual) {
          const f32x4 rv = *(const f32x4*)(residual + o);
          v[0] += rv[0]; v[1] += rv[1]; v[2] += rv[2]; v[3] += rv[3];
        }
        if constexpr (sizeof(TO) == 4) {
          f32x4 sv = {v[0], v[1], v[2], v[3]};
          *(f32x4*)((float*)out + o) = sv;
          if constexpr (!SWIGLU) {
            if (nm.emit_operand) {      // uniform; N is a multiple of 64: the 16 lanes of a row are all here or none is
              float wn[4];
              if (nm.emit_w_is_f32) {
                const f32x4 w4 = *(const f32x4*)((const float*)nm.emit_w + n);
                wn[0] = w4[0]; wn[1] = w4[1]; wn[2] = w4[2]; wn[3] = w4[3];
              } else {
                const bf16x4 w4 = *(const bf16x4*)((const bf16_t*)nm.emit_w + n);
                wn[0] = (float)w4[0]; wn[1] = (float)w4[1]; wn[2] = (float)w4[2]; wn[3] = (float)w4[3];
              }
              bf16x4 ev = {(bf16_t)(wn[0] * v[0]), (bf16_t)(wn[1] * v[1]), (bf16_t)(wn[2] * v[2]), (bf16_t)(wn[3] * v[3])};
              *(bf16x4*)(nm.emit_operand + (int64_t)m * nm.emit_ld + n) = ev;
              const float sq = group_sum<16>((v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]));
              if (lane % 16 == 0) nm.emit_sumsq[(int64_t)m * nm.emit_parts + n / 64] = sq;
            }
          }
        } else {
          bf16x4 sv = {(bf16_t)v[0], (bf16_t)v[1], (bf16_t)v[2], (bf16_t)v[3]};
          *(bf16x4*)((bf16_t*)out + o) = sv;
        }
      } else {
        for (int e = 0; e < 4 && n + e < N; ++e) {
          float x = v[e];
          if (residual) x += residual[o + e];
          out[o + e] = from_f32<TO>(x);
        }
      }
    }
    // the area is written again for the next 32 rows
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

template <int BM, int BN, int WM, int WN, typename TO, bool SWIGLU, bool FULL>
static int launch_gemm_bf16_full(const bf16_t* a, const bf16_t* w, TO* out, const float* residual,
                                 const TileNorm& row_scale, int M, int N, int K, int64_t lda, int64_t ldo,
                                 int k_per_split, hipStream_t stream) {
  using S = GemmShape<BM, BN, WM, WN>;
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute((const void*)gemm_bf16_kernel<BM, BN, WM, WN, TO, SWIGLU, FULL>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)S::SMEM_ALL) != hipSuccess)
      return TL_ERR_LAUNCH;
    configured = true;
  }
  // a tile's rows are addressed with 32-bit byte offsets from its first row
  if ((int64_t)BM * lda * 2 >= 0x7fffffff || (int64_t)BN * K * 2 >= 0x7fffffff) return TL_ERR_ARG;
  if (row_scale.emit_operand && (SWIGLU || sizeof(TO) != 4 || N % 64 || ldo % 4 || k_per_split > 0)) return TL_ERR_ARG;
  if (row_scale.in_sumsq && k_per_split > 0) return TL_ERR_ARG;      // a split product has no epilogue of its own
  const int64_t splits = k_per_split > 0 ? (K + k_per_split - 1) / k_per_split : 1;
  const int64_t total = (int64_t)((N + BN - 1) / BN) * ((M + BM - 1) / BM) * splits;
  const int64_t grid = (total + B_XCDS - 1) / B_XCDS * B_XCDS;
  if (grid > 0x7fffffff) return TL_ERR_ARG;
  hipLaunchKernelGGL((gemm_bf16_kernel<BM, BN, WM, WN, TO, SWIGLU, FULL>), dim3((unsigned)grid), dim3(S::THREADS),
                     S::SMEM_ALL, stream, a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split);
  static_assert(sizeof(TileNorm) <= 96, "passed by value");
  return TL_OK;
}

template <int BM, int BN, int WM, int WN, typename TO, bool SWIGLU>
static int launch_gemm_bf16(const bf16_t* a, const bf16_t* w, TO* out, const float* residual, const TileNorm& row_scale,
                            int M, int N, int K, int64_t lda, int64_t ldo, int k_per_split, hipStream_t stream) {
  if (M % BM == 0 && N % BN == 0 && K % B_BK == 0)
    return launch_gemm_bf16_full<BM, BN, WM, WN, TO, SWIGLU, true>(a, w, out, residual, row_scale, M, N, K, lda, ldo,
                                                                   k_per_split, stream);
  return launch_gemm_bf16_full<BM, BN, WM, WN, TO, SWIGLU, false>(a, w, out, residual, row_scale, M, N, K, lda, ldo,
                                                                  k_per_split, stream);
}

// Which tile: the one with the smallest estimated time.  A compute unit works through
// ceil(workgroups / 256) tiles one after the other, each at the rate that its tile shape reaches
// on a full chip (measured, TFLOP/s: the larger the tile, the fewer operand bytes per flop).
struct TileChoice {
  int bm, bn;
  double rate;
};
static const TileChoice kTiles[4] = {{256, 256, 1060.}, {256, 128, 900.}, {128, 128, 760.}, {64, 128, 640.}};

static double tile_cost(int c, int M, int N) {
  const int64_t wgs = (int64_t)((M + kTiles[c].bm - 1) / kTiles[c].bm) * ((N + kTiles[c].bn - 1) / kTiles[c].bn);
  return (double)((wgs + 255) / 256) * kTiles[c].bm * kTiles[c].bn / kTiles[c].rate;
}

static int best_tile(int M, int N, double* cost) {
  int best = 0;
  double best_cost = 0.;
  for (int c = 0; c < 4; ++c) {
    const double t = tile_cost(c, M, N);
    if (c == 0 || t < best_cost) {
      best = c;
      best_cost = t;
    }
  }
  if (cost) *cost = best_cost;
  return best;
}

template <typename TO, bool SWIGLU>
static int launch_gemm_bf16_tile(int c, const bf16_t* a, const bf16_t* w, TO* out, const float* residual,
                                 const TileNorm& row_scale, int M, int N, int K, int64_t lda, int64_t ldo,
                                 int k_per_split, hipStream_t stream) {
  switch (c) {
    case 0:
      return launch_gemm_bf16<256, 256, 2, 4, TO, SWIGLU>(a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split,
                                                          stream);
    case 1:
      return launch_gemm_bf16<256, 128, 4, 2, TO, SWIGLU>(a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split,
                                                          stream);
    case 2:
      return launch_gemm_bf16<128, 128, 4, 2, TO, SWIGLU>(a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split,
                                                          stream);
    default:
      return launch_gemm_bf16<64, 128, 2, 2, TO, SWIGLU>(a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split,
                                                         stream);
  }
}

// tile: 1..4 force a tile shape, 0 lets the sizes decide.  Then a wide product may be launched in
// two parts: as many columns as fill the chip in whole rounds of the largest tile, and the rest
// with whatever tile suits the rest; a single tile shape would leave the last round of
// workgroups mostly empty (2048 x 11264: 352 tiles of 256 x 256 on 256 compute units).
template <typename TO, bool SWIGLU>
static int launch_gemm_bf16_any(const bf16_t* a, const bf16_t* w, TO* out, const float* residual,
                                const TileNorm& row_scale, int M, int N, int K, int64_t lda, int64_t ldo,
                                int tile, int k_per_split, hipStream_t stream) {
  if (tile >= 1 && tile <= 4)
    return launch_gemm_bf16_tile<TO, SWIGLU>(tile - 1, a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split,
                                             stream);
  double whole_cost;
  const int whole = best_tile(M, N, &whole_cost);
  if (k_per_split == 0) {
    const int tiles_m = (M + 255) / 256;
    const int cols_per_round = 256 / tiles_m * 256;          // columns that one round of 256 x 256 tiles covers
    const int n_first = cols_per_round > 0 ? N / cols_per_round * cols_per_round : 0;
    if (n_first > 0 && n_first < N) {
      double rest_cost;
      const int rest = best_tile(M, N - n_first, &rest_cost);
      if (tile_cost(0, M, n_first) + rest_cost < whole_cost) {
        int rc = launch_gemm_bf16_tile<TO, SWIGLU>(0, a, w, out, residual, row_scale, M, n_first, K, lda, ldo, 0, stream);
        if (rc != TL_OK) return rc;
        const int64_t o_off = SWIGLU ? n_first / 2 : n_first;
        TileNorm rest_norm = row_scale;      // what it emits belongs to columns n_first on (a multiple of 256)
        if (rest_norm.emit_operand) {
          rest_norm.emit_w = rest_norm.emit_w_is_f32 ? (const void*)((const float*)rest_norm.emit_w + n_first)
                                                     : (const void*)((const bf16_t*)rest_norm.emit_w + n_first);
          rest_norm.emit_operand += n_first;
          rest_norm.emit_sumsq += n_first / 64;
        }
        return launch_gemm_bf16_tile<TO, SWIGLU>(rest, a, w + (int64_t)n_first * K, out + o_off,
                                                 residual ? residual + o_off : nullptr, rest_norm, M, N - n_first, K,
                                                 lda, ldo, 0, stream);
      }
    }
  }
  return launch_gemm_bf16_tile<TO, SWIGLU>(whole, a, w, out, residual, row_scale, M, N, K, lda, ldo, k_per_split, stream);
}

// ------------------------------------------- split k for few rows: everything in flight
// At most 64 rows, the inner size split over workgroups.  A workgroup's share of both operands (64
// rows of activations and 128 weight rows per 64 k) goes straight into LDS
// (global_load_lds_dwordx4: no registers in between), as a ring of six slabs of 64 k, so that five
// slabs (120 KB) are on their way while one is multiplied; a share of up to six slabs is requested
// at once and the kernel is one round trip to memory long.  The tiled kernel above keeps one k
// step of 64 in flight and pays a round trip for each.
// A slab in LDS: [A: 8 groups of 8 rows | W: 16 groups of 8 rows][8 rows x 128 bytes]; one load
// instruction of a wave fills one group (1 KB, lane i -> bytes 16 i); the 16-byte chunk c of row r
// stands at position c ^ (r % 8), so that the fragment reads of 32 rows do not collide.
// Result: float32 partial products [split, M, N] for splitk_reduce_kernel.  K must be a multiple of 64.
constexpr int O_BM = 64, O_BN = 128, O_WAVES = 8, O_THREADS = O_WAVES * TL_WAVE, O_SLAB_K = 64, O_RING = 6;
constexpr int O_GROUPS = (O_BM + O_BN) / 8, O_GROUP_BYTES = 8 * O_SLAB_K * 2, O_SLAB_BYTES = O_GROUPS * O_GROUP_BYTES;
typedef __attribute__((address_space(3))) void* tl_lds_ptr;
typedef const __attribute__((address_space(1))) void* tl_global_ptr;

// waits until at most 3 * later of this wave's loads are outstanding (three loads a slab)
__device__ __forceinline__ void oneshot_wait(int later) {
  switch (later) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    case 1: __builtin_amdgcn_s_waitcnt(0x0F73); break;
    case 2: __builtin_amdgcn_s_waitcnt(0x0F76); break;
    case 3: __builtin_amdgcn_s_waitcnt(0x0F79); break;
    default: __builtin_amdgcn_s_waitcnt(0x0F7C); break;       // 12
  }
}

__global__ __launch_bounds__(O_THREADS) void gemm_oneshot_bf16_kernel(const bf16_t* __restrict__ a,
                                                                      const bf16_t* __restrict__ w,
                                                                      float* __restrict__ partial, int M, int N, int K,
                                                                      int64_t lda, int slabs_per_split) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char oneshot_smem[];
  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int n0 = blockIdx.x * O_BN, split = blockIdx.y, m0 = blockIdx.z * O_BM;
  const int nslabs = K / O_SLAB_K, s0 = split * slabs_per_split, s1 = min(nslabs, s0 + slabs_per_split);
  const int mine = s1 - s0;                       // at least one: the grid has no empty split
  // requests: of every slab wave v fills group v (8 activation rows) and groups 8 + v and 16 + v
  // (16 weight rows); a lane's three addresses move on by 64 k from slab to slab
  static_assert(O_BM / 8 == O_WAVES && O_BN / 8 == 2 * O_WAVES, "one activation group and two weight groups a wave");
  const int wv = __builtin_amdgcn_readfirstlane(wave);
  const int lrow = lane / 8, lchunk = (lane % 8) ^ lrow;
  const int64_t k_first = (int64_t)s0 * O_SLAB_K + lchunk * 8;
  const bf16_t* src[3] = {a + (int64_t)min(m0 + wv * 8 + lrow, M - 1) * lda + k_first,
                          w + (int64_t)min(n0 + wv * 8 + lrow, N - 1) * K + k_first,
                          w + (int64_t)min(n0 + (O_WAVES + wv) * 8 + lrow, N - 1) * K + k_first};
  auto request = [&](int sl) {                    // slab sl of this workgroup, into buffer sl % O_RING
    unsigned char* sb = oneshot_smem + (sl % O_RING) * O_SLAB_BYTES + wv * O_GROUP_BYTES;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      __builtin_amdgcn_global_load_lds((tl_global_ptr)src[j], (tl_lds_ptr)(sb + j * O_WAVES * O_GROUP_BYTES), 16, 0, 0);
      src[j] += O_SLAB_K;
    }
  };
  for (int sl = 0; sl < min(mine, O_RING - 1); ++sl) request(sl);
  // wave (wm, wn) owns rows wm*32.., columns wn*32..; result transposed (rows of the instruction are
  // output columns), so a lane ends up with four consecutive columns of one row
  const int wm = wave / 4, wn = wave % 4;
  const int r8 = lane % 8;
  const int lane_off = ((lane % 32) / 8) * O_GROUP_BYTES + r8 * 128;
  const int a_off = (wm * 32 / 8) * O_GROUP_BYTES + lane_off;
  const int w_off = (O_BM / 8 + wn * 32 / 8) * O_GROUP_BYTES + lane_off;
  f32x16 acc;
#pragma unroll
  for (int r = 0; r < 16; ++r) acc[r] = 0.f;
  for (int sl = 0; sl < mine; ++sl) {
    // slab sl has landed for this wave once only the slabs requested after it are outstanding;
    // after the barrier it has landed for everybody, and nobody reads slab sl - 1 any more, whose
    // buffer the next request takes
    // (a bare barrier: __syncthreads() would also wait for every outstanding load, the slabs still on
    // their way included; the counter above is the wait that is needed, and the fragment reads of
    // the previous slab were consumed by its matrix instructions before any wave gets here)
    oneshot_wait(min(mine - 1, sl + O_RING - 2) - sl);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (sl + O_RING - 1 < mine) request(sl + O_RING - 1);
    const unsigned char* sb = oneshot_smem + (sl % O_RING) * O_SLAB_BYTES;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int pos = ((2 * ks + lane / 32) ^ r8) * 16;
      const bf16x8 fa = *(const bf16x8*)(sb + a_off + pos);
      const bf16x8 fw = *(const bf16x8*)(sb + w_off + pos);
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fw, fa, acc, 0, 0, 0);
    }
  }
  float* out = partial + (int64_t)split * M * N;
  const int m = m0 + wm * 32 + lane % 32;
  if (m < M) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wn * 32 + q * 8 + (lane / 32) * 4;
      if ((N % 4 == 0) && n + 3 < N) {
        *(f32x4*)(out + (int64_t)m * N + n) = f32x4{acc[q * 4 + 0], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]};
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) out[(int64_t)m * N + n + e] = acc[q * 4 + e];
      }
    }
  }
}

// Whether and how this kernel takes a product of 17 to 64 rows: slabs of 64 k per split (0: not this
// kernel).  The number of splits with the smallest estimated time: rounds of workgroups over the 256
// compute units, each as long as a workgroup takes to fetch its share (about 35 GB/s), and the second
// kernel's reading of the partial sums.
static int oneshot_plan(int M, int N, int K, int* slabs_per_split) {
  *slabs_per_split = 0;
  if (M <= 16 || K % O_SLAB_K || K < 4 * O_SLAB_K) return 1;
  // measured on whole decode steps: small weight matrices with few rows are faster in the few-row
  // kernel (one launch); up to 32 rows for matrices of 6 M weights (3 % of a step at 32 rows; from
  // 36 rows on this kernel is 2 to 7 % of a step faster), up to 18 rows for 17 M weights (4096 x 4096:
  // from 22 rows on this kernel is 1 to 2 % of a step faster)
  const int64_t weights = (int64_t)N * K;
  const int tiles = ((M + O_BM - 1) / O_BM) * ((N + O_BN - 1) / O_BN), nslabs = K / O_SLAB_K;
  if (M <= O_BM && ((weights <= ((int64_t)6 << 20) && M <= 32) || (weights <= ((int64_t)17 << 20) && K <= 4096 && M <= 18) ||
                    (tiles > 128 && M <= 32)))
    return 1;
  int best = 1, best_per = 0;
  double best_t = 0.;
  for (int want = 2; want <= 16; ++want) {
    const int per = (nslabs + want - 1) / want;
    // measured on whole steps: shares of fewer than four slabs lose to fewer, longer ones
    if (per < (nslabs >= 8 ? 4 : 2)) break;
    const int splits = (nslabs + per - 1) / per;
    if (splits < 2) continue;
    const int rounds = (tiles * splits + 255) / 256;
    const double t = rounds * (2.0 + per * (O_SLAB_BYTES / 35e3)) + 1.5 + splits * (double)M * N * 4 / 3e6;
    if (best == 1 || t < best_t) {
      best = splits;
      best_per = per;
      best_t = t;
    }
  }
  *slabs_per_split = best_per;
  return best;
}

// ------------------------------------------------------------ split k: the second kernel
// Adds up the partial products [splits, M, N] of a product whose inner size was split over
// workgroups and applies what the product's own epilogue would have: row factor (given, or from
// sums of squares handed over by the producer of the input), residual, SiLU-gate, output type; it
// can also prepare the next norm (operand and sums of squares per chunk of 1024 columns).  One
// workgroup per (row, chunk of 1024 columns), four consecutive columns per thread.
constexpr int R_THREADS = 256, R_CHUNK = R_THREADS * 4;

struct ReduceArgs {
  const float* partial;
  int splits, M, N;
  void* out;
  int64_t ldo;
  const float* residual;
  const float* row_scale;
  const float* in_sumsq;
  int in_parts, in_width;
  float in_eps;
  const void* emit_w;
  int emit_w_is_f32;
  bf16_t* emit_operand;
  float* emit_sumsq;
};

template <typename TO, bool SWIGLU>
__global__ __launch_bounds__(R_THREADS) void splitk_reduce_kernel(const ReduceArgs p) {
  __shared__ float red[R_THREADS / TL_WAVE];
  const int m = blockIdx.x, tid = threadIdx.x;
  const int n = blockIdx.y * R_CHUNK + tid * 4;
  const int N = p.N;
  // Everything that has to come from memory is requested before anything is used: the kernel is
  // a few dependent round trips long, and every one it saves counts.
  float t = 0.f;
  if (p.in_sumsq)
    for (int q = tid; q < p.in_parts; q += R_THREADS) t += p.in_sumsq[(int64_t)m * p.in_parts + q];
  float scale = p.row_scale ? p.row_scale[m] : 1.f;
  float res[4] = {0.f, 0.f, 0.f, 0.f}, wn[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (!SWIGLU) {
    for (int e = 0; e < 4 && n + e < N; ++e) {
      if (p.residual) res[e] = p.residual[(int64_t)m * p.ldo + n + e];
      if (p.emit_operand)
        wn[e] = p.emit_w_is_f32 ? ((const float*)p.emit_w)[n + e] : (float)((const bf16_t*)p.emit_w)[n + e];
    }
  }
  const bool vec = (N % 4 == 0);
  float v[4] = {0.f, 0.f, 0.f, 0.f};
  if (n < N) {
    if (vec) {
      // eight splits at a time, their loads in flight together; added in the order of the splits
      for (int sp0 = 0; sp0 < p.splits; sp0 += 8) {
        f32x4 x[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          x[u] = *(const f32x4*)(p.partial + ((int64_t)min(sp0 + u, p.splits - 1) * p.M + m) * N + n);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          if (sp0 + u < p.splits) {
            v[0] += x[u][0]; v[1] += x[u][1]; v[2] += x[u][2]; v[3] += x[u][3];
          }
        }
      }
    } else {
      for (int sp = 0; sp < p.splits; ++sp) {
        const float* src = p.partial + ((int64_t)sp * p.M + m) * N + n;
        for (int e = 0; e < 4 && n + e < N; ++e) v[e] += src[e];
      }
    }
  }
  if (p.in_sumsq) {      // uniform
    t = block_sum<R_THREADS / TL_WAVE>(t, red);
    scale = 1.f / sqrtf(t / (float)p.in_width + p.in_eps);
  }
  TO* out = (TO*)p.out;
  float sq = 0.f;
  if (n < N) {
    if constexpr (SWIGLU) {   // (gate, up, gate, up) -> two outputs; N is even and n a multiple of 4
      out[(int64_t)m * p.ldo + n / 2] = from_f32<TO>(swiglu_pair_fast(v[0] * scale, v[1] * scale));
      if (n + 2 < N)
        out[(int64_t)m * p.ldo + n / 2 + 1] = from_f32<TO>(swiglu_pair_fast(v[2] * scale, v[3] * scale));
    } else {
      for (int e = 0; e < 4 && n + e < N; ++e) {
        const float x = v[e] * scale + res[e];
        out[(int64_t)m * p.ldo + n + e] = from_f32<TO>(x);
        if (p.emit_operand) {
          p.emit_operand[(int64_t)m * N + n + e] = (bf16_t)(wn[e] * x);
          sq += x * x;
        }
      }
    }
  }
  if (p.emit_operand) {       // uniform
    sq = block_sum<R_THREADS / TL_WAVE>(sq, red);
    if (tid == 0) p.emit_sumsq[(int64_t)m * gridDim.y + blockIdx.y] = sq;
  }
}

// How a bfloat16 product of these sizes is best split: returns the number of splits (1: not at
// all) and sets the tile (as tl_linear_tile's) and the inner size per split.  Splitting pays when
// the output has too few tiles to fill 256 compute units and the rows are too many for the
// few-row kernel to stream the weights at full rate.
static int splitk_plan(int M, int N, int K, int* tile, int* k_per_split) {
  *tile = 0;
  *k_per_split = 0;
  // The ring kernel's sizes.  Up to 64 rows: it or the few-row kernel.  Beyond (tiles of 64 rows side by
  // side), measured: it beats the k-step loop up to 128 rows on matrices up to 4096 x 6144 and up to 256
  // rows on small ones; its one accumulator tile a wave is no match for the tiled kernel beyond that.
  const int64_t weights = (int64_t)N * K;
  const bool ring_rows = M <= O_BM || (M <= 128 && N <= 6144 && weights <= ((int64_t)26 << 20)) ||
                         (M <= 256 && weights <= ((int64_t)6 << 20));
  if (M > 16 && ring_rows && K % O_SLAB_K == 0 && K >= 4 * O_SLAB_K) {
    int slabs;
    const int one = oneshot_plan(M, N, K, &slabs);
    *tile = -1;
    *k_per_split = slabs * O_SLAB_K;
    return one;
  }
  if (M <= 16 || K < 8 * B_BK) return 1;
  const int bm = M <= 64 ? 64 : 128, bn = 128;
  const int64_t wgs = (int64_t)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
  if (wgs >= 160) return 1;
  if (M <= 64 && (int64_t)N * K < (int64_t)8 << 20) return 1;      // small weights: the few-row kernel is faster
  const int nk = (K + B_BK - 1) / B_BK;
  const int want = (int)((256 + wgs - 1) / wgs);
  int per = (nk + want - 1) / want;
  if (per < 4) per = 4;
  const int splits = (nk + per - 1) / per;
  if (splits < 2) return 1;
  *tile = M <= 64 ? 4 : 3;
  *k_per_split = per * B_BK;
  return splits;
}

// ============================================================ bfloat16, few rows
// Decode-shaped products (M <= 64): the weight matrix is streamed once and is the
// whole cost, and a step is a chain of such kernels, so the kernel is built around
// (a) many 16-byte loads in flight and (b) as few dependent memory round trips and
// as few launches as possible.  A workgroup of eight wave64 owns 16 output columns
// (16 weight rows; 32 or 64 when there are more than 16 activation rows); the waves split K in
// blocks of 128 and each accumulates a
// 16 x 16 tile per group of 16 activation rows and 16 columns with v_mfma_f32_16x16x32_bf16
// (weight rows as the A operand read straight from global memory, activations as
// the B operand).  Partial tiles meet in LDS and are added in a fixed order, so
// results are deterministic.
//
// Fused into it, to save launches: a prologue on the activations, either RMSNorm of
// the float32 residual stream (statistics recomputed by every workgroup: a few KB
// from L2) or SiLU-gate of a [M, 2K] gate|up matrix; an optional gather of input
// rows; and the residual add in the epilogue, whose operand is fetched before the
// main loop starts.
constexpr int S_WAVES = 8, S_THREADS = S_WAVES * TL_WAVE, S_COLS = 16, S_KBLK = 128;
enum { PRO_NONE = 0, PRO_NORM = 1 };

struct SkinnyArgs {
  const void* a;            // PRO_NONE: bf16 [M, K]; PRO_NORM: float [rows, K]
  const bf16_t* w;          // [N, K]
  void* out;                // [M, N]
  const float* residual;    // [M, N] or null
  const void* norm_w;       // PRO_NORM: [K], float or bf16
  const int32_t* rows;      // optional gather of input rows
  const float* row_scale;   // optional factor of each output row (a norm applied by an earlier kernel)
  float eps;
  int norm_w_is_f32;
  int M, N, K;
  int64_t lda, ldo;
  // A norm handed from producer to consumer.  The producer (float32 output, no SiLU-gate) also
  // writes emit_operand[m, n] = bf16(emit_w[n] * out[m, n]) and, per group of columns (one group
  // a workgroup: 16 columns, or 8), the sum of out^2 into emit_sumsq[m, group].  The consumer takes
  // such an operand as `a` and turns in_sumsq [rows, in_parts] into its row factor
  // 1 / sqrt(sum / in_width + in_eps).
  const void* emit_w = nullptr;
  int emit_w_is_f32 = 0;
  bf16_t* emit_operand = nullptr;
  float* emit_sumsq = nullptr;
  const float* in_sumsq = nullptr;
  int in_parts = 0, in_width = 0;
  float in_eps = 0.f;
  // The columns a workgroup owns, even, at most 16 a column tile (0: all of them).  Fewer make one
  // balanced round of workgroups out of a product whose column tiles do not divide by 256.
  int cols_wg = 0;
};

// One 8-wide k chunk of an activation row, as loaded (Raw) and as an MFMA operand.  With the norm
// prologue the operand is w * x of the float32 residual stream (rounded to bfloat16) and `ss`
// collects x^2: the row's 1 / rms is a common factor of the whole dot product and is applied to
// the result instead, so nothing has to wait for the row statistics.  Loading and converting are
// separate steps so that the loads of the next k block can be in flight while this one is used.
template <int PRO>
struct SkinnyChunk;
template <>
struct SkinnyChunk<PRO_NONE> {
  bf16x8 v;
  __device__ __forceinline__ void load(const SkinnyArgs& p, int64_t off) { v = *(const bf16x8*)((const bf16_t*)p.a + off); }
};
template <>
struct SkinnyChunk<PRO_NORM> {
  f32x4 x0, x1;
  __device__ __forceinline__ void load(const SkinnyArgs& p, int64_t off) {
    const float* x = (const float*)p.a + off;
    x0 = *(const f32x4*)x;
    x1 = *(const f32x4*)(x + 4);
  }
};
// the norm weights of one k chunk, as floats
struct NormChunk {
  f32x4 w0, w1;
  __device__ __forceinline__ void load(const SkinnyArgs& p, int k) {
    if (p.norm_w_is_f32) {
      w0 = *(const f32x4*)((const float*)p.norm_w + k);
      w1 = *(const f32x4*)((const float*)p.norm_w + k + 4);
    } else {
      const bf16x8 w8 = *(const bf16x8*)((const bf16_t*)p.norm_w + k);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        w0[e] = (float)w8[e];
        w1[e] = (float)w8[4 + e];
      }
    }
  }
};
// `k_ok`: the chunk lies inside the row (it counts towards the sum of squares); the product itself
// is protected by zeroing the weight chunk instead.
__device__ __forceinline__ bf16x8 skinny_operand(const SkinnyChunk<PRO_NONE>& c, const NormChunk&, bool, float&) {
  return c.v;
}
__device__ __forceinline__ bf16x8 skinny_operand(const SkinnyChunk<PRO_NORM>& c, const NormChunk& nw, bool k_ok,
                                                 float& ss) {
  bf16x8 r;
  float q = 0.f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    r[e] = (bf16_t)(nw.w0[e] * c.x0[e]);
    r[4 + e] = (bf16_t)(nw.w1[e] * c.x1[e]);
    q += c.x0[e] * c.x0[e] + c.x1[e] * c.x1[e];
  }
  ss += k_ok ? q : 0.f;
  return r;
}

// DEEP: two register stages also with one tile, for long inner sizes, where a wave works through
// several stages and the chain of their memory round trips sets the kernel's duration.
//
// HALF (at most 8 activation rows, one tile, no prologue): a workgroup owns 8 columns only, so that
// a matrix with few rows still gives every compute unit a workgroup; what a workgroup can have in
// flight, not the memory system, bounds these kernels.  The 16 x 16 MFMA tile is then used as two
// 8 x 8 tiles that split k: weight row i of the operand is column i % 8 at k offset (i / 8) * 32,
// activation column j is row j % 8 at k offset (j / 8) * 32, and the wanted products are the two
// diagonal blocks of the result, added in the epilogue.  One MFMA so covers 64 k, and a load
// instruction reads whole 128-byte lines of 8 weight rows.
template <int MT, int CT, bool DEEP, typename TO, int PRO, bool SWIGLU, bool HALF>
__global__ __launch_bounds__(S_THREADS) void gemm_skinny_bf16_kernel(const SkinnyArgs p) {
  static_assert(!HALF || (MT == 1 && CT == 1 && PRO == PRO_NONE && !SWIGLU), "HALF: one plain tile");
  constexpr int COLS = HALF ? 8 : S_COLS;          // columns of a tile that are outputs
  constexpr int KW = HALF ? 64 : 32;               // k covered by one MFMA
  constexpr int KBLK = 4 * KW;                     // k covered by a block of four MFMAs
  extern __shared__ __attribute__((aligned(16))) unsigned char skinny_smem[];
  typedef float Tile[16][17];
  Tile* part = (Tile*)skinny_smem;                                  // [S_WAVES][MT * CT]
  float* ss_part = (float*)(part + S_WAVES * MT * CT);              // [S_WAVES][MT * 16]
  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int M = p.M, N = p.N, K = p.K;
  const int cw = (!HALF && p.cols_wg > 0) ? p.cols_wg : COLS * CT;      // columns of this workgroup
  const int n0 = blockIdx.x * cw;
  const int r16 = lane % 16, g = lane / 16;
  const int rr = HALF ? r16 % 8 : r16;             // the weight row / activation row this lane feeds
  const int kh = HALF ? (r16 / 8) * 32 : 0;        // and its k offset inside an MFMA's range
  const bf16_t* wrow[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) wrow[ct] = p.w + (int64_t)min(n0 + min(ct * 16 + rr, cw - 1), N - 1) * K;

  // epilogue operands first: their latency hides behind the main loop
  constexpr int TILES = MT * CT;
  constexpr int EPT = (TILES * 256 + S_THREADS - 1) / S_THREADS;
  float res_v[EPT];
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = tid + j * S_THREADS;
    const int tile = e / 256;
    const int m = HALF ? e / 8 : (tile / CT) * 16 + (e % 256) / 16;
    const int n = HALF ? n0 + e % 8 : n0 + (tile % CT) * 16 + e % 16;
    res_v[j] = (p.residual && e < (HALF ? 64 : TILES * 256) && m < M && n < N && n - n0 < cw) ? p.residual[(int64_t)m * p.ldo + n] : 0.f;
  }

  // input row of each activation row this lane feeds
  int64_t row_off[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + rr;
    const int src = p.rows ? p.rows[min(m, M - 1)] : min(m, M - 1);
    row_off[mt] = (int64_t)src * p.lda;
  }

  // Row factors of a norm whose sums of squares arrive in parts: one wave per row, fixed order.
  // The first 256 parts of a row are requested here, ahead of everything else, and added up once
  // the first weights have been requested (see the main loop).
  float* scale_s = ss_part + S_WAVES * MT * 16;                      // [MT * 16]
  constexpr int RPW = MT * 16 / S_WAVES;                             // rows per wave
  constexpr int PRE = 4;                                             // parts requested ahead, in wavefuls
  float pre[RPW][PRE];
  if (p.in_sumsq) {
#pragma unroll
    for (int ri = 0; ri < RPW; ++ri) {
      const int m = min(wave + ri * S_WAVES, M - 1);
      const int64_t src = p.rows ? p.rows[m] : m;
      const bool row_there = wave + ri * S_WAVES < M;        // the same for the whole wave
#pragma unroll
      for (int h = 0; h < PRE; ++h) {
        const int q = lane + h * TL_WAVE;
        pre[ri][h] = 0.f;
        if (!row_there || h * TL_WAVE >= p.in_parts) continue;      // the same for the whole wave: nothing to ask for
        if (q < p.in_parts) pre[ri][h] = p.in_sumsq[src * p.in_parts + q];
      }
    }
  }
  auto row_factors = [&]() {
    if (!p.in_sumsq) return;
#pragma unroll
    for (int ri = 0; ri < RPW; ++ri) {
      const int r = wave + ri * S_WAVES;
      float t = (pre[ri][0] + pre[ri][1]) + (pre[ri][2] + pre[ri][3]);
      if (p.in_parts > PRE * TL_WAVE) {
        const int m = min(r, M - 1);
        const int64_t src = p.rows ? p.rows[m] : m;
        for (int q = lane + PRE * TL_WAVE; q < p.in_parts; q += TL_WAVE) t += p.in_sumsq[src * p.in_parts + q];
      }
      t = wave_sum(t);
      if (lane == 0) scale_s[r] = 1.f / sqrtf(t / (float)p.in_width + p.in_eps);
    }
  };

  // A stage is UN k blocks of 128 (all loads of a stage are issued together).  Where the
  // registers allow, two stages take turns, so the loads of the next stage are in flight while
  // this one is multiplied; with one tile the registers are better spent on a second resident
  // workgroup.  Loads are unconditional with the address clamped into the matrix: a predicated
  // load would become a branch and the stages could not overlap.  Rows beyond M or N only feed
  // outputs that are never written; a chunk beyond K is zeroed on the weight side when it is used.
  constexpr int UN = TILES == 1 ? 2 : 1;
  constexpr bool TWO_STAGES = DEEP || (TILES > 1 && MT + CT <= 5);
  struct Stage {
    bf16x8 fw[UN][CT][4];
    SkinnyChunk<PRO> fa[UN][MT][4];
    NormChunk nw[PRO == PRO_NORM ? UN : 1][PRO == PRO_NORM ? 4 : 1];
  };
  const int nblk = (K + KBLK - 1) / KBLK;
  auto load = [&](Stage& st, int blk) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      // MFMA i of the block covers k = i*32 .. i*32+31, lane group g its 8 k from g*8: one load
      // instruction then reads 64 contiguous bytes of each of the 16 weight rows
      if (u > 0 && blk + u * S_WAVES >= nblk) continue;      // the same for the whole wave: no such block
      const int kb = (blk + u * S_WAVES) * KBLK + kh + g * 8;
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
#pragma unroll
        for (int i = 0; i < 4; ++i) st.fw[u][ct][i] = *(const bf16x8*)(wrow[ct] + min(kb + i * KW, K - 8));
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (u > 0 && blk + u * S_WAVES >= nblk) continue;
      const int kb = (blk + u * S_WAVES) * KBLK + kh + g * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int k = min(kb + i * KW, K - 8);
        if constexpr (PRO == PRO_NORM) st.nw[u][i].load(p, k);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) st.fa[u][mt][i].load(p, row_off[mt] + k);
      }
    }
  };
  f32x4 acc[MT][CT];
  float ss[MT];                            // this lane's share of sum x^2 of its rows (norm prologue)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    ss[mt] = 0.f;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) acc[mt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  auto multiply = [&](const Stage& st, int blk) {
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      if (u > 0 && blk + u * S_WAVES >= nblk) continue;      // nothing was loaded for it
      const int kb = (blk + u * S_WAVES) * KBLK + kh + g * 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool k_ok = kb + i * KW < K;
        bf16x8 z = {};
        bf16x8 fa[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          fa[mt] = skinny_operand(st.fa[u][mt][i], st.nw[PRO == PRO_NORM ? u : 0][PRO == PRO_NORM ? i : 0], k_ok,
                                  ss[mt]);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) {
          const bf16x8 fw = k_ok ? st.fw[u][ct][i] : z;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[mt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw, fa[mt], acc[mt][ct], 0, 0, 0);
        }
      }
    }
  };
  constexpr int STEP = S_WAVES * UN;
  // The row factors are worked out while the first weights are on their way: their operands were
  // requested before and arrive first, and the wave has nothing else to do until the weights come.
  if constexpr (TWO_STAGES) {
    Stage s0, s1;
    int blk = wave;
    if (blk < nblk) load(s0, blk);
    if (blk + STEP < nblk) load(s1, blk + STEP);
    row_factors();
    if (blk < nblk) {
      while (true) {
        const int b1 = blk + STEP;
        multiply(s0, blk);
        if (b1 >= nblk) break;
        const int b2 = b1 + STEP;
        if (b2 < nblk) load(s0, b2);
        multiply(s1, b1);
        if (b2 >= nblk) break;
        blk = b2;
        if (blk + STEP < nblk) load(s1, blk + STEP);
      }
    }
  } else {
    Stage s0;
    int blk = wave;
    if (blk < nblk) load(s0, blk);
    row_factors();
    while (blk < nblk) {
      multiply(s0, blk);
      blk += STEP;
      if (blk < nblk) load(s0, blk);
    }
  }
  // tile layout: lane holds rows (weight rows) g*4 + r, column (activation row) r16
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int r = 0; r < 4; ++r) part[wave * TILES + mt * CT + ct][g * 4 + r][r16] = acc[mt][ct][r];
  if constexpr (PRO == PRO_NORM) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float t = ss[mt];
      t = sum_over_rows(t);
      if (g == 0) ss_part[wave * (MT * 16) + mt * 16 + r16] = t;
    }
  }
  __syncthreads();
  TO* out = (TO*)p.out;
#pragma unroll
  for (int j = 0; j < EPT; ++j) {
    const int e = tid + j * S_THREADS;
    if (e >= (HALF ? 64 : TILES * 256)) continue;       // whole waves: 256 elements are four waves
    const int tile = e / 256, m_local = HALF ? e / 8 : (e % 256) / 16, nn = HALF ? e % 8 : e % 16;
    const int m = (tile / CT) * 16 + m_local, n = n0 + (tile % CT) * 16 + nn;
    const bool valid = m < M && n < N && n - n0 < cw;
    float scale = 1.f;                    // the row factor left out of the operands
    if (p.row_scale) scale = p.row_scale[min(m, M - 1)];
    if (p.in_sumsq) scale = scale_s[(tile / CT) * 16 + m_local];
    if constexpr (PRO == PRO_NORM) {
      float t = 0.f;
#pragma unroll
      for (int wv = 0; wv < S_WAVES; ++wv) t += ss_part[wv * (MT * 16) + (tile / CT) * 16 + m_local];
      scale = 1.f / sqrtf(t / (float)K + p.eps);
    }
    if constexpr (SWIGLU) {   // columns (2j, 2j+1) = (gate_j, up_j): even threads make one output of a pair
      if ((nn & 1) || !valid) continue;
      float gv = 0.f, uv = 0.f;
#pragma unroll
      for (int wv = 0; wv < S_WAVES; ++wv) {
        gv += part[wv * TILES + tile][nn][m_local];
        uv += part[wv * TILES + tile][nn + 1][m_local];
      }
      out[(int64_t)m * p.ldo + n / 2] = from_f32<TO>(swiglu_pair_fast(gv * scale, uv * scale));
    } else {
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < S_WAVES; ++wv) {
        v += part[wv * TILES + tile][nn][m_local];
        if constexpr (HALF) v += part[wv * TILES + tile][nn + 8][m_local + 8];
      }
      v = v * scale + res_v[j];
      if (valid) out[(int64_t)m * p.ldo + n] = from_f32<TO>(v);
      if constexpr (sizeof(TO) == 4) {
        if (p.emit_operand) {             // uniform: the lanes of a row group stay together
          if (valid) {
            const float wn = p.emit_w_is_f32 ? ((const float*)p.emit_w)[n] : (float)((const bf16_t*)p.emit_w)[n];
            p.emit_operand[(int64_t)m * N + n] = (bf16_t)(wn * v);
          }
          float sq = valid ? v * v : 0.f;
          sq = group_sum<COLS>(sq);
          if (nn == 0 && m < M) {
            if (CT > 1 && cw != COLS * CT) {
              // a part per workgroup and column tile, empty ones (beyond N) included
              p.emit_sumsq[(int64_t)m * ((N + cw - 1) / cw * CT) + blockIdx.x * CT + tile % CT] = sq;
            } else if (n < N) {     // a column group that begins beyond N has no part of its own
              if (cw == COLS * CT) p.emit_sumsq[(int64_t)m * ((N + COLS - 1) / COLS) + (n0 / COLS + tile % CT)] = sq;
              else p.emit_sumsq[(int64_t)m * ((N + cw - 1) / cw) + blockIdx.x] = sq;
            }
          }
        }
      }
    }
  }
}

// Column tiles per workgroup: every workgroup reads all M activation rows, so with more rows it
// should own more columns, or the activations are read more often than the weights.
template <int MT, int CT, bool DEEP, typename TO, int PRO, bool SWIGLU, bool HALF = false>
static int launch_skinny_deep(const SkinnyArgs& p, hipStream_t stream) {
  constexpr size_t smem = (size_t)S_WAVES * MT * CT * 16 * 17 * sizeof(float) + (size_t)(S_WAVES + 1) * MT * 16 * sizeof(float);
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute((const void*)gemm_skinny_bf16_kernel<MT, CT, DEEP, TO, PRO, SWIGLU, HALF>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return TL_ERR_LAUNCH;
    configured = true;
  }
  constexpr int cols = HALF ? 8 : S_COLS * CT;
  const int cw = (!HALF && p.cols_wg > 0) ? p.cols_wg : cols;
  dim3 g((p.N + cw - 1) / cw), b(S_THREADS);
  hipLaunchKernelGGL((gemm_skinny_bf16_kernel<MT, CT, DEEP, TO, PRO, SWIGLU, HALF>), g, b, smem, stream, p);
  return TL_OK;
}

// Columns a workgroup owns in the plain one-tile kernel: 16, or fewer (even) where that turns 129
// to 255 workgroups, which leave compute units idle, into one round of at most 256; 8 where 16
// would leave half of the compute units without a workgroup (whole decode steps of 9 to 16 rows
// with products of 2,048 columns: 3 % faster).
static int skinny_cols_wg(int N) {
  const int tiles = (N + S_COLS - 1) / S_COLS;
  if (tiles > 64 && tiles <= 128) return 8;
  if (tiles <= 128 || tiles >= 256) return S_COLS;
  const int cw = (N + 255) / 256;
  return cw + (cw & 1);
}

// Columns a workgroup owns with `ct` (2 to 4) column tiles: what makes exactly 256 workgroups, where
// that needs all `ct` tiles (0: all columns of the tiles).
static int skinny_cols_wg_tiles(int N, int ct) {
  const int cw = (N + 255) / 256 + ((N + 255) / 256 & 1);
  return cw > S_COLS * (ct - 1) && cw < S_COLS * ct ? cw : 0;
}

// 8 columns a workgroup: for at most 8 rows and an inner size that gives every wave at least
// one block of four MFMAs, where that still gives no more workgroups than there are compute
// units (measured: otherwise it is slower).
static bool skinny_half(int M, int N, int K) { return M <= 8 && K >= 2048 && (N + 7) / 8 <= 256; }

template <int MT, int CT, typename TO, int PRO, bool SWIGLU>
static int launch_skinny_tile(const SkinnyArgs& p, hipStream_t stream) {
  if constexpr (MT * CT == 1 && PRO == PRO_NONE && !SWIGLU) {
    if (skinny_half(p.M, p.N, p.K)) {
      if (p.K > 4096) return launch_skinny_deep<MT, CT, true, TO, PRO, SWIGLU, true>(p, stream);
      return launch_skinny_deep<MT, CT, false, TO, PRO, SWIGLU, true>(p, stream);
    }
  }
  if constexpr (CT == 1) {
    SkinnyArgs q = p;
    q.cols_wg = skinny_cols_wg(p.N);
    if constexpr (MT == 1 && PRO == PRO_NONE) {
      if (p.K > 4096) return launch_skinny_deep<MT, CT, true, TO, PRO, SWIGLU>(q, stream);
    }
    return launch_skinny_deep<MT, CT, false, TO, PRO, SWIGLU>(q, stream);
  }
  return launch_skinny_deep<MT, CT, false, TO, PRO, SWIGLU>(p, stream);
}

// More column tiles only while at least 256 workgroups remain: fewer cannot pull the weights
// through fast enough.
template <int MT, typename TO, bool SWIGLU>
static int launch_skinny_rows(const SkinnyArgs& p, hipStream_t stream) {
  if (p.N >= 256 * 64) return launch_skinny_tile<MT, 4, TO, PRO_NONE, SWIGLU>(p, stream);
  if (p.N >= 256 * 32) return launch_skinny_tile<MT, 2, TO, PRO_NONE, SWIGLU>(p, stream);
  return launch_skinny_tile<MT, 1, TO, PRO_NONE, SWIGLU>(p, stream);
}

template <typename TO, int PRO, bool SWIGLU>
static int launch_skinny(const SkinnyArgs& p, hipStream_t stream) {
  const int mt = (p.M + 15) / 16;
  if (mt == 1) {
    if constexpr (PRO == PRO_NONE) {
      // A workgroup fetches at a rate of its own, and every workgroup fetches all activation rows:
      // the product is fastest with ONE round of workgroups over the 256 compute units, each owning
      // as many column tiles as that takes (up to four).  (Also with few rows: timed alone, more
      // workgroups looked faster below 8 rows; whole decode steps are 1 % faster at 4 rows with
      // one round and equal at 1 and 2.)  Wider products run several rounds: one column tile below
      // 8 rows, two from 8 rows on, where the activation rows a workgroup fetches weigh as much as
      // its weights (whole decode steps at hidden 4096, intermediate 14336, vocabulary 128256:
      // 3 % faster at 8 rows and 9 % at 16 with two tiles, 2 to 6 % slower at 1 to 6; four tiles
      // are slower than two at 16 rows).
      const int ct = (p.N + 256 * S_COLS - 1) / (256 * S_COLS);
      if (ct >= 2 && ct <= 4) {
        // exactly 256 workgroups where the columns allow it: the last column tile of each is partly used
        // (whole decode steps: 0.3 % faster at hidden 2048, 0.7 to 1.4 % at hidden 4096, where q/k/v went
        // from 192 workgroups to 256)
        SkinnyArgs q = p;
        q.cols_wg = skinny_cols_wg_tiles(p.N, ct);
        if (ct == 2) return launch_skinny_tile<1, 2, TO, PRO, SWIGLU>(q, stream);
        if (ct == 3) return launch_skinny_tile<1, 3, TO, PRO, SWIGLU>(q, stream);
        return launch_skinny_tile<1, 4, TO, PRO, SWIGLU>(q, stream);
      }
      // (below 8 rows too where one tile would leave the last of the kernel's stages, 16 k blocks of 128
      // over the eight waves, half empty or emptier at a long inner size: inner size 5120 x 27,648
      // columns at 1 row, 52 us against 61)
      const int tail_blocks = ((p.K + S_KBLK - 1) / S_KBLK) % (2 * S_WAVES);
      const bool half_empty_stage = p.K > 4096 && tail_blocks >= 1 && tail_blocks <= S_WAVES;
      if (ct > 4 && (p.M >= 8 || half_empty_stage)) {
        // several rounds of two column tiles: as many columns a workgroup (17 to 32, even) as make whole
        // rounds of 256 workgroups (28,672 columns: 1,024 workgroups of 28 instead of 896 of 32, which
        // are four rounds as well)
        SkinnyArgs q = p;
        const int rounds = (p.N + 256 * 2 * S_COLS - 1) / (256 * 2 * S_COLS);
        const int cw = (p.N + rounds * 256 - 1) / (rounds * 256);
        q.cols_wg = cw + (cw & 1);
        // (a product that prepares a norm keeps whole tiles: its parts are counted per 16 columns)
        if (q.cols_wg <= S_COLS || q.cols_wg >= 2 * S_COLS || p.emit_operand) q.cols_wg = 0;
        return launch_skinny_tile<1, 2, TO, PRO, SWIGLU>(q, stream);
      }
    }
    return launch_skinny_tile<1, 1, TO, PRO, SWIGLU>(p, stream);
  }
  if constexpr (PRO == PRO_NONE) {       // the norm prologue exists for one row tile only
    if (mt == 2) return launch_skinny_rows<2, TO, SWIGLU>(p, stream);
    if (mt == 3) return launch_skinny_rows<3, TO, SWIGLU>(p, stream);
    return launch_skinny_rows<4, TO, SWIGLU>(p, stream);
  }
  return TL_ERR_ARG;
}

template <int PRO>
static int launch_skinny_out(const SkinnyArgs& p, int out_dtype, bool swiglu, hipStream_t stream) {
  if (out_dtype == 0 && !swiglu) return launch_skinny<float, PRO, false>(p, stream);
  if (out_dtype == 1 && !swiglu) return launch_skinny<bf16_t, PRO, false>(p, stream);
  if (out_dtype == 1 && swiglu) return launch_skinny<bf16_t, PRO, true>(p, stream);
  return TL_ERR_ARG;
}

// Column tiles a workgroup of the float32 few-row kernel owns: one, or, with one row tile and more
// than 256 column tiles of 16, up to three (four would not leave the registers for a piece of weights
// ahead) while the block sums fit into LDS, and of them as many columns (*cols_wg, even; 0: all) as make
// whole rounds of 256 workgroups: 5,120 columns are one round of 20, 15,360 two rounds of 30, 28,672
// three rounds of 38, where whole tiles would leave the last round a quarter full.
static int f32_rows_col_tiles(int M, int N, int K, int cols, int* cols_wg = nullptr) {
  if (cols_wg) *cols_wg = 0;
  if (M > 16 || cols != 16) return 1;
  const int tiles = (N + 15) / 16, nkb = (K + F_KBLOCK - 1) / F_KBLOCK;
  if (tiles <= 256) return 1;
  for (int rounds = 1; rounds <= 1024; ++rounds) {
    int cw = (N + 256 * rounds - 1) / (256 * rounds);
    cw += cw & 1;
    const int ct = (cw + 15) / 16;
    if (ct > 3 || (size_t)nkb * 16 * 16 * ct * sizeof(float) > 96 * 1024) continue;
    if (cols_wg && cw < 16 * ct && ct > 1) *cols_wg = cw;
    return ct;
  }
  return 1;
}

}  // namespace

extern "C" {

// Float32, at most 64 rows: out = rmsnorm(x; norm_w, eps) @ w.T, then the epilogue of tl_linear_tile
// (0: + residual, 1: SiLU-gate), the norm inside the product's kernel.  Returns TL_ERR_ARG for sizes
// that kernel does not take (tl_linear_norm_f32_ok says which).
int tl_linear_norm_f32_ok(int M, int N, int K, int64_t lda) {
  const int nkb = (K + F_KBLOCK - 1) / F_KBLOCK, mts = (M + 15) / 16;
  const int cols = (N + 7) / 8 <= 256 ? 8 : 16;
  const size_t smem = (size_t)mts * nkb * 16 * (cols + 1) * sizeof(float);
  return M > 0 && M <= 16 * FR_MAX_MT && K % 4 == 0 && lda % 4 == 0 && smem <= 96 * 1024;
}

// Column tiles the plain float32 few-row product gives a workgroup at these sizes.  More than one: the
// product is so wide that a norm in front of it is cheaper as a kernel of its own (tl_norm_prescale_f32)
// with its factors applied to this product's sums than inside tl_linear_norm_f32, which fetches a
// workgroup's activation rows once per column tile; the bits are the same either way.
int tl_linear_f32_col_tiles(int M, int N, int K) {
  return f32_rows_col_tiles(M, N, K, (N + 7) / 8 <= 256 ? 8 : 16);
}

int tl_linear_norm_f32(const float* x, const float* norm_w, float eps, const float* w, float* out,
                       const float* residual, int M, int N, int K, int64_t lda, int64_t ldo, int epilogue,
                       hipStream_t stream) {
  const bool swiglu = epilogue == 1;
  if (!tl_linear_norm_f32_ok(M, N, K, lda) || N <= 0 || lda < K || ldo < (swiglu ? N / 2 : N) || epilogue < 0 ||
      epilogue > 1 || ((uintptr_t)x | (uintptr_t)w | (uintptr_t)norm_w) % 16 != 0)
    return TL_ERR_ARG;
  if (swiglu && ((N & 1) || residual)) return TL_ERR_ARG;
  const int nkb = (K + F_KBLOCK - 1) / F_KBLOCK, mts = (M + 15) / 16;
  const int cols = (N + 7) / 8 <= 256 ? 8 : 16;
  const size_t smem = (size_t)mts * nkb * 16 * (cols + 1) * sizeof(float);
  static bool configured = false;
  if (!configured) {
    const void* kernels[4] = {(const void*)gemm_f32_rows_kernel<true, 16, true>, (const void*)gemm_f32_rows_kernel<false, 16, true>,
                              (const void*)gemm_f32_rows_kernel<true, 8, true>, (const void*)gemm_f32_rows_kernel<false, 8, true>};
    for (const void* k : kernels)
      if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess) return TL_ERR_LAUNCH;
    configured = true;
  }
  dim3 gr((N + cols - 1) / cols);
#define TL_F32_ROWS_NORM(SW, CO)                                                                                 \
  hipLaunchKernelGGL((gemm_f32_rows_kernel<SW, CO, true>), gr, dim3(FR_THREADS), smem, stream, x, w, out, residual, M, \
                     N, K, lda, ldo, norm_w, eps)
  if (swiglu && cols == 16) TL_F32_ROWS_NORM(true, 16);
  else if (swiglu) TL_F32_ROWS_NORM(true, 8);
  else if (cols == 16) TL_F32_ROWS_NORM(false, 16);
  else TL_F32_ROWS_NORM(false, 8);
#undef TL_F32_ROWS_NORM
  return tl_launch_status();
}

// Float32, any number of rows: h[m, :] = norm_w * x[rows[m] or m, :] and inv_rms[m] = 1 / rms of that
// row, for a product that takes inv_rms as its row_scale: together rmsnorm(x) @ w.T with the bits of
// tl_linear_norm_f32.  h is [n_rows, K] contiguous.
int tl_norm_prescale_f32(const float* x, const float* norm_w, const int32_t* rows, float* h, float* inv_rms,
                         int n_rows, int K, int64_t lda, float eps, hipStream_t stream) {
  if (n_rows <= 0) return TL_OK;
  if (K <= 0 || lda < K) return TL_ERR_ARG;
  const int nkb = (K + F_KBLOCK - 1) / F_KBLOCK;
  const size_t smem = (size_t)nkb * 4 * sizeof(float);
  if (smem > 48 * 1024) return TL_ERR_ARG;
  const bool vec = K % 4 == 0 && lda % 4 == 0 && ((uintptr_t)x | (uintptr_t)norm_w | (uintptr_t)h) % 16 == 0;
  if (vec)
    hipLaunchKernelGGL(norm_prescale_f32_kernel<true>, dim3(n_rows), dim3(FN_THREADS), smem, stream, x, norm_w, rows, h,
                       inv_rms, K, lda, eps);
  else
    hipLaunchKernelGGL(norm_prescale_f32_kernel<false>, dim3(n_rows), dim3(FN_THREADS), smem, stream, x, norm_w, rows,
                       h, inv_rms, K, lda, eps);
  return tl_launch_status();
}

// out = a @ w.T, then an epilogue.  dtype: element type of a and w (0 float32, 1 bfloat16);
// out_dtype: of out.  lda: row stride of a in elements; ldo: row stride of out and residual.
// row_scale (optional): every row m of the product is multiplied by row_scale[m] before the epilogue.
// epilogue 0: (+ residual[m, n]), out is [M, N].
// epilogue 1: SiLU-gate of interleaved columns, out[m, j] = silu(c[m, 2j]) * c[m, 2j+1], out is
//             [M, N/2] of the input's type; N must be even; no residual.
// tile (bfloat16, M > 64): 0 lets the size decide; 1..4 force 256x256, 256x128, 128x128, 64x128.
int tl_linear_tile(const void* a, const void* w, void* out, const float* residual, const float* row_scale, int M,
                   int N, int K, int64_t lda, int64_t ldo, int dtype, int out_dtype, int epilogue, int tile,
                   hipStream_t stream) {
  if (M <= 0) return TL_OK;
  const bool swiglu = epilogue == 1;
  if (N <= 0 || K <= 0 || lda < K || ldo < (swiglu ? N / 2 : N) || epilogue < 0 || epilogue > 1 || tile < 0 ||
      tile > 4)
    return TL_ERR_ARG;
  if (swiglu && ((N & 1) || residual || out_dtype != dtype)) return TL_ERR_ARG;
  if (dtype == 0) {
    if (out_dtype != 0) return TL_ERR_ARG;
    const bool vec = K % 4 == 0 && lda % 4 == 0 && ((uintptr_t)a | (uintptr_t)w) % 16 == 0;
    const int nkb = (K + F_KBLOCK - 1) / F_KBLOCK;
    const int mts = (M + 15) / 16;
    // One row tile: 8 columns a workgroup where that still is one round of workgroups over the 256
    // compute units (a workgroup fills a compute unit: more than 256 of them would run in two rounds).
    // More row tiles (17 to 64 rows, up to 256 by the estimate below): whole matrix tiles of 16 columns, and the row tiles shared out
    // over as many groups of workgroups (1, 2 or 4) as it takes to give every compute unit a
    // workgroup and to fit the block sums into LDS.
    int cols = (N + 7) / 8 <= 256 ? 8 : 16, groups = 1;
    if (mts > 1) {
      cols = 16;
      const int col_tiles = (N + 15) / 16;
      // (more groups only while they stay within one round of 256 workgroups: a second, partly filled
      // round costs as much as a full one)
      while (groups < mts && (col_tiles * groups * 2 <= 256 || (size_t)((mts + groups - 1) / groups) * nkb * 16 * cols * sizeof(float) > 96 * 1024))
        groups *= 2;
    }
    const int tiles_wg = (mts + groups - 1) / groups;
    int cols_wg = 0;
    const int ct = f32_rows_col_tiles(M, N, K, cols, &cols_wg);
    const size_t rows_smem = (size_t)tiles_wg * nkb * 16 * cols * ct * sizeof(float);
    // Up to 64 rows the few-row kernel; up to 256 where it is estimated faster than the tiled kernel, whose few
    // tiles each walk the whole inner size (measured at inner size 2048: 87 us a round of up to 352 tiles of
    // 64 x 64, 204 us a round of 128 x 128; the few-row kernel 0.66 us per row tile and million weights:
    // 2048 x 2048 at 128 rows 25 us against 89, 5632 x 2048 at 256 rows 124 against 232).  The bits are the same.
    bool few_rows = M <= 16 * FR_MAX_MT;
    if (!few_rows && M <= 256) {
      const int64_t big_t = ceil_div64(N, 128) * ceil_div64(M, 128), small_t = ceil_div64(N, 64) * ceil_div64(M, 64);
      const bool small_tiles = (double)ceil_div64(small_t, 256) / (4 * 0.6) < (double)ceil_div64(big_t, 256);
      const double tiled_us = (K / 2048.0) * (small_tiles ? 87.0 * (small_t > 352 ? small_t / 352.0 : 1.0)
                                                          : 204.0 * (double)ceil_div64(big_t, 256));
      // (a long inner size leaves LDS for the block sums of one or two row tiles a workgroup only, and the
      // weights are then fetched once per row tile: 14336 x 4096 at 256 rows 876 us against 657)
      const double per_tile = tiles_wg >= 4 ? 0.66 : (tiles_wg >= 2 ? 0.8 : 0.98);
      few_rows = per_tile * mts * ((double)N * K / 1e6) + 8.0 < tiled_us;
    }
    if (few_rows && vec && rows_smem <= 96 * 1024) {
      static bool configured = false;
      if (!configured) {
        const void* kernels[12] = {(const void*)gemm_f32_rows_kernel<true, 8, false, false, 1, true>,
                                   (const void*)gemm_f32_rows_kernel<false, 8, false, false, 1, true>,
                                   (const void*)gemm_f32_rows_kernel<true, 16>, (const void*)gemm_f32_rows_kernel<false, 16>,
                                   (const void*)gemm_f32_rows_kernel<true, 8>, (const void*)gemm_f32_rows_kernel<false, 8>,
                                   (const void*)gemm_f32_rows_kernel<true, 16, false, true>,
                                   (const void*)gemm_f32_rows_kernel<false, 16, false, true>,
                                   (const void*)gemm_f32_rows_kernel<true, 16, false, false, 2>,
                                   (const void*)gemm_f32_rows_kernel<false, 16, false, false, 2>,
                                   (const void*)gemm_f32_rows_kernel<true, 16, false, false, 3>,
                                   (const void*)gemm_f32_rows_kernel<false, 16, false, false, 3>};
        for (const void* k : kernels)
          if (hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024) != hipSuccess)
            return TL_ERR_LAUNCH;
        configured = true;
      }
      const int cw = cols_wg > 0 ? cols_wg : cols * ct;
      dim3 gr((N + cw - 1) / cw, (mts + tiles_wg - 1) / tiles_wg);
#define TL_F32_ROWS_K(...)                                                                                          \
  hipLaunchKernelGGL((gemm_f32_rows_kernel<__VA_ARGS__>), gr, dim3(FR_THREADS), rows_smem, stream, (const float*)a, \
                     (const float*)w, (float*)out, residual, M, N, K, lda, ldo, (const float*)nullptr, 0.f, row_scale, \
                     tiles_wg, cols_wg)
#define TL_F32_ROWS(SW, CO, WI, CTI) TL_F32_ROWS_K(SW, CO, false, WI, CTI)
#define TL_F32_ROWS_CT(SW)                                                                                           \
  do {                                                                                                               \
    if (ct == 3) TL_F32_ROWS(SW, 16, false, 3);                                                                      \
    else if (ct == 2) TL_F32_ROWS(SW, 16, false, 2);                                                                 \
    else TL_F32_ROWS(SW, 16, false, 1);                                                                              \
  } while (0)
      if (mts > 1 && swiglu) TL_F32_ROWS(true, 16, true, 1);
      else if (mts > 1) TL_F32_ROWS(false, 16, true, 1);
      else if (swiglu && cols == 16) TL_F32_ROWS_CT(true);
      else if (swiglu && M <= 8) TL_F32_ROWS_K(true, 8, false, false, 1, true);      // cols == 8: pairs of k blocks
      else if (swiglu) TL_F32_ROWS(true, 8, false, 1);
      else if (cols == 16) TL_F32_ROWS_CT(false);
      else if (M <= 8) TL_F32_ROWS_K(false, 8, false, false, 1, true);
      else TL_F32_ROWS(false, 8, false, 1);
#undef TL_F32_ROWS_CT
#undef TL_F32_ROWS
#undef TL_F32_ROWS_K
      return tl_launch_status();
    }
    // 128 x 128 tiles, or 64 x 64 where those take fewer rounds of workgroups over the 256 compute
    // units even at 0.6 of the larger tile's rate (it fetches twice the operand bytes per flop)
    const int64_t big = ceil_div64(N, 128) * ceil_div64(M, 128), small = ceil_div64(N, 64) * ceil_div64(M, 64);
    const bool use_small = (double)ceil_div64(small, 256) / (4 * 0.6) < (double)ceil_div64(big, 256);
    const int bt = use_small ? 64 : 128;
    dim3 g((N + bt - 1) / bt, (M + bt - 1) / bt);
#define TL_F32_TILED(SW, VE)                                                                                        \
  do {                                                                                                              \
    if (use_small)                                                                                                  \
      hipLaunchKernelGGL((gemm_f32_kernel<SW, VE, 2>), g, dim3(F_THREADS), 0, stream, (const float*)a,              \
                         (const float*)w, (float*)out, residual, M, N, K, lda, ldo, row_scale);                     \
    else                                                                                                            \
      hipLaunchKernelGGL((gemm_f32_kernel<SW, VE, 4>), g, dim3(F_THREADS), 0, stream, (const float*)a,              \
                         (const float*)w, (float*)out, residual, M, N, K, lda, ldo, row_scale);                     \
  } while (0)
    if (swiglu && vec) TL_F32_TILED(true, true);
    else if (swiglu) TL_F32_TILED(true, false);
    else if (vec) TL_F32_TILED(false, true);
    else TL_F32_TILED(false, false);
#undef TL_F32_TILED
  } else if (dtype == 1) {
    if (K % 8 || lda % 8) return TL_ERR_ARG;
    if (out_dtype != 0 && out_dtype != 1) return TL_ERR_ARG;
    if (M <= 64) {
      SkinnyArgs p{a, (const bf16_t*)w, out, residual, nullptr, nullptr, row_scale, 0.f, 0, M, N, K, lda, ldo};
      const int rc = launch_skinny_out<PRO_NONE>(p, out_dtype, swiglu, stream);
      if (rc != TL_OK) return rc;
    } else {
      int rc;
      if (swiglu)
        rc = launch_gemm_bf16_any<bf16_t, true>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)out, residual, row_scale,
                                                M, N, K, lda, ldo, tile, 0, stream);
      else if (out_dtype == 0)
        rc = launch_gemm_bf16_any<float, false>((const bf16_t*)a, (const bf16_t*)w, (float*)out, residual, row_scale,
                                                M, N, K, lda, ldo, tile, 0, stream);
      else
        rc = launch_gemm_bf16_any<bf16_t, false>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)out, residual,
                                                 row_scale, M, N, K, lda, ldo, tile, 0, stream);
      if (rc != TL_OK) return rc;
    }
  } else {
    return TL_ERR_ARG;
  }
  return tl_launch_status();
}

int tl_linear(const void* a, const void* w, void* out, const float* residual, const float* row_scale, int M,
              int N, int K, int64_t lda, int64_t ldo, int dtype, int out_dtype, int epilogue,
              hipStream_t stream) {
  return tl_linear_tile(a, w, out, residual, row_scale, M, N, K, lda, ldo, dtype, out_dtype, epilogue, 0, stream);
}

// The bfloat16 product that takes part in handing a norm from one product to the next (see
// SkinnyArgs and TileNorm): the few-row kernel up to 64 rows, the tiled kernel beyond (no row
// gather then; a producer needs N to be a multiple of 64).  Consumer side: in_sumsq [rows of a,
// in_parts] (a is then the operand a producer wrote; `rows` gathers rows of both).  Producer side
// (out_dtype 0, epilogue 0): emit_w [N] (element type emit_w_dtype), emit_operand bf16 [M, N],
// emit_sumsq float [M, tl_handoff_parts(M, N, K)].  Either side may be absent.
int tl_linear_handoff(const void* a, const void* w, void* out, const float* residual, const int32_t* rows,
                      const float* in_sumsq, int in_parts, float in_eps, int in_width, const void* emit_w,
                      int emit_w_dtype, void* emit_operand, float* emit_sumsq, int M, int N, int K, int64_t lda,
                      int64_t ldo, int out_dtype, int epilogue, hipStream_t stream) {
  if (M <= 0) return TL_OK;
  const bool swiglu = epilogue == 1;
  if (N <= 0 || K <= 0 || K % 8 || lda % 8 || lda < K || ldo < (swiglu ? N / 2 : N) || epilogue < 0 ||
      epilogue > 1 || (out_dtype != 0 && out_dtype != 1))
    return TL_ERR_ARG;
  if (swiglu && ((N & 1) || residual || out_dtype != 1)) return TL_ERR_ARG;
  if (in_sumsq && (in_parts <= 0 || in_width <= 0)) return TL_ERR_ARG;
  const bool emit = emit_operand != nullptr;
  if (emit && (!emit_w || !emit_sumsq || swiglu || out_dtype != 0 || (emit_w_dtype != 0 && emit_w_dtype != 1)))
    return TL_ERR_ARG;
  if (M > 64) {      // the tiled kernel
    if (rows || (emit && (N % 64 || ldo % 4))) return TL_ERR_ARG;
    TileNorm nm;
    if (emit) {
      nm.emit_w = emit_w;
      nm.emit_w_is_f32 = emit_w_dtype == 0 ? 1 : 0;
      nm.emit_operand = (bf16_t*)emit_operand;
      nm.emit_ld = N;
      nm.emit_sumsq = emit_sumsq;
      nm.emit_parts = N / 64;
    }
    if (in_sumsq) {
      nm.in_sumsq = in_sumsq;
      nm.in_parts = in_parts;
      nm.in_width = in_width;
      nm.in_eps = in_eps;
    }
    int rc;
    if (swiglu)
      rc = launch_gemm_bf16_any<bf16_t, true>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)out, residual, nm, M, N, K,
                                              lda, ldo, 0, 0, stream);
    else if (out_dtype == 0)
      rc = launch_gemm_bf16_any<float, false>((const bf16_t*)a, (const bf16_t*)w, (float*)out, residual, nm, M, N, K,
                                              lda, ldo, 0, 0, stream);
    else
      rc = launch_gemm_bf16_any<bf16_t, false>((const bf16_t*)a, (const bf16_t*)w, (bf16_t*)out, residual, nm, M, N, K,
                                               lda, ldo, 0, 0, stream);
    if (rc != TL_OK) return rc;
    return tl_launch_status();
  }
  SkinnyArgs p{a, (const bf16_t*)w, out, residual, nullptr, rows, nullptr, 0.f, 0, M, N, K, lda, ldo};
  if (emit) {
    p.emit_w = emit_w;
    p.emit_w_is_f32 = emit_w_dtype == 0 ? 1 : 0;
    p.emit_operand = (bf16_t*)emit_operand;
    p.emit_sumsq = emit_sumsq;
  }
  if (in_sumsq) {
    p.in_sumsq = in_sumsq;
    p.in_parts = in_parts;
    p.in_width = in_width;
    p.in_eps = in_eps;
  }
  const int rc = launch_skinny_out<PRO_NONE>(p, out_dtype, swiglu, stream);
  if (rc != TL_OK) return rc;
  return tl_launch_status();
}

// How many partial sums of squares per row tl_linear_handoff writes as a producer for these sizes
// (few rows: one per workgroup, per 16 columns, or per 8 where workgroups own 8; beyond: one per 64
// columns).
int tl_handoff_parts(int M, int N, int K) {
  if (M > 64) return (N + 63) / 64;
  if (skinny_half(M, N, K)) return (N + 7) / 8;
  // one column tile a workgroup (see launch_skinny and launch_skinny_rows): a part per workgroup
  if (M <= 16 && N > 256 * S_COLS && N <= 4 * 256 * S_COLS) {       // two to four column tiles a workgroup
    const int ct = (N + 256 * S_COLS - 1) / (256 * S_COLS), cwt = skinny_cols_wg_tiles(N, ct);
    return cwt ? (N + cwt - 1) / cwt * ct : (N + S_COLS - 1) / S_COLS;
  }
  const bool one_tile = M <= 16 || N < 256 * 32;
  const int cw = one_tile ? skinny_cols_wg(N) : S_COLS;
  return (N + cw - 1) / cw;
}

// See splitk_plan.  A caller that gets more than one split allocates a float32 workspace of
// splits * M * N elements and calls tl_linear_splitk with the same sizes.
int tl_splitk_plan(int M, int N, int K) {
  int tile, kps;
  return splitk_plan(M, N, K, &tile, &kps);
}

// The bfloat16 product with its inner size split over workgroups: partial products into
// `workspace` (float32 [splits, M, N], splits as tl_splitk_plan says), then one kernel that adds
// them up and applies the epilogue.  Arguments as tl_linear and tl_linear_handoff (no row gather);
// emit_sumsq is float [M, ceil(N / 1024)].
int tl_linear_splitk(const void* a, const void* w, void* out, const float* residual, const float* row_scale,
                     const float* in_sumsq, int in_parts, float in_eps, int in_width, const void* emit_w,
                     int emit_w_dtype, void* emit_operand, float* emit_sumsq, int M, int N, int K, int64_t lda,
                     int64_t ldo, int out_dtype, int epilogue, float* workspace, hipStream_t stream) {
  const bool swiglu = epilogue == 1;
  if (M <= 0 || N <= 0 || K <= 0 || K % 8 || lda % 8 || lda < K || ldo < (swiglu ? N / 2 : N) || epilogue < 0 ||
      epilogue > 1 || (out_dtype != 0 && out_dtype != 1) || !workspace)
    return TL_ERR_ARG;
  if (swiglu && ((N & 1) || residual || out_dtype != 1)) return TL_ERR_ARG;
  if (in_sumsq && (in_parts <= 0 || in_width <= 0)) return TL_ERR_ARG;
  const bool emit = emit_operand != nullptr;
  if (emit && (!emit_w || !emit_sumsq || swiglu || out_dtype != 0 || (emit_w_dtype != 0 && emit_w_dtype != 1)))
    return TL_ERR_ARG;
  int tile, kps;
  const int splits = splitk_plan(M, N, K, &tile, &kps);
  if (splits < 2) return TL_ERR_ARG;
  int rc = TL_OK;
  if (tile < 0) {
    const int slabs = kps / O_SLAB_K;
    const size_t smem = (size_t)(slabs < O_RING ? slabs : O_RING) * O_SLAB_BYTES;
    static bool configured = false;
    if (!configured) {
      if (hipFuncSetAttribute((const void*)gemm_oneshot_bf16_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              O_RING * O_SLAB_BYTES) != hipSuccess)
        return TL_ERR_LAUNCH;
      configured = true;
    }
    hipLaunchKernelGGL(gemm_oneshot_bf16_kernel, dim3((N + O_BN - 1) / O_BN, splits, (M + O_BM - 1) / O_BM), dim3(O_THREADS), smem, stream,
                       (const bf16_t*)a, (const bf16_t*)w, workspace, M, N, K, lda, slabs);
  } else {
    rc = launch_gemm_bf16_any<float, false>((const bf16_t*)a, (const bf16_t*)w, workspace, nullptr, nullptr, M, N, K, lda,
                                            N, tile, kps, stream);
  }
  if (rc != TL_OK) return rc;
  ReduceArgs p{workspace, splits, M, N, out, ldo, residual, row_scale, in_sumsq, in_parts, in_width, in_eps, emit_w,
               emit_w_dtype == 0 ? 1 : 0, (bf16_t*)emit_operand, emit_sumsq};
  if (M > 65535) return TL_ERR_ARG;
  dim3 g(M, (N + R_CHUNK - 1) / R_CHUNK), b(R_THREADS);
  if (swiglu)
    hipLaunchKernelGGL((splitk_reduce_kernel<bf16_t, true>), g, b, 0, stream, p);
  else if (out_dtype == 0)
    hipLaunchKernelGGL((splitk_reduce_kernel<float, false>), g, b, 0, stream, p);
  else
    hipLaunchKernelGGL((splitk_reduce_kernel<bf16_t, false>), g, b, 0, stream, p);
  return tl_launch_status();
}

// Few-row (M <= 16) bfloat16 product whose input is the float32 residual stream: the rows of a
// (gathered through `rows` if given) are RMS-normalised with norm_w (float32 or bfloat16) and eps
// inside the kernel.  Epilogues as in tl_linear.
int tl_linear_norm(const void* a, const void* w, void* out, const float* residual, const void* norm_w,
                   const int32_t* rows, float eps, int norm_w_dtype, int M, int N, int K, int64_t lda,
                   int64_t ldo, int out_dtype, int epilogue, hipStream_t stream) {
  if (M <= 0) return TL_OK;
  const bool swiglu = epilogue == 1;
  if (M > 16 || N <= 0 || K <= 0 || K % 8 || lda % 8 || lda < K || ldo < (swiglu ? N / 2 : N) || !norm_w ||
      (norm_w_dtype != 0 && norm_w_dtype != 1) || epilogue < 0 || epilogue > 1)
    return TL_ERR_ARG;
  if (swiglu && ((N & 1) || residual)) return TL_ERR_ARG;
  SkinnyArgs p{a, (const bf16_t*)w, out, residual, norm_w, rows, nullptr, eps, norm_w_dtype == 0 ? 1 : 0, M, N, K, lda, ldo};
  const int rc = launch_skinny_out<PRO_NORM>(p, out_dtype, swiglu, stream);
  if (rc != TL_OK) return rc;
  return tl_launch_status();
}

}  // extern "C"
