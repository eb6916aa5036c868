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
#include "no_alloc.h"
#include <mutex>
#include <type_traits>

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


// ============================================================== bfloat16 on MFMA
// flash_attn_bf16_kernel: the same function on the matrix cores, for head sizes
// that are multiples of 16 up to 128 and up to 16 query heads per kv head.
//
// A workgroup (eight wave64, four for heads beyond 64 dims) owns a tile of 16 query rows that
// share one request and one kv head: `tile_ntok` consecutive tokens times the G query heads of the
// group, row = token * G + head.  The waves split the 64-key tiles of the request's
// cache between them (and `n_splits` workgroups split them further for decoding
// with few requests) and merge their running (max, sum, output) at the end.  A wave reads its
// tile by itself: keys straight from memory into MFMA operands, values through a private LDS
// area.  (Sixteen waves a workgroup were measured slower at every context length: what a compute
// unit can have in flight is the limit, so keys are better spread over more workgroups.)
// Scores are computed transposed, S^T = K Q^T, with
// v_mfma_f32_16x16x32_bf16: a lane then holds 16 scores of ONE query row, so the
// online softmax is lane-local up to two shuffles, the probabilities are already in
// the B-operand layout of the second product O^T = V^T P^T, and the output
// accumulator of a lane belongs to that same row.  The probabilities enter the second
// product as a sum of two bfloat16 terms, so no accuracy is lost against a float32
// softmax times bfloat16 values.  V is staged in LDS as it is and transposed by the reads.
// Value rows of a tile outside [kv_begin, kv_end) read finite stand-in data: stale pages may hold
// anything, and 0 * NaN is NaN.
constexpr int FA_KT = 64;
constexpr int FA_VPAD = 8;      // padding of a row of the row-major V tile in LDS (elements)
constexpr float kNegBig = -1.0e30f;   // "no key yet": finite, so exp2(m - m') never sees inf - inf

// Two probabilities as two bfloat16 terms each, p = hi + lo, packed pairwise.  hi is p with the low
// 16 bits cut off (exact, one mask), lo = p - hi is exact in float32 and rounded to bfloat16: the
// pair carries 16 bits of p, as rounding hi would, for three vector instructions a value
// instead of four.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void split_pair(float pa, float pc, uint32_t& hi, uint32_t& lo) {
  const uint32_t ba = __float_as_uint(pa), bc = __float_as_uint(pc);
  hi = __builtin_amdgcn_perm(bc, ba, 0x07060302u);          // upper halves of both, a in the low word
  const f32x2 rest = {pa - __uint_as_float(ba & 0xffff0000u), pc - __uint_as_float(bc & 0xffff0000u)};
  lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(rest, bf16x2));
}

// The LDS transpose load of gfx950 (ds_read_b64_tr_b16).  The 16 lanes of a group each name four
// consecutive 16-bit elements; lane i of the group receives element i % 4 of the four chunks named
// by lanes i / 4, 4 + i / 4, 8 + i / 4 and 12 + i / 4.  With lane s naming V[key0 + s / 4][d0 + 4 * (s % 4) ..]
// of a row-major tile, lane i gets V[key0 .. key0 + 3][d0 + i]: four consecutive keys of one dim,
// half an MFMA operand of V^T, without the tile ever being stored transposed.
typedef short i16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x4 lds_read_transposed(const bf16_t* p) {
  return __builtin_bit_cast(bf16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)p));
}

// Optional fusion for decode steps (every tile is ONE new token): the query and the new key are
// rotated here and the new key and value are written to the cache here, instead of by a kernel of
// their own (rope_store_kernel) before this one.  q then points at the token's unrotated qkv row.
struct FusedRope {
  const float* cos_t;      // [positions, HD / 2]; null: nothing is fused
  const float* sin_t;
  bf16_t* k_cache_w;       // the caches, writable
  bf16_t* v_cache_w;
  int k_off, v_off;        // element offsets of this row's k and v heads from its q heads
};

// Rotate-half of 8 dims starting at d0 (a multiple of 8): own chunk x, partner chunk y = the dims
// d0 +- HD/2, with the 8 angles of the chunk in registers (c8, s8 = cos and sin of the pairs
// j0 .. j0 + 7).  The expressions are rope_store_kernel's; how the compiler fuses their
// multiplications and additions is its own choice in each kernel, so once in some ten thousand
// elements the two kernels differ in the last bit of a rotated value.
template <int HD>
__device__ __forceinline__ bf16x8 rotate_chunk_regs(const bf16x8 x, const bf16x8 y, int d0, const float* c8,
                                                    const float* s8) {
  bf16x8 r;
  const bool first = d0 < HD / 2;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float a = first ? (float)x[e] : (float)y[e];     // the pair's first-half value
    const float b = first ? (float)y[e] : (float)x[e];     // and its second-half value
    r[e] = (bf16_t)(first ? c8[e] * a - s8[e] * b : s8[e] * a + c8[e] * b);
  }
  return r;
}

template <int HDT, int WAVES>
__global__ __launch_bounds__(WAVES * TL_WAVE) void flash_attn_bf16_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_req, const int32_t* __restrict__ tile_tok0,
    const int32_t* __restrict__ tile_ntok, const int32_t* __restrict__ positions, bf16_t* __restrict__ out,
    int64_t out_stride, float* __restrict__ part_o, float* __restrict__ part_ml, int nq, int nkv,
    int block_size, float scale, int window, int n_splits, int n_tokens, const FusedRope fused) {
  constexpr int HD = HDT * 16;
  constexpr int KS = (HD + 31) / 32;       // k-steps of the score product
  constexpr int VS = HD + FA_VPAD;         // row stride of a wave's V tile in LDS
  constexpr int WAVE_ELEMS = FA_KT * VS;   // a wave's LDS area: its V tile, [key][dim]
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  bf16_t* smem = (bf16_t*)smem_raw;

  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int r16 = lane % 16, g = lane / 16;
  const int tile = blockIdx.x, kvh = blockIdx.y, split = blockIdx.z;
  const int G = nq / nkv;
  // no tile lists: tile i is token i of request i (a decode step), known without a round trip
  const int req = tile_req ? tile_req[tile] : tile, tok0 = tile_req ? tile_tok0[tile] : tile;
  const int ntok = tile_req ? tile_ntok[tile] : 1;
  const int32_t* bt = block_tables + (int64_t)req * max_blocks;
  bf16_t* Vl = smem + wave * WAVE_ELEMS;
  const bool do_rope = fused.cos_t != nullptr;
  // Key tiles are dealt out in turn (see below), so without a window this wave's first tile is
  // known here: the pages of this lane's rows in it (one value row, four key rows) are requested
  // together with the position.  The index is clamped into the table; an entry that belongs to no
  // key of the request is not used.
  // One lookup a lane: the page of key row `lane` of the 64-key tile that begins at key j0, as the
  // table holds it (any arithmetic on it here would make the wave wait for it here).  The lanes
  // hand the pages of the rows they load to each other.
  const int bs_shift = (block_size & (block_size - 1)) == 0 ? __builtin_ctz(block_size) : -1;
  auto page_index = [&](int j) { return bs_shift >= 0 ? j >> bs_shift : j / block_size; };     // uniform choice
  auto pages_at = [&](int j0) { return bt[min(page_index(j0 + lane), max_blocks - 1)]; };
  // (of the wave's first tile if the key range begins at 0: known without the positions)
  int next_pages = pages_at((split * WAVES + wave) * FA_KT);

  // this lane's query row
  const int tok_local = r16 / G, hh = r16 % G;
  const bool row_valid = tok_local < ntok;
  const int tok = tok0 + (row_valid ? tok_local : 0);
  const int head = kvh * G + hh;
  // The kernel begins with two round trips to memory and no more.  First everything whose address
  // the launch gives: the page lookup above, the position, the raw chunks of the query row (own
  // and partner dims).  Then what needs the position: the first key tile, the angles and, in the
  // wave that owns the new token's tile, its page and the raw chunks of its key.  All loads are unconditional (rows
  // and dims clamped into the tensors, the results masked later): asked for one by one under
  // their conditions they were seven round trips in a row.
  const int pos = row_valid ? positions[tok] : -1;
  bf16x8 qx[KS], qy[KS], kx[KS], ky[KS];
  {
    const bf16_t* qrow = q + (int64_t)tok * q_stride + (int64_t)head * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int dc = min(ks * 32 + g * 8, HD - 8), dp = (dc + HD / 2) % HD;
      qx[ks] = *(const bf16x8*)(qrow + dc);
      if (do_rope) qy[ks] = *(const bf16x8*)(qrow + dp);      // uniform
    }
  }
  const int row_lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;

  // key range of the tile: union over its rows
  const int hi = row_max_i32(pos), lo = row_min_i32(row_valid ? row_lo : 0x7fffffff);
  const int kv_end = hi + 1, kv_begin = lo;
  const int first_tile = kv_begin / FA_KT, last_tile = (kv_end + FA_KT - 1) / FA_KT;
  // Key tiles are dealt out in turn: tile (it0 + it) * stride + split * WAVES + wave belongs to
  // iteration `it` of this wave.  Which tiles a wave gets then does not depend on the positions,
  // so the page of its first tile can be looked up before the positions have arrived.
  const int stride = WAVES * n_splits, mine = split * WAVES + wave;
  const int it0 = first_tile / stride;
  const int iters = (last_tile - mine + stride - 1) / stride - it0;      // may be <= 0: no tile
  // fused mode: the one new token of the tile, at position kv_end - 1
  const int new_pos = kv_end - 1;
  // (a tile without a valid row has new_pos -1: it reads the angles of position 0 and uses nothing)
  const float* cs = do_rope ? fused.cos_t + (int64_t)max(new_pos, 0) * (HD / 2) : nullptr;
  const float* sn = do_rope ? fused.sin_t + (int64_t)max(new_pos, 0) * (HD / 2) : nullptr;

  const int new_tile = new_pos / FA_KT;
  const bool owns_new = do_rope && new_tile % (WAVES * n_splits) == split * WAVES + wave;
  float m_run = kNegBig, l_run = 0.f;
  f32x4 o[HDT];
#pragma unroll
  for (int dt = 0; dt < HDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  const float c_log2 = scale * 1.44269504088896341f;     // scores are kept in units of log2 e

  // A wave reads its 64-key tile by itself, so nothing in this loop waits for another wave.  Keys
  // go straight from memory into MFMA operands (lane (r16, g) holds dims ks*32 + g*8.. of key rows
  // kt*16 + r16: the layout the score product wants); values pass through an LDS area of the wave's
  // own, [key][dim] as they are; the reads for the second product transpose them.
  constexpr int VCH = HD / 8;
  bf16x8 k_op[4][KS], v_stage[VCH];
  // rows of the cache fit 32 bits (checked on the host); only the last product is 64 bits wide
  auto row_offset = [&](int j, int blk) {
    const int row = (blk * nkv + kvh) * block_size + (j - page_index(j) * block_size);
    return (int64_t)row * HD;
  };
  // Fused mode: the new token's key is rotated by the lanes that will hold its chunks as operands
  // (in the wave whose tile it falls into) and written to the cache; its value is read from the
  // qkv row where the loop would read the cache.  Both happen below, once the first key tile has
  // been requested.
  const bf16_t* new_v = do_rope ? q + (int64_t)tok0 * q_stride + fused.v_off + (int64_t)kvh * HD : nullptr;
  bf16x8 new_k[KS];
  // Loads are unconditional and nothing is done to what they bring before it is used: a predicated
  // load would become a branch, and a select on a loaded register makes the wave wait for the load
  // where the select stands, so that the next tile's rows would not be on their way while this
  // tile is worked on.  A key row outside the tile's key range reads row 0 of page 0: whatever it
  // holds reaches that key's scores only, which the mask replaces.  A value row outside the range
  // must be finite (its probabilities are exact zeros, and 0 * NaN is NaN; stale pages may hold
  // anything), so it reads finite data that is at hand: HD elements of the query row.  The key
  // dims beyond HD of the last k step (head sizes that are no multiple of 32) repeat dims of the
  // row and meet zeros in the query operand.
  // Values are requested as whole rows (chunk f = c * 64 + lane of the tile's 64 rows x VCH chunks,
  // so that a load instruction covers 1 KB of consecutive rows): with a row per lane an instruction
  // touched 64 cache lines for 16 bytes each, and looking those up was what a round of tiles cost.
  const bf16_t* finite_row = q + (int64_t)tok0 * q_stride + (int64_t)kvh * G * HD;
  auto tile_base = [&](int it) { return ((it0 + it) * stride + mine) * FA_KT; };
  auto fetch = [&](int it, int pages_raw) {
    const int base = tile_base(it);
    const int pages = max(pages_raw, 0);
    const bf16_t* kp[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      const int row = kt * 16 + r16, j = base + row;
      const bool k_in = j >= kv_begin && j < kv_end;
      const int64_t off = row_offset(j, __shfl(pages, row, TL_WAVE));
      kp[kt] = k_cache + (k_in ? off : 0);
    }
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) k_op[kt][ks] = *(const bf16x8*)(kp[kt] + min(ks * 32 + g * 8, HD - 8));
#pragma unroll
    for (int c = 0; c < VCH; ++c) {
      const int f = c * TL_WAVE + lane, row = f / VCH, ch = f % VCH, j = base + row;
      const bool v_in = j >= kv_begin && j < kv_end;
      const int64_t off = row_offset(j, __shfl(pages, row, TL_WAVE));
      const bf16_t* vp = v_in ? v_cache + off : finite_row;
      if (do_rope && j == new_pos) vp = new_v;      // not in the cache yet
      v_stage[c] = *(const bf16x8*)(vp + ch * 8);
    }
  };
  // The next tile is requested as soon as the registers of this one are free, and its pages are
  // looked up an iteration before that, so that the request does not begin with a round trip.
  // (Two tiles in flight per wave, in two register sets, were measured to gain nothing: what a
  // compute unit can have on its way from memory is the limit, about 40 GB/s.)
  if (iters > 0) {
    if (it0 != 0) next_pages = pages_at(tile_base(0));
    fetch(0, next_pages);
    if (iters > 1) next_pages = pages_at(tile_base(1));
  }
  // the rest of the second round, behind the key tile: this lane's angles (the chunk of dims d and
  // d + HD/2 shares the pairs j0 .. j0 + 7) and, where this wave owns the new token's tile, its page
  float c8[KS][8], s8[KS][8];
  int new_page = 0;
  if (do_rope) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int dc = min(ks * 32 + g * 8, HD - 8), j0 = dc < HD / 2 ? dc : dc - HD / 2;
      const f32x4 ca = *(const f32x4*)(cs + j0), cb = *(const f32x4*)(cs + j0 + 4);
      const f32x4 sa = *(const f32x4*)(sn + j0), sb = *(const f32x4*)(sn + j0 + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        c8[ks][e] = ca[e];
        c8[ks][4 + e] = cb[e];
        s8[ks][e] = sa[e];
        s8[ks][4 + e] = sb[e];
      }
    }
    if (owns_new) {
      new_page = bt[new_pos / block_size];
      if (r16 == new_pos % 16) {      // the lanes that will hold the new key's chunks as operands
        const bf16_t* krow = q + (int64_t)tok0 * q_stride + fused.k_off + (int64_t)kvh * HD;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          const int dc = min(ks * 32 + g * 8, HD - 8), dp = (dc + HD / 2) % HD;
          kx[ks] = *(const bf16x8*)(krow + dc);
          ky[ks] = *(const bf16x8*)(krow + dp);
        }
      }
    }
  }
  const int64_t new_off = owns_new ? row_offset(new_pos, new_page) : 0;      // the same for every lane
  // query fragments (B operand): row r16, dims ks*32 + g*8 .. +8, rotated in fused mode; and the
  // new token's key
  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d = ks * 32 + g * 8;
    bf16x8 z = {};
    qf[ks] = do_rope ? rotate_chunk_regs<HD>(qx[ks], qy[ks], d, c8[ks], s8[ks]) : qx[ks];
    if (!(row_valid && d < HD)) qf[ks] = z;
    // (the slots beyond HD of the last k step meet zeros of the query operand: they must hold
    // something finite, since 0 * NaN is NaN and a register nobody wrote may hold anything)
    new_k[ks] = z;
    if (owns_new && r16 == new_pos % 16 && d < HD) {
      new_k[ks] = rotate_chunk_regs<HD>(kx[ks], ky[ks], d, c8[ks], s8[ks]);
      *(bf16x8*)(fused.k_cache_w + new_off + d) = new_k[ks];
    }
  }

  for (int it = 0; it < iters; ++it) {
    const int kt_idx = (it0 + it) * stride + mine;
    if (do_rope && kt_idx == new_tile) {
      // the new token's own key (rotated above) takes the place of what its cache row held, and its
      // value, fetched from the qkv row instead of the cache, is written to the cache
      if (r16 == new_pos % 16) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int ks = 0; ks < KS; ++ks)
            if (kt == (new_pos % FA_KT) / 16) k_op[kt][ks] = new_k[ks];
      }
#pragma unroll
      for (int c = 0; c < VCH; ++c) {
        const int f = c * TL_WAVE + lane;
        if (f / VCH == new_pos % FA_KT) *(bf16x8*)(fused.v_cache_w + new_off + (f % VCH) * 8) = v_stage[c];
      }
    }
    // values: registers -> this wave's LDS area, [key][dim] as they are (the reads transpose)
#pragma unroll
    for (int c = 0; c < VCH; ++c) {
      const int f = c * TL_WAVE + lane;
      *(bf16x8*)(Vl + (f / VCH) * VS + (f % VCH) * 8) = v_stage[c];
    }
    // scores, transposed: sc[kt][r] = S^T[key kt*16 + g*4 + r][row r16]
    f32x4 sc[4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      sc[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        sc[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_op[kt][ks], qf[ks], sc[kt], 0, 0, 0);
    }
    if (it + 1 < iters) {
      fetch(it + 1, next_pages);
      if (it + 2 < iters) next_pages = pages_at(tile_base(it + 2));
    }
    // the LDS operations of one wave are carried out in order; the fences keep the compiler from
    // moving the reads of other lanes' rows above the writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    {
      float m_tile = kNegBig;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int j = kt_idx * FA_KT + kt * 16 + g * 4 + r;
          const bool ok = row_valid && j <= pos && j >= row_lo;
          const float sv = ok ? sc[kt][r] : -INFINITY;
          sc[kt][r] = sv;
          m_tile = fmaxf(m_tile, sv);
        }
      m_tile = max_over_rows(m_tile);
      const float m_new = fmaxf(m_run, m_tile * c_log2);   // the scale is positive: the maximum commutes
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float p = __builtin_amdgcn_exp2f(fmaf(sc[kt][r], c_log2, -m_new));
          sc[kt][r] = p;
          psum += p;
        }
      psum = sum_over_rows(psum);
      l_run = l_run * alpha + psum;
      m_run = m_new;
#pragma unroll
      for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[dt][r] *= alpha;
      // O^T += V^T P^T; the k slots of a step are keys (2s)*16 + g*4 + 0..3 and (2s+1)*16 + g*4 + 0..3
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        // probabilities as two bfloat16 terms, p = hi + lo: the product then carries 16 bits of p
        u32x4 hi, lo;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          uint32_t h0, l0, h1, l1;
          split_pair(sc[2 * st][2 * r], sc[2 * st][2 * r + 1], h0, l0);
          split_pair(sc[2 * st + 1][2 * r], sc[2 * st + 1][2 * r + 1], h1, l1);
          hi[r] = h0;
          lo[r] = l0;
          hi[2 + r] = h1;
          lo[2 + r] = l1;
        }
        const bf16x8 pb = __builtin_bit_cast(bf16x8, hi), pl = __builtin_bit_cast(bf16x8, lo);
        // lane s of a group names keys g*4 + s/4 of a 16-key block, dims dt*16 + 4*(s%4) ..
        const bf16_t* vsrc = Vl + ((2 * st) * 16 + g * 4 + r16 / 4) * VS + 4 * (r16 % 4);
        bf16x8 vf[HDT];
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) {
          const bf16x4 lo4 = lds_read_transposed(vsrc + dt * 16);
          const bf16x4 hi4 = lds_read_transposed(vsrc + 16 * VS + dt * 16);
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            vf[dt][r] = lo4[r];
            vf[dt][4 + r] = hi4[r];
          }
        }
        // the two products into one accumulator are kept HDT MFMAs apart
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pb, o[dt], 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[dt], pl, o[dt], 0, 0, 0);
      }
    }
    // this wave's reads of its area are done before the next tile is written over it
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  __syncthreads();      // the merge below writes over the staging areas

  // merge the waves: each leaves (m, l, O[16][HD]) as floats in its own LDS area
  constexpr int MROW = HD + 2;
  float* Mw = (float*)(smem + wave * WAVE_ELEMS);
#pragma unroll
  for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) Mw[r16 * MROW + dt * 16 + g * 4 + r] = o[dt][r];
  if (g == 0) {
    Mw[r16 * MROW + HD] = m_run;
    Mw[r16 * MROW + HD + 1] = l_run;
  }
  __syncthreads();
  for (int e = tid; e < 16 * HD; e += WAVES * TL_WAVE) {      // one output element a thread
    const int row = e / HD, d = e % HD;
    const int t_local = row / G, h_local = row % G;
    if (t_local >= ntok) continue;
    const int t = tok0 + t_local, h = kvh * G + h_local;
    float mw[WAVES], M = kNegBig;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) {
      mw[wv] = ((const float*)(smem + wv * WAVE_ELEMS))[row * MROW + HD];
      M = fmaxf(M, mw[wv]);
    }
    float L = 0.f, acc = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv) {
      const float* area = (const float*)(smem + wv * WAVE_ELEMS) + row * MROW;
      const float wgt = __builtin_amdgcn_exp2f(mw[wv] - M);      // a wave without keys has l = 0 and O = 0
      L += wgt * area[HD + 1];
      acc += wgt * area[d];
    }
    if (n_splits == 1) {
      out[(int64_t)t * out_stride + (int64_t)h * HD + d] = (bf16_t)(L > 0.f ? acc / L : 0.f);
    } else {
      part_o[(((int64_t)split * n_tokens + t) * nq + h) * HD + d] = acc;
      if (d == 0) {
        float* ml = part_ml + (((int64_t)split * n_tokens + t) * nq + h) * 2;
        ml[0] = M;       // in units of log2 e
        ml[1] = L;
      }
    }
  }
}

// ====================================================== float32 on the matrix cores
// attention_f32_kernel: true float32 (v_mfma_f32_16x16x4_f32 for both products, float32 softmax)
// for every step, prompt portions and decoded tokens alike.  The result of a query row does not
// depend, to the bit, on what else is in the batch, on how the tokens were cut into steps or on
// how the keys are spread over workgroups, because the terms are always combined in ONE tree:
//   * keys in tiles of 64 at absolute positions 64 t .. 64 t + 63; a tile gives (m, l, O) from scratch:
//     m the largest score, l = sum exp2(s - m), O = sum exp2(s - m) v (scores in units of log2 e);
//   * the tiles of a chunk of 4 (256 keys) are merged in ascending order, starting from "nothing";
//   * the chunks are merged in ascending order, starting from "nothing".
// `merge_f32` is the one merge; a tile or chunk that holds no visible key merges as an exact no-op,
// so skipping it changes nothing.  A workgroup (four waves) owns 16 query rows of one request and
// kv head (tokens times the heads of the group, as in the bfloat16 kernels) and either walks all
// chunks itself (gridDim.z == 1) or owns chunk blockIdx.z and leaves its (m, l, O) in `part` for
// attention_f32_combine_kernel.  Its waves take the tiles of a chunk in turn; a wave reads keys
// straight into the first product's operands and stages values through an LDS area of its own.
constexpr int A32_WAVES = 4, A32_THREADS = A32_WAVES * TL_WAVE, A32_CHUNK = 4;
constexpr int A32_VW = 64, A32_VS = A32_VW + 4;      // value columns staged at a time, row stride in LDS

__device__ __forceinline__ void merge_f32(float& M, float& L, float m, float l, float& wa, float& wb) {
  const float Mn = fmaxf(M, m);
  wa = __builtin_amdgcn_exp2f(M - Mn);
  wb = __builtin_amdgcn_exp2f(m - Mn);
  const float lb = l * wb;
  L = __builtin_fmaf(L, wa, lb);
  M = Mn;
}
__device__ __forceinline__ float merge_f32_value(float O, float o, float wa, float wb) {
  const float ob = o * wb;
  return __builtin_fmaf(O, wa, ob);
}

// One tile of 64 keys at kb for the 16 query rows of a wave: (m, l, O) from scratch.  `finite_row`: any
// HD finite floats (read in place of value rows outside the request's keys); Vl: the wave's own LDS area.
template <int HDT>
__device__ __forceinline__ void attention_f32_tile(int kb, const int32_t* __restrict__ bt, int max_blocks, int block_size,
                                                   int nkv, int kvh, const float* __restrict__ k_cache,
                                                   const float* __restrict__ v_cache, const float* __restrict__ finite_row,
                                                   const f32x4 (&qf)[HDT], float c_log2, bool row_valid, int pos, int row_lo,
                                                   int kv_begin, int kv_end, float* Vl, float& m_t, float& l_t,
                                                   f32x4 (&o)[HDT]) {
  constexpr int HD = HDT * 16;
  const int lane = threadIdx.x % TL_WAVE, l16 = lane % 16, kk = lane / 16;
  // Everything the tile needs from memory is requested together, in two rounds (page numbers,
  // then rows): loads are unconditional, with the index clamped into the table; a conditional
  // load would become a branch, and every branch one more round trip in a row.  A key row
  // outside the request's keys is read from row 0 of page 0 (its scores are masked below,
  // whatever they are); a value row outside from the query rows of this tile's first token
  // (finite numbers: its probabilities are exact zeros, and stale pages may hold NaN, for which
  // 0 * NaN is NaN).  Nothing is selected into loaded registers, which would make the wave wait
  // for the rows where the select stands.
  constexpr int VPRE = (HD < A32_VW ? HD : A32_VW) / 4;
  const int vkey = kb + lane;
  const bool v_in_range = vkey >= kv_begin && vkey < kv_end;
  bool k_in[4];
  int page_k[4];
#pragma unroll
  for (int st = 0; st < 4; ++st) {
    const int key = kb + st * 16 + l16;
    k_in[st] = key < kv_end;
    page_k[st] = bt[min(key / block_size, max_blocks - 1)];
  }
  const int page_v = bt[min(vkey / block_size, max_blocks - 1)];
  auto row_of = [&](int page, int key, bool in) {
    const int64_t off = (((int64_t)max(page, 0) * nkv + kvh) * block_size + (key - (key / block_size) * block_size)) * HD;
    return in ? off : (int64_t)0;
  };
  const float* vrow = v_in_range ? v_cache + row_of(page_v, vkey, true) : finite_row;
  f32x4 vpre[VPRE];
#pragma unroll
  for (int ch = 0; ch < VPRE; ++ch) vpre[ch] = *(const f32x4*)(vrow + ch * 4);
  // ---- scores S^T = K Q^T: lane (l16, kk) of subtile st holds keys kb + 16 st + 4 kk + r of row l16
  f32x4 sc[4];
  constexpr int STB = HDT <= 4 ? 4 : 2;       // subtiles whose key rows are in registers together
#pragma unroll
  for (int s0 = 0; s0 < 4; s0 += STB) {
    f32x4 kf[STB][HDT];
#pragma unroll
    for (int si = 0; si < STB; ++si) {
      const float* krow = k_cache + row_of(page_k[s0 + si], kb + (s0 + si) * 16 + l16, k_in[s0 + si]);
#pragma unroll
      for (int g4 = 0; g4 < HDT; ++g4) kf[si][g4] = *(const f32x4*)(krow + g4 * 16 + kk * 4);
    }
#pragma unroll
    for (int si = 0; si < STB; ++si) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int g4 = 0; g4 < HDT; ++g4) {
        const f32x4 kv = kf[si][g4];
#pragma unroll
        for (int e = 0; e < 4; ++e) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kv[e], qf[g4][e], acc, 0, 0, 0);
      }
      sc[s0 + si] = acc;
    }
  }
  // ---- the tile's softmax from scratch
  m_t = -INFINITY;
#pragma unroll
  for (int st = 0; st < 4; ++st)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = kb + st * 16 + kk * 4 + r;
      const bool vis = row_valid && key <= pos && key >= row_lo;
      sc[st][r] = vis ? sc[st][r] * c_log2 : -INFINITY;
      m_t = fmaxf(m_t, sc[st][r]);
    }
  m_t = fmaxf(max_over_rows(m_t), kNegBig);
  l_t = 0.f;
#pragma unroll
  for (int st = 0; st < 4; ++st)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      sc[st][r] = __builtin_amdgcn_exp2f(sc[st][r] - m_t);
      l_t += sc[st][r];
    }
  l_t = sum_over_rows(l_t);
  // ---- O^T = V^T P^T, the values staged 64 columns at a time (lane = key row)
#pragma unroll
  for (int dt = 0; dt < HDT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  {
#pragma unroll
    for (int dh = 0; dh < (HD + A32_VW - 1) / A32_VW; ++dh) {
      constexpr int full = A32_VW / 4;
      const int chunks = min(full, (HD - dh * A32_VW) / 4);
      if (dh > 0) {       // this wave's reads of the columns staged before are done
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      }
#pragma unroll
      for (int ch = 0; ch < full; ++ch)
        if (ch < chunks) {
          f32x4 v;
          if (dh == 0) v = vpre[ch < VPRE ? ch : 0];
          else v = *(const f32x4*)(vrow + dh * A32_VW + ch * 4);
          *(f32x4*)(&Vl[lane * A32_VS + ch * 4]) = v;
        }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int dl = 0; dl < A32_VW / 16; ++dl) {
        const int dt = dh * (A32_VW / 16) + dl;
        if (dt < HDT) {
#pragma unroll
          for (int st = 0; st < 4; ++st)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const float vf = Vl[(st * 16 + kk * 4 + r) * A32_VS + dl * 16 + l16];
              o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf, sc[st][r], o[dt], 0, 0, 0);
            }
        }
      }
    }
    // the area is free for the wave's next tile
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

template <int HDT>
__global__ __launch_bounds__(A32_THREADS) void attention_f32_kernel(
    const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_req, const int32_t* __restrict__ tile_tok0,
    const int32_t* __restrict__ tile_ntok, const int32_t* __restrict__ positions, float* __restrict__ out,
    int64_t out_stride, float* __restrict__ part, int nq, int nkv, int block_size, float scale, int window,
    int n_tokens) {
  constexpr int HD = HDT * 16;
  constexpr int PS = HD + 4;                       // row stride of a tile's O in LDS
  constexpr int EPT = 16 * HD / A32_THREADS;       // output elements a thread merges (= HDT)
  extern __shared__ __attribute__((aligned(16))) float smem32[];
  float* Vl_all = smem32;                                          // [waves][64][A32_VS]
  float* Po = smem32 + A32_WAVES * FA_KT * A32_VS;                 // [tiles of a chunk][16 rows][PS]
  float* Pml = Po + A32_CHUNK * 16 * PS;                           // [tiles of a chunk][16 rows][2]

  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int l16 = lane % 16, kk = lane / 16;
  const int tile = blockIdx.x, kvh = blockIdx.y;
  const int G = nq / nkv, TW = 16 / G;
  const int req = tile_req ? tile_req[tile] : tile, tok0 = tile_req ? tile_tok0[tile] : tile;
  const int ntok = tile_req ? tile_ntok[tile] : 1;
  if (ntok <= 0) return;                           // a padding tile (whole workgroup)
  const int32_t* bt = block_tables + (int64_t)req * max_blocks;
  float* Vl = Vl_all + wave * FA_KT * A32_VS;

  // this lane's query row (the second operand's column l16)
  const int tok_local = l16 / G, hh = l16 % G;
  const bool row_valid = tok_local < TW && tok_local < ntok;
  const int tok = tok0 + (row_valid ? tok_local : 0);
  const int pos = row_valid ? positions[tok] : -1;
  const int row_lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int hi = row_max_i32(pos), lo = row_min_i32(row_valid ? row_lo : 0x7fffffff);
  const int kv_end = hi + 1, kv_begin = lo;
  const int first_tile = kv_begin / FA_KT, last_tile = (kv_end + FA_KT - 1) / FA_KT;
  const int c_first = gridDim.z > 1 ? (int)blockIdx.z : first_tile / A32_CHUNK;
  const int c_last = gridDim.z > 1 ? (int)blockIdx.z + 1 : (last_tile + A32_CHUNK - 1) / A32_CHUNK;

  f32x4 qf[HDT];
  {
    const float* qrow = q + (int64_t)tok * q_stride + (int64_t)(kvh * G + hh) * HD;
#pragma unroll
    for (int g4 = 0; g4 < HDT; ++g4)
      qf[g4] = row_valid ? *(const f32x4*)(qrow + g4 * 16 + kk * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float c_log2 = scale * 1.44269504088896341f;

  // the elements this thread merges: e = tid + 256 u -> (row e / HD, dim e % HD)
  float Mrun[EPT], Lrun[EPT], Orun[EPT];
#pragma unroll
  for (int u = 0; u < EPT; ++u) {
    Mrun[u] = kNegBig;
    Lrun[u] = 0.f;
    Orun[u] = 0.f;
  }

  for (int c = c_first; c < c_last; ++c) {
    const int t_lo = max(c * A32_CHUNK, first_tile), t_hi = min((c + 1) * A32_CHUNK, last_tile);
    for (int t = t_lo + wave; t < t_hi; t += A32_WAVES) {
      float m_t, l_t;
      f32x4 o[HDT];
      attention_f32_tile<HDT>(t * FA_KT, bt, max_blocks, block_size, nkv, kvh, k_cache, v_cache,
                              q + (int64_t)tok0 * q_stride + (int64_t)kvh * G * HD, qf, c_log2, row_valid, pos, row_lo,
                              kv_begin, kv_end, Vl, m_t, l_t, o);
      // ---- the tile's (m, l, O) to its slot: lane (l16, kk) holds row l16, dims 16 dt + 4 kk + r
      const int slot = t - c * A32_CHUNK;
#pragma unroll
      for (int dt = 0; dt < HDT; ++dt) *(f32x4*)(&Po[(slot * 16 + l16) * PS + dt * 16 + kk * 4]) = o[dt];
      if (kk == 0) {
        Pml[(slot * 16 + l16) * 2] = m_t;
        Pml[(slot * 16 + l16) * 2 + 1] = l_t;
      }
    }
    __syncthreads();
    // ---- merge the chunk's tiles in ascending order, then the chunk into the running result
#pragma unroll
    for (int u = 0; u < EPT; ++u) {
      const int e = tid + A32_THREADS * u, row = e / HD, d = e % HD;
      float Mc = kNegBig, Lc = 0.f, Oc = 0.f, wa, wb;
      for (int t = t_lo; t < t_hi; ++t) {
        const int slot = t - c * A32_CHUNK;
        merge_f32(Mc, Lc, Pml[(slot * 16 + row) * 2], Pml[(slot * 16 + row) * 2 + 1], wa, wb);
        Oc = merge_f32_value(Oc, Po[(slot * 16 + row) * PS + d], wa, wb);
      }
      merge_f32(Mrun[u], Lrun[u], Mc, Lc, wa, wb);
      Orun[u] = merge_f32_value(Orun[u], Oc, wa, wb);
    }
    __syncthreads();      // the slots are written again in the next chunk
  }

#pragma unroll
  for (int u = 0; u < EPT; ++u) {
    const int e = tid + A32_THREADS * u, row = e / HD, d = e % HD;
    const int t_local = row / G, h_local = row % G;
    if (t_local >= TW || t_local >= ntok) continue;
    const int t = tok0 + t_local, h = kvh * G + h_local;
    if (gridDim.z == 1) {
      out[(int64_t)t * out_stride + (int64_t)h * HD + d] = Lrun[u] > 0.f ? Orun[u] / Lrun[u] : 0.f;
    } else {
      float* pr = part + (((int64_t)blockIdx.z * n_tokens + t) * nq + h) * (HD + 2);
      pr[d] = Orun[u];
      if (d == 0) {
        pr[HD] = Mrun[u];
        pr[HD + 1] = Lrun[u];
      }
    }
  }
}

// The same function for steps of many query tiles (prompts): a WAVE owns a query tile of 16 rows and walks
// all its key tiles alone, merging them in registers in the one order (tiles of a chunk ascending from
// "nothing", chunks ascending from "nothing"): the very operations attention_f32_kernel applies per
// element, so the bits are the same.  The four waves of a workgroup own neighbouring query tiles of one kv
// head, walk nearly the same keys at nearly the same time and find each other's key and value rows in the
// compute unit's cache; with one tile a workgroup every 16 rows fetched all their keys from the L2, and a
// whole prompt was bound by that (2,048 tokens, heads of 64: 537 us a layer).
template <int HDT>
__global__ __launch_bounds__(A32_THREADS) void attention_f32_rows_kernel(
    const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_req, const int32_t* __restrict__ tile_tok0,
    const int32_t* __restrict__ tile_ntok, const int32_t* __restrict__ positions, float* __restrict__ out,
    int64_t out_stride, int nq, int nkv, int block_size, float scale, int window, int n_tiles) {
  constexpr int HD = HDT * 16;
  extern __shared__ __attribute__((aligned(16))) float smem32[];
  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int l16 = lane % 16, kk = lane / 16;
  const int tile = blockIdx.x * A32_WAVES + wave, kvh = blockIdx.y;
  if (tile >= n_tiles) return;                     // whole waves; the kernel has no workgroup barrier
  const int G = nq / nkv, TW = 16 / G;
  const int req = tile_req ? tile_req[tile] : tile, tok0 = tile_req ? tile_tok0[tile] : tile;
  const int ntok = tile_req ? tile_ntok[tile] : 1;
  if (ntok <= 0) return;                           // a padding tile
  const int32_t* bt = block_tables + (int64_t)req * max_blocks;
  float* Vl = smem32 + wave * FA_KT * A32_VS;

  const int tok_local = l16 / G, hh = l16 % G;
  const bool row_valid = tok_local < TW && tok_local < ntok;
  const int tok = tok0 + (row_valid ? tok_local : 0);
  const int pos = row_valid ? positions[tok] : -1;
  const int row_lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int hi = row_max_i32(pos), lo = row_min_i32(row_valid ? row_lo : 0x7fffffff);
  const int kv_end = hi + 1, kv_begin = lo;
  const int first_tile = kv_begin / FA_KT, last_tile = (kv_end + FA_KT - 1) / FA_KT;
  const int c_first = first_tile / A32_CHUNK, c_last = (last_tile + A32_CHUNK - 1) / A32_CHUNK;

  f32x4 qf[HDT];
  {
    const float* qrow = q + (int64_t)tok * q_stride + (int64_t)(kvh * G + hh) * HD;
#pragma unroll
    for (int g4 = 0; g4 < HDT; ++g4)
      qf[g4] = row_valid ? *(const f32x4*)(qrow + g4 * 16 + kk * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float c_log2 = scale * 1.44269504088896341f;
  const float* finite_row = q + (int64_t)tok0 * q_stride + (int64_t)kvh * G * HD;

  // lane (l16, kk) holds row l16, dims 16 dt + 4 kk + r of the running result
  float Mrun = kNegBig, Lrun = 0.f;
  f32x4 Orun[HDT];
#pragma unroll
  for (int dt = 0; dt < HDT; ++dt) Orun[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int c = c_first; c < c_last; ++c) {
    const int t_lo = max(c * A32_CHUNK, first_tile), t_hi = min((c + 1) * A32_CHUNK, last_tile);
    float Mc = kNegBig, Lc = 0.f, wa, wb;
    f32x4 Oc[HDT];
#pragma unroll
    for (int dt = 0; dt < HDT; ++dt) Oc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int t = t_lo; t < t_hi; ++t) {
      float m_t, l_t;
      f32x4 o[HDT];
      attention_f32_tile<HDT>(t * FA_KT, bt, max_blocks, block_size, nkv, kvh, k_cache, v_cache, finite_row, qf, c_log2,
                              row_valid, pos, row_lo, kv_begin, kv_end, Vl, m_t, l_t, o);
      merge_f32(Mc, Lc, m_t, l_t, wa, wb);
#pragma unroll
      for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) Oc[dt][r] = merge_f32_value(Oc[dt][r], o[dt][r], wa, wb);
    }
    merge_f32(Mrun, Lrun, Mc, Lc, wa, wb);
#pragma unroll
    for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
      for (int r = 0; r < 4; ++r) Orun[dt][r] = merge_f32_value(Orun[dt][r], Oc[dt][r], wa, wb);
  }
  if (!row_valid) return;
  float* orow = out + (int64_t)tok * out_stride + (int64_t)(kvh * G + hh) * HD;
#pragma unroll
  for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
    for (int r = 0; r < 4; ++r) orow[dt * 16 + kk * 4 + r] = Lrun > 0.f ? Orun[dt][r] / Lrun : 0.f;
}

// Merges the chunks that attention_f32_kernel left in `part` [chunks][tokens][heads][hd + 2], in
// ascending order from "nothing": the very sequence of operations of a workgroup that walks the
// chunks itself.  One wave per (token, head).
__global__ __launch_bounds__(TL_WAVE) void attention_f32_combine_kernel(const float* __restrict__ part,
                                                                       float* __restrict__ out, int64_t out_stride,
                                                                       int n_tokens, int nq, int hd, int n_chunks) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  for (int d = lane; d < hd; d += TL_WAVE) {
    float M = kNegBig, L = 0.f, O = 0.f, wa, wb;
    for (int c = 0; c < n_chunks; ++c) {
      const float* pr = part + (((int64_t)c * n_tokens + t) * nq + h) * (hd + 2);
      merge_f32(M, L, pr[hd], pr[hd + 1], wa, wb);
      O = merge_f32_value(O, pr[d], wa, wb);
    }
    out[(int64_t)t * out_stride + (int64_t)h * hd + d] = L > 0.f ? O / L : 0.f;
  }
}

// flash_prefill_bf16_kernel: the same mathematics arranged for prompt portions.  A workgroup
// owns up to 8 query tiles (one per wave, 128 rows: for 8 heads per kv head that is 16 tokens) of
// consecutive tokens of one request, and all eight waves work on the SAME 64-key tile, staged and
// transposed once per workgroup; so a key or value row is fetched once per 128 query rows.  There
// is nothing to merge at the end: every row lives in one lane group of one wave.  Eight waves
// with one query tile each rather than four with two: the workgroup with the most keys sets the
// kernel's duration, and its time per key tile is the work of one wave.
constexpr int FP_RT = 1;                      // query tiles (of 16 rows) per wave
// waves (query tiles) of a workgroup: 8, or 4 where 8 would leave compute units without work

template <int HDT, int WAVES>
__global__ __launch_bounds__(WAVES * TL_WAVE) void flash_prefill_bf16_kernel(
    const bf16_t* __restrict__ q, int64_t q_stride, const bf16_t* __restrict__ k_cache,
    const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_tables, int max_blocks,
    const int32_t* __restrict__ tile_req, const int32_t* __restrict__ tile_tok0,
    const int32_t* __restrict__ tile_ntok, const int32_t* __restrict__ positions, bf16_t* __restrict__ out,
    int64_t out_stride, float* __restrict__ part_o, float* __restrict__ part_ml, int n_tiles, int n_tokens,
    int n_splits, int nq, int nkv, int block_size, int bs_shift, float scale, int window) {
  constexpr int HD = HDT * 16;
  constexpr int KS = (HD + 31) / 32;
  constexpr int KP = KS * 32 + 8;
  // two staging buffers: the next key tile is written while the current one is worked on, so a
  // key tile costs one barrier
  __shared__ __attribute__((aligned(16))) bf16_t Kbuf[2][FA_KT * KP];
  constexpr int VS = HD + FA_VPAD;         // row stride of the row-major V tile
  __shared__ __attribute__((aligned(16))) bf16_t Vbuf[2][FA_KT * VS];

  const int tid = threadIdx.x, lane = tid % TL_WAVE, wave = tid / TL_WAVE;
  const int r16 = lane % 16, g = lane / 16;
  // Later tiles of a prompt have more keys to go through.  The first half of the workgroups takes
  // the items (tile, kv head) from the heaviest down, the second half from the lightest up: all
  // of them are resident at once when they fit, workgroup i beside workgroup i + half on the same
  // compute unit, and so every compute unit gets about the same number of key tiles.
  const int total = n_tiles * nkv, half = total / 2;
  const int L = blockIdx.x % total, split = blockIdx.x / total;      // n_splits workgroups share a tile's keys
  const int item = L < half ? L : total - 1 - (L - half);
  const int tile = n_tiles - 1 - item / nkv, kvh = item % nkv;
  const int G = nq / nkv, TW = 16 / G;
  const int req = tile_req[tile], tok0 = tile_tok0[tile], ntok = tile_ntok[tile];
  if (ntok <= 0) return;      // a padding tile of a step laid out for more tiles than it has (whole workgroup)
  const int32_t* bt = block_tables + (int64_t)req * max_blocks;

  // the tokens of a tile are consecutive tokens of one request, so their positions are consecutive
  const int pos_first = positions[tok0], pos_last = pos_first + ntok - 1;
  const int kv_end = pos_last + 1;
  const int kv_begin = (window > 0 && pos_first + 1 > window) ? pos_first + 1 - window : 0;
  int first_tile = kv_begin / FA_KT, last_tile = (kv_end + FA_KT - 1) / FA_KT;
  if (n_splits > 1) {       // this workgroup's share of the key tiles (possibly none)
    const int per = (last_tile - first_tile + n_splits - 1) / n_splits;
    first_tile = min(first_tile + split * per, last_tile);
    last_tile = min(first_tile + per, last_tile);
  }

  // this lane's query rows, one per query tile of its wave
  bool row_valid[FP_RT];
  int pos[FP_RT], row_lo[FP_RT], tok[FP_RT];
  const int head = kvh * G + r16 % G;
  bf16x8 qf[FP_RT][KS];
#pragma unroll
  for (int rt = 0; rt < FP_RT; ++rt) {
    const int tok_local = (wave * FP_RT + rt) * TW + r16 / G;
    row_valid[rt] = r16 / G < TW && tok_local < ntok;
    tok[rt] = tok0 + (row_valid[rt] ? tok_local : 0);
    pos[rt] = row_valid[rt] ? pos_first + tok_local : -1;
    row_lo[rt] = (window > 0 && pos[rt] + 1 > window) ? pos[rt] + 1 - window : 0;
    const bf16_t* qrow = q + (int64_t)tok[rt] * q_stride + (int64_t)head * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d = ks * 32 + g * 8;
      bf16x8 z = {};
      qf[rt][ks] = (row_valid[rt] && d < HD) ? *(const bf16x8*)(qrow + d) : z;
    }
  }
  // a wave whose rows all end before a key tile begins has nothing to do in it
  int wave_hi = pos[0];
#pragma unroll
  for (int rt = 1; rt < FP_RT; ++rt) wave_hi = max(wave_hi, pos[rt]);
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) wave_hi = max(wave_hi, __shfl_xor(wave_hi, off, TL_WAVE));

  // The running maximum starts at a large negative FINITE number, so exp2(m - m') is never
  // exp2(-inf + inf); a masked score is -inf and its probability exp2(-inf) = 0.
  // The softmax denominator is accumulated by the matrix cores: a row of ones beside V^T adds up
  // the very probabilities (both bfloat16 terms) that enter the output, in an accumulator of its
  // own, which is rescaled with the output.  That saves the adds and two cross-lane exchanges per
  // key tile, and numerator and denominator see the same rounding.
  float m_run[FP_RT];
  f32x4 l_acc[FP_RT];
  f32x4 o[FP_RT][HDT];
#pragma unroll
  for (int rt = 0; rt < FP_RT; ++rt) {
    m_run[rt] = kNegBig;
    l_acc[rt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < HDT; ++dt) o[rt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  const float c_log2 = scale * 1.44269504088896341f;     // scores are kept in units of log2 e
  // smallest position and largest window start among this wave's valid rows: a key tile that lies
  // wholly between them is visible to every row and needs no mask
  int wave_lo_pos = 0x7fffffff, wave_hi_lo = 0;
#pragma unroll
  for (int rt = 0; rt < FP_RT; ++rt)
    if (row_valid[rt]) {
      wave_lo_pos = min(wave_lo_pos, pos[rt]);
      wave_hi_lo = max(wave_hi_lo, row_lo[rt]);
    }
#pragma unroll
  for (int off = 8; off > 0; off >>= 1) {
    wave_lo_pos = min(wave_lo_pos, __shfl_xor(wave_lo_pos, off, TL_WAVE));
    wave_hi_lo = max(wave_hi_lo, __shfl_xor(wave_hi_lo, off, TL_WAVE));
  }
  bool all_valid = true;
#pragma unroll
  for (int rt = 0; rt < FP_RT; ++rt) all_valid = all_valid && row_valid[rt];
  all_valid = __all(all_valid);

  // staging registers: thread = (key row `lane`, chunk group `wave`); the rows of the next tile are
  // requested while the current tile is being worked on
  constexpr int KC = (KS * 4 + WAVES - 1) / WAVES, VC = (HD / 8 + WAVES - 1) / WAVES;
  bf16x8 k_stage[KC], v_stage[VC];
  // The page of this thread's key row is looked up one tile further ahead than the row itself is
  // requested, so that the request does not begin with a dependent round trip to memory.
  // Rows of a tile outside the request's keys [kv_begin, kv_end) are read from the nearest row
  // inside instead (finite data of the same request; every score of such a key is masked, and its
  // probability is an exact zero): so no load is predicated, which would make it a branch.
  auto key_row = [&](int kt_idx) { return min(max(kt_idx * FA_KT + lane, kv_begin), kv_end - 1); };
  auto page_of_row = [&](int kt_idx) {
    const int j = key_row(kt_idx);
    return bt[bs_shift >= 0 ? j >> bs_shift : j / block_size];     // uniform choice: no division
  };
  auto fetch_tile = [&](int kt_idx, int blk) {
    const int j = key_row(kt_idx);
    const int jb = bs_shift >= 0 ? j >> bs_shift : j / block_size;
    // rows of the cache fit 32 bits (checked on the host); only the last product is 64 bits wide
    const int row = (max(blk, 0) * nkv + kvh) * block_size + (j - jb * block_size);
    const bf16_t* kp = k_cache + (int64_t)row * HD;
    const bf16_t* vp = v_cache + (int64_t)row * HD;
#pragma unroll
    for (int ci = 0; ci < KC; ++ci) {
      const int c = ci * WAVES + wave;
      bf16x8 z = {};
      k_stage[ci] = z;
      if (c * 8 < HD) k_stage[ci] = *(const bf16x8*)(kp + c * 8);      // uniform: the dims beyond HD stay zero
    }
#pragma unroll
    for (int ci = 0; ci < VC; ++ci) {
      const int c = ci * WAVES + wave;
      bf16x8 z = {};
      v_stage[ci] = z;
      if (c < HD / 8) v_stage[ci] = *(const bf16x8*)(vp + c * 8);
    }
  };
  // registers -> LDS, both tiles as they are (the reads of V transpose)
  auto store_tile = [&](int buf) {
    bf16_t* Kl = Kbuf[buf];
    bf16_t* Vl = Vbuf[buf];
#pragma unroll
    for (int ci = 0; ci < KC; ++ci) {
      const int c = ci * WAVES + wave;
      if (c < KS * 4) *(bf16x8*)(Kl + lane * KP + c * 8) = k_stage[ci];
    }
#pragma unroll
    for (int ci = 0; ci < VC; ++ci) {
      const int c = ci * WAVES + wave;
      if (c < HD / 8) *(bf16x8*)(Vl + lane * VS + c * 8) = v_stage[ci];
    }
  };
  int next_page = 0;      // of the tile that is requested next
  if (first_tile < last_tile) {
    fetch_tile(first_tile, page_of_row(first_tile));
    if (first_tile + 1 < last_tile) next_page = page_of_row(first_tile + 1);
    store_tile(0);
    if (first_tile + 1 < last_tile) {
      fetch_tile(first_tile + 1, next_page);
      if (first_tile + 2 < last_tile) next_page = page_of_row(first_tile + 2);
    }
  }
  // Every load so far has arrived before the loop begins: the queries above all.  The compiler's
  // placement of waits sees a way into the loop on which they are still in flight (around the
  // block above) and would otherwise wait for ALL loads before the first matrix instruction of
  // every iteration, just after the next tile's rows have been requested.  The first tile's
  // rows are needed here anyway; the second tile's are waited for too, this once.
  __builtin_amdgcn_s_waitcnt(0x0F70);      // vmcnt(0)
  __syncthreads();

  for (int kt_idx = first_tile; kt_idx < last_tile; ++kt_idx) {
    const int cur = (kt_idx - first_tile) & 1;
    // the next tile (requested one iteration ago) goes into the other buffer, which every wave
    // has finished reading before the last barrier; then the tile after it is requested
    if (kt_idx + 1 < last_tile) {
      store_tile(cur ^ 1);
      if (kt_idx + 2 < last_tile) {
        fetch_tile(kt_idx + 2, next_page);
        if (kt_idx + 3 < last_tile) next_page = page_of_row(kt_idx + 3);
      }
    }
    const bf16_t* Kl = Kbuf[cur];
    const bf16_t* Vl = Vbuf[cur];
    // The whole tile in two compilations, with and without the mask: written as one body with a
    // uniform condition around the mask, the compiler turns the condition into selects and every
    // tile pays the mask's 65 vector instructions (of about 200).
    auto work_on_tile = [&](auto with_mask) {
      constexpr bool MASK = decltype(with_mask)::value;
      f32x4 sc[FP_RT][4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int rt = 0; rt < FP_RT; ++rt) sc[rt][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
      // k steps outermost: consecutive MFMAs then write different accumulators and need not wait
      // for each other
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
#pragma unroll
        for (int kt = 0; kt < 4; ++kt) {
          const bf16x8 kf = *(const bf16x8*)(Kl + (kt * 16 + r16) * KP + ks * 32 + g * 8);
#pragma unroll
          for (int rt = 0; rt < FP_RT; ++rt)
            sc[rt][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[rt][ks], sc[rt][kt], 0, 0, 0);
        }
      bf16x8 pb[FP_RT][2], pl[FP_RT][2];
      const int tile_j0 = kt_idx * FA_KT;
#pragma unroll
      for (int rt = 0; rt < FP_RT; ++rt) {
        float m_tile = kNegBig;
        if constexpr (!MASK) {
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) m_tile = fmaxf(m_tile, sc[rt][kt][r]);
        } else {
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int j = tile_j0 + kt * 16 + g * 4 + r;
              const bool ok = row_valid[rt] && j <= pos[rt] && j >= row_lo[rt];
              const float sv = ok ? sc[rt][kt][r] : -INFINITY;
              sc[rt][kt][r] = sv;
              m_tile = fmaxf(m_tile, sv);
            }
        }
        m_tile = max_over_rows(m_tile);
        // the maximum is taken over raw scores (the scale is positive) and scaled once
        const float m_new = fmaxf(m_run[rt], m_tile * c_log2);
        const float alpha = __builtin_amdgcn_exp2f(m_run[rt] - m_new);
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r) sc[rt][kt][r] = __builtin_amdgcn_exp2f(fmaf(sc[rt][kt][r], c_log2, -m_new));
        m_run[rt] = m_new;
        if (__any(alpha != 1.f)) {
#pragma unroll
          for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
            for (int r = 0; r < 4; ++r) o[rt][dt][r] *= alpha;
#pragma unroll
          for (int r = 0; r < 4; ++r) l_acc[rt][r] *= alpha;
        }
#pragma unroll
        for (int st = 0; st < 2; ++st) {
          u32x4 hi_w, lo_w;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            // probabilities 2w and 2w + 1 of this step (two of key block 2 st, then two of 2 st + 1)
            const float pa = sc[rt][2 * st + w / 2][(w % 2) * 2], pc = sc[rt][2 * st + w / 2][(w % 2) * 2 + 1];
            uint32_t hi, lo;
            split_pair(pa, pc, hi, lo);
            hi_w[w] = hi;
            lo_w[w] = lo;
          }
          pb[rt][st] = __builtin_bit_cast(bf16x8, hi_w);
          pl[rt][st] = __builtin_bit_cast(bf16x8, lo_w);
        }
      }
      bf16x8 vfr[2][HDT];
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int dt = 0; dt < HDT; ++dt) {
          // lane s of a group names keys g*4 + s/4 of a 16-key block, dims dt*16 + 4*(s%4) ..
          const bf16_t* vsrc = Vl + ((2 * st) * 16 + g * 4 + r16 / 4) * VS + dt * 16 + 4 * (r16 % 4);
          const bf16x4 lo4 = lds_read_transposed(vsrc);
          const bf16x4 hi4 = lds_read_transposed(vsrc + 16 * VS);
          bf16x8 vf;
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            vf[r] = lo4[r];
            vf[4 + r] = hi4[r];
          }
          vfr[st][dt] = vf;
        }
      // the four products into one accumulator are kept at least four MFMAs apart
      bf16x8 ones;
#pragma unroll
      for (int e = 0; e < 8; ++e) ones[e] = (bf16_t)1.f;
#pragma unroll
      for (int st = 0; st < 2; ++st)
#pragma unroll
        for (int lo = 0; lo < 2; ++lo) {
#pragma unroll
          for (int dt = 0; dt < HDT; ++dt)
#pragma unroll
            for (int rt = 0; rt < FP_RT; ++rt)
              o[rt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfr[st][dt], lo ? pl[rt][st] : pb[rt][st], o[rt][dt],
                                                                  0, 0, 0);
#pragma unroll
          for (int rt = 0; rt < FP_RT; ++rt)
            l_acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, lo ? pl[rt][st] : pb[rt][st], l_acc[rt], 0, 0, 0);
        }
    };
    if (kt_idx * FA_KT <= wave_hi) {
      // a key tile that lies wholly between the wave's smallest position and its largest window
      // start is visible to every row
      const int tile_j0 = kt_idx * FA_KT;
      const bool no_mask = all_valid && tile_j0 + FA_KT - 1 <= wave_lo_pos && tile_j0 >= wave_hi_lo;
      if (no_mask) work_on_tile(std::false_type{});
      else work_on_tile(std::true_type{});
    }
    __syncthreads();
  }
#pragma unroll
  for (int rt = 0; rt < FP_RT; ++rt) {
    if (!row_valid[rt]) continue;
    const float l = l_acc[rt][0];         // every element of the lane's column holds the row's sum
    if (n_splits > 1) {       // unnormalised, for flash_combine_kernel
      const int64_t at = ((int64_t)split * n_tokens + tok[rt]) * nq + head;
#pragma unroll
      for (int dt = 0; dt < HDT; ++dt) *(f32x4*)(part_o + at * HD + dt * 16 + g * 4) = o[rt][dt];
      if (g == 0) {
        part_ml[at * 2] = m_run[rt];
        part_ml[at * 2 + 1] = l;
      }
      continue;
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16_t* orow = out + (int64_t)tok[rt] * out_stride + (int64_t)head * HD + g * 4;
#pragma unroll
    for (int dt = 0; dt < HDT; ++dt) {
      bf16x4 v4;
#pragma unroll
      for (int r = 0; r < 4; ++r) v4[r] = (bf16_t)(o[rt][dt][r] * inv);
      *(bf16x4*)(orow + dt * 16) = v4;
    }
  }
}

// Merges the partial results of `n_splits` workgroups per (token, head).  One wave per (token,
// head); everything is requested before anything is used (up to 16 splits at a time), because a
// dependent round trip to memory costs as much as the rest of this kernel.  FC_BATCH is the
// smallest of 2, 4, 8, 16 that covers n_splits (16 beyond), so that few splits ask for little.
template <int FC_BATCH>
__global__ __launch_bounds__(TL_WAVE) void flash_combine_kernel(const float* __restrict__ part_o,
                                                                const float* __restrict__ part_ml,
                                                                bf16_t* __restrict__ out, int64_t out_stride,
                                                                int n_tokens, int nq, int hd, int n_splits) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int64_t row = (int64_t)t * nq + h, step = (int64_t)n_tokens * nq;      // split s: row + s * step
  // maxima are in units of log2 e; a split without keys has l = 0 and O = 0
  if (n_splits <= FC_BATCH) {      // the usual case: ONE round trip, the maximum comes from the same loads
    float m[FC_BATCH], l[FC_BATCH];
#pragma unroll
    for (int u = 0; u < FC_BATCH; ++u) {
      const int64_t base = row + (int64_t)min(u, n_splits - 1) * step;
      m[u] = part_ml[base * 2];
      l[u] = part_ml[base * 2 + 1];
    }
    for (int d = lane; d < hd; d += TL_WAVE) {
      float o[FC_BATCH];
#pragma unroll
      for (int u = 0; u < FC_BATCH; ++u) o[u] = part_o[(row + (int64_t)min(u, n_splits - 1) * step) * hd + d];
      float M = kNegBig;
#pragma unroll
      for (int u = 0; u < FC_BATCH; ++u) M = fmaxf(M, m[u]);      // a repeated split changes nothing
      float acc = 0.f, L = 0.f;
#pragma unroll
      for (int u = 0; u < FC_BATCH; ++u) {
        if (u < n_splits) {
          const float wgt = __builtin_amdgcn_exp2f(m[u] - M);
          L += wgt * l[u];
          acc += wgt * o[u];
        }
      }
      out[(int64_t)t * out_stride + (int64_t)h * hd + d] = (bf16_t)(L > 0.f ? acc / L : 0.f);
    }
    return;
  }
  // lane s holds the maximum of split s, s + 64, ...
  float M = kNegBig;
  for (int s0 = 0; s0 < n_splits; s0 += TL_WAVE) {
    const int s = s0 + lane;
    M = fmaxf(M, s < n_splits ? part_ml[(row + s * step) * 2] : kNegBig);
  }
  M = wave_max(M);
  for (int d = lane; d < hd; d += TL_WAVE) {
    float acc = 0.f, L = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += FC_BATCH) {
      float m[FC_BATCH], l[FC_BATCH], o[FC_BATCH];
#pragma unroll
      for (int u = 0; u < FC_BATCH; ++u) {
        const int64_t base = row + (int64_t)min(s0 + u, n_splits - 1) * step;
        m[u] = part_ml[base * 2];
        l[u] = part_ml[base * 2 + 1];
        o[u] = part_o[base * hd + d];
      }
#pragma unroll
      for (int u = 0; u < FC_BATCH; ++u) {
        if (s0 + u < n_splits) {
          const float wgt = __builtin_amdgcn_exp2f(m[u] - M);
          L += wgt * l[u];
          acc += wgt * o[u];
        }
      }
    }
    out[(int64_t)t * out_stride + (int64_t)h * hd + d] = (bf16_t)(L > 0.f ? acc / L : 0.f);
  }
}

template <int HDT, int WAVES>
static int launch_flash_w(const bf16_t* q, int64_t q_stride, const bf16_t* k_cache, const bf16_t* v_cache,
                          const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                          const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions, bf16_t* out,
                          int64_t out_stride, float* part_o, float* part_ml, int n_tiles, int n_tokens, int nq,
                          int nkv, int block_size, float scale, int window, int n_splits, const FusedRope& fused,
                          hipStream_t stream) {
  constexpr int HD = HDT * 16;
  constexpr size_t stage = (size_t)WAVES * FA_KT * (HD + FA_VPAD) * sizeof(bf16_t);
  static_assert((size_t)FA_KT * (HD + FA_VPAD) * sizeof(bf16_t) >= 16 * (HD + 2) * sizeof(float),
                "a wave's merge area must fit its staging area");
  static bool configured = false;
  if (!configured) {
    if (hipFuncSetAttribute((const void*)flash_attn_bf16_kernel<HDT, WAVES>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)stage) != hipSuccess)
      return TL_ERR_LAUNCH;
    configured = true;
  }
  hipLaunchKernelGGL((flash_attn_bf16_kernel<HDT, WAVES>), dim3(n_tiles, nkv, n_splits), dim3(WAVES * TL_WAVE), stage,
                     stream, q, q_stride, k_cache, v_cache, block_tables, max_blocks, tile_req, tile_tok0, tile_ntok,
                     positions, out, out_stride, part_o, part_ml, nq, nkv, block_size, scale, window, n_splits,
                     n_tokens, fused);
  return TL_OK;
}

// Waves of a flash_attn_bf16_kernel workgroup, for a launch of `groups` query tiles x kv heads.
// A tile's keys and values are 16 registers per 16 dims of the head: with eight waves (256
// registers a wave) the heads beyond 64 dims spilled 27 to 74 registers to memory and the kernel
// took twice the time that four waves take.  Smaller heads take eight waves where the launch has
// many workgroups anyway, and four (with the keys shared out over twice the workgroups) where it
// has few: measured on whole decode steps, batch 1 and 8 gain 1 %, batch 64 would lose 2 %.
static int flash_waves(int hd, int groups) { return hd <= 64 && groups > 64 ? 8 : 4; }

template <int HDT>
static int launch_flash(const bf16_t* q, int64_t q_stride, const bf16_t* k_cache, const bf16_t* v_cache,
                        const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                        const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions, bf16_t* out,
                        int64_t out_stride, float* part_o, float* part_ml, int n_tiles, int n_tokens, int nq, int nkv,
                        int block_size, float scale, int window, int n_splits, const FusedRope& fused,
                        hipStream_t stream) {
  if constexpr (HDT <= 4) {
    if (flash_waves(HDT * 16, n_tiles * nkv) == 8)
      return launch_flash_w<HDT, 8>(q, q_stride, k_cache, v_cache, block_tables, max_blocks, tile_req, tile_tok0,
                                    tile_ntok, positions, out, out_stride, part_o, part_ml, n_tiles, n_tokens, nq, nkv,
                                    block_size, scale, window, n_splits, fused, stream);
  }
  return launch_flash_w<HDT, 4>(q, q_stride, k_cache, v_cache, block_tables, max_blocks, tile_req, tile_tok0, tile_ntok,
                                positions, out, out_stride, part_o, part_ml, n_tiles, n_tokens, nq, nkv, block_size,
                                scale, window, n_splits, fused, stream);
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

// float32 on the matrix cores, for every kind of step.  Tiles as tl_flash_attention (null: tile i
// is token i of request i).  n_chunks == 1: a workgroup walks all keys of its tile; n_chunks > 1: it
// must be at least ceil(longest context / 256), chunk c goes to workgroup (., ., c) and `part`
// [n_chunks, n_tokens, nq, hd + 2] floats is scratch.  Either way the same bits.
int tl_attention_f32(const float* q, int64_t q_stride, const float* k_cache, const float* v_cache,
                     const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                     const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions, float* out,
                     int64_t out_stride, float* part, int n_tiles, int n_tokens, int nq, int nkv, int hd,
                     int block_size, float scale, int window, int n_chunks, hipStream_t stream) {
  if (n_tiles <= 0 || n_tokens <= 0) return TL_OK;
  if (nq <= 0 || nkv <= 0 || nq % nkv || nq / nkv > 16 || hd <= 0 || hd % 16 || hd > 128 || block_size <= 0 ||
      max_blocks <= 0 || window < 0 || n_chunks < 1 || nkv > 65535 || n_chunks > 65535 || q_stride % 4 ||
      out_stride % 1)
    return TL_ERR_ARG;
  if (n_chunks > 1 && !part) return TL_ERR_ARG;
  if (!tile_req && (tile_tok0 || tile_ntok || n_tiles != n_tokens)) return TL_ERR_ARG;
  if (tile_req && (!tile_tok0 || !tile_ntok)) return TL_ERR_ARG;
  const size_t smem = (size_t)(A32_WAVES * FA_KT * A32_VS + A32_CHUNK * 16 * (hd + 4) + A32_CHUNK * 16 * 2) * sizeof(float);
  // Many query tiles (prompts): a wave a tile, four neighbouring tiles a workgroup; few (decode steps, small
  // steps): a workgroup a tile, its waves sharing the key tiles out.  The same bits either way.
  if (n_chunks == 1 && (int64_t)n_tiles * nkv >= 1024) {
    const size_t smem_rows = (size_t)A32_WAVES * FA_KT * A32_VS * sizeof(float);
#define TL_A32_ROWS(HDT)                                                                                          \
  case HDT: {                                                                                                     \
    static bool configured = false;                                                                               \
    if (!configured) {                                                                                            \
      if (hipFuncSetAttribute((const void*)attention_f32_rows_kernel<HDT>,                                        \
                              hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem_rows) != hipSuccess)          \
        return TL_ERR_LAUNCH;                                                                                     \
      configured = true;                                                                                          \
    }                                                                                                             \
    hipLaunchKernelGGL(attention_f32_rows_kernel<HDT>, dim3((n_tiles + A32_WAVES - 1) / A32_WAVES, nkv),           \
                       dim3(A32_THREADS), smem_rows, stream, q, q_stride, k_cache, v_cache, block_tables,          \
                       max_blocks, tile_req, tile_tok0, tile_ntok, positions, out, out_stride, nq, nkv,            \
                       block_size, scale, window, n_tiles);                                                        \
  } break;
    switch (hd / 16) {
      TL_A32_ROWS(1) TL_A32_ROWS(2) TL_A32_ROWS(3) TL_A32_ROWS(4)
      TL_A32_ROWS(5) TL_A32_ROWS(6) TL_A32_ROWS(7) TL_A32_ROWS(8)
    }
#undef TL_A32_ROWS
    return tl_launch_status();
  }
#define TL_A32_CASE(HDT)                                                                                          \
  case HDT: {                                                                                                     \
    static bool configured = false;                                                                               \
    if (!configured) {                                                                                            \
      if (hipFuncSetAttribute((const void*)attention_f32_kernel<HDT>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)smem) != hipSuccess)                                                           \
        return TL_ERR_LAUNCH;                                                                                     \
      configured = true;                                                                                          \
    }                                                                                                             \
    hipLaunchKernelGGL(attention_f32_kernel<HDT>, dim3(n_tiles, nkv, n_chunks), dim3(A32_THREADS), smem, stream,  \
                       q, q_stride, k_cache, v_cache, block_tables, max_blocks, tile_req, tile_tok0, tile_ntok,   \
                       positions, out, out_stride, part, nq, nkv, block_size, scale, window, n_tokens);           \
  } break;
  switch (hd / 16) {
    TL_A32_CASE(1) TL_A32_CASE(2) TL_A32_CASE(3) TL_A32_CASE(4)
    TL_A32_CASE(5) TL_A32_CASE(6) TL_A32_CASE(7) TL_A32_CASE(8)
  }
#undef TL_A32_CASE
  if (n_chunks > 1)
    hipLaunchKernelGGL(attention_f32_combine_kernel, dim3(n_tokens, nq), dim3(TL_WAVE), 0, stream, part, out,
                       out_stride, n_tokens, nq, hd, n_chunks);
  return tl_launch_status();
}

// bfloat16 only, for steps that hold prompt portions.  Tiles describe groups of at most
// tile_waves * (16 / (nq / nkv)) consecutive tokens of one request; tile_waves is 8, or 4 for steps
// with so few tiles that workgroups of eight waves would leave compute units without work.
int tl_flash_prefill(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                     const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                     const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions, void* out,
                     int64_t out_stride, float* part_o, float* part_ml, int n_tiles, int n_tokens, int nq, int nkv,
                     int hd, int block_size, float scale, int window, int tile_waves, int n_splits,
                     hipStream_t stream) {
  if (n_tiles <= 0) return TL_OK;
  if (tile_waves != 8 && tile_waves != 4) return TL_ERR_ARG;
  // n_splits > 1: the key tiles of a query tile are shared out over that many workgroups, whose
  // results (part_o [n_splits, n_tokens, nq, hd], part_ml [n_splits, n_tokens, nq, 2]) a second kernel merges
  if (n_splits < 1 || n_splits > 64 || n_tokens <= 0 || (n_splits > 1 && (!part_o || !part_ml)) ||
      (int64_t)n_tiles * nkv * n_splits > 0x7fffffff)
    return TL_ERR_ARG;
  if (nq <= 0 || nkv <= 0 || nq % nkv || nq / nkv > 16 || hd <= 0 || hd % 16 || hd > 128 || block_size <= 0 ||
      max_blocks <= 0 || window < 0 || nkv > 65535 || (int64_t)n_tiles * nkv > 0x7fffffff || q_stride % 8 ||
      out_stride % 4)
    return TL_ERR_ARG;
  int bs_shift = -1;      // log2 of the page size where it is a power of two
  for (int sh = 0; sh < 31; ++sh)
    if ((1 << sh) == block_size) bs_shift = sh;
#define TL_PREFILL_LAUNCH(HDT, W)                                                                                 \
  hipLaunchKernelGGL((flash_prefill_bf16_kernel<HDT, W>), dim3(n_tiles * nkv * n_splits), dim3(W * TL_WAVE), 0,   \
                     stream, (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,          \
                     block_tables, max_blocks, tile_req, tile_tok0, tile_ntok, positions, (bf16_t*)out,           \
                     out_stride, part_o, part_ml, n_tiles, n_tokens, n_splits, nq, nkv, block_size, bs_shift,     \
                     scale, window)
#define TL_PREFILL_CASE(HDT)                        \
  case HDT:                                         \
    if (tile_waves == 8) TL_PREFILL_LAUNCH(HDT, 8); \
    else TL_PREFILL_LAUNCH(HDT, 4);                 \
    break;
  switch (hd / 16) {
    TL_PREFILL_CASE(1) TL_PREFILL_CASE(2) TL_PREFILL_CASE(3) TL_PREFILL_CASE(4)
    TL_PREFILL_CASE(5) TL_PREFILL_CASE(6) TL_PREFILL_CASE(7) TL_PREFILL_CASE(8)
  }
#undef TL_PREFILL_CASE
#undef TL_PREFILL_LAUNCH
#define TL_COMBINE(B)                                                                                          \
  hipLaunchKernelGGL(flash_combine_kernel<B>, dim3(n_tokens, nq), dim3(TL_WAVE), 0, stream, part_o, part_ml, \
                     (bf16_t*)out, out_stride, n_tokens, nq, hd, n_splits)
  if (n_splits > 8) TL_COMBINE(16);
  else if (n_splits > 4) TL_COMBINE(8);
  else if (n_splits > 2) TL_COMBINE(4);
  else if (n_splits > 1) TL_COMBINE(2);
#undef TL_COMBINE
  return tl_launch_status();
}

// How many waves of a workgroup of tl_flash_attention share a query tile's keys, a 64-key tile each at
// a time, in a launch of `groups` query tiles x kv heads (the caller sizes n_splits by it).
int tl_flash_waves(int hd, int groups) { return flash_waves(hd, groups); }

// bfloat16 only.  Tiles: tile_req / tile_tok0 / tile_ntok [n_tiles] describe groups of at most
// 16 / (nq / nkv) consecutive tokens of one request; all three null: tile i is token i of request i.  With n_splits > 1, part_o
// [n_splits, n_tokens, nq, hd] and part_ml [n_splits, n_tokens, nq, 2] (float32) are scratch.
static int flash_attention_any(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                               const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                               const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions, void* out,
                               int64_t out_stride, float* part_o, float* part_ml, int n_tiles, int n_tokens, int nq,
                               int nkv, int hd, int block_size, float scale, int window, int n_splits,
                               const float* rope_cos, const float* rope_sin, int fuse_store, hipStream_t stream) {
  if (n_tiles <= 0 || n_tokens <= 0) return TL_OK;
  if (nq <= 0 || nkv <= 0 || nq % nkv || nq / nkv > 16 || hd <= 0 || hd % 16 || hd > 128 || block_size <= 0 ||
      max_blocks <= 0 || window < 0 || n_splits < 1 || nkv > 65535 || n_splits > 65535 || q_stride % 8)
    return TL_ERR_ARG;
  if (n_splits > 1 && (!part_o || !part_ml)) return TL_ERR_ARG;
  if (!tile_req && (tile_tok0 || tile_ntok || n_tiles != n_tokens)) return TL_ERR_ARG;
  if (tile_req && (!tile_tok0 || !tile_ntok)) return TL_ERR_ARG;
  // fused rotation and cache write: q is the first slice of rows [q heads | k heads | v heads], every
  // tile is one token, the whole head is rotated
  if (fuse_store && (!rope_cos || !rope_sin || n_tiles != n_tokens)) return TL_ERR_ARG;
  FusedRope fused{fuse_store ? rope_cos : nullptr, fuse_store ? rope_sin : nullptr, (bf16_t*)k_cache, (bf16_t*)v_cache,
                  nq * hd, (nq + nkv) * hd};
  int rc = TL_ERR_ARG;
#define TL_FLASH_CASE(HDT)                                                                                       \
  case HDT:                                                                                                      \
    rc = launch_flash<HDT>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache,           \
                           block_tables, max_blocks, tile_req, tile_tok0, tile_ntok, positions, (bf16_t*)out,    \
                           out_stride, part_o, part_ml, n_tiles, n_tokens, nq, nkv, block_size, scale, window,   \
                           n_splits, fused, stream);                                                             \
    break;
  switch (hd / 16) {
    TL_FLASH_CASE(1) TL_FLASH_CASE(2) TL_FLASH_CASE(3) TL_FLASH_CASE(4)
    TL_FLASH_CASE(5) TL_FLASH_CASE(6) TL_FLASH_CASE(7) TL_FLASH_CASE(8)
  }
#undef TL_FLASH_CASE
  if (rc != TL_OK) return rc;
#define TL_COMBINE(B)                                                                                          \
  hipLaunchKernelGGL(flash_combine_kernel<B>, dim3(n_tokens, nq), dim3(TL_WAVE), 0, stream, part_o, part_ml, \
                     (bf16_t*)out, out_stride, n_tokens, nq, hd, n_splits)
  if (n_splits > 8) TL_COMBINE(16);
  else if (n_splits > 4) TL_COMBINE(8);
  else if (n_splits > 2) TL_COMBINE(4);
  else if (n_splits > 1) TL_COMBINE(2);
#undef TL_COMBINE
  return tl_launch_status();
}

int tl_flash_attention(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                       const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                       const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions, void* out,
                       int64_t out_stride, float* part_o, float* part_ml, int n_tiles, int n_tokens, int nq,
                       int nkv, int hd, int block_size, float scale, int window, int n_splits,
                       const float* rope_cos, const float* rope_sin, int fuse_store, hipStream_t stream) {
  return flash_attention_any(q, q_stride, k_cache, v_cache, block_tables, max_blocks, tile_req, tile_tok0, tile_ntok,
                             positions, out, out_stride, part_o, part_ml, n_tiles, n_tokens, nq, nkv, hd, block_size,
                             scale, window, n_splits, rope_cos, rope_sin, fuse_store, stream);
}

// ------------------------------------------------ the entry point that allocates nothing
// The partial results of split attention live in a device array that is part of the library
// itself.  Each GPU holds its own copy at its own address, which the host learns once per device
// with hipGetSymbolAddress; kernels receive that address like any other buffer.
static __device__ __align__(256) float scratch[TL_STATIC_SCRATCH_FLOATS];

constexpr int kMaxDevices = 64;
static float* g_scratch_of_device[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

// The address of the current device's copy of `scratch` (looked up at the first call on that device).
static int static_scratch_of_current_device(float** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return TL_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_of_device[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return TL_ERR_LAUNCH;
    g_scratch_of_device[dev] = (float*)p;
  }
  *ptr = g_scratch_of_device[dev];
  return TL_OK;
}

int64_t tl_static_scratch_floats(void) { return (int64_t)TL_STATIC_SCRATCH_FLOATS; }

int tl_flash_attention_static(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                              const int32_t* block_tables, int max_blocks, const int32_t* tile_req,
                              const int32_t* tile_tok0, const int32_t* tile_ntok, const int32_t* positions,
                              void* out, int64_t out_stride, int n_tiles, int n_tokens, int nq, int nkv, int hd,
                              int block_size, float scale, int window, int n_splits, const float* rope_cos,
                              const float* rope_sin, int fuse_store, hipStream_t stream) {
  if (n_tiles <= 0 || n_tokens <= 0) return TL_OK;
  if (n_splits < 1 || nq <= 0 || hd <= 0) return TL_ERR_ARG;
  float* part_o = nullptr;
  float* part_ml = nullptr;
  if (n_splits > 1) {
    const int64_t rows = (int64_t)n_splits * n_tokens * nq;
    if (rows * (hd + 2) > (int64_t)TL_STATIC_SCRATCH_FLOATS) return TL_ERR_SCRATCH;
    float* base = nullptr;
    const int rc = static_scratch_of_current_device(&base);
    if (rc != TL_OK) return rc;
    // Every partial that the merge reads is written by this very call (a workgroup without keys
    // writes a neutral partial), so nothing has to start at zero and what an earlier, larger call
    // left behind is never read.
    part_o = base;
    part_ml = base + rows * hd;
  }
  return flash_attention_any(q, q_stride, k_cache, v_cache, block_tables, max_blocks, tile_req, tile_tok0, tile_ntok,
                             positions, out, out_stride, part_o, part_ml, n_tiles, n_tokens, nq, nkv, hd, block_size,
                             scale, window, n_splits, rope_cos, rope_sin, fuse_store, stream);
}

}  // extern "C"
