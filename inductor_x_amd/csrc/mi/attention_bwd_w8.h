// Fused attention backward (bf16 or fp16, head dimension 128): eight wavefronts per workgroup, two per
// SIMD, three kernels after a small statistics pass, no atomics.
//
// With P = exp(S - m) / l recomputed from the forward's row statistics (S = Q K^T * scale,
// m = row maximum, l = row sum), D = rowsum(dO * O) and dS = P * (dO V^T - D):
//     dV = P^T dO        dK = scale * dS^T Q        dQ = scale * dS K
// The statistics pass folds m and l into one exponent offset per row, m log2(e) + log2(l), so a
// probability costs one fused multiply-add and one exp2.
//
//   dQ kernel   a wavefront owns 32 queries (lane = query), a workgroup 256; loop over 64-key tiles:
//               S^T = K Q^T, dP^T = V dO^T (A from LDS, B = Q / dO fragments in registers),
//               dS^T is at once the B operand of dQ^T += K^T dS^T (A = the K tile read transposed).
//   dK kernel   a wavefront owns 32 keys (lane = key), loop over 64-query tiles:
//               S = Q K^T, dP = dO V^T (A from LDS, B = K / V fragments in registers),
//               dK^T += Q^T dS (A = the Q tile read transposed).
//   dV kernel   same orientation: S = Q K^T, dV^T += dO^T P.
//
// dK and dV are separate kernels (the scores are recomputed three times in all, eight matrix
// products instead of the textbook five): together their accumulators, operands and staging
// registers need more than the 256 registers a wavefront has at two wavefronts per SIMD, and two
// wavefronts per SIMD -- one in its MFMAs while the other recomputes probabilities -- is worth
// more than the product saved.
//
// Every 64-row tile travels memory -> LDS by direct 16-byte `buffer_load ... lds` copies exactly as it
// lies in memory ([64][128], one 1 KiB block = four rows per wavefront instruction, double-buffered, one
// barrier per tile), the 16-byte chunks of a row XOR-swizzled on the way in by the choice of the global
// chunk a lane fetches (bwd8_swz).  The transposed operand of the update product (K^T, Q^T, dO^T) is
// formed by transposing LDS reads (`ds_read_b64_tr_b16`) of the same tile that a score product reads
// along its rows: one copy serves both.  No tile passes through registers.
// Sequence lengths need only be multiples of 64: rows of a last partial block are clamped for
// loads and not stored.
#pragma once

#include "attention.h"

namespace mi {

constexpr int kBwd8Waves = 8;
constexpr int kBwd8Threads = 64 * kBwd8Waves;
constexpr int kBwd8BlockRows = 32 * kBwd8Waves;  // queries (dQ) or keys (dK, dV) per workgroup
constexpr int kBwd8Tile = kAttnBN * kAttnD;           // [64][128] tile as it lies in memory, elements
constexpr int kBwd8StatBytes = kAttnBN * 2 * 4;       // (exponent offset, D) of a query tile
constexpr int kBwd8DqBufBytes = 2 * kBwd8Tile * 2;                    // K, V
constexpr int kBwd8DkBufBytes = 2 * kBwd8Tile * 2 + kBwd8StatBytes;   // Q, dO
constexpr int kBwd8DvBufBytes = 2 * kBwd8Tile * 2 + kBwd8StatBytes;   // Q, dO
constexpr int kBwd8DqLdsBytes = 2 * kBwd8DqBufBytes;
constexpr int kBwd8DkLdsBytes = 2 * kBwd8DkBufBytes;
constexpr int kBwd8DvLdsBytes = 2 * kBwd8DvBufBytes;
constexpr float kBwd8Log2e = 1.4426950408889634f;
// LDS fragments are read this many MFMA steps ahead in the unmasked loops (0: left to the compiler); measured at
// [4,32,4096,128]: two steps ahead is worth 6 % in the causal dK and 8 % in the unmasked dV, more changes nothing
#ifndef BWD8_PREFETCH
#define BWD8_PREFETCH 2
#endif
#ifndef BWD8_PREFETCH_DK
#define BWD8_PREFETCH_DK 2
#endif
#ifndef BWD8_PREFETCH_DK_CAUSAL
#define BWD8_PREFETCH_DK_CAUSAL 2
#endif
#ifndef BWD8_PREFETCH_DV
#define BWD8_PREFETCH_DV 2
#endif
#ifndef BWD8_STAGED_CAUSAL
#define BWD8_STAGED_CAUSAL 1
#endif

// stats[row] = (m log2 e + log2 l, sum_d dO[row, d] * O[row, d]); 16 lanes per row.
template <typename T>
__device__ __forceinline__ void attention_bwd_stats(const T* __restrict__ O, const T* __restrict__ dO,
                                                    const float* __restrict__ softmax_max,
                                                    const float* __restrict__ softmax_sum,
                                                    float* __restrict__ stats, int rows) {
  const int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 4;
  const int part = threadIdx.x & 15;
  float acc = 0.f;
  if (row < rows) {
    typedef typename AttnElem<T>::x8 x8_t;
    const x8_t o = *reinterpret_cast<const x8_t*>(O + static_cast<size_t>(row) * kAttnD + 8 * part);
    const x8_t d = *reinterpret_cast<const x8_t*>(dO + static_cast<size_t>(row) * kAttnD + 8 * part);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = fmaf(static_cast<float>(o[e]), static_cast<float>(d[e]), acc);
  }
#pragma unroll
  for (int off = 8; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (row < rows && part == 0) {
    const float m = softmax_max[static_cast<size_t>(row) * 8];
    const float l = softmax_sum[static_cast<size_t>(row) * 8];
    Vec<float, 2> st;
    st[0] = fmaf(m, kBwd8Log2e, __builtin_amdgcn_logf(l));
    st[1] = acc;
    store_vec<float, 2>(stats + 2 * static_cast<size_t>(row), st);
  }
}

// Staging of a [64][128] tile of 16-bit elements by 512 threads.  Row form: 2 x 16 bytes per thread, stored
// row-major.  Column form: 4 rows x 4 columns per thread (4 x 8 bytes), stored transposed with the
// row index (the contraction axis of the MFMA that reads the tile) permuted, and optionally
// row-major as well.
// Chunk swizzle of a tile row: the 16-byte chunk c of row r lies at position c ^ bwd8_swz(r), a linear map
// of the four low row bits (r0 -> chunk bits 1 and 3, r1 -> bit 2, r2 -> bit 0, r3 -> bit 3).  Sixteen
// consecutive rows get sixteen different positions, which keeps the 16-byte reads along the rows (one row per
// lane) off each other's banks; and the four consecutive rows that one pass of a transposing read touches
// (32 bytes of each) differ in chunk bits 1, 2 and 3 the way the forward's V swizzle makes them differ.
// Measured at [4,32,4096,128]: as fast as two copies under the two separate swizzles, one tile copy less.
__device__ __forceinline__ int bwd8_swz(int row) {
  const int r0 = row & 1, r1 = (row >> 1) & 1, r2 = (row >> 2) & 1, r3 = (row >> 3) & 1;
  return (r0 << 1) | (r1 << 2) | r2 | ((r0 ^ r3) << 3);
}

// One [64][128] tile, memory -> LDS: the eight wavefronts copy two 1 KiB blocks (four rows) each; lane l of
// an instruction fills LDS chunk l of the block (row 4 b + l / 16, chunk position l % 16) with the global
// chunk that the swizzle puts there.
template <typename T>
__device__ __forceinline__ void bwd8_copy_tile(const T* __restrict__ src, T* dst, int wave, int lane) {
  const int blk_row = lane >> 4, blk_pos = lane & 15;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int b = 2 * wave + u;
    const int row = 4 * b + blk_row;
    const int voff = (row * kAttnD + 8 * (blk_pos ^ bwd8_swz(row))) * 2;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(
        __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(src), 0, kBwd8Tile * 2, 0x00020000),
        (__attribute__((address_space(3))) void*)(dst + b * 512), 16, voff, 0, 0, 0);
  }
}
// A operand along the rows of a tile: row `row`, d slice s, half g
template <typename T>
__device__ __forceinline__ typename AttnElem<T>::x8 bwd8_row_frag(const T* tile, int row, int s, int g) {
  return *reinterpret_cast<const typename AttnElem<T>::x8*>(tile + row * kAttnD + 8 * ((2 * s + g) ^ bwd8_swz(row)));
}
// Per-lane element offsets of the transposing reads, one per d block: in every group of 16 lanes, lane s
// points at four consecutive d of row 4 g + s / 4 (+ 8 for the second read) and receives, for its own d,
// the four rows of the group -- the order in which the accumulator layout of the first product delivers
// the rows as a B operand.
template <int DB>
__device__ __forceinline__ void bwd8_tr_offsets(int (&off)[DB], int lane) {
  const int sl16 = lane & 15, grp = lane >> 4;
  const int row_l = 4 * (grp >> 1) + (sl16 >> 2);
  const int c_l = 2 * (grp & 1) + ((sl16 & 3) >> 1);
#pragma unroll
  for (int db = 0; db < DB; ++db)
    off[db] = row_l * kAttnD + 8 * ((4 * db + c_l) ^ bwd8_swz(row_l)) + 4 * (sl16 & 1);
}
// A operand across the rows of a tile (the tile transposed): d block via its offset, row slice t of 16
template <typename T>
__device__ __forceinline__ typename AttnElem<T>::x8 bwd8_tr_frag(const T* tile, int off, int t) {
  typedef AttnElem<T> E;
  const T* p0 = tile + 16 * t * kAttnD + off;
  const typename E::x4 lo = E::read_tr(p0);
  // eight rows further down the chunk sits bwd8_swz(8) positions away (the swizzle is linear in the row bits)
  const typename E::x4 hi = E::read_tr(tile + (16 * t + 8) * kAttnD + (off ^ (8 * bwd8_swz(8))));
  typename E::x8 r;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    r[e] = lo[e];
    r[4 + e] = hi[e];
  }
  return r;
}
// Accumulators (transposed: lane = row of the output, registers = head dimension) of one wavefront's
// 32 rows -> memory.  Stored from the registers a wavefront instruction would write 32 separate
// 16-byte pieces; instead the block goes through the wavefront's own 8 KiB of the (idle) tile
// buffers, 16-byte chunks XOR-swizzled by the row, and leaves as whole 256-byte rows, four per
// instruction.  The caller has passed the barrier that ends the last tile; `rows` of the 32 exist.
// STAGED = false stores from the registers (BWD8_STAGED_CAUSAL = 0 selects it for the causal kernels; measured
// at [4,32,4096,128] the staged form is 2 % faster in dK and dV since the tiles stopped passing through
// registers, and was slower before, when those kernels spilled).
template <bool STAGED, typename T, int DB>
__device__ __forceinline__ void bwd8_store_acc(T* __restrict__ dst_block, const f32x16_t (&acc)[DB], float factor,
                                               T* stage, int lane, int rows) {
  typedef typename AttnElem<T>::x4 x4_t;
  const int li = lane & 31, g = lane >> 5;
  if constexpr (!STAGED) {
  if (li < rows) {
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        x4_t o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) o4[e] = static_cast<T>(acc[db][4 * rq + e] * factor);
        *reinterpret_cast<x4_t*>(dst_block + li * kAttnD + 32 * db + 8 * rq + 4 * g) = o4;
      }
  }
  return;
  }
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      x4_t o4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o4[e] = static_cast<T>(acc[db][4 * rq + e] * factor);
      *reinterpret_cast<x4_t*>(stage + li * kAttnD + 8 * ((4 * db + rq) ^ (li & 15)) + 4 * g) = o4;
    }
  const int c16 = lane & 15;
#pragma nounroll
  for (int j = 0; j < 8; ++j) {  // rolled: the kernels that call this have no registers to spare
    const int row = 4 * j + (lane >> 4);
    const u32x4_t v16 = *reinterpret_cast<const u32x4_t*>(stage + row * kAttnD + 8 * (c16 ^ (row & 15)));
    if (row < rows) *reinterpret_cast<u32x4_t*>(dst_block + row * kAttnD + 8 * c16) = v16;
  }
}
template <int DB>
__device__ __forceinline__ void bwd8_zero(f32x16_t (&acc)[DB]) {
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;
}

// ---------------------------------------------------------------------------------------------
// dQ
// ---------------------------------------------------------------------------------------------
// DH (both kernels below): columns of the 128-wide head that carry data, 128 or 64; with 64 (a smaller
// head zero-padded by the caller) the d slices and d blocks that hold only zeros are skipped and the
// upper 64 columns of the result are left undefined.
// BITS (both kernels below): a bit mask for this head, one 64-bit word per (row, tile of the other axis)
// laid out [S][S / 64], bit j set = the pair is hidden (dQ: row = query, bit = key of the tile; dK / dV:
// row = key, bit = query of the tile, i.e. the words of the transposed mask); hidden pairs get the
// probability zero.  The word of the next tile is fetched with that tile's operands.  tile_lo .. tile_hi (BITS
// only): the tiles of the other axis outside this range hold no visible pair for any row of the block (the
// host derives the range from the mask words) and are left out of the loop.
template <typename T, bool CAUSAL, int DH = 128, bool BITS = false>
__device__ __forceinline__ void attention_bwd8_dq(const T* __restrict__ Q, const T* __restrict__ K,
                                                  const T* __restrict__ V, const T* __restrict__ dO,
                                                  const float* __restrict__ stats, T* __restrict__ dQ,
                                                  int S, int q_block, int head, float scale,
                                                  const unsigned char* __restrict__ head_mask = nullptr,
                                                  int tile_lo = 0, int tile_hi = 0x7fffff) {
  typedef AttnElem<T> E;
  typedef typename E::x8 x8_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const T* __restrict__ Kh = K + head_off;
  const T* __restrict__ Vh = V + head_off;
  const int q0 = q_block * kBwd8BlockRows;
  const int qw = q0 + wave * 32;       // first query of this wavefront
  const int qi = qw + li;
  const bool valid = qi < S;
  const int qc = valid ? qi : S - 1;   // rows past the end read the last row and are never stored
  const size_t qrow = head_off + static_cast<size_t>(qc) * kAttnD;

  static_assert(DH == 128 || DH == 64, "128 or 64 data columns");
  constexpr int DS = DH / 16, DB = DH / 32;   // d slices of a score product, d blocks of the result
  constexpr int N1 = 2 * DS, N2 = 4 * DB;     // MFMA steps of the score phase and of the update phase
  x8_t qf[DS], dof[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    qf[s] = *reinterpret_cast<const x8_t*>(Q + qrow + 16 * s + 8 * g);
    dof[s] = *reinterpret_cast<const x8_t*>(dO + qrow + 16 * s + 8 * g);
  }
  const Vec<float, 2> st = load_vec<float, 2>(stats + 2 * (static_cast<size_t>(head) * S + qc));
  const float m2 = st[0], delta = st[1];
  const float c2 = scale * kBwd8Log2e;

  f32x16_t acc[DB];
  bwd8_zero(acc);

  const int all_tiles = S / kAttnBN;
  const int end_tiles = CAUSAL ? min((q0 + kBwd8BlockRows) / kAttnBN, all_tiles) : all_tiles;
  const int n_tiles = BITS ? min(end_tiles, max(tile_hi, 0) + 1) : end_tiles;  // one past the last tile visited
  const int first = BITS ? min(max(tile_lo, 0), n_tiles - 1) : 0;            // first tile visited
  const int wave_last_tile = (CAUSAL && qw < S) ? (qw + 31) / kAttnBN : (qw < S ? n_tiles - 1 : -1);

  auto buf = [&](int b) { return reinterpret_cast<T*>(attn_lds + b * kBwd8DqBufBytes); };
  int tr_off[DB];
  bwd8_tr_offsets(tr_off, lane);
  u32x2_t mk_next, mk_cur;  // mask words of this lane's query: the tile being loaded, the tile being computed
  // requests tile `tile` into its buffer (free since the barrier that ended the tile before last)
  auto load_tile = [&](int tile) {
    const T* kp = Kh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    T* Ks = buf(tile & 1);  // K for both kinds of read, V behind it
    bwd8_copy_tile(kp, Ks, wave, lane);
    bwd8_copy_tile(Vh + static_cast<size_t>(tile) * kAttnBN * kAttnD, Ks + kBwd8Tile, wave, lane);
    if constexpr (BITS)
      mk_next = *reinterpret_cast<const u32x2_t*>(head_mask + (static_cast<size_t>(qc) * all_tiles + tile) * 8);
  };
  // the requested tile has landed (for this wavefront's copies; the barrier that follows covers the rest)
  auto finish_tile = [&]() {
    if constexpr (BITS) mk_cur = mk_next;
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  };

  auto compute = [&](int tile, auto mask_c) {
    constexpr bool MASK = decltype(mask_c)::value;
    const T* Ks = buf(tile & 1);
    const T* Vs = Ks + kBwd8Tile;
    const T* Kt = Ks;  // the same tile, read transposed
    const int key0 = tile * kAttnBN;
    x8_t dsf[2][2];
#if BWD8_PREFETCH > 0
    if constexpr (!MASK && !BITS) {  // the masked instantiations have no registers for fragments in flight
    // The 32 MFMA steps of a tile (16 score / dP pairs, then 16 dQ updates) read their LDS
    // fragments BWD8_PREFETCH steps ahead, across the boundaries between the phases, with the
    // order pinned by scheduling fences: the softmax arithmetic of a key block then runs while
    // the fragments of the next steps are already in flight.
    constexpr int PF = BWD8_PREFETCH;
    x8_t ka[N1], va[N1], ta[N2];
    auto issue = [&](auto ic) {
      constexpr int i = decltype(ic)::value;
      if constexpr (i < N1) {
        ka[i] = bwd8_row_frag(Ks, 32 * (i / DS) + li, i % DS, g);
        va[i] = bwd8_row_frag(Vs, 32 * (i / DS) + li, i % DS, g);
      } else if constexpr (i < N1 + N2) {
        ta[i - N1] = bwd8_tr_frag(Kt, tr_off[(i - N1) % DB], (i - N1) / DB);
      }
    };
    static_for<PF>([&](auto ic) { issue(ic); });
    f32x16_t sacc, pacc;
    static_for<N1 + N2>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      issue(std::integral_constant<int, i + PF>{});
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (i < N1) {
        constexpr int kb = i / DS, s_ = i % DS;
        if constexpr (s_ == 0) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            sacc[r] = 0.f;
            pacc[r] = 0.f;
          }
        }
        sacc = E::mfma(ka[i], qf[s_], sacc);
        pacc = E::mfma(va[i], dof[s_], pacc);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (s_ == DS - 1) {
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float p = __builtin_amdgcn_exp2f(fmaf(sacc[r], c2, -m2));
            if (MASK && key0 + 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3) > qi) p = 0.f;
            if (BITS && ((mk_cur[kb] >> (8 * (r >> 2) + 4 * g + (r & 3))) & 1u)) p = 0.f;
            dsf[kb][r >> 3][r & 7] = static_cast<T>(p * (pacc[r] - delta));
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
        constexpr int j = i - N1, t = j / DB, db = j % DB;
        acc[db] = E::mfma(ta[j], dsf[t >> 1][t & 1], acc[db]);
        __builtin_amdgcn_sched_barrier(0);
      }
    });
    return;
    }
#endif
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      f32x16_t sacc, pacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sacc[r] = 0.f;
        pacc[r] = 0.f;
      }
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        sacc = E::mfma(bwd8_row_frag(Ks, 32 * kb + li, s, g), qf[s], sacc);
        pacc = E::mfma(bwd8_row_frag(Vs, 32 * kb + li, s, g), dof[s], pacc);
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float p = __builtin_amdgcn_exp2f(fmaf(sacc[r], c2, -m2));
        if (MASK && key0 + 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3) > qi) p = 0.f;
        if (BITS && ((mk_cur[kb] >> (8 * (r >> 2) + 4 * g + (r & 3))) & 1u)) p = 0.f;
        dsf[kb][r >> 3][r & 7] = static_cast<T>(p * (pacc[r] - delta));
      }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int db = 0; db < DB; ++db)
        acc[db] = E::mfma(bwd8_tr_frag(Kt, tr_off[db], t), dsf[t >> 1][t & 1], acc[db]);
  };

  // Under a causal mask only the tiles that overlap the block's own queries (the last four) need
  // the mask or are skipped by some wavefronts; they run in a loop of their own so that the loop
  // over the tiles before them carries no masking code.
  const int first_diag = CAUSAL ? max(min(q0 / kAttnBN, n_tiles), first) : n_tiles;
  load_tile(first);
  finish_tile();
  __syncthreads();
  for (int tile = first; tile < first_diag; ++tile) {
    if (tile + 1 < n_tiles) load_tile(tile + 1);
    if (tile <= wave_last_tile) compute(tile, attn_flag<false>{});
    finish_tile();
    __syncthreads();
  }
  if constexpr (CAUSAL) {
#pragma nounroll
    for (int tile = first_diag; tile < n_tiles; ++tile) {
      if (tile + 1 < n_tiles) load_tile(tile + 1);
      if (tile <= wave_last_tile) compute(tile, attn_flag<true>{});
      finish_tile();
      __syncthreads();
    }
  }
  bwd8_store_acc<!CAUSAL || BWD8_STAGED_CAUSAL>(dQ + head_off + static_cast<size_t>(qw) * kAttnD, acc, scale,
                 reinterpret_cast<T*>(attn_lds) + wave * (32 * kAttnD), lane, S - qw);
  __syncthreads();  // the staging reads are done before a following block refills the tile buffers
}

// ---------------------------------------------------------------------------------------------
// dK (WHICH = 0) and dV (WHICH = 1): a wavefront owns 32 keys, loop over query tiles
// ---------------------------------------------------------------------------------------------
template <typename T, bool CAUSAL, int WHICH, int DH = 128, bool BITS = false>
__device__ __forceinline__ void attention_bwd8_dkv(const T* __restrict__ Q, const T* __restrict__ K,
                                                   const T* __restrict__ V, const T* __restrict__ dO,
                                                   const float* __restrict__ stats, T* __restrict__ dKV,
                                                   int S, int k_block, int head, float scale,
                                                   const unsigned char* __restrict__ head_mask = nullptr,
                                                   int tile_lo = 0, int tile_hi = 0x7fffff) {
  constexpr bool DK = WHICH == 0;
  constexpr int BUF = DK ? kBwd8DkBufBytes : kBwd8DvBufBytes;
  constexpr int STAT_OFF = BUF - kBwd8StatBytes;
  typedef AttnElem<T> E;
  typedef typename E::x8 x8_t;
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const T* __restrict__ Qh = Q + head_off;
  const T* __restrict__ dOh = dO + head_off;
  const int k0 = k_block * kBwd8BlockRows;
  const int kw = k0 + wave * 32;  // first key of this wavefront
  const int kj = kw + li;
  const bool valid = kj < S;
  const int kc = valid ? kj : S - 1;
  const size_t krow = head_off + static_cast<size_t>(kc) * kAttnD;

  static_assert(DH == 128 || DH == 64, "128 or 64 data columns");
  constexpr int DS = DH / 16, DB = DH / 32;
  constexpr int N1 = 2 * DS, N2 = 4 * DB;
  x8_t kf[DS], vf[DK ? DS : 1];
#pragma unroll
  for (int s = 0; s < DS; ++s) {
    kf[s] = *reinterpret_cast<const x8_t*>(K + krow + 16 * s + 8 * g);
    if constexpr (DK) vf[s] = *reinterpret_cast<const x8_t*>(V + krow + 16 * s + 8 * g);
  }
  f32x16_t acc[DB];
  bwd8_zero(acc);
  const float c2 = scale * kBwd8Log2e;

  const int all_qtiles = S / kAttnBN;
  const int n_qtiles = BITS ? min(all_qtiles, max(tile_hi, 0) + 1) : all_qtiles;  // one past the last query tile visited
  // first query tile visited: under a causal mask the first one that sees a key of the block
  const int first_tile = BITS ? min(max(CAUSAL ? k0 / kAttnBN : 0, tile_lo), n_qtiles) : (CAUSAL ? k0 / kAttnBN : 0);
  const int wave_first_tile = kw < S ? (CAUSAL ? kw / kAttnBN : 0) : all_qtiles;

  // DK reads Q both ways and dO along its rows; DV reads Q along its rows and dO transposed
  int tr_off[DB];
  bwd8_tr_offsets(tr_off, lane);
  Vec<float, 2> sst;
  u32x2_t mk_next, mk_cur;  // words of the transposed mask for this lane's key: tile being loaded / computed
  // requests query tile `tile` into its buffer (free since the barrier that ended the tile before last)
  auto load_tile = [&](int tile) {
    const T* qp = Qh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    const T* dp = dOh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    T* base = reinterpret_cast<T*>(attn_lds + (tile & 1) * BUF);
    bwd8_copy_tile(qp, base, wave, lane);               // Q: along its rows, and transposed for dK
    bwd8_copy_tile(dp, base + kBwd8Tile, wave, lane);   // dO: along its rows for dK, transposed for dV
    if constexpr (BITS)
      mk_next = *reinterpret_cast<const u32x2_t*>(head_mask + (static_cast<size_t>(kc) * all_qtiles + tile) * 8);
    if (tid < kAttnBN) sst = load_vec<float, 2>(stats + 2 * (static_cast<size_t>(head) * S + tile * kAttnBN + tid));
  };
  // the requested tile has landed (this wavefront's copies; the barrier that follows covers the rest) and its
  // row statistics go to their place behind the tiles
  auto finish_tile = [&](int b) {
    if constexpr (BITS) mk_cur = mk_next;
    if (tid < kAttnBN) store_vec<float, 2>(reinterpret_cast<float*>(attn_lds + b * BUF + STAT_OFF) + 2 * tid, sst);
    __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  };

  auto compute = [&](int tile, auto mask_c) {
    constexpr bool MASK = decltype(mask_c)::value;
    const T* base = reinterpret_cast<const T*>(attn_lds + (tile & 1) * BUF);
    const T* Qs = base;
    const T* dOs = base + kBwd8Tile;                                 // DK only
    const T* Tt = DK ? base : base + kBwd8Tile;                      // the tile read transposed: Q (DK) or dO (DV)
    const float* st = reinterpret_cast<const float*>(attn_lds + (tile & 1) * BUF + STAT_OFF);
    const int q0t = tile * kAttnBN;
    x8_t bf[2][2];  // [query block][half]: P (dV) or dS (dK) as B operands, contraction over the queries
    auto probabilities = [&](auto qbc, const f32x16_t& sacc, const f32x16_t& pacc) {
      constexpr int qb = decltype(qbc)::value;
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        // rows 32 qb + 8 rq + 4 g + (0..3) of the query tile and their statistics
        const int row0 = 32 * qb + 8 * rq + 4 * g;
        const Vec<float, 4> sa = load_vec<float, 4>(st + 2 * row0);
        const Vec<float, 4> sb = load_vec<float, 4>(st + 2 * row0 + 4);
        const float mrow[4] = {sa[0], sa[2], sb[0], sb[2]};
        const float drow[4] = {sa[1], sa[3], sb[1], sb[3]};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * rq + e;
          float p = __builtin_amdgcn_exp2f(fmaf(sacc[r], c2, -mrow[e]));
          if (MASK && kj > q0t + row0 + e) p = 0.f;
          if (BITS && ((mk_cur[qb] >> (8 * rq + 4 * g + e)) & 1u)) p = 0.f;
          if constexpr (DK)
            bf[qb][r >> 3][r & 7] = static_cast<T>(p * (pacc[r] - drow[e]));
          else
            bf[qb][r >> 3][r & 7] = static_cast<T>(p);
        }
      }
    };
    constexpr int PF = DK ? (CAUSAL ? BWD8_PREFETCH_DK_CAUSAL : BWD8_PREFETCH_DK) : BWD8_PREFETCH_DV;
    if constexpr (PF > 0 && !MASK && !BITS) {
      // as in the dQ kernel: LDS fragments read PF steps ahead across the phases of the tile
      x8_t qa[N1], da[DK ? N1 : 1], ta[N2];
      auto issue = [&](auto ic) {
        constexpr int i = decltype(ic)::value;
        if constexpr (i < N1) {
          qa[i] = bwd8_row_frag(Qs, 32 * (i / DS) + li, i % DS, g);
          if constexpr (DK) da[i] = bwd8_row_frag(dOs, 32 * (i / DS) + li, i % DS, g);
        } else if constexpr (i < N1 + N2) {
          ta[i - N1] = bwd8_tr_frag(Tt, tr_off[(i - N1) % DB], (i - N1) / DB);
        }
      };
      static_for<PF>([&](auto ic) { issue(ic); });
      f32x16_t sacc, pacc;
      static_for<N1 + N2>([&](auto ic) {
        constexpr int i = decltype(ic)::value;
        issue(std::integral_constant<int, i + PF>{});
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (i < N1) {
          constexpr int qb = i / DS, s_ = i % DS;
          if constexpr (s_ == 0) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
              sacc[r] = 0.f;
              pacc[r] = 0.f;
            }
          }
          sacc = E::mfma(qa[i], kf[s_], sacc);
          if constexpr (DK) pacc = E::mfma(da[i], vf[s_], pacc);
          __builtin_amdgcn_sched_barrier(0);
          if constexpr (s_ == DS - 1) {
            probabilities(std::integral_constant<int, qb>{}, sacc, pacc);
            __builtin_amdgcn_sched_barrier(0);
          }
        } else {
          constexpr int j = i - N1, t = j / DB, db = j % DB;
          acc[db] = E::mfma(ta[j], bf[t >> 1][t & 1], acc[db]);
          __builtin_amdgcn_sched_barrier(0);
        }
      });
      return;
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      f32x16_t sacc, pacc;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        sacc[r] = 0.f;
        pacc[r] = 0.f;
      }
#pragma unroll
      for (int s = 0; s < DS; ++s) {
        sacc = E::mfma(bwd8_row_frag(Qs, 32 * qb + li, s, g), kf[s], sacc);
        if constexpr (DK)
          pacc = E::mfma(bwd8_row_frag(dOs, 32 * qb + li, s, g), vf[s], pacc);
      }
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int row0 = 32 * qb + 8 * rq + 4 * g;
        const Vec<float, 4> sa = load_vec<float, 4>(st + 2 * row0);
        const Vec<float, 4> sb = load_vec<float, 4>(st + 2 * row0 + 4);
        const float mrow[4] = {sa[0], sa[2], sb[0], sb[2]};
        const float drow[4] = {sa[1], sa[3], sb[1], sb[3]};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int r = 4 * rq + e;
          float p = __builtin_amdgcn_exp2f(fmaf(sacc[r], c2, -mrow[e]));
          if (MASK && kj > q0t + row0 + e) p = 0.f;
          if (BITS && ((mk_cur[qb] >> (8 * rq + 4 * g + e)) & 1u)) p = 0.f;
          if constexpr (DK)
            bf[qb][r >> 3][r & 7] = static_cast<T>(p * (pacc[r] - drow[e]));
          else
            bf[qb][r >> 3][r & 7] = static_cast<T>(p);
        }
      }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int db = 0; db < DB; ++db)
        acc[db] = E::mfma(bwd8_tr_frag(Tt, tr_off[db], t), bf[t >> 1][t & 1], acc[db]);
  };

  if (first_tile < n_qtiles) {
    load_tile(first_tile);
    finish_tile(first_tile & 1);
  }
  __syncthreads();
  // Under a causal mask the first four query tiles overlap the block's own keys: a loop of their
  // own with the mask (and wavefronts whose keys come later skipping), then the unmasked rest.
  const int after_diag = CAUSAL ? max(min(k0 / kAttnBN + kBwd8BlockRows / kAttnBN, n_qtiles), first_tile) : first_tile;
  if constexpr (CAUSAL) {
#pragma nounroll
    for (int tile = first_tile; tile < after_diag; ++tile) {
      if (tile + 1 < n_qtiles) load_tile(tile + 1);
      if (tile >= wave_first_tile) compute(tile, attn_flag<true>{});
      if (tile + 1 < n_qtiles) finish_tile((tile + 1) & 1);
      __syncthreads();
    }
  }
  for (int tile = after_diag; tile < n_qtiles; ++tile) {
    if (tile + 1 < n_qtiles) load_tile(tile + 1);
    if (kw < S) compute(tile, attn_flag<false>{});
    if (tile + 1 < n_qtiles) finish_tile((tile + 1) & 1);
    __syncthreads();
  }
  bwd8_store_acc<!CAUSAL || BWD8_STAGED_CAUSAL>(dKV + head_off + static_cast<size_t>(kw) * kAttnD, acc, DK ? scale : 1.0f,
                 reinterpret_cast<T*>(attn_lds) + wave * (32 * kAttnD), lane, S - kw);
  __syncthreads();  // the staging reads are done before a following block refills the tile buffers
}

}  // namespace mi
