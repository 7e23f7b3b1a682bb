// Fused attention forward, 32 queries per wavefront, two wavefronts per SIMD, K and V tiles brought
// into LDS by direct global -> LDS loads and V read back transposed.  Operand layouts: attention.h.
//
// Software pipeline per 64-key tile, matrix and vector work of each wavefront interleaved chunk by
// chunk (one LDS fragment read two chunks ahead, one MFMA, a slice of the vector work):
//     A   matrix:  O += V^T(t-1) P(t-1)      vector:  row max of S(t), first half of P(t)
//     B   matrix:  S(t+1) = K(t+1) Q^T       vector:  second half of P(t)
// With 32 queries a wavefront needs 200-240 registers, so a SIMD holds two, and the vector
// instructions of one issue in the shadow of the other's MFMAs.  How a tile travels:
//   - K and V tiles go memory -> LDS with 16-byte `buffer_load ... lds` (gfx950): no staging registers, no
//     LDS store instructions, no byte permutes.  One wavefront instruction fills a 1 KiB block (four
//     256-byte rows); which global 16-byte chunk a lane fetches is free, so the chunks of a row are
//     XOR-swizzled on the way in (K by row mod 16; V by a 4-entry table that keeps the transposing
//     reads of 16- and 32-lane groups on distinct banks).  The loads of iteration t are issued in its
//     first two chunks into the buffers iteration t - 1 released, and must only have landed by the
//     barrier that ends the iteration.
//   - V stays [key][d] in LDS; the V^T operand of O^T += V^T P^T is read with two
//     `ds_read_b64_tr_b16` per fragment: in every group of 16 lanes, lane s points at four consecutive
//     d of key 4 g + s / 4 and receives, for its own d, the four keys of the group -- which is the
//     key order P arrives in from the first product's accumulator layout.
// Element type (bf16 or fp16), causal mask and bounds handling are template arguments.  RAGGED
// instantiations take any sequence lengths: query rows past the end are computed on a copy of the
// last row and not stored, keys past the end read as zeros (the tile copies are bounded buffer
// loads) and are masked in the softmax of the last tile; the others require lengths that are
// multiples of 256 (queries) and 128 (keys) and carry none of that code.
#pragma once

#include "attention.h"


namespace mi {

constexpr int kAttnV5Waves = 8;
constexpr int kAttnV5BM = kAttnV5Waves * 32;

// Timeline hook: the kernel calls mark(point, head, q_block) at seven fixed points of a query block
// (0 entry, 1 queries and first two K tiles landed, 2 first score product and tile step done, 3 unguarded
// tile steps done, 4 all tile steps done, 5 output stores issued, 6 block done).  The default does nothing
// and leaves no code; the measurement build under csrc/probes records a clock there.
struct AttnNoTimeline {
  __device__ __forceinline__ void mark(int, int, int) const {}
};

// WAVES = 8: one workgroup of 256 queries per CU.  WAVES = 4: 128 queries per workgroup and two
// workgroups per CU (64 KiB of LDS each), so the two wavefronts of a SIMD belong to different
// workgroups, share no barrier and drift apart in phase.
// DH: columns of the 128-wide head that carry data, 128 or 64.  With 64 (a smaller head zero-padded
// to 128 by the caller) the d slices and d blocks that hold only zeros are skipped: half the matrix
// instructions and half the LDS fragment reads per tile; the tiles still travel 128 wide and the
// upper 64 output columns are left undefined (the caller drops them).
// MASKED: a bit mask for this head, one 64-bit word per (query, key tile) laid out [Sq][tiles], bit j of
// a word set = key 64 tile + j is hidden from the query, is applied to the scores besides the causal
// mask; needs RAGGED.  A lane fetches the word of its query for the next tile (one bounded 8-byte buffer
// load: zero past the end) while the current tile is worked on.  A row with every key hidden gives zeros,
// maximum 0 and sum 1.  tile_lo .. tile_hi (MASKED only): the key tiles outside this range hold no key that
// any query of the block may see (the host derives the range from the mask words); they are neither
// copied nor computed, which is what makes a sliding window or a block-sparse mask cheaper than a dense one.
template <typename T, bool CAUSAL, bool RAGGED, int WAVES = kAttnV5Waves, int DH = 128, bool MASKED = false,
          typename TL = AttnNoTimeline>
__device__ __forceinline__ void attention_fwd_d128_v5(const T* __restrict__ Q, const T* __restrict__ K,
                                                      const T* __restrict__ V, T* __restrict__ O,
                                                      float* __restrict__ softmax_max,
                                                      float* __restrict__ softmax_sum, int Sq, int Sk,
                                                      int q_block, int head, float scale_log2e,
                                                      const unsigned char* __restrict__ head_mask = nullptr,
                                                      TL timeline = TL(), int tile_lo = 0, int tile_hi = 0x7fffff) {
  typedef AttnElem<T> E;
  typedef typename E::x8 x8_t;
  constexpr bool GUARDED = CAUSAL || RAGGED;  // the last tiles of a block run the guarded copy of the loop
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  // K and V tiles as they come from memory, [64 rows][128] bf16 without padding, 16-byte chunks of a
  // row XOR-swizzled; written by direct global -> LDS loads (one 1 KiB block = four rows per
  // wavefront instruction), two buffers each
  constexpr int kTileElems = 64 * 128;
  T* Kbuf = reinterpret_cast<T*>(attn_lds);
  T* Vbuf = Kbuf + 2 * kTileElems;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int g = lane >> 5;

  constexpr int BM = WAVES * 32;
  const int q0 = q_block * BM;
  // MASKED: key tiles before tile_lo and after tile_hi are left out; the loop below then walks tiles relative to
  // tile_lo, keys are counted from `shift` and the sequence ends with tile tile_hi
  const int all_tiles = (Sk + kAttnBN - 1) / kAttnBN;
  if constexpr (MASKED) {
    tile_lo = max(0, min(tile_lo, CAUSAL ? min(q0 / kAttnBN, all_tiles - 1) : all_tiles - 1));
    tile_hi = max(tile_lo, tile_hi);
  }
  const int shift = MASKED ? tile_lo * kAttnBN : 0;
  const int Sk_end = MASKED ? min(Sk, (tile_hi + 1) * kAttnBN) : Sk;  // first key that is not looked at
  const int Sk_rel = Sk_end - shift;                                  // keys the loop covers

  const size_t head_off = static_cast<size_t>(head) * Sq * kAttnD;
  const size_t kv_off = static_cast<size_t>(head) * Sk * kAttnD + static_cast<size_t>(shift) * kAttnD;
  const T* __restrict__ Qh = Q + head_off;
  const T* __restrict__ Kh = K + kv_off;
  const T* __restrict__ Vh = V + kv_off;

  static_assert(WAVES == 8, "8 wavefronts");
  static_assert(DH == 128 || DH == 64, "128 or 64 data columns");
  static_assert(!MASKED || RAGGED, "the masked instantiations are the bounds-checking ones");
  constexpr int DS = DH / 16;  // d slices of a score product
  constexpr int DB = DH / 32;  // d blocks of the output
  constexpr int NA = 4 * DB;   // chunks (= MFMAs) of phase A
  constexpr int NB = 2 * DS;   // chunks of phase B
  static_assert(sizeof(T) == 2, "16-bit elements");
  // Wavefronts 4..7 take the 32-query sub-blocks in reverse order: with a causal mask a sub-block
  // needs 1 + sub / 2 of the four diagonal tiles, and the two wavefronts that share a SIMD
  // (w and w + 4) then have five tiles of diagonal work between them on every SIMD instead of
  // four to six.
#ifndef MI_ATTN_V5_BALANCE
#define MI_ATTN_V5_BALANCE 1
#endif
  const int sub = (CAUSAL && MI_ATTN_V5_BALANCE && WAVES == 8 && wave >= 4) ? 11 - wave : wave;
  const int qi = q0 + sub * 32 + li;
  const int qi_ld = RAGGED ? min(qi, Sq - 1) : qi;  // rows past the end work on a copy of the last row

  timeline.mark(0, head, q_block);
  x8_t qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s)
    qf[s] = *reinterpret_cast<const x8_t*>(Qh + static_cast<size_t>(qi_ld) * kAttnD + 16 * s + 8 * g);

  f32x16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_run = -__builtin_inff(), m_true = -__builtin_inff(), l_run = 0.f, alpha = 1.f;

  // Tiles that hold keys at all, tiles this block can see, and the (even) number the loop walks:
  // the pipeline below is unrolled over pairs of tiles, so an odd count is padded with one tile
  // that lies wholly past the end (zeros from the bounded loads, skipped like a tile above the
  // diagonal).
  const int real_tiles = RAGGED ? (Sk_rel + kAttnBN - 1) / kAttnBN : Sk / kAttnBN;
  const int vis_tiles = CAUSAL ? min(real_tiles, (q0 + BM - shift) / kAttnBN) : real_tiles;
  const int n_tiles = RAGGED ? 2 * ((vis_tiles + 1) / 2) : vis_tiles;
  // first tile that needs the guarded loop: the diagonal, or the tile that holds the end of the keys
  const int first_masked = CAUSAL ? (q0 - shift) / kAttnBN : (RAGGED ? Sk_rel / kAttnBN : n_tiles);

  // direct global -> LDS copies: block b of a tile (rows 4 b .. 4 b + 3) is written by one wavefront
  // instruction, lane l filling LDS chunk l of the block (row 4 b + l / 16, chunk position l % 16)
  // with the global chunk that the swizzle puts there
  const int blk_row = lane >> 4;
  const int blk_pos = lane & 15;
  const int kv_bytes = RAGGED ? Sk_rel * kAttnD * 2 : 0x7fffffff;  // loads past a head's keys return zeros
  auto issue_tile = [&](const T* __restrict__ src, T* dst, int tile, auto swz) {
#pragma unroll
    for (int u = 0; u < 16 / WAVES; ++u) {
      const int b = (16 / WAVES) * wave + u;
      const int row = 4 * b + blk_row;
      const int gchunk = blk_pos ^ swz(row);
      // The buffer form of the copy (base = this head's K or V, byte offset per lane).  With the global
      // form (global_load_lds) the compiler's wait-count pass sees a FLAT access pending on both
      // counters and turns every later wait for an LDS fragment into lgkmcnt(0), a full drain that
      // undoes the two-chunk prefetch; with the buffer form the waits are lgkmcnt(1) / (2), the kernel
      // needs 200 / 228 registers instead of 206 / 256 + 4 spilled, and runs about 1 % faster.
      const int voff = ((tile * kAttnBN + row) * kAttnD + 8 * gchunk) * 2;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(
          __builtin_amdgcn_make_buffer_rsrc(const_cast<T*>(src), 0, kv_bytes, 0x00020000),
          (__attribute__((address_space(3))) void*)(dst + b * 512), 16, voff, 0, 0, 0);
    }
  };
  auto swz_k = [](int row) { return row & 15; };
  auto swz_v = [](int row) { return (0xE4A0 >> (4 * (row & 3))) & 15; };  // 0, 10, 4, 14
  auto issue_k = [&](int tile, int buf) { issue_tile(Kh, Kbuf + buf * kTileElems, tile, swz_k); };
  auto issue_v = [&](int tile, int buf) { issue_tile(Vh, Vbuf + buf * kTileElems, tile, swz_v); };

  f32x16_t sacc[2];  // [key block]
  u32x4_t pw[4];     // P of the current tile: [key slice of 16] x four 32-bit words

  // K fragment of chunk i of phase B (key block i / DS, d slice i % DS): row 32 kb + li, chunk 2 ks + g
  int k_off[DS];
#pragma unroll
  for (int ks = 0; ks < DS; ++ks) k_off[ks] = li * kAttnD + 8 * ((2 * ks + g) ^ (li & 15));
  auto k_frag = [&](const T* Ks, int i) {
    return *reinterpret_cast<const x8_t*>(Ks + 32 * (i / DS) * kAttnD + k_off[i % DS]);
  };
  // V^T fragment of chunk i of phase A (key slice t4 = i / DB, d block db = i % DB) by two transposing
  // LDS reads: in each group of 16 lanes, lane s points at four consecutive d of key
  // 4 g + s / 4 (+ 8 for the second read) and receives, for its own d, the four keys of the group
  int v_off[DB];
  {
    const int sl16 = lane & 15, grp = lane >> 4;
    const int key_l = 4 * (grp >> 1) + (sl16 >> 2);
    const int f = (0xE4A0 >> (4 * (key_l & 3))) & 15;
    const int c_l = 2 * (grp & 1) + ((sl16 & 3) >> 1);
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_off[db] = key_l * kAttnD + 8 * (((4 * db) ^ (f & 12)) + (c_l ^ (f & 2))) + 4 * (sl16 & 1);
  }
  auto v_frag = [&](const T* Vt, int i) {
    const int t4 = i / DB, db = i % DB;
    const T* p0 = Vt + 16 * t4 * kAttnD + v_off[db];
    const typename E::x4 lo = E::read_tr(p0);
    const typename E::x4 hi = E::read_tr(p0 + 8 * kAttnD);
    x8_t r;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      r[e] = lo[e];
      r[4 + e] = hi[e];
    }
    return r;
  };

  // last key this lane's query may see: itself under a causal mask, the last key there is otherwise
  const int key_limit = (CAUSAL ? (RAGGED ? min(qi_ld, Sk_end - 1) : qi) : Sk_end - 1) - shift;
  auto apply_mask = [&](int tile) {
    const int d = key_limit - (tile * kAttnBN + 4 * g);  // keys with local offset > d are masked
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (32 * kb + 8 * (r >> 2) + (r & 3) > d) sacc[kb][r] = -__builtin_inff();
  };
  // ---- byte mask of this head: dwords of row qi_ld that hold the lane's keys of one tile ----
  u32x2_t mk;  // bits 0..31: the first key block of the tile, 32..63: the second
  const int mask_tiles = (Sk + kAttnBN - 1) / kAttnBN;
  auto mask_fetch = [&](int tile) {
    if constexpr (MASKED) {
      const auto rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<unsigned char*>(head_mask), 0, Sq * mask_tiles * 8, 0x00020000);
      mk = __builtin_amdgcn_raw_buffer_load_b64(rsrc, (qi_ld * mask_tiles + min(tile + tile_lo, mask_tiles)) * 8, 0, 0);
      if (tile + tile_lo >= mask_tiles) mk = u32x2_t{0u, 0u};  // tiles past the end hold no keys (already hidden by the length)
    }
  };
  // hides what the fetched dwords mark in S(tile) and requests the dwords of the next tile
  auto mask_apply = [&](int tile) {
    if constexpr (MASKED) {
      // masks are mostly runs of visible or of hidden keys: a tile none of whose keys is hidden from
      // any query of the wavefront (all its dwords zero) skips the selects
      if (__any((mk[0] | mk[1]) != 0)) {
        // accumulator register r of key block kb is key 32 kb + 8 (r / 4) + 4 g + r % 4
        const uint32_t b0 = mk[0] >> (4 * g), b1 = mk[1] >> (4 * g);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          if ((b0 >> (8 * (r >> 2) + (r & 3))) & 1u) sacc[0][r] = -__builtin_inff();
          if ((b1 >> (8 * (r >> 2) + (r & 3))) & 1u) sacc[1][r] = -__builtin_inff();
        }
      }
      mask_fetch(tile + 1);
    }
  };
  float mpart, mx, m_new, psum;
  auto softmax_rowmax = [&](auto kb_c) {
    constexpr int kb = decltype(kb_c)::value;
    float a = sacc[kb][0];
#pragma unroll
    for (int r = 1; r < 16; ++r) a = fmaxf(a, sacc[kb][r]);
    if constexpr (kb == 0) {
      mpart = a;
    } else {
      a = fmaxf(a, mpart);
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(a), false, false);
      mx = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
  };
  auto softmax_ref = [&]() {
    m_true = fmaxf(m_true, mx * scale_log2e);
    // a finite floor keeps rows whose keys have all been hidden so far free of inf - inf
    if constexpr (MASKED) m_true = fmaxf(m_true, -1e30f);
    m_new = m_true > m_run + kAttnSlack ? m_true : m_run;
    alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    psum = 0.f;
  };
  auto softmax_word = [&](auto t4_c, auto j_c) {  // word j of key slice t4
    constexpr int t4 = decltype(t4_c)::value, j = decltype(j_c)::value;
    constexpr int kb = t4 >> 1;
    constexpr int r = 8 * (t4 & 1) + 2 * j;
    const float p0 = __builtin_amdgcn_exp2f(fmaf(sacc[kb][r], scale_log2e, -m_new));
    const float p1 = __builtin_amdgcn_exp2f(fmaf(sacc[kb][r + 1], scale_log2e, -m_new));
    psum += p0 + p1;
    typename E::x2 pk;
    pk[0] = static_cast<T>(p0);
    pk[1] = static_cast<T>(p1);
    uint32_t word = __builtin_bit_cast(uint32_t, pk);
    asm volatile("" : "+v"(word), "+v"(psum));  // keep the work in this slot of the schedule
    pw[t4][j] = word;
  };

  // ---- phase A: O += V^T(tile-1) P(tile-1) beside the first part of the softmax step on S(tile) ----
  // GUARD: the wavefront-uniform flags do_pv / do_sm switch the matrix and the softmax work of the
  // phase off (diagonal tiles that lie wholly above this wavefront's queries); without GUARD they
  // are ignored and the phase is straight-line code.
  auto phase_a = [&](auto pv_c, auto odd_c, int k_tile, int v_tile, auto guard_c, bool do_pv, bool do_sm) {
    constexpr bool DO_PV = decltype(pv_c)::value;
    constexpr bool GUARD = decltype(guard_c)::value;
    constexpr int ODD = decltype(odd_c)::value ? 1 : 0;
    const T* Vt = Vbuf + (1 - ODD) * kTileElems;
    x8_t f[NA];
    if constexpr (DO_PV) {
      if (!GUARD || do_pv) {
        f[0] = v_frag(Vt, 0);
        f[1] = v_frag(Vt, 1);
      }
    }
    static_for<NA>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int t4 = i / DB, db = i % DB;
      if constexpr (DO_PV) {
        if (!GUARD || do_pv) {
          if constexpr (i + 2 < NA) f[i + 2] = v_frag(Vt, i + 2);
          oacc[db] = E::mfma(f[i], __builtin_bit_cast(x8_t, pw[t4]), oacc[db]);
        }
      }
      if constexpr (i == 0) issue_k(k_tile, ODD);
      if constexpr (i == 1) issue_v(v_tile, ODD);
      if (!GUARD || do_sm) {
        if constexpr (DH == 128) {
          if constexpr (i == 0) softmax_rowmax(std::integral_constant<int, 0>());
          if constexpr (i == 1) softmax_rowmax(std::integral_constant<int, 1>());
          if constexpr (i == 2) softmax_ref();
          // key slice j of P may be rewritten once chunk 4 j + 3 has issued its MFMA
          if constexpr (i >= 4 && i < 12)
            softmax_word(std::integral_constant<int, (i >= 4 && i < 12) ? (i >> 2) - 1 : 0>(), std::integral_constant<int, (i & 3)>());
        } else {
          // eight chunks: key slice j of P may be rewritten once chunk 2 j + 1 has issued its MFMA
          if constexpr (i == 0) {
            softmax_rowmax(std::integral_constant<int, 0>());
            softmax_rowmax(std::integral_constant<int, 1>());
          }
          if constexpr (i == 1) softmax_ref();
          if constexpr (i >= 2 && i < 6) {
            softmax_word(std::integral_constant<int, (i >= 2 && i < 6) ? (i - 2) / 2 : 0>(), std::integral_constant<int, 2 * (i & 1)>());
            softmax_word(std::integral_constant<int, (i >= 2 && i < 6) ? (i - 2) / 2 : 0>(), std::integral_constant<int, 2 * (i & 1) + 1>());
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto rescale = [&]() {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
  };
  // ---- phase B: S(tile+1) = K(tile+1) Q^T beside the rest of P(tile) and the LDS writes ----
  auto phase_b = [&](auto qk_c, auto odd_c, auto guard_c, bool do_qk, bool do_sm) {
    constexpr bool DO_QK = decltype(qk_c)::value;
    constexpr bool GUARD = decltype(guard_c)::value;
    constexpr int ODD = decltype(odd_c)::value ? 1 : 0;
    const T* Ks = Kbuf + (1 - ODD) * kTileElems;
    x8_t f[NB];
    if constexpr (DO_QK) {
      if (!GUARD || do_qk) {
        f[0] = k_frag(Ks, 0);
        f[1] = k_frag(Ks, 1);
      }
    }
    static_for<NB>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int kb = i / DS, ks = i % DS;
      if constexpr (DO_QK) {
        if (!GUARD || do_qk) {
          if constexpr (i + 2 < NB) f[i + 2] = k_frag(Ks, i + 2);
          if constexpr (ks == 0) {
            f32x16_t z;
#pragma unroll
            for (int r = 0; r < 16; ++r) z[r] = 0.f;
            sacc[kb] = E::mfma(f[i], qf[ks], z);
          } else {
            sacc[kb] = E::mfma(f[i], qf[ks], sacc[kb]);
          }
        }
      }
      if (!GUARD || do_sm) {
        // key slices 2 and 3 of P read S's second key block, which chunk DS starts to overwrite
        if constexpr (DH == 128) {
          if constexpr (i < 8) softmax_word(std::integral_constant<int, 2 + (i >> 2)>(), std::integral_constant<int, (i & 3)>());
          if constexpr (i == 7) l_run = fmaf(l_run, alpha, psum);
        } else {
          if constexpr (i < 4) {
            softmax_word(std::integral_constant<int, 2 + (i >> 1)>(), std::integral_constant<int, 2 * (i & 1)>());
            softmax_word(std::integral_constant<int, 2 + (i >> 1)>(), std::integral_constant<int, 2 * (i & 1) + 1>());
          }
          if constexpr (i == 3) l_run = fmaf(l_run, alpha, psum);
        }
      }
      if constexpr (i == NB - 1) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): this iteration's tiles have landed
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // ---- prologue: K(0), K(1) in LDS, S(0) ----
  mask_fetch(0);
  issue_k(0, 0);
  issue_k(1, 1);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): Q fragments and the tiles above have landed
  __syncthreads();
  timeline.mark(1, head, q_block);
  {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
    for (int i = 0; i < NB; ++i)
      sacc[i / DS] = E::mfma(k_frag(Kbuf, i), qf[i % DS], sacc[i / DS]);
  }
  __syncthreads();  // K buffer 0 is rewritten in iteration 0

  using Yes = std::true_type;
  using No = std::false_type;
  // last key tile this wavefront's queries can see (only the diagonal tiles differ between wavefronts)
  const int last_tile =
      CAUSAL ? (RAGGED ? min((min(q0 + sub * 32 + 31, Sq - 1) - shift) / kAttnBN, real_tiles - 1) : first_masked + (sub >> 1))
             : real_tiles - 1;
  if (GUARDED && 0 == last_tile) apply_mask(0);
  mask_apply(0);
  phase_a(No(), No(), min(2, n_tiles - 1), 0, No(), true, true);
  phase_b(Yes(), No(), No(), true, true);
  __syncthreads();

  auto pair = [&](int t, auto mask_c) {
    constexpr bool MASK = decltype(mask_c)::value;
    {
      if constexpr (MASK) {
        if (t == last_tile) apply_mask(t);
      }
      mask_apply(t);
      const bool sm = !MASK || t <= last_tile;
      phase_a(Yes(), Yes(), min(t + 2, n_tiles - 1), t, mask_c, t - 1 <= last_tile, sm);  // K past the end: a harmless reload
      if (sm) rescale();
      phase_b(Yes(), Yes(), mask_c, t + 1 <= last_tile, sm);
      __syncthreads();
    }
    {
      const int u = t + 1;
      if constexpr (MASK) {
        if (u == last_tile) apply_mask(u);
      }
      mask_apply(u);
      const bool sm = !MASK || u <= last_tile;
      phase_a(Yes(), No(), min(u + 2, n_tiles - 1), u, mask_c, u - 1 <= last_tile, sm);
      if (sm) rescale();
      phase_b(Yes(), No(), mask_c, u + 1 <= last_tile, sm);
      __syncthreads();
    }
  };
  timeline.mark(2, head, q_block);
  int t = 1;
  for (; t + 1 < first_masked; t += 2) pair(t, No());
  timeline.mark(3, head, q_block);
  if constexpr (GUARDED) {
    for (; t < n_tiles - 1; t += 2) pair(t, Yes());
  }
  {
    t = n_tiles - 1;
    const bool sm = t <= last_tile;
    if (GUARDED && t == last_tile) apply_mask(t);
    mask_apply(t);
    phase_a(Yes(), Yes(), t, t, std::integral_constant<bool, GUARDED>(), t - 1 <= last_tile, sm);
    if (sm) rescale();
    phase_b(No(), Yes(), std::integral_constant<bool, GUARDED>(), false, sm);
    __syncthreads();
    if (sm) {
      const T* Vt = Vbuf + kTileElems;
#pragma unroll
      for (int i = 0; i < NA; ++i)
        oacc[i % DB] = E::mfma(v_frag(Vt, i), __builtin_bit_cast(x8_t, pw[i / DB]), oacc[i % DB]);
    }
  }

  timeline.mark(4, head, q_block);
  // ---- epilogue ----
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
  const float l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  const bool hidden_row = MASKED && l_tot == 0.f;  // every key of this query was hidden
  const float inv_l = hidden_row ? 0.f : 1.0f / l_tot;
  const float l_true = hidden_row ? 1.0f : l_tot * __builtin_amdgcn_exp2f(m_run - m_true);
  // The accumulators hold O^T: a lane owns one query and, per register quad, four consecutive d.
  // Stored from there a wavefront instruction would write 32 separate 16-byte pieces, one per row;
  // measured on MI355X those partial-line writes kept a workgroup's CU busy for about 5 us per query
  // block (7 % of the causal launch).  So the tile goes through LDS once: every wavefront writes its
  // 32 x 128 block into its own 8 KiB of the (now idle) K/V buffers, 16-byte chunks XOR-swizzled by the
  // row, and reads it back row-wise, so that one instruction stores four whole 256-byte rows.
  __syncthreads();  // every wavefront is done with the K and V tiles
  {
    T* stage = reinterpret_cast<T*>(attn_lds) + wave * (32 * kAttnD);
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        typename E::x4 o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) o4[e] = static_cast<T>(oacc[db][4 * rq + e] * inv_l);
        *reinterpret_cast<typename E::x4*>(stage + li * kAttnD + 8 * ((4 * db + rq) ^ (li & 15)) + 4 * g) = o4;
      }
    T* __restrict__ oblk = O + head_off + static_cast<size_t>(q0 + sub * 32) * kAttnD;
    const int c16 = lane & 15;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int row = 4 * j + (lane >> 4);
      const u32x4_t v16 = *reinterpret_cast<const u32x4_t*>(stage + row * kAttnD + 8 * (c16 ^ (row & 15)));
      if (!RAGGED || q0 + sub * 32 + row < Sq) *reinterpret_cast<u32x4_t*>(oblk + row * kAttnD + 8 * c16) = v16;
    }
  }
  timeline.mark(5, head, q_block);
  if (g == 0 && (!RAGGED || qi < Sq)) {
    const size_t so = (static_cast<size_t>(head) * Sq + qi) * 8;
    const float m_nat = hidden_row ? 0.f : m_true * 0.69314718055994530942f;
    Vec<float, 4> mv, lv;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mv[e] = m_nat;
      lv[e] = l_true;
    }
    store_vec<float, 4>(softmax_max + so, mv);
    store_vec<float, 4>(softmax_max + so + 4, mv);
    store_vec<float, 4>(softmax_sum + so, lv);
    store_vec<float, 4>(softmax_sum + so + 4, lv);
  }
  __syncthreads();  // the staging reads are done before a following query block refills the K buffers
  timeline.mark(6, head, q_block);
}

// One workgroup of a persistent launch.  Workgroup -> (head, query block) mapping: hardware deals consecutive
// workgroup ids round-robin to the 8 accelerator dies, each with its own L2.  Ids that land on one die walk
// the query blocks of one head before moving to the next head, so a head's K and V are fetched into a single
// L2.  Under a causal mask query block b visits 4 b + 4 key tiles; a work item is the pair (b, n - 1 - b), the
// longer member first, so every item is the same amount of work.  The grid is at most one workgroup per CU and
// every workgroup walks the work items id = blockIdx.x, blockIdx.x + gridDim.x, ... (gridDim.x is a multiple
// of 8, so a workgroup stays on the heads of its own die).
template <typename T, bool CAUSAL, bool RAGGED, int DH = 128, bool MASKED = false, typename TL = AttnNoTimeline>
__device__ __forceinline__ void attention_entry_v5(const T* q, const T* k, const T* v, T* o, float* smax,
                                                   float* ssum, int n_heads, int Sq, int Sk,
                                                   float scale_log2e, const unsigned char* mask = nullptr,
                                                   long long mask_batch_stride = 0, long long mask_head_stride = 0,
                                                   int heads_per_batch = 1, TL timeline = TL(),
                                                   const int* tile_ranges = nullptr, int range_batch_stride = 0,
                                                   int range_head_stride = 0) {
  constexpr int XCDS = 8;
  const int n_qb = (Sq + kAttnV5BM - 1) / kAttnV5BM;
  const int per_head = CAUSAL ? (n_qb + 1) / 2 : n_qb;
  const int total = XCDS * ((n_heads + XCDS - 1) / XCDS) * per_head;
#pragma nounroll
  for (int id = blockIdx.x; id < total; id += gridDim.x) {
    const int xcd = id % XCDS;
    const int slot = id / XCDS;
    const int head = (slot / per_head) * XCDS + xcd;
    if (head >= n_heads) continue;
    // the [Sq][tiles] 64-bit mask words of this head (byte strides; 0 where the mask broadcasts over batch or heads)
    const unsigned char* hm =
        MASKED ? mask + (head / heads_per_batch) * mask_batch_stride + (head % heads_per_batch) * mask_head_stride : nullptr;
    // (first, last) key tile that holds a visible key, per query block: [B or 1][N or 1][query blocks][2]
    const int* hr = (MASKED && tile_ranges)
                        ? tile_ranges + (head / heads_per_batch) * range_batch_stride + (head % heads_per_batch) * range_head_stride
                        : nullptr;
    auto range_lo = [&](int qb) { return hr ? hr[2 * qb] : 0; };
    auto range_hi = [&](int qb) { return hr ? hr[2 * qb + 1] : 0x7fffff; };
    if (CAUSAL) {
      const int lo = slot % per_head;
      const int hi = n_qb - 1 - lo;
      const int n_pass = lo != hi ? 2 : 1;
#pragma nounroll
      for (int pass = 0; pass < n_pass; ++pass)
        attention_fwd_d128_v5<T, true, RAGGED, kAttnV5Waves, DH, MASKED, TL>(q, k, v, o, smax, ssum, Sq, Sk, pass == 0 ? hi : lo,
                                                                             head, scale_log2e, hm, timeline,
                                                                             range_lo(pass == 0 ? hi : lo), range_hi(pass == 0 ? hi : lo));
    } else {
      attention_fwd_d128_v5<T, false, RAGGED, kAttnV5Waves, DH, MASKED, TL>(q, k, v, o, smax, ssum, Sq, Sk, slot % per_head, head,
                                                                            scale_log2e, hm, timeline, range_lo(slot % per_head),
                                                                            range_hi(slot % per_head));
    }
  }
}

}  // namespace mi
