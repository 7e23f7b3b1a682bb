// Fused attention forward, 64 queries per wavefront, one wavefront per SIMD.
//
// Same mathematics, operand layouts and LDS tile formats as attention.h.  What
// changes is the shape of the work per wavefront: it owns two blocks of 32
// queries (X and Y), so every K fragment and every V^T fragment read from LDS
// feeds two MFMAs instead of one, which halves LDS traffic per flop (with one
// fragment per MFMA four SIMDs ask LDS for 4 KiB every 32 cycles, its full
// bandwidth).  A workgroup is 4 wavefronts (256 queries); with ~450 registers
// per lane a SIMD holds a single wavefront, so the matrix core and the vector
// ALU are kept busy from one instruction stream.  Iteration t is two phases:
//     A   matrix:  O += V^T(t-1) P(t-1)      vector:  row max of S(t), first half of P(t)
//     B   matrix:  S(t+1) = K(t+1) Q^T       vector:  second half of P(t); K(t+2), V(t) -> LDS
// P lives in one set of registers: the words for key slice j of P(t) are produced only
// after the MFMAs that read slice j of P(t-1) have been issued, and the second half
// before the MFMAs of phase B overwrite S's second key block.
// Each phase is written as 16 chunks of {one LDS fragment read two chunks
// ahead, two MFMAs, one slice of the vector work}; a scheduling fence between
// chunks keeps the compiler from regrouping them, which both fixes the
// interleave and bounds the number of fragments in flight.  K and V^T tiles are
// double-buffered in LDS; one barrier per iteration.
//
#pragma once

#include <type_traits>
#include <utility>

#include "attention.h"

namespace mi {

constexpr int kAttnV2Waves = 4;
constexpr int kAttnV2QueriesPerWave = 64;
constexpr int kAttnV2BM = kAttnV2Waves * kAttnV2QueriesPerWave;
constexpr int kAttnV2KElems = kAttnBN * kAttnKStride;
constexpr int kAttnV2VElems = kAttnD * kAttnVStride;
constexpr int kAttnV2LdsBytes = 2 * (kAttnV2KElems + kAttnV2VElems) * 2;
// The reference maximum of the online softmax moves only when the true maximum has grown
// past it by more than this many powers of two.  Until then probabilities are at most
// 2^slack (no overflow, same relative precision in bf16 and fp32), numerator and
// denominator stay consistent, and the 128 accumulator registers per lane need no
// rescaling: with 64 queries per wavefront some query raises its maximum in most tiles,
// but hardly ever by a factor of 256.
constexpr float kAttnV2Slack = 8.0f;
// LDS fragments are requested this many chunks (of two MFMAs) before they are used.
#ifndef ATTN_V2_PREFETCH
#define ATTN_V2_PREFETCH 2
#endif
constexpr int kAttnV2Prefetch = ATTN_V2_PREFETCH;
// Row sum of the probabilities: in fp32 before rounding (false; what softmax_sum is
// defined as), or of the bf16-rounded values the matrix core multiplies with V, by a
// two-element dot product (true; one vector instruction per pair fewer, ~1e-3 relative
// difference in softmax_sum).
constexpr bool kAttnV2RowSumOfRounded = false;

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));

template <bool B>
using attn_flag = std::integral_constant<bool, B>;

template <int... I, class F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, F&& f) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// P of one tile for both query blocks, as MFMA B operands: [query block][key slice of 16]
// holds four 32-bit words = eight bf16 probabilities.  Words are written whole, so no
// register is ever updated in part.
struct AttnV2P {
  u32x4_t w[2][4];
};

__device__ __forceinline__ bf16x8_t attn_as_bf16x8(u32x4_t x) {
  return __builtin_bit_cast(bf16x8_t, x);
}

// S += A * B with the accumulator in vector registers and B (a Q fragment) in the
// accumulation register file.  Written as inline assembly because the compiler picks one
// register file for the accumulators of all MFMAs of a kernel, and the softmax reads S
// with vector instructions.  Operands come from LDS loads, earlier MFMAs or constants
// only, so no vector-ALU -> MFMA hazard arises on the input side; the caller separates
// the last of these from the first vector read of S (attn_mfma_result_fence).
__device__ __forceinline__ void attn_mfma_vacc(f32x16_t& acc, bf16x8_t a, bf16x8_t b) {
  asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "a"(b));
}
__device__ __forceinline__ void attn_mfma_vacc_first(f32x16_t& acc, bf16x8_t a, bf16x8_t b) {
  // early clobber: the result registers must not overlap the operands
  asm("v_mfma_f32_32x32x16_bf16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a), "a"(b));
}
// The hardware does not interlock a vector-ALU access to registers that an MFMA in flight
// is still going to write (12 idle issue slots after an 8-pass MFMA such as this one; the
// fence gives 16), and the compiler cannot see MFMAs inside inline assembly.  The fence takes S as
// in/out operands so that data flow orders it after the last MFMA and before every read.
__device__ __forceinline__ void attn_mfma_result_fence(f32x16_t& a, f32x16_t& b, f32x16_t& c, f32x16_t& d) {
  asm volatile("s_nop 15" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

template <bool CAUSAL>
__device__ __forceinline__ void attention_fwd_d128_v2(const bf16_t* __restrict__ Q,
                                                      const bf16_t* __restrict__ K,
                                                      const bf16_t* __restrict__ V,
                                                      bf16_t* __restrict__ O,
                                                      float* __restrict__ softmax_max,
                                                      float* __restrict__ softmax_sum, int S,
                                                      int q_block, int head, float scale_log2e) {
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  bf16_t* Kbuf = reinterpret_cast<bf16_t*>(attn_lds);
  bf16_t* Vbuf = Kbuf + 2 * kAttnV2KElems;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int g = lane >> 5;

  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const bf16_t* __restrict__ Qh = Q + head_off;
  const bf16_t* __restrict__ Kh = K + head_off;
  const bf16_t* __restrict__ Vh = V + head_off;

  const int q0 = q_block * kAttnV2BM;
  const int qw = q0 + wave * kAttnV2QueriesPerWave;  // first query of this wavefront
  int qi[2];
  qi[0] = qw + li;
  qi[1] = qw + 32 + li;

  bf16x8_t qf[2][8];
#pragma unroll
  for (int sub = 0; sub < 2; ++sub)
#pragma unroll
    for (int s = 0; s < 8; ++s)
      qf[sub][s] =
          *reinterpret_cast<const bf16x8_t*>(Qh + static_cast<size_t>(qi[sub]) * kAttnD + 16 * s + 8 * g);

  f32x16_t oacc[2][4];
#pragma unroll
  for (int sub = 0; sub < 2; ++sub)
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int r = 0; r < 16; ++r) oacc[sub][db][r] = 0.f;
  // m_run is the reference maximum the probabilities are scaled by; it follows the true
  // running maximum m_true lazily (see kAttnV2Slack) so that O rarely needs rescaling.
  float m_run[2] = {-__builtin_inff(), -__builtin_inff()};
  float m_true[2] = {-__builtin_inff(), -__builtin_inff()};
  float l_run[2] = {0.f, 0.f};
  float alpha[2] = {1.f, 1.f};

  const int n_tiles = CAUSAL ? (q0 + kAttnV2BM) / kAttnBN : S / kAttnBN;
  // under a causal mask only the last four tiles straddle the diagonal of some wavefront
  const int first_masked = CAUSAL ? n_tiles - kAttnV2BM / kAttnBN : n_tiles;

  // global -> register -> LDS staging, every thread 4 x 16 bytes of K and of V per tile
  u32x4_t kst[4], vst[4];
  const int k_row = tid >> 4;
  const int k_col = (tid & 15) * 8;
  const int v_kg = tid >> 4;
  const int v_dg = tid & 15;
  const int v_pos = attn_vt_pos(4 * v_kg);
  auto load_k_part = [&](int tile, int u) {
    const bf16_t* kp = Kh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    kst[u] = *reinterpret_cast<const u32x4_t*>(kp + static_cast<size_t>(k_row + 16 * u) * kAttnD + k_col);
  };
  auto load_k = [&](int tile) {
#pragma unroll
    for (int u = 0; u < 4; ++u) load_k_part(tile, u);
  };
  auto store_k_part = [&](int buf, int u) {
    bf16_t* Ks = Kbuf + buf * kAttnV2KElems;
    *reinterpret_cast<u32x4_t*>(Ks + (k_row + 16 * u) * kAttnKStride + k_col) = kst[u];
  };
  auto load_v_part = [&](int tile, int u) {
    const bf16_t* vp = Vh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    vst[u] = *reinterpret_cast<const u32x4_t*>(vp + static_cast<size_t>(4 * v_kg + u) * kAttnD + 8 * v_dg);
  };
  auto load_v = [&](int tile) {
#pragma unroll
    for (int u = 0; u < 4; ++u) load_v_part(tile, u);
  };
  // dword e2 of each staged V row holds d = 2 e2 (low half, odd = 0) and 2 e2 + 1 (high half)
  auto store_v_half = [&](int buf, int e2, int odd) {
    bf16_t* Vt = Vbuf + buf * kAttnV2VElems;
    const uint32_t a0 = vst[0][e2], a1 = vst[1][e2], a2 = vst[2][e2], a3 = vst[3][e2];
    const uint32_t sel = odd ? 0x07060302u : 0x05040100u;
    u32x2_t w;
    w[0] = __builtin_amdgcn_perm(a1, a0, sel);
    w[1] = __builtin_amdgcn_perm(a3, a2, sel);
    *reinterpret_cast<u32x2_t*>(Vt + attn_vt_offset(8 * v_dg + 2 * e2 + odd, v_pos)) = w;
  };

  f32x16_t sacc[2][2];  // [query block][key block]

  auto k_frag = [&](const bf16_t* Ks, int i) {  // chunk i of phase B: key block i / 8, d slice i % 8
    return *reinterpret_cast<const bf16x8_t*>(Ks + (32 * (i >> 3) + li) * kAttnKStride + 16 * (i & 7) + 8 * g);
  };
  // V^T fragment of chunk i of phase A (key slice t4 = i / 4, d block db = i % 4) sits at
  // attn_vt_offset(32 db + li, 16 t4 + 8 g).  Its swizzled 16-byte chunk index is
  // ((li ^ li>>3) & 7) ^ g ^ 2 t4 ^ 4 (db & 1): four lane-dependent bases cover all sixteen
  // fragments, the rest is a compile-time offset.
  int v_base[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
    v_base[j] = li * kAttnVStride + ((((li ^ (li >> 3)) & 7) ^ g ^ (2 * j)) << 3);
  auto v_frag = [&](const bf16_t* Vt, int i) {
    const int t4 = i >> 2, db = i & 3;
    return *reinterpret_cast<const bf16x8_t*>(Vt + v_base[t4 ^ (2 * (db & 1))] + 32 * db * kAttnVStride);
  };

  // ---- vector work of the softmax step on S(tile), cut into slices ----
  float mx[2], m_new[2], psum[2];
  AttnV2P pf;  // P of the current tile, overwritten slice by slice (see the file comment)
  // Causal mask of a tile on the diagonal band, applied to S in place.  Only the last
  // four tiles of a query block need it, so it runs as a short separate step in front
  // of phase A rather than as a second copy of the interleaved code.
  auto apply_mask = [&](int tile) {
    const int key0 = tile * kAttnBN + 4 * g;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      const int d = qi[sub] - key0;  // keys with local offset > d are masked
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (32 * kb + 8 * (r >> 2) + (r & 3) > d) sacc[sub][kb][r] = -__builtin_inff();
    }
  };
  // row maximum of one query block (chunks 0 and 1 of phase A), one key block per half
  float mpart[2];
  auto softmax_rowmax = [&](auto sub_c, auto half_c) {
    constexpr int sub = decltype(sub_c)::value;
    constexpr int kb = decltype(half_c)::value;
    float a = sacc[sub][kb][0];
#pragma unroll
    for (int r = 1; r < 16; ++r) a = fmaxf(a, sacc[sub][kb][r]);
    if constexpr (kb == 0) {
      mpart[sub] = a;
    } else {
      a = fmaxf(a, mpart[sub]);
      // lanes l and l + 32 hold the two halves of a query's keys: exchange through the
      // vector ALU (no LDS round trip to wait for)
      const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(a), false, false);
      mx[sub] = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    }
  };
  // reference maximum and rescale factor (slice 2 of phase A)
  auto softmax_ref = [&]() {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      m_true[sub] = fmaxf(m_true[sub], mx[sub] * scale_log2e);
      m_new[sub] = m_true[sub] > m_run[sub] + kAttnV2Slack ? m_true[sub] : m_run[sub];
      alpha[sub] = __builtin_amdgcn_exp2f(m_run[sub] - m_new[sub]);
      m_run[sub] = m_new[sub];
      psum[sub] = 0.f;
    }
  };
  // word w8 of the eight words of key slice t4 (16 keys x both query blocks):
  // query block w8 / 4, word w8 % 4
  auto softmax_word = [&](auto t4_c, auto w8_c) {
    constexpr int t4 = decltype(t4_c)::value;
    constexpr int w8 = decltype(w8_c)::value;
    constexpr int kb = t4 >> 1;
    constexpr int sub = w8 >> 2;
    constexpr int r = 8 * (t4 & 1) + 2 * (w8 & 3);
    bf16x2_t ones;
    ones[0] = static_cast<bf16_t>(1.0f);
    ones[1] = static_cast<bf16_t>(1.0f);
    bf16x2_t pk;
    const float p0 = __builtin_amdgcn_exp2f(fmaf(sacc[sub][kb][r], scale_log2e, -m_new[sub]));
    const float p1 = __builtin_amdgcn_exp2f(fmaf(sacc[sub][kb][r + 1], scale_log2e, -m_new[sub]));
    pk[0] = static_cast<bf16_t>(p0);
    pk[1] = static_cast<bf16_t>(p1);
    if constexpr (kAttnV2RowSumOfRounded) psum[sub] = __builtin_amdgcn_fdot2_f32_bf16(pk, ones, psum[sub], false);
    else psum[sub] += p0 + p1;
    uint32_t word = __builtin_bit_cast(uint32_t, pk);
    // Nothing reads P before the next phase A, and the optimiser would move this whole
    // computation there, out of the shadow of the MFMAs: pin it to this slice.
    asm volatile("" : "+v"(word), "+v"(psum[sub]));
    pf.w[sub][t4][w8 & 3] = word;
  };
  auto softmax_finish = [&]() {
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) l_run[sub] = fmaf(l_run[sub], alpha[sub], psum[sub]);
  };

  // ---- phase A: O += V^T(tile-1) P(tile-1) alongside the first part of the softmax step on S(tile) ----
  // odd_c: parity of `tile` (LDS buffer indices become compile-time constants)
  auto phase_a = [&](auto pv_c, auto odd_c, int k_tile, int v_tile) {
    constexpr bool DO_PV = decltype(pv_c)::value;
    constexpr int ODD = decltype(odd_c)::value ? 1 : 0;
    const bf16_t* Vt = Vbuf + (1 - ODD) * kAttnV2VElems;
    bf16x8_t f[16];
    if constexpr (DO_PV) {
#pragma unroll
      for (int j = 0; j < kAttnV2Prefetch; ++j) f[j] = v_frag(Vt, j);
    }
    // every chunk is two halves of {one MFMA, half of the chunk's vector work}, so that the
    // second MFMA finds the matrix pipe free when it is issued
    static_for<16>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int t4 = i >> 2, db = i & 3;
      static_for<2>([&](auto hc) {
        constexpr int h = decltype(hc)::value;
        if constexpr (DO_PV) {
          if constexpr (h == 0 && i + kAttnV2Prefetch < 16) f[i + kAttnV2Prefetch] = v_frag(Vt, i + kAttnV2Prefetch);
          oacc[h][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[i], attn_as_bf16x8(pf.w[h][t4]), oacc[h][db], 0, 0, 0);
        }
        // the global loads of the tiles that phase B stores to LDS, one per half chunk so
        // that the memory pipeline's queue never fills
        if constexpr (i < 4) {
          if constexpr (h == 0) load_k_part(k_tile, i);
          else load_v_part(v_tile, i);
        }
        if constexpr (i == 0) softmax_rowmax(std::integral_constant<int, 0>(), hc);
        if constexpr (i == 1) softmax_rowmax(std::integral_constant<int, 1>(), hc);
        if constexpr (i == 2 && h == 0) softmax_ref();
        // Key slice j of P may be rewritten once chunk 4 j + 3 has issued its MFMAs.  Slices 0
        // and 1 (S's first key block) are done here, slices 2 and 3 in phase B, which leaves
        // both phases with about as many vector instructions as fit beside their MFMAs.
        if constexpr (i >= 4 && i < 8)
          softmax_word(std::integral_constant<int, 0>(), std::integral_constant<int, (i >= 4 && i < 8 ? 2 * (i - 4) + h : 0)>());
        if constexpr (i >= 8 && h == 0)
          softmax_word(std::integral_constant<int, 1>(), std::integral_constant<int, (i >= 8 ? i - 8 : 0)>());
        __builtin_amdgcn_sched_barrier(0);
      });
    });
  };

  auto rescale = [&]() {
    if (__any(alpha[0] != 1.0f || alpha[1] != 1.0f)) {
#pragma unroll
      for (int sub = 0; sub < 2; ++sub)
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int r = 0; r < 16; ++r) oacc[sub][db][r] *= alpha[sub];
    }
  };

  // ---- phase B: S(tile+1) = K(tile+1) Q^T alongside the rest of P(tile) and the LDS writes of
  //      K(tile+2), V(tile) ----
  auto phase_b = [&](auto qk_c, auto odd_c) {
    constexpr bool DO_QK = decltype(qk_c)::value;
    constexpr int ODD = decltype(odd_c)::value ? 1 : 0;
    const bf16_t* Ks = Kbuf + (1 - ODD) * kAttnV2KElems;
    constexpr int wbuf = ODD;
    bf16x8_t f[16];
    if constexpr (DO_QK) {
#pragma unroll
      for (int j = 0; j < kAttnV2Prefetch; ++j) f[j] = k_frag(Ks, j);
    }
    static_for<16>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int kb = i >> 3, ks = i & 7;
      static_for<2>([&](auto hc) {
        constexpr int h = decltype(hc)::value;
        if constexpr (DO_QK) {
          if constexpr (h == 0 && i + kAttnV2Prefetch < 16) f[i + kAttnV2Prefetch] = k_frag(Ks, i + kAttnV2Prefetch);
          if constexpr (ks == 0) attn_mfma_vacc_first(sacc[h][kb], f[i], qf[h][ks]);
          else attn_mfma_vacc(sacc[h][kb], f[i], qf[h][ks]);
        }
        // key slices 2 and 3 of P read S's second key block, which chunk 8 starts to overwrite
        if constexpr (i < 8)
          softmax_word(std::integral_constant<int, 2 + (i >> 2)>(), std::integral_constant<int, 2 * (i & 3) + h>());
        if constexpr (i == 7 && h == 1) softmax_finish();
        if constexpr (i >= 8 && i < 12 && h == 0) store_k_part(wbuf, i - 8);
        if constexpr (i >= 12) store_v_half(wbuf, i - 12, h);
        __builtin_amdgcn_sched_barrier(0);
      });
    });
    if constexpr (DO_QK) attn_mfma_result_fence(sacc[0][0], sacc[0][1], sacc[1][0], sacc[1][1]);
  };

  // ---- prologue: K(0), K(1) in LDS, S(0) ----
  load_k(0);
#pragma unroll
  for (int u = 0; u < 4; ++u) store_k_part(0, u);
  load_k(1);
#pragma unroll
  for (int u = 0; u < 4; ++u) store_k_part(1, u);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): Q fragments and the tiles above have landed
  __syncthreads();
  {
    // S(0) through phase B's matrix half: tile index -1 reads K buffer 0, no staging
    const bf16_t* Ks = Kbuf;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const bf16x8_t a = k_frag(Ks, i);
      if ((i & 7) == 0) {
        attn_mfma_vacc_first(sacc[0][i >> 3], a, qf[0][i & 7]);
        attn_mfma_vacc_first(sacc[1][i >> 3], a, qf[1][i & 7]);
      } else {
        attn_mfma_vacc(sacc[0][i >> 3], a, qf[0][i & 7]);
        attn_mfma_vacc(sacc[1][i >> 3], a, qf[1][i & 7]);
      }
    }
    attn_mfma_result_fence(sacc[0][0], sacc[0][1], sacc[1][0], sacc[1][1]);
  }
  __syncthreads();  // K buffer 0 is rewritten in iteration 0

  using T = std::true_type;
  using F = std::false_type;

  // ---- iteration 0: no previous tile to multiply ----
  if (CAUSAL && 0 >= first_masked) apply_mask(0);
  phase_a(F(), F(), 2, 0);
  phase_b(T(), F());
  __syncthreads();

  // ---- iterations 1 .. n_tiles-2, two per trip (odd tile, even tile) ----
  // Two copies of the loop: tiles wholly below the diagonal need no mask, and keeping the
  // masking out of that loop keeps it free of branches; the second copy masks every tile
  // (a no-op for a tile that lies below the diagonal after all).
  auto pair = [&](int t, auto mask_c) {
    constexpr bool MASK = decltype(mask_c)::value;
    {
      if constexpr (MASK) apply_mask(t);
      phase_a(T(), T(), min(t + 2, n_tiles - 1), t);  // K past the end: a harmless reload
      rescale();
      phase_b(T(), T());
      __syncthreads();
    }
    {
      const int u = t + 1;
      if constexpr (MASK) apply_mask(u);
      phase_a(T(), F(), min(u + 2, n_tiles - 1), u);
      rescale();
      phase_b(T(), F());
      __syncthreads();
    }
  };
  int t = 1;
  for (; t + 1 < first_masked; t += 2) pair(t, F());
  if constexpr (CAUSAL) {
    for (; t < n_tiles - 1; t += 2) pair(t, T());
  }

  // ---- last iteration (n_tiles - 1 is odd): no next S; then the final product ----
  {
    t = n_tiles - 1;
    if (CAUSAL) apply_mask(t);
    phase_a(T(), T(), t, t);
    rescale();
    phase_b(F(), T());
    __syncthreads();
    const bf16_t* Vt = Vbuf + kAttnV2VElems;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const bf16x8_t a = v_frag(Vt, i);
      const int t4 = i >> 2, db = i & 3;
      oacc[0][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, attn_as_bf16x8(pf.w[0][t4]), oacc[0][db], 0, 0, 0);
      oacc[1][db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, attn_as_bf16x8(pf.w[1][t4]), oacc[1][db], 0, 0, 0);
    }
  }

  // ---- epilogue: normalise, store O and the softmax statistics ----
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    const float l_tot = l_run[sub] + __shfl_xor(l_run[sub], 32, kWave);
    const float inv_l = 1.0f / l_tot;
    // the statistics are reported against the true maximum
    const float l_true = l_tot * __builtin_amdgcn_exp2f(m_run[sub] - m_true[sub]);
    bf16_t* __restrict__ orow = O + head_off + static_cast<size_t>(qi[sub]) * kAttnD;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        bf16x4_t o4;
#pragma unroll
        for (int e = 0; e < 4; ++e) o4[e] = static_cast<bf16_t>(oacc[sub][db][4 * rq + e] * inv_l);
        *reinterpret_cast<bf16x4_t*>(orow + 32 * db + 8 * rq + 4 * g) = o4;
      }
    if (g == 0) {
      const size_t so = (static_cast<size_t>(head) * S + qi[sub]) * 8;
      const float m_nat = m_true[sub] * 0.69314718055994530942f;
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
  }
}

}  // namespace mi
