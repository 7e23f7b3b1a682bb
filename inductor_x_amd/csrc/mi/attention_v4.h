// Fused attention forward, 32 queries per wavefront, two wavefronts per SIMD, with the
// matrix and vector work of each wavefront interleaved instruction by instruction.
//
// Same mathematics, operand layouts and LDS tile formats as attention.h, and the same
// two-phase software pipeline as attention_v2.h:
//     A   matrix:  O += V^T(t-1) P(t-1)      vector:  row max of S(t), first half of P(t)
//     B   matrix:  S(t+1) = K(t+1) Q^T       vector:  second half of P(t); K(t+2), V(t) -> LDS
// in chunks of {one LDS fragment read ahead, one MFMA, a slice of the vector work}.  With
// 32 queries a wavefront needs ~210 registers, so a SIMD holds two, and the vector
// instructions of one issue for free in the shadow of the other's MFMAs (vector
// instructions issued in the shadow of the wavefront's own MFMA still cost about half).
// The price is one LDS fragment per MFMA, which keeps LDS near its bandwidth limit.
#pragma once

#include "attention_v2.h"

namespace mi {

constexpr int kAttnV4Waves = 8;
constexpr int kAttnV4BM = kAttnV4Waves * 32;

template <bool CAUSAL>
__device__ __forceinline__ void attention_fwd_d128_v4(const bf16_t* __restrict__ Q,
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

  const int q0 = q_block * kAttnV4BM;
  const int qi = q0 + wave * 32 + li;

  bf16x8_t qf[8];
#pragma unroll
  for (int s = 0; s < 8; ++s)
    qf[s] = *reinterpret_cast<const bf16x8_t*>(Qh + static_cast<size_t>(qi) * kAttnD + 16 * s + 8 * g);

  f32x16_t oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_run = -__builtin_inff(), m_true = -__builtin_inff(), l_run = 0.f, alpha = 1.f;

  const int n_tiles = CAUSAL ? (q0 + kAttnV4BM) / kAttnBN : S / kAttnBN;
  const int first_masked = CAUSAL ? n_tiles - kAttnV4BM / kAttnBN : n_tiles;

  // global -> register -> LDS copies: every thread 2 x 16 bytes of K and 4 x 8 bytes of V per tile
  u32x4_t kst[2];
  u32x2_t vst[4];
  const int k_row = tid >> 4;
  const int k_col = (tid & 15) * 8;
  const int v_kg = tid >> 5;  // keys 4 v_kg .. + 3
  const int v_dg = tid & 31;  // d 4 v_dg .. + 3
  const int v_pos = attn_vt_pos(4 * v_kg);
  auto load_k_part = [&](int tile, int u) {
    const bf16_t* kp = Kh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    kst[u] = *reinterpret_cast<const u32x4_t*>(kp + static_cast<size_t>(k_row + 32 * u) * kAttnD + k_col);
  };
  auto store_k_part = [&](int buf, int u) {
    bf16_t* Ks = Kbuf + buf * kAttnV2KElems;
    *reinterpret_cast<u32x4_t*>(Ks + (k_row + 32 * u) * kAttnKStride + k_col) = kst[u];
  };
  auto load_v_part = [&](int tile, int u) {
    const bf16_t* vp = Vh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    vst[u] = *reinterpret_cast<const u32x2_t*>(vp + static_cast<size_t>(4 * v_kg + u) * kAttnD + 4 * v_dg);
  };
  // dword e2 of each copied V row holds d = 4 v_dg + 2 e2 (low half, odd = 0) and + 1 (high half)
  auto store_v_part = [&](int buf, int e2, int odd) {
    bf16_t* Vt = Vbuf + buf * kAttnV2VElems;
    const uint32_t a0 = vst[0][e2], a1 = vst[1][e2], a2 = vst[2][e2], a3 = vst[3][e2];
    const uint32_t sel = odd ? 0x07060302u : 0x05040100u;
    u32x2_t w;
    w[0] = __builtin_amdgcn_perm(a1, a0, sel);
    w[1] = __builtin_amdgcn_perm(a3, a2, sel);
    *reinterpret_cast<u32x2_t*>(Vt + attn_vt_offset(4 * v_dg + 2 * e2 + odd, v_pos)) = w;
  };

  f32x16_t sacc[2];  // [key block]
  u32x4_t pw[4];     // P of the current tile: [key slice of 16] x four 32-bit words

  auto k_frag = [&](const bf16_t* Ks, int i) {  // chunk i of phase B: key block i / 8, d slice i % 8
    return *reinterpret_cast<const bf16x8_t*>(Ks + (32 * (i >> 3) + li) * kAttnKStride + 16 * (i & 7) + 8 * g);
  };
  int v_base[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) v_base[j] = li * kAttnVStride + ((((li ^ (li >> 3)) & 7) ^ g ^ (2 * j)) << 3);
  auto v_frag = [&](const bf16_t* Vt, int i) {  // chunk i of phase A: key slice i / 4, d block i % 4
    const int t4 = i >> 2, db = i & 3;
    return *reinterpret_cast<const bf16x8_t*>(Vt + v_base[t4 ^ (2 * (db & 1))] + 32 * db * kAttnVStride);
  };

  auto apply_mask = [&](int tile) {
    const int d = qi - (tile * kAttnBN + 4 * g);  // keys with local offset > d are masked
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        if (32 * kb + 8 * (r >> 2) + (r & 3) > d) sacc[kb][r] = -__builtin_inff();
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
    m_new = m_true > m_run + kAttnV2Slack ? m_true : m_run;
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
    bf16x2_t pk;
    pk[0] = static_cast<bf16_t>(p0);
    pk[1] = static_cast<bf16_t>(p1);
    uint32_t word = __builtin_bit_cast(uint32_t, pk);
    asm volatile("" : "+v"(word), "+v"(psum));  // keep the work in this slot of the schedule
    pw[t4][j] = word;
  };

  // ---- phase A: O += V^T(tile-1) P(tile-1) beside the first part of the softmax step on S(tile) ----
  auto phase_a = [&](auto pv_c, auto odd_c, int k_tile, int v_tile) {
    constexpr bool DO_PV = decltype(pv_c)::value;
    constexpr int ODD = decltype(odd_c)::value ? 1 : 0;
    const bf16_t* Vt = Vbuf + (1 - ODD) * kAttnV2VElems;
    bf16x8_t f[16];
    if constexpr (DO_PV) {
      f[0] = v_frag(Vt, 0);
      f[1] = v_frag(Vt, 1);
    }
    static_for<16>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int t4 = i >> 2, db = i & 3;
      if constexpr (DO_PV) {
        if constexpr (i + 2 < 16) f[i + 2] = v_frag(Vt, i + 2);
        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[i], attn_as_bf16x8(pw[t4]), oacc[db], 0, 0, 0);
      }
      if constexpr (i < 2) load_k_part(k_tile, i);
      if constexpr (i >= 2 && i < 6) load_v_part(v_tile, (i >= 2 && i < 6) ? i - 2 : 0);
      if constexpr (i == 0) softmax_rowmax(std::integral_constant<int, 0>());
      if constexpr (i == 1) softmax_rowmax(std::integral_constant<int, 1>());
      if constexpr (i == 2) softmax_ref();
      // key slice j of P may be rewritten once chunk 4 j + 3 has issued its MFMA
      if constexpr (i >= 4 && i < 12)
        softmax_word(std::integral_constant<int, (i >= 4 && i < 12) ? (i >> 2) - 1 : 0>(), std::integral_constant<int, (i & 3)>());
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto rescale = [&]() {
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
  };
  // ---- phase B: S(tile+1) = K(tile+1) Q^T beside the rest of P(tile) and the LDS writes ----
  auto phase_b = [&](auto qk_c, auto odd_c) {
    constexpr bool DO_QK = decltype(qk_c)::value;
    constexpr int ODD = decltype(odd_c)::value ? 1 : 0;
    const bf16_t* Ks = Kbuf + (1 - ODD) * kAttnV2KElems;
    constexpr int wbuf = ODD;
    bf16x8_t f[16];
    if constexpr (DO_QK) {
      f[0] = k_frag(Ks, 0);
      f[1] = k_frag(Ks, 1);
    }
    static_for<16>([&](auto ic) {
      constexpr int i = decltype(ic)::value;
      constexpr int kb = i >> 3, ks = i & 7;
      if constexpr (DO_QK) {
        if constexpr (i + 2 < 16) f[i + 2] = k_frag(Ks, i + 2);
        if constexpr (ks == 0) {
          f32x16_t z;
#pragma unroll
          for (int r = 0; r < 16; ++r) z[r] = 0.f;
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[i], qf[ks], z, 0, 0, 0);
        } else {
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(f[i], qf[ks], sacc[kb], 0, 0, 0);
        }
      }
      // key slices 2 and 3 of P read S's second key block, which chunk 8 starts to overwrite
      if constexpr (i < 8) softmax_word(std::integral_constant<int, 2 + (i >> 2)>(), std::integral_constant<int, (i & 3)>());
      if constexpr (i == 7) l_run = fmaf(l_run, alpha, psum);
      if constexpr (i >= 8 && i < 10) store_k_part(wbuf, (i >= 8 && i < 10) ? i - 8 : 0);
      if constexpr (i >= 12) store_v_part(wbuf, (i - 12) >> 1, (i - 12) & 1);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  // ---- prologue: K(0), K(1) in LDS, S(0) ----
  load_k_part(0, 0);
  load_k_part(0, 1);
  store_k_part(0, 0);
  store_k_part(0, 1);
  load_k_part(1, 0);
  load_k_part(1, 1);
  store_k_part(1, 0);
  store_k_part(1, 1);
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): Q fragments and the tiles above have landed
  __syncthreads();
  {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      sacc[i >> 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_frag(Kbuf, i), qf[i & 7], sacc[i >> 3], 0, 0, 0);
  }
  __syncthreads();  // K buffer 0 is rewritten in iteration 0

  using T = std::true_type;
  using F = std::false_type;
  if (CAUSAL && 0 >= first_masked) apply_mask(0);
  phase_a(F(), F(), 2, 0);
  phase_b(T(), F());
  __syncthreads();

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
  {
    t = n_tiles - 1;
    if (CAUSAL) apply_mask(t);
    phase_a(T(), T(), t, t);
    rescale();
    phase_b(F(), T());
    __syncthreads();
    const bf16_t* Vt = Vbuf + kAttnV2VElems;
#pragma unroll
    for (int i = 0; i < 16; ++i)
      oacc[i & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_frag(Vt, i), attn_as_bf16x8(pw[i >> 2]), oacc[i & 3], 0, 0, 0);
  }

  // ---- epilogue ----
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run), __float_as_uint(l_run), false, false);
  const float l_tot = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  const float inv_l = 1.0f / l_tot;
  const float l_true = l_tot * __builtin_amdgcn_exp2f(m_run - m_true);
  bf16_t* __restrict__ orow = O + head_off + static_cast<size_t>(qi) * kAttnD;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      bf16x4_t o4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o4[e] = static_cast<bf16_t>(oacc[db][4 * rq + e] * inv_l);
      *reinterpret_cast<bf16x4_t*>(orow + 32 * db + 8 * rq + 4 * g) = o4;
    }
  if (g == 0) {
    const size_t so = (static_cast<size_t>(head) * S + qi) * 8;
    const float m_nat = m_true * 0.69314718055994530942f;
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

}  // namespace mi
