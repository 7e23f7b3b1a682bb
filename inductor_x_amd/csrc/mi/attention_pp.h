// Fused attention forward, "ping-pong" schedule for 8 wavefronts per workgroup.
//
// Same mathematics, operand layouts and LDS tiles as attention.h; what changes
// is when each wavefront does what.  A SIMD holds two wavefronts of the
// workgroup (wave w and wave w + 4).  Per key tile a wavefront has a matrix
// phase (O^T += V^T P^T of the previous tile, then S^T = K Q^T of this tile:
// 32 MFMAs back to back) and a vector phase (online softmax of this tile, and
// its share of copying the next tiles into LDS).  Waves 0-3 ("group A") and
// waves 4-7 ("group B") run these phases in opposite order with a workgroup
// barrier between phases, so on every SIMD one wavefront feeds the matrix core
// while the other runs the softmax on the vector ALU; without the stagger the
// barrier lines all wavefronts up in the same phase and the two units take
// turns idling.  Group A copies V tiles to LDS, group B copies K tiles, each
// during its own vector phase, with the global loads issued one phase earlier.
//
// Timeline (intervals are separated by workgroup barriers, n = key tiles):
//   interval      1        2        3        4        5     ...
//   group A    M(0)     V(0)     M(1)     V(1)     M(2)
//   group B    stage K1 M(0)     V(0)     M(1)     V(1)
//   M(i) = PV(i-1) + QK(i),  V(i) = softmax(i) + copy-in (A: V tile i, B: K tile i+2)
// K tile i is read in intervals 2i+1 (A) and 2i+2 (B) and replaced in 2i+3;
// V tile i is written in 2i+2 and read in 2i+3 (A) and 2i+4 (B); both are
// double-buffered, so no interval reads a buffer that is being written.
#pragma once

#include "attention.h"

namespace mi {

constexpr int kAttnPPWaves = 8;
constexpr int kAttnPPKElems = kAttnBN * kAttnKStride;
constexpr int kAttnPPVElems = kAttnD * kAttnVStride;
constexpr int kAttnPPLdsBytes = 2 * (kAttnPPKElems + kAttnPPVElems) * 2;

template <bool CAUSAL>
__device__ __forceinline__ void attention_fwd_d128_pingpong(const bf16_t* __restrict__ Q,
                                                            const bf16_t* __restrict__ K,
                                                            const bf16_t* __restrict__ V,
                                                            bf16_t* __restrict__ O,
                                                            float* __restrict__ softmax_max,
                                                            float* __restrict__ softmax_sum, int S,
                                                            int q_block, int head, float scale_log2e) {
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  bf16_t* Kbuf = reinterpret_cast<bf16_t*>(attn_lds);  // two K tiles
  bf16_t* Vbuf = Kbuf + 2 * kAttnPPKElems;             // two V^T tiles

  constexpr int BM = kAttnRowsPerWave * kAttnPPWaves;
  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int g = lane >> 5;
  const bool group_b = wave >= 4;

  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const bf16_t* __restrict__ Qh = Q + head_off;
  const bf16_t* __restrict__ Kh = K + head_off;
  const bf16_t* __restrict__ Vh = V + head_off;

  const int q0 = q_block * BM;
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
  float m_run = -__builtin_inff();
  float l_run = 0.f;

  const int n_tiles = CAUSAL ? (q0 + BM) / kAttnBN : S / kAttnBN;
  const int wave_last_tile = CAUSAL ? (q0 + wave * 32 + 31) / kAttnBN : n_tiles - 1;

  // staging registers: a K tile (group B) or a V tile (group A), 4 x 16 bytes per thread
  u32x4_t st[4];
  const int stid = tid & 255;
  const int k_row = stid >> 4;
  const int k_col = (stid & 15) * 8;
  const int v_kg = stid >> 4;
  const int v_dg = stid & 15;

  auto load_k = [&](int tile) {
    const bf16_t* kp = Kh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      st[u] = *reinterpret_cast<const u32x4_t*>(kp + static_cast<size_t>(k_row + 16 * u) * kAttnD + k_col);
  };
  auto store_k = [&](int buf) {
    bf16_t* Ks = Kbuf + buf * kAttnPPKElems;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      *reinterpret_cast<u32x4_t*>(Ks + (k_row + 16 * u) * kAttnKStride + k_col) = st[u];
  };
  auto load_v = [&](int tile) {
    const bf16_t* vp = Vh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      st[u] = *reinterpret_cast<const u32x4_t*>(vp + static_cast<size_t>(4 * v_kg + u) * kAttnD + 8 * v_dg);
  };
  auto store_v = [&](int buf) {
    bf16_t* Vt = Vbuf + buf * kAttnPPVElems;
    const int pos = attn_vt_pos(4 * v_kg);
#pragma unroll
    for (int e2 = 0; e2 < 4; ++e2) {
      const uint32_t a0 = st[0][e2], a1 = st[1][e2], a2 = st[2][e2], a3 = st[3][e2];
      u32x2_t lo, hi;
      lo[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100u);
      lo[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100u);
      hi[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302u);
      hi[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302u);
      *reinterpret_cast<u32x2_t*>(Vt + attn_vt_offset(8 * v_dg + 2 * e2, pos)) = lo;
      *reinterpret_cast<u32x2_t*>(Vt + attn_vt_offset(8 * v_dg + 2 * e2 + 1, pos)) = hi;
    }
  };

  f32x16_t sacc[2];
  bf16x8_t pf[2][2];

  auto qk = [&](int tile) {
    const bf16_t* Ks = Kbuf + (tile & 1) * kAttnPPKElems;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const bf16x8_t a =
            *reinterpret_cast<const bf16x8_t*>(Ks + (32 * kb + li) * kAttnKStride + 16 * s + 8 * g);
        sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[s], sacc[kb], 0, 0, 0);
      }
    }
  };
  auto pv = [&](int tile) {
    const bf16_t* Vt = Vbuf + (tile & 1) * kAttnPPVElems;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const bf16x8_t a =
            *reinterpret_cast<const bf16x8_t*>(Vt + attn_vt_offset(32 * db + li, 16 * t + 8 * g));
        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[t >> 1][t & 1], oacc[db], 0, 0, 0);
      }
    }
  };
  auto softmax = [&](int tile) {
    const int key0 = tile * kAttnBN;
    if (CAUSAL && key0 + kAttnBN - 1 > q0 + wave * 32) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = key0 + 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3);
          if (key > qi) sacc[kb][r] = -__builtin_inff();
        }
    }
    float mx = sacc[0][0];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, sacc[kb][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m_run, mx * scale_log2e);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    float psum = 0.f;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float p = __builtin_amdgcn_exp2f(fmaf(sacc[kb][r], scale_log2e, -m_new));
        psum += p;
        pf[kb][r >> 3][r & 7] = static_cast<bf16_t>(p);
      }
    l_run = fmaf(l_run, alpha, psum);
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) oacc[db][r] *= alpha;
    }
  };

  // prologue: K tile 0 in place, every load issued so far landed (0x0F70 = vmcnt(0))
  if (group_b) {
    load_k(0);
    store_k(0);
  }
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();

  if (!group_b) {
    for (int i = 0; i <= n_tiles; ++i) {
      // matrix phase
      if (i < n_tiles) load_v(i);
      __builtin_amdgcn_s_setprio(1);
      if (i >= 1 && i - 1 <= wave_last_tile) pv(i - 1);
      if (i < n_tiles && i <= wave_last_tile) qk(i);
      __builtin_amdgcn_s_setprio(0);
      __syncthreads();
      // vector phase
      if (i < n_tiles && i <= wave_last_tile) softmax(i);
      if (i < n_tiles) store_v(i & 1);
      __syncthreads();
    }
    __syncthreads();  // pairs with group B's extra first interval
  } else {
    if (n_tiles > 1) {
      load_k(1);
      store_k(1);
    }
    __syncthreads();
    for (int i = 0; i <= n_tiles; ++i) {
      if (i + 2 < n_tiles) load_k(i + 2);
      __builtin_amdgcn_s_setprio(1);
      if (i >= 1 && i - 1 <= wave_last_tile) pv(i - 1);
      if (i < n_tiles && i <= wave_last_tile) qk(i);
      __builtin_amdgcn_s_setprio(0);
      __syncthreads();
      if (i < n_tiles && i <= wave_last_tile) softmax(i);
      if (i + 2 < n_tiles) store_k(i & 1);
      __syncthreads();
    }
  }

  // epilogue: normalise, store O and the softmax statistics
  const float l_tot = l_run + __shfl_xor(l_run, 32, kWave);
  const float inv_l = 1.0f / l_tot;
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
    const float m_nat = m_run * 0.69314718055994530942f;
    Vec<float, 4> mv, lv;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      mv[e] = m_nat;
      lv[e] = l_tot;
    }
    store_vec<float, 4>(softmax_max + so, mv);
    store_vec<float, 4>(softmax_max + so + 4, mv);
    store_vec<float, 4>(softmax_sum + so, lv);
    store_vec<float, 4>(softmax_sum + so + 4, lv);
  }
}

}  // namespace mi
