// Fused attention forward for gfx950, bf16 in / bf16 out, fp32 softmax:
//   O = softmax(Q K^T * scale [+ causal mask]) V,   layout [B, N, S, D], D = 128.
// Also writes the per-row softmax maximum and sum ([B, N, S, 8] fp32, value
// repeated over the last axis), the two statistics the reference's fused
// attention op returns besides the output
// (reference inductor_x/npu_fusion_attention_graph.py:17-35,45-74).
//
// Mapping onto the matrix cores (v_mfma_f32_32x32x16_bf16, 64-lane wavefronts)
// -------------------------------------------------------------------------
// A workgroup is 4 or 8 wavefronts; a wavefront owns 32 consecutive queries, the
// workgroup 128 or 256.  Keys/values are visited in tiles of 64, staged in LDS and
// shared by the 4 wavefronts.  Both products are computed transposed so that a
// lane always works for ONE query (column n = lane % 32 of every accumulator):
//
//   S^T [key, query] = K [key, d] * Q^T [d, query]      A = K tile (LDS), B = Q (registers)
//   O^T [d,   query] = V^T [d, key] * P^T [key, query]  A = V^T tile (LDS), B = P^T (registers)
//
// With that choice the S^T accumulator a lane holds (16 keys x 1 query per
// 32-key block) is already the B operand of the second product, the running
// max / sum of a query live in the same lane as its scores and its output
// column, and rescaling O is a per-lane scalar multiply: no cross-lane traffic
// apart from one xor-32 shuffle for the row maximum.
//
// Operand layouts of the instruction (lane l, i = l % 32, g = l / 32):
//   A: row i,  k = 8 g + e   (e = 0..7, one 16-byte register group)
//   B: col i,  k = 8 g + e
//   C: col i,  row = 8 (r / 4) + 4 g + r % 4   (r = 0..15)
// The second product contracts over keys.  Its B operand (P^T) arrives in the C
// layout, i.e. element e of step (kb, h) is key 32 kb + 16 h + 8 (e / 4) + 4 g + e % 4.
// The V^T tile is therefore stored in LDS with its key axis permuted the same
// way (bits 2 and 3 of the key index swapped inside every group of 16), so the
// A operand is a single 16-byte LDS read (chunks are additionally XOR-swizzled
// against bank conflicts, see attn_vt_offset).  V arrives from memory as [key, d];
// the transposition happens in registers while the tile is copied to LDS
// (four keys x eight d per thread -> eight 8-byte LDS writes).
#pragma once

#include "common.h"

namespace mi {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

constexpr int kAttnD = 128;       // head dimension
constexpr int kAttnRowsPerWave = 32;  // queries per wavefront; a workgroup owns 32 * WAVES
constexpr int kAttnBN = 64;       // keys per tile
constexpr int kAttnKStride = 136; // bf16 per K row in LDS (128 + 8 pad, rows stay 16-byte aligned)
constexpr int kAttnVStride = 64;  // bf16 per V^T row in LDS (unpadded; 16-byte chunks are XOR-swizzled)

constexpr int kAttnTileElems = kAttnBN * kAttnKStride + kAttnD * kAttnVStride;  // one K + V^T tile
constexpr int kAttnLdsBytes = 2 * kAttnTileElems * 2;  // double-buffered

// Position of key j (0..63) on the permuted key axis of the V^T tile.
__device__ __forceinline__ int attn_vt_pos(int j) {
  return (j & ~12) | ((j & 4) << 1) | ((j & 8) >> 1);
}

// Element offset of (row d, permuted key position p) in the V^T tile.  Rows are
// 128 bytes = one pass over all LDS banks, so the eight 16-byte chunks of a row
// are XOR-swizzled with bits of d: the low three bits spread the rows that the
// lanes of one MFMA operand read (d = base + lane), bits 3..5 spread the rows
// that the lanes of one transposing write hit (d = 8 * lane + const).
__device__ __forceinline__ int attn_vt_offset(int d, int p) {
  const int chunk = (p >> 3) ^ ((d ^ (d >> 3)) & 7);
  return d * kAttnVStride + chunk * 8 + (p & 7);
}

template <bool CAUSAL, int WAVES>
__device__ __forceinline__ void attention_fwd_d128(const bf16_t* __restrict__ Q,
                                                   const bf16_t* __restrict__ K,
                                                   const bf16_t* __restrict__ V,
                                                   bf16_t* __restrict__ O,
                                                   float* __restrict__ softmax_max,
                                                   float* __restrict__ softmax_sum, int S,
                                                   int q_block, int head, float scale_log2e) {
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  bf16_t* lds_base = reinterpret_cast<bf16_t*>(attn_lds);

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int li = lane & 31;
  const int g = lane >> 5;

  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const bf16_t* __restrict__ Qh = Q + head_off;
  const bf16_t* __restrict__ Kh = K + head_off;
  const bf16_t* __restrict__ Vh = V + head_off;

  constexpr int BM = kAttnRowsPerWave * WAVES;  // queries per workgroup
  const int q0 = q_block * BM;
  const int qi = q0 + wave * 32 + li;  // this lane's query

  // Q fragments stay in registers for the whole kernel: 8 k-steps x 8 bf16.
  bf16x8_t qf[8];
#pragma unroll
  for (int s = 0; s < 8; ++s)
    qf[s] = *reinterpret_cast<const bf16x8_t*>(Qh + static_cast<size_t>(qi) * kAttnD + 16 * s + 8 * g);

  f32x16_t oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) oacc[db][r] = 0.f;
  float m_run = -__builtin_inff();  // running max, log2 domain
  float l_run = 0.f;                // running sum of this lane's half of the keys

  // Number of key tiles this workgroup visits, and the last one this wavefront needs.
  const int n_tiles = CAUSAL ? (q0 + BM) / kAttnBN : S / kAttnBN;
  const int wave_last_tile = CAUSAL ? (q0 + wave * 32 + 31) / kAttnBN : n_tiles - 1;

  // global -> register -> LDS staging of one K tile and one V tile.  With 4
  // wavefronts every thread moves 4 x 16 bytes of K and 4 x 16 bytes of V; with
  // 8 wavefronts the first four stage V and the last four stage K (the role is
  // uniform per wavefront, so there is no divergence).
  constexpr bool SPLIT = (WAVES == 8);
  static_assert(WAVES == 4 || WAVES == 8, "4 or 8 wavefronts per workgroup");
  const int stid = tid & 255;
  const bool do_k = SPLIT ? (tid >= 256) : true;
  const bool do_v = SPLIT ? (tid < 256) : true;
  u32x4_t kst[4], vst[4];
  const int k_row = stid >> 4;           // + 16 * u
  const int k_col = (stid & 15) * 8;
  const int v_kg = stid >> 4;            // keys 4 v_kg .. 4 v_kg + 3
  const int v_dg = stid & 15;            // d 8 v_dg .. 8 v_dg + 7
  auto load_tile = [&](int tile) {
    const bf16_t* kp = Kh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    const bf16_t* vp = Vh + static_cast<size_t>(tile) * kAttnBN * kAttnD;
    if (do_k) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        kst[u] = *reinterpret_cast<const u32x4_t*>(kp + static_cast<size_t>(k_row + 16 * u) * kAttnD + k_col);
    }
    if (do_v) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        vst[u] = *reinterpret_cast<const u32x4_t*>(vp + static_cast<size_t>(4 * v_kg + u) * kAttnD + 8 * v_dg);
    }
  };
  auto store_tile = [&](int buf) {
    bf16_t* Ks = lds_base + buf * kAttnTileElems;
    bf16_t* Vt = Ks + kAttnBN * kAttnKStride;
    if (do_k) {
#pragma unroll
      for (int u = 0; u < 4; ++u)
        *reinterpret_cast<u32x4_t*>(Ks + (k_row + 16 * u) * kAttnKStride + k_col) = kst[u];
    }
    if (do_v) {
      // 4 keys x 8 d  ->  8 rows (d) of 4 consecutive permuted key positions
      const int pos = attn_vt_pos(4 * v_kg);
#pragma unroll
      for (int e2 = 0; e2 < 4; ++e2) {
        // dword e2 of each staged row holds d = 2 e2 (low half) and 2 e2 + 1 (high half)
        const uint32_t a0 = vst[0][e2], a1 = vst[1][e2], a2 = vst[2][e2], a3 = vst[3][e2];
        u32x2_t lo, hi;
        // byte permutes: low halves of (a0, a1) / high halves of (a0, a1)
        lo[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100u);
        lo[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100u);
        hi[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302u);
        hi[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302u);
        *reinterpret_cast<u32x2_t*>(Vt + attn_vt_offset(8 * v_dg + 2 * e2, pos)) = lo;
        *reinterpret_cast<u32x2_t*>(Vt + attn_vt_offset(8 * v_dg + 2 * e2 + 1, pos)) = hi;
      }
    }
  };

  // Two LDS buffers: while the math runs on one, the next tile travels
  // global -> registers -> the other buffer; one barrier per tile.
  load_tile(0);
  store_tile(0);
  // Every load issued so far (Q fragments included) must have landed before
  // the loop: otherwise the waits for Q would be placed inside the loop, where
  // they would also wait for each tile's prefetch.  0x0F70 = vmcnt(0) only.
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  for (int tile = 0; tile < n_tiles; ++tile) {
    const bf16_t* Ks = lds_base + (tile & 1) * kAttnTileElems;
    const bf16_t* Vt = Ks + kAttnBN * kAttnKStride;
    if (tile + 1 < n_tiles) load_tile(tile + 1);  // in flight during the math below

    if (tile <= wave_last_tile) {
      // ---- S^T = K Q^T : 2 blocks of 32 keys x 8 k-steps
      f32x16_t sacc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) sacc[kb][r] = 0.f;
      // the two key blocks are independent accumulation chains: alternate them
#pragma unroll
      for (int s = 0; s < 8; ++s) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          const bf16x8_t a =
              *reinterpret_cast<const bf16x8_t*>(Ks + (32 * kb + li) * kAttnKStride + 16 * s + 8 * g);
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[s], sacc[kb], 0, 0, 0);
        }
      }

      // ---- causal mask (only tiles that straddle the diagonal need it)
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

      // ---- online softmax, log2 domain
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
      bf16x8_t pf[2][2];
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

      // ---- O^T += V^T P^T : 4 blocks of 32 d x 4 k-steps of 16 keys
#pragma unroll
      for (int t = 0; t < 4; ++t) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const bf16x8_t a =
              *reinterpret_cast<const bf16x8_t*>(Vt + attn_vt_offset(32 * db + li, 16 * t + 8 * g));
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[t >> 1][t & 1], oacc[db], 0, 0, 0);
        }
      }
    }
    if (tile + 1 < n_tiles) store_tile((tile + 1) & 1);
    __syncthreads();  // next tile visible; this tile's buffer free for the tile after next
  }

  // ---- epilogue: normalise, store O and the softmax statistics
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
