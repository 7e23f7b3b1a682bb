// Fused attention backward (bf16, head dimension 128), two kernels, no atomics.
//
// With P = exp(S - m) / l recomputed from the forward's row statistics (S = Q K^T * scale,
// m = row maximum, l = row sum), D = rowsum(dO * O) and dS = P * (dO V^T - D) * scale:
//     dV = P^T dO        dK = dS^T Q        dQ = dS K
// Same MFMA (v_mfma_f32_32x32x16_bf16), LDS tile formats and transposing copies as the forward
// (attention.h).  Every product is arranged so that the accumulator layout of one MFMA is
// directly the B operand of the next:
//
//   dQ kernel   a wavefront owns 32 queries (lane = query), loops over key tiles:
//               S^T = K Q^T, dP^T = V dO^T  (A from LDS, B = Q / dO fragments in registers),
//               dS^T as B operand,  dQ^T += K^T dS^T  (A = transposed K tile).
//   dKV kernel  a wavefront owns 32 keys (lane = key), loops over query tiles:
//               S = Q K^T, dP = dO V^T  (A from LDS, B = K / V fragments in registers),
//               P and dS as B operands,  dV^T += dO^T P,  dK^T += Q^T dS
//               (A = transposed dO / Q tiles, query axis permuted as attn_vt_pos).
//               Row statistics of the query tile (m, 1/l, D) come through LDS.
//
// The scores are recomputed once per kernel (7 matrix products in total instead of 5), which
// buys independence of the two kernels and reproducible results.
#pragma once

#include "attention_v2.h"

namespace mi {

constexpr int kBwdRowTile = kAttnBN * kAttnKStride;  // [64][136] row-major tile, elements
constexpr int kBwdColTile = kAttnD * kAttnVStride;   // [128][64] transposed tile, elements
constexpr int kBwdDqBufElems = 2 * kBwdRowTile + kBwdColTile;       // K, V, K^T
constexpr int kBwdDqLdsBytes = 2 * kBwdDqBufElems * 2;
constexpr int kBwdDkvStatFloats = 3 * kAttnBN;                      // m, 1/l, D of a query tile
constexpr int kBwdDkvBufBytes = (2 * kBwdRowTile + 2 * kBwdColTile) * 2 + kBwdDkvStatFloats * 4;
constexpr int kBwdDkvLdsBytes = 2 * kBwdDkvBufBytes;
constexpr float kLog2e = 1.4426950408889634f;

// delta[h, q] = sum_d dO[h, q, d] * O[h, q, d]; 16 lanes per row, 8 elements each.
__device__ __forceinline__ void attention_bwd_delta(const bf16_t* __restrict__ O, const bf16_t* __restrict__ dO,
                                                    float* __restrict__ delta, int rows) {
  const int row = (blockIdx.x * blockDim.x + threadIdx.x) >> 4;
  const int part = threadIdx.x & 15;
  float acc = 0.f;
  if (row < rows) {
    const bf16x8_t o = *reinterpret_cast<const bf16x8_t*>(O + static_cast<size_t>(row) * kAttnD + 8 * part);
    const bf16x8_t d = *reinterpret_cast<const bf16x8_t*>(dO + static_cast<size_t>(row) * kAttnD + 8 * part);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc = fmaf(static_cast<float>(o[e]), static_cast<float>(d[e]), acc);
  }
#pragma unroll
  for (int off = 8; off >= 1; off >>= 1) acc += __shfl_xor(acc, off, kWave);
  if (row < rows && part == 0) delta[row] = acc;
}

// Copies shared by both kernels: a [64][128] bf16 tile travels global -> registers (every one of
// 256 threads: 4 rows x 8 columns) -> LDS, row-major and / or transposed.
struct BwdTileRegs {
  u32x4_t r[4];
};
__device__ __forceinline__ void bwd_tile_load(BwdTileRegs& t, const bf16_t* __restrict__ src, int tid) {
  const int rg = tid >> 4, cg = tid & 15;
#pragma unroll
  for (int u = 0; u < 4; ++u)
    t.r[u] = *reinterpret_cast<const u32x4_t*>(src + static_cast<size_t>(4 * rg + u) * kAttnD + 8 * cg);
}
__device__ __forceinline__ void bwd_tile_store_rows(const BwdTileRegs& t, bf16_t* dst, int tid) {
  const int rg = tid >> 4, cg = tid & 15;
#pragma unroll
  for (int u = 0; u < 4; ++u) *reinterpret_cast<u32x4_t*>(dst + (4 * rg + u) * kAttnKStride + 8 * cg) = t.r[u];
}
// transposed, the row index (the contraction axis of the MFMA that reads the tile) permuted
__device__ __forceinline__ void bwd_tile_store_cols(const BwdTileRegs& t, bf16_t* dst, int tid) {
  const int rg = tid >> 4, cg = tid & 15;
  const int pos = attn_vt_pos(4 * rg);
#pragma unroll
  for (int e2 = 0; e2 < 4; ++e2) {
    const uint32_t a0 = t.r[0][e2], a1 = t.r[1][e2], a2 = t.r[2][e2], a3 = t.r[3][e2];
    u32x2_t lo, hi;
    lo[0] = __builtin_amdgcn_perm(a1, a0, 0x05040100u);
    lo[1] = __builtin_amdgcn_perm(a3, a2, 0x05040100u);
    hi[0] = __builtin_amdgcn_perm(a1, a0, 0x07060302u);
    hi[1] = __builtin_amdgcn_perm(a3, a2, 0x07060302u);
    *reinterpret_cast<u32x2_t*>(dst + attn_vt_offset(8 * cg + 2 * e2, pos)) = lo;
    *reinterpret_cast<u32x2_t*>(dst + attn_vt_offset(8 * cg + 2 * e2 + 1, pos)) = hi;
  }
}
__device__ __forceinline__ bf16x8_t bwd_row_frag(const bf16_t* tile, int row, int s, int g) {
  return *reinterpret_cast<const bf16x8_t*>(tile + row * kAttnKStride + 16 * s + 8 * g);
}
__device__ __forceinline__ bf16x8_t bwd_col_frag(const bf16_t* tile, int row, int t, int g) {
  return *reinterpret_cast<const bf16x8_t*>(tile + attn_vt_offset(row, 16 * t + 8 * g));
}
__device__ __forceinline__ void bwd_store_acc_rows(bf16_t* __restrict__ dst_row, const f32x16_t (&acc)[4], int g) {
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int rq = 0; rq < 4; ++rq) {
      bf16x4_t o4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o4[e] = static_cast<bf16_t>(acc[db][4 * rq + e]);
      *reinterpret_cast<bf16x4_t*>(dst_row + 32 * db + 8 * rq + 4 * g) = o4;
    }
}

// ---------------------------------------------------------------------------------------------
// dQ: 4 wavefronts, 128 queries per workgroup
// ---------------------------------------------------------------------------------------------
template <bool CAUSAL>
__device__ __forceinline__ void attention_bwd_dq(const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K,
                                                 const bf16_t* __restrict__ V, const bf16_t* __restrict__ O,
                                                 const bf16_t* __restrict__ dO,
                                                 const float* __restrict__ softmax_max,
                                                 const float* __restrict__ softmax_sum,
                                                 bf16_t* __restrict__ dQ, int S, int q_block, int head,
                                                 float scale) {
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  bf16_t* lds = reinterpret_cast<bf16_t*>(attn_lds);
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const bf16_t* __restrict__ Kh = K + head_off;
  const bf16_t* __restrict__ Vh = V + head_off;
  constexpr int BM = 128;
  const int q0 = q_block * BM;
  const int qi = q0 + wave * 32 + li;
  const size_t qrow = head_off + static_cast<size_t>(qi) * kAttnD;

  bf16x8_t qf[8], dof[8];
  float dpart = 0.f;
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    qf[s] = *reinterpret_cast<const bf16x8_t*>(Q + qrow + 16 * s + 8 * g);
    dof[s] = *reinterpret_cast<const bf16x8_t*>(dO + qrow + 16 * s + 8 * g);
    const bf16x8_t of = *reinterpret_cast<const bf16x8_t*>(O + qrow + 16 * s + 8 * g);
#pragma unroll
    for (int e = 0; e < 8; ++e) dpart = fmaf(static_cast<float>(dof[s][e]), static_cast<float>(of[e]), dpart);
  }
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(dpart), __float_as_uint(dpart), false, false);
  const float delta = __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
  const size_t so = (static_cast<size_t>(head) * S + qi) * 8;
  const float m2 = softmax_max[so] * kLog2e;
  const float linv = 1.0f / softmax_sum[so];
  const float c2 = scale * kLog2e;

  f32x16_t acc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[db][r] = 0.f;

  const int n_tiles = CAUSAL ? (q0 + BM) / kAttnBN : S / kAttnBN;
  const int wave_last_tile = CAUSAL ? (q0 + wave * 32 + 31) / kAttnBN : n_tiles - 1;

  BwdTileRegs kt, vt;
  auto load_tile = [&](int tile) {
    bwd_tile_load(kt, Kh + static_cast<size_t>(tile) * kAttnBN * kAttnD, tid);
    bwd_tile_load(vt, Vh + static_cast<size_t>(tile) * kAttnBN * kAttnD, tid);
  };
  auto store_tile = [&](int buf) {
    bf16_t* Ks = lds + buf * kBwdDqBufElems;
    bwd_tile_store_rows(kt, Ks, tid);
    bwd_tile_store_rows(vt, Ks + kBwdRowTile, tid);
    bwd_tile_store_cols(kt, Ks + 2 * kBwdRowTile, tid);
  };

  load_tile(0);
  store_tile(0);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  for (int tile = 0; tile < n_tiles; ++tile) {
    const bf16_t* Ks = lds + (tile & 1) * kBwdDqBufElems;
    const bf16_t* Vs = Ks + kBwdRowTile;
    const bf16_t* Kt = Ks + 2 * kBwdRowTile;
    if (tile + 1 < n_tiles) load_tile(tile + 1);

    if (tile <= wave_last_tile) {
      f32x16_t sacc[2], pacc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sacc[kb][r] = 0.f;
          pacc[kb][r] = 0.f;
        }
#pragma unroll
      for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) {
          sacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_row_frag(Ks, 32 * kb + li, s, g), qf[s], sacc[kb], 0, 0, 0);
          pacc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_row_frag(Vs, 32 * kb + li, s, g), dof[s], pacc[kb], 0, 0, 0);
        }
      const int key0 = tile * kAttnBN;
      const bool diag = CAUSAL && key0 + kAttnBN - 1 > q0 + wave * 32;
      bf16x8_t dsf[2][2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float p = __builtin_amdgcn_exp2f(fmaf(sacc[kb][r], c2, -m2)) * linv;
          if (diag && key0 + 32 * kb + 8 * (r >> 2) + 4 * g + (r & 3) > qi) p = 0.f;
          dsf[kb][r >> 3][r & 7] = static_cast<bf16_t>(p * (pacc[kb][r] - delta) * scale);
        }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int db = 0; db < 4; ++db)
          acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_col_frag(Kt, 32 * db + li, t, g), dsf[t >> 1][t & 1], acc[db], 0, 0, 0);
    }
    if (tile + 1 < n_tiles) store_tile((tile + 1) & 1);
    __syncthreads();
  }
  bwd_store_acc_rows(dQ + qrow, acc, g);
}

// ---------------------------------------------------------------------------------------------
// dK, dV: 4 wavefronts, 128 keys per workgroup
// ---------------------------------------------------------------------------------------------
template <bool CAUSAL>
__device__ __forceinline__ void attention_bwd_dkv(const bf16_t* __restrict__ Q, const bf16_t* __restrict__ K,
                                                  const bf16_t* __restrict__ V, const bf16_t* __restrict__ dO,
                                                  const float* __restrict__ softmax_max,
                                                  const float* __restrict__ softmax_sum,
                                                  const float* __restrict__ delta, bf16_t* __restrict__ dK,
                                                  bf16_t* __restrict__ dV, int S, int k_block, int head,
                                                  float scale) {
  extern __shared__ __attribute__((aligned(16))) unsigned char attn_lds[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, li = lane & 31, g = lane >> 5;
  const size_t head_off = static_cast<size_t>(head) * S * kAttnD;
  const bf16_t* __restrict__ Qh = Q + head_off;
  const bf16_t* __restrict__ dOh = dO + head_off;
  constexpr int BK = 128;
  const int k0 = k_block * BK;
  const int kw = k0 + wave * 32;  // first key of this wavefront
  const int kj = kw + li;
  const size_t krow = head_off + static_cast<size_t>(kj) * kAttnD;

  bf16x8_t kf[8], vf[8];
#pragma unroll
  for (int s = 0; s < 8; ++s) {
    kf[s] = *reinterpret_cast<const bf16x8_t*>(K + krow + 16 * s + 8 * g);
    vf[s] = *reinterpret_cast<const bf16x8_t*>(V + krow + 16 * s + 8 * g);
  }
  f32x16_t dkacc[4], dvacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      dkacc[db][r] = 0.f;
      dvacc[db][r] = 0.f;
    }
  const float c2 = scale * kLog2e;

  const int n_qtiles = S / kAttnBN;
  const int first_tile = CAUSAL ? k0 / kAttnBN : 0;           // first query tile that sees a key of the block
  const int wave_first_tile = CAUSAL ? kw / kAttnBN : 0;

  auto buf_rows = [&](int buf) { return reinterpret_cast<bf16_t*>(attn_lds + buf * kBwdDkvBufBytes); };
  auto buf_stats = [&](int buf) {
    return reinterpret_cast<float*>(attn_lds + buf * kBwdDkvBufBytes + (2 * kBwdRowTile + 2 * kBwdColTile) * 2);
  };
  BwdTileRegs qt, dt;
  float st_m = 0.f, st_l = 1.f, st_d = 0.f;
  auto load_tile = [&](int tile) {
    bwd_tile_load(qt, Qh + static_cast<size_t>(tile) * kAttnBN * kAttnD, tid);
    bwd_tile_load(dt, dOh + static_cast<size_t>(tile) * kAttnBN * kAttnD, tid);
    if (tid < kAttnBN) {
      const size_t row = static_cast<size_t>(head) * S + tile * kAttnBN + tid;
      st_m = softmax_max[row * 8];
      st_l = softmax_sum[row * 8];
      st_d = delta[row];
    }
  };
  auto store_tile = [&](int buf) {
    bf16_t* Qs = buf_rows(buf);
    bwd_tile_store_rows(qt, Qs, tid);
    bwd_tile_store_rows(dt, Qs + kBwdRowTile, tid);
    bwd_tile_store_cols(qt, Qs + 2 * kBwdRowTile, tid);
    bwd_tile_store_cols(dt, Qs + 2 * kBwdRowTile + kBwdColTile, tid);
    if (tid < kAttnBN) {
      float* st = buf_stats(buf);
      st[tid] = st_m * kLog2e;
      st[kAttnBN + tid] = 1.0f / st_l;
      st[2 * kAttnBN + tid] = st_d;
    }
  };

  load_tile(first_tile);
  store_tile(first_tile & 1);
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  for (int tile = first_tile; tile < n_qtiles; ++tile) {
    const bf16_t* Qs = buf_rows(tile & 1);
    const bf16_t* dOs = Qs + kBwdRowTile;
    const bf16_t* Qt = Qs + 2 * kBwdRowTile;
    const bf16_t* dOt = Qt + kBwdColTile;
    const float* st = buf_stats(tile & 1);
    if (tile + 1 < n_qtiles) load_tile(tile + 1);

    if (tile >= wave_first_tile) {
      const int q0t = tile * kAttnBN;
      const bool diag = CAUSAL && q0t < kw + 31;
      bf16x8_t pf[2][2], dsf[2][2];  // [query block][half]: B operands, contraction over the queries
#pragma unroll
      for (int qb = 0; qb < 2; ++qb) {
        f32x16_t sacc, pacc;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          sacc[r] = 0.f;
          pacc[r] = 0.f;
        }
#pragma unroll
        for (int s = 0; s < 8; ++s) {
          sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_row_frag(Qs, 32 * qb + li, s, g), kf[s], sacc, 0, 0, 0);
          pacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_row_frag(dOs, 32 * qb + li, s, g), vf[s], pacc, 0, 0, 0);
        }
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          // rows 32 qb + 8 rq + 4 g + (0..3) of the query tile: their statistics
          const int row0 = 32 * qb + 8 * rq + 4 * g;
          const Vec<float, 4> mv = load_vec<float, 4>(st + row0);
          const Vec<float, 4> lv = load_vec<float, 4>(st + kAttnBN + row0);
          const Vec<float, 4> dv = load_vec<float, 4>(st + 2 * kAttnBN + row0);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int r = 4 * rq + e;
            float p = __builtin_amdgcn_exp2f(fmaf(sacc[r], c2, -mv[e])) * lv[e];
            if (diag && kj > q0t + row0 + e) p = 0.f;
            pf[qb][r >> 3][r & 7] = static_cast<bf16_t>(p);
            dsf[qb][r >> 3][r & 7] = static_cast<bf16_t>(p * (pacc[r] - dv[e]) * scale);
          }
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          dvacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_col_frag(dOt, 32 * db + li, t, g), pf[t >> 1][t & 1], dvacc[db], 0, 0, 0);
          dkacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bwd_col_frag(Qt, 32 * db + li, t, g), dsf[t >> 1][t & 1], dkacc[db], 0, 0, 0);
        }
    }
    if (tile + 1 < n_qtiles) store_tile((tile + 1) & 1);
    __syncthreads();
  }
  bwd_store_acc_rows(dK + krow, dkacc, g);
  bwd_store_acc_rows(dV + krow, dvacc, g);
}

}  // namespace mi
