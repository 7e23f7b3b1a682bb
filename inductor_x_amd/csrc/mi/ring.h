// Ring-attention merge step in one kernel: two partial attention results over disjoint key sets,
// each with the row maximum and row sum of its softmax, become the result over the union.
//
// Same mathematics and layouts as the reference's scenario and its hand-written kernel
// (reference test/npu_indexing/attn_cp_test.py:36-59,
// test/npu_indexing/written/attn_cp_triton_kernel_3d.py:15-82):
//     m      = max(prev_max, cur_max)                      element-wise on [B, N, S, 8] fp32
//     a, b   = prev_sum * exp(prev_max - m), cur_sum * exp(cur_max - m)
//     sum    = a + b
//     out    = prev_out * (a / sum)[..., 0] + cur_out * (b / sum)[..., 0]
// with the attention outputs laid out [S, B, H] (H = N * D; head n owns columns n D .. n D + D - 1)
// and the statistics [B, N, S, 8].  The two layouts run against each other: consecutive s are 32
// bytes apart in the statistics and a whole [B, H] row apart in the outputs.  A workgroup therefore
// owns a tile of ST consecutive s by NT consecutive heads: its statistics are NT runs of ST * 32
// bytes, read once by one thread per (s, head), and its outputs ST runs of NT * D elements.  The two
// scale factors of every (s, head) cross from the thread that computed them to the threads that
// stream that head's D columns through LDS; nothing but the operands and results touches memory.
#pragma once

#include "common.h"

namespace mi {

// maximum that passes a NaN on, as torch.maximum does
__device__ __forceinline__ float ring_max_nan(float a, float b) {
  return (a != a) ? a : ((b != b) ? b : fmaxf(a, b));
}

// T: element type of the attention outputs (bf16_t, f16_t or float); D: head dimension;
// ST: consecutive sequence positions per workgroup.  256 threads; a head's D columns are covered
// by TPR = D / VEC lanes of 16 bytes, so a workgroup spans NT = 256 / TPR heads.  Measured on MI355X
// at bf16 [8192, 1, 6144] with 48 heads (377 MB per call, replayed): ST = 8 with all eight rows of a
// thread in flight 58.3 us, ST = 4 60.0, ST = 16 62.6 (four rows in flight) / 70.1 (eight), ST = 32 74;
// requesting the first rows before the statistics are read costs 1 - 9 us in every shape.
// STREAM: loads and stores of the attention outputs carry the non-temporal hint (the caller
// sets it when the operands are larger than the memory-side cache can hold anyway).
template <typename T, int D, int ST, bool STREAM>
__device__ __forceinline__ void ring_forward_update(
    const T* __restrict__ prev_out, const float* __restrict__ prev_max, const float* __restrict__ prev_sum,
    const T* __restrict__ cur_out, const float* __restrict__ cur_max, const float* __restrict__ cur_sum,
    T* __restrict__ out, float* __restrict__ out_max, float* __restrict__ out_sum, int S, int B, int N,
    long long prev_n_stride, long long cur_n_stride) {
  constexpr int VEC = 16 / sizeof(T);
  constexpr int TPR = D / VEC;
  static_assert(D % VEC == 0 && TPR >= 1 && TPR <= 256 && 256 % TPR == 0, "head dimension must tile 256 threads");
  constexpr int NT = 256 / TPR;
  constexpr int PAIRS = ST * NT;
  __shared__ float scale_prev[PAIRS];
  __shared__ float scale_cur[PAIRS];

  const int s0 = blockIdx.x * ST;
  const int n0 = blockIdx.y * NT;
  const int b = blockIdx.z;
  const int tid = threadIdx.x;

  // output side of this thread: (head, 16-byte piece of its D columns), rows s0 .. s0 + ST - 1
  const int n_l = tid / TPR;
  const int n = n0 + n_l;
  const size_t H = static_cast<size_t>(N) * D;
  const size_t col = static_cast<size_t>(n) * D + static_cast<size_t>(tid % TPR) * VEC;
  constexpr int BATCH = ST % 8 == 0 ? 8 : (ST % 4 == 0 ? 4 : 1);  // rows whose loads are in flight together
  Vec<T, VEC> pv[BATCH], cv[BATCH];
  auto load_rows = [&](int r0) {
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int s = s0 + r0 + j;
      if (n < N && s < S) {
        const size_t off = (static_cast<size_t>(s) * B + b) * H + col;
        pv[j] = load_vec_hint<T, VEC, STREAM>(prev_out + off);
        cv[j] = load_vec_hint<T, VEC, STREAM>(cur_out + off);
      }
    }
  };

  // ---- statistics: one thread per (head, s), s fastest, eight fp32 per array ----
  for (int p = tid; p < PAIRS; p += 256) {
    const int pn_l = p / ST, s_l = p % ST;
    const int pn = n0 + pn_l, s = s0 + s_l;
    if (pn < N && s < S) {
      const size_t po = static_cast<size_t>(b * N + pn) * prev_n_stride + static_cast<size_t>(s) * 8;
      const size_t co = static_cast<size_t>(b * N + pn) * cur_n_stride + static_cast<size_t>(s) * 8;
      float sp = 0.f, sc = 0.f;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const Vec<float, 4> pm = load_vec<float, 4>(prev_max + po + 4 * h);
        const Vec<float, 4> cm = load_vec<float, 4>(cur_max + co + 4 * h);
        const Vec<float, 4> ps = load_vec<float, 4>(prev_sum + po + 4 * h);
        const Vec<float, 4> cs = load_vec<float, 4>(cur_sum + co + 4 * h);
        Vec<float, 4> m, tot;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          m[e] = ring_max_nan(pm[e], cm[e]);
          const float a = ps[e] * expf(pm[e] - m[e]);
          const float c = cs[e] * expf(cm[e] - m[e]);
          tot[e] = a + c;
          if (h == 0 && e == 0) {
            sp = a / tot[e];
            sc = c / tot[e];
          }
        }
        // the results take the layout (and head stride) of the current step's statistics
        store_vec<float, 4>(out_max + co + 4 * h, m);
        store_vec<float, 4>(out_sum + co + 4 * h, tot);
      }
      scale_prev[s_l * NT + pn_l] = sp;
      scale_cur[s_l * NT + pn_l] = sc;
    }
  }
  __syncthreads();

  // ---- outputs: BATCH rows at a time ----
  if (n >= N) return;
#pragma unroll
  for (int r0 = 0; r0 < ST; r0 += BATCH) {
    load_rows(r0);
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int s = s0 + r0 + j;
      if (s < S) {
        const float sp = scale_prev[(r0 + j) * NT + n_l];
        const float sc = scale_cur[(r0 + j) * NT + n_l];
        Vec<T, VEC> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o[e] = from_f32<T>(to_f32(pv[j][e]) * sp + to_f32(cv[j][e]) * sc);
        store_vec<T, VEC, true>(out + (static_cast<size_t>(s) * B + b) * H + col, o);
      }
    }
  }
}

}  // namespace mi
