// Column ("higher-order") reductions: the reduced axis is the strided outer
// axis and the kept axis is contiguous
// (reference inductor_x/codegen/triton.py:1003-1031 for the classification,
// reference inductor_x/codegen/split_tiling.py:159-165 for the case this file
// is built for: a reduced axis longer than 32768 that has to be cut across
// cores).
//
// Two-pass workgroup-partial scheme, no atomics:
//   pass 1  grid (column tiles, SPLITS).  A workgroup owns CT*4 columns and
//           every SPLITS-th batch of rows; thread (ct, rl) walks rows rl, rl+RL,
//           ... of a batch with float4 loads, so a wavefront reads 1 KiB runs.  Row
//           lanes are folded through LDS and one partial per (split, column)
//           goes to a workspace.
//   pass 2  folds the SPLITS partials of each column.
// One sweep produces mean, variance and argmax together, so the input is read
// from HBM exactly once.
//
// Variance: each thread accumulates sums of (x - c) and (x - c)^2 with c its
// first sample, turns them into (n, mean, M2) and every further merge uses
// Chan's formula.  That is the two-pass definition the reference lowers to
// (reference inductor_x/lowering.py:270-293) computed without a second read.
// Argmax follows maximum_with_index: greater wins, NaN beats numbers, ties keep
// the lower row (reference inductor_x/codegen/triton.py:1217-1233).
#pragma once

#include "common.h"

namespace mi {

constexpr int kColFields = 5;  // state words folded through LDS: n, mean, m2, best value, best row (int bits)
constexpr int kColPartWords = 4;  // words per (split, column) in the workspace: mean, m2, best value, best row

// Rows that split `split` owns when batches of `batch` rows are dealt out round-robin over
// `nsplit` splits (batch b to split b % nsplit, the last, partly filled batch included).  The
// count is a function of the launch geometry alone, so the partials do not carry it.
__device__ __forceinline__ int col_split_rows(int rows, int nsplit, int batch, int split) {
  const int full = rows / batch;
  int n = full > split ? ((full - 1 - split) / nsplit + 1) * batch : 0;
  if (full % nsplit == split) n += rows - full * batch;
  return n;
}

struct ColState {
  Moments m;
  ArgVal a;
};

__device__ __forceinline__ ColState col_state_empty() {
  ColState s;
  s.m.n = 0.f;
  s.m.mean = 0.f;
  s.m.m2 = 0.f;
  s.a.v = -__builtin_inff();
  s.a.i = 0x7fffffff;
  return s;
}

__device__ __forceinline__ ColState col_state_combine(const ColState& a, const ColState& b) {
  ColState r;
  r.m = moments_combine(a.m, b.m);
  r.a = arg_combine<true>(a.a, b.a);
  return r;
}

// True when a later row's value x must replace the running best: x is greater,
// or x is NaN while best is not.  !(x <= best) covers "greater or unordered";
// the second term keeps a NaN best in place.  Written with bitwise operators so
// it compiles to two compares and a mask AND instead of branches.
__device__ __forceinline__ bool col_argmax_update(float x, float best) {
  return static_cast<bool>(static_cast<int>(!(x <= best)) & static_cast<int>(best == best));
}

// Fold the RL row lanes of a workgroup (thread = rl * CT + ct).  On return the threads with
// rl == 0 hold the result.  Row lanes that share a wavefront (CT < 64) meet through lane
// exchanges; what is left, GROUPS = RL / (row lanes per wavefront) states per column in different
// wavefronts, is halved through LDS while more than four remain and then collected by row lane 0
// in one round: a 32 x 8 workgroup needs one exchange and one barrier.  lds holds
// col_fold_planes(CT, RL) * CT * 4 * kColFields floats (the host computes the same number).
__host__ __device__ constexpr int col_fold_in_wave(int ct, int rl) {
  return ct < kWave ? (kWave / ct < rl ? kWave / ct : rl) : 1;
}
__host__ __device__ constexpr int col_fold_planes(int ct, int rl) {
  const int groups = rl / col_fold_in_wave(ct, rl);
  if (groups <= 1) return 0;
  const int tree = groups > 4 ? groups / 2 : 0;
  const int last = (groups < 4 ? groups : 4) - 1;
  return tree > last ? tree : last;
}

__device__ __forceinline__ void col_state_put(float* lds, int plane, int slot, const ColState (&st)[4]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    lds[0 * plane + slot + k] = st[k].m.n;
    lds[1 * plane + slot + k] = st[k].m.mean;
    lds[2 * plane + slot + k] = st[k].m.m2;
    lds[3 * plane + slot + k] = st[k].a.v;
    lds[4 * plane + slot + k] = __int_as_float(st[k].a.i);
  }
}
__device__ __forceinline__ void col_state_take(const float* lds, int plane, int slot, ColState (&st)[4]) {
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    ColState o;
    o.m.n = lds[0 * plane + slot + k];
    o.m.mean = lds[1 * plane + slot + k];
    o.m.m2 = lds[2 * plane + slot + k];
    o.a.v = lds[3 * plane + slot + k];
    o.a.i = __float_as_int(lds[4 * plane + slot + k]);
    st[k] = col_state_combine(st[k], o);
  }
}

template <int CT, int RL>
__device__ __forceinline__ void col_fold_row_lanes(ColState (&st)[4], int ct, int rl, float* lds) {
  if constexpr (RL > 1) {
    constexpr int IN_WAVE = col_fold_in_wave(CT, RL);
    constexpr int GROUPS = RL / IN_WAVE;
    constexpr int PLANE = col_fold_planes(CT, RL) * CT * 4;
#pragma unroll
    for (int off = CT; off < CT * IN_WAVE; off <<= 1) {
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        ColState o;
        o.m.n = __shfl_xor(st[k].m.n, off, kWave);
        o.m.mean = __shfl_xor(st[k].m.mean, off, kWave);
        o.m.m2 = __shfl_xor(st[k].m.m2, off, kWave);
        o.a.v = __shfl_xor(st[k].a.v, off, kWave);
        o.a.i = __shfl_xor(st[k].a.i, off, kWave);
        st[k] = col_state_combine(st[k], o);
      }
    }
    if constexpr (GROUPS > 1) {
      const int grp = rl / IN_WAVE;
      const bool lead = rl % IN_WAVE == 0;
      int left = GROUPS;
#pragma unroll
      for (int half = GROUPS / 2; half >= 4; half >>= 1) {
        if (lead && grp >= half && grp < 2 * half) col_state_put(lds, PLANE, ((grp - half) * CT + ct) * 4, st);
        __syncthreads();
        if (lead && grp < half) col_state_take(lds, PLANE, (grp * CT + ct) * 4, st);
        __syncthreads();
        left = half;
      }
      // at most four groups are left
      if (lead && grp >= 1 && grp < left) col_state_put(lds, PLANE, ((grp - 1) * CT + ct) * 4, st);
      __syncthreads();
      if (rl == 0) {
        for (int g2 = 1; g2 < left; ++g2) col_state_take(lds, PLANE, ((g2 - 1) * CT + ct) * 4, st);
      }
    }
  }
}

// Pass 1.  Requires cols % 4 == 0 and x 16-byte aligned (checked by the host).
// part is [kColPartWords][nsplit][cols] floats (mean, M2, best value, best row; the row count
// of a split follows from the geometry, col_split_rows).  Rows are dealt out in batches of
// RL * UNROLL consecutive rows, batch b going to split b % nsplit: at any moment
// the nsplit workgroups of a column tile read one contiguous stretch of
// nsplit * RL * UNROLL rows.  Measured on MI355X at [65536, 512] against one
// contiguous slice of rows per workgroup: 27.2 us against 28.6 us for both passes,
// and half as many workgroups (each with twice the loads in flight) do as well,
// which halves the partials the second pass reads.
template <int CT, int RL, int UNROLL, int PF = 2>
__device__ __forceinline__ void col_stats_sweep(const float* __restrict__ x, int rows, int cols,
                                                int nsplit, ColState (&st)[4], float* lds_dyn) {
  constexpr int BATCH = RL * UNROLL;
  const int ct = threadIdx.x % CT;
  const int rl = threadIdx.x / CT;
  const int col = (blockIdx.x * CT + ct) * 4;
  const int split = blockIdx.y;
  const bool live = col < cols;
  const int full = rows / BATCH;  // batches with all their rows present

#pragma unroll
  for (int k = 0; k < 4; ++k) st[k] = col_state_empty();

  const int r0 = split * BATCH + rl;
  if (live && r0 < rows) {
    const float* __restrict__ base = x + static_cast<size_t>(rl) * cols + col;
    const size_t row_step = static_cast<size_t>(RL) * cols;
    const size_t batch_step = static_cast<size_t>(BATCH) * cols;
    // The first sample is the shift of the sums and the first candidate; the sweep
    // below meets it again, where it adds zero and never replaces itself.
    const Vec<float, 4> first = load_vec<float, 4, true>(base + split * batch_step);
    float c[4], s1[4], s2[4], best[4];
    int bi[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      c[k] = first[k];
      s1[k] = 0.f;
      s2[k] = 0.f;
      best[k] = first[k];
      bi[k] = r0;
    }
    int cnt = 0;
    int b = split;
    // PF batches of UNROLL rows each are held per thread: while one is folded, the loads of the
    // other PF - 1 are in flight (buffer j is refilled with the batch PF turns ahead as soon as
    // its values have been used, so the order of rows a thread sees stays increasing).
    Vec<float, 4> v[PF][UNROLL];
#pragma unroll
    for (int j = 0; j < PF; ++j) {
      if (b + j * nsplit < full) {
#pragma unroll
        for (int u = 0; u < UNROLL; ++u)
          v[j][u] = load_vec_readonly<float, 4>(base + (b + j * nsplit) * batch_step + u * row_step);
      }
    }
    while (b < full) {
#pragma unroll
      for (int j = 0; j < PF; ++j) {
        if (b < full) {
          const int r = b * BATCH + rl;
#pragma unroll
          for (int u = 0; u < UNROLL; ++u) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
              const float xv = v[j][u][k];
              const float d = xv - c[k];
              s1[k] += d;
              s2[k] = fmaf(d, d, s2[k]);
              const bool upd = xv > best[k];
              best[k] = upd ? xv : best[k];
              bi[k] = upd ? (r + u * RL) : bi[k];
            }
          }
          cnt += UNROLL;
          const int bn = b + PF * nsplit;
          if (bn < full) {
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) v[j][u] = load_vec_readonly<float, 4>(base + bn * batch_step + u * row_step);
          }
          b += nsplit;
        }
      }
    }
    // the last, partly filled batch belongs to workgroup full % nsplit
    if (b == full) {
      for (int r = full * BATCH + rl; r < rows; r += RL) {
        const Vec<float, 4> t = load_vec<float, 4, true>(x + static_cast<size_t>(r) * cols + col);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const float xv = t[k];
          const float d = xv - c[k];
          s1[k] += d;
          s2[k] = fmaf(d, d, s2[k]);
          const bool upd = xv > best[k];
          best[k] = upd ? xv : best[k];
          bi[k] = upd ? r : bi[k];
        }
        cnt += 1;
      }
    }
    // NaN samples are skipped by the plain "greater" above; they (and +inf meeting
    // -inf) leave a NaN in the shifted sum, which sends the column through the full
    // rule once more: NaN beats numbers, the first NaN wins.
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if (s1[k] != s1[k]) {
        float bv = first[k];
        int bidx = r0;
        for (int bb = split; bb * BATCH < rows; bb += nsplit) {
          for (int r = bb * BATCH + rl; r < min(rows, (bb + 1) * BATCH); r += RL) {
            const float xv = x[static_cast<size_t>(r) * cols + col + k];
            const bool upd = col_argmax_update(xv, bv);
            bv = upd ? xv : bv;
            bidx = upd ? r : bidx;
          }
        }
        best[k] = bv;
        bi[k] = bidx;
      }
    }
    const float n = static_cast<float>(cnt);
    const float inv_n = 1.0f / n;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      st[k].m.n = n;
      st[k].m.mean = c[k] + s1[k] * inv_n;
      const float m2 = s2[k] - s1[k] * s1[k] * inv_n;
      st[k].m.m2 = (m2 < 0.f) ? 0.f : m2;
      st[k].a.v = best[k];
      st[k].a.i = bi[k];
    }
  }

  col_fold_row_lanes<CT, RL>(st, ct, rl, lds_dyn);
}

// Pass 1 of the two-launch form: sweep, then one plain partial per (split, column).
template <int CT, int RL, int UNROLL, int PF = 2>
__device__ __forceinline__ void col_stats_partial(const float* __restrict__ x,
                                                         float* __restrict__ part, int rows,
                                                         int cols, int nsplit) {
  extern __shared__ float lds_dyn[];
  ColState st[4];
  col_stats_sweep<CT, RL, UNROLL, PF>(x, rows, cols, nsplit, st, lds_dyn);
  const int ct = threadIdx.x % CT;
  const int rl = threadIdx.x / CT;
  const int col = (blockIdx.x * CT + ct) * 4;
  const int split = blockIdx.y;
  if (col < cols && rl == 0) {
    const size_t plane = static_cast<size_t>(nsplit) * cols;
    const size_t o = static_cast<size_t>(split) * cols + col;
    Vec<float, 4> f1, f2, f3, f4;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      f1[k] = st[k].m.mean;
      f2[k] = st[k].m.m2;
      f3[k] = st[k].a.v;
      f4[k] = __int_as_float(st[k].a.i);
    }
    store_vec<float, 4>(part + 0 * plane + o, f1);
    store_vec<float, 4>(part + 1 * plane + o, f2);
    store_vec<float, 4>(part + 2 * plane + o, f3);
    store_vec<float, 4>(part + 3 * plane + o, f4);
  }
}

// Pass 2.  A workgroup of CPW * SL threads finishes CPW columns (CPW a power of two <= 64,
// CPW * SL a multiple of 64); thread (c, sl), c fastest, folds splits sl, sl + SL, ... in
// increasing order.  Every partial word a thread needs is requested before the first one is
// used (BATCH splits at a time), the split lanes of a wavefront then meet through lane
// exchanges and the wavefronts through one round of LDS: the pass is a chain of one memory
// round trip, log2(64 / CPW) exchanges and one barrier.  `batch` is the first pass's
// RL * UNROLL, from which the row count of each split follows.
template <int CPW, int SL, int BATCH = 4>
__device__ __forceinline__ void col_stats_final(const float* __restrict__ part,
                                                float* __restrict__ mean_out,
                                                float* __restrict__ var_out,
                                                long long* __restrict__ argmax_out, int cols,
                                                int nsplit, int rows, int batch, float correction) {
  static_assert(CPW >= 1 && CPW <= kWave && (CPW & (CPW - 1)) == 0, "CPW must be a power of two <= 64");
  static_assert((CPW * SL) % kWave == 0, "whole wavefronts");
  constexpr int WAVES = CPW * SL / kWave;
  __shared__ float lds[WAVES > 1 ? kColFields * WAVES * CPW : 1];
  const int c = threadIdx.x % CPW;
  const int sl = threadIdx.x / CPW;
  const int col = blockIdx.x * CPW + c;
  const size_t plane = static_cast<size_t>(nsplit) * cols;
  ColState st = col_state_empty();
  if (col < cols) {
    for (int s0 = sl; s0 < nsplit; s0 += SL * BATCH) {
      float f[BATCH][kColPartWords];
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        const int s = s0 + b * SL;
        const size_t o = static_cast<size_t>(s < nsplit ? s : s0) * cols + col;
#pragma unroll
        for (int k = 0; k < kColPartWords; ++k) f[b][k] = part[k * plane + o];
      }
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        const int s = s0 + b * SL;
        if (s < nsplit) {
          ColState t;
          t.m.n = static_cast<float>(col_split_rows(rows, nsplit, batch, s));
          t.m.mean = f[b][0];
          t.m.m2 = f[b][1];
          t.a.v = f[b][2];
          t.a.i = __float_as_int(f[b][3]);
          st = col_state_combine(st, t);
        }
      }
    }
  }
  // split lanes of one wavefront: lanes c, c + CPW, c + 2 CPW, ...
#pragma unroll
  for (int off = CPW; off < kWave; off <<= 1) {
    ColState o;
    o.m.n = __shfl_xor(st.m.n, off, kWave);
    o.m.mean = __shfl_xor(st.m.mean, off, kWave);
    o.m.m2 = __shfl_xor(st.m.m2, off, kWave);
    o.a.v = __shfl_xor(st.a.v, off, kWave);
    o.a.i = __shfl_xor(st.a.i, off, kWave);
    st = col_state_combine(st, o);
  }
  if constexpr (WAVES > 1) {
    const int wave = threadIdx.x / kWave;
    constexpr int PLANE = WAVES * CPW;
    if ((threadIdx.x % kWave) < CPW) {
      const int t = wave * CPW + c;
      lds[0 * PLANE + t] = st.m.n;
      lds[1 * PLANE + t] = st.m.mean;
      lds[2 * PLANE + t] = st.m.m2;
      lds[3 * PLANE + t] = st.a.v;
      lds[4 * PLANE + t] = __int_as_float(st.a.i);
    }
    __syncthreads();
    if (threadIdx.x < CPW) {
#pragma unroll
      for (int w = 1; w < WAVES; ++w) {
        const int t = w * CPW + c;
        ColState b;
        b.m.n = lds[0 * PLANE + t];
        b.m.mean = lds[1 * PLANE + t];
        b.m.m2 = lds[2 * PLANE + t];
        b.a.v = lds[3 * PLANE + t];
        b.a.i = __float_as_int(lds[4 * PLANE + t]);
        st = col_state_combine(st, b);
      }
    }
  }
  if (threadIdx.x < CPW && col < cols) {
    mean_out[col] = st.m.mean;
    const float denom = fmaxf(st.m.n - correction, 0.f);
    var_out[col] = st.m.m2 / denom;
    argmax_out[col] = static_cast<long long>(st.a.i);
  }
}

}  // namespace mi
