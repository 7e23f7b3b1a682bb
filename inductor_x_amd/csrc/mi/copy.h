// Indexing / layout kernels: row gather through an int64 index vector and
// strided (permuted) copies whose innermost axis stays contiguous.  Both move
// raw 16-byte vectors, so they are exact for every element type.
//
// In the reference the gather is an eager fallback
// (reference inductor_x/lowering.py:327-330,338) with an indirect-load path in
// the code generator (reference inductor_x/codegen/triton.py:1665-1717), and a
// permuted copy is a pointwise kernel tiled over the two axes that are
// contiguous on the read and on the write side
// (reference inductor_x/codegen/split_tiling.py:85-154).
#pragma once

#include "common.h"

namespace mi {

// out[i, :] = table[idx[i], :].  TPR threads share one row; a workgroup of
// BLOCK threads handles RPT * (BLOCK / TPR) consecutive rows.  Negative indices
// wrap once (Python semantics); anything still out of range is clamped so the
// kernel never reads outside the table.
template <typename T, int VEC, int BLOCK, int TPR, int RPT>
__device__ __forceinline__ void gather_rows(const T* __restrict__ table,
                                            const long long* __restrict__ idx,
                                            T* __restrict__ out, int nidx, int row_elems,
                                            int table_rows) {
  constexpr int ROWS = BLOCK / TPR;
  const int lane = threadIdx.x % TPR;
  const int sub = threadIdx.x / TPR;
  const int row0 = (blockIdx.x * RPT) * ROWS + sub;
  long long src[RPT];
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const int row = row0 + j * ROWS;
    long long i = (row < nidx) ? idx[row] : 0;
    if (i < 0) i += table_rows;
    i = i < 0 ? 0 : (i >= table_rows ? table_rows - 1 : i);
    src[j] = i;
  }
  for (int c = lane * VEC; c < row_elems; c += TPR * VEC) {
    Vec<T, VEC> v[RPT];
#pragma unroll
    for (int j = 0; j < RPT; ++j) {
      const int row = row0 + j * ROWS;
      if (row < nidx) v[j] = load_vec<T, VEC, true>(table + static_cast<size_t>(src[j]) * row_elems + c);
    }
#pragma unroll
    for (int j = 0; j < RPT; ++j) {
      const int row = row0 + j * ROWS;
      if (row < nidx) store_vec<T, VEC, true>(out + static_cast<size_t>(row) * row_elems + c, v[j]);
    }
  }
}

// 4-D permuted copy with a contiguous innermost axis on both sides:
//   out[a][b][c][0:inner]  (contiguous, sizes n0, n1, n2, inner)
//     = in[a*s0 + b*s1 + c*s2 + (0:inner)]
// A workgroup copies a tile of T1 values of b by T2 values of c for one a.
// Threads are ordered so consecutive "chunks" (one inner run each) advance
// along c, i.e. along the output's contiguous direction, while the tile as a
// whole covers T1 x T2 inner runs of the input; with T1 spanning the axis that
// is adjacent in the input, both sides see long contiguous runs.
// TPC = threads per chunk (inner / VEC rounded up to a power of two <= 64).
template <typename T, int VEC, int BLOCK, int TPC, int T1, int T2>
__device__ __forceinline__ void permute_copy_tiled(const T* __restrict__ in, T* __restrict__ out,
                                                   int n0, int n1, int n2, int inner,
                                                   long long s0, long long s1, long long s2) {
  constexpr int CHUNKS_PER_PASS = BLOCK / TPC;
  constexpr int CHUNKS = T1 * T2;
  static_assert(CHUNKS % CHUNKS_PER_PASS == 0, "tile must be whole passes");
  constexpr int PASSES = CHUNKS / CHUNKS_PER_PASS;
  const int tiles_c = (n2 + T2 - 1) / T2;
  const int tiles_b = (n1 + T1 - 1) / T1;
  int t = blockIdx.x;
  const int tc = t % tiles_c;
  t /= tiles_c;
  const int tb = t % tiles_b;
  const int a = t / tiles_b;
  const int lane = threadIdx.x % TPC;
  const int chunk0 = threadIdx.x / TPC;
  const int e = lane * VEC;
  if (e >= inner) return;

  Vec<T, VEC> v[PASSES];
  bool ok[PASSES];
  size_t dst[PASSES];
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    const int chunk = p * CHUNKS_PER_PASS + chunk0;
    const int c = tc * T2 + chunk % T2;
    const int b = tb * T1 + chunk / T2;
    ok[p] = (b < n1) && (c < n2);
    if (ok[p]) {
      v[p] = load_vec<T, VEC, true>(in + a * s0 + b * s1 + c * s2 + e);
      dst[p] = ((static_cast<size_t>(a) * n1 + b) * n2 + c) * inner + e;
    }
  }
#pragma unroll
  for (int p = 0; p < PASSES; ++p) {
    if (ok[p]) store_vec<T, VEC, true>(out + dst[p], v[p]);
  }
}

}  // namespace mi
