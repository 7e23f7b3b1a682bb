// Row (last-dimension) reduction kernels: the contiguous axis is reduced,
// every other axis is flattened into "rows".
//
// Thread mapping: TPR consecutive threads cooperate on one row and a workgroup
// of BLOCK threads carries BLOCK / TPR rows, so short rows still fill a
// wavefront.  Each thread walks its row in 16-byte vectors, TPR vectors apart,
// which makes every wavefront access a run of 1 KiB.  Partial results are
// combined with DPP inside a wavefront and through LDS across wavefronts.
//
// These kernels take the place of the reference's looped and persistent
// row-reduction code shapes (reference inductor_x/codegen/triton.py:1208-1253
// and :1163-1207): `row_reduce_looped` is the looped form with a per-thread
// accumulator, `row_persistent` keeps the whole row in registers so a value
// computed from the reduction can be applied without re-reading memory.
#pragma once

#include "common.h"

namespace mi {

// Prog contract (looped form)
//   static constexpr int VEC          elements handled per call of partial()
//   float identity() const            neutral element
//   float partial(row, r) const       reduction of elements [r, r + VEC) of `row`
//   float combine(a, b) const         associative combine
//   void  finish(row, total) const    consume the row's result (one thread calls it)
template <class Prog, int BLOCK, int TPR, int UNROLL>
__device__ __forceinline__ void row_reduce_looped(const Prog& p, int xnumel, int rnumel) {
  static_assert(BLOCK % TPR == 0, "TPR must divide BLOCK");
  constexpr int ROWS = BLOCK / TPR;
  __shared__ float lds[BLOCK / kWave > 0 ? BLOCK / kWave : 1];
  const int row = blockIdx.x * ROWS + threadIdx.x / TPR;
  const int lane = threadIdx.x % TPR;
  float acc = p.identity();
  if (row < xnumel) {
#pragma unroll UNROLL
    for (int r = lane * Prog::VEC; r < rnumel; r += TPR * Prog::VEC) acc = p.combine(acc, p.partial(row, r));
  }
  struct Op {
    const Prog& p;
    __device__ __forceinline__ float operator()(float a, float b) const { return p.combine(a, b); }
  };
  acc = group_reduce<BLOCK, TPR>(acc, Op{p}, lds);
  if (row < xnumel && lane == 0) p.finish(row, acc);
}

}  // namespace mi
