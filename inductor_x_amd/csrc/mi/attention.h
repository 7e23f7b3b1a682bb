// Fused attention for gfx950: operand layouts, tile formats and small helpers shared by the forward
// kernel (attention_v5.h) and the backward kernels (attention_bwd_w8.h).
//   O = softmax(Q K^T * scale [+ causal mask]) V,   layout [B, N, S, D], D = 128, 16-bit in / out,
// fp32 softmax.  The forward also writes the per-row softmax maximum and sum ([B, N, S, 8] fp32,
// value repeated over the last axis), the two statistics the reference's fused attention op returns
// besides the output (reference inductor_x/npu_fusion_attention_graph.py:17-35,45-74).
//
// Mapping onto the matrix cores (v_mfma_f32_32x32x16_bf16, 64-lane wavefronts)
// -------------------------------------------------------------------------
// A workgroup is 8 wavefronts; a wavefront owns 32 consecutive queries, the
// workgroup 256.  Keys/values are visited in tiles of 64, staged in LDS and
// shared by the wavefronts.  Both products are computed transposed so that a
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
// The forward reads its V^T fragments in that key order with transposing LDS reads of the
// untransposed tile.  The backward kernels keep transposed tiles in LDS with the permuted axis
// stored the same way (bits 2 and 3 of the index swapped inside every group of 16), so that
// operand is a single 16-byte LDS read (chunks are additionally XOR-swizzled against bank
// conflicts, see attn_vt_offset); the transposition happens in registers while the tile is
// copied to LDS.
#pragma once

#include <type_traits>
#include <utility>

#include "common.h"

namespace mi {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
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

// The reference maximum of the online softmax moves only when the true maximum has grown past it
// by more than this many powers of two.  Until then probabilities are at most 2^slack (no overflow,
// same relative precision in 16 bits and fp32), numerator and denominator stay consistent, and the
// output accumulators need no rescaling: some query of a wavefront raises its maximum in most
// tiles, but hardly ever by a factor of 256.
constexpr float kAttnSlack = 8.0f;

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

__device__ __forceinline__ bf16x8_t attn_as_bf16x8(u32x4_t x) {
  return __builtin_bit_cast(bf16x8_t, x);
}

// What differs between the two 16-bit element types: the matrix instruction, the transposing LDS
// read and the rounding of a probability pair into one 32-bit word.
template <typename T>
struct AttnElem;
template <>
struct AttnElem<bf16_t> {
  typedef __bf16 x8 __attribute__((ext_vector_type(8)));
  typedef __bf16 x4 __attribute__((ext_vector_type(4)));
  typedef __bf16 x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 x4v __attribute__((__vector_size__(4 * sizeof(__bf16))));
  static __device__ __forceinline__ f32x16_t mfma(x8 a, x8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ x4 read_tr(const __bf16* p) {
    return __builtin_bit_cast(x4, __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) x4v*)(p)));
  }
};
template <>
struct AttnElem<f16_t> {
  typedef _Float16 x8 __attribute__((ext_vector_type(8)));
  typedef _Float16 x4 __attribute__((ext_vector_type(4)));
  typedef _Float16 x2 __attribute__((ext_vector_type(2)));
  typedef __fp16 x4v __attribute__((__vector_size__(4 * sizeof(__fp16))));
  static __device__ __forceinline__ f32x16_t mfma(x8 a, x8 b, f32x16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ x4 read_tr(const _Float16* p) {
    return __builtin_bit_cast(x4, __builtin_amdgcn_ds_read_tr16_b64_v4f16((__attribute__((address_space(3))) x4v*)(p)));
  }
};

}  // namespace mi
