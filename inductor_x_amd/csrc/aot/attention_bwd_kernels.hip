// Fused attention backward instantiations (bf16 and fp16, head dimension 128): eight wavefronts per
// workgroup on 256 rows, a statistics pass and separate dQ, dK and dV kernels (mi/attention_bwd_w8.h).
// Workgroup -> (head, block): consecutive workgroup ids go to consecutive dies, so the heads of
// one die share its L2.
#include "../mi/attention_bwd_w8.h"

using namespace mi;

template <bool CAUSAL, bool HEAVY_LAST>
__device__ __forceinline__ bool bwd_block_of(int n_heads, int n_blocks, int& head, int& block) {
  constexpr int XCDS = 8;
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  head = (slot / n_blocks) * XCDS + xcd;
  const int b = slot % n_blocks;
  block = (CAUSAL && HEAVY_LAST) ? n_blocks - 1 - b : b;
  return head < n_heads;
}

#define BWD_STATS(NAME, T)                                                                             \
  extern "C" __global__ __launch_bounds__(256) void NAME(const T* o, const T* d_o, const float* smax,  \
                                                         const float* ssum, float* stats, int rows) {  \
    attention_bwd_stats<T>(o, d_o, smax, ssum, stats, rows);                                           \
  }
BWD_STATS(attention_bwd_stats_bf16_d128, bf16_t)
BWD_STATS(attention_bwd_stats_f16_d128, f16_t)

// Work unit of a workgroup: one block of 256 rows, or under a causal mask the pair of blocks
// (u, n - 1 - u), whose tile counts add up to the same number for every u, so that all
// workgroups take equally long and the heads in flight on a die stay in step.
template <bool CAUSAL, class Body>
__device__ __forceinline__ void bwd8_for_blocks(int n_heads, int S, Body&& body) {
  const int n_blocks = (S + kBwd8BlockRows - 1) / kBwd8BlockRows;
  const int n_units = CAUSAL ? (n_blocks + 1) / 2 : n_blocks;
  int head, u;
  if (!bwd_block_of<false, false>(n_heads, n_units, head, u)) return;
  if constexpr (CAUSAL) {
    const int other = n_blocks - 1 - u;
#pragma nounroll
    for (int half = 0; half < 2; ++half) {
      if (half == 1 && other == u) break;
      body(head, half ? u : other);
    }
  } else {
    body(head, u);
  }
}

#define BWD8_DQ_DH(NAME, T, CAUSAL, DH)                                                                \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                           \
      const T* q, const T* k, const T* v, const T* d_o, const float* stats, T* dq, int n_heads, int S, \
      float scale) {                                                                                   \
    bwd8_for_blocks<CAUSAL>(n_heads, S, [&](int head, int block) {                                     \
      attention_bwd8_dq<T, CAUSAL, DH>(q, k, v, d_o, stats, dq, S, block, head, scale);                \
    });                                                                                                \
  }
#define BWD8_DQ(NAME, T, CAUSAL) BWD8_DQ_DH(NAME, T, CAUSAL, 128)
BWD8_DQ(attention_bwd8_dq_bf16_d128_causal, bf16_t, true)
BWD8_DQ(attention_bwd8_dq_bf16_d128_full, bf16_t, false)
BWD8_DQ(attention_bwd8_dq_f16_d128_causal, f16_t, true)
BWD8_DQ(attention_bwd8_dq_f16_d128_full, f16_t, false)

#define BWD8_DKV_DH(NAME, T, CAUSAL, WHICH, DH)                                                        \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                           \
      const T* q, const T* k, const T* v, const T* d_o, const float* stats, T* out, int n_heads,       \
      int S, float scale) {                                                                            \
    bwd8_for_blocks<CAUSAL>(n_heads, S, [&](int head, int block) {                                     \
      attention_bwd8_dkv<T, CAUSAL, WHICH, DH>(q, k, v, d_o, stats, out, S, block, head, scale);       \
    });                                                                                                \
  }
#define BWD8_DKV(NAME, T, CAUSAL, WHICH) BWD8_DKV_DH(NAME, T, CAUSAL, WHICH, 128)
BWD8_DKV(attention_bwd8_dk_bf16_d128_causal, bf16_t, true, 0)
BWD8_DKV(attention_bwd8_dk_bf16_d128_full, bf16_t, false, 0)
BWD8_DKV(attention_bwd8_dv_bf16_d128_causal, bf16_t, true, 1)
BWD8_DKV(attention_bwd8_dv_bf16_d128_full, bf16_t, false, 1)
BWD8_DKV(attention_bwd8_dk_f16_d128_causal, f16_t, true, 0)
BWD8_DKV(attention_bwd8_dk_f16_d128_full, f16_t, false, 0)
BWD8_DKV(attention_bwd8_dv_f16_d128_causal, f16_t, true, 1)
BWD8_DKV(attention_bwd8_dv_f16_d128_full, f16_t, false, 1)

// Heads of at most 64 columns, zero-padded to 128 by the caller: the all-zero d slices and d blocks
// are skipped (half the matrix work, the same tiles).
#define BWD8_D64(T, TN)                                                           \
  BWD8_DQ_DH(attention_bwd8_dq_##TN##_d64_causal, T, true, 64)                     \
  BWD8_DQ_DH(attention_bwd8_dq_##TN##_d64_full, T, false, 64)                      \
  BWD8_DKV_DH(attention_bwd8_dk_##TN##_d64_causal, T, true, 0, 64)                 \
  BWD8_DKV_DH(attention_bwd8_dk_##TN##_d64_full, T, false, 0, 64)                  \
  BWD8_DKV_DH(attention_bwd8_dv_##TN##_d64_causal, T, true, 1, 64)                 \
  BWD8_DKV_DH(attention_bwd8_dv_##TN##_d64_full, T, false, 1, 64)
BWD8_D64(bf16_t, bf16)
BWD8_D64(f16_t, f16)

// With a bit mask (64-bit words [B or 1, N or 1, S, S / 64], byte strides; dQ takes the words of the mask,
// dK and dV those of its transpose): hidden pairs get the probability zero.  tile_ranges (may be null): per
// block of 256 rows the first and last tile of the other axis with a visible pair, int [B or 1, N or 1,
// ceil(S / 256), 2] with batch and head strides in elements; tiles outside are not visited.
#define BWD8_MASKED(NAME, T, CAUSAL, BODY)                                                             \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                           \
      const T* q, const T* k, const T* v, const T* d_o, const float* stats, T* out, int n_heads,       \
      int S, float scale, const unsigned char* mask, long long mask_batch_stride,                      \
      long long mask_head_stride, int heads_per_batch, const int* tile_ranges, int range_batch_stride, \
      int range_head_stride) {                                                                         \
    bwd8_for_blocks<CAUSAL>(n_heads, S, [&](int head, int block) {                                     \
      const unsigned char* hm =                                                                        \
          mask + (head / heads_per_batch) * mask_batch_stride + (head % heads_per_batch) * mask_head_stride; \
      const int* hr = tile_ranges ? tile_ranges + (head / heads_per_batch) * range_batch_stride +      \
                                        (head % heads_per_batch) * range_head_stride + 2 * block       \
                                  : nullptr;                                                           \
      const int lo = hr ? hr[0] : 0, hi = hr ? hr[1] : 0x7fffff;                                       \
      BODY;                                                                                            \
    });                                                                                                \
  }
#define BWD8_MASKED_ALL(T, TN)                                                                                     \
  BWD8_MASKED(attention_bwd8_dq_##TN##_d128_causal_masked, T, true,                                               \
              (attention_bwd8_dq<T, true, 128, true>(q, k, v, d_o, stats, out, S, block, head, scale, hm, lo, hi)))         \
  BWD8_MASKED(attention_bwd8_dq_##TN##_d128_full_masked, T, false,                                                \
              (attention_bwd8_dq<T, false, 128, true>(q, k, v, d_o, stats, out, S, block, head, scale, hm, lo, hi)))        \
  BWD8_MASKED(attention_bwd8_dk_##TN##_d128_causal_masked, T, true,                                               \
              (attention_bwd8_dkv<T, true, 0, 128, true>(q, k, v, d_o, stats, out, S, block, head, scale, hm, lo, hi)))     \
  BWD8_MASKED(attention_bwd8_dk_##TN##_d128_full_masked, T, false,                                                \
              (attention_bwd8_dkv<T, false, 0, 128, true>(q, k, v, d_o, stats, out, S, block, head, scale, hm, lo, hi)))    \
  BWD8_MASKED(attention_bwd8_dv_##TN##_d128_causal_masked, T, true,                                               \
              (attention_bwd8_dkv<T, true, 1, 128, true>(q, k, v, d_o, stats, out, S, block, head, scale, hm, lo, hi)))     \
  BWD8_MASKED(attention_bwd8_dv_##TN##_d128_full_masked, T, false,                                                \
              (attention_bwd8_dkv<T, false, 1, 128, true>(q, k, v, d_o, stats, out, S, block, head, scale, hm, lo, hi)))
BWD8_MASKED_ALL(bf16_t, bf16)
BWD8_MASKED_ALL(f16_t, f16)
