// Fused attention forward instantiations (bf16 and fp16, head dimension 128).
//
// The launch is persistent (attention_entry_v5: at most one workgroup per CU, each walking its list of query
// blocks).  No workgroup is dispatched between two items and
// the output stores of one item drain while the next one loads its queries and first key tiles;
// measured on MI355X at [4,32,4096,128] causal: 2 % over one workgroup per item.
#include "../mi/attention_v5.h"

using namespace mi;

// 512 threads, 256 queries per workgroup, one workgroup per CU, 64 KiB of LDS.
#define ATTENTION_V5_DH(NAME, T, CAUSAL, RAGGED, DH)                                                  \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(const T* q, const T* k, const T* v,       \
                                                            T* o, float* smax, float* ssum,           \
                                                            int n_heads, int Sq, int Sk,              \
                                                            float scale_log2e) {                      \
    attention_entry_v5<T, CAUSAL, RAGGED, DH>(q, k, v, o, smax, ssum, n_heads, Sq, Sk, scale_log2e);  \
  }
#define ATTENTION_V5(NAME, T, CAUSAL, RAGGED) ATTENTION_V5_DH(NAME, T, CAUSAL, RAGGED, 128)

ATTENTION_V5(fused_attention_fwd_bf16_d128_causal_v5, bf16_t, true, false)
ATTENTION_V5(fused_attention_fwd_bf16_d128_full_v5, bf16_t, false, false)
ATTENTION_V5(fused_attention_fwd_bf16_d128_causal_v5_ragged, bf16_t, true, true)
ATTENTION_V5(fused_attention_fwd_bf16_d128_full_v5_ragged, bf16_t, false, true)
ATTENTION_V5(fused_attention_fwd_f16_d128_causal_v5, f16_t, true, false)
ATTENTION_V5(fused_attention_fwd_f16_d128_full_v5, f16_t, false, false)
ATTENTION_V5(fused_attention_fwd_f16_d128_causal_v5_ragged, f16_t, true, true)
ATTENTION_V5(fused_attention_fwd_f16_d128_full_v5_ragged, f16_t, false, true)
// Heads of at most 64 columns, zero-padded to 128 by the caller: the same tiles, half the matrix work
// (the all-zero d slices and d blocks are skipped); any sequence lengths.
ATTENTION_V5_DH(fused_attention_fwd_bf16_d64_causal_v5, bf16_t, true, true, 64)
ATTENTION_V5_DH(fused_attention_fwd_bf16_d64_full_v5, bf16_t, false, true, 64)
ATTENTION_V5_DH(fused_attention_fwd_f16_d64_causal_v5, f16_t, true, true, 64)
ATTENTION_V5_DH(fused_attention_fwd_f16_d64_full_v5, f16_t, false, true, 64)

// With a bit mask, 64-bit words [B or 1, N or 1, Sq, ceil(Sk / 64)] (bit set = hidden), any sequence lengths;
// tile_ranges (may be null): per query block of 256 the first and last key tile with a visible key,
// int [B or 1, N or 1, ceil(Sq / 256), 2] with its batch and head strides in elements.
#define ATTENTION_V5_MASKED(NAME, T, CAUSAL)                                                            \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                            \
      const T* q, const T* k, const T* v, T* o, float* smax, float* ssum, int n_heads, int Sq, int Sk,  \
      float scale_log2e, const unsigned char* mask, long long mask_batch_stride,                        \
      long long mask_head_stride, int heads_per_batch, const int* tile_ranges, int range_batch_stride,  \
      int range_head_stride) {                                                                          \
    attention_entry_v5<T, CAUSAL, true, 128, true>(q, k, v, o, smax, ssum, n_heads, Sq, Sk, scale_log2e, \
                                                   mask, mask_batch_stride, mask_head_stride,           \
                                                   heads_per_batch, AttnNoTimeline(), tile_ranges,      \
                                                   range_batch_stride, range_head_stride);              \
  }
ATTENTION_V5_MASKED(fused_attention_fwd_bf16_d128_causal_v5_masked, bf16_t, true)
ATTENTION_V5_MASKED(fused_attention_fwd_bf16_d128_full_v5_masked, bf16_t, false)
ATTENTION_V5_MASKED(fused_attention_fwd_f16_d128_causal_v5_masked, f16_t, true)
ATTENTION_V5_MASKED(fused_attention_fwd_f16_d128_full_v5_masked, f16_t, false)
