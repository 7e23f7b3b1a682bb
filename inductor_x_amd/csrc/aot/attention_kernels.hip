// Fused attention forward instantiations (bf16 and fp16, head dimension 128).
//
// Workgroup -> (head, query block) mapping: hardware deals consecutive workgroup ids round-robin to
// the 8 accelerator dies, each with its own L2.  Ids that land on one die walk the query blocks of
// one head before moving to the next head, so a head's K and V are fetched into a single L2.  Under
// a causal mask query block b visits 4 b + 4 key tiles; a work item is the pair (b, n - 1 - b), the
// longer member first, so every item is the same amount of work.
//
// The launch is persistent: the grid is at most one workgroup per CU and every workgroup walks the
// work items id = blockIdx.x, blockIdx.x + gridDim.x, ... (gridDim.x is a multiple of 8, so a
// workgroup stays on the heads of its own die).  No workgroup is dispatched between two items and
// the output stores of one item drain while the next one loads its queries and first key tiles;
// measured on MI355X at [4,32,4096,128] causal: 2 % over one workgroup per item.
#include "../mi/attention_v5.h"

using namespace mi;

template <typename T, bool CAUSAL, bool RAGGED, int DH = 128, bool MASKED = false>
__device__ __forceinline__ void attention_entry_v5(const T* q, const T* k, const T* v, T* o, float* smax,
                                                   float* ssum, int n_heads, int Sq, int Sk,
                                                   float scale_log2e, const unsigned char* mask = nullptr,
                                                   long long mask_batch_stride = 0, long long mask_head_stride = 0,
                                                   int heads_per_batch = 1) {
  constexpr int XCDS = 8;
  const int n_qb = (Sq + kAttnV5BM - 1) / kAttnV5BM;
  const int per_head = CAUSAL ? (n_qb + 1) / 2 : n_qb;
  const int total = XCDS * ((n_heads + XCDS - 1) / XCDS) * per_head;
#pragma nounroll
  for (int id = blockIdx.x; id < total; id += gridDim.x) {
    const int xcd = id % XCDS;
    const int slot = id / XCDS;
    const int head = (slot / per_head) * XCDS + xcd;
    if (head >= n_heads) continue;
    // the [Sq][tiles] 64-bit mask words of this head (byte strides; 0 where the mask broadcasts over batch or heads)
    const unsigned char* hm =
        MASKED ? mask + (head / heads_per_batch) * mask_batch_stride + (head % heads_per_batch) * mask_head_stride : nullptr;
    if (CAUSAL) {
      const int lo = slot % per_head;
      const int hi = n_qb - 1 - lo;
      const int n_pass = lo != hi ? 2 : 1;
#pragma nounroll
      for (int pass = 0; pass < n_pass; ++pass)
        attention_fwd_d128_v5<T, true, RAGGED, kAttnV5Waves, DH, MASKED>(q, k, v, o, smax, ssum, Sq, Sk, pass == 0 ? hi : lo, head,
                                                                         scale_log2e, hm);
    } else {
      attention_fwd_d128_v5<T, false, RAGGED, kAttnV5Waves, DH, MASKED>(q, k, v, o, smax, ssum, Sq, Sk, slot % per_head, head,
                                                                        scale_log2e, hm);
    }
  }
}

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

// With a bit mask, 64-bit words [B or 1, N or 1, Sq, ceil(Sk / 64)] (bit set = hidden), any sequence lengths.
#define ATTENTION_V5_MASKED(NAME, T, CAUSAL)                                                            \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                            \
      const T* q, const T* k, const T* v, T* o, float* smax, float* ssum, int n_heads, int Sq, int Sk,  \
      float scale_log2e, const unsigned char* mask, long long mask_batch_stride,                        \
      long long mask_head_stride, int heads_per_batch) {                                                \
    attention_entry_v5<T, CAUSAL, true, 128, true>(q, k, v, o, smax, ssum, n_heads, Sq, Sk, scale_log2e, \
                                                   mask, mask_batch_stride, mask_head_stride,           \
                                                   heads_per_batch);                                    \
  }
ATTENTION_V5_MASKED(fused_attention_fwd_bf16_d128_causal_v5_masked, bf16_t, true)
ATTENTION_V5_MASKED(fused_attention_fwd_bf16_d128_full_v5_masked, bf16_t, false)
ATTENTION_V5_MASKED(fused_attention_fwd_f16_d128_causal_v5_masked, f16_t, true)
ATTENTION_V5_MASKED(fused_attention_fwd_f16_d128_full_v5_masked, f16_t, false)
