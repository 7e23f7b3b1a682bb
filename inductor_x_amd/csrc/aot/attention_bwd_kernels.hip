// Fused attention backward instantiations (bf16, head dimension 128); see mi/attention_bwd.h.
// Workgroup -> (head, block): consecutive workgroup ids go to consecutive dies, so the heads of
// one die share its L2; within a head the blocks with the most tiles come first under a causal mask.
#include "../mi/attention_bwd.h"

using namespace mi;

extern "C" __global__ __launch_bounds__(256) void attention_bwd_delta_bf16_d128(const bf16_t* o, const bf16_t* d_o,
                                                                                 float* delta, int rows) {
  attention_bwd_delta(o, d_o, delta, rows);
}

template <bool CAUSAL, bool HEAVY_LAST>
__device__ __forceinline__ bool bwd_block_of(int n_heads, int n_blocks, int& head, int& block) {
  constexpr int XCDS = 8;
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  head = (slot / n_blocks) * XCDS + xcd;
  const int b = slot % n_blocks;
  // query blocks get heavier towards the end of the sequence, key blocks towards its start
  block = (CAUSAL && HEAVY_LAST) ? n_blocks - 1 - b : b;
  return head < n_heads;
}

#define BWD_DQ(NAME, CAUSAL)                                                                           \
  extern "C" __global__ __launch_bounds__(256, 1) void NAME(                                           \
      const bf16_t* q, const bf16_t* k, const bf16_t* v, const bf16_t* o, const bf16_t* d_o,            \
      const float* smax, const float* ssum, bf16_t* dq, int n_heads, int S, float scale) {             \
    int head, block;                                                                                   \
    if (!bwd_block_of<CAUSAL, true>(n_heads, S / 128, head, block)) return;                            \
    attention_bwd_dq<CAUSAL>(q, k, v, o, d_o, smax, ssum, dq, S, block, head, scale);                  \
  }
BWD_DQ(attention_bwd_dq_bf16_d128_causal, true)
BWD_DQ(attention_bwd_dq_bf16_d128_full, false)

#define BWD_DKV(NAME, CAUSAL)                                                                          \
  extern "C" __global__ __launch_bounds__(256, 1) void NAME(                                           \
      const bf16_t* q, const bf16_t* k, const bf16_t* v, const bf16_t* d_o, const float* smax,          \
      const float* ssum, const float* delta, bf16_t* dk, bf16_t* dv, int n_heads, int S, float scale) { \
    int head, block;                                                                                   \
    if (!bwd_block_of<CAUSAL, false>(n_heads, S / 128, head, block)) return;                           \
    attention_bwd_dkv<CAUSAL>(q, k, v, d_o, smax, ssum, delta, dk, dv, S, block, head, scale);         \
  }
BWD_DKV(attention_bwd_dkv_bf16_d128_causal, true)
BWD_DKV(attention_bwd_dkv_bf16_d128_full, false)
