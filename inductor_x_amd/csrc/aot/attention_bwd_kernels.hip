// Fused attention backward instantiations (bf16, head dimension 128): eight wavefronts per
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

extern "C" __global__ __launch_bounds__(256) void attention_bwd_stats_bf16_d128(
    const bf16_t* o, const bf16_t* d_o, const float* smax, const float* ssum, float* stats, int rows) {
  attention_bwd_stats(o, d_o, smax, ssum, stats, rows);
}

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

#define BWD8_DQ(NAME, CAUSAL)                                                                          \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                           \
      const bf16_t* q, const bf16_t* k, const bf16_t* v, const bf16_t* d_o, const float* stats,         \
      bf16_t* dq, int n_heads, int S, float scale) {                                                   \
    bwd8_for_blocks<CAUSAL>(n_heads, S, [&](int head, int block) {                                     \
      attention_bwd8_dq<CAUSAL>(q, k, v, d_o, stats, dq, S, block, head, scale);                       \
    });                                                                                                \
  }
BWD8_DQ(attention_bwd8_dq_bf16_d128_causal, true)
BWD8_DQ(attention_bwd8_dq_bf16_d128_full, false)

#define BWD8_DKV(NAME, CAUSAL, WHICH)                                                                  \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                           \
      const bf16_t* q, const bf16_t* k, const bf16_t* v, const bf16_t* d_o, const float* stats,         \
      bf16_t* out, int n_heads, int S, float scale) {                                                  \
    bwd8_for_blocks<CAUSAL>(n_heads, S, [&](int head, int block) {                                     \
      attention_bwd8_dkv<CAUSAL, WHICH>(q, k, v, d_o, stats, out, S, block, head, scale);              \
    });                                                                                                \
  }
BWD8_DKV(attention_bwd8_dk_bf16_d128_causal, true, 0)
BWD8_DKV(attention_bwd8_dk_bf16_d128_full, false, 0)
BWD8_DKV(attention_bwd8_dv_bf16_d128_causal, true, 1)
BWD8_DKV(attention_bwd8_dv_bf16_d128_full, false, 1)
