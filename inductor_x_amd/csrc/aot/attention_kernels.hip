// Fused attention forward instantiations (bf16, head dimension 128).
//
// Workgroup -> (head, query block) mapping: hardware deals consecutive
// workgroup ids round-robin to the 8 accelerator dies, each with its own L2.
// Ids that land on one die walk the query blocks of one head before moving to
// the next head, so a head's K and V are fetched into a single L2.  With a
// causal mask the heaviest query blocks (most key tiles) are issued first.
#include "../mi/attention.h"

using namespace mi;

template <bool CAUSAL>
__device__ __forceinline__ void attention_entry(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                                bf16_t* o, float* smax, float* ssum, int n_heads,
                                                int S, float scale_log2e) {
  constexpr int XCDS = 8;
  const int n_qb = S / kAttnBM;
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  const int head = (slot / n_qb) * XCDS + xcd;
  int qb = slot % n_qb;
  if (head >= n_heads) return;
  if (CAUSAL) qb = n_qb - 1 - qb;
  attention_fwd_d128<CAUSAL>(q, k, v, o, smax, ssum, S, qb, head, scale_log2e);
}

extern "C" __global__ __launch_bounds__(kAttnThreads) void fused_attention_fwd_bf16_d128_causal(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry<true>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}

extern "C" __global__ __launch_bounds__(kAttnThreads) void fused_attention_fwd_bf16_d128_full(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry<false>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
