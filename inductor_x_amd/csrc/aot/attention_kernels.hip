// Fused attention forward instantiations (bf16, head dimension 128).
//
// Workgroup -> (head, query block) mapping: hardware deals consecutive
// workgroup ids round-robin to the 8 accelerator dies, each with its own L2.
// Ids that land on one die walk the query blocks of one head before moving to
// the next head, so a head's K and V are fetched into a single L2.  With a
// causal mask the heaviest query blocks (most key tiles) are issued first.
#include "../mi/attention_pp.h"
#include "../mi/attention_v2.h"
#include "../mi/attention_v4.h"
#include "../mi/attention_v5.h"

using namespace mi;

template <bool CAUSAL, int WAVES>
__device__ __forceinline__ void attention_entry(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                                bf16_t* o, float* smax, float* ssum, int n_heads,
                                                int S, float scale_log2e) {
  constexpr int XCDS = 8;
  const int n_qb = S / (kAttnRowsPerWave * WAVES);
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  const int head = (slot / n_qb) * XCDS + xcd;
  int qb = slot % n_qb;
  if (head >= n_heads) return;
  if (CAUSAL) qb = n_qb - 1 - qb;
  attention_fwd_d128<CAUSAL, WAVES>(q, k, v, o, smax, ssum, S, qb, head, scale_log2e);
}

// w4: 256 threads, 128 queries per workgroup, two workgroups per CU.
// w8: 512 threads, 256 queries per workgroup, one workgroup per CU.
#define ATTENTION_VARIANT(NAME, CAUSAL, WAVES, MINBLOCKS)                                      \
  extern "C" __global__ __launch_bounds__(64 * WAVES, MINBLOCKS) void NAME(                    \
      const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,  \
      int n_heads, int S, float scale_log2e) {                                                 \
    attention_entry<CAUSAL, WAVES>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);           \
  }

ATTENTION_VARIANT(fused_attention_fwd_bf16_d128_causal_w4, true, 4, 2)
ATTENTION_VARIANT(fused_attention_fwd_bf16_d128_full_w4, false, 4, 2)
ATTENTION_VARIANT(fused_attention_fwd_bf16_d128_causal_w8, true, 8, 1)
ATTENTION_VARIANT(fused_attention_fwd_bf16_d128_full_w8, false, 8, 1)

// pp: 512 threads, 256 queries per workgroup, the two wavefronts of every SIMD
// alternate between the matrix phase and the softmax phase (attention_pp.h).
template <bool CAUSAL>
__device__ __forceinline__ void attention_entry_pp(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                                   bf16_t* o, float* smax, float* ssum, int n_heads,
                                                   int S, float scale_log2e) {
  constexpr int XCDS = 8;
  const int n_qb = S / (kAttnRowsPerWave * kAttnPPWaves);
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  if (CAUSAL) {
    // Under a causal mask query block b visits 4 b + 4 key tiles.  A workgroup
    // takes blocks b and n_qb - 1 - b one after the other, so every workgroup
    // does the same amount of work and the last round of the launch is full.
    const int n_pair = (n_qb + 1) / 2;
    const int head = (slot / n_pair) * XCDS + xcd;
    const int lo = slot % n_pair;
    const int hi = n_qb - 1 - lo;
    if (head >= n_heads) return;
    attention_fwd_d128_pingpong<true>(q, k, v, o, smax, ssum, S, hi, head, scale_log2e);
    if (lo != hi) attention_fwd_d128_pingpong<true>(q, k, v, o, smax, ssum, S, lo, head, scale_log2e);
  } else {
    const int head = (slot / n_qb) * XCDS + xcd;
    const int qb = slot % n_qb;
    if (head >= n_heads) return;
    attention_fwd_d128_pingpong<false>(q, k, v, o, smax, ssum, S, qb, head, scale_log2e);
  }
}

extern "C" __global__ __launch_bounds__(512, 1) void fused_attention_fwd_bf16_d128_causal_pp(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_pp<true>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
extern "C" __global__ __launch_bounds__(512, 1) void fused_attention_fwd_bf16_d128_full_pp(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_pp<false>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}

// v2: 256 threads, 64 queries per wavefront, one wavefront per SIMD (attention_v2.h).
template <bool CAUSAL>
__device__ __forceinline__ void attention_entry_v2(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                                   bf16_t* o, float* smax, float* ssum, int n_heads,
                                                   int S, float scale_log2e) {
  constexpr int XCDS = 8;
  const int n_qb = S / kAttnV2BM;
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  if (CAUSAL) {
    const int n_pair = (n_qb + 1) / 2;
    const int head = (slot / n_pair) * XCDS + xcd;
    const int lo = slot % n_pair;
    const int hi = n_qb - 1 - lo;
    if (head >= n_heads) return;
    // one copy of the code for both members of the pair (the longer one first)
    const int n_pass = lo != hi ? 2 : 1;
#pragma nounroll
    for (int pass = 0; pass < n_pass; ++pass)
      attention_fwd_d128_v2<true>(q, k, v, o, smax, ssum, S, pass == 0 ? hi : lo, head, scale_log2e);
  } else {
    const int head = (slot / n_qb) * XCDS + xcd;
    const int qb = slot % n_qb;
    if (head >= n_heads) return;
    attention_fwd_d128_v2<false>(q, k, v, o, smax, ssum, S, qb, head, scale_log2e);
  }
}

extern "C" __global__ __launch_bounds__(256, 1) void fused_attention_fwd_bf16_d128_causal_v2(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v2<true>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
extern "C" __global__ __launch_bounds__(256, 1) void fused_attention_fwd_bf16_d128_full_v2(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v2<false>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}

// v4: 512 threads, 32 queries per wavefront, MFMA and softmax interleaved per wavefront
// (attention_v4.h).
template <bool CAUSAL>
__device__ __forceinline__ void attention_entry_v4(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                                   bf16_t* o, float* smax, float* ssum, int n_heads,
                                                   int S, float scale_log2e) {
  constexpr int XCDS = 8;
  const int n_qb = S / kAttnV4BM;
  const int id = blockIdx.x;
  const int xcd = id % XCDS;
  const int slot = id / XCDS;
  if (CAUSAL) {
    const int n_pair = (n_qb + 1) / 2;
    const int head = (slot / n_pair) * XCDS + xcd;
    const int lo = slot % n_pair;
    const int hi = n_qb - 1 - lo;
    if (head >= n_heads) return;
    const int n_pass = lo != hi ? 2 : 1;
#pragma nounroll
    for (int pass = 0; pass < n_pass; ++pass)
      attention_fwd_d128_v4<true>(q, k, v, o, smax, ssum, S, pass == 0 ? hi : lo, head, scale_log2e);
  } else {
    const int head = (slot / n_qb) * XCDS + xcd;
    const int qb = slot % n_qb;
    if (head >= n_heads) return;
    attention_fwd_d128_v4<false>(q, k, v, o, smax, ssum, S, qb, head, scale_log2e);
  }
}

extern "C" __global__ __launch_bounds__(512, 1) void fused_attention_fwd_bf16_d128_causal_v4(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v4<true>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
extern "C" __global__ __launch_bounds__(512, 1) void fused_attention_fwd_bf16_d128_full_v4(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v4<false>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}

// v5: the v4 schedule with K and V tiles loaded straight into LDS and V read back transposed
// (attention_v5.h).  64 KiB of LDS.  The launch is persistent: the grid is at most one workgroup
// per CU and every workgroup walks the work items id = blockIdx.x, blockIdx.x + gridDim.x, ...
// (gridDim.x is a multiple of 8, so a workgroup stays on the heads of its own die).  Between two
// items nothing waits: the output stores of one item drain while the next one loads its queries
// and first key tiles, and no workgroup has to be dispatched in between.  Measured on MI355X at
// [4,32,4096,128]: one workgroup per item spent about 3.4 us per query block on the drain and the
// next dispatch.
template <bool CAUSAL, int WAVES = kAttnV5Waves>
__device__ __forceinline__ void attention_entry_v5(const bf16_t* q, const bf16_t* k, const bf16_t* v,
                                                   bf16_t* o, float* smax, float* ssum, int n_heads,
                                                   int S, float scale_log2e) {
  constexpr int XCDS = 8;
  const int n_qb = S / (32 * WAVES);
  const int per_head = CAUSAL ? (n_qb + 1) / 2 : n_qb;
  const int total = XCDS * ((n_heads + XCDS - 1) / XCDS) * per_head;
#pragma nounroll
  for (int id = blockIdx.x; id < total; id += gridDim.x) {
    const int xcd = id % XCDS;
    const int slot = id / XCDS;
    const int head = (slot / per_head) * XCDS + xcd;
    if (head >= n_heads) continue;
    if (CAUSAL) {
      const int lo = slot % per_head;
      const int hi = n_qb - 1 - lo;
      const int n_pass = lo != hi ? 2 : 1;
#pragma nounroll
      for (int pass = 0; pass < n_pass; ++pass)
        attention_fwd_d128_v5<true, WAVES>(q, k, v, o, smax, ssum, S, pass == 0 ? hi : lo, head, scale_log2e);
    } else {
      attention_fwd_d128_v5<false, WAVES>(q, k, v, o, smax, ssum, S, slot % per_head, head, scale_log2e);
    }
  }
}

extern "C" __global__ __launch_bounds__(512, 1) void fused_attention_fwd_bf16_d128_causal_v5(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v5<true>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
extern "C" __global__ __launch_bounds__(512, 1) void fused_attention_fwd_bf16_d128_full_v5(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v5<false>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}

// v5h: the v5 kernel with four wavefronts (128 queries) per workgroup and two workgroups per CU.
extern "C" __global__ __launch_bounds__(256, 2) void fused_attention_fwd_bf16_d128_causal_v5h(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v5<true, 4>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
extern "C" __global__ __launch_bounds__(256, 2) void fused_attention_fwd_bf16_d128_full_v5h(
    const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum,
    int n_heads, int S, float scale_log2e) {
  attention_entry_v5<false, 4>(q, k, v, o, smax, ssum, n_heads, S, scale_log2e);
}
