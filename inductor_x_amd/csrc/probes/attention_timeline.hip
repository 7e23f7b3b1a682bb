// Measurement build of the fused attention forward, not part of any graph: the shipped kernel template
// with a timeline hook that records the 100 MHz real-time clock at seven points of every query block
// (attention_v5.h, AttnNoTimeline).  Wavefronts 0 and 7 of a workgroup write eight 64-bit words per query
// block into `times`, laid out [head][query block][wavefront 0 | 7][8]: words 0..6 are the clock at the
// seven points, word 7 is the workgroup id.  bench.py --attention-timeline launches it and prints where a
// workgroup's time goes; the stores and clock reads cost about 0.1 us per point.
#include "../mi/attention_v5.h"

using namespace mi;

namespace {

struct AttnTimeline {
  unsigned long long* times;
  int blocks_per_head;
  __device__ __forceinline__ void mark(int point, int head, int q_block) const {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0 && (wave == 0 || wave == 7)) {
      unsigned long long* slot =
          times + (static_cast<size_t>(head * blocks_per_head + q_block) * 2 + (wave ? 1 : 0)) * 8;
      slot[point] = __builtin_amdgcn_s_memrealtime();
      if (point == 0) slot[7] = blockIdx.x;
    }
  }
};

}  // namespace

#define ATTENTION_TIMELINE(NAME, CAUSAL)                                                                     \
  extern "C" __global__ __launch_bounds__(512, 1) void NAME(                                                 \
      const bf16_t* q, const bf16_t* k, const bf16_t* v, bf16_t* o, float* smax, float* ssum, int n_heads,   \
      int Sq, int Sk, float scale_log2e, unsigned long long* times) {                                        \
    attention_entry_v5<bf16_t, CAUSAL, false, 128, false, AttnTimeline>(                                     \
        q, k, v, o, smax, ssum, n_heads, Sq, Sk, scale_log2e, nullptr, 0, 0, 1,                              \
        AttnTimeline{times, Sq / kAttnV5BM});                                                                \
  }

ATTENTION_TIMELINE(attention_timeline_bf16_d128_causal, true)
ATTENTION_TIMELINE(attention_timeline_bf16_d128_full, false)
