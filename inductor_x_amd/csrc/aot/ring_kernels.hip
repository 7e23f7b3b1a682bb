// Ring-attention merge step (forward_update) instantiations: one kernel per element type of the
// attention outputs, head dimensions 128 and 64, 8 (or 16) sequence positions per workgroup; each
// with plain and with non-temporal loads of the outputs (`_nt`).
#include "../mi/ring.h"

using namespace mi;

#define RING_FWD_VARIANT(NAME, T, D, ST, STREAM)                                                   \
  extern "C" __global__ __launch_bounds__(256) void NAME(                                          \
      const T* prev_out, const float* prev_max, const float* prev_sum, const T* cur_out,           \
      const float* cur_max, const float* cur_sum, T* out, float* out_max, float* out_sum, int S,   \
      int B, int N, long long prev_n_stride, long long cur_n_stride) {                             \
    ring_forward_update<T, D, ST, STREAM>(prev_out, prev_max, prev_sum, cur_out, cur_max, cur_sum, \
                                          out, out_max, out_sum, S, B, N, prev_n_stride,           \
                                          cur_n_stride);                                           \
  }

RING_FWD_VARIANT(ring_forward_update_bf16_d128_s16, bf16_t, 128, 16, false)
RING_FWD_VARIANT(ring_forward_update_bf16_d128_s16_nt, bf16_t, 128, 16, true)
RING_FWD_VARIANT(ring_forward_update_bf16_d128_s8, bf16_t, 128, 8, false)
RING_FWD_VARIANT(ring_forward_update_bf16_d128_s8_nt, bf16_t, 128, 8, true)
RING_FWD_VARIANT(ring_forward_update_f16_d128_s8, f16_t, 128, 8, false)
RING_FWD_VARIANT(ring_forward_update_f16_d128_s8_nt, f16_t, 128, 8, true)
RING_FWD_VARIANT(ring_forward_update_f32_d128_s8, float, 128, 8, false)
RING_FWD_VARIANT(ring_forward_update_f32_d128_s8_nt, float, 128, 8, true)
RING_FWD_VARIANT(ring_forward_update_bf16_d64_s8, bf16_t, 64, 8, false)
RING_FWD_VARIANT(ring_forward_update_bf16_d64_s8_nt, bf16_t, 64, 8, true)
RING_FWD_VARIANT(ring_forward_update_f16_d64_s8, f16_t, 64, 8, false)
RING_FWD_VARIANT(ring_forward_update_f16_d64_s8_nt, f16_t, 64, 8, true)
RING_FWD_VARIANT(ring_forward_update_f32_d64_s8, float, 64, 8, false)
RING_FWD_VARIANT(ring_forward_update_f32_d64_s8_nt, float, 64, 8, true)

