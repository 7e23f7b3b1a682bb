// Split column reduction for the third benchmark graph: per-column mean,
// variance (correction given at run time) and int64 argmax over dim 0 of an fp32
// matrix, in one sweep over the input plus a small combine pass.
#include "../mi/col.h"

using namespace mi;

// Dynamic LDS for pass 1: col_fold_planes(CT, RL) * CT * 4 * 5 floats.
#define COL_PARTIAL_VARIANT(CT, RL, UNROLL)                                                   \
  extern "C" __global__ __launch_bounds__(CT* RL) void                                        \
      col_mean_var_argmax_partial_f32_c##CT##_r##RL##_u##UNROLL(                              \
          const float* x, float* part, int rows, int cols, int nsplit) {                      \
    col_stats_partial<CT, RL, UNROLL>(x, part, rows, cols, nsplit);                           \
  }

// the same with PF batches of loads held per thread instead of two
#define COL_PARTIAL_VARIANT_PF(CT, RL, UNROLL, PF)                                            \
  extern "C" __global__ __launch_bounds__(CT* RL) void                                        \
      col_mean_var_argmax_partial_f32_c##CT##_r##RL##_u##UNROLL##_p##PF(                      \
          const float* x, float* part, int rows, int cols, int nsplit) {                      \
    col_stats_partial<CT, RL, UNROLL, PF>(x, part, rows, cols, nsplit);                       \
  }

COL_PARTIAL_VARIANT_PF(32, 8, 8, 3)
COL_PARTIAL_VARIANT_PF(32, 8, 8, 4)
COL_PARTIAL_VARIANT_PF(32, 8, 4, 3)
COL_PARTIAL_VARIANT_PF(32, 8, 4, 4)
COL_PARTIAL_VARIANT_PF(32, 16, 4, 3)
COL_PARTIAL_VARIANT_PF(32, 16, 8, 3)
COL_PARTIAL_VARIANT_PF(32, 8, 16, 3)
COL_PARTIAL_VARIANT_PF(64, 8, 8, 3)

COL_PARTIAL_VARIANT(128, 2, 4)
COL_PARTIAL_VARIANT(128, 2, 8)
COL_PARTIAL_VARIANT(128, 4, 4)
COL_PARTIAL_VARIANT(128, 4, 8)
COL_PARTIAL_VARIANT(128, 8, 4)
COL_PARTIAL_VARIANT(128, 8, 8)
COL_PARTIAL_VARIANT(64, 4, 4)
COL_PARTIAL_VARIANT(64, 4, 8)
COL_PARTIAL_VARIANT(64, 8, 4)
COL_PARTIAL_VARIANT(64, 16, 4)
COL_PARTIAL_VARIANT(64, 1, 8)
COL_PARTIAL_VARIANT(16, 16, 4)
COL_PARTIAL_VARIANT(1, 64, 4)
COL_PARTIAL_VARIANT(16, 64, 4)
COL_PARTIAL_VARIANT(32, 32, 4)
COL_PARTIAL_VARIANT(32, 16, 4)
COL_PARTIAL_VARIANT(16, 32, 4)
COL_PARTIAL_VARIANT(64, 8, 8)
COL_PARTIAL_VARIANT(32, 8, 4)
COL_PARTIAL_VARIANT(32, 8, 8)
COL_PARTIAL_VARIANT(32, 16, 8)
COL_PARTIAL_VARIANT(64, 16, 8)
COL_PARTIAL_VARIANT(64, 4, 16)
COL_PARTIAL_VARIANT(32, 8, 16)
COL_PARTIAL_VARIANT(128, 4, 16)
COL_PARTIAL_VARIANT(128, 2, 16)
COL_PARTIAL_VARIANT(16, 16, 8)

#define COL_FINAL_VARIANT(CPW, SL)                                                            \
  extern "C" __global__ __launch_bounds__(CPW* SL) void                                       \
      col_mean_var_argmax_final_f32_c##CPW##_s##SL(const float* part, float* mean_out,        \
                                                   float* var_out, long long* argmax_out,     \
                                                   int cols, int nsplit, int rows, int batch, \
                                                   float correction) {                        \
    col_stats_final<CPW, SL>(part, mean_out, var_out, argmax_out, cols, nsplit, rows, batch,  \
                             correction);                                                     \
  }

COL_FINAL_VARIANT(16, 16)
COL_FINAL_VARIANT(16, 32)
COL_FINAL_VARIANT(8, 64)
COL_FINAL_VARIANT(8, 32)
COL_FINAL_VARIANT(4, 64)
COL_FINAL_VARIANT(64, 4)
COL_FINAL_VARIANT(4, 16)
COL_FINAL_VARIANT(4, 32)
COL_FINAL_VARIANT(2, 64)
COL_FINAL_VARIANT(2, 32)
COL_FINAL_VARIANT(8, 16)
COL_FINAL_VARIANT(8, 8)
COL_FINAL_VARIANT(16, 4)
COL_FINAL_VARIANT(16, 8)
