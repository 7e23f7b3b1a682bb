// Row-reduction kernels for the two row-shaped graphs of the benchmark:
//   fused_relu_sigmoid_rowsum_f32 :  y[i] = sum_j relu(2*x[i,j]+1) * sigmoid(x[i,j])
//   add_rmsnorm_bf16              :  s = h + r ;  out = s * rsqrt(mean(s^2) + eps) * w
// Numerics follow the reference's lowering: sums accumulate and return fp32
// (reference inductor_x/lowering.py:204-215), 16-bit inputs are widened on load
// and rounded only at the stores (reference inductor_x/codegen/triton.py:1431-1433).
#include "../mi/row.h"

using namespace mi;

namespace {

struct ReluSigmoidRowSum {
  static constexpr int VEC = 4;
  const float* __restrict__ x;
  float* __restrict__ y;
  int rnumel;
  __device__ __forceinline__ float identity() const { return 0.f; }
  __device__ __forceinline__ float combine(float a, float b) const { return a + b; }
  __device__ __forceinline__ float partial(int row, int r) const {
    const Vec<float, 4> v = load_vec_readonly<float, 4>(x + static_cast<size_t>(row) * rnumel + r);
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const float t = v[k];
      const float a = fmaxf(2.0f * t + 1.0f, 0.0f);
      s += a * __builtin_amdgcn_rcpf(1.0f + __expf(-t));
    }
    return s;
  }
  __device__ __forceinline__ void finish(int row, float total) const { y[row] = total; }
};

// Whole row resident in registers: ITERS vectors of 8 bf16 per thread.
template <int BLOCK, int TPR, int ITERS>
__device__ __forceinline__ void add_rmsnorm_bf16_body(const bf16_t* __restrict__ h,
                                                      const bf16_t* __restrict__ r,
                                                      const bf16_t* __restrict__ w,
                                                      bf16_t* __restrict__ out,
                                                      bf16_t* __restrict__ sum_out, int rows,
                                                      int cols, float eps) {
  constexpr int VEC = 8;
  constexpr int ROWS = BLOCK / TPR;
  __shared__ float lds[BLOCK / kWave];
  const int row = blockIdx.x * ROWS + threadIdx.x / TPR;
  const int lane = threadIdx.x % TPR;
  const bool live = row < rows;
  const size_t base = static_cast<size_t>(live ? row : 0) * cols;

  float s[ITERS][VEC];
  Vec<bf16_t, VEC> wv[ITERS];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = (it * TPR + lane) * VEC;
    if (live && c < cols) {
      const Vec<bf16_t, VEC> hv = load_vec<bf16_t, VEC, true>(h + base + c);
      const Vec<bf16_t, VEC> rv = load_vec<bf16_t, VEC, true>(r + base + c);
      wv[it] = load_vec<bf16_t, VEC>(w + c);
      Vec<bf16_t, VEC> sv;
#pragma unroll
      for (int k = 0; k < VEC; ++k) {
        const float t = to_f32(hv[k]) + to_f32(rv[k]);
        s[it][k] = t;
        sv[k] = from_f32<bf16_t>(t);
        ss += t * t;
      }
      store_vec<bf16_t, VEC, true>(sum_out + base + c, sv);
    } else {
#pragma unroll
      for (int k = 0; k < VEC; ++k) s[it][k] = 0.f;
    }
  }
  ss = group_reduce<BLOCK, TPR>(ss, SumOp(), lds);
  const float rs = rsqrtf(ss / static_cast<float>(cols) + eps);
#pragma unroll
  for (int it = 0; it < ITERS; ++it) {
    const int c = (it * TPR + lane) * VEC;
    if (live && c < cols) {
      Vec<bf16_t, VEC> ov;
#pragma unroll
      for (int k = 0; k < VEC; ++k) ov[k] = from_f32<bf16_t>(s[it][k] * rs * to_f32(wv[it][k]));
      store_vec<bf16_t, VEC, true>(out + base + c, ov);
    }
  }
}

}  // namespace

#define ROWSUM_VARIANT(BLOCK, TPR, UNROLL)                                                      \
  extern "C" __global__ __launch_bounds__(BLOCK) void                                           \
      fused_relu_sigmoid_rowsum_f32_b##BLOCK##_t##TPR(const float* x, float* y, int xnumel,     \
                                                      int rnumel) {                             \
    ReluSigmoidRowSum p{x, y, rnumel};                                                          \
    row_reduce_looped<ReluSigmoidRowSum, BLOCK, TPR, UNROLL>(p, xnumel, rnumel);                \
  }

ROWSUM_VARIANT(256, 256, 4)
ROWSUM_VARIANT(256, 128, 8)
ROWSUM_VARIANT(256, 64, 8)
ROWSUM_VARIANT(512, 512, 2)
ROWSUM_VARIANT(1024, 1024, 1)
ROWSUM_VARIANT(512, 256, 4)
ROWSUM_VARIANT(512, 128, 8)
ROWSUM_VARIANT(128, 128, 8)
ROWSUM_VARIANT(64, 64, 16)
ROWSUM_VARIANT(128, 64, 16)
ROWSUM_VARIANT(512, 64, 16)

#define RMSNORM_VARIANT(BLOCK, TPR, ITERS)                                                      \
  extern "C" __global__ __launch_bounds__(BLOCK) void                                           \
      add_rmsnorm_bf16_b##BLOCK##_t##TPR##_i##ITERS(const bf16_t* h, const bf16_t* r,           \
                                                    const bf16_t* w, bf16_t* out,               \
                                                    bf16_t* sum_out, int rows, int cols,        \
                                                    float eps) {                                \
    add_rmsnorm_bf16_body<BLOCK, TPR, ITERS>(h, r, w, out, sum_out, rows, cols, eps);           \
  }

// cols <= TPR * 8 * ITERS must hold; the host picks the variant.
RMSNORM_VARIANT(256, 256, 2)
RMSNORM_VARIANT(256, 128, 4)
RMSNORM_VARIANT(256, 64, 8)
RMSNORM_VARIANT(512, 512, 1)
RMSNORM_VARIANT(256, 256, 1)
RMSNORM_VARIANT(256, 256, 4)
RMSNORM_VARIANT(256, 64, 1)
RMSNORM_VARIANT(256, 64, 2)
RMSNORM_VARIANT(256, 64, 4)
RMSNORM_VARIANT(512, 512, 2)
RMSNORM_VARIANT(512, 512, 4)
