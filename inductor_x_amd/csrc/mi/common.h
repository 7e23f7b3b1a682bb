// Device-side building blocks shared by every gfx950 kernel of the backend:
// 128-bit vector access, bf16 conversion, wavefront (64-lane) DPP/shuffle
// reductions and LDS-staged workgroup reductions.
//
// This header plays the role the reference gives to its Triton helper shims
// (reference inductor_x/npu_triton_helpers.py:4-18): the small set of device
// functions that generated kernels are allowed to call.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mi {

constexpr int kWave = 64;  // CDNA4 wavefront width

typedef __bf16 bf16_t;
typedef _Float16 f16_t;

// ---------------------------------------------------------------------------
// Vector access.  A Vec<T, N> of 16 bytes moves as one global_load_dwordx4 /
// global_store_dwordx4; narrower ones as dwordx2 / dword / short.
// ---------------------------------------------------------------------------
template <int BYTES>
struct RawBits;
template <>
struct RawBits<16> {
  typedef uint32_t type __attribute__((ext_vector_type(4)));
};
template <>
struct RawBits<8> {
  typedef uint32_t type __attribute__((ext_vector_type(2)));
};
template <>
struct RawBits<4> {
  typedef uint32_t type;
};
template <>
struct RawBits<2> {
  typedef uint16_t type;
};
template <>
struct RawBits<1> {
  typedef uint8_t type;
};

template <typename T, int N>
struct alignas(sizeof(T) * N) Vec {
  T v[N];
  __device__ __forceinline__ T& operator[](int i) { return v[i]; }
  __device__ __forceinline__ const T& operator[](int i) const { return v[i]; }
};

// STREAM = true marks the access non-temporal (data touched once).  Whether the
// hint is honoured is a build-time switch per direction, so it can be measured.
// Measured on MI355X (add+rmsnorm, gather, permute at 128-512 MiB): the hint on
// loads costs 10-15 % of bandwidth, the hint on stores gains up to 20 %.
#ifndef MI_NT_LOADS
#define MI_NT_LOADS 0
#endif
#ifndef MI_NT_STORES
#define MI_NT_STORES 1
#endif
template <typename T, int N, bool STREAM = false>
__device__ __forceinline__ Vec<T, N> load_vec(const T* __restrict__ p) {
  constexpr int B = sizeof(T) * N;
  static_assert(B == 16 || B == 8 || B == 4 || B == 2 || B == 1, "vector must be 1..16 bytes");
  typedef typename RawBits<B>::type raw_t;
  raw_t r;
  if constexpr (STREAM && MI_NT_LOADS) {
    r = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p));
  } else {
    r = *reinterpret_cast<const raw_t*>(p);
  }
  Vec<T, N> out;
  __builtin_memcpy(&out, &r, B);
  return out;
}

// Load whose non-temporal hint is a template argument of the kernel itself (not a build-time
// switch): for kernel families that are instantiated both ways and picked per launch from the size
// of what the launch reads.
template <typename T, int N, bool NONTEMPORAL>
__device__ __forceinline__ Vec<T, N> load_vec_hint(const T* __restrict__ p) {
  constexpr int B = sizeof(T) * N;
  static_assert(B == 16 || B == 8 || B == 4 || B == 2 || B == 1, "vector must be 1..16 bytes");
  typedef typename RawBits<B>::type raw_t;
  raw_t r;
  if constexpr (NONTEMPORAL) {
    r = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p));
  } else {
    r = *reinterpret_cast<const raw_t*>(p);
  }
  Vec<T, N> out;
  __builtin_memcpy(&out, &r, B);
  return out;
}

// Load for kernels that only read (a reduction's sweep over its input), with a hint switch of
// its own.  Measured on MI355X with a plain summing kernel: 1 GiB streams at 7.2-7.3 TB/s with
// the non-temporal hint against 6.5-6.7 TB/s without, 128 MiB takes 17.9 us against 19.0 us.
// The hint also keeps the data out of the memory-side cache: a 16 MiB row sum that is launched
// again on the same input goes from 3.4 to 4.4 us with it, and the column statistics sweep of
// 128 MiB is 0.2 us slower, so it is off by default.
#ifndef MI_NT_READONLY
#define MI_NT_READONLY 0
#endif
template <typename T, int N>
__device__ __forceinline__ Vec<T, N> load_vec_readonly(const T* __restrict__ p) {
  constexpr int B = sizeof(T) * N;
  typedef typename RawBits<B>::type raw_t;
  raw_t r;
  if constexpr (MI_NT_READONLY) {
    r = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p));
  } else {
    r = *reinterpret_cast<const raw_t*>(p);
  }
  Vec<T, N> out;
  __builtin_memcpy(&out, &r, B);
  return out;
}

template <typename T, int N, bool STREAM = false>
__device__ __forceinline__ void store_vec(T* __restrict__ p, const Vec<T, N>& val) {
  constexpr int B = sizeof(T) * N;
  static_assert(B == 16 || B == 8 || B == 4 || B == 2 || B == 1, "vector must be 1..16 bytes");
  typedef typename RawBits<B>::type raw_t;
  raw_t r;
  __builtin_memcpy(&r, &val, B);
  if constexpr (STREAM && MI_NT_STORES) {
    __builtin_nontemporal_store(r, reinterpret_cast<raw_t*>(p));
  } else {
    *reinterpret_cast<raw_t*>(p) = r;
  }
}

// ---------------------------------------------------------------------------
// Element conversion.  Loads of 16-bit floats are widened to fp32 and all
// arithmetic stays in fp32; rounding (RNE) happens only when a value is
// stored (reference inductor_x/codegen/triton.py:1431-1433).
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ float to_f32(T x) {
  return static_cast<float>(x);
}
template <typename T>
__device__ __forceinline__ T from_f32(float x) {
  return static_cast<T>(x);
}

// ---------------------------------------------------------------------------
// Wavefront reductions.  Steps inside a 16-lane row use DPP (no LDS traffic);
// the two cross-row steps use a lane shuffle.  All 64 lanes end with the
// result, and the combination order is fixed, so results are reproducible.
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_move(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}

constexpr int kDppQuadSwap1 = 0xB1;      // quad_perm [1,0,3,2]
constexpr int kDppQuadSwap2 = 0x4E;      // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i <-> 7-i inside 8 lanes
constexpr int kDppRowMirror = 0x140;      // lane i <-> 15-i inside 16 lanes

struct SumOp {
  __device__ __forceinline__ float operator()(float a, float b) const { return a + b; }
};
struct MaxOp {
  // NaN-propagating maximum, as torch.max.
  __device__ __forceinline__ float operator()(float a, float b) const {
    // one maximum, one unordered compare, one select
    return __builtin_isunordered(a, b) ? __builtin_nanf("") : __builtin_fmaxf(a, b);
  }
};
struct MinOp {
  __device__ __forceinline__ float operator()(float a, float b) const {
    return __builtin_isunordered(a, b) ? __builtin_nanf("") : __builtin_fminf(a, b);
  }
};

// Reduce over groups of WIDTH consecutive lanes (WIDTH a power of two <= 64).
template <int WIDTH = kWave, class Op>
__device__ __forceinline__ float wave_reduce(float v, Op op) {
  static_assert(WIDTH >= 1 && WIDTH <= 64 && (WIDTH & (WIDTH - 1)) == 0, "bad reduce width");
  if constexpr (WIDTH >= 2) v = op(v, dpp_move<kDppQuadSwap1>(v));
  if constexpr (WIDTH >= 4) v = op(v, dpp_move<kDppQuadSwap2>(v));
  if constexpr (WIDTH >= 8) v = op(v, dpp_move<kDppRowHalfMirror>(v));
  if constexpr (WIDTH >= 16) v = op(v, dpp_move<kDppRowMirror>(v));
  if constexpr (WIDTH >= 32) v = op(v, __shfl_xor(v, 16, kWave));
  if constexpr (WIDTH >= 64) v = op(v, __shfl_xor(v, 32, kWave));
  return v;
}

template <int WIDTH = kWave>
__device__ __forceinline__ float wave_sum(float v) {
  return wave_reduce<WIDTH>(v, SumOp());
}

// Workgroup reduction of one float per thread over groups of GROUP consecutive
// threads (GROUP a power of two, a multiple of 64 when > 64).  `lds` must hold
// BLOCK / 64 floats and may be reused after the call returns (a barrier is
// issued on both sides).  Every thread of the group receives the result.
template <int BLOCK, int GROUP, class Op>
__device__ __forceinline__ float group_reduce(float v, Op op, float* lds) {
  if constexpr (GROUP <= kWave) {
    return wave_reduce<GROUP>(v, op);
  } else {
    static_assert(GROUP % kWave == 0 && BLOCK % GROUP == 0, "group must be whole waves");
    constexpr int WAVES_PER_GROUP = GROUP / kWave;
    v = wave_reduce<kWave>(v, op);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = v;
    __syncthreads();
    // lane j of every wavefront takes the partial of wavefront j of its group; the partials
    // then meet in log2 steps inside 16 lanes (at most 16 wavefronts per workgroup)
    static_assert(WAVES_PER_GROUP <= 16, "a workgroup has at most 16 wavefronts");
    const int first = (wave / WAVES_PER_GROUP) * WAVES_PER_GROUP;
    return wave_reduce<WAVES_PER_GROUP>(lds[first + (threadIdx.x & (WAVES_PER_GROUP - 1))], op);
  }
}

// ---------------------------------------------------------------------------
// Arg-reduction element.  Combination rule (the one Inductor's
// maximum_with_index implements and the reference inherits,
// reference inductor_x/codegen/triton.py:1217-1233): the greater value wins,
// NaN beats every number, equal values (or two NaNs) keep the lower index.
// ---------------------------------------------------------------------------
struct ArgVal {
  float v;
  int i;
};

__device__ __forceinline__ bool argmax_takes_b(float av, int ai, float bv, int bi) {
  const bool a_nan = av != av, b_nan = bv != bv;
  const bool eq = (av == bv) || (a_nan && b_nan);
  return (bv > av) || (b_nan && !a_nan) || (eq && bi < ai);
}
__device__ __forceinline__ bool argmin_takes_b(float av, int ai, float bv, int bi) {
  const bool a_nan = av != av, b_nan = bv != bv;
  const bool eq = (av == bv) || (a_nan && b_nan);
  return (bv < av) || (b_nan && !a_nan) || (eq && bi < ai);
}

template <bool IS_MAX>
__device__ __forceinline__ ArgVal arg_combine(ArgVal a, ArgVal b) {
  const bool take_b = IS_MAX ? argmax_takes_b(a.v, a.i, b.v, b.i) : argmin_takes_b(a.v, a.i, b.v, b.i);
  return take_b ? b : a;
}

template <int WIDTH, bool IS_MAX>
__device__ __forceinline__ ArgVal wave_arg_reduce(ArgVal a) {
#pragma unroll
  for (int off = 1; off < WIDTH; off <<= 1) {
    ArgVal b;
    b.v = __shfl_xor(a.v, off, kWave);
    b.i = __shfl_xor(a.i, off, kWave);
    a = arg_combine<IS_MAX>(a, b);
  }
  return a;
}

// ---------------------------------------------------------------------------
// Running (count, mean, M2) triple and Chan's pairwise combination.
// ---------------------------------------------------------------------------
struct Moments {
  float n, mean, m2;
};

__device__ __forceinline__ Moments moments_combine(Moments a, Moments b) {
  const float n = a.n + b.n;
  if (n == 0.f) return a;
  const float delta = b.mean - a.mean;
  const float wb = b.n * __builtin_amdgcn_rcpf(n);
  Moments r;
  r.n = n;
  r.mean = a.mean + delta * wb;
  r.m2 = a.m2 + b.m2 + delta * delta * a.n * wb;
  return r;
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + __expf(-x)); }

}  // namespace mi
