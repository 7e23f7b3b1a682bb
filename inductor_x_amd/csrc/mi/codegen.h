// Building blocks for kernels emitted by the Inductor code generator.
//
// A generated kernel is straight-line C++ over two kinds of values: scalars
// (uniform for the thread) and V<T, N> register vectors (N consecutive
// elements along the contiguous axis).  Every operator and math function below
// accepts any mix of the two, so the generator prints one expression per
// Inductor op and lets overload resolution widen scalars where needed.
//
// Four code shapes are built from these pieces (the first three mirror the reference's
// pointwise / row-reduction / higher-order-reduction kernel bodies,
// reference inductor_x/codegen/triton.py:693-815, 1103-1262):
//   pointwise  one V per thread, 128-bit loads and stores where the index
//              is contiguous along the vector axis, gathers elsewhere;
//   row        TPR threads share a row, each holds one V of it (or walks
//              the row in a loop), results meet through DPP and LDS;
//   column     every vector lane is its own output column, row lanes of the
//              workgroup meet through LDS, slices of the reduced axis meet
//              through a workspace and a second kernel (or not at all when one
//              slice is enough);
//   colloop    the column thread mapping in one kernel: a loop over the reduced
//              axis per phase, folded states shared with every row lane.
#pragma once

#include <type_traits>

#include "common.h"

namespace mi {

typedef long long i64;

// ---------------------------------------------------------------------------
// register vector + scalar/vector-generic elementwise application
// ---------------------------------------------------------------------------
template <typename T, int N>
struct V {
  T v[N];
  __device__ __forceinline__ T& operator[](int i) { return v[i]; }
  __device__ __forceinline__ const T& operator[](int i) const { return v[i]; }
};

template <class A>
struct Tr {
  static constexpr int n = 0;
  typedef A elem;
};
template <class T, int N>
struct Tr<V<T, N>> {
  static constexpr int n = N;
  typedef T elem;
};

template <class A>
__device__ __forceinline__ auto at(const A& a, int i) {
  if constexpr (Tr<A>::n != 0) {
    return a.v[i];
  } else {
    return a;
  }
}

// A value that is the same for all N elements of a thread, as N lanes (no-op for vectors): a
// reduction must count it once per element.
template <int N, class A>
__device__ __forceinline__ auto splat(const A& a) {
  if constexpr (Tr<A>::n != 0 || N <= 1) {
    return a;
  } else {
    V<A, N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = a;
    return r;
  }
}

template <int... Ns>
struct MaxN;
template <int A>
struct MaxN<A> {
  static constexpr int value = A;
};
template <int A, int... Rest>
struct MaxN<A, Rest...> {
  static constexpr int value = A > MaxN<Rest...>::value ? A : MaxN<Rest...>::value;
};

template <class F, class... A>
__device__ __forceinline__ auto apply(F f, const A&... a) {
  constexpr int n = MaxN<Tr<A>::n...>::value;
  if constexpr (n == 0) {
    return f(a...);
  } else {
    V<decltype(f(at(a, 0)...)), n> r;
#pragma unroll
    for (int i = 0; i < n; ++i) r.v[i] = f(at(a, i)...);
    return r;
  }
}

template <class A, class B>
using EnableIfAnyVec = typename std::enable_if<(Tr<A>::n != 0 || Tr<B>::n != 0), int>::type;

#define MI_BINARY_OPERATOR(OP)                                                         \
  template <class A, class B, EnableIfAnyVec<A, B> = 0>                                \
  __device__ __forceinline__ auto operator OP(const A& a, const B& b) {                \
    return apply([](auto x, auto y) { return x OP y; }, a, b);                         \
  }
MI_BINARY_OPERATOR(+)
MI_BINARY_OPERATOR(-)
MI_BINARY_OPERATOR(*)
MI_BINARY_OPERATOR(/)
MI_BINARY_OPERATOR(%)
MI_BINARY_OPERATOR(<)
MI_BINARY_OPERATOR(<=)
MI_BINARY_OPERATOR(>)
MI_BINARY_OPERATOR(>=)
MI_BINARY_OPERATOR(==)
MI_BINARY_OPERATOR(!=)
MI_BINARY_OPERATOR(&)
MI_BINARY_OPERATOR(|)
MI_BINARY_OPERATOR(^)
MI_BINARY_OPERATOR(<<)
MI_BINARY_OPERATOR(>>)
MI_BINARY_OPERATOR(&&)
MI_BINARY_OPERATOR(||)
#undef MI_BINARY_OPERATOR

template <class T, int N>
__device__ __forceinline__ auto operator-(const V<T, N>& a) {
  return apply([](auto x) { return -x; }, a);
}
template <class T, int N>
__device__ __forceinline__ auto operator!(const V<T, N>& a) {
  return apply([](auto x) { return !x; }, a);
}
template <class T, int N>
__device__ __forceinline__ auto operator~(const V<T, N>& a) {
  return apply([](auto x) { return ~x; }, a);
}

// 0, 1, ..., N-1 as a vector (N == 1 gives a plain 0 so scalar code stays scalar)
template <int N>
__device__ __forceinline__ auto iota() {
  if constexpr (N == 1) {
    return 0;
  } else {
    V<int, N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = i;
    return r;
  }
}

// A float that the target integer type cannot hold (a negative number to uint8) is undefined
// in a direct conversion, and the optimiser may then garble neighbouring lanes of the vector as
// well.  Narrow and unsigned integer targets are reached through a wider signed integer, which
// wraps the way ATen's own conversion does (c10 static_cast_with_inter_type: uint8 via int64).
template <class T, class A>
__device__ __forceinline__ auto cast(const A& a) {
  return apply(
      [](auto x) {
        typedef decltype(x) X;
        if constexpr (std::is_floating_point<X>::value && std::is_integral<T>::value &&
                      !std::is_same<T, bool>::value && (sizeof(T) < 4 || std::is_unsigned<T>::value)) {
          if constexpr (sizeof(T) < 4) {
            return static_cast<T>(static_cast<int>(x));
          } else {
            return static_cast<T>(static_cast<long long>(x));
          }
        } else {
          return static_cast<T>(x);
        }
      },
      a);
}
template <class T, class A>
__device__ __forceinline__ auto bitcast(const A& a) {
  return apply([](auto x) { return __builtin_bit_cast(T, x); }, a);
}
template <class C, class A, class B>
__device__ __forceinline__ auto where(const C& c, const A& a, const B& b) {
  return apply(
      [](bool cc, auto x, auto y) {
        typedef decltype(true ? x : y) R;
        return cc ? static_cast<R>(x) : static_cast<R>(y);
      },
      c, a, b);
}

// ---------------------------------------------------------------------------
// math (fp32 unless noted)
// ---------------------------------------------------------------------------
// tanh and erf as odd rational functions x * P(x^2) / Q(x^2) on a clamped argument (both are
// within 4e-7 of 1 in magnitude beyond the clamp): seven and four (five) fused multiply-adds and
// one reciprocal, no branches, measured against double precision at 2.2 million points:
// relative error <= 4.5e-7 for both.  The library routines branch on the magnitude of the
// argument, and a wavefront pays for every branch its lanes take: an activation over a large
// tensor was bound by them, not by memory.  NaN passes through the comparisons of the clamp.
__device__ __forceinline__ float clamp_keep_nan(float x, float lim) { return x < -lim ? -lim : (x > lim ? lim : x); }
__device__ __forceinline__ float tanh_f32(float x) {
  x = clamp_keep_nan(x, 9.0f);
  const float t = x * x;
  float p = -2.76076847742355e-16f;
  p = fmaf(p, t, 2.00018790482477e-13f);
  p = fmaf(p, t, -8.60467152213735e-11f);
  p = fmaf(p, t, 5.12229709037114e-08f);
  p = fmaf(p, t, 1.48572235717979e-05f);
  p = fmaf(p, t, 6.37261928875436e-04f);
  p = fmaf(p, t, 4.89352455891786e-03f);
  float q = 1.19825839466702e-06f;
  q = fmaf(q, t, 1.18534705686654e-04f);
  q = fmaf(q, t, 2.26843463243900e-03f);
  q = fmaf(q, t, 4.89352518554385e-03f);
  return (p * x) * __builtin_amdgcn_rcpf(q);
}
__device__ __forceinline__ float erf_f32(float x) {
  x = clamp_keep_nan(x, 4.0f);
  const float t = x * x;
  float p = -2.72614225801306e-10f;
  p = fmaf(p, t, 2.77068142495902e-08f);
  p = fmaf(p, t, -2.10102402082508e-06f);
  p = fmaf(p, t, -5.69250639462346e-05f);
  p = fmaf(p, t, -7.34990630326855e-04f);
  p = fmaf(p, t, -2.95459980854025e-03f);
  p = fmaf(p, t, -1.60960333262415e-02f);
  float q = -1.45660718464996e-05f;
  q = fmaf(q, t, -2.13374055278905e-04f);
  q = fmaf(q, t, -1.68282697438203e-03f);
  q = fmaf(q, t, -7.37332916720468e-03f);
  q = fmaf(q, t, -1.42647390514189e-02f);
  return (p * x) * __builtin_amdgcn_rcpf(q);
}

// Float and double forms: fp64 tensors are computed in fp64 (x is the element, already of its
// own type); everything narrower has been widened to fp32 by the load.
#define MI_UNARY_FN(NAME, FEXPR, DEXPR)                           \
  template <class A>                                              \
  __device__ __forceinline__ auto NAME(const A& a) {              \
    return apply(                                                 \
        [](auto x) {                                              \
          if constexpr (std::is_same<decltype(x), double>::value) { \
            return DEXPR;                                         \
          } else {                                                \
            return FEXPR;                                         \
          }                                                       \
        },                                                        \
        a);                                                       \
  }
MI_UNARY_FN(exp, __expf(static_cast<float>(x)), ::exp(x))
MI_UNARY_FN(exp2, __builtin_amdgcn_exp2f(static_cast<float>(x)), ::exp2(x))
MI_UNARY_FN(expm1, ::expm1f(static_cast<float>(x)), ::expm1(x))
MI_UNARY_FN(log, ::logf(static_cast<float>(x)), ::log(x))
MI_UNARY_FN(log2, ::log2f(static_cast<float>(x)), ::log2(x))
MI_UNARY_FN(log10, ::log10f(static_cast<float>(x)), ::log10(x))
MI_UNARY_FN(log1p, ::log1pf(static_cast<float>(x)), ::log1p(x))
MI_UNARY_FN(sqrt, ::sqrtf(static_cast<float>(x)), ::sqrt(x))
MI_UNARY_FN(rsqrt, ::rsqrtf(static_cast<float>(x)), 1.0 / ::sqrt(x))
MI_UNARY_FN(sin, ::sinf(static_cast<float>(x)), ::sin(x))
MI_UNARY_FN(cos, ::cosf(static_cast<float>(x)), ::cos(x))
MI_UNARY_FN(tan, ::tanf(static_cast<float>(x)), ::tan(x))
MI_UNARY_FN(tanh, tanh_f32(static_cast<float>(x)), ::tanh(x))
MI_UNARY_FN(sinh, ::sinhf(static_cast<float>(x)), ::sinh(x))
MI_UNARY_FN(cosh, ::coshf(static_cast<float>(x)), ::cosh(x))
MI_UNARY_FN(asin, ::asinf(static_cast<float>(x)), ::asin(x))
MI_UNARY_FN(acos, ::acosf(static_cast<float>(x)), ::acos(x))
MI_UNARY_FN(atan, ::atanf(static_cast<float>(x)), ::atan(x))
MI_UNARY_FN(erf, erf_f32(static_cast<float>(x)), ::erf(x))
MI_UNARY_FN(erfc, ::erfcf(static_cast<float>(x)), ::erfc(x))
MI_UNARY_FN(lgamma, ::lgammaf(static_cast<float>(x)), ::lgamma(x))
MI_UNARY_FN(floor, ::floorf(static_cast<float>(x)), ::floor(x))
MI_UNARY_FN(ceil, ::ceilf(static_cast<float>(x)), ::ceil(x))
MI_UNARY_FN(trunc, ::truncf(static_cast<float>(x)), ::trunc(x))
MI_UNARY_FN(round, ::nearbyintf(static_cast<float>(x)), ::nearbyint(x))
MI_UNARY_FN(reciprocal, 1.0f / static_cast<float>(x), 1.0 / x)
MI_UNARY_FN(sigmoid, __builtin_amdgcn_rcpf(1.0f + __expf(-static_cast<float>(x))), 1.0 / (1.0 + ::exp(-x)))
MI_UNARY_FN(isnan, (x != x), (x != x))
MI_UNARY_FN(isinf, (::isinf(static_cast<float>(x)) != 0), (::isinf(x) != 0))
MI_UNARY_FN(signbit, (::signbit(static_cast<float>(x)) != 0), (::signbit(x) != 0))
MI_UNARY_FN(abs, (x < 0 ? -x : x), ::fabs(x))
MI_UNARY_FN(logical_not, (!x), (!x))
// relu keeps NaN (a plain fmaxf would drop it)
MI_UNARY_FN(relu, (x != x ? x : (x > 0 ? x : static_cast<decltype(x)>(0))), (x != x ? x : (x > 0 ? x : 0.0)))
#undef MI_UNARY_FN

template <class A>
__device__ __forceinline__ auto sign(const A& a) {
  return apply([](auto x) { return static_cast<decltype(x)>((x > 0) - (x < 0)); }, a);
}

#define MI_BINARY_FN(NAME, EXPR)                                   \
  template <class A, class B>                                      \
  __device__ __forceinline__ auto NAME(const A& a, const B& b) {   \
    return apply([](auto x, auto y) { return EXPR; }, a, b);       \
  }
// NaN-propagating, as torch.maximum / torch.minimum
MI_BINARY_FN(maximum, (x != x ? x : (y != y ? static_cast<decltype(x)>(y) : (x > y ? x : static_cast<decltype(x)>(y)))))
MI_BINARY_FN(minimum, (x != x ? x : (y != y ? static_cast<decltype(x)>(y) : (x < y ? x : static_cast<decltype(x)>(y)))))
#undef MI_BINARY_FN
#define MI_BINARY_MATH(NAME, FFN, DFN)                                                         \
  template <class A, class B>                                                                  \
  __device__ __forceinline__ auto NAME(const A& a, const B& b) {                               \
    return apply(                                                                              \
        [](auto x, auto y) {                                                                   \
          if constexpr (std::is_same<decltype(x), double>::value || std::is_same<decltype(y), double>::value) { \
            return DFN(static_cast<double>(x), static_cast<double>(y));                        \
          } else {                                                                             \
            return FFN(static_cast<float>(x), static_cast<float>(y));                          \
          }                                                                                    \
        },                                                                                     \
        a, b);                                                                                 \
  }
MI_BINARY_MATH(pow, ::powf, ::pow)
MI_BINARY_MATH(atan2, ::atan2f, ::atan2)
MI_BINARY_MATH(fmod, ::fmodf, ::fmod)
MI_BINARY_MATH(copysign, ::copysignf, ::copysign)
#undef MI_BINARY_MATH
#define MI_BINARY_FN(NAME, EXPR)                                   \
  template <class A, class B>                                      \
  __device__ __forceinline__ auto NAME(const A& a, const B& b) {   \
    return apply([](auto x, auto y) { return EXPR; }, a, b);       \
  }
// Python-style integer floor division and modulo
MI_BINARY_FN(floordiv, ((x / y) - ((x % y != 0) && ((x < 0) != (y < 0)) ? 1 : 0)))
MI_BINARY_FN(pymod, (((x % y) != 0 && ((x % y) < 0) != (y < 0)) ? (x % y) + y : (x % y)))
MI_BINARY_FN(truncdiv, (x / y))
MI_BINARY_FN(logical_and, (static_cast<bool>(x) && static_cast<bool>(y)))
MI_BINARY_FN(logical_or, (static_cast<bool>(x) || static_cast<bool>(y)))
MI_BINARY_FN(logical_xor, (static_cast<bool>(x) != static_cast<bool>(y)))
// float remainder with the sign of the divisor (torch.remainder)
MI_BINARY_FN(remainder_f, (::fmodf(static_cast<float>(x), static_cast<float>(y)) != 0.f &&
                                   ((::fmodf(static_cast<float>(x), static_cast<float>(y)) < 0.f) != (static_cast<float>(y) < 0.f))
                               ? ::fmodf(static_cast<float>(x), static_cast<float>(y)) + static_cast<float>(y)
                               : ::fmodf(static_cast<float>(x), static_cast<float>(y))))
#undef MI_BINARY_FN

// Division.  A vector divided by a value that is uniform for the thread (a row sum, a norm)
// takes one correctly rounded reciprocal and a multiplication per element (within one ulp of
// the quotient); everything else is the IEEE division.
template <class A, class B>
__device__ __forceinline__ auto truediv(const A& a, const B& b) {
  if constexpr (Tr<A>::n != 0 && Tr<B>::n == 0 && !std::is_same<B, double>::value &&
                !std::is_same<typename Tr<A>::elem, double>::value) {
    const float inv = 1.0f / static_cast<float>(b);
    return apply([inv](auto x) { return static_cast<float>(x) * inv; }, a);
  } else {
    return apply(
        [](auto x, auto y) {
          if constexpr (std::is_same<decltype(x), double>::value || std::is_same<decltype(y), double>::value) {
            return static_cast<double>(x) / static_cast<double>(y);
          } else {
            return static_cast<float>(x) / static_cast<float>(y);
          }
        },
        a, b);
  }
}

template <class A, class B, class C>
__device__ __forceinline__ auto fma(const A& a, const B& b, const C& c) {
  return apply([](float x, float y, float z) { return ::fmaf(x, y, z); }, a, b, c);
}

// ---------------------------------------------------------------------------
// loads / stores
// ---------------------------------------------------------------------------
// Contiguous, aligned run of N elements starting at p (N * sizeof(T) bytes,
// moved in 16-byte pieces).  The generator proves contiguity and alignment.
template <int N, class T>
__device__ __forceinline__ auto vload(const T* __restrict__ p) {
  if constexpr (N == 1) {
    return *p;
  } else {
    constexpr int PER = (16 / sizeof(T)) < N ? (16 / sizeof(T)) : N;
    V<T, N> r;
#pragma unroll
    for (int c = 0; c < N / PER; ++c) {
      const Vec<T, PER> t = load_vec<T, PER>(p + c * PER);
#pragma unroll
      for (int i = 0; i < PER; ++i) r.v[c * PER + i] = t[i];
    }
    return r;
  }
}

// vload with the non-temporal hint, for operands a kernel reads once when its read set is too
// large to be found in the memory-side cache again.  Measured on MI355X with bf16 adds of 96 MiB
// tensors: three launches over six distinct tensors (604 MB in turn) move 5.65 TB/s with plain
// loads and 6.5 TB/s with the hint; the same launch repeated on one pair of tensors (201 MB, which
// the 256 MiB cache keeps) moves 7.2 TB/s plain and 6.6 TB/s hinted.  The generator decides per kernel.
template <int N, class T>
__device__ __forceinline__ auto vload_s(const T* __restrict__ p) {
  if constexpr (N == 1) {
    return *p;
  } else {
    constexpr int PER = (16 / sizeof(T)) < N ? (16 / sizeof(T)) : N;
    typedef typename RawBits<sizeof(T) * PER>::type raw_t;
    V<T, N> r;
#pragma unroll
    for (int c = 0; c < N / PER; ++c) {
      const raw_t bits = __builtin_nontemporal_load(reinterpret_cast<const raw_t*>(p + c * PER));
      Vec<T, PER> t;
      __builtin_memcpy(&t, &bits, sizeof(bits));
#pragma unroll
      for (int i = 0; i < PER; ++i) r.v[c * PER + i] = t[i];
    }
    return r;
  }
}

template <int N, bool STREAM, class T>
__device__ __forceinline__ auto vload_x(const T* __restrict__ p) {
  if constexpr (STREAM) {
    return vload_s<N, T>(p);
  } else {
    return vload<N, T>(p);
  }
}

// Contiguous run aligned to its element only.  The access is still one wide instruction per 16
// bytes: gfx950 under ROCm runs with unaligned global access enabled, and the compiler emits
// global_load_dwordx4 / global_store_dwordx4 for an under-aligned aggregate of that size.
template <class T, int N>
struct __attribute__((packed, aligned(alignof(T)))) UnalignedRun {
  T v[N];
};
template <int N, class T>
__device__ __forceinline__ auto vload_u(const T* __restrict__ p) {
  if constexpr (N == 1) {
    return *p;
  } else {
    constexpr int PER = (16 / sizeof(T)) < N ? (16 / sizeof(T)) : N;
    V<T, N> r;
#pragma unroll
    for (int c = 0; c < N / PER; ++c) {
      const UnalignedRun<T, PER> t = *reinterpret_cast<const UnalignedRun<T, PER>*>(p + c * PER);
#pragma unroll
      for (int i = 0; i < PER; ++i) r.v[c * PER + i] = t.v[i];
    }
    return r;
  }
}

// Register tile for an operand whose contiguous axis is not the kernel's vector axis.  Row e
// holds the N elements that vector lane e needs over the N steps of the (fully unrolled) loop
// along the operand's own contiguous axis: N contiguous loads `stride` elements apart fill it at
// the first step, and step u takes column u, which is register renaming once u is a constant.
template <class T, int N>
struct Tile {
  V<T, N> row[N];
};
template <int N, class T, class S>
__device__ __forceinline__ void tile_fill(Tile<T, N>& t, const T* __restrict__ p, S stride) {
#pragma unroll
  for (int e = 0; e < N; ++e) t.row[e] = vload<N, T>(p + e * stride);
}
template <int N, class T, class S>
__device__ __forceinline__ void tile_fill_u(Tile<T, N>& t, const T* __restrict__ p, S stride) {
#pragma unroll
  for (int e = 0; e < N; ++e) t.row[e] = vload_u<N, T>(p + e * stride);
}
template <int N, class T>
__device__ __forceinline__ V<T, N> tile_col(const Tile<T, N>& t, int u) {
  V<T, N> r;
#pragma unroll
  for (int e = 0; e < N; ++e) r.v[e] = t.row[e].v[u];
  return r;
}

// ---------------------------------------------------------------------------
// Random numbers: counter-based Philox-4x32 with ten rounds, keyed by the graph's 64-bit seed and
// counted by the element's offset -- the generator and the integer -> float maps that Inductor's
// own GPU code generation uses (triton.language.random: philox, uint_to_uniform_float,
// pair_uniform_to_normal; torch/_inductor/runtime/triton_helpers.py: randint64), so a graph sees the
// same stream whichever backend compiled it.  Stateless: the value of an element depends on
// (seed, offset) only.
// ---------------------------------------------------------------------------
struct Philox4 {
  uint32_t r[4];
};
__device__ __forceinline__ Philox4 philox4x32_10(i64 seed, uint32_t offset) {
  constexpr uint32_t KEY_A = 0x9E3779B9u, KEY_B = 0xBB67AE85u, ROUND_A = 0xD2511F53u, ROUND_B = 0xCD9E8D57u;
  uint32_t k0 = static_cast<uint32_t>(static_cast<unsigned long long>(seed));
  uint32_t k1 = static_cast<uint32_t>(static_cast<unsigned long long>(seed) >> 32);
  uint32_t c0 = offset, c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint32_t p0 = c0, p2 = c2;
    c0 = __umulhi(ROUND_B, p2) ^ c1 ^ k0;
    c2 = __umulhi(ROUND_A, p0) ^ c3 ^ k1;
    c1 = ROUND_B * p2;
    c3 = ROUND_A * p0;
    k0 += KEY_A;
    k1 += KEY_B;
  }
  return {{c0, c1, c2, c3}};
}
// uniform in [0, 1): the 31 low bits of |x| as a signed integer, scaled by 2^-31 (rounded down a little)
__device__ __forceinline__ float philox_uniform(uint32_t bits) {
  int x = static_cast<int>(bits);
  x = x < 0 ? -x - 1 : x;
  return static_cast<float>(x) * 4.6566127342e-10f;
}
template <class S, class O>
__device__ __forceinline__ auto rand(const S& seed, const O& offset) {
  return apply([](auto s, auto o) { return philox_uniform(philox4x32_10(static_cast<i64>(s), static_cast<uint32_t>(o)).r[0]); },
               seed, offset);
}
template <class S, class O>
__device__ __forceinline__ auto randn(const S& seed, const O& offset) {
  return apply(
      [](auto s, auto o) {
        const Philox4 p = philox4x32_10(static_cast<i64>(s), static_cast<uint32_t>(o));
        const float u1 = ::fmaxf(1.0e-7f, philox_uniform(p.r[0]));
        const float th = 6.283185307179586f * philox_uniform(p.r[1]);
        return ::sqrtf(-2.0f * ::logf(u1)) * ::cosf(th);
      },
      seed, offset);
}
template <class S, class O, class L, class H>
__device__ __forceinline__ auto randint64(const S& seed, const O& offset, const L& low, const H& high) {
  return apply(
      [](auto s, auto o, auto lo, auto hi) {
        const Philox4 p = philox4x32_10(static_cast<i64>(s), static_cast<uint32_t>(o));
        const unsigned long long word = static_cast<unsigned long long>(p.r[0]) | (static_cast<unsigned long long>(p.r[1]) << 32);
        const unsigned long long size = static_cast<unsigned long long>(static_cast<i64>(hi) - static_cast<i64>(lo));
        return static_cast<i64>(word % size) + static_cast<i64>(lo);
      },
      seed, offset, low, high);
}

// Element-wise indexed load: idx scalar -> scalar, idx vector -> vector.
// Indirect indices: the index a generated indirect load reads with when the one it was given lies
// outside [0, size) (the nearest valid one), and whether an index is inside (stores and atomics
// through an index outside the buffer are dropped).  Out-of-range indices are an error of the
// program being compiled; this keeps that error from touching memory the kernel does not own.
template <class A, class S>
__device__ __forceinline__ auto clamp_index(const A& a, S size) {
  return apply(
      [size](auto x) {
        typedef decltype(x) T;
        const T hi = size > 0 ? static_cast<T>(size) - 1 : static_cast<T>(0);  // an empty axis clamps to 0, not -1
        return x < 0 ? static_cast<T>(0) : (x > hi ? hi : x);
      },
      a);
}
template <class A, class S>
__device__ __forceinline__ auto index_in_range(const A& a, S size) {
  return apply([size](auto x) { return x >= 0 && static_cast<long long>(x) < static_cast<long long>(size); }, a);
}

template <class T, class I>
__device__ __forceinline__ auto gather(const T* __restrict__ p, const I& idx) {
  return apply([p](auto i) { return p[i]; }, idx);
}

// Masked forms: lanes whose mask is false read nothing and yield `other`.
template <int N, bool ALIGNED = true, class T, class M, class O>
__device__ __forceinline__ auto vload_m(const T* __restrict__ p, const M& mask, O other) {
  if constexpr (N == 1) {
    return static_cast<bool>(at(mask, 0)) ? *p : static_cast<T>(other);
  } else {
    V<T, N> r;
    bool all = true;
#pragma unroll
    for (int i = 0; i < N; ++i) all = all && static_cast<bool>(at(mask, i));
    if (all) {
      if constexpr (ALIGNED) {
        r = vload<N, T>(p);
      } else {
        r = vload_u<N, T>(p);
      }
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) r.v[i] = static_cast<bool>(at(mask, i)) ? p[i] : static_cast<T>(other);
    }
    return r;
  }
}
template <class T, class I, class M, class O>
__device__ __forceinline__ auto gather_m(const T* __restrict__ p, const I& idx, const M& mask, O other) {
  return apply([p, other](auto i, bool m) { return m ? p[i] : static_cast<T>(other); }, idx, mask);
}

// STREAM marks the store non-temporal; the generator sets it for buffers far
// larger than the caches (a measured gain of up to 20 % on copy-like kernels).
template <int N, bool STREAM = false, class T, class A>
__device__ __forceinline__ void vstore(T* __restrict__ p, const A& val) {
  if constexpr (N == 1) {
    *p = static_cast<T>(at(val, 0));
  } else {
    constexpr int PER = (16 / sizeof(T)) < N ? (16 / sizeof(T)) : N;
    if constexpr (N == PER) {
      // written without the chunk loop: inside it the compiler drops the non-temporal hint
      Vec<T, PER> t;
#pragma unroll
      for (int i = 0; i < PER; ++i) t[i] = static_cast<T>(at(val, i));
      store_vec<T, PER, STREAM>(p, t);
    } else {
#pragma unroll
      for (int c = 0; c < N / PER; ++c) {
        Vec<T, PER> t;
#pragma unroll
        for (int i = 0; i < PER; ++i) t[i] = static_cast<T>(at(val, c * PER + i));
        store_vec<T, PER, STREAM>(p + c * PER, t);
      }
    }
  }
}
template <int N, class T, class A>
__device__ __forceinline__ void vstore_u(T* __restrict__ p, const A& val) {
  if constexpr (N <= 1) {
    p[0] = static_cast<T>(at(val, 0));
  } else {
    constexpr int PER = (16 / sizeof(T)) < N ? (16 / sizeof(T)) : N;
#pragma unroll
    for (int c = 0; c < N / PER; ++c) {
      UnalignedRun<T, PER> t;
#pragma unroll
      for (int i = 0; i < PER; ++i) t.v[i] = static_cast<T>(at(val, c * PER + i));
      *reinterpret_cast<UnalignedRun<T, PER>*>(p + c * PER) = t;
    }
  }
}
template <int N, bool STREAM = false, class T, class A, class M>
__device__ __forceinline__ void vstore_m(T* __restrict__ p, const A& val, const M& mask) {
  bool all = true;
#pragma unroll
  for (int i = 0; i < N; ++i) all = all && static_cast<bool>(at(mask, i));
  if (all) {
    vstore<N, STREAM>(p, val);
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i)
      if (static_cast<bool>(at(mask, i))) p[i] = static_cast<T>(at(val, i));
  }
}
// Element-wise indexed store (scatter): idx and/or val may be vectors.
template <int N, class T, class I, class A, class M>
__device__ __forceinline__ void scatter_m(T* __restrict__ p, const I& idx, const A& val, const M& mask) {
#pragma unroll
  for (int i = 0; i < (N < 1 ? 1 : N); ++i)
    if (static_cast<bool>(at(mask, i))) p[at(idx, i)] = static_cast<T>(at(val, i));
}

// Accumulating scatter (index_put / scatter_add / embedding gradients): one atomic per element.
// 32- and 64-bit types use the memory atomics; narrower ones (bf16, fp16, 8- and 16-bit
// integers) update their slice of the enclosing aligned 32-bit word in a compare-and-swap loop.
template <class T, class A>
__device__ __forceinline__ void atomic_accumulate(T* p, A v) {
  if constexpr (std::is_same<T, float>::value || std::is_same<T, double>::value || std::is_same<T, int>::value ||
                std::is_same<T, unsigned>::value) {
    atomicAdd(p, static_cast<T>(v));
  } else if constexpr (sizeof(T) == 8) {
    atomicAdd(reinterpret_cast<unsigned long long*>(p), static_cast<unsigned long long>(static_cast<T>(v)));
  } else {
    static_assert(sizeof(T) < 4, "unexpected element size");
    typedef typename RawBits<sizeof(T)>::type bits_t;
    const unsigned long long a = reinterpret_cast<unsigned long long>(p);
    unsigned* word = reinterpret_cast<unsigned*>(a & ~3ull);
    const unsigned shift = static_cast<unsigned>(a & 3ull) * 8u;
    const unsigned field = ((1u << (8 * sizeof(T))) - 1u) << shift;
    unsigned seen = *word;
    while (true) {
      const bits_t cur_bits = static_cast<bits_t>((seen & field) >> shift);
      T cur;
      __builtin_memcpy(&cur, &cur_bits, sizeof(T));
      T next;
      if constexpr (std::is_integral<T>::value) {
        next = static_cast<T>(cur + static_cast<T>(v));
      } else {
        next = from_f32<T>(to_f32(cur) + static_cast<float>(v));
      }
      bits_t next_bits;
      __builtin_memcpy(&next_bits, &next, sizeof(T));
      const unsigned want = (seen & ~field) | (static_cast<unsigned>(next_bits) << shift);
      const unsigned was = atomicCAS(word, seen, want);
      if (was == seen) break;
      seen = was;
    }
  }
}
template <int N, class T, class I, class A, class M>
__device__ __forceinline__ void scatter_add_m(T* __restrict__ p, const I& idx, const A& val, const M& mask) {
#pragma unroll
  for (int i = 0; i < (N < 1 ? 1 : N); ++i)
    if (static_cast<bool>(at(mask, i))) atomic_accumulate(p + at(idx, i), at(val, i));
}

// ---------------------------------------------------------------------------
// reduction kinds.  Thread-level state T (cheap per-element step), merge-level
// state M (what travels between threads), W floats per M on the wire.
// Combination rules for arg-reductions and NaN handling follow
// reference inductor_x/codegen/triton.py:1217-1233 (maximum_with_index).
// ---------------------------------------------------------------------------
struct RedSum {
  typedef float T;
  typedef float M;
  static constexpr int W = 1;
  __device__ static T init() { return 0.f; }
  __device__ static T first(float v, int) { return step(init(), v, 0); }
  __device__ static T step_fast(T s, float v, int) { return step(s, v, 0); }
  __device__ static M finish_n(T s, float) { return finish(s); }
  __device__ static T step(T s, float v, int) { return s + v; }
  __device__ static M finish(T s) { return s; }
  __device__ static M empty() { return 0.f; }
  __device__ static M merge(M a, M b) { return a + b; }
  __device__ static void enc(M m, float* w) { w[0] = m; }
  __device__ static M dec(const float* w) { return w[0]; }
  typedef SumOp Op;
};
struct RedProd {
  typedef float T;
  typedef float M;
  static constexpr int W = 1;
  __device__ static T init() { return 1.f; }
  __device__ static T first(float v, int) { return step(init(), v, 0); }
  __device__ static T step_fast(T s, float v, int) { return step(s, v, 0); }
  __device__ static M finish_n(T s, float) { return finish(s); }
  __device__ static T step(T s, float v, int) { return s * v; }
  __device__ static M finish(T s) { return s; }
  __device__ static M empty() { return 1.f; }
  __device__ static M merge(M a, M b) { return a * b; }
  __device__ static void enc(M m, float* w) { w[0] = m; }
  __device__ static M dec(const float* w) { return w[0]; }
  struct Op {
    __device__ __forceinline__ float operator()(float a, float b) const { return a * b; }
  };
};
// The thread state of a maximum / minimum keeps "a NaN was seen" beside the running extremum of
// the numbers (three instructions per element instead of the six of a NaN-propagating
// comparison); the two are folded into one NaN-propagating value when the thread is done.
struct ExtremumState {
  float m, nan;
};
struct RedMax {
  typedef ExtremumState T;
  typedef float M;
  static constexpr int W = 1;
  __device__ static T init() {
    T t;
    t.m = -__builtin_inff();
    t.nan = 0.f;
    return t;
  }
  __device__ static T first(float v, int) { return step(init(), v, 0); }
  __device__ static T step_fast(T s, float v, int) { return step(s, v, 0); }
  __device__ static M finish_n(T s, float) { return finish(s); }
  __device__ static T step(T s, float v, int) {
    s.m = __builtin_fmaxf(s.m, v);
    s.nan = (v != v) ? 1.f : s.nan;
    return s;
  }
  __device__ static M finish(T s) { return (s.nan != 0.f) ? __builtin_nanf("") : s.m; }
  __device__ static M empty() { return -__builtin_inff(); }
  __device__ static M merge(M a, M b) { return MaxOp()(a, b); }
  __device__ static void enc(M m, float* w) { w[0] = m; }
  __device__ static M dec(const float* w) { return w[0]; }
  typedef MaxOp Op;
};
struct RedMin {
  typedef ExtremumState T;
  typedef float M;
  static constexpr int W = 1;
  __device__ static T init() {
    T t;
    t.m = __builtin_inff();
    t.nan = 0.f;
    return t;
  }
  __device__ static T first(float v, int) { return step(init(), v, 0); }
  __device__ static T step_fast(T s, float v, int) { return step(s, v, 0); }
  __device__ static M finish_n(T s, float) { return finish(s); }
  __device__ static T step(T s, float v, int) {
    s.m = __builtin_fminf(s.m, v);
    s.nan = (v != v) ? 1.f : s.nan;
    return s;
  }
  __device__ static M finish(T s) { return (s.nan != 0.f) ? __builtin_nanf("") : s.m; }
  __device__ static M empty() { return __builtin_inff(); }
  __device__ static M merge(M a, M b) { return MinOp()(a, b); }
  __device__ static void enc(M m, float* w) { w[0] = m; }
  __device__ static M dec(const float* w) { return w[0]; }
  typedef MinOp Op;
};
struct RedAny {
  typedef float T;
  typedef float M;
  static constexpr int W = 1;
  __device__ static T init() { return 0.f; }
  __device__ static T first(float v, int) { return step(init(), v, 0); }
  __device__ static T step_fast(T s, float v, int) { return step(s, v, 0); }
  __device__ static M finish_n(T s, float) { return finish(s); }
  __device__ static T step(T s, float v, int) { return (s != 0.f || v != 0.f) ? 1.f : 0.f; }
  __device__ static M finish(T s) { return s; }
  __device__ static M empty() { return 0.f; }
  __device__ static M merge(M a, M b) { return (a != 0.f || b != 0.f) ? 1.f : 0.f; }
  __device__ static void enc(M m, float* w) { w[0] = m; }
  __device__ static M dec(const float* w) { return w[0]; }
  struct Op {
    __device__ __forceinline__ float operator()(float a, float b) const { return (a != 0.f || b != 0.f) ? 1.f : 0.f; }
  };
};
template <bool IS_MAX>
struct RedArg {
  typedef ArgVal T;
  typedef ArgVal M;
  static constexpr int W = 2;
  __device__ static T init() {
    ArgVal a;
    a.v = IS_MAX ? -__builtin_inff() : __builtin_inff();
    a.i = 0x7fffffff;
    return a;
  }
  // A thread meets its elements in increasing index order, so an equal value
  // never replaces: take v when it is better or NaN (unordered) unless the
  // running best is already NaN; the untouched state takes anything.
  __device__ static T step(T s, float v, int idx) {
    const bool better = IS_MAX ? !(v <= s.v) : !(v >= s.v);
    const bool take = static_cast<bool>((static_cast<int>(better) & static_cast<int>(s.v == s.v)) |
                                        static_cast<int>(s.i == 0x7fffffff));
    s.v = take ? v : s.v;
    s.i = take ? idx : s.i;
    return s;
  }
  __device__ static T first(float v, int idx) {
    ArgVal a;
    a.v = v;
    a.i = idx;
    return a;
  }
  // after the first element the state is never the untouched one
  __device__ static T step_fast(T s, float v, int idx) {
    const bool better = IS_MAX ? !(v <= s.v) : !(v >= s.v);
    const bool take = static_cast<bool>(static_cast<int>(better) & static_cast<int>(s.v == s.v));
    s.v = take ? v : s.v;
    s.i = take ? idx : s.i;
    return s;
  }
  __device__ static M finish_n(T s, float) { return s; }
  __device__ static M finish(T s) { return s; }
  __device__ static M empty() { return init(); }
  __device__ static M merge(M a, M b) { return arg_combine<IS_MAX>(a, b); }
  __device__ static void enc(M m, float* w) {
    w[0] = m.v;
    w[1] = __int_as_float(m.i);
  }
  __device__ static M dec(const float* w) {
    ArgVal a;
    a.v = w[0];
    a.i = __float_as_int(w[1]);
    return a;
  }
};
typedef RedArg<true> RedArgMax;
typedef RedArg<false> RedArgMin;

// Mean / M2 / count.  A thread accumulates shifted sums (shift = its first
// sample), which costs three flops per element and is as stable as Welford's
// update; merges use Chan's formula.  The definition restated is the two-pass
// one of reference inductor_x/lowering.py:270-293.
struct RedWelford {
  struct T {
    float n, c, s1, s2;
  };
  typedef Moments M;
  static constexpr int W = 3;
  __device__ static T init() {
    T t;
    t.n = 0.f;
    t.c = 0.f;
    t.s1 = 0.f;
    t.s2 = 0.f;
    return t;
  }
  __device__ static T step(T s, float v, int) {
    s.c = (s.n == 0.f) ? v : s.c;
    const float d = v - s.c;
    s.s1 += d;
    s.s2 = fmaf(d, d, s.s2);
    s.n += 1.f;
    return s;
  }
  __device__ static T first(float v, int) {
    T t;
    t.n = 1.f;
    t.c = v;
    t.s1 = 0.f;
    t.s2 = 0.f;
    return t;
  }
  // the count is kept by the caller (it is the same for every lane)
  __device__ static T step_fast(T s, float v, int) {
    const float d = v - s.c;
    s.s1 += d;
    s.s2 = fmaf(d, d, s.s2);
    return s;
  }
  __device__ static M finish_n(T s, float n) {
    s.n = n;
    return finish(s);
  }
  __device__ static M finish(T s) {
    Moments m;
    m.n = s.n;
    if (s.n == 0.f) {
      m.mean = 0.f;
      m.m2 = 0.f;
      return m;
    }
    const float inv = 1.0f / s.n;
    m.mean = s.c + s.s1 * inv;
    const float m2 = s.s2 - s.s1 * s.s1 * inv;
    m.m2 = (m2 < 0.f) ? 0.f : m2;
    return m;
  }
  __device__ static M empty() {
    Moments m;
    m.n = 0.f;
    m.mean = 0.f;
    m.m2 = 0.f;
    return m;
  }
  __device__ static M merge(M a, M b) { return moments_combine(a, b); }
  __device__ static void enc(M m, float* w) {
    w[0] = m.n;
    w[1] = m.mean;
    w[2] = m.m2;
  }
  __device__ static M dec(const float* w) {
    Moments m;
    m.n = w[0];
    m.mean = w[1];
    m.m2 = w[2];
    return m;
  }
};

// Sum, product, maximum and minimum of 64-bit values, integer (exact) or double.  The state is
// one 64-bit value; where states travel as float words (lane exchanges, LDS, the column
// workspace) it goes as its two 32-bit halves, bit for bit: those paths only move words, they
// never do arithmetic on them.  Extrema of doubles propagate NaN, as torch does.
enum class IntOp { Sum, Prod, Max, Min };
template <class VAL, IntOp OP>
struct RedWide {
  typedef VAL V;  // the type a value is converted to before step()
  typedef VAL T;
  typedef VAL M;
  static constexpr int W = 2;
  static constexpr bool kFloat = std::is_same<VAL, double>::value;
  __device__ static T init() {
    if constexpr (OP == IntOp::Sum) return static_cast<VAL>(0);
    if constexpr (OP == IntOp::Prod) return static_cast<VAL>(1);
    if constexpr (kFloat) {
      return OP == IntOp::Max ? -__builtin_inf() : __builtin_inf();
    } else {
      return OP == IntOp::Max ? static_cast<VAL>(0x8000000000000000ull) : static_cast<VAL>(0x7fffffffffffffffull);
    }
  }
  __device__ static M empty() { return init(); }
  __device__ static M merge(M a, M b) {
    if constexpr (OP == IntOp::Sum) return a + b;
    if constexpr (OP == IntOp::Prod) return a * b;
    if constexpr (kFloat) {
      if (a != a) return a;
      if (b != b) return b;
    }
    if constexpr (OP == IntOp::Max) return a > b ? a : b;
    return a < b ? a : b;
  }
  __device__ static T step(T s, VAL v, int) { return merge(s, v); }
  __device__ static T first(VAL v, int) { return v; }
  __device__ static T step_fast(T s, VAL v, int) { return merge(s, v); }
  __device__ static M finish(T s) { return s; }
  __device__ static M finish_n(T s, float) { return s; }
  __device__ static void enc(M m, float* w) {
    const unsigned long long u = __builtin_bit_cast(unsigned long long, m);
    w[0] = __builtin_bit_cast(float, static_cast<unsigned>(u & 0xffffffffull));
    w[1] = __builtin_bit_cast(float, static_cast<unsigned>(u >> 32));
  }
  __device__ static M dec(const float* w) {
    const unsigned long long lo = __builtin_bit_cast(unsigned, w[0]);
    const unsigned long long hi = __builtin_bit_cast(unsigned, w[1]);
    return __builtin_bit_cast(VAL, lo | (hi << 32));
  }
};
template <IntOp OP>
using RedInt = RedWide<i64, OP>;
template <IntOp OP>
using RedF64 = RedWide<double, OP>;
// The type values are converted to on their way into R::step: float unless R names another.
template <class R, class = void>
struct ValueOf {
  typedef float type;
};
template <class R>
struct ValueOf<R, std::void_t<typename R::V>> {
  typedef typename R::V type;
};

// Maximum and sum of exp(x - maximum) of a row in one sweep ("online softmax"): the state is the
// running maximum m and the sum s of exp(x - m) over what has been seen; a larger maximum rescales
// the sum.  While the maximum is -inf the scale is taken as 1 (exp(-inf - -inf) would be NaN), as
// in torch/_inductor/runtime/triton_helpers.py:192-212.  NaN inputs make both results NaN.
struct SoftmaxState {
  float m, s;
};
__device__ __forceinline__ float softmax_scale(float from, float to) {
  return (to == -__builtin_inff()) ? 1.0f : __expf(from - to);
}
struct RedOnlineSoftmax {
  typedef SoftmaxState T;
  typedef SoftmaxState M;
  static constexpr int W = 2;
  __device__ static T init() {
    T t;
    t.m = -__builtin_inff();
    t.s = 0.f;
    return t;
  }
  __device__ static M empty() { return init(); }
  __device__ static M merge(M a, M b) {
    M r;
    r.m = MaxOp()(a.m, b.m);
    r.s = a.s * softmax_scale(a.m, r.m) + b.s * softmax_scale(b.m, r.m);
    return r;
  }
  __device__ static T step(T s, float v, int) {
    T r;
    r.m = MaxOp()(s.m, v);
    r.s = s.s * softmax_scale(s.m, r.m) + softmax_scale(v, r.m);
    return r;
  }
  __device__ static T first(float v, int) { return step(init(), v, 0); }
  __device__ static T step_fast(T s, float v, int) { return step(s, v, 0); }
  __device__ static M finish(T s) { return s; }
  __device__ static M finish_n(T s, float) { return s; }
  __device__ static void enc(M m, float* w) {
    w[0] = m.m;
    w[1] = m.s;
  }
  __device__ static M dec(const float* w) {
    M m;
    m.m = w[0];
    m.s = w[1];
    return m;
  }
};
// One vector of a row at a time: the vector's own maximum first, so the running sum is rescaled
// once per vector and every element costs one exponential.
template <class VT, class MT>
__device__ __forceinline__ SoftmaxState softmax_step(SoftmaxState a, const VT& val, const MT& mask) {
  constexpr int n = Tr<VT>::n == 0 ? 1 : Tr<VT>::n;
  float vm = -__builtin_inff();
#pragma unroll
  for (int i = 0; i < n; ++i)
    if (static_cast<bool>(at(mask, i))) vm = MaxOp()(vm, static_cast<float>(at(val, i)));
  SoftmaxState r;
  r.m = MaxOp()(a.m, vm);
  const float ref = (r.m == -__builtin_inff()) ? 0.f : r.m;
  float add = 0.f;
#pragma unroll
  for (int i = 0; i < n; ++i)
    if (static_cast<bool>(at(mask, i))) add += __expf(static_cast<float>(at(val, i)) - ref);
  // with the maximum still -inf every term above is exp(-inf) = 0; count the elements instead,
  // which is what a scale of 1 per element amounts to
  if (r.m == -__builtin_inff()) {
    add = 0.f;
#pragma unroll
    for (int i = 0; i < n; ++i)
      if (static_cast<bool>(at(mask, i))) add += 1.f;
  }
  r.s = a.s * softmax_scale(a.m, r.m) + add;
  return r;
}
struct GetSoftmaxMax {
  __device__ __forceinline__ float operator()(const SoftmaxState& m) const { return m.m; }
};
struct GetSoftmaxSum {
  __device__ __forceinline__ float operator()(const SoftmaxState& m) const { return m.s; }
};

// Reduction whose inputs are moments already (the second stage of a variance that was split
// into slices): the thread state is the merged moments.
struct RedMoments {
  typedef Moments T;
  typedef Moments M;
  static constexpr int W = 3;
  __device__ static T init() { return RedWelford::empty(); }
  __device__ static M finish(T s) { return s; }
  __device__ static M empty() { return RedWelford::empty(); }
  __device__ static M merge(M a, M b) { return moments_combine(a, b); }
  __device__ static void enc(M m, float* w) { RedWelford::enc(m, w); }
  __device__ static M dec(const float* w) { return RedWelford::dec(w); }
};
template <class V1, class V2, class V3, class MT>
__device__ __forceinline__ Moments moments_step(Moments s, const V1& mean, const V2& m2, const V3& weight,
                                                const MT& mask) {
  constexpr int n = MaxN<Tr<V1>::n, Tr<V2>::n, Tr<V3>::n, Tr<MT>::n>::value == 0
                        ? 1
                        : MaxN<Tr<V1>::n, Tr<V2>::n, Tr<V3>::n, Tr<MT>::n>::value;
#pragma unroll
  for (int i = 0; i < n; ++i)
    if (static_cast<bool>(at(mask, i))) {
      Moments m;
      m.n = static_cast<float>(at(weight, i));
      m.mean = static_cast<float>(at(mean, i));
      m.m2 = static_cast<float>(at(m2, i));
      s = moments_combine(s, m);
    }
  return s;
}

// ---------------------------------------------------------------------------
// row shape: reduce a thread's vector, then the TPR threads of the row
// ---------------------------------------------------------------------------
// Butterfly over the low lanes of a wavefront for any merge state.
template <class R, int WIDTH>
__device__ __forceinline__ typename R::M wave_merge(typename R::M m) {
#pragma unroll
  for (int off = 1; off < WIDTH; off <<= 1) {
    float w[R::W], o[R::W];
    R::enc(m, w);
#pragma unroll
    for (int k = 0; k < R::W; ++k) o[k] = __shfl_xor(w[k], off, kWave);
    // keep the operand order fixed by lane so every lane computes the same value
    const bool low = (threadIdx.x & off) == 0;
    const typename R::M other = R::dec(o);
    m = low ? R::merge(m, other) : R::merge(other, m);
  }
  return m;
}

template <class R, class = void>
struct HasOp : std::false_type {};
template <class R>
struct HasOp<R, std::void_t<typename R::Op>> : std::true_type {};

// Sums of K values per thread over the TPR threads of a row at once: DPP steps per value, one
// round through LDS for rows wider than a wavefront.  lds: at least (BLOCK / 64) * K floats.
template <int BLOCK, int TPR, int K>
__device__ __forceinline__ void group_sums(float (&v)[K], float* lds) {
  if constexpr (TPR <= kWave) {
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_reduce<TPR>(v[k], SumOp());
  } else {
    constexpr int WPG = TPR / kWave;
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_reduce<kWave>(v[k], SumOp());
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) {
#pragma unroll
      for (int k = 0; k < K; ++k) lds[wave * K + k] = v[k];
    }
    __syncthreads();
    const int src = (wave / WPG) * WPG + (threadIdx.x & (WPG - 1));
#pragma unroll
    for (int k = 0; k < K; ++k) v[k] = wave_reduce<WPG>(lds[src * K + k], SumOp());
  }
}

// Moments of the union of the threads' samples by plain sums instead of pairwise merges: the
// total count and mean first, then every thread's M2 moved to that mean.
template <int BLOCK, int TPR>
__device__ __forceinline__ Moments group_moments(Moments m, float* lds) {
  float a[2] = {m.n, m.n * m.mean};
  group_sums<BLOCK, TPR, 2>(a, lds);
  Moments r;
  r.n = a[0];
  r.mean = (a[0] > 0.f) ? a[1] / a[0] : 0.f;
  const float d = m.mean - r.mean;
  float b[1] = {m.m2 + m.n * d * d};
  group_sums<BLOCK, TPR, 1>(b, lds);
  r.m2 = b[0];
  return r;
}

// lds: at least (BLOCK / 64) * R::W floats.  All threads of the group receive
// the result.  Reductions of one float with a plain binary operation and moments take the
// DPP paths; only states that must travel as a whole (value + index) use the butterfly.
template <class R, int BLOCK, int TPR>
__device__ __forceinline__ typename R::M group_merge(typename R::M m, float* lds) {
  if constexpr (HasOp<R>::value) {
    return group_reduce<BLOCK, TPR>(m, typename R::Op(), lds);
  } else if constexpr (std::is_same<typename R::M, Moments>::value) {
    return group_moments<BLOCK, TPR>(m, lds);
  } else if constexpr (TPR <= kWave) {
    return wave_merge<R, TPR>(m);
  } else {
    constexpr int WPG = TPR / kWave;
    m = wave_merge<R, kWave>(m);
    const int wave = threadIdx.x / kWave;
    __syncthreads();
    if ((threadIdx.x & (kWave - 1)) == 0) {
      float w[R::W];
      R::enc(m, w);
#pragma unroll
      for (int k = 0; k < R::W; ++k) lds[wave * R::W + k] = w[k];
    }
    __syncthreads();
    const int src = (wave / WPG) * WPG + (threadIdx.x & (WPG - 1));
    return wave_merge<R, WPG>(R::dec(lds + src * R::W));
  }
}

// Fold one vector of values (with their reduction indices and a validity mask)
// into a thread state.
template <class R, class VT, class IT, class MT>
__device__ __forceinline__ typename R::T thread_step(typename R::T s, const VT& val, const IT& idx, const MT& mask) {
  constexpr int n = Tr<VT>::n == 0 ? (Tr<IT>::n == 0 ? (Tr<MT>::n == 0 ? 1 : Tr<MT>::n) : Tr<IT>::n) : Tr<VT>::n;
#pragma unroll
  for (int i = 0; i < n; ++i)
    if (static_cast<bool>(at(mask, i)))
      s = R::step(s, static_cast<typename ValueOf<R>::type>(at(val, i)), static_cast<int>(at(idx, i)));
  return s;
}

// Plain fp32 sums and maxima take the DPP path of common.h.
template <int BLOCK, int TPR, class VT, class MT>
__device__ __forceinline__ float row_sum(const VT& val, const MT& mask, float* lds) {
  constexpr int n = Tr<VT>::n == 0 ? 1 : Tr<VT>::n;
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < n; ++i) s += static_cast<bool>(at(mask, i)) ? static_cast<float>(at(val, i)) : 0.f;
  return group_reduce<BLOCK, TPR>(s, SumOp(), lds);
}

// ---------------------------------------------------------------------------
// column shape
// ---------------------------------------------------------------------------
// Per-thread: N independent columns, each with its own thread state.  The
// mask is uniform for the thread (the generator only runs live columns), so the
// first row takes a peeled path and the remaining rows the cheap update.
template <class R, int N>
struct ColAcc {
  typename R::T s[N];
  int cnt;
  __device__ __forceinline__ void init() {
    cnt = 0;
#pragma unroll
    for (int i = 0; i < N; ++i) s[i] = R::init();
  }
  template <class VT>
  __device__ __forceinline__ void step(const VT& val, int ridx, bool mask) {
    if (!mask) return;
    if (cnt == 0) {
#pragma unroll
      for (int i = 0; i < N; ++i) s[i] = R::first(static_cast<typename ValueOf<R>::type>(at(val, i)), ridx);
    } else {
#pragma unroll
      for (int i = 0; i < N; ++i) s[i] = R::step_fast(s[i], static_cast<typename ValueOf<R>::type>(at(val, i)), ridx);
    }
    ++cnt;
  }
  __device__ __forceinline__ typename R::M finish(int i) const {
    return cnt == 0 ? R::empty() : R::finish_n(s[i], static_cast<float>(cnt));
  }
};

// Stands in for the accumulator of a reduction whose result is derived from another one's state.
struct ColAccNone {
  template <class VT>
  __device__ __forceinline__ void step(const VT&, int, bool) {}
};

// Per-thread: N independent columns whose inputs are moments already.
template <int N>
struct ColMomentsAcc {
  Moments s[N];
  __device__ __forceinline__ void init() {
#pragma unroll
    for (int i = 0; i < N; ++i) s[i] = RedWelford::empty();
  }
  template <class V1, class V2, class V3>
  __device__ __forceinline__ void step(const V1& mean, const V2& m2, const V3& weight) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      Moments m;
      m.n = static_cast<float>(at(weight, i));
      m.mean = static_cast<float>(at(mean, i));
      m.m2 = static_cast<float>(at(m2, i));
      s[i] = moments_combine(s[i], m);
    }
  }
  __device__ __forceinline__ Moments finish(int i) const { return s[i]; }
};

// Fold the RL row lanes of a workgroup (thread = rl * CT + ct).  lds holds
// (RL / 2) * CT * N * R::W floats.  Afterwards threads with rl == 0 own the result.
template <class R, int N, int CT, int RL>
__device__ __forceinline__ void col_fold(typename R::M (&m)[N], int ct, int rl, float* lds) {
  if constexpr (RL > 1) {
    constexpr int PLANE = (RL / 2) * CT * N;
#pragma unroll
    for (int half = RL / 2; half >= 1; half >>= 1) {
      __syncthreads();
      if (rl >= half && rl < 2 * half) {
        const int slot = ((rl - half) * CT + ct) * N;
#pragma unroll
        for (int i = 0; i < N; ++i) {
          float w[R::W];
          R::enc(m[i], w);
#pragma unroll
          for (int k = 0; k < R::W; ++k) lds[k * PLANE + slot + i] = w[k];
        }
      }
      __syncthreads();
      if (rl < half) {
        const int slot = (rl * CT + ct) * N;
#pragma unroll
        for (int i = 0; i < N; ++i) {
          float w[R::W];
#pragma unroll
          for (int k = 0; k < R::W; ++k) w[k] = lds[k * PLANE + slot + i];
          m[i] = R::merge(m[i], R::dec(w));
        }
      }
    }
  }
}

// The fold of col_fold for every reduction of a kernel at once, with as few barriers as the
// shape allows: row lanes that share a wavefront (CT < 64) meet through lane exchanges, the
// remaining groups are halved through LDS while more than four are left and then collected in
// one round.  Every state travels as its float words (enc / dec), so a state of any width folds
// the same way.  lds holds col_fold_all_planes(CT, RL) * CT * N * (sum of R::W) floats.
// Afterwards threads with rl == 0 own the results.  Merges are commutative up to rounding
// (arg-reductions break ties by index, moments by Chan's symmetric formula).
__host__ __device__ constexpr int col_fold_all_in_wave(int ct, int rl) {
  return ct >= kWave ? 1 : (kWave / ct < rl ? kWave / ct : rl);
}
__host__ __device__ constexpr int col_fold_all_planes(int ct, int rl) {
  const int groups = rl / col_fold_all_in_wave(ct, rl);
  if (groups <= 1) return 0;
  const int tree = groups > 4 ? groups / 2 : 0;
  const int last = (groups < 4 ? groups : 4) - 1;
  return tree > last ? tree : last;
}
template <class R, int N>
__device__ __forceinline__ void col_state_exchange(typename R::M (&m)[N], int off) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    float w[R::W];
    R::enc(m[i], w);
#pragma unroll
    for (int k = 0; k < R::W; ++k) w[k] = __shfl_xor(w[k], off, kWave);
    m[i] = R::merge(m[i], R::dec(w));
  }
}
template <class R, int N>
__device__ __forceinline__ void col_state_put(float* lds, int plane, int slot, int& word, const typename R::M (&m)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    float w[R::W];
    R::enc(m[i], w);
#pragma unroll
    for (int k = 0; k < R::W; ++k) lds[(word + k) * plane + slot + i] = w[k];
  }
  word += R::W;
}
template <class R, int N>
__device__ __forceinline__ void col_state_take(const float* lds, int plane, int slot, int& word, typename R::M (&m)[N]) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    float w[R::W];
#pragma unroll
    for (int k = 0; k < R::W; ++k) w[k] = lds[(word + k) * plane + slot + i];
    m[i] = R::merge(m[i], R::dec(w));
  }
  word += R::W;
}
template <int N, int CT, int RL, class... R>
__device__ __forceinline__ void col_fold_all(float* lds, int ct, int rl, typename R::M (&... m)[N]) {
  if constexpr (RL > 1) {
    constexpr int IN_WAVE = col_fold_all_in_wave(CT, RL);
    constexpr int GROUPS = RL / IN_WAVE;
    constexpr int PLANE = col_fold_all_planes(CT, RL) * CT * N;
#pragma unroll
    for (int off = CT; off < CT * IN_WAVE; off <<= 1) (col_state_exchange<R, N>(m, off), ...);
    if constexpr (GROUPS > 1) {
      const int grp = rl / IN_WAVE;
      const bool lead = rl % IN_WAVE == 0;
      int left = GROUPS;
#pragma unroll
      for (int half = GROUPS / 2; half >= 4; half >>= 1) {
        if (lead && grp >= half && grp < 2 * half) {
          int word = 0;
          (col_state_put<R, N>(lds, PLANE, ((grp - half) * CT + ct) * N, word, m), ...);
        }
        __syncthreads();
        if (lead && grp < half) {
          int word = 0;
          (col_state_take<R, N>(lds, PLANE, (grp * CT + ct) * N, word, m), ...);
        }
        __syncthreads();
        left = half;
      }
      // at most four groups are left: one round
      if (lead && grp >= 1 && grp < left) {
        int word = 0;
        (col_state_put<R, N>(lds, PLANE, ((grp - 1) * CT + ct) * N, word, m), ...);
      }
      __syncthreads();
      if (rl == 0) {
        for (int g2 = 1; g2 < left; ++g2) {
          int word = 0;
          (col_state_take<R, N>(lds, PLANE, ((g2 - 1) * CT + ct) * N, word, m), ...);
        }
      }
    }
  }
}

// After col_fold: hand the folded states of row lane 0 to every row lane (same LDS area).
template <class R, int N, int CT, int RL>
__device__ __forceinline__ void col_share(typename R::M (&m)[N], int ct, int rl, float* lds) {
  if constexpr (RL > 1) {
    constexpr int PLANE = CT * N;
    __syncthreads();
    if (rl == 0) {
#pragma unroll
      for (int i = 0; i < N; ++i) {
        float w[R::W];
        R::enc(m[i], w);
#pragma unroll
        for (int k = 0; k < R::W; ++k) lds[k * PLANE + ct * N + i] = w[k];
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
      float w[R::W];
#pragma unroll
      for (int k = 0; k < R::W; ++k) w[k] = lds[k * PLANE + ct * N + i];
      m[i] = R::dec(w);
    }
  }
}

// One field of N per-column states as a register vector.
struct GetSelf {
  template <class M>
  __device__ __forceinline__ float operator()(const M& m) const { return m; }
};
struct GetSelfInt {
  __device__ __forceinline__ i64 operator()(i64 m) const { return m; }
};
struct GetSelfF64 {
  __device__ __forceinline__ double operator()(double m) const { return m; }
};
struct GetMean {
  __device__ __forceinline__ float operator()(const Moments& m) const { return m.mean; }
};
struct GetM2 {
  __device__ __forceinline__ float operator()(const Moments& m) const { return m.m2; }
};
struct GetCount {
  __device__ __forceinline__ float operator()(const Moments& m) const { return m.n; }
};
struct GetIndex {
  __device__ __forceinline__ i64 operator()(const ArgVal& m) const { return static_cast<i64>(m.i); }
};
struct GetNonzero {
  __device__ __forceinline__ bool operator()(float m) const { return m != 0.f; }
};
template <int N, class M, class G>
__device__ __forceinline__ auto col_get(const M (&m)[N], G get) {
  if constexpr (N == 1) {
    return get(m[0]);
  } else {
    V<decltype(get(m[0])), N> r;
#pragma unroll
    for (int i = 0; i < N; ++i) r.v[i] = get(m[i]);
    return r;
  }
}

// The values one row's loads of a column sweep deliver, kept together so a whole batch of rows
// can be in flight while the previous batch is folded (unpacked with a structured binding).
template <class A> struct Pack1 { A a; };
template <class A, class B> struct Pack2 { A a; B b; };
template <class A, class B, class C> struct Pack3 { A a; B b; C c; };
template <class A, class B, class C, class D> struct Pack4 { A a; B b; C c; D d; };
template <class A> __device__ __forceinline__ Pack1<A> pack(const A& a) { return {a}; }
template <class A, class B> __device__ __forceinline__ Pack2<A, B> pack(const A& a, const B& b) { return {a, b}; }
template <class A, class B, class C>
__device__ __forceinline__ Pack3<A, B, C> pack(const A& a, const B& b, const C& c) { return {a, b, c}; }
template <class A, class B, class C, class D>
__device__ __forceinline__ Pack4<A, B, C, D> pack(const A& a, const B& b, const C& c, const D& d) { return {a, b, c, d}; }

// Workspace layout for one reduction: [R::W][nsplit][xnumel] floats.
template <class R, int N>
__device__ __forceinline__ void col_store_partial(float* __restrict__ ws, const typename R::M (&m)[N], i64 x0,
                                                  i64 xnumel, int split, int nsplit) {
  const i64 plane = static_cast<i64>(nsplit) * xnumel;
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if (x0 + i < xnumel) {
      float w[R::W];
      R::enc(m[i], w);
#pragma unroll
      for (int k = 0; k < R::W; ++k) ws[k * plane + static_cast<i64>(split) * xnumel + x0 + i] = w[k];
    }
  }
}

// Second pass for one column x, in two steps so that a kernel with several reductions can have
// the loads of all of them in flight before the first barrier: thread sl of SL merges splits
// sl, sl+SL, ... (batched loads), then the SL lanes are folded through LDS (SL * W floats per
// column slot; `slot` = the column's index inside the workgroup, CPW of them).
template <class R, int SL>
__device__ __forceinline__ typename R::M col_final_gather(const float* __restrict__ ws, i64 x, i64 xnumel,
                                                          int nsplit, int sl, bool live) {
  constexpr int BATCH = 8;  // with SL = 32 lanes per column: 256 partials in one round of loads
  const i64 plane = static_cast<i64>(nsplit) * xnumel;
  typename R::M m = R::empty();
  if (live) {
    for (int s0 = sl; s0 < nsplit; s0 += SL * BATCH) {
      float w[BATCH][R::W];
#pragma unroll
      for (int b = 0; b < BATCH; ++b) {
        const int s = s0 + b * SL;
        const i64 o = static_cast<i64>(s < nsplit ? s : s0) * xnumel + x;
#pragma unroll
        for (int k = 0; k < R::W; ++k) w[b][k] = ws[k * plane + o];
      }
#pragma unroll
      for (int b = 0; b < BATCH; ++b)
        if (s0 + b * SL < nsplit) m = R::merge(m, R::dec(w[b]));
    }
  }
  return m;
}
template <class R, int CPW, int SL>
__device__ __forceinline__ typename R::M col_final_fold(typename R::M m, int slot, int sl, float* lds) {
  constexpr int PLANE = CPW * SL;
  const int me = sl * CPW + slot;
  __syncthreads();
  {
    float w[R::W];
    R::enc(m, w);
#pragma unroll
    for (int k = 0; k < R::W; ++k) lds[k * PLANE + me] = w[k];
  }
  __syncthreads();
#pragma unroll
  for (int half = SL / 2; half >= 1; half >>= 1) {
    if (sl < half) {
      float w[R::W];
#pragma unroll
      for (int k = 0; k < R::W; ++k) w[k] = lds[k * PLANE + (sl + half) * CPW + slot];
      m = R::merge(m, R::dec(w));
      R::enc(m, w);
#pragma unroll
      for (int k = 0; k < R::W; ++k) lds[k * PLANE + me] = w[k];
    }
    __syncthreads();
  }
  return m;  // valid where sl == 0
}
// The same fold for several reductions at once (one tree, one set of barriers): every state
// has its own words in LDS, CPW * SL * (sum of R::W) floats in all.
template <class R>
struct RedTag {
  typedef R type;
};
template <class R>
__device__ __forceinline__ void col_final_exchange(typename R::M& m, int off) {
  float w[R::W];
  R::enc(m, w);
#pragma unroll
  for (int k = 0; k < R::W; ++k) w[k] = __shfl_xor(w[k], off, kWave);
  m = R::merge(m, R::dec(w));
}
// Thread (slot, sl) = sl * CPW + slot.  The split lanes of a column that share a wavefront meet
// through lane exchanges (CPW * SL <= 64: no LDS and no barrier at all); with several wavefronts
// the first lane of every further wavefront hands its state over through LDS in one round
// (lds: (waves - 1) * CPW * (sum of R::W) floats at least).  Valid afterwards where sl == 0.
template <int CPW, int SL, class... R>
__device__ __forceinline__ void col_final_fold_all(float* lds, int slot, int sl, typename R::M&... m) {
  static_assert(CPW <= kWave && (CPW & (CPW - 1)) == 0 && (SL & (SL - 1)) == 0, "CPW, SL: powers of two, CPW <= 64");
  constexpr int SLW = (kWave / CPW) < SL ? (kWave / CPW) : SL;  // split lanes of a column per wavefront
  constexpr int WAVES = SL / SLW;
#pragma unroll
  for (int off = CPW; off < CPW * SLW; off <<= 1) (col_final_exchange<R>(m, off), ...);
  if constexpr (WAVES > 1) {
    constexpr int PLANE = (WAVES - 1) * CPW;
    const int wave = sl / SLW;
    auto put = [&](auto tag, auto& mm, int& off) {
      typedef typename decltype(tag)::type RR;
      float w[RR::W];
      RR::enc(mm, w);
#pragma unroll
      for (int k = 0; k < RR::W; ++k) lds[(off + k) * PLANE + (wave - 1) * CPW + slot] = w[k];
      off += RR::W;
    };
    auto take = [&](auto tag, auto& mm, int& off, int from) {
      typedef typename decltype(tag)::type RR;
      float w[RR::W];
#pragma unroll
      for (int k = 0; k < RR::W; ++k) w[k] = lds[(off + k) * PLANE + (from - 1) * CPW + slot];
      mm = RR::merge(mm, RR::dec(w));
      off += RR::W;
    };
    if (wave >= 1 && sl % SLW == 0) {
      int off = 0;
      (put(RedTag<R>{}, m, off), ...);
    }
    __syncthreads();
    if (sl == 0) {
      for (int from = 1; from < WAVES; ++from) {
        int off = 0;
        (take(RedTag<R>{}, m, off, from), ...);
      }
    }
  }
}

template <class R, int CPW, int SL>
__device__ __forceinline__ typename R::M col_final(const float* __restrict__ ws, i64 x, i64 xnumel, int nsplit,
                                                   int slot, int sl, bool live, float* lds) {
  return col_final_fold<R, CPW, SL>(col_final_gather<R, SL>(ws, x, xnumel, nsplit, sl, live), slot, sl, lds);
}

}  // namespace mi
