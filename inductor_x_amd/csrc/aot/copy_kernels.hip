// Gather and permuted-copy kernels for the fourth benchmark graph.  Elements
// are moved as raw 16-bit words, eight per thread access, so bf16 and fp16
// share the same code and results are bit-exact.
#include "../mi/copy.h"

using namespace mi;

#define GATHER_VARIANT(BLOCK, TPR, RPT)                                                       \
  extern "C" __global__ __launch_bounds__(BLOCK) void gather_rows_b16_b##BLOCK##_t##TPR##_r##RPT( \
      const uint16_t* table, const long long* idx, uint16_t* out, int nidx, int row_elems,    \
      int table_rows) {                                                                       \
    gather_rows<uint16_t, 8, BLOCK, TPR, RPT>(table, idx, out, nidx, row_elems, table_rows);  \
  }

GATHER_VARIANT(256, 128, 1)
GATHER_VARIANT(256, 128, 2)
GATHER_VARIANT(256, 128, 4)
GATHER_VARIANT(256, 64, 1)
GATHER_VARIANT(256, 64, 2)
GATHER_VARIANT(256, 64, 4)
GATHER_VARIANT(256, 16, 1)
GATHER_VARIANT(256, 16, 4)

extern "C" __global__ __launch_bounds__(256) void gather_rows_b32_b256_t64_r2(
    const uint32_t* table, const long long* idx, uint32_t* out, int nidx, int row_elems,
    int table_rows) {
  gather_rows<uint32_t, 4, 256, 64, 2>(table, idx, out, nidx, row_elems, table_rows);
}

#define PERMUTE_VARIANT(BLOCK, TPC, T1, T2)                                                   \
  extern "C" __global__ __launch_bounds__(BLOCK) void                                         \
      permute_copy_b16_b##BLOCK##_p##TPC##_t##T1##x##T2(const uint16_t* in, uint16_t* out,    \
                                                        int n0, int n1, int n2, int inner,    \
                                                        long long s0, long long s1,           \
                                                        long long s2) {                       \
    permute_copy_tiled<uint16_t, 8, BLOCK, TPC, T1, T2>(in, out, n0, n1, n2, inner, s0, s1,   \
                                                        s2);                                  \
  }

PERMUTE_VARIANT(256, 16, 32, 8)
PERMUTE_VARIANT(256, 16, 32, 4)
PERMUTE_VARIANT(256, 16, 32, 2)
PERMUTE_VARIANT(256, 16, 16, 8)
PERMUTE_VARIANT(256, 16, 8, 8)
PERMUTE_VARIANT(256, 16, 4, 16)
PERMUTE_VARIANT(256, 16, 1, 64)
PERMUTE_VARIANT(256, 16, 1, 128)
PERMUTE_VARIANT(256, 16, 1, 16)
PERMUTE_VARIANT(256, 16, 2, 8)
PERMUTE_VARIANT(256, 8, 1, 32)
PERMUTE_VARIANT(256, 4, 1, 64)
PERMUTE_VARIANT(256, 64, 1, 4)
PERMUTE_VARIANT(256, 64, 4, 4)
PERMUTE_VARIANT(256, 16, 8, 4)
PERMUTE_VARIANT(256, 16, 16, 4)
PERMUTE_VARIANT(256, 16, 4, 8)
PERMUTE_VARIANT(256, 16, 8, 2)
PERMUTE_VARIANT(256, 16, 4, 4)

extern "C" __global__ __launch_bounds__(256) void permute_copy_b32_b256_p16_t8x8(
    const uint32_t* in, uint32_t* out, int n0, int n1, int n2, int inner, long long s0,
    long long s1, long long s2) {
  permute_copy_tiled<uint32_t, 4, 256, 16, 8, 8>(in, out, n0, n1, n2, inner, s0, s1, s2);
}

// Plain contiguous copy, 16 bytes per thread.  Used as the known-size probe that
// calibrates the HBM byte counters (FETCH_SIZE / WRITE_SIZE) in profiles.
extern "C" __global__ __launch_bounds__(256) void copy_b128(const uint32_t* in, uint32_t* out,
                                                            long long n_vec) {
  const long long i = static_cast<long long>(blockIdx.x) * 256 + threadIdx.x;
  if (i < n_vec) store_vec<uint32_t, 4, true>(out + 4 * i, load_vec<uint32_t, 4>(in + 4 * i));
}
