// Helpers shared by the kernels whose waves split K over a column group (few activation rows against many weight
// rows): the waves' partial tiles added up in wave 0, and the column count that deals a product's columns out evenly.
#pragma once
#include "common.h"

namespace vkt {

using V4F = float __attribute__((ext_vector_type(4)));

// The partial tiles of a workgroup's waves added up in wave 0.  Where LDS holds half the waves' tiles, a
// tree: in each round the upper half of the remaining waves hands its tiles to the lower half (two
// barriers per round, log2(WAVES) rounds, a fixed order); otherwise wave by wave.
template <int MT, int NT, int WAVES>
constexpr int kPartSlots = (WAVES / 2) * MT * NT <= 32 ? WAVES / 2 : 1;

template <int MT, int NT, int WAVES>
__device__ __forceinline__ void add_wave_tiles(V4F (&acc)[MT][NT], V4F* part, int wave, int lane) {
  if constexpr (kPartSlots<MT, NT, WAVES> > 1) {
#pragma unroll
    for (int half = WAVES / 2; half >= 1; half /= 2) {
      if (wave >= half && wave < 2 * half) {
#pragma unroll
        for (int i = 0; i < MT * NT; ++i) part[((wave - half) * MT * NT + i) * 64 + lane] = acc[i / NT][i % NT];
      }
      __syncthreads();
      if (wave < half) {
#pragma unroll
        for (int i = 0; i < MT * NT; ++i) acc[i / NT][i % NT] += part[(wave * MT * NT + i) * 64 + lane];
      }
      if (half > 1) __syncthreads();
    }
  } else {
    for (int w = 1; w < WAVES; ++w) {
      __syncthreads();
      if (wave == w) {
#pragma unroll
        for (int i = 0; i < MT * NT; ++i) part[i * 64 + lane] = acc[i / NT][i % NT];
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int i = 0; i < MT * NT; ++i) acc[i / NT][i % NT] += part[i * 64 + lane];
      }
    }
  }
}

// Columns per workgroup of a kernel that gives a workgroup at most 16 nt columns: fewer where that deals the columns
// out over a whole number of workgroups per compute unit (a multiple of 4, at least 8).
inline uint32_t staged_cols(uint32_t n, int nt, uint32_t cus) {
  const uint32_t cols = 16 * nt, wgs = (n + cols - 1) / cols, even = (wgs + cus - 1) / cus * cus;
  // (not below 8: half of a matrix-core tile's columns are then zeros, and fewer columns than compute units x 8
  // leave some units without a workgroup, which costs less than workgroups of 16 on a quarter of them)
  const uint32_t share = ((n + even - 1) / even + 3) / 4 * 4, fewer = share < 8 ? 8 : share;
  return fewer < cols ? fewer : cols;
}

}  // namespace vkt
