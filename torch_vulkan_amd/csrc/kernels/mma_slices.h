// K in slices over workgroups for the tile kernel (mma_tile.h), for products of 65 rows and more whose tiles are too
// few for the machine: a workgroup of the tile kernel walks all of K, so 128 x 128 tiles of a 128 x 8192 product keep
// 64 of 256 compute units busy for the whole launch.
//
// The tile kernel already runs batches of products; slice s of K is batch s of a product whose operands begin
// s * (k / slices) bytes into their rows (both operands are rows of k) and whose "outputs" are float32 partial sums in
// the workspace, [slice][m][n]: SliceProblem is that product (weights stored [k, n]: a slice begins k / slices rows
// down).  A second launch adds the slices up in slice order (the result does not depend on timing) and runs the real
// problem's epilogue on 4 consecutive columns of a row, the unit every problem's store<DT>() takes.
#pragma once
#include <string>
#include <type_traits>

#include "kernels.h"
#include "mma_tile.h"

namespace vkt {
namespace {

template <bool TRB>
struct SliceProblem {
  static constexpr bool kTransA = false, kTransB = TRB;  // (TRB: the second operand stored [k, n], 16-bit values)
  static constexpr bool kRegisterEpilogue = false;
  uint64_t a, b;
  uint32_t m, n, k, lda, ldb, batches;  // (k: bytes of one slice; batches: the slices)
  uint64_t a_batch, b_batch;            // (a slice's offset: k bytes into the rows; for [k, n] weights k / 2 rows)
  uint64_t partial;                     // float32 [batches][m][n]
  struct Whole {
    uint32_t vec_ok;
  };
  struct Columns {};
  __device__ __forceinline__ Whole whole() const { return Whole{(n & 3u) == 0 ? 1u : 0u}; }
  __device__ __forceinline__ Columns columns(uint32_t, uint32_t, const Whole&) const { return Columns{}; }
  template <int DT>
  __device__ __forceinline__ void store(uint32_t batch, uint32_t row, uint32_t col, const V4F& t, const Columns&, const Whole&) const {
    float* const out = reinterpret_cast<float*>(partial) + (uint64_t(batch) * m + row) * n + col;
    if constexpr (DT >= 0) {
      *reinterpret_cast<V4F*>(out) = t;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (col + r < n) out[r] = t[r];
    }
  }
  template <class F>
  __device__ __forceinline__ void for_output_type(bool full, const Whole& w, F&& f) const {
    if (w.vec_ok && full) f(std::integral_constant<int, 0>{});
    else f(std::integral_constant<int, -1>{});
  }
};

// The slices of one product added up in slice order, then the problem's epilogue: a thread per 4 consecutive columns
// of a row (four slices' loads in flight).
template <class Problem>
__global__ __launch_bounds__(256) void mma_slices_finish(Problem p, uint32_t slices, uint64_t partial) {
  const uint32_t quads = (p.n + 3) / 4;
  const uint64_t id = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (id >= uint64_t(p.m) * quads) return;
  const uint32_t row = uint32_t(id / quads), col = uint32_t(id % quads) * 4;
  const uint64_t plane = uint64_t(p.m) * p.n;
  const float* const mine = reinterpret_cast<const float*>(partial) + uint64_t(row) * p.n + col;
  V4F sum = {0.0f, 0.0f, 0.0f, 0.0f};
  if ((p.n & 3u) == 0) {
    sum = *reinterpret_cast<const V4F*>(mine);
    uint32_t s = 1;
    for (; s + 4 <= slices; s += 4) {
      const V4F a = *reinterpret_cast<const V4F*>(mine + s * plane), b = *reinterpret_cast<const V4F*>(mine + (s + 1) * plane);
      const V4F c = *reinterpret_cast<const V4F*>(mine + (s + 2) * plane), d = *reinterpret_cast<const V4F*>(mine + (s + 3) * plane);
      sum += a, sum += b, sum += c, sum += d;
    }
    for (; s < slices; ++s) sum += *reinterpret_cast<const V4F*>(mine + s * plane);
  } else {
    for (uint32_t s = 0; s < slices; ++s)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (col + r < p.n) sum[r] = s == 0 ? mine[s * plane + r] : sum[r] + mine[s * plane + r];
  }
  const auto whole = p.whole();
  const auto cs = p.columns(0, col, whole);
  p.for_output_type(col + 3 < p.n, whole, [&](auto dt) { p.template store<decltype(dt)::value>(0, row, col, sum, cs, whole); });
}

// How many slices of K serve a product of m rows whose operands are rows of k bytes: a power of two that divides the
// steps of 128 bytes, leaves a slice 1024 bytes and more, brings the 128 x 128 tiles up to two workgroups per compute
// unit at most, and whose partial sums fit `budget` bytes.  1: the product is not split.
inline uint32_t tile_slices(uint32_t m, uint32_t n, uint32_t k_bytes, uint32_t cus, uint64_t budget) {
  if (k_bytes % BK) return 1;
  const uint32_t steps = k_bytes / BK;
  const uint64_t tiles = uint64_t((m + 127) / 128) * ((n + 127) / 128);
  uint32_t s = 1;
  while (s < 16 && steps % (2 * s) == 0 && steps / (2 * s) >= 8 && tiles * (2 * s) <= 2ull * cus && uint64_t(2 * s) * m * n * 4 <= budget) s *= 2;
  return s;
}

// Launches the 128 x 128 tile kernel of the given arithmetic over `slices` slices of K and the second launch.
// (MF32: the 32 x 32 matrix-core tiles, which the widened and 16-bit forms are built on.)
template <int FA, int FB, bool MF32, int MATH, class Problem>
int launch_tile_slices(const Problem& p, uint32_t slices, const Machine& mc, hipStream_t stream, std::string* err, const char* name) {
  constexpr bool TRB = Problem::kTransB;  // (k-major operands run on the tile kernel's direct-load form)
  static_assert(!Problem::kTransA, "slices of K: the first operand in rows of k");
  SliceProblem<TRB> sp;
  sp.a = p.a, sp.b = p.b, sp.m = p.m, sp.n = p.n, sp.k = p.k / slices, sp.lda = p.lda, sp.ldb = p.ldb, sp.batches = slices;
  sp.a_batch = sp.k, sp.b_batch = TRB ? uint64_t(sp.k / 2) * p.ldb : uint64_t(sp.k), sp.partial = mc.workspace;
  const int rc = launch_mma_tile<2, 2, 4, 4, FA, FB, MF32, TRB, MATH>(sp, mc.compute_units, stream, err, name);
  if (rc != 0) return rc;
  const uint64_t threads = uint64_t(p.m) * ((p.n + 3) / 4);
  hipLaunchKernelGGL((mma_slices_finish<Problem>), dim3(uint32_t((threads + 255) / 256)), dim3(256), 0, stream, p, slices, mc.workspace);
  return 0;
}

}  // namespace
}  // namespace vkt
