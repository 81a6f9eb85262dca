// The few-row product on the matrix cores: C = A [m,k] x B [n,k]^T for m <= 64 (decode at small batch), both operands
// in rows of k (A row-major, B stored as its columns: the Linear layout), float8 or 16-bit values.
//
// Such a product is the weight stream, N x K values read once, and the tile kernels (mma_tile.h, mma_stream.h), which
// give a workgroup 128 or 256 rows x as many columns, cover a quarter of the machine at N = 8192.  Here a workgroup owns
// a run of at most 16 NT columns (weight rows) and all rows of A, and its waves take the chunks of 256 bytes of k in
// turn (rotated against the other workgroups', so that rows a power of two apart are not all read at the same offsets
// at the same time).  A wave's load instruction fetches 4 weight rows x 256 contiguous bytes, into registers a chunk
// ahead, and from there into the wave's own LDS region, 16-byte pieces swizzled by the row, to come back in the matrix
// core's operand shape: lane (c, g) holds 16 bytes of weight row c (two operands of the 16x16x32 float8 instructions,
// one of the 16-bit ones; weights first, so a lane ends with 4 consecutive columns of one row), against the same 16
// bytes of k of activation row c, loaded from global memory (the rows of A come from L2).  The waves' partial tiles
// meet in wave 0, which runs the problem's epilogue (the tile kernels' interface: whole / columns / store).
// (The 16x16x32 float8 instruction runs at half the rate of the 128-deep one the tile kernels use: at 64 rows the
// matrix cores' share is ~4 us of a launch the weights hold to 12 and more.)
// Where the column groups are too few for the machine, K is cut into slices over workgroups (gridDim.y; a second launch
// adds the slices' tiles up in slice order); a batch of such products (gridDim.z) is a workgroup per batch, column
// group and slice.  mma_skinny_kn below is the same product for weights stored [k, n].
#pragma once
#include <string>
#include <type_traits>

#include "kernels.h"
#include "limits.h"
#include "mma_tile.h"
#include "wave_tiles.h"

namespace vkt {
namespace {

template <int FA, int FB>
__device__ __forceinline__ V4F mfma_f8x32(long w, long a, const V4F& acc) {
  // first operand: weights (format FB), second: activations (format FA); 0 = e4m3fn, 1 = e5m2
  if constexpr (FB == 0 && FA == 0) return __builtin_amdgcn_mfma_f32_16x16x32_fp8_fp8(w, a, acc, 0, 0, 0);
  else if constexpr (FB == 0 && FA == 1) return __builtin_amdgcn_mfma_f32_16x16x32_fp8_bf8(w, a, acc, 0, 0, 0);
  else if constexpr (FB == 1 && FA == 0) return __builtin_amdgcn_mfma_f32_16x16x32_bf8_fp8(w, a, acc, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_bf8_bf8(w, a, acc, 0, 0, 0);
}

// 8 float8 values widened exactly to bfloat16 (two values per conversion instruction).
template <int F>
__device__ __forceinline__ V8BF widen8(uint32_t lo, uint32_t hi) {
  const V2BF p0 = widen_pair<F, false>(int(lo)), p1 = widen_pair<F, true>(int(lo));
  const V2BF p2 = widen_pair<F, false>(int(hi)), p3 = widen_pair<F, true>(int(hi));
  return V8BF{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

// 16 bytes of a weight row against the same 16 bytes of k of MT activation rows, into the tiles of column tile t.
// MATH: kMathFp8 (the float8 instruction), kMathFp8Wide (float8 widened exactly to bfloat16: float32 precision of the
// sums), kMathBf16, kMathF16.
template <int MT, int NT, int FA, int FB, int MATH>
__device__ __forceinline__ void skinny_step(const U4& wv, const U4 (&a)[MT][4], int j, int t, V4F (&acc)[MT][NT]) {
  if constexpr (MATH == kMathFp8) {
    const long w0 = long(uint64_t(wv[0]) | uint64_t(wv[1]) << 32), w1 = long(uint64_t(wv[2]) | uint64_t(wv[3]) << 32);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const long a0 = long(uint64_t(a[mt][j][0]) | uint64_t(a[mt][j][1]) << 32), a1 = long(uint64_t(a[mt][j][2]) | uint64_t(a[mt][j][3]) << 32);
      acc[mt][t] = mfma_f8x32<FA, FB>(w0, a0, acc[mt][t]);
      acc[mt][t] = mfma_f8x32<FA, FB>(w1, a1, acc[mt][t]);
    }
  } else if constexpr (MATH == kMathFp8Wide) {
    const V8BF w0 = widen8<FB>(wv[0], wv[1]), w1 = widen8<FB>(wv[2], wv[3]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, widen8<FA>(a[mt][j][0], a[mt][j][1]), acc[mt][t], 0, 0, 0);
      acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, widen8<FA>(a[mt][j][2], a[mt][j][3]), acc[mt][t], 0, 0, 0);
    }
  } else if constexpr (MATH == kMathBf16) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(V8BF, wv), __builtin_bit_cast(V8BF, a[mt][j]), acc[mt][t], 0, 0, 0);
  } else {
    using V8H = _Float16 __attribute__((ext_vector_type(8)));
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      acc[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(V8H, wv), __builtin_bit_cast(V8H, a[mt][j]), acc[mt][t], 0, 0, 0);
  }
}

// The epilogue of one 16 x 16 tile: lane (c, g) holds row row0 + c, columns col0 + 4 g .. + 3.
template <class Problem>
__device__ __forceinline__ void skinny_store_tile(const Problem& p, uint32_t batch, uint32_t row0, uint32_t col0, uint32_t n_end, const V4F& acc, int lane) {
  const uint32_t row = row0 + (lane & 15), col = col0 + 4 * (lane >> 4);
  if (col >= n_end || row >= p.m) return;
  const auto whole = p.whole();
  const auto cs = p.columns(batch, col, whole);
  p.for_output_type(col + 3 < p.n, whole, [&](auto dt) { p.template store<decltype(dt)::value>(batch, row, col, acc, cs, whole); });
}

// The epilogue of one workgroup's tiles: lane (c, g) holds, per tile (mt, t), row 16 mt + c, columns n0 + 16 t + 4 g .. + 3.
template <int MT, int NT, class Problem>
__device__ __forceinline__ void skinny_store(const Problem& p, uint32_t batch, uint32_t n0, uint32_t n_end, const V4F (&acc)[MT][NT], int lane) {
  const int c = lane & 15, g = lane >> 4;
  const auto whole = p.whole();
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const uint32_t col = n0 + 16 * t + 4 * g;
    if (col >= n_end) continue;
    const auto cs = p.columns(batch, col, whole);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const uint32_t row = 16 * mt + c;
      if (row >= p.m) continue;
      p.for_output_type(col + 3 < p.n, whole, [&](auto dt) { p.template store<decltype(dt)::value>(batch, row, col, acc[mt][t], cs, whole); });
    }
  }
}

// p.k, p.lda, p.ldb, p.a_batch, p.b_batch in bytes; k a multiple of 16, rows and bases 16-byte aligned; p.m <= 16 MT.
// gridDim.z = p.batches.  gridDim.y slices of K
// (chunks_per_slice chunks of 256 bytes each), one per workgroup of the column group: with more than one, wave 0
// leaves the workgroup's tiles in the workspace and mma_skinny_finish adds the slices up in slice order.
template <int MT, int NT, int WAVES, int FA, int FB, int MATH, class Problem>
__global__ __launch_bounds__(WAVES * 64) void mma_skinny(Problem p, uint32_t cols_per_wg, uint32_t chunks_per_slice, uint64_t workspace) {
  constexpr uint32_t TILE = 16 * 256, REGION = NT * TILE;  // bytes of LDS per tile of 16 weight rows, per wave
  extern __shared__ __attribute__((aligned(16))) uint8_t staged[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  uint8_t* const mine = staged + uint32_t(wave) * REGION;
  const uint32_t total = (p.k + 255) / 256, q_begin = blockIdx.y * chunks_per_slice;
  if (q_begin >= total) return;  // (an empty slice, which the launcher does not make: the chunk count below would wrap around)
  const uint32_t count = (q_begin + chunks_per_slice < total ? q_begin + chunks_per_slice : total) - q_begin;  // (no slice is empty)
  const uint32_t n0 = blockIdx.x * cols_per_wg, n_end = n0 + cols_per_wg < p.n ? n0 + cols_per_wg : p.n;
  // loads: instruction i of tile t fetches rows 4 i .. 4 i + 3; this lane row 4 i + (lane / 16), slot lane % 16
  uint64_t wsrc[NT][4];
  uint32_t wk[4];  // byte offset within the chunk of the 16 bytes this lane fetches
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const uint32_t row = 4 * i + g;
    wk[i] = ((uint32_t(c) ^ row) & 15u) * 16;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const uint32_t n = n0 + 16 * t + row < n_end ? n0 + 16 * t + row : n_end - 1;  // (rows past the end: the last one again, from the caches)
      wsrc[t][i] = p.b + uint64_t(blockIdx.z) * p.b_batch + uint64_t(n) * p.ldb;
    }
  }
  uint64_t arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const uint32_t m = uint32_t(16 * mt + c) < p.m ? 16 * mt + c : p.m - 1;
    arow[mt] = p.a + uint64_t(blockIdx.z) * p.a_batch + uint64_t(m) * p.lda + 16 * g;
  }
  V4F acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = V4F{0.0f, 0.0f, 0.0f, 0.0f};

  const U4 zero = {0, 0, 0, 0};
  U4 wr[NT][4];
  auto request = [&](uint32_t q) {
    const uint32_t k0 = q * 256;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // (no branch around a load: bytes past k are fetched from the row's start and replaced by zeros, so that an
        // infinity there does not meet the zeros that stand for the activations past k)
        const bool inside = k0 + wk[i] < p.k;
        const U4 v = ldg_stream<U4>(wsrc[t][i] + (inside ? k0 + wk[i] : 0u));
        wr[t][i] = inside ? v : zero;
      }
  };
  const uint32_t rot = (blockIdx.x * 5u) % count;
  auto chunk_at = [&](uint32_t i) { return q_begin + (i + rot) % count; };  // the i-th chunk this workgroup works on
  if (uint32_t(wave) < count) request(chunk_at(wave));
  for (uint32_t i = wave; i < count; i += WAVES) {
    const uint32_t k0 = chunk_at(i) * 256;
    U4 a[MT][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool inside = k0 + 64 * j + 16 * g < p.k;  // (k is a multiple of 16 bytes)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bool real = inside && uint32_t(16 * mt + c) < p.m;  // (rows past m are zeros, not loads)
        a[mt][j] = real ? ldg<U4>(arow[mt] + k0 + 64 * j) : zero;
      }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i2 = 0; i2 < 4; ++i2) *reinterpret_cast<U4*>(mine + (t * 16 + 4 * i2) * 256 + lane * 16) = wr[t][i2];
    if (i + WAVES < count) request(chunk_at(i + WAVES));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        // (a wave's LDS operations execute in order: these reads see the writes above)
        const U4 wv = *reinterpret_cast<const U4*>(mine + (t * 16 + c) * 256 + (((4 * j + g) ^ c) & 15) * 16);
        skinny_step<MT, NT, FA, FB, MATH>(wv, a, j, t, acc);
      }
    }
  }

  // the waves' partial tiles meet in wave 0 (through the staging memory, once every wave is done with it)
  __syncthreads();
  add_wave_tiles<MT, NT, WAVES>(acc, reinterpret_cast<V4F*>(staged), wave, lane);
  if (wave != 0) return;
  if (gridDim.y > 1) {
    V4F* const out = reinterpret_cast<V4F*>(workspace) + ((uint64_t(blockIdx.z) * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y) * (MT * NT * 64);
#pragma unroll
    for (int i = 0; i < MT * NT; ++i) out[i * 64 + lane] = acc[i / NT][i % NT];
    return;
  }
  skinny_store<MT, NT>(p, blockIdx.z, n0, n_end, acc, lane);
}

// Adds up the slices of one column group, in slice order, and runs the epilogue: a workgroup per group, a wave per
// 16 x 16 tile (four slices' loads in flight at a time; one wave for all of a group's tiles took 6.2 us for 8 slices of 8).
template <int MT, int NT, class Problem>
__global__ __launch_bounds__(64 * MT * NT) void mma_skinny_finish(Problem p, uint32_t cols_per_wg, uint32_t slices, uint64_t workspace) {
  constexpr uint32_t GROUP = MT * NT * 64;  // V4F per slice of a group
  const int lane = threadIdx.x & 63, tile = threadIdx.x >> 6;
  const V4F* const mine = reinterpret_cast<const V4F*>(workspace) + (uint64_t(blockIdx.z) * gridDim.x + blockIdx.x) * slices * GROUP + tile * 64 + lane;
  V4F acc = mine[0];
  uint32_t sl = 1;
  for (; sl + 4 <= slices; sl += 4) {
    const V4F a = mine[uint64_t(sl) * GROUP], b = mine[uint64_t(sl + 1) * GROUP], c = mine[uint64_t(sl + 2) * GROUP], d = mine[uint64_t(sl + 3) * GROUP];
    acc += a, acc += b, acc += c, acc += d;
  }
  for (; sl < slices; ++sl) acc += mine[uint64_t(sl) * GROUP];
  const uint32_t n0 = blockIdx.x * cols_per_wg;
  skinny_store_tile(p, blockIdx.z, 16 * (tile / NT), n0 + 16 * (tile % NT), n0 + cols_per_wg < p.n ? n0 + cols_per_wg : p.n, acc, lane);
}

template <int MT, int NT, int WAVES, int FA, int FB, int MATH, class Problem>
int launch_skinny_one(const Problem& p, uint32_t cols, uint32_t slices, uint64_t workspace, hipStream_t stream, std::string* err, const char* name) {
  auto kernel = mma_skinny<MT, NT, WAVES, FA, FB, MATH, Problem>;
  constexpr uint32_t stage_bytes = WAVES * NT * 16 * 256, part_bytes = kPartSlots<MT, NT, WAVES> * MT * NT * 1024;
  constexpr uint32_t lds = stage_bytes > part_bytes ? stage_bytes : part_bytes;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
      (void)hipGetLastError();
      *err = std::string(name) + ": cannot reserve " + std::to_string(lds) + " bytes of LDS";
      return -1;
    }
    configured = true;
  }
  const uint32_t groups = (p.n + cols - 1) / cols;
  const KSlices cut = k_slices((p.k + 255) / 256, slices);  // (no empty slice)
  slices = cut.slices;
  const uint32_t per_slice = cut.chunks_per_slice;
  hipLaunchKernelGGL(kernel, dim3(groups, slices, p.batches), dim3(WAVES * 64), lds, stream, p, cols, per_slice, workspace);
  if (slices > 1) hipLaunchKernelGGL((mma_skinny_finish<MT, NT, Problem>), dim3(groups, 1, p.batches), dim3(64 * MT * NT), 0, stream, p, cols, slices, workspace);
  return 0;
}

// Launches the few-row kernel where it serves: up to 64 rows, rows of k of 1024 bytes and more, 64 columns and more.
// Enough columns to give every compute unit a workgroup: 16, 32 or 64 columns per workgroup, whichever leaves the
// busiest compute unit the fewest bytes to take in, (workgroups on it) x (columns + rows) x K: every workgroup reads all
// rows of A beside its weights (64 columns as one workgroup per unit run a quarter slower than their bytes say).
// K in slices over workgroups (a second launch adds the slices' tiles up in slice order) where that brings more of
// the machine to bear.  The rules are read off every (columns, slices) of 14 shapes x 5 row counts x both element
// sizes (what they pick is 0.7 % behind the best form on average, 11 % at worst):
//  - 32 columns per workgroup and a power of two of slices that brings the workgroups up to one per compute unit
//    while a slice keeps two chunks (rows of k of 4096 bytes and more; 2048 from 33 rows on); up to 16 rows: twice the
//    slices where they stay 14 chunks long (two workgroups per unit: 8 x 14336 x 4096 bf16, 28.5 -> 23.5 us), and no
//    slices where 16 columns per workgroup fill the machine anyway;
//  - 49 to 64 rows against 4096 columns and more, 17 to 32 against 8192 and more (rows of k of 8192 bytes and more):
//    64 columns per workgroup, which halves the activations the workgroups re-read, and slices up to one workgroup
//    per unit (two at 32 rows): 64 x 8192 x 8192, 30.6 -> 27.3 us fp8, 50.0 -> 42.2 bf16.
// us before / with slices, fp8: 64 rows, K = 28672, N = 1024: 74.9 / 18.8; K = 8192, N = 1024: 25.5 / 11.2; 8 rows,
// K = 16384, N = 512: 11.4 / 7.8.  forced_nt: that many 16s of columns instead; forced_slices likewise (tests, tuning).
// -2: not this kernel's problem; -1: the workspace is fixed and too small for the plan (*err says so).
template <int FA, int FB, int MATH, class Problem>
int launch_mma_skinny(const Problem& p, const Machine& mc, uint32_t forced_nt, uint32_t forced_slices, hipStream_t stream, std::string* err,
                      const char* name) {
  // (batches: a workgroup per batch, column group and slice; a batch of short rows, k of 256 bytes and more, is served too)
  const uint32_t batches = p.batches;
  if (p.m > 64 || p.n < 64 || batches == 0 || batches > 65535 || p.k < 256) return -2;
  const uint32_t cus = uint32_t(mc.compute_units), chunks = (p.k + 255) / 256;
  const int mt = p.m <= 16 ? 1 : p.m <= 32 ? 2 : 4;
  // a batch of rows of k too short for a workgroup's waves to share (q @ k.T of a batch of attention heads: k = 128
  // values): workgroups of one wave and 64 columns, up to 16 rows
  if (batches > 1 && chunks < 8 && mt == 1 && !forced_nt && !forced_slices) return launch_skinny_one<1, 4, 1, FA, FB, MATH>(p, 64, 1, 0, stream, err, name);
  if (p.k < 1024) return -2;
  auto built = [&](int t) { return !((mt == 1 && t == 4) || (mt == 4 && t == 1)); };  // (the shapes that are built)
  int nt = 2;
  uint32_t slices = 1;
  auto fill = [&](uint32_t groups, uint32_t limit) {  // slices that bring `groups` up to `limit` workgroups
    uint32_t sl = 1;
    while (groups * sl * 2 <= limit && chunks / (sl * 2) >= 2) sl *= 2;
    return sl;
  };
  if (mt == 4 && p.m > 48 && p.n >= 4096 && p.k >= 8192) {
    nt = 4, slices = fill((p.n + 63) / 64 * batches, cus);
  } else if (mt == 2 && p.n >= 8192 && p.k >= 8192) {
    nt = 4, slices = fill((p.n + 63) / 64 * batches, 2 * cus);
  } else if (p.k >= (mt == 4 ? 2048u : 4096u)) {
    const uint32_t groups = (p.n + 31) / 32 * batches;
    slices = fill(groups, cus);
    if (p.m <= 16 && slices > 1) {
      if (groups * slices <= cus && chunks / (slices * 2) >= 14) slices *= 2;
      else if ((p.n + 15) / 16 * batches >= cus) slices = 1;
    }
  }
  if (slices == 1) {
    float best = 1e30f;
    for (int t = 1; t <= 4; t *= 2) {
      if (!built(t)) continue;
      const uint32_t cols = batches == 1 ? staged_cols(p.n, t, cus) : 16u * t, workgroups = (p.n + cols - 1) / cols * batches;
      const float cost = float((workgroups + cus - 1) / cus) * float(cols + p.m) * float(p.k) * (t == 4 && workgroups <= cus ? 1.25f : 1.0f);
      if (cost < best) best = cost, nt = t;
    }
  }
  if (forced_nt && built(int(forced_nt))) nt = int(forced_nt), slices = 1;
  if (forced_slices) slices = forced_slices;
  while (slices > 1 && slices * 2 > chunks) --slices;
  const uint32_t cols = slices == 1 && batches == 1 ? staged_cols(p.n, nt, cus) : 16u * nt;
  const uint64_t need = slices > 1 ? uint64_t((p.n + cols - 1) / cols) * batches * slices * mt * nt * 1024 : 0;
  if (need > mc.workspace_bytes) {
    if (mc.workspace_fixed) {
      *err = std::string(name) + ": this product's partial sums need " + std::to_string(need) + " bytes of workspace, the fixed workspace holds " +
             std::to_string(mc.workspace_bytes);
      return -1;
    }
    return -2;
  }
  // few columns against long rows without slices: 16 waves per workgroup where half of the compute units or more would
  // have none (a workgroup's waves take the chunks of k in turn: twice the waves, half the turns)
  if (mt == 1 && nt == 1 && slices == 1 && (p.n + cols - 1) / cols * batches * 2 <= cus && p.k >= 32 * 256)
    return launch_skinny_one<1, 1, 16, FA, FB, MATH>(p, cols, 1, 0, stream, err, name);
#define VKT_SKINNY_CASE(MT_, NT_, W_) \
  if (mt == MT_ && nt == NT_) return launch_skinny_one<MT_, NT_, W_, FA, FB, MATH>(p, cols, slices, mc.workspace, stream, err, name);
  VKT_SKINNY_CASE(1, 1, 8) VKT_SKINNY_CASE(1, 2, 8) VKT_SKINNY_CASE(2, 1, 8) VKT_SKINNY_CASE(2, 2, 8) VKT_SKINNY_CASE(2, 4, 4)
  VKT_SKINNY_CASE(4, 2, 8) VKT_SKINNY_CASE(4, 4, 4)
#undef VKT_SKINNY_CASE
  return -2;
}

// ---- The same product with the weights stored [k, n] (x @ w: rows of n, ldb bytes apart; 16-bit values).
// A workgroup owns 64 columns and all rows of A; its 8 waves take chunks of 64 rows of k in turn.  A wave's load
// instruction fetches 8 rows of k x 128 contiguous bytes (the workgroup's 64 columns), into registers a chunk ahead
// and from there into the wave's own 8 KiB of LDS in the global layout, and the matrix core's weight operand (lane
// (c, g): 8 values of k of column c) comes out of it through the transposing LDS read, two reads of 4 rows of k
// each.  16-byte pieces are swizzled by the row of k so that neither side has bank conflicts.  K in slices over
// workgroups as above (64 columns per workgroup are 128 workgroups at N = 8192).
template <int MT, int WAVES, int MATH, class Problem>
__global__ __launch_bounds__(WAVES * 64) void mma_skinny_kn(Problem p, uint32_t cols_per_wg, uint32_t chunks_per_slice, uint64_t workspace) {
  constexpr int NT = 4;
  constexpr uint32_t KC = 64, REGION = KC * 128;
  using V4S = short __attribute__((ext_vector_type(4)));
  extern __shared__ __attribute__((aligned(16))) uint8_t staged[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  uint8_t* const mine = staged + uint32_t(wave) * REGION;
  const uint32_t kv = p.k / 2, total = (kv + KC - 1) / KC, q_begin = blockIdx.y * chunks_per_slice;
  if (q_begin >= total) return;  // (an empty slice, which the launcher does not make)
  const uint32_t count = (q_begin + chunks_per_slice < total ? q_begin + chunks_per_slice : total) - q_begin;  // (no slice is empty)
  // the workgroup's columns: cols_per_wg of them (a multiple of 8, 64 at most; 64 when K is sliced over workgroups)
  const uint32_t n0 = blockIdx.x * cols_per_wg, n_end = n0 + cols_per_wg < p.n ? n0 + cols_per_wg : p.n;
  auto swizzle = [](uint32_t row) { return ((row & 3u) << 1) | ((row >> 3) & 1u); };
  // loads: instruction i fetches rows 8 i .. 8 i + 7 of the chunk; this lane row 8 i + lane / 8, piece lane % 8
  const uint32_t lrow = uint32_t(lane) >> 3, piece = uint32_t(lane) & 7u;
  const bool col_inside = n0 + 8 * piece < n_end;  // (n and the column count are multiples of 8: a piece is inside or outside as a whole)
  const uint64_t wbase = p.b + uint64_t(blockIdx.z) * p.b_batch, wsrc = wbase + uint64_t(n0 + 8 * piece) * 2;
  uint64_t arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const uint32_t m = uint32_t(16 * mt + c) < p.m ? 16 * mt + c : p.m - 1;
    arow[mt] = p.a + uint64_t(blockIdx.z) * p.a_batch + uint64_t(m) * p.lda + 16 * g;
  }
  V4F acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = V4F{0.0f, 0.0f, 0.0f, 0.0f};
  const U4 zero = {0, 0, 0, 0};
  U4 wr[8];
  auto request = [&](uint32_t q) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t k = q * KC + 8 * i + lrow;
      // (no branch around a load: what lies past k or n is fetched from the matrix's start and replaced by zeros)
      const bool inside = col_inside && k < kv;
      const U4 v = ldg_stream<U4>(inside ? wsrc + uint64_t(k) * p.ldb : wbase);
      wr[i] = inside ? v : zero;
    }
  };
  const uint32_t rot = (blockIdx.x * 5u) % count;
  auto chunk_at = [&](uint32_t i) { return q_begin + (i + rot) % count; };  // the i-th chunk this workgroup works on
  if (uint32_t(wave) < count) request(chunk_at(wave));
  for (uint32_t i = wave; i < count; i += WAVES) {
    const uint32_t k0 = chunk_at(i) * KC;
    U4 a[MT][4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool inside = k0 + 32 * j + 8 * g < kv;  // (k is a multiple of 8 values)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bool real = inside && uint32_t(16 * mt + c) < p.m;  // (rows past m are zeros, not loads)
        a[mt][j] = real ? ldg<U4>(arow[mt] + uint64_t(k0 + 32 * j) * 2) : zero;
        a[mt][j + 2] = zero;
      }
    }
#pragma unroll
    for (int i2 = 0; i2 < 8; ++i2) {
      const uint32_t row = 8 * i2 + lrow;
      *reinterpret_cast<U4*>(mine + row * 128 + ((piece ^ swizzle(row)) * 16)) = wr[i2];
    }
    if (i + WAVES < count) request(chunk_at(i + WAVES));
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        // (a wave's LDS operations execute in order: these reads see the writes above)
        // lane (c, g): column 16 t + c, k = 32 j + 8 g .. + 7: two reads of 4 rows of k; in each, lane c of a group of
        // 16 points at row + c / 4, values 4 (c % 4) .. + 3 of the tile's 16 columns, and receives column c's four
        U4 wv;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
          const uint32_t row = 32 * j + 8 * g + 4 * q + (uint32_t(c) >> 2);
          const uint32_t at = 2 * t + ((uint32_t(c) & 3u) >> 1);
          const V4S v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) V4S*)(mine + row * 128 + ((at ^ swizzle(row)) * 16) + (uint32_t(c) & 1u) * 8));
          const U2 w = __builtin_bit_cast(U2, v);
          wv[2 * q] = w.x, wv[2 * q + 1] = w.y;
        }
        skinny_step<MT, NT, 0, 0, MATH>(wv, a, j, t, acc);
      }
    }
  }
  __syncthreads();
  add_wave_tiles<MT, NT, WAVES>(acc, reinterpret_cast<V4F*>(staged), wave, lane);
  if (wave != 0) return;
  if (gridDim.y > 1) {
    V4F* const out = reinterpret_cast<V4F*>(workspace) + ((uint64_t(blockIdx.z) * gridDim.x + blockIdx.x) * gridDim.y + blockIdx.y) * (MT * NT * 64);
#pragma unroll
    for (int i = 0; i < MT * NT; ++i) out[i * 64 + lane] = acc[i / NT][i % NT];
    return;
  }
  skinny_store<MT, NT>(p, blockIdx.z, n0, n_end, acc, lane);
}

template <int MT, int MATH, class Problem>
int launch_skinny_kn_one(const Problem& p, uint32_t cols, uint32_t slices, uint64_t workspace, hipStream_t stream, std::string* err, const char* name) {
  constexpr int WAVES = 8;
  auto kernel = mma_skinny_kn<MT, WAVES, MATH, Problem>;
  constexpr uint32_t stage_bytes = WAVES * 64 * 128, part_bytes = kPartSlots<MT, 4, WAVES> * MT * 4 * 1024;
  constexpr uint32_t lds = stage_bytes > part_bytes ? stage_bytes : part_bytes;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
      (void)hipGetLastError();
      *err = std::string(name) + ": cannot reserve " + std::to_string(lds) + " bytes of LDS";
      return -1;
    }
    configured = true;
  }
  const uint32_t groups = (p.n + cols - 1) / cols;
  const KSlices cut = k_slices((p.k / 2 + 63) / 64, slices);  // (no empty slice)
  slices = cut.slices;
  const uint32_t per_slice = cut.chunks_per_slice;
  hipLaunchKernelGGL(kernel, dim3(groups, slices, p.batches), dim3(WAVES * 64), lds, stream, p, cols, per_slice, workspace);
  if (slices > 1) hipLaunchKernelGGL((mma_skinny_finish<MT, 4, Problem>), dim3(groups, 1, p.batches), dim3(64 * MT * 4), 0, stream, p, cols, slices, workspace);
  return 0;
}

// Up to 64 rows against weights stored [k, n] (16-bit values; n a multiple of 8, rows of k 16-byte aligned; 512 values
// of k and more, 64 columns and more).  Slices of K: a power of two that brings the workgroups up to one per compute
// unit while a wave keeps a chunk per slice; forced_slices instead (tests, tuning).  Return values as above.
template <int MATH, class Problem>
int launch_mma_skinny_kn(const Problem& p, const Machine& mc, uint32_t forced_slices, hipStream_t stream, std::string* err, const char* name) {
  const uint32_t batches = p.batches;
  if (p.m > 64 || p.k < 1024 || p.n < 64 || p.n % 8 || batches == 0 || batches > 65535) return -2;
  const uint32_t cus = uint32_t(mc.compute_units), chunks = (p.k / 2 + 63) / 64, groups = (p.n + 63) / 64 * batches;
  const int mt = p.m <= 16 ? 1 : p.m <= 32 ? 2 : 4;
  uint32_t slices = 1;
  while (groups * slices * 2 <= cus && chunks / (slices * 2) >= 8) slices *= 2;
  if (forced_slices) slices = forced_slices;
  while (slices > 1 && slices * 2 > chunks) --slices;
  const uint64_t need = slices > 1 ? uint64_t(groups) * slices * mt * 4 * 1024 : 0;
  if (need > mc.workspace_bytes) {
    if (mc.workspace_fixed) {
      *err = std::string(name) + ": this product's partial sums need " + std::to_string(need) + " bytes of workspace, the fixed workspace holds " +
             std::to_string(mc.workspace_bytes);
      return -1;
    }
    return -2;
  }
  // (64 columns whatever their count: dealt out evenly, N = 28672 in 56s, a workgroup's runs of 112 bytes straddle the
  //  128-byte lines and share them with its neighbours': 160 us against 92)
  const uint32_t cols = 64;
  if (mt == 1) return launch_skinny_kn_one<1, MATH>(p, cols, slices, mc.workspace, stream, err, name);
  if (mt == 2) return launch_skinny_kn_one<2, MATH>(p, cols, slices, mc.workspace, stream, err, name);
  return launch_skinny_kn_one<4, MATH>(p, cols, slices, mc.workspace, stream, err, name);
}

}  // namespace
}  // namespace vkt
