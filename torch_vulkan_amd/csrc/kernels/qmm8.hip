// aten::_weight_int8pack_mm on gfx950:  C[m,n] = round_T( scale[n] * sum_k A[m,k] * B[n,k] )
// for A [M,K] float32/float16/bfloat16 (unit stride along K), B int8 [N,K] contiguous,
// per-output-channel scales [N] in A's dtype, C [M,N] in A's dtype.
// Replaces the reference's crates/vkcore/shaders/qmm8.slang (GEMV :78-111, tiles :113-173)
// behind the same parameter block (crates/pyvk/csrc/quant.cpp:31-37).
//
// The op is a stream over the N*K weight bytes (HBM-bound up to M in the tens), so the
// kernels are built around that stream:
//   qmm8_gemv    M <= 16.  A wave owns COLS weight rows and walks K with one 16-byte
//                load per lane per row (1 KiB contiguous per wave per load, several in
//                flight), widens int8 -> float32 in registers (exact), accumulates every
//                row of A against it in float32 and reduces across the wave with DPP.
//                KSPLIT waves of a workgroup share a column group when N alone would
//                leave the machine's 1024 SIMDs short of work.  The per-channel scale is
//                applied once to the finished sum (the reference scales each weight; the
//                two differ by one float32 rounding, inside its test's tolerance).
//   qmm8_generic any shape, stride or alignment (K not a multiple of 16, unaligned rows):
//                a wave per output column, byte loads.
//   qmm8_mfma    4 < M (bfloat16 / float16 activations).  The stream is the same, the
//                arithmetic moves to the matrix cores: int8 weights widen exactly to
//                bfloat16 / float16 in registers, V_MFMA_F32_16X16X32_{BF16,F16} multiplies a
//                16-column weight fragment (converted once) against up to four 16-row
//                activation tiles, float32 accumulate.  The waves of a workgroup split K and
//                add their partial tiles in wave order through LDS (deterministic).
// Rows beyond the largest kernel's are served by the launcher in chunks (the weight stream
// is then re-read per chunk).
#include "common.h"
#include <type_traits>

#include "kernels.h"
#include "limits.h"
#include "wave_tiles.h"

namespace vkt {
namespace {

template <class T>
__device__ __forceinline__ void widen16_to_operands(const U4& v, U4* lo, U4* hi);

// a.x * w.x + a.y * w.y + acc on two 16-bit pairs (float32 result; the products of 16-bit values are exact)
template <class T>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t w, float acc) {
  if constexpr (T::dtype == VKT_BF16) {
    typedef __bf16 V2BF __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(V2BF, a), __builtin_bit_cast(V2BF, w), acc, false);
  } else {
    typedef _Float16 V2H __attribute__((ext_vector_type(2)));
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(V2H, a), __builtin_bit_cast(V2H, w), acc, false);
  }
}

template <class T, int ROWS, int COLS, int KSPLIT>
__global__ __launch_bounds__(256) void qmm8_gemv(Q8Params p) {
  constexpr int WAVES = 4, GROUPS = WAVES / KSPLIT;
  constexpr uint64_t item = sizeof(typename T::storage);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = wave / KSPLIT, ks = wave % KSPLIT;
  const uint32_t n0 = (blockIdx.x * GROUPS + grp) * COLS;

  float acc[ROWS][COLS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[r][c] = 0.0f;

  // rows of B this wave reads (clamped: the tail group re-reads the last row, masked at the store)
  uint64_t brow[COLS];
#pragma unroll
  for (int c = 0; c < COLS; ++c) {
    uint32_t n = n0 + c < p.n ? n0 + c : p.n - 1;
    brow[c] = p.b + uint64_t(n) * p.k;
  }
  uint64_t arow[ROWS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r) {
    uint32_t m = uint32_t(r) < p.m ? uint32_t(r) : p.m - 1;
    arow[r] = p.a + uint64_t(int64_t(m) * p.a_sm * int64_t(item));
  }

  for (uint32_t k = (ks * 64 + lane) * 16; k < p.k; k += 1024 * KSPLIT) {
    U4 wv[COLS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) wv[c] = ldg_stream<U4>(brow[c] + k);
    if constexpr (T::dtype != VKT_F32) {
      // 16-bit activations: the weights widen (exactly) to the activations' type once, and each row takes 8
      // two-element dot products per 16 weights, its activations as they are in memory (no conversions)
      U4 wlo[COLS], whi[COLS];
#pragma unroll
      for (int c = 0; c < COLS; ++c) widen16_to_operands<T>(wv[c], &wlo[c], &whi[c]);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        const U4 a0 = ldg<U4>(arow[r] + k * item), a1 = ldg<U4>(arow[r] + k * item + 16);
#pragma unroll
        for (int c = 0; c < COLS; ++c) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[r][c] = dot2<T>(a0[i], wlo[c][i], acc[r][c]);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[r][c] = dot2<T>(a1[i], whi[c][i], acc[r][c]);
        }
      }
    } else {
      float w[COLS][16];
#pragma unroll
      for (int c = 0; c < COLS; ++c) widen16_i8(wv[c], w[c]);
#pragma unroll
      for (int r = 0; r < ROWS; ++r) {
        float a[16];
        load16_f32<T>(arow[r] + k * item, a);
#pragma unroll
        for (int c = 0; c < COLS; ++c)
#pragma unroll
          for (int i = 0; i < 16; ++i) acc[r][c] = fmaf(a[i], w[c][i], acc[r][c]);
      }
    }
  }

#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[r][c] = wave_sum(acc[r][c]);

  __shared__ float part[WAVES][ROWS * COLS];
  if constexpr (KSPLIT > 1) {
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int c = 0; c < COLS; ++c) part[wave][r * COLS + c] = acc[r][c];
    }
    __syncthreads();
    if (ks != 0) return;
  }
  // lane (r, c) of the group's first wave finishes output (r, n0 + c)
  if (lane < ROWS * COLS) {
    const int r = lane / COLS, c = lane % COLS;
    float sum = 0.0f;
    // select acc[r][c] without dynamic register indexing
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr)
#pragma unroll
      for (int cc = 0; cc < COLS; ++cc)
        if (rr == r && cc == c) sum = acc[rr][cc];
    if constexpr (KSPLIT > 1) {
      sum = part[wave][lane];
#pragma unroll
      for (int s = 1; s < KSPLIT; ++s) sum += part[wave + s][lane];
    }
    const uint32_t n = n0 + c;
    if (uint32_t(r) < p.m && n < p.n) {
      const float scale = load_f32<T>(p.scales + n * item);
      store_f32<T>(p.c + (uint64_t(r) * p.n + n) * item, sum * scale);
    }
  }
}

// One activation row (the decode case): a persistent grid streams the weights.  A few workgroups per compute unit are
// launched (sixteen waves per unit, each with 4-8 KiB of weight loads in flight, saturate the memory system; thousands
// of short-lived workgroups pay for their launch, their ramp and their epilogue's dependent loads one after the other),
// and the waves walk through the weight rows in a fixed round-robin order.  A row is cut into chunks of 1 KiB (a
// wave's 16-byte load); KS waves of a workgroup (a team) share a row, wave ks taking chunks ks, ks + KS, ..., at most
// CH of them, and a team handles R rows per iteration.  What a lane needs of the activation row (CH x 16 values) stays
// in its registers for the whole kernel: the row is staged once per workgroup through LDS, requested before the first
// weights.  With KS > 1 the waves' sums meet in LDS (one barrier per iteration; all waves of a workgroup make the same
// number of iterations).
template <class T, int CH, int KS, int R>
__global__ __launch_bounds__(256) void qmm8_stream(Q8Params p) {
  constexpr int TEAMS = 4 / KS;
  constexpr bool F32 = T::dtype == VKT_F32;
  constexpr uint32_t item = sizeof(typename T::storage);
  extern __shared__ __attribute__((aligned(16))) uint8_t x_lds[];
  __shared__ float part[2][4][R];
  // (the wave's number as a scalar: row numbers and row addresses are then scalars too, and the loads take a scalar
  // base plus the lane's offset instead of per-lane 64-bit address arithmetic)
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t team = wave / KS, ks = wave % KS;
  const uint32_t chunks = (p.k + 1023) / 1024;
  // Row groups of R rows; a workgroup takes TEAMS neighbouring groups at a time (one per team), round-robin over the
  // grid, so that all its waves make the same number of iterations (the barriers below match).
  const uint32_t groups = (p.n + R - 1) / R, supers = (groups + TEAMS - 1) / TEAMS;
  if (blockIdx.x >= supers) return;  // (the whole workgroup, before any barrier)
  const uint32_t mine = (supers - blockIdx.x + gridDim.x - 1) / gridDim.x;
  auto group_of = [&](uint32_t i) { return (blockIdx.x + i * gridDim.x) * TEAMS + team; };

  // the activation row: global -> LDS (once per workgroup) -> this lane's CH x 16 values.  Requested before the
  // first weights (loads return in the order issued, and the row, which comes from L2, is needed first).
  const uint32_t x_pieces = p.k * item / 16;  // (k is a multiple of 16: whole pieces)
  constexpr int XP = (CH * KS * int(item) + 3) / 4;  // pieces per thread: k <= CH * KS * 1024
  U4 staged[XP];
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    // (no branch around a load: the compiler would wait for it on the spot; pieces past the row read its start)
    const uint32_t piece = tid + 256 * i;
    staged[i] = ldg<U4>(p.a + uint64_t(piece < x_pieces ? piece : 0) * 16);
  }
  __builtin_amdgcn_sched_barrier(0);  // (the scheduler would put the weights' loads first)

  uint32_t chunk_at[CH];  // byte offset of this lane's 16 bytes within a weight row, per chunk (0 past k)
  bool chunk_ok[CH];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const uint32_t c = ks + KS * j, at = c * 1024 + lane * 16;
    chunk_ok[j] = c < chunks && at < p.k;
    chunk_at[j] = chunk_ok[j] ? at : 0;
  }
  // (rows past n: the last row again, not stored)
  auto request = [&](U4 (&w)[R][CH], float* scale, uint32_t g) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const uint32_t n = g * R + r < p.n ? g * R + r : p.n - 1;
      const VKT_GLOBAL uint8_t* row = reinterpret_cast<const VKT_GLOBAL uint8_t*>(p.b + uint64_t(n) * p.k);
#pragma unroll
      for (int j = 0; j < CH; ++j) w[r][j] = __builtin_nontemporal_load(reinterpret_cast<const VKT_GLOBAL U4*>(row + chunk_at[j]));
    }
    // lane r of the team's first wave finishes row r: its scale comes with the weights, not after the sums
    const uint32_t n = g * R + (lane < uint32_t(R) ? lane : 0);
    *scale = load_f32<T>(p.scales + uint64_t(n < p.n ? n : p.n - 1) * item);
  };
  U4 cur[R][CH];
  float cur_scale;
  request(cur, &cur_scale, group_of(0));

#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const uint32_t piece = tid + 256 * i;
    if (piece < x_pieces) *reinterpret_cast<U4*>(x_lds + piece * 16) = staged[i];
  }
  __syncthreads();
  // values of k beyond the row are zeros (their weights are read from the row's start)
  float xf[F32 ? CH : 1][16];
  U4 xh[F32 ? 1 : CH][2];
#pragma unroll
  for (int j = 0; j < CH; ++j) {
    const uint32_t at = (ks + KS * j) * 1024 + lane * 16;  // first value of k
    if constexpr (F32) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const F4 v = chunk_ok[j] ? *reinterpret_cast<const F4*>(x_lds + (at + 4 * q) * 4) : F4{0.0f, 0.0f, 0.0f, 0.0f};
        xf[j][4 * q] = v.x, xf[j][4 * q + 1] = v.y, xf[j][4 * q + 2] = v.z, xf[j][4 * q + 3] = v.w;
      }
    } else {
#pragma unroll
      for (int q = 0; q < 2; ++q) xh[j][q] = chunk_ok[j] ? *reinterpret_cast<const U4*>(x_lds + (at + 8 * q) * 2) : U4{0, 0, 0, 0};
    }
  }

  // one group: products, sums over the wave, over the team's waves, scale, store
  auto finish = [&](const U4 (&w)[R][CH], float scale, uint32_t g, uint32_t i) {
    float sum[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // (two chains of dependent multiply-adds per chunk: one chain leaves the vector unit waiting for its own results)
      float acc[CH][2];
#pragma unroll
      for (int j = 0; j < CH; ++j) {
        acc[j][0] = acc[j][1] = 0.0f;
        if constexpr (F32) {
          float v[16];
          widen16_i8(w[r][j], v);
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[j][e & 1] = fmaf(xf[j][e], v[e], acc[j][e & 1]);
        } else {
          U4 lo, hi;
          widen16_to_operands<T>(w[r][j], &lo, &hi);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[j][0] = dot2<T>(xh[j][0][e], lo[e], acc[j][0]);
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[j][1] = dot2<T>(xh[j][1][e], hi[e], acc[j][1]);
        }
      }
      float row = 0.0f;
#pragma unroll
      for (int j = 0; j < CH; ++j) row += acc[j][0] + acc[j][1];
      sum[r] = wave_sum(row);
    }
    float total = 0.0f;
    if constexpr (KS > 1) {
      if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) part[i & 1][wave][r] = sum[r];
      }
      __syncthreads();  // (one per iteration: the next iteration writes the other half of `part`)
      if (ks == 0 && lane < uint32_t(R)) {
        total = part[i & 1][wave][lane];
#pragma unroll
        for (int q = 1; q < KS; ++q) total += part[i & 1][wave + q][lane];
      }
    } else {
#pragma unroll
      for (int r = 0; r < R; ++r) total = lane == uint32_t(r) ? sum[r] : total;
    }
    const uint32_t n = g * R + lane;
    if (ks == 0 && lane < uint32_t(R) && n < p.n) store_f32<T>(p.c + uint64_t(n) * item, total * scale);
  };

  // No software prefetch: the waves of a SIMD, each with its own group's loads in flight, cover each other's waits.
  // (A second register set filled an iteration ahead was tried in three forms: the compiler's waits for it came out as
  // waits for everything in flight.  So was one more pass through the products' code on zeros while the first loads
  // are on their way: a launch starts with a cold instruction cache, and a wave's first run through straight-line code
  // is held up at every 64-byte line of it, measured at ~40 ns a line; the register copies that form needed made it
  // wait for the loads all the same.)
  // (one copy of the products' code: every line of it that a launch runs through for the first time costs it time)
#pragma clang loop unroll(disable)
  for (uint32_t i = 0; i < mine; ++i) {
    if (i != 0) request(cur, &cur_scale, group_of(i));
    finish(cur, cur_scale, group_of(i), i);
  }
}

// One row through qmm8_stream where it applies (k up to 16384, 16-byte aligned rows).  variant bits 8-11 override
// the workgroups per compute unit, bits 12-15 the rows per iteration (tuning).  False: not this kernel's shape.
template <class T>
bool launch_stream(const Q8Params& p, uint32_t variant, const Machine& mc, hipStream_t stream) {
  const uint32_t chunks = (p.k + 1023) / 1024;
  if (p.m != 1 || chunks > 16 || p.k == 0) return false;
  const int ks = chunks <= 4 ? 1 : chunks <= 8 ? 2 : 4, ch = int((chunks + ks - 1) / ks);
  // rows per team and iteration: 8 KiB of weights in flight per wave (6 KiB with three chunks per row)
  const uint32_t teams = 4 / ks, per_cu = (variant >> 8) & 0xf ? (variant >> 8) & 0xf : 2;
  uint32_t rows_per = ch == 1 ? 8 : ch == 2 ? 4 : 2;
  if ((variant >> 12) & 0xf) rows_per = (variant >> 12) & 0xf;  // (tuning)
  const uint32_t groups = (p.n + rows_per - 1) / rows_per;
  uint32_t grid = uint32_t(mc.compute_units) * per_cu;
  if (grid * teams > groups) grid = (groups + teams - 1) / teams;
  const uint32_t lds = (p.k * sizeof(typename T::storage) + 15) / 16 * 16;
#define VKT_STREAM_CASE(CH_, KS_, R_)                                                                          \
  if (ch == CH_ && ks == KS_ && rows_per == R_) {                                                              \
    auto kernel = qmm8_stream<T, CH_, KS_, R_>;                                                                \
    static bool configured = false; /* guarded by the runtime's stream mutex */                                \
    if (!configured) {                                                                                         \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024) != hipSuccess) { \
        (void)hipGetLastError();                                                                               \
        return false;                                                                                          \
      }                                                                                                        \
      configured = true;                                                                                       \
    }                                                                                                          \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, stream, p);                                         \
    return true;                                                                                               \
  }
  VKT_STREAM_CASE(1, 1, 8) VKT_STREAM_CASE(2, 1, 4) VKT_STREAM_CASE(3, 1, 2) VKT_STREAM_CASE(4, 1, 2)
  VKT_STREAM_CASE(1, 1, 4) VKT_STREAM_CASE(2, 1, 2) VKT_STREAM_CASE(3, 1, 1) VKT_STREAM_CASE(4, 1, 1)
  VKT_STREAM_CASE(3, 2, 2) VKT_STREAM_CASE(4, 2, 2) VKT_STREAM_CASE(3, 4, 2) VKT_STREAM_CASE(4, 4, 2)
  VKT_STREAM_CASE(3, 2, 1) VKT_STREAM_CASE(4, 2, 1) VKT_STREAM_CASE(3, 4, 1) VKT_STREAM_CASE(4, 4, 1)
#undef VKT_STREAM_CASE
  return false;
}

// Any shape: a wave per output column, lanes strided along k with element loads, rows of
// A in chunks of 8.
template <class T>
__global__ __launch_bounds__(256) void qmm8_generic(Q8Params p) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t n = blockIdx.x * 4 + wave;
  if (n >= p.n) return;
  const uint64_t brow = p.b + uint64_t(n) * p.k;
  const float scale = load_f32<T>(p.scales + n * item);
  for (uint32_t m0 = blockIdx.y * 8; m0 < p.m; m0 += gridDim.y * 8) {
    float acc[8];
#pragma unroll
    for (int r = 0; r < 8; ++r) acc[r] = 0.0f;
    for (uint32_t k = lane; k < p.k; k += 64) {
      const float w = float(int(ldg<int8_t>(brow + k)));
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        const uint32_t m = m0 + r < p.m ? m0 + r : p.m - 1;
        acc[r] = fmaf(load_f32<T>(p.a + uint64_t((int64_t(m) * p.a_sm + k) * int64_t(item))), w, acc[r]);
      }
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const float sum = wave_sum(acc[r]);
      if (lane == 0 && m0 + r < p.m) store_f32<T>(p.c + (uint64_t(m0 + r) * p.n + n) * item, sum * scale);
    }
  }
}

using V8BF = __bf16 __attribute__((ext_vector_type(8)));
using V8H = _Float16 __attribute__((ext_vector_type(8)));

// 16 int8 weights (one 16-byte load) as two MFMA operands of 8 elements in T (exact).
template <class T>
__device__ __forceinline__ void widen16_to_operands(const U4& v, U4* lo, U4* hi) {
  uint32_t out[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float f0 = float(int(int8_t(v[i]))), f1 = float(int(int8_t(v[i] >> 8)));
    const float f2 = float(int(int8_t(v[i] >> 16))), f3 = float(int(int8_t(v[i] >> 24)));
    if constexpr (T::dtype == VKT_BF16 || T::dtype == VKT_F32) {  // (float32 activations go to the bfloat16 matrix core in three parts)
      // an integer of magnitude <= 128 is its float32's upper 16 bits
      out[2 * i] = __builtin_amdgcn_perm(f32_bits(f1), f32_bits(f0), 0x07060302u);
      out[2 * i + 1] = __builtin_amdgcn_perm(f32_bits(f3), f32_bits(f2), 0x07060302u);
    } else {
      out[2 * i] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(f0, f1));
      out[2 * i + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(f2, f3));
    }
  }
  *lo = U4{out[0], out[1], out[2], out[3]};
  *hi = U4{out[4], out[5], out[6], out[7]};
}

template <class T>
__device__ __forceinline__ V4F mfma16(const U4& w, const U4& a, const V4F& acc) {
  if constexpr (T::dtype == VKT_BF16 || T::dtype == VKT_F32)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(V8BF, w), __builtin_bit_cast(V8BF, a), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(V8H, w), __builtin_bit_cast(V8H, a), acc, 0, 0, 0);
}

// A workgroup owns 16*NT output columns; its WAVES waves take the 64-wide k-steps in turn.
// Lane (c = lane % 16, g = lane / 16) streams 16 bytes of weight row n0 + 16 t + c at
// k0 + 16 g (two MFMA operands) and the matching 16 activations of rows 16 mt + c; the
// MFMA's first operand is the weights, so the lane ends with C[16 mt + c][n0 + 16 t + 4 g + r].
// The epilogue of the matrix-core kernels: lane (c = lane % 16, g = lane / 16) holds, per
// tile (mt, t), the sums of row m0 + 16 mt + c for columns n0 + 16 t + 4 g .. + 3.
template <class T, int MT, int NT>
__device__ __forceinline__ void store_tiles(const Q8Params& p, uint32_t n0, const V4F (&acc)[MT][NT], int lane, uint32_t n_end = ~0u, uint32_t m0 = 0) {
  n_end = n_end < p.n ? n_end : p.n;  // (columns from n_end on are another workgroup's; a multiple of 4, or n)
  constexpr uint64_t item = sizeof(typename T::storage);  // (scales and outputs have the activations' type)
  constexpr bool F32 = T::dtype == VKT_F32;
  const int c = lane & 15, g = lane >> 4;
  const bool vec_ok = (p.n & 3u) == 0 && (p.c & (4 * item - 1)) == 0;
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const uint32_t n = n0 + 16 * t + 4 * g;
    float scale[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) scale[r] = load_f32<T>(p.scales + (n + r < p.n ? n + r : p.n - 1) * item);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const uint32_t m = m0 + 16 * mt + c;
      if (m >= p.m || n >= n_end) continue;
      const uint64_t at = p.c + (uint64_t(m) * p.n + n) * item;
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = acc[mt][t][r] * scale[r];
      if constexpr (F32) {
        if (vec_ok && n + 3 < n_end) {
          stg<F4>(at, F4{v[0], v[1], v[2], v[3]});
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < n_end) stg<float>(at + r * item, v[r]);
        }
      } else {
        uint32_t h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = T::dtype == VKT_BF16 ? f32_to_bf16(v[r]) : f32_to_f16(v[r]);
        if (vec_ok && n + 3 < n_end) {
          stg<U2>(at, U2{h[0] | h[1] << 16, h[2] | h[3] << 16});
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < n_end) stg<uint16_t>(at + r * item, uint16_t(h[r]));
        }
      }
    }
  }
}

template <class T, int MT, int NT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void qmm8_mfma(Q8Params p, uint32_t chunks_per_slice, uint64_t workspace) {
  constexpr uint64_t item = 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  // gridDim.y slices of K (in chunks of 64 values), one per workgroup of the column group
  const uint32_t k_begin = blockIdx.y * chunks_per_slice * 64;
  const uint32_t k_end = k_begin + chunks_per_slice * 64 < p.k ? k_begin + chunks_per_slice * 64 : p.k;
  const uint32_t n0 = blockIdx.x * 16 * NT;
  uint64_t brow[NT], arow[MT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const uint32_t n = n0 + 16 * t + c < p.n ? n0 + 16 * t + c : p.n - 1;
    brow[t] = p.b + uint64_t(n) * p.k + 16 * g;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const uint32_t m = uint32_t(16 * mt + c) < p.m ? 16 * mt + c : p.m - 1;
    arow[mt] = p.a + uint64_t(int64_t(m) * p.a_sm * int64_t(item)) + 32 * g;
  }
  V4F acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = V4F{0.0f, 0.0f, 0.0f, 0.0f};

  const U4 zero = {0, 0, 0, 0};
#pragma unroll 2
  for (uint32_t k0 = k_begin + wave * 64; k0 < k_end; k0 += WAVES * 64) {
    const bool inside = k0 + 16 * g < p.k;  // (k is a multiple of 16)
    U4 wv[NT], a0[MT], a1[MT];
#pragma unroll
    for (int t = 0; t < NT; ++t) wv[t] = inside ? ldg_stream<U4>(brow[t] + k0) : zero;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const bool real = inside && uint32_t(16 * mt + c) < p.m;  // (rows past m are zeros, not loads)
      a0[mt] = real ? ldg<U4>(arow[mt] + k0 * item) : zero;
      a1[mt] = real ? ldg<U4>(arow[mt] + k0 * item + 16) : zero;
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      U4 wlo, whi;
      widen16_to_operands<T>(wv[t], &wlo, &whi);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        acc[mt][t] = mfma16<T>(wlo, a0[mt], acc[mt][t]);
        acc[mt][t] = mfma16<T>(whi, a1[mt], acc[mt][t]);
      }
    }
  }

  // the waves' partial tiles meet in wave 0
  __shared__ V4F part[kPartSlots<MT, NT, WAVES>][MT * NT][64];
  add_wave_tiles<MT, NT, WAVES>(acc, &part[0][0][0], wave, lane);
  if (wave != 0) return;
  if (gridDim.y > 1) {
    // one of several slices of K: the tile goes to the workspace, and qmm8_mfma_finish adds
    // the slices up in slice order
    V4F* const mine = reinterpret_cast<V4F*>(workspace) + (uint64_t(blockIdx.x) * gridDim.y + blockIdx.y) * (MT * NT * 64);
#pragma unroll
    for (int i = 0; i < MT * NT; ++i) mine[i * 64 + lane] = acc[i / NT][i % NT];
    return;
  }
  store_tiles<T, MT, NT>(p, n0, acc, lane);
}

// The same product with the weights staged through LDS, so that HBM sees long runs: a wave's
// load instruction fetches 4 weight rows x 256 contiguous bytes (in qmm8_mfma it is 16 rows x 64
// bytes, a pattern this memory system serves ~30 % slower) straight into the wave's own LDS
// region (global_load_lds_dwordx4: lane l's 16 bytes land at region + 16 l).  The matrix-core
// operand layout (lane (c, g): row c, bytes 16 g ..) is then a 16-byte LDS read.  The 16-byte
// chunk q of row r sits at slot q ^ r, so that the 16 lanes of a read (rows 0..15, one logical
// chunk) fall on 16 different slots of the 256-byte bank line; the swizzle costs nothing, the
// lane simply fetches the chunk that belongs in its slot.  A wave works on chunks of 256
// values of k: all loads of a chunk are issued, awaited (vmcnt(0)) and consumed; the waves of a
// workgroup drift apart and keep the memory pipeline full between them.
// PLANES = 3 (float32 outputs): the activations are three bfloat16 planes [3][m][k] whose sum the float32 activations
// are, exactly (qmm8_split_rows wrote them); every weight fragment multiplies the three planes' fragments one after
// the other into the same sums, which is the product of the float32 values added up in float32.
template <class T, int MT, int NT, int WAVES, int PLANES>
__global__ __launch_bounds__(WAVES * 64) void qmm8_mfma_staged(Q8Params p, uint32_t chunks_per_slice, uint64_t workspace, uint32_t cols_per_wg) {
  constexpr uint64_t item = 2;  // (of the activations as this kernel reads them)
  const uint64_t plane_bytes = PLANES > 1 ? uint64_t(p.m) * p.k * item : 0;  // (planes: rows k values apart)
  constexpr uint32_t TILE = 16 * 256, REGION = NT * TILE;  // bytes of LDS per tile of 16 rows, per wave
  extern __shared__ __attribute__((aligned(16))) uint8_t staged[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  uint8_t* const mine = staged + uint32_t(wave) * REGION;
  const uint32_t total = (p.k + 255) / 256;
  const uint32_t q_begin = blockIdx.y * chunks_per_slice;
  const uint32_t q_end = q_begin + chunks_per_slice < total ? q_begin + chunks_per_slice : total;
  if (q_begin >= total) return;  // (an empty slice, which the launchers do not make: the chunk count below would wrap around)
  // the workgroup's columns: cols_per_wg of them (at most 16 NT, a multiple of 4; 16 NT when K is sliced over workgroups)
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
      wsrc[t][i] = p.b + uint64_t(n) * p.k;
    }
  }
  uint64_t arow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const uint32_t m = uint32_t(16 * mt + c) < p.m ? 16 * mt + c : p.m - 1;
    arow[mt] = p.a + uint64_t(int64_t(m) * p.a_sm * int64_t(item)) + 32 * g;
  }
  V4F acc[MT][NT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[mt][t] = V4F{0.0f, 0.0f, 0.0f, 0.0f};

  const U4 zero = {0, 0, 0, 0};
  // The weights of a chunk are loaded into registers a chunk ahead (non-temporal 16-byte loads: this part streams
  // from HBM ~1.5x as fast that way as straight into LDS with global_load_lds_dwordx4, measured with the loads alone)
  // and written to the wave's region when their turn comes.
  U4 wr[NT][4];
  auto request = [&](uint32_t q) {
    const uint32_t k0 = q * 256;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        // (bytes past k are fetched from the row's start instead: their activations are zeros below)
        wr[t][i] = ldg_stream<U4>(wsrc[t][i] + (k0 + wk[i] < p.k ? k0 + wk[i] : 0u));
      }
  };
  // Workgroups start at different chunks of their slice and wrap around: with rows a power of two apart, all
  // workgroups reading the same offsets of their rows at the same time keep to a few memory channels.
  const uint32_t count = q_end - q_begin, rot = (blockIdx.x * 5u) % count;
  auto chunk_at = [&](uint32_t i) { return q_begin + (i + rot) % count; };  // the i-th chunk this workgroup works on
  if (uint32_t(wave) < count) request(chunk_at(wave));
  for (uint32_t i = wave; i < count; i += WAVES) {
    const uint32_t q = chunk_at(i);
    const uint32_t k0 = q * 256;
    U4 a0[PLANES][MT][4], a1[PLANES][MT][4];
#pragma unroll
    for (int pl = 0; pl < PLANES; ++pl)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const bool inside = k0 + 64 * j + 16 * g < p.k;  // (k is a multiple of 16)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          // (rows past m are zeros, not loads: with 8 rows that is half of the activation traffic)
          const bool real = inside && uint32_t(16 * mt + c) < p.m;
          a0[pl][mt][j] = real ? ldg<U4>(arow[mt] + pl * plane_bytes + (k0 + 64 * j) * item) : zero;
          a1[pl][mt][j] = real ? ldg<U4>(arow[mt] + pl * plane_bytes + (k0 + 64 * j) * item + 16) : zero;
        }
      }
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) *reinterpret_cast<U4*>(mine + (t * 16 + 4 * i) * 256 + lane * 16) = wr[t][i];
    if (i + WAVES < count) request(chunk_at(i + WAVES));
#pragma unroll
    for (int j = 0; j < 4; ++j) {
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        // (a wave's LDS operations execute in order: these reads see the writes above)
        const U4 wv = *reinterpret_cast<const U4*>(mine + (t * 16 + c) * 256 + (((4 * j + g) ^ c) & 15) * 16);
        U4 wlo, whi;
        widen16_to_operands<T>(wv, &wlo, &whi);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
          for (int pl = 0; pl < PLANES; ++pl) {
            acc[mt][t] = mfma16<T>(wlo, a0[pl][mt][j], acc[mt][t]);
            acc[mt][t] = mfma16<T>(whi, a1[pl][mt][j], acc[mt][t]);
          }
      }
    }
  }

  // the waves' partial tiles meet in wave 0 (through the staging memory, once every wave is done with it)
  __syncthreads();
  add_wave_tiles<MT, NT, WAVES>(acc, reinterpret_cast<V4F*>(staged), wave, lane);
  if (wave != 0) return;
  if (gridDim.y > 1) {
    V4F* const out = reinterpret_cast<V4F*>(workspace) + (uint64_t(blockIdx.x) * gridDim.y + blockIdx.y) * (MT * NT * 64);
#pragma unroll
    for (int i = 0; i < MT * NT; ++i) out[i * 64 + lane] = acc[i / NT][i % NT];
    return;
  }
  store_tiles<T, MT, NT>(p, n0, acc, lane, n_end);
}

// Adds up the slices of one column group, in slice order, and runs the epilogue: a workgroup per group, its waves (one
// per 16 x 16 tile, 16 at most) take the tiles in turn, four slices' loads in flight.
template <int MT, int NT>
constexpr int kFinishWaves = MT * NT < 16 ? MT * NT : 16;
template <class T, int MT, int NT>
__global__ __launch_bounds__((64 * kFinishWaves<MT, NT>)) void qmm8_mfma_finish(Q8Params p, uint32_t slices, uint64_t workspace) {
  constexpr uint32_t GROUP = MT * NT * 64;  // V4F per slice of a group
  const int lane = threadIdx.x & 63;
  for (int tile = threadIdx.x >> 6; tile < MT * NT; tile += kFinishWaves<MT, NT>) {
    const V4F* const mine = reinterpret_cast<const V4F*>(workspace) + uint64_t(blockIdx.x) * slices * GROUP + tile * 64 + lane;
    V4F acc[1][1];
    acc[0][0] = mine[0];
    uint32_t sl = 1;
    for (; sl + 4 <= slices; sl += 4) {
      const V4F a = mine[uint64_t(sl) * GROUP], b = mine[uint64_t(sl + 1) * GROUP], c = mine[uint64_t(sl + 2) * GROUP], d = mine[uint64_t(sl + 3) * GROUP];
      acc[0][0] += a, acc[0][0] += b, acc[0][0] += c, acc[0][0] += d;
    }
    for (; sl < slices; ++sl) acc[0][0] += mine[uint64_t(sl) * GROUP];
    store_tiles<T, 1, 1>(p, blockIdx.x * 16 * NT + 16 * (tile % NT), acc, lane, ~0u, 16 * (tile / NT));
  }
}

template <class T, int MT, int NT>
void launch_mfma_waves(const Q8Params& p, int waves, uint32_t slices, const Machine& mc, hipStream_t stream) {
  const dim3 grid((p.n + 16 * NT - 1) / (16 * NT), slices);
  const uint32_t chunks = (p.k + 63) / 64, per_slice = (chunks + slices - 1) / slices;
  switch (waves) {
    case 4: hipLaunchKernelGGL((qmm8_mfma<T, MT, NT, 4>), grid, dim3(256), 0, stream, p, per_slice, mc.workspace); break;
    case 8: hipLaunchKernelGGL((qmm8_mfma<T, MT, NT, 8>), grid, dim3(512), 0, stream, p, per_slice, mc.workspace); break;
    default: hipLaunchKernelGGL((qmm8_mfma<T, MT, NT, 16>), grid, dim3(1024), 0, stream, p, per_slice, mc.workspace); break;
  }
  if (slices > 1) hipLaunchKernelGGL((qmm8_mfma_finish<T, MT, NT>), dim3(grid.x), dim3(64 * kFinishWaves<MT, NT>), 0, stream, p, slices, mc.workspace);
}

template <class T, int MT, int NT, int WAVES, int PLANES = 1>
bool launch_staged_one(const Q8Params& p, uint32_t slices, const Machine& mc, hipStream_t stream) {
  auto kernel = qmm8_mfma_staged<T, MT, NT, WAVES, PLANES>;
  constexpr uint32_t stage_bytes = WAVES * NT * 16 * 256, part_bytes = kPartSlots<MT, NT, WAVES> * MT * NT * 1024;
  constexpr uint32_t lds = stage_bytes > part_bytes ? stage_bytes : part_bytes;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
      (void)hipGetLastError();
      return false;
    }
    configured = true;
  }
  // One slice: the columns are dealt out evenly over a whole number of workgroups per compute unit (N = 14336 in 32s is
  // 448 workgroups, two for 192 of 256 units and one for the rest, and the launch lasts as long as the two take; in 28s
  // it is 512, two for each: the same bytes everywhere).  Several slices: whole tiles, which the second launch expects.
  const uint32_t cols = slices == 1 ? staged_cols(p.n, NT, uint32_t(mc.compute_units)) : 16 * NT;
  const KSlices cut = k_slices((p.k + 255) / 256, slices);  // (no empty slice: 65 chunks in 16 slices of 5 are 13 slices)
  slices = cut.slices;
  const uint32_t per_slice = cut.chunks_per_slice;
  const dim3 grid((p.n + cols - 1) / cols, slices);
  hipLaunchKernelGGL(kernel, grid, dim3(WAVES * 64), lds, stream, p, per_slice, mc.workspace, cols);
  if (slices > 1) hipLaunchKernelGGL((qmm8_mfma_finish<T, MT, NT>), dim3(grid.x), dim3(64 * kFinishWaves<MT, NT>), 0, stream, p, slices, mc.workspace);
  return true;
}

// The staged kernel for up to 32 rows (MT <= 2: the activations of a chunk fit in registers next to the
// accumulators).  variant = NT | WAVES << 8 | SLICES << 24 | 1 << 18.  False if this shape is not built.
template <class T>
bool launch_staged(const Q8Params& p, int mt, int nt, int waves, uint32_t slices, const Machine& mc, hipStream_t stream) {
#define VKT_STAGED_CASE(MT_, NT_, W_) \
  if (mt == MT_ && nt == NT_ && waves == W_) return launch_staged_one<T, MT_, NT_, W_>(p, slices, mc, stream);
  VKT_STAGED_CASE(1, 1, 4) VKT_STAGED_CASE(1, 2, 4) VKT_STAGED_CASE(1, 4, 4) VKT_STAGED_CASE(1, 1, 8) VKT_STAGED_CASE(1, 2, 8) VKT_STAGED_CASE(1, 4, 8)
  VKT_STAGED_CASE(2, 1, 4) VKT_STAGED_CASE(2, 2, 4) VKT_STAGED_CASE(2, 4, 4) VKT_STAGED_CASE(2, 1, 8) VKT_STAGED_CASE(2, 2, 8) VKT_STAGED_CASE(2, 4, 8)
#undef VKT_STAGED_CASE
  return false;
}

// Three to eight rows of 16-bit activations, rows of up to 4096 values, many columns (batched decode at small batch
// against a vocabulary-sized projection of a small model: K = 2048 or 3072, N = 128256): the weight stream of the
// one-row kernels with the arithmetic on the matrix cores.  One workgroup of 8 waves per compute unit stays for the
// whole launch and owns a run of consecutive columns, the same count for every workgroup.  A column group is 16
// weight rows; KS waves share its K, each taking every KS-th chunk of 512 bytes of every row: 8 loads of 2 rows x 512
// contiguous bytes, into registers, two chunks ahead.  A chunk goes through the wave's own 8 KiB of LDS (16-byte
// pieces swizzled by the row, so that neither side has a bank conflict) to come back in the matrix core's operand
// shape (lane (c, g): row c, 16 bytes of k), is widened exactly to the activations' type and multiplied by the
// activations' fragments.  Those come out of LDS too: all rows of A (8 rows x K <= 4096 values), staged once per
// workgroup and asked for before any weights.  The KS partial tiles of a group meet in LDS, added in wave order.
// (The slice kernels above give a workgroup's waves K / 256 chunks to share: with short rows that is one chunk per
// wave and nothing to overlap.  With longer rows they win: K = 4096, N = 128256: 89.9 us against 88.4 here, K = 8192:
// 172 against 180 with the activations loaded per chunk, a form this kernel had and lost.)
// What was measured (8 x 4096 x 14336, timestamps inside the kernel): a compute unit accepts about 64 KiB of loads
// before the issue of further ones blocks, and its older waves issue first.  So the second chunk in flight buys
// little at the start and much in the steady state (the stream runs at 6.2 TB/s; a chunk costs a pair of waves
// 1.45 us, which is the vector units' time: widening 16 weights is 24 instructions of 4-5 cycles, the matrix cores'
// two instructions of 16 cycles per 64 values of k hide behind them), and the younger wave of every SIMD gets its
// chunks later than the older one throughout: a unit's last two microseconds stream for half of its waves.  (A
// barrier of issue per chunk, which keeps the waves level, costs more than that: 17.6 against 16.6 us.)  The loop
// over a chunk's eight 64-value steps is rolled (a launch starts with a cold instruction cache).
constexpr uint32_t kRowsChunk = 512, kRowsRegion = 16 * kRowsChunk, kRowsWaves = 8;
constexpr int kRawBuffer = 0x00020000;  // descriptor word 3: raw (unstructured) buffer, 32-bit data format
constexpr int kLoadStream = 2;          // the nt bit: read once

// activations in LDS: per row and block of 64 values the eight 16-byte pieces are kept as [first halves of the four
// k-groups | second halves], so that the 32 distinct pieces one read instruction fetches (8 rows x 4 groups) cover
// every bank twice; the row pitch is 64 bytes past a multiple of 256
// (rows run to the end of the last 512-value chunk, zeros past k)
__host__ __device__ inline uint32_t rows_a_pitch(uint32_t k) { return 2 * ((k + 511) / 512 * 512) + 64; }
__device__ __forceinline__ uint32_t rows_a_slot(uint32_t piece) { return (piece / 8) * 128 + (piece & 1u) * 64 + ((piece & 7u) >> 1) * 16; }

template <class T, int KS>
__global__ __launch_bounds__(512) void qmm8_rows(Q8Params p, uint32_t cols_per_wg) {
  constexpr uint64_t item = 2;
  constexpr uint32_t TEAMS = kRowsWaves / KS;
  extern __shared__ __attribute__((aligned(16))) uint8_t rows_lds[];
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t c = lane & 15, g = lane >> 4, team = wave / KS, ks = wave % KS;
  const uint32_t chunks = (p.k + kRowsChunk - 1) / kRowsChunk, per_wave = (chunks + KS - 1) / KS;
  const uint32_t a_pitch = rows_a_pitch(p.k), a_bytes = 8 * a_pitch;
  uint8_t* const region = rows_lds + a_bytes + wave * kRowsRegion;
  V4F* const parts = reinterpret_cast<V4F*>(rows_lds + a_bytes + kRowsWaves * kRowsRegion);  // [2][8 waves][64 lanes]
  uint16_t* const scales_lds = reinterpret_cast<uint16_t*>(parts + 2 * kRowsWaves * 64);  // [8 waves][16]

  // A workgroup owns cols_per_wg consecutive columns (a multiple of 8; the same count for every workgroup, so that
  // every compute unit streams the same bytes: with whole groups of 16 dealt out, 896 groups leave 32 of 256 units
  // idle or give 192 of them twice the work of the rest), as groups of 16 of which the last may be partial.  In round
  // i team t works on the workgroup's group i * TEAMS + t (all teams make the same number of rounds: the barrier
  // below is the workgroup's).
  const uint32_t col_begin = blockIdx.x * cols_per_wg, col_end = min(col_begin + cols_per_wg, p.n);
  const uint32_t rounds = ((cols_per_wg + 15) / 16 + TEAMS - 1) / TEAMS;
  auto first_col = [&](uint32_t round) { return col_begin + (round * TEAMS + team) * 16; };  // (at or past col_end: no group)
  // (workgroups walk K from different starting chunks and wrap around: with rows a power of two apart, all of them
  // reading the same offsets of their rows at the same time keep to a few memory channels)
  const uint32_t rot = (blockIdx.x * 3u) % chunks;
  const uint32_t items = rounds * per_wave;  // (group, chunk) pairs of this wave, some of them past the end
  // Two chunks are in flight per wave (registers), requested as soon as the registers are free.
  U4 w[2][8];
  uint16_t scl[2];
  // Weights, scales and activations are read through buffer descriptors: a load whose offset lies past
  // the buffer returns zeros and touches no memory, so rows past n, pieces past k and requests past the wave's last
  // item cost nothing, and every request is the same number of loads on every path (each wait below is then for its
  // own chunk only: a path without its loads would make every later wait a wait for everything).
  const __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(p.b), 0, int(p.n * p.k), kRawBuffer);
  const __amdgpu_buffer_rsrc_t s_rsrc = __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(p.scales), 0, int(p.n * item), kRawBuffer);
  const __amdgpu_buffer_rsrc_t a_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void*>(p.a), 0, int((uint32_t(p.m - 1) * uint32_t(p.a_sm) + p.k) * item), kRawBuffer);
  auto request = [&](auto set, uint32_t j) {
    constexpr int S = decltype(set)::value;
    // (the fences keep one request's loads together and in program order, which is what the waits count on)
    __builtin_amdgcn_sched_barrier(0);
    const uint32_t n0 = first_col(j / per_wave), turn = (j % per_wave) * KS + ks, chunk = (turn + rot) % chunks;
    const uint32_t dead = j < items && n0 < col_end && turn < chunks ? 0u : ~0u;  // (all ones: past every buffer)
    const uint32_t at = chunk * kRowsChunk + (lane & 31u) * 16;
    const uint32_t row0 = n0 + (lane >> 5), gone = dead | (at < p.k ? 0u : ~0u);
#pragma unroll
    for (int i = 0; i < 8; ++i)  // rows 2 i + lane / 32
      w[S][i] = __builtin_amdgcn_raw_buffer_load_b128(b_rsrc, ((row0 + 2 * i) * p.k + at) | gone | (row0 + 2 * i < col_end ? 0u : ~0u), 0, kLoadStream);
    // the group's 16 scales come with every chunk and go through LDS with it (loaded in the epilogue they would be
    // waited for behind two chunks in flight)
    scl[S] = __builtin_amdgcn_raw_buffer_load_b16(s_rsrc, ((n0 + c) * uint32_t(item)) | dead | (n0 + c < col_end ? 0u : ~0u), 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  };
  {
    // all rows, once per workgroup: row i's piece `tid` (a row has at most 512 pieces), through the same kind of
    // descriptor; asked for before any weights.  The two barriers before the one that publishes A are barriers of
    // ISSUE, not of data: a compute unit accepts ~64 KiB of loads and lets the oldest wave's instructions go first, so
    // without them the first waves' second chunks are accepted before the last wave's first one, that wave cannot
    // reach the code that writes its pieces of A to LDS, and everyone waits for it (compute started 5.7 us into the
    // launch; with them 3.8-4.6)
    U4 a_regs[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      a_regs[i] = __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, (tid * 16 + i * uint32_t(p.a_sm) * uint32_t(item)) | (uint32_t(i) < p.m && tid * 8 < p.k ? 0u : ~0u), 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    request(std::integral_constant<int, 0>{}, 0);
    __builtin_amdgcn_s_barrier();  // (every wave's first chunk before any wave's second)
    __builtin_amdgcn_sched_barrier(0);
    if (tid * 16 < a_pitch - 64) {
      uint32_t at = rows_a_slot(tid);
#pragma unroll
      for (int i = 0; i < 8; ++i, at += a_pitch) *reinterpret_cast<U4*>(rows_lds + at) = a_regs[i];
    }
    __syncthreads();
    request(std::integral_constant<int, 1>{}, 1);
  }
  const uint8_t* const a_frag = rows_lds + (c & 7u) * a_pitch + 16 * g;

  V4F acc0 = {0.0f, 0.0f, 0.0f, 0.0f}, acc1 = acc0;
  auto work = [&](auto set, uint32_t j) {
    constexpr int S = decltype(set)::value;
    const uint32_t round = j / per_wave, turn = (j % per_wave) * KS + ks, chunk = (turn + rot) % chunks, n0 = first_col(round);
    // the chunk's 16 rows into the wave's region: piece q of row r at slot q ^ r
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t r = 2 * i + (lane >> 5);
      *reinterpret_cast<U4*>(region + r * kRowsChunk + (((lane & 31u) ^ r) * 16)) = w[S][i];
    }
    scales_lds[wave * 16 + c] = scl[S];  // (four lanes write each, the same value)
    request(set, j + 2);
    if (j < items && turn < chunks && n0 < col_end) {
      const uint32_t k0 = chunk * kRowsChunk;
      // a step's operand reads are issued a step ahead (two register sets, used in turn)
      struct Step {
        U4 wv, a0, a1;
      };
      auto fetch = [&](Step& x, uint32_t s) {
        // (a wave's LDS operations execute in order: these reads see the writes above)
        x.wv = *reinterpret_cast<const U4*>(region + c * kRowsChunk + (((4 * s + g) ^ c) * 16));
        x.a0 = *reinterpret_cast<const U4*>(a_frag + 2 * (k0 + 64 * s));
        x.a1 = *reinterpret_cast<const U4*>(a_frag + 2 * (k0 + 64 * s) + 64);
      };
      auto multiply = [&](const Step& x) {
        U4 wlo, whi;
        widen16_to_operands<T>(x.wv, &wlo, &whi);
        acc0 = mfma16<T>(wlo, x.a0, acc0);
        acc1 = mfma16<T>(whi, x.a1, acc1);
      };
      Step even, odd;
      fetch(even, 0);
#pragma clang loop unroll(disable)
      for (uint32_t s = 0; s < 8; s += 2) {
        fetch(odd, s + 1);
        __builtin_amdgcn_sched_barrier(0);  // (the scheduler would move each read down to its first use)
        multiply(even);
        fetch(even, s + 2 < 8 ? s + 2 : 7);
        __builtin_amdgcn_sched_barrier(0);
        multiply(odd);
      }
    }
    if (j < items && (j + 1) % per_wave == 0) {  // the round's last chunk: the team's tiles meet in its first wave, added in wave order
      V4F sum;
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] = acc0[r] + acc1[r];
      if constexpr (KS > 1) {
        V4F* const slot = parts + (round & 1u) * (kRowsWaves * 64);  // (two sets of slots: one barrier per round)
        slot[wave * 64 + lane] = sum;
        __syncthreads();
        if (ks == 0) {
#pragma unroll
          for (int q = 1; q < KS; ++q) {
            const V4F v = slot[(wave + q) * 64 + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) sum[r] += v[r];
          }
        }
      }
      // lane (c, g): row c, columns n0 + 4 g .. + 3 (a partial group ends at col_end, a multiple of 8 or n)
      const uint32_t n = n0 + 4 * g;
      if (ks == 0 && c < p.m && n < col_end) {
        const uint64_t to = p.c + (uint64_t(c) * p.n + n) * item;
        uint32_t h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const uint16_t bits = scales_lds[wave * 16 + 4 * g + r];
          const float v = sum[r] * (T::dtype == VKT_BF16 ? bf16_to_f32(bits) : f16_to_f32(bits));
          h[r] = T::dtype == VKT_BF16 ? f32_to_bf16(v) : f32_to_f16(v);
        }
        if ((p.n & 3u) == 0 && (p.c & 7u) == 0) {
          stg<U2>(to, U2{h[0] | h[1] << 16, h[2] | h[3] << 16});
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < col_end) stg<uint16_t>(to + r * item, uint16_t(h[r]));
        }
      }
      acc0 = acc1 = V4F{0.0f, 0.0f, 0.0f, 0.0f};
    }
  };
  // (every wave of the workgroup runs the same number of items: the barriers inside are met by all)
#pragma clang loop unroll(disable)
  for (uint32_t j = 0; j < items; j += 2) {  // (an odd count's last pass works on nothing: both sets of registers take turns on every path)
    work(std::integral_constant<int, 0>{}, j);
    work(std::integral_constant<int, 1>{}, j + 1);
  }
}

// The kernel above where it applies: 3 to 8 rows of at most 4096 values, k a multiple of 16 (checked by the caller).
// False: not this kernel's shape.
template <class T>
bool launch_rows_kernel(const Q8Params& p, bool whatever_the_size, const Machine& mc, hipStream_t stream) {
  // (rows of A as a whole in LDS: 8 x 4096 values at most; 16-byte pieces)
  if (p.m < 3 || p.m > 8 || p.k < 512 || p.k > 4096 || p.n < 16) return false;
  // Measured against the slice kernels below (8 rows, microseconds, this kernel first).  It pays with rows shorter
  // than 4096 values, of which a slice kernel's waves get one chunk each, where a workgroup has 8 groups or more:
  //   K x N 1024 x 131072: 28.4 / 31.3, 2048 x 32768: 16.2 / 17.3, 2048 x 50304: 24.5 / 26.9, 2048 x 65536: 26.5 / 31.8,
  //   2048 x 128256: 47.6 / 58.3, 3072 x 32768: 21.0 / 22.2, 3072 x 65536: 37.2 / 40.6;
  // not with K = 4096 (4096 x 14336: 15.3 / 14.2, 4096 x 32000: 25.7 / 26.1, 4096 x 49152: 38.6 / 37.2, 4096 x 65536: 48.4 /
  // 48.4, 4096 x 128256: 88.4 / 89.9, at 4 rows 86.8 / 86.2) and not with few columns per compute unit.
  {
    const uint32_t cus0 = uint32_t(mc.compute_units), units = (p.n + 15) / 16 < cus0 ? (p.n + 15) / 16 : cus0;
    const bool pays = p.k < 4096 && (p.n + units - 1) / units >= 121;
    if (!whatever_the_size && !pays) return false;
  }
  // (32-bit byte offsets into B and A, each within a buffer descriptor of fewer than 2^31 bytes)
  if (uint64_t(p.n) * p.k >= (1ull << 31) || p.a_sm < int64_t(p.k) || (uint64_t(p.m - 1) * uint64_t(p.a_sm) + p.k) * 2 >= (1ull << 31)) return false;
  const uint32_t cus = uint32_t(mc.compute_units), groups = (p.n + 15) / 16;
  // columns per workgroup: the same for every compute unit, a multiple of 8; waves per group: as few as give most of
  // the workgroup's 8 waves a share of a group
  uint32_t grid = groups < cus ? groups : cus;
  const uint32_t cols_per_wg = ((p.n + grid - 1) / grid + 7) / 8 * 8;
  grid = (p.n + cols_per_wg - 1) / cols_per_wg;
  const uint32_t local = (cols_per_wg + 15) / 16;
  const int ks = local >= 5 ? 1 : local >= 3 ? 2 : local == 2 ? 4 : 8;
  const uint32_t lds = 8 * rows_a_pitch(p.k) + kRowsWaves * kRowsRegion + 2 * kRowsWaves * 64 * 16 + kRowsWaves * 32;
#define VKT_ROWS_CASE(KS_)                                                                                                   \
  if (ks == KS_) {                                                                                                           \
    auto kernel = qmm8_rows<T, KS_>;                                                                                         \
    static bool configured = false; /* guarded by the runtime's stream mutex */                                              \
    if (!configured) {                                                                                                       \
      if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 152 * 1024) != hipSuccess) { \
        (void)hipGetLastError();                                                                                             \
        return false;                                                                                                        \
      }                                                                                                                      \
      configured = true;                                                                                                     \
    }                                                                                                                        \
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(512), lds, stream, p, cols_per_wg);                                          \
    return true;                                                                                                             \
  }
  VKT_ROWS_CASE(1) VKT_ROWS_CASE(2) VKT_ROWS_CASE(4) VKT_ROWS_CASE(8)
#undef VKT_ROWS_CASE
  return false;
}

// 33 to a few hundred rows (batched decode): a tile kernel.  A workgroup of 8 waves owns 64 rows x 128 columns and a
// slice of K, walked in steps of 128 values.  Both operand tiles of a step are loaded into registers four steps
// ahead and written to one of two LDS stages a step before they are multiplied: the activations [64 rows][256 bytes]
// once per workgroup, the raw int8 weights [128 rows][128 bytes] in runs of 128 contiguous bytes per row.  16-byte
// chunks are swizzled by the row's low bits (the lane fetches the chunk that belongs in its slot), so that the
// operand-shaped reads (16 lanes = 16 rows at one logical chunk) are conflict free.  The waves split the step's K,
// not only its columns: wave (kc, nh) multiplies all 64 rows by columns 64 nh .. + 63 over the 32 values 32 kc .. + 31
// of each step, so a step costs the LDS 48 KB of fragment reads (every wave reading its own 32 x 32 outputs'
// operands: 96 KB) and every weight is widened once per workgroup.  After the loop the four k-parts of a column half
// meet through LDS, added in a fixed order.  K is cut into slices across workgroups until the grid fills the machine;
// the slices' float32 tiles meet in the runtime's workspace and qmm8_tile_finish adds them in slice order, scales
// and stores.
constexpr uint32_t kTileStepK = 128, kTileAhead = 4;
constexpr uint32_t kTileLds = 8 * 16 * 1024;  // the k-parts' meeting place; the two operand stages use its first half (float32 activations: all of it)
constexpr int vmcnt_only(int n) { return 0x0f70 | (n & 15) | ((n >> 4) << 14); }  // s_waitcnt vmcnt(n), nothing else

// Eight float32 values as three bfloat16 operands whose sum they are, exactly: the upper 16 bits of the value, of what
// that leaves, and of what that leaves (8 + 8 + 8 significant bits; every subtraction is exact).  Infinities and NaNs
// stay in the first part alone.
__device__ __forceinline__ void split_f32x8(const U4& x0, const U4& x1, U4* hi, U4* mid, U4* lo) {
  uint32_t h[8], m[8], l[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const uint32_t bits = i < 4 ? x0[i] : x1[i - 4];
    const bool special = (bits & 0x7f800000u) == 0x7f800000u;
    h[i] = (special && (bits & 0x007fffffu) ? bits | 0x00400000u : bits) & 0xffff0000u;
    const float r1 = special ? 0.0f : __builtin_bit_cast(float, bits) - __builtin_bit_cast(float, h[i]);
    m[i] = f32_bits(r1) & 0xffff0000u;
    const float r2 = r1 - __builtin_bit_cast(float, m[i]);
    l[i] = f32_bits(r2) & 0xffff0000u;
  }
  auto pack = [](const uint32_t (&v)[8]) {
    return U4{v[0] >> 16 | v[1], v[2] >> 16 | v[3], v[4] >> 16 | v[5], v[6] >> 16 | v[7]};
  };
  *hi = pack(h), *mid = pack(m), *lo = pack(l);
}

bool workspace_refused(const Machine& mc, uint64_t need, std::string* err);

// float32 activation rows [m][k] (rows a_sm values apart) as three bfloat16 planes [3][m][k]: a thread per 8 values.
__global__ __launch_bounds__(256) void qmm8_split_rows(Q8Params p, uint64_t planes) {
  const uint32_t per_row = p.k / 8, id = blockIdx.x * 256 + threadIdx.x;  // (k is a multiple of 16)
  if (id >= p.m * per_row) return;
  const uint32_t m = id / per_row, piece = id % per_row;
  const uint64_t src = p.a + uint64_t(int64_t(m) * p.a_sm * 4) + piece * 32ull;
  const U4 x0 = ldg<U4>(src), x1 = ldg<U4>(src + 16);
  U4 part[3];
  split_f32x8(x0, x1, &part[0], &part[1], &part[2]);
  const uint64_t plane = uint64_t(p.m) * p.k * 2;
#pragma unroll
  for (int q = 0; q < 3; ++q) stg<U4>(planes + q * plane + (uint64_t(m) * p.k + piece * 8ull) * 2, part[q]);
}

// 2 to 16 rows of float32 activations on the matrix cores: the rows are split into their three bfloat16 planes by a
// launch of its own (into the workspace), and the staged kernel multiplies every weight fragment by the planes'
// fragments.  Columns per workgroup as for 16-bit activations, with three times their activation bytes.  Returns the
// estimated microseconds of both launches in *estimate_us when stream is null (nothing is launched then); false
// where the path does not apply.
inline bool launch_split_staged(const Q8Params& p0, const Machine& mc, hipStream_t stream, bool launch, float* estimate_us, std::string* err, int* rc) {
  *rc = 0;
  if (p0.m < 2 || p0.m > 16 || p0.k < 1024 || p0.n < 64 || uint64_t(p0.m) * p0.k >= (1ull << 28)) return false;
  const uint64_t planes_bytes = (3ull * p0.m * p0.k * 2 + 255) / 256 * 256;
  const uint32_t cus = uint32_t(mc.compute_units);
  int nt = 1;
  uint32_t slices = 1;
  float best = 1e30f;
  // few columns against long rows: 32 columns per workgroup and K in slices over workgroups, as for 16-bit rows (the
  // slices' tiles lie behind the planes in the workspace); 8 rows, K = 8192, N = 1024: 18.5 us on the one-row kernels
  if (p0.k >= 4096 && (p0.n + 31) / 32 * 4 <= cus) {
    const uint32_t groups = (p0.n + 31) / 32, chunks = (p0.k + 255) / 256;
    while (groups * slices * 2 <= cus && chunks / (slices * 2) >= 2) slices *= 2;
    if (slices > 1 && chunks / (slices * 2) >= 14) slices *= 2;
    if (slices > 1) nt = 2, best = float(32 + 6 * p0.m) * float(p0.k) / float(slices) / 30e3f + 2.5f;  // (a third launch)
  }
  if (slices == 1) {
    for (int t = 1; t <= 4; t *= 2) {
      const uint32_t cols = staged_cols(p0.n, t, cus), workgroups = (p0.n + cols - 1) / cols;
      const float cost = float((workgroups + cus - 1) / cus) * float(cols + 6 * p0.m) * float(p0.k) / 30e3f * (t == 4 && workgroups <= cus ? 1.25f : 1.0f);
      if (cost < best) best = cost, nt = t;
    }
  }
  *estimate_us = best + 6.5f;  // (what two launches in a row cost before their bytes: K = N = 1024 takes 6.3-8.1 us)
  const uint64_t need = planes_bytes + (slices > 1 ? uint64_t((p0.n + 31) / 32) * slices * 2 * 1024 : 0);
  if (!launch) return need <= mc.workspace_bytes || mc.workspace_fixed;
  if (workspace_refused(mc, need, err)) {
    *rc = -1;
    return true;
  }
  if (need > mc.workspace_bytes) return false;
  const uint32_t threads = p0.m * (p0.k / 8);
  hipLaunchKernelGGL(qmm8_split_rows, dim3((threads + 255) / 256), dim3(256), 0, stream, p0, mc.workspace);
  Q8Params p = p0;
  p.a = mc.workspace, p.a_sm = p0.k;
  Machine tiles = mc;  // (the slices' tiles: behind the planes)
  tiles.workspace = mc.workspace + planes_bytes, tiles.workspace_bytes = mc.workspace_bytes - planes_bytes;
  const int waves = nt < 4 && p0.k >= 16 * 256 ? 8 : 4;
  bool ok = false;
  if (nt == 1) ok = waves == 8 ? launch_staged_one<f32_t, 1, 1, 8, 3>(p, 1, mc, stream) : launch_staged_one<f32_t, 1, 1, 4, 3>(p, 1, mc, stream);
  else if (nt == 2) ok = waves == 8 ? launch_staged_one<f32_t, 1, 2, 8, 3>(p, slices, tiles, stream) : launch_staged_one<f32_t, 1, 2, 4, 3>(p, 1, mc, stream);
  else ok = launch_staged_one<f32_t, 1, 4, 4, 3>(p, 1, mc, stream);
  if (!ok) {
    *err = "qmm8: cannot reserve LDS for the staged kernel";
    *rc = -1;
  }
  return true;
}

template <class T>
__global__ __launch_bounds__(512) void qmm8_tile(Q8Params p, uint32_t steps_per_slice, uint64_t workspace) {
  // float32 activations: split into three bfloat16 parts when they are written to LDS (three planes of the 16-bit
  // layout), and every weight fragment multiplies the three planes' fragments one after the other, so the product is
  // that of the float32 values, added up in float32 (the matrix core's products of bfloat16 values are exact)
  constexpr bool F32 = T::dtype == VKT_F32;
  constexpr int PLANES = F32 ? 3 : 1, A_LOADS = F32 ? 2 : 1;
  constexpr uint32_t PLANE = 64 * 256, A_BYTES = PLANES * PLANE, B_BYTES = 128 * 128, STAGE = A_BYTES + B_BYTES;
  constexpr uint32_t ITEM = F32 ? 4 : 2, OUT_ITEM = ITEM;
  constexpr int PER_STEP = 2 * A_LOADS + 2;  // loads per lane and step
  // steps in flight from memory (even: a step's parity names its register sets).  float32 activations: two, whose
  // steps take three times as long and whose loads are half as many again (four would not fit the registers: 80
  // bytes per lane went to scratch memory)
  constexpr int AHEAD = F32 ? 2 : int(kTileAhead);
  static_assert(2 * STAGE <= kTileLds, "two stages");
  extern __shared__ __attribute__((aligned(16))) uint8_t tile_lds[];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, c = lane & 15, g = lane >> 4;
  const int kc = wave & 3, nh = wave >> 2;
  const uint32_t n0 = blockIdx.x * 128, m0 = blockIdx.y * 64, slice = blockIdx.z;
  const uint32_t steps = p.k / kTileStepK;
  const uint32_t s_begin = slice * steps_per_slice, s_end = s_begin + steps_per_slice < steps ? s_begin + steps_per_slice : steps;

  // Loads of one step: activations 16 wave-loads of 4 rows x 128 values (8 values per lane), weights 16 of 8 rows x 128
  // bytes; a wave issues 2 + 2 (float32: 4 + 2), into registers, kTileAhead steps ahead, and writes them to LDS (16
  // bytes per lane and plane, lane after lane) one step before they are multiplied.  (Straight into LDS with
  // global_load_lds_dwordx4 the same stream runs at 2.6 TB/s from 112 compute units where this path gives 4.1-4.4:
  // measured with the loads alone.)
  uint64_t a_src[2], b_src[2];
  uint32_t a_dst[2], b_dst[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t row = (wave * 2 + i) * 4 + (lane >> 4), slot = lane & 15u;
    const uint32_t m = m0 + row < p.m ? m0 + row : p.m - 1;
    a_src[i] = p.a + uint64_t(int64_t(m) * p.a_sm * int64_t(ITEM)) + ((slot ^ (row & 15u)) * 8 * ITEM);
    a_dst[i] = (wave * 2 + i) * 1024 + lane * 16;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const uint32_t row = (wave * 2 + i) * 8 + (lane >> 3), slot = lane & 7u;
    const uint32_t n = n0 + row < p.n ? n0 + row : p.n - 1;
    b_src[i] = p.b + uint64_t(n) * p.k + ((slot ^ ((row >> 1) & 7u)) * 16);
    b_dst[i] = A_BYTES + (wave * 2 + i) * 1024 + lane * 16;
  }
  U4 ra[AHEAD][2][A_LOADS], rb[AHEAD][2];
  auto request = [&](auto set, uint32_t step) {
    constexpr int R = decltype(set)::value;
    const uint32_t st = step < s_end ? step : s_end - 1;  // (past the end the last step again, never published: the count of loads in flight stays the same)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int h = 0; h < A_LOADS; ++h) ra[R][i][h] = ldg<U4>(a_src[i] + uint64_t(st) * kTileStepK * ITEM + 16 * h);
#pragma unroll
    for (int i = 0; i < 2; ++i) rb[R][i] = ldg_stream<U4>(b_src[i] + uint64_t(st) * kTileStepK);
  };
  auto publish = [&](auto set, uint32_t step) {
    constexpr int R = decltype(set)::value;
    uint8_t* base = tile_lds + ((step - s_begin) & 1u) * STAGE;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if constexpr (F32) {
        U4 part[3];
        split_f32x8(ra[R][i][0], ra[R][i][A_LOADS - 1], &part[0], &part[1], &part[2]);
#pragma unroll
        for (int q = 0; q < 3; ++q) *reinterpret_cast<U4*>(base + q * PLANE + a_dst[i]) = part[q];
      } else {
        *reinterpret_cast<U4*>(base + a_dst[i]) = ra[R][i][0];
      }
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<U4*>(base + b_dst[i]) = rb[R][i];
  };

  V4F acc[4][4];  // [row tile][column tile of this half]
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int t = 0; t < 4; ++t) acc[mt][t] = V4F{0.0f, 0.0f, 0.0f, 0.0f};

  // Fragments of step s + 1 are read from LDS (8 reads per lane, into the other of two register sets) while step s is
  // widened and multiplied, so the LDS, the vector units and the matrix cores work at the same time; three further
  // steps are in flight from memory.  Loads land in the order issued: "at most three steps' worth outstanding" means
  // everything older has landed.
  // lane (c, g): activations of row 16 mt + c, weights of column 64 nh + 16 t + c, both at k = 32 kc + 8 g .. + 7
  U4 fa[2][4];
  U2 fw[2][4];
  uint32_t a_off[4], w_off[4];
#pragma unroll
  for (int mt = 0; mt < 4; ++mt) {
    const uint32_t row = 16 * mt + c;
    a_off[mt] = row * 256 + (((4 * kc + g) ^ (row & 15u)) * 16);
  }
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const uint32_t row = 64 * nh + 16 * t + c;
    w_off[t] = row * 128 + (((2 * kc + (g >> 1)) ^ ((row >> 1) & 7u)) * 16) + 8 * (g & 1);
  }
  auto read_weights = [&](auto set, uint32_t step) {
    constexpr int S = decltype(set)::value;
    const uint8_t* tb = tile_lds + ((step - s_begin) & 1u) * STAGE + A_BYTES;
#pragma unroll
    for (int t = 0; t < 4; ++t) fw[S][t] = *reinterpret_cast<const U2*>(tb + w_off[t]);
  };
  auto read_activations = [&](auto set, uint32_t step, uint32_t plane) {
    constexpr int S = decltype(set)::value;
    const uint8_t* ta = tile_lds + ((step - s_begin) & 1u) * STAGE + plane * PLANE;
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) fa[S][mt] = *reinterpret_cast<const U4*>(ta + a_off[mt]);
  };
  auto multiply = [&](auto aset, auto wset) {
    constexpr int S = decltype(aset)::value, W = decltype(wset)::value;
#pragma unroll
    for (int t = 0; t < 4; t += 2) {
      U4 w0, w1;
      widen16_to_operands<T>(U4{fw[W][t][0], fw[W][t][1], fw[W][t + 1][0], fw[W][t + 1][1]}, &w0, &w1);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[mt][t] = mfma16<T>(w0, fa[S][mt], acc[mt][t]);
#pragma unroll
      for (int mt = 0; mt < 4; ++mt) acc[mt][t + 1] = mfma16<T>(w1, fa[S][mt], acc[mt][t + 1]);
    }
  };
  // J = (step - s_begin) % AHEAD.  The weights' register set is the step's parity; the activations' set changes
  // with every plane: sub-step (step, plane) uses set (PLANES * J + plane) % 2.
  auto iteration = [&](auto index, auto guarded, uint32_t step) {
    constexpr int J = decltype(index)::value, NEXT = (J + 1) % AHEAD;
    constexpr bool GUARDED = decltype(guarded)::value;  // the last steps of the slice: step + 1 may be past the end
    // the registers of step + 1 have landed; they go to the stage that step - 1 was read from, and the register set
    // takes the loads of step + 1 + AHEAD.  16-bit activations: every wave's reads of that stage had returned
    // before it passed the last barrier.  float32: a wave reads planes 1 and 2 of a step during the step itself, so
    // a barrier of its own comes first.
    if constexpr (F32) __syncthreads();
    __builtin_amdgcn_s_waitcnt(vmcnt_only((AHEAD - 1) * PER_STEP));
    if (!GUARDED || step + 1 < s_end) publish(std::integral_constant<int, NEXT>{}, step + 1);
    request(std::integral_constant<int, NEXT>{}, step + 1 + AHEAD);
    __syncthreads();
#pragma unroll
    for (int plane = 0; plane < PLANES; ++plane) {
      const int set = (PLANES * J + plane) & 1;
      // the fragments of the next sub-step: the next plane of this step, or plane 0 (and the weights) of step + 1
      if (plane + 1 < PLANES) {
        if (set) read_activations(std::integral_constant<int, 0>{}, step, plane + 1);
        else read_activations(std::integral_constant<int, 1>{}, step, plane + 1);
      } else if (!GUARDED || step + 1 < s_end) {
        if (set) read_activations(std::integral_constant<int, 0>{}, step + 1, 0);
        else read_activations(std::integral_constant<int, 1>{}, step + 1, 0);
        read_weights(std::integral_constant<int, (J + 1) & 1>{}, step + 1);
      }
      __builtin_amdgcn_sched_barrier(0);  // (the scheduler would move each read down to its first use)
      if (set) multiply(std::integral_constant<int, 1>{}, std::integral_constant<int, J & 1>{});
      else multiply(std::integral_constant<int, 0>{}, std::integral_constant<int, J & 1>{});
    }
  };
  request(std::integral_constant<int, 0>{}, s_begin);
  request(std::integral_constant<int, 1>{}, s_begin + 1);
  if constexpr (AHEAD == 4) {
    request(std::integral_constant<int, 2>{}, s_begin + 2);
    request(std::integral_constant<int, 3>{}, s_begin + 3);
  }
  __builtin_amdgcn_s_waitcnt(vmcnt_only((AHEAD - 1) * PER_STEP));  // the first of the steps in flight has landed
  publish(std::integral_constant<int, 0>{}, s_begin);
  request(std::integral_constant<int, 0>{}, s_begin + AHEAD);
  __syncthreads();
  read_activations(std::integral_constant<int, 0>{}, s_begin, 0);
  read_weights(std::integral_constant<int, 0>{}, s_begin);
  // groups of four steps with a step after them: straight-line code; then the last one to four steps
  uint32_t step = s_begin;
  constexpr std::false_type plain{};
  constexpr std::true_type guarded{};
  for (; step + AHEAD < s_end; step += AHEAD) {
    iteration(std::integral_constant<int, 0>{}, plain, step);
    iteration(std::integral_constant<int, 1>{}, plain, step + 1);
    if constexpr (AHEAD == 4) {
      iteration(std::integral_constant<int, 2>{}, plain, step + 2);
      iteration(std::integral_constant<int, 3>{}, plain, step + 3);
    }
  }
  iteration(std::integral_constant<int, 0>{}, guarded, step);
  if (step + 1 < s_end) iteration(std::integral_constant<int, 1>{}, guarded, step + 1);
  if constexpr (AHEAD == 4) {
    if (step + 2 < s_end) iteration(std::integral_constant<int, 2>{}, guarded, step + 2);
    if (step + 3 < s_end) iteration(std::integral_constant<int, 3>{}, guarded, step + 3);
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // (the re-reads of the last step, requested past the end)

  // The four k-parts of a column half meet through LDS (8 waves x 16 tiles x 1 KiB = 128 KiB): wave
  // (kc, nh) adds up row tile kc, its own part and the three others in the order of kc.
  __syncthreads();  // (every wave is done reading fragments: the stages are free)
  V4F* const parts = reinterpret_cast<V4F*>(tile_lds);
#pragma unroll
  for (int mt = 0; mt < 4; ++mt)
#pragma unroll
    for (int t = 0; t < 4; ++t) parts[(wave * 16 + mt * 4 + t) * 64 + lane] = acc[mt][t];
  __syncthreads();
  V4F sum[4];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    sum[t] = parts[((nh * 4 + 0) * 16 + kc * 4 + t) * 64 + lane];
#pragma unroll
    for (int q = 1; q < 4; ++q) {
      const V4F v = parts[((nh * 4 + q) * 16 + kc * 4 + t) * 64 + lane];
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[t][r] += v[r];
    }
  }

  // lane (c, g) holds, per column tile t, row 16 kc + c, columns 64 nh + 16 t + 4 g .. + 3.
  // (Letting the last workgroup to arrive at a tile add the slices up inside this kernel, instead of a second launch,
  // was tried: the slices then have to cross between the dies' L2s, and both device-scope fences and write-through
  // stores with device-scope loads made the kernel 1.5-3x slower.)
  const bool sliced = gridDim.z > 1;
  const uint32_t m = m0 + 16 * kc + c;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const uint32_t n = n0 + 64 * nh + 16 * t + 4 * g;
    if (m >= p.m || n >= p.n) continue;
    if (sliced) {
      float* out = reinterpret_cast<float*>(workspace) + (uint64_t(slice) * p.m + m) * p.n + n;
      if ((p.n & 3u) == 0) *reinterpret_cast<V4F*>(out) = sum[t];
      else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n + r < p.n) out[r] = sum[t][r];
      }
    } else {
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) v[r] = sum[t][r] * load_f32<T>(p.scales + uint64_t(n + r < p.n ? n + r : p.n - 1) * ITEM);
      const uint64_t at = p.c + (uint64_t(m) * p.n + n) * OUT_ITEM;
      if constexpr (F32) {
        if ((p.n & 3u) == 0 && (p.c & 15u) == 0) stg<F4>(at, F4{v[0], v[1], v[2], v[3]});
        else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < p.n) stg<float>(at + 4 * r, v[r]);
        }
      } else {
        uint32_t h[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) h[r] = T::dtype == VKT_BF16 ? f32_to_bf16(v[r]) : f32_to_f16(v[r]);
        if ((p.n & 3u) == 0 && (p.c & 7u) == 0) stg<U2>(at, U2{h[0] | h[1] << 16, h[2] | h[3] << 16});
        else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < p.n) stg<uint16_t>(at + 2 * r, uint16_t(h[r]));
        }
      }
    }
  }
}

// The slices of qmm8_tile added in slice order, scaled and stored: one thread per 4 consecutive outputs (n a multiple
// of 4) or per output.
template <class T>
__global__ __launch_bounds__(256) void qmm8_tile_finish(Q8Params p, uint32_t slices, uint64_t workspace, uint32_t vec) {
  const uint64_t total = uint64_t(p.m) * p.n, per = vec ? 4 : 1, i = (uint64_t(blockIdx.x) * 256 + threadIdx.x) * per;
  if (i >= total) return;
  const float* part = reinterpret_cast<const float*>(workspace);
  float v[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  if (vec) {
    // eight slices' loads are in flight together; the additions keep the slice order
    for (uint32_t s0 = 0; s0 < slices; s0 += 8) {
      V4F t[8];
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u)
        if (s0 + u < slices) t[u] = *reinterpret_cast<const V4F*>(part + uint64_t(s0 + u) * total + i);
#pragma unroll
      for (uint32_t u = 0; u < 8; ++u)
        if (s0 + u < slices) {
#pragma unroll
          for (int r = 0; r < 4; ++r) v[r] = s0 + u == 0 ? t[u][r] : v[r] + t[u][r];
        }
    }
  } else {
    for (uint32_t s = 0; s < slices; ++s) {
      const float t = part[uint64_t(s) * total + i];
      v[0] = s == 0 ? t : v[0] + t;
    }
  }
  const uint32_t n = uint32_t(i % p.n);
  constexpr uint32_t ITEM = T::dtype == VKT_F32 ? 4 : 2;
  float y[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) y[r] = v[r] * load_f32<T>(p.scales + uint64_t(n + r < p.n ? n + r : p.n - 1) * ITEM);
  if constexpr (T::dtype == VKT_F32) {
    if (vec && (p.c & 15u) == 0) stg<F4>(p.c + i * 4, F4{y[0], y[1], y[2], y[3]});
    else {
      for (uint32_t r = 0; r < per; ++r) stg<float>(p.c + (i + r) * 4, y[r]);
    }
  } else {
    uint32_t h[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) h[r] = T::dtype == VKT_BF16 ? f32_to_bf16(y[r]) : f32_to_f16(y[r]);
    if (vec && (p.c & 7u) == 0) stg<U2>(p.c + i * 2, U2{h[0] | h[1] << 16, h[2] | h[3] << 16});
    else {
      for (uint32_t r = 0; r < per; ++r) stg<uint16_t>(p.c + (i + r) * 2, uint16_t(h[r]));
    }
  }
}

// A product whose planned split over workgroups needs `need` bytes of workspace, on a machine whose workspace
// cannot be traded for another plan: an error that names both sizes.
bool workspace_refused(const Machine& mc, uint64_t need, std::string* err) {
  if (!mc.workspace_fixed || need <= mc.workspace_bytes) return false;
  *err = "qmm8: this product's partial sums need " + std::to_string(need) + " bytes of workspace, the fixed workspace holds " +
         std::to_string(mc.workspace_bytes);
  return true;
}

// The tile kernel's count of K-slices with the shortest estimated launch (4 steps per slice at least), and that
// estimate in microseconds, from what was measured at 64 rows: every round of workgroups over the machine takes 3
// (until its first operands are in LDS) + 0.72 per step (three times that with float32 activations, whose planes are
// multiplied one after the other); more than one slice costs the second launch, 4.5, and its partial tiles written
// and read back at 5 TB/s.  (Rounding tiles x slices to the nearest count of compute units, the rule before, gave
// N = 11008 three slices: 258 workgroups on 256 units, two rounds of 11 steps, 31.2-32.6 us; two slices, one round
// of 16 steps: 22.6-22.9.)
template <class T>
float tile_estimate_us(const Q8Params& p, const Machine& mc, uint32_t* slices) {
  const uint32_t gx = (p.n + 127) / 128, gy = (p.m + 63) / 64, steps = p.k / kTileStepK;
  const uint32_t cus = uint32_t(mc.compute_units), most = steps / 4 ? steps / 4 : 1;
  const float step_us = T::dtype == VKT_F32 ? 2.2f : 0.72f, partial_us = float(p.m) * float(p.n) * 8.0f / 5e6f;
  float best = 1e30f;
  *slices = 1;
  for (uint32_t s = 1; s <= most && s <= 64; ++s) {
    const uint32_t rounds = (gx * gy * s + cus - 1) / cus;
    const float cost = float(rounds) * (3.0f + step_us * float((steps + s - 1) / s)) + (s > 1 ? 4.5f + partial_us * float(s) : 0.0f);
    if (cost < best) best = cost, *slices = s;
  }
  return best;
}

// Launches the tile kernel if it takes the product (k a multiple of its step, 16-byte aligned activation rows):
// 1 launched, 0 not this kernel's shape, -1 refused (*err set).
template <class T>
int launch_tile_kernel(const Q8Params& p, uint32_t want_slices, const Machine& mc, hipStream_t stream, std::string* err) {
  if (p.k % kTileStepK != 0 || p.k == 0 || (int64_t(p.a_sm) * int64_t(sizeof(typename T::storage))) % 16 != 0 || p.a_sm <= 0) return 0;
  constexpr uint32_t lds = kTileLds;
  auto kernel = qmm8_tile<T>;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) != hipSuccess) {
      (void)hipGetLastError();
      return 0;
    }
    configured = true;
  }
  const uint32_t gx = (p.n + 127) / 128, gy = (p.m + 63) / 64, steps = p.k / kTileStepK;
  uint32_t slices = want_slices;
  if (slices == 0) tile_estimate_us<T>(p, mc, &slices);
  if (slices > 1 && workspace_refused(mc, uint64_t(slices) * p.m * p.n * 4, err)) return -1;
  while (slices > 1 && uint64_t(slices) * p.m * p.n * 4 > mc.workspace_bytes) --slices;
  uint32_t per_slice = (steps + slices - 1) / slices;
  slices = (steps + per_slice - 1) / per_slice;
  if (gy > 65535 || slices > 65535) return 0;
  hipLaunchKernelGGL(kernel, dim3(gx, gy, slices), dim3(512), lds, stream, p, per_slice, mc.workspace);
  if (slices > 1) {
    const uint32_t vec = (p.n & 3u) == 0;
    const uint64_t threads = (uint64_t(p.m) * p.n + (vec ? 3 : 0)) / (vec ? 4 : 1);
    hipLaunchKernelGGL(qmm8_tile_finish<T>, dim3(uint32_t((threads + 255) / 256)), dim3(256), 0, stream, p, slices, mc.workspace, vec);
  }
  return 1;
}

// Rows (<= 64) of 16-bit activations on the matrix cores.  A workgroup takes 64 columns
// where there are that many, so that an activation fragment is reused over 4 weight
// fragments (every workgroup reads all the activations of its slice of K from L2: with 16
// columns per workgroup that traffic is several times the weight stream once M reaches 64),
// and K is cut into slices across workgroups until the grid covers the machine about
// twice.  variant = NT | WAVES << 8 | SLICES << 24 overrides the plan (tuning, tests).
struct MfmaPlan {
  bool staged;
  int nt, waves;
  uint32_t slices;
  float estimate_us;  // of the launch, for 9 to 32 rows (0: none made)
};

inline MfmaPlan plan_mfma(const Q8Params& p, uint32_t variant, const Machine& mc) {
  int nt = p.n >= 64 ? 4 : 1, waves = p.m > 32 ? 4 : 8;  // (measured: K = 4096 and 14336, N = 14336 and 4096)
  uint32_t slices = 1;
  float estimate = 0.0f;
  if (variant & 0xffff) {
    nt = variant & 0xff;
    waves = (variant >> 8) & 0xff;
    slices = (variant >> 24) ? (variant >> 24) : 1;
  } else {
    const uint32_t groups = (p.n + 16 * nt - 1) / (16 * nt), chunks = (p.k + 63) / 64;
    while (waves > 4 && chunks < uint32_t(waves)) waves /= 2;
    // The count of slices that leaves the busiest compute unit the least work: (workgroups on it) x (a slice's share
    // of K), plus a little per slice for its partial tile; at least 2 chunks per wave.  (Rounding groups x slices to
    // the nearest count of compute units, the rule before, gave N = 6400 three slices, 300 workgroups on 256 units;
    // five make 500, two for nearly every unit: 38.9 -> 29.5 us at 16 rows, K = 14336.)
    const uint32_t cus = uint32_t(mc.compute_units), most = chunks / (2u * waves) ? chunks / (2u * waves) : 1;
    float best = 1e30f;
    for (uint32_t s = 1; s <= most && s <= 16; ++s) {
      const float cost = float((groups * s + cus - 1) / cus) / float(s) + 0.005f * float(s);
      if (cost < best) best = cost, slices = s;
    }
  }
  // Few columns against long rows (N = 1024 or 2048, the key / value projections of a model with grouped heads; rows
  // of 4096 values and more): the staged kernel with 32 columns per workgroup and K in slices over workgroups, a power
  // of two that brings them up to one per compute unit while a slice keeps two chunks of 256 values (up to 16 rows:
  // twice that where slices stay 14 chunks long), their tiles added up by a second launch.  Read off every (columns,
  // slices) of 14 shapes x 3 row counts; us before / after at 8 rows: K = 28672, N = 1024: 23.5 / 11.5; K = 16384, N =
  // 512: 14.8 / 7.9; K = 8192, N = 2048: 10.5 / 8.8; at 32 rows, K = 4096, N = 1024: 11.9 / 8.1.  From N = 4096 on the
  // slices gain nothing (the activations are two bytes a value here, and every workgroup re-reads its slice of them).
  // (17 to 32 rows: up to N = 1024; at 2048 the unsliced plan is level, 11.3 against 11.8 us)
  if (!(variant & 0xffff) && !((variant >> 19) & 1) && p.m <= 32 && p.k >= 4096 && p.n >= 64 &&
      (p.n + 31) / 32 * (p.m <= 16 ? 4 : 8) <= uint32_t(mc.compute_units)) {
    const uint32_t cus = uint32_t(mc.compute_units), groups = (p.n + 31) / 32, chunks = (p.k + 255) / 256;
    uint32_t s = 1;
    while (groups * s * 2 <= cus && chunks / (s * 2) >= 2) s *= 2;
    if (p.m <= 16 && s > 1 && chunks / (s * 2) >= 14) s *= 2;
    if (s > 1) return MfmaPlan{true, 2, 8, s, 0.0f};  // (no estimate: the tile kernel is not weighed against it; K = 28672, N = 1024 at 32 rows: 16.9 against 18.1 us)
  }
  // Up to 8 rows the kernel that stages the weights through LDS wins (measured at K = 4096 / N = 14336 and the
  // reverse: 15.8 against 17.1 us, 15.1-16.4 against 17.3-18.4); from 16 rows on the activations' own traffic
  // levels the two.  variant bit 18 asks for it explicitly, bit 19 for the plain kernel.
  bool staged = (variant >> 18) & 1;
  if (!(variant & 0xffff) && !((variant >> 19) & 1) && p.m <= 8 && p.k >= 2048 && p.n >= 64) {
    staged = true;
    // 32 columns per workgroup where 16 would make two or more workgroups per compute unit, otherwise 16 (the launch
    // below then deals the columns out evenly, 28 or 20 per workgroup where 32 do not divide them over the machine).
    // Measured at 8 rows, microseconds with 16 / 32 columns (K x N): 5120 x 13824: 21.0 / 17.5, 6144 x 16384: 24.8 / 21.5,
    // 4096 x 14336: 19.6 / 14.3, 4096 x 28672: 34.6 / 25.0, 3072 x 9216: 12.0 / 10.3, 2048 x 8192: 7.1 / 6.7, 4096 x 8192:
    // 11.7 / 10.6, 8192 x 9216: 22.1 / 20.8, 14336 x 8192: 28.1 / 23.8, 8192 x 28672: 53.0 / 43.0, 14336 x 14336: 48.6 / 39.2,
    // 16384 x 16384: 59.8 / 54.0, 12288 x 32768: 83.4 / 72.6; and 4096 x 4096: 8.2 / 8.6, 14336 x 4096: 15.4 / 17.4,
    // 16384 x 4096: 19.5 / 21.4.  4 rows order the same way.  (8192 x 8192 read 18.4 / 20.4 until the workgroups' chunk
    // orders were rotated against each other: 17.9 / 15.6 since.)
    const uint32_t groups16 = (p.n + 15) / 16;
    nt = groups16 >= 2u * uint32_t(mc.compute_units) ? 2 : 1, waves = 8, slices = 1;
  } else if (!(variant & 0xffff) && !((variant >> 19) & 1) && p.m <= 32 && p.k >= 2048 && p.n >= 64) {
    // 9 to 32 rows.  Every workgroup reads all rows of the activations next to its own weights, and what a launch
    // lasts is what its busiest compute unit takes in: (workgroups on it) x (columns + 2 rows) x K bytes, at ~30 KB/us
    // with the weights staged, ~23 with the plain kernel (whose K-slices cost a second launch, ~4.5 us).  16, 32 or 64
    // columns per workgroup, whichever leaves the busiest unit least (64 as one workgroup per unit runs a quarter
    // slower than its bytes say).  Measured, us at 9 / 16 / 32 rows with this choice against the rule before it (64
    // columns for K <= 8192 and N >= 8192, else the plain kernel): K = N = 8192: 16.2 / 18.9 / 25.3 against 23.0 /
    // 23.9 / 29.2; K = N = 4096: 7.5 / 8.6 / 12.2 against 9.3 / 9.7 / 12.2; K = 4096, N = 14336: 14.3 / 16.8 / 21.1
    // against 16.3 / 16.9 / 21.1; K = 14336, N = 4096: 16.2 / 18.9 / 24.1 against 18.0 / 18.9 / 24.1.
    const uint32_t cus = uint32_t(mc.compute_units);
    const auto busiest = [&](uint32_t workgroups, uint32_t cols, uint32_t k_share) {
      return float((workgroups + cus - 1) / cus) * float(cols + 2 * p.m) * float(k_share);
    };
    const uint32_t plain_groups = (p.n + 16 * nt - 1) / (16 * nt);
    float best = busiest(plain_groups * slices, 16 * nt, (p.k + slices - 1) / slices) / 23e3f + (slices > 1 ? 4.5f : 0.0f);
    for (int t = 1; t <= 4; t *= 2) {
      const uint32_t cols = staged_cols(p.n, t, cus), workgroups = (p.n + cols - 1) / cols;
      const float cost = busiest(workgroups, cols, p.k) / 30e3f * (t == 4 && workgroups <= cus ? 1.25f : 1.0f);
      if (cost < best) best = cost, staged = true, nt = t;
    }
    if (staged) waves = nt < 4 && p.k >= 16 * 256 ? 8 : 4, slices = 1;
    estimate = best;
  }
  return MfmaPlan{staged, nt, waves, slices, estimate};
}

template <class T>
int launch_mfma(const Q8Params& p, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err) {
  const int mt = p.m <= 16 ? 1 : p.m <= 32 ? 2 : 4;
  const MfmaPlan plan = plan_mfma(p, variant, mc);
  const bool staged = plan.staged;
  const int nt = plan.nt, waves = plan.waves;
  uint32_t slices = plan.slices;
  if (staged) {  // chunks of 256 values of k
    const uint64_t sgroups = (p.n + 16 * nt - 1) / (16 * nt);
    const uint32_t schunks = (p.k + 255) / 256;
    if (slices > 1 && workspace_refused(mc, sgroups * slices * mt * nt * 1024, err)) return -1;
    while (slices > 1 && (sgroups * slices * mt * nt * 1024 > mc.workspace_bytes || (schunks + slices - 1) / slices * (slices - 1) >= schunks)) --slices;
    if (mt <= 2 && launch_staged<T>(p, mt, nt, waves, slices, mc, stream)) return 0;
  }
  // the workspace holds groups * slices tiles of MT * NT KiB
  const uint64_t groups = (p.n + 16 * nt - 1) / (16 * nt);
  if (slices > 1 && workspace_refused(mc, groups * slices * mt * nt * 1024, err)) return -1;
  while (slices > 1 && groups * slices * mt * nt * 1024 > mc.workspace_bytes) --slices;
  const uint32_t chunks = (p.k + 63) / 64;
  while (slices > 1 && (chunks + slices - 1) / slices * (slices - 1) >= chunks) --slices;  // no empty slice
#define VKT_MFMA_CASE(MT_, NT_)                                           \
  if (mt == MT_ && nt == NT_) {                                           \
    launch_mfma_waves<T, MT_, NT_>(p, waves, slices, mc, stream);         \
    return 0;                                                             \
  }
  VKT_MFMA_CASE(1, 1) VKT_MFMA_CASE(1, 2) VKT_MFMA_CASE(1, 4)
  VKT_MFMA_CASE(2, 1) VKT_MFMA_CASE(2, 2) VKT_MFMA_CASE(2, 4)
  VKT_MFMA_CASE(4, 1) VKT_MFMA_CASE(4, 2) VKT_MFMA_CASE(4, 4)
  VKT_MFMA_CASE(1, 8) VKT_MFMA_CASE(2, 8) VKT_MFMA_CASE(4, 8)
#undef VKT_MFMA_CASE
  launch_mfma_waves<T, 4, 1>(p, waves, slices, mc, stream);
  return 0;
}


template <class T, int ROWS, int COLS, int KSPLIT>
void launch_gemv(const Q8Params& p, hipStream_t stream) {
  constexpr int per_wg = COLS * (4 / KSPLIT);
  const uint32_t grid = (p.n + per_wg - 1) / per_wg;
  hipLaunchKernelGGL((qmm8_gemv<T, ROWS, COLS, KSPLIT>), dim3(grid), dim3(256), 0, stream, p);
}

template <class T, int ROWS, int COLS>
bool launch_gemv_ks(const Q8Params& p, int ksplit, hipStream_t stream) {
  switch (ksplit) {
    case 1: launch_gemv<T, ROWS, COLS, 1>(p, stream); return true;
    case 2: launch_gemv<T, ROWS, COLS, 2>(p, stream); return true;
    case 4: launch_gemv<T, ROWS, COLS, 4>(p, stream); return true;
  }
  return false;
}

template <class T, int ROWS, int CA, int CB>
bool launch_gemv_cols(const Q8Params& p, int cols, int ksplit, hipStream_t stream) {
  if (cols == CA) return launch_gemv_ks<T, ROWS, CA>(p, ksplit, stream);
  if (cols == CB) return launch_gemv_ks<T, ROWS, CB>(p, ksplit, stream);
  return false;
}

// Picks COLS and KSPLIT.  Measured on MI355X (M = 1, weights rotated through HBM): many
// small waves beat few large ones, because the whole weight stream is then in flight at
// once: 2 columns per wave and K split over the 4 waves of a workgroup while a wave still
// gets one full 1 KiB load per column; rows beyond 4 leave fewer registers per column.
void plan_gemv(const Q8Params& p, int rows, bool sixteen_bit, const Machine&, int* cols, int* ksplit) {
  *cols = rows <= 4 ? 2 : (p.n >= 8192 ? 2 : 1);
  *ksplit = p.k >= 4096 ? (p.k <= 8192 ? 4 : 2) : (p.k >= 2048 ? 2 : 1);
  // two rows of 16-bit activations (dot products on pairs): 4 columns per wave, K over the 4 waves (measured on the
  // Llama shapes: 14.0-14.2 us against 14.9-17.0)
  if (rows == 2 && sixteen_bit && p.k >= 4096 && p.n >= 4096) *cols = 4, *ksplit = 4;
}

template <class T>
int launch_qmm8_t(const Q8Params& p0, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err) {
  const size_t item = sizeof(typename T::storage);
  const bool vector_ok = p0.k % 16 == 0 && p0.a % 16 == 0 && p0.b % 16 == 0 &&
                         (p0.m == 1 || (int64_t(p0.a_sm) * int64_t(item)) % 16 == 0) && !((variant >> 16) & 1);
  if (!vector_ok) {
    const uint32_t gy = p0.m <= 8 ? 1 : (p0.m + 7) / 8 < 64 ? (p0.m + 7) / 8 : 64;
    hipLaunchKernelGGL((qmm8_generic<T>), dim3((p0.n + 3) / 4, gy), dim3(256), 0, stream, p0);
    return 0;
  }
  if constexpr (T::dtype != VKT_F32) {
    // many rows (prefill): one product on the tile kernel over weights widened into the runtime's scratch region
    // (variant bit 20 keeps the row-block kernels, for tests and tuning)
    const uint64_t need = q8_gemm_scratch_bytes(p0, T::dtype, mc);
    if (need != 0 && need <= mc.scratch_bytes && !((variant >> 20) & 1) && !(variant & 0xffff)) return launch_q8_gemm(p0, T::dtype, mc, stream, err);
    // more than 32 rows (batched decode): the tile kernel (variant bit 21 forces it with bits 24+ slices, bit 22 keeps it off).
    // 17 to 32 rows: where its estimated launch is the shorter one by 5 % or more (it multiplies 64 rows whatever the
    // count, but reads the activations once per 128 columns; measured at 24 rows, tile kernel / the others: K = 28672,
    // N = 4096: 31.1 / 38.5 us, 14336 x 4096: 21.1 / 23.2, 8192 x 8192: 22.1 / 23.2, 2048 x 32000: 19.2 / 20.9; 4096 x 14336:
    // 20.6 / 19.5, 4096 x 4096: 12.8 / 10.9 stay).
    bool tile = p0.m > 32;
    if (variant == 0 && p0.m > 16 && p0.m <= 32 && p0.k % kTileStepK == 0) {
      uint32_t unused;
      const MfmaPlan other = plan_mfma(p0, 0, mc);
      tile = other.estimate_us > 0.0f && tile_estimate_us<T>(p0, mc, &unused) < 0.95f * other.estimate_us;
    }
    if (((tile && !(variant & 0xffff)) || ((variant >> 21) & 1)) && !((variant >> 22) & 1) && !((variant >> 17) & 1) && !((variant >> 18) & 1) &&
        !((variant >> 19) & 1) && !((variant >> 20) & 1)) {
      const int rc = launch_tile_kernel<T>(p0, variant >> 24, mc, stream, err);
      if (rc != 0) return rc < 0 ? -1 : 0;
    }
    // From 3 rows on the matrix cores win: the GEMV kernels convert every weight and multiply it once per row on
    // the vector units (measured at K = 4096, N = 14336: 10.5, 16.4, 23.0, 23.4 us for 1 to 4 rows; the matrix
    // cores take 16 us for up to 8).  variant bit 17 forces the GEMV kernels (tests, tuning).
    // (two rows against 32 column groups and more per compute unit pair go there too: 3-6 % ahead of the vector units,
    //  K = 4096, N = 14336: 13.5 against 13.9 us, N = 128256: 86 against 92; with fewer columns 9 % behind.  Bit 18: the
    //  staged matrix-core kernel for one and two rows whatever the shape.)
    const bool two_rows = p0.m == 2 && variant == 0 && p0.k >= 2048 && (p0.n + 15) / 16 >= 2u * uint32_t(mc.compute_units);
    // (few columns: the matrix-core kernels give a workgroup 8 columns at least, the vector-unit kernels 1 or 2, and
    //  there the many small workgroups win although they multiply every weight once per row: K = 8192, N = 1024 at 3 / 4 /
    //  8 rows 5.8 / 5.9 / 8.6 us against 8.6 / 8.8 / 9.3; K = 4096, N = 2048 at 3 / 4: 5.4 against 6.3 / 6.4; N = 4096: 8.0
    //  against 7.0, the other way round)
    const uint32_t few = 8u * uint32_t(mc.compute_units);
    const bool few_columns = variant == 0 && ((p0.m <= 4 && p0.n <= few) || (p0.m <= 8 && 2 * p0.n <= few && p0.k <= 4096)) && (p0.m <= 2 || p0.k <= 8192);
    // (longer rows: the staged kernel with K in slices over workgroups: K = 8192, N = 1024 at 5 to 8 rows 7.5 against
    //  9.0 us; K = 28672, N = 1024 at 4 rows: 11.5 against 25.2)
    if ((p0.m > 2 || two_rows || ((variant >> 18) & 1)) && !few_columns && !((variant >> 17) & 1)) {
      // 3 to 8 short rows against many columns: the wave-per-column-group kernel where it pays (variant bit 23 keeps the kernels below)
      // (bits 8-15 with bits 0-7 clear ask for it whatever the size: tests, tuning)
      const bool asked = !(variant & 0xff) && ((variant >> 8) & 0xff);
      if ((asked || !(variant & 0xffff)) && !((variant >> 18) & 3) && !((variant >> 23) & 1) && launch_rows_kernel<T>(p0, asked, mc, stream)) return 0;
      for (uint32_t r0 = 0; r0 < p0.m; r0 += 64) {
        Q8Params p = p0;
        p.m = p0.m - r0 < 64 ? p0.m - r0 : 64;
        p.a = p0.a + uint64_t(int64_t(r0) * p0.a_sm * int64_t(item));
        p.c = p0.c + uint64_t(r0) * p0.n * item;
        if (launch_mfma<T>(p, variant, mc, stream, err) != 0) return -1;
      }
      return 0;
    }
  }
  if constexpr (T::dtype == VKT_F32) {
    // More than 16 rows of float32 activations: the tile kernel on the activations' three bfloat16 parts, one pass over
    // the weights per 64 rows.  3 to 16 rows: where its estimated launch is well below that of the one-row kernels
    // below, which multiply every weight once per row on the vector units (kernels of 4, 8 and 16 rows: ~2.5 us + rows
    // x weights / 3.8 MB/us) and read the weights once per 16 rows.  Measured, us at 3 / 4 / 8 / 16 rows, one-row
    // kernels against the tile kernel: K = N = 4096: 16.8 / 18.2 / 34.5 / 64.5 against 17.4-18.7; K = 4096, N = 14336:
    // 50.4 / 54.4 / 102 / 111 against 47; K = N = 8192: 63 / 69 / 124 / 126 against 49-50; K = N = 2048: 5.6 / 5.9 / 10.7 /
    // 18.8 against 15.2-15.4 (so only 16 rows move); K = N = 1024: 3.7 / 3.7 / 4.6 / 7.0 against 14.6-14.9 (none do).
    // variant bit 21 forces the tile kernel (bits 24+ slices), bit 22 keeps it off.
    // 2 to 16 rows: split into bfloat16 planes by a launch of its own and multiplied by the staged matrix-core kernel,
    // where the estimate of the two launches is the shortest of the three (variant bit 18 asks for that path, bit 19
    // keeps it off).
    bool tile = p0.m > 16;
    if ((variant == 0 || variant == (1u << 18) || variant == (1u << 19)) && p0.m >= 2 && p0.m <= 16) {
      uint32_t unused;
      const float rows = p0.m <= 2 ? 2.0f : p0.m <= 4 ? 4.0f : p0.m <= 8 ? 8.0f : 16.0f, one_row_us = 2.5f + rows * float(p0.n) * float(p0.k) / 3.8e6f;
      const float tile_us = p0.m >= 3 && p0.k % kTileStepK == 0 ? tile_estimate_us<T>(p0, mc, &unused) : 1e30f;
      float split_us = 1e30f;
      int rc = 0;
      const bool can_split = !((variant >> 19) & 1) && launch_split_staged(p0, mc, stream, false, &split_us, err, &rc);
      if (can_split && (((variant >> 18) & 1) || (split_us < 0.9f * one_row_us && split_us < tile_us))) {
        if (launch_split_staged(p0, mc, stream, true, &split_us, err, &rc)) return rc;
      }
      tile = variant != (1u << 18) && tile_us < 0.8f * one_row_us;
    }
    if (((tile && !(variant & 0xffff)) || ((variant >> 21) & 1)) && !((variant >> 22) & 1) && !((variant >> 17) & 1)) {
      const int rc = launch_tile_kernel<T>(p0, variant >> 24, mc, stream, err);
      if (rc != 0) return rc < 0 ? -1 : 0;
    }
  }
  // One row of float32 activations: the persistent streaming kernel (measured at K = N = 4096: 4.85 us against 5.8; a
  // workgroup of the other kernel reads 4 KiB of activations per 2 KiB of weights).  With 16-bit activations the two
  // are level at every shape tried (K = 4096 ... 14336, N = 4096 ... 14336) and the other one stays.  variant bit 23
  // keeps the other kernel; bits 8-15 (with bits 0-7 clear) ask for this one whatever the type (tests, tuning).
  if (p0.m == 1 && !(variant & 0xff) && !((variant >> 23) & 1) && !((variant >> 17) & 1) &&
      (T::dtype == VKT_F32 || ((variant >> 8) & 0xff)) && launch_stream<T>(p0, variant, mc, stream))
    return 0;
  for (uint32_t r0 = 0; r0 < p0.m; r0 += 16) {
    Q8Params p = p0;
    p.m = p0.m - r0 < 16 ? p0.m - r0 : 16;
    p.a = p0.a + uint64_t(int64_t(r0) * p0.a_sm * int64_t(item));
    p.c = p0.c + uint64_t(r0) * p0.n * item;
    const int rows = p.m <= 1 ? 1 : p.m <= 2 ? 2 : p.m <= 4 ? 4 : p.m <= 8 ? 8 : 16;
    int cols, ksplit;
    plan_gemv(p, rows, T::dtype != VKT_F32, mc, &cols, &ksplit);
    if (variant & 0xffff) {
      cols = variant & 0xff;
      ksplit = (variant >> 8) & 0xff;
    }
    bool ok = false;
    switch (rows) {
      case 1: ok = launch_gemv_cols<T, 1, 2, 4>(p, cols, ksplit, stream); break;
      case 2: ok = launch_gemv_cols<T, 2, 2, 4>(p, cols, ksplit, stream); break;
      case 4: ok = launch_gemv_cols<T, 4, 2, 4>(p, cols, ksplit, stream); break;
      case 8: ok = launch_gemv_cols<T, 8, 1, 2>(p, cols, ksplit, stream); break;
      case 16: ok = launch_gemv_cols<T, 16, 1, 2>(p, cols, ksplit, stream); break;
    }
    if (!ok) {
      *err = "qmm8: no kernel variant COLS=" + std::to_string(cols) + " KSPLIT=" + std::to_string(ksplit) +
             " for " + std::to_string(rows) + " rows";
      return -1;
    }
  }
  return 0;
}

}  // namespace

int launch_qmm8(const Q8Params& p, int dtype, uint32_t variant, const Machine& mc, hipStream_t stream,
                std::string* err) {
  if (p.a_sk != 1) {
    *err = "qmm8: A must have unit stride along k (a_sk == 1)";
    return -1;
  }
  if (p.m == 0 || p.n == 0) return 0;
  if (p.a == 0 || p.b == 0 || p.scales == 0 || p.c == 0) {
    *err = "qmm8: null tensor address";
    return -1;
  }
  if (uint64_t(p.n) * p.k >= (1ull << 32) || uint64_t(p.m) * p.n >= (1ull << 32)) {
    *err = "qmm8: weights or output too large for 32-bit indexing";
    return -1;
  }
  int rc;
  switch (dtype) {
    case VKT_F32: rc = launch_qmm8_t<f32_t>(p, variant, mc, stream, err); break;
    case VKT_F16: rc = launch_qmm8_t<f16_t>(p, variant, mc, stream, err); break;
    case VKT_BF16: rc = launch_qmm8_t<bf16_t>(p, variant, mc, stream, err); break;
    default: *err = "qmm8: unsupported dtype"; return -1;
  }
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "qmm8: kernel launch failed";
    return -1;
  }
  return rc;
}

}  // namespace vkt
