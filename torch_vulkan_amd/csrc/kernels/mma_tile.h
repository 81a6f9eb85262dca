// The matrix-core tile kernel shared by aten::_scaled_mm (float8 operands) and the 16-bit
// matrix product: a workgroup computes a BM x BN tile of A [m, k] x B [n, k]^T, both operands
// rows of k contiguous BYTES (p.k counts bytes: float8 values, or 2 per 16-bit value),
// K in steps of 128 bytes through double-buffered LDS.  What differs between the users is
// the instruction that multiplies two 32-byte fragments (MATH) and the epilogue, which the
// problem type P supplies:
//   fields   a, b, lda, ldb (bytes), m, n, k (bytes), batches, a_batch, b_batch (bytes)
//   whole()                              per-launch constants of the epilogue
//   columns(batch, n, whole)             per-lane constants of columns n .. n + 3
//   store<DT>(batch, m, n, t, cols, whole)   finish and store 4 outputs of row m
//   for_output_type(full, whole, f)      call f(integral_constant<int, DT>) for the output type
//   kRegisterEpilogue                    the problem also offers the epilogue that stores straight from the accumulators:
//     register_epilogue(whole)             whether this launch takes it (bfloat16 output, aligned)
//     row_scale(m, whole), column_terms(n, whole, scale[4], bias[4])   what an output needs: acc * row_scale * scale[c] + bias[c]
//   kTransA, kTransB                     16-bit operands only: the operand is stored k-major, i.e.
//                                        as [k, m] (or [k, n]) rows lda (ldb) bytes apart, contiguous
//                                        along m (n); m (n) a multiple of 8, k of 64 values
// A k-major operand keeps its global layout in LDS ([64 k][BM or BN values], 16-byte chunks
// swizzled by the row's low bits) and the matrix-core fragments come out of it through the
// transposing LDS read (ds_read_b64_tr_b16: 16 lanes read a 4 (k) x 16 block of 2-byte
// values and each receives the 4 values of one column), so no layout costs a pass over memory.
#pragma once

#include <type_traits>

#include <string>

#include "common.h"

namespace vkt {
namespace {

constexpr int kMathFp8 = 0, kMathFp8Wide = 1, kMathBf16 = 2, kMathF16 = 3;

using V8I = int __attribute__((ext_vector_type(8)));
using V4I = int __attribute__((ext_vector_type(4)));
using V4F = float __attribute__((ext_vector_type(4)));

constexpr int BK = 128;  // bytes (= fp8 values) of K per step, one MFMA deep

template <int FA, int FB>
__device__ __forceinline__ V4F mfma_f8(const V8I& first, const V8I& second, const V4F& acc) {
  // first operand: rows of B (format FB), second: rows of A (format FA); zero scale
  // operands select the unscaled instruction
  return __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(first, second, acc, FB, FA, 0, 0, 0, 0);
}

using V16F = float __attribute__((ext_vector_type(16)));
template <int FA, int FB>
__device__ __forceinline__ V16F mfma_f8_32(const V8I& first, const V8I& second, const V16F& acc) {
  return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(first, second, acc, FB, FA, 0, 0, 0, 0);
}

// The exact path: float8 values widen exactly to bfloat16 (two per instruction), and the
// bfloat16 matrix core adds its products at float32 precision (measured: within 2^-27 of
// sum|a||b|).  Slice q of a 32-byte fragment = its bytes 8 q .. 8 q + 7: both operands are
// sliced alike, so every product pairs the same k.
using V8BF = __bf16 __attribute__((ext_vector_type(8)));
using V2BF = __bf16 __attribute__((ext_vector_type(2)));
template <int F, bool HI>
__device__ __forceinline__ V2BF widen_pair(int word) {
  if constexpr (F == 0) return __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(word, 1.0f, HI);
  else return __builtin_amdgcn_cvt_scalef32_pk_bf16_bf8(word, 1.0f, HI);
}
template <int F>
__device__ __forceinline__ V8BF widen_slice(const V8I& frag, int q) {
  const V2BF p0 = widen_pair<F, false>(frag[2 * q]), p1 = widen_pair<F, true>(frag[2 * q]);
  const V2BF p2 = widen_pair<F, false>(frag[2 * q + 1]), p3 = widen_pair<F, true>(frag[2 * q + 1]);
  return V8BF{p0.x, p0.y, p1.x, p1.y, p2.x, p2.y, p3.x, p3.y};
}

// LDS tile: rows of 128 bytes; 16-byte chunk c of row r sits at chunk c ^ ((r >> 1) & 7).
// The LDS serves 16 lanes of a 128-bit read per clock from 64 banks (256 bytes), and the 16
// lanes of a fragment read hold 16 consecutive rows at one logical chunk: two rows share a
// 256-byte line, and the key changes every two rows, so the 16 lanes land on 16 different
// 16-byte slots of the line (keying on r & 7 made rows r and r + 8 collide: measured as 4
// conflict cycles on every read).
__device__ __forceinline__ uint32_t tile_offset(uint32_t row, uint32_t chunk) {
  return row * BK + ((chunk ^ ((row >> 1) & 7u)) << 4);
}


using V8H = _Float16 __attribute__((ext_vector_type(8)));
// Half q (16 bytes) of a 32-byte fragment.
__device__ __forceinline__ V4I half_of(const V8I& f, int q) { return V4I{f[4 * q], f[4 * q + 1], f[4 * q + 2], f[4 * q + 3]}; }
template <int MATH>
__device__ __forceinline__ V16F mfma_16bit(const V4I& first, const V4I& second, const V16F& acc) {
  if constexpr (MATH == kMathBf16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(V8BF, first), __builtin_bit_cast(V8BF, second), acc, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(V8H, first), __builtin_bit_cast(V8H, second), acc, 0, 0, 0);
}

template <int WAVES_M, int WAVES_N, int TM, int TN, int FA, int FB, bool MF32, bool DIRECT, int MATH, class P>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void mma_tile(P p, uint32_t tiles_m, uint32_t tiles_n) {
  constexpr bool WIDE = MATH == kMathFp8Wide;
  static_assert(MATH == kMathFp8 || MF32, "the widened and 16-bit forms are built on the 32x32 tiles");
  constexpr bool TRA = P::kTransA, TRB = P::kTransB;
  static_assert(!(TRA || TRB) || (DIRECT && MF32 && (MATH == kMathBf16 || MATH == kMathF16)),
                "k-major operands: 16-bit values, direct loads, 32x32 tiles");
  constexpr int NT = WAVES_M * WAVES_N * 64;
  constexpr int BM = WAVES_M * TM * 16, BN = WAVES_N * TN * 16;
  constexpr int A_CHUNKS = BM * 8 / NT, B_CHUNKS = BN * 8 / NT;  // 16-byte chunks per thread per step
  static_assert(BM * 8 % NT == 0 && BN * 8 % NT == 0, "tile rows must divide over the threads");
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr uint32_t STAGE = (BM + BN) * BK;

  // tile order: groups of 8 consecutive workgroups land on the 8 XCDs round-robin, so
  // workgroup w runs on XCD w % 8.  Each XCD is given a contiguous band of tiles in
  // column-major order within a panel of `PANEL` tile rows, which keeps the operand rows
  // it touches resident in that XCD's L2.
  // The grid is persistent: about as many workgroups as fit the machine at once, each
  // walking through the slots of its XCD's band.  A tile's output stores then drain while
  // the next tile's main loop runs, instead of all compute units writing (and then all
  // starting cold) at the same moments.
  const uint32_t per_batch = tiles_m * tiles_n, total = per_batch * p.batches, per = (total + 7) / 8;
  for (uint32_t slot = blockIdx.x >> 3; slot < per; slot += gridDim.x >> 3) {
  const uint32_t wb = (blockIdx.x & 7u) * per + slot;
  if (wb >= total) break;  // whole workgroups only, and between barriers
  const uint32_t batch = wb / per_batch, w = wb % per_batch;
  const uint64_t a_base = p.a + uint64_t(batch) * p.a_batch, b_base = p.b + uint64_t(batch) * p.b_batch;
  constexpr uint32_t PANEL = 8;
  const uint32_t panel = w / (PANEL * tiles_n), in_panel = w % (PANEL * tiles_n);
  const uint32_t rows_here = tiles_m - panel * PANEL < PANEL ? tiles_m - panel * PANEL : PANEL;
  const uint32_t tile_m = panel * PANEL + in_panel % rows_here, tile_n = in_panel / rows_here;
  const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int l16 = lane & 15, g = lane >> 4;

  // global -> register staging: chunk id = tid + NT * i -> (row, chunk)
  uint64_t a_src[A_CHUNKS], b_src[B_CHUNKS];
  uint32_t a_dst[A_CHUNKS], b_dst[B_CHUNKS], a_k[A_CHUNKS], b_k[B_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; ++i) {
    // DIRECT: the load lands at LDS slot id (lane order), so the lane fetches the logical
    // chunk that the swizzle keeps in that slot
    if constexpr (TRA) {
      // slot id of the [64 k][BM values] tile -> (k row, chunk of 8 values along m); chunks past m repeat the last one
      const uint32_t id = tid + NT * i, row = id / (BM / 8), c = (id % (BM / 8)) ^ ((row & 3u) << 2);
      const uint32_t mc = m0 / 8 + c < p.m / 8 ? m0 / 8 + c : p.m / 8 - 1;
      a_src[i] = a_base + uint64_t(row) * p.lda + mc * 16;
      a_dst[i] = 0, a_k[i] = 0;
      continue;
    }
    const uint32_t id = tid + NT * i, row = id >> 3, c = DIRECT ? (id & 7u) ^ ((row >> 1) & 7u) : id & 7u;
    const uint32_t m = m0 + row < p.m ? m0 + row : p.m - 1;
    a_src[i] = a_base + uint64_t(m) * p.lda + c * 16;
    a_dst[i] = tile_offset(row, c);
    a_k[i] = c * 16;
  }
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) {
    if constexpr (TRB) {
      const uint32_t id = tid + NT * i, row = id / (BN / 8), c = (id % (BN / 8)) ^ ((row & 3u) << 2);
      const uint32_t nc = n0 / 8 + c < p.n / 8 ? n0 / 8 + c : p.n / 8 - 1;
      b_src[i] = b_base + uint64_t(row) * p.ldb + nc * 16;
      b_dst[i] = 0, b_k[i] = 0;
      continue;
    }
    const uint32_t id = tid + NT * i, row = id >> 3, c = DIRECT ? (id & 7u) ^ ((row >> 1) & 7u) : id & 7u;
    const uint32_t n = n0 + row < p.n ? n0 + row : p.n - 1;
    b_src[i] = b_base + uint64_t(n) * p.ldb + c * 16;
    b_dst[i] = BM * BK + tile_offset(row, c);
    b_k[i] = c * 16;
  }

  // MF32: the wave's sub-tile as (TM/2) x (TN/2) tiles of 32x32 (V_MFMA_F32_32X32X64_F8F6F4,
  // two per k-step along k); otherwise TM x TN tiles of 16x16 (one 16X16X128 per k-step).
  // Both leave a lane with groups of 4 consecutive output columns of one row.
  constexpr int TM2 = MF32 ? TM / 2 : 1, TN2 = MF32 ? TN / 2 : 1;
  V4F acc[MF32 ? 1 : TM][MF32 ? 1 : TN];
  V16F acc32[TM2][TN2];
  if constexpr (MF32) {
#pragma unroll
    for (int i = 0; i < TM2; ++i)
#pragma unroll
      for (int j = 0; j < TN2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc32[i][j][r] = 0.0f;
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = V4F{0.0f, 0.0f, 0.0f, 0.0f};
  }

  // Operand staging, software pipelined by hand.  One wave per SIMD means nothing else hides
  // what this wave does not: every global load and LDS write is issued between two MFMAs,
  // never in a block of its own.  While the matrix core works through step s the wave writes
  // the chunks of step s+1 from registers to LDS (first half of the step) and loads the
  // chunks of step s+2 into the same registers (second half).
  constexpr int NC = A_CHUNKS + B_CHUNKS;      // chunks per thread per step
  constexpr int NSIDE = DIRECT ? NC : 2 * NC, NMFMA = MF32 ? TM * TN / 2 : TM * TN;  // side operations / MFMAs per step
  V4I reg[NC];
  const V4I zero = {0, 0, 0, 0};
  const uint32_t steps = (p.k + BK - 1) / BK;
  // chunk c: A chunks first, then B chunks
  // A full step's chunk is loaded as is: nothing may touch the register until the LDS write,
  // or the wave would wait for the load where it was issued.  Only the last step of a k that
  // is not a multiple of 128 pays for a select (chunks beyond k read as zeros).
  auto load_chunk = [&](int c, uint32_t k0) {
    const uint64_t src = c < A_CHUNKS ? a_src[c < A_CHUNKS ? c : 0] : b_src[c < A_CHUNKS ? 0 : c - A_CHUNKS];
    reg[c] = ldg<V4I>(src + k0);
  };
  auto load_chunk_tail = [&](int c, uint32_t k0) {
    const uint64_t src = c < A_CHUNKS ? a_src[c < A_CHUNKS ? c : 0] : b_src[c < A_CHUNKS ? 0 : c - A_CHUNKS];
    const uint32_t kc = c < A_CHUNKS ? a_k[c < A_CHUNKS ? c : 0] : b_k[c < A_CHUNKS ? 0 : c - A_CHUNKS];
    const bool inside = k0 + kc < p.k;
    const V4I v = ldg<V4I>(src + (inside ? k0 : 0));  // (k >= 16: chunk 0 of the row exists)
    reg[c] = inside ? v : zero;
  };
  const uint32_t full_steps = p.k / BK;  // steps whose 128 bytes all lie inside k
  auto load_step = [&](int c, uint32_t step) {
    if (step < full_steps) load_chunk(c, step * BK);
    else load_chunk_tail(c, step * BK);
  };
  auto store_chunk = [&](int c, uint32_t stage) {
    const uint32_t dst = c < A_CHUNKS ? a_dst[c < A_CHUNKS ? c : 0] : b_dst[c < A_CHUNKS ? 0 : c - A_CHUNKS];
    *reinterpret_cast<V4I*>(lds + stage * STAGE + dst) = reg[c];
  };
  auto fragment = [&](const uint8_t* tile, uint32_t row) {
    const V4I lo = *reinterpret_cast<const V4I*>(tile + tile_offset(row, 2 * g));
    const V4I hi = *reinterpret_cast<const V4I*>(tile + tile_offset(row, 2 * g + 1));
    return V8I{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  // Side operation `op` of step s: [0,NC) write the chunks of step s+1 to LDS, [NC,2NC) load
  // the chunks of step s+2 into the same registers (all writes first: when the next step's
  // writes begin, every load is at least half a step old).  STEADY: both steps exist and are
  // full, so the code is straight-line (a branch here would make the compiler wait for
  // every load where it is issued).
  // DIRECT (k a multiple of 128): global_load_lds_dwordx4 moves a chunk from global memory
  // straight into LDS (a wave's 64 lanes fill 1 KiB at a wave-uniform base, in lane order):
  // no staging registers, no LDS write instructions.  The chunks of step s+1 go into the
  // stage that step s-1 read, while step s computes.
  auto direct_chunk = [&](int c, uint32_t step) {
    const uint64_t src = c < A_CHUNKS ? a_src[c < A_CHUNKS ? c : 0] : b_src[c < A_CHUNKS ? 0 : c - A_CHUNKS];
    const uint32_t tile_base = c < A_CHUNKS ? uint32_t(c) * NT * 16 : BM * BK + uint32_t(c - A_CHUNKS) * NT * 16;
    uint8_t* dst = lds + (step & 1u) * STAGE + tile_base + uint32_t(wave) * 1024;
    // a step is 128 bytes along a k-contiguous row, or 64 rows of a k-major operand
    const uint64_t advance = c < A_CHUNKS ? (TRA ? uint64_t(BK / 2) * p.lda : uint64_t(BK)) : (TRB ? uint64_t(BK / 2) * p.ldb : uint64_t(BK));
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const VKT_GLOBAL void*>(src + uint64_t(step) * advance),
                                     (__attribute__((address_space(3))) void*)(dst), 16, 0, 0);
  };
  auto side = [&](int op, uint32_t s, auto steady) {
    constexpr bool kSteady = decltype(steady)::value;
    if constexpr (DIRECT) {
      if (kSteady || s + 1 < steps) direct_chunk(op, s + 1);
    } else if (op < NC) {
      if (kSteady || s + 1 < steps) store_chunk(op, (s + 1) & 1u);
    } else {
      if (kSteady) load_chunk(op - NC, (s + 2) * BK);
      else if (s + 2 < steps) load_step(op - NC, s + 2);
    }
  };
  // One k-step: the wave's TM x TN MFMAs with the side operations and the LDS reads of the
  // next row fragment spread between them; the scheduling barriers keep the compiler from
  // moving anything back into blocks.
  auto step = [&](uint32_t s, auto steady) {
    const uint8_t* ta = lds + (s & 1u) * STAGE;
    const uint8_t* tb = ta + BM * BK;
    if constexpr (MF32) {
      // lane: row lane % 32 of a 32-row tile, 32 bytes of k at chunk pair 4 kk + 2 (lane / 32)
      const int l32 = lane & 31, h = lane >> 5;
      auto frag32 = [&](const uint8_t* tile, uint32_t row, int kk) {
        const V4I lo = *reinterpret_cast<const V4I*>(tile + tile_offset(row, 4 * kk + 2 * h));
        const V4I hi = *reinterpret_cast<const V4I*>(tile + tile_offset(row, 4 * kk + 2 * h + 1));
        return V8I{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
      };
      // LDS answers in the order asked: the first MFMA needs the first row fragment and the
      // first column fragment, so those are asked for first; the column fragments of the
      // second half of k are asked for once the first MFMAs are under way
      // (row fragments are asked for two groups of MFMAs ahead: one group, 256 cycles, is
      // less than an LDS read takes while the direct loads are writing into the same LDS)
      // The same fragment out of a k-major tile [64 k][W values]: for each half q of the fragment the 8
      // values k = 32 kk + 16 h + 8 q .. + 7 of column `col`, by two transposing reads of 4 k each.  Lane i
      // of a group of 16 points at row k + i / 4, values 4 (i % 4) .. + 3 of the group's 16 columns.
      auto frag32_t = [&](const uint8_t* tile, uint32_t width, uint32_t col0, int kk) {
        using V4S = short __attribute__((ext_vector_type(4)));
        V8I f;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t k = 32 * kk + 16 * h + 4 * t + (l16 >> 2);
          const uint32_t value = col0 + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);  // first of the 4 values this lane points at
          const uint32_t chunk = (value >> 3) ^ ((k & 3u) << 2);
          const V4S v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
              (__attribute__((address_space(3))) V4S*)(tile + k * width * 2 + chunk * 16 + (value & 7u) * 2));
          const U2 w = __builtin_bit_cast(U2, v);
          f[2 * t] = int(w.x), f[2 * t + 1] = int(w.y);
        }
        return f;
      };
      auto row_frag = [&](int gi) {
        if constexpr (TRA) return frag32_t(ta, BM, (wm * TM2 + gi % TM2) * 32, gi / TM2);
        else return frag32(ta, (wm * TM2 + gi % TM2) * 32 + l32, gi / TM2);
      };
      auto col_frag = [&](int j, int kk) {
        if constexpr (TRB) return frag32_t(tb, BN, (wn * TN2 + j) * 32, kk);
        else return frag32(tb, (wn * TN2 + j) * 32 + l32, kk);
      };
      // With two waves per SIMD (8 waves) the column fragments of the second half of k take the registers of the
      // first half's, each right after its last use (256 registers per wave do not hold both halves next to the
      // accumulators), and row fragments are asked for one group ahead: the other wave covers the LDS latency.
      constexpr bool kLean = WAVES_M * WAVES_N > 4;
      V8I af = row_frag(0);
      V8I bf[kLean ? 1 : 2][TN2];
#pragma unroll
      for (int j = 0; j < TN2; ++j) bf[0][j] = col_frag(j, 0);
      V8I next = row_frag(1 < 2 * TM2 ? 1 : 0);
#pragma unroll
      for (int gi = 0; gi < 2 * TM2; ++gi) {
        const int kk = gi / TM2, i = gi % TM2;
        V8I next2 = next;
        if (gi + 2 < 2 * TM2) next2 = row_frag(gi + 2);
        if (gi == 0 && !kLean) {
#pragma unroll
          for (int j = 0; j < TN2; ++j) bf[kLean ? 0 : 1][j] = col_frag(j, 1);
        }
        V8BF af_wide[WIDE ? 4 : 1];
        if constexpr (WIDE) {
#pragma unroll
          for (int q = 0; q < 4; ++q) af_wide[q] = widen_slice<FA>(af, q);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < TN2; ++j) {
          const int n = gi * TN2 + j;
          // DIRECT: the step ends by waiting for its loads, so they are all issued at its
          // start (FRONT per MFMA), not spread over it: the last one then has most of the
          // step to land instead of none of it
          constexpr int FRONT = 2;
          const int lo_op = DIRECT ? (n * FRONT < NSIDE ? n * FRONT : NSIDE) : n * NSIDE / NMFMA;
          const int hi_op = DIRECT ? ((n + 1) * FRONT < NSIDE ? (n + 1) * FRONT : NSIDE) : (n + 1) * NSIDE / NMFMA;
#pragma unroll
          for (int op = lo_op; op < hi_op; ++op) {
            side(op, s, steady);
            __builtin_amdgcn_sched_barrier(0);
          }
          if constexpr (WIDE) {
#pragma unroll
            for (int q = 0; q < 4; ++q)
              acc32[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(widen_slice<FB>(bf[kLean ? 0 : kk][j], q), af_wide[q], acc32[i][j], 0, 0, 0);
          } else if constexpr (MATH == kMathBf16 || MATH == kMathF16) {
            // 16-bit elements: a fragment's 32 bytes are two operands of 8 values
#pragma unroll
            for (int q = 0; q < 2; ++q) acc32[i][j] = mfma_16bit<MATH>(half_of(bf[kLean ? 0 : kk][j], q), half_of(af, q), acc32[i][j]);
          } else {
            acc32[i][j] = mfma_f8_32<FA, FB>(bf[kLean ? 0 : kk][j], af, acc32[i][j]);
          }
          if (kLean && gi == TM2 - 1) bf[0][j] = col_frag(j, 1);
        }
        __builtin_amdgcn_sched_barrier(0);
        af = next;
        next = next2;
      }
    } else {
      V8I bf[TN];
#pragma unroll
      for (int j = 0; j < TN; ++j) bf[j] = fragment(tb, (wn * TN + j) * 16 + l16);
      V8I af = fragment(ta, (wm * TM) * 16 + l16);
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        V8I next = af;
        if (i + 1 < TM) next = fragment(ta, (wm * TM + i + 1) * 16 + l16);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int n = i * TN + j;
          const int lo_op = n * NSIDE / NMFMA, hi_op = (n + 1) * NSIDE / NMFMA;
#pragma unroll
          for (int op = lo_op; op < hi_op; ++op) {
            side(op, s, steady);
            __builtin_amdgcn_sched_barrier(0);
          }
          acc[i][j] = mfma_f8<FA, FB>(bf[j], af, acc[i][j]);
        }
        __builtin_amdgcn_sched_barrier(0);
        af = next;
      }
    }
    if constexpr (DIRECT) __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this step's LDS-direct loads have landed
    __syncthreads();
  };

  uint32_t s = 0;
  if constexpr (DIRECT) {
#pragma unroll
    for (int c = 0; c < NC; ++c) direct_chunk(c, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    for (; s + 1 < steps; ++s) step(s, std::true_type{});
    for (; s < steps; ++s) step(s, std::false_type{});
  } else {
    // prologue: step 0 into LDS, step 1 into the registers
#pragma unroll
    for (int c = 0; c < NC; ++c) load_step(c, 0);
#pragma unroll
    for (int c = 0; c < NC; ++c) store_chunk(c, 0);
    if (steps > 1) {
#pragma unroll
      for (int c = 0; c < NC; ++c) load_step(c, 1);
    }
    __syncthreads();
    for (; s + 2 < full_steps; ++s) step(s, std::true_type{});
    for (; s < steps; ++s) step(s, std::false_type{});
  }

  const auto whole = p.whole();  // what the epilogue needs once per launch
  const uint32_t wm0 = m0 + wm * TM * 16, wn0 = n0 + wn * TN * 16;
  // Epilogue from the registers (bfloat16 outputs of whole tiles): no LDS, no barrier, so nothing holds a wave back
  // once its last matrix-core instruction has gone, and the next tile's first loads may land in LDS meanwhile.  A 32 x 32
  // matrix-core tile leaves lane l with row l % 32 and, for q = 0..3, columns 8 q + 4 (l / 32) .. + 3: two lanes 32
  // apart hold the two halves of 8 consecutive outputs.  v_permlane32_swap puts them together (lanes below 32 take
  // chunk q = 0 or 2 of their row, lanes from 32 chunk 1 or 3), and every lane stores 16 bytes; a store instruction
  // of a wave writes 32 rows x 32 consecutive bytes.
  bool from_registers = false;
  if constexpr (MF32 && P::kRegisterEpilogue) {
    from_registers = p.register_epilogue(whole) && n0 + BN <= p.n;  // (the same for every wave of the workgroup)
    if (from_registers) {
      const uint32_t l32 = lane & 31, h = lane >> 5;
#pragma unroll
      for (int j = 0; j < TN2; ++j) {
        float scale[4][4], bias[4][4];  // of this lane's columns wn0 + 32 j + 8 q + 4 h + r
#pragma unroll
        for (int q = 0; q < 4; ++q) p.column_terms(wn0 + 32 * j + 8 * q + 4 * h, whole, scale[q], bias[q]);
#pragma unroll
        for (int i = 0; i < TM2; ++i) {
          const uint32_t m = wm0 + 32 * i + l32;
          const float rs = p.row_scale(m < p.m ? m : p.m - 1, whole);
          const V16F& t = acc32[i][j];
#pragma unroll
          for (int qp = 0; qp < 2; ++qp) {
            uint32_t lo[2], hi[2];  // chunks 2 qp and 2 qp + 1 as two bfloat16 pairs each
#pragma unroll
            for (int e = 0; e < 2; ++e) {
              const int q0 = 2 * qp, q1 = 2 * qp + 1;
              lo[e] = pack_bf16(t[4 * q0 + 2 * e] * (rs * scale[q0][2 * e]) + bias[q0][2 * e],
                                t[4 * q0 + 2 * e + 1] * (rs * scale[q0][2 * e + 1]) + bias[q0][2 * e + 1]);
              hi[e] = pack_bf16(t[4 * q1 + 2 * e] * (rs * scale[q1][2 * e]) + bias[q1][2 * e],
                                t[4 * q1 + 2 * e + 1] * (rs * scale[q1][2 * e + 1]) + bias[q1][2 * e + 1]);
            }
            // lanes 32.. of `lo` change places with lanes ..31 of `hi`
            const auto s0 = __builtin_amdgcn_permlane32_swap(lo[0], hi[0], false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(lo[1], hi[1], false, false);
            const uint32_t n = wn0 + 32 * j + 8 * (2 * qp + h);
            if (m < p.m) p.store_bf16x8(batch, m, n, U4{s0[0], s1[0], s0[1], s1[1]});
          }
        }
      }
    }
  }
  if (!from_registers) {
  // Epilogue through LDS.  A lane holds out[m = .. + l16][n = .. + 4 g + r], r = 0..3, for each of its
  // TM x TN tiles.  Each wave transposes its sub-tile through its own slice of LDS (the
  // operand buffers are dead by now), 64 columns at a time, so that the scale / bias / cast
  // code exists once (a loop, not TM*TN unrolled copies) and every store instruction of a
  // wave writes four rows of 64 consecutive outputs.
  constexpr uint32_t EP_ROW = 256;                    // bytes: 64 float32 columns
  constexpr uint32_t EP_WAVE = TM * 16 * EP_ROW;      // bytes of LDS per wave
  float* ep = reinterpret_cast<float*>(lds + wave * EP_WAVE);
#pragma unroll
  for (int pass = 0; pass < TN / 4; ++pass) {
    // (the first pass may start only when every wave is done reading operands; later ones
    // when this wave's previous pass has been read back)
    __syncthreads();
    if constexpr (MF32) {
      // a 32x32 tile leaves lane l with row l % 32 and, for q = 0..3, columns 8 q + 4 (l / 32) .. + 3
#pragma unroll
      for (int i = 0; i < TM2; ++i)
#pragma unroll
        for (int jj = 0; jj < 2; ++jj)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const uint32_t row = i * 32 + (lane & 31), chunk = jj * 8 + 2 * q + (lane >> 5);
            const V16F& t = acc32[i][pass * 2 + jj];
            *reinterpret_cast<V4F*>(reinterpret_cast<uint8_t*>(ep) + row * EP_ROW + ((chunk ^ (row & 15u)) << 4)) =
                V4F{t[4 * q], t[4 * q + 1], t[4 * q + 2], t[4 * q + 3]};
          }
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const uint32_t row = i * 16 + l16, chunk = jj * 4 + g;
          *reinterpret_cast<V4F*>(reinterpret_cast<uint8_t*>(ep) + row * EP_ROW + ((chunk ^ (row & 15u)) << 4)) =
              acc[i][pass * 4 + jj];
        }
    }
    __syncthreads();
    // lane -> (row offset lane / 16, chunk lane % 16): 4 consecutive columns, fixed over the loop
    const uint32_t chunk = lane & 15, n = wn0 + pass * 64 + chunk * 4;
    const auto cols = p.columns(batch, n, whole);  // what the lane's 4 columns need (scales, bias ...)
    // The row loop, once per output type (so that its body is straight-line and four rows'
    // LDS reads and the epilogue's own loads are in flight together).
    auto rows = [&](auto dt) {
      constexpr int DT = decltype(dt)::value;
      // (the register-staged 256x256 kernels have no registers to spare for the unrolling)
      constexpr int UNROLL = (DIRECT || TM * TN < 64) ? 4 : 1;
#pragma unroll UNROLL
      for (uint32_t it = 0; it < TM * 4; ++it) {
        const uint32_t row = it * 4 + (lane >> 4), m = wm0 + row;
        const V4F t = *reinterpret_cast<const V4F*>(reinterpret_cast<const uint8_t*>(ep) + row * EP_ROW +
                                                     ((chunk ^ (row & 15u)) << 4));
        if (m >= p.m || n >= p.n) continue;
        p.template store<DT>(batch, m, n, t, cols, whole);
      }
    };
    // (DT: the output type, chosen outside the loop; -1: element by element, for unaligned
    // outputs and the columns past n)
    p.for_output_type(n + 3 < p.n, whole, rows);
  }
  __syncthreads();  // the next tile's operands overwrite the LDS the epilogue has just read
  }  // (epilogue through LDS)
  }  // (tile loop)
}


// Launches the tile kernel for problem p (persistent grid: as many workgroups as are resident
// at once, in multiples of 8, one per XCD).
template <int WAVES_M, int WAVES_N, int TM, int TN, int FA, int FB, bool MF32, bool DIRECT, int MATH, class P>
int launch_mma_tile(const P& p, int compute_units, hipStream_t stream, std::string* err, const char* who) {
  constexpr int BM = WAVES_M * TM * 16, BN = WAVES_N * TN * 16;
  constexpr uint32_t operand_bytes = 2 * (BM + BN) * BK, epilogue_bytes = WAVES_M * WAVES_N * TM * 16 * 256;
  constexpr uint32_t lds_bytes = operand_bytes > epilogue_bytes ? operand_bytes : epilogue_bytes;
  static_assert(TN % 4 == 0, "the epilogue moves 64 columns (4 tiles) per pass");
  auto kernel = mma_tile<WAVES_M, WAVES_N, TM, TN, FA, FB, MF32, DIRECT, MATH, P>;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            lds_bytes) != hipSuccess) {
      (void)hipGetLastError();
      *err = std::string(who) + ": cannot reserve " + std::to_string(lds_bytes) + " bytes of LDS";
      return -1;
    }
    configured = true;
  }
  const uint32_t tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  const uint64_t total = uint64_t(tiles_m) * tiles_n * p.batches;
  if (total >= (1ull << 31)) {
    *err = std::string(who) + ": too many tiles";
    return -1;
  }
  const uint32_t per_cu = lds_bytes > 80 * 1024 ? 1 : (lds_bytes > 53 * 1024 ? 2 : 3);
  const uint64_t resident = (uint64_t(compute_units) * per_cu + 7) / 8 * 8;
  const uint64_t grid = (total + 7) / 8 * 8 < resident ? (total + 7) / 8 * 8 : resident;
  hipLaunchKernelGGL(kernel, dim3(uint32_t(grid)), dim3(WAVES_M * WAVES_N * 64), lds_bytes, stream, p, tiles_m, tiles_n);
  return 0;
}

}  // namespace
}  // namespace vkt
