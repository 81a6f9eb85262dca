// aten::_scaled_mm on gfx950 as one fused kernel:
//   out[m,n] = cast( (sum_k f32(A[m,k]) * f32(B[k,n])) * scale_a[m|0] * scale_b[n|0] + bias[n] ) [* 1/scale_result]
// for float8 (e4m3fn / e5m2, any mix) A [M,K] row-major and B [K,N] column-major (stored as
// [N,K] rows), float32 scales per tensor or per row / column.  It replaces the reference's
// composite (crates/pyvk/csrc/quant.cpp:279-300: two table-gather upcasts, two multiplies, a
// float32 GEMM on shader cores, bias add, cast, copy: seven passes over full-size float32
// temporaries) with the product on the fp8 matrix cores and everything else in the epilogue.
// Products of two float8 values are exact in float32.  The matrix core, however, adds the
// 128 products of one instruction in a fixed-point window: each product is aligned to the
// largest exponent of its group and bits more than ~14 below it are dropped (measured on
// gfx950: 448*1 + 0.0625*1 is kept, 448*1 + 0.0156*1 loses the small term; the accumulator
// input itself is added in full float32).  On random data that is an error of ~2^-16 of
// sum|a||b| per output, invisible at bfloat16 / float8 output precision (eps >= 2^-8) but
// not at float32.  So the path is chosen by the precision the caller asked for:
//   bfloat16 / float8 outputs  -> fp8mm_mfma (this is the 5 PFLOP/s path)
//   float32 / float16 outputs  -> the same kernel with each float8 fragment widened (exactly)
//                                 to bfloat16 in registers and fed to the bfloat16 matrix
//                                 core, which keeps float32 precision (half the rate: 2.5
//                                 PFLOP/s peak); inside the reference test's bound
//                                 eps*|want| + 2^-20 * sum|a||b| (tests/python/test_quant.py:124-126)
// The scales multiply once per output instead of once per operand element (one rounding
// less than the reference, inside the same bound).
//
//   fp8mm_mfma     V_MFMA_F32_32X32X64_F8F6F4 / 16X16X128 (8192 flop/clk/CU: the only fp8 rate
//                  that reaches the 5 PFLOP/s peak; the 16x16x32 fp8 instruction runs at half).
//                  A workgroup computes a BM x BN tile, K in steps of 128 bytes; both
//                  operand tiles are staged in LDS (double buffered, 16-byte chunks XOR-
//                  swizzled by row pair so that the 32-byte-per-lane fragment reads are
//                  conflict free), each wave owns a (TM*16) x (TN*16) sub-tile in registers.
//                  The B matrix feeds the MFMA's first operand and A its second, so a lane
//                  ends up with 4 consecutive output columns of one row (vector stores).
//   fp8mm_generic  any shape / alignment: one thread per output, float32 FMA.
#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace vkt {
namespace {

using V8I = int __attribute__((ext_vector_type(8)));
using V4I = int __attribute__((ext_vector_type(4)));
using V4F = float __attribute__((ext_vector_type(4)));

constexpr int BK = 128;  // bytes (= fp8 values) of K per step, one MFMA deep

__device__ __forceinline__ float load_any_f32(uint64_t base, uint64_t i, uint32_t dtype) {
  if (dtype == VKT_F32) return ldg<float>(base + 4 * i);
  if (dtype == VKT_F16) return f16_to_f32(ldg<uint16_t>(base + 2 * i));
  return bf16_to_f32(ldg<uint16_t>(base + 2 * i));
}

// Scales, bias and the output scale for one output value.
__device__ __forceinline__ float finish(const F8Params& p, float acc, float sa, float sb, uint32_t n, float inv) {
  float v = acc * (sa * sb);
  if (p.bias) v += load_any_f32(p.bias, n, p.bias_dtype);
  if (p.out_dtype == VKT_E4M3 || p.out_dtype == VKT_E5M2) v *= inv;
  return v;
}

__device__ __forceinline__ void store_out(const F8Params& p, uint64_t index, float v) {
  switch (p.out_dtype) {
    case VKT_F32: stg<float>(p.out + index * 4, v); break;
    case VKT_F16: stg<uint16_t>(p.out + index * 2, f32_to_f16(v)); break;
    case VKT_BF16: stg<uint16_t>(p.out + index * 2, f32_to_bf16(v)); break;
    default: stg<uint8_t>(p.out + index, uint8_t(f32_to_fp8(v, int(p.out_dtype)))); break;
  }
}

// Two float32 -> two bfloat16 in one word: v_cvt_pk_bf16_f32 (round to nearest even); NaN
// becomes 0x7fc0 as c10 writes it.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  using V2 = __bf16 __attribute__((ext_vector_type(2)));
  const float qnan = bits_f32(0x7fc00000u);
  a = a != a ? qnan : a;
  b = b != b ? qnan : b;
  return __builtin_bit_cast(uint32_t, V2{static_cast<__bf16>(a), static_cast<__bf16>(b)});
}

__device__ __forceinline__ float output_inv(const F8Params& p) {
  if (!(p.out_dtype == VKT_E4M3 || p.out_dtype == VKT_E5M2)) return 1.0f;
  return 1.0f / (p.scale_result ? ldg<float>(p.scale_result) : 1.0f);
}

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

template <int WAVES_M, int WAVES_N, int TM, int TN, int FA, int FB, bool MF32 = false, bool DIRECT = false, bool WIDE = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void fp8mm_mfma(F8Params p, uint32_t tiles_m, uint32_t tiles_n) {
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
  const uint32_t total = tiles_m * tiles_n, per = (total + 7) / 8;
  for (uint32_t slot = blockIdx.x >> 3; slot < per; slot += gridDim.x >> 3) {
  const uint32_t w = (blockIdx.x & 7u) * per + slot;
  if (w >= total) break;  // whole workgroups only, and between barriers
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
    const uint32_t id = tid + NT * i, row = id >> 3, c = DIRECT ? (id & 7u) ^ ((row >> 1) & 7u) : id & 7u;
    const uint32_t m = m0 + row < p.m ? m0 + row : p.m - 1;
    a_src[i] = p.a + uint64_t(m) * p.lda + c * 16;
    a_dst[i] = tile_offset(row, c);
    a_k[i] = c * 16;
  }
#pragma unroll
  for (int i = 0; i < B_CHUNKS; ++i) {
    const uint32_t id = tid + NT * i, row = id >> 3, c = DIRECT ? (id & 7u) ^ ((row >> 1) & 7u) : id & 7u;
    const uint32_t n = n0 + row < p.n ? n0 + row : p.n - 1;
    b_src[i] = p.b + uint64_t(n) * p.ldb + c * 16;
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
    __builtin_amdgcn_global_load_lds(reinterpret_cast<const VKT_GLOBAL void*>(src + uint64_t(step) * BK),
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
      auto row_frag = [&](int gi) { return frag32(ta, (wm * TM2 + gi % TM2) * 32 + l32, gi / TM2); };
      V8I af = row_frag(0);
      V8I bf[2][TN2];
#pragma unroll
      for (int j = 0; j < TN2; ++j) bf[0][j] = frag32(tb, (wn * TN2 + j) * 32 + l32, 0);
      V8I next = row_frag(1 < 2 * TM2 ? 1 : 0);
#pragma unroll
      for (int gi = 0; gi < 2 * TM2; ++gi) {
        const int kk = gi / TM2, i = gi % TM2;
        V8I next2 = next;
        if (gi + 2 < 2 * TM2) next2 = row_frag(gi + 2);
        if (gi == 0) {
#pragma unroll
          for (int j = 0; j < TN2; ++j) bf[1][j] = frag32(tb, (wn * TN2 + j) * 32 + l32, 1);
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
              acc32[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(widen_slice<FB>(bf[kk][j], q), af_wide[q], acc32[i][j], 0, 0, 0);
          } else {
            acc32[i][j] = mfma_f8_32<FA, FB>(bf[kk][j], af, acc32[i][j]);
          }
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

  // Epilogue.  A lane holds out[m = .. + l16][n = .. + 4 g + r], r = 0..3, for each of its
  // TM x TN tiles.  Each wave transposes its sub-tile through its own slice of LDS (the
  // operand buffers are dead by now), 64 columns at a time, so that the scale / bias / cast
  // code exists once (a loop, not TM*TN unrolled copies) and every store instruction of a
  // wave writes four rows of 64 consecutive outputs.
  constexpr uint32_t EP_ROW = 256;                    // bytes: 64 float32 columns
  constexpr uint32_t EP_WAVE = TM * 16 * EP_ROW;      // bytes of LDS per wave
  float* ep = reinterpret_cast<float*>(lds + wave * EP_WAVE);
  const float inv = output_inv(p);
  const float sa_all = p.rowwise ? 0.0f : ldg<float>(p.scale_a), sb_all = p.rowwise ? 0.0f : ldg<float>(p.scale_b);
  const bool vec_ok = (p.ldo & 3u) == 0 && (p.out & 15u) == 0;
  const uint32_t wm0 = m0 + wm * TM * 16, wn0 = n0 + wn * TN * 16;
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
    float sb[4], bias[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const uint32_t nn = n + r < p.n ? n + r : p.n - 1;
      sb[r] = p.rowwise ? ldg<float>(p.scale_b + 4ull * nn) : sb_all;
      bias[r] = p.bias ? load_any_f32(p.bias, nn, p.bias_dtype) : 0.0f;
    }
    // The row loop, once per output type (chosen outside the loop, so that its body is
    // straight-line and four rows' LDS reads and scale loads are in flight together).
    // DT < 0: any type, element by element (unaligned outputs and the columns past n).
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
        const float sa = p.rowwise ? ldg<float>(p.scale_a + 4ull * m) : sa_all;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          v[r] = t[r] * (sa * sb[r]);
          if (p.bias) v[r] += bias[r];
          if (DT < 0 || DT == VKT_E4M3 || DT == VKT_E5M2) v[r] *= inv;  // (inv is 1 for the other types)
        }
        const uint64_t index = uint64_t(m) * p.ldo + n;
        if constexpr (DT == VKT_F32) {
          stg<F4>(p.out + index * 4, F4{v[0], v[1], v[2], v[3]});
        } else if constexpr (DT == VKT_BF16) {
          stg<U2>(p.out + index * 2, U2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])});
        } else if constexpr (DT == VKT_F16) {
          stg<U2>(p.out + index * 2, U2{uint32_t(f32_to_f16(v[0])) | uint32_t(f32_to_f16(v[1])) << 16,
                                        uint32_t(f32_to_f16(v[2])) | uint32_t(f32_to_f16(v[3])) << 16});
        } else if constexpr (DT == VKT_E4M3 || DT == VKT_E5M2) {
          stg<uint32_t>(p.out + index, pack2_fp8<DT>(v[0], v[1]) | pack2_fp8<DT>(v[2], v[3]) << 16);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n + r < p.n) store_out(p, index + r, v[r]);
        }
      }
    };
    if (vec_ok && n + 3 < p.n) {
      switch (p.out_dtype) {
        case VKT_F32: rows(std::integral_constant<int, VKT_F32>{}); break;
        case VKT_BF16: rows(std::integral_constant<int, VKT_BF16>{}); break;
        case VKT_F16: rows(std::integral_constant<int, VKT_F16>{}); break;
        case VKT_E4M3: rows(std::integral_constant<int, VKT_E4M3>{}); break;
        default: rows(std::integral_constant<int, VKT_E5M2>{}); break;
      }
    } else {
      rows(std::integral_constant<int, -1>{});
    }
  }
  __syncthreads();  // the next tile's operands overwrite the LDS the epilogue has just read
  }  // (tile loop)
}

// Any shape, stride or alignment: one thread per output.
__global__ __launch_bounds__(256) void fp8mm_generic(F8Params p) {
  const uint32_t n = blockIdx.x * 64 + (threadIdx.x & 63), m = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (m >= p.m || n >= p.n) return;
  const uint64_t arow = p.a + uint64_t(m) * p.lda, brow = p.b + uint64_t(n) * p.ldb;
  float acc = 0.0f;
  for (uint32_t k = 0; k < p.k; ++k)
    acc = fmaf(fp8_to_f32(ldg<uint8_t>(arow + k), int(p.fmt_a)), fp8_to_f32(ldg<uint8_t>(brow + k), int(p.fmt_b)), acc);
  const float sa = ldg<float>(p.scale_a + (p.rowwise ? 4ull * m : 0)), sb = ldg<float>(p.scale_b + (p.rowwise ? 4ull * n : 0));
  store_out(p, uint64_t(m) * p.ldo + n, finish(p, acc, sa, sb, n, output_inv(p)));
}

template <int WAVES_M, int WAVES_N, int TM, int TN, int FA, int FB, bool MF32 = false, bool DIRECT = false, bool WIDE = false>
int launch_tile(const F8Params& p, int compute_units, hipStream_t stream, std::string* err) {
  constexpr int BM = WAVES_M * TM * 16, BN = WAVES_N * TN * 16;
  constexpr uint32_t operand_bytes = 2 * (BM + BN) * BK, epilogue_bytes = WAVES_M * WAVES_N * TM * 16 * 256;
  constexpr uint32_t lds_bytes = operand_bytes > epilogue_bytes ? operand_bytes : epilogue_bytes;
  static_assert(TN % 4 == 0, "the epilogue moves 64 columns (4 tiles) per pass");
  static_assert(!WIDE || MF32, "the exact path is built on the 32x32 tiles");
  auto kernel = fp8mm_mfma<WAVES_M, WAVES_N, TM, TN, FA, FB, MF32, DIRECT, WIDE>;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                            lds_bytes) != hipSuccess) {
      (void)hipGetLastError();
      *err = "fp8mm: cannot reserve " + std::to_string(lds_bytes) + " bytes of LDS";
      return -1;
    }
    configured = true;
  }
  const uint32_t tiles_m = (p.m + BM - 1) / BM, tiles_n = (p.n + BN - 1) / BN;
  const uint64_t total = uint64_t(tiles_m) * tiles_n;
  if (total >= (1ull << 31)) {
    *err = "fp8mm: too many tiles";
    return -1;
  }
  // as many workgroups as are resident at once (LDS decides), in multiples of 8 (one per XCD)
  const uint32_t per_cu = lds_bytes > 80 * 1024 ? 1 : (lds_bytes > 53 * 1024 ? 2 : 3);
  const uint64_t resident = (uint64_t(compute_units) * per_cu + 7) / 8 * 8;
  const uint64_t grid = (total + 7) / 8 * 8 < resident ? (total + 7) / 8 * 8 : resident;
  hipLaunchKernelGGL(kernel, dim3(uint32_t(grid)), dim3(WAVES_M * WAVES_N * 64), lds_bytes, stream, p, tiles_m, tiles_n);
  return 0;
}

template <int FA, int FB>
int launch_formats(const F8Params& p, uint32_t variant, int compute_units, hipStream_t stream, std::string* err) {
  // variant 0: planned.  Explicit variants run the MFMA kernel whatever the output dtype
  // (tests, tuning): 1: 128x128 tiles (4 waves of 64x64, 16x16x128 MFMA); 2: 256x256 (4 waves of
  // 128x128, 16x16x128); 3: 256x128; 4: 256x256 with the 32x32x64 MFMA (measured ~10 % faster
  // than 16x16x128 at equal work); 5: as 4 with global-to-LDS direct loads when k is a
  // multiple of 128 (else 4).  255: the one-thread-per-output kernel.
  // 6 / 7: the exact path (float8 widened to bfloat16 in registers, 32x32x16 bfloat16 MFMA) on
  // 256x256 / 128x128 tiles: what float32 and float16 outputs get.
  const bool big = uint64_t(p.m) * p.n >= (1ull << 20);
  if (variant == 0) variant = (p.out_dtype == VKT_F32 || p.out_dtype == VKT_F16) ? (big ? 6 : 7) : (big ? 5 : 1);
  switch (variant) {
    case 6:
      if (p.k % BK == 0) return launch_tile<2, 2, 8, 8, FA, FB, true, true, true>(p, compute_units, stream, err);
      return launch_tile<2, 2, 8, 4, FA, FB, true, false, true>(p, compute_units, stream, err);  // (256x256 without the direct loads runs out of registers)
    case 7: return launch_tile<2, 2, 4, 4, FA, FB, true, false, true>(p, compute_units, stream, err);
    case 1: return launch_tile<2, 2, 4, 4, FA, FB>(p, compute_units, stream, err);
    case 2: return launch_tile<2, 2, 8, 8, FA, FB>(p, compute_units, stream, err);
    case 3: return launch_tile<2, 2, 8, 4, FA, FB>(p, compute_units, stream, err);
    case 4: return launch_tile<2, 2, 8, 8, FA, FB, true>(p, compute_units, stream, err);
    case 5:
      if (p.k % BK == 0) return launch_tile<2, 2, 8, 8, FA, FB, true, true>(p, compute_units, stream, err);
      return launch_tile<2, 2, 8, 8, FA, FB, true>(p, compute_units, stream, err);
  }
  *err = "fp8mm: unknown variant " + std::to_string(variant);
  return -1;
}

}  // namespace

int launch_fp8mm(const F8Params& p, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err) {
  if (p.m == 0 || p.n == 0) return 0;
  auto fp8 = [](uint32_t f) { return f == VKT_E4M3 || f == VKT_E5M2; };
  if (!fp8(p.fmt_a) || !fp8(p.fmt_b)) {
    *err = "fp8mm: operands must be e4m3fn or e5m2";
    return -1;
  }
  if (p.out_dtype > VKT_E5M2 || p.bias_dtype > VKT_BF16) {
    *err = "fp8mm: unsupported output or bias dtype";
    return -1;
  }
  if (!p.a || !p.b || !p.scale_a || !p.scale_b || !p.out) {
    *err = "fp8mm: null tensor address";
    return -1;
  }
  if (p.lda < p.k || p.ldb < p.k || p.ldo < p.n) {
    *err = "fp8mm: row strides shorter than the rows";
    return -1;
  }
  if (uint64_t(p.m) * p.ldo >= (1ull << 32)) {
    *err = "fp8mm: output too large for 32-bit indexing";
    return -1;
  }
  int rc;
  if (p.k == 0 || p.k % 16 || p.lda % 16 || p.ldb % 16 || (p.a & 15) || (p.b & 15) || variant == 255) {
    if ((p.m + 3) / 4 > 65535) {
      *err = "fp8mm: too many rows for the unaligned path";
      return -1;
    }
    hipLaunchKernelGGL(fp8mm_generic, dim3((p.n + 63) / 64, (p.m + 3) / 4), dim3(256), 0, stream, p);
    rc = 0;
  } else if (p.fmt_a == VKT_E4M3 && p.fmt_b == VKT_E4M3) {
    rc = launch_formats<0, 0>(p, variant, mc.compute_units, stream, err);
  } else if (p.fmt_a == VKT_E5M2 && p.fmt_b == VKT_E4M3) {
    rc = launch_formats<1, 0>(p, variant, mc.compute_units, stream, err);
  } else if (p.fmt_a == VKT_E4M3 && p.fmt_b == VKT_E5M2) {
    rc = launch_formats<0, 1>(p, variant, mc.compute_units, stream, err);
  } else {
    rc = launch_formats<1, 1>(p, variant, mc.compute_units, stream, err);
  }
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "fp8mm: kernel launch failed";
    return -1;
  }
  return rc;
}

}  // namespace vkt
