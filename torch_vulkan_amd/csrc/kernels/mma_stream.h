// The matrix-core kernel for large products with bfloat16 output: 256 x 256 tiles of A [m, k] x B [n, k]^T (rows of k
// contiguous bytes, as in mma_tile.h) on 8 waves of 64 x 128, K in steps of 128 bytes through two LDS stages of 64 KiB.
// It differs from mma_tile in how a workgroup's time is laid out, after measuring where mma_tile's goes (one wave's
// clock read at four points of every step): the matrix cores were busy 58-66 % of the cycles; the rest was the wave
// issuing address arithmetic for its LDS-direct loads (380 cycles a step) and all eight waves starting every step
// with empty fragment registers right after the barrier (460 cycles a step).  Here:
//   * A workgroup's tiles form ONE stream of steps.  The loads run two steps ahead of the arithmetic and cross from
//     a tile into the next one, so a tile's first operands are in LDS before its predecessor's epilogue starts, and
//     the epilogue (straight from the accumulators, no LDS) overlaps the loads in flight.
//   * The barrier of a step sits in its MIDDLE: by then a wave has read every fragment of the step (the second half
//     of k is read during the first half's matrix-core instructions), so after the barrier the stage is free for
//     the loads of step + 2, the other stage (landed: every wave waited for its own loads before the barrier) may be
//     read for step + 1, and the wave still holds eight matrix-core instructions' worth of operands.  No wave ever
//     waits for LDS with an idle matrix core.
//   * An LDS-direct load costs three instructions: the global address is a uniform base (scalar registers, advanced
//     by scalar adds) plus a per-lane 32-bit offset that is constant for the whole tile, and a wave's four loads of
//     an operand differ by the instruction's immediate offset, which moves the LDS address and the global address
//     alike (the per-lane offsets compensate).  They are written as inline assembly: the compiler's own form of the
//     instruction makes it wait for ALL outstanding LDS reads before every use of any of them.
//     The compiler therefore does not know these loads: the kernel waits for them itself (s_waitcnt vmcnt) and the
//     compiler's own waits, which count only what it knows, can only be longer than needed.
// The problem type P is mma_tile's, restricted to what the epilogue from the registers serves (P::kRegisterEpilogue):
// bfloat16 outputs, rows 16-byte aligned, n a multiple of 8; k a multiple of 128 and at least 256.
#pragma once

#include "mma_tile.h"

namespace vkt {
namespace {

// One LDS-direct load of 16 bytes per lane: global address `base` + `offset` + OFF, LDS address `lds_at` + OFF + 16 * lane.
template <int OFF>
__device__ __forceinline__ void load_to_lds(uint32_t offset, uint64_t base, uint32_t lds_at) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3" ::"v"(offset), "s"(base), "s"(lds_at), "i"(OFF)
               : "memory", "m0");
}

template <int FA, int FB, class P>
__global__ __launch_bounds__(512) void mma_stream(P p, uint32_t tiles_m, uint32_t tiles_n) {
  static_assert(P::kRegisterEpilogue && !P::kTransA && !P::kTransB, "float8-style operands, epilogue from the registers");
  constexpr uint32_t BM = 256, BN = 256, STAGE = (BM + BN) * BK, B_AT = BM * BK;
  constexpr int TM2 = 2, TN2 = 4;  // a wave's 64 x 128 as 32 x 32 matrix-core tiles
  constexpr uint32_t BIAS = 3072;  // keeps the per-lane offsets non-negative (they carry -1024 i for load i of 4)
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  const uint32_t lds0 = uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void*)(lds)));

  const uint32_t lane = threadIdx.x & 63u, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t wm = wave >> 1, wn = wave & 1u, l32 = lane & 31u, h = lane >> 5;
  const uint32_t steps = p.k / BK;

  // this workgroup's tiles: slot first, first + stride, ... of its XCD's band (the order of mma_tile)
  const uint32_t per_batch = tiles_m * tiles_n, total = per_batch * p.batches, per = (total + 7) / 8;
  const uint32_t first = blockIdx.x >> 3, stride = gridDim.x >> 3, band = (blockIdx.x & 7u) * per;
  if (first >= per || band + first >= total) return;
  const uint32_t band_end = total - band < per ? total - band : per;
  const uint32_t mine = (band_end - first + stride - 1) / stride;
  struct Tile {
    uint32_t batch, m0, n0;
  };
  auto tile_at = [&](uint32_t index) {
    const uint32_t wb = band + first + index * stride, batch = wb / per_batch, w = wb % per_batch;
    constexpr uint32_t PANEL = 8;
    const uint32_t panel = w / (PANEL * tiles_n), in_panel = w % (PANEL * tiles_n);
    const uint32_t rows_here = tiles_m - panel * PANEL < PANEL ? tiles_m - panel * PANEL : PANEL;
    return Tile{batch, (panel * PANEL + in_panel % rows_here) * BM, (in_panel / rows_here) * BN};
  };

  // The load stream: step load_s of tile load_tile is the next to be asked for.  Wave w brings rows 32 w .. 32 w + 31 of
  // both operand tiles, 8 rows (1 KiB of LDS, in lane order) per instruction; a lane fetches the logical chunk that the
  // swizzle keeps in its slot.
  uint32_t load_tile = 0, load_s = 0;
  uint64_t load_a = 0, load_b = 0;  // uniform: the tile's first row, less BIAS
  uint32_t off_a[4], off_b[4];
  auto load_setup = [&](uint32_t index) {
    const Tile t = tile_at(index);
    load_a = p.a + uint64_t(t.batch) * p.a_batch + uint64_t(t.m0) * p.lda - BIAS;
    load_b = p.b + uint64_t(t.batch) * p.b_batch + uint64_t(t.n0) * p.ldb - BIAS;
#pragma unroll
    for (uint32_t i = 0; i < 4; ++i) {
      const uint32_t r = wave * 32 + 8 * i + (lane >> 3), c = (lane & 7u) ^ ((r >> 1) & 7u);
      const uint32_t ra = t.m0 + r < p.m ? r : p.m - 1 - t.m0, rb = t.n0 + r < p.n ? r : p.n - 1 - t.n0;  // rows past the end repeat the last one
      off_a[i] = ra * p.lda + c * 16 + BIAS - 1024 * i;
      off_b[i] = rb * p.ldb + c * 16 + BIAS - 1024 * i;
    }
  };
  auto load_piece = [&](int piece, uint32_t stage) {
    const uint64_t a = load_a + uint64_t(load_s) * BK, b = load_b + uint64_t(load_s) * BK;
    const uint32_t at = lds0 + stage * STAGE + wave * 4096;
    switch (piece) {
      case 0: load_to_lds<0>(off_a[0], a, at); break;
      case 1: load_to_lds<1024>(off_a[1], a, at); break;
      case 2: load_to_lds<2048>(off_a[2], a, at); break;
      case 3: load_to_lds<3072>(off_a[3], a, at); break;
      case 4: load_to_lds<0>(off_b[0], b, at + B_AT); break;
      case 5: load_to_lds<1024>(off_b[1], b, at + B_AT); break;
      case 6: load_to_lds<2048>(off_b[2], b, at + B_AT); break;
      default: load_to_lds<3072>(off_b[3], b, at + B_AT); break;
    }
  };
  auto load_advance = [&]() {
    if (++load_s == steps) {
      load_s = 0;
      if (++load_tile < mine) load_setup(load_tile);
    }
  };

  // Fragment addresses.  Lane: row l32 of a 32-row block, 32 bytes of k at chunks 4 kk + 2 h and + 1; the swizzle key of
  // the row depends on l32 alone, so one base serves every block (immediate offsets) and the chunk variants are XORs.
  const uint32_t key = (l32 >> 1) & 7u, x0 = l32 * BK + (((2 * h) ^ key) << 4);
  uint32_t at_a[2][2], at_b[2][2];  // [kk][low / high chunk], of stage 0
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const uint32_t x = x0 ^ (kk * 64) ^ (c * 16);
      at_a[kk][c] = x + wm * (64 * BK);
      at_b[kk][c] = x + B_AT + wn * (128 * BK);
    }
  auto fragment = [&](const uint32_t (&at)[2], uint32_t block, uint32_t stage) {
    const V4I lo = *reinterpret_cast<const V4I*>(lds + stage * STAGE + at[0] + block * (32 * BK));
    const V4I hi = *reinterpret_cast<const V4I*>(lds + stage * STAGE + at[1] + block * (32 * BK));
    return V8I{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };

  V16F acc[TM2][TN2];
  auto clear = [&]() {
#pragma unroll
    for (int i = 0; i < TM2; ++i)
#pragma unroll
      for (int j = 0; j < TN2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  };
  clear();
  const auto whole = p.whole();

  // The epilogue of mma_tile's register path, for this wave's 64 x 128 of tile t.
  auto epilogue = [&](const Tile& t) {
    const uint32_t wm0 = t.m0 + wm * 64, wn0 = t.n0 + wn * 128;
#pragma unroll
    for (int j = 0; j < TN2; ++j) {
      float scale[4][4], bias[4][4];  // of this lane's columns wn0 + 32 j + 8 q + 4 h + r
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t n = wn0 + 32 * j + 8 * q + 4 * h;
        p.column_terms(n + 4 <= p.n ? n : p.n - 4, whole, scale[q], bias[q]);
      }
#pragma unroll
      for (int i = 0; i < TM2; ++i) {
        const uint32_t m = wm0 + 32 * i + l32;
        const float rs = p.row_scale(m < p.m ? m : p.m - 1, whole);
        const V16F& v = acc[i][j];
#pragma unroll
        for (int qp = 0; qp < 2; ++qp) {
          uint32_t lo[2], hi[2];  // chunks 2 qp and 2 qp + 1 as two bfloat16 pairs each
#pragma unroll
          for (int e = 0; e < 2; ++e) {
            const int q0 = 2 * qp, q1 = 2 * qp + 1;
            lo[e] = pack_bf16(v[4 * q0 + 2 * e] * (rs * scale[q0][2 * e]) + bias[q0][2 * e],
                              v[4 * q0 + 2 * e + 1] * (rs * scale[q0][2 * e + 1]) + bias[q0][2 * e + 1]);
            hi[e] = pack_bf16(v[4 * q1 + 2 * e] * (rs * scale[q1][2 * e]) + bias[q1][2 * e],
                              v[4 * q1 + 2 * e + 1] * (rs * scale[q1][2 * e + 1]) + bias[q1][2 * e + 1]);
          }
          // lanes 32.. of `lo` change places with lanes ..31 of `hi`: a lane then holds 8 consecutive outputs of its row
          const auto s0 = __builtin_amdgcn_permlane32_swap(lo[0], hi[0], false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(lo[1], hi[1], false, false);
          const uint32_t n = wn0 + 32 * j + 8 * (2 * qp + h);
          if (m < p.m && n + 8 <= p.n) p.store_bf16x8(t.batch, m, n, U4{s0[0], s1[0], s0[1], s1[1]});
        }
      }
    }
  };

  // Prologue: steps 0 and 1 of the stream into stages 0 and 1; the fragments of step 0's first half.
  const uint32_t stream = mine * steps;
  load_setup(0);
#pragma unroll
  for (int c = 0; c < 8; ++c) load_piece(c, 0);
  load_advance();
#pragma unroll
  for (int c = 0; c < 8; ++c) load_piece(c, 1);  // (steps >= 2: a second step always exists)
  load_advance();
  __builtin_amdgcn_s_waitcnt(0x0f70 | 8);  // vmcnt(8): stage 0 has landed
  __syncthreads();
  V8I a_first[2], a_second[2], b_first[TN2], b_second[TN2];  // of the first / second half of k (kk = 0 / 1)
#pragma unroll
  for (int j = 0; j < TN2; ++j) {
    if (j < 2) a_first[j] = fragment(at_a[0], j, 0);
    b_first[j] = fragment(at_b[0], j, 0);
  }

  uint32_t tile = 0, s = 0;
  for (uint32_t t = 0; t < stream; ++t) {
    const uint32_t stage = t & 1u;
    // First half of k: 8 matrix-core instructions, with the reads of the second half's fragments between them.
#pragma unroll
    for (int i = 0; i < TM2; ++i) {
#pragma unroll
      for (int j = 0; j < TN2; ++j) {
        acc[i][j] = mfma_f8_32<FA, FB>(b_first[j], a_first[i], acc[i][j]);
        if (i == 0) {
          if (j == 0) a_second[0] = fragment(at_a[1], 0, stage);
          b_second[j] = fragment(at_b[1], j, stage);
          if (j == TN2 - 1) a_second[1] = fragment(at_a[1], 1, stage);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // Every fragment of this stage is in registers, and this wave's loads of the next stage have landed.
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) and lgkmcnt(0)
    __syncthreads();
    // Second half: the stage just read takes the loads of step t + 2; the other stage gives step t + 1's first fragments.
    const bool more = t + 2 < stream;
#pragma unroll
    for (int i = 0; i < TM2; ++i) {
#pragma unroll
      for (int j = 0; j < TN2; ++j) {
        acc[i][j] = mfma_f8_32<FA, FB>(b_second[j], a_second[i], acc[i][j]);
        if (i == 0) {
          if (more) {
            load_piece(2 * j, stage);
            load_piece(2 * j + 1, stage);
          }
          if (j == 0) a_first[0] = fragment(at_a[0], 0, stage ^ 1u);
          b_first[j] = fragment(at_b[0], j, stage ^ 1u);
          if (j == TN2 - 1) a_first[1] = fragment(at_a[0], 1, stage ^ 1u);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (more) load_advance();
    if (++s == steps) {
      epilogue(tile_at(tile));
      clear();
      s = 0, ++tile;
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // nothing of this workgroup may still be on its way into LDS
}

// Whether mma_stream serves problem p (the caller has checked the operands' alignment).
template <class P>
bool mma_stream_serves(const P& p) {
  return p.k % BK == 0 && p.k >= 2 * BK && p.n % 8 == 0 && p.n >= 8 && p.m >= 1;
}

template <int FA, int FB, class P>
int launch_mma_stream(const P& p, int compute_units, hipStream_t stream, std::string* err, const char* who) {
  constexpr uint32_t lds_bytes = 2 * (256 + 256) * BK;
  auto kernel = mma_stream<FA, FB, P>;
  static bool configured = false;  // guarded by the runtime's stream mutex
  if (!configured) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) {
      (void)hipGetLastError();
      *err = std::string(who) + ": cannot reserve " + std::to_string(lds_bytes) + " bytes of LDS";
      return -1;
    }
    configured = true;
  }
  const uint32_t tiles_m = (p.m + 255) / 256, tiles_n = (p.n + 255) / 256;
  const uint64_t total = uint64_t(tiles_m) * tiles_n * p.batches;
  if (total * (p.k / BK) >= (1ull << 31)) {
    *err = std::string(who) + ": too many tiles";
    return -1;
  }
  const uint64_t resident = (uint64_t(compute_units) + 7) / 8 * 8;
  const uint64_t grid = (total + 7) / 8 * 8 < resident ? (total + 7) / 8 * 8 : resident;
  hipLaunchKernelGGL(kernel, dim3(uint32_t(grid)), dim3(512), lds_bytes, stream, p, tiles_m, tiles_n);
  return 0;
}

}  // namespace
}  // namespace vkt
