// The matrix-core kernel for large products with 16-bit outputs (float8 operands for _scaled_mm, 16-bit operands for
// the matrix product and the many-row int8 product): 256 x 256 tiles of A [m, k] x B [n, k]^T (rows of k contiguous
// bytes, as in mma_tile.h) on 8 waves of 64 x 128, K in steps of 128 bytes through two LDS stages of 64 KiB.
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
// (4 waves of 128 x 128, one per SIMD with the accumulators in the second half of the register file, would read two
// thirds of the fragment bytes per instruction.  Tried: correct, but the compiler keeps fragments in the
// accumulators' half of the file and spills both inside the loop, 860 bytes of scratch and ten times slower.)
// The problem type P supplies the operands as mma_tile's does (a, b, lda, ldb in bytes, m, n, k in bytes, batches,
// a_batch, b_batch) and the epilogue of 4 consecutive outputs of a row, as one lane holds them in its accumulators:
//   whole()                                            per-launch constants
//   rows(batch, m, whole)                              per-lane constants of row m
//   columns4(batch, n, whole)                          per-lane constants of columns n .. n + 3
//   finish4(batch, m, n, sums[4], rows, columns4, whole, values[4])   the outputs as float32
//   pack4(values[4], whole, out[2])                    converted: two words of 16-bit outputs, or one of 8-bit
//   narrow(whole)                                      whether outputs are 8-bit
//   store8(batch, m, n, U4) / store8_narrow(batch, m, n, U2)     8 consecutive outputs of a row
// k a multiple of 128 bytes and at least 256, n a multiple of 8, 16-byte aligned operand rows.
#pragma once

#include "limits.h"
#include "mma_tile.h"

namespace vkt {
namespace {

// One LDS-direct load of 16 bytes per lane: global address `base` + `offset` + OFF, LDS address `lds_at` + OFF + 16 * lane.
// (M0 is written in every statement that uses it and by nothing else in this kernel: no other instruction the compiler
// emits here reads it, and a clobber of a reserved register is not something the compiler honours anyway.)
template <int OFF>
__device__ __forceinline__ void load_to_lds(uint32_t offset, uint64_t base, uint32_t lds_at) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3" ::"v"(offset), "s"(base), "s"(lds_at), "i"(OFF)
               : "memory");
}

template <int FA, int FB, int MATH, class P>
__global__ __launch_bounds__(512) void mma_stream(P p, uint32_t tiles_m, uint32_t tiles_n) {
  static_assert(!P::kTransA && !P::kTransB, "operands contiguous along k");
  constexpr int WM = 4;  // waves along m: 8 waves of 64 x 128
  constexpr uint32_t BM = 256, BN = 256, STAGE = (BM + BN) * BK, B_AT = BM * BK;
  constexpr int WAVES = WM * 2, TM2 = 8 / WM, TN2 = 4;  // a wave's (256 / WM) x 128 as 32 x 32 matrix-core tiles
  constexpr int ROWS = 256 / WAVES, PER = ROWS / 8;    // rows of each operand tile a wave brings; loads per operand and step
  constexpr int NM = TM2 * TN2;                        // matrix-core tiles per half step
  constexpr uint32_t BIAS = 3072;  // keeps the per-lane offsets non-negative (they carry -1024 (i % 4) for load i)
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

  // The load stream: step load_s of tile load_tile is the next to be asked for.  Wave w brings rows ROWS w .. + ROWS - 1
  // of both operand tiles, 8 rows (1 KiB of LDS, in lane order) per instruction; a lane fetches the logical chunk that
  // the swizzle keeps in its slot.
  uint32_t load_tile = 0, load_s = 0;
  uint64_t load_a = 0, load_b = 0;  // uniform: the tile's first row, less BIAS
  uint32_t off_a[PER], off_b[PER];
  auto load_setup = [&](uint32_t index) {
    const Tile t = tile_at(index);
    load_a = p.a + uint64_t(t.batch) * p.a_batch + uint64_t(t.m0) * p.lda - BIAS;
    load_b = p.b + uint64_t(t.batch) * p.b_batch + uint64_t(t.n0) * p.ldb - BIAS;
    // (The lane's rows and chunks are worked out anew for every tile: as values that do not change in the loop the
    // compiler computes them once, finds no register to keep them in, and reloads them here from scratch memory,
    // each reload waiting for every load into LDS in flight: 1.5 us per tile.)
    // (the lane number likewise: counted anew, two instructions, rather than kept or reloaded)
    uint32_t ln;
    asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(ln));
#pragma unroll
    for (uint32_t i = 0; i < uint32_t(PER); ++i) {
      const uint32_t r = wave * ROWS + 8 * i + (ln >> 3), c = (ln & 7u) ^ ((r >> 1) & 7u);
      const uint32_t ra = t.m0 + r < p.m ? r : p.m - 1 - t.m0, rb = t.n0 + r < p.n ? r : p.n - 1 - t.n0;  // rows past the end repeat the last one
      off_a[i] = ra * p.lda + c * 16 + BIAS - 1024 * (i & 3u);
      off_b[i] = rb * p.ldb + c * 16 + BIAS - 1024 * (i & 3u);
    }
  };
  auto load_piece = [&](int piece, uint32_t stage) {  // pieces 0 .. PER - 1: the first operand's, PER .. 2 PER - 1: the second's
    const bool second = piece >= PER;
    const int i = second ? piece - PER : piece;
    const uint64_t base = (second ? load_b : load_a) + uint64_t(load_s) * BK;
    const uint32_t at = lds0 + stage * STAGE + (second ? B_AT : 0u) + wave * (ROWS * BK) + uint32_t(i >> 2) * 4096;
    const uint32_t offset = second ? off_b[i < PER ? i : 0] : off_a[i < PER ? i : 0];
    switch (i & 3) {
      case 0: load_to_lds<0>(offset, base, at); break;
      case 1: load_to_lds<1024>(offset, base, at); break;
      case 2: load_to_lds<2048>(offset, base, at); break;
      default: load_to_lds<3072>(offset, base, at); break;
    }
  };
  // (The rare paths of the loop, a new tile for the loads and the epilogue, end by waiting for what they have asked
  // for themselves.  Scalar and LDS results share a counter: with scalar loads possibly pending where the paths meet
  // again the compiler would wait for EVERY fragment read before the next step's first matrix-core instruction.  The
  // epilogue waits for its vector loads and stores as well, which the middle of the next step would do anyway: a
  // vector load that the compiler believes pending there costs a wait at the head of every step, for the loads into
  // LDS that still have half a step to land.)
  auto load_advance = [&]() {
    if (++load_s == steps) {
      load_s = 0;
      if (++load_tile < mine) load_setup(load_tile);
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    }
  };

  // Fragment addresses.  Lane: row l32 of a 32-row block, 32 bytes of k at chunks 4 kk + 2 h and + 1; the swizzle key of
  // the row depends on l32 alone, so one base serves every block (immediate offsets) and the chunk variants are XORs.
  const uint32_t key = (l32 >> 1) & 7u, x0 = l32 * BK + (((2 * h) ^ key) << 4);
  // (The second operand's addresses differ from the first's by the same amount in every lane: one set of registers.)
  uint32_t at[2][2];  // [kk][low / high chunk]: the first operand's, of stage 0
#pragma unroll
  for (int kk = 0; kk < 2; ++kk)
#pragma unroll
    for (int c = 0; c < 2; ++c) at[kk][c] = (x0 ^ (kk * 64) ^ (c * 16)) + wm * (TM2 * 32 * BK);
  const uint32_t a_to_b = B_AT + wn * (128 * BK) - wm * (TM2 * 32 * BK);
  auto fragment = [&](const uint32_t (&at)[2], uint32_t uniform) {
    const V4I lo = *reinterpret_cast<const V4I*>(lds + uniform + at[0]);
    const V4I hi = *reinterpret_cast<const V4I*>(lds + uniform + at[1]);
    return V8I{lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
  };
  auto fragment_a = [&](int kk, uint32_t block, uint32_t stage) { return fragment(at[kk], stage * STAGE + block * (32 * BK)); };
  auto fragment_b = [&](int kk, uint32_t block, uint32_t stage) { return fragment(at[kk], stage * STAGE + a_to_b + block * (32 * BK)); };
  auto multiply = [&](const V8I& b, const V8I& a, const V16F& c) {
    if constexpr (MATH == kMathFp8) {
      return mfma_f8_32<FA, FB>(b, a, c);
    } else {  // 16-bit values: a fragment's 32 bytes are two operands of 8 values
      return mfma_16bit<MATH>(half_of(b, 1), half_of(a, 1), mfma_16bit<MATH>(half_of(b, 0), half_of(a, 0), c));
    }
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

  // The epilogue, straight from the accumulators.  A 32 x 32 matrix-core tile leaves lane l with row l % 32 and, for
  // q = 0..3, columns 8 q + 4 (l / 32) .. + 3.  A lane finishes and packs its own values; three exchanges between lanes
  // (32, 16 and 8 apart: two swap instructions and a row rotation) then bring the 128 bytes that two column blocks
  // side by side hold of a row into 8 neighbouring lanes, so that a store instruction writes 8 whole 128-byte lines.
  // What the epilogue costs is the time its stores take to drain (every workgroup stores its tile at about the same
  // time, with the matrix cores idle).  Stores that write 32 or 64 bytes of each of their rows take as long, in any
  // order tried, but put 1.5 times the output's bytes on the way to memory (counted: 201 MiB for the 128 MiB of
  // 8192 x 8192 bfloat16 outputs); with whole lines the count is the output's size.  Non-temporal stores are 1.5 times
  // slower, and waiting after every few stores, or starting the workgroups a few microseconds apart, only costs.
  auto epilogue = [&](const Tile& t) {
    const uint32_t wm0 = t.m0 + wm * (TM2 * 32), wn0 = t.n0 + wn * 128;
    typename P::Rows rows[TM2];
#pragma unroll
    for (int i = 0; i < TM2; ++i) {
      const uint32_t m = wm0 + 32 * i + l32;
      rows[i] = p.rows(t.batch, m < p.m ? m : p.m - 1, whole);
    }
    const bool narrow = p.narrow(whole);
    // One 32 x 32 tile, finished, packed and exchanged twice: [0] the 8 outputs (16-bit: 4 words, 8-bit: 2) at
    // row lane % 16, [1] at row 16 + lane % 16, both of chunk {0, 2, 1, 3}[lane / 16] of the tile's four chunks of 8
    // columns.  (First exchange, lanes 32 apart: the two halves of a chunk meet.  Second, lanes 16 apart: the lanes of
    // rows 16 .. 31 give their first chunk for the second chunk of the lanes 16 below.)
    struct Packed {
      uint32_t w[2][4];
    };
    auto packed_tile = [&](int i, int j, const uint32_t (&first_column)[4], const typename P::Columns4 (&columns)[4]) {
      const uint32_t m = wm0 + 32 * i + l32, row = m < p.m ? m : p.m - 1;
      const V16F& v = acc[i][j];
      Packed out;
#pragma unroll
      for (int qp = 0; qp < 2; ++qp) {
        const float first[4] = {v[8 * qp], v[8 * qp + 1], v[8 * qp + 2], v[8 * qp + 3]};
        const float second[4] = {v[8 * qp + 4], v[8 * qp + 5], v[8 * qp + 6], v[8 * qp + 7]};
        float f0[4], f1[4];
        p.finish4(t.batch, row, first_column[2 * qp], first, rows[i], columns[2 * qp], whole, f0);
        p.finish4(t.batch, row, first_column[2 * qp + 1], second, rows[i], columns[2 * qp + 1], whole, f1);
        uint32_t lo[2] = {0, 0}, hi[2] = {0, 0};
        p.pack4(f0, whole, lo);
        p.pack4(f1, whole, hi);
        const auto s0 = __builtin_amdgcn_permlane32_swap(lo[0], hi[0], false, false);
        const auto s1 = __builtin_amdgcn_permlane32_swap(lo[1], hi[1], false, false);
        out.w[qp][0] = s0[0], out.w[qp][1] = narrow ? s0[1] : s1[0], out.w[qp][2] = s0[1], out.w[qp][3] = s1[1];
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const auto x = __builtin_amdgcn_permlane16_swap(out.w[0][e], out.w[1][e], false, false);
        out.w[0][e] = x[0], out.w[1][e] = x[1];
      }
      return out;
    };
    // Two column blocks side by side are 128 bytes of a row of 16-bit outputs.  A third exchange, between lanes 8 apart
    // (lanes 8 .. 15 of every 16 give their left block's words for the right block's of the lanes 8 below), leaves a
    // store instruction with whole 128-byte lines: rows lane % 8 (+ 8, 16, 24 for the four stores), left or right block
    // by lane / 8 % 2, chunk by lane / 16.  (Stores of 32 or 64 bytes per row wrote 1.5 times the output's bytes to
    // memory, whatever their order: counted.)
    const bool upper8 = (lane & 8u) != 0;
    auto exchange8 = [&](uint32_t& left, uint32_t& right) {
      const uint32_t give = upper8 ? left : right;
      const uint32_t got = uint32_t(__builtin_amdgcn_update_dpp(0, int(give), 0x128 /* row_ror:8 */, 0xf, 0xf, false));
      left = upper8 ? got : left;
      right = upper8 ? right : got;
    };
#pragma unroll
    for (int jp = 0; jp < TN2 / 2; ++jp) {
      Packed left[TM2];
#pragma unroll
      for (int jj = 0; jj < 2; ++jj) {
        const int j = 2 * jp + jj;
        uint32_t first_column[4];  // of this lane's four columns in chunk q of column block j (inside the matrix)
        typename P::Columns4 columns[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t n = wn0 + 32 * j + 8 * q + 4 * h;
          first_column[q] = n + 4 <= p.n ? n : p.n - 4;
          columns[q] = p.columns4(t.batch, first_column[q], whole);
        }
#pragma unroll
        for (int i = 0; i < TM2; ++i) {
          if (jj == 0) {
            left[i] = packed_tile(i, j, first_column, columns);
            continue;
          }
          Packed right = packed_tile(i, j, first_column, columns);
#pragma unroll
          for (int half = 0; half < 2; ++half)
#pragma unroll
            for (int e = 0; e < 4; ++e) exchange8(left[i].w[half][e], right.w[half][e]);
          const uint32_t n = wn0 + 32 * (2 * jp + ((lane >> 3) & 1u)) + 8 * (2 * ((lane >> 4) & 1u) + h);
#pragma unroll
          for (int part = 0; part < 4; ++part) {  // rows lane % 8 + 8 part: left[half = 0], right[0], left[1], right[1]
            const uint32_t mm = wm0 + 32 * i + 8 * part + (lane & 7u);
            const uint32_t(&w)[4] = (part & 1) ? right.w[part >> 1] : left[i].w[part >> 1];
            const bool inside = mm < p.m && n + 8 <= p.n;
            if (!narrow) {
              if (inside) p.store8(t.batch, mm, n, U4{w[0], w[1], w[2], w[3]});
            } else {
              if (inside) p.store8_narrow(t.batch, mm, n, U2{w[0], w[1]});
            }
          }
        }
      }
    }
  };

  // Prologue: steps 0 and 1 of the stream into stages 0 and 1; the fragments of step 0's first half.
  const uint32_t stream = mine * steps;
  load_setup(0);
#pragma unroll
  for (int c = 0; c < 2 * PER; ++c) load_piece(c, 0);
  load_advance();
#pragma unroll
  for (int c = 0; c < 2 * PER; ++c) load_piece(c, 1);  // (steps >= 2: a second step always exists)
  load_advance();
  __builtin_amdgcn_s_waitcnt(0x0f70 | (2 * PER));  // vmcnt(2 PER): stage 0 has landed
  __syncthreads();
  V8I a_first[TM2], a_second[TM2], b_first[TN2], b_second[TN2];  // of the first / second half of k (kk = 0 / 1)
  // the fragments of a half step, read between the first TN2 matrix-core instructions of the half step before, in the
  // order they are needed: with instruction 0 row block 0 and column block 0, with instruction j column block j, with
  // the last of them the other row blocks (all reads are out within the first half of the instructions, so the wait
  // for them at the barrier finds them done)
  auto read_fragments = [&](int n, V8I (&a)[TM2], V8I (&b)[TN2], int kk, uint32_t stage) {
    if (n >= TN2) return;
    if (n == 0) a[0] = fragment_a(kk, 0, stage);
    b[n < TN2 ? n : 0] = fragment_b(kk, n, stage);
    if (n == TN2 - 1) {
#pragma unroll
      for (int i = 1; i < TM2; ++i) a[i] = fragment_a(kk, i, stage);
    }
  };
#pragma unroll
  for (int n = 0; n < TN2; ++n) read_fragments(n, a_first, b_first, 0, 0);

  uint32_t tile = 0, s = 0;
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): (as above: nothing scalar pending on the way into the loop either)
  for (uint32_t t = 0; t < stream; ++t) {
    const uint32_t stage = t & 1u;
    // First half of k, with the reads of the second half's fragments between the matrix-core instructions.
#pragma unroll
    for (int n = 0; n < NM; ++n) {
      const int i = n / TN2, j = n % TN2;
      acc[i][j] = multiply(b_first[j], a_first[i], acc[i][j]);
      read_fragments(n, a_second, b_second, 1, stage);
      __builtin_amdgcn_sched_barrier(0);
    }
    // Every fragment of this stage is in registers, and this wave's loads of the next stage have landed.
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) and lgkmcnt(0)
    __syncthreads();
    // Second half: the stage just read takes the loads of step t + 2; the other stage gives step t + 1's first fragments.
    const bool more = t + 2 < stream;
#pragma unroll
    for (int n = 0; n < NM; ++n) {
      const int i = n / TN2, j = n % TN2;
      acc[i][j] = multiply(b_second[j], a_second[i], acc[i][j]);
      if (n < PER && more) {
        load_piece(2 * n, stage);
        load_piece(2 * n + 1, stage);
      }
      read_fragments(n, a_first, b_first, 0, stage ^ 1u);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) load_advance();
    if (++s == steps) {
      epilogue(tile_at(tile));
      clear();
      s = 0, ++tile;
      __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) and lgkmcnt(0)
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // nothing of this workgroup may still be on its way into LDS
}

// Whether mma_stream serves problem p (the caller has checked the operands' alignment).
template <class P>
bool mma_stream_serves(const P& p) {
  return p.k % BK == 0 && p.k >= 2 * BK && p.n % 8 == 0 && p.n >= 8 && p.m >= 1 && mma_stream_strides_ok(p.lda, p.ldb);
}

template <int FA, int FB, int MATH, class P>
int launch_mma_stream(const P& p, int compute_units, hipStream_t stream, std::string* err, const char* who) {
  constexpr uint32_t lds_bytes = 2 * (256 + 256) * BK;
  auto kernel = mma_stream<FA, FB, MATH, P>;
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
