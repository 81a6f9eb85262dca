// Calibration kernels for the rooflines: what the memory system and the fp8 matrix cores of this part sustain with
// nothing else in the way.  They compute nothing useful; bench.py times them beside the kernels they bound, so that
// "this launch geometry cannot stream faster than X" and "these operands cannot be multiplied faster than Y" are
// measured figures.  No counterpart in the reference.
//   "probe_read", spec {GEOMETRY}      16-byte non-temporal loads of src[0 .. n*k) in the launch geometry of a product
//                                       kernel: 0 / 1 the int8 GEMV's (2 weight rows per wave, K over 4 / 2 waves of a
//                                       workgroup), 2 the int4 streaming kernel's (a workgroup per 16 columns, 8 loads of
//                                       1 KiB per wave and round, then 32 bytes of scales per lane), 3 a persistent grid
//                                       (a workgroup per compute unit x 8, each wave striding over the whole buffer)
//   "probe_mfma_f8", spec {OPERANDS}   a register-only loop of V_MFMA_F32_32X32X64_F8F6F4 (4 waves per workgroup, 4
//                                       accumulator tiles per wave): 0 all-zero operands, 1 random bits held in the same
//                                       registers throughout, 2 fresh operands for every instruction (made by vector
//                                       operations, no memory at all); dst + 64 / + 72 receive the loop's shader cycles
//                                       and its ticks of the 100 MHz clock (the clock the part held)
//   "probe_delay", spec {}              one wave that waits `iters` microseconds on the constant-rate clock and exits: a
//                                       timing loop queues it first so that the launches behind it are all queued by the
//                                       time the device reaches them (the device, not the host, then sets the pace)
#include "common.h"
#include "kernels.h"

namespace vkt {
namespace {

__global__ __launch_bounds__(64) void probe_delay(uint64_t ticks) {
  const uint64_t start = wall_clock64();
  // (bounded by construction: the clock advances whatever else happens)
  while (wall_clock64() - start < ticks) __builtin_amdgcn_s_sleep(32);
}

__device__ __forceinline__ void sink(uint64_t dst, const U4& acc) {
  // (never true for the buffers bench.py passes; keeps the loads alive)
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345679u) stg<uint32_t>(dst, 1u);
}

template <int COLS, int KSPLIT>
__global__ __launch_bounds__(256) void probe_read_gemv(ProbeParams p) {
  constexpr int GROUPS = 4 / KSPLIT;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, grp = wave / KSPLIT, ks = wave % KSPLIT;
  const uint32_t n0 = (blockIdx.x * GROUPS + grp) * COLS;
  uint64_t row[COLS];
#pragma unroll
  for (int c = 0; c < COLS; ++c) row[c] = p.src + uint64_t(n0 + c < p.n ? n0 + c : p.n - 1) * p.k;
  U4 acc = {0, 0, 0, 0};
  for (uint32_t k = (ks * 64 + lane) * 16; k < p.k; k += 1024 * KSPLIT) {
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc ^= ldg_stream<U4>(row[c] + k);
  }
  sink(p.dst, acc);
}

// n columns in tiles of 16, k in rounds of 4096 values: [tile][round][wave 4][unit 8][lane 64] x 16 bytes of nibbles,
// then [tile][round][wave 4][lane 64] x 32 bytes of scales (blocks of 32 values)
__global__ __launch_bounds__(256) void probe_read_int4(ProbeParams p) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t tiles = (p.n + 15) / 16, rounds = (p.k + 4095) / 4096;
  const uint64_t scale_off = uint64_t(tiles) * rounds * 4 * 8 * 64 * 16;
  U4 acc = {0, 0, 0, 0};
  for (uint32_t round = 0; round < rounds; ++round) {
    const uint64_t base = (uint64_t(blockIdx.x) * rounds + round) * 4 + wave;
    const uint64_t sp = p.src + scale_off + (base * 64 + lane) * 32;
    acc ^= ldg_stream<U4>(sp);
    acc ^= ldg_stream<U4>(sp + 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) acc ^= ldg_stream<U4>(p.src + ((base * 8 + j) * 64 + lane) * 16);
  }
  sink(p.dst, acc);
}

// every wave of the grid takes runs of 8 KiB (8 loads of 1 KiB in flight), striding by the grid
__global__ __launch_bounds__(256) void probe_read_persistent(ProbeParams p) {
  const uint64_t bytes = uint64_t(p.n) * p.k, waves = uint64_t(gridDim.x) * 4;
  const uint64_t wave = uint64_t(blockIdx.x) * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  U4 acc = {0, 0, 0, 0};
  for (uint64_t at = wave * 8192; at + 8192 <= bytes; at += waves * 8192) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc ^= ldg_stream<U4>(p.src + at + j * 1024 + lane * 16);
  }
  sink(p.dst, acc);
}

using V8I = int __attribute__((ext_vector_type(8)));
using V16F = float __attribute__((ext_vector_type(16)));

template <int OPERANDS>
__global__ __launch_bounds__(256) void probe_mfma_f8(ProbeParams p) {
  // a 2 x 2 arrangement of 32 x 32 tiles: two row fragments, two column fragments of 32 bytes per lane
  V8I a[2], b[2];
  const uint32_t seed = (blockIdx.x * 256 + threadIdx.x) * 2654435761u + 12345u;
#pragma unroll
  for (int f = 0; f < 2; ++f)
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      // (the mask clears the lowest mantissa bit of every byte: no NaN codes among the random operands)
      a[f][r] = OPERANDS == 0 ? 0 : int(((seed + 97u * r + 13u * f) * 1664525u + 1013904223u) & 0xfefefefeu);
      b[f][r] = OPERANDS == 0 ? 0 : int(((seed + 89u * r + 17u * f) * 22695477u + 1u) & 0xfefefefeu);
    }
  V16F acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const uint64_t cycles0 = clock64(), ticks0 = wall_clock64();
  for (uint32_t it = 0; it < p.iters; ++it) {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        if constexpr (OPERANDS == 2) {
          // fresh bits for this instruction: about half the bits of half of each fragment's registers flip (one
          // exclusive-or per register, 8 vector operations per matrix-core instruction: more would make the loop
          // wait for the vector unit; the masks keep the lowest mantissa bit of every byte clear: no NaN code appears)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            a[i][2 * r + (j & 1)] ^= int(0x5ac6963au + 0x02040810u * uint32_t(r) + 0x20406080u * uint32_t(j)) & int(0xfefefefeu);
            b[j][2 * r + (i & 1)] ^= int(0xc6a4d2b8u + 0x04081020u * uint32_t(r) + 0x10204080u * uint32_t(i)) & int(0xfefefefeu);
          }
        }
        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(b[j], a[i], acc[i][j], 0, 0, 0, 0, 0, 0);
      }
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  if (s == 1.2345e-30f) stg<float>(p.dst, s);
  // the clock the loop ran at: shader cycles and ticks of the constant 100 MHz clock, first wave of the first workgroup
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    stg<uint64_t>(p.dst + 64, clock64() - cycles0);
    stg<uint64_t>(p.dst + 72, wall_clock64() - ticks0);
  }
}

}  // namespace

int launch_probe_read(const ProbeParams& p, uint32_t geometry, const Machine& mc, hipStream_t stream, std::string* err) {
  if (!p.src || !p.dst || p.n == 0 || p.k == 0 || (p.src & 15) || p.k % 16) {
    *err = "probe_read: null or unaligned address, or k not a multiple of 16";
    return -1;
  }
  // geometry 2 walks the int4 streaming side-car of an [n, k] weight in whole tiles of 16 columns and whole rounds of
  // 4096 values: src holds vkt_qmm4c_bytes(n, k, 32) bytes, of which (n / 16) (k / 4096) 40960 are read
  if (geometry == 2 && (p.n % 16 != 0 || p.k % 4096 != 0)) {
    *err = "probe_read: GEOMETRY 2 takes n a multiple of 16 and k a multiple of 4096";
    return -1;
  }
  switch (geometry) {
    case 0: hipLaunchKernelGGL((probe_read_gemv<2, 4>), dim3((p.n + 1) / 2), dim3(256), 0, stream, p); break;
    case 1: hipLaunchKernelGGL((probe_read_gemv<2, 2>), dim3((p.n + 3) / 4), dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL(probe_read_int4, dim3((p.n + 15) / 16), dim3(256), 0, stream, p); break;
    case 3: hipLaunchKernelGGL(probe_read_persistent, dim3(uint32_t(mc.compute_units) * 8), dim3(256), 0, stream, p); break;
    default: *err = "probe_read: GEOMETRY must be 0 to 3"; return -1;
  }
  if (hipGetLastError() != hipSuccess) {
    *err = "probe_read: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_probe_delay(const ProbeParams& p, hipStream_t stream, std::string* err) {
  if (p.iters > 100000) {
    *err = "probe_delay: at most 100000 microseconds";
    return -1;
  }
  int rate_khz = 100000;  // the constant-rate clock: 100 MHz unless the device says otherwise
  int dev = 0;
  if (hipGetDevice(&dev) == hipSuccess) (void)hipDeviceGetAttribute(&rate_khz, hipDeviceAttributeWallClockRate, dev);
  if (rate_khz <= 0) rate_khz = 100000;
  hipLaunchKernelGGL(probe_delay, dim3(1), dim3(64), 0, stream, uint64_t(p.iters) * uint64_t(rate_khz) / 1000);
  if (hipGetLastError() != hipSuccess) {
    *err = "probe_delay: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_probe_mfma(const ProbeParams& p, uint32_t operands, const Machine& mc, hipStream_t stream, std::string* err) {
  // (the loop's clock counts are stored at dst + 64 and dst + 72: dst holds at least 80 bytes)
  if (!p.dst || (p.dst & 7) || p.iters == 0) {
    *err = "probe_mfma_f8: null or unaligned address (dst: 80 bytes, 8-byte aligned), or no iterations";
    return -1;
  }
  const dim3 grid(uint32_t(mc.compute_units));
  switch (operands) {
    case 0: hipLaunchKernelGGL(probe_mfma_f8<0>, grid, dim3(256), 0, stream, p); break;
    case 1: hipLaunchKernelGGL(probe_mfma_f8<1>, grid, dim3(256), 0, stream, p); break;
    case 2: hipLaunchKernelGGL(probe_mfma_f8<2>, grid, dim3(256), 0, stream, p); break;
    default: *err = "probe_mfma_f8: OPERANDS must be 0, 1 or 2"; return -1;
  }
  if (hipGetLastError() != hipSuccess) {
    *err = "probe_mfma_f8: kernel launch failed";
    return -1;
  }
  return 0;
}

}  // namespace vkt
