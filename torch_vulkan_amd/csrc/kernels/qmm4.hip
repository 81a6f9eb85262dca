// aten::_dyn_quant_matmul_4bit on gfx950, bit for bit as the reference computes it
// (crates/vkcore/shaders/qmm4.slang; host side crates/pyvk/csrc/quant.cpp:146-204):
//   phase 0  each input row quantised to int8 (asymmetric; scale = 255 / range correctly
//            rounded, zero point rounded half-to-even, values rounded half-away)
//   phase 1  per block of `bs` values of k, in order: the exact int32 sum of
//            (q - zp) * (nibble - 8), converted and multiplied by the block's float32 scale,
//            added to a float32 accumulator (the first block assigns); then * 1/scale_row,
//            + bias, clamp to the finite range, store (bfloat16 by truncation).
// Every float32 operation below is a single IEEE operation: this file is compiled with
// contraction off, '/' is HIP's correctly rounded division, and nothing is reassociated.
// Integer sums are exact, so they are free to be reordered, and that is where the speed
// comes from.
//
// Two families behind the C ABI:
//   "qmm4_*"   the reference's parameter block and buffers as they are (int32 q, the
//              float32-expanded packed vector: 4 bytes of traffic per byte of nibbles).
//   "qmm4c_*"  the streaming path.  "qmm4c_pack" rewrites the packed vector once into a
//              compact side-car (two nibbles per byte, 16 bytes per lane per load,
//              laid out so that every load of a wave is 1 KiB contiguous); phase 0 writes
//              int8 activations in the byte order v_dot4 wants plus per-unit sums;
//              phase 1 is an HBM stream over the side-car:
//                - a wave owns 4 output columns, one per DPP row of 16 lanes; the 16 lanes
//                  of a row split K into runs of 8 units (a unit = 32 values of k = one
//                  16-byte load);
//                - nibbles stay unsigned: sum (q+nzp)(nib-8) = dot(q,nib) - 8 sum(q)
//                  + nzp (sum(nib) - 8*32), all v_dot4_i32_i8 and integer adds;
//                - the float32 block terms must be added in block order, so the lanes of a
//                  row pass the running sum along with DPP row rotates: 16 short phases per
//                  round of 128 units, no LDS, no atomics.
#pragma clang fp contract(off)

#include "common.h"
#include "kernels.h"

namespace vkt {
namespace {

constexpr int kUnit = 32;          // values of k per 16-byte load of nibbles
constexpr int kUnitsPerLane = 8;   // units a lane handles per round
constexpr int kRoundUnits = 128;   // 16 lanes * 8 units
constexpr int kTileCols = 4;       // output columns per wave

__device__ __forceinline__ float round_away(float x) {  // std::round, qmm4.slang:112-118
  float t = truncf(x);
  if (fabsf(x - t) >= 0.5f) t += x < 0.0f ? -1.0f : 1.0f;
  return t;
}

struct RowQuant {
  float scale, recip;
  int izp;
};

// qmm4.slang:153-171 on every lane (deterministic, so no broadcast is needed).
__device__ __forceinline__ RowQuant row_quant(float mn, float mx, bool groupwise) {
  const float qmin = -128.0f, qmax = 127.0f;
  const float rmin = fminf(0.0f, mn), rmax = fmaxf(0.0f, mx);
  RowQuant r;
  r.scale = rmin == rmax ? 1.0f : (qmax - qmin) / (rmax - rmin);
  r.recip = r.scale != 0.0f ? 1.0f / r.scale : 0.0f;
  const float dmin = rmin * r.scale, dmax = rmax * r.scale;
  const float err = groupwise ? ((qmin + dmin) + qmax) + dmax : (qmin + dmin) + (qmax + dmax);
  float zp = err > 0.0f ? qmin - dmin : qmax - dmax;
  zp = fminf(fmaxf(zp, qmin), qmax);
  r.izp = int(rintf(zp));  // half to even
  return r;
}

__device__ __forceinline__ int quantise(float v, const RowQuant& r) {
  int q = int(round_away(v * r.scale)) + r.izp;
  return q < -128 ? -128 : (q > 127 ? 127 : q);
}

// Row range over a workgroup of 256 threads.
template <class T>
__device__ __forceinline__ void row_range(uint64_t row, uint32_t k, float* mn_out, float* mx_out) {
  constexpr uint64_t item = sizeof(typename T::storage);
  __shared__ float smin[4], smax[4];
  float mn = 3.40282347e38f, mx = -3.40282347e38f;
  for (uint32_t i = threadIdx.x; i < k; i += 256) {
    const float v = load_f32<T>(row + i * item);
    mn = fminf(mn, v);
    mx = fmaxf(mx, v);
  }
  mn = wave_min(mn);
  mx = wave_max(mx);
  if ((threadIdx.x & 63) == 0) smin[threadIdx.x >> 6] = mn, smax[threadIdx.x >> 6] = mx;
  __syncthreads();
  *mn_out = fminf(fminf(smin[0], smin[1]), fminf(smin[2], smin[3]));
  *mx_out = fmaxf(fmaxf(smax[0], smax[1]), fmaxf(smax[2], smax[3]));
}

// ------------------------------------------------------------------ reference-layout path

// Phase 0, one workgroup per row: q int32 [m,k], rows[2m] = bits(1/scale), rows[2m+1] = -zp.
template <class T>
__global__ __launch_bounds__(256) void qmm4_rowquant(Q4Params p, uint32_t groupwise) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const uint32_t m = blockIdx.x;
  const uint64_t row = p.inp + uint64_t(m) * p.k * item;
  float mn, mx;
  row_range<T>(row, p.k, &mn, &mx);
  const RowQuant rq = row_quant(mn, mx, groupwise != 0);
  if (threadIdx.x == 0) {
    stg<uint32_t>(p.rows + 8ull * m, f32_bits(rq.recip));
    stg<int32_t>(p.rows + 8ull * m + 4, -rq.izp);
  }
  for (uint32_t i = threadIdx.x; i < p.k; i += 256)
    stg<int32_t>(p.q + (uint64_t(m) * p.k + i) * 4, quantise(load_f32<T>(row + i * item), rq));
}

template <class T>
__device__ __forceinline__ void finish_store(uint64_t out, float acc, float recip, bool has_bias, float bias) {
  acc = acc * recip;
  if (has_bias) acc = acc + bias;
  const float hi = T::dtype == VKT_BF16 ? 3.38953139e38f : 3.40282347e38f;
  acc = acc < -hi ? -hi : acc;  // NaN passes (qmm4.slang:236-242)
  acc = hi < acc ? hi : acc;
  if constexpr (T::dtype == VKT_BF16) stg<uint16_t>(out, uint16_t(f32_bits(acc) >> 16));  // truncation (:244)
  else stg<float>(out, acc);
}

// Phase 1 over the float32-expanded packed vector: one thread per output, 64 consecutive
// columns per wave.
template <class T>
__global__ __launch_bounds__(256) void qmm4_matmul_expanded(Q4Params p) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const uint32_t n = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (n >= p.n) return;
  const uint32_t rstride = (p.k + 1) / 2, nblocks = (p.k + p.bs - 1) / p.bs;
  const uint64_t wcount = uint64_t(p.n) * p.k / 2;
  const int nzp = ldg<int32_t>(p.rows + 8ull * m + 4);
  const uint64_t qrow = p.q + uint64_t(m) * p.k * 4, wrow = p.packed + uint64_t(n) * rstride * 4;
  float acc = 0.0f;
  for (uint32_t blk = 0; blk < nblocks; ++blk) {
    const uint32_t k0 = blk * p.bs, k1 = k0 + p.bs < p.k ? k0 + p.bs : p.k;
    int iacc = 0;
    for (uint32_t k = k0; k < k1; ++k) {
      const uint32_t byte = uint32_t(ldg<float>(wrow + (k / 2) * 4ull));
      const int w = int((byte >> (4 * (k & 1))) & 15u) - 8;
      iacc += (ldg<int32_t>(qrow + k * 4ull) + nzp) * w;
    }
    const float t = float(iacc) * ldg<float>(p.packed + (wcount + uint64_t(n) * nblocks + blk) * 4);
    acc = blk == 0 ? t : acc + t;
  }
  const float recip = bits_f32(ldg<uint32_t>(p.rows + 8ull * m));
  const float bias = p.has_bias ? ldg<float>(p.packed + (wcount + uint64_t(p.n) * nblocks + n) * 4) : 0.0f;
  finish_store<T>(p.out + (uint64_t(m) * p.n + n) * item, acc, recip, p.has_bias != 0, bias);
}

// ------------------------------------------------------------------ compact (streaming) path

struct CompactLayout {
  uint32_t nunits, rounds, tiles, upb;  // units per block (0: channelwise)
  uint64_t nib_bytes, scale_off, scale_bytes, bias_off, total;
  uint32_t kpad;  // values of k per activation row in the scratch (rounds * 4096)
};

__host__ __device__ inline bool compact_layout(uint32_t n, uint32_t k, uint32_t bs, CompactLayout* L) {
  if (n == 0 || k == 0 || bs == 0) return false;
  const bool channelwise = bs == k;
  if (!channelwise && !(bs == 32 || bs == 64 || bs == 128 || bs == 256)) return false;
  if (!channelwise && k % bs != 0) return false;
  L->nunits = (k + kUnit - 1) / kUnit;
  L->rounds = (L->nunits + kRoundUnits - 1) / kRoundUnits;
  L->tiles = (n + kTileCols - 1) / kTileCols;
  L->upb = channelwise ? 0 : bs / kUnit;
  L->nib_bytes = uint64_t(L->tiles) * L->rounds * kUnitsPerLane * 64 * 16;
  L->scale_off = L->nib_bytes;
  L->scale_bytes = channelwise ? round_up_u64(uint64_t(n) * 4, 256)
                               : uint64_t(L->tiles) * L->rounds * (kUnitsPerLane / L->upb) * 64 * 4;
  L->bias_off = L->scale_off + L->scale_bytes;
  L->total = L->bias_off + round_up_u64(uint64_t(n) * 4, 256);
  L->kpad = L->rounds * kRoundUnits * kUnit;
  return true;
}

// One thread per 16-byte unit of the side-car (and, in the same grid, per scale slot).
__global__ __launch_bounds__(256) void qmm4c_pack_kernel(Q4PackParams p, CompactLayout L) {
  const uint32_t rstride = (p.k + 1) / 2, nblocks = (p.k + p.bs - 1) / p.bs;
  const uint64_t wcount = uint64_t(p.n) * p.k / 2;
  const uint64_t slots = L.nib_bytes / 16;
  const uint64_t id = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (id < slots) {
    const uint32_t lane = id & 63, j = (id >> 6) % kUnitsPerLane;
    const uint64_t tr = id / (64 * kUnitsPerLane);
    const uint32_t round = tr % L.rounds, tile = tr / L.rounds;
    const uint32_t n = tile * kTileCols + (lane >> 4), unit = round * kRoundUnits + (lane & 15) * kUnitsPerLane + j;
    U4 out;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte_index = unit * 16 + d * 4 + b;
        uint32_t byte = 0x88;  // weight 0
        if (n < p.n && byte_index < rstride) {
          byte = uint32_t(ldg<float>(p.packed + (uint64_t(n) * rstride + byte_index) * 4)) & 0xffu;
          // K odd: the last byte's high nibble lies beyond k (weight 0)
          if ((p.k & 1) && byte_index == rstride - 1) byte = (byte & 0x0f) | 0x80;
        }
        word |= byte << (8 * b);
      }
      out[d] = word;
    }
    stg<U4>(p.compact + id * 16, out);
    return;
  }
  uint64_t sid = id - slots;
  if (L.upb != 0) {
    const uint32_t bpl = kUnitsPerLane / L.upb;
    const uint64_t sslots = L.scale_bytes / 4;
    if (sid < sslots) {
      const uint32_t lane = sid & 63, jb = (sid >> 6) % bpl;
      const uint64_t tr = sid / (64 * bpl);
      const uint32_t round = tr % L.rounds, tile = tr / L.rounds;
      const uint32_t n = tile * kTileCols + (lane >> 4);
      const uint32_t blk = (round * kRoundUnits + (lane & 15) * kUnitsPerLane) / L.upb + jb;
      float s = 0.0f;
      if (n < p.n && blk < nblocks) s = ldg<float>(p.packed + (wcount + uint64_t(n) * nblocks + blk) * 4);
      stg<float>(p.compact + L.scale_off + sid * 4, s);
      return;
    }
    sid -= sslots;
  } else {
    if (sid < p.n) {
      stg<float>(p.compact + L.scale_off + sid * 4, ldg<float>(p.packed + (wcount + sid) * 4));
      return;
    }
    sid -= p.n;
  }
  if (sid < p.n) {
    const float b = p.has_bias ? ldg<float>(p.packed + (wcount + uint64_t(p.n) * nblocks + sid) * 4) : 0.0f;
    stg<float>(p.compact + L.bias_off + sid * 4, b);
  }
}

// Phase 0 for the streaming path, one workgroup per row: int8 activations in dot order
// (within each 8 values of k: k0 k2 k4 k6 | k1 k3 k5 k7, matching the low / high nibbles of
// 4 packed bytes), zero beyond k up to kpad; per-unit sums sq [m][kpad/32] int32 after them.
template <class T>
__global__ __launch_bounds__(256) void qmm4c_rowquant(Q4CParams p, uint32_t groupwise, uint32_t kpad) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const uint32_t m = blockIdx.x;
  const uint64_t row = p.inp + uint64_t(m) * p.k * item;
  float mn, mx;
  row_range<T>(row, p.k, &mn, &mx);
  const RowQuant rq = row_quant(mn, mx, groupwise != 0);
  if (threadIdx.x == 0) {
    stg<uint32_t>(p.rows + 8ull * m, f32_bits(rq.recip));
    stg<int32_t>(p.rows + 8ull * m + 4, -rq.izp);
  }
  const uint64_t qrow = p.q + uint64_t(m) * kpad;
  const uint64_t sq = p.q + uint64_t(p.m) * kpad + uint64_t(m) * (kpad / kUnit) * 4;
  // a thread quantises 8 consecutive values of k (two dot operands); 4 threads make a unit
  for (uint32_t g = threadIdx.x; g < kpad / 8; g += 256) {
    int q[8], sum = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t k = g * 8 + i;
      q[i] = k < p.k ? quantise(load_f32<T>(row + k * item), rq) : 0;
      sum += q[i];
    }
    U2 o;
    o.x = uint32_t(q[0] & 255) | uint32_t(q[2] & 255) << 8 | uint32_t(q[4] & 255) << 16 | uint32_t(q[6] & 255) << 24;
    o.y = uint32_t(q[1] & 255) | uint32_t(q[3] & 255) << 8 | uint32_t(q[5] & 255) << 16 | uint32_t(q[7] & 255) << 24;
    stg<U2>(qrow + g * 8ull, o);
    sum += dpp_i32<kQuadSwap1>(sum);  // the 4 threads of a unit are one quad (256 % 4 == 0)
    sum += dpp_i32<kQuadSwap2>(sum);
    if ((g & 3) == 0) stg<int32_t>(sq + (g / 4) * 4ull, sum);
  }
}

constexpr int kRowRor1 = 0x121;  // DPP row_ror:1: lane i of each row of 16 reads lane i-1 (mod 16)

// Phase 1, groupwise (UPB = units per block: 1, 2, 4 or 8), MR rows of activations per pass.
template <class T, int MR, int UPB>
__global__ __launch_bounds__(256) void qmm4c_gemv(Q4CParams p, CompactLayout L, uint32_t m0) {
  constexpr uint64_t item = sizeof(typename T::storage);
  constexpr int BPL = kUnitsPerLane / UPB;  // blocks per lane per round
  const int lane = threadIdx.x & 63, part = lane & 15;
  const uint32_t tile = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= L.tiles) return;  // whole waves only: no barrier follows
  const uint32_t n = tile * kTileCols + (lane >> 4);
  const uint32_t nblocks = p.k / p.bs;

  int nzp[MR];
  uint64_t qrow[MR], sqrow[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    const uint32_t m = m0 + r < p.m ? m0 + r : p.m - 1;
    nzp[r] = ldg<int32_t>(p.rows + 8ull * m + 4);
    qrow[r] = p.q + uint64_t(m) * L.kpad;
    sqrow[r] = p.q + uint64_t(p.m) * L.kpad + uint64_t(m) * (L.kpad / kUnit) * 4;
  }
  float acc[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) acc[r] = 0.0f;

  for (uint32_t round = 0; round < L.rounds; ++round) {
    const uint64_t base = (uint64_t(tile) * L.rounds + round);
    U4 w[kUnitsPerLane];
#pragma unroll
    for (int j = 0; j < kUnitsPerLane; ++j) w[j] = ldg<U4>(p.compact + ((base * kUnitsPerLane + j) * 64 + lane) * 16);
    float s[BPL];
#pragma unroll
    for (int jb = 0; jb < BPL; ++jb) s[jb] = ldg<float>(p.compact + L.scale_off + ((base * BPL + jb) * 64 + lane) * 4);
    const uint32_t unit0 = round * kRoundUnits + part * kUnitsPerLane;

    float t[MR][BPL];
#pragma unroll
    for (int jb = 0; jb < BPL; ++jb) {
      int iacc[MR], ones = 0;
#pragma unroll
      for (int r = 0; r < MR; ++r) iacc[r] = 0;
#pragma unroll
      for (int ju = 0; ju < UPB; ++ju) {
        const int j = jb * UPB + ju;
        uint32_t lo[4], hi[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          lo[d] = w[j][d] & 0x0f0f0f0fu;
          hi[d] = (w[j][d] >> 4) & 0x0f0f0f0fu;
          ones = __builtin_amdgcn_sdot4(0x01010101, int(lo[d]), ones, false);
          ones = __builtin_amdgcn_sdot4(0x01010101, int(hi[d]), ones, false);
        }
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const U4 qa = ldg<U4>(qrow[r] + uint64_t(unit0 + j) * kUnit);
          const U4 qb = ldg<U4>(qrow[r] + uint64_t(unit0 + j) * kUnit + 16);
          const uint32_t qq[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
          int a = iacc[r];
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            a = __builtin_amdgcn_sdot4(int(qq[2 * d]), int(lo[d]), a, false);
            a = __builtin_amdgcn_sdot4(int(qq[2 * d + 1]), int(hi[d]), a, false);
          }
          iacc[r] = a - 8 * ldg<int32_t>(sqrow[r] + uint64_t(unit0 + j) * 4);
        }
      }
#pragma unroll
      for (int r = 0; r < MR; ++r) t[r][jb] = float(iacc[r] + nzp[r] * (ones - 8 * kUnit * UPB)) * s[jb];
    }

    // pass the running float32 sums along each row of 16 lanes, in block order
    const uint32_t blk0 = unit0 / UPB;
#pragma unroll 1
    for (int ph = 0; ph < 16; ++ph) {
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        float a = dpp_f32<kRowRor1>(acc[r]);
        if (part == ph) {
#pragma unroll
          for (int jb = 0; jb < BPL; ++jb) {
            const uint32_t blk = blk0 + jb;
            if (blk < nblocks) a = blk == 0 ? t[r][jb] : a + t[r][jb];
          }
          acc[r] = a;
        }
      }
    }
  }
  if (part == 15 && n < p.n) {
    const float bias = ldg<float>(p.compact + L.bias_off + n * 4ull);
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      if (m0 + r < p.m) {
        const float recip = bits_f32(ldg<uint32_t>(p.rows + 8ull * (m0 + r)));
        finish_store<T>(p.out + (uint64_t(m0 + r) * p.n + n) * item, acc[r], recip, p.has_bias != 0, bias);
      }
    }
  }
}

// Phase 1, channelwise (one block spanning K): integer partial sums per lane, one integer
// reduction over the row of 16 lanes, one float32 scaling.
template <class T, int MR>
__global__ __launch_bounds__(256) void qmm4c_gemv_channelwise(Q4CParams p, CompactLayout L, uint32_t m0) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const int lane = threadIdx.x & 63, part = lane & 15;
  const uint32_t tile = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (tile >= L.tiles) return;
  const uint32_t n = tile * kTileCols + (lane >> 4);
  int nzp[MR], iacc[MR], ones = 0;
  uint64_t qrow[MR], sqrow[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    const uint32_t m = m0 + r < p.m ? m0 + r : p.m - 1;
    nzp[r] = ldg<int32_t>(p.rows + 8ull * m + 4);
    qrow[r] = p.q + uint64_t(m) * L.kpad;
    sqrow[r] = p.q + uint64_t(p.m) * L.kpad + uint64_t(m) * (L.kpad / kUnit) * 4;
    iacc[r] = 0;
  }
  for (uint32_t round = 0; round < L.rounds; ++round) {
    const uint64_t base = (uint64_t(tile) * L.rounds + round);
    U4 w[kUnitsPerLane];
#pragma unroll
    for (int j = 0; j < kUnitsPerLane; ++j) w[j] = ldg<U4>(p.compact + ((base * kUnitsPerLane + j) * 64 + lane) * 16);
    const uint32_t unit0 = round * kRoundUnits + part * kUnitsPerLane;
#pragma unroll
    for (int j = 0; j < kUnitsPerLane; ++j) {
      uint32_t lo[4], hi[4];
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        lo[d] = w[j][d] & 0x0f0f0f0fu;
        hi[d] = (w[j][d] >> 4) & 0x0f0f0f0fu;
        ones = __builtin_amdgcn_sdot4(0x01010101, int(lo[d]), ones, false);
        ones = __builtin_amdgcn_sdot4(0x01010101, int(hi[d]), ones, false);
      }
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        const U4 qa = ldg<U4>(qrow[r] + uint64_t(unit0 + j) * kUnit);
        const U4 qb = ldg<U4>(qrow[r] + uint64_t(unit0 + j) * kUnit + 16);
        const uint32_t qq[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
        int a = iacc[r];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          a = __builtin_amdgcn_sdot4(int(qq[2 * d]), int(lo[d]), a, false);
          a = __builtin_amdgcn_sdot4(int(qq[2 * d + 1]), int(hi[d]), a, false);
        }
        iacc[r] = a - 8 * ldg<int32_t>(sqrow[r] + uint64_t(unit0 + j) * 4);
      }
    }
  }
  // every unit a lane visited (padding included) holds 32 nibbles; padding nibbles are 8
  ones -= 8 * kUnit * kUnitsPerLane * int(L.rounds);
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    int v = iacc[r] + nzp[r] * ones;
    v += dpp_i32<kQuadSwap1>(v);
    v += dpp_i32<kQuadSwap2>(v);
    v += dpp_i32<kRowHalfMirror>(v);
    v += dpp_i32<kRowMirror>(v);
    iacc[r] = v;
  }
  if (part == 15 && n < p.n) {
    const float s = ldg<float>(p.compact + L.scale_off + n * 4ull);
    const float bias = ldg<float>(p.compact + L.bias_off + n * 4ull);
#pragma unroll
    for (int r = 0; r < MR; ++r) {
      if (m0 + r < p.m) {
        const float recip = bits_f32(ldg<uint32_t>(p.rows + 8ull * (m0 + r)));
        finish_store<T>(p.out + (uint64_t(m0 + r) * p.n + n) * item, float(iacc[r]) * s, recip, p.has_bias != 0, bias);
      }
    }
  }
}

bool check_q4_shape(uint32_t m, uint32_t n, uint32_t k, uint32_t bs, std::string* err) {
  if (bs == 0 || !(bs == k || (bs % 32 == 0 && k % bs == 0))) {
    *err = "qmm4: block size must equal k or be a multiple of 32 dividing k";
    return false;
  }
  if (uint64_t(m) * (k > n ? k : n) >= (1ull << 31) || uint64_t(n) * k >= (1ull << 32)) {
    *err = "qmm4: too large for 32-bit indexing";
    return false;
  }
  return true;
}

template <class T, int MR>
void launch_gemv_upb(const Q4CParams& p, const CompactLayout& L, uint32_t m0, hipStream_t stream) {
  const dim3 grid((L.tiles + 3) / 4), block(256);
  switch (L.upb) {
    case 0: hipLaunchKernelGGL((qmm4c_gemv_channelwise<T, MR>), grid, block, 0, stream, p, L, m0); break;
    case 1: hipLaunchKernelGGL((qmm4c_gemv<T, MR, 1>), grid, block, 0, stream, p, L, m0); break;
    case 2: hipLaunchKernelGGL((qmm4c_gemv<T, MR, 2>), grid, block, 0, stream, p, L, m0); break;
    case 4: hipLaunchKernelGGL((qmm4c_gemv<T, MR, 4>), grid, block, 0, stream, p, L, m0); break;
    case 8: hipLaunchKernelGGL((qmm4c_gemv<T, MR, 8>), grid, block, 0, stream, p, L, m0); break;
  }
}

template <class T>
void launch_gemv_rows(const Q4CParams& p, const CompactLayout& L, hipStream_t stream) {
  for (uint32_t m0 = 0; m0 < p.m; m0 += 4) {
    const uint32_t rows = p.m - m0;
    if (rows >= 4) launch_gemv_upb<T, 4>(p, L, m0, stream);
    else if (rows == 3) launch_gemv_upb<T, 3>(p, L, m0, stream);
    else if (rows == 2) launch_gemv_upb<T, 2>(p, L, m0, stream);
    else launch_gemv_upb<T, 1>(p, L, m0, stream);
  }
}

}  // namespace

uint64_t qmm4c_bytes(uint32_t n, uint32_t k, uint32_t bs) {
  CompactLayout L;
  return compact_layout(n, k, bs, &L) ? L.total : 0;
}

uint64_t qmm4c_q_bytes(uint32_t m, uint32_t k) {
  if (m == 0 || k == 0) return 0;
  const uint64_t nunits = (k + kUnit - 1) / kUnit, rounds = (nunits + kRoundUnits - 1) / kRoundUnits;
  const uint64_t kpad = rounds * kRoundUnits * kUnit;
  return round_up_u64(uint64_t(m) * kpad + uint64_t(m) * (kpad / kUnit) * 4, 256);
}

int launch_qmm4(const Q4Params& p, int dtype, uint32_t phase, uint32_t groupwise, const Machine&, hipStream_t stream,
                std::string* err) {
  if (p.m == 0 || p.n == 0) return 0;
  if (!check_q4_shape(p.m, p.n, p.k, p.bs, err)) return -1;
  if (!p.inp || !p.q || !p.rows || !p.packed || !p.out) {
    *err = "qmm4: null tensor address";
    return -1;
  }
  if (p.m > 65535) {
    *err = "qmm4: at most 65535 rows per dispatch";  // quant.cpp:187-189 chunks the rows
    return -1;
  }
  if (groupwise != (p.bs != p.k ? 1u : 0u)) {
    *err = "qmm4: GROUPWISE must be 1 exactly when bs != k";
    return -1;
  }
  if (phase == 0) {
    if (dtype == VKT_F32) hipLaunchKernelGGL((qmm4_rowquant<f32_t>), dim3(p.m), dim3(256), 0, stream, p, groupwise);
    else hipLaunchKernelGGL((qmm4_rowquant<bf16_t>), dim3(p.m), dim3(256), 0, stream, p, groupwise);
  } else if (phase == 1) {
    const dim3 grid((p.n + 255) / 256, p.m);
    if (dtype == VKT_F32) hipLaunchKernelGGL((qmm4_matmul_expanded<f32_t>), grid, dim3(256), 0, stream, p);
    else hipLaunchKernelGGL((qmm4_matmul_expanded<bf16_t>), grid, dim3(256), 0, stream, p);
  } else {
    *err = "qmm4: PHASE must be 0 or 1";
    return -1;
  }
  if (hipGetLastError() != hipSuccess) {
    *err = "qmm4: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_qmm4c_pack(const Q4PackParams& p, const Machine&, hipStream_t stream, std::string* err) {
  CompactLayout L;
  if (!check_q4_shape(1, p.n, p.k, p.bs, err)) return -1;
  if (!compact_layout(p.n, p.k, p.bs, &L)) {
    *err = "qmm4c_pack: this shape has no compact form (groupwise block sizes: 32, 64, 128, 256)";
    return -1;
  }
  if (!p.packed || !p.compact || (p.compact & 15)) {
    *err = "qmm4c_pack: null or unaligned address";
    return -1;
  }
  const uint64_t threads = L.nib_bytes / 16 + (L.upb ? L.scale_bytes / 4 : p.n) + p.n;
  const uint64_t groups = (threads + 255) / 256;
  if (groups >= (1ull << 31)) {
    *err = "qmm4c_pack: too large";
    return -1;
  }
  hipLaunchKernelGGL(qmm4c_pack_kernel, dim3(uint32_t(groups)), dim3(256), 0, stream, p, L);
  if (hipGetLastError() != hipSuccess) {
    *err = "qmm4c_pack: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_qmm4c(const Q4CParams& p, int dtype, uint32_t phase, uint32_t groupwise, uint32_t, const Machine&,
                 hipStream_t stream, std::string* err) {
  if (p.m == 0 || p.n == 0) return 0;
  CompactLayout L;
  if (!check_q4_shape(p.m, p.n, p.k, p.bs, err)) return -1;
  if (!compact_layout(p.n, p.k, p.bs, &L)) {
    *err = "qmm4c: this shape has no compact form (groupwise block sizes: 32, 64, 128, 256)";
    return -1;
  }
  if (groupwise != (p.bs != p.k ? 1u : 0u)) {
    *err = "qmm4c: GROUPWISE must be 1 exactly when bs != k";
    return -1;
  }
  if (!p.inp || !p.q || !p.rows || !p.out || (p.q & 15)) {
    *err = "qmm4c: null or unaligned tensor address";
    return -1;
  }
  if (phase == 0) {
    if (p.m > 65535) {
      *err = "qmm4c: at most 65535 rows per dispatch";
      return -1;
    }
    if (dtype == VKT_F32)
      hipLaunchKernelGGL((qmm4c_rowquant<f32_t>), dim3(p.m), dim3(256), 0, stream, p, groupwise, L.kpad);
    else
      hipLaunchKernelGGL((qmm4c_rowquant<bf16_t>), dim3(p.m), dim3(256), 0, stream, p, groupwise, L.kpad);
  } else if (phase == 1) {
    if (!p.compact || (p.compact & 15)) {
      *err = "qmm4c: null or unaligned side-car address";
      return -1;
    }
    if (dtype == VKT_F32) launch_gemv_rows<f32_t>(p, L, stream);
    else launch_gemv_rows<bf16_t>(p, L, stream);
  } else {
    *err = "qmm4c: PHASE must be 0 or 1";
    return -1;
  }
  if (hipGetLastError() != hipSuccess) {
    *err = "qmm4c: kernel launch failed";
    return -1;
  }
  return 0;
}

}  // namespace vkt
