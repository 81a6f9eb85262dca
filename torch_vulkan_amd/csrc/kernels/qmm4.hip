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
//   "qmm4c_*"  the compact path.  "qmm4c_pack" rewrites the packed vector once into a
//              compact side-car (two nibbles per byte, 16 bytes per lane per load, laid out
//              so that every load instruction of a wave reads 1 KiB contiguous), in one of
//              two layouts: for the matrix cores (more than 4 rows; described further down)
//              or for the streaming kernel (at most 4 rows per launch), where the product
//              is an HBM stream over it:
//                - a workgroup of 4 waves owns 16 output columns; lane = (column, k-part):
//                  the 16 k-parts (4 waves x 4 groups of 16 lanes) split K into runs of
//                  8 units per round (a unit = 32 values of k = one 16-byte load);
//                - everything integer runs on v_dot8_i32_i4: weights nib-8 are nib^8 read
//                  as signed nibbles (one xor per 8 weights), activations q = 16 qh + ql are
//                  kept as two signed-nibble planes qh and ql-8, so
//                  sum (q+nzp) w = 16 dot8(qh,w) + dot8(ql-8,w) + (8+nzp) dot8(1,w):
//                  four instructions per 8 weights, no unpacking;
//                - the float32 block terms must be added in block order: every lane leaves
//                  its terms in LDS at their blocks' places and one thread per output adds
//                  a round's terms in order.  Starting from -0.0f and padding with -0.0f makes
//                  every step a plain addition (x + -0 = x, -0 + t = t) with the reference's bits.
#pragma clang fp contract(off)

#include <type_traits>

#include "common.h"
#include "kernels.h"

namespace vkt {
namespace {

constexpr int kUnit = 32;          // values of k per 16-byte load of nibbles
constexpr int kUnitsPerLane = 8;   // units a lane handles per round
constexpr int kRoundUnits = 128;   // 16 k-parts * 8 units
constexpr int kTileCols = 16;      // output columns per workgroup
constexpr int kFusedGroups = 8;    // groups of 8 activations a thread quantises in the fused kernel

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

// Workgroup-wide min / max of per-thread values (NW waves).
template <int NW = 4>
__device__ __forceinline__ void block_range(float* mn, float* mx) {
  __shared__ float bmin[NW], bmax[NW];
  const float a = wave_min(*mn), b = wave_max(*mx);
  if ((threadIdx.x & 63) == 0) bmin[threadIdx.x >> 6] = a, bmax[threadIdx.x >> 6] = b;
  __syncthreads();
  float lo = bmin[0], hi = bmax[0];
#pragma unroll
  for (int w = 1; w < NW; ++w) lo = fminf(lo, bmin[w]), hi = fmaxf(hi, bmax[w]);
  *mn = lo, *mx = hi;
}

// 8 consecutive elements at a 16-byte aligned address (float32: 32-byte aligned pairs).
template <class T>
__device__ __forceinline__ void load8_f32(uint64_t addr, float (&x)[8]);
template <>
__device__ __forceinline__ void load8_f32<f32_t>(uint64_t addr, float (&x)[8]) {
  const F4 a = ldg<F4>(addr), b = ldg<F4>(addr + 16);
  x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = b.x, x[5] = b.y, x[6] = b.z, x[7] = b.w;
}
template <>
__device__ __forceinline__ void load8_f32<bf16_t>(uint64_t addr, float (&x)[8]) {
  const U4 v = ldg<U4>(addr);
#pragma unroll
  for (int j = 0; j < 4; ++j) x[2 * j] = bits_f32(v[j] << 16), x[2 * j + 1] = bits_f32(v[j] & 0xffff0000u);
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
  uint32_t kpad;  // values of k per activation row in LDS / scratch (rounds * 4096)
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
  // [tile][round][wave 4][unit 8][lane 64] x 16 bytes
  L->nib_bytes = uint64_t(L->tiles) * L->rounds * 4 * kUnitsPerLane * 64 * 16;
  L->scale_off = L->nib_bytes;
  // groupwise: [tile][round][wave 4][lane 64][blocks per lane] float32; channelwise: [n]
  L->scale_bytes = channelwise ? round_up_u64(uint64_t(n) * 4, 256)
                               : uint64_t(L->tiles) * L->rounds * 4 * 64 * (kUnitsPerLane / L->upb) * 4;
  L->bias_off = L->scale_off + L->scale_bytes;
  L->total = L->bias_off + round_up_u64(uint64_t(n) * 4, 256);
  L->kpad = L->rounds * kRoundUnits * kUnit;
  return true;
}

// One thread per 16-byte unit of the side-car, then per scale slot, then per bias.
__global__ __launch_bounds__(256) void qmm4c_pack_kernel(Q4PackParams p, CompactLayout L) {
  const uint32_t rstride = (p.k + 1) / 2, nblocks = (p.k + p.bs - 1) / p.bs;
  const uint64_t wcount = uint64_t(p.n) * p.k / 2;
  const uint64_t slots = L.nib_bytes / 16;
  const uint64_t id = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (id < slots) {
    const uint32_t lane = id & 63, j = (id >> 6) & 7, wave = (id >> 9) & 3;
    const uint64_t tr = id >> 11;
    const uint32_t round = tr % L.rounds, tile = tr / L.rounds;
    const uint32_t n = tile * kTileCols + (lane & 15), part = wave * 4 + (lane >> 4);
    const uint32_t unit = round * kRoundUnits + part * kUnitsPerLane + j;
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
      const uint32_t jb = sid % bpl, lane = (sid / bpl) & 63, wave = (sid / (bpl * 64)) & 3;
      const uint64_t tr = sid / (bpl * 256);
      const uint32_t round = tr % L.rounds, tile = tr / L.rounds;
      const uint32_t n = tile * kTileCols + (lane & 15), part = wave * 4 + (lane >> 4);
      const uint32_t blk = (round * kRoundUnits + part * kUnitsPerLane) / L.upb + jb;
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

// 8 quantised values -> their two signed-nibble planes: hi = q >> 4, lo = (q & 15) - 8,
// nibble i of each word belonging to the i-th value.
__device__ __forceinline__ void nibble_planes(const int (&q)[8], uint32_t* hi, uint32_t* lo) {
  uint32_t h = 0, l = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    h |= (uint32_t(q[i] >> 4) & 15u) << (4 * i);
    l |= ((uint32_t(q[i]) & 15u) ^ 8u) << (4 * i);
  }
  *hi = h, *lo = l;
}

// Activation rows as the streaming kernel reads them: per unit of 32 values 16 bytes of hi
// nibbles then 16 bytes of lo nibbles.  In LDS a row carries 16 bytes of padding after every
// 256 (one lane's run of 8 units), so that the four k-parts a wave reads at once, 256 bytes
// apart, fall on different banks.
__host__ __device__ inline uint32_t q_row_bytes(uint32_t kpad) { return kpad + kpad / 256 * 16; }
constexpr uint32_t kTermPitch = 132;  // floats per (row, column) of a round's block terms: 128 + 4, so that the 16
                                      // columns' 16-byte reads fall on different banks
// (per team of 4 waves: the carried sums [rows][16], 64 bytes, and a round's block terms)
__host__ __device__ inline uint32_t q_team_bytes(uint32_t rows) { return rows * kTileCols * 4 + 64 + rows * kTileCols * kTermPitch * 4; }
__host__ __device__ inline uint32_t q_lds_bytes(uint32_t rows, uint32_t kpad, uint32_t teams = 1) {
  return rows * q_row_bytes(kpad) + teams * q_team_bytes(rows);
}
__device__ __forceinline__ uint32_t q_group_offset(uint32_t g) {  // byte offset of 8 values' hi word
  const uint32_t unit = g >> 2, d = g & 3;
  return unit * kUnit + unit / 8 * 16 + d * 4;
}

// Phase 0 for the two-launch form, one workgroup per row: nibble planes into q
// ([m][kpad] bytes, no padding), rows[2m] = bits(1/scale), rows[2m+1] = -zero_point.
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
  for (uint32_t g = threadIdx.x; g < kpad / 8; g += 256) {
    int q[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t k = g * 8 + i;
      q[i] = k < p.k ? quantise(load_f32<T>(row + k * item), rq) : 0;
    }
    uint32_t hi, lo;
    nibble_planes(q, &hi, &lo);
    const uint64_t at = qrow + (g >> 2) * kUnit + (g & 3) * 4;
    stg<uint32_t>(at, hi);
    stg<uint32_t>(at + 16, lo);
  }
}

// The streaming kernel.  UPB = units per scale block (1, 2, 4, 8), or 0 for channelwise (one
// block spanning K).  XG != 0 (fused): the workgroup quantises its MR activation rows itself (phase 0
// folded in: no second launch, no scratch round trip); otherwise it stages the planes that
// phase 0 left in global memory.  The inner loop reads activations from LDS and weights
// straight from HBM.
template <class T, int MR, int UPB, int XG, int TEAMS>
__global__ __launch_bounds__(256 * TEAMS) void qmm4c_stream(Q4CParams p, CompactLayout L, uint32_t m0, uint32_t groupwise) {
  constexpr bool FUSED = XG != 0;  // XG: groups of 8 activations a thread quantises (k <= 2048 * XG)
  constexpr uint64_t item = sizeof(typename T::storage);
  constexpr int BPL = UPB ? kUnitsPerLane / UPB : 1;  // blocks per lane per round
  constexpr int UN = UPB ? UPB : kUnitsPerLane;       // units of a block within a lane
  extern __shared__ __attribute__((aligned(16))) uint8_t q_lds[];
  constexpr int XGT = (XG + TEAMS - 1) / TEAMS;  // groups of 8 activations per thread of the whole workgroup
  // A team of 4 waves per column tile; the teams of a workgroup share the quantised activation rows (read and
  // quantised once per workgroup).  tid, wave: within the team; wtid: within the workgroup.
  const int wtid = threadIdx.x, team = wtid >> 8, tid = wtid & 255, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4, part = wave * 4 + grp;
  // (a team past the last tile works on the last tile again and stores nothing: it keeps to the barriers)
  const bool live = blockIdx.x * TEAMS + team < L.tiles;
  const uint32_t tile = live ? blockIdx.x * TEAMS + team : L.tiles - 1, n = tile * kTileCols + col;
  const uint32_t nblocks = UPB ? p.k / p.bs : 1;
  const uint32_t qs = q_row_bytes(L.kpad);
  float* const carry = reinterpret_cast<float*>(q_lds + MR * qs + team * q_team_bytes(MR));  // [MR][16]
  int* const itotal = reinterpret_cast<int*>(carry);                    // (channelwise: integer totals)
  float* const terms = carry + MR * kTileCols + 16;                     // [MR][16][kTermPitch]: a round's block terms

  // (every thread: a load without a branch around it; asked for first, so that it is there long before the sums are)
  const float bias = ldg<float>(p.compact + L.bias_off + (n < p.n ? n : p.n - 1) * 4ull);

  // Loads return in the order they were issued.  The first row's activations are asked for first (they come
  // from L2 and the row quantisation waits for them alone), then the first round's weights and scales: the
  // HBM stream runs while the row is quantised.  (Weights first made the quantisation wait for the stream:
  // 2.5 us of 9.7 at K = 4096.)
  U4 w[kUnitsPerLane];
  float s[BPL];
  auto request_round = [&](uint32_t round) {
    const uint64_t base = (uint64_t(tile) * L.rounds + round) * 4 + wave;
    // (scales first: a block's term needs its scale as soon as its weights are in)
    if constexpr (UPB != 0) {
      const uint64_t sp = p.compact + L.scale_off + (base * 64 + lane) * BPL * 4;
      if constexpr (BPL == 8) {
        const F4 s0 = ldg_stream<F4>(sp), s1 = ldg_stream<F4>(sp + 16);
        s[0] = s0.x, s[1] = s0.y, s[2] = s0.z, s[3] = s0.w, s[4] = s1.x, s[5] = s1.y, s[6] = s1.z, s[7] = s1.w;
      } else if constexpr (BPL == 4) {
        const F4 s0 = ldg<F4>(sp);
        s[0] = s0.x, s[1] = s0.y, s[2] = s0.z, s[3] = s0.w;
      } else {
#pragma unroll
        for (int jb = 0; jb < BPL; ++jb) s[jb] = ldg<float>(sp + 4 * jb);
      }
    }
#pragma unroll
    for (int j = 0; j < kUnitsPerLane; ++j) w[j] = ldg_stream<U4>(p.compact + ((base * kUnitsPerLane + j) * 64 + lane) * 16);
  };
  if constexpr (!FUSED) request_round(0);

  int nzp8[MR];  // 8 - zero_point
  float recip[MR];
#pragma unroll
  for (int r = 0; r < MR; ++r) {
    const uint32_t m = m0 + r < p.m ? m0 + r : p.m - 1;
    if constexpr (FUSED) {
      const uint64_t row = p.inp + uint64_t(m) * p.k * item;
      // A thread owns the groups of 8 values g = tid + 256 i, i < XG: all loads are in flight together, the row's
      // range is reduced from registers and the values are quantised from registers.  (The launcher fuses only
      // when k is a multiple of 8, rows are 16-byte aligned and k <= 2048 * XG; otherwise it runs phase 0 itself.)
      // No branch goes around a load (groups past the row read its first group again): the compiler then knows how
      // many younger loads there are and waits for the row alone, not for the weights requested after it.
      const uint32_t groups = p.k / 8;
      float x[XGT ? XGT : 1][8];
      float mn = 3.40282347e38f, mx = -3.40282347e38f;
#pragma unroll
      for (int i = 0; i < XGT; ++i) {
        const uint32_t g = wtid + 256 * TEAMS * i;
        load8_f32<T>(row + uint64_t(g < groups ? g : 0) * 8 * item, x[i]);
      }
      if (r == 0) request_round(0);
#pragma unroll
      for (int i = 0; i < XGT; ++i) {
        const bool inside = uint32_t(wtid + 256 * TEAMS * i) < groups;
#pragma unroll
        for (int e = 0; e < 8; ++e) mn = fminf(mn, inside ? x[i][e] : mn), mx = fmaxf(mx, inside ? x[i][e] : mx);
      }
      block_range<4 * TEAMS>(&mn, &mx);
      const RowQuant rq = row_quant(mn, mx, groupwise != 0);
      nzp8[r] = 8 - rq.izp;
      recip[r] = rq.recip;
#pragma unroll
      for (int i = 0; i < XGT; ++i) {
        const uint32_t g = wtid + 256 * TEAMS * i;
        if (g < L.kpad / 8) {
          uint32_t hi = 0, lo = 0x88888888u;  // beyond k: value 0 = planes (0, 0 - 8)
          if (g < groups) {
            int q[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) q[e] = quantise(x[i][e], rq);
            nibble_planes(q, &hi, &lo);
          }
          uint8_t* at = q_lds + r * qs + q_group_offset(g);
          *reinterpret_cast<uint32_t*>(at) = hi;
          *reinterpret_cast<uint32_t*>(at + 16) = lo;
        }
      }
      __syncthreads();  // (the range scratch is reused by the next row)
    } else {
      nzp8[r] = 8 + ldg<int32_t>(p.rows + 8ull * m + 4);
      recip[r] = bits_f32(ldg<uint32_t>(p.rows + 8ull * m));
      const uint64_t src = p.q + uint64_t(m) * L.kpad;
      for (uint32_t c = wtid; c < L.kpad / 16; c += 256 * TEAMS)
        *reinterpret_cast<U4*>(q_lds + r * qs + c * 16 + c / 16 * 16) = ldg<U4>(src + c * 16ull);
    }
  }
  if (tid < MR * kTileCols) carry[tid] = UPB ? -0.0f : 0.0f;  // (integer 0 and +0.0f share their bits)
  __syncthreads();

  float acc[MR];
  int tot_a[MR], tot_b[MR], tot_c = 0;
#pragma unroll
  for (int r = 0; r < MR; ++r) acc[r] = 0.0f, tot_a[r] = 0, tot_b[r] = 0;

  for (uint32_t round = 0; round < L.rounds; ++round) {
    const uint32_t unit0 = round * kRoundUnits + part * kUnitsPerLane;
    const uint8_t* qbase = q_lds + unit0 * kUnit + unit0 / 8 * 16;

    // With one row the round's activation planes are read from LDS into registers before the first weight is
    // touched: the reads then wait under the weights' flight time, not between the products (measured per workgroup at
    // one row: products 0.75 us after the weights' arrival with a pair of reads in front of every unit's products).
    constexpr bool PRELOAD = MR == 1;
    U4 qreg[PRELOAD ? MR : 1][kUnitsPerLane][2];
    if constexpr (PRELOAD) {
#pragma unroll
      for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int j = 0; j < kUnitsPerLane; ++j) {
          qreg[r][j][0] = *reinterpret_cast<const U4*>(qbase + r * qs + j * kUnit);
          qreg[r][j][1] = *reinterpret_cast<const U4*>(qbase + r * qs + j * kUnit + 16);
        }
      __builtin_amdgcn_sched_barrier(0);  // (the scheduler would move each read down to its first use)
    }
    float t[MR][BPL];
#pragma unroll
    for (int jb = 0; jb < BPL; ++jb) {
      int da[MR], db[MR], dc = 0;
#pragma unroll
      for (int r = 0; r < MR; ++r) da[r] = 0, db[r] = 0;
#pragma unroll
      for (int ju = 0; ju < UN; ++ju) {
        const int j = jb * UN + ju;
        uint32_t ws[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          ws[d] = w[j][d] ^ 0x88888888u;  // nib - 8 as signed nibbles
          dc = __builtin_amdgcn_sdot8(0x11111111, int(ws[d]), dc, false);
        }
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const U4 qh = PRELOAD ? qreg[PRELOAD ? r : 0][j][0] : *reinterpret_cast<const U4*>(qbase + r * qs + j * kUnit);
          const U4 ql = PRELOAD ? qreg[PRELOAD ? r : 0][j][1] : *reinterpret_cast<const U4*>(qbase + r * qs + j * kUnit + 16);
#pragma unroll
          for (int d = 0; d < 4; ++d) {
            da[r] = __builtin_amdgcn_sdot8(int(qh[d]), int(ws[d]), da[r], false);
            db[r] = __builtin_amdgcn_sdot8(int(ql[d]), int(ws[d]), db[r], false);
          }
        }
      }
      if constexpr (UPB != 0) {
        const bool valid = unit0 / UPB + jb < nblocks;
#pragma unroll
        for (int r = 0; r < MR; ++r) {
          const int iacc = (da[r] << 4) + db[r] + nzp8[r] * dc;
          t[r][jb] = valid ? float(iacc) * s[jb] : -0.0f;
        }
      } else {
        tot_c += dc;
#pragma unroll
        for (int r = 0; r < MR; ++r) tot_a[r] += da[r], tot_b[r] += db[r];
      }
    }

    // the next round's weights and scales are requested as soon as this round's are used up
    if (round + 1 < L.rounds) request_round(round + 1);
    if constexpr (UPB != 0) {
      // The float32 block terms must be added in block order.  Every lane leaves its terms in LDS at the
      // place of their blocks; then one thread per (row, column) adds the round's 16 * BPL terms in
      // order (16-byte reads, the only sequential part: ~130 dependent additions per round).
#pragma unroll
      for (int r = 0; r < MR; ++r) {
        float* at = terms + (r * kTileCols + col) * kTermPitch + part * BPL;
        if constexpr (BPL % 4 == 0) {
#pragma unroll
          for (int jb = 0; jb < BPL; jb += 4) *reinterpret_cast<F4*>(at + jb) = F4{t[r][jb], t[r][jb + 1], t[r][jb + 2], t[r][jb + 3]};
        } else {
#pragma unroll
          for (int jb = 0; jb < BPL; ++jb) at[jb] = t[r][jb];
        }
      }
      __syncthreads();
      if (wave == 0 && grp < MR) {
        // (thread (grp, col) of the first wave owns row grp, column col; its sum lives in acc[0])
        const float* from = terms + (grp * kTileCols + col) * kTermPitch;
        float a = round == 0 ? -0.0f : acc[0];
        // The terms are read 16 reads at a time, all before the first addition of their batch: the additions are a
        // chain of dependent operations, and with a read in front of every few of them the chain waits for LDS at
        // every step (0.75 us per round; batches keep the kernel at three waves per SIMD).
        constexpr int BATCH = 4 * BPL < 16 ? 4 * BPL : 16;
#pragma unroll
        for (int b0 = 0; b0 < 4 * BPL; b0 += BATCH) {
          F4 v[BATCH];
#pragma unroll
          for (int b = 0; b < BATCH; ++b) v[b] = *reinterpret_cast<const F4*>(from + 4 * (b0 + b));
          __builtin_amdgcn_sched_barrier(0);
#pragma unroll
          for (int b = 0; b < BATCH; ++b) {
            a = a + v[b].x;
            a = a + v[b].y;
            a = a + v[b].z;
            a = a + v[b].w;
          }
          __builtin_amdgcn_sched_barrier(0);
        }
        acc[0] = a;
      }
      __syncthreads();  // (the next round overwrites the terms)
    }
  }
  if constexpr (UPB == 0) {
    // one block: exact integer totals over the 16 k-parts, then one scaling
#pragma unroll
    for (int r = 0; r < MR; ++r) atomicAdd(&itotal[r * kTileCols + col], (tot_a[r] << 4) + tot_b[r] + nzp8[r] * tot_c);
    __syncthreads();
    if (part == 15) {
      const float s = ldg<float>(p.compact + L.scale_off + (n < p.n ? n : p.n - 1) * 4ull);
#pragma unroll
      for (int r = 0; r < MR; ++r) acc[r] = float(itotal[r * kTileCols + col]) * s;
    }
  }
  if constexpr (UPB != 0) {
    if (live && wave == 0 && grp < MR && n < p.n && m0 + grp < p.m) {
      float rc = recip[0];
#pragma unroll
      for (int r = 1; r < MR; ++r) rc = grp == r ? recip[r] : rc;
      finish_store<T>(p.out + (uint64_t(m0 + grp) * p.n + n) * item, acc[0], rc, p.has_bias != 0, bias);
    }
  } else if (live && part == 15 && n < p.n) {
#pragma unroll
    for (int r = 0; r < MR; ++r)
      if (m0 + r < p.m) finish_store<T>(p.out + (uint64_t(m0 + r) * p.n + n) * item, acc[r], recip[r], p.has_bias != 0, bias);
  }
}

// ------------------------------------------------------------------ compact path on the matrix cores
//
// For more than 4 rows the integer sums move to v_mfma_i32_16x16x32_i8, over a second
// side-car layout ("matrix layout"):
//   - a unit (32 values of k) of a tile of 16 columns against a tile of 16 rows is one MFMA
//     shape: lane (x = lane % 16, kg = lane / 16) supplies 8 values k = 32 u + 8 kg .. + 7 of
//     activation row x (first operand) and of weight column x (second operand), and
//     receives the sums of column x for rows 4 kg .. + 3;
//   - weights stay unsigned: a word of 8 nibbles becomes the operand's 8 bytes with two ANDs
//     and a shift, and
//       sum (q + nzp) (nib - 8) = sum q nib + sum q (-8) + nzp sum nib - 256 nzp
//     is four chained MFMAs: the activations against the nibbles, the activations against a
//     constant operand of -8, and two whose first operand holds nzp in every position, split
//     in two halves that fit a signed byte (nzp reaches 128); the last term enters as the
//     first MFMA's accumulator input.  No integer work is left for the vector ALU;
//   - the float32 block terms are produced 4 waves wide and added in block order by the
//     thread that owns the output (see qmm4m_tile);
//   - blocks beyond K hold nibble 8 (weight 0) and scale -1: their term is (+0) * -1 = -0.0f,
//     which leaves the running sum as it is, bit for bit.

struct MatrixLayout {
  uint32_t nunits, quads, tiles, upb;  // quads: groups of 4 units, padded to a multiple of 16
  uint64_t nib_bytes, scale_off, scale_bytes, bias_off, total;
};

__host__ __device__ inline bool matrix_layout(uint32_t n, uint32_t k, uint32_t bs, MatrixLayout* L) {
  if (n == 0 || k == 0 || bs == 0) return false;
  const bool channelwise = bs == k;
  if (!channelwise && !(bs == 32 || bs == 64 || bs == 128 || bs == 256)) return false;
  if (!channelwise && k % bs != 0) return false;
  L->nunits = (k + kUnit - 1) / kUnit;
  L->quads = (L->nunits + 63) / 64 * 16;
  L->tiles = (n + kTileCols - 1) / kTileCols;
  L->upb = channelwise ? 0 : bs / kUnit;
  // [quad][tile][lane 64] x 16 bytes: word j of a lane = 8 nibbles of unit 4 quad + j.  Quad-major:
  // the waves of a launch advance through K together, and what they read at any one time is then
  // one contiguous run over all tiles, spread evenly over the memory channels
  L->nib_bytes = uint64_t(L->tiles) * L->quads * 64 * 16;
  L->scale_off = L->nib_bytes;
  // groupwise: [quad][tile][column 16][unit 4] float32 (a block's scale repeated for each of
  // its units); channelwise: [n]
  L->scale_bytes = channelwise ? round_up_u64(uint64_t(n) * 4, 256) : uint64_t(L->tiles) * L->quads * 16 * 16;
  L->bias_off = L->scale_off + L->scale_bytes;
  L->total = L->bias_off + round_up_u64(uint64_t(n) * 4, 256);
  return true;
}

__global__ __launch_bounds__(256) void qmm4m_pack_kernel(Q4PackParams p, MatrixLayout L) {
  const uint32_t rstride = (p.k + 1) / 2, nblocks = (p.k + p.bs - 1) / p.bs;
  const uint64_t wcount = uint64_t(p.n) * p.k / 2;
  const uint64_t slots = L.nib_bytes / 16;
  const uint64_t id = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (id < slots) {
    const uint32_t lane = id & 63;
    const uint64_t tq = id >> 6;
    const uint32_t tile = tq % L.tiles, quad = tq / L.tiles;
    const uint32_t n = tile * kTileCols + (lane & 15), kg = lane >> 4;
    U4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const uint32_t byte_index = (quad * 4 + j) * 16 + kg * 4 + b;
        uint32_t byte = 0x88;  // weight 0
        if (n < p.n && byte_index < rstride) {
          byte = uint32_t(ldg<float>(p.packed + (uint64_t(n) * rstride + byte_index) * 4)) & 0xffu;
          if ((p.k & 1) && byte_index == rstride - 1) byte = (byte & 0x0f) | 0x80;
        }
        word |= byte << (8 * b);
      }
      out[j] = word;
    }
    stg<U4>(p.compact + id * 16, out);
    return;
  }
  uint64_t sid = id - slots;
  if (L.upb != 0) {
    const uint64_t sslots = L.scale_bytes / 4;
    if (sid < sslots) {
      const uint32_t j = sid & 3, col = (sid >> 2) & 15;
      const uint64_t tq = sid >> 6;
      const uint32_t tile = tq % L.tiles, quad = tq / L.tiles;
      const uint32_t n = tile * kTileCols + col, blk = (quad * 4 + j) / L.upb;
      float s = -1.0f;
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

// 8 quantised values as the MFMA operand's 8 bytes: even positions, then odd positions
// (the order in which the weight nibbles come apart).
__device__ __forceinline__ U2 operand_bytes(const int (&q)[8]) {
  U2 r;
  r.x = (uint32_t(q[0]) & 255u) | (uint32_t(q[2]) & 255u) << 8 | (uint32_t(q[4]) & 255u) << 16 | uint32_t(q[6]) << 24;
  r.y = (uint32_t(q[1]) & 255u) | (uint32_t(q[3]) & 255u) << 8 | (uint32_t(q[5]) & 255u) << 16 | uint32_t(q[7]) << 24;
  return r;
}

// The activation scratch of the matrix layout: [row tile][quad][half 2][lane = kg * 16 + m % 16]
// [unit 2] x 8 bytes (a wave reads a half of a quad as 64 consecutive 16-byte pieces).
__device__ __forceinline__ uint64_t operand_offset(uint32_t m, uint32_t g, uint32_t quads) {
  const uint32_t unit = g >> 2, kg = g & 3, j = unit & 3;
  return (((uint64_t(m >> 4) * quads + (unit >> 2)) * 2 + (j >> 1)) * 64 + kg * 16 + (m & 15)) * 16 + (j & 1) * 8;
}

// Phase 0 for the matrix layout, one workgroup per row.  FAST: k is a multiple of 8, at most
// 2048 * kFusedGroups, rows 16-byte aligned: the row is read once, into registers.
template <class T, bool FAST>
__global__ __launch_bounds__(256) void qmm4m_rowquant(Q4CParams p, uint32_t groupwise, uint32_t quads) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const uint32_t m = blockIdx.x, tid = threadIdx.x;
  const uint64_t row = p.inp + uint64_t(m) * p.k * item;
  const uint32_t groups_all = quads * 16;
  if constexpr (FAST) {
    const uint32_t groups = p.k / 8;
    float x[kFusedGroups][8];
    float mn = 3.40282347e38f, mx = -3.40282347e38f;
#pragma unroll
    for (int i = 0; i < kFusedGroups; ++i) {
      const uint32_t g = tid + 256 * i;
      if (g < groups) load8_f32<T>(row + g * 8 * item, x[i]);
    }
#pragma unroll
    for (int i = 0; i < kFusedGroups; ++i) {
      if (uint32_t(tid + 256 * i) < groups) {
#pragma unroll
        for (int e = 0; e < 8; ++e) mn = fminf(mn, x[i][e]), mx = fmaxf(mx, x[i][e]);
      }
    }
    block_range(&mn, &mx);
    const RowQuant rq = row_quant(mn, mx, groupwise != 0);
    if (tid == 0) {
      stg<uint32_t>(p.rows + 8ull * m, f32_bits(rq.recip));
      stg<int32_t>(p.rows + 8ull * m + 4, -rq.izp);
    }
#pragma unroll
    for (int i = 0; i < kFusedGroups; ++i) {
      const uint32_t g = tid + 256 * i;
      if (g < groups_all) {
        U2 v = {0u, 0u};
        if (g < groups) {
          int q[8];
#pragma unroll
          for (int e = 0; e < 8; ++e) q[e] = quantise(x[i][e], rq);
          v = operand_bytes(q);
        }
        stg<U2>(p.q + operand_offset(m, g, quads), v);
      }
    }
  } else {
    float mn, mx;
    row_range<T>(row, p.k, &mn, &mx);
    const RowQuant rq = row_quant(mn, mx, groupwise != 0);
    if (tid == 0) {
      stg<uint32_t>(p.rows + 8ull * m, f32_bits(rq.recip));
      stg<int32_t>(p.rows + 8ull * m + 4, -rq.izp);
    }
    for (uint32_t g = tid; g < groups_all; g += 256) {
      int q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t k = g * 8 + e;
        q[e] = k < p.k ? quantise(load_f32<T>(row + k * item), rq) : 0;
      }
      stg<U2>(p.q + operand_offset(m, g, quads), operand_bytes(q));
    }
  }
}

using V4I = int __attribute__((ext_vector_type(4)));

constexpr int kGroupQuads = 16;  // quads per workgroup and load group: 4 per wave

// The matrix-core kernel.  A workgroup is one tile of 16 columns against one tile of 16 rows
// (blockIdx.y, starting at row m0); its 4 waves share K.  Work proceeds in steps of 4 quads
// (8 for blocks of 256), one quad (two) per wave: each wave turns its units into float32
// block terms - four MFMAs per unit, then convert and scale - and leaves them in LDS;
// after a barrier, thread (row, column) adds the step's terms to its running sum in block
// order.  That addition is the only part of the operator that has to be sequential, and it
// is 1/16 of the terms per thread; everything else runs 4 waves wide per tile, with several
// workgroups per compute unit to hide each other's latencies.  The term buffer is double
// buffered, so a step costs one barrier.  Weights and scales are loaded a group of 4 quads
// per wave ahead (two register sets, used alternately), activations - which every
// workgroup of the row tile re-reads, from L2 - one step ahead.
template <class T, int UPB>
__global__ __launch_bounds__(256) void qmm4m_tile(Q4CParams p, MatrixLayout L, uint32_t m0) {
  constexpr uint64_t item = sizeof(typename T::storage);
  constexpr int QW = UPB == 8 ? 2 : 1;               // quads per wave per step
  constexpr int SPG = 4 / QW;                         // steps per group
  constexpr int BW = UPB ? 4 * QW / UPB : 0;          // blocks per wave per step
  constexpr int NB = 4 * BW;                          // blocks per step
  __shared__ __attribute__((aligned(16))) float terms[2][NB ? NB : 1][256];  // [buffer][block][output]
  const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t tile = blockIdx.x;
  const uint32_t col = lane & 15, kg = lane >> 4;
  const uint32_t row0 = m0 + blockIdx.y * 16;  // a multiple of 16, below p.m

  V4I unit_const;  // -256 nzp: per unit, for the rows this lane receives
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const uint32_t m = row0 + kg * 4 + r < p.m ? row0 + kg * 4 + r : p.m - 1;
    unit_const[r] = -256 * ldg<int32_t>(p.rows + 8ull * m + 4);
  }
  // -zero_point of the row this lane feeds as first operand, in two halves that fit a byte
  long nz_a, nz_b;
  {
    const uint32_t m = row0 + col < p.m ? row0 + col : p.m - 1;
    const int nzp = ldg<int32_t>(p.rows + 8ull * m + 4);
    const int h1 = nzp >> 1, h2 = nzp - h1;
    const uint32_t w1 = (uint32_t(h1) & 255u) * 0x01010101u, w2 = (uint32_t(h2) & 255u) * 0x01010101u;
    nz_a = long(uint64_t(w1) | uint64_t(w1) << 32);
    nz_b = long(uint64_t(w2) | uint64_t(w2) << 32);
  }
  const long minus8 = long(0xf8f8f8f8f8f8f8f8ull);

  const uint64_t wbase = p.compact + (uint64_t(tile) * 64 + lane) * 16;             // + quad * wstep
  const uint64_t sbase = p.compact + L.scale_off + (uint64_t(tile) * 16 + col) * 16;  // + quad * sstep
  const uint64_t wstep = uint64_t(L.tiles) * 1024, sstep = uint64_t(L.tiles) * 256;
  const uint64_t qbase = p.q + (uint64_t(row0 >> 4) * L.quads * 128 + lane) * 16;    // + quad * 2048 (+ 1024)

  // the quad of this wave's slot sl (0..3) in group g: consecutive waves take consecutive
  // quads (pairs of quads), so that a step's blocks lie in LDS in the order of K
  auto quad_of = [&](uint32_t g, int sl) -> uint32_t {
    return QW == 1 ? g * kGroupQuads + sl * 4 + wave : g * kGroupQuads + (sl >> 1) * 8 + wave * 2 + (sl & 1);
  };
  struct Set {
    U4 w[4];
    F4 s[4];
  };
  auto load_set = [&](Set& set, uint32_t g) {
#pragma unroll
    for (int sl = 0; sl < 4; ++sl) {
      const uint32_t quad = quad_of(g, sl);
      set.w[sl] = ldg_stream<U4>(wbase + quad * wstep);
      if constexpr (UPB != 0) set.s[sl] = ldg<F4>(sbase + quad * sstep);
    }
  };

  const uint32_t groups = L.quads / kGroupQuads;
  Set set_a, set_b;
  load_set(set_a, 0);
  U4 qn[QW][2];  // the next step's activations
  auto load_q = [&](uint32_t g, int st) {
#pragma unroll
    for (int x = 0; x < QW; ++x) {
      const uint64_t at = qbase + uint64_t(quad_of(g, st * QW + x)) * 2048;
      qn[x][0] = ldg<U4>(at), qn[x][1] = ldg<U4>(at + 1024);
    }
  };
  load_q(0, 0);

  float acc = -0.0f;       // of this thread's output
  V4I d = {0, 0, 0, 0};    // (channelwise: the wave's integer sums over all its units)
  uint32_t parity = 0;

  auto process = [&](const Set& set, uint32_t g) {
#pragma unroll
    for (int st = 0; st < SPG; ++st) {
      U4 qc[QW][2];
#pragma unroll
      for (int x = 0; x < QW; ++x) qc[x][0] = qn[x][0], qc[x][1] = qn[x][1];
      // the next step's activations (of the next group at the last step; beyond the end the
      // last group again, unused)
      if (st + 1 < SPG) load_q(g, st + 1);
      else load_q(g + 1 < groups ? g + 1 : g, 0);
#pragma unroll
      for (int x = 0; x < QW; ++x) {
        const int sl = st * QW + x;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const uint32_t v = set.w[sl][j];
          const long b = long(uint64_t(v & 0x0f0f0f0fu) | uint64_t((v >> 4) & 0x0f0f0f0fu) << 32);
          const U4& qq = qc[x][j >> 1];
          const long a = long(uint64_t(qq[(j & 1) * 2]) | uint64_t(qq[(j & 1) * 2 + 1]) << 32);
          constexpr int mask = UPB ? UPB - 1 : 0;
          const int u = x * 4 + j;  // unit within the wave's step
          const bool first = UPB != 0 && (u & mask) == 0;
          if constexpr (UPB == 1) {
            // a block per unit: a chain of its own, the constant as the first accumulator input (no copy)
            V4I x = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, unit_const, 0, 0, 0);
            x = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, minus8, x, 0, 0, 0);
            x = __builtin_amdgcn_mfma_i32_16x16x32_i8(nz_a, b, x, 0, 0, 0);
            x = __builtin_amdgcn_mfma_i32_16x16x32_i8(nz_b, b, x, 0, 0, 0);
            float* at = &terms[parity][wave * BW + u][lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) at[r * 64] = float(x[r]) * set.s[sl][j];
          } else {
            d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, first ? unit_const * (UPB ? UPB : 1) : d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, minus8, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_i32_16x16x32_i8(nz_a, b, d, 0, 0, 0);
            d = __builtin_amdgcn_mfma_i32_16x16x32_i8(nz_b, b, d, 0, 0, 0);
            if constexpr (UPB != 0) {
              if ((u & mask) == mask) {  // the block's last unit
                // position r * 64 + lane for row 4 kg + r: a wave's 64 stores of one r fall on 64 banks
                float* at = &terms[parity][wave * BW + u / UPB][lane];
#pragma unroll
                for (int r = 0; r < 4; ++r) at[r * 64] = float(d[r]) * set.s[sl][j];
              }
            }
          }
        }
      }
      if constexpr (UPB != 0) {
        __syncthreads();
#pragma unroll
        for (int blk = 0; blk < NB; ++blk) acc = acc + terms[parity][blk][tid];
        parity ^= 1;
      }
    }
  };

  for (uint32_t g = 0; g < groups; g += 2) {
    if (g + 1 < groups) load_set(set_b, g + 1);
    process(set_a, g);
    if (g + 1 < groups) {
      if (g + 2 < groups) load_set(set_a, g + 2);
      process(set_b, g + 1);
    }
  }

  // thread tid = r * 64 + kg * 16 + column owns row 4 kg + r
  const uint32_t row = ((tid >> 4) & 3) * 4 + (tid >> 6), n = tile * kTileCols + (tid & 15), m = row0 + row;
  if constexpr (UPB == 0) {
    // one block: the waves' integer sums meet in LDS, then one scaling
    __shared__ int totals[4][256];
#pragma unroll
    for (int r = 0; r < 4; ++r) totals[wave][r * 64 + lane] = d[r];
    __syncthreads();
    const uint32_t mc = m < p.m ? m : p.m - 1;
    const int nzp = ldg<int32_t>(p.rows + 8ull * mc + 4);
    const int iacc = totals[0][tid] + totals[1][tid] + totals[2][tid] + totals[3][tid] - 256 * nzp * int(L.quads * 4);
    acc = float(iacc) * ldg<float>(p.compact + L.scale_off + (n < p.n ? n : p.n - 1) * 4ull);
  }
  if (n < p.n && m < p.m) {
    const float recip = bits_f32(ldg<uint32_t>(p.rows + 8ull * m));
    const float bias = ldg<float>(p.compact + L.bias_off + n * 4ull);
    finish_store<T>(p.out + (uint64_t(m) * p.n + n) * item, acc, recip, p.has_bias != 0, bias);
  }
}

// Many rows: a wave per tile of RT x CT matrix-core tiles (16 rows x 16 columns each).  A workgroup is 4 waves
// with the same rows and neighbouring column tiles (the activations, the larger operand, come from the vector cache
// for three of them).  Each wave walks all of K by itself, so the block terms of its outputs come in block order and
// are added in registers: no LDS, no barriers.  Operands are requested kRowsAhead quads ahead, always (past the end
// the last quad again), so that the loop body is straight-line code.
constexpr int kRowsAhead = 2;

template <class T, int UPB, int RT, int CT>
__global__ __launch_bounds__(256) void qmm4m_rows(Q4CParams p, MatrixLayout L, uint32_t m0) {
  constexpr uint64_t item = sizeof(typename T::storage);
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t col = lane & 15, kg = lane >> 4;
  const uint32_t tile0 = (blockIdx.x * 4 + wave) * CT;
  const uint32_t row0 = m0 + blockIdx.y * (16 * RT);
  if (row0 >= p.m || tile0 >= L.tiles) return;  // (a whole wave, and the kernel has no barrier)

  V4I unit_const[RT];  // -256 nzp, for the rows this lane receives
  int nzp_r[RT][4];
  long nz_a[RT], nz_b[RT];
  uint64_t qbase[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const uint32_t rt = row0 + 16 * t < p.m ? row0 + 16 * t : row0;  // (a row tile past the end: the first again, not stored)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const uint32_t m = rt + kg * 4 + r < p.m ? rt + kg * 4 + r : p.m - 1;
      nzp_r[t][r] = ldg<int32_t>(p.rows + 8ull * m + 4);
      unit_const[t][r] = -256 * nzp_r[t][r];
    }
    const uint32_t m = rt + col < p.m ? rt + col : p.m - 1;
    const int nzp = ldg<int32_t>(p.rows + 8ull * m + 4);
    const int h1 = nzp >> 1, h2 = nzp - h1;
    const uint32_t w1 = (uint32_t(h1) & 255u) * 0x01010101u, w2 = (uint32_t(h2) & 255u) * 0x01010101u;
    nz_a[t] = long(uint64_t(w1) | uint64_t(w1) << 32);
    nz_b[t] = long(uint64_t(w2) | uint64_t(w2) << 32);
    qbase[t] = p.q + (uint64_t(rt >> 4) * L.quads * 128 + lane) * 16;
  }
  const long minus8 = long(0xf8f8f8f8f8f8f8f8ull);
  const V4I minus8x4 = V4I{int(0xf8f8f8f8u), int(0xf8f8f8f8u), int(0xf8f8f8f8u), int(0xf8f8f8f8u)};
  V4I nz_a4[RT], nz_b4[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    nz_a4[t] = V4I{int(nz_a[t]), int(nz_a[t]), int(nz_a[t]), int(nz_a[t])};
    nz_b4[t] = V4I{int(nz_b[t]), int(nz_b[t]), int(nz_b[t]), int(nz_b[t])};
  }
  uint64_t wbase[CT], sbase[CT];
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const uint32_t tile = tile0 + c < L.tiles ? tile0 + c : tile0;
    wbase[c] = p.compact + (uint64_t(tile) * 64 + lane) * 16;
    sbase[c] = p.compact + L.scale_off + (uint64_t(tile) * 16 + col) * 16;
  }
  const uint64_t wstep = uint64_t(L.tiles) * 1024, sstep = uint64_t(L.tiles) * 256;

  struct Set {
    U4 w[CT], q0[RT], q1[RT];
    F4 s[CT];
  };
  Set sets[kRowsAhead];
  auto request = [&](Set& set, uint32_t quad) {
    quad = quad < L.quads ? quad : L.quads - 1;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      set.q0[t] = ldg<U4>(qbase[t] + uint64_t(quad) * 2048);
      set.q1[t] = ldg<U4>(qbase[t] + uint64_t(quad) * 2048 + 1024);
    }
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      set.w[c] = ldg_stream<U4>(wbase[c] + quad * wstep);
      if constexpr (UPB != 0) set.s[c] = ldg<F4>(sbase[c] + quad * sstep);
    }
  };
#pragma unroll
  for (int i = 0; i < kRowsAhead; ++i) request(sets[i], i);

  float acc[RT][CT][4];
  V4I d[RT][CT], d2[RT][CT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int c = 0; c < CT; ++c) {
      d[t][c] = d2[t][c] = V4I{0, 0, 0, 0};
#pragma unroll
      for (int r = 0; r < 4; ++r) acc[t][c][r] = -0.0f;
    }
  // (quads is a multiple of 16, so of kRowsAhead, and blocks of up to 8 units start at even quads)
  for (uint32_t quad0 = 0; quad0 < L.quads; quad0 += kRowsAhead) {
#pragma unroll
    for (int i = 0; i < kRowsAhead; ++i) {
      const Set cur = sets[i];
      request(sets[i], quad0 + i + kRowsAhead);
      constexpr int mask = UPB ? UPB - 1 : 0;
      if constexpr (UPB == 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          long b[CT];
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            const uint32_t v = cur.w[c][j];
            b[c] = long(uint64_t(v & 0x0f0f0f0fu) | uint64_t((v >> 4) & 0x0f0f0f0fu) << 32);
          }
#pragma unroll
          for (int t = 0; t < RT; ++t) {
            const U4& qq = j < 2 ? cur.q0[t] : cur.q1[t];
            const long a = long(uint64_t(qq[(j & 1) * 2]) | uint64_t(qq[(j & 1) * 2 + 1]) << 32);
#pragma unroll
            for (int c = 0; c < CT; ++c) {
              V4I x = unit_const[t];
              x = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b[c], x, 0, 0, 0);
              x = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, minus8, x, 0, 0, 0);
              x = __builtin_amdgcn_mfma_i32_16x16x32_i8(nz_a[t], b[c], x, 0, 0, 0);
              x = __builtin_amdgcn_mfma_i32_16x16x32_i8(nz_b[t], b[c], x, 0, 0, 0);
#pragma unroll
              for (int r = 0; r < 4; ++r) acc[t][c][r] = acc[t][c][r] + float(x[r]) * cur.s[c][j];  // in block order
            }
          }
        }
      } else {
        // Blocks of two units and more: two units, 64 values of k, per matrix-core instruction (the full-rate form),
        // and the zero-point products as a chain of their own (integers: any order).
#pragma unroll
        for (int j = 0; j < 4; j += 2) {
          const int u = i * 4 + j;
          const bool first = UPB != 0 && (u & mask) == 0, last = UPB != 0 && ((u + 1) & mask) == mask;
          V4I b[CT];
#pragma unroll
          for (int c = 0; c < CT; ++c) {
            const uint32_t v0 = cur.w[c][j], v1 = cur.w[c][j + 1];
            b[c] = V4I{int(v0 & 0x0f0f0f0fu), int((v0 >> 4) & 0x0f0f0f0fu), int(v1 & 0x0f0f0f0fu), int((v1 >> 4) & 0x0f0f0f0fu)};
          }
#pragma unroll
          for (int t = 0; t < RT; ++t) {
            const U4& qq = j < 2 ? cur.q0[t] : cur.q1[t];
            const V4I a = V4I{int(qq[0]), int(qq[1]), int(qq[2]), int(qq[3])};
#pragma unroll
            for (int c = 0; c < CT; ++c) {
              V4I x = first ? unit_const[t] * (UPB ? UPB : 1) : d[t][c];
              V4I y = first ? V4I{0, 0, 0, 0} : d2[t][c];
              x = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b[c], x, 0, 0, 0);
              y = __builtin_amdgcn_mfma_i32_16x16x64_i8(nz_a4[t], b[c], y, 0, 0, 0);
              x = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, minus8x4, x, 0, 0, 0);
              y = __builtin_amdgcn_mfma_i32_16x16x64_i8(nz_b4[t], b[c], y, 0, 0, 0);
              d2[t][c] = y;
              if (last) {  // the block's term, added in block order
                x = x + y;
#pragma unroll
                for (int r = 0; r < 4; ++r) acc[t][c][r] = acc[t][c][r] + float(x[r]) * cur.s[c][j + 1];
              }
              d[t][c] = x;
            }
          }
        }
      }
    }
    // The four matrix-core instructions of a unit are a dependent chain, 16 cycles apart: with one tile per wave the
    // float32 work of the unit before it (4 conversions, 4 products, 4 sums, and the unpacking) is put in between,
    // four instructions at a time.  (With more tiles per wave the chains of the tiles overlap by themselves, and
    // prescribing the order made those kernels slower.)
    if constexpr (UPB != 0 && RT * CT == 1) {
#pragma unroll
      for (int g = 0; g < kRowsAhead * 4 * 4; ++g) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
      }
    }
  }
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const uint32_t n = (tile0 + c) * kTileCols + col;
    if (tile0 + c >= L.tiles || n >= p.n) continue;
    const float bias = ldg<float>(p.compact + L.bias_off + n * 4ull);
    float s = 0.0f;
    if constexpr (UPB == 0) s = ldg<float>(p.compact + L.scale_off + n * 4ull);
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const uint32_t m = row0 + 16 * t + kg * 4 + r;
        if (m >= p.m) continue;
        float v = acc[t][c][r];
        if constexpr (UPB == 0) v = float(d[t][c][r] + d2[t][c][r] - 256 * nzp_r[t][r] * int(L.quads * 4)) * s;
        finish_store<T>(p.out + (uint64_t(m) * p.n + n) * item, v, bits_f32(ldg<uint32_t>(p.rows + 8ull * m)), p.has_bias != 0, bias);
      }
  }
}

template <class T, int RT, int CT>
int launch_rows(const Q4CParams& p, const MatrixLayout& M, uint32_t m0, uint32_t rows, hipStream_t stream) {
  const dim3 grid((M.tiles + 4 * CT - 1) / (4 * CT), (rows + 16 * RT - 1) / (16 * RT));
  switch (M.upb) {
    case 0: hipLaunchKernelGGL((qmm4m_rows<T, 0, RT, CT>), grid, dim3(256), 0, stream, p, M, m0); break;
    case 1: hipLaunchKernelGGL((qmm4m_rows<T, 1, RT, CT>), grid, dim3(256), 0, stream, p, M, m0); break;
    case 2: hipLaunchKernelGGL((qmm4m_rows<T, 2, RT, CT>), grid, dim3(256), 0, stream, p, M, m0); break;
    case 4: hipLaunchKernelGGL((qmm4m_rows<T, 4, RT, CT>), grid, dim3(256), 0, stream, p, M, m0); break;
    case 8: hipLaunchKernelGGL((qmm4m_rows<T, 8, RT, CT>), grid, dim3(256), 0, stream, p, M, m0); break;
    default: return -1;
  }
  return 0;
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

template <class T, int MR, int UPB, int XG, int TEAMS>
int launch_stream_one(const Q4CParams& p, const CompactLayout& L, uint32_t m0, uint32_t groupwise, hipStream_t stream,
                      std::string* err) {
  auto kernel = qmm4c_stream<T, MR, UPB, XG, TEAMS>;
  const uint32_t lds = q_lds_bytes(MR, L.kpad, TEAMS);
  static uint32_t reserved = 48 * 1024;  // guarded by the runtime's stream mutex
  if (lds > reserved) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, lds) !=
        hipSuccess) {
      (void)hipGetLastError();
      *err = "qmm4c: cannot reserve " + std::to_string(lds) + " bytes of LDS";
      return -1;
    }
    reserved = lds;
  }
  hipLaunchKernelGGL(kernel, dim3((L.tiles + TEAMS - 1) / TEAMS), dim3(256 * TEAMS), lds, stream, p, L, m0, groupwise);
  return 0;
}

// Several tiles per workgroup only where the kernel keeps to its registers with 512 or 768 threads (blocks of 32 and
// 64 values up to three rows, blocks of 128 at two rows, or three rows and two tiles): the other forms spill 100 to
// 760 bytes per lane and run with one tile per workgroup.
template <int MR, int UPB, int TEAMS>
constexpr int kTeamsThatFit = TEAMS == 1 || (MR <= 3 && (UPB == 1 || UPB == 2)) || (UPB == 4 && (MR == 2 || (MR == 3 && TEAMS == 2))) ? TEAMS : 1;

template <class T, int MR, int XG, int TEAMS>
int launch_stream_upb(const Q4CParams& p, const CompactLayout& L, uint32_t m0, uint32_t groupwise, hipStream_t stream,
                      std::string* err) {
  switch (L.upb) {
    case 0: return launch_stream_one<T, MR, 0, XG, kTeamsThatFit<MR, 0, TEAMS>>(p, L, m0, groupwise, stream, err);
    case 1: return launch_stream_one<T, MR, 1, XG, kTeamsThatFit<MR, 1, TEAMS>>(p, L, m0, groupwise, stream, err);
    case 2: return launch_stream_one<T, MR, 2, XG, kTeamsThatFit<MR, 2, TEAMS>>(p, L, m0, groupwise, stream, err);
    case 4: return launch_stream_one<T, MR, 4, XG, kTeamsThatFit<MR, 4, TEAMS>>(p, L, m0, groupwise, stream, err);
    case 8: return launch_stream_one<T, MR, 8, XG, kTeamsThatFit<MR, 8, TEAMS>>(p, L, m0, groupwise, stream, err);
  }
  *err = "qmm4c: bad layout";
  return -1;
}

// Column tiles per workgroup.  Every workgroup reads (and, fused, quantises) the activation rows for itself.  With
// two rows and more, and up to three tiles per compute unit, one workgroup per unit with that many tiles is ~10 %
// faster than as many workgroups (K = 4096, 2 rows, 256 units: 8192 columns 8.8 against 9.8 us, 11008 columns 11.0
// against 12.3).  With one row it is level to slower (the launch is a chain of waits, not of bytes, and three
// workgroups a unit that start at different times overlap their waits better than twelve waves in step), and so it
// is with more workgroups than units (16384 columns as 512 workgroups of two tiles: 16.1 against 14.5 us).
inline int stream_teams(const CompactLayout& L, uint32_t rows, int cus) {
  const uint32_t per_unit = (L.tiles + cus - 1) / cus;
  return rows >= 2 && per_unit <= 3 && q_lds_bytes(rows, L.kpad, per_unit) <= 144 * 1024 ? int(per_unit) : 1;
}

template <class T, int MR, int XG>
int launch_stream_teams(const Q4CParams& p, const CompactLayout& L, uint32_t m0, uint32_t groupwise, int teams,
                        hipStream_t stream, std::string* err) {
  // (several tiles per workgroup only in the fused form for rows of up to 4096 values, the one decode runs on, and
  // only with two rows and more)
  if constexpr (XG == 2 && MR >= 2) {
    if (teams == 3) return launch_stream_upb<T, MR, XG, 3>(p, L, m0, groupwise, stream, err);
    if (teams == 2) return launch_stream_upb<T, MR, XG, 2>(p, L, m0, groupwise, stream, err);
  }
  return launch_stream_upb<T, MR, XG, 1>(p, L, m0, groupwise, stream, err);
}

// Rows in groups of at most 4 (fewer when the activations of 4 rows would not fit in LDS).
// forced_teams: 0 = by the rule above.
template <class T, int XG>
int launch_stream_rows(const Q4CParams& p, const CompactLayout& L, uint32_t groupwise, uint32_t forced_teams, int cus,
                       hipStream_t stream, std::string* err) {
  uint32_t per = 4;
  while (per > 1 && q_lds_bytes(per, L.kpad) > 144 * 1024) per /= 2;
  if (q_lds_bytes(per, L.kpad) > 144 * 1024) {
    *err = "qmm4c: k too large for the streaming kernel";
    return -1;
  }
  for (uint32_t m0 = 0; m0 < p.m; m0 += per) {
    const uint32_t rows = p.m - m0 < per ? p.m - m0 : per;
    int teams = XG == 2 ? stream_teams(L, rows, cus) : 1;
    if (forced_teams != 0 && q_lds_bytes(rows, L.kpad, forced_teams) <= 144 * 1024) teams = int(forced_teams);
    int rc;
    if (rows >= 4) rc = launch_stream_teams<T, 4, XG>(p, L, m0, groupwise, teams, stream, err);
    else if (rows == 3) rc = launch_stream_teams<T, 3, XG>(p, L, m0, groupwise, teams, stream, err);
    else if (rows == 2) rc = launch_stream_teams<T, 2, XG>(p, L, m0, groupwise, teams, stream, err);
    else rc = launch_stream_teams<T, 1, XG>(p, L, m0, groupwise, teams, stream, err);
    if (rc != 0) return rc;
  }
  return 0;
}

}  // namespace

uint64_t qmm4c_bytes(uint32_t n, uint32_t k, uint32_t bs) {
  CompactLayout L;
  MatrixLayout M;
  if (!compact_layout(n, k, bs, &L) || !matrix_layout(n, k, bs, &M)) return 0;
  return L.total > M.total ? L.total : M.total;  // either layout fits
}

uint64_t qmm4c_q_bytes(uint32_t m, uint32_t k) {
  if (m == 0 || k == 0) return 0;
  const uint64_t nunits = (k + kUnit - 1) / kUnit, rounds = (nunits + kRoundUnits - 1) / kRoundUnits;
  const uint64_t streaming = uint64_t(m) * rounds * kRoundUnits * kUnit;
  const uint64_t matrix = uint64_t((m + 15) / 16) * ((nunits + 63) / 64 * 16) * 2048;
  return round_up_u64(streaming > matrix ? streaming : matrix, 256);
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

int launch_qmm4c_pack(const Q4PackParams& p, uint32_t layout, const Machine&, hipStream_t stream, std::string* err) {
  CompactLayout L;
  MatrixLayout M;
  if (!check_q4_shape(1, p.n, p.k, p.bs, err)) return -1;
  if (!compact_layout(p.n, p.k, p.bs, &L) || !matrix_layout(p.n, p.k, p.bs, &M)) {
    *err = "qmm4c_pack: this shape has no compact form (groupwise block sizes: 32, 64, 128, 256)";
    return -1;
  }
  if (layout > 1) {
    *err = "qmm4c_pack: LAYOUT must be 0 (streaming) or 1 (matrix cores)";
    return -1;
  }
  if (!p.packed || !p.compact || (p.compact & 15)) {
    *err = "qmm4c_pack: null or unaligned address";
    return -1;
  }
  const uint64_t threads = layout == 0 ? L.nib_bytes / 16 + (L.upb ? L.scale_bytes / 4 : p.n) + p.n
                                       : M.nib_bytes / 16 + (M.upb ? M.scale_bytes / 4 : p.n) + p.n;
  const uint64_t groups = (threads + 255) / 256;
  if (groups >= (1ull << 31)) {
    *err = "qmm4c_pack: too large";
    return -1;
  }
  if (layout == 0) hipLaunchKernelGGL(qmm4c_pack_kernel, dim3(uint32_t(groups)), dim3(256), 0, stream, p, L);
  else hipLaunchKernelGGL(qmm4m_pack_kernel, dim3(uint32_t(groups)), dim3(256), 0, stream, p, M);
  if (hipGetLastError() != hipSuccess) {
    *err = "qmm4c_pack: kernel launch failed";
    return -1;
  }
  return 0;
}

// The matrix-layout form of the product: phase 0, 1 or 2 (= 0 then 1).
template <class T>
int launch_matrix(const Q4CParams& p, uint32_t phase_and_flags, uint32_t groupwise, hipStream_t stream, std::string* err) {
  constexpr uint32_t item = sizeof(typename T::storage);
  const uint32_t phase = phase_and_flags & 15u, flags = phase_and_flags & ~15u;
  MatrixLayout M;
  if (!matrix_layout(p.n, p.k, p.bs, &M)) {
    *err = "qmm4c: this shape has no compact form (groupwise block sizes: 32, 64, 128, 256)";
    return -1;
  }
  if (!p.q || !p.rows || (p.q & 15)) {
    *err = "qmm4c: null or unaligned tensor address";
    return -1;
  }
  if (phase == 0 || phase == 2) {
    if (p.m > 65535) {
      *err = "qmm4c: at most 65535 rows per dispatch";
      return -1;
    }
    const bool fast = p.k % 8 == 0 && p.k <= 2048u * kFusedGroups && (p.inp & 15) == 0 && (uint64_t(p.k) * item) % 16 == 0;
    if (fast) hipLaunchKernelGGL((qmm4m_rowquant<T, true>), dim3(p.m), dim3(256), 0, stream, p, groupwise, M.quads);
    else hipLaunchKernelGGL((qmm4m_rowquant<T, false>), dim3(p.m), dim3(256), 0, stream, p, groupwise, M.quads);
  }
  if (phase == 1 || phase == 2) {
    if (!p.compact || (p.compact & 15)) {
      *err = "qmm4c: null or unaligned side-car address";
      return -1;
    }
    // Enough row tiles x column tiles to give every SIMD two waves (two and a half channelwise): a wave per tile walks all of K; fewer: the
    // one-row-tile kernel, whose four waves split K.  Phase values 1 | 2 with bit 4 (16) set keep the one-row-tile
    // kernel, with bit 5 (32) force the wave-per-tile kernel (tests, tuning).
    const bool rows_kernel = ((uint64_t((p.m + 15) / 16) * M.tiles >= (M.upb ? 2048u : 2560u) && !(flags & 16)) || (flags & 32));
    // (wave tiles of 2 x 2, 2 x 1 or 1 x 1 matrix-core tiles: the largest that leaves every SIMD two and a half
    //  waves; flag bits 6-7 choose: 1 = 1 x 1, 2 = 2 x 1, 3 = 2 x 2)
    for (uint32_t m0 = 0; rows_kernel && m0 < p.m; m0 += 16 * 1024) {
      const uint32_t rows = p.m - m0 < 16 * 1024 ? p.m - m0 : 16 * 1024;
      uint32_t shape = (flags >> 6) & 3u;
      if (shape == 0)
        shape = uint64_t((rows + 31) / 32) * ((M.tiles + 1) / 2) >= 2560 ? 3 : uint64_t((rows + 31) / 32) * M.tiles >= 2560 ? 2 : 1;
      const int rc = shape == 3 ? launch_rows<T, 2, 2>(p, M, m0, rows, stream)
                   : shape == 2 ? launch_rows<T, 2, 1>(p, M, m0, rows, stream)
                                : launch_rows<T, 1, 1>(p, M, m0, rows, stream);
      if (rc != 0) {
        *err = "qmm4c: bad layout";
        return -1;
      }
    }
    for (uint32_t m0 = 0; !rows_kernel && m0 < p.m; m0 += 16 * 1024) {
      const uint32_t rows = p.m - m0 < 16 * 1024 ? p.m - m0 : 16 * 1024;
      const dim3 grid(M.tiles, (rows + 15) / 16);
      switch (M.upb) {
        case 0: hipLaunchKernelGGL((qmm4m_tile<T, 0>), grid, dim3(256), 0, stream, p, M, m0); break;
        case 1: hipLaunchKernelGGL((qmm4m_tile<T, 1>), grid, dim3(256), 0, stream, p, M, m0); break;
        case 2: hipLaunchKernelGGL((qmm4m_tile<T, 2>), grid, dim3(256), 0, stream, p, M, m0); break;
        case 4: hipLaunchKernelGGL((qmm4m_tile<T, 4>), grid, dim3(256), 0, stream, p, M, m0); break;
        case 8: hipLaunchKernelGGL((qmm4m_tile<T, 8>), grid, dim3(256), 0, stream, p, M, m0); break;
        default: *err = "qmm4c: bad layout"; return -1;
      }
    }
  }
  return 0;
}

int launch_qmm4c(const Q4CParams& p, int dtype, uint32_t phase, uint32_t groupwise, uint32_t layout, const Machine& mc,
                 hipStream_t stream, std::string* err) {
  if (p.m == 0 || p.n == 0) return 0;
  CompactLayout L;
  if (!check_q4_shape(p.m, p.n, p.k, p.bs, err)) return -1;
  if (layout > 1) {
    *err = "qmm4c: LAYOUT must be 0 (streaming) or 1 (matrix cores)";
    return -1;
  }
  if (layout == 1) {
    if (groupwise != (p.bs != p.k ? 1u : 0u)) {
      *err = "qmm4c: GROUPWISE must be 1 exactly when bs != k";
      return -1;
    }
    if (!p.inp || !p.out || (phase & 15u) > 2 || (phase & ~255u)) {
      *err = (phase & 15u) > 2 || (phase & ~255u) ? "qmm4c: PHASE must be 0, 1 or 2" : "qmm4c: null or unaligned tensor address";
      return -1;
    }
    const int rc = dtype == VKT_F32 ? launch_matrix<f32_t>(p, phase, groupwise, stream, err)
                                    : launch_matrix<bf16_t>(p, phase, groupwise, stream, err);
    if (rc != 0) return rc;
    if (hipGetLastError() != hipSuccess) {
      *err = "qmm4c: kernel launch failed";
      return -1;
    }
    return 0;
  }
  if (!compact_layout(p.n, p.k, p.bs, &L)) {
    *err = "qmm4c: this shape has no compact form (groupwise block sizes: 32, 64, 128, 256)";
    return -1;
  }
  if (groupwise != (p.bs != p.k ? 1u : 0u)) {
    *err = "qmm4c: GROUPWISE must be 1 exactly when bs != k";
    return -1;
  }
  // (phase 2 with 1, 2 or 3 in bits 8-9: that many column tiles per workgroup instead of the launcher's choice; tests, tuning)
  uint32_t forced_teams = 0;
  if ((phase & 255u) == 2 && (phase >> 8) <= 3) forced_teams = phase >> 8, phase = 2;
  if (!p.inp || !p.out || (phase != 2 && (!p.q || !p.rows || (p.q & 15)))) {
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
    const int rc = dtype == VKT_F32 ? launch_stream_rows<f32_t, 0>(p, L, groupwise, 0, mc.compute_units, stream, err)
                                    : launch_stream_rows<bf16_t, 0>(p, L, groupwise, 0, mc.compute_units, stream, err);
    if (rc != 0) return rc;
  } else if (phase == 2) {
    // both phases in one launch per group of rows when the rows can be quantised from
    // registers (then p.q and p.rows are not touched); otherwise phase 0, then phase 1
    if (!p.compact || (p.compact & 15)) {
      *err = "qmm4c: null or unaligned side-car address";
      return -1;
    }
    const uint32_t item = dtype == VKT_F32 ? 4 : 2;
    const bool fuse = p.k % 8 == 0 && p.k <= 2048u * kFusedGroups && (p.inp & 15) == 0 && (uint64_t(p.k) * item) % 16 == 0;
    if (!fuse) {
      int rc = launch_qmm4c(p, dtype, 0, groupwise, 0, mc, stream, err);
      if (rc == 0) rc = launch_qmm4c(p, dtype, 1, groupwise, 0, mc, stream, err);
      return rc;
    }
    // (a thread quantises 2 groups of 8 activations where that covers the row, else up to kFusedGroups)
    const bool few = p.k <= 4096;
    const int rc = dtype == VKT_F32 ? (few ? launch_stream_rows<f32_t, 2>(p, L, groupwise, forced_teams, mc.compute_units, stream, err)
                                           : launch_stream_rows<f32_t, kFusedGroups>(p, L, groupwise, 0, mc.compute_units, stream, err))
                                    : (few ? launch_stream_rows<bf16_t, 2>(p, L, groupwise, forced_teams, mc.compute_units, stream, err)
                                           : launch_stream_rows<bf16_t, kFusedGroups>(p, L, groupwise, 0, mc.compute_units, stream, err));
    if (rc != 0) return rc;
  } else {
    *err = "qmm4c: PHASE must be 0, 1 or 2";
    return -1;
  }
  if (hipGetLastError() != hipSuccess) {
    *err = "qmm4c: kernel launch failed";
    return -1;
  }
  return 0;
}

}  // namespace vkt
