// Strided data movement on gfx950: same-size copies (contiguous(), transposes, slices,
// broadcasts) and fills, behind the reference's kernel names and parameter blocks ("move_b<S>",
// shaders/move.slang; "copy8_b<S>", shaders/copy8.slang; launched from
// crates/pyvk/csrc/backend.cpp:664-671 and :806-816).  The reference moves one element per
// thread whatever the layout; here the launcher reads the strides and picks the form that keeps
// HBM accesses whole:
//   move_units      both sides contiguous along the innermost dim (or a fill): the element is
//                   widened to the largest unit (up to 16 bytes) that the sizes, strides and
//                   addresses allow, one unit per thread, consecutive lanes on consecutive units
//   move_transpose  the two sides are contiguous along different dims: 64 x 64 element tiles
//                   through LDS, read along the source's contiguous dim, written along the
//                   destination's (padded rows: no bank conflicts either way)
//   move_units      anything else (broadcast sources, strided innermost dims): element by element
// All are pure byte moves: results are bit-exact whatever the element type.
#include "kernels.h"
#include "strided.h"
#include <cstring>

namespace vkt {
namespace {

template <class X>
__device__ __forceinline__ X fill_unit(const MovePlan& p);
template <>
__device__ __forceinline__ uint8_t fill_unit<uint8_t>(const MovePlan& p) { return uint8_t(p.fill[0]); }
template <>
__device__ __forceinline__ uint16_t fill_unit<uint16_t>(const MovePlan& p) { return uint16_t(p.fill[0]); }
template <>
__device__ __forceinline__ uint32_t fill_unit<uint32_t>(const MovePlan& p) { return p.fill[0]; }
template <>
__device__ __forceinline__ U2 fill_unit<U2>(const MovePlan& p) { return U2{p.fill[0], p.fill[1]}; }
template <>
__device__ __forceinline__ U4 fill_unit<U4>(const MovePlan& p) { return U4{p.fill[0], p.fill[1], p.fill[2], p.fill[3]}; }

// One unit per thread, grid stride.  LINEAR: one dim, both strides 1 (no index arithmetic).
template <class X, bool FILL, bool LINEAR>
__global__ __launch_bounds__(256) void move_units(MovePlan p) {
  const uint64_t stride = uint64_t(gridDim.x) * 256;
  const X value = fill_unit<X>(p);
  for (uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x; i < p.n; i += stride) {
    int64_t o = int64_t(i), a = int64_t(i);
    if constexpr (!LINEAR) plan_offsets(p, uint32_t(i), &o, &a);
    if constexpr (FILL) stg<X>(p.out + o * int64_t(sizeof(X)), value);
    else stg<X>(p.out + o * int64_t(sizeof(X)), ldg<X>(p.a + a * int64_t(sizeof(X))));
  }
}

constexpr uint32_t kTile = 64;

// Block index -> tile (tp, tq); what is left in *b indexes the other dims.  Blocks that run together
// cover 16 x 16 tiles (where the counts allow) rather than a line of tiles, so that neither the
// reads nor the writes of a power-of-two transpose land on a few memory channels (+10 % measured).
__device__ __forceinline__ void tile_of_block(uint32_t* b, uint32_t tiles_p, uint32_t tiles_q, uint32_t* tp, uint32_t* tq) {
  uint32_t r = *b;
  if (tiles_p % 16 == 0 && tiles_q % 16 == 0) {
    const uint32_t in = r % 256;
    r /= 256;
    const uint32_t sp = r % (tiles_p / 16);
    r /= tiles_p / 16;
    const uint32_t sq = r % (tiles_q / 16);
    r /= tiles_q / 16;
    *tp = sp * 16 + in % 16, *tq = sq * 16 + in / 16;
  } else {
    *tq = r % tiles_q;
    r /= tiles_q;
    *tp = r % tiles_p;
    r /= tiles_p;
  }
  *b = r;
}

// Offsets (in units) of the dims other than dp and dq for the linear index b.
__device__ __forceinline__ void outer_offsets(const MovePlan& p, uint32_t b, uint32_t dp, uint32_t dq, int64_t* o, int64_t* a) {
#pragma unroll
  for (uint32_t d = 0; d < kMaxDims; ++d) {
    if (d < p.ndim && d != dp && d != dq) {
      const uint32_t s = p.size[d], q = b / s, c = b - q * s;
      b = q;
      *o += int64_t(c) * p.so[d];
      *a += int64_t(c) * p.sa[d];
    }
  }
}

// Tiles over dims dp (the destination's contiguous one) and dq (the source's); the other dims
// select the tile's origin.  Grid x = tiles_p * tiles_q * (product of the other sizes).
template <class X>
__global__ __launch_bounds__(256) void move_transpose(MovePlan p, uint32_t dp, uint32_t dq, uint32_t tiles_p, uint32_t tiles_q) {
  constexpr uint32_t S = sizeof(X), PITCH = kTile * S + (S < 4 ? 4 : S);  // odd number of words (or of 8 / 16-byte units) per row
  __shared__ __attribute__((aligned(16))) uint8_t tile[kTile * PITCH];
  uint32_t b = blockIdx.x, tp, tq;
  tile_of_block(&b, tiles_p, tiles_q, &tp, &tq);
  int64_t o = 0, a = 0;
  outer_offsets(p, b, dp, dq, &o, &a);
  const uint32_t np = p.size[dp], nq = p.size[dq], p0 = tp * kTile, q0 = tq * kTile;
  const uint32_t lane = threadIdx.x % kTile, row = threadIdx.x / kTile;
  const int64_t sap = p.sa[dp], saq = p.sa[dq], sop = p.so[dp], soq = p.so[dq];
  constexpr uint32_t PER = kTile * kTile / 256;  // elements per thread: all loads are issued before the first use
  X v[PER];
  const bool whole = p0 + kTile <= np && q0 + kTile <= nq;  // (uniform: the edge tests leave the inner tiles' loops)
  const uint64_t from = p.a + (a + (p0 + row) * sap + (q0 + lane) * saq) * int64_t(S);
  if (whole) {
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i) v[i] = ldg<X>(from + uint64_t(i) * 4 * sap * S);
  } else {
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i)
      v[i] = (p0 + row + 4 * i < np && q0 + lane < nq) ? ldg<X>(from + uint64_t(i) * 4 * sap * S) : X{};
  }
#pragma unroll
  for (uint32_t i = 0; i < PER; ++i) *reinterpret_cast<X*>(tile + (row + 4 * i) * PITCH + lane * S) = v[i];
  __syncthreads();
#pragma unroll
  for (uint32_t i = 0; i < PER; ++i) v[i] = *reinterpret_cast<const X*>(tile + lane * PITCH + (row + 4 * i) * S);
  const uint64_t to = p.out + (o + (p0 + lane) * sop + (q0 + row) * soq) * int64_t(S);
  if (whole) {
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i) stg<X>(to + uint64_t(i) * 4 * soq * S, v[i]);
  } else {
#pragma unroll
    for (uint32_t i = 0; i < PER; ++i)
      if (p0 + lane < np && q0 + row + 4 * i < nq) stg<X>(to + uint64_t(i) * 4 * soq * S, v[i]);
  }
}

constexpr uint32_t kPairTile = 128;

// The transpose of 2-byte elements in 4-byte accesses: a thread loads the same two columns of two
// adjacent source rows, regroups the four elements in registers (v_perm_b32) into the two words
// the destination holds along its contiguous dim, and the tile turns words in LDS.  Tiles of
// 128 x 128 elements: 256 contiguous bytes per wave access either side.  Even sizes and strides,
// 4-byte aligned addresses (checked by the launcher).
__global__ __launch_bounds__(256) void move_transpose_pairs(MovePlan p, uint32_t dp, uint32_t dq, uint32_t tiles_p, uint32_t tiles_q) {
  constexpr uint32_t HALF = kPairTile / 2, PITCH = HALF + 1, PER = HALF / 4;  // words per LDS row; row pairs per wave
  __shared__ uint32_t tile[kPairTile * PITCH];  // [q][p / 2]
  uint32_t b = blockIdx.x, tp, tq;
  tile_of_block(&b, tiles_p, tiles_q, &tp, &tq);
  int64_t o = 0, a = 0;
  outer_offsets(p, b, dp, dq, &o, &a);
  const uint32_t np = p.size[dp], nq = p.size[dq], p0 = tp * kPairTile, q0 = tq * kPairTile;
  const uint32_t lane = threadIdx.x % 64, wave = threadIdx.x / 64;
  const int64_t sap = p.sa[dp], soq = p.so[dq];
  const bool whole = p0 + kPairTile <= np && q0 + kPairTile <= nq;
  uint32_t lo[PER], hi[PER];
  // rows p0 + 2 (wave + 4 i) and the next one, columns q0 + 2 lane and the next one
  const uint64_t from = p.a + (a + (p0 + 2 * wave) * sap + (q0 + 2 * lane)) * 2;
#pragma unroll
  for (uint32_t i = 0; i < PER; ++i) {
    const bool in = whole || (p0 + 2 * (wave + 4 * i) < np && q0 + 2 * lane < nq);
    lo[i] = in ? ldg<uint32_t>(from + uint64_t(8 * i) * sap * 2) : 0u;
    hi[i] = in ? ldg<uint32_t>(from + uint64_t(8 * i + 1) * sap * 2) : 0u;
  }
#pragma unroll
  for (uint32_t i = 0; i < PER; ++i) {
    const uint32_t pair = wave + 4 * i;
    tile[(2 * lane) * PITCH + pair] = __builtin_amdgcn_perm(hi[i], lo[i], 0x05040100);      // column q: rows p, p + 1
    tile[(2 * lane + 1) * PITCH + pair] = __builtin_amdgcn_perm(hi[i], lo[i], 0x07060302);  // column q + 1
  }
  __syncthreads();
  // destination rows q0 + wave + 4 i, words p0 / 2 + lane
  const uint64_t to = p.out + (o + (q0 + wave) * soq + (p0 + 2 * lane)) * 2;
#pragma unroll 8
  for (uint32_t i = 0; i < kPairTile / 4; ++i) {
    const uint32_t v = tile[(wave + 4 * i) * PITCH + lane];
    if (whole || (q0 + wave + 4 * i < nq && p0 + 2 * lane < np)) stg<uint32_t>(to + uint64_t(4 * i) * soq * 2, v);
  }
}

uint32_t groups_for(uint64_t units, const Machine& mc) {
  const uint64_t want = (units + 255) / 256, cap = uint64_t(mc.compute_units) * 64;
  return uint32_t(want < 1 ? 1 : (want < cap ? want : cap));
}

// Doubles the unit while the innermost dim is contiguous on both sides and everything else stays whole.
void widen(MovePlan* p, bool fill) {
  if (p->ndim == 0 || p->so[0] != 1 || (!fill && p->sa[0] != 1)) return;
  while (p->unit < 16) {
    const uint64_t twice = uint64_t(p->unit) * 2;
    bool ok = p->size[0] % 2 == 0 && p->out % twice == 0 && (fill || p->a % twice == 0);
    for (uint32_t d = 1; d < p->ndim && ok; ++d) ok = p->so[d] % 2 == 0 && (fill || p->sa[d] % 2 == 0);
    if (!ok) return;
    p->size[0] /= 2, p->n /= 2, p->unit *= 2;
    for (uint32_t d = 1; d < p->ndim; ++d) p->so[d] /= 2, p->sa[d] /= 2;
    if (p->size[0] == 1) {  // the dim is used up: drop it (what is left is not contiguous by construction)
      for (uint32_t d = 1; d < p->ndim; ++d) p->size[d - 1] = p->size[d], p->so[d - 1] = p->so[d], p->sa[d - 1] = p->sa[d];
      --p->ndim;
      if (p->ndim == 0 || p->so[0] != 1 || (!fill && p->sa[0] != 1)) return;
    }
  }
}

template <class X, bool FILL>
void launch_units(const MovePlan& p, const Machine& mc, hipStream_t stream) {
  const bool linear = p.ndim == 0 || (p.ndim == 1 && p.so[0] == 1 && (FILL || p.sa[0] == 1));
  const dim3 grid(groups_for(p.n, mc));
  if (linear) hipLaunchKernelGGL((move_units<X, FILL, true>), grid, dim3(256), 0, stream, p);
  else hipLaunchKernelGGL((move_units<X, FILL, false>), grid, dim3(256), 0, stream, p);
}

template <bool FILL>
void launch_units_any(const MovePlan& p, const Machine& mc, hipStream_t stream) {
  switch (p.unit) {
    case 1: return launch_units<uint8_t, FILL>(p, mc, stream);
    case 2: return launch_units<uint16_t, FILL>(p, mc, stream);
    case 4: return launch_units<uint32_t, FILL>(p, mc, stream);
    case 8: return launch_units<U2, FILL>(p, mc, stream);
    default: return launch_units<U4, FILL>(p, mc, stream);
  }
}

// The dims the tiled transpose runs over, if the layout is one: the destination contiguous along
// dp, the source along another dim dq, both long enough to fill tiles.
bool transpose_dims(const MovePlan& p, uint32_t* dp, uint32_t* dq, uint64_t* blocks, uint32_t* tiles_p, uint32_t* tiles_q) {
  int bp = -1, bq = -1;
  for (uint32_t d = 0; d < p.ndim; ++d) {
    if (p.so[d] == 1 && p.sa[d] == 1) return false;  // (contiguous together: move_units is already whole)
    if (p.so[d] == 1 && (bp < 0 || p.size[d] > p.size[bp])) bp = int(d);
    if (p.sa[d] == 1 && (bq < 0 || p.size[d] > p.size[bq])) bq = int(d);
  }
  if (bp < 0 || bq < 0 || bp == bq || p.size[bp] < 16 || p.size[bq] < 16 || p.unit > 8) return false;
  *dp = uint32_t(bp), *dq = uint32_t(bq);
  *tiles_p = (p.size[bp] + kTile - 1) / kTile, *tiles_q = (p.size[bq] + kTile - 1) / kTile;
  uint64_t total = uint64_t(*tiles_p) * *tiles_q;
  for (uint32_t d = 0; d < p.ndim; ++d)
    if (int(d) != bp && int(d) != bq) total *= p.size[d];
  *blocks = total;
  return total < (1ull << 31);
}

int run_copy(MovePlan p, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err) {
  // variant 0: planned; 1: element by element as given; 2: widened units only (no transpose)
  if (variant > 2) {
    *err = "move: unknown variant " + std::to_string(variant);
    return -1;
  }
  uint32_t dp, dq, tiles_p, tiles_q;
  uint64_t blocks;
  if (variant == 0 && transpose_dims(p, &dp, &dq, &blocks, &tiles_p, &tiles_q)) {
    if (p.unit == 2 && p.size[dp] >= 64 && p.size[dq] >= 64) {
      bool even = p.size[dp] % 2 == 0 && p.size[dq] % 2 == 0 && p.a % 4 == 0 && p.out % 4 == 0;
      for (uint32_t d = 0; d < p.ndim && even; ++d) even = (d == dq || p.sa[d] % 2 == 0) && (d == dp || p.so[d] % 2 == 0);
      const uint32_t pairs_p = (p.size[dp] + kPairTile - 1) / kPairTile, pairs_q = (p.size[dq] + kPairTile - 1) / kPairTile;
      const uint64_t total = blocks / (uint64_t(tiles_p) * tiles_q) * pairs_p * pairs_q;
      if (even) {
        hipLaunchKernelGGL(move_transpose_pairs, dim3(uint32_t(total)), dim3(256), 0, stream, p, dp, dq, pairs_p, pairs_q);
        return 0;
      }
    }
    const dim3 grid{uint32_t(blocks)};
    switch (p.unit) {
      case 1: hipLaunchKernelGGL((move_transpose<uint8_t>), grid, dim3(256), 0, stream, p, dp, dq, tiles_p, tiles_q); break;
      case 2: hipLaunchKernelGGL((move_transpose<uint16_t>), grid, dim3(256), 0, stream, p, dp, dq, tiles_p, tiles_q); break;
      case 4: hipLaunchKernelGGL((move_transpose<uint32_t>), grid, dim3(256), 0, stream, p, dp, dq, tiles_p, tiles_q); break;
      default: hipLaunchKernelGGL((move_transpose<U2>), grid, dim3(256), 0, stream, p, dp, dq, tiles_p, tiles_q); break;
    }
    return 0;
  }
  if (variant != 1) widen(&p, false);
  launch_units_any<false>(p, mc, stream);
  return 0;
}

uint32_t item_of(const char* label) {
  if (!std::strcmp(label, "b1")) return 1;
  if (!std::strcmp(label, "b2")) return 2;
  if (!std::strcmp(label, "b4")) return 4;
  if (!std::strcmp(label, "b8")) return 8;
  if (!std::strcmp(label, "b16")) return 16;
  return 0;
}

int finish(int rc, std::string* err) {
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "move: kernel launch failed";
    return -1;
  }
  return rc;
}

}  // namespace

int launch_move(const StridedParams& s, const char* size_label, uint32_t op, uint32_t variant, const Machine& mc,
                hipStream_t stream, std::string* err) {
  const uint32_t item = item_of(size_label);
  if (item == 0) {
    *err = std::string("unknown kernel move_") + size_label;
    return -1;
  }
  if (op != VKT_MOVE_COPY && op != VKT_MOVE_FILL) {
    *err = "move: only the copy and fill opcodes are built (gather / scatter are not)";
    return -1;
  }
  if (s.n == 0) return 0;
  if (!s.out || (op == VKT_MOVE_COPY && !s.a) || s.out % item != 0 || (op == VKT_MOVE_COPY && s.a % item != 0)) {
    *err = "move: null or misaligned tensor address";
    return -1;
  }
  MovePlan p;
  if (!plan_from(s.out, s.a, s.n, s.ndim, 4, s.size, s.so, op == VKT_MOVE_COPY ? s.sa : nullptr, item, "move", &p, err)) return -1;
  if (op == VKT_MOVE_COPY) return finish(run_copy(p, variant, mc, stream, err), err);
  // the element's bits, repeated over 16 bytes
  uint8_t bytes[16], pattern[16];
  std::memcpy(bytes, &s.alpha, 8);
  std::memcpy(bytes + 8, &s.beta, 8);
  for (uint32_t i = 0; i < 16; ++i) pattern[i] = bytes[i % item];
  std::memcpy(p.fill, pattern, 16);
  if (variant != 1) widen(&p, true);
  launch_units_any<true>(p, mc, stream);
  return finish(0, err);
}

int launch_copy8(const Copy8Params& c, const char* size_label, uint32_t variant, const Machine& mc, hipStream_t stream,
                 std::string* err) {
  const uint32_t item = item_of(size_label);
  if (item == 0) {
    *err = std::string("unknown kernel copy8_") + size_label;
    return -1;
  }
  if (c.n == 0) return 0;
  if (!c.out || !c.a || c.out % item != 0 || c.a % item != 0) {
    *err = "copy8: null or misaligned tensor address";
    return -1;
  }
  MovePlan p;
  if (!plan_from(c.out, c.a, c.n, c.ndim, 8, c.size, c.so, c.sa, item, "copy8", &p, err)) return -1;
  return finish(run_copy(p, variant, mc, stream, err), err);
}

}  // namespace vkt
