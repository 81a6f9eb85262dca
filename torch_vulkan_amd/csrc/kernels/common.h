// Device helpers shared by the gfx950 kernels: 16-byte loads, element conversions with
// the rounding the operators specify, and wave64 reductions through DPP.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../../include/vkt.h"

namespace vkt {

constexpr int kWave = 64;

__host__ __device__ inline uint64_t round_up_u64(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

using U4 = uint32_t __attribute__((ext_vector_type(4)));
using U2 = uint32_t __attribute__((ext_vector_type(2)));
using F4 = float __attribute__((ext_vector_type(4)));

// Tensor addresses arrive as 64-bit integers in the parameter blocks; loads and stores go
// through global-address-space pointers so that they compile to global_* (not flat_*)
// memory instructions.
#define VKT_GLOBAL __attribute__((address_space(1)))
template <class X>
__device__ __forceinline__ X ldg(uint64_t addr) {
  return *reinterpret_cast<const VKT_GLOBAL X*>(addr);
}
// A load of data that is read exactly once (the weight stream): non-temporal, so that it
// does not displace the activations and scales that every wave re-reads from L2.
template <class X>
__device__ __forceinline__ X ldg_stream(uint64_t addr) {
  return __builtin_nontemporal_load(reinterpret_cast<const VKT_GLOBAL X*>(addr));
}
template <class X>
__device__ __forceinline__ void stg(uint64_t addr, X v) {
  *reinterpret_cast<VKT_GLOBAL X*>(addr) = v;
}

// A store of data that this kernel does not read again (a streamed output): non-temporal.
template <class X>
__device__ __forceinline__ void stg_stream(uint64_t addr, X v) {
  __builtin_nontemporal_store(v, reinterpret_cast<VKT_GLOBAL X*>(addr));
}

__device__ __forceinline__ float bits_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
inline float bits_f32_host(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f32_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// Storage element types.  16-bit floats are carried as raw bits so that every rounding
// is written out here and not left to a library type.
struct f32_t {
  using storage = float;
  static constexpr int dtype = VKT_F32;
};
struct f16_t {
  using storage = uint16_t;
  static constexpr int dtype = VKT_F16;
};
struct bf16_t {
  using storage = uint16_t;
  static constexpr int dtype = VKT_BF16;
};

__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return bits_f32(h << 16); }
// round to nearest even; NaN -> 0x7fc0
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  uint32_t r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
  return (f != f) ? uint16_t(0x7fc0) : uint16_t(r);
}
__device__ __forceinline__ float f16_to_f32(uint32_t h) {
  return float(__builtin_bit_cast(_Float16, uint16_t(h)));  // v_cvt_f32_f16: exact
}
__device__ __forceinline__ uint16_t f32_to_f16(float f) {
  return __builtin_bit_cast(uint16_t, _Float16(f));  // v_cvt_f16_f32: round to nearest even (default mode)
}

// One element at a byte address, widened to / rounded from float32.
template <class T>
__device__ __forceinline__ float load_f32(uint64_t addr);
template <>
__device__ __forceinline__ float load_f32<f32_t>(uint64_t addr) { return ldg<float>(addr); }
template <>
__device__ __forceinline__ float load_f32<f16_t>(uint64_t addr) { return f16_to_f32(ldg<uint16_t>(addr)); }
template <>
__device__ __forceinline__ float load_f32<bf16_t>(uint64_t addr) { return bf16_to_f32(ldg<uint16_t>(addr)); }

template <class T>
__device__ __forceinline__ void store_f32(uint64_t addr, float v);
template <>
__device__ __forceinline__ void store_f32<f32_t>(uint64_t addr, float v) { stg<float>(addr, v); }
template <>
__device__ __forceinline__ void store_f32<f16_t>(uint64_t addr, float v) { stg<uint16_t>(addr, f32_to_f16(v)); }
template <>
__device__ __forceinline__ void store_f32<bf16_t>(uint64_t addr, float v) { stg<uint16_t>(addr, f32_to_bf16(v)); }

// 16 consecutive elements (16-byte aligned address) widened to float32.
template <class T>
__device__ __forceinline__ void load16_f32(uint64_t addr, float (&a)[16]);
template <>
__device__ __forceinline__ void load16_f32<f32_t>(uint64_t addr, float (&a)[16]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    F4 v = ldg<F4>(addr + 16 * i);
    a[4 * i] = v.x, a[4 * i + 1] = v.y, a[4 * i + 2] = v.z, a[4 * i + 3] = v.w;
  }
}
template <>
__device__ __forceinline__ void load16_f32<bf16_t>(uint64_t addr, float (&a)[16]) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    U4 v = ldg<U4>(addr + 16 * i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[8 * i + 2 * j] = bits_f32(v[j] << 16);
      a[8 * i + 2 * j + 1] = bits_f32(v[j] & 0xffff0000u);
    }
  }
}
template <>
__device__ __forceinline__ void load16_f32<f16_t>(uint64_t addr, float (&a)[16]) {
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    U4 v = ldg<U4>(addr + 16 * i);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      a[8 * i + 2 * j] = f16_to_f32(v[j] & 0xffffu);
      a[8 * i + 2 * j + 1] = f16_to_f32(v[j] >> 16);
    }
  }
}

// 16 int8 values (one 16-byte load) widened to float32 (exact).
__device__ __forceinline__ void widen16_i8(const U4& v, float (&w)[16]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
#pragma unroll
    for (int j = 0; j < 4; ++j) w[4 * i + j] = float(int(int8_t(v[i] >> (8 * j))));
  }
}

// ---- float8 element conversions (exact decode; encode as c10 converts: round to nearest even,
// e4m3fn overflow -> NaN, e5m2 overflow -> inf) ----
__device__ __forceinline__ float fp8_to_f32(uint32_t c, int fmt) {
  const uint32_t sign = (c & 0x80u) << 24;
  if (fmt == VKT_E4M3) {
    const uint32_t e = (c >> 3) & 15u, m = c & 7u;
    if (e == 15 && m == 7) return bits_f32(sign | 0x7ff00000u);
    if (e == 0) return bits_f32(sign | f32_bits(float(m) * 0.001953125f));  // m * 2^-9
    return bits_f32(sign | ((e + 120u) << 23) | (m << 20));
  }
  const uint32_t e = (c >> 2) & 31u, m = c & 3u;
  if (e == 31) return bits_f32(sign | 0x7f800000u | (m << 21));
  if (e == 0) return bits_f32(sign | f32_bits(float(m) * 1.52587890625e-05f));  // m * 2^-16
  return bits_f32(sign | ((e + 112u) << 23) | (m << 21));
}

__device__ __forceinline__ uint32_t f32_to_fp8(float f, int fmt) {
  const uint32_t u = f32_bits(f), sign = (u >> 24) & 0x80u, mag = u & 0x7fffffffu;
  const int mbits = fmt == VKT_E4M3 ? 3 : 2, bias = fmt == VKT_E4M3 ? 7 : 15;
  if (mag > 0x7f800000u) return sign | 0x7fu;
  if (fmt == VKT_E4M3) {
    if (mag >= 0x43f00000u) return sign | 0x7fu;  // >= 480: NaN (no saturation)
  } else {
    if (mag >= 0x47800000u) return sign | 0x7cu;  // >= 65536: inf
  }
  if ((mag >> 23) == 0) return sign;  // zero and float32 denormals
  const int e = int(mag >> 23) - 127, emin = 1 - bias;
  const uint32_t m = (mag & 0x7fffffu) | 0x800000u;
  const int shift = 23 - mbits + (e < emin ? emin - e : 0);
  if (shift > 25) return sign;
  uint32_t keep = m >> shift;
  const uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1u))) ++keep;
  const uint32_t out = e < emin ? keep : ((uint32_t(e + bias) << mbits) + (keep - (1u << mbits)));
  return sign | out;
}

// Two float32 -> two float8 codes (low 16 bits) with the hardware conversion.  On gfx950
// v_cvt_pk_fp8_f32 / v_cvt_pk_bf8_f32 agree with f32_to_fp8 above on every one of the 2^32
// float32 bit patterns that is not a NaN (checked exhaustively on the device: overflow to
// NaN / inf, subnormals and ties included); a NaN comes out with another payload, so NaNs are
// given the code c10 writes, sign | 0x7f.
template <int FMT>
__device__ __forceinline__ uint32_t pack2_fp8(float a, float b) {
  const uint32_t na = ((f32_bits(a) >> 24) & 0x80u) | 0x7fu, nb = ((f32_bits(b) >> 24) & 0x80u) | 0x7fu;
  uint32_t r;
  if constexpr (FMT == VKT_E4M3) r = uint32_t(__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false));
  else r = uint32_t(__builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false));
  const uint32_t ca = a != a ? na : (r & 0xffu), cb = b != b ? nb : ((r >> 8) & 0xffu);
  return ca | cb << 8;
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

// Four float32 -> four bfloat16 in two words, as pack_bf16 writes them.  NaN is rare: one comparison per pair of values
// and one branch of the whole wave decide whether any lane has to look at its values one by one.
__device__ __forceinline__ void pack_bf16x4(const float (&v)[4], uint32_t (&packed)[2]) {
  using V2 = __bf16 __attribute__((ext_vector_type(2)));
  const bool odd = __builtin_isunordered(v[0], v[1]) | __builtin_isunordered(v[2], v[3]);
  if (__builtin_amdgcn_ballot_w64(odd) != 0) {
    packed[0] = pack_bf16(v[0], v[1]), packed[1] = pack_bf16(v[2], v[3]);
  } else {
    packed[0] = __builtin_bit_cast(uint32_t, V2{static_cast<__bf16>(v[0]), static_cast<__bf16>(v[1])});
    packed[1] = __builtin_bit_cast(uint32_t, V2{static_cast<__bf16>(v[2]), static_cast<__bf16>(v[3])});
  }
}

// Four float32 -> four values of the 16-bit type T in two words.
template <class T>
__device__ __forceinline__ void pack_16bit_x4(const float (&v)[4], uint32_t (&packed)[2]) {
  if constexpr (T::dtype == VKT_BF16) {
    pack_bf16x4(v, packed);
  } else {
    packed[0] = uint32_t(f32_to_f16(v[0])) | uint32_t(f32_to_f16(v[1])) << 16;
    packed[1] = uint32_t(f32_to_f16(v[2])) | uint32_t(f32_to_f16(v[3])) << 16;
  }
}

// ---- wave64 reductions through DPP (no LDS traffic) ----
template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp_f32(float v) {
  return __builtin_bit_cast(
      float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xf, true));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
constexpr int kQuadSwap1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kQuadSwap2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kRowHalfMirror = 0x141;
constexpr int kRowMirror = 0x140;

// Sum over each row of 16 lanes, left in every lane of the row.
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_f32<kQuadSwap1>(v);
  v += dpp_f32<kQuadSwap2>(v);
  v += dpp_f32<kRowHalfMirror>(v);
  v += dpp_f32<kRowMirror>(v);
  return v;
}
// Sum over the 64 lanes (wave-uniform result).
__device__ __forceinline__ float wave_sum(float v) {
  v = row16_sum(v);
  int b = __builtin_bit_cast(int, v);
  float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  float s2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  float s3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return (s0 + s1) + (s2 + s3);
}
__device__ __forceinline__ float wave_min(float v) {
  v = fminf(v, dpp_f32<kQuadSwap1>(v));
  v = fminf(v, dpp_f32<kQuadSwap2>(v));
  v = fminf(v, dpp_f32<kRowHalfMirror>(v));
  v = fminf(v, dpp_f32<kRowMirror>(v));
  int b = __builtin_bit_cast(int, v);
  float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  float s2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  float s3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return fminf(fminf(s0, s1), fminf(s2, s3));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp_f32<kQuadSwap1>(v));
  v = fmaxf(v, dpp_f32<kQuadSwap2>(v));
  v = fmaxf(v, dpp_f32<kRowHalfMirror>(v));
  v = fmaxf(v, dpp_f32<kRowMirror>(v));
  int b = __builtin_bit_cast(int, v);
  float s0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0));
  float s1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16));
  float s2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32));
  float s3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
  return fmaxf(fmaxf(s0, s1), fmaxf(s2, s3));
}

}  // namespace vkt
