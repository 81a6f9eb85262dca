// The float8 steps either side of aten::_scaled_mm, as HBM-streaming kernels:
//   cast_fp8    elementwise conversion where one side is float8 (e4m3fn / e5m2) and the other
//               float32 / float16 / bfloat16, bit for bit as the CPU converts: through float32,
//               round to nearest even, e4m3fn overflow -> NaN, e5m2 overflow -> inf (the reference
//               builds the same mapping from c10's own conversions as lookup tables,
//               crates/pyvk/csrc/backend.cpp:486-586; its test is
//               tests/python/test_fallback_ops.py:469-485).
//   fp8_quant   the producer in front of _scaled_mm: per row (or with one given scale)
//                 a     = max(max_k |x[m,k]|, 1e-12)         (NaN elements do not count)
//                 scale = a / fmax                           (what _scaled_mm takes as scale_a)
//                 q     = cast(clamp(x * (fmax / a), -fmax, fmax))
//               every step a single float32 operation, fmax = 448 (e4m3fn) or 57344 (e5m2).
//               The reference has no such kernel (its float8 tensors come from casts alone).
// Both read and write each byte once: 16 elements per thread, 16-byte accesses.
#include "kernels.h"
#include "strided.h"

namespace vkt {
namespace {

inline bool is_fp8_host(uint32_t dt) { return dt == VKT_E4M3 || dt == VKT_E5M2; }
__host__ __device__ inline uint32_t item_size(uint32_t dt) { return dt == VKT_F32 ? 4 : (dt == VKT_F16 || dt == VKT_BF16 ? 2 : 1); }

// 16 consecutive elements of any supported type, as float32 (address aligned to 16 elements).
template <uint32_t DT>
__device__ __forceinline__ void load16_any(uint64_t addr, float (&x)[16]) {
  if constexpr (DT == VKT_F32) load16_f32<f32_t>(addr, x);
  else if constexpr (DT == VKT_F16) load16_f32<f16_t>(addr, x);
  else if constexpr (DT == VKT_BF16) load16_f32<bf16_t>(addr, x);
  else {
    const U4 v = ldg<U4>(addr);
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = fp8_to_f32((v[i / 4] >> (8 * (i % 4))) & 0xffu, int(DT));
  }
}
template <uint32_t DT>
__device__ __forceinline__ float load1_any(uint64_t base, uint64_t i) {
  if constexpr (DT == VKT_F32) return ldg<float>(base + 4 * i);
  else if constexpr (DT == VKT_F16) return f16_to_f32(ldg<uint16_t>(base + 2 * i));
  else if constexpr (DT == VKT_BF16) return bf16_to_f32(ldg<uint16_t>(base + 2 * i));
  else return fp8_to_f32(ldg<uint8_t>(base + i), int(DT));
}
template <uint32_t DT>
__device__ __forceinline__ void store16_any(uint64_t addr, const float (&x)[16]) {
  if constexpr (DT == VKT_F32) {
#pragma unroll
    for (int i = 0; i < 4; ++i) stg<F4>(addr + 16 * i, F4{x[4 * i], x[4 * i + 1], x[4 * i + 2], x[4 * i + 3]});
  } else if constexpr (DT == VKT_F16 || DT == VKT_BF16) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      U4 v;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float a = x[8 * h + 2 * j], b = x[8 * h + 2 * j + 1];
        v[j] = DT == VKT_F16 ? uint32_t(f32_to_f16(a)) | uint32_t(f32_to_f16(b)) << 16
                             : uint32_t(f32_to_bf16(a)) | uint32_t(f32_to_bf16(b)) << 16;
      }
      stg<U4>(addr + 16 * h, v);
    }
  } else {
    U4 v;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = pack2_fp8<int(DT)>(x[4 * j], x[4 * j + 1]) | pack2_fp8<int(DT)>(x[4 * j + 2], x[4 * j + 3]) << 16;
    stg<U4>(addr, v);
  }
}
template <uint32_t DT>
__device__ __forceinline__ void store1_any(uint64_t base, uint64_t i, float v) {
  if constexpr (DT == VKT_F32) stg<float>(base + 4 * i, v);
  else if constexpr (DT == VKT_F16) stg<uint16_t>(base + 2 * i, f32_to_f16(v));
  else if constexpr (DT == VKT_BF16) stg<uint16_t>(base + 2 * i, f32_to_bf16(v));
  else stg<uint8_t>(base + i, uint8_t(f32_to_fp8(v, int(DT))));
}

// One thread per 16 elements (grid stride); `vector` when both addresses are aligned to 16
// elements of their types, else element by element.
template <uint32_t SRC, uint32_t DST>
__global__ __launch_bounds__(256) void cast_kernel(CastParams p, uint32_t vector) {
  const uint64_t stride = uint64_t(gridDim.x) * 256, i0 = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (vector) {
    const uint64_t body = p.n / 16;
    for (uint64_t j = i0; j < body; j += stride) {
      float x[16];
      load16_any<SRC>(p.src + j * 16 * item_size(SRC), x);
      store16_any<DST>(p.dst + j * 16 * item_size(DST), x);
    }
    if (i0 < (p.n & 15)) store1_any<DST>(p.dst, body * 16 + i0, load1_any<SRC>(p.src, body * 16 + i0));
  } else {
    for (uint64_t j = i0; j < p.n; j += stride) store1_any<DST>(p.dst, j, load1_any<SRC>(p.src, j));
  }
}

// out = DST(a) over a strided index space, one element per thread (the reference's
// shaders/cast.slang); dense layouts take cast_kernel instead.
template <uint32_t SRC, uint32_t DST>
__global__ __launch_bounds__(256) void cast_strided(MovePlan p) {
  const uint64_t stride = uint64_t(gridDim.x) * 256;
  for (uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x; i < p.n; i += stride) {
    int64_t o, a;
    plan_offsets(p, uint32_t(i), &o, &a);
    store1_any<DST>(p.out, uint64_t(o), load1_any<SRC>(p.a, uint64_t(a)));
  }
}

// Workgroup-wide maximum of per-thread values (256 threads).
__device__ __forceinline__ float block_max(float v) {
  __shared__ float part[4];
  v = wave_max(v);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = v;
  __syncthreads();
  const float r = fmaxf(fmaxf(part[0], part[1]), fmaxf(part[2], part[3]));
  __syncthreads();  // (part is reused by the next call)
  return r;
}

__device__ __forceinline__ float clamp_keep_nan(float y, float fmax) {
  y = y < -fmax ? -fmax : y;
  return fmax < y ? fmax : y;
}

constexpr int kQuantGroups = 4;  // groups of 16 values a thread keeps in registers in the one-pass form

// One workgroup per row.  ONE_PASS: k is a multiple of 16, at most 4096 * kQuantGroups, rows
// aligned to 16 elements: the row is read once, into registers.  ROWWISE = 0: p.scale holds
// one given scale (an input); 1: the row's scale is computed and written to p.scale[m].
template <uint32_t SRC, uint32_t FMT, bool ONE_PASS>
__global__ __launch_bounds__(256) void fp8_quant_kernel(F8QuantParams p, uint32_t rowwise) {
  const uint32_t m = blockIdx.x, tid = threadIdx.x;
  const float fmax = FMT == VKT_E4M3 ? 448.0f : 57344.0f;
  const uint64_t row = p.src + uint64_t(m) * p.lds * item_size(SRC), out = p.dst + uint64_t(m) * p.ldd;
  float x[kQuantGroups][16];
  const uint32_t groups = p.k / 16;
  float a;
  if (rowwise) {
    float amax = 0.0f;
    if constexpr (ONE_PASS) {
#pragma unroll
      for (int i = 0; i < kQuantGroups; ++i)
        if (tid + 256 * i < groups) load16_any<SRC>(row + uint64_t(tid + 256 * i) * 16 * item_size(SRC), x[i]);
#pragma unroll
      for (int i = 0; i < kQuantGroups; ++i)
        if (tid + 256 * i < groups) {
#pragma unroll
          for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(x[i][e]));  // (fmaxf drops NaN)
        }
    } else {
      for (uint32_t k = tid; k < p.k; k += 256) amax = fmaxf(amax, fabsf(load1_any<SRC>(row, k)));
    }
    a = fmaxf(block_max(amax), 1e-12f);
    if (tid == 0) stg<float>(p.scale + 4ull * m, a / fmax);
  } else {
    a = ldg<float>(p.scale) * fmax;  // the given scale is a / fmax
    if constexpr (ONE_PASS) {
#pragma unroll
      for (int i = 0; i < kQuantGroups; ++i)
        if (tid + 256 * i < groups) load16_any<SRC>(row + uint64_t(tid + 256 * i) * 16 * item_size(SRC), x[i]);
    }
  }
  const float inv = fmax / a;
  if constexpr (ONE_PASS) {
#pragma unroll
    for (int i = 0; i < kQuantGroups; ++i)
      if (tid + 256 * i < groups) {
        float y[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) y[e] = clamp_keep_nan(x[i][e] * inv, fmax);
        store16_any<FMT>(out + uint64_t(tid + 256 * i) * 16, y);
      }
  } else {
    for (uint32_t k = tid; k < p.k; k += 256)
      store1_any<FMT>(out, k, clamp_keep_nan(load1_any<SRC>(row, k) * inv, fmax));
  }
}

template <uint32_t SRC>
int launch_cast_from(const CastParams& p, uint32_t vector, uint32_t groups, hipStream_t stream, std::string* err) {
  switch (p.dst_dtype) {
    case VKT_F32: hipLaunchKernelGGL((cast_kernel<SRC, VKT_F32>), dim3(groups), dim3(256), 0, stream, p, vector); return 0;
    case VKT_F16: hipLaunchKernelGGL((cast_kernel<SRC, VKT_F16>), dim3(groups), dim3(256), 0, stream, p, vector); return 0;
    case VKT_BF16: hipLaunchKernelGGL((cast_kernel<SRC, VKT_BF16>), dim3(groups), dim3(256), 0, stream, p, vector); return 0;
    case VKT_E4M3: hipLaunchKernelGGL((cast_kernel<SRC, VKT_E4M3>), dim3(groups), dim3(256), 0, stream, p, vector); return 0;
    case VKT_E5M2: hipLaunchKernelGGL((cast_kernel<SRC, VKT_E5M2>), dim3(groups), dim3(256), 0, stream, p, vector); return 0;
  }
  *err = "cast_fp8: unsupported destination dtype";
  return -1;
}

template <uint32_t SRC, uint32_t FMT>
void launch_quant(const F8QuantParams& p, uint32_t rowwise, hipStream_t stream) {
  const bool one_pass = p.k % 16 == 0 && p.k <= 4096u * kQuantGroups && (p.src % (16 * item_size(SRC))) == 0 &&
                        (uint64_t(p.lds) * item_size(SRC)) % (16 * item_size(SRC)) == 0 && p.dst % 16 == 0 && p.ldd % 16 == 0;
  if (one_pass) hipLaunchKernelGGL((fp8_quant_kernel<SRC, FMT, true>), dim3(p.m), dim3(256), 0, stream, p, rowwise);
  else hipLaunchKernelGGL((fp8_quant_kernel<SRC, FMT, false>), dim3(p.m), dim3(256), 0, stream, p, rowwise);
}

}  // namespace

int launch_cast_fp8(const CastParams& p, const Machine& mc, hipStream_t stream, std::string* err) {
  if (p.n == 0) return 0;
  if (p.src_dtype > VKT_E5M2 || p.dst_dtype > VKT_E5M2) {
    *err = "cast_fp8: the types are float32, float16, bfloat16, e4m3fn and e5m2";
    return -1;
  }
  if (!p.src || !p.dst) {
    *err = "cast_fp8: null tensor address";
    return -1;
  }
  const uint32_t vector = (p.src % (16 * item_size(p.src_dtype)) == 0 && p.dst % (16 * item_size(p.dst_dtype)) == 0) ? 1 : 0;
  const uint64_t units = vector ? (p.n + 15) / 16 : p.n, cap = uint64_t(mc.compute_units) * 32;
  const uint64_t want = (units + 255) / 256;
  const uint32_t groups = uint32_t(want < 1 ? 1 : (want < cap ? want : cap));
  int rc;
  switch (p.src_dtype) {
    case VKT_F32: rc = launch_cast_from<VKT_F32>(p, vector, groups, stream, err); break;
    case VKT_F16: rc = launch_cast_from<VKT_F16>(p, vector, groups, stream, err); break;
    case VKT_BF16: rc = launch_cast_from<VKT_BF16>(p, vector, groups, stream, err); break;
    case VKT_E4M3: rc = launch_cast_from<VKT_E4M3>(p, vector, groups, stream, err); break;
    default: rc = launch_cast_from<VKT_E5M2>(p, vector, groups, stream, err); break;
  }
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "cast_fp8: kernel launch failed";
    return -1;
  }
  return rc;
}

int launch_cast_strided(const StridedParams& s, int src_dtype, int dst_dtype, const Machine& mc, hipStream_t stream,
                        std::string* err) {
  if (s.n == 0) return 0;
  const uint32_t si = item_size(uint32_t(src_dtype)), di = item_size(uint32_t(dst_dtype));
  if (!s.out || !s.a || s.out % di != 0 || s.a % si != 0) {
    *err = "cast: null or misaligned tensor address";
    return -1;
  }
  MovePlan p;
  if (!plan_from(s.out, s.a, s.n, s.ndim, 4, s.size, s.so, s.sa, di, "cast", &p, err)) return -1;
  if (p.ndim == 0 || (p.ndim == 1 && p.so[0] == 1 && p.sa[0] == 1)) {  // dense: 16 elements per thread
    CastParams c{};
    c.src = s.a, c.dst = s.out, c.n = s.n, c.src_dtype = uint32_t(src_dtype), c.dst_dtype = uint32_t(dst_dtype);
    return launch_cast_fp8(c, mc, stream, err);
  }
  const uint64_t want = (p.n + 255) / 256, cap = uint64_t(mc.compute_units) * 64;
  const dim3 grid(uint32_t(want < cap ? want : cap));
#define VKT_CAST_CASE(S, D) \
  if (src_dtype == S && dst_dtype == D) hipLaunchKernelGGL((cast_strided<S, D>), grid, dim3(256), 0, stream, p);
  VKT_CAST_CASE(VKT_F32, VKT_F16) VKT_CAST_CASE(VKT_F32, VKT_BF16) VKT_CAST_CASE(VKT_F16, VKT_F32)
  VKT_CAST_CASE(VKT_F16, VKT_BF16) VKT_CAST_CASE(VKT_BF16, VKT_F32) VKT_CAST_CASE(VKT_BF16, VKT_F16)
#undef VKT_CAST_CASE
  if (hipGetLastError() != hipSuccess) {
    *err = "cast: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_fp8_quant(const F8QuantParams& p, uint32_t rowwise, const Machine&, hipStream_t stream, std::string* err) {
  if (p.m == 0 || p.k == 0) return 0;
  if (p.src_dtype > VKT_BF16 || !is_fp8_host(p.dst_fmt)) {
    *err = "fp8_quant: float32 / float16 / bfloat16 in, e4m3fn / e5m2 out";
    return -1;
  }
  if (rowwise > 1) {
    *err = "fp8_quant: ROWWISE must be 0 or 1";
    return -1;
  }
  if (!p.src || !p.dst || !p.scale || (p.scale & 3)) {
    *err = "fp8_quant: null or unaligned tensor address";
    return -1;
  }
  if (p.lds < p.k || p.ldd < p.k) {
    *err = "fp8_quant: row strides shorter than the rows";
    return -1;
  }
#define VKT_QUANT_CASE(S, F) \
  if (p.src_dtype == S && p.dst_fmt == F) launch_quant<S, F>(p, rowwise, stream);
  VKT_QUANT_CASE(VKT_F32, VKT_E4M3) VKT_QUANT_CASE(VKT_F32, VKT_E5M2)
  VKT_QUANT_CASE(VKT_F16, VKT_E4M3) VKT_QUANT_CASE(VKT_F16, VKT_E5M2)
  VKT_QUANT_CASE(VKT_BF16, VKT_E4M3) VKT_QUANT_CASE(VKT_BF16, VKT_E5M2)
#undef VKT_QUANT_CASE
  if (hipGetLastError() != hipSuccess) {
    *err = "fp8_quant: kernel launch failed";
    return -1;
  }
  return 0;
}

}  // namespace vkt
