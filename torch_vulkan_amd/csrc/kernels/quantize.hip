// Per-tensor affine quantised tensors and fake quantisation on gfx950, one fused HBM-streaming
// kernel per operator where the reference composes each from a dozen elementwise operators over
// full-size temporaries (crates/pyvk/csrc/quantized.cpp:72-130; python/torch_vulkan/_kernels.py:
// 1613-1676).  The arithmetic is the x86 CPU's, step by step (single float32 operations: this
// file is compiled without contraction; the one fused multiply-add is explicit):
//   quantize_affine    q = clamp(int32(nearbyint(min(x * (1.0f / scale), 2147483520))) + zp)  (8-bit;
//                      a NaN takes the upper bound, as FBGEMM's vector code does);
//                      qint32: float(nearbyint(x / scale) + zp) clamped, a NaN -> INT32_MIN
//   dequantize_affine  x = scale * float(q - zp), the difference in wrapping int32
//   fake_quant         q = nearbyint(x * (1.0f / scale)) + zp; mask = qmin <= q <= qmax;
//                      out = (clamp(q) - zp) * scale; per channel q passes through int64 first
//                      (what int64 cannot hold becomes its minimum) and a float zero point enters
//                      as fma(x, 1.0f / scale, zp); outputs in the input's type
// Dense tensors (the operator layer makes strided ones contiguous first).
#include "common.h"
#include "kernels.h"

namespace vkt {
namespace {

constexpr int kPer = 4;    // elements per thread and step: 16 bytes of float32 per lane, a wave's access contiguous
constexpr int kBatch = 4;  // steps whose loads a thread issues together

// The raw bits of kPer elements of an element type, loaded whole (aligned) or element by element (`left` of them exist).
template <int BYTES>
struct Raw;
template <>
struct Raw<4> { using type = U4; };
template <>
struct Raw<2> { using type = U2; };
template <>
struct Raw<1> { using type = uint32_t; };

template <int BYTES>
__device__ __forceinline__ typename Raw<BYTES>::type load_raw(uint64_t addr, bool whole, uint64_t left) {
  using R = typename Raw<BYTES>::type;
  if (whole) return ldg<R>(addr);
  if constexpr (BYTES == 4) {
    U4 r = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < kPer; ++e) r[e] = uint64_t(e) < left ? ldg<uint32_t>(addr + 4 * e) : 0u;
    return r;
  } else if constexpr (BYTES == 2) {
    U2 r = {0, 0};
#pragma unroll
    for (int e = 0; e < kPer; ++e) r[e / 2] |= (uint64_t(e) < left ? uint32_t(ldg<uint16_t>(addr + 2 * e)) : 0u) << (16 * (e % 2));
    return r;
  } else {
    uint32_t r = 0;
#pragma unroll
    for (int e = 0; e < kPer; ++e) r |= (uint64_t(e) < left ? uint32_t(ldg<uint8_t>(addr + e)) : 0u) << (8 * e);
    return r;
  }
}

template <int BYTES>
__device__ __forceinline__ void store_raw(uint64_t addr, bool whole, uint64_t left, typename Raw<BYTES>::type r) {
  using R = typename Raw<BYTES>::type;
  if (whole) {
    stg<R>(addr, r);
    return;
  }
#pragma unroll
  for (int e = 0; e < kPer; ++e) {
    if (uint64_t(e) >= left) continue;
    if constexpr (BYTES == 4) stg<uint32_t>(addr + 4 * e, r[e]);
    else if constexpr (BYTES == 2) stg<uint16_t>(addr + 2 * e, uint16_t(r[e / 2] >> (16 * (e % 2))));
    else stg<uint8_t>(addr + e, uint8_t(r >> (8 * e)));
  }
}

// Element e of raw bits as float32 (T: f32_t, f16_t, bf16_t).
template <class T>
__device__ __forceinline__ float element_f32(const typename Raw<(T::dtype == VKT_F32 ? 4 : 2)>::type& r, int e) {
  if constexpr (T::dtype == VKT_F32) return bits_f32(r[e]);
  else {
    const uint32_t h = (r[e / 2] >> (16 * (e % 2))) & 0xffffu;
    return T::dtype == VKT_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
  }
}
template <class T>
__device__ __forceinline__ typename Raw<(T::dtype == VKT_F32 ? 4 : 2)>::type pack_f32(const float (&x)[kPer]) {
  if constexpr (T::dtype == VKT_F32) return U4{f32_bits(x[0]), f32_bits(x[1]), f32_bits(x[2]), f32_bits(x[3])};
  else if constexpr (T::dtype == VKT_BF16)
    return U2{uint32_t(f32_to_bf16(x[0])) | uint32_t(f32_to_bf16(x[1])) << 16, uint32_t(f32_to_bf16(x[2])) | uint32_t(f32_to_bf16(x[3])) << 16};
  else
    return U2{uint32_t(f32_to_f16(x[0])) | uint32_t(f32_to_f16(x[1])) << 16, uint32_t(f32_to_f16(x[2])) | uint32_t(f32_to_f16(x[3])) << 16};
}

// Groups of kPer elements over the grid: kBatch of them at a time while all are whole (their loads are issued
// together, then each is finished), the rest one by one.  load(i, whole, left) -> raw; finish(i, whole, left, raw).
template <class LOAD, class FINISH>
__device__ __forceinline__ void stream_groups(uint64_t n, uint32_t vec, LOAD load, FINISH finish) {
  const uint64_t stride = uint64_t(gridDim.x) * 256, groups = (n + kPer - 1) / kPer, full = vec ? n / kPer : 0;
  uint64_t g = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  for (; g + (kBatch - 1) * stride < full; g += kBatch * stride) {
    decltype(load(0, true, 0)) raw[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) raw[b] = load((g + b * stride) * kPer, true, kPer);
#pragma unroll
    for (int b = 0; b < kBatch; ++b) finish((g + b * stride) * kPer, true, kPer, raw[b]);
  }
  for (; g < groups; g += stride) {
    const uint64_t i = g * kPer, left = n - i;
    const bool whole = g < full;
    finish(i, whole, left, load(i, whole, left));
  }
}

__device__ __forceinline__ int32_t quantize8(float x, float inv, int32_t zp, int32_t lo, int32_t hi) {
  const float top = 2147483520.0f, t = x * inv;
  const float tc = t != t ? top : (t < top ? t : top);
  float r = __builtin_rintf(tc);
  r = r < -2147483648.0f ? -2147483648.0f : r;
  const int32_t q = int32_t(uint32_t(int32_t(r)) + uint32_t(zp));  // (the CPU's int32 add wraps)
  return q < lo ? lo : (q > hi ? hi : q);
}

__device__ __forceinline__ int32_t quantize32(float x, float inv, int32_t zp) {
  const float r = __builtin_rintf(x * inv) + float(zp);
  if (r != r) return INT32_MIN;
  if (r >= 2147483648.0f) return INT32_MAX;
  if (r <= -2147483648.0f) return INT32_MIN;
  return int32_t(r);
}

// QTYPE 0: quint8, 1: qint8, 2: qint32.  `vec`: both addresses allow whole accesses.
template <int QTYPE>
__global__ __launch_bounds__(256) void quantize_kernel(QuantParams p, float inv, uint32_t vec) {
  constexpr int QB = QTYPE == 2 ? 4 : 1;
  stream_groups(
      p.n, vec, [&](uint64_t i, bool whole, uint64_t left) { return load_raw<4>(p.src + 4 * i, whole, left); },
      [&](uint64_t i, bool whole, uint64_t left, const U4& raw) {
        typename Raw<QB>::type out{};
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
          const float x = bits_f32(raw[e]);
          if constexpr (QTYPE == 2) out[e] = uint32_t(quantize32(x, inv, p.zero_point));
          else out |= (uint32_t(quantize8(x, inv, p.zero_point, QTYPE == 0 ? 0 : -128, QTYPE == 0 ? 255 : 127)) & 0xffu) << (8 * e);
        }
        store_raw<QB>(p.dst + QB * i, whole, left, out);
      });
}

template <int QTYPE>
__global__ __launch_bounds__(256) void dequantize_kernel(QuantParams p, float scale, uint32_t vec) {
  constexpr int QB = QTYPE == 2 ? 4 : 1;
  stream_groups(
      p.n, vec, [&](uint64_t i, bool whole, uint64_t left) { return load_raw<QB>(p.src + QB * i, whole, left); },
      [&](uint64_t i, bool whole, uint64_t left, const typename Raw<QB>::type& raw) {
        float x[kPer];
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
          int32_t q;
          if constexpr (QTYPE == 2) q = int32_t(raw[e]);
          else q = QTYPE == 0 ? int32_t((raw >> (8 * e)) & 0xffu) : int32_t(int8_t((raw >> (8 * e)) & 0xffu));
          x[e] = float(int32_t(uint32_t(q) - uint32_t(p.zero_point))) * scale;
        }
        store_raw<4>(p.dst + 4 * i, whole, left, pack_f32<f32_t>(x));
      });
}

// MODE 0: per tensor; 1: per channel, int32 zero points; 2: per channel, float32 zero points.
template <class T, int MODE>
__global__ __launch_bounds__(256) void fake_quant_kernel(QuantParams p, float scale, float inv, uint32_t vec) {
  constexpr int ITEM = T::dtype == VKT_F32 ? 4 : 2;
  const float lo = float(p.qmin), hi = float(p.qmax), zp_tensor = float(p.zero_point);
  stream_groups(
      p.n, vec, [&](uint64_t i, bool whole, uint64_t left) { return load_raw<ITEM>(p.src + ITEM * i, whole, left); },
      [&](uint64_t i, bool whole, uint64_t left, const typename Raw<ITEM>::type& raw) {
        float y[kPer];
        uint32_t m_word = 0;
#pragma unroll
        for (int e = 0; e < kPer; ++e) {
          const float x = element_f32<T>(raw, e);
          bool inside;
          if constexpr (MODE == 0) {
            const float q = __builtin_rintf(x * inv) + zp_tensor;
            inside = q >= lo && q <= hi;
            const float qc = q != q ? lo : (q < lo ? lo : (q > hi ? hi : q));
            y[e] = (qc - zp_tensor) * scale;
          } else {
            const uint32_t c = uint32_t((uint32_t(i) + e) / p.inner) % p.channels;  // (n < 2^32, checked by the launcher)
            const float sc = ldg<float>(p.scales + 4 * uint64_t(c)), ci = 1.0f / sc;
            float zp, q;
            if constexpr (MODE == 1) {
              zp = float(ldg<int32_t>(p.zero_points + 4 * uint64_t(c)));
              q = __builtin_rintf(x * ci) + zp;
            } else {
              zp = ldg<float>(p.zero_points + 4 * uint64_t(c));
              q = __builtin_rintf(__builtin_fmaf(x, ci, zp));
            }
            const bool fits = q > -9223372036854775808.0f && q < 9223372036854775808.0f;
            const long long qi = fits ? (long long)q : INT64_MIN;
            inside = qi >= p.qmin && qi <= p.qmax;
            const long long qc = qi < p.qmin ? p.qmin : (qi > p.qmax ? p.qmax : qi);
            y[e] = float((double(qc) - double(zp)) * double(sc));
          }
          m_word |= uint32_t(inside) << (8 * e);
        }
        store_raw<ITEM>(p.dst + ITEM * i, whole, left, pack_f32<T>(y));
        store_raw<1>(p.mask + i, whole, left, m_word);
      });
}

// Row-wise minimum and maximum (the observer in front of fake quantisation): block (part, row) reduces
// columns [part * chunk, (part + 1) * chunk) of its row; a NaN anywhere in the range makes both results NaN,
// as torch.aminmax.  Results as float32 at out[row * parts + part].
template <class T>
__global__ __launch_bounds__(256) void aminmax_kernel(MinMaxParams p, uint64_t out_min, uint64_t out_max, uint32_t parts, uint32_t chunk,
                                                      uint32_t vec) {
  constexpr uint32_t ITEM = T::dtype == VKT_F32 ? 4 : 2;
  const uint32_t part = blockIdx.x, row = blockIdx.y, tid = threadIdx.x;
  const uint64_t base = p.src + uint64_t(row) * p.ld * ITEM;
  const uint32_t lo = part * chunk, hi = lo + chunk < p.cols ? lo + chunk : p.cols;
  float mn = __builtin_inff(), mx = -__builtin_inff(), bad = 0.0f;
  auto take = [&](float v) {
    mn = fminf(mn, v), mx = fmaxf(mx, v);  // (both drop a NaN: it is counted apart)
    bad = v != v ? 1.0f : bad;
  };
  if (vec) {  // rows and chunks start on 16 bytes
    for (uint32_t c = lo + tid * kPer; c + kPer <= hi; c += 256 * kPer) {
      const auto raw = ldg<typename Raw<ITEM>::type>(base + uint64_t(c) * ITEM);
#pragma unroll
      for (int e = 0; e < kPer; ++e) take(element_f32<T>(raw, e));
    }
    const uint32_t tail = lo + (hi - lo) / kPer * kPer;
    if (tail + tid < hi) take(load_f32<T>(base + uint64_t(tail + tid) * ITEM));
  } else {
    for (uint32_t c = lo + tid; c < hi; c += 256) take(load_f32<T>(base + uint64_t(c) * ITEM));
  }
  mn = wave_min(mn), mx = wave_max(mx), bad = wave_max(bad);
  __shared__ float part_min[4], part_max[4], part_bad[4];
  if ((tid & 63) == 0) part_min[tid >> 6] = mn, part_max[tid >> 6] = mx, part_bad[tid >> 6] = bad;
  __syncthreads();
  if (tid == 0) {
    mn = fminf(fminf(part_min[0], part_min[1]), fminf(part_min[2], part_min[3]));
    mx = fmaxf(fmaxf(part_max[0], part_max[1]), fmaxf(part_max[2], part_max[3]));
    bad = fmaxf(fmaxf(part_bad[0], part_bad[1]), fmaxf(part_bad[2], part_bad[3]));
    const float nan = __builtin_nanf("");
    stg<float>(out_min + 4ull * (uint64_t(row) * parts + part), bad != 0.0f ? nan : mn);
    stg<float>(out_max + 4ull * (uint64_t(row) * parts + part), bad != 0.0f ? nan : mx);
  }
}

// Combines the parts of each row (one thread per row; a NaN part makes the row NaN).
__global__ __launch_bounds__(256) void aminmax_finish(uint64_t part_min, uint64_t part_max, uint64_t out_min, uint64_t out_max, uint32_t rows,
                                                      uint32_t parts) {
  const uint32_t row = blockIdx.x * 256 + threadIdx.x;
  if (row >= rows) return;
  float mn = __builtin_inff(), mx = -__builtin_inff();
  bool bad = false;
  for (uint32_t q = 0; q < parts; ++q) {
    const float a = ldg<float>(part_min + 4ull * (uint64_t(row) * parts + q)), b = ldg<float>(part_max + 4ull * (uint64_t(row) * parts + q));
    bad = bad || a != a;
    mn = fminf(mn, a), mx = fmaxf(mx, b);
  }
  const float nan = __builtin_nanf("");
  stg<float>(out_min + 4ull * row, bad ? nan : mn);
  stg<float>(out_max + 4ull * row, bad ? nan : mx);
}

uint32_t groups_for(uint64_t n, const Machine& mc) {
  const uint64_t want = ((n + kPer - 1) / kPer + 255) / 256, cap = uint64_t(mc.compute_units) * 64;
  return uint32_t(want < 1 ? 1 : (want < cap ? want : cap));
}

int done(const char* who, std::string* err) {
  if (hipGetLastError() != hipSuccess) {
    *err = std::string(who) + ": kernel launch failed";
    return -1;
  }
  return 0;
}

}  // namespace

int launch_aminmax(const MinMaxParams& p, const Machine& mc, hipStream_t stream, std::string* err) {
  if (p.rows == 0) return 0;
  if (p.dtype > VKT_BF16 || p.cols == 0 || p.ld < p.cols || p.rows > 65535) {
    *err = "aminmax: float32 / float16 / bfloat16 rows of at least one column, at most 65535 rows, ld >= cols";
    return -1;
  }
  const uint64_t item = p.dtype == VKT_F32 ? 4 : 2;
  if (!p.src || !p.out_min || !p.out_max || p.src % item != 0 || p.out_min % 4 != 0 || p.out_max % 4 != 0) {
    *err = "aminmax: null or misaligned tensor address";
    return -1;
  }
  // enough blocks to fill the machine: rows split into parts of whole 4 Ki-column chunks
  const uint32_t unit = 256 * kPer * 4;
  uint32_t parts = (uint32_t(mc.compute_units) * 4 + p.rows - 1) / p.rows;
  const uint32_t most = (p.cols + unit - 1) / unit;
  parts = parts < 1 ? 1 : (parts > most ? most : parts);
  const uint32_t chunk = ((p.cols + parts - 1) / parts + unit - 1) / unit * unit;
  parts = (p.cols + chunk - 1) / chunk;
  if (parts > 1 && uint64_t(p.rows) * parts * 8 > mc.workspace_bytes) {
    *err = "aminmax: workspace too small";
    return -1;
  }
  const uint64_t pmin = parts > 1 ? mc.workspace : p.out_min, pmax = parts > 1 ? mc.workspace + uint64_t(p.rows) * parts * 4 : p.out_max;
  const uint32_t vec = p.src % 16 == 0 && (uint64_t(p.ld) * item) % 16 == 0;
  const dim3 grid(parts, p.rows);
  if (p.dtype == VKT_F32) hipLaunchKernelGGL(aminmax_kernel<f32_t>, grid, dim3(256), 0, stream, p, pmin, pmax, parts, chunk, vec);
  else if (p.dtype == VKT_F16) hipLaunchKernelGGL(aminmax_kernel<f16_t>, grid, dim3(256), 0, stream, p, pmin, pmax, parts, chunk, vec);
  else hipLaunchKernelGGL(aminmax_kernel<bf16_t>, grid, dim3(256), 0, stream, p, pmin, pmax, parts, chunk, vec);
  if (parts > 1) hipLaunchKernelGGL(aminmax_finish, dim3((p.rows + 255) / 256), dim3(256), 0, stream, pmin, pmax, p.out_min, p.out_max, p.rows, parts);
  return done("aminmax", err);
}

int launch_quantize_affine(const QuantParams& p, uint32_t qtype, bool dequantize, const Machine& mc, hipStream_t stream,
                           std::string* err) {
  const char* who = dequantize ? "dequantize_affine" : "quantize_affine";
  if (p.n == 0) return 0;
  if (qtype > 2) {
    *err = std::string(who) + ": QTYPE is 0 (quint8), 1 (qint8) or 2 (qint32)";
    return -1;
  }
  const uint64_t qitem = qtype == 2 ? 4 : 1;
  const uint64_t f = dequantize ? p.dst : p.src, q = dequantize ? p.src : p.dst;
  if (!p.src || !p.dst || f % 4 != 0 || q % qitem != 0) {
    *err = std::string(who) + ": null or misaligned tensor address";
    return -1;
  }
  const float scale = bits_f32_host(p.scale_bits);
  const uint32_t vec = f % 16 == 0 && q % (qitem * kPer) == 0;
  const dim3 grid(groups_for(p.n, mc));
  if (dequantize) {
    if (qtype == 0) hipLaunchKernelGGL(dequantize_kernel<0>, grid, dim3(256), 0, stream, p, scale, vec);
    else if (qtype == 1) hipLaunchKernelGGL(dequantize_kernel<1>, grid, dim3(256), 0, stream, p, scale, vec);
    else hipLaunchKernelGGL(dequantize_kernel<2>, grid, dim3(256), 0, stream, p, scale, vec);
  } else {
    const float inv = 1.0f / scale;  // (rounded once, as the CPU's)
    if (qtype == 0) hipLaunchKernelGGL(quantize_kernel<0>, grid, dim3(256), 0, stream, p, inv, vec);
    else if (qtype == 1) hipLaunchKernelGGL(quantize_kernel<1>, grid, dim3(256), 0, stream, p, inv, vec);
    else hipLaunchKernelGGL(quantize_kernel<2>, grid, dim3(256), 0, stream, p, inv, vec);
  }
  return done(who, err);
}

template <class T>
void launch_fake_quant_t(const QuantParams& p, uint32_t mode, float scale, float inv, uint32_t vec, dim3 grid, hipStream_t stream) {
  if (mode == 0) hipLaunchKernelGGL((fake_quant_kernel<T, 0>), grid, dim3(256), 0, stream, p, scale, inv, vec);
  else if (mode == 1) hipLaunchKernelGGL((fake_quant_kernel<T, 1>), grid, dim3(256), 0, stream, p, scale, inv, vec);
  else hipLaunchKernelGGL((fake_quant_kernel<T, 2>), grid, dim3(256), 0, stream, p, scale, inv, vec);
}

int launch_fake_quant(const QuantParams& p, uint32_t per_channel, uint32_t zp_float, const Machine& mc, hipStream_t stream,
                      std::string* err) {
  if (p.n == 0) return 0;
  if (p.dtype > VKT_BF16 || per_channel > 1 || zp_float > 1 || (!per_channel && zp_float)) {
    *err = "fake_quant: float32 / float16 / bfloat16 tensors; spec {PER_CHANNEL, ZP_FLOAT} (a float zero point only per channel)";
    return -1;
  }
  const uint64_t item = p.dtype == VKT_F32 ? 4 : 2;
  if (!p.src || !p.dst || !p.mask || p.src % item != 0 || p.dst % item != 0) {
    *err = "fake_quant: null or misaligned tensor address";
    return -1;
  }
  if (per_channel && (!p.scales || !p.zero_points || p.scales % 4 != 0 || p.zero_points % 4 != 0 || p.channels == 0 || p.inner == 0 ||
                      p.n >= (1ull << 32))) {
    *err = "fake_quant: per channel needs scales, zero points, channels, inner and fewer than 2^32 elements";
    return -1;
  }
  if (p.qmin > p.qmax) {
    *err = "fake_quant: qmin above qmax";
    return -1;
  }
  const float scale = bits_f32_host(p.scale_bits), inv = 1.0f / scale;
  const uint32_t vec = p.src % (item * kPer) == 0 && p.dst % (item * kPer) == 0 && p.mask % kPer == 0;
  const uint32_t mode = per_channel ? 1 + zp_float : 0;
  const dim3 grid(groups_for(p.n, mc));
  if (p.dtype == VKT_F32) launch_fake_quant_t<f32_t>(p, mode, scale, inv, vec, grid, stream);
  else if (p.dtype == VKT_F16) launch_fake_quant_t<f16_t>(p, mode, scale, inv, vec, grid, stream);
  else launch_fake_quant_t<bf16_t>(p, mode, scale, inv, vec, grid, stream);
  return done("fake_quant", err);
}

}  // namespace vkt
