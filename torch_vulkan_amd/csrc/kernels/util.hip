// Byte fill and device-to-device copy as ordinary kernels on the runtime's stream (the
// reference's stream has fill and copy commands of its own: crates/vkcore/src/stream.rs,
// exercised by crates/vkcore/tests/runtime.rs:93-116).  Kernels rather than
// hipMemsetAsync / hipMemcpyAsync so that they are ordered, traceable and graph-capturable
// like every other dispatch.
#include "common.h"
#include "kernels.h"

namespace vkt {
namespace {

__global__ __launch_bounds__(256) void fill_kernel(uint64_t dst, uint32_t value, uint64_t nbytes) {
  const uint64_t stride = uint64_t(gridDim.x) * 256;
  const uint64_t head = (16 - (dst & 15)) & 15;  // bytes before the first 16-byte boundary
  const uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (i < head && i < nbytes) stg<uint8_t>(dst + i, uint8_t(value));
  if (nbytes <= head) return;
  const uint64_t body = (nbytes - head) / 16;
  const uint32_t word = value * 0x01010101u;
  const U4 v = {word, word, word, word};
  for (uint64_t j = i; j < body; j += stride) stg<U4>(dst + head + j * 16, v);
  const uint64_t tail0 = head + body * 16;
  if (i < 16 && tail0 + i < nbytes) stg<uint8_t>(dst + tail0 + i, uint8_t(value));
}

// 16-byte copies when source and destination are both 16-byte aligned, else bytes.
__global__ __launch_bounds__(256) void copy_kernel(uint64_t dst, uint64_t src, uint64_t nbytes, uint32_t aligned) {
  const uint64_t stride = uint64_t(gridDim.x) * 256, i = uint64_t(blockIdx.x) * 256 + threadIdx.x;
  if (aligned) {
    const uint64_t body = nbytes / 16;
    for (uint64_t j = i; j < body; j += stride) stg<U4>(dst + j * 16, ldg<U4>(src + j * 16));
    if (i < (nbytes & 15)) stg<uint8_t>(dst + body * 16 + i, ldg<uint8_t>(src + body * 16 + i));
  } else {
    for (uint64_t j = i; j < nbytes; j += stride) stg<uint8_t>(dst + j, ldg<uint8_t>(src + j));
  }
}

__device__ __forceinline__ float any_f32(uint64_t base, uint64_t i, uint32_t dtype) {
  if (dtype == VKT_F32) return ldg<float>(base + 4 * i);
  if (dtype == VKT_F16) return f16_to_f32(ldg<uint16_t>(base + 2 * i));
  return bf16_to_f32(ldg<uint16_t>(base + 2 * i));
}

// The packed float32 vector of the int4 op: bytes, scales and bias widened (all exact).
__global__ __launch_bounds__(256) void packvec_kernel(Q4VecParams p) {
  const uint64_t total = uint64_t(p.nw) + p.ns + p.nb, stride = uint64_t(gridDim.x) * 256;
  for (uint64_t i = uint64_t(blockIdx.x) * 256 + threadIdx.x; i < total; i += stride) {
    float v;
    if (i < p.nw) v = float(ldg<uint8_t>(p.weights + i));
    else if (i < uint64_t(p.nw) + p.ns) v = any_f32(p.scales, i - p.nw, p.scales_dtype);
    else v = any_f32(p.bias, i - p.nw - p.ns, p.bias_dtype);
    stg<float>(p.out + 4 * i, v);
  }
}

uint32_t groups_for(uint64_t units) {
  const uint64_t want = (units + 255) / 256 + 1;
  return uint32_t(want < 16384 ? want : 16384);
}

}  // namespace

int launch_fill(uint64_t dst, uint8_t value, uint64_t nbytes, hipStream_t stream, std::string* err) {
  hipLaunchKernelGGL(fill_kernel, dim3(groups_for(nbytes / 16)), dim3(256), 0, stream, dst, uint32_t(value), nbytes);
  if (hipGetLastError() != hipSuccess) {
    *err = "fill: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_qmm4_packvec(const Q4VecParams& p, hipStream_t stream, std::string* err) {
  const uint64_t total = uint64_t(p.nw) + p.ns + p.nb;
  if (total == 0) return 0;
  if (!p.out || (p.nw && !p.weights) || (p.ns && !p.scales) || (p.nb && !p.bias) || p.scales_dtype > VKT_BF16 ||
      p.bias_dtype > VKT_BF16) {
    *err = "qmm4_packvec: null address or unsupported dtype";
    return -1;
  }
  hipLaunchKernelGGL(packvec_kernel, dim3(groups_for(total)), dim3(256), 0, stream, p);
  if (hipGetLastError() != hipSuccess) {
    *err = "qmm4_packvec: kernel launch failed";
    return -1;
  }
  return 0;
}

int launch_copy(uint64_t dst, uint64_t src, uint64_t nbytes, hipStream_t stream, std::string* err) {
  if ((dst < src + nbytes) && (src < dst + nbytes)) {
    *err = "copy: source and destination overlap";
    return -1;
  }
  const uint32_t aligned = ((dst | src) & 15) == 0;
  hipLaunchKernelGGL(copy_kernel, dim3(groups_for(aligned ? nbytes / 16 : nbytes)), dim3(256), 0, stream, dst, src,
                     nbytes, aligned);
  if (hipGetLastError() != hipSuccess) {
    *err = "copy: kernel launch failed";
    return -1;
  }
  return 0;
}

}  // namespace vkt
