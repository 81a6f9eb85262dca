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
