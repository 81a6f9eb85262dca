// Shared declarations of the torch layer of device "vk" (the counterpart of the reference's
// crates/pyvk/csrc/vk.h, cut down to what the quantized-matmul path uses).
#pragma once

#include <ATen/ATen.h>
#include <ATen/core/dispatch/Dispatcher.h>
#include <ATen/core/stack.h>

#include <cstdint>
#include <string>
#include <vector>

#include "../../../include/vkt.h"

namespace vk {

constexpr c10::DeviceType kDevice = c10::DeviceType::PrivateUse1;

// rc of a vkt_* call -> exception "torch_vulkan: <message>" (reference vk.h:75-77).
void check(int rc);

// Waits for queued GPU work.
void synchronize();

c10::Allocator* allocator();

// Device address of the first element of `t` (0 for an empty tensor).  The DataPtr of a vk
// tensor is the device pointer, so this is t.data_ptr() (reference vk.h:117-122 looks it up
// in a host-pointer map).  The _out form materializes copy-on-write storage first.
uint64_t gpu_address(const at::TensorBase& t);
uint64_t gpu_address_out(const at::TensorBase& t);

// Tells the op layer that the memory of vk tensor `t` is about to be written: whatever it has derived from the old
// contents and cannot tell stale by a version counter (inference tensors carry none) is dropped.  Called by
// gpu_address_out and by the copy and fill paths.
void note_write(const at::TensorBase& t);

// Records that `op` ran on the CPU instead of the GPU; under TORCH_VK_STRICT raises
// NotImplementedError instead (reference vk.h: record_fallback).
void record_fallback(const std::string& op);

// Runs `op` on CPU copies of the stack's vk tensors, recorded as a fallback.
void run_fallback(const c10::OperatorHandle& op, torch::jit::Stack* stack, bool error_on_views);

// dst[...] = the elements at src_base + sum_d index_d * src_strides[d] (element strides per dim of dst, 0 =
// broadcast, negative allowed), converting between float32 / float16 / bfloat16 if src_type differs.  False
// where no device kernel covers the case.
bool copy_strided_on_device(const at::Tensor& dst, uint64_t src_base, const std::vector<int64_t>& src_strides,
                            at::ScalarType src_type);

// A dense copy of quantised vk tensor q in memory format mf, with q's quantizer.
at::Tensor vk_clone_quantized(const at::Tensor& q, at::MemoryFormat mf);

inline bool is_vk(const at::Tensor& t) { return t.device().type() == kDevice; }

// The library's code of an element type (-1: not one of its types).
inline int vkt_dtype(at::ScalarType t) {
  switch (t) {
    case at::kFloat: return VKT_F32;
    case at::kHalf: return VKT_F16;
    case at::kBFloat16: return VKT_BF16;
    case at::kFloat8_e4m3fn: return VKT_E4M3;
    case at::kFloat8_e5m2: return VKT_E5M2;
    default: return -1;
  }
}

// Runs aten op `name.overload` without a vk kernel (reference vk.h:372-379).
template <typename... Args>
torch::jit::Stack on_cpu(const char* name, const char* overload, const Args&... args) {
  auto op = c10::Dispatcher::singleton().findSchemaOrThrow(name, overload);
  torch::jit::Stack stack;
  (stack.emplace_back(args), ...);
  run_fallback(op, &stack, /*error_on_views=*/false);
  return stack;
}

// Queues `kernel` with its parameter block (at most 128 bytes) (reference vk.h:383-389).
template <typename P>
void dispatch(const std::string& kernel, const std::vector<uint32_t>& spec, const P& params, uint32_t gx,
              uint32_t gy = 1, uint32_t gz = 1) {
  static_assert(sizeof(P) <= 128, "parameter blocks are limited to 128 bytes");
  check(vkt_dispatch(kernel.c_str(), spec.data(), spec.size(), reinterpret_cast<const uint8_t*>(&params), sizeof(P), gx,
                     gy, gz));
}

}  // namespace vk
