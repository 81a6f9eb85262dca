// The PyTorch side of the device "vk": the minimal subset of the reference's backend
// (crates/pyvk/csrc/backend.cpp) that the quantized-matmul path needs, over the C ABI in
// include/vkt.h.  Plain C++ against libtorch's CPU library: no HIP headers here, exactly
// as the reference keeps only its C++ layer tied to PyTorch's ABI.
//
//   allocator            reference backend.cpp:118-160 (VkAllocator): vkt_alloc / vkt_free;
//                        the DataPtr holds the device pointer itself, so gpu_address(t) is
//                        t.data_ptr() and the reference's address map (:170-192) is gone
//   device guard, hooks  :286-369 (one device, one stream)
//   empty / resize / views / set_   :391-465
//   _copy_from, _local_scalar_dense :765-805; host <-> device through vkt_copy_*; strided,
//                        broadcasting and float32 / float16 / bfloat16-converting copies and
//                        fills run on the device ("move_b<S>", "copy8_b<S>", "cast_<s>_<d>":
//                        :633-717, :806-826); other conversions are staged through the CPU
//   boxed CPU fallback   :1696-1740, counted per op (fallback_counts), an error under
//                        TORCH_VK_STRICT
// The aten kernels of the path live in quant.cpp.
#include "vk.h"

#include <ATen/EmptyTensor.h>
#include <ATen/native/CPUFallback.h>
#include <ATen/native/Resize.h>
#include <ATen/ops/_reshape_alias_native.h>
#include <ATen/ops/as_strided_native.h>
#include <ATen/ops/set_native.h>
#include <ATen/ops/view_native.h>
#include <c10/core/impl/DeviceGuardImplInterface.h>
#include <torch/library.h>

#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>

namespace vk {

void check(int rc) { TORCH_CHECK(rc == 0, "torch_vulkan: ", vkt_last_error()); }

void synchronize() { check(vkt_synchronize()); }

// ------------------------------------------------------------------ allocator

namespace {

void delete_allocation(void* handle) { vkt_free(handle); }

struct VkAllocator final : c10::Allocator {
  c10::DataPtr allocate(size_t nbytes) override {
    const c10::Device device(kDevice, 0);
    if (nbytes == 0) return {nullptr, nullptr, &delete_allocation, device};
    VktAlloc a{};
    check(vkt_alloc(nbytes, &a));
    return {reinterpret_cast<void*>(a.address), a.handle, &delete_allocation, device};
  }
  c10::DeleterFnPtr raw_deleter() const override { return nullptr; }  // (the context is the handle, not the data)
  void copy_data(void* dest, const void* src, std::size_t count) const override {
    check(vkt_copy_on_device(reinterpret_cast<uint64_t>(dest), reinterpret_cast<uint64_t>(src), count));
  }
};

VkAllocator g_allocator;

// One device, one in-order stream (reference backend.cpp:286-308).
struct VkGuardImpl final : c10::impl::DeviceGuardImplInterface {
  c10::DeviceType type() const override { return kDevice; }
  c10::Device exchangeDevice(c10::Device) const override { return c10::Device(kDevice, 0); }
  c10::Device getDevice() const override { return c10::Device(kDevice, 0); }
  void setDevice(c10::Device d) const override { TORCH_CHECK(d.index() <= 0, "vk has one device"); }
  void uncheckedSetDevice(c10::Device) const noexcept override {}
  c10::Stream getStream(c10::Device d) const override { return c10::Stream(c10::Stream::DEFAULT, d); }
  c10::Stream exchangeStream(c10::Stream s) const override { return s; }
  c10::DeviceIndex deviceCount() const noexcept override { return 1; }
  bool queryStream(const c10::Stream&) const override { return true; }
  void synchronizeStream(const c10::Stream&) const override { synchronize(); }
  void synchronizeDevice(const c10::DeviceIndex) const override { synchronize(); }
  void recordDataPtrOnStream(const c10::DataPtr&, const c10::Stream&) const override {}
};

// ------------------------------------------------------------------ fallback accounting

std::mutex g_fallback_mutex;
std::map<std::string, uint64_t> g_fallbacks;

bool strict() {
  static const bool on = [] {
    const char* v = std::getenv("TORCH_VK_STRICT");
    return v && *v && std::string(v) != "0";
  }();
  return on;
}

}  // namespace

c10::Allocator* allocator() { return &g_allocator; }

void record_fallback(const std::string& op) {
  TORCH_CHECK_NOT_IMPLEMENTED(!strict(), op, " has no vk kernel (TORCH_VK_STRICT)");
  std::lock_guard<std::mutex> lock(g_fallback_mutex);
  ++g_fallbacks[op];
}

uint64_t gpu_address(const at::TensorBase& t) {
  return t.numel() == 0 ? 0 : reinterpret_cast<uint64_t>(t.const_data_ptr());
}

uint64_t gpu_address_out(const at::TensorBase& t) {
  if (t.numel() == 0) return 0;
  note_write(t);
  return reinterpret_cast<uint64_t>(t.mutable_data_ptr());  // (materializes copy-on-write storage)
}

namespace {

// ------------------------------------------------------------------ creation, views, resize

at::Tensor empty_memory_format(c10::SymIntArrayRef size, std::optional<at::ScalarType> dtype,
                               std::optional<at::Layout> layout, std::optional<at::Device> device,
                               std::optional<bool> pin_memory, std::optional<at::MemoryFormat> memory_format) {
  TORCH_CHECK(!pin_memory.value_or(false), "vk tensors cannot be pinned");
  TORCH_CHECK(layout.value_or(at::kStrided) == at::kStrided, "vk tensors are strided");
  const auto ks = c10::DispatchKeySet(c10::DispatchKey::PrivateUse1);
  return at::detail::empty_generic(C10_AS_INTARRAYREF_SLOW(size), &g_allocator, ks,
                                   dtype.value_or(at::get_default_dtype_as_scalartype()), memory_format);
}

at::Tensor empty_strided(c10::SymIntArrayRef size, c10::SymIntArrayRef stride, std::optional<at::ScalarType> dtype,
                         std::optional<at::Layout> layout, std::optional<at::Device> device,
                         std::optional<bool> pin_memory) {
  TORCH_CHECK(!pin_memory.value_or(false), "vk tensors cannot be pinned");
  const auto ks = c10::DispatchKeySet(c10::DispatchKey::PrivateUse1);
  return at::detail::empty_strided_generic(C10_AS_INTARRAYREF_SLOW(size), C10_AS_INTARRAYREF_SLOW(stride),
                                           &g_allocator, ks, dtype.value_or(at::get_default_dtype_as_scalartype()));
}

// Storage growth keeps the old bytes (reference backend.cpp:412-440).
void grow_storage(c10::StorageImpl* storage, size_t nbytes) {
  if (nbytes <= storage->nbytes()) return;
  TORCH_CHECK(storage->resizable(), "Trying to resize storage that is not resizable");
  c10::DataPtr fresh = g_allocator.allocate(nbytes);
  const size_t keep = storage->nbytes();
  if (keep != 0 && storage->data() != nullptr) {
    check(vkt_copy_on_device(reinterpret_cast<uint64_t>(fresh.get()), reinterpret_cast<uint64_t>(storage->data()), keep));
  }
  storage->set_data_ptr_noswap(std::move(fresh));
  storage->set_nbytes(nbytes);
}

const at::Tensor& resize_(const at::Tensor& self, c10::SymIntArrayRef size,
                          std::optional<at::MemoryFormat> memory_format) {
  auto sizes = C10_AS_INTARRAYREF_SLOW(size);
  auto* impl = self.unsafeGetTensorImpl();
  impl->set_sizes_contiguous(sizes);
  const size_t need = (impl->storage_offset() + impl->numel()) * self.dtype().itemsize();
  grow_storage(self.storage().unsafeGetStorageImpl(), need);
  if (memory_format && *memory_format != at::MemoryFormat::Preserve) impl->empty_tensor_restride(*memory_format);
  return self;
}

at::Tensor& set_source_storage(at::Tensor& self, at::Storage source) {
  return at::native::set_(self, std::move(source));
}
at::Tensor& set_source_storage_offset(at::Tensor& self, at::Storage source, c10::SymInt offset,
                                      c10::SymIntArrayRef size, c10::SymIntArrayRef stride) {
  return at::native::set_storage_meta__symint(self, std::move(source), std::move(offset), size, stride);
}
at::Tensor& set_source_tensor(at::Tensor& self, const at::Tensor& source) { return at::native::set_tensor_(self, source); }

// ------------------------------------------------------------------ copies

// The bytes [lo, hi) of a vk tensor's storage that its elements span (as element offsets
// from data_ptr; hi exclusive).  Empty tensors span nothing.
std::pair<int64_t, int64_t> element_span(const at::Tensor& t) {
  int64_t lo = 0, hi = 0;
  if (t.numel() == 0) return {0, 0};
  for (int64_t d = 0; d < t.dim(); ++d) {
    const int64_t reach = (t.size(d) - 1) * t.stride(d);
    if (reach >= 0) hi += reach;
    else lo += reach;
  }
  return {lo, hi + 1};
}

// A CPU tensor with t's sizes and strides over a host copy of the bytes t spans.
at::Tensor host_mirror(const at::Tensor& t, bool download) {
  const auto [lo, hi] = element_span(t);
  const int64_t item = t.element_size();
  at::Tensor bytes = at::empty({(hi - lo) * item}, at::TensorOptions().dtype(at::kByte));
  if (download && hi > lo) {
    check(vkt_copy_to_host(bytes.data_ptr(), reinterpret_cast<uint64_t>(t.const_data_ptr()) + uint64_t(lo * item),
                           uint64_t((hi - lo) * item)));
  }
  at::Tensor flat = at::empty({0}, at::TensorOptions().dtype(t.scalar_type()));
  flat.set_(bytes.storage(), -lo, t.sizes(), t.strides());
  return flat;
}

bool plain(const at::Tensor& t) { return t.is_non_overlapping_and_dense(); }

// ---- strided moves on the device (reference launch.cpp:55-83 launch<K>, :108-150 copy_many_dims;
// strided.h:35-121 merge_dims / for_each_dispatch)

struct MergedDims {
  std::vector<int64_t> size, so, sa;  // innermost first
};

// dst's index space with src broadcast to it: dims of size 1 dropped, dims that are contiguous on
// both sides merged.
MergedDims merged_dims(const at::Tensor& dst, const std::vector<int64_t>* src_strides) {
  MergedDims m;
  for (int64_t i = dst.dim() - 1; i >= 0; --i) {
    const int64_t n = dst.size(i);
    if (n == 1) continue;
    const int64_t o = dst.stride(i);
    const int64_t a = src_strides ? (*src_strides)[size_t(i)] : 0;
    if (!m.size.empty() && o == m.so.back() * m.size.back() && a == m.sa.back() * m.size.back()) {
      m.size.back() *= n;
      continue;
    }
    m.size.push_back(n), m.so.push_back(o), m.sa.push_back(a);
  }
  return m;
}

// Runs `emit(count, ndim, out offset, a offset)` over the innermost `inner` dims for every index of the rest.
template <class F>
bool for_each_launch(const MergedDims& m, size_t inner_max, F&& emit) {
  const size_t inner = std::min(m.size.size(), inner_max);
  int64_t count = 1, span_o = 0, span_a = 0;
  for (size_t d = 0; d < inner; ++d) {
    count *= m.size[d];
    span_o += (m.size[d] - 1) * std::abs(m.so[d]), span_a += (m.size[d] - 1) * std::abs(m.sa[d]);
  }
  if (count >= (int64_t(1) << 32) || span_o >= (int64_t(1) << 31) || span_a >= (int64_t(1) << 31)) return false;
  std::vector<int64_t> index(m.size.size() - inner, 0);
  while (true) {
    int64_t oo = 0, ao = 0;
    for (size_t j = 0; j < index.size(); ++j) oo += index[j] * m.so[inner + j], ao += index[j] * m.sa[inner + j];
    emit(count, inner, oo, ao);
    size_t j = 0;
    for (; j < index.size(); ++j) {
      if (++index[j] < m.size[inner + j]) break;
      index[j] = 0;
    }
    if (j == index.size()) return true;
  }
}

const char* size_label(int64_t item) {
  switch (item) {
    case 1: return "b1";
    case 2: return "b2";
    case 4: return "b4";
    case 8: return "b8";
    case 16: return "b16";
    default: return nullptr;
  }
}

const char* float_label(at::ScalarType t) {
  return t == at::kFloat ? "f32" : t == at::kHalf ? "f16" : t == at::kBFloat16 ? "bf16" : nullptr;
}

}  // namespace

// The device side of copies between vk tensors (reference backend.cpp:633-690 copy_vk_to_vk):
// dst[...] = the elements of type src_type at src_base + sum_d index_d * src_strides[d] (element strides, one
// per dim of dst, 0 where the source broadcasts, negative ones allowed).
bool copy_strided_on_device(const at::Tensor& dst, uint64_t src_base, const std::vector<int64_t>& src_strides,
                            at::ScalarType src_type) {
  if (dst.is_conj() || dst.is_neg()) return false;
  note_write(dst);
  const bool same = src_type == dst.scalar_type();
  const char* label = size_label(dst.element_size());
  std::string kernel;
  if (same && label) kernel = std::string("move_") + label;
  else if (!same && float_label(src_type) && float_label(dst.scalar_type()))
    kernel = std::string("cast_") + float_label(src_type) + "_" + float_label(dst.scalar_type());
  else return false;
  if (dst.numel() == 0) return true;
  const MergedDims m = merged_dims(dst, &src_strides);
  const uint64_t out = reinterpret_cast<uint64_t>(dst.mutable_data_ptr()), a = src_base;
  const int64_t oi = dst.element_size(), ai = int64_t(c10::elementSize(src_type));
  if (same && m.size.size() > 4) {  // up to 8 dims in one launch (reference copy_many_dims)
    const std::string k8 = std::string("copy8_") + label;
    return for_each_launch(m, 8, [&](int64_t count, size_t ndim, int64_t oo, int64_t ao) {
      Copy8Params p{};
      p.out = out + uint64_t(oo * oi), p.a = a + uint64_t(ao * ai), p.n = uint32_t(count), p.ndim = uint32_t(ndim);
      for (size_t d = 0; d < 8; ++d) {
        p.size[d] = d < ndim ? uint32_t(m.size[d]) : 1u;
        p.so[d] = d < ndim ? int32_t(m.so[d]) : 0, p.sa[d] = d < ndim ? int32_t(m.sa[d]) : 0;
      }
      dispatch(k8, {}, p, 1);
    });
  }
  return for_each_launch(m, 4, [&](int64_t count, size_t ndim, int64_t oo, int64_t ao) {
    StridedParams p{};
    p.out = out + uint64_t(oo * oi), p.a = a + uint64_t(ao * ai), p.n = uint32_t(count), p.ndim = uint32_t(ndim);
    for (size_t d = 0; d < 4; ++d) {
      p.size[d] = d < ndim ? uint32_t(m.size[d]) : 1u;
      p.so[d] = d < ndim ? int32_t(m.so[d]) : 0, p.sa[d] = d < ndim ? int32_t(m.sa[d]) : 0;
    }
    dispatch(kernel, {VKT_MOVE_COPY}, p, 1);
  });
}

namespace {

// dst (vk) <- src (vk) with strides, broadcasting and float32 / float16 / bfloat16 conversion.
bool copy_on_device(const at::Tensor& dst, const at::Tensor& src) {
  if (src.is_conj() || src.is_neg()) return false;
  std::vector<int64_t> strides(size_t(dst.dim()), 0);
  const int64_t pad = dst.dim() - src.dim();
  for (int64_t i = pad; i < dst.dim(); ++i)
    if (src.size(i - pad) != 1) strides[size_t(i)] = src.stride(i - pad);
  return copy_strided_on_device(dst, reinterpret_cast<uint64_t>(src.const_data_ptr()), strides, src.scalar_type());
}

// self[...] = value on the device (reference backend.cpp:806-816 fill_scalar).
bool fill_on_device(const at::Tensor& self, const at::Scalar& value) {
  const char* label = size_label(self.element_size());
  if (!label || self.is_conj() || self.is_neg()) return false;
  if (self.numel() == 0) return true;
  note_write(self);
  at::Tensor v = at::scalar_tensor(value, at::TensorOptions().dtype(self.scalar_type()));
  uint64_t bits[2] = {0, 0};
  std::memcpy(bits, v.const_data_ptr(), size_t(v.element_size()));
  const MergedDims m = merged_dims(self, nullptr);
  const uint64_t out = reinterpret_cast<uint64_t>(self.mutable_data_ptr());
  const int64_t item = self.element_size();
  return for_each_launch(m, 4, [&](int64_t count, size_t ndim, int64_t oo, int64_t) {
    StridedParams p{};
    p.out = out + uint64_t(oo * item), p.alpha = bits[0], p.beta = bits[1], p.n = uint32_t(count), p.ndim = uint32_t(ndim);
    for (size_t d = 0; d < 4; ++d) p.size[d] = d < ndim ? uint32_t(m.size[d]) : 1u, p.so[d] = d < ndim ? int32_t(m.so[d]) : 0;
    dispatch(std::string("move_") + label, {VKT_MOVE_FILL}, p, 1);
  });
}

// dst <- src where at least one is on vk (reference backend.cpp:765-790).
at::Tensor copy_from(const at::Tensor& src, const at::Tensor& dst, bool non_blocking) {
  TORCH_CHECK(src.sizes() == dst.sizes() || src.numel() == 1 || at::is_expandable_to(src.sizes(), dst.sizes()),
              "copy_: shapes do not broadcast: ", src.sizes(), " -> ", dst.sizes());
  if (dst.numel() == 0) return dst;
  if (is_vk(dst)) note_write(dst);
  const bool same_layout = src.scalar_type() == dst.scalar_type() && src.sizes() == dst.sizes() &&
                           src.strides() == dst.strides() && plain(src) && plain(dst) && !src.is_conj() &&
                           !src.is_neg();
  const uint64_t nbytes = uint64_t(dst.numel()) * dst.element_size();
  if (same_layout) {
    const auto [slo, shi] = element_span(src);
    const auto [dlo, dhi] = element_span(dst);
    (void)shi, (void)dhi;
    const int64_t item = dst.element_size();
    if (is_vk(src) && is_vk(dst)) {
      check(vkt_copy_on_device(reinterpret_cast<uint64_t>(dst.mutable_data_ptr()) + uint64_t(dlo * item),
                               reinterpret_cast<uint64_t>(src.const_data_ptr()) + uint64_t(slo * item), nbytes));
    } else if (is_vk(dst)) {
      check(vkt_copy_to_device(reinterpret_cast<uint64_t>(dst.mutable_data_ptr()) + uint64_t(dlo * item),
                               static_cast<const char*>(src.const_data_ptr()) + slo * item, nbytes));
    } else {
      check(vkt_copy_to_host(static_cast<char*>(dst.mutable_data_ptr()) + dlo * item,
                             reinterpret_cast<uint64_t>(src.const_data_ptr()) + uint64_t(slo * item), nbytes));
    }
    return dst;
  }
  // float8 <-> float32 / float16 / bfloat16 between two vk tensors of the same dense layout:
  // converted on the device, bit for bit as the CPU converts (reference backend.cpp:534-586)
  if (is_vk(src) && is_vk(dst) && src.sizes() == dst.sizes() && src.strides() == dst.strides() && plain(src) &&
      plain(dst) && !src.is_conj() && !src.is_neg()) {
    const int sdt = vkt_dtype(src.scalar_type()), ddt = vkt_dtype(dst.scalar_type());
    const bool s8 = sdt == VKT_E4M3 || sdt == VKT_E5M2, d8 = ddt == VKT_E4M3 || ddt == VKT_E5M2;
    if (sdt >= 0 && ddt >= 0 && (s8 || d8)) {
      const auto [slo, shi] = element_span(src);
      const auto [dlo, dhi] = element_span(dst);
      (void)shi, (void)dhi;
      CastParams p{};
      p.src = reinterpret_cast<uint64_t>(src.const_data_ptr()) + uint64_t(slo * src.element_size());
      p.dst = reinterpret_cast<uint64_t>(dst.mutable_data_ptr()) + uint64_t(dlo * dst.element_size());
      p.n = uint64_t(dst.numel());
      p.src_dtype = uint32_t(sdt);
      p.dst_dtype = uint32_t(ddt);
      dispatch("cast_fp8", {}, p, 1);
      return dst;
    }
  }
  // strides, broadcasting, float conversions: on the device (host <-> device through a dense staging tensor,
  // reference backend.cpp:697-717 copy_cpu_to_vk)
  if (is_vk(src) && is_vk(dst) && copy_on_device(dst, src)) return dst;
  if (is_vk(dst) && !is_vk(src) && size_label(dst.element_size()) && !dst.is_conj() && !dst.is_neg()) {
    at::Tensor host = src.to(dst.scalar_type()).expand(dst.sizes()).contiguous();
    at::Tensor staging = at::empty(dst.sizes(), dst.options());
    check(vkt_copy_to_device(reinterpret_cast<uint64_t>(staging.mutable_data_ptr()), host.const_data_ptr(), nbytes));
    if (copy_on_device(dst, staging)) return dst;
  }
  if (is_vk(src) && !is_vk(dst) && size_label(src.element_size()) && !src.is_conj() && !src.is_neg() &&
      !plain(src) && src.numel() > 0) {
    at::Tensor staging = at::empty(src.sizes(), src.options());
    if (copy_on_device(staging, src)) {
      at::Tensor host = at::empty(src.sizes(), src.options().device(at::kCPU));
      check(vkt_copy_to_host(host.mutable_data_ptr(), reinterpret_cast<uint64_t>(staging.const_data_ptr()),
                             uint64_t(src.numel()) * src.element_size()));
      dst.copy_(host);
      return dst;
    }
  }
  // anything else: through host mirrors
  at::Tensor s = is_vk(src) ? host_mirror(src, true) : src;
  if (!is_vk(dst)) {
    dst.copy_(s);
    return dst;
  }
  at::Tensor d = host_mirror(dst, /*download=*/!plain(dst));
  d.copy_(s);
  const auto [lo, hi] = element_span(dst);
  const int64_t item = dst.element_size();
  check(vkt_copy_to_device(reinterpret_cast<uint64_t>(dst.mutable_data_ptr()) + uint64_t(lo * item),
                           d.storage().data(), uint64_t((hi - lo) * item)));
  return dst;
}

at::Tensor copy_from_and_resize(const at::Tensor& src, const at::Tensor& dst) {
  at::native::resize_output(dst, src.sizes());
  return copy_from(src, dst, false);
}

at::Scalar local_scalar_dense(const at::Tensor& self) {
  TORCH_CHECK(self.numel() == 1, "a Tensor with ", self.numel(), " elements cannot be converted to Scalar");
  return host_mirror(self, true).item();
}

at::Tensor& fill_scalar(at::Tensor& self, const at::Scalar& value) {
  if (!fill_on_device(self, value)) {
    record_fallback("aten::fill_.Scalar");
    at::Tensor host = at::full(self.sizes(), value, self.options().device(at::kCPU));
    copy_from(host, self, false);
  }
  return self;
}

at::Tensor& fill_tensor(at::Tensor& self, const at::Tensor& value) {
  TORCH_CHECK(value.dim() == 0, "fill_ only supports 0-dimension value tensor but got tensor with ", value.dim(),
              " dimensions.");
  return fill_scalar(self, value.item());
}

at::Tensor& zero_(at::Tensor& self) { return fill_scalar(self, 0); }

// ------------------------------------------------------------------ CPU fallback

void boxed_fallback(const c10::OperatorHandle& op, torch::jit::Stack* stack) {
  record_fallback(c10::toString(op.operator_name()));
  at::native::cpu_fallback(op, stack);
}

}  // namespace

void run_fallback(const c10::OperatorHandle& op, torch::jit::Stack* stack, bool) { boxed_fallback(op, stack); }

}  // namespace vk

C10_REGISTER_GUARD_IMPL(PrivateUse1, vk::VkGuardImpl)

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  using namespace vk;
  m.impl("empty.memory_format", &empty_memory_format);
  m.impl("empty_strided", &empty_strided);
  m.impl("as_strided", &at::native::as_strided_tensorimpl);
  m.impl("view", &at::native::view);
  m.impl("_reshape_alias", &at::native::_reshape_alias);
  m.impl("resize_", &resize_);
  m.impl("set_.source_Storage", &set_source_storage);
  m.impl("set_.source_Storage_storage_offset", &set_source_storage_offset);
  m.impl("set_.source_Tensor", &set_source_tensor);
  m.impl("_copy_from", &copy_from);
  m.impl("_copy_from_and_resize", &copy_from_and_resize);
  m.impl("_local_scalar_dense", &local_scalar_dense);
  m.impl("fill_.Scalar", &fill_scalar);
  m.impl("fill_.Tensor", &fill_tensor);
  m.impl("zero_", &zero_);
}

TORCH_LIBRARY_IMPL(_, PrivateUse1, m) { m.fallback(torch::CppFunction::makeFromBoxedFunction<&vk::boxed_fallback>()); }

// ------------------------------------------------------------------ entry points for the Python package
// (the reference exports these from C++ to its pyo3 module: backend.cpp:1795-1850)

extern "C" {

void vkt_register_backend() {
  static std::once_flag once;
  std::call_once(once, [] { c10::SetAllocator(vk::kDevice, vk::allocator()); });
}

void vkt_record_fallback(const char* op) { vk::record_fallback(op); }

// "op=count\n..." into buf (at most cap bytes, NUL terminated); returns the bytes needed.
size_t vkt_fallback_counts(char* buf, size_t cap) {
  std::string text;
  {
    std::lock_guard<std::mutex> lock(vk::g_fallback_mutex);
    for (const auto& kv : vk::g_fallbacks) text += kv.first + "=" + std::to_string(kv.second) + "\n";
  }
  if (buf && cap) {
    const size_t n = text.size() < cap - 1 ? text.size() : cap - 1;
    std::memcpy(buf, text.data(), n);
    buf[n] = 0;
  }
  return text.size() + 1;
}

}  // extern "C"
