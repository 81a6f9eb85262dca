// Per-tensor affine quantised tensors (quint8, qint8, qint32) and fake quantisation for device
// "vk" on MI355X: what the reference registers in crates/pyvk/csrc/quantized.cpp:169-190 and
// python/torch_vulkan/_kernels.py:2134-2136, with its checks and messages.  A quantised tensor's
// storage is an ordinary vk buffer of its integers with the quantizer carried alongside
// (reference quantized.cpp:1-12).  Where the reference composes each operator from elementwise
// kernels over temporaries, here each is one dispatch: "quantize_affine", "dequantize_affine",
// "fake_quant"; copies, clones and flips are strided device moves.
#include "vk.h"

#include <ATen/NativeFunctions.h>
#include <ATen/native/Resize.h>
#include <ATen/quantized/QTensorImpl.h>
#include <ATen/quantized/Quantizer.h>
#include <torch/library.h>

#include <cmath>
#include <cstring>
#include <limits>

namespace vk {
namespace {

at::ScalarType underlying(at::ScalarType q) {  // (reference quantized.cpp:28-40)
  switch (q) {
    case at::kQUInt8: return at::kByte;
    case at::kQInt8: return at::kChar;
    case at::kQInt32: return at::kInt;
    default:
      TORCH_CHECK_NOT_IMPLEMENTED(false, "torch_vulkan: quantized dtype ", q, " is not supported (quint8, qint8 and qint32 are)");
  }
}

uint32_t qtype_code(at::ScalarType q) { return q == at::kQUInt8 ? 0u : q == at::kQInt8 ? 1u : 2u; }

void check_per_tensor_affine(const at::Tensor& q) {
  TORCH_CHECK_NOT_IMPLEMENTED(q.qscheme() == at::kPerTensorAffine,
                              "torch_vulkan: only per-tensor affine quantized tensors are supported, got ", q.qscheme());
}

// The integers of quantised tensor q as a vk tensor sharing its storage (reference :49-53).
at::Tensor raw(const at::Tensor& q) {
  at::Tensor r = at::empty({0}, q.options().dtype(underlying(q.scalar_type())));
  r.set_(q.storage(), q.storage_offset(), q.sizes(), q.strides());
  return r;
}

at::Tensor like(const at::Tensor& q, at::IntArrayRef sizes, at::MemoryFormat mf = at::MemoryFormat::Contiguous) {
  return at::new_qtensor(sizes, q.options().memory_format(mf), q.quantizer());
}

uint32_t float_bits(double v) {
  const float f = static_cast<float>(v);
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

at::Tensor quantize_per_tensor(const at::Tensor& self, double scale, int64_t zero_point, at::ScalarType dtype) {
  TORCH_CHECK(self.scalar_type() == at::kFloat, "Quantize only works on Float Tensor, got ", self.scalar_type());
  underlying(dtype);
  const at::MemoryFormat mf = self.suggest_memory_format();
  auto quantizer = at::make_per_tensor_affine_quantizer(scale, zero_point, dtype);
  at::Tensor q = at::new_qtensor(self.sizes(), self.options().dtype(dtype).memory_format(mf), quantizer);
  if (q.numel() == 0) return q;
  at::Tensor x = self.contiguous(mf);  // (the same dense layout as q: one flat pass)
  QuantParams p{};
  p.src = gpu_address(x), p.dst = gpu_address_out(q), p.n = static_cast<uint64_t>(q.numel());
  p.scale_bits = float_bits(scale), p.zero_point = static_cast<int32_t>(zero_point);
  dispatch("quantize_affine", {qtype_code(dtype)}, p, 1);
  return q;
}

at::Tensor quantize_per_tensor_tensor_qparams(const at::Tensor& self, const at::Tensor& scale, const at::Tensor& zero_point,
                                              at::ScalarType dtype) {
  return vk::quantize_per_tensor(self, scale.item<double>(), zero_point.item<int64_t>(), dtype);
}

at::Tensor dequantize(const at::Tensor& self) {
  check_per_tensor_affine(self);
  const at::MemoryFormat mf = self.suggest_memory_format();
  at::Tensor q = self.is_non_overlapping_and_dense() ? self : vk_clone_quantized(self, mf);
  at::Tensor out = at::empty_strided(q.sizes(), q.strides(), q.options().dtype(at::kFloat));
  if (out.numel() == 0) return out;
  QuantParams p{};
  p.src = gpu_address(q), p.dst = gpu_address_out(out), p.n = static_cast<uint64_t>(q.numel());
  p.scale_bits = float_bits(self.q_scale()), p.zero_point = static_cast<int32_t>(self.q_zero_point());
  dispatch("dequantize_affine", {qtype_code(self.scalar_type())}, p, 1);
  return out;
}

at::Tensor int_repr(const at::Tensor& self) { return raw(self).clone(at::MemoryFormat::Preserve); }

at::Tensor clone(const at::Tensor& self, std::optional<at::MemoryFormat> memory_format) {
  at::MemoryFormat mf = memory_format.value_or(at::MemoryFormat::Preserve);
  if (mf == at::MemoryFormat::Preserve) mf = self.suggest_memory_format();
  return vk_clone_quantized(self, mf);
}

at::Tensor& copy_(at::Tensor& self, const at::Tensor& src, bool /*non_blocking*/) {  // (reference :140-159)
  TORCH_CHECK(self.is_quantized() && src.is_quantized(), "torch_vulkan: copies between quantized and other tensors are not supported");
  TORCH_CHECK(self.scalar_type() == src.scalar_type(), "Quantized Copy only works with same qtype");
  TORCH_CHECK(self.qscheme() == src.qscheme(), "Quantized Copy only works with same qscheme");
  at::set_quantizer_(self, src.quantizer());
  if (is_vk(self) && is_vk(src)) {
    raw(self).copy_(raw(src));
  } else {
    // (to or from the CPU: the integers, through a dense tensor of their dtype)
    at::Tensor s = src.is_cpu() ? src.int_repr() : raw(src);
    at::Tensor d = self.is_cpu() ? at::empty({0}, s.options().device(at::kCPU)) : raw(self);
    if (self.is_cpu()) d.set_(self.storage(), self.storage_offset(), self.sizes(), self.strides());
    d.copy_(s);
  }
  return self;
}

// out[i...] = self[.., size - 1 - i, ..] along dims: a strided device move whose source starts at the last
// element of each flipped dim and walks backwards.
at::Tensor flip_raw(const at::Tensor& self, at::IntArrayRef dims) {
  at::Tensor out = at::empty(self.sizes(), self.options());
  if (out.numel() == 0) return out;
  std::vector<int64_t> strides(self.strides().begin(), self.strides().end());
  int64_t offset = 0;
  std::vector<bool> seen(static_cast<size_t>(self.dim()), false);
  for (int64_t d : dims) {
    const int64_t w = at::maybe_wrap_dim(d, self.dim());
    TORCH_CHECK(!seen[static_cast<size_t>(w)], "dim ", w, " appears multiple times in the list of dims");
    seen[static_cast<size_t>(w)] = true;
    offset += (self.size(w) - 1) * strides[static_cast<size_t>(w)];
    strides[static_cast<size_t>(w)] = -strides[static_cast<size_t>(w)];
  }
  const uint64_t base = gpu_address(self) + static_cast<uint64_t>(offset * self.element_size());
  if (!copy_strided_on_device(out, base, strides, self.scalar_type())) {
    return on_cpu("aten::flip", "", self, dims)[0].toTensor();
  }
  return out;
}

at::Tensor flip_quantized(const at::Tensor& self, at::IntArrayRef dims) {
  at::Tensor out = like(self, self.sizes());
  raw(out).copy_(flip_raw(raw(self), dims));
  return out;
}

// ---------------------------------------------------------------- fake quantisation (reference _kernels.py:1613-1676)

std::tuple<at::Tensor, at::Tensor> fake_quant_launch(const at::Tensor& self, const at::Tensor* scales, const at::Tensor* zero_points,
                                                      double scale, int64_t zero_point, int64_t axis, int64_t quant_min,
                                                      int64_t quant_max) {
  const int dt = vkt_dtype(self.scalar_type());
  TORCH_CHECK_NOT_IMPLEMENTED(dt == VKT_F32 || dt == VKT_F16 || dt == VKT_BF16, "torch_vulkan: fake quantisation of ", self.scalar_type(),
                              " tensors is not supported (float32, float16 and bfloat16 are)");
  const bool per_channel = scales != nullptr;
  // per tensor: any dense layout as it is (elementwise); per channel: contiguous, so that a flat index names its channel
  at::Tensor x = per_channel ? self.contiguous() : (self.is_non_overlapping_and_dense() ? self : self.contiguous());
  at::Tensor out = at::empty_strided(x.sizes(), x.strides(), x.options());
  at::Tensor mask = at::empty_strided(x.sizes(), x.strides(), x.options().dtype(at::kBool));
  if (x.numel() == 0) return {out, mask};
  QuantParams p{};
  p.src = gpu_address(x), p.dst = gpu_address_out(out), p.mask = gpu_address_out(mask), p.n = static_cast<uint64_t>(x.numel());
  p.qmin = quant_min, p.qmax = quant_max, p.dtype = static_cast<uint32_t>(dt);
  if (!per_channel) {
    p.scale_bits = float_bits(scale), p.zero_point = static_cast<int32_t>(zero_point);
    dispatch("fake_quant", {0u, 0u}, p, 1);
    return {out, mask};
  }
  TORCH_CHECK(x.numel() < (int64_t(1) << 32), "torch_vulkan: per-channel fake quantisation of 2^32 or more elements");
  const bool float_zp = zero_points->is_floating_point();
  at::Tensor s = scales->to(at::kFloat).contiguous();
  at::Tensor z = float_zp ? zero_points->to(at::kFloat).contiguous() : zero_points->contiguous();
  int64_t inner = 1;
  for (int64_t d = axis + 1; d < x.dim(); ++d) inner *= x.size(d);
  p.scales = gpu_address(s), p.zero_points = gpu_address(z);
  p.channels = static_cast<uint32_t>(x.size(axis)), p.inner = static_cast<uint32_t>(inner);
  dispatch("fake_quant", {1u, float_zp ? 1u : 0u}, p, 1);
  return {out, mask};
}

std::tuple<at::Tensor, at::Tensor> fake_quant_tensor_qparams(const at::Tensor& self, const at::Tensor& scale, const at::Tensor& zero_point,
                                                              const at::Tensor& fake_quant_enabled, int64_t quant_min,
                                                              int64_t quant_max) {
  TORCH_CHECK(quant_min <= quant_max, "`quant_min` should be less than or \
        equal to `quant_max`.");
  if (fake_quant_enabled.reshape({-1})[0].item<int64_t>() == 0) {
    return {self.clone(at::MemoryFormat::Preserve), at::ones_like(self, self.options().dtype(at::kBool))};
  }
  return fake_quant_launch(self, nullptr, nullptr, scale.reshape({-1})[0].item<double>(), zero_point.reshape({-1})[0].item<int64_t>(), 0,
                           quant_min, quant_max);
}

std::tuple<at::Tensor, at::Tensor> fake_quant_per_tensor(const at::Tensor& self, double scale, int64_t zero_point, int64_t quant_min,
                                                          int64_t quant_max) {
  TORCH_CHECK(quant_min <= quant_max, "`quant_min` should be less than or \
        equal to `quant_max`.");
  TORCH_CHECK(zero_point >= quant_min && zero_point <= quant_max, "`zero_point` must be between `quant_min` and `quant_max`.");
  return fake_quant_launch(self, nullptr, nullptr, scale, zero_point, 0, quant_min, quant_max);
}

std::tuple<at::Tensor, at::Tensor> fake_quant_per_channel(const at::Tensor& self, const at::Tensor& scale, const at::Tensor& zero_point,
                                                           int64_t axis, int64_t quant_min, int64_t quant_max) {
  // (ATen's checks, as the reference restates them: _kernels.py:1652-1667)
  TORCH_CHECK(scale.scalar_type() == at::kFloat || scale.scalar_type() == at::kBFloat16, "Scale must be Float or BFloat16, found ",
              scale.scalar_type());
  TORCH_CHECK(zero_point.scalar_type() == at::kInt || zero_point.scalar_type() == at::kFloat || zero_point.scalar_type() == at::kHalf,
              "Zero-point must be Int32, Float or Half, found ", zero_point.scalar_type());
  TORCH_CHECK(scale.dim() == 1, "scale should be a 1-D tensor");
  TORCH_CHECK(zero_point.dim() == 1, "zero point should be a 1-D tensor");
  TORCH_CHECK(scale.numel() == zero_point.numel(), "scale and zero-point need to have the same dimensions");
  TORCH_CHECK(axis >= 0 && axis <= self.dim(), "`axis` must be between 0 and number of dimensions of input");
  TORCH_CHECK(axis < self.dim() && scale.numel() == self.size(axis), "dimensions of scale and zero-point are not consistent with input tensor");
  TORCH_CHECK(quant_min <= quant_max, "`quant_min` should be less than or \
        equal to `quant_max`.");
  if (!zero_point.is_floating_point() && zero_point.numel() > 0) {
    at::Tensor z = zero_point.cpu();
    TORCH_CHECK(z.min().item<int64_t>() >= quant_min && z.max().item<int64_t>() <= quant_max,
                "`zero_point` must be between `quant_min` and `quant_max`.");
  }
  return fake_quant_launch(self, &scale, &zero_point, 0.0, 0, axis, quant_min, quant_max);
}

// ---------------------------------------------------------------- the QAT observer (reference _kernels.py:1678-1762)

// (scale, zero point) from a range as the CPU chooses them (ATen's quant_utils::ChooseQuantizationParams; the
// scale is a float32 from the start, the zero point is derived from it in double).
std::pair<float, int32_t> choose_qparams(float mn, float mx, int32_t qmin, int32_t qmax, bool preserve_sparsity) {
  TORCH_CHECK(mn <= mx, "In ChooseQuantizationParams, min should be less than or equal to max");
  if (mn < 0 && mx > 0 && preserve_sparsity) {
    const int32_t sqmin = -((qmax - qmin) / 2 + 1), sqmax = (qmax - qmin) / 2;
    const double a = std::fabs(static_cast<double>(mn / static_cast<float>(sqmin)));
    const double b = std::fabs(static_cast<double>(mx / static_cast<float>(sqmax)));
    const double max_scale = a > b ? a : b;
    mn = static_cast<float>(max_scale * sqmin), mx = static_cast<float>(max_scale * sqmax);
  }
  mn = mn < 0.0f ? mn : 0.0f, mx = mx > 0.0f ? mx : 0.0f;
  TORCH_CHECK(qmin < qmax, "In ChooseQuantizationParams, qmin should be less than qmax");
  float scale = static_cast<float>((static_cast<double>(mx) - static_cast<double>(mn)) / static_cast<double>(qmax - qmin));
  if (scale == 0.0f || std::isinf(1.0f / scale)) scale = 0.1f;
  TORCH_CHECK(scale > 0, "quantization scale should be > 0");
  const float small = 6.1e-5f;
  if (scale < small) {
    const float org = scale;
    scale = small;
    if (mn == 0.0f) mx = small * static_cast<float>(qmax - qmin);
    else if (mx == 0.0f) mn = -small * static_cast<float>(qmax - qmin);
    else {
      const float amp = small / org;
      mn = mn * amp, mx = mx * amp;
    }
  }
  const double ds = static_cast<double>(scale);
  const double z_min = qmin - static_cast<double>(mn) / ds, z_max = qmax - static_cast<double>(mx) / ds;
  const double e_min = std::fabs(static_cast<double>(qmin)) - std::fabs(static_cast<double>(mn) / ds);
  const double e_max = std::fabs(static_cast<double>(qmax)) - std::fabs(static_cast<double>(mx) / ds);
  double z = e_min < e_max ? z_min : z_max;
  if (mn < 0 && mx > 0 && preserve_sparsity) z = (qmin + qmax) / 2.0;
  const int32_t zp = z < qmin ? qmin : (z > qmax ? qmax : static_cast<int32_t>(std::nearbyint(z)));
  return {scale, zp};
}

std::tuple<at::Tensor, at::Tensor> fused_moving_avg_obs_fq_helper(const at::Tensor& self, const at::Tensor& observer_on,
                                                                   const at::Tensor& fake_quant_on, at::Tensor& running_min,
                                                                   at::Tensor& running_max, at::Tensor& scale, at::Tensor& zero_point,
                                                                   double averaging_const, int64_t quant_min, int64_t quant_max,
                                                                   int64_t ch_axis, bool per_row_fake_quant, bool symmetric_quant) {
  TORCH_CHECK(ch_axis < self.dim(), "Error in fused_moving_avg_obs_fake_quant_cpu: ch_axis must be < self.dim()");
  const int dt = vkt_dtype(self.scalar_type());
  TORCH_CHECK_NOT_IMPLEMENTED(dt == VKT_F32 || dt == VKT_F16 || dt == VKT_BF16, "torch_vulkan: the fake-quantisation observer takes float32, float16 and bfloat16 tensors");
  const bool observe = observer_on.reshape({-1})[0].item<int64_t>() != 0;
  at::Tensor x = self;
  if (per_row_fake_quant) {
    if (self.dim() != 2) {
      std::vector<int64_t> perm(static_cast<size_t>(self.dim()));
      for (size_t i = 0; i < perm.size(); ++i) perm[i] = static_cast<int64_t>(i);
      perm[static_cast<size_t>(ch_axis)] = 0, perm[0] = ch_axis;
      x = self.permute(perm).flatten(1);
    }
    const int64_t size = self.size(ch_axis);
    if (running_min.numel() == 0) {
      running_min.resize_({size}).fill_(std::numeric_limits<float>::infinity());
      running_max.resize_({size}).fill_(-std::numeric_limits<float>::infinity());
      scale.resize_({size});
      zero_point.resize_({size});
    }
  }
  // the running range lives on the device; its few values are updated on the host, as the reference does
  at::Tensor rmin = running_min.to(at::kCPU, at::kFloat).contiguous().clone(), rmax = running_max.to(at::kCPU, at::kFloat).contiguous().clone();
  if (observe) {
    if (per_row_fake_quant) {
      TORCH_CHECK(ch_axis == 0, "Per-channel FakeQuant in fused_moving_avg_obs_fake_quant is only supported on axis == 0");
    }
    at::Tensor rows = (per_row_fake_quant ? x : x.reshape({1, -1})).contiguous();
    TORCH_CHECK(rows.size(0) == rmin.numel() && rows.size(0) < 65536 && rows.size(1) > 0 && rows.size(1) < (int64_t(1) << 32),
                "torch_vulkan: the observer's running range has ", rmin.numel(), " values for ", rows.size(0), " rows");
    at::Tensor cur_min = at::empty({rows.size(0)}, rows.options().dtype(at::kFloat)), cur_max = at::empty_like(cur_min);
    MinMaxParams p{};
    p.src = gpu_address(rows), p.out_min = gpu_address_out(cur_min), p.out_max = gpu_address_out(cur_max);
    p.rows = static_cast<uint32_t>(rows.size(0)), p.cols = static_cast<uint32_t>(rows.size(1)), p.ld = p.cols;
    p.dtype = static_cast<uint32_t>(dt);
    dispatch("aminmax", {}, p, 1);
    at::Tensor cmin = cur_min.cpu(), cmax = cur_max.cpu();
    const float c = static_cast<float>(averaging_const);
    float* lo = rmin.data_ptr<float>();
    float* hi = rmax.data_ptr<float>();
    const float* a = cmin.const_data_ptr<float>();
    const float* b = cmax.const_data_ptr<float>();
    for (int64_t i = 0; i < rmin.numel(); ++i) {
      // (a value that is still infinite takes this batch's; single float32 operations, as the CPU's)
      volatile float dl = a[i] - lo[i], dh = b[i] - hi[i];
      volatile float pl = c * dl, ph = c * dh;
      lo[i] = std::isinf(lo[i]) ? a[i] : lo[i] + pl;
      hi[i] = std::isinf(hi[i]) ? b[i] : hi[i] + ph;
    }
    running_min.copy_(rmin.reshape(running_min.sizes()));
    running_max.copy_(rmax.reshape(running_max.sizes()));
  }
  if (fake_quant_on.reshape({-1})[0].item<int64_t>() == 0) {
    return {self.clone(at::MemoryFormat::Preserve), at::ones_like(self, self.options().dtype(at::kBool))};
  }
  const int64_t count = per_row_fake_quant ? rmin.numel() : 1;
  at::Tensor scales = at::empty({count}, at::kFloat), zps = at::empty({count}, at::kInt);
  for (int64_t i = 0; i < count; ++i) {
    auto qp = choose_qparams(rmin.const_data_ptr<float>()[i], rmax.const_data_ptr<float>()[i], static_cast<int32_t>(quant_min),
                             static_cast<int32_t>(quant_max), symmetric_quant);
    scales.data_ptr<float>()[i] = qp.first, zps.data_ptr<int32_t>()[i] = qp.second;
  }
  scale.reshape({-1}).narrow(0, 0, count).copy_(scales);
  zero_point.reshape({-1}).narrow(0, 0, count).copy_(zps.to(zero_point.scalar_type()));
  if (per_row_fake_quant) return fake_quant_per_channel(self, scale, zero_point, ch_axis, quant_min, quant_max);
  TORCH_CHECK(quant_min <= quant_max, "`quant_min` should be less than or \
        equal to `quant_max`.");
  return fake_quant_launch(self, nullptr, nullptr, scales.data_ptr<float>()[0], zps.data_ptr<int32_t>()[0], 0, quant_min, quant_max);
}

}  // namespace

// A dense copy of quantised tensor q in memory format mf, its quantizer kept.
at::Tensor vk_clone_quantized(const at::Tensor& q, at::MemoryFormat mf) {
  at::Tensor out = like(q, q.sizes(), mf);
  raw(out).copy_(raw(q));
  return out;
}

}  // namespace vk

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  m.impl("quantize_per_tensor", TORCH_FN(vk::quantize_per_tensor));
  m.impl("quantize_per_tensor.tensor_qparams", TORCH_FN(vk::quantize_per_tensor_tensor_qparams));
  m.impl("_fake_quantize_per_tensor_affine_cachemask_tensor_qparams", TORCH_FN(vk::fake_quant_tensor_qparams));
  m.impl("fake_quantize_per_tensor_affine_cachemask", TORCH_FN(vk::fake_quant_per_tensor));
  m.impl("fake_quantize_per_channel_affine_cachemask", TORCH_FN(vk::fake_quant_per_channel));
  m.impl("flip", TORCH_FN(vk::flip_raw));
  m.impl("_fused_moving_avg_obs_fq_helper", TORCH_FN(vk::fused_moving_avg_obs_fq_helper));
}

TORCH_LIBRARY_IMPL(aten, QuantizedPrivateUse1, m) {
  m.impl("_empty_affine_quantized", TORCH_FN(at::native::empty_affine_quantized));
  m.impl("empty_quantized", TORCH_FN(at::native::empty_quantized));
  m.impl("empty.memory_format", TORCH_FN(at::native::empty_unknown_quantized));
  m.impl("empty_strided", TORCH_FN(at::native::empty_strided_unknown_quantized));
  m.impl("view", TORCH_FN(at::native::view));
  m.impl("_reshape_alias", TORCH_FN(at::native::_reshape_alias));
  m.impl("as_strided", TORCH_FN(at::native::as_strided_qtensorimpl));
  m.impl("q_scale", TORCH_FN(at::native::q_scale_quant));
  m.impl("q_zero_point", TORCH_FN(at::native::q_zero_point_quant));
  m.impl("qscheme", TORCH_FN(at::native::qscheme_quant));
  m.impl("dequantize.self", TORCH_FN(vk::dequantize));
  m.impl("int_repr", TORCH_FN(vk::int_repr));
  m.impl("clone", TORCH_FN(vk::clone));
  m.impl("copy_", TORCH_FN(vk::copy_));
  m.impl("flip", TORCH_FN(vk::flip_quantized));
}
