// Quantised matrix products for device "vk" on MI355X: the aten schemas the reference
// registers (crates/pyvk/csrc/quant.cpp:315-322), with its argument checks and messages
// (which are the CPU kernels'), each queued through the C ABI onto the gfx950 kernels:
//
//   _weight_int8pack_mm          "qmm8_<T>"   (reference :59-119; parameter block :31-37)
//   _dyn_quant_pack_4bit_weight  "qmm4_packvec" (reference :127-144 composes casts + cat)
//   _dyn_quant_matmul_4bit       "qmm4c_<T>" over a compact side-car built once per packed
//                                tensor, else "qmm4_<T>" on the reference's buffers (:146-204)
//   _scaled_mm / _scaled_mm.out  "fp8mm": one fused kernel in place of the composite at :279-300
#include "vk.h"

#include <ATen/native/Resize.h>
#include <c10/util/intrusive_ptr.h>
#include <torch/library.h>

#include <algorithm>
#include <list>
#include <mutex>
#include <sstream>

namespace vk {
namespace {

constexpr int64_t kMaxRows = 65535;  // rows per dispatch of the int4 kernels (quant.cpp:29)

const char* float_label(at::ScalarType t) {  // (reference quant.cpp:47-51)
  if (t == at::kFloat) return "f32";
  if (t == at::kHalf) return "f16";
  if (t == at::kBFloat16) return "bf16";
  return nullptr;
}

bool all_vk(std::initializer_list<const at::Tensor*> ts) {
  return std::all_of(ts.begin(), ts.end(), [](const at::Tensor* t) { return t == nullptr || is_vk(*t); });
}

// ------------------------------------------------------------ int8 weights

at::Tensor weight_int8pack_mm(const at::Tensor& A, const at::Tensor& B, const at::Tensor& scales) {
  // (ATen/native/LinearAlgebra.cpp _weight_int8pack_mm_cpu's checks, reference quant.cpp:60-72)
  static constexpr const char* func = "_weight_int8pack_mm_cpu";
  auto M = A.size(0);
  auto N = B.size(0);
  auto K = A.size(1);
  TORCH_CHECK(A.dtype() == at::kBFloat16 || A.dtype() == at::kHalf || A.dtype() == at::kFloat, func,
              " : expect A to be either 32-bit or 16-bit float tensor.");
  TORCH_CHECK(A.dim() == 2, func, " : expect A to be 2D tensor.");
  TORCH_CHECK(A.stride(1) == 1, func, " : A must be contiguous on the last dimension.");
  TORCH_CHECK(B.dtype() == at::kChar, func, " : expect B to be int8 tensor.");
  TORCH_CHECK(B.is_contiguous(), func, " : expect B to be contiguous.");
  TORCH_CHECK(B.size(1) == K, func, " : expect B.size(1) == ", K);
  TORCH_CHECK(scales.dim() == 1 && scales.size(0) == N, func, " : expect scales to be 1d tensor with size ", N);

  const char* label = float_label(A.scalar_type());
  if (!all_vk({&A, &B, &scales}) || label == nullptr || A.stride(0) >= (int64_t(1) << 31) ||
      B.numel() >= (int64_t(1) << 32) || M * N >= (int64_t(1) << 32)) {
    return on_cpu("aten::_weight_int8pack_mm", "", A, B, scales)[0].toTensor();
  }
  at::Tensor C = at::empty({M, N}, A.options());
  if (C.numel() == 0) return C;
  // (the CPU reads the scales as A's dtype)
  at::Tensor s = scales.to(A.scalar_type()).contiguous();
  Q8Params p{};
  p.a = gpu_address(A);
  p.b = gpu_address(B);
  p.scales = gpu_address(s);
  p.c = gpu_address_out(C);
  p.m = static_cast<uint32_t>(M);
  p.n = static_cast<uint32_t>(N);
  p.k = static_cast<uint32_t>(K);
  p.a_sm = static_cast<int32_t>(A.stride(0));
  p.a_sk = 1;
  // (the reference's specialisation constant: ROWS = M for its GEMV path, 0 for tiles; the
  // library plans the launch from the block)
  dispatch(std::string("qmm8_") + label, {M <= 8 ? static_cast<uint32_t>(M) : 0u}, p, 1);
  return C;
}

// ------------------------------------------------------------ int4 weights, int8 activations

at::Tensor dyn_quant_pack_4bit_weight(const at::Tensor& weights, const at::Tensor& scales_zeros,
                                      const std::optional<at::Tensor>& bias, int64_t block_size,
                                      int64_t in_features, int64_t out_features) {
  TORCH_CHECK(weights.dtype() == at::kByte, "_dyn_quant_pack_4bit_weight_cpu", " : expect weight to be kByte.");
  TORCH_CHECK(block_size == in_features || (!(block_size % 32) && !(in_features % block_size)),
              "_dyn_quant_pack_4bit_weight_cpu", ": Group size should be multiple of 32, in_features [", in_features,
              "]. Provided ", block_size);
  const bool has_bias = bias.has_value() && bias->defined();
  const int sdt = vkt_dtype(scales_zeros.scalar_type()), bdt = has_bias ? vkt_dtype(bias->scalar_type()) : VKT_F32;
  const int64_t total = weights.numel() + scales_zeros.numel() + (has_bias ? bias->numel() : 0);
  if (!all_vk({&weights, &scales_zeros, has_bias ? &*bias : nullptr}) || sdt < 0 || sdt > VKT_BF16 || bdt < 0 ||
      bdt > VKT_BF16 || total >= (int64_t(1) << 32)) {
    return on_cpu("aten::_dyn_quant_pack_4bit_weight", "", weights, scales_zeros, bias, block_size, in_features,
                  out_features)[0]
        .toTensor();
  }
  // the CPU's reference layout (reference quant.cpp:123-144): cat(bytes, scales, bias) as float32
  at::Tensor w = weights.contiguous(), s = scales_zeros.contiguous();
  at::Tensor b = has_bias ? bias->contiguous() : at::Tensor();
  at::Tensor out = at::empty({total}, weights.options().dtype(at::kFloat));
  if (total == 0) return out;
  Q4VecParams p{};
  p.weights = gpu_address(w);
  p.scales = gpu_address(s);
  p.bias = has_bias ? gpu_address(b) : 0;
  p.out = gpu_address_out(out);
  p.nw = static_cast<uint32_t>(w.numel());
  p.ns = static_cast<uint32_t>(s.numel());
  p.nb = has_bias ? static_cast<uint32_t>(b.numel()) : 0;
  p.scales_dtype = static_cast<uint32_t>(sdt);
  p.bias_dtype = static_cast<uint32_t>(bdt);
  dispatch("qmm4_packvec", {}, p, 1);
  return out;
}

// Compact side-cars of packed weight vectors, per live packed tensor and layout (0: streamed
// by the kernel for at most 3 rows, 1: for the matrix cores; a weight that sees both kinds of
// call holds both, each the size of the nibbles plus scales): keyed by the storage, its data
// pointer and the tensor's version counter, dropped when the storage dies or the tensor is
// written to.  (The reference streams the float32-expanded vector
// itself: 4 bytes of traffic per byte of nibbles.)
struct SideCar {
  c10::weak_intrusive_ptr<c10::StorageImpl> storage;
  const void* data;
  int64_t version;
  int64_t offset, numel, bs, k, n;
  uint32_t layout;
  at::Tensor compact;
};
std::mutex g_sidecar_mutex;
std::list<SideCar> g_sidecars;

at::Tensor sidecar_for(const at::Tensor& packed, int64_t bs, int64_t K, int64_t N, bool has_bias, uint32_t layout) {
  const uint64_t bytes = vkt_qmm4c_bytes(static_cast<uint32_t>(N), static_cast<uint32_t>(K), static_cast<uint32_t>(bs));
  if (bytes == 0) return at::Tensor();
  std::lock_guard<std::mutex> lock(g_sidecar_mutex);
  for (auto it = g_sidecars.begin(); it != g_sidecars.end();) {
    if (it->storage.expired()) {
      it = g_sidecars.erase(it);
      continue;
    }
    if (it->storage._unsafe_get_target() == packed.storage().unsafeGetStorageImpl() && it->data == packed.const_data_ptr() &&
        it->version == packed._version() && it->offset == packed.storage_offset() && it->numel == packed.numel() &&
        it->bs == bs && it->k == K && it->n == N && it->layout == layout) {
      return it->compact;
    }
    ++it;
  }
  at::Tensor compact = at::empty({static_cast<int64_t>(bytes)}, packed.options().dtype(at::kByte));
  Q4PackParams p{};
  p.packed = gpu_address(packed);
  p.compact = gpu_address_out(compact);
  p.n = static_cast<uint32_t>(N);
  p.k = static_cast<uint32_t>(K);
  p.bs = static_cast<uint32_t>(bs);
  p.has_bias = has_bias ? 1u : 0u;
  dispatch("qmm4c_pack", {layout}, p, 1);
  if (g_sidecars.size() >= 64) g_sidecars.pop_front();
  g_sidecars.push_back(SideCar{c10::weak_intrusive_ptr<c10::StorageImpl>(packed.storage().getWeakStorageImpl()),
                               packed.const_data_ptr(), packed._version(), packed.storage_offset(), packed.numel(), bs,
                               K, N, layout, compact});
  return compact;
}

at::Tensor dyn_quant_matmul_4bit(const at::Tensor& inp, const at::Tensor& packed_weights, int64_t block_size,
                                 int64_t in_features, int64_t out_features) {
  // (ATen/native/LinearAlgebra.cpp _dyn_quant_matmul_4bit_cpu, reference quant.cpp:146-177)
  TORCH_CHECK(inp.dtype() == at::kFloat || (inp.dtype() == at::kBFloat16 && block_size == in_features),
              "_dyn_quant_matmul_4bit_cpu", " : expect input to be float32 or bfloat16 tensor.");
  TORCH_CHECK(block_size == in_features || (!(block_size % 32) && !(in_features % block_size)),
              "_dyn_quant_matmul_4bit_cpu", ": Group size should be multiple of 32, in_features [", in_features,
              "]. Provided ", block_size);
  TORCH_CHECK(inp.dim() == 2 && inp.size(1) == in_features, "_dyn_quant_matmul_4bit: expected input of shape [M, ",
              in_features, "], got ", inp.sizes());
  auto M = inp.size(0);
  const char* label = float_label(inp.scalar_type());
  if (!all_vk({&inp, &packed_weights}) || label == nullptr ||
      M * std::max<int64_t>(in_features, out_features) >= (int64_t(1) << 31) ||
      packed_weights.numel() >= (int64_t(1) << 31)) {
    return on_cpu("aten::_dyn_quant_matmul_4bit", "", inp, packed_weights, block_size, in_features, out_features)[0]
        .toTensor();
  }
  int64_t N = out_features, K = in_features;
  at::Tensor output = at::empty({M, N}, inp.options());
  const int64_t weights_elements = N * K / 2;
  const int64_t scale_elements = N * (K / block_size);
  TORCH_CHECK(packed_weights.numel() >= (weights_elements + scale_elements), "Invalid packed weight tensor size");
  int64_t bias_elements = packed_weights.numel() - (weights_elements + scale_elements);
  if (bias_elements) {
    TORCH_CHECK(bias_elements == N, "Expected bias length to match output dimension");
  }
  if (output.numel() == 0) return output;
  at::Tensor x = inp.contiguous();
  at::Tensor packed = packed_weights.to(at::kFloat).contiguous();
  const uint32_t groupwise = block_size != K ? 1u : 0u;
  const int64_t item = x.element_size();

  const uint32_t layout = M > 3 ? 1u : 0u;  // (measured at K = 4096, N = 11008: 4 rows take 19.0 us streaming, 15.3 on the matrix cores)
  at::Tensor compact = sidecar_for(packed, block_size, K, N, bias_elements != 0, layout);
  if (compact.defined()) {
    for (int64_t r0 = 0; r0 < M; r0 += kMaxRows) {
      const int64_t rows_here = std::min<int64_t>(M - r0, kMaxRows);
      at::Tensor q = at::empty({static_cast<int64_t>(vkt_qmm4c_q_bytes(static_cast<uint32_t>(rows_here),
                                                                      static_cast<uint32_t>(K)))},
                               inp.options().dtype(at::kByte));
      at::Tensor rows = at::empty({rows_here, 2}, inp.options().dtype(at::kFloat));
      Q4CParams p{};
      p.inp = gpu_address(x) + static_cast<uint64_t>(r0 * K * item);
      p.q = gpu_address_out(q);
      p.rows = gpu_address_out(rows);
      p.compact = gpu_address(compact);
      p.out = gpu_address_out(output) + static_cast<uint64_t>(r0 * N * item);
      p.m = static_cast<uint32_t>(rows_here);
      p.n = static_cast<uint32_t>(N);
      p.k = static_cast<uint32_t>(K);
      p.bs = static_cast<uint32_t>(block_size);
      p.has_bias = bias_elements != 0 ? 1u : 0u;
      dispatch(std::string("qmm4c_") + label, {2u, groupwise, layout}, p, 1);
    }
    return output;
  }
  // no compact form: the reference's two launches on its own buffers (quant.cpp:178-202)
  at::Tensor q = at::empty({M, K}, inp.options().dtype(at::kInt));
  at::Tensor rows = at::empty({M, 2}, inp.options().dtype(at::kFloat));
  for (int64_t r0 = 0; r0 < M; r0 += kMaxRows) {
    const int64_t rows_here = std::min<int64_t>(M - r0, kMaxRows);
    Q4Params p{};
    p.inp = gpu_address(x) + static_cast<uint64_t>(r0 * K * item);
    p.q = gpu_address_out(q) + static_cast<uint64_t>(r0 * K * 4);
    p.rows = gpu_address_out(rows) + static_cast<uint64_t>(r0 * 2 * 4);
    p.packed = gpu_address(packed);
    p.out = gpu_address_out(output) + static_cast<uint64_t>(r0 * N * item);
    p.m = static_cast<uint32_t>(rows_here);
    p.n = static_cast<uint32_t>(N);
    p.k = static_cast<uint32_t>(K);
    p.bs = static_cast<uint32_t>(block_size);
    p.has_bias = bias_elements != 0 ? 1u : 0u;
    dispatch(std::string("qmm4_") + label, {0u, groupwise}, p, static_cast<uint32_t>(rows_here));
    dispatch(std::string("qmm4_") + label, {1u, groupwise}, p, static_cast<uint32_t>((N + 31) / 32),
             static_cast<uint32_t>((rows_here + 7) / 8));
  }
  return output;
}

// ------------------------------------------------------------ float8 (_scaled_mm)

// (ATen/native/ScaledBlas.cpp: invalid_scaling_config; reference quant.cpp:209-223)
[[noreturn]] void invalid_scaling_config(const at::Tensor& mat_a, const at::Tensor& mat_b, const at::Tensor& scale_a,
                                         const at::Tensor& scale_b) {
  std::stringstream ss;
  ss << "Invalid scaling configuration.\n";
  ss << "- For TensorWise scaling, a and b should be float8, scales should be float and singletons.\n";
  ss << "- For RowWise scaling, a and b should be float8, scales should be float, scale_a should be (";
  ss << mat_a.size(0) << ", 1) and scale_b should be (1, " << mat_b.size(1) << "), and both should be contiguous.\n";
  ss << "Got mat_a.dtype()=" << mat_a.scalar_type();
  ss << ", scale_a.dtype()=" << scale_a.scalar_type() << ", scale_a.size()=" << scale_a.sizes()
     << ", scale_a.stride()=" << scale_a.strides();
  ss << ", mat_b.dtype()=" << mat_b.scalar_type();
  ss << ", scale_b.dtype()=" << scale_b.scalar_type() << ", scale_b.size()=" << scale_b.sizes()
     << " and scale_b.stride()=" << scale_b.strides();
  TORCH_CHECK_VALUE(false, ss.str());
}

bool is_tensorwise(const at::Tensor& t, const at::Tensor& scale) {
  return at::isFloat8Type(t.scalar_type()) && scale.scalar_type() == at::kFloat && scale.numel() == 1;
}

bool is_rowwise(const at::Tensor& t, const at::Tensor& scale) {
  return at::isFloat8Type(t.scalar_type()) && scale.scalar_type() == at::kFloat && scale.dim() == 2 &&
         scale.size(0) == t.size(0) && scale.size(1) == 1 && scale.is_contiguous();
}

at::Tensor& scaled_mm_out(const at::Tensor& mat1, const at::Tensor& mat2, const at::Tensor& scale_a,
                          const at::Tensor& scale_b, const std::optional<at::Tensor>& bias,
                          const std::optional<at::Tensor>& scale_result, std::optional<c10::ScalarType> out_dtype,
                          bool use_fast_accum, at::Tensor& out) {
  const bool has_bias = bias.has_value() && bias->defined();
  const bool has_sr = scale_result.has_value() && scale_result->defined();
  const int fa = vkt_dtype(mat1.scalar_type()), fb = vkt_dtype(mat2.scalar_type());
  const bool fp8_ok = (fa == VKT_E4M3 || fa == VKT_E5M2) && (fb == VKT_E4M3 || fb == VKT_E5M2);
  if (!all_vk({&mat1, &mat2, &out, &scale_a, &scale_b, has_bias ? &*bias : nullptr, has_sr ? &*scale_result : nullptr}) ||
      (at::isFloat8Type(mat1.scalar_type()) && at::isFloat8Type(mat2.scalar_type()) && !fp8_ok) ||
      vkt_dtype(out.scalar_type()) < 0 || (has_bias && (vkt_dtype(bias->scalar_type()) < 0 ||
                                                        vkt_dtype(bias->scalar_type()) > VKT_BF16))) {
    on_cpu("aten::_scaled_mm", "out", mat1, mat2, scale_a, scale_b, bias, scale_result, out_dtype, use_fast_accum, out);
    return out;
  }
  // (ScaledBlas.cpp _scaled_mm_out_cpu's checks, reference quant.cpp:243-277)
  TORCH_CHECK_VALUE(!out_dtype || *out_dtype == out.scalar_type(), "out_dtype must match output matrix type");
  bool tensorwise = false;
  if (is_tensorwise(mat1, scale_a) && is_tensorwise(mat2.t(), scale_b.t())) {
    tensorwise = true;
  } else if (!(is_rowwise(mat1, scale_a) && is_rowwise(mat2.t(), scale_b.t()))) {
    invalid_scaling_config(mat1, mat2, scale_a, scale_b);
  }
  TORCH_CHECK(mat1.dim() == 2, "mat1 must be a matrix");
  TORCH_CHECK(mat2.dim() == 2, "mat2 must be a matrix");
  TORCH_CHECK(mat1.sizes()[1] == mat2.sizes()[0], "mat_a and mat_b shapes cannot be multiplied (", mat1.sizes()[0],
              "x", mat1.sizes()[1], " and ", mat2.sizes()[0], "x", mat2.sizes()[1], ")");
  if (tensorwise) {
    TORCH_CHECK_VALUE(at::isFloat8Type(mat1.scalar_type()) && at::isFloat8Type(mat2.scalar_type()),
                      "mat1 and mat2 must be fp8 types, got: ", mat1.scalar_type(), mat2.scalar_type());
    TORCH_CHECK_VALUE(scale_a.numel() == 1 && scale_a.scalar_type() == at::kFloat, "scale_a must have 1 Float element");
    TORCH_CHECK_VALUE(scale_b.numel() == 1 && scale_b.scalar_type() == at::kFloat, "scale_b must have 1 Float element");
  } else {
    TORCH_CHECK_VALUE(at::isFloat8Type(mat1.scalar_type()) && at::isFloat8Type(mat2.scalar_type()),
                      "mat1 and mat_b must be fp8 types, got: ", mat1.scalar_type(), mat2.scalar_type());
    TORCH_CHECK_VALUE(scale_a.size(0) == mat1.size(0) && scale_a.size(1) == 1, "scale_a must have shape [",
                      mat1.size(0), ", 1], got [", scale_a.sizes(), "]");
    TORCH_CHECK_VALUE(scale_a.numel() == mat1.size(0) && scale_a.scalar_type() == at::kFloat, "scale_a must have ",
                      mat1.size(0), " Float elements, got ", scale_a.numel());
    TORCH_CHECK_VALUE(scale_b.numel() == mat2.size(1) && scale_b.scalar_type() == at::kFloat, "scale_b must have ",
                      mat2.size(1), " Float elements, got ", scale_b.numel());
    TORCH_CHECK_VALUE(scale_a.stride(1) == 1, "expected scale_a.stride(1) to be 1, but got ", scale_a.stride(1));
    TORCH_CHECK_VALUE(scale_b.stride(1) == 1, "expected scale_b.stride(1) to be 1, but got ", scale_b.stride(1));
  }
  TORCH_CHECK(!has_sr || (scale_result->numel() == 1 && scale_result->scalar_type() == at::kFloat),
              "scale_result must be a float scalar");
  TORCH_CHECK(!has_bias || bias->numel() == mat2.sizes()[1], "Bias must be size ", mat2.sizes()[1], " but got ",
              bias->numel());
  TORCH_CHECK(at::isFloat8Type(mat1.scalar_type()), "Expected mat1 to be Float8 matrix got ", mat1.scalar_type());
  TORCH_CHECK(at::isFloat8Type(mat2.scalar_type()), "Expected mat2 to be Float8 matrix got ", mat2.scalar_type());

  const int64_t M = mat1.size(0), K = mat1.size(1), N = mat2.size(1);
  at::native::resize_output(out, {M, N});
  if (out.numel() == 0) return out;
  // The kernel reads A as rows of K and B as columns of K (the layouts the op is used with);
  // other layouts are repacked once.  The output is written densely.
  at::Tensor a = mat1.stride(1) == 1 && mat1.stride(0) >= K ? mat1 : mat1.contiguous();
  at::Tensor bt = mat2.t();  // [N, K]
  if (!(bt.stride(1) == 1 && bt.stride(0) >= K)) bt = bt.contiguous();
  at::Tensor o = out.is_contiguous() ? out : at::empty({M, N}, out.options());
  at::Tensor sa = scale_a.contiguous(), sb = scale_b.contiguous();
  at::Tensor b = has_bias ? bias->contiguous() : at::Tensor();
  TORCH_CHECK(K < (int64_t(1) << 32) && a.stride(0) < (int64_t(1) << 32) && bt.stride(0) < (int64_t(1) << 32) &&
                  M * N < (int64_t(1) << 32),
              "_scaled_mm: too large for 32-bit indexing");
  F8Params p{};
  p.a = gpu_address(a);
  p.b = gpu_address(bt);
  p.scale_a = gpu_address(sa);
  p.scale_b = gpu_address(sb);
  p.bias = has_bias ? gpu_address(b) : 0;
  // (the scale of a float8 result is read on the device: no host synchronisation, unlike
  // the reference's scale_result->item<float>() at quant.cpp:296)
  p.scale_result = has_sr ? gpu_address(*scale_result) : 0;
  p.out = gpu_address_out(o);
  p.m = static_cast<uint32_t>(M);
  p.n = static_cast<uint32_t>(N);
  p.k = static_cast<uint32_t>(K);
  p.lda = static_cast<uint32_t>(M == 1 ? K : a.stride(0));
  p.ldb = static_cast<uint32_t>(N == 1 ? K : bt.stride(0));
  p.ldo = static_cast<uint32_t>(N);
  p.fmt_a = static_cast<uint32_t>(fa);
  p.fmt_b = static_cast<uint32_t>(fb);
  p.out_dtype = static_cast<uint32_t>(vkt_dtype(o.scalar_type()));
  p.bias_dtype = has_bias ? static_cast<uint32_t>(vkt_dtype(b.scalar_type())) : VKT_F32;
  p.rowwise = tensorwise ? 0u : 1u;
  if (K == 0) {
    // an empty product: zeros (+ bias), through the same epilogue, needs one valid k: fall back
    on_cpu("aten::_scaled_mm", "out", mat1, mat2, scale_a, scale_b, bias, scale_result, out_dtype, use_fast_accum, out);
    return out;
  }
  dispatch("fp8mm", {0u}, p, 1);
  if (!o.is_same(out)) out.copy_(o);
  return out;
}

at::Tensor scaled_mm(const at::Tensor& mat_a, const at::Tensor& mat_b, const at::Tensor& scale_a,
                     const at::Tensor& scale_b, const std::optional<at::Tensor>& bias,
                     const std::optional<at::Tensor>& scale_result, std::optional<c10::ScalarType> out_dtype,
                     bool use_fast_accum) {
  const auto out_dtype_ = out_dtype.value_or(mat_a.scalar_type());
  at::Tensor out = at::empty({0}, mat_a.options().dtype(out_dtype_));
  return scaled_mm_out(mat_a, mat_b, scale_a, scale_b, bias, scale_result, out_dtype, use_fast_accum, out);
}

}  // namespace
}  // namespace vk

namespace vk {
namespace {

// vk::fp8_quant_rowwise(x [M,K] float32 / float16 / bfloat16, dtype) -> (q [M,K] float8, scale [M,1]
// float32): the producer in front of _scaled_mm (kernel "fp8_quant"), scale as _scaled_mm
// takes a rowwise scale_a (for mat2 quantise the [N,K] weight and pass q.t(), scale.t()).
// No counterpart in the reference: its float8 tensors come from casts alone.
std::tuple<at::Tensor, at::Tensor> fp8_quant_rowwise(const at::Tensor& x, at::ScalarType dtype) {
  TORCH_CHECK(x.dim() == 2, "fp8_quant_rowwise: expected a 2-D input, got ", x.sizes());
  TORCH_CHECK(dtype == at::kFloat8_e4m3fn || dtype == at::kFloat8_e5m2,
              "fp8_quant_rowwise: dtype must be float8_e4m3fn or float8_e5m2, got ", dtype);
  const int sdt = vkt_dtype(x.scalar_type());
  TORCH_CHECK(sdt >= 0 && sdt <= VKT_BF16, "fp8_quant_rowwise: input must be float32, float16 or bfloat16, got ",
              x.scalar_type());
  TORCH_CHECK(is_vk(x), "fp8_quant_rowwise: input must be on the vk device");
  const int64_t M = x.size(0), K = x.size(1);
  TORCH_CHECK(M < (int64_t(1) << 31) && K < (int64_t(1) << 31), "fp8_quant_rowwise: too large");
  at::Tensor xc = x.contiguous();
  at::Tensor q = at::empty({M, K}, x.options().dtype(dtype));
  at::Tensor scale = at::empty({M, 1}, x.options().dtype(at::kFloat));
  if (M == 0 || K == 0) {
    // (rows without elements: the scale of an all-zero row)
    if (M != 0) scale.fill_(1e-12f / (dtype == at::kFloat8_e4m3fn ? 448.0f : 57344.0f));
    return {q, scale};
  }
  F8QuantParams p{};
  p.src = gpu_address(xc);
  p.dst = gpu_address_out(q);
  p.scale = gpu_address_out(scale);
  p.m = static_cast<uint32_t>(M);
  p.k = static_cast<uint32_t>(K);
  p.lds = p.ldd = static_cast<uint32_t>(K);
  p.src_dtype = static_cast<uint32_t>(sdt);
  p.dst_fmt = static_cast<uint32_t>(vkt_dtype(dtype));
  dispatch("fp8_quant", {1u}, p, static_cast<uint32_t>(M));
  return {q, scale};
}

}  // namespace
}  // namespace vk

TORCH_LIBRARY(vk, m) { m.def("fp8_quant_rowwise(Tensor x, ScalarType dtype) -> (Tensor, Tensor)"); }
TORCH_LIBRARY_IMPL(vk, PrivateUse1, m) { m.impl("fp8_quant_rowwise", &vk::fp8_quant_rowwise); }

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  using namespace vk;
  m.impl("_weight_int8pack_mm", &weight_int8pack_mm);
  m.impl("_dyn_quant_pack_4bit_weight", &dyn_quant_pack_4bit_weight);
  m.impl("_dyn_quant_matmul_4bit", &dyn_quant_matmul_4bit);
  m.impl("_scaled_mm", &scaled_mm);
  m.impl("_scaled_mm.out", &scaled_mm_out);
}
