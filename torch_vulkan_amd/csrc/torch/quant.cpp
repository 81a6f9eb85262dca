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
#include <atomic>
#include <mutex>
#include <sstream>
#include <unordered_map>

namespace vk {
namespace {

// ------------------------------------------------------------ shared pieces

// "<family>_<f32|f16|bf16>" for a float element type the kernels of `family` are built for, else "".
std::string float_kernel(const char* family, at::ScalarType t) {
  const int code = vkt_dtype(t);
  if (code < VKT_F32 || code > VKT_BF16) return std::string();
  static const char* const suffix[] = {"f32", "f16", "bf16"};
  return std::string(family) + "_" + suffix[code];
}

// Whether every tensor given (absent optionals aside) lives on the device.
inline bool resident(const at::Tensor& t) { return !t.defined() || is_vk(t); }
inline bool resident(const std::optional<at::Tensor>& t) { return !t.has_value() || resident(*t); }
template <class First, class... Rest>
bool resident(const First& first, const Rest&... rest) {
  return resident(first) && resident(rest...);
}

inline bool present(const std::optional<at::Tensor>& t) { return t.has_value() && t->defined(); }

constexpr int64_t kIndexLimit = int64_t(1) << 32;  // the kernels index with 32 bits
constexpr int64_t kRowsPerDispatch = 65535;        // of the int4 kernels (the reference's grid limit, quant.cpp:29)

// f(first_row, rows) over [0, rows_total) in pieces the int4 kernels take in one dispatch.
template <class F>
void in_row_pieces(int64_t rows_total, F&& f) {
  for (int64_t first = 0; first < rows_total; first += kRowsPerDispatch) f(first, std::min(rows_total - first, kRowsPerDispatch));
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

  const std::string kernel = float_kernel("qmm8", A.scalar_type());
  const bool indexable = A.stride(0) < (int64_t(1) << 31) && B.numel() < kIndexLimit && M * N < kIndexLimit;
  if (kernel.empty() || !indexable || !resident(A, B, scales))
    return on_cpu("aten::_weight_int8pack_mm", "", A, B, scales)[0].toTensor();

  at::Tensor C = at::empty({M, N}, A.options());
  if (C.numel() == 0) return C;
  const at::Tensor s = scales.to(A.scalar_type()).contiguous();  // the kernels read scales in A's type, as the CPU does
  Q8Params p{};
  p.a = gpu_address(A), p.b = gpu_address(B), p.scales = gpu_address(s), p.c = gpu_address_out(C);
  p.m = static_cast<uint32_t>(M), p.n = static_cast<uint32_t>(N), p.k = static_cast<uint32_t>(K);
  p.a_sm = static_cast<int32_t>(A.stride(0)), p.a_sk = 1;
  // spec[0] mirrors the reference's ROWS constant (M on its GEMV path, 0 on its tile path); the library plans
  // the launch from the block and only checks it for consistency
  dispatch(kernel, {M <= 8 ? static_cast<uint32_t>(M) : 0u}, p, 1);
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
  const bool with_bias = present(bias);
  const int scale_code = vkt_dtype(scales_zeros.scalar_type());
  const int bias_code = with_bias ? vkt_dtype(bias->scalar_type()) : VKT_F32;
  const int64_t total = weights.numel() + scales_zeros.numel() + (with_bias ? bias->numel() : 0);
  const auto float_code = [](int c) { return c >= VKT_F32 && c <= VKT_BF16; };
  if (!float_code(scale_code) || !float_code(bias_code) || total >= kIndexLimit || !resident(weights, scales_zeros, bias))
    return on_cpu("aten::_dyn_quant_pack_4bit_weight", "", weights, scales_zeros, bias, block_size, in_features, out_features)[0]
        .toTensor();

  // the CPU's layout (reference quant.cpp:123-144): [bytes | scales | bias], every element widened to float32
  const at::Tensor w = weights.contiguous(), s = scales_zeros.contiguous();
  const at::Tensor b = with_bias ? bias->contiguous() : at::Tensor();
  at::Tensor vec = at::empty({total}, weights.options().dtype(at::kFloat));
  if (total == 0) return vec;
  Q4VecParams p{};
  p.weights = gpu_address(w), p.scales = gpu_address(s), p.bias = with_bias ? gpu_address(b) : 0, p.out = gpu_address_out(vec);
  p.nw = static_cast<uint32_t>(w.numel()), p.ns = static_cast<uint32_t>(s.numel());
  p.nb = with_bias ? static_cast<uint32_t>(b.numel()) : 0;
  p.scales_dtype = static_cast<uint32_t>(scale_code), p.bias_dtype = static_cast<uint32_t>(bias_code);
  dispatch("qmm4_packvec", {}, p, 1);
  return vec;
}

// Compact side-cars of packed weight vectors.  The packed tensor the op receives is the CPU's float32 vector
// (4 bytes per byte of nibbles); the kernels stream a compact rewrite of it, built once per packed tensor and
// kernel layout (0: the streaming kernel, up to 3 rows; 1: the matrix cores) and kept for as long as the packed
// tensor's storage lives.  A hash map from (storage, view, shape, layout) to the side-car; an entry is stale when
// the storage has died or the tensor has been written since (version counter).  The map is unbounded: a side-car
// is 0.3x the bytes of the vector it belongs to, and it goes when that vector's storage goes (dead entries are
// swept every kSweepEvery insertions and by sidecar_clear).
struct SideCarKey {
  const c10::StorageImpl* storage;
  const void* data;
  int64_t offset, numel, bs, k, n;
  uint32_t layout;
  bool operator==(const SideCarKey& o) const {
    return storage == o.storage && data == o.data && offset == o.offset && numel == o.numel && bs == o.bs && k == o.k && n == o.n &&
           layout == o.layout;
  }
};
struct SideCarKeyHash {
  size_t operator()(const SideCarKey& key) const {
    uint64_t h = 0x9e3779b97f4a7c15ull;
    for (uint64_t v : {reinterpret_cast<uint64_t>(key.storage), reinterpret_cast<uint64_t>(key.data), uint64_t(key.offset), uint64_t(key.numel),
                       uint64_t(key.bs), uint64_t(key.k), uint64_t(key.n), uint64_t(key.layout)})
      h = (h ^ v) * 0x100000001b3ull + (h >> 29);
    return size_t(h);
  }
};
struct SideCarEntry {
  c10::weak_intrusive_ptr<c10::StorageImpl> owner;
  int64_t version;
  bool inference;  // built from an inference tensor: no version counter tells it stale, vk::note_write drops it
  at::Tensor compact;
};
constexpr size_t kSweepEvery = 64;
std::mutex g_sidecar_mutex;
std::unordered_map<SideCarKey, SideCarEntry, SideCarKeyHash> g_sidecars;
size_t g_sidecar_inserts = 0;
std::atomic<size_t> g_inference_sidecars{0};  // entries with `inference` set (read without the mutex by note_write)

// The version that tells whether a tensor was written to since its side-car was built.  Inference tensors carry
// no counter: in-place writes under torch.inference_mode() are legal and bump nothing, so their entries are dropped
// by the write paths of the op layer instead (sidecars_note_write).
int64_t write_version(const at::Tensor& t) { return t.is_inference() ? 0 : static_cast<int64_t>(t._version()); }

std::unordered_map<SideCarKey, SideCarEntry, SideCarKeyHash>::iterator erase_sidecar_locked(
    std::unordered_map<SideCarKey, SideCarEntry, SideCarKeyHash>::iterator it) {
  if (it->second.inference) g_inference_sidecars.fetch_sub(1, std::memory_order_relaxed);
  return g_sidecars.erase(it);
}

void sweep_sidecars_locked() {
  for (auto it = g_sidecars.begin(); it != g_sidecars.end();) it = it->second.owner.expired() ? erase_sidecar_locked(it) : std::next(it);
}

at::Tensor sidecar_for(const at::Tensor& packed, int64_t bs, int64_t K, int64_t N, bool with_bias, uint32_t layout) {
  const uint64_t bytes = vkt_qmm4c_bytes(static_cast<uint32_t>(N), static_cast<uint32_t>(K), static_cast<uint32_t>(bs));
  if (bytes == 0) return at::Tensor();  // (block sizes without a compact form)
  const SideCarKey key{packed.storage().unsafeGetStorageImpl(), packed.const_data_ptr(), packed.storage_offset(), packed.numel(), bs, K, N, layout};
  const int64_t version = write_version(packed);
  std::lock_guard<std::mutex> lock(g_sidecar_mutex);
  const auto found = g_sidecars.find(key);
  if (found != g_sidecars.end() && !found->second.owner.expired() && found->second.version == version) return found->second.compact;

  at::Tensor compact = at::empty({static_cast<int64_t>(bytes)}, packed.options().dtype(at::kByte));
  Q4PackParams p{};
  // (the new tensor's address directly: gpu_address_out would report a write to the cache, whose mutex is held here)
  p.packed = gpu_address(packed), p.compact = reinterpret_cast<uint64_t>(compact.mutable_data_ptr());
  p.n = static_cast<uint32_t>(N), p.k = static_cast<uint32_t>(K), p.bs = static_cast<uint32_t>(bs), p.has_bias = with_bias ? 1u : 0u;
  dispatch("qmm4c_pack", {layout}, p, 1);
  if (++g_sidecar_inserts % kSweepEvery == 0) sweep_sidecars_locked();
  if (const auto stale = g_sidecars.find(key); stale != g_sidecars.end()) erase_sidecar_locked(stale);  // (an older version's entry)
  const bool inference = packed.is_inference();
  if (inference) g_inference_sidecars.fetch_add(1, std::memory_order_relaxed);
  g_sidecars.insert_or_assign(key, SideCarEntry{c10::weak_intrusive_ptr<c10::StorageImpl>(packed.storage().getWeakStorageImpl()), version, inference, compact});
  return compact;
}

// A write into an inference tensor: the side-cars built from its storage go (the next product rebuilds them).
void sidecars_note_write(const at::TensorBase& t) {
  if (g_inference_sidecars.load(std::memory_order_relaxed) == 0 || !t.is_inference() || !t.has_storage()) return;
  const c10::StorageImpl* storage = t.storage().unsafeGetStorageImpl();
  std::lock_guard<std::mutex> lock(g_sidecar_mutex);
  for (auto it = g_sidecars.begin(); it != g_sidecars.end();) it = it->first.storage == storage ? erase_sidecar_locked(it) : std::next(it);
}

// (entries, bytes) of the side-car cache after dropping dead entries; clear = true empties it.
std::tuple<int64_t, int64_t> sidecar_cache(bool clear) {
  std::lock_guard<std::mutex> lock(g_sidecar_mutex);
  if (clear) {
    g_sidecars.clear();
    g_inference_sidecars.store(0, std::memory_order_relaxed);
  }
  sweep_sidecars_locked();
  int64_t bytes = 0;
  for (const auto& kv : g_sidecars) bytes += kv.second.compact.numel();
  return {static_cast<int64_t>(g_sidecars.size()), bytes};
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
  const int64_t M = inp.size(0), N = out_features, K = in_features;
  const std::string family = float_kernel("", inp.scalar_type());  // "_f32" | "_bf16"
  const bool indexable = M * std::max(K, N) < (int64_t(1) << 31) && packed_weights.numel() < (int64_t(1) << 31);
  if (family.empty() || !indexable || !resident(inp, packed_weights))
    return on_cpu("aten::_dyn_quant_matmul_4bit", "", inp, packed_weights, block_size, in_features, out_features)[0].toTensor();

  at::Tensor output = at::empty({M, N}, inp.options());
  const int64_t weights_elements = N * K / 2;
  const int64_t scale_elements = N * (K / block_size);
  TORCH_CHECK(packed_weights.numel() >= (weights_elements + scale_elements), "Invalid packed weight tensor size");
  int64_t bias_elements = packed_weights.numel() - (weights_elements + scale_elements);
  if (bias_elements) {
    TORCH_CHECK(bias_elements == N, "Expected bias length to match output dimension");
  }
  if (output.numel() == 0) return output;

  const at::Tensor x = inp.contiguous();
  const at::Tensor packed = packed_weights.to(at::kFloat).contiguous();
  const uint32_t groupwise = block_size != K ? 1u : 0u, with_bias = bias_elements != 0 ? 1u : 0u;
  const int64_t item = x.element_size();
  const uint64_t x_at = gpu_address(x), out_at = gpu_address_out(output);
  // what both parameter blocks share: shapes, and the addresses of a piece of rows
  auto fill_piece = [&](auto& p, int64_t first, int64_t rows) {
    p.inp = x_at + static_cast<uint64_t>(first * K * item);
    p.out = out_at + static_cast<uint64_t>(first * N * item);
    p.m = static_cast<uint32_t>(rows), p.n = static_cast<uint32_t>(N), p.k = static_cast<uint32_t>(K);
    p.bs = static_cast<uint32_t>(block_size), p.has_bias = with_bias;
  };

  // up to 3 rows stream the side-car through the vector units; more go to the matrix cores (measured at
  // K = 4096, N = 11008: 4 rows take 19.0 us streaming, 15.3 on the matrix cores)
  const uint32_t layout = M > 3 ? 1u : 0u;
  const at::Tensor compact = sidecar_for(packed, block_size, K, N, with_bias != 0, layout);
  if (compact.defined()) {
    in_row_pieces(M, [&](int64_t first, int64_t rows) {
      // activation scratch of this piece (quantised rows, and per row 1/scale and -zero_point)
      at::Tensor q = at::empty({static_cast<int64_t>(vkt_qmm4c_q_bytes(static_cast<uint32_t>(rows), static_cast<uint32_t>(K)))},
                               inp.options().dtype(at::kByte));
      at::Tensor row_params = at::empty({rows, 2}, inp.options().dtype(at::kFloat));
      Q4CParams p{};
      fill_piece(p, first, rows);
      p.q = gpu_address_out(q), p.rows = gpu_address_out(row_params), p.compact = gpu_address(compact);
      dispatch("qmm4c" + family, {2u, groupwise, layout}, p, 1);  // phase 2: row quantisation + product
    });
    return output;
  }
  // a block size without a compact form: the reference's own buffers and its two launches (quant.cpp:178-202)
  at::Tensor q = at::empty({M, K}, inp.options().dtype(at::kInt));
  at::Tensor row_params = at::empty({M, 2}, inp.options().dtype(at::kFloat));
  const uint64_t q_at = gpu_address_out(q), rows_at = gpu_address_out(row_params), packed_at = gpu_address(packed);
  in_row_pieces(M, [&](int64_t first, int64_t rows) {
    Q4Params p{};
    fill_piece(p, first, rows);
    p.q = q_at + static_cast<uint64_t>(first * K * 4), p.rows = rows_at + static_cast<uint64_t>(first * 8), p.packed = packed_at;
    dispatch("qmm4" + family, {0u, groupwise}, p, static_cast<uint32_t>(rows));
    dispatch("qmm4" + family, {1u, groupwise}, p, static_cast<uint32_t>((N + 31) / 32), static_cast<uint32_t>((rows + 7) / 8));
  });
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

// How the scales of a _scaled_mm call apply (ScaledBlas.cpp's two accepted forms; reference quant.cpp:225-249).
// Both operands are judged the same way, mat2 and scale_b through their transposes: one float32 scale per tensor,
// or a contiguous [rows, 1] float32 column of them.
enum class Scaling { kPerTensor, kPerRow, kInvalid };
Scaling scaling_of(const at::Tensor& mat1, const at::Tensor& mat2, const at::Tensor& scale_a, const at::Tensor& scale_b) {
  struct Fit {
    bool single, column;
  };
  const auto judge = [](const at::Tensor& t, const at::Tensor& scale) {
    if (!at::isFloat8Type(t.scalar_type()) || scale.scalar_type() != at::kFloat) return Fit{false, false};
    return Fit{scale.numel() == 1,
               scale.dim() == 2 && scale.size(0) == t.size(0) && scale.size(1) == 1 && scale.is_contiguous()};
  };
  const Fit a = judge(mat1, scale_a), b = judge(mat2.t(), scale_b.t());
  // (a [1, 1] scale fits both forms; one scale per tensor is tried first, as on the CPU)
  return a.single && b.single ? Scaling::kPerTensor : a.column && b.column ? Scaling::kPerRow : Scaling::kInvalid;
}

at::Tensor& scaled_mm_out(const at::Tensor& mat1, const at::Tensor& mat2, const at::Tensor& scale_a,
                          const at::Tensor& scale_b, const std::optional<at::Tensor>& bias,
                          const std::optional<at::Tensor>& scale_result, std::optional<c10::ScalarType> out_dtype,
                          bool use_fast_accum, at::Tensor& out) {
  const bool with_bias = present(bias), with_result_scale = present(scale_result);
  const int fmt_a = vkt_dtype(mat1.scalar_type()), fmt_b = vkt_dtype(mat2.scalar_type());
  const auto fp8_code = [](int c) { return c == VKT_E4M3 || c == VKT_E5M2; };
  // float8 formats without a kernel (the fnuz ones), outputs or biases of other types, or host tensors: the CPU's op
  const bool other_fp8 = at::isFloat8Type(mat1.scalar_type()) && at::isFloat8Type(mat2.scalar_type()) && !(fp8_code(fmt_a) && fp8_code(fmt_b));
  const bool bias_ok = !with_bias || (vkt_dtype(bias->scalar_type()) >= VKT_F32 && vkt_dtype(bias->scalar_type()) <= VKT_BF16);
  if (other_fp8 || vkt_dtype(out.scalar_type()) < 0 || !bias_ok || !resident(mat1, mat2, out, scale_a, scale_b, bias, scale_result)) {
    on_cpu("aten::_scaled_mm", "out", mat1, mat2, scale_a, scale_b, bias, scale_result, out_dtype, use_fast_accum, out);
    return out;
  }
  // (ScaledBlas.cpp _scaled_mm_out_cpu's checks, reference quant.cpp:243-277)
  TORCH_CHECK_VALUE(!out_dtype || *out_dtype == out.scalar_type(), "out_dtype must match output matrix type");
  const Scaling scaling = scaling_of(mat1, mat2, scale_a, scale_b);
  if (scaling == Scaling::kInvalid) invalid_scaling_config(mat1, mat2, scale_a, scale_b);
  TORCH_CHECK(mat1.dim() == 2, "mat1 must be a matrix");
  TORCH_CHECK(mat2.dim() == 2, "mat2 must be a matrix");
  TORCH_CHECK(mat1.sizes()[1] == mat2.sizes()[0], "mat_a and mat_b shapes cannot be multiplied (", mat1.sizes()[0],
              "x", mat1.sizes()[1], " and ", mat2.sizes()[0], "x", mat2.sizes()[1], ")");
  if (scaling == Scaling::kPerTensor) {
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
  TORCH_CHECK(!with_result_scale || (scale_result->numel() == 1 && scale_result->scalar_type() == at::kFloat),
              "scale_result must be a float scalar");
  TORCH_CHECK(!with_bias || bias->numel() == mat2.sizes()[1], "Bias must be size ", mat2.sizes()[1], " but got ",
              bias->numel());
  TORCH_CHECK(at::isFloat8Type(mat1.scalar_type()), "Expected mat1 to be Float8 matrix got ", mat1.scalar_type());
  TORCH_CHECK(at::isFloat8Type(mat2.scalar_type()), "Expected mat2 to be Float8 matrix got ", mat2.scalar_type());

  const int64_t M = mat1.size(0), K = mat1.size(1), N = mat2.size(1);
  at::native::resize_output(out, {M, N});
  if (out.numel() == 0) return out;
  // The kernel takes both operands as rows of K bytes (A row-major, mat2 column-major: the layouts the op is
  // used with) and writes a dense output; anything else is repacked once.
  const auto rows_of_k = [K](const at::Tensor& t) { return t.stride(1) == 1 && t.stride(0) >= K; };
  const at::Tensor a = rows_of_k(mat1) ? mat1 : mat1.contiguous();
  const at::Tensor mat2_t = mat2.t();  // [N, K]
  const at::Tensor b = rows_of_k(mat2_t) ? mat2_t : mat2_t.contiguous();
  at::Tensor dense_out = out.is_contiguous() ? out : at::empty({M, N}, out.options());
  const at::Tensor sa = scale_a.contiguous(), sb = scale_b.contiguous();
  const at::Tensor bias_c = with_bias ? bias->contiguous() : at::Tensor();
  TORCH_CHECK(K < kIndexLimit && a.stride(0) < kIndexLimit && b.stride(0) < kIndexLimit && M * N < kIndexLimit,
              "_scaled_mm: too large for 32-bit indexing");
  // The result's scale applies when a float8 output was asked for by out_dtype (absent: bfloat16), as on the CPU
  // and in the reference (quant.cpp:293-297): the functional form without out_dtype returns float8 unscaled.
  const bool scale_the_result = with_result_scale && at::isFloat8Type(out_dtype.value_or(at::kBFloat16));
  F8Params p{};
  p.a = gpu_address(a), p.b = gpu_address(b), p.scale_a = gpu_address(sa), p.scale_b = gpu_address(sb);
  p.bias = with_bias ? gpu_address(bias_c) : 0;
  // (read on the device: no host synchronisation, unlike the reference's scale_result->item<float>())
  p.scale_result = scale_the_result ? gpu_address(*scale_result) : 0;
  p.out = gpu_address_out(dense_out);
  p.m = static_cast<uint32_t>(M), p.n = static_cast<uint32_t>(N), p.k = static_cast<uint32_t>(K);
  // (K == 0: the operands are empty, the product is zeros + bias through the same epilogue)
  p.lda = static_cast<uint32_t>(M == 1 || K == 0 ? K : a.stride(0));
  p.ldb = static_cast<uint32_t>(N == 1 || K == 0 ? K : b.stride(0));
  p.ldo = static_cast<uint32_t>(N);
  p.fmt_a = static_cast<uint32_t>(fmt_a), p.fmt_b = static_cast<uint32_t>(fmt_b);
  p.out_dtype = static_cast<uint32_t>(vkt_dtype(dense_out.scalar_type()));
  p.bias_dtype = with_bias ? static_cast<uint32_t>(vkt_dtype(bias_c.scalar_type())) : VKT_F32;
  p.rowwise = scaling == Scaling::kPerRow ? 1u : 0u;
  dispatch("fp8mm", {0u}, p, 1);
  if (!dense_out.is_same(out)) out.copy_(dense_out);
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

void note_write(const at::TensorBase& t) { sidecars_note_write(t); }

}  // namespace vk

TORCH_LIBRARY(vk, m) {
  m.def("fp8_quant_rowwise(Tensor x, ScalarType dtype) -> (Tensor, Tensor)");
  // the int4 side-car cache: (live entries, bytes they hold); clear = True drops them all first
  m.def("sidecar_cache(bool clear=False) -> (int, int)", &vk::sidecar_cache);
}
TORCH_LIBRARY_IMPL(vk, PrivateUse1, m) { m.impl("fp8_quant_rowwise", &vk::fp8_quant_rowwise); }

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  using namespace vk;
  m.impl("_weight_int8pack_mm", &weight_int8pack_mm);
  m.impl("_dyn_quant_pack_4bit_weight", &dyn_quant_pack_4bit_weight);
  m.impl("_dyn_quant_matmul_4bit", &dyn_quant_matmul_4bit);
  m.impl("_scaled_mm", &scaled_mm);
  m.impl("_scaled_mm.out", &scaled_mm_out);
}
