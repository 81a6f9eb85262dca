// Matrix products of float16 / bfloat16 tensors for device "vk" on MI355X: mm, bmm, addmm and
// baddbmm (the unquantised Linear next to the quantised ops), as the reference registers them
// (crates/pyvk/csrc/linalg.cpp:662-668) with its checks and messages (which are the CPU's),
// queued as "gemmcm_f16" / "gemmcm_bf16" with the reference's parameter block (:25-34, :183-211;
// the float32 alpha / beta of its 16-bit route, :248-249).  Operands keep their strides: the
// library picks the matrix-core tiles or its strided kernel from the block.  Other element types
// run on the CPU, recorded as fallbacks.
#include "vk.h"

#include <ATen/ExpandUtils.h>
#include <ATen/native/Resize.h>
#include <torch/library.h>

#include <cstring>

namespace vk {
namespace {

constexpr int64_t kMaxBatch = 65535;  // matrices per dispatch (grid z), as the reference (:473)

bool fits_i32(const at::Tensor& t) {
  for (int64_t d = 0; d < t.dim(); d++) {
    if (t.stride(d) >= (int64_t(1) << 31) || t.stride(d) < 0 || t.size(d) >= (int64_t(1) << 31)) return false;
  }
  return true;
}

uint64_t f32_bits(double v) {
  float f = static_cast<float>(v);
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}

// c = alpha a @ b (+ beta cin) over 3-D views a [B,M,K], b [B,K,N], c and cin [B,M,N] (cin may
// broadcast through zero strides; read only when beta != 0).  False where no kernel runs it.
bool gemm(const at::Tensor& a_in, const at::Tensor& b_in, const at::Tensor& c, const at::Tensor* cin_in,
          const at::Scalar& alpha, const at::Scalar& beta) {
  at::ScalarType t = c.scalar_type();
  if ((t != at::kHalf && t != at::kBFloat16) || alpha.isComplex() || beta.isComplex()) return false;
  at::Tensor a = a_in.resolve_conj().resolve_neg(), b = b_in.resolve_conj().resolve_neg();
  at::Tensor cin = cin_in != nullptr ? cin_in->resolve_conj().resolve_neg() : at::Tensor();
  if (a.scalar_type() != t || b.scalar_type() != t || (cin.defined() && cin.scalar_type() != t)) return false;
  for (const at::Tensor* x : std::initializer_list<const at::Tensor*>{&a, &b, &c, &cin}) {
    if (x->defined() && (!is_vk(*x) || !fits_i32(*x))) return false;
  }
  if (c.size(0) > kMaxBatch) return false;
  if (c.numel() == 0) return true;
  const bool use_cin = cin.defined() && beta.toDouble() != 0.0;
  GemmParams p{};
  p.a = gpu_address(a);
  p.b = gpu_address(b);
  p.c = gpu_address_out(c);
  p.cin = use_cin ? gpu_address(cin) : 0;
  p.alpha = f32_bits(alpha.toDouble());
  p.beta = f32_bits(beta.toDouble());
  p.m = static_cast<uint32_t>(c.size(1));
  p.n = static_cast<uint32_t>(c.size(2));
  p.k = static_cast<uint32_t>(a.size(2));
  p.a_sb = static_cast<int32_t>(a.stride(0)), p.a_sm = static_cast<int32_t>(a.stride(1)), p.a_sk = static_cast<int32_t>(a.stride(2));
  p.b_sb = static_cast<int32_t>(b.stride(0)), p.b_sk = static_cast<int32_t>(b.stride(1)), p.b_sn = static_cast<int32_t>(b.stride(2));
  p.c_sb = static_cast<int32_t>(c.stride(0)), p.c_sm = static_cast<int32_t>(c.stride(1)), p.c_sn = static_cast<int32_t>(c.stride(2));
  if (use_cin) {
    p.cin_sb = static_cast<int32_t>(cin.stride(0)), p.cin_sm = static_cast<int32_t>(cin.stride(1));
    p.cin_sn = static_cast<int32_t>(cin.stride(2));
  }
  dispatch(t == at::kHalf ? "gemmcm_f16" : "gemmcm_bf16", {use_cin ? 1u : 0u}, p, 1, 1, static_cast<uint32_t>(c.size(0)));
  return true;
}

at::Tensor& mm_out(const at::Tensor& self, const at::Tensor& mat2, at::Tensor& out) {
  TORCH_CHECK(self.dim() == 2 && mat2.dim() == 2, "self must be a matrix");
  TORCH_CHECK(self.size(1) == mat2.size(0), "mat1 and mat2 shapes cannot be multiplied (", self.size(0), "x", self.size(1),
              " and ", mat2.size(0), "x", mat2.size(1), ")");
  at::native::resize_output(out, {self.size(0), mat2.size(1)});
  TORCH_CHECK(out.dtype() == self.dtype(), "Expected out tensor to have dtype ", self.dtype(), ", but got ", out.dtype(),
              " instead");
  TORCH_CHECK(self.dtype() == mat2.dtype(), "expected m1 and m2 to have the same dtype, but got: ", self.dtype(),
              " != ", mat2.dtype());  // (the CPU's checks, reference linalg.cpp:440-443)
  if (!gemm(self.unsqueeze(0), mat2.unsqueeze(0), out.unsqueeze(0), nullptr, 1, 0)) {
    on_cpu("aten::mm", "out", self, mat2, out);
  }
  return out;
}

at::Tensor mm(const at::Tensor& self, const at::Tensor& mat2) {
  TORCH_CHECK(self.dim() == 2 && mat2.dim() == 2, "self must be a matrix");
  at::Tensor out = at::empty({self.size(0), mat2.size(1)}, self.options());
  return mm_out(self, mat2, out);
}

at::Tensor& bmm_out(const at::Tensor& self, const at::Tensor& mat2, at::Tensor& out) {
  TORCH_CHECK(self.dim() == 3 && mat2.dim() == 3, "batch1 must be a 3D tensor");
  TORCH_CHECK(self.size(0) == mat2.size(0) && self.size(2) == mat2.size(1), "Expected size for first two dimensions of batch2 tensor to be: [",
              self.size(0), ", ", self.size(2), "] but got: [", mat2.size(0), ", ", mat2.size(1), "].");
  at::native::resize_output(out, {self.size(0), self.size(1), mat2.size(2)});
  bool ok = false;
  if (self.size(0) > kMaxBatch && out.scalar_type() == self.scalar_type()) {
    ok = true;  // (more matrices than one dispatch takes: in chunks, reference :473-486)
    for (int64_t s = 0; s < self.size(0) && ok; s += kMaxBatch) {
      int64_t len = std::min(kMaxBatch, self.size(0) - s);
      ok = gemm(self.narrow(0, s, len), mat2.narrow(0, s, len), out.narrow(0, s, len), nullptr, 1, 0);
    }
  }
  if (!ok && !gemm(self, mat2, out, nullptr, 1, 0)) {
    on_cpu("aten::bmm", "out", self, mat2, out);
  }
  return out;
}

at::Tensor bmm(const at::Tensor& self, const at::Tensor& mat2) {
  TORCH_CHECK(self.dim() == 3 && mat2.dim() == 3, "batch1 must be a 3D tensor");
  at::Tensor out = at::empty({self.size(0), self.size(1), mat2.size(2)}, self.options());
  return bmm_out(self, mat2, out);
}

at::Tensor& addmm_out(const at::Tensor& self, const at::Tensor& mat1, const at::Tensor& mat2, const at::Scalar& beta,
                      const at::Scalar& alpha, at::Tensor& out) {
  TORCH_CHECK(mat1.dim() == 2 && mat2.dim() == 2, "mat1 must be a matrix, got ", mat1.dim(), "-D tensor");
  TORCH_CHECK(mat1.size(1) == mat2.size(0), "mat1 and mat2 shapes cannot be multiplied (", mat1.size(0), "x", mat1.size(1),
              " and ", mat2.size(0), "x", mat2.size(1), ")");
  int64_t m = mat1.size(0), n = mat2.size(1);
  at::native::resize_output(out, {m, n});
  TORCH_CHECK(out.dtype() == self.dtype(), "Expected out tensor to have dtype ", self.dtype(), ", but got ", out.dtype(),
              " instead");  // (the CPU's check, reference :497-498)
  bool done = false;
  if (is_vk(self)) {
    at::Tensor cin = self.expand({m, n}).unsqueeze(0);  // (more than 2 dims: expand's error, as the CPU's)
    done = gemm(mat1.unsqueeze(0), mat2.unsqueeze(0), out.unsqueeze(0), &cin, alpha, beta);
  }
  if (!done) {
    on_cpu("aten::addmm", "out", self, mat1, mat2, beta, alpha, out);
  }
  return out;
}

at::Tensor addmm(const at::Tensor& self, const at::Tensor& mat1, const at::Tensor& mat2, const at::Scalar& beta,
                 const at::Scalar& alpha) {
  TORCH_CHECK(mat1.dim() == 2 && mat2.dim() == 2, "mat1 must be a matrix, got ", mat1.dim(), "-D tensor");
  at::Tensor out = at::empty({mat1.size(0), mat2.size(1)}, self.options());
  return addmm_out(self, mat1, mat2, beta, alpha, out);
}

at::Tensor& baddbmm_out(const at::Tensor& self, const at::Tensor& batch1, const at::Tensor& batch2, const at::Scalar& beta,
                        const at::Scalar& alpha, at::Tensor& out) {
  TORCH_CHECK(batch1.dim() == 3 && batch2.dim() == 3, "batch1 must be a 3D tensor");
  TORCH_CHECK(batch1.size(0) == batch2.size(0) && batch1.size(2) == batch2.size(1),
              "Expected size for first two dimensions of batch2 tensor to be: [", batch1.size(0), ", ", batch1.size(2),
              "] but got: [", batch2.size(0), ", ", batch2.size(1), "].");
  std::vector<int64_t> shape = {batch1.size(0), batch1.size(1), batch2.size(2)};
  at::native::resize_output(out, shape);
  bool done = false;
  if (self.dim() <= 3 && is_vk(self)) {
    at::Tensor cin = self.expand(shape);
    done = gemm(batch1, batch2, out, &cin, alpha, beta);
  }
  if (!done) {
    on_cpu("aten::baddbmm", "out", self, batch1, batch2, beta, alpha, out);
  }
  return out;
}

at::Tensor baddbmm(const at::Tensor& self, const at::Tensor& batch1, const at::Tensor& batch2, const at::Scalar& beta,
                   const at::Scalar& alpha) {
  TORCH_CHECK(batch1.dim() == 3 && batch2.dim() == 3, "batch1 must be a 3D tensor");
  at::Tensor out = at::empty({batch1.size(0), batch1.size(1), batch2.size(2)}, self.options());
  return baddbmm_out(self, batch1, batch2, beta, alpha, out);
}

}  // namespace
}  // namespace vk

TORCH_LIBRARY_IMPL(aten, PrivateUse1, m) {
  using namespace vk;
  m.impl("mm", &vk::mm);
  m.impl("mm.out", &mm_out);
  m.impl("bmm", &vk::bmm);
  m.impl("bmm.out", &bmm_out);
  m.impl("addmm", &vk::addmm);
  m.impl("addmm.out", &addmm_out);
  m.impl("baddbmm", &vk::baddbmm);
  m.impl("baddbmm.out", &baddbmm_out);
}
