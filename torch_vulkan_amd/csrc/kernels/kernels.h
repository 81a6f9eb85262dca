// Launchers of the gfx950 kernels.  Each validates what its kernels assume about
// shapes, strides and alignment before launching (a wrong launch is a GPU fault, not an
// error code), queues its kernels on `stream` and returns 0, or sets *err and returns -1.
#pragma once

#include <hip/hip_runtime.h>

#include <string>

#include "../../../include/vkt.h"

namespace vkt {

struct Machine {
  int compute_units = 256;
  // device memory the runtime owns for kernels that split one product over several
  // workgroups: partial results between a kernel and the one that adds them up
  uint64_t workspace = 0, workspace_bytes = 0;
  // the workspace cannot be traded for a different plan: a product whose planned split needs more of it than
  // workspace_bytes is an error, not a product with fewer slices (the no-allocation entry point)
  bool workspace_fixed = false;
  // a second region that the runtime grows on demand, for whole operands rewritten before a product
  // (the int8 weights of a many-row product widened to 16 bits); queued uses are ordered by the one stream
  uint64_t scratch = 0, scratch_bytes = 0;
};

// _weight_int8pack_mm with at least kQ8GemmRows rows of 16-bit activations runs as one tile-kernel product over
// weights widened into the scratch region: the bytes of scratch it needs (0: not this path), and the launch.
constexpr uint32_t kQ8GemmRows = 192;
uint64_t q8_gemm_scratch_bytes(const Q8Params& p, int dtype, const Machine& mc);
int launch_q8_gemm(const Q8Params& p, int dtype, const Machine& mc, hipStream_t stream, std::string* err);

// spec[1] of the qmm8 kernels: 0 = planned by the library; otherwise an explicit
// variant id (COLS | KSPLIT << 8 | FORCE_GENERIC << 16) used by tuning sweeps.
int launch_qmm8(const Q8Params& p, int dtype, uint32_t variant, const Machine& mc, hipStream_t stream,
                std::string* err);
int launch_qmm4(const Q4Params& p, int dtype, uint32_t phase, uint32_t groupwise, const Machine& mc,
                hipStream_t stream, std::string* err);
int launch_qmm4_packvec(const Q4VecParams& p, hipStream_t stream, std::string* err);
int launch_qmm4c_pack(const Q4PackParams& p, uint32_t layout, const Machine& mc, hipStream_t stream, std::string* err);
int launch_qmm4c(const Q4CParams& p, int dtype, uint32_t phase, uint32_t groupwise, uint32_t layout,
                 const Machine& mc, hipStream_t stream, std::string* err);
int launch_fp8mm(const F8Params& p, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err);
int launch_gemm16(const GemmParams& p, int dtype, uint32_t use_cin, uint32_t batch, uint32_t variant, const Machine& mc,
                  hipStream_t stream, std::string* err);
int launch_cast_fp8(const CastParams& p, const Machine& mc, hipStream_t stream, std::string* err);
int launch_cast_strided(const StridedParams& s, int src_dtype, int dst_dtype, const Machine& mc, hipStream_t stream,
                        std::string* err);
// "move_<size_label>" (op: VKT_MOVE_COPY | VKT_MOVE_FILL) and "copy8_<size_label>"; variant 0 plans the
// form from the strides, 1 moves element by element as given, 2 widens units but never tiles.
int launch_move(const StridedParams& s, const char* size_label, uint32_t op, uint32_t variant, const Machine& mc,
                hipStream_t stream, std::string* err);
int launch_copy8(const Copy8Params& c, const char* size_label, uint32_t variant, const Machine& mc, hipStream_t stream,
                 std::string* err);
int launch_quantize_affine(const QuantParams& p, uint32_t qtype, bool dequantize, const Machine& mc, hipStream_t stream,
                           std::string* err);
int launch_aminmax(const MinMaxParams& p, const Machine& mc, hipStream_t stream, std::string* err);
int launch_fake_quant(const QuantParams& p, uint32_t per_channel, uint32_t zp_float, const Machine& mc, hipStream_t stream,
                      std::string* err);
int launch_fp8_quant(const F8QuantParams& p, uint32_t rowwise, const Machine& mc, hipStream_t stream, std::string* err);
int launch_probe_read(const ProbeParams& p, uint32_t geometry, const Machine& mc, hipStream_t stream, std::string* err);
int launch_probe_mfma(const ProbeParams& p, uint32_t operands, const Machine& mc, hipStream_t stream, std::string* err);
int launch_probe_delay(const ProbeParams& p, hipStream_t stream, std::string* err);
int launch_fill(uint64_t dst, uint8_t value, uint64_t nbytes, hipStream_t stream, std::string* err);
int launch_copy(uint64_t dst, uint64_t src, uint64_t nbytes, hipStream_t stream, std::string* err);

uint64_t qmm4c_bytes(uint32_t n, uint32_t k, uint32_t bs);
uint64_t qmm4c_q_bytes(uint32_t m, uint32_t k);

}  // namespace vkt
