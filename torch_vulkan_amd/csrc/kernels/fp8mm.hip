// aten::_scaled_mm on gfx950 as one fused kernel:
//   out[m,n] = cast( (sum_k f32(A[m,k]) * f32(B[k,n])) * scale_a[m|0] * scale_b[n|0] + bias[n] ) [* 1/scale_result]
// for float8 (e4m3fn / e5m2, any mix) A [M,K] row-major and B [K,N] column-major (stored as
// [N,K] rows), float32 scales per tensor or per row / column.  It replaces the reference's
// composite (crates/pyvk/csrc/quant.cpp:279-300: two table-gather upcasts, two multiplies, a
// float32 GEMM on shader cores, bias add, cast, copy: seven passes over full-size float32
// temporaries) with the product on the fp8 matrix cores and everything else in the epilogue.
// Products of two float8 values are exact in float32.  The matrix core, however, adds the
// 128 products of one instruction in a fixed-point window: each product is aligned to the
// largest exponent of its group and bits more than ~14 below it are dropped (measured on
// gfx950: 448*1 + 0.0625*1 is kept, 448*1 + 0.0156*1 loses the small term; the accumulator
// input itself is added in full float32).  On random data that is an error of ~2^-16 of
// sum|a||b| per output, invisible at bfloat16 / float8 output precision (eps >= 2^-8) but
// not at float32.  So the path is chosen by the precision the caller asked for:
//   bfloat16 / float8 outputs  -> mma_tile on the fp8 matrix cores (this is the 5 PFLOP/s path)
//   float32 / float16 outputs  -> the same kernel with each float8 fragment widened (exactly)
//                                 to bfloat16 in registers and fed to the bfloat16 matrix
//                                 core, which keeps float32 precision (half the rate: 2.5
//                                 PFLOP/s peak); inside the reference test's bound
//                                 eps*|want| + 2^-20 * sum|a||b| (tests/python/test_quant.py:124-126)
// The scales multiply once per output instead of once per operand element (one rounding
// less than the reference, inside the same bound).
//
//   mma_tile       (mma_tile.h) V_MFMA_F32_32X32X64_F8F6F4 / 16X16X128 (8192 flop/clk/CU: the only fp8 rate
//                  that reaches the 5 PFLOP/s peak; the 16x16x32 fp8 instruction runs at half).
//                  A workgroup computes a BM x BN tile, K in steps of 128 bytes; both
//                  operand tiles are staged in LDS (double buffered, 16-byte chunks XOR-
//                  swizzled by row pair so that the 32-byte-per-lane fragment reads are
//                  conflict free), each wave owns a (TM*16) x (TN*16) sub-tile in registers.
//                  The B matrix feeds the MFMA's first operand and A its second, so a lane
//                  ends up with 4 consecutive output columns of one row (vector stores).
//   fp8mm_generic  any shape / alignment: one thread per output, float32 FMA.
#include "kernels.h"
#include "mma_stream.h"
#include "mma_tile.h"
#include "mma_skinny.h"
#include "mma_slices.h"

namespace vkt {
namespace {

__device__ __forceinline__ float load_any_f32(uint64_t base, uint64_t i, uint32_t dtype) {
  if (dtype == VKT_F32) return ldg<float>(base + 4 * i);
  if (dtype == VKT_F16) return f16_to_f32(ldg<uint16_t>(base + 2 * i));
  return bf16_to_f32(ldg<uint16_t>(base + 2 * i));
}

// Scales, bias and the output scale for one output value.
__device__ __forceinline__ float finish(const F8Params& p, float acc, float sa, float sb, uint32_t n, float inv) {
  float v = acc * (sa * sb);
  if (p.bias) v += load_any_f32(p.bias, n, p.bias_dtype);
  if (p.out_dtype == VKT_E4M3 || p.out_dtype == VKT_E5M2) v *= inv;
  return v;
}

__device__ __forceinline__ void store_out(const F8Params& p, uint64_t index, float v) {
  switch (p.out_dtype) {
    case VKT_F32: stg<float>(p.out + index * 4, v); break;
    case VKT_F16: stg<uint16_t>(p.out + index * 2, f32_to_f16(v)); break;
    case VKT_BF16: stg<uint16_t>(p.out + index * 2, f32_to_bf16(v)); break;
    default: stg<uint8_t>(p.out + index, uint8_t(f32_to_fp8(v, int(p.out_dtype)))); break;
  }
}

__device__ __forceinline__ float output_inv(const F8Params& p) {
  if (!(p.out_dtype == VKT_E4M3 || p.out_dtype == VKT_E5M2)) return 1.0f;
  return 1.0f / (p.scale_result ? ldg<float>(p.scale_result) : 1.0f);
}

// _scaled_mm as a problem of the tile kernel: float8 operands, and in the epilogue the scales,
// the bias, the output scale and the cast.
struct F8Problem : F8Params {
  static constexpr bool kTransA = false, kTransB = false;  // float8 operands are rows of k
  uint32_t batches = 1;
  uint64_t a_batch = 0, b_batch = 0;
  struct Whole {
    float inv, sa_all, sb_all;
    bool vec_ok;
  };
  struct Columns {
    float sb[4], bias[4];
  };
  __device__ __forceinline__ Whole whole() const {
    return Whole{output_inv(*this), rowwise ? 0.0f : ldg<float>(scale_a), rowwise ? 0.0f : ldg<float>(scale_b),
                 (ldo & 3u) == 0 && (out & 15u) == 0};
  }
  __device__ __forceinline__ Columns columns(uint32_t, uint32_t col, const Whole& w) const {
    Columns c;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const uint32_t nn = col + r < n ? col + r : n - 1;
      c.sb[r] = rowwise ? ldg<float>(scale_b + 4ull * nn) : w.sb_all;
      c.bias[r] = bias ? load_any_f32(bias, nn, bias_dtype) : 0.0f;
    }
    return c;
  }
  template <int DT>
  __device__ __forceinline__ void store(uint32_t, uint32_t row, uint32_t col, const V4F& t, const Columns& c,
                                        const Whole& w) const {
    const float sa = rowwise ? ldg<float>(scale_a + 4ull * row) : w.sa_all;
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = t[r] * (sa * c.sb[r]);
      if (bias) v[r] += c.bias[r];
      if (DT < 0 || DT == VKT_E4M3 || DT == VKT_E5M2) v[r] *= w.inv;  // (inv is 1 for the other types)
    }
    const uint64_t index = uint64_t(row) * ldo + col;
    if constexpr (DT == VKT_F32) {
      stg<F4>(out + index * 4, F4{v[0], v[1], v[2], v[3]});
    } else if constexpr (DT == VKT_BF16) {
      stg<U2>(out + index * 2, U2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])});
    } else if constexpr (DT == VKT_F16) {
      stg<U2>(out + index * 2, U2{uint32_t(f32_to_f16(v[0])) | uint32_t(f32_to_f16(v[1])) << 16,
                                  uint32_t(f32_to_f16(v[2])) | uint32_t(f32_to_f16(v[3])) << 16});
    } else if constexpr (DT == VKT_E4M3 || DT == VKT_E5M2) {
      stg<uint32_t>(out + index, pack2_fp8<DT>(v[0], v[1]) | pack2_fp8<DT>(v[2], v[3]) << 16);
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (col + r < n) store_out(*this, index + r, v[r]);
    }
  }
  // the epilogue that stores straight from the accumulators: bfloat16 outputs, 16-byte aligned rows
  static constexpr bool kRegisterEpilogue = true;
  __device__ __forceinline__ bool register_epilogue(const Whole&) const {
    return out_dtype == VKT_BF16 && (ldo & 7u) == 0 && (out & 15u) == 0;
  }
  __device__ __forceinline__ float row_scale(uint32_t row, const Whole& w) const {
    return rowwise ? ldg<float>(scale_a + 4ull * row) : w.sa_all;
  }
  // scale and bias of columns col .. col + 3 (all inside n)
  __device__ __forceinline__ void column_terms(uint32_t col, const Whole& w, float (&s)[4], float (&b)[4]) const {
    if (rowwise) {
      const F4 v = ldg<F4>(scale_b + 4ull * col);
      s[0] = v.x, s[1] = v.y, s[2] = v.z, s[3] = v.w;
    } else {
      s[0] = s[1] = s[2] = s[3] = w.sb_all;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) b[r] = bias ? load_any_f32(bias, col + r, bias_dtype) : -0.0f;  // (adding -0.0f changes nothing, a zero's sign included)
  }
  __device__ __forceinline__ void store_bf16x8(uint32_t, uint32_t row, uint32_t col, const U4& v) const {
    stg<U4>(out + (uint64_t(row) * ldo + col) * 2, v);
  }
  // the stream kernel's epilogue (bfloat16 or float8 outputs)
  struct Rows {
    float scale;
  };
  struct Columns4 {
    float scale[4], bias[4];
  };
  __device__ __forceinline__ Rows rows(uint32_t, uint32_t row, const Whole& w) const { return Rows{row_scale(row, w)}; }
  __device__ __forceinline__ Columns4 columns4(uint32_t, uint32_t col, const Whole& w) const {
    Columns4 c;
    column_terms(col, w, c.scale, c.bias);
    return c;
  }
  __device__ __forceinline__ bool narrow(const Whole&) const { return out_dtype != VKT_BF16; }
  __device__ __forceinline__ void finish4(uint32_t, uint32_t, uint32_t, const float (&t)[4], const Rows& r, const Columns4& c, const Whole&,
                                          float (&v)[4]) const {
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = t[e] * (r.scale * c.scale[e]) + c.bias[e];
  }
  __device__ __forceinline__ void pack4(const float (&f)[4], const Whole& w, uint32_t (&packed)[2]) const {
    if (out_dtype == VKT_BF16) {
      pack_bf16x4(f, packed);
    } else {  // float8 outputs: the output scale
      const float v[4] = {f[0] * w.inv, f[1] * w.inv, f[2] * w.inv, f[3] * w.inv};
      packed[0] = out_dtype == VKT_E4M3 ? pack2_fp8<VKT_E4M3>(v[0], v[1]) | pack2_fp8<VKT_E4M3>(v[2], v[3]) << 16
                                        : pack2_fp8<VKT_E5M2>(v[0], v[1]) | pack2_fp8<VKT_E5M2>(v[2], v[3]) << 16;
      packed[1] = 0;
    }
  }
  __device__ __forceinline__ void store8(uint32_t, uint32_t row, uint32_t col, const U4& v) const {
    stg<U4>(out + (uint64_t(row) * ldo + col) * 2, v);
  }
  __device__ __forceinline__ void store8_narrow(uint32_t, uint32_t row, uint32_t col, const U2& v) const {
    stg<U2>(out + uint64_t(row) * ldo + col, v);
  }
  template <class F>
  __device__ __forceinline__ void for_output_type(bool full, const Whole& w, F&& f) const {
    if (w.vec_ok && full) {
      switch (out_dtype) {
        case VKT_F32: f(std::integral_constant<int, VKT_F32>{}); break;
        case VKT_BF16: f(std::integral_constant<int, VKT_BF16>{}); break;
        case VKT_F16: f(std::integral_constant<int, VKT_F16>{}); break;
        case VKT_E4M3: f(std::integral_constant<int, VKT_E4M3>{}); break;
        default: f(std::integral_constant<int, VKT_E5M2>{}); break;
      }
    } else {
      f(std::integral_constant<int, -1>{});
    }
  }
};

// Any shape, stride or alignment: one thread per output.
__global__ __launch_bounds__(256) void fp8mm_generic(F8Params p) {
  const uint32_t n = blockIdx.x * 64 + (threadIdx.x & 63), m = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (m >= p.m || n >= p.n) return;
  const uint64_t arow = p.a + uint64_t(m) * p.lda, brow = p.b + uint64_t(n) * p.ldb;
  float acc = 0.0f;
  for (uint32_t k = 0; k < p.k; ++k)
    acc = fmaf(fp8_to_f32(ldg<uint8_t>(arow + k), int(p.fmt_a)), fp8_to_f32(ldg<uint8_t>(brow + k), int(p.fmt_b)), acc);
  const float sa = ldg<float>(p.scale_a + (p.rowwise ? 4ull * m : 0)), sb = ldg<float>(p.scale_b + (p.rowwise ? 4ull * n : 0));
  store_out(p, uint64_t(m) * p.ldo + n, finish(p, acc, sa, sb, n, output_inv(p)));
}

// One and two rows of A on the vector units (the shape of the int8 op's one-row kernel): a wave streams COLS weight
// rows with 16-byte non-temporal loads, KSPLIT waves of the workgroup share a row's k; both operands are widened
// exactly to bfloat16 (two values per conversion instruction) and multiplied by two-element dot products into float32
// sums (products of two float8 values are exact in float32), so every output type is served at float32 precision.
// Many small workgroups have the whole weight stream in flight at once, and a workgroup may own as few as 2 columns:
// few columns against long rows keep the machine busy where the matrix-core kernel's 8 to 16 columns per workgroup do
// not (K = 8192, N = 1024: 4.5 against 6.8 us).
template <int F>
__device__ __forceinline__ void widen16_pairs(const U4& v, uint32_t (&out)[8]) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = __builtin_bit_cast(uint32_t, widen_pair<F, false>(int(v[i])));
    out[2 * i + 1] = __builtin_bit_cast(uint32_t, widen_pair<F, true>(int(v[i])));
  }
}

template <int ROWS, int COLS, int KSPLIT, int FA, int FB>
__global__ __launch_bounds__(256) void fp8mm_gemv(F8Params p) {
  constexpr int WAVES = 4, GROUPS = WAVES / KSPLIT;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int grp = wave / KSPLIT, ks = wave % KSPLIT;
  const uint32_t n0 = (blockIdx.x * GROUPS + grp) * COLS;
  float acc[ROWS][COLS];
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[r][c] = 0.0f;
  // (clamped: the tail group re-reads the last row, masked at the store)
  uint64_t brow[COLS], arow[ROWS];
#pragma unroll
  for (int c = 0; c < COLS; ++c) brow[c] = p.b + uint64_t(n0 + c < p.n ? n0 + c : p.n - 1) * p.ldb;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) arow[r] = p.a + uint64_t(uint32_t(r) < p.m ? uint32_t(r) : p.m - 1) * p.lda;

  for (uint32_t k = (ks * 64 + lane) * 16; k < p.k; k += 1024 * KSPLIT) {  // (k is a multiple of 16)
    U4 wv[COLS], av[ROWS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) wv[c] = ldg_stream<U4>(brow[c] + k);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) av[r] = ldg<U4>(arow[r] + k);
    uint32_t w[COLS][8], a[ROWS][8];
#pragma unroll
    for (int c = 0; c < COLS; ++c) widen16_pairs<FB>(wv[c], w[c]);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) widen16_pairs<FA>(av[r], a[r]);
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int i = 0; i < 8; ++i)
          acc[r][c] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(V2BF, a[r][i]), __builtin_bit_cast(V2BF, w[c][i]), acc[r][c], false);
  }
#pragma unroll
  for (int r = 0; r < ROWS; ++r)
#pragma unroll
    for (int c = 0; c < COLS; ++c) acc[r][c] = wave_sum(acc[r][c]);

  __shared__ float part[WAVES][ROWS * COLS];
  if constexpr (KSPLIT > 1) {
    if (lane == 0) {
#pragma unroll
      for (int r = 0; r < ROWS; ++r)
#pragma unroll
        for (int c = 0; c < COLS; ++c) part[wave][r * COLS + c] = acc[r][c];
    }
    __syncthreads();
    if (ks != 0) return;
  }
  // lane (r, c) of the group's first wave finishes output (r, n0 + c)
  if (lane < ROWS * COLS) {
    const int r = lane / COLS, c = lane % COLS;
    float sum = 0.0f;
#pragma unroll
    for (int rr = 0; rr < ROWS; ++rr)
#pragma unroll
      for (int cc = 0; cc < COLS; ++cc)
        if (rr == r && cc == c) sum = acc[rr][cc];  // (no dynamic register indexing)
    if constexpr (KSPLIT > 1) {
      sum = part[wave][lane];
#pragma unroll
      for (int s = 1; s < KSPLIT; ++s) sum += part[wave + s][lane];
    }
    const uint32_t n = n0 + c;
    if (uint32_t(r) < p.m && n < p.n) {
      const float sa = ldg<float>(p.scale_a + (p.rowwise ? 4ull * r : 0)), sb = ldg<float>(p.scale_b + (p.rowwise ? 4ull * n : 0));
      store_out(p, uint64_t(r) * p.ldo + n, finish(p, sum, sa, sb, n, output_inv(p)));
    }
  }
}

// -2: not this kernel's problem (more than four rows, short rows).
// One and two rows always; three and four where the matrix-core kernel would have fewer workgroups than half the
// machine's compute units (us at 3 rows, this kernel / that one: K = 8192, N = 1024: 4.8 / 7.0; K = 16384, N = 512:
// 8.3 / 9.4; but K = 4096, N = 14336: 16.9 / 12.4); forced: whatever the column count.
template <int FA, int FB>
int launch_gemv(const F8Params& p, int compute_units, bool forced, hipStream_t stream) {
  if (p.m > 4 || p.k < 1024) return -2;
  if (p.m > 2 && !forced && p.n > 8u * uint32_t(compute_units)) return -2;
  const int rows = p.m <= 1 ? 1 : p.m <= 2 ? 2 : 4;
  const int ksplit = p.k >= 4096 ? (p.k <= 8192 ? 4 : 2) : (p.k >= 2048 ? 2 : 1);  // (the int8 op's rule: a wave keeps one full 1 KiB load per column)
  const dim3 grid((p.n + 2 * (4 / ksplit) - 1) / (2 * (4 / ksplit)));
#define VKT_F8_GEMV_CASE(R_, KS_) \
  if (rows == R_ && ksplit == KS_) { hipLaunchKernelGGL((fp8mm_gemv<R_, 2, KS_, FA, FB>), grid, dim3(256), 0, stream, p); return 0; }
  VKT_F8_GEMV_CASE(1, 1) VKT_F8_GEMV_CASE(1, 2) VKT_F8_GEMV_CASE(1, 4) VKT_F8_GEMV_CASE(2, 1) VKT_F8_GEMV_CASE(2, 2) VKT_F8_GEMV_CASE(2, 4)
  VKT_F8_GEMV_CASE(4, 1) VKT_F8_GEMV_CASE(4, 2) VKT_F8_GEMV_CASE(4, 4)
#undef VKT_F8_GEMV_CASE
  return -2;
}

// The few-row kernel (mma_skinny.h) where it serves; bfloat16 and float8 outputs on the fp8 matrix-core instruction,
// float32 and float16 outputs on exactly widened operands (the precision rule of the tile kernels).  -2: not served.
template <int FA, int FB>
int launch_skinny(const F8Params& p0, const Machine& mc, uint32_t forced_nt, uint32_t forced_slices, hipStream_t stream, std::string* err) {
  F8Problem p;
  static_cast<F8Params&>(p) = p0;
  if (p0.out_dtype == VKT_F32 || p0.out_dtype == VKT_F16) return launch_mma_skinny<FA, FB, kMathFp8Wide>(p, mc, forced_nt, forced_slices, stream, err, "fp8mm");
  return launch_mma_skinny<FA, FB, kMathFp8>(p, mc, forced_nt, forced_slices, stream, err, "fp8mm");
}

// The 128 x 128 tile kernel with K in slices over workgroups (mma_slices.h): the float8 instruction for bfloat16 and
// float8 outputs, exactly widened operands for float32 and float16 outputs.
template <int FA, int FB>
int launch_sliced(const F8Params& p0, uint32_t slices, const Machine& mc, hipStream_t stream, std::string* err) {
  F8Problem p;
  static_cast<F8Params&>(p) = p0;
  if (slices < 2 || p0.k % (BK * slices) || uint64_t(slices) * p0.m * p0.n * 4 > mc.workspace_bytes) {
    *err = "fp8mm: " + std::to_string(slices) + " slices of K do not divide its steps of 128 bytes, or their partial sums do not fit the workspace";
    return -1;
  }
  if (p0.out_dtype == VKT_F32 || p0.out_dtype == VKT_F16) return launch_tile_slices<FA, FB, true, kMathFp8Wide>(p, slices, mc, stream, err, "fp8mm");
  return launch_tile_slices<FA, FB, false, kMathFp8>(p, slices, mc, stream, err, "fp8mm");
}

template <int WAVES_M, int WAVES_N, int TM, int TN, int FA, int FB, bool MF32 = false, bool DIRECT = false, bool WIDE = false>
int launch_tile(const F8Params& p, int compute_units, hipStream_t stream, std::string* err) {
  F8Problem problem;
  static_cast<F8Params&>(problem) = p;
  return launch_mma_tile<WAVES_M, WAVES_N, TM, TN, FA, FB, MF32, DIRECT, WIDE ? kMathFp8Wide : kMathFp8>(
      problem, compute_units, stream, err, "fp8mm");
}

// The stream kernel, where it serves the problem (bfloat16 or float8 output in aligned rows); -2: it does not.
template <int FA, int FB>
int launch_stream(const F8Params& p, int compute_units, hipStream_t stream, std::string* err) {
  F8Problem problem;
  static_cast<F8Params&>(problem) = p;
  const bool float8_out = p.out_dtype == VKT_E4M3 || p.out_dtype == VKT_E5M2;
  if (!(p.out_dtype == VKT_BF16 || float8_out) || p.ldo % 8 || p.out % (float8_out ? 8 : 16) || !mma_stream_serves(problem)) return -2;
  return launch_mma_stream<FA, FB, kMathFp8>(problem, compute_units, stream, err, "fp8mm");
}

template <int FA, int FB>
int launch_formats(const F8Params& p, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err) {
  const int compute_units = mc.compute_units;
  // variant 0: planned.  Explicit variants run the MFMA kernel whatever the output dtype
  // (tests, tuning): 1: 128x128 tiles (4 waves of 64x64, 16x16x128 MFMA); 2: 256x256 (4 waves of
  // 128x128, 16x16x128); 3: 256x128; 4: 256x256 with the 32x32x64 MFMA (measured ~10 % faster
  // than 16x16x128 at equal work); 5: as 4 with global-to-LDS direct loads when k is a
  // multiple of 128 (else 4); 8: as 5 with 8 waves of 64x128 instead of 4 of 128x128 (two waves per SIMD cover each
  // other's waits: 8192^3 2.34-2.42 -> 2.56-2.59 PFLOP/s; what they get where the stream kernel does not serve).  11: the stream kernel of
  // mma_stream.h where it serves the problem (large bfloat16 and float8 outputs get it), else 8.  255: the one-thread-per-output kernel.
  // 6 / 7: the exact path (float8 widened to bfloat16 in registers, 32x32x16 bfloat16 MFMA) on
  // 256x256 / 128x128 tiles: what float32 and float16 outputs get.
  const bool big = uint64_t(p.m) * p.n >= (1ull << 20);
  if (variant == 0 || variant == 13) {  // 13: the vector-unit kernel for one and two rows where it serves (what they get), else as planned
    const int rc = launch_gemv<FA, FB>(p, compute_units, variant == 13, stream);
    if (rc != -2) return rc;
    variant = 0;
  }
  if (variant == 0 || (variant & 0xff) == 12) {  // 12: the few-row kernel where it serves (what up to 64 rows get), else as planned; bits 8-11: 16s of columns per workgroup, bits 12-16: slices of K
    const int rc = launch_skinny<FA, FB>(p, mc, (variant >> 8) & 15u, (variant >> 12) & 31u, stream, err);
    if (rc != -2) return rc;
    // 65 rows and more against tiles that are half the machine or less: the 128 x 128 tile kernel with K in slices
    // over workgroups (mma_slices.h; variant 14 asks for it, bits 8-12: slices)
    if (variant == 0 && p.m > 64) {
      const uint64_t budget = mc.workspace_bytes < VKT_STATIC_SCRATCH_BYTES ? mc.workspace_bytes : VKT_STATIC_SCRATCH_BYTES;
      const uint32_t slices = tile_slices(p.m, p.n, p.k, uint32_t(mc.compute_units), budget);
      if (slices >= 2 && uint64_t((p.m + 127) / 128) * ((p.n + 127) / 128) * 2 <= uint64_t(mc.compute_units)) return launch_sliced<FA, FB>(p, slices, mc, stream, err);
    }
    // 65 to 256 rows against few tiles: the few-row kernel over blocks of 64 rows, where that many passes over the
    // weights are estimated shorter than the tile kernel, whose workgroups each walk all of K and are a quarter of the
    // machine at N = 8192 (us at 128 rows, tile kernel / two passes: 8192 x 8192: 73 / 56; 14336 x 4096: 123 / 54; 4096 x
    // 4096: 40 / 27; 4096 x 14336 and 8192 x 28672 stay: 43 and 94 against 57 and 176).  A pass: ~8 us + weights at
    // 2.95 MB/us; the 128 x 128 tile kernel: ~9 us per 1024 values of k and round of tiles.
    if (variant == 0 && p.m > 64 && p.m <= 256 && p.k >= 1024 && p.n >= 64) {
      const uint32_t passes = (p.m + 63) / 64, tiles = ((p.m + 127) / 128) * ((p.n + 127) / 128), cus = uint32_t(mc.compute_units);
      const float pass_us = 8.0f + float(p.n) * float(p.k) / 2.95e6f, tile_us = float(p.k) / 1024.0f * 9.0f * float((tiles + cus - 1) / cus);
      if (float(passes) * pass_us < 0.9f * tile_us) {
        const uint32_t out_item = p.out_dtype == VKT_F32 ? 4 : (p.out_dtype == VKT_F16 || p.out_dtype == VKT_BF16) ? 2 : 1;
        for (uint32_t r0 = 0; r0 < p.m; r0 += 64) {
          F8Params q = p;
          q.m = p.m - r0 < 64 ? p.m - r0 : 64;
          q.a = p.a + uint64_t(r0) * p.lda;
          q.out = p.out + uint64_t(r0) * p.ldo * out_item;
          if (p.rowwise) q.scale_a = p.scale_a + uint64_t(r0) * 4;
          const int rb = launch_skinny<FA, FB>(q, mc, 0, 0, stream, err);
          if (rb != 0) {  // (-2 cannot be: the shape was checked above; a refused workspace ends the product)
            if (rb == -2) *err = "fp8mm: the few-row kernel does not serve a block of rows";
            return -1;
          }
        }
        return 0;
      }
    }
    variant = 0;
  }
  // (256 x 256 tiles where they give the machine enough workgroups, else 128 x 128: the exact path from one tile per
  //  compute unit on (2048 x 4096 x 4096: 94 us on 128 x 128 tiles against 116; 1024 x 8192 x 8192: 164 against 200),
  //  the float8 path from one per four units on (512 x 8192 x 8192: 64 against 82 us; at 1024 rows the stream kernel
  //  is ahead, 91 against 99))
  const uint64_t tiles256 = uint64_t((p.m + 255) / 256) * ((p.n + 255) / 256), cus = uint64_t(compute_units);
  if (variant == 0)
    variant = (p.out_dtype == VKT_F32 || p.out_dtype == VKT_F16) ? (big && tiles256 >= cus ? 6 : 7) : (big && 4 * tiles256 > cus ? 11 : 1);
  if ((variant & 0xff) == 14) return launch_sliced<FA, FB>(p, (variant >> 8) & 31u, mc, stream, err);
  switch (variant) {
    case 6:
      if (p.k % BK == 0) return launch_tile<2, 2, 8, 8, FA, FB, true, true, true>(p, compute_units, stream, err);
      return launch_tile<2, 2, 8, 4, FA, FB, true, false, true>(p, compute_units, stream, err);  // (256x256 without the direct loads runs out of registers)
    case 7: return launch_tile<2, 2, 4, 4, FA, FB, true, false, true>(p, compute_units, stream, err);
    case 1: return launch_tile<2, 2, 4, 4, FA, FB>(p, compute_units, stream, err);
    case 2: return launch_tile<2, 2, 8, 8, FA, FB>(p, compute_units, stream, err);
    case 3: return launch_tile<2, 2, 8, 4, FA, FB>(p, compute_units, stream, err);
    case 4: return launch_tile<2, 2, 8, 8, FA, FB, true>(p, compute_units, stream, err);
    case 9:  // as 6 with 8 waves of 64x128
      if (p.k % BK == 0) return launch_tile<4, 2, 4, 8, FA, FB, true, true, true>(p, compute_units, stream, err);
      return launch_tile<2, 2, 8, 4, FA, FB, true, false, true>(p, compute_units, stream, err);
    case 11: {  // the stream kernel (mma_stream.h), else 8
      const int rc = launch_stream<FA, FB>(p, compute_units, stream, err);
      if (rc != -2) return rc;
    }
      [[fallthrough]];
    case 8:  // 256x256 tiles over 8 waves of 64x128 (two waves per SIMD), direct loads
      if (p.k % BK == 0) return launch_tile<4, 2, 4, 8, FA, FB, true, true>(p, compute_units, stream, err);
      return launch_tile<2, 2, 8, 8, FA, FB, true>(p, compute_units, stream, err);
    case 5:
      if (p.k % BK == 0) return launch_tile<2, 2, 8, 8, FA, FB, true, true>(p, compute_units, stream, err);
      return launch_tile<2, 2, 8, 8, FA, FB, true>(p, compute_units, stream, err);
  }
  *err = "fp8mm: unknown variant " + std::to_string(variant);
  return -1;
}

}  // namespace

int launch_fp8mm(const F8Params& p, uint32_t variant, const Machine& mc, hipStream_t stream, std::string* err) {
  if (p.m == 0 || p.n == 0) return 0;
  auto fp8 = [](uint32_t f) { return f == VKT_E4M3 || f == VKT_E5M2; };
  if (!fp8(p.fmt_a) || !fp8(p.fmt_b)) {
    *err = "fp8mm: operands must be e4m3fn or e5m2";
    return -1;
  }
  if (p.out_dtype > VKT_E5M2 || p.bias_dtype > VKT_BF16) {
    *err = "fp8mm: unsupported output or bias dtype";
    return -1;
  }
  // (k == 0: an empty product, zeros through the epilogue; the operands are then empty and may have no address)
  if ((p.k != 0 && (!p.a || !p.b)) || !p.scale_a || !p.scale_b || !p.out) {
    *err = "fp8mm: null tensor address";
    return -1;
  }
  if (p.lda < p.k || p.ldb < p.k || p.ldo < p.n) {
    *err = "fp8mm: row strides shorter than the rows";
    return -1;
  }
  if (uint64_t(p.m) * p.ldo >= (1ull << 32)) {
    *err = "fp8mm: output too large for 32-bit indexing";
    return -1;
  }
  int rc;
  if (p.k == 0 || p.k % 16 || p.lda % 16 || p.ldb % 16 || (p.a & 15) || (p.b & 15) || variant == 255) {
    if ((p.m + 3) / 4 > 65535) {
      *err = "fp8mm: too many rows for the unaligned path";
      return -1;
    }
    hipLaunchKernelGGL(fp8mm_generic, dim3((p.n + 63) / 64, (p.m + 3) / 4), dim3(256), 0, stream, p);
    rc = 0;
  } else if (p.fmt_a == VKT_E4M3 && p.fmt_b == VKT_E4M3) {
    rc = launch_formats<0, 0>(p, variant, mc, stream, err);
  } else if (p.fmt_a == VKT_E5M2 && p.fmt_b == VKT_E4M3) {
    rc = launch_formats<1, 0>(p, variant, mc, stream, err);
  } else if (p.fmt_a == VKT_E4M3 && p.fmt_b == VKT_E5M2) {
    rc = launch_formats<0, 1>(p, variant, mc, stream, err);
  } else {
    rc = launch_formats<1, 1>(p, variant, mc, stream, err);
  }
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "fp8mm: kernel launch failed";
    return -1;
  }
  return rc;
}

}  // namespace vkt
