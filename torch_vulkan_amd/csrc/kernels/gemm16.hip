// The unquantised Linear next to the quantised ops: C[b] = alpha * A[b] @ B[b] (+ beta * Cin[b])
// for bfloat16 / float16 matrices, products accumulated in float32 and rounded once - the
// contract of the reference's cooperative-matrix kernel (crates/vkcore/shaders/gemmcm.slang,
// host side crates/pyvk/csrc/linalg.cpp:227-255), behind its kernel names ("gemmcm_bf16",
// "gemmcm_f16"), parameter block (GemmParams, strides in elements) and spec {USE_CIN, ..}.
//   - operands whose rows are 16-byte aligned and contiguous along one of their two dims, C
//     contiguous along n: the tile kernel of _scaled_mm (mma_tile.h: 256x256x64-value workgroup
//     tiles, direct global-to-LDS loads, persistent grid) with V_MFMA_F32_32X32X16_{BF16,F16}
//     and an alpha / beta epilogue.  A contiguous along k and B along k (x @ W.t(), the Linear
//     layout) takes k a multiple of 8; an operand contiguous along m or n (x @ W, x.t() @ y:
//     what backward passes produce) is read through the transposing LDS load and takes k a
//     multiple of 64 and m (n) of 8;
//   - everything else (strided views, odd sizes): one thread per output over the strides as
//     given.  Correct for any strides, and slow.
#include "kernels.h"
#include "mma_stream.h"
#include "mma_tile.h"
#include "mma_skinny.h"
#include "mma_slices.h"

namespace vkt {
namespace {

__device__ __forceinline__ float slot_float(uint64_t slot) { return bits_f32(uint32_t(slot)); }

template <class T, bool TRA = false, bool TRB = false>
struct GemmProblem {
  static constexpr bool kTransA = TRA, kTransB = TRB;
  static constexpr bool kRegisterEpilogue = false;
  // operands as the tile kernel takes them (bytes)
  uint64_t a, b;
  uint32_t m, n, k, lda, ldb, batches;
  uint64_t a_batch, b_batch;
  // epilogue
  uint64_t c, cin;
  float alpha, beta;
  int32_t c_sm, c_sb, cin_sm, cin_sn, cin_sb;  // elements (c_sn is 1 here)
  struct Whole {
    uint32_t vec_ok;
  };
  struct Columns {};
  // (a word, not a bool: the one-byte struct stayed in memory, 8 bytes of scratch per lane in the kernels that use it; in
  // the few-row kernel's second launch it went through LDS, indexed by a workgroup size read from the dispatch packet
  // in host memory: 12 us in a 3 us kernel)
  __device__ __forceinline__ Whole whole() const { return Whole{((uint32_t(c_sm) & 3u) | (uint32_t(c_sb) & 3u) | (uint32_t(c) & 7u)) == 0 ? 1u : 0u}; }
  __device__ __forceinline__ Columns columns(uint32_t, uint32_t, const Whole&) const { return Columns{}; }
  template <int DT>
  __device__ __forceinline__ void store(uint32_t batch, uint32_t row, uint32_t col, const V4F& t, const Columns&,
                                        const Whole&) const {
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = alpha * t[r];
      if (cin != 0 && (DT >= 0 || col + r < n)) {  // beta == 0 never reads Cin (it may hold NaN): then cin is 0
        const int64_t at = int64_t(batch) * cin_sb + int64_t(row) * cin_sm + int64_t(col + r) * cin_sn;
        v[r] += beta * load_f32<T>(cin + uint64_t(at * 2));
      }
    }
    const uint64_t out = c + uint64_t((int64_t(batch) * c_sb + int64_t(row) * c_sm + int64_t(col)) * 2);
    if constexpr (DT >= 0) {
      if constexpr (T::dtype == VKT_BF16) stg<U2>(out, U2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])});
      else stg<U2>(out, U2{uint32_t(f32_to_f16(v[0])) | uint32_t(f32_to_f16(v[1])) << 16,
                           uint32_t(f32_to_f16(v[2])) | uint32_t(f32_to_f16(v[3])) << 16});
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (col + r < n) store_f32<T>(out + 2 * r, v[r]);
    }
  }
  template <class F>
  __device__ __forceinline__ void for_output_type(bool full, const Whole& w, F&& f) const {
    if (w.vec_ok && full) f(std::integral_constant<int, T::dtype>{});
    else f(std::integral_constant<int, -1>{});
  }
  // the stream kernel's epilogue (C rows and batches 16-byte aligned)
  struct Rows {};
  struct Columns4 {};
  __device__ __forceinline__ Rows rows(uint32_t, uint32_t, const Whole&) const { return Rows{}; }
  __device__ __forceinline__ Columns4 columns4(uint32_t, uint32_t, const Whole&) const { return Columns4{}; }
  __device__ __forceinline__ bool narrow(const Whole&) const { return false; }
  __device__ __forceinline__ void finish4(uint32_t batch, uint32_t row, uint32_t col, const float (&t)[4], const Rows&, const Columns4&, const Whole&,
                                          float (&v)[4]) const {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      v[r] = alpha * t[r];
      if (cin != 0) {  // beta == 0 never reads Cin (it may hold NaN): then cin is 0
        const int64_t at = int64_t(batch) * cin_sb + int64_t(row) * cin_sm + int64_t(col + r) * cin_sn;
        v[r] += beta * load_f32<T>(cin + uint64_t(at * 2));
      }
    }
  }
  __device__ __forceinline__ void pack4(const float (&v)[4], const Whole&, uint32_t (&packed)[2]) const { pack_16bit_x4<T>(v, packed); }
  __device__ __forceinline__ void store8(uint32_t batch, uint32_t row, uint32_t col, const U4& v) const {
    stg<U4>(c + uint64_t((int64_t(batch) * c_sb + int64_t(row) * c_sm + int64_t(col)) * 2), v);
  }
  __device__ __forceinline__ void store8_narrow(uint32_t, uint32_t, uint32_t, const U2&) const {}
};

// Any strides: one thread per output, float32 accumulation.
template <class T>
__global__ __launch_bounds__(256) void gemm16_generic(GemmParams p, uint32_t use_cin) {
  const uint32_t n = blockIdx.x * 64 + (threadIdx.x & 63), m = blockIdx.y * 4 + (threadIdx.x >> 6), batch = blockIdx.z;
  if (m >= p.m || n >= p.n) return;
  const int64_t a0 = int64_t(batch) * p.a_sb + int64_t(m) * p.a_sm, b0 = int64_t(batch) * p.b_sb + int64_t(n) * p.b_sn;
  float acc = 0.0f;
  for (uint32_t k = 0; k < p.k; ++k)
    acc = fmaf(load_f32<T>(p.a + uint64_t((a0 + int64_t(k) * p.a_sk) * 2)), load_f32<T>(p.b + uint64_t((b0 + int64_t(k) * p.b_sk) * 2)), acc);
  float v = slot_float(p.alpha) * acc;
  if (use_cin) {
    const int64_t at = int64_t(batch) * p.cin_sb + int64_t(m) * p.cin_sm + int64_t(n) * p.cin_sn;
    v += slot_float(p.beta) * load_f32<T>(p.cin + uint64_t(at * 2));
  }
  store_f32<T>(p.c + uint64_t((int64_t(batch) * p.c_sb + int64_t(m) * p.c_sm + int64_t(n) * p.c_sn) * 2), v);
}

// One and two rows of A in the Linear layout on the vector units (three and four against few columns): a wave streams
// 2 weight rows with 16-byte non-temporal loads, 1, 2 or 4 waves of the workgroup share a row's k, two-element dot
// products into float32 sums (products of two 16-bit values are exact in float32), wave sums by DPP, the K-parts
// through LDS.  Many small workgroups have the whole weight stream in flight at once; the matrix-core kernel needs 8
// to 16 columns per workgroup and leaves most of the machine idle against few columns.  g.k, g.lda, g.ldb in bytes.
template <class T, int ROWS, int COLS, int KSPLIT>
__global__ __launch_bounds__(256) void gemm16_gemv(GemmProblem<T> g) {
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
  for (int c = 0; c < COLS; ++c) brow[c] = g.b + uint64_t(n0 + c < g.n ? n0 + c : g.n - 1) * g.ldb;
#pragma unroll
  for (int r = 0; r < ROWS; ++r) arow[r] = g.a + uint64_t(uint32_t(r) < g.m ? uint32_t(r) : g.m - 1) * g.lda;
  for (uint32_t k = (ks * 64 + lane) * 16; k < g.k; k += 1024 * KSPLIT) {  // (k is a multiple of 16 bytes)
    U4 wv[COLS], av[ROWS];
#pragma unroll
    for (int c = 0; c < COLS; ++c) wv[c] = ldg_stream<U4>(brow[c] + k);
#pragma unroll
    for (int r = 0; r < ROWS; ++r) av[r] = ldg<U4>(arow[r] + k);
#pragma unroll
    for (int r = 0; r < ROWS; ++r)
#pragma unroll
      for (int c = 0; c < COLS; ++c)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const uint32_t x = av[r][i], y = wv[c][i];  // (values: a bit cast of a vector's element expression reads element 0)
          if constexpr (T::dtype == VKT_BF16) {
            acc[r][c] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(V2BF, x), __builtin_bit_cast(V2BF, y), acc[r][c], false);
          } else {
            typedef _Float16 V2H __attribute__((ext_vector_type(2)));
            acc[r][c] = __builtin_amdgcn_fdot2(__builtin_bit_cast(V2H, x), __builtin_bit_cast(V2H, y), acc[r][c], false);
          }
        }
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
    if (uint32_t(r) < g.m && n < g.n) {
      float v = g.alpha * sum;
      if (g.cin != 0) v += g.beta * load_f32<T>(g.cin + uint64_t((int64_t(r) * g.cin_sm + int64_t(n) * g.cin_sn) * 2));  // (beta == 0 never reads Cin: then cin is 0)
      store_f32<T>(g.c + uint64_t((int64_t(r) * g.c_sm + int64_t(n)) * 2), v);
    }
  }
}

// One and two rows always; three and four where the matrix-core kernel would have fewer workgroups than half the
// machine's compute units; forced: up to four rows whatever the column count.  -2: not this kernel's problem.
template <class T>
int launch_gemv16(const GemmProblem<T>& g, int compute_units, bool forced, hipStream_t stream) {
  if (g.m > 4 || g.k < 1024) return -2;
  if (g.m > 2 && !forced && g.n > 8u * uint32_t(compute_units)) return -2;
  // (two long rows against many columns: 25.3 against 23.6 us at K = N = 8192; level at K = 4096, N = 14336; ahead elsewhere)
  if (g.m == 2 && !forced && g.k >= 2 * 8192 && g.n >= 8192) return -2;
  const int rows = g.m <= 1 ? 1 : g.m <= 2 ? 2 : 4;
  const int ksplit = g.k >= 4096 ? (g.k <= 8192 ? 4 : 2) : (g.k >= 2048 ? 2 : 1);  // (a wave keeps one full 1 KiB load per column)
  const dim3 grid((g.n + 2 * (4 / ksplit) - 1) / (2 * (4 / ksplit)));
#define VKT_G16_GEMV_CASE(R_, KS_) \
  if (rows == R_ && ksplit == KS_) { hipLaunchKernelGGL((gemm16_gemv<T, R_, 2, KS_>), grid, dim3(256), 0, stream, g); return 0; }
  VKT_G16_GEMV_CASE(1, 1) VKT_G16_GEMV_CASE(1, 2) VKT_G16_GEMV_CASE(1, 4) VKT_G16_GEMV_CASE(2, 1) VKT_G16_GEMV_CASE(2, 2) VKT_G16_GEMV_CASE(2, 4)
  VKT_G16_GEMV_CASE(4, 1) VKT_G16_GEMV_CASE(4, 2) VKT_G16_GEMV_CASE(4, 4)
#undef VKT_G16_GEMV_CASE
  return -2;
}

template <class T, bool TRA, bool TRB>
int launch_tiles(const GemmParams& p, uint32_t use_cin, uint32_t batch, uint32_t variant, const Machine& mc, hipStream_t stream,
                 std::string* err) {
  constexpr int MATH = T::dtype == VKT_BF16 ? kMathBf16 : kMathF16;
  GemmProblem<T, TRA, TRB> g;
  g.a = p.a, g.b = p.b, g.m = p.m, g.n = p.n, g.k = p.k * 2;
  g.lda = uint32_t(TRA ? p.a_sk : p.a_sm) * 2, g.ldb = uint32_t(TRB ? p.b_sk : p.b_sn) * 2;
  g.batches = batch, g.a_batch = uint64_t(p.a_sb) * 2, g.b_batch = uint64_t(p.b_sb) * 2;
  g.c = p.c, g.cin = use_cin ? p.cin : 0;
  g.alpha = bits_f32_host(uint32_t(p.alpha)), g.beta = bits_f32_host(uint32_t(p.beta));
  g.c_sm = p.c_sm, g.c_sb = p.c_sb, g.cin_sm = p.cin_sm, g.cin_sn = p.cin_sn, g.cin_sb = p.cin_sb;
  // Up to 64 rows against weights in rows of k (x @ w.T at decode): the few-row kernel (mma_skinny.h), whose
  // workgroups own runs of columns and whose waves split K: the product is the weight stream, and 128 x 128 tiles put
  // 64 workgroups on the machine at N = 8192 (variant 7 asks for it; bits 8-11: 16s of columns per workgroup).
  if constexpr (!TRA && !TRB) {
    if ((variant == 0 || variant == 8) && batch == 1) {  // 8: the vector-unit kernel for up to four rows
      const int rc = launch_gemv16<T>(g, mc.compute_units, variant == 8, stream);
      if (rc != -2) return rc;
    }
    if (variant == 8) variant = 0;
    if (variant == 0 || (variant & 0xff) == 7) {  // (batches too: a batch of few-row products, attention at decode)
      const int rc = launch_mma_skinny<0, 0, MATH>(g, mc, (variant >> 8) & 15u, (variant >> 12) & 31u, stream, err, "gemmcm");
      if (rc != -2) return rc;
    }
  }
  if ((variant & 0xff) == 7) variant = 0;
  // The same few rows against weights stored [k, n] (x @ w): the few-row kernel that reads the weights through the
  // transposing LDS read (variant 9 asks for it; bits 12-16: slices of K over workgroups).
  if constexpr (!TRA && TRB) {
    if (variant == 0 || (variant & 0xff) == 9) {
      const int rc = launch_mma_skinny_kn<MATH>(g, mc, (variant >> 12) & 31u, stream, err, "gemmcm");
      if (rc != -2) return rc;
    }
  }
  if ((variant & 0xff) == 9) variant = 0;
  // 65 rows and more against tiles that are half the machine or less, A in rows of k: the 128 x 128 tile kernel with K
  // in slices over workgroups (mma_slices.h; variant 10 asks for it, bits 8-12: slices)
  if constexpr (!TRA) {
    if ((variant == 0 || (variant & 0xff) == 10) && batch == 1) {
      const bool asked = (variant & 0xff) == 10;
      const uint64_t budget = mc.workspace_bytes < VKT_STATIC_SCRATCH_BYTES ? mc.workspace_bytes : VKT_STATIC_SCRATCH_BYTES;
      const uint32_t slices = asked ? (variant >> 8) & 31u : (p.m > 64 ? tile_slices(p.m, p.n, g.k, uint32_t(mc.compute_units), budget) : 1);
      if (asked && (slices < 2 || g.k % (BK * slices) || uint64_t(slices) * p.m * p.n * 4 > mc.workspace_bytes)) {
        *err = "gemmcm: " + std::to_string(slices) + " slices of K do not divide its steps of 64 values, or their partial sums do not fit the workspace";
        return -1;
      }
      if (asked || (slices >= 2 && uint64_t((p.m + 127) / 128) * ((p.n + 127) / 128) * 2 <= uint64_t(mc.compute_units)))
        return launch_tile_slices<0, 0, true, MATH>(g, slices, mc, stream, err, "gemmcm");
    }
  }
  if ((variant & 0xff) == 10) variant = 0;
  // 65 to 256 rows against few tiles, either weight layout: the few-row kernels over blocks of 64 rows, where that many
  // passes over the weights are estimated shorter than the tile kernel, whose workgroups each walk all of K and are a
  // quarter of the machine at N = 8192 (us at 128 rows, tile kernel / two passes: 8192 x 8192: 113 / 86; 14336 x 4096:
  // 195 / 79; 4096 x 4096: 58 / 37; 4096 x 14336 and 8192 x 28672 stay).  A pass: ~8 us + weights at 3.9 MB/us; the
  // 128 x 128 tile kernel: ~14 us per 1024 values of k and round of tiles.
  if constexpr (!TRA) {
    if (variant == 0 && p.m > 64 && p.m <= 256 && p.k >= 512 && p.n >= 64 && batch <= 65535) {
      const uint32_t passes = (p.m + 63) / 64, cus = uint32_t(mc.compute_units);
      const uint64_t tiles = uint64_t((p.m + 127) / 128) * ((p.n + 127) / 128) * batch;
      const float pass_us = 8.0f + float(p.n) * float(p.k) * 2.0f * float(batch) / 3.9e6f;
      const float tile_us = float(p.k) / 1024.0f * 14.0f * float((tiles + cus - 1) / cus);
      if (float(passes) * pass_us < 0.9f * tile_us) {
        for (uint32_t r0 = 0; r0 < p.m; r0 += 64) {
          GemmProblem<T, TRA, TRB> q = g;
          q.m = p.m - r0 < 64 ? p.m - r0 : 64;
          q.a = g.a + uint64_t(r0) * g.lda;
          q.c = g.c + uint64_t(int64_t(r0) * g.c_sm * 2);
          if (g.cin) q.cin = g.cin + uint64_t(int64_t(r0) * g.cin_sm * 2);
          int rb;
          if constexpr (TRB) rb = launch_mma_skinny_kn<MATH>(q, mc, 0, stream, err, "gemmcm");
          else rb = launch_mma_skinny<0, 0, MATH>(q, mc, 0, 0, stream, err, "gemmcm");
          if (rb == -2 && r0 == 0) break;  // (not served: nothing is launched yet, the tile kernels take the product)
          if (rb != 0) {
            if (rb == -2) *err = "gemmcm: the few-row kernel does not serve a block of rows";
            return -1;
          }
          if (r0 + 64 >= p.m) return 0;
        }
      }
    }
  }
  const bool direct_ok = g.k % BK == 0;
  // variant 0: planned; 1: 128x128 tiles; 2: 256x128; 3: 256x256 with direct loads; 4: 128x128 with direct loads;
  // 5: 256x256 with direct loads over 8 waves; 6: the stream kernel (mma_stream.h; else 3)
  // (direct loads: k a multiple of 64; k-major operands run on the direct forms only)
  if (variant == 0) {
    // 256 x 256 tiles where they give every compute unit one, else 128 x 128
    // (from five eighths of a tile per unit on: 1024 x 4096 x 14336 is 224 tiles on 256 units, 121 us on the stream
    //  kernel against 163 on 128 x 128 tiles; 168 tiles: 142 against 152; at 128 tiles the small tiles are level or ahead)
    const bool large = uint64_t((p.m + 255) / 256) * ((p.n + 255) / 256) * batch * 8 >= uint64_t(mc.compute_units) * 5;
    // (both operands k-major: 8 waves, whose transposing LDS reads cover each other: 8192^3 0.94 -> 1.11-1.13 PFLOP/s;
    //  with k-contiguous operands the 8-wave form reads 1.5x the LDS bytes and is 3-5 % slower)
    variant = large ? (direct_ok ? (TRA && TRB ? 5 : 3) : 2) : (TRA || TRB ? 4 : 1);
    // both operands contiguous along k (x @ w.T): the stream kernel where it serves (8192^3: 0.94-1.00 -> 0.89 ms)
    if (!TRA && !TRB && variant == 3) variant = 6;
  }
  const bool stream_ok = direct_ok && g.k >= 2 * BK && p.n % 8 == 0 && p.c_sm % 8 == 0 && p.c_sb % 8 == 0 && p.c % 16 == 0 &&
                         mma_stream_strides_ok(g.lda, g.ldb);
  if (variant == 6 && !stream_ok) variant = 3;
  if constexpr (!TRA && !TRB) {
    // 6: the stream kernel (mma_stream.h) where it serves the problem: k a multiple of 64 values and at least 128, n a multiple of 8, C in 16-byte aligned rows
    if (variant == 6) return launch_mma_stream<0, 0, MATH>(g, mc.compute_units, stream, err, "gemmcm");
    if (variant == 1) return launch_mma_tile<2, 2, 4, 4, 0, 0, true, false, MATH>(g, mc.compute_units, stream, err, "gemmcm");
    if (variant == 2) return launch_mma_tile<2, 2, 8, 4, 0, 0, true, false, MATH>(g, mc.compute_units, stream, err, "gemmcm");
  }
  if (variant == 3 && direct_ok) return launch_mma_tile<2, 2, 8, 8, 0, 0, true, true, MATH>(g, mc.compute_units, stream, err, "gemmcm");
  if (variant == 4 && direct_ok) return launch_mma_tile<2, 2, 4, 4, 0, 0, true, true, MATH>(g, mc.compute_units, stream, err, "gemmcm");
  // 5: 256x256 over 8 waves of 64x128 (two waves per SIMD), direct loads
  if (variant == 5 && direct_ok) return launch_mma_tile<4, 2, 4, 8, 0, 0, true, true, MATH>(g, mc.compute_units, stream, err, "gemmcm");
  *err = "gemmcm: unknown variant " + std::to_string(variant) + " for this k and layout";
  return -1;
}

template <class T>
int launch_gemm16_t(const GemmParams& p, uint32_t use_cin, uint32_t batch, uint32_t variant, const Machine& mc,
                    hipStream_t stream, std::string* err) {
  // an operand is k-contiguous (rows of k), or k-major (contiguous along m / n, rows of k apart)
  auto rows_ok = [](int32_t contiguous, int32_t pitch, int32_t batch_stride, uint64_t base, uint32_t row_len) {
    return contiguous == 1 && pitch > 0 && pitch % 8 == 0 && uint32_t(pitch) >= row_len && batch_stride >= 0 &&
           batch_stride % 8 == 0 && base % 16 == 0;
  };
  const bool a_k = rows_ok(p.a_sk, p.a_sm, p.a_sb, p.a, p.k), b_k = rows_ok(p.b_sk, p.b_sn, p.b_sb, p.b, p.k);
  const bool a_m = !a_k && p.m % 8 == 0 && rows_ok(p.a_sm, p.a_sk, p.a_sb, p.a, p.m);
  const bool b_n = !b_k && p.n % 8 == 0 && rows_ok(p.b_sn, p.b_sk, p.b_sb, p.b, p.n);
  const bool k_ok = p.k != 0 && (a_m || b_n ? p.k % 64 == 0 : p.k % 8 == 0);
  const bool tiles_ok = (a_k || a_m) && (b_k || b_n) && k_ok && p.c_sn == 1 && p.c_sm > 0 && p.c_sb >= 0 && variant != 255;
  if (!tiles_ok) {
    if ((p.m + 3) / 4 > 65535 || batch > 65535) {
      *err = "gemmcm: too many rows or batches for the strided kernel";
      return -1;
    }
    hipLaunchKernelGGL((gemm16_generic<T>), dim3((p.n + 63) / 64, (p.m + 3) / 4, batch), dim3(256), 0, stream, p, use_cin);
    return 0;
  }
  if (a_m && b_n) return launch_tiles<T, true, true>(p, use_cin, batch, variant, mc, stream, err);
  if (a_m) return launch_tiles<T, true, false>(p, use_cin, batch, variant, mc, stream, err);
  if (b_n) return launch_tiles<T, false, true>(p, use_cin, batch, variant, mc, stream, err);
  return launch_tiles<T, false, false>(p, use_cin, batch, variant, mc, stream, err);
}

// ---- _weight_int8pack_mm for many rows (prefill): the int8 weights are widened once into a scratch matrix of the
// activations' type (exact) and the product runs on the tile kernel above, the per-column scales applied to the
// float32 sums in the epilogue, as the decode kernels do.  The row-block kernels of qmm8.hip re-read every weight
// once per 64 rows; from a few hundred rows on that costs more than the one extra pass over the weights.

template <class T>
struct Q8GemmProblem {
  static constexpr bool kTransA = false, kTransB = false;
  static constexpr bool kRegisterEpilogue = false;
  uint64_t a, b;
  uint32_t m, n, k, lda, ldb, batches;
  uint64_t a_batch, b_batch;
  uint64_t c, scales;
  struct Whole {
    uint32_t vec_ok;  // (a word, as in GemmProblem)
  };
  struct Columns {
    float s[4];
  };
  __device__ __forceinline__ Whole whole() const { return Whole{((n & 3u) | (uint32_t(c) & 7u)) == 0 ? 1u : 0u}; }
  __device__ __forceinline__ Columns columns(uint32_t, uint32_t col, const Whole&) const {
    Columns cs;
#pragma unroll
    for (int r = 0; r < 4; ++r) cs.s[r] = load_f32<T>(scales + uint64_t(col + r < n ? col + r : n - 1) * 2);
    return cs;
  }
  template <int DT>
  __device__ __forceinline__ void store(uint32_t, uint32_t row, uint32_t col, const V4F& t, const Columns& cs, const Whole&) const {
    float v[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = t[r] * cs.s[r];
    const uint64_t out = c + (uint64_t(row) * n + col) * 2;
    if constexpr (DT >= 0) {
      if constexpr (T::dtype == VKT_BF16) stg<U2>(out, U2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])});
      else stg<U2>(out, U2{uint32_t(f32_to_f16(v[0])) | uint32_t(f32_to_f16(v[1])) << 16,
                           uint32_t(f32_to_f16(v[2])) | uint32_t(f32_to_f16(v[3])) << 16});
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (col + r < n) store_f32<T>(out + 2 * r, v[r]);
    }
  }
  template <class F>
  __device__ __forceinline__ void for_output_type(bool full, const Whole& w, F&& f) const {
    if (w.vec_ok && full) f(std::integral_constant<int, T::dtype>{});
    else f(std::integral_constant<int, -1>{});
  }
  // the stream kernel's epilogue (n a multiple of 8, C and the scales 16-byte aligned)
  struct Rows {};
  struct Columns4 {
    float s[4];
  };
  __device__ __forceinline__ Rows rows(uint32_t, uint32_t, const Whole&) const { return Rows{}; }
  __device__ __forceinline__ Columns4 columns4(uint32_t, uint32_t col, const Whole&) const {
    Columns4 cs;
    const U2 raw = ldg<U2>(scales + uint64_t(col) * 2);  // (col a multiple of 4)
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      if constexpr (T::dtype == VKT_BF16) cs.s[2 * e] = bits_f32(raw[e] << 16), cs.s[2 * e + 1] = bits_f32(raw[e] & 0xffff0000u);
      else cs.s[2 * e] = f16_to_f32(uint16_t(raw[e])), cs.s[2 * e + 1] = f16_to_f32(uint16_t(raw[e] >> 16));
    }
    return cs;
  }
  __device__ __forceinline__ bool narrow(const Whole&) const { return false; }
  __device__ __forceinline__ void finish4(uint32_t, uint32_t, uint32_t, const float (&t)[4], const Rows&, const Columns4& cs, const Whole&,
                                          float (&v)[4]) const {
#pragma unroll
    for (int r = 0; r < 4; ++r) v[r] = t[r] * cs.s[r];
  }
  __device__ __forceinline__ void pack4(const float (&v)[4], const Whole&, uint32_t (&packed)[2]) const { pack_16bit_x4<T>(v, packed); }
  __device__ __forceinline__ void store8(uint32_t, uint32_t row, uint32_t col, const U4& v) const { stg<U4>(c + (uint64_t(row) * n + col) * 2, v); }
  __device__ __forceinline__ void store8_narrow(uint32_t, uint32_t, uint32_t, const U2&) const {}
};

// 16 int8 values per thread -> 16 values of T (integers of magnitude <= 128 are exact in both 16-bit types).
template <class T>
__global__ __launch_bounds__(256) void widen_i8_kernel(uint64_t src, uint64_t dst, uint64_t groups) {
  const uint64_t stride = uint64_t(gridDim.x) * 256;
  for (uint64_t g = uint64_t(blockIdx.x) * 256 + threadIdx.x; g < groups; g += stride) {
    const U4 v = ldg_stream<U4>(src + g * 16);
    uint32_t out[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float f0 = float(int(int8_t(v[i]))), f1 = float(int(int8_t(v[i] >> 8)));
      const float f2 = float(int(int8_t(v[i] >> 16))), f3 = float(int(int8_t(v[i] >> 24)));
      if constexpr (T::dtype == VKT_BF16) {
        out[2 * i] = __builtin_amdgcn_perm(f32_bits(f1), f32_bits(f0), 0x07060302u);
        out[2 * i + 1] = __builtin_amdgcn_perm(f32_bits(f3), f32_bits(f2), 0x07060302u);
      } else {
        out[2 * i] = uint32_t(f32_to_f16(f0)) | uint32_t(f32_to_f16(f1)) << 16;
        out[2 * i + 1] = uint32_t(f32_to_f16(f2)) | uint32_t(f32_to_f16(f3)) << 16;
      }
    }
    stg<U4>(dst + g * 32, U4{out[0], out[1], out[2], out[3]});
    stg<U4>(dst + g * 32 + 16, U4{out[4], out[5], out[6], out[7]});
  }
}

template <class T>
int launch_q8_gemm_t(const Q8Params& p, const Machine& mc, hipStream_t stream, std::string* err) {
  constexpr int MATH = T::dtype == VKT_BF16 ? kMathBf16 : kMathF16;
  const uint64_t groups = uint64_t(p.n) * p.k / 16, want = (groups + 255) / 256, cap = uint64_t(mc.compute_units) * 32;
  hipLaunchKernelGGL(widen_i8_kernel<T>, dim3(uint32_t(want < cap ? want : cap)), dim3(256), 0, stream, p.b, mc.scratch, groups);
  Q8GemmProblem<T> g;
  g.a = p.a, g.b = mc.scratch, g.m = p.m, g.n = p.n, g.k = p.k * 2, g.lda = uint32_t(p.a_sm) * 2, g.ldb = p.k * 2;
  g.batches = 1, g.a_batch = 0, g.b_batch = 0, g.c = p.c, g.scales = p.scales;
  const bool large = uint64_t((p.m + 255) / 256) * ((p.n + 255) / 256) * 8 >= uint64_t(mc.compute_units) * 5;  // (as for the 16-bit product)
  if (g.k % BK == 0) {
    if (large && g.k >= 2 * BK && p.n % 8 == 0 && p.c % 16 == 0 && p.scales % 16 == 0 && mma_stream_strides_ok(g.lda, g.ldb))
      return launch_mma_stream<0, 0, MATH>(g, mc.compute_units, stream, err, "qmm8");
    if (large) return launch_mma_tile<2, 2, 8, 8, 0, 0, true, true, MATH>(g, mc.compute_units, stream, err, "qmm8");
    return launch_mma_tile<2, 2, 4, 4, 0, 0, true, true, MATH>(g, mc.compute_units, stream, err, "qmm8");
  }
  if (large) return launch_mma_tile<2, 2, 8, 4, 0, 0, true, false, MATH>(g, mc.compute_units, stream, err, "qmm8");
  return launch_mma_tile<2, 2, 4, 4, 0, 0, true, false, MATH>(g, mc.compute_units, stream, err, "qmm8");
}

}  // namespace

uint64_t q8_gemm_scratch_bytes(const Q8Params& p, int dtype, const Machine& mc) {
  // (worth it where 128 x 128 tiles give every compute unit one: fewer tiles leave most of the machine idle, and the
  // row-block kernels, which split K, do better)
  if (uint64_t((p.m + 127) / 128) * ((p.n + 127) / 128) < uint64_t(mc.compute_units)) return 0;
  // (weights whose widening does not stay in the 256 MiB last-level cache, one byte read and two written per weight:
  // the pass costs ~0.75 us per million weights and the product ~0.0021 per million weights and row, rows rounded up
  // to 128, against ~0.29 per pass of the 64-row tile kernel: up to 320 rows that one is ahead; K = 8192, N = 28672 at
  // 191 / 192 rows: 203 us on it / 317 widened; K = 4096, N = 128256: 448 / 612)
  if (uint64_t(p.n) * p.k * 3 > (256ull << 20)) {
    const float passes = float((p.m + 63) / 64), rows = float((p.m + 127) / 128 * 128);
    if (passes * 0.29f < 0.75f + 0.0021f * rows) return 0;
  }
  const bool fits = (dtype == VKT_BF16 || dtype == VKT_F16) && p.m >= kQ8GemmRows && p.k % 16 == 0 && p.a % 16 == 0 && p.b % 16 == 0 &&
                    p.a_sm > 0 && p.a_sm % 8 == 0 && uint32_t(p.a_sm) >= p.k && p.a_sk == 1 && p.n > 0;
  return fits ? uint64_t(p.n) * p.k * 2 : 0;
}

int launch_q8_gemm(const Q8Params& p, int dtype, const Machine& mc, hipStream_t stream, std::string* err) {
  const int rc = dtype == VKT_BF16 ? launch_q8_gemm_t<bf16_t>(p, mc, stream, err) : launch_q8_gemm_t<f16_t>(p, mc, stream, err);
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "qmm8: kernel launch failed";
    return -1;
  }
  return rc;
}

int launch_gemm16(const GemmParams& p, int dtype, uint32_t use_cin, uint32_t batch, uint32_t variant, const Machine& mc,
                  hipStream_t stream, std::string* err) {
  if (p.m == 0 || p.n == 0 || batch == 0) return 0;
  if ((p.k != 0 && (!p.a || !p.b)) || !p.c || (use_cin && !p.cin)) {
    *err = "gemmcm: null tensor address";
    return -1;
  }
  if (use_cin > 1) {
    *err = "gemmcm: USE_CIN must be 0 or 1";
    return -1;
  }
  const int rc = dtype == VKT_BF16 ? launch_gemm16_t<bf16_t>(p, use_cin, batch, variant, mc, stream, err)
                                   : launch_gemm16_t<f16_t>(p, use_cin, batch, variant, mc, stream, err);
  if (rc == 0 && hipGetLastError() != hipSuccess) {
    *err = "gemmcm: kernel launch failed";
    return -1;
  }
  return rc;
}

}  // namespace vkt
