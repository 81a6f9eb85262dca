/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE.
 *
 * CPU restatement (plain C) of the arithmetic of torch-vulkan's quantized-matmul
 * path.  Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may
 * load this; the product path (the HIP library) never links or calls it.
 *
 * Build: gcc -O2 -ffp-contract=off -fno-fast-math (see oracle/Makefile).  Contraction
 * must stay off: the int4 path is specified without fused multiply-adds.
 *
 * Each function cites the reference file:line it follows.  Where the arithmetic
 * truth lives in PyTorch's CPU kernels (torch 2.14.1 pinned by the reference's
 * tools/torch-version; torch 2.10.0 importable here), the function restates the
 * published algorithm and the tests pin it against that torch CPU op.
 *
 * Pinning status (tests/test_oracle_*.py):
 *   orc_f32_to_{bf16,f16,e4m3fn,e5m2}, orc_fp8_to_f32  pinned: torch CPU casts (all 256
 *       codes, every halfway point between adjacent codes, saturation/NaN/-0)
 *   orc_qmm8            pinned: f64 closed form, torch CPU _weight_int8pack_mm,
 *                               brute-force tiny cases, column/row linearity
 *   orc_q4_pack         pinned: torch CPU _dyn_quant_pack_4bit_weight (bit-exact)
 *   orc_q4_rowquant     pinned: through orc_q4_matmul (bit-exact vs torch CPU) and
 *                               closed-form cases (constant rows, zero rows)
 *   orc_q4_matmul       pinned: torch CPU _dyn_quant_matmul_4bit (bit-exact), golden
 *   orc_scaled_mm       pinned: torch CPU _scaled_mm (per-tensor), f64 closed form,
 *                               identity / power-of-two cases that are exact
 *   orc_gemm16          pinned: float64 closed form by numpy, torch CPU float32 matmul of the same
 *                               16-bit values (inside the reference test's bound), exactly
 *                               representable cases (small integers, identity, powers of two)
 *   orc_cast            pinned: torch CPU Tensor.to() between float32 / float16 / bfloat16 and
 *                               both float8 formats (the reference's own vectors,
 *                               tests/python/test_fallback_ops.py:469-485, plus all 256 codes)
 *   orc_move            pinned: numpy strided views (as_strided) and torch CPU copy_ / contiguous() /
 *                               fill_ on the same layouts: transposes, slices, broadcasts, up to 8 dims
 *   orc_cast_strided    pinned: torch CPU Tensor.to() over the same strided views
 *   orc_quantize_affine, orc_dequantize_affine   pinned: torch CPU quantize_per_tensor / int_repr /
 *                               dequantize (the x86 FBGEMM build) for quint8, qint8, qint32 on random
 *                               values, every rounding tie, NaN, infinities and values beyond int32
 *   orc_fake_quant      pinned: torch CPU _fake_quantize_per_tensor_affine_cachemask_tensor_qparams and
 *                               fake_quantize_per_channel_affine_cachemask (int32 and float zero points)
 *                               on the same kinds of values, outputs and masks bit for bit
 *   orc_choose_qparams, orc_observe   pinned: torch CPU _fused_moving_avg_obs_fq_helper over several steps
 *                               (running min / max, scale, zero point and the fake-quantised output bit
 *                               for bit; per tensor and per row, symmetric or not, three averaging constants)
 *   orc_fp8_quant_rows  pinned: the same steps composed from torch CPU operators (amax, clamp,
 *                               true_divide, mul, clamp, to(float8)), rows whose maximum is
 *                               fmax exactly (the scale is 1: a plain cast), power-of-two
 *                               rescaling, zero rows
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { ORC_F32 = 0, ORC_F16 = 1, ORC_BF16 = 2, ORC_E4M3 = 3, ORC_E5M2 = 4 };

static inline uint32_t f2u(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float u2f(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ------------------------------------------------------------------ casts */

/* float32 -> bfloat16, round to nearest even, NaN -> 0x7fc0
 * (reference crates/vkcore/shaders/qmm8.slang:54-67, cast.slang:31-39). */
uint16_t orc_f32_to_bf16(float f) {
  if (isnan(f)) return 0x7fc0;
  uint32_t u = f2u(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

float orc_bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }

/* float32 -> IEEE binary16, round to nearest even (reference _half.slang:7-38 states
 * the same textbook conversion; equal to torch's .to(float16)). */
uint16_t orc_f32_to_f16(float f) {
  uint32_t u = f2u(f), sign = (u >> 16) & 0x8000u, mag = u & 0x7fffffffu;
  if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);        /* NaN */
  if (mag >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);       /* >= 65520 -> inf */
  if (mag < 0x33000001u) return (uint16_t)sign;                    /* <= 2^-25 -> 0 (tie to even) */
  int e = (int)(mag >> 23) - 127;
  uint32_t m = (mag & 0x7fffffu) | 0x800000u;
  int shift = e < -14 ? 13 + (-14 - e) : 13;                        /* bits dropped */
  uint32_t keep = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1u))) keep++;
  uint32_t out;
  if (e < -14) out = keep;                                          /* subnormal (may carry into normal) */
  else out = ((uint32_t)(e + 15) << 10) + (keep - 0x400u);          /* carry propagates into exponent */
  return (uint16_t)(sign | out);
}

float orc_f16_to_f32(uint16_t h) {
  uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 31u, m = h & 0x3ffu;
  if (e == 31) return u2f(sign | 0x7f800000u | (m << 13));
  if (e == 0) {
    float v = ldexpf((float)m, -24);
    return sign ? -v : v;
  }
  return u2f(sign | ((e + 112u) << 23) | (m << 13));
}

/* float8 -> float32 (exact).  e4m3fn: bias 7, no infinities, 0x7f/0xff NaN.
 * e5m2: bias 15, IEEE-like (reference backend.cpp:486-495 builds the same 256-entry
 * table from the CPU's conversion). */
float orc_fp8_to_f32(uint8_t c, int fmt) {
  int sign = c >> 7;
  float v;
  if (fmt == ORC_E4M3) {
    int e = (c >> 3) & 15, m = c & 7;
    if (e == 15 && m == 7) return u2f(0x7ff00000u | ((uint32_t)sign << 31)); /* c10 keeps the payload bits */
    v = e == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10);
  } else {
    int e = (c >> 2) & 31, m = c & 3;
    if (e == 31) return u2f(0x7f800000u | ((uint32_t)m << 21) | ((uint32_t)sign << 31)); /* inf, or NaN with payload */
    v = e == 0 ? ldexpf((float)m, -16) : ldexpf((float)(4 + m), e - 17);
  }
  return sign ? -v : v;
}

/* float32 -> float8 as c10 converts (c10/util/Float8_e4m3fn.h, Float8_e5m2.h;
 * reference backend.cpp:538-586 reproduces these through threshold tables):
 * round to nearest even; e4m3fn: magnitude >= 480 (first value that would round
 * beyond 448) or NaN -> 0x7f (NaN), no saturation; e5m2: overflow -> inf,
 * NaN -> 0x7f-class quiet NaN (0x7e | payload bit; c10 gives 0x7f for all NaNs
 * whose top mantissa bits are set; tests pin the canonical NaN only). */
uint8_t orc_f32_to_fp8(float f, int fmt) {
  uint32_t u = f2u(f), sign = (u >> 24) & 0x80u, mag = u & 0x7fffffffu;
  int mbits = fmt == ORC_E4M3 ? 3 : 2, bias = fmt == ORC_E4M3 ? 7 : 15;
  if (mag > 0x7f800000u) return (uint8_t)(sign | 0x7fu);
  if (fmt == ORC_E4M3) {
    if (mag >= 0x43f00000u) return (uint8_t)(sign | 0x7fu); /* >= 480 (incl. inf) -> NaN */
  } else {
    if (mag >= 0x47800000u) return (uint8_t)(sign | 0x7cu); /* >= 65536 (incl. inf) -> inf */
  }
  if (mag == 0) return (uint8_t)sign;
  int e = (int)(mag >> 23) - 127;
  uint32_t m = (mag & 0x7fffffu) | 0x800000u; /* 24-bit significand (flushes f32 denormals: far below range) */
  if ((mag >> 23) == 0) return (uint8_t)sign;
  int emin = 1 - bias;
  int shift = 23 - mbits + (e < emin ? emin - e : 0);
  if (shift > 25) return (uint8_t)sign;
  uint32_t keep = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (keep & 1u))) keep++;
  uint32_t out;
  if (e < emin) out = keep;
  else out = ((uint32_t)(e + bias) << mbits) + (keep - (1u << mbits));
  /* e5m2 values that round up to 2^16 become inf (0x7c) by the carry; e4m3fn's
   * largest finite 448 = 0x7e, rounding up from [464,480) gives 0x7f = NaN as c10. */
  return (uint8_t)(sign | out);
}

static float load_as_f32(const void* p, int64_t i, int dtype) {
  switch (dtype) {
    case ORC_F32: return ((const float*)p)[i];
    case ORC_F16: return orc_f16_to_f32(((const uint16_t*)p)[i]);
    case ORC_BF16: return orc_bf16_to_f32(((const uint16_t*)p)[i]);
    default: return orc_fp8_to_f32(((const uint8_t*)p)[i], dtype);
  }
}

static void store_from_f32(void* p, int64_t i, int dtype, float v) {
  switch (dtype) {
    case ORC_F32: ((float*)p)[i] = v; break;
    case ORC_F16: ((uint16_t*)p)[i] = orc_f32_to_f16(v); break;
    case ORC_BF16: ((uint16_t*)p)[i] = orc_f32_to_bf16(v); break;
    default: ((uint8_t*)p)[i] = orc_f32_to_fp8(v, dtype); break;
  }
}

/* ------------------------------------------------------------------ int8 weights */

/* aten::_weight_int8pack_mm as the reference computes it
 * (crates/pyvk/csrc/quant.cpp:59-119; crates/vkcore/shaders/qmm8.slang:78-111,113-173):
 * each weight dequantised per element to float32 as float(b) * float(scale) (one
 * rounding), products accumulated, the result rounded once to A's dtype.  The
 * reference's summation order is an implementation detail (its own test allows
 * eps*|want| + 2^-20 * sum|a||w|, tests/python/test_quant.py:36-37); this
 * restatement accumulates the float32-rounded per-element terms in float64 and
 * rounds once, i.e. it is the centre of that tolerance band.
 * a: [M,K] rows a_sm elements apart; b: int8 [N,K]; scales: [N] in A's dtype;
 * c: contiguous [M,N] in A's dtype; c64 (optional): the float64 sums; mag (optional):
 * sum_k |a||w| in float64 for the tolerance. */
void orc_qmm8(const void* a, int dtype, int64_t a_sm, const int8_t* b, const void* scales, void* c, double* c64,
              double* mag, int64_t M, int64_t N, int64_t K) {
  float* arow = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
  for (int64_t m = 0; m < M; m++) {
    for (int64_t k = 0; k < K; k++) arow[k] = load_as_f32(a, m * a_sm + k, dtype);
    for (int64_t n = 0; n < N; n++) {
      float s = load_as_f32(scales, n, dtype);
      double acc = 0.0, ab = 0.0;
      const int8_t* brow = b + n * K;
      for (int64_t k = 0; k < K; k++) {
        float w = (float)(int)brow[k] * s; /* qmm8.slang:89 */
        double t = (double)arow[k] * (double)w;
        acc += t;
        ab += fabs(t);
      }
      store_from_f32(c, m * N + n, dtype, (float)acc);
      if (c64) c64[m * N + n] = acc;
      if (mag) mag[m * N + n] = ab;
    }
  }
  free(arow);
}

/* The same with float32 accumulation in the reference's GEMV order
 * (qmm8.slang:87-109: lane l sums k = l, l+32, ...; the 32 partials are then added
 * serially in lane order), without contraction.  Used to show that an
 * implementation-order float32 sum sits inside the tolerance band. */
void orc_qmm8_f32order(const void* a, int dtype, int64_t a_sm, const int8_t* b, const void* scales, void* c,
                       int64_t M, int64_t N, int64_t K) {
  for (int64_t m = 0; m < M; m++)
    for (int64_t n = 0; n < N; n++) {
      float s = load_as_f32(scales, n, dtype), part[32];
      for (int l = 0; l < 32; l++) {
        float acc = 0.0f;
        for (int64_t k = l; k < K; k += 32) {
          float w = (float)(int)b[n * K + k] * s;
          acc = acc + load_as_f32(a, m * a_sm + k, dtype) * w;
        }
        part[l] = acc;
      }
      float sum = 0.0f;
      for (int l = 0; l < 32; l++) sum = sum + part[l];
      store_from_f32(c, m * N + n, dtype, sum);
    }
}

/* ------------------------------------------------------------------ int4 weights */

/* aten::_dyn_quant_pack_4bit_weight (reference quant.cpp:127-144): a float32 vector
 * cat(bytes -> f32, scales -> f32, bias -> f32).  scales_dtype: ORC_F32 or ORC_BF16.
 * Returns the number of floats written. */
int64_t orc_q4_pack(const uint8_t* w, int64_t nbytes, const void* scales, int scales_dtype, int64_t nscales,
                    const float* bias, int64_t nbias, float* out) {
  int64_t o = 0;
  for (int64_t i = 0; i < nbytes; i++) out[o++] = (float)w[i];
  for (int64_t i = 0; i < nscales; i++) out[o++] = load_as_f32(scales, i, scales_dtype);
  for (int64_t i = 0; i < nbias; i++) out[o++] = bias[i];
  return o;
}

/* std::round (halfway away from zero), reference qmm4.slang:112-118. */
static float round_away(float x) {
  float t = truncf(x);
  if (fabsf(x - t) >= 0.5f) t += x < 0.0f ? -1.0f : 1.0f;
  return t;
}

/* Row quantisation, reference qmm4.slang:132-181 (PHASE 0): asymmetric int8 per row.
 * x: [M,K] (f32 or bf16); q: int32 [M,K]; recip: [M] = 1/scale; nzp: [M] = -zero_point.
 * IEEE binary32 throughout, '/' correctly rounded (what div_exact, :89-109, achieves),
 * zero point rounded half-to-even (m_round_even, _fmath.slang:540-547). */
void orc_q4_rowquant(const void* x, int dtype, int64_t M, int64_t K, int groupwise, int32_t* q, float* recip,
                     int32_t* nzp) {
  const float qmin = -128.0f, qmax = 127.0f;
  for (int64_t m = 0; m < M; m++) {
    float mn = 3.40282347e38f, mx = -3.40282347e38f;
    for (int64_t k = 0; k < K; k++) {
      float v = load_as_f32(x, m * K + k, dtype);
      mn = fminf(mn, v);
      mx = fmaxf(mx, v);
    }
    float rmin = fminf(0.0f, mn), rmax = fmaxf(0.0f, mx);
    float scale = rmin == rmax ? 1.0f : (qmax - qmin) / (rmax - rmin);
    float rc = scale != 0.0f ? 1.0f / scale : 0.0f;
    float dmin = rmin * scale, dmax = rmax * scale;
    float err = groupwise ? ((qmin + dmin) + qmax) + dmax : (qmin + dmin) + (qmax + dmax);
    float zp = err > 0.0f ? qmin - dmin : qmax - dmax;
    zp = fminf(fmaxf(zp, qmin), qmax);
    int32_t izp = (int32_t)nearbyintf(zp);
    recip[m] = rc;
    nzp[m] = -izp;
    for (int64_t k = 0; k < K; k++) {
      int32_t v = (int32_t)round_away(load_as_f32(x, m * K + k, dtype) * scale) + izp;
      q[m * K + k] = v < -128 ? -128 : (v > 127 ? 127 : v);
    }
  }
}

/* aten::_dyn_quant_matmul_4bit, reference quant.cpp:146-204 + qmm4.slang:183-247
 * (PHASE 1).  packed: float32 vector [bytes | scales | bias]; out: [M,N] in x's dtype
 * (bf16 stored by truncation, :244).  iacc_out (optional): int32 [M,N,nblocks] block
 * sums, the integer accumulators the contract calls bit-exact. */
void orc_q4_matmul(const void* x, int dtype, const float* packed, int64_t packed_numel, int64_t M, int64_t K,
                   int64_t N, int64_t bs, void* out, int32_t* iacc_out) {
  int groupwise = bs != K;
  int64_t rstride = (K + 1) / 2, wcount = N * K / 2, nblocks = (K + bs - 1) / bs;
  int has_bias = packed_numel - (wcount + N * (K / bs)) != 0;
  int32_t* q = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M * K > 0 ? M * K : 1));
  float* recip = (float*)malloc(sizeof(float) * (size_t)(M > 0 ? M : 1));
  int32_t* nzp = (int32_t*)malloc(sizeof(int32_t) * (size_t)(M > 0 ? M : 1));
  orc_q4_rowquant(x, dtype, M, K, groupwise, q, recip, nzp);
  const float hi = dtype == ORC_BF16 ? 3.38953139e38f : 3.40282347e38f;
  for (int64_t m = 0; m < M; m++)
    for (int64_t n = 0; n < N; n++) {
      float acc = 0.0f;
      for (int64_t blk = 0; blk < nblocks; blk++) {
        int32_t iacc = 0;
        int64_t k1 = (blk + 1) * bs < K ? (blk + 1) * bs : K;
        for (int64_t k = blk * bs; k < k1; k++) {
          uint32_t byte = (uint32_t)packed[n * rstride + k / 2];
          int32_t w = (int32_t)((byte >> (4 * (k & 1))) & 15u) - 8;
          iacc += q[m * K + k] * w;
          iacc += nzp[m] * w;
        }
        if (iacc_out) iacc_out[(m * N + n) * nblocks + blk] = iacc;
        float t = (float)iacc * packed[wcount + n * nblocks + blk];
        acc = blk == 0 ? t : acc + t; /* :225-226: the first block assigns (keeps -0) */
      }
      acc = acc * recip[m];
      if (has_bias) acc = acc + packed[wcount + N * nblocks + n];
      acc = acc < -hi ? -hi : acc; /* NaN passes, :236-242 */
      acc = hi < acc ? hi : acc;
      if (dtype == ORC_BF16) ((uint16_t*)out)[m * N + n] = (uint16_t)(f2u(acc) >> 16);
      else ((float*)out)[m * N + n] = acc;
    }
  free(q);
  free(recip);
  free(nzp);
}

/* ------------------------------------------------------------------ float8 */

/* aten::_scaled_mm as the reference computes it (quant.cpp:279-300): exact upcasts,
 * a = f32(mat1) * scale_a, b = f32(mat2) * scale_b in float32, out_tmp = a @ b
 * (+ bias), * (1 / scale_result) when the output is float8, cast once.
 * a: fp8 [M,K] row-major (fmt_a); bt: fp8 [N,K] row-major = mat2 column-major (fmt_b);
 * sa: [1] or [M]; sb: [1] or [N] (rowwise != 0); bias: [N] in bias_dtype or NULL;
 * scale_result: pointer to one float or NULL; out: [M,N] in out_dtype.
 * The float32 product's summation order is open (test_quant.py:124-126 allows
 * eps*|want| + 2^-20*mag): sums are carried in float64 and rounded to float32 once.
 * mag (optional): sum_k |a||b| (float64). */
void orc_scaled_mm(const uint8_t* a, int fmt_a, const uint8_t* bt, int fmt_b, const float* sa, const float* sb,
                   int rowwise, const void* bias, int bias_dtype, const float* scale_result, void* out,
                   int out_dtype, double* mag, int64_t M, int64_t N, int64_t K) {
  float ta[256], tb[256];
  for (int i = 0; i < 256; i++) {
    ta[i] = orc_fp8_to_f32((uint8_t)i, fmt_a);
    tb[i] = orc_fp8_to_f32((uint8_t)i, fmt_b);
  }
  float* arow = (float*)malloc(sizeof(float) * (size_t)(K > 0 ? K : 1));
  int out_fp8 = out_dtype == ORC_E4M3 || out_dtype == ORC_E5M2;
  float inv = 1.0f;
  if (out_fp8) inv = 1.0f / (scale_result ? *scale_result : 1.0f);
  for (int64_t m = 0; m < M; m++) {
    float s1 = rowwise ? sa[m] : sa[0];
    for (int64_t k = 0; k < K; k++) arow[k] = ta[a[m * K + k]] * s1;
    for (int64_t n = 0; n < N; n++) {
      float s2 = rowwise ? sb[n] : sb[0];
      double acc = 0.0, ab = 0.0;
      const uint8_t* brow = bt + n * K;
      for (int64_t k = 0; k < K; k++) {
        float bv = tb[brow[k]] * s2;
        double t = (double)arow[k] * (double)bv;
        acc += t;
        ab += fabs(t);
      }
      float r = (float)acc;
      if (bias) r = r + load_as_f32(bias, n, bias_dtype);
      if (out_fp8) r = r * inv;
      store_from_f32(out, m * N + n, out_dtype, r);
      if (mag) mag[m * N + n] = ab;
    }
  }
  free(arow);
}

/* ------------------------------------------------------------------ float8 casts and producer */

/* Elementwise conversion where one side is float8: through float32, as the reference's copy
 * between a float8 tensor and a float tensor (crates/pyvk/csrc/backend.cpp:534-586, tables
 * built from c10's conversions) and as c10 itself converts. */
void orc_cast(const void* src, int src_dtype, void* dst, int dst_dtype, int64_t n) {
  for (int64_t i = 0; i < n; i++) store_from_f32(dst, i, dst_dtype, load_as_f32(src, i, src_dtype));
}

/* Strided data movement by element size (crates/vkcore/shaders/move.slang:37-52 with the index
 * arithmetic of _strided.slang:68-86, copy8.slang:36-66): linear index i is split into per-dim
 * coordinates, innermost dim first; out[sum c so] = a[sum c sa] (fill = 0) or the fill value.
 * Strides in elements of `item` bytes. */
void orc_move(uint8_t* out, const uint8_t* a, int64_t item, int64_t n, int ndim, const int64_t* size, const int64_t* so,
              const int64_t* sa, int fill, const uint8_t* value) {
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i, o = 0, s = 0;
    for (int d = 0; d < ndim; d++) {
      const int64_t c = rem % size[d];
      rem /= size[d];
      o += c * so[d];
      if (!fill) s += c * sa[d];
    }
    memcpy(out + o * item, fill ? value : a + s * item, (size_t)item);
  }
}

/* out = dst_dtype(a) over the same index space (crates/vkcore/shaders/cast.slang: through
 * float32, round to nearest even); strides in elements of each side. */
void orc_cast_strided(void* out, int dst_dtype, const void* a, int src_dtype, int64_t n, int ndim, const int64_t* size,
                      const int64_t* so, const int64_t* sa) {
  for (int64_t i = 0; i < n; i++) {
    int64_t rem = i, o = 0, s = 0;
    for (int d = 0; d < ndim; d++) {
      const int64_t c = rem % size[d];
      rem /= size[d];
      o += c * so[d];
      s += c * sa[d];
    }
    store_from_f32(out, o, dst_dtype, load_as_f32(a, s, src_dtype));
  }
}

/* ------------------------------------------------------------------ per-tensor affine quantised tensors */

enum { ORC_QUINT8 = 0, ORC_QINT8 = 1, ORC_QINT32 = 2 };

/* quantize_per_tensor as PyTorch's x86 CPU build computes it (FBGEMM's Quantize), restated from the
 * reference's composition (crates/pyvk/csrc/quantized.cpp:72-116):
 *   8-bit: t = x * (1.0f / scale) clipped at the largest float below 2^31 (a NaN too), rounded to
 *          nearest even as int32 (below -2^31: INT32_MIN), plus the zero point (wrapping), clamped;
 *   qint32: float(nearbyint(t) + zero_point), a NaN -> qmin, clamped. */
void orc_quantize_affine(const float* x, int64_t n, float scale, int32_t zero_point, int qtype, void* out) {
  const float inv = 1.0f / scale;
  for (int64_t i = 0; i < n; i++) {
    const float t = x[i] * inv;
    if (qtype == ORC_QINT32) {
      const float r = nearbyintf(t) + (float)zero_point;
      int64_t q;
      if (isnan(r)) q = INT32_MIN;
      else if (r >= 2147483648.0f) q = INT32_MAX;
      else if (r <= -2147483648.0f) q = INT32_MIN;
      else q = (int64_t)r;
      ((int32_t*)out)[i] = (int32_t)q;
      continue;
    }
    const float top = 2147483520.0f;
    const float tc = isnan(t) ? top : (t < top ? t : top);
    const float r = nearbyintf(tc);
    const int64_t base = r < -2147483648.0f ? (int64_t)INT32_MIN : (int64_t)r;
    int32_t q = (int32_t)(uint32_t)(uint64_t)(base + zero_point); /* (wraps as the int32 add does) */
    const int32_t lo = qtype == ORC_QUINT8 ? 0 : -128, hi = qtype == ORC_QUINT8 ? 255 : 127;
    q = q < lo ? lo : (q > hi ? hi : q);
    if (qtype == ORC_QUINT8) ((uint8_t*)out)[i] = (uint8_t)q;
    else ((int8_t*)out)[i] = (int8_t)q;
  }
}

/* dequantize: scale * float(q - zero_point), the difference in wrapping int32
 * (crates/pyvk/csrc/quantized.cpp:123-130). */
void orc_dequantize_affine(const void* q, int qtype, int64_t n, float scale, int32_t zero_point, float* out) {
  for (int64_t i = 0; i < n; i++) {
    const int32_t v = qtype == ORC_QUINT8 ? ((const uint8_t*)q)[i] : qtype == ORC_QINT8 ? ((const int8_t*)q)[i] : ((const int32_t*)q)[i];
    const int32_t d = (int32_t)((uint32_t)v - (uint32_t)zero_point);
    out[i] = (float)d * scale;
  }
}

/* Fake quantisation with its mask (python/torch_vulkan/_kernels.py:1613-1630, which restates ATen's CPU
 * kernels).  x: float32 values of element type dtype's tensor; element i belongs to channel
 * (i / inner) % channels.  scales float32 [channels]; zero points int32 (zp_float 0) or float32 (1).
 *   per tensor (per_channel 0): q = nearbyint(x * inv) + zp in float32; mask = qmin <= q <= qmax;
 *       a NaN q counts as qmin; out = (clamp(q) - zp) * scale.
 *   per channel: q is converted to int64 before the mask and the clamp (as ATen does): a q that
 *       int64 cannot hold (NaN, infinities, |q| >= 2^63) becomes INT64_MIN, so qmin; with a float zero
 *       point q = lrintf(zp + x * inv), which PyTorch's x86 build evaluates as one fused multiply-add
 *       (measured: 7 of 8 million random values differ otherwise; the reference's composition rounds the
 *       product first); the output is computed in double and rounded once.
 * The output is rounded to dtype. */
void orc_fake_quant(const void* x, int dtype, int64_t n, const float* scales, const void* zps, int zp_float,
                    int64_t channels, int64_t inner, int per_channel, int64_t qmin, int64_t qmax, void* out,
                    uint8_t* mask) {
  for (int64_t i = 0; i < n; i++) {
    const int64_t c = per_channel ? (i / inner) % channels : 0;
    const float sc = scales[c], inv = 1.0f / sc; /* (a zero scale divides to infinity, as the CPU's) */
    const float zp = zp_float ? ((const float*)zps)[c] : (float)((const int32_t*)zps)[c];
    const float v = load_as_f32(x, i, dtype);
    float q;
    if (per_channel && zp_float) q = nearbyintf(fmaf(v, inv, zp)); /* (one rounding: see above) */
    else q = nearbyintf(v * inv) + zp;
    int inside;
    float result;
    if (per_channel) {
      const int fits = q > -9223372036854775808.0f && q < 9223372036854775808.0f; /* (false for a NaN) */
      const int64_t qi = fits ? (int64_t)q : INT64_MIN;
      inside = qi >= qmin && qi <= qmax;
      const int64_t qc = qi < qmin ? qmin : (qi > qmax ? qmax : qi);
      /* (ATen clamps with fmin / fmax, i.e. in double, and stays there: one rounding at the end) */
      result = (float)(((double)qc - (double)zp) * (double)sc);
    } else {
      inside = q >= (float)qmin && q <= (float)qmax;
      const float qc = isnan(q) ? (float)qmin : (q < (float)qmin ? (float)qmin : (q > (float)qmax ? (float)qmax : q));
      result = (qc - zp) * sc;
    }
    store_from_f32(out, i, dtype, result);
    mask[i] = (uint8_t)inside;
  }
}

/* Quantisation parameters from a range, as the CPU chooses them (ATen's
 * quant_utils::ChooseQuantizationParams, restated by the reference in
 * python/torch_vulkan/_kernels.py:1678-1716): the float32 and double steps as written there.
 * Returns 0, or -1 where ATen raises (min above max). */
int orc_choose_qparams(float mn, float mx, int32_t qmin, int32_t qmax, int preserve_sparsity, float* scale_out,
                       int32_t* zp_out) {
  if (!(mn <= mx)) return -1;
  if (mn < 0 && mx > 0 && preserve_sparsity) {
    const int32_t sqmin = -((qmax - qmin) / 2 + 1), sqmax = (qmax - qmin) / 2;
    const double a = fabs((double)(mn / (float)sqmin)), b = fabs((double)(mx / (float)sqmax));
    const double max_scale = a > b ? a : b;
    mn = (float)(max_scale * sqmin), mx = (float)(max_scale * sqmax);
  }
  mn = mn < 0.0f ? mn : 0.0f, mx = mx > 0.0f ? mx : 0.0f;
  /* (the difference in double, the scale itself a float32: what the zero point below is derived from.
   * torch 2.10's CPU build behaves so: ranges [-a, a] put the zero point on a tie that tells the two apart;
   * the reference's restatement keeps the scale in double) */
  float scale = (float)(((double)mx - (double)mn) / (double)(qmax - qmin));
  if (scale == 0.0f || isinf(1.0f / scale)) scale = 0.1f;
  const float small = 6.1e-5f;
  if (scale < small) {
    const float org = scale;
    scale = small;
    if (mn == 0.0f) mx = small * (float)(qmax - qmin);
    else if (mx == 0.0f) mn = -small * (float)(qmax - qmin);
    else {
      const float amp = small / org;
      mn = mn * amp, mx = mx * amp;
    }
  }
  const double z_min = qmin - (double)mn / (double)scale, z_max = qmax - (double)mx / (double)scale;
  const double e_min = fabs((double)qmin) - fabs((double)mn / (double)scale), e_max = fabs((double)qmax) - fabs((double)mx / (double)scale);
  double z = e_min < e_max ? z_min : z_max;
  if (mn < 0 && mx > 0 && preserve_sparsity) z = (qmin + qmax) / 2.0;
  *zp_out = z < qmin ? qmin : (z > qmax ? qmax : (int32_t)nearbyint(z));
  *scale_out = scale;
  return 0;
}

/* One observer step on the running range (python/torch_vulkan/_kernels.py:1740-1750): a running value that
 * is still infinite takes this batch's, otherwise run + c * (cur - run) in single float32 operations. */
void orc_observe(float* run_min, float* run_max, const float* cur_min, const float* cur_max, int64_t n, float c) {
  for (int64_t i = 0; i < n; i++) {
    run_min[i] = isinf(run_min[i]) ? cur_min[i] : run_min[i] + c * (cur_min[i] - run_min[i]);
    run_max[i] = isinf(run_max[i]) ? cur_max[i] : run_max[i] + c * (cur_max[i] - run_max[i]);
  }
}

/* The float8 producer in front of _scaled_mm (no counterpart in the reference: the step a float8
 * pipeline needs on the device before the product).  Per row, or with one given scale:
 *   a = max(max_k |x|, 1e-12) (NaN elements do not count); scale = a / fmax;
 *   q = cast(clamp(x * (fmax / a), -fmax, fmax)); every step one float32 operation.
 * rowwise 0: scales[0] is an input and a = scales[0] * fmax. */
void orc_fp8_quant_rows(const void* x, int dtype, int64_t M, int64_t K, int64_t ldx, int fmt, int rowwise, uint8_t* q,
                        int64_t ldq, float* scales) {
  const float fmax = fmt == ORC_E4M3 ? 448.0f : 57344.0f;
  for (int64_t m = 0; m < M; m++) {
    float a;
    if (rowwise) {
      float amax = 0.0f;
      for (int64_t k = 0; k < K; k++) {
        const float v = fabsf(load_as_f32(x, m * ldx + k, dtype));
        if (v > amax) amax = v; /* (a NaN compares false) */
      }
      a = amax > 1e-12f ? amax : 1e-12f;
      scales[m] = a / fmax;
    } else {
      a = scales[0] * fmax;
    }
    const volatile float inv = fmax / a;
    for (int64_t k = 0; k < K; k++) {
      volatile float y = load_as_f32(x, m * ldx + k, dtype) * inv;
      if (y < -fmax) y = -fmax;
      if (fmax < y) y = fmax;
      q[m * ldq + k] = orc_f32_to_fp8(y, fmt);
    }
  }
}

/* ------------------------------------------------------------------ 16-bit matrix product */

/* C[b] = alpha * A[b] @ B[b] (+ beta * Cin[b]) for bfloat16 / float16 operands as the reference's
 * cooperative-matrix kernel specifies it (crates/vkcore/shaders/gemmcm.slang:293-310,
 * crates/pyvk/csrc/linalg.cpp:227-255): products accumulated in float32, alpha and beta
 * applied in float32, one rounding to the 16-bit type.  The summation order is an
 * implementation detail (the reference's test allows eps*|want| + 2^-20 * sum|a||b|,
 * tests/python/test_matmul.py:250-264); this restatement sums in float64, the centre of that
 * band.  Strides in elements (any sign, 0 for a broadcast Cin); mag (optional) receives
 * |alpha| sum|a||b| + |beta||cin|. */
void orc_gemm16(const void* a, const void* b, const void* cin, void* c, int dtype, int64_t B, int64_t M, int64_t N, int64_t K,
                const int64_t* sa, const int64_t* sb, const int64_t* sc, const int64_t* scin, float alpha, float beta,
                double* mag) {
  for (int64_t bb = 0; bb < B; bb++)
    for (int64_t m = 0; m < M; m++)
      for (int64_t n = 0; n < N; n++) {
        double acc = 0.0, am = 0.0;
        for (int64_t k = 0; k < K; k++) {
          const double x = load_as_f32(a, bb * sa[0] + m * sa[1] + k * sa[2], dtype);
          const double y = load_as_f32(b, bb * sb[0] + k * sb[1] + n * sb[2], dtype);
          acc += x * y;
          am += fabs(x * y);
        }
        double v = (double)alpha * acc, vm = fabs((double)alpha) * am;
        if (cin) {
          const double ci = load_as_f32(cin, bb * scin[0] + m * scin[1] + n * scin[2], dtype);
          v += (double)beta * ci;
          vm += fabs((double)beta * ci);
        }
        store_from_f32(c, bb * sc[0] + m * sc[1] + n * sc[2], dtype, (float)v);
        if (mag) mag[(bb * M + m) * N + n] = vm;
      }
}
