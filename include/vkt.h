/*
 * C ABI of the MI355X (gfx950) runtime for torch-vulkan's quantized-matmul path.
 *
 * The first block reproduces, name for name and argument for argument, the C ABI the
 * reference's C++ backend binds (reference crates/pyvk/csrc/vk.h:49-69, implemented in
 * Rust at crates/pyvk/src/ffi.rs:42-206).  A backend built against those declarations
 * links against this library unchanged.  Conventions (ffi.rs:1-28): every fallible
 * function returns 0 on success and -1 on failure; the message of the last failure on
 * the calling thread is returned by vkt_last_error().
 *
 * Differences that follow from HIP (device memory is not host-mapped):
 *   - VktAlloc.host is always NULL; VktAlloc.address is the device pointer.
 *   - host <-> device transfers go through vkt_copy_* (second block).
 *   - vkt_dispatch takes the grid for signature compatibility; for the kernels of this
 *     path the launch geometry is planned by the library from the parameter block
 *     (a grid of 0 workgroups in any dimension is still an error, as in the reference).
 *
 * The parameter blocks ("push constants", at most 128 bytes, copied at call time) are
 * declared at the end; Q8Params and Q4Params keep the reference's layouts
 * (crates/pyvk/csrc/quant.cpp:31-43).
 */
#ifndef VKT_H
#define VKT_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---------------------------------------------------------------- reference C ABI */

/* vk.h:50-55 / ffi.rs:31-40 */
typedef struct VktAlloc {
  void* handle;     /* opaque, pass to vkt_free */
  uint8_t* host;    /* NULL: HBM is not host-mapped */
  uint64_t address; /* device address of the first byte (256-byte aligned) */
  uint64_t size;    /* usable bytes (>= the request) */
} VktAlloc;

const char* vkt_last_error(void);                                  /* vk.h:56, ffi.rs:42-45 */
int vkt_alloc(uint64_t nbytes, VktAlloc* out);                     /* vk.h:57, ffi.rs:47-60 */
void vkt_free(void* handle);                                       /* vk.h:58, ffi.rs:62-72 (no-op after shutdown) */
int vkt_synchronize(void);                                         /* vk.h:59, ffi.rs:74-80 */
int vkt_empty_cache(void);                                         /* vk.h:60, ffi.rs:82-95 */
void vkt_memory_stats(uint64_t* allocated, uint64_t* reserved);    /* vk.h:61, ffi.rs:97-110 */
/* vk.h:62-63, ffi.rs:112-142: queue kernel `name` specialised with spec[0..nspec),
 * parameters push[0..npush), asynchronously and in order with all earlier work. */
int vkt_dispatch(const char* name, const uint32_t* spec, size_t nspec, const uint8_t* push, size_t npush, uint32_t gx,
                 uint32_t gy, uint32_t gz);
int vkt_grid_1d(uint64_t n, uint32_t* groups, uint32_t* stride);   /* vk.h:64, ffi.rs:150-162 */
int vkt_has_float64(void);                                         /* vk.h:65, ffi.rs:164-168 */
uint32_t vkt_vendor_id(void);                                      /* vk.h:66, ffi.rs:170-174 (0x1002) */
uint32_t vkt_capabilities(void);                                   /* vk.h:67, ffi.rs:190-206 (Feature bits, vk.h:92-101) */
uint32_t vkt_kernel_subgroup_size(const char* name);               /* vk.h:68, ffi.rs:176-188 (64 for this path's kernels) */

/* ---------------------------------------------------------------- HIP additions */

/* Blocking transfers, ordered after all queued work (the reference memcpy()s through
 * VktAlloc.host after vkt_synchronize(): backend.cpp:692-699,781-788). */
int vkt_copy_to_device(uint64_t dst_address, const void* src, uint64_t nbytes);
int vkt_copy_to_host(void* dst, uint64_t src_address, uint64_t nbytes);
/* Queued (asynchronous, in order) device copy and byte fill. */
int vkt_copy_on_device(uint64_t dst_address, uint64_t src_address, uint64_t nbytes);
int vkt_fill(uint64_t dst_address, uint8_t value, uint64_t nbytes);

/* Device facts for rooflines and planning. */
typedef struct VktDeviceInfo {
  char name[64];      /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
  uint32_t compute_units;
  uint32_t clock_khz; /* maximum engine clock */
  uint32_t mem_clock_khz;
  uint32_t mem_bus_bits;
  uint64_t hbm_bytes;
  uint32_t lds_bytes_per_block;
  uint32_t l2_bytes;
} VktDeviceInfo;
int vkt_device_info(VktDeviceInfo* out);

/* Timing on the stream the kernels run on (HIP events). */
int vkt_event_create(void** event);
int vkt_event_record(void* event);
int vkt_event_elapsed_ms(void* start, void* stop, float* ms); /* waits for `stop` */
void vkt_event_destroy(void* event);

/* vkt_dispatch for callers that cannot allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid it).  No counterpart in the reference.  Same arguments, same kernels, same results; the
 * difference is where the kernels' own workspace lives (the partial sums of a product that is split over
 * workgroups, e.g. "qmm8_bf16" at 64 rows): here it is a fixed array of VKT_STATIC_SCRATCH_BYTES in the library's
 * code object, one per device, held until the process ends, and the call makes no hipMalloc / hipFree (vkt_dispatch
 * takes its workspace from the pool at its first call and grows a second region for many-row int8 products).
 *   - The runtime must be running: call any other function (e.g. vkt_device_info) once at start-up.
 *   - A product whose planned split needs more workspace than the array holds returns -1 with a message that
 *     names both sizes; it is never re-planned with fewer slices.  Many-row int8 products do not widen their
 *     weights here: they run on the row-block kernels.
 *   - Calls are queued on the runtime's one in-order stream like every other dispatch, so two calls never overlap on
 *     the device; the array keeps the last call's partial sums, and every kernel writes what it later reads (nothing
 *     has to start at zero). */
#define VKT_STATIC_SCRATCH_BYTES (16u << 20)
int vkt_dispatch_static(const char* name, const uint32_t* spec, size_t nspec, const uint8_t* push, size_t npush,
                        uint32_t gx, uint32_t gy, uint32_t gz);

uint64_t vkt_dispatch_count(void); /* kernels queued so far (reference pyvk/src/lib.rs:112-116) */
void vkt_shutdown(void);           /* releases the device; later vkt_free calls are no-ops */

/* Bytes of the compact int4 side-car that "qmm4c_pack" writes for an [N,K] weight with
 * blocks of `bs` (0 if the shape has no compact form). */
uint64_t vkt_qmm4c_bytes(uint32_t n, uint32_t k, uint32_t bs);
/* Bytes of the activation scratch (`q` of Q4CParams) for m rows of k values. */
uint64_t vkt_qmm4c_q_bytes(uint32_t m, uint32_t k);

/* ---------------------------------------------------------------- parameter blocks */

/* "qmm8_f32" | "qmm8_f16" | "qmm8_bf16", spec {ROWS}: C = A @ (B * scales).T
 * (quant.cpp:31-37, qmm8.slang:21-33).  56 bytes.  ROWS is 0 or m.  An optional second entry overrides the
 * launcher's choice of kernel and shape (tests, tuning; 0 or absent: planned): bits 0-7 columns per wave or
 * column tiles per workgroup, 8-15 waves that split K, 24+ slices of K over workgroups; bit 16 the any-shape
 * kernel, 17 the vector-unit kernels, 18 / 19 the matrix-core kernel with / without staging through LDS, 20 no
 * widened-weights product for many rows, 21 / 22 the 64 x 128 tile kernel forced / off; one row: bit 23 keeps the
 * kernel with a workgroup per pair of columns, bits 8-11 / 12-15 (bits 0-7 clear) ask for the persistent streaming
 * kernel with that many workgroups per compute unit / rows per iteration; 3 to 8 rows: bit 23 keeps the slice
 * kernels where the planner would take the kernel whose waves own column groups (large products), bits 8-15 (bits
 * 0-7 clear) ask for that kernel whatever the size; float32 activations, 2 to 16 rows: exactly bit 18 / bit 19 asks for /
 * keeps off the path that splits the rows into bfloat16 planes for the staged matrix-core kernel. */
typedef struct Q8Params {
  uint64_t a, b, scales, c; /* A [m,k] (row stride a_sm, a_sk must be 1), B int8 [n,k], scales [n], C [m,n] */
  uint32_t m, n, k;
  int32_t a_sm, a_sk; /* in elements */
  uint32_t pad;
} Q8Params;

/* "qmm4_f32" | "qmm4_bf16", spec {PHASE, GROUPWISE} (quant.cpp:39-43, qmm4.slang:34-47).
 * PHASE 0 quantises the rows of inp into q (int32 [m,k]) and rows ([m,2]: bits of
 * 1/scale, -zero_point); PHASE 1 multiplies with the float32-expanded packed weights.
 * 64 bytes. */
typedef struct Q4Params {
  uint64_t inp, q, rows, packed, out;
  uint32_t m, n, k, bs, has_bias, pad;
} Q4Params;

/* "qmm4_packvec", spec {}: aten::_dyn_quant_pack_4bit_weight (quant.cpp:127-144): the
 * float32 vector cat(weights bytes -> f32, scales -> f32, bias -> f32), in one kernel. */
typedef struct Q4VecParams {
  uint64_t weights, scales, bias, out; /* bias may be 0 */
  uint32_t nw, ns, nb;                 /* element counts */
  uint32_t scales_dtype, bias_dtype;   /* VKT_F32 | VKT_F16 | VKT_BF16 */
  uint32_t pad;
} Q4VecParams;

/* "qmm4c_pack", spec {LAYOUT}: packed float32 vector -> compact side-car (two nibbles per
 * byte, float32 scales, bias; vkt_qmm4c_bytes bytes) in one of two layouts:
 *   LAYOUT 0  for the streaming kernel (v_dot8_i32_i4; at most 4 rows per launch: the
 *             decode case)
 *   LAYOUT 1  for the matrix-core kernel (v_mfma_i32_16x16x32_i8; tiles of 16 rows).
 * A side-car serves only products of the layout it was packed for. */
typedef struct Q4PackParams {
  uint64_t packed, compact;
  uint32_t n, k, bs, has_bias;
} Q4PackParams;

/* "qmm4c_f32" | "qmm4c_bf16", spec {PHASE, GROUPWISE, LAYOUT}: as qmm4, over the compact
 * side-car of that LAYOUT.  PHASE 0 writes the quantised activations into q
 * (vkt_qmm4c_q_bytes; the arrangement differs per layout) and rows; PHASE 1 is the
 * product; PHASE 2 does both: with LAYOUT 0 in one launch per 4 rows where the rows can
 * be quantised from registers (k a multiple of 8, at most 16384), otherwise as PHASE 0
 * then 1.  Results are bit-identical to qmm4.  With LAYOUT 1, bits 4-7 of PHASE override the choice
 * between the two product kernels, which give the same bits (tests, tuning): 16 keeps the kernel whose four waves
 * split K, 32 forces the one whose waves each walk all of K (| 64, 128, 192: 1, 2, 4 tiles of 16 x 16 per wave).
 * With LAYOUT 0, PHASE 2 with 1, 2 or 3 in bits 8-9 fixes the column tiles per workgroup (same bits). */
typedef struct Q4CParams {
  uint64_t inp, q, rows, compact, out;
  uint32_t m, n, k, bs, has_bias, pad;
} Q4CParams;

/* "gemmcm_bf16" | "gemmcm_f16", spec {USE_CIN, (ignored), (ignored), VARIANT}; grid z = batches:
 * C[b] = alpha * A[b] @ B[b] (+ beta * Cin[b] when USE_CIN), 16-bit operands, float32
 * accumulation, one rounding (the reference's block, linalg.cpp:25-34, and kernel,
 * shaders/gemmcm.slang).  Strides in elements; alpha and beta hold float32 bits in their low
 * words.  112 bytes.  VARIANT (tests, tuning; 0: planned): 1-5 tile shapes, 6 the stream kernel, 7 the few-row kernel
 * (x @ w.T with up to 64 rows; bits 8-11: 16s of columns per workgroup, bits 12-16: slices of K over workgroups), 8 the
 * vector-unit kernel (x @ w.T, up to 4 rows), 9 the few-row kernel for weights stored [k, n] (x @ w with up to 64 rows;
 * bits 12-16: slices of K), 10 the 128 x 128 tile kernel with K in slices over workgroups (x @ w.T; bits 8-12: slices,
 * which must divide k's steps of 64 values), 255 one thread per output.  Batches of few-row products take the few-row
 * kernels too. */
typedef struct GemmParams {
  uint64_t a, b, c, cin;
  uint64_t alpha, beta;
  uint32_t m, n, k, pad;
  int32_t a_sm, a_sk, a_sb;
  int32_t b_sk, b_sn, b_sb;
  int32_t c_sm, c_sn, c_sb;
  int32_t cin_sm, cin_sn, cin_sb;
} GemmParams;

/* "move_b1" | "move_b2" | "move_b4" | "move_b8" | "move_b16", spec {OP}: data movement by
 * element size, strided (the reference's block, launch.cpp:18-27, and kernel, shaders/move.slang).
 *   OP VKT_MOVE_COPY  out[sum c_d so[d]] = a[sum c_d sa[d]] over 0 <= c_d < size[d]
 *   OP VKT_MOVE_FILL  out[...] = the value whose bits are in alpha (and beta for 16 bytes)
 * Dims innermost first, ndim <= 4, n = product of the sizes, strides in elements (0 =
 * broadcast); b, sb, gamma and stride are not used (the library sizes its own grid).  The
 * gather / scatter opcodes of the reference are not built.
 * Also "cast_<src>_<dst>" with src, dst in f32 | f16 | bf16, spec {}: out = dst(a) over the same
 * block (shaders/cast.slang: through float32, round to nearest even).  128 bytes. */
typedef struct StridedParams {
  uint64_t out, a, b;
  uint64_t alpha, beta, gamma;
  uint32_t n, ndim, stride, pad;
  uint32_t size[4];
  int32_t so[4], sa[4], sb[4];
} StridedParams;

/* "copy8_b1" ... "copy8_b16", spec {}: out = a, strided over up to 8 dims (the reference's
 * block, launch.cpp:84-90, and kernel, shaders/copy8.slang).  128 bytes. */
typedef struct Copy8Params {
  uint64_t out, a;
  uint32_t n, ndim, stride, pad;
  uint32_t size[8];
  int32_t so[8], sa[8];
} Copy8Params;

enum { VKT_MOVE_COPY = 0, VKT_MOVE_FILL = 1 }; /* shaders/opcodes.txt:206-207 */

/* "cast_fp8", spec {}: dst[i] = convert(src[i]), i < n, where one side is VKT_E4M3 / VKT_E5M2
 * and the other VKT_F32 / VKT_F16 / VKT_BF16 (or the other float8 format; two non-float8 types are
 * accepted too: the dense form of "cast_<src>_<dst>"): through float32,
 * bit for bit as the CPU converts (what the reference's copy between a float8 tensor and
 * a float tensor does with lookup tables, backend.cpp:534-586).  32 bytes. */
typedef struct CastParams {
  uint64_t src, dst, n;
  uint32_t src_dtype, dst_dtype;
} CastParams;

/* "fp8_quant", spec {ROWWISE}: the float8 producer in front of _scaled_mm.  src [m,k]
 * (float32 / float16 / bfloat16, rows lds elements apart) -> dst [m,k] float8 (rows ldd bytes
 * apart).  ROWWISE 1: scale[r] = max(max_k |src[r,k]|, 1e-12) / fmax is written (float32 [m],
 * what _scaled_mm takes as a rowwise scale); ROWWISE 0: scale[0] is read (one scale for the
 * tensor).  dst = convert(clamp(src * (fmax / (scale * fmax)), -fmax, fmax)), every step one
 * float32 operation; fmax = 448 (e4m3fn) or 57344 (e5m2).  No counterpart in the reference
 * (its float8 tensors come from casts alone).  48 bytes. */
typedef struct F8QuantParams {
  uint64_t src, dst, scale;
  uint32_t m, k, lds, ldd;
  uint32_t src_dtype, dst_fmt;
} F8QuantParams;

/* Per-tensor affine quantised tensors and fake quantisation, each one fused kernel (the reference
 * composes them from elementwise operators: quantized.cpp:72-130, _kernels.py:1613-1676), bit
 * for bit what PyTorch's x86 CPU kernels compute:
 *   "quantize_affine", spec {QTYPE}    src float32 [n] -> dst quint8 (QTYPE 0) | qint8 (1) | qint32 (2)
 *   "dequantize_affine", spec {QTYPE}  src integers [n] -> dst float32 = scale * float(q - zero_point)
 *   "fake_quant", spec {PER_CHANNEL, ZP_FLOAT}   src [n] (dtype) -> dst [n] (dtype), mask [n] bytes;
 *        per tensor: scale_bits, zero_point; per channel: scales float32 [channels], zero_points
 *        int32 or float32 [channels], element i in channel (i / inner) % channels.
 * Dense tensors.  88 bytes. */
typedef struct QuantParams {
  uint64_t src, dst, mask, scales, zero_points, n;
  uint32_t scale_bits; /* float32 bits of the scale */
  int32_t zero_point;
  int64_t qmin, qmax;
  uint32_t channels, inner;
  uint32_t dtype; /* fake_quant: VKT_F32 | VKT_F16 | VKT_BF16 */
  uint32_t pad;
} QuantParams;

/* "aminmax", spec {}: out_min[r], out_max[r] (float32) = the minimum and maximum of row r of src
 * [rows, cols] (dtype, rows ld elements apart); a NaN in a row makes both NaN, as torch.aminmax.
 * The range step of the fake-quantisation observer (_kernels.py:1744-1746).  40 bytes. */
typedef struct MinMaxParams {
  uint64_t src, out_min, out_max;
  uint32_t rows, cols, ld;
  uint32_t dtype; /* VKT_F32 | VKT_F16 | VKT_BF16 */
} MinMaxParams;

/* "fp8mm", spec {}: out = cast((f32(A)*sa) @ (f32(B)*sb) + bias) [* 1/scale_result]
 * (quant.cpp:279-300 fused into one kernel).  A: fp8 [m,k] row-major (lda bytes);
 * B: fp8, column-major, i.e. [n,k] rows ldb bytes apart.  104 bytes.  An optional entry overrides the launcher's
 * choice of kernel (tests, tuning; 0 or absent: planned): 1-9 tile shapes, 11 the stream kernel, 12 the few-row kernel
 * (up to 64 rows; bits 8-11: 16s of columns per workgroup, bits 12-16: slices of K over workgroups), 13 the vector-unit
 * kernel (up to 4 rows), 14 the 128 x 128 tile kernel with K in slices over workgroups (bits 8-12: slices, which must
 * divide k's steps of 128 bytes), 255 one thread per output. */
typedef struct F8Params {
  uint64_t a, b, scale_a, scale_b, bias, scale_result, out; /* bias / scale_result may be 0 */
  uint32_t m, n, k;
  uint32_t lda, ldb, ldo;  /* row strides in elements */
  uint32_t fmt_a, fmt_b;   /* VKT_E4M3 | VKT_E5M2 */
  uint32_t out_dtype;      /* VKT_F32 | VKT_F16 | VKT_BF16 | VKT_E4M3 | VKT_E5M2 */
  uint32_t bias_dtype;     /* VKT_F32 | VKT_F16 | VKT_BF16 */
  uint32_t rowwise;        /* 0: one scale each; 1: scale_a [m], scale_b [n] */
  uint32_t pad;
} F8Params;

/* "probe_read", spec {GEOMETRY} and "probe_mfma_f8", spec {OPERANDS}: calibration kernels for the rooflines (what
 * a launch geometry can stream, what the fp8 matrix cores sustain on given operand bits).  probe_read reads src and
 * writes nothing (dst: any valid 4-byte address): GEOMETRY 0, 1, 3 read the n * k bytes at src (k a multiple of 16);
 * GEOMETRY 2 reads the int4 streaming side-car of an [n, k] weight with blocks of 32, so src holds
 * vkt_qmm4c_bytes(n, k, 32) bytes and n is a multiple of 16, k of 4096 (anything else is refused).  probe_mfma_f8
 * runs `iters` iterations of 4 matrix-core instructions per wave, 4 waves on every compute unit, reads no memory
 * and stores the loop's shader cycles and 100 MHz ticks at dst + 64 and dst + 72: dst holds at least 80 bytes and is
 * 8-byte aligned.  "probe_delay", spec {}: one wave that waits
 * `iters` microseconds (at most 100000) and exits; a timing loop queues it in front of its launches so that the host
 * has queued them all before the device starts on them.  No counterpart in the reference.  32 bytes. */
typedef struct ProbeParams {
  uint64_t src, dst;
  uint32_t n, k, iters, pad;
} ProbeParams;

enum { VKT_F32 = 0, VKT_F16 = 1, VKT_BF16 = 2, VKT_E4M3 = 3, VKT_E5M2 = 4 };

#ifdef __cplusplus
}
#endif
#endif /* VKT_H */
