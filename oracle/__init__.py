"""TEST INFRASTRUCTURE — not product code.

ctypes/numpy front end of the C restatement in ``qmm_oracle.c`` (the CPU oracle of the
quantized-matmul path).  Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s
``cpu_baseline`` leg may import this package; the product path never does.

Arrays are numpy; 16-bit floats travel as their uint16 bit patterns and float8 as uint8
codes, so nothing here depends on torch.
"""
import ctypes
import os
import subprocess

import numpy as np

F32, F16, BF16, E4M3, E5M2 = 0, 1, 2, 3, 4
_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_lib = None


def build(force=False):
    """Compiles qmm_oracle.c with gcc (see Makefile)."""
    src = os.path.join(_HERE, "qmm_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        L = _lib
        L.orc_f32_to_bf16.restype = ctypes.c_uint16
        L.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_f32_to_fp8.restype = ctypes.c_uint8
        L.orc_f32_to_fp8.argtypes = [ctypes.c_float, ctypes.c_int]
        L.orc_fp8_to_f32.restype = ctypes.c_float
        L.orc_fp8_to_f32.argtypes = [ctypes.c_uint8, ctypes.c_int]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_q4_pack.restype = ctypes.c_int64
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a)
    return a if dtype is None else a.astype(dtype, copy=False)


_NP = {F32: np.float32, F16: np.uint16, BF16: np.uint16, E4M3: np.uint8, E5M2: np.uint8}
I64 = ctypes.c_int64


# ------------------------------------------------------------------ casts (vectorised loops in Python: small inputs only)
def f32_to_bf16(x):
    x = np.asarray(x, np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return np.where(np.isnan(x), np.uint16(0x7FC0), r)


def bf16_to_f32(h):
    return (np.asarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def f32_to_f16(x):
    L = lib()
    x = np.asarray(x, np.float32)
    return np.array([L.orc_f32_to_f16(float(v)) for v in x.ravel()], np.uint16).reshape(x.shape)


def f32_to_fp8(x, fmt):
    L = lib()
    x = np.asarray(x, np.float32)
    return np.array([L.orc_f32_to_fp8(ctypes.c_float(v), fmt) for v in x.ravel()], np.uint8).reshape(x.shape)


def fp8_table(fmt):
    L = lib()
    return np.array([L.orc_fp8_to_f32(i, fmt) for i in range(256)], np.float32)


def to_f32(a, dtype):
    if dtype == F32:
        return np.asarray(a, np.float32)
    if dtype == BF16:
        return bf16_to_f32(a)
    if dtype == F16:
        return np.asarray(a, np.uint16).view(np.float16).astype(np.float32)
    return fp8_table(dtype)[np.asarray(a, np.uint8)]


# ------------------------------------------------------------------ ops
def qmm8(a, dtype, b, scales, want_f64=False):
    """_weight_int8pack_mm.  a: [M,K] storage array of `dtype`, unit stride along K, any
    row stride (a numpy view such as base[::2] is read in place); b int8 [N,K]; scales [N]
    storage array of `dtype`.  Returns c (storage array [M,N]) or (c, c64, mag)."""
    a = np.asarray(a, _NP[dtype])
    b = _c(b, np.int8)
    scales = _c(scales, _NP[dtype])
    N, K = b.shape
    M = a.shape[0]
    if M > 1 and K > 1 and a.strides[1] != a.itemsize:
        a = np.ascontiguousarray(a)
    a_sm = a.strides[0] // a.itemsize if M > 1 else K
    c = np.empty((M, N), _NP[dtype])
    c64 = np.empty((M, N), np.float64)
    mag = np.empty((M, N), np.float64)
    lib().orc_qmm8(_p(a), dtype, I64(a_sm), _p(b), _p(scales), _p(c), _p(c64), _p(mag), I64(M), I64(N), I64(K))
    return (c, c64, mag) if want_f64 else c


def qmm8_f32order(a, dtype, b, scales):
    a = _c(a, _NP[dtype])
    b = _c(b, np.int8)
    scales = _c(scales, _NP[dtype])
    (M, K), N = a.shape, b.shape[0]
    c = np.empty((M, N), _NP[dtype])
    lib().orc_qmm8_f32order(_p(a), dtype, I64(K), _p(b), _p(scales), _p(c), I64(M), I64(N), I64(K))
    return c


def q4_pack(w, scales, scales_dtype, bias):
    """_dyn_quant_pack_4bit_weight: float32 vector [bytes | scales | bias]."""
    w = _c(w, np.uint8)
    scales = _c(scales, _NP[scales_dtype])
    nb = 0 if bias is None else bias.size
    bias = None if bias is None else _c(bias, np.float32)
    out = np.empty(w.size + scales.size + nb, np.float32)
    n = lib().orc_q4_pack(_p(w), I64(w.size), _p(scales), scales_dtype, I64(scales.size), _p(bias), I64(nb), _p(out))
    assert n == out.size
    return out


def q4_rowquant(x, dtype, groupwise):
    x = _c(x, _NP[dtype])
    M, K = x.shape
    q = np.empty((M, K), np.int32)
    recip = np.empty(M, np.float32)
    nzp = np.empty(M, np.int32)
    lib().orc_q4_rowquant(_p(x), dtype, I64(M), I64(K), int(bool(groupwise)), _p(q), _p(recip), _p(nzp))
    return q, recip, nzp


def q4_matmul(x, dtype, packed, bs, K, N, want_iacc=False):
    """_dyn_quant_matmul_4bit.  Returns out [M,N] (storage array) or (out, iacc[M,N,nblocks])."""
    x = _c(x, _NP[dtype])
    packed = _c(packed, np.float32)
    M = x.shape[0]
    out = np.empty((M, N), _NP[dtype])
    nblocks = (K + bs - 1) // bs
    iacc = np.empty((M, N, nblocks), np.int32) if want_iacc else None
    lib().orc_q4_matmul(_p(x), dtype, _p(packed), I64(packed.size), I64(M), I64(K), I64(N), I64(bs), _p(out), _p(iacc))
    return (out, iacc) if want_iacc else out


def scaled_mm(a, fmt_a, bt, fmt_b, sa, sb, rowwise, bias=None, bias_dtype=F32, scale_result=None, out_dtype=BF16,
              want_mag=False):
    """_scaled_mm.  a: uint8 codes [M,K]; bt: uint8 codes [N,K] (mat2 column-major);
    sa/sb float32 ([1] or [M]/[N])."""
    a = _c(a, np.uint8)
    bt = _c(bt, np.uint8)
    (M, K), N = a.shape, bt.shape[0]
    sa = _c(np.asarray(sa, np.float32).reshape(-1))
    sb = _c(np.asarray(sb, np.float32).reshape(-1))
    bias = None if bias is None else _c(bias, _NP[bias_dtype])
    sr = None if scale_result is None else np.asarray([scale_result], np.float32)
    out = np.empty((M, N), _NP[out_dtype])
    mag = np.empty((M, N), np.float64) if want_mag else None
    lib().orc_scaled_mm(_p(a), fmt_a, _p(bt), fmt_b, _p(sa), _p(sb), int(bool(rowwise)), _p(bias), bias_dtype, _p(sr),
                        _p(out), out_dtype, _p(mag), I64(M), I64(N), I64(K))
    return (out, mag) if want_mag else out


def cast(a, src_dtype, dst_dtype):
    """Elementwise conversion where one side is float8 (through float32, as c10)."""
    a = _c(a, _NP[src_dtype])
    out = np.empty(a.shape, _NP[dst_dtype])
    lib().orc_cast(_p(a), src_dtype, _p(out), dst_dtype, I64(a.size))
    return out


def fp8_quant(x, dtype, fmt, scale=None):
    """The float8 producer: rowwise scales computed (scale is None) or one given scale.
    Returns (codes uint8 [M,K], scales float32 [M] or [1])."""
    x = _c(x, _NP[dtype])
    m, k = x.shape
    q = np.empty((m, k), np.uint8)
    rowwise = scale is None
    scales = np.empty(m, np.float32) if rowwise else np.asarray([scale], np.float32)
    lib().orc_fp8_quant_rows(_p(x), dtype, I64(m), I64(k), I64(k), fmt, int(rowwise), _p(q), I64(k), _p(scales))
    return q, scales


def _layout(dst, src):
    """(sizes, dst strides, src strides) in elements, innermost dim first, src broadcast to dst."""
    size = np.array(dst.shape[::-1], np.int64)
    so = np.array([x // dst.itemsize for x in dst.strides[::-1]], np.int64)
    if src is None:
        return size, so, np.zeros_like(so)
    src = np.broadcast_to(src, dst.shape)
    return size, so, np.array([x // src.itemsize for x in src.strides[::-1]], np.int64)


def _base(a):
    return ctypes.c_void_p(a.__array_interface__["data"][0])


def move(dst, src=None, value=None):
    """dst[...] = src (any strides either side, src broadcast to dst), or the fill value's bytes: the strided
    move kernel's index arithmetic.  dst is a numpy array (written in place); non-negative strides."""
    size, so, sa = _layout(dst, src)
    if dst.size == 0:
        return dst
    if src is not None:
        src = np.broadcast_to(src, dst.shape)
        assert src.itemsize == dst.itemsize
        lib().orc_move(_base(dst), _base(src), I64(dst.itemsize), I64(dst.size), len(size), _p(size), _p(so), _p(sa), 0, None)
    else:
        v = np.frombuffer(np.asarray(value).tobytes(), np.uint8).copy()
        assert v.size == dst.itemsize
        lib().orc_move(_base(dst), None, I64(dst.itemsize), I64(dst.size), len(size), _p(size), _p(so), _p(sa), 1, _p(v))
    return dst


def cast_strided(dst, dst_dtype, src, src_dtype):
    """dst[...] = dst_dtype(src) over strided views (uint16 views for the 16-bit types, float32 else)."""
    size, so, sa = _layout(dst, src)
    if dst.size:
        src = np.broadcast_to(src, dst.shape)
        lib().orc_cast_strided(_base(dst), dst_dtype, _base(src), src_dtype, I64(dst.size), len(size), _p(size), _p(so), _p(sa))
    return dst


QUINT8, QINT8, QINT32 = 0, 1, 2
_QNP = {QUINT8: np.uint8, QINT8: np.int8, QINT32: np.int32}


def quantize_affine(x, scale, zero_point, qtype):
    """quantize_per_tensor's integers (x86 / FBGEMM semantics) of a float32 array."""
    x = _c(x, np.float32)
    out = np.empty(x.shape, _QNP[qtype])
    lib().orc_quantize_affine(_p(x), I64(x.size), ctypes.c_float(scale), ctypes.c_int32(zero_point), qtype, _p(out))
    return out


def dequantize_affine(q, scale, zero_point, qtype):
    q = _c(q, _QNP[qtype])
    out = np.empty(q.shape, np.float32)
    lib().orc_dequantize_affine(_p(q), qtype, I64(q.size), ctypes.c_float(scale), ctypes.c_int32(zero_point), _p(out))
    return out


def fake_quant(x, dtype, scales, zero_points, qmin, qmax, axis=None):
    """(output in x's type, mask uint8) of fake quantisation: per tensor (axis None; scales / zero_points of one
    element) or per channel along `axis` (zero_points int32 or float32)."""
    x = _c(x, _NP[dtype])
    scales = _c(np.atleast_1d(scales), np.float32)
    zps = np.atleast_1d(zero_points)
    zp_float = int(zps.dtype.kind == "f")
    zps = _c(zps, np.float32 if zp_float else np.int32)
    channels = x.shape[axis] if axis is not None else 1
    inner = int(np.prod(x.shape[axis + 1:])) if axis is not None else 1
    out, mask = np.empty(x.shape, _NP[dtype]), np.empty(x.shape, np.uint8)
    lib().orc_fake_quant(_p(x), dtype, I64(x.size), _p(scales), _p(zps), zp_float, I64(channels), I64(inner),
                         int(axis is not None), I64(qmin), I64(qmax), _p(out), _p(mask))
    return out, mask


def choose_qparams(mn, mx, qmin, qmax, symmetric):
    """(scale float32, zero point) from a range, as the CPU's observer chooses them."""
    sc, zp = ctypes.c_float(), ctypes.c_int32()
    rc = lib().orc_choose_qparams(ctypes.c_float(mn), ctypes.c_float(mx), ctypes.c_int32(qmin), ctypes.c_int32(qmax), int(symmetric),
                                  ctypes.byref(sc), ctypes.byref(zp))
    if rc != 0:
        raise ValueError("In ChooseQuantizationParams, min should be less than or equal to max")
    return np.float32(sc.value), zp.value


def observe_fake_quant(x, dtype, run_min, run_max, averaging_const, qmin, qmax, per_row, symmetric):
    """One step of the fused moving-average observer with fake quantisation on (observer on): updates run_min /
    run_max (float32 arrays, in place), returns (output, mask, scales float32, zero points int32)."""
    xf = to_f32(x, dtype) if dtype != F32 else np.asarray(x, np.float32)
    rows = xf.reshape(xf.shape[0], -1) if per_row else xf.reshape(1, -1)
    nan = np.isnan(rows).any(axis=1)
    cur_min = np.where(nan, np.float32("nan"), rows.min(axis=1)).astype(np.float32)
    cur_max = np.where(nan, np.float32("nan"), rows.max(axis=1)).astype(np.float32)
    lib().orc_observe(_p(run_min), _p(run_max), _p(cur_min), _p(cur_max), I64(run_min.size), ctypes.c_float(averaging_const))
    qp = [choose_qparams(a, b, qmin, qmax, symmetric) for a, b in zip(run_min, run_max)]
    scales, zps = np.array([q[0] for q in qp], np.float32), np.array([q[1] for q in qp], np.int32)
    out, mask = fake_quant(x, dtype, scales, zps, qmin, qmax, axis=0 if per_row else None)
    return out, mask, scales, zps


def _strided(a):
    """(base pointer, element strides) of a numpy array viewed as [B, R, C]."""
    a3 = a if a.ndim == 3 else a[None]
    st = np.array([x // a.itemsize for x in a3.strides], np.int64)
    return a3, st


def gemm16(a, b, dtype, cin=None, alpha=1.0, beta=0.0, want_mag=False):
    """alpha * a @ b (+ beta * cin) for uint16 views of bfloat16 / float16 arrays [B,]M,K and [B,]K,N
    (any strides); cin broadcastable to the result.  Returns the 16-bit result [B,]M,N (and the magnitude bound)."""
    a3, sa = _strided(np.asarray(a))
    b3, sb = _strided(np.asarray(b))
    B, M, K = a3.shape
    N = b3.shape[2]
    out = np.empty((B, M, N), np.uint16)
    sc = np.array([M * N, N, 1], np.int64)
    mag = np.empty((B, M, N), np.float64) if want_mag else None
    if cin is not None:
        c3 = np.broadcast_to(np.asarray(cin), (B, M, N))
        scin = np.array([x // 2 for x in c3.strides], np.int64)
        cp = ctypes.c_void_p(c3.__array_interface__["data"][0])
    else:
        scin, cp = np.zeros(3, np.int64), None
    # base pointers at element (0,0,0): negative strides are handled by the element offsets
    lib().orc_gemm16(ctypes.c_void_p(a3.__array_interface__["data"][0]), ctypes.c_void_p(b3.__array_interface__["data"][0]),
                     cp, _p(out), dtype, I64(B), I64(M), I64(N), I64(K), _p(sa), _p(sb), _p(sc), _p(scin),
                     ctypes.c_float(alpha), ctypes.c_float(beta), _p(mag) if want_mag else None)
    res = out if np.asarray(a).ndim == 3 else out[0]
    if want_mag:
        return res, (mag if np.asarray(a).ndim == 3 else mag[0])
    return res
