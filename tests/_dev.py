"""Runs the quantized-matmul kernels through the C ABI (vkt_alloc / vkt_copy_* /
vkt_dispatch) on numpy storage arrays, the way the reference's C++ op layer drives its
runtime (crates/pyvk/csrc/quant.cpp).  GPU tests only."""
import ctypes

import numpy as np

import oracle
from torch_vulkan_amd import abi

_NP = {oracle.F32: np.float32, oracle.F16: np.uint16, oracle.BF16: np.uint16, oracle.E4M3: np.uint8,
       oracle.E5M2: np.uint8}


def qmm8(a, odt, b, s, variant=0, row_step=1, static=False):
    """_weight_int8pack_mm.  a: storage array [M_total,K]; rows taken every `row_step`
    (a strided A as in a[::2]); returns the storage array [M,N].  static: through vkt_dispatch_static."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b, dtype=np.int8)
    s = np.ascontiguousarray(s)
    k, n = a.shape[1], b.shape[0]
    m = (a.shape[0] + row_step - 1) // row_step
    da, db, ds = abi.Buffer.from_numpy(a), abi.Buffer.from_numpy(b), abi.Buffer.from_numpy(s)
    dc = abi.Buffer(max(m * n * a.itemsize, 1))
    p = abi.Q8Params(a=da.address, b=db.address, scales=ds.address, c=dc.address, m=m, n=n, k=k, a_sm=k * row_step,
                     a_sk=1)
    # the reference's launch: ROWS = M for M <= 8, else the tile grid (quant.cpp:86-118)
    spec = [m if m <= 8 else 0, variant]
    grid = ((n + 7) // 8,) if m <= 8 else ((n + 63) // 64, (m + 63) // 64)
    if m and n:
        abi.dispatch("qmm8_" + abi.SUFFIX[odt], spec, p, grid, static=static)
    return dc.to_numpy(_NP[odt], (m, n))


def q4_reference_layout(x, odt, packed, bs, k, n, want_intermediates=False):
    """_dyn_quant_matmul_4bit through the reference's own parameter block and buffers
    ("qmm4_*": int32 q, float32-expanded packed vector; quant.cpp:178-202)."""
    x = np.ascontiguousarray(x)
    packed = np.ascontiguousarray(packed, dtype=np.float32)
    m = x.shape[0]
    dx, dp = abi.Buffer.from_numpy(x), abi.Buffer.from_numpy(packed)
    dq, dr = abi.Buffer(max(m * k * 4, 1)), abi.Buffer(max(m * 8, 1))
    do = abi.Buffer(max(m * n * x.itemsize, 1))
    wcount, nscale = n * k // 2, n * (k // bs)
    has_bias = int(packed.size - (wcount + nscale) != 0)
    p = abi.Q4Params(inp=dx.address, q=dq.address, rows=dr.address, packed=dp.address, out=do.address, m=m, n=n, k=k,
                     bs=bs, has_bias=has_bias)
    g = int(bs != k)
    name = "qmm4_" + abi.SUFFIX[odt]
    if m and n:
        abi.dispatch(name, [0, g], p, (m,))
        abi.dispatch(name, [1, g], p, ((n + 31) // 32, (m + 7) // 8))
    out = do.to_numpy(_NP[odt], (m, n))
    if want_intermediates:
        rows = dr.to_numpy(np.uint32, (m, 2))
        return out, dq.to_numpy(np.int32, (m, k)), rows[:, 0].view(np.float32), rows[:, 1].view(np.int32)
    return out


class CompactWeights:
    """The compact side-car of a packed float32 vector ("qmm4c_pack"), built once."""

    def __init__(self, packed, bs, k, n, layout=0):
        packed = np.ascontiguousarray(packed, dtype=np.float32)
        self.layout = layout  # 0: streaming (at most 4 rows at a time), 1: matrix cores
        nbytes = abi.lib().vkt_qmm4c_bytes(n, k, bs)
        assert nbytes, "no compact form"
        self.n, self.k, self.bs = n, k, bs
        self.has_bias = int(packed.size - (n * k // 2 + n * (k // bs)) != 0)
        dp = abi.Buffer.from_numpy(packed)
        self.buf = abi.Buffer(nbytes)
        p = abi.Q4PackParams(packed=dp.address, compact=self.buf.address, n=n, k=k, bs=bs, has_bias=self.has_bias)
        abi.dispatch("qmm4c_pack", [layout], p)
        abi.synchronize()
        dp.free()


def q4_compact(x, odt, cw, fused=True, flags=0):
    """_dyn_quant_matmul_4bit through the streaming path ("qmm4c_*"): one fused launch
    (PHASE 2), or row quantisation (PHASE 0) then the product (PHASE 1).  flags (matrix-core layout): 16 keeps the
    one-row-tile kernel, 32 forces the wave-per-tile kernel (| 64: one tile per wave, | 128: two, | 192: four)."""
    x = np.ascontiguousarray(x)
    m, n, k, bs = x.shape[0], cw.n, cw.k, cw.bs
    dx = abi.Buffer.from_numpy(x)
    dq = abi.Buffer(max(abi.lib().vkt_qmm4c_q_bytes(m, k), 1))
    dr = abi.Buffer(max(m * 8, 1))
    do = abi.Buffer(max(m * n * x.itemsize, 1))
    p = abi.Q4CParams(inp=dx.address, q=dq.address, rows=dr.address, compact=cw.buf.address, out=do.address, m=m, n=n,
                      k=k, bs=bs, has_bias=cw.has_bias)
    g = int(bs != k)
    name = "qmm4c_" + abi.SUFFIX[odt]
    if m and n and fused:
        abi.dispatch(name, [2 | flags, g, cw.layout], p, ((n + 31) // 32, (m + 7) // 8))
    elif m and n:
        abi.dispatch(name, [0, g, cw.layout], p, (m,))
        abi.dispatch(name, [1 | flags, g, cw.layout], p, ((n + 31) // 32, (m + 7) // 8))
    return do.to_numpy(_NP[odt], (m, n))


def scaled_mm(a, fmt_a, bt, fmt_b, sa, sb, rowwise, bias=None, bias_dtype=oracle.F32, scale_result=None,
              out_dtype=oracle.BF16, variant=0, static=False):
    """_scaled_mm ("fp8mm").  a: uint8 codes [M,K]; bt: uint8 codes [N,K] (mat2 column-major).  static: through
    vkt_dispatch_static."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    bt = np.ascontiguousarray(bt, dtype=np.uint8)
    (m, k), n = a.shape, bt.shape[0]
    sa = np.ascontiguousarray(np.asarray(sa, np.float32).reshape(-1))
    sb = np.ascontiguousarray(np.asarray(sb, np.float32).reshape(-1))
    da, db = abi.Buffer.from_numpy(a), abi.Buffer.from_numpy(bt)
    dsa, dsb = abi.Buffer.from_numpy(sa), abi.Buffer.from_numpy(sb)
    dbias = None if bias is None else abi.Buffer.from_numpy(np.ascontiguousarray(bias))
    dsr = None if scale_result is None else abi.Buffer.from_numpy(np.asarray([scale_result], np.float32))
    item = np.dtype(_NP[out_dtype]).itemsize
    do = abi.Buffer(max(m * n * item, 1))
    p = abi.F8Params(a=da.address, b=db.address, scale_a=dsa.address, scale_b=dsb.address,
                     bias=dbias.address if dbias else 0, scale_result=dsr.address if dsr else 0, out=do.address, m=m,
                     n=n, k=k, lda=k, ldb=k, ldo=n, fmt_a=fmt_a, fmt_b=fmt_b, out_dtype=out_dtype,
                     bias_dtype=bias_dtype, rowwise=int(bool(rowwise)))
    if m and n:
        abi.dispatch("fp8mm", [variant], p, static=static)
    return do.to_numpy(_NP[out_dtype], (m, n))


def cast(a, src_dtype, dst_dtype, skew=0):
    """Elementwise float8 cast ("cast_fp8").  skew: elements by which both device addresses are
    moved off their 16-element alignment (the element-by-element form of the kernel)."""
    a = np.ascontiguousarray(a, dtype=_NP[src_dtype]).reshape(-1)
    n = a.size
    si, di = a.itemsize, np.dtype(_NP[dst_dtype]).itemsize
    dsrc = abi.Buffer(max((n + skew) * si, 1))
    ddst = abi.Buffer(max((n + skew) * di, 1))
    if n:
        abi.check(abi.lib().vkt_copy_to_device(dsrc.address + skew * si, a.ctypes.data, n * si))
        p = abi.CastParams(src=dsrc.address + skew * si, dst=ddst.address + skew * di, n=n, src_dtype=src_dtype,
                           dst_dtype=dst_dtype)
        abi.dispatch("cast_fp8", [], p)
    return ddst.to_numpy(_NP[dst_dtype], (n + skew,))[skew:]


def fp8_quant(x, dtype, fmt, scale=None, pad=0):
    """The float8 producer ("fp8_quant"): rowwise scales computed, or one given scale.
    pad: extra elements between rows on both sides (row strides larger than k)."""
    x = np.ascontiguousarray(x, dtype=_NP[dtype])
    m, k = x.shape
    lds = ldd = k + pad
    xs = np.zeros((m, lds), _NP[dtype])
    xs[:, :k] = x
    dx = abi.Buffer.from_numpy(xs)
    dq = abi.Buffer(max(m * ldd, 1))
    abi.check(abi.lib().vkt_fill(dq.address, 0xAB, max(m * ldd, 1)))
    rowwise = scale is None
    ds = abi.Buffer(max(m * 4, 4)) if rowwise else abi.Buffer.from_numpy(np.asarray([scale], np.float32))
    p = abi.F8QuantParams(src=dx.address, dst=dq.address, scale=ds.address, m=m, k=k, lds=lds, ldd=ldd, src_dtype=dtype,
                          dst_fmt=fmt)
    if m and k:
        abi.dispatch("fp8_quant", [int(rowwise)], p)
    q = dq.to_numpy(np.uint8, (m, ldd))
    assert (q[:, k:] == 0xAB).all(), "the producer wrote between rows"
    return q[:, :k], ds.to_numpy(np.float32, (m if rowwise else 1,))


def _device_view(arr):
    """Uploads the bytes a (possibly strided) numpy array spans; returns (buffer, address of
    element [0,...,0], element strides)."""
    arr = np.asarray(arr)
    lo = sum(min(0, (n - 1) * st) for n, st in zip(arr.shape, arr.strides))
    hi = sum(max(0, (n - 1) * st) for n, st in zip(arr.shape, arr.strides)) + arr.itemsize
    base = arr.__array_interface__["data"][0] + lo
    raw = (ctypes.c_uint8 * (hi - lo)).from_address(base)
    buf = abi.Buffer(max(hi - lo, 1))
    abi.check(abi.lib().vkt_copy_to_device(buf.address, ctypes.addressof(raw), hi - lo))
    return buf, buf.address - lo, [st // arr.itemsize for st in arr.strides]


def gemm16(a, b, dtype, cin=None, alpha=1.0, beta=0.0, variant=0, static=False):
    """alpha * a @ b (+ beta * cin) through "gemmcm_<T>": a [B,]M,K and b [B,]K,N as uint16 views with
    any strides; cin broadcastable to the result (zero strides).  static: through vkt_dispatch_static."""
    a3 = np.asarray(a) if np.asarray(a).ndim == 3 else np.asarray(a)[None]
    b3 = np.asarray(b) if np.asarray(b).ndim == 3 else np.asarray(b)[None]
    B, M, K = a3.shape
    N = b3.shape[2]
    ba, pa, sa = _device_view(a3)
    bb, pb, sb = _device_view(b3)
    out = abi.Buffer(max(B * M * N * 2, 1))
    p = abi.GemmParams(a=pa, b=pb, c=out.address, m=M, n=N, k=K, a_sb=sa[0], a_sm=sa[1], a_sk=sa[2], b_sb=sb[0],
                       b_sk=sb[1], b_sn=sb[2], c_sb=M * N, c_sm=N, c_sn=1,
                       alpha=int(np.float32(alpha).view(np.uint32)), beta=int(np.float32(beta).view(np.uint32)))
    use_cin = cin is not None and beta != 0.0
    if use_cin:
        c3 = np.broadcast_to(np.asarray(cin), (B, M, N))
        bc, pc, sc = _device_view(c3)
        p.cin, p.cin_sb, p.cin_sm, p.cin_sn = pc, sc[0], sc[1], sc[2]
    if B and M and N:
        abi.dispatch("gemmcm_" + abi.SUFFIX[dtype], [int(use_cin), 0, 0, variant], p, (1, 1, B), static=static)
    res = out.to_numpy(np.uint16, (B, M, N))
    return res if np.asarray(a).ndim == 3 else res[0]


def _span(arr):
    """(lowest byte offset, byte length) of the memory a strided numpy view touches, relative to element [0,..,0]."""
    lo = sum(min(0, (n - 1) * st) for n, st in zip(arr.shape, arr.strides))
    hi = sum(max(0, (n - 1) * st) for n, st in zip(arr.shape, arr.strides)) + arr.itemsize
    return lo, hi - lo


def _upload_span(arr):
    lo, length = _span(arr)
    raw = (ctypes.c_uint8 * length).from_address(arr.__array_interface__["data"][0] + lo)
    buf = abi.Buffer(length)
    abi.check(abi.lib().vkt_copy_to_device(buf.address, ctypes.addressof(raw), length))
    return buf, buf.address - lo, raw


def _dims(dst, src):
    size = list(dst.shape[::-1])
    so = [st // dst.itemsize for st in dst.strides[::-1]]
    sa = [st // src.itemsize for st in np.broadcast_to(src, dst.shape).strides[::-1]] if src is not None else [0] * len(size)
    return size, so, sa


def move(dst, src=None, value=None, variant=0, cast=None):
    """dst[...] = src (broadcast) or the fill value, on the device, through "move_b<S>" (up to 4 dims) or
    "copy8_b<S>" (5 to 8); cast=(src_label, dst_label) runs "cast_<src>_<dst>" instead.  dst's memory is
    uploaded first and read back, so untouched elements show as unchanged."""
    if dst.size == 0:
        return dst
    size, so, sa = _dims(dst, src)
    dbuf, daddr, draw = _upload_span(dst)
    if src is not None:
        src = np.broadcast_to(src, dst.shape)
        sbuf, saddr, _ = _upload_span(src)
    label = "b%d" % dst.itemsize
    if len(size) <= 4:
        p = abi.StridedParams(out=daddr, a=saddr if src is not None else 0, n=dst.size, ndim=len(size))
        for d in range(len(size)):
            p.size[d], p.so[d], p.sa[d] = size[d], so[d], sa[d]
        for d in range(len(size), 4):
            p.size[d] = 1
        if cast is not None:
            abi.dispatch("cast_%s_%s" % cast, [], p)
        elif src is not None:
            abi.dispatch("move_" + label, [abi.MOVE_COPY, 0, variant], p)
        else:
            bits = np.frombuffer(np.asarray(value).tobytes().ljust(16, b"\0"), np.uint64)
            p.alpha, p.beta = int(bits[0]), int(bits[1])
            abi.dispatch("move_" + label, [abi.MOVE_FILL, 0, variant], p)
    else:
        assert src is not None and cast is None and len(size) <= 8
        p = abi.Copy8Params(out=daddr, a=saddr, n=dst.size, ndim=len(size))
        for d in range(8):
            p.size[d], p.so[d], p.sa[d] = (size[d], so[d], sa[d]) if d < len(size) else (1, 0, 0)
        abi.dispatch("copy8_" + label, [variant], p)
    abi.check(abi.lib().vkt_copy_to_host(ctypes.addressof(draw), dbuf.address, len(draw)))
    return dst


_QNP = {0: np.uint8, 1: np.int8, 2: np.int32}


def quantize_affine(x, scale, zero_point, qtype, skew=0):
    """float32 array -> integers of quint8 (0) / qint8 (1) / qint32 (2); skew: elements by which both
    buffers are offset from their allocations (exercises the unaligned form)."""
    x = np.ascontiguousarray(x, np.float32)
    qdt = np.dtype(_QNP[qtype])
    src, dst = abi.Buffer(x.nbytes + 4 * skew + 4), abi.Buffer(x.size * qdt.itemsize + skew * qdt.itemsize + 4)
    abi.check(abi.lib().vkt_copy_to_device(src.address + 4 * skew, x.ctypes.data, x.nbytes))
    p = abi.QuantParams(src=src.address + 4 * skew, dst=dst.address + qdt.itemsize * skew, n=x.size,
                        scale_bits=int(np.float32(scale).view(np.uint32)), zero_point=zero_point)
    abi.dispatch("quantize_affine", [qtype], p)
    out = np.empty(x.shape, qdt)
    abi.check(abi.lib().vkt_copy_to_host(out.ctypes.data, dst.address + qdt.itemsize * skew, out.nbytes))
    return out


def dequantize_affine(q, scale, zero_point, qtype, skew=0):
    q = np.ascontiguousarray(q, _QNP[qtype])
    src, dst = abi.Buffer(q.nbytes + q.itemsize * skew + 4), abi.Buffer(q.size * 4 + 4 * skew + 4)
    abi.check(abi.lib().vkt_copy_to_device(src.address + q.itemsize * skew, q.ctypes.data, q.nbytes))
    p = abi.QuantParams(src=src.address + q.itemsize * skew, dst=dst.address + 4 * skew, n=q.size,
                        scale_bits=int(np.float32(scale).view(np.uint32)), zero_point=zero_point)
    abi.dispatch("dequantize_affine", [qtype], p)
    out = np.empty(q.shape, np.float32)
    abi.check(abi.lib().vkt_copy_to_host(out.ctypes.data, dst.address + 4 * skew, out.nbytes))
    return out


def fake_quant(x, dtype, scales, zero_points, qmin, qmax, axis=None, skew=0):
    """(output in x's type, mask uint8): x a float32 array (dtype F32) or a uint16 view (F16 / BF16)."""
    x = np.ascontiguousarray(x)
    item = x.itemsize
    src, dst, mask = abi.Buffer(x.nbytes + item * skew + 4), abi.Buffer(x.nbytes + item * skew + 4), abi.Buffer(x.size + skew + 4)
    abi.check(abi.lib().vkt_copy_to_device(src.address + item * skew, x.ctypes.data, x.nbytes))
    scales = np.ascontiguousarray(np.atleast_1d(scales), np.float32)
    zps = np.atleast_1d(zero_points)
    zp_float = int(zps.dtype.kind == "f")
    zps = np.ascontiguousarray(zps, np.float32 if zp_float else np.int32)
    p = abi.QuantParams(src=src.address + item * skew, dst=dst.address + item * skew, mask=mask.address + skew, n=x.size,
                        qmin=qmin, qmax=qmax, dtype=dtype)
    if axis is None:
        p.scale_bits, p.zero_point = int(scales[0].view(np.uint32)), int(zps[0])
        abi.dispatch("fake_quant", [0, 0], p)
    else:
        ds, dz = abi.Buffer.from_numpy(scales), abi.Buffer.from_numpy(zps)
        p.scales, p.zero_points, p.channels, p.inner = ds.address, dz.address, x.shape[axis], int(np.prod(x.shape[axis + 1:]))
        abi.dispatch("fake_quant", [1, zp_float], p)
    out, m = np.empty(x.shape, x.dtype), np.empty(x.shape, np.uint8)
    abi.check(abi.lib().vkt_copy_to_host(out.ctypes.data, dst.address + item * skew, out.nbytes))
    abi.check(abi.lib().vkt_copy_to_host(m.ctypes.data, mask.address + skew, m.nbytes))
    return out, m


def aminmax(x, dtype, ld=None, static=False):
    """(min, max) float32 per row of a 2-d array (float32, or a uint16 view of float16 / bfloat16 values); ld: row
    pitch in elements of the device copy (rows further apart than they are long).  static: through vkt_dispatch_static."""
    x = np.ascontiguousarray(x)
    rows, cols = x.shape
    ld = ld or cols
    padded = np.zeros((rows, ld), x.dtype)
    padded[:, :cols] = x
    src = abi.Buffer.from_numpy(padded)
    lo, hi = abi.Buffer(4 * rows), abi.Buffer(4 * rows)
    abi.dispatch("aminmax", [], abi.MinMaxParams(src=src.address, out_min=lo.address, out_max=hi.address, rows=rows, cols=cols, ld=ld, dtype=dtype), static=static)
    return lo.to_numpy(np.float32, (rows,)), hi.to_numpy(np.float32, (rows,))
