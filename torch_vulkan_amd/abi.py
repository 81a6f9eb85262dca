"""ctypes binding of the C ABI in include/vkt.h (libvkt_mi355.so).

This is the thinnest possible host side: the same twelve ``vkt_*`` functions the reference's
C++ backend binds (crates/pyvk/csrc/vk.h:49-69), the HIP additions, and the parameter blocks.
There is no CPU fallback anywhere below this module: if the library is missing or there is
no gfx950 device, calls raise.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libvkt_mi355.so")

F32, F16, BF16, E4M3, E5M2 = 0, 1, 2, 3, 4
SUFFIX = {F32: "f32", F16: "f16", BF16: "bf16"}
u64, u32, i32 = ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int32


class VktError(RuntimeError):
    pass


class VktAlloc(ctypes.Structure):
    _fields_ = [("handle", ctypes.c_void_p), ("host", ctypes.c_void_p), ("address", u64), ("size", u64)]


class VktDeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("compute_units", u32), ("clock_khz", u32), ("mem_clock_khz", u32),
                ("mem_bus_bits", u32), ("hbm_bytes", u64), ("lds_bytes_per_block", u32), ("l2_bytes", u32)]


class Q8Params(ctypes.Structure):  # reference quant.cpp:31-37
    _fields_ = [("a", u64), ("b", u64), ("scales", u64), ("c", u64), ("m", u32), ("n", u32), ("k", u32),
                ("a_sm", i32), ("a_sk", i32), ("pad", u32)]


class Q4Params(ctypes.Structure):  # reference quant.cpp:39-43
    _fields_ = [("inp", u64), ("q", u64), ("rows", u64), ("packed", u64), ("out", u64), ("m", u32), ("n", u32),
                ("k", u32), ("bs", u32), ("has_bias", u32), ("pad", u32)]


class Q4VecParams(ctypes.Structure):
    _fields_ = [("weights", u64), ("scales", u64), ("bias", u64), ("out", u64), ("nw", u32), ("ns", u32), ("nb", u32),
                ("scales_dtype", u32), ("bias_dtype", u32), ("pad", u32)]


class Q4PackParams(ctypes.Structure):
    _fields_ = [("packed", u64), ("compact", u64), ("n", u32), ("k", u32), ("bs", u32), ("has_bias", u32)]


class Q4CParams(ctypes.Structure):
    _fields_ = [("inp", u64), ("q", u64), ("rows", u64), ("compact", u64), ("out", u64), ("m", u32), ("n", u32),
                ("k", u32), ("bs", u32), ("has_bias", u32), ("pad", u32)]


class F8Params(ctypes.Structure):
    _fields_ = [("a", u64), ("b", u64), ("scale_a", u64), ("scale_b", u64), ("bias", u64), ("scale_result", u64),
                ("out", u64), ("m", u32), ("n", u32), ("k", u32), ("lda", u32), ("ldb", u32), ("ldo", u32),
                ("fmt_a", u32), ("fmt_b", u32), ("out_dtype", u32), ("bias_dtype", u32), ("rowwise", u32), ("pad", u32)]


class GemmParams(ctypes.Structure):
    _fields_ = [("a", u64), ("b", u64), ("c", u64), ("cin", u64), ("alpha", u64), ("beta", u64),
                ("m", u32), ("n", u32), ("k", u32), ("pad", u32)] + [
                    (name, ctypes.c_int32) for name in ("a_sm", "a_sk", "a_sb", "b_sk", "b_sn", "b_sb", "c_sm", "c_sn", "c_sb",
                                                        "cin_sm", "cin_sn", "cin_sb")]


class StridedParams(ctypes.Structure):
    _fields_ = [("out", u64), ("a", u64), ("b", u64), ("alpha", u64), ("beta", u64), ("gamma", u64),
                ("n", u32), ("ndim", u32), ("stride", u32), ("pad", u32), ("size", u32 * 4),
                ("so", i32 * 4), ("sa", i32 * 4), ("sb", i32 * 4)]


class Copy8Params(ctypes.Structure):
    _fields_ = [("out", u64), ("a", u64), ("n", u32), ("ndim", u32), ("stride", u32), ("pad", u32),
                ("size", u32 * 8), ("so", i32 * 8), ("sa", i32 * 8)]


class QuantParams(ctypes.Structure):
    _fields_ = [("src", u64), ("dst", u64), ("mask", u64), ("scales", u64), ("zero_points", u64), ("n", u64),
                ("scale_bits", u32), ("zero_point", i32), ("qmin", ctypes.c_int64), ("qmax", ctypes.c_int64),
                ("channels", u32), ("inner", u32), ("dtype", u32), ("pad", u32)]


class MinMaxParams(ctypes.Structure):
    _fields_ = [("src", u64), ("out_min", u64), ("out_max", u64), ("rows", u32), ("cols", u32), ("ld", u32), ("dtype", u32)]


MOVE_COPY, MOVE_FILL = 0, 1


class CastParams(ctypes.Structure):
    _fields_ = [("src", u64), ("dst", u64), ("n", u64), ("src_dtype", u32), ("dst_dtype", u32)]


class F8QuantParams(ctypes.Structure):
    _fields_ = [("src", u64), ("dst", u64), ("scale", u64), ("m", u32), ("k", u32), ("lds", u32), ("ldd", u32),
                ("src_dtype", u32), ("dst_fmt", u32)]


class ProbeParams(ctypes.Structure):
    # "probe_read": dst any valid 4-byte address; geometry 2 reads vkt_qmm4c_bytes(n, k, 32) bytes at src (n a multiple
    # of 16, k of 4096).  "probe_mfma_f8": dst holds at least 80 bytes, 8-byte aligned (clock counts at +64 and +72).
    _fields_ = [("src", u64), ("dst", u64), ("n", u32), ("k", u32), ("iters", u32), ("pad", u32)]


assert ctypes.sizeof(ProbeParams) == 32
assert ctypes.sizeof(Q8Params) == 56 and ctypes.sizeof(Q4Params) == 64 and ctypes.sizeof(F8Params) == 104
assert ctypes.sizeof(CastParams) == 32 and ctypes.sizeof(F8QuantParams) == 48 and ctypes.sizeof(GemmParams) == 112
assert ctypes.sizeof(StridedParams) == 128 and ctypes.sizeof(Copy8Params) == 128 and ctypes.sizeof(QuantParams) == 88 and ctypes.sizeof(MinMaxParams) == 40

# every symbol include/vkt.h declares
SYMBOLS = ["vkt_last_error", "vkt_alloc", "vkt_free", "vkt_synchronize", "vkt_empty_cache", "vkt_memory_stats",
           "vkt_dispatch", "vkt_grid_1d", "vkt_has_float64", "vkt_vendor_id", "vkt_capabilities",
           "vkt_kernel_subgroup_size", "vkt_copy_to_device", "vkt_copy_to_host", "vkt_copy_on_device", "vkt_fill",
           "vkt_device_info", "vkt_event_create", "vkt_event_record", "vkt_event_elapsed_ms", "vkt_event_destroy",
           "vkt_dispatch_count", "vkt_dispatch_static", "vkt_shutdown", "vkt_qmm4c_bytes", "vkt_qmm4c_q_bytes"]

_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no other path."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise VktError(f"{LIB_PATH} is missing: build it with `python -m torch_vulkan_amd.build`")
        L = ctypes.CDLL(LIB_PATH)
        L.vkt_last_error.restype = ctypes.c_char_p
        L.vkt_alloc.argtypes = [u64, ctypes.POINTER(VktAlloc)]
        L.vkt_free.argtypes = [ctypes.c_void_p]
        L.vkt_free.restype = None
        L.vkt_memory_stats.argtypes = [ctypes.POINTER(u64), ctypes.POINTER(u64)]
        L.vkt_memory_stats.restype = None
        L.vkt_dispatch.argtypes = [ctypes.c_char_p, ctypes.POINTER(u32), ctypes.c_size_t, ctypes.c_void_p,
                                   ctypes.c_size_t, u32, u32, u32]
        L.vkt_dispatch_static.argtypes = L.vkt_dispatch.argtypes
        L.vkt_grid_1d.argtypes = [u64, ctypes.POINTER(u32), ctypes.POINTER(u32)]
        L.vkt_vendor_id.restype = u32
        L.vkt_capabilities.restype = u32
        L.vkt_kernel_subgroup_size.argtypes = [ctypes.c_char_p]
        L.vkt_kernel_subgroup_size.restype = u32
        L.vkt_copy_to_device.argtypes = [u64, ctypes.c_void_p, u64]
        L.vkt_copy_to_host.argtypes = [ctypes.c_void_p, u64, u64]
        L.vkt_copy_on_device.argtypes = [u64, u64, u64]
        L.vkt_fill.argtypes = [u64, ctypes.c_uint8, u64]
        L.vkt_device_info.argtypes = [ctypes.POINTER(VktDeviceInfo)]
        L.vkt_event_create.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        L.vkt_event_record.argtypes = [ctypes.c_void_p]
        L.vkt_event_elapsed_ms.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_float)]
        L.vkt_event_destroy.argtypes = [ctypes.c_void_p]
        L.vkt_event_destroy.restype = None
        L.vkt_dispatch_count.restype = u64
        L.vkt_shutdown.restype = None
        L.vkt_qmm4c_bytes.argtypes = [u32, u32, u32]
        L.vkt_qmm4c_bytes.restype = u64
        L.vkt_qmm4c_q_bytes.argtypes = [u32, u32]
        L.vkt_qmm4c_q_bytes.restype = u64
        _lib = L
    return _lib


def check(rc):
    if rc != 0:
        raise VktError("torch_vulkan: " + lib().vkt_last_error().decode(errors="replace"))


class Buffer:
    """A device allocation from the library's pool (vkt_alloc / vkt_free)."""

    def __init__(self, nbytes):
        self._a = VktAlloc()
        check(lib().vkt_alloc(int(nbytes), ctypes.byref(self._a)))
        self.nbytes = int(nbytes)

    @property
    def address(self):
        return self._a.address

    @property
    def size(self):
        return self._a.size

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(max(a.nbytes, 1))
        if a.nbytes:
            check(lib().vkt_copy_to_device(b.address, a.ctypes.data_as(ctypes.c_void_p), a.nbytes))
        return b

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype)
        assert out.nbytes <= self.size
        if out.nbytes:
            check(lib().vkt_copy_to_host(out.ctypes.data_as(ctypes.c_void_p), self.address, out.nbytes))
        return out

    def free(self):
        if self._a.handle:
            lib().vkt_free(self._a.handle)
            self._a.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


STATIC_SCRATCH_BYTES = 16 << 20  # VKT_STATIC_SCRATCH_BYTES


def dispatch(name, spec, params, grid=(1, 1, 1), static=False):
    """vkt_dispatch: kernel `name`, specialisation constants `spec`, parameter block `params`.
    static: through vkt_dispatch_static (the kernels' workspace is the library's fixed array; no allocation)."""
    arr = (u32 * max(len(spec), 1))(*spec)
    gx, gy, gz = (list(grid) + [1, 1])[:3]
    fn = lib().vkt_dispatch_static if static else lib().vkt_dispatch
    check(fn(name.encode(), arr, len(spec), ctypes.byref(params), ctypes.sizeof(params), gx, gy, gz))


def synchronize():
    check(lib().vkt_synchronize())


def device_info():
    info = VktDeviceInfo()
    check(lib().vkt_device_info(ctypes.byref(info)))
    return info


class Event:
    def __init__(self):
        self._e = ctypes.c_void_p()
        check(lib().vkt_event_create(ctypes.byref(self._e)))

    def record(self):
        check(lib().vkt_event_record(self._e))
        return self

    def elapsed_ms(self, stop):
        ms = ctypes.c_float()
        check(lib().vkt_event_elapsed_ms(self._e, stop._e, ctypes.byref(ms)))
        return ms.value

    def __del__(self):
        try:
            lib().vkt_event_destroy(self._e)
        except Exception:
            pass
