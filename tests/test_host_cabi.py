"""CPU-only checks of the host side: the C-ABI library loads and exports every symbol
include/vkt.h declares, the parameter blocks have the reference's sizes, errors follow
the 0 / -1 + vkt_last_error convention, and the pool's policy (best fit, coalescing,
dedicated blocks, trim, out-of-memory retry) behaves as the reference's unit tests expect
of it (crates/vkcore/src/memory.rs:288-327, crates/vkcore/tests/runtime.rs:118-164)."""
import ctypes
import os
import re

import pytest

from torch_vulkan_amd import abi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_exported():
    text = open(os.path.join(ROOT, "include", "vkt.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    declared = sorted(set(re.findall(r"\b(vkt_[a-z0-9_]+)\s*\(", text)))
    assert declared and sorted(abi.SYMBOLS) == declared
    L = abi.lib()
    for name in declared:
        assert getattr(L, name) is not None


def test_parameter_block_sizes():
    # quant.cpp:37,43 static_asserts; at most 128 bytes of push constants (vk.h:386)
    assert ctypes.sizeof(abi.Q8Params) == 56
    assert ctypes.sizeof(abi.Q4Params) == 64
    assert ctypes.sizeof(abi.CastParams) == 32 and ctypes.sizeof(abi.F8QuantParams) == 48
    assert ctypes.sizeof(abi.GemmParams) == 112  # the reference's block (linalg.cpp:25-34)
    assert ctypes.sizeof(abi.StridedParams) == 128 and abi.StridedParams.size.offset == 64  # launch.cpp:28-31
    assert ctypes.sizeof(abi.QuantParams) == 88 and ctypes.sizeof(abi.MinMaxParams) == 40
    assert ctypes.sizeof(abi.Copy8Params) == 128 and abi.Copy8Params.size.offset == 32 and abi.Copy8Params.sa.offset == 96  # :90-91
    for t in (abi.Q4PackParams, abi.Q4CParams, abi.F8Params):
        assert ctypes.sizeof(t) <= 128
    assert ctypes.sizeof(abi.VktAlloc) == 32


def _has_gpu():
    return os.path.exists("/dev/kfd") and os.access("/dev/kfd", os.R_OK | os.W_OK)


@pytest.mark.skipif(_has_gpu(), reason="checks the failure path on a machine without a GPU")
def test_fails_loudly_without_gpu():
    L = abi.lib()
    a = abi.VktAlloc()
    assert L.vkt_alloc(256, ctypes.byref(a)) == -1
    assert b"GPU" in L.vkt_last_error()
    with pytest.raises(abi.VktError, match="no usable GPU"):
        abi.Buffer(16)
    with pytest.raises(abi.VktError):
        abi.dispatch("qmm8_f32", [1], abi.Q8Params())
    # queries degrade as the reference's do without a device (ffi.rs:164-206)
    assert L.vkt_capabilities() == 0 and L.vkt_vendor_id() == 0 and L.vkt_has_float64() == 0
    assert L.vkt_synchronize() == 0 and L.vkt_empty_cache() == 0
    L.vkt_free(None)


def test_compact_sizes():
    L = abi.lib()
    # config 3: nibbles N*K/2 + scales 4*N*K/32 + bias
    n, k = 11008, 4096
    total = L.vkt_qmm4c_bytes(n, k, 32)
    assert n * k // 2 + 4 * n * k // 32 + 4 * n <= total <= n * k // 2 + 4 * n * k // 32 + 4 * n + 512
    assert L.vkt_qmm4c_bytes(n, k, 96) == 0 and L.vkt_qmm4c_bytes(n, k, k) > 0
    # the activation scratch serves either layout: rows * K rounded up to 4096 for the streaming
    # kernel, tiles of 16 rows * K rounded up to 2048 for the matrix-core kernel
    assert L.vkt_qmm4c_q_bytes(1, 4096) == 16 * 4096 and L.vkt_qmm4c_q_bytes(3, 100) == 16 * 2048
    assert L.vkt_qmm4c_q_bytes(40, 8192) == 48 * 8192 and L.vkt_qmm4c_q_bytes(0, 64) == 0


# ------------------------------------------------------------------ pool policy
class FakePool:
    def __init__(self, capacity, block=1 << 20):
        self.L = ctypes.CDLL(os.path.join(os.path.dirname(abi.LIB_PATH), "libvkt_hosttest.so"))
        self.L.vkt_test_pool_new.restype = ctypes.c_void_p
        self.L.vkt_test_pool_new.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
        self.L.vkt_test_pool_alloc.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.POINTER(ctypes.c_uint64)]
        self.L.vkt_test_pool_free.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]
        self.L.vkt_test_pool_trim.argtypes = [ctypes.c_void_p]
        self.L.vkt_test_pool_trim.restype = ctypes.c_uint64
        self.L.vkt_test_pool_stats.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]
        self.L.vkt_test_pool_error.argtypes = [ctypes.c_void_p]
        self.L.vkt_test_pool_error.restype = ctypes.c_char_p
        self.L.vkt_test_pool_delete.argtypes = [ctypes.c_void_p]
        self.p = self.L.vkt_test_pool_new(capacity, block)

    def alloc(self, n):
        out = (ctypes.c_uint64 * 3)()
        if self.L.vkt_test_pool_alloc(self.p, n, out) != 0:
            raise MemoryError(self.L.vkt_test_pool_error(self.p).decode())
        return tuple(out)

    def free(self, a):
        self.L.vkt_test_pool_free(self.p, (ctypes.c_uint64 * 3)(*a))

    def trim(self):
        return self.L.vkt_test_pool_trim(self.p)

    def stats(self):
        out = (ctypes.c_uint64 * 5)()
        self.L.vkt_test_pool_stats(self.p, out)
        return dict(zip(("allocated", "reserved", "blocks", "mapped", "idle_calls"), out))

    def __del__(self):
        self.L.vkt_test_pool_delete(self.p)


def test_pool_alignment_and_reuse():
    p = FakePool(1 << 30)
    a = p.alloc(1)
    b = p.alloc(300)
    assert a[0] % 256 == 0 and b[0] % 256 == 0 and a[1] == 256 and b[1] == 512
    assert b[0] == a[0] + 256 and p.stats()["blocks"] == 1
    p.free(a)
    c = p.alloc(200)  # freed memory is handed out again immediately (stream-ordered reuse)
    assert c[0] == a[0]
    assert p.stats()["allocated"] == 256 + 512


def test_pool_best_fit_and_coalescing():
    p = FakePool(1 << 30)
    xs = [p.alloc(256 * s) for s in (4, 1, 8, 1, 2, 1)]  # sizes in units of 256
    p.free(xs[0]), p.free(xs[2]), p.free(xs[4])  # holes of 4, 8, 2 units
    a = p.alloc(256 * 2)
    assert a[0] == xs[4][0]  # the tightest hole, not the first
    b = p.alloc(256 * 3)
    assert b[0] == xs[0][0]
    p.free(a), p.free(b)
    p.free(xs[1])  # joins holes 0 and 2 through 1: 4 + 1 + 8 units
    c = p.alloc(256 * 13)
    assert c[0] == xs[0][0]
    for x in (xs[3], xs[5], c):
        p.free(x)
    assert p.stats()["allocated"] == 0
    d = p.alloc((1 << 20) // 2)  # the whole block coalesced back: half a block still fits in it
    assert p.stats()["blocks"] == 1 and d[2] == 0


def test_pool_dedicated_blocks_and_trim():
    p = FakePool(1 << 30, block=1 << 20)
    small = p.alloc(1000)
    big = p.alloc(5 << 20)  # larger than half a block: its own block, 2 MiB granule
    assert big[1] == 6 << 20 and big[2] != small[2]
    s = p.stats()
    assert s["blocks"] == 2 and s["reserved"] == (1 << 20) + (6 << 20)
    p.free(big)
    assert p.trim() == 6 << 20  # only the unused block goes back
    assert p.stats()["blocks"] == 1 and p.stats()["mapped"] == 1
    big2 = p.alloc(5 << 20)
    p.free(big2)
    big3 = p.alloc((5 << 20) + 4096)  # a cached dedicated block of sufficient size is reused
    assert big3[0] == big2[0] and p.stats()["blocks"] == 2
    p.free(big3), p.free(small)
    assert p.trim() == (1 << 20) + (6 << 20) and p.stats()["reserved"] == 0


def test_pool_oom_trims_and_retries_once():
    p = FakePool(8 << 20, block=1 << 20)
    a = p.alloc(4 << 20)
    p.free(a)  # cached: 4 MiB reserved, unused
    b = p.alloc(6 << 20)  # does not fit next to the cached block: wait idle, trim, retry
    s = p.stats()
    assert s["idle_calls"] == 1 and s["blocks"] == 1 and s["reserved"] == 6 << 20
    with pytest.raises(MemoryError, match="out of memory"):
        p.alloc(6 << 20)
    p.free(b)
    assert p.stats()["allocated"] == 0


def test_pool_zero_and_huge():
    p = FakePool(1 << 30)
    z = p.alloc(0)
    assert z[1] == 256
    with pytest.raises(MemoryError):
        p.alloc((1 << 64) - 1)


def test_stream_kernel_stride_bound():
    """The stream kernel's per-lane operand offsets are 32-bit (row 255 of a tile at 255 * ld bytes, plus chunk
    offset and bias): strides that would wrap must be refused by the launchers' predicate (kernels/limits.h)."""
    L = ctypes.CDLL(os.path.join(os.path.dirname(abi.LIB_PATH), "libvkt_hosttest.so"))
    L.shim_mma_stream_strides_ok.argtypes = [ctypes.c_uint64, ctypes.c_uint64]
    ok = L.shim_mma_stream_strides_ok
    assert ok(8192, 8192) and ok(28672, 8192) and ok(1 << 20, 64)
    limit = ((1 << 32) - 4096) // 255  # the largest stride whose row 255 still fits with the bias
    assert ok(limit - 1, 16) and ok(16, limit - 1)
    assert not ok(limit + 1, 16) and not ok(16, limit + 1) and not ok(1 << 25, 1 << 25)
    for ld in (limit - 1, limit + 1, 1 << 24, 1 << 31):
        assert bool(ok(ld, 128)) == (255 * ld + 4096 < 1 << 32)


def test_k_slices_leave_no_slice_empty():
    """The launchers that cut K into slices over workgroups take the slice count from kernels/limits.h: every slice
    they launch holds a chunk (the kernels count a slice's chunks in unsigned arithmetic), the slices cover all
    chunks, and never more slices than asked for."""
    L = ctypes.CDLL(os.path.join(os.path.dirname(abi.LIB_PATH), "libvkt_hosttest.so"))
    L.shim_k_slices.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
    L.shim_k_slices.restype = ctypes.c_uint64
    for chunks in list(range(1, 130)) + [224, 448, 1000, 65535]:
        for wanted in list(range(0, 40)) + [64, 1 << 20]:
            r = L.shim_k_slices(chunks, wanted)
            slices, per = r & 0xffffffff, r >> 32
            assert 1 <= slices <= max(wanted, 1) and per >= 1
            assert (slices - 1) * per < chunks <= slices * per, (chunks, wanted, slices, per)
    r = L.shim_k_slices(65, 16)
    assert (r & 0xffffffff, r >> 32) == (13, 5)
