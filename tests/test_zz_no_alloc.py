"""vkt_dispatch_static, the dispatch entry point that allocates nothing: the kernels' workspace is a fixed array in
the library instead of pool memory.  Its results are compared with vkt_dispatch's on products that are split over
workgroups (so that the workspace is really used), on calls in a row of decreasing size (the array keeps the last
call's contents), and a product whose split needs more than the array holds must be refused."""
import ctypes

import numpy as np
import pytest
import torch

import _dev
import oracle
from _util import bits, gen, ref_tol
from torch_vulkan_amd import abi

pytestmark = pytest.mark.gpu


def _case(m, k, n, seed):
    a = torch.randn(m, k, generator=gen(seed)).bfloat16()
    b = torch.randint(-128, 128, (n, k), dtype=torch.int8, generator=gen(seed + 1))
    s = torch.empty(n).uniform_(0.005, 0.02, generator=gen(seed + 2)).bfloat16()
    return bits(a), b.numpy(), bits(s)


def test_static_dispatch_matches_dispatch():
    abi.device_info()  # starts the runtime: the static entry point does not
    # 64 rows x 8 slices of K (tile kernel + finish: 8.4 MB of partial sums), then smaller products: 40 rows on the
    # same kernels, and 16 rows on the kernel whose workgroups write whole matrix-core tiles to the workspace
    for i, (m, k, n) in enumerate([(64, 14336, 4096), (40, 4096, 1024), (16, 14336, 4096)]):
        a, b, s = _case(m, k, n, 100 + 10 * i)
        want = _dev.qmm8(a, oracle.BF16, b, s)
        got = _dev.qmm8(a, oracle.BF16, b, s, static=True)
        assert np.array_equal(got, want), (m, k, n)
        if m == 40:  # against the oracle too
            _, c64, mag = oracle.qmm8(a, oracle.BF16, b, s, want_f64=True)
            assert (np.abs(oracle.bf16_to_f32(got) - c64) <= ref_tol(c64, mag, oracle.BF16)).all()


def test_static_dispatch_few_row_products_in_slices():
    """The few-row kernel of the float8 and 16-bit products cuts K into slices over workgroups where columns are few,
    their tiles in the workspace: the same outputs from the fixed array, on calls in a row of decreasing size."""
    abi.device_info()
    for i, (m, k, n) in enumerate([(64, 8192, 2048), (32, 8192, 1024), (8, 4096, 1024)]):
        a = bits((torch.randn(m, k, generator=gen(300 + i)) * 0.5).bfloat16())
        w = bits((torch.randn(n, k, generator=gen(310 + i)) * 0.5).bfloat16())
        want = _dev.gemm16(a, w.T, oracle.BF16, variant=7 | 2 << 8 | 4 << 12)
        assert np.array_equal(_dev.gemm16(a, w.T, oracle.BF16, variant=7 | 2 << 8 | 4 << 12, static=True), want), (m, k, n)
        assert np.array_equal(_dev.gemm16(a, w.T, oracle.BF16, static=True), _dev.gemm16(a, w.T, oracle.BF16)), (m, k, n)
        a8 = bits((torch.randn(m, k, generator=gen(320 + i))).to(torch.float8_e4m3fn))
        w8 = bits((torch.randn(n, k, generator=gen(330 + i))).to(torch.float8_e4m3fn))
        sa, sb = np.full(m, 0.5, np.float32), np.full(n, 1.5, np.float32)
        for variant in (12 | 1 << 8 | 8 << 12, 0):
            want = _dev.scaled_mm(a8, oracle.E4M3, w8, oracle.E4M3, sa, sb, True, variant=variant)
            assert np.array_equal(_dev.scaled_mm(a8, oracle.E4M3, w8, oracle.E4M3, sa, sb, True, variant=variant, static=True), want), (m, k, n)
    # the int8 op against few columns: 16-bit rows, and float32 rows (three bfloat16 planes, the slices' tiles behind them)
    for i, (m, k, n) in enumerate([(16, 8192, 1024), (8, 4096, 520)]):
        a, b, s = _case(m, k, n, 350 + 10 * i)
        assert np.array_equal(_dev.qmm8(a, oracle.BF16, b, s, static=True), _dev.qmm8(a, oracle.BF16, b, s)), (m, k, n)
        a32 = torch.randn(m, k, generator=gen(360 + i)).numpy()
        s32 = torch.empty(n).uniform_(0.005, 0.02, generator=gen(370 + i)).numpy()
        assert np.array_equal(_dev.qmm8(a32, oracle.F32, b, s32, static=True), _dev.qmm8(a32, oracle.F32, b, s32)), (m, k, n)
    # 65 rows and more against few tiles: the tile kernel with K in slices, its partial sums in the array (both entry
    # points plan against the array's size, so their outputs are the same bits)
    for i, (m, k, n) in enumerate([(256, 8192, 2048), (128, 4096, 1024)]):
        a = bits((torch.randn(m, k, generator=gen(380 + i)) * 0.5).bfloat16())
        w = bits((torch.randn(n, k, generator=gen(385 + i)) * 0.5).bfloat16())
        assert np.array_equal(_dev.gemm16(a, w.T, oracle.BF16, static=True), _dev.gemm16(a, w.T, oracle.BF16)), (m, k, n)
        a8 = bits((torch.randn(m, k, generator=gen(390 + i))).to(torch.float8_e4m3fn))
        w8 = bits((torch.randn(n, k, generator=gen(395 + i))).to(torch.float8_e4m3fn))
        sa, sb = np.full(m, 0.5, np.float32), np.full(n, 1.5, np.float32)
        want = _dev.scaled_mm(a8, oracle.E4M3, w8, oracle.E4M3, sa, sb, True)
        assert np.array_equal(_dev.scaled_mm(a8, oracle.E4M3, w8, oracle.E4M3, sa, sb, True, static=True), want), (m, k, n)
    # more partial sums than the array holds: refused, not re-planned
    m, k, n = 64, 8192, 16384
    a = bits((torch.randn(m, k, generator=gen(340)) * 0.5).bfloat16())
    w = bits((torch.randn(n, k, generator=gen(341)) * 0.5).bfloat16())
    assert (n // 32) * 31 * 4 * 2 * 1024 > abi.STATIC_SCRATCH_BYTES
    with pytest.raises(abi.VktError, match="fixed workspace holds"):
        _dev.gemm16(a, w.T, oracle.BF16, variant=7 | 2 << 8 | 31 << 12, static=True)


def test_static_dispatch_refuses_more_than_the_array_holds():
    abi.device_info()
    a, b, s = _case(64, 4096, 4096, 200)
    forced = (1 << 21) | (32 << 24)  # the tile kernel with 32 slices of K: 32 x 64 x 4096 x 4 bytes of partial sums
    assert 32 * 64 * 4096 * 4 > abi.STATIC_SCRATCH_BYTES
    with pytest.raises(abi.VktError, match="fixed workspace holds"):
        _dev.qmm8(a, oracle.BF16, b, s, variant=forced, static=True)
    # the same call through vkt_dispatch runs (with as many slices as its workspace holds), and the static entry
    # point still works afterwards
    want = _dev.qmm8(a, oracle.BF16, b, s, variant=forced)
    got = _dev.qmm8(a, oracle.BF16, b, s, static=True)
    _, c64, mag = oracle.qmm8(a, oracle.BF16, b, s, want_f64=True)
    for out in (want, got):
        assert (np.abs(oracle.bf16_to_f32(out) - c64) <= ref_tol(c64, mag, oracle.BF16)).all()


def _memory():
    a, r = abi.u64(), abi.u64()
    abi.lib().vkt_memory_stats(ctypes.byref(a), ctypes.byref(r))
    return a.value, r.value


def test_static_dispatch_allocates_nothing():
    """With the pool's kernel memory given back (vkt_empty_cache drops the workspace that vkt_dispatch had taken), a
    static dispatch of a split product leaves the pool's figures as they were, and its result stands against the oracle
    without vkt_dispatch having run in between."""
    abi.device_info()
    m, k, n = 64, 14336, 4096
    a, b, s = _case(m, k, n, 300)
    da, db, ds = abi.Buffer.from_numpy(a), abi.Buffer.from_numpy(b), abi.Buffer.from_numpy(s)
    dc = abi.Buffer(m * n * 2)
    p = abi.Q8Params(a=da.address, b=db.address, scales=ds.address, c=dc.address, m=m, n=n, k=k, a_sm=k, a_sk=1)
    abi.check(abi.lib().vkt_empty_cache())
    before = _memory()
    abi.dispatch("qmm8_bf16", [0, 0], p, ((n + 63) // 64, 1), static=True)
    abi.synchronize()
    assert _memory() == before
    got = dc.to_numpy(np.uint16, (m, n))
    _, c64, mag = oracle.qmm8(a, oracle.BF16, b, s, want_f64=True)
    assert (np.abs(oracle.bf16_to_f32(got) - c64) <= ref_tol(c64, mag, oracle.BF16)).all()


def test_static_dispatch_aminmax():
    """The other user of the workspace: row ranges whose rows are split over workgroups (partial ranges meet in the
    workspace).  Two calls in a row, the second smaller; equal to vkt_dispatch's and to numpy's."""
    abi.device_info()
    for rows, cols, seed in ((3, 300000, 7), (2, 70000, 8)):
        x = (torch.randn(rows, cols, generator=gen(seed)) * 3).numpy()
        want = _dev.aminmax(x, oracle.F32)
        got = _dev.aminmax(x, oracle.F32, static=True)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
        assert np.array_equal(got[0], x.min(axis=1)) and np.array_equal(got[1], x.max(axis=1))
