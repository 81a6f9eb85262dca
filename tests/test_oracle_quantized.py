"""Pins of the oracle's per-tensor affine quantisation and fake quantisation against PyTorch's CPU
kernels (the x86 build, whose quantize_per_tensor goes through FBGEMM): integers, dequantised values,
fake-quantised outputs and masks bit for bit, on random values, rounding ties, NaN, infinities and
values beyond the integer ranges (the reference's vectors: tests/python/test_fallback_ops.py:972-1004)."""
import numpy as np
import pytest
import torch

import oracle

QT = {oracle.QUINT8: torch.quint8, oracle.QINT8: torch.qint8, oracle.QINT32: torch.qint32}
SPECIAL = [float("nan"), float("inf"), -float("inf"), 0.05, 0.15, -0.05, 1e30, 3e9, -3e9, -1e30, 214748352.0, 12.35, -12.85, 0.25,
           -0.0, 1e-30, 2.5e8, -2.5e8, 2147483520.0, 4e18, -4e18, 9.3e17, 1e19, -1e19]


def values(scale, seed=0):
    g = torch.Generator().manual_seed(seed)
    ties = (torch.arange(-300, 300).float() + 0.5) * scale
    return torch.cat([torch.randn(4000, generator=g) * 20, torch.tensor(SPECIAL), ties, ties + 1e-4, ties - 1e-4])


@pytest.mark.parametrize("qtype", [oracle.QUINT8, oracle.QINT8, oracle.QINT32])
@pytest.mark.parametrize("scale,zp", [(0.1, 5), (0.05, 0), (1.0, -3), (3.7e-3, 100), (2.0**-10, 17)])
def test_quantize_and_dequantize(qtype, scale, zp):
    if qtype == oracle.QUINT8 and zp < 0:
        zp = 3
    x = values(scale)
    want = torch.quantize_per_tensor(x, scale, zp, QT[qtype])
    got = oracle.quantize_affine(x.numpy(), scale, zp, qtype)
    assert np.array_equal(got, want.int_repr().numpy())
    assert np.array_equal(oracle.dequantize_affine(got, scale, zp, qtype), want.dequantize().numpy())


def test_reference_vectors():
    """The reference's own case (test_fallback_ops.py:991-999): scale 0.1, zero point 5."""
    g = torch.Generator().manual_seed(0)
    x = torch.cat([torch.randn(40, generator=g) * 20, torch.tensor([float("nan"), float("inf"), -float("inf"), 0.05, 0.15, -0.05, 1e30, 3e9])])
    for qtype, qd in QT.items():
        c = torch.quantize_per_tensor(x, 0.1, 5, qd)
        q = oracle.quantize_affine(x.numpy(), 0.1, 5, qtype)
        assert np.array_equal(q, c.int_repr().numpy())
        assert np.array_equal(oracle.dequantize_affine(q, 0.1, 5, qtype), c.dequantize().numpy())


def test_dequantize_wraps_like_int32():
    q = np.array([2**31 - 1, -(2**31), 0, 7], np.int32)
    t = torch._make_per_tensor_quantized_tensor(torch.from_numpy(q), 0.5, -5)
    assert np.array_equal(oracle.dequantize_affine(q, 0.5, -5, oracle.QINT32), t.dequantize().numpy())


TD = {oracle.F32: torch.float32, oracle.F16: torch.float16, oracle.BF16: torch.bfloat16}


def as_np(t):
    return t.numpy() if t.dtype == torch.float32 else t.view(torch.int16).numpy().view(np.uint16)


def same(got, want):
    """Bit equality, NaNs matching NaNs."""
    gf, wf = oracle.to_f32(got[0], got[2]), want[0].float().numpy()
    nan = np.isnan(wf)
    assert np.array_equal(np.isnan(gf), nan) and np.array_equal(got[0][~nan], as_np(want[0])[~nan])
    assert np.array_equal(got[1].astype(bool), want[1].numpy())


@pytest.mark.parametrize("dtype", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("scale,zp,qmin,qmax", [(0.05, 3, 0, 255), (0.1, 0, -128, 127), (0.02, -7, -128, 127), (0.5, 250, 0, 255),
                                                (1e-3, 12345, -(2**31), 2**31 - 1), (0.37, -70000, -(2**23), 2**23)])
def test_fake_quant_per_tensor(dtype, scale, zp, qmin, qmax):
    x = values(scale).to(TD[dtype])
    f = torch.ops.aten._fake_quantize_per_tensor_affine_cachemask_tensor_qparams
    want = f(x, torch.tensor([scale]), torch.tensor([zp], dtype=torch.int32), torch.ones(1, dtype=torch.long), qmin, qmax)
    out, mask = oracle.fake_quant(as_np(x), dtype, [scale], np.array([zp], np.int32), qmin, qmax)
    same((out, mask, dtype), want)


@pytest.mark.parametrize("dtype", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("float_zp", [False, True])
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_fake_quant_per_channel(dtype, float_zp, axis):
    x = values(0.05)[:4704].reshape(4, 3, 392).to(TD[dtype])
    c = x.shape[axis]
    g = torch.Generator().manual_seed(3)
    scales = torch.rand(c, generator=g) * 0.2 + 0.01
    zps = (torch.rand(c, generator=g) * 200 + 20) if float_zp else torch.randint(0, 255, (c,), generator=g, dtype=torch.int32)
    want = torch.ops.aten.fake_quantize_per_channel_affine_cachemask(x, scales, zps, axis, 0, 255)
    out, mask = oracle.fake_quant(as_np(x), dtype, scales.numpy(), zps.numpy(), 0, 255, axis=axis)
    same((out, mask, dtype), want)
    # a wide integer range: differences beyond 2^24 are not exact in float32
    if not float_zp:
        zps = zps * 40000 - 3000000
    want = torch.ops.aten.fake_quantize_per_channel_affine_cachemask(x * 1e6, scales, zps, axis, -(2**26), 2**26)
    out, mask = oracle.fake_quant(as_np(x * 1e6), dtype, scales.numpy(), zps.numpy(), -(2**26), 2**26, axis=axis)
    same((out, mask, dtype), want)


@pytest.mark.parametrize("per_row", [False, True])
@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("qrange", [(0, 255), (-128, 127)])
@pytest.mark.parametrize("c", [0.25, 0.01, 0.9])
def test_observer_steps(per_row, symmetric, qrange, c):
    """The QAT observer with fake quantisation as the reference tests it (tests/python/test_fallback_ops.py:947-969),
    over several steps: the running range starts infinite, then moves; every state and output as the CPU's."""
    g = torch.Generator().manual_seed(0)
    size = 4 if per_row else 1
    cpu = [torch.full((size,), float("inf")), torch.full((size,), float("-inf")), torch.ones(size), torch.zeros(size, dtype=torch.int32)]
    rmin, rmax = np.full(size, np.inf, np.float32), np.full(size, -np.inf, np.float32)
    for step in range(5):
        scale_step = [0.1, 1.1, 1e-7, 30.0, 2.1][step]
        x = torch.randn(4, 3, 5, generator=g) * scale_step - 0.5 * step
        out, mask = torch.ops.aten._fused_moving_avg_obs_fq_helper(x, torch.tensor([1]), torch.tensor([1]), cpu[0], cpu[1], cpu[2], cpu[3],
                                                                   c, qrange[0], qrange[1], 0, per_row, symmetric)
        got = oracle.observe_fake_quant(x.numpy(), oracle.F32, rmin, rmax, c, qrange[0], qrange[1], per_row, symmetric)
        assert np.array_equal(rmin, cpu[0].numpy()) and np.array_equal(rmax, cpu[1].numpy())
        assert np.array_equal(got[2], cpu[2].numpy()) and np.array_equal(got[3], cpu[3].numpy())
        assert np.array_equal(got[0], out.numpy()) and np.array_equal(got[1].astype(bool), mask.numpy())


@pytest.mark.parametrize("mn,mx", [(-1.0, 2.0), (0.0, 0.0), (-1e-9, 1e-9), (0.5, 3.0), (-4.0, -1.0), (-1e-6, 0.0), (0.0, 2e-5), (-3e38, 3e38),
                                   (-0.7, 0.7), (-1.0, 1.0), (-2e38, 2e38), (-1e-5, 1e-5), (-1e-5, 3e-5)])
def test_choose_qparams_special_ranges(mn, mx):
    """Ranges that take the special branches (zero range, tiny scale, one-sided), through the CPU observer itself."""
    for sym in (False, True):
        for qr in ((0, 255), (-128, 127)):
            st = [torch.tensor([mn]), torch.tensor([mx]), torch.ones(1), torch.zeros(1, dtype=torch.int32)]
            torch.ops.aten._fused_moving_avg_obs_fq_helper(torch.zeros(2, 2), torch.tensor([0]), torch.tensor([1]), st[0], st[1], st[2], st[3],
                                                           0.25, qr[0], qr[1], 0, False, sym)
            sc, zp = oracle.choose_qparams(mn, mx, qr[0], qr[1], sym)
            assert sc == st[2].item() and zp == st[3].item(), (mn, mx, sym, qr, sc, zp, st[2].item(), st[3].item())
