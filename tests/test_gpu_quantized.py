"""GPU parity of the per-tensor affine quantisation kernels ("quantize_affine", "dequantize_affine",
"fake_quant") through the C ABI: bit for bit against the oracle (itself pinned against PyTorch's CPU
kernels) and against PyTorch's CPU operators directly, on random values, rounding ties, NaN, infinities
and values beyond the integer ranges (the reference's vectors: tests/python/test_fallback_ops.py:972-1004)."""
import numpy as np
import pytest
import torch

import oracle
from test_oracle_quantized import QT, TD, as_np, values

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("skew", [0, 1])
@pytest.mark.parametrize("qtype", [oracle.QUINT8, oracle.QINT8, oracle.QINT32])
@pytest.mark.parametrize("scale,zp", [(0.1, 5), (0.05, 0), (1.0, 3), (3.7e-3, 100)])
def test_quantize_and_dequantize(qtype, scale, zp, skew):
    import _dev
    x = values(scale)
    want = oracle.quantize_affine(x.numpy(), scale, zp, qtype)
    got = _dev.quantize_affine(x.numpy(), scale, zp, qtype, skew=skew)
    assert np.array_equal(got, want)
    cpu = torch.quantize_per_tensor(x, scale, zp, QT[qtype])
    assert np.array_equal(got, cpu.int_repr().numpy())
    back = _dev.dequantize_affine(got, scale, zp, qtype, skew=skew)
    assert np.array_equal(back, oracle.dequantize_affine(want, scale, zp, qtype)) and np.array_equal(back, cpu.dequantize().numpy())


def test_dequantize_wraps_like_int32():
    import _dev
    q = np.array([2**31 - 1, -(2**31), 0, 7], np.int32)
    assert np.array_equal(_dev.dequantize_affine(q, 0.5, -5, oracle.QINT32), oracle.dequantize_affine(q, 0.5, -5, oracle.QINT32))


def same_bits(got, want, dtype):
    nan = np.isnan(oracle.to_f32(want[0], dtype))
    assert np.array_equal(np.isnan(oracle.to_f32(got[0], dtype)), nan)
    assert np.array_equal(got[0][~nan], want[0][~nan]) and np.array_equal(got[1], want[1])


@pytest.mark.parametrize("skew", [0, 3])
@pytest.mark.parametrize("dtype", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("scale,zp,qmin,qmax", [(0.05, 3, 0, 255), (0.1, 0, -128, 127), (0.02, -7, -128, 127),
                                                (1e-3, 12345, -(2**31), 2**31 - 1)])
def test_fake_quant_per_tensor(dtype, scale, zp, qmin, qmax, skew):
    import _dev
    x = as_np(values(scale).to(TD[dtype]))
    want = oracle.fake_quant(x, dtype, [scale], np.array([zp], np.int32), qmin, qmax)
    got = _dev.fake_quant(x, dtype, [scale], np.array([zp], np.int32), qmin, qmax, skew=skew)
    same_bits(got, want, dtype)


@pytest.mark.parametrize("dtype", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("float_zp", [False, True])
@pytest.mark.parametrize("axis", [0, 1, 2])
def test_fake_quant_per_channel(dtype, float_zp, axis):
    import _dev
    xt = values(0.05)[:4704].reshape(4, 3, 392).to(TD[dtype])
    c = xt.shape[axis]
    g = torch.Generator().manual_seed(3)
    scales = torch.rand(c, generator=g) * 0.2 + 0.01
    zps = (torch.rand(c, generator=g) * 200 + 20) if float_zp else torch.randint(0, 255, (c,), generator=g, dtype=torch.int32)
    for factor, lo, hi in ((1.0, 0, 255), (1e6, -(2**26), 2**26)):
        x = as_np((xt * factor).to(TD[dtype]))
        want = oracle.fake_quant(x, dtype, scales.numpy(), zps.numpy(), lo, hi, axis=axis)
        got = _dev.fake_quant(x, dtype, scales.numpy(), zps.numpy(), lo, hi, axis=axis)
        same_bits(got, want, dtype)
    cpu = torch.ops.aten.fake_quantize_per_channel_affine_cachemask(xt, scales, zps, axis, 0, 255)
    got = _dev.fake_quant(as_np(xt), dtype, scales.numpy(), zps.numpy(), 0, 255, axis=axis)
    same_bits(got, (as_np(cpu[0]), cpu[1].numpy().astype(np.uint8)), dtype)


def test_fake_quant_large_against_cpu():
    """8 Mi random float32 values with a float zero point per channel: every output and mask bit as the CPU's
    (the fused multiply-add of the float zero-point form shows in about one value per million)."""
    import _dev
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, 1 << 21, generator=g) * 3
    scales, zps = torch.tensor([0.0123, 0.0371, 0.05, 0.1]), torch.tensor([3.37, 100.61, 17.5, 200.123])
    cpu = torch.ops.aten.fake_quantize_per_channel_affine_cachemask(x, scales, zps, 0, 0, 255)
    got = _dev.fake_quant(x.numpy(), oracle.F32, scales.numpy(), zps.numpy(), 0, 255, axis=0)
    assert np.array_equal(got[0], cpu[0].numpy()) and np.array_equal(got[1].astype(bool), cpu[1].numpy())
    f = torch.ops.aten._fake_quantize_per_tensor_affine_cachemask_tensor_qparams
    cpu = f(x, torch.tensor([0.0123]), torch.tensor([3], dtype=torch.int32), torch.ones(1, dtype=torch.long), 0, 255)
    got = _dev.fake_quant(x.numpy(), oracle.F32, [0.0123], np.array([3], np.int32), 0, 255)
    assert np.array_equal(got[0], cpu[0].numpy()) and np.array_equal(got[1].astype(bool), cpu[1].numpy())


@pytest.mark.parametrize("dtype", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("rows,cols,ld", [(1, 1, 1), (1, 60, 60), (4, 15, 15), (3, 5000, 5000), (1, 300000, 300000), (7, 70001, 70004), (600, 33, 40),
                                           (2, 1 << 21, 1 << 21)])
def test_aminmax(dtype, rows, cols, ld):
    """Row-wise minimum and maximum as torch.aminmax(x, dim=1) (exact: a selection), NaN rows included."""
    import _dev
    x = (torch.randn(rows, cols, generator=torch.Generator().manual_seed(rows + cols)) * 10).to(TD[dtype])
    if rows > 1 and cols > 3:
        x[1, cols // 2] = float("nan")
        x[0, cols - 1] = 1e4
    lo, hi = _dev.aminmax(as_np(x), dtype, ld=ld)
    want = torch.aminmax(x.float(), dim=1)
    assert np.array_equal(lo, want.min.numpy(), equal_nan=True) and np.array_equal(hi, want.max.numpy(), equal_nan=True)


def test_errors():
    from torch_vulkan_amd import abi
    buf = abi.Buffer(4096)
    p = abi.QuantParams(src=buf.address, dst=buf.address, mask=buf.address, n=16, qmin=0, qmax=255)
    with pytest.raises(abi.VktError, match="QTYPE"):
        abi.dispatch("quantize_affine", [3], p)
    with pytest.raises(abi.VktError, match="per channel needs"):
        abi.dispatch("fake_quant", [1, 0], p)
    with pytest.raises(abi.VktError, match="only per channel"):
        abi.dispatch("fake_quant", [0, 1], p)
    p.qmin = 300
    with pytest.raises(abi.VktError, match="qmin above qmax"):
        abi.dispatch("fake_quant", [0, 0], p)
    p.src = 0
    with pytest.raises(abi.VktError, match="null or misaligned"):
        abi.dispatch("dequantize_affine", [0], p)
