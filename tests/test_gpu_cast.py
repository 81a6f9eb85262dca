"""GPU parity of the float8 steps either side of _scaled_mm, through the C ABI: the elementwise
cast ("cast_fp8") bit for bit against the oracle and PyTorch's CPU Tensor.to() (the reference's
vectors, tests/python/test_fallback_ops.py:469-485, all 256 codes, every rounding midpoint,
large arrays, unaligned addresses), and the producer ("fp8_quant") bit for bit against the
oracle, then end to end into _scaled_mm."""
import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen
from test_oracle_cast import FLOAT8, FMAX, WIDE, every_halfway_point, reference_vectors, torch_producer

pytestmark = pytest.mark.gpu


def same_codes(got, want, dtype):
    """Equal bit for bit, NaNs as NaNs (their payloads are not part of the contract)."""
    gf, wf = oracle.to_f32(got, dtype), oracle.to_f32(want, dtype)
    nan = np.isnan(wf)
    return np.array_equal(got[~nan], want[~nan]) and np.isnan(gf[nan]).all()


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("src", WIDE, ids=str)
@pytest.mark.parametrize("skew", [0, 3])
def test_cast_to_float8(f8, src, skew):
    import _dev
    x = torch.cat([reference_vectors(), torch.from_numpy(every_halfway_point(f8))]).to(src)
    got = _dev.cast(bits(x), ODT[src], ODT[f8], skew=skew)
    assert same_codes(got, oracle.cast(bits(x), ODT[src], ODT[f8]), ODT[f8])
    assert same_codes(got, bits(x.to(f8)), ODT[f8])


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("dst", WIDE + FLOAT8, ids=str)
def test_cast_from_float8(f8, dst):
    import _dev
    if dst == f8:
        pytest.skip("same dtype: a byte copy")
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).repeat(5)[:1237].view(f8)
    for skew in (0, 1):
        got = _dev.cast(bits(codes), ODT[f8], ODT[dst], skew=skew)
        assert same_codes(got, oracle.cast(bits(codes), ODT[f8], ODT[dst]), ODT[dst])
        assert same_codes(got, bits(codes.to(dst)), ODT[dst])


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
def test_cast_large_and_round_trip(f8):
    """16 Mi values: against PyTorch's CPU cast, and float8 -> float32 -> float8 is the identity on codes."""
    import _dev
    x = torch.randn(1 << 24, generator=gen(40)) * torch.tensor([0.01, 1.0, 100.0, 1e4]).repeat(1 << 22)
    got = _dev.cast(x.numpy(), oracle.F32, ODT[f8])
    assert same_codes(got, bits(x.to(f8)), ODT[f8])
    back = _dev.cast(got, ODT[f8], oracle.F32)
    again = _dev.cast(back, oracle.F32, ODT[f8])
    assert same_codes(again, got, ODT[f8])
    assert _dev.cast(np.zeros(0, np.float32), oracle.F32, ODT[f8]).size == 0


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("src", WIDE, ids=str)
@pytest.mark.parametrize("m,k,pad", [(7, 100, 0), (3, 4096, 0), (16, 33, 5), (2, 1, 0), (5, 16384, 16), (3, 20000, 0),
                                     (300, 256, 0), (1, 16, 16)])
def test_producer_rowwise(f8, src, m, k, pad):
    import _dev
    x = (torch.randn(m, k, generator=gen(50 + k)) * (3.0 if k % 2 else 0.02)).to(src)
    if m > 1:
        x[1, k // 2] = float("nan")  # does not take part in the row's scale
        x[0] = 0  # a zero row
    q, s = _dev.fp8_quant(bits(x), ODT[src], ODT[f8], pad=pad)
    wq, ws = oracle.fp8_quant(bits(x), ODT[src], ODT[f8])
    assert np.array_equal(s.view(np.uint32), ws.view(np.uint32))
    assert same_codes(q, wq, ODT[f8])
    if m > 2:  # the rows without NaN: PyTorch's CPU operators, composed
        tq, ts = torch_producer(x[2:], f8)
        assert np.array_equal(s[2:].view(np.uint32), ts.view(np.uint32)) and np.array_equal(q[2:], tq)


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
def test_producer_given_scale(f8):
    import _dev
    x = torch.randn(9, 512, generator=gen(60)) * 4
    for scale in (0.03125, 0.0123):
        q, s = _dev.fp8_quant(x.numpy(), oracle.F32, ODT[f8], scale=scale)
        wq, _ = oracle.fp8_quant(x.numpy(), oracle.F32, ODT[f8], scale=scale)
        assert np.array_equal(q, wq) and s[0] == np.float32(scale)


def test_producer_into_scaled_mm():
    """bfloat16 activations and weights -> rowwise e4m3fn on the device -> _scaled_mm: the product of
    the dequantised operands exactly as the oracle computes it, and within float8 resolution of the
    unquantised product."""
    import _dev
    m, k, n = 96, 1024, 160
    a = (torch.randn(m, k, generator=gen(70)) * 0.5).bfloat16()
    w = (torch.randn(n, k, generator=gen(71)) * 0.05).bfloat16()
    qa, sa = _dev.fp8_quant(bits(a), oracle.BF16, oracle.E4M3)
    qw, sw = _dev.fp8_quant(bits(w), oracle.BF16, oracle.E4M3)
    got = _dev.scaled_mm(qa, oracle.E4M3, qw, oracle.E4M3, sa, sw, True, out_dtype=oracle.F32)
    want, mag = oracle.scaled_mm(qa, oracle.E4M3, qw, oracle.E4M3, sa, sw, True, out_dtype=oracle.F32, want_mag=True)
    assert (np.abs(got.astype(np.float64) - want) <= 2.0**-23 * np.abs(want) + 2.0**-20 * mag).all()
    full = a.double() @ w.double().t()
    scale = (a.double().abs() @ w.double().abs().t()).numpy()
    assert (np.abs(got - full.numpy()) <= 2 * 2.0**-4 * scale / np.sqrt(k) * 4 + 1e-6).all()


def test_cast_errors():
    from torch_vulkan_amd import abi
    buf = abi.Buffer(4096)
    p = abi.CastParams(src=buf.address, dst=buf.address, n=16, src_dtype=abi.F32, dst_dtype=7)
    with pytest.raises(abi.VktError, match="the types are"):
        abi.dispatch("cast_fp8", [], p)
    q = abi.F8QuantParams(src=buf.address, dst=buf.address, scale=buf.address, m=1, k=16, lds=8, ldd=16, src_dtype=abi.F32,
                          dst_fmt=abi.E4M3)
    with pytest.raises(abi.VktError, match="strides"):
        abi.dispatch("fp8_quant", [1], q)
    q.lds = 16
    q.dst_fmt = abi.BF16
    with pytest.raises(abi.VktError, match="e4m3fn / e5m2 out"):
        abi.dispatch("fp8_quant", [1], q)
