"""Pins of the oracle's float8 cast and producer (CPU only): orc_cast against PyTorch's CPU
Tensor.to() on the reference's own vectors (tests/python/test_fallback_ops.py:469-485: values
that round, saturate, overflow, NaN, inf, -0) and all 256 codes; orc_fp8_quant_rows against
the same steps composed from PyTorch CPU operators and against closed forms."""
import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen

FLOAT8 = [torch.float8_e4m3fn, torch.float8_e5m2]
WIDE = [torch.float32, torch.float16, torch.bfloat16]
FMAX = {torch.float8_e4m3fn: 448.0, torch.float8_e5m2: 57344.0}


def reference_vectors():
    special = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 448.0, 464.0, 465.0, 479.9, 480.0,
                            57344.0, 61440.0, 61441.0, 65536.0, 1e-9, -1e-9, 2.0 ** -9, 2.0 ** -10, 2.0 ** -17, 1e30,
                            2.0 ** -6, 2.0 ** -7, 1.5 * 2.0 ** -10, 2.5 * 2.0 ** -10, 2.0 ** -14, 2.0 ** -16, 1.5 * 2.0 ** -17])
    return torch.cat([torch.randn(300, generator=gen(1)) * 3, torch.randn(300, generator=gen(2)) * 300,
                      torch.randn(300, generator=gen(3)) * 60000, special, -special])


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("src", WIDE, ids=str)
def test_cast_to_float8(f8, src):
    x = reference_vectors().to(src)
    want = bits(x.to(f8))
    assert np.array_equal(oracle.cast(bits(x), ODT[src], ODT[f8]), want)


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("dst", WIDE + FLOAT8, ids=str)
def test_cast_from_float8_all_codes(f8, dst):
    if dst == f8:
        pytest.skip("same dtype: a byte copy")
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(f8)
    want = bits(codes.to(dst))
    got = oracle.cast(bits(codes), ODT[f8], ODT[dst])
    nan = np.isnan(oracle.to_f32(want, ODT[dst]))
    assert np.array_equal(got[~nan], want[~nan]) and np.isnan(oracle.to_f32(got, ODT[dst])[nan]).all()


def every_halfway_point(f8):
    """All midpoints between adjacent finite float8 values (the rounding decisions), and their float32 neighbours."""
    table = oracle.fp8_table(ODT[f8])
    finite = np.sort(np.unique(table[np.isfinite(table)]))
    mid = ((finite[:-1].astype(np.float64) + finite[1:]) / 2).astype(np.float32)
    return np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf))])


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
def test_cast_halfway_points(f8):
    x = torch.from_numpy(every_halfway_point(f8))
    assert np.array_equal(oracle.cast(x.numpy(), oracle.F32, ODT[f8]), bits(x.to(f8)))


def torch_producer(x, f8, scale=None):
    """The producer's steps with PyTorch's CPU operators (each a single float32 operation)."""
    fmax = torch.tensor(FMAX[f8], dtype=torch.float32)
    xf = x.float()
    if scale is None:
        a = torch.clamp(xf.abs().amax(dim=1, keepdim=True), min=1e-12)
        scales = torch.true_divide(a, fmax)
    else:
        scales = torch.tensor([[scale]], dtype=torch.float32)
        a = scales * fmax
    inv = torch.true_divide(fmax, a)
    y = torch.clamp(xf * inv, -FMAX[f8], FMAX[f8])
    return bits(y.to(f8)), scales.reshape(-1).numpy()


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("src", WIDE, ids=str)
@pytest.mark.parametrize("m,k,spread", [(7, 100, 1.0), (3, 4096, 30.0), (16, 33, 1e-3), (2, 1, 5.0)])
def test_producer_rowwise_vs_torch(f8, src, m, k, spread):
    x = (torch.randn(m, k, generator=gen(10 + k)) * spread).to(src)
    q, s = oracle.fp8_quant(bits(x), ODT[src], ODT[f8])
    wq, ws = torch_producer(x, f8)
    assert np.array_equal(s.view(np.uint32), ws.view(np.uint32))
    assert np.array_equal(q, wq)


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
def test_producer_given_scale_vs_torch(f8):
    x = torch.randn(5, 64, generator=gen(20)) * 4
    for scale in (0.03125, 0.0123, 1.0):
        q, s = oracle.fp8_quant(x.numpy(), oracle.F32, ODT[f8], scale=scale)
        wq, _ = torch_producer(x, f8, scale=scale)
        assert np.array_equal(q, wq) and s[0] == np.float32(scale)


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
def test_producer_closed_forms(f8):
    fmax = FMAX[f8]
    # a row whose maximum is fmax: scale 1, the producer is the plain cast
    x = torch.randn(4, 200, generator=gen(30)) * 20
    x[:, 0] = fmax
    x = x.clamp(-fmax, fmax)
    q, s = oracle.fp8_quant(x.numpy(), oracle.F32, ODT[f8])
    assert (s == 1.0).all() and np.array_equal(q, bits(x.to(f8)))
    # rescaling the input by a power of two changes the scale by that factor and no code
    q2, s2 = oracle.fp8_quant((x * 0.125).numpy(), oracle.F32, ODT[f8])
    assert np.array_equal(q2, q) and np.array_equal(s2, s * 0.125)
    # zero rows: scale 1e-12 / fmax, all codes zero; the largest magnitude of a row maps to +-fmax
    q0, s0 = oracle.fp8_quant(np.zeros((2, 16), np.float32), oracle.F32, ODT[f8])
    assert (q0 == 0).all() and np.array_equal(s0, np.full(2, np.float32(1e-12) / np.float32(fmax), np.float32))
    y = torch.randn(6, 50, generator=gen(31))
    qy, _ = oracle.fp8_quant(y.numpy(), oracle.F32, ODT[f8])
    top = np.abs(oracle.fp8_table(ODT[f8])[qy]).max(axis=1)
    assert (top == fmax).all()
    # NaN elements do not take part in the scale and stay NaN
    z = y.clone()
    z[1, 3] = float("nan")
    qz, sz = oracle.fp8_quant(z.numpy(), oracle.F32, ODT[f8])
    keep = np.ones(50, bool)
    keep[3] = False
    assert np.isnan(oracle.fp8_table(ODT[f8])[qz[1, 3]]) and np.array_equal(qz[0], qy[0])
    y_wo = y.clone()
    y_wo[1, 3] = 0.0
    qw, sw = oracle.fp8_quant(y_wo.numpy(), oracle.F32, ODT[f8])
    assert sz[1] == sw[1] and np.array_equal(qz[1][keep], qw[1][keep])
