"""Pins of the oracle's 16-bit matrix product (CPU only): against the float64 closed form by
numpy, against PyTorch's CPU float32 product of the same 16-bit values inside the reference
test's bound (tests/python/test_matmul.py:250-264), and on cases whose result is exact."""
import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen

DTYPES = [torch.bfloat16, torch.float16]


def as_f64(t):
    return t.double().numpy()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("m,k,n", [(5, 16, 7), (17, 200, 9), (3, 1000, 5), (8, 1, 6)])
def test_gemm16_closed_form_and_torch(dtype, m, k, n):
    a = torch.randn(m, k, generator=gen(1)).to(dtype)
    b = torch.randn(k, n, generator=gen(2)).to(dtype)
    got, mag = oracle.gemm16(bits(a), bits(b), ODT[dtype], want_mag=True)
    exact = as_f64(a) @ as_f64(b)
    assert np.allclose(mag, np.abs(as_f64(a)) @ np.abs(as_f64(b)), rtol=1e-12)
    gf = oracle.to_f32(got, ODT[dtype]).astype(np.float64)
    eps = torch.finfo(dtype).eps
    # one rounding of the exact sum: within half an ulp (eps/2 relative, plus the 16-bit subnormal step)
    assert (np.abs(gf - exact) <= eps / 2 * np.abs(exact) + 2.0**-25).all()
    want = (a.float() @ b.float()).to(dtype).float().numpy()
    assert (np.abs(gf - want) <= eps * np.maximum(np.abs(want), 2.0**-14) + 2.0**-20 * mag).all()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_layouts_alpha_beta_batches(dtype):
    a = torch.randn(3, 6, 20, generator=gen(3)).to(dtype)
    b = torch.randn(3, 20, 9, generator=gen(4)).to(dtype)
    bias = torch.randn(9, generator=gen(5)).to(dtype)
    base = oracle.gemm16(bits(a), bits(b), ODT[dtype])
    # column-major operands and strided views give the same values
    at = bits(a.transpose(1, 2).contiguous()).transpose(0, 2, 1)
    bt = bits(b.transpose(1, 2).contiguous()).transpose(0, 2, 1)
    assert np.array_equal(oracle.gemm16(at, bt, ODT[dtype]), base)
    assert np.array_equal(oracle.gemm16(bits(a)[:, ::2], bits(b), ODT[dtype]), base[:, ::2])
    got = oracle.gemm16(bits(a), bits(b), ODT[dtype], cin=bits(bias), alpha=2.0, beta=0.5)
    exact = 2.0 * (as_f64(a) @ as_f64(b)) + 0.5 * as_f64(bias)
    eps = torch.finfo(dtype).eps
    assert (np.abs(oracle.to_f32(got, ODT[dtype]) - exact) <= eps / 2 * np.abs(exact) + 2.0**-25).all()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_exact_cases(dtype):
    # small integers: every product and sum is exact in the 16-bit type
    a = torch.randint(-4, 5, (7, 12), generator=gen(6)).to(dtype)
    b = torch.randint(-4, 5, (12, 5), generator=gen(7)).to(dtype)
    want = (a.double() @ b.double()).to(dtype)
    assert np.array_equal(oracle.gemm16(bits(a), bits(b), ODT[dtype]), bits(want))
    # identity and a power-of-two alpha
    x = torch.randn(6, 6, generator=gen(8)).to(dtype)
    eye = torch.eye(6).to(dtype)
    assert np.array_equal(oracle.gemm16(bits(x), bits(eye), ODT[dtype]), bits(x))
    assert np.array_equal(oracle.gemm16(bits(x), bits(eye), ODT[dtype], alpha=0.25), bits((x.float() * 0.25).to(dtype)))
