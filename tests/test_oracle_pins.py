"""Pins the CPU oracle (oracle/qmm_oracle.c) before anything trusts it.

The reference's own tests hold no golden files for this path: every expectation in
tests/python/test_quant.py is computed live from PyTorch's CPU kernels, which is where the
arithmetic truth lives.  So each oracle function is checked here against (i) the torch CPU
op on the reference's own parametrisations and seeds, (ii) the frozen fixtures in
tests/golden/, and (iii) checks the mathematics fixes (closed forms, brute force on tiny
inputs, exactly representable cases), chosen so that a dropped term, a wrong nibble order,
a transposed operand or a wrong rounding mode fails at least one of them."""
import os

import numpy as np
import pytest
import torch

import oracle
from _cases import FLOAT8, FLOAT8_OUT, FLOAT8_PAIRS, INT4_SHAPES, INT8_SHAPES, float8_case, int4_rows, int4_weights, int8_case
from _util import ODT, bits, gen, ref_tol, unbits

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


# ------------------------------------------------------------------ casts
@pytest.mark.parametrize("dtype", FLOAT8)
def test_fp8_decode_all_codes(dtype):
    # reference tests/python/test_fallback_ops.py:469-485: all 256 codes, bit-exact
    want = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(dtype).float().numpy()
    got = oracle.fp8_table(ODT[dtype])
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def _halfway_probe(dtype):
    """Every representable value, every midpoint between neighbours, and one float32 ulp
    either side of each midpoint; plus saturation, NaN, infinities, -0, denormals."""
    vals = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(dtype).float()
    vals = vals[torch.isfinite(vals)].unique().double()
    mids = (vals[1:] + vals[:-1]) / 2
    pts = torch.cat([vals, mids]).float()
    u = pts.view(torch.int32)
    pts = torch.cat([pts, (u + 1).view(torch.float32), (u - 1).view(torch.float32)])
    extra = torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 1e-45, -1e-45, 1e-30, 448.0, 463.9,
                          464.0, 464.1, 479.9, 480.0, 1e6, -1e6, 57344.0, 61439.9, 61440.0, 61440.1, 65535.9, 65536.0,
                          3.4e38, 2.0**-9, 2.0**-10, 2.0**-10 * 1.0001, 2.0**-17, 2.0**-16, 2.0**-17 * 1.0001])
    return torch.cat([pts, extra])


@pytest.mark.parametrize("dtype", FLOAT8)
def test_fp8_encode_matches_torch(dtype):
    x = _halfway_probe(dtype)
    want = x.to(dtype).view(torch.uint8).numpy()
    got = oracle.f32_to_fp8(x.numpy(), ODT[dtype])
    nan = torch.isnan(x).numpy()
    assert np.array_equal(got[~nan], want[~nan])
    assert np.array_equal(got[nan] & 0x7F, want[nan] & 0x7F)
    g = torch.randn(20000, generator=gen(5)) * torch.tensor(10.0) ** torch.randint(-6, 6, (20000,), generator=gen(6))
    assert np.array_equal(oracle.f32_to_fp8(g.numpy(), ODT[dtype]), g.to(dtype).view(torch.uint8).numpy())


def test_f16_bf16_encode_matches_torch():
    g = torch.randn(20000, generator=gen(7)) * torch.tensor(10.0) ** torch.randint(-9, 6, (20000,), generator=gen(8))
    edge = torch.tensor([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0001, 2.0**-26,
                         float("inf"), -float("inf"), 6.1e-5, 6.0e-8, 1.00048828125, 1.0009765625 + 2.0**-11])
    x = torch.cat([g, edge])
    assert np.array_equal(oracle.f32_to_f16(x.numpy()), bits(x.half()))
    assert np.array_equal(oracle.f32_to_bf16(x.numpy()), bits(x.bfloat16()))
    assert oracle.f32_to_bf16(np.float32("nan")) == 0x7FC0


# ------------------------------------------------------------------ int8
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", INT8_SHAPES)
def test_qmm8_vs_closed_form_and_torch(dtype, m, k, n):
    a, b, s = int8_case(dtype, m, k, n)
    odt = ODT[dtype]
    c, c64, mag = oracle.qmm8(bits(a), odt, b.numpy(), bits(s), want_f64=True)
    # closed form of the reference's test (test_quant.py:32): float64 here
    w = (b.float() * s.float()[:, None]).double()
    truth = (a.double() @ w.t()).numpy()
    assert np.allclose(c64, truth, rtol=1e-12, atol=1e-12)
    assert np.allclose(mag, (a.double().abs() @ w.abs().t()).numpy(), rtol=1e-12)
    got = unbits(c, dtype).float().numpy()
    want = torch.from_numpy(truth).to(dtype).float().numpy()
    assert np.array_equal(got, want)  # one rounding of the float64 sum
    # the torch CPU op (its bf16 path needs K % 16 == 0: test_quant.py:28-31)
    if dtype == torch.float32 or k % 16 == 0:
        cpu = torch._weight_int8pack_mm(a, b, s).float().numpy()
        assert (np.abs(cpu - truth) <= ref_tol(truth, mag, odt) * 2).all()
    # the reference's own float32 summation order sits inside the band
    ordered = unbits(oracle.qmm8_f32order(bits(a), odt, b.numpy(), bits(s)), dtype).float().numpy()
    assert (np.abs(ordered - truth) <= ref_tol(truth, mag, odt)).all()
    # a row slice of A (test_quant.py:35) is read in place
    sliced = oracle.qmm8(bits(a)[::2], odt, b.numpy(), bits(s))
    assert np.array_equal(sliced, c[::2])


def test_qmm8_brute_force_tiny():
    # integers small enough that every float32 operation is exact
    a = np.array([[1.0, -2.0, 3.0], [0.5, 4.0, -1.0]], np.float32)
    b = np.array([[1, 2, 3], [-128, 127, 0], [5, -5, 5], [0, 0, 1]], np.int8)
    s = np.array([1.0, 0.5, 2.0, 0.25], np.float32)
    want = np.zeros((2, 4))
    for m in range(2):
        for n in range(4):
            want[m, n] = sum(float(a[m, k]) * (float(b[n, k]) * float(s[n])) for k in range(3))
    assert np.array_equal(oracle.qmm8(a, oracle.F32, b, s).astype(np.float64), want)
    # not symmetric in (m, n): a transposed operand would fail
    assert want[0, 1] != want[1, 0]


# ------------------------------------------------------------------ int4
@pytest.mark.parametrize("m,k,n,bs,bias", INT4_SHAPES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_q4_bit_exact_vs_torch_cpu(m, k, n, bs, bias, dtype):
    if dtype == torch.bfloat16 and bs != k:
        pytest.skip("bfloat16 inputs are channelwise only (the CPU's check)")
    w, sc, bvec = int4_weights(n, k, bs, bias=bias)
    x = int4_rows(m, k, dtype)
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, bvec, bs, k, n)
    want = torch._dyn_quant_matmul_4bit(x, packed, bs, k, n)
    mine = oracle.q4_pack(w.numpy(), bits(sc), ODT[sc.dtype], None if bvec is None else bvec.numpy())
    assert np.array_equal(mine.view(np.uint32), packed.numpy().view(np.uint32))
    got, iacc = oracle.q4_matmul(bits(x), ODT[dtype], mine, bs, k, n, want_iacc=True)
    assert np.array_equal(got, bits(want))
    # the int32 block sums by brute force from the oracle's own row quantisation
    q, recip, nzp = oracle.q4_rowquant(bits(x), ODT[dtype], bs != k)
    wn = w.numpy()
    nib = np.empty((n, k), np.int64)
    nib[:, 0::2] = wn & 15
    nib[:, 1::2] = wn >> 4
    nib -= 8
    qz = q.astype(np.int64) + nzp[:, None]
    nblocks = (k + bs - 1) // bs
    brute = np.stack([qz[:, i * bs:(i + 1) * bs] @ nib[:, i * bs:(i + 1) * bs].T for i in range(nblocks)], axis=-1)
    assert np.array_equal(iacc.astype(np.int64), brute)


def test_q4_rowquant_closed_forms():
    # zero row: scale 1, zero point 0... rmin == rmax == 0 -> scale = 1, zp: err = (-128+0)+(127+0) = -1 -> 127 - 0
    x = np.zeros((1, 32), np.float32)
    q, recip, nzp = oracle.q4_rowquant(x, oracle.F32, True)
    assert recip[0] == 1.0 and nzp[0] == -127 and (q == 127).all()
    # a row spanning exactly [-128, 127]: scale 1, zero point 0, q = round-half-away(x)
    x = np.array([[-128.0, 127.0, 0.5, -0.5, 1.5, 2.5, -2.5, 3.49]], np.float32)
    q, recip, nzp = oracle.q4_rowquant(x, oracle.F32, False)
    assert recip[0] == 1.0 and nzp[0] == 0
    assert q[0].tolist() == [-128, 127, 1, -1, 2, 3, -3, 3]  # halves go away from zero, not to even
    # positive-only row [0, 255]: scale 1, zp = -128 exactly
    x = np.array([[0.0, 255.0, 10.0, 100.25]], np.float32)
    q, recip, nzp = oracle.q4_rowquant(x, oracle.F32, True)
    assert nzp[0] == 128 and q[0].tolist() == [-128, 127, -118, -28]
    # zero point lands on a half: rmin=-0.5, rmax=254.5 -> scale 1, dmin=-0.5: err = ((-128-0.5)+127)+254.5 > 0
    # -> zp = -128 + 0.5 = -127.5 -> half-to-even gives -128 (round-half-away would give -128 too);
    # rmin=-1.5 -> zp=-126.5 -> even = -126 (half-away would give -127)
    x = np.array([[-1.5, 253.5]], np.float32)
    q, recip, nzp = oracle.q4_rowquant(x, oracle.F32, True)
    assert recip[0] == 1.0 and nzp[0] == 126


def test_q4_nibble_order_and_block_scales():
    # one row, K=64, bs=32, activations chosen so that q - zp reproduces them exactly:
    # x spans [-128,127] -> scale 1, zp 0.  Weights: distinct per nibble position.
    k, n = 64, 2
    x = np.zeros((1, k), np.float32)
    x[0, 0], x[0, 1] = -128.0, 127.0
    x[0, 2], x[0, 3], x[0, 40] = 3.0, 5.0, 7.0
    w = np.full((n, k // 2), 0x88, np.uint8)  # nibbles 8 -> weight 0
    w[0, 1] = 0x9A  # k=2: low nibble 0xA -> +2 ; k=3: high nibble 9 -> +1
    w[1, 20] = 0x08 | (0xF << 4)  # k=40 low nibble 8 -> 0, k=41 high nibble 15 -> +7 (x[41]=0)
    w[1, 20] = 0x0F  # k=40: low nibble 15 -> +7; k=41: high nibble 0 -> -8 (x[41]=0)
    sc = np.array([[0.5, 100.0], [100.0, 0.25]], np.float32)
    packed = oracle.q4_pack(w, sc, oracle.F32, None)
    out, iacc = oracle.q4_matmul(x, oracle.F32, packed, 32, k, n, want_iacc=True)
    assert iacc[0, 0].tolist() == [3 * 2 + 5 * 1, 0]
    assert iacc[0, 1].tolist() == [0, 7 * 7]
    assert out[0].tolist() == [11 * 0.5, 49 * 0.25]


# ------------------------------------------------------------------ float8
@pytest.mark.parametrize("fa,fb", FLOAT8_PAIRS)
@pytest.mark.parametrize("out_dtype", FLOAT8_OUT)
@pytest.mark.parametrize("rowwise", [False, True])
def test_scaled_mm_vs_torch_cpu(fa, fb, out_dtype, rowwise):
    # the reference's parametrisation (test_quant.py:101-128); the CPU op of torch 2.10 rejects rowwise scales: closed form there
    a, b, sa, sb, bias, scale_result, res_dtype = float8_case(fa, fb, out_dtype, rowwise)
    got, mag = oracle.scaled_mm(bits(a), ODT[fa], bits(b.t()), ODT[fb], sa.numpy(), sb.numpy(), rowwise,
                                None if bias is None else bits(bias), oracle.BF16,
                                None if scale_result is None else 2.0, ODT[res_dtype], want_mag=True)
    got = unbits(got, res_dtype).float().numpy()
    closed = (a.float() * sa).double() @ (b.float() * sb).double()
    if bias is not None:
        closed = closed.float() + bias.float()
    if scale_result is not None:
        closed = closed.float() * 0.5
    closed = closed.float().to(res_dtype).float().numpy()
    if scale_result is not None:
        mag = mag / 2
    tol = ref_tol(closed, mag, ODT[res_dtype])
    assert (np.abs(got - closed) <= tol).all()
    try:
        want = torch._scaled_mm(a, b, sa, sb, bias=bias, out_dtype=out_dtype, scale_result=scale_result)
    except (RuntimeError, ValueError) as e:
        assert rowwise, e  # torch 2.10's CPU kernel: per-tensor scales only
        return
    assert (np.abs(got - want.float().numpy()) <= tol).all()


def test_scaled_mm_exact_cases():
    # powers of two and small integers: every product and sum is exact, so the result is
    # pinned bit for bit; B's layout ([N,K] rows = mat2 columns) and the scale axes are
    # distinguishable (a transposed scale or operand changes the answer).
    t4 = oracle.fp8_table(oracle.E4M3)
    code = {float(v): i for i, v in enumerate(t4) if np.isfinite(v)}
    A = np.array([[1.0, 2.0, 0.0, -3.0], [0.5, 0.0, 4.0, 1.0]], np.float32)  # [M=2,K=4]
    Bt = np.array([[1.0, 1.0, 1.0, 1.0], [2.0, -1.0, 0.5, 0.0], [0.0, 0.0, 0.0, 8.0]], np.float32)  # [N=3,K=4]
    a = np.vectorize(code.get)(A).astype(np.uint8)
    bt = np.vectorize(code.get)(Bt).astype(np.uint8)
    sa, sb = np.array([2.0, 0.5], np.float32), np.array([1.0, 4.0, 0.25], np.float32)
    want = (A * sa[:, None]) @ (Bt * sb[:, None]).T
    got = oracle.scaled_mm(a, oracle.E4M3, bt, oracle.E4M3, sa, sb, True, out_dtype=oracle.F32)
    assert np.array_equal(got, want)
    got = oracle.scaled_mm(a, oracle.E4M3, bt, oracle.E4M3, [0.5], [4.0], False, bias=np.array([1.0, 2.0, 3.0], np.float32),
                           bias_dtype=oracle.F32, out_dtype=oracle.F32)
    assert np.array_equal(got, (A @ Bt.T) * 2.0 + np.array([1.0, 2.0, 3.0], np.float32))


# ------------------------------------------------------------------ frozen fixtures
def test_golden_fixtures():
    """tests/golden/*.npz were written by tests/golden/make_golden.py from torch 2.10's CPU
    ops on the reference's parametrisations; the oracle must reproduce them (bit-exact for
    the int4 op, packed layout and fp8 codes; within the reference's band otherwise)."""
    g = np.load(os.path.join(GOLDEN, "q4.npz"))
    for i in range(len(INT4_SHAPES)):
        m, k, n, bs, bias = (int(v) for v in g[f"c{i}_shape"])  # (large-N cases frozen at 64 features)
        for tag, odt in (("f32", oracle.F32), ("bf16", oracle.BF16)):
            key = f"c{i}_{tag}"
            if key + "_out" not in g:
                continue
            out = oracle.q4_matmul(g[key + "_x"], odt, g[f"c{i}_packed"], bs, k, n)
            assert np.array_equal(out, g[key + "_out"]), key
    g = np.load(os.path.join(GOLDEN, "q8.npz"))
    for key in [k[:-2] for k in g.files if k.endswith("_a")]:
        odt = int(g[key + "_odt"])
        c, c64, mag = oracle.qmm8(g[key + "_a"], odt, g[key + "_b"], g[key + "_s"], want_f64=True)
        want = oracle.to_f32(g[key + "_out"], odt).astype(np.float64)
        assert (np.abs(want - c64) <= 2 * ref_tol(c64, mag, odt)).all(), key
    g = np.load(os.path.join(GOLDEN, "f8.npz"))
    for key in [k[:-2] for k in g.files if k.endswith("_a")]:
        fa, fb, odt = (int(v) for v in g[key + "_fmt"])
        got, mag = oracle.scaled_mm(g[key + "_a"], fa, g[key + "_bt"], fb, g[key + "_sa"], g[key + "_sb"], False,
                                    g[key + "_bias"] if key + "_bias" in g else None, oracle.BF16,
                                    float(g[key + "_sr"]) if key + "_sr" in g else None, odt, want_mag=True)
        want = oracle.to_f32(g[key + "_out"], odt).astype(np.float64)
        if key + "_sr" in g:
            mag = mag / float(g[key + "_sr"])
        assert (np.abs(oracle.to_f32(got, odt) - want) <= ref_tol(want, mag, odt)).all(), key
