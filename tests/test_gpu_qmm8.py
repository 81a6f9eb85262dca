"""GPU parity of _weight_int8pack_mm (kernels "qmm8_*") through the C ABI against the
oracle: the reference's own shapes and seeds (tests/python/test_quant.py:20-40), the frozen
fixtures, the BASELINE configurations, and size-independent properties at full size."""
import os

import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen, ref_tol, unbits
from _cases import INT8_SHAPES, int8_case

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def check_q8(got_bits, a, b, s, dtype, rows=slice(None)):
    odt = ODT[dtype]
    c, c64, mag = oracle.qmm8(bits(a), odt, b.numpy(), bits(s), want_f64=True)
    got = unbits(got_bits, dtype).float().numpy().astype(np.float64)
    # the reference's bound, eps*|want| + 2^-20*mag (test_quant.py:36-37), around the float64 sum
    tol = ref_tol(c64, mag, odt)[rows]
    err = np.abs(got - c64[rows])
    assert (err <= tol).all(), f"max excess {np.max(err - tol)}"
    return got, c64[rows]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", INT8_SHAPES + [(1, 4096, 4096), (8, 4096, 640), (16, 2048, 130), (3, 1024, 7),
                                               (17, 256, 33), (2, 16, 1), (1, 48, 5)])
def test_qmm8_reference_shapes(dtype, m, k, n):
    import _dev
    a, b, s = int8_case(dtype, m, k, n)
    got = _dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s))
    assert got.shape == (m, n)
    check_q8(got, a, b, s, dtype)
    # a row slice of A (A's rows strided), as test_quant.py:35
    sliced = _dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), row_step=2)
    check_q8(sliced, a, b, s, dtype, rows=slice(None, None, 2))


@pytest.mark.parametrize("variant", [2 | 1 << 8, 2 | 2 << 8, 2 | 4 << 8, 4 | 1 << 8, 4 | 2 << 8, 4 | 4 << 8, 1 << 16])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_qmm8_every_variant(variant, dtype):
    """Each (COLS, KSPLIT) instantiation and the generic kernel give results inside the band."""
    import _dev
    for m, k, n in [(1, 4096, 130), (4, 2064, 67)]:
        a, b, s = int8_case(dtype, m, k, n)
        check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=variant), a, b, s, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("k", [16, 1008, 1024, 2048, 2064, 3072, 4096, 4112, 6144, 8192, 8208, 12288, 14336, 16384])
def test_qmm8_one_row_streaming_kernel(dtype, k):
    """One activation row through the persistent streaming kernel: every split of a row over a workgroup's waves
    (1 to 4 chunks of 1 KiB per wave, 1, 2 or 4 waves per row), rows that end inside a chunk, fewer rows than a
    workgroup takes per iteration, more iterations than one, and the rows-per-iteration forms the planner picks from."""
    import _dev
    for n in (1, 7, 300):
        a, b, s = int8_case(dtype, 1, k, n)
        for variant in (2 << 8, 1 << 8 | 1 << 12, 3 << 8 | 2 << 12):
            if (variant >> 12) == 2 and k <= 1024 or (variant >> 12) == 1 and k <= 2048:
                continue  # (forms that are not built: short rows take 8 or 4 rows per iteration)
            check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=variant), a, b, s, dtype)
    # enough rows for several iterations per wave on a full grid
    a, b, s = int8_case(dtype, 1, k, 9000 if k <= 4096 else 3000)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=1 << 8), a, b, s, dtype)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("variant", [0, 1 | 4 << 8, 2 | 8 << 8, 4 | 16 << 8, 4 | 8 << 8 | 3 << 24, 1 | 4 << 8 | 16 << 24,
                                     1 << 17, 1 << 18, 1 | 4 << 8 | 1 << 18, 2 | 8 << 8 | 1 << 18, 4 | 4 << 8 | 1 << 18,
                                     4 | 8 << 8 | 3 << 24 | 1 << 18, 2 | 4 << 8 | 16 << 24 | 1 << 18])
@pytest.mark.parametrize("m,k,n", [(5, 1024, 40), (16, 4096, 67), (33, 2048, 130), (64, 4160, 96), (70, 512, 36)])
def test_qmm8_matrix_core_variants(dtype, variant, m, k, n):
    """4 < M with 16-bit activations runs on the matrix cores: every (columns, k-split)
    instantiation, K sliced over several workgroups (bits 24+; the slices meet in the
    library's workspace), the GEMV kernels forced on the same problem (bit 17), and the kernel that stages the
    weights through LDS (bit 18; up to 32 rows, otherwise the plain one runs)."""
    import _dev
    a, b, s = int8_case(dtype, m, k, n)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=variant), a, b, s, dtype)
    sliced_variant = variant if (m + 1) // 2 > 4 else 0  # (4 rows or fewer: the GEMV kernels plan themselves)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=sliced_variant, row_step=2), a, b, s, dtype,
             rows=slice(None, None, 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(8, 2048, 8195), (5, 2048, 9216), (8, 2048, 13824), (3, 2048, 8200), (20, 2048, 8196),
                                   (32, 2048, 14336), (8, 2048, 2049), (8, 2304, 2100), (8, 2048, 14336)])
def test_qmm8_columns_dealt_out_evenly(dtype, m, k, n):
    """3 to 32 rows on the kernel that stages weights through LDS, planned by the library: the launch deals the columns
    out over a whole number of workgroups per compute unit, so a workgroup owns 12, 20, 28, 36 or 56 columns and not
    whole tiles of 16; n off the vector width (scalar stores), a last workgroup with fewer columns, rows of A further
    apart than k."""
    import _dev
    a, b, s = int8_case(dtype, m, k, n, seeds={"a": 4, "b": 5, "scales": 6})
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s)), a, b, s, dtype)
    if (m + 1) // 2 >= 3:
        check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), row_step=2), a, b, s, dtype, rows=slice(None, None, 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(8, 8192, 1024), (7, 28672, 64), (16, 4096, 1000), (5, 16384, 516), (20, 4112, 264), (32, 16384, 520), (32, 8192, 2048)])
def test_qmm8_few_columns_k_slices(dtype, m, k, n):
    """Few columns against long rows, planned by the library: the staged kernel with K in slices over workgroups, the
    slices' tiles added up in slice order by a second launch (a wave per tile); slices that do not divide the chunks
    of k, column counts that leave a short last workgroup and ragged vectors, rows of A further apart than k."""
    import _dev
    a, b, s = int8_case(dtype, m, k, n, seeds={"a": 14, "b": 15, "scales": 16})
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s)), a, b, s, dtype)
    if (m + 1) // 2 >= 5:
        check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), row_step=2), a, b, s, dtype, rows=slice(None, None, 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(8, 512, 24600), (5, 1024, 33001), (8, 4096, 14336), (3, 3088, 12300), (7, 2064, 8192),
                                   (8, 4080, 4096), (4, 528, 70), (6, 512, 16), (8, 3600, 1000), (8, 2048, 34000)])
def test_qmm8_rows_kernel(dtype, m, k, n):
    """3 to 8 short rows against many columns run on the kernel whose waves own column groups (asked for here
    whatever the size: variant bits 8-15; the last shape is one the planner sends there itself): 1, 2, 4 and 8 waves
    per group, one and several rounds per workgroup, a partial last group, k off the chunk size, n off the group and
    vector sizes, rows of A further apart than k."""
    import _dev
    # (seeds of its own: among the first table's scales for n > 27482 is the smallest float16 subnormal, and a float16
    # output that small is further from the float64 sum than the bound allows however it is rounded)
    a, b, s = int8_case(dtype, m, k, n, seeds={"a": 4, "b": 5, "scales": 6})
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=1 << 8), a, b, s, dtype)
    if (m + 1) // 2 >= 3:  # (fewer rows are other kernels')
        check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=1 << 8, row_step=2), a, b, s, dtype, rows=slice(None, None, 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(192, 512, 200), (2100, 64, 2060), (300, 1088, 7000), (1024, 256, 4100), (4096, 72, 2056)])
def test_qmm8_many_rows(dtype, m, k, n):
    """From 192 rows on (prefill) the weights are widened once into the library's scratch region and the product runs
    on the tile kernel; the row-block kernels (variant bit 20) give the same results to the test's bound."""
    import _dev
    a, b, s = int8_case(dtype, m, k, n)
    got = _dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s))
    check_q8(got, a, b, s, dtype)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=1 << 20), a, b, s, dtype)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), row_step=2), a, b, s, dtype, rows=slice(None, None, 2))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("variant", [0, 1 << 21, 1 << 21 | 1 << 24, 1 << 21 | 3 << 24, 1 << 22])
@pytest.mark.parametrize("m,k,n", [(16, 256, 128), (64, 1024, 200), (33, 2048, 130), (70, 512, 257), (130, 768, 96), (5, 512, 64)])
def test_qmm8_tile_kernel(dtype, variant, m, k, n):
    """More than 32 rows with k a multiple of 256 run on the tile kernel (64 x 128 tiles, K sliced over workgroups,
    slices met in the workspace): planned, forced with 1 and 3 slices (bit 21; also with fewer rows), and switched off (bit 22)."""
    import _dev
    a, b, s = int8_case(dtype, m, k, n)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=variant), a, b, s, dtype)
    if m > 8:
        check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), variant=variant, row_step=2), a, b, s, dtype, rows=slice(None, None, 2))


@pytest.mark.parametrize("variant", [0, 1 << 21 | 1 << 24, 1 << 21 | 3 << 24, 1 << 22])
@pytest.mark.parametrize("m,k,n", [(17, 256, 128), (32, 1024, 200), (64, 2048, 130), (70, 512, 257), (130, 768, 96), (200, 4096, 520)])
def test_qmm8_float32_rows_on_tile_kernel(variant, m, k, n):
    """More than 16 rows of float32 activations with k a multiple of 128 run on the tile kernel, the activations split
    into three bfloat16 parts that add up to them exactly (one pass over the weights per 64 rows): planned, forced with
    1 and 3 slices, and switched off (bit 22: the one-row kernels, a pass per 16 rows); strided rows as well."""
    import _dev
    a, b, s = int8_case(torch.float32, m, k, n)
    check_q8(_dev.qmm8(bits(a), ODT[torch.float32], b.numpy(), bits(s), variant=variant), a, b, s, torch.float32)
    check_q8(_dev.qmm8(bits(a), ODT[torch.float32], b.numpy(), bits(s), variant=variant, row_step=2), a, b, s, torch.float32,
             rows=slice(None, None, 2))


def test_qmm8_float32_rows_special_values():
    """Infinities, NaNs (also one whose payload sits in the low mantissa bits), zeros, subnormal and huge finite values
    among float32 activations on the tile kernel: each output is what float64 arithmetic on the same operands gives
    (an infinity or NaN where that is one, else within the bound)."""
    import _dev
    m, k, n = 40, 256, 64
    a, b, s = int8_case(torch.float32, m, k, n)
    a = a.clone()
    a[1, 5] = float("inf")
    a[2, 7] = float("-inf")
    a[3, 9] = float("nan")
    a[4, 11] = torch.tensor(0x7f800001, dtype=torch.int32).view(torch.float32)
    a[5, :] = 0.0
    a[6, 3] = 1e-41
    a[7, 2] = 3.0e38
    b = b.clone()
    b[:, 2] = 1  # (keeps row 7 finite)
    got = unbits(_dev.qmm8(bits(a), ODT[torch.float32], b.numpy(), bits(s)), torch.float32).numpy().astype(np.float64)
    want = (a.double() @ b.double().t() * s.double()).numpy()
    nan, inf = np.isnan(want), np.isinf(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(got[inf], want[inf])
    fin = ~(nan | inf)
    mag = (a.double().abs() @ b.double().abs().t() * s.double().abs()).numpy()
    assert (np.abs(got - want)[fin] <= (2.0 ** -23 * np.abs(want) + 2.0 ** -20 * mag)[fin]).all()


@pytest.mark.parametrize("variant", [0, 1 << 18, 1 << 19])
@pytest.mark.parametrize("m,k,n", [(2, 1024, 64), (3, 2064, 200), (5, 4096, 1000), (8, 1040, 77), (13, 3072, 4100), (16, 4096, 4128), (9, 8192, 520),
                                   (8, 8192, 1024), (5, 16400, 264), (16, 28672, 72)])  # (few columns against long rows: K in slices over workgroups)
def test_qmm8_float32_few_rows_on_matrix_cores(variant, m, k, n):
    """2 to 16 rows of float32 activations: split into three bfloat16 planes by a launch of its own and multiplied by
    the staged matrix-core kernel (forced with bit 18, planned, and switched off with bit 19); rows of k not a multiple
    of 256, every column count per workgroup, strided rows as well."""
    import _dev
    a, b, s = int8_case(torch.float32, m, k, n)
    check_q8(_dev.qmm8(bits(a), ODT[torch.float32], b.numpy(), bits(s), variant=variant), a, b, s, torch.float32)
    check_q8(_dev.qmm8(bits(a), ODT[torch.float32], b.numpy(), bits(s), variant=variant, row_step=2), a, b, s, torch.float32,
             rows=slice(None, None, 2))


def test_qmm8_float32_few_rows_special_values():
    """The same special values through the three-plane split of the few-row path: infinities and NaNs come out where
    float64 arithmetic has them, the rest within the bound."""
    import _dev
    m, k, n = 8, 1024, 64
    a, b, s = int8_case(torch.float32, m, k, n)
    a = a.clone()
    a[1, 5] = float("inf")
    a[2, 7] = float("-inf")
    a[3, 9] = float("nan")
    a[4, 11] = torch.tensor(0x7f800001, dtype=torch.int32).view(torch.float32)
    a[5, :] = 0.0
    a[6, 3] = 1e-41
    a[7, 2] = 3.0e38
    b = b.clone()
    b[:, 2] = 1  # (keeps row 7 finite)
    got = unbits(_dev.qmm8(bits(a), ODT[torch.float32], b.numpy(), bits(s), variant=1 << 18), torch.float32).numpy().astype(np.float64)
    want = (a.double() @ b.double().t() * s.double()).numpy()
    nan, inf = np.isnan(want), np.isinf(want)
    assert np.array_equal(np.isnan(got), nan) and np.array_equal(got[inf], want[inf])
    fin = ~(nan | inf)
    mag = (a.double().abs() @ b.double().abs().t() * s.double().abs()).numpy()
    assert (np.abs(got - want)[fin] <= (2.0 ** -23 * np.abs(want) + 2.0 ** -20 * mag)[fin]).all()


def test_qmm8_config1_vs_torch_cpu():
    """BASELINE config 1: fp32, M=1, K=N=4096, within rtol/atol 1e-4 of PyTorch's CPU op."""
    import _dev
    x = torch.randn(1, 4096, generator=gen(1010))
    w = torch.randint(-128, 128, (4096, 4096), dtype=torch.int8, generator=gen(1011))
    s = torch.empty(4096).uniform_(0.005, 0.02, generator=gen(1012))
    got = torch.from_numpy(_dev.qmm8(x.numpy(), oracle.F32, w.numpy(), s.numpy()))
    want = torch._weight_int8pack_mm(x, w, s)
    truth = (x.double() @ (w.float() * s[:, None]).double().t()).float()
    # the CPU op's own float32 summation noise can exceed 1e-4 near zero outputs; the float64
    # closed form is the tighter judge, the CPU op is checked at the stated tolerance where
    # it agrees with the closed form itself
    assert torch.allclose(got, truth, rtol=1e-4, atol=1e-4)
    ok = torch.isclose(want, truth, rtol=1e-4, atol=1e-4)
    assert torch.allclose(got[ok], want[ok], rtol=1e-4, atol=2e-4)
    check_q8(got.numpy(), x, w, s, torch.float32)


@pytest.mark.parametrize("m", [1, 8, 64])
@pytest.mark.parametrize("k,n", [(4096, 14336), (14336, 4096)])
def test_qmm8_config2_llama_mlp(m, k, n):
    """BASELINE config 2: bf16, Llama-3-8B MLP shapes, rtol/atol 1e-2 vs PyTorch's CPU op."""
    import _dev
    x = torch.randn(m, k, generator=gen(1020)).bfloat16()
    w = torch.randint(-128, 128, (n, k), dtype=torch.int8, generator=gen(1021))
    s = torch.empty(n).uniform_(0.005, 0.02, generator=gen(1022)).bfloat16()
    got = unbits(_dev.qmm8(bits(x), oracle.BF16, w.numpy(), bits(s)), torch.bfloat16)
    want = torch._weight_int8pack_mm(x, w, s)
    assert torch.allclose(got.float(), want.float(), rtol=1e-2, atol=1e-2)
    # linearity in the scales: doubling them (exact in bf16) doubles every output bit for bit
    got2 = unbits(_dev.qmm8(bits(x), oracle.BF16, w.numpy(), bits(s * 2)), torch.bfloat16)
    assert torch.equal(got2.float(), got.float() * 2)
    # a row of zeros gives zeros; a one-hot row picks a column of w*s exactly
    x0 = torch.zeros(2, k).bfloat16()
    x0[1, 5] = 1.0
    r = unbits(_dev.qmm8(bits(x0), oracle.BF16, w.numpy(), bits(s)), torch.bfloat16).float()
    assert (r[0] == 0).all()
    assert torch.equal(r[1], (w[:, 5].float() * s.float()).bfloat16().float())


def test_qmm8_golden_fixtures():
    import _dev
    g = np.load(os.path.join(GOLDEN, "q8.npz"))
    for key in [k[:-2] for k in g.files if k.endswith("_a")]:
        odt = int(g[key + "_odt"])
        got = _dev.qmm8(g[key + "_a"], odt, g[key + "_b"], g[key + "_s"])
        c, c64, mag = oracle.qmm8(g[key + "_a"], odt, g[key + "_b"], g[key + "_s"], want_f64=True)
        tol = ref_tol(c64, mag, odt)
        assert (np.abs(oracle.to_f32(got, odt) - c64) <= tol).all(), key
        assert (np.abs(oracle.to_f32(got, odt).astype(np.float64) - oracle.to_f32(g[key + "_out"], odt)) <= 2 * tol).all()


@pytest.mark.parametrize("m", [1, 5, 40])
def test_qmm8_vocabulary_sized_weights(m):
    """A 1 GiB weight (N = 128256, K = 8192: byte offsets beyond 2^30) against the oracle on the last rows of the
    weight, and against the same product of a slice of the weight on the first."""
    import _dev
    n, k = 128256, 8192
    rng = np.random.default_rng(5)
    b = rng.integers(-128, 128, (n, k), dtype=np.int8)
    a = torch.randn(m, k, generator=gen(6)).bfloat16()
    s = (torch.rand(n, generator=gen(7)) / 50).bfloat16()
    got = _dev.qmm8(bits(a), oracle.BF16, b, bits(s))
    assert got.shape == (m, n)
    for lo, hi in ((0, 300), (n - 300, n)):
        bs_, ss_ = torch.from_numpy(b[lo:hi].copy()), s[lo:hi]
        check_q8(np.ascontiguousarray(got[:, lo:hi]), a, bs_, ss_, torch.bfloat16)


def test_qmm8_empty_and_errors():
    import _dev
    from torch_vulkan_amd import abi
    a = np.zeros((0, 64), np.float32)
    assert _dev.qmm8(a, oracle.F32, np.zeros((5, 64), np.int8), np.ones(5, np.float32)).shape == (0, 5)
    buf = abi.Buffer(1024)
    p = abi.Q8Params(a=buf.address, b=buf.address, scales=buf.address, c=buf.address, m=1, n=4, k=16, a_sm=16, a_sk=2)
    with pytest.raises(abi.VktError, match="unit stride"):
        abi.dispatch("qmm8_f32", [1], p)
    with pytest.raises(abi.VktError, match="unknown kernel"):
        abi.dispatch("qmm8_f64", [1], p)
    with pytest.raises(abi.VktError, match="56 bytes"):
        abi.dispatch("qmm8_f32", [1], abi.Q4Params())
    p.a_sk = 1
    with pytest.raises(abi.VktError, match="empty grid"):
        abi.dispatch("qmm8_f32", [1], p, (0, 1, 1))
    with pytest.raises(abi.VktError, match="does not match"):
        abi.dispatch("qmm8_f32", [3], p)
    # weights of 4 GiB and more are refused before anything is launched (32-bit indexing in the kernels)
    p.n, p.k, p.a_sm = 70000, 65536, 65536
    with pytest.raises(abi.VktError, match="too large"):
        abi.dispatch("qmm8_f32", [1], p)
    p.n, p.k, p.a_sm = 4, 16, 16
    p.b = 0
    with pytest.raises(abi.VktError, match="null tensor address"):
        abi.dispatch("qmm8_f32", [1], p)
