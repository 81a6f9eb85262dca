"""GPU parity of the 16-bit matrix product ("gemmcm_bf16" / "gemmcm_f16") through the C ABI, as
the reference tests its cooperative-matrix kernel (tests/python/test_matmul.py:250-284): every
layout of the operands, edges of every size, strided views, batches, alpha / beta and a
broadcast bias, inside eps*|want| + 2^-20 * sum|a||b| of the oracle and of PyTorch's CPU product."""
import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen

pytestmark = pytest.mark.gpu
DTYPES = [torch.bfloat16, torch.float16]


def close(got, want, mag, dtype):
    gf, wf = oracle.to_f32(got, ODT[dtype]).astype(np.float64), oracle.to_f32(want, ODT[dtype]).astype(np.float64)
    tol = torch.finfo(dtype).eps * np.maximum(np.abs(wf), 2.0**-14) + 2.0**-20 * mag
    assert (np.abs(gf - wf) <= tol).all(), float(np.max(np.abs(gf - wf) - tol))


def col_major(x):
    """The same values with the last two dims stored column by column."""
    return np.ascontiguousarray(np.swapaxes(x, -1, -2)).swapaxes(-1, -2)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("m,k,n", [(64, 32, 64), (65, 33, 63), (17, 200, 129), (128, 1, 96), (3, 1000, 5), (256, 64, 256),
                                   (300, 136, 260), (1, 64, 1)])
def test_gemm16_layouts(dtype, m, k, n):
    import _dev
    a = bits(torch.randn(m, k, generator=gen(1)).to(dtype))
    b = bits(torch.randn(k, n, generator=gen(2)).to(dtype))
    want, mag = oracle.gemm16(a, b, ODT[dtype], want_mag=True)
    for x, y in [(a, b), (col_major(a), col_major(b)), (a, col_major(b)), (col_major(a), b)]:
        close(_dev.gemm16(x, y, ODT[dtype]), want, mag, dtype)
    close(_dev.gemm16(a[::2], b, ODT[dtype]), want[::2], mag[::2], dtype)  # a strided view
    cpu = bits((torch.from_numpy(oracle.to_f32(a, ODT[dtype])) @ torch.from_numpy(oracle.to_f32(b, ODT[dtype]))).to(dtype))
    close(_dev.gemm16(a, col_major(b), ODT[dtype]), cpu, mag, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 5, 6, 255])
@pytest.mark.parametrize("m,k,n", [(130, 256, 70), (257, 384, 129), (64, 1088, 300), (300, 128, 520), (300, 320, 520), (1, 128, 8)])
def test_gemm16_tile_variants(dtype, variant, m, k, n):
    """The Linear layout (both operands contiguous along k) through every tile variant and the strided kernel."""
    import _dev
    a = bits((torch.randn(m, k, generator=gen(3)) * 0.5).to(dtype))
    w = bits((torch.randn(n, k, generator=gen(4)) * 0.5).to(dtype))  # B = w.T: rows of k
    want, mag = oracle.gemm16(a, w.T, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a, w.T, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(5)).to(dtype))
    want2, mag2 = oracle.gemm16(a, w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a, w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", [0, 7, 7 | 1 << 8, 7 | 2 << 8, 7 | 4 << 8])
@pytest.mark.parametrize("m,k,n", [(1, 512, 64), (7, 1032, 200), (16, 2048, 1000), (17, 520, 77), (33, 1536, 4100), (64, 2048, 1032), (50, 4096, 520),
                                   (3, 4096, 264), (12, 8192, 100)])  # (few columns against long rows: 8 columns and 16 waves per workgroup)
def test_gemm16_few_rows(dtype, variant, m, k, n):
    """Up to 64 rows in the Linear layout (x @ w.T at decode) run on the kernel whose workgroups own runs of columns
    and whose waves split K: planned (what these shapes get) and asked for with 16, 32 and 64 columns per workgroup;
    every row-tile count, k not a multiple of 128, short last workgroups and ragged vectors; alpha, beta and a bias;
    a strided view of the rows."""
    import _dev
    a = bits((torch.randn(2 * m, k, generator=gen(23)) * 0.5).to(dtype))
    w = bits((torch.randn(n, k, generator=gen(24)) * 0.5).to(dtype))  # B = w.T: rows of k
    want, mag = oracle.gemm16(a[::2], w.T, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a[::2], w.T, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(25)).to(dtype))
    want2, mag2 = oracle.gemm16(a[:m], w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a[:m], w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", [0, 8])
@pytest.mark.parametrize("m,k,n", [(1, 512, 64), (1, 2048, 1001), (2, 1032, 200), (2, 4096, 77), (1, 8192, 30), (3, 520, 130), (4, 2048, 520), (4, 512, 9)])
def test_gemm16_one_to_four_rows_on_vector_units(dtype, variant, m, k, n):
    """One and two rows in the Linear layout (three and four against few columns) run on the vector-unit kernel:
    two-element dot products into float32 sums; planned and asked for (variant 8); every split of K over a workgroup's
    waves, short last workgroups; alpha, beta and a bias; a strided view of the rows."""
    import _dev
    a = bits((torch.randn(2 * m, k, generator=gen(33)) * 0.5).to(dtype))
    w = bits((torch.randn(n, k, generator=gen(34)) * 0.5).to(dtype))  # B = w.T: rows of k
    want, mag = oracle.gemm16(a[::2], w.T, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a[::2], w.T, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(35)).to(dtype))
    want2, mag2 = oracle.gemm16(a[:m], w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a[:m], w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("m,k,n,nt,slices", [(5, 2048, 80, 1, 2), (16, 1032, 64, 2, 2), (33, 4096, 200, 2, 4), (20, 2056, 1000, 1, 3), (64, 8200, 520, 4, 8),
                                              (50, 28672, 100, 2, 16), (64, 2048, 72, 2, 31),
                                              # planned: few columns against long rows (slices of K over workgroups)
                                              (8, 8192, 1024, 0, 0), (32, 4096, 1024, 0, 0), (32, 16384, 520, 0, 0), (64, 8192, 1000, 0, 0)])
def test_gemm16_few_rows_k_slices(dtype, m, k, n, nt, slices):
    """The few-row kernel with K cut into slices over workgroups (their tiles through the workspace, added up by a
    second launch): asked for (columns per workgroup and slice count in the variant word: slices that do not divide the
    chunks of k, a last slice that is short, more slices asked for than half the chunks) and planned (few columns:
    what N = 1024 and 2048 get); alpha, beta and a bias through the second launch's epilogue."""
    import _dev
    variant = 7 | nt << 8 | slices << 12 if nt else 0
    a = bits((torch.randn(m, k, generator=gen(53)) * 0.5).to(dtype))
    w = bits((torch.randn(n, k, generator=gen(54)) * 0.5).to(dtype))
    want, mag = oracle.gemm16(a, w.T, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a, w.T, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(55)).to(dtype))
    want2, mag2 = oracle.gemm16(a, w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a, w.T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", [0, 9, 9 | 2 << 12, 9 | 3 << 12, 9 | 8 << 12])
@pytest.mark.parametrize("m,k,n", [(1, 512, 64), (7, 1088, 200), (16, 2048, 1000), (17, 576, 72), (33, 1536, 4104), (64, 2048, 1032), (50, 4096, 520),
                                   (8, 512, 14344)])  # (one slice, many columns, a short last workgroup)
def test_gemm16_few_rows_weights_in_rows_of_n(dtype, variant, m, k, n):
    """Up to 64 rows against weights stored [k, n] (x @ w) run on the few-row kernel that reads the weights through the
    transposing LDS read: planned and asked for (variant 9), with K in slices over workgroups (slices that do not
    divide the chunks of k); every row-tile count, short last workgroups; alpha, beta and a bias; a strided view of
    the rows."""
    import _dev
    a = bits((torch.randn(2 * m, k, generator=gen(63)) * 0.5).to(dtype))
    w = bits((torch.randn(k, n, generator=gen(64)) * 0.5).to(dtype))
    want, mag = oracle.gemm16(a[::2], w, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a[::2], w, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(65)).to(dtype))
    want2, mag2 = oracle.gemm16(a[:m], w, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a[:m], w, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_few_rows_weights_in_rows_of_n_infinities(dtype):
    """Columns past n and an infinity at the matrix's start (where the loads of what lies outside go): no 0 x inf."""
    import _dev
    m, k, n = 5, 512, 72
    a = (torch.randn(m, k, generator=gen(73)) * 0.5).to(dtype)
    w = (torch.randn(k, n, generator=gen(74)) * 0.5).to(dtype)
    a[:, 0] = 1.0
    w[0, :] = float("inf")
    w[0, 3] = float("-inf")
    for variant in (9, 0, 9 | 2 << 12):
        got = oracle.to_f32(_dev.gemm16(bits(a), bits(w), ODT[dtype], variant=variant), ODT[dtype])
        want = np.full((m, n), np.inf, np.float32)
        want[:, 3] = -np.inf
        assert np.array_equal(got, want), variant


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("batch,m,k,n,layout,variant", [
    (6, 1, 128, 520, "nt", 0), (5, 8, 128, 200, "nt", 0), (9, 16, 256, 72, "nt", 0),          # rows of k too short to share: a wave per 64 columns
    (3, 16, 2048, 264, "nt", 0), (4, 33, 1024, 130, "nt", 0), (2, 64, 4096, 520, "nt", 7 | 2 << 8 | 4 << 12), (3, 5, 8192, 100, "nt", 0),
    (7, 1, 1024, 128, "nn", 0), (3, 8, 4096, 128, "nn", 0), (2, 40, 576, 200, "nn", 0), (3, 16, 2048, 72, "nn", 9 | 3 << 12)])
def test_gemm16_batched_few_rows(dtype, batch, m, k, n, layout, variant):
    """A batch of few-row products (attention at decode: q @ k.T with rows of k of one head's length, p @ v with the
    values in rows of n) runs on the few-row kernels, a workgroup per batch, column group and slice of K: batch strides
    of all three matrices, a bias broadcast over rows and batches, weights shared by the batches (batch stride 0)."""
    import _dev
    a = bits((torch.randn(batch, m, k, generator=gen(83)) * 0.5).to(dtype))
    w = bits((torch.randn(batch, n, k, generator=gen(84)) * 0.5).to(dtype))
    b = w.transpose(0, 2, 1) if layout == "nt" else np.ascontiguousarray(w.transpose(0, 2, 1))
    want, mag = oracle.gemm16(a, b, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(85)).to(dtype))
    want2, mag2 = oracle.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)
    shared = np.broadcast_to(b[:1], b.shape)
    full = bits(torch.randn(batch, m, n, generator=gen(86)).to(dtype))  # (baddbmm: an addend of the result's shape)
    want3, mag3 = oracle.gemm16(a, shared, ODT[dtype], cin=full, alpha=0.5, beta=-1.0, want_mag=True)
    close(_dev.gemm16(a, shared, ODT[dtype], cin=full, alpha=0.5, beta=-1.0, variant=variant), want3, mag3, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("m,k,n,variant", [(128, 1024, 264, 10 | 2 << 8), (200, 2048, 520, 10 | 4 << 8), (70, 4096, 77, 10 | 16 << 8),
                                           (130, 4096, 520, 0), (96, 8192, 264, 0), (512, 2048, 262, 0), (300, 3584, 520, 0)])
def test_gemm16_tile_kernel_k_slices(dtype, m, k, n, variant, layout="nt"):
    """65 rows and more against few tiles (x @ w.T): the 128 x 128 tile kernel with K in slices over workgroups, the
    slices' float32 partial sums in the workspace, added up in slice order by a second launch that runs the epilogue:
    asked for (variant 10) and planned; rows and columns past the last whole tile, n off the vector width; alpha, beta,
    a bias and an addend of the result's shape."""
    import _dev
    a = bits((torch.randn(m, k, generator=gen(103)) * 0.5).to(dtype))
    w = bits((torch.randn(n, k, generator=gen(104)) * 0.5).to(dtype))
    b = w.T if layout == "nt" else np.ascontiguousarray(w.T)  # ("nn": the weights stored [k, n])
    want, mag = oracle.gemm16(a, b, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], variant=variant), want, mag, dtype)
    bias = bits(torch.randn(n, generator=gen(105)).to(dtype))
    want2, mag2 = oracle.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)
    full = bits(torch.randn(m, n, generator=gen(106)).to(dtype))
    want3, mag3 = oracle.gemm16(a, b, ODT[dtype], cin=full, alpha=0.5, beta=-1.0, want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], cin=full, alpha=0.5, beta=-1.0, variant=variant), want3, mag3, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("m,k,n,variant", [(200, 2048, 264, 10 | 4 << 8), (130, 4096, 520, 0), (300, 3584, 72, 0)])
def test_gemm16_tile_kernel_k_slices_weights_in_rows_of_n(dtype, m, k, n, variant):
    """The same against weights stored [k, n] (x @ w): a slice of K begins k / slices rows down the weights."""
    test_gemm16_tile_kernel_k_slices(dtype, m, k, n, variant, layout="nn")


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("batch,m,k,n,layout", [(1, 96, 4104, 520, "nt"), (1, 130, 4096, 264, "nn"), (1, 256, 8200, 72, "nt"), (2, 100, 2048, 128, "nn"), (3, 65, 2048, 200, "nt")])
def test_gemm16_row_blocks_on_few_row_kernels(dtype, batch, m, k, n, layout):
    """65 to 256 rows against few columns (few tiles for the tile kernels, whose workgroups each walk all of K) run as
    passes of the few-row kernels over blocks of 64 rows: a short last block, both weight layouts, batches, an addend
    of the result's shape (its rows offset with the block's) and a broadcast bias."""
    import _dev
    a = bits((torch.randn(batch, m, k, generator=gen(93)) * 0.5).to(dtype))
    w = bits((torch.randn(batch, n, k, generator=gen(94)) * 0.5).to(dtype))
    b = w.transpose(0, 2, 1) if layout == "nt" else np.ascontiguousarray(w.transpose(0, 2, 1))
    want, mag = oracle.gemm16(a, b, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype]), want, mag, dtype)
    full = bits(torch.randn(batch, m, n, generator=gen(95)).to(dtype))
    want2, mag2 = oracle.gemm16(a, b, ODT[dtype], cin=full, alpha=0.5, beta=-1.0, want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], cin=full, alpha=0.5, beta=-1.0), want2, mag2, dtype)
    bias = bits(torch.randn(n, generator=gen(96)).to(dtype))
    want3, mag3 = oracle.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5), want3, mag3, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_few_rows_infinite_weights(dtype):
    """Rows of k that end inside a chunk of the few-row kernel, weight rows that start with an infinity: the outputs
    are the infinities float arithmetic gives (what stands in for the values past k must not meet them as 0 x inf)."""
    import _dev
    m, k, n = 5, 520, 80
    a = (torch.randn(m, k, generator=gen(43)) * 0.5).to(dtype)
    w = (torch.randn(n, k, generator=gen(44)) * 0.5).to(dtype)
    a[:, 0] = 1.0
    w[:, 0] = float("inf")
    w[3, 0] = float("-inf")
    for variant in (7, 7 | 1 << 8, 0):
        got = oracle.to_f32(_dev.gemm16(bits(a), bits(w).T, ODT[dtype], variant=variant), ODT[dtype])
        want = np.full((m, n), np.inf, np.float32)
        want[:, 3] = -np.inf
        assert np.array_equal(got, want), variant


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_stream_kernel(dtype):
    """The stream kernel (variant 6; what large products in the Linear layout get): more tiles than workgroups, so
    streams that run through two tiles; batches; a broadcast bias; rows and columns past the last whole tile.  Every
    output against the oracle, and bit for bit the tile kernel's (same products, same order)."""
    import _dev
    for batch, m, k, n in [(1, 4352, 192, 4360), (3, 515, 256, 1032)]:
        a = bits((torch.randn(batch, m, k, generator=gen(13)) * 0.5).to(dtype))
        w = bits((torch.randn(batch, n, k, generator=gen(14)) * 0.5).to(dtype))
        bias = bits(torch.randn(n, generator=gen(15)).to(dtype))
        got = {v: _dev.gemm16(a, w.transpose(0, 2, 1), ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=v) for v in (6, 3)}
        assert np.array_equal(got[6], got[3])
        if m * n <= 1 << 20:
            want, mag = oracle.gemm16(a, w.transpose(0, 2, 1), ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
            close(got[6], want, mag, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_stream_kernel_nan_and_inf(dtype):
    """NaN and infinities through the stream kernel's epilogue (its bfloat16 conversion looks at its values one by one
    only where a wave has seen a NaN): a NaN operand of either sign, infinities of both signs in one column (inf - inf)
    and against a zero row (0 x inf).  Bit for bit the tile kernel's outputs; NaN and infinities where the oracle has
    them; a bfloat16 NaN is 0x7fc0 as c10 writes it."""
    import _dev
    m, k, n = 512, 128, 520
    a = bits((torch.randn(m, k, generator=gen(16)) * 0.5).to(dtype)).copy()
    w = bits((torch.randn(n, k, generator=gen(17)) * 0.5).to(dtype)).copy()
    nan, inf = (0x7FC1, 0x7F80) if dtype == torch.bfloat16 else (0x7E01, 0x7C00)
    a[3, 17], a[300, 5] = nan, nan | 0x8000
    a[7, :] = 0
    w[9, 40], w[9, 41] = inf, inf | 0x8000
    w[260, 100] = inf
    got = {v: _dev.gemm16(a, w.T, ODT[dtype], variant=v) for v in (6, 3)}
    assert np.array_equal(got[6], got[3])
    want = oracle.to_f32(oracle.gemm16(a, w.T, ODT[dtype]), ODT[dtype])
    have = oracle.to_f32(got[6], ODT[dtype])
    assert np.array_equal(np.isnan(have), np.isnan(want)) and np.isnan(want[3]).all() and np.isnan(want[7, 9]) and np.isnan(want[7, 260])
    assert np.array_equal(np.isinf(have), np.isinf(want)) and np.array_equal(np.sign(have[np.isinf(have)]), np.sign(want[np.isinf(want)]))
    assert np.isinf(want[:, 260]).sum() > m // 2
    if dtype == torch.bfloat16:
        assert (got[6][np.isnan(have)] == 0x7FC0).all()


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("variant", [0, 3, 4, 5])
@pytest.mark.parametrize("m,k,n", [(128, 64, 136), (264, 192, 520), (1032, 128, 1024), (8, 64, 8)])
def test_gemm16_k_major_operands(dtype, variant, m, k, n):
    """Operands contiguous along m / n (x @ W with W row-major, x.t() @ y): the matrix-core tiles read them
    through the transposing LDS load; every combination with the k-contiguous form, batched, with a bias."""
    import _dev
    a = bits((torch.randn(2, m, k, generator=gen(11)) * 0.5).to(dtype))
    b = bits((torch.randn(2, k, n, generator=gen(12)) * 0.5).to(dtype))
    bias = bits(torch.randn(n, generator=gen(13)).to(dtype))
    want, mag = oracle.gemm16(a, b, ODT[dtype], want_mag=True)
    want2, mag2 = oracle.gemm16(a, b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    for x, y in [(a, b), (col_major(a), b), (a, col_major(b)), (col_major(a), col_major(b))]:
        close(_dev.gemm16(x, y, ODT[dtype], variant=variant), want, mag, dtype)
    close(_dev.gemm16(col_major(a), b, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, variant=variant), want2, mag2, dtype)
    # one matrix of a larger one: rows further apart than they are long
    big_a, big_b = np.zeros((2, m, k + 64), np.uint16), np.zeros((2, k, n + 8), np.uint16)
    big_a[:, :, :k], big_b[:, :, :n] = a, b
    close(_dev.gemm16(big_a[:, :, :k], big_b[:, :, :n], ODT[dtype], variant=variant), want, mag, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_gemm16_batches_and_bias(dtype):
    import _dev
    a = bits(torch.randn(3, 40, 72, generator=gen(6)).to(dtype))
    w = bits(torch.randn(3, 50, 72, generator=gen(7)).to(dtype))
    bias = bits(torch.randn(50, generator=gen(8)).to(dtype))
    want, mag = oracle.gemm16(a, w.transpose(0, 2, 1), ODT[dtype], want_mag=True)
    close(_dev.gemm16(a, w.transpose(0, 2, 1), ODT[dtype]), want, mag, dtype)
    want, mag = oracle.gemm16(a[0], w[0].T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5, want_mag=True)
    close(_dev.gemm16(a[0], w[0].T, ODT[dtype], cin=bias, alpha=2.0, beta=0.5), want, mag, dtype)
    # beta == 0 ignores Cin entirely, NaN included (gemmcm.slang:309)
    nan_bias = np.full(50, 0x7FC0 if dtype == torch.bfloat16 else 0x7E00, np.uint16)
    want0, mag0 = oracle.gemm16(a[0], w[0].T, ODT[dtype], want_mag=True)
    close(_dev.gemm16(a[0], w[0].T, ODT[dtype], cin=nan_bias, beta=0.0), want0, mag0, dtype)


def test_gemm16_config_8192_cubed():
    """The reference's adjacent benchmark shape (bf16 8192^3): sampled rows / columns against the float64 closed form."""
    import _dev
    m = n = k = 8192
    a = torch.randn(m, k, generator=gen(9)).bfloat16()
    w = torch.randn(n, k, generator=gen(10)).bfloat16()
    got = _dev.gemm16(bits(a), bits(w).T, oracle.BF16)
    rows, cols = np.array([0, 1, 255, 256, 4095, 8191]), np.array([0, 3, 127, 128, 5000, 8191])
    exact = a[rows].double().numpy() @ w[cols].double().numpy().T
    mag = np.abs(a[rows].double().numpy()) @ np.abs(w[cols].double().numpy()).T
    sub = oracle.bf16_to_f32(got[np.ix_(rows, cols)]).astype(np.float64)
    assert (np.abs(sub - exact) <= 2.0**-7 * np.maximum(np.abs(exact), 2.0**-14) + 2.0**-20 * mag).all()


def test_gemm16_errors():
    from torch_vulkan_amd import abi
    buf = abi.Buffer(4096)
    p = abi.GemmParams(a=buf.address, b=buf.address, c=buf.address, m=4, n=4, k=8, a_sm=8, a_sk=1, b_sk=1, b_sn=8, c_sm=4,
                       c_sn=1)
    with pytest.raises(abi.VktError, match="null tensor address"):
        abi.dispatch("gemmcm_bf16", [1], p)
    with pytest.raises(abi.VktError, match="unknown kernel"):
        abi.dispatch("gemmcm_f32", [0], p)
    with pytest.raises(abi.VktError, match="unknown variant"):
        abi.dispatch("gemmcm_bf16", [0, 0, 0, 11], p)
