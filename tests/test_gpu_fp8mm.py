"""GPU parity of _scaled_mm (kernel "fp8mm") through the C ABI against the oracle and
PyTorch's CPU op: the reference's parametrisation (tests/python/test_quant.py:101-128: every
mix of e4m3fn / e5m2 operands, five output dtypes, tensor-wise and row-wise scales, bias,
scale_result), the frozen fixtures, tile-edge shapes, and the BASELINE shapes through
properties that do not need a full-size CPU product."""
import os

import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen, ref_tol, unbits

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FLOAT8 = [torch.float8_e4m3fn, torch.float8_e5m2]


# The fp8 matrix core adds the 128 products of one instruction in a fixed-point window
# ~14 bits below the largest product (a hardware property, measured: ~2^-15.3 of sum|a||b| on
# random data); bfloat16 / float8 outputs take that path, float32 / float16 outputs (and
# variants 6, 7) run the bfloat16 matrix core on exactly widened operands, inside the
# reference's own bound.
HW_WINDOW = 2.0**-13


def on_matrix_cores(odt, variant, k):
    variant &= 0xff  # (the bits above: columns per workgroup and slices of the few-row kernel)
    if variant in (6, 7, 255) or k % 16:
        return False
    if variant == 13:  # the vector-unit kernel for up to four rows: float32 sums whatever the output type
        return False
    return variant in (1, 2, 3, 4, 5, 8, 11, 12) or odt in (oracle.BF16, oracle.E4M3, oracle.E5M2)


def run_case(m, k, n, fa, fb, out_dtype, rowwise, bias_dtype=None, scale_result=None, variant=0, seed=1, scale=1.0):
    import _dev
    a = (torch.randn(m, k, generator=gen(seed)) * scale).to(fa)
    bt = (torch.randn(n, k, generator=gen(seed + 1)) * scale).to(fb)
    sa = torch.rand(m, 1, generator=gen(seed + 2)) + 0.5 if rowwise else torch.tensor(1.25)
    sb = torch.rand(1, n, generator=gen(seed + 3)) + 0.5 if rowwise else torch.tensor(0.75)
    bias = None if bias_dtype is None else torch.randn(n, generator=gen(seed + 4)).to(bias_dtype)
    res = out_dtype or fa
    kw = dict(bias=None if bias is None else bits(bias), bias_dtype=ODT[bias_dtype] if bias is not None else 0,
              scale_result=scale_result, out_dtype=ODT[res])
    want, mag = oracle.scaled_mm(bits(a), ODT[fa], bits(bt), ODT[fb], sa.numpy(), sb.numpy(), rowwise, want_mag=True,
                                 **kw)
    got = _dev.scaled_mm(bits(a), ODT[fa], bits(bt), ODT[fb], sa.numpy(), sb.numpy(), rowwise, variant=variant, **kw)
    want_f, got_f = oracle.to_f32(want, ODT[res]).astype(np.float64), oracle.to_f32(got, ODT[res]).astype(np.float64)
    if scale_result is not None:
        mag = mag / scale_result
    tol = ref_tol(want_f, mag, ODT[res])  # eps*|want| + 2^-20*mag, test_quant.py:124-126
    if on_matrix_cores(ODT[res], variant, k):
        tol = tol + HW_WINDOW * mag
    finite = np.isfinite(want_f)
    assert np.array_equal(np.isfinite(got_f), finite)
    assert (np.abs(got_f - want_f)[finite] <= tol[finite]).all(), float(np.max((np.abs(got_f - want_f) - tol)[finite]))
    return a, bt, sa, sb, bias, got_f


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[0], FLOAT8[1]),
                                   (FLOAT8[1], FLOAT8[1])])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32, torch.float16, torch.float8_e4m3fn, None])
@pytest.mark.parametrize("rowwise", [False, True])
def test_scaled_mm_reference_cases(fa, fb, out_dtype, rowwise):
    bias_dtype = torch.bfloat16 if out_dtype == torch.bfloat16 else None
    sr = 2.0 if out_dtype == torch.float8_e4m3fn else None
    a, bt, sa, sb, bias, got = run_case(16, 32, 48, fa, fb, out_dtype, rowwise, bias_dtype, sr)
    if not rowwise:  # torch 2.10's CPU kernel takes per-tensor scales only
        want = torch._scaled_mm(a, bt.t(), sa, sb, bias=bias, out_dtype=out_dtype,
                                scale_result=None if sr is None else torch.tensor(sr)).float().numpy()
        res = ODT[out_dtype or fa]
        mag = ((a.float() * sa).abs() @ (bt.float() * sb).abs().t()).numpy() / (sr or 1.0)
        tol = ref_tol(want, mag, res) + (HW_WINDOW * mag if on_matrix_cores(res, 0, 32) else 0)
        assert (np.abs(got - want) <= tol).all()
        if res == oracle.BF16:  # the stated bar for bfloat16 outputs
            assert np.allclose(got, want, rtol=1e-2, atol=1e-2)
        if res == oracle.F32:
            assert np.allclose(got, want, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("m,k,n", [(1, 16, 1), (130, 256, 70), (257, 384, 129), (64, 1040, 300), (300, 128, 520),
                                   (5, 100, 7), (33, 48, 17)])
@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6, 7, 8, 11, 255])
@pytest.mark.parametrize("rowwise", [False, True])
def test_scaled_mm_tile_edges(m, k, n, variant, rowwise):
    """Shapes that are not multiples of any tile, K tails (K % 128 != 0, K % 16 != 0 -> the
    unaligned kernel), every tile variant and the one-thread-per-output kernel (255)."""
    run_case(m, k, n, FLOAT8[0], FLOAT8[0], torch.bfloat16, rowwise, torch.float32, variant=variant, seed=20)
    run_case(m, k, n, FLOAT8[1], FLOAT8[0], torch.float32, rowwise, variant=variant, seed=30)


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[0], FLOAT8[1]), (FLOAT8[1], FLOAT8[1])])
@pytest.mark.parametrize("m,k,n,out_dtype,rowwise", [
    (1, 1024, 64, torch.bfloat16, False), (7, 2064, 200, torch.bfloat16, True), (16, 4096, 1000, torch.float8_e4m3fn, True),
    (17, 1040, 77, torch.bfloat16, True), (32, 3072, 4100, torch.bfloat16, False), (33, 1024, 130, torch.float8_e5m2, False),
    (64, 4096, 4128, torch.bfloat16, True), (50, 8192, 520, torch.bfloat16, True),
    # float32 and float16 outputs: the same kernel on operands widened exactly to bfloat16 (no window in the bound)
    (5, 2064, 300, torch.float32, True), (40, 1024, 64, torch.float16, False), (16, 4096, 4100, torch.float32, False),
    # few columns against long rows: 8 columns and 16 waves per workgroup
    (4, 8192, 264, torch.bfloat16, True), (9, 16384, 100, torch.float32, False)])
def test_scaled_mm_few_rows(fa, fb, m, k, n, out_dtype, rowwise):
    """Up to 64 rows with bfloat16 or float8 outputs run on the kernel whose workgroups own runs of columns and whose
    waves split K (planned, which is what these shapes get, and asked for as variant 12): every row-tile count, rows of
    k not a multiple of 256, column counts that leave short workgroups and ragged vectors, bias and output scale."""
    bias_dtype = torch.bfloat16 if out_dtype == torch.bfloat16 else None
    sr = 2.0 if out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2) else None
    for variant in (0, 12) if sr or bias_dtype else (0,):
        run_case(m, k, n, fa, fb, out_dtype, rowwise, bias_dtype, sr, variant=variant, seed=m + n)


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[0], FLOAT8[1])])
@pytest.mark.parametrize("m,k,n,out_dtype,rowwise,variant", [
    (128, 2048, 264, torch.bfloat16, True, 14 | 2 << 8), (200, 4096, 520, torch.float32, False, 14 | 4 << 8), (70, 8192, 77, torch.float8_e4m3fn, True, 14 | 16 << 8),
    (130, 8192, 1000, torch.bfloat16, True, 0), (96, 16384, 520, torch.float16, True, 0), (512, 4096, 1030, torch.bfloat16, False, 0),
    (300, 14336, 520, torch.float32, True, 0), (256, 8192, 1024, torch.float8_e5m2, True, 0)])
def test_scaled_mm_tile_kernel_k_slices(fa, fb, m, k, n, out_dtype, rowwise, variant):
    """65 rows and more against few tiles: the 128 x 128 tile kernel with K in slices over workgroups, the slices'
    float32 partial sums in the workspace, added up in slice order by a second launch that runs the epilogue (scales,
    bias, output scale, cast): asked for (variant 14) and planned; every output type, rows and columns past the last
    whole tile, n off the vector width."""
    bias_dtype = torch.bfloat16 if out_dtype == torch.bfloat16 else None
    sr = 2.0 if out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2) else None
    run_case(m, k, n, fa, fb, out_dtype, rowwise, bias_dtype, sr, variant=variant, seed=m + n)


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0])])
@pytest.mark.parametrize("m,k,n,out_dtype,rowwise", [
    (96, 8208, 520, torch.bfloat16, True), (130, 4112, 264, torch.float32, True), (256, 16400, 128, torch.bfloat16, False),
    (65, 4112, 200, torch.float8_e4m3fn, True), (100, 8208, 1000, torch.float16, False)])  # (k not in steps of 128 bytes: no slices of the tile kernel)
def test_scaled_mm_row_blocks_on_few_row_kernel(fa, fb, m, k, n, out_dtype, rowwise):
    """65 to 256 rows against few columns (few tiles for the tile kernels, whose workgroups each walk all of K) run as
    passes of the few-row kernel over blocks of 64 rows: a short last block, the row scales and output rows offset with
    the block, every output size."""
    bias_dtype = torch.bfloat16 if out_dtype == torch.bfloat16 else None
    sr = 2.0 if out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2) else None
    run_case(m, k, n, fa, fb, out_dtype, rowwise, bias_dtype, sr, seed=m + n)


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[1])])
@pytest.mark.parametrize("m,k,n,out_dtype,rowwise,nt,slices", [
    (5, 4096, 80, torch.bfloat16, True, 1, 2), (16, 2064, 64, torch.float8_e4m3fn, False, 2, 2), (33, 8192, 200, torch.bfloat16, True, 2, 4),
    (20, 4112, 1000, torch.float32, True, 1, 3), (64, 16400, 520, torch.bfloat16, False, 4, 8), (50, 28672, 100, torch.float16, True, 2, 16),
    (64, 4096, 72, torch.bfloat16, True, 2, 31),
    # planned: few columns against long rows (slices of K over workgroups)
    (8, 16384, 1024, torch.bfloat16, True, 0, 0), (32, 8192, 1024, torch.float32, False, 0, 0), (32, 28672, 1024, torch.bfloat16, True, 0, 0),
    (64, 8192, 2000, torch.float8_e5m2, True, 0, 0)])
def test_scaled_mm_few_rows_k_slices(fa, fb, m, k, n, out_dtype, rowwise, nt, slices):
    """The few-row kernel with K cut into slices over workgroups (their tiles through the workspace, added up by a
    second launch, which runs the epilogue): asked for (slices that do not divide the chunks of k, a short last slice,
    more slices asked for than half the chunks) and planned (what N = 1024 and 2048 get); every output type."""
    bias_dtype = torch.bfloat16 if out_dtype == torch.bfloat16 else None
    sr = 2.0 if out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2) else None
    run_case(m, k, n, fa, fb, out_dtype, rowwise, bias_dtype, sr, variant=12 | nt << 8 | slices << 12 if nt else 0, seed=m + n)


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[0], FLOAT8[1]), (FLOAT8[1], FLOAT8[1])])
@pytest.mark.parametrize("m,k,n,out_dtype,rowwise", [
    (1, 1024, 64, torch.bfloat16, False), (1, 4096, 1001, torch.bfloat16, True), (2, 2064, 200, torch.float8_e4m3fn, True),
    (2, 8192, 77, torch.float32, True), (1, 16384, 30, torch.float16, False), (3, 1040, 130, torch.bfloat16, True),
    (4, 4096, 520, torch.float8_e5m2, False), (4, 1024, 9, torch.float32, True)])
def test_scaled_mm_one_to_four_rows_on_vector_units(fa, fb, m, k, n, out_dtype, rowwise):
    """One and two rows (and three and four against few columns) run on the vector-unit kernel: both operands widened
    exactly to bfloat16, two-element dot products into float32 sums.  Asked for as variant 13 and as planned; every
    split of K over a workgroup's waves, column counts that leave the last workgroup short, every output type."""
    bias_dtype = torch.bfloat16 if out_dtype == torch.bfloat16 else None
    sr = 2.0 if out_dtype in (torch.float8_e4m3fn, torch.float8_e5m2) else None
    for variant in (13, 0):
        run_case(m, k, n, fa, fb, out_dtype, rowwise, bias_dtype, sr, variant=variant, seed=3 * m + n)


def test_scaled_mm_fp8_output_saturation_and_nan():
    # large products: e4m3fn output overflows to NaN (c10 does not saturate), e5m2 to inf
    run_case(32, 256, 32, FLOAT8[0], FLOAT8[0], torch.float8_e4m3fn, False, scale=8.0)
    run_case(32, 256, 32, FLOAT8[0], FLOAT8[0], torch.float8_e5m2, False, scale=30.0, scale_result=0.01)


def test_scaled_mm_golden_fixtures():
    import _dev
    g = np.load(os.path.join(GOLDEN, "f8.npz"))
    for key in [k[:-2] for k in g.files if k.endswith("_a")]:
        fa, fb, odt = (int(v) for v in g[key + "_fmt"])
        kw = dict(bias=g[key + "_bias"] if key + "_bias" in g else None, bias_dtype=oracle.BF16,
                  scale_result=float(g[key + "_sr"]) if key + "_sr" in g else None, out_dtype=odt)
        got = _dev.scaled_mm(g[key + "_a"], fa, g[key + "_bt"], fb, g[key + "_sa"], g[key + "_sb"], False, **kw)
        _, mag = oracle.scaled_mm(g[key + "_a"], fa, g[key + "_bt"], fb, g[key + "_sa"], g[key + "_sb"], False,
                                  want_mag=True, **kw)
        want = oracle.to_f32(g[key + "_out"], odt).astype(np.float64)
        if key + "_sr" in g:
            mag = mag / float(g[key + "_sr"])
        tol = ref_tol(want, mag, odt) + (HW_WINDOW * mag if on_matrix_cores(odt, 0, 32) else 0)
        assert (np.abs(oracle.to_f32(got, odt) - want) <= tol).all(), key


def _closed_form(a_rows, bt_rows, sa_rows, sb_cols):
    """(float64 sum, magnitude sum) of rows of A against rows of B^T, scaled."""
    af = oracle.fp8_table(oracle.E4M3)[a_rows].astype(np.float64)
    bf = oracle.fp8_table(oracle.E4M3)[bt_rows].astype(np.float64)
    scale = np.asarray(sa_rows, np.float64).reshape(-1, 1) * np.asarray(sb_cols, np.float64).reshape(1, -1)
    return (af @ bf.T) * scale, (np.abs(af) @ np.abs(bf).T) * scale


def _stripes_check(a, bt, sa, sb, got, rows, cols, rowwise):
    """Whole output rows `rows` (every column) and whole output columns `cols` (every row) against the float64
    closed form: stripes that cross every tile, wave and epilogue-pass boundary of the kernel, so that a tile, wave
    or pass written to the wrong place cannot hide between sampled points."""
    m, n = a.shape[0], bt.shape[0]
    sa_all = sa.reshape(-1) if rowwise else np.full(m, float(sa))
    sb_all = sb.reshape(-1) if rowwise else np.full(n, float(sb))

    def check(sub, truth, mag):
        sub = oracle.bf16_to_f32(sub).astype(np.float64)
        assert (np.abs(sub - truth) <= ref_tol(truth, mag, oracle.BF16) + HW_WINDOW * mag).all()
        assert np.allclose(sub, truth, rtol=1e-2, atol=1e-2)  # the stated bar for bfloat16 outputs

    for c0 in range(0, n, 4096):  # (columns in pieces: the float64 operand of a piece is 256 MB)
        truth, mag = _closed_form(a[rows], bt[c0:c0 + 4096], sa_all[rows], sb_all[c0:c0 + 4096])
        check(got[rows][:, c0:c0 + 4096], truth, mag)
    for r0 in range(0, m, 4096):
        truth, mag = _closed_form(a[r0:r0 + 4096], bt[cols], sa_all[r0:r0 + 4096], sb_all[cols])
        check(got[r0:r0 + 4096][:, cols], truth, mag)


# rows / columns either side of every boundary of the 256 x 256 tile kernel: its waves' 64 x 128 sub-tiles, the
# matrix-core tiles of 32, the epilogue's passes of 64 columns, tile edges, panel edges (8 tile rows), the last ones
BOUNDARY_ROWS = [0, 31, 32, 63, 64, 255, 256, 2047, 2048]
BOUNDARY_COLS = [0, 3, 4, 63, 64, 127, 128, 255, 256, 1023]


def test_scaled_mm_config4_8192_cubed():
    """BASELINE config 4: e4m3fn 8192^3, per-tensor scales 0.5 / 0.5, bf16 out.  A full CPU product takes an hour,
    so: whole rows and whole columns across every kernel boundary against the float64 closed form, and an exactness
    property over the whole output (scaling an operand by 2 doubles every output bit for bit)."""
    import _dev
    m = n = k = 8192
    a = torch.randn(m, k, generator=gen(1040)).clamp(-448, 448).to(torch.float8_e4m3fn)
    bt = torch.randn(n, k, generator=gen(1041)).clamp(-448, 448).to(torch.float8_e4m3fn)
    got = _dev.scaled_mm(bits(a), oracle.E4M3, bits(bt), oracle.E4M3, [0.5], [0.5], False, out_dtype=oracle.BF16)
    _stripes_check(bits(a), bits(bt), np.float32(0.5), np.float32(0.5), got, np.array(BOUNDARY_ROWS + [4095, 4096, m - 1]),
                   np.array(BOUNDARY_COLS + [5000, n - 2, n - 1]), False)
    got2 = _dev.scaled_mm(bits(a), oracle.E4M3, bits(bt), oracle.E4M3, [1.0], [0.5], False, out_dtype=oracle.BF16)
    assert np.array_equal(oracle.bf16_to_f32(got2), oracle.bf16_to_f32(got) * 2)


@pytest.mark.parametrize("variant,out_dtype", [(8, oracle.BF16), (11, oracle.BF16), (5, oracle.BF16), (9, oracle.F32), (6, oracle.F32)])
def test_scaled_mm_large_tile_kernels_on_ragged_shapes(variant, out_dtype):
    """The 256 x 256 tile kernels (8 waves of 64 x 128 and 4 waves of 128 x 128; fp8 matrix cores and the widened,
    exact form) forced at a shape whose rows and columns are no multiple of any tile, wave or pass size: every output
    against the oracle."""
    import _dev
    m, k, n = 300, 1024, 520
    a = torch.randn(m, k, generator=gen(1070)).to(torch.float8_e4m3fn)
    bt = torch.randn(n, k, generator=gen(1071)).to(torch.float8_e4m3fn)
    sa = torch.empty(m, 1).uniform_(0.5, 2, generator=gen(1072)).numpy()
    sb = torch.empty(1, n).uniform_(0.5, 2, generator=gen(1073)).numpy()
    bias = torch.randn(n, generator=gen(1074)).numpy()
    got = _dev.scaled_mm(bits(a), oracle.E4M3, bits(bt), oracle.E4M3, sa, sb, True, bias=bias, bias_dtype=oracle.F32,
                         out_dtype=out_dtype, variant=variant)
    want, mag = oracle.scaled_mm(bits(a), oracle.E4M3, bits(bt), oracle.E4M3, sa, sb, True, bias, oracle.F32, None, out_dtype,
                                 want_mag=True)
    want = oracle.to_f32(want, out_dtype).astype(np.float64)
    tol = ref_tol(want, mag, out_dtype) + (HW_WINDOW * mag if out_dtype == oracle.BF16 else 0)
    assert got.shape == (m, n) and (np.abs(oracle.to_f32(got, out_dtype) - want) <= tol).all()


@pytest.mark.parametrize("m,k,n,rowwise,with_bias,fb", [
    (257, 256, 264, False, True, 0),     # the fewest steps it takes; one row and 8 columns beyond a tile
    (1, 512, 8, False, False, 0),        # one row, 8 columns
    (515, 640, 1032, True, True, 1),     # e5m2 second operand
    (4352, 384, 4360, True, False, 0),   # 306 tiles: more than there are workgroups, so streams that run through two tiles
])
def test_scaled_mm_stream_kernel(m, k, n, rowwise, with_bias, fb):
    """The stream kernel (variant 11: loads that run ahead across tiles, barrier in the middle of a step) forced at
    shapes it serves: every output against the oracle, and bit for bit the tile kernel's (same products, same order)."""
    import _dev
    a = torch.randn(m, k, generator=gen(1080)).to(FLOAT8[0])
    bt = torch.randn(n, k, generator=gen(1081)).to(FLOAT8[fb])
    if rowwise:
        sa = torch.empty(m, 1).uniform_(0.5, 2, generator=gen(1082)).numpy()
        sb = torch.empty(1, n).uniform_(0.5, 2, generator=gen(1083)).numpy()
    else:
        sa, sb = np.array([0.75], dtype=np.float32), np.array([1.5], dtype=np.float32)
    bias = torch.randn(n, generator=gen(1084)).numpy() if with_bias else None
    kw = dict(bias=bias, bias_dtype=oracle.F32) if with_bias else {}
    got = {v: _dev.scaled_mm(bits(a), oracle.E4M3, bits(bt), ODT[FLOAT8[fb]], sa, sb, rowwise, out_dtype=oracle.BF16, variant=v, **kw)
           for v in (11, 8)}
    assert got[11].shape == (m, n) and np.array_equal(got[11], got[8])
    if m * n <= 1 << 20:
        want, mag = oracle.scaled_mm(bits(a), oracle.E4M3, bits(bt), ODT[FLOAT8[fb]], sa, sb, rowwise, bias, oracle.F32, None, oracle.BF16,
                                     want_mag=True)
        want = oracle.to_f32(want, oracle.BF16).astype(np.float64)
        assert (np.abs(oracle.to_f32(got[11], oracle.BF16) - want) <= ref_tol(want, mag, oracle.BF16) + HW_WINDOW * mag).all()
    # float8 outputs with an output scale: 8 codes per store
    for odt in (oracle.E4M3, oracle.E5M2):
        out8 = {v: _dev.scaled_mm(bits(a), oracle.E4M3, bits(bt), ODT[FLOAT8[fb]], sa, sb, rowwise, out_dtype=odt, scale_result=16.0, variant=v, **kw)
                for v in (11, 8)}
        assert np.array_equal(out8[11], out8[8])
        if m * n <= 1 << 20:
            want, mag = oracle.scaled_mm(bits(a), oracle.E4M3, bits(bt), ODT[FLOAT8[fb]], sa, sb, rowwise, bias, oracle.F32, 16.0, odt, want_mag=True)
            want = oracle.to_f32(want, odt).astype(np.float64)
            fin = np.isfinite(want)
            err = np.abs(oracle.to_f32(out8[11], odt).astype(np.float64) - want)
            # (one step of the output format where the sums' small differences cross a rounding boundary: below the
            #  smallest normal value a step is a fixed 2^-9 / 2^-16, not a fraction of the value)
            step = 2.0 ** -9 if odt == oracle.E4M3 else 2.0 ** -16
            assert (err[fin] <= (ref_tol(want, mag / 16.0, odt) + HW_WINDOW * mag / 16.0 + step)[fin]).all()


def test_scaled_mm_stream_kernel_nan_and_inf():
    """NaN and infinities through the stream kernel's epilogue, whose bfloat16 conversion looks at its values one by one
    only where a wave has seen a NaN: NaN operands (both e4m3fn codes), e5m2 infinities of both signs (inf - inf and
    0 x inf included) and a NaN in the bias.  Every NaN output is 0x7fc0 as c10 writes it, the outputs are bit for bit
    the tile kernel's, and NaN / infinity sit where the oracle has them."""
    import _dev
    m, k, n = 512, 256, 520
    a = bits(torch.randn(m, k, generator=gen(1095)).to(FLOAT8[0])).copy()
    bt = bits(torch.randn(n, k, generator=gen(1096)).to(FLOAT8[1])).copy()
    a[3, 17], a[300, 5] = 0x7F, 0xFF            # e4m3fn NaN of either sign
    a[7, :] = 0                                  # a zero row: 0 x inf below
    bt[9, 40], bt[9, 41] = 0x7C, 0xFC            # e5m2 +inf and -inf in one column: inf - inf or +-inf
    bt[260, 100] = 0x7C                          # +inf alone
    bt[519, 0] = 0x7E                            # e5m2 NaN
    bias = torch.randn(n, generator=gen(1097)).numpy()
    bias[33] = np.nan
    sa, sb = np.array([0.5], dtype=np.float32), np.array([2.0], dtype=np.float32)
    got = {v: _dev.scaled_mm(a, oracle.E4M3, bt, oracle.E5M2, sa, sb, False, bias=bias, bias_dtype=oracle.F32, out_dtype=oracle.BF16, variant=v)
           for v in (11, 8)}
    assert np.array_equal(got[11], got[8])
    want = oracle.to_f32(oracle.scaled_mm(a, oracle.E4M3, bt, oracle.E5M2, sa, sb, False, bias, oracle.F32, None, oracle.BF16), oracle.BF16)
    have = oracle.to_f32(got[11], oracle.BF16)
    assert np.array_equal(np.isnan(have), np.isnan(want)) and np.isnan(want[3]).all() and np.isnan(want[:, 33]).all() and np.isnan(want[7, 9])
    assert np.array_equal(np.isinf(have), np.isinf(want)) and np.array_equal(np.sign(have[np.isinf(have)]), np.sign(want[np.isinf(want)]))
    assert np.isinf(want[:, 260]).sum() > m // 2
    assert (got[11][np.isnan(have)] == 0x7FC0).all()


def test_scaled_mm_zero_sums_keep_their_sign():
    """A negative scale turns a zero sum into -0.0; without a bias it must stay -0.0 in the output (the kernels add the
    bias from registers: an absent bias is -0.0f, whose addition changes nothing), with a bias of +0.0 it becomes +0.0."""
    import _dev
    m, k, n = 256, 256, 256
    a = np.zeros((m, k), dtype=np.uint8)
    bt = bits(torch.randn(n, k, generator=gen(1090)).to(FLOAT8[0]))
    for variant in (11, 8, 1):
        got = _dev.scaled_mm(a, oracle.E4M3, bt, oracle.E4M3, np.array([-1.0], np.float32), np.array([1.0], np.float32), False,
                             out_dtype=oracle.BF16, variant=variant)
        assert (got == 0x8000).all(), variant
        got = _dev.scaled_mm(a, oracle.E4M3, bt, oracle.E4M3, np.array([-1.0], np.float32), np.array([1.0], np.float32), False,
                             bias=np.zeros(n, np.float32), bias_dtype=oracle.F32, out_dtype=oracle.BF16, variant=variant)
        assert (got == 0).all(), variant


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[1], FLOAT8[1])])
def test_scaled_mm_float32_output_large(fa, fb):
    """float32 output at a size where the path matters (the exact kernel on 256x256 tiles, direct-to-LDS loads):
    whole rows and whole columns either side of every tile, wave and matrix-core-tile boundary, each inside the
    reference's bound eps*|want| + 2^-20*sum|a||b| and within the stated 1e-4 of the float64 closed form."""
    import _dev
    m, k, n = 1024, 8192, 1280
    a = torch.randn(m, k, generator=gen(1060)).to(fa)
    bt = torch.randn(n, k, generator=gen(1061)).to(fb)
    sa = torch.empty(m, 1).uniform_(0.5, 2, generator=gen(1062)).numpy()
    sb = torch.empty(1, n).uniform_(0.5, 2, generator=gen(1063)).numpy()
    got = _dev.scaled_mm(bits(a), ODT[fa], bits(bt), ODT[fb], sa, sb, True, out_dtype=oracle.F32).astype(np.float64)
    af = oracle.fp8_table(ODT[fa])[bits(a)].astype(np.float64)
    bf = oracle.fp8_table(ODT[fb])[bits(bt)].astype(np.float64)
    rows, cols = np.array([0, 31, 32, 63, 64, 127, 128, 255, 256, 700, 1023]), np.array([0, 1, 31, 32, 127, 128, 255, 256, 1023, 1024, 1279])

    def stripe(sub, x, y, scale):
        truth, mag = (x @ y.T) * scale, (np.abs(x) @ np.abs(y).T) * scale
        assert (np.abs(sub - truth) <= ref_tol(truth, mag, oracle.F32)).all()
        assert np.allclose(sub, truth, rtol=1e-4, atol=1e-4)
    stripe(got[rows], af[rows], bf, sa.reshape(-1)[rows][:, None].astype(np.float64) * sb.reshape(1, -1))   # whole rows
    stripe(got[:, cols], af, bf[cols], sa.reshape(-1, 1).astype(np.float64) * sb.reshape(-1)[cols][None, :])  # whole columns


def test_scaled_mm_config5_rowwise_70b():
    """BASELINE config 5: rowwise scales, M=4096, K=8192, N=28672, bf16 out."""
    import _dev
    m, k, n = 4096, 8192, 28672
    a = torch.randn(m, k, generator=gen(1050)).to(torch.float8_e4m3fn)
    bt = torch.randn(n, k, generator=gen(1051)).to(torch.float8_e4m3fn)
    sa = torch.empty(m, 1).uniform_(0.5, 2, generator=gen(1052)).numpy()
    sb = torch.empty(1, n).uniform_(0.5, 2, generator=gen(1053)).numpy()
    got = _dev.scaled_mm(bits(a), oracle.E4M3, bits(bt), oracle.E4M3, sa, sb, True, out_dtype=oracle.BF16)
    _stripes_check(bits(a), bits(bt), sa, sb, got, np.array(BOUNDARY_ROWS + [m - 1]),
                   np.array(BOUNDARY_COLS + [14335, 14336, n - 256, n - 1]), True)


def test_scaled_mm_errors():
    from torch_vulkan_amd import abi
    buf = abi.Buffer(4096)
    p = abi.F8Params(a=buf.address, b=buf.address, scale_a=buf.address, scale_b=buf.address, out=buf.address, m=4, n=4,
                     k=16, lda=16, ldb=16, ldo=4, fmt_a=abi.E4M3, fmt_b=abi.F32, out_dtype=abi.BF16)
    with pytest.raises(abi.VktError, match="e4m3fn or e5m2"):
        abi.dispatch("fp8mm", [0], p)
    p.fmt_b = abi.E5M2
    p.lda = 8
    with pytest.raises(abi.VktError, match="strides"):
        abi.dispatch("fp8mm", [0], p)
    p.lda = 16
    with pytest.raises(abi.VktError, match="unknown variant"):
        abi.dispatch("fp8mm", [99], p)
