"""GPU parity of the strided data-movement kernels ("move_b<S>", "copy8_b<S>", "cast_<src>_<dst>")
through the C ABI against the oracle's restatement of the reference's index arithmetic and against
PyTorch's CPU contiguous() / copy_ / fill_ / to(): bit-exact (byte moves and correctly rounded casts)."""
import numpy as np
import pytest
import torch

import oracle

pytestmark = pytest.mark.gpu
DTYPES = [np.uint8, np.uint16, np.float32, np.int64, np.complex128]


def rng(seed):
    return np.random.default_rng(seed)


def random_array(shape, dtype, seed):
    raw = rng(seed).integers(0, 256, int(np.prod(shape)) * np.dtype(dtype).itemsize, dtype=np.uint8)
    return raw.view(dtype).reshape(shape)


CASES = [
    ((70, 130), lambda x: x.T),  # transpose: tiles through LDS
    ((257, 64), lambda x: x.T),
    ((33, 48), lambda x: x[::2, 8:40]),  # rows of a slice: widened units
    ((7, 9), lambda x: x[::2, 1::3]),  # strided innermost dim: element by element
    ((4, 50, 66), lambda x: x.transpose(2, 0, 1)),
    ((3, 40, 5, 36), lambda x: x.transpose(0, 3, 2, 1)),
    ((3, 70, 130), lambda x: x.transpose(0, 2, 1)),  # batched transposes: 2-byte elements move as pairs
    ((2, 64, 3, 66), lambda x: x.transpose(0, 3, 2, 1)),  # transpose of dims 1 and 3 under two outer dims
    ((3, 4, 5, 6), lambda x: x.transpose(0, 3, 1, 2)[:, ::2]),
    ((2, 3, 2, 3, 2, 3), lambda x: x.transpose(5, 4, 3, 2, 1, 0)),  # more than 4 dims: copy8
    ((2, 2, 3, 2, 2, 2, 3, 32), lambda x: x.transpose(6, 0, 7, 1, 5, 2, 4, 3)),
    ((1, 64), lambda x: np.broadcast_to(x, (40, 64))),  # broadcast rows
    ((40, 1), lambda x: np.broadcast_to(x, (40, 64))),  # broadcast columns (stride 0 innermost)
    ((1,), lambda x: x),
    ((4096,), lambda x: x[3:4003]),  # misaligned 1-d
]


@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("case", range(len(CASES)))
def test_copy(dtype, case, variant):
    import _dev
    shape, view = CASES[case]
    src = view(random_array(shape, dtype, case))
    want = oracle.move(np.zeros(src.shape, dtype), src)
    assert want.tobytes() == np.ascontiguousarray(src).tobytes()
    got = _dev.move(np.zeros(src.shape, dtype), src, variant=variant)
    assert got.tobytes() == want.tobytes()
    # into every other row of a larger destination: the rows between stay as they were
    big = random_array((src.shape[0] * 2,) + src.shape[1:], dtype, 99)
    want_big = big.copy()
    oracle.move(want_big[::2], src)
    _dev.move(big[::2], src, variant=variant)
    assert big.tobytes() == want_big.tobytes()


@pytest.mark.parametrize("dtype", DTYPES, ids=lambda d: np.dtype(d).name)
def test_copy_into_transposed_destination(dtype):
    """x.t().copy_(y): the destination is the side that is not contiguous along the innermost dim."""
    import _dev
    src = random_array((100, 72), dtype, 3)
    dst = np.zeros((72, 100), dtype)
    _dev.move(dst.T, src)
    assert dst.tobytes() == np.ascontiguousarray(src.T).tobytes()


@pytest.mark.parametrize("variant", [0, 1])
@pytest.mark.parametrize("dtype,value", [(np.uint8, 200), (np.uint16, 0xBEEF), (np.float32, -1.5), (np.int64, -(2**40) + 3),
                                         (np.complex128, 1.5 - 2j)])
def test_fill(dtype, value, variant):
    import _dev
    for shape, cut in [((5, 6, 7), np.s_[1::2, :, ::3]), ((64, 128), np.s_[:, :]), ((33, 48), np.s_[::2, 8:40]), ((1001,), np.s_[1:])]:
        got, want = random_array(shape, dtype, 7), random_array(shape, dtype, 7)
        oracle.move(want[cut], value=np.asarray(value, dtype))
        _dev.move(got[cut], value=np.asarray(value, dtype), variant=variant)
        assert got.tobytes() == want.tobytes()
    t = torch.zeros(5, 6, dtype=torch.from_numpy(np.zeros(1, dtype)).dtype)
    t[:, ::2].fill_(value)
    got = np.zeros((5, 6), dtype)
    _dev.move(got[:, ::2], value=np.asarray(value, dtype))
    assert got.tobytes() == t.numpy().tobytes()


LABEL = {oracle.F32: "f32", oracle.F16: "f16", oracle.BF16: "bf16"}
TORCH_DT = {oracle.F32: torch.float32, oracle.F16: torch.float16, oracle.BF16: torch.bfloat16}


def as_np(t):
    return t.numpy() if t.dtype == torch.float32 else t.view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("src", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("dst", [oracle.F32, oracle.F16, oracle.BF16])
def test_cast_strided(src, dst):
    import _dev
    if src == dst:
        pytest.skip("same type: a move")
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(6, 40, 33, generator=g) * 300).to(TORCH_DT[src])
    x[0, 0, :5] = torch.tensor([float("inf"), -0.0, 65520.0, 1e-8, -65504.0]).to(TORCH_DT[src])
    xn = as_np(x)
    out_dt = as_np(torch.zeros(1, dtype=TORCH_DT[dst])).dtype
    for view in (lambda a: a, lambda a: a.transpose(2, 0, 1)[:, ::2], lambda a: a[:, ::3, 1:30], lambda a: np.broadcast_to(a[0, 0], (7, 33))):
        v = view(xn)
        want = oracle.cast_strided(np.zeros(v.shape, out_dt), dst, v, src)
        got = _dev.move(np.zeros(v.shape, out_dt), v, cast=(LABEL[src], LABEL[dst]))
        assert got.tobytes() == want.tobytes()
    # against PyTorch's CPU conversion of the same view
    tv = x.permute(2, 0, 1)[:, ::2]
    got = _dev.move(np.zeros(tuple(tv.shape), out_dt), xn.transpose(2, 0, 1)[:, ::2], cast=(LABEL[src], LABEL[dst]))
    assert got.tobytes() == as_np(tv.to(TORCH_DT[dst]).contiguous()).tobytes()


def test_large_transpose_and_rows():
    """bf16 4096 x 8192 transposed and its even rows: the bench shapes, checked whole."""
    import _dev
    src = random_array((4096, 8192), np.uint16, 11)
    got = _dev.move(np.zeros((8192, 4096), np.uint16), src.T)
    assert np.array_equal(got, src.T)
    got = _dev.move(np.zeros((2048, 8192), np.uint16), src[::2])
    assert np.array_equal(got, src[::2])


def test_errors():
    from torch_vulkan_amd import abi
    buf = abi.Buffer(4096)
    p = abi.StridedParams(out=buf.address, a=buf.address, n=12, ndim=2)
    p.size[0], p.size[1], p.size[2], p.size[3] = 3, 5, 1, 1
    with pytest.raises(abi.VktError, match="product of the sizes"):
        abi.dispatch("move_b4", [abi.MOVE_COPY], p)
    p.n = 15
    with pytest.raises(abi.VktError, match="copy and fill"):
        abi.dispatch("move_b4", [2], p)
    with pytest.raises(abi.VktError, match="unknown kernel"):
        abi.dispatch("move_b3", [0], p)
    p.a = 0
    with pytest.raises(abi.VktError, match="null or misaligned"):
        abi.dispatch("move_b4", [abi.MOVE_COPY], p)
    p.a = buf.address + 2
    with pytest.raises(abi.VktError, match="null or misaligned"):
        abi.dispatch("move_b4", [abi.MOVE_COPY], p)
    with pytest.raises(abi.VktError, match="unknown kernel"):
        abi.dispatch("cast_f32_i8", [], p)
