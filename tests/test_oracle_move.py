"""Pins of the oracle's strided move and strided cast (oracle.move, oracle.cast_strided) against numpy
views and PyTorch's CPU copy_ / contiguous() / fill_ / to(): the layouts the reference's callers
produce (transposes, slices, broadcasts, im2col-like views of up to 8 dims)."""
import numpy as np
import pytest
import torch

import oracle


def rng(seed):
    return np.random.default_rng(seed)


CASES = [
    # (base shape, view builder)
    ((6, 10), lambda x: x.T),
    ((7, 9), lambda x: x[::2, 1::3]),
    ((4, 5, 6), lambda x: x.transpose(2, 0, 1)),
    ((3, 4, 5, 6), lambda x: x.transpose(0, 3, 1, 2)[:, ::2]),
    ((2, 3, 2, 3, 2, 3), lambda x: x.transpose(5, 4, 3, 2, 1, 0)),
    ((2, 2, 3, 2, 2, 2, 3, 2), lambda x: x.transpose(7, 0, 6, 1, 5, 2, 4, 3)),
    ((1, 7), lambda x: np.broadcast_to(x, (5, 7))),
    ((5, 1), lambda x: np.broadcast_to(x, (5, 7))),
]


@pytest.mark.parametrize("dtype", [np.uint8, np.uint16, np.float32, np.int64, np.complex128], ids=lambda d: np.dtype(d).name)
@pytest.mark.parametrize("case", range(len(CASES)))
def test_move_matches_numpy_and_torch(dtype, case):
    shape, view = CASES[case]
    base = (rng(case).integers(0, 250, shape)).astype(dtype)
    src = view(base)
    want = np.ascontiguousarray(src)
    got = oracle.move(np.zeros(src.shape, dtype), src)
    assert got.tobytes() == want.tobytes()
    # into a strided destination, as copy_ does; untouched elements stay
    buf = np.full((src.shape[0] * 2,) + src.shape[1:], 7, dtype)
    oracle.move(buf[::2], src)
    t = torch.full(buf.shape, 7, dtype=torch.from_numpy(buf).dtype)
    t[::2].copy_(torch.from_numpy(np.ascontiguousarray(src)))
    assert buf.tobytes() == t.numpy().tobytes()


def test_move_contiguous_is_torch_contiguous():
    x = torch.arange(2 * 3 * 4 * 5, dtype=torch.int32).reshape(2, 3, 4, 5)
    for perm in [(3, 2, 1, 0), (0, 2, 1, 3), (1, 0, 3, 2)]:
        v = x.permute(perm)
        got = oracle.move(np.empty(tuple(v.shape), np.int32), v.numpy())
        assert np.array_equal(got, v.contiguous().numpy())


@pytest.mark.parametrize("dtype,value", [(np.uint8, 200), (np.uint16, 0xBEEF), (np.float32, -1.5), (np.int64, -(2**40) + 3),
                                         (np.complex128, 1.5 - 2j)])
def test_fill(dtype, value):
    buf = np.zeros((5, 6, 7), dtype)
    oracle.move(buf[1::2, :, ::3], value=np.asarray(value, dtype))
    want = torch.zeros(5, 6, 7, dtype=torch.from_numpy(buf).dtype)
    want[1::2, :, ::3].fill_(value)
    assert buf.tobytes() == want.numpy().tobytes()


TORCH_DT = {oracle.F32: torch.float32, oracle.F16: torch.float16, oracle.BF16: torch.bfloat16}


def as_np(t):
    return t.numpy() if t.dtype == torch.float32 else t.view(torch.int16).numpy().view(np.uint16)


@pytest.mark.parametrize("src", [oracle.F32, oracle.F16, oracle.BF16])
@pytest.mark.parametrize("dst", [oracle.F32, oracle.F16, oracle.BF16])
def test_cast_strided_matches_torch(src, dst):
    if src == dst:
        pytest.skip("same type: a move")
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(6, 8, 5, generator=g) * 300).to(TORCH_DT[src])
    x[0, 0, :4] = torch.tensor([float("nan"), float("inf"), -0.0, 65520.0]).to(TORCH_DT[src])
    v = x.permute(2, 0, 1)[:, ::2]
    want = v.to(TORCH_DT[dst]).contiguous()
    got = oracle.cast_strided(np.zeros(tuple(v.shape), as_np(want).dtype), dst, as_np(x).transpose(2, 0, 1)[:, ::2], src)
    nan = torch.isnan(want.float()).numpy()
    assert np.array_equal(got[~nan], as_np(want)[~nan])
    assert np.isnan(oracle.to_f32(got[nan], dst)).all()
    # broadcast source into a strided destination
    row = x[0, 0]
    out = torch.zeros(4, 10, dtype=TORCH_DT[dst])
    out[:, ::2].copy_(row)
    buf = np.zeros((4, 10), as_np(out).dtype)
    oracle.cast_strided(buf[:, ::2], dst, as_np(row), src)
    assert np.array_equal(buf[~torch.isnan(out.float()).numpy()], as_np(out)[~torch.isnan(out.float()).numpy()])
