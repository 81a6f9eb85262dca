"""GPU parity of _dyn_quant_matmul_4bit through the C ABI: both kernel families ("qmm4_*"
on the reference's buffers, "qmm4c_*" streaming the compact side-car) must equal the oracle
and PyTorch's CPU op bit for bit (reference tests/python/test_quant.py:61-84)."""
import os

import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen
from _cases import INT4_SHAPES, int4_rows, int4_weights

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
EXTRA = [(2, 4096, 300, 32, True), (3, 14336, 20, 32, True), (9, 28672, 6, 128, False), (4, 4096 + 2048, 12, 64, False), (7, 8192, 9, 128, True), (3, 512, 5, 256, False),
         (6, 4160, 10, 4160, True), (1, 32, 1, 32, False), (5, 8, 3, 8, True),
         # more than 4 rows: the matrix-core layout's row tiles (16 rows each, 64 rows per launch)
         (70, 512, 40, 64, True), (33, 1056, 17, 32, False), (16, 4096, 64, 128, True), (20, 4160, 10, 4160, False),
         (130, 96, 33, 32, True), (17, 2048, 16, 256, False),
         # many rows: a wave per tile that walks all of K, every block size of the matrix-core layout
         (64, 4160, 40, 4160, True), (200, 1024, 48, 128, False), (100, 2048, 20, 256, True), (49, 640, 130, 64, False),
         # more rows than one launch of the matrix-core kernels takes (16384)
         (16400, 64, 20, 32, True)]


@pytest.mark.parametrize("m,k,n,bs,bias", INT4_SHAPES + EXTRA)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_q4_bit_exact(m, k, n, bs, bias, dtype):
    import _dev
    from torch_vulkan_amd import abi
    if dtype == torch.bfloat16 and bs != k:
        pytest.skip("bfloat16 inputs are channelwise only (the CPU's check)")
    w, sc, bvec = int4_weights(n, k, bs, bias=bias)
    x = int4_rows(m, k, dtype)
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, bvec, bs, k, n)
    want = bits(torch._dyn_quant_matmul_4bit(x, packed, bs, k, n))
    odt = ODT[dtype]
    assert np.array_equal(oracle.q4_matmul(bits(x), odt, packed.numpy(), bs, k, n), want)
    got, q, recip, nzp = _dev.q4_reference_layout(bits(x), odt, packed.numpy(), bs, k, n, want_intermediates=True)
    oq, orecip, onzp = oracle.q4_rowquant(bits(x), odt, bs != k)
    assert np.array_equal(q, oq) and np.array_equal(nzp, onzp)
    assert np.array_equal(recip.view(np.uint32), orecip.view(np.uint32))
    assert np.array_equal(got, want)
    if abi.lib().vkt_qmm4c_bytes(n, k, bs):
        cw = _dev.CompactWeights(packed.numpy(), bs, k, n)
        assert np.array_equal(_dev.q4_compact(bits(x), odt, cw, fused=True), want)
        assert np.array_equal(_dev.q4_compact(bits(x), odt, cw, fused=False), want)
        cm = _dev.CompactWeights(packed.numpy(), bs, k, n, layout=1)
        assert np.array_equal(_dev.q4_compact(bits(x), odt, cm, fused=True), want)
        assert np.array_equal(_dev.q4_compact(bits(x), odt, cm, fused=False), want)
        if m > 4:  # both matrix-core kernels, whichever the row count selects
            assert np.array_equal(_dev.q4_compact(bits(x), odt, cm, fused=False, flags=16), want)
            assert np.array_equal(_dev.q4_compact(bits(x), odt, cm, fused=True, flags=32 | 64), want)
            assert np.array_equal(_dev.q4_compact(bits(x), odt, cm, fused=False, flags=32 | 128), want)
            assert np.array_equal(_dev.q4_compact(bits(x), odt, cm, fused=True, flags=32 | 192), want)


@pytest.mark.parametrize("m", [1, 32])
def test_q4_config3(m):
    """BASELINE config 3: K=4096, N=11008, bs=32, bias, fp32 activations ~N(0,1)."""
    import _dev
    n, k, bs = 11008, 4096, 32
    w4 = torch.randint(0, 16, (n, k), dtype=torch.uint8, generator=gen(1030))
    wbytes = (w4[:, 0::2] + 16 * w4[:, 1::2]).contiguous()
    sc = torch.empty(n, k // bs).uniform_(0.01, 0.05, generator=gen(1031))
    bias = torch.randn(n, generator=gen(1032)) * 0.1
    x = torch.randn(m, k, generator=gen(1033))
    packed = torch._dyn_quant_pack_4bit_weight(wbytes, sc, bias, bs, k, n)
    # The oracle restates the reference's arithmetic (qmm4.slang, compiled in precise mode:
    # a multiplication, then an addition per block).  PyTorch's x86 CPU build contracts that
    # pair into a fused multiply-add, which shows once scales carry a full float32 mantissa
    # (the reference's own tests use bfloat16-valued scales, where the products are exact
    # and both agree bit for bit).  So: bit-exact against the oracle, and within the stated
    # float32 tolerance of the CPU op.
    want = oracle.q4_matmul(x.numpy(), oracle.F32, packed.numpy(), bs, k, n)
    cpu = torch._dyn_quant_matmul_4bit(x, packed, bs, k, n).numpy()
    cw = _dev.CompactWeights(packed.numpy(), bs, k, n)
    got = _dev.q4_compact(x.numpy(), oracle.F32, cw)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.allclose(got, cpu, rtol=1e-4, atol=1e-4)
    got = _dev.q4_compact(x.numpy(), oracle.F32, _dev.CompactWeights(packed.numpy(), bs, k, n, layout=1))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    if m == 1:
        got = _dev.q4_reference_layout(x.numpy(), oracle.F32, packed.numpy(), bs, k, n)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # bfloat16-valued scales: equal to the CPU op bit for bit as well
    packed_b = torch._dyn_quant_pack_4bit_weight(wbytes, sc.bfloat16(), bias, bs, k, n)
    cpu_b = torch._dyn_quant_matmul_4bit(x, packed_b, bs, k, n).numpy()
    got_b = _dev.q4_compact(x.numpy(), oracle.F32, _dev.CompactWeights(packed_b.numpy(), bs, k, n))
    assert np.array_equal(got_b.view(np.uint32), cpu_b.view(np.uint32))


@pytest.mark.parametrize("m,k,n,bs,bias", [(2, 4096, 4128, 32, True), (3, 2048, 8200, 64, False), (2, 1024, 40, 128, True),
                                           (3, 4096, 16, 4096, False), (2, 512, 12300, 256, True)])
def test_q4_several_tiles_per_workgroup(m, k, n, bs, bias):
    """Two and three rows on the streaming kernel with two and three column tiles per workgroup (the launcher's choice
    when a compute unit has that many tiles; forced here through the phase word's bits 8-9), tile counts that leave
    the last workgroup short of tiles."""
    import _dev
    w, sc, bvec = int4_weights(n, k, bs, bias=bias)
    x = int4_rows(m, k, torch.float32)
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, bvec, bs, k, n).numpy()
    want = oracle.q4_matmul(bits(x), oracle.F32, packed, bs, k, n)
    cw = _dev.CompactWeights(packed, bs, k, n)
    for teams in (0, 1, 2, 3):
        got = _dev.q4_compact(bits(x), oracle.F32, cw, flags=teams << 8)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), teams


def test_q4_golden_fixtures():
    import _dev
    g = np.load(os.path.join(GOLDEN, "q4.npz"))
    for i in range(len(INT4_SHAPES)):
        m, k, n, bs, bias = (int(v) for v in g[f"c{i}_shape"])
        for tag, odt in (("f32", oracle.F32), ("bf16", oracle.BF16)):
            key = f"c{i}_{tag}"
            if key + "_out" not in g:
                continue
            assert np.array_equal(_dev.q4_reference_layout(g[key + "_x"], odt, g[f"c{i}_packed"], bs, k, n),
                                  g[key + "_out"]), key
            cw = _dev.CompactWeights(g[f"c{i}_packed"], bs, k, n)
            assert np.array_equal(_dev.q4_compact(g[key + "_x"], odt, cw), g[key + "_out"]), key
            cm = _dev.CompactWeights(g[f"c{i}_packed"], bs, k, n, layout=1)
            assert np.array_equal(_dev.q4_compact(g[key + "_x"], odt, cm), g[key + "_out"]), key


def test_q4_errors():
    from torch_vulkan_amd import abi
    buf = abi.Buffer(4096)
    p = abi.Q4Params(inp=buf.address, q=buf.address, rows=buf.address, packed=buf.address, out=buf.address, m=1, n=2,
                     k=64, bs=48, has_bias=0)
    with pytest.raises(abi.VktError, match="multiple of 32"):
        abi.dispatch("qmm4_f32", [0, 1], p)
    p.bs = 32
    with pytest.raises(abi.VktError, match="GROUPWISE"):
        abi.dispatch("qmm4_f32", [0, 0], p)
    with pytest.raises(abi.VktError, match="PHASE"):
        abi.dispatch("qmm4_f32", [2, 1], p)
    c = abi.Q4CParams(inp=buf.address, q=buf.address, rows=buf.address, compact=buf.address, out=buf.address, m=1, n=2,
                      k=64, bs=32, has_bias=0)
    with pytest.raises(abi.VktError, match="PHASE"):
        abi.dispatch("qmm4c_f32", [3, 1], c)
    with pytest.raises(abi.VktError, match="LAYOUT"):
        abi.dispatch("qmm4c_f32", [2, 1, 2], c)
    with pytest.raises(abi.VktError, match="unknown kernel"):
        abi.dispatch("qmm4_f16", [0, 1], p)
    assert abi.lib().vkt_qmm4c_bytes(8, 96, 96) > 0 and abi.lib().vkt_qmm4c_bytes(8, 192, 96) == 0
