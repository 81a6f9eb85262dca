"""Seeded random shapes through the kernels' own planners (no variant bits), chosen to fall on both sides of every
threshold at which a launcher changes kernels: row counts around 1-4, 8-9, 32-33, 191-193 (int8 weights) and 3-5,
16-17, the waves-per-SIMD threshold of the many-row kernel (int4 weights); k on and off the multiples the fast
kernels need; odd n.  int8 results stay inside the reference's band around the float64 sum, int4 results equal the
oracle bit for bit."""
import numpy as np
import pytest
import torch

import oracle
from _util import ODT, bits, gen
from test_gpu_qmm8 import check_q8
from _cases import int4_rows, int4_weights, int8_case

pytestmark = pytest.mark.gpu


def _q8_shapes():
    rng = np.random.default_rng(20260)
    out = []
    for m in (1, 2, 3, 4, 5, 8, 9, 16, 31, 32, 33, 40, 64, 65, 100, 128, 191, 192, 193, 300):
        for _ in range(2):
            k = int(rng.choice([64, 128, 192, 256, 384, 512, 1000, 1024, 1032, 2048, 2304]))
            n = int(rng.choice([1, 7, 64, 100, 128, 255, 256, 520, 1024, 2049]))
            out.append((m, k, n))
    # enough 128 x 128 tiles for the widened-weights product, and one short of it
    out += [(256, 512, 128 * 128), (256, 512, 128 * 127), (192, 256, 128 * 170)]
    # two rows on both sides of 32 column groups per pair of compute units; 9 to 32 rows where 16, 32 and 64 columns per
    # workgroup are the plan, and 17 to 32 where the tile kernel is; float32 rows on the three-plane path and off it
    out += [(2, 2048, 8192), (2, 2048, 8176), (9, 2048, 4096), (12, 2048, 8200), (16, 2304, 14336), (24, 4096, 2048), (24, 7168, 1024),
            (32, 2048, 6400), (3, 1024, 2048), (4, 4096, 1024), (8, 2048, 4100), (16, 1024, 8192)]
    return out


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("m,k,n", _q8_shapes())
def test_qmm8_planner(dtype, m, k, n):
    import _dev
    if dtype != torch.bfloat16 and m * n * k > 1 << 27:
        pytest.skip("large case: bfloat16 only")
    a, b, s = int8_case(dtype, m, k, n)
    check_q8(_dev.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s)), a, b, s, dtype)


def _q4_shapes():
    rng = np.random.default_rng(20261)
    out = []
    for m in (1, 2, 3, 4, 5, 15, 16, 17, 32, 48, 63, 64, 65, 97, 160):
        for _ in range(2):
            bs = int(rng.choice([32, 64, 128, 256, 0]))
            k = int(rng.choice([256, 512, 768, 1024, 2048])) if bs else int(rng.choice([96, 160, 1000, 1056, 2048]))
            n = int(rng.choice([1, 5, 16, 33, 100, 256, 700]))
            out.append((m, k, n, bs or k, bool(rng.integers(2))))
    # row tiles x column tiles on both sides of 2048 / 2560 (a wave per tile from there), and of the wave-tile sizes
    out += [(512, 128, 1024, 32, True), (512, 128, 1008, 32, False), (640, 128, 1024, 32, True), (640, 128, 1008, 32, False), (640, 96, 1024, 96, False), (1280, 64, 1024, 64, True), (2560, 256, 1030, 128, False),
            (650, 96, 1024, 96, True), (1290, 64, 2048, 64, False)]
    return out


@pytest.mark.parametrize("m,k,n,bs,bias", _q4_shapes())
def test_qmm4_planner(m, k, n, bs, bias):
    import _dev
    from torch_vulkan_amd import abi
    w, sc, bvec = int4_weights(n, k, bs, seed=11, bias=bias)
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, bvec, bs, k, n).numpy()
    for dtype in (torch.float32, torch.bfloat16):
        if dtype == torch.bfloat16 and bs != k:
            continue
        x = int4_rows(m, k, dtype)
        want = oracle.q4_matmul(bits(x), ODT[dtype], packed, bs, k, n)
        if not abi.lib().vkt_qmm4c_bytes(n, k, bs):
            assert np.array_equal(_dev.q4_reference_layout(bits(x), ODT[dtype], packed, bs, k, n), want)
            continue
        for layout in (0, 1):
            cw = _dev.CompactWeights(packed, bs, k, n, layout=layout)
            assert np.array_equal(_dev.q4_compact(bits(x), ODT[dtype], cw, fused=True), want), (layout, dtype)
