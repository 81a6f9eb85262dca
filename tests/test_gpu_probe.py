"""The calibration kernels behind bench.py's ceilings are reachable by name through vkt_dispatch: their launchers
must refuse arguments that would make them read or write outside the buffers the header describes."""
import numpy as np
import pytest

from torch_vulkan_amd import abi

pytestmark = pytest.mark.gpu


def test_probe_read_geometry_2_takes_whole_tiles_and_rounds():
    src, dst = abi.Buffer(4096), abi.Buffer(256)
    for n, k in ((8, 64), (16, 64), (8, 4096), (24, 8192)):
        with pytest.raises(abi.VktError, match="GEOMETRY 2"):
            abi.dispatch("probe_read", [2], abi.ProbeParams(src=src.address, dst=dst.address, n=n, k=k))
    # a whole tile and round: the side-car's size is what is read
    nbytes = abi.lib().vkt_qmm4c_bytes(16, 4096, 32)
    assert nbytes >= 16 * 4096 // 2 + 16 * (4096 // 32) * 4
    side = abi.Buffer(nbytes)
    abi.check(abi.lib().vkt_fill(side.address, 1, nbytes))
    abi.dispatch("probe_read", [2], abi.ProbeParams(src=side.address, dst=dst.address, n=16, k=4096))
    with pytest.raises(abi.VktError, match="multiple of 16"):
        abi.dispatch("probe_read", [0], abi.ProbeParams(src=src.address, dst=dst.address, n=4, k=24))
    abi.synchronize()


def test_probe_mfma_destination():
    dst = abi.Buffer(256)
    with pytest.raises(abi.VktError, match="8-byte aligned"):
        abi.dispatch("probe_mfma_f8", [0], abi.ProbeParams(dst=dst.address + 4, iters=4))
    abi.check(abi.lib().vkt_fill(dst.address, 0, 256))
    abi.dispatch("probe_mfma_f8", [0], abi.ProbeParams(dst=dst.address, iters=16))
    cycles, ticks = (int(v) for v in dst.to_numpy(np.uint64, (32,))[8:10])
    assert cycles > 0 and ticks >= 0
