"""Helpers shared by the tests: seeded generators (the reference's tests draw from
torch.Generator().manual_seed(seed), tests/python/test_quant.py:16-17), storage-array
conversions between torch tensors and the numpy bit patterns the oracle and the C ABI
take, and the reference's magnitude-aware tolerance (test_quant.py:36-37,124-126)."""
import numpy as np
import torch

import oracle

ODT = {torch.float32: oracle.F32, torch.float16: oracle.F16, torch.bfloat16: oracle.BF16,
       torch.float8_e4m3fn: oracle.E4M3, torch.float8_e5m2: oracle.E5M2}
EPS = {oracle.F32: 2.0**-23, oracle.F16: 2.0**-10, oracle.BF16: 2.0**-7, oracle.E4M3: 2.0**-3, oracle.E5M2: 2.0**-2}


def gen(seed):
    return torch.Generator().manual_seed(seed)


def bits(t):
    """torch tensor -> numpy storage array (float32 as is, 16-bit floats as uint16,
    float8 as uint8 codes, integers as is).  Keeps strides of 2-D row-strided views."""
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return t.view(torch.uint8).numpy()
    return t.numpy()


def unbits(a, dtype):
    """numpy storage array -> torch tensor of `dtype`."""
    a = np.ascontiguousarray(a)
    if dtype in (torch.float16, torch.bfloat16):
        return torch.from_numpy(a.view(np.int16)).view(dtype)
    if dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        return torch.from_numpy(a).view(dtype)
    return torch.from_numpy(a)


def ref_tol(want_f32, mag, odt):
    """eps * |want| + 2^-20 * mag  (reference tests/python/test_quant.py:36-37)."""
    return EPS[odt] * np.abs(want_f32.astype(np.float64)) + 2.0**-20 * mag


class no_fallback:
    """with no_fallback(tv): ... fails if an op inside ran on the CPU instead of the device (the per-op fallback
    counters of the backend moved), naming the ops.  The reference guards its device tests the same way."""

    def __init__(self, backend):
        self.backend = backend

    def __enter__(self):
        self.start = dict(self.backend.fallback_counts())
        return self

    def __exit__(self, exc_type, exc, tb):
        if exc_type is None:
            moved = sorted(op for op, count in self.backend.fallback_counts().items() if count != self.start.get(op, 0))
            assert not moved, "fell back to the CPU: " + ", ".join(moved)
        return False


def to_device(value, device="vk"):
    """Tensors (also inside tuples, lists and dict values) moved to `device`; everything else as is."""
    if isinstance(value, torch.Tensor):
        return value.to(device)
    if isinstance(value, (tuple, list)):
        return type(value)(to_device(v, device) for v in value)
    if isinstance(value, dict):
        return {k: to_device(v, device) for k, v in value.items()}
    return value
