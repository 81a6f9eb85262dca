"""Writes the frozen fixtures q4.npz, q8.npz, f8.npz next to this file.

The reference keeps no golden files for the quantized-matmul path: its tests compute every
expectation live from PyTorch's CPU kernels (tests/python/test_quant.py).  This script does
the same once, with the installed torch (CPU ops only; nothing from the reference is
imported or run), on the reference's parametrisations and seeds, so that the expected
outputs are frozen data.  Run: python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from _util import ODT, bits, gen  # noqa: E402
from _cases import FLOAT8_OUT, FLOAT8_PAIRS, INT4_SHAPES, INT8_SHAPES, float8_case, int4_rows, int4_weights, int8_case  # noqa: E402


def main():
    torch.set_num_threads(1)
    out = {}
    for i, (m, k, n, bs, bias) in enumerate(INT4_SHAPES):
        if n > 100:  # keep fixtures small: the large-N cases keep 64 output features
            n = 64
        w, sc, bvec = int4_weights(n, k, bs, bias=bias)
        packed = torch._dyn_quant_pack_4bit_weight(w, sc, bvec, bs, k, n)
        out[f"c{i}_packed"] = packed.numpy()
        out[f"c{i}_shape"] = np.array([m, k, n, bs, int(bias)])
        for tag, dtype in (("f32", torch.float32), ("bf16", torch.bfloat16)):
            if dtype == torch.bfloat16 and bs != k:
                continue
            x = int4_rows(m, k, dtype)
            out[f"c{i}_{tag}_x"] = bits(x)
            out[f"c{i}_{tag}_out"] = bits(torch._dyn_quant_matmul_4bit(x, packed, bs, k, n))
    np.savez_compressed(os.path.join(HERE, "q4.npz"), **out)

    out = {}
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        for (m, k, n) in INT8_SHAPES:
            if dtype != torch.float32 and k % 16:
                continue  # the CPU's 16-bit kernels read 16 values of k at a time (test_quant.py:28-31)
            if k == 4096:
                n = 40
            a, b, s = int8_case(dtype, m, k, n)
            key = f"{str(dtype).split('.')[1]}_{m}x{k}x{n}"
            out[key + "_a"], out[key + "_b"], out[key + "_s"] = bits(a), b.numpy(), bits(s)
            out[key + "_odt"] = np.array(ODT[dtype])
            out[key + "_out"] = bits(torch._weight_int8pack_mm(a, b, s))
    np.savez_compressed(os.path.join(HERE, "q8.npz"), **out)

    out = {}
    for fa, fb in FLOAT8_PAIRS:
        for out_dtype in FLOAT8_OUT:
            a, b, sa, sb, bias, sr, _ = float8_case(fa, fb, out_dtype, rowwise=False)
            want = torch._scaled_mm(a, b, sa, sb, bias=bias, out_dtype=out_dtype, scale_result=sr)
            key = f"{ODT[fa]}{ODT[fb]}_{str(out_dtype).split('.')[-1]}"
            out[key + "_a"], out[key + "_bt"] = bits(a), bits(b.t().contiguous())
            out[key + "_sa"], out[key + "_sb"] = sa.numpy().reshape(1), sb.numpy().reshape(1)
            out[key + "_fmt"] = np.array([ODT[fa], ODT[fb], ODT[want.dtype]])
            if bias is not None:
                out[key + "_bias"] = bits(bias)
            if sr is not None:
                out[key + "_sr"] = np.array(2.0, np.float32)
            out[key + "_out"] = bits(want)
    np.savez_compressed(os.path.join(HERE, "f8.npz"), **out)


if __name__ == "__main__":
    main()
