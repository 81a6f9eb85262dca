#!/usr/bin/env python3
"""Benchmark of the quantized-matmul path on one MI355X, through the C ABI.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--all] [--no-extra] [--no-cpu] [--verbose]

A "step" is one pass of the hot path over one batch of seeded synthetic input: one
`_weight_int8pack_mm` / `_dyn_quant_matmul_4bit` / `_scaled_mm` call's kernels, queued through
vkt_dispatch with every input already resident in HBM.  The headline workload is the
configuration the metric is quoted on: M=1 bf16 int8-weight GEMV at the Llama-3-8B gate/up
shape (K=4096, N=14336).  GEMV workloads rotate through more than 512 MiB of distinct weight
copies so that the figure is HBM bandwidth and not the 256 MB last-level cache.

Prints ONE JSON line.  `value` is algorithmic bytes (or flops) per step / wall time per step
over exactly K timed steps bracketed by device synchronisation; `roofline.achieved` is the
same work / the kernel's average duration from HIP events recorded on the stream the
kernels run on.  `cpu_baseline` is PyTorch's own CPU kernel for the same op on all host cores
(the CPU path the reference quotes its numbers against), `cpu_oracle_port` the scalar C
restatement under oracle/ on one core, both on a bounded sample that `sample` describes.
`extra` carries the other BASELINE configurations, one short entry each (key, value, unit,
frac of the published peak, kernel time, CPU figure), the configurations the targets are
stated on last; `ceilings` what bare loads and a register-only matrix-core loop sustain in
the same run.  --all adds the workloads beside the BASELINE configurations (prefill shapes,
the float8 producer, 16-bit products, strided copies, affine quantisation); --verbose keeps
every entry's full roofline object.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E, published
FP8_PEAK_TFLOPS = 5000.0    # MI355X dense fp8 MFMA, published
BF16_PEAK_TFLOPS = 2500.0   # MI355X dense bf16 / fp16 MFMA, published
INT8_PEAK_TOPS = 5000.0     # MI355X dense int8 MFMA, published


def _abi():
    from torch_vulkan_amd import abi
    return abi


class Launch:
    """One prebuilt vkt_dispatch call (no per-call Python allocation in the timed loop)."""

    def __init__(self, abi, name, spec, params, batches=1):
        self.fn = abi.lib().vkt_dispatch
        self.batches = batches  # (the grid's third entry: what "gemmcm_*" takes its batch count from)
        self.name = name.encode()
        self.spec = (abi.u32 * max(len(spec), 1))(*spec)
        self.nspec = len(spec)
        self.params = params
        self.ref = ctypes.byref(params)
        self.size = ctypes.sizeof(params)
        self.abi = abi

    def __call__(self):
        if self.fn(self.name, self.spec, self.nspec, self.ref, self.size, 1, 1, self.batches) != 0:
            self.abi.check(-1)


class Timing(tuple):
    """(wall ms per step, event ms per step); .median: the median over five equal parts of the timed loop of the
    event time per step (the whole loop where it has fewer than 10 steps)."""
    median = None


_DELAY = {}


def queue_delay(abi, microseconds):
    """Queues the one-wave kernel that waits `microseconds` ("probe_delay"): what follows it on the stream is queued by
    the host while the device waits, so the device then runs it back to back."""
    if "launch" not in _DELAY:
        _DELAY["params"] = abi.ProbeParams()
        _DELAY["launch"] = Launch(abi, "probe_delay", [], _DELAY["params"])
    _DELAY["params"].iters = int(min(max(microseconds, 1), 100000))
    _DELAY["launch"]()


def time_steps(abi, step_fns, steps, warmup):
    """Runs step_fns[i % len] for `warmup` untimed and `steps` timed steps: wall time per step between two device
    synchronisations (the host queues a step as soon as the one before is queued).  Then the same `steps` steps once
    more behind a queued delay, with events at five equally spaced marks: the device's own time per step, with every
    launch already in its queue (the host needs 3-5 us to queue a launch, as long as the shortest kernels here run)."""
    n = len(step_fns)
    seq = [step_fns[i % n] for i in range(max(steps, warmup))]
    for f in seq[:warmup]:
        f()
    abi.synchronize()
    t0 = time.perf_counter()
    for f in seq[:steps]:
        f()
    abi.synchronize()
    t1 = time.perf_counter()
    parts = 5 if steps >= 10 else 1
    marks = [steps * j // parts for j in range(parts + 1)]
    events = [abi.Event() for _ in marks]
    queue_delay(abi, 8 * steps + 200)
    events[0].record()
    at = 1
    for i, f in enumerate(seq[:steps]):
        f()
        if i + 1 == marks[at]:
            events[at].record()
            at += 1
    abi.synchronize()
    t = Timing(((t1 - t0) * 1e3 / steps, events[0].elapsed_ms(events[-1]) / steps))
    per = sorted(events[j].elapsed_ms(events[j + 1]) / (marks[j + 1] - marks[j]) for j in range(parts))
    t.median = per[len(per) // 2]
    return t


def timed(abi, fns, steps, warmup, resident=True):
    """Timing fields of a workload result: the rotation over distinct weight copies (HBM), and where there is a
    rotation also the same launch on one copy over and over (cache resident, labelled so)."""
    t = time_steps(abi, fns, steps, warmup)
    out = dict(wall_ms=t[0], event_ms=t[1], event_ms_median=t.median, copies=len(fns))
    if len(fns) > 1 and resident:
        out["cache_resident_ms"] = time_steps(abi, fns[:1], steps, warmup)[1]
    return out


def rotation(nbytes, floor_mib=512):
    return max(2, int(floor_mib * (1 << 20) // max(nbytes, 1)) + 1)


# ------------------------------------------------------------------ workloads
def wl_q8(abi, m, k, n, dtype, steps, warmup, seed=1020, prefill=False, variant=0):
    """_weight_int8pack_mm: x ~N(0,1) [m,k]; w int8 uniform [n,k]; scales ~U(0.005,0.02) [n].  prefill: many rows,
    priced against the matrix cores' bf16 rate (the weights are widened once, then one tile-kernel product)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    tdt = {abi.F32: torch.float32, abi.BF16: torch.bfloat16, abi.F16: torch.float16}[dtype]
    x = torch.randn(m, k, generator=g).to(tdt)
    w = torch.randint(-128, 128, (n, k), dtype=torch.int8, generator=g)
    s = torch.empty(n).uniform_(0.005, 0.02, generator=g).to(tdt)
    item = x.element_size()
    as_np = (lambda t: t.numpy()) if dtype == abi.F32 else (lambda t: t.view(torch.int16).numpy())
    dx, ds = abi.Buffer.from_numpy(as_np(x)), abi.Buffer.from_numpy(as_np(s))
    copies = [abi.Buffer.from_numpy(w.numpy())]
    for _ in range(rotation(n * k) - 1):
        b = abi.Buffer(n * k)
        abi.check(abi.lib().vkt_copy_on_device(b.address, copies[0].address, n * k))
        copies.append(b)
    out = abi.Buffer(m * n * item)
    fns = [Launch(abi, "qmm8_" + abi.SUFFIX[dtype], [0, variant],
                  abi.Q8Params(a=dx.address, b=c.address, scales=ds.address, c=out.address, m=m, n=n, k=k, a_sm=k,
                               a_sk=1)) for c in copies]
    work = n * k + item * (m * k + n + m * n)  # weights once + activations + scales + output
    keep = (x, w, s)
    if prefill:
        return dict(kind="mfma", peak=BF16_PEAK_TFLOPS, metric="int8-weight prefill TFLOP/s (% of bf16 MFMA peak)", work=2 * m * n * k,
                    bytes=work, inputs=None, name=f"_weight_int8pack_mm {abi.SUFFIX[dtype]} M={m} K={k} N={n} (prefill)",
                    **timed(abi, fns, steps, max(warmup, len(fns)), resident=False))
    return dict(kind="hbm", work=work, flops=2 * m * n * k, inputs=keep,
                name=f"_weight_int8pack_mm {abi.SUFFIX[dtype]} M={m} K={k} N={n}" + (f" (variant {variant:#x})" if variant else ""),
                **timed(abi, fns, steps, warmup))


def wl_q4(abi, m, k, n, bs, steps, warmup, seed=1030, prefill=False, phase=2):
    """_dyn_quant_matmul_4bit on the compact side-car: up to 4 rows the streaming layout with
    row quantisation fused into the launch, above that the matrix-core layout (two launches)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    w4 = torch.randint(0, 16, (n, k), dtype=torch.uint8, generator=g)
    wbytes = (w4[:, 0::2] + 16 * w4[:, 1::2]).contiguous()
    sc = torch.empty(n, k // bs).uniform_(0.01, 0.05, generator=g)
    bias = torch.randn(n, generator=g) * 0.1
    x = torch.randn(m, k, generator=g)
    packed = torch._dyn_quant_pack_4bit_weight(wbytes, sc, bias, bs, k, n)
    L = abi.lib()
    cbytes = L.vkt_qmm4c_bytes(n, k, bs)
    dp = abi.Buffer.from_numpy(packed.numpy())
    first = abi.Buffer(cbytes)
    layout = 1 if m > 3 else 0
    abi.dispatch("qmm4c_pack", [layout], abi.Q4PackParams(packed=dp.address, compact=first.address, n=n, k=k, bs=bs,
                                                    has_bias=1))
    abi.synchronize()
    dp.free()
    copies = [first]
    for _ in range(rotation(cbytes) - 1):
        b = abi.Buffer(cbytes)
        abi.check(L.vkt_copy_on_device(b.address, first.address, cbytes))
        copies.append(b)
    dx = abi.Buffer.from_numpy(x.numpy())
    dq, dr = abi.Buffer(L.vkt_qmm4c_q_bytes(m, k)), abi.Buffer(m * 8)
    out = abi.Buffer(m * n * 4)
    fns = []
    for c in copies:
        p = abi.Q4CParams(inp=dx.address, q=dq.address, rows=dr.address, compact=c.address, out=out.address, m=m, n=n,
                          k=k, bs=bs, has_bias=1)
        fns.append(Launch(abi, "qmm4c_f32", [phase, 1, layout], p))  # row quantisation + product
    work = n * k // 2 + 4 * n * (k // bs) + 4 * n + 4 * m * k + 4 * m * n
    if prefill:  # many rows: the matrix cores' int8 rate is the published bound
        return dict(kind="mfma", peak=INT8_PEAK_TOPS, metric="int4-weight prefill TOP/s (% of int8 MFMA peak)", work=2 * m * n * k,
                    bytes=work, inputs=None, name=f"_dyn_quant_matmul_4bit f32 M={m} K={k} N={n} bs={bs} (prefill)",
                    **timed(abi, fns, steps, max(warmup, len(fns)), resident=False))
    return dict(kind="hbm", work=work, flops=2 * m * n * k, inputs=(x, packed),
                name=f"_dyn_quant_matmul_4bit f32 M={m} K={k} N={n} bs={bs} (compact side-car)",
                shape=(n, bs), reference_layout_bytes=int(packed.numel()) * 4 + 4 * m * k + 4 * m * n, **timed(abi, fns, steps, warmup))


def wl_fp8(abi, m, k, n, rowwise, steps, warmup, seed=1040, zero_operands=False, variant=0, decode=False, f32_out=False):
    """_scaled_mm e4m3fn x e4m3fn -> bf16; A row-major, B column-major.  zero_operands: the same
    launch on all-zero matrices: the matrix cores' sustained rate depends on how many operand
    bits toggle (the part is power limited), and this is the data-independent end of that range.
    decode: few rows; the product is the weight stream, priced against HBM, over copies of the weights taken in
    turn (one copy would stay in the last-level cache)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).clamp(-448, 448).to(torch.float8_e4m3fn)
    bt = torch.randn(n, k, generator=g).clamp(-448, 448).to(torch.float8_e4m3fn)
    if zero_operands:
        a, bt = torch.zeros_like(a), torch.zeros_like(bt)
    if rowwise:
        sa = torch.empty(m).uniform_(0.5, 2, generator=g)
        sb = torch.empty(n).uniform_(0.5, 2, generator=g)
    else:
        sa, sb = torch.tensor([0.5]), torch.tensor([0.5])
    da, db = abi.Buffer.from_numpy(a.view(torch.uint8).numpy()), abi.Buffer.from_numpy(bt.view(torch.uint8).numpy())
    dsa, dsb = abi.Buffer.from_numpy(sa.numpy()), abi.Buffer.from_numpy(sb.numpy())
    out = abi.Buffer(m * n * (4 if f32_out else 2))
    p = abi.F8Params(a=da.address, b=db.address, scale_a=dsa.address, scale_b=dsb.address, out=out.address, m=m, n=n,
                     k=k, lda=k, ldb=k, ldo=n, fmt_a=abi.E4M3, fmt_b=abi.E4M3, out_dtype=abi.F32 if f32_out else abi.BF16, rowwise=int(rowwise))
    if decode:
        copies = [db]
        for _ in range(rotation(n * k) - 1):
            b = abi.Buffer(n * k)
            abi.check(abi.lib().vkt_copy_on_device(b.address, db.address, n * k))
            copies.append(b)
        fns = []
        for c in copies:
            q = abi.F8Params(a=da.address, b=c.address, scale_a=dsa.address, scale_b=dsb.address, out=out.address, m=m, n=n,
                             k=k, lda=k, ldb=k, ldo=n, fmt_a=abi.E4M3, fmt_b=abi.E4M3, out_dtype=abi.BF16, rowwise=int(rowwise))
            fns.append(Launch(abi, "fp8mm", [variant], q))
        return dict(kind="hbm", work=n * k + m * k + 2 * m * n + 4 * (m + n if rowwise else 2), flops=2 * m * n * k, inputs=None,
                    name=f"_scaled_mm e4m3fn {'rowwise' if rowwise else 'per-tensor'} M={m} K={k} N={n} -> bf16 (decode)",
                    **timed(abi, fns, steps, warmup))
    fns = [Launch(abi, "fp8mm", [variant], p)]
    tm = time_steps(abi, fns, steps, warmup)
    return dict(kind="mfma", work=2 * m * n * k, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median, bytes=m * k + n * k + 2 * m * n,
                inputs=(a, bt, sa, sb), copies=1,
                name=f"_scaled_mm e4m3fn {'rowwise' if rowwise else 'per-tensor'} M={m} K={k} N={n} -> bf16"
                     + (" (all-zero operands)" if zero_operands else ""))


def wl_gemm16(abi, m, k, n, steps, warmup, seed=1090, layout="nt", decode=False, variant=0):
    """bfloat16 mm, x [m,k] @ w -> [m,n]: the unquantised product next to the path.  layout "nt": w stored
    [n,k] (x @ w.T, the Linear layout); "nn": w stored [k,n] (x @ w); "tn": x stored [k,m] as well (x.t() @ w)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    a, w = torch.randn(m, k, generator=g).bfloat16(), torch.randn(n, k, generator=g).bfloat16()
    da, dw = abi.Buffer.from_numpy(a.view(torch.int16).numpy()), abi.Buffer.from_numpy(w.view(torch.int16).numpy())
    out = abi.Buffer(m * n * 2)
    p = abi.GemmParams(a=da.address, b=dw.address, c=out.address, m=m, n=n, k=k, a_sm=k, a_sk=1, b_sk=1, b_sn=k, c_sm=n,
                       c_sn=1, alpha=int(np.float32(1).view(np.uint32)))
    if layout in ("nn", "tn"):  # (the same bytes read as the other layout: the values do not matter to the timing)
        p.b_sk, p.b_sn = n, 1
    if layout == "tn":
        p.a_sm, p.a_sk = 1, m
    if decode:  # few rows: the product is the weight stream, over copies of the weights taken in turn, priced against HBM
        copies = [dw]
        for _ in range(rotation(2 * n * k) - 1):
            b = abi.Buffer(2 * n * k)
            abi.check(abi.lib().vkt_copy_on_device(b.address, dw.address, 2 * n * k))
            copies.append(b)
        fns = []
        for c in copies:
            q = abi.GemmParams.from_buffer_copy(p)
            q.b = c.address
            fns.append(Launch(abi, "gemmcm_bf16", [0, 0, 0, variant], q))
        return dict(kind="hbm", work=2 * (n * k + m * k + m * n), flops=2 * m * n * k, inputs=None,
                    name=f"mm bf16 M={m} K={k} N={n} ({layout}, decode)", **timed(abi, fns, steps, warmup))
    tm = time_steps(abi, [Launch(abi, "gemmcm_bf16", [0, 0, 0, variant], p)], steps, warmup)
    return dict(kind="mfma", peak=BF16_PEAK_TFLOPS, metric="bf16 mm TFLOP/s (% of MFMA peak)", work=2 * m * n * k, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median,
                bytes=2 * (m * k + n * k + m * n), inputs=None, copies=1, name=f"mm bf16 M={m} K={k} N={n} ({layout}: " + {"nt": "x @ w.T, the Linear layout", "nn": "x @ w", "tn": "x.T @ w"}[layout] + ")")


def wl_bmm16(abi, batches, m, k, n, steps, warmup, layout, seed=1180):
    """A batch of few-row bfloat16 products, the shape of attention at decode: layout "nt": w stored [batches, n, k]
    (q @ k.T: k the head dimension, n the cached positions); "nn": w stored [batches, k, n] (p @ v).  Priced against HBM
    (the cached keys or values, 0.25 to 1 GiB here, do not fit the caches)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(batches * m * k, generator=g).bfloat16()
    w = torch.randn(1 << 20, generator=g).bfloat16().repeat(batches * n * k >> 20)  # (the values do not matter to the timing)
    da, dw = abi.Buffer.from_numpy(a.view(torch.int16).numpy()), abi.Buffer.from_numpy(w.view(torch.int16).numpy())
    out = abi.Buffer(batches * m * n * 2)
    p = abi.GemmParams(a=da.address, b=dw.address, c=out.address, m=m, n=n, k=k, a_sb=m * k, a_sm=k, a_sk=1, b_sb=n * k, c_sb=m * n, c_sm=n,
                       c_sn=1, alpha=int(np.float32(1).view(np.uint32)))
    p.b_sk, p.b_sn = (1, k) if layout == "nt" else (n, 1)
    fns = [Launch(abi, "gemmcm_bf16", [0, 0, 0, 0], p, batches=batches)]
    return dict(kind="hbm", work=2 * batches * (n * k + m * k + m * n), flops=2 * batches * m * n * k, inputs=None,
                name=f"bmm bf16 {batches} x (M={m} K={k} N={n}) ({layout}, decode)", **timed(abi, fns, steps, warmup))


def wl_cast(abi, n, steps, warmup, seed=1070):
    """bfloat16 -> e4m3fn elementwise cast of n values (the float8 step in front of _scaled_mm)."""
    import torch
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(1 << 20, generator=g).bfloat16().repeat(n >> 20)
    dx = abi.Buffer.from_numpy(x.view(torch.int16).numpy())
    out = abi.Buffer(n)
    p = abi.CastParams(src=dx.address, dst=out.address, n=n, src_dtype=abi.BF16, dst_dtype=abi.E4M3)
    tm = time_steps(abi, [Launch(abi, "cast_fp8", [], p)], steps, warmup)
    return dict(kind="hbm", work=3 * n, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median, flops=0, inputs=None, copies=1,
                name=f"cast bf16 -> e4m3fn, {n >> 20} Mi values")


def wl_quant(abi, m, k, steps, warmup, seed=1080):
    """The rowwise float8 producer: bfloat16 [m,k] -> e4m3fn [m,k] + float32 scales [m]."""
    import torch
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g).bfloat16()
    dx = abi.Buffer.from_numpy(x.view(torch.int16).numpy())
    out, scales = abi.Buffer(m * k), abi.Buffer(m * 4)
    p = abi.F8QuantParams(src=dx.address, dst=out.address, scale=scales.address, m=m, k=k, lds=k, ldd=k,
                          src_dtype=abi.BF16, dst_fmt=abi.E4M3)
    tm = time_steps(abi, [Launch(abi, "fp8_quant", [1], p)], steps, warmup)
    return dict(kind="hbm", work=3 * m * k + 4 * m, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median, flops=0, inputs=None, copies=1,
                name=f"fp8_quant rowwise bf16 -> e4m3fn M={m} K={k}")


def wl_move(abi, kind, steps, warmup, rows=16384, cols=16384):
    """Strided same-size copies of bfloat16 [rows, cols]: "transpose" (x.t().contiguous()) or "rows"
    (x[::2].contiguous()): bytes read + bytes written per launch."""
    src, item = abi.Buffer(rows * cols * 2), 2
    abi.check(abi.lib().vkt_fill(src.address, 1, rows * cols * 2))
    p = abi.StridedParams(a=src.address, ndim=2)
    if kind == "transpose":
        out = abi.Buffer(rows * cols * 2)
        p.n, sizes, so, sa, name, work = rows * cols, (rows, cols), (1, rows), (cols, 1), "move_b2", 2 * rows * cols * item
    else:
        out = abi.Buffer(rows * cols)
        p.n, sizes, so, sa, name, work = rows // 2 * cols, (cols, rows // 2), (1, cols), (1, 2 * cols), "move_b2", rows * cols * item
    p.out = out.address
    for d in range(4):
        p.size[d], p.so[d], p.sa[d] = (sizes[d], so[d], sa[d]) if d < 2 else (1, 0, 0)
    tm = time_steps(abi, [Launch(abi, name, [abi.MOVE_COPY], p)], steps, warmup)
    label = {"transpose": "x.t().contiguous()", "rows": "x[::2].contiguous()"}[kind]
    return dict(kind="hbm", metric="strided copy GB/s (% of HBM peak)", work=work, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median, flops=0, inputs=None,
                copies=1, name=f"{name} {label}, bfloat16 [{rows}, {cols}]")


def wl_affine(abi, kind, n, steps, warmup, seed=1100):
    """Per-tensor affine quantisation of n float32 values: "quantize" (-> quint8), "dequantize" (quint8 -> float32),
    "fake_quant" (-> float32 + mask bytes): bytes read + written per launch."""
    import torch
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(1 << 20, generator=g) * 20).repeat(n >> 20)
    scale_bits = int(np.float32(0.1).view(np.uint32))
    if kind == "quantize":
        src, dst = abi.Buffer.from_numpy(x.numpy()), abi.Buffer(n)
        p, name, spec, work = abi.QuantParams(src=src.address, dst=dst.address, n=n, scale_bits=scale_bits, zero_point=5), "quantize_affine", [0], 5 * n
    elif kind == "dequantize":
        src, dst = abi.Buffer.from_numpy(torch.quantize_per_tensor(x, 0.1, 5, torch.quint8).int_repr().numpy()), abi.Buffer(4 * n)
        p, name, spec, work = abi.QuantParams(src=src.address, dst=dst.address, n=n, scale_bits=scale_bits, zero_point=5), "dequantize_affine", [0], 5 * n
    else:
        src, dst, mask = abi.Buffer.from_numpy(x.numpy()), abi.Buffer(4 * n), abi.Buffer(n)
        p = abi.QuantParams(src=src.address, dst=dst.address, mask=mask.address, n=n, scale_bits=scale_bits, zero_point=5, qmin=0,
                            qmax=255, dtype=abi.F32)
        name, spec, work = "fake_quant", [0, 0], 9 * n
    tm = time_steps(abi, [Launch(abi, name, spec, p)], steps, warmup)
    return dict(kind="hbm", metric="affine quantisation GB/s (% of HBM peak)", work=work, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median, flops=0,
                inputs=None, copies=1, name=f"{name} float32 / quint8 per tensor, {n >> 20} Mi values")


def wl_copy(abi, nbytes, steps, warmup):
    """A plain device-to-device copy of known size (calibrates the HBM traffic counters)."""
    src, dst = abi.Buffer(nbytes), abi.Buffer(nbytes)
    abi.check(abi.lib().vkt_fill(src.address, 1, nbytes))
    L = abi.lib()

    def step():
        abi.check(L.vkt_copy_on_device(dst.address, src.address, nbytes))
    tm = time_steps(abi, [step], steps, warmup)
    return dict(kind="hbm", work=2 * nbytes, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median, flops=0, inputs=None, copies=1,
                name=f"device copy of {nbytes >> 20} MiB (read + write)")


def wl_probe_read(abi, n, k, geometry, steps, warmup, label):
    """Bare 16-byte non-temporal loads of n * k bytes in a product kernel's launch geometry (kernel "probe_read"),
    rotated through more than 512 MiB like the product itself: what that geometry can stream at all."""
    nbytes = n * k if geometry != 2 else abi.lib().vkt_qmm4c_bytes(n, k, 32)
    sink = abi.Buffer(256)
    copies = [abi.Buffer(nbytes) for _ in range(rotation(nbytes))]
    for c in copies:
        abi.check(abi.lib().vkt_fill(c.address, 1, nbytes))
    fns = [Launch(abi, "probe_read", [geometry], abi.ProbeParams(src=c.address, dst=sink.address, n=n, k=k)) for c in copies]
    work = n * k if geometry != 2 else n * k // 2 + 4 * n * (k // 32)
    tm = time_steps(abi, fns, steps, warmup)
    return dict(kind="hbm", metric="bare read GB/s (% of HBM peak)", work=work, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median,
                flops=0, inputs=None, copies=len(fns), name=f"probe_read {label}: {work} bytes")


def wl_probe_mfma(abi, operands, steps, warmup, iters=4096):
    """A register-only loop of fp8 32x32x64 matrix-core instructions on every compute unit (kernel "probe_mfma_f8"):
    operands 0 all zero, 1 random bits held in registers, 2 fresh bits for every instruction."""
    sink = abi.Buffer(256)
    info = abi.device_info()
    fns = [Launch(abi, "probe_mfma_f8", [operands], abi.ProbeParams(dst=sink.address, iters=iters))]
    tm = time_steps(abi, fns, steps, warmup)
    work = info.compute_units * 4 * iters * 4 * 2 * 32 * 32 * 64
    import numpy as np
    cycles, ticks = (int(v) for v in sink.to_numpy(np.uint64, (32,))[8:10])
    label = {0: "all-zero operands", 1: "random operands held in registers", 2: "fresh random operands per instruction"}[operands]
    return dict(kind="mfma", metric="fp8 MFMA loop TFLOP/s (% of MFMA peak)", work=work, wall_ms=tm[0], event_ms=tm[1], event_ms_median=tm.median,
                bytes=0, inputs=None, copies=1, clock_ghz=round(cycles / (10.0 * ticks), 3) if ticks else None,
                name=f"probe_mfma_f8, {label}")


# The BASELINE.json configurations.  Order of the extras in the output: the configurations the targets are stated on
# come last (a stored tail of the line keeps them).
BASELINE = {
    # configs[1]: the configuration the metric is quoted on
    "c2_m1_k4096_n14336": lambda abi, s, w: wl_q8(abi, 1, 4096, 14336, abi.BF16, s, w),
    "c2_m8_k4096_n14336": lambda abi, s, w: wl_q8(abi, 8, 4096, 14336, abi.BF16, s, w),
    "c2_m8_k14336_n4096": lambda abi, s, w: wl_q8(abi, 8, 14336, 4096, abi.BF16, s, w),
    "c2_m64_k4096_n14336": lambda abi, s, w: wl_q8(abi, 64, 4096, 14336, abi.BF16, s, w),
    "c2_m64_k14336_n4096": lambda abi, s, w: wl_q8(abi, 64, 14336, 4096, abi.BF16, s, w),
    "c3_int4_m32": lambda abi, s, w: wl_q4(abi, 32, 4096, 11008, 32, max(s // 4, 5), w),
    "c2_m1_k14336_n4096": lambda abi, s, w: wl_q8(abi, 1, 14336, 4096, abi.BF16, s, w),
    "c5_fp8_rowwise_70b": lambda abi, s, w: wl_fp8(abi, 4096, 8192, 28672, True, max(s // 2, 30), max(w, 5), seed=1050),
    "c1_f32_m1_k4096_n4096": lambda abi, s, w: wl_q8(abi, 1, 4096, 4096, abi.F32, s, w, seed=1010),
    "c3_int4_m1": lambda abi, s, w: wl_q4(abi, 1, 4096, 11008, 32, s, w),
    "c4_fp8_8192": lambda abi, s, w: wl_fp8(abi, 8192, 8192, 8192, False, max(s // 2, 30), max(w, 5)),
}
# The same operators at decode off the BASELINE grid (in `extra` of the default run, after the BASELINE configurations):
# few rows of _scaled_mm, float32 rows and 16 rows of _weight_int8pack_mm, and the unquantised Linear beside them.
DECODE = {
    "f8_decode_m1_k8192_n8192": lambda abi, s, w: wl_fp8(abi, 1, 8192, 8192, True, s, w, decode=True),
    "f8_decode_m16_k8192_n28672": lambda abi, s, w: wl_fp8(abi, 16, 8192, 28672, True, s, w, decode=True),
    "q8_f32_m8_k4096_n14336": lambda abi, s, w: wl_q8(abi, 8, 4096, 14336, abi.F32, s, w, seed=1150),
    "q8_m16_k8192_n8192": lambda abi, s, w: wl_q8(abi, 16, 8192, 8192, abi.BF16, s, w, seed=1160),
    "mm_bf16_decode_m8_k8192_n8192": lambda abi, s, w: wl_gemm16(abi, 8, 8192, 8192, s, w, decode=True),
    # (128 rows against 64 tiles of 128 x 128: the tile kernel with K in slices over workgroups)
    "f8_decode_m128_k8192_n8192": lambda abi, s, w: wl_fp8(abi, 128, 8192, 8192, True, s, w, decode=True),
    # (attention at decode, 32 sequences x 32 heads of 128 values, 4096 cached positions: p @ v)
    "bmm_bf16_decode_pv_b1024_k4096_n128": lambda abi, s, w: wl_bmm16(abi, 1024, 1, 4096, 128, max(s // 4, 10), w, "nn"),
}
# Beside the BASELINE configurations (--all, or by name): many rows of the same operators, the steps either side of
# the path, the planner off the Llama grid, config 4's launch on all-zero operands.
OTHER = {
    "c2_prefill_m4096_k4096_n14336": lambda abi, s, w: wl_q8(abi, 4096, 4096, 14336, abi.BF16, max(s // 20, 5), max(w // 4, 3), prefill=True),
    "c3_int4_prefill_m2048": lambda abi, s, w: wl_q4(abi, 2048, 4096, 11008, 32, max(s // 10, 5), w, prefill=True),
    "q8_f32_m64_k4096_n4096": lambda abi, s, w: wl_q8(abi, 64, 4096, 4096, abi.F32, s, w, seed=1010),
    "q8_f32_m64_k4096_n4096_row_kernels": lambda abi, s, w: wl_q8(abi, 64, 4096, 4096, abi.F32, max(s // 4, 5), w, seed=1010, variant=1 << 22),
    "q8_f32_m64_k14336_n4096": lambda abi, s, w: wl_q8(abi, 64, 14336, 4096, abi.F32, s, w),
    "q8_m1_k5120_n13824": lambda abi, s, w: wl_q8(abi, 1, 5120, 13824, abi.BF16, s, w, seed=1110),
    "q8_m1_k8192_n8192": lambda abi, s, w: wl_q8(abi, 1, 8192, 8192, abi.BF16, s, w, seed=1120),
    "q8_m8_k5120_n13824": lambda abi, s, w: wl_q8(abi, 8, 5120, 13824, abi.BF16, s, w, seed=1110),
    "q8_m64_k8192_n8192": lambda abi, s, w: wl_q8(abi, 64, 8192, 8192, abi.BF16, s, w, seed=1120),
    "q8_m8_k4096_n128256": lambda abi, s, w: wl_q8(abi, 8, 4096, 128256, abi.BF16, max(s // 4, 10), w, seed=1130),  # (a vocabulary-sized projection)
    "q8_m8_k2048_n128256": lambda abi, s, w: wl_q8(abi, 8, 2048, 128256, abi.BF16, max(s // 4, 10), w, seed=1140),  # (the same of a smaller model)
    "f8_cast_bf16_e4m3_256mi": lambda abi, s, w: wl_cast(abi, 1 << 28, max(s // 10, 5), max(w // 4, 3)),
    "f8_quant_rowwise_bf16_16384x16384": lambda abi, s, w: wl_quant(abi, 16384, 16384, max(s // 10, 5), max(w // 4, 3)),
    "mm_bf16_8192": lambda abi, s, w: wl_gemm16(abi, 8192, 8192, 8192, max(s // 10, 5), max(w // 4, 3)),
    "mm_bf16_8192_nn": lambda abi, s, w: wl_gemm16(abi, 8192, 8192, 8192, max(s // 10, 5), max(w // 4, 3), layout="nn"),
    "mm_bf16_8192_tn": lambda abi, s, w: wl_gemm16(abi, 8192, 8192, 8192, max(s // 10, 5), max(w // 4, 3), layout="tn"),
    "move_transpose_bf16_16384": lambda abi, s, w: wl_move(abi, "transpose", max(s // 10, 5), max(w // 4, 3)),
    "move_rows_bf16_16384": lambda abi, s, w: wl_move(abi, "rows", max(s // 10, 5), max(w // 4, 3)),
    "affine_quantize_256mi": lambda abi, s, w: wl_affine(abi, "quantize", 1 << 28, max(s // 10, 5), max(w // 4, 3)),
    "affine_dequantize_256mi": lambda abi, s, w: wl_affine(abi, "dequantize", 1 << 28, max(s // 10, 5), max(w // 4, 3)),
    "affine_fake_quant_256mi": lambda abi, s, w: wl_affine(abi, "fake_quant", 1 << 28, max(s // 10, 5), max(w // 4, 3)),
    "f8_decode_m64_k8192_n8192": lambda abi, s, w: wl_fp8(abi, 64, 8192, 8192, True, s, w, decode=True),
    # (few columns against long rows, the key / value projections of a model with grouped heads: K in slices over workgroups)
    "f8_decode_m64_k28672_n1024": lambda abi, s, w: wl_fp8(abi, 64, 28672, 1024, True, s, w, decode=True),
    "mm_bf16_decode_m32_k8192_n2048": lambda abi, s, w: wl_gemm16(abi, 32, 8192, 2048, s, w, decode=True),
    "q8_m8_k8192_n1024": lambda abi, s, w: wl_q8(abi, 8, 8192, 1024, abi.BF16, s, w, seed=1170),
    "mm_bf16_decode_m128_k8192_n8192": lambda abi, s, w: wl_gemm16(abi, 128, 8192, 8192, s, w, decode=True),
    # (attention at decode: q @ k.T)
    "bmm_bf16_decode_qk_b1024_k128_n4096": lambda abi, s, w: wl_bmm16(abi, 1024, 1, 128, 4096, max(s // 4, 10), w, "nt"),
    "mm_bf16_decode_nn_m8_k8192_n8192": lambda abi, s, w: wl_gemm16(abi, 8, 8192, 8192, s, w, decode=True, layout="nn"),  # (weights stored [k, n])
    "c4_fp8_8192_zero_operands": lambda abi, s, w: wl_fp8(abi, 8192, 8192, 8192, False, max(s // 2, 30), max(w, 5), zero_operands=True),
}
# Ceilings measured in the same run (`ceilings` of the output line; also selectable by name): bare 16-byte loads of
# each GEMV configuration's weight bytes in its kernel's launch geometry, a persistent-grid read, a device copy of known
# size (calibrates the traffic counters), and the register-only fp8 matrix-core loop on three kinds of operand bits.
CALIBRATION = {
    "probe_read_c1_16mb": lambda abi, s, w: wl_probe_read(abi, 4096, 4096, 0, s, w, "config 1 (4096 x 4096 int8, GEMV geometry)"),
    "probe_read_c3_28mb": lambda abi, s, w: wl_probe_read(abi, 11008, 4096, 2, s, w, "config 3 (int4 side-car, streaming geometry)"),
    "probe_read_c2_58mb": lambda abi, s, w: wl_probe_read(abi, 14336, 4096, 0, s, w, "config 2 (14336 x 4096 int8, GEMV geometry)"),
    "probe_read_c2_58mb_k14336": lambda abi, s, w: wl_probe_read(abi, 4096, 14336, 1, s, w, "config 2 (4096 x 14336 int8, GEMV geometry)"),
    "probe_read_persistent_58mb": lambda abi, s, w: wl_probe_read(abi, 14336, 4096, 3, s, w, "58 MB, persistent grid"),
    "probe_read_persistent_16mb": lambda abi, s, w: wl_probe_read(abi, 4096, 4096, 3, s, w, "16 MB, persistent grid"),
    "probe_mfma_f8_zero": lambda abi, s, w: wl_probe_mfma(abi, 0, max(s // 10, 5), max(w // 4, 3)),
    "probe_mfma_f8_held": lambda abi, s, w: wl_probe_mfma(abi, 1, max(s // 10, 5), max(w // 4, 3)),
    "probe_mfma_f8_fresh": lambda abi, s, w: wl_probe_mfma(abi, 2, max(s // 10, 5), max(w // 4, 3)),
    "copy_256mib": lambda abi, s, w: wl_copy(abi, 256 << 20, max(s // 4, 5), w),
}
# configurations whose extra entry also carries the op's cost through PyTorch's dispatcher (the headline always does)
DISPATCHER_TOO = ("c3_int4_m1", "c3_int4_m32", "c4_fp8_8192", "c1_f32_m1_k4096_n4096")
WORKLOADS = {**BASELINE, **DECODE, **OTHER}
HEADLINE = "c2_m1_k4096_n14336"


def summarise(r):
    """Throughput and roofline of one workload result."""
    if r["kind"] == "hbm":
        value, unit, peak = r["work"] / r["wall_ms"] / 1e6, "GB/s", HBM_PEAK_GBPS
        achieved = r["work"] / r["event_ms"] / 1e6
    else:
        value, unit, peak = r["work"] / r["wall_ms"] / 1e9, "TFLOP/s", r.get("peak", FP8_PEAK_TFLOPS)
        achieved = r["work"] / r["event_ms"] / 1e9
    roof = dict(bound=r["kind"], achieved=round(achieved, 1), peak=peak, unit=unit, frac=round(achieved / peak, 4),
                traffic=None, algorithmic=r["work"])  # algorithmic: bytes (or operations) per step that `achieved` prices
    if r.get("event_ms_median"):  # the same figure from the median fifth of the timed loop
        roof["achieved_median_of_5"] = round(achieved * r["event_ms"] / r["event_ms_median"], 1)
    if r.get("cache_resident_ms"):  # one weight copy over and over: L2 / Infinity Cache, not HBM (reported, not priced)
        roof["cache_resident"] = dict(achieved=round(achieved * r["event_ms"] / r["cache_resident_ms"], 1), unit=unit,
                                      kernel_ms=round(r["cache_resident_ms"], 5))
    return value, unit, roof


def _median_time(fn, reps, warm=1):
    for _ in range(warm):
        fn()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return sorted(ts)[len(ts) // 2]


def cpu_baselines(abi, name, r, port=False):
    """The CPU beside the GPU figure, on the same seeded inputs: `cpu_baseline` = PyTorch's CPU kernel of the op on all
    host cores (what the reference's own numbers are quoted against), on a bounded sample; port=True adds
    `cpu_oracle_port`, the scalar C restatement on one core."""
    import torch
    out = {}
    cores = torch.get_num_threads()
    if not r.get("inputs"):
        return out
    if name.startswith(("c1", "c2", "q8_")):
        x, w, s = r["inputs"]
        reps = 15 if x.shape[0] <= 8 else 5
        dt = _median_time(lambda: torch._weight_int8pack_mm(x, w, s), reps)
        out["cpu_baseline"] = dict(value=round(r["work"] / dt / 1e9, 3), unit="GB/s", cores=cores, kind="reference",
                                   sample=f"torch._weight_int8pack_mm on CPU tensors (PyTorch's own kernel of the op: the CPU path the reference "
                                          f"is quoted against), full workload, median of {reps} calls, {dt * 1e3:.2f} ms; host has {os.cpu_count()} CPUs")
        if port:
            import oracle
            odt = {torch.float32: oracle.F32, torch.bfloat16: oracle.BF16, torch.float16: oracle.F16}[x.dtype]
            xb = x.numpy() if odt == oracle.F32 else x.view(torch.int16).numpy().view(np.uint16)
            sb = s.numpy() if odt == oracle.F32 else s.view(torch.int16).numpy().view(np.uint16)
            oracle.qmm8(xb, odt, w.numpy()[:64], sb[:64])  # load + warm
            reps, t0 = 0, time.perf_counter()
            while time.perf_counter() - t0 < 3.0 and reps < 100:
                oracle.qmm8(xb, odt, w.numpy(), sb)
                reps += 1
            dt = (time.perf_counter() - t0) / reps
            out["cpu_oracle_port"] = dict(value=round(r["work"] / dt / 1e9, 3), unit="GB/s", cores=1, kind="port",
                                          sample=f"{reps} full passes through oracle/qmm_oracle.c (scalar C restatement), {dt * 1e3:.1f} ms each")
    elif name.startswith("c3"):
        x, packed = r["inputs"]
        m, k = x.shape
        n, bs = r["shape"]
        reps = 3
        dt = _median_time(lambda: torch._dyn_quant_matmul_4bit(x, packed, bs, k, n), reps)
        out["cpu_baseline"] = dict(value=round(r["work"] / dt / 1e9, 3), unit="GB/s", cores=cores, kind="reference",
                                   sample=f"torch._dyn_quant_matmul_4bit on CPU tensors (float32-expanded packed vector), full workload, "
                                          f"median of {reps} calls, {dt * 1e3:.1f} ms; priced on the same algorithmic bytes as the GPU figure")
    elif name.startswith(("c4", "c5")):
        a, bt, sa, sb = r["inputs"]
        m, k = a.shape
        n = bt.shape[0]
        rowwise = sa.numel() > 1
        rows = min(m, 1024)  # a bounded sample: the first rows of A against all of B
        a_s, sa_s = a[:rows], (sa[:rows].reshape(rows, 1) if rowwise else sa)
        sb_s = sb.reshape(1, n) if rowwise else sb

        def closed_form():
            return ((a_s.float() * sa_s) @ (bt.float() * sb_s.reshape(-1, 1) if rowwise else bt.float() * sb_s).t()).bfloat16()
        dt = _median_time(closed_form, 1, warm=0)
        out["cpu_baseline"] = dict(value=round(2.0 * rows * n * k / dt / 1e12, 4), unit="TFLOP/s", cores=cores, kind="reference",
                                   sample=f"the emulated closed form ((A.float()*sa) @ (B.float()*sb)).bfloat16() in PyTorch on the CPU (what the "
                                          f"reference's composite computes; torch's CPU _scaled_mm kernel " + ("rejects rowwise scales" if rowwise else "is a scalar loop, timed below") +
                                          f"), first {rows} of {m} rows of A against all of B, one call, {dt:.2f} s")
        if not rowwise:
            e = 768  # torch's CPU _scaled_mm itself, at a reduced size (a scalar reference kernel: cubic extrapolation)
            dt = _median_time(lambda: torch._scaled_mm(a[:e, :e].contiguous(), bt[:e, :e].contiguous().t(), sa.reshape(()), sb.reshape(()), out_dtype=torch.bfloat16), 1, warm=0)
            out["cpu_scaled_mm_op"] = dict(value=round(2.0 * e ** 3 / dt / 1e12, 6), unit="TFLOP/s", cores=cores, kind="reference",
                                           sample=f"torch._scaled_mm on CPU tensors at {e}^3 (one call, {dt:.2f} s); at this rate {m}x{k}x{n} would take "
                                                  f"{dt * (m * k * n) / e ** 3 / 60:.0f} min")
    return out


def through_dispatcher(abi, name, r, calls=200):
    """The same op called through PyTorch's dispatcher on device "vk" tensors (schema -> op layer -> C ABI -> kernel),
    one weight tensor over and over: wall time per call with the queue kept full and the host's time to issue a call,
    beside the kernel's own time on the same resident weights, so that the host's share shows.  int8: torch._weight_int8pack_mm;
    int4: torch._dyn_quant_matmul_4bit (the side-car of the packed weights is built by the first call and cached);
    float8: torch._scaled_mm."""
    import torch
    import torch_vulkan_amd.backend as tv
    if not r.get("inputs"):
        return None
    if name.startswith(("c1", "c2", "q8_")):
        x, w, s = (t.to("vk") for t in r["inputs"])
        op, call = "torch._weight_int8pack_mm", lambda: torch._weight_int8pack_mm(x, w, s)
    elif name.startswith("c3"):
        x, packed = (t.to("vk") for t in r["inputs"])
        (n, bs), k = r["shape"], x.shape[1]
        op, call = "torch._dyn_quant_matmul_4bit", lambda: torch._dyn_quant_matmul_4bit(x, packed, bs, k, n)
    elif name.startswith(("c4", "c5")):
        a, bt, sa, sb = r["inputs"]
        rowwise = sa.numel() > 1
        a, b = a.to("vk"), bt.to("vk").t()
        sa = (sa.reshape(-1, 1) if rowwise else sa.reshape(())).to("vk")
        sb = (sb.reshape(1, -1) if rowwise else sb.reshape(())).to("vk")
        op, call = "torch._scaled_mm", lambda: torch._scaled_mm(a, b, sa, sb, out_dtype=torch.bfloat16)
        calls = min(calls, 50)
    else:
        return None
    before = tv.fallback_counts()
    for _ in range(min(20, calls)):
        call()
    abi.synchronize()
    t0 = time.perf_counter()
    for _ in range(calls):
        call()
    t_issue = time.perf_counter()
    abi.synchronize()
    t1 = time.perf_counter()
    if tv.fallback_counts() != before:
        raise RuntimeError(f"bench.py: {op} on device vk fell back to the CPU")
    resident_ms = r.get("cache_resident_ms") or (r["event_ms"] if r.get("copies") == 1 else None)
    return dict(op=op + " on device vk", calls=calls, us_per_call=round((t1 - t0) * 1e6 / calls, 2),
                host_issue_us_per_call=round((t_issue - t0) * 1e6 / calls, 2),
                kernel_us_cache_resident=round(resident_ms * 1e3, 2) if resident_ms else None)


def load_traffic():
    """HBM traffic per launch measured with rocprofv3 --pmc (profiles/traffic.json), if recorded."""
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def load_counters():
    """Matrix-core busy fraction and the shader clock during the dominant kernel, from rocprofv3 --pmc runs
    (profiles/counters.json: SQ_VALU_MFMA_BUSY_CYCLES / (4 SIMDs x SQ_BUSY_CU_CYCLES); busy cycles per compute unit
    / the kernel's duration in the kernel trace), if recorded."""
    try:
        with open(os.path.join(ROOT, "profiles", "counters.json")) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def compact(key, rr, v, u, rf, cpu):
    """One short entry of `extra`."""
    # value and frac from the same clock (HIP events on the runtime's stream); the wall time per step, which includes the
    # two synchronisations around the timed loop, under its own key
    e = {"key": key, "value": rf["achieved"], "unit": u, "frac": rf["frac"], "kernel_ms": round(rr["event_ms"], 5),
         "wall_ms": round(rr["wall_ms"], 5)}
    if rf.get("counters"):
        e["counters"] = rf["counters"]
    if "cache_resident" in rf:
        e["resident_ms"] = rf["cache_resident"]["kernel_ms"]
    if rf.get("traffic"):
        e["traffic"] = rf["traffic"]
    if cpu.get("cpu_baseline"):
        c = cpu["cpu_baseline"]
        e["cpu"] = {"value": c["value"], "unit": c["unit"], "cores": c["cores"]}
    return e


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS) + sorted(CALIBRATION))
    ap.add_argument("--all", action="store_true", help="also the workloads beside the BASELINE configurations")
    ap.add_argument("--no-extra", action="store_true", help="only the selected workload")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--verbose", action="store_true", help="full roofline objects and CPU samples for every entry")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build is a one-GPU path (no collectives, no sharding); run with --gpus 1")
    abi = _abi()
    info = abi.device_info()
    traffic = load_traffic()
    counters = load_counters()

    r = {**WORKLOADS, **CALIBRATION}[args.workload](abi, args.steps, args.warmup)
    value, unit, roof = summarise(r)
    roof["traffic"] = traffic.get(args.workload)
    if counters.get(args.workload):
        roof["counters"] = counters[args.workload]
    if r["kind"] == "hbm":
        metric, dtype = "M=1 int8 GEMV GB/s (% of HBM peak)", "f32 accumulate (bf16 activations, int8 weights)"
    else:
        metric, dtype = "fp8 _scaled_mm TFLOP/s (% of MFMA peak)", "f32 accumulate (fp8 e4m3 operands)"
    if args.workload.startswith("c1"):
        dtype = "f32"
    elif args.workload.startswith("c3"):
        metric, dtype = "M=1 int4 GEMV GB/s (% of HBM peak)", "int32 block sums, f32 accumulate (int4 weights, int8 activations)"
    line = {
        "metric": r.get("metric") or metric,
        "value": round(value, 1), "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(r["wall_ms"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic (seeded)",
        "config": {"workload": r["name"], "key": args.workload, "weight_copies_rotated": r["copies"],
                   "device": info.name.decode(), "compute_units": info.compute_units},
        "roofline": roof,
    }
    if r.get("clock_ghz"):
        line["config"]["clock_ghz"] = r["clock_ghz"]
    if not args.no_cpu:
        line.update(cpu_baselines(abi, args.workload, r, port=True))
        line["through_dispatcher"] = through_dispatcher(abi, args.workload, r)
    if "cpu_baseline" not in line:
        line["cpu_baseline"] = None
    del r
    if not args.no_extra:
        # what bare loads and a register-only matrix-core loop sustain, in this run on this box (GB/s, TFLOP/s)
        ceilings = {}
        for key, fn in CALIBRATION.items():
            if key == args.workload or key == "copy_256mib":
                continue
            rr = fn(abi, args.steps, args.warmup)
            v, u, rf = summarise(rr)
            ceilings[key] = {"achieved": rf["achieved"], "unit": u, "kernel_ms": round(rr["event_ms"], 5)}
            if rr.get("clock_ghz"):
                ceilings[key]["clock_ghz"] = rr["clock_ghz"]  # (shader cycles per tick of the constant clock, read in the kernel)
            del rr
        line["ceilings"] = ceilings
        extra = []
        for name, fn in ({**OTHER, **BASELINE, **DECODE} if args.all else {**BASELINE, **DECODE}).items():
            if name == args.workload:
                continue
            rr = fn(abi, args.steps, args.warmup)
            v, u, rf = summarise(rr)
            rf["traffic"] = traffic.get(name)
            if counters.get(name):
                rf["counters"] = counters[name]
            cpu = {} if args.no_cpu or name not in BASELINE else cpu_baselines(abi, name, rr)
            e = compact(name, rr, v, u, rf, cpu)
            if not args.no_cpu and name in DISPATCHER_TOO:  # the full op through the dispatcher, host issue time beside it
                d = through_dispatcher(abi, name, rr, calls=100)
                if d:
                    e["dispatcher"] = {"us_per_call": d["us_per_call"], "host_issue_us": d["host_issue_us_per_call"]}
            if args.verbose:
                e.update(workload=rr["name"], ms_per_step=round(rr["wall_ms"], 5), roofline=rf, **cpu)
                if rr["kind"] == "hbm":
                    e["tflops"] = round(rr["flops"] / rr["event_ms"] / 1e9, 2)
                else:
                    e["hbm_gbps_algorithmic"] = round(rr["bytes"] / rr["event_ms"] / 1e6, 1)
                if "reference_layout_bytes" in rr:
                    e["reference_layout_bytes"] = rr["reference_layout_bytes"]
            extra.append(e)
            del rr
        line["extra"] = extra
    print(json.dumps(line))


if __name__ == "__main__":
    main()
