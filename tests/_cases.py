"""Seeded inputs of the parity tests, in one place.

The shapes and seeds of the first tables are the reference's own parametrisations
(tests/python/test_quant.py:20-21,61-63,101-103): they are data, and the frozen fixtures under
tests/golden/ were drawn from them.  Everything is built through draw(), a small recipe
interpreter, so that a test reads as "which tensors, from which seeds" and nothing else."""
import collections

import torch

# ---------------------------------------------------------------- tables (data)
INT8_SHAPES = [(32, 64, 48), (1, 4096, 300), (5, 100, 17), (70, 33, 5), (65, 1, 66)]  # (m, k, n)
INT8_SEEDS = {"a": 1, "b": 2, "scales": 3}
# (m, k, n, block size, bias)
INT4_SHAPES = [(1, 64, 4096, 32, False), (32, 128, 11008, 32, True), (5, 96, 70, 96, True), (3, 100, 9, 100, False),
               (4, 256, 16, 64, True), (9, 64, 33, 64, False)]
INT4_WEIGHT_SEED, INT4_ROWS_SEED = 7, 11
FLOAT8 = [torch.float8_e4m3fn, torch.float8_e5m2]
FLOAT8_PAIRS = [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[0], FLOAT8[1])]
FLOAT8_OUT = [torch.bfloat16, torch.float32, torch.float16, torch.float8_e4m3fn, None]
FLOAT8_SHAPE = (16, 32, 48)  # (m, k, n)
FLOAT8_SEEDS = {"a": 1, "b": 2, "scale_a": 3, "scale_b": 4, "bias": 5}


def draw(recipe, seed):
    """One tensor from a recipe (kind, shape, *args) and a seed:
    ("normal", shape[, factor]) ("uniform", shape[, divisor]) ("range", shape, lo, hi) ("bytes", shape)
    ("int8", shape) ("nibbles", shape)."""
    kind, shape, *args = recipe
    g = torch.Generator().manual_seed(seed)
    if kind == "normal":
        t = torch.randn(*shape, generator=g)
        return t * args[0] if args else t
    if kind == "uniform":
        t = torch.rand(*shape, generator=g)
        return t / args[0] if args else t
    if kind == "range":
        return torch.empty(*shape).uniform_(args[0], args[1], generator=g)
    if kind == "int8":
        return torch.randint(-128, 128, shape, dtype=torch.int8, generator=g)
    if kind == "bytes":
        return torch.randint(0, 256, shape, dtype=torch.uint8, generator=g)
    if kind == "nibbles":
        return torch.randint(0, 16, shape, dtype=torch.uint8, generator=g)
    raise ValueError(kind)


Int8Case = collections.namedtuple("Int8Case", "a b scales")
Int4Weights = collections.namedtuple("Int4Weights", "nibble_bytes scales bias")


def int8_case(dtype, m, k, n, seeds=INT8_SEEDS):
    """Activations ~N(0,1) in `dtype`, int8 weights, per-channel scales below 0.02 in `dtype`."""
    return Int8Case(draw(("normal", (m, k)), seeds["a"]).to(dtype), draw(("int8", (n, k)), seeds["b"]),
                    draw(("uniform", (n,), 50), seeds["scales"]).to(dtype))


def int4_weights(n, k, bs, seed=INT4_WEIGHT_SEED, bias=False):
    """Packed nibble bytes [n, k/2], scales below 0.1 per block (bfloat16-valued when groupwise, float32 for one
    block per channel), and an optional N(0,1) bias: seeds seed, seed + 1, seed + 2."""
    blocks = 1 if bs == k else k // bs
    scales = draw(("uniform", (n, blocks), 10), seed + 1)
    return Int4Weights(draw(("bytes", (n, k // 2)), seed), scales if bs == k else scales.bfloat16(),
                       draw(("normal", (n,)), seed + 2) if bias else None)


def int4_rows(m, k, dtype, seed=INT4_ROWS_SEED):
    """Activations 3 N(0,1); the first row half zeros, the second all negative (rows whose range touches zero from
    one side exercise both branches of the zero-point choice)."""
    x = draw(("normal", (m, k), 3), seed).to(dtype)
    x[0, : k // 2] = 0.0
    if m > 1:
        x[1] = -x[1].abs()
    return x


Float8Case = collections.namedtuple("Float8Case", "a b scale_a scale_b bias scale_result result_dtype")


def float8_case(fa, fb, out_dtype, rowwise, shape=FLOAT8_SHAPE, seeds=FLOAT8_SEEDS):
    """A row-major, B column-major ([n, k] storage, transposed view); scales in [0.5, 1.5) per row / column, or
    1.25 and 0.75; a bfloat16 bias with bfloat16 outputs, a result scale of 2 with float8 outputs."""
    m, k, n = shape
    a = draw(("normal", (m, k)), seeds["a"]).to(fa)
    b = draw(("normal", (n, k)), seeds["b"]).to(fb).t()
    if rowwise:
        sa, sb = draw(("uniform", (m, 1)), seeds["scale_a"]) + 0.5, draw(("uniform", (1, n)), seeds["scale_b"]) + 0.5
    else:
        sa, sb = torch.tensor(1.25), torch.tensor(0.75)
    bias = draw(("normal", (n,)), seeds["bias"]).bfloat16() if out_dtype == torch.bfloat16 else None
    sr = torch.tensor(2.0) if out_dtype == torch.float8_e4m3fn else None
    return Float8Case(a, b, sa, sb, bias, sr, out_dtype or fa)


# ---------------------------------------------------------------- the rows beside the path (tables)
INF, NAN = float("inf"), float("nan")
# float8 casts: two normal draws (spreads 3 and 300, 300 values each) and the values at which a conversion saturates,
# overflows, underflows, or meets NaN, infinities and the signed zero (test_fallback_ops.py:469-485 lists the same)
CAST_DRAWS = [(("normal", (300,), 3), 0), (("normal", (300,), 300), 1)]
CAST_EDGES = [0.0, -0.0, INF, -INF, NAN, 448.0, 464.0, 57344.0, 61440.0, 1e-9, -1e-9, 2.0**-9, 2.0**-10, 2.0**-17, 1e30]
# 16-bit products (m, k, n): whole tiles, ragged edges, k = 1, tall and flat, both tile sizes of the matrix-core kernel
GEMM16_SHAPES = [(64, 32, 64), (65, 33, 63), (17, 200, 129), (128, 1, 96), (3, 1000, 5), (300, 256, 260), (304, 256, 264)]
GEMM16_SEEDS = {"a": 1, "b": 2}
GEMM16_BATCHED = {"a": (("normal", (3, 40, 72)), 3), "b": (("normal", (3, 50, 72)), 4), "bias": (("normal", (50,)), 5)}
# affine quantisation: 40 values of spread 20 and the ones that meet NaN, infinities, ties and the integer ranges
AFFINE_DRAW = (("normal", (40,), 20), 0)
AFFINE_EDGES = [NAN, INF, -INF, 0.05, 0.15, -0.05, 1e30, 3e9]
AFFINE_QPARAMS = (0.1, 5)
FAKE_QUANT_ROWS = [[-1.3, 0.0, 0.26, 4.0], [NAN, INF, -0.5, 1e-3]]
FAKE_QUANT_TENSOR = {"scale": 0.05, "zero_point": 3, "range": (0, 255)}
FAKE_QUANT_BIG = (("normal", (2, 3, 500), 4), 4)
# the fused observer: four steps whose inputs widen and drift, the last with a small averaging constant
OBSERVER_STEPS = [(0.1, 0.0, 0.25), (1.1, -0.5, 0.25), (2.1, -1.0, 0.25), (3.1, -1.5, 0.01)]  # (spread, shift, averaging constant)
OBSERVER_INPUT = (4, 3, 5)


def cast_values():
    return torch.cat([draw(r, seed) for r, seed in CAST_DRAWS] + [torch.tensor(CAST_EDGES)])


def affine_values():
    return torch.cat([draw(*AFFINE_DRAW), torch.tensor(AFFINE_EDGES)]).view(6, 8)


def per_channel_cases():
    """(input, axis, scales, zero points) of the per-channel fake quantisation: the small matrix with integer and
    float zero points, a larger tensor along each axis, a 16-bit one, a transposed view."""
    small, big = torch.tensor(FAKE_QUANT_ROWS), draw(*FAKE_QUANT_BIG)
    wide_scales = draw(("uniform", (500,), 10), 5) + 0.01
    return [(small, 0, torch.tensor([0.05, 0.2]), torch.tensor([3, 250], dtype=torch.int32)),
            (small, 0, torch.tensor([0.05, 0.2]), torch.tensor([3.25, 250.5])),
            (big, 1, torch.tensor([0.05, 0.2, 0.01]), torch.tensor([3, 250, 128], dtype=torch.int32)),
            (big.bfloat16(), 2, wide_scales, torch.randint(0, 255, (500,), dtype=torch.int32, generator=torch.Generator().manual_seed(6))),
            (big.transpose(0, 2), 0, wide_scales, draw(("uniform", (500,)), 7) * 200)]
