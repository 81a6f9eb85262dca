"""The five quantised aten ops on device "vk": each op called on device tensors, with nothing allowed to fall back
to the CPU, against the oracle (and PyTorch's CPU op where it has one), on the reference's parametrisations
(tests/python/test_quant.py:20-21,61-63,101-103, kept as tables in _cases.py), on the frozen fixtures under
tests/golden/, and on the op layer's own behaviour (side-car cache, inference tensors, empty products, errors).
The C++ op layer (csrc/torch/quant.cpp) reaches the kernels through the C ABI."""
import os

import numpy as np
import pytest
import torch

import oracle
from _cases import (AFFINE_QPARAMS, FAKE_QUANT_BIG, FAKE_QUANT_ROWS, FAKE_QUANT_TENSOR, FLOAT8, FLOAT8_OUT, FLOAT8_PAIRS, GEMM16_BATCHED,
                    GEMM16_SEEDS, GEMM16_SHAPES, INF, INT4_SHAPES, INT8_SHAPES, OBSERVER_INPUT, OBSERVER_STEPS, affine_values, cast_values,
                    draw, float8_case, int4_rows, int4_weights, int8_case, per_channel_cases)
from _util import ODT, bits, no_fallback as on_gpu, ref_tol, to_device, unbits

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
# bfloat16 / float8 results come off the fp8 matrix cores, whose products are added in a
# window ~14 bits below the largest (a hardware property); float32 / float16 results are exact sums
HW_WINDOW = 2.0**-13


@pytest.fixture(scope="module")
def tv():
    import torch_vulkan_amd.backend as tv
    assert tv.is_available() and (tv.capabilities() & 12) == 12  # 8- and 16-bit storage
    return tv


def gen(seed):
    return torch.Generator().manual_seed(seed)


def on_vk(tv, op, *args, **kwargs):
    """op(*args, **kwargs) with every tensor moved to the device, nothing allowed to run on the CPU; the results
    come back as host tensors (a tuple stays a tuple)."""
    with on_gpu(tv):
        out = op(*to_device(args), **to_device(kwargs))
    assert all(t.device.type == "vk" for t in (out if isinstance(out, tuple) else (out,)))
    return to_device(out, "cpu")


def raises_each(table, call):
    """table: (exception type, message pattern, arguments); call(*arguments) must raise that."""
    for kind, pattern, arguments in table:
        with pytest.raises(kind, match=pattern):
            call(*arguments)


def test_device_round_trip(tv):
    x = torch.randn(5, 7, generator=gen(0))
    d = x.to("vk")
    assert d.device.type == "vk" and torch.equal(d.cpu(), x)
    assert torch.equal(d[::2].cpu(), x[::2]) and torch.equal(d.t().contiguous().cpu(), x.t().contiguous())
    assert torch.equal(d.to(torch.bfloat16).cpu(), x.bfloat16())  # (converted on the device: cast_f32_bf16)
    for dt in (torch.int8, torch.uint8, torch.float16, torch.bfloat16, torch.float8_e4m3fn, torch.float8_e5m2):
        y = (x * 10).to(dt)
        assert torch.equal(y.to("vk").cpu().view(torch.uint8), y.view(torch.uint8))
    assert d[1, 2].item() == x[1, 2].item()
    stats = tv.memory_stats()
    assert stats["allocated_bytes"] > 0 and stats["reserved_bytes"] >= stats["allocated_bytes"]
    torch.vk.synchronize()


# ------------------------------------------------------------------ _weight_int8pack_mm
def within_int8_band(got, dtype, a, b, s, rows=slice(None)):
    """|got - float64 sum| <= eps |sum| + 2^-20 sum|a||w| (the bound the reference's test states), from the oracle."""
    _, c64, mag = oracle.qmm8(bits(a), ODT[dtype], b.numpy(), bits(s), want_f64=True)
    assert got.dtype == dtype and got.shape == c64[rows].shape
    excess = np.abs(got.double().numpy() - c64[rows]) - ref_tol(c64, mag, ODT[dtype])[rows]
    assert (excess <= 0).all(), excess.max()


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16], ids=str)
@pytest.mark.parametrize("shape", INT8_SHAPES, ids=str)
def test_int8_weight_product(tv, dtype, shape):
    case = int8_case(dtype, *shape)
    within_int8_band(on_vk(tv, torch._weight_int8pack_mm, *case), dtype, *case)
    # every other row of A, read in place through the row stride
    with on_gpu(tv):
        a, b, s = to_device(tuple(case))
        strided = torch._weight_int8pack_mm(a[::2], b, s).cpu()
    within_int8_band(strided, dtype, *case, rows=slice(None, None, 2))


def test_int8_weight_product_fixtures(tv):
    """The frozen CPU results (tests/golden/q8.npz): the device inside twice the band around them that the oracle's
    float64 sum is held to (both sides are roundings of that sum)."""
    g = np.load(os.path.join(GOLDEN, "q8.npz"))
    for key in sorted(k[:-2] for k in g.files if k.endswith("_a")):
        odt = int(g[key + "_odt"])
        dtype = {v: k for k, v in ODT.items()}[odt]
        a, s, b = unbits(g[key + "_a"], dtype), unbits(g[key + "_s"], dtype), torch.from_numpy(g[key + "_b"])
        got = on_vk(tv, torch._weight_int8pack_mm, a, b, s)
        _, c64, mag = oracle.qmm8(g[key + "_a"], odt, g[key + "_b"], g[key + "_s"], want_f64=True)
        frozen = oracle.to_f32(g[key + "_out"], odt).astype(np.float64)
        assert (np.abs(got.double().numpy() - frozen) <= 2 * ref_tol(c64, mag, odt)).all(), key


def test_int8_weight_product_refusals(tv):
    a, b, s = to_device((torch.randn(4, 8), torch.zeros(3, 8, dtype=torch.int8), torch.ones(3)))
    raises_each([(RuntimeError, "expect B to be int8 tensor", (a, b.float(), s)),
                 (RuntimeError, "expect scales to be 1d tensor with size 3", (a, b, s[:2])),
                 (RuntimeError, "A must be contiguous on the last dimension", (a.t().contiguous().t(), b[:, :4], s))],
                torch._weight_int8pack_mm)


# ------------------------------------------------------------------ _dyn_quant_pack_4bit_weight / _dyn_quant_matmul_4bit
INT4_DTYPES = [(torch.float32, True), (torch.bfloat16, False)]  # (activation type, also with groupwise blocks)


@pytest.mark.parametrize("m,k,n,bs,bias", INT4_SHAPES)
@pytest.mark.parametrize("dtype,groupwise_too", INT4_DTYPES, ids=["float32", "bfloat16"])
def test_int4_product_bit_exact(tv, m, k, n, bs, bias, dtype, groupwise_too):
    if bs != k and not groupwise_too:
        pytest.skip("bfloat16 activations take one block per channel only (the CPU's check)")
    weights = int4_weights(n, k, bs, bias=bias)
    x = int4_rows(m, k, dtype)
    # the expectation: the oracle's packed vector and product, which the CPU's ops must equal bit for bit too
    packed = oracle.q4_pack(weights.nibble_bytes.numpy(), bits(weights.scales), ODT[weights.scales.dtype],
                            None if weights.bias is None else weights.bias.numpy())
    want = oracle.q4_matmul(bits(x), ODT[dtype], packed, bs, k, n)
    assert np.array_equal(bits(torch._dyn_quant_matmul_4bit(x, torch.from_numpy(packed), bs, k, n)), want)
    with on_gpu(tv):
        packed_on_device = torch._dyn_quant_pack_4bit_weight(*to_device(tuple(weights)), bs, k, n)
        x_vk = x.to("vk")
        products = [torch._dyn_quant_matmul_4bit(x_vk, packed_on_device, bs, k, n),
                    torch._dyn_quant_matmul_4bit(x_vk, packed_on_device, bs, k, n),  # (from the cached side-car)
                    torch._dyn_quant_matmul_4bit(x_vk, torch.from_numpy(packed).to("vk"), bs, k, n)]  # (packed on the host)
    assert np.array_equal(packed_on_device.cpu().numpy().view(np.uint32), packed.view(np.uint32))
    for got in products:
        assert got.dtype == dtype and np.array_equal(bits(got.cpu()), want)


def test_int4_product_fixtures(tv):
    """The frozen CPU results (tests/golden/q4.npz), bit for bit."""
    g = np.load(os.path.join(GOLDEN, "q4.npz"))
    for i in range(len(INT4_SHAPES)):
        m, k, n, bs, _ = (int(v) for v in g[f"c{i}_shape"])
        for tag, dtype in (("f32", torch.float32), ("bf16", torch.bfloat16)):
            if f"c{i}_{tag}_out" not in g:
                continue
            got = on_vk(tv, torch._dyn_quant_matmul_4bit, unbits(g[f"c{i}_{tag}_x"], dtype), torch.from_numpy(g[f"c{i}_packed"]), bs, k, n)
            assert np.array_equal(bits(got), g[f"c{i}_{tag}_out"]), (i, tag)


def test_int4_under_inference_mode(tv):
    """Inference tensors carry no version counter: packing and multiplying under torch.inference_mode() (and
    no_grad) must work and agree with the CPU."""
    n, k, bs = 24, 128, 32
    weights = int4_weights(n, k, bs, seed=31, bias=True)
    x = int4_rows(5, k, torch.float32, seed=32)
    want = torch._dyn_quant_matmul_4bit(x, torch._dyn_quant_pack_4bit_weight(*weights, bs, k, n), bs, k, n)
    for mode in (torch.inference_mode, torch.no_grad):
        with mode(), on_gpu(tv):
            packed = torch._dyn_quant_pack_4bit_weight(*to_device(tuple(weights)), bs, k, n)
            first = torch._dyn_quant_matmul_4bit(x.to("vk"), packed, bs, k, n)
            one_row = torch._dyn_quant_matmul_4bit(x[:1].to("vk"), packed, bs, k, n)  # (the other side-car layout)
            again = torch._dyn_quant_matmul_4bit(x.to("vk"), packed, bs, k, n)
        assert torch.equal(first.cpu(), want) and torch.equal(again.cpu(), want) and torch.equal(one_row.cpu(), want[:1])


def test_int4_inference_tensor_rewritten_in_place(tv):
    """In-place writes under torch.inference_mode() bump no version counter: the op layer's write paths drop the
    side-cars of the written storage themselves, so the next product sees the new weights (both side-car layouts)."""
    n, k, bs = 24, 128, 32
    x = int4_rows(5, k, torch.float32, seed=32)
    packs = [torch._dyn_quant_pack_4bit_weight(*int4_weights(n, k, bs, seed=s, bias=True), bs, k, n) for s in (41, 42, 43)]
    wants = [torch._dyn_quant_matmul_4bit(x, p, bs, k, n) for p in packs]
    with torch.inference_mode(), on_gpu(tv):
        packed = packs[0].to("vk")
        assert packed.is_inference()
        for rows in (5, 1):
            assert torch.equal(torch._dyn_quant_matmul_4bit(x[:rows].to("vk"), packed, bs, k, n).cpu(), wants[0][:rows])
        packed.copy_(packs[1])  # host -> device copy into the same storage
        for rows in (5, 1):
            assert torch.equal(torch._dyn_quant_matmul_4bit(x[:rows].to("vk"), packed, bs, k, n).cpu(), wants[1][:rows])
        packed.copy_(packs[2].to("vk"))  # device -> device copy
        for rows in (5, 1):
            assert torch.equal(torch._dyn_quant_matmul_4bit(x[:rows].to("vk"), packed, bs, k, n).cpu(), wants[2][:rows])
        packed.view(-1)[: n * k // 2].zero_()  # a fill through a view: every nibble byte 0, weights -8
        zeroed = packs[2].clone()
        zeroed[: n * k // 2] = 0
        assert torch.equal(torch._dyn_quant_matmul_4bit(x.to("vk"), packed, bs, k, n).cpu(), torch._dyn_quant_matmul_4bit(x, zeroed, bs, k, n))


def test_int4_sidecar_follows_writes(tv):
    """A side-car belongs to one version of the packed tensor: writing into the packed weights must show in the
    next product."""
    n, k, bs = 16, 64, 32
    weights = int4_weights(n, k, bs, seed=3)
    x = draw(("normal", (2, k)), 5)
    packed = torch._dyn_quant_pack_4bit_weight(*weights, bs, k, n)
    flipped = packed.clone()
    flipped[: n * k // 2] = 255.0 - flipped[: n * k // 2]
    on_device = packed.to("vk")
    before = torch._dyn_quant_matmul_4bit(x.to("vk"), on_device, bs, k, n).cpu()
    on_device.copy_(flipped)
    after = torch._dyn_quant_matmul_4bit(x.to("vk"), on_device, bs, k, n).cpu()
    assert torch.equal(before, torch._dyn_quant_matmul_4bit(x, packed, bs, k, n))
    assert torch.equal(after, torch._dyn_quant_matmul_4bit(x, flipped, bs, k, n))


def test_int4_sidecars_of_a_whole_model(tv):
    """300 live packed weights (more linear layers than Llama-3-8B has), decoded twice: the second pass must find
    every side-car (no "qmm4c_pack": one dispatch per product), results unchanged; a dead weight's side-car goes."""
    n, k, bs, layers = 16, 64, 32, 300
    torch.ops.vk.sidecar_cache(True)
    x = draw(("normal", (1, k)), 40).to("vk")
    base = int4_weights(n, k, bs, seed=41, bias=True)
    packed = []
    for layer in range(layers):
        nibble_bytes = base.nibble_bytes.roll(layer, 1)  # a different weight per layer, cheaply
        packed.append(torch._dyn_quant_pack_4bit_weight(nibble_bytes, base.scales, base.bias, bs, k, n).to("vk"))
    with on_gpu(tv):
        start = tv.dispatch_count()
        first = [torch._dyn_quant_matmul_4bit(x, w, bs, k, n) for w in packed]
        middle = tv.dispatch_count()
        second = [torch._dyn_quant_matmul_4bit(x, w, bs, k, n) for w in packed]
        end = tv.dispatch_count()
    assert middle - start == 2 * layers and end - middle == layers
    entries, held = torch.ops.vk.sidecar_cache()
    assert entries == layers and held >= layers * n * k // 2
    for layer in (0, 1, 150, 299):
        want = torch._dyn_quant_matmul_4bit(x.cpu(), packed[layer].cpu(), bs, k, n)
        assert torch.equal(first[layer].cpu(), want) and torch.equal(second[layer].cpu(), want)
    del packed[:100]
    assert torch.ops.vk.sidecar_cache()[0] == layers - 100
    assert torch.ops.vk.sidecar_cache(True) == (0, 0)


def test_int4_refusals(tv):
    n, k = 8, 64
    weights = int4_weights(n, k, 32, seed=3)
    w, sc = weights.nibble_bytes.to("vk"), weights.scales.to("vk")
    raises_each([(RuntimeError, "Group size should be multiple of 32", (w, sc, None, 48, k, n)),
                 (RuntimeError, "expect weight to be kByte", (w.cpu().to(torch.int8).to("vk"), sc, None, 32, k, n))],
                torch._dyn_quant_pack_4bit_weight)
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, None, 32, k, n)
    x = torch.randn(2, k).to("vk")
    raises_each([(RuntimeError, "expect input to be float32 or bfloat16 tensor", (x.cpu().bfloat16().to("vk"), packed, 32, k, n)),
                 (RuntimeError, "Invalid packed weight tensor size", (x, packed[:100], 32, k, n))],
                torch._dyn_quant_matmul_4bit)


# ------------------------------------------------------------------ _scaled_mm
def scaled_mm_expectation(case):
    """(expected values as float64 in the result type's precision, allowed error) from the oracle: its float64-accurate
    sum rounded once, the reference's bound eps |want| + 2^-20 sum|a||b| and, for results that come off the fp8
    matrix cores, their summation window."""
    a, b, sa, sb, bias, sr, res_dtype = case
    want, mag = oracle.scaled_mm(bits(a), ODT[a.dtype], bits(b.t()), ODT[b.dtype], sa.numpy(), sb.numpy(), sa.numel() > 1,
                                 None if bias is None else bits(bias), oracle.BF16, None if sr is None else float(sr),
                                 ODT[res_dtype], want_mag=True)
    want = oracle.to_f32(want, ODT[res_dtype]).astype(np.float64)
    mag = mag / (float(sr) if sr is not None else 1.0)
    tol = ref_tol(want, mag, ODT[res_dtype])
    if res_dtype not in (torch.float32, torch.float16):
        tol = tol + HW_WINDOW * mag
    return want, tol


@pytest.mark.parametrize("fa,fb", FLOAT8_PAIRS, ids=str)
@pytest.mark.parametrize("out_dtype", FLOAT8_OUT, ids=str)
@pytest.mark.parametrize("rowwise", [False, True], ids=["per_tensor", "per_row"])
def test_scaled_mm(tv, fa, fb, out_dtype, rowwise):
    case = float8_case(fa, fb, out_dtype, rowwise)
    want, tol = scaled_mm_expectation(case)
    options = dict(bias=case.bias, scale_result=case.scale_result, out_dtype=out_dtype)
    functional = on_vk(tv, torch._scaled_mm, case.a, case.b, case.scale_a, case.scale_b, **options)
    with on_gpu(tv):
        into = torch.empty(0, dtype=case.result_dtype).to("vk")
        torch._scaled_mm(*to_device((case.a, case.b, case.scale_a, case.scale_b)), **to_device(options), out=into)
    for got in (functional, into.cpu()):
        assert got.dtype == case.result_dtype and got.shape == want.shape
        assert (np.abs(got.double().numpy() - want) <= tol).all()


def test_scaled_mm_fixtures(tv):
    """The frozen CPU results (tests/golden/f8.npz, per-tensor scales)."""
    g = np.load(os.path.join(GOLDEN, "f8.npz"))
    torch_type = {v: k for k, v in ODT.items()}
    for key in sorted(k[:-2] for k in g.files if k.endswith("_a")):
        fa, fb, odt = (int(v) for v in g[key + "_fmt"])
        sr = float(g[key + "_sr"]) if key + "_sr" in g else None
        bias = unbits(g[key + "_bias"], torch.bfloat16) if key + "_bias" in g else None
        _, mag = oracle.scaled_mm(g[key + "_a"], fa, g[key + "_bt"], fb, g[key + "_sa"], g[key + "_sb"], False,
                                  None if bias is None else bits(bias), oracle.BF16, sr, odt, want_mag=True)
        mag = mag / (sr or 1.0)
        frozen = oracle.to_f32(g[key + "_out"], odt).astype(np.float64)
        asked = None if key.endswith("_None") else torch_type[odt]
        got = on_vk(tv, torch._scaled_mm, unbits(g[key + "_a"], torch_type[fa]), unbits(g[key + "_bt"], torch_type[fb]).t(),
                    torch.tensor(float(g[key + "_sa"][0])), torch.tensor(float(g[key + "_sb"][0])), bias=bias,
                    scale_result=None if sr is None else torch.tensor(sr), out_dtype=asked)
        tol = ref_tol(frozen, mag, odt) + (0 if torch_type[odt] in (torch.float32, torch.float16) else HW_WINDOW * mag)
        assert got.dtype == torch_type[odt] and (np.abs(got.double().numpy() - frozen) <= tol).all(), key


def test_scaled_mm_result_scale_needs_a_float8_out_dtype(tv):
    """scale_result applies when out_dtype asks for float8; without out_dtype the functional form returns the
    operands' float8 type unscaled, as the CPU's op does."""
    case = float8_case(FLOAT8[0], FLOAT8[0], None, False)
    sr = torch.tensor(4.0)
    plain = torch._scaled_mm(case.a, case.b, case.scale_a, case.scale_b)
    assert torch.equal(torch._scaled_mm(case.a, case.b, case.scale_a, case.scale_b, scale_result=sr).view(torch.uint8),
                       plain.view(torch.uint8))  # (the CPU ignores it here)
    unscaled = on_vk(tv, torch._scaled_mm, case.a, case.b, case.scale_a, case.scale_b, scale_result=sr)
    without = on_vk(tv, torch._scaled_mm, case.a, case.b, case.scale_a, case.scale_b)
    scaled = on_vk(tv, torch._scaled_mm, case.a, case.b, case.scale_a, case.scale_b, scale_result=sr, out_dtype=FLOAT8[0])
    assert unscaled.dtype == FLOAT8[0] and torch.equal(unscaled.view(torch.uint8), without.view(torch.uint8))
    want, tol = scaled_mm_expectation(case)
    assert (np.abs(unscaled.double().numpy() - want) <= tol).all()
    assert (np.abs(scaled.double().numpy() * 4.0 - want) <= 4.0 * tol + 2.0**-3 * np.abs(want)).all()
    assert not torch.equal(scaled.view(torch.uint8), unscaled.view(torch.uint8))


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32, torch.float8_e4m3fn], ids=str)
def test_scaled_mm_of_no_columns_of_k(tv, out_dtype):
    """K = 0: the product is zeros, the bias and the cast still apply, and it runs on the device."""
    a = torch.zeros(5, 0).to(FLOAT8[0])
    b = torch.zeros(7, 0).to(FLOAT8[0]).t()
    bias = draw(("normal", (7,)), 8).bfloat16()
    one = torch.tensor(1.0)
    got = on_vk(tv, torch._scaled_mm, a, b, one, one, bias=bias, out_dtype=out_dtype)
    assert got.shape == (5, 7) and got.dtype == out_dtype
    assert torch.equal(got.float(), bias.float().to(out_dtype).float().expand(5, 7))
    rows = on_vk(tv, torch._scaled_mm, a, b, torch.ones(5, 1), torch.ones(1, 7), out_dtype=out_dtype)
    assert (rows.float() == 0).all()


def test_scaled_mm_refusals(tv):
    a = torch.randn(4, 8).to(FLOAT8[0]).to("vk")
    b = torch.randn(6, 8).to(FLOAT8[0]).to("vk").t()
    one = torch.tensor(1.0).to("vk")
    raises_each([(ValueError, "Invalid scaling configuration", ((a, b, torch.ones(3).to("vk"), one), {})),
                 (ValueError, "out_dtype must match output matrix type",
                  ((a, b, one, one), dict(out_dtype=torch.float32, out=torch.empty(0, dtype=torch.half).to("vk")))),
                 (RuntimeError, "Bias must be size 6", ((a, b, one, one), dict(bias=torch.ones(5).to("vk"), out_dtype=torch.float32)))],
                lambda args, kwargs: torch._scaled_mm(*args, **kwargs))


def test_empty_inputs(tv):
    """No rows: every op of the path returns an empty result of the right shape and type (and launches nothing wrong)."""
    with on_gpu(tv):
        b = torch.randint(-128, 128, (5, 64), dtype=torch.int8, generator=gen(1)).to("vk")
        out = torch._weight_int8pack_mm(torch.zeros(0, 64, dtype=torch.bfloat16).to("vk"), b, torch.ones(5, dtype=torch.bfloat16).to("vk"))
        assert out.shape == (0, 5) and out.dtype == torch.bfloat16
        packed = torch._dyn_quant_pack_4bit_weight(*int4_weights(6, 64, 32, seed=3, bias=True), 32, 64, 6).to("vk")
        out = torch._dyn_quant_matmul_4bit(torch.zeros(0, 64).to("vk"), packed, 32, 64, 6)
        assert out.shape == (0, 6) and out.dtype == torch.float32
        a8 = torch.zeros(0, 32).to(torch.float8_e4m3fn).to("vk")
        b8 = torch.zeros(16, 32).to(torch.float8_e4m3fn).to("vk").t()
        one = torch.ones(()).to("vk")
        out = torch._scaled_mm(a8, b8, one, one, out_dtype=torch.bfloat16)
        assert out.shape == (0, 16) and out.dtype == torch.bfloat16
        out = torch.mm(torch.zeros(0, 8, dtype=torch.bfloat16).to("vk"), torch.zeros(8, 4, dtype=torch.bfloat16).to("vk"))
        assert out.shape == (0, 4)


def test_fallback_is_counted(tv):
    """An op without a vk kernel runs on the CPU and shows in fallback_counts (what on_gpu() watches)."""
    before = sum(tv.fallback_counts().values())
    y = torch.ones(3).to("vk") + 1
    assert torch.equal(y.cpu(), torch.full((3,), 2.0)) and sum(tv.fallback_counts().values()) > before


def same_float_bits(got, want_bits, dtype):
    """got (host tensor) holds want_bits (a storage array of the oracle) bit for bit; NaNs need only be NaNs."""
    g, nan = bits(got), np.isnan(oracle.to_f32(want_bits, ODT[dtype]))
    assert got.dtype == dtype and g.shape == want_bits.shape
    assert np.array_equal(np.isnan(oracle.to_f32(g, ODT[dtype])), nan) and np.array_equal(g[~nan], want_bits[~nan])


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("wide", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_float8_casts(tv, f8, wide):
    """Tensor.to() between a float8 type and a wider float type, on the device (one cast_fp8 launch each way):
    the oracle's conversion (pinned against c10's on every code and rounding midpoint) decides, PyTorch's CPU
    conversion agrees.  Inputs: _cases.cast_values (draws plus the saturating / overflowing / special values) one
    way, all 256 codes the other."""
    values = cast_values().to(wide)
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(f8)
    launches = tv.dispatch_count()
    narrowed, widened = on_vk(tv, lambda v, c: (v.to(f8), c.to(wide)), values, codes)
    assert tv.dispatch_count() - launches == 2
    assert np.array_equal(bits(narrowed), oracle.cast(bits(values), ODT[wide], ODT[f8]))
    assert np.array_equal(bits(narrowed), bits(values.to(f8)))
    same_float_bits(widened, oracle.cast(bits(codes), ODT[f8], ODT[wide]), wide)
    same_float_bits(widened, bits(codes.to(wide)), wide)


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("src", [torch.float32, torch.bfloat16], ids=str)
def test_fp8_quant_rowwise_into_scaled_mm(tv, f8, src):
    """torch.ops.vk.fp8_quant_rowwise (the producer in front of _scaled_mm): bit for bit the same
    steps composed from PyTorch's CPU operators, and its outputs go straight into _scaled_mm."""
    fmax = 448.0 if f8 == torch.float8_e4m3fn else 57344.0
    a = (torch.randn(48, 256, generator=gen(5)) * 0.7).to(src)
    w = (torch.randn(80, 256, generator=gen(6)) * 0.04).to(src)
    with on_gpu(tv):
        qa, sa = torch.ops.vk.fp8_quant_rowwise(a.to("vk"), f8)
        qw, sw = torch.ops.vk.fp8_quant_rowwise(w.to("vk"), torch.float8_e4m3fn)
        out = torch._scaled_mm(qa, qw.t(), sa, sw.t(), out_dtype=torch.float32)

    def on_cpu(x, dt, top):
        amax = torch.clamp(x.float().abs().amax(dim=1, keepdim=True), min=1e-12)
        scale = torch.true_divide(amax, torch.tensor(top))
        y = torch.clamp(x.float() * torch.true_divide(torch.tensor(top), amax), -top, top)
        return y.to(dt), scale

    ca, csa = on_cpu(a, f8, fmax)
    cw, csw = on_cpu(w, torch.float8_e4m3fn, 448.0)
    assert torch.equal(qa.cpu().view(torch.uint8), ca.view(torch.uint8)) and torch.equal(sa.cpu(), csa)
    assert torch.equal(qw.cpu().view(torch.uint8), cw.view(torch.uint8)) and torch.equal(sw.cpu(), csw)
    want = (ca.float() * csa).double() @ (cw.float() * csw).double().t()
    mag = (ca.float() * csa).abs().double() @ (cw.float() * csw).abs().double().t()
    assert ((out.cpu().double() - want).abs() <= 2.0**-23 * want.abs() + 2.0**-20 * mag).all()
    with pytest.raises(RuntimeError, match="float8_e4m3fn or float8_e5m2"):
        torch.ops.vk.fp8_quant_rowwise(a.to("vk"), torch.bfloat16)


def inside_gemm_band(got, dtype, a, b, cin=None, alpha=1.0, beta=0.0):
    """got against the oracle's alpha a @ b + beta cin (float32 sums, one rounding): within one unit of the 16-bit
    type of it plus 2^-20 of the summed magnitudes (the order of the sums is free), the reference's bound for its
    matrix-core kernel."""
    want, mag = oracle.gemm16(bits(a), bits(b), ODT[dtype], cin=None if cin is None else bits(cin), alpha=alpha, beta=beta, want_mag=True)
    want = oracle.to_f32(want, ODT[dtype]).astype(np.float64)
    assert got.dtype == dtype and tuple(got.shape) == want.shape
    band = EPS16[dtype] * np.maximum(np.abs(want), 2.0**-14) + 2.0**-20 * mag
    excess = np.abs(got.double().numpy() - want) - band
    assert (excess <= 0).all(), excess.max()


EPS16 = {torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=str)
def test_16bit_matrix_products(tv, dtype):
    """torch.mm / bmm / addmm / baddbmm / linear of 16-bit tensors on device "vk" run on the matrix-core kernels
    ("gemmcm_<T>") and stay inside the oracle's band: the shapes of _cases.GEMM16_SHAPES in all four operand
    layouts and through a row-strided view, then batches with a broadcast bias, an out= that has to be resized,
    and k = 0."""
    for m, k, n in GEMM16_SHAPES:
        a = draw(("normal", (m, k)), GEMM16_SEEDS["a"]).to(dtype)
        b = draw(("normal", (k, n)), GEMM16_SEEDS["b"]).to(dtype)
        column_major = lambda t: t.t().contiguous().t()
        for x, y in ((a, b), (column_major(a), column_major(b)), (a, column_major(b)), (column_major(a), b)):
            inside_gemm_band(on_vk(tv, torch.mm, x, y), dtype, a, b)
        inside_gemm_band(on_vk(tv, lambda x, y: x[::2] @ y, a, b), dtype, a[::2], b)
    a, b, bias = (draw(*GEMM16_BATCHED[name]).to(dtype) for name in ("a", "b", "bias"))
    bt = b.transpose(1, 2)
    inside_gemm_band(on_vk(tv, torch.bmm, a, bt), dtype, a, bt)
    inside_gemm_band(on_vk(tv, lambda c, x, y: torch.addmm(c, x, y, beta=0.5, alpha=2.0), bias, a[0], bt[0]), dtype, a[0], bt[0],
                     cin=bias, alpha=2.0, beta=0.5)
    inside_gemm_band(on_vk(tv, lambda c, x, y: torch.baddbmm(c, x, y, beta=0.5, alpha=2.0), bias, a, bt), dtype, a, bt, cin=bias,
                     alpha=2.0, beta=0.5)
    inside_gemm_band(on_vk(tv, torch.nn.functional.linear, a, b[0], bias), dtype, a, bt[:1].expand(3, -1, -1), cin=bias, beta=1.0)

    def into_empty_out(x, y):
        out = torch.empty(0, dtype=dtype, device="vk")
        torch.mm(x, y, out=out)
        return out
    inside_gemm_band(on_vk(tv, into_empty_out, a[1], bt[1]), dtype, a[1], bt[1])
    nothing = on_vk(tv, torch.mm, a[0, :, :0], bt[0, :0])
    assert nothing.shape == (40, 50) and not nothing.any()
    assert tv.kernel_subgroup_size("gemmcm_bf16") == 64 and tv.kernel_subgroup_size("gemmcm_f16") == 64
    raises_each([(RuntimeError, "cannot be multiplied", (a[0], b[0])), (RuntimeError, "same dtype", (a[0], bt[0].float()))],
                lambda x, y: torch.mm(x.to("vk"), y.to("vk")))


def test_strided_copies_and_fills_on_the_device(tv):
    """contiguous(), copy_ between strided / broadcast views, float conversions and fill_ / zero_ run as
    device kernels (the dispatch count moves, nothing falls back), bit for bit as the CPU."""
    x = torch.randn(6, 40, 66, generator=gen(21))
    d = x.to("vk")
    with on_gpu(tv):
        n0 = tv.dispatch_count()
        t = d.transpose(1, 2).contiguous()
        p = d.permute(2, 0, 1)[:, ::2].contiguous()
        h = d.to(torch.float16)
        b = d.transpose(0, 2).to(torch.bfloat16)
        back = b.to(torch.float32)
        z = torch.empty(5, 7, device="vk").fill_(2.5)
        z[:, ::2].zero_()
        w = torch.empty(4, 66, device="vk")
        w.copy_(d[0, 3])  # a broadcast row
        e = torch.empty(3, 4, dtype=torch.int64, device="vk").fill_(-7)
        assert tv.dispatch_count() - n0 == 9  # one kernel each
    assert torch.equal(t.cpu(), x.transpose(1, 2).contiguous()) and t.is_contiguous()
    assert torch.equal(p.cpu(), x.permute(2, 0, 1)[:, ::2].contiguous())
    assert torch.equal(h.cpu(), x.half()) and torch.equal(b.cpu(), x.transpose(0, 2).bfloat16())
    assert torch.equal(back.cpu(), x.transpose(0, 2).bfloat16().float())
    want = torch.full((5, 7), 2.5)
    want[:, ::2] = 0
    assert torch.equal(z.cpu(), want) and torch.equal(w.cpu(), x[0, 3].expand(4, 66)) and (e.cpu() == -7).all()
    # host <-> device with strides on the device side: staged densely, scattered / gathered by the kernels
    y = torch.zeros(8, 10).to("vk")
    y[::2, 1:9].copy_(x[0, :4, :8])
    ref = torch.zeros(8, 10)
    ref[::2, 1:9] = x[0, :4, :8]
    assert torch.equal(y.cpu(), ref) and torch.equal(y[::2, 1:9].cpu(), x[0, :4, :8])
    # what the quantised ops take: a non-contiguous activation and int8 weight made contiguous on the device
    wq = torch.randint(-128, 128, (48, 64), dtype=torch.int8, generator=gen(22))
    with on_gpu(tv):
        wt = wq.to("vk").t().contiguous().t().contiguous()
    assert torch.equal(wt.cpu(), wq)


QTYPE = {torch.quint8: oracle.QUINT8, torch.qint8: oracle.QINT8, torch.qint32: oracle.QINT32}


@pytest.mark.parametrize("qdtype", list(QTYPE), ids=str)
def test_quantized_per_tensor(tv, qdtype):
    """Per-tensor affine quantised tensors on device "vk" (csrc/torch/quantized.cpp): the integers of
    quantize_per_tensor are the oracle's (the x86 CPU's arithmetic) on _cases.affine_values, dequantize gives the
    oracle's floats, and what only moves the integers around (flip, clone, a transposed input, qparams given as
    tensors, device <-> host) moves them unchanged; the quantiser's parameters read back as set."""
    x = affine_values()
    scale, zero_point = AFFINE_QPARAMS
    ints = oracle.quantize_affine(x.numpy(), scale, zero_point, QTYPE[qdtype])
    floats = oracle.dequantize_affine(ints, scale, zero_point, QTYPE[qdtype])
    with on_gpu(tv):
        q = torch.quantize_per_tensor(x.to("vk"), scale, zero_point, qdtype)
        assert q.is_quantized and q.device.type == "vk" and q.dtype == qdtype and q.qscheme() == torch.per_tensor_affine
        assert q.q_scale() == scale and q.q_zero_point() == zero_point
        moved = {"as quantised": q.int_repr(), "cloned": q.clone().int_repr(), "flipped": q.flip((0, 1)).int_repr(),
                 "transposed input": torch.quantize_per_tensor(x.to("vk").t(), scale, zero_point, qdtype).int_repr(),
                 "tensor qparams": torch.quantize_per_tensor(x.to("vk"), torch.tensor(scale).to("vk"), torch.tensor(zero_point).to("vk"),
                                                             qdtype).int_repr()}
        back = q.dequantize()
        blank = torch._empty_affine_quantized([5, 5, 5, 5], scale=2, zero_point=3, dtype=qdtype, device="vk")
    expect = {"as quantised": ints, "cloned": ints, "flipped": ints[::-1, ::-1], "transposed input": ints.T, "tensor qparams": ints}
    for name, got in moved.items():
        assert np.array_equal(got.cpu().numpy(), expect[name]), name
    assert np.array_equal(back.cpu().numpy(), floats, equal_nan=True)
    cpu = torch.quantize_per_tensor(x, scale, zero_point, qdtype)
    assert np.array_equal(cpu.int_repr().numpy(), ints)  # (PyTorch's CPU kernel agrees with the oracle)
    assert np.array_equal(q.cpu().int_repr().numpy(), ints) and np.array_equal(cpu.to("vk").int_repr().cpu().numpy(), ints)
    assert blank.flatten(0, -1).shape == (625,) and blank.ravel().shape == (625,)
    raises_each([(RuntimeError, "only works on Float", (x.half(),))], lambda t: torch.quantize_per_tensor(t.to("vk"), scale, zero_point, qdtype))


def same_fake_quant(got, want, dtype):
    """(output, mask) from the device against the oracle's pair of storage arrays."""
    same_float_bits(got[0], want[0], dtype)
    assert np.array_equal(got[1].numpy().astype(np.uint8), want[1])


def test_fake_quantize_cachemask_ops(tv):
    """The fake-quantisation operators with their masks on device "vk", one fused kernel each, against the oracle
    (the CPU's arithmetic, fused multiply-add of the float-zero-point form included): per tensor with qparams in
    tensors (switched on and off), per channel over _cases.per_channel_cases (integer and float zero points, a
    16-bit input, a transposed view), and the plain per-tensor operator."""
    x = torch.tensor(FAKE_QUANT_ROWS)
    scale, zero_point, (lo, hi) = (FAKE_QUANT_TENSOR[k] for k in ("scale", "zero_point", "range"))
    per_tensor = torch.ops.aten._fake_quantize_per_tensor_affine_cachemask_tensor_qparams
    switch = lambda on: torch.full((1,), int(on), dtype=torch.long)
    want = oracle.fake_quant(x.numpy(), oracle.F32, [scale], np.array([zero_point], np.int32), lo, hi)
    same_fake_quant(on_vk(tv, per_tensor, x, torch.tensor([scale]), torch.tensor([zero_point], dtype=torch.int32), switch(True), lo, hi),
                    want, torch.float32)
    passed, mask = on_vk(tv, per_tensor, x, torch.tensor([scale]), torch.tensor([zero_point], dtype=torch.int32), switch(False), lo, hi)
    same_float_bits(passed, x.numpy(), torch.float32)  # switched off: the input, every element inside
    assert mask.all()
    per_channel = torch.ops.aten.fake_quantize_per_channel_affine_cachemask
    for inp, axis, scales, zero_points in per_channel_cases():
        dense = inp.contiguous()
        want = oracle.fake_quant(bits(dense), ODT[inp.dtype], scales.numpy(), zero_points.numpy(), lo, hi, axis=axis)
        got = on_vk(tv, per_channel, inp, scales, zero_points, axis, lo, hi)
        assert got[0].shape == inp.shape
        same_fake_quant(got, want, inp.dtype)
    big = draw(*FAKE_QUANT_BIG)
    plain = on_vk(tv, torch.fake_quantize_per_tensor_affine, big, scale, zero_point, lo, hi)
    same_float_bits(plain, oracle.fake_quant(big.numpy(), oracle.F32, [scale], np.array([zero_point], np.int32), lo, hi)[0], torch.float32)
    raises_each([(RuntimeError, "must be between", (torch.tensor([3, 300], dtype=torch.int32),))],
                lambda zps: per_channel(x.to("vk"), torch.tensor([0.05, 0.2]).to("vk"), zps.to("vk"), 0, lo, hi))


@pytest.mark.parametrize("per_row", [False, True])
@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("qrange", [(0, 255), (-128, 127)])
def test_fused_moving_avg_obs_fake_quant(tv, per_row, symmetric, qrange):
    """_fused_moving_avg_obs_fq_helper on device "vk" over _cases.OBSERVER_STEPS: the running range (infinite at
    first, then a moving average), the scale and zero point chosen from it and the fake-quantised output, each step
    against the oracle's step and PyTorch's CPU operator, both bit for bit."""
    channels = OBSERVER_INPUT[0] if per_row else 1
    fresh = lambda: [torch.full((channels,), INF), torch.full((channels,), -INF), torch.ones(channels), torch.zeros(channels, dtype=torch.int32)]
    on_device, on_host = [t.to("vk") for t in fresh()], fresh()
    run_min, run_max = np.full(channels, np.inf, np.float32), np.full(channels, -np.inf, np.float32)
    helper = torch.ops.aten._fused_moving_avg_obs_fq_helper
    one = torch.tensor([1])
    g = gen(0)
    for spread, shift, averaging in OBSERVER_STEPS:
        x = torch.randn(*OBSERVER_INPUT, generator=g) * spread + shift
        with on_gpu(tv):
            out, mask = helper(x.to("vk"), one.to("vk"), one.to("vk"), *on_device, averaging, qrange[0], qrange[1], 0, per_row, symmetric)
        want_out, want_mask, scales, zero_points = oracle.observe_fake_quant(x.numpy(), oracle.F32, run_min, run_max, averaging, qrange[0],
                                                                               qrange[1], per_row, symmetric)
        same_fake_quant((out.cpu(), mask.cpu()), (want_out, want_mask), torch.float32)
        for got, want in zip(on_device, (run_min, run_max, scales, zero_points)):
            assert np.array_equal(got.cpu().numpy(), want)
        host_out, host_mask = helper(x, one, one, *on_host, averaging, qrange[0], qrange[1], 0, per_row, symmetric)
        assert torch.equal(out.cpu(), host_out) and torch.equal(mask.cpu(), host_mask)
        for got, want in zip(on_device, on_host):
            assert torch.equal(got.cpu(), want)
