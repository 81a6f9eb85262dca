"""The five quantised aten ops on device "vk": each op called on device tensors, with nothing allowed to fall back
to the CPU, against the oracle (and PyTorch's CPU op where it has one), on the reference's parametrisations
(tests/python/test_quant.py:20-21,61-63,101-103, kept as tables in _cases.py), on the frozen fixtures under
tests/golden/, and on the op layer's own behaviour (side-car cache, inference tensors, empty products, errors).
The C++ op layer (csrc/torch/quant.cpp) reaches the kernels through the C ABI."""
import contextlib
import os

import numpy as np
import pytest
import torch

import oracle
from _cases import (FLOAT8, FLOAT8_OUT, FLOAT8_PAIRS, INT4_SHAPES, INT8_SHAPES, draw, float8_case, int4_rows, int4_weights,
                    int8_case)
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


@pytest.mark.parametrize("f8", FLOAT8, ids=str)
@pytest.mark.parametrize("src", [torch.float32, torch.float16, torch.bfloat16], ids=str)
def test_float8_casts(tv, f8, src):
    """The reference's float8 cast test for the types _scaled_mm takes
    (tests/python/test_fallback_ops.py:469-485): every float8 code to the wider type, and values
    that round, saturate, overflow and are NaN, inf or -0 to float8, bit for bit as the CPU's,
    converted on the device (cast_fp8 counts its dispatches)."""
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(f8)
    x = torch.cat([torch.randn(300, generator=gen(0)) * 3, torch.randn(300, generator=gen(1)) * 300,
                   torch.tensor([0.0, -0.0, float("inf"), -float("inf"), float("nan"), 448.0, 464.0, 57344.0, 61440.0,
                                 1e-9, -1e-9, 2.0 ** -9, 2.0 ** -10, 2.0 ** -17, 1e30])]).to(src)
    dx = x.to("vk")
    dcodes = codes.to("vk")
    before = tv.dispatch_count()
    with on_gpu(tv):
        got = dx.to(f8)
        back = dcodes.to(src)
    assert tv.dispatch_count() - before == 2  # both conversions ran as kernels
    assert torch.equal(got.cpu().view(torch.uint8), x.to(f8).view(torch.uint8))
    torch.testing.assert_close(back.cpu(), codes.to(src), equal_nan=True, atol=0, rtol=0)


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


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_16bit_matrix_products(tv, dtype):
    """mm / bmm / addmm of 16-bit tensors on the matrix cores, as the reference tests its
    cooperative-matrix kernel (tests/python/test_matmul.py:250-284): float32 sums rounded once, one
    ulp from the CPU's float32 product plus summation-order error relative to the products'
    magnitudes; every layout, a strided view, batches, alpha / beta with a broadcast bias."""

    def want(x, y):
        return (x.float() @ y.float()).to(dtype)

    def close(got, ref, mag):
        assert got.device.type == "vk" and got.dtype == dtype and got.shape == ref.shape
        got, ref = got.cpu().float(), ref.float()
        tol = torch.finfo(dtype).eps * ref.abs().clamp_min(2**-14) + 2**-20 * mag
        assert ((got - ref).abs() <= tol).all(), (got - ref).abs().max().item()

    for m, k, n in [(64, 32, 64), (65, 33, 63), (17, 200, 129), (128, 1, 96), (3, 1000, 5), (300, 256, 260), (304, 256, 264)]:
        a, b = torch.randn(m, k, generator=gen(1)).to(dtype), torch.randn(k, n, generator=gen(2)).to(dtype)
        at, bt = a.t().contiguous().t(), b.t().contiguous().t()  # (column-major)
        for x, y in [(a, b), (at, bt), (a, bt), (at, b)]:
            with on_gpu(tv):
                got = x.to("vk") @ y.to("vk")
            close(got, want(a, b), a.float().abs() @ b.float().abs())
        with on_gpu(tv):
            got = a.to("vk")[::2] @ b.to("vk")
        close(got, want(a[::2], b), a[::2].float().abs() @ b.float().abs())
    a, b = torch.randn(3, 40, 72, generator=gen(3)).to(dtype), torch.randn(3, 50, 72, generator=gen(4)).to(dtype)
    bias = torch.randn(50, generator=gen(5)).to(dtype)
    with on_gpu(tv):
        got_t = torch.bmm(a.to("vk"), b.to("vk").transpose(1, 2))
        got_add = torch.addmm(bias.to("vk"), a[0].to("vk"), b[0].to("vk").t(), beta=0.5, alpha=2.0)
        got_lin = torch.nn.functional.linear(a.to("vk"), b[0].to("vk"), bias.to("vk"))  # [3,40,72] x [50,72]^T + bias
        got_badd = torch.baddbmm(bias.to("vk"), a.to("vk"), b.to("vk").transpose(1, 2), beta=0.5, alpha=2.0)
        out = torch.empty(0, dtype=dtype, device="vk")
        torch.mm(a[1].to("vk"), b[1].to("vk").t(), out=out)
        empty_k = torch.mm(a[0, :, :0].to("vk"), b[0, :, :0].to("vk").t())
    mag_t = a.float().abs() @ b.float().abs().transpose(1, 2)
    close(got_t, want(a, b.transpose(1, 2)), mag_t)
    close(out, want(a[1], b[1].t()), mag_t[1])
    close(got_add, (0.5 * bias.float() + 2.0 * (a[0].float() @ b[0].float().t())).to(dtype), 0.5 * bias.float().abs() + 2.0 * mag_t[0])
    close(got_badd, (0.5 * bias.float() + 2.0 * (a.float() @ b.float().transpose(1, 2))).to(dtype), 0.5 * bias.float().abs() + 2.0 * mag_t)
    close(got_lin, (a.float() @ b[0].float().t() + bias.float()).to(dtype), a.float().abs() @ b[0].float().abs().t() + bias.float().abs())
    assert empty_k.shape == (40, 50) and (empty_k.cpu() == 0).all()  # (k = 0: sums of nothing)
    assert tv.kernel_subgroup_size("gemmcm_bf16") == 64 and tv.kernel_subgroup_size("gemmcm_f16") == 64
    with pytest.raises(RuntimeError, match="cannot be multiplied"):
        torch.mm(a[0].to("vk"), b[0].to("vk"))
    with pytest.raises(RuntimeError, match="same dtype"):
        torch.mm(a[0].to("vk"), b[0].t().float().to("vk"))


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


@pytest.mark.parametrize("qdtype", [torch.quint8, torch.qint8, torch.qint32])
def test_quantized_per_tensor(tv, qdtype):
    """Legacy quantised tensors on vk as the reference tests them (tests/python/test_fallback_ops.py:986-1006):
    quantize_per_tensor, the getters, int_repr, dequantize, flip, clone and copies, bit for bit as the CPU's."""
    x = torch.cat([torch.randn(40, generator=gen(0)) * 20,
                   torch.tensor([float("nan"), float("inf"), -float("inf"), 0.05, 0.15, -0.05, 1e30, 3e9])]).view(6, 8)
    c = torch.quantize_per_tensor(x, 0.1, 5, qdtype)
    with on_gpu(tv):
        v = torch.quantize_per_tensor(x.to("vk"), 0.1, 5, qdtype)
        assert v.is_quantized and v.device.type == "vk" and v.dtype == qdtype
        assert (v.q_scale(), v.q_zero_point(), v.qscheme()) == (c.q_scale(), c.q_zero_point(), c.qscheme())
        ints, deq, flipped, cloned = v.int_repr(), v.dequantize(), v.flip((0, 1)), v.clone()
        t = torch.quantize_per_tensor(x.to("vk").t(), 0.1, 5, qdtype)  # a strided input
        by_tensor = torch.quantize_per_tensor(x.to("vk"), torch.tensor(0.1).to("vk"), torch.tensor(5).to("vk"), qdtype)
        e = torch._empty_affine_quantized([5, 5, 5, 5], scale=2, zero_point=3, dtype=qdtype, device="vk")
    assert torch.equal(ints.cpu(), c.int_repr()) and torch.equal(deq.cpu(), c.dequantize())
    assert torch.equal(flipped.int_repr().cpu(), c.flip((0, 1)).int_repr()) and torch.equal(cloned.int_repr().cpu(), c.int_repr())
    assert torch.equal(t.int_repr().cpu(), c.int_repr().t()) and torch.equal(by_tensor.int_repr().cpu(), c.int_repr())
    assert torch.equal(v.cpu().int_repr(), c.int_repr())
    back = c.to("vk")
    assert back.is_quantized and torch.equal(back.int_repr().cpu(), c.int_repr())
    assert e.flatten(0, -1).shape == (625,) and e.ravel().shape == (625,)
    with pytest.raises(RuntimeError, match="only works on Float"):
        torch.quantize_per_tensor(x.half().to("vk"), 0.1, 5, qdtype)


def test_fake_quantize_cachemask_ops(tv):
    """As the reference's test (tests/python/test_fallback_ops.py:972-984), plus float zero points and 16-bit inputs."""
    x = torch.tensor([[-1.3, 0.0, 0.26, 4.0], [float("nan"), float("inf"), -0.5, 1e-3]])
    v = lambda t: t.to("vk")
    sc, zp = torch.tensor([0.05]), torch.tensor([3], dtype=torch.int32)
    on = torch.ones(1, dtype=torch.long)
    f = torch.ops.aten._fake_quantize_per_tensor_affine_cachemask_tensor_qparams
    with on_gpu(tv):
        got = f(v(x), v(sc), v(zp), v(on), 0, 255)
        off = f(v(x), v(sc), v(zp), v(torch.zeros(1, dtype=torch.long)), 0, 255)
    for a, b in zip(got, f(x, sc, zp, on, 0, 255)):
        assert torch.equal(a.cpu().nan_to_num(), b.nan_to_num())
    assert torch.equal(off[0].cpu().nan_to_num(), x.nan_to_num()) and off[1].cpu().all()
    scs, zps = torch.tensor([0.05, 0.2]), torch.tensor([3, 250], dtype=torch.int32)
    g = torch.ops.aten.fake_quantize_per_channel_affine_cachemask
    big = torch.randn(2, 3, 500, generator=gen(4)) * 4
    for inp, axis, s, z in [(x, 0, scs, zps), (x, 0, scs, torch.tensor([3.25, 250.5])), (big, 1, torch.tensor([0.05, 0.2, 0.01]), torch.tensor([3, 250, 128], dtype=torch.int32)),
                            (big.bfloat16(), 2, torch.rand(500, generator=gen(5)) * 0.1 + 0.01, torch.randint(0, 255, (500,), dtype=torch.int32, generator=gen(6))),
                            (big.transpose(0, 2), 0, torch.rand(500, generator=gen(5)) * 0.1 + 0.01, torch.rand(500, generator=gen(7)) * 200)]:
        with on_gpu(tv):
            got = g(v(inp), v(s), v(z), axis, 0, 255)
        for a, b in zip(got, g(inp, s, z, axis, 0, 255)):
            assert a.shape == b.shape and torch.equal(a.cpu().float().nan_to_num(), b.float().nan_to_num())
    with on_gpu(tv):
        got = torch.fake_quantize_per_tensor_affine(v(big), 0.05, 3, 0, 255)
    assert torch.equal(got.cpu(), torch.fake_quantize_per_tensor_affine(big, 0.05, 3, 0, 255))
    with pytest.raises(RuntimeError, match="must be between"):
        g(v(x), v(scs), v(torch.tensor([3, 300], dtype=torch.int32)), 0, 0, 255)


@pytest.mark.parametrize("per_row", [False, True])
@pytest.mark.parametrize("symmetric", [False, True])
@pytest.mark.parametrize("qrange", [(0, 255), (-128, 127)])
def test_fused_moving_avg_obs_fake_quant(tv, per_row, symmetric, qrange):
    """The QAT observer and fake quantisation as the reference tests them (tests/python/test_fallback_ops.py:947-969):
    bit for bit as the CPU's over several steps (the running min / max start infinite, then move)."""
    g = gen(0)
    size = 4 if per_row else 1
    state = {d: [torch.full((size,), float("inf")), torch.full((size,), float("-inf")), torch.ones(size),
                 torch.zeros(size, dtype=torch.int32)] for d in ("cpu", "vk")}
    state["vk"] = [t.to("vk") for t in state["vk"]]
    for step in range(4):
        x = torch.randn(4, 3, 5, generator=g) * (0.1 + step) - 0.5 * step
        got = {}
        for d in ("cpu", "vk"):
            rmin, rmax, s, z = state[d]
            with (on_gpu(tv) if d == "vk" else contextlib.nullcontext()):
                out, mask = torch.ops.aten._fused_moving_avg_obs_fq_helper(
                    x.to(d), torch.tensor([1]).to(d), torch.tensor([1]).to(d), rmin, rmax, s, z, 0.01 if step == 3 else 0.25,
                    qrange[0], qrange[1], 0, per_row, symmetric)
            got[d] = [t.cpu() for t in (out, mask, rmin, rmax, s, z)]
        for a, b in zip(got["cpu"], got["vk"]):
            assert torch.equal(a, b)
