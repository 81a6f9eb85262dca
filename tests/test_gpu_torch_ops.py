"""The five quantised aten ops on device "vk", written as the reference's own tests are
(tests/python/test_quant.py): each op on "vk" against PyTorch's CPU result, with the
reference's `on_gpu()` assertion that nothing fell back to the CPU (tests/python/_util.py:28-35).
The C++ op layer (csrc/torch/quant.cpp) reaches the kernels through the C ABI."""
import contextlib

import pytest
import torch

pytestmark = pytest.mark.gpu
FLOAT8 = [torch.float8_e4m3fn, torch.float8_e5m2]
# bfloat16 / float8 results come off the fp8 matrix cores, whose products are added in a
# window ~14 bits below the largest (a hardware property); float32 / float16 results are exact sums
HW_WINDOW = 2.0**-13


@pytest.fixture(scope="module")
def tv():
    import torch_vulkan_amd.backend as tv
    assert tv.is_available() and (tv.capabilities() & 12) == 12  # 8- and 16-bit storage (test_quant.py:12)
    return tv


@contextlib.contextmanager
def on_gpu(tv):
    """Fails if anything inside falls back to the CPU."""
    before = tv.fallback_counts()
    yield
    after = tv.fallback_counts()
    new = {k: v - before.get(k, 0) for k, v in after.items() if v != before.get(k, 0)}
    assert not new, f"ran on the CPU: {new}"


def gen(seed):
    return torch.Generator().manual_seed(seed)


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


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(32, 64, 48), (1, 4096, 300), (5, 100, 17), (70, 33, 5), (65, 1, 66)])
def test_weight_int8pack_mm(tv, dtype, m, k, n):
    a = torch.randn(m, k, generator=gen(1)).to(dtype)
    b = torch.randint(-128, 128, (n, k), dtype=torch.int8, generator=gen(2))
    s = (torch.rand(n, generator=gen(3)) / 50).to(dtype)
    want = (a.float() @ (b.float() * s.float()[:, None]).t()).to(dtype)
    with on_gpu(tv):
        got = torch._weight_int8pack_mm(a.to("vk"), b.to("vk"), s.to("vk"))
        sliced = torch._weight_int8pack_mm(a.to("vk")[::2], b.to("vk"), s.to("vk"))
    mag = a.float().abs() @ (b.float() * s.float()[:, None]).abs().t()
    tol = torch.finfo(dtype).eps * want.float().abs() + 2**-20 * mag
    assert got.dtype == want.dtype and got.shape == want.shape and got.device.type == "vk"
    assert ((got.cpu().float() - want.float()).abs() <= tol).all()
    assert ((sliced.cpu().float() - want[::2].float()).abs() <= tol[::2]).all()


def test_weight_int8pack_mm_errors(tv):
    a, b, s = torch.randn(4, 8).to("vk"), torch.zeros(3, 8, dtype=torch.int8).to("vk"), torch.ones(3).to("vk")
    with pytest.raises(RuntimeError, match="expect B to be int8 tensor"):
        torch._weight_int8pack_mm(a, b.float(), s)
    with pytest.raises(RuntimeError, match="expect scales to be 1d tensor with size 3"):
        torch._weight_int8pack_mm(a, b, s[:2])
    with pytest.raises(RuntimeError, match="A must be contiguous on the last dimension"):
        torch._weight_int8pack_mm(a.t().contiguous().t(), b[:, :4], s)


def pack_case(n, k, bs, seed, bias):
    w = torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, generator=gen(seed))
    nb = 1 if bs == k else k // bs
    sc = torch.rand(n, nb, generator=gen(seed + 1)) / 10
    sc = sc if bs == k else sc.to(torch.bfloat16)
    return w, sc, (torch.randn(n, generator=gen(seed + 2)) if bias else None)


@pytest.mark.parametrize("m,k,n,bs,bias", [(1, 64, 4096, 32, False), (32, 128, 11008, 32, True), (5, 96, 70, 96, True),
                                           (3, 100, 9, 100, False), (4, 256, 16, 64, True), (9, 64, 33, 64, False)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dyn_quant_matmul_4bit_exact(tv, m, k, n, bs, bias, dtype):
    if dtype == torch.bfloat16 and bs != k:
        pytest.skip("bfloat16 inputs are channelwise only (the CPU's check)")
    w, sc, bvec = pack_case(n, k, bs, 7, bias)
    x = (torch.randn(m, k, generator=gen(11)) * 3).to(dtype)
    x[0, : k // 2] = 0.0
    if m > 1:
        x[1] = -x[1].abs()
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, bvec, bs, k, n)
    want = torch._dyn_quant_matmul_4bit(x, packed, bs, k, n)
    with on_gpu(tv):
        packed_vk = torch._dyn_quant_pack_4bit_weight(w.to("vk"), sc.to("vk"), None if bvec is None else bvec.to("vk"),
                                                      bs, k, n)
        got = torch._dyn_quant_matmul_4bit(x.to("vk"), packed_vk, bs, k, n)
        again = torch._dyn_quant_matmul_4bit(x.to("vk"), packed_vk, bs, k, n)  # (the cached side-car)
        got_cpu_packed = torch._dyn_quant_matmul_4bit(x.to("vk"), packed.to("vk"), bs, k, n)
    assert torch.equal(packed_vk.cpu(), packed)
    assert got.dtype == want.dtype
    assert torch.equal(got.cpu(), want) and torch.equal(again.cpu(), want)
    assert torch.equal(got_cpu_packed.cpu(), want)


def test_dyn_quant_sidecar_follows_writes(tv):
    """The cached side-car is keyed by the packed tensor's version: an in-place change of the
    packed weights must show in the next product."""
    w, sc, _ = pack_case(16, 64, 32, 3, False)
    x = torch.randn(2, 64, generator=gen(5))
    packed = torch._dyn_quant_pack_4bit_weight(w, sc, None, 32, 64, 16)
    pv = packed.to("vk")
    first = torch._dyn_quant_matmul_4bit(x.to("vk"), pv, 32, 64, 16).cpu()
    packed2 = packed.clone()
    packed2[: 16 * 32] = 255.0 - packed2[: 16 * 32]
    pv.copy_(packed2)
    second = torch._dyn_quant_matmul_4bit(x.to("vk"), pv, 32, 64, 16).cpu()
    assert torch.equal(first, torch._dyn_quant_matmul_4bit(x, packed, 32, 64, 16))
    assert torch.equal(second, torch._dyn_quant_matmul_4bit(x, packed2, 32, 64, 16))


def test_dyn_quant_errors(tv):
    x = torch.randn(2, 64).to("vk")
    w, sc, _ = pack_case(8, 64, 32, 3, False)
    with pytest.raises(RuntimeError, match="Group size should be multiple of 32"):
        torch._dyn_quant_pack_4bit_weight(w.to("vk"), sc.to("vk"), None, 48, 64, 8)
    with pytest.raises(RuntimeError, match="expect weight to be kByte"):
        torch._dyn_quant_pack_4bit_weight(w.to(torch.int8).to("vk"), sc.to("vk"), None, 32, 64, 8)
    packed = torch._dyn_quant_pack_4bit_weight(w.to("vk"), sc.to("vk"), None, 32, 64, 8)
    with pytest.raises(RuntimeError, match="expect input to be float32 or bfloat16 tensor"):
        torch._dyn_quant_matmul_4bit(x.cpu().bfloat16().to("vk"), packed, 32, 64, 8)
    with pytest.raises(RuntimeError, match="Invalid packed weight tensor size"):
        torch._dyn_quant_matmul_4bit(x, packed[:100], 32, 64, 8)


@pytest.mark.parametrize("fa,fb", [(FLOAT8[0], FLOAT8[0]), (FLOAT8[1], FLOAT8[0]), (FLOAT8[0], FLOAT8[1])])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32, torch.float16, torch.float8_e4m3fn, None])
@pytest.mark.parametrize("rowwise", [False, True])
def test_scaled_mm(tv, fa, fb, out_dtype, rowwise):
    a = torch.randn(16, 32, generator=gen(1)).to(fa)
    b = torch.randn(48, 32, generator=gen(2)).to(fb).t()
    sa = torch.rand(16, 1, generator=gen(3)) + 0.5 if rowwise else torch.tensor(1.25)
    sb = torch.rand(1, 48, generator=gen(4)) + 0.5 if rowwise else torch.tensor(0.75)
    bias = torch.randn(48, generator=gen(5)).to(torch.bfloat16) if out_dtype == torch.bfloat16 else None
    scale_result = torch.tensor(2.0) if out_dtype == torch.float8_e4m3fn else None
    kw = dict(bias=bias, out_dtype=out_dtype, scale_result=scale_result)
    res_dtype = out_dtype or fa
    if rowwise:  # torch 2.10's CPU kernel takes per-tensor scales only: the closed form it emulates
        want = (a.float() * sa) @ (b.float() * sb)
        want = want + bias.float() if bias is not None else want
        want = (want * 0.5 if scale_result is not None else want).to(res_dtype)
    else:
        want = torch._scaled_mm(a, b, sa, sb, **kw)
    vkw = {k: (v.to("vk") if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
    with on_gpu(tv):
        got = torch._scaled_mm(a.to("vk"), b.to("vk"), sa.to("vk"), sb.to("vk"), **vkw)
        out = torch.empty(0, dtype=want.dtype).to("vk")
        torch._scaled_mm(a.to("vk"), b.to("vk"), sa.to("vk"), sb.to("vk"), **vkw, out=out)
    assert got.dtype == want.dtype and got.shape == want.shape
    mag = (a.float() * sa).abs() @ (b.float() * sb).abs() / (2.0 if scale_result is not None else 1.0)
    eps = torch.finfo(want.dtype).eps
    tol = eps * want.float().abs() + 2**-20 * mag
    if want.dtype not in (torch.float32, torch.float16):
        tol = tol + HW_WINDOW * mag
    for res in (got, out):
        assert ((res.cpu().float() - want.float()).abs() <= tol).all()


def test_scaled_mm_errors(tv):
    a = torch.randn(4, 8).to(FLOAT8[0]).to("vk")
    b = torch.randn(6, 8).to(FLOAT8[0]).to("vk").t()
    one = torch.tensor(1.0).to("vk")
    with pytest.raises(ValueError, match="Invalid scaling configuration"):
        torch._scaled_mm(a, b, torch.ones(3).to("vk"), one)
    with pytest.raises(ValueError, match="out_dtype must match output matrix type"):
        torch._scaled_mm(a, b, one, one, out_dtype=torch.float32, out=torch.empty(0, dtype=torch.half).to("vk"))
    with pytest.raises(RuntimeError, match="Bias must be size 6"):
        torch._scaled_mm(a, b, one, one, bias=torch.ones(5).to("vk"), out_dtype=torch.float32)


def test_empty_inputs(tv):
    """No rows: every op of the path returns an empty result of the right shape and type (and launches nothing wrong)."""
    with on_gpu(tv):
        b = torch.randint(-128, 128, (5, 64), dtype=torch.int8, generator=gen(1)).to("vk")
        out = torch._weight_int8pack_mm(torch.zeros(0, 64, dtype=torch.bfloat16).to("vk"), b, torch.ones(5, dtype=torch.bfloat16).to("vk"))
        assert out.shape == (0, 5) and out.dtype == torch.bfloat16
        w, sc, bias = pack_case(6, 64, 32, 3, True)
        packed = torch._dyn_quant_pack_4bit_weight(w, sc, bias, 32, 64, 6).to("vk")
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
