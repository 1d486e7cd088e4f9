"""GPU parity of the fake-quant kernels and the QAT modules against the CPU oracle (bit-exact values and qparams)."""
import pytest
import torch
from torch import nn

from oracle import fake_quant_oracle as fq
from tests.helpers import bits_equal
from torchtune_amd import ops
from torchtune_amd.qat import (
    FakeQuantizeConfig,
    FakeQuantizer,
    Int8DynActInt4WeightLinear,
    Int8DynActInt4WeightQATLinear,
    Int8DynActInt4WeightQATQuantizer,
)
from torchtune_amd.training import quantization

pytestmark = pytest.mark.gpu
DEV = "cuda"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,K", [(1, 8), (5, 24), (64, 4096), (9, 4104), (5, 8192), (7, 14336), (3, 28672), (6, 32768), (4, 40000), (130, 512)])
def test_per_token_bit_exact(dtype, rows, K):
    g = torch.Generator().manual_seed(rows * 1000 + K)
    x = (torch.randn(rows, K, generator=g) * 1.7).to(dtype)
    if rows > 4:
        x[1] = 0
        x[2] = x[2].abs()
        x[3] = -x[3].abs()
        x[4, ::2] *= 50
    want, ws, wz = fq.fq_per_token_int8_asym(x)
    got, gs, gz = ops.fq_per_token_int8_asym(x.to(DEV))
    assert bits_equal(got.cpu(), want) and torch.equal(gs.cpu(), ws) and torch.equal(gz.cpu(), wz)
    out_only, s_none, z_none = ops.fq_per_token_int8_asym(x.to(DEV), want_qparams=False)
    assert s_none is None and z_none is None and bits_equal(out_only.cpu(), want)


def test_per_token_keeps_leading_dimensions():
    x = torch.randn(2, 3, 64, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16)
    got, s, z = ops.fq_per_token_int8_asym(x.to(DEV))
    want, ws, wz = fq.fq_per_token_int8_asym(x.view(6, 64))
    assert got.shape == x.shape and s.shape == (6,) and bits_equal(got.cpu().view(6, 64), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("g", [8, 16, 32, 64, 256, 512])
def test_per_group_and_convert_bit_exact(dtype, g):
    gen = torch.Generator().manual_seed(g)
    w = (torch.randn(96, 1024, generator=gen) * 0.02).to(dtype)
    w[0, :g] = 0
    w[1, :g] = 7.5 * 0.01
    want, ws = fq.fq_per_group_int4_sym(w, g)
    got, gs = ops.fq_per_group_int4_sym(w.to(DEV), g)
    assert bits_equal(got.cpu(), want) and torch.equal(gs.cpu(), ws)
    wq, ws2, wz = fq.quantize_per_group_int4(w, g)
    gq, gs2, gz = ops.quantize_per_group_int4(w.to(DEV), g)
    assert gq.dtype == torch.int8 and torch.equal(gq.cpu(), wq) and torch.equal(gs2.cpu(), ws2) and torch.equal(gz.cpu(), wz)


def test_ragged_tail_of_the_last_workgroup():
    # 3 x 40 elements with groups of 8: 15 chunks, far less than one workgroup's 1024
    w = (torch.randn(3, 40, generator=torch.Generator().manual_seed(1)) * 0.1).to(torch.bfloat16)
    want, ws = fq.fq_per_group_int4_sym(w, 8)
    got, gs = ops.fq_per_group_int4_sym(w.to(DEV), 8)
    assert bits_equal(got.cpu(), want) and torch.equal(gs.cpu(), ws)


def test_fake_quantizer_modules_and_straight_through_gradient():
    act = FakeQuantizer(FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False))
    wgt = FakeQuantizer(FakeQuantizeConfig(torch.int4, group_size=32))
    x = torch.randn(4, 8, 128, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    xd = x.to(DEV).requires_grad_()
    y = act(xd)
    want, ws, wz = fq.fq_per_token_int8_asym(x.view(-1, 128))
    assert bits_equal(y.detach().cpu().view(-1, 128), want)
    assert torch.equal(act.scale.cpu(), ws) and torch.equal(act.zero_point.cpu(), wz) and act.zero_point.dtype == torch.int32
    gy = torch.randn_like(y)
    y.backward(gy)
    assert torch.equal(xd.grad, gy)  # dy/dx = 1
    act.enabled = False
    assert act(xd) is xd
    w = (torch.randn(64, 128, generator=torch.Generator().manual_seed(3)) * 0.02).to(torch.bfloat16)
    assert bits_equal(wgt(w.to(DEV)).cpu(), fq.fq_per_group_int4_sym(w, 32)[0])
    assert torch.equal(wgt.scale.cpu(), fq.fq_per_group_int4_sym(w, 32)[1]) and wgt.zero_point is None


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_qat_linear_forward_backward_vs_oracle(dtype):
    gen = torch.Generator().manual_seed(4)
    N, K, M, g = 256, 512, 96, 32
    w = (torch.randn(N, K, generator=gen) * 0.02).to(dtype)
    x = torch.randn(M, K, generator=gen).to(dtype)
    lin = Int8DynActInt4WeightQATLinear(K, N, bias=False, device=DEV, groupsize=g, precision=dtype)
    with torch.no_grad():
        lin.weight.copy_(w)
    xd = x.to(DEV).requires_grad_()
    y = lin(xd)
    (y.float() ** 2).sum().backward()
    xo, wo = x.clone().requires_grad_(), w.clone().requires_grad_()
    yo = fq.fake_quantized_linear(xo, wo, g)
    (yo.float() ** 2).sum().backward()
    tol = dict(rtol=1e-2, atol=1e-2) if dtype == torch.bfloat16 else dict(rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(y.detach().cpu().float(), yo.detach().float(), **tol)
    torch.testing.assert_close(xd.grad.cpu().float(), xo.grad.float(), **tol)
    gw, gwo = lin.weight.grad.cpu().float(), wo.grad.float()
    torch.testing.assert_close(gw, gwo, rtol=2e-2, atol=2e-2 * float(gwo.abs().max()))
    # toggles of torchtune/training/quantization.py:56-71
    lin.apply(quantization._get_disable_fake_quant("8da4w-qat"))
    torch.testing.assert_close(lin(xd).detach().cpu().float(), (x.float() @ w.float().T), **(tol if dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)))
    lin.apply(quantization._get_enable_fake_quant("8da4w-qat"))
    assert lin.weight_fake_quantizer.enabled and lin.activation_fake_quantizer.enabled


def test_prepare_then_convert_is_bit_exact_and_consistent():
    gen = torch.Generator().manual_seed(5)
    model = nn.Sequential(nn.Linear(256, 512, bias=False), nn.Sequential(nn.Linear(512, 128, bias=True))).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        for p in model.parameters():
            p.copy_((torch.randn(p.shape, generator=gen) * 0.05).to(torch.bfloat16))
    w0 = model[0].weight.detach().cpu().clone()
    w1 = model[1][0].weight.detach().cpu().clone()
    qz = Int8DynActInt4WeightQATQuantizer(groupsize=32, precision=torch.bfloat16)
    model = qz.prepare(model)
    x = torch.randn(10, 256, generator=gen).to(torch.bfloat16).to(DEV)
    y_fake = model(x)
    model = qz.convert(model)
    c0, c1 = model[0], model[1][0]
    assert isinstance(c0, Int8DynActInt4WeightLinear) and isinstance(c1, Int8DynActInt4WeightLinear)
    for conv, w in ((c0, w0), (c1, w1)):
        q, s, z = fq.quantize_per_group_int4(w, 32)
        assert conv.weight.dtype == torch.int8 and torch.equal(conv.weight.cpu(), q)
        assert int(conv.weight.min()) >= -8 and int(conv.weight.max()) <= 7
        assert torch.equal(conv.scales.cpu(), s) and torch.equal(conv.zeros.cpu(), z) and conv.scales.shape == (w.shape[0], w.shape[1] // 32)
    # the converted model computes what the fake-quantised model computed
    torch.testing.assert_close(model(x).float(), y_fake.float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("g", [8, 32, 256])
def test_converted_weight_dequantises_to_the_fake_quantised_weight(dtype, g):
    """dequantise(convert(W)) must be bit-identical to fake_quantise(W): that is what makes the converted model compute
    what the fake-quantised model trained with; also with non-zero zero points against the eager formula."""
    gen = torch.Generator().manual_seed(9)
    w = (torch.randn(96, 512, generator=gen) * 0.1).to(dtype)
    fq_w, _ = fq.fq_per_group_int4_sym(w, g)
    q, s, z = fq.quantize_per_group_int4(w, g)
    got = ops.dequantize_per_group_int4(q.to(DEV), s.to(DEV), z.to(DEV), g, dtype)
    assert bits_equal(got.cpu(), fq_w)
    assert bits_equal(ops.dequantize_per_group_int4(q.to(DEV), s.to(DEV), None, g, dtype).cpu(), fq_w)
    zz = torch.randint(-3, 4, z.shape, generator=gen).float()
    want = ((q.view(96, -1, g).float() - zz[:, :, None]) * s[:, :, None]).to(dtype).view(96, 512)
    assert bits_equal(ops.dequantize_per_group_int4(q.to(DEV), s.to(DEV), zz.to(DEV), g, dtype).cpu(), want)


# ---- weight-only int4 ("4w-qat") -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype,qp", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16), (torch.float32, torch.float32)])
@pytest.mark.parametrize("g", [8, 32, 64, 128, 256, 512])
def test_uint4_asym_fake_quant_convert_and_dequant_bit_exact(dtype, qp, g):
    gen = torch.Generator().manual_seed(100 + g)
    w = (torch.randn(96, 1024, generator=gen) * 0.02 + 0.003).to(dtype)
    w[0, :g] = 0.25          # constant group: the 1e-6 floor of the scale
    w[1, :g] = w[1, :g].abs() + 1.0  # all-positive group far from zero
    w[2, :g] *= 1e-5         # tiny dynamic range
    w[3, :g] = 1.0           # a range of one bf16 ulp next to 1.0: the rounded zero point pushes offsets far
    w[3, 1] = 1.0078125      # beyond 15 steps (they clamp)
    w[4, :g] = w[4, :g] * 3e3 - 7e4  # large magnitudes, range much smaller than the offset
    want, ws, wz = fq.fq_per_group_uint4_asym(w, g, qp)
    got, gs, gz = ops.fq_per_group_uint4_asym(w.to(DEV), g, qp)
    assert bits_equal(got.cpu(), want)
    assert bits_equal(gs.cpu(), ws.float()) and bits_equal(gz.cpu(), wz.float())
    only, s_none, z_none = ops.fq_per_group_uint4_asym(w.to(DEV), g, qp, want_qparams=False)
    assert s_none is None and z_none is None and bits_equal(only.cpu(), want)
    wq, ws2, wz2 = fq.quantize_per_group_uint4(w, g, qp)
    gq, gs2, gz2 = ops.quantize_per_group_uint4(w.to(DEV), g, qp)
    assert gq.dtype == torch.uint8 and gq.shape == (96, 512) and torch.equal(gq.cpu(), wq)
    assert bits_equal(gs2.cpu(), ws2.float()) and bits_equal(gz2.cpu(), wz2.float())
    dense = ops.dequantize_per_group_uint4(gq, gs2, gz2, g, dtype)
    assert bits_equal(dense.cpu(), want)  # the converted weight is exactly what training saw


def test_uint4_asym_ragged_tail_and_validation():
    # a chunk count that does not fill the last workgroup, and leading dimensions
    w = torch.randn(3, 5, 64, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    got, s, z = ops.fq_per_group_uint4_asym(w.to(DEV), 32)
    want, ws, wz = fq.fq_per_group_uint4_asym(w.view(15, 64), 32)
    assert got.shape == w.shape and s.shape == (15, 2) and bits_equal(got.cpu().view(15, 64), want)
    with pytest.raises(ValueError, match="divisible by group_size"):
        ops.fq_per_group_uint4_asym(torch.zeros(4, 48, device=DEV), 32)
    with pytest.raises(ValueError, match="power of two"):
        ops.quantize_per_group_uint4(torch.zeros(4, 48, device=DEV), 24)
    with pytest.raises(TypeError):
        ops.dequantize_per_group_uint4(torch.zeros(4, 24, dtype=torch.int8, device=DEV), torch.ones(4, 1), torch.ones(4, 1), 48, torch.bfloat16)


def test_weight_only_int4_qat_prepare_train_convert():
    """Int4WeightOnlyQATQuantizer end to end: the prepared layer computes F.linear(x, fq(W)) with straight-through
    gradients; the converted layer reproduces the same output from packed codes and bf16 scales_and_zeros."""
    from torchtune_amd.qat import Int4WeightOnlyQATLinear, Int4WeightOnlyQATQuantizer, WeightOnlyInt4Linear

    gen = torch.Generator().manual_seed(21)
    K, N, g = 512, 192, 64
    W = (torch.randn(N, K, generator=gen) * 0.05).to(torch.bfloat16)
    x = torch.randn(4, 33, K, generator=gen).to(torch.bfloat16)
    model = nn.Sequential(nn.Linear(K, N, bias=False)).to(torch.bfloat16)
    with torch.no_grad():
        model[0].weight.copy_(W)
    model = model.to(DEV)
    qz = Int4WeightOnlyQATQuantizer(groupsize=g)
    model = qz.prepare(model)
    layer = model[0]
    assert isinstance(layer, Int4WeightOnlyQATLinear)
    xd = x.to(DEV).requires_grad_(True)
    y = layer(xd)
    w_fq, ws, wz = fq.fq_per_group_uint4_asym(W, g)
    torch.testing.assert_close(y.float().cpu(), (x.float() @ w_fq.float().T), rtol=1e-2, atol=1e-2)
    assert bits_equal(layer.weight_fake_quantizer.scale.cpu(), ws) and bits_equal(layer.weight_fake_quantizer.zero_point.cpu(), wz)
    gy = torch.randn(y.shape, generator=gen).to(torch.bfloat16)
    y.backward(gy.to(DEV))
    # straight-through: the weight gradient is gy^T x, the input gradient goes through the fake-quantised weight
    torch.testing.assert_close(layer.weight.grad.float().cpu(), gy.float().view(-1, N).T @ x.float().view(-1, K), rtol=1e-2, atol=2e-2)
    torch.testing.assert_close(xd.grad.float().cpu(), gy.float() @ w_fq.float(), rtol=1e-2, atol=1e-2)
    y_ref = y.detach()
    model = qz.convert(model)
    conv = model[0]
    assert isinstance(conv, WeightOnlyInt4Linear) and conv.weight.dtype == torch.uint8 and conv.weight.shape == (N, K // 2)
    wq, _, _ = fq.quantize_per_group_uint4(W, g)
    assert torch.equal(conv.weight.cpu(), wq)
    assert bits_equal(conv.scales_and_zeros[..., 0].t().contiguous().cpu(), ws)
    assert bits_equal(conv.scales_and_zeros[..., 1].t().contiguous().cpu(), wz)
    assert bits_equal(conv.dense_weight().cpu(), w_fq)
    assert bits_equal(conv(x.to(DEV)), y_ref)
    sd = conv.state_dict()
    assert set(sd) == {"weight", "scales_and_zeros"}


def test_post_training_quantizers_use_the_convert_arithmetic():
    """Int8DynActInt4WeightQuantizer / Int4WeightOnlyQuantizer `.quantize(model)` (torchtune/training/quantization.py:79-121,
    what recipes/quantize.py:94 calls for the non-QAT modes) give the layers that QAT `convert` gives for the same weights."""
    from torchtune_amd.qat import Int4WeightOnlyQATQuantizer, WeightOnlyInt4Linear

    gen = torch.Generator().manual_seed(33)
    K, N = 512, 128
    W = (torch.randn(N, K, generator=gen) * 0.03).to(torch.bfloat16)
    b = (torch.randn(N, generator=gen) * 0.1).to(torch.bfloat16)
    x = torch.randn(5, K, generator=gen).to(torch.bfloat16).to(DEV)

    def fresh(bias):
        m = nn.Sequential(nn.Linear(K, N, bias=bias), nn.ReLU(), nn.Sequential(nn.Linear(N, 128, bias=False))).to(torch.bfloat16)
        with torch.no_grad():
            m[0].weight.copy_(W)
            if bias:
                m[0].bias.copy_(b)
        return m.to(DEV)

    ptq = quantization.Int8DynActInt4WeightQuantizer(groupsize=32).quantize(fresh(True))
    assert isinstance(ptq[0], Int8DynActInt4WeightLinear) and isinstance(ptq[2][0], Int8DynActInt4WeightLinear)
    qz = Int8DynActInt4WeightQATQuantizer(groupsize=32, precision=torch.bfloat16)
    qat = qz.convert(qz.prepare(fresh(True)))
    assert torch.equal(ptq[0].weight, qat[0].weight) and torch.equal(ptq[0].scales, qat[0].scales)
    assert bits_equal(ptq[0](x), qat[0](x))  # (the second layer is randomly initialised per model)
    wq, ws, _ = fq.quantize_per_group_int4(W, 32)
    assert torch.equal(ptq[0].weight.cpu(), wq) and torch.equal(ptq[0].scales.cpu(), ws)

    ptq4 = quantization.Int4WeightOnlyQuantizer(groupsize=64).quantize(fresh(True))
    assert isinstance(ptq4[0], WeightOnlyInt4Linear) and ptq4[0].bias is not None
    q4 = Int4WeightOnlyQATQuantizer(groupsize=64)
    qat4 = q4.convert(q4.prepare(fresh(False)))
    assert torch.equal(ptq4[0].weight, qat4[0].weight) and bits_equal(ptq4[0].scales_and_zeros, qat4[0].scales_and_zeros)
    w_fq, _, _ = fq.fq_per_group_uint4_asym(W, 64)
    torch.testing.assert_close(ptq4[0](x).float().cpu(), x.float().cpu() @ w_fq.float().T + b.float(), rtol=1e-2, atol=1e-2)
    with pytest.raises(ValueError, match="divisible by groupsize"):
        quantization.Int8DynActInt4WeightQuantizer(groupsize=256).quantize(nn.Sequential(nn.Linear(96, 8)).to(DEV))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_bf16_scale_precision_bit_exact(dtype):
    """scale_precision = bfloat16 (the QAT benchmark configuration asks for bf16 scales; the reference's default is float32): the scale
    is rounded to bf16 once chosen and the rounded scale quantises and dequantises, in the per-token, the per-group and
    the convert kernels, and the converted layer reproduces the fake-quantised one."""
    gen = torch.Generator().manual_seed(41)
    x = (torch.randn(37, 1024, generator=gen) * 1.9).to(dtype)
    x[1] = 0
    want, ws, wz = fq.fq_per_token_int8_asym(x, torch.bfloat16)
    got, gs, gz = ops.fq_per_token_int8_asym(x.to(DEV), qparam_dtype=torch.bfloat16)
    assert bits_equal(got.cpu(), want) and torch.equal(gs.cpu(), ws) and torch.equal(gz.cpu(), wz)
    long_row = (torch.randn(3, 40000, generator=gen) * 1.1).to(dtype)  # the streaming variant of the kernel
    want, ws, _ = fq.fq_per_token_int8_asym(long_row, torch.bfloat16)
    got, gs, _ = ops.fq_per_token_int8_asym(long_row.to(DEV), qparam_dtype=torch.bfloat16)
    assert bits_equal(got.cpu(), want) and torch.equal(gs.cpu(), ws)
    w = (torch.randn(64, 1024, generator=gen) * 0.02).to(dtype)
    for g in (32, 256):
        want, ws = fq.fq_per_group_int4_sym(w, g, torch.bfloat16)
        got, gs = ops.fq_per_group_int4_sym(w.to(DEV), g, qparam_dtype=torch.bfloat16)
        assert bits_equal(got.cpu(), want) and torch.equal(gs.cpu(), ws)
        wq, ws2, _ = fq.quantize_per_group_int4(w, g, torch.bfloat16)
        gq, gs2, _ = ops.quantize_per_group_int4(w.to(DEV), g, torch.bfloat16)
        assert torch.equal(gq.cpu(), wq) and torch.equal(gs2.cpu(), ws2)
    # module level: prepare -> forward -> convert with bf16 scales
    lin = nn.Sequential(nn.Linear(1024, 64, bias=False)).to(dtype)
    with torch.no_grad():
        lin[0].weight.copy_(w)
    lin = lin.to(DEV)
    qz = Int8DynActInt4WeightQATQuantizer(groupsize=32, precision=dtype, scales_precision=torch.bfloat16)
    lin = qz.prepare(lin)
    xd = x.to(DEV)
    y_fq = lin(xd)
    x_fq, _, _ = fq.fq_per_token_int8_asym(x, torch.bfloat16)
    w_fq, w_s = fq.fq_per_group_int4_sym(w, 32, torch.bfloat16)
    torch.testing.assert_close(y_fq.float().cpu(), x_fq.float() @ w_fq.float().T, rtol=1e-2, atol=1e-2)
    assert lin[0].weight_fake_quantizer.scale.dtype == torch.bfloat16
    assert torch.equal(lin[0].weight_fake_quantizer.scale.float().cpu(), w_s)
    conv = qz.convert(lin)
    assert conv[0].scales.dtype == torch.bfloat16 and torch.equal(conv[0].scales.float().cpu(), w_s)
    assert bits_equal(conv(xd), y_fq)  # the converted layer computes what training saw


def test_qat_lora_linear_forward_backward_and_frozen_weight_cache():
    """QATLoRALinear (torchtune/modules/peft/lora.py:150-306) with both fake quantisers on the GPU:
    y = F.linear(fq(x), fq(W)) + (alpha / r) B A x against the oracle's fake quantisation; gradients reach x and the
    adapters only.  The fake-quantised frozen weight is built once and rebuilt after the weight is written."""
    from torchtune_amd.modules.peft import LoRALinear, QATLoRALinear

    gen = torch.Generator().manual_seed(77)
    K, N, r, alpha, g = 256, 192, 8, 16.0, 32
    W = (torch.randn(N, K, generator=gen) * 0.05).to(torch.bfloat16)
    A = (torch.randn(r, K, generator=gen) * 0.05).to(torch.bfloat16)
    B = (torch.randn(N, r, generator=gen) * 0.05).to(torch.bfloat16)
    x = torch.randn(3, 17, K, generator=gen).to(torch.bfloat16)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(DEV):
            base = LoRALinear(K, N, rank=r, alpha=alpha)
    finally:
        torch.set_default_dtype(prev)
    with torch.no_grad():
        base.weight.copy_(W.to(DEV))
        base.lora_a.weight.copy_(A.to(DEV))
        base.lora_b.weight.copy_(B.to(DEV))
    layer = QATLoRALinear.from_lora_linear(
        base, FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False), FakeQuantizeConfig(torch.int4, group_size=g))
    layer.weight.requires_grad_(False)
    xd = x.to(DEV).requires_grad_()

    def expected(Wc):
        x_fq, _, _ = fq.fq_per_token_int8_asym(x.view(-1, K))
        w_fq, _ = fq.fq_per_group_int4_sym(Wc, g)
        out = x_fq.float() @ w_fq.float().T + (alpha / r) * ((x.view(-1, K).float() @ A.float().T) @ B.float().T)
        return out.view(3, 17, N), w_fq

    want, w_fq = expected(W)
    launches = []
    ops.set_fq_timer(lambda kind, *a: launches.append(kind))  # counts launches; returning None records no events
    try:
        y = layer(xd)
        y2 = layer(xd)
        # the weight side ran once; so did the activation side: the second forward got the same, unmodified tensor
        assert launches.count("per_group") == 1 and launches.count("per_token") == 1
        torch.testing.assert_close(y.float().cpu(), want, rtol=2e-2, atol=2e-2)
        assert bits_equal(y, y2)
        y.float().sum().backward()
        assert xd.grad is not None and layer.lora_a.weight.grad is not None and layer.lora_b.weight.grad is not None
        assert layer.weight.grad is None
        torch.testing.assert_close(xd.grad.float().cpu().view(-1, K)[0],
                                   (w_fq.float().sum(0) + (alpha / r) * (B.float().sum(0) @ A.float())), rtol=2e-2, atol=2e-2)
        # writing the weight invalidates the cached fake-quantised copy
        W2 = (W.float() * 1.5).to(torch.bfloat16)
        with torch.no_grad():
            layer.weight.copy_(W2.to(DEV))
        y3 = layer(xd)
        assert launches.count("per_group") == 2
        torch.testing.assert_close(y3.float().cpu(), expected(W2)[0], rtol=2e-2, atol=2e-2)
        # a trainable base weight is never cached (its gradient must flow through the straight-through estimator)
        layer.weight.requires_grad_(True)
        layer(xd).float().sum().backward()
        assert layer.weight.grad is not None and launches.count("per_group") == 3
    finally:
        ops.set_fq_timer(None)


def test_qat_lora_linear_on_the_tiled_gemm_many_tokens():
    """QATLoRALinear.forward (torchtune/modules/peft/lora.py:248-264) at a training size: the frozen weight's fake
    quantisation held in the GEMM's tile order, base product and adapter from one launch per direction
    (``ttamd_tiled_lora_linear_bf16``).  Compared with the layer's eager composition (``TILED_GEMM = False``: F.linear on
    the row-major fake-quantised weight plus the adapter's two matmuls) and with the oracle's fake quantisation in fp32:
    output, grad-input and adapter gradients (rtol 1e-2 / atol scaled with the magnitude of the result, the bar of the
    other GEMM tests); the tiles are rebuilt when the weight is written."""
    from torchtune_amd.modules.peft import LoRALinear, QATLoRALinear

    gen = torch.Generator().manual_seed(3)
    K, N, r, alpha, g, M = 2048, 2048, 16, 32.0, 32, 8192 + 64   # 33 x 8 = 264 tiles of 256 x 256 in both directions
    W = (torch.randn(N, K, generator=gen) * 0.02).to(torch.bfloat16)
    A = (torch.randn(r, K, generator=gen) * 0.02).to(torch.bfloat16)
    B = (torch.randn(N, r, generator=gen) * 0.02).to(torch.bfloat16)
    x = torch.randn(M, K, generator=gen).to(torch.bfloat16)
    gy = (torch.randn(M, N, generator=gen) * 0.1).to(torch.bfloat16)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device(DEV):
            base = LoRALinear(K, N, rank=r, alpha=alpha)
    finally:
        torch.set_default_dtype(prev)
    with torch.no_grad():
        base.weight.copy_(W.to(DEV))
        base.lora_a.weight.copy_(A.to(DEV))
        base.lora_b.weight.copy_(B.to(DEV))
    layer = QATLoRALinear.from_lora_linear(
        base, FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False), FakeQuantizeConfig(torch.int4, group_size=g))
    layer.weight.requires_grad_(False)

    def run(tiled):
        layer.TILED_GEMM = tiled
        layer.zero_grad()
        xd = x.to(DEV).requires_grad_()
        assert layer._tiled_ok(xd) == tiled
        y = layer(xd)
        y.backward(gy.to(DEV))
        return y.detach(), xd.grad, layer.lora_a.weight.grad.clone(), layer.lora_b.weight.grad.clone()

    try:
        y1, gx1, ga1, gb1 = run(True)
        y0, gx0, ga0, gb0 = run(False)
    finally:
        layer.TILED_GEMM = True
    assert layer.weight.grad is None
    for a, b in ((y1, y0), (gx1, gx0), (ga1, ga0), (gb1, gb0)):
        torch.testing.assert_close(a.float(), b.float(), rtol=1e-2, atol=1e-2 * max(1.0, float(b.float().abs().max()) / 8))
    # the oracle's fake quantisation, products in fp32 (row blocks keep the CPU work small)
    rows = slice(0, 512)
    x_fq, _, _ = fq.fq_per_token_int8_asym(x[rows])
    w_fq, w_scale = fq.fq_per_group_int4_sym(W, g)
    want = x_fq.float() @ w_fq.float().T + (alpha / r) * ((x[rows].float() @ A.float().T) @ B.float().T)
    torch.testing.assert_close(y1[rows].float().cpu(), want, rtol=1e-2, atol=1e-2)
    want_gx = gy[rows].float() @ w_fq.float() + (alpha / r) * ((gy[rows].float() @ B.float()) @ A.float())
    torch.testing.assert_close(gx1[rows].float().cpu(), want_gx, rtol=1e-2, atol=1e-2 * max(1.0, float(want_gx.abs().max()) / 8))
    assert torch.equal(layer.weight_fake_quantizer.scale.float().cpu(), w_scale)
    # writing the weight rebuilds the tiles
    with torch.no_grad():
        layer.weight.copy_((W.float() * 1.5).to(torch.bfloat16).to(DEV))
    y2 = layer(x.to(DEV))
    w2_fq, _ = fq.fq_per_group_int4_sym((W.float() * 1.5).to(torch.bfloat16), g)
    want2 = x_fq.float() @ w2_fq.float().T + (alpha / r) * ((x[rows].float() @ A.float().T) @ B.float().T)
    torch.testing.assert_close(y2[rows].float().cpu(), want2, rtol=1e-2, atol=1e-2)


def test_per_token_result_is_shared_between_sibling_quantizers(monkeypatch):
    """q/k/v (and gate/up) fake-quantise the same activation tensor: the second and third quantizer reuse the first
    one's result while the very same, unmodified tensor object comes in; a modified or different tensor is recomputed;
    results equal the unshared ones bit for bit and every quantizer still records its own scale / zero point."""
    from torchtune_amd import ops
    from torchtune_amd.qat import FakeQuantizeConfig, FakeQuantizer, PerToken

    calls = []
    real = ops.fq_per_token_int8_asym

    def counting(*a, **kw):
        calls.append(1)
        return real(*a, **kw)

    monkeypatch.setattr(ops, "fq_per_token_int8_asym", counting)
    cfg = FakeQuantizeConfig(torch.int8, PerToken(), is_symmetric=False)
    qs = [FakeQuantizer(cfg) for _ in range(3)]
    g = torch.Generator(device="cuda").manual_seed(12)
    x = torch.randn(64, 512, device="cuda", generator=g).to(torch.bfloat16).requires_grad_()
    outs = [q(x) for q in qs]
    assert len(calls) == 1
    assert all(torch.equal(outs[0], o) for o in outs[1:])
    assert all(torch.equal(qs[0].scale, q.scale) and torch.equal(qs[0].zero_point, q.zero_point) for q in qs[1:])
    sum(o.float().sum() for o in outs).backward()
    assert torch.equal(x.grad, torch.full_like(x, 3.0))  # three straight-through paths
    monkeypatch.setattr(FakeQuantizer, "share_identical_inputs", False)
    ref = FakeQuantizer(cfg)(x)
    assert len(calls) == 2 and torch.equal(ref, outs[0])
    monkeypatch.setattr(FakeQuantizer, "share_identical_inputs", True)
    y = x.detach().clone()
    a = qs[0](y)
    n = len(calls)
    with torch.no_grad():
        y.mul_(2.0)  # same object, new version: must not hit
    b = qs[1](y)
    assert len(calls) == n + 1 and not torch.equal(a, b)
    z = y.clone()  # equal values, another tensor: recomputed
    c = qs[2](z)
    assert len(calls) == n + 2 and torch.equal(b, c)


def test_prepare_with_default_quantizer_arguments_runs_a_bf16_model():
    """The north-star QAT config builds the quantizer with a group size only (recipes/configs/llama3/8B_qat_full.yaml:62-64,
    precision left at its float32 default) on a bf16 model: the prepared model must keep bf16 weights, train, and match
    the oracle."""
    gen = torch.Generator().manual_seed(11)
    model = nn.Sequential(nn.Linear(256, 128, bias=False)).to(DEV).to(torch.bfloat16)
    w = (torch.randn(128, 256, generator=gen) * 0.05).to(torch.bfloat16)
    with torch.no_grad():
        model[0].weight.copy_(w)
    param = model[0].weight
    model = Int8DynActInt4WeightQATQuantizer(groupsize=32).prepare(model)
    assert model[0].weight is param and model[0].weight.dtype == torch.bfloat16
    x = torch.randn(6, 256, generator=gen).to(torch.bfloat16)
    xd = x.to(DEV).requires_grad_()
    y = model(xd)
    assert y.dtype == torch.bfloat16
    (y.float() ** 2).sum().backward()
    xo, wo = x.clone().requires_grad_(), w.clone().requires_grad_()
    yo = fq.fake_quantized_linear(xo, wo, 32)
    (yo.float() ** 2).sum().backward()
    torch.testing.assert_close(y.detach().cpu().float(), yo.detach().float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(xd.grad.cpu().float(), xo.grad.float(), rtol=1e-2, atol=1e-2)
    with torch.inference_mode():  # evaluation / generation loops run under inference_mode
        yi = model(x.to(DEV))
    torch.testing.assert_close(yi.cpu().float(), yo.detach().float(), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_version_dependent_conventions_are_parameters(dtype):
    """The constants on which versions of the reference's quantisation package differ (the lower bound of each scale, and
    whether the weight-only uint4 scheme bounds the range or the quotient) are arguments of the `_conv` entry points and
    of the oracle; with any setting the kernels stay bit-exact against the oracle, and the defaults are unchanged."""
    g = torch.Generator().manual_seed(17)
    w = (torch.randn(96, 1024, generator=g) * 0.02).to(dtype)
    w[3] *= 1e-4   # groups whose scale falls under the larger bounds
    w[5] = 0
    bf16_eps = float(torch.finfo(torch.bfloat16).eps)  # the bound a version that takes eps from a bf16 weight would use
    for eps in (None, bf16_eps, 1e-5):
        fqd, sd = ops.fq_per_group_int4_sym(w.to(DEV), 32, eps=eps)
        fo, so = fq.fq_per_group_int4_sym(w, 32, eps=eps)
        assert bits_equal(fqd.cpu(), fo) and bits_equal(sd.cpu(), so), eps
        q, s, z = ops.quantize_per_group_int4(w.to(DEV), 32, eps=eps)
        qo, so2, zo = fq.quantize_per_group_int4(w, 32, eps=eps)
        assert torch.equal(q.cpu(), qo) and bits_equal(s.cpu(), so2), eps
    # with the bf16 bound most groups of an N(0, 0.02) weight sit on the bound: the setting matters
    assert float((ops.fq_per_group_int4_sym(w.to(DEV), 32, eps=bf16_eps)[1] == bf16_eps).float().mean()) > 0.5
    x = (torch.randn(40, 512, generator=g) * 1.5).to(dtype)
    x[1] *= 1e-5
    x[2] = 0
    for eps in (None, 1e-3, bf16_eps):
        od, sd, zd = ops.fq_per_token_int8_asym(x.to(DEV), eps=eps)
        oo, so, zo = fq.fq_per_token_int8_asym(x, eps=eps)
        assert bits_equal(od.cpu(), oo) and bits_equal(sd.cpu(), so) and torch.equal(zd.cpu(), zo), eps
    u = (torch.randn(64, 512, generator=g) * 0.02).to(dtype)
    u[7] = u[7, 0]            # constant groups: range 0, the bound decides the scale
    u[9] = u[9] * 1e-5
    for min_scale, first in ((1e-6, False), (1e-6, True), (1e-3, False), (1e-3, True), (3e-7, True)):
        od, sd, zd = ops.fq_per_group_uint4_asym(u.to(DEV), 64, torch.bfloat16, min_scale=min_scale, clamp_range_first=first)
        oo, so, zo = fq.fq_per_group_uint4_asym(u, 64, torch.bfloat16, min_scale=min_scale, clamp_range_first=first)
        assert bits_equal(od.cpu(), oo), (min_scale, first)
        assert bits_equal(sd.cpu(), so.float()) and bits_equal(zd.cpu(), zo.float()), (min_scale, first)
        qd, _, _ = ops.quantize_per_group_uint4(u.to(DEV), 64, torch.bfloat16, min_scale=min_scale, clamp_range_first=first)
        qo, _, _ = fq.quantize_per_group_uint4(u, 64, torch.bfloat16, min_scale=min_scale, clamp_range_first=first)
        assert torch.equal(qd.cpu(), qo), (min_scale, first)
    # the config carries eps to the kernels
    cfg = FakeQuantizeConfig(torch.int4, group_size=32, is_symmetric=True, eps=bf16_eps)
    fqz = FakeQuantizer(cfg)
    out = fqz(w.to(DEV))
    assert bits_equal(out.cpu(), fq.fq_per_group_int4_sym(w, 32, eps=bf16_eps)[0])
