"""Every distinct projection of the benchmark configurations at its full size, on the GPU.

Shapes (``[N, K]``, tokens M, rank, alpha) are those of the reference's builders: ``llama3_2_1b``
(``torchtune/models/llama3_2/_model_builders.py:20-46``: dim 2048, 8 kv heads of 64, hidden 8192; QLoRA with rank 8,
alpha 16 on 4 x 2048 tokens), ``llama3_1_8b`` and ``llama3_1_70b`` (``torchtune/models/llama3_1/_model_builders.py:20-59``:
dim 4096 / 8192, 8 kv heads of 128, hidden 14336 / 28672; rank 16, alpha 32 on 4 x 2048 / 1 x 4096 tokens).

These tensors are too large for an eager CPU pass, so parity is shown in two links:

* the quantisation itself against the CPU oracle on slices of whole scaler blocks (the first and the last 64 rows):
  codes, scaler bytes, factors and dequantised values bit for bit, with the one quantity that couples the whole tensor,
  the scaler mean, checked separately against an exact fp64 mean;
* the fused layer (forward, grad-input, both adapter gradients) against fp32 matmuls of that bit-exactly dequantised
  weight on the GPU, at rtol 1e-2 / atol 1e-2 (bf16 inputs, fp32 accumulation on both sides; adapter gradients at 4e-3 of
  their largest entry), plus the CPU oracle's own unfused bf16 forward on the slice.

The 8da4w configuration gets the same treatment: fake quantisation and ``convert()`` at the full weight and activation
sizes against the oracle on row slices (both schemes are row-local), and size-independent properties on the whole
tensors."""
import pytest
import torch

from oracle import fake_quant_oracle as fqo
from oracle import lora_oracle, nf4_oracle
from tests.helpers import bits_equal
from torchtune_amd import harness, ops
from torchtune_amd.modules.peft import LoRALinear
from torchtune_amd.nf4_tensor import to_nf4
from torchtune_amd.qat import Int8DynActInt4WeightLinear, Int8DynActInt4WeightQATQuantizer

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16

PROJECTIONS = [
    # config, N, K, tokens, rank, alpha
    ("1b q,o", 2048, 2048, 8192, 8, 16.0),
    ("1b k,v", 512, 2048, 8192, 8, 16.0),
    ("1b gate,up", 8192, 2048, 8192, 8, 16.0),
    ("1b down", 2048, 8192, 8192, 8, 16.0),
    ("8b q,o", 4096, 4096, 8192, 16, 32.0),
    ("8b k,v", 1024, 4096, 8192, 16, 32.0),
    ("8b gate,up", 14336, 4096, 8192, 16, 32.0),
    ("8b down", 4096, 14336, 8192, 16, 32.0),
    ("70b q,o", 8192, 8192, 4096, 16, 32.0),
    ("70b k,v", 1024, 8192, 4096, 16, 32.0),
    ("70b gate,up", 28672, 8192, 4096, 16, 32.0),
    ("70b down", 8192, 28672, 4096, 16, 32.0),
]


def _slice_parts(t, r0, rows, K):
    """The NF4 parts of rows [r0, r0 + rows) of the GPU tensor ``t`` (whole scaler blocks), on the CPU."""
    b0, nb = r0 * K // 64, rows * K // 64
    assert b0 % 256 == 0 and nb % 256 == 0
    return (t.quantized_data[r0 * K // 2:(r0 + rows) * K // 2].cpu(), t.quantized_scalers[b0:b0 + nb].cpu(),
            t.quantization_factor[b0 // 256:(b0 + nb) // 256].cpu())


@pytest.mark.parametrize("name,N,K,M,r,alpha", PROJECTIONS, ids=[p[0].replace(" ", "_").replace(",", "+") for p in PROJECTIONS])
def test_projection_at_full_size(name, N, K, M, r, alpha):
    g = torch.Generator(device=DEV).manual_seed(N * 31 + K)
    w = (torch.randn(N, K, device=DEV, generator=g) * 0.02).to(BF)
    with torch.device(DEV):
        prev = torch.get_default_dtype()
        torch.set_default_dtype(BF)
        try:
            layer = LoRALinear(K, N, rank=r, alpha=alpha, quantize_base=True)
        finally:
            torch.set_default_dtype(prev)
    A = lora_oracle.lora_a_init_(torch.empty(r, K), torch.Generator().manual_seed(N + K)).to(BF)
    B = (torch.randn(N, r, generator=torch.Generator().manual_seed(N - K)) * 0.01).to(BF)
    with torch.no_grad():
        layer.weight.copy_(w)
        layer.lora_a.weight.copy_(A.to(DEV))
        layer.lora_b.weight.copy_(B.to(DEV))
    t = layer.weight

    # ---- link 1: the quantisation against the oracle
    absmax = w.view(-1, 64).abs().amax(1)
    exact_mean = (absmax.double().sum() / absmax.numel()).float().to(BF)  # fp64 sums of bf16 values are exact at this size
    assert bits_equal(t.scaler_mean.reshape(1), exact_mean.reshape(1))
    D = t.get_original_weight()
    for r0 in (0, N - 64):
        p = nf4_oracle.nf4_quantize(w[r0:r0 + 64].cpu(), 64, 256, mean=t.scaler_mean)
        codes, scalers, factors = _slice_parts(t, r0, 64, K)
        assert torch.equal(codes, p.quantized_data), f"{name}: codes of rows {r0}.."
        assert torch.equal(scalers, p.quantized_scalers), f"{name}: scaler bytes of rows {r0}.."
        assert bits_equal(factors, p.quantization_factor), f"{name}: factors of rows {r0}.."
        assert bits_equal(D[r0:r0 + 64].cpu(), nf4_oracle.nf4_dequantize(p)), f"{name}: dequantised rows {r0}.."
    # requantisation idempotence, the reference's own invariant (tests/torchtune/modules/peft/test_lora.py:229-237)
    assert torch.equal(to_nf4(D).quantized_data, t.quantized_data)
    del w, absmax

    # ---- link 2: the fused layer against fp32 matmuls of the bit-exact dequantised weight
    s = alpha / r
    x = torch.randn(M, K, device=DEV, generator=g).to(BF).requires_grad_()
    gy = torch.randn(M, N, device=DEV, generator=g).to(BF)
    y = layer(x)
    y.backward(gy)
    Df = D.float()
    Af, Bf = A.to(DEV).float(), B.to(DEV).float()
    xf = x.detach().float()
    h = (xf @ Af.T).to(BF).float()       # the hidden activation is stored in bf16 by design
    ref_y = xf @ Df.T
    ref_y += s * (h @ Bf.T)
    torch.testing.assert_close(y.detach().float(), ref_y, rtol=1e-2, atol=1e-2)
    ref_y_slice = ref_y[:256, N - 64:].cpu()
    del ref_y
    gyf = gy.float()
    gh = (s * (gyf @ Bf)).to(BF).float()
    ref_gx = gyf @ Df
    ref_gx += gh @ Af
    torch.testing.assert_close(x.grad.float(), ref_gx, rtol=1e-2, atol=1e-2 * max(1.0, float(ref_gx.abs().max()) / 8))
    del ref_gx, Df
    ref_ga = gh.T @ xf
    ref_gb = s * (gyf.T @ h)
    # one bf16 rounding of an fp32-accumulated result, the bound the small cases of test_gpu_lora_linear.py hold
    for got, want in ((layer.lora_a.weight.grad, ref_ga), (layer.lora_b.weight.grad, ref_gb)):
        torch.testing.assert_close(got.float(), want, rtol=4e-3, atol=4e-3 * float(want.abs().max()))

    # ---- the oracle's own unfused bf16 forward on the last 64 output columns and the first 256 tokens
    r0 = N - 64
    p = nf4_oracle.nf4_quantize(layer.weight.get_original_weight()[r0:].cpu(), 64, 256, mean=t.scaler_mean)
    yo = lora_oracle.lora_linear_forward(x.detach()[:256].cpu(), p, A, B[r0:], alpha, r)
    # The oracle's bf16 matmul on the CPU carries an error of its own that grows with K (its distance from the fp32
    # evaluation is measured here); the kernel has to agree with the oracle to within that, and be no further from the
    # fp32 evaluation than the oracle is.
    y_slice = y.detach()[:256, r0:].cpu().float()
    oracle_err = float((yo.float() - ref_y_slice).abs().max())
    torch.testing.assert_close(y_slice, yo.float(), rtol=1e-2, atol=max(1e-2, 1.5 * oracle_err))
    assert float((y_slice - ref_y_slice).abs().max()) <= max(oracle_err, 1e-2 + 1e-2 * float(ref_y_slice.abs().max()))
    # determinism of the whole layer
    assert torch.equal(layer(x.detach()), y.detach())


def test_two_layer_70b_width_stack_with_activation_checkpointing():
    """Config 5's layer shapes (dim 8192, 64 heads / 8 kv heads, hidden 28672) with per-layer activation checkpointing on
    1 x 4096 tokens, two layers deep: the step with the forward recomputed inside backward must give the loss of the step
    without checkpointing exactly and the same adapter gradients (to bf16 rounding: autograd sums the three gradients of
    a layer's input in a different order when the graph is rebuilt, and PyTorch's attention backward is not bitwise
    reproducible), and every adapter must receive a gradient."""
    shape = harness.LlamaShape("llama3_1_70b_two_layers", 2, 8192, 64, 8, 28672)
    tokens = torch.randint(0, shape.vocab, (1, 4096), device=DEV, generator=torch.Generator(device=DEV).manual_seed(1))
    labels = torch.randint(0, shape.vocab, (1, 4096), device=DEV, generator=torch.Generator(device=DEV).manual_seed(2))
    results = []
    for ac in (True, False):
        model = harness.build_qlora_decoder(shape, 16, 32.0, device=DEV, seed=0, activation_checkpointing=ac)
        with torch.no_grad():  # lora_b starts at zero: give the adapters something to do
            gen = torch.Generator(device=DEV).manual_seed(3)
            for n, prm in model.named_parameters():
                if n.endswith("lora_b.weight"):
                    prm.copy_((torch.randn(prm.shape, device=DEV, generator=gen) * 0.01).to(prm.dtype))
        loss = harness.train_step(model, tokens, labels)
        torch.cuda.synchronize()
        grads = {n: prm.grad.clone() for n, prm in model.named_parameters() if prm.requires_grad}
        assert torch.isfinite(loss)
        assert len(grads) == 2 * 7 * 2
        for n, gr in grads.items():
            assert torch.isfinite(gr).all() and float(gr.float().abs().max()) > 0, n
        results.append((float(loss), grads))
        del model, grads
        torch.cuda.empty_cache()
    (l_ac, g_ac), (l_plain, g_plain) = results
    assert l_ac == l_plain
    for n in g_ac:
        want = g_plain[n].float()
        torch.testing.assert_close(g_ac[n].float(), want, rtol=4e-3, atol=4e-3 * float(want.abs().max()), msg=n)


# ---------------------------------------------------------------------------------------------------------------------
# config 4: 8da4w QAT at the 8B sizes (2 x 4096 tokens, group size 32)
# ---------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336), (128256, 4096)], ids=["gate+up", "down", "output"])
def test_convert_and_weight_fake_quant_at_full_size(N, K):
    gsz = 32
    g = torch.Generator(device=DEV).manual_seed(N + K)
    w = (torch.randn(N, K, device=DEV, generator=g) * 0.02).to(BF)
    q, scale, zeros = ops.quantize_per_group_int4(w, gsz)
    fq, fscale = ops.fq_per_group_int4_sym(w, gsz)
    # row slices against the oracle (the scheme is local to a group): first, middle and last rows
    for r0 in (0, (N // 2) // 64 * 64, N - 64):
        qo, so, zo = fqo.quantize_per_group_int4(w[r0:r0 + 64].cpu(), gsz)
        assert torch.equal(q[r0:r0 + 64].cpu(), qo) and bits_equal(scale[r0:r0 + 64].cpu(), so) and torch.equal(zeros[r0:r0 + 64].cpu(), zo)
        fo, fso = fqo.fq_per_group_int4_sym(w[r0:r0 + 64].cpu(), gsz)
        assert bits_equal(fq[r0:r0 + 64].cpu(), fo) and bits_equal(fscale[r0:r0 + 64].cpu(), fso)
    # whole-tensor properties: the int4 range, zero zero-points, the closed form of the scale, and convert() describing
    # exactly the weight the fake-quantised layer trained with
    assert q.dtype == torch.int8 and int(q.min()) >= -8 and int(q.max()) <= 7
    assert not zeros.any()
    amax = w.float().view(N, K // gsz, gsz).abs().amax(-1)
    want_scale = torch.clamp(amax / 7.5, min=torch.finfo(torch.float32).eps)
    # (to one ulp: the GPU's eager division by a constant is not the correctly rounded quotient the kernel and the
    # CPU oracle compute; the slices above are the bit-exact check)
    torch.testing.assert_close(scale, want_scale, rtol=2.5e-7, atol=0.0)
    assert bits_equal(scale, fscale)
    assert bits_equal(ops.dequantize_per_group_int4(q, scale, zeros, gsz, BF), fq)
    # fake quantisation is idempotent given its own grid: the codes of fq(w) are the codes of w
    on_grid = (fq.float().view(N, K // gsz, gsz) / scale.unsqueeze(-1)).round()
    assert torch.equal(on_grid.view(N, K).to(torch.int8), q)


@pytest.mark.parametrize("K", [4096, 14336])
def test_activation_fake_quant_at_full_size(K):
    M = 8192
    g = torch.Generator(device=DEV).manual_seed(K)
    x = (torch.randn(M, K, device=DEV, generator=g) * 1.3).to(BF)
    out, scale, zp = ops.fq_per_token_int8_asym(x)
    for r0 in (0, 4096, M - 64):
        oo, so, zo = fqo.fq_per_token_int8_asym(x[r0:r0 + 64].cpu())
        assert bits_equal(out[r0:r0 + 64].cpu(), oo) and bits_equal(scale[r0:r0 + 64].cpu(), so.reshape(-1))
        assert torch.equal(zp[r0:r0 + 64].cpu(), zo.reshape(-1).to(torch.int32))
    # whole-tensor properties: every output lies inside its row's int8 range (to bf16 rounding), the closed form of the scale
    qv = out.float() / scale[:, None] + zp[:, None]
    assert float(qv.min()) >= -128.6 and float(qv.max()) <= 127.6
    mn = x.float().amin(1).clamp(max=0)
    mx = x.float().amax(1).clamp(min=0)
    torch.testing.assert_close(scale, torch.clamp((mx - mn) / 255.0, min=torch.finfo(torch.float32).eps), rtol=2.5e-7, atol=0.0)


def test_qat_linear_at_full_size_against_the_oracle_on_slices():
    """The 8B gate projection as the prepared QAT linear at 2 x 4096 tokens: forward and both gradients against the CPU
    oracle of the same layer restricted to row slices (fake quantisation is row-local on both operands), then
    ``convert()`` and the converted layer's forward."""
    N, K, M, gsz = 14336, 4096, 8192, 32
    g = torch.Generator(device=DEV).manual_seed(7)
    model = torch.nn.Sequential(torch.nn.Linear(K, N, bias=False)).to(DEV).to(BF)
    with torch.no_grad():
        model[0].weight.copy_((torch.randn(N, K, device=DEV, generator=g) * 0.02).to(BF))
    w = model[0].weight.detach().clone()
    qz = Int8DynActInt4WeightQATQuantizer(groupsize=gsz)
    model = qz.prepare(model)
    x = torch.randn(M, K, device=DEV, generator=g).to(BF).requires_grad_()
    y = model(x)
    gy = torch.randn(M, N, device=DEV, generator=g).to(BF)
    y.backward(gy)
    for m0, n0 in ((0, 0), (M - 128, N - 64)):
        xo = x.detach()[m0:m0 + 128].cpu().requires_grad_()
        wo = w[n0:n0 + 64].cpu().requires_grad_()
        yo = fqo.fake_quantized_linear(xo, wo, gsz)
        torch.testing.assert_close(y.detach()[m0:m0 + 128, n0:n0 + 64].cpu().float(), yo.detach().float(), rtol=1e-2, atol=1e-2)
    # straight-through gradients: fp32 matmuls of the bit-exact fake-quantised operands
    xq, _, _ = ops.fq_per_token_int8_asym(x.detach(), want_qparams=False)
    wq, _ = ops.fq_per_group_int4_sym(w, gsz, want_scale=False)
    ref_gx = gy.float() @ wq.float()
    torch.testing.assert_close(x.grad.float(), ref_gx, rtol=1e-2, atol=1e-2 * max(1.0, float(ref_gx.abs().max()) / 8))
    ref_gw = gy.float().T @ xq.float()
    torch.testing.assert_close(model[0].weight.grad.float(), ref_gw, rtol=4e-3, atol=4e-3 * float(ref_gw.abs().max()))
    del ref_gx, ref_gw
    model = qz.convert(model)
    assert isinstance(model[0], Int8DynActInt4WeightLinear)
    qo, so, _ = fqo.quantize_per_group_int4(w[:64].cpu(), gsz)
    assert torch.equal(model[0].weight[:64].cpu(), qo) and bits_equal(model[0].scales[:64].cpu(), so)
    torch.testing.assert_close(model(x.detach()).float(), y.detach().float(), rtol=1e-2, atol=1e-2)
