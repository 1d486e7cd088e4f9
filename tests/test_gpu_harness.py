"""The Llama-shaped harness on the GPU: one step of a tiny QLoRA decoder, fused path against the composed path."""
import pytest
import torch

from torchtune_amd import harness
from torchtune_amd.modules.peft import LoRALinear
from torchtune_amd.nf4_tensor import NF4Tensor

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_tiny_qlora_decoder_step_fused_equals_composed(monkeypatch):
    model = harness.build_qlora_decoder("tiny", rank=8, alpha=16.0, device=DEV, seed=0)
    trainable = [n for n, p in model.named_parameters() if p.requires_grad]
    assert trainable and all("lora_" in n for n in trainable)
    assert all(isinstance(l.attn.q_proj.weight, NF4Tensor) for l in model.layers)
    assert not isinstance(model.output.weight, NF4Tensor)
    g = torch.Generator(device=DEV).manual_seed(1)
    tokens = torch.randint(0, 1024, (2, 192), device=DEV, generator=g)
    labels = torch.randint(0, 1024, (2, 192), device=DEV, generator=g)
    loss = harness.train_step(model, tokens, labels)
    grads = {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}
    assert set(grads) == set(trainable) and torch.isfinite(loss) and 6.0 < float(loss) < 8.0  # ~ln(1024)
    model.zero_grad(set_to_none=True)
    # composed path: linear_nf4 + separate adapter GEMMs, the structure of the reference's forward
    monkeypatch.setattr(LoRALinear, "_fused", lambda self, x: False)
    loss2 = harness.train_step(model, tokens, labels)
    torch.testing.assert_close(loss, loss2, rtol=2e-3, atol=2e-3)
    for n, p in model.named_parameters():
        if p.grad is not None:
            ref = p.grad.float()
            torch.testing.assert_close(grads[n].float(), ref, rtol=5e-2, atol=5e-2 * float(ref.abs().max()) + 1e-6)


def test_activation_checkpointing_gives_the_same_step():
    a = harness.build_qlora_decoder("tiny", rank=8, alpha=16.0, device=DEV, seed=0)
    b = harness.build_qlora_decoder("tiny", rank=8, alpha=16.0, device=DEV, seed=0, activation_checkpointing=True)
    tokens = torch.randint(0, 1024, (1, 128), device=DEV, generator=torch.Generator(device=DEV).manual_seed(2))
    la, lb = harness.train_step(a, tokens, tokens), harness.train_step(b, tokens, tokens)
    assert torch.equal(la, lb)
    for (n, p), (_, q) in zip(a.named_parameters(), b.named_parameters()):
        if p.grad is not None:
            assert torch.equal(p.grad, q.grad), n


@pytest.mark.parametrize("kind", ["qlora", "qat"])
def test_residual_additions_inside_the_norm_pass_give_the_same_step(monkeypatch, kind):
    """``harness.FUSED_ADD_NORM``: the additions of the residual stream inside the RMSNorm pass that follows each of them
    against additions of their own: the same loss and the same gradients, bit for bit (QLoRA: adapter gradients; QAT:
    every weight and norm scale, so the scale-gradient form of the norm's backward runs as well)."""
    build = (lambda: harness.build_qlora_decoder("tiny", rank=8, alpha=16.0, device=DEV, seed=0)) if kind == "qlora" else \
            (lambda: harness.build_qat_decoder("tiny", groupsize=32, device=DEV, seed=0))
    tokens = torch.randint(0, 1024, (2, 160), device=DEV, generator=torch.Generator(device=DEV).manual_seed(4))
    out = []
    for fused in (True, False):
        monkeypatch.setattr(harness, "FUSED_ADD_NORM", fused)
        model = build()
        loss = harness.train_step(model, tokens, tokens)
        out.append((loss, {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(out[0][0], out[1][0])
    assert set(out[0][1]) == set(out[1][1]) and out[0][1]
    for n, gr in out[0][1].items():
        assert torch.equal(gr, out[1][1][n]), n


def test_one_launch_for_rope_and_head_expansion_gives_the_same_step(monkeypatch):
    """``harness.FUSED_QKV_POST``: the rotary embedding of q and k and the expansion of the key / value heads as one launch
    per direction against the four launches they replace: the same loss and adapter gradients, bit for bit."""
    tokens = torch.randint(0, 1024, (2, 160), device=DEV, generator=torch.Generator(device=DEV).manual_seed(6))
    out = []
    for fused in (True, False):
        monkeypatch.setattr(harness, "FUSED_QKV_POST", fused)
        model = harness.build_qlora_decoder("tiny", rank=8, alpha=16.0, device=DEV, seed=0)
        assert model.layers[0].attn.n_kv != model.layers[0].attn.n_heads
        loss = harness.train_step(model, tokens, tokens)
        out.append((loss, {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None}))
    assert torch.equal(out[0][0], out[1][0])
    assert set(out[0][1]) == set(out[1][1]) and out[0][1]
    for n, gr in out[0][1].items():
        assert torch.equal(gr, out[1][1][n]), n


def test_tiny_qat_decoder_step():
    model = harness.build_qat_decoder("tiny", groupsize=32, device=DEV, seed=0)
    tokens = torch.randint(0, 1024, (2, 64), device=DEV, generator=torch.Generator(device=DEV).manual_seed(3))
    loss = harness.train_step(model, tokens, tokens)
    assert torch.isfinite(loss)
    assert all(p.grad is not None for n, p in model.named_parameters() if "weight" in n and "tok_embeddings" not in n)


def test_attention_backends_agree_and_match_an_fp32_reference(monkeypatch):
    """The stack asks PyTorch for its "efficient" attention backend (its backward is much faster here than "flash").
    Output and q/k/v gradients of both backends must agree with an fp32 softmax(QK^T)V computed with plain matmuls,
    at the 8B head shape, and one decoder step must give the same loss and gradients with either backend."""
    g = torch.Generator(device=DEV).manual_seed(5)
    b, h, s, d = 2, 8, 512, 128
    q, k, v = (torch.randn(b, s, h, d, device=DEV, generator=g).to(torch.bfloat16).requires_grad_() for _ in range(3))
    go = torch.randn(b, h, s, d, device=DEV, generator=g).to(torch.bfloat16)
    qf, kf, vf = (t.detach().float().transpose(1, 2).requires_grad_() for t in (q, k, v))
    att = (qf @ kf.transpose(-1, -2)) / d ** 0.5
    att = att.masked_fill(torch.ones(s, s, device=DEV, dtype=torch.bool).triu(1), float("-inf")).softmax(-1)
    ref = att @ vf
    ref.backward(go.float())
    for backend in ("efficient", "flash"):
        monkeypatch.setattr(harness, "SDPA_BACKEND", backend)
        for t in (q, k, v):
            t.grad = None
        out = harness._sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        out.backward(go)
        torch.testing.assert_close(out.float(), ref.detach(), rtol=2e-2, atol=2e-2, msg=backend)
        for got, want in ((q.grad, qf.grad), (k.grad, kf.grad), (v.grad, vf.grad)):
            want = want.transpose(1, 2)
            torch.testing.assert_close(got.float(), want, rtol=2e-2, atol=2e-2 * float(want.abs().max()), msg=backend)
    model = harness.build_qlora_decoder("tiny", rank=8, alpha=16.0, device=DEV, seed=0)
    tokens = torch.randint(0, 1024, (2, 192), device=DEV, generator=g)
    results = {}
    for backend in ("efficient", "flash"):
        monkeypatch.setattr(harness, "SDPA_BACKEND", backend)
        model.zero_grad(set_to_none=True)
        loss = harness.train_step(model, tokens, tokens)
        results[backend] = (loss, {n: p.grad.clone() for n, p in model.named_parameters() if p.grad is not None})
    torch.testing.assert_close(results["efficient"][0], results["flash"][0], rtol=2e-3, atol=2e-3)
    for n, ge in results["efficient"][1].items():
        gf = results["flash"][1][n].float()
        torch.testing.assert_close(ge.float(), gf, rtol=5e-2, atol=5e-2 * float(gf.abs().max()) + 1e-6, msg=n)
