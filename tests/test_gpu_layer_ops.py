"""GPU parity of the single-pass RMSNorm / rotary / SwiGLU kernels (forward and backward, through autograd and through the
C ABI) against the eager CPU oracle.  Floating-point kernels: bf16 results within rtol 1e-2 / atol 1e-2 of the oracle
(both sides compute in fp32 and round to bf16 at the same points; summation order and exp / rsqrt differ), and for the
element-wise ones at most one bf16 ulp apart."""
import pytest
import torch

from oracle import layer_oracle as lo
from torchtune_amd import _lib, ops
from torchtune_amd.modules import layer_ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def _close(got, want, rtol=1e-2, atol=1e-2):
    torch.testing.assert_close(got.float().cpu(), want.float(), rtol=rtol, atol=atol)


def _within_ulps(got, want, n):
    w = want.float()
    ulp = torch.maximum(w.abs(), torch.tensor(2.0 ** -120)) * 2.0 ** -7
    assert torch.all((got.float().cpu() - w).abs() <= n * ulp)


@pytest.mark.parametrize("rows,D", [(5, 64), (33, 2048), (64, 4096), (9, 8192), (7, 4104)])
def test_rms_norm_forward_backward(rows, D):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(rows, D, generator=g).to(BF).requires_grad_()
    w = (torch.rand(D, generator=g) + 0.5).to(BF).requires_grad_()
    gy = torch.randn(rows, D, generator=g).to(BF)
    want = lo.rms_norm(x, w, 1e-5)
    want.backward(gy)
    m = layer_ops.RMSNorm(D, 1e-5).to(DEV, BF)
    with torch.no_grad():
        m.scale.copy_(w)
    xd = x.detach().to(DEV).requires_grad_()
    got = m(xd)
    got.backward(gy.to(DEV))
    _within_ulps(got, want, 2)
    _close(xd.grad, x.grad)
    _close(m.scale.grad, w.grad, rtol=2e-2, atol=2e-2 * float(w.grad.float().abs().max()))
    # frozen scale: no scale gradient is computed, the input gradient is unchanged
    m.scale.requires_grad_(False)
    xd2 = x.detach().to(DEV).requires_grad_()
    m(xd2).backward(gy.to(DEV))
    assert torch.equal(xd2.grad, xd.grad)


def test_rms_norm_backward_when_workgroups_walk_several_rows():
    """More rows than the scale-gradient form has workgroups (1024): each walks two or three rows, asking for the next one
    while it works on the current; input and scale gradients against the oracle's autograd, and the input gradient
    against the form without a scale gradient bit for bit."""
    rows, D = 2500, 4096
    g = torch.Generator().manual_seed(3)
    x = torch.randn(rows, D, generator=g).to(BF).requires_grad_()
    w = (torch.rand(D, generator=g) + 0.5).to(BF).requires_grad_()
    gy = torch.randn(rows, D, generator=g).to(BF)
    lo.rms_norm(x, w, 1e-5).backward(gy)
    m = layer_ops.RMSNorm(D, 1e-5).to(DEV, BF)
    with torch.no_grad():
        m.scale.copy_(w)
    xd = x.detach().to(DEV).requires_grad_()
    m(xd).backward(gy.to(DEV))
    _close(xd.grad, x.grad)
    _close(m.scale.grad, w.grad, rtol=2e-2, atol=2e-2 * float(w.grad.float().abs().max()))
    m.scale.requires_grad_(False)
    xd2 = x.detach().to(DEV).requires_grad_()
    m(xd2).backward(gy.to(DEV))
    assert torch.equal(xd2.grad, xd.grad)


@pytest.mark.parametrize("rows,D,train_scale", [(5, 64, True), (70, 4096, True), (2500, 4096, True), (33, 8192, False), (9, 4104, False)])
def test_add_rms_norm_equals_the_addition_followed_by_the_norm_bitwise(rows, D, train_scale):
    """``add_rms_norm(x, r, norm)`` against ``h = x + r; norm(h)``: both outputs and the gradients of x, r and the scale
    bit for bit, with gradients arriving on both outputs (as in a decoder layer) and on the normalised one alone."""
    g = torch.Generator().manual_seed(rows + D)
    x = torch.randn(rows, D, generator=g).to(BF).to(DEV)
    r = torch.randn(rows, D, generator=g).to(BF).to(DEV)
    gh = torch.randn(rows, D, generator=g).to(BF).to(DEV)
    gn = torch.randn(rows, D, generator=g).to(BF).to(DEV)
    m = layer_ops.RMSNorm(D, 1e-5).to(DEV, BF)
    with torch.no_grad():
        m.scale.copy_((torch.rand(D, generator=g) + 0.5).to(BF))
    m.scale.requires_grad_(train_scale)

    def run(fused, both):
        m.zero_grad()
        xa, ra = x.clone().requires_grad_(), r.clone().requires_grad_()
        if fused:
            h, n = layer_ops.add_rms_norm(xa, ra, m)
        else:
            h = xa + ra
            n = m(h)
        if both:
            torch.autograd.backward([h, n], [gh, gn])
        else:
            n.backward(gn)
        out = [h.detach(), n.detach(), xa.grad, ra.grad]
        return out + ([m.scale.grad.clone()] if train_scale else [])

    for both in (True, False):
        for a, b in zip(run(True, both), run(False, both)):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_rms_norm_leading_dimensions_and_validation():
    x = torch.randn(2, 3, 256, device=DEV).to(BF)
    w = torch.ones(256, device=DEV, dtype=BF)
    y, rstd = ops.rms_norm_fwd(x, w, 1e-6)
    assert y.shape == x.shape and rstd.shape == (6,)
    _close(y, lo.rms_norm(x.cpu(), w.cpu(), 1e-6))
    lib = _lib.load()
    assert lib.ttamd_rms_norm_fwd_bf16(x.data_ptr(), w.data_ptr(), 1e-6, y.data_ptr(), None, 6, 100, None) == -1
    assert b"multiple of 8" in lib.ttamd_last_error()
    with pytest.raises(RuntimeError, match="HIP kernels"):
        ops.rms_norm_fwd(x.cpu(), w.cpu(), 1e-6)


@pytest.mark.parametrize("b,s,nh,hd", [(1, 5, 1, 8), (2, 37, 4, 64), (2, 128, 8, 128)])
def test_rope_forward_backward(b, s, nh, hd):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(b, s, nh, hd, generator=g).to(BF).requires_grad_()
    gy = torch.randn(b, s, nh, hd, generator=g).to(BF)
    cache = lo.rope_cache(s + 3, hd, 500000.0)  # a longer table than the sequence: only the first s rows are used
    want = lo.rope(x, cache)
    want.backward(gy)
    xd = x.detach().to(DEV).requires_grad_()
    got = layer_ops.apply_rope(xd, cache.to(DEV))
    got.backward(gy.to(DEV))
    _within_ulps(got, want, 1)
    _within_ulps(xd.grad, x.grad, 1)
    assert torch.equal(got[:, 0].cpu(), x.detach()[:, 0])


@pytest.mark.parametrize("shape", [(8,), (3, 40), (4, 128, 1024)])
def test_swiglu_forward_backward(shape):
    g = torch.Generator().manual_seed(2)
    a = (torch.randn(shape, generator=g) * 3).to(BF).requires_grad_()
    u = torch.randn(shape, generator=g).to(BF).requires_grad_()
    go = torch.randn(shape, generator=g).to(BF)
    want = lo.swiglu(a, u)
    want.backward(go)
    ad, ud = a.detach().to(DEV).requires_grad_(), u.detach().to(DEV).requires_grad_()
    got = layer_ops.swiglu(ad, ud)
    got.backward(go.to(DEV))
    _within_ulps(got, want, 2)
    _close(ad.grad, a.grad)
    _close(ud.grad, u.grad)


def test_full_size_properties_8b_activations():
    """8192 x 4096 / 8192 x 14336: properties that hold at any size."""
    g = torch.Generator(device=DEV).manual_seed(3)
    x = torch.randn(8192, 4096, device=DEV, generator=g).to(BF)
    y, rstd = ops.rms_norm_fwd(x, torch.ones(4096, device=DEV, dtype=BF), 0.0)
    torch.testing.assert_close(y.float().pow(2).mean(-1), torch.ones(8192, device=DEV), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(rstd, torch.rsqrt(x.float().pow(2).mean(-1)), rtol=1e-5, atol=1e-6)
    q = torch.randn(4, 2048, 32, 128, device=DEV, generator=g).to(BF)
    cache = lo.rope_cache(2048, 128, 500000.0).to(DEV)
    r = ops.rope(q, cache)
    torch.testing.assert_close(r.float().view(-1, 2).norm(dim=-1), q.float().view(-1, 2).norm(dim=-1), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(ops.rope(r, cache, inverse=True).float(), q.float(), rtol=2e-2, atol=2e-2)
    a = torch.randn(8192, 14336, device=DEV, generator=g).to(BF)
    z = ops.swiglu_fwd(a, torch.ones_like(a))
    torch.testing.assert_close(z.float(), torch.nn.functional.silu(a.float()), rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("rows,V", [(7, 1024), (33, 128256), (5, 131072), (4, 8)])
def test_cross_entropy_forward_backward(rows, V):
    g = torch.Generator().manual_seed(4)
    logits = (torch.randn(rows, V, generator=g) * 3).to(BF).requires_grad_()
    target = torch.randint(0, V, (rows,), generator=g)
    target[rows // 2] = -100  # an ignored row
    target[0] = V - 1
    want = lo.cross_entropy_sum(logits, target) * 0.25
    want.backward()
    ld = logits.detach().to(DEV).requires_grad_()
    got = layer_ops.cross_entropy_sum(ld, target.to(DEV), scale=0.25)
    (got * 2.0).backward()  # the incoming gradient rescales the stored one
    torch.testing.assert_close(got.cpu(), want.detach(), rtol=1e-4, atol=1e-4)
    # gradients are probabilities (<= 1) times 0.25 * 2, rounded to bf16
    torch.testing.assert_close(ld.grad.cpu().float(), 2.0 * logits.grad.float(), rtol=1e-2, atol=1e-5)
    assert torch.count_nonzero(ld.grad[rows // 2]) == 0
    per_row, _ = ops.cross_entropy_fwd_bwd(ld.detach(), target.to(DEV))
    ref_rows = torch.nn.functional.cross_entropy(logits.detach().float(), target, reduction="none")
    torch.testing.assert_close(per_row.cpu(), ref_rows, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("rows,D,V,train_weight", [(37, 256, 1024, False), (64, 128, 4096, True)])
def test_linear_cross_entropy_node_matches_projection_then_loss(rows, D, V, train_weight):
    """Vocabulary projection + loss as one autograd node: the same loss as ``cross_entropy_sum(linear(h, W))`` and the
    same gradients for the hidden states (and the weight when it trains), with an incoming gradient other than 1."""
    g = torch.Generator(device=DEV).manual_seed(rows + V)
    h = torch.randn(rows, D, device=DEV, generator=g).to(BF)
    W = (torch.randn(V, D, device=DEV, generator=g) * 0.1).to(BF)
    target = torch.randint(0, V, (rows,), device=DEV, generator=g)
    target[1] = -100
    outs = []
    for fused in (False, True):
        hh = h.clone().requires_grad_()
        ww = W.clone().requires_grad_(train_weight)
        if fused:
            loss = layer_ops.linear_cross_entropy_sum(hh, ww, target, scale=1.0 / rows)
        else:
            loss = layer_ops.cross_entropy_sum(torch.nn.functional.linear(hh, ww), target, scale=1.0 / rows)
        (loss * 3.0).backward()
        outs.append((loss.detach(), hh.grad, ww.grad))
    torch.testing.assert_close(outs[0][0], outs[1][0], rtol=0, atol=0)
    torch.testing.assert_close(outs[0][1].float(), outs[1][1].float(), rtol=2e-2, atol=1e-2 * float(outs[0][1].abs().max()))
    if train_weight:
        torch.testing.assert_close(outs[0][2].float(), outs[1][2].float(), rtol=2e-2, atol=1e-2 * float(outs[0][2].abs().max()))
    else:
        assert outs[1][2] is None
    # against fp32 autograd on the same operands
    hf, wf = h.float().requires_grad_(), W.float().requires_grad_()
    ref = torch.nn.functional.cross_entropy(hf @ wf.T, target, reduction="sum") / rows
    (ref * 3.0).backward()
    torch.testing.assert_close(outs[1][0], ref.detach(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(outs[1][1].float(), hf.grad, rtol=5e-2, atol=2e-2 * float(hf.grad.abs().max()))


@pytest.mark.parametrize("b,s,nkv,rep,hd", [(2, 33, 8, 4, 128), (1, 7, 2, 3, 64), (3, 5, 1, 8, 8), (1, 4, 4, 1, 16)])
def test_repeat_kv_forward_backward(b, s, nkv, rep, hd):
    """Grouped-query expansion: the forward is exactly ``unsqueeze(3).expand(...).flatten(2, 3)``; the backward is the
    sum over a head's copies, accumulated in fp32 and rounded once (bit-equal to the fp32 sum rounded to bf16)."""
    g = torch.Generator(device=DEV).manual_seed(b * 100 + s)
    x = torch.randn(b, s, nkv, hd, device=DEV, generator=g).to(BF).requires_grad_()
    y = layer_ops.repeat_kv(x, rep)
    want = x.detach().unsqueeze(3).expand(b, s, nkv, rep, hd).flatten(2, 3)
    assert y.shape == (b, s, nkv * rep, hd) and torch.equal(y, want)
    gy = torch.randn(b, s, nkv * rep, hd, device=DEV, generator=g).to(BF)
    y.backward(gy)
    gsum = torch.zeros(b, s, nkv, hd, device=DEV, dtype=torch.float32)
    for r in range(rep):  # the kernel's order
        gsum = gsum + gy.view(b, s, nkv, rep, hd)[:, :, :, r].float()
    assert torch.equal(x.grad, gsum.to(BF))
    with pytest.raises(ValueError):
        ops.repeat_kv(x.detach()[0], rep)
    with pytest.raises(ValueError):
        ops.repeat_kv_bwd(gy, rep + 1 if (nkv * rep) % (rep + 1) else rep * nkv * 2 + 1)


@pytest.mark.parametrize("b,s,nh,nkv,hd", [(2, 33, 8, 2, 128), (1, 7, 6, 2, 64), (3, 5, 8, 1, 8), (1, 4, 4, 4, 16), (2, 256, 32, 8, 128),
                                            (4, 2048, 32, 8, 128), (1, 4096, 64, 8, 128), (4, 2048, 32, 8, 64)])
def test_qkv_rope_repeat_equals_rope_then_repeat_bitwise(b, s, nh, nkv, hd):
    """``qkv_rope_repeat`` against ``apply_rope`` on q and k followed by ``repeat_kv`` on k and v: the three outputs and the
    gradients of q, k, v bit for bit (also with one key / value head per query head, where the expansion is a copy)."""
    g = torch.Generator().manual_seed(11)
    q0 = torch.randn(b, s, nh, hd, generator=g).to(BF).to(DEV)
    k0, v0 = (torch.randn(b, s, nkv, hd, generator=g).to(BF).to(DEV) for _ in range(2))
    gos = [torch.randn(b, s, nh, hd, generator=g).to(BF).to(DEV) for _ in range(3)]
    pos = torch.arange(s, dtype=torch.float32)
    theta = 1.0 / (10000.0 ** (torch.arange(0, hd, 2, dtype=torch.float32) / hd))
    ang = torch.outer(pos, theta)
    cache = torch.stack([ang.cos(), ang.sin()], dim=-1).to(DEV)
    rep = nh // nkv
    res = []
    for fused in (True, False):
        q, k, v = (t.clone().requires_grad_() for t in (q0, k0, v0))
        if fused:
            outs = layer_ops.qkv_rope_repeat(q, k, v, cache)
        else:
            outs = (layer_ops.apply_rope(q, cache), layer_ops.repeat_kv(layer_ops.apply_rope(k, cache), rep),
                    layer_ops.repeat_kv(v, rep))
        torch.autograd.backward(outs, gos)
        res.append([*outs, q.grad, k.grad, v.grad])
    for i, (x, y) in enumerate(zip(*res)):
        assert x.shape == y.shape and torch.equal(x, y), i


def test_qkv_rope_repeat_refuses_heads_that_do_not_divide():
    q = torch.zeros(1, 4, 6, 16, dtype=BF, device=DEV)
    k = torch.zeros(1, 4, 4, 16, dtype=BF, device=DEV)
    cache = torch.zeros(4, 8, 2, device=DEV)
    with pytest.raises(ValueError, match="heads"):
        ops.qkv_rope_repeat(q, k, k, cache)
