"""Pins for oracle/layer_oracle.py (RMSNorm, rotary embedding, SwiGLU): library routines, closed forms, invariants."""
import torch
import torch.nn.functional as F

from oracle import layer_oracle as lo


def test_rms_norm_against_library_routine_and_closed_forms():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 96, generator=g)
    w = torch.rand(96, generator=g) + 0.5
    torch.testing.assert_close(lo.rms_norm(x, w, 1e-5), F.rms_norm(x, (96,), w, 1e-5), rtol=1e-6, atol=1e-6)
    # with unit scale and eps -> 0 every output row has unit root mean square
    y = lo.rms_norm(x, torch.ones(96), 0.0)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(7), rtol=1e-5, atol=1e-5)
    # a constant row c normalises to sign(c) * scale / sqrt(1 + eps / c^2)
    c = torch.full((1, 96), -3.0)
    torch.testing.assert_close(lo.rms_norm(c, w, 0.9), (-w / (1 + 0.9 / 9.0) ** 0.5)[None], rtol=1e-6, atol=1e-6)
    # bf16: the normalised value is rounded to bf16 BEFORE the scale multiplies it
    xb = x.to(torch.bfloat16)
    wb = w.to(torch.bfloat16)
    xn = (xb.float() * torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)).to(torch.bfloat16)
    assert torch.equal(lo.rms_norm(xb, wb, 1e-5), xn * wb)


def test_rope_is_complex_multiplication_with_its_invariants():
    g = torch.Generator().manual_seed(1)
    b, s, nh, hd = 2, 9, 3, 16
    x = torch.randn(b, s, nh, hd, generator=g)
    cache = lo.rope_cache(s, hd, 10000.0)
    y = lo.rope(x, cache)
    # same thing as multiplying the pairs, seen as complex numbers, by exp(i * pos * theta_j)
    theta = 1.0 / (10000.0 ** (torch.arange(0, hd, 2).float() / hd))
    ang = torch.arange(s).float()[:, None] * theta[None]
    z = torch.view_as_complex(x.reshape(b, s, nh, hd // 2, 2).contiguous()) * torch.polar(torch.ones_like(ang), ang)[None, :, None]
    torch.testing.assert_close(y, torch.view_as_real(z).flatten(3), rtol=1e-5, atol=1e-5)
    # invariants: position 0 is untouched, every pair keeps its norm, the table holds cos^2 + sin^2 = 1
    assert torch.equal(y[:, 0], x[:, 0])
    torch.testing.assert_close(y.reshape(b, s, nh, -1, 2).norm(dim=-1), x.reshape(b, s, nh, -1, 2).norm(dim=-1), rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(cache.pow(2).sum(-1), torch.ones(s, hd // 2), rtol=1e-6, atol=1e-6)
    # rotating by the negated sines undoes it (what the kernel's backward relies on)
    inv = cache.clone()
    inv[..., 1] *= -1
    torch.testing.assert_close(lo.rope(y, inv), x, rtol=1e-5, atol=1e-5)


def test_swiglu_against_fp64_and_gradients():
    g = torch.Generator().manual_seed(2)
    a = torch.randn(5, 33, generator=g, dtype=torch.float64, requires_grad=True)
    u = torch.randn(5, 33, generator=g, dtype=torch.float64, requires_grad=True)
    want = a / (1 + torch.exp(-a)) * u
    torch.testing.assert_close(lo.swiglu(a, u), want)
    assert torch.autograd.gradcheck(lo.swiglu, (a, u))
    s = torch.sigmoid(a)
    ga, gu = torch.autograd.grad(lo.swiglu(a, u).sum(), (a, u))
    torch.testing.assert_close(ga, u * s * (1 + a * (1 - s)))
    torch.testing.assert_close(gu, a * s)


def test_cross_entropy_sum_closed_forms():
    # uniform logits: loss = log(V) per row; a dominant correct class: loss -> 0; ignored rows contribute nothing
    V = 50
    z = torch.zeros(3, V)
    t = torch.tensor([1, 7, -100])
    import math

    torch.testing.assert_close(lo.cross_entropy_sum(z, t), torch.tensor(2 * math.log(V)))
    big = torch.full((1, V), -30.0)
    big[0, 4] = 30.0
    assert float(lo.cross_entropy_sum(big, torch.tensor([4]))) < 1e-6
    # gradient = softmax - onehot
    x = torch.randn(2, V, dtype=torch.float64, requires_grad=True)
    tt = torch.tensor([3, 9])
    lo.cross_entropy_sum(x, tt).backward()
    want = torch.softmax(x.detach().float(), -1)
    want[0, 3] -= 1
    want[1, 9] -= 1
    torch.testing.assert_close(x.grad.float(), want, rtol=1e-5, atol=1e-6)
