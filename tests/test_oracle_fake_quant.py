"""Pins the fake-quant oracle (oracle/fake_quant_oracle.py, oracle/nf4_ref.c): closed forms, grid and range
invariants, idempotence, tiny exhaustive cases, agreement of the two restatements, straight-through backward."""
import pytest
import torch

from oracle import fake_quant_oracle as fq
from tests.helpers import bits_equal, c_fq_per_group, c_fq_per_token

DTYPES = [torch.bfloat16, torch.float32]
EPS = torch.finfo(torch.float32).eps


def test_per_token_qparams_closed_form():
    # row spanning [-1, 3]: scale = 4/255; zp: descaled min = -63.75, max = 191.25;
    # (-128 - 63.75) + (127 + 191.25) > 0 -> zp = qmin - descaled_min = -128 + 63.75 = -64.25 -> round -> -64
    x = torch.tensor([[-1.0, 0.5, 3.0, 0.0]])
    scale, zp = fq.choose_qparams_per_token_asym(x)
    assert scale.item() == pytest.approx(4.0 / 255.0, rel=1e-7)
    assert zp.item() == -64 and zp.dtype == torch.int32 and scale.dtype == torch.float32
    # all-positive row: the range is widened to include 0 -> min 0 maps to qmin exactly
    x = torch.tensor([[1.0, 2.0, 4.0, 3.0]])
    scale, zp = fq.choose_qparams_per_token_asym(x)
    assert scale.item() == pytest.approx(4.0 / 255.0, rel=1e-7) and zp.item() == -128
    # all-negative row -> max 0 maps to qmax
    scale, zp = fq.choose_qparams_per_token_asym(-x)
    assert zp.item() == 127
    # all-zero row: scale falls back to eps, zero-point stays in range, output is exactly zero
    out, scale, zp = fq.fq_per_token_int8_asym(torch.zeros(1, 8))
    assert scale.item() == EPS and -128 <= zp.item() <= 127 and torch.all(out == 0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_per_token_outputs_lie_on_the_grid(dtype):
    g = torch.Generator().manual_seed(0)
    x = (torch.randn(16, 256, generator=g) * 3).to(dtype)
    out, scale, zp = fq.fq_per_token_int8_asym(x)
    assert out.dtype == dtype and out.shape == x.shape
    # every output equals dtype(k * scale) for an integer k in [qmin - zp, qmax - zp]
    k = torch.round(out.float() / scale[:, None])
    assert torch.all(k >= (-128 - zp)[:, None]) and torch.all(k <= (127 - zp)[:, None])
    assert bits_equal((k.to(dtype) * scale[:, None]).to(dtype), out)
    # quantisation error of in-range values is at most half a step (plus the dtype's own rounding)
    tol = 0.5 * scale[:, None] + out.float().abs() * (2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -23)
    assert torch.all((out.float() - x.float()).abs() <= tol * 1.0001)
    # the row extremes are representable: min/max are reproduced within half a step
    assert torch.all((out.float().amax(1) - x.float().amax(1).clamp(min=0)).abs() <= scale)


def test_per_token_fixed_qparams_idempotent():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(8, 128, generator=g)
    scale, zp = fq.choose_qparams_per_token_asym(x)
    _, once = fq._fake_quantize(x, scale, zp, -128, 127)
    _, twice = fq._fake_quantize(once, scale, zp, -128, 127)
    assert torch.equal(once, twice)


def test_per_token_tiny_exhaustive():
    # rows of 2 values on a coarse grid: brute-force nearest grid point (ties to even code) must match
    vals = torch.linspace(-2, 2, 17)
    for a in vals:
        for b in vals:
            x = torch.tensor([[a.item(), b.item()]])
            out, scale, zp = fq.fq_per_token_int8_asym(x)
            codes = torch.arange(-128, 128)
            grid = (codes - zp.item()).float() * scale.item()
            for j in range(2):
                pos = x[0, j] * (1.0 / scale.item())
                q = int(torch.clamp(torch.round(pos) + zp.item(), -128, 127).item())
                assert out[0, j].item() == grid[q + 128].item()
                assert abs(out[0, j].item() - x[0, j].item()) <= 0.5 * scale.item() * 1.001


def test_per_group_closed_form():
    # one group [-7.5 .. 7.5]: amax 7.5 -> scale exactly 1; codes = round half to even, clamped to [-8, 7]
    w = torch.tensor([[-7.5, -6.5, -0.5, 0.5, 1.5, 2.5, 7.4, 7.5]])
    out, scale = fq.fq_per_group_int4_sym(w, 8)
    assert scale.item() == 1.0
    assert out.tolist() == [[-8.0, -6.0, -0.0 + 0.0, 0.0, 2.0, 2.0, 7.0, 7.0]]  # 7.5 -> round 8 -> clamp 7
    q, s2, zeros = fq.quantize_per_group_int4(w, 8)
    assert q.dtype == torch.int8 and q.tolist() == [[-8, -6, 0, 0, 2, 2, 7, 7]]
    assert torch.equal(s2, scale) and torch.all(zeros == 0)
    # a zero group: eps scale, zero output
    out, scale = fq.fq_per_group_int4_sym(torch.zeros(1, 8), 8)
    assert scale.item() == EPS and torch.all(out == 0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("g", [8, 32, 256])
def test_per_group_invariants(dtype, g):
    gen = torch.Generator().manual_seed(2)
    w = (torch.randn(32, 512, generator=gen) * 0.02).to(dtype)
    out, scale = fq.fq_per_group_int4_sym(w, g)
    q, s2, _ = fq.quantize_per_group_int4(w, g)
    assert torch.equal(scale, s2) and scale.shape == (32, 512 // g)
    assert int(q.min()) >= -8 and int(q.max()) <= 7
    amax = w.float().view(32, -1, g).abs().amax(-1)
    assert torch.equal(scale, (amax / 7.5).clamp(min=EPS))
    # fake-quant output == dequantised convert() output
    deq = (q.view(32, -1, g).to(dtype) * scale[..., None]).to(dtype).view(32, 512)
    assert bits_equal(deq, out)
    # the group's absmax element maps to +-7.5 up to rounding of w * (1/scale) -> code 7, -7 or -8
    idx = w.float().view(32, -1, g).abs().argmax(-1, keepdim=True)
    at = q.view(32, -1, g).gather(-1, idx)
    assert torch.all((at == 7) | (at == -7) | (at == -8) | (amax[..., None] == 0))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("scale_dtype", [torch.float32, torch.bfloat16])
def test_two_restatements_agree(c_oracle, dtype, scale_dtype):
    qp_bf16 = scale_dtype == torch.bfloat16
    gen = torch.Generator().manual_seed(3)
    x = (torch.randn(64, 512, generator=gen) * 2).to(dtype)
    x[3] = 0
    x[4] = x[4].abs()
    ot, st, zt = fq.fq_per_token_int8_asym(x, scale_dtype)
    oc, sc, zc = c_fq_per_token(c_oracle, x, qp_bf16)
    assert bits_equal(ot, oc) and torch.equal(st, sc) and torch.equal(zt, zc)
    w = (torch.randn(64, 512, generator=gen) * 0.02).to(dtype)
    w[0, :32] = 0
    for g in (8, 32, 128):
        ft, s1 = fq.fq_per_group_int4_sym(w, g, scale_dtype)
        qt, _, _ = fq.quantize_per_group_int4(w, g, scale_dtype)
        fc, qc, s2 = c_fq_per_group(c_oracle, w, g, qp_bf16)
        assert bits_equal(ft, fc) and torch.equal(qt, qc) and torch.equal(s1, s2)


def test_bf16_scale_precision_rounds_the_scale_before_use():
    """scale_precision = bf16: the scale the kernel reports is a bf16 value, the zero point is the one chosen with the
    fp32 scale, and outputs lie on the grid of the ROUNDED scale."""
    gen = torch.Generator().manual_seed(12)
    x = torch.randn(16, 256, generator=gen) * 1.3
    o32, s32, z32 = fq.fq_per_token_int8_asym(x)
    o16, s16, z16 = fq.fq_per_token_int8_asym(x, torch.bfloat16)
    assert torch.equal(z32, z16) and torch.equal(s16, s32.to(torch.bfloat16).float()) and not torch.equal(s16, s32)
    k = torch.round(o16 / s16[:, None])
    assert bits_equal(k * s16[:, None], o16) and not bits_equal(o16, o32)
    w = torch.randn(8, 256, generator=gen) * 0.02
    f16, sw16 = fq.fq_per_group_int4_sym(w, 32, torch.bfloat16)
    _, sw32 = fq.fq_per_group_int4_sym(w, 32)
    assert torch.equal(sw16, sw32.to(torch.bfloat16).float())
    kk = torch.round(f16.view(8, 8, 32) / sw16[..., None])
    assert bits_equal((kk * sw16[..., None]).view(8, 256), f16) and kk.abs().max() <= 8
    q16, _, _ = fq.quantize_per_group_int4(w, 32, torch.bfloat16)
    assert torch.equal(q16.float().view(8, 8, 32), kk)


def test_straight_through_backward():
    gen = torch.Generator().manual_seed(4)
    x = torch.randn(4, 64, generator=gen, requires_grad=True)
    w = (torch.randn(16, 64, generator=gen) * 0.1).requires_grad_()
    y = fq.fake_quantized_linear(x, w, 32)
    gy = torch.randn(4, 16, generator=gen)
    y.backward(gy)
    x_fq = fq.fq_per_token_int8_asym(x.detach())[0]
    w_fq = fq.fq_per_group_int4_sym(w.detach(), 32)[0]
    torch.testing.assert_close(y, x_fq @ w_fq.T)
    torch.testing.assert_close(x.grad, gy @ w_fq)  # gradient passes straight through both fake quantisers
    torch.testing.assert_close(w.grad, gy.T @ x_fq)


# ---- weight-only int4 ("4w-qat"): asymmetric uint4 with a floating-point zero point --------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_uint4_asym_closed_form(dtype):
    # a group that is exactly the 16-point grid min + k * step: scale = step, zero = min + 8 * step, codes = k,
    # fake quantisation is the identity (all values exact in bf16)
    k = torch.arange(16, dtype=torch.float32)
    for lo, step in ((-1.0, 0.125), (1.0, 0.125), (-4.0, 0.25)):
        w = (lo + step * k).to(dtype)[None, :]
        out, scale, zero = fq.fq_per_group_uint4_asym(w, 16)
        assert scale.dtype == torch.bfloat16 and zero.dtype == torch.bfloat16
        assert scale.item() == step and zero.item() == lo + 8 * step
        assert bits_equal(out, w)
        packed, _, _ = fq.quantize_per_group_uint4(w, 16)
        # even element in the high nibble
        assert packed.tolist() == [[(2 * i) << 4 | (2 * i + 1) for i in range(8)]]
    # the range is NOT widened to include zero: an all-positive group keeps its own minimum as code 0
    w = torch.tensor([[1.0, 2.875] + [2.0] * 14]).to(dtype)
    packed, scale, zero = fq.quantize_per_group_uint4(w, 16)
    assert scale.item() == 0.125 and zero.item() == 2.0 and packed[0, 0].item() == (0 << 4) | 15
    # a constant group: scale falls back to 1e-6 (rounded to the qparam dtype) and the value survives within a step
    w = torch.full((1, 16), 0.5).to(dtype)
    out, scale, zero = fq.fq_per_group_uint4_asym(w, 16)
    assert scale.item() == torch.tensor(1e-6).to(torch.bfloat16).item()
    assert torch.all((out.float() - 0.5).abs() <= 2.0 ** -8)


@pytest.mark.parametrize("g", [32, 128, 256])
def test_uint4_asym_invariants(g):
    gen = torch.Generator().manual_seed(3)
    w = torch.randn(24, 512, generator=gen) * 0.05 + 0.01
    out, scale, zero = fq.fq_per_group_uint4_asym(w, g, qparam_dtype=torch.float32)
    packed, s2, z2 = fq.quantize_per_group_uint4(w, g, qparam_dtype=torch.float32)
    assert torch.equal(scale, s2) and torch.equal(zero, z2)
    codes = torch.stack([packed >> 4, packed & 15], dim=-1).reshape(24, 512).float()
    assert codes.min() == 0 and codes.max() == 15
    wg, cg = w.view(24, 512 // g, g), codes.view(24, 512 // g, g)
    # the group minimum takes code 0 and the maximum code 15
    assert torch.all(cg.gather(-1, wg.argmin(-1, keepdim=True)) == 0)
    assert torch.all(cg.gather(-1, wg.argmax(-1, keepdim=True)) == 15)
    # codes are monotone in the value, the error is at most half a step (fp32 arithmetic slack aside)
    order = wg.argsort(-1)
    assert torch.all(cg.gather(-1, order).diff(dim=-1) >= 0)
    assert torch.all((out - w).view(24, 512 // g, g).abs() <= 0.5 * scale[..., None] * 1.001)
    # brute force: the chosen code is the nearest of the 16 grid points zero + (q - 8) * scale
    grid = zero[..., None, None] + (torch.arange(16.0) - 8.0) * scale[..., None, None]  # [rows, G, 1, 16]
    dist = (wg[..., None] - grid).abs()
    best = dist.min(-1).values
    chosen = dist.gather(-1, cg.long()[..., None])[..., 0]
    assert torch.all(chosen <= best + 1e-6 * scale[..., None])
    # dequantising the packed codes reproduces the fake-quantised tensor bit for bit
    assert bits_equal(fq.dequantize_per_group_uint4(packed, scale, zero, g, torch.float32), out)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("qp", [torch.bfloat16, torch.float32])
def test_uint4_asym_two_restatements_agree(c_oracle, dtype, qp):
    from tests.helpers import c_fq_per_group_uint4_asym

    gen = torch.Generator().manual_seed(4)
    for g, std, shift in ((32, 0.02, 0.0), (64, 1.0, 0.3), (256, 5.0, -2.0), (8, 1e-7, 0.0)):
        w = (torch.randn(16, 512, generator=gen) * std + shift).to(dtype)
        out, scale, zero = fq.fq_per_group_uint4_asym(w, g, qparam_dtype=qp)
        packed, _, _ = fq.quantize_per_group_uint4(w, g, qparam_dtype=qp)
        fc, qc, sc, zc = c_fq_per_group_uint4_asym(c_oracle, w, g, qp == torch.bfloat16)
        assert bits_equal(scale.float(), sc) and bits_equal(zero.float(), zc)
        assert torch.equal(torch.stack([packed >> 4, packed & 15], dim=-1).reshape(16, 512), qc)
        assert bits_equal(out, fc)
        assert bits_equal(fq.dequantize_per_group_uint4(packed, scale, zero, g, dtype), out)


# ---- an independent implementation: the quantized_decomposed ops that ship inside PyTorch itself -------------
def _decomposed_ops():
    from torch.ao.quantization.fx import _decomposed  # noqa: F401  (registers torch.ops.quantized_decomposed)

    return torch.ops.quantized_decomposed


def test_per_token_agrees_with_pytorchs_own_decomposed_ops():
    """torch/ao/quantization/fx/_decomposed.py holds PyTorch's implementation of the same 8-bit dynamic per-token
    asymmetric scheme (qparams after XNNPACK, quantise = mul(1/scale).add(zp).round().clamp, dequantise = (q - zp) * scale).
    The oracle must give the same qparams, codes and fake-quantised values on fp32 rows."""
    ops = _decomposed_ops()
    gen = torch.Generator().manual_seed(7)
    x = torch.randn(64, 384, generator=gen) * 2.5
    x[0] = 0
    x[1] = x[1].abs() + 0.5
    x[2] = -x[2].abs() - 0.5
    x[3, ::3] *= 40
    scale, zp = ops.choose_qparams_per_token_asymmetric(x, torch.int8)
    got, s, z = fq.fq_per_token_int8_asym(x)
    assert torch.equal(scale.to(torch.float32).reshape(-1), s) and torch.equal(zp.to(torch.int32).reshape(-1), z)
    q = ops.quantize_per_token(x, scale.to(torch.float32), zp.to(torch.int32), -128, 127, torch.int8)
    dq = ops.dequantize_per_token(q, scale.to(torch.float32), zp.to(torch.int32), -128, 127, torch.int8, torch.float32)
    assert bits_equal(dq, got)
    q_oracle, _ = fq._fake_quantize(x, s[:, None], z[:, None], -128, 127)
    assert torch.equal(q.to(torch.float32), q_oracle)


@pytest.mark.parametrize("g", [32, 256])
def test_per_group_agrees_with_pytorchs_own_decomposed_ops(g):
    """Same for the group-wise int4 weights: with the oracle's scales, PyTorch's quantize_per_channel_group /
    dequantize_per_channel_group give the oracle's int4 codes and fake-quantised weight."""
    ops = _decomposed_ops()
    gen = torch.Generator().manual_seed(8)
    w = torch.randn(48, 512, generator=gen) * 0.03
    w[0, :g] = 0
    want, scale = fq.fq_per_group_int4_sym(w, g)
    codes, s2, zeros = fq.quantize_per_group_int4(w, g)
    assert torch.equal(scale, s2) and torch.all(zeros == 0)
    zp = torch.zeros_like(scale, dtype=torch.int32)
    q = ops.quantize_per_channel_group(w, scale, zp, -8, 7, torch.int8, g)
    assert torch.equal(q, codes)
    dq = ops.dequantize_per_channel_group(q, scale, zp, -8, 7, torch.int8, g, torch.float32)
    assert bits_equal(dq, want)
