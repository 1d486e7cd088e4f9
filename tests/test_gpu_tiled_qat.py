"""GPU parity of the 8da4w fake-quantised linear on the library's own GEMM: the weight's per-group int4 fake quantisation
written straight into the GEMM's tile order (``ttamd_fq_per_group_int4_sym_tiled_bf16``) and the plain tiled GEMM
(``ttamd_tiled_linear_bf16``) for forward and grad-input.

The staged values are checked bit for bit: with one-hot rows as activations every output of the GEMM is a single product
1 * fq(W)[n][k], so the GEMM's output IS the staged weight and must equal ``ops.fq_per_group_int4_sym`` (itself bit-exact
against the CPU oracle in tests/test_gpu_fake_quant.py) — for the forward tiles and for the transposed tiles."""
import pytest
import torch

from oracle import fake_quant_oracle as fq
from torchtune_amd import ops, qat
from torchtune_amd.qat import Int8DynActInt4WeightQATLinear

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def _weight(N, K, seed):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(N, K, generator=g) * 0.02).to(BF)
    w[0, :64] = 0                 # an all-zero group: the scale falls back to eps
    w[1, :32] = 7.5 * 0.01        # exact grid points
    w[2] = -w[2].abs()            # one-signed rows
    return w


def _one_hot(M, K):
    x = torch.zeros(M, K, dtype=BF, device=DEV)
    x[torch.arange(M, device=DEV), torch.arange(M, device=DEV) % K] = 1.0
    return x


@pytest.mark.parametrize("N,K,g", [(256, 512, 32), (192, 448, 64), (320, 1024, 128), (128, 768, 256)])
@pytest.mark.parametrize("scales", [torch.float32, torch.bfloat16])
def test_staged_fake_quantised_weight_is_bit_exact_in_both_layouts(N, K, g, scales):
    w = _weight(N, K, seed=N + K + g)
    want, want_scale = ops.fq_per_group_int4_sym(w.to(DEV), g, qparam_dtype=scales)
    ref, ref_scale = fq.fq_per_group_int4_sym(w, g) if scales == torch.float32 else (None, None)
    if ref is not None:  # the row-major kernel against the oracle, for completeness of the chain
        assert torch.equal(want.cpu().view(torch.int16), ref.view(torch.int16)) and torch.equal(want_scale.cpu(), ref_scale)
    tf, tb, scale = ops.fq_per_group_int4_sym_tiled(w.to(DEV), g, qparam_dtype=scales)
    assert torch.equal(scale, want_scale)
    M = max(K, N)
    y = ops.tiled_linear(_one_hot(M, K), tf, N)            # row m = column m % K of fq(W)
    assert torch.equal(y[:K].view(torch.int16), want.t().contiguous().view(torch.int16))
    gx = ops.tiled_linear(_one_hot(M, N), tb, K)           # row m = row m % N of fq(W)
    assert torch.equal(gx[:N].view(torch.int16), want.view(torch.int16))
    only_f = ops.fq_per_group_int4_sym_tiled(w.to(DEV), g, backward=False, want_scale=False, qparam_dtype=scales)
    assert only_f[1] is None and only_f[2] is None and torch.equal(only_f[0], tf)


@pytest.mark.parametrize("N,K", [(14336, 4096), (4096, 14336), (128256, 4096)])
def test_staged_weight_at_the_full_sizes_of_the_8b_qat_configuration(N, K):
    """gate / up, down and the output projection at their real sizes (``torchtune/models/llama3_1/_model_builders.py:20-59``),
    group 32 as in ``recipes/configs/llama3_1/8B_qat_full.yaml``: every staged value of both layouts, read back through
    the GEMM with one-hot activations, equals the row-major fake quantisation bit for bit."""
    g = 32
    w = _weight(N, K, seed=N + K).to(DEV)
    want, want_scale = ops.fq_per_group_int4_sym(w, g)
    tf, tb, scale = ops.fq_per_group_int4_sym_tiled(w, g)
    assert torch.equal(scale, want_scale)
    rows = 4096
    assert K >= rows and N >= rows
    for k0 in sorted(set(range(0, K - rows + 1, rows)) | {K - rows}):   # forward tiles: row m = column k0 + m of fq(W)
        x = torch.zeros(rows, K, dtype=BF, device=DEV)
        x[torch.arange(rows, device=DEV), k0 + torch.arange(rows, device=DEV)] = 1.0
        y = ops.tiled_linear(x, tf, N)
        assert torch.equal(y.view(torch.int16), want[:, k0:k0 + rows].t().contiguous().view(torch.int16)), k0
    bases = {0, (N // 2 // 256) * 256, N - rows} if N > 4 * rows else set(range(0, N - rows + 1, rows)) | {N - rows}
    for n0 in sorted(bases):                                     # transposed tiles: row m = row n0 + m of fq(W)
        gy = torch.zeros(rows, N, dtype=BF, device=DEV)
        gy[torch.arange(rows, device=DEV), n0 + torch.arange(rows, device=DEV)] = 1.0
        gx = ops.tiled_linear(gy, tb, K)
        assert torch.equal(gx.view(torch.int16), want[n0:n0 + rows].view(torch.int16)), n0


def test_unsupported_group_size_is_refused():
    w = _weight(128, 512, 1).to(DEV)
    with pytest.raises(ValueError):
        ops.fq_per_group_int4_sym_tiled(w, 16)


@pytest.mark.parametrize("bias", [False, True])
def test_qat_linear_on_the_tiled_gemm_vs_oracle_and_vs_default_path(bias, monkeypatch):
    gen = torch.Generator().manual_seed(5)
    N, K, M, g = 320, 512, 2048 + 19, 32
    w = (torch.randn(N, K, generator=gen) * 0.02).to(BF)
    b = (torch.randn(N, generator=gen) * 0.1).to(BF) if bias else None
    x = torch.randn(M, K, generator=gen).to(BF)

    def run(tiled):
        monkeypatch.setattr(qat, "TILED_GEMM", tiled)
        monkeypatch.setattr(qat, "TILED_GEMM_MIN_TILES", 0)   # a small layer: the path is chosen from a full round of tiles up
        lin = Int8DynActInt4WeightQATLinear(K, N, bias=bias, device=DEV, groupsize=g, precision=BF)
        with torch.no_grad():
            lin.weight.copy_(w)
            if bias:
                lin.bias.copy_(b)
        xd = x.to(DEV).requires_grad_()
        assert lin._tiled_ok(xd) == tiled
        y = lin(xd)
        (y.float() ** 2).sum().backward()
        return y.detach(), xd.grad, lin.weight.grad, (lin.bias.grad if bias else None), lin.weight_fake_quantizer.scale

    y1, gx1, gw1, gb1, s1 = run(True)
    y0, gx0, gw0, gb0, s0 = run(False)
    assert torch.equal(s1, s0)
    torch.testing.assert_close(y1.float(), y0.float(), rtol=1e-2, atol=2e-3)
    torch.testing.assert_close(gx1.float(), gx0.float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(gw1.float(), gw0.float(), rtol=2e-2, atol=2e-2 * float(gw0.float().abs().max()))
    if bias:
        torch.testing.assert_close(gb1.float(), gb0.float(), rtol=1e-2, atol=1e-2 * float(gb0.float().abs().max()))
    # the CPU oracle (the reference's op sequence)
    xo, wo = x.clone().requires_grad_(), w.clone().requires_grad_()
    yo = fq.fake_quantized_linear(xo, wo, g)
    if bias:
        yo = yo + b
    (yo.float() ** 2).sum().backward()
    torch.testing.assert_close(y1.cpu().float(), yo.detach().float(), rtol=1e-2, atol=1e-2)
    gxo = xo.grad.float()
    torch.testing.assert_close(gx1.cpu().float(), gxo, rtol=1e-2, atol=1e-2 * max(1.0, float(gxo.abs().max()) / 8))
    gwo = wo.grad.float()
    torch.testing.assert_close(gw1.cpu().float(), gwo, rtol=2e-2, atol=2e-2 * float(gwo.abs().max()))


@pytest.mark.parametrize("Ns,K,bias", [((512, 256, 256), 512, False), ((1024, 1024), 256, True)], ids=["qkv", "gate_up_bias"])
def test_fake_quantized_group_matches_layer_by_layer(Ns, K, bias, monkeypatch):
    """``fake_quantized_linear_group`` (q / k / v, gate / up of a fake-quantised model as one node) against calling the
    layers in turn on the same tiled GEMM: outputs bit for bit (the same kernel on the same tiles, whatever launch the
    member's columns ride in), weight and bias gradients bit for bit (the same products), the grad-input within rtol 1e-2
    (the group sums the members in fp32 inside the GEMM, the layer-by-layer path rounds each member to bf16 and adds)
    and at least as close to the fp32 evaluation; the stacked tiles hold each member's ``fq_per_group_int4_sym`` values
    bit for bit (one-hot read-back); every quantizer records the scales of its own weight."""
    monkeypatch.setattr(qat, "TILED_GEMM_MIN_TILES", 0)
    gen = torch.Generator().manual_seed(len(Ns) + K)
    M, g = 2048 + 64, 32
    layers = []
    for N in Ns:
        lin = Int8DynActInt4WeightQATLinear(K, N, bias=bias, device=DEV, groupsize=g, precision=BF)
        with torch.no_grad():
            lin.weight.copy_((torch.randn(N, K, generator=gen) * 0.02).to(BF))
            if bias:
                lin.bias.copy_((torch.randn(N, generator=gen) * 0.1).to(BF))
        layers.append(lin)
    x = torch.randn(M, K, generator=gen).to(BF).to(DEV)
    gys = [torch.randn(M, N, generator=gen).to(BF).to(DEV) for N in Ns]

    def run(group):
        for l in layers:
            l.zero_grad()
        xd = x.clone().requires_grad_()
        assert qat._group_tiled_ok(xd, layers)
        ys = qat.fake_quantized_linear_group(xd, layers) if group else tuple(l(xd) for l in layers)
        torch.autograd.backward(ys, gys)
        return ([y.detach() for y in ys], xd.grad, [l.weight.grad.clone() for l in layers],
                [l.bias.grad.clone() if bias else None for l in layers], [l.weight_fake_quantizer.scale.clone() for l in layers])

    ys1, gx1, gw1, gb1, sc1 = run(True)
    ys0, gx0, gw0, gb0, sc0 = run(False)
    for a, b in zip(ys1, ys0):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for a, b in zip(gw1, gw0):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for a, b in zip(sc1, sc0):
        assert torch.equal(a, b)
    if bias:
        for a, b in zip(gb1, gb0):
            assert torch.equal(a, b)
    want = sum(gy.float() @ ops.fq_per_group_int4_sym(l.weight.detach(), g)[0].float() for gy, l in zip(gys, layers))
    scale = max(1.0, float(want.abs().max()) / 8)
    torch.testing.assert_close(gx1.float(), want, rtol=1e-2, atol=1e-2 * scale)
    assert float((gx1.float() - want).abs().max()) <= float((gx0.float() - want).abs().max()) + 1e-3 * scale
    # the stacks, read back through the group GEMMs with one-hot activations
    tf, tb, _ = ops.fq_int4_sym_tiled_group([l.weight.detach() for l in layers], g)
    eye = torch.zeros(max(K, 2048), K, dtype=BF, device=DEV)
    eye[torch.arange(K, device=DEV), torch.arange(K, device=DEV)] = 1.0
    for y, l in zip(ops.tiled_linear_group_fwd(eye, tf, list(Ns)), layers):
        want_w = ops.fq_per_group_int4_sym(l.weight.detach(), g)[0]
        assert torch.equal(y[:K].view(torch.int16), want_w.t().contiguous().view(torch.int16))
    for i, l in enumerate(layers):   # row m of gy_i one-hot at column m: gx row m = row m of fq(W_i); the other members are zero
        want_w = ops.fq_per_group_int4_sym(l.weight.detach(), g)[0]
        rows = max(Ns[i], 2048)
        hot = [torch.zeros(rows, N, dtype=BF, device=DEV) for N in Ns]
        hot[i][torch.arange(Ns[i], device=DEV), torch.arange(Ns[i], device=DEV)] = 1.0
        gx = ops.tiled_linear_group_dx(hot, tb, K)
        assert torch.equal(gx[:Ns[i]].view(torch.int16), want_w.view(torch.int16))


@pytest.mark.parametrize("N,K,M", [(1024, 256, 2048 + 64), (4096, 512, 2048)], ids=["small", "full_round"])
def test_fake_quantized_gated_pair_matches_group_then_swiglu(N, K, M, monkeypatch):
    """``fake_quantized_swiglu_group`` (gate / up of a fake-quantised feed-forward with ``silu(gate) * up`` written by the
    pair's GEMM launch, forward tiles in the paired layout) against the plain group followed by the stand-alone SwiGLU op:
    the product and every gradient bit for bit."""
    from torchtune_amd.modules import layer_ops

    monkeypatch.setattr(qat, "TILED_GEMM_MIN_TILES", 0)
    gen = torch.Generator().manual_seed(N + K)
    g = 32
    layers = []
    for _ in range(2):
        lin = Int8DynActInt4WeightQATLinear(K, N, bias=False, device=DEV, groupsize=g, precision=BF)
        with torch.no_grad():
            lin.weight.copy_((torch.randn(N, K, generator=gen) * 0.05).to(BF))
        layers.append(lin)
    x = torch.randn(M, K, generator=gen).to(BF).to(DEV)
    gact = torch.randn(M, N, generator=gen).to(BF).to(DEV)

    def run(gated):
        for l in layers:
            l.zero_grad()
        xd = x.clone().requires_grad_()
        if gated:
            act = qat.fake_quantized_swiglu_group(xd, layers[0], layers[1])
            assert act is not None
        else:
            gg, uu = qat.fake_quantized_linear_group(xd, layers)
            act = layer_ops.swiglu(gg, uu)
        act.backward(gact)
        return [act.detach(), xd.grad] + [l.weight.grad.clone() for l in layers]

    for a, b in zip(run(True), run(False)):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    layers[1].weight_fake_quantizer.enabled = False
    assert qat.fake_quantized_swiglu_group(x, layers[0], layers[1]) is None



def test_output_projection_and_loss_as_one_node_equals_the_two_nodes():
    """``FakeQuantizedLinear.cross_entropy_sum``: the fake-quantised vocabulary projection and the loss of a chunk of rows
    as one autograd node against the layer followed by ``layer_ops.cross_entropy_sum``.  With the loss's own gradient (1)
    coming in: the same loss, input gradient and weight gradient bit for bit (the factor multiplies other operands, and
    multiplying by one is exact); with another factor: within a rounding of bf16."""
    from torchtune_amd.modules import layer_ops

    M, K, N = 2048, 8192, 8192
    gen = torch.Generator(device=DEV).manual_seed(21)
    layer = Int8DynActInt4WeightQATLinear(K, N, bias=False, groupsize=32, device=DEV, precision=BF)
    with torch.no_grad():
        layer.weight.copy_((torch.randn(N, K, device=DEV, generator=gen) * 0.02).to(BF))
    x = torch.randn(M, K, device=DEV, generator=gen).to(BF)
    target = torch.randint(0, N, (M,), device=DEV, generator=gen)
    target[::7] = -100

    def run(fused: bool, factor: float):
        layer.zero_grad(set_to_none=True)
        xg = x.clone().requires_grad_()
        if fused:
            loss = layer.cross_entropy_sum(xg, target, scale=1.0 / M)
            assert loss is not None
        else:
            loss = layer_ops.cross_entropy_sum(layer(xg), target, scale=1.0 / M)
        (loss * factor).backward()
        return loss.detach(), xg.grad, layer.weight.grad

    a, b = run(True, 1.0), run(False, 1.0)
    assert torch.equal(a[0], b[0])
    assert torch.equal(a[1].view(torch.int16), b[1].view(torch.int16))
    assert torch.equal(a[2].view(torch.int16), b[2].view(torch.int16))
    assert float(a[2].float().abs().max()) > 0
    a, b = run(True, 3.0), run(False, 3.0)
    for u, v in zip(a[1:], b[1:]):
        torch.testing.assert_close(u.float(), v.float(), rtol=2.0 ** -6, atol=2.0 ** -7 * float(v.float().abs().max()))
    # a layer with a bias, or too small for the library's own GEMM, is left to the caller
    small = Int8DynActInt4WeightQATLinear(256, 512, bias=False, groupsize=32, device=DEV, precision=BF)
    assert small.cross_entropy_sum(torch.randn(64, 256, device=DEV).to(BF), torch.zeros(64, dtype=torch.long, device=DEV)) is None
