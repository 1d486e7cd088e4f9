"""Groups of LoRA linears with a common input (q/k/v, gate/up) on the GPU.

What is compared with what:

* ``h_cat``, every ``y_i`` and ``gh_cat`` against the member-by-member entry points: bit for bit (the group kernels sum
  in the same order);
* ``grad A_i`` / ``grad B_i`` against the member-by-member call: the fp32 partial sums are taken over row ranges chosen
  for the whole batch, so the values agree up to the order of fp32 additions (rtol 1e-2, atol 1e-2 of the largest
  entry; both sides are bf16 roundings of fp32 sums of the same products);
* the grouped grad-input against an fp32 evaluation on the bit-exact dequantised weights (rtol 1e-2 / atol scaled like
  the per-linear tests) and against the sum of the member-by-member results (which rounds each member to bf16 first:
  the grouped value must be at least as close to the fp32 evaluation);
* the module-level function against the CPU oracle's unfused graph of the same layers (rtol 1e-2 / atol 1e-2, the bar of
  the per-linear tests), and against calling the layers one by one.
"""
import pytest
import torch

from oracle import lora_oracle, nf4_oracle
from torchtune_amd import ops
from torchtune_amd.modules import layer_ops
from torchtune_amd.modules.peft import LoRALinear, group_applies, lora_feed_forward, lora_linear_group, lora_swiglu_group
from torchtune_amd.nf4_tensor import to_nf4

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def _members(K, Ns, ranks, seed, bias=False):
    g = torch.Generator().manual_seed(seed)
    out = []
    for N, r in zip(Ns, ranks):
        W = (torch.randn(N, K, generator=g) * 0.02).to(BF)
        A = lora_oracle.lora_a_init_(torch.empty(r, K), g).to(BF)
        B = (torch.randn(N, r, generator=g) * 0.01).to(BF)
        b = (torch.randn(N, generator=g) * 0.1).to(BF) if bias else None
        t = to_nf4(W.to(DEV))
        m = ops.GroupMember(t.quantized_data, t.block_scalers(), t.backward_copy(), A.to(DEV), B.to(DEV),
                            b.to(DEV) if bias else None, 32.0 / r, N)
        out.append((m, t, W, A, B, b))
    return out


SHAPES = [
    # M, K, Ns, ranks
    (1, 512, (256, 64, 64), (8, 8, 8)),
    (16, 1024, (512, 128, 128), (16, 16, 16)),
    (33, 2048, (8192, 8192), (16, 16)),            # wide members: two row tiles per workgroup
    (64, 8192, (512, 64, 64), (8, 16, 8)),          # deep contraction: sixteen waves
    (40, 1024, (8192, 256), (16, 16)),              # members with different launch shapes: two launches
    (200, 512, (256, 128, 128), (16, 16, 16)),      # tiled kernels, sliced contraction
    (1000, 1024, (512, 256, 256, 64), (32, 16, 8, 8)),
    (4096, 1024, (1024, 256, 256), (16, 16, 16)),   # 256-row tiles, unsliced rank-r products
    (2048, 256, (4096, 4096), (32, 32)),
    (2048, 256, (4096, 4096), (40, 24)),            # many-token launch, a rank beyond 32: two steps of adapter operands
    (2048, 64, (4096, 2048, 2048), (8, 16, 8)),     # many-token launch over the shortest contraction
]


@pytest.mark.parametrize("M,K,Ns,ranks", SHAPES, ids=[f"M{s[0]}_K{s[1]}_{'x'.join(map(str, s[2]))}_r{'x'.join(map(str, s[3]))}" for s in SHAPES])
@pytest.mark.parametrize("bias", [False, True], ids=["nobias", "bias"])
def test_group_forward_matches_member_calls_bitwise(M, K, Ns, ranks, bias):
    """Bit-equal wherever the group and the member call run the same kernel.  A group of many tokens can reach the 256
    output tiles of the expanded-weight GEMM where a member alone does not (then the member runs the fused kernel, with
    another order of summation inside the matrix instructions): those members are compared at rtol 1e-2 / atol 2e-3."""
    from torchtune_amd import _lib

    lib = _lib.load()
    mem = _members(K, Ns, ranks, seed=M + K, bias=bias)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(7)).to(BF).to(DEV)
    h_cat, ys = ops.lora_group_fwd(x, [m[0] for m in mem])
    group_expands = all(N % 256 == 0 for N in Ns) and bool(lib.ttamd_nf4_gemm_expands_weight(M, sum(Ns), K))
    off = 0
    for (m, t, *_), y in zip(mem, ys):
        r = m.lora_a.shape[0]
        h = ops.lora_hidden(x, m.lora_a)
        assert torch.equal(h_cat[:, off:off + r], h), "hidden activation"
        y1 = ops.nf4_lora_linear_fwd(x, m.qdata, m.block_scalers, m.N, h, m.lora_b, m.scale, m.bias,
                                     block_scalers_t=m.transposed[1])
        if group_expands and not lib.ttamd_nf4_gemm_expands_weight(M, m.N, K):
            torch.testing.assert_close(y.float(), y1.float(), rtol=1e-2, atol=2e-3)
        else:
            assert torch.equal(y, y1), "member output"
        off += r
    assert off == h_cat.shape[1]


@pytest.mark.parametrize("M,K,Ns,ranks", SHAPES, ids=[f"M{s[0]}_K{s[1]}_{'x'.join(map(str, s[2]))}_r{'x'.join(map(str, s[3]))}" for s in SHAPES])
def test_group_backward_against_member_calls_and_fp32(M, K, Ns, ranks):
    mem = _members(K, Ns, ranks, seed=3 * M + K)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    gys = [torch.randn(M, N, generator=g).to(BF).to(DEV) for N in Ns]
    members = [m[0] for m in mem]
    h_cat, _ = ops.lora_group_fwd(x, members)
    gx, grads, gh_cat = ops.lora_group_bwd(x, h_cat, members, gys)

    ref_gx = torch.zeros(M, K, dtype=torch.float32, device=DEV)
    sum_members = None
    off = 0
    for (m, t, *_), gy, (ga, gb) in zip(mem, gys, grads):
        r = m.lora_a.shape[0]
        h = h_cat[:, off:off + r].contiguous()
        gh1, ga1, gb1 = ops.lora_bwd(gy, x, h, m.lora_b, m.scale)
        assert torch.equal(gh_cat[:, off:off + r], gh1), "hidden gradient"
        for got, want in ((ga, ga1), (gb, gb1)):
            torch.testing.assert_close(got.float(), want.float(), rtol=1e-2, atol=1e-2 * float(want.float().abs().max()) + 1e-30)
        # the adapter gradients against fp32 matmuls as well
        want_a = gh1.float().T @ x.float()
        want_b = m.scale * (gy.float().T @ h.float())
        torch.testing.assert_close(ga.float(), want_a, rtol=2e-2, atol=2e-2 * float(want_a.abs().max()) + 1e-30)
        torch.testing.assert_close(gb.float(), want_b, rtol=2e-2, atol=2e-2 * float(want_b.abs().max()) + 1e-30)
        gx1 = ops.nf4_linear_bwd_dx(gy, m.qdata, m.block_scalers, K, gh1, m.lora_a, transposed=m.transposed)
        sum_members = gx1 if sum_members is None else sum_members + gx1
        ref_gx += gy.float() @ t.get_original_weight().float() + gh1.float() @ m.lora_a.float()
        off += r
    scale = max(1.0, float(ref_gx.abs().max()) / 8)
    torch.testing.assert_close(gx.float(), ref_gx, rtol=1e-2, atol=1e-2 * scale)
    torch.testing.assert_close(gx.float(), sum_members.float(), rtol=2e-2, atol=2e-2 * scale)
    # one rounding instead of one per member and per addition: no further from the fp32 evaluation
    err_group = float((gx.float() - ref_gx).abs().mean())
    err_members = float((sum_members.float() - ref_gx).abs().mean())
    assert err_group <= err_members * 1.001 + 1e-12
    # deterministic
    gx2, grads2, _ = ops.lora_group_bwd(x, h_cat, members, gys)
    assert torch.equal(gx, gx2) and all(torch.equal(a, c) and torch.equal(b, d) for (a, b), (c, d) in zip(grads, grads2))


WIDE_SHAPES = [
    # M, K, Ns, ranks: every member at least 8192 wide, of rank <= 16, 1024 rows or more: gh and gB come from one pass over gy
    (1024, 256, (8192,), (16,)),
    (1030, 512, (8192 + 64, 8192), (8, 16)),           # a last column group of 64 columns, a last row step of 6 rows, two ranks
    (2048 + 40, 256, (16384, 8192, 8192), (16, 8, 8)),
    (8192, 4096, (14336, 14336), (16, 16)),            # the 8B gate / up pair at its real size (batch 4 x 2048)
]


@pytest.mark.parametrize("M,K,Ns,ranks", WIDE_SHAPES, ids=[f"M{s[0]}_K{s[1]}_{'x'.join(map(str, s[2]))}_r{'x'.join(map(str, s[3]))}" for s in WIDE_SHAPES])
def test_rank_r_backward_of_wide_members_against_fp32(M, K, Ns, ranks):
    """The adapter gradients of wide members, where ``gh`` and ``grad B`` are two products of one pass over ``gy``: every
    output against fp32 matmuls of the same bf16 operands (``gh`` and ``grad B`` are bf16 roundings of fp32 sums: rtol 1e-2,
    atol 1e-2 of the largest entry), the group's ``gh`` against the member-by-member calls bit for bit (its sums are
    taken per column group, whatever the row ranges), and two runs against each other bit for bit."""
    mem = _members(K, Ns, ranks, seed=M + K + len(Ns))
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    gys = [torch.randn(M, N, generator=g).to(BF).to(DEV) for N in Ns]
    h_cat = (torch.randn(M, sum(ranks), generator=g) * 0.5).to(BF).to(DEV)
    members = [m[0] for m in mem]
    _, grads, gh_cat = ops.lora_group_bwd(x, h_cat, members, gys, want_gx=False)
    _, grads2, gh_cat2 = ops.lora_group_bwd(x, h_cat, members, gys, want_gx=False)
    assert torch.equal(gh_cat, gh_cat2) and all(torch.equal(a, c) and torch.equal(b, d) for (a, b), (c, d) in zip(grads, grads2))
    off = 0
    for (m, *_), gy, (ga, gb) in zip(mem, gys, grads):
        r = m.lora_a.shape[0]
        h = h_cat[:, off:off + r].contiguous()
        gh = gh_cat[:, off:off + r]
        want_h = m.scale * (gy.float() @ m.lora_b.float())
        want_a = gh.float().T @ x.float()
        want_b = m.scale * (gy.float().T @ h.float())
        for got, want in ((gh, want_h), (ga, want_a), (gb, want_b)):
            torch.testing.assert_close(got.float(), want, rtol=1e-2, atol=1e-2 * float(want.abs().max()) + 1e-30)
        gh1, ga1, gb1 = ops.lora_bwd(gy, x, h, m.lora_b, m.scale)
        assert torch.equal(gh, gh1), "hidden gradient"
        for got, want in ((ga, ga1), (gb, gb1)):
            torch.testing.assert_close(got.float(), want.float(), rtol=1e-2, atol=1e-2 * float(want.float().abs().max()) + 1e-30)
        off += r


def _layers(K, Ns, ranks, alpha, bias, seed):
    layers = []
    g = torch.Generator().manual_seed(seed)
    prev = torch.get_default_dtype()
    torch.set_default_dtype(BF)
    try:
        with torch.device(DEV):
            for N, r in zip(Ns, ranks):
                layers.append(LoRALinear(K, N, rank=r, alpha=alpha, use_bias=bias, quantize_base=True))
    finally:
        torch.set_default_dtype(prev)
    params = []
    with torch.no_grad():
        for layer, N, r in zip(layers, Ns, ranks):
            W = (torch.randn(N, K, generator=g) * 0.02).to(BF)
            A = lora_oracle.lora_a_init_(torch.empty(r, K), g).to(BF)
            B = (torch.randn(N, r, generator=g) * 0.01).to(BF)
            b = (torch.randn(N, generator=g) * 0.1).to(BF) if bias else None
            layer.weight.copy_(W.to(DEV))
            layer.lora_a.weight.copy_(A.to(DEV))
            layer.lora_b.weight.copy_(B.to(DEV))
            if bias:
                layer.bias.copy_(b.to(DEV))
            params.append((W, A, B, b))
    return layers, params


@pytest.mark.parametrize("M,K,Ns,ranks,bias", [
    (8, 512, (256, 64, 64), (8, 8, 8), False),
    (300, 512, (256, 128, 128), (16, 16, 16), True),
    (520, 1024, (512, 512), (16, 16), False),
], ids=["decode_qkv", "qkv_bias", "gate_up"])
def test_module_group_against_oracle_and_layerwise(M, K, Ns, ranks, bias):
    alpha = 32.0
    layers, params = _layers(K, Ns, ranks, alpha, bias, seed=M)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g).to(BF)
    gys = [torch.randn(M, N, generator=g).to(BF) for N in Ns]
    xg = x.to(DEV).requires_grad_()
    assert group_applies(xg, layers)
    ys = lora_linear_group(xg, layers)
    torch.autograd.backward(ys, [gy.to(DEV) for gy in gys])
    got = {"gx": xg.grad.clone(), "ga": [l.lora_a.weight.grad.clone() for l in layers],
           "gb": [l.lora_b.weight.grad.clone() for l in layers],
           "gbias": [l.bias.grad.clone() if bias else None for l in layers]}

    # ---- layer by layer through the per-linear path
    for l in layers:
        l.zero_grad()
    xl = x.to(DEV).requires_grad_()
    yl = [l(xl) for l in layers]
    torch.autograd.backward(yl, [gy.to(DEV) for gy in gys])
    for a, b in zip(ys, yl):
        assert torch.equal(a, b)
    scale = max(1.0, float(xl.grad.float().abs().max()) / 8)
    torch.testing.assert_close(got["gx"].float(), xl.grad.float(), rtol=2e-2, atol=2e-2 * scale)
    for i, l in enumerate(layers):
        for mine, theirs in ((got["ga"][i], l.lora_a.weight.grad), (got["gb"][i], l.lora_b.weight.grad)):
            torch.testing.assert_close(mine.float(), theirs.float(), rtol=1e-2, atol=1e-2 * float(theirs.float().abs().max()) + 1e-30)
        if bias:
            assert torch.equal(got["gbias"][i], l.bias.grad)

    # ---- the CPU oracle: the reference's unfused bf16 graph of the same layers on the same input
    xo = x.clone().requires_grad_()
    outs, leaves = [], []
    for (W, A, B, b), r in zip(params, ranks):
        n_blocks = W.numel() // 64
        p = nf4_oracle.nf4_quantize(W, 64, 256 if n_blocks % 256 == 0 else n_blocks)
        Ao, Bo = A.clone().requires_grad_(), B.clone().requires_grad_()
        outs.append(lora_oracle.lora_linear_forward(xo, p, Ao, Bo, alpha, r, bias=b))
        leaves.append((Ao, Bo))
    torch.autograd.backward(outs, gys)
    for y, yo in zip(ys, outs):
        torch.testing.assert_close(y.detach().cpu().float(), yo.detach().float(), rtol=1e-2, atol=1e-2)
    sc = max(1.0, float(xo.grad.float().abs().max()) / 8)
    torch.testing.assert_close(got["gx"].cpu().float(), xo.grad.float(), rtol=1e-2, atol=2e-2 * sc)
    for i, (Ao, Bo) in enumerate(leaves):
        for mine, theirs in ((got["ga"][i], Ao.grad), (got["gb"][i], Bo.grad)):
            torch.testing.assert_close(mine.cpu().float(), theirs.float(), rtol=2e-2, atol=2e-2 * float(theirs.float().abs().max()) + 1e-30)


GATED_SHAPES = [
    # M, K, width, ranks, bias        (256 tiles of 256 x 256 and 2048 rows: the product is written by the GEMM launch)
    (2048, 256, 4096, (16, 16), False),
    (2048 + 192, 512, 4096, (16, 8), True),     # a last row tile with 192 rows
    (4096, 1024, 2048, (32, 0 + 16), False),
    (8192, 256, 1024, (16, 16), True),
    (8192, 4096, 14336, (16, 16), False),       # the 8B feed-forward at its real size (batch 4 x 2048)
    (4096, 8192, 28672, (16, 16), False),       # the 70B feed-forward (batch 1 x 4096)
    (16, 512, 1024, (8, 8), False),             # few tokens: group launch + a pass of its own
    (300, 512, 512, (16, 16), True),            # tiled kernels + a pass of its own
    (2048, 256, 1152, (16, 16), False),         # many tokens, too few tiles for the expanded path
    (2048, 256, 4096, (40, 24), False),         # a rank beyond 32: the members' adapter operands in entries of their own
    (2048, 64, 4096, (16, 8), True),            # the shortest contraction: the adapter's operands are requested up front
    (2048, 128, 4096, (8, 32), False),          # two trips of the loop, both past the weight
]


@pytest.mark.parametrize("M,K,width,ranks,bias", GATED_SHAPES, ids=[f"M{s[0]}_K{s[1]}_W{s[2]}" for s in GATED_SHAPES])
def test_gated_pair_equals_group_forward_plus_swiglu_bitwise(M, K, width, ranks, bias):
    """``ttamd_nf4_lora_group_swiglu_fwd_bf16``: both projections equal the plain group call's bit for bit (the same GEMM
    on the same operands, whatever the order of the weight's columns in the scratch copy) and the gated product equals
    ``ttamd_swiglu_fwd_bf16`` of them bit for bit; that kernel is itself compared with the reference's
    ``F.silu(g) * u`` in bf16 in tests/test_gpu_layer_ops.py."""
    mem = _members(K, (width, width), ranks, seed=M + K + width, bias=bias)
    members = [m[0] for m in mem]
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(11)).to(BF).to(DEV)
    h0, (g0, u0) = ops.lora_group_fwd(x, members)
    h1, (g1, u1, act) = ops.lora_group_fwd(x, members, swiglu=True)
    assert torch.equal(h0, h1)
    assert torch.equal(g0.view(torch.int16), g1.view(torch.int16)) and torch.equal(u0.view(torch.int16), u1.view(torch.int16))
    assert torch.equal(act.view(torch.int16), ops.swiglu_fwd(g0, u0).view(torch.int16))
    # and the definition, evaluated by torch on the same bf16 projections
    want = torch.nn.functional.silu(g0) * u0
    torch.testing.assert_close(act.float(), want.float(), rtol=2e-2, atol=1e-3)


def test_gated_pair_rejects_unequal_widths():
    mem = _members(512, (256, 128), (8, 8), seed=3)
    x = torch.randn(8, 512, device=DEV, dtype=BF)
    with pytest.raises(ValueError):
        ops.lora_group_fwd(x, [m[0] for m in mem], swiglu=True)
    with pytest.raises(ValueError):
        ops.lora_group_fwd(x, [mem[0][0]], swiglu=True)


@pytest.mark.parametrize("M,K,width", [(2048, 256, 4096), (64, 512, 512)], ids=["epilogue", "own_pass"])
def test_gated_module_function_matches_group_then_swiglu(M, K, width):
    """``lora_swiglu_group`` against ``lora_linear_group`` followed by the stand-alone SwiGLU op: output and every
    gradient bit for bit (same kernels on the same values in backward)."""
    layers, _ = _layers(K, (width, width), (16, 16), 32.0, False, seed=M + width)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    gact = torch.randn(M, width, generator=g).to(BF).to(DEV)

    def run(gated):
        for l in layers:
            l.zero_grad()
        xg = x.clone().requires_grad_()
        if gated:
            act = lora_swiglu_group(xg, layers[0], layers[1])
            assert act is not None
        else:
            gg, uu = lora_linear_group(xg, layers)
            act = layer_ops.swiglu(gg, uu)
        act.backward(gact)
        return [act.detach(), xg.grad] + [p.grad.clone() for l in layers for p in (l.lora_a.weight, l.lora_b.weight)]

    for a, b in zip(run(True), run(False)):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    layers[1].disabled = True
    assert lora_swiglu_group(x, layers[0], layers[1]) is None   # the caller falls back to its own multiply


DX_SWIGLU_SHAPES = [
    # M, N (rows of the weight), K (its columns = width of gate and up), rank, transposed copies
    (4096, 256, 4096, 16, False),            # 256 tiles of 256 x 256: the two gradients leave the GEMM's epilogue
    (4096, 256, 4096, 16, True),
    (2048 + 192, 512, 8192, 8, False),       # a last row tile with 192 rows
    (2048, 320, 4352, 0, False),             # no adapter; 136 tiles (a partly filled round)
    (8192, 4096, 14336, 16, False),          # the 8B down projection at its real size (batch 4 x 2048)
    (4096, 8192, 28672, 16, False),          # the 70B one (batch 1 x 4096)
    (16, 512, 1024, 8, True),                # few tokens: the grad-input as usual, then the stand-alone kernel in place
    (300, 512, 512, 16, False),
    (2048, 256, 1152, 16, True),             # many tokens, too few tiles for the expanded path
]


@pytest.mark.parametrize("M,N,K,rank,copies", DX_SWIGLU_SHAPES, ids=[f"M{s[0]}_N{s[1]}_K{s[2]}_r{s[3]}{'_t' if s[4] else ''}" for s in DX_SWIGLU_SHAPES])
def test_grad_input_carried_through_swiglu_equals_the_two_steps_bitwise(M, N, K, rank, copies):
    """``ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16`` against ``ttamd_nf4_linear_bwd_dx_ws_bf16`` followed by
    ``ttamd_swiglu_bwd_bf16``: both gradients bit for bit (the same GEMM, the same arithmetic on its rounded result).
    Those two are themselves compared with fp32 matmuls of the dequantised weight (tests/test_gpu_lora_linear.py) and
    with autograd's backward of ``F.silu(g) * u`` in bf16 (tests/test_gpu_layer_ops.py)."""
    g = torch.Generator().manual_seed(M + N + K)
    W = (torch.randn(N, K, generator=g) * 0.02).to(BF)
    t = to_nf4(W.to(DEV))
    gy = torch.randn(M, N, generator=g).to(BF).to(DEV)
    gate = torch.randn(M, K, generator=g).to(BF).to(DEV)
    up = torch.randn(M, K, generator=g).to(BF).to(DEV)
    gh = A = None
    if rank:
        gh = (torch.randn(M, rank, generator=g) * 0.1).to(BF).to(DEV)
        A = lora_oracle.lora_a_init_(torch.empty(rank, K), g).to(BF).to(DEV)
    tr = t.backward_copy() if copies else None
    gx = ops.nf4_linear_bwd_dx(gy, t.quantized_data, t.block_scalers(), K, gh, A, transposed=tr)
    gg0, gu0 = ops.swiglu_bwd(gx, gate, up)
    gg1, gu1 = ops.nf4_linear_bwd_dx(gy, t.quantized_data, t.block_scalers(), K, gh, A, transposed=tr, swiglu=(gate, up))
    assert torch.equal(gg0.view(torch.int16), gg1.view(torch.int16))
    assert torch.equal(gu0.view(torch.int16), gu1.view(torch.int16))


def test_grad_input_carried_through_swiglu_rejects_mismatched_gate():
    t = to_nf4((torch.randn(128, 256) * 0.02).to(BF).to(DEV))
    gy = torch.randn(8, 128, device=DEV, dtype=BF)
    good = torch.randn(8, 256, device=DEV, dtype=BF)
    with pytest.raises(ValueError):
        ops.nf4_linear_bwd_dx(gy, t.quantized_data, t.block_scalers(), 256, swiglu=(good, good[:, :128]))
    with pytest.raises(ValueError):
        ops.nf4_linear_bwd_dx(gy, t.quantized_data, t.block_scalers(), 256, swiglu=(good[:4], good[:4]))


@pytest.mark.parametrize("M,K,width", [(4096, 512, 4096), (64, 512, 512)], ids=["epilogue", "own_pass"])
def test_feed_forward_node_matches_gated_pair_then_down(M, K, width):
    """``lora_feed_forward`` against ``down(lora_swiglu_group(x, gate, up))``: output and every gradient bit for bit."""
    pair, _ = _layers(K, (width, width), (16, 16), 32.0, False, seed=M + width)
    (down,), _ = _layers(width, (K,), (16,), 32.0, False, seed=M + width + 1)
    layers = list(pair) + [down]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    gy = torch.randn(M, K, generator=g).to(BF).to(DEV)

    def run(node):
        for l in layers:
            l.zero_grad()
        xg = x.clone().requires_grad_()
        y = lora_feed_forward(xg, *layers) if node else down(lora_swiglu_group(xg, pair[0], pair[1]))
        assert y is not None
        y.backward(gy)
        return [y.detach(), xg.grad] + [p.grad.clone() for l in layers for p in (l.lora_a.weight, l.lora_b.weight)]

    for a, b in zip(run(True), run(False)):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    down.disabled = True
    assert lora_feed_forward(x, *layers) is None   # the caller composes the layers itself
    down.disabled = False
    (narrow,), _ = _layers(width // 2, (K,), (16,), 32.0, False, seed=5)
    assert lora_feed_forward(x, pair[0], pair[1], narrow) is None


def test_group_falls_back_when_it_does_not_apply():
    layers, _ = _layers(512, (256, 128), (16, 16), 32.0, False, seed=1)
    x = torch.randn(4, 512, device=DEV, dtype=BF)
    layers[1].disabled = True
    assert not group_applies(x, layers)
    ys = lora_linear_group(x, layers)
    assert torch.equal(ys[0], layers[0](x)) and torch.equal(ys[1], layers[1](x))
    layers[1].disabled = False
    assert group_applies(x, layers)
    assert not group_applies(x.float(), layers)
    five, _ = _layers(512, (64,) * 5, (8,) * 5, 16.0, False, seed=2)
    assert not group_applies(x, five)
    big_ranks, _ = _layers(512, (64, 64), (64, 8), 16.0, False, seed=3)
    assert not group_applies(x, big_ranks)  # ranks sum to more than 64
    assert len(lora_linear_group(x, big_ranks)) == 2


def test_group_rejects_mismatched_operands():
    mem = _members(512, (128, 64), (8, 8), seed=9)
    members = [m[0] for m in mem]
    x = torch.randn(8, 512, device=DEV, dtype=BF)
    with pytest.raises(ValueError):
        ops.lora_group_fwd(torch.randn(8, 256, device=DEV, dtype=BF), members)
    bad = ops.GroupMember(members[0].qdata, members[0].block_scalers, members[0].transposed, members[0].lora_a,
                          members[1].lora_b, None, 1.0, members[0].N)
    with pytest.raises(ValueError):
        ops.lora_group_fwd(x, [bad])
    h_cat, _ = ops.lora_group_fwd(x, members)
    with pytest.raises(ValueError):
        ops.lora_group_bwd(x, h_cat[:, :8].contiguous(), members, [torch.zeros(8, 128, device=DEV, dtype=BF),
                                                                    torch.zeros(8, 64, device=DEV, dtype=BF)])
    with pytest.raises(ValueError):
        ops.lora_group_fwd(x, members * 3)  # six members


@pytest.mark.parametrize("M,K,N,ranks", [
    (8192, 4096, 14336, (16, 16)),   # the 8B gate / up pair: the pass that forms the gradients also multiplies them
    (1100, 512, 8192, (16, 8)),      # ragged rows, different ranks, still wide
    (2048, 512, 8256, (8, 8)),       # a width that is no multiple of the 256-column groups
    (300, 512, 1024, (16, 16)),      # narrow: the two steps one after the other inside the call
])
def test_swiglu_backward_inside_the_adapter_backward_equals_the_two_steps_bitwise(M, K, N, ranks):
    """``ops.lora_group_bwd(..., swiglu=(gact, gate, up))`` (``ttamd_lora_group_swiglu_bwd_bf16``) against
    ``ops.swiglu_bwd`` followed by ``ops.lora_group_bwd`` on its results: gh, grad A and (through the grouped grad-input,
    which reads the gradients the call left in memory) gx bit for bit; grad B up to the order of its fp32 sums over the
    row ranges (the pair kernel cuts the rows into twice as many ranges: rtol 2^-7, atol 2^-7 of the largest entry)."""
    mem = _members(K, (N, N), ranks, seed=M + N)
    members = [m[0] for m in mem]
    g = torch.Generator().manual_seed(9)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    h_cat = (torch.randn(M, sum(ranks), generator=g) * 0.5).to(BF).to(DEV)
    gact = torch.randn(M, N, generator=g).to(BF).to(DEV)
    gate = (torch.randn(M, N, generator=g) * 2).to(BF).to(DEV)
    up = torch.randn(M, N, generator=g).to(BF).to(DEV)
    ggate, gup = ops.swiglu_bwd(gact, gate, up)
    gx0, grads0, gh0 = ops.lora_group_bwd(x, h_cat, members, [ggate, gup], want_gx=True)
    gx1, grads1, gh1 = ops.lora_group_bwd(x, h_cat, members, None, want_gx=True, swiglu=(gact, gate, up))
    assert torch.equal(gh0.view(torch.int16), gh1.view(torch.int16))
    assert torch.equal(gx0.view(torch.int16), gx1.view(torch.int16))
    for (a0, b0), (a1, b1) in zip(grads0, grads1):
        assert torch.equal(a0.view(torch.int16), a1.view(torch.int16))
        torch.testing.assert_close(b1.float(), b0.float(), rtol=2.0 ** -7, atol=2.0 ** -7 * float(b0.float().abs().max()))
    assert float(gh1.float().abs().max()) > 0 and float(gx1.float().abs().max()) > 0
