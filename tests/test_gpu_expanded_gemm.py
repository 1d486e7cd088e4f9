"""GPU parity of the many-token path of the NF4 + LoRA linear: the weight expanded once per call into scratch memory,
then the plain bf16 GEMM (``nf4_gemm_dense.hip``), forward and grad-input, single layers and groups.

Three kinds of checks:
* bit-exact: with one-hot activations every output is a single product 1 * Wd[n][k], so the GEMM's output IS the expanded
  weight; it must equal ``ops.nf4_dequantize`` (itself bit-exact against the oracle in tests/test_gpu_nf4.py) bit for
  bit, for the three layouts the expansion kernel reads (natural scalers, transposed scalers, transposed copy);
* against the CPU oracle (the reference's unfused bf16 graph), rtol 1e-2 / atol 1e-2 as for the fused kernel;
* against the fused kernel on the same inputs (both accumulate in fp32 and round once, in a different order of
  summation): rtol 1e-2 / atol 2e-3 at unit-variance activations.
"""
import pytest
import torch

from oracle import lora_oracle, nf4_oracle
from torchtune_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def _quantized(N, K, seed):
    g = torch.Generator().manual_seed(seed)
    W = (torch.randn(N, K, generator=g) * 0.02).to(BF)
    n_blocks = N * K // 64
    sbs = 256 if n_blocks % 256 == 0 else n_blocks
    qdata, qscal, qfac, mean = ops.nf4_quantize(W.to(DEV), 64, sbs)[:4]
    bscal = ops.nf4_block_scalers(qscal, qfac, mean, sbs)
    dense = ops.nf4_dequantize(qdata, qscal, qfac, mean, (N, K), 64, sbs)
    return W, sbs, qdata, bscal, dense


def _expands(M, n_out, k):
    return bool(_lib.load().ttamd_nf4_gemm_expands_weight(M, n_out, k))


def _one_hot(M, K):
    x = torch.zeros(M, K, dtype=BF, device=DEV)
    x[torch.arange(M, device=DEV), torch.arange(M, device=DEV) % K] = 1.0
    return x


@pytest.mark.parametrize("N,K,with_transposed_scalers", [(8192, 256, False), (8192, 256, True), (8256, 192, True)])
def test_forward_output_is_the_expanded_weight_bit_for_bit(N, K, with_transposed_scalers):
    M = 2048
    assert _expands(M, N, K)
    _, _, qdata, bscal, dense = _quantized(N, K, seed=N + K)
    scal_t = ops.nf4_transpose_for_backward(qdata, bscal, N, K)[1] if with_transposed_scalers else None
    y = ops.nf4_lora_linear_fwd(_one_hot(M, K), qdata, bscal, N, block_scalers_t=scal_t)
    want = dense.t().repeat((M + K - 1) // K, 1)[:M]  # row m = column m % K of the weight
    assert torch.equal(y.view(torch.int16), want.contiguous().view(torch.int16))


def test_grad_input_output_is_the_expanded_weight_bit_for_bit():
    M, N, K = 2048, 256, 8192
    assert _expands(M, K, N)
    _, _, qdata, bscal, dense = _quantized(N, K, seed=7)
    tr = ops.nf4_transpose_for_backward(qdata, bscal, N, K)
    gx = ops.nf4_linear_bwd_dx(_one_hot(M, N), qdata, bscal, K, transposed=tr)
    want = dense.repeat((M + N - 1) // N, 1)[:M]  # row m = row m % N of the weight
    assert torch.equal(gx.view(torch.int16), want.contiguous().view(torch.int16))


CASES = [
    # M, N, K, rank, bias: at least 256 tiles of 256 x 256 and 2048 tokens, so the library expands the weight
    (2048, 8192, 256, 16, False),
    (2048 + 37, 8192, 192, 8, True),      # ragged token count (a ninth, partial m-tile)
    (4096, 4096 + 64, 320, 24, True),     # output width not a multiple of the tile, rank not a multiple of 16
    (4096, 4096, 512, 64, False),         # two 32-wide steps of the adapter contraction
    (2048, 8192, 128, 0, True),           # no adapter (FrozenNF4Linear / linear_nf4)
]


def _case(M, N, K, r, bias, seed):
    g = torch.Generator().manual_seed(seed)
    W, sbs, qdata, bscal, dense = _quantized(N, K, seed)
    A = lora_oracle.lora_a_init_(torch.empty(max(r, 1), K), g).to(BF)[:r] if r else None
    B = (torch.randn(N, r, generator=g) * 0.01).to(BF) if r else None
    b = (torch.randn(N, generator=g) * 0.1).to(BF) if bias else None
    x = torch.randn(M, K, generator=g).to(BF)
    gy = torch.randn(M, N, generator=g).to(BF)
    return W, sbs, qdata, bscal, dense, A, B, b, x, gy


def _run(M, N, K, r, scale, qdata, bscal, A, B, b, x, gy, tr):
    xd, gyd = x.to(DEV), gy.to(DEV)
    h = ops.lora_hidden(xd, A.to(DEV)) if r else None
    y = ops.nf4_lora_linear_fwd(xd, qdata, bscal, N, h, B.to(DEV) if r else None, scale, b.to(DEV) if b is not None else None,
                                block_scalers_t=tr[1])
    gh = ops.lora_bwd(gyd, xd, h, B.to(DEV), scale)[0] if r else None
    gx = ops.nf4_linear_bwd_dx(gyd, qdata, bscal, K, gh, A.to(DEV) if r else None, transposed=tr)
    return y, gx


@pytest.mark.parametrize("M,N,K,r,bias", CASES)
def test_expanded_path_vs_oracle_and_vs_fused_kernel(M, N, K, r, bias, monkeypatch):
    assert _expands(M, N, K)
    alpha = 2.0 * max(r, 1)
    scale = alpha / max(r, 1)
    W, sbs, qdata, bscal, dense, A, B, b, x, gy = _case(M, N, K, r, bias, seed=M + N + K + r)
    tr = ops.nf4_transpose_for_backward(qdata, bscal, N, K)
    y, gx = _run(M, N, K, r, scale, qdata, bscal, A, B, b, x, gy, tr)
    monkeypatch.setattr(ops, "EXPANDED_WEIGHT_PATH", False)
    y_f, gx_f = _run(M, N, K, r, scale, qdata, bscal, A, B, b, x, gy, tr)
    torch.testing.assert_close(y.float(), y_f.float(), rtol=1e-2, atol=2e-3)
    if _expands(M, K, N):
        torch.testing.assert_close(gx.float(), gx_f.float(), rtol=1e-2, atol=2e-3)
    # the oracle: the reference's unfused bf16 graph on the CPU
    p = nf4_oracle.nf4_quantize(W, 64, sbs)
    xo = x.clone().requires_grad_()
    if r:
        yo = lora_oracle.lora_linear_forward(xo, p, A, B, alpha, r, bias=b)
    else:
        yo = lora_oracle.lora_linear_forward(xo, p, None, None, 0.0, 1, bias=b, disabled=True)
    yo.backward(gy)
    torch.testing.assert_close(y.cpu().float(), yo.detach().float(), rtol=1e-2, atol=1e-2)
    torch.testing.assert_close(gx.cpu().float(), xo.grad.float(), rtol=1e-2, atol=1e-2)


def test_grad_input_expanded_at_a_wide_layer_vs_fp32_matmul():
    """Grad-input with the contraction over a long output dimension (the shape class of gate / up projections)."""
    M, N, K = 2048, 1024, 8192
    assert _expands(M, K, N)
    _, _, qdata, bscal, dense = _quantized(N, K, seed=3)
    g = torch.Generator().manual_seed(5)
    gy = torch.randn(M, N, generator=g).to(BF).to(DEV)
    A = (torch.randn(16, K, generator=g) * 0.02).to(BF).to(DEV)
    gh = torch.randn(M, 16, generator=g).to(BF).to(DEV)
    tr = ops.nf4_transpose_for_backward(qdata, bscal, N, K)
    gx = ops.nf4_linear_bwd_dx(gy, qdata, bscal, K, gh, A, transposed=tr)
    want = gy.float() @ dense.float() + gh.float() @ A.float()
    torch.testing.assert_close(gx.float(), want, rtol=1e-2, atol=1e-2)


def test_column_scale_in_the_epilogue():
    """DoRA's per-column factor is applied after the bias, as in the fused kernel: y = (x W^T + s h B^T + bias) * c."""
    M, N, K, r = 2048, 8192, 128, 16
    W, sbs, qdata, bscal, dense, A, B, b, x, gy = _case(M, N, K, r, True, seed=11)
    g = torch.Generator().manual_seed(13)
    c = (1.0 + 0.1 * torch.randn(N, generator=g)).to(BF)
    xd = x.to(DEV)
    h = ops.lora_hidden(xd, A.to(DEV))
    y = ops.nf4_lora_linear_fwd(xd, qdata, bscal, N, h, B.to(DEV), 2.0, b.to(DEV), col_scale=c.to(DEV))
    want = (xd.float() @ dense.float().T + 2.0 * h.float() @ B.to(DEV).float().T + b.to(DEV).float()) * c.to(DEV).float()
    torch.testing.assert_close(y.float(), want, rtol=1e-2, atol=1e-2)


def test_group_grad_input_over_concatenated_members(monkeypatch):
    """gx of q / k / v-like members with a common input: one expanded GEMM over the members' concatenated output
    columns against the fused kernel's grouped launch and against fp32 matmuls of the dequantised weights."""
    M, K = 2048, 8192
    Ns, ranks = (512, 128, 192), (16, 8, 16)
    g = torch.Generator().manual_seed(17)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    members, gys, denses = [], [], []
    for i, (N, r) in enumerate(zip(Ns, ranks)):
        _, _, qdata, bscal, dense = _quantized(N, K, seed=20 + i)
        A = (torch.randn(r, K, generator=g) * 0.02).to(BF).to(DEV)
        B = (torch.randn(N, r, generator=g) * 0.01).to(BF).to(DEV)
        tr = ops.nf4_transpose_for_backward(qdata, bscal, N, K)
        members.append(ops.GroupMember(qdata=qdata, block_scalers=bscal, N=N, lora_a=A, lora_b=B, scale=2.0, bias=None, transposed=tr))
        gys.append(torch.randn(M, N, generator=g).to(BF).to(DEV))
        denses.append(dense)
    assert _lib.load().ttamd_nf4_group_bwd_dx_workspace_bytes(ops._group_array("t", members, K, gys, M)[0], len(members), M, K) == 2 * K * sum(Ns)
    h_cat, _ = ops.lora_group_fwd(x, members)
    gx, _, gh_cat = ops.lora_group_bwd(x, h_cat, members, gys)
    monkeypatch.setattr(ops, "EXPANDED_WEIGHT_PATH", False)
    gx_f, _, _ = ops.lora_group_bwd(x, h_cat, members, gys)
    torch.testing.assert_close(gx.float(), gx_f.float(), rtol=1e-2, atol=2e-3)
    want = torch.zeros(M, K, dtype=torch.float32, device=DEV)
    off = 0
    for m, gy, dense, r in zip(members, gys, denses, ranks):
        want += gy.float() @ dense.float() + gh_cat[:, off:off + r].float() @ m.lora_a.float()
        off += r
    torch.testing.assert_close(gx.float(), want, rtol=1e-2, atol=1e-2)


def test_smaller_workspace_keeps_the_fused_kernel():
    """The ABI rule: less workspace than ``ttamd_nf4_gemm_workspace_bytes`` says (or none) is not an error."""
    M, N, K = 2048, 8192, 128
    _, _, qdata, bscal, dense = _quantized(N, K, seed=23)
    x = torch.randn(M, K, generator=torch.Generator().manual_seed(1)).to(BF).to(DEV)
    lib = _lib.load()
    need = lib.ttamd_nf4_gemm_workspace_bytes(M, N, K)
    assert need == 2 * N * K
    y = [torch.empty(M, N, dtype=BF, device=DEV) for _ in range(3)]
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    for out, (p, nbytes) in zip(y, [(ws.data_ptr(), need), (ws.data_ptr(), need - 1), (None, 0)]):
        rc = lib.ttamd_nf4_lora_linear_fwd_ws_bf16(x.data_ptr(), qdata.data_ptr(), bscal.data_ptr(), None, None, None, 0, 0.0, None, None,
                                                   out.data_ptr(), M, N, K, p, nbytes, s)
        _lib.check(rc, "fwd_ws")
    assert torch.equal(y[1], y[2])  # both ran the fused kernel
    torch.testing.assert_close(y[0].float(), y[1].float(), rtol=1e-2, atol=2e-3)
    torch.testing.assert_close(y[0].float(), x.float() @ dense.float().T, rtol=1e-2, atol=1e-2)


def test_group_forward_over_concatenated_outputs(monkeypatch):
    """Forward of members with a common input (widths multiples of 256, one of them with a bias): one expanded GEMM over
    the concatenated output columns against the member-by-member fused kernel and against fp32 matmuls."""
    M, K = 2048, 192
    Ns, ranks = (4096, 2048, 2048 + 256), (16, 8, 24)
    g = torch.Generator().manual_seed(29)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    members, denses = [], []
    for i, (N, r) in enumerate(zip(Ns, ranks)):
        _, _, qdata, bscal, dense = _quantized(N, K, seed=40 + i)
        A = (torch.randn(r, K, generator=g) * 0.05).to(BF).to(DEV)
        B = (torch.randn(N, r, generator=g) * 0.05).to(BF).to(DEV)
        bias = (torch.randn(N, generator=g) * 0.1).to(BF).to(DEV) if i == 1 else None
        tr = ops.nf4_transpose_for_backward(qdata, bscal, N, K) if i != 2 else None  # member 2: natural scaler layout
        members.append(ops.GroupMember(qdata=qdata, block_scalers=bscal, N=N, lora_a=A, lora_b=B, scale=0.5 * (i + 1), bias=bias, transposed=tr))
        denses.append(dense)
    ys0 = [torch.empty(M, N, dtype=BF, device=DEV) for N in Ns]
    arr = ops._group_array("t", members, K, ys0, M)[0]
    assert _lib.load().ttamd_lora_group_fwd_workspace_bytes(arr, len(members), M, K) == 2 * K * sum(Ns)
    h_cat, ys = ops.lora_group_fwd(x, members)
    monkeypatch.setattr(ops, "EXPANDED_WEIGHT_PATH", False)
    h_cat_f, ys_f = ops.lora_group_fwd(x, members)
    assert torch.equal(h_cat, h_cat_f)
    off = 0
    for m, y, y_f, dense, r in zip(members, ys, ys_f, denses, ranks):
        torch.testing.assert_close(y.float(), y_f.float(), rtol=1e-2, atol=2e-3)
        want = x.float() @ dense.float().T + m.scale * h_cat[:, off:off + r].float() @ m.lora_b.float().T
        if m.bias is not None:
            want = want + m.bias.float()
        torch.testing.assert_close(y.float(), want, rtol=1e-2, atol=1e-2)
        off += r


@pytest.mark.parametrize("N,K", [(256, 8192), (320, 8192 + 64)])
def test_grad_input_without_transposed_copy_is_the_expanded_weight_bit_for_bit(N, K):
    """No transposed copy: W^T is expanded from the weight's own codes (a block turned through LDS)."""
    M = 2048
    assert _expands(M, K, N)
    _, _, qdata, bscal, dense = _quantized(N, K, seed=N + 3)
    gx = ops.nf4_linear_bwd_dx(_one_hot(M, N), qdata, bscal, K, transposed=None)
    want = dense.repeat((M + N - 1) // N, 1)[:M]
    assert torch.equal(gx.view(torch.int16), want.contiguous().view(torch.int16))


def test_group_without_transposed_copies_equals_group_with_them():
    """A group whose members keep no transposed copy: forward from natural scalers, grad-input expanded from the weights'
    own codes; both bit-equal to the same group with the copies (the GEMM sees the same expanded values)."""
    M, K = 2048, 8192
    Ns, ranks = (512, 256), (16, 8)
    g = torch.Generator().manual_seed(31)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    with_tr, without = [], []
    gys = []
    for i, (N, r) in enumerate(zip(Ns, ranks)):
        _, _, qdata, bscal, _ = _quantized(N, K, seed=50 + i)
        A = (torch.randn(r, K, generator=g) * 0.02).to(BF).to(DEV)
        B = (torch.randn(N, r, generator=g) * 0.01).to(BF).to(DEV)
        tr = ops.nf4_transpose_for_backward(qdata, bscal, N, K)
        with_tr.append(ops.GroupMember(qdata, bscal, tr, A, B, None, 2.0, N))
        without.append(ops.GroupMember(qdata, bscal, None, A, B, None, 2.0, N))
        gys.append(torch.randn(M, N, generator=g).to(BF).to(DEV))
    assert ops.group_dx_expands(M, K, Ns)
    h1, _ = ops.lora_group_fwd(x, with_tr)
    gx1, _, _ = ops.lora_group_bwd(x, h1, with_tr, gys)
    h2, _ = ops.lora_group_fwd(x, without)
    gx2, _, _ = ops.lora_group_bwd(x, h2, without, gys)
    assert torch.equal(h1, h2) and torch.equal(gx1, gx2)


SWEEP = [
    # M, N, K, rank: shortest contractions (one and two 64-wide entries), ragged rows, widths off the 256 grid
    (2048, 8192, 64, 8), (2048, 8192, 128, 16), (2049, 8192 + 192, 192, 8), (2304, 7424, 320, 32), (3000, 5568, 448, 16),
    (8192, 2048, 256, 8), (4096, 4096, 1024, 16), (2048, 16384, 64, 0),
    # ranks beyond 32 (two steps of adapter operands), also over the shortest contractions
    (2048, 8192, 64, 64), (2048, 8192, 128, 40), (2304, 7424, 320, 64),
]


@pytest.mark.parametrize("M,N,K,r", SWEEP)
def test_expanded_path_sweep_vs_fp32_matmul_of_the_dequantised_weight(M, N, K, r):
    """Forward and (where the transposed shape is served too) grad-input over a sweep of shapes, against fp32 matmuls of
    the dequantised weight — a parity statement because that dequantisation is bit-exact against the oracle
    (tests/test_gpu_nf4.py) and the expanded copy is bit-exact against it (first tests of this file)."""
    assert _expands(M, N, K)
    W, sbs, qdata, bscal, dense, A, B, b, x, gy = _case(M, N, K, r, True, seed=M + 7 * N + K + r)
    xd, gyd = x.to(DEV), gy.to(DEV)
    h = ops.lora_hidden(xd, A.to(DEV)) if r else None
    y = ops.nf4_lora_linear_fwd(xd, qdata, bscal, N, h, B.to(DEV) if r else None, 1.5, b.to(DEV))
    want = xd.float() @ dense.float().T + b.to(DEV).float()
    if r:
        want = want + 1.5 * h.float() @ B.to(DEV).float().T
    torch.testing.assert_close(y.float(), want, rtol=1e-2, atol=1e-2)
    if _expands(M, K, N):
        gh = ops.lora_bwd(gyd, xd, h, B.to(DEV), 1.5)[0] if r else None
        gx = ops.nf4_linear_bwd_dx(gyd, qdata, bscal, K, gh, A.to(DEV) if r else None, transposed=None)
        want = gyd.float() @ dense.float()
        if r:
            want = want + gh.float() @ A.to(DEV).float()
        torch.testing.assert_close(gx.float(), want, rtol=1e-2, atol=1e-2 * max(1.0, float(want.abs().max()) / 8))


def _lora_layers(dims, K, rank, seed):
    """LoRALinear layers over NF4 with a common input width, non-zero adapters, on the GPU."""
    from torchtune_amd.modules.peft import LoRALinear

    torch.manual_seed(seed)
    layers = []
    prev = torch.get_default_dtype()
    torch.set_default_dtype(BF)
    try:
        for N in dims:
            with torch.device(DEV):
                layer = LoRALinear(K, N, rank=rank, alpha=2.0 * rank, quantize_base=True)
            with torch.no_grad():
                layer.lora_b.weight.normal_(0, 0.02)
            layers.append(layer)
    finally:
        torch.set_default_dtype(prev)
    return layers


def _grads(fn, x, layers):
    for layer in layers:
        layer.zero_grad(set_to_none=True)
    xg = x.clone().requires_grad_()
    out = fn(xg)
    outs = out if isinstance(out, tuple) else (out,)
    g = torch.Generator(device=DEV).manual_seed(99)
    torch.autograd.backward(outs, [torch.randn(o.shape, device=DEV, generator=g).to(BF) for o in outs])
    return [xg.grad] + [p.grad for layer in layers for p in (layer.lora_a.weight, layer.lora_b.weight)], [o.detach() for o in outs]


@pytest.mark.parametrize("kind", ["single", "single_two_stage_calls", "qkv_group", "gated_pair", "feed_forward"])
def test_one_expansion_serves_both_directions(kind, monkeypatch):
    """With ``ops.KEEP_FORWARD_TILES_MAX_TOKENS`` at or above the token count the forward call's expanded weight stays
    with the autograd node and the grad-input GEMM reads those forward tiles through transposing LDS reads
    (``ttamd_tiled_linear_dx_bf16`` / ``ttamd_nf4_group_bwd_dx_tiles_bf16``) instead of expanding the weight again.  Same
    products in the same order as the launch on tiles of the transposed weight: every gradient bit for bit - except for
    the gated pair, whose tiles interleave the two members 128 columns at a time, so its grad-input sums the same
    products in another order (rtol 1e-2, atol 2e-3 of unit-variance gradients)."""
    from torchtune_amd.modules.peft import group as group_mod
    from torchtune_amd.modules.peft import lora as lora_mod

    M, K = 2048, 8192   # 8 row tiles: both directions of every layer below give the many-token launch its 256 tiles
    g = torch.Generator(device=DEV).manual_seed(5)
    x = torch.randn(M, K, device=DEV, generator=g).to(BF)
    if kind.startswith("single"):
        layers = _lora_layers([8192], K, 16, seed=1)
        fn = lambda t: layers[0](t)
        if kind == "single_two_stage_calls":
            monkeypatch.setattr(lora_mod, "ONE_CALL_PER_DIRECTION", False)
    elif kind == "qkv_group":
        layers = _lora_layers([4096, 2048, 2048], K, 16, seed=2)
        fn = lambda t: group_mod.lora_linear_group(t, layers)
    elif kind == "gated_pair":
        layers = _lora_layers([4096, 4096], K, 16, seed=3)
        fn = lambda t: group_mod.lora_swiglu_group(t, layers[0], layers[1])
    else:
        layers = _lora_layers([4096, 4096], K, 16, seed=4) + _lora_layers([8192], 4096, 16, seed=5)
        fn = lambda t: group_mod.lora_feed_forward(t, layers[0], layers[1], layers[2])
    calls = {"tiles": 0}
    lib = _lib.load()
    for name in ("ttamd_tiled_linear_dx_bf16", "ttamd_nf4_group_bwd_dx_tiles_bf16"):
        real = getattr(lib, name)

        def counted(*a, _real=real):
            calls["tiles"] += 1
            return _real(*a)

        monkeypatch.setattr(lib, name, counted)
    monkeypatch.setattr(ops, "KEEP_FORWARD_TILES_MAX_TOKENS", 0)
    want, out0 = _grads(fn, x, layers)
    assert calls["tiles"] == 0
    monkeypatch.setattr(ops, "KEEP_FORWARD_TILES_MAX_TOKENS", M)
    got, out1 = _grads(fn, x, layers)
    # the single layer's one-call backward takes the tiles inside the library; the other routes call the entry points above
    if kind != "single":
        assert calls["tiles"] >= 1
    for a, b in zip(out0, out1):
        assert torch.equal(a, b)
    exact = kind in ("single", "single_two_stage_calls", "qkv_group")
    for i, (a, b) in enumerate(zip(got, want)):
        if exact or i > 0 and kind == "gated_pair":
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), (kind, i)
        else:
            torch.testing.assert_close(a.float(), b.float(), rtol=1e-2, atol=2e-3 * max(1.0, float(b.float().abs().max()) / 4))
    # with activation checkpointing: the recomputation keeps the tiles, the first (no-grad) pass does not
    from torch.utils.checkpoint import checkpoint

    ck, _ = _grads(lambda t: checkpoint(fn, t, use_reentrant=False), x, layers)
    for a, b in zip(ck, got):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


@pytest.mark.parametrize("kind", ["single", "qkv_group", "gated_pair", "feed_forward"])
def test_kept_tiles_do_not_outlive_the_first_pass_of_a_checkpointed_forward(kind, monkeypatch):
    """The kept tiles are one of the node's saved tensors, so a checkpointed forward (``use_reentrant=False``) lets go of
    them with everything else it saved: between the forward and the backward of a checkpointed layer no more memory is
    allocated than with the tiles not kept at all (2 B per weight element otherwise - every layer's, in a stack of
    checkpointed layers); without checkpointing they are held, which is what keeping them means."""
    from torch.utils.checkpoint import checkpoint
    from torchtune_amd.modules.peft import group as group_mod

    M, K = 2048, 8192
    g = torch.Generator(device=DEV).manual_seed(6)
    x = torch.randn(M, K, device=DEV, generator=g).to(BF)
    if kind == "single":
        layers = _lora_layers([8192], K, 16, seed=1)
        fn = lambda t: layers[0](t)
    elif kind == "qkv_group":
        layers = _lora_layers([4096, 2048, 2048], K, 16, seed=2)
        fn = lambda t: group_mod.lora_linear_group(t, layers)
    elif kind == "gated_pair":
        layers = _lora_layers([4096, 4096], K, 16, seed=3)
        fn = lambda t: group_mod.lora_swiglu_group(t, layers[0], layers[1])
    else:
        layers = _lora_layers([4096, 4096], K, 16, seed=4) + _lora_layers([8192], 4096, 16, seed=5)
        fn = lambda t: group_mod.lora_feed_forward(t, layers[0], layers[1], layers[2])
    weight_elements = sum(layer.weight.shape[0] * layer.weight.shape[1] for layer in layers if layer.weight.shape[1] == K)

    def held_after_forward(keep_tokens, checkpointed):
        monkeypatch.setattr(ops, "KEEP_FORWARD_TILES_MAX_TOKENS", keep_tokens)
        xg = x.clone().requires_grad_()
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = checkpoint(fn, xg, use_reentrant=False) if checkpointed else fn(xg)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - before
        outs = out if isinstance(out, tuple) else (out,)
        torch.autograd.backward(outs, [torch.ones_like(o) for o in outs])
        return held

    held_after_forward(M, True)   # first calls build the weights' derived caches: not part of what is compared
    assert held_after_forward(M, True) == held_after_forward(0, True)
    assert held_after_forward(M, False) - held_after_forward(0, False) >= 2 * weight_elements


@pytest.mark.parametrize("kind", ["single", "qkv_group", "gated_pair"])
def test_expanded_weights_kept_across_calls(kind, monkeypatch):
    """With a budget in ``ops.RESIDENT_TILES_MAX_BYTES`` the first many-token forward of a layer (or group) leaves its
    expanded weights with the weight; later calls run forward and grad-input on them and launch no expansion.  Outputs and
    gradients: the bits of the calls that expand per call with the forward's tiles handed to the backward
    (``KEEP_FORWARD_TILES_MAX_TOKENS``); a write into the weight drops the tiles; no budget, nothing kept."""
    from torchtune_amd.modules.peft import group as group_mod

    M, K = 2048, 8192
    g = torch.Generator(device=DEV).manual_seed(6)
    x = torch.randn(M, K, device=DEV, generator=g).to(BF)
    if kind == "single":
        layers = _lora_layers([8192], K, 16, seed=11)
        fn = lambda t: layers[0](t)
        tiles_bytes = 2 * 8192 * K
    elif kind == "qkv_group":
        layers = _lora_layers([4096, 2048, 2048], K, 16, seed=12)
        fn = lambda t: group_mod.lora_linear_group(t, layers)
        tiles_bytes = 2 * 8192 * K
    else:
        layers = _lora_layers([4096, 4096], K, 16, seed=13)
        fn = lambda t: group_mod.lora_swiglu_group(t, layers[0], layers[1])
        tiles_bytes = 2 * 8192 * K
    monkeypatch.setattr(ops, "KEEP_FORWARD_TILES_MAX_TOKENS", M)
    monkeypatch.setattr(ops, "RESIDENT_TILES_MAX_BYTES", 0)
    want, out0 = _grads(fn, x, layers)
    assert ops.resident_tiles_bytes() == 0
    # a budget too small for this layer: nothing is kept, nothing changes
    monkeypatch.setattr(ops, "RESIDENT_TILES_MAX_BYTES", tiles_bytes // 2)
    small, out_small = _grads(fn, x, layers)
    assert ops.resident_tiles_bytes() == 0
    for a, b in zip(small + out_small, want + out0):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    monkeypatch.setattr(ops, "RESIDENT_TILES_MAX_BYTES", 1 << 32)
    first, out1 = _grads(fn, x, layers)    # expands, leaves the tiles
    held = ops.resident_tiles_bytes()
    assert tiles_bytes <= held <= tiles_bytes + (8 << 20)
    expansions = {"n": 0}
    lib = _lib.load()
    for name in ("ttamd_qlora_linear_fwd_bf16", "ttamd_nf4_lora_linear_fwd_ws_bf16", "ttamd_nf4_lora_group_fwd_bf16",
                 "ttamd_nf4_lora_group_swiglu_fwd_bf16", "ttamd_nf4_group_bwd_dx_ws_bf16", "ttamd_nf4_linear_bwd_dx_ws_bf16"):
        real = getattr(lib, name)

        def counted(*a, _real=real):
            expansions["n"] += 1
            return _real(*a)

        monkeypatch.setattr(lib, name, counted)
    second, out2 = _grads(fn, x, layers)   # runs on them: none of the entry points that expand is called
    assert expansions["n"] == 0
    assert ops.resident_tiles_bytes() == held
    for a, b, c in zip(first + out1, second + out2, want + out0):
        assert torch.equal(a.view(torch.int16), c.view(torch.int16))
        assert torch.equal(b.view(torch.int16), c.view(torch.int16))
    # with activation checkpointing both passes of the forward run on the kept tiles
    from torch.utils.checkpoint import checkpoint

    ck, _ = _grads(lambda t: checkpoint(fn, t, use_reentrant=False), x, layers)
    assert expansions["n"] == 0
    for a, b in zip(ck, want):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # a write into a weight drops the tiles: the next call follows the new weight and leaves new tiles
    from torchtune_amd import to_nf4

    last = layers[-1]
    new_w = to_nf4((torch.randn(last.weight.shape, device=DEV, generator=g) * 0.02).to(BF))
    with torch.no_grad():
        last.weight.copy_(new_w)
    third, out3 = _grads(fn, x, layers)
    assert expansions["n"] >= 1
    monkeypatch.setattr(ops, "RESIDENT_TILES_MAX_BYTES", 0)
    fresh, out_fresh = _grads(fn, x, layers)
    for a, b in zip(third + out3, fresh + out_fresh):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert not torch.equal(out3[-1], out2[-1])
    del layers, fn, last, new_w
    import gc

    gc.collect()
    assert ops.resident_tiles_bytes() == 0
