"""GPU parity of the weight-gradient GEMM ``c = a.T @ b`` (both operands transposed on their way through LDS) and a
determinism check of the two-waves-per-SIMD GEMM kernels.

Oracle: the product in fp32 / fp64 on the same bf16 inputs (the reference computes this matmul in bf16 with fp32
accumulation as well); tolerance rtol 1e-2 / atol 1e-2 scaled with the magnitude of the result, as for the other GEMMs.
With one-hot rows in ``a`` the result is a row of ``b`` exactly (one product 1 * b[m][k], zeros elsewhere), which pins the
operand transposition and the swizzled LDS layout bit for bit."""
import pytest
import torch

from torchtune_amd import _lib, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def test_one_hot_rows_select_rows_of_b_bit_for_bit():
    M, N, K = 512, 256, 512
    g = torch.Generator().manual_seed(0)
    b = torch.randn(M, K, generator=g).to(BF).to(DEV)
    a = torch.zeros(M, N, dtype=BF, device=DEV)
    perm = torch.randperm(M, generator=g)[:N].to(DEV)          # column n of a is one-hot at row perm[n]
    a[perm, torch.arange(N, device=DEV)] = 1.0
    c = ops.gemm_tn(a, b)
    assert torch.equal(c.view(torch.int16), b[perm].contiguous().view(torch.int16))
    # and the other way round: one-hot columns of b select columns of a
    a2 = torch.randn(M, N, generator=g).to(BF).to(DEV)
    b2 = torch.zeros(M, K, dtype=BF, device=DEV)
    perm2 = torch.randperm(M, generator=g)[:K].to(DEV)
    b2[perm2, torch.arange(K, device=DEV)] = 1.0
    c2 = ops.gemm_tn(a2, b2)
    assert torch.equal(c2.view(torch.int16), a2[perm2].t().contiguous().view(torch.int16))


@pytest.mark.parametrize("M,N,K", [(32, 256, 256), (96, 256, 512), (1024, 512, 256), (4096, 1024, 768), (8192, 4096, 4096), (2080, 1792, 1280)])
def test_against_fp32_matmul(M, N, K):
    assert ops.gemm_tn_applies(M, N, K)
    g = torch.Generator().manual_seed(M + N + K)
    a = torch.randn(M, N, generator=g).to(BF).to(DEV)
    b = torch.randn(M, K, generator=g).to(BF).to(DEV)
    c = ops.gemm_tn(a, b)
    want = a.float().t() @ b.float()
    scale = max(1.0, float(want.abs().max()) / 8)
    torch.testing.assert_close(c.float(), want, rtol=1e-2, atol=1e-2 * scale)


@pytest.mark.parametrize("M,N,K", [(8192, 14336, 4096), (8192, 4096, 14336), (4096, 128256, 4096)])
def test_full_size_weight_gradients_of_the_8b_qat_configuration(M, N, K):
    """gate / up, down and one 4096-token chunk of the output projection at their real sizes (batch 2 x 4096,
    ``recipes/configs/llama3_1/8B_qat_full.yaml``; shapes from ``torchtune/models/llama3_1/_model_builders.py:20-59``):
    one-hot rows pin the large-grid indexing bit for bit, random operands are compared with the fp32 product in row
    blocks (the fp32 result of the widest case would not be worth its 2 GB)."""
    assert ops.gemm_tn_applies(M, N, K)
    g = torch.Generator().manual_seed(N + K)
    b = torch.randn(M, K, generator=g).to(BF).to(DEV)
    a = torch.zeros(M, N, dtype=BF, device=DEV)
    R = min(M, N)
    cols = torch.randperm(N, generator=g)[:R].to(DEV)           # row m < R of a is one-hot at column cols[m]
    a[torch.arange(R, device=DEV), cols] = 1.0
    c = ops.gemm_tn(a, b)
    assert torch.equal(c[cols].view(torch.int16), b[:R].view(torch.int16))
    untouched = torch.ones(N, dtype=torch.bool, device=DEV)
    untouched[cols] = False
    assert int(c[untouched].view(torch.int16).count_nonzero()) == 0
    del a, c
    a = torch.randn(M, N, generator=g).to(BF).to(DEV)
    c = ops.gemm_tn(a, b)
    bf = b.float()
    for n0 in range(0, N, 16384):
        want = a[:, n0:n0 + 16384].float().t() @ bf
        scale = max(1.0, float(want.abs().max()) / 8)
        torch.testing.assert_close(c[n0:n0 + 16384].float(), want, rtol=1e-2, atol=1e-2 * scale)


@pytest.mark.parametrize("M,K,Ns", [
    (64, 256, (256, 256)),
    (1024, 512, (512, 256, 256, 768)),
    (8192, 4096, (4096, 1024, 1024)),        # q / k / v of the 8B shape at batch 2 x 4096: 384 tiles, one launch
    (8192, 4096, (14336, 14336)),            # gate / up: seven full rounds instead of two launches of three and a half
], ids=["small", "four_members", "qkv_8b", "gate_up_8b"])
def test_group_launch_equals_member_launches_bitwise(M, K, Ns, monkeypatch):
    """``ttamd_gemm_tn_group_bf16`` against one ``ttamd_gemm_tn_bf16`` per member: the same tiles and the same order of
    sums, so the same bits; the member launches are themselves compared with fp32 products above.  (Without slices of
    the contraction: which tiles of a launch are cut depends on the launch's tile count, see the next test.)"""
    monkeypatch.setattr(ops, "TN_TAIL_SLICES", False)
    g = torch.Generator().manual_seed(M + K + len(Ns))
    b = torch.randn(M, K, generator=g).to(BF).to(DEV)
    a_list = [torch.randn(M, N, generator=g).to(BF).to(DEV) for N in Ns]
    cs = ops.gemm_tn_group(a_list, b)
    assert [tuple(c.shape) for c in cs] == [(N, K) for N in Ns]
    for a, c in zip(a_list, cs):
        assert torch.equal(c.view(torch.int16), ops.gemm_tn(a, b).view(torch.int16))


@pytest.mark.parametrize("M,K,Ns", [
    (8192, 4096, (4096, 1024, 1024)),   # q / k / v at batch 2 x 4096: 384 tiles = one whole round + 128 tiles in two slices
    (8192, 14336, (4096,)),             # down projection: 896 tiles = three rounds + 128 tiles in two slices
    (8192, 4096, (1024,)),              # a k / v projection alone: 64 tiles in four slices
    (4096, 1024, (512, 256)),           # 12 tiles in four slices (a slice keeps at least 32 steps of the 128)
    (8192, 4096, (14336, 14336)),       # whole rounds: nothing is cut
], ids=["qkv_8b", "down_8b", "kv_alone", "few_tiles", "whole_rounds"])
def test_contraction_slices_of_the_last_partial_round(M, K, Ns, monkeypatch):
    """With the workspace ``ttamd_gemm_tn_workspace_bytes`` asks for, the tiles beyond the last whole round of 256 run as
    slices of the contraction whose fp32 partial tiles a second launch adds in slice order: against the fp32 product at
    the tolerance of the unsliced launch, within one bf16 rounding of the unsliced launch (only the order of the fp32
    sums differs), bit-identical from run to run, exact for one-hot operands, and a workspace that is too small falls
    back to the unsliced launch's bits."""
    lib = _lib.load()
    n_total = sum(Ns)
    need = int(lib.ttamd_gemm_tn_workspace_bytes(M, n_total, K))
    tiles = (n_total // 256) * (K // 256)
    if tiles % 256 == 0:
        assert need == 0
    else:
        assert need > 0 and need % (256 * 256 * 4) == 0 and need // (256 * 256 * 4) <= 256
    g = torch.Generator().manual_seed(M + K + n_total)
    b = torch.randn(M, K, generator=g).to(BF).to(DEV)
    a_list = [torch.randn(M, N, generator=g).to(BF).to(DEV) for N in Ns]
    run = (lambda: ops.gemm_tn_group(a_list, b)) if len(Ns) > 1 else (lambda: [ops.gemm_tn(a_list[0], b)])
    sliced = run()
    again = run()
    monkeypatch.setattr(ops, "TN_TAIL_SLICES", False)
    plain = run()
    for a, c, c2, c0 in zip(a_list, sliced, again, plain):
        assert torch.equal(c.view(torch.int16), c2.view(torch.int16))
        want = a.float().t() @ b.float()
        scale = max(1.0, float(want.abs().max()) / 8)
        torch.testing.assert_close(c.float(), want, rtol=1e-2, atol=1e-2 * scale)
        torch.testing.assert_close(c.float(), c0.float(), rtol=2.0 ** -7, atol=2.0 ** -7 * scale)
        if need == 0:
            assert torch.equal(c.view(torch.int16), c0.view(torch.int16))
    if need:
        # through the C ABI with a workspace one byte short: the unsliced launch
        a, N = a_list[0], Ns[0]
        if len(Ns) == 1:
            ws = torch.empty(need, dtype=torch.uint8, device=DEV)
            c = torch.empty(N, K, dtype=BF, device=DEV)
            st = torch.cuda.current_stream().cuda_stream
            assert lib.ttamd_gemm_tn_ws_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, ws.data_ptr(), need - 1, st) == 0
            assert torch.equal(c.view(torch.int16), plain[0].view(torch.int16))
            assert lib.ttamd_gemm_tn_ws_bf16(a.data_ptr(), b.data_ptr(), c.data_ptr(), M, N, K, ws.data_ptr(), need, st) == 0
            assert torch.equal(c.view(torch.int16), sliced[0].view(torch.int16))
        # one-hot rows of a select rows of b exactly, sliced or not
        monkeypatch.setattr(ops, "TN_TAIL_SLICES", True)
        a1 = torch.zeros(M, Ns[0], dtype=BF, device=DEV)
        R = min(M, Ns[0])
        cols = torch.randperm(Ns[0], generator=g)[:R].to(DEV)
        a1[torch.arange(R, device=DEV), cols] = 1.0
        c1 = ops.gemm_tn_group([a1] + a_list[1:], b)[0] if len(Ns) > 1 else ops.gemm_tn(a1, b)
        assert torch.equal(c1[cols].view(torch.int16), b[:R].view(torch.int16))


def test_group_launch_refuses_bad_members():
    b = torch.zeros(64, 256, dtype=BF, device=DEV)
    ok = torch.zeros(64, 256, dtype=BF, device=DEV)
    with pytest.raises(Exception):
        ops.gemm_tn_group([ok, torch.zeros(64, 320, dtype=BF, device=DEV)], b)     # width not a multiple of 256
    with pytest.raises(ValueError):
        ops.gemm_tn_group([ok, torch.zeros(32, 256, dtype=BF, device=DEV)], b)     # rows differ
    with pytest.raises(ValueError):
        ops.gemm_tn_group([ok] * (_lib.GROUP_MAX + 1), b)


def test_unsupported_shapes_are_refused():
    lib = _lib.load()
    assert not ops.gemm_tn_applies(100, 256, 256) and not ops.gemm_tn_applies(64, 320, 256) and not ops.gemm_tn_applies(64, 256, 64)
    a = torch.zeros(64, 320, dtype=BF, device=DEV)
    b = torch.zeros(64, 256, dtype=BF, device=DEV)
    with pytest.raises(Exception):
        ops.gemm_tn(a, b)
    assert b"gemm_tn" in lib.ttamd_last_error()


def test_two_waves_per_simd_kernels_are_deterministic():
    """The same launch twenty times over: identical bits every time, for the expanded-weight GEMM (forward of an NF4
    layer), the tiled GEMM and the transposing GEMM.  The waves of these kernels hand LDS stages to each other across
    workgroup barriers while loads are in flight; a read that raced with a later load would show up here."""
    M, N, K = 4096, 4096, 2048
    g = torch.Generator().manual_seed(3)
    W = (torch.randn(N, K, generator=g) * 0.02).to(BF).to(DEV)
    qdata, qscal, qfac, mean = ops.nf4_quantize(W, 64, 256)
    bscal = ops.nf4_block_scalers(qscal, qfac, mean, 256)
    x = torch.randn(M, K, generator=g).to(BF).to(DEV)
    gy = torch.randn(M, N, generator=g).to(BF).to(DEV)
    tf, tb, _ = ops.fq_per_group_int4_sym_tiled(W, 32)
    first = None
    for _ in range(20):
        out = (ops.nf4_lora_linear_fwd(x, qdata, bscal, N), ops.nf4_linear_bwd_dx(gy, qdata, bscal, K, transposed=None),
               ops.tiled_linear(x, tf, N), ops.tiled_linear(gy, tb, K), ops.gemm_tn(gy, x))
        if first is None:
            first = out
        else:
            for a, b in zip(first, out):
                assert torch.equal(a, b)
