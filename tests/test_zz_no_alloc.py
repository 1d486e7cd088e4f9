"""The allocation-free variant of the adapter's hidden product: bit-identical to the workspace variant, also on a second,
smaller call that finds the previous call's partial sums in the built-in scratch array."""
import pytest
import torch

from torchtune_amd import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _both(lib, x, a):
    M, K = x.shape
    r = a.shape[0]
    st = torch.cuda.current_stream().cuda_stream
    want = torch.empty(M, r, dtype=torch.bfloat16, device=DEV)
    nbytes = max(int(lib.ttamd_lora_fwd_workspace_bytes(M, K, r)), 16)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
    _lib.check(lib.ttamd_lora_hidden_bf16(x.data_ptr(), a.data_ptr(), want.data_ptr(), M, K, r, ws.data_ptr(), nbytes, st), "lora_hidden")
    got = torch.full((M, r), float("nan"), dtype=torch.bfloat16, device=DEV)
    _lib.check(lib.ttamd_lora_hidden_static_bf16(x.data_ptr(), a.data_ptr(), got.data_ptr(), M, K, r, st), "lora_hidden_static")
    torch.cuda.synchronize()
    return got, want


def test_static_scratch_variant_matches_the_workspace_variant_on_consecutive_calls():
    lib = _lib.load()
    assert lib.ttamd_lora_hidden_static_max_bytes() == 2 << 20
    g = torch.Generator(device=DEV).manual_seed(0)
    # (M, K, rank): sliced along K with many partial rows, then smaller inputs that reuse part of the same scratch, then a
    # direct (unsliced) launch and the few-token sizes of decode
    for M, K, r in [(512, 14336, 64), (96, 4096, 16), (33, 1024, 8), (8192, 4096, 16), (1, 4096, 16), (2048, 8192, 32)]:
        x = torch.randn(M, K, device=DEV, generator=g).to(torch.bfloat16)
        a = (torch.randn(r, K, device=DEV, generator=g) * 0.05).to(torch.bfloat16)
        got, want = _both(lib, x, a)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (M, K, r)
        ref = x.float() @ a.float().T
        torch.testing.assert_close(got.float(), ref, rtol=1e-2, atol=1e-2 * max(1.0, float(ref.abs().max()) / 8))


def test_static_scratch_variant_allocates_nothing():
    """With inputs and output in place, a call changes neither the device's free memory nor torch's own accounting."""
    lib = _lib.load()
    assert lib.ttamd_lora_hidden_static_init() == 0  # the symbol query of a device's first use, outside the measured call
    g = torch.Generator(device=DEV).manual_seed(1)
    M, K, r = 512, 14336, 64  # sliced along K: the partial sums use the built-in array
    assert 0 < lib.ttamd_lora_fwd_workspace_bytes(M, K, r) <= lib.ttamd_lora_hidden_static_max_bytes()
    x = torch.randn(M, K, device=DEV, generator=g).to(torch.bfloat16)
    a = (torch.randn(r, K, device=DEV, generator=g) * 0.05).to(torch.bfloat16)
    h = torch.empty(M, r, dtype=torch.bfloat16, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.ttamd_lora_hidden_static_bf16(x.data_ptr(), a.data_ptr(), h.data_ptr(), M, K, r, st) == 0  # warm: code loaded
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    alloc0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        assert lib.ttamd_lora_hidden_static_bf16(x.data_ptr(), a.data_ptr(), h.data_ptr(), M, K, r, st) == 0
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (alloc0, reserved0)


def test_static_scratch_variant_rejects_bad_arguments():
    lib = _lib.load()
    x = torch.zeros(64, 128, dtype=torch.bfloat16, device=DEV)
    a = torch.zeros(8, 128, dtype=torch.bfloat16, device=DEV)
    h = torch.zeros(64, 8, dtype=torch.bfloat16, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.ttamd_lora_hidden_static_bf16(x.data_ptr(), a.data_ptr(), h.data_ptr(), 64, 100, 8, st) == -1   # K % 64
    assert lib.ttamd_lora_hidden_static_bf16(x.data_ptr(), a.data_ptr(), h.data_ptr(), 64, 128, 12, st) == -1  # rank % 8
    assert lib.ttamd_lora_hidden_static_bf16(None, a.data_ptr(), h.data_ptr(), 64, 128, 8, st) == -1
    assert b"lora_hidden_static" in lib.ttamd_last_error()
