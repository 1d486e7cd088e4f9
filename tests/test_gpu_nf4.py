"""GPU parity of the NF4 codec kernels against the CPU oracle: bit-exact codes, scaler bytes, factors, mean and
dequantised values, through the Python binding and through raw C-ABI calls."""
import ctypes

import pytest
import torch

from oracle import nf4_oracle
from tests.helpers import bits_equal, seeded_weight
from torchtune_amd import _lib, ops
from torchtune_amd.nf4_tensor import NF4Tensor, to_nf4

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _assert_matches_oracle(t: NF4Tensor, p: nf4_oracle.NF4Parts):
    assert torch.equal(t.quantized_data.cpu(), p.quantized_data)
    assert torch.equal(t.quantized_scalers.cpu(), p.quantized_scalers)
    assert bits_equal(t.quantization_factor.cpu(), p.quantization_factor)
    assert bits_equal(t.scaler_mean.cpu().reshape(1), p.scaler_mean.reshape(1))
    assert bits_equal(t.nf4.cpu(), p.nf4)
    assert (t.block_size, t.n_blocks, t.scaler_block_size) == (p.block_size, p.n_blocks, p.scaler_block_size)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize(
    "shape,bs,sbs",
    [((2048, 2048), 64, 256), ((512, 512), 8, 4), ((512, 512), 16, 256), ((64, 2048), 128, 32), ((16384,), 64, 256),
     ((1024, 64), 64, 1), ((512, 1024), 512, 8), ((768, 128), 64, 3)],
)
def test_quantise_and_dequantise_bit_exact(dtype, shape, bs, sbs):
    w = seeded_weight(shape, dtype, seed=0)
    if w.dim() == 2:
        w[1, 3] = 0.4  # outlier
        w[2] = 0  # a run of all-zero blocks
    p = nf4_oracle.nf4_quantize(w, bs, sbs)
    t = to_nf4(w.to(DEV), bs, sbs)
    _assert_matches_oracle(t, p)
    d = t.get_original_weight()
    assert d.shape == w.shape and d.dtype == dtype and d.is_cuda
    want = nf4_oracle.nf4_dequantize(p)
    # all-zero blocks dequantise to +-0 * scaler: compare bits
    assert bits_equal(d.cpu(), want)
    assert torch.equal(t.block_scalers().cpu(), nf4_oracle.nf4_dequantize_scalers(p).float())


def test_config1_weight_through_raw_c_abi():
    # BASELINE config 1: bf16 [2048, 2048] ~ N(0, 0.02), seed 0, block 64 / scaler block 256
    torch.manual_seed(0)
    w = (torch.randn(2048, 2048) * 0.02).to(torch.bfloat16)
    p = nf4_oracle.nf4_quantize(w, 64, 256)
    lib = _lib.load()
    wd = w.to(DEV)
    numel = w.numel()
    qdata = torch.empty(numel // 2, dtype=torch.uint8, device=DEV)
    qs = torch.empty(numel // 64, dtype=torch.int8, device=DEV)
    qf = torch.empty(numel // 64 // 256, dtype=torch.bfloat16, device=DEV)
    mean = torch.empty(1, dtype=torch.bfloat16, device=DEV)
    ws = torch.empty(lib.ttamd_nf4_quantize_workspace_bytes(numel, 64), dtype=torch.uint8, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    rc = lib.ttamd_nf4_quantize(wd.data_ptr(), 0, numel, 64, 256, qdata.data_ptr(), qs.data_ptr(), qf.data_ptr(),
                                mean.data_ptr(), ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, lib.ttamd_last_error()
    out = torch.empty(numel, dtype=torch.bfloat16, device=DEV)
    rc = lib.ttamd_nf4_dequantize(qdata.data_ptr(), qs.data_ptr(), qf.data_ptr(), mean.data_ptr(), 0, numel, 64, 256,
                                  out.data_ptr(), stream)
    assert rc == 0, lib.ttamd_last_error()
    torch.cuda.synchronize()
    assert torch.equal(qdata.cpu(), p.quantized_data) and torch.equal(qs.cpu(), p.quantized_scalers)
    assert bits_equal(qf.cpu(), p.quantization_factor) and bits_equal(mean.cpu(), p.scaler_mean.reshape(1))
    assert bits_equal(out.cpu().view(2048, 2048), nf4_oracle.nf4_dequantize(p))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dequantise_every_code_and_scaler_byte(dtype):
    codes = torch.arange(16, dtype=torch.uint8)
    packed = ((codes[:, None] << 4) | codes[None, :]).flatten().repeat(256)
    qs = torch.arange(-128, 128, dtype=torch.int8)
    for factor, mean in ((257.0, 0.0625), (1000.0, 0.02), (3.0, -0.5)):
        p = nf4_oracle.NF4Parts(512, 256, 256, qs, torch.tensor([factor], dtype=dtype), torch.tensor(mean, dtype=dtype), packed,
                                torch.tensor(nf4_oracle.NF4_TABLE, dtype=dtype), torch.Size([256, 512]), dtype)
        got = ops.nf4_dequantize(packed.to(DEV), qs.to(DEV), p.quantization_factor.to(DEV), p.scaler_mean.to(DEV), (256, 512),
                                 512, 256)
        assert bits_equal(got.cpu(), nf4_oracle.nf4_dequantize(p))


def test_degenerate_inputs():
    z = to_nf4(torch.zeros(512, 512, dtype=torch.bfloat16, device=DEV))
    assert torch.all(z.quantized_data == 0) and torch.all(z.quantized_scalers == 0)
    const = torch.full((512, 512), 0.25, dtype=torch.bfloat16)
    t = to_nf4(const.to(DEV))
    _assert_matches_oracle(t, nf4_oracle.nf4_quantize(const, 64, 256))
    assert torch.equal(t.get_original_weight().cpu(), const)
    with pytest.raises(AssertionError, match="divisible by block size"):
        to_nf4(torch.zeros(100, 3, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(AssertionError, match="scaler_block_size"):
        to_nf4(torch.zeros(64, 64, dtype=torch.bfloat16, device=DEV))
    with pytest.raises(ValueError, match="power of two"):
        to_nf4(torch.zeros(96, 96, dtype=torch.bfloat16, device=DEV), 24, 4)


def test_full_size_properties_mlp_weight():
    # Llama-3.1-8B gate projection [14336, 4096]: too large for the eager oracle in a test, so check what must
    # hold at any size: requantisation idempotence, absmax element on an end code, reconstruction error bound,
    # and agreement with the oracle on a slice of whole scaler blocks
    g = torch.Generator(device=DEV).manual_seed(0)
    w = (torch.randn(14336, 4096, device=DEV, generator=g) * 0.02).to(torch.bfloat16)
    t = to_nf4(w)
    d = t.get_original_weight()
    t2 = to_nf4(d)
    assert torch.equal(t.quantized_data, t2.quantized_data)
    blocks = w.view(-1, 64).float()
    absmax = blocks.abs().amax(1)
    err = (d.view(-1, 64).float() - blocks).abs().amax(1)
    scaler = t.block_scalers().float()
    assert torch.all(err <= absmax * 0.1519 * 1.02 + (scaler - absmax).abs() + 1e-3 * absmax)
    codes = torch.stack([t.quantized_data >> 4, t.quantized_data & 0xF], dim=1).flatten().view(-1, 64)
    at = codes.gather(1, blocks.abs().argmax(1, keepdim=True))
    assert torch.all((at == 0) | (at == 15))
    rows = 64  # 64 rows x 4096 = 4096 blocks = 16 scaler blocks; codes do not depend on the rest of the tensor
    p = nf4_oracle.nf4_quantize(w[:rows].cpu(), 64, 256)
    assert torch.equal(t.quantized_data[: rows * 4096 // 2].cpu(), p.quantized_data)


def test_cpu_resident_tensor_is_staged_through_the_gpu():
    w = seeded_weight((512, 512), torch.bfloat16, seed=9)
    t = to_nf4(w)  # CPU in, CPU out, arithmetic on the GPU
    assert t.device.type == "cpu" and t.quantized_data.device.type == "cpu"
    _assert_matches_oracle(t, nf4_oracle.nf4_quantize(w, 64, 256))
    assert bits_equal(t.get_original_weight(), nf4_oracle.nf4_dequantize(nf4_oracle.nf4_quantize(w, 64, 256)))
    g = t.to(DEV)
    assert isinstance(g, NF4Tensor) and g.quantized_data.is_cuda and torch.equal(g.cpu().quantized_data, t.quantized_data)
