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
    # single-layer benchmark configuration: bf16 [2048, 2048] ~ N(0, 0.02), seed 0, block 64 / scaler block 256
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


def test_every_bf16_scaled_value_and_divisor_range():
    """The bf16 quantise kernel looks codes up in a table and shares one reciprocal per block.  (1) Blocks with absmax 1
    whose other elements sweep every bf16 pattern in [-1, 1]: each pattern must get the oracle's code.  (2) Blocks
    whose absmax runs over all binades, denormals included, with elements at random fractions of it."""
    pats = torch.cat([torch.arange(0x0000, 0x3F81), torch.arange(0x8000, 0xBF81)]).to(torch.int32)
    n_blocks = (pats.numel() + 62) // 63
    body = torch.zeros(n_blocks * 63, dtype=torch.int32)
    body[: pats.numel()] = pats
    w = torch.empty(n_blocks, 64, dtype=torch.bfloat16)
    w[:, 0] = 1.0
    w[:, 1:] = body.to(torch.int16).view(torch.bfloat16).view(n_blocks, 63)
    _assert_matches_oracle(to_nf4(w.to(DEV), 64, 1), nf4_oracle.nf4_quantize(w, 64, 1))

    g = torch.Generator().manual_seed(5)
    amax_bits = torch.randint(0x0001, 0x7F80, (4096,), generator=g, dtype=torch.int32)
    amax_bits[:64] = torch.arange(1, 65)  # denormal divisors: the plain-division path
    amax = amax_bits.to(torch.int16).view(torch.bfloat16)
    frac = torch.rand(4096, 64, generator=g) * 2 - 1
    w = (frac * amax.float()[:, None]).to(torch.bfloat16)
    w[:, 7] = amax
    w[1::2, 7] *= -1
    # codes only: absmaxes spanning 2^-133 .. 2^127 are outside the range where the mean of the absmaxes (and with it
    # the scaler bytes) is independent of the summation order
    assert torch.equal(to_nf4(w.to(DEV), 64, 256).quantized_data.cpu(), nf4_oracle.nf4_quantize(w, 64, 256).quantized_data)


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


def test_one_dimensional_tensor_round_trip():
    """``to_nf4`` takes tensors of one or two dimensions (the reference asserts ``dim() <= 2``): a flat tensor gives the
    same codes and scalers as the same data viewed as a matrix, and dequantises back to its own shape."""
    g = torch.Generator(device="cuda").manual_seed(3)
    flat = (torch.randn(256 * 64 * 2, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
    a = to_nf4(flat)
    b = to_nf4(flat.view(128, 256))
    assert a.shape == flat.shape and a.get_original_weight().shape == flat.shape
    assert torch.equal(a.quantized_data, b.quantized_data) and torch.equal(a.quantized_scalers, b.quantized_scalers)
    assert torch.equal(a.get_original_weight(), b.get_original_weight().view(-1))
