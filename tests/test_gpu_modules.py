"""The reference's own module-level tests for this path, restated against this package on the GPU
(tests/torchtune/modules/peft/test_lora.py, tests/torchtune/modules/low_precision/test_nf4_linear.py,
tests/torchtune/modules/low_precision/test_nf4_dispatch_registration.py)."""
import copy
from functools import partial

import pytest
import torch
from torch import nn

from oracle import lora_oracle, nf4_oracle
from torchtune_amd.modules.common_utils import reparametrize_as_dtype_state_dict_post_hook
from torchtune_amd.modules.low_precision import FrozenNF4Linear
from torchtune_amd.modules.peft import LoRALinear
from torchtune_amd.nf4_tensor import NF4Tensor, to_nf4

pytestmark = pytest.mark.gpu
DEV = "cuda"


class _default_dtype:
    def __init__(self, dtype):
        self.dtype = dtype

    def __enter__(self):
        self.prev = torch.get_default_dtype()
        torch.set_default_dtype(self.dtype)

    def __exit__(self, *a):
        torch.set_default_dtype(self.prev)


def _fixed_init(model):
    with torch.no_grad():
        for _, p in model.named_parameters():
            p.copy_(lora_oracle.fixed_init_tensor(p.shape, dtype=p.dtype).to(p.device))


def _qlora(use_bias, dtype, **kw):
    with _default_dtype(dtype), torch.device(DEV):
        m = LoRALinear(512, 512, rank=4, alpha=1.0, use_bias=use_bias, quantize_base=True, **kw)
    _fixed_init(m)
    return m


def _lora(use_bias, dtype):
    with _default_dtype(dtype), torch.device(DEV):
        m = LoRALinear(512, 512, rank=4, alpha=1.0, use_bias=use_bias)
    _fixed_init(m)
    return m


def test_inplace_copy_attribute_set():
    z = to_nf4(torch.rand(512, 512, dtype=torch.bfloat16, device=DEV))
    assert set(z.__dict__.keys()) == {"block_size", "n_blocks", "scaler_block_size", "quantized_scalers", "quantization_factor",
                                      "scaler_mean", "quantized_data", "nf4"}


@pytest.mark.parametrize("use_bias", [True, False])
def test_lora_weight_nf4_when_quantized(use_bias):
    m = _qlora(use_bias, torch.bfloat16)
    assert isinstance(m.weight, NF4Tensor)
    if use_bias:
        assert not isinstance(m.bias, NF4Tensor) and m.bias.dtype == torch.bfloat16
    m2 = _qlora(True, torch.bfloat16, block_size=8, scaler_block_size=4)
    assert m2.weight.block_size == 8 and m2.weight.scaler_block_size == 4 and not isinstance(m2.bias, NF4Tensor)


@pytest.mark.parametrize("use_bias,dtype", [(False, torch.bfloat16), (True, torch.float32), (False, torch.float32)])
def test_qlora_parity(use_bias, dtype):
    # tests/torchtune/modules/peft/test_lora.py:157-182: same output as a dense LoRA layer holding the dequantised weight
    torch.manual_seed(16)
    q = _qlora(use_bias, dtype)
    d = _lora(use_bias, dtype)
    d.weight.data = q.weight.to(dtype)
    if use_bias:
        d.bias.data = q.bias.detach().clone()
    x = torch.randn(2, 32, 512, dtype=dtype, device=DEV)
    out_d, out_q = d(x), q(x)
    if dtype == torch.bfloat16:
        # rank 4 is not a multiple of 8, so this goes through linear_nf4 (fused base GEMM) + library adapter GEMMs
        torch.testing.assert_close(out_d, out_q, rtol=1.6e-2, atol=1e-5)  # the reference's own (default bf16) tolerances
    else:
        torch.testing.assert_close(out_d, out_q, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_quantized_state_dict(dtype):
    # tests/torchtune/modules/peft/test_lora.py:184-237
    with _default_dtype(dtype), torch.device(DEV):
        layer = LoRALinear(512, 512, rank=4, alpha=1.0, quantize_base=True)
    layer._register_state_dict_hook(partial(reparametrize_as_dtype_state_dict_post_hook, dtype=dtype, offload_to_cpu=False))
    sd = layer.state_dict()
    for v in sd.values():
        assert v.dtype == dtype and not isinstance(v, NF4Tensor)
    with _default_dtype(dtype), torch.device(DEV):
        reload = LoRALinear(512, 512, rank=4, alpha=1.0, quantize_base=True)
    reload.weight = nn.Parameter(to_nf4(torch.zeros_like(layer.weight.get_original_weight(), dtype=dtype, device=layer.weight.device)))
    assert not torch.allclose(layer.weight.quantized_data, reload.weight.quantized_data)
    reload.load_state_dict(sd)
    assert torch.allclose(layer.weight.quantized_data, reload.weight.quantized_data)
    assert torch.equal(layer.weight.quantized_scalers, reload.weight.quantized_scalers)
    # the offloading variant returns CPU tensors
    sd_cpu = {"weight": layer.weight.detach()}
    reparametrize_as_dtype_state_dict_post_hook(layer, sd_cpu, dtype=dtype)
    assert sd_cpu["weight"].device.type == "cpu" and torch.equal(sd_cpu["weight"], sd["weight"].cpu())


@pytest.mark.parametrize("pinned", [True, False])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_state_dict_offload_writes_host_memory_directly(pinned, out_dtype, monkeypatch):
    """`offload_to_cpu=True` (the default of torchtune/modules/common_utils.py:24-59): the dense weight must equal
    the on-device dequantisation bit for bit whether it lands in pinned memory or goes through the staging buffer."""
    from torchtune_amd.modules import common_utils

    monkeypatch.setattr(common_utils, "PINNED_OFFLOAD", pinned)
    w = to_nf4((torch.randn(768, 1024, device=DEV) * 0.02).to(torch.bfloat16))
    other = torch.ones(3, device=DEV)
    expect = w.get_original_weight().to(out_dtype).cpu()
    for _ in range(2):  # the second pass reuses the staging buffer
        sd = {"weight": w, "other": other}
        reparametrize_as_dtype_state_dict_post_hook(None, sd, dtype=out_dtype, offload_to_cpu=True)
        got = sd["weight"]
        assert got.device.type == "cpu" and got.dtype == out_dtype and got.shape == (768, 1024)
        assert got.is_pinned() == pinned
        assert torch.equal(got, expect)
        assert sd["other"] is other
    # the kernel refuses host memory it cannot reach
    with pytest.raises(ValueError, match="pinned host memory"):
        w.get_original_weight(out=torch.empty(768, 1024, dtype=torch.bfloat16))
    with pytest.raises(ValueError, match="contiguous"):
        w.get_original_weight(out=torch.empty(768, 512, dtype=torch.bfloat16, device=DEV))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_frozen_nf4_linear(dtype):
    # tests/torchtune/modules/low_precision/test_nf4_linear.py:24-70
    lin = FrozenNF4Linear(512, 512, device=DEV, dtype=dtype)
    params = list(lin.parameters())
    assert len(params) == 1 and isinstance(params[0], NF4Tensor) and not params[0].requires_grad
    sd = lin.state_dict()
    assert len(sd) == 1 and isinstance(sd["weight"], NF4Tensor)
    for bias in (True, False):
        l2 = FrozenNF4Linear(512, 512, device=DEV, dtype=dtype, bias=bias)
        inp = torch.randn(2, 512, dtype=dtype, device=DEV, requires_grad=True)
        out = l2(inp)
        assert out.dtype == dtype
        out.sum().backward()
        assert inp.grad is not None and inp.grad.dtype == dtype and l2.weight.grad is None
    l3 = FrozenNF4Linear(512, 512, device=DEV, dtype=torch.bfloat16, block_size=16, scaler_block_size=256)
    assert l3.weight.block_size == 16 and l3.weight.scaler_block_size == 256


def test_clone_deepcopy_and_block_scaler_cache():
    t = to_nf4((torch.randn(512, 512, device=DEV) * 0.02).to(torch.bfloat16), 64, 32)
    c = t.clone()  # re-quantisation of the dequantised weight with the default granularity
    assert isinstance(c, NF4Tensor) and c.block_size == 64 and c.scaler_block_size == 256
    assert torch.equal(c.quantized_data, t.quantized_data)
    lin = FrozenNF4Linear(512, 512, device=DEV, dtype=torch.bfloat16)
    lin2 = copy.deepcopy(lin)
    assert isinstance(lin2.weight, NF4Tensor) and torch.equal(lin2.weight.quantized_data, lin.weight.quantized_data)
    assert lin2.weight.quantized_data.data_ptr() != lin.weight.quantized_data.data_ptr()
    s1 = lin.weight.block_scalers()
    assert lin.weight.block_scalers() is s1  # cached
    with torch.no_grad():
        lin.weight.copy_((torch.randn(512, 512, device=DEV) * 0.05).to(torch.bfloat16))
    s2 = lin.weight.block_scalers()
    assert s2 is not s1 and not torch.equal(s1, s2)  # in-place re-quantisation invalidates the cache
    x = torch.randn(4, 512, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    torch.testing.assert_close(lin(x).float(), x.float() @ lin.weight.get_original_weight().float().T, rtol=1e-2, atol=1e-2)
    # the transposed copy used by the grad-input GEMM follows the weight too, and can be switched off
    import torchtune_amd.nf4_tensor as nf4_mod
    c1 = lin.weight.backward_copy()
    assert lin.weight.backward_copy() is c1
    gy = torch.randn(4, 512, device=DEV, dtype=torch.bfloat16)
    (g_fast,) = torch.autograd.grad(lin(x), x, gy)
    with torch.no_grad():
        lin.weight.copy_((torch.randn(512, 512, device=DEV) * 0.05).to(torch.bfloat16))
    assert lin.weight.backward_copy() is not c1
    (g_new,) = torch.autograd.grad(lin(x), x, gy)
    torch.testing.assert_close(g_new.float(), gy.float() @ lin.weight.get_original_weight().float(), rtol=1e-2, atol=1e-2)
    assert not torch.equal(g_new, g_fast)
    nf4_mod.BACKWARD_COPY = False
    try:
        assert lin.weight.backward_copy() is None
        (g_slow,) = torch.autograd.grad(lin(x), x, gy)
    finally:
        nf4_mod.BACKWARD_COPY = True
    torch.testing.assert_close(g_slow.float(), g_new.float(), rtol=1e-2, atol=1e-2)


def test_load_dense_state_dict_into_nf4_model_and_back():
    with _default_dtype(torch.bfloat16), torch.device(DEV):
        layer = LoRALinear(512, 512, rank=8, alpha=16.0, quantize_base=True)
    dense = {"weight": (torch.randn(512, 512) * 0.02).to(torch.bfloat16), "lora_a.weight": torch.randn(8, 512).to(torch.bfloat16),
             "lora_b.weight": torch.randn(512, 8).to(torch.bfloat16)}
    layer.load_state_dict(dense)
    want = to_nf4(dense["weight"].to(DEV))
    assert torch.equal(layer.weight.quantized_data, want.quantized_data)
    fp32 = {k: v.float() for k, v in dense.items()}
    layer.load_state_dict(fp32)  # a float32 checkpoint loads too (cast to the parameter dtype, then quantised)
    assert torch.equal(layer.weight.quantized_data, want.quantized_data)


@pytest.mark.parametrize("N,K,r", [(512, 512, 8), (320, 2240, 16), (256, 4096, 64)])
def test_merged_checkpoint_weight_vs_oracle(N, K, r):
    """get_merged_lora_ckpt on a state dict that still holds the NF4 weight: one HIP pass (dequantise + rank-r update)
    against the eager sequence dequantise -> `+= (alpha/r) * B @ A` in bf16.  The three bf16 roundings are the same;
    only the fp32 summation order of the rank-r product may differ from the CPU BLAS, so: within one bf16 ulp
    everywhere, bit-equal almost everywhere, and exactly the dequantised weight when B is zero."""
    from oracle import lora_oracle
    from torchtune_amd.modules.peft import get_merged_lora_ckpt

    g = torch.Generator().manual_seed(3)
    W = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    A = (torch.randn(r, K, generator=g) * 0.05).to(torch.bfloat16)
    B = (torch.randn(N, r, generator=g) * 0.05).to(torch.bfloat16)
    alpha = 2.0 * r
    sbs = 256 if (N * K // 64) % 256 == 0 else N * K // 64
    want = lora_oracle.merged_weight(nf4_oracle.nf4_quantize(W, 64, sbs), A, B, alpha, r)
    t = to_nf4(W.to(DEV), 64, sbs)
    sd = {"l.weight": t, "l.lora_a.weight": A.to(DEV), "l.lora_b.weight": B.to(DEV), "other": torch.ones(1)}
    out = get_merged_lora_ckpt(sd, rank=r, alpha=alpha)
    assert out.keys() == {"l.weight", "other"}
    got = out["l.weight"].cpu()
    assert got.dtype == torch.bfloat16 and got.shape == (N, K)
    ulp = torch.maximum(want.float().abs(), torch.tensor(2.0 ** -126)) * 2.0 ** -7
    assert torch.all((got.float() - want.float()).abs() <= ulp)
    assert (got.view(torch.int16) == want.view(torch.int16)).float().mean() > 0.98
    sd0 = {"l.weight": t, "l.lora_a.weight": A.to(DEV), "l.lora_b.weight": torch.zeros_like(B).to(DEV)}
    assert torch.equal(get_merged_lora_ckpt(sd0, rank=r, alpha=alpha)["l.weight"], t.get_original_weight())
    # offloading variant: the kernel stores the merged weight straight into pinned host memory, same bits
    sd_h = {"l.weight": t, "l.lora_a.weight": A.to(DEV), "l.lora_b.weight": B.to(DEV)}
    host = get_merged_lora_ckpt(sd_h, rank=r, alpha=alpha, offload_to_cpu=True)["l.weight"]
    assert host.device.type == "cpu" and host.is_pinned() and torch.equal(host, got)


def test_write_through_an_alias_invalidates_the_derived_caches():
    """``param.data.copy_(w)`` / ``param.detach().copy_(w)`` write through an alias that has inner tensor objects of its
    own; the fused forward and backward of the original parameter must then use the scalers and the transposed codes of
    the new weight (checked against the oracle of the new weight)."""
    torch.manual_seed(3)
    with _default_dtype(torch.bfloat16), torch.device(DEV):
        layer = LoRALinear(512, 512, rank=8, alpha=8.0, quantize_base=True)  # rank 8: the fused kernels
    with torch.no_grad():
        layer.lora_b.weight.copy_((torch.randn(512, 8) * 0.01).to(torch.bfloat16))
    x = torch.randn(70, 512, dtype=torch.bfloat16)
    layer(x.to(DEV)).sum().backward()  # fills the block-scaler and transposed-copy caches of the old weight
    for write in (lambda w: layer.weight.data.copy_(w), lambda w: layer.weight.detach().copy_(w)):
        w_new = (torch.randn(512, 512) * 0.05).to(torch.bfloat16)  # unlike the old weight in every block scaler
        with torch.no_grad():
            write(w_new.to(DEV))
        parts = nf4_oracle.nf4_quantize(w_new, 64, 256)
        assert torch.equal(layer.weight.get_original_weight().cpu(), nf4_oracle.nf4_dequantize(parts))
        xd = x.to(DEV).requires_grad_()
        y = layer(xd)
        (y.float() ** 2).sum().backward()
        xo = x.clone().requires_grad_()
        yo = lora_oracle.lora_linear_forward(xo, parts, layer.lora_a.weight.detach().cpu(), layer.lora_b.weight.detach().cpu(), 8.0, 8)
        (yo.float() ** 2).sum().backward()
        torch.testing.assert_close(y.detach().cpu().float(), yo.detach().float(), rtol=1e-2, atol=2e-2)
        gx = xo.grad.float()
        torch.testing.assert_close(xd.grad.cpu().float(), gx, rtol=1e-2, atol=2e-2 * max(1.0, float(gx.abs().max()) / 8))  # the oracle's own backward rounds to bf16 after every op


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_low_ram_state_dict_hook_matches_the_ordinary_hook(out_dtype, monkeypatch):
    """torchtune/modules/common_utils.py:136-237: with the low-host-RAM switch on, the checkpoint of a QLoRA layer holds
    the same dense values (bit for bit) as the ordinary hook's, in one file-backed mapping on the CPU, and loads back into
    an NF4 layer."""
    from torchtune_amd.modules import common_utils

    with _default_dtype(torch.bfloat16), torch.device(DEV):  # random init: no all-zero blocks, so requantisation is exact
        layer = LoRALinear(512, 512, rank=4, alpha=1.0, use_bias=True, quantize_base=True)
    want = {"weight": layer.weight.detach(), "bias": layer.bias.detach(), "lora_a.weight": layer.lora_a.weight.detach(),
            "lora_b.weight": layer.lora_b.weight.detach()}
    reparametrize_as_dtype_state_dict_post_hook(layer, want, dtype=out_dtype, offload_to_cpu=True)
    monkeypatch.setattr(common_utils, "_use_low_cpu_ram", True)
    common_utils._register_reparametrize_state_dict_hooks(layer, dtype=out_dtype, offload_to_cpu=True)
    sd = layer.state_dict()
    assert set(sd) == set(want)
    storages = {v.untyped_storage().data_ptr() for v in sd.values()}
    assert len(storages) == 1
    for k, v in sd.items():
        assert v.device.type == "cpu" and not isinstance(v, NF4Tensor) and v.dtype == want[k].dtype
        assert torch.equal(v, want[k].cpu()), k
    assert sd["weight"].dtype == out_dtype
    with _default_dtype(torch.bfloat16), torch.device(DEV):
        reload = LoRALinear(512, 512, rank=4, alpha=1.0, use_bias=True, quantize_base=True)
    assert not torch.equal(reload.weight.quantized_data, layer.weight.quantized_data)
    reload.load_state_dict(sd)
    assert torch.equal(reload.weight.quantized_data, layer.weight.quantized_data)
