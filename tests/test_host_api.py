"""CPU-only checks of the host side: the C-ABI library loads and exports every declared symbol, argument
validation works without a GPU, the shared rounding code matches the oracle exhaustively, and the Python surface
mirrors the reference's (names, attributes, error messages)."""
import ctypes
import os
import re
import subprocess

import pytest
import torch
from torch import nn

import torchtune_amd
from oracle import lora_oracle, nf4_oracle
from torchtune_amd import _lib, ops
from torchtune_amd.modules.low_precision import FrozenNF4Linear
from torchtune_amd.modules.peft import LoRALinear, QATLoRALinear, get_adapter_params, set_trainable_params
from torchtune_amd.nf4_tensor import NF4Tensor, to_nf4
from torchtune_amd.qat import (
    FakeQuantizeConfig,
    FakeQuantizedLinear,
    FakeQuantizer,
    Int8DynActInt4WeightQATLinear,
    Int8DynActInt4WeightQATQuantizer,
)
from torchtune_amd.training import quantization

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "torchtune_amd.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ttamd_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_symbols()
    assert len(declared) >= 15
    for name in declared:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == declared, "ctypes prototypes and header disagree"
    assert lib.ttamd_version() == _lib.ABI_VERSION == 1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(_lib.LibraryNotBuiltError, match="no compute path without its HIP library"):
        _lib.load()


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    aligned = ctypes.c_void_p((p.value + 255) & ~255)
    # numel not divisible by the block size
    rc = lib.ttamd_nf4_quantize(aligned, 0, 100, 64, 256, aligned, aligned, aligned, aligned, aligned, 4096, None)
    assert rc == -1 and b"divisible by block_size" in lib.ttamd_last_error()
    rc = lib.ttamd_nf4_quantize(aligned, 0, 64 * 10, 64, 256, aligned, aligned, aligned, aligned, aligned, 4096, None)
    assert rc == -1 and b"scaler_block_size" in lib.ttamd_last_error()
    rc = lib.ttamd_nf4_quantize(aligned, 7, 64 * 256, 64, 256, aligned, aligned, aligned, aligned, aligned, 4096, None)
    assert rc == -1 and b"dtype" in lib.ttamd_last_error()
    rc = lib.ttamd_nf4_quantize(None, 0, 64 * 256, 64, 256, aligned, aligned, aligned, aligned, aligned, 4096, None)
    assert rc == -1 and b"null" in lib.ttamd_last_error()
    # workspace too small is its own code
    rc = lib.ttamd_nf4_quantize(aligned, 0, 64 * 256, 64, 256, aligned, aligned, aligned, aligned, aligned, 16, None)
    assert rc == -3 and b"workspace" in lib.ttamd_last_error()
    assert lib.ttamd_nf4_quantize_workspace_bytes(64 * 256, 64) >= 256 * 4
    # fused GEMM shape rules
    rc = lib.ttamd_nf4_lora_linear_fwd_bf16(aligned, aligned, aligned, None, None, None, 0, 0.0, None, aligned, 8, 64, 100, None)
    assert rc == -1 and b"multiple of the NF4 block size" in lib.ttamd_last_error()
    rc = lib.ttamd_nf4_lora_linear_fwd_bf16(aligned, aligned, aligned, None, None, None, 8, 2.0, None, aligned, 8, 64, 64, None)
    assert rc == -1 and b"adapter pointers" in lib.ttamd_last_error()
    rc = lib.ttamd_nf4_linear_bwd_dx_bf16(aligned, aligned, aligned, None, None, aligned, aligned, 12, aligned, 8, 64, 64, None)
    assert rc == -1 and b"rank" in lib.ttamd_last_error()
    rc = lib.ttamd_fq_per_group_int4_sym(aligned, 0, 4, 64, 24, 1, aligned, None, None)
    assert rc == -1 and b"group_size" in lib.ttamd_last_error()
    rc = lib.ttamd_fq_per_token_int8_asym(aligned, 0, 4, 12, 1, aligned, None, None, None)
    assert rc == -1 and b"multiple of 8" in lib.ttamd_last_error()
    with pytest.raises(ValueError, match="multiple of 8"):
        _lib.check(rc, "fq_per_token")


@pytest.fixture(scope="module")
def host_math(tmp_path_factory):
    """torchtune_amd/csrc/nf4_math.h compiled for the host: the same source the kernels use."""
    d = tmp_path_factory.mktemp("hostmath")
    src = d / "host_math.cpp"
    src.write_text(
        '#include "%s"\n'
        'extern "C" int code_bf16(float s) { return ttamd::nf4_nearest_code<true>(s); }\n'
        'extern "C" int code_f32(float s) { return ttamd::nf4_nearest_code<false>(s); }\n'
        'extern "C" float scaler_bf16(int q, float f, float m) { return ttamd::nf4_block_scaler<true>(q, f, m); }\n'
        'extern "C" float scaler_f32(int q, float f, float m) { return ttamd::nf4_block_scaler<false>(q, f, m); }\n'
        'extern "C" void codes_bf16(const float* s, int n, int* out) { for (int i = 0; i < n; ++i) out[i] = code_bf16(s[i]); }\n'
        'extern "C" void codes_f32(const float* s, int n, int* out) { for (int i = 0; i < n; ++i) out[i] = code_f32(s[i]); }\n'
        % os.path.join(ROOT, "torchtune_amd", "csrc", "nf4_math.h")
    )
    so = d / "host_math.so"
    subprocess.run(["g++", "-O2", "-std=c++17", "-shared", "-fPIC", "-ffp-contract=off", str(src), "-o", str(so)], check=True)
    lib = ctypes.CDLL(str(so))
    lib.scaler_bf16.restype = ctypes.c_float
    lib.scaler_bf16.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_float]
    lib.scaler_f32.restype = ctypes.c_float
    lib.scaler_f32.argtypes = [ctypes.c_int, ctypes.c_float, ctypes.c_float]
    return lib


def test_kernel_code_search_matches_oracle_on_every_bf16_pattern(host_math):
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    table = torch.tensor(nf4_oracle.NF4_TABLE, dtype=torch.bfloat16)
    want = (pats[:, None] - table[None, :]).abs().argmin(dim=-1).to(torch.int32)
    want[pats.isnan()] = 0
    s = pats.float().contiguous()
    got = torch.empty(65536, dtype=torch.int32)
    host_math.codes_bf16(ctypes.c_void_p(s.data_ptr()), 65536, ctypes.c_void_p(got.data_ptr()))
    assert torch.equal(got, want)


def test_kernel_code_search_matches_oracle_fp32(host_math):
    g = torch.Generator().manual_seed(0)
    table = torch.tensor(nf4_oracle.NF4_TABLE)
    mids = (table[1:] + table[:-1]) / 2
    near = torch.cat([mids + d for d in (-2e-7, -6e-8, 0.0, 6e-8, 2e-7)])
    s = torch.cat([torch.rand(200000, generator=g) * 2 - 1, table, near, torch.tensor([float("nan"), 0.0, -0.0])]).contiguous()
    want = (s[:, None] - table[None, :]).abs().argmin(dim=-1).to(torch.int32)
    want[s.isnan()] = 0
    got = torch.empty(s.numel(), dtype=torch.int32)
    host_math.codes_f32(ctypes.c_void_p(s.data_ptr()), s.numel(), ctypes.c_void_p(got.data_ptr()))
    assert torch.equal(got, want)


def test_kernel_block_scaler_matches_oracle(host_math):
    for dtype, fn in ((torch.bfloat16, host_math.scaler_bf16), (torch.float32, host_math.scaler_f32)):
        for factor, mean in ((257.0, 0.0625), (999.0, 0.0211), (3.0, -0.5)):
            qs = torch.arange(-128, 128, dtype=torch.int8)
            p = nf4_oracle.NF4Parts(64, 256, 256, qs, torch.tensor([factor], dtype=dtype), torch.tensor(mean, dtype=dtype),
                                    torch.zeros(64 * 128, dtype=torch.uint8), torch.tensor(nf4_oracle.NF4_TABLE, dtype=dtype),
                                    torch.Size([256, 64]), dtype)
            want = nf4_oracle.nf4_dequantize_scalers(p).float()
            f, m = p.quantization_factor.float().item(), p.scaler_mean.float().item()
            got = torch.tensor([fn(int(q), f, m) for q in qs])
            assert torch.equal(got, want)


# ---- Python surface ---------------------------------------------------------------------------------------
def test_lora_linear_surface_and_known_answer():
    m = LoRALinear(in_dim=64, out_dim=128, rank=4, alpha=1.0, use_bias=True)
    for attr in ("in_dim", "out_dim", "rank", "alpha", "use_bias", "_quantize_base", "disabled", "merged", "weight", "bias",
                 "dropout", "lora_a", "lora_b"):
        assert hasattr(m, attr)
    assert m.adapter_params() == ["lora_a.weight", "lora_b.weight"]
    assert isinstance(m.dropout, nn.Identity) and isinstance(LoRALinear(8, 8, 2, 1.0, dropout=0.1).dropout, nn.Dropout)
    assert torch.all(m.lora_b.weight == 0)  # B starts at zero
    assert m.lora_a.weight.abs().max() <= 1 / 64 ** 0.5
    assert [n for n, _ in m.named_parameters()] == ["weight", "bias", "lora_a.weight", "lora_b.weight"]
    with torch.no_grad():
        for _, p in m.named_parameters():
            p.copy_(lora_oracle.fixed_init_tensor(p.shape))
    torch.manual_seed(16)
    x = torch.randn(2, 32, 64)
    torch.testing.assert_close(m(x).mean(), torch.tensor(1.1252), atol=1e-4, rtol=1e-6)
    m.disabled = True
    torch.testing.assert_close(m(x), torch.nn.functional.linear(x, m.weight, m.bias))
    set_trainable_params(m, get_adapter_params(m))
    assert [n for n, p in m.named_parameters() if p.requires_grad] == ["lora_a.weight", "lora_b.weight"]


def test_lora_linear_rejects_quantisation_kwargs_without_quantize_base():
    with pytest.raises(ValueError, match="``quantize_base`` is False, but received the following quantization arguments"):
        LoRALinear(512, 512, 4, 1.0, use_bias=True, quantize_base=False, block_size=8, scaler_block_size=4)


def test_qat_lora_linear_surface():
    base = LoRALinear(64, 128, 4, 1.0)
    with torch.no_grad():
        for _, p in base.named_parameters():
            p.copy_(lora_oracle.fixed_init_tensor(p.shape))
    q = QATLoRALinear.from_lora_linear(base)
    assert isinstance(q.activation_fake_quantizer, nn.Identity) and isinstance(q.weight_fake_quantizer, nn.Identity)
    assert q.weight is base.weight and q.lora_a.weight is base.lora_a.weight
    torch.manual_seed(16)
    torch.testing.assert_close(q(torch.randn(2, 32, 64)).mean(), torch.tensor(0.6291), atol=1e-4, rtol=1e-6)
    with pytest.raises(ValueError, match="Bias is not supported in QAT \\+ LoRA yet"):
        QATLoRALinear.from_lora_linear(LoRALinear(64, 128, 4, 1.0, use_bias=True))
    with pytest.raises(ValueError, match="in_dim \\(100\\) must be divisible by group_size \\(32\\)"):
        QATLoRALinear(100, 64, 4, 1.0, weight_qat_config=FakeQuantizeConfig(torch.int4, group_size=32))


def test_quantisation_needs_a_gpu_and_says_so():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(RuntimeError, match="needs an AMD GPU"):
        to_nf4(torch.randn(512, 512))
    with pytest.raises(RuntimeError, match="needs an AMD GPU"):
        LoRALinear(512, 512, 8, 16.0, quantize_base=True)
    with pytest.raises(RuntimeError, match="expected a tensor on an AMD GPU"):
        ops.fq_per_token_int8_asym(torch.randn(4, 64))


def _cpu_nf4(shape=(512, 512), dtype=torch.bfloat16, bs=64, sbs=256) -> NF4Tensor:
    """An NF4Tensor assembled from oracle parts, so the host-side tensor mechanics can run without a GPU."""
    p = nf4_oracle.nf4_quantize((torch.randn(shape, generator=torch.Generator().manual_seed(0)) * 0.02).to(dtype), bs, sbs)
    return NF4Tensor(p.shape, p.dtype, p.block_size, p.n_blocks, p.scaler_block_size, p.quantized_scalers,
                     p.quantization_factor, p.scaler_mean, p.quantized_data, p.nf4)


def test_nf4_tensor_host_mechanics():
    t = _cpu_nf4()
    # the attribute set pinned by tests/torchtune/modules/low_precision/test_nf4_dispatch_registration.py:22-31
    assert set(t.__dict__.keys()) == {"block_size", "n_blocks", "scaler_block_size", "quantized_scalers", "quantization_factor",
                                      "scaler_mean", "quantized_data", "nf4"}
    assert t.shape == (512, 512) and t.dtype == torch.bfloat16 and t.device.type == "cpu" and not t.is_meta
    assert t.quantized_data.dtype == torch.uint8 and t.quantized_data.numel() == 512 * 512 // 2
    assert t.quantized_scalers.dtype == torch.int8 and t.quantization_factor.dtype == torch.bfloat16 and t.nf4.numel() == 16
    d = t.detach()
    assert isinstance(d, NF4Tensor) and d.quantized_data.data_ptr() == t.quantized_data.data_ptr()
    p = nn.Parameter(t, requires_grad=False)
    assert isinstance(p, NF4Tensor) and not p.requires_grad
    lin = nn.Linear(512, 512, bias=False, dtype=torch.bfloat16)
    torch.utils.swap_tensors(lin.weight, p)
    assert isinstance(lin.weight, NF4Tensor)
    sd = lin.state_dict()
    assert isinstance(sd["weight"], NF4Tensor) and len(sd) == 1
    # same-layout NF4 -> NF4 copy_ copies the packed representation without arithmetic
    other = _cpu_nf4()
    other.quantized_data.zero_()
    other.copy_(t)
    assert torch.equal(other.quantized_data, t.quantized_data) and torch.equal(other, t)
    assert "NF4Tensor(shape=(512, 512)" in repr(t)
    names, ctx = t.__tensor_flatten__()
    back = NF4Tensor.__tensor_unflatten__({n: getattr(t, n) for n in names}, ctx)
    assert torch.equal(back, t)


def test_fake_quantize_config_validation():
    c = FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False)
    assert c.group_size is None and not c.is_symmetric and c.scale_precision == torch.float32 and c.zero_point_precision == torch.int32
    w = FakeQuantizeConfig(torch.int4, group_size=32)
    assert w.group_size == 32 and w.is_symmetric and w.mapping_type == "SYMMETRIC"
    assert FakeQuantizeConfig(torch.int4, "per_group", group_size=8).group_size == 8
    with pytest.raises(ValueError, match="Cannot set both"):
        FakeQuantizeConfig(torch.int4, "per_group", group_size=8, mapping_type="symmetric", is_symmetric=True)
    with pytest.raises(ValueError, match="At least one of"):
        FakeQuantizeConfig(torch.int4)
    with pytest.raises(ValueError, match="Unexpected granularity"):
        FakeQuantizeConfig(torch.int8, "per_banana")
    with pytest.raises(NotImplementedError):
        FakeQuantizer(FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=True))
    with pytest.raises(NotImplementedError):
        FakeQuantizeConfig(torch.float16, "per_token")


def test_quantizer_prepare_and_toggles_on_cpu():
    model = nn.Sequential(nn.Linear(64, 128, bias=False), nn.ReLU(), nn.Sequential(nn.Linear(128, 64), nn.Linear(50, 8)))
    qz = Int8DynActInt4WeightQATQuantizer(groupsize=32)
    assert quantization.get_quantizer_mode(qz) == "8da4w-qat" and quantization.get_quantizer_mode(object()) is None
    w0 = model[0].weight.detach().clone()
    model = qz.prepare(model)
    assert isinstance(model[0], Int8DynActInt4WeightQATLinear) and isinstance(model[0], FakeQuantizedLinear)
    assert isinstance(model[2][0], Int8DynActInt4WeightQATLinear) and model[2][0].bias is not None
    assert type(model[2][1]) is nn.Linear  # 50 % 32 != 0: left alone
    assert torch.equal(model[0].weight, w0)
    assert model[0].activation_fake_quantizer.config.granularity.__class__.__name__ == "PerToken"
    assert model[0].weight_fake_quantizer.config.group_size == 32
    assert qz.get_weight_fake_quantize_config().group_size == 32 and not qz.get_activation_fake_quantize_config().is_symmetric
    disable = quantization._get_disable_fake_quant("8da4w-qat")
    enable = quantization._get_enable_fake_quant("8da4w-qat")
    model.apply(disable)
    assert not model[0].activation_fake_quantizer.enabled and not model[0].weight_fake_quantizer.enabled
    x = torch.randn(3, 64)
    torch.testing.assert_close(model[0](x), x @ w0.T)  # disabled fake quant = plain linear, no kernel involved
    model.apply(enable)
    assert model[2][0].weight_fake_quantizer.enabled
    assert quantization._get_enable_fake_quant("4w") is None
    with pytest.raises(ValueError, match="must be == 0"):
        FakeQuantizedLinear(50, 8, weight_config=FakeQuantizeConfig(torch.int4, group_size=32))


def test_weight_only_int4_quantizer_prepare_and_toggles_on_cpu():
    """The "4w-qat" mode (torchtune/training/quantization.py:27,125-127): module swap, shape rule, config, toggles."""
    from torchtune_amd.qat import Int4WeightOnlyQATLinear, Int4WeightOnlyQATQuantizer, WeightOnlyInt4Linear, ZeroPointDomain

    model = nn.Sequential(nn.Linear(256, 64, bias=False), nn.Linear(256, 8, bias=True), nn.Linear(160, 8, bias=False)).to(torch.bfloat16)
    qz = Int4WeightOnlyQATQuantizer(groupsize=32)
    assert quantization.get_quantizer_mode(qz) == "4w-qat"
    w0 = model[0].weight.detach().clone()
    model = qz.prepare(model)
    assert isinstance(model[0], Int4WeightOnlyQATLinear) and isinstance(model[0], FakeQuantizedLinear)
    assert type(model[1]) is nn.Linear  # has a bias: left alone
    assert type(model[2]) is nn.Linear  # 160 % (16 * inner_k_tiles) != 0: left alone
    assert model[0].activation_fake_quantizer is None and torch.equal(model[0].weight, w0)
    cfg = model[0].weight_fake_quantizer.config
    assert (cfg.dtype, cfg.group_size, cfg.is_symmetric, cfg.zero_point_domain) == (torch.uint4, 32, False, ZeroPointDomain.FLOAT)
    assert cfg.scale_precision == torch.bfloat16 and cfg.zero_point_precision == torch.bfloat16
    model.apply(quantization._get_disable_fake_quant("4w-qat"))
    assert not model[0].weight_fake_quantizer.enabled
    x = torch.randn(3, 256).to(torch.bfloat16)
    torch.testing.assert_close(model[0](x), x @ w0.T)  # disabled fake quant = plain linear, no kernel involved
    model.apply(quantization._get_enable_fake_quant("4w-qat"))
    assert model[0].weight_fake_quantizer.enabled
    with pytest.raises(ValueError, match="Padding for QAT 4w is not supported yet"):
        Int4WeightOnlyQATLinear(160, 8, groupsize=32)
    with pytest.raises(AssertionError):
        Int4WeightOnlyQATQuantizer(groupsize=48)
    with pytest.raises(NotImplementedError):  # integer zero points for uint4 have no kernel
        FakeQuantizer(FakeQuantizeConfig(torch.uint4, group_size=32, is_symmetric=False))
    conv = WeightOnlyInt4Linear(256, 64, groupsize=32)
    assert conv.weight.shape == (64, 128) and conv.weight.dtype == torch.uint8
    assert conv.scales_and_zeros.shape == (8, 64, 2) and conv.scales_and_zeros.dtype == torch.bfloat16


def test_quantizer_modes_cover_the_reference_table():
    """Every entry of the reference's mode tables (torchtune/training/quantization.py:94-97,124-127,141-163)."""
    expect = {
        quantization.Int8DynActInt4WeightQuantizer: "8da4w",
        quantization.Int8DynActInt4WeightQATQuantizer: "8da4w-qat",
        quantization.Int4WeightOnlyQuantizer: "4w",
        quantization.Int4WeightOnlyQATQuantizer: "4w-qat",
        quantization.Int4WeightOnlyQATQuantizerModuleSwap: "4w-qat-module-swap",
        quantization.Int8DynActInt4WeightQATQuantizerModuleSwap: "8da4w-qat-module-swap",
    }
    for cls, mode in expect.items():
        assert quantization.get_quantizer_mode(cls()) == mode
        has_toggle = "qat" in mode
        assert (quantization._get_enable_fake_quant(mode) is not None) == has_toggle
        assert (quantization._get_disable_fake_quant(mode) is not None) == has_toggle
    assert quantization.Int8DynActInt4WeightQuantizer().groupsize == 256
    assert (quantization.Int4WeightOnlyQuantizer().groupsize, quantization.Int4WeightOnlyQuantizer().inner_k_tiles) == (128, 8)
    assert quantization.disable_8da4w_fake_quant_module_swap is quantization._disable_linear_fake_quant
    assert quantization.enable_4w_fake_quant_module_swap is quantization._enable_linear_fake_quant


def test_swap_lora_linear_with_qat():
    model = nn.Sequential(LoRALinear(64, 64, 4, 1.0), nn.Sequential(LoRALinear(64, 32, 4, 1.0)))
    quantization.swap_lora_linear_with_qat(model, None, FakeQuantizeConfig(torch.int4, group_size=32))
    assert isinstance(model[0], QATLoRALinear) and isinstance(model[1][0], QATLoRALinear)
    assert isinstance(model[0].weight_fake_quantizer, FakeQuantizer) and isinstance(model[0].activation_fake_quantizer, nn.Identity)


def test_package_exports():
    for name in ("NF4Tensor", "to_nf4", "linear_nf4", "implements", "FrozenNF4Linear", "LoRALinear", "QATLoRALinear",
                 "Int8DynActInt4WeightQATQuantizer", "FakeQuantizeConfig", "FakeQuantizer", "FakeQuantizedLinear"):
        assert hasattr(torchtune_amd, name)
    assert FrozenNF4Linear.__mro__[1] is nn.Linear


def test_reference_known_answer_merged_lora_ckpt():
    """The 6x4 merged weight the reference's own test holds (tests/torchtune/modules/peft/test_utils.py:451-480),
    through get_merged_lora_ckpt on dense CPU tensors; the adapter entries are deleted and the dict is returned."""
    import json
    import os

    from torchtune_amd.modules.peft import get_merged_lora_ckpt

    with open(os.path.join(os.path.dirname(__file__), "golden", "reference_known_answers.json")) as f:
        kat = json.load(f)["merged_lora_ckpt"]
    sd = {
        "0.weight": 3 * torch.ones(6, 4),
        "0.lora_a.weight": torch.tensor(kat["lora_a"], dtype=torch.float32),
        "0.lora_b.weight": torch.tensor(kat["lora_b"], dtype=torch.float32),
        "1.weight": torch.zeros(3, 6),
        "1.bias": torch.zeros(3),
    }
    out = get_merged_lora_ckpt(sd, rank=kat["rank"], alpha=kat["alpha"])
    assert out is sd and out.keys() == {"0.weight", "1.weight", "1.bias"}
    torch.testing.assert_close(out["0.weight"], torch.tensor(kat["expected_merged_weight"]), atol=kat["atol"], rtol=kat["rtol"])
    # the DoRA variant of the same test (test_utils.py:435-447,459-468): the magnitude is folded in and deleted
    sd = {
        "0.weight": 3 * torch.ones(6, 4),
        "0.lora_a.weight": torch.tensor(kat["lora_a"], dtype=torch.float32),
        "0.lora_b.weight": torch.tensor(kat["lora_b"], dtype=torch.float32),
        "0.magnitude": torch.tensor(kat["magnitude"], dtype=torch.float32),
        "1.weight": torch.zeros(3, 6),
        "1.bias": torch.zeros(3),
    }
    out = get_merged_lora_ckpt(sd, rank=kat["rank"], alpha=kat["alpha"])
    assert out is sd and out.keys() == {"0.weight", "1.weight", "1.bias"}
    torch.testing.assert_close(out["0.weight"], torch.tensor(kat["expected_merged_dora_weight"]), atol=kat["atol"], rtol=kat["rtol"])
    with pytest.raises(NotImplementedError):
        get_merged_lora_ckpt({"m.experts.weight": torch.ones(2, 2), "m.experts.lora_a.weight": torch.ones(1, 2),
                              "m.experts.lora_b.weight": torch.ones(2, 1)}, rank=1, alpha=1.0)


def test_disable_adapter_and_adapter_state_dict():
    """tests/torchtune/modules/peft/test_utils.py:214-238,512-522: inside ``disable_adapter`` a LoRA model answers like
    its base model and the flag is restored afterwards (also after an exception); ``get_adapter_state_dict`` keeps the
    ``lora`` / ``magnitude`` entries only."""
    from torch import nn

    from torchtune_amd.modules.peft import DoRALinear, LoRALinear, disable_adapter, get_adapter_state_dict

    torch.manual_seed(0)
    base = nn.Sequential(nn.Linear(2, 6, bias=False), nn.Linear(6, 3))
    lora = nn.Sequential(LoRALinear(2, 6, rank=4, alpha=1.0), nn.Linear(6, 3))
    for p in list(base.parameters()) + list(lora.parameters()):
        nn.init.constant_(p, 1.0)
    x = torch.randn(2, 2)
    assert not torch.allclose(base(x), lora(x))
    with disable_adapter(lora):
        assert lora[0].disabled is True
        out = lora(x)
    assert lora[0].disabled is False
    torch.testing.assert_close(base(x), out)
    with pytest.raises(RuntimeError, match="boom"):
        with disable_adapter(lora):
            raise RuntimeError("boom")
    assert lora[0].disabled is False
    model = nn.Sequential(LoRALinear(8, 8, rank=2, alpha=1.0), DoRALinear(8, 8, rank=2, alpha=1.0), nn.Linear(8, 8))
    sd = get_adapter_state_dict(model.state_dict())
    assert sorted(sd) == ["0.lora_a.weight", "0.lora_b.weight", "1.lora_a.weight", "1.lora_b.weight", "1.magnitude"]
    assert all(v.device.type == "cpu" for v in sd.values())


def test_gemm_workspace_query_is_a_host_function():
    """``ttamd_nf4_gemm_workspace_bytes`` needs no GPU: it is 0 where the launch uses no scratch memory (the few-token
    kernel: M <= 16, and M <= 32 on weights of at most 2^25 elements; launches with more than 128 tiles of 128 x 256 but
    fewer than 256 of 256 x 256 or fewer than 2048 tokens; two-slice launches of a short contraction), slices * M * n_out * 4 bytes with 2 <= slices <= 16 and at least
    four 64-wide k-steps per slice where the contraction is sliced, and 2 * n_out * k bytes (the weight expanded once)
    from 2048 tokens and 256 tiles of 256 x 256 up, which ``ttamd_nf4_gemm_expands_weight`` tells apart."""
    from torchtune_amd import _lib

    lib = _lib.load()
    q = lib.ttamd_nf4_gemm_workspace_bytes
    e = lib.ttamd_nf4_gemm_expands_weight
    assert q(1, 4096, 4096) == 0 and q(16, 14336, 4096) == 0 and q(32, 4096, 4096) == 0
    assert q(33, 4096, 4096) == 16 * 33 * 4096 * 4 and q(64, 4096, 4096) == 16 * 64 * 4096 * 4   # slices from 33 tokens
    assert q(17, 14336, 4096) > 0 and q(17, 4096, 14336) > 0                                     # large weights: from 17
    assert q(8192, 4096, 4096) == 2 * 4096 * 4096 and e(8192, 4096, 4096) == 1
    assert q(16384, 1024, 4096) == 2 * 1024 * 4096 and e(16384, 1024, 4096) == 1
    assert q(8192, 14336, 4096) == q(8192, 4096, 14336) == 2 * 4096 * 14336
    assert q(8192, 1024, 4096) == 0 and e(8192, 1024, 4096) == 0  # 128 tiles of 256 x 256: the fused kernel's 128-row tiles
    assert q(1536, 16384, 4096) == 0 and e(1536, 16384, 4096) == 0  # fewer than 2048 tokens
    assert q(2048, 2048, 2048) == 0  # 128 tiles, two slices of 16 k-steps: not worth the reduction
    assert e(1, 4096, 4096) == 0 and e(128, 4096, 4096) == 0 and e(4096, 1024, 8192) == 0
    assert q(0, 4096, 4096) == 0 and q(128, 0, 4096) == 0
    for M, N, K, slices in [(128, 4096, 4096, 16), (512, 4096, 4096, 4), (1024, 4096, 4096, 2), (65, 256, 512, 2),
                            (300, 512, 1024, 4), (4096, 1024, 8192, 2)]:
        assert q(M, N, K) == slices * M * N * 4, (M, N, K)


def test_group_grad_input_workspace_query_bounds_the_concatenated_contraction():
    """``ttamd_nf4_group_bwd_dx_workspace_bytes`` (a host function; the pointers are only checked for alignment) offers
    the expanded-weight launch for the q / k / v and gate / up groups of the 8B shapes and refuses it (0: the caller
    stays on the per-member fused kernels) once the members' concatenated columns outgrow the launch's 32-bit offsets,
    although every member on its own would fit."""
    from torchtune_amd import _lib

    lib = _lib.load()

    def members(ns):
        arr = (_lib.LoraGroupMember * len(ns))()
        for i, n in enumerate(ns):
            for f in ("quantized_data", "block_scalers", "lora_a", "lora_b", "y"):
                setattr(arr[i], f, 0x1000)
            arr[i].N, arr[i].rank, arr[i].scale = n, 16, 2.0
        return arr

    q = lib.ttamd_nf4_group_bwd_dx_workspace_bytes
    assert q(members([4096, 1024, 1024]), 3, 8192, 4096) == 2 * 4096 * 6144
    assert q(members([14336, 14336]), 2, 8192, 4096) == 2 * 4096 * 28672
    wide = (1 << 20) - 64                       # 2048 rows x this many columns x 2 bytes: just below 2^32 per member
    assert 2048 * wide * 2 < 1 << 32 <= 2048 * 4 * wide * 2
    assert q(members([wide]), 1, 2048, 8192) == 2 * 8192 * wide
    assert q(members([wide] * 4), 4, 2048, 8192) == 0
    assert q(members([1 << 20]), 1, 2048, 8192) == 0   # one member beyond its own bound


def test_built_in_scratch_holds_every_plan_of_the_hidden_product():
    """The partial sums `ttamd_lora_hidden_static_bf16` keeps in its 2 MiB device array never outgrow it: the workspace
    query of the same plan (a host function) over every row count up to 8192 and beyond, long contractions, rank 64."""
    lib = _lib.load()
    limit = lib.ttamd_lora_hidden_static_max_bytes()
    assert limit == 2 << 20
    worst = 0
    for K in (64, 4096, 14336, 64 * 8 * 256, 1 << 20):
        for M in list(range(1, 8193)) + [8193, 12288, 16384, 65536, 1 << 20]:
            worst = max(worst, lib.ttamd_lora_fwd_workspace_bytes(M, K, 64))
    assert 0 < worst <= limit, worst


def test_bench_refuses_more_than_one_gpu():
    """``bench.py --gpus N`` with N > 1 exits with a message before touching any device."""
    import subprocess
    import sys
    from pathlib import Path

    root = Path(__file__).resolve().parents[1]
    proc = subprocess.run([sys.executable, str(root / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stdout + proc.stderr)


def test_to_nf4_preconditions_are_the_reference_asserts():
    """The four asserts of ``NF4Tensor.from_tensor`` fire before anything touches a device: at most two dimensions,
    numel divisible by the block size, contiguous, number of blocks divisible by the scaler block size."""
    from torchtune_amd import to_nf4

    with pytest.raises(AssertionError, match="dim <= 2"):
        to_nf4(torch.zeros(2, 64, 256, dtype=torch.bfloat16))
    with pytest.raises(AssertionError, match="divisible by block size"):
        to_nf4(torch.zeros(100, 3, dtype=torch.bfloat16))
    with pytest.raises(AssertionError, match="contiguous"):
        to_nf4(torch.zeros(512, 512, dtype=torch.bfloat16).t())
    with pytest.raises(AssertionError, match="divisible by scaler_block_size"):
        to_nf4(torch.zeros(64, 64, dtype=torch.bfloat16))  # 64 blocks, scaler blocks of 256


def test_tiled_entry_points_validate_their_arguments_on_the_host():
    """``ttamd_tiled_linear_bf16`` / ``ttamd_fq_per_group_int4_sym_tiled_bf16`` refuse bad arguments before any launch
    (no GPU needed): null or misaligned pointers, dimensions that are not multiples of 64, group sizes the kernel does
    not serve (``TTAMD_EUNSUPPORTED``), a non-positive eps."""
    import ctypes

    from torchtune_amd import _lib

    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 15) & ~15
    assert lib.ttamd_tiled_weight_bytes(128, 256) == 2 * 128 * 256 and lib.ttamd_tiled_weight_bytes(0, 256) == 0
    EINVAL, EUNSUPPORTED = -1, -2
    codes = {lib.ttamd_tiled_linear_bf16(None, p, None, p, 64, 64, 64, None),
             lib.ttamd_tiled_linear_bf16(p, p, None, p + 2, 64, 64, 64, None),
             lib.ttamd_tiled_linear_bf16(p, p, None, p, 64, 96, 64, None),
             lib.ttamd_tiled_linear_bf16(p, p, None, p, 64, 64, 32, None),
             lib.ttamd_tiled_linear_bf16(p, p, None, p, 0, 64, 64, None)}
    assert codes == {EINVAL}, codes
    assert b"tiled_linear" in lib.ttamd_last_error()
    F32 = 1  # TTAMD_F32
    q = lib.ttamd_fq_per_group_int4_sym_tiled_bf16
    assert q(None, 64, 64, 32, F32, 1e-7, p, None, None, None) == EINVAL
    assert q(p, 64, 64, 32, F32, 1e-7, None, None, None, None) == EINVAL          # no output at all
    assert q(p, 64, 96, 32, F32, 1e-7, p, None, None, None) == EINVAL             # K not a multiple of 64
    assert q(p, 64, 64, 32, F32, 0.0, p, None, None, None) == EINVAL              # eps
    assert q(p, 64, 64, 32, 7, 1e-7, p, None, None, None) == EINVAL               # qparam dtype code
    assert q(p, 64, 64, 16, F32, 1e-7, p, None, None, None) == EUNSUPPORTED       # group size
    assert q(p, 64, 192, 128, F32, 1e-7, p, None, None, None) == EUNSUPPORTED     # group does not divide K
    assert b"group size" in lib.ttamd_last_error()


def test_gated_group_entry_point_validates_its_arguments_on_the_host():
    """``ttamd_nf4_lora_group_swiglu_fwd_bf16`` takes exactly the gate and the up projection, of equal width, and a
    non-null aligned output for the gated product; refused before any launch."""
    import ctypes

    from torchtune_amd import _lib

    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    arr = (_lib.LoraGroupMember * 2)()
    for e, n in zip(arr, (128, 64)):
        e.N, e.rank, e.scale = n, 8, 1.0
    f = lib.ttamd_nf4_lora_group_swiglu_fwd_bf16
    assert f(p, arr, 2, p, p, 8, 64, None, 0, None) == -1 and b"equal width" in lib.ttamd_last_error()
    assert f(p, arr, 1, p, p, 8, 64, None, 0, None) == -1
    arr[1].N = 128
    assert f(p, arr, 2, p, None, 8, 64, None, 0, None) == -1 and b"act" in lib.ttamd_last_error()



def test_grad_input_swiglu_entry_point_validates_its_arguments_on_the_host():
    """``ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16`` wants gate, up and both gradients (non-null, 16-byte aligned) on top of
    what the plain grad-input entry point checks; refused before any launch."""
    import ctypes

    from torchtune_amd import _lib

    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = (ctypes.addressof(buf) + 15) & ~15
    f = lib.ttamd_nf4_linear_bwd_dx_swiglu_ws_bf16
    #        gy codes scal codes_t scal_t gh   lora_a rank gate up ggate gup  M  N   K   ws  bytes stream
    assert f(p, p, p, None, None, None, None, 0, None, p, p, p, 8, 64, 64, None, 0, None) == -1 and b"null" in lib.ttamd_last_error()
    assert f(p, p, p, None, None, None, None, 0, p, p, p, None, 8, 64, 64, None, 0, None) == -1
    assert f(p, p, p, None, None, None, None, 0, p, p + 2, p, p, 8, 64, 64, None, 0, None) == -1 and b"aligned" in lib.ttamd_last_error()
    assert f(p, p, p, None, None, None, None, 0, p, p, p, p, 8, 64, 96, None, 0, None) == -1      # K not a multiple of 64
    assert f(p, p, p, p, None, None, None, 0, p, p, p, p, 8, 64, 64, None, 0, None) == -1 and b"together" in lib.ttamd_last_error()
