"""Host-side behaviour that must hold before any kernel is launched (all on the CPU): quantizer ``prepare`` keeps the
model's parameters as they are, shape mismatches raise instead of reaching a kernel, the fake quantizer works under
``inference_mode``, and the reference's call of ``get_merged_lora_ckpt`` binds."""
import gc

import pytest
import torch
from torch import nn

from oracle import nf4_oracle
from torchtune_amd import nf4_tensor, ops, qat
from torchtune_amd.modules.peft import LoRALinear, get_merged_lora_ckpt
from torchtune_amd.modules.peft import dora as dora_mod
from torchtune_amd.modules.peft import lora as lora_mod
from torchtune_amd.nf4_tensor import NF4Tensor, linear_nf4
from torchtune_amd.qat import FakeQuantizeConfig, FakeQuantizer, Int4WeightOnlyQATQuantizer, Int8DynActInt4WeightQATQuantizer


def _cpu_nf4(shape=(256, 128)) -> NF4Tensor:
    p = nf4_oracle.nf4_quantize((torch.randn(shape, generator=torch.Generator().manual_seed(0)) * 0.02).to(torch.bfloat16), 64, 256)
    return NF4Tensor(p.shape, p.dtype, p.block_size, p.n_blocks, p.scaler_block_size, p.quantized_scalers,
                     p.quantization_factor, p.scaler_mean, p.quantized_data, p.nf4)


@pytest.mark.parametrize("quantizer", [Int8DynActInt4WeightQATQuantizer(groupsize=32), Int4WeightOnlyQATQuantizer(groupsize=32)])
def test_prepare_with_default_precision_keeps_dtype_and_parameter_objects(quantizer):
    """The reference's QAT configs give the quantizer a group size only (recipes/configs/llama3/8B_qat_full.yaml:62-64)
    on a bf16 model: the swap must hand the new module the very Parameter it found, not a float32 copy."""
    model = nn.Sequential(nn.Linear(128, 256, bias=False), nn.Sequential(nn.Linear(256, 128, bias=False))).to(torch.bfloat16)
    before = [model[0].weight, model[1][0].weight]
    model[0].weight.requires_grad_(False)
    model = quantizer.prepare(model)
    after = [model[0].weight, model[1][0].weight]
    assert isinstance(model[0], qat.FakeQuantizedLinear) and isinstance(model[1][0], qat.FakeQuantizedLinear)
    for b, a in zip(before, after):
        assert a is b and a.dtype == torch.bfloat16 and a.device.type == "cpu"
    assert not model[0].weight.requires_grad and model[1][0].weight.requires_grad
    assert len(list(model.parameters())) == 2
    # disabled fake quant = the plain linear in the model's dtype (no kernel involved)
    model.apply(lambda m: m.disable_fake_quant() if hasattr(m, "disable_fake_quant") else None)
    x = torch.randn(3, 128).to(torch.bfloat16)
    assert model(x).dtype == torch.bfloat16


def test_prepare_keeps_bias_parameter():
    model = nn.Sequential(nn.Linear(64, 32, bias=True)).to(torch.bfloat16)
    bias = model[0].bias
    Int8DynActInt4WeightQATQuantizer(groupsize=32).prepare(model)
    assert model[0].bias is bias and model[0].bias.dtype == torch.bfloat16


def test_wrong_inner_dimension_raises_before_any_kernel(monkeypatch):
    """F.linear's shape error, raised on the host: the kernels would otherwise take K from the activation and read the
    packed weight out of bounds."""
    w = _cpu_nf4((256, 128))

    def boom(*a, **k):
        raise AssertionError("a kernel wrapper was reached")

    for name in ("lora_hidden", "nf4_lora_linear_fwd", "nf4_dora_weight_norm"):
        monkeypatch.setattr(ops, name, boom)
    for bad in (torch.randn(4, 192), torch.randn(2, 3, 64), torch.randn(4, 256)):
        with pytest.raises(RuntimeError, match="shapes cannot be multiplied"):
            linear_nf4(bad.to(torch.bfloat16), w)
        with pytest.raises(RuntimeError, match="shapes cannot be multiplied"):
            lora_mod._QLoRALinearFn.apply(bad.to(torch.bfloat16), w, torch.zeros(8, 128), torch.zeros(256, 8), None, 2.0)
        with pytest.raises(RuntimeError, match="shapes cannot be multiplied"):
            dora_mod._QDoRALinearFn.apply(bad.to(torch.bfloat16), w, torch.zeros(8, 128), torch.zeros(256, 8), torch.ones(256), None, 2.0)


def test_ops_wrappers_check_operand_sizes(monkeypatch):
    """The C side sees pointers only, so the tensor-level wrappers compare every operand with [N, K] first."""
    monkeypatch.setattr(ops, "_need_gpu", lambda t, what: None)

    class NoLib:
        def __getattr__(self, name):
            raise AssertionError(f"{name} was called")

    monkeypatch.setattr(ops._lib, "load", lambda: NoLib())
    N, K, M, r = 256, 128, 16, 8
    bf = torch.bfloat16
    x = torch.zeros(M, K, dtype=bf)
    qd = torch.zeros(N * K // 2, dtype=torch.uint8)
    bs = torch.zeros(N * K // 64)
    h, B, A = torch.zeros(M, r, dtype=bf), torch.zeros(N, r, dtype=bf), torch.zeros(r, K, dtype=bf)
    gy = torch.zeros(M, N, dtype=bf)
    cases = [
        lambda: ops.nf4_lora_linear_fwd(torch.zeros(M, K + 64, dtype=bf), qd, bs, N),                 # K taken from x
        lambda: ops.nf4_lora_linear_fwd(x, qd[:-64], bs, N),                                          # short codes
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs[:-1], N),                                           # short scalers
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs, N, block_scalers_t=bs[:-1]),
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs, N, h[:-1], B, 2.0),                                # h rows
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs, N, h, B[:-1], 2.0),                                # lora_b rows
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs, N, h, torch.zeros(N, 2 * r, dtype=bf), 2.0),      # rank mismatch
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs, N, bias=torch.zeros(N - 1, dtype=bf)),
        lambda: ops.nf4_lora_linear_fwd(x, qd, bs, N, col_scale=torch.zeros(N + 1, dtype=bf)),
        lambda: ops.nf4_linear_bwd_dx(gy, qd, bs, K + 64),
        lambda: ops.nf4_linear_bwd_dx(gy, qd, bs, K, h, A[:, :-8]),
        lambda: ops.nf4_linear_bwd_dx(gy, qd, bs, K, transposed=(qd[:-2], bs)),
        lambda: ops.lora_hidden(x, torch.zeros(r, K + 8, dtype=bf)),
        lambda: ops.lora_bwd(gy, x[:-1], h, B, 2.0),
        lambda: ops.lora_bwd(gy, x, h, B[:-1], 2.0),
        lambda: ops.nf4_transpose_for_backward(qd, bs, N, K + 64),
    ]
    for i, case in enumerate(cases):
        with pytest.raises(ValueError):
            case()


def test_fake_quantizer_under_inference_mode_and_cache_lifetime(monkeypatch):
    """Inference tensors have no version counter: the sibling-sharing cache must step aside instead of raising, and it
    must not keep an activation alive once the caller has dropped it."""
    calls = []

    def fake_kernel(x, want_qparams=True, qparam_dtype=torch.float32, eps=None):
        calls.append(x.shape)
        return x.clone(), torch.ones(x.shape[0]), torch.zeros(x.shape[0], dtype=torch.int32)

    monkeypatch.setattr(ops, "fq_per_token_int8_asym", fake_kernel)
    fq = FakeQuantizer(FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False))
    fq2 = FakeQuantizer(FakeQuantizeConfig(torch.int8, "per_token", is_symmetric=False))
    with torch.inference_mode():
        x = torch.randn(4, 64)
        assert x.is_inference()
        fq(x)
        fq2(x)
    assert len(calls) == 2  # nothing shared, nothing raised
    y = torch.randn(4, 64)  # created outside, used inside: still no sharing under inference_mode
    with torch.inference_mode():
        fq(y)
    assert len(calls) == 3
    # ordinary mode: the second quantizer reuses the first one's result for the same tensor object ...
    z = torch.randn(4, 64)
    fq(z)
    fq2(z)
    assert len(calls) == 4
    z.add_(1.0)  # ... but not after an in-place write
    fq2(z)
    assert len(calls) == 5
    # ... and the entry lets go of the activation when the caller does
    entry = FakeQuantizer._last.entry
    assert entry is not None and entry[0]() is z
    del z
    gc.collect()
    assert getattr(FakeQuantizer._last, "entry", None) is None


def test_nf4_cache_is_invalidated_through_aliases():
    """A write through an alias (``param.data.copy_``) gives the alias inner tensor objects of its own: the derived-data
    caches of the original must still go stale.  Checked on the key the caches use."""
    t = _cpu_nf4((256, 128))
    p = nn.Parameter(t, requires_grad=False)
    g0 = nf4_tensor._generation(p.quantized_scalers)
    alias = p.data
    assert alias.quantized_scalers is not p.quantized_scalers
    assert alias.quantized_scalers.untyped_storage().data_ptr() == p.quantized_scalers.untyped_storage().data_ptr()
    alias.copy_(_cpu_nf4((256, 128)))  # same-layout NF4 copy: no arithmetic, runs on the CPU
    assert nf4_tensor._generation(p.quantized_scalers) == g0 + 1
    assert nf4_tensor._generation(alias.quantized_scalers) == g0 + 1
    p.detach().copy_(_cpu_nf4((256, 128)))
    assert nf4_tensor._generation(p.quantized_scalers) == g0 + 2


def test_get_merged_lora_ckpt_binds_like_the_reference_call():
    """torchtune/training/checkpointing/_checkpoint_client.py:177-182 passes ``use_distributed_barriers`` by keyword."""
    sd = {"m.weight": torch.ones(4, 4), "m.lora_a.weight": torch.ones(2, 4), "m.lora_b.weight": torch.ones(4, 2)}
    out = get_merged_lora_ckpt(sd, rank=2, alpha=4.0, use_distributed_barriers=True)
    torch.testing.assert_close(out["m.weight"], torch.full((4, 4), 1.0 + 2.0 * 2.0))
    sd = {"m.weight": torch.ones(4, 4), "m.lora_a.weight": torch.ones(2, 4), "m.lora_b.weight": torch.ones(4, 2)}
    get_merged_lora_ckpt(sd, 2, 4.0, False)  # positional fourth argument is the barrier flag, not an offload switch
    assert not sd["m.weight"].is_cuda
    with pytest.raises(TypeError):
        get_merged_lora_ckpt(sd, 2, 4.0, False, True)  # offload_to_cpu is keyword-only


def test_low_ram_state_dict_hook_puts_every_entry_in_one_shared_mapping(monkeypatch):
    """The switch and the contract of torchtune/modules/common_utils.py:136-237 on a model without NF4 entries (those
    need the GPU): values and dtypes unchanged, every tensor a CPU tensor over the same file-backed storage, no file
    left behind, and the ordinary hook when the switch is off."""
    import glob
    import tempfile

    from torchtune_amd.modules import common_utils

    model = nn.Sequential(nn.Linear(8, 4), nn.Linear(4, 2, bias=False).to(torch.bfloat16))
    want = {k: v.detach().clone() for k, v in model.state_dict().items()}
    monkeypatch.setattr(common_utils, "_use_low_cpu_ram", True)
    common_utils._register_reparametrize_state_dict_hooks(model, dtype=torch.bfloat16, offload_to_cpu=True)
    sd = model.state_dict()
    assert list(sd) == list(want)
    storages = set()
    for k, v in sd.items():
        assert v.device.type == "cpu" and v.dtype == want[k].dtype and torch.equal(v, want[k])
        storages.add(v.untyped_storage().data_ptr())
    assert len(storages) == 1  # one mapping
    assert not glob.glob(tempfile.gettempdir() + "/torchtune_amd_state_dict_*")
    # the entries are copies: writing to the model does not change the checkpoint
    with torch.no_grad():
        model[0].weight.add_(1.0)
    assert torch.equal(sd["0.weight"], want["0.weight"])
    monkeypatch.setattr(common_utils, "_use_low_cpu_ram", False)
    plain = nn.Linear(8, 4)
    common_utils._register_reparametrize_state_dict_hooks(plain)
    assert plain.state_dict()["weight"].data_ptr() == plain.weight.data_ptr()  # the ordinary hook leaves dense entries alone
