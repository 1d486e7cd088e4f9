"""``torchtune_amd.compat.install()``: the dotted ``torchao`` names the reference imports resolve to this package.

The import statements below are the ones the reference's hot-path modules execute (file:line given beside each); the
reference itself is neither imported nor needed."""
import sys
import types

import pytest

import torchtune_amd
from torchtune_amd import compat, nf4_tensor, qat

REFERENCE_IMPORTS = [
    # torchtune/modules/peft/lora.py:15-16, modules/peft/dora.py:15-16, modules/low_precision/nf4_linear.py:12-13
    "from torchao.quantization import to_nf4",
    "from torchao.quantization.quantize_.workflows.nf4.nf4_tensor import linear_nf4",
    # torchtune/modules/common_utils.py:19, training/_distributed.py:39, training/_activation_offloading.py:13,16
    "from torchao.quantization import NF4Tensor",
    "from torchao.quantization import NF4Tensor, to_nf4",
    "import torchao",
    # torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:8-9
    "from torchao.quantization.quantize_.workflows.nf4.nf4_tensor import implements as nf4_tensor_impl",
    # torchtune/modules/peft/lora.py:222-223
    "from torchao.quantization.qat.api import FakeQuantizeConfig",
    "from torchao.quantization.qat.fake_quantizer import FakeQuantizer",
    # torchtune/training/quantization.py:12-30,47
    "from torchao.float8 import convert_to_float8_training as _convert_to_float8_training_torchao, Float8LinearConfig",
    "from torchao.float8.float8_tensor_parallel import Float8ColwiseParallel, Float8RowwiseParallel",
    "from torchao.quantization import Int4WeightOnlyConfig, Int8DynamicActivationIntxWeightConfig, quantize_",
    "from torchao.quantization.quantize_.workflows import Int4PackingFormat",
    "from torchao.quantization.qat import Int4WeightOnlyQATQuantizer, Int8DynActInt4WeightQATQuantizer",
    "from torchao.quantization.granularity import PerGroup",
    "from torchao.quantization import qat",
    # recipes/full_finetune_distributed.py:23, torchtune/models/llama3/_parallelism.py:18
    "from torchao.float8 import precompute_float8_dynamic_scale_for_fsdp",
    "from torchao.float8.float8_tensor_parallel import PrepareFloat8ModuleInput",
]


@pytest.fixture
def installed():
    if "torchao" in sys.modules and not compat.is_installed():
        pytest.skip("a real torchao is imported in this process")
    compat.install()
    yield
    compat.uninstall()


@pytest.mark.parametrize("stmt", REFERENCE_IMPORTS)
def test_reference_import_lines_resolve(installed, stmt):
    ns = {}
    exec(stmt, ns)
    assert len(ns) > 1


def test_names_are_this_packages_implementations(installed):
    ns = {}
    for stmt in REFERENCE_IMPORTS:
        exec(stmt, ns)
    assert ns["to_nf4"] is nf4_tensor.to_nf4 is torchtune_amd.to_nf4
    assert ns["NF4Tensor"] is nf4_tensor.NF4Tensor
    assert ns["linear_nf4"] is nf4_tensor.linear_nf4 and ns["nf4_tensor_impl"] is nf4_tensor.implements
    assert ns["FakeQuantizeConfig"] is qat.FakeQuantizeConfig and ns["FakeQuantizer"] is qat.FakeQuantizer
    assert ns["Int8DynActInt4WeightQATQuantizer"] is qat.Int8DynActInt4WeightQATQuantizer
    assert ns["Int4WeightOnlyQATQuantizer"] is qat.Int4WeightOnlyQATQuantizer
    assert ns["PerGroup"] is qat.PerGroup
    # `quantize_` is a function on the package and a package in sys.modules, as in torchao
    assert callable(ns["quantize_"]) and isinstance(sys.modules["torchao.quantization.quantize_"], types.ModuleType)
    assert ns["Int4PackingFormat"].TILE_PACKED_TO_4D.value == "tile_packed_to_4d"
    # the version check of torchtune/training/_activation_offloading.py:188 (a string comparison) passes
    assert not (ns["torchao"].__version__ < "0.6.0.dev20240917")
    # float8 names exist and refuse to be used
    with pytest.raises(NotImplementedError):
        ns["_convert_to_float8_training_torchao"](None)
    with pytest.raises(NotImplementedError):
        ns["Float8LinearConfig"]()


def test_post_training_configs_dispatch_to_the_converters(installed, monkeypatch):
    import torch
    from torch import nn

    from torchao.quantization import Int4WeightOnlyConfig, Int8DynamicActivationIntxWeightConfig, quantize_
    from torchao.quantization.granularity import PerGroup
    from torchao.quantization.quantize_.workflows import Int4PackingFormat

    calls = []
    monkeypatch.setattr(qat, "quantize_linears_8da4w", lambda m, g: calls.append(("8da4w", g)))
    monkeypatch.setattr(qat, "quantize_linears_4w", lambda m, g, t: calls.append(("4w", g, t)))
    model = nn.Sequential(nn.Linear(64, 64))
    # the two calls of torchtune/training/quantization.py:88-90 and :114-120
    quantize_(model, Int8DynamicActivationIntxWeightConfig(weight_dtype=torch.int4, weight_granularity=PerGroup(32)))
    quantize_(model, Int4WeightOnlyConfig(group_size=128, int4_packing_format=Int4PackingFormat.TILE_PACKED_TO_4D))
    assert calls == [("8da4w", 32), ("4w", 128, 8)]
    with pytest.raises(NotImplementedError):
        Int8DynamicActivationIntxWeightConfig(weight_dtype=torch.int8, weight_granularity=PerGroup(32))


def test_install_is_idempotent_and_reversible_and_never_shadows_a_real_torchao():
    if "torchao" in sys.modules and not compat.is_installed():
        pytest.skip("a real torchao is imported in this process")
    compat.install()
    first = sys.modules["torchao"]
    compat.install()
    assert sys.modules["torchao"] is first and compat.is_installed()
    assert set(compat.ALIASED_MODULES) <= set(sys.modules)
    compat.uninstall()
    assert not compat.is_installed() and not any(n == "torchao" or n.startswith("torchao.") for n in sys.modules)
    sys.modules["torchao"] = types.ModuleType("torchao")  # stands for a real installation
    try:
        with pytest.raises(RuntimeError, match="not shadowing"):
            compat.install()
    finally:
        del sys.modules["torchao"]
