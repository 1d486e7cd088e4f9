"""Opt-in binding at the seam the reference actually imports through.

torchtune takes every name of the quantized-linear path from the third-party ``torchao`` package:

    from torchao.quantization import to_nf4, NF4Tensor                       torchtune/modules/peft/lora.py:15,
                                                                             modules/low_precision/nf4_linear.py:12,
                                                                             modules/common_utils.py:19,
                                                                             training/_distributed.py:39,
                                                                             training/_activation_offloading.py:16
    from torchao.quantization.quantize_.workflows.nf4.nf4_tensor import linear_nf4, implements
                                                                             modules/peft/lora.py:16, nf4_linear.py:13,
                                                                             low_precision/_register_nf4_dispatch_ops.py:9
    from torchao.quantization.qat.api import FakeQuantizeConfig              modules/peft/lora.py:222
    from torchao.quantization.qat.fake_quantizer import FakeQuantizer        modules/peft/lora.py:223
    from torchao.quantization import Int4WeightOnlyConfig, Int8DynamicActivationIntxWeightConfig, quantize_
    from torchao.quantization.quantize_.workflows import Int4PackingFormat
    from torchao.quantization.qat import Int4WeightOnlyQATQuantizer, Int8DynActInt4WeightQATQuantizer
    from torchao.quantization.granularity import PerGroup                    training/quantization.py:20-30

``install()`` registers modules under exactly those dotted names in ``sys.modules`` whose attributes are this package's
HIP-backed implementations, so an unmodified torchtune checkout (its recipes, builders and module classes) imports and
runs on them.  Nothing is installed unless ``install()`` is called, and it refuses to shadow a real ``torchao``.

Names torchtune imports from ``torchao`` for features outside this path (float8 training: ``torchao.float8``) are present
so that ``import torchtune`` succeeds, and raise ``NotImplementedError`` when used.
"""
from __future__ import annotations

import enum
import sys
import types
from typing import Dict, Optional

import torch
from torch import nn

from . import nf4_tensor, qat

__all__ = ["install", "uninstall", "is_installed", "ALIASED_MODULES"]

_MARK = "__torchtune_amd_alias__"
# torchtune/training/_activation_offloading.py:188 compares ``torchao.__version__ < "0.6.0.dev20240917"`` as STRINGS, so the
# alias reports a version whose text sorts after that one (a two-digit minor version would sort before it)
VERSION = "0.9.0+torchtune_amd"


class Int4PackingFormat(str, enum.Enum):
    """Packing formats of the weight-only int4 configuration (``training/quantization.py:25,117``).  Only the names
    matter here: the converted linear of this package keeps one plain packing (two codes per byte)."""

    PLAIN = "plain"
    PRESHUFFLED = "preshuffled"
    MARLIN_SPARSE = "marlin_sparse"
    OPAQUE = "opaque"
    PLAIN_INT32 = "plain_int32"
    TILE_PACKED_TO_4D = "tile_packed_to_4d"


class Int8DynamicActivationIntxWeightConfig:
    """``Int8DynamicActivationIntxWeightConfig(weight_dtype=torch.int4, weight_granularity=PerGroup(g))``
    (``training/quantization.py:88-90``): int8 per-token dynamic activations, int4 per-group symmetric weights."""

    def __init__(self, weight_dtype: torch.dtype = torch.int8, weight_granularity=None, **kwargs):
        if weight_dtype != torch.int4:
            raise NotImplementedError(f"only weight_dtype=torch.int4 has kernels, got {weight_dtype}")
        if not isinstance(weight_granularity, qat.PerGroup):
            raise NotImplementedError("weight_granularity must be PerGroup(group_size)")
        if kwargs:
            raise NotImplementedError(f"unsupported arguments: {sorted(kwargs)}")
        self.weight_dtype = weight_dtype
        self.weight_granularity = weight_granularity


class Int4WeightOnlyConfig:
    """``Int4WeightOnlyConfig(group_size=g, int4_packing_format=...)`` (``training/quantization.py:114-119``)."""

    def __init__(self, group_size: int = 128, int4_packing_format=Int4PackingFormat.PLAIN, **kwargs):
        if kwargs:
            raise NotImplementedError(f"unsupported arguments: {sorted(kwargs)}")
        self.group_size = group_size
        self.int4_packing_format = int4_packing_format


def quantize_(model: nn.Module, config, *args, **kwargs) -> None:
    """``quantize_(model, config)``: post-training quantisation in place (``training/quantization.py:90,120``)."""
    if isinstance(config, Int8DynamicActivationIntxWeightConfig):
        qat.quantize_linears_8da4w(model, config.weight_granularity.group_size)
    elif isinstance(config, Int4WeightOnlyConfig):
        qat.quantize_linears_4w(model, config.group_size, 8)
    else:
        raise NotImplementedError(f"quantize_: no kernel for {type(config).__name__}")


def _float8_unavailable(name: str):
    def raiser(*args, **kwargs):
        raise NotImplementedError(f"torchao.float8.{name}: float8 training is not part of torchtune_amd")

    raiser.__name__ = name
    return raiser


class _Float8Placeholder:
    """Stands where torchtune expects a float8 class; any use raises."""

    def __init__(self, *args, **kwargs):
        raise NotImplementedError(f"torchao.float8.{type(self).__name__}: float8 training is not part of torchtune_amd")


def _module_table() -> Dict[str, dict]:
    nf4_names = {
        "NF4Tensor": nf4_tensor.NF4Tensor,
        "to_nf4": nf4_tensor.to_nf4,
        "linear_nf4": nf4_tensor.linear_nf4,
        "implements": nf4_tensor.implements,
    }
    qat_names = {
        "Int4WeightOnlyQATQuantizer": qat.Int4WeightOnlyQATQuantizer,
        "Int8DynActInt4WeightQATQuantizer": qat.Int8DynActInt4WeightQATQuantizer,
        "FakeQuantizeConfig": qat.FakeQuantizeConfig,
        "FakeQuantizer": qat.FakeQuantizer,
        "FakeQuantizedLinear": qat.FakeQuantizedLinear,
    }
    float8 = {
        "convert_to_float8_training": _float8_unavailable("convert_to_float8_training"),
        "precompute_float8_dynamic_scale_for_fsdp": _float8_unavailable("precompute_float8_dynamic_scale_for_fsdp"),
        "Float8LinearConfig": type("Float8LinearConfig", (_Float8Placeholder,), {}),
    }
    float8_tp = {
        name: type(name, (_Float8Placeholder,), {})
        for name in ("Float8ColwiseParallel", "Float8RowwiseParallel", "PrepareFloat8ModuleInput")
    }
    return {
        "torchao": {"__version__": VERSION},
        "torchao.quantization": {
            "NF4Tensor": nf4_tensor.NF4Tensor,
            "to_nf4": nf4_tensor.to_nf4,
            "quantize_": quantize_,  # the function wins the attribute; the package of the same name is in sys.modules
            "Int4WeightOnlyConfig": Int4WeightOnlyConfig,
            "Int8DynamicActivationIntxWeightConfig": Int8DynamicActivationIntxWeightConfig,
        },
        "torchao.quantization.quantize_": {},
        "torchao.quantization.quantize_.workflows": {"Int4PackingFormat": Int4PackingFormat},
        "torchao.quantization.quantize_.workflows.nf4": {},
        "torchao.quantization.quantize_.workflows.nf4.nf4_tensor": nf4_names,
        "torchao.quantization.granularity": {"PerGroup": qat.PerGroup, "PerToken": qat.PerToken},
        "torchao.quantization.qat": qat_names,
        "torchao.quantization.qat.api": {"FakeQuantizeConfig": qat.FakeQuantizeConfig},
        "torchao.quantization.qat.fake_quantizer": {"FakeQuantizer": qat.FakeQuantizer},
        "torchao.quantization.qat.linear": {
            "FakeQuantizedLinear": qat.FakeQuantizedLinear,
            "Int8DynActInt4WeightQATLinear": qat.Int8DynActInt4WeightQATLinear,
            "Int4WeightOnlyQATLinear": qat.Int4WeightOnlyQATLinear,
        },
        "torchao.float8": float8,
        "torchao.float8.float8_tensor_parallel": float8_tp,
    }


ALIASED_MODULES = tuple(_module_table())


def is_installed() -> bool:
    mod = sys.modules.get("torchao")
    return mod is not None and getattr(mod, _MARK, False)


def install(force: bool = False) -> None:
    """Make the ``torchao`` names torchtune imports resolve to this package.  Idempotent.

    Raises ``RuntimeError`` if a real ``torchao`` is already imported or importable (its arithmetic and this package's
    would be mixed behind one name); ``force=True`` shadows it anyway."""
    if is_installed():
        return
    if not force:
        if "torchao" in sys.modules:
            raise RuntimeError("torchtune_amd.compat.install(): a real `torchao` is already imported; not shadowing it")
        import importlib.util

        if importlib.util.find_spec("torchao") is not None:
            raise RuntimeError("torchtune_amd.compat.install(): a real `torchao` is installed; pass force=True to shadow it")
    table = _module_table()
    created: Dict[str, types.ModuleType] = {}
    for name, attrs in table.items():
        mod = types.ModuleType(name, f"torchtune_amd alias of {name}")
        setattr(mod, _MARK, True)
        mod.__path__ = []  # every alias may have sub-modules
        mod.__package__ = name
        for key, value in attrs.items():
            setattr(mod, key, value)
        created[name] = mod
    # parents expose their children as attributes, except where a function of the same name must win (`quantize_`)
    for name, mod in created.items():
        parent, _, child = name.rpartition(".")
        if parent and not hasattr(created[parent], child):
            setattr(created[parent], child, mod)
    sys.modules.update(created)


def uninstall() -> None:
    """Remove the aliases ``install()`` registered (modules that already imported names from them keep those names)."""
    for name in list(sys.modules):
        if (name == "torchao" or name.startswith("torchao.")) and getattr(sys.modules[name], _MARK, False):
            del sys.modules[name]
