"""Quantizer names and fake-quant toggles under the dotpaths the reference's recipes and YAML configs use
(``torchtune/training/quantization.py:26-29,56-71,94-97,125-127,167-244``), bound to the HIP-backed implementations."""
from __future__ import annotations

from typing import Callable, Optional

from torch import nn

from ..modules.peft.lora import LoRALinear, QATLoRALinear
from ..qat import (
    FakeQuantizeConfig,
    FakeQuantizedLinear,
    Int4WeightOnlyQATQuantizer,
    Int8DynActInt4WeightQATQuantizer,
)

__all__ = [
    "get_quantizer_mode",
    "Int4WeightOnlyQATQuantizer",
    "Int8DynActInt4WeightQATQuantizer",
    "swap_lora_linear_with_qat",
]

_quantizer_to_mode = {Int8DynActInt4WeightQATQuantizer: "8da4w-qat", Int4WeightOnlyQATQuantizer: "4w-qat"}


def _enable_linear_fake_quant(mod: nn.Module, enabled: bool = True) -> None:
    """Switch both fake quantizers of a ``FakeQuantizedLinear`` on or off (use with ``model.apply``)."""
    if isinstance(mod, FakeQuantizedLinear):
        for fq in (mod.activation_fake_quantizer, mod.weight_fake_quantizer):
            if fq is not None:
                fq.enabled = enabled


def _disable_linear_fake_quant(mod: nn.Module) -> None:
    _enable_linear_fake_quant(mod, enabled=False)


_quantizer_mode_to_disable_fake_quant = {"8da4w-qat": _disable_linear_fake_quant, "4w-qat": _disable_linear_fake_quant}
_quantizer_mode_to_enable_fake_quant = {"8da4w-qat": _enable_linear_fake_quant, "4w-qat": _enable_linear_fake_quant}


def get_quantizer_mode(quantizer: Optional[Callable]) -> Optional[str]:
    """"8da4w-qat" for :class:`Int8DynActInt4WeightQATQuantizer`, "4w-qat" for :class:`Int4WeightOnlyQATQuantizer`,
    None for anything unknown."""
    return _quantizer_to_mode.get(type(quantizer), None)


def _get_disable_fake_quant(quantizer_mode: str) -> Optional[Callable]:
    return _quantizer_mode_to_disable_fake_quant.get(quantizer_mode, None)


def _get_enable_fake_quant(quantizer_mode: str) -> Optional[Callable]:
    return _quantizer_mode_to_enable_fake_quant.get(quantizer_mode, None)


def swap_lora_linear_with_qat(
    module: nn.Module,
    activation_qat_config: Optional[FakeQuantizeConfig] = None,
    weight_qat_config: Optional[FakeQuantizeConfig] = None,
) -> None:
    """Replace every ``LoRALinear`` under ``module`` by a ``QATLoRALinear`` sharing its weights."""
    for name, child in module.named_children():
        if isinstance(child, LoRALinear):
            setattr(module, name, QATLoRALinear.from_lora_linear(child, activation_qat_config, weight_qat_config))
        else:
            swap_lora_linear_with_qat(child, activation_qat_config, weight_qat_config)
