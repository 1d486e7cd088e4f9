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
    quantize_linears_4w,
    quantize_linears_8da4w,
)

__all__ = [
    "get_quantizer_mode",
    "Int4WeightOnlyQuantizer",
    "Int4WeightOnlyQATQuantizer",
    "Int4WeightOnlyQATQuantizerModuleSwap",
    "Int8DynActInt4WeightQuantizer",
    "Int8DynActInt4WeightQATQuantizer",
    "Int8DynActInt4WeightQATQuantizerModuleSwap",
    "swap_lora_linear_with_qat",
]


class Int8DynActInt4WeightQuantizer:
    """Post-training counterpart of the 8da4w scheme (``torchtune/training/quantization.py:79-91``, mode "8da4w"):
    ``quantize(model)`` replaces every linear by the converted int4 linear, with the arithmetic ``convert`` uses."""

    def __init__(self, groupsize: int = 256):
        self.groupsize = groupsize

    def quantize(self, model: nn.Module) -> nn.Module:
        return quantize_linears_8da4w(model, self.groupsize)


class Int4WeightOnlyQuantizer:
    """Post-training weight-only int4 (``torchtune/training/quantization.py:105-121``, mode "4w")."""

    def __init__(self, groupsize: int = 128, inner_k_tiles: int = 8):
        self.groupsize = groupsize
        self.inner_k_tiles = inner_k_tiles

    def quantize(self, model: nn.Module) -> nn.Module:
        return quantize_linears_4w(model, self.groupsize, self.inner_k_tiles)


class Int4WeightOnlyQATQuantizerModuleSwap(Int4WeightOnlyQATQuantizer):
    """Older name of the same quantizer (``torchtune/training/quantization.py:136-147``)."""


class Int8DynActInt4WeightQATQuantizerModuleSwap(Int8DynActInt4WeightQATQuantizer):
    """Older name of the same quantizer (``torchtune/training/quantization.py:151-163``)."""


_quantizer_to_mode = {
    Int8DynActInt4WeightQuantizer: "8da4w",
    Int8DynActInt4WeightQATQuantizer: "8da4w-qat",
    Int4WeightOnlyQuantizer: "4w",
    Int4WeightOnlyQATQuantizer: "4w-qat",
    Int4WeightOnlyQATQuantizerModuleSwap: "4w-qat-module-swap",
    Int8DynActInt4WeightQATQuantizerModuleSwap: "8da4w-qat-module-swap",
}


def _enable_linear_fake_quant(mod: nn.Module, enabled: bool = True) -> None:
    """Switch both fake quantizers of a ``FakeQuantizedLinear`` on or off (use with ``model.apply``)."""
    if isinstance(mod, FakeQuantizedLinear):
        for fq in (mod.activation_fake_quantizer, mod.weight_fake_quantizer):
            if fq is not None:
                fq.enabled = enabled


def _disable_linear_fake_quant(mod: nn.Module) -> None:
    _enable_linear_fake_quant(mod, enabled=False)


disable_4w_fake_quant_module_swap = _disable_linear_fake_quant
enable_4w_fake_quant_module_swap = _enable_linear_fake_quant
disable_8da4w_fake_quant_module_swap = _disable_linear_fake_quant
enable_8da4w_fake_quant_module_swap = _enable_linear_fake_quant

_QAT_MODES = ("8da4w-qat", "4w-qat", "4w-qat-module-swap", "8da4w-qat-module-swap")
_quantizer_mode_to_disable_fake_quant = {mode: _disable_linear_fake_quant for mode in _QAT_MODES}
_quantizer_mode_to_enable_fake_quant = {mode: _enable_linear_fake_quant for mode in _QAT_MODES}


def get_quantizer_mode(quantizer: Optional[Callable]) -> Optional[str]:
    """The mode string of a quantizer ("8da4w", "8da4w-qat", "4w", "4w-qat" and the two "-module-swap" aliases);
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
