"""torchtune_amd — MI355X (gfx950) implementation of torchtune's quantized-linear hot path:
QLoRA ``LoRALinear`` / ``FrozenNF4Linear`` over NF4 weights and the 8da4w QAT fake-quant linear.

All arithmetic runs in ``lib/libtorchtune_amd.so`` (hand-written HIP, plain C ABI); build it with
``python -m torchtune_amd.build``.
"""
from .nf4_tensor import NF4Tensor, implements, linear_nf4, to_nf4
from .modules.low_precision import FrozenNF4Linear
from .modules.peft import DoRALinear, LoRALinear, QATLoRALinear
from .qat import (
    FakeQuantizeConfig,
    FakeQuantizedLinear,
    FakeQuantizer,
    Int4WeightOnlyQATLinear,
    Int4WeightOnlyQATQuantizer,
    Int8DynActInt4WeightLinear,
    Int8DynActInt4WeightQATLinear,
    Int8DynActInt4WeightQATQuantizer,
    WeightOnlyInt4Linear,
    ZeroPointDomain,
)

__all__ = [
    "NF4Tensor",
    "to_nf4",
    "linear_nf4",
    "implements",
    "FrozenNF4Linear",
    "LoRALinear",
    "DoRALinear",
    "QATLoRALinear",
    "FakeQuantizeConfig",
    "FakeQuantizer",
    "FakeQuantizedLinear",
    "Int8DynActInt4WeightQATQuantizer",
    "Int8DynActInt4WeightQATLinear",
    "Int8DynActInt4WeightLinear",
    "Int4WeightOnlyQATQuantizer",
    "Int4WeightOnlyQATLinear",
    "WeightOnlyInt4Linear",
    "ZeroPointDomain",
]
