"""Adapter layers of the quantized-linear path (LoRA, QAT + LoRA, DoRA over dense or NF4 base weights) and the small
amount of adapter bookkeeping their callers need."""
from ._adapter_base import LowRankAdapterLinear
from ._utils import (AdapterModule, disable_adapter, get_adapter_params, get_adapter_state_dict, get_merged_lora_ckpt,
                     set_trainable_params)
from .dora import DoRALinear
from .group import group_applies, lora_feed_forward, lora_linear_group, lora_swiglu_group
from .lora import LoRALinear, QATLoRALinear, TrainableParams

__all__ = (
    "LoRALinear",
    "QATLoRALinear",
    "DoRALinear",
    "LowRankAdapterLinear",
    "TrainableParams",
    "AdapterModule",
    "get_adapter_params",
    "set_trainable_params",
    "get_merged_lora_ckpt",
    "get_adapter_state_dict",
    "disable_adapter",
    "lora_linear_group",
    "lora_feed_forward",
    "lora_swiglu_group",
    "group_applies",
)
