from ._utils import AdapterModule, get_adapter_params, get_merged_lora_ckpt, set_trainable_params
from .dora import DoRALinear
from .lora import LoRALinear, QATLoRALinear, TrainableParams

__all__ = [
    "AdapterModule",
    "DoRALinear",
    "LoRALinear",
    "QATLoRALinear",
    "TrainableParams",
    "get_adapter_params",
    "get_merged_lora_ckpt",
    "set_trainable_params",
]
