from .low_precision import FrozenNF4Linear
from .peft import LoRALinear, QATLoRALinear

__all__ = ["FrozenNF4Linear", "LoRALinear", "QATLoRALinear"]
