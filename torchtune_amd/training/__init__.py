from . import quantization

__all__ = ["quantization"]
