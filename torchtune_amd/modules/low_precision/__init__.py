from .nf4_linear import FrozenNF4Linear

__all__ = ["FrozenNF4Linear"]
