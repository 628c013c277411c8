from .conv import UnoptimizedConv2d
from .linear import UnoptimizedLinear

__all__ = ["UnoptimizedLinear", "UnoptimizedConv2d"]
