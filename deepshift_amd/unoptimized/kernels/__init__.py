from .kernels import conv2d, linear

__all__ = ["linear", "conv2d"]
