"""Float multiply-accumulate comparator (mirror of the reference's ``unoptimized`` package).

``convert_to_unoptimized(model)`` swaps every ``nn.Linear`` / ``nn.Conv2d`` for a module that runs
the plain fp32 HIP kernel with the same structure and data movement as the shift kernel
(``ds_mul_linear_f32`` / ``ds_mul_conv2d_f32``), so that "shift against multiply" is timed on equal
terms, as the reference does with ``--use-kernel True --shift-depth 0`` (imagenet.py:245-246).
"""
from .convert import convert_to_unoptimized
from .modules import UnoptimizedConv2d, UnoptimizedLinear

__all__ = ["convert_to_unoptimized", "UnoptimizedLinear", "UnoptimizedConv2d"]
