"""``UnoptimizedLinear``: an ``nn.Linear`` whose forward pass is the comparator's float
multiply-accumulate kernel (the role of unoptimized/modules/linear.py:13-51 in the reference)."""
import torch.nn as nn

from .. import kernels


class UnoptimizedLinear(nn.Linear):
    """Same parameters, initialisation and ``repr`` as ``nn.Linear``; only the arithmetic moves to
    ``ds_mul_linear_f32``."""

    def forward(self, input):
        return kernels.linear(input, self.weight, self.bias)
