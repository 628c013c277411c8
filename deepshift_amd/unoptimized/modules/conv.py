"""``UnoptimizedConv2d``: an ``nn.Conv2d`` whose forward pass pads with zeros and runs the
comparator's float multiply-accumulate kernel on the padded input (the role of
unoptimized/modules/conv.py:12-93 in the reference)."""
import torch.nn as nn
import torch.nn.functional as F

from .. import kernels


class UnoptimizedConv2d(nn.Conv2d):
    """Same parameters, initialisation and ``repr`` as ``nn.Conv2d``; zero padding, dilation 1 and
    groups 1 only -- what the kernel (and the reference's) covers."""

    def forward(self, input):
        if tuple(self.dilation) != (1, 1) or self.groups != 1:
            raise NotImplementedError("the comparator kernel supports dilation=1 and groups=1 only")
        if self.padding_mode != 'zeros' or isinstance(self.padding, str):
            raise NotImplementedError("the comparator kernel supports explicit zero padding only")
        ph, pw = self.padding
        padded = F.pad(input, (pw, pw, ph, ph))
        return kernels.conv2d(padded, self.weight, self.bias, self.stride, self.padding)
