"""DeepShift-Q layers: the counterpart of the reference's ``deepshift/modules_q.py``.

``LinearShiftQ`` (modules_q.py:69-138) and ``Conv2dShiftQ`` (modules_q.py:262-309) keep a float
``weight`` that is clamped to [2^shift_range[0], 2^shift_range[1]] in magnitude and rounded to a
signed power of two on every forward.  With ``use_kernel=True`` the rounded weight's
(shift, sign) codes run through the same fixed-point shift kernel as the PS layers
(LinearShiftQFunction.forward modules_q.py:20-43, Conv2dShiftQFunction.forward :146-170); the
input is rounded to fixed point first in both layers (modules_q.py:118,286).

The reference's ``LinearShiftQ`` passes its arguments to the kernel branch in the wrong slots
(modules_q.py:125) and so never ran with ``use_kernel=True``; here it does what the function body
evidently intends.
"""
import math

import torch.nn as nn
import torch.nn.functional as F
from torch.nn import init
from torch.nn.modules.utils import _pair

from . import kernels, ste, utils
from .modules import (_FixedBias, _PackedWeightsMixin, _param_tensor, _params_key, _circular_pad,
                      conv_cpu_forward, conv_kernel_forward, linear_cpu_forward)

__all__ = ["LinearShiftQ", "Conv2dShiftQ"]


def _shift_range_q(weight_bits):
    # binary sign, so the whole code range is available for the shift (modules_q.py:80)
    return (-1 * (2 ** (weight_bits - 1) - 1), 0)


def module_codes_q(module):
    """(shift, sign) of the power-of-two rounding of ``module.weight``, clamped like the forward pass
    does (modules_q.py:116,21 / :284,147)."""
    w = module.weight.detach().clone()
    w = utils.clampabs(w, 2 ** module.shift_range[0], 2 ** module.shift_range[1])
    return utils.get_shift_and_sign(w, 'deterministic')


def pack_module_weights_q(module):
    """Pack the power-of-two rounding of ``module.weight``: on the GPU straight from the float weights
    (clamping |w| to [2^lo, 2^hi] then rounding log2 equals rounding then clamping the shift to
    [lo, hi]; exact zeros stay zero, utils.py:44-52), elsewhere through the float codes."""
    if module.weight.is_cuda:
        module.conc_weight = utils.convert_weights(module.weight, module.shift_range)
    else:
        module.conc_weight = utils.compress_bits(*module_codes_q(module))
    object.__setattr__(module, "_packed_from", _params_key(module.weight))
    return module.conc_weight


class _PackedQMixin(_PackedWeightsMixin):
    def _weight_params(self):
        return (self.weight,)

    def _pack(self):
        return pack_module_weights_q(self)


class LinearShiftQ(_PackedQMixin, nn.Module):
    def __init__(self, in_features, out_features, bias=True, check_grad=False, use_kernel=False,
                 use_cuda=True, rounding='deterministic', weight_bits=5, act_integer_bits=16,
                 act_fraction_bits=16):
        super(LinearShiftQ, self).__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.use_kernel = use_kernel
        self.check_grad = check_grad
        self.use_cuda = use_cuda
        self.rounding = rounding
        self.shift_range = _shift_range_q(weight_bits)
        self.act_integer_bits, self.act_fraction_bits = act_integer_bits, act_fraction_bits
        self.weight = nn.Parameter(_param_tensor(check_grad, out_features, in_features))
        if bias:
            self.bias = nn.Parameter(_param_tensor(check_grad, out_features))
        else:
            self.register_parameter('bias', None)
        self._fixed_bias = _FixedBias()
        self.reset_parameters()

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in)
            init.uniform_(self.bias, -bound, bound)

    def _kernel_forward(self, input, relu=False):
        I, Fb = self.act_integer_bits, self.act_fraction_bits
        lead = input.shape[:-1]
        x2d = input.reshape(-1, self.in_features).float()
        if not self.use_cuda:
            shift, sign = module_codes_q(self)
            out = linear_cpu_forward(x2d, shift, sign, self.bias, I, Fb, round_to_fixed=True)
            out = torch.relu(out) if relu else out
            return out.reshape(*lead, self.out_features)
        conc_weight = self.packed_weights()
        bias = self._fixed_bias.get(self.bias, I, Fb, round_to_fixed=True)
        tiled = kernels._tiled_of(conc_weight, self.out_features, self.in_features)
        out = kernels.linear_layer(x2d, tiled, bias, self.out_features, kernels.kernel_bits(conc_weight),
                                   conc_weight.base, I, Fb, round_to_fixed=True, relu=relu)
        return out.reshape(*lead, self.out_features)

    def forward(self, input):
        if self.use_kernel:
            # packed from the clamped weight (pack_module_weights_q): nothing left to clamp per call
            return self._kernel_forward(input)
        self.weight.data = ste.clampabs(self.weight.data, 2 ** self.shift_range[0],
                                        2 ** self.shift_range[1])
        weight_q = ste.round_power_of_2(self.weight, self.rounding)
        input_fixed_point = ste.round_fixed_point(input, self.act_integer_bits,
                                                  self.act_fraction_bits)
        out = input_fixed_point.mm(weight_q.t())
        if self.bias is not None:
            # modules_q.py:129: the un-rounded bias is added on this path
            out = out + self.bias.unsqueeze(0).expand_as(out)
        return out

    def extra_repr(self):
        return 'in_features={}, out_features={}, bias={}'.format(
            self.in_features, self.out_features, self.bias is not None)


class Conv2dShiftQ(_PackedQMixin, nn.Module):
    __constants__ = ['stride', 'padding', 'dilation', 'groups', 'bias', 'padding_mode']

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode='zeros', check_grad=False, use_kernel=False,
                 use_cuda=True, rounding='deterministic', weight_bits=5, act_integer_bits=16,
                 act_fraction_bits=16):
        super(Conv2dShiftQ, self).__init__()
        if in_channels % groups != 0:
            raise ValueError('in_channels must be divisible by groups')
        if out_channels % groups != 0:
            raise ValueError('out_channels must be divisible by groups')
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = _pair(kernel_size)
        self.stride = _pair(stride)
        self.padding = _pair(padding)
        self.dilation = _pair(dilation)
        self.transposed = False
        self.output_padding = _pair(0)
        self.groups = groups
        self.padding_mode = padding_mode
        self.use_kernel = use_kernel
        self.use_cuda = use_cuda
        self.rounding = rounding
        self.shift_range = _shift_range_q(weight_bits)
        self.act_integer_bits, self.act_fraction_bits = act_integer_bits, act_fraction_bits
        self.weight = nn.Parameter(_param_tensor(check_grad, out_channels, in_channels // groups,
                                                 *self.kernel_size))
        if bias:
            self.bias = nn.Parameter(_param_tensor(check_grad, out_channels))
        else:
            self.register_parameter('bias', None)
        self._fixed_bias = _FixedBias()
        self.reset_parameters()

    def reset_parameters(self):
        init.kaiming_uniform_(self.weight, a=math.sqrt(5))
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.weight)
            bound = 1 / math.sqrt(fan_in)
            init.uniform_(self.bias, -bound, bound)

    def forward(self, input):
        if self.use_kernel:
            if not self.use_cuda:
                return conv_cpu_forward(self, input, *module_codes_q(self))
            return conv_kernel_forward(self, input, self.packed_weights())
        self.weight.data = ste.clampabs(self.weight.data, 2 ** self.shift_range[0],
                                        2 ** self.shift_range[1])
        weight_q = ste.round_power_of_2(self.weight, self.rounding)
        input_fixed_point = ste.round_fixed_point(input, self.act_integer_bits,
                                                  self.act_fraction_bits)
        if self.bias is not None:
            bias_fixed_point = ste.round_fixed_point(self.bias, self.act_integer_bits,
                                                     self.act_fraction_bits)
        else:
            bias_fixed_point = None
        if self.padding_mode == 'circular':
            input_padded = _circular_pad(input_fixed_point, self.padding)
            padding = _pair(0)
        else:
            input_padded = input_fixed_point
            padding = self.padding
        return F.conv2d(input_padded, weight_q, bias_fixed_point, self.stride, padding,
                        self.dilation, self.groups)

    def extra_repr(self):
        s = ('{in_channels}, {out_channels}, kernel_size={kernel_size}, stride={stride}')
        if self.padding != (0,) * len(self.padding):
            s += ', padding={padding}'
        if self.groups != 1:
            s += ', groups={groups}'
        if self.bias is None:
            s += ', bias=False'
        return s.format(**self.__dict__)
