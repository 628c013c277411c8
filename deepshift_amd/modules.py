"""DeepShift-PS layers: the counterpart of the reference's ``deepshift/modules.py``.

``LinearShift`` (modules.py:78-142) and ``Conv2dShift`` (modules.py:292-340) keep the reference's
constructor arguments, parameters (``shift``, ``sign``, ``bias``) and attributes
(``conc_weight``, ``use_kernel``, ``use_cuda``, ``shift_range``, ...).  With ``use_kernel=True``
the forward pass is the fixed-point shift kernel on the GPU:

    float input --quantise--> int32 --shift-add kernel on packed weights--> int32 --/2^F--> float

(LinearShiftFunction.forward modules.py:24-31, Conv2dShiftFunction.forward :152-162), otherwise
the float path of the reference (``F.linear`` / ``F.conv2d`` with +-2^shift weights, :135,:339).
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn import init
from torch.nn.modules.utils import _pair

from . import kernels, ste, utils

__all__ = ["LinearShift", "Conv2dShift"]


def _shift_range(weight_bits):
    # one code point of the sign/shift alphabet is kept for ternary signs (modules.py:88)
    return (-1 * (2 ** (weight_bits - 1) - 2), 0)


def _param_tensor(check_grad, *shape):
    # double precision when the layer is built for gradient checking (modules.py:98-101)
    return torch.empty(*shape, dtype=torch.float64 if check_grad else torch.float32)


def module_codes(module):
    """The (shift, sign) a PS layer computes with: clamped to ``shift_range`` and rounded the way
    the float path reads them (modules.py:125-128,313-316)."""
    shift = module.shift.detach().clamp(*module.shift_range).round()
    sign = module.sign.detach().round().sign()
    return shift, sign


def _params_key(*params):
    """Identity and version of the parameters packed weights were built from."""
    return tuple((p.data_ptr(), p._version, p.device) for p in params)


class _PackedWeightsMixin:
    """``conc_weight`` as the reference has it (an attribute that is None until the first kernel
    forward, modules.py:25-27), plus what the reference lacks: packed words that were built from the
    layer's own parameters are rebuilt when those parameters change (``load_state_dict``, fine-tuning
    then evaluating, ``round_shift_weights``).  A ``conc_weight`` assigned from outside is used as
    given.  Changes are seen through the parameters' storage address and version counter, i.e. every
    in-place update of the parameter itself and every assignment to ``.data``; an in-place operation
    on ``param.data`` bypasses the version counter -- set ``conc_weight = None`` after one."""

    _conc_weight = None
    _packed_from = None

    @property
    def conc_weight(self):
        return self._conc_weight

    @conc_weight.setter
    def conc_weight(self, value):
        object.__setattr__(self, "_conc_weight", value)
        object.__setattr__(self, "_packed_from", None)

    def _weight_params(self):
        return (self.shift, self.sign)

    def _pack(self):
        return pack_module_weights(self)

    def __getstate__(self):
        # the hand-off buffers of the fused pipeline (GPU scratch that the next forward pass rebuilds)
        # do not travel with copy.deepcopy / pickling of the module
        state = self.__dict__.copy()
        state.pop("_handoff_buffers", None)
        return state

    def packed_weights(self):
        """The layer's ConcWeight, (re)built if it is missing or older than the parameters."""
        if self._conc_weight is None or (self._packed_from is not None and
                                         self._packed_from != _params_key(*self._weight_params())):
            self._pack()
        return self._conc_weight


def pack_module_weights(module):
    """Build ``module.conc_weight`` from its (shift, sign) parameters (see :func:`module_codes`)."""
    shift, sign = module_codes(module)
    module.conc_weight = utils.compress_bits(shift, sign)
    object.__setattr__(module, "_packed_from", _params_key(module.shift, module.sign))
    return module.conc_weight


class _FixedBias:
    """int32 fixed-point copy of a float bias, rebuilt only when the parameter changes."""

    def __init__(self):
        self.key = None
        self.value = None

    def get(self, bias, integer_bits, fraction_bits, round_to_fixed):
        if bias is None:
            return None
        key = (bias.data_ptr(), bias._version, integer_bits, fraction_bits, round_to_fixed)
        if key != self.key:
            self.value = kernels.quantize(bias.detach().float(), integer_bits, fraction_bits,
                                          round_to_fixed)
            self.key = key
        return self.value


def pack_from_float_weight(module, weight):
    """Conversion of a trained float layer (convert.py:72-76): the packed words straight from the float
    weights in device passes (``utils.convert_weights``), valid for the module's (shift, sign)
    parameters when those were just derived from the same weights with ``get_shift_and_sign``."""
    if not weight.is_cuda:
        return pack_module_weights(module)
    module.conc_weight = utils.convert_weights(weight, module.shift_range)
    object.__setattr__(module, "_packed_from", _params_key(module.shift, module.sign))
    return module.conc_weight


class LinearShift(_PackedWeightsMixin, nn.Module):
    def __init__(self, in_features, out_features, bias=True, check_grad=False, freeze_sign=False,
                 use_kernel=False, use_cuda=True, rounding='deterministic', weight_bits=5,
                 act_integer_bits=16, act_fraction_bits=16):
        super(LinearShift, self).__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.use_kernel = use_kernel
        self.check_grad = check_grad
        self.use_cuda = use_cuda
        self.rounding = rounding
        self.shift_range = _shift_range(weight_bits)
        self.act_integer_bits, self.act_fraction_bits = act_integer_bits, act_fraction_bits

        self.shift = nn.Parameter(_param_tensor(check_grad, out_features, in_features))
        self.sign = nn.Parameter(_param_tensor(check_grad, out_features, in_features),
                                 requires_grad=(freeze_sign == False))  # noqa: E712
        if bias:
            self.bias = nn.Parameter(_param_tensor(check_grad, out_features))
        else:
            self.register_parameter('bias', None)
        self._fixed_bias = _FixedBias()
        self.reset_parameters()

    def reset_parameters(self):
        self.shift.data.uniform_(*self.shift_range)
        self.sign.data.uniform_(-1, 1)
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.shift)
            bound = 1 / math.sqrt(fan_in)
            init.uniform_(self.bias, -bound, bound)

    def _kernel_forward(self, input, relu=False):
        # modules.py:24-31: the input is cast, NOT rounded/clamped first (truncation toward zero)
        # (relu: a ReLU follows the layer and runs in its launch -- fuse.FusedLinearShift)
        I, Fb = self.act_integer_bits, self.act_fraction_bits
        lead = input.shape[:-1]
        x2d = input.reshape(-1, self.in_features).float()
        if not self.use_cuda:
            shift, sign = module_codes(self)
            out = linear_cpu_forward(x2d, shift, sign, self.bias, I, Fb, round_to_fixed=False)
            out = torch.relu(out) if relu else out
            return out.reshape(*lead, self.out_features)
        conc_weight = self.packed_weights()
        bias = self._fixed_bias.get(self.bias, I, Fb, round_to_fixed=False)
        tiled = kernels._tiled_of(conc_weight, self.out_features, self.in_features)
        out = kernels.linear_layer(x2d, tiled, bias, self.out_features, kernels.kernel_bits(conc_weight),
                                   conc_weight.base, I, Fb, round_to_fixed=False, relu=relu)
        return out.reshape(*lead, self.out_features)

    def forward(self, input):
        if self.use_kernel:
            # the packed weights already hold the clamped, rounded codes (pack_module_weights), so
            # the per-call clamp of the float parameter (modules.py:125) would change nothing here
            return self._kernel_forward(input)
        self.shift.data = ste.clamp(self.shift.data, *self.shift_range)
        shift_rounded = ste.round(self.shift, rounding=self.rounding)
        sign_rounded_signed = ste.sign(ste.round(self.sign, rounding=self.rounding))
        weight_ps = ste.unsym_grad_mul(2 ** shift_rounded, sign_rounded_signed)
        return F.linear(input, weight_ps, self.bias)

    def extra_repr(self):
        return 'in_features={}, out_features={}, bias={}'.format(
            self.in_features, self.out_features, self.bias is not None)


class _ConvNdShift(_PackedWeightsMixin, nn.Module):
    __constants__ = ['stride', 'padding', 'dilation', 'groups', 'bias', 'padding_mode']

    def __init__(self, in_channels, out_channels, kernel_size, stride, padding, dilation, transposed,
                 output_padding, groups, bias, padding_mode, check_grad=False, freeze_sign=False,
                 rounding='deterministic', weight_bits=5, act_integer_bits=16,
                 act_fraction_bits=16):
        super(_ConvNdShift, self).__init__()
        if in_channels % groups != 0:
            raise ValueError('in_channels must be divisible by groups')
        if out_channels % groups != 0:
            raise ValueError('out_channels must be divisible by groups')
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.transposed = transposed
        self.output_padding = output_padding
        self.groups = groups
        self.padding_mode = padding_mode
        self.rounding = rounding
        self.shift_range = _shift_range(weight_bits)
        self.act_integer_bits, self.act_fraction_bits = act_integer_bits, act_fraction_bits

        if transposed:
            wshape = (in_channels, out_channels // groups) + tuple(kernel_size)
        else:
            wshape = (out_channels, in_channels // groups) + tuple(kernel_size)
        self.shift = nn.Parameter(_param_tensor(check_grad, *wshape))
        self.sign = nn.Parameter(_param_tensor(check_grad, *wshape),
                                 requires_grad=(freeze_sign == False))  # noqa: E712
        if bias:
            self.bias = nn.Parameter(_param_tensor(check_grad, out_channels))
        else:
            self.register_parameter('bias', None)
        self._fixed_bias = _FixedBias()
        self.reset_parameters()

    def reset_parameters(self):
        self.shift.data.uniform_(-10, -1)  # modules.py:268
        self.sign.data.uniform_(-1, 1)
        if self.bias is not None:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.shift)
            bound = 1 / math.sqrt(fan_in)
            init.uniform_(self.bias, -bound, bound)

    def extra_repr(self):
        s = ('{in_channels}, {out_channels}, kernel_size={kernel_size}'
             ', stride={stride}')
        if self.padding != (0,) * len(self.padding):
            s += ', padding={padding}'
        if self.dilation != (1,) * len(self.dilation):
            s += ', dilation={dilation}'
        if self.output_padding != (0,) * len(self.output_padding):
            s += ', output_padding={output_padding}'
        if self.groups != 1:
            s += ', groups={groups}'
        if self.bias is None:
            s += ', bias=False'
        return s.format(**self.__dict__)


def _circular_pad(x, padding):
    # modules.py:323-328: circular padding is materialised, then the convolution runs unpadded
    expanded = ((padding[1] + 1) // 2, padding[1] // 2, (padding[0] + 1) // 2, padding[0] // 2)
    return F.pad(x, expanded, mode='circular')


def _host_fixed(x, integer_bits, fraction_bits, round_to_fixed):
    """float CPU tensor -> int32 fixed point with the GPU passes' arithmetic: ``round_to_fixed`` then
    ``* 2^F`` (utils.py:7-21, modules.py:153), or the saturating truncating cast alone
    (modules.py:25)."""
    x = x.detach().float().cpu()
    if round_to_fixed:
        x = utils.round_to_fixed(x, integer_bits, fraction_bits)
    scaled = (x.double() * 2.0 ** fraction_bits).trunc()
    scaled = torch.nan_to_num(scaled, nan=0.0).clamp(-2.0 ** 31, 2.0 ** 31 - 1)
    return scaled.to(torch.int32)


def linear_cpu_forward(x2d, shift, sign, bias, integer_bits, fraction_bits, round_to_fixed):
    """LinearShift / LinearShiftQ with ``use_kernel=True, use_cuda=False``: the library's host kernel
    on the unpacked codes (modules.py:24-31 with kernels.py:22-24)."""
    xq = _host_fixed(x2d, integer_bits, fraction_bits, round_to_fixed)
    bq = None if bias is None else _host_fixed(bias, integer_bits, fraction_bits, round_to_fixed)
    out = kernels.linear(xq, shift, sign, bq, None, use_cuda=False)
    return (out.float() / 2.0 ** fraction_bits).to(x2d.device)


def conv_cpu_forward(module, input, shift, sign):
    """Conv2dShift / Conv2dShiftQ with ``use_kernel=True, use_cuda=False`` (modules.py:152-162 with
    kernels.py:57-63)."""
    if module.dilation != (1, 1) or module.groups != 1:
        raise NotImplementedError("the shift kernel supports dilation=1 and groups=1 only")
    I, Fb = module.act_integer_bits, module.act_fraction_bits
    padding = module.padding
    x = input.float()
    if module.padding_mode == 'circular':
        x = _circular_pad(x, padding)
        padding = (0, 0)
    xq = _host_fixed(x, I, Fb, True)
    bq = None if module.bias is None else _host_fixed(module.bias, I, Fb, True)
    out = kernels.conv2d(xq, shift, sign, bq, None, module.stride, padding, use_cuda=False)
    return (out.float() / 2.0 ** Fb).to(input.device)


# Switch for the fused convolution epilogue (kernels.conv2d_tiled_fused); off = always the separate
# conversion pass, which the tests compare it with.
_FUSE_EPILOGUE = True
_FUSE_INT8 = True   # ... and the int8 kernel's (kernels.conv2d_paired_fused)


def _small_for_int8(module, input_shape, field_bits):
    """The int8 kernel works on tiles of 384 pixels x 64 channels; a layer with few of them and a short
    reduction (the 1x1 shortcuts of a ResNet-18) is served better by the int32 kernels' smaller tiles.
    Measured: below about 8000 (tile, K group) units the int32 path wins."""
    Nb, _, H, W = input_shape
    ph, pw = (0, 0) if module.padding_mode == 'circular' else module.padding
    if module.padding_mode == 'circular':
        H, W = H + module.padding[0], W + module.padding[1]
    OH = (H + 2 * ph - module.kernel_size[0]) // module.stride[0] + 1
    OW = (W + 2 * pw - module.kernel_size[1]) // module.stride[1] + 1
    tiles = -(-Nb * OH * OW // 384) * (module.out_channels // 64)
    K = module.in_channels * module.kernel_size[0] * module.kernel_size[1]
    groups = -(-K // (32 // ((field_bits & 0xff) + 1)))
    return tiles * groups < 8192


def conv_kernel_forward(module, input, conc_weight, scale=None, shift=None, residual=None, relu=False,
                        prequantized=False, emit=None, pool=None, input_nonneg=False):
    """Fixed-point shift convolution of a float NCHW input (modules.py:152-162,317-337).

    ``scale``/``shift`` (per output channel), ``residual`` and ``relu`` describe what follows the
    layer (a folded BatchNorm, a shortcut add, ReLU); when any is given it is applied in the same
    pass that converts the int32 result back to float.

    ``prequantized``: ``input`` is already the layer's round-to-fixed, zero padded int32 input (made
    by the layer before it).  ``emit = (padding, integer_bits, fraction_bits, want_float)``: also
    produce that form of the result for the next shift convolution (a fifth element gives its dtype:
    int8 for a consumer on the int8 kernel); the return value is then ``(out, q)``, or ``q`` alone when
    ``want_float`` is false.  ``pool = (kernel, stride, padding)``:
    a max pooling follows the ReLU (no residual) and runs in the same pass.  ``input_nonneg``: the
    producer of a prequantized input vouches that it is the output of a ReLU (the int8 kernel then
    knows a tighter bound on the activations and widens its 16-bit sums less often)."""
    if not module.use_cuda:
        raise ValueError("conv_kernel_forward is the GPU path; use_cuda=False layers run conv_cpu_forward")
    if module.dilation != (1, 1) or module.groups != 1:
        raise NotImplementedError("the shift kernel supports dilation=1 and groups=1 only")
    I, Fb = module.act_integer_bits, module.act_fraction_bits
    # formats of at most 8 bits on narrow shift fields: int8 activations, two pixels per register
    fields = kernels.paired_fields(conc_weight, module.out_channels, I, Fb)
    if prequantized:
        xq = input
    else:
        if fields and _small_for_int8(module, input.shape, fields[1]):
            fields = None
        padding = module.padding
        input = input.float()
        if module.padding_mode == 'circular':
            input = _circular_pad(input, padding)
            padding = (0, 0)
        # round_to_fixed + cast + zero padding in one pass
        xq = kernels.quantize_pad(input, padding, I, Fb, round_to_fixed=True,
                                  dtype=torch.int8 if fields else torch.int32)
    bias = module._fixed_bias.get(module.bias, I, Fb, round_to_fixed=True)
    if xq.dtype == torch.int8:
        if not fields:
            raise ValueError("this layer has no int8 kernel; hand it int32 activations")
        blob = kernels._paired_of(conc_weight, fields, module.out_channels, module.in_channels,
                                  module.kernel_size[0], module.kernel_size[1])
        # round_to_fixed clamps to [-2^(I-1), 2^(I-1) - 1] (utils.py:7-21): |x| <= 2^(I+F-1), and after
        # a ReLU x <= (2^(I-1) - 1) * 2^F
        bound = (2 ** (I - 1) - 1) * 2 ** Fb if (prequantized and input_nonneg) else 2 ** (I + Fb - 1)
        if pool is None and _FUSE_EPILOGUE and _FUSE_INT8:
            # the int8 kernel's fused launch: dequantisation, affine / residual / ReLU and the next layer's
            # conversion in the epilogue; no pre-fill, no atomics, no int32 sums, no separate pass
            want_float, spec = True, None
            if emit is not None:
                next_padding, next_I, next_F, want_float = emit[:4]
                spec = (next_padding, next_I, next_F, emit[4] if len(emit) == 5 else torch.int32)
            cache = module.__dict__.setdefault("_handoff_buffers", {})
            f, q = kernels.conv2d_paired_fused(xq, blob, bias, module.out_channels, module.kernel_size,
                                               module.stride, fields[1], max(1, bound), Fb, scale, shift,
                                               residual, relu, spec, want_float, cache)
            if emit is None:
                return f
            return (f, q) if want_float else q
        out = kernels.conv2d_paired(xq, blob, bias, module.out_channels, module.kernel_size, module.stride,
                                    fields[1], max(1, bound))
    else:
        tiled = kernels._tiled_of(conc_weight, module.out_channels, module.in_channels,
                                  module.kernel_size[0], module.kernel_size[1])
        kbits = kernels.kernel_bits(conc_weight)
        if pool is None and _FUSE_EPILOGUE and kernels.conv2d_fusable(
                xq.shape, module.out_channels, module.kernel_size, module.stride, kbits, conc_weight.base):
            # the layer's epilogue does the dequantisation, the affine / residual / ReLU and the next
            # layer's conversion while the tile is still on chip: the int32 sums are never stored
            want_float, spec = True, None
            if emit is not None:
                next_padding, next_I, next_F, want_float = emit[:4]
                spec = (next_padding, next_I, next_F, emit[4] if len(emit) == 5 else torch.int32)
            # the consumers' padded input lives in a buffer of this layer that is zeroed once: the kernel
            # then writes the interior only (the next forward pass overwrites it, in stream order)
            cache = module.__dict__.setdefault("_handoff_buffers", {})
            f, q = kernels.conv2d_tiled_fused(xq, tiled, bias, module.out_channels, module.kernel_size,
                                              module.stride, kbits, Fb, scale, shift, residual, relu, spec,
                                              want_float, cache)
            if emit is None:
                return f
            return (f, q) if want_float else q
        out = kernels.conv2d_tiled(xq, tiled, bias, module.out_channels, module.kernel_size,
                                   module.stride, kbits, conc_weight.base)
    emit_dtype = torch.int32
    if emit is not None and len(emit) == 5:
        emit, emit_dtype = emit[:4], emit[4]
    if pool is not None:
        if residual is not None:
            raise ValueError("a fused max pooling cannot follow a residual add")
        if emit is None:
            return kernels.requantize_affine_maxpool(out, Fb, scale, shift, relu, pool)[0]
        next_padding, next_I, next_F, want_float = emit
        f, q = kernels.requantize_affine_maxpool(out, Fb, scale, shift, relu, pool, next_padding,
                                                 next_I, next_F, want_float, emit_dtype)
        return (f, q) if want_float else q
    if emit is not None:
        next_padding, next_I, next_F, want_float = emit
        f, q = kernels.requantize_affine_pad(out, Fb, scale, shift, residual, relu, next_padding,
                                             next_I, next_F, want_float, emit_dtype)
        return (f, q) if want_float else q
    if scale is None and shift is None and residual is None and not relu:
        return kernels.dequantize(out, Fb)
    return kernels.dequantize_affine(out, Fb, scale, shift, residual, relu)


class Conv2dShift(_ConvNdShift):
    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, padding_mode='zeros', check_grad=False, freeze_sign=False,
                 use_kernel=False, use_cuda=True, rounding='deterministic', weight_bits=5,
                 act_integer_bits=16, act_fraction_bits=16):
        kernel_size = _pair(kernel_size)
        stride = _pair(stride)
        padding = _pair(padding)
        dilation = _pair(dilation)
        self.use_kernel = use_kernel
        self.use_cuda = use_cuda
        super(Conv2dShift, self).__init__(
            in_channels, out_channels, kernel_size, stride, padding, dilation, False, _pair(0),
            groups, bias, padding_mode, check_grad, freeze_sign, rounding, weight_bits,
            act_integer_bits, act_fraction_bits)

    def forward(self, input):
        if self.use_kernel:
            if not self.use_cuda:
                return conv_cpu_forward(self, input, *module_codes(self))
            return conv_kernel_forward(self, input, self.packed_weights())
        self.shift.data = ste.clamp(self.shift.data, *self.shift_range)

        shift_rounded = ste.round(self.shift, self.rounding)
        sign_rounded_signed = ste.sign(ste.round(self.sign, self.rounding))
        weight_ps = ste.unsym_grad_mul(2 ** shift_rounded, sign_rounded_signed)
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
        return F.conv2d(input_padded, weight_ps, bias_fixed_point, self.stride, padding,
                        self.dilation, self.groups)
