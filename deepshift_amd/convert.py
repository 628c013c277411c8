"""Model conversion: the counterpart of the reference's ``deepshift/convert.py``.

``convert_to_shift`` (convert.py:11-81) walks ``model._modules`` from the LAST layer backwards,
replacing ``nn.Linear`` / ``nn.Conv2d`` with shift layers until ``shift_depth`` layers are
converted; ``round_shift_weights`` (convert.py:83-105) snaps the parameters to the values the
fixed-point kernel uses; ``count_layer_type`` (convert.py:107-115) counts layers of a type.

One deliberate difference: packed kernel weights are built from the shifts AFTER clamping them to
the layer's ``shift_range`` (the reference packs first and clamps later in ``forward``,
modules.py:125,313), so the kernel path and the float path of a converted model always use the
same power-of-two weights.
"""
import copy

import torch.nn as nn

from . import modules, modules_q, utils

__all__ = ["convert_to_shift", "round_shift_weights", "count_layer_type"]


def _kernel_on_gpu(use_kernel, use_cuda):
    return use_cuda == True and use_kernel == True  # noqa: E712


def _convert_linear(linear, shift_type, convert_weights, freeze_sign, kw):
    has_bias = linear.bias is not None
    if shift_type == 'Q':
        layer = modules_q.LinearShiftQ(linear.in_features, linear.out_features, has_bias, **kw)
        layer.weight = linear.weight
        if has_bias:
            layer.bias.data = utils.round_to_fixed(linear.bias, integer_bits=kw['act_integer_bits'],
                                                   fraction_bits=kw['act_fraction_bits'])
        if _kernel_on_gpu(kw['use_kernel'], kw['use_cuda']):
            modules_q.pack_module_weights_q(layer)
    elif shift_type == 'PS':
        layer = modules.LinearShift(linear.in_features, linear.out_features, has_bias,
                                    freeze_sign=freeze_sign, **kw)
        if convert_weights == True:  # noqa: E712
            layer.shift.data, layer.sign.data = utils.get_shift_and_sign(linear.weight)
            layer.bias = linear.bias
            if _kernel_on_gpu(kw['use_kernel'], kw['use_cuda']):
                modules.pack_from_float_weight(layer, linear.weight)
    else:
        raise ValueError('Unsupported shift_type argument: ', shift_type)
    return layer.to(linear.weight.device)


def _convert_conv2d(conv, shift_type, convert_weights, freeze_sign, kw):
    has_bias = conv.bias is not None
    args = (conv.in_channels, conv.out_channels, conv.kernel_size, conv.stride, conv.padding,
            conv.dilation, conv.groups, has_bias, conv.padding_mode)
    if shift_type == 'Q':
        layer = modules_q.Conv2dShiftQ(*args, **kw)
        layer.weight = conv.weight
        if has_bias:
            layer.bias.data = utils.round_to_fixed(conv.bias, integer_bits=kw['act_integer_bits'],
                                                   fraction_bits=kw['act_fraction_bits'])
        if _kernel_on_gpu(kw['use_kernel'], kw['use_cuda']):
            modules_q.pack_module_weights_q(layer)
    elif shift_type == 'PS':
        layer = modules.Conv2dShift(*args, freeze_sign=freeze_sign, **kw)
        if convert_weights == True:  # noqa: E712
            layer.shift.data, layer.sign.data = utils.get_shift_and_sign(conv.weight)
            layer.bias = conv.bias
        layer = layer.to(conv.weight.device)
        if _kernel_on_gpu(kw['use_kernel'], kw['use_cuda']):
            if convert_weights == True:  # noqa: E712
                modules.pack_from_float_weight(layer, conv.weight)
            else:
                modules.pack_module_weights(layer)
    else:
        raise ValueError('Unsupported shift_type argument: ', shift_type)
    return layer.to(conv.weight.device)


def convert_to_shift(model, shift_depth, shift_type, convert_all_linear=True, convert_weights=False,
                     freeze_sign=False, use_kernel=False, use_cuda=True, rounding='deterministic',
                     weight_bits=5, act_integer_bits=16, act_fraction_bits=16):
    """Replace Linear/Conv2d layers by shift layers, last layer first; returns (model, count)."""
    kw = dict(use_kernel=use_kernel, use_cuda=use_cuda, rounding=rounding, weight_bits=weight_bits,
              act_integer_bits=act_integer_bits, act_fraction_bits=act_fraction_bits)
    conversion_count = 0
    for name, module in reversed(model._modules.items()):
        if len(list(module.children())) > 0:
            model._modules[name], num_converted = convert_to_shift(
                model=module, shift_depth=shift_depth - conversion_count, shift_type=shift_type,
                convert_all_linear=convert_all_linear, convert_weights=convert_weights,
                freeze_sign=freeze_sign, **kw)
            conversion_count += num_converted
        if type(module) == nn.Linear and (convert_all_linear == True  # noqa: E712
                                          or conversion_count < shift_depth):
            model._modules[name] = _convert_linear(module, shift_type, convert_weights, freeze_sign,
                                                   kw)
            if convert_all_linear == False:  # noqa: E712
                conversion_count += 1
        if type(module) == nn.Conv2d and conversion_count < shift_depth:
            model._modules[name] = _convert_conv2d(module, shift_type, convert_weights, freeze_sign,
                                                   kw)
            conversion_count += 1
    return model, conversion_count


def round_shift_weights(model, clone=False, weight_bits=5, act_integer_bits=16,
                        act_fraction_bits=16):
    """Round shift/sign (PS) or weight (Q) and the biases to their quantised values."""
    if clone:
        model = copy.deepcopy(model)
    for name, module in reversed(model._modules.items()):
        if len(list(module.children())) > 0:
            model._modules[name] = round_shift_weights(
                model=module, weight_bits=weight_bits, act_integer_bits=act_integer_bits,
                act_fraction_bits=act_fraction_bits)
        if type(module) in (modules.LinearShift, modules.Conv2dShift):
            module.shift.data = module.shift.round()
            module.sign.data = module.sign.round().sign()
            if module.bias is not None:
                module.bias.data = utils.round_to_fixed(module.bias, integer_bits=act_integer_bits,
                                                        fraction_bits=act_fraction_bits)
        elif type(module) in (modules_q.LinearShiftQ, modules_q.Conv2dShiftQ):
            module.weight.data = utils.clampabs(module.weight.data, 2 ** module.shift_range[0],
                                                2 ** module.shift_range[1])
            module.weight.data = utils.round_power_of_2(module.weight)
            if module.bias is not None:
                module.bias.data = utils.round_to_fixed(module.bias, integer_bits=act_integer_bits,
                                                        fraction_bits=act_fraction_bits)
    return model


def count_layer_type(model, layer_type):
    count = 0
    for name, module in model._modules.items():
        if len(list(module.children())) > 0:
            count += count_layer_type(model=module, layer_type=layer_type)
        if type(module) == layer_type:
            count += 1
    return count
