"""``convert_to_unoptimized`` (unoptimized/convert.py:8-30 in the reference): every ``nn.Linear`` /
``nn.Conv2d`` becomes its comparator counterpart, sharing the original parameters."""
import torch.nn as nn

from .modules import UnoptimizedConv2d, UnoptimizedLinear


def convert_to_unoptimized(model):
    for name, module in model._modules.items():
        if module is None:
            continue
        if len(list(module.children())) > 0:
            model._modules[name] = convert_to_unoptimized(model=module)
        if type(module) == nn.Linear:
            new = UnoptimizedLinear(module.in_features, module.out_features, module.bias is not None)
            new.weight = module.weight
            new.bias = module.bias
            model._modules[name] = new
        if type(module) == nn.Conv2d:
            new = UnoptimizedConv2d(module.in_channels, module.out_channels, module.kernel_size,
                                    module.stride, module.padding, module.dilation, module.groups,
                                    module.bias is not None, module.padding_mode)
            new.weight = module.weight
            new.bias = module.bias
            model._modules[name] = new
    return model
