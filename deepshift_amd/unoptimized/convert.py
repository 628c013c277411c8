"""``convert_to_unoptimized`` (unoptimized/convert.py:8-30 in the reference): every ``nn.Linear`` /
``nn.Conv2d`` of a model becomes its comparator counterpart and keeps its parameters."""
import torch.nn as nn

from .modules import UnoptimizedConv2d, UnoptimizedLinear


def _as_comparator(layer):
    """The comparator module for an exact ``nn.Linear`` / ``nn.Conv2d`` (subclasses are left alone),
    sharing the layer's parameter objects; ``None`` for anything else."""
    if type(layer) is nn.Linear:
        twin = UnoptimizedLinear(layer.in_features, layer.out_features, bias=layer.bias is not None)
    elif type(layer) is nn.Conv2d:
        twin = UnoptimizedConv2d(layer.in_channels, layer.out_channels, layer.kernel_size, layer.stride,
                                 layer.padding, layer.dilation, layer.groups, layer.bias is not None,
                                 layer.padding_mode)
    else:
        return None
    twin.weight, twin.bias = layer.weight, layer.bias
    return twin.to(layer.weight.device)


def convert_to_unoptimized(model):
    for name, child in list(model.named_children()):
        twin = _as_comparator(child)
        if twin is not None:
            setattr(model, name, twin)
        else:
            convert_to_unoptimized(child)
    return model
