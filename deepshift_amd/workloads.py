"""The benchmark workloads of the shift-kernel path: plain-PyTorch network definitions (to be run
through ``convert_to_shift``) and their shift-layer shape tables.

The reference evaluates torchvision / CIFAR model-zoo networks (imagenet.py:214-219,
cifar10_models/resnet.py:23-140, mnist.py:23-39); torchvision is not a dependency here, so the
same textbook topologies are spelled out with stock ``nn`` layers.  Only ``nn.Conv2d`` and
``nn.Linear`` are touched by the conversion (convert.py:19,48); BatchNorm / ReLU / pooling stay
fp32 PyTorch ops between the shift layers, as in the reference.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = ["MLP", "ResNet18", "ResNet20", "ResNet50", "shift_layer_shapes", "randomize_batchnorm"]


class MLP(nn.Module):
    """784-512-512-10 with ReLU between layers (mnist.py:23-39, eval mode: dropout is identity)."""

    def __init__(self, sizes=(784, 512, 512, 10)):
        super().__init__()
        self.layers = nn.ModuleList([nn.Linear(a, b) for a, b in zip(sizes[:-1], sizes[1:])])

    def forward(self, x):
        x = x.reshape(x.shape[0], -1)
        for i, layer in enumerate(self.layers):
            x = layer(x)
            if i + 1 < len(self.layers):
                x = F.relu(x)
        return x


def _conv_bn(cin, cout, k, stride, pad):
    return nn.Sequential(nn.Conv2d(cin, cout, k, stride, pad, bias=False), nn.BatchNorm2d(cout))


class BasicBlock(nn.Module):
    def __init__(self, cin, cout, stride, shortcut):
        super().__init__()
        self.a = _conv_bn(cin, cout, 3, stride, 1)
        self.b = _conv_bn(cout, cout, 3, 1, 1)
        self.shortcut = shortcut

    def forward(self, x):
        out = self.b(F.relu(self.a(x)))
        return F.relu(out + (x if self.shortcut is None else self.shortcut(x)))


class Bottleneck(nn.Module):
    def __init__(self, cin, mid, stride, shortcut):
        super().__init__()
        self.a = _conv_bn(cin, mid, 1, 1, 0)
        self.b = _conv_bn(mid, mid, 3, stride, 1)
        self.c = _conv_bn(mid, mid * 4, 1, 1, 0)
        self.shortcut = shortcut

    def forward(self, x):
        out = self.c(F.relu(self.b(F.relu(self.a(x)))))
        return F.relu(out + (x if self.shortcut is None else self.shortcut(x)))


class _ImageNetResNet(nn.Module):
    def __init__(self, block, depths, num_classes):
        super().__init__()
        self.stem = _conv_bn(3, 64, 7, 2, 3)
        expansion = 1 if block is BasicBlock else 4
        stages, cin = [], 64
        for i, depth in enumerate(depths):
            width = 64 * 2 ** i
            for j in range(depth):
                stride = 2 if (i > 0 and j == 0) else 1
                cout = width * expansion
                shortcut = None
                if stride != 1 or cin != cout:
                    shortcut = _conv_bn(cin, cout, 1, stride, 0)
                stages.append(block(cin, width, stride, shortcut))
                cin = cout
        self.stages = nn.Sequential(*stages)
        self.fc = nn.Linear(cin, num_classes)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.stem(x)), 3, 2, 1)
        x = self.stages(x)
        x = F.adaptive_avg_pool2d(x, 1).flatten(1)
        return self.fc(x)


class ResNet18(_ImageNetResNet):
    """7x7/2 stem, max-pool, 4 x 2 basic blocks (64..512), FC 512 -> 1000: 21 shift layers."""

    def __init__(self, num_classes=1000):
        super().__init__(BasicBlock, (2, 2, 2, 2), num_classes)


class ResNet50(_ImageNetResNet):
    """Bottleneck 1x1/3x3/1x1 blocks (3, 4, 6, 3), FC 2048 -> 1000: 54 shift layers."""

    def __init__(self, num_classes=1000):
        super().__init__(Bottleneck, (3, 4, 6, 3), num_classes)


class _PadShortcut(nn.Module):
    """Parameter-free shortcut of the CIFAR ResNet: subsample by 2 and zero pad the channels
    (cifar10_models/resnet.py:38-40)."""

    def __init__(self, pad):
        super().__init__()
        self.pad = pad

    def forward(self, x):
        return F.pad(x[:, :, ::2, ::2], (0, 0, 0, 0, self.pad, self.pad))


class ResNet20(nn.Module):
    """CIFAR ResNet-20: 3x3 stem, 3 stages x 3 basic blocks (16/32/64), FC 64 -> 10
    (cifar10_models/resnet.py:85-140): 20 shift layers."""

    def __init__(self, num_classes=10):
        super().__init__()
        self.stem = _conv_bn(3, 16, 3, 1, 1)
        blocks, cin = [], 16
        for i, width in enumerate((16, 32, 64)):
            for j in range(3):
                stride = 2 if (i > 0 and j == 0) else 1
                shortcut = _PadShortcut(width // 4) if stride != 1 else None
                blocks.append(BasicBlock(cin, width, stride, shortcut))
                cin = width
        self.stages = nn.Sequential(*blocks)
        self.fc = nn.Linear(64, num_classes)

    def forward(self, x):
        x = self.stages(F.relu(self.stem(x)))
        x = F.adaptive_avg_pool2d(x, 1).flatten(1)
        return self.fc(x)


def randomize_batchnorm(model, generator=None):
    """Give every BatchNorm random (seeded) running statistics and affine terms."""
    for m in model.modules():
        if isinstance(m, nn.BatchNorm2d):
            m.running_mean.copy_(torch.randn(m.num_features, generator=generator) * 0.1)
            m.running_var.copy_(torch.rand(m.num_features, generator=generator) * 0.5 + 0.75)
            m.weight.data.copy_(torch.rand(m.num_features, generator=generator) * 0.5 + 0.75)
            m.bias.data.copy_(torch.randn(m.num_features, generator=generator) * 0.1)
    return model


def shift_layer_shapes(model, chw, batch):
    """Trace one batch-1 forward pass and list every Conv2d / Linear, scaled to ``batch``, as a
    dict: kind, name, M (rows / output pixels), K, N, and the geometry needed to replay the layer."""
    shapes = []
    hooks = []

    def conv_hook(name):
        def hook(mod, inp, out):
            x = inp[0]
            Nb, C, H, W = x.shape
            fh, fw = mod.kernel_size
            shapes.append(dict(kind="conv", name=name, Nb=batch, C=C, H=H, W=W, O=mod.out_channels,
                               FH=fh, FW=fw, stride=tuple(mod.stride), padding=tuple(mod.padding),
                               M=batch * out.shape[2] * out.shape[3], K=C * fh * fw,
                               N=mod.out_channels))
        return hook

    def linear_hook(name):
        def hook(mod, inp, out):
            x = inp[0]
            shapes.append(dict(kind="linear", name=name, M=batch * x.shape[0], K=mod.in_features,
                               N=mod.out_features))
        return hook

    for name, mod in model.named_modules():
        if isinstance(mod, nn.Conv2d):
            hooks.append(mod.register_forward_hook(conv_hook(name)))
        elif isinstance(mod, nn.Linear):
            hooks.append(mod.register_forward_hook(linear_hook(name)))
    was_training = model.training
    model.eval()
    with torch.no_grad():
        device = next(model.parameters()).device
        model(torch.zeros(1, *chw, device=device))
    model.train(was_training)
    for h in hooks:
        h.remove()
    return shapes
