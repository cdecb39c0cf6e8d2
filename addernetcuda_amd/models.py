"""The reference's other AdderNets as callers of ``adder2d``: ResNet-50, a VGG-small stack and the CIFAR DenseNet.

``resnet50`` has the architecture, parameter names and state_dict keys of the reference's resnet50.py:19-119:
a regular 7x7 stride-2 stem convolution, BatchNorm, ReLU and 3x3 max pooling (resnet50.py:63-67), four stages
of [3, 4, 6, 3] bottleneck blocks whose 1x1 / 3x3 / 1x1 convolutions are adder2d (resnet50.py:8-16, 19-33),
adder2d 1x1 + BatchNorm downsample on the first block of every stage (resnet50.py:84-90), global average
pooling, a regular 1x1 convolution classifier followed by BatchNorm (resnet50.py:72-74, 110-114).

``vgg_small`` is the CIFAR VGG-small stack, 128-128-M-256-256-M-512-512-M on 32x32 inputs (4x4 maps at the end)
with conv - BatchNorm - ReLU units as built by vgg.py:66-80; the layers are adder2d 3x3 pad 1 (vgg.py:16-18)
except, by default, the first one on the 3-channel image (``first_adder=True`` makes that one an adder layer
too, as vgg.py does), and a linear classifier.

``densenet_cifar`` has the architecture and state_dict keys of the reference's densenet.py:9-109: a regular 3x3
stem convolution (densenet.py:41), four dense stages of [6, 12, 24, 16] pre-activation bottlenecks (BatchNorm - ReLU
- adder2d 1x1 to 4 x growth channels - BatchNorm - ReLU - adder2d 3x3 to ``growth_rate`` = 12 channels, output
concatenated in front of the input, densenet.py:9-21), transitions of BatchNorm - ReLU - adder2d 1x1 halving the
channels - 2x2 average pooling (densenet.py:24-33), BatchNorm - ReLU - 4x4 average pooling - linear classifier
(densenet.py:67-68, 92-95).  Its layers have channel counts that are multiples of 12, not of 16.

All take ``adder2d_cls`` to build the same network around another implementation of the layer (the tests do
this with their CPU reference), and ``fused=False`` to build it from stock ``nn.BatchNorm2d`` / ``nn.ReLU``
modules exactly as the reference's model files do -- the adder layers are then the only thing that differs
from the reference.  With ``fused=True`` the BatchNorm layers are ``BatchNormAct2d`` (same parameters, buffers
and keys) and take their statistics from the adder kernels' epilogue.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from . import adder as _adder
from .bn_act import BatchNormAct2d
from .resnet20 import BasicBlock

_conv_bn = BasicBlock._conv_bn   # conv -> BatchNorm (+ residual) (+ ReLU), statistics from the conv's epilogue


def _bn(channels, relu, fused):
    return BatchNormAct2d(channels, relu=relu) if fused else nn.BatchNorm2d(channels)


class Bottleneck(nn.Module):
    expansion = 4

    def __init__(self, inplanes, planes, stride=1, downsample=None, adder2d_cls=None, fused=True, **adder_kw):
        super().__init__()
        make = adder2d_cls or _adder.adder2d
        self.fused = fused
        self.conv1 = make(inplanes, planes, kernel_size=1, stride=1, padding=0, bias=False, **adder_kw)
        self.bn1 = _bn(planes, True, fused)
        self.conv2 = make(planes, planes, kernel_size=3, stride=stride, padding=1, bias=False, **adder_kw)
        self.bn2 = _bn(planes, True, fused)
        self.conv3 = make(planes, planes * self.expansion, kernel_size=1, stride=1, padding=0, bias=False, **adder_kw)
        self.bn3 = _bn(planes * self.expansion, True, fused)
        self.relu = nn.ReLU(inplace=True)
        self.downsample = downsample
        self.stride = stride

    def forward(self, x):
        if not self.fused:   # the reference's own sequence of modules (resnet50.py:35-56)
            identity = x
            out = self.relu(self.bn1(self.conv1(x)))
            out = self.relu(self.bn2(self.conv2(out)))
            out = self.bn3(self.conv3(out))
            if self.downsample is not None:
                identity = self.downsample(x)
            out = out + identity
            return self.relu(out)
        if self.bn1.training and x.is_cuda and x.requires_grad and hasattr(self.conv1, "forward_with_stats"):
            # the shortcut leaves through conv1's autograd node, see BasicBlock.forward
            out, stats, shortcut = self.conv1.forward_with_stats(x, with_shortcut=True)
            out = self.bn1(out, stats=stats)
        else:
            out, shortcut = _conv_bn(self.conv1, self.bn1, x), x
        out = _conv_bn(self.conv2, self.bn2, out)
        if self.downsample is not None:
            shortcut = _conv_bn(self.downsample[0], self.downsample[1], shortcut)
        return _conv_bn(self.conv3, self.bn3, out, shortcut)       # bn + residual + relu


class ResNet50(nn.Module):
    def __init__(self, layers=(3, 4, 6, 3), num_classes=1000, adder2d_cls=None, fused=True, **adder_kw):
        super().__init__()
        self._make, self._adder_kw, self.fused = adder2d_cls or _adder.adder2d, adder_kw, fused
        self.inplanes = 64
        self.conv1 = nn.Conv2d(3, 64, kernel_size=7, stride=2, padding=3, bias=False)
        self.bn1 = _bn(64, True, fused)
        self.relu = nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(kernel_size=3, stride=2, padding=1)
        self.layer1 = self._make_layer(64, layers[0])
        self.layer2 = self._make_layer(128, layers[1], stride=2)
        self.layer3 = self._make_layer(256, layers[2], stride=2)
        self.layer4 = self._make_layer(512, layers[3], stride=2)
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Conv2d(512 * Bottleneck.expansion, num_classes, 1)
        self.bn2 = nn.BatchNorm2d(num_classes)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out", nonlinearity="relu")
            elif isinstance(m, nn.BatchNorm2d):
                nn.init.ones_(m.weight)
                nn.init.zeros_(m.bias)

    def _make_layer(self, planes, blocks, stride=1):
        downsample = None
        if stride != 1 or self.inplanes != planes * Bottleneck.expansion:
            downsample = nn.Sequential(
                self._make(self.inplanes, planes * Bottleneck.expansion, kernel_size=1, stride=stride, bias=False,
                           **self._adder_kw),
                _bn(planes * Bottleneck.expansion, False, self.fused))
        stage = [Bottleneck(self.inplanes, planes, stride, downsample, adder2d_cls=self._make, fused=self.fused,
                            **self._adder_kw)]
        self.inplanes = planes * Bottleneck.expansion
        stage += [Bottleneck(self.inplanes, planes, adder2d_cls=self._make, fused=self.fused, **self._adder_kw)
                  for _ in range(1, blocks)]
        return nn.Sequential(*stage)

    def forward(self, x):
        x = self.bn1(self.conv1(x))
        if not self.fused:
            x = self.relu(x)
        x = self.maxpool(x)
        x = self.layer4(self.layer3(self.layer2(self.layer1(x))))
        x = self.bn2(self.fc(self.avgpool(x)))
        return x.view(x.size(0), -1)


def resnet50(**kwargs):
    """resnet50.py:117-119."""
    return ResNet50((3, 4, 6, 3), **kwargs)


class VGGSmall(nn.Module):
    cfg = (128, 128, "M", 256, 256, "M", 512, 512, "M")

    def __init__(self, num_classes=10, adder2d_cls=None, fused=True, first_adder=False, **adder_kw):
        super().__init__()
        make = adder2d_cls or _adder.adder2d
        self.fused = fused
        layers, channels = [], 3
        for v in self.cfg:
            if v == "M":
                layers.append(nn.MaxPool2d(kernel_size=2, stride=2))
                continue
            if channels == 3 and not first_adder:
                conv = nn.Conv2d(3, v, kernel_size=3, padding=1, bias=False)
            else:
                conv = make(channels, v, kernel_size=3, stride=1, padding=1, bias=False, **adder_kw)
            layers += [conv, _bn(v, True, fused)]
            if not fused:
                layers.append(nn.ReLU(inplace=False))
            channels = v
        self.features = nn.Sequential(*layers)
        self.classifier = nn.Linear(512 * 4 * 4, num_classes)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out", nonlinearity="relu")

    def forward(self, x):
        if not self.fused:
            x = self.features(x)
        else:
            mods = list(self.features)
            i = 0
            while i < len(mods):
                if isinstance(mods[i], nn.MaxPool2d):
                    x, i = mods[i](x), i + 1
                else:
                    x, i = _conv_bn(mods[i], mods[i + 1], x), i + 2   # conv, BatchNorm + ReLU
        return self.classifier(x.reshape(x.size(0), -1))


def vgg_small(**kwargs):
    return VGGSmall(**kwargs)


class _PreAct:
    """BatchNorm - ReLU in front of a layer: one fused module, or the stock BatchNorm followed by F.relu."""

    @staticmethod
    def make(channels, fused):
        return BatchNormAct2d(channels, relu=True) if fused else nn.BatchNorm2d(channels)


def _bn_relu(bn, x):
    return bn(x) if isinstance(bn, BatchNormAct2d) else F.relu(bn(x))


class DenseBottleneck(nn.Module):
    def __init__(self, in_planes, growth_rate, adder2d_cls=None, fused=True, **adder_kw):
        super().__init__()
        make = adder2d_cls or _adder.adder2d
        self.bn1 = _PreAct.make(in_planes, fused)
        self.conv1 = make(in_planes, 4 * growth_rate, kernel_size=1, bias=False, **adder_kw)
        self.bn2 = _PreAct.make(4 * growth_rate, fused)
        self.conv2 = make(4 * growth_rate, growth_rate, kernel_size=3, padding=1, bias=False, **adder_kw)

    def forward(self, x):
        y = self.conv1(_bn_relu(self.bn1, x))
        y = self.conv2(_bn_relu(self.bn2, y))
        return torch.cat([y, x], 1)


class Transition(nn.Module):
    def __init__(self, in_planes, out_planes, adder2d_cls=None, fused=True, **adder_kw):
        super().__init__()
        make = adder2d_cls or _adder.adder2d
        self.bn = _PreAct.make(in_planes, fused)
        self.conv = make(in_planes, out_planes, kernel_size=1, bias=False, **adder_kw)

    def forward(self, x):
        return F.avg_pool2d(self.conv(_bn_relu(self.bn, x)), 2)


class DenseNet(nn.Module):
    def __init__(self, num_block=(6, 12, 24, 16), growth_rate=12, reduction=0.5, num_classes=10, adder2d_cls=None,
                 fused=True, **adder_kw):
        super().__init__()
        self.growth_rate = growth_rate
        kw = dict(adder2d_cls=adder2d_cls, fused=fused, **adder_kw)
        planes = 2 * growth_rate
        self.conv1 = nn.Conv2d(3, planes, kernel_size=3, padding=1, bias=False)
        for i, blocks in enumerate(num_block, start=1):
            stage = []
            for _ in range(blocks):
                stage.append(DenseBottleneck(planes, growth_rate, **kw))
                planes += growth_rate
            setattr(self, f"dense{i}", nn.Sequential(*stage))
            if i < len(num_block):
                out_planes = int(math.floor(planes * reduction))
                setattr(self, f"trans{i}", Transition(planes, out_planes, **kw))
                planes = out_planes
        self.stages = len(num_block)
        self.bn = _PreAct.make(planes, fused)
        self.linear = nn.Linear(planes, num_classes)

    def forward(self, x):
        x = self.conv1(x)
        for i in range(1, self.stages + 1):
            x = getattr(self, f"dense{i}")(x)
            if i < self.stages:
                x = getattr(self, f"trans{i}")(x)
        x = F.avg_pool2d(_bn_relu(self.bn, x), 4)
        return self.linear(x.view(x.size(0), -1))


def densenet_cifar(**kwargs):
    """densenet.py:108-109."""
    return DenseNet((6, 12, 24, 16), growth_rate=12, **kwargs)
