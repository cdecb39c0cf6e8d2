"""The reference's other AdderNets as callers of ``adder2d``: ResNet-50, a VGG-small stack and the CIFAR DenseNet.

``resnet50`` has the architecture, parameter names and state_dict keys of the reference's resnet50.py:19-119:
a regular 7x7 stride-2 stem convolution, BatchNorm, ReLU and 3x3 max pooling (resnet50.py:63-67), four stages
of [3, 4, 6, 3] bottleneck blocks whose 1x1 / 3x3 / 1x1 convolutions are adder2d (resnet50.py:8-16, 19-33),
adder2d 1x1 + BatchNorm downsample on the first block of every stage (resnet50.py:84-90), global average
pooling, a regular 1x1 convolution classifier followed by BatchNorm (resnet50.py:72-74, 110-114).

``vgg11`` ... ``vgg19_bn`` (and the ``_nd`` / ``_nd_s`` / ``_nd_ss`` / ``vgg19_small_add`` variants) are the VGG family
of vgg.py:21-170 with its state_dict keys: all-adder features including the 3-channel first layer, five poolings,
the Linear(512) classifier stacks.  ``DenseNet121`` / ``169`` / ``201`` / ``161`` are densenet.py:93-106.

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
from .unit import adder_bn_act
from .resnet20 import StemConv2d   # nn.Conv2d with the same parameters; forward and weight gradient through the tiled kernels


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
        # every conv -> bn (-> + shortcut) -> relu group is one autograd node (unit.py), see BasicBlock.forward
        if self.bn1.training and x.is_cuda and x.requires_grad:
            out, shortcut = adder_bn_act(self.conv1, self.bn1, x, with_shortcut=True)
        else:
            out, shortcut = adder_bn_act(self.conv1, self.bn1, x), x
        out = adder_bn_act(self.conv2, self.bn2, out)
        if self.downsample is not None:
            shortcut = adder_bn_act(self.downsample[0], self.downsample[1], shortcut)
        return adder_bn_act(self.conv3, self.bn3, out, residual=shortcut)       # bn + residual + relu


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
                conv = (StemConv2d if fused else nn.Conv2d)(3, v, kernel_size=3, padding=1, bias=False)
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
                    x, i = adder_bn_act(mods[i], mods[i + 1], x), i + 2   # conv, BatchNorm + ReLU
        return self.classifier(x.reshape(x.size(0), -1))


def vgg_small(**kwargs):
    """The benchmark configuration "VGG-small-style AdderNet" (128-128-M-256-256-M-512-512-M, batch 128).  It is a
    harness for those layer shapes, not one of vgg.py's networks: its keys and its 8192-wide classifier match no
    reference VGG checkpoint -- for those use the ``vgg11`` ... ``vgg19_bn`` factories below."""
    return VGGSmall(**kwargs)


# ---- the VGG family of vgg.py ---------------------------------------------------------------------------
VGG_CFG = {   # vgg.py:75-81: channels per adder layer, "M" = 2x2 max pooling
    "A": (64, "M", 128, "M", 256, 256, "M", 512, 512, "M", 512, 512, "M"),
    "B": (64, 64, "M", 128, 128, "M", 256, 256, "M", 512, 512, "M", 512, 512, "M"),
    "D": (64, 64, "M", 128, 128, "M", 256, 256, 256, "M", 512, 512, 512, "M", 512, 512, 512, "M"),
    "E": (64, 64, "M", 128, 128, "M", 256, 256, 256, 256, "M", 512, 512, 512, 512, "M", 512, 512, 512, 512, "M"),
}


class VGG(nn.Module):
    """vgg.py:21-57 with the same module indices, hence the same state_dict keys (``features.<i>.adder``,
    ``features.<i+1>.weight`` ..., ``classifier.<j>.weight``): every convolution is an adder layer, the one on the
    3-channel image included (vgg.py:60-66); five poolings take a 32x32 input to 1x1 x 512; the classifier is
    [Dropout] - [Linear 512 - ReLU - [Dropout]] - [Linear 512 - ReLU] - Linear(512, classes) depending on
    ``dropout`` / ``small`` / ``supersmall`` (vgg.py:28-39).  ``fused``: the BatchNorm modules are
    ``BatchNormAct2d`` and run the ReLU that follows them (which stays in ``features`` as a placeholder)."""

    def __init__(self, cfg, num_classes=10, dropout=True, small=False, supersmall=False, batch_norm=True,
                 adder2d_cls=None, fused=True, **adder_kw):
        super().__init__()
        make = adder2d_cls or _adder.adder2d
        self.fused = fused and batch_norm
        layers, channels = [], 3
        for v in VGG_CFG[cfg] if isinstance(cfg, str) else cfg:
            if v == "M":
                layers.append(nn.MaxPool2d(kernel_size=2, stride=2))
                continue
            layers.append(make(channels, v, kernel_size=3, stride=1, padding=1, bias=False, **adder_kw))
            if batch_norm:
                layers.append(_bn(v, True, self.fused))
            layers.append(nn.ReLU(inplace=False))
            channels = v
        self.features = nn.Sequential(*layers)
        head = []
        if dropout or supersmall:
            head.append(nn.Dropout())
        if not (small or supersmall):
            head += [nn.Linear(512, 512), nn.ReLU()]
            if dropout:
                head.append(nn.Dropout())
        if not supersmall:
            head += [nn.Linear(512, 512), nn.ReLU()]
        head.append(nn.Linear(512, num_classes))
        self.classifier = nn.Sequential(*head)

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
                    x, i = adder_bn_act(mods[i], mods[i + 1], x), i + 3   # adder layer, BatchNorm + ReLU, (ReLU placeholder)
        return self.classifier(x.view(x.size(0), -1))


def _vgg_factory(cfg, doc, **fixed):
    def build(**kwargs):
        return VGG(cfg, **{**fixed, **kwargs})
    build.__doc__ = doc
    return build


# vgg.py:84-170 (every variant there builds its features with batch normalisation: make_layers' default)
vgg11 = _vgg_factory("A", "vgg.py:84-86")
vgg11_nd = _vgg_factory("A", "vgg.py:88-90", dropout=False)
vgg11_nd_s = _vgg_factory("A", "vgg.py:92-94", dropout=False, small=True)
vgg11_nd_ss = _vgg_factory("A", "vgg.py:96-98", dropout=False, small=True, supersmall=True)
vgg11_bn = _vgg_factory("A", "vgg.py:100-102")
vgg13 = _vgg_factory("B", "vgg.py:105-107")
vgg13_nd = _vgg_factory("B", "vgg.py:109-111", dropout=False)
vgg13_nd_s = _vgg_factory("B", "vgg.py:113-115", dropout=False, small=True)
vgg13_nd_ss = _vgg_factory("B", "vgg.py:117-119", dropout=False, small=True, supersmall=True)
vgg13_bn = _vgg_factory("B", "vgg.py:122-124")
vgg16 = _vgg_factory("D", "vgg.py:127-129")
vgg16_nd = _vgg_factory("D", "vgg.py:131-133", dropout=False)
vgg16_nd_s = _vgg_factory("D", "vgg.py:135-137", dropout=False, small=True)
vgg16_nd_ss = _vgg_factory("D", "vgg.py:139-141", dropout=False, small=True, supersmall=True)
vgg16_bn = _vgg_factory("D", "vgg.py:144-146")
vgg19 = _vgg_factory("E", "vgg.py:149-151")
vgg19_nd = _vgg_factory("E", "vgg.py:153-155", dropout=False)
vgg19_small_add = _vgg_factory("E", "vgg.py:157-159", dropout=False, small=True)
vgg19_nd_ss = _vgg_factory("E", "vgg.py:161-163", dropout=False, small=True, supersmall=True)
vgg19_bn = _vgg_factory("E", "vgg.py:168-170")


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
        self.conv1 = (StemConv2d if fused else nn.Conv2d)(3, planes, kernel_size=3, padding=1, bias=False)
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


def DenseNet121(**kwargs):
    """densenet.py:93-94."""
    return DenseNet((6, 12, 24, 16), growth_rate=32, **kwargs)


def DenseNet169(**kwargs):
    """densenet.py:97-98."""
    return DenseNet((6, 12, 32, 32), growth_rate=32, **kwargs)


def DenseNet201(**kwargs):
    """densenet.py:101-102."""
    return DenseNet((6, 12, 48, 32), growth_rate=32, **kwargs)


def DenseNet161(**kwargs):
    """densenet.py:105-106."""
    return DenseNet((6, 12, 36, 24), growth_rate=48, **kwargs)
