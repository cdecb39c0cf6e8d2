"""CIFAR ResNet-20 AdderNet: the harness model for the adder-conv kernels.

Same architecture and state_dict keys as the reference's resnet20.py:7-97:
regular 3x3 stem conv (resnet20.py:49), three stages of three BasicBlocks at
16/32/64 channels whose convs are adder2d 3x3 pad 1 (resnet20.py:7-9,16-20),
adder2d 1x1 stride-2 + BatchNorm downsample on the first block of stages 2
and 3 (resnet20.py:66-70), 8x8 average pool, a regular 1x1 conv classifier
followed by BatchNorm (resnet20.py:55-57,89-93), BatchNorm weights 1 / biases 0
(resnet20.py:59-62).

``adder2d_cls`` lets a caller build the same network around another
implementation of the layer (the tests do this with their CPU reference).

The BatchNorm layers are ``BatchNormAct2d``: the same module as nn.BatchNorm2d
(parameters, buffers, state_dict keys) with the ReLU, and in the second half
of a block the residual add, folded into its GPU kernels.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F

from . import adder as _adder
from .bn_act import BatchNormAct2d, bn_forward, bn_backward
from .unit import adder_bn_act
from .head import head_applies, pool_fc_bn


class BasicBlock(nn.Module):
    expansion = 1

    def __init__(self, inplanes, planes, stride=1, downsample=None, adder2d_cls=None, fused=True, **adder_kw):
        super().__init__()
        make = adder2d_cls or _adder.adder2d
        self.fused = fused
        self.conv1 = make(inplanes, planes, kernel_size=3, stride=stride, padding=1, bias=False, **adder_kw)
        self.bn1 = BatchNormAct2d(planes, relu=True) if fused else nn.BatchNorm2d(planes)
        self.relu = nn.ReLU(inplace=True)    # fused: kept for the reference's module layout; the ReLUs run inside bn1 / bn2
        self.conv2 = make(planes, planes, kernel_size=3, stride=1, padding=1, bias=False, **adder_kw)
        self.bn2 = BatchNormAct2d(planes, relu=True) if fused else nn.BatchNorm2d(planes)
        self.downsample = downsample
        self.stride = stride

    def forward(self, x):
        if not self.fused:   # the module sequence of resnet20.py:28-39, stock torch modules around the adder layers
            residual = x
            out = self.relu(self.bn1(self.conv1(x)))
            out = self.bn2(self.conv2(out))
            if self.downsample is not None:
                residual = self.downsample(x)
            out += residual
            return self.relu(out)
        # every conv -> bn (-> + shortcut) -> relu group is one autograd node (unit.py): the BatchNorm statistics
        # come out of the adder kernel's epilogue, and in the backward pass the BatchNorm's own two passes are
        # folded into the adder kernels on either side of it
        if self.bn1.training and x.is_cuda and x.requires_grad:
            # x leaves conv1's node a second time and feeds the shortcut from there, so that the shortcut's
            # gradient is added to conv1's input gradient by the kernel that computes it, not by a launch of its own
            ds = self.downsample
            side = ds[0] if isinstance(ds, nn.Sequential) and len(ds) == 2 else None   # the strided 1x1 layer beside conv1
            out, shortcut = adder_bn_act(self.conv1, self.bn1, x, with_shortcut=True, side_conv=side)
        else:
            out, shortcut = adder_bn_act(self.conv1, self.bn1, x), x
        if self.downsample is not None:
            ds = self.downsample
            if isinstance(ds, nn.Sequential) and len(ds) == 2 and isinstance(ds[1], BatchNormAct2d):
                shortcut = adder_bn_act(ds[0], ds[1], shortcut)
            else:
                shortcut = ds(shortcut)
        return adder_bn_act(self.conv2, self.bn2, out, residual=shortcut)


class _conv2d_matrix_grad(torch.autograd.Function):
    """An ordinary convolution whose weight gradient comes from the adder library's matrix-core kernel."""

    @staticmethod
    def forward(ctx, x, w, stride, padding):
        x, w = x.contiguous(), w.contiguous()
        ctx.save_for_backward(x, w)
        ctx.conf = (stride, padding)
        ctx.set_materialize_grads(False)
        y, stats = _adder.plain_conv2d_forward(x, w, stride, padding)
        if y is None:   # no tiled kernel for this geometry
            y, stats = F.conv2d(x, w, None, stride, padding), None
        if stats is None:
            stats = torch.empty(0, device=x.device, dtype=torch.float64)
        ctx.mark_non_differentiable(stats)
        return y, stats

    @staticmethod
    def backward(ctx, gy, _unused=None):
        if gy is None:
            return None, None, None, None
        x, w = ctx.saved_tensors
        stride, padding = ctx.conf
        gx = gw = None
        if ctx.needs_input_grad[0]:
            gx = torch.nn.grad.conv2d_input(x.shape, w, gy, stride, padding)
        if ctx.needs_input_grad[1]:
            gw = _adder.conv2d_weight_grad(gy, x, w, stride, padding)
            if gw is None:
                gw = torch.nn.grad.conv2d_weight(x, w.shape, gy, stride, padding)
        return gx, gw, None, None


class _conv_bn_act(torch.autograd.Function):
    """``relu(bn(conv(x)))`` for an ordinary convolution as one autograd node, the counterpart of unit.py for the
    stem (resnet20.py:49-51, 81-83): when the adder layer that consumes the output has left the BatchNorm's
    backward sums (``BnLink``), the weight-gradient kernel forms the convolution's output gradient itself and the
    BatchNorm's two backward passes are not run.  The input is an image batch: no input gradient on that path."""

    @staticmethod
    def forward(ctx, x, w, gamma, beta, running_mean, running_var, num_batches, momentum, eps, relu, stride, padding):
        x, w = x.contiguous(), w.contiguous()
        conv_out, stats = _adder.plain_conv2d_forward(x, w, stride, padding)
        if conv_out is None:   # no tiled kernel for this geometry
            conv_out, stats = F.conv2d(x, w, None, stride, padding), None
        y, mean, rstd, mask = bn_forward(conv_out, gamma, beta, None, running_mean, running_var, num_batches, momentum,
                                         eps, relu, stats)
        ctx.save_for_backward(x, w, conv_out, y if relu and mask is None else None, gamma, mean, rstd, mask)
        ctx.conf, ctx.relu = (stride, padding), relu
        ctx.out_link = _adder.BnLink(conv_out, mean, rstd, gamma, relu, beta)
        return y

    @staticmethod
    def backward(ctx, dy):
        x, w, conv_out, y, gamma, mean, rstd, mask = ctx.saved_tensors
        stride, padding = ctx.conf
        dy = dy.contiguous()
        link, ctx.out_link = ctx.out_link, None
        gx = gw = dgamma = dbeta = None
        # (link is None on a second pass through a retained graph: the separate BatchNorm backward below)
        if (link is not None and not ctx.needs_input_grad[0] and ctx.needs_input_grad[1] and link.claims(dy)
                and all(t.data_ptr() % 16 == 0 for t in (x, conv_out, dy))):
            gw = _adder.conv2d_weight_grad(dy, x, w, stride, padding, out_link=link)   # None: not with this kernel
            if gw is not None:
                dgamma, dbeta = link.dgamma, link.dbeta
        if link is not None:
            link.dz = None
        if gw is None:
            gy, _, dgamma, dbeta = bn_backward(dy, y, mask, conv_out, gamma, mean, rstd, ctx.relu, False)
            if ctx.needs_input_grad[0]:
                gx = torch.nn.grad.conv2d_input(x.shape, w, gy, stride, padding)
            if ctx.needs_input_grad[1]:
                gw = _adder.conv2d_weight_grad(gy, x, w, stride, padding)
                if gw is None:
                    gw = torch.nn.grad.conv2d_weight(x, w.shape, gy, stride, padding)
        return gx, gw, dgamma, dbeta, None, None, None, None, None, None, None, None


class StemConv2d(nn.Conv2d):
    """``nn.Conv2d`` (resnet20.py:49) with the same parameters and state_dict; on the GPU in training its
    weight gradient -- a sum over N*H*W positions into 16 x 27 values, which the vendor library spends six
    launches and three layout changes on -- runs through the kernel that does the same reduction for the
    adder layers."""

    def forward(self, x):
        if not self._plain(x):
            return super().forward(x)
        return _conv2d_matrix_grad.apply(x, self.weight, self.stride[0], self.padding[0])[0]

    def _plain(self, x):
        return (x.is_cuda and x.dtype == torch.float32 and self.bias is None and self.groups == 1
                and self.dilation == (1, 1) and self.padding_mode == "zeros" and torch.is_grad_enabled()
                and self.stride[0] == self.stride[1] and isinstance(self.padding[0], int)
                and self.padding[0] == self.padding[1])

    def forward_bn_act(self, x, bn):
        """``bn(self(x))`` with the ReLU of ``bn`` (a ``BatchNormAct2d``) as one autograd node where that is possible
        (see ``_conv_bn_act``), else as the separate modules."""
        if not (self._plain(x) and isinstance(bn, BatchNormAct2d) and bn._fusable(x)):
            out, stats = self.forward_with_stats(x)
            return bn(out, stats=stats) if isinstance(bn, BatchNormAct2d) else bn(out)
        rm = bn.running_mean if bn.track_running_stats else None
        rv = bn.running_var if bn.track_running_stats else None
        nb = bn.num_batches_tracked if bn.track_running_stats else None
        out = _conv_bn_act.apply(x, self.weight, bn.weight.contiguous(), bn.bias.contiguous(), rm, rv, nb, bn.momentum,
                                 bn.eps, bn.relu, self.stride[0], self.padding[0])
        if out.grad_fn is not None and hasattr(out.grad_fn, "out_link"):
            out.grad_fn.out_link.attach(out)
        return out

    def forward_with_stats(self, x):
        """(output, stats) like ``adder2d.forward_with_stats``: the BatchNorm partial sums of the output from the
        kernel's epilogue, or None."""
        if not self._plain(x):
            return super().forward(x), None
        y, stats = _conv2d_matrix_grad.apply(x, self.weight, self.stride[0], self.padding[0])
        return y, (stats if stats.numel() else None)


class ResNet(nn.Module):
    def __init__(self, block, layers, num_classes=10, adder2d_cls=None, fused=True, **adder_kw):
        """``fused=False``: stock ``nn.Conv2d`` / ``nn.BatchNorm2d`` / ``nn.ReLU`` modules in the reference's own
        sequence (resnet20.py:28-39, 80-93), i.e. the reference's model file with only the adder layer exchanged."""
        super().__init__()
        self._make = adder2d_cls or _adder.adder2d
        self._adder_kw = adder_kw
        self.fused = fused
        self.inplanes = 16
        self.conv1 = (StemConv2d if fused else nn.Conv2d)(3, 16, kernel_size=3, stride=1, padding=1, bias=False)
        self.bn1 = BatchNormAct2d(16, relu=True) if fused else nn.BatchNorm2d(16)
        self.relu = nn.ReLU(inplace=True)
        self.layer1 = self._make_layer(block, 16, layers[0])
        self.layer2 = self._make_layer(block, 32, layers[1], stride=2)
        self.layer3 = self._make_layer(block, 64, layers[2], stride=2)
        self.avgpool = nn.AvgPool2d(8, stride=1)
        self.fc = nn.Conv2d(64 * block.expansion, num_classes, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(num_classes)
        for m in self.modules():
            if isinstance(m, nn.BatchNorm2d):
                nn.init.ones_(m.weight)
                nn.init.zeros_(m.bias)

    def _make_layer(self, block, planes, blocks, stride=1):
        downsample = None
        if stride != 1 or self.inplanes != planes * block.expansion:
            downsample = nn.Sequential(
                self._make(self.inplanes, planes * block.expansion, kernel_size=1, stride=stride, bias=False,
                           **self._adder_kw),
                BatchNormAct2d(planes * block.expansion, relu=False) if self.fused
                else nn.BatchNorm2d(planes * block.expansion))
        kw = dict(adder2d_cls=self._make, fused=self.fused, **self._adder_kw)
        stage = [block(self.inplanes, planes, stride, downsample, **kw)]
        self.inplanes = planes * block.expansion
        stage += [block(self.inplanes, planes, **kw) for _ in range(1, blocks)]
        return nn.Sequential(*stage)

    def forward(self, x):
        if not self.fused:   # resnet20.py:80-93
            x = self.relu(self.bn1(self.conv1(x)))
            x = self.avgpool(self.layer3(self.layer2(self.layer1(x))))
            x = self.bn2(self.fc(x))
            return x.view(x.size(0), -1)
        if self.bn1.training and x.is_cuda and hasattr(self.conv1, "forward_bn_act"):
            x = self.conv1.forward_bn_act(x, self.bn1)
        elif self.bn1.training and x.is_cuda and hasattr(self.conv1, "forward_with_stats"):
            x, stats = self.conv1.forward_with_stats(x)
            x = self.bn1(x, stats=stats)
        else:
            x = self.bn1(self.conv1(x))
        x = self.layer3(self.layer2(self.layer1(x)))
        if x.shape[2] == 8 and x.shape[3] == 8 and head_applies(x, self.fc, self.bn2):
            return pool_fc_bn(x, self.fc, self.bn2)   # AvgPool2d(8) of an 8x8 map, fc and bn2 in two launches
        if x.shape[2] == 8 and x.shape[3] == 8:
            x = x.mean(dim=(2, 3), keepdim=True)   # AvgPool2d(8) of an 8x8 map, as one reduction kernel
        else:
            x = self.avgpool(x)
        fc = self.fc
        if x.shape[2] == 1 and x.shape[3] == 1 and fc.kernel_size == (1, 1) and fc.bias is None and fc.groups == 1:
            # a 1x1 convolution of a 1x1 map is a matrix product; as F.linear its weight gradient is a plain GEMM,
            # where the vendor convolution's weight gradient adds its partial sums with atomics in an order that
            # changes from run to run (the only kernel of the training step whose result did)
            x = F.linear(x.flatten(1), fc.weight.flatten(1))[:, :, None, None]
        else:
            x = fc(x)
        x = self.bn2(x)
        return x.view(x.size(0), -1)


def resnet20(**kwargs):
    """resnet20.py:96-97."""
    return ResNet(BasicBlock, [3, 3, 3], **kwargs)
