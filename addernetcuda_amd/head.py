"""The classifier head of the ResNets as one autograd node: ``bn(fc(avgpool(x)))`` of resnet20.py:89-93.

``AvgPool2d`` over the whole map, the bias-free 1x1 ``fc`` convolution (a matrix product on the 1x1 map that is
left) and the training-mode ``BatchNorm2d`` work on N x 64 and N x 10 values: the framework's own operators take
four launches of 5-10 us forward and four backward for them; csrc/head.hip takes two and two, with every sum in a
fixed order.  Anything the kernels do not cover (eval mode, CPU tensors, other dtypes, a map that is not pooled to
1x1, an ``fc`` with a bias) goes through the ordinary modules.
"""
import torch
from torch.autograd import Function

from ._lib import lib, check, ptr, stream_ptr, on_device


class _pool_fc_bn(Function):
    @staticmethod
    def forward(ctx, x, w, gamma, beta, running_mean, running_var, num_batches, momentum, eps):
        x, w = x.contiguous(), w.contiguous()
        N, C = x.shape[0], x.shape[1]
        HW = x.shape[2] * x.shape[3]
        J = w.shape[0]
        dev = x.device
        pooled = torch.empty((N, C), dtype=torch.float32, device=dev)
        z = torch.empty((N, J), dtype=torch.float32, device=dev)
        y = torch.empty((N, J), dtype=torch.float32, device=dev)
        mean = torch.empty(J, dtype=torch.float32, device=dev)
        rstd = torch.empty(J, dtype=torch.float32, device=dev)
        with on_device(dev):
            check(lib.adder_head_fwd_f32(ptr(x), ptr(w), ptr(gamma), ptr(beta), ptr(pooled), ptr(z), ptr(y), ptr(mean),
                                         ptr(rstd), ptr(running_mean), ptr(running_var), ptr(num_batches),
                                         float(momentum), float(eps), N, C, HW, J, stream_ptr(dev)),
                  "adder_head_fwd_f32")
        ctx.save_for_backward(pooled, z, w, gamma, mean, rstd)
        ctx.x_shape = tuple(x.shape)
        return y

    @staticmethod
    def backward(ctx, dy):
        pooled, z, w, gamma, mean, rstd = ctx.saved_tensors
        N, C, H, W = ctx.x_shape
        J = w.shape[0]
        dev = dy.device
        dy = dy.contiguous()
        if dy.dtype != torch.float32:
            raise RuntimeError("pool_fc_bn: grad_output must be float32")
        dz = torch.empty((N, J), dtype=torch.float32, device=dev)
        dx = torch.empty(ctx.x_shape, dtype=torch.float32, device=dev) if ctx.needs_input_grad[0] else None
        dw = torch.empty_like(w)
        dgamma, dbeta = torch.empty_like(gamma), torch.empty_like(gamma)
        with on_device(dev):
            check(lib.adder_head_bwd_f32(ptr(dy), ptr(z), ptr(pooled), ptr(w), ptr(gamma), ptr(mean), ptr(rstd), ptr(dz),
                                         ptr(dx), ptr(dw), ptr(dgamma), ptr(dbeta), N, C, H * W, J, stream_ptr(dev)),
                  "adder_head_bwd_f32")
        return dx, dw, dgamma, dbeta, None, None, None, None, None


def head_applies(x, fc, bn):
    """Whether ``pool_fc_bn`` has kernels for this input and these modules (else the caller runs the modules)."""
    if not (isinstance(fc, torch.nn.Conv2d) and isinstance(bn, torch.nn.BatchNorm2d)):
        return False
    if not (x.is_cuda and x.dtype == torch.float32 and x.dim() == 4 and torch.is_grad_enabled() and bn.training):
        return False
    if not (fc.kernel_size == (1, 1) and fc.stride == (1, 1) and fc.padding == (0, 0) and fc.bias is None
            and fc.groups == 1 and fc.dilation == (1, 1) and fc.weight.dtype == torch.float32
            and fc.weight.device == x.device and fc.in_channels == x.shape[1]):
        return False
    if not (bn.affine and bn.momentum is not None and bn.num_features == fc.out_channels
            and bn.weight.dtype == torch.float32 and bn.weight.device == x.device):
        return False
    N, C, H, W = x.shape
    return bool(lib.adder_head_supported(N, C, H * W, fc.out_channels))


def pool_fc_bn(x, fc, bn):
    """``bn(fc(mean of x over its map))`` as (N, classes), for modules and inputs that ``head_applies`` accepts."""
    rm = bn.running_mean if bn.track_running_stats else None
    rv = bn.running_var if bn.track_running_stats else None
    nb = bn.num_batches_tracked if bn.track_running_stats else None
    w = fc.weight.view(fc.out_channels, fc.in_channels)
    return _pool_fc_bn.apply(x, w, bn.weight.contiguous(), bn.bias.contiguous(), rm, rv, nb, bn.momentum, bn.eps)


class _cross_entropy(Function):
    @staticmethod
    def forward(ctx, logits, target):
        logits, target = logits.contiguous(), target.contiguous()
        N, J = logits.shape
        dev = logits.device
        loss = torch.empty((), dtype=torch.float32, device=dev)
        lse = torch.empty(N, dtype=torch.float32, device=dev)
        with on_device(dev):
            check(lib.adder_cross_entropy_fwd_f32(ptr(logits), ptr(target), ptr(loss), ptr(lse), N, J, stream_ptr(dev)),
                  "adder_cross_entropy_fwd_f32")
        ctx.save_for_backward(logits, target, lse)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        logits, target, lse = ctx.saved_tensors
        N, J = logits.shape
        dev = logits.device
        grad_loss = grad_loss.to(torch.float32).contiguous()
        grad = torch.empty_like(logits)
        with on_device(dev):
            check(lib.adder_cross_entropy_bwd_f32(ptr(logits), ptr(target), ptr(lse), ptr(grad_loss), ptr(grad), N, J,
                                                  stream_ptr(dev)), "adder_cross_entropy_bwd_f32")
        return grad, None


def cross_entropy(logits, target):
    """``torch.nn.functional.cross_entropy(logits, target)`` with its defaults (class indices, mean over the batch;
    main.py:66,90) -- in one launch each way for float32 GPU logits of at most 32 classes, else the framework's."""
    if (logits.is_cuda and logits.dtype == torch.float32 and logits.dim() == 2 and 0 < logits.shape[1] <= 32
            and logits.shape[0] > 0 and target.dtype == torch.int64 and target.dim() == 1
            and target.shape[0] == logits.shape[0] and target.device == logits.device):
        return _cross_entropy.apply(logits, target)
    return torch.nn.functional.cross_entropy(logits, target)
