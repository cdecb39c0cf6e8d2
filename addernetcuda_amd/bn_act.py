"""BatchNorm2d fused with the residual add and ReLU that follow every adder layer.

``BatchNormAct2d`` is an ``nn.BatchNorm2d`` (same parameters, buffers and state_dict keys) whose
training-mode forward on the GPU runs as two HIP passes, statistics then
``relu(gamma * (x - mean) * rstd + beta [+ residual])``, and whose backward is two more; see
csrc/bn_act.hip.  It replaces the separate bn / += residual / relu ops of resnet20.py:28-39.
Anything the fused kernels do not cover (eval mode, CPU tensors, non-fp32) goes through the
ordinary torch ops with identical semantics.
"""
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd import Function

from ._lib import lib, check, ptr, stream_ptr, on_device, bn_act_sizes


def _workspace(N, C, HW, device):
    need = bn_act_sizes(N, C, HW)[0]
    return torch.empty(max(need, 256), dtype=torch.uint8, device=device), need


def bn_forward(x, weight, bias, residual, running_mean, running_var, num_batches, momentum, eps, relu, stats=None):
    """The forward launches shared by the autograd nodes: (y, mean, rstd, mask) for contiguous float32 GPU
    tensors; ``mask`` is the ReLU sign mask (None where the kernels have none for this shape)."""
    N, C = x.shape[0], x.shape[1]
    HW = x.numel() // (N * C)
    dev = x.device
    y = torch.empty_like(x)
    mean = torch.empty(C, dtype=torch.float32, device=dev)
    rstd = torch.empty(C, dtype=torch.float32, device=dev)
    # the backward needs y only for its sign: one bit per element where the kernels offer it
    mask = None
    if relu and all(t is None or t.data_ptr() % 16 == 0 for t in (x, y, residual)):
        words = bn_act_sizes(N, C, HW)[1]
        if words:
            mask = torch.empty(words, dtype=torch.int32, device=dev)
    with on_device(dev):
        if stats is not None:
            # the layer that produced x already summed x and x*x per channel (adder.forward_with_stats)
            if stats.dtype != torch.float64 or stats.dim() != 3 or stats.shape[0] != C or stats.shape[2] != 2 \
                    or not stats.is_contiguous() or stats.device != dev:
                raise RuntimeError("stats must be a contiguous float64 tensor (C, slots, 2) on the device of x")
            check(lib.adder_bn_act_fwd_stats_f32(ptr(x), ptr(residual), ptr(weight), ptr(bias), ptr(y), ptr(mask),
                                                 ptr(mean), ptr(rstd), ptr(running_mean), ptr(running_var), ptr(num_batches),
                                                 float(momentum), float(eps), int(relu), N, C, HW, ptr(stats),
                                                 int(stats.shape[1]), stream_ptr(dev)), "adder_bn_act_fwd_stats_f32")
        else:
            ws, nbytes = _workspace(N, C, HW, dev)
            check(lib.adder_bn_act_fwd_f32(ptr(x), ptr(residual), ptr(weight), ptr(bias), ptr(y), ptr(mask),
                                           ptr(mean), ptr(rstd), ptr(running_mean), ptr(running_var), ptr(num_batches),
                                           float(momentum), float(eps), int(relu), N, C, HW, ptr(ws), nbytes,
                                           stream_ptr(dev)), "adder_bn_act_fwd_f32")
    return y, mean, rstd, mask


def bn_backward(dy, y, mask, x, weight, mean, rstd, relu, has_res):
    """The two backward passes: (dx, dres or None, dgamma, dbeta); ``y`` is only read where there is no ``mask``."""
    N, C = x.shape[0], x.shape[1]
    HW = x.numel() // (N * C)
    dev = x.device
    dx = torch.empty_like(x)
    dres = torch.empty_like(x) if has_res else None
    dgamma, dbeta = torch.empty_like(weight), torch.empty_like(weight)
    if mask is not None and dy.data_ptr() % 16:
        dy = dy.clone()   # the masked kernels move float4 groups
    with on_device(dev):
        ws, nbytes = _workspace(N, C, HW, dev)
        check(lib.adder_bn_act_bwd_f32(ptr(dy), ptr(y), ptr(mask), ptr(x), ptr(weight), ptr(mean), ptr(rstd), ptr(dx),
                                       ptr(dres), ptr(dgamma), ptr(dbeta), int(relu), N, C, HW, ptr(ws), nbytes,
                                       stream_ptr(dev)), "adder_bn_act_bwd_f32")
    return dx, dres, dgamma, dbeta


class _bn_act(Function):
    @staticmethod
    def forward(ctx, x, weight, bias, residual, running_mean, running_var, num_batches, momentum, eps, relu,
                stats=None):
        x = x.contiguous()
        if residual is not None:
            residual = residual.contiguous()
        y, mean, rstd, mask = bn_forward(x, weight, bias, residual, running_mean, running_var, num_batches, momentum,
                                         eps, relu, stats)
        ctx.save_for_backward(x, y if relu and mask is None else None, weight, mean, rstd, mask)
        ctx.relu, ctx.has_res = relu, residual is not None
        return y

    @staticmethod
    def backward(ctx, dy):
        x, y, weight, mean, rstd, mask = ctx.saved_tensors
        dx, dres, dgamma, dbeta = bn_backward(dy.contiguous(), y, mask, x, weight, mean, rstd, ctx.relu, ctx.has_res)
        return dx, dgamma, dbeta, dres, None, None, None, None, None, None, None


class BatchNormAct2d(nn.BatchNorm2d):
    """``y = act(batch_norm(x) [+ residual])`` with ``act`` = ReLU when ``relu`` is set."""

    def __init__(self, num_features, relu=True, **kwargs):
        super().__init__(num_features, **kwargs)
        self.relu = relu

    def _fusable(self, x):
        # momentum=None (cumulative average) needs the batch count on the host: left to torch
        return (self.training and x.is_cuda and x.dtype == torch.float32 and self.affine and x.dim() == 4
                and self.weight.dtype == torch.float32 and self.momentum is not None)

    def forward(self, x, residual=None, stats=None):
        """``stats``: optional per-channel partial sums of x and x*x from the layer that produced x
        (``adder2d.forward_with_stats``); they replace this module's own statistics pass."""
        if not self._fusable(x):
            out = super().forward(x)
            if residual is not None:
                out = out + residual
            return F.relu(out) if self.relu else out
        rm = self.running_mean if self.track_running_stats else None
        rv = self.running_var if self.track_running_stats else None
        nb = self.num_batches_tracked if self.track_running_stats else None   # advanced inside the kernel
        weight, bias = self.weight.contiguous(), self.bias.contiguous()
        if residual is not None and (residual.shape != x.shape or residual.dtype != torch.float32
                                     or residual.device != x.device):
            # the kernels read the residual as a dense fp32 tensor shaped like x; anything else (a broadcast
            # shape, another dtype) is added the way the reference adds it (resnet20.py:37): BatchNorm alone
            # from the kernels, then torch's add and ReLU
            out = _bn_act.apply(x, weight, bias, None, rm, rv, nb, self.momentum, self.eps, False, stats) + residual
            return F.relu(out) if self.relu else out
        return _bn_act.apply(x, weight, bias, residual, rm, rv, nb, self.momentum, self.eps, self.relu, stats)
