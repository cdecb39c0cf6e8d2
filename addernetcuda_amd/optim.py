"""``torch.optim.SGD`` (main.py:67 of the reference: momentum 0.9, weight decay 5e-4) with the update of all
parameters of a group in one launch.

A network of adder layers has many small parameters (ResNet-20: 65 tensors, 272 000 values); the framework's
fused update takes two launches of 15 us for them, csrc/sgd.hip one of 5 us.  Same update rule, same
``state_dict`` (``momentum_buffer`` per parameter), same constructor; what the kernel does not cover (Nesterov,
dampening, ``maximize``, no momentum, parameters that are not contiguous float32 GPU tensors, sparse gradients) is
left to ``torch.optim.SGD.step``.  As with the framework's fused update, a float learning rate is frozen into a
captured graph; pass the rate as a one-element float32 device tensor to change it between replays.
"""
import ctypes

import torch

from ._lib import lib, check, stream_ptr, on_device

_MAX = 96   # ADDER_SGD_BATCH_MAX


class SGD(torch.optim.SGD):
    def __init__(self, params, lr=1e-3, momentum=0.0, dampening=0.0, weight_decay=0.0, nesterov=False, *,
                 maximize=False):
        super().__init__(params, lr=lr, momentum=momentum, dampening=dampening, weight_decay=weight_decay,
                         nesterov=nesterov, maximize=maximize, foreach=False, fused=False)

    @staticmethod
    def _kernel_takes(group, params):
        if group["momentum"] <= 0 or group["dampening"] != 0 or group["nesterov"] or group["maximize"]:
            return False
        lr = group["lr"]
        if isinstance(lr, torch.Tensor) and not (lr.is_cuda and lr.dtype == torch.float32 and lr.numel() == 1):
            return False
        dev = params[0].device
        for p in params:
            g = p.grad
            if not (p.is_cuda and p.device == dev and p.dtype == torch.float32 and p.is_contiguous()
                    and g.dtype == torch.float32 and g.device == dev and not g.is_sparse and g.is_contiguous()
                    and p.numel() > 0):
                return False
        return True

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        rest = []
        for group in self.param_groups:
            params = [p for p in group["params"] if p.grad is not None]
            if not params:
                continue
            if not self._kernel_takes(group, params):
                rest.append(group)
                continue
            bufs = []
            for p in params:
                state = self.state[p]
                if state.get("momentum_buffer") is None:
                    # (zeros: the first update then leaves buf = grad + weight_decay * p, as torch.optim.SGD does)
                    state["momentum_buffer"] = torch.zeros_like(p, memory_format=torch.contiguous_format)
                bufs.append(state["momentum_buffer"])
            lr = group["lr"]
            lr_ptr, lr_val = (lr.data_ptr(), 0.0) if isinstance(lr, torch.Tensor) else (None, float(lr))
            dev = params[0].device
            with on_device(dev):
                for i in range(0, len(params), _MAX):
                    ps, bs = params[i:i + _MAX], bufs[i:i + _MAX]
                    k = len(ps)
                    pa = (ctypes.c_void_p * k)(*[p.data_ptr() for p in ps])
                    ga = (ctypes.c_void_p * k)(*[p.grad.data_ptr() for p in ps])
                    ba = (ctypes.c_void_p * k)(*[b.data_ptr() for b in bs])
                    na = (ctypes.c_long * k)(*[p.numel() for p in ps])
                    check(lib.adder_sgd_momentum_step_f32(k, pa, ga, ba, na, lr_ptr, lr_val, float(group["momentum"]),
                                                          float(group["weight_decay"]), stream_ptr(dev)),
                          "adder_sgd_momentum_step_f32")
        if rest:   # the groups the kernel does not take: the framework's own update, group by group
            kept = self.param_groups
            try:
                self.param_groups = rest
                super().step()
            finally:
                self.param_groups = kept
        return loss
