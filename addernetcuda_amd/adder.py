"""Drop-in for the reference's ``adder.py``: ``adder2d``, ``adder2d_function`` and ``adder``.

``adder2d`` / ``adder2d_function`` keep the reference signatures (adder.py:22,
83-85) but run the fused NCHW kernels: no unfold, no permute copies, no fold,
and the adaptive grad_W scaling of adder.py:78 happens inside the backward
launch.  ``adder.apply(W_col, X_col)`` keeps the column-matrix contract of
adder.py:43-80 for callers that build X_col themselves.

Everything is float32, like the reference.  One optional mode deviates, and only when asked for by passing a
bfloat16 input: activations and their gradients stored as bfloat16, weights and all accumulation unchanged
(``_adder_nchw_bf16``).
"""
import ctypes
import math

import torch
import torch.nn as nn
from torch.autograd import Function

from . import adder_cuda
from ._lib import (lib, check, ptr, require_gpu_f32, require_gpu_bf16, same_device, stream_ptr, conv_dims,
                   conv2d_bwd_workspace, fwd_stats_slots, on_device, GradWStage, BnLinks, bwd_bn_slots,
                   ADDER_OK, ADDER_ERR_UNSUPPORTED)

DEFAULT_ETA = 0.2  # adder.py:78 divides by 5


class adder(Function):
    """Column-matrix autograd function, same contract as adder.py:43-80."""

    @staticmethod
    def forward(ctx, W_col, X_col, eta=DEFAULT_ETA):
        W_col, X_col = W_col.contiguous(), X_col.contiguous()
        ctx.save_for_backward(W_col, X_col)
        ctx.eta = eta
        output = torch.empty((W_col.size(0), X_col.size(1)), device=W_col.device, dtype=W_col.dtype)
        adder_cuda.ADDER_CONV(X_col, W_col, output)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        W_col, X_col = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_W_col = torch.zeros_like(W_col)
        grad_X_col = torch.zeros_like(X_col)
        adder_cuda.ADDER_BACKWARD(grad_output, X_col, W_col, grad_W_col, grad_X_col)
        if ctx.eta:
            dev = grad_W_col.device
            n = grad_W_col.numel()
            need = ctypes.c_size_t(0)
            check(lib.adder_norm_scale_workspace_bytes(n, ctypes.byref(need)), "adder_norm_scale_workspace_bytes")
            ws = torch.empty(need.value, dtype=torch.uint8, device=dev)
            with on_device(dev):
                check(lib.adder_grad_norm_scale_f32(ptr(grad_W_col), n, float(ctx.eta), 1e-12, ptr(ws), need.value,
                                                    stream_ptr(dev)), "adder_grad_norm_scale_f32")
        return grad_W_col, grad_X_col, None


# while a batched_eta_scaling() block is open: one entry per layer whose weight gradient is pending,
# (weight, eta, stage, workspace) -- stage / workspace are None where only the scaling is pending.
# A module global and not a thread-local: the block is entered on the caller's thread, while the backward nodes
# that append to it run on the autograd engine's device thread.
_eta_batch = None


class batched_eta_scaling:
    """``with batched_eta_scaling(): loss.backward()`` -- inside the block the adder layers only reduce their
    weight gradient to partial slabs (or, for layers without such a kernel, to the raw gradient), and the block's
    exit finishes all of them -- slab sums, ``- w * sum gy``, and the scaling of adder.py:78 -- in a few kernel
    launches in all instead of two or three per layer.  Until then ``weight.grad`` is allocated but not
    meaningful; after the block it holds what it would hold without it.

    It only takes over layers whose weight is a leaf with ``grad is None`` when their backward runs (the usual
    ``zero_grad(set_to_none=True)`` loop); all others are finished on the spot as always.  One backward pass
    per block.  If the block is left by an exception, the gradients of the layers it had taken over are set to
    None (they were never finished).  A weight with a gradient hook registered on it (``register_hook``,
    ``register_post_accumulate_grad_hook``) is not taken over either, so the hook sees the finished gradient.  Not
    for ``torch.autograd.grad``."""

    def __enter__(self):
        global _eta_batch
        if _eta_batch is not None:
            raise RuntimeError("batched_eta_scaling blocks do not nest")
        _eta_batch = []
        return self

    def __exit__(self, exc_type, exc, tb):
        global _eta_batch
        pending, _eta_batch = _eta_batch, None

        def drop_pending_gradients():
            # a staged weight's .grad is allocated memory whose slabs were never summed (or a raw, unscaled
            # gradient): it must not survive an exceptional exit, or a caller that catches the error and steps the
            # optimizer anyway would apply it
            for W, _, _, _ in pending:
                W.grad = None

        if exc_type is not None:
            drop_pending_gradients()
            return False
        by_device, staged = {}, {}
        for W, eta, stage, ws in pending:
            g = W.grad
            if g is None or g.dtype != torch.float32 or not g.is_contiguous():
                drop_pending_gradients()
                raise RuntimeError("batched_eta_scaling: a weight's .grad is missing or not a contiguous float32 "
                                   "tensor at the end of the block")
            if stage is None:
                by_device.setdefault(g.device, []).append((g, eta))
            else:
                stage.gw = g.data_ptr()   # autograd may have handed the gradient over in another tensor
                staged.setdefault(g.device, []).append(stage)
        for dev, stages in staged.items():
            with on_device(dev):
                for i in range(0, len(stages), 32):
                    chunk = stages[i:i + 32]
                    arr = (GradWStage * len(chunk))(*chunk)
                    need = ctypes.c_size_t(0)
                    check(lib.adder_grad_w_finish_workspace_bytes(len(chunk), arr, ctypes.byref(need)),
                          "adder_grad_w_finish_workspace_bytes")
                    ws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=dev)
                    check(lib.adder_grad_w_finish_f32(len(chunk), arr, ptr(ws), need.value, stream_ptr(dev)),
                          "adder_grad_w_finish_f32")
        for dev, items in by_device.items():
            with on_device(dev):
                for i in range(0, len(items), 64):
                    chunk = items[i:i + 64]
                    count = len(chunk)
                    ptrs = (ctypes.c_void_p * count)(*[g.data_ptr() for g, _ in chunk])
                    sizes = (ctypes.c_long * count)(*[g.numel() for g, _ in chunk])
                    etas = (ctypes.c_float * count)(*[float(eta) for _, eta in chunk])
                    need = ctypes.c_size_t(0)
                    check(lib.adder_norm_scale_batched_workspace_bytes(count, ctypes.byref(need)),
                          "adder_norm_scale_batched_workspace_bytes")
                    ws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=dev)
                    check(lib.adder_grad_norm_scale_batched_f32(count, ptrs, sizes, etas, 1e-12, ptr(ws), need.value,
                                                                stream_ptr(dev)), "adder_grad_norm_scale_batched_f32")
        return False


def _has_grad_hooks(W):
    """A weight somebody watches during the backward pass (``register_hook``, ``register_post_accumulate_grad_hook``):
    such a hook must see the finished gradient, so ``batched_eta_scaling`` leaves the layer to finish on the spot."""
    return bool(getattr(W, "_backward_hooks", None)) or bool(getattr(W, "_post_accumulate_grad_hooks", None))


def conv_forward(X, W, stride, padding, with_stats):
    """The forward launch shared by the autograd nodes: (out, stats or None, dims) for contiguous float32 GPU
    tensors.  ``stats`` are the per-channel partial sums of out and out**2 for the BatchNorm that follows
    (bn_act.py), where ``with_stats`` is set and the layer's kernel has that epilogue."""
    require_gpu_f32(X, "X")
    require_gpu_f32(W, "W")
    dev = same_device(X, W)
    dims, Ho, Wo = conv_dims(X.shape, W.shape, stride, padding)
    out = torch.empty((X.size(0), W.size(0), Ho, Wo), device=dev, dtype=torch.float32)
    stats = None
    with on_device(dev):
        slots = fwd_stats_slots(dims) if with_stats else 0
        if slots > 0:
            stats = torch.empty((W.size(0), slots, 2), device=dev, dtype=torch.float64)
            status = lib.adder_conv2d_fwd_stats_f32(ptr(X), ptr(W), ptr(out), ptr(stats), slots, *dims, stream_ptr(dev))
            if status == ADDER_ERR_UNSUPPORTED:   # e.g. tensors that are not 16-byte aligned: the kernel that sums was turned down
                stats, slots = None, 0
            else:
                check(status, "adder_conv2d_fwd_stats_f32")
        if slots <= 0:
            check(lib.adder_conv2d_fwd_f32(ptr(X), ptr(W), ptr(out), *dims, stream_ptr(dev)), "adder_conv2d_fwd_f32")
    return out, stats, dims


class SideOutput:
    """The output of a strided 1x1 layer that was computed by the strided 3x3 layer beside it (same input: the first
    layer and the downsample layer of a residual block that halves the map; ``adder_conv2d_fwd_pair_stats_f32``).
    Made by the 3x3 layer's node, attached to the tensor that carries x on to the 1x1 layer, and taken by that
    layer's node in place of its own forward launch if it is asked for exactly this product."""
    __slots__ = ("x_ptr", "x_shape", "x_version", "w_ptr", "w_version", "out", "stats", "side_gy", "side_w")

    def __init__(self, x, w, out, stats):
        self.x_ptr, self.x_shape, self.x_version = x.data_ptr(), tuple(x.shape), x._version
        self.w_ptr, self.w_version = w.data_ptr(), w._version
        self.out, self.stats = out, stats
        # backward: the 1x1 layer's node leaves its output gradient and weights here instead of computing its input
        # gradient, and the 3x3 layer's node, which runs after it, adds that gradient to its own (conv_backward)
        self.side_gy = self.side_w = None

    @staticmethod
    def of(x, w, stride, padding):
        """(out, stats, the SideOutput) if ``x`` carries the product of exactly this 1x1 / stride-2 / pad-0 layer,
        else None."""
        side = getattr(x, "_adder_side_output", None)
        if (side is None or side.out is None or stride != 2 or padding != 0 or tuple(w.shape[2:]) != (1, 1)
                or side.x_ptr != x.data_ptr() or side.x_shape != tuple(x.shape) or side.x_version != x._version
                or side.w_ptr != w.data_ptr() or side.w_version != w._version or not w.is_contiguous()):
            return None
        out, stats = side.out, side.stats
        side.out = side.stats = None   # taken once
        return out, stats, side


def conv_forward_pair(X, W, W_side, stride, padding):
    """``conv_forward`` (with statistics) of a strided 3x3 layer and, in the same launch, of the strided 1x1 layer
    ``W_side`` on the same input: (out, stats, out_side, stats_side, dims), or None where that kernel does not apply
    (the caller then runs the two layers one after the other)."""
    if (stride != 2 or padding != 1 or tuple(W.shape[2:]) != (3, 3) or tuple(W_side.shape) != (W.size(0), W.size(1), 1, 1)
            or not W_side.is_cuda or W_side.dtype != torch.float32 or W_side.device != X.device):
        return None
    require_gpu_f32(X, "X")
    require_gpu_f32(W, "W")
    dev = same_device(X, W)
    dims, Ho, Wo = conv_dims(X.shape, W.shape, stride, padding)
    with on_device(dev):
        slots = fwd_stats_slots(dims)
        if slots <= 0:
            return None
        out = torch.empty((X.size(0), W.size(0), Ho, Wo), device=dev, dtype=torch.float32)
        out_side = torch.empty_like(out)
        stats = torch.empty((W.size(0), slots, 2), device=dev, dtype=torch.float64)
        stats_side = torch.empty_like(stats)
        status = lib.adder_conv2d_fwd_pair_stats_f32(ptr(X), ptr(W), ptr(W_side), ptr(out), ptr(out_side), ptr(stats),
                                                     ptr(stats_side), slots, *dims, stream_ptr(dev))
        if status == ADDER_ERR_UNSUPPORTED:
            return None
        check(status, "adder_conv2d_fwd_pair_stats_f32")
    return out, stats, out_side, stats_side, dims


class BnLink:
    """What passes between the backward of a layer and the BatchNorm on either side of it when the BatchNorm's
    backward is folded into the layer's kernels (``adder_bn_links`` of the C ABI; unit.py drives it).

    Made in the forward of the BatchNorm's node, which records the BatchNorm's input, statistics and weight; the
    layer that consumes the BatchNorm's output keeps a reference.  In the backward pass the consumer runs first:
    its input-gradient kernel leaves ``dz`` (the gradient of the BatchNorm's output before the ReLU) as its result
    and the partial sums of the BatchNorm's backward (``sums``, (C, slots, 2) float32).  The node of the BatchNorm,
    when it is handed exactly that ``dz`` tensor, skips its own two passes: the weight-gradient kernel of the layer
    in front of the BatchNorm adds the sums, forms its output gradient from them and fills ``dgamma`` / ``dbeta``."""
    __slots__ = ("bn_x", "mean", "rstd", "gamma", "beta", "beta_version", "relu", "out_ptr", "out_shape", "out_version", "dz",
                 "dz_version", "sums", "dgamma", "dbeta")

    def __init__(self, bn_x, mean, rstd, gamma, relu, beta=None):
        """``beta``: the BatchNorm's bias, given only when nothing was added to the BatchNorm's output (no residual):
        the consumer's kernel can then recover xhat from its own input instead of reading ``bn_x``."""
        self.bn_x, self.mean, self.rstd, self.gamma, self.beta, self.relu = bn_x, mean, rstd, gamma, beta, relu
        self.beta_version = None if beta is None else (beta._version, gamma._version)
        self.out_ptr = self.out_shape = self.out_version = None
        self.dz = self.dz_version = self.sums = self.dgamma = self.dbeta = None

    def attach(self, out):
        """Tie the link to the tensor that left the BatchNorm's node; consumers find it as ``out._adder_bn_link``."""
        self.out_ptr, self.out_shape, self.out_version = out.data_ptr(), tuple(out.shape), out._version
        out._adder_bn_link = self

    @staticmethod
    def of(x):
        """The link of the node that produced ``x``, if ``x`` still is what that node returned."""
        link = getattr(x, "_adder_bn_link", None)
        if (link is None or link.out_ptr != x.data_ptr() or link.out_shape != tuple(x.shape)
                or link.out_version != x._version or not x.is_contiguous()):
            return None
        return link

    def claims(self, dy):
        """Whether ``dy`` is the very tensor the consumer's kernel wrote (not a sum autograd formed from it)."""
        dz = self.dz
        return (dz is not None and self.sums is not None and dy.data_ptr() == dz.data_ptr() and dy.shape == dz.shape
                and dy._version == self.dz_version and dy.is_contiguous())

    def fill_out_half(self, links, gy_formed):
        """The out_* half of ``links`` (a BnLinks) for the layer in front of this BatchNorm."""
        links.out_x, links.out_gy = ptr(self.bn_x), ptr(gy_formed)
        links.out_part, links.out_slots = ptr(self.sums), self.sums.size(1)
        links.out_gamma, links.out_mean, links.out_rstd = ptr(self.gamma), ptr(self.mean), ptr(self.rstd)
        links.out_dgamma, links.out_dbeta = ptr(self.dgamma), ptr(self.dbeta)


def _aligned16(*tensors):
    return all(t is None or t.data_ptr() % 16 == 0 for t in tensors)


def side_input_grad(X, side_gy, side_w):
    """grad_X of the strided 1x1 / pad 0 layer ``side_w`` on X, from that layer's output gradient (its own kernel)."""
    dims1 = conv_dims(X.shape, side_w.shape, 2, 0)[0]
    gx = torch.empty_like(X)
    with on_device(X.device):
        check(lib.adder_conv2d_bwd_f32(ptr(side_gy), ptr(X), ptr(side_w), ptr(gx), None, 0.0, None, 0, *dims1,
                                       stream_ptr(X.device)), "adder_conv2d_bwd_f32")
    return gx


def conv_backward(X, W, grad_out, grad_short, dims, eta, need_x, need_w, w_is_given, out_link=None, in_link=None,
                  side=None):
    """The backward launches shared by the autograd nodes: (grad_X, grad_W), either None where not needed.

    ``grad_short``: a second gradient of X (a residual shortcut), added to grad_X by the kernel where it can.
    ``out_link``: a BnLink that ``claims`` grad_out -- ``grad_out`` is then dz of the BatchNorm behind the layer, and
    the weight-gradient kernel fills the link's dgamma / dbeta (the caller has checked ``bwd_bn_slots(dims)``, the
    alignment of the tensors and ``need_w``).
    ``in_link``: the BnLink of the BatchNorm whose output X is -- grad_X leaves as dz, and the link receives dz, the
    sums and empty dgamma / dbeta (same checks by the caller, and ``need_x``).
    ``side``: (side_gy, side_w) of the strided 1x1 layer that reads X beside this (strided 3x3) layer and has left its
    input gradient to this call: added inside the input-gradient kernel where that takes ``in_link``, else computed
    by the 1x1 layer's own kernel and added like ``grad_short``."""
    dev = X.device
    if side is not None and need_x:
        N, Ci, H, W_ = X.shape
        if not (in_link is not None and H % 2 == 0 and W_ % 2 == 0 and _aligned16(*side)
                and side[0].is_contiguous() and side[1].is_contiguous()):
            extra = side_input_grad(X, side[0].contiguous(), side[1].contiguous())
            grad_short = extra if grad_short is None else grad_short + extra
            side = None
    else:
        side = None
    gx = torch.empty_like(X) if need_x else None
    gw = torch.empty_like(W) if need_w else None
    eta = float(eta or 0.0)
    links = None
    part = slots = None
    if out_link is not None or in_link is not None:
        links = BnLinks()
        if out_link is not None:
            gy_formed = torch.empty_like(grad_out)
            out_link.fill_out_half(links, gy_formed)
        if in_link is not None:
            slots = bwd_bn_slots(dims)
            part = torch.empty((X.size(1), slots, 2), device=dev, dtype=torch.float32)
            links.in_x, links.in_mean, links.in_rstd = ptr(in_link.bn_x), ptr(in_link.mean), ptr(in_link.rstd)
            links.in_part, links.in_slots, links.in_relu = ptr(part), slots, int(in_link.relu)
            if in_link.beta is not None and in_link.beta_version == (in_link.beta._version, in_link.gamma._version):
                links.in_gamma, links.in_beta = ptr(in_link.gamma), ptr(in_link.beta)
            if side is not None:
                links.side_gy, links.side_w = ptr(side[0]), ptr(side[1])
    if _eta_batch is not None and need_w and any(W is entry[0] for entry in _eta_batch):
        raise RuntimeError("batched_eta_scaling: this weight already has a pending gradient in the block "
                           "(one backward pass per block, no weight shared between layers)")
    staged = False
    if (_eta_batch is not None and need_w and w_is_given and W.is_leaf and W.grad is None and not _has_grad_hooks(W)):
        with on_device(dev):
            ws, nbytes = conv2d_bwd_workspace(dims, dev)
            stage = GradWStage()
            if out_link is not None:
                status = lib.adder_conv2d_grad_w_staged_bn_f32(ptr(grad_out), ptr(X), ptr(W), ptr(gw), eta, ptr(ws), nbytes,
                                                               *dims, ctypes.byref(links), ctypes.byref(stage),
                                                               stream_ptr(dev))
            else:
                status = lib.adder_conv2d_grad_w_staged_f32(ptr(grad_out), ptr(X), ptr(W), ptr(gw), eta, ptr(ws), nbytes,
                                                            *dims, ctypes.byref(stage), stream_ptr(dev))
        if status == 0:      # slabs only; finished with all the others when the block ends
            _eta_batch.append((W, eta, stage, ws))
            staged = True
        elif status != ADDER_ERR_UNSUPPORTED or out_link is not None:
            check(status, "adder_conv2d_grad_w_staged_f32")
        elif eta > 0.0:      # no slab kernel for this layer: raw gradient now, scaled when the block ends
            _eta_batch.append((W, eta, None, None))
            eta = 0.0
    gw_out = gw
    if staged:
        gw = None
        if out_link is not None:   # the staged kernel has formed the gradient of the layer's output
            grad_out = gy_formed
            links.out_x = links.out_part = links.out_gy = None
    if need_x or gw is not None:
        with on_device(dev):
            ws, nbytes = conv2d_bwd_workspace(dims, dev) if gw is not None else (None, 0)
            if links is not None and (in_link is not None or links.out_x):
                check(lib.adder_conv2d_bwd_bn_f32(ptr(grad_out), ptr(X), ptr(W), ptr(grad_short), ptr(gx), ptr(gw), eta,
                                                  ptr(ws), nbytes, *dims, ctypes.byref(links), stream_ptr(dev)),
                      "adder_conv2d_bwd_bn_f32")
            else:
                fused = False
                if need_x and grad_short is not None:
                    status = lib.adder_conv2d_bwd_add_f32(ptr(grad_out), ptr(X), ptr(W), ptr(grad_short), ptr(gx),
                                                          ptr(gw), eta, ptr(ws), nbytes, *dims, stream_ptr(dev))
                    fused = status == 0
                    if status not in (ADDER_OK, ADDER_ERR_UNSUPPORTED):   # unsupported: this layer's grad_X kernel has no fused add
                        check(status, "adder_conv2d_bwd_add_f32")
                if not fused:
                    check(lib.adder_conv2d_bwd_f32(ptr(grad_out), ptr(X), ptr(W), ptr(gx), ptr(gw), eta, ptr(ws), nbytes,
                                                   *dims, stream_ptr(dev)), "adder_conv2d_bwd_f32")
                    if need_x and grad_short is not None:
                        gx += grad_short
            if in_link is not None:
                in_link.sums = part
                in_link.dgamma = torch.empty(X.size(1), device=dev, dtype=torch.float32)
                in_link.dbeta = torch.empty(X.size(1), device=dev, dtype=torch.float32)
                in_link.dz, in_link.dz_version = gx, gx._version
    return gx, gw_out


def bn_links_usable(dims, *tensors):
    """Whether the layer has the backward kernels that take BatchNorm links and the tensors suit them."""
    return bwd_bn_slots(dims) > 0 and _aligned16(*tensors)


class _adder_nchw(Function):
    """Fused NCHW forward / backward (replaces adder.py:22-41 + 43-80 in one step each)."""

    @staticmethod
    def forward(ctx, X, W, stride, padding, eta, with_stats=False, with_shortcut=False):
        ctx.w_is_given = W.is_contiguous()   # then the saved W is the caller's own tensor (its .grad is visible)
        X, W = X.contiguous(), W.contiguous()
        out, stats, dims = conv_forward(X, W, stride, padding, with_stats)
        dev = X.device
        ctx.save_for_backward(X, W)  # the NCHW input, not the 9x larger X_col the reference keeps
        ctx.dims, ctx.eta = dims, eta
        if not with_stats and not with_shortcut:
            return out
        ctx.set_materialize_grads(False)   # no zero-filled gradients for outputs nobody differentiates
        outputs = [out]
        if with_stats:
            if stats is None:   # no statistics epilogue for this shape: an empty tensor stands for "none"
                stats = torch.empty(0, device=dev, dtype=torch.float64)
            ctx.mark_non_differentiable(stats)
            outputs.append(stats)
        if with_shortcut:
            # X again, as an output of this node: what is back-propagated into it (a residual shortcut) reaches
            # backward() together with grad_out and is added to grad_X by the kernel that computes grad_X
            outputs.append(X.view_as(X))
        return tuple(outputs)

    @staticmethod
    def backward(ctx, grad_out, *more):
        # more: the (absent) gradient of the statistics and / or the gradient of the shortcut output
        grad_short = next((g for g in more if g is not None), None)
        if grad_out is None:
            return grad_short, None, None, None, None, None, None
        X, W = ctx.saved_tensors
        grad_out = grad_out.contiguous()
        require_gpu_f32(grad_out, "grad_output")
        if grad_short is not None:
            grad_short = grad_short.contiguous()
        gx, gw = conv_backward(X, W, grad_out, grad_short, ctx.dims, ctx.eta, ctx.needs_input_grad[0],
                               ctx.needs_input_grad[1], ctx.w_is_given)
        return gx, gw, None, None, None, None, None


class _adder_nchw_bf16(Function):
    """The optional reduced-storage mode: X, the output and their gradients are bfloat16 tensors (half the HBM
    traffic and activation memory), W and its gradient stay float32, and every sum is accumulated exactly as in the
    float32 path (fp32 for the output and grad_X, fp64 for grad_W); results are rounded to bfloat16 once, on the
    way out.  The reference has no such mode (adder.cu:310-318 is float only); it is chosen by passing a bfloat16
    input and is never a default."""

    @staticmethod
    def forward(ctx, X, W, stride, padding, eta):
        X, W = X.contiguous(), W.contiguous()
        require_gpu_bf16(X, "X")
        require_gpu_f32(W, "W")
        dev = same_device(X, W)
        dims, Ho, Wo = conv_dims(X.shape, W.shape, stride, padding)
        out = torch.empty((X.size(0), W.size(0), Ho, Wo), device=dev, dtype=torch.bfloat16)
        with on_device(dev):
            check(lib.adder_conv2d_fwd_bf16(ptr(X), ptr(W), ptr(out), *dims, stream_ptr(dev)), "adder_conv2d_fwd_bf16")
        ctx.save_for_backward(X, W)
        ctx.dims, ctx.eta = dims, eta
        return out

    @staticmethod
    def backward(ctx, grad_out):
        X, W = ctx.saved_tensors
        grad_out = grad_out.to(torch.bfloat16).contiguous()
        require_gpu_bf16(grad_out, "grad_output")
        dev = X.device
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        gx = torch.empty_like(X) if need_x else None
        gw = torch.empty_like(W) if need_w else None
        if need_x or need_w:
            with on_device(dev):
                ws, nbytes = conv2d_bwd_workspace(ctx.dims, dev) if need_w else (None, 0)
                check(lib.adder_conv2d_bwd_bf16(ptr(grad_out), ptr(X), ptr(W), ptr(gx), ptr(gw), float(ctx.eta or 0.0),
                                                ptr(ws), nbytes, *ctx.dims, stream_ptr(dev)), "adder_conv2d_bwd_bf16")
        return gx, gw, None, None, None


def plain_conv2d_forward(X, W, stride, padding):
    """An *ordinary* convolution ``F.conv2d(X, W, None, stride, padding)`` through the adder forward's tiled
    kernel (3x3 / stride 1 / pad 1), with the BatchNorm partial sums of its output: (y, stats), or (None, None)
    where the geometry has no such kernel."""
    require_gpu_f32(X, "X")
    require_gpu_f32(W, "W")
    dev = same_device(X, W)
    dims, Ho, Wo = conv_dims(X.shape, W.shape, stride, padding)
    with on_device(dev):
        slots = fwd_stats_slots(dims)
        y = torch.empty((X.size(0), W.size(0), Ho, Wo), device=dev, dtype=torch.float32)
        stats = torch.empty((W.size(0), slots, 2), device=dev, dtype=torch.float64) if slots else None
        status = lib.adder_plain_conv2d_fwd_f32(ptr(X), ptr(W), ptr(y), ptr(stats), slots, *dims, stream_ptr(dev))
    if status == ADDER_ERR_UNSUPPORTED:
        return None, None
    check(status, "adder_plain_conv2d_fwd_f32")
    return y, stats


def conv2d_weight_grad(grad_out, X, W, stride, padding, out_link=None):
    """Weight gradient of an *ordinary* convolution ``F.conv2d(X, W, None, stride, padding)``, i.e. the
    ``sum x * gy`` half of the adder layer's weight gradient, from the same fp64 matrix-core kernel (the slab
    finalize leaves the ``- w * sum gy`` term out).  Inside a ``batched_eta_scaling()`` block it is finished
    together with the adder layers' gradients.  Returns None where the geometry has no such kernel.
    ``out_link``: a BnLink that ``claims`` grad_out -- ``grad_out`` is then dz of the BatchNorm behind the
    convolution, and the kernel forms the convolution's output gradient from it and fills the link's dgamma / dbeta
    (None is returned, and nothing launched, where the kernel cannot)."""
    grad_out, X = grad_out.contiguous(), X.contiguous()
    require_gpu_f32(grad_out, "grad_output")
    require_gpu_f32(X, "X")
    dev = X.device
    dims, _, _ = conv_dims(X.shape, W.shape, stride, padding)
    gw = torch.empty(W.shape, device=dev, dtype=torch.float32)
    with on_device(dev):
        ws, nbytes = conv2d_bwd_workspace(dims, dev)
        stage = GradWStage()
        if out_link is not None:
            links = BnLinks()
            out_link.fill_out_half(links, None)
            status = lib.adder_conv2d_grad_w_staged_bn_f32(ptr(grad_out), ptr(X), None, ptr(gw), 0.0, ptr(ws), nbytes,
                                                           *dims, ctypes.byref(links), ctypes.byref(stage),
                                                           stream_ptr(dev))
        else:
            status = lib.adder_conv2d_grad_w_staged_f32(ptr(grad_out), ptr(X), None, ptr(gw), 0.0, ptr(ws), nbytes,
                                                        *dims, ctypes.byref(stage), stream_ptr(dev))
        if status == ADDER_ERR_UNSUPPORTED:
            return None
        check(status, "adder_conv2d_grad_w_staged_f32")
        if (_eta_batch is not None and W.is_leaf and W.grad is None and W.is_contiguous() and not _has_grad_hooks(W)
                and not any(W is entry[0] for entry in _eta_batch)):
            _eta_batch.append((W, 0.0, stage, ws))
            return gw
        arr = (GradWStage * 1)(stage)
        need = ctypes.c_size_t(0)
        check(lib.adder_grad_w_finish_workspace_bytes(1, arr, ctypes.byref(need)), "adder_grad_w_finish_workspace_bytes")
        fws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=dev)
        check(lib.adder_grad_w_finish_f32(1, arr, ptr(fws), need.value, stream_ptr(dev)), "adder_grad_w_finish_f32")
    return gw


def adder2d_function(X, W, stride=1, padding=0, eta=DEFAULT_ETA):
    """Same call as adder.py:22; ``eta`` (default 0.2 = the reference's /5) is the only addition."""
    if W.size(2) != W.size(3):
        # the reference passes only h_filter to unfold (adder.py:32): kernels are square
        raise RuntimeError("adder2d_function expects a square kernel")
    if X.dtype == torch.bfloat16:   # opt-in: bfloat16 activations, float32 weights and accumulation
        return _adder_nchw_bf16.apply(X, W if W.dtype == torch.float32 else W.float(), int(stride), int(padding), eta)
    return _adder_nchw.apply(X, W, int(stride), int(padding), eta)


def adder2d_function_with_stats(X, W, stride=1, padding=0, eta=DEFAULT_ETA, with_shortcut=False):
    """``adder2d_function`` that also returns the BatchNorm partial sums of its output, a float64 tensor
    (Co, slots, 2) for ``BatchNormAct2d(..., stats=)``, or None where the kernel has no such epilogue.
    ``with_shortcut``: a third result, X itself as an output of the layer's autograd node; use it as the
    residual shortcut and the shortcut's gradient is added to grad_X inside the grad_X kernel instead of
    by a separate autograd accumulation."""
    if W.size(2) != W.size(3):
        raise RuntimeError("adder2d_function expects a square kernel")
    res = _adder_nchw.apply(X, W, int(stride), int(padding), eta, True, bool(with_shortcut))
    out, stats = res[0], (res[1] if res[1].numel() else None)
    return (out, stats, res[2]) if with_shortcut else (out, stats)


class adder2d(nn.Module):
    """Same constructor and parameter names (``adder``, ``b``) as adder.py:83-108."""

    def __init__(self, input_channel, output_channel, kernel_size, stride=1, padding=0, bias=False,
                 depth_wise=False, eta=DEFAULT_ETA):
        super(adder2d, self).__init__()
        if depth_wise:
            # adder.py:94-95 builds a (Co,1,k,k) weight for this flag but adder2d_function never
            # honours it (adder.py:29 is commented out), so the reference fails on a shape mismatch
            raise NotImplementedError("depth_wise=True is not supported (it is not wired in the reference either)")
        self.stride = stride
        self.padding = padding
        self.input_channel = input_channel
        self.output_channel = output_channel
        self.kernel_size = kernel_size
        self.depth_wise = depth_wise
        self.eta = eta
        self.adder = torch.nn.Parameter(
            nn.init.normal_(torch.randn(output_channel, input_channel, kernel_size, kernel_size)))
        self.bias = bias
        if bias:
            self.b = torch.nn.Parameter(nn.init.uniform_(torch.zeros(output_channel)))

    def forward(self, x):
        output = adder2d_function(x, self.adder, self.stride, self.padding, self.eta)
        if self.bias:
            output = output + self.b.to(output.dtype).unsqueeze(0).unsqueeze(2).unsqueeze(3)
        return output

    def forward_with_stats(self, x, with_shortcut=False):
        """(output, stats): ``stats`` are the BatchNorm partial sums of the output for
        ``BatchNormAct2d.forward(..., stats=stats)``, or None (bias layers, shapes without the epilogue).
        ``with_shortcut``: (output, stats, shortcut) with ``shortcut`` = x routed through this layer's
        autograd node (see ``adder2d_function_with_stats``)."""
        if self.bias or x.dtype != torch.float32:   # (the statistics epilogue belongs to the float32 kernels)
            return (self.forward(x), None, x) if with_shortcut else (self.forward(x), None)
        return adder2d_function_with_stats(x, self.adder, self.stride, self.padding, self.eta, with_shortcut)

    def extra_repr(self):
        return (f"{self.input_channel}, {self.output_channel}, kernel_size={self.kernel_size}, "
                f"stride={self.stride}, padding={self.padding}, bias={self.bias}, eta={self.eta}")
