"""An adder layer, the BatchNorm behind it, the shortcut add and the ReLU as ONE autograd node.

The reference runs ``relu(bn(conv(x)) [+ shortcut])`` as four autograd nodes (resnet20.py:28-39).  The forward here
is the same two launches as ``adder2d.forward_with_stats`` + ``BatchNormAct2d`` (the BatchNorm statistics come out
of the adder kernel's epilogue).  What one node buys is the backward: the two passes of the BatchNorm backward
disappear into the adder kernels on either side of the BatchNorm.

    ... -> [adder A -> BatchNorm P -> + shortcut -> ReLU] -> [adder B -> BatchNorm Q -> ...] -> ...
                 unit U                                            unit V

* V's input-gradient kernel has x = U's output and its own result in registers: it writes
  dz = (grad_X + shortcut gradient) * [x > 0], which is the gradient of P's output before the ReLU and of the
  shortcut, together with P's per-channel partial sums of dz and dz * xhat (``BnLink``).
* U's backward is handed that very tensor by autograd, recognises it (``BnLink.claims``), and A's weight-gradient
  kernel adds the partial sums (which gives dgamma, dbeta and four coefficients per channel) and forms A's output
  gradient from (dz, A's output, coefficients) while staging it, leaving it in memory for A's input-gradient
  kernel.

Whenever the hand-over does not apply (autograd summed several gradients into a new tensor, the consumer is not
an adder layer with such kernels, the weights are frozen, a tensor is not 16-byte aligned) the node runs the
BatchNorm backward of bn_act.py and the plain adder backward: same results, two more passes.

What V returns as the gradient of U's output is dz, i.e. already zero where the ReLU was inactive.  That is what
back-propagation needs (U applies the same mask again); a hook on U's output sees the masked values.
"""
import torch
from torch.autograd import Function

from . import adder as _adder
from ._lib import require_gpu_f32, bwd_bn_slots, conv_dims
from .bn_act import BatchNormAct2d, bn_forward, bn_backward


def _engine_will_run(node):
    """Whether the autograd engine runs (or captures the input of) ``node`` in the backward pass that is under way;
    True when that cannot be told."""
    if node is None:
        return False
    try:
        return bool(torch._C._will_engine_execute_node(node))
    except Exception:   # not inside a backward pass, or a torch without this query
        return True


class _adder_bn_act(Function):
    @staticmethod
    def forward(ctx, X, W, gamma, beta, residual, running_mean, running_var, num_batches, momentum, eps, relu, stride,
                padding, eta, with_shortcut, in_link, side_weight, given):
        ctx.w_is_given = W.is_contiguous()
        X, W = X.contiguous(), W.contiguous()
        if residual is not None:
            residual = residual.contiguous()
        ctx.side = ctx.pair = None
        pair = None
        if given is not None:      # this layer's product came out of the launch of the 3x3 layer beside it
            conv_out, stats, ctx.pair = given
            dims = conv_dims(X.shape, W.shape, stride, padding)[0]
        else:
            if side_weight is not None and with_shortcut:
                pair = _adder.conv_forward_pair(X, W, side_weight, stride, padding)
            if pair is not None:
                conv_out, stats, out_side, stats_side, dims = pair
                ctx.side = ctx.pair = _adder.SideOutput(X, side_weight, out_side, stats_side)
            else:
                conv_out, stats, dims = _adder.conv_forward(X, W, stride, padding, True)
        y, mean, rstd, mask = bn_forward(conv_out, gamma, beta, residual, running_mean, running_var, num_batches,
                                         momentum, eps, relu, stats)
        ctx.save_for_backward(X, W, conv_out, y if relu and mask is None else None, gamma, mean, rstd, mask)
        ctx.dims, ctx.eta, ctx.relu, ctx.has_res = dims, eta, relu, residual is not None
        ctx.with_shortcut = with_shortcut
        ctx.in_link = in_link
        # (a layer without the kernels that take the link could not use what its consumer would prepare)
        ctx.out_link = (_adder.BnLink(conv_out, mean, rstd, gamma, relu, None if residual is not None else beta)
                        if bwd_bn_slots(dims) > 0 else None)
        ctx.set_materialize_grads(False)
        if with_shortcut:
            # X again, as an output of this node: see adder._adder_nchw.forward
            return y, X.view_as(X)
        return y

    @staticmethod
    def backward(ctx, dy, grad_short=None):
        X, W, conv_out, y, gamma, mean, rstd, mask = ctx.saved_tensors
        need_x, need_w = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        pair, ctx.pair = ctx.pair, None
        side = None
        if pair is not None and ctx.with_shortcut and pair.side_gy is not None:
            # the strided 1x1 layer beside this one has left its input gradient to this node
            side, pair.side_gy, pair.side_w = (pair.side_gy, pair.side_w), None, None
        if dy is None:   # only the shortcut output was used
            if side is not None and need_x:
                extra = _adder.side_input_grad(X, *side)
                grad_short = extra if grad_short is None else grad_short + extra
            return (grad_short,) + (None,) * 17
        dy = dy.contiguous()
        require_gpu_f32(dy, "grad_output")
        if grad_short is not None:
            grad_short = grad_short.contiguous()
        usable = _adder.bn_links_usable(ctx.dims, X, W, conv_out, dy, grad_short)
        out_link, in_link = ctx.out_link, ctx.in_link
        ctx.out_link = ctx.in_link = None
        if usable and need_w and out_link is not None and out_link.claims(dy):
            # dy is dz, written by the consumer's kernel together with this BatchNorm's sums
            gy, dres, dgamma, dbeta = dy, (dy if ctx.has_res else None), out_link.dgamma, out_link.dbeta
        else:
            gy, dres, dgamma, dbeta = bn_backward(dy, y, mask, conv_out, gamma, mean, rstd, ctx.relu, ctx.has_res)
            out_link = None
        if out_link is not None:
            out_link.dz = None   # (the tensor is kept alive by autograd for as long as it is needed)
        if not (usable and need_x and in_link is not None and X.data_ptr() == in_link.out_ptr):
            in_link = None
        if pair is not None and not ctx.with_shortcut and need_x and not _engine_will_run(ctx.next_functions[0][0]):
            # needs_input_grad is fixed when the graph is built; in this pass nothing upstream of this layer was asked
            # for (torch.autograd.grad(loss, [this layer's weight])): no input gradient, and nothing to hand over
            need_x = False
        if pair is not None and not ctx.with_shortcut and need_x and X.is_contiguous():
            # this is the 1x1 layer of the pair: its input gradient is left to the 3x3 layer's node, which runs next
            pair.side_gy, pair.side_w = gy.contiguous(), W
            need_x = False

            def collected(pair=pair):   # runs when this backward pass is over
                if pair.side_gy is not None:
                    pair.side_gy = pair.side_w = None
                    raise RuntimeError("adder_bn_act: the input gradient of a paired 1x1 layer was left to the 3x3 layer "
                                       "beside it, whose backward did not run in this pass (differentiate with respect "
                                       "to the block's input, not to the `shortcut` tensor between the two layers)")
            torch.autograd.Variable._execution_engine.queue_callback(collected)
        gx, gw = _adder.conv_backward(X, W, gy, grad_short, ctx.dims, ctx.eta, need_x, need_w, ctx.w_is_given,
                                      out_link=out_link, in_link=in_link, side=side)
        return (gx, gw, dgamma, dbeta, dres) + (None,) * 13


def adder_bn_act(conv, bn, x, residual=None, with_shortcut=False, side_conv=None):
    """``bn(conv(x)) [+ residual]`` followed by the ReLU of ``bn`` (a ``BatchNormAct2d``), as one autograd node where
    that is possible (training on the GPU, float32, an ``adder2d`` without bias), else as the separate modules.
    ``with_shortcut``: returns (out, shortcut) with ``shortcut`` = x routed through the node, so that a residual
    shortcut's gradient is added inside the input-gradient kernel.
    ``side_conv`` (with ``with_shortcut``): the strided 1x1 ``adder2d`` that is applied to ``shortcut`` next (the
    downsample layer of the block): where ``conv`` is a strided 3x3 layer its kernel computes that layer's output
    too, and the call of ``adder_bn_act(side_conv, ..., shortcut)`` finds it ready.  In the backward pass that
    layer's node then leaves its input gradient to this node (``adder.SideOutput``), whose strided input-gradient
    kernel adds it on the positions the 1x1 layer read -- so ``shortcut`` is for ``side_conv`` and nothing else:
    a gradient taken with respect to ``shortcut`` itself would miss that part."""
    ok = (isinstance(conv, _adder.adder2d) and isinstance(bn, BatchNormAct2d) and not conv.bias and bn._fusable(x)
          and torch.is_grad_enabled() and conv.adder.dtype == torch.float32
          and (residual is None or (residual.shape[1:] == (conv.output_channel,) + _out_hw(conv, x)
                                    and residual.shape[0] == x.shape[0] and residual.dtype == torch.float32
                                    and residual.device == x.device)))
    if not ok:
        if (not with_shortcut and residual is None and hasattr(conv, "forward_bn_act") and bn.training and x.is_cuda
                and torch.is_grad_enabled()):
            return conv.forward_bn_act(x, bn)   # an ordinary convolution with the same kernels (the stem of a network)
        if with_shortcut:
            if hasattr(conv, "forward_with_stats") and bn.training and x.is_cuda:
                out, stats, shortcut = conv.forward_with_stats(x, with_shortcut=True)
                return bn(out, residual=residual, stats=stats), shortcut
            return bn(conv(x), residual=residual), x
        if hasattr(conv, "forward_with_stats") and bn.training and x.is_cuda:
            out, stats = conv.forward_with_stats(x)
            return bn(out, residual=residual, stats=stats)
        return bn(conv(x), residual=residual)
    rm = bn.running_mean if bn.track_running_stats else None
    rv = bn.running_var if bn.track_running_stats else None
    nb = bn.num_batches_tracked if bn.track_running_stats else None
    side_weight = None
    if (with_shortcut and isinstance(side_conv, _adder.adder2d) and not side_conv.bias
            and side_conv.adder.dtype == torch.float32 and side_conv.adder.is_contiguous()):
        side_weight = side_conv.adder.detach()
    given = _adder.SideOutput.of(x, conv.adder, int(conv.stride), int(conv.padding)) if residual is None else None
    res = _adder_bn_act.apply(x, conv.adder, bn.weight.contiguous(), bn.bias.contiguous(), residual, rm, rv, nb,
                              bn.momentum, bn.eps, bn.relu, int(conv.stride), int(conv.padding), conv.eta,
                              bool(with_shortcut), _adder.BnLink.of(x), side_weight, given)
    out = res[0] if with_shortcut else res
    link = getattr(out.grad_fn, "out_link", None)
    if link is not None:
        link.attach(out)
    if with_shortcut:
        side = getattr(out.grad_fn, "side", None)
        if side is not None:
            out.grad_fn.side = None
            # (the node saw x; what travels on is its second output, another tensor object on the same memory)
            side.x_ptr, side.x_shape, side.x_version = res[1].data_ptr(), tuple(res[1].shape), res[1]._version
            side.w_ptr, side.w_version = side_conv.adder.data_ptr(), side_conv.adder._version
            res[1]._adder_side_output = side
    return res


def _out_hw(conv, x):
    k, s, p = conv.kernel_size, conv.stride, conv.padding
    return ((x.shape[2] - k + 2 * p) // s + 1, (x.shape[3] - k + 2 * p) // s + 1)
