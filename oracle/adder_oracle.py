"""Pure-PyTorch CPU restatement of the reference AdderNet operator.

TEST INFRASTRUCTURE ONLY -- the product path never imports this file.

Every function names the reference lines it follows (paths are relative to the
reference checkout):

* col-layout forward      adder_cuda/test_cuda.py:18-22, adder.py:55
* col-layout grad_W       adder_cuda/test_cuda.py:35-41, adder.py:70
* col-layout grad_X       adder_cuda/test_cuda.py:57-60, adder.py:74
* adaptive grad_W scaling adder.py:78
* im2col / layout glue    adder.py:22-41
* autograd wiring         adder.py:43-80
* nn.Module               adder.py:83-108

How each function is pinned (none of the reference's files carries golden
vectors, so the pins are mathematical; they live in tests/test_oracle_pins.py):

* col_forward   == -torch.cdist(W, X.T, p=1); brute-force fp64 loops; W=0 and
                   X=0 closed forms (the latter pins "padding is a zero tap").
* col_grad_w    == G @ X.T - W * G.sum(1) (GEMM identity), the first term being
                   torch.nn.grad.conv2d_weight through the unfold layout.
* col_grad_x    unsaturated regime == W.T @ G - X * G.sum(0); saturated regime
                   == -+G.sum(0); brute force.
* unfold layout == per-sample F.unfold, column index l*N + n; C oracle
                   (oracle/adder_oracle.c) indexes NCHW directly and must agree.
* eta_scale     ||result||_2 == eta*sqrt(numel); scale invariance; zero -> zero.
"""
import math

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd import Function

DEFAULT_ETA = 0.2  # adder.py:78 divides by 5


def _chunks(total, step):
    for s in range(0, total, step):
        yield s, min(total, s + step)


def _chunk_len(Co, K, budget_elems=1 << 25):
    return max(1, budget_elems // max(1, Co * K))


def col_forward(X_col, W_col):
    """out[co, nl] = -sum_k |W[co,k] - X[k,nl]|  (test_cuda.py:18-22, adder.py:55).

    Chunked over nl only to bound the (Co, K, chunk) temporary; the arithmetic
    per output element is the reference expression unchanged.
    """
    Co, K = W_col.shape
    NL = X_col.shape[1]
    out = torch.empty((Co, NL), dtype=X_col.dtype, device=X_col.device)
    step = _chunk_len(Co, K)
    for a, b in _chunks(NL, step):
        out[:, a:b] = -(W_col.unsqueeze(2) - X_col[:, a:b].unsqueeze(0)).abs().sum(1)
    return out


def col_grad_w(X_col, W_col, grad_output):
    """grad_W[co,k] = sum_nl (X[k,nl] - W[co,k]) * g[co,nl]  (test_cuda.py:35-41, adder.py:70)."""
    Co, K = W_col.shape
    NL = X_col.shape[1]
    acc = torch.zeros((Co, K), dtype=X_col.dtype, device=X_col.device)
    step = _chunk_len(Co, K)
    for a, b in _chunks(NL, step):
        acc += ((X_col[:, a:b].unsqueeze(0) - W_col.unsqueeze(2))
                * grad_output[:, a:b].unsqueeze(1)).sum(2)
    return acc


def col_grad_x(X_col, W_col, grad_output):
    """grad_X[k,nl] = sum_co clamp(W[co,k]-X[k,nl], -1, 1) * g[co,nl]  (test_cuda.py:57-60, adder.py:74).

    Written exactly as the reference writes it: -(X - W).clamp(-1, 1) * g.
    """
    Co, K = W_col.shape
    NL = X_col.shape[1]
    out = torch.empty((K, NL), dtype=X_col.dtype, device=X_col.device)
    step = _chunk_len(Co, K)
    for a, b in _chunks(NL, step):
        out[:, a:b] = (-(X_col[:, a:b].unsqueeze(0) - W_col.unsqueeze(2)).clamp(-1, 1)
                       * grad_output[:, a:b].unsqueeze(1)).sum(0)
    return out


def eta_scale(grad_W_col, eta=DEFAULT_ETA):
    """grad_W / max(||grad_W||_2, 1e-12) * sqrt(Co*K) * eta  (adder.py:78, eta = 1/5 there)."""
    n = grad_W_col.numel()
    return grad_W_col / grad_W_col.norm(p=2).clamp(min=1e-12) * math.sqrt(n) * eta


def out_size(h_x, h_filter, padding, stride):
    """int((h - k + 2p)/s + 1)  (adder.py:26-31)."""
    return int((h_x - h_filter + 2 * padding) / stride + 1)


def im2col(X, h_filter, stride, padding):
    """(N,C,H,W) -> (K, L*N) with column index l*N + n  (adder.py:32-33)."""
    n_x, d_x, h_x, w_x = X.shape
    h_out = out_size(h_x, h_filter, padding, stride)
    w_out = out_size(w_x, h_filter, padding, stride)
    X_col = F.unfold(X.reshape(1, -1, h_x, w_x), h_filter, dilation=1, padding=padding,
                     stride=stride).view(n_x, -1, h_out * w_out)
    X_col = X_col.permute(1, 2, 0).contiguous().view(X_col.size(1), -1)
    return X_col, h_out, w_out


def col2im(grad_X_col, x_shape, h_filter, stride, padding):
    """Adjoint of :func:`im2col` (what autograd does through adder.py:32-33): fold."""
    n_x, d_x, h_x, w_x = x_shape
    K = d_x * h_filter * h_filter
    g = grad_X_col.view(K, -1, n_x).permute(2, 0, 1).contiguous()  # (N, K, L)
    return F.fold(g, (h_x, w_x), h_filter, dilation=1, padding=padding, stride=stride)


def out_to_nchw(out_col, n_filters, h_out, w_out, n_x):
    """(Co, L*N) -> NCHW  (adder.py:38-39)."""
    return out_col.view(n_filters, h_out, w_out, n_x).permute(3, 0, 1, 2).contiguous()


def nchw_to_out_col(g):
    """Adjoint of :func:`out_to_nchw`: NCHW grad -> (Co, L*N)."""
    n_x, co, h_out, w_out = g.shape
    return g.permute(1, 2, 3, 0).contiguous().view(co, -1)


def conv2d_forward(X, W, stride=1, padding=0):
    """NCHW forward through the unfold path  (adder.py:22-41)."""
    n_filters, _, h_filter, _ = W.shape
    X_col, h_out, w_out = im2col(X, h_filter, stride, padding)
    out = col_forward(X_col, W.reshape(n_filters, -1))
    return out_to_nchw(out, n_filters, h_out, w_out, X.shape[0])


def conv2d_backward(grad_y, X, W, stride=1, padding=0, eta=DEFAULT_ETA):
    """NCHW backward through the unfold path: (grad_X, grad_W raw, grad_W scaled).

    grad_W raw/scaled follow adder.py:66-78; grad_X is fold(grad_X_col).
    ``eta=None`` or 0 leaves the third result equal to the raw gradient.
    """
    n_filters, _, h_filter, _ = W.shape
    X_col, _, _ = im2col(X, h_filter, stride, padding)
    W_col = W.reshape(n_filters, -1)
    g_col = nchw_to_out_col(grad_y)
    gw = col_grad_w(X_col, W_col, g_col)
    gx_col = col_grad_x(X_col, W_col, g_col)
    gx = col2im(gx_col, X.shape, h_filter, stride, padding)
    gws = eta_scale(gw, eta) if eta else gw
    return gx, gw.view_as(W), gws.view_as(W)


class adder(Function):
    """Same autograd contract as adder.py:43-80, arithmetic from the formulas above."""
    eta = DEFAULT_ETA

    @staticmethod
    def forward(ctx, W_col, X_col, eta=DEFAULT_ETA):
        ctx.save_for_backward(W_col, X_col)
        ctx.eta = eta
        return col_forward(X_col, W_col)

    @staticmethod
    def backward(ctx, grad_output):
        W_col, X_col = ctx.saved_tensors
        grad_W_col = col_grad_w(X_col, W_col, grad_output)
        grad_X_col = col_grad_x(X_col, W_col, grad_output)
        grad_W_col = eta_scale(grad_W_col, ctx.eta)
        return grad_W_col, grad_X_col, None


def adder2d_function(X, W, stride=1, padding=0, eta=DEFAULT_ETA):
    """adder.py:22-41 with the extension call replaced by the formulas."""
    n_filters, _, h_filter, _ = W.size()
    n_x = X.size(0)
    X_col, h_out, w_out = im2col(X, h_filter, stride, padding)
    W_col = W.view(n_filters, -1)
    out = adder.apply(W_col, X_col, eta)
    return out_to_nchw(out, n_filters, h_out, w_out, n_x)


class adder2d(nn.Module):
    """adder.py:83-108 (parameter names ``adder`` and ``b`` kept)."""

    def __init__(self, input_channel, output_channel, kernel_size, stride=1, padding=0,
                 bias=False, depth_wise=False, eta=DEFAULT_ETA):
        super().__init__()
        if depth_wise:
            raise NotImplementedError("depth_wise is not wired in the reference either (adder.py:29)")
        self.stride, self.padding = stride, padding
        self.input_channel, self.output_channel = input_channel, output_channel
        self.kernel_size, self.eta = kernel_size, eta
        self.adder = nn.Parameter(nn.init.normal_(
            torch.randn(output_channel, input_channel, kernel_size, kernel_size)))
        self.bias = bias
        if bias:
            self.b = nn.Parameter(nn.init.uniform_(torch.zeros(output_channel)))

    def forward(self, x):
        output = adder2d_function(x, self.adder, self.stride, self.padding, self.eta)
        if self.bias:
            output = output + self.b.unsqueeze(0).unsqueeze(2).unsqueeze(3)
        return output
