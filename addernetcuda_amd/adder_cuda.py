"""Drop-in for the reference's ``adder_cuda`` extension module.

Same four functions, same argument order, same in-place contract as the pybind
module of adder_cuda/adder_cuda.cpp:88-93: tensors are caller-allocated, ``out``
is overwritten, ``grad_W`` / ``grad_X`` are accumulated into (callers zero them
first, adder.py:66-67).  Where the reference asserts device and contiguity only
(adder_cuda.cpp:33-35) and aborts the process on unsupported sizes
(adder.cu:295-296, 437-438), these raise RuntimeError for every inconsistency
and accept any Co / K / NL.
"""
import ctypes

import torch

from . import _lib
from ._lib import lib, check, ptr, require_gpu_f32, same_device, stream_ptr, on_device


def _col_shapes(x, w, **others):
    if x.dim() != 2 or w.dim() != 2:
        raise RuntimeError("x must be (K, NL) and w must be (Co, K)")
    K, NL = x.shape
    Co, Kw = w.shape
    if Kw != K:
        raise RuntimeError(f"w has K={Kw} columns but x has K={K} rows")
    expect = {"y": (Co, NL), "grad_y": (Co, NL), "grad_w": (Co, K), "grad_i": (K, NL)}
    for name, t in others.items():
        if tuple(t.shape) != expect[name]:
            raise RuntimeError(f"{name} must have shape {expect[name]}, got {tuple(t.shape)}")
    return K, NL, Co


def _ws(K, NL, Co, device):
    need = ctypes.c_size_t(0)
    check(lib.adder_col_bwd_workspace_bytes(K, NL, Co, ctypes.byref(need)), "adder_col_bwd_workspace_bytes")
    if need.value == 0:
        return None, 0
    return torch.empty(need.value, dtype=torch.uint8, device=device), need.value


def ADDER_CONV(x, w, y):
    """y[co, nl] = -sum_k |w[co,k] - x[k,nl]|   (adder_cuda.cpp:37-46)."""
    for t, n in ((x, "x"), (w, "w"), (y, "y")):
        require_gpu_f32(t, n)
    dev = same_device(x, w, y)
    K, NL, Co = _col_shapes(x, w, y=y)
    with on_device(dev):
        check(lib.adder_col_fwd_f32(ptr(x), ptr(w), ptr(y), K, NL, Co, stream_ptr(dev)), "ADDER_CONV")


def ADDER_CONV_WEIGHT(grad_y, x, w, grad_w):
    """grad_w[co,k] += sum_nl (x[k,nl] - w[co,k]) * grad_y[co,nl]   (adder_cuda.cpp:48-59)."""
    for t, n in ((grad_y, "grad_y"), (x, "x"), (w, "w"), (grad_w, "grad_w")):
        require_gpu_f32(t, n)
    dev = same_device(grad_y, x, w, grad_w)
    K, NL, Co = _col_shapes(x, w, grad_y=grad_y, grad_w=grad_w)
    with on_device(dev):
        ws, nbytes = _ws(K, NL, Co, dev)
        check(lib.adder_col_gradw_f32(ptr(grad_y), ptr(x), ptr(w), ptr(grad_w), K, NL, Co, ptr(ws), nbytes,
                                      stream_ptr(dev)), "ADDER_CONV_WEIGHT")


def ADDER_CONV_INPUT(grad_y, x, w, grad_i):
    """grad_i[k,nl] += sum_co hardtanh(w[co,k] - x[k,nl]) * grad_y[co,nl]   (adder_cuda.cpp:61-72)."""
    for t, n in ((grad_y, "grad_y"), (x, "x"), (w, "w"), (grad_i, "grad_i")):
        require_gpu_f32(t, n)
    dev = same_device(grad_y, x, w, grad_i)
    K, NL, Co = _col_shapes(x, w, grad_y=grad_y, grad_i=grad_i)
    with on_device(dev):
        check(lib.adder_col_gradx_f32(ptr(grad_y), ptr(x), ptr(w), ptr(grad_i), K, NL, Co, stream_ptr(dev)),
              "ADDER_CONV_INPUT")


def ADDER_BACKWARD(grad_y, x, w, grad_w, grad_i):
    """Both gradients in one call   (adder_cuda.cpp:74-86)."""
    for t, n in ((grad_y, "grad_y"), (x, "x"), (w, "w"), (grad_w, "grad_w"), (grad_i, "grad_i")):
        require_gpu_f32(t, n)
    dev = same_device(grad_y, x, w, grad_w, grad_i)
    K, NL, Co = _col_shapes(x, w, grad_y=grad_y, grad_w=grad_w, grad_i=grad_i)
    with on_device(dev):
        ws, nbytes = _ws(K, NL, Co, dev)
        check(lib.adder_col_bwd_f32(ptr(grad_y), ptr(x), ptr(w), ptr(grad_w), ptr(grad_i), K, NL, Co, ptr(ws),
                                    nbytes, stream_ptr(dev)), "ADDER_BACKWARD")


__all__ = ["ADDER_CONV", "ADDER_CONV_WEIGHT", "ADDER_CONV_INPUT", "ADDER_BACKWARD"]
