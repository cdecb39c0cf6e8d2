"""ctypes front end for oracle/adder_oracle.c (TEST INFRASTRUCTURE ONLY).

Takes and returns torch CPU tensors; results are float64.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libadder_oracle.so")
_lib = None


def build(force=False):
    """Compile the C oracle with gcc (idempotent unless ``force``)."""
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(
            os.path.join(_HERE, "adder_oracle.c")):
        subprocess.check_call(["make", "-C", _HERE, "-B", "_build/libadder_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _fp(t):
    assert t.dtype == torch.float32 and t.is_contiguous() and t.device.type == "cpu"
    return ctypes.c_void_p(t.data_ptr())


def _dp(t):
    assert t.dtype == torch.float64 and t.is_contiguous()
    return ctypes.c_void_p(t.data_ptr())


def out_dim(h, k, p, s):
    return lib().oracle_out_dim(h, k, p, s)


def _dims(x, w, s, p):
    N, Ci, H, W = x.shape
    Co, Ci2, kh, kw = w.shape
    assert Ci == Ci2
    return [ctypes.c_int(v) for v in (N, Ci, H, W, Co, kh, kw, s, p)]


def conv2d_fwd(x, w, stride, padding):
    N, Ci, H, W = x.shape
    Co, _, kh, kw = w.shape
    y = torch.empty((N, Co, out_dim(H, kh, padding, stride), out_dim(W, kw, padding, stride)),
                    dtype=torch.float64)
    lib().oracle_conv2d_fwd(_fp(x), _fp(w), _dp(y), *_dims(x, w, stride, padding))
    return y


def conv2d_grad_w(gy, x, w, stride, padding):
    gw = torch.empty(w.shape, dtype=torch.float64)
    lib().oracle_conv2d_grad_w(_fp(gy), _fp(x), _fp(w), _dp(gw), *_dims(x, w, stride, padding))
    return gw


def conv2d_grad_x(gy, x, w, stride, padding):
    gx = torch.empty(x.shape, dtype=torch.float64)
    lib().oracle_conv2d_grad_x(_fp(gy), _fp(x), _fp(w), _dp(gx), *_dims(x, w, stride, padding))
    return gx


def eta_scale(g, eta):
    g = g.contiguous()
    out = torch.empty_like(g)
    lib().oracle_eta_scale(_dp(g), _dp(out), ctypes.c_size_t(g.numel()), ctypes.c_double(eta))
    return out


def col_fwd(X, W):
    K, NL = X.shape
    Co = W.shape[0]
    out = torch.empty((Co, NL), dtype=torch.float64)
    lib().oracle_col_fwd(_fp(X), _fp(W), _dp(out), ctypes.c_int(K), ctypes.c_long(NL), ctypes.c_int(Co))
    return out


def col_grad_w(g, X, W):
    K, NL = X.shape
    Co = W.shape[0]
    gw = torch.empty((Co, K), dtype=torch.float64)
    lib().oracle_col_grad_w(_fp(g), _fp(X), _fp(W), _dp(gw), ctypes.c_int(K), ctypes.c_long(NL), ctypes.c_int(Co))
    return gw


def col_grad_x(g, X, W):
    K, NL = X.shape
    Co = W.shape[0]
    gx = torch.empty((K, NL), dtype=torch.float64)
    lib().oracle_col_grad_x(_fp(g), _fp(X), _fp(W), _dp(gx), ctypes.c_int(K), ctypes.c_long(NL), ctypes.c_int(Co))
    return gx
