"""ctypes binding of libaddernet_hip.so (the C ABI declared in include/addernet_hip.h)."""
import ctypes
import functools
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# ADDERNET_HIP_LIB: another build of the same library (a debug build, a tuning variant) instead of the in-tree one
LIB_PATH = os.environ.get("ADDERNET_HIP_LIB") or os.path.join(_HERE, "libaddernet_hip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `python addernetcuda_amd/build.py` "
        "(hipcc, gfx950). There is no fallback implementation.")

lib = ctypes.CDLL(LIB_PATH)

# adder_status of include/addernet_hip.h
ADDER_OK, ADDER_ERR_NULL_POINTER, ADDER_ERR_BAD_SHAPE, ADDER_ERR_TOO_LARGE = 0, -1, -2, -3
ADDER_ERR_WORKSPACE, ADDER_ERR_HIP, ADDER_ERR_ALIAS, ADDER_ERR_UNSUPPORTED = -4, -5, -6, -7

_i, _l, _f, _p, _sz = ctypes.c_int, ctypes.c_long, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t
_szp = ctypes.POINTER(ctypes.c_size_t)

_SIGNATURES = {
    "adder_strerror": (ctypes.c_char_p, [_i]),
    "adder_last_hip_error": (ctypes.c_char_p, []),
    "adder_abi_version": (_i, []),
    "adder_out_dim": (_i, [_i, _i, _i, _i]),
    "adder_conv2d_fwd_f32": (_i, [_p, _p, _p] + [_i] * 9 + [_p]),
    "adder_conv2d_fwd_stats_slots": (_i, [_i] * 9 + [ctypes.POINTER(ctypes.c_int)]),
    "adder_conv2d_fwd_pair_stats_f32": (_i, [_p] * 7 + [_i] * 10 + [_p]),
    "adder_conv2d_fwd_stats_f32": (_i, [_p, _p, _p, _p, _i] + [_i] * 9 + [_p]),
    "adder_plain_conv2d_fwd_f32": (_i, [_p, _p, _p, _p, _i] + [_i] * 9 + [_p]),
    "adder_conv2d_bwd_workspace_bytes": (_i, [_i] * 9 + [_szp]),
    "adder_conv2d_bwd_f32": (_i, [_p, _p, _p, _p, _p, _f, _p, _sz] + [_i] * 9 + [_p]),
    "adder_conv2d_bwd_add_f32": (_i, [_p, _p, _p, _p, _p, _p, _f, _p, _sz] + [_i] * 9 + [_p]),
    "adder_conv2d_fwd_bf16": (_i, [_p, _p, _p] + [_i] * 9 + [_p]),
    "adder_conv2d_bwd_bf16": (_i, [_p, _p, _p, _p, _p, _f, _p, _sz] + [_i] * 9 + [_p]),
    "adder_conv2d_bwd_noalloc_f32": (_i, [_p, _p, _p, _p, _p, _f] + [_i] * 9 + [_p]),
    "adder_col_fwd_f32": (_i, [_p, _p, _p, _i, _l, _i, _p]),
    "adder_col_bwd_workspace_bytes": (_i, [_i, _l, _i, _szp]),
    "adder_col_bwd_f32": (_i, [_p, _p, _p, _p, _p, _i, _l, _i, _p, _sz, _p]),
    "adder_col_gradw_f32": (_i, [_p, _p, _p, _p, _i, _l, _i, _p, _sz, _p]),
    "adder_col_gradx_f32": (_i, [_p, _p, _p, _p, _i, _l, _i, _p]),
    "adder_norm_scale_workspace_bytes": (_i, [_l, _szp]),
    "adder_grad_norm_scale_f32": (_i, [_p, _l, _f, _f, _p, _sz, _p]),
    "adder_conv2d_grad_w_staged_f32": (_i, [_p, _p, _p, _p, _f, _p, _sz] + [_i] * 9 + [_p, _p]),
    "adder_grad_w_finish_workspace_bytes": (_i, [_i, _p, _szp]),
    "adder_grad_w_finish_f32": (_i, [_i, _p, _p, _sz, _p]),
    "adder_norm_scale_batched_workspace_bytes": (_i, [_i, _szp]),
    "adder_grad_norm_scale_batched_f32": (_i, [_i, _p, _p, _p, _f, _p, _sz, _p]),
    "adder_bn_act_workspace_bytes": (_i, [_i, _i, _i, _szp]),
    "adder_bn_act_mask_words": (_i, [_i, _i, _i, _szp]),
    "adder_bn_act_fwd_f32": (_i, [_p] * 11 + [_f, _f, _i, _i, _i, _i, _p, _sz, _p]),
    "adder_bn_act_fwd_stats_f32": (_i, [_p] * 11 + [_f, _f, _i, _i, _i, _i, _p, _i, _p]),
    "adder_bn_act_bwd_f32": (_i, [_p] * 11 + [_i, _i, _i, _i, _p, _sz, _p]),
    "adder_conv2d_bwd_bn_slots": (_i, [_i] * 9 + [ctypes.POINTER(ctypes.c_int)]),
    "adder_conv2d_bwd_bn_f32": (_i, [_p, _p, _p, _p, _p, _p, _f, _p, _sz] + [_i] * 9 + [_p, _p]),
    "adder_conv2d_grad_w_staged_bn_f32": (_i, [_p, _p, _p, _p, _f, _p, _sz] + [_i] * 9 + [_p, _p, _p]),
    "adder_bn_bwd_coef_f32": (_i, [_p, _i, _p, _p, _p, ctypes.c_double, _p, _p, _p, _i, _p]),
    "adder_head_supported": (_i, [_i, _i, _i, _i]),
    "adder_head_fwd_f32": (_i, [_p] * 12 + [_f, _f, _i, _i, _i, _i, _p]),
    "adder_head_bwd_f32": (_i, [_p] * 12 + [_i, _i, _i, _i, _p]),
    "adder_cross_entropy_fwd_f32": (_i, [_p, _p, _p, _p, _i, _i, _p]),
    "adder_cross_entropy_bwd_f32": (_i, [_p, _p, _p, _p, _p, _i, _i, _p]),
    "adder_sgd_momentum_step_f32": (_i, [_i, _p, _p, _p, _p, _p, _f, _f, _f, _p]),
}
for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(lib, _name)
    _fn.restype, _fn.argtypes = _res, _args

EXPORTED = tuple(_SIGNATURES)


class GradWStage(ctypes.Structure):
    """adder_grad_w_stage of include/addernet_hip.h."""
    _fields_ = [("part", ctypes.c_void_p), ("sgpart", ctypes.c_void_p), ("w", ctypes.c_void_p),
                ("gw", ctypes.c_void_p), ("slots", ctypes.c_int), ("Co", ctypes.c_int), ("K", ctypes.c_int),
                ("fp64", ctypes.c_int), ("eta", ctypes.c_float)]


class BnLinks(ctypes.Structure):
    """adder_bn_links of include/addernet_hip.h."""
    _fields_ = [("out_x", ctypes.c_void_p), ("out_coef", ctypes.c_void_p), ("out_gy", ctypes.c_void_p),
                ("in_x", ctypes.c_void_p),
                ("in_mean", ctypes.c_void_p), ("in_rstd", ctypes.c_void_p), ("in_part", ctypes.c_void_p),
                ("in_slots", ctypes.c_int), ("in_relu", ctypes.c_int), ("in_gamma", ctypes.c_void_p),
                ("in_beta", ctypes.c_void_p), ("side_gy", ctypes.c_void_p), ("side_w", ctypes.c_void_p),
                ("out_part", ctypes.c_void_p), ("out_slots", ctypes.c_int), ("out_gamma", ctypes.c_void_p),
                ("out_mean", ctypes.c_void_p), ("out_rstd", ctypes.c_void_p), ("out_dgamma", ctypes.c_void_p),
                ("out_dbeta", ctypes.c_void_p)]


def check(status, what):
    """Turn a negative adder_status into the RuntimeError the reference's AT_ASSERTM would raise."""
    if status != 0:
        msg = lib.adder_strerror(status).decode()
        if status == ADDER_ERR_HIP:
            msg += ": " + lib.adder_last_hip_error().decode()
        raise RuntimeError(f"{what}: {msg}")


def require_gpu_bf16(t, name):
    """The same checks for an activation tensor of the optional bfloat16 storage mode."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != torch.bfloat16:
        raise RuntimeError(f"{name} must be bfloat16, got {t.dtype}")


def require_gpu_f32(t, name):
    """CHECK_INPUT of adder_cuda.cpp:33-35 (device + contiguity) plus the dtype the kernels assume."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if t.dtype != torch.float32:
        raise RuntimeError(f"{name} must be float32, got {t.dtype}")


def same_device(*tensors):
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError("all tensors must be on the same device")
    return dev


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device):
    """The current HIP stream of ``device`` as the integer handle the C ABI takes."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def ptr(t):
    """Device address of a tensor (None -> NULL) for a ``void *`` / ``float *`` argument."""
    return t.data_ptr() if t is not None else None


class on_device:
    """``with on_device(dev):`` makes ``dev`` the current HIP device for the launches inside, like
    ``torch.cuda.device`` but without touching the runtime when it already is (the usual case)."""
    __slots__ = ("index", "previous")

    def __init__(self, device):
        self.index = device.index

    def __enter__(self):
        self.previous = None
        if self.index is not None:
            current = torch.cuda.current_device()
            if current != self.index:
                self.previous = current
                torch.cuda.set_device(self.index)
        return self

    def __exit__(self, exc_type, exc, tb):
        if self.previous is not None:
            torch.cuda.set_device(self.previous)
        return False


@functools.lru_cache(maxsize=4096)
def _conv_dims(x_shape, w_shape, stride, padding):
    N, Ci, H, W = x_shape
    Co, Ciw, kh, kw = w_shape
    if Ci != Ciw:
        raise RuntimeError(f"input has {Ci} channels but the weight expects {Ciw}")
    Ho, Wo = lib.adder_out_dim(H, kh, padding, stride), lib.adder_out_dim(W, kw, padding, stride)
    if Ho <= 0 or Wo <= 0:
        raise RuntimeError(f"empty output for input {tuple(x_shape)}, kernel {kh}x{kw}, "
                           f"stride {stride}, padding {padding}")
    return (N, Ci, H, W, Co, kh, kw, stride, padding), Ho, Wo


def conv_dims(x_shape, w_shape, stride, padding):
    """(N, Ci, H, W, Co, kh, kw, stride, padding), Ho, Wo of a layer; the answers are cached per geometry."""
    return _conv_dims(tuple(x_shape), tuple(w_shape), stride, padding)


@functools.lru_cache(maxsize=4096)
def fwd_stats_slots(dims):
    """Slots of the forward's BatchNorm partial sums for this geometry (0: the kernel has no such epilogue)."""
    slots = ctypes.c_int(0)
    check(lib.adder_conv2d_fwd_stats_slots(*dims, ctypes.byref(slots)), "adder_conv2d_fwd_stats_slots")
    return slots.value


@functools.lru_cache(maxsize=4096)
def conv2d_bwd_workspace_bytes(dims):
    need = ctypes.c_size_t(0)
    check(lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)), "adder_conv2d_bwd_workspace_bytes")
    return need.value


def conv2d_bwd_workspace(dims, device):
    need = conv2d_bwd_workspace_bytes(dims)
    # torch's caching allocator hands out >=512-byte aligned blocks and is graph-capture safe
    return torch.empty(max(need, 256), dtype=torch.uint8, device=device), need


@functools.lru_cache(maxsize=4096)
def bn_act_sizes(N, C, HW):
    """(workspace bytes, sign-mask words) of the fused BatchNorm kernels for an (N, C, HW) tensor."""
    need, words = ctypes.c_size_t(0), ctypes.c_size_t(0)
    check(lib.adder_bn_act_workspace_bytes(N, C, HW, ctypes.byref(need)), "adder_bn_act_workspace_bytes")
    check(lib.adder_bn_act_mask_words(N, C, HW, ctypes.byref(words)), "adder_bn_act_mask_words")
    return need.value, words.value


@functools.lru_cache(maxsize=4096)
def bwd_bn_slots(dims):
    """Partial-sum slots of the backward kernels that take BatchNorm links for this geometry (0: none do)."""
    slots = ctypes.c_int(0)
    check(lib.adder_conv2d_bwd_bn_slots(*dims, ctypes.byref(slots)), "adder_conv2d_bwd_bn_slots")
    return slots.value
