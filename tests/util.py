"""Seeded synthetic tensors shared by the tests (CPU float32)."""
import math

import torch

RTOL, ATOL = 1e-5, 1e-4  # the parity bar for forward and both gradients


def make_case(N, Ci, H, W, Co, k, stride, pad, seed=0, w_init="kaiming", x_scale=1.0):
    g = torch.Generator().manual_seed(1000 + seed)
    x = torch.randn(N, Ci, H, W, generator=g) * x_scale
    K = Ci * k * k
    if w_init == "kaiming":      # std = sqrt(2 / fan_in)
        w = torch.randn(Co, Ci, k, k, generator=g) * math.sqrt(2.0 / K)
    elif w_init == "normal":     # what adder2d itself draws (adder.py:97)
        w = torch.randn(Co, Ci, k, k, generator=g)
    else:                        # test_cuda.py:64-66 scales by 5
        w = torch.randn(Co, Ci, k, k, generator=g) * 5
    Ho = (H - k + 2 * pad) // stride + 1
    Wo = (W - k + 2 * pad) // stride + 1
    gy = torch.randn(N, Co, Ho, Wo, generator=g)
    return x, w, gy


def assert_close(actual, expected, what, rtol=RTOL, atol=ATOL):
    """allclose against a float64 truth, with a readable failure message."""
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    err = (a - e).abs()
    bound = atol + rtol * e.abs()
    bad = err > bound
    if bad.any():
        idx = torch.nonzero(bad)[0].tolist()
        raise AssertionError(
            f"{what}: {int(bad.sum())}/{bad.numel()} elements outside rtol={rtol} atol={atol}; "
            f"max abs err {err.max().item():.3e} (|ref| max {e.abs().max().item():.3e}); first at {idx}: "
            f"{a[tuple(idx)].item()} vs {e[tuple(idx)].item()}")
