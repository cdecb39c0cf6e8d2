"""adder_conv2d_bwd_noalloc_f32: the backward pass with its scratch inside the library's device image.

Called through the C ABI and held to the bar of the entry point it mirrors, adder_conv2d_bwd_f32: same
kernels, same fixed summation order, so both gradients must be bit-identical -- on two calls in a row, the
second on a smaller layer (the scratch then still holds the first call's slabs)."""
import ctypes

import pytest
import torch

from tests.util import make_case, assert_close


def _both(case, eta, gpu):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, conv_dims, check, conv2d_bwd_workspace
    s, p = case[6], case[7]
    x, w, gy = (t.to(gpu) for t in make_case(*case))
    dims, _, _ = conv_dims(x.shape, w.shape, s, p)
    st = stream_ptr(gpu)
    ws, nbytes = conv2d_bwd_workspace(dims, gpu)
    gx_a, gw_a = torch.full_like(x, float("nan")), torch.full_like(w, float("nan"))
    check(lib.adder_conv2d_bwd_f32(ptr(gy), ptr(x), ptr(w), ptr(gx_a), ptr(gw_a), eta, ptr(ws), nbytes, *dims, st),
          "adder_conv2d_bwd_f32")
    gx_b, gw_b = torch.full_like(x, float("nan")), torch.full_like(w, float("nan"))
    check(lib.adder_conv2d_bwd_noalloc_f32(ptr(gy), ptr(x), ptr(w), ptr(gx_b), ptr(gw_b), eta, *dims, st),
          "adder_conv2d_bwd_noalloc_f32")
    torch.cuda.synchronize()
    return (x, w, gy), (gx_a, gw_a), (gx_b, gw_b)


@pytest.mark.gpu
def test_two_calls_in_a_row_match_the_entry_point_with_a_workspace(gpu):
    from oracle import c_oracle, adder_oracle
    # (N, Ci, H, W, Co, k, stride, pad): a 3x3 layer on the matrix-core slab kernel, then a smaller one, then a
    # strided 1x1 layer (fp32 slabs) and a 5x5 layer (no slabs: only the norm partials use the scratch)
    for case, eta in (((8, 16, 32, 32, 16, 3, 1, 1), 0.2), ((3, 16, 16, 16, 8, 3, 1, 1), 0.1),
                      ((4, 16, 16, 16, 32, 1, 2, 0), 0.2), ((2, 3, 9, 9, 5, 5, 1, 2), 0.0)):
        (x, w, gy), (gx_a, gw_a), (gx_b, gw_b) = _both(case, eta, gpu)
        assert torch.equal(gx_a, gx_b), case
        assert torch.equal(gw_a, gw_b), case
        s, p = case[6], case[7]
        assert_close(gx_b, c_oracle.conv2d_grad_x(gy.cpu(), x.cpu(), w.cpu(), s, p), f"grad_X {case}")
        want = c_oracle.conv2d_grad_w(gy.cpu(), x.cpu(), w.cpu(), s, p)
        if eta:
            want = adder_oracle.eta_scale(want, eta)
        assert_close(gw_b, want, f"grad_W {case}")


@pytest.mark.gpu
def test_full_batch_resnet20_layer_fits_the_scratch(gpu):
    """The 16 -> 16 3x3 @32x32 layer at batch 256 is the largest workspace of ResNet-20 and must fit."""
    case = (256, 16, 32, 32, 16, 3, 1, 1)
    _, (gx_a, gw_a), (gx_b, gw_b) = _both(case, 0.1, gpu)
    assert torch.equal(gx_a, gx_b) and torch.equal(gw_a, gw_b)
    assert torch.isfinite(gw_b).all()


def test_layers_beyond_the_scratch_are_refused_before_any_launch():
    """Needs no GPU: the size check comes before the first HIP call."""
    from addernetcuda_amd._lib import lib
    P = ctypes.c_void_p
    gy, x, w, gx, gw = (P(a << 28) for a in range(1, 6))
    big = (128, 512, 8, 8, 512, 3, 3, 1, 1)              # VGG 512 -> 512: tens of MB of fp64 slabs
    need = ctypes.c_size_t()
    assert lib.adder_conv2d_bwd_workspace_bytes(*big, ctypes.byref(need)) == 0
    assert need.value > 8 << 20
    assert lib.adder_conv2d_bwd_noalloc_f32(gy, x, w, gx, gw, 0.2, *big, None) == -4
    assert lib.adder_strerror(-4) == b"workspace missing, misaligned or too small"
    assert lib.adder_conv2d_bwd_noalloc_f32(gy, x, w, None, None, 0.2, *big, None) == -1
    assert lib.adder_conv2d_bwd_noalloc_f32(None, x, w, gx, gw, 0.2, *big, None) == -1
