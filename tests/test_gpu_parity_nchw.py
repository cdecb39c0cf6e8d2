"""HIP kernels (through the C ABI) against the CPU oracles, fused NCHW entry points.

Truth is the float64 plain-C oracle (oracle/adder_oracle.c); the tolerance is
the parity bar rtol 1e-5 / atol 1e-4.
"""
import ctypes

import pytest
import torch

from tests.util import make_case, assert_close

pytestmark = pytest.mark.gpu

# (N, Ci, H, W, Co, k, stride, pad)
TILED = [
    (3, 16, 32, 32, 16, 3, 1, 1),   # 32-wide tiled path
    (2, 32, 16, 16, 32, 3, 1, 1),   # 16-wide tiled path
    (5, 64, 8, 8, 64, 3, 1, 1),     # 8-wide tiled path, N not a multiple of the image group
    (2, 5, 12, 20, 7, 3, 1, 1),     # channel tails, H != W, partial tiles
    (1, 3, 9, 40, 4, 3, 1, 1),      # two tiles along W
    (2, 12, 8, 8, 12, 3, 1, 1),     # DenseNet-style 12 channels
    (2, 20, 12, 20, 12, 3, 1, 1),   # channel tails on the tiled path (Ci, Co not multiples of 8)
    (1, 24, 4, 4, 48, 3, 1, 1),     # map smaller than a tile
    (2, 16, 32, 32, 32, 3, 2, 1),   # ResNet-20 strided 3x3, 32 -> 16
    (3, 32, 16, 16, 64, 3, 2, 1),   # ResNet-20 strided 3x3, 16 -> 8
    (2, 6, 14, 24, 10, 3, 2, 1),    # strided, channel tails, partial tiles (Ho = 7, Wo = 12)
    (2, 5, 12, 20, 7, 3, 2, 1),     # strided, Wo = 10 (forward tiled, gradients generic)
    (2, 16, 14, 14, 16, 3, 1, 1),   # ResNet-50 14-wide maps: rows not float4-aligned, 16-wide tile
    (2, 16, 7, 7, 24, 3, 1, 1),     # 7-wide maps, 8-wide tile
    (1, 8, 30, 30, 8, 3, 1, 1),     # W = 30 on the 32-wide tile
    (2, 9, 10, 18, 8, 3, 1, 1),     # odd channel count and W = 18
    (2, 8, 28, 28, 16, 3, 2, 1),    # strided, Wo = 14
    (2, 16, 14, 14, 16, 3, 2, 1),   # strided, W = 14 -> Wo = 7
    (2, 8, 24, 40, 12, 3, 1, 1),    # wide map, 24 rows: tiles of 8 rows in four-wave workgroups
    (3, 8, 20, 24, 8, 3, 1, 1),     # wide map, 20 rows: tiles of 4 rows of two images, odd image count
    (2, 16, 56, 56, 8, 3, 1, 1),    # ResNet-50's 56x56 maps (7 x 8 rows)
    (3, 8, 28, 28, 8, 3, 1, 1),     # ... and 28x28 (7 x 4 rows)
    (5, 3, 32, 32, 16, 3, 1, 1),    # three input channels on a wide map (a stem's shape): the weight gradient's 32-column block
    (3, 2, 24, 36, 20, 3, 1, 1),    # ... two channels, channel tail on Co
    (2, 1, 32, 30, 8, 3, 1, 1),     # ... one channel, rows that are not whole float4 groups
    (2, 16, 32, 32, 32, 1, 2, 0),   # ResNet-20 1x1 stride-2 downsample
    (2, 32, 16, 16, 64, 1, 2, 0),   # second downsample
    (2, 8, 8, 8, 16, 1, 1, 0),      # 1x1 stride 1
    (3, 13, 12, 12, 9, 1, 2, 0),    # 1x1 stride 2 with channel tails
    (2, 9, 6, 12, 20, 1, 1, 0),     # 1x1 stride 1 with channel tails
    (3, 16, 14, 14, 24, 1, 1, 0),   # 1x1 on a 14x14 plane (walked as one row of 196)
    (3, 64, 14, 14, 72, 1, 1, 0),   # tiled 1x1 kernels (>= 64 channels): 196-position planes, channel tail on Co
    (5, 72, 7, 7, 64, 1, 1, 0),     # tiled 1x1, 49-position planes (four images per tile, N = 5), Ci = 72
    (2, 64, 20, 20, 64, 1, 1, 0),   # tiled 1x1, 400-position planes: several tiles per plane
    (2, 64, 28, 28, 72, 1, 2, 0),   # 1x1 stride 2 with many channels, Wo = 14
    (3, 68, 14, 14, 64, 1, 2, 0),   # 1x1 stride 2, W = 14 -> Wo = 7, Ci = 68
    (3, 12, 7, 7, 20, 1, 1, 0),     # 1x1 on a 7x7 plane: 49 elements, element-wise loads, partial last group
    (1, 5, 3, 5, 3, 1, 1, 0),       # 1x1, 15-element planes
    (2, 16, 14, 14, 24, 1, 2, 0),   # 1x1 stride 2, 14 -> 7 (ResNet-50's last downsample): odd output width
    (2, 6, 9, 9, 10, 1, 2, 0),      # 1x1 stride 2 on odd maps: the last column and row have no right / lower neighbour
    (2, 4, 6, 10, 8, 1, 2, 0),      # 1x1 stride 2, W = 10 (even, not a multiple of 4), Wo = 5
]
GENERIC = [
    (2, 4, 9, 9, 6, 3, 2, 1),       # strided 3x3, odd size
    (2, 3, 7, 7, 5, 3, 1, 1),       # W % 4 != 0
    (1, 4, 11, 9, 6, 5, 1, 2),      # 5x5
    (2, 3, 11, 9, 4, 3, 3, 2),      # stride 3, floor output size
    (1, 2, 16, 16, 3, 7, 2, 3),     # 7x7 stride 2
    (2, 4, 6, 6, 4, 3, 1, 0),       # no padding
    (1, 1, 1, 1, 1, 1, 1, 0),       # smallest possible
]


def _run_fwd(case, gpu, **kw):
    from addernetcuda_amd import adder
    x, w, gy = make_case(*case, **kw)
    y = adder.adder2d_function(x.to(gpu), w.to(gpu), case[6], case[7])
    torch.cuda.synchronize()
    return x, w, gy, y


@pytest.mark.parametrize("case", TILED + GENERIC, ids=str)
def test_forward_matches_oracle(case, gpu):
    from oracle import c_oracle
    x, w, gy, y = _run_fwd(case, gpu)
    assert_close(y, c_oracle.conv2d_fwd(x, w, case[6], case[7]), f"forward {case}")


@pytest.mark.parametrize("w_init", ["normal", "times5"])
def test_forward_other_weight_scales(w_init, gpu):
    from oracle import c_oracle
    case = (2, 16, 32, 32, 16, 3, 1, 1)
    x, w, gy, y = _run_fwd(case, gpu, w_init=w_init, x_scale=5.0 if w_init == "times5" else 1.0)
    assert_close(y, c_oracle.conv2d_fwd(x, w, 1, 1), f"forward {w_init}")


@pytest.mark.parametrize("case", TILED + GENERIC, ids=str)
def test_backward_matches_oracle(case, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle
    s, p = case[6], case[7]
    x, w, gy = make_case(*case)
    xg = x.to(gpu).requires_grad_(True)
    wg = w.to(gpu).requires_grad_(True)
    for eta in (0.0, 0.2):
        xg.grad = wg.grad = None
        y = adder.adder2d_function(xg, wg, s, p, eta=eta)
        y.backward(gy.to(gpu))
        torch.cuda.synchronize()
        gw_true = c_oracle.conv2d_grad_w(gy, x, w, s, p)
        if eta:
            gw_true = c_oracle.eta_scale(gw_true, eta)
        assert_close(wg.grad, gw_true, f"grad_W eta={eta} {case}")
        assert_close(xg.grad, c_oracle.conv2d_grad_x(gy, x, w, s, p), f"grad_X {case}")


def test_backward_is_deterministic(gpu):
    from addernetcuda_amd import adder
    case = (4, 16, 32, 32, 16, 3, 1, 1)
    x, w, gy = make_case(*case)
    outs = []
    for _ in range(2):
        xg = x.to(gpu).requires_grad_(True)
        wg = w.to(gpu).requires_grad_(True)
        adder.adder2d_function(xg, wg, 1, 1).backward(gy.to(gpu))
        outs.append((xg.grad.clone(), wg.grad.clone()))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


def test_clamp_saturates_both_ways(gpu):
    """x far above / below w: every tap contributes exactly -g / +g (hardtanh limits, adder.cu:17)."""
    from addernetcuda_amd import adder
    N, C, H = 2, 4, 8
    w = torch.zeros(C, C, 3, 3)
    gy = torch.randn(N, C, H, H, generator=torch.Generator().manual_seed(5))
    expect = torch.nn.functional.conv_transpose2d(gy, torch.ones(C, C, 3, 3), padding=1)
    for sign in (+1.0, -1.0):
        x = torch.full((N, C, H, H), 10.0 * sign)
        xg = x.to(gpu).requires_grad_(True)
        adder.adder2d_function(xg, w.to(gpu), 1, 1).backward(gy.to(gpu))
        assert_close(xg.grad, -sign * expect, f"saturated sign={sign}")


@pytest.mark.parametrize("x_scale", [0.05, 20.0, 3000.0])
@pytest.mark.parametrize("case", [(4, 16, 16, 16, 32, 3, 1, 1), (4, 32, 16, 16, 32, 3, 2, 1), (4, 64, 8, 8, 64, 1, 1, 0),
                                  (4, 16, 16, 16, 32, 1, 2, 0)], ids=str)
def test_grad_x_does_not_degrade_with_the_scale_of_x(case, x_scale, gpu):
    """The tiled grad_X kernels evaluate hardtanh(w - x) as 2 * sat(0.5 w + (0.5 - 0.5 x)) - 1; the
    rounding of 0.5 - 0.5 x must not show for activations much smaller or larger than the weights
    (terms that do not saturate have |x| <= |w| + 1 whatever the scale of x)."""
    from addernetcuda_amd import adder
    from oracle import c_oracle
    s, p = case[6], case[7]
    x, w, gy = make_case(*case, w_init="normal", x_scale=x_scale)
    xg = x.to(gpu).requires_grad_(True)
    adder.adder2d_function(xg, w.to(gpu), s, p, eta=0.0).backward(gy.to(gpu))
    assert_close(xg.grad, c_oracle.conv2d_grad_x(gy, x, w, s, p), f"grad_X x_scale={x_scale} {case}")


def _random_cases(count, seed):
    """Seeded random layer shapes around the kernels' switch points: channel counts on both sides of 64 and of
    the tile sizes, map sizes that are and are not multiples of 4, kernels 1 / 3 / 5, strides 1..3."""
    import random
    rnd = random.Random(seed)
    cases = []
    while len(cases) < count:
        k = rnd.choice([1, 1, 3, 3, 3, 5])
        s = rnd.choice([1, 1, 2, 3])
        p = {1: 0, 3: rnd.choice([0, 1, 1]), 5: 2}[k]
        ci = rnd.choice([1, 3, 7, 8, 16, 24, 63, 64, 65, 72, 130])
        co = rnd.choice([1, 5, 8, 16, 33, 63, 64, 65, 96])
        h, w = rnd.randint(k, 19), rnd.randint(k, 19)
        n = rnd.randint(1, 5)
        if ci * co * k * k * n * h * w > 6e7:     # keeps the C oracle at a fraction of a second per case
            continue
        cases.append((n, ci, h, w, co, k, s, p))
    return cases


def _random_1x1_cases(count, seed):
    """1x1 layers with >= 64 channels on both sides (the tiled single-tap kernels and, with a stride, their
    sampled-position variants), on planes of 4 .. 225 positions."""
    import random
    rnd = random.Random(seed)
    return [(rnd.randint(1, 5), rnd.choice([64, 72, 80, 128, 136]), rnd.randint(2, 15), rnd.randint(2, 15),
             rnd.choice([64, 65, 96, 130]), 1, rnd.choice([1, 2, 2, 3]), 0) for _ in range(count)]


@pytest.mark.parametrize("case", _random_cases(40, 2024) + _random_1x1_cases(16, 7), ids=str)
def test_random_shapes_match_oracle(case, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle
    s, p = case[6], case[7]
    x, w, gy = make_case(*case, w_init="normal", seed=sum(case))
    xg, wg = x.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
    y = adder.adder2d_function(xg, wg, s, p, eta=0.0)
    y.backward(gy.to(gpu))
    torch.cuda.synchronize()
    assert_close(y, c_oracle.conv2d_fwd(x, w, s, p), f"forward {case}")
    assert_close(xg.grad, c_oracle.conv2d_grad_x(gy, x, w, s, p), f"grad_X {case}")
    assert_close(wg.grad, c_oracle.conv2d_grad_w(gy, x, w, s, p), f"grad_W {case}")


@pytest.mark.parametrize("case", [(3, 16, 32, 32, 16, 3, 1, 1), (2, 32, 16, 16, 32, 3, 1, 1), (5, 64, 8, 8, 64, 3, 1, 1),
                                  (2, 9, 10, 18, 8, 3, 1, 1), (2, 16, 14, 14, 24, 1, 1, 0), (2, 6, 14, 24, 10, 3, 2, 1),
                                  (2, 16, 32, 32, 32, 3, 2, 1), (3, 32, 16, 16, 64, 3, 2, 1), (2, 5, 12, 20, 7, 3, 2, 1),
                                  # the tiled 1x1 kernels (from 64 input channels): large and small planes, planes that
                                  # are not whole groups of four
                                  (2, 64, 14, 14, 64, 1, 1, 0), (4, 64, 8, 8, 256, 1, 1, 0), (2, 128, 7, 7, 128, 1, 1, 0),
                                  (3, 256, 6, 6, 64, 1, 1, 0), (40, 72, 8, 8, 56, 1, 1, 0)],
                         ids=str)
def test_shortcut_gradient_is_added_to_grad_x(case, gpu):
    """with_shortcut: x leaves the layer's autograd node a second time; what is back-propagated into that output
    must come out added to grad_X (inside the grad_X kernel for the tiled 3x3 stride-1 layers, by a plain add
    elsewhere), exactly as if the caller had used x itself."""
    from addernetcuda_amd import adder
    from oracle import c_oracle
    s, p = case[6], case[7]
    x, w, gy = make_case(*case)
    gs = torch.randn(x.shape, generator=torch.Generator().manual_seed(99))
    xg, wg = x.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
    y, stats, shortcut = adder.adder2d_function_with_stats(xg, wg, s, p, eta=0.0, with_shortcut=True)
    assert shortcut.data_ptr() == xg.data_ptr() and torch.equal(shortcut, xg)
    torch.autograd.backward([y, shortcut], [gy.to(gpu), gs.to(gpu)])
    torch.cuda.synchronize()
    assert_close(y, c_oracle.conv2d_fwd(x, w, s, p), f"forward {case}")
    assert_close(xg.grad, c_oracle.conv2d_grad_x(gy, x, w, s, p) + gs.double(), f"grad_X + shortcut {case}")
    assert_close(wg.grad, c_oracle.conv2d_grad_w(gy, x, w, s, p), f"grad_W {case}")
    # only the shortcut is used downstream: its gradient passes through unchanged
    x2 = x.to(gpu).requires_grad_(True)
    _, _, sc2 = adder.adder2d_function_with_stats(x2, w.to(gpu), s, p, eta=0.0, with_shortcut=True)
    sc2.backward(gs.to(gpu))
    assert torch.equal(x2.grad.cpu(), gs)


def test_batched_eta_scaling_leaves_the_same_gradients(gpu):
    """Inside batched_eta_scaling() the layers leave raw weight gradients and the block's exit scales them all
    at once: .grad afterwards must equal what the layers produce on their own, for every layer, bit for bit
    in the norm's fp64 sum order or to rounding (two different reduction trees): compare to 1e-6 relative."""
    from addernetcuda_amd import adder
    shapes = [(16, 16, 3, 1, 1), (16, 32, 1, 2, 0), (32, 32, 3, 1, 1), (32, 24, 3, 2, 1), (24, 8, 5, 1, 2)]
    g = torch.Generator().manual_seed(3)
    x0 = torch.randn(4, 16, 16, 16, generator=g).to(gpu)

    def run(batched):
        torch.manual_seed(0)
        layers = [adder.adder2d(ci, co, k, stride=s, padding=p, eta=0.1 * (i + 1)).to(gpu)
                  for i, (ci, co, k, s, p) in enumerate(shapes)]
        h = x0
        for layer in layers:
            h = layer(h)
        loss = h.square().mean()
        if batched:
            with adder.batched_eta_scaling():
                loss.backward()
        else:
            loss.backward()
        torch.cuda.synchronize()
        return [layer.adder.grad.clone() for layer in layers]

    plain, batched = run(False), run(True)
    for a, b, shp in zip(plain, batched, shapes):
        assert torch.allclose(a, b, rtol=1e-6, atol=0.0), shp
        n = a.numel()
    # a second backward into existing .grad inside the block is scaled on the spot and accumulated, as without it
    layer = adder.adder2d(8, 8, 3, padding=1).to(gpu)
    xin = torch.randn(2, 8, 6, 6, generator=g).to(gpu)
    layer(xin).sum().backward()
    first = layer.adder.grad.clone()
    with adder.batched_eta_scaling():
        layer(xin).sum().backward()
    assert torch.allclose(layer.adder.grad, 2 * first, rtol=1e-6, atol=0.0)


# (N, Ci, H, W, Co, kh, kw, stride, pad): kernels that are not square.  The reference's operator assumes square
# ones (adder.py:32 hands unfold the kernel's height only) and so does this build's Python layer; the C ABI takes
# kh and kw separately, serves such layers with the generic kernels, and is held to the same oracle.
NON_SQUARE = [(2, 5, 9, 11, 6, 3, 1, 1, 1), (2, 4, 8, 12, 7, 1, 3, 1, 1), (1, 3, 10, 9, 4, 3, 5, 2, 2),
              (2, 6, 7, 7, 5, 1, 2, 1, 0), (1, 8, 12, 12, 8, 3, 1, 2, 1)]


@pytest.mark.parametrize("case", NON_SQUARE, ids=str)
def test_non_square_kernels_through_the_c_abi(case, gpu):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, check
    from oracle import c_oracle
    N, Ci, H, W, Co, kh, kw, s, p = case
    g = torch.Generator().manual_seed(77 + kh * 10 + kw)
    x = torch.randn(N, Ci, H, W, generator=g)
    w = torch.randn(Co, Ci, kh, kw, generator=g) * 0.5
    Ho, Wo = (H - kh + 2 * p) // s + 1, (W - kw + 2 * p) // s + 1
    gy = torch.randn(N, Co, Ho, Wo, generator=g)
    dims = (N, Ci, H, W, Co, kh, kw, s, p)
    xg, wg, gyg = x.to(gpu), w.to(gpu), gy.to(gpu)
    y, gx, gw = torch.empty(N, Co, Ho, Wo, device=gpu), torch.empty_like(xg), torch.empty_like(wg)
    need = ctypes.c_size_t()
    check(lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)), "workspace")
    ws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=gpu)
    st = stream_ptr(gpu)
    check(lib.adder_conv2d_fwd_f32(ptr(xg), ptr(wg), ptr(y), *dims, st), "fwd")
    check(lib.adder_conv2d_bwd_f32(ptr(gyg), ptr(xg), ptr(wg), ptr(gx), ptr(gw), 0.0, ptr(ws), need.value, *dims, st), "bwd")
    torch.cuda.synchronize()
    assert_close(y, c_oracle.conv2d_fwd(x, w, s, p), f"forward {case}")
    assert_close(gx, c_oracle.conv2d_grad_x(gy, x, w, s, p), f"grad_X {case}")
    assert_close(gw, c_oracle.conv2d_grad_w(gy, x, w, s, p), f"raw grad_W {case}")
