"""Layer shapes of the other reference models (VGG-small-style stack, ResNet-50 bottlenecks, DenseNet-BC)
at reduced batch against the float64 C oracle: large K (up to 4608), 1x1 and strided layers on
56/28/14/7-wide maps, 12-channel growth, the 3-channel VGG stem."""
import pytest
import torch

from tests.util import make_case, assert_close

pytestmark = pytest.mark.gpu

# (N, Ci, H, W, Co, k, stride, pad)
SHAPES = [
    (2, 128, 32, 32, 128, 3, 1, 1),    # VGG-small 128->128 @32, K = 1152
    (2, 256, 16, 16, 256, 3, 1, 1),    # K = 2304
    (2, 512, 8, 8, 512, 3, 1, 1),      # K = 4608
    (2, 3, 32, 32, 64, 3, 1, 1),       # vgg.py:60-66: the 3-channel stem is an adder layer too
    (1, 64, 56, 56, 64, 3, 1, 1),      # ResNet-50 3x3 @56
    (1, 64, 56, 56, 256, 1, 1, 0),     # 1x1 expand @56
    (1, 256, 56, 56, 512, 1, 2, 0),    # 1x1 stride-2 downsample 56 -> 28
    (1, 128, 56, 56, 128, 3, 2, 1),    # strided 3x3 56 -> 28
    (2, 256, 14, 14, 256, 3, 1, 1),    # 14-wide maps (W % 4 != 0)
    (2, 1024, 14, 14, 256, 1, 1, 0),   # 1x1 reduce @14, K = 1024
    (2, 512, 7, 7, 512, 3, 1, 1),      # 7-wide maps
    (2, 2048, 7, 7, 512, 1, 1, 0),     # K = 2048
    (3, 24, 32, 32, 48, 1, 1, 0),      # DenseNet-BC bottleneck 1x1 (densenet.py:12-14)
    (3, 48, 32, 32, 12, 3, 1, 1),      # DenseNet-BC growth conv, Co = 12
    (1, 32, 16, 16, 640, 3, 2, 1),     # strided 3x3 with > 2304 terms per input position (three-instruction grad_X form)
    (64, 1024, 7, 7, 64, 1, 1, 0),     # 1x1 on 49-position planes with many images x channel blocks (the larger small-plane grad_X tile)
    (3, 84, 32, 32, 48, 1, 1, 0),      # DenseNet 1x1 with >= 64 input channels, a multiple of 4 but not of 8
    (5, 132, 8, 8, 48, 1, 1, 0),       # ... on 64-position planes
    (6, 372, 4, 4, 48, 1, 1, 0),       # ... the last dense stage: 16-position planes
    (2, 180, 16, 16, 96, 1, 2, 0),     # ... with a stride
    (2, 64, 12, 12, 65, 1, 1, 0),      # 1x1 grad_X units of two output channels, odd channel count
    (2, 64, 7, 7, 70, 1, 1, 0),        # ... units of eight output channels, 70 = 8 * 8 + 6
    (3, 72, 14, 14, 67, 1, 2, 0),      # ... the same on a sampled (strided) layer
    (2, 128, 5, 5, 130, 1, 1, 0),      # 128 x 128-channel weight-gradient blocks with a 2-channel tail, 25-position planes
]


@pytest.mark.parametrize("case", SHAPES, ids=str)
def test_layer_matches_oracle(case, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle
    s, p = case[6], case[7]
    x, w, gy = make_case(*case, w_init="normal")          # adder2d's own N(0,1) init (adder.py:97)
    xg, wg = x.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
    y = adder.adder2d_function(xg, wg, s, p, eta=0.0)
    y.backward(gy.to(gpu))
    torch.cuda.synchronize()
    assert_close(y, c_oracle.conv2d_fwd(x, w, s, p), f"forward {case}")
    assert_close(xg.grad, c_oracle.conv2d_grad_x(gy, x, w, s, p), f"grad_X {case}")
    assert_close(wg.grad, c_oracle.conv2d_grad_w(gy, x, w, s, p), f"grad_W {case}")


@pytest.mark.parametrize("case", [(2, 64, 28, 28, 96, 1, 2, 0), (2, 128, 14, 14, 64, 1, 2, 0), (1, 64, 9, 9, 64, 1, 3, 0),
                                  (3, 64, 7, 7, 128, 1, 2, 0), (2, 72, 10, 6, 64, 1, 2, 0), (5, 64, 8, 8, 64, 1, 4, 0),
                                  (2, 68, 18, 18, 40, 1, 2, 0), (3, 76, 7, 9, 64, 1, 3, 0),
                                  (2, 256, 28, 28, 128, 1, 2, 0), (3, 128, 14, 14, 256, 1, 2, 0),
                                  (4, 1024, 14, 14, 2048, 1, 2, 0)], ids=str)
def test_strided_1x1_with_many_channels_walks_the_sampled_positions(case, gpu):
    """From 64 channels on, the tiled kernels walk the sampled positions x[:, :, ::s, ::s] of a strided 1x1
    layer like a stride-1 plane; results and both gradients (the input gradient stored together with the
    exact zeros in between) must be those of the strided layer."""
    from addernetcuda_amd import adder
    from oracle import c_oracle
    N, Ci, H, W, Co, k, s, p = case
    x, w, gy = make_case(*case)
    xg, wg = x.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
    y = adder.adder2d_function(xg, wg, s, p, eta=0.0)
    y.backward(gy.to(gpu))
    torch.cuda.synchronize()
    assert_close(y, c_oracle.conv2d_fwd(x, w, s, p), "y")
    assert_close(xg.grad, c_oracle.conv2d_grad_x(gy, x, w, s, p), "grad_x")
    assert_close(wg.grad, c_oracle.conv2d_grad_w(gy, x, w, s, p), "grad_w")
    mask = torch.ones(H, W, dtype=torch.bool)
    mask[::s, ::s] = False
    assert (xg.grad.cpu()[:, :, mask] == 0).all()
