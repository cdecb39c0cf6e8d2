"""Margin of the two-instruction input gradient (hardtanh(w - x) = 2 sat(w/2 + (1/2 - x/2)) - 1, a doubled sum with
a second sum taken off) on the layers with the most terms per output that still use it.

The form costs accuracy against the three-instruction one, so layers above a term count keep the latter
(grad_x.hip: 1152 terms for 3x3 layers, 1024 for single-tap ones).  This test runs the layers that sit at those
switch points -- 128 -> 128 3x3 and ResNet-50's 256 -> 1024 @14x14 -- two below them (128 -> 512 @28x28, ResNet-20's
64 -> 64 @8x8) and two above, which run the three-instruction form (VGG-small's 256 -> 256 @16x16 and
512 -> 512 @8x8), over 8 seeds x {Kaiming, N(0,1)} weights x input scale {1, 5} and holds the worst
element of every case to 0.7 of the parity tolerance 1e-4 + 1e-5 |gx| against the float64 C oracle
(test_cuda.py:57-60; adder.cu:17,246).  The input gradient of an image depends on that image alone, so four
images per case stand for any batch size.
"""
import ctypes
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

# (Ci, H, W, Co, k, stride, pad), terms per input position = Co * k * k
LAYERS = [(128, 16, 16, 128, 3, 1, 1), (256, 14, 14, 1024, 1, 1, 0), (128, 28, 28, 512, 1, 1, 0), (64, 8, 8, 64, 3, 1, 1),
          (256, 16, 16, 256, 3, 1, 1), (512, 8, 8, 512, 3, 1, 1)]
IMAGES = 4
MARGIN = 0.7


@pytest.mark.parametrize("layer", LAYERS, ids=str)
def test_two_instruction_input_gradient_keeps_its_margin(layer, gpu):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, check
    from oracle import c_oracle
    Ci, H, W, Co, k, s, p = layer
    dims = (IMAGES, Ci, H, W, Co, k, k, s, p)
    worst = {}
    for w_init in ("kaiming", "normal"):
        for x_scale in (1.0, 5.0):
            for seed in range(8):
                g = torch.Generator().manual_seed(9000 + 100 * seed + Ci + Co)
                x = torch.randn(IMAGES, Ci, H, W, generator=g) * x_scale
                w = torch.randn(Co, Ci, k, k, generator=g) * (math.sqrt(2.0 / (Ci * k * k)) if w_init == "kaiming" else 1.0)
                gy = torch.randn(IMAGES, Co, H, W, generator=g)
                xg, wg, gyg = x.to(gpu), w.to(gpu), gy.to(gpu)
                gx = torch.empty_like(xg)
                check(lib.adder_conv2d_bwd_f32(ptr(gyg), ptr(xg), ptr(wg), ptr(gx), None, 0.0, None, 0, *dims,
                                               stream_ptr(gpu)), "adder_conv2d_bwd_f32")
                torch.cuda.synchronize()
                ref = c_oracle.conv2d_grad_x(gy, x, w, s, p)
                ratio = ((gx.double().cpu() - ref).abs() / (1e-4 + 1e-5 * ref.abs())).max().item()
                key = (w_init, x_scale)
                worst[key] = max(worst.get(key, 0.0), ratio)
                assert ratio <= MARGIN, (f"{layer} {w_init} weights, x scale {x_scale}, seed {seed}: worst element at "
                                         f"{ratio:.2f} of the tolerance (bar {MARGIN})")
    print(f"\ngrad_X margin {layer}: " + ", ".join(f"{k[0]} x{k[1]:g}: {v:.2f}" for k, v in worst.items()))
