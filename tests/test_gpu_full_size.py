"""The benchmark's own layer shapes at batch 256: checks that do not need a CPU oracle pass over
6e8 terms -- a slice of images against the float64 C oracle (forward and grad_X are per-image),
an independent float64 GEMM on the GPU for grad_W, and size-independent properties."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_close

pytestmark = pytest.mark.gpu

N = 256
# (Ci, H, W, Co, k, stride, pad): the ResNet-20 adder-layer shapes
LAYERS = [(16, 32, 32, 16, 3, 1, 1), (32, 16, 16, 32, 3, 1, 1), (64, 8, 8, 64, 3, 1, 1), (16, 32, 32, 32, 3, 2, 1),
          (32, 16, 16, 64, 3, 2, 1), (16, 32, 32, 32, 1, 2, 0), (32, 16, 16, 64, 1, 2, 0)]
PICK = [0, 1, 100, 255]


def _data(Ci, H, W, Co, k, s, p, gpu):
    g = torch.Generator(device=gpu).manual_seed(1000 + Ci + Co + k + s)
    x = torch.randn(N, Ci, H, W, device=gpu, generator=g)
    w = torch.randn(Co, Ci, k, k, device=gpu, generator=g) * math.sqrt(2.0 / (Ci * k * k))
    Ho, Wo = (H - k + 2 * p) // s + 1, (W - k + 2 * p) // s + 1
    gy = torch.randn(N, Co, Ho, Wo, device=gpu, generator=g)
    return x, w, gy


@pytest.mark.parametrize("layer", LAYERS, ids=str)
def test_full_batch_layer(layer, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle
    Ci, H, W, Co, k, s, p = layer
    x, w, gy = _data(*layer, gpu)
    xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    y = adder.adder2d_function(xg, wg, s, p, eta=0.0)
    y.backward(gy)
    torch.cuda.synchronize()

    # forward and grad_X are independent per image: a slice against the float64 C oracle
    xs, ws, gs = x[PICK].cpu(), w.cpu(), gy[PICK].cpu()
    assert_close(y[PICK], c_oracle.conv2d_fwd(xs, ws, s, p), f"forward slice {layer}")
    assert_close(xg.grad[PICK], c_oracle.conv2d_grad_x(gs, xs, ws, s, p), f"grad_X slice {layer}")

    # grad_W sums over the whole batch: float64 GEMM identity on the GPU, image by image
    acc = torch.zeros(Co, Ci * k * k, dtype=torch.float64, device=gpu)
    for a in range(0, N, 32):
        cols = F.unfold(x[a:a + 32].double(), k, padding=p, stride=s)            # (n, K, L)
        acc += torch.einsum("ncl,nkl->ck", gy[a:a + 32].double().flatten(2), cols)
    want = acc.view_as(w) - w.double() * gy.double().sum(dim=(0, 2, 3)).view(-1, 1, 1, 1)
    assert_close(wg.grad, want, f"grad_W {layer}")

    # properties: y <= 0; backward is linear in gy; eta fixes the norm of grad_W
    assert (y <= 0).all()
    xg.grad = wg.grad = None
    y2 = adder.adder2d_function(xg, wg, s, p, eta=0.1)
    assert torch.equal(y2, y)                                                      # deterministic
    y2.backward(2.0 * gy)
    assert wg.grad.norm().item() == pytest.approx(0.1 * math.sqrt(w.numel()), rel=1e-4)
    xg2 = x.clone().requires_grad_(True)
    adder.adder2d_function(xg2, w, s, p).backward(gy)
    assert torch.allclose(xg.grad, 2.0 * xg2.grad, rtol=1e-5, atol=1e-5)
    if s == 2:                                                                     # unsampled pixels stay exactly 0
        if k == 1:
            assert (xg.grad[:, :, 1::2, :] == 0).all() and (xg.grad[:, :, :, 1::2] == 0).all()
