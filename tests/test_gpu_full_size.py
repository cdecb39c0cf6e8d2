"""The layer shapes of the three model configurations at their full batch sizes (ResNet-20 at 256, the
VGG-small stack at 128, ResNet-50 at 224x224 at 64): launch grids, partial-slab counts and workspace sizes all
depend on the batch, so the reduced-batch parity tests do not cover these code paths.  Checks that do not
need a CPU oracle pass over 1e10 terms: a slice of images against the float64 C oracle (forward and grad_X are
per-image), an independent float64 GEMM on the GPU for grad_W (raw and eta-scaled, element by element), and
size-independent properties."""
import math

import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (N, Ci, H, W, Co, k, stride, pad)
RESNET20 = [(256,) + l for l in [                       # resnet20.py:16-20, 52-54, 66-70
    (16, 32, 32, 16, 3, 1, 1), (32, 16, 16, 32, 3, 1, 1), (64, 8, 8, 64, 3, 1, 1), (16, 32, 32, 32, 3, 2, 1),
    (32, 16, 16, 64, 3, 2, 1), (16, 32, 32, 32, 1, 2, 0), (32, 16, 16, 64, 1, 2, 0)]]
VGG_SMALL = [(128,) + l for l in [                      # 3x3 layers at 128 / 256 / 512 channels, K up to 4608
    (128, 32, 32, 128, 3, 1, 1), (128, 16, 16, 256, 3, 1, 1), (256, 16, 16, 256, 3, 1, 1),
    (256, 8, 8, 512, 3, 1, 1), (512, 8, 8, 512, 3, 1, 1)]]
RESNET50 = [(64,) + l for l in [                        # every distinct layer shape of resnet50.py:19-33, 84-98
    (64, 56, 56, 256, 1, 1, 0), (64, 56, 56, 64, 1, 1, 0), (64, 56, 56, 64, 3, 1, 1),
    (256, 56, 56, 64, 1, 1, 0), (256, 56, 56, 512, 1, 2, 0), (256, 56, 56, 128, 1, 1, 0),
    (128, 56, 56, 128, 3, 2, 1), (128, 28, 28, 512, 1, 1, 0), (512, 28, 28, 128, 1, 1, 0),
    (128, 28, 28, 128, 3, 1, 1), (512, 28, 28, 1024, 1, 2, 0), (512, 28, 28, 256, 1, 1, 0),
    (256, 28, 28, 256, 3, 2, 1), (256, 14, 14, 1024, 1, 1, 0), (1024, 14, 14, 256, 1, 1, 0),
    (256, 14, 14, 256, 3, 1, 1), (1024, 14, 14, 2048, 1, 2, 0), (1024, 14, 14, 512, 1, 1, 0),
    (512, 14, 14, 512, 3, 2, 1), (512, 7, 7, 2048, 1, 1, 0), (2048, 7, 7, 512, 1, 1, 0),
    (512, 7, 7, 512, 3, 1, 1)]]
LAYERS = RESNET20 + VGG_SMALL + RESNET50


def _data(N, Ci, H, W, Co, k, s, p, gpu):
    g = torch.Generator(device=gpu).manual_seed(1000 + Ci + Co + k + s)
    x = torch.randn(N, Ci, H, W, device=gpu, generator=g)
    w = torch.randn(Co, Ci, k, k, device=gpu, generator=g) * math.sqrt(2.0 / (Ci * k * k))
    Ho, Wo = (H - k + 2 * p) // s + 1, (W - k + 2 * p) // s + 1
    gy = torch.randn(N, Co, Ho, Wo, device=gpu, generator=g)
    return x, w, gy


@pytest.mark.parametrize("layer", LAYERS, ids=str)
def test_full_batch_layer(layer, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle, adder_oracle
    N, Ci, H, W, Co, k, s, p = layer
    PICK = [0, 1, N // 2 - 1, N - 1] if Co * Ci * k * k * H * W <= 2 ** 28 else [0, N - 1]   # oracle time
    CH = 32 if Ci * k * k * H * W <= 2 ** 21 else 4                                       # images per unfold
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
    for a in range(0, N, CH):
        cols = F.unfold(x[a:a + CH].double(), k, padding=p, stride=s)            # (n, K, L)
        acc += torch.einsum("ncl,nkl->ck", gy[a:a + CH].double().flatten(2), cols)
        del cols
    want = acc.view_as(w) - w.double() * gy.double().sum(dim=(0, 2, 3)).view(-1, 1, 1, 1)
    assert_close(wg.grad, want, f"grad_W {layer}")

    # properties: y <= 0; backward is linear in gy; the scaling of adder.py:78, element by element
    assert (y <= 0).all()
    xg.grad = wg.grad = None
    y2 = adder.adder2d_function(xg, wg, s, p, eta=0.1)
    assert torch.equal(y2, y)                                                      # deterministic
    y2.backward(2.0 * gy)
    assert_close(wg.grad, adder_oracle.eta_scale(2.0 * want, 0.1), f"eta-scaled grad_W {layer}")
    assert wg.grad.norm().item() == pytest.approx(0.1 * math.sqrt(w.numel()), rel=1e-4)
    xg2 = x.clone().requires_grad_(True)
    adder.adder2d_function(xg2, w, s, p).backward(gy)
    assert torch.allclose(xg.grad, 2.0 * xg2.grad, rtol=1e-5, atol=1e-5)
    if s == 2:                                                                     # unsampled pixels stay exactly 0
        if k == 1:
            assert (xg.grad[:, :, 1::2, :] == 0).all() and (xg.grad[:, :, :, 1::2] == 0).all()


# the layer shapes above whose kernels carry the BatchNorm links (3x3 / pad 1, and 1x1 stride 1 from 64 channels on
# planes of whole float4 groups), at their full batch
LINKED = [l for l in RESNET20 if l[5] == 3] + [(64, 64, 56, 56, 256, 1, 1, 0), (64, 256, 56, 56, 64, 1, 1, 0),
                                               (64, 512, 28, 28, 128, 1, 1, 0)]


@pytest.mark.parametrize("from_x", [False, True], ids=["reads_bn_input", "xhat_from_x"])
@pytest.mark.parametrize("layer", LINKED, ids=str)
def test_full_batch_links(layer, from_x, gpu):
    """The backward with both BatchNorm links at full batch (slot counts and grids depend on it), against the
    library's plain kernels -- which the test above holds to the oracle -- and float64 BatchNorm arithmetic on the
    GPU: the output gradient the weight-gradient kernel forms, both gradients, the partial sums of the BatchNorm in
    front."""
    import ctypes
    from addernetcuda_amd._lib import lib, check, ptr, stream_ptr, BnLinks, bwd_bn_slots, conv_dims, conv2d_bwd_workspace
    N, Ci, H, W, Co, k, s, p = layer
    g = torch.Generator(device=gpu).manual_seed(7 + Ci + Co + k + s)
    b = lambda v: v[None, :, None, None]
    bn_in = torch.randn(N, Ci, H, W, device=gpu, generator=g) * 20 - 90
    mean, rstd = bn_in.mean((0, 2, 3)), 1.0 / bn_in.std((0, 2, 3))
    gamma, beta = torch.rand(Ci, device=gpu, generator=g) + 0.5, torch.randn(Ci, device=gpu, generator=g) * 0.3
    x = (bn_in - b(mean)) * b(rstd * gamma) + b(beta)
    if not from_x:
        x = x + torch.randn(x.shape, device=gpu, generator=g)          # a residual: xhat cannot come from x
    x = torch.relu(x)
    w = torch.randn(Co, Ci, k, k, device=gpu, generator=g) * math.sqrt(2.0 / (Ci * k * k))
    dims, Ho, Wo = conv_dims(x.shape, w.shape, s, p)
    slots = bwd_bn_slots(dims)
    assert slots > 0
    y = torch.randn(N, Co, Ho, Wo, device=gpu, generator=g) * 20 - 90
    dz = torch.randn(N, Co, Ho, Wo, device=gpu, generator=g) * (torch.rand(N, Co, Ho, Wo, device=gpu, generator=g) > 0.4)
    coef = torch.randn(Co, 4, device=gpu, generator=g) * torch.tensor([1.0, 0.01, 0.0, 0.1], device=gpu)
    coef[:, 2] = y.mean((0, 2, 3))
    gadd = torch.randn(x.shape, device=gpu, generator=g)
    st = stream_ptr(gpu)
    ws, nbytes = conv2d_bwd_workspace(dims, gpu)

    part = torch.full((Ci, slots, 2), float("nan"), dtype=torch.float32, device=gpu)
    gy_out = torch.empty_like(dz)
    links = BnLinks(ptr(y), ptr(coef), ptr(gy_out), ptr(bn_in), ptr(mean), ptr(rstd), ptr(part), slots, 1,
                    ptr(gamma) if from_x else None, ptr(beta) if from_x else None)
    gx, gw = torch.empty_like(x), torch.empty_like(w)
    check(lib.adder_conv2d_bwd_bn_f32(ptr(dz), ptr(x), ptr(w), ptr(gadd), ptr(gx), ptr(gw), 0.1, ptr(ws), nbytes, *dims,
                                      ctypes.byref(links), st), "adder_conv2d_bwd_bn_f32")
    torch.cuda.synchronize()

    c = coef.double()
    want_gy = b(c[:, 0]) * dz.double() + b(c[:, 1]) * (y.double() - b(c[:, 2])) - b(c[:, 3])
    assert_close(gy_out, want_gy, f"formed gy {layer}", rtol=1e-5, atol=1e-5)
    # the same kernels without the links, on the gradient that was formed
    gx0, gw0 = torch.empty_like(x), torch.empty_like(w)
    check(lib.adder_conv2d_bwd_f32(ptr(gy_out), ptr(x), ptr(w), ptr(gx0), ptr(gw0), 0.1, ptr(ws), nbytes, *dims, st),
          "adder_conv2d_bwd_f32")
    torch.cuda.synchronize()
    assert torch.equal(gw, gw0)
    assert torch.equal(gx, (gx0 + gadd) * (x > 0))
    xhat = (bn_in.double() - b(mean.double())) * b(rstd.double())
    want = torch.stack([gx.double().sum((0, 2, 3)), (gx.double() * xhat).sum((0, 2, 3))], 1)
    assert torch.isfinite(part).all()
    scale = max(1.0, float(want.abs().max()))
    assert_close(part.double().sum(1) / scale, want / scale, f"sums of dz, dz * xhat {layer}", rtol=1e-5, atol=1e-5)
