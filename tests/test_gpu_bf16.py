"""The optional bfloat16-storage mode (activations and their gradients in bfloat16, float32 weights, float32 /
float64 accumulation) against the float64 oracle evaluated on the same bfloat16-rounded inputs.

The bar: the output and grad_X are rounded to bfloat16 once, on the way out, so each may be off by one bfloat16
unit in the last place (2^-8 relative) plus the float32 path's own tolerance; the weight gradient is a float32
result of fp64 sums and is held to the float32 bar, rtol 1e-5 / atol 1e-4."""
import pytest
import torch

from tests.util import make_case, assert_close

pytestmark = pytest.mark.gpu

BF16_ULP = 2.0 ** -8

# (N, Ci, H, W, Co, k, stride, pad): the tiled 3x3 kernels at every tile width and stride, rows that are not
# whole groups of four, channel tails, then layers that take the generic kernels (1x1 stride 2, 5x5, 3 channels)
SHAPES = [(4, 16, 32, 32, 16, 3, 1, 1), (3, 32, 16, 16, 32, 3, 1, 1), (5, 64, 8, 8, 64, 3, 1, 1),
          (3, 16, 32, 32, 32, 3, 2, 1), (4, 32, 16, 16, 64, 3, 2, 1), (2, 20, 14, 14, 12, 3, 1, 1),
          (2, 9, 7, 10, 5, 3, 1, 1), (2, 16, 32, 32, 32, 1, 2, 0), (2, 6, 11, 11, 4, 5, 2, 2), (2, 3, 32, 32, 16, 3, 1, 1),
          (2, 64, 14, 14, 64, 1, 1, 0)]


def _close_bf16(got, want, what):
    g, w = got.detach().double().cpu(), want.double()
    bad = (g - w).abs() > BF16_ULP * w.abs() + 2e-4
    assert not bad.any(), f"{what}: {int(bad.sum())}/{bad.numel()} outside one bfloat16 ulp; worst {((g - w).abs()).max():.3e}"


@pytest.mark.parametrize("case", SHAPES, ids=str)
def test_bfloat16_storage_matches_the_oracle_on_the_rounded_inputs(case, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle, adder_oracle
    s, p = case[6], case[7]
    x, w, gy = make_case(*case)
    xb, gb = x.bfloat16(), gy.bfloat16()
    xr, gr = xb.float(), gb.float()                 # what the kernels see, exactly
    xg, wg = xb.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
    y = adder.adder2d_function(xg, wg, s, p, eta=0.0)
    assert y.dtype == torch.bfloat16
    y.backward(gb.to(gpu))
    torch.cuda.synchronize()
    assert xg.grad.dtype == torch.bfloat16 and wg.grad.dtype == torch.float32
    _close_bf16(y, c_oracle.conv2d_fwd(xr, w, s, p), f"forward {case}")
    _close_bf16(xg.grad, c_oracle.conv2d_grad_x(gr, xr, w, s, p), f"grad_X {case}")
    want_w = c_oracle.conv2d_grad_w(gr, xr, w, s, p)
    assert_close(wg.grad, want_w, f"grad_W {case}")
    # the scaling of adder.py:78 on top
    wg.grad = None
    adder.adder2d_function(xg, wg, s, p, eta=0.2).backward(gb.to(gpu))
    assert_close(wg.grad, adder_oracle.eta_scale(want_w, 0.2), f"eta-scaled grad_W {case}")


def test_the_module_takes_bfloat16_activations_with_float32_parameters(gpu):
    from addernetcuda_amd import adder
    torch.manual_seed(0)
    layer = adder.adder2d(16, 32, 3, stride=1, padding=1, bias=True).to(gpu)
    x = torch.randn(4, 16, 16, 16, device=gpu)
    ref = layer(x)                                     # float32 path
    out = layer(x.bfloat16())
    assert out.dtype == torch.bfloat16 and layer.adder.dtype == torch.float32
    # against the float32 result: the input rounding (2^-9 per element, averaged over 144 terms) and one output rounding
    assert torch.allclose(out.float(), ref, rtol=2 * BF16_ULP, atol=0.05)
    out.float().sum().backward()
    assert layer.adder.grad.dtype == torch.float32 and torch.isfinite(layer.adder.grad).all()
    # float32 inputs still take the float32 kernels bit for bit
    assert torch.equal(layer(x), ref)
