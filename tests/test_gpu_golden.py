"""The committed integer fixtures (tests/golden/adder_small_int.json: exact answers from literal integer loop
nests over the reference's formulas, adder_cuda/test_cuda.py:18-22, 35-41, 57-60) through the HIP path.

Small integers are exact in fp32, in the fp64 matrix-core weight gradient and in both arithmetic forms of the
input gradient (0.5 * w + (0.5 - 0.5 * x) is exact wherever w - x is), so every result must match bit for bit:
through adder2d_function (fused NCHW kernels) and through the four adder_cuda.ADDER_* entry points on the
unfolded matrices."""
import json
import os

import pytest
import torch

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def _fixtures():
    with open(os.path.join(HERE, "golden", "adder_small_int.json")) as f:
        return json.load(f)


def _tensors(fx, gpu):
    x, w, gy = (torch.tensor(fx[n], dtype=torch.float32, device=gpu) for n in ("x", "w", "gy"))
    y, gw, gx = (torch.tensor(fx[n], dtype=torch.float32, device=gpu) for n in ("y", "gw", "gx"))
    return x, w, gy, y, gw, gx


@pytest.mark.parametrize("fx", _fixtures(), ids=lambda f: str(f["dims"]))
def test_fused_nchw_path_reproduces_the_fixtures_exactly(fx, gpu):
    from addernetcuda_amd import adder
    N, Ci, H, W, Co, k, s, p = fx["dims"]
    x, w, gy, y, gw, gx = _tensors(fx, gpu)
    xg, wg = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    out = adder.adder2d_function(xg, wg, s, p, eta=0.0)
    out.backward(gy)
    assert torch.equal(out.detach(), y)
    assert torch.equal(xg.grad, gx)
    assert torch.equal(wg.grad, gw)
    # the module, and the shortcut-add epilogue of the input-gradient kernels: gx + an integer tensor
    layer = adder.adder2d(Ci, Co, k, stride=s, padding=p, eta=0.0).to(gpu)
    with torch.no_grad():
        layer.adder.copy_(w)
    xg2 = x.clone().requires_grad_(True)
    out2, _, short = layer.forward_with_stats(xg2, with_shortcut=True)
    extra = torch.arange(x.numel(), device=gpu, dtype=torch.float32).view_as(x) % 7 - 3
    torch.autograd.backward([out2, short], [gy, extra])
    assert torch.equal(out2.detach(), y)
    assert torch.equal(xg2.grad, gx + extra)
    assert torch.equal(layer.adder.grad, gw)


@pytest.mark.parametrize("fx", _fixtures(), ids=lambda f: str(f["dims"]))
def test_column_matrix_entry_points_reproduce_the_fixtures_exactly(fx, gpu):
    """ADDER_CONV / ADDER_BACKWARD / ADDER_CONV_WEIGHT / ADDER_CONV_INPUT on the matrices adder.py:32-34 builds,
    results folded back the way autograd folds them (adder.py:38-39 and the adjoint of the unfold)."""
    from addernetcuda_amd import adder_cuda
    from oracle import adder_oracle as O
    N, Ci, H, W, Co, k, s, p = fx["dims"]
    x, w, gy, y, gw, gx = _tensors(fx, gpu)
    X_col, ho, wo = O.im2col(x, k, s, p)
    W_col = w.reshape(Co, -1).contiguous()
    out = torch.empty(Co, X_col.shape[1], device=gpu)
    adder_cuda.ADDER_CONV(X_col, W_col, out)
    assert torch.equal(O.out_to_nchw(out, Co, ho, wo, N), y)
    g_col = O.nchw_to_out_col(gy)
    gW, gX = torch.zeros_like(W_col), torch.zeros_like(X_col)
    adder_cuda.ADDER_BACKWARD(g_col, X_col, W_col, gW, gX)
    assert torch.equal(gW.view_as(w), gw)
    assert torch.equal(O.col2im(gX, x.shape, k, s, p), gx)
    gW2, gX2 = torch.zeros_like(W_col), torch.zeros_like(X_col)
    adder_cuda.ADDER_CONV_WEIGHT(g_col, X_col, W_col, gW2)
    adder_cuda.ADDER_CONV_INPUT(g_col, X_col, W_col, gX2)
    assert torch.equal(gW2, gW) and torch.equal(gX2, gX)
