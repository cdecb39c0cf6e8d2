"""Fused BatchNorm + residual + ReLU (csrc/bn_act.hip) against torch's own ops evaluated in float64."""
import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (N, C, H, W)
SHAPES = [(8, 16, 32, 32), (4, 64, 8, 8), (256, 16, 32, 32), (3, 5, 7, 7), (2, 10, 1, 1), (5, 33, 6, 10)]


def _reference(x, res, gamma, beta, relu, dy, eps):
    x, gamma, beta, dy = (t.double().clone().requires_grad_(t is not dy) for t in (x, gamma, beta, dy))
    res = res.double().clone().requires_grad_(True) if res is not None else None
    rm, rv = torch.zeros_like(gamma), torch.ones_like(gamma)
    out = F.batch_norm(x, rm, rv, gamma, beta, training=True, momentum=0.1, eps=eps)
    if res is not None:
        out = out + res
    if relu:
        out = F.relu(out)
    out.backward(dy)
    return out.detach(), x.grad, (res.grad if res is not None else None), gamma.grad, beta.grad, rm, rv


@pytest.mark.parametrize("shape", SHAPES, ids=str)
@pytest.mark.parametrize("relu", [True, False])
@pytest.mark.parametrize("with_res", [True, False])
def test_matches_torch_in_float64(shape, relu, with_res, gpu):
    from addernetcuda_amd.bn_act import BatchNormAct2d
    N, C, H, W = shape
    if N * H * W < 2:
        pytest.skip("batch norm needs more than one value per channel")
    g = torch.Generator().manual_seed(N + C + H)
    x = torch.randn(shape, generator=g) * 30 - 140          # adder outputs: large negative mean
    res = torch.randn(shape, generator=g) if with_res else None
    dy = torch.randn(shape, generator=g)
    m = BatchNormAct2d(C, relu=relu).to(gpu).train()
    with torch.no_grad():
        m.weight.copy_(torch.rand(C, generator=g) + 0.5)
        m.bias.copy_(torch.randn(C, generator=g))
    xg = x.to(gpu).requires_grad_(True)
    rg = res.to(gpu).requires_grad_(True) if with_res else None
    y = m(xg, rg)
    y.backward(dy.to(gpu))
    torch.cuda.synchronize()
    want = _reference(x, res, m.weight.detach().cpu(), m.bias.detach().cpu(), relu, dy, m.eps)
    assert_close(y, want[0], "y")
    assert_close(xg.grad, want[1], "dx")
    if with_res:
        assert_close(rg.grad, want[2], "dresidual")
    assert_close(m.weight.grad, want[3], "dgamma", rtol=1e-5, atol=1e-3)
    assert_close(m.bias.grad, want[4], "dbeta", rtol=1e-5, atol=1e-3)
    assert_close(m.running_mean, want[5], "running_mean")
    assert_close(m.running_var, want[6], "running_var", rtol=1e-5, atol=1e-3)
    assert int(m.num_batches_tracked) == 1


def test_eval_mode_and_state_dict_are_those_of_batchnorm2d(gpu):
    from addernetcuda_amd.bn_act import BatchNormAct2d
    a = BatchNormAct2d(8, relu=True).to(gpu)
    b = torch.nn.BatchNorm2d(8).to(gpu)
    assert set(a.state_dict()) == set(b.state_dict())
    x = torch.randn(4, 8, 6, 6, device=gpu)
    a.train(), b.train()
    for _ in range(3):
        ya, yb = a(x), F.relu(b(x))
        assert torch.allclose(ya, yb, rtol=1e-4, atol=1e-5)
    assert torch.allclose(a.running_mean, b.running_mean, atol=1e-6) and torch.allclose(a.running_var, b.running_var, atol=1e-5)
    a.eval(), b.eval()
    assert torch.allclose(a(x), F.relu(b(x)), rtol=1e-5, atol=1e-6)
