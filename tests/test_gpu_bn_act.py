"""Fused BatchNorm + residual + ReLU (csrc/bn_act.hip) against torch's own ops evaluated in float64."""
import pytest
import torch
import torch.nn.functional as F

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (N, C, H, W)
SHAPES = [(8, 16, 32, 32), (4, 64, 8, 8), (256, 16, 32, 32), (3, 5, 7, 7), (2, 10, 1, 1), (5, 33, 6, 10),
          (2, 3, 4, 8), (3, 7, 16, 6)]   # the last two: the smallest planes that get a ReLU sign mask (32 and 96 elements)


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


@pytest.mark.parametrize("shape", [(6, 12, 8, 8), (3, 7, 5, 3), (16, 4, 16, 32)], ids=str)
def test_statistics_survive_a_mean_far_from_zero(shape, gpu):
    """Inputs with |mean| = 1000 x std (x = -100 + 0.1 z): a sum of fp32 squares has no digit of the variance left;
    the statistics pass squares and sums in float64.  No ReLU here -- with the mean kept in float32 a gate that
    sits on a value of 1e-4 may flip, which is not what this test is about."""
    from addernetcuda_amd.bn_act import BatchNormAct2d
    g = torch.Generator().manual_seed(sum(shape))
    x = torch.randn(shape, generator=g) * 0.1 - 100.0
    dy = torch.randn(shape, generator=g)
    m = BatchNormAct2d(shape[1], relu=False).to(gpu).train()
    xg = x.to(gpu).requires_grad_(True)
    y = m(xg)
    y.backward(dy.to(gpu))
    torch.cuda.synchronize()
    want = _reference(x, None, m.weight.detach().cpu(), m.bias.detach().cpu(), False, dy, m.eps)
    # x - mean carries the float32 spacing of values around 100 (7.6e-6) over a std of 0.1
    assert_close(y, want[0], "y", rtol=1e-3, atol=1e-3)
    assert_close(xg.grad, want[1], "dx", rtol=1e-3, atol=1e-2)
    assert_close(m.running_var, want[6], "running_var", rtol=1e-4, atol=1e-6)


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


# (N, Ci, H, W, Co, k, stride, pad): one case per tiled forward kernel, with channel / tile / width tails
STATS_CASES = [
    (3, 16, 32, 32, 16, 3, 1, 1), (2, 32, 16, 16, 32, 3, 1, 1), (5, 64, 8, 8, 64, 3, 1, 1),
    (2, 5, 12, 20, 7, 3, 1, 1), (2, 16, 32, 32, 32, 3, 2, 1), (3, 32, 16, 16, 64, 3, 2, 1),
    (2, 16, 14, 14, 20, 3, 1, 1), (2, 9, 10, 18, 8, 3, 1, 1),
    (2, 16, 32, 32, 32, 1, 2, 0), (3, 32, 16, 16, 64, 1, 2, 0), (2, 8, 8, 8, 4, 1, 1, 0), (3, 12, 7, 7, 20, 1, 1, 0),
    (2, 6, 9, 9, 10, 1, 2, 0), (3, 64, 14, 14, 72, 1, 1, 0), (2, 64, 28, 28, 72, 1, 2, 0),   # 1x1 kernels, element-wise and tiled
    (3, 84, 16, 16, 48, 1, 1, 0), (5, 68, 8, 8, 20, 1, 1, 0), (2, 76, 20, 20, 24, 1, 2, 0),   # ... units of four input channels
    (2, 8, 24, 40, 12, 3, 1, 1), (3, 8, 20, 24, 8, 3, 1, 1), (2, 16, 56, 56, 8, 3, 1, 1),    # wide maps, 8- and 4-row tiles
    (2, 64, 56, 56, 72, 1, 2, 0), (3, 72, 14, 14, 130, 1, 2, 0),                             # strided 1x1, 64-channel blocks
]


@pytest.mark.parametrize("case", STATS_CASES, ids=str)
def test_forward_statistics_epilogue_sums_the_output(case, gpu):
    """The partial sums the adder forward writes for the BatchNorm behind it add up to sum(y) and sum(y*y)
    per channel, and the output itself is the one the plain call gives."""
    from addernetcuda_amd import adder
    N, Ci, H, W, Co, k, s, p = case
    g = torch.Generator().manual_seed(sum(case))
    x = torch.randn(N, Ci, H, W, generator=g).to(gpu)
    w = (torch.randn(Co, Ci, k, k, generator=g) * (2.0 / (Ci * k * k)) ** 0.5).to(gpu)
    y_plain = adder.adder2d_function(x, w, s, p)
    y, stats = adder.adder2d_function_with_stats(x, w, s, p)
    torch.cuda.synchronize()
    assert stats is not None and stats.dtype == torch.float64 and stats.shape[0] == Co and stats.shape[2] == 2
    assert torch.equal(y, y_plain)
    tot = stats.sum(dim=1).cpu()
    yd = y.double().cpu()
    assert torch.allclose(tot[:, 0], yd.sum(dim=(0, 2, 3)), rtol=1e-6, atol=1e-6)
    assert torch.allclose(tot[:, 1], (yd * yd).sum(dim=(0, 2, 3)), rtol=1e-6, atol=1e-6)


def test_layers_without_the_epilogue_report_none(gpu):
    from addernetcuda_amd import adder
    x = torch.randn(2, 8, 8, 8, device=gpu)
    for k, s, p in ((5, 1, 2), (1, 3, 0), (3, 1, 0)):
        w = torch.randn(4, 8, k, k, device=gpu)
        y, stats = adder.adder2d_function_with_stats(x, w, s, p)
        assert stats is None and torch.equal(y, adder.adder2d_function(x, w, s, p))
    layer = adder.adder2d(8, 4, 3, padding=1, bias=True).to(gpu)
    assert layer.forward_with_stats(x)[1] is None          # the bias would not be in the sums
    # a tensor that is not 16-byte aligned: whichever kernel takes it, the output is the plain call's and the
    # statistics, if any, are its sums
    for shape, co, k, p in (((2, 64, 8, 8), 64, 1, 0), ((2, 16, 8, 8), 8, 3, 1)):
        numel = shape[0] * shape[1] * shape[2] * shape[3]
        xm = torch.randn(numel + 1, device=gpu)[1:].view(shape)
        assert xm.data_ptr() % 16 == 4
        w = torch.randn(co, shape[1], k, k, device=gpu)
        y, stats = adder.adder2d_function_with_stats(xm, w, 1, p)
        want = adder.adder2d_function(xm.clone(), w, 1, p)
        assert torch.allclose(y, want, rtol=1e-6, atol=1e-4)
        if stats is not None:
            assert torch.allclose(stats.sum(dim=1)[:, 0], want.double().sum(dim=(0, 2, 3)), rtol=1e-6, atol=1e-3)


@pytest.mark.parametrize("with_res", [False, True])
def test_batchnorm_from_precomputed_statistics_equals_its_own_pass(with_res, gpu):
    from addernetcuda_amd import adder
    from addernetcuda_amd.bn_act import BatchNormAct2d
    g = torch.Generator().manual_seed(11)
    x = torch.randn(6, 16, 16, 16, generator=g).to(gpu)
    layer = adder.adder2d(16, 24, 3, padding=1).to(gpu)
    res = torch.randn(6, 24, 16, 16, generator=g).to(gpu) if with_res else None
    # relu off: a ReLU gate that flips on a last-bit difference of the statistics would dominate the comparison
    a, b = BatchNormAct2d(24, relu=False).to(gpu).train(), BatchNormAct2d(24, relu=False).to(gpu).train()
    dy = torch.randn(6, 24, 16, 16, generator=g).to(gpu)   # (sum of squares of a normalised tensor is constant)
    outs = []
    for bn, fused in ((a, True), (b, False)):
        xin = x.clone().requires_grad_(True)
        layer.zero_grad()
        if fused:
            y, stats = layer.forward_with_stats(xin)
            assert stats is not None
            out = bn(y, residual=res, stats=stats)
        else:
            out = bn(layer(xin), residual=res)
        (out * dy).sum().backward()
        outs.append((out.detach(), xin.grad, layer.adder.grad.clone(), bn.weight.grad, bn.running_mean.clone(),
                     bn.running_var.clone()))
    torch.cuda.synchronize()
    for got, want, name in zip(outs[0], outs[1], ("y", "dx", "dw", "dgamma", "running_mean", "running_var")):
        # the two paths add the same numbers in a different order: statistics agree to ~1e-7, what is
        # back-propagated through them to ~1e-5 of the largest entry
        assert torch.allclose(got, want, rtol=1e-4, atol=1e-4 * max(1.0, want.abs().max().item())), name
    assert int(a.num_batches_tracked) == 1


def test_a_residual_that_is_not_shaped_like_x_is_added_the_way_torch_adds_it(gpu):
    """The kernels read the residual as a dense fp32 tensor shaped like x; a broadcast shape or another dtype
    goes through torch's add instead of being misread."""
    from addernetcuda_amd.bn_act import BatchNormAct2d
    torch.manual_seed(5)
    x = torch.randn(4, 6, 8, 8, device=gpu)
    for res in (torch.randn(1, 6, 1, 1, device=gpu), torch.randn(4, 6, 8, 8, device=gpu).double()):
        for relu in (True, False):
            bn = BatchNormAct2d(6, relu=relu).to(gpu)
            ref = torch.nn.BatchNorm2d(6).to(gpu).double()
            want = ref(x.double()) + res.double()
            want = torch.relu(want) if relu else want
            got = bn(x, residual=res)
            assert torch.allclose(got.double(), want, rtol=1e-5, atol=1e-5)
            assert torch.allclose(bn.running_var.double(), ref.running_var, rtol=1e-5, atol=1e-6)
