"""The classifier head kernels (csrc/head.hip: average pool over the map, bias-free 1x1 fc, training-mode
BatchNorm2d; resnet20.py:55-57, 89-93 of the reference) against the same torch modules evaluated in float64."""
import copy

import pytest
import torch
import torch.nn as nn

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (N, C, H, W, classes)
SHAPES = [(256, 64, 8, 8, 10), (5, 16, 4, 4, 3), (32, 128, 2, 2, 32), (4, 1, 16, 16, 1), (7, 256, 2, 4, 10),
          (64, 64, 8, 8, 100 // 4)]


def _modules(C, J, seed):
    torch.manual_seed(seed)
    fc = nn.Conv2d(C, J, 1, bias=False)
    bn = nn.BatchNorm2d(J)
    with torch.no_grad():
        bn.weight.uniform_(0.5, 1.5)
        bn.bias.normal_(0, 0.3)
        bn.running_mean.normal_(0, 0.1)
        bn.running_var.uniform_(0.5, 2.0)
    return fc, bn


@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_matches_the_modules_in_float64(shape, gpu):
    from addernetcuda_amd.head import head_applies, pool_fc_bn
    N, C, H, W, J = shape
    fc, bn = _modules(C, J, 11 + sum(shape))
    g = torch.Generator().manual_seed(3 + sum(shape))
    x = torch.randn(N, C, H, W, generator=g) * 2 + 0.5
    dy = torch.randn(N, J, generator=g)

    # float64 truth with the very same modules
    fc64, bn64 = copy.deepcopy(fc).double(), copy.deepcopy(bn).double()
    x64 = x.double().requires_grad_(True)
    y64 = bn64(fc64(x64.mean((2, 3), keepdim=True))).view(N, J)
    y64.backward(dy.double())

    fcg, bng = copy.deepcopy(fc).to(gpu), copy.deepcopy(bn).to(gpu)
    xg = x.to(gpu).requires_grad_(True)
    assert head_applies(xg, fcg, bng)
    y = pool_fc_bn(xg, fcg, bng)
    y.backward(dy.to(gpu))
    torch.cuda.synchronize()
    assert_close(y, y64, "logits", rtol=1e-4, atol=1e-4)
    assert_close(bng.running_mean, bn64.running_mean, "running_mean", rtol=1e-5, atol=1e-6)
    assert_close(bng.running_var, bn64.running_var, "running_var", rtol=1e-5, atol=1e-6)
    assert int(bng.num_batches_tracked) == int(bn64.num_batches_tracked) == 1
    scale = lambda t: max(1.0, float(t.abs().max()))
    for got, want, name in ((xg.grad, x64.grad, "dx"), (fcg.weight.grad, fc64.weight.grad, "dw"),
                            (bng.weight.grad, bn64.weight.grad, "dgamma"), (bng.bias.grad, bn64.bias.grad, "dbeta")):
        s = scale(want)
        assert_close(got / s, want / s, name, rtol=1e-4, atol=2e-5)


def test_two_runs_give_the_same_bits(gpu):
    from addernetcuda_amd.head import pool_fc_bn
    fc, bn = _modules(64, 10, 5)
    x = torch.randn(256, 64, 8, 8, generator=torch.Generator().manual_seed(9)).to(gpu)
    dy = torch.randn(256, 10, generator=torch.Generator().manual_seed(10)).to(gpu)
    results = []
    for _ in range(2):
        fcg, bng = copy.deepcopy(fc).to(gpu), copy.deepcopy(bn).to(gpu)
        xg = x.clone().requires_grad_(True)
        y = pool_fc_bn(xg, fcg, bng)
        y.backward(dy)
        results.append((y.detach(), xg.grad, fcg.weight.grad, bng.weight.grad, bng.bias.grad, bng.running_var))
    torch.cuda.synchronize()
    for a, b in zip(*results):
        assert torch.equal(a, b)


def test_the_model_takes_the_head_and_agrees_with_the_modules(gpu, monkeypatch):
    """ResNet-20 with and without the head kernels: same logits and gradients to float32 accuracy; and what the
    kernels do not cover (eval mode) runs through the modules."""
    from addernetcuda_amd import resnet20 as r20
    torch.manual_seed(0)
    model_a = r20.resnet20().to(gpu).train()
    model_b = copy.deepcopy(model_a)
    x = torch.randn(8, 3, 32, 32, generator=torch.Generator().manual_seed(1)).to(gpu)
    calls = []
    real = r20.pool_fc_bn
    monkeypatch.setattr(r20, "pool_fc_bn", lambda *a: (calls.append(1), real(*a))[1])
    ya = model_a(x)
    assert calls == [1]
    monkeypatch.setattr(r20, "head_applies", lambda *a: False)
    yb = model_b(x)
    assert calls == [1]
    assert_close(ya, yb.double(), "logits", rtol=1e-4, atol=1e-4)
    ya.square().mean().backward()
    yb.square().mean().backward()
    for (name, pa), pb in zip(model_a.named_parameters(), model_b.parameters()):
        s = max(1e-3, float(pb.grad.abs().max()))
        assert_close(pa.grad / s, (pb.grad / s).double(), name, rtol=2e-3, atol=2e-3)
    assert_close(model_a.bn2.running_var, model_b.bn2.running_var.double(), "running_var", rtol=1e-4, atol=1e-6)
    monkeypatch.undo()
    model_a.eval()
    with torch.no_grad():
        assert model_a(x).shape == (8, 10)


def test_refusals(gpu):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, ADDER_ERR_UNSUPPORTED, ADDER_ERR_NULL_POINTER, ADDER_ERR_ALIAS
    from addernetcuda_amd.head import head_applies
    assert lib.adder_head_supported(256, 64, 64, 10) == 1
    assert lib.adder_head_supported(1, 64, 64, 10) == 0        # batch statistics of one value
    assert lib.adder_head_supported(8, 48, 64, 10) == 0        # channels that do not divide the workgroup
    assert lib.adder_head_supported(5, 2, 64, 10) == 0         # a pooled matrix that is not whole float4 groups
    assert lib.adder_head_supported(8, 64, 49, 10) == 0        # a 7x7 plane
    assert lib.adder_head_supported(8, 64, 64, 33) == 0
    assert lib.adder_head_supported(4096, 256, 64, 10) == 0    # the pooled matrix would not fit the LDS
    t = torch.zeros(8 * 64 * 64, device=gpu)
    st = stream_ptr(gpu)
    args = lambda x, pooled: (ptr(x), ptr(t), ptr(t), ptr(t), ptr(pooled), ptr(t), ptr(t), ptr(t), ptr(t), None, None, None,
                              0.1, 1e-5)
    assert lib.adder_head_fwd_f32(*args(t, t), 8, 64, 49, 10, st) == ADDER_ERR_UNSUPPORTED
    assert lib.adder_head_fwd_f32(*args(None, t), 8, 64, 64, 10, st) == ADDER_ERR_NULL_POINTER
    assert lib.adder_head_fwd_f32(*args(t, t), 8, 64, 64, 10, st) == ADDER_ERR_ALIAS
    fc, bn = nn.Conv2d(64, 10, 1, bias=True).to(gpu), nn.BatchNorm2d(10).to(gpu)
    assert not head_applies(torch.zeros(8, 64, 8, 8, device=gpu), fc, bn)      # an fc with a bias


@pytest.mark.parametrize("shape", [(256, 10), (7, 3), (1, 1), (1500, 32), (64, 17)], ids=str)
def test_cross_entropy_matches_torch_in_float64(shape, gpu):
    from addernetcuda_amd.head import cross_entropy
    N, J = shape
    g = torch.Generator().manual_seed(5 + N + J)
    logits = torch.randn(N, J, generator=g) * 4
    target = torch.randint(0, J, (N,), generator=g)
    l64 = logits.double().requires_grad_(True)
    ref = torch.nn.functional.cross_entropy(l64, target)
    ref.backward(torch.tensor(0.7, dtype=torch.float64))
    lg = logits.to(gpu).requires_grad_(True)
    loss = cross_entropy(lg, target.to(gpu))
    assert loss.shape == () and loss.grad_fn is not None and "_cross_entropy" in type(loss.grad_fn).__name__
    loss.backward(torch.tensor(0.7, device=gpu))
    torch.cuda.synchronize()
    assert_close(loss, ref.detach(), "loss", rtol=1e-6, atol=1e-6)
    assert_close(lg.grad, l64.grad, "gradient of the logits", rtol=1e-5, atol=1e-7)
    # two runs: the same bits
    lg2 = logits.to(gpu).requires_grad_(True)
    loss2 = cross_entropy(lg2, target.to(gpu))
    loss2.backward(torch.tensor(0.7, device=gpu))
    assert torch.equal(loss2, loss) and torch.equal(lg2.grad, lg.grad)


def test_cross_entropy_leaves_the_rest_to_torch(gpu):
    from addernetcuda_amd.head import cross_entropy
    logits = torch.randn(8, 100, device=gpu, requires_grad=True)      # more classes than the kernel keeps in registers
    target = torch.randint(0, 100, (8,), device=gpu)
    loss = cross_entropy(logits, target)
    assert "_cross_entropy" not in type(loss.grad_fn).__name__
    assert torch.equal(loss, torch.nn.functional.cross_entropy(logits, target))
    cpu = cross_entropy(torch.randn(4, 5), torch.randint(0, 5, (4,)))
    assert cpu.shape == ()
