"""adder layer + BatchNorm + shortcut + ReLU as one autograd node (addernetcuda_amd/unit.py): chains of such
nodes against the same chain built from the oracle's adder layer and torch's own BatchNorm / ReLU in float64,
and the bookkeeping that decides when a BatchNorm backward is folded into its neighbours' kernels."""
import copy

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from tests.util import assert_close

pytestmark = pytest.mark.gpu


class _Chain(nn.Module):
    """The layers of the chain the tests run (_forward_units / _forward_reference): a ReLU input -> [a, bn, relu] ->
    [a2, bn, relu] -> [b, bn, + shortcut, relu] -> [c (strided), bn, relu] -> [d, bn]; a2 / bna2 are added by _nets."""

    def __init__(self, ch, stride, adder2d_cls, bn_cls):
        super().__init__()
        mk = lambda ci, co, s: adder2d_cls(ci, co, 3, stride=s, padding=1, bias=False, eta=0.1)
        self.a, self.b, self.c, self.d = mk(ch, ch, 1), mk(ch, ch, 1), mk(ch, 2 * ch, stride), mk(2 * ch, 2 * ch, 1)
        self.bna, self.bnb, self.bnc, self.bnd = bn_cls(ch, True), bn_cls(ch, True), bn_cls(2 * ch, True), bn_cls(2 * ch, False)
        for bn in (self.bna, self.bnb, self.bnc, self.bnd):
            nn.init.uniform_(bn.weight, 0.5, 1.5)
            nn.init.normal_(bn.bias, 0.0, 0.2)


def _forward_units(net, x):
    from addernetcuda_amd.unit import adder_bn_act
    x1 = adder_bn_act(net.a, net.bna, x)
    mid, short = adder_bn_act(net.a2, net.bna2, x1, with_shortcut=True)       # first half of a residual block
    x2 = adder_bn_act(net.b, net.bnb, mid, residual=short)                   # second half: + shortcut, relu
    x3 = adder_bn_act(net.c, net.bnc, x2)                                    # strided layer
    return adder_bn_act(net.d, net.bnd, x3)                                  # no ReLU behind the last BatchNorm


def _forward_separate(net, x):
    """The same chain with the adder layers and the BatchNorms as separate autograd nodes (the library's own
    unfolded path: identical forward kernels, so identical activations and ReLU gates)."""
    def cb(conv, bn, t, residual=None):
        out, stats = conv.forward_with_stats(t)
        return bn(out, residual=residual, stats=stats)
    x1 = cb(net.a, net.bna, x)
    out, stats, short = net.a2.forward_with_stats(x1, with_shortcut=True)
    mid = net.bna2(out, stats=stats)
    x2 = cb(net.b, net.bnb, mid, short)
    x3 = cb(net.c, net.bnc, x2)
    return cb(net.d, net.bnd, x3)


def _mostly_close(actual, expected, what, rtol, atol, max_bad):
    """allclose for all but a fraction ``max_bad`` of the elements: behind several BatchNorm + ReLU stages a float32
    activation within 1e-6 of zero now and then falls on the other side of the gate than its float64 twin, which
    moves the gradients in the cone below it by a percent or so."""
    a, e = actual.detach().double().cpu(), expected.detach().double().cpu()
    bad = ((a - e).abs() > atol + rtol * e.abs()).double().sum().item()
    assert bad <= max(1.0, max_bad * a.numel()), f"{what}: {int(bad)} of {a.numel()} elements outside rtol={rtol} atol={atol}"
    assert (a - e).abs().max().item() <= 0.05 * e.abs().max().item() + atol, what


def _forward_reference(net, x):
    bn = lambda m, t: F.batch_norm(t, None, None, m.weight, m.bias, True, 0.1, m.eps)
    x1 = F.relu(bn(net.bna, net.a(x)))
    mid = F.relu(bn(net.bna2, net.a2(x1)))
    x2 = F.relu(bn(net.bnb, net.b(mid)) + x1)
    x3 = F.relu(bn(net.bnc, net.c(x2)))
    return bn(net.bnd, net.d(x3))


def _nets(gpu, ch, stride, seed):
    from addernetcuda_amd.adder import adder2d
    from addernetcuda_amd.bn_act import BatchNormAct2d
    from oracle import adder_oracle
    torch.manual_seed(seed)
    hip = _Chain(ch, stride, adder2d, lambda c, relu: BatchNormAct2d(c, relu=relu))
    hip.a2 = adder2d(ch, ch, 3, stride=1, padding=1, bias=False, eta=0.1)
    hip.bna2 = BatchNormAct2d(ch, relu=True)
    hip = hip.to(gpu).train()
    ref = _Chain(ch, stride, adder_oracle.adder2d, lambda c, relu: nn.BatchNorm2d(c))
    ref.a2 = adder_oracle.adder2d(ch, ch, 3, stride=1, padding=1, bias=False, eta=0.1)
    ref.bna2 = nn.BatchNorm2d(ch)
    ref.load_state_dict(hip.state_dict())
    return hip, ref.to(gpu).double().train()


# (N, channels, H, W, stride of layer c, BatchNorm backwards that are NOT folded away).  Only the last unit gets its
# gradient from somewhere else; in the last case the strided layer's output rows (10 wide) are not whole float4
# groups, so neither it nor the layer behind it has the kernels, and three units run their own BatchNorm backward.
@pytest.mark.parametrize("shape", [(8, 16, 32, 32, 1, 1), (8, 16, 32, 32, 2, 1), (6, 32, 16, 16, 2, 1),
                                   (4, 64, 8, 8, 1, 1), (3, 12, 16, 20, 2, 3)], ids=str)
def test_chain_of_units_matches_float64_reference(shape, gpu, monkeypatch):
    N, ch, H, W, stride, unfused = shape
    from addernetcuda_amd import unit
    hip, ref = _nets(gpu, ch, stride, 7 + sum(shape))
    g = torch.Generator(device=gpu).manual_seed(3)
    x = torch.relu(torch.randn(N, ch, H, W, device=gpu, generator=g)).requires_grad_(True)
    x64 = x.detach().double().requires_grad_(True)
    unfused_calls = []
    real = unit.bn_backward
    monkeypatch.setattr(unit, "bn_backward", lambda *a, **k: (unfused_calls.append(1), real(*a, **k))[1])
    out = _forward_units(hip, x)
    want = _forward_reference(ref, x64)
    assert_close(out, want, "output", rtol=1e-4, atol=1e-3)
    gout = torch.randn(out.shape, device=gpu, generator=g)
    out.backward(gout)
    want.backward(gout.double())
    torch.cuda.synchronize()
    assert len(unfused_calls) == unfused
    _mostly_close(x.grad, x64.grad, "grad of the input", 1e-3, 1e-3, 0.005)
    got, truth = dict(hip.named_parameters()), dict(ref.named_parameters())
    for name, p in got.items():
        scale = max(1.0, float(truth[name].grad.abs().max()))
        _mostly_close(p.grad / scale, truth[name].grad / scale, name, 1e-3, 2e-3, 0.005)
    # and tightly against the same kernels run as separate autograd nodes (same activations, same gates)
    twin = copy.deepcopy(hip)
    for p in twin.parameters():
        p.grad = None
    xs = x.detach().clone().requires_grad_(True)
    _forward_separate(twin, xs).backward(gout)
    torch.cuda.synchronize()
    assert_close(x.grad, xs.grad, "grad of the input vs separate nodes", rtol=1e-4, atol=1e-4)
    for name, p in twin.named_parameters():
        scale = max(1.0, float(p.grad.abs().max()))
        assert_close(got[name].grad / scale, p.grad / scale, name + " vs separate nodes", rtol=1e-4, atol=1e-4)


def test_hand_over_is_declined_when_autograd_sums_gradients(gpu, monkeypatch):
    """A unit's output that also feeds something else: autograd adds the two gradients into a new tensor, which the
    unit must not mistake for the consumer's dz -- it runs its own BatchNorm backward, and the result is right."""
    from addernetcuda_amd import unit
    from addernetcuda_amd.unit import adder_bn_act
    hip, ref = _nets(gpu, 16, 1, 11)
    x = torch.relu(torch.randn(4, 16, 16, 16, device=gpu)).requires_grad_(True)
    x64 = x.detach().double().requires_grad_(True)
    calls = []
    real = unit.bn_backward
    monkeypatch.setattr(unit, "bn_backward", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    x1 = adder_bn_act(hip.a, hip.bna, x)
    out = adder_bn_act(hip.b, hip.bnb, x1) + 3.0 * x1          # x1 has two consumers
    bn = lambda m, t: F.batch_norm(t, None, None, m.weight, m.bias, True, 0.1, m.eps)
    r1 = F.relu(bn(ref.bna, ref.a(x64)))
    want = F.relu(bn(ref.bnb, ref.b(r1))) + 3.0 * r1
    gout = torch.randn_like(out)
    out.backward(gout)
    want.backward(gout.double())
    assert len(calls) == 2
    assert_close(x.grad, x64.grad, "grad of the input", rtol=1e-3, atol=1e-3)
    assert_close(hip.bna.weight.grad, ref.bna.weight.grad, "dgamma", rtol=1e-3, atol=1e-3)


def test_frozen_weights_and_eval_mode_take_the_plain_paths(gpu):
    from addernetcuda_amd.unit import adder_bn_act
    hip, ref = _nets(gpu, 16, 1, 13)
    hip.a.adder.requires_grad_(False)
    ref.a.adder.requires_grad_(False)
    x = torch.relu(torch.randn(4, 16, 16, 16, device=gpu)).requires_grad_(True)
    x64 = x.detach().double().requires_grad_(True)
    out = adder_bn_act(hip.b, hip.bnb, adder_bn_act(hip.a, hip.bna, x))
    bn = lambda m, t: F.batch_norm(t, None, None, m.weight, m.bias, True, 0.1, m.eps)
    want = F.relu(bn(ref.bnb, ref.b(F.relu(bn(ref.bna, ref.a(x64))))))
    gout = torch.randn_like(out)
    out.backward(gout)
    want.backward(gout.double())
    assert hip.a.adder.grad is None
    assert_close(x.grad, x64.grad, "grad of the input", rtol=1e-3, atol=1e-3)
    hip.eval()
    with torch.no_grad():
        y = adder_bn_act(hip.a, hip.bna, x)
        assert_close(y, F.relu(hip.bna(hip.a(x))), "eval-mode output")


def test_batched_eta_scaling_with_units(gpu):
    """Inside a batched_eta_scaling() block the units stage their weight gradients (the kernel that stages is also
    the one that forms the layer's output gradient): same gradients as without the block."""
    from addernetcuda_amd.adder import batched_eta_scaling
    hip, _ = _nets(gpu, 16, 2, 17)
    twin = copy.deepcopy(hip)
    x = torch.relu(torch.randn(8, 16, 32, 32, device=gpu))
    gout = None
    grads = []
    for net, batched in ((hip, True), (twin, False)):
        xi = x.clone().requires_grad_(True)
        out = _forward_units(net, xi)
        gout = torch.randn_like(out) if gout is None else gout
        if batched:
            with batched_eta_scaling():
                out.backward(gout)
        else:
            out.backward(gout)
        grads.append((xi.grad, {n: p.grad for n, p in net.named_parameters()}))
    assert torch.equal(grads[0][0], grads[1][0])
    for name in grads[0][1]:
        assert_close(grads[0][1][name], grads[1][1][name], name, rtol=1e-6, atol=1e-7)


def test_resnet20_runs_three_batchnorm_backwards_of_its_own(gpu, monkeypatch):
    """Of the 21 BatchNorms behind convolutions in ResNet-20, 18 have their backward folded into the adder kernels
    around them (the stem's included); the two downsample BatchNorms (1x1 layers, no such kernels) and the last one
    (its gradient comes from the pooling layer) run their own two passes."""
    from addernetcuda_amd import unit, resnet20 as r20
    calls = []
    for mod in (unit, r20):
        real = mod.bn_backward
        monkeypatch.setattr(mod, "bn_backward", lambda *a, _real=real, **k: (calls.append(1), _real(*a, **k))[1])
    torch.manual_seed(0)
    net = r20.resnet20(eta=0.1).to(gpu).train()
    x = torch.randn(8, 3, 32, 32, device=gpu)
    F.cross_entropy(net(x), torch.randint(0, 10, (8,), device=gpu)).backward()
    torch.cuda.synchronize()
    assert len(calls) == 3
    assert all(p.grad is not None and torch.isfinite(p.grad).all() for p in net.parameters())


def _unit_chain_grads(net, x, gout, forward=None):
    xi = x.clone().requires_grad_(True)
    out = (forward or _forward_units)(net, xi)
    out.backward(gout)
    return xi.grad, {n: p.grad.clone() for n, p in net.named_parameters()}


def test_units_under_activation_checkpointing(gpu):
    """torch.utils.checkpoint re-runs the forward inside the backward pass (new nodes, new links, new tensors):
    the chain of units must give the gradients it gives without checkpointing."""
    from torch.utils.checkpoint import checkpoint
    hip, _ = _nets(gpu, 16, 2, 23)
    twin = copy.deepcopy(hip)
    x = torch.relu(torch.randn(4, 16, 32, 32, device=gpu))
    gout = torch.randn(4, 32, 16, 16, device=gpu)
    gx0, gp0 = _unit_chain_grads(twin, x, gout)
    xi = x.clone().requires_grad_(True)
    out = checkpoint(lambda t: _forward_units(hip, t), xi, use_reentrant=False)
    out.backward(gout)
    assert_close(xi.grad, gx0, "input gradient under checkpointing", rtol=1e-5, atol=1e-5)
    for n, p in hip.named_parameters():
        scale = max(1.0, float(gp0[n].abs().max()))
        assert_close(p.grad / scale, gp0[n] / scale, n + " under checkpointing", rtol=1e-5, atol=1e-5)


def test_autograd_grad_with_respect_to_the_chain_input(gpu):
    """torch.autograd.grad(out, x): only the input gradient is asked for, no weight gradient -- the hand-over needs
    the weight-gradient kernel (it is the one that forms a layer's output gradient), so every unit must take the
    plain path and still deliver the same input gradient as a full backward pass."""
    hip, _ = _nets(gpu, 16, 2, 29)
    x = torch.relu(torch.randn(4, 16, 32, 32, device=gpu))
    gout = torch.randn(4, 32, 16, 16, device=gpu)
    gx0, _ = _unit_chain_grads(copy.deepcopy(hip), x, gout)
    xi = x.clone().requires_grad_(True)
    (gx,) = torch.autograd.grad(_forward_units(hip, xi), xi, gout)
    assert_close(gx, gx0, "input gradient from autograd.grad", rtol=1e-4, atol=1e-4)
    assert all(p.grad is None for p in hip.parameters())
    # ... and with respect to one weight in the middle of the chain only
    xi = x.clone().requires_grad_(True)
    (gw,) = torch.autograd.grad(_forward_units(hip, xi), hip.b.adder, gout)
    _, gp0 = _unit_chain_grads(copy.deepcopy(hip), x, gout)
    scale = max(1.0, float(gp0["b.adder"].abs().max()))
    assert_close(gw / scale, gp0["b.adder"] / scale, "one weight's gradient from autograd.grad", rtol=1e-4, atol=1e-4)


def test_weight_hook_inside_batched_eta_scaling_sees_the_finished_gradient(gpu):
    """A register_hook on an adder weight runs during the backward pass; inside batched_eta_scaling() that layer is
    therefore not taken over (its gradient would be unfinished slabs at that moment) while the others still are."""
    from addernetcuda_amd import adder as adder_mod
    from addernetcuda_amd.adder import batched_eta_scaling
    hip, _ = _nets(gpu, 16, 1, 31)
    x = torch.relu(torch.randn(4, 16, 16, 16, device=gpu))
    gout = torch.randn(4, 32, 16, 16, device=gpu)
    _, gp0 = _unit_chain_grads(copy.deepcopy(hip), x, gout)
    seen = {}
    handle = hip.b.adder.register_hook(lambda g: seen.__setitem__("b", g.clone()))
    xi = x.clone().requires_grad_(True)
    out = _forward_units(hip, xi)
    with batched_eta_scaling():
        out.backward(gout)
        pending = [id(entry[0]) for entry in adder_mod._eta_batch]
    handle.remove()
    assert id(hip.b.adder) not in pending and id(hip.a.adder) in pending
    assert_close(seen["b"], gp0["b.adder"], "gradient seen by the hook", rtol=1e-5, atol=1e-6)
    for n, p in hip.named_parameters():
        scale = max(1.0, float(gp0[n].abs().max()))
        assert_close(p.grad / scale, gp0[n] / scale, n, rtol=1e-5, atol=1e-6)
