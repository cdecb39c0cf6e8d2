"""ResNet-20 AdderNet training on the HIP layer: against the same network built on the oracle layer,
and the captured HIP graph against the eager step."""
import copy

import pytest
import torch

pytestmark = pytest.mark.gpu


def _pair(gpu, batch, eta=0.1, seed=0):
    from addernetcuda_amd.resnet20 import resnet20
    from oracle import adder_oracle
    torch.manual_seed(seed)
    hip = resnet20(eta=eta).to(gpu)
    # pure-torch unfold formulas inside stock torch modules, run on the GPU
    ref = resnet20(adder2d_cls=adder_oracle.adder2d, eta=eta, fused=False).to(gpu)
    ref.load_state_dict(hip.state_dict())
    g = torch.Generator(device=gpu).manual_seed(seed + 1)
    x = torch.randn(batch, 3, 32, 32, device=gpu, generator=g)
    y = torch.randint(0, 10, (batch,), device=gpu, generator=g)
    return hip, ref, x, y


def test_one_step_matches_the_unfold_reference_path(gpu):
    """Same weights, same batch: logits, loss and every gradient against the reference formulation in float64.

    Forward values must agree tightly.  Gradients cannot: behind 19 BatchNorm + ReLU stages a 1e-5 difference
    in an activation flips the occasional ReLU gate (measured: 0-2 of ~3 million gates, for the HIP path and
    for the reference's own fp32 evaluation alike), and one flipped gate near the loss moves every gradient
    below it by percents of its largest entry.  So each gradient tensor may deviate by at most 15 % of its
    largest entry and the median deviation over all tensors must stay below 2 %; the kernels themselves are
    held to rtol 1e-5 / atol 1e-4 per layer in the parity tests."""
    import copy
    import statistics
    hip, ref, x, y = _pair(gpu, 16)
    ref64 = copy.deepcopy(ref).double()
    outs = []
    for m, xx in ((hip, x), (ref64, x.double())):
        logits = m(xx)
        loss = torch.nn.functional.cross_entropy(logits, y)
        loss.backward()
        outs.append((logits.detach().double(), loss.item()))
    assert torch.allclose(outs[0][0], outs[1][0], rtol=1e-3, atol=1e-3)
    assert outs[0][1] == pytest.approx(outs[1][1], rel=1e-5)
    ph, pt = dict(hip.named_parameters()), dict(ref64.named_parameters())
    rel = {}
    for name in ph:
        truth = pt[name].grad
        rel[name] = (ph[name].grad.double() - truth).abs().max().item() / (truth.abs().max().item() + 1e-12)
    worst = max(rel, key=rel.get)
    assert rel[worst] <= 0.15, (worst, rel[worst])
    assert statistics.median(rel.values()) <= 0.02, sorted(rel.items(), key=lambda kv: -kv[1])[:5]


BATCH, STEPS = 256, 50     # the third benchmark configuration: batch 256, 50 steps, SGD momentum 0.9, eta 0.1


def _sgd(model):
    return torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=5e-4)   # main.py:67


def _train(model, x, y, steps=STEPS):
    opt = _sgd(model)
    losses = []
    for _ in range(steps):
        opt.zero_grad(set_to_none=True)
        loss = torch.nn.functional.cross_entropy(model(x), y)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    return losses


def _reference_net(gpu, state, dtype):
    """The reference's model file as it stands (stock Conv2d / BatchNorm2d / ReLU modules, resnet20.py:28-39,
    80-93) around the oracle's unfold-formula adder layer: nothing of the HIP library runs in it."""
    from addernetcuda_amd.resnet20 import resnet20
    from oracle import adder_oracle
    net = resnet20(adder2d_cls=adder_oracle.adder2d, eta=0.1, fused=False).to(gpu)
    net.load_state_dict(state)
    return net.to(dtype)


def test_training_is_bit_reproducible_at_batch_256(gpu):
    """Two runs of 50 training steps from the same weights give the same 50 losses, bit for bit, and the same
    final weights: no kernel of the step adds in an order that changes from run to run (the reference's
    backward does, adder.cu:266-267).  The classifier runs as a matrix product for this reason (resnet20.py
    of this package): the vendor convolution's weight gradient was the one kernel that did not reproduce."""
    hip, _, x, y = _pair(gpu, BATCH)
    state = copy.deepcopy(hip.state_dict())
    first = _train(hip, x, y)
    end = copy.deepcopy(hip.state_dict())
    hip.load_state_dict(state)
    second = _train(hip, x, y)
    assert first == second
    for k, v in hip.state_dict().items():
        assert torch.equal(v, end[k]), k


def test_every_step_of_a_50_step_run_matches_the_reference_step(gpu):
    """Config 3 (batch 256, 50 steps), one step at a time along the reference trajectory.

    The trajectory is the reference path's own, computed in float64.  At every step t the HIP network and the
    reference path in fp32 are both put into the float64 run's state (weights, BatchNorm buffers, momentum),
    take one training step, and are compared with what the float64 step gives from that state:
      * the loss at the common state (the forward pass) -- to 1e-5 relative;
      * the loss after the step, i.e. the float64 network's loss at the weights each fp32 step produced against
        its loss at its own new weights (the backward pass, the eta scaling and the update in one number) -- to
        1e-3 * max(1, |loss|) at each of the 50 steps, and
        to three times the largest deviation the reference path's own fp32 step has shown so far (+ 1e-5).
    Measured on MI355X: forward <= 9e-7 (fp32 reference path: 7e-6), step <= 5e-5 (fp32 reference path: 1.5e-4).
    Compared like this, nothing accumulates: see the free-running test below for why that matters."""
    import torch.nn.functional as F
    from addernetcuda_amd.resnet20 import resnet20
    torch.manual_seed(0)
    hip = resnet20(eta=0.1).to(gpu)
    ref32 = _reference_net(gpu, hip.state_dict(), torch.float32)
    ref64 = _reference_net(gpu, hip.state_dict(), torch.float64)
    probe = copy.deepcopy(ref64)
    g = torch.Generator(device=gpu).manual_seed(1)
    x = torch.randn(BATCH, 3, 32, 32, device=gpu, generator=g)
    y = torch.randint(0, 10, (BATCH,), device=gpu, generator=g)
    xd = x.double()
    o_hip, o_32, o_64 = _sgd(hip), _sgd(ref32), _sgd(ref64)

    def put_into_reference_state(model, opt):
        model.load_state_dict(ref64.state_dict())
        for p, q in zip(model.parameters(), ref64.parameters()):
            buf = o_64.state.get(q, {}).get("momentum_buffer")
            if buf is not None:
                opt.state[p]["momentum_buffer"] = buf.to(p.dtype).clone()

    def one_step(model, opt, inp):
        opt.zero_grad(set_to_none=True)
        loss = F.cross_entropy(model(inp), y)
        loss.backward()
        opt.step()
        return loss.item()

    envelope = 0.0
    worst = {"fwd_hip": 0.0, "fwd_ref32": 0.0, "step_hip": 0.0, "step_ref32": 0.0}
    for t in range(STEPS):
        put_into_reference_state(hip, o_hip)
        put_into_reference_state(ref32, o_32)
        l_hip, l_32, l_64 = one_step(hip, o_hip, x), one_step(ref32, o_32, x), one_step(ref64, o_64, xd)
        assert abs(l_hip - l_64) <= 1e-5 * max(1.0, abs(l_64)), (t, l_hip, l_64)
        with torch.no_grad():
            after_64 = F.cross_entropy(ref64(xd), y).item()
            dev = {}
            for name, m in (("hip", hip), ("ref32", ref32)):
                probe.load_state_dict(m.state_dict())
                dev[name] = abs(F.cross_entropy(probe(xd), y).item() - after_64)
        envelope = max(envelope, dev["ref32"])
        assert dev["hip"] <= 1e-3 * max(1.0, abs(after_64)), (t, dev)
        assert dev["hip"] <= 3.0 * envelope + 1e-5, (t, dev, envelope)
        for k, v in (("fwd_hip", abs(l_hip - l_64)), ("fwd_ref32", abs(l_32 - l_64)), ("step_hip", dev["hip"]),
                     ("step_ref32", dev["ref32"])):
            worst[k] = max(worst[k], v)
    print("largest deviations from the float64 reference step over 50 steps:", worst)
    assert l_64 < 0.5 * 2.7276   # the trajectory does fit the batch (loss 2.73 -> 0.83)


def test_free_running_loss_curves_track_the_float64_reference(gpu):
    """Config 3 free-running: 50 steps of the HIP network and of the reference path in fp32, each on its own
    trajectory, against the reference path in float64, all from the same weights on the same batch.

    fp32 training of this network does not keep two implementations together: the eta-normalised updates at
    lr 0.1 amplify a last-bit difference by one to two orders of magnitude per step in the first steps
    (measured, MI355X: the reference path's fp32 run is 1e-6 from its float64 run at step 0, 1.4e-5 at step 1,
    6e-4 at step 2, 1.3e-3 at step 3, 2e-2 at step 7, 5e-2 at step 10, and two runs of that same fp32 code are
    5e-3 apart at step 6 because torch's fold / reduction kernels add in varying order).  The per-step gate
    proposed for this curve -- 1e-3 for ten steps -- is therefore missed by the reference against itself from
    step 3 on, and which implementation is closer at a given later step is a coin toss.  What is asserted:
      * steps 0-2 within 1e-3 * max(1, |loss|) of the float64 curve (measured 5e-4 at step 2; a wrong eta, a
        dropped padding tap or a wrong sign in one layer shows as > 1e-2 there);
      * over all 50 steps, the HIP curve tracks the float64 curve as closely as the reference's own fp32 run
        does: mean log10 deviation no more than log10(3) above that of the fp32 reference, over the first ten
        steps and over all fifty (a mean over steps is what makes this a measurement instead of a coin toss);
      * all three fit the batch.
    The per-step comparison that does hold 1e-3 at each of the 50 steps is the test above."""
    import math
    from addernetcuda_amd.resnet20 import resnet20
    torch.manual_seed(0)
    hip = resnet20(eta=0.1).to(gpu)
    state = copy.deepcopy(hip.state_dict())
    g = torch.Generator(device=gpu).manual_seed(1)
    x = torch.randn(BATCH, 3, 32, 32, device=gpu, generator=g)
    y = torch.randint(0, 10, (BATCH,), device=gpu, generator=g)
    c_hip = _train(hip, x, y)
    c_32 = _train(_reference_net(gpu, state, torch.float32), x, y)
    c_64 = _train(_reference_net(gpu, state, torch.float64), x.double(), y)
    d_hip = [abs(a - b) for a, b in zip(c_hip, c_64)]
    d_32 = [abs(a - b) for a, b in zip(c_32, c_64)]
    for t in range(3):
        assert d_hip[t] <= 1e-3 * max(1.0, abs(c_64[t])), (t, c_hip[t], c_64[t])
    mean_log = lambda d: sum(math.log10(v + 1e-7) for v in d) / len(d)
    print("mean log10 deviation from the float64 curve: hip %.2f, fp32 reference %.2f; largest: %.3f, %.3f"
          % (mean_log(d_hip), mean_log(d_32), max(d_hip), max(d_32)))
    assert mean_log(d_hip[:10]) <= mean_log(d_32[:10]) + math.log10(3.0)
    assert mean_log(d_hip) <= mean_log(d_32) + math.log10(3.0)
    for c in (c_hip, c_32, c_64):
        assert min(c[-5:]) < 0.5 * c[0]


def test_captured_graph_replays_match_the_eager_step(gpu):
    """The whole training step as one HIP graph: every replay, with eager work and synchronisation in
    between, must land on the same weights as the eager step from the same state."""
    import bench
    model, opt, x, y = bench.build_training(gpu)
    graph, loss = bench.capture_step(model, opt, x, y)
    eager = bench.make_step(model, opt, x, y)
    for _ in range(4):
        saved = ({k: v.clone() for k, v in model.state_dict().items()}, copy.deepcopy(opt.state_dict()))
        graph.replay()
        torch.cuda.synchronize()
        lg = loss.item()
        got = {k: v.clone() for k, v in model.state_dict().items()}
        model.load_state_dict(saved[0])
        opt.load_state_dict(saved[1])
        le = eager().item()
        torch.cuda.synchronize()
        want = model.state_dict()
        assert lg == pytest.approx(le, rel=1e-5)
        for k in got:
            assert torch.allclose(got[k].float(), want[k].float(), rtol=1e-4, atol=1e-5), k


def test_state_dict_round_trip_and_eval_forward(gpu):
    from addernetcuda_amd.resnet20 import resnet20
    torch.manual_seed(3)
    a, b = resnet20().to(gpu), resnet20().to(gpu)
    b.load_state_dict(a.state_dict())
    a.eval(), b.eval()
    x = torch.randn(8, 3, 32, 32, device=gpu)
    with torch.no_grad():
        assert torch.equal(a(x), b(x))


def test_stem_convolution_weight_gradient_matches_torch(gpu):
    """StemConv2d: an ordinary convolution; its weight gradient comes from the adder library's matrix-core
    kernel (sum x * gy, no weight term) and must be the float64 gradient of F.conv2d to the parity bar, alone
    and inside a batched_eta_scaling() block; its input gradient and its state_dict are nn.Conv2d's."""
    from addernetcuda_amd import adder
    from addernetcuda_amd.resnet20 import StemConv2d
    from tests.util import assert_close
    g = torch.Generator().manual_seed(11)
    for shape, co, stride in (((6, 3, 32, 32), 16, 1), ((3, 5, 14, 10), 7, 1), ((4, 8, 16, 16), 12, 2)):
        x = torch.randn(shape, generator=g)
        gy_shape = None
        conv = StemConv2d(shape[1], co, 3, stride=stride, padding=1, bias=False).to(gpu)
        assert list(conv.state_dict()) == ["weight"]
        w = conv.weight.detach().cpu()
        xd = x.double().requires_grad_(True)
        wd = w.double().requires_grad_(True)
        yd = torch.nn.functional.conv2d(xd, wd, None, stride, 1)
        gy = torch.randn(yd.shape, generator=g)
        yd.backward(gy.double())
        for batched in (False, True):
            conv.weight.grad = None
            xg = x.to(gpu).requires_grad_(True)
            y = conv(xg)
            assert_close(y, yd.detach(), f"stem forward {shape}", rtol=1e-5, atol=1e-5)
            if batched:
                with adder.batched_eta_scaling():
                    y.backward(gy.to(gpu))
            else:
                y.backward(gy.to(gpu))
            torch.cuda.synchronize()
            assert_close(conv.weight.grad, wd.grad, f"stem grad_W {shape} batched={batched}", rtol=1e-5, atol=1e-4)
            assert_close(xg.grad, xd.grad, f"stem grad_X {shape}", rtol=1e-4, atol=1e-4)
        y2, stats = conv.forward_with_stats(x.to(gpu))
        if stride == 1:     # the tiled kernel: statistics of the output from its epilogue
            assert stats is not None
            tot = stats.sum(dim=1).cpu()
            assert torch.allclose(tot[:, 0], yd.detach().sum(dim=(0, 2, 3)), rtol=1e-5, atol=1e-4)
            assert torch.allclose(tot[:, 1], (yd.detach() ** 2).sum(dim=(0, 2, 3)), rtol=1e-5, atol=1e-4)
        else:
            assert stats is None
        assert_close(y2, yd.detach(), f"stem forward_with_stats {shape}", rtol=1e-5, atol=1e-5)
