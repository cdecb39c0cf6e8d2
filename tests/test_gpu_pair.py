"""A strided 3x3 layer and the strided 1x1 layer on the same input in one launch (adder_conv2d_fwd_pair_stats_f32):
both outputs against the float64 C oracle, the statistics against float64 sums, refusals, and the hand-over between
the two autograd nodes of a residual block that halves the map (resnet20.py:66-70)."""
import ctypes

import pytest
import torch

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (N, Ci, H, W, Co): the two ResNet-20 blocks at reduced batch, wide maps, many channels (the third tile shape),
# channel counts that do not fill a group, a ragged batch
CASES = [(6, 16, 32, 32, 32), (5, 32, 16, 16, 64), (2, 8, 64, 64, 8), (3, 128, 8, 8, 130), (3, 10, 12, 20, 7),
         (7, 16, 8, 8, 16)]


def _call(case, gpu, seed=0):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, conv_dims, fwd_stats_slots
    N, Ci, H, W, Co = case
    g = torch.Generator().manual_seed(seed + sum(case))
    x = torch.randn(N, Ci, H, W, generator=g)
    w = torch.randn(Co, Ci, 3, 3, generator=g) * 0.3
    ws = torch.randn(Co, Ci, 1, 1, generator=g) * 0.3
    dims, Ho, Wo = conv_dims(x.shape, w.shape, 2, 1)
    slots = fwd_stats_slots(dims)
    xg, wg, wsg = x.to(gpu), w.to(gpu), ws.to(gpu)
    y, ys = (torch.full((N, Co, Ho, Wo), float("nan"), device=gpu) for _ in range(2))
    st, sts = (torch.full((Co, max(slots, 1), 2), float("nan"), dtype=torch.float64, device=gpu) for _ in range(2))
    rc = lib.adder_conv2d_fwd_pair_stats_f32(ptr(xg), ptr(wg), ptr(wsg), ptr(y), ptr(ys), ptr(st), ptr(sts), slots, *dims,
                                             stream_ptr(gpu))
    torch.cuda.synchronize()
    return rc, (x, w, ws), (y, ys, st, sts)


@pytest.mark.parametrize("case", CASES, ids=str)
def test_pair_matches_the_two_layers(case, gpu):
    from oracle import c_oracle
    rc, (x, w, ws), (y, ys, st, sts) = _call(case, gpu)
    assert rc == 0
    want, want_s = c_oracle.conv2d_fwd(x, w, 2, 1), c_oracle.conv2d_fwd(x, ws, 2, 0)
    assert want.shape == want_s.shape
    assert_close(y, want, f"3x3 output {case}")
    assert_close(ys, want_s, f"1x1 output {case}")
    for got, ref, what in ((st, want, "3x3"), (sts, want_s, "1x1")):
        ref = ref.double()
        sums = torch.stack([ref.sum((0, 2, 3)), (ref * ref).sum((0, 2, 3))], 1)
        assert torch.isfinite(got).all()
        assert_close(got.sum(1), sums, f"statistics of the {what} output {case}", rtol=1e-6, atol=1e-6)


def test_pair_refusals(gpu):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr
    t = torch.zeros(1 << 16, device=gpu)
    d = torch.zeros(1 << 12, dtype=torch.float64, device=gpu)
    call = lambda *dims, slots=1: lib.adder_conv2d_fwd_pair_stats_f32(ptr(t), ptr(t[4096:]), ptr(t[8192:]), ptr(t[16384:]),
                                                                       ptr(t[32768:]), ptr(d), ptr(d[2048:]), slots, *dims,
                                                                       stream_ptr(gpu))
    assert call(2, 8, 8, 8, 8, 3, 3, 1, 1) == -7          # stride 1
    assert call(2, 8, 8, 8, 8, 1, 1, 2, 0) == -7          # not a 3x3 layer
    assert call(2, 8, 7, 7, 8, 3, 3, 2, 1) == -7          # odd map: the two layers' outputs differ in size
    assert call(2, 8, 6, 6, 8, 3, 3, 2, 1) == -7          # rows that are not whole groups of four
    assert call(2, 8, 8, 8, 8, 3, 3, 2, 1, slots=77) == -2
    assert lib.adder_conv2d_fwd_pair_stats_f32(ptr(t), ptr(t), None, ptr(t), ptr(t), ptr(d), ptr(d), 1, 2, 8, 8, 8, 8, 3, 3, 2, 1,
                                               stream_ptr(gpu)) == -1


def test_block_hands_the_side_output_over(gpu, monkeypatch):
    """The first block of a ResNet-20 stage: conv1's launch also computes the downsample layer's output, the
    downsample node takes it instead of launching its own kernel, and nothing changes in what the block computes."""
    from addernetcuda_amd import adder, resnet20
    from addernetcuda_amd.bn_act import BatchNormAct2d
    import torch.nn as nn
    torch.manual_seed(3)

    def make():
        torch.manual_seed(11)
        ds = nn.Sequential(adder.adder2d(16, 32, kernel_size=1, stride=2, padding=0, bias=False),
                           BatchNormAct2d(32, relu=False))
        return resnet20.BasicBlock(16, 32, stride=2, downsample=ds).to(gpu).train()

    x = torch.randn(6, 16, 32, 32, device=gpu)
    gy = torch.randn(6, 32, 16, 16, device=gpu)
    taken = []
    orig = adder.SideOutput.of
    monkeypatch.setattr(adder.SideOutput, "of", staticmethod(lambda *a: taken.append(orig(*a)) or taken[-1]))
    a = make()
    xa = x.clone().requires_grad_(True)
    ya = a(xa)
    ya.backward(gy)
    assert sum(t is not None for t in taken) == 1

    monkeypatch.setattr(adder, "conv_forward_pair", lambda *args: None)     # the same block, two launches
    taken.clear()
    b = make()
    xb = x.clone().requires_grad_(True)
    yb = b(xb)
    yb.backward(gy)
    assert all(t is None for t in taken)
    # (the 1x1 layer's output is the same bit for bit; its statistics are summed over other slots, so the BatchNorm's
    # mean and variance differ in their last bits)
    assert_close(ya, yb, "block output", rtol=1e-5, atol=1e-5)
    assert_close(xa.grad, xb.grad, "input gradient", rtol=1e-4, atol=1e-4)
    for (n, p), (_, q) in zip(a.named_parameters(), b.named_parameters()):
        assert_close(p.grad, q.grad, n, rtol=1e-4, atol=1e-4)
    # the product is handed only to the layer it was computed for
    monkeypatch.undo()
    c = make()
    from addernetcuda_amd.unit import adder_bn_act
    xc = x.clone().requires_grad_(True)
    out, shortcut = adder_bn_act(c.conv1, c.bn1, xc * 1.0, with_shortcut=True, side_conv=c.downsample[0])
    assert getattr(shortcut, "_adder_side_output", None) is not None
    assert orig(shortcut, c.downsample[0].adder, 2, 1) is None             # asked for another layer geometry
    assert orig(shortcut, c.conv1.adder, 2, 0) is None                     # ... another weight
    assert orig(shortcut.clone(), c.downsample[0].adder, 2, 0) is None     # ... another tensor
    assert orig(shortcut, c.downsample[0].adder, 2, 0) is not None
    assert orig(shortcut, c.downsample[0].adder, 2, 0) is None             # taken once
