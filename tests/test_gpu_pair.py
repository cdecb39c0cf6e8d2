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


@pytest.mark.parametrize("case", [(6, 16, 32, 32, 32), (5, 32, 16, 16, 64), (3, 128, 8, 8, 130), (2, 8, 64, 64, 8),
                                  (4, 8, 8, 8, 600)], ids=str)   # the last one: the three-instruction form
@pytest.mark.parametrize("with_add", [False, True])
def test_side_input_gradient_inside_the_strided_kernel(case, with_add, gpu):
    """adder_bn_links.side_gy / side_w: the strided 1x1 layer's input gradient added inside the strided 3x3 layer's
    linked input-gradient kernel, against the same call with that gradient computed by the 1x1 layer's own kernel
    (held to the oracle in test_gpu_parity_nchw.py) and passed as gx_add."""
    from addernetcuda_amd._lib import lib, check, ptr, stream_ptr, conv_dims, BnLinks, bwd_bn_slots
    N, Ci, H, W, Co = case
    g = torch.Generator(device=gpu).manual_seed(sum(case))
    b = lambda v: v[None, :, None, None]
    bn_in = torch.randn(N, Ci, H, W, device=gpu, generator=g) * 20 - 90
    mean, rstd = bn_in.mean((0, 2, 3)), 1.0 / bn_in.std((0, 2, 3))
    x = torch.relu((bn_in - b(mean)) * b(rstd) + torch.randn(N, Ci, H, W, device=gpu, generator=g))
    w = torch.randn(Co, Ci, 3, 3, device=gpu, generator=g) * 0.3
    ws = torch.randn(Co, Ci, 1, 1, device=gpu, generator=g) * 0.3
    dims, Ho, Wo = conv_dims(x.shape, w.shape, 2, 1)
    dims1, _, _ = conv_dims(x.shape, ws.shape, 2, 0)
    gy = torch.randn(N, Co, Ho, Wo, device=gpu, generator=g)
    gyd = torch.randn(N, Co, Ho, Wo, device=gpu, generator=g)
    more = torch.randn(x.shape, device=gpu, generator=g) if with_add else None
    slots = bwd_bn_slots(dims)
    assert slots > 0
    st = stream_ptr(gpu)
    gxd, gxa, gxb = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    pa = torch.empty(Ci, slots, 2, dtype=torch.float32, device=gpu)
    pb = torch.full_like(pa, float("nan"))
    la = BnLinks(None, None, None, ptr(bn_in), ptr(mean), ptr(rstd), ptr(pa), slots, 1)
    lb = BnLinks(None, None, None, ptr(bn_in), ptr(mean), ptr(rstd), ptr(pb), slots, 1, None, None, ptr(gyd), ptr(ws))
    check(lib.adder_conv2d_bwd_f32(ptr(gyd), ptr(x), ptr(ws), ptr(gxd), None, 0.0, None, 0, *dims1, st), "1x1 grad_X")
    add = gxd + more if with_add else gxd
    check(lib.adder_conv2d_bwd_bn_f32(ptr(gy), ptr(x), ptr(w), ptr(add), ptr(gxa), None, 0.0, None, 0, *dims,
                                      ctypes.byref(la), st), "gx_add")
    check(lib.adder_conv2d_bwd_bn_f32(ptr(gy), ptr(x), ptr(w), ptr(more), ptr(gxb), None, 0.0, None, 0, *dims,
                                      ctypes.byref(lb), st), "side")
    torch.cuda.synchronize()
    assert_close(gxb, gxa, f"dz {case}", rtol=1e-5, atol=1e-4)
    scale = max(1.0, float(pa.double().sum(1).abs().max()))
    assert_close(pb.double().sum(1) / scale, pa.double().sum(1) / scale, f"sums {case}", rtol=1e-6, atol=1e-6)
    # refusals: one of the two pointers, no in-links, a stride-1 layer
    lc = BnLinks(None, None, None, ptr(bn_in), ptr(mean), ptr(rstd), ptr(pb), slots, 1, None, None, ptr(gyd), None)
    assert lib.adder_conv2d_bwd_bn_f32(ptr(gy), ptr(x), ptr(w), None, ptr(gxb), None, 0.0, None, 0, *dims,
                                       ctypes.byref(lc), st) == -1
    ld = BnLinks(None, None, None, None, None, None, None, 0, 0, None, None, ptr(gyd), ptr(ws))
    assert lib.adder_conv2d_bwd_bn_f32(ptr(gy), ptr(x), ptr(w), None, ptr(gxb), None, 0.0, None, 0, *dims,
                                       ctypes.byref(ld), st) == -7


def test_pair_in_a_chain_of_units(gpu, monkeypatch):
    """A unit in front of a block that halves the map, so that the block's first layer has a BatchNorm link on its
    input and the 1x1 layer's input gradient is added inside its strided kernel: gradients against the same
    network with the pair switched off."""
    from addernetcuda_amd import adder, resnet20
    from addernetcuda_amd.bn_act import BatchNormAct2d
    from addernetcuda_amd.unit import adder_bn_act
    import torch.nn as nn

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            torch.manual_seed(5)
            self.conv0 = adder.adder2d(8, 16, kernel_size=3, stride=1, padding=1, bias=False)
            self.bn0 = BatchNormAct2d(16, relu=True)
            ds = nn.Sequential(adder.adder2d(16, 32, kernel_size=1, stride=2, padding=0, bias=False),
                               BatchNormAct2d(32, relu=False))
            self.block = resnet20.BasicBlock(16, 32, stride=2, downsample=ds)

        def forward(self, x):
            return self.block(adder_bn_act(self.conv0, self.bn0, x))

    x = torch.randn(6, 8, 16, 16, device=gpu)
    gy = torch.randn(6, 32, 8, 8, device=gpu)
    used = []
    orig = adder.conv_backward
    monkeypatch.setattr(adder, "conv_backward", lambda *a, **k: used.append(k.get("side")) or orig(*a, **k))
    a = Net().to(gpu).train()
    xa = x.clone().requires_grad_(True)
    a(xa).backward(gy)
    assert sum(u is not None for u in used) == 1          # the 3x3 layer's call carried the 1x1 layer's gradient
    monkeypatch.setattr(adder, "conv_forward_pair", lambda *args: None)
    used.clear()
    b = Net().to(gpu).train()
    xb = x.clone().requires_grad_(True)
    b(xb).backward(gy)
    assert all(u is None for u in used)
    assert_close(xa.grad, xb.grad, "input gradient", rtol=1e-4, atol=1e-4)
    for (n, p), (_, q) in zip(a.named_parameters(), b.named_parameters()):
        assert_close(p.grad, q.grad, n, rtol=1e-4, atol=1e-4)


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


def test_second_backward_through_a_retained_graph(gpu):
    """The hand-over between the two nodes is used once; a second backward pass through a retained graph takes the
    plain path and must deliver the same gradients again."""
    from addernetcuda_amd import adder, resnet20
    from addernetcuda_amd.bn_act import BatchNormAct2d
    import torch.nn as nn
    torch.manual_seed(2)
    ds = nn.Sequential(adder.adder2d(16, 32, kernel_size=1, stride=2, padding=0, bias=False), BatchNormAct2d(32, relu=False))
    block = resnet20.BasicBlock(16, 32, stride=2, downsample=ds).to(gpu).train()
    x = torch.randn(4, 16, 16, 16, device=gpu, requires_grad=True)
    gy = torch.randn(4, 32, 8, 8, device=gpu)
    y = block(x)
    y.backward(gy, retain_graph=True)
    first = [x.grad.clone()] + [p.grad.clone() for p in block.parameters()]
    x.grad = None
    for p in block.parameters():
        p.grad = None
    y.backward(gy)
    second = [x.grad] + [p.grad for p in block.parameters()]
    for a, b in zip(first, second):
        assert_close(b, a, "second pass", rtol=1e-4, atol=1e-4)


def test_uncollected_side_gradient_is_an_error(gpu):
    """Differentiating with respect to the tensor between the two layers of a pair would silently miss the 1x1
    layer's part (it is left to the 3x3 layer's node): that must be an error, not a wrong number."""
    from addernetcuda_amd import adder
    from addernetcuda_amd.bn_act import BatchNormAct2d
    from addernetcuda_amd.unit import adder_bn_act
    torch.manual_seed(4)
    conv1 = adder.adder2d(16, 32, kernel_size=3, stride=2, padding=1, bias=False).to(gpu)
    side = adder.adder2d(16, 32, kernel_size=1, stride=2, padding=0, bias=False).to(gpu)
    bn1, bns = BatchNormAct2d(32, relu=True).to(gpu).train(), BatchNormAct2d(32, relu=False).to(gpu).train()
    x = torch.randn(4, 16, 16, 16, device=gpu, requires_grad=True)
    out, shortcut = adder_bn_act(conv1, bn1, x, with_shortcut=True, side_conv=side)
    ys = adder_bn_act(side, bns, shortcut)
    with pytest.raises(RuntimeError, match="paired 1x1 layer"):
        torch.autograd.grad(ys.sum(), shortcut)


def test_gradient_of_the_paired_layers_own_parameters_only(gpu):
    """torch.autograd.grad with respect to the downsample layer's weight (and its BatchNorm) alone never runs the
    3x3 layer's node: the 1x1 node must then neither hand its input gradient over nor raise, and what it returns
    must equal the same parameters' gradients from a full backward pass."""
    from addernetcuda_amd import adder, resnet20
    from addernetcuda_amd.bn_act import BatchNormAct2d
    import torch.nn as nn
    torch.manual_seed(6)
    ds = nn.Sequential(adder.adder2d(16, 32, kernel_size=1, stride=2, padding=0, bias=False), BatchNormAct2d(32, relu=False))
    block = resnet20.BasicBlock(16, 32, stride=2, downsample=ds).to(gpu).train()
    x = torch.randn(4, 16, 16, 16, device=gpu, requires_grad=True)
    gy = torch.randn(4, 32, 8, 8, device=gpu)
    params = [ds[0].adder, ds[1].weight, ds[1].bias]
    y = block(x)
    only = torch.autograd.grad(y, params, gy, retain_graph=True)
    y2 = block(x)
    y2.backward(gy)
    for got, p in zip(only, params):
        assert_close(got, p.grad, "gradient of the downsample branch's parameters", rtol=1e-4, atol=1e-4)


def test_second_backward_through_a_retained_graph_of_the_whole_network(gpu):
    """The stem's convolution + BatchNorm node (resnet20._conv_bn_act) hands over like the adder units do; a second
    pass through a retained graph finds the hand-over used up and must take the plain path with the same result."""
    from addernetcuda_amd.resnet20 import resnet20
    torch.manual_seed(8)
    model = resnet20(eta=0.1).to(gpu).train()
    x = torch.randn(8, 3, 32, 32, device=gpu)
    t = torch.randint(0, 10, (8,), device=gpu)
    loss = torch.nn.functional.cross_entropy(model(x), t)
    loss.backward(retain_graph=True)
    first = {n: p.grad.clone() for n, p in model.named_parameters()}
    model.zero_grad(set_to_none=True)
    loss.backward()
    for n, p in model.named_parameters():
        scale = first[n].abs().max().item() + 1e-6
        assert (p.grad - first[n]).abs().max().item() <= 1e-3 * scale, n
