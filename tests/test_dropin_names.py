"""The reference's model files write ``import adder`` (resnet20.py:3, resnet50.py:5, vgg.py:6, densenet.py:5) and its
operator file writes ``import adder_cuda`` (adder.py:15).  ``addernetcuda_amd.install()`` -- or the ``dropin``
directory on the path -- makes those two top-level names bind to this build, so that code written against the
reference's names runs without an edit.  The network below is written the way a user of the reference writes one:
nothing but ``import adder`` / ``adder.adder2d(...)`` and ``torch.nn``.
"""
import importlib
import os
import subprocess
import sys

import pytest
import torch
import torch.nn as nn

from util import assert_close

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _residual_net(adder_module, width=16, classes=10):
    """A two-stage residual network of the shape resnet20.py:7-93 builds (3x3 adder layers with BatchNorm and ReLU,
    a strided 1x1 adder layer on the shortcut, ordinary stem and classifier), from ``adder_module.adder2d`` alone."""
    a2d = adder_module.adder2d

    class Block(nn.Module):
        def __init__(self, cin, cout, stride):
            super().__init__()
            self.c1 = a2d(cin, cout, kernel_size=3, stride=stride, padding=1, bias=False)
            self.b1 = nn.BatchNorm2d(cout)
            self.c2 = a2d(cout, cout, kernel_size=3, stride=1, padding=1, bias=False)
            self.b2 = nn.BatchNorm2d(cout)
            self.short = None
            if stride != 1 or cin != cout:
                self.short = nn.Sequential(a2d(cin, cout, kernel_size=1, stride=stride, bias=False), nn.BatchNorm2d(cout))

        def forward(self, x):
            y = torch.relu(self.b1(self.c1(x)))
            y = self.b2(self.c2(y))
            return torch.relu(y + (x if self.short is None else self.short(x)))

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.stem = nn.Sequential(nn.Conv2d(3, width, 3, 1, 1, bias=False), nn.BatchNorm2d(width), nn.ReLU())
            self.stage1 = Block(width, width, 1)
            self.stage2 = Block(width, 2 * width, 2)
            self.head = nn.Linear(2 * width, classes)

        def forward(self, x):
            x = self.stage2(self.stage1(self.stem(x)))
            return self.head(x.mean(dim=(2, 3)))

    return Net()


@pytest.fixture
def installed():
    import addernetcuda_amd
    addernetcuda_amd.install()
    yield addernetcuda_amd
    addernetcuda_amd.uninstall()


def test_install_binds_both_names_and_uninstall_releases_them(installed):
    import adder
    import adder_cuda
    assert adder is installed.adder and adder_cuda is installed.adder_cuda
    for name in ("adder2d", "adder2d_function", "adder"):            # adder.py:22, 43, 83
        assert hasattr(adder, name)
    for name in ("ADDER_CONV", "ADDER_BACKWARD", "ADDER_CONV_WEIGHT", "ADDER_CONV_INPUT"):   # adder_cuda.cpp:88-93
        assert callable(getattr(adder_cuda, name))
    layer = adder.adder2d(4, 8, 3, stride=2, padding=1, bias=True)   # the reference's constructor, positional too
    assert tuple(layer.adder.shape) == (8, 4, 3, 3) and tuple(layer.b.shape) == (8,)
    installed.uninstall()
    assert "adder" not in sys.modules and "adder_cuda" not in sys.modules


def test_install_refuses_to_shadow_a_foreign_module():
    import types
    import addernetcuda_amd
    sys.modules["adder"] = types.ModuleType("adder")
    try:
        with pytest.raises(ImportError, match="already imported"):
            addernetcuda_amd.install()
        addernetcuda_amd.install(force=True)
        assert sys.modules["adder"] is addernetcuda_amd.adder
    finally:
        addernetcuda_amd.uninstall()
        sys.modules.pop("adder", None)


def test_dropin_directory_on_the_path_binds_both_names():
    """A fresh interpreter with nothing but PYTHONPATH set, as a user of the reference would run its scripts."""
    env = dict(os.environ, PYTHONPATH=os.pathsep.join([os.path.join(ROOT, "addernetcuda_amd", "dropin"), ROOT]))
    code = ("import adder, adder_cuda, addernetcuda_amd as pkg; "
            "assert adder is pkg.adder and adder_cuda is pkg.adder_cuda; "
            "import adder as again; assert again is pkg.adder; print('bound')")
    out = subprocess.run([sys.executable, "-c", code], env=env, cwd="/tmp", capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "bound" in out.stdout, out.stderr


@pytest.mark.gpu
def test_network_written_against_the_reference_names_trains_like_its_oracle_twin(gpu, installed):
    """One SGD step of the network above built from ``import adder`` on the GPU, against the same network built
    from the CPU oracle's layer (float64): loss, every gradient, every updated parameter."""
    import adder                     # noqa: F811  (the top-level name, as the reference's files import it)
    from oracle import adder_oracle
    torch.manual_seed(3)
    ref = _residual_net(adder_oracle).double()
    net = _residual_net(adder)
    net.load_state_dict({k: v.float() for k, v in ref.state_dict().items()})
    net = net.to(gpu)
    assert type(net.stage1.c1).__module__ == "addernetcuda_amd.adder"
    x = torch.randn(8, 3, 16, 16, dtype=torch.float64)
    t = torch.randint(0, 10, (8,))
    opts = [torch.optim.SGD(m.parameters(), lr=0.05, momentum=0.9) for m in (ref, net)]
    losses = []
    for m, o, xx, tt in ((ref, opts[0], x, t), (net, opts[1], x.float().to(gpu), t.to(gpu))):
        m.train()
        o.zero_grad()
        loss = nn.functional.cross_entropy(m(xx), tt)
        loss.backward()
        losses.append(loss.item())
    assert abs(losses[0] - losses[1]) <= 1e-4 * max(1.0, abs(losses[0]))
    for (n, p), (_, q) in zip(net.named_parameters(), ref.named_parameters()):
        scale = q.grad.abs().max().item() + 1e-12
        # (a handful of ReLU gates flip between an fp32 and an fp64 forward: bounded relative to the tensor's size)
        assert (p.grad.double().cpu() - q.grad).abs().max().item() <= 2e-3 * scale, n
    for o in opts:
        o.step()
    for (n, p), (_, q) in zip(net.named_parameters(), ref.named_parameters()):
        assert_close(p, q, n, rtol=1e-4, atol=1e-4)


@pytest.mark.gpu
def test_extension_names_as_the_reference_script_calls_them(gpu, installed):
    """adder_cuda/test_cuda.py:63-85, 134-158 in miniature: the four entry points through the top-level name."""
    import adder_cuda                # noqa: F811
    from oracle import adder_oracle
    g = torch.Generator().manual_seed(5)
    K, NL, Co = 72, 256, 8
    X, W, G = torch.randn(K, NL, generator=g), torch.randn(Co, K, generator=g), torch.randn(Co, NL, generator=g)
    Xg, Wg, Gg = X.to(gpu), W.to(gpu), G.to(gpu)
    out = torch.zeros(Co, NL, device=gpu)
    adder_cuda.ADDER_CONV(Xg, Wg, out)
    assert_close(out, adder_oracle.col_forward(X.double(), W.double()), "ADDER_CONV")
    gw, gx = torch.zeros(Co, K, device=gpu), torch.zeros(K, NL, device=gpu)
    adder_cuda.ADDER_BACKWARD(Gg, Xg, Wg, gw, gx)
    assert_close(gw, adder_oracle.col_grad_w(X.double(), W.double(), G.double()), "ADDER_BACKWARD grad_w")
    assert_close(gx, adder_oracle.col_grad_x(X.double(), W.double(), G.double()), "ADDER_BACKWARD grad_i")
