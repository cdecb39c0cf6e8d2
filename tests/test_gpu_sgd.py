"""``addernetcuda_amd.optim.SGD`` (csrc/sgd.hip: all parameters of a group in one launch) against
``torch.optim.SGD`` of main.py:67 -- the same update rule, evaluated by the framework in float64 and float32."""
import copy

import pytest
import torch

from tests.util import assert_close

pytestmark = pytest.mark.gpu

SHAPES = [(16, 3, 3, 3), (16,), (16,), (16, 16, 3, 3), (64, 64, 3, 3), (10, 64, 1, 1), (10,), (5, 7), (1,), (1023,),
          (1025,), (2049,)]


def _params(dev, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.nn.Parameter(torch.randn(s, generator=g).to(dev, dtype)) for s in SHAPES]


def _set_grads(params, seed):
    g = torch.Generator().manual_seed(seed)
    for p in params:
        p.grad = torch.randn(p.shape, generator=g).to(p.device, p.dtype)


@pytest.mark.parametrize("wd", [5e-4, 0.0])
def test_three_steps_match_torch_sgd(wd, gpu):
    from addernetcuda_amd.optim import SGD
    ours = _params(gpu, torch.float32, 1)
    ref32 = _params(gpu, torch.float32, 1)
    ref64 = _params("cpu", torch.float64, 1)
    for a, b in zip(ref64, ours):   # the float64 run starts from the float32 values
        a.data.copy_(b.detach().double().cpu())
    kw = dict(lr=0.1, momentum=0.9, weight_decay=wd)
    o, r32, r64 = SGD(ours, **kw), torch.optim.SGD(ref32, **kw), torch.optim.SGD(ref64, **kw)
    for step in range(3):
        for ps in (ours, ref32, ref64):
            _set_grads(ps, 100 + step)
        o.step(); r32.step(); r64.step()
    torch.cuda.synchronize()
    for a, b, c in zip(ours, ref32, ref64):
        assert_close(a, c, "parameter vs float64", rtol=1e-5, atol=1e-6)
        assert_close(a, b.double(), "parameter vs torch float32", rtol=1e-6, atol=1e-6)
        assert_close(o.state[a]["momentum_buffer"], r64.state[c]["momentum_buffer"], "momentum buffer", rtol=1e-5, atol=1e-6)
    # the state has torch.optim.SGD's layout: it loads into the framework's optimizer and back
    r32.load_state_dict(o.state_dict())
    o.load_state_dict(r32.state_dict())


def test_device_learning_rate_and_fallback_groups(gpu):
    from addernetcuda_amd.optim import SGD
    lr = torch.tensor(0.1, device=gpu)
    ours, ref = _params(gpu, torch.float32, 2), _params(gpu, torch.float32, 2)
    # second group: Nesterov, which the kernel leaves to the framework
    o = SGD([{"params": ours[:6]}, {"params": ours[6:], "nesterov": True}], lr=lr, momentum=0.9, weight_decay=5e-4)
    r = torch.optim.SGD([{"params": ref[:6]}, {"params": ref[6:], "nesterov": True}], lr=0.1, momentum=0.9,
                        weight_decay=5e-4)
    for step, rate in enumerate((0.1, 0.05)):
        lr.fill_(rate)
        for g in r.param_groups:
            g["lr"] = rate
        _set_grads(ours, 7 + step)
        _set_grads(ref, 7 + step)
        o.step(); r.step()
    torch.cuda.synchronize()
    for a, b in zip(ours, ref):
        assert_close(a, b.double(), "parameter", rtol=1e-6, atol=1e-6)


def test_refusals(gpu):
    import ctypes
    from addernetcuda_amd._lib import lib, stream_ptr, ADDER_ERR_ALIAS, ADDER_ERR_BAD_SHAPE, ADDER_ERR_NULL_POINTER
    t = torch.zeros(64, device=gpu)
    one = (ctypes.c_void_p * 1)(t.data_ptr())
    n = (ctypes.c_long * 1)(64)
    st = stream_ptr(gpu)
    assert lib.adder_sgd_momentum_step_f32(1, one, one, one, n, None, 0.1, 0.9, 0.0, st) == ADDER_ERR_ALIAS
    assert lib.adder_sgd_momentum_step_f32(0, one, one, one, n, None, 0.1, 0.9, 0.0, st) == ADDER_ERR_BAD_SHAPE
    assert lib.adder_sgd_momentum_step_f32(97, one, one, one, n, None, 0.1, 0.9, 0.0, st) == ADDER_ERR_BAD_SHAPE
    assert lib.adder_sgd_momentum_step_f32(1, one, None, one, n, None, 0.1, 0.9, 0.0, st) == ADDER_ERR_NULL_POINTER
