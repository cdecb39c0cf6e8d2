"""Host-side mirror of the reference operator surface: argument checks, module layout, model structure.
None of this launches a kernel."""
import pytest
import torch


def test_adder2d_matches_the_reference_constructor_and_parameter_names():
    from addernetcuda_amd import adder
    m = adder.adder2d(3, 8, 3, stride=2, padding=1, bias=True)
    params = dict(m.named_parameters())
    assert set(params) == {"adder", "b"}                         # adder.py:95-100
    assert params["adder"].shape == (8, 3, 3, 3) and params["b"].shape == (8,)
    assert (m.stride, m.padding, m.input_channel, m.output_channel, m.kernel_size) == (2, 1, 3, 8, 3)
    assert m.eta == 0.2                                          # adder.py:78 divides by 5
    assert (params["b"] >= 0).all() and (params["b"] <= 1).all()  # uniform_(0, 1), adder.py:100
    big = adder.adder2d(64, 64, 3)
    assert abs(big.adder.mean().item()) < 0.05 and abs(big.adder.std().item() - 1.0) < 0.05   # N(0,1), adder.py:97
    assert "b" not in dict(adder.adder2d(3, 8, 3).named_parameters())


def test_depth_wise_is_refused_with_a_clear_error():
    from addernetcuda_amd import adder
    with pytest.raises(NotImplementedError, match="depth_wise"):
        adder.adder2d(8, 8, 3, depth_wise=True)


def test_cpu_tensors_are_refused_like_check_cuda():
    """adder_cuda.cpp:33 asserts is_cuda; there is no CPU fallback here either."""
    from addernetcuda_amd import adder, adder_cuda
    x, w = torch.randn(1, 2, 4, 4), torch.randn(3, 2, 3, 3)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        adder.adder2d_function(x, w, 1, 1)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        adder_cuda.ADDER_CONV(torch.randn(18, 16), torch.randn(3, 18), torch.zeros(3, 16))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        adder_cuda.ADDER_BACKWARD(torch.randn(3, 16), torch.randn(18, 16), torch.randn(3, 18), torch.zeros(3, 18),
                                  torch.zeros(18, 16))


def test_non_square_kernels_are_refused():
    from addernetcuda_amd import adder
    with pytest.raises(RuntimeError, match="square"):
        adder.adder2d_function(torch.randn(1, 2, 4, 4), torch.randn(3, 2, 3, 1), 1, 1)


def test_argument_validators():
    from addernetcuda_amd import _lib
    with pytest.raises(TypeError):
        _lib.require_gpu_f32([1, 2], "x")
    with pytest.raises(RuntimeError, match="channels"):
        _lib.conv_dims((1, 3, 8, 8), (4, 2, 3, 3), 1, 1)
    with pytest.raises(RuntimeError, match="empty output"):
        _lib.conv_dims((1, 3, 2, 2), (4, 3, 5, 5), 1, 0)
    dims, Ho, Wo = _lib.conv_dims((2, 3, 32, 32), (16, 3, 3, 3), 2, 1)
    assert dims == (2, 3, 32, 32, 16, 3, 3, 2, 1) and (Ho, Wo) == (16, 16)


def test_resnet20_structure():
    from addernetcuda_amd import adder
    from addernetcuda_amd.resnet20 import resnet20
    torch.manual_seed(0)
    m = resnet20()
    assert sum(p.numel() for p in m.parameters()) == 272484
    layers = [mod for mod in m.modules() if isinstance(mod, adder.adder2d)]
    assert len(layers) == 20
    assert sum(1 for l in layers if l.kernel_size == 1) == 2 and sum(1 for l in layers if l.stride == 2) == 4
    keys = set(m.state_dict())
    for k in ("conv1.weight", "bn1.weight", "layer1.0.conv1.adder", "layer1.2.conv2.adder", "layer2.0.downsample.0.adder",
              "layer2.0.downsample.1.running_mean", "layer3.2.bn2.bias", "fc.weight", "bn2.num_batches_tracked"):
        assert k in keys
    assert not isinstance(m.conv1, adder.adder2d) and not isinstance(m.fc, adder.adder2d)   # resnet20.py:49,56
    # per-image adder work: 40.37 M (co, k, position) terms
    shapes = [(6, 16, 16, 9, 32), (1, 16, 32, 1, 16), (1, 16, 32, 9, 16), (5, 32, 32, 9, 16), (1, 32, 64, 1, 8),
              (1, 32, 64, 9, 8), (5, 64, 64, 9, 8)]
    assert sum(c * ci * co * kk * ho * ho for c, ci, co, kk, ho in shapes) == 40370176


def test_resnet20_runs_on_the_cpu_oracle_layer():
    """The same network built around the test oracle's layer trains for a step on CPU."""
    from addernetcuda_amd.resnet20 import resnet20
    from oracle import adder_oracle
    torch.manual_seed(0)
    m = resnet20(adder2d_cls=adder_oracle.adder2d, eta=0.1)
    x, y = torch.randn(2, 3, 32, 32), torch.tensor([1, 7])
    loss = torch.nn.functional.cross_entropy(m(x), y)
    loss.backward()
    g = m.layer1[0].conv1.adder.grad
    assert g.norm().item() == pytest.approx(0.1 * (16 * 16 * 9) ** 0.5, rel=1e-4)


# ---- training-script counterpart (addernetcuda_amd/train.py) ----------------------------------

def test_cosine_lr_matches_the_reference_schedule():
    import math
    from addernetcuda_amd.train import cosine_lr
    for epoch in (1, 37, 200, 399):
        assert cosine_lr(epoch, 400) == pytest.approx(0.025 * (1 + math.cos(float(epoch) / 400 * math.pi)))   # main.py:71
    assert cosine_lr(400, 400) == pytest.approx(0.0, abs=1e-12)


def test_augment_is_crop_of_the_padded_image_with_optional_flip():
    from addernetcuda_amd.train import augment
    g = torch.Generator().manual_seed(3)
    x = torch.randn(16, 3, 32, 32)
    out = augment(x, torch.Generator().manual_seed(5))
    assert out.shape == x.shape and out.is_contiguous()
    padded = torch.nn.functional.pad(x, (4, 4, 4, 4))
    flips = 0
    for n in range(16):
        crops = [(dy, dx, f) for dy in range(9) for dx in range(9) for f in (False, True)
                 if torch.equal(out[n], padded[n, :, dy:dy + 32, dx:dx + 32].flip(2) if f
                                else padded[n, :, dy:dy + 32, dx:dx + 32])]
        assert len(crops) == 1, "every output must be exactly one crop of its own padded image"
        flips += crops[0][2]
    assert 0 < flips < 16


def test_normalise_uses_the_cifar_constants():
    from addernetcuda_amd.train import normalise, CIFAR_MEAN, CIFAR_STD
    x = torch.full((1, 3, 32, 32), 255, dtype=torch.uint8)
    y = normalise(x)
    for c in range(3):
        assert y[0, c, 0, 0].item() == pytest.approx((1.0 - CIFAR_MEAN[c]) / CIFAR_STD[c], rel=1e-6)


def test_npz_loader_accepts_both_image_layouts(tmp_path):
    import numpy as np
    from addernetcuda_amd.train import load_arrays
    rng = np.random.default_rng(0)
    nhwc = rng.integers(0, 256, (6, 32, 32, 3), dtype=np.uint8)
    y = rng.integers(0, 10, 6)
    p = tmp_path / "d.npz"
    np.savez(p, x_train=nhwc, y_train=y, x_test=nhwc.transpose(0, 3, 1, 2), y_test=y)
    d = load_arrays(str(p), torch.device("cpu"))
    assert d["train"][0].shape == (6, 3, 32, 32) and torch.equal(d["train"][0], d["test"][0])
    assert d["train"][1].dtype == torch.int64


def test_batched_eta_scaling_drops_unfinished_gradients_on_an_exceptional_exit():
    """A weight the block had taken over holds an allocated but unfinished .grad; leaving the block through an
    exception (or failing in its exit) must not leave that memory where an optimizer could apply it."""
    import pytest
    from addernetcuda_amd import adder
    w1 = torch.nn.Parameter(torch.zeros(4, 3, 3, 3))
    w2 = torch.nn.Parameter(torch.zeros(2, 2))
    with pytest.raises(KeyboardInterrupt):
        with adder.batched_eta_scaling():
            w1.grad = torch.full_like(w1, 123.0)              # stands for the unsummed slabs' target
            adder._eta_batch.append((w1, 0.2, None, None))
            raise KeyboardInterrupt
    assert w1.grad is None and adder._eta_batch is None
    with pytest.raises(RuntimeError, match="missing"):
        with adder.batched_eta_scaling():
            w1.grad = torch.full_like(w1, 123.0)
            adder._eta_batch.append((w1, 0.2, None, None))
            adder._eta_batch.append((w2, 0.2, None, None))    # its .grad never arrived
    assert w1.grad is None and w2.grad is None and adder._eta_batch is None
