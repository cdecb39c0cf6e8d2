"""The training-script counterpart end to end on a small synthetic set: the loss falls, the evaluation
pass runs with a batch size the reference would have skipped (main.py:114), and the checkpoint it writes
has the reference's state_dict keys and reloads into a fresh model."""
import os

import pytest
import torch

pytestmark = pytest.mark.gpu


def test_two_epochs_learn_and_checkpoint(gpu, tmp_path):
    from addernetcuda_amd import train
    from addernetcuda_amd.resnet20 import resnet20
    args = train.parse_args(["--synthetic", "2000", "--epochs", "6", "--batch-size", "100",
                             "--test-batch-size", "50", "--output-dir", str(tmp_path), "--seed", "1"])
    hist = train.run(args)
    assert len(hist) == 6
    assert all(torch.isfinite(torch.tensor([h["train_loss"], h["test_loss"]])).all() for h in hist)
    assert hist[-1]["train_loss"] < hist[0]["train_loss"]
    assert hist[-1]["accuracy"] > 0.5          # ten classes of clearly separable patterns (0.84 when written)
    ckpt = os.path.join(str(tmp_path), "addernet.pt")
    assert os.path.exists(ckpt)
    state = torch.load(ckpt, map_location="cpu", weights_only=True)
    assert "layer1.0.conv1.adder" in state and "layer2.0.downsample.0.adder" in state and "bn2.running_mean" in state
    fresh = resnet20().to(gpu)
    fresh.load_state_dict(state)               # strict: same keys as the reference's resnet20.py
    # the evaluation-only pass (test.py's job) reproduces the accuracy of the epoch that wrote the checkpoint
    best = max(h["accuracy"] for h in hist)
    ev = train.run(train.parse_args(["--synthetic", "2000", "--resume", ckpt, "--eval-only", "--test-batch-size", "50",
                                     "--seed", "1"]))
    assert abs(ev[0]["accuracy"] - best) < 1e-6


def test_other_architectures_train(gpu, tmp_path):
    """--arch: the VGG-small stack through the same loop (graph capture included)."""
    from addernetcuda_amd import train
    hist = train.run(train.parse_args(["--arch", "vgg_small", "--synthetic", "2000", "--epochs", "6", "--batch-size", "100",
                                       "--test-batch-size", "50", "--output-dir", str(tmp_path), "--seed", "2"]))
    assert len(hist) == 6 and all(h["train_loss"] == h["train_loss"] for h in hist)      # finite, not NaN
    assert hist[-1]["train_loss"] < hist[0]["train_loss"]
    assert max(h["accuracy"] for h in hist) > 0.4          # 0.72 when written
    state = torch.load(os.path.join(str(tmp_path), "addernet.pt"), map_location="cpu", weights_only=True)
    assert "features.2.adder" in state and "classifier.weight" in state


def test_bfloat16_activation_mode_trains(gpu, tmp_path):
    """--bf16-activations: the optional reduced-storage mode through the same loop, eager and captured."""
    from addernetcuda_amd import train
    for extra in (["--no-graph"], []):
        hist = train.run(train.parse_args(["--synthetic", "2000", "--epochs", "5", "--batch-size", "100", "--test-batch-size",
                                           "50", "--output-dir", str(tmp_path), "--seed", "3", "--bf16-activations"] + extra))
        assert all(h["train_loss"] == h["train_loss"] for h in hist)
        assert hist[-1]["train_loss"] < hist[0]["train_loss"]
        assert max(h["accuracy"] for h in hist) > 0.4
