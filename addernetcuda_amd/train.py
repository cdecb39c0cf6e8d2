"""Training / evaluation loop for the ResNet-20 AdderNet: the counterpart of the reference's main.py.

What it keeps from main.py: SGD(momentum 0.9, weight decay 5e-4) (main.py:67), the per-epoch cosine
learning rate ``lr = 0.025 * (1 + cos(pi * epoch / epochs))`` (main.py:69-73), random-crop(32, pad 4) +
horizontal-flip augmentation and the CIFAR-10 normalisation constants (main.py:40-50), an evaluation pass
after every epoch and a ``state_dict`` checkpoint of the best model (main.py:105-128), whose keys are the
reference's (`adder`, `b`, BatchNorm names), so checkpoints move between the two code bases (test.py:39).

What it drops: the CIFAR download and wandb (no network here; data comes from an ``.npz`` file or is
synthetic), and the guards that skip batches whose size is not a multiple of 12 (main.py:83,114) — the
kernels take any batch size.  Augmentation runs on the GPU on uint8-derived tensors, so no worker
processes are needed.  What it adds: the training step of a full batch runs as one captured HIP graph
(``--no-graph`` keeps it eager): 2.3 instead of 3.5 ms per batch of 256.

    python -m addernetcuda_amd.train --synthetic 4096 --epochs 2
    python -m addernetcuda_amd.train --data cifar10.npz --epochs 400 --output-dir models/
    python -m addernetcuda_amd.train --data cifar10.npz --resume models/addernet.pt --eval-only
    (npz keys: x_train (N,32,32,3) or (N,3,32,32) uint8, y_train (N,), x_test, y_test)
"""
import argparse
import math
import os
import time

import torch
import torch.nn.functional as F

CIFAR_MEAN = (0.4914, 0.4822, 0.4465)
CIFAR_STD = (0.2023, 0.1994, 0.2010)


def cosine_lr(epoch, epochs, peak=0.05):
    """main.py:71 with its constants named: 0.025 * (1 + cos(pi * epoch / 400)), epoch counted from 1."""
    return 0.5 * peak * (1.0 + math.cos(float(epoch) / epochs * math.pi))


def normalise(images_u8):
    """uint8 (N,3,32,32) -> float32, transforms.ToTensor + Normalize of main.py:43-44."""
    x = images_u8.float().div_(255.0)
    mean = torch.tensor(CIFAR_MEAN, device=x.device).view(1, 3, 1, 1)
    std = torch.tensor(CIFAR_STD, device=x.device).view(1, 3, 1, 1)
    return (x - mean) / std


def augment(x, generator=None):
    """RandomCrop(32, padding=4) + RandomHorizontalFlip (main.py:41-42) on a normalised batch, per image."""
    n = x.shape[0]
    padded = F.pad(x, (4, 4, 4, 4))
    dy = torch.randint(0, 9, (n,), device=x.device, generator=generator)
    dx = torch.randint(0, 9, (n,), device=x.device, generator=generator)
    flip = torch.rand(n, device=x.device, generator=generator) < 0.5
    rows = dy.view(n, 1) + torch.arange(32, device=x.device).view(1, 32)            # (n, 32)
    cols = dx.view(n, 1) + torch.arange(32, device=x.device).view(1, 32)
    cols = torch.where(flip.view(n, 1), cols.flip(1), cols)
    idx_n = torch.arange(n, device=x.device).view(n, 1, 1, 1)
    idx_c = torch.arange(x.shape[1], device=x.device).view(1, -1, 1, 1)
    return padded[idx_n, idx_c, rows.view(n, 1, 32, 1), cols.view(n, 1, 1, 32)].contiguous()


def load_arrays(path, device):
    import numpy as np
    with np.load(path) as z:   # allow_pickle stays False
        out = {}
        for split in ("train", "test"):
            x = torch.from_numpy(z[f"x_{split}"])
            if x.dim() != 4:
                raise ValueError(f"x_{split}: expected 4 dimensions, got {tuple(x.shape)}")
            if x.shape[-1] == 3 and x.shape[1] != 3:
                x = x.permute(0, 3, 1, 2)
            out[split] = (x.contiguous().to(device), torch.from_numpy(z[f"y_{split}"]).long().to(device))
    return out


def synthetic_arrays(n, device, classes=10, seed=0):
    """A learnable stand-in for CIFAR: class-dependent colour blobs plus noise, uint8."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    proto = torch.rand(classes, 3, 32, 32, generator=g)
    proto = F.avg_pool2d(proto, 5, stride=1, padding=2)
    proto = (0.5 + 4.0 * (proto - 0.5)).clamp(0, 1)     # smooth, high-contrast class patterns
    out = {}
    for split, m in (("train", n), ("test", max(n // 8, 64))):
        y = torch.randint(0, classes, (m,), generator=g)
        x = proto[y] + 0.15 * torch.randn(m, 3, 32, 32, generator=g)
        out[split] = ((x.clamp(0, 1) * 255).to(torch.uint8).to(device), y.to(device))
    return out


def forward_pass(net, images, bf16=False):
    """Logits of a batch.  ``bf16``: the optional reduced-storage mode -- the images enter as bfloat16 under
    torch.autocast, so every activation between the layers is stored as bfloat16 and the adder layers take their
    bfloat16-storage kernels (float32 weights, float32 / float64 accumulation); the fused BatchNorm kernels are
    float32 only, so BatchNorm / ReLU then run as torch's own ops."""
    if not bf16:
        return net(images)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        return net(images.bfloat16()).float()


def evaluate(net, x_u8, y, batch, bf16=False):
    net.eval()
    correct, loss_sum = 0, 0.0
    with torch.no_grad():
        for i in range(0, x_u8.shape[0], batch):
            logits = forward_pass(net, normalise(x_u8[i:i + batch]), bf16)
            loss_sum += F.cross_entropy(logits, y[i:i + batch], reduction="sum").item()
            correct += (logits.argmax(1) == y[i:i + batch]).sum().item()
    n = x_u8.shape[0]
    return loss_sum / n, correct / n


def train_step(net, opt, images, labels, bf16=False):
    from addernetcuda_amd.adder import batched_eta_scaling
    from addernetcuda_amd.head import cross_entropy
    opt.zero_grad(set_to_none=True)
    loss = cross_entropy(forward_pass(net, images, bf16), labels)   # nn.CrossEntropyLoss of main.py:66,90
    with batched_eta_scaling():   # the adaptive scaling of all adder layers in two launches
        loss.backward()
    opt.step()
    return loss.detach()


class GraphedStep:
    """``train_step`` for one fixed batch shape as a captured HIP graph: the eager step spends more time in
    Python and launch calls than the GPU spends on the kernels.  The first ``warmup`` calls run eagerly (they are
    real training steps), the next one is captured, all later ones replay the capture on fresh data copied into
    the graph's input buffers.  The learning rate must be a device tensor of the optimizer (a float would be
    frozen into the graph); BatchNorm's running statistics and the optimizer state are updated by the graph's
    own kernels.  All calls must come from the same (non-default) stream."""

    def __init__(self, net, opt, warmup=3, bf16=False):
        self.net, self.opt, self.warmup, self.bf16 = net, opt, warmup, bf16
        self.graph = self.images = self.labels = self.loss = None
        self.calls = 0

    def __call__(self, images, labels):
        self.calls += 1
        if self.graph is None and self.calls <= self.warmup:
            return train_step(self.net, self.opt, images, labels, self.bf16)
        if self.graph is None:
            self.images, self.labels = images.clone(), labels.clone()
            self.opt.zero_grad(set_to_none=True)
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=torch.cuda.current_stream()):
                self.loss = train_step(self.net, self.opt, self.images, self.labels, self.bf16)
        else:
            self.images.copy_(images)
            self.labels.copy_(labels)
        self.graph.replay()
        return self.loss.clone()


def train_one_epoch(net, opt, x_u8, y, batch, generator=None, graphed=None, bf16=False):
    """``graphed``: a GraphedStep for batches of exactly ``batch`` images (the tail batch runs eagerly)."""
    net.train()
    n = x_u8.shape[0]
    perm = torch.randperm(n, device=x_u8.device, generator=generator)
    losses = []
    for i in range(0, n, batch):
        idx = perm[i:i + batch]
        if idx.numel() < 2:     # BatchNorm needs more than one value per channel
            break
        images = augment(normalise(x_u8[idx]), generator)
        step = graphed if graphed is not None and idx.numel() == batch else None
        losses.append(step(images, y[idx]) if step else train_step(net, opt, images, y[idx], bf16))
    return torch.stack(losses).mean().item()


ARCHS = ("resnet20", "vgg_small", "densenet_cifar", "resnet50")


def build_network(arch, eta, num_classes=10):
    """The reference's networks for 32x32 inputs (main.py:66 builds resnet20; vgg.py, densenet.py and resnet50.py
    are its other model files)."""
    if arch == "resnet20":
        from addernetcuda_amd.resnet20 import resnet20
        return resnet20(eta=eta, num_classes=num_classes)
    if arch not in ARCHS:
        raise ValueError(f"unknown architecture {arch!r}: one of {ARCHS}")
    from addernetcuda_amd import models
    return getattr(models, arch)(eta=eta, num_classes=num_classes)


def run(args):
    if not torch.cuda.is_available():
        raise RuntimeError("addernetcuda_amd.train needs an MI355X: the adder kernels have no CPU path")
    dev = torch.device("cuda:0")
    torch.manual_seed(args.seed)
    data = synthetic_arrays(args.synthetic, dev, seed=args.seed) if args.data is None else load_arrays(args.data, dev)
    net = build_network(args.arch, args.eta).to(dev)
    if args.resume:
        net.load_state_dict(torch.load(args.resume, map_location=dev, weights_only=True))
    # the learning rate lives on the device so that the captured step sees each epoch's value
    lr_now = torch.tensor(float(args.lr), device=dev)
    from addernetcuda_amd.optim import SGD   # torch.optim.SGD's rule and state, all parameters in one launch
    opt = SGD(net.parameters(), lr=lr_now, momentum=0.9, weight_decay=5e-4)
    if args.eval_only:   # the reference's test.py: load a checkpoint, one pass over the test split
        test_loss, acc = evaluate(net, *data["test"], args.test_batch_size, args.bf16_activations)
        print(f"test loss {test_loss:.4f}  accuracy {acc:.4f}", flush=True)
        return [{"epoch": 0, "test_loss": test_loss, "accuracy": acc}]
    os.makedirs(args.output_dir, exist_ok=True)
    gen = torch.Generator(device=dev).manual_seed(args.seed)
    graphed = None if args.no_graph else GraphedStep(net, opt, bf16=args.bf16_activations)
    stream = torch.cuda.Stream()   # graph capture needs a stream of its own; the eager steps share it
    best, history = 0.0, []
    for epoch in range(1, args.epochs + 1):
        lr = cosine_lr(epoch, args.epochs, args.lr)
        torch.cuda.synchronize()
        lr_now.fill_(lr)
        t0 = time.time()
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            train_loss = train_one_epoch(net, opt, *data["train"], args.batch_size, gen, graphed, args.bf16_activations)
        torch.cuda.synchronize()
        dt = time.time() - t0
        test_loss, acc = evaluate(net, *data["test"], args.test_batch_size, args.bf16_activations)
        history.append({"epoch": epoch, "lr": lr, "train_loss": train_loss, "test_loss": test_loss, "accuracy": acc,
                        "seconds": dt})
        print(f"epoch {epoch}: lr {lr:.5f}  train loss {train_loss:.4f}  test loss {test_loss:.4f}  "
              f"accuracy {acc:.4f}  {dt:.1f} s", flush=True)
        if acc > best:
            best = acc
            torch.save(net.state_dict(), os.path.join(args.output_dir, "addernet.pt"))
    return history


def parse_args(argv=None):
    p = argparse.ArgumentParser(description="train an AdderNet (ResNet-20 by default) on an MI355X")
    p.add_argument("--data", type=str, default=None, help=".npz with x_train, y_train, x_test, y_test (uint8 images)")
    p.add_argument("--synthetic", type=int, default=8192, help="training-set size when --data is not given")
    p.add_argument("--output-dir", type=str, default="./models/")
    p.add_argument("--resume", type=str, default=None, help="state_dict to start from")
    p.add_argument("--eval-only", action="store_true", help="evaluate the --resume checkpoint and stop (test.py:74-80)")
    p.add_argument("--epochs", type=int, default=400)                 # main.py:135
    p.add_argument("--batch-size", type=int, default=256)
    p.add_argument("--test-batch-size", type=int, default=500)
    p.add_argument("--lr", type=float, default=0.05, help="peak of the cosine schedule (main.py:71: 2 x 0.025)")
    p.add_argument("--eta", type=float, default=0.2, help="adaptive grad_W scale, adder.py:78 uses 1/5")
    p.add_argument("--no-graph", action="store_true", help="run every training step eagerly instead of as a HIP graph")
    p.add_argument("--bf16-activations", action="store_true",
                   help="optional mode: activations stored as bfloat16 between the layers (float32 weights, float32 / "
                        "float64 accumulation in the adder kernels); the default, like the reference, is float32 throughout")
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--arch", choices=ARCHS, default="resnet20", help="network (main.py:66 trains resnet20)")
    return p.parse_args(argv)


if __name__ == "__main__":
    run(parse_args())
