#!/usr/bin/env python3
"""ResNet-20 AdderNet training-step benchmark on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-graph] [--no-cpu] [--layers]

Prints ONE JSON line.  `value` is milliseconds per training step (forward +
backward + SGD) of the ResNet-20 AdderNet at batch 256, 3x32x32 fp32 synthetic
input resident in HBM; `layers` carries, per adder-layer shape of the network,
the time, TFLOP/s and fraction of the fp32 vector peak of each of the three
kernels; `roofline` is the dominant kernel; `cpu_baseline` is the CPU oracle's
training step (batch 8, scaled to 256) timed on this box's host cores.
"""
import argparse
import ctypes
import json
import math
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP64_MFMA_TFLOPS = 78.6       # MI355X fp64 matrix peak: the 3x3 weight gradient runs on v_mfma_f64_16x16x4_f64
PEAK_FP32_TFLOPS = 157.3           # MI355X vendor fp32 vector peak (256 CU x 64 lanes x 2 (packed) x 2 (FMA) x 2.4 GHz)
# lane-instructions per second: a SIMD starts two vector instructions per 4-cycle slot when two of its
# waves are ready (one per wave), so 256 CU x 4 SIMD x 2 x 64 lanes / 4 cycles x 2.4 GHz; with an FMA in
# every slot this is the 157.3 TFLOP/s above.
PEAK_VALU_ISSUE = 2 * 256 * 64 * 2.4e9
BATCH = 256
ETA = 0.1
# HBM bytes per launch of the dominant kernel, from the rocprofv3 counter passes kept under profiles/
# (37.0 MB fetched + 19.1 MB written; cannot be read without the profiler attached)
DOMINANT_TRAFFIC_BYTES = 56.1e6

# distinct adder-layer shapes of ResNet-20 at 32x32 input: (count, Ci, H, W, Co, k, stride, pad)
RESNET20_LAYERS = [
    (6, 16, 32, 32, 16, 3, 1, 1),
    (1, 16, 32, 32, 32, 1, 2, 0),
    (1, 16, 32, 32, 32, 3, 2, 1),
    (5, 32, 16, 16, 32, 3, 1, 1),
    (1, 32, 16, 16, 64, 1, 2, 0),
    (1, 32, 16, 16, 64, 3, 2, 1),
    (5, 64, 8, 8, 64, 3, 1, 1),
]
# adder layers of the two other model configurations the reference ships (vgg.py / resnet50.py shapes at the
# batch sizes its README quotes): (count, Ci, H, W, Co, k, stride, pad); batch 128 and 64
VGG_SMALL_LAYERS = [
    (1, 128, 32, 32, 128, 3, 1, 1), (1, 128, 16, 16, 256, 3, 1, 1), (1, 256, 16, 16, 256, 3, 1, 1),
    (1, 256, 8, 8, 512, 3, 1, 1), (1, 512, 8, 8, 512, 3, 1, 1),
]
RESNET50_LAYERS = [
    (4, 64, 56, 56, 256, 1, 1, 0), (1, 64, 56, 56, 64, 1, 1, 0), (3, 64, 56, 56, 64, 3, 1, 1),
    (2, 256, 56, 56, 64, 1, 1, 0), (1, 256, 56, 56, 512, 1, 2, 0), (1, 256, 56, 56, 128, 1, 1, 0),
    (1, 128, 56, 56, 128, 3, 2, 1), (4, 128, 28, 28, 512, 1, 1, 0), (3, 512, 28, 28, 128, 1, 1, 0),
    (3, 128, 28, 28, 128, 3, 1, 1), (1, 512, 28, 28, 1024, 1, 2, 0), (1, 512, 28, 28, 256, 1, 1, 0),
    (1, 256, 28, 28, 256, 3, 2, 1), (6, 256, 14, 14, 1024, 1, 1, 0), (5, 1024, 14, 14, 256, 1, 1, 0),
    (5, 256, 14, 14, 256, 3, 1, 1), (1, 1024, 14, 14, 2048, 1, 2, 0), (1, 1024, 14, 14, 512, 1, 1, 0),
    (1, 512, 14, 14, 512, 3, 2, 1), (3, 512, 7, 7, 2048, 1, 1, 0), (2, 2048, 7, 7, 512, 1, 1, 0),
    (2, 512, 7, 7, 512, 3, 1, 1),
]
LAYER_SETS = {"resnet20": (BATCH, RESNET20_LAYERS), "vgg_small": (128, VGG_SMALL_LAYERS),
              "resnet50": (64, RESNET50_LAYERS)}
# flops per (co, k, position) term and the fewest fp32 VALU instructions that implement it
OPS = {"fwd": (2, 2), "grad_x": (4, 2), "grad_w": (3, 1)}


# seconds of the same call before every timing; ADDER_BENCH_WARM_S=0 for profiler runs that should hold few dispatches
WARM_SECONDS = float(os.environ.get("ADDER_BENCH_WARM_S", "0.04"))


def event_time(fn, warmup, iters):
    """Average seconds per call, HIP events on the stream the kernels are launched on (torch's current one).

    The card raises its clocks over the first tens of milliseconds of continuous work (the same kernel measures
    31.8, 30.6 and 28.7 us as the 1st, 3rd and 7th timing of a process), so every timing is preceded by
    WARM_SECONDS of the same call: what is reported is the rate the kernels run at inside a training step.
    """
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < WARM_SECONDS:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e-3 / iters


def layer_ops(N, Ci, H, W, Co, k, stride, pad, dev):
    """The three C-ABI calls of one layer shape on synthetic tensors; returns (E, {op: callable})."""
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, conv_dims, check
    g = torch.Generator(device=dev).manual_seed(1000 + Ci + Co + k + stride)
    x = torch.randn(N, Ci, H, W, device=dev, generator=g)
    w = torch.randn(Co, Ci, k, k, device=dev, generator=g) * math.sqrt(2.0 / (Ci * k * k))
    dims, Ho, Wo = conv_dims(x.shape, w.shape, stride, pad)
    y = torch.empty(N, Co, Ho, Wo, device=dev)
    gy = torch.randn(N, Co, Ho, Wo, device=dev, generator=g)
    gx, gw = torch.empty_like(x), torch.empty_like(w)
    need = ctypes.c_size_t()
    check(lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)), "workspace")
    ws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=dev)
    st = stream_ptr(dev)
    E = Co * Ci * k * k * N * Ho * Wo
    nx, ny, nw = 4 * x.numel(), 4 * y.numel(), 4 * w.numel()
    # algorithmic HBM bytes of each call: every tensor it reads or writes crosses HBM once.  A 1x1 layer with a
    # stride reads x at every stride-th row and column only: the rows it skips never leave HBM, the columns it skips
    # share their 128-byte lines with the ones it reads, so x counts with 1 / stride of its bytes where it is read
    # (grad_X still writes all of gx, the zeros included).
    rx = nx // stride if k == 1 else nx
    nbytes = {"fwd": rx + nw + ny, "grad_x": rx + nx + ny + nw, "grad_w": rx + ny + 2 * nw}
    keep = [x, w, y, gy, gx, gw, ws]
    ops = {
        "fwd": lambda: check(lib.adder_conv2d_fwd_f32(ptr(x), ptr(w), ptr(y), *dims, st), "fwd"),
        "grad_x": lambda: check(lib.adder_conv2d_bwd_f32(ptr(gy), ptr(x), ptr(w), ptr(gx), None, 0.0, None, 0,
                                                         *dims, st), "grad_x"),
        "grad_w": lambda: check(lib.adder_conv2d_bwd_f32(ptr(gy), ptr(x), ptr(w), None, ptr(gw), ETA, ptr(ws),
                                                         need.value, *dims, st), "grad_w"),
    }
    # The calls as the training step makes them for a layer between two BatchNorms (unit.py): grad_W forms the
    # layer's output gradient from (dz, the layer's output, 4 coefficients per channel) and leaves it in memory,
    # grad_X reads it, masks its result with x > 0 and leaves the sums of the BatchNorm in front of the layer.
    from addernetcuda_amd._lib import BnLinks, bwd_bn_slots
    slots = bwd_bn_slots(dims)
    if slots > 0:
        bn_in = torch.randn(N, Ci, H, W, device=dev, generator=g) * 20 - 90
        mean, rstd = bn_in.mean((0, 2, 3)), 1.0 / bn_in.std((0, 2, 3))
        part = torch.empty(Ci, slots, 2, dtype=torch.float32, device=dev)
        coef = torch.randn(Co, 4, device=dev, generator=g) * 0.01
        yo = torch.randn(N, Co, Ho, Wo, device=dev, generator=g) * 20 - 90
        gyo = torch.empty_like(gy)
        # (the BatchNorm in front with its weight and bias, as for a unit whose input had no residual added: the
        # stride-1 3x3 and 1x1 kernels then take xhat from x and do not read bn_in; 2 of 3 launches of a ResNet step)
        gamma, beta = torch.ones(Ci, device=dev), torch.zeros(Ci, device=dev)
        lx = BnLinks(None, None, None, ptr(bn_in), ptr(mean), ptr(rstd), ptr(part), slots, 1, ptr(gamma), ptr(beta))
        lw = BnLinks(ptr(yo), ptr(coef), ptr(gyo), None, None, None, None, 0, 0)
        keep += [bn_in, mean, rstd, part, coef, yo, gyo, lx, lw, gamma, beta]
        ops["grad_x_bn"] = lambda: check(lib.adder_conv2d_bwd_bn_f32(ptr(gy), ptr(x), ptr(w), None, ptr(gx), None, 0.0,
                                                                      None, 0, *dims, ctypes.byref(lx), st), "grad_x_bn")
        ops["grad_w_bn"] = lambda: check(lib.adder_conv2d_bwd_bn_f32(ptr(gy), ptr(x), ptr(w), None, None, ptr(gw), ETA,
                                                                      ptr(ws), need.value, *dims, ctypes.byref(lw), st),
                                         "grad_w_bn")
        # + the partial sums, + the BatchNorm's input where the kernel reads it (stride 2)
        nbytes["grad_x_bn"] = nbytes["grad_x"] + 8 * Ci * slots + (nx if stride != 1 else 0)
        nbytes["grad_w_bn"] = nbytes["grad_w"] + 2 * ny                 # + the layer's output, + the formed gradient
    return E, ops, keep, nbytes


def bench_layers(dev, warmup=5, iters=20, which="resnet20"):
    rows = []
    batch, layers = LAYER_SETS[which]
    for cnt, Ci, H, W, Co, k, s, p in layers:
        E, ops, keep, nbytes = layer_ops(batch, Ci, H, W, Co, k, s, p, dev)
        for name, fn in ops.items():
            t = event_time(fn, warmup, iters)
            flop, slots = OPS[name[:-3] if name.endswith("_bn") else name]
            row = {
                "layer": f"{Ci}->{Co} k{k} s{s} p{p} @{H}x{W}", "count": cnt, "op": name, "us": round(t * 1e6, 2),
                "tflops": round(flop * E / t / 1e12, 2),
                "frac_fp32_peak": round(flop * E / t / 1e12 / PEAK_FP32_TFLOPS, 4),
                "algorithmic_bytes": nbytes[name], "hbm_gbs": round(nbytes[name] / t / 1e9, 1),
                "frac_hbm_peak": round(nbytes[name] / t / 1e9 / PEAK_HBM_GBS, 4),
            }
            if name in ("grad_w", "grad_w_bn") and k == 3:   # fp64 matrix-core kernel (+ finalize and scaling launches)
                row["frac_fp64_mfma_peak"] = round(2 * E / t / 1e12 / PEAK_FP64_MFMA_TFLOPS, 4)
            else:
                row["valu_issue_util"] = round(slots * E / t / PEAK_VALU_ISSUE, 4)
            rows.append(row)
        del keep
    return rows


# column-matrix shapes (Co, K, NL) for the literal ADDER_* entry points: the default of the reference's
# comparison script (adder_cuda/test_cuda.py:161-176) and the dominant ResNet-20 layer as adder.py:22-41 unfolds it
COL_SHAPES = [(32, 288, 1024), (16, 144, 262144)]
PEAK_HBM_GBS = 8000.0


def bench_col(dev, warmup=3, iters=10):
    """The four entry points of the reference extension on (K, NL) column matrices: time, GB/s against the HBM
    peak (these kernels stream X_col, which is 9x the activation for a 3x3 layer) and TFLOP/s."""
    from addernetcuda_amd import adder_cuda
    rows = []
    for Co, K, NL in COL_SHAPES:
        g = torch.Generator(device=dev).manual_seed(1000 + Co + K)
        X = torch.randn(K, NL, device=dev, generator=g)
        Wm = torch.randn(Co, K, device=dev, generator=g) * math.sqrt(2.0 / K)
        gy = torch.randn(Co, NL, device=dev, generator=g)
        out, gW, gX = torch.empty(Co, NL, device=dev), torch.zeros(Co, K, device=dev), torch.zeros(K, NL, device=dev)
        E = Co * K * NL
        # algorithmic HBM bytes; gradients are accumulated into (read + written), as the reference's atomicAdd does
        b_x, b_w, b_y = 4 * K * NL, 4 * Co * K, 4 * Co * NL
        ops = {
            "ADDER_CONV": (lambda: adder_cuda.ADDER_CONV(X, Wm, out), 2, b_x + b_w + b_y),
            "ADDER_CONV_WEIGHT": (lambda: adder_cuda.ADDER_CONV_WEIGHT(gy, X, Wm, gW), 3, b_x + b_y + 3 * b_w),
            "ADDER_CONV_INPUT": (lambda: adder_cuda.ADDER_CONV_INPUT(gy, X, Wm, gX), 4, 3 * b_x + b_y + b_w),
            "ADDER_BACKWARD": (lambda: adder_cuda.ADDER_BACKWARD(gy, X, Wm, gW, gX), 7, 3 * b_x + b_y + 3 * b_w),
        }
        for name, (fn, flop, nbytes) in ops.items():
            t = event_time(fn, warmup, iters)
            rows.append({"shape": f"Co={Co} K={K} NL={NL}", "op": name, "us": round(t * 1e6, 2),
                         "algorithmic_bytes": nbytes, "gbs": round(nbytes / t / 1e9, 1),
                         "frac_hbm_peak": round(nbytes / t / 1e9 / PEAK_HBM_GBS, 4),
                         "tflops": round(flop * E / t / 1e12, 2),
                         "frac_fp32_peak": round(flop * E / t / 1e12 / PEAK_FP32_TFLOPS, 4)})
    return rows


def dominant_kernel(dev, steps):
    """grad_x of the 16->16 3x3 @32x32 layer, as the training step launches it (with the statistics of the
    BatchNorm in front of the layer in its epilogue): the kernel with the largest share of a training step.
    `plain_kernel` repeats the figures for the same kernel without that epilogue (adder_conv2d_bwd_f32)."""
    cnt, Ci, H, W, Co, k, s, p = RESNET20_LAYERS[0]
    E, ops, keep, nbytes = layer_ops(BATCH, Ci, H, W, Co, k, s, p, dev)
    t = event_time(ops["grad_x_bn"], 5, max(20, steps))
    t_plain = event_time(ops["grad_x"], 5, max(20, steps))
    flop = OPS["grad_x"][0] * E
    achieved = flop / t / 1e12
    return {
        "plain_kernel": {"avg_launch_us": round(t_plain * 1e6, 2), "achieved": round(flop / t_plain / 1e12, 2),
                         "frac": round(flop / t_plain / 1e12 / PEAK_FP32_TFLOPS, 4),
                         "algorithmic_bytes": nbytes["grad_x"]},
        "bound": "valu", "kernel": "adder::grad_x_3x3s1_kernel<..., FUSE = true> (16->16, 3x3 s1 p1, 32x32, batch 256; "
                                   "masks its result and sums it for the BatchNorm in front of the layer)",
        "achieved": round(achieved, 2), "peak": PEAK_FP32_TFLOPS, "unit": "TFLOP/s",
        "frac": round(achieved / PEAK_FP32_TFLOPS, 4), "traffic": DOMINANT_TRAFFIC_BYTES,
        "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a 256 MiB copy: "
                          "profiles/grad_x_3x3s1_resnet20_16to16_32x32_bs256.md",
        "algorithmic_bytes": nbytes["grad_x_bn"],
        "avg_launch_us": round(t * 1e6, 2), "flop_per_launch": flop,
        "valu_issue_util": round(OPS["grad_x"][1] * E / t / PEAK_VALU_ISSUE, 4),
        "note": "fp32 VALU-bound (|a-b| accumulation has no FMA/MFMA form). The 157.3 TFLOP/s peak needs an FMA "
                "in each of the two vector issue slots a SIMD has per 4 cycles; this op spends 2 instructions "
                "(v_fma with the clamp modifier, v_fmac) on the 4 flop of a term (sub, clamp, mul, add), so the "
                "peak itself is its ceiling. valu_issue_util is the share of the two-slot issue rate taken by "
                "those 2 instructions per term. The flop count is the adder layer's alone: the epilogue (mask, two "
                "sums per channel; xhat comes from the x the lanes hold) is the first pass of a BatchNorm backward that no longer "
                "runs as a kernel of its own.",
    }


def parity_gate(dev, images=4):
    """Before anything is timed: forward, grad_X, raw and eta-scaled grad_W of the three config-2 layer shapes (a few
    images each) through the C ABI against the float64 C oracle, at the bar rtol 1e-5 / atol 1e-4.  Reported per
    output as the worst element's share of that tolerance, next to the same figure for the float32 pure-PyTorch
    oracle (the reference's formulas) against the same float64 truth.  Raises if the HIP path misses the bar."""
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, conv_dims, check
    from oracle import c_oracle, adder_oracle
    rows = []
    for cnt, Ci, H, W, Co, k, s, p in RESNET20_LAYERS:
        if not (k == 3 and s == 1):
            continue
        g = torch.Generator().manual_seed(2000 + Ci)
        x = torch.randn(images, Ci, H, W, generator=g)
        w = torch.randn(Co, Ci, k, k, generator=g) * math.sqrt(2.0 / (Ci * k * k))
        gy = torch.randn(images, Co, H, W, generator=g)
        dims, Ho, Wo = conv_dims(x.shape, w.shape, s, p)
        xg, wg, gyg = x.to(dev), w.to(dev), gy.to(dev)
        y, gx, gw, gws = torch.empty_like(gyg), torch.empty_like(xg), torch.empty_like(wg), torch.empty_like(wg)
        need = ctypes.c_size_t()
        check(lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)), "workspace")
        ws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=dev)
        st = stream_ptr(dev)
        check(lib.adder_conv2d_fwd_f32(ptr(xg), ptr(wg), ptr(y), *dims, st), "fwd")
        check(lib.adder_conv2d_bwd_f32(ptr(gyg), ptr(xg), ptr(wg), ptr(gx), ptr(gw), 0.0, ptr(ws), need.value, *dims, st), "bwd")
        check(lib.adder_conv2d_bwd_f32(ptr(gyg), ptr(xg), ptr(wg), None, ptr(gws), ETA, ptr(ws), need.value, *dims, st), "bwd")
        torch.cuda.synchronize()
        truth = {"fwd": c_oracle.conv2d_fwd(x, w, s, p), "grad_x": c_oracle.conv2d_grad_x(gy, x, w, s, p),
                 "grad_w": c_oracle.conv2d_grad_w(gy, x, w, s, p)}
        truth["grad_w_eta_scaled"] = c_oracle.eta_scale(truth["grad_w"], ETA)
        o_gx, o_gw, o_gws = adder_oracle.conv2d_backward(gy, x, w, s, p, eta=ETA)
        torch32 = {"fwd": adder_oracle.conv2d_forward(x, w, s, p), "grad_x": o_gx, "grad_w": o_gw, "grad_w_eta_scaled": o_gws}
        hip = {"fwd": y, "grad_x": gx, "grad_w": gw, "grad_w_eta_scaled": gws}
        share = lambda got, want: float(((got.double().cpu() - want).abs() / (1e-4 + 1e-5 * want.abs())).max())
        row = {"layer": f"{Ci}->{Co} k{k} s{s} p{p} @{H}x{W}", "images": images}
        for name, want in truth.items():
            row[name] = {"hip_share_of_tolerance": round(share(hip[name], want), 4),
                         "torch_f32_oracle_share_of_tolerance": round(share(torch32[name], want), 4)}
            if not row[name]["hip_share_of_tolerance"] <= 1.0:
                raise SystemExit(f"bench.py: parity gate failed before timing: {row['layer']} {name} at "
                                 f"{row[name]['hip_share_of_tolerance']} of rtol 1e-5 / atol 1e-4")
        rows.append(row)
    return rows


def make_step(model, opt, x, y):
    from addernetcuda_amd.adder import batched_eta_scaling

    def step():
        opt.zero_grad(set_to_none=True)
        loss = getattr(model, "criterion", torch.nn.functional.cross_entropy)(model(x), y)
        with batched_eta_scaling():   # adder.py:78 for all adder layers in two launches after the backward pass
            loss.backward()
        opt.step()
        return loss
    return step


# the reference's three model configurations: (batch, input size, classes)
MODELS = {"resnet20": (BATCH, 32, 10), "vgg_small": (128, 32, 10), "resnet50": (64, 224, 1000),
          "densenet_cifar": (64, 32, 10)}


def build_training(dev, seed=0, which="resnet20", fused=True):
    torch.manual_seed(seed)
    batch, size, classes = MODELS[which]
    if which == "resnet20":
        from addernetcuda_amd.resnet20 import resnet20
        model = resnet20(eta=ETA, fused=fused)
    else:
        from addernetcuda_amd import models
        model = getattr(models, which)(num_classes=classes, eta=ETA, fused=fused)
    model = model.to(dev)
    # nn.CrossEntropyLoss of main.py:66 -- one launch each way for up to 32 classes; the framework's own with the
    # reference's stock modules
    from addernetcuda_amd.head import cross_entropy
    model.criterion = cross_entropy if fused else torch.nn.functional.cross_entropy
    # torch.optim.SGD's update rule and state (main.py:67) with all parameters in one launch; with the reference's
    # stock modules (fused=False) the framework's own fused update
    if fused:
        from addernetcuda_amd.optim import SGD
        opt = SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=5e-4)
    else:
        opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=5e-4, fused=True)
    g = torch.Generator(device=dev).manual_seed(seed + 1)
    x = torch.randn(batch, 3, size, size, device=dev, generator=g)
    y = torch.randint(0, classes, (batch,), device=dev, generator=g)
    return model, opt, x, y


def capture_step(model, opt, x, y):
    """Whole training step as one HIP graph (the eager step is launch-bound on the host)."""
    step = make_step(model, opt, x, y)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    opt.zero_grad(set_to_none=True)
    from addernetcuda_amd.adder import batched_eta_scaling
    with torch.cuda.graph(graph):
        loss = getattr(model, "criterion", torch.nn.functional.cross_entropy)(model(x), y)
        with batched_eta_scaling():
            loss.backward()
        opt.step()
    return graph, loss


def graph_matches_eager(dev, replays=4, which="resnet20", fused=True):
    """Replay the captured step from a saved state and run the eager step from the same state, several times.

    Torch's own kernels are not run-to-run deterministic, so trajectories cannot be compared over many steps;
    one step from identical weights, momentum and BatchNorm statistics can.
    """
    import copy
    model, opt, x, y = build_training(dev, which=which, fused=fused)
    graph, loss = capture_step(model, opt, x, y)
    eager = make_step(model, opt, x, y)
    worst = 0.0
    losses = []
    for _ in range(replays):
        saved = ({k: v.clone() for k, v in model.state_dict().items()}, copy.deepcopy(opt.state_dict()))
        graph.replay()
        torch.cuda.synchronize()
        lg = loss.item()
        pg = {k: v.clone() for k, v in model.state_dict().items()}
        model.load_state_dict(saved[0])
        opt.load_state_dict(saved[1])
        le = eager().item()
        torch.cuda.synchronize()
        pe = model.state_dict()
        worst = max(worst, max((pg[k].float() - pe[k].float()).abs().max().item() for k in pg))
        losses.append((lg, le))
    ok = worst <= 1e-4 and all(abs(a - b) <= 1e-4 * max(1.0, abs(b)) for a, b in losses)
    return ok, worst, losses


def layer_set_summary(rows):
    """Adder-kernel time per training step of a layer set and the flop-weighted fraction of the fp32 vector peak
    over all of its adder kernels (forward 2, grad_X 4, grad_W 3 flop per term), from the rows of the plain entry
    points (the *_bn rows time the same layers' backward calls with the BatchNorm links)."""
    rows = [r for r in rows if not r["op"].endswith("_bn")]
    t = sum(r["us"] * r["count"] for r in rows) * 1e-6
    flop = sum(r["tflops"] * 1e12 * r["us"] * 1e-6 * r["count"] for r in rows)
    return {"adder_kernel_ms_per_step": round(t * 1e3, 3), "adder_kernels_tflops": round(flop / t / 1e12, 2),
            "adder_kernels_frac_fp32_peak": round(flop / t / 1e12 / PEAK_FP32_TFLOPS, 4)}


def time_training(dev, which, fused, steps, warmup, use_graph=True, replays=2):
    """ms per training step of one model configuration: captured as one HIP graph when its replays reproduce
    the eager step from the same state, eagerly otherwise."""
    mode, graph_check = "eager", None
    if use_graph:
        ok, worst, losses = graph_matches_eager(dev, replays=replays, which=which, fused=fused)
        graph_check = {"ok": ok, "max_param_diff_vs_eager_step": worst,
                       "loss_graph_vs_eager": [[round(a, 6), round(b, 6)] for a, b in losses]}
        if ok:
            mode = "hipgraph"
    model, opt, x, y = build_training(dev, which=which, fused=fused)
    if mode == "hipgraph":
        graph, loss = capture_step(model, opt, x, y)
        run = graph.replay
    else:
        run = make_step(model, opt, x, y)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    del run, model, opt
    if mode == "hipgraph":
        del graph, loss
    torch.cuda.empty_cache()
    return ms, mode, graph_check


def other_configs(dev):
    """The two other model configurations and the stock-module ResNet-20, one compact record each."""
    out = []
    for which, fused, label in (("resnet20", False, "ResNet-20 bs256, the reference's model file with stock nn.Conv2d / "
                                                    "BatchNorm2d / ReLU modules (only the adder layers differ)"),
                                ("vgg_small", True, "VGG-small AdderNet bs128, 3x32x32 (K up to 4608)"),
                                ("resnet50", True, "ResNet-50 AdderNet bs64, 3x224x224, 1000 classes")):
        ms, mode, check = time_training(dev, which, fused, steps=10, warmup=3)
        rec = {"config": label, "ms_per_step": round(ms, 3), "images_per_s": round(MODELS[which][0] / ms * 1e3, 1),
               "step_mode": mode, "graph_check_ok": None if check is None else check["ok"]}
        if which in LAYER_SETS and fused:
            rec.update(layer_set_summary(bench_layers(dev, warmup=2, iters=5, which=which)))
        out.append(rec)
    return out


def cpu_model_name():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_layer_baseline(repeats=3):   # ~25 s of host work
    """The per-layer benchmark configuration on the host: the three 3x3 / stride 1 / pad 1 layer shapes (16, 32, 64 channels at 32, 16, 8
    pixels, batch 256) through the chunked torch oracle -- unfold (adder.py:32-33), forward (test_cuda.py:18-22),
    grad_W (test_cuda.py:35-41), grad_X (test_cuda.py:57-60), and grad_W with the scaling of adder.py:78 -- each
    the median of `repeats` runs."""
    from oracle import adder_oracle as o
    rows = []
    for cnt, Ci, H, W, Co, k, s, p in RESNET20_LAYERS:
        if not (k == 3 and s == 1):
            continue
        g = torch.Generator().manual_seed(1000 + Ci + Co + k + s)
        x = torch.randn(BATCH, Ci, H, W, generator=g)
        w = torch.randn(Co, Ci, k, k, generator=g) * math.sqrt(2.0 / (Ci * k * k))
        gy = torch.randn(BATCH, Co, H, W, generator=g)
        E = Co * Ci * k * k * BATCH * H * W
        W_col = w.reshape(Co, -1)
        state = {}

        def unfold():
            state["X"], _, _ = o.im2col(x, k, s, p)
            state["g"] = o.nchw_to_out_col(gy)
        unfold()
        ops = {
            "unfold": (unfold, 0),
            "fwd": (lambda: o.col_forward(state["X"], W_col), 2),
            "grad_w": (lambda: state.__setitem__("gw", o.col_grad_w(state["X"], W_col, state["g"])), 3),
            "grad_x": (lambda: o.col_grad_x(state["X"], W_col, state["g"]), 4),
            "grad_w_eta_scaled": (lambda: o.eta_scale(o.col_grad_w(state["X"], W_col, state["g"]), ETA), 3),
        }
        for name, (fn, flop) in ops.items():
            times = []
            for _ in range(repeats):
                t0 = time.perf_counter()
                fn()
                times.append(time.perf_counter() - t0)
            med = statistics.median(times)
            row = {"layer": f"{Ci}->{Co} k{k} s{s} p{p} @{H}x{W}", "batch": BATCH, "op": name, "ms": round(med * 1e3, 1)}
            if flop:
                row["gflops"] = round(flop * E / med / 1e9, 1)
            rows.append(row)
    return rows


def cpu_baseline(repeats=15):   # ~10 s of host work
    """The CPU oracle's ResNet-20 training step at batch 8 (seeded), median of `repeats`, scaled to batch 256."""
    from addernetcuda_amd.resnet20 import resnet20
    from oracle import adder_oracle
    torch.manual_seed(0)
    model = resnet20(adder2d_cls=adder_oracle.adder2d, eta=ETA)
    opt = torch.optim.SGD(model.parameters(), lr=0.1, momentum=0.9, weight_decay=5e-4)
    bs = 8
    x = torch.randn(bs, 3, 32, 32)
    y = torch.randint(0, 10, (bs,))
    step = make_step(model, opt, x, y)
    step()
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {
        "value": round(med * 1e3 * (BATCH / bs), 1), "unit": "ms/batch (batch 256)", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"ResNet-20 AdderNet fwd+bwd+SGD at batch {bs} through the pure-PyTorch unfold oracle, median of "
                  f"{repeats} steps = {med * 1e3:.0f} ms, scaled x{BATCH // bs} to batch 256",
        "host_cpus": os.cpu_count(), "cpu_model": cpu_model_name(),
        "layers": cpu_layer_baseline(),
        "layers_note": "the per-layer benchmark configuration on the host cores: the three stride-1 3x3 shapes at batch 256 through the "
                       "chunked pure-PyTorch oracle (the formulas of adder_cuda/test_cuda.py:18-22,35-41,57-60 and "
                       "adder.py:78 on the unfolded (K, L*N) matrix), median of 3 runs each, all intra-op threads",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-graph", action="store_true", help="time the eager step instead of the captured HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-layers", action="store_true", help="skip the per-layer table")
    ap.add_argument("--no-other", action="store_true",
                    help="skip the other model configurations (VGG-small bs128, ResNet-50 bs64, stock-module ResNet-20)")
    ap.add_argument("--roofline-only", action="store_true",
                    help="launch only the dominant kernel (and one 256 MiB device copy as a counter yardstick); "
                         "meant to run under rocprofv3 --pmc / --kernel-trace")
    ap.add_argument("--layers-only", action="store_true",
                    help="run only the per-layer table (7 ResNet-20 layer shapes x forward / grad_X / grad_W); "
                         "meant to run under rocprofv3 --pmc / --kernel-trace")
    ap.add_argument("--model", choices=sorted(MODELS), default="resnet20",
                    help="resnet20 (default) is the benchmark; vgg_small (batch 128) and resnet50 (batch 64, 224x224) "
                         "time the training step of the reference's two other model configurations and print a "
                         "shorter line")
    ap.add_argument("--stock-modules", action="store_true",
                    help="with --model vgg_small / resnet50 / densenet_cifar: build the network from stock "
                         "nn.BatchNorm2d / ReLU modules as the reference's model files do (only the adder layers differ)")
    ap.add_argument("--layer-set", choices=sorted(LAYER_SETS) + ["col"], default="resnet20",
                    help="with --layers-only: the adder layers of ResNet-20 (batch 256), the VGG-small stack "
                         "(batch 128), ResNet-50 at 224x224 (batch 64), or col: the reference extension's four "
                         "column-matrix entry points (adder_cuda.ADDER_*) at two shapes")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU; --gpus must be 1 (every box here has a single MI355X)")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.roofline_only:
        src = torch.empty(64 << 20, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)            # 256 MiB read + 256 MiB written per launch
        torch.cuda.synchronize()
        print(json.dumps({"roofline": dominant_kernel(dev, args.steps), "copy_bytes_each_way": src.numel() * 4}))
        return

    if args.layers_only and args.layer_set == "col":
        print(json.dumps({"layer_set": "col", "layers": bench_col(dev, iters=max(3, min(args.steps, 20)))}))
        return

    if args.layers_only:
        rows = bench_layers(dev, warmup=2, iters=max(3, min(args.steps, 20)), which=args.layer_set)
        print(json.dumps({"layer_set": args.layer_set, "batch": LAYER_SETS[args.layer_set][0], "layers": rows,
                          **layer_set_summary(rows)}))
        return

    gate = None if args.no_cpu else parity_gate(dev)   # (needs the oracle, like the CPU leg)
    fused = not args.stock_modules
    ms, mode, graph_check = time_training(dev, args.model, fused, args.steps, args.warmup, use_graph=not args.no_graph,
                                          replays=4 if args.model == "resnet20" else 2)

    if args.model != "resnet20" or not fused:
        batch, size, classes = MODELS[args.model]
        print(json.dumps({
            "metric": f"{args.model} AdderNet train ms/batch (bs{batch})", "value": round(ms, 3), "unit": "ms/batch",
            "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 3),
            "higher_is_better": False, "dtype": "f32", "data": "synthetic",
            "config": {"workload": f"{args.model} AdderNet, batch {batch}, 3x{size}x{size}, {classes} classes, SGD "
                                   "momentum 0.9 lr 0.1 wd 5e-4, adaptive eta 0.1, fwd+bwd+optimizer",
                       "step_mode": mode,
                       "modules": "fused BatchNorm+ReLU kernels" if fused else "stock nn.BatchNorm2d / ReLU"},
            "images_per_s": round(batch / ms * 1e3, 1), "graph_check": graph_check}))
        return

    out = {
        "metric": "ResNet-20 AdderNet train ms/batch (bs256)", "value": round(ms, 3), "unit": "ms/batch",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 3),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "ResNet-20 AdderNet, batch 256, 3x32x32, 10 classes, SGD momentum 0.9 lr 0.1 wd 5e-4, "
                               "adaptive eta 0.1, fwd+bwd+optimizer; BatchNorm / ReLU / residual add run as this "
                               "library's fused kernels (BatchNormAct2d), the BatchNorm backward passes inside the "
                               "adder backward kernels on either side of each BatchNorm (unit.py), the strided 1x1 downsample "
                               "layers inside the strided 3x3 kernels beside them (forward and grad_X), and the regular "
                               "3->16 stem convolution through the tiled forward / slab weight-gradient kernels "
                               "(StemConv2d); the same step with stock torch modules is other_configs[0]",
                   "step_mode": mode},
        "images_per_s": round(BATCH / ms * 1e3, 1),
        "roofline": dominant_kernel(dev, args.steps),
    }
    if graph_check is not None:
        out["graph_check"] = graph_check
    if gate is not None:
        out["parity_gate"] = {"bar": "rtol 1e-5 / atol 1e-4 against the float64 C oracle, worst element as a share of it",
                              "layers": gate}
    if not args.no_layers:
        rows = bench_layers(dev)
        out["layers"] = rows
        out.update(layer_set_summary(rows))
        out["col_path"] = bench_col(dev)
    if not args.no_other:
        out["other_configs"] = other_configs(dev)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
