"""The BatchNorm backward passes folded into the adder backward kernels (adder_conv2d_bwd_bn_f32,
adder_conv2d_grad_w_staged_bn_f32, adder_bn_bwd_coef_f32 or the sums added by the grad_W kernel), through the C ABI, against the oracle's adder
backward and the textbook BatchNorm backward evaluated in float64.

Chain under test:  xp -> BatchNorm P -> (+ residual) -> ReLU -> x -> adder layer B -> y -> BatchNorm Q -> ...
  in-links  : B's grad_X kernel leaves dz = (grad_X + gx_add) * [x > 0] and P's sums of dz, dz * xhat;
  out-links : B's grad_W kernel takes dzq (the masked gradient of Q's output), y and Q's coefficients instead of
              gy, and leaves gy in memory for B's grad_X kernel.
"""
import ctypes

import pytest
import torch

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (N, Ci, H, W, Co, stride[, kernel size = 3]); 3x3 layers have pad 1, 1x1 layers pad 0
CASES = [(8, 16, 32, 32, 16, 1), (6, 16, 32, 32, 32, 2), (8, 32, 16, 16, 32, 1), (8, 32, 16, 16, 64, 2),
         (8, 64, 8, 8, 64, 1), (3, 20, 16, 16, 24, 1), (5, 12, 32, 32, 40, 1), (3, 6, 24, 40, 9, 2),
         (2, 5, 12, 20, 3, 1), (4, 8, 8, 8, 260, 1),   # the last one: the three-instruction grad_X form (2340 terms)
         # wide maps whose height is not a multiple of 16: tiles of 8 rows (24, 56) and of 4 rows x two images (20, 28;
         # three images: the last tile holds one)
         (2, 8, 24, 40, 8, 1), (3, 8, 20, 24, 12, 1), (2, 16, 56, 56, 8, 1), (3, 8, 28, 28, 8, 1),
         # 1x1 layers: planes of 196 and 784 positions, planes of 64 (few and many workgroups), 128-channel blocks
         (4, 64, 14, 14, 256, 1, 1), (2, 256, 28, 28, 64, 1, 1), (8, 64, 8, 8, 64, 1, 1), (40, 72, 8, 8, 64, 1, 1),
         (3, 128, 8, 8, 128, 1, 1), (2, 128, 14, 14, 136, 1, 1), (2, 64, 6, 6, 1100, 1, 1)]


def _geom(case):
    N, Ci, H, W, Co, s = case[:6]
    k = case[6] if len(case) > 6 else 3
    return N, Ci, H, W, Co, s, k, k // 2


def _make(case, seed):
    N, Ci, H, W, Co, s, k, pad = _geom(case)
    g = torch.Generator().manual_seed(seed)
    xp = torch.randn(N, Ci, H, W, generator=g) * 20 - 90            # an adder layer's output: large negative mean
    res = torch.randn(N, Ci, H, W, generator=g)
    gamma_p = torch.rand(Ci, generator=g) + 0.5
    beta_p = torch.randn(Ci, generator=g) * 0.3
    w = torch.randn(Co, Ci, k, k, generator=g) * 0.5
    Ho, Wo = (H - k + 2 * pad) // s + 1, (W - k + 2 * pad) // s + 1
    dzq = torch.randn(N, Co, Ho, Wo, generator=g)
    dzq = dzq * (torch.rand(dzq.shape, generator=g) > 0.4)          # a ReLU-masked gradient
    gamma_q = torch.rand(Co, generator=g) + 0.5
    gx_add = torch.randn(N, Ci, H, W, generator=g)
    return xp, res, gamma_p, beta_p, w, dzq, gamma_q, gx_add


def _stats(t):
    mean = t.mean((0, 2, 3))
    var = t.var((0, 2, 3), unbiased=False)
    return mean, 1.0 / torch.sqrt(var + 1e-5)


def _bn_input_grad(dz, x, gamma, mean, rstd):
    """dx, dgamma, dbeta of a training-mode BatchNorm from the gradient dz of its output (float64)."""
    b = lambda v: v[None, :, None, None]
    xhat = (x - b(mean)) * b(rstd)
    dbeta, dgamma = dz.sum((0, 2, 3)), (dz * xhat).sum((0, 2, 3))
    cnt = dz.numel() / dz.shape[1]
    return b(gamma * rstd) * (dz - b(dbeta) / cnt - xhat * b(dgamma) / cnt), dgamma, dbeta


@pytest.mark.parametrize("case", CASES, ids=str)
@pytest.mark.parametrize("with_add", [False, True])
@pytest.mark.parametrize("from_x", [False, True], ids=["reads_bn_input", "xhat_from_x"])
def test_fused_backward_matches_the_unfused_chain_in_float64(case, with_add, from_x, gpu):
    """``from_x``: P's output went through nothing but the ReLU, and the links carry P's weight and bias so that the
    kernel may take xhat from x; two channels are then outside what it accepts for that (a tiny and a negative
    weight: the first must read P's input after all, the second divides by a negative number)."""
    from addernetcuda_amd._lib import lib, check, ptr, stream_ptr, BnLinks, bwd_bn_slots, conv_dims, conv2d_bwd_workspace
    from oracle import adder_oracle
    N, Ci, H, W, Co, s, k, pad = _geom(case)
    xp, res, gamma_p, beta_p, w, dzq, gamma_q, gx_add = _make(case, 17 + sum(case))
    if from_x:
        res = torch.zeros_like(res)
        gamma_p[0], gamma_p[1], beta_p[0] = 1e-3, -0.7, 0.2
    dims, Ho, Wo = conv_dims((N, Ci, H, W), w.shape, s, pad)
    slots = bwd_bn_slots(dims)
    assert slots > 0

    # ---- float64 truth -------------------------------------------------------------------
    mean_p, rstd_p = _stats(xp.double())
    b = lambda v: v[None, :, None, None]
    # x as float32 would hold it (the kernels read the float32 tensor, and its sign is the ReLU gate)
    mean_p32, rstd_p32 = mean_p.float(), rstd_p.float()
    x = torch.relu((xp - b(mean_p32)) * b(rstd_p32 * gamma_p) + b(beta_p) + res)
    y = adder_oracle.conv2d_forward(x.double(), w.double(), s, pad)
    y32 = y.float()
    mean_q, rstd_q = _stats(y32.double())
    mean_q32, rstd_q32 = mean_q.float(), rstd_q.float()
    gy, dgamma_q, dbeta_q = _bn_input_grad(dzq.double(), y32.double(), gamma_q.double(), mean_q32.double(),
                                           rstd_q32.double())
    gx, gw_raw, gw_scaled = adder_oracle.conv2d_backward(gy, x.double(), w.double(), s, pad, 0.2)
    if with_add:
        gx = gx + gx_add.double()
    dz = gx * (x > 0)
    xhat_p = (xp.double() - b(mean_p32.double())) * b(rstd_p32.double())
    want_part = torch.stack([dz.sum((0, 2, 3)), (dz * xhat_p).sum((0, 2, 3))], 1)

    # ---- the library -----------------------------------------------------------------------
    d = lambda t: t.to(gpu).contiguous() if t is not None else None
    xg, wg, dzqg, y32g, xpg, addg = d(x), d(w), d(dzq), d(y32), d(xp), d(gx_add if with_add else None)
    mean_pg, rstd_pg, mean_qg, rstd_qg, gamma_qg = d(mean_p32), d(rstd_p32), d(mean_q32), d(rstd_q32), d(gamma_q)
    st = stream_ptr(gpu)
    # Q's coefficients from one slot of partial sums (what B's consumer would have left)
    xhat_q = (y32.double() - b(mean_q32.double())) * b(rstd_q32.double())
    part_q = torch.stack([dzq.double().sum((0, 2, 3)), (dzq.double() * xhat_q).sum((0, 2, 3))], 1).view(Co, 1, 2)
    part_q = part_q.float()                                         # (the slots hold float32 totals)
    part_qg = d(part_q)
    coef = torch.empty(Co, 4, device=gpu)
    dgq, dbq = torch.empty(Co, device=gpu), torch.empty(Co, device=gpu)
    check(lib.adder_bn_bwd_coef_f32(ptr(part_qg), 1, ptr(gamma_qg), ptr(mean_qg), ptr(rstd_qg), float(N * Ho * Wo),
                                    ptr(coef), ptr(dgq), ptr(dbq), Co, st), "adder_bn_bwd_coef_f32")
    assert_close(dgq, dgamma_q, "dgamma of Q", rtol=1e-5, atol=1e-3)
    assert_close(dbq, dbeta_q, "dbeta of Q", rtol=1e-5, atol=1e-3)

    part = torch.full((Ci, slots, 2), float("nan"), dtype=torch.float32, device=gpu)
    gy_out = torch.full_like(dzqg, float("nan"))
    gamma_pg, beta_pg = (d(gamma_p), d(beta_p)) if from_x else (None, None)
    links = BnLinks(ptr(y32g), ptr(coef), ptr(gy_out), ptr(xpg), ptr(mean_pg), ptr(rstd_pg), ptr(part), slots, 1,
                    ptr(gamma_pg), ptr(beta_pg))
    gxg, gwg = torch.empty_like(xg), torch.empty_like(wg)
    ws, nbytes = conv2d_bwd_workspace(dims, gpu)
    check(lib.adder_conv2d_bwd_bn_f32(ptr(dzqg), ptr(xg), ptr(wg), ptr(addg), ptr(gxg), ptr(gwg), 0.2, ptr(ws), nbytes,
                                      *dims, ctypes.byref(links), st), "adder_conv2d_bwd_bn_f32")
    torch.cuda.synchronize()
    assert_close(gy_out, gy, "gradient of y left by the grad_W kernel", rtol=1e-5, atol=1e-5)
    # grad_X inherits the rounding of gy = k * dz + ... (a float32 value of size ~1), which the plain backward gets exact
    assert_close(gxg, dz, "dz", rtol=2e-5, atol=2e-4)
    assert_close(gwg, gw_scaled, "grad_W (scaled)", rtol=2e-5, atol=2e-4)
    got_part = part.double().sum(1)
    assert torch.isfinite(part).all()
    scale = max(1.0, float(want_part.abs().max()))
    assert_close(got_part / scale, want_part / scale, "sums of dz, dz * xhat", rtol=1e-5, atol=1e-5)

    # the staged weight gradient with the same link, finished on its own
    from addernetcuda_amd._lib import GradWStage
    stage = GradWStage()
    gw2 = torch.empty_like(wg)
    gy_out2 = torch.empty_like(dzqg)
    links_w = BnLinks(ptr(y32g), ptr(coef), ptr(gy_out2), None, None, None, None, 0, 0)
    check(lib.adder_conv2d_grad_w_staged_bn_f32(ptr(dzqg), ptr(xg), ptr(wg), ptr(gw2), 0.2, ptr(ws), nbytes, *dims,
                                                ctypes.byref(links_w), ctypes.byref(stage), st),
          "adder_conv2d_grad_w_staged_bn_f32")
    arr = (GradWStage * 1)(stage)
    need = ctypes.c_size_t(0)
    check(lib.adder_grad_w_finish_workspace_bytes(1, arr, ctypes.byref(need)), "adder_grad_w_finish_workspace_bytes")
    fws = torch.empty(max(need.value, 256), dtype=torch.uint8, device=gpu)
    check(lib.adder_grad_w_finish_f32(1, arr, ptr(fws), need.value, st), "adder_grad_w_finish_f32")
    torch.cuda.synchronize()
    assert torch.equal(gw2, gwg), "staged and one-call weight gradients differ"
    assert torch.equal(gy_out2, gy_out)
    # ... and the input gradient from what it left, with the in-links alone (the order a caller that stages uses)
    links_x = BnLinks(None, None, None, ptr(xpg), ptr(mean_pg), ptr(rstd_pg), ptr(part), slots, 1, ptr(gamma_pg),
                      ptr(beta_pg))
    gx2 = torch.empty_like(xg)
    check(lib.adder_conv2d_bwd_bn_f32(ptr(gy_out2), ptr(xg), ptr(wg), ptr(addg), ptr(gx2), None, 0.0, None, 0, *dims,
                                      ctypes.byref(links_x), st), "adder_conv2d_bwd_bn_f32")
    torch.cuda.synchronize()
    assert torch.equal(gx2, gxg)

    # the same with Q's sums handed to the grad_W kernel itself (out_part) instead of ready coefficients: one slot
    # gives the very same bits; many slots the same values (an even count is read two slots at a time: less than one
    # load per lane, several rounds of loads with a tail; an odd count slot by slot)
    for S in (1, 6, 1100, 333):
        if S == 1:
            part_s = part_qg
        else:
            g = torch.Generator().manual_seed(S)
            pieces = torch.randn(Co, S, 2, generator=g, dtype=torch.float64)
            pieces[:, -1] += part_q.view(Co, 2).double() - pieces.sum(1)
            part_s = d(pieces.float())
        dg3, db3 = torch.full((Co,), float("nan"), device=gpu), torch.full((Co,), float("nan"), device=gpu)
        gy_out3, gw3, gx3 = torch.full_like(dzqg, float("nan")), torch.empty_like(wg), torch.empty_like(xg)
        part3 = torch.full((Ci, slots, 2), float("nan"), dtype=torch.float32, device=gpu)
        links3 = BnLinks(ptr(y32g), None, ptr(gy_out3), ptr(xpg), ptr(mean_pg), ptr(rstd_pg), ptr(part3), slots, 1,
                         ptr(gamma_pg), ptr(beta_pg), None, None, ptr(part_s), S, ptr(gamma_qg), ptr(mean_qg),
                         ptr(rstd_qg), ptr(dg3), ptr(db3))
        check(lib.adder_conv2d_bwd_bn_f32(ptr(dzqg), ptr(xg), ptr(wg), ptr(addg), ptr(gx3), ptr(gw3), 0.2, ptr(ws),
                                          nbytes, *dims, ctypes.byref(links3), st), "adder_conv2d_bwd_bn_f32")
        stage3 = GradWStage()
        gw4, gy_out4 = torch.empty_like(wg), torch.empty_like(dzqg)
        dg4, db4 = torch.empty(Co, device=gpu), torch.empty(Co, device=gpu)
        links4 = BnLinks(ptr(y32g), None, ptr(gy_out4), None, None, None, None, 0, 0, None, None, None, None,
                         ptr(part_s), S, ptr(gamma_qg), ptr(mean_qg), ptr(rstd_qg), ptr(dg4), ptr(db4))
        check(lib.adder_conv2d_grad_w_staged_bn_f32(ptr(dzqg), ptr(xg), ptr(wg), ptr(gw4), 0.2, ptr(ws), nbytes, *dims,
                                                    ctypes.byref(links4), ctypes.byref(stage3), st),
              "adder_conv2d_grad_w_staged_bn_f32")
        arr3 = (GradWStage * 1)(stage3)
        check(lib.adder_grad_w_finish_f32(1, arr3, ptr(fws), need.value, st), "adder_grad_w_finish_f32")
        torch.cuda.synchronize()
        assert torch.equal(gw4, gw3) and torch.equal(gy_out4, gy_out3)
        assert torch.equal(dg4, dg3) and torch.equal(db4, db3)
        if S == 1:
            assert torch.equal(dg3, dgq) and torch.equal(db3, dbq)
            assert torch.equal(gy_out3, gy_out) and torch.equal(gw3, gwg) and torch.equal(gx3, gxg)
            assert torch.equal(part3, part)
        else:
            assert_close(dg3, dgamma_q, "dgamma of Q from the grad_W kernel", rtol=1e-5, atol=1e-3)
            assert_close(db3, dbeta_q, "dbeta of Q from the grad_W kernel", rtol=1e-5, atol=1e-3)
            assert_close(gy_out3, gy, "gradient of y (sums added in the kernel)", rtol=1e-5, atol=1e-5)
            assert_close(gx3, dz, "dz (sums added in the kernel)", rtol=2e-5, atol=2e-4)
            assert_close(gw3, gw_scaled, "grad_W (sums added in the kernel)", rtol=2e-5, atol=2e-4)


@pytest.mark.parametrize("case", [(8, 16, 32, 32, 16, 1), (8, 32, 16, 16, 64, 2), (3, 20, 16, 16, 24, 1),
                                  (4, 64, 14, 14, 96, 1, 1)], ids=str)
def test_each_half_of_the_links_alone(case, gpu):
    """Only in-links (a plain gy) against the library's own unfused kernels, with and without the ReLU gate."""
    from addernetcuda_amd._lib import lib, check, ptr, stream_ptr, BnLinks, bwd_bn_slots, conv_dims, conv2d_bwd_workspace
    N, Ci, H, W, Co, s, k, pad = _geom(case)
    xp, res, gamma_p, beta_p, w, dzq, gamma_q, gx_add = _make(case, 5 + sum(case))
    dims, Ho, Wo = conv_dims((N, Ci, H, W), w.shape, s, pad)
    slots = bwd_bn_slots(dims)
    st = stream_ptr(gpu)
    d = lambda t: t.to(gpu).contiguous()
    x = torch.relu(torch.randn(N, Ci, H, W, generator=torch.Generator().manual_seed(3)))
    xg, wg, gyg, xpg = d(x), d(w), d(dzq), d(xp)
    ws, nbytes = conv2d_bwd_workspace(dims, gpu)
    gx0, gw0 = torch.empty_like(xg), torch.empty_like(wg)
    check(lib.adder_conv2d_bwd_f32(ptr(gyg), ptr(xg), ptr(wg), ptr(gx0), ptr(gw0), 0.2, ptr(ws), nbytes, *dims, st),
          "adder_conv2d_bwd_f32")
    # in-links only: same gy; the result is the plain one masked, the weight gradient is unchanged
    mean, rstd = d(torch.randn(Ci) - 90), d(torch.rand(Ci) * 0.05 + 0.02)
    part = torch.empty((Ci, slots, 2), dtype=torch.float32, device=gpu)
    links = BnLinks(None, None, None, ptr(xpg), ptr(mean), ptr(rstd), ptr(part), slots, 1)
    gx1, gw1 = torch.empty_like(xg), torch.empty_like(wg)
    check(lib.adder_conv2d_bwd_bn_f32(ptr(gyg), ptr(xg), ptr(wg), None, ptr(gx1), ptr(gw1), 0.2, ptr(ws), nbytes, *dims,
                                      ctypes.byref(links), st), "adder_conv2d_bwd_bn_f32")
    torch.cuda.synchronize()
    assert torch.equal(gx1, gx0 * (xg > 0))
    assert torch.equal(gw1, gw0)
    xhat = (xpg.double() - mean.double()[None, :, None, None]) * rstd.double()[None, :, None, None]
    want = torch.stack([gx1.double().sum((0, 2, 3)), (gx1.double() * xhat).sum((0, 2, 3))], 1)
    scale = max(1.0, float(want.abs().max()))
    assert_close(part.double().sum(1) / scale, want / scale, "partial sums", rtol=1e-5, atol=1e-5)
    # without the ReLU gate the result is the plain one
    links.in_relu = 0
    check(lib.adder_conv2d_bwd_bn_f32(ptr(gyg), ptr(xg), ptr(wg), None, ptr(gx1), None, 0.0, None, 0, *dims,
                                      ctypes.byref(links), st), "adder_conv2d_bwd_bn_f32")
    torch.cuda.synchronize()
    assert torch.equal(gx1, gx0)


def test_refusals(gpu):
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, BnLinks, bwd_bn_slots, conv_dims
    dims, _, _ = conv_dims((2, 16, 8, 8), (16, 16, 1, 1), 1, 0)
    assert bwd_bn_slots(dims) == 0                       # no fused kernels for 1x1 layers with fewer than 64 channels
    dims49, _, _ = conv_dims((2, 64, 7, 7), (64, 64, 1, 1), 1, 0)
    assert bwd_bn_slots(dims49) == 0                     # ... nor for planes that are not whole groups of four
    dims_s2, _, _ = conv_dims((2, 64, 8, 8), (64, 64, 1, 1), 2, 0)
    assert bwd_bn_slots(dims_s2) == 0                    # ... nor for strided 1x1 layers
    dims7, _, _ = conv_dims((2, 16, 7, 7), (16, 16, 3, 3), 1, 1)
    assert bwd_bn_slots(dims7) == 0                      # rows that are not whole groups of four
    t = torch.zeros(2 * 16 * 8 * 8, device=gpu)
    links = BnLinks(None, None, None, None, None, None, None, 0, 0)
    rc = lib.adder_conv2d_bwd_bn_f32(ptr(t), ptr(t), ptr(t), None, ptr(t), None, 0.0, None, 0, *dims, ctypes.byref(links),
                                     stream_ptr(gpu))
    assert rc == -7
    dims3, _, _ = conv_dims((2, 16, 8, 8), (16, 16, 3, 3), 1, 1)
    slots3 = bwd_bn_slots(dims3)
    part = torch.empty(16 * slots3 * 2, dtype=torch.float32, device=gpu)
    links = BnLinks(None, None, None, ptr(t), ptr(t), ptr(t), ptr(part), slots3, 1, ptr(t), None)   # weight, no bias
    rc = lib.adder_conv2d_bwd_bn_f32(ptr(t), ptr(t), ptr(t), None, ptr(t), None, 0.0, None, 0, *dims3, ctypes.byref(links),
                                     stream_ptr(gpu))
    assert rc == -1
    links = BnLinks(ptr(t), None, None, None, None, None, None, 0, 0)     # out_x without out_coef or out_part
    rc = lib.adder_conv2d_bwd_bn_f32(ptr(t), ptr(t), ptr(t), None, ptr(t), None, 0.0, None, 0, *dims3, ctypes.byref(links),
                                     stream_ptr(gpu))
    assert rc == -1
    links = BnLinks(ptr(t), ptr(t), None, None, None, None, None, 0, 0, None, None, None, None, ptr(part), 1, ptr(t), ptr(t),
                    ptr(t), ptr(t), ptr(t))                               # both of them
    rc = lib.adder_conv2d_bwd_bn_f32(ptr(t), ptr(t), ptr(t), None, ptr(t), None, 0.0, None, 0, *dims3, ctypes.byref(links),
                                     stream_ptr(gpu))
    assert rc == -1
    links = BnLinks(ptr(t), None, None, None, None, None, None, 0, 0, None, None, None, None, ptr(part), 1, ptr(t), ptr(t),
                    ptr(t), None, ptr(t))                                 # out_part without a place for dgamma
    rc = lib.adder_conv2d_bwd_bn_f32(ptr(t), ptr(t), ptr(t), None, ptr(t), None, 0.0, None, 0, *dims3, ctypes.byref(links),
                                     stream_ptr(gpu))
    assert rc == -1
