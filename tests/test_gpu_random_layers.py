"""A seeded sweep of random layer geometries through adder2d -- forward, both gradients, the statistics epilogue and
the shortcut gradient added inside grad_X -- against the float64 C oracle.  The draw favours what selects a kernel:
1x1 / 3x3 / 5x5, strides 1-3, channel counts around the thresholds of the tiled and matrix-core kernels (48, 64,
128, multiples of 4 that are not multiples of 8, odd tails), planes of 16 to 1024 positions with widths that are
and are not multiples of 4."""
import random

import pytest
import torch

from tests.util import make_case, assert_close

pytestmark = pytest.mark.gpu


def _draw(rnd):
    k = rnd.choice([1, 1, 3, 3, 3, 5])
    s = rnd.choice([1, 1, 2, 3] if k != 3 else [1, 1, 2])
    p = {1: rnd.choice([0, 0, 1]), 3: rnd.choice([1, 1, 1, 0]), 5: 2}[k]
    Ci = rnd.choice([64, 68, 72, 76, 96, 128, 132, 136, 160, 200, 256]) if rnd.random() < 0.6 else rnd.randint(1, 40)
    Co = rnd.choice([48, 64, 65, 70, 96, 128, 130, 192, 256, 260]) if rnd.random() < 0.6 else rnd.randint(1, 40)
    H = rnd.choice([4, 5, 7, 8, 9, 14, 16, 17, 28, 32])
    W = rnd.choice([4, 5, 7, 8, 9, 14, 16, 17, 20, 28, 32])
    return rnd.randint(1, 6), Ci, H, W, Co, k, s, p


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_geometries_match_the_oracle(seed, gpu):
    from addernetcuda_amd import adder
    from oracle import c_oracle
    rnd = random.Random(seed)
    done = 0
    while done < 120:
        case = _draw(rnd)
        N, Ci, H, W, Co, k, s, p = case
        Ho, Wo = (H - k + 2 * p) // s + 1, (W - k + 2 * p) // s + 1
        if Ho <= 0 or Wo <= 0 or N * Ho * Wo * Co * Ci * k * k > 1e8:
            continue
        x, w, gy = make_case(*case, seed=seed * 1000 + done, w_init=rnd.choice(["kaiming", "normal"]))
        xg, wg = x.to(gpu).requires_grad_(True), w.to(gpu).requires_grad_(True)
        with_shortcut = rnd.random() < 0.5
        if with_shortcut:
            y, stats, shortcut = adder.adder2d_function_with_stats(xg, wg, s, p, eta=0.0, with_shortcut=True)
            gs = torch.randn(x.shape, generator=torch.Generator().manual_seed(done))
            ((y * gy.to(gpu)).sum() + (shortcut * gs.to(gpu)).sum()).backward()
        else:
            y, stats = adder.adder2d_function_with_stats(xg, wg, s, p, eta=0.0)
            y.backward(gy.to(gpu))
        torch.cuda.synchronize()
        want_y = c_oracle.conv2d_fwd(x, w, s, p)
        want_gx = c_oracle.conv2d_grad_x(gy, x, w, s, p)
        if with_shortcut:
            want_gx = want_gx + gs.double()
        assert_close(y, want_y, f"forward {case}")
        assert_close(xg.grad, want_gx, f"grad_X {case} shortcut={with_shortcut}")
        assert_close(wg.grad, c_oracle.conv2d_grad_w(gy, x, w, s, p), f"grad_W {case}")
        if stats is not None:
            tot = stats.sum(dim=1).cpu()
            assert torch.allclose(tot[:, 0], want_y.sum(dim=(0, 2, 3)), rtol=1e-5, atol=1e-3), f"sum(y) {case}"
            assert torch.allclose(tot[:, 1], (want_y * want_y).sum(dim=(0, 2, 3)), rtol=1e-5, atol=1e-2), f"sum(y*y) {case}"
        done += 1
