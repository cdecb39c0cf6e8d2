"""Pins for the CPU oracles (oracle/adder_oracle.py, oracle/adder_oracle.c).

The reference has no golden vectors, so every oracle function is pinned by
things its formula does not restate: a library routine it must reduce to, a
closed form, an invariant, brute-force loops, exact integer fixtures, and the
agreement of two restatements that share no code (unfold-based torch vs
direct-index C).  A dropped term, a wrong sign, a transposed operand or a wrong
im2col order fails at least one of them.
"""
import json
import math
import os

import pytest
import torch
import torch.nn.functional as F

from oracle import adder_oracle as O
from oracle import c_oracle as C

D = torch.float64
HERE = os.path.dirname(os.path.abspath(__file__))


def rnd(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=D) * scale


# ------------------------------------------------------------------ forward
def test_col_forward_is_negative_l1_cdist():
    W, X = rnd(7, 30, seed=1), rnd(30, 50, seed=2)
    assert torch.allclose(O.col_forward(X, W), -torch.cdist(W, X.t(), p=1), atol=1e-12)


def test_col_forward_brute_force():
    W, X = rnd(3, 5, seed=3), rnd(5, 4, seed=4)
    out = O.col_forward(X, W)
    for co in range(3):
        for nl in range(4):
            assert out[co, nl].item() == pytest.approx(-sum(abs(W[co, k] - X[k, nl]).item() for k in range(5)), abs=1e-12)


@pytest.mark.parametrize("s,p,k", [(1, 1, 3), (2, 1, 3), (1, 0, 3), (2, 0, 1), (3, 2, 5)])
def test_forward_zero_weight_is_box_filter_of_abs_x(s, p, k):
    x = rnd(2, 3, 9, 8, seed=5)
    w = torch.zeros(4, 3, k, k, dtype=D)
    want = -F.conv2d(x.abs(), torch.ones(4, 3, k, k, dtype=D), stride=s, padding=p)
    assert torch.allclose(O.conv2d_forward(x, w, s, p), want, atol=1e-12)
    assert torch.allclose(C.conv2d_fwd(x.float(), w.float(), s, p), -F.conv2d(x.float().double().abs(), torch.ones(4, 3, k, k, dtype=D), stride=s, padding=p), atol=1e-12)


def test_forward_zero_input_counts_padding_taps():
    """x = 0 everywhere: every tap, padded or not, contributes |w|, so borders equal the interior."""
    w = rnd(4, 3, 3, 3, seed=6)
    y = O.conv2d_forward(torch.zeros(2, 3, 6, 7, dtype=D), w, 1, 1)
    want = -w.abs().sum(dim=(1, 2, 3))
    assert torch.allclose(y, want.view(1, 4, 1, 1).expand_as(y), atol=1e-12)
    yc = C.conv2d_fwd(torch.zeros(2, 3, 6, 7), w.float(), 1, 1)
    assert torch.allclose(yc, (-w.float().double().abs().sum(dim=(1, 2, 3))).view(1, 4, 1, 1).expand_as(yc), atol=1e-12)


def test_forward_nonpositive_and_permutation_invariant():
    W, X = rnd(5, 12, seed=7), rnd(12, 9, seed=8)
    out = O.col_forward(X, W)
    assert (out <= 0).all()
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(9))
    assert torch.allclose(O.col_forward(X[perm], W[:, perm]), out, atol=1e-12)


def test_forward_translation_invariant_without_padding():
    x, w = rnd(1, 2, 6, 6, seed=10), rnd(3, 2, 3, 3, seed=11)
    assert torch.allclose(O.conv2d_forward(x + 2.5, w + 2.5, 1, 0), O.conv2d_forward(x, w, 1, 0), atol=1e-12)
    # with padding the zero taps do not move, so the same shift must change the border
    assert not torch.allclose(O.conv2d_forward(x + 2.5, w + 2.5, 1, 1), O.conv2d_forward(x, w, 1, 1), atol=1e-6)


# ------------------------------------------------------------------ layout
@pytest.mark.parametrize("s,p,k,H,W", [(1, 1, 3, 5, 6), (2, 1, 3, 7, 8), (2, 0, 1, 6, 6), (3, 2, 5, 11, 9)])
def test_im2col_matches_per_sample_unfold_and_column_order(s, p, k, H, W):
    x = rnd(3, 2, H, W, seed=12)
    X_col, Ho, Wo = O.im2col(x, k, s, p)
    assert (Ho, Wo) == ((H - k + 2 * p) // s + 1, (W - k + 2 * p) // s + 1)
    per_sample = F.unfold(x, k, padding=p, stride=s)          # (N, K, L)
    N, K, L = per_sample.shape
    assert X_col.shape == (K, L * N)
    for n in range(N):
        assert torch.equal(X_col.view(K, L, N)[:, :, n], per_sample[n])   # column index = l*N + n
    assert C.out_dim(H, k, p, s) == Ho and C.out_dim(W, k, p, s) == Wo


def test_col2im_is_fold_and_skips_unsampled_pixels():
    x_shape = (2, 3, 6, 6)
    gcol = rnd(3, 9 * 2, seed=13)                       # k=1, s=2, p=0 -> K=3, L=9
    gx = O.col2im(gcol, x_shape, 1, 2, 0)
    assert (gx[:, :, 1::2, :] == 0).all() and (gx[:, :, :, 1::2] == 0).all()
    g = gcol.view(3, 9, 2).permute(2, 0, 1)
    assert torch.equal(gx[:, :, ::2, ::2].reshape(2, 3, 9), g)


# ------------------------------------------------------------------ grad_W
def test_col_grad_w_gemm_identity():
    X, W, G = rnd(20, 33, seed=14), rnd(6, 20, seed=15), rnd(6, 33, seed=16)
    want = G @ X.t() - W * G.sum(1, keepdim=True)
    assert torch.allclose(O.col_grad_w(X, W, G), want, atol=1e-10)


@pytest.mark.parametrize("s,p,k", [(1, 1, 3), (2, 1, 3), (2, 0, 1)])
def test_grad_w_first_term_is_conv_weight_gradient(s, p, k):
    x, w = rnd(2, 3, 8, 8, seed=17), rnd(4, 3, k, k, seed=18)
    gy = rnd(*O.conv2d_forward(x, w, s, p).shape, seed=19)
    _, gw, _ = O.conv2d_backward(gy, x, w, s, p, eta=0)
    lib = torch.nn.grad.conv2d_weight(x, w.shape, gy, stride=s, padding=p)
    want = lib - w * gy.sum(dim=(0, 2, 3)).view(-1, 1, 1, 1)
    assert torch.allclose(gw, want, atol=1e-10)
    assert torch.allclose(C.conv2d_grad_w(gy.float(), x.float(), w.float(), s, p),
                          torch.nn.grad.conv2d_weight(x.float().double(), w.shape, gy.float().double(), stride=s, padding=p)
                          - w.float().double() * gy.float().double().sum(dim=(0, 2, 3)).view(-1, 1, 1, 1), atol=1e-10)


# ------------------------------------------------------------------ grad_X
def test_col_grad_x_unsaturated_is_linear():
    X, W = rnd(10, 21, seed=20).clamp(-2, 2) * 0.2, rnd(5, 10, seed=21).clamp(-2, 2) * 0.2   # |W - X| < 1
    assert (W.unsqueeze(2) - X.unsqueeze(0)).abs().max() < 1
    G = rnd(5, 21, seed=22)
    want = W.t() @ G - X * G.sum(0, keepdim=True)
    assert torch.allclose(O.col_grad_x(X, W, G), want, atol=1e-12)


def test_col_grad_x_saturated_both_ways_and_boundary():
    G = rnd(5, 21, seed=23)
    W = rnd(5, 10, seed=24, scale=0.1)
    hi = torch.full((10, 21), 5.0, dtype=D)
    assert torch.allclose(O.col_grad_x(hi, W, G), -G.sum(0, keepdim=True).expand(10, 21), atol=1e-12)
    assert torch.allclose(O.col_grad_x(-hi, W, G), G.sum(0, keepdim=True).expand(10, 21), atol=1e-12)
    # exactly at the clamp boundary the slope is still the identity: W - X = +-1 -> +-1
    Wb = torch.zeros(1, 1, dtype=D)
    assert O.col_grad_x(torch.tensor([[1.0]], dtype=D), Wb, torch.tensor([[3.0]], dtype=D)).item() == -3.0
    assert O.col_grad_x(torch.tensor([[-1.0]], dtype=D), Wb, torch.tensor([[3.0]], dtype=D)).item() == 3.0


@pytest.mark.parametrize("s,p,k", [(1, 1, 3), (2, 1, 3), (2, 0, 1)])
def test_grad_x_nchw_regimes_are_transposed_convolutions(s, p, k):
    w = rnd(4, 3, k, k, seed=25).clamp(-2, 2) * 0.2
    x = rnd(2, 3, 8, 8, seed=26).clamp(-2, 2) * 0.2
    gy = rnd(*O.conv2d_forward(x, w, s, p).shape, seed=27)
    opad = (8 + 2 * p - k) % s
    ones = torch.ones(4, 3, k, k, dtype=D)
    gx, _, _ = O.conv2d_backward(gy, x, w, s, p, eta=0)
    want = F.conv_transpose2d(gy, w, stride=s, padding=p, output_padding=opad) \
        - x * F.conv_transpose2d(gy, ones, stride=s, padding=p, output_padding=opad)
    assert torch.allclose(gx, want, atol=1e-10)
    gx_sat, _, _ = O.conv2d_backward(gy, x + 10, w, s, p, eta=0)
    assert torch.allclose(gx_sat, -F.conv_transpose2d(gy, ones, stride=s, padding=p, output_padding=opad), atol=1e-10)
    assert torch.allclose(C.conv2d_grad_x(gy.float(), (x + 10).float(), w.float(), s, p),
                          -F.conv_transpose2d(gy.float().double(), ones, stride=s, padding=p, output_padding=opad), atol=1e-10)


def test_backward_is_the_surrogate_not_the_true_derivative():
    """d/dW of -|W - X| is sign(X - W); the reference back-propagates X - W instead (adder.py:70)."""
    X, W, G = rnd(4, 6, seed=28, scale=3), rnd(2, 4, seed=29, scale=3), torch.ones(2, 6, dtype=D)
    true = torch.sign(X.unsqueeze(0) - W.unsqueeze(2)).sum(2)
    assert not torch.allclose(O.col_grad_w(X, W, G), true)


# ------------------------------------------------------------------ eta scaling
def test_eta_scale_invariants():
    g = rnd(8, 27, seed=30, scale=7)
    for eta in (0.2, 0.1):
        out = O.eta_scale(g, eta)
        assert out.norm().item() == pytest.approx(eta * math.sqrt(g.numel()), rel=1e-12)
        assert torch.allclose(O.eta_scale(g * 123.0, eta), out, atol=1e-12)          # scale of G drops out
        assert torch.allclose(out / out.norm(), g / g.norm(), atol=1e-12)           # direction kept
        assert torch.allclose(C.eta_scale(g, eta), out, atol=1e-12)
    assert (O.eta_scale(torch.zeros(3, 5, dtype=D)) == 0).all()                      # 0 / 1e-12 = 0
    assert O.DEFAULT_ETA == 0.2                                                      # adder.py:78 divides by 5


# ------------------------------------------------------------------ two restatements, no shared code
SHAPES = [(2, 3, 5, 6, 4, 3, 1, 1), (2, 3, 7, 8, 4, 3, 2, 1), (1, 2, 5, 5, 3, 3, 1, 0), (2, 4, 6, 6, 5, 1, 2, 0),
          (1, 2, 11, 9, 3, 5, 3, 2), (1, 1, 1, 1, 1, 1, 1, 0), (2, 2, 9, 9, 3, 7, 2, 3)]


@pytest.mark.parametrize("shape", SHAPES, ids=str)
def test_c_oracle_agrees_with_torch_oracle(shape):
    N, Ci, H, W, Co, k, s, p = shape
    x, w = rnd(N, Ci, H, W, seed=31).float(), rnd(Co, Ci, k, k, seed=32).float()
    y = O.conv2d_forward(x.double(), w.double(), s, p)
    gy = rnd(*y.shape, seed=33).float()
    gx, gw, gws = O.conv2d_backward(gy.double(), x.double(), w.double(), s, p, eta=0.2)
    assert torch.allclose(C.conv2d_fwd(x, w, s, p), y, atol=1e-12)
    assert torch.allclose(C.conv2d_grad_x(gy, x, w, s, p), gx, atol=1e-12)
    assert torch.allclose(C.conv2d_grad_w(gy, x, w, s, p), gw, atol=1e-11)
    assert torch.allclose(C.eta_scale(C.conv2d_grad_w(gy, x, w, s, p), 0.2), gws, atol=1e-12)


def test_c_col_entry_points_agree_with_torch_oracle():
    X, W, G = rnd(27, 40, seed=34).float(), rnd(6, 27, seed=35).float(), rnd(6, 40, seed=36).float()
    assert torch.allclose(C.col_fwd(X, W), O.col_forward(X.double(), W.double()), atol=1e-12)
    assert torch.allclose(C.col_grad_w(G, X, W), O.col_grad_w(X.double(), W.double(), G.double()), atol=1e-11)
    assert torch.allclose(C.col_grad_x(G, X, W), O.col_grad_x(X.double(), W.double(), G.double()), atol=1e-12)


# ------------------------------------------------------------------ exact integer fixtures
def _fixtures():
    with open(os.path.join(HERE, "golden", "adder_small_int.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("fx", _fixtures(), ids=lambda f: str(f["dims"]))
def test_oracles_reproduce_integer_fixtures_exactly(fx):
    N, Ci, H, W, Co, k, s, p = fx["dims"]
    x, w, gy = (torch.tensor(fx[n], dtype=torch.float32) for n in ("x", "w", "gy"))
    y, gw, gx = (torch.tensor(fx[n], dtype=D) for n in ("y", "gw", "gx"))
    assert torch.equal(O.conv2d_forward(x, w, s, p).double(), y)          # fp32 is exact on small integers
    ogx, ogw, _ = O.conv2d_backward(gy, x, w, s, p, eta=0)
    assert torch.equal(ogx.double(), gx) and torch.equal(ogw.double(), gw)
    assert torch.equal(C.conv2d_fwd(x, w, s, p), y)
    assert torch.equal(C.conv2d_grad_w(gy, x, w, s, p), gw)
    assert torch.equal(C.conv2d_grad_x(gy, x, w, s, p), gx)


# ------------------------------------------------------------------ autograd wiring and module
def test_oracle_autograd_function_and_module():
    torch.manual_seed(0)
    m = O.adder2d(3, 4, 3, stride=2, padding=1, bias=True)
    assert set(dict(m.named_parameters())) == {"adder", "b"}
    assert m.adder.shape == (4, 3, 3, 3) and m.b.shape == (4,)
    x = torch.randn(2, 3, 7, 7, requires_grad=True)
    y = m(x)
    gy = torch.randn_like(y)
    y.backward(gy)
    gx, _, gws = O.conv2d_backward(gy, x.detach(), m.adder.detach(), 2, 1, eta=0.2)
    assert torch.allclose(x.grad, gx) and torch.allclose(m.adder.grad, gws)
    assert torch.allclose(m.b.grad, gy.sum(dim=(0, 2, 3)))
    base = O.conv2d_forward(x.detach(), m.adder.detach(), 2, 1)
    assert torch.allclose(y.detach(), base + m.b.detach().view(1, -1, 1, 1))
