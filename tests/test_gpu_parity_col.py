"""Column-matrix entry points (the reference extension's literal signatures) against the oracles."""
import pytest
import torch

from tests.util import assert_close

pytestmark = pytest.mark.gpu

# (Co, K, NL): test_cuda.py:165-171 default (N=16, Co=32, Ci=32, k=3, HWo=8), then ragged sizes the
# reference aborts on (adder.cu:286-297: Co and NL must both be multiples of 16 or of 12)
CASES = [(32, 288, 1024), (16, 144, 512), (12, 36, 240), (7, 27, 101), (1, 1, 1), (33, 5, 300), (5, 130, 64),
         # many columns (two columns per lane, slabs from every workgroup) with a ragged last group; 17..32 and more
         # than 32 output channels (other kernels); tile tails on both sides of the weight-gradient product
         (16, 144, 65544), (9, 20, 70004), (24, 50, 66000), (48, 40, 2052), (64, 576, 1000), (20, 200, 4100),
         (40, 150, 66562),
         # few columns (one launch for both gradients, a workgroup per row or pair of rows of X over all columns):
         # 1, 2, 4 and 8 columns per thread, a tall matrix with an odd row count, more channels than a batch of gy
         (5, 7, 3), (17, 9, 1500), (40, 1031, 300), (64, 33, 2048), (130, 12, 700), (3, 2050, 513)]


def _data(Co, K, NL, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(K, NL, generator=g) * scale, torch.randn(Co, K, generator=g) * scale,
            torch.randn(Co, NL, generator=g))


@pytest.mark.parametrize("case", CASES, ids=str)
def test_adder_conv(case, gpu):
    from addernetcuda_amd import adder_cuda
    from oracle import c_oracle
    X, W, _ = _data(*case, scale=5.0)                    # test_cuda.py:64-66 scales by 5
    out = torch.full((case[0], case[2]), 7.0, device=gpu)   # overwritten, not accumulated
    adder_cuda.ADDER_CONV(X.to(gpu), W.to(gpu), out)
    assert_close(out, c_oracle.col_fwd(X, W), f"ADDER_CONV {case}")


@pytest.mark.parametrize("case", CASES, ids=str)
def test_adder_backward_and_its_two_halves(case, gpu):
    from addernetcuda_amd import adder_cuda
    from oracle import c_oracle
    X, W, G = _data(*case, seed=1)
    Xg, Wg, Gg = X.to(gpu), W.to(gpu), G.to(gpu)
    gw_true, gx_true = c_oracle.col_grad_w(G, X, W), c_oracle.col_grad_x(G, X, W)
    gw, gx = torch.zeros_like(Wg), torch.zeros_like(Xg)
    adder_cuda.ADDER_BACKWARD(Gg, Xg, Wg, gw, gx)
    assert_close(gw, gw_true, f"ADDER_BACKWARD grad_w {case}")
    assert_close(gx, gx_true, f"ADDER_BACKWARD grad_i {case}")
    gw2, gx2 = torch.zeros_like(Wg), torch.zeros_like(Xg)
    adder_cuda.ADDER_CONV_WEIGHT(Gg, Xg, Wg, gw2)
    adder_cuda.ADDER_CONV_INPUT(Gg, Xg, Wg, gx2)
    # (ADDER_BACKWARD may take both gradients in one pass over X: the same sums in another order for grad_w)
    assert torch.equal(gx2, gx) and torch.allclose(gw2, gw, rtol=1e-6, atol=1e-6)


def test_gradients_accumulate_into_their_outputs(gpu):
    """The reference atomically adds into caller-zeroed buffers (adder.cu:266-267); a second call doubles them."""
    from addernetcuda_amd import adder_cuda
    X, W, G = (t.to(gpu) for t in _data(16, 72, 256, seed=2))
    gw, gx = torch.zeros_like(W), torch.zeros_like(X)
    adder_cuda.ADDER_BACKWARD(G, X, W, gw, gx)
    once_w, once_x = gw.clone(), gx.clone()
    adder_cuda.ADDER_BACKWARD(G, X, W, gw, gx)
    assert torch.allclose(gw, 2 * once_w, rtol=1e-6, atol=1e-6) and torch.allclose(gx, 2 * once_x, rtol=1e-6, atol=1e-6)


def test_conv_input_follows_the_stated_maths_not_the_macro_slip(gpu):
    """adder.cu:170 expands HARDTANH un-parenthesised, so its saturated branch forgets to multiply by g.
    test_cuda.py:57-60 states the intended result; with W - X < -1 everywhere that is -sum_co g."""
    from addernetcuda_amd import adder_cuda
    G = torch.randn(4, 32, generator=torch.Generator().manual_seed(3))
    X, W = torch.full((6, 32), 9.0), torch.zeros(4, 6)
    gx = torch.zeros(6, 32, device=gpu)
    adder_cuda.ADDER_CONV_INPUT(G.to(gpu), X.to(gpu), W.to(gpu), gx)
    assert_close(gx, -G.double().sum(0, keepdim=True).expand(6, 32), "saturated grad_i")


def test_shape_and_layout_errors_raise(gpu):
    from addernetcuda_amd import adder_cuda
    X, W, G = (t.to(gpu) for t in _data(8, 18, 64))
    out = torch.zeros(8, 64, device=gpu)
    with pytest.raises(RuntimeError, match="contiguous"):
        adder_cuda.ADDER_CONV(X.t().contiguous().t(), W, out)
    with pytest.raises(RuntimeError, match="float32"):
        adder_cuda.ADDER_CONV(X.double(), W, out)
    with pytest.raises(RuntimeError, match="K="):
        adder_cuda.ADDER_CONV(X[:17].contiguous(), W, out)
    with pytest.raises(RuntimeError, match="shape"):
        adder_cuda.ADDER_CONV(X, W, torch.zeros(8, 63, device=gpu))
    with pytest.raises(RuntimeError, match="overlaps"):
        adder_cuda.ADDER_CONV_INPUT(G, X, W, X)


def test_adder_function_matches_oracle_autograd(gpu):
    """adder.apply(W_col, X_col) keeps adder.py:43-80: raw grad_X, eta-scaled grad_W."""
    from addernetcuda_amd import adder
    from oracle import adder_oracle
    X, W, G = _data(16, 144, 400, seed=4)
    Wg, Xg = W.to(gpu).requires_grad_(True), X.to(gpu).requires_grad_(True)
    out = adder.adder.apply(Wg, Xg)
    out.backward(G.to(gpu))
    Wd, Xd = W.double().requires_grad_(True), X.double().requires_grad_(True)
    ref = adder_oracle.adder.apply(Wd, Xd)
    ref.backward(G.double())
    assert_close(out, ref, "adder.apply forward")
    assert_close(Wg.grad, Wd.grad, "adder.apply grad_W (scaled)")
    assert_close(Xg.grad, Xd.grad, "adder.apply grad_X")


def test_norm_scale_entry_point(gpu):
    import ctypes
    from addernetcuda_amd._lib import lib, ptr, stream_ptr, check
    from oracle import adder_oracle
    for n, scale in ((2304, 3.0), (36864, 1e-3), (5, 1.0), (3_000_000, 0.5)):
        g = torch.randn(n, generator=torch.Generator().manual_seed(n)) * scale
        gg = g.to(gpu)
        need = ctypes.c_size_t()
        check(lib.adder_norm_scale_workspace_bytes(n, ctypes.byref(need)), "ws")
        ws = torch.empty(need.value, dtype=torch.uint8, device=gpu)
        check(lib.adder_grad_norm_scale_f32(ptr(gg), n, 0.1, 1e-12, ptr(ws), need.value, stream_ptr(gpu)), "scale")
        assert_close(gg, adder_oracle.eta_scale(g.double(), 0.1), f"norm scale n={n}", rtol=1e-5, atol=1e-6)
    z = torch.zeros(100, device=gpu)
    check(lib.adder_grad_norm_scale_f32(ptr(z), 100, 0.2, 1e-12, ptr(ws), need.value, stream_ptr(gpu)), "scale")
    assert (z == 0).all()
