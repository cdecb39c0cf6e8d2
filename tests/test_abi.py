"""The C-ABI library loads, exports every symbol the header declares, and rejects bad
arguments before touching the GPU (so all of this runs on a machine without one)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "addernet_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"ADDER_API\s+(?:const\s+)?\w+\s*\*?\s*(adder_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for must in ("adder_conv2d_fwd_f32", "adder_conv2d_bwd_f32", "adder_conv2d_bwd_workspace_bytes",
                 "adder_col_fwd_f32", "adder_col_bwd_f32", "adder_col_gradw_f32", "adder_col_gradx_f32",
                 "adder_grad_norm_scale_f32", "adder_strerror"):
        assert must in names
    assert len(names) >= 14


def test_library_exports_every_declared_symbol():
    from addernetcuda_amd import _lib
    assert os.path.exists(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(_lib.lib, name), f"{name} is declared in the header but not exported"
        assert name in _lib.EXPORTED, f"{name} has no ctypes signature in _lib.py"


def test_status_strings_and_version():
    from addernetcuda_amd._lib import lib
    assert lib.adder_abi_version() == 6
    assert lib.adder_strerror(0) == b"ok"
    seen = {lib.adder_strerror(c) for c in range(-7, 1)}
    assert len(seen) == 8 and b"unknown status" not in seen
    assert lib.adder_strerror(-99) == b"unknown status"


@pytest.mark.parametrize("h,k,p,s,want", [(32, 3, 1, 1, 32), (32, 3, 1, 2, 16), (32, 1, 0, 2, 16), (7, 3, 1, 2, 4),
                                           (11, 5, 2, 3, 4), (5, 3, 0, 1, 3), (2, 3, 0, 1, 0), (0, 3, 1, 1, 0)])
def test_out_dim_follows_the_reference_formula(h, k, p, s, want):
    from addernetcuda_amd._lib import lib
    assert lib.adder_out_dim(h, k, p, s) == want
    if want > 0:
        assert want == int((h - k + 2 * p) / s + 1)      # adder.py:26-31


def test_forward_rejects_bad_arguments_without_a_gpu():
    from addernetcuda_amd._lib import lib
    P = ctypes.c_void_p
    ok = (P(4096), P(8192), P(1 << 20))
    assert lib.adder_conv2d_fwd_f32(None, ok[1], ok[2], 1, 1, 4, 4, 1, 3, 3, 1, 1, None) == -1
    assert lib.adder_conv2d_fwd_f32(ok[0], ok[1], None, 1, 1, 4, 4, 1, 3, 3, 1, 1, None) == -1
    assert lib.adder_conv2d_fwd_f32(*ok, 0, 1, 4, 4, 1, 3, 3, 1, 1, None) == -2      # N = 0
    assert lib.adder_conv2d_fwd_f32(*ok, 1, 1, 4, 4, 1, 3, 3, 0, 1, None) == -2      # stride 0
    assert lib.adder_conv2d_fwd_f32(*ok, 1, 1, 4, 4, 1, 3, 3, 1, -1, None) == -2     # negative padding
    assert lib.adder_conv2d_fwd_f32(*ok, 1, 1, 2, 2, 1, 5, 5, 1, 0, None) == -2      # kernel larger than input
    assert lib.adder_conv2d_fwd_f32(*ok, 1 << 20, 64, 64, 64, 1, 3, 3, 1, 1, None) == -3   # > 2^31-1 elements
    assert lib.adder_conv2d_fwd_f32(P(4096), P(8192), P(4100), 1, 1, 4, 4, 1, 3, 3, 1, 1, None) == -6  # y overlaps x


def test_backward_rejects_bad_arguments_without_a_gpu():
    from addernetcuda_amd._lib import lib
    P = ctypes.c_void_p
    dims = (2, 4, 8, 8, 4, 3, 3, 1, 1)
    need = ctypes.c_size_t()
    assert lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)) == 0 and need.value >= 256
    assert lib.adder_conv2d_bwd_workspace_bytes(*dims, None) == -1
    gy, x, w, gx, gw, ws = (P(a << 20) for a in range(1, 7))
    call = lib.adder_conv2d_bwd_f32
    assert call(None, x, w, gx, gw, 0.2, ws, need.value, *dims, None) == -1
    assert call(gy, x, w, None, None, 0.2, ws, need.value, *dims, None) == -1        # nothing to compute
    assert call(gy, x, w, gx, gw, -1.0, ws, need.value, *dims, None) == -2           # negative eta
    assert call(gy, x, w, gx, gw, float("nan"), ws, need.value, *dims, None) == -2
    assert call(gy, x, w, gx, gw, 0.2, None, 0, *dims, None) == -4                   # grad_w needs scratch
    assert call(gy, x, w, gx, gw, 0.2, ws, need.value - 1, *dims, None) == -4
    assert call(gy, x, w, gx, gw, 0.2, P((6 << 20) + 8), need.value, *dims, None) == -4   # misaligned scratch
    assert call(gy, x, w, x, gw, 0.2, ws, need.value, *dims, None) == -6             # gx aliases x
    assert call(gy, x, w, gx, gw, 0.2, gw, need.value, *dims, None) == -6            # scratch aliases gw


def test_column_entry_points_reject_bad_arguments_without_a_gpu():
    from addernetcuda_amd._lib import lib
    P = ctypes.c_void_p
    a, b, c, d, e = (P(k << 24) for k in range(1, 6))
    assert lib.adder_col_fwd_f32(a, b, None, 9, 16, 4, None) == -1
    assert lib.adder_col_fwd_f32(a, b, c, 0, 16, 4, None) == -2
    assert lib.adder_col_fwd_f32(a, b, c, 9, 1 << 40, 4, None) == -3
    assert lib.adder_col_fwd_f32(a, b, a, 9, 16, 4, None) == -6
    assert lib.adder_col_bwd_f32(a, b, c, d, None, 9, 16, 4, None, 0, None) == -1
    assert lib.adder_col_gradw_f32(a, b, c, c, 9, 16, 4, None, 0, None) == -6
    assert lib.adder_col_gradx_f32(a, b, c, b, 9, 16, 4, None) == -6
    n = ctypes.c_size_t(123)
    assert lib.adder_col_bwd_workspace_bytes(9, 16, 4, ctypes.byref(n)) == 0
    assert lib.adder_grad_norm_scale_f32(None, 10, 0.2, 1e-12, a, 1 << 20, None) == -1
    assert lib.adder_grad_norm_scale_f32(a, 0, 0.2, 1e-12, b, 1 << 20, None) == -2
    assert lib.adder_grad_norm_scale_f32(a, 10, 0.2, 0.0, b, 1 << 20, None) == -2    # eps must be positive
    assert lib.adder_grad_norm_scale_f32(a, 10, 0.2, 1e-12, None, 0, None) == -4


def test_workspace_is_large_enough_for_the_partials_of_big_layers():
    from addernetcuda_amd._lib import lib
    need = ctypes.c_size_t()
    for dims in [(256, 16, 32, 32, 16, 3, 3, 1, 1), (256, 64, 8, 8, 64, 3, 3, 1, 1), (128, 512, 8, 8, 512, 3, 3, 1, 1),
                 (64, 256, 56, 56, 64, 1, 1, 1, 0)]:
        assert lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)) == 0
        assert need.value % 256 == 0 and need.value < (2 << 30)


def test_statistics_variants_validate_without_a_gpu():
    """adder_conv2d_fwd_stats_* / adder_bn_act_fwd_stats_f32: slot counts are a host-side function of the
    dimensions; bad arguments are refused before any HIP call."""
    from addernetcuda_amd._lib import lib
    slots = ctypes.c_int(-1)
    dims32 = (256, 16, 32, 32, 16, 3, 3, 1, 1)
    assert lib.adder_conv2d_fwd_stats_slots(*dims32, ctypes.byref(slots)) == 0 and slots.value > 0
    n32 = slots.value
    assert lib.adder_conv2d_fwd_stats_slots(128, 16, 32, 32, 16, 3, 3, 1, 1, ctypes.byref(slots)) == 0
    assert slots.value * 2 == n32                                  # slots follow the number of position waves
    for k, s, p in ((1, 1, 0), (1, 2, 0)):
        assert lib.adder_conv2d_fwd_stats_slots(4, 8, 16, 16, 8, k, k, s, p, ctypes.byref(slots)) == 0
        assert slots.value > 0                                     # the 1x1 kernels have the epilogue too
    for k, s, p in ((5, 1, 2), (3, 3, 1), (1, 3, 0)):
        assert lib.adder_conv2d_fwd_stats_slots(4, 8, 16, 16, 8, k, k, s, p, ctypes.byref(slots)) == 0
        assert slots.value == 0                                    # no statistics epilogue for these kernels
    assert lib.adder_conv2d_fwd_stats_slots(*dims32, None) == -1
    fake = ctypes.c_void_p(4096)
    assert lib.adder_conv2d_fwd_stats_f32(fake, fake, fake, None, n32, *dims32, None) == -1
    assert lib.adder_conv2d_fwd_stats_f32(fake, fake, ctypes.c_void_p(1 << 40), ctypes.c_void_p(1 << 41), n32 + 1,
                                          *dims32, None) == -2     # slot count must be the one reported
    assert lib.adder_conv2d_fwd_stats_f32(fake, fake, ctypes.c_void_p(1 << 40), ctypes.c_void_p(1 << 41), 4,
                                          4, 8, 16, 16, 8, 5, 5, 1, 2, None) == -7
    bn = lib.adder_bn_act_fwd_stats_f32
    args = [fake] * 5 + [None] + [fake] * 5 + [0.1, 1e-5, 1, 4, 8, 64]
    assert bn(*args, None, 4, None) == -1
    assert bn(*args, fake, 0, None) == -2


def test_relu_mask_is_offered_for_whole_word_planes_only():
    """adder_bn_act_mask_words: one bit per element when H*W is a multiple of 32, otherwise no mask; a mask
    passed for such a shape, or without ReLU, is refused before any HIP call."""
    from addernetcuda_amd._lib import lib
    words = ctypes.c_size_t(99)
    assert lib.adder_bn_act_mask_words(256, 16, 1024, ctypes.byref(words)) == 0 and words.value == 256 * 16 * 32
    assert lib.adder_bn_act_mask_words(4, 8, 64, ctypes.byref(words)) == 0 and words.value == 4 * 8 * 2
    assert lib.adder_bn_act_mask_words(4, 8, 49, ctypes.byref(words)) == 0 and words.value == 0
    assert lib.adder_bn_act_mask_words(4, 8, 64, None) == -1
    fake = ctypes.c_void_p(4096)
    ws = ctypes.c_void_p(1 << 20)
    fwd_args = [fake] * 11 + [0.1, 1e-5]
    assert lib.adder_bn_act_fwd_f32(*fwd_args, 1, 4, 8, 49, ws, 1 << 20, None) == -7    # no mask for 7x7 planes
    assert lib.adder_bn_act_fwd_f32(*fwd_args, 0, 4, 8, 64, ws, 1 << 20, None) == -7    # no mask without ReLU
    bwd_args = [fake] * 11
    assert lib.adder_bn_act_bwd_f32(*bwd_args, 1, 4, 8, 49, ws, 1 << 20, None) == -7
    no_y_no_mask = [fake, None, None] + [fake] * 8
    assert lib.adder_bn_act_bwd_f32(*no_y_no_mask, 1, 4, 8, 64, ws, 1 << 20, None) == -1


def test_staged_grad_w_and_batched_scaling_validate_without_a_gpu():
    """The entry points that finish many layers at once refuse bad arguments before any HIP call."""
    from addernetcuda_amd._lib import lib, GradWStage
    fake = ctypes.c_void_p(1 << 20)
    need = ctypes.c_size_t(0)
    # batched scaling
    assert lib.adder_norm_scale_batched_workspace_bytes(20, ctypes.byref(need)) == 0 and need.value > 0
    assert lib.adder_norm_scale_batched_workspace_bytes(65, ctypes.byref(need)) == -2
    ptrs = (ctypes.c_void_p * 2)(4096, 8192)
    sizes = (ctypes.c_long * 2)(100, 0)
    etas = (ctypes.c_float * 2)(0.1, 0.1)
    assert lib.adder_grad_norm_scale_batched_f32(2, ptrs, sizes, etas, 1e-12, fake, 1 << 20, None) == -2   # n = 0
    assert lib.adder_grad_norm_scale_batched_f32(2, None, sizes, etas, 1e-12, fake, 1 << 20, None) == -1
    # staged grad_W
    stage = GradWStage()
    dims = (4, 16, 8, 8, 16, 3, 3, 1, 1)
    assert lib.adder_conv2d_grad_w_staged_f32(fake, fake, fake, None, 0.1, fake, 1 << 30, *dims, ctypes.byref(stage),
                                              None) == -1
    assert lib.adder_conv2d_grad_w_staged_f32(fake, fake, fake, ctypes.c_void_p(1 << 40), 0.1, fake, 16, *dims,
                                              ctypes.byref(stage), None) == -4                              # workspace
    stages = (GradWStage * 1)(GradWStage(4096, 4096, 4096, 4096, 0, 16, 144, 1, 0.1))
    assert lib.adder_grad_w_finish_workspace_bytes(1, stages, ctypes.byref(need)) == -2                    # slots = 0
    stages[0].slots = 8
    # (one double per workgroup of the finish, which covers at most 64 of the 16 * 144 outputs)
    assert lib.adder_grad_w_finish_workspace_bytes(1, stages, ctypes.byref(need)) == 0 and need.value >= 16 * 144 // 64 * 8
    assert lib.adder_grad_w_finish_f32(33, stages, fake, 1 << 20, None) == -2
    assert lib.adder_grad_w_finish_f32(1, stages, fake, 16, None) == -4


def test_bn_linked_backward_checks_every_link_field_for_aliasing_without_a_gpu():
    """adder_conv2d_bwd_bn_f32: each read-only field of adder_bn_links (the BatchNorm's weight and bias, the side
    layer's gradient and weights as well) against each output, before any HIP call."""
    from addernetcuda_amd._lib import lib, BnLinks, ADDER_ERR_ALIAS
    P = ctypes.c_void_p
    dims = (4, 16, 16, 16, 32, 3, 3, 2, 1)     # a strided 3x3 layer: the side fields apply
    slots = ctypes.c_int()
    assert lib.adder_conv2d_bwd_bn_slots(*dims, ctypes.byref(slots)) == 0 and slots.value > 0
    need = ctypes.c_size_t()
    assert lib.adder_conv2d_bwd_workspace_bytes(*dims, ctypes.byref(need)) == 0
    MB = 1 << 20
    a = {n: (i + 1) * 16 * MB for i, n in enumerate(
        ("gy", "x", "w", "gx", "gw", "ws", "in_x", "mean", "rstd", "part", "gamma", "beta", "side_gy", "side_w"))}

    def call(**over):
        v = dict(a, **over)
        links = BnLinks(None, None, None, v["in_x"], v["mean"], v["rstd"], v["part"], slots.value, 1, v["gamma"], v["beta"],
                        v["side_gy"], v["side_w"])
        return lib.adder_conv2d_bwd_bn_f32(P(v["gy"]), P(v["x"]), P(v["w"]), None, P(v["gx"]), P(v["gw"]), 0.1, P(v["ws"]),
                                           need.value, *dims, ctypes.byref(links), None)

    # (never called with all-valid arguments: the addresses are made up, and on a machine with a GPU that would launch)
    for field in ("gamma", "beta", "side_gy", "side_w", "mean", "rstd", "in_x"):
        for out in ("gx", "gw", "part", "ws"):
            assert call(**{field: a[out] + 64}) == ADDER_ERR_ALIAS, (field, out)
