"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on the same
seeded inputs.  fp32 bar: max-abs/rel 1e-4 (written as rtol=atol=1e-4 below);
integer-valued inputs must match exactly."""
import json
import os

import numpy as np
import pytest

from conv_cases import REFERENCE_MATRIX, case, case_id, make_tensors, small_cases

pytestmark = pytest.mark.gpu

TOL = dict(rtol=1e-4, atol=1e-4)
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def cfg_of(orc, c):
    return orc.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])


def oracle_conv(orc, c, x, w, bias, threads=8):
    return orc.conv2d_forward(x, w, bias, cfg_of(orc, c), c["activation"], threads=threads)


@pytest.fixture(scope="module")
def gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpu_util

    return gpu_util


# ------------------------------------------------------------ implicit GEMM
@pytest.mark.parametrize("c,bhw", small_cases(), ids=case_id)
def test_gemm_reference_matrix(gpu, oracle_mod, c, bhw):
    x, w, bias = make_tensors(c, bhw, seed=99)
    print("case", case_id(c), bhw, flush=True)
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)


def test_config1_single_layer(gpu, oracle_mod):
    # [16,64,56,56] * [64,64,3,3], s1 p1, bias, fused ReLU
    c = case(3, 1, 1, 1, 64, 64, True, 1, True)
    x, w, bias = make_tensors(c, (16, 56, 56), seed=1)
    got, algo = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)
    assert (got == 0).any() and (got > 0).any()  # the ReLU really cut something


RESNET18_LAYERS = [  # (kernel, pad, stride, cin, cout, HW) -- the conv shapes of the ResNet-18 stack
    (7, 3, 2, 3, 64, 224), (3, 1, 1, 64, 64, 56), (3, 1, 2, 64, 128, 56), (1, 0, 2, 64, 128, 56), (3, 1, 1, 128, 128, 28),
    (3, 1, 2, 128, 256, 28), (1, 0, 2, 128, 256, 28), (3, 1, 1, 256, 256, 14), (3, 1, 2, 256, 512, 14),
    (1, 0, 2, 256, 512, 14), (3, 1, 1, 512, 512, 7),
]


@pytest.mark.parametrize("layer", RESNET18_LAYERS, ids=lambda l: "k%d_s%d_%dto%d_at%d" % (l[0], l[2], l[3], l[4], l[5]))
def test_resnet18_layer_shapes(gpu, oracle_mod, layer):
    k, p, s, cin, cout, hw = layer
    c = case(k, p, s, 1, cin, cout, True, 1, True)
    batch = 2 if hw > 56 else 3
    x, w, bias = make_tensors(c, (batch, hw, hw), seed=hw + cin)
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm", batch_hint=64)
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)


def test_split_k_through_workspace(gpu, oracle_mod):
    # few output tiles, long K: the launch splits K over several workgroups and reduces the
    # partial sums from the workspace; a missing workspace is a validation error
    import torch

    import dlprimitives_amd as dlp

    c = case(3, 1, 1, 1, 256, 512, True, 1, True)
    x, w, bias = make_tensors(c, (2, 7, 7), seed=4)
    want = oracle_conv(oracle_mod, c, x, w, bias)
    st = gpu.settings_of(c, x.shape)
    op = dlp.Conv2DForward.create(st, True, "relu", "gemm")
    assert op.workspace() > 0
    xd, wd, bd = gpu.dev(x), gpu.dev(w), gpu.dev(bias)
    y = torch.full(want.shape, float("nan"), device="cuda:0")
    op.enqueue(xd, wd, bd, y, torch.empty(op.workspace(), dtype=torch.uint8, device="cuda:0"), 0.0)
    torch.cuda.synchronize()
    np.testing.assert_allclose(y.cpu().numpy(), want, **TOL)
    with pytest.raises(dlp.ValidationError):
        op.enqueue(xd, wd, bd, y, None, 0.0)
    old = np.random.default_rng(0).standard_normal(want.shape).astype(np.float32)
    y = gpu.dev(old)
    op.enqueue(xd, wd, bd, y, torch.empty(op.workspace(), dtype=torch.uint8, device="cuda:0"), 0.25)
    torch.cuda.synchronize()
    np.testing.assert_allclose(y.cpu().numpy(), oracle_mod.apply_factor(want, old, 0.25), **TOL)


# Stride-1 3x3 "same" convolutions with Cin/groups % 16 == 0 and Cout/groups > 32 run the LDS-patch
# kernel, whose K stages are dealt evenly to the workgroups (stream-K): a tile is in general
# computed in pieces that meet through the workspace.  (batch, cin, cout, groups, H, W)
PATCH_SHAPES = [
    (3, 64, 64, 1, 56, 56),    # whole tiles
    (18, 64, 64, 1, 56, 56),   # more tiles than workgroups: pieces of 4-stage tiles
    (5, 128, 128, 1, 28, 28),  # 8 stages per tile, tiles cross image rows
    (7, 256, 256, 1, 14, 14),  # tiles cross images, N tail
    (5, 512, 512, 1, 7, 7),    # up to three images per tile, 32 stages per tile
    (3, 64, 128, 2, 9, 11),    # groups, odd width
    (2, 48, 80, 1, 6, 62),     # widest supported row; 3 stages (odd), Cout off the tile size
    (2, 48, 80, 1, 6, 63),     # one pixel wider: the gathering kernel
    (2, 32, 64, 1, 20, 112),   # wide rows (the gathering kernel from here on): tiles inside a row and across two rows
    (1, 16, 48, 1, 5, 224),    # a tile is a piece of one row
    (2, 16, 64, 1, 3, 70),     # three rows: every tile touches the top or the bottom of the plane
    (5, 32, 64, 1, 1, 64),     # one row per image
    (3, 16, 40, 1, 2, 97),     # odd width, tiles crossing images, N tail
    (2, 64, 96, 2, 9, 65),     # groups
    (4, 32, 64, 1, 5, 6),      # plane below 32 pixels: the gathering kernel
    (1, 16, 40, 1, 40, 40),    # one stage per tile
]


@pytest.mark.parametrize("shape", PATCH_SHAPES, ids=lambda s: "b%d_%dto%d_g%d_%dx%d" % s)
def test_patch_kernel_stream_k(gpu, oracle_mod, shape):
    b, cin, cout, groups, h, w_ = shape
    c = case(3, 1, 1, 1, cin, cout, True, groups, True)
    x, w, bias = make_tensors(c, (b, h, w_), seed=b * 1000 + cin + h)
    print("patch case", shape, flush=True)
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)
    # pieces are added in a fixed order: a second run gives the same bits
    again, _ = gpu.run_conv(c, x, w, bias, algo="gemm")
    assert np.array_equal(got, again)
    # factor contract on the same path
    old = np.random.default_rng(5).standard_normal(want.shape).astype(np.float32)
    got_f, _ = gpu.run_conv(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    np.testing.assert_allclose(got_f, oracle_mod.apply_factor(want, old, 0.5), **TOL)


# 3x3 stride-2 pad-1 convolutions with Cin/groups % 16 == 0 and Cout/groups > 32 run the same kernel on patch rows of 512:
# (batch, cin, cout, groups, H, W)
STRIDED_PATCH_SHAPES = [
    (3, 128, 128, 1, 56, 56),  # patch rows of 448: tiles inside an image ...
    (5, 128, 256, 1, 28, 28),  # ... rows of 384
    (9, 256, 512, 1, 14, 14),  # ... rows of 320, tiles across two and three images
    (3, 256, 128, 2, 9, 11),   # odd sizes (the last column and row have no right / lower neighbour), groups
    (2, 128, 64, 1, 17, 33),   # odd sizes, tiles crossing rows at every offset
    (2, 144, 80, 1, 12, 112),  # wide rows (512), 9 stages, Cout off the tile size
    (1, 128, 40, 1, 64, 64),
    (3, 64, 128, 1, 56, 56),   # fewer than 128 input channels: the gathering kernel
    (4, 128, 64, 1, 8, 8),     # output plane below 32 pixels: the gathering kernel
    (2, 128, 64, 1, 6, 300),   # patch longer than the rows: the gathering kernel
]


@pytest.mark.parametrize("shape", STRIDED_PATCH_SHAPES, ids=lambda s: "b%d_%dto%d_g%d_%dx%d" % s)
def test_strided_patch_kernel(gpu, oracle_mod, shape):
    b, cin, cout, groups, h, w_ = shape
    c = case(3, 1, 2, 1, cin, cout, True, groups, True)
    x, w, bias = make_tensors(c, (b, h, w_), seed=b * 1000 + cin + h)
    print("strided patch case", shape, flush=True)
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)
    again, _ = gpu.run_conv(c, x, w, bias, algo="gemm")
    assert np.array_equal(got, again)
    old = np.random.default_rng(5).standard_normal(want.shape).astype(np.float32)
    got_f, _ = gpu.run_conv(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    np.testing.assert_allclose(got_f, oracle_mod.apply_factor(want, old, 0.5), **TOL)
    # integer-valued tensors: exact whatever the order of the sum
    rng = np.random.default_rng(13)
    xi = rng.integers(-3, 4, size=x.shape).astype(np.float32)
    wi = rng.integers(-2, 3, size=w.shape).astype(np.float32)
    bi = rng.integers(-5, 6, size=bias.shape).astype(np.float32)
    got_i, _ = gpu.run_conv(c, xi, wi, bi, algo="gemm")
    assert np.array_equal(got_i, oracle_conv(oracle_mod, c, xi, wi, bi))


def test_patch_kernel_integer_exact_and_small_workspace(gpu):
    # integer-valued tensors: every summation order gives the same fp32 result, so pieces that
    # were mis-addressed, dropped or added twice cannot hide behind a tolerance.  The same op is
    # then run with a workspace sized for batch 1: too small for the pieces, so every workgroup
    # takes whole tiles, and the result must not change.
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(11)
    c = case(3, 1, 1, 1, 128, 192, True, 1, False)
    x = np.round(rng.standard_normal((6, 128, 14, 14)) * 2).astype(np.float32)
    w = np.round(rng.standard_normal((192, 128, 3, 3)) * 2).astype(np.float32)
    bias = np.round(rng.standard_normal(192) * 3).astype(np.float32)
    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(bias).double(),
                                      stride=1, padding=1).numpy()
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    assert np.array_equal(got.astype(np.float64), want)
    op_small = dlp.Conv2DForward.create(gpu.settings_of(c, (1, 128, 14, 14)), True, "identity", "gemm")
    op_full = dlp.Conv2DForward.create(gpu.settings_of(c, x.shape), True, "identity", "gemm")
    assert 0 < op_small.workspace() < op_full.workspace()
    y = torch.full(want.shape, float("nan"), dtype=torch.float32, device="cuda:0")
    op_full.enqueue(gpu.dev(x), gpu.dev(w), gpu.dev(bias), y, torch.empty(op_small.workspace(), dtype=torch.uint8, device="cuda:0"), 0.0)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy().astype(np.float64), want)


# 7x7 / stride 2 convolutions of 3 channels (the ResNet stem) run a kernel of their own: a band of four output rows per
# workgroup, input rows and filter rows in LDS, blocks of 32 pixels handed out inside the workgroup.
# (batch, cout, H, W, pad, bias, activation)
STEM_SHAPES = [
    (2, 64, 224, 224, 3, True, "relu"),       # the real shape: 28 bands of 14 blocks
    (3, 64, 37, 53, 3, True, "identity"),     # width off the 16-byte loads, last band of three rows
    (1, 8, 9, 12, 3, False, "relu"),          # one m tile with eight filters, OH = 5
    (2, 72, 40, 64, 3, True, "tanh"),         # second m tile holds eight filters
    (2, 128, 30, 36, 2, True, "relu6"),       # two whole m tiles, pad 2
    (1, 16, 21, 20, 0, True, "identity"),     # no padding
    (2, 24, 7, 8, 3, True, "sigmoid"),        # image as small as the filter
    (2, 32, 33, 44, (3, 1), True, "relu"),    # different row / column padding
    (2, 16, 20, 232, (0, 4), False, "relu"),  # widest row the LDS rows hold
    (5, 64, 64, 64, 3, True, "relu"),
]


@pytest.mark.parametrize("shape", STEM_SHAPES, ids=lambda s: "b%d_o%d_%dx%d_p%s_%s" % (s[0], s[1], s[2], s[3], s[4], s[6]))
def test_stem_kernel(gpu, oracle_mod, shape):
    b, cout, h, w_, pad, has_bias, act = shape
    c = case(7, pad, 2, 1, 3, cout, has_bias, 1, False)
    c["activation"] = act
    x, w, bias = make_tensors(c, (b, h, w_), seed=b * 100 + cout + w_)
    print("stem case", shape, flush=True)
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)
    again, _ = gpu.run_conv(c, x, w, bias, algo="gemm")
    assert np.array_equal(got, again)
    old = np.random.default_rng(5).standard_normal(want.shape).astype(np.float32)
    got_f, _ = gpu.run_conv(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    np.testing.assert_allclose(got_f, oracle_mod.apply_factor(want, old, 0.5), **TOL)


def test_stem_kernel_integer_exact_and_unaligned_input(gpu):
    # integer-valued tensors: every summation order gives the same fp32 result, which must EQUAL the integer result;
    # the input starts 4 bytes off a 16-byte boundary the second time (the kernel then loads single elements)
    import torch
    import dlprimitives_amd as dlp

    rng = np.random.default_rng(11)
    x = np.round(rng.standard_normal((3, 3, 50, 72)) * 3).astype(np.float32)
    w = np.round(rng.standard_normal((40, 3, 7, 7)) * 3).astype(np.float32)
    bias = np.round(rng.standard_normal(40) * 3).astype(np.float32)
    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(bias).double(),
                                      stride=2, padding=3).numpy()
    st = dlp.Conv2DSettings(3, 40, 7, 2, 1, 3, 1, x.shape)
    op = dlp.Conv2DForward.create(st, True, "identity", "gemm")
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    wd, bd = torch.from_numpy(w).cuda(), torch.from_numpy(bias).cuda()
    for shift in (0, 1):
        store = torch.zeros(x.size + 8, dtype=torch.float32, device="cuda:0")
        xd = store[shift:shift + x.size].view(x.shape)
        xd.copy_(torch.from_numpy(x))
        assert xd.data_ptr() % 16 == 4 * shift
        y = torch.full(want.shape, float("nan"), dtype=torch.float32, device="cuda:0")
        op.enqueue(xd, wd, bd, y, ws)
        torch.cuda.synchronize()
        assert np.array_equal(y.cpu().numpy().astype(np.float64), want), shift


def test_gemm_integer_exact(gpu):
    # integer-valued inputs: fp32 sums are exact in any order, so the MFMA result must
    # EQUAL the integer result -- catches any indexing/layout slip that a tolerance could hide
    rng = np.random.default_rng(7)
    c = case(3, 1, 2, 1, 20, 70, True, 1, False)
    x = np.round(rng.standard_normal((3, 20, 13, 17)) * 3).astype(np.float32)
    w = np.round(rng.standard_normal((70, 20, 3, 3)) * 3).astype(np.float32)
    bias = np.round(rng.standard_normal(70) * 3).astype(np.float32)
    import torch

    want = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(bias).double(),
                                      stride=2, padding=1).numpy()
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm")
    assert np.array_equal(got.astype(np.float64), want)


@pytest.mark.parametrize("algo,c,bhw", [
    ("gemm", case(3, 1, 1, 1, 16, 24, True, 1, True), (2, 11, 9)),
    ("winograd", case(3, 1, 1, 1, 16, 24, True, 1, True), (2, 11, 9)),
    ("depthwise_separable", case(3, 1, 1, 1, 24, 24, True, 24, True), (2, 11, 9)),
    ("depthwise_separable", case(3, 1, 2, 1, 24, 24, True, 24, True), (2, 11, 9)),
], ids=lambda v: v if isinstance(v, str) else None)
def test_factor_contract(gpu, oracle_mod, algo, c, bhw):
    # y = factor*y_old + act(conv + bias); activation applies to the new term only
    x, w, bias = make_tensors(c, bhw, seed=5)
    base, used = gpu.run_conv(c, x, w, bias, algo=algo, expect_algo=algo)
    old = np.random.default_rng(1).standard_normal(base.shape).astype(np.float32)
    got, _ = gpu.run_conv(c, x, w, bias, algo=algo, factor=0.5, y_init=old)
    want = oracle_mod.apply_factor(oracle_conv(oracle_mod, c, x, w, bias), old, 0.5)
    np.testing.assert_allclose(got, want, **TOL)


@pytest.mark.parametrize("act", ["identity", "relu", "tanh", "sigmoid", "relu6"])
def test_activations(gpu, oracle_mod, act):
    c = case(3, 1, 1, 1, 8, 12, True, 1, False)
    c["activation"] = act
    x, w, bias = make_tensors(c, (2, 9, 9), seed=3)
    w *= 6  # push values beyond the relu6 knee
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm")
    np.testing.assert_allclose(got, oracle_conv(oracle_mod, c, x, w, bias), **TOL)


def test_empty_batch_and_shape_errors(gpu):
    import torch

    import dlprimitives_amd as dlp

    st = dlp.Conv2DSettings(4, 8, 3, 1, 1, 1, 1, (2, 4, 8, 8))
    op = dlp.Conv2DForward.create(st, True, "relu", "gemm")
    x = torch.zeros((0, 4, 8, 8), device="cuda:0")
    w = torch.zeros((8, 4, 3, 3), device="cuda:0")
    b = torch.zeros(8, device="cuda:0")
    y = torch.zeros((0, 8, 8, 8), device="cuda:0")
    op.enqueue(x, w, b, y)  # empty batch is a no-op
    with pytest.raises(dlp.ValidationError):  # bias flag mismatch (src/gemm.cpp:526-533)
        op.enqueue(torch.zeros((1, 4, 8, 8), device="cuda:0"), w, None, torch.zeros((1, 8, 8, 8), device="cuda:0"))
    with pytest.raises(dlp.ValidationError):  # H/W changed without re-create
        op.enqueue(torch.zeros((1, 4, 9, 8), device="cuda:0"), w, b, torch.zeros((1, 8, 9, 8), device="cuda:0"))
    torch.cuda.synchronize()


# ------------------------------------------------------------ algorithm choice
def test_algorithm_selection_rules(gpu):
    import dlprimitives_amd as dlp

    def algo(c, hw, name, batch=2):
        st = gpu.settings_of(c, (batch, c["cin"], hw, hw))
        return dlp.Conv2DForward.create(st, False, "identity", name).algo()

    c33 = case(3, 1, 1, 1, 16, 16, False, 1, False)
    assert algo(c33, 8, "") == "winograd" and algo(c33, 8, "auto") == "winograd" and algo(c33, 8, "gemm") == "gemm"
    assert algo(case(3, 1, 1, 1, 4, 16, False, 1, False), 8, "") == "gemm"  # < 8 channels: not recommended
    big = case(3, 1, 1, 1, 48, 96, False, 1, False)  # LDS-patch kernel, fewer than 128 input channels: the automatic choice keeps the GEMM
    assert algo(big, 28, "") == "gemm" and algo(big, 28, "auto") == "gemm" and algo(big, 28, "winograd") == "winograd"
    assert algo(big, 112, "") == "winograd"  # too wide for the patch rows: Winograd against the gathering GEMM
    assert algo(case(3, 1, 1, 1, 64, 96, False, 1, False), 28, "", 64) == "gemm"      # filters off 64: 32 output channels per workgroup
    assert algo(case(3, 1, 1, 1, 64, 64, False, 1, False), 28, "", 64) == "winograd"  # 64 channels in, a multiple of 64 out: Winograd again
    assert algo(case(3, 1, 1, 1, 128, 128, False, 1, False), 28, "", 64) == "winograd"
    # ... as long as the batch of the settings leaves the Winograd kernel one and a half workgroups per compute unit
    assert algo(case(3, 1, 1, 1, 128, 128, False, 1, False), 28, "", 2) == "gemm"
    assert algo(case(3, 1, 1, 1, 512, 512, False, 1, False), 7, "", 32) == "gemm"
    assert algo(case(3, 1, 1, 1, 512, 512, False, 1, False), 7, "", 64) == "winograd"
    assert algo(case(3, 1, 1, 1, 128, 128, False, 1, False), 28, "winograd", 2) == "winograd"  # asked for by name: always
    assert algo(case(3, 1, 1, 1, 4, 16, False, 1, False), 8, "winograd") == "winograd"
    assert algo(case(3, 1, 2, 1, 16, 16, False, 1, False), 8, "winograd") == "gemm"  # incompatible -> silent gemm
    dw = case(3, 1, 1, 1, 16, 16, False, 16, False)
    assert algo(dw, 8, "") == "depthwise_separable" and algo(dw, 8, "gemm") == "gemm"
    assert algo(case(5, 2, 1, 1, 16, 16, False, 16, False), 8, "depthwise_separable") == "depthwise_separable"
    assert algo(case(3, 0, 1, 1, 16, 16, False, 16, False), 8, "depthwise_separable") == "gemm"  # pad != k/2


# ------------------------------------------------------------ Winograd
@pytest.mark.parametrize("shape", [(2, 128, 128, 28, 28), (2, 256, 256, 14, 14), (3, 8, 16, 7, 9), (1, 16, 8, 1, 1), (2, 24, 40, 5, 6),
                                   (5, 16, 16, 13, 13),
                                   (2, 12, 20, 9, 10),    # Cin not a multiple of the K chunk (masked channel tail), rows staged in LDS
                                   (3, 3, 8, 8, 8),       # fewer channels than one K chunk
                                   (1, 16, 32, 56, 56),   # rows of 32 tiles do not fit the staging buffer: patches gathered from global memory
                                   (1, 11, 8, 10, 120),   # the same with a masked channel tail and a wide image
                                   (40, 8, 8, 3, 3),      # more than four images per workgroup
                                   (9, 16, 16, 7, 7)],    # a workgroup's tiles span three images
                         ids=lambda s: "b%d_c%d_n%d_%dx%d" % s)
def test_winograd_three_way(gpu, oracle_mod, shape):
    B, C, N, H, W = shape
    c = case(3, 1, 1, 1, C, N, True, 1, True)
    x, w, bias = make_tensors(c, (B, H, W), seed=C + H)
    got, _ = gpu.run_conv(c, x, w, bias, algo="winograd", expect_algo="winograd")
    gemm, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    wino_cpu = oracle_mod.winograd_forward(x, w, bias, "relu")
    direct = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, wino_cpu, **TOL)
    np.testing.assert_allclose(got, direct, **TOL)
    np.testing.assert_allclose(got, gemm, **TOL)


# Enough workgroups for the chip and a multiple of 64 filters: a workgroup takes two blocks of 32 output channels
@pytest.mark.parametrize("shape", [(8, 8, 512, 28, 28),    # rows staged in LDS
                                   (8, 12, 512, 28, 28),   # masked channel tail
                                   (4, 8, 512, 56, 56),    # patches gathered from global memory
                                   (33, 16, 1024, 14, 14)],  # tiles of a workgroup span images
                         ids=lambda s: "b%d_c%d_n%d_%dx%d" % s)
def test_winograd_two_blocks_per_workgroup(gpu, oracle_mod, shape):
    import dlprimitives_amd as dlp

    B, C, N, H, W = shape
    c = case(3, 1, 1, 1, C, N, True, 1, True)
    x, w, bias = make_tensors(c, (B, H, W), seed=C + H)
    dlp.timing_enable(True)
    dlp.timing_reset()
    got, _ = gpu.run_conv(c, x, w, bias, algo="winograd", expect_algo="winograd")
    kernels = [k for (_, _, k) in dlp.timing_records(kernels=True) if k.startswith("wino_fused_kernel")]
    dlp.timing_enable(False)
    assert kernels and all(k.endswith(", 2>") for k in kernels), kernels
    np.testing.assert_allclose(got, oracle_conv(oracle_mod, c, x, w, bias), **TOL)
    old = np.random.default_rng(5).standard_normal(got.shape).astype(np.float32)
    got_f, _ = gpu.run_conv(c, x, w, bias, algo="winograd", factor=0.5, y_init=old)
    np.testing.assert_allclose(got_f, oracle_mod.apply_factor(got, old, 0.5), rtol=1e-5, atol=1e-5)


def test_winograd_batch_larger_than_hint_is_chunked(gpu, oracle_mod):
    c = case(3, 1, 1, 1, 16, 16, True, 1, False)
    x, w, bias = make_tensors(c, (7, 10, 10), seed=2)
    got, _ = gpu.run_conv(c, x, w, bias, algo="winograd", expect_algo="winograd", batch_hint=2)
    np.testing.assert_allclose(got, oracle_mod.winograd_forward(x, w, bias, "identity"), **TOL)


# ------------------------------------------------------------ depthwise
DW_SHAPES = [(144, 56), (192, 28), (384, 14), (960, 7)]


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ch,hw", DW_SHAPES)
def test_depthwise_mobilenet_shapes(gpu, oracle_mod, ch, hw, stride):
    c = case(3, 1, stride, 1, ch, ch, True, ch, False)
    c["activation"] = "relu6"
    x, w, bias = make_tensors(c, (2, hw, hw), seed=ch)
    w *= 4
    got, _ = gpu.run_conv(c, x, w, bias, algo="depthwise_separable", expect_algo="depthwise_separable", batch_hint=64)
    want = oracle_conv(oracle_mod, c, x, w, bias)  # reference semantics for stride 2: grouped GEMM conv
    np.testing.assert_allclose(got, want, **TOL)
    if stride == 1:
        np.testing.assert_allclose(got, oracle_mod.depthwise_forward(x, w, bias, "relu6"), **TOL)
    as_gemm, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    np.testing.assert_allclose(got, as_gemm, **TOL)


@pytest.mark.parametrize("geom", [(3, 1, 5, 9, 31), (3, 2, 5, 9, 31), (3, 1, 3, 1, 1), (3, 2, 6, 2, 3), (5, 1, 7, 12, 10), (7, 1, 4, 9, 9), (3, 1, 2, 70, 3),
                                  (3, 2, 2, 3, 70)], ids=lambda g: "k%d_s%d_c%d_%dx%d" % g)
def test_depthwise_odd_shapes(gpu, oracle_mod, geom):
    k, s, ch, h, w_ = geom
    c = case(k, k // 2, s, 1, ch, ch, True, ch, True)
    x, w, bias = make_tensors(c, (3, h, w_), seed=h * w_)
    got, _ = gpu.run_conv(c, x, w, bias, algo="depthwise_separable", expect_algo="depthwise_separable")
    np.testing.assert_allclose(got, oracle_conv(oracle_mod, c, x, w, bias), **TOL)


@pytest.mark.parametrize("geom", [(1, 5, 7, 7, 3), (2, 5, 7, 7, 3), (1, 130, 7, 7, 1), (1, 3, 56, 56, 2), (2, 3, 56, 56, 1), (1, 7, 14, 21, 2), (1, 2, 64, 64, 1),
                                  (1, 2, 65, 64, 1), (2, 6, 13, 13, 5)], ids=lambda g: "s%d_c%d_%dx%d_b%d" % g)
@pytest.mark.parametrize("unaligned", [False, True])
def test_depthwise_plane_runs(gpu, oracle_mod, geom, unaligned):
    """3x3 depthwise planes of at most 16 KB go through LDS in runs of whole planes: run tails (fewer planes than a run, a last
    16-byte piece cut short), 1 and 2 tasks per thread, the largest plane that fits (64 x 64) and the first that does not, the
    factor path -- and tensors that do not start on a 16-byte boundary, which take the strip kernel."""
    import torch

    import dlprimitives_amd as dlp

    s, ch, h, w_, b = geom
    c = case(3, 1, s, 1, ch, ch, True, ch, True)
    x, w, bias = make_tensors(c, (b, h, w_), seed=ch + h)
    want = oracle_conv(oracle_mod, c, x, w, bias)
    st = gpu.settings_of(c, x.shape)
    op = dlp.Conv2DForward.create(st, True, "relu", "depthwise_separable")
    assert op.algo() == "depthwise_separable"
    off = 1 if unaligned else 0
    xbuf = torch.zeros(x.size + off, device="cuda:0")
    ybuf = torch.full((want.size + off,), float("nan"), device="cuda:0")
    xd, yd = xbuf[off:].view(x.shape), ybuf[off:].view(want.shape)
    xd.copy_(torch.from_numpy(x))
    op.enqueue(xd, gpu.dev(w), gpu.dev(bias), yd, None, 0.0)
    torch.cuda.synchronize()
    np.testing.assert_allclose(yd.cpu().numpy(), want, **TOL)
    old = np.random.default_rng(1).standard_normal(want.shape).astype(np.float32)
    yd.copy_(torch.from_numpy(old))
    op.enqueue(xd, gpu.dev(w), gpu.dev(bias), yd, None, 0.5)
    torch.cuda.synchronize()
    np.testing.assert_allclose(yd.cpu().numpy(), oracle_mod.apply_factor(want, old, 0.5), **TOL)


@pytest.mark.parametrize("geom", [(1, 3, 28, 28, 2), (1, 5, 30, 33, 3), (1, 2, 20, 64, 2), (1, 3, 9, 100, 2), (1, 2, 23, 128, 1), (1, 2, 11, 200, 2),
                                  (1, 2, 8, 256, 2), (2, 3, 28, 28, 2), (2, 5, 15, 22, 3), (2, 2, 33, 128, 2), (2, 2, 17, 132, 2), (2, 2, 9, 256, 2),
                                  (2, 7, 14, 14, 5), (1, 70, 7, 64, 1)], ids=lambda g: "s%d_c%d_%dx%d_b%d" % g)
@pytest.mark.parametrize("act", ["relu6", "identity", "tanh"])
def test_depthwise_register_strips(gpu, oracle_mod, geom, act):
    """fp32 3x3 depthwise planes of 400 elements and more (100 at stride 2) are computed in strips of 7 output rows held in
    registers, one, two or four input columns per lane depending on the width: every width class at both strides, heights that
    end a strip early, strips per wavefront that do not fill it, a last wavefront with idle strips, no bias, the factor path,
    and integer-valued tensors, which must come out exact."""
    import torch

    import dlprimitives_amd as dlp

    s, ch, h, w_, b = geom
    c = case(3, 1, s, 1, ch, ch, act != "identity", ch, False)
    c["activation"] = act
    x, w, bias = make_tensors(c, (b, h, w_), seed=ch * 1000 + h * w_)
    want = oracle_conv(oracle_mod, c, x, w, bias)
    got, _ = gpu.run_conv(c, x, w, bias, algo="depthwise_separable", expect_algo="depthwise_separable")
    np.testing.assert_allclose(got, want, **TOL)
    old = np.random.default_rng(2).standard_normal(want.shape).astype(np.float32)
    got, _ = gpu.run_conv(c, x, w, bias, algo="depthwise_separable", factor=-0.75, y_init=old)
    np.testing.assert_allclose(got, oracle_mod.apply_factor(want, old, -0.75), **TOL)
    if act != "tanh":
        rng = np.random.default_rng(7)
        xi = rng.integers(-4, 5, size=x.shape).astype(np.float32)
        wi = rng.integers(-3, 4, size=w.shape).astype(np.float32)
        bi = None if bias is None else rng.integers(-5, 6, size=bias.shape).astype(np.float32)
        got, _ = gpu.run_conv(c, xi, wi, bi, algo="depthwise_separable")
        assert np.array_equal(got, oracle_conv(oracle_mod, c, xi, wi, bi))


# ------------------------------------------------------------ pointwise followers of the depthwise blocks
@pytest.mark.parametrize("pw", [(144, 24, 56), (144, 32, 28), (192, 32, 28), (192, 64, 14), (384, 64, 14), (384, 96, 14), (960, 160, 7), (960, 320, 7)],
                         ids=lambda p: "%dto%d_at%d" % p)
def test_pointwise_1x1(gpu, oracle_mod, pw):
    cin, cout, hw = pw
    c = case(1, 0, 1, 1, cin, cout, True, 1, False)
    c["activation"] = "relu6"
    x, w, bias = make_tensors(c, (2, hw, hw), seed=cin)
    got, _ = gpu.run_conv(c, x, w, bias, expect_algo="gemm")
    np.testing.assert_allclose(got, oracle_conv(oracle_mod, c, x, w, bias), **TOL)


# 1x1 convolutions whose last tile of 64 filters would be at most half full run on tiles of 32 filters x 128 pixels
# (cin, cout, H, W, batch, stride, activation)
NARROW_TILE_SHAPES = [(384, 96, 14, 14, 3, 1, "relu6"), (960, 160, 7, 7, 2, 1, "relu"), (48, 96, 9, 11, 3, 1, "identity"), (32, 65, 5, 7, 2, 1, "relu"),
                      (128, 96, 28, 28, 2, 2, "relu"), (20, 70, 6, 6, 2, 1, "tanh")]


@pytest.mark.parametrize("shape", NARROW_TILE_SHAPES, ids=lambda s: "%dto%d_%dx%d_b%d_s%d_%s" % s)
def test_pointwise_tiles_of_32_filters(gpu, oracle_mod, shape):
    import torch

    import dlprimitives_amd as dlp

    cin, cout, h, w_, b, stride, act = shape
    c = case(1, 0, stride, 1, cin, cout, True, 1, False)
    c["activation"] = act
    x, w, bias = make_tensors(c, (b, h, w_), seed=cin + cout)
    dlp.timing_enable(True)
    dlp.timing_reset()
    got, _ = gpu.run_conv(c, x, w, bias, algo="gemm", expect_algo="gemm")
    kernels = [k for (_, _, k) in dlp.timing_records(kernels=True) if k.startswith("conv_gemm_f32_kernel")]
    dlp.timing_enable(False)
    assert kernels and all(k.startswith("conv_gemm_f32_kernel<float, 32, 128") for k in kernels), kernels
    want = oracle_conv(oracle_mod, c, x, w, bias)
    np.testing.assert_allclose(got, want, **TOL)
    old = np.random.default_rng(5).standard_normal(want.shape).astype(np.float32)
    got_f, _ = gpu.run_conv(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    np.testing.assert_allclose(got_f, oracle_mod.apply_factor(want, old, 0.5), **TOL)
    # packed once + enqueue_packed gives the same bits as enqueue
    op = dlp.Conv2DForward.create(gpu.settings_of(c, x.shape), True, act, "gemm")
    packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    op.pack(gpu.dev(w), packed)
    y2 = torch.full(want.shape, float("nan"), dtype=torch.float32, device="cuda:0")
    op.enqueue_packed(gpu.dev(x), gpu.dev(w), packed, gpu.dev(bias), y2, ws, 0.0)
    torch.cuda.synchronize()
    np.testing.assert_allclose(y2.cpu().numpy(), got, rtol=1e-6, atol=1e-6)
    if act != "tanh":  # integer-valued tensors: exact whatever the order of the sum
        rng = np.random.default_rng(13)
        xi = rng.integers(-3, 4, size=x.shape).astype(np.float32)
        wi = rng.integers(-2, 3, size=w.shape).astype(np.float32)
        bi = rng.integers(-5, 6, size=(cout,)).astype(np.float32)
        got_i, _ = gpu.run_conv(c, xi, wi, bi, algo="gemm")
        assert np.array_equal(got_i, oracle_conv(oracle_mod, c, xi, wi, bi))


# ------------------------------------------------------------ InnerProduct
def test_inner_product_reference_goldens(gpu):
    doc = json.load(open(os.path.join(GOLDEN, "inner_product_fwd.json")))
    n = 0
    for t in doc["tests"]:
        o = t["options"]
        if not t["params"]:
            continue
        w = np.array(t["params"][0], dtype=np.float32).reshape(o["outputs"], o["inputs"])
        bias = np.array(t["params"][1], dtype=np.float32) if o["bias"] else None
        for cs in t["cases"]:
            if "in" not in cs:
                continue
            x = np.array(cs["in"][0], dtype=np.float32).reshape(cs["in_shapes"][0])
            want = np.array(cs["out"][0], dtype=np.float32).reshape(cs["out_shapes"][0])
            np.testing.assert_allclose(gpu.run_ip(x, w, bias, o["activation"]), want, **TOL)
            n += 1
    assert n == 28


@pytest.mark.parametrize("bio", [(128, 2048, 1000), (1, 512, 1000), (8, 1024, 1024), (50, 333, 77), (2, 1, 1), (3, 1030, 70), (200, 512, 64),
                                 (33, 4100, 31), (16, 25088, 96)], ids=lambda v: "b%d_%dto%d" % v)
@pytest.mark.parametrize("bias", [True, False])
def test_inner_product_vs_oracle(gpu, oracle_mod, bio, bias):
    B, I, O = bio
    rng = np.random.default_rng(B + I)
    x = rng.uniform(-1, 1, (B, I)).astype(np.float32)
    w = (rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, O).astype(np.float32) if bias else None
    np.testing.assert_allclose(gpu.run_ip(x, w, b, "relu"), oracle_mod.ip_forward(x, w, b, "relu"), **TOL)


def test_inner_product_same_op_many_calls(gpu, oracle_mod):
    """One op object, batches that grow and shrink: the op-owned partial-sum buffer is regrown, the tile
    counters return to zero after every call, and the result does not depend on the call history."""
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(5)
    I, O = 2048, 1000
    w = (rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, O).astype(np.float32)
    op = dlp.IPForward.create(dlp.IPSettings(I, O, 8), True, "identity")
    wd, bd = gpu.dev(w), gpu.dev(b)
    first = {}
    for B in (8, 128, 8, 40, 128, 1):
        x = rng.uniform(-1, 1, (B, I)).astype(np.float32) if B not in first else first[B][0]
        yd = torch.full((B, O), float("nan"), dtype=torch.float32, device="cuda:0")
        op.enqueue(gpu.dev(x), wd, bd, yd)
        op.enqueue(gpu.dev(x), wd, bd, yd)  # back to back on the stream
        torch.cuda.synchronize()
        got = yd.cpu().numpy()
        np.testing.assert_allclose(got, oracle_mod.ip_forward(x, w, b), **TOL)
        if B in first:
            assert np.array_equal(got, first[B][1])  # slices are added in a fixed order
        first[B] = (x, got)


# Weight matrices whose rows start on 16-byte boundaries are streamed through LDS in runs of 1 KB per row (ip_stream_kernel).
# (batch, inputs, outputs, activation, bias)
IP_STREAM_SHAPES = [(16, 4096, 1024, "relu", True),      # whole chunks of 256 k, one batch chunk
                    (1, 24, 5, "identity", True),        # one short chunk, one row, five outputs
                    (3, 260, 40, "relu", True),          # a chunk and four k
                    (5, 4100, 1030, "identity", True),   # a last chunk of 4 k, outputs off the block of 32
                    (33, 4096, 1056, "relu", False),     # two batch chunks
                    (130, 8200, 520, "tanh", True)]      # five batch chunks, a short last chunk


@pytest.mark.parametrize("shape", IP_STREAM_SHAPES, ids=lambda s: "b%d_%dto%d_%s_%s" % s)
def test_inner_product_streamed_weights(gpu, oracle_mod, shape):
    import torch

    import dlprimitives_amd as dlp

    B, I, O, act, with_bias = shape
    rng = np.random.default_rng(B + I)
    x = rng.uniform(-1, 1, (B, I)).astype(np.float32)
    w = (rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, O).astype(np.float32) if with_bias else None
    dlp.timing_enable(True)
    dlp.timing_reset()
    got = gpu.run_ip(x, w, b, act)
    kernels = [k for (_, _, k) in dlp.timing_records(kernels=True)]
    dlp.timing_enable(False)
    assert kernels and kernels[-1].startswith("ip_stream_kernel"), kernels
    np.testing.assert_allclose(got, oracle_mod.ip_forward(x, w, b, act), **TOL)
    # one operator, this batch and a smaller one, twice each: counters return to zero, a batch repeats bit for bit (the number
    # of K slices, and with it the order of the sum, depends on the batch)
    op = dlp.IPForward.create(dlp.IPSettings(I, O, B), with_bias, act)
    wd, bd = gpu.dev(w), gpu.dev(b)
    seen = {}
    for rows in (B, max(1, B // 3), B, max(1, B // 3)):
        yd = torch.full((rows, O), float("nan"), dtype=torch.float32, device="cuda:0")
        op.enqueue(gpu.dev(x[:rows]), wd, bd, yd)
        op.enqueue(gpu.dev(x[:rows]), wd, bd, yd)
        torch.cuda.synchronize()
        out = yd.cpu().numpy()
        np.testing.assert_allclose(out, got[:rows], **TOL)
        if rows in seen:
            assert np.array_equal(out, seen[rows])
        seen[rows] = out
    assert np.array_equal(seen[B], got)
    # integer-valued operands: exact whatever the order of the sum
    xi = rng.integers(-3, 4, (B, I)).astype(np.float32)
    wi = rng.integers(-3, 4, (O, I)).astype(np.float32)
    if act != "tanh":
        want = xi.astype(np.int64) @ wi.astype(np.int64).T
        if with_bias:
            bi = rng.integers(-5, 6, O).astype(np.float32)
            want = want + bi.astype(np.int64)
        else:
            bi = None
        if act == "relu":
            want = np.maximum(want, 0)
        assert np.array_equal(gpu.run_ip(xi, wi, bi, act), want.astype(np.float32))


def test_inner_product_integer_exact(gpu):
    # integer-valued operands: every partial sum is exact in fp32, so the split over K slices and the
    # pairing of k inside a matrix instruction must reproduce the integer result exactly
    rng = np.random.default_rng(9)
    x = rng.integers(-3, 4, (70, 1203)).astype(np.float32)
    w = rng.integers(-3, 4, (45, 1203)).astype(np.float32)
    b = rng.integers(-5, 6, 45).astype(np.float32)
    want = (x.astype(np.int64) @ w.astype(np.int64).T + b.astype(np.int64)).astype(np.float32)
    assert np.array_equal(gpu.run_ip(x, w, b), want)


def test_inner_product_flattens_trailing_dims(gpu, oracle_mod):
    # x may be rank > 2: inputs = size_no_batch (src/core/ip.cpp:30)
    rng = np.random.default_rng(0)
    x = rng.uniform(-1, 1, (4, 8, 3, 3)).astype(np.float32)
    w = rng.standard_normal((10, 72)).astype(np.float32)
    np.testing.assert_allclose(gpu.run_ip(x, w, None), oracle_mod.ip_forward(x, w, None), **TOL)


# (cin, cout, H, W, batch): shapes that conv_pointwise_f32_kernel takes (at most 32 output channels, H * W % 4 == 0, Cin % 16 == 0,
# at least 1024 tiles of 128 pixels)
POINTWISE_STREAM_SHAPES = [
    (16, 24, 56, 56, 42),    # 131 712 pixels: 1029 tiles; rows 24..31 of the block are padding
    (144, 32, 56, 56, 42),   # K = 2 chunks + 16
    (80, 5, 60, 60, 37),     # one chunk + 16, a last pixel tile that is cut short (133 200 pixels)
]


@pytest.mark.parametrize("shape", POINTWISE_STREAM_SHAPES, ids=lambda s: "%dto%d_%dx%d_b%d" % s)
def test_pointwise_streaming_kernel(gpu, oracle_mod, shape):
    import torch

    import dlprimitives_amd as dlp

    cin, cout, h, w_, b = shape
    for act, with_bias in (("relu6", True), ("identity", False)):
        c = case(1, 0, 1, 1, cin, cout, with_bias, 1, False)
        c["activation"] = act
        x, w, bias = make_tensors(c, (b, h, w_), seed=cin + cout)
        w *= 3
        want = oracle_conv(oracle_mod, c, x, w, bias)
        st = gpu.settings_of(c, x.shape)
        op = dlp.Conv2DForward.create(st, with_bias, act, "gemm")
        xd, wd, bd = gpu.dev(x), gpu.dev(w), gpu.dev(bias)
        ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
        y = torch.full(want.shape, float("nan"), device="cuda:0")
        dlp.timing_reset()
        dlp.timing_enable(True)
        op.enqueue(xd, wd, bd, y, ws, 0.0)
        torch.cuda.synchronize()
        dlp.timing_enable(False)
        kernels = [k for (_, _, k) in dlp.timing_records(kernels=True)]
        dlp.timing_reset()
        assert any(k.startswith("conv_pointwise_f32_kernel") for k in kernels), kernels
        np.testing.assert_allclose(y.cpu().numpy(), want, **TOL)
        # y = factor * y + act(...)
        old = np.random.default_rng(1).standard_normal(want.shape).astype(np.float32)
        y = gpu.dev(old)
        op.enqueue(xd, wd, bd, y, ws, 0.5)
        torch.cuda.synchronize()
        np.testing.assert_allclose(y.cpu().numpy(), oracle_mod.apply_factor(want, old, 0.5), **TOL)
        # y = act(conv + bias + factor * y): the residual form
        op.accumulate_before_activation(True)
        y = gpu.dev(old)
        op.enqueue(xd, wd, bd, y, ws, 1.0)
        torch.cuda.synchronize()
        lin = oracle_conv(oracle_mod, dict(c, activation="identity"), x, w, bias) + old
        np.testing.assert_allclose(y.cpu().numpy(), np.clip(lin, 0, 6) if act == "relu6" else lin, **TOL)
        # weights packed ahead of time: same kernel, same result
        op.accumulate_before_activation(False)
        packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
        op.pack(wd, packed)
        y = torch.full(want.shape, float("nan"), device="cuda:0")
        op.enqueue_packed(xd, wd, packed, bd, y, ws, 0.0)
        torch.cuda.synchronize()
        np.testing.assert_allclose(y.cpu().numpy(), want, **TOL)


PACKED_CASES = [  # cin, cout, k, s, p, groups, hw, batch, algo, dtype
    (64, 64, 3, 1, 1, 1, 28, 4, "gemm", "float32"),       # LDS-patch kernel, stream-K counters in the scratch
    (64, 64, 3, 1, 1, 1, 28, 4, "winograd", "float32"),
    (128, 256, 3, 2, 1, 1, 14, 8, "gemm", "float32"),     # split-K counters
    (3, 64, 7, 2, 3, 1, 64, 2, "gemm", "float32"),
    (48, 48, 3, 1, 1, 48, 20, 3, "", "float32"),          # depthwise: nothing to pack
    (24, 40, 1, 1, 0, 2, 9, 2, "gemm", "float32"),
    (64, 256, 1, 1, 0, 1, 28, 4, "gemm", "bfloat16"),     # weights read in place
    (64, 64, 3, 1, 1, 1, 28, 4, "gemm", "bfloat16"),
    (128, 128, 3, 2, 1, 1, 28, 4, "gemm", "bfloat16"),
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", PACKED_CASES, ids=lambda c: "c%d_o%d_k%d_s%d_g%d_%s_%s" % (c[0], c[1], c[2], c[3], c[5], c[8] or "auto", c[9]))
def test_gpu_packed_weights_give_the_same_bits(case):
    """dlp_conv2d_fwd_pack + dlp_conv2d_fwd_enqueue_packed against dlp_conv2d_fwd_enqueue (which is checked against
    the oracle above): same kernels on the same operands, so the outputs must be identical; the packed buffer is
    reused by three calls, one with another batch, while the scratch is shared with a second operator."""
    import torch

    import dlprimitives_amd as dlp

    cin, cout, k, s, p, groups, hw, batch, algo, dtype = case
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    code = dlp.capi.FLOAT_DATA if dtype == "float32" else dlp.capi.BFLOAT16_DATA
    torch.manual_seed(cin * 31 + cout)
    st = dlp.Conv2DSettings(cin, cout, k, s, 1, p, groups, (batch, cin, hw, hw), dtype=code)
    op = dlp.Conv2DForward.create(st, True, "relu", algo)
    other = dlp.Conv2DForward.create(st, True, "relu", algo)
    w = (torch.randn(cout, cin // groups, k, k, device="cuda:0") * 0.1).to(tdt)
    bias = torch.randn(cout, device="cuda:0")
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
    assert op.packed_size() <= max(op.workspace(), 0) + 256
    op.pack(w, packed)
    for b in (batch, batch, max(batch // 2, 1)):
        x = torch.randn(b, cin, hw, hw, device="cuda:0").to(tdt)
        oshape = dlp.conv2d_output_shape(st, x.shape)
        want = torch.empty(oshape, device="cuda:0", dtype=tdt)
        other.enqueue(x, w, bias, want, ws)  # also scribbles over the shared scratch
        got = torch.full(oshape, float("nan"), device="cuda:0", dtype=tdt)
        op.enqueue_packed(x, w, packed, bias, got, ws)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (b, float((got.float() - want.float()).abs().max()))
        old = torch.randn(oshape, device="cuda:0").to(tdt)
        got2, want2 = old.clone(), old.clone()
        other.enqueue(x, w, bias, want2, ws, 0.5)
        op.enqueue_packed(x, w, packed, bias, got2, ws, 0.5)
        assert torch.equal(got2, want2)


RESIDUAL_CASES = [  # cin, cout, k, s, p, hw, batch, algo
    (64, 64, 3, 1, 1, 28, 4, "gemm"),       # LDS-patch kernel
    (64, 256, 1, 1, 0, 28, 4, "gemm"),      # buffer-store epilogue
    (24, 37, 1, 1, 0, 9, 3, "gemm"),        # 37 filters: per-element epilogue
    (256, 512, 3, 2, 1, 14, 8, "gemm"),     # split-K, reduced in place
    (64, 64, 3, 1, 1, 28, 4, "winograd"),
    (32, 48, 3, 1, 1, 13, 2, "winograd"),   # odd planes: cut tiles
    (3, 64, 7, 2, 3, 45, 2, "gemm"),        # stem kernel
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", RESIDUAL_CASES, ids=lambda c: "c%d_o%d_k%d_s%d_h%d_%s" % (c[0], c[1], c[2], c[3], c[5], c[7]))
@pytest.mark.parametrize("activation,factor", [("relu", 1.0), ("tanh", 0.5), ("identity", -2.0)])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_accumulate_before_activation(case, activation, factor, dtype):
    """y = act(conv(x, w) + bias + factor * y): a residual sum in the convolution's epilogue, against torch in float64
    (1e-4; bfloat16 tensors 2e-2: the sum is rounded once before and once after the old value joins, as it is when
    the sum is an operator of its own); plain and packed enqueue; factor 0 must leave the usual result."""
    import torch

    import dlprimitives_amd as dlp

    cin, cout, k, s, p, hw, batch, algo = case
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    tol = 1e-4 if dtype == "float32" else 2e-2
    torch.manual_seed(cin + cout + k)
    st = dlp.Conv2DSettings(cin, cout, k, s, 1, p, 1, (batch, cin, hw, hw), dtype=dlp.capi.FLOAT_DATA if dtype == "float32" else dlp.capi.BFLOAT16_DATA)
    op = dlp.Conv2DForward.create(st, True, activation, algo)
    assert op.algo() == algo
    op.accumulate_before_activation(True)
    x = torch.randn(batch, cin, hw, hw, device="cuda:0").to(tdt)
    w = (torch.randn(cout, cin, k, k, device="cuda:0") * (2.0 / (cin * k * k)) ** 0.5).to(tdt)
    bias = torch.randn(cout, device="cuda:0")
    conv = torch.nn.functional.conv2d(x.double().cpu(), w.double().cpu(), bias.double().cpu(), s, p)
    old = torch.randn(conv.shape, device="cuda:0").to(tdt)
    act = {"relu": torch.relu, "tanh": torch.tanh, "identity": lambda v: v}[activation]
    want = act(conv + factor * old.double().cpu())
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    y = old.clone()
    op.enqueue(x, w, bias, y, ws, factor)
    err = float((y.double().cpu() - want).abs().max() / want.abs().max())
    assert err < tol, err
    packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
    op.pack(w, packed)
    y2 = old.clone()
    op.enqueue_packed(x, w, packed, bias, y2, ws, factor)
    assert torch.equal(y, y2)
    y3 = torch.full(conv.shape, float("nan"), device="cuda:0", dtype=tdt)
    op.enqueue(x, w, bias, y3, ws, 0.0)
    err = float((y3.double().cpu() - act(conv)).abs().max() / act(conv).abs().max())
    assert err < tol, err


def test_accumulate_before_activation_is_refused_where_not_built():
    import dlprimitives_amd as dlp

    dw = dlp.Conv2DForward.create(dlp.Conv2DSettings(16, 16, 3, 1, 1, 1, 16, (1, 16, 8, 8)), False, "relu", "depthwise_separable")
    with pytest.raises(dlp.NotImplementedErrorDlprim):
        dw.accumulate_before_activation(True)
    dw.accumulate_before_activation(False)
