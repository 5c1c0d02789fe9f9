"""Depthwise 3x3 + pointwise 1x1 in one launch (dlp_dwpw_fwd_*) against the CPU oracle run as the reference runs the
pair: the depthwise convolution (its own kernel's operation order), then the 1x1 convolution through im2col + sgemm.
fp32 bar rtol = atol = 1e-4; integer-valued tensors must match exactly."""
import numpy as np
import pytest

from conv_cases import case, make_tensors

pytestmark = pytest.mark.gpu

TOL = dict(rtol=1e-4, atol=1e-4)


def oracle_pair(orc, x, wd, bd, act1, stride, wp, bp, act2):
    ch = x.shape[1]
    cfg1 = orc.make_cfg(ch, ch, 3, stride, 1, 1, ch)
    t = orc.conv2d_forward(x, wd, bd, cfg1, act1, threads=8)
    cfg2 = orc.make_cfg(ch, wp.shape[0], 1, 1, 1, 0, 1)
    return orc.conv2d_forward(t, wp, bp, cfg2, act2, threads=8)


def tensors(ch, cout, b, h, w_, seed, with_bias=True, integer=False):
    rng = np.random.default_rng(seed)
    if integer:
        x = rng.integers(-3, 4, (b, ch, h, w_)).astype(np.float32)
        wd = rng.integers(-2, 3, (ch, 1, 3, 3)).astype(np.float32)
        wp = rng.integers(-2, 3, (cout, ch, 1, 1)).astype(np.float32)
        bd = rng.integers(-3, 4, ch).astype(np.float32) if with_bias else None
        bp = rng.integers(-3, 4, cout).astype(np.float32) if with_bias else None
    else:
        x = rng.standard_normal((b, ch, h, w_)).astype(np.float32)
        wd = (rng.standard_normal((ch, 1, 3, 3)) * 0.5).astype(np.float32)
        wp = (rng.standard_normal((cout, ch, 1, 1)) * (2.0 / ch) ** 0.5).astype(np.float32)
        bd = (rng.standard_normal(ch) * 0.3).astype(np.float32) if with_bias else None
        bp = (rng.standard_normal(cout) * 0.3).astype(np.float32) if with_bias else None
    return x, wd, bd, wp, bp


def run_fused(x, wd, bd, act1, stride, wp, bp, act2, factor=0.0, y_init=None, accumulate_first=False, batch_hint=None):
    import torch

    import dlprimitives_amd as dlp
    from gpu_util import dev

    b, ch, h, w_ = x.shape
    st = dlp.Conv2DSettings(ch, ch, 3, stride, 1, 1, ch, (batch_hint or b, ch, h, w_))
    assert dlp.DepthwisePointwiseForward.supported(st, act1, wp.shape[0], act2)
    op = dlp.DepthwisePointwiseForward.create(st, bd is not None, act1, wp.shape[0], bp is not None, act2)
    if accumulate_first:
        op.accumulate_before_activation(True)
    oh, ow = (h + 2 - 3) // stride + 1, (w_ + 2 - 3) // stride + 1
    if y_init is not None:
        yd = dev(y_init)
    else:
        yd = torch.full((b, wp.shape[0], oh, ow), float("nan"), dtype=torch.float32, device="cuda:0")
    op.enqueue(dev(x), dev(wd), dev(bd), dev(wp), dev(bp), yd, factor)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


# the depthwise -> pointwise pairs of the MobileNet blocks (channels, filters, image, stride) that the fused kernel takes: the
# 14 x 14 and 7 x 7 pairs stay two operators (faster there)
MOBILENET_PAIRS = [(144, 24, 56, 1), (144, 32, 56, 2), (192, 32, 28, 1), (192, 64, 28, 2)]


@pytest.mark.parametrize("pair", MOBILENET_PAIRS, ids=lambda p: "c%d_to%d_at%d_s%d" % p)
def test_mobilenet_pairs(oracle_mod, pair):
    ch, cout, hw, stride = pair
    print("pair", pair, flush=True)
    x, wd, bd, wp, bp = tensors(ch, cout, 3, hw, hw, seed=ch + cout)
    got = run_fused(x, wd, bd, "relu6", stride, wp, bp, "identity", batch_hint=64)
    want = oracle_pair(oracle_mod, x, wd, bd, "relu6", stride, wp, bp, "identity")
    np.testing.assert_allclose(got, want, **TOL)
    xi, wdi, bdi, wpi, bpi = tensors(ch, cout, 2, hw, hw, seed=ch, integer=True)
    got = run_fused(xi, wdi, bdi, "relu6", stride, wpi, bpi, "relu")
    want = oracle_pair(oracle_mod, xi, wdi, bdi, "relu6", stride, wpi, bpi, "relu")
    assert np.array_equal(got, want)


# (channels, filters, H, W, stride, batch): partial last bands, widths below the LDS pitch, filters off the 32-row blocks,
# odd heights at stride 2, a single chunk of channels, every row of the kernel's variant table (chunks of 4, 8, 16 channels;
# more than 96 filters; work items of 2 and 4 pixels)
ODD_SHAPES = [(8, 5, 13, 56, 1, 2), (16, 40, 20, 44, 1, 3), (24, 128, 20, 28, 1, 2), (8, 33, 31, 24, 1, 1), (8, 7, 56, 48, 2, 2), (16, 70, 13, 40, 2, 2),
              (16, 96, 28, 28, 2, 3), (8, 17, 27, 20, 2, 2), (48, 64, 26, 28, 1, 5), (16, 100, 36, 16, 1, 3), (8, 3, 128, 4, 1, 2), (32, 100, 30, 24, 2, 1),
              (4, 9, 12, 52, 1, 1)]


@pytest.mark.parametrize("shape", ODD_SHAPES, ids=lambda s: "c%d_to%d_%dx%d_s%d_b%d" % s)
def test_odd_shapes(oracle_mod, shape):
    ch, cout, h, w_, stride, b = shape
    print("shape", shape, flush=True)
    for act1, act2, with_bias in (("relu6", "identity", True), ("identity", "relu", False), ("relu", "relu6", True)):
        x, wd, bd, wp, bp = tensors(ch, cout, b, h, w_, seed=h * w_ + cout, with_bias=with_bias)
        got = run_fused(x, wd, bd, act1, stride, wp, bp, act2)
        want = oracle_pair(oracle_mod, x, wd, bd, act1, stride, wp, bp, act2)
        np.testing.assert_allclose(got, want, **TOL)


def test_factor_and_residual(oracle_mod):
    ch, cout, hw = 48, 24, 28
    x, wd, bd, wp, bp = tensors(ch, cout, 2, hw, hw, seed=5)
    want = oracle_pair(oracle_mod, x, wd, bd, "relu6", 1, wp, bp, "relu")
    old = np.random.default_rng(2).standard_normal(want.shape).astype(np.float32)
    got = run_fused(x, wd, bd, "relu6", 1, wp, bp, "relu", factor=0.5, y_init=old)
    np.testing.assert_allclose(got, oracle_mod.apply_factor(want, old, 0.5), **TOL)
    # the residual form: y = act(conv + bias + factor * y)
    lin = oracle_pair(oracle_mod, x, wd, bd, "relu6", 1, wp, bp, "identity")
    got = run_fused(x, wd, bd, "relu6", 1, wp, bp, "relu", factor=1.0, y_init=old, accumulate_first=True)
    np.testing.assert_allclose(got, np.maximum(lin + old, 0.0), **TOL)


def test_unsupported_shapes_are_refused():
    import dlprimitives_amd as dlp

    for ch, cout, hw, k, stride, pad in ((960, 160, 7, 3, 1, 1), (384, 64, 14, 3, 1, 1), (144, 24, 112, 3, 1, 1), (144, 200, 56, 3, 1, 1), (144, 24, 56, 5, 1, 2),
                                         (18, 24, 56, 3, 1, 1), (144, 24, 54, 3, 1, 1)):
        st = dlp.Conv2DSettings(ch, ch, k, stride, 1, pad, ch, (4, ch, hw, hw))
        assert not dlp.DepthwisePointwiseForward.supported(st, "relu6", cout, "identity")
        with pytest.raises(dlp.NotImplementedErrorDlprim):
            dlp.DepthwisePointwiseForward.create(st, True, "relu6", cout, True, "identity")
    st = dlp.Conv2DSettings(144, 144, 3, 1, 1, 1, 144, (4, 144, 56, 56))
    assert not dlp.DepthwisePointwiseForward.supported(st, "tanh", 24, "identity")


def test_full_size_equals_torch_float64():
    """The launches the benchmark times (batch 64), integer-valued tensors: the result must EQUAL torch in float64."""
    import torch
    import torch.nn.functional as F

    for ch, cout, hw, stride in ((144, 24, 56, 1), (144, 32, 56, 2), (192, 32, 28, 1), (192, 64, 28, 2)):
        print("full size", ch, cout, hw, stride, flush=True)
        x, wd, bd, wp, bp = tensors(ch, cout, 64, hw, hw, seed=cout, integer=True)
        got = run_fused(x, wd, bd, "relu6", stride, wp, bp, "identity")
        t = torch.clamp(F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wd).double(), torch.from_numpy(bd).double(), stride=stride, padding=1, groups=ch), 0, 6)
        want = F.conv2d(t, torch.from_numpy(wp).double(), torch.from_numpy(bp).double()).numpy()
        assert np.array_equal(got.astype(np.float64), want)
