"""TransposedConvolution2D (src/ops/conv2d.cpp:559-805 in the reference).

CPU: the oracle's restatement of the reference CPU path (bias fill, data-gradient pass of the convolution with swapped
channels, activation last) is pinned against torch.nn.functional.conv_transpose2d -- the library routine the reference's own
fixture generator takes as truth (tests/make_test_cases_from_pt.py) -- over strides, dilations, paddings, output paddings and
groups, and the output-shape rule against torch's.  GPU: the HIP operator through the C ABI against the oracle (fp32 bar
1e-4) and, with integer-valued tensors, exactly against torch in float64.
"""
import numpy as np
import pytest

# (cin, cout, kernel, stride, dilate, pad, output_pad, groups, batch, H, W)
CASES = [
    (8, 6, 3, 1, 1, 1, 0, 1, 2, 9, 11),
    (8, 6, 3, 2, 1, 1, 1, 1, 2, 9, 11),        # the usual "upsample by two": k3 s2 p1 op1
    (16, 16, 4, 2, 1, 1, 0, 1, 3, 7, 7),        # k4 s2 p1 (GAN generators)
    (12, 8, 3, 2, 1, 0, 0, 4, 2, 6, 5),         # groups
    (6, 6, 3, 2, 1, 1, 1, 6, 2, 8, 8),          # depthwise
    (4, 10, (3, 5), (2, 3), (2, 1), (1, 2), (1, 2), 2, 2, 5, 6),  # everything asymmetric
    (32, 16, 2, 2, 1, 0, 0, 1, 2, 14, 14),      # k2 s2: no overlap
    (5, 7, 1, 1, 1, 0, 0, 1, 3, 4, 4),          # pointwise
    (64, 32, 3, 1, 1, 1, 0, 1, 2, 28, 28),      # stride 1: a plain convolution with the flipped filter
    (3, 4, 5, 3, 1, 2, 2, 1, 1, 10, 3),
]


def _pair(v):
    return (v, v) if isinstance(v, int) else tuple(v)


def _ids(c):
    return "c%dto%d_k%s_s%s_d%s_p%s_op%s_g%d" % (c[0], c[1], c[2], c[3], c[4], c[5], c[6], c[7])


def _tensors(c, seed, integers=False):
    cin, cout, k, s, d, p, op, g, b, h, w_ = c
    rng = np.random.default_rng(seed)
    kh, kw = _pair(k)
    if integers:
        x = rng.integers(-3, 4, (b, cin, h, w_)).astype(np.float32)
        w = rng.integers(-2, 3, (cin, cout // g, kh, kw)).astype(np.float32)
        bias = rng.integers(-5, 6, cout).astype(np.float32)
    else:
        x = rng.uniform(-1, 1, (b, cin, h, w_)).astype(np.float32)
        w = (rng.standard_normal((cin, cout // g, kh, kw)) * 0.3).astype(np.float32)
        bias = rng.uniform(-0.5, 0.5, cout).astype(np.float32)
    return x, w, bias


def _torch(c, x, w, bias, activation, f64=False):
    import torch
    import torch.nn.functional as F

    cin, cout, k, s, d, p, op, g = c[:8]
    dt = torch.float64 if f64 else torch.float32
    y = F.conv_transpose2d(torch.from_numpy(x).to(dt), torch.from_numpy(w).to(dt), torch.from_numpy(bias).to(dt) if bias is not None else None,
                           stride=_pair(s), padding=_pair(p), output_padding=_pair(op), groups=g, dilation=_pair(d))
    if activation == "relu":
        y = y.clamp(min=0)
    elif activation == "tanh":
        y = y.tanh()
    return y.float().numpy()


@pytest.mark.parametrize("c", CASES, ids=_ids)
def test_oracle_against_torch(oracle_mod, c):
    cin, cout, k, s, d, p, op, g = c[:8]
    cfg = oracle_mod.make_cfg(cin, cout, k, s, d, p, g)
    for activation, with_bias in (("identity", True), ("relu", False), ("tanh", True)):
        x, w, bias = _tensors(c, 3)
        b = bias if with_bias else None
        got = oracle_mod.tconv2d_forward(x, w, b, cfg, _pair(op), activation)
        want = _torch(c, x, w, b, activation)
        assert got.shape == want.shape == oracle_mod.tconv2d_output_shape(cfg, x.shape, _pair(op))
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    # integer-valued tensors: every sum is exact, whatever its order
    x, w, bias = _tensors(c, 4, integers=True)
    assert np.array_equal(oracle_mod.tconv2d_forward(x, w, bias, cfg, _pair(op)), _torch(c, x, w, bias, "identity", f64=True))


def test_output_shape_rule(oracle_mod):
    # o = (i - 1) * s - 2 * p + d * (k - 1) + output_pad + 1, src/core/conv.cpp:31-43
    cfg = oracle_mod.make_cfg(4, 6, (3, 5), (2, 3), (2, 1), (1, 2), 2)
    assert oracle_mod.tconv2d_output_shape(cfg, (2, 4, 5, 6), (1, 2)) == (2, 6, (5 - 1) * 2 - 2 + 2 * 2 + 1 + 1, (6 - 1) * 3 - 4 + 4 + 2 + 1)
    with pytest.raises(ValueError):
        oracle_mod.tconv2d_output_shape(cfg, (2, 5, 5, 6), (0, 0))  # channels


def test_host_shape_and_validation_without_a_gpu():
    import dlprimitives_amd as dlp

    st = dlp.Conv2DSettings(8, 6, 3, 2, 1, 1, 1, (2, 8, 9, 11))
    assert dlp.conv2d_transposed_output_shape(st, (2, 8, 9, 11), (1, 1)) == (2, 6, 18, 22)
    with pytest.raises(dlp.ValidationError):
        dlp.conv2d_transposed_output_shape(st, (2, 7, 9, 11), (1, 1))
    with pytest.raises(dlp.ValidationError):  # an output_pad of a whole stride describes the next larger input
        dlp.TransposedConv2DForward.create(st, (2, 0), True)


@pytest.fixture(scope="module")
def gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    import gpu_util

    return gpu_util


def _run_gpu(gpu, c, x, w, bias, activation, batch_hint=None):
    import torch

    import dlprimitives_amd as dlp

    cin, cout, k, s, d, p, op, g = c[:8]
    hint = (batch_hint or x.shape[0],) + tuple(x.shape[1:])
    st = dlp.Conv2DSettings(cin, cout, k, s, d, p, g, hint)
    t = dlp.TransposedConv2DForward.create(st, _pair(op), bias is not None, activation)
    y = torch.full(t.output_shape(x.shape), float("nan"), device="cuda:0")
    ws = torch.empty(max(t.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    outs = []
    for _ in range(2):  # the same operator twice: nothing may depend on what the first call left in y or the workspace
        t.enqueue(gpu.dev(x), gpu.dev(w), gpu.dev(bias), y, ws)
        torch.cuda.synchronize()
        outs.append(y.cpu().numpy())
    assert np.array_equal(outs[0], outs[1])
    return outs[0]


@pytest.mark.gpu
@pytest.mark.parametrize("c", CASES, ids=_ids)
def test_gpu_against_oracle(gpu, oracle_mod, c):
    cin, cout, k, s, d, p, op, g = c[:8]
    cfg = oracle_mod.make_cfg(cin, cout, k, s, d, p, g)
    for activation, with_bias in (("identity", True), ("relu", False), ("tanh", True), ("relu6", True)):
        x, w, bias = _tensors(c, 11)
        b = bias if with_bias else None
        got = _run_gpu(gpu, c, x, w, b, activation)
        np.testing.assert_allclose(got, oracle_mod.tconv2d_forward(x, w, b, cfg, _pair(op), activation), rtol=1e-4, atol=1e-4)
    x, w, bias = _tensors(c, 12, integers=True)
    assert np.array_equal(_run_gpu(gpu, c, x, w, bias, "identity"), _torch(c, x, w, bias, "identity", f64=True))


@pytest.mark.gpu
def test_gpu_batch_other_than_the_hint(gpu, oracle_mod):
    c = (16, 8, 3, 2, 1, 1, 1, 1, 5, 12, 12)
    cfg = oracle_mod.make_cfg(16, 8, 3, 2, 1, 1, 1)
    x, w, bias = _tensors(c, 21)
    got = _run_gpu(gpu, c, x, w, bias, "relu", batch_hint=8)
    np.testing.assert_allclose(got, oracle_mod.tconv2d_forward(x, w, bias, cfg, (1, 1), "relu"), rtol=1e-4, atol=1e-4)
