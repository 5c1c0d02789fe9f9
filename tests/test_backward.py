"""Convolution gradients (dlp_conv2d_bwd_data_*, dlp_conv2d_bwd_filter_*, dlp_bias_bwd_enqueue) against the
CPU oracle's restatement of Convolution2D::backward_data_cpu / backward_filter_cpu / BWBias::backward_cpu,
on the geometry matrix of the reference's own convolution tests, and at ResNet-18 layer sizes through the
identities <dy, conv(x, w)> = <backward_data(dy, w), x> = <backward_filter(dy, x), w>, which need no oracle
run (the forward operator is checked separately).  Tolerance 1e-4 of the result's largest magnitude.
"""
import numpy as np
import pytest

from conv_cases import REFERENCE_MATRIX, case_id, make_tensors, small_cases

TOL = 1e-4


def _dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def _settings(dlp, c, shape):
    return dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], shape)


def _ws(torch, nbytes):
    return torch.empty(max(nbytes, 1), dtype=torch.uint8, device="cuda:0")


def _close(got, want, what):
    scale = max(float(np.abs(want).max()), 1e-6)
    err = float(np.abs(got - want).max()) / scale
    assert err < TOL, (what, err)


def test_backward_symbols_are_exported():
    import dlprimitives_amd as dlp

    for name in ("dlp_conv2d_bwd_data_create", "dlp_conv2d_bwd_data_algo", "dlp_conv2d_bwd_data_workspace", "dlp_conv2d_bwd_data_enqueue",
                 "dlp_conv2d_bwd_data_destroy", "dlp_conv2d_bwd_filter_create", "dlp_conv2d_bwd_filter_algo", "dlp_conv2d_bwd_filter_workspace",
                 "dlp_conv2d_bwd_filter_enqueue", "dlp_conv2d_bwd_filter_destroy", "dlp_bias_bwd_enqueue"):
        assert hasattr(dlp.lib(), name)


def test_backward_create_rejects_bad_arguments():
    """Rejected before anything touches a device."""
    import dlprimitives_amd as dlp

    s = dlp.Conv2DSettings(8, 16, 3, 2, 1, 1, 1, (4, 8, 17, 17))
    with pytest.raises(dlp.ValidationError):
        dlp.Conv2DBackwardData.create(dlp.Conv2DSettings(8, 16, 3, 1, 1, 1, 3, (1, 8, 8, 8)))
    with pytest.raises(dlp.ValidationError):
        dlp.Conv2DBackwardFilter.create(s, "fft")
    with pytest.raises(dlp.NotImplementedErrorDlprim):
        dlp.Conv2DBackwardData.create(dlp.Conv2DSettings(8, 16, 1, 1, 1, 1, 1, (1, 8, 8, 8)))  # stride 1 with pad > dilate * (kernel - 1)
    with pytest.raises(dlp.NotImplementedErrorDlprim):
        dlp.Conv2DBackwardFilter.create(dlp.Conv2DSettings(8, 16, 3, 1, 1, 1, 1, (1, 8, 8, 8), dtype=dlp.capi.BFLOAT16_DATA))
    f = dlp.Conv2DBackwardFilter.create(s)
    assert f.algo() == "gemm" and f.workspace() > 0


@pytest.mark.gpu
def test_gpu_backward_data_workspace():
    import dlprimitives_amd as dlp

    s = dlp.Conv2DSettings(8, 16, 3, 2, 1, 1, 1, (4, 8, 17, 17))
    d = dlp.Conv2DBackwardData.create(s)
    assert d.algo() in ("gemm", "winograd", "depthwise_separable")
    # the four stride phases of dx (4 x 8 x 17 x 17 floats in all) and their filters (16 x 8 x 9 taps in all)
    assert d.workspace() >= 4 * 8 * 17 * 17 * 4 + 16 * 8 * 9 * 4


def _run_case(dlp, torch, oracle_mod, c, bhw, seed, factor_dx=0.0, factor_dw=0.0, algo=""):
    x, w, _ = make_tensors(c, bhw, seed=seed)
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    rng = np.random.default_rng(seed + 1)
    dy = rng.standard_normal(oracle_mod.conv2d_output_shape(cfg, x.shape)).astype(np.float32)
    old_dx = rng.standard_normal(x.shape).astype(np.float32)
    old_dw = rng.standard_normal(w.shape).astype(np.float32)
    s = _settings(dlp, c, x.shape)
    out = {}
    strided = c["stride"] != (1, 1)
    if strided or (c["pad"][0] <= c["dilate"][0] * (c["kernel"][0] - 1) and c["pad"][1] <= c["dilate"][1] * (c["kernel"][1] - 1)):
        op = dlp.Conv2DBackwardData.create(s, algo)
        dx = _dev(old_dx) if factor_dx else torch.full(x.shape, float("nan"), device="cuda:0")
        op.enqueue(dx, _dev(w), _dev(dy), _ws(torch, op.workspace()), factor_dx)
        want = oracle_mod.conv2d_backward_data(dy, w, cfg, x.shape, old_dx if factor_dx else None, factor_dx)
        _close(dx.cpu().numpy(), want, "dx")
        out["dx"] = op.algo()
    op = dlp.Conv2DBackwardFilter.create(s, algo)
    dw = _dev(old_dw) if factor_dw else torch.full(w.shape, float("nan"), device="cuda:0")
    op.enqueue(_dev(x), dw, _dev(dy), _ws(torch, op.workspace()), factor_dw)
    want = oracle_mod.conv2d_backward_filter(dy, x, cfg, old_dw if factor_dw else None, factor_dw)
    _close(dw.cpu().numpy(), want, "dw")
    return out


@pytest.mark.gpu
@pytest.mark.parametrize("c,bhw", small_cases(1e7), ids=case_id)
def test_gpu_backward_reference_matrix(oracle_mod, c, bhw):
    import torch

    import dlprimitives_amd as dlp

    _run_case(dlp, torch, oracle_mod, c, bhw, 77)


@pytest.mark.gpu
@pytest.mark.parametrize("algo", ["", "gemm", "winograd", "depthwise_separable"])
def test_gpu_backward_accumulates_with_factor(oracle_mod, algo):
    """result = factor * old + gradient (src/ops/conv2d.cpp:426-435), for every algorithm name."""
    import torch

    import dlprimitives_amd as dlp

    for c, bhw in [(REFERENCE_MATRIX[5], (2, 10, 10)), (REFERENCE_MATRIX[14], (2, 19, 19)), (REFERENCE_MATRIX[15], (3, 20, 20))]:
        _run_case(dlp, torch, oracle_mod, c, bhw, 5, factor_dx=0.5, factor_dw=-2.0, algo=algo)
        _run_case(dlp, torch, oracle_mod, c, bhw, 6, factor_dx=1.0, factor_dw=1.0, algo=algo)


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(6, 6, 1, 1, 1, (3, 9, 11)), (4, 8, 2, 1, 1, (2, 12, 7)), (5, 5, 1, 2, 1, (70, 8, 8)), (3, 12, 1, 1, 0, (1, 5, 5)),
                                   (16, 16, (2, 1), (1, 2), (2, 0), (2, 17, 20))], ids=str)
def test_gpu_depthwise_backward(oracle_mod, shape):
    """One input channel per group (channel multiplier 1, 2, 4), strides, dilation, more images than slices."""
    import torch

    import dlprimitives_amd as dlp
    from conv_cases import case

    cin, cout, stride, dilate, pad, bhw = shape
    c = case(3, pad, stride, dilate, cin, cout, False, cin, False)
    _run_case(dlp, torch, oracle_mod, c, bhw, 21)
    _run_case(dlp, torch, oracle_mod, c, bhw, 22, factor_dx=0.5, factor_dw=2.0)


@pytest.mark.gpu
@pytest.mark.parametrize("geom", [(3, 2, 1, 1, 9), (3, 2, 1, 1, 10), (3, 2, 1, 0, 9), (1, 2, 1, 0, 9), (1, 2, 1, 0, 10), (5, 3, 1, 2, 11), (5, 2, 2, 3, 13),
                                  (3, 3, 2, 5, 9), (4, 2, 1, 1, 8), (2, 4, 1, 0, 11), (7, 2, 1, 3, 20), ((3, 5), (2, 3), (3, 2), (1, 2), 17),
                                  ((1, 3), (2, 1), (1, 1), (0, 1), 8), (3, (1, 2), 1, 1, 7)], ids=str)
def test_gpu_strided_backward_data_phases(oracle_mod, geom):
    """Strides, dilations and paddings that give phases with no, one and several taps, phases that start
    before or after dy's first row, rows of dx the forward window never reached, padding beyond the filter."""
    import torch

    import dlprimitives_amd as dlp
    from conv_cases import case

    k, s, d, p, hw = geom
    for groups, cin, cout in ((1, 5, 7), (2, 4, 6)):
        c = case(k, p, s, d, cin, cout, False, groups, False)
        _run_case(dlp, torch, oracle_mod, c, (2, hw, hw + 3), 31)
        _run_case(dlp, torch, oracle_mod, c, (3, hw + 2, hw), 32, factor_dx=-0.5, factor_dw=0.0)


LAYERS = [  # ResNet-18 / MobileNet-v2 layer shapes: cin, cout, k, s, p, groups, H, batch
    (64, 64, 3, 1, 1, 1, 56, 16),
    (64, 128, 3, 2, 1, 1, 56, 16),
    (64, 128, 1, 2, 0, 1, 56, 16),
    (256, 512, 3, 2, 1, 1, 14, 16),
    (512, 512, 3, 1, 1, 1, 7, 16),
    (3, 64, 7, 2, 3, 1, 224, 4),
    (144, 144, 3, 2, 1, 144, 56, 8),
    (32, 192, 1, 1, 0, 1, 28, 16),
]


@pytest.mark.gpu
@pytest.mark.parametrize("layer", LAYERS, ids=lambda l: "c%d_o%d_k%d_s%d_g%d_h%d_b%d" % (l[0], l[1], l[2], l[3], l[5], l[6], l[7]))
def test_gpu_backward_is_the_adjoint_of_forward_at_layer_sizes(layer):
    """Integer-valued tensors small enough that every product sum is exact in fp32: the three inner
    products must then agree to the last bit, whatever the order of summation."""
    import torch

    import dlprimitives_amd as dlp

    cin, cout, k, s, p, g, H, B = layer
    rng = np.random.default_rng(cin * 7 + cout)
    x = rng.integers(-2, 3, (B, cin, H, H)).astype(np.float32)
    w = rng.integers(-2, 3, (cout, cin // g, k, k)).astype(np.float32)
    st = dlp.Conv2DSettings(cin, cout, k, s, 1, p, g, x.shape)
    oshape = dlp.conv2d_output_shape(st, x.shape)
    dy = rng.integers(-1, 2, oshape).astype(np.float32)
    tx, tw, tdy = _dev(x), _dev(w), _dev(dy)
    fwd = dlp.Conv2DForward.create(st, False, "identity", "gemm")
    y = torch.empty(oshape, device="cuda:0")
    fwd.enqueue(tx, tw, None, y, _ws(torch, fwd.workspace()))
    lhs = float((y.double() * tdy.double()).sum())
    bd = dlp.Conv2DBackwardData.create(st)
    dx = torch.full(x.shape, float("nan"), device="cuda:0")
    bd.enqueue(dx, tw, tdy, _ws(torch, bd.workspace()))
    bf = dlp.Conv2DBackwardFilter.create(st)
    dw = torch.full(w.shape, float("nan"), device="cuda:0")
    bf.enqueue(tx, dw, tdy, _ws(torch, bf.workspace()))
    assert float((dx.double() * tx.double()).sum()) == lhs
    assert float((dw.double() * tw.double()).sum()) == lhs
    # a second run into the same tensors gives the same bits (the reduction order is fixed)
    dw2 = torch.full(w.shape, float("nan"), device="cuda:0")
    bf.enqueue(tx, dw2, tdy, _ws(torch, bf.workspace()))
    assert torch.equal(dw, dw2)


@pytest.mark.gpu
def test_gpu_backward_filter_batch_other_than_planned(oracle_mod):
    """The workspace was sized for the batch in the settings; other batches run with it, batch 0 scales."""
    import torch

    import dlprimitives_amd as dlp

    c = REFERENCE_MATRIX[5]
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    s = _settings(dlp, c, (2, c["cin"], 12, 12))
    op = dlp.Conv2DBackwardFilter.create(s)
    ws = _ws(torch, op.workspace())
    rng = np.random.default_rng(3)
    for batch in (1, 2, 5):
        x = rng.standard_normal((batch, c["cin"], 12, 12)).astype(np.float32)
        dy = rng.standard_normal((batch, c["cout"], 12, 12)).astype(np.float32)
        dw = torch.full((c["cout"], c["cin"], 3, 3), float("nan"), device="cuda:0")
        op.enqueue(_dev(x), dw, _dev(dy), ws)
        _close(dw.cpu().numpy(), oracle_mod.conv2d_backward_filter(dy, x, cfg), "dw batch %d" % batch)
    old = rng.standard_normal((c["cout"], c["cin"], 3, 3)).astype(np.float32)
    dw = _dev(old)
    op.enqueue(torch.empty((0, c["cin"], 12, 12), device="cuda:0"), dw, torch.empty((0, c["cout"], 12, 12), device="cuda:0"), ws, 0.5)
    np.testing.assert_array_equal(dw.cpu().numpy(), old * np.float32(0.5))


@pytest.mark.gpu
def test_gpu_bias_backward(oracle_mod):
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(8)
    for shape in [(3, 5, 4, 7), (16, 64, 56, 56), (7, 10), (1, 1, 1, 1), (2, 1000, 1, 1)]:
        dy = rng.standard_normal(shape).astype(np.float32)
        old = rng.standard_normal(shape[1]).astype(np.float32)
        db = torch.full((shape[1],), float("nan"), device="cuda:0")
        dlp.bias_backward(_dev(dy), db)
        want = dy.astype(np.float64).sum(tuple(i for i in range(len(shape)) if i != 1))
        np.testing.assert_allclose(db.cpu().numpy(), want, rtol=1e-4, atol=1e-4 * np.abs(want).max())
        np.testing.assert_allclose(db.cpu().numpy(), oracle_mod.bias_backward(dy), rtol=1e-4, atol=1e-4 * np.abs(want).max())
        db = _dev(old)
        dlp.bias_backward(_dev(dy), db, 2.0)
        np.testing.assert_allclose(db.cpu().numpy(), want + 2 * old, rtol=1e-4, atol=1e-4 * np.abs(want).max())
