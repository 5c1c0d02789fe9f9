"""Pins the CPU oracle (oracle/dlp_oracle.c) before anything is compared with it.

Each oracle function is checked against something that is NOT a retyping of its
own formula: the reference's golden vectors, the reference's own BLAS/activation
code compiled into oracle/_ref, an independent direct convolution in double, the
library routine torch.nn.functional.conv2d (the truth of the reference's own
fixture generator), and closed forms.
"""
import json
import os

import numpy as np
import pytest
import torch

from conv_cases import REFERENCE_MATRIX, case_id, make_tensors, small_cases

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def cfg_of(orc, c):
    return orc.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])


def torch_conv(x, w, bias, c):
    y = torch.nn.functional.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(),
                                   None if bias is None else torch.from_numpy(bias).double(),
                                   stride=c["stride"], padding=c["pad"], dilation=c["dilate"], groups=c["groups"])
    if c["activation"] == "relu":
        y = torch.relu(y)
    return y.numpy()


# ---------------------------------------------------------------- output shape
@pytest.mark.parametrize("c", REFERENCE_MATRIX, ids=case_id)
def test_output_shape_matches_torch(oracle_mod, c):
    for (b, h, w) in [(1, 32, 32), (2, 19, 21), (3, 57, 40)]:
        if h + 2 * c["pad"][0] < c["dilate"][0] * (c["kernel"][0] - 1) + 1:
            continue
        if w + 2 * c["pad"][1] < c["dilate"][1] * (c["kernel"][1] - 1) + 1:
            continue
        want = torch.nn.functional.conv2d(torch.zeros(b, c["cin"], h, w), torch.zeros(c["cout"], c["cin"] // c["groups"], *c["kernel"]),
                                          stride=c["stride"], padding=c["pad"], dilation=c["dilate"], groups=c["groups"]).shape
        assert oracle_mod.conv2d_output_shape(cfg_of(oracle_mod, c), (b, c["cin"], h, w)) == tuple(want)


def test_output_shape_closed_form_and_errors(oracle_mod):
    # ResNet stem 7x7/2 pad 3: 224 -> 112 ; 3x3/2 pad 1: 56 -> 28 ; 1x1/2: 56 -> 28
    assert oracle_mod.conv2d_output_shape(oracle_mod.make_cfg(3, 64, 7, 2, 1, 3), (64, 3, 224, 224)) == (64, 64, 112, 112)
    assert oracle_mod.conv2d_output_shape(oracle_mod.make_cfg(64, 128, 3, 2, 1, 1), (1, 64, 56, 56)) == (1, 128, 28, 28)
    assert oracle_mod.conv2d_output_shape(oracle_mod.make_cfg(64, 128, 1, 2, 1, 0), (1, 64, 56, 56)) == (1, 128, 28, 28)
    with pytest.raises(ValueError):  # channel mismatch
        oracle_mod.conv2d_output_shape(oracle_mod.make_cfg(3, 8, 3), (1, 4, 8, 8))
    with pytest.raises(ValueError):  # kernel larger than padded input
        oracle_mod.conv2d_output_shape(oracle_mod.make_cfg(3, 8, 5), (1, 3, 2, 2))


# ---------------------------------------------------------------- activations
def test_activation_reference_goldens(oracle_mod):
    doc = json.load(open(os.path.join(GOLDEN, "activation_fwd.json")))
    n = 0
    for t in doc["tests"]:
        for cs in t["cases"]:
            if "in" not in cs:
                continue
            got = oracle_mod.apply_activation(np.array(cs["in"][0], dtype=np.float32), t["options"]["activation"])
            np.testing.assert_allclose(got, np.array(cs["out"][0], dtype=np.float32), rtol=1e-6, atol=1e-6)
            n += 1
    assert n >= 5


@pytest.mark.parametrize("act", ["identity", "relu", "tanh", "sigmoid", "relu6"])
def test_activation_bit_exact_vs_compiled_reference(oracle_mod, act):
    if oracle_mod.ref() is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    x = np.random.default_rng(5).uniform(-9, 9, size=4097).astype(np.float32)
    assert np.array_equal(oracle_mod.apply_activation(x, act), oracle_mod.ref_apply_activation(x, act))


# ---------------------------------------------------------------- sgemm
@pytest.mark.parametrize("mnk", [(1, 1, 1), (3, 5, 7), (64, 50, 576), (17, 129, 33), (128, 31, 1)])
@pytest.mark.parametrize("beta", [0.0, 2.0])
def test_sgemm_nt_bit_exact_vs_compiled_reference(oracle_mod, mnk, beta):
    if oracle_mod.ref() is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    M, N, K = mnk
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    A = rng.standard_normal((M, K)).astype(np.float32)
    B = rng.standard_normal((N, K)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    got = oracle_mod.sgemm_nt(A, B, C0, alpha=1.0, beta=beta)
    want = oracle_mod.ref_sgemm(A, B, False, True, C0, alpha=1.0, beta=beta)
    assert np.array_equal(got, want)


def test_sgemm_nt_integer_exact(oracle_mod):
    # integer-valued inputs make fp32 exact whatever the summation order
    # (the property the reference's tests/test_gemm.cpp:40-117 relies on)
    rng = np.random.default_rng(11)
    A = np.round(rng.standard_normal((37, 91)) * 3).astype(np.float32)
    B = np.round(rng.standard_normal((53, 91)) * 3).astype(np.float32)
    want = (A.astype(np.int64) @ B.astype(np.int64).T).astype(np.float32)
    assert np.array_equal(oracle_mod.sgemm_nt(A, B), want)


# ---------------------------------------------------------------- im2col + conv
def test_im2col_column_order(oracle_mod):
    # a one-hot image makes every matrix entry name its own source pixel
    cfg = oracle_mod.make_cfg(2, 1, (2, 3), (1, 2), (2, 1), (1, 1))
    H, W = 5, 6
    img = np.arange(2 * H * W, dtype=np.float32).reshape(2, H, W) + 1
    OH, OW = oracle_mod.conv2d_output_shape(cfg, (1, 2, H, W))[2:]
    mat = oracle_mod.im2col(img, cfg, (OH, OW))
    for r in range(OH):
        for c in range(OW):
            for ch in range(2):
                for ky in range(2):
                    for kx in range(3):
                        y, x = r * 1 - 1 + ky * 2, c * 2 - 1 + kx * 1
                        want = img[ch, y, x] if 0 <= y < H and 0 <= x < W else 0.0
                        assert mat[r * OW + c, ch * 6 + ky * 3 + kx] == want


@pytest.mark.parametrize("c,bhw", small_cases(), ids=case_id)
def test_conv_vs_direct_f64_and_torch(oracle_mod, c, bhw):
    x, w, bias = make_tensors(c, bhw, seed=1234)
    cfg = cfg_of(oracle_mod, c)
    got = oracle_mod.conv2d_forward(x, w, bias, cfg, c["activation"])
    direct = oracle_mod.conv2d_direct_f64(x, w, bias, cfg, c["activation"])
    lib = torch_conv(x, w, bias, c)
    assert got.shape == lib.shape
    np.testing.assert_allclose(direct, lib, rtol=1e-9, atol=1e-9)
    np.testing.assert_allclose(got, lib, rtol=2e-5, atol=2e-5)


def test_conv_1x1_is_matmul_and_delta_is_shift(oracle_mod):
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (2, 6, 5, 7)).astype(np.float32)
    w = rng.standard_normal((4, 6, 1, 1)).astype(np.float32)
    y = oracle_mod.conv2d_forward(x, w, None, oracle_mod.make_cfg(6, 4, 1))
    want = np.einsum("oc,bchw->bohw", w[:, :, 0, 0].astype(np.float64), x.astype(np.float64))
    np.testing.assert_allclose(y, want, rtol=1e-5, atol=1e-6)
    # 3x3 kernel with a single 1 at (ky,kx) = (0,2), pad 1: y[r,c] = x[r-1,c+1]
    wd = np.zeros((1, 1, 3, 3), dtype=np.float32)
    wd[0, 0, 0, 2] = 1
    xs = rng.uniform(-1, 1, (1, 1, 6, 6)).astype(np.float32)
    ys = oracle_mod.conv2d_forward(xs, wd, None, oracle_mod.make_cfg(1, 1, 3, 1, 1, 1))
    want = np.zeros_like(xs)
    want[0, 0, 1:, :-1] = xs[0, 0, :-1, 1:]
    assert np.array_equal(ys, want)


def test_conv_multithreaded_equals_single(oracle_mod):
    c = REFERENCE_MATRIX[13]
    x, w, bias = make_tensors(c, (5, 9, 11), seed=8)
    cfg = cfg_of(oracle_mod, c)
    assert np.array_equal(oracle_mod.conv2d_forward(x, w, bias, cfg, "relu6", threads=1),
                          oracle_mod.conv2d_forward(x, w, bias, cfg, "relu6", threads=3))


def test_factor_contract(oracle_mod):
    rng = np.random.default_rng(2)
    new = rng.standard_normal(100).astype(np.float32)
    old = rng.standard_normal(100).astype(np.float32)
    assert np.array_equal(oracle_mod.apply_factor(new, old, 0.0), new)
    np.testing.assert_allclose(oracle_mod.apply_factor(new, old, 0.5), old * 0.5 + new, rtol=1e-6)


# ---------------------------------------------------------------- inner product
def test_inner_product_reference_goldens(oracle_mod):
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
            got = oracle_mod.ip_forward(x, w, bias, o["activation"])
            np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
            n += 1
    assert n == 28


# ---------------------------------------------------------------- winograd
def test_winograd_filter_transform_vs_published_matrices(oracle_mod):
    G = np.array([[1, 0, 0], [0.5, 0.5, 0.5], [0.5, -0.5, 0.5], [0, 0, 1]], dtype=np.float64)
    w = np.random.default_rng(4).standard_normal((5, 3, 3, 3)).astype(np.float32)
    u = oracle_mod.winograd_filter_transform(w).reshape(5, 3, 4, 4)
    want = np.einsum("ij,ncjk,lk->ncil", G, w.astype(np.float64), G)
    np.testing.assert_allclose(u, want, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape", [(1, 1, 1, 4, 4), (2, 3, 5, 7, 9), (1, 16, 8, 14, 14), (3, 8, 16, 5, 6), (1, 4, 4, 1, 1)])
@pytest.mark.parametrize("act", ["identity", "relu"])
def test_winograd_equals_direct(oracle_mod, shape, act):
    B, C, N, H, W = shape
    rng = np.random.default_rng(B + C + N + H)
    x = rng.uniform(-1, 1, (B, C, H, W)).astype(np.float32)
    w = (rng.standard_normal((N, C, 3, 3)) * np.sqrt(2 / (9 * C))).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, N).astype(np.float32)
    want = oracle_mod.conv2d_direct_f64(x, w, bias, oracle_mod.make_cfg(C, N, 3, 1, 1, 1), act)
    got = oracle_mod.winograd_forward(x, w, bias, act)
    np.testing.assert_allclose(got, want, rtol=1e-4, atol=2e-5)
    old = rng.standard_normal(got.shape).astype(np.float32)
    got2 = oracle_mod.winograd_forward(x, w, bias, act, factor=0.5, y_old=old)
    np.testing.assert_allclose(got2, old * 0.5 + got, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- depthwise
@pytest.mark.parametrize("shape", [(2, 5, 7, 9, 3), (1, 8, 14, 14, 3), (1, 3, 6, 5, 5), (2, 4, 1, 1, 3)])
def test_depthwise_equals_grouped_conv(oracle_mod, shape):
    B, C, H, W, K = shape
    rng = np.random.default_rng(C * H)
    x = rng.uniform(-1, 1, (B, C, H, W)).astype(np.float32)
    w = rng.standard_normal((C, 1, K, K)).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, C).astype(np.float32)
    want = oracle_mod.conv2d_direct_f64(x, w, bias, oracle_mod.make_cfg(C, C, K, 1, 1, K // 2, C), "relu6")
    got = oracle_mod.depthwise_forward(x, w, bias, "relu6")
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)


def test_bf16_round_matches_torch(oracle_mod):
    x = np.random.default_rng(9).standard_normal(10000).astype(np.float32) * 100
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(oracle_mod.bf16_round(x), want)


# ---------------------------------------------------------------- backward (the gradient operators)
@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("mnk", [(1, 1, 1), (3, 5, 7), (24, 50, 36), (17, 129, 33)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_sgemm_nn_tn_bit_exact_vs_compiled_reference(oracle_mod, mnk, beta, ta):
    if oracle_mod.ref() is None:
        pytest.skip("oracle/_ref not built (reference tree absent)")
    M, N, K = mnk
    rng = np.random.default_rng(M * 1000 + N * 10 + K)
    A = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    B = rng.standard_normal((K, N)).astype(np.float32)
    C0 = rng.standard_normal((M, N)).astype(np.float32)
    got = oracle_mod.sgemm(A, B, ta, False, C0, alpha=1.0, beta=beta)
    want = oracle_mod.ref_sgemm(A, B, ta, False, C0, alpha=1.0, beta=beta)
    assert np.array_equal(got, want)
    np.testing.assert_allclose(got, (A.T if ta else A).astype(np.float64) @ B + beta * C0, rtol=1e-4, atol=1e-4)


def torch_conv_grads(x, w, dy, c):
    xt = torch.from_numpy(x).double().requires_grad_(True)
    wt = torch.from_numpy(w).double().requires_grad_(True)
    y = torch.nn.functional.conv2d(xt, wt, None, stride=c["stride"], padding=c["pad"], dilation=c["dilate"], groups=c["groups"])
    y.backward(torch.from_numpy(dy).double())
    return xt.grad.numpy(), wt.grad.numpy()


@pytest.mark.parametrize("c,bhw", small_cases(), ids=case_id)
def test_conv_backward_vs_torch_autograd(oracle_mod, c, bhw):
    """Both gradient restatements against torch's autograd of the library convolution, and the
    accumulate contract (result = factor * old + gradient) against the same."""
    x, w, _ = make_tensors(c, bhw, seed=4321)
    cfg = cfg_of(oracle_mod, c)
    rng = np.random.default_rng(99)
    dy = rng.standard_normal(oracle_mod.conv2d_output_shape(cfg, x.shape)).astype(np.float32)
    want_dx, want_dw = torch_conv_grads(x, w, dy, c)
    dx = oracle_mod.conv2d_backward_data(dy, w, cfg, x.shape)
    dw = oracle_mod.conv2d_backward_filter(dy, x, cfg)
    np.testing.assert_allclose(dx, want_dx, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(want_dx).max()))
    np.testing.assert_allclose(dw, want_dw, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(want_dw).max()))
    old_dx = rng.standard_normal(x.shape).astype(np.float32)
    old_dw = rng.standard_normal(w.shape).astype(np.float32)
    dx2 = oracle_mod.conv2d_backward_data(dy, w, cfg, x.shape, old_dx, 0.5)
    dw2 = oracle_mod.conv2d_backward_filter(dy, x, cfg, old_dw, -2.0)
    np.testing.assert_allclose(dx2, want_dx + 0.5 * old_dx, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(want_dx).max()))
    np.testing.assert_allclose(dw2, want_dw - 2.0 * old_dw, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(want_dw).max()))


def test_conv_backward_is_the_adjoint_of_forward(oracle_mod):
    """<dy, conv(x, w)> = <backward_data(dy, w), x> = <backward_filter(dy, x), w>: the forward oracle is
    pinned by the reference's goldens; the identities tie both gradients to it without any formula."""
    rng = np.random.default_rng(5)
    for (cin, cout, k, s, d, p, g, hw) in [(4, 6, 3, 2, 1, 1, 2, (9, 8)), (3, 5, (2, 3), (1, 2), (2, 1), (1, 2), 1, (7, 10)), (8, 8, 3, 1, 1, 1, 8, (6, 6))]:
        cfg = oracle_mod.make_cfg(cin, cout, k, s, d, p, g)
        kh, kw = (k, k) if isinstance(k, int) else k
        x = np.round(rng.standard_normal((2, cin) + hw) * 4).astype(np.float32)
        w = np.round(rng.standard_normal((cout, cin // g, kh, kw)) * 4).astype(np.float32)
        y = oracle_mod.conv2d_forward(x, w, None, cfg)
        dy = np.round(rng.standard_normal(y.shape) * 4).astype(np.float32)
        lhs = float((dy.astype(np.float64) * y).sum())
        # integer-valued tensors: every sum is exact in fp32, so the identities hold exactly
        assert float((oracle_mod.conv2d_backward_data(dy, w, cfg, x.shape).astype(np.float64) * x).sum()) == lhs
        assert float((oracle_mod.conv2d_backward_filter(dy, x, cfg).astype(np.float64) * w).sum()) == lhs


def test_bias_backward_closed_form(oracle_mod):
    rng = np.random.default_rng(6)
    dy = np.round(rng.standard_normal((3, 5, 4, 7)) * 8).astype(np.float32)
    old = np.round(rng.standard_normal(5) * 8).astype(np.float32)
    assert np.array_equal(oracle_mod.bias_backward(dy), dy.sum((0, 2, 3)))
    assert np.array_equal(oracle_mod.bias_backward(dy, old, 2.0), dy.sum((0, 2, 3)) + 2 * old)
    assert np.array_equal(oracle_mod.bias_backward(dy[:, :, 0, 0]), dy[:, :, 0, 0].sum(0))
