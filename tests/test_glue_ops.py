"""Glue operators (pooling, global pooling, elementwise): oracle pinned by the reference's
golden vectors on the CPU; HIP kernels against those goldens and the oracle on the GPU."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = dict(rtol=1e-5, atol=1e-5)


def golden_cases(name):
    doc = json.load(open(os.path.join(GOLDEN, name)))
    for t in doc["tests"]:
        for cs in t["cases"]:
            if "in" in cs:
                x = np.array(cs["in"][0], dtype=np.float32).reshape(cs["in_shapes"][0])
                y = np.array(cs["out"][0], dtype=np.float32).reshape(cs["out_shapes"][0])
                yield t["options"], x, y


def shape_cases(name):
    doc = json.load(open(os.path.join(GOLDEN, name)))
    for t in doc["tests"]:
        for cs in t["cases"]:
            yield t["options"], cs["in_shapes"][0], cs["out_shapes"][0]


# ------------------------------------------------------------------ CPU: pin the oracle
def test_oracle_pooling_reference_goldens(oracle_mod):
    n = 0
    for o, x, want in golden_cases("pooling2d_fwd.json"):
        got = oracle_mod.pool2d_forward(x, o["kernel"], o["pad"], o["stride"], o["mode"], o["count_include_pad"], o["ceil_mode"])
        assert got.shape == want.shape, (o, x.shape)
        np.testing.assert_allclose(got, want, **TOL)
        n += 1
    assert n == 96


def test_oracle_pool_output_size_matches_every_reference_shape(oracle_mod):
    n = 0
    for o, ish, osh in shape_cases("pooling2d_fwd.json"):
        k, p, s = [v if isinstance(v, list) else [v, v] for v in (o["kernel"], o["pad"], o["stride"])]
        for d in range(2):
            assert oracle_mod.pool_output_size(ish[2 + d], k[d], p[d], s[d], o["ceil_mode"]) == osh[2 + d]
        n += 1
    assert n == 144


def test_oracle_global_pooling_reference_goldens(oracle_mod):
    n = 0
    for o, x, want in golden_cases("global_pooling_fwd.json"):
        np.testing.assert_allclose(oracle_mod.global_pool_forward(x, o["mode"]), want, **TOL)
        n += 1
    assert n == 8


def test_oracle_eltwise_closed_forms(oracle_mod):
    rng = np.random.default_rng(0)
    a = rng.standard_normal(1000).astype(np.float32)
    b = rng.standard_normal(1000).astype(np.float32)
    np.testing.assert_allclose(oracle_mod.eltwise_forward(a, b, "sum", 1.0, 1.0, "relu"), np.maximum(a + b, 0), rtol=1e-6)
    np.testing.assert_allclose(oracle_mod.eltwise_forward(a, b, "sum", 2.0, -0.5), 2 * a - 0.5 * b, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle_mod.eltwise_forward(a, b, "prod", 2.0, 3.0), a * b * 6, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle_mod.eltwise_forward(a, b, "max", 1.0, 2.0), np.maximum(a, 2 * b), rtol=1e-6)


def test_pool_output_size_host_side(oracle_mod):
    import dlprimitives_amd as dlp

    for (n, k, p, s, c) in [(224, 3, 1, 2, False), (112, 3, 1, 2, False), (5, 2, 0, 2, True), (7, 3, 1, 3, True), (65, 5, 2, 4, True)]:
        assert dlp.pool2d_output_size(n, k, p, s, c) == oracle_mod.pool_output_size(n, k, p, s, c)
    assert dlp.pool2d_output_size(112, 3, 1, 2) == 56  # the ResNet stem pooling
    with pytest.raises(dlp.ValidationError):
        dlp.pool2d_output_size(2, 5, 1, 1)


# ------------------------------------------------------------------ GPU
def _dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def _make_pool(dlp, o):
    if o["mode"] == "max":
        return dlp.Pooling2DForward.create_max_pooling(o["kernel"], o["pad"], o["stride"])
    return dlp.Pooling2DForward.create_avg_pooling(o["kernel"], o["pad"], o["stride"], o["count_include_pad"])


@pytest.mark.gpu
def test_gpu_pooling_reference_goldens():
    import torch

    import dlprimitives_amd as dlp

    n = 0
    for o, x, want in golden_cases("pooling2d_fwd.json"):
        y = torch.full(want.shape, float("nan"), device="cuda:0")
        _make_pool(dlp, o).enqueue(_dev(x), y)
        torch.cuda.synchronize()
        np.testing.assert_allclose(y.cpu().numpy(), want, **TOL)
        n += 1
    assert n == 96


@pytest.mark.gpu
def test_gpu_pooling_large_shapes_vs_oracle(oracle_mod):
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(1)
    seen = 0
    for o, ish, osh in shape_cases("pooling2d_fwd.json"):
        if np.prod(ish) < 5000 or np.prod(ish) > 3e6:
            continue
        x = rng.standard_normal(ish).astype(np.float32)
        y = torch.full(tuple(osh), float("nan"), device="cuda:0")
        _make_pool(dlp, o).enqueue(_dev(x), y)
        torch.cuda.synchronize()
        want = oracle_mod.pool2d_forward(x, o["kernel"], o["pad"], o["stride"], o["mode"], o["count_include_pad"], o["ceil_mode"])
        np.testing.assert_allclose(y.cpu().numpy(), want, **TOL)
        seen += 1
    assert seen >= 20
    # the ResNet stem max pool 3x3/2 pad 1 at its real plane size
    x = rng.standard_normal((2, 64, 112, 112)).astype(np.float32)
    y = torch.empty((2, 64, 56, 56), device="cuda:0")
    dlp.Pooling2DForward.create_max_pooling(3, 1, 2).enqueue(_dev(x), y)
    torch.cuda.synchronize()
    assert np.array_equal(y.cpu().numpy(), oracle_mod.pool2d_forward(x, 3, 1, 2, "max"))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_maxpool_3x3_stride2_pad1_shapes(oracle_mod, dtype):
    """The strip kernel behind max pooling 3x3 / stride 2 / pad 1: odd and even sizes, planes smaller than a
    strip, rows shorter than a wavefront, ceil-mode output sizes, and rows of whole groups of eight columns (four outputs per lane);
    a maximum of stored values is exact."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA

    rng = np.random.default_rng(3)
    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    for (b, c, h, w, ceil_mode) in [(2, 3, 112, 112, 0), (1, 5, 7, 7, 0), (3, 2, 13, 9, 1), (2, 4, 30, 31, 0), (1, 1, 2, 2, 0), (2, 7, 15, 64, 1),
                                    (1, 2, 57, 130, 0), (2, 3, 56, 48, 0), (1, 2, 9, 8, 0), (3, 1, 113, 16, 0), (1, 65, 5, 24, 0)]:
        x = rng.standard_normal((b, c, h, w)).astype(np.float32)
        if dtype == "bfloat16":
            x = oracle_mod.bf16_round(x)
        oh = dlp.pool2d_output_size(h, 3, 1, 2, ceil_mode)
        ow = dlp.pool2d_output_size(w, 3, 1, 2, ceil_mode)
        y = torch.full((b, c, oh, ow), float("nan"), dtype=tdt, device="cuda:0")
        op = dlp.Pooling2DForward.create_max_pooling(3, 1, 2, dtype=BFLOAT16_DATA if dtype == "bfloat16" else FLOAT_DATA)
        op.enqueue(torch.from_numpy(x).cuda().to(tdt), y)
        torch.cuda.synchronize()
        want = oracle_mod.pool2d_forward(x, 3, 1, 2, "max", ceil_mode=ceil_mode)
        assert want.shape == (b, c, oh, ow)
        assert np.array_equal(y.float().cpu().numpy(), want), (b, c, h, w, ceil_mode)


@pytest.mark.gpu
def test_gpu_global_pooling(oracle_mod):
    import torch

    import dlprimitives_amd as dlp

    for o, x, want in golden_cases("global_pooling_fwd.json"):
        op = dlp.Pooling2DForward.create_global_max_pooling() if o["mode"] == "max" else dlp.Pooling2DForward.create_global_avg_pooling()
        y = torch.full(want.shape, float("nan"), device="cuda:0")
        op.enqueue(_dev(x), y)
        torch.cuda.synchronize()
        np.testing.assert_allclose(y.cpu().numpy(), want, **TOL)
    rng = np.random.default_rng(2)
    for shape in [(4, 2048, 7, 7), (3, 512, 7, 7), (2, 5, 33, 17), (1, 1, 1, 1)]:
        x = rng.standard_normal(shape).astype(np.float32)
        for mode in ("max", "avg"):
            op = dlp.Pooling2DForward.create_global_max_pooling() if mode == "max" else dlp.Pooling2DForward.create_global_avg_pooling()
            y = torch.full(shape[:2] + (1, 1), float("nan"), device="cuda:0")
            op.enqueue(_dev(x), y)
            torch.cuda.synchronize()
            np.testing.assert_allclose(y.cpu().numpy(), oracle_mod.global_pool_forward(x, mode), **TOL)


@pytest.mark.gpu
def test_gpu_eltwise(oracle_mod):
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(3)
    for n in (1, 1000, 64 * 256 * 56 * 56 // 16 + 3):
        a = rng.standard_normal(n).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        for (op, c1, c2, act) in [("sum", 1.0, 1.0, "relu"), ("sum", 0.5, -2.0, "identity"), ("prod", 2.0, 3.0, "tanh"), ("max", 1.0, 2.0, "relu6")]:
            c = torch.full((n,), float("nan"), device="cuda:0")
            dlp.eltwise_forward(_dev(a), _dev(b), c, op, c1, c2, act)
            torch.cuda.synchronize()
            np.testing.assert_allclose(c.cpu().numpy(), oracle_mod.eltwise_forward(a, b, op, c1, c2, act), rtol=1e-6, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_eltwise_alignments_and_tails(oracle_mod, dtype):
    """The 16-byte vector body, its scalar tail, and operands that are not 16-byte aligned."""
    import torch

    import dlprimitives_amd as dlp

    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(5)
    for n, off in [(4099, 0), (4099, 1), (37, 3), (8 * 1024, 0), (5, 0)]:
        a = oracle_mod.bf16_round(rng.standard_normal(n + off).astype(np.float32))
        b = oracle_mod.bf16_round(rng.standard_normal(n + off).astype(np.float32))
        ta, tb = _dev(a).to(tdt)[off:], _dev(b).to(tdt)[off:]
        c = torch.full((n + off,), float("nan"), device="cuda:0", dtype=tdt)[off:]
        dlp.eltwise_forward(ta, tb, c, "sum", 1.0, 1.0, "relu")
        torch.cuda.synchronize()
        want = oracle_mod.eltwise_forward(a[off:], b[off:], "sum", 1.0, 1.0, "relu")
        np.testing.assert_allclose(c.float().cpu().numpy(), want, rtol=2 ** -8 if dtype == "bfloat16" else 1e-6, atol=1e-6)


def test_oracle_batch_norm_matches_torch(oracle_mod):
    """The oracle's fixed-statistics batch normalisation against torch's library routine (eval mode)."""
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(11)
    x = rng.standard_normal((3, 7, 5, 4)).astype(np.float32)
    mean, var = rng.standard_normal(7).astype(np.float32), rng.uniform(0.2, 3.0, 7).astype(np.float32)
    gamma, beta = rng.standard_normal(7).astype(np.float32), rng.standard_normal(7).astype(np.float32)
    for eps in (1e-5, 1e-2):
        want = F.batch_norm(torch.from_numpy(x).double(), torch.from_numpy(mean).double(), torch.from_numpy(var).double(),
                            torch.from_numpy(gamma).double(), torch.from_numpy(beta).double(), False, 0.0, eps).numpy()
        np.testing.assert_allclose(oracle_mod.batch_norm_forward(x, mean, var, gamma, beta, eps), want, rtol=1e-5, atol=1e-5)
        want = F.batch_norm(torch.from_numpy(x).double(), torch.from_numpy(mean).double(), torch.from_numpy(var).double(), None, None, False, 0.0, eps).numpy()
        np.testing.assert_allclose(oracle_mod.batch_norm_forward(x, mean, var, eps=eps, activation="relu"), np.maximum(want, 0), rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_activation_forward(oracle_mod, dtype):
    import torch

    import dlprimitives_amd as dlp

    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(12)
    for n, off in [(1, 0), (4099, 0), (4099, 1), (37, 3), (1 << 20, 0)]:
        x = oracle_mod.bf16_round(rng.uniform(-8, 8, n + off).astype(np.float32))
        for act in ("identity", "relu", "tanh", "sigmoid", "relu6"):
            tx = _dev(x).to(tdt)[off:]
            y = torch.full((n + off,), float("nan"), device="cuda:0", dtype=tdt)[off:]
            dlp.activation_forward(tx, y, act)
            want = oracle_mod.apply_activation(x[off:], act)
            np.testing.assert_allclose(y.float().cpu().numpy(), want, rtol=2 ** -8 if dtype == "bfloat16" else 1e-6, atol=1e-6)
            dlp.activation_forward(tx, tx, act)  # in place
            np.testing.assert_array_equal(tx.float().cpu().numpy(), y.float().cpu().numpy())


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_channel_affine_is_batch_norm_with_fixed_statistics(oracle_mod, dtype):
    """Planes that are and are not a multiple of the vector width, one-element planes (after global
    pooling / inner product), more than 65535 planes, unaligned tensors, in place."""
    import torch

    import dlprimitives_amd as dlp

    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(13)
    for shape, off, act in [((2, 5, 7, 9), 0, "relu"), ((3, 16, 8, 8), 0, "identity"), ((3, 16, 8, 8), 1, "relu6"), ((4, 9), 0, "tanh"),
                            ((64, 2048, 2, 2), 0, "relu"), ((2, 3, 1, 24), 4, "sigmoid"), ((1, 1, 3, 1), 0, "identity")]:
        n = int(np.prod(shape))
        c = shape[1]
        x = oracle_mod.bf16_round(rng.standard_normal(n + off).astype(np.float32))
        mean, var = rng.standard_normal(c).astype(np.float32), rng.uniform(0.3, 2.0, c).astype(np.float32)
        gamma, beta = rng.uniform(0.5, 1.5, c).astype(np.float32), rng.standard_normal(c).astype(np.float32)
        alpha = (np.float32(1) / np.sqrt(var + np.float32(1e-5))) * gamma
        shift = gamma * (-mean * (np.float32(1) / np.sqrt(var + np.float32(1e-5)))) + beta
        tx = _dev(x).to(tdt)[off:].view(shape)
        y = torch.full((n + off,), float("nan"), device="cuda:0", dtype=tdt)[off:].view(shape)
        dlp.channel_affine_forward(tx, _dev(alpha), _dev(shift), y, act)
        want = oracle_mod.batch_norm_forward(x[off:].reshape(shape), mean, var, gamma, beta, 1e-5, act)
        np.testing.assert_allclose(y.float().cpu().numpy(), want, rtol=2 ** -7 if dtype == "bfloat16" else 1e-5, atol=2 ** -7 if dtype == "bfloat16" else 1e-5)
        dlp.channel_affine_forward(tx, _dev(alpha), _dev(shift), tx, act)
        np.testing.assert_array_equal(tx.float().cpu().numpy(), y.float().cpu().numpy())


def _softmax_cases(log):
    doc = json.load(open(os.path.join(GOLDEN, "log_softmax_fwd.json" if log else "softmax_fwd.json")))
    assert doc["operator"] == "Softmax" and doc["tests"][0]["options"] == {"log": log}
    for c in doc["tests"][0]["cases"]:
        if "in" not in c:
            continue  # the reference's "compare with the CPU operator on random inputs" cases hold no values
        shape = c["in_shapes"][0]
        yield np.asarray(c["in"][0], dtype=np.float32).reshape(shape), np.asarray(c["out"][0], dtype=np.float32).reshape(shape)


@pytest.mark.parametrize("log", [False, True])
def test_oracle_softmax_reference_goldens(oracle_mod, log):
    """The golden cases of the reference's own tests (tests/test_case_softmax.json, test_case_log_softmax.json)."""
    n = 0
    for x, want in _softmax_cases(log):
        np.testing.assert_allclose(oracle_mod.softmax_forward(x, log), want, rtol=2e-5, atol=1e-6)
        n += 1
    assert n == 46


@pytest.mark.gpu
@pytest.mark.parametrize("log", [False, True])
def test_gpu_softmax_reference_goldens(oracle_mod, log):
    import torch

    import dlprimitives_amd as dlp

    for x, want in _softmax_cases(log):
        y = torch.full(x.shape, float("nan"), device="cuda:0")
        dlp.softmax_forward(_dev(x), y, log)
        np.testing.assert_allclose(y.cpu().numpy(), want, rtol=2e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_softmax_inner_dimension_in_place(oracle_mod, dtype):
    """[B, C, S] tensors (softmax over dimension 1, as the reference does for three dimensions), in place, bfloat16 storage."""
    import torch

    import dlprimitives_amd as dlp

    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    rng = np.random.default_rng(14)
    for shape in [(3, 7, 5), (2, 100, 1), (1, 1000, 3), (5, 1, 4), (4, 65)]:
        x = oracle_mod.bf16_round(rng.standard_normal(shape).astype(np.float32) * 3)
        for log in (False, True):
            t = _dev(x).to(tdt)
            dlp.softmax_forward(t, t, log)
            want = oracle_mod.softmax_forward(x, log)
            np.testing.assert_allclose(t.float().cpu().numpy(), want, rtol=2 ** -7 if dtype == "bfloat16" else 2e-5, atol=2 ** -7 if dtype == "bfloat16" else 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "uint8"])
def test_gpu_slice_copy(dtype):
    """The copy behind Concat and Slice (core::SliceCopy::tensor_slice_copy with scale 0): ranges along every axis, rows that allow
    16-, 4-, 2- and 1-byte units; what lies outside the range of the target stays as it was."""
    import torch

    import dlprimitives_amd as dlp

    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(4)

    def rnd(shape):
        t = torch.randint(0, 200, shape, generator=g)
        return t.to(tdt).cuda()

    for shape_s, shape_d, dim, so, do, ln in [((3, 8, 5, 4), (3, 20, 5, 4), 1, 0, 12, 8), ((3, 8, 5, 4), (3, 20, 5, 4), 1, 3, 1, 5), ((2, 3, 7), (2, 3, 11), 2, 2, 4, 5),
                                              ((4, 6), (9, 6), 0, 1, 5, 3), ((2, 5, 3, 3), (2, 5, 3, 3), 1, 0, 0, 5), ((5, 1, 1), (5, 3, 1), 1, 0, 2, 1),
                                              ((2, 16, 8, 8), (2, 48, 8, 8), 1, 0, 16, 16)]:
        src, dst = rnd(shape_s), rnd(shape_d)
        want = dst.clone()
        want.narrow(dim, do, ln).copy_(src.narrow(dim, so, ln))
        dlp.slice_copy(dst, do, src, so, ln, dim)
        torch.cuda.synchronize()
        assert torch.equal(dst, want), (shape_s, shape_d, dim, so, do, ln)
    with pytest.raises(dlp.ValidationError):
        dlp.slice_copy(rnd((2, 4)), 3, rnd((2, 4)), 0, 2, 1)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_eltwise_broadcast(dtype):
    """Elementwise with inputs that broadcast (numpy's rule, src/ops/elementwise.cpp:223) against torch: per-channel and per-plane
    operands, ranks that differ, both operands broadcasting, scalars; sum / prod / max with coefficients and an activation."""
    import torch

    import dlprimitives_amd as dlp

    tdt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(9)
    shapes = [((3, 8, 5, 7), (3, 8, 1, 1)), ((3, 8, 5, 7), (1, 8, 1, 1)), ((8, 1, 1), (3, 8, 5, 7)), ((3, 1, 5, 1), (1, 8, 1, 7)), ((4, 6), (6,)),
              ((2, 3, 4, 5), (1,)), ((2, 3, 4, 5), (4, 1)), ((5, 1), (1, 9)), ((2, 1, 3, 4), (2, 5, 3, 4)), ((2, 1, 3, 1), (1, 5, 3, 6))]
    for k, (sa, sb) in enumerate(shapes):
        a = torch.randn(sa, generator=g).to(tdt).cuda()
        b = torch.randn(sb, generator=g).to(tdt).cuda()
        op = ("sum", "prod", "max")[k % 3]
        act = ("identity", "relu", "tanh")[(k // 3) % 3]
        c1, c2 = 0.5 + 0.25 * k, -1.25 + 0.5 * k
        out_shape = torch.broadcast_shapes(sa, sb)
        c = torch.full(out_shape, float("nan"), dtype=tdt, device="cuda:0")
        dlp.eltwise_forward(a, b, c, op, c1, c2, act)
        torch.cuda.synchronize()
        af, bf = a.float() * c1, b.float() * c2
        want = {"sum": af + bf, "prod": af * bf, "max": torch.maximum(af, bf)}[op]
        want = {"identity": lambda v: v, "relu": torch.relu, "tanh": torch.tanh}[act](want)
        tol = dict(rtol=1e-5, atol=1e-6) if dtype == "float32" else dict(rtol=2 ** -7, atol=2 ** -7)
        assert torch.allclose(c.float(), want.to(tdt).float() if dtype == "bfloat16" else want, **tol), (sa, sb, op, act)
    a = torch.zeros((2, 3), device="cuda:0")
    with pytest.raises(dlp.ValidationError):
        dlp.eltwise_forward(a, torch.zeros((2, 4), device="cuda:0"), torch.zeros((2, 4), device="cuda:0"))
    with pytest.raises(dlp.NotImplementedErrorDlprim):  # five runs of dimensions that alternate between the operands
        dlp.eltwise_forward(torch.zeros((2, 1, 2, 1, 2), device="cuda:0"), torch.zeros((1, 2, 1, 2, 1), device="cuda:0"), torch.zeros((2, 2, 2, 2, 2), device="cuda:0"))

