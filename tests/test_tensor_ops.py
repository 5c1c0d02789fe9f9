"""Interpolation, Reduction, the three losses, and the pointwise / Concat / Slice goldens: the oracle pinned on the CPU by the
reference's golden vectors and by torch; the HIP kernels against the same goldens and, on larger shapes, against the oracle."""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
TOL = dict(rtol=1e-5, atol=1e-5)
BF16_TOL = dict(rtol=1.0 / 128, atol=1e-2)  # one bfloat16 rounding of the result (8 bits of mantissa)


def golden(name):
    """(options, [inputs], [outputs]) of every case of a fixture that carries tensors"""
    doc = json.load(open(os.path.join(GOLDEN, name)))
    for t in doc["tests"]:
        for cs in t["cases"]:
            if "in" in cs:
                xs = [np.array(v, dtype=np.float32).reshape(s) for v, s in zip(cs["in"], cs["in_shapes"])]
                ys = [np.array(v, dtype=np.float32).reshape(s) for v, s in zip(cs["out"], cs["out_shapes"])]
                yield t["options"], xs, ys


def interp_args(o):
    return dict(method=o["method"], scale=(o["scale_y"], o["scale_x"]), align_corners=o["align_corners"])


def reduce_args(o):
    return dict(method=o["method"], dims=o.get("dims"), start_axis=o.get("start_axis", 0), output_scale=o.get("output_scale", 1.0))


# ------------------------------------------------------------------ CPU: pin the oracle
def test_oracle_interpolation_reference_goldens(oracle_mod):
    n = 0
    for o, (x,), (want,) in golden("interpolation_fwd.json"):
        hw = oracle_mod.interpolate_output_size(x.shape[2:], (o["out_h"], o["out_w"]), (o["scale_y"], o["scale_x"]))
        assert hw == want.shape[2:]
        got = oracle_mod.interpolate2d_forward(x, hw, **interp_args(o))
        np.testing.assert_allclose(got, want, **TOL)
        n += 1
    assert n == 84


@pytest.mark.parametrize("method,align", [("nearest", False), ("nearest-exact", False), ("bilinear", False), ("bilinear", True)])
def test_oracle_interpolation_matches_torch(oracle_mod, method, align):
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(5)
    for (H, W), (OH, OW) in [((5, 7), (10, 14)), ((9, 6), (4, 11)), ((16, 16), (37, 23)), ((3, 300), (7, 129)), ((1, 1), (4, 4))]:
        x = rng.standard_normal((2, 3, H, W)).astype(np.float32)
        kw = dict(align_corners=align) if method == "bilinear" else {}
        want = F.interpolate(torch.from_numpy(x), size=(OH, OW), mode=method, **kw).numpy()
        got = oracle_mod.interpolate2d_forward(x, (OH, OW), method=method, align_corners=align)
        np.testing.assert_allclose(got, want, **TOL)
    # an explicit scale: the step is 1 / scale, the size int(in * scale)
    x = rng.standard_normal((1, 2, 7, 9)).astype(np.float32)
    hw = oracle_mod.interpolate_output_size((7, 9), scale=(3.4, 0.7))
    assert hw == (23, 6)
    kw = dict(align_corners=align) if method == "bilinear" else {}
    want = F.interpolate(torch.from_numpy(x), scale_factor=(3.4, 0.7), mode=method, **kw).numpy()
    np.testing.assert_allclose(oracle_mod.interpolate2d_forward(x, hw, method=method, scale=(3.4, 0.7), align_corners=align), want, **TOL)


def test_oracle_reduction_reference_goldens(oracle_mod):
    n = 0
    for o, (x,), (want,) in golden("reduction_fwd.json"):
        got = oracle_mod.reduction_forward(x, keep_dim=o["keep_dim"], **reduce_args(o))
        assert got.shape == want.shape
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
        n += 1
    assert n >= 128


def test_oracle_reduction_against_float64(oracle_mod):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 5, 7, 4)).astype(np.float32)
    x64 = x.astype(np.float64)
    np.testing.assert_allclose(oracle_mod.reduction_forward(x, "sum", dims=[1, 3], keep_dim=False), x64.sum(axis=(1, 3)), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle_mod.reduction_forward(x, "sumsq", dims=[0], keep_dim=True), (x64**2).sum(axis=0, keepdims=True), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle_mod.reduction_forward(x, "abssum", start_axis=2, keep_dim=False), np.abs(x64).sum(axis=(2, 3)), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle_mod.reduction_forward(x, "mean", start_axis=-1, output_scale=0.5, keep_dim=False), 0.5 * x64.mean(axis=3), rtol=1e-5,
                               atol=1e-6)
    assert oracle_mod.reduction_forward(x, "sum", keep_dim=False).shape == (1,)


def test_oracle_losses_reference_goldens(oracle_mod):
    n = 0
    for o, (a, b), (want,) in golden("mse_loss_fwd.json"):
        np.testing.assert_allclose(oracle_mod.mse_loss_forward(a, b, o["reduce"]).reshape(want.shape), want, **TOL)
        n += 1
    assert n == 9
    n = 0
    for o, (x, lbl), (want,) in golden("nll_loss_fwd.json"):
        np.testing.assert_allclose(oracle_mod.nll_loss_forward(x, lbl, o["reduce"]), want, **TOL)
        n += 1
    assert n >= 60
    n = 0
    for o, (x, lbl), (want,) in golden("softmax_loss_fwd.json"):
        np.testing.assert_allclose(oracle_mod.softmax_loss_forward(x, lbl), want, **TOL)
        n += 1
    assert n >= 20


def test_oracle_losses_match_torch(oracle_mod):
    import torch
    import torch.nn.functional as F

    rng = np.random.default_rng(11)
    x = rng.standard_normal((17, 23)).astype(np.float32)
    lbl = rng.integers(0, 23, 17)
    for red in ("none", "sum", "mean"):
        want = F.nll_loss(torch.from_numpy(x), torch.from_numpy(lbl), reduction=red).numpy()
        np.testing.assert_allclose(oracle_mod.nll_loss_forward(x, lbl, red).reshape(want.shape), want, **TOL)
        b = rng.standard_normal(x.shape).astype(np.float32)
        want = F.mse_loss(torch.from_numpy(x), torch.from_numpy(b), reduction=red).numpy()
        np.testing.assert_allclose(oracle_mod.mse_loss_forward(x, b, red).reshape(want.shape), want, **TOL)
    want = F.cross_entropy(torch.from_numpy(x), torch.from_numpy(lbl)).numpy()
    np.testing.assert_allclose(oracle_mod.softmax_loss_forward(x, lbl)[0], want, **TOL)
    # labels outside the classes add nothing
    bad = lbl.copy()
    bad[3], bad[5] = -1, 23
    rows = oracle_mod.nll_loss_forward(x, bad, "none")
    assert rows[3] == 0 and rows[5] == 0 and rows[4] == -x[4, lbl[4]]


def test_reduce_workspace_query_and_validation():
    """host side of dlp_reduce_fwd_*: no kernel runs"""
    import ctypes

    import dlprimitives_amd as dlp

    L = dlp.lib()
    L.dlp_reduce_fwd_workspace.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_size_t)]
    L.dlp_last_error.restype = ctypes.c_char_p

    def query(shape, mask, method=0, dtype=3):
        arr = ctypes.c_int * len(shape)
        need = ctypes.c_size_t(12345)
        rc = L.dlp_reduce_fwd_workspace(dtype, method, len(shape), arr(*shape), arr(*mask), ctypes.byref(need))
        return rc, need.value

    assert query([128, 2048, 7, 7], [0, 0, 1, 1]) == (0, 0)  # many outputs: one piece each
    rc, need = query([1 << 24], [1])  # one output over 16 M elements: cut into pieces of 4-byte partial sums
    assert rc == 0 and 4 * 2 <= need <= 4 * 1024
    assert query([4, 4], [1, 0], method=7)[0] == 1  # unknown method: validation error
    assert query([4, 4], [1, 0], dtype=4)[0] == 2  # double_data: not implemented
    # seven alternating groups: four kept ones are more than the kernels take
    assert query([2, 3, 2, 3, 2, 3, 2], [0, 1, 0, 1, 0, 1, 0])[0] == 2
    assert b"three" in L.dlp_last_error()
    # extents of 1 and neighbours of one kind do not count as groups
    assert query([2, 1, 3, 4, 1, 5, 6, 7], [0, 1, 0, 1, 1, 1, 0, 0])[0] == 0
    # an extent of 0: no workspace; no outputs is a call that does nothing, outputs over no elements an error (before any pointer is read)
    assert query([4, 0, 3], [0, 1, 0]) == (0, 0) and query([0, 5], [0, 1]) == (0, 0)
    L.dlp_reduce_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    arr2 = ctypes.c_int * 2
    assert L.dlp_reduce_fwd_enqueue(3, 0, 1.0, 2, arr2(0, 5), arr2(0, 1), None, None, None, 0, None) == 0
    assert L.dlp_reduce_fwd_enqueue(3, 0, 1.0, 2, arr2(5, 0), arr2(0, 1), None, None, None, 0, None) == 1
    assert b"no elements" in L.dlp_last_error()


# ------------------------------------------------------------------ GPU
def _dev(a, dtype="float32"):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    return t.to(torch.bfloat16) if dtype == "bfloat16" else t


def _nan(shape, dtype="float32"):
    import torch

    return torch.full(tuple(shape), float("nan"), device="cuda:0", dtype=torch.bfloat16 if dtype == "bfloat16" else torch.float32)


def _host(t):
    import torch

    torch.cuda.synchronize()
    return t.float().cpu().numpy()


@pytest.mark.gpu
def test_gpu_interpolation_reference_goldens():
    import dlprimitives_amd as dlp

    n = 0
    for o, (x,), (want,) in golden("interpolation_fwd.json"):
        y = _nan(want.shape)
        dlp.interpolate2d_forward(_dev(x), y, o["method"], o["scale_y"], o["scale_x"], o["align_corners"])
        np.testing.assert_allclose(_host(y), want, **TOL)
        n += 1
    assert n == 84


@pytest.mark.gpu
def test_gpu_interpolation_reference_shapes_vs_oracle(oracle_mod):
    """the cases the reference's test runs against its own CPU operator on random inputs: the same shapes against the oracle"""
    import dlprimitives_amd as dlp

    rng = np.random.default_rng(17)
    doc = json.load(open(os.path.join(GOLDEN, "interpolation_fwd.json")))
    n = 0
    for t in doc["tests"]:
        o = t["options"]
        for cs in t["cases"]:
            if "in" in cs or cs["in_shapes"][0][0] > 4:
                continue
            x = rng.standard_normal(cs["in_shapes"][0]).astype(np.float32)
            hw = tuple(cs["out_shapes"][0][2:])
            assert hw == oracle_mod.interpolate_output_size(x.shape[2:], (o["out_h"], o["out_w"]), (o["scale_y"], o["scale_x"]))
            y = _nan(cs["out_shapes"][0])
            dlp.interpolate2d_forward(_dev(x), y, o["method"], o["scale_y"], o["scale_x"], o["align_corners"])
            np.testing.assert_allclose(_host(y), oracle_mod.interpolate2d_forward(x, hw, **interp_args(o)), **TOL)
            n += 1
    assert n == 168


INTERP_SHAPES = [
    # (planes as batch x channels, input, output): narrow rows that share a block, rows wider than one block, shrinking, one pixel
    ((2, 3), (14, 14), (28, 28)),
    ((1, 5), (7, 9), (23, 29)),
    ((3, 2), (33, 65), (20, 300)),
    ((1, 2), (20, 700), (9, 513)),
    ((64, 32), (7, 7), (14, 14)),
    ((2, 2), (1, 1), (5, 3)),
    ((1, 1), (6, 4), (1, 1)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("method,align", [("nearest", False), ("nearest-exact", False), ("bilinear", False), ("bilinear", True)])
def test_gpu_interpolation_shapes_vs_oracle(oracle_mod, method, align, dtype):
    import dlprimitives_amd as dlp

    rng = np.random.default_rng(21)
    for (B, C), (H, W), (OH, OW) in INTERP_SHAPES:
        x = rng.standard_normal((B, C, H, W)).astype(np.float32)
        if dtype == "bfloat16":
            x = oracle_mod.bf16_round(x)
        want = oracle_mod.interpolate2d_forward(x, (OH, OW), method=method, align_corners=align)
        y = _nan((B, C, OH, OW), dtype)
        dlp.interpolate2d_forward(_dev(x, dtype), y, method, align_corners=align)
        got = _host(y)
        if method != "bilinear":
            np.testing.assert_array_equal(got, want)  # a copy of input values, in either type
        else:
            np.testing.assert_allclose(got, want, **(BF16_TOL if dtype == "bfloat16" else TOL))
    # explicit scales; a size that does not follow from them is refused
    x = rng.standard_normal((2, 2, 7, 9)).astype(np.float32)
    hw = oracle_mod.interpolate_output_size((7, 9), scale=(3.4, 0.7))
    y = _nan((2, 2) + hw)
    dlp.interpolate2d_forward(_dev(x), y, method, 3.4, 0.7, align)
    np.testing.assert_allclose(_host(y), oracle_mod.interpolate2d_forward(x, hw, method=method, scale=(3.4, 0.7), align_corners=align), **TOL)
    if not align:  # with align_corners the steps follow from the sizes alone, as in the reference (src/core/interpolate.cpp:28-31)
        with pytest.raises(dlp.ValidationError):
            dlp.interpolate2d_forward(_dev(x), _nan((2, 2, 24, 6)), method, 3.4, 0.7, align)
    if method != "bilinear":
        with pytest.raises(dlp.ValidationError):
            dlp.interpolate2d_forward(_dev(x), y, method, 3.4, 0.7, True)


@pytest.mark.gpu
def test_gpu_interpolation_random_sizes(oracle_mod):
    """80 random input / output sizes (1 to 40 and a few wide ones), planes, methods and explicit factors against the oracle"""
    import dlprimitives_amd as dlp

    rng = np.random.default_rng(88)
    methods = [("nearest", False), ("nearest-exact", False), ("bilinear", False), ("bilinear", True)]
    for it in range(80):
        method, align = methods[it % 4]
        H, W = int(rng.integers(1, 41)), int(rng.integers(1, 41))
        if it % 9 == 0:
            W = int(rng.integers(250, 700))
        planes = (int(rng.integers(1, 4)), int(rng.integers(1, 6)))
        x = rng.standard_normal(planes + (H, W)).astype(np.float32)
        if it % 3 == 0:  # explicit factors: the size is int(in * factor)
            scale = (float(rng.choice([0.5, 0.75, 1.0, 1.5, 2.0, 3.4])), float(rng.choice([0.5, 0.7, 1.0, 2.0, 3.3])))
            hw = oracle_mod.interpolate_output_size((H, W), scale=scale)
            if hw[0] < 1 or hw[1] < 1:
                continue
        else:
            scale = (-1.0, -1.0)
            hw = (int(rng.integers(1, 50)), int(rng.integers(1, 50)))
        want = oracle_mod.interpolate2d_forward(x, hw, method=method, scale=scale, align_corners=align)
        y = _nan(planes + hw)
        dlp.interpolate2d_forward(_dev(x), y, method, scale[0], scale[1], align)
        got = _host(y)
        if method == "bilinear":
            np.testing.assert_allclose(got, want, err_msg=str((it, method, align, x.shape, hw, scale)), **TOL)
        else:
            assert np.array_equal(got, want), (it, method, x.shape, hw, scale)


@pytest.mark.gpu
def test_gpu_reduction_reference_goldens():
    import dlprimitives_amd as dlp

    n = 0
    for o, (x,), (want,) in golden("reduction_fwd.json"):
        y = _nan(want.shape)
        dlp.reduction_forward(_dev(x), y, **reduce_args(o))
        np.testing.assert_allclose(_host(y), want, rtol=1e-5, atol=1e-5)
        n += 1
    assert n >= 128


REDUCE_SHAPES = [
    # shape, reduced axes: which kernel and which path inside it each one takes
    ((64, 32, 7, 7), [2, 3]),  # a short contiguous run per output (49 elements: no wide loads)
    ((16, 24, 8, 8), [2, 3]),  # 64 elements, wide loads
    ((6, 10, 300), [2]),  # one wave per output
    ((5, 4100), [1]),  # one block per output
    ((3, 1 << 18), [1]),  # few outputs, long runs: cut into pieces
    ((1 << 20,), [0]),  # everything into one value
    ((1000003,), [0]),  # the same with an odd length
    ((8, 16, 30, 30), [1]),  # the channels of every pixel: neighbouring outputs per lane
    ((40, 5, 9), [0]),  # the batch
    ((4, 6, 5, 7), [0, 2]),  # two separate groups, the innermost dimension kept
    ((4, 6, 5, 7), [1, 3]),  # two separate groups, the innermost dimension reduced
    ((3, 4, 5, 6, 7), [1, 3, 4]),
    ((2, 3, 4, 5, 6, 7), [0, 2, 4]),
    ((70000, 3), [0]),  # a long reduction for three outputs: pieces in the second grid dimension
    ((2, 1, 5, 1), [1, 3]),  # only extents of 1 are reduced: a copy
    ((64, 16, 8, 8), [0, 2, 3]),  # per channel: two separate reduced groups, the inner one of whole 16-byte packs
    ((33, 8, 40), [0]),  # the innermost kept dimension of whole packs: several outputs per lane
    ((3000, 8, 40), [0, 1]),  # the same, cut into pieces
]


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("method", ["sum", "sumsq", "abssum", "mean"])
def test_gpu_reduction_shapes_vs_float64(oracle_mod, method, dtype):
    import dlprimitives_amd as dlp

    rng = np.random.default_rng(31)
    split = 0
    for shape, dims in REDUCE_SHAPES:
        x = (rng.standard_normal(shape) + 0.25).astype(np.float32)
        if dtype == "bfloat16":
            x = oracle_mod.bf16_round(x)
        x64 = x.astype(np.float64)
        term = {"sum": x64, "mean": x64, "sumsq": x64 * x64, "abssum": np.abs(x64)}[method]
        want = 0.75 * (term.mean(axis=tuple(dims)) if method == "mean" else term.sum(axis=tuple(dims)))
        scale = 0.75 * np.abs(term).sum(axis=tuple(dims)) / (np.prod([shape[d] for d in dims]) if method == "mean" else 1)
        y = _nan(want.shape if want.shape else (1,), dtype)
        split += dlp.reduction_forward(_dev(x, dtype), y, method, dims=dims, output_scale=0.75) > 0
        got = _host(y).reshape(want.shape)
        # fp32 sums in some order: a few ulp of the sum of magnitudes; bf16 results carry one more rounding
        tol = 2e-6 * scale + (np.abs(want) / 128 if dtype == "bfloat16" else 0) + 1e-30
        assert np.all(np.abs(got - want) <= tol), (shape, dims, float(np.max(np.abs(got - want) / tol)))
    assert split >= 3  # the cut reductions were among them


@pytest.mark.gpu
def test_gpu_reduction_random_shapes_and_masks():
    """120 random tensors of rank 1 to 6 (extents 1 to 9, now and then one long axis) with random sets of reduced axes: every way the
    axes can group into kept / reduced runs, every kernel variant behind them"""
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(77)
    methods = ["sum", "sumsq", "abssum", "mean"]
    seen_not_implemented = 0
    for it in range(120):
        rank = int(rng.integers(1, 7))
        shape = [int(rng.integers(1, 10)) for _ in range(rank)]
        if rng.random() < 0.5:
            shape[int(rng.integers(0, rank))] = int(rng.choice([64, 200, 1000, 4096, 20000]))
        mask = [bool(rng.integers(0, 2)) for _ in range(rank)]
        if not any(mask):
            mask[int(rng.integers(0, rank))] = True
        dims = [i for i, m in enumerate(mask) if m]
        method = methods[it % 4]
        x = rng.standard_normal(shape).astype(np.float32)
        x64 = x.astype(np.float64)
        term = {"sum": x64, "mean": x64, "sumsq": x64 * x64, "abssum": np.abs(x64)}[method]
        want = term.mean(axis=tuple(dims), keepdims=True) if method == "mean" else term.sum(axis=tuple(dims), keepdims=True)
        bound = np.abs(term).sum(axis=tuple(dims), keepdims=True) / (np.prod([shape[d] for d in dims]) if method == "mean" else 1)
        y = _nan(want.shape)
        try:
            dlp.reduction_forward(_dev(x), y, method, dims=dims)
        except dlp.NotImplementedErrorDlprim:
            seen_not_implemented += 1  # more than three separate groups of one kind: rank 7 and up only
            continue
        got = _host(y)
        assert np.all(np.abs(got - want) <= 2e-6 * bound + 1e-30), (shape, dims, method)
    assert seen_not_implemented == 0


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_tensor_ops_on_unaligned_addresses(oracle_mod, dtype):
    """tensors that start one element past a 16-byte address: the kernels fall back to element-wise accesses"""
    import torch

    import dlprimitives_amd as dlp

    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    rng = np.random.default_rng(33)

    def shifted(a):
        buf = torch.zeros(a.size + 1, device="cuda:0", dtype=tdt)
        v = buf[1:].view(a.shape)
        v.copy_(torch.from_numpy(a).to(tdt))
        assert v.data_ptr() % 16 != 0
        return v

    for shape, dims in [((6, 8, 64), [2]), ((6, 8, 64), [0]), ((4, 16, 8, 8), [0, 2, 3])]:
        x = oracle_mod.bf16_round(rng.standard_normal(shape).astype(np.float32))
        want = x.astype(np.float64).sum(axis=tuple(dims))
        y = shifted(np.zeros(want.shape, np.float32))
        dlp.reduction_forward(shifted(x), y, "sum", dims=dims)
        np.testing.assert_allclose(_host(y), want, **(BF16_TOL if dtype == "bfloat16" else dict(rtol=1e-5, atol=1e-5)))
    x = oracle_mod.bf16_round(rng.standard_normal((2, 3, 5, 8)).astype(np.float32))
    y = shifted(np.zeros((2, 3, 10, 16), np.float32))
    dlp.interpolate2d_forward(shifted(x), y, "bilinear")
    np.testing.assert_allclose(_host(y), oracle_mod.interpolate2d_forward(x, (10, 16), "bilinear"), **(BF16_TOL if dtype == "bfloat16" else TOL))
    x = oracle_mod.bf16_round(rng.standard_normal((5, 64)).astype(np.float32))
    lbl = torch.arange(5, dtype=torch.int32, device="cuda:0")
    y = shifted(np.zeros(1, np.float32))
    dlp.softmax_loss_forward(shifted(x), lbl, y)
    np.testing.assert_allclose(_host(y), oracle_mod.softmax_loss_forward(x, np.arange(5)), **(BF16_TOL if dtype == "bfloat16" else TOL))
    b = oracle_mod.bf16_round(rng.standard_normal((5, 64)).astype(np.float32))
    dlp.mse_loss_forward(shifted(x), shifted(b), y, "sum")
    np.testing.assert_allclose(_host(y), oracle_mod.mse_loss_forward(x, b, "sum"), **(BF16_TOL if dtype == "bfloat16" else TOL))


@pytest.mark.gpu
def test_gpu_reduction_repeats_bit_for_bit_and_start_axis():
    import torch

    import dlprimitives_amd as dlp

    x = torch.randn(3, 1 << 18, device="cuda:0")
    a, b = _nan((3,)), _nan((3,))
    assert dlp.reduction_forward(x, a, "sumsq", dims=[1]) > 0
    dlp.reduction_forward(x, b, "sumsq", dims=[-1])
    assert torch.equal(a, b)
    y = _nan((4, 1, 1))
    x = torch.randn(4, 6, 5, device="cuda:0")
    dlp.reduction_forward(x, y, "mean", start_axis=-2)
    np.testing.assert_allclose(_host(y).reshape(4), x.double().mean(dim=(1, 2)).cpu().numpy(), rtol=1e-5, atol=1e-6)
    with pytest.raises(dlp.ValidationError):
        dlp.reduction_forward(x, y, "sum", dims=[3])


@pytest.mark.gpu
@pytest.mark.parametrize("labels", ["float32", "int32"])
def test_gpu_losses_reference_goldens(labels):
    import torch

    import dlprimitives_amd as dlp

    def lab(v):
        return torch.from_numpy(v.astype(labels)).to("cuda:0")

    n = 0
    for o, (x, lbl), (want,) in golden("nll_loss_fwd.json"):
        y = _nan(want.shape)
        dlp.nll_loss_forward(_dev(x), lab(lbl), y, o["reduce"])
        np.testing.assert_allclose(_host(y), want, **TOL)
        n += 1
    for o, (x, lbl), (want,) in golden("softmax_loss_fwd.json"):
        y = _nan(want.shape)
        dlp.softmax_loss_forward(_dev(x), lab(lbl), y)
        np.testing.assert_allclose(_host(y), want, **TOL)
        n += 1
    if labels == "float32":
        for o, (a, b), (want,) in golden("mse_loss_fwd.json"):
            y = _nan(want.shape)
            dlp.mse_loss_forward(_dev(a), _dev(b), y, o["reduce"])
            np.testing.assert_allclose(_host(y), want, **TOL)
            n += 1
    assert n >= 80


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpu_losses_large_vs_oracle(oracle_mod, dtype):
    import torch

    import dlprimitives_amd as dlp

    rng = np.random.default_rng(41)
    tol = BF16_TOL if dtype == "bfloat16" else dict(rtol=2e-5, atol=1e-5)
    for batch, classes in [(128, 1000), (1000, 10), (3, 4099), (1, 1)]:
        x = (3 * rng.standard_normal((batch, classes))).astype(np.float32)
        if dtype == "bfloat16":
            x = oracle_mod.bf16_round(x)
        lbl = rng.integers(0, classes, batch)
        if batch > 5:
            lbl[2], lbl[4] = -3, classes  # outside: these rows add nothing
        for as_int in (True, False):
            lab = torch.from_numpy(lbl.astype(np.int32 if as_int else np.float32)).to("cuda:0")
            y = _nan((1,), dtype)
            dlp.softmax_loss_forward(_dev(x, dtype), lab, y)
            np.testing.assert_allclose(_host(y), oracle_mod.softmax_loss_forward(x, lbl), **tol)
            for red in ("none", "sum", "mean"):
                want = oracle_mod.nll_loss_forward(x, lbl, red)
                y = _nan(want.shape, dtype)
                dlp.nll_loss_forward(_dev(x, dtype), lab, y, red)
                np.testing.assert_allclose(_host(y), want, **(tol if red == "none" or dtype == "float32" else dict(rtol=1e-2, atol=1e-2 * np.abs(x).max())))
    for n in (1, 1000, 1 << 20, (1 << 20) + 3):
        a = rng.standard_normal(n).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        if dtype == "bfloat16":
            a, b = oracle_mod.bf16_round(a), oracle_mod.bf16_round(b)
        d = a.astype(np.float64) - b.astype(np.float64)
        for red, want in (("none", d * d), ("sum", np.array([(d * d).sum()])), ("mean", np.array([(d * d).mean()]))):
            y = _nan(want.shape, dtype)
            dlp.mse_loss_forward(_dev(a, dtype), _dev(b, dtype), y, red)
            np.testing.assert_allclose(_host(y), want, **(BF16_TOL if dtype == "bfloat16" else dict(rtol=2e-5, atol=1e-6)))
    with pytest.raises(dlp.NotImplementedErrorDlprim):
        dlp.nll_loss_forward(_dev(np.zeros((2, 2), np.float32)), torch.zeros(2, dtype=torch.int64, device="cuda:0"), _nan((1,)))


@pytest.mark.gpu
def test_gpu_pointwise_concat_slice_reference_goldens():
    import torch

    import dlprimitives_amd as dlp

    n = 0
    for name, op in (("abs_fwd.json", "abs"), ("hardtanh_fwd.json", "hardtanh"), ("threshold_fwd.json", "threshold")):
        for o, (x,), (want,) in golden(name):
            y = _nan(want.shape)
            p = (o.get("min_val", -1.0), o.get("max_val", 1.0)) if op == "hardtanh" else (o.get("threshold", 0.0), 0.0)
            dlp.pointwise_forward(_dev(x), y, op, *p)
            np.testing.assert_allclose(_host(y), want, **TOL)
            n += 1
    for o, xs, (want,) in golden("concat_fwd.json"):
        y = _nan(want.shape)
        at = 0
        for x in xs:
            dlp.slice_copy(y, at, _dev(x), 0, x.shape[o["dim"]], o["dim"])
            at += x.shape[o["dim"]]
        np.testing.assert_array_equal(_host(y), want)
        n += 1
    for o, (x,), (want,) in golden("slice_fwd.json"):
        y = _nan(want.shape)
        dlp.slice_copy(y, 0, _dev(x), o["begin"], o["end"] - o["begin"], o["dim"])
        np.testing.assert_array_equal(_host(y), want)
        n += 1
    assert n >= 25
