"""GPU parity at the sizes the benchmark times (batch 64 / 128), through the C ABI.

The oracle needs minutes at these sizes, so the check is the integer-exact property of the reference's GEMM test
(tests/test_gemm.cpp:40-117): tensors hold small integers, every product and partial sum is then exactly
representable in fp32 (and in bf16 storage where used), whatever the order of summation, and the result must EQUAL
torch.nn.functional.conv2d evaluated in float64 on the CPU.  What changes with the batch is what this pins: the
stream-K distribution over 768 workgroups, the finer split of the last partial round of tiles, the split-K slice
counts, the batch chunking of Winograd, the strip / plane decomposition of the depthwise kernels.

Every launch runs twice on one operator object and the two results must be bit-identical (the last-arriver
reductions add in a fixed order; counters return to zero).
"""
import numpy as np
import pytest

from dlprimitives_amd.workloads import MOBILENET_DEPTHWISE, MOBILENET_POINTWISE, RESNET18_CONVS, RESNET50_CONVS, WINOGRAD_SHAPES, conv

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    import torch

    assert torch.cuda.is_available(), "these tests need the MI355X"
    torch.set_num_threads(16)
    import gpu_util

    return gpu_util


def _int_tensors(L, batch, seed, wmax=2):
    """integer-valued x in [-3, 3], w in [-wmax, wmax], bias in [-5, 5]: |sum| < 2^24 for every K of the workloads"""
    rng = np.random.default_rng(seed)
    cin_g = L["cin"] // L["groups"]
    x = rng.integers(-3, 4, (batch, L["cin"], L["hw"], L["hw"])).astype(np.float32)
    w = rng.integers(-wmax, wmax + 1, (L["cout"], cin_g, L["kernel"], L["kernel"])).astype(np.float32)
    b = rng.integers(-5, 6, L["cout"]).astype(np.float32)
    return x, w, b


def _torch_reference(L, x, w, b, bf16_out=False):
    import torch
    import torch.nn.functional as F

    y = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(b).double(), stride=L["stride"], padding=L["pad"],
                 groups=L["groups"])
    act = L["activation"]
    if act == "relu":
        y = y.clamp_(min=0)
    elif act == "relu6":
        y = y.clamp_(min=0, max=6)
    else:
        assert act == "identity"
    y = y.float()
    if bf16_out:
        y = y.to(torch.bfloat16).float()  # one round-to-nearest-even of the exact fp32 value, as the epilogue does
    return y.numpy()


def _run_twice(L, x, w, b, algo, batch, bf16=False):
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA

    tdt = torch.bfloat16 if bf16 else torch.float32
    st = dlp.Conv2DSettings(L["cin"], L["cout"], L["kernel"], L["stride"], 1, L["pad"], L["groups"], x.shape, dtype=BFLOAT16_DATA if bf16 else FLOAT_DATA)
    op = dlp.Conv2DForward.create(st, True, L["activation"], algo)
    assert op.algo() == algo, (op.algo(), algo)
    xd, wd, bd = torch.from_numpy(x).cuda().to(tdt), torch.from_numpy(w).cuda().to(tdt), torch.from_numpy(b).cuda()
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    outs = []
    for _ in range(2):
        y = torch.full((batch, L["cout"], L["ohw"], L["ohw"]), float("nan"), dtype=tdt, device="cuda:0")
        op.enqueue(xd, wd, bd, y, ws, 0.0)
        torch.cuda.synchronize()
        outs.append(y.float().cpu().numpy())
    # the same through the entry points a caller with constant filters uses (pack once, enqueue_packed): what the benchmark's
    # packed configurations and dlprim::Net run; must give the same bits as enqueue
    packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
    op.pack(wd, packed)
    for _ in range(2):
        y = torch.full((batch, L["cout"], L["ohw"], L["ohw"]), float("nan"), dtype=tdt, device="cuda:0")
        op.enqueue_packed(xd, wd, packed, bd, y, ws, 0.0)
        torch.cuda.synchronize()
        assert np.array_equal(y.float().cpu().numpy(), outs[0]), "enqueue_packed differs from enqueue"
    return outs


def _check(L, algo, batch, seed, bf16=False, wmax=2):
    x, w, b = _int_tensors(L, batch, seed, wmax)
    print("full size:", L["name"], algo, "batch", batch, "bf16" if bf16 else "fp32", flush=True)
    first, second = _run_twice(L, x, w, b, algo, batch, bf16)
    want = _torch_reference(L, x, w, b, bf16)
    assert np.array_equal(first, want), "max |diff| %g" % np.abs(first - want).max()
    assert np.array_equal(first, second)


@pytest.mark.parametrize("L", RESNET18_CONVS[:2] + RESNET18_CONVS[5:8] + RESNET18_CONVS[10:13] + RESNET18_CONVS[15:18], ids=lambda L: L["name"])
def test_resnet18_layers_batch64_gemm(gpu, L):
    # (the repeated 3x3 stride-1 layers of a stage have one shape: one of them each)
    _check(L, "gemm", 64, seed=L["hw"] + L["cin"])


@pytest.mark.parametrize("shape", WINOGRAD_SHAPES, ids=lambda s: "b%d_%dto%d_at%d" % s)
@pytest.mark.parametrize("algo", ["winograd", "gemm"])
def test_winograd_shapes_batch64(gpu, shape, algo):
    # Winograd's transforms divide by 2 and 4: with filter values that are multiples of 4 every intermediate
    # stays an integer (G k G^T has entries k/4 sums), so the exact comparison holds for it as well
    b, ci, co, hw = shape
    L = conv("3x3_%dto%d_at%d" % (ci, co, hw), 3, 1, 1, ci, co, hw)
    x, w, bias = _int_tensors(L, b, seed=ci + hw, wmax=1)
    w *= 4.0
    first, second = _run_twice(L, x, w, bias, algo, b)
    want = _torch_reference(L, x, w, bias)
    assert np.array_equal(first, want), "max |diff| %g" % np.abs(first - want).max()
    assert np.array_equal(first, second)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("ch,hw", MOBILENET_DEPTHWISE)
def test_depthwise_batch64(gpu, ch, hw, stride):
    L = conv("dw3x3s%d_c%d_at%d" % (stride, ch, hw), 3, stride, 1, ch, ch, hw, groups=ch, activation="relu6")
    _check(L, "depthwise_separable", 64, seed=ch + stride)


@pytest.mark.parametrize("pw", MOBILENET_POINTWISE, ids=lambda p: "%dto%d_at%d" % p)
def test_pointwise_batch64(gpu, pw):
    ci, co, hw = pw
    L = conv("pw1x1_%dto%d_at%d" % (ci, co, hw), 1, 1, 0, ci, co, hw, activation="relu6")
    _check(L, "gemm", 64, seed=ci + co)


def _r50(name):
    return next(L for L in RESNET50_CONVS if L["name"] == name)


@pytest.mark.parametrize("name", ["l1_1_3x3_64to64_at56", "l2_0_1x1_256to128_at56", "l2_0_3x3s2_128to128_at56", "l3_1_1x1_1024to256_at14",
                                  "l4_0_ds_1x1s2_1024to2048_at14", "l4_2_3x3_512to512_at7"])
def test_resnet50_layers_batch128_bf16(gpu, name):
    # bf16 storage: x in [-3, 3] and w in [-1, 1] are bf16 values, sums are exact in fp32, the one rounding to bf16
    # at the end is applied to the reference as well; identity layers would exceed 256 (the largest range in which
    # bf16 holds every integer) only in the rounding, which both sides do alike
    _check(_r50(name), "gemm", 128, seed=len(name), bf16=True, wmax=1)


@pytest.mark.parametrize("name", ["l1_0_1x1_64to256_at56", "l3_1_1x1_256to1024_at14"])
@pytest.mark.parametrize("bf16", [False, True], ids=["fp32", "bf16"])
def test_resnet50_residual_epilogue_batch128(gpu, name, bf16):
    """accumulate_first on two 1x1 layers that end ResNet-50 blocks, at the benchmark's batch: y = relu(conv + bias + y_old) with
    the skip branch already in y, through enqueue_packed, twice; integer tensors, exact."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA

    L = dict(_r50(name))
    L["activation"] = "identity"
    batch = 128
    x, w, b = _int_tensors(L, batch, seed=len(name) + 7, wmax=1)
    skip = np.random.default_rng(9).integers(-4, 5, (batch, L["cout"], L["ohw"], L["ohw"])).astype(np.float32)
    conv_out = _torch_reference(L, x, w, b)
    want = np.maximum(conv_out + skip, 0.0)
    tdt = torch.bfloat16 if bf16 else torch.float32
    if bf16:
        want = torch.from_numpy(want).to(torch.bfloat16).float().numpy()
    st = dlp.Conv2DSettings(L["cin"], L["cout"], L["kernel"], L["stride"], 1, L["pad"], L["groups"], x.shape, dtype=BFLOAT16_DATA if bf16 else FLOAT_DATA)
    op = dlp.Conv2DForward.create(st, True, "relu", "gemm")
    op.accumulate_before_activation(True)
    xd, wd, bd = torch.from_numpy(x).cuda().to(tdt), torch.from_numpy(w).cuda().to(tdt), torch.from_numpy(b).cuda()
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
    op.pack(wd, packed)
    for _ in range(2):
        y = torch.from_numpy(skip).cuda().to(tdt)
        op.enqueue_packed(xd, wd, packed, bd, y, ws, 1.0)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        assert np.array_equal(got, want), "max |diff| %g" % np.abs(got - want).max()
