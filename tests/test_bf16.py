"""bfloat16 storage (x, w, y as bf16; bias, accumulation and epilogue in fp32): the reference has
no reduced-precision path, so the bar is 1e-2 relative to the fp32 reference (the oracle)."""
import numpy as np
import pytest

from conv_cases import case, case_id, make_tensors

pytestmark = pytest.mark.gpu


def _bf(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0").to(torch.bfloat16)


def run_conv_bf16(c, x, w, bias, algo="", factor=0.0, y_init=None):
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    st = dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], x.shape, dtype=BFLOAT16_DATA)
    op = dlp.Conv2DForward.create(st, bias is not None, c["activation"], algo)
    assert op.algo() == (algo if algo else "gemm")
    y = _bf(y_init) if y_init is not None else torch.full(dlp.conv2d_output_shape(st, x.shape), float("nan"), dtype=torch.bfloat16, device="cuda:0")
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    bd = torch.from_numpy(bias).cuda() if bias is not None else None
    op.enqueue(_bf(x), _bf(w), bd, y, ws, factor)
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


CASES = [
    (case(3, 1, 1, 1, 64, 64, True, 1, True), (2, 56, 56)),
    (case(1, 0, 1, 1, 256, 64, True, 1, True), (2, 56, 56)),
    (case(1, 0, 2, 1, 256, 512, True, 1, False), (2, 56, 56)),
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (2, 224, 224)),
    (case(3, 1, 2, 1, 128, 128, True, 1, True), (2, 56, 56)),
    (case(3, 1, 1, 1, 512, 512, True, 1, True), (3, 7, 7)),      # split-K path
    (case((3, 5), (1, 2), (2, 3), (3, 2), 3, 8, False, 1, False), (2, 19, 19)),
    (case(3, 1, 1, 1, 8, 8, True, 8, False), (2, 10, 10)),       # depthwise geometry through gemm (channel-major K, one channel per group)
    # bf16 matrix instruction, tap-major K order (Cin/groups % 32 == 0)
    (case(1, 0, 1, 1, 64, 256, True, 1, True), (5, 7, 7)),       # odd pixel count per image: padded column numbering
    (case(1, 0, 1, 1, 2048, 512, True, 1, True), (3, 7, 7)),     # long K, split over workgroups
    (case(3, 2, 1, 2, 64, 64, True, 1, True), (2, 13, 13)),      # dilated, odd width
    (case(3, 1, 1, 1, 64, 96, False, 2, True), (3, 9, 12)),      # two groups, Cout off the tile sizes
    (case(5, 2, 1, 1, 32, 48, True, 1, False), (2, 9, 9)),       # 25 taps
    (case((3, 1), (1, 0), 1, 1, 32, 32, True, 1, False), (1, 1, 1)),  # a single pixel: both ends of the tensor in one pair
    # dense loader (1x1, stride 1, no padding, H*W % 4 == 0: wide loads + register transpose) and wide output stores
    (case(1, 0, 1, 1, 64, 256, True, 1, True), (2, 56, 56)),     # 8-pixel runs, 128x128 tiles, two K tiles
    (case(1, 0, 1, 1, 1024, 256, True, 1, True), (3, 14, 14)),   # 4-pixel runs, tiles crossing images, pixel tail
    (case(1, 0, 1, 1, 256, 64, False, 1, False), (3, 14, 14)),   # 4-pixel runs, 64x256 tiles: every wavefront loads every tile
    (case(1, 0, 1, 1, 64, 80, True, 1, True), (3, 8, 8)),        # Cout off the tile size
    (case(1, 0, 1, 1, 128, 96, True, 2, False), (3, 6, 6)),      # two groups
    (case(1, 0, 1, 1, 2048, 512, True, 1, True), (2, 8, 8)),     # long K: split-K slices start in the middle of the loader rotation
    (case(1, 0, 1, 1, 160, 64, True, 1, True), (5, 4, 10)),      # five K tiles, 8-pixel runs, 64x256 tiles
    (case(3, 1, 1, 1, 64, 64, True, 1, True), (2, 13, 14)),      # 2-pixel output runs
    # dense loader on 1x1 stride-2 convolutions (even image sizes): every other pixel of every other row
    (case(1, 0, 2, 1, 64, 128, True, 1, True), (3, 28, 28)),     # output width 14: runs of 2 output pixels
    (case(1, 0, 2, 1, 64, 64, True, 1, False), (2, 16, 16)),     # 64x256 tiles, runs of 4
    (case(1, 0, 2, 1, 96, 160, False, 1, True), (2, 12, 20)),    # not square, Cout off the tile size, three K tiles
    (case(1, 0, 2, 1, 32, 64, True, 1, True), (2, 14, 14)),      # odd output width: the gather loader
    # LDS-patch kernel (stride-1 3x3 "same", H*W % 4 == 0): the tile's input patch is loaded once per 32 channels
    (case(3, 1, 1, 1, 128, 128, True, 1, True), (3, 28, 28)),    # 128-pixel tiles, 8-pixel loads, pixel tail
    (case(3, 1, 1, 1, 256, 256, True, 1, True), (5, 14, 14)),    # 4-pixel loads, tiles crossing an image boundary
    (case(3, 1, 1, 1, 64, 64, False, 1, False), (4, 14, 14)),    # 256-pixel tiles over three images
    (case(3, 1, 1, 1, 96, 128, True, 1, True), (2, 16, 16)),     # three stages (odd)
    (case(3, 1, 1, 1, 64, 256, True, 2, True), (2, 12, 12)),     # two groups of 32 channels: a single stage
    (case(3, 1, 1, 1, 32, 128, True, 1, True), (5, 8, 8)),       # images smaller than a tile: three segments
    (case(3, 1, 1, 1, 64, 64, True, 1, True), (1, 4, 60)),       # wide, flat image
    # channels-last staging (strided or size-changing kernels, odd image sizes): the input is copied [image][pixel][channel] first
    (case(3, 0, 1, 1, 32, 64, True, 1, True), (2, 12, 12)),
    (case(3, 1, 2, 1, 256, 256, True, 1, True), (2, 28, 28)),    # 784 pixels: 64-pixel transposition tiles, 16-byte reads, last tile partial
    (case(3, 1, 2, 1, 96, 64, True, 1, True), (2, 17, 19)),      # 323 pixels, odd: element-wise reads; 96 channels: half a channel block
    (case(3, 1, 1, 1, 96, 160, False, 1, True), (3, 7, 7)),      # whole-image transposition (49 pixels), 96 channels
    (case(1, 0, 2, 1, 64, 128, True, 1, True), (3, 15, 15)),     # 1x1 stride 2 on an odd image: the copy takes the stride over
    (case(1, 0, (2, 1), 1, 64, 64, True, 1, True), (2, 9, 10)),  # ... in one direction only
    (case(3, (2, 0), (1, 2), (2, 1), 64, 96, True, 2, True), (2, 11, 14)),  # groups, dilation, uneven padding and stride together
]


@pytest.mark.parametrize("c,bhw", CASES, ids=case_id)
def test_bf16_conv_vs_fp32_reference(oracle_mod, c, bhw):
    x, w, bias = make_tensors(c, bhw, seed=21)
    got = run_conv_bf16(c, x, w, bias, algo="gemm")
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    # the fp32 reference on the fp32 tensors: bf16 storage may cost up to 1e-2 relative
    want = oracle_mod.conv2d_forward(x, w, bias, cfg, c["activation"], threads=8)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-2 * scale
    # and against the oracle fed the same bf16-rounded operands only the output rounding (2^-9) remains
    want_r = oracle_mod.conv2d_forward(oracle_mod.bf16_round(x), oracle_mod.bf16_round(w), bias, cfg, c["activation"], threads=8)
    np.testing.assert_allclose(got, want_r, rtol=2 ** -8, atol=1e-4 * scale)


# ResNet-50 layer shapes at the full batch of configuration 5 (many tiles, images crossing tiles)
FULL_BATCH_CASES = [
    (case(1, 0, 1, 1, 128, 128, True, 1, True), (128, 28, 28)),
    (case(1, 0, 1, 1, 160, 128, True, 1, True), (127, 28, 28)),   # odd number of K tiles, partial last tile
    (case(3, 1, 1, 1, 128, 128, True, 1, True), (64, 28, 28)),    # LDS-patch kernel, 392 tiles
    (case(3, 1, 1, 1, 64, 64, True, 1, True), (8, 56, 56)),       # LDS-patch kernel, 256-pixel tiles
]


@pytest.mark.parametrize("c,bhw", FULL_BATCH_CASES, ids=case_id)
def test_bf16_full_batch(oracle_mod, c, bhw):
    x, w, bias = make_tensors(c, bhw, seed=31)
    x, w = oracle_mod.bf16_round(x), oracle_mod.bf16_round(w)
    got = run_conv_bf16(c, x, w, bias, algo="gemm")
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    want = oracle_mod.conv2d_forward(x, w, bias, cfg, c["activation"], threads=8)
    np.testing.assert_allclose(got, want, rtol=2 ** -8, atol=1e-4 * np.abs(want).max())


@pytest.mark.parametrize("cin,cout,bhw", [(64, 64, (2, 56, 56)), (24, 40, (3, 13, 9)), (128, 128, (4, 28, 28)), (512, 512, (3, 7, 7))])
def test_bf16_winograd_vs_fp32_reference(oracle_mod, cin, cout, bhw):
    c = case(3, 1, 1, 1, cin, cout, True, 1, True)
    x, w, bias = make_tensors(c, bhw, seed=22)
    got = run_conv_bf16(c, x, w, bias, algo="winograd")
    cfg = oracle_mod.make_cfg(cin, cout, 3, 1, 1, 1, 1)
    want = oracle_mod.conv2d_forward(x, w, bias, cfg, "relu", threads=8)
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= 1e-2 * scale
    want_r = oracle_mod.conv2d_forward(oracle_mod.bf16_round(x), oracle_mod.bf16_round(w), bias, cfg, "relu", threads=8)
    np.testing.assert_allclose(got, want_r, rtol=2 ** -8, atol=2e-4 * scale)


@pytest.mark.parametrize("ch,hw,stride,k", [(144, 56, 1, 3), (192, 28, 2, 3), (40, 9, 1, 3), (24, 11, 2, 3), (16, 12, 1, 5)])
def test_bf16_depthwise_vs_fp32_reference(oracle_mod, ch, hw, stride, k):
    c = case(k, k // 2, stride, 1, ch, ch, True, ch, False)
    c = dict(c, activation="relu6")
    x, w, bias = make_tensors(c, (2, hw, hw), seed=23)
    got = run_conv_bf16(c, x, w, bias, algo="depthwise_separable")
    cfg = oracle_mod.make_cfg(ch, ch, k, stride, 1, k // 2, ch)
    want_r = oracle_mod.conv2d_forward(oracle_mod.bf16_round(x), oracle_mod.bf16_round(w), bias, cfg, "relu6", threads=8)
    np.testing.assert_allclose(got, want_r, rtol=2 ** -8, atol=1e-3)
    want = oracle_mod.conv2d_forward(x, w, bias, cfg, "relu6", threads=8)
    assert np.abs(got - want).max() <= 1e-2 * max(np.abs(want).max(), 1.0)


# the 3-channel 7x7 stride-2 stem kernel: (case, (batch, H, W)); integer-valued tensors must come out exactly
STEM_CASES = [
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (3, 224, 224)),    # the ResNet stem: 16-byte loads and stores
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (2, 100, 92)),     # rows off the 16-byte units: 2-byte loads and stores
    (case(7, 3, 2, 1, 3, 24, False, 1, False), (2, 45, 96)),    # fewer filters than a block, odd height, no bias
    (case(7, 1, 2, 1, 3, 96, True, 1, True), (2, 70, 88)),      # padding 1, two filter tiles (the second half empty)
    (case(7, (2, 5), 2, 1, 3, 40, True, 1, False), (5, 33, 64)),  # uneven padding; bands that end with the image
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (1, 7, 8)),        # a single band of four pixels per row
]


@pytest.mark.parametrize("c,bhw", STEM_CASES, ids=case_id)
def test_bf16_stem(oracle_mod, c, bhw):
    print("stem", c["pad"], c["cout"], bhw, flush=True)
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    x, w, bias = make_tensors(c, bhw, seed=41)
    x, w = oracle_mod.bf16_round(x), oracle_mod.bf16_round(w)
    got = run_conv_bf16(c, x, w, bias, algo="gemm")
    want = oracle_mod.conv2d_forward(x, w, bias, cfg, c["activation"], threads=8)
    np.testing.assert_allclose(got, want, rtol=2 ** -8, atol=1e-4 * np.abs(want).max())
    rng = np.random.default_rng(3)
    xi = rng.integers(-2, 3, x.shape).astype(np.float32)
    wi = rng.integers(-1, 2, w.shape).astype(np.float32)
    bi = rng.integers(-3, 4, c["cout"]).astype(np.float32) if c["bias"] else None
    want = oracle_mod.conv2d_forward(xi, wi, bi, cfg, c["activation"], threads=8)
    assert np.abs(want).max() <= 256  # exactly representable in bf16
    assert np.array_equal(run_conv_bf16(c, xi, wi, bi, algo="gemm"), want)
    # accumulation with the old y (2-byte path), after the activation
    old = rng.standard_normal(want.shape).astype(np.float32)
    got = run_conv_bf16(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    want = oracle_mod.apply_factor(oracle_mod.conv2d_forward(x, w, bias, cfg, c["activation"], threads=8), oracle_mod.bf16_round(old), 0.5)
    np.testing.assert_allclose(got, want, rtol=2 ** -8, atol=1e-3)


# the stem with its max pooling inside: (case, (batch, H, W)); every one takes workgroup ranges that start in the middle of an image
STEM_POOL_CASES = [
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (5, 224, 224)),    # the ResNet stem: 56 x 56 pooled
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (130, 64, 64)),    # more images than workgroups: ranges span images; 32 x 32 -> 16 x 16
    (case(7, 3, 2, 1, 3, 40, False, 1, False), (3, 72, 96)),    # fewer filters than a tile, no bias, no activation (negative maxima); 36 x 48 -> 18 x 24
    (case(7, 3, 2, 1, 3, 96, True, 1, True), (2, 90, 160)),     # two filter tiles; 45 rows: the last pooled row looks at two rows only; 45 x 80 -> 23 x 40
    (case(7, 3, 2, 1, 3, 64, True, 1, True), (3, 20, 32)),      # 10 x 16 -> 5 x 8: one run of pooled columns, three units an image
]


@pytest.mark.parametrize("c,bhw", STEM_POOL_CASES, ids=case_id)
def test_bf16_stem_with_max_pooling_inside(oracle_mod, c, bhw):
    """dlp_conv2d_fwd_fuse_max_pool against the convolution and Pooling2D run one after the other: the same values bit for bit,
    and against the oracle's convolution followed by a numpy pooling"""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    print("stem+pool", c["pad"], c["cout"], bhw, flush=True)
    x, w, bias = make_tensors(c, bhw, seed=43)
    x, w = oracle_mod.bf16_round(x), oracle_mod.bf16_round(w)
    st = dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], x.shape, dtype=BFLOAT16_DATA)
    xd, wd = _bf(x), _bf(w)
    bd = torch.from_numpy(bias).cuda() if bias is not None else None
    plain = dlp.Conv2DForward.create(st, bias is not None, c["activation"], "gemm")
    oshape = dlp.conv2d_output_shape(st, x.shape)
    mid = torch.full(oshape, float("nan"), dtype=torch.bfloat16, device="cuda:0")
    ws = torch.empty(max(plain.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    plain.enqueue(xd, wd, bd, mid, ws)
    pshape = (oshape[0], oshape[1], dlp.pool2d_output_size(oshape[2], 3, 1, 2), dlp.pool2d_output_size(oshape[3], 3, 1, 2))
    want = torch.full(pshape, float("nan"), dtype=torch.bfloat16, device="cuda:0")
    dlp.Pooling2DForward.create_max_pooling(3, 1, 2, dtype=BFLOAT16_DATA).enqueue(mid, want)
    fused = dlp.Conv2DForward.create(st, bias is not None, c["activation"], "gemm")
    fused.fuse_max_pool(3, 2, 1)
    got = torch.full(pshape, float("nan"), dtype=torch.bfloat16, device="cuda:0")
    fused.enqueue(xd, wd, bd, got, ws)
    torch.cuda.synchronize()
    got, want = got.float().cpu().numpy(), want.float().cpu().numpy()
    assert not np.isnan(got).any()
    assert np.array_equal(got, want)
    # and the oracle: its fp32 convolution, pooled here
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    conv = oracle_mod.conv2d_forward(x[:2], w, bias, cfg, c["activation"], threads=8)
    padded = np.full(conv.shape[:2] + (conv.shape[2] + 2, conv.shape[3] + 2), -np.inf, np.float32)
    padded[:, :, 1:-1, 1:-1] = conv
    ref = np.full((2,) + pshape[1:], -np.inf, np.float32)
    for dy in range(3):
        for dx in range(3):
            ref = np.maximum(ref, padded[:, :, dy:dy + 2 * pshape[2]:2, dx:dx + 2 * pshape[3]:2][:, :, :pshape[2], :pshape[3]])
    np.testing.assert_allclose(got[:2], ref, rtol=2 ** -8, atol=1e-4 * np.abs(ref).max())


def test_bf16_stem_max_pooling_is_refused_where_not_served():
    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA, NotImplementedErrorDlprim

    def stem(dtype, hw=(224, 224), act="relu", k=7, cin=3):
        st = dlp.Conv2DSettings(cin, 64, k, 2, 1, k // 2, 1, (2, cin) + hw, dtype=dtype)
        return dlp.Conv2DForward.create(st, True, act, "gemm")

    stem(BFLOAT16_DATA).fuse_max_pool(3, 2, 1)
    for args in [(2, 2, 0), (3, 1, 1), (3, 2, 0)]:  # other poolings
        with pytest.raises(NotImplementedErrorDlprim):
            stem(BFLOAT16_DATA).fuse_max_pool(*args)
    with pytest.raises(NotImplementedErrorDlprim):
        stem(BFLOAT16_DATA).fuse_max_pool(3, 2, 1, ceil_mode=True)
    with pytest.raises(NotImplementedErrorDlprim):
        stem(FLOAT_DATA).fuse_max_pool(3, 2, 1)               # float tensors
    with pytest.raises(NotImplementedErrorDlprim):
        stem(BFLOAT16_DATA, hw=(100, 92)).fuse_max_pool(3, 2, 1)  # rows off the 8-pixel runs
    with pytest.raises(NotImplementedErrorDlprim):
        stem(BFLOAT16_DATA, act="tanh").fuse_max_pool(3, 2, 1)
    with pytest.raises(NotImplementedErrorDlprim):
        stem(BFLOAT16_DATA, k=3, cin=32).fuse_max_pool(3, 2, 1)   # not the stem kernel
    op = stem(BFLOAT16_DATA)
    op.fuse_max_pool(3, 2, 1)
    with pytest.raises(NotImplementedErrorDlprim):
        op.channels_last(False, True)

DENSE_1X1_CASES = [
    # 1x1 convolutions of 64 / 128 channels over thousands of pixels (the short-K layers of a ResNet-50 bottleneck): the dense loader
    # with two or four K tiles per workgroup, plain, bit-exact on integers, and with both ways of adding the old y
    (case(1, 0, 1, 1, 64, 256, True, 1, True), (2, 56, 56)),     # two m tiles of 128
    (case(1, 0, 1, 1, 128, 512, True, 1, True), (6, 28, 28)),    # four m tiles, the last pixel tile partial, tiles crossing images
    (case(1, 0, 1, 1, 64, 64, False, 1, False), (3, 40, 40)),    # 64 filters, no bias, no activation
    (case(1, 0, 1, 1, 128, 192, True, 1, True), (5, 32, 32)),    # 192 filters: a partial m tile
    (case(1, 0, 1, 1, 64, 128, True, 1, True), (1, 64, 72)),     # one image, not square
]


@pytest.mark.parametrize("c,bhw", DENSE_1X1_CASES, ids=case_id)
def test_bf16_dense_1x1_with_old_y(oracle_mod, c, bhw):
    print("dense 1x1", c["cin"], c["cout"], bhw, flush=True)
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    x, w, bias = make_tensors(c, bhw, seed=51)
    x, w = oracle_mod.bf16_round(x), oracle_mod.bf16_round(w)
    want = oracle_mod.conv2d_forward(x, w, bias, cfg, c["activation"], threads=8)
    np.testing.assert_allclose(run_conv_bf16(c, x, w, bias, algo="gemm"), want, rtol=2 ** -8, atol=1e-4 * np.abs(want).max())
    # integer-valued tensors: every product and sum is exact, the result must equal the reference bit for bit
    rng = np.random.default_rng(4)
    xi = rng.integers(-2, 3, x.shape).astype(np.float32)
    wi = rng.integers(-1, 2, w.shape).astype(np.float32)
    bi = rng.integers(-3, 4, c["cout"]).astype(np.float32) if c["bias"] else None
    wanti = oracle_mod.conv2d_forward(xi, wi, bi, cfg, c["activation"], threads=8)
    assert np.abs(wanti).max() <= 256  # exactly representable in bf16
    assert np.array_equal(run_conv_bf16(c, xi, wi, bi, algo="gemm"), wanti)
    # y = factor * y_old + act(conv), and the residual form y = act(conv + factor * y_old)
    old = rng.standard_normal(want.shape).astype(np.float32)
    got = run_conv_bf16(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    np.testing.assert_allclose(got, oracle_mod.apply_factor(want, oracle_mod.bf16_round(old), 0.5), rtol=2 ** -8, atol=1e-3)
    st = dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], x.shape, dtype=BFLOAT16_DATA)
    op = dlp.Conv2DForward.create(st, bias is not None, c["activation"], "gemm")
    op.accumulate_before_activation(True)
    y = _bf(old)
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
    op.enqueue(_bf(x), _bf(w), torch.from_numpy(bias).cuda() if bias is not None else None, y, ws, 0.5)
    torch.cuda.synchronize()
    conv = oracle_mod.conv2d_forward(x, w, bias, cfg, "identity", threads=8)
    pre = conv + 0.5 * oracle_mod.bf16_round(old)
    # the convolution's value is rounded to bf16 once before the old y joins it: an error relative to the convolution, not to the sum
    np.testing.assert_allclose(y.float().cpu().numpy(), oracle_mod.apply_activation(pre.astype(np.float32), c["activation"]), rtol=2 ** -8,
                               atol=2 ** -8 * np.abs(conv).max())


# Channels-last tensors (dlp_conv2d_fwd_set_channels_last): x and / or y as [image][row][column][channel].  Every loader that
# can feed a channels-last output (dense 1x1, LDS patch, staged copy) and the channels-last loader on every kind of geometry.
CHANNELS_LAST_CASES = [
    (case(1, 0, 1, 1, 1024, 256, True, 1, True), (3, 14, 14)),    # long K, tiles crossing images, pixel tail
    (case(1, 0, 1, 1, 64, 256, True, 1, True), (2, 56, 56)),      # two K tiles, many pixel tiles
    (case(1, 0, 1, 1, 256, 64, False, 1, False), (3, 14, 14)),    # 64 x 256 tiles
    (case(1, 0, 1, 1, 64, 80, True, 1, True), (3, 8, 8)),         # output channels off the tile size
    (case(1, 0, 1, 1, 128, 96, True, 2, False), (3, 6, 6)),       # two groups
    (case(1, 0, 1, 1, 2048, 512, True, 1, True), (3, 7, 7)),      # split over K slices: the channels-last reduction
    (case(1, 0, 2, 1, 256, 512, True, 1, False), (2, 28, 28)),    # 1x1 stride 2 read in place
    (case(1, 0, 2, 1, 64, 128, True, 1, True), (3, 15, 15)),      # ... on an odd image
    (case(3, 1, 2, 1, 128, 128, True, 1, True), (2, 28, 28)),     # 3x3 stride 2
    (case(3, 1, 1, 1, 128, 128, True, 1, True), (3, 28, 28)),     # 3x3 stride 1: LDS-patch kernel unless x is channels-last
    (case(3, 1, 1, 1, 512, 512, True, 1, True), (3, 7, 7)),       # 7x7 planes, split-K
    (case(3, (2, 0), (1, 2), (2, 1), 64, 96, True, 2, True), (2, 11, 14)),  # groups, dilation, uneven padding and stride together
    (case(5, 2, 1, 1, 32, 48, True, 1, False), (2, 9, 9)),        # 25 taps
    (case(1, 0, 1, 1, 1024, 96, True, 1, True), (4, 7, 7)),       # split-K, pixels in fours, output channels off the 64 of a reduction workgroup
]


@pytest.mark.parametrize("layouts", [(True, False), (False, True), (True, True)], ids=["x", "y", "xy"])
@pytest.mark.parametrize("c,bhw", CHANNELS_LAST_CASES, ids=case_id)
def test_bf16_channels_last(oracle_mod, c, bhw, layouts):
    print("channels-last", layouts, c["cin"], c["cout"], c["kernel"], c["stride"], bhw, flush=True)
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    x_cl, y_cl = layouts
    cfg = oracle_mod.make_cfg(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"])
    x, w, bias = make_tensors(c, bhw, seed=77)
    x, w = oracle_mod.bf16_round(x), oracle_mod.bf16_round(w)
    conv = oracle_mod.conv2d_forward(x, w, bias, cfg, "identity", threads=8)
    want = oracle_mod.apply_activation(conv, c["activation"])
    st = dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], x.shape, dtype=BFLOAT16_DATA)
    bd = torch.from_numpy(bias).cuda() if bias is not None else None
    xd = _bf(x.transpose(0, 2, 3, 1)) if x_cl else _bf(x)

    def run(op, old=None, factor=0.0):
        ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda:0")
        if old is None:
            y = torch.full(want.shape, float("nan"), dtype=torch.bfloat16, device="cuda:0")
        else:
            y = _bf(old)
        if y_cl:
            y = y.permute(0, 2, 3, 1).contiguous()
        op.enqueue(xd, _bf(w), bd, y, ws, factor)
        torch.cuda.synchronize()
        got = y.float().cpu().numpy()
        return got.transpose(0, 3, 1, 2) if y_cl else got

    op = dlp.Conv2DForward.create(st, bias is not None, c["activation"], "gemm")
    op.channels_last(x_cl, y_cl)
    got = run(op)
    assert not np.isnan(got).any()
    np.testing.assert_allclose(got, want, rtol=2 ** -8, atol=1e-4 * np.abs(want).max())
    # the residual form y = act(conv + factor * y_old), the old y in the layout of the new one
    op.accumulate_before_activation(True)
    old = np.random.default_rng(5).standard_normal(want.shape).astype(np.float32)
    got = run(op, old, 0.5)
    pre = conv + 0.5 * oracle_mod.bf16_round(old)
    np.testing.assert_allclose(got, oracle_mod.apply_activation(pre.astype(np.float32), c["activation"]), rtol=2 ** -8,
                               atol=2 ** -8 * np.abs(conv).max())
    # integer-valued tensors: every product and sum is exact, the result must equal the reference bit for bit
    rng = np.random.default_rng(4)
    xi = rng.integers(-2, 3, x.shape).astype(np.float32)
    wi = rng.integers(-1, 2, w.shape).astype(np.float32)
    wanti = oracle_mod.conv2d_forward(xi, wi, bias * 0 if bias is not None else None, cfg, c["activation"], threads=8)
    if np.abs(wanti).max() <= 256:  # exactly representable in bf16
        op.accumulate_before_activation(False)
        xd = _bf(xi.transpose(0, 2, 3, 1)) if x_cl else _bf(xi)
        w = wi
        bd = torch.zeros_like(bd) if bd is not None else None
        assert np.array_equal(run(op), wanti)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_global_pooling_channels_last(dtype):
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA, NotImplementedErrorDlprim

    tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    code = BFLOAT16_DATA if dtype == "bfloat16" else FLOAT_DATA
    rng = np.random.default_rng(2)
    for shape in [(3, 2048, 7, 7), (2, 72, 5, 9), (1, 8, 1, 1), (2, 10, 3, 3), (5, 6, 7, 7)]:  # the last two: one channel per thread
        x = torch.from_numpy(rng.standard_normal(shape).astype(np.float32)).cuda().to(tdt)
        for make in (dlp.Pooling2DForward.create_global_avg_pooling, dlp.Pooling2DForward.create_global_max_pooling):
            want = torch.empty((shape[0], shape[1], 1, 1), dtype=tdt, device="cuda:0")
            make(dtype=code).enqueue(x, want)
            op = make(dtype=code)
            op.channels_last(True)
            got = torch.full_like(want, float("nan"))
            op.enqueue(x.permute(0, 2, 3, 1).contiguous(), got)
            torch.cuda.synchronize()
            # the same fp32 sums in another order, rounded to the storage type once
            np.testing.assert_allclose(got.float().cpu().numpy(), want.float().cpu().numpy(), rtol=2 ** -7 if dtype == "bfloat16" else 1e-5, atol=1e-6)
    with pytest.raises(NotImplementedErrorDlprim):
        dlp.Pooling2DForward.create_max_pooling(3, 1, 2, dtype=code).channels_last(True)


def test_bf16_channels_last_is_refused_where_not_served(oracle_mod):
    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA, NotImplementedErrorDlprim

    def op_of(cin, cout, k, dtype, act="relu", algo="gemm", groups=1, hw=14):
        st = dlp.Conv2DSettings(cin, cout, k, 1, 1, k // 2, groups, (2, cin, hw, hw), dtype=dtype)
        return dlp.Conv2DForward.create(st, True, act, algo)

    with pytest.raises(NotImplementedErrorDlprim):
        op_of(64, 64, 1, FLOAT_DATA).channels_last(True, True)       # float tensors
    with pytest.raises(NotImplementedErrorDlprim):
        op_of(48, 64, 1, BFLOAT16_DATA).channels_last(True, False)   # input channels off 32
    with pytest.raises(NotImplementedErrorDlprim):
        op_of(64, 36, 1, BFLOAT16_DATA).channels_last(False, True)   # output channels off 8
    with pytest.raises(NotImplementedErrorDlprim):
        op_of(64, 64, 1, BFLOAT16_DATA, act="tanh").channels_last(True, True)
    with pytest.raises(NotImplementedErrorDlprim):
        op_of(64, 64, 3, BFLOAT16_DATA, algo="winograd").channels_last(True, True)
    op = op_of(48, 64, 1, BFLOAT16_DATA)
    op.channels_last(False, True)  # the output alone is served
    op.channels_last(False, False)


def test_bf16_factor_contract(oracle_mod):
    c = case(3, 1, 1, 1, 16, 24, True, 1, True)
    x, w, bias = make_tensors(c, (2, 11, 9), seed=5)
    cfg = oracle_mod.make_cfg(16, 24, 3, 1, 1, 1, 1)
    old = np.random.default_rng(1).standard_normal((2, 24, 11, 9)).astype(np.float32)
    got = run_conv_bf16(c, x, w, bias, algo="gemm", factor=0.5, y_init=old)
    want = oracle_mod.apply_factor(oracle_mod.conv2d_forward(oracle_mod.bf16_round(x), oracle_mod.bf16_round(w), bias, cfg, "relu"),
                                   oracle_mod.bf16_round(old), 0.5)
    np.testing.assert_allclose(got, want, rtol=2 ** -8, atol=1e-3)


def test_bf16_glue_and_inner_product(oracle_mod):
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    rng = np.random.default_rng(4)
    x = oracle_mod.bf16_round(rng.standard_normal((2, 16, 14, 14)).astype(np.float32))
    y = torch.empty((2, 16, 7, 7), dtype=torch.bfloat16, device="cuda:0")
    dlp.Pooling2DForward.create_max_pooling(3, 1, 2, dtype=BFLOAT16_DATA).enqueue(_bf(x), y)
    torch.cuda.synchronize()
    assert np.array_equal(y.float().cpu().numpy(), oracle_mod.pool2d_forward(x, 3, 1, 2, "max"))  # max of bf16 values is exact
    g = torch.empty((2, 16, 1, 1), dtype=torch.bfloat16, device="cuda:0")
    dlp.Pooling2DForward.create_global_avg_pooling(dtype=BFLOAT16_DATA).enqueue(_bf(x), g)
    b2 = oracle_mod.bf16_round(rng.standard_normal(x.shape).astype(np.float32))
    s = torch.empty(x.shape, dtype=torch.bfloat16, device="cuda:0")
    dlp.eltwise_forward(_bf(x), _bf(b2), s, "sum", 1.0, 1.0, "relu")
    torch.cuda.synchronize()
    np.testing.assert_allclose(g.float().cpu().numpy(), oracle_mod.global_pool_forward(x, "avg"), rtol=2 ** -8, atol=1e-3)
    np.testing.assert_allclose(s.float().cpu().numpy(), oracle_mod.eltwise_forward(x, b2, "sum", 1.0, 1.0, "relu"), rtol=2 ** -8, atol=1e-3)
    xi = rng.uniform(-1, 1, (128, 2048)).astype(np.float32)
    wi = (rng.standard_normal((1000, 2048)) / np.sqrt(2048)).astype(np.float32)
    bi = rng.uniform(-0.1, 0.1, 1000).astype(np.float32)
    ip = dlp.IPForward.create(dlp.IPSettings(2048, 1000, 128, dtype=BFLOAT16_DATA), True, "identity")
    yi = torch.empty((128, 1000), dtype=torch.bfloat16, device="cuda:0")
    ip.enqueue(_bf(xi), _bf(wi), torch.from_numpy(bi).cuda(), yi)
    torch.cuda.synchronize()
    want = oracle_mod.ip_forward(xi, wi, bi)
    assert np.abs(yi.float().cpu().numpy() - want).max() <= 1e-2 * np.abs(want).max()
    # a partial last group of k (In % 16 != 0), Out and batch off the block sizes; and an odd In (rows not dword aligned:
    # the implicit-GEMM fallback)
    for (B, I, O) in ((37, 1000 + 6, 75), (5, 333, 20)):
        xi = oracle_mod.bf16_round(rng.uniform(-1, 1, (B, I)).astype(np.float32))
        wi = oracle_mod.bf16_round((rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32))
        bi = rng.uniform(-0.1, 0.1, O).astype(np.float32)
        ip = dlp.IPForward.create(dlp.IPSettings(I, O, B, dtype=BFLOAT16_DATA), True, "relu")
        yi = torch.full((B, O), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        ip.enqueue(_bf(xi), _bf(wi), torch.from_numpy(bi).cuda(), yi)
        torch.cuda.synchronize()
        np.testing.assert_allclose(yi.float().cpu().numpy(), oracle_mod.ip_forward(xi, wi, bi, "relu"), rtol=2 ** -8, atol=1e-3)


def test_bf16_inner_product_streamed_weights(oracle_mod):
    """bf16 weight matrices of 16 MB and more go through ip_stream_kernel: 512 k per chunk, a short last chunk, outputs and batch
    off the block sizes; integer-valued operands must come out exact."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA

    rng = np.random.default_rng(14)
    for (B, I, O, act) in ((16, 8192, 1024, "relu"), (37, 8200, 1030, "identity")):
        xi = oracle_mod.bf16_round(rng.uniform(-1, 1, (B, I)).astype(np.float32))
        wi = oracle_mod.bf16_round((rng.standard_normal((O, I)) / np.sqrt(I)).astype(np.float32))
        bi = rng.uniform(-0.1, 0.1, O).astype(np.float32)
        ip = dlp.IPForward.create(dlp.IPSettings(I, O, B, dtype=BFLOAT16_DATA), True, act)
        yi = torch.full((B, O), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        dlp.timing_enable(True)
        dlp.timing_reset()
        ip.enqueue(_bf(xi), _bf(wi), torch.from_numpy(bi).cuda(), yi)
        torch.cuda.synchronize()
        kernels = [k for (_, _, k) in dlp.timing_records(kernels=True)]
        dlp.timing_enable(False)
        assert kernels and kernels[-1].startswith("ip_stream_kernel"), kernels
        np.testing.assert_allclose(yi.float().cpu().numpy(), oracle_mod.ip_forward(xi, wi, bi, act), rtol=2 ** -8, atol=1e-3)
        xq = rng.integers(-2, 3, (B, I)).astype(np.float32)
        wq = rng.integers(-1, 2, (O, I)).astype(np.float32)
        want = (xq.astype(np.int64) @ wq.astype(np.int64).T).astype(np.float32)
        ip2 = dlp.IPForward.create(dlp.IPSettings(I, O, B, dtype=BFLOAT16_DATA), False, "identity")
        yq = torch.full((B, O), float("nan"), dtype=torch.bfloat16, device="cuda:0")
        ip2.enqueue(_bf(xq), _bf(wq), None, yq)
        torch.cuda.synchronize()
        assert np.array_equal(yq.float().cpu().numpy(), oracle_mod.bf16_round(want))  # the sum is exact in fp32, rounded once


def test_resnet50_bf16_logits_vs_fp32_reference(oracle_mod):
    """Configuration 5 at a batch the CPU oracle finishes in seconds: ResNet-50 forward with bf16
    storage against the fp32 reference path on the same fp32 weights and inputs, 1e-2 relative."""
    import torch

    from dlprimitives_amd import graphs
    from graph_oracle import run_graph_on_oracle

    ops = graphs.resnet50()
    params = graphs.random_parameters(ops, seed=11)
    x = np.random.default_rng(3).standard_normal((4, 3, 224, 224)).astype(np.float32)
    want = run_graph_on_oracle(oracle_mod, ops, params, x)
    for fuse_residual in (False, True):  # residual sums as operators of their own, and in the epilogues of the 1x1 convolutions
        runner = graphs.GraphRunner(ops, params, x.shape, algo="", dtype="bfloat16", fuse_residual=fuse_residual)
        got = runner.forward(torch.from_numpy(x).cuda().to(torch.bfloat16)).float().cpu().numpy()
        rel = np.abs(got - want).max() / np.abs(want).max()
        print("resnet50 bf16 vs fp32 reference (sums fused: %s): max relative error of the logits %.4f" % (fuse_residual, rel))
        assert rel <= 1e-2
        assert (got.argmax(1) == want.argmax(1)).all()


def test_resnet50_bf16_benchmarked_deployment_logits(oracle_mod):
    """The form of configuration 5 that bench.py times: batch 128, bf16 storage, algo "gemm", residual sums in the epilogues of
    the 1x1 convolutions, filters packed once (enqueue_packed).  Images are independent, so 4 of the 128 logit rows are compared
    with the fp32 reference path run on those 4 images: 1e-2 relative to the largest logit, same arg-max."""
    import torch

    from dlprimitives_amd import graphs
    from graph_oracle import run_graph_on_oracle

    ops = graphs.resnet50()
    params = graphs.random_parameters(ops, seed=11)
    x = np.random.default_rng(5).standard_normal((128, 3, 224, 224)).astype(np.float32)
    pick = [0, 41, 86, 127]
    want = run_graph_on_oracle(oracle_mod, ops, params, np.ascontiguousarray(x[pick]))
    runner = graphs.GraphRunner(ops, params, x.shape, algo="gemm", dtype="bfloat16", fuse_residual=True, prepack=True)
    xd = torch.from_numpy(x).cuda().to(torch.bfloat16)
    first = runner.forward(xd).float().cpu().numpy()
    again = runner.forward(xd).float().cpu().numpy()  # a second pass over the packed filters and the operators' own counters
    assert first.shape == (128, want.shape[1])
    assert np.array_equal(first, again)
    got = first[pick]
    rel = np.abs(got - want).max() / np.abs(want).max()
    print("resnet50 bf16 b128, sums fused, filters packed once: max relative error of 4 logit rows %.4f" % rel)
    assert rel <= 1e-2
    assert (got.argmax(1) == want.argmax(1)).all()
    # the same deployment with the tensors between convolutions kept channels-last wherever the planner finds it pays
    del runner
    runner = graphs.GraphRunner(ops, params, x.shape, algo="gemm", dtype="bfloat16", fuse_residual=True, prepack=True, channels_last=True)
    assert len(runner.cl) >= 25, sorted(runner.cl)  # about half of the tensors between the 53 convolutions
    assert "data" not in runner.cl and "stem" not in runner.cl and "logits" not in runner.cl
    cl_first = runner.forward(xd).float().cpu().numpy()
    cl_again = runner.forward(xd).float().cpu().numpy()
    assert np.array_equal(cl_first, cl_again)
    rel_cl = np.abs(cl_first[pick] - want).max() / np.abs(want).max()
    print("... channels-last (%d tensors): max relative error %.4f; against the run above %.4f" %
          (len(runner.cl), rel_cl, np.abs(cl_first - first).max() / np.abs(want).max()))
    assert rel_cl <= 1e-2
    assert (cl_first[pick].argmax(1) == want.argmax(1)).all()
    # ... and with the stem's max pooling inside the stem's kernel, which is the form that bench.py times: the pooled tensor is the
    # same bit for bit, so the logits are those of the run above
    del runner
    runner = graphs.GraphRunner(ops, params, x.shape, algo="gemm", dtype="bfloat16", fuse_residual=True, prepack=True, channels_last=True,
                                fuse_stem_pool=True)
    assert sum(1 for o in runner.ops if o.get("pool")) == 1 and not any(o["op"] == "maxpool" for o in runner.ops)
    pooled = runner.forward(xd).float().cpu().numpy()
    assert np.array_equal(pooled, cl_first)
