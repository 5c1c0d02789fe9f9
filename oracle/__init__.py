"""CPU oracle bindings -- TEST INFRASTRUCTURE ONLY.

ctypes/numpy front end of ``oracle/liboracle.so`` (the C restatement of the
dlprimitives CPU operators in ``dlp_oracle.c``) and, when it has been built, of
``oracle/_ref/libdlprim_ref.so`` (the reference's own internal BLAS and
activation helpers compiled from the reference sources).

Interpolation, Reduction and the losses (``interpolate2d_forward``, ``reduction_forward``, ``mse_loss_forward``,
``nll_loss_forward``, ``softmax_loss_forward``) are numpy restatements of the reference's CPU operators; each is
pinned by the reference's golden cases (``tests/golden/*_fwd.json``) and by the matching torch routine in
``tests/test_tensor_ops.py``.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import
this package, and only as the checker.  The shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "libdlprim_ref.so")

ACTIVATIONS = {"identity": 0, "relu": 1, "tanh": 2, "sigmoid": 3, "relu6": 4}


def build(force=False):
    """Compile the oracle (and oracle/_ref when the reference tree is present)."""
    args = ["make", "-C", _HERE]
    if force:
        args.insert(1, "-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


class _Cfg(ctypes.Structure):
    _fields_ = [
        ("channels_in", ctypes.c_int),
        ("channels_out", ctypes.c_int),
        ("kernel", ctypes.c_int * 2),
        ("stride", ctypes.c_int * 2),
        ("dilate", ctypes.c_int * 2),
        ("pad", ctypes.c_int * 2),
        ("groups", ctypes.c_int),
    ]


_lib = None
_ref = None
_fp = ctypes.POINTER(ctypes.c_float)
_dp = ctypes.POINTER(ctypes.c_double)
_ip = ctypes.POINTER(ctypes.c_int)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.orc_conv2d_output_shape.restype = ctypes.c_int
        L.orc_conv2d_workspace.restype = ctypes.c_size_t
        L.orc_conv2d_forward.restype = ctypes.c_int
        L.orc_conv2d_forward_mt.restype = ctypes.c_int
        L.orc_conv2d_direct_f64.restype = ctypes.c_int
        L.orc_winograd_forward.restype = ctypes.c_int
        L.orc_depthwise_forward.restype = ctypes.c_int
        L.orc_pool_output_size.restype = ctypes.c_int
        L.orc_bf16_round.restype = ctypes.c_float
        L.orc_bf16_round.argtypes = [ctypes.c_float]
        _lib = L
    return _lib


def ref():
    """The compiled reference pieces, or None when oracle/_ref was not built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        _ref = ctypes.CDLL(_REF_PATH)
    return _ref


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a):
    return a.ctypes.data_as(_fp) if a is not None else None


def _pair(v):
    if isinstance(v, (tuple, list)):
        return int(v[0]), int(v[1])
    return int(v), int(v)


def make_cfg(cin, cout, kernel, stride=1, dilate=1, pad=0, groups=1):
    c = _Cfg()
    c.channels_in, c.channels_out, c.groups = int(cin), int(cout), int(groups)
    c.kernel[:] = _pair(kernel)
    c.stride[:] = _pair(stride)
    c.dilate[:] = _pair(dilate)
    c.pad[:] = _pair(pad)
    return c


def _act(a):
    return ACTIVATIONS[a] if isinstance(a, str) else int(a)


def conv2d_output_shape(cfg, in_shape):
    ish = (ctypes.c_int * 4)(*[int(v) for v in in_shape])
    osh = (ctypes.c_int * 4)()
    if lib().orc_conv2d_output_shape(ctypes.byref(cfg), ish, osh) != 0:
        raise ValueError("invalid convolution configuration")
    return tuple(osh)


def conv2d_forward(x, w, bias, cfg, activation="identity", threads=1):
    """Convolution2D::forward_cpu restated; ``threads`` != 1 distributes images over OpenMP."""
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    ish = (ctypes.c_int * 4)(*x.shape)
    y = np.empty(conv2d_output_shape(cfg, x.shape), dtype=np.float32)
    if threads == 1:
        ws = np.empty(max(1, lib().orc_conv2d_workspace(ctypes.byref(cfg), ish) // 4), dtype=np.float32)
        r = lib().orc_conv2d_forward(ctypes.byref(cfg), ish, _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _ptr(ws), _act(activation))
    else:
        r = lib().orc_conv2d_forward_mt(ctypes.byref(cfg), ish, _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _act(activation), int(threads))
    if r < 0:
        raise ValueError("invalid convolution configuration")
    return y


def conv2d_backward_data(dy, w, cfg, in_shape, dx_old=None, factor=0.0):
    """Convolution2D::backward_data_cpu restated: returns factor * dx_old + gradient with respect to x."""
    dy, w = _f32(dy), _f32(w)
    ish = (ctypes.c_int * 4)(*in_shape)
    dx = _f32(dx_old).copy() if dx_old is not None else np.zeros(tuple(in_shape), dtype=np.float32)
    ws = np.empty(max(1, lib().orc_conv2d_workspace(ctypes.byref(cfg), ish) // 4), dtype=np.float32)
    if lib().orc_conv2d_backward_data(ctypes.byref(cfg), ish, _ptr(dy), _ptr(w), _ptr(dx), _ptr(ws), ctypes.c_float(factor)) < 0:
        raise ValueError("invalid convolution configuration")
    return dx


def tconv2d_output_shape(cfg, in_shape, output_pad=(0, 0)):
    """Conv2DBase::get_output_shape_transposed restated"""
    ish = (ctypes.c_int * 4)(*in_shape)
    op = (ctypes.c_int * 2)(*output_pad)
    osh = (ctypes.c_int * 4)()
    if lib().orc_tconv2d_output_shape(ctypes.byref(cfg), ish, op, osh) < 0:
        raise ValueError("invalid transposed convolution configuration")
    return tuple(osh)


def tconv2d_forward(x, w, bias, cfg, output_pad=(0, 0), activation="identity"):
    """TransposedConvolution2D::forward (CPU path) restated; cfg describes the transposed operator
    (channels_in = x.shape[1]); w is [channels_in, channels_out / groups, kh, kw]."""
    x, w = _f32(x), _f32(w)
    osh = tconv2d_output_shape(cfg, x.shape, output_pad)
    y = np.empty(osh, dtype=np.float32)
    conv = make_cfg(cfg.channels_out, cfg.channels_in, tuple(cfg.kernel), tuple(cfg.stride), tuple(cfg.dilate), tuple(cfg.pad), cfg.groups)
    ws = np.empty(max(1, lib().orc_conv2d_workspace(ctypes.byref(conv), (ctypes.c_int * 4)(*osh)) // 4), dtype=np.float32)
    b = _f32(bias) if bias is not None else None
    rc = lib().orc_tconv2d_forward(ctypes.byref(cfg), (ctypes.c_int * 4)(*x.shape), (ctypes.c_int * 2)(*output_pad), _ptr(x), _ptr(w),
                                   _ptr(b) if b is not None else None, _ptr(y), _ptr(ws), ACTIVATIONS[activation])
    if rc < 0:
        raise ValueError("invalid transposed convolution configuration")
    return y


def conv2d_backward_filter(dy, x, cfg, dw_old=None, factor=0.0):
    """Convolution2D::backward_filter_cpu restated: returns factor * dw_old + gradient with respect to w."""
    dy, x = _f32(dy), _f32(x)
    ish = (ctypes.c_int * 4)(*x.shape)
    shape = (cfg.channels_out, cfg.channels_in // cfg.groups, cfg.kernel[0], cfg.kernel[1])
    dw = _f32(dw_old).copy() if dw_old is not None else np.zeros(shape, dtype=np.float32)
    ws = np.empty(max(1, lib().orc_conv2d_workspace(ctypes.byref(cfg), ish) // 4), dtype=np.float32)
    if lib().orc_conv2d_backward_filter(ctypes.byref(cfg), ish, _ptr(dy), _ptr(x), _ptr(dw), _ptr(ws), ctypes.c_float(factor)) < 0:
        raise ValueError("invalid convolution configuration")
    return dw


def bias_backward(dy, db_old=None, beta=0.0):
    """BWBias::backward_cpu restated: db[f] = beta * db_old[f] + sum of dy over batch and plane."""
    dy = _f32(dy)
    features = dy.shape[1]
    db = _f32(db_old).copy() if db_old is not None else np.zeros(features, dtype=np.float32)
    lib().orc_bias_backward(int(dy.shape[0]), int(features), int(dy.size // max(dy.shape[0] * features, 1)), _ptr(dy), _ptr(db), ctypes.c_float(beta))
    return db


def sgemm(A, B, trans_a=False, trans_b=False, C=None, alpha=1.0, beta=0.0):
    """The restated my_cblas products (nt, nn, tn), row-major, with the reference's loop orders."""
    A, B = _f32(A), _f32(B)
    M = A.shape[1] if trans_a else A.shape[0]
    K = A.shape[0] if trans_a else A.shape[1]
    N = B.shape[0] if trans_b else B.shape[1]
    out = _f32(C).copy() if C is not None else np.zeros((M, N), dtype=np.float32)
    fn = {(False, True): lib().orc_sgemm_nt, (False, False): lib().orc_sgemm_nn, (True, False): lib().orc_sgemm_tn}[(bool(trans_a), bool(trans_b))]
    fn(M, N, K, ctypes.c_float(alpha), _ptr(A), int(A.shape[1]), _ptr(B), int(B.shape[1]), ctypes.c_float(beta), _ptr(out), N)
    return out


def conv2d_direct_f64(x, w, bias, cfg, activation="identity"):
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    ish = (ctypes.c_int * 4)(*x.shape)
    y = np.empty(conv2d_output_shape(cfg, x.shape), dtype=np.float64)
    r = lib().orc_conv2d_direct_f64(ctypes.byref(cfg), ish, _ptr(x), _ptr(w), _ptr(bias), y.ctypes.data_as(_dp), _act(activation))
    if r != 0:
        raise ValueError("invalid convolution configuration")
    return y


def apply_factor(y_new, y_old, factor):
    y = _f32(y_new).copy()
    yo = _f32(y_old)
    lib().orc_apply_factor(_ptr(y), _ptr(yo), ctypes.c_size_t(y.size), ctypes.c_float(factor))
    return y


def apply_activation(a, activation):
    a = _f32(a).copy()
    lib().orc_apply_activation(_ptr(a), ctypes.c_size_t(a.size), _act(activation))
    return a


def sgemm_nt(A, B, C=None, alpha=1.0, beta=0.0):
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[0]
    C = np.zeros((M, N), dtype=np.float32) if C is None else _f32(C).copy()
    lib().orc_sgemm_nt(M, N, K, ctypes.c_float(alpha), _ptr(A), K, _ptr(B), K, ctypes.c_float(beta), _ptr(C), N)
    return C


def im2col(img, cfg, out_hw):
    img = _f32(img)
    cin_g, H, W = img.shape
    OH, OW = out_hw
    mat = np.empty((OH * OW, cin_g * cfg.kernel[0] * cfg.kernel[1]), dtype=np.float32)
    lib().orc_im2col(ctypes.byref(cfg), cin_g, H, W, OH, OW, _ptr(img), _ptr(mat))
    return mat


def ip_forward(x, w, bias, activation="identity"):
    x, w = _f32(x), _f32(w)
    batch = x.shape[0]
    x2 = x.reshape(batch, -1)
    bias = _f32(bias) if bias is not None else None
    y = np.empty((batch, w.shape[0]), dtype=np.float32)
    lib().orc_ip_forward(batch, x2.shape[1], w.shape[0], _ptr(x2), _ptr(w), _ptr(bias), _ptr(y), _act(activation))
    return y


def winograd_filter_transform(w):
    w = _f32(w)
    cout, cin = w.shape[:2]
    u = np.empty((cout, cin, 16), dtype=np.float32)
    lib().orc_winograd_filter_transform(cout, cin, _ptr(w), _ptr(u))
    return u


def winograd_forward(x, w, bias, activation="identity", factor=0.0, y_old=None):
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    B, C, H, W = x.shape
    N = w.shape[0]
    y = np.zeros((B, N, H, W), dtype=np.float32) if y_old is None else _f32(y_old).copy()
    u = np.empty(16 * C * N, dtype=np.float32)
    r = lib().orc_winograd_forward(B, C, N, H, W, _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _ptr(u), _act(activation), ctypes.c_float(factor))
    if r != 0:
        raise ValueError("invalid winograd configuration")
    return y


def depthwise_forward(x, w, bias, activation="identity", factor=0.0, y_old=None):
    x, w = _f32(x), _f32(w)
    bias = _f32(bias) if bias is not None else None
    B, C, H, W = x.shape
    kern = w.shape[-1]
    y = np.zeros((B, C, H, W), dtype=np.float32) if y_old is None else _f32(y_old).copy()
    r = lib().orc_depthwise_forward(B, C, H, W, kern, _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _act(activation), ctypes.c_float(factor))
    if r != 0:
        raise ValueError("invalid depthwise configuration")
    return y


def pool_output_size(in_size, kernel, pad, stride, ceil_mode):
    r = lib().orc_pool_output_size(int(in_size), int(kernel), int(pad), int(stride), int(bool(ceil_mode)))
    if r < 0:
        raise ValueError("invalid pooling configuration")
    return r


def pool2d_forward(x, kernel, pad, stride, mode, count_include_pad=False, ceil_mode=False):
    """Pooling2D::forward_cpu restated; mode 'max' or 'avg'."""
    x = _f32(x)
    B, C, H, W = x.shape
    k, p, s = _pair(kernel), _pair(pad), _pair(stride)
    OH = pool_output_size(H, k[0], p[0], s[0], ceil_mode)
    OW = pool_output_size(W, k[1], p[1], s[1], ceil_mode)
    y = np.empty((B, C, OH, OW), dtype=np.float32)
    i2 = ctypes.c_int * 2
    lib().orc_pool2d_forward(B * C, H, W, OH, OW, i2(*k), i2(*p), i2(*s), 0 if mode == "max" else 1, int(bool(count_include_pad)),
                             _ptr(x), _ptr(y))
    return y


def global_pool_forward(x, mode):
    x = _f32(x)
    B, C = x.shape[:2]
    y = np.empty((B, C, 1, 1), dtype=np.float32)
    lib().orc_global_pool_forward(ctypes.c_size_t(B * C), ctypes.c_size_t(x[0, 0].size), 0 if mode == "max" else 1, _ptr(x), _ptr(y))
    return y


ELTWISE_OPS = {"sum": 0, "prod": 1, "max": 2}


def eltwise_forward(a, b, op="sum", coef1=1.0, coef2=1.0, activation="identity"):
    a, b = _f32(a), _f32(b)
    c = np.empty_like(a)
    lib().orc_eltwise_forward(ctypes.c_size_t(a.size), ELTWISE_OPS[op], ctypes.c_float(coef1), ctypes.c_float(coef2), _act(activation),
                              _ptr(a), _ptr(b), _ptr(c))
    return c


def batch_norm_forward(x, mean, var, gamma=None, beta=None, eps=1e-5, activation="identity"):
    """BatchNorm::forward_cpu with fixed statistics (src/ops/batch_normalization.cpp:176-181): per channel
    alpha = 1/sqrt(var + eps), beta' = -mean * alpha, with gamma/beta alpha *= gamma, beta' = gamma * beta' + beta
    (compute_conv_parameters, :210-227), then y = alpha * x + beta' (cpu_forward_data, :196-206), all in float32,
    and the operator's activation.  Pinned against torch.nn.functional.batch_norm in tests/test_glue_ops.py."""
    x = _f32(x)
    one = np.float32(1.0)
    alpha = one / np.sqrt(_f32(var) + np.float32(eps))
    shift = -_f32(mean) * alpha
    if gamma is not None:
        alpha = alpha * _f32(gamma)
        shift = _f32(gamma) * shift + _f32(beta)
    shape = (1, -1) + (1,) * (x.ndim - 2)
    y = alpha.reshape(shape) * x + shift.reshape(shape)
    return apply_activation(y.astype(np.float32), activation).reshape(x.shape)


def softmax_forward(x, log=False):
    """Softmax::forward_cpu, src/ops/softmax.cpp:189-222: over dimension 1 of [B, C] or [B, C, S]; per column the maximum,
    sum of expf(x - max) in float32 in index order, then expf(x - max) * (1 / sum), or x - max - logf(sum) for log."""
    x = _f32(x)
    shape = x.shape
    v = x.reshape(shape[0], shape[1], -1)
    m = v.max(axis=1, keepdims=True)
    e = np.exp((v - m).astype(np.float32)).astype(np.float32)
    total = np.zeros((v.shape[0], 1, v.shape[2]), dtype=np.float32)
    for j in range(v.shape[1]):
        total[:, 0, :] += e[:, j, :]
    if log:
        y = (v - m) + (-np.log(total)).astype(np.float32)
    else:
        y = e * (np.float32(1.0) / total)
    return y.astype(np.float32).reshape(shape)


def interpolate_output_size(in_hw, out_hw=(-1, -1), scale=(-1.0, -1.0)):
    """Interpolation::calc_size, src/ops/interpolation.cpp:53-69: the given size, or int(in * scale) per axis"""
    if out_hw[0] > 0:
        return int(out_hw[0]), int(out_hw[1])
    return int(in_hw[0] * scale[0]), int(in_hw[1] * scale[1])


def _interp_step(scale, src, tgt, align_corners):
    """Interpolation::calc_bin_scale, src/ops/interpolation.cpp:121-131 (float results)"""
    if align_corners:
        return np.float32(0) if tgt <= 1 else np.float32(float(src - 1) / (tgt - 1))
    if scale > 0:
        return np.float32(1.0 / scale)
    return np.float32(float(src) / tgt)


def interpolate2d_forward(x, out_hw, method="nearest", scale=(-1.0, -1.0), align_corners=False):
    """Interpolation::forward on the CPU, src/ops/interpolation.cpp: nearest / nearest-exact as forward_cpu (:271-305: source index
    min(int((p + offset) * step), size - 1), offset 0 or 0.5, step float(1 / scale) or float(in) / out), bilinear as
    bilinear_fwd_bwd_cpu with HandleFWD (:86-96,133-195: position max(step * (p + 0.5) - 0.5, 0) or step * p with align_corners,
    neighbours p0 and p0 + 1 (clamped), weights from the fraction), all in float32.  The HIP bilinear kernel blends along the row
    and then between rows, this restatement follows the reference's four weighted taps: tests compare the two to a tolerance
    (nearest is compared bit for bit)."""
    x = _f32(x)
    B, C, H, W = x.shape
    OH, OW = out_hw
    f = np.float32
    if method in ("nearest", "nearest-exact"):
        vs = f(1.0 / scale[0]) if scale[0] > 0 else f(H) / f(OH)
        hs = f(1.0 / scale[1]) if scale[1] > 0 else f(W) / f(OW)
        offset = f(0.0 if method == "nearest" else 0.5)
        rows = np.minimum(((np.arange(OH, dtype=np.float32) + offset) * vs).astype(np.int32), H - 1)
        cols = np.minimum(((np.arange(OW, dtype=np.float32) + offset) * hs).astype(np.int32), W - 1)
        return np.ascontiguousarray(x[:, :, rows][:, :, :, cols])
    assert method == "bilinear"

    def axis(step, size, n):
        p = np.arange(n, dtype=np.float32)
        pos = step * p if align_corners else np.maximum(step * (p + f(0.5)) - f(0.5), f(0))
        pos = pos.astype(np.float32)
        p0 = pos.astype(np.int32)
        p1 = p0 + (p0 < size - 1)
        w1 = (pos - p0.astype(np.float32)).astype(np.float32)
        return p0, p1, (f(1) - w1).astype(np.float32), w1

    r0, r1, wr0, wr1 = axis(_interp_step(scale[0], H, OH, align_corners), H, OH)
    c0, c1, wc0, wc1 = axis(_interp_step(scale[1], W, OW, align_corners), W, OW)
    top = wc0 * x[:, :, r0][:, :, :, c0] + wc1 * x[:, :, r0][:, :, :, c1]
    bottom = wc0 * x[:, :, r1][:, :, :, c0] + wc1 * x[:, :, r1][:, :, :, c1]
    y = wr0[:, None] * top.astype(np.float32) + wr1[:, None] * bottom.astype(np.float32)
    return y.astype(np.float32)


def reduction_dims(rank, dims=None, start_axis=0):
    """Reduction::setup, src/ops/reduction.cpp:49-69: the axes that are reduced"""
    if dims is None:
        if start_axis < 0:
            start_axis += rank
        assert 0 <= start_axis < rank
        return list(range(start_axis, rank))
    return sorted({d + rank if d < 0 else d for d in dims})


def reduction_forward(x, method="sum", dims=None, start_axis=0, output_scale=1.0, keep_dim=True):
    """Reduction::forward_cpu, src/ops/reduction.cpp:296-330: float32 sums of x, x*x or |x| in memory order into the kept positions,
    then one multiplication by output_scale (mean: output_scale * outputs / elements, get_coeff :323-329); the output shape keeps
    the reduced axes as 1 or drops them (calc_shapes :133-151)."""
    x = _f32(x)
    axes = reduction_dims(x.ndim, dims, start_axis)
    term = {"sum": x, "mean": x, "sumsq": x * x, "abssum": np.abs(x)}[method]
    # sequential float32 accumulation in memory order: move the reduced axes behind the kept ones, keeping their order
    kept = [a for a in range(x.ndim) if a not in axes]
    t = np.transpose(term, kept + axes).reshape(int(np.prod([x.shape[a] for a in kept], dtype=np.int64)), -1)
    acc = np.zeros(t.shape[0], dtype=np.float32)
    for j in range(t.shape[1]):
        acc += t[:, j]
    coeff = np.float32(output_scale)
    if method == "mean":
        coeff = np.float32(np.float32(output_scale) * np.float32(acc.size) / np.float32(x.size))
    if coeff != np.float32(1.0):
        acc = acc * coeff
    shape = [1 if a in axes else x.shape[a] for a in range(x.ndim)] if keep_dim else [x.shape[a] for a in kept]
    return acc.astype(np.float32).reshape(shape if shape else [1])


def mse_loss_forward(a, b, reduce="mean"):
    """MSELoss::forward_cpu, src/ops/mse_loss.cpp:70-92: (a - b)^2 per element, or their float32 sum in index order (mean: * 1 / size)"""
    a, b = _f32(a), _f32(b)
    d = (a - b).astype(np.float32)
    sq = (d * d).astype(np.float32)
    if reduce == "none":
        return sq
    total = np.float32(0)
    for v in sq.reshape(-1):
        total = np.float32(total + v)
    if reduce == "mean":
        total = np.float32(total * np.float32(1.0 / a.size))
    return np.array([total], dtype=np.float32)


def nll_loss_forward(x, labels, reduce="mean"):
    """NLLLoss::forwad_cpu, src/ops/nll_loss.cpp:59-86: -x[b][label[b]] per row (0 for a label outside the classes), or the float32 sum
    over the rows (mean: * 1 / batch)"""
    x = _f32(x)
    idx = np.asarray(labels).astype(np.int64).reshape(-1)
    ok = (idx >= 0) & (idx < x.shape[1])
    rows = np.where(ok, -x[np.arange(x.shape[0]), np.clip(idx, 0, x.shape[1] - 1)], np.float32(0)).astype(np.float32)
    if reduce == "none":
        return rows
    total = np.float32(0)
    for v in rows:
        total = np.float32(total + v)
    if reduce == "mean":
        total = np.float32(total * np.float32(1.0 / x.shape[0]))
    return np.array([total], dtype=np.float32)


def softmax_loss_forward(x, labels):
    """SoftmaxWithLoss::forward_cpu_loss, src/ops/softmax.cpp:134-155: per row the maximum, the float32 sum of expf(x - max) in index
    order, loss -= x[label] - max - logf(sum); the total divided by the batch.  (The CPU code checks label < classes; the kernel,
    src/kernels/softmax_with_loss.cl, adds 0 for such a row -- the behaviour kept here.)"""
    x = _f32(x)
    idx = np.asarray(labels).astype(np.int64).reshape(-1)
    total = np.float32(0)
    for b in range(x.shape[0]):
        m = x[b].max()
        s = np.float32(0)
        for v in np.exp((x[b] - m).astype(np.float32)).astype(np.float32):
            s = np.float32(s + v)
        if 0 <= idx[b] < x.shape[1]:
            total = np.float32(total - np.float32(np.float32(x[b, idx[b]] - m) - np.log(s).astype(np.float32)))
    return np.array([np.float32(total / np.float32(x.shape[0]))], dtype=np.float32)


def bf16_round(a):
    a = _f32(a).copy()
    lib().orc_bf16_round_array(_ptr(a), ctypes.c_size_t(a.size))
    return a


# --- the compiled reference pieces (oracle/_ref) ---------------------------------

def ref_sgemm(A, B, trans_a=False, trans_b=False, C=None, alpha=1.0, beta=0.0):
    R = ref()
    A, B = _f32(A), _f32(B)
    M = A.shape[1] if trans_a else A.shape[0]
    K = A.shape[0] if trans_a else A.shape[1]
    N = B.shape[0] if trans_b else B.shape[1]
    C = np.zeros((M, N), dtype=np.float32) if C is None else _f32(C).copy()
    R.ref_cblas_sgemm(int(trans_a), int(trans_b), M, N, K, ctypes.c_float(alpha), _ptr(A), A.shape[1], _ptr(B), B.shape[1], ctypes.c_float(beta), _ptr(C), N)
    return C


def ref_apply_activation(a, activation):
    a = _f32(a).copy()
    ref().ref_apply_activation(_ptr(a), ctypes.c_size_t(a.size), _act(activation))
    return a
