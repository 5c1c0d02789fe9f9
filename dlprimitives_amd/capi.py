"""ctypes binding of include/dlprim_hip.h, mirroring dlprim::core's operator API.

Names follow the reference (include/dlprim/core/conv.hpp:17-58,
include/dlprim/core/ip.hpp:19-45): ``Conv2DSettings``, ``Conv2DForward.create``
/ ``enqueue`` / ``algo`` / ``workspace`` / ``get_output_shape``, ``IPSettings``,
``IPForward.create`` / ``enqueue``.  Errors come back as the reference's
exception kinds (ValidationError, NotImplementedError).

There is no fallback of any kind: if the HIP library is missing, loading fails.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libdlprim_hip.so")

ACTIVATIONS = {"identity": 0, "relu": 1, "tanh": 2, "sigmoid": 3, "relu6": 4}
FLOAT_DATA, HALF_DATA, BFLOAT16_DATA = 3, 2, 10


class DlprimError(RuntimeError):
    pass


class ValidationError(DlprimError):
    """dlprim::ValidationError"""


class NotImplementedErrorDlprim(DlprimError):
    """dlprim::NotImplementedError"""


class _Settings(ctypes.Structure):
    _fields_ = [
        ("channels_in", ctypes.c_int),
        ("channels_out", ctypes.c_int),
        ("kernel", ctypes.c_int * 2),
        ("stride", ctypes.c_int * 2),
        ("dilate", ctypes.c_int * 2),
        ("pad", ctypes.c_int * 2),
        ("groups", ctypes.c_int),
        ("shape", ctypes.c_int * 4),
        ("dtype", ctypes.c_int),
    ]


class _IPSettings(ctypes.Structure):
    _fields_ = [
        ("inputs", ctypes.c_int),
        ("outputs", ctypes.c_int),
        ("optimal_batch_size", ctypes.c_int),
        ("dtype", ctypes.c_int),
    ]


def library_path():
    return _LIB


def build_library():
    """Compile libdlprim_hip.so for gfx950 (hipcc cross-compiles without a GPU)."""
    subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), "-j8"], check=True, stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise DlprimError(
                "libdlprim_hip.so is not built (%s); run `make -C dlprimitives_amd/csrc` -- there is no CPU fallback" % _LIB)
        # This binding works on torch tensors, and torch ships a HIP runtime of its own: it has to be the one
        # the process loads first.  With the library (and the system's runtime behind it) loaded before torch,
        # torch's own initialisation afterwards reports "No HIP GPUs are available".
        import torch  # noqa: F401

        L = ctypes.CDLL(_LIB)
        L.dlp_last_error.restype = ctypes.c_char_p
        L.dlp_conv2d_fwd_algo.restype = ctypes.c_char_p
        L.dlp_conv2d_fwd_algo.argtypes = [ctypes.c_void_p]
        L.dlp_conv2d_fwd_workspace.restype = ctypes.c_size_t
        L.dlp_conv2d_fwd_workspace.argtypes = [ctypes.c_void_p]
        L.dlp_conv2d_fwd_create.argtypes = [ctypes.POINTER(_Settings), ctypes.c_int, ctypes.c_int, ctypes.c_char_p,
                                            ctypes.POINTER(ctypes.c_void_p)]
        L.dlp_conv2d_fwd_enqueue.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.c_void_p, ctypes.c_void_p,
                                             ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float,
                                             ctypes.c_void_p]
        L.dlp_conv2d_fwd_destroy.argtypes = [ctypes.c_void_p]
        L.dlp_conv2d_fwd_destroy.restype = None
        for kind in ("data", "filter"):
            pre = "dlp_conv2d_bwd_%s_" % kind
            getattr(L, pre + "create").argtypes = [ctypes.POINTER(_Settings), ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
            getattr(L, pre + "algo").restype = ctypes.c_char_p
            getattr(L, pre + "algo").argtypes = [ctypes.c_void_p]
            getattr(L, pre + "workspace").restype = ctypes.c_size_t
            getattr(L, pre + "workspace").argtypes = [ctypes.c_void_p]
            getattr(L, pre + "enqueue").argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                    ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_void_p]
            getattr(L, pre + "destroy").argtypes = [ctypes.c_void_p]
            getattr(L, pre + "destroy").restype = None
        L.dlp_bias_bwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float,
                                           ctypes.c_void_p]
        L.dlp_conv2d_output_shape.argtypes = [ctypes.POINTER(_Settings), ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.dlp_ip_fwd_create.argtypes = [ctypes.POINTER(_IPSettings), ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_void_p)]
        L.dlp_ip_fwd_enqueue.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_void_p, ctypes.c_void_p]
        L.dlp_ip_fwd_enqueue_no_alloc.argtypes = L.dlp_ip_fwd_enqueue.argtypes
        L.dlp_ip_fwd_destroy.argtypes = [ctypes.c_void_p]
        L.dlp_ip_fwd_destroy.restype = None
        _lib = L
    return _lib


def timing_enable(on=True):
    """ExecutionContext::enable_timing analogue: bracket every kernel launch with HIP events."""
    _check(lib().dlp_timing_enable(1 if on else 0))


def timing_reset():
    _check(lib().dlp_timing_reset())


def timing_count():
    n = ctypes.c_int()
    _check(lib().dlp_timing_count(ctypes.byref(n)))
    return n.value


def timing_records(first=0, last=None, kernels=False):
    """[(section, milliseconds)] of the kernels launched since the last reset (waits for them);
    with kernels=True [(section, milliseconds, kernel name as a profiler lists it)]."""
    last = timing_count() if last is None else last
    out = []
    name = ctypes.create_string_buffer(64)
    kname = ctypes.create_string_buffer(256)
    ms = ctypes.c_float()
    for i in range(first, last):
        _check(lib().dlp_timing_get(i, name, 64, ctypes.byref(ms)))
        if kernels:
            _check(lib().dlp_timing_get_kernel(i, kname, 256))
            out.append((name.value.decode(), ms.value, kname.value.decode()))
        else:
            out.append((name.value.decode(), ms.value))
    return out


def _check(rc):
    if rc == 0:
        return
    msg = lib().dlp_last_error().decode()
    if rc == 1:
        raise ValidationError(msg)
    if rc == 2:
        raise NotImplementedErrorDlprim(msg)
    raise DlprimError(msg)


def _pair(v):
    if isinstance(v, (tuple, list)):
        return int(v[0]), int(v[1])
    return int(v), int(v)


def _act(a):
    return ACTIVATIONS[a] if isinstance(a, str) else int(a)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _stream(stream):
    if stream is None:
        import torch

        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    return ctypes.c_void_p(int(stream))


class Conv2DSettings:
    """core::Conv2DSettings: Convolution2DConfigBase + input shape (batch is a hint) + dtype."""

    def __init__(self, channels_in, channels_out, kernel, stride=1, dilate=1, pad=0, groups=1, shape=None, dtype=FLOAT_DATA):
        self.channels_in, self.channels_out, self.groups = int(channels_in), int(channels_out), int(groups)
        self.kernel, self.stride, self.dilate, self.pad = _pair(kernel), _pair(stride), _pair(dilate), _pair(pad)
        self.shape = tuple(int(v) for v in shape)
        self.dtype = dtype

    def _c(self):
        s = _Settings()
        s.channels_in, s.channels_out, s.groups, s.dtype = self.channels_in, self.channels_out, self.groups, self.dtype
        s.kernel[:], s.stride[:], s.dilate[:], s.pad[:] = self.kernel, self.stride, self.dilate, self.pad
        s.shape[:] = self.shape
        return s


def conv2d_output_shape(settings, in_shape):
    """Conv2DBase::get_output_shape"""
    ish = (ctypes.c_int * 4)(*[int(v) for v in in_shape])
    osh = (ctypes.c_int * 4)()
    c = settings._c()
    _check(lib().dlp_conv2d_output_shape(ctypes.byref(c), ish, osh))
    return tuple(osh)


class Conv2DForward:
    """core::Conv2DForward"""

    def __init__(self, handle, settings):
        self._h = handle
        self.settings = settings

    @staticmethod
    def create(settings, bias, activation="identity", algo=""):
        h = ctypes.c_void_p()
        c = settings._c()
        _check(lib().dlp_conv2d_fwd_create(ctypes.byref(c), int(bool(bias)), _act(activation), (algo or "").encode(), ctypes.byref(h)))
        return Conv2DForward(h, settings)

    get_output_shape = staticmethod(conv2d_output_shape)

    def algo(self):
        return lib().dlp_conv2d_fwd_algo(self._h).decode()

    def workspace(self):
        return int(lib().dlp_conv2d_fwd_workspace(self._h))

    def enqueue(self, x, w, bias, y, ws=None, factor=0.0, stream=None):
        """x, w, bias, y, ws: torch device tensors (ws: uint8 of >= workspace() bytes)."""
        xs = self._x_shape(x)
        ws_bytes = ws.numel() * ws.element_size() if ws is not None else 0
        _check(lib().dlp_conv2d_fwd_enqueue(self._h, xs, _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _ptr(ws), ws_bytes,
                                            float(factor), _stream(stream)))

    def accumulate_before_activation(self, on=True):
        """y = act(conv + bias + factor * y) instead of factor * y + act(conv + bias)"""
        lib().dlp_conv2d_fwd_set_accumulate_first.argtypes = [ctypes.c_void_p, ctypes.c_int]
        _check(lib().dlp_conv2d_fwd_set_accumulate_first(self._h, int(bool(on))))

    def channels_last(self, x=False, y=False):
        """dlp_conv2d_fwd_set_channels_last: the operator reads x / writes y as [image][row][column][channel] (bfloat16 gemm
        only; NotImplementedError otherwise).  Call before workspace().  A channels-last x is passed to enqueue as a tensor
        of shape [B, H, W, C]."""
        lib().dlp_conv2d_fwd_set_channels_last.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        _check(lib().dlp_conv2d_fwd_set_channels_last(self._h, int(bool(x)), int(bool(y))))
        self._x_channels_last = bool(x)

    def fuse_max_pool(self, kernel=3, stride=2, pad=1, ceil_mode=False):
        """dlp_conv2d_fwd_fuse_max_pool: enqueue writes max_pool(act(conv + bias)), a tensor of the pooled shape, and never the
        convolution's own output (the bfloat16 stem of a ResNet and its 3x3 stride-2 pad-1 pooling; NotImplementedError otherwise)"""
        lib().dlp_conv2d_fwd_fuse_max_pool.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        _check(lib().dlp_conv2d_fwd_fuse_max_pool(self._h, int(kernel), int(stride), int(pad), int(bool(ceil_mode))))

    def _x_shape(self, x):
        """the [B, C, H, W] that the C interface takes, whatever the layout of x"""
        if getattr(self, "_x_channels_last", False):
            return (ctypes.c_int * 4)(int(x.shape[0]), self.settings.channels_in, self.settings.shape[2], self.settings.shape[3])
        return (ctypes.c_int * 4)(*x.shape)

    def packed_size(self):
        """bytes of the buffer that pack() fills (0: nothing to transform)"""
        lib().dlp_conv2d_fwd_packed_bytes.restype = ctypes.c_size_t
        lib().dlp_conv2d_fwd_packed_bytes.argtypes = [ctypes.c_void_p]
        return int(lib().dlp_conv2d_fwd_packed_bytes(self._h))

    def pack(self, w, packed, stream=None):
        """transform weights that stay constant once; packed: uint8 device tensor of packed_size() bytes"""
        lib().dlp_conv2d_fwd_pack.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        _check(lib().dlp_conv2d_fwd_pack(self._h, _ptr(w), _ptr(packed), _stream(stream)))

    def enqueue_packed(self, x, w, packed, bias, y, ws=None, factor=0.0, stream=None):
        """enqueue() on weights that pack() transformed earlier; ws is per-call scratch only"""
        lib().dlp_conv2d_fwd_enqueue_packed.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float,
                                                        ctypes.c_void_p]
        xs = self._x_shape(x)
        ws_bytes = ws.numel() * ws.element_size() if ws is not None else 0
        _check(lib().dlp_conv2d_fwd_enqueue_packed(self._h, xs, _ptr(x), _ptr(w), _ptr(packed), _ptr(bias), _ptr(y), _ptr(ws), ws_bytes,
                                                   float(factor), _stream(stream)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().dlp_conv2d_fwd_destroy(self._h)
            self._h = None


class DepthwisePointwiseForward:
    """Depthwise 3x3 + pointwise 1x1 convolution in one launch (dlp_dwpw_fwd_*): no counterpart in the reference,
    which runs them as two Convolution2D operators with the depthwise result written to memory in between."""

    def __init__(self, handle, settings, channels_out):
        self._h = handle
        self.settings = settings
        self.channels_out = channels_out

    @staticmethod
    def supported(settings, dw_activation, channels_out, pw_activation):
        L = lib()
        L.dlp_dwpw_fwd_supported.argtypes = [ctypes.POINTER(_Settings), ctypes.c_int, ctypes.c_int, ctypes.c_int]
        c = settings._c()
        return bool(L.dlp_dwpw_fwd_supported(ctypes.byref(c), _act(dw_activation), int(channels_out), _act(pw_activation)))

    @staticmethod
    def create(settings, dw_bias, dw_activation, channels_out, pw_bias, pw_activation="identity"):
        """settings: the depthwise layer (groups = channels, kernel 3, pad 1, stride 1 or 2, shape of x)"""
        L = lib()
        L.dlp_dwpw_fwd_create.argtypes = [ctypes.POINTER(_Settings), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                          ctypes.POINTER(ctypes.c_void_p)]
        L.dlp_dwpw_fwd_enqueue.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p]
        L.dlp_dwpw_fwd_set_accumulate_first.argtypes = [ctypes.c_void_p, ctypes.c_int]
        L.dlp_dwpw_fwd_destroy.argtypes = [ctypes.c_void_p]
        L.dlp_dwpw_fwd_destroy.restype = None
        h = ctypes.c_void_p()
        c = settings._c()
        _check(L.dlp_dwpw_fwd_create(ctypes.byref(c), int(bool(dw_bias)), _act(dw_activation), int(channels_out), int(bool(pw_bias)),
                                     _act(pw_activation), ctypes.byref(h)))
        return DepthwisePointwiseForward(h, settings, int(channels_out))

    def accumulate_before_activation(self, on=True):
        _check(lib().dlp_dwpw_fwd_set_accumulate_first(self._h, int(bool(on))))

    def enqueue(self, x, dw_w, dw_bias, pw_w, pw_bias, y, factor=0.0, stream=None):
        xs = (ctypes.c_int * 4)(*x.shape)
        _check(lib().dlp_dwpw_fwd_enqueue(self._h, xs, _ptr(x), _ptr(dw_w), _ptr(dw_bias), _ptr(pw_w), _ptr(pw_bias), _ptr(y), float(factor),
                                          _stream(stream)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().dlp_dwpw_fwd_destroy(self._h)
            self._h = None


class _Conv2DBackward:
    _kind = None

    def __init__(self, handle, settings):
        self._h = handle
        self.settings = settings

    @classmethod
    def create(cls, settings, algo=""):
        h = ctypes.c_void_p()
        c = settings._c()
        _check(getattr(lib(), "dlp_conv2d_bwd_%s_create" % cls._kind)(ctypes.byref(c), (algo or "").encode(), ctypes.byref(h)))
        return cls(h, settings)

    def algo(self):
        return getattr(lib(), "dlp_conv2d_bwd_%s_algo" % self._kind)(self._h).decode()

    def workspace(self):
        return int(getattr(lib(), "dlp_conv2d_bwd_%s_workspace" % self._kind)(self._h))

    def __del__(self):
        if getattr(self, "_h", None):
            getattr(lib(), "dlp_conv2d_bwd_%s_destroy" % self._kind)(self._h)
            self._h = None


class Conv2DBackwardData(_Conv2DBackward):
    """core::Conv2DBackwardData"""

    _kind = "data"

    def enqueue(self, dx, w, dy, ws=None, factor=0.0, stream=None):
        """dx = factor * dx + gradient with respect to x; ws: uint8 tensor of >= workspace() bytes"""
        xs = (ctypes.c_int * 4)(*dx.shape)
        ws_bytes = ws.numel() * ws.element_size() if ws is not None else 0
        _check(lib().dlp_conv2d_bwd_data_enqueue(self._h, xs, _ptr(dx), _ptr(w), _ptr(dy), _ptr(ws), ws_bytes, float(factor), _stream(stream)))


class Conv2DBackwardFilter(_Conv2DBackward):
    """core::Conv2DBackwardFilter"""

    _kind = "filter"

    def enqueue(self, x, dw, dy, ws=None, factor=0.0, stream=None):
        """dw = factor * dw + gradient with respect to the filter"""
        xs = (ctypes.c_int * 4)(*x.shape)
        ws_bytes = ws.numel() * ws.element_size() if ws is not None else 0
        _check(lib().dlp_conv2d_bwd_filter_enqueue(self._h, xs, _ptr(x), _ptr(dw), _ptr(dy), _ptr(ws), ws_bytes, float(factor), _stream(stream)))


def conv2d_transposed_output_shape(settings, in_shape, output_pad=(0, 0)):
    """Conv2DBase::get_output_shape_transposed"""
    L = lib()
    L.dlp_conv2d_transposed_output_shape.argtypes = [ctypes.POINTER(_Settings), ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                                     ctypes.POINTER(ctypes.c_int)]
    ish = (ctypes.c_int * 4)(*[int(v) for v in in_shape])
    osh = (ctypes.c_int * 4)()
    c = settings._c()
    _check(L.dlp_conv2d_transposed_output_shape(ctypes.byref(c), ish, (ctypes.c_int * 2)(*_pair(output_pad)), osh))
    return tuple(osh)


class TransposedConv2DForward:
    """TransposedConvolution2D::forward on the device: `settings` describe the transposed operator
    (channels_in = channels of x, shape = shape of x); w is [channels_in, channels_out / groups, kh, kw]."""

    def __init__(self, handle, settings, output_pad):
        self._h = handle
        self.settings = settings
        self.output_pad = output_pad

    @staticmethod
    def create(settings, output_pad=(0, 0), bias=True, activation="identity", algo=""):
        L = lib()
        L.dlp_tconv2d_fwd_create.argtypes = [ctypes.POINTER(_Settings), ctypes.POINTER(ctypes.c_int), ctypes.c_int, ctypes.c_int, ctypes.c_char_p,
                                             ctypes.POINTER(ctypes.c_void_p)]
        L.dlp_tconv2d_fwd_algo.restype = ctypes.c_char_p
        L.dlp_tconv2d_fwd_algo.argtypes = [ctypes.c_void_p]
        L.dlp_tconv2d_fwd_workspace.restype = ctypes.c_size_t
        L.dlp_tconv2d_fwd_workspace.argtypes = [ctypes.c_void_p]
        L.dlp_tconv2d_fwd_enqueue.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                              ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
        L.dlp_tconv2d_fwd_destroy.argtypes = [ctypes.c_void_p]
        L.dlp_tconv2d_fwd_destroy.restype = None
        h = ctypes.c_void_p()
        c = settings._c()
        _check(L.dlp_tconv2d_fwd_create(ctypes.byref(c), (ctypes.c_int * 2)(*_pair(output_pad)), int(bool(bias)), _act(activation),
                                        (algo or "").encode(), ctypes.byref(h)))
        return TransposedConv2DForward(h, settings, _pair(output_pad))

    def algo(self):
        return lib().dlp_tconv2d_fwd_algo(self._h).decode()

    def workspace(self):
        return int(lib().dlp_tconv2d_fwd_workspace(self._h))

    def output_shape(self, in_shape):
        return conv2d_transposed_output_shape(self.settings, in_shape, self.output_pad)

    def enqueue(self, x, w, bias, y, ws=None, stream=None):
        xs = (ctypes.c_int * 4)(*x.shape)
        ws_bytes = ws.numel() * ws.element_size() if ws is not None else 0
        _check(lib().dlp_tconv2d_fwd_enqueue(self._h, xs, _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _ptr(ws), ws_bytes, _stream(stream)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().dlp_tconv2d_fwd_destroy(self._h)
            self._h = None


def bias_backward(dy, db, beta=0.0, stream=None):
    """core::BiasBackwardFilter::enqueue: db[f] = beta * db[f] + sum of dy[:, f] over batch and plane"""
    batch, features = int(dy.shape[0]), int(dy.shape[1])
    plane = dy.numel() // max(batch * features, 1) if batch else 1
    _check(lib().dlp_bias_bwd_enqueue(torch_dtype_code(dy), batch, features, max(plane, 1), _ptr(dy), _ptr(db), float(beta), _stream(stream)))


class IPSettings:
    """core::IPSettings"""

    def __init__(self, inputs, outputs, optimal_batch_size=-1, dtype=FLOAT_DATA):
        self.inputs, self.outputs, self.optimal_batch_size, self.dtype = int(inputs), int(outputs), int(optimal_batch_size), dtype

    def _c(self):
        s = _IPSettings()
        s.inputs, s.outputs, s.optimal_batch_size, s.dtype = self.inputs, self.outputs, self.optimal_batch_size, self.dtype
        return s


class IPForward:
    """core::IPForward"""

    def __init__(self, handle, settings):
        self._h = handle
        self.settings = settings

    @staticmethod
    def create(settings, bias, activation="identity"):
        h = ctypes.c_void_p()
        c = settings._c()
        _check(lib().dlp_ip_fwd_create(ctypes.byref(c), int(bool(bias)), _act(activation), ctypes.byref(h)))
        return IPForward(h, settings)

    def enqueue(self, x, w, bias, y, stream=None):
        _check(lib().dlp_ip_fwd_enqueue(self._h, int(x.shape[0]), _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _stream(stream)))

    def enqueue_no_alloc(self, x, w, bias, y, stream=None):
        """enqueue() with its scratch in the library's own device array: no device allocation, bounded sizes"""
        _check(lib().dlp_ip_fwd_enqueue_no_alloc(self._h, int(x.shape[0]), _ptr(x), _ptr(w), _ptr(bias), _ptr(y), _stream(stream)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().dlp_ip_fwd_destroy(self._h)
            self._h = None


# ---- glue operators (pooling, global pooling, elementwise) ---------------------------

def pool2d_output_size(in_size, kernel, pad, stride, ceil_mode=False):
    """core::calc_pooling_output_size"""
    out = ctypes.c_int()
    _check(lib().dlp_pool2d_output_size(int(in_size), int(kernel), int(pad), int(stride), int(bool(ceil_mode)), ctypes.byref(out)))
    return out.value


class Pooling2DForward:
    """core::Pooling2DForward"""

    def __init__(self, handle):
        self._h = handle

    @staticmethod
    def _create(fn, *args):
        h = ctypes.c_void_p()
        _check(fn(*args, ctypes.byref(h)))
        return Pooling2DForward(h)

    @staticmethod
    def create_max_pooling(kernel, pad, stride, dtype=FLOAT_DATA):
        i2 = ctypes.c_int * 2
        return Pooling2DForward._create(lib().dlp_pool2d_fwd_create_max, i2(*_pair(kernel)), i2(*_pair(pad)), i2(*_pair(stride)), dtype)

    @staticmethod
    def create_avg_pooling(kernel, pad, stride, count_include_pad=False, dtype=FLOAT_DATA):
        i2 = ctypes.c_int * 2
        return Pooling2DForward._create(lib().dlp_pool2d_fwd_create_avg, i2(*_pair(kernel)), i2(*_pair(pad)), i2(*_pair(stride)),
                                        int(bool(count_include_pad)), dtype)

    @staticmethod
    def create_global_max_pooling(dtype=FLOAT_DATA):
        return Pooling2DForward._create(lib().dlp_pool2d_fwd_create_global_max, dtype)

    @staticmethod
    def create_global_avg_pooling(dtype=FLOAT_DATA):
        return Pooling2DForward._create(lib().dlp_pool2d_fwd_create_global_avg, dtype)

    def workspace(self):
        return 0

    def channels_last(self, on=True):
        """dlp_pool2d_fwd_set_channels_last (global pooling only): x is passed to enqueue as a tensor of shape [B, H, W, C]"""
        lib().dlp_pool2d_fwd_set_channels_last.argtypes = [ctypes.c_void_p, ctypes.c_int]
        _check(lib().dlp_pool2d_fwd_set_channels_last(self._h, int(bool(on))))
        self._channels_last = bool(on)

    def enqueue(self, x, y, stream=None):
        if getattr(self, "_channels_last", False):
            xs = (ctypes.c_int * 4)(int(x.shape[0]), int(x.shape[3]), int(x.shape[1]), int(x.shape[2]))
        else:
            xs = (ctypes.c_int * 4)(*x.shape)
        ys = (ctypes.c_int * 4)(*y.shape)
        lib().dlp_pool2d_fwd_enqueue.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int), ctypes.c_void_p,
                                                 ctypes.c_void_p, ctypes.c_void_p]
        _check(lib().dlp_pool2d_fwd_enqueue(self._h, xs, ys, _ptr(x), _ptr(y), _stream(stream)))

    def __del__(self):
        if getattr(self, "_h", None):
            lib().dlp_pool2d_fwd_destroy.argtypes = [ctypes.c_void_p]
            lib().dlp_pool2d_fwd_destroy.restype = None
            lib().dlp_pool2d_fwd_destroy(self._h)
            self._h = None


ELTWISE_OPS = {"sum": 0, "prod": 1, "max": 2}


def torch_dtype_code(t):
    """dlprim DataType of a torch tensor (float32 -> float_data, bfloat16 -> bfloat16_data)."""
    import torch

    if t.dtype == torch.float32:
        return FLOAT_DATA
    if t.dtype == torch.bfloat16:
        return BFLOAT16_DATA
    raise ValidationError("unsupported tensor dtype %s" % t.dtype)


def eltwise_forward(a, b, c, operation="sum", coef1=1.0, coef2=1.0, activation="identity", stream=None):
    """Elementwise::forward: c = act(op(coef1*a, coef2*b)); shapes that differ broadcast by numpy's rule (c has the broadcast shape)"""
    if tuple(a.shape) != tuple(b.shape):
        rank = max(a.dim(), b.dim())
        sa = [1] * (rank - a.dim()) + [int(d) for d in a.shape]
        sb = [1] * (rank - b.dim()) + [int(d) for d in b.shape]
        arr = ctypes.c_int * rank
        lib().dlp_eltwise_bcast_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_int,
                                                        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        _check(lib().dlp_eltwise_bcast_fwd_enqueue(torch_dtype_code(a), ELTWISE_OPS[operation], float(coef1), float(coef2), _act(activation), rank,
                                                   arr(*sa), arr(*sb), _ptr(a), _ptr(b), _ptr(c), _stream(stream)))
        return
    lib().dlp_eltwise_fwd_enqueue_dtype.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_size_t,
                                                    ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    _check(lib().dlp_eltwise_fwd_enqueue_dtype(torch_dtype_code(a), ELTWISE_OPS[operation], float(coef1), float(coef2), _act(activation),
                                               a.numel(), _ptr(a), _ptr(b), _ptr(c), _stream(stream)))


def slice_copy(dst, dst_offset, src, src_offset, length, dim=1, stream=None):
    """The copy of Concat::forward / Slice::forward: dst[..., dst_offset:dst_offset+length, ...] = src[..., src_offset:src_offset+length, ...]
    along axis `dim` of two contiguous tensors that agree in every other dimension."""
    if dst.dim() != src.dim() or dst.dtype != src.dtype or not (dst.is_contiguous() and src.is_contiguous()):
        raise ValidationError("slice_copy: contiguous tensors of the same rank and type are needed")
    for j in range(dst.dim()):
        if j != dim and dst.shape[j] != src.shape[j]:
            raise ValidationError("slice_copy: the tensors differ outside the axis")
    if dst_offset < 0 or src_offset < 0 or dst_offset + length > dst.shape[dim] or src_offset + length > src.shape[dim]:
        raise ValidationError("slice_copy: range outside the axis")
    es = dst.element_size()
    outer = 1
    for j in range(dim):
        outer *= int(dst.shape[j])
    inner = es
    for j in range(dim + 1, dst.dim()):
        inner *= int(dst.shape[j])
    lib().dlp_copy2d_enqueue.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_size_t, ctypes.c_void_p]
    _check(lib().dlp_copy2d_enqueue(dst.data_ptr() + dst_offset * inner, int(dst.shape[dim]) * inner, src.data_ptr() + src_offset * inner,
                                    int(src.shape[dim]) * inner, length * inner, outer, _stream(stream)))


def activation_forward(x, y, activation, stream=None):
    """Activation::forward: y = act(x); y may be x"""
    lib().dlp_activation_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    _check(lib().dlp_activation_fwd_enqueue(torch_dtype_code(x), _act(activation), x.numel(), _ptr(x), _ptr(y), _stream(stream)))


def channel_affine_forward(x, scale, shift, y, activation="identity", stream=None):
    """BatchNorm::forward with fixed statistics: y[b,c,...] = act(x[b,c,...] * scale[c] + shift[c]); scale and shift are float32"""
    if x.dim() < 2 or scale.numel() != x.shape[1] or shift.numel() != x.shape[1]:
        raise ValidationError("channel_affine: scale/shift need one value per channel")
    batch, channels = int(x.shape[0]), int(x.shape[1])
    plane = x.numel() // max(batch * channels, 1)
    lib().dlp_channel_affine_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                                     ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    _check(lib().dlp_channel_affine_fwd_enqueue(torch_dtype_code(x), _act(activation), batch, channels, plane, _ptr(x), _ptr(scale), _ptr(shift),
                                                _ptr(y), _stream(stream)))


def softmax_forward(x, y, log=False, stream=None):
    """Softmax::forward over dimension 1 of a [B, C] or [B, C, S] tensor (log: log-softmax)"""
    if x.dim() not in (2, 3):
        raise ValidationError("softmax: 2 or 3 dimensions")
    inner = int(x.shape[2]) if x.dim() == 3 else 1
    lib().dlp_softmax_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p,
                                              ctypes.c_void_p]
    _check(lib().dlp_softmax_fwd_enqueue(torch_dtype_code(x), int(bool(log)), int(x.shape[0]), int(x.shape[1]), inner, _ptr(x), _ptr(y),
                                         _stream(stream)))


INTERPOLATE_METHODS = {"nearest": 0, "nearest-exact": 1, "bilinear": 2}
REDUCE_METHODS = {"sum": 0, "sumsq": 1, "abssum": 2, "mean": 3}
LOSS_REDUCE = {"none": 0, "sum": 1, "mean": 2}
INT32_DATA = 19


def interpolate2d_forward(x, y, method="nearest", scale_y=-1.0, scale_x=-1.0, align_corners=False, stream=None):
    """core::interpolate2d: x [B, C, H, W] -> y [B, C, OH, OW]; without scales the steps follow from the two sizes"""
    if x.dim() != 4 or y.dim() != 4 or tuple(x.shape[:2]) != tuple(y.shape[:2]):
        raise ValidationError("interpolate2d: two 4-d tensors with the same batch and channels")
    lib().dlp_interpolate2d_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_double, ctypes.c_double] + [ctypes.c_int] * 5 + [
        ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
    if method not in INTERPOLATE_METHODS:
        raise ValidationError("Unsupported interpolation method " + str(method))
    _check(lib().dlp_interpolate2d_fwd_enqueue(torch_dtype_code(x), INTERPOLATE_METHODS[method], int(bool(align_corners)), float(scale_y), float(scale_x),
                                               int(x.shape[0] * x.shape[1]), int(x.shape[2]), int(x.shape[3]), int(y.shape[2]), int(y.shape[3]),
                                               _ptr(x), _ptr(y), _stream(stream)))


def _label_code(labels):
    import torch

    if labels.dtype == torch.float32:
        return FLOAT_DATA
    if labels.dtype == torch.int32:
        return INT32_DATA
    raise NotImplementedErrorDlprim("labels must be either int or float")


def _workspace(nbytes, like):
    import torch

    return torch.empty(max(int(nbytes), 4), dtype=torch.uint8, device=like.device)


def reduction_forward(x, y, method="sum", dims=None, start_axis=0, output_scale=1.0, stream=None):
    """Reduction::forward: y = sum / sumsq / abssum / mean of x over `dims` (or over every axis from `start_axis` on); y holds the kept
    elements in order, with or without the reduced axes as extents of 1"""
    rank = x.dim()
    if dims is None:
        if start_axis < 0:
            start_axis += rank
        if not 0 <= start_axis < rank:
            raise ValidationError("reduction: start_axis outside the tensor")
        dims = range(start_axis, rank)
    mask = [0] * rank
    for d in dims:
        if d < 0:
            d += rank
        if not 0 <= d < rank:
            raise ValidationError("reduction: axis outside the tensor")
        mask[d] = 1
    arr = ctypes.c_int * rank
    shape = arr(*[int(d) for d in x.shape])
    red = arr(*mask)
    code = torch_dtype_code(x)
    need = ctypes.c_size_t(0)
    L = lib()
    L.dlp_reduce_fwd_workspace.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.POINTER(ctypes.c_size_t)]
    _check(L.dlp_reduce_fwd_workspace(code, REDUCE_METHODS[method], rank, shape, red, ctypes.byref(need)))
    ws = _workspace(need.value, x)
    L.dlp_reduce_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p]
    _check(L.dlp_reduce_fwd_enqueue(code, REDUCE_METHODS[method], float(output_scale), rank, shape, red, _ptr(x), _ptr(y), _ptr(ws), ws.numel(),
                                    _stream(stream)))
    return need.value


def mse_loss_forward(a, b, y, reduce="mean", stream=None):
    """MSELoss::forward: y = (a - b)^2 elementwise, or the sum / mean of that in y[0]"""
    if tuple(a.shape) != tuple(b.shape):
        raise ValidationError("MSE loss: the inputs differ in shape")
    code = torch_dtype_code(a)
    need = ctypes.c_size_t(0)
    L = lib()
    L.dlp_mse_loss_fwd_workspace.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_size_t, ctypes.POINTER(ctypes.c_size_t)]
    _check(L.dlp_mse_loss_fwd_workspace(code, LOSS_REDUCE[reduce], a.numel(), ctypes.byref(need)))
    ws = _workspace(need.value, a)
    L.dlp_mse_loss_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                           ctypes.c_size_t, ctypes.c_void_p]
    _check(L.dlp_mse_loss_fwd_enqueue(code, LOSS_REDUCE[reduce], a.numel(), _ptr(a), _ptr(b), _ptr(y), _ptr(ws), ws.numel(), _stream(stream)))


def nll_loss_forward(x, labels, y, reduce="mean", stream=None):
    """NLLLoss::forward: x [B, C] (log-probabilities), labels [B] float32 or int32; y [B] for reduce 'none', else y [1]"""
    if x.dim() != 2 or labels.numel() != x.shape[0]:
        raise ValidationError("NLL loss: x [batch, classes] and one label per row")
    lib().dlp_nll_loss_fwd_enqueue.argtypes = [ctypes.c_int] * 5 + [ctypes.c_void_p] * 4
    _check(lib().dlp_nll_loss_fwd_enqueue(torch_dtype_code(x), _label_code(labels), LOSS_REDUCE[reduce], int(x.shape[0]), int(x.shape[1]), _ptr(x),
                                          _ptr(labels), _ptr(y), _stream(stream)))


def softmax_loss_forward(x, labels, y, stream=None):
    """SoftmaxWithLoss::forward: y[0] = mean cross entropy of the rows of x [B, C] against labels [B] (float32 or int32)"""
    if x.dim() != 2 or labels.numel() != x.shape[0]:
        raise ValidationError("softmax loss: x [batch, classes] and one label per row")
    need = ctypes.c_size_t(0)
    L = lib()
    L.dlp_softmax_loss_fwd_workspace.argtypes = [ctypes.c_int, ctypes.POINTER(ctypes.c_size_t)]
    _check(L.dlp_softmax_loss_fwd_workspace(int(x.shape[0]), ctypes.byref(need)))
    ws = _workspace(need.value, x)
    L.dlp_softmax_loss_fwd_enqueue.argtypes = [ctypes.c_int] * 4 + [ctypes.c_void_p] * 4 + [ctypes.c_size_t, ctypes.c_void_p]
    _check(L.dlp_softmax_loss_fwd_enqueue(torch_dtype_code(x), _label_code(labels), int(x.shape[0]), int(x.shape[1]), _ptr(x), _ptr(labels), _ptr(y),
                                          _ptr(ws), ws.numel(), _stream(stream)))


POINTWISE_OPS = {"threshold": 0, "abs": 1, "hardtanh": 2}


def pointwise_forward(x, y, operation, p0=0.0, p1=0.0, stream=None):
    """Threshold / Abs / Hardtanh::forward: y = x > p0 | |x| | clamp(x, p0, p1); y may be x"""
    lib().dlp_pointwise_fwd_enqueue.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_float, ctypes.c_float, ctypes.c_size_t, ctypes.c_void_p,
                                                ctypes.c_void_p, ctypes.c_void_p]
    _check(lib().dlp_pointwise_fwd_enqueue(torch_dtype_code(x), POINTWISE_OPS[operation], float(p0), float(p1), x.numel(), _ptr(x), _ptr(y),
                                           _stream(stream)))
