"""Network descriptions and parameter files in dlprimitives' formats, for dlprim::Net
(include/dlprim/net.hpp).

* the network JSON of docs/network_json_format.md: {"inputs": [{"name", "shape"}], "outputs": [names],
  "operators": [{"name", "type", "inputs", "outputs", "params", "options"}]};
* the DLPW parameter file (writer src/net.cpp:63-101, reader :204-305): the bytes "DLPW", the header
  length as a big-endian uint32, a JSON header {"tensors": {name: {"dtype", "shape", "size", "start"}}}
  and the tensors' raw little-endian data, `start` counted from the end of the header.

NetBuilder writes the operator list the way the reference's ONNX converter does for torchvision
models (separate BatchNorm operators, in-place Activation operators), so that the loader's graph
rewrites have the same input they would get from the reference's own files.
"""
import json
import struct

import numpy as np


def save_dlpw(path, tensors):
    """tensors: {name: float32 array}, written in dict order."""
    header = {"tensors": {}}
    start = 0
    blobs = []
    for name, t in tensors.items():
        a = np.ascontiguousarray(t, dtype="<f4")
        header["tensors"][name] = {"dtype": "float", "shape": list(a.shape), "size": a.nbytes, "start": start}
        start += a.nbytes
        blobs.append(a.tobytes())
    text = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(b"DLPW" + struct.pack(">I", len(text)) + text)
        for b in blobs:
            f.write(b)


def load_dlpw(path):
    with open(path, "rb") as f:
        data = f.read()
    if data[:4] != b"DLPW":
        raise ValueError("%s is not a DLPW file" % path)
    (n,) = struct.unpack(">I", data[4:8])
    header = json.loads(data[8 : 8 + n].decode())
    body = memoryview(data)[8 + n :]
    out = {}
    for name, spec in header["tensors"].items():
        if spec.get("dtype", "float") != "float":
            raise ValueError("tensor %s: dtype %s" % (name, spec["dtype"]))
        raw = body[spec["start"] : spec["start"] + spec["size"]]
        out[name] = np.frombuffer(raw, dtype="<f4").reshape(spec["shape"]).copy()
    return out


def _pair(v):
    return [v, v] if isinstance(v, int) else list(v)


class NetBuilder:
    """Builds the JSON document and tracks shapes so parameter shapes are known."""

    def __init__(self, name, shape):
        self.doc = {"inputs": [{"name": name, "shape": list(shape)}], "outputs": [], "operators": []}
        self.shapes = {name: tuple(shape)}
        self.param_shapes = {}
        self._n = 0

    def _op(self, kind, type_, inputs, outputs, options, params=None):
        name = "%s_%d" % (kind, self._n)
        self._n += 1
        op = {"name": name, "type": type_, "inputs": list(inputs), "outputs": list(outputs)}
        if params:
            op["params"] = list(params)
        op["options"] = options
        self.doc["operators"].append(op)
        return name

    def input(self, name, shape, dtype=None):
        """another input; dtype "int" for the labels of a loss (default: float)"""
        spec = {"name": name, "shape": list(shape)}
        if dtype is not None:
            spec["dtype"] = dtype
        self.doc["inputs"].append(spec)
        self.shapes[name] = tuple(shape)
        return name

    def conv(self, src, dst, cout, k, stride=1, pad=0, groups=1, bias=False, activation=None, dilate=1, prefix=None, scalar_options=False):
        n, cin, h, w = self.shapes[src]
        k2, s2, p2, d2 = _pair(k), _pair(stride), _pair(pad), _pair(dilate)
        opts = {"bias": bias, "groups": groups, "channels_out": cout, "channels_in": cin}
        if scalar_options and k2[0] == k2[1] and s2[0] == s2[1] and p2[0] == p2[1]:
            opts.update(kernel=k2[0], stride=s2[0], pad=p2[0])
        else:
            opts.update(kernel=k2, stride=s2, dilate=d2, pad=p2)
        if activation:
            opts["activation"] = activation
        prefix = prefix or dst
        params = [prefix + ".weight"] + ([prefix + ".bias"] if bias else [])
        self._op("Conv", "Convolution2D", [src], [dst], opts, params)
        self.param_shapes[params[0]] = (cout, cin // groups, k2[0], k2[1])
        if bias:
            self.param_shapes[params[1]] = (cout,)
        ho = (h + 2 * p2[0] - d2[0] * (k2[0] - 1) - 1) // s2[0] + 1
        wo = (w + 2 * p2[1] - d2[1] * (k2[1] - 1) - 1) // s2[1] + 1
        self.shapes[dst] = (n, cout, ho, wo)
        return dst

    def tconv(self, src, dst, cout, k, stride=1, pad=0, output_pad=0, groups=1, bias=False, activation=None, dilate=1, prefix=None):
        """TransposedConvolution2D: weights [channels_in, channels_out / groups, kh, kw] (src/ops/conv2d.cpp:629-634)"""
        n, cin, h, w = self.shapes[src]
        k2, s2, p2, d2, o2 = _pair(k), _pair(stride), _pair(pad), _pair(dilate), _pair(output_pad)
        opts = {"bias": bias, "groups": groups, "channels_out": cout, "channels_in": cin, "kernel": k2, "stride": s2, "dilate": d2, "pad": p2,
                "output_pad": o2}
        if activation:
            opts["activation"] = activation
        prefix = prefix or dst
        params = [prefix + ".weight"] + ([prefix + ".bias"] if bias else [])
        self._op("ConvTranspose", "TransposedConvolution2D", [src], [dst], opts, params)
        self.param_shapes[params[0]] = (cin, cout // groups, k2[0], k2[1])
        if bias:
            self.param_shapes[params[1]] = (cout,)
        ho = (h - 1) * s2[0] - 2 * p2[0] + d2[0] * (k2[0] - 1) + o2[0] + 1
        wo = (w - 1) * s2[1] - 2 * p2[1] + d2[1] * (k2[1] - 1) + o2[1] + 1
        self.shapes[dst] = (n, cout, ho, wo)
        return dst

    def bn(self, src, dst, eps=1e-5, affine=True, activation=None, prefix=None):
        c = self.shapes[src][1]
        prefix = prefix or dst
        names = [prefix + ".running_mean", prefix + ".running_var"] + ([prefix + ".weight", prefix + ".bias"] if affine else [])
        opts = {"eps": eps, "momentum": 0.1}
        if not affine:
            opts["affine"] = False
        if activation:
            opts["activation"] = activation
        self._op("BatchNormalization", "BatchNorm", [src], [dst], opts, names)
        for nm in names:
            self.param_shapes[nm] = (c,)
        self.shapes[dst] = self.shapes[src]
        return dst

    def act(self, src, activation, dst=None):
        dst = dst or src
        self._op(activation.capitalize(), "Activation", [src], [dst], {"activation": activation})
        self.shapes[dst] = self.shapes[src]
        return dst

    def pool(self, src, dst, mode, k, stride=1, pad=0, ceil_mode=False, count_include_pad=False):
        n, c, h, w = self.shapes[src]
        k2, s2, p2 = _pair(k), _pair(stride), _pair(pad)
        opts = {"kernel": k2, "stride": s2, "pad": p2, "count_include_pad": int(count_include_pad), "mode": mode}
        if ceil_mode:
            opts["ceil_mode"] = True
        self._op("Pool", "Pooling2D", [src], [dst], opts)

        def out(size, k, p, s):
            if ceil_mode:
                o = -(-(size + 2 * p - k) // s) + 1
                if (o - 1) * s >= size + p:
                    o -= 1
                return o
            return (size + 2 * p - k) // s + 1

        self.shapes[dst] = (n, c, out(h, k2[0], p2[0], s2[0]), out(w, k2[1], p2[1], s2[1]))
        return dst

    def global_pool(self, src, dst, mode):
        n, c = self.shapes[src][:2]
        self._op("GlobalPool", "GlobalPooling", [src], [dst], {"mode": mode})
        self.shapes[dst] = (n, c, 1, 1)
        return dst

    def eltwise(self, a, b, dst, operation="sum", coef1=None, coef2=None, activation=None):
        opts = {"operation": operation}
        if coef1 is not None:
            opts["coef1"] = coef1
        if coef2 is not None:
            opts["coef2"] = coef2
        if activation:
            opts["activation"] = activation
        self._op("Add", "Elementwise", [a, b], [dst], opts)
        self.shapes[dst] = tuple(np.broadcast_shapes(self.shapes[a], self.shapes[b]))
        return dst

    def ip(self, src, dst, outputs, bias=True, activation=None, prefix=None):
        s = self.shapes[src]
        inputs = int(np.prod(s[1:]))
        opts = {"bias": bias, "outputs": outputs, "inputs": inputs}
        if activation:
            opts["activation"] = activation
        prefix = prefix or dst
        params = [prefix + ".weight"] + ([prefix + ".bias"] if bias else [])
        self._op("Gemm", "InnerProduct", [src], [dst], opts, params)
        self.param_shapes[params[0]] = (outputs, inputs)
        if bias:
            self.param_shapes[params[1]] = (outputs,)
        self.shapes[dst] = (s[0], outputs)
        return dst

    def flatten(self, src, dst):
        s = self.shapes[src]
        self._op("Flatten", "Flatten", [src], [dst], {})
        self.shapes[dst] = (s[0], int(np.prod(s[1:])))
        return dst

    def pointwise(self, src, dst, kind, **options):
        """Threshold (threshold=), Abs, Hardtanh (min_val=, max_val=)"""
        self._op(kind, kind, [src], [dst], dict(options))
        self.shapes[dst] = self.shapes[src]
        return dst

    def concat(self, srcs, dst, dim=1):
        shapes = [self.shapes[s] for s in srcs]
        self._op("Concat", "Concat", list(srcs), [dst], {"dim": dim})
        out = list(shapes[0])
        out[dim] = sum(sh[dim] for sh in shapes)
        self.shapes[dst] = tuple(out)
        return dst

    def slice(self, src, dst, begin=0, end=-1, dim=1):
        s = list(self.shapes[src])
        self._op("Slice", "Slice", [src], [dst], {"dim": dim, "begin": begin, "end": end})
        s[dim] = (s[dim] if end == -1 else end) - begin
        self.shapes[dst] = tuple(s)
        return dst

    def reshape(self, src, dst, dims):
        s = self.shapes[src]
        self._op("Reshape", "Reshape", [src], [dst], {"dims": list(dims)})
        out = [s[i] if d == 0 else d for i, d in enumerate(dims)]
        if -1 in out:
            known = int(np.prod([d for d in out if d != -1]))
            out[out.index(-1)] = int(np.prod(s)) // known
        self.shapes[dst] = tuple(out)
        return dst

    def squeeze(self, src, dst, dims=None):
        s = self.shapes[src]
        opts = {"dims": list(dims)} if dims is not None else {"all": True}
        self._op("Squeeze", "Squeeze", [src], [dst], opts)
        axes = [d % len(s) for d in dims] if dims is not None else [i for i, d in enumerate(s) if d == 1]
        self.shapes[dst] = tuple(d for i, d in enumerate(s) if i not in axes) or (1,)
        return dst

    def softmax(self, src, dst, log=False):
        self._op("Softmax", "Softmax", [src], [dst], {"log": bool(log)})
        self.shapes[dst] = self.shapes[src]
        return dst

    def interpolation(self, src, dst, method="nearest", out_hw=None, scale=None, align_corners=False):
        """Interpolation to a size (out_hw) or by factors (scale = (scale_y, scale_x)): nearest, nearest-exact or bilinear"""
        n, c, h, w = self.shapes[src]
        opts = {"method": method, "align_corners": bool(align_corners)}
        if out_hw is not None:
            opts.update(out_h=int(out_hw[0]), out_w=int(out_hw[1]))
            hw = (int(out_hw[0]), int(out_hw[1]))
        else:
            opts.update(scale_y=scale[0], scale_x=scale[1])
            hw = (int(h * scale[0]), int(w * scale[1]))
        self._op("Interpolation", "Interpolation", [src], [dst], opts)
        self.shapes[dst] = (n, c) + hw
        return dst

    def reduction(self, src, dst, method="sum", dims=None, start_axis=None, keep_dim=True, output_scale=None):
        """Reduction over `dims`, or over every axis from `start_axis` (default 0) on"""
        s = self.shapes[src]
        opts = {"method": method, "keep_dim": bool(keep_dim)}
        if dims is not None:
            opts["dims"] = list(dims)
            axes = {d % len(s) for d in dims}
        else:
            if start_axis is not None:
                opts["start_axis"] = start_axis
            axes = set(range((start_axis or 0) % len(s), len(s)))
        if output_scale is not None:
            opts["output_scale"] = output_scale
        self._op("Reduction", "Reduction", [src], [dst], opts)
        out = [1 if i in axes else d for i, d in enumerate(s) if keep_dim or i not in axes]
        self.shapes[dst] = tuple(out) or (1,)
        return dst

    def parameter(self, dst, shape, pname=None):
        """Parameter: a tensor whose values are a parameter of the network"""
        pname = pname or dst + ".value"
        self._op("Parameter", "Parameter", [], [dst], {"shape": list(shape), "dtype": "float"}, [pname])
        self.param_shapes[pname] = tuple(shape)
        self.shapes[dst] = tuple(shape)
        return dst

    def mse_loss(self, a, b, dst, reduce="mean"):
        self._op("MSELoss", "MSELoss", [a, b], [dst], {"reduce": reduce})
        self.shapes[dst] = self.shapes[a] if reduce == "none" else (1,)
        return dst

    def nll_loss(self, src, labels, dst, reduce="mean"):
        self._op("NLLLoss", "NLLLoss", [src, labels], [dst], {"reduce": reduce})
        self.shapes[dst] = (self.shapes[src][0],) if reduce == "none" else (1,)
        return dst

    def softmax_loss(self, src, labels, dst):
        self._op("SoftmaxWithLoss", "SoftmaxWithLoss", [src, labels], [dst], {})
        self.shapes[dst] = (1,)
        return dst

    def output(self, name):
        self.doc["outputs"].append(name)

    def random_parameters(self, seed):
        """Parameters with activations of order one through deep stacks: He-scaled weights,
        running variances in [0.5, 1.5], gammas in [0.5, 1.5]."""
        rng = np.random.default_rng(seed)
        out = {}
        for name, shape in self.param_shapes.items():
            if name.endswith("running_var"):
                t = rng.uniform(0.5, 1.5, shape)
            elif name.endswith("running_mean"):
                t = rng.uniform(-0.3, 0.3, shape)
            elif len(shape) == 1 and name.endswith(".weight"):
                t = rng.uniform(0.5, 1.5, shape)
            elif name.endswith(".value"):  # a Parameter operator's tensor
                t = rng.uniform(-1.0, 1.0, shape)
            elif len(shape) == 1:
                t = rng.uniform(-0.2, 0.2, shape)
            else:
                fan_in = int(np.prod(shape[1:]))
                t = rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)
            out[name] = t.astype(np.float32)
        return out


def resnet18(batch, size=224, classes=1000):
    """The operator list of docs/nets_for_benchmark/resnet18-b16.js at another batch / image size."""
    b = NetBuilder("data", (batch, 3, size, size))
    t = b.conv("data", "c1", 64, 7, 2, 3, prefix="conv1")
    t = b.act(b.bn(t, "bn1"), "relu")
    t = b.pool(t, "pool1", "max", 3, 2, 1)
    cin = 64
    for stage, cout in enumerate((64, 128, 256, 512), 1):
        for block in range(2):
            s = 2 if (stage > 1 and block == 0) else 1
            p = "layer%d.%d" % (stage, block)
            u = b.act(b.bn(b.conv(t, p + ".c1", cout, 3, s, 1, prefix=p + ".conv1"), p + ".bn1"), "relu")
            u = b.bn(b.conv(u, p + ".c2", cout, 3, 1, 1, prefix=p + ".conv2"), p + ".bn2")
            skip = t
            if s != 1 or cin != cout:
                skip = b.bn(b.conv(t, p + ".ds", cout, 1, s, 0, prefix=p + ".downsample.0"), p + ".downsample.1")
            t = b.eltwise(u, skip, p + ".sum", activation="relu")
            cin = cout
    t = b.global_pool(t, "gap", "avg")
    b.ip(t, "loss", classes, prefix="fc")
    b.output("loss")
    return b


def resnet50(batch, size=224, classes=1000):
    """The operator list of docs/nets_for_benchmark/resnet50-b16.js (stride on the 3x3)."""
    b = NetBuilder("data", (batch, 3, size, size))
    t = b.act(b.bn(b.conv("data", "c1", 64, 7, 2, 3, prefix="conv1"), "bn1"), "relu")
    t = b.pool(t, "pool1", "max", 3, 2, 1)
    cin = 64
    for stage, (mid, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3)), 1):
        cout = mid * 4
        for block in range(blocks):
            s = 2 if (stage > 1 and block == 0) else 1
            p = "layer%d.%d" % (stage, block)
            u = b.act(b.bn(b.conv(t, p + ".c1", mid, 1, 1, 0, prefix=p + ".conv1"), p + ".bn1"), "relu")
            u = b.act(b.bn(b.conv(u, p + ".c2", mid, 3, s, 1, prefix=p + ".conv2"), p + ".bn2"), "relu")
            u = b.bn(b.conv(u, p + ".c3", cout, 1, 1, 0, prefix=p + ".conv3"), p + ".bn3")
            skip = t
            if s != 1 or cin != cout:
                skip = b.bn(b.conv(t, p + ".ds", cout, 1, s, 0, prefix=p + ".downsample.0"), p + ".downsample.1")
            t = b.eltwise(u, skip, p + ".sum", activation="relu")
            cin = cout
    t = b.global_pool(t, "gap", "avg")
    b.ip(t, "loss", classes, prefix="fc")
    b.output("loss")
    return b


def mobilenet_v2(batch, size=224, classes=1000, activation="relu6"):
    """The operator list of docs/nets_for_benchmark/mobilenet_v2-b16.js: stem, 17 inverted-residual
    blocks (the first without expansion, 10 with a skip connection), 1x1 to 1280, classifier."""
    b = NetBuilder("data", (batch, 3, size, size))

    def cbr(src, name, cout, k, s, groups=1, act=True):
        t = b.bn(b.conv(src, name + ".c", cout, k, s, k // 2, groups=groups, prefix=name + ".0"), name + ".1")
        return b.act(t, activation) if act else t

    t = cbr("data", "f0", 32, 3, 2)
    i = 1
    for expand, cout, repeats, stride in ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)):
        for r in range(repeats):
            s = stride if r == 0 else 1
            cin = b.shapes[t][1]
            u = t
            if expand != 1:
                u = cbr(u, "f%d.ex" % i, cin * expand, 1, 1)
            u = cbr(u, "f%d.dw" % i, cin * expand, 3, s, groups=cin * expand)
            u = cbr(u, "f%d.pw" % i, cout, 1, 1, act=False)
            t = b.eltwise(t, u, "f%d.sum" % i) if (s == 1 and cin == cout) else u
            i += 1
    t = cbr(t, "f%d" % i, 1280, 1, 1)
    t = b.global_pool(t, "gap", "avg")
    b.ip(t, "loss", classes, prefix="classifier")
    b.output("loss")
    return b


def alexnet(batch, size=224, classes=1000, hidden=4096):
    """The operator list of docs/nets_for_benchmark/alexnet-b16.js at another batch / image size / width of the hidden layers:
    convolutions 11x11/4, 5x5 and 3x3 with bias and ReLU in their epilogues, max pooling 3x3/2 without padding, the 1x1
    average pooling that the exporter leaves where torchvision's adaptive pooling is the identity, and three inner products,
    the first of which takes the 4-D tensor as it is."""
    b = NetBuilder("data", (batch, 3, size, size))
    x = b.conv("data", "c1", 64, 11, 4, 2, bias=True, activation="relu")
    x = b.pool(x, "p1", "max", 3, 2, 0)
    x = b.conv(x, "c2", 192, 5, 1, 2, bias=True, activation="relu")
    x = b.pool(x, "p2", "max", 3, 2, 0)
    x = b.conv(x, "c3", 384, 3, 1, 1, bias=True, activation="relu")
    x = b.conv(x, "c4", 256, 3, 1, 1, bias=True, activation="relu")
    x = b.conv(x, "c5", 256, 3, 1, 1, bias=True, activation="relu")
    x = b.pool(x, "p5", "max", 3, 2, 0)
    x = b.pool(x, "p6", "avg", 1, 1, 0)
    x = b.ip(x, "f6", hidden, activation="relu")
    x = b.ip(x, "f7", hidden, activation="relu")
    b.ip(x, "loss", classes)
    b.output("loss")
    return b


def vgg16(batch, size=224, classes=1000, hidden=4096):
    """The operator list of docs/nets_for_benchmark/vgg16-b16.js at another batch / image size / width of the hidden layers:
    thirteen 3x3 convolutions with bias and ReLU, five max poolings 2x2/2, the identity average pooling and three inner products."""
    b = NetBuilder("data", (batch, 3, size, size))
    x = "data"
    n = 0
    for block, (cout, convs) in enumerate(((64, 2), (128, 2), (256, 3), (512, 3), (512, 3))):
        for _ in range(convs):
            n += 1
            x = b.conv(x, "c%d" % n, cout, 3, 1, 1, bias=True, activation="relu")
        x = b.pool(x, "p%d" % (block + 1), "max", 2, 2, 0)
    x = b.pool(x, "p6", "avg", 1, 1, 0)
    x = b.ip(x, "f6", hidden, activation="relu")
    x = b.ip(x, "f7", hidden, activation="relu")
    b.ip(x, "loss", classes)
    b.output("loss")
    return b

