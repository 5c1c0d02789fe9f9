"""ResNet-18 / ResNet-50 forward graphs (shapes of the reference's
docs/nets_for_benchmark/resnet18-b16.js and resnet50-b16.js, torchvision v1.5: stride on
the 3x3) with batch norm folded into the preceding convolution, and a small executor that
runs them on the GPU through the C ABI: convolution, pooling, elementwise, global pooling
and inner product are the library's operators; this module only wires tensors.

An op is a dict: conv {cin,cout,k,s,p,act}, maxpool {k,s,p}, add {act}, gap, ip {inputs,outputs};
`src` names its input tensor(s), `dst` its output.
"""
import numpy as np


def _conv(ops, src, dst, cin, cout, k, s, p, act):
    ops.append(dict(op="conv", src=src, dst=dst, cin=cin, cout=cout, k=k, s=s, p=p, act=act))
    return dst


def resnet18():
    ops = []
    t = _conv(ops, "data", "stem", 3, 64, 7, 2, 3, "relu")
    ops.append(dict(op="maxpool", src=t, dst="pool", k=3, s=2, p=1))
    t, cin = "pool", 64
    for stage, cout in enumerate((64, 128, 256, 512), 1):
        for block in range(2):
            s = 2 if (stage > 1 and block == 0) else 1
            name = "l%d_%d" % (stage, block)
            a = _conv(ops, t, name + "_a", cin, cout, 3, s, 1, "relu")
            b = _conv(ops, a, name + "_b", cout, cout, 3, 1, 1, "identity")
            skip = t
            if s != 1 or cin != cout:
                skip = _conv(ops, t, name + "_ds", cin, cout, 1, s, 0, "identity")
            ops.append(dict(op="add", src=[b, skip], dst=name, act="relu"))
            t, cin = name, cout
    ops.append(dict(op="gap", src=t, dst="gap"))
    ops.append(dict(op="ip", src="gap", dst="logits", inputs=512, outputs=1000))
    return ops


def resnet50():
    ops = []
    t = _conv(ops, "data", "stem", 3, 64, 7, 2, 3, "relu")
    ops.append(dict(op="maxpool", src=t, dst="pool", k=3, s=2, p=1))
    t, cin = "pool", 64
    for stage, (mid, blocks) in enumerate(((64, 3), (128, 4), (256, 6), (512, 3)), 1):
        cout = mid * 4
        for block in range(blocks):
            s = 2 if (stage > 1 and block == 0) else 1
            name = "l%d_%d" % (stage, block)
            a = _conv(ops, t, name + "_a", cin, mid, 1, 1, 0, "relu")
            b = _conv(ops, a, name + "_b", mid, mid, 3, s, 1, "relu")
            c = _conv(ops, b, name + "_c", mid, cout, 1, 1, 0, "identity")
            skip = t
            if s != 1 or cin != cout:
                skip = _conv(ops, t, name + "_ds", cin, cout, 1, s, 0, "identity")
            ops.append(dict(op="add", src=[c, skip], dst=name, act="relu"))
            t, cin = name, cout
    ops.append(dict(op="gap", src=t, dst="gap"))
    ops.append(dict(op="ip", src="gap", dst="logits", inputs=2048, outputs=1000))
    return ops


def fold_batchnorm(w, gamma, beta, mean, var, eps=1e-5):
    """W' = W * gamma/sqrt(var+eps) per output channel, b' = beta - mean*gamma/sqrt(var+eps)
    (closed form of the reference's BatchNorm inference, src/ops/batch_normalization.cpp:210-232)."""
    scale = (gamma / np.sqrt(var + eps)).astype(np.float32)
    return (w * scale[:, None, None, None]).astype(np.float32), (beta - mean * scale).astype(np.float32)


def random_parameters(ops, seed):
    """Kaiming-normal conv weights with random BN statistics folded in; inner product weights."""
    rng = np.random.default_rng(seed)
    params = {}
    for o in ops:
        if o["op"] == "conv":
            fan_in = o["cin"] * o["k"] * o["k"]
            w = (rng.standard_normal((o["cout"], o["cin"], o["k"], o["k"])) * np.sqrt(2.0 / fan_in)).astype(np.float32)
            gamma = rng.uniform(0.5, 1.0, o["cout"]).astype(np.float32)
            beta = rng.uniform(-0.1, 0.1, o["cout"]).astype(np.float32)
            mean = (rng.standard_normal(o["cout"]) * 0.1).astype(np.float32)
            var = rng.uniform(0.5, 1.5, o["cout"]).astype(np.float32)
            params[o["dst"]] = fold_batchnorm(w, gamma, beta, mean, var)
        elif o["op"] == "ip":
            w = (rng.standard_normal((o["outputs"], o["inputs"])) / np.sqrt(o["inputs"])).astype(np.float32)
            params[o["dst"]] = (w, rng.uniform(-0.1, 0.1, o["outputs"]).astype(np.float32))
    return params


def conv_out(n, k, s, p):
    return (n + 2 * p - (k - 1) - 1) // s + 1


def infer_shapes(ops, in_shape):
    """tensor name -> shape"""
    import dlprimitives_amd as dlp

    shapes = {"data": tuple(in_shape)}
    for o in ops:
        if o["op"] == "conv":
            b, _, h, w = shapes[o["src"]]
            oh, ow = conv_out(h, o["k"], o["s"], o["p"]), conv_out(w, o["k"], o["s"], o["p"])
            if o.get("pool"):  # the max pooling runs inside the convolution: the tensor is the pooled one
                k, s, p = o["pool"]
                oh, ow = dlp.pool2d_output_size(oh, k, p, s), dlp.pool2d_output_size(ow, k, p, s)
            shapes[o["dst"]] = (b, o["cout"], oh, ow)
        elif o["op"] == "maxpool":
            b, c, h, w = shapes[o["src"]]
            shapes[o["dst"]] = (b, c, dlp.pool2d_output_size(h, o["k"], o["p"], o["s"]), dlp.pool2d_output_size(w, o["k"], o["p"], o["s"]))
        elif o["op"] == "add":
            shapes[o["dst"]] = shapes[o["src"][0]]
        elif o["op"] == "gap":
            b, c = shapes[o["src"]][:2]
            shapes[o["dst"]] = (b, c, 1, 1)
        elif o["op"] == "ip":
            shapes[o["dst"]] = (shapes[o["src"]][0], o["outputs"])
    return shapes


class GraphRunner:
    """Runs a graph on cuda:0 through the C ABI: operators are created once for a batch size."""

    def __init__(self, ops, params, in_shape, algo="", dtype="float32", fuse_residual=False, prepack=False, channels_last=False, fuse_stem_pool=False):
        """dtype "float32" or "bfloat16": storage type of activations and weights (bias stays fp32).
        fuse_residual: a residual sum whose later branch is a 1x1 convolution runs in that convolution's epilogue
        (dlp_conv2d_fwd_set_accumulate_first: y = act(conv + bias + y) written over the other branch), which is what
        dlprim::Net does with the same graphs; 3x3 convolutions keep their sum as an operator.
        prepack: the filters are transformed once here (dlp_conv2d_fwd_pack) and forward() calls enqueue_packed, as a
        network with constant weights does (dlprim::Net::copy_parameters_to_device); otherwise every enqueue transforms
        its filter again, which is the contract of the reference's enqueue.
        channels_last (bfloat16, algorithm gemm): tensors between convolutions are kept as [image][row][column][channel]
        wherever every operator that touches them can take that layout and one of the readers is faster on it
        (dlp_conv2d_fwd_set_channels_last; see _plan_layouts).  Input, logits and parameters keep their layout.
        fuse_stem_pool (bfloat16): a max pooling that is the only reader of a convolution runs inside that convolution where
        dlp_conv2d_fwd_fuse_max_pool takes it (the 7x7 stride-2 stem of a ResNet and its 3x3 stride-2 pooling)."""
        import torch

        import dlprimitives_amd as dlp
        from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA

        ops = [dict(o) for o in ops]
        alias = {}
        if fuse_residual:
            ops = self._fuse_residual_sums(ops, alias)
        if fuse_stem_pool and dtype == "bfloat16":
            ops = self._fuse_max_pooling(ops, in_shape, algo)
        self.ops = ops
        self.shapes = infer_shapes(ops, in_shape)
        tdt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        code = BFLOAT16_DATA if dtype == "bfloat16" else FLOAT_DATA
        self.cl = self._plan_layouts(ops, alias, self.shapes) if (channels_last and dtype == "bfloat16" and algo in ("", "auto", "gemm")) else set()
        stored = lambda n, s: (s[0], s[2], s[3], s[1]) if n in self.cl else s
        self.t = {n: torch.empty(stored(n, s), dtype=tdt, device="cuda:0") for n, s in self.shapes.items() if n not in alias}
        for n in self.shapes:  # the output of a fused sum lies over the branch it was added to (chains of blocks: follow the aliases)
            if n in alias:
                m = alias[n]
                while m in alias:
                    m = alias[m]
                self.t[n] = self.t[m]
        self.p = {n: (torch.from_numpy(w).cuda().to(tdt), torch.from_numpy(b).cuda()) for n, (w, b) in params.items()}
        self.k = []
        self.packed = {}
        ws_bytes = 1
        for o in ops:
            if o["op"] == "conv":
                st = dlp.Conv2DSettings(o["cin"], o["cout"], o["k"], o["s"], 1, o["p"], 1, self.shapes[o["src"]], dtype=code)
                op = dlp.Conv2DForward.create(st, True, o["act"], algo)
                if o.get("residual"):
                    op.accumulate_before_activation(True)
                if o.get("pool"):
                    op.fuse_max_pool(*o["pool"])
                if o["src"] in self.cl or o["dst"] in self.cl:
                    op.channels_last(o["src"] in self.cl, o["dst"] in self.cl)
                ws_bytes = max(ws_bytes, op.workspace())
                if prepack:
                    buf = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda:0")
                    op.pack(self.p[o.get("pname", o["dst"])][0], buf)
                    self.packed[len(self.k)] = buf
            elif o["op"] == "maxpool":
                op = dlp.Pooling2DForward.create_max_pooling(o["k"], o["p"], o["s"], dtype=code)
            elif o["op"] == "gap":
                op = dlp.Pooling2DForward.create_global_avg_pooling(dtype=code)
                if o["src"] in self.cl:
                    op.channels_last(True)
            elif o["op"] == "ip":
                op = dlp.IPForward.create(dlp.IPSettings(o["inputs"], o["outputs"], in_shape[0], dtype=code), True, "identity")
            else:
                op = None
            self.k.append(op)
        # one workspace shared by all operators, as the reference's Net does
        self.ws = torch.empty(ws_bytes, dtype=torch.uint8, device="cuda:0")

    @staticmethod
    def _plan_layouts(ops, alias, shapes):
        """Names of the tensors kept channels-last.  Tensors that share memory (the output of a fused residual sum lies over the
        branch it was added to) share a layout.  A group becomes channels-last when every operator that writes it is a
        convolution that can (channels in multiples of 32 in, of 8 out: the bf16 matrix-instruction kernel with K tiles of one
        filter tap), every reader is such a convolution or the global pooling, and at least one reader gains: measured inside
        ResNet-50 at batch 128, the channels-last loader beats the others on 1x1 layers of more than 64 input channels, on
        everything with a stride and on 7 x 7 images, and loses to the LDS-patch kernel on 3x3 stride-1 layers of larger images
        (14 x 14: 43 against 48 us) and to the dense loader on 1x1 layers of 64 channels (52 against 55 us)."""
        def root(n):
            while n in alias:
                n = alias[n]
            return n

        def conv_ok(o):
            return o["op"] == "conv" and o["cin"] % 32 == 0 and o["cout"] % 8 == 0

        def gains(o):
            if o["op"] != "conv":
                return False
            _, _, h, w = shapes[o["src"]]
            if o["k"] == 3 and o["s"] == 1:
                return h * w < 14 * 14
            return not (o["k"] == 1 and o["s"] == 1 and o["cin"] <= 64)

        writers, readers = {}, {}
        for o in ops:
            for n in (o["src"] if isinstance(o["src"], list) else [o["src"]]):
                readers.setdefault(root(n), []).append(o)
            writers.setdefault(root(o["dst"]), []).append(o)
        chosen = set()
        for g, ws in writers.items():
            rs = readers.get(g, [])
            if all(conv_ok(o) for o in ws) and rs and all(conv_ok(o) or o["op"] == "gap" for o in rs) and any(gains(o) for o in rs):
                chosen.add(g)
        return {n for n in shapes if root(n) in chosen}

    @staticmethod
    def _fuse_max_pooling(ops, in_shape, algo):
        """conv -> maxpool with nothing else reading the convolution's output: the convolution takes the pooling along (key "pool":
        kernel, stride, pad) and writes the pooling's tensor, where the library can do that; otherwise the pair stays as it is"""
        import dlprimitives_amd as dlp
        from dlprimitives_amd.capi import BFLOAT16_DATA, NotImplementedErrorDlprim

        shapes = infer_shapes(ops, in_shape)
        out = []
        for o in ops:
            prev = out[-1] if out else None
            if (o["op"] == "maxpool" and prev is not None and prev["op"] == "conv" and prev["dst"] == o["src"] and not prev.get("residual")
                    and sum(1 for q in ops if o["src"] == q["src"] or (isinstance(q["src"], list) and o["src"] in q["src"])) == 1):
                st = dlp.Conv2DSettings(prev["cin"], prev["cout"], prev["k"], prev["s"], 1, prev["p"], 1, shapes[prev["src"]], dtype=BFLOAT16_DATA)
                try:
                    dlp.Conv2DForward.create(st, True, prev["act"], algo).fuse_max_pool(o["k"], o["s"], o["p"])
                except NotImplementedErrorDlprim:
                    out.append(o)
                    continue
                prev.update(pool=(o["k"], o["s"], o["p"]), pname=prev.get("pname", prev["dst"]), dst=o["dst"])
                continue
            out.append(o)
        return out

    @staticmethod
    def _fuse_residual_sums(ops, alias):
        """add(c, skip) with c = a 1x1 convolution without activation that only the sum reads: the convolution takes the
        sum's activation, reads skip as its old output and writes the sum's tensor, which shares skip's memory; the
        convolution that makes skip (the downsample) moves in front of it.  skip must not be read after the sum."""
        out = []
        for i, o in enumerate(ops):
            if o["op"] != "add":
                out.append(o)
                continue
            c, skip = o["src"]
            ci = next((k for k, q in enumerate(out) if q["dst"] == c), None)
            later = any((skip == q["src"] or (isinstance(q["src"], list) and skip in q["src"])) for q in ops[i + 1:])
            readers_c = sum(1 for q in ops if c == q["src"] or (isinstance(q["src"], list) and c in q["src"]))
            if ci is None or out[ci]["op"] != "conv" or out[ci]["k"] != 1 or out[ci]["act"] != "identity" or later or readers_c != 1 or skip == "data":
                out.append(o)
                continue
            conv = out.pop(ci)  # appended again below: behind everything made so far, the other branch included
            conv.update(act=o["act"], residual=True, pname=conv["dst"], dst=o["dst"])
            alias[o["dst"]] = skip
            out.append(conv)
        return out

    def forward(self, x=None):
        import dlprimitives_amd as dlp

        if x is not None:
            self.t["data"].copy_(x)
        for i, (o, op) in enumerate(zip(self.ops, self.k)):
            if o["op"] == "conv":
                w, b = self.p[o.get("pname", o["dst"])]
                factor = 1.0 if o.get("residual") else 0.0
                if i in self.packed:
                    op.enqueue_packed(self.t[o["src"]], w, self.packed[i], b, self.t[o["dst"]], self.ws, factor)
                else:
                    op.enqueue(self.t[o["src"]], w, b, self.t[o["dst"]], self.ws, factor)
            elif o["op"] in ("maxpool", "gap"):
                op.enqueue(self.t[o["src"]], self.t[o["dst"]])
            elif o["op"] == "add":
                dlp.eltwise_forward(self.t[o["src"][0]], self.t[o["src"][1]], self.t[o["dst"]], "sum", 1.0, 1.0, o["act"])
            elif o["op"] == "ip":
                w, b = self.p[o["dst"]]
                op.enqueue(self.t[o["src"]], w, b, self.t[o["dst"]])
        return self.t[self.ops[-1]["dst"]]

    def flops(self):
        total = 0.0
        for o in self.ops:
            if o["op"] == "conv":
                b, _, h, w = self.shapes[o["src"]]
                total += 2.0 * b * o["cout"] * conv_out(h, o["k"], o["s"], o["p"]) * conv_out(w, o["k"], o["s"], o["p"]) * o["cin"] * o["k"] * o["k"]
            elif o["op"] == "ip":
                total += 2.0 * self.shapes[o["dst"]][0] * o["inputs"] * o["outputs"]
        return total
