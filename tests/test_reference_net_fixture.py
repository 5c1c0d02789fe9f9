"""The reference's own whole-network golden fixture (tests/test_net.json + tests/test_weights.json, checked by its
tests/test_net.cpp): a small residual CNN -- convolutions with and without bias, fused ReLU, max pooling, BatchNorm
on batch statistics, a residual sum, global average pooling, an inner product and a softmax loss -- with its
parameters, one batch of data and labels, and the parameter gradients (`param_diff`) that one forward + backward
pass must give.  The two files are kept as data under tests/golden/reference_test_*.json.

Here the convolutions' forward pass, backward data, backward filter and bias gradient are this library's GPU
operators (inside a torch.autograd.Function); everything else of the step is torch.  The CPU test runs the same
interpretation with torch's own convolution, which shows that the fixture is read the way the reference wrote it.
Bar: the reference's own (tests/test_net.cpp:17-43: 1e-5 absolute, scaled by the tensor's deviation when above 1),
loosened to 1e-4 of the gradient's largest magnitude.
"""
import json
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_fixture():
    net = json.load(open(os.path.join(GOLDEN, "reference_test_net.json")))
    entries = json.load(open(os.path.join(GOLDEN, "reference_test_weights.json")))
    values = {}
    for e in entries:
        values[(e["name"], e["type"])] = np.asarray(e["value"], dtype=np.float32)
    return net, values


def pair(v, default):
    if v is None:
        return default
    return (v, v) if isinstance(v, int) else tuple(v)


def make_dlp_conv():
    import dlprimitives_amd as dlp

    def ws(n):
        return torch.empty(max(n, 1), dtype=torch.uint8, device="cuda:0")

    class DlpConv(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, w, b, stride, pad, dilate, groups):
            x, w = x.contiguous(), w.contiguous()
            st = dlp.Conv2DSettings(x.shape[1], w.shape[0], tuple(w.shape[2:]), stride, dilate, pad, groups, tuple(x.shape))
            op = dlp.Conv2DForward.create(st, b is not None, "identity", "")
            y = torch.full(dlp.conv2d_output_shape(st, x.shape), float("nan"), device=x.device)
            op.enqueue(x, w, b, y, ws(op.workspace()))
            ctx.save_for_backward(x, w)
            ctx.st, ctx.has_bias = st, b is not None
            return y

        @staticmethod
        def backward(ctx, dy):
            x, w = ctx.saved_tensors
            dy = dy.contiguous()
            dx = torch.full(x.shape, float("nan"), device=x.device)
            bd = dlp.Conv2DBackwardData.create(ctx.st)
            bd.enqueue(dx, w, dy, ws(bd.workspace()))
            dw = torch.full(w.shape, float("nan"), device=x.device)
            bf = dlp.Conv2DBackwardFilter.create(ctx.st)
            bf.enqueue(x, dw, dy, ws(bf.workspace()))
            db = None
            if ctx.has_bias:
                db = torch.full((w.shape[0],), float("nan"), device=x.device)
                dlp.bias_backward(dy, db)
            return dx, dw, db, None, None, None, None

    return lambda x, w, b, stride, pad, dilate, groups: DlpConv.apply(x, w, b, stride, pad, dilate, groups)


def run_step(conv, device):
    """Forward + backward of the fixture's network; returns {parameter name: gradient}."""
    net, values = load_fixture()
    t = {}
    for i in net["inputs"]:
        t[i["name"]] = torch.from_numpy(values[(i["name"], "data")].reshape(i["shape"])).to(device)
    params = {}

    def P(name, shape, grad=True):
        v = torch.from_numpy(values[(name, "param")].reshape(shape)).to(device)
        params[name] = v.requires_grad_(grad)
        return params[name]

    for op in net["operators"]:
        o = op.get("options", {})
        x = t[op["inputs"][0]]
        kind, name = op["type"], op["name"]
        if kind == "Convolution2D":
            k, groups = pair(o["kernel"], None), o.get("groups", 1)
            w = P(name + ".0", (o["channels_out"], x.shape[1] // groups, k[0], k[1]))
            b = P(name + ".1", (o["channels_out"],)) if o.get("bias", True) else None
            y = conv(x, w, b, pair(o.get("stride"), (1, 1)), pair(o.get("pad"), (0, 0)), pair(o.get("dilate"), (1, 1)), groups)
        elif kind == "Pooling2D":
            assert o.get("mode", "max") == "max"
            y = F.max_pool2d(x, pair(o["kernel"], None), pair(o.get("stride"), (1, 1)), pair(o.get("pad"), (0, 0)))
        elif kind == "BatchNorm":  # the test runs in train mode: batch statistics, running sums updated
            c = x.shape[1]
            y = F.batch_norm(x, P(name + ".0", (c,), False), P(name + ".1", (c,), False), P(name + ".2", (c,)), P(name + ".3", (c,)), True,
                             o.get("momentum", 0.1), o.get("eps", 1e-5))
        elif kind == "Activation":
            y = x
        elif kind == "Elementwise":
            assert o.get("operation", "sum") == "sum"
            y = x + t[op["inputs"][1]]
        elif kind == "GlobalPooling":
            assert o["mode"] == "avg"
            y = x.mean((2, 3), keepdim=True)
        elif kind == "Flatten":
            y = x.reshape(x.shape[0], -1)
        elif kind == "InnerProduct":
            y = F.linear(x, P(name + ".0", (o["outputs"], x.shape[1])), P(name + ".1", (o["outputs"],)) if o.get("bias", True) else None)
        elif kind == "SoftmaxWithLoss":  # mean over the batch of -log softmax[label] (src/ops/softmax.cpp:134-155)
            y = F.cross_entropy(x, t[op["inputs"][1]].reshape(-1).long(), reduction="mean").reshape(1)
        else:
            raise AssertionError(kind)
        act = o.get("activation", "identity")
        assert act in ("identity", "relu")
        t[op["outputs"][0]] = torch.relu(y) if act == "relu" else y
    loss = t[net["outputs"][0]]
    loss.backward(torch.from_numpy(values[("loss", "data_diff")]).to(device))
    return {n: p.grad.detach().cpu().numpy().reshape(-1) for n, p in params.items() if p.grad is not None}, values


def check(grads, values):
    want_names = sorted(n for (n, kind) in values if kind == "param_diff")
    assert sorted(grads) == want_names
    for n in want_names:
        want = values[(n, "param_diff")]
        err = np.abs(grads[n] - want).max() / max(np.abs(want).max(), 1e-6)
        print("%-8s %5d values  max |grad| %.3e  max err / max %.2e" % (n, want.size, np.abs(want).max(), err))
        assert err < 1e-4, (n, err)


def test_fixture_is_read_as_the_reference_wrote_it():
    grads, values = run_step(lambda x, w, b, s, p, d, g: F.conv2d(x, w, b, s, p, d, g), "cpu")
    check(grads, values)


@pytest.mark.gpu
def test_gpu_reference_training_step_with_dlp_convolutions():
    grads, values = run_step(make_dlp_conv(), "cuda:0")
    check(grads, values)
