"""Helpers for the GPU parity tests: every call goes through the C ABI."""
import numpy as np
import torch

import dlprimitives_amd as dlp


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0") if a is not None else None


def settings_of(c, in_shape):
    return dlp.Conv2DSettings(c["cin"], c["cout"], c["kernel"], c["stride"], c["dilate"], c["pad"], c["groups"], in_shape)


def run_conv(c, x, w, bias, algo="", factor=0.0, y_init=None, expect_algo=None, batch_hint=None):
    """Create + enqueue through the C ABI; returns (y as numpy, algo name)."""
    hint_shape = (batch_hint if batch_hint is not None else x.shape[0],) + tuple(x.shape[1:])
    st = settings_of(c, hint_shape)
    op = dlp.Conv2DForward.create(st, bias is not None, c["activation"], algo)
    if expect_algo is not None:
        assert op.algo() == expect_algo, (op.algo(), expect_algo)
    out_shape = dlp.conv2d_output_shape(st, x.shape)
    xd, wd, bd = dev(x), dev(w), dev(bias)
    if y_init is not None:
        yd = dev(y_init.astype(np.float32))
    else:
        # poison: factor == 0 must overwrite, never read (NaNs must not propagate)
        yd = torch.full(out_shape, float("nan"), dtype=torch.float32, device="cuda:0")
    ws_bytes = op.workspace()
    ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device="cuda:0") if ws_bytes else None
    op.enqueue(xd, wd, bd, yd, ws, factor)
    torch.cuda.synchronize()
    return yd.cpu().numpy(), op.algo()


def run_ip(x, w, bias, activation="identity"):
    batch = x.shape[0]
    inputs = int(np.prod(x.shape[1:]))
    op = dlp.IPForward.create(dlp.IPSettings(inputs, w.shape[0], batch), bias is not None, activation)
    yd = torch.full((batch, w.shape[0]), float("nan"), dtype=torch.float32, device="cuda:0")
    op.enqueue(dev(x), dev(w), dev(bias), yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()
