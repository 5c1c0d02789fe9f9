"""Timings of Interpolation, Reduction and the losses on one GPU:  python -m dlprimitives_amd.bench_tensor_ops

Every line: the call, microseconds per call (HIP events over `--iters` calls after `--warmup`), and the bytes the operator must move
(inputs read once + outputs written once) divided by that time.  Tensors live on the device before the timed region.
"""
import argparse

import torch

import dlprimitives_amd as dlp


def timed(fn, warmup, iters):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / iters * 1e3


REDUCTIONS = [
    ((128, 2048, 7, 7), [2, 3], "mean"),
    ((64, 256, 56, 56), [2, 3], "sumsq"),
    ((64, 256, 56, 56), [1], "mean"),
    ((64, 256, 56, 56), [0], "sum"),
    ((64, 256, 56, 56), [0, 2, 3], "sum"),
    ((1 << 26,), [0], "sum"),
    ((4096, 4096), [1], "abssum"),
    ((4096, 4096), [0], "abssum"),
]
INTERPOLATIONS = [
    ((32, 256, 56, 56), (112, 112), "bilinear"),
    ((32, 256, 56, 56), (112, 112), "nearest"),
    ((64, 512, 14, 14), (28, 28), "bilinear"),
    ((16, 64, 224, 224), (112, 112), "bilinear"),
]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--dtype", choices=["float32", "bfloat16", "both"], default="both")
    args = ap.parse_args()
    dtypes = [torch.float32, torch.bfloat16] if args.dtype == "both" else [getattr(torch, args.dtype)]
    for dt in dtypes:
        es = torch.empty(0, dtype=dt).element_size()
        print("==", str(dt).replace("torch.", ""))
        for shape, dims, method in REDUCTIONS:
            x = torch.randn(shape, device="cuda", dtype=dt)
            y = torch.empty([1 if i in dims else d for i, d in enumerate(shape)], device="cuda", dtype=dt)
            us = timed(lambda: dlp.reduction_forward(x, y, method, dims=dims), args.warmup, args.iters)
            print("reduction %-20s dims %-10s %-7s %8.1f us %6.2f TB/s" % (shape, dims, method, us, (x.numel() + y.numel()) * es / us / 1e6))
        for (b, c, h, w), (oh, ow), method in INTERPOLATIONS:
            x = torch.randn(b, c, h, w, device="cuda", dtype=dt)
            y = torch.empty(b, c, oh, ow, device="cuda", dtype=dt)
            us = timed(lambda: dlp.interpolate2d_forward(x, y, method), args.warmup, args.iters)
            print("interpolation %-20s -> %-10s %-9s %8.1f us %6.2f TB/s" % ((b, c, h, w), (oh, ow), method, us, (x.numel() + y.numel()) * es / us / 1e6))
        a = torch.randn(1 << 26, device="cuda", dtype=dt)
        b = torch.randn(1 << 26, device="cuda", dtype=dt)
        y = torch.empty(1, device="cuda", dtype=dt)
        us = timed(lambda: dlp.mse_loss_forward(a, b, y, "mean"), args.warmup, args.iters)
        print("mse_loss mean, 64 M elements %35.1f us %6.2f TB/s" % (us, 2 * a.numel() * es / us / 1e6))
        del a, b
        x = torch.randn(4096, 32000, device="cuda", dtype=dt)
        labels = torch.randint(0, 32000, (4096,), device="cuda", dtype=torch.int32)
        us = timed(lambda: dlp.softmax_loss_forward(x, labels, y), args.warmup, args.iters)
        print("softmax_loss 4096 x 32000 %38.1f us %6.2f TB/s" % (us, x.numel() * es / us / 1e6))
        logp = torch.log_softmax(x.float(), 1).to(dt)
        us = timed(lambda: dlp.nll_loss_forward(logp, labels, y, "mean"), args.warmup, args.iters)
        print("nll_loss 4096 x 32000 (reads 4096 values) %22.1f us" % us)
        del x, logp


if __name__ == "__main__":
    main()
