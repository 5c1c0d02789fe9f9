#!/usr/bin/env python3
"""Benchmark of the convolution forward hot path on one MI355X.

Default workload (the configuration the headline metric is quoted on): the 20
convolutions of the ResNet-18 conv stack, forward, fp32 NCHW, batch 64, BN folded
into weights + bias, fused ReLU, algorithm "gemm" (implicit GEMM on fp32 MFMA).
A step = one pass over all layers of the workload, launched back to back on one
stream, with every tensor already resident in HBM.  Synthetic data: inputs
uniform[-1,1], weights Kaiming-normal, bias uniform[-0.1,0.1], fixed seed.

Other workloads (same JSON contract, for the remaining configurations):
  --workload mobilenet      depthwise 3x3 stride 1/2 (HBM bound) + 1x1 pointwise, ReLU6
  --workload winograd       the two Winograd shapes, algo winograd
  --workload winograd-gemm  the same two shapes through the implicit GEMM
  --workload resnet18-full / resnet50-full   whole network forward incl. pooling, adds, GAP, IP
  --workload resnet18-backward   gradients of the 20 ResNet-18 convolutions (backward filter for all,
                            backward data for all but conv1, whose input needs none), fp32

Prints ONE JSON line.  `value` = images/s of the whole workload; `gflops_per_s` is
the same run expressed with the reference's flop accounting (tools/flops.cpp:660).
`roofline` describes the kernel that takes the largest share of a step; its launch
durations are measured in a second pass by the library's per-kernel timing (one HIP
event pair around every kernel launch, on the launch stream), so they are the
durations a profiler's kernel trace shows for that kernel name.  `cpu_baseline` is the CPU oracle (a
restatement of the reference's single-threaded im2col + sgemm CPU path) timed on
this host on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

FP32_MATRIX_PEAK_TFLOPS = 157.3
BF16_MATRIX_PEAK_TFLOPS = 2500.0
HBM_PEAK_GBS = 8000.0
BASELINE_METRIC = "conv2d fwd GFLOP/s + % of MI355X roofline; ResNet-18 b64 images/sec"

# HBM bytes per launch of the dominant kernel of each workload at batch 64, from hardware
# counters (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, one counter per run, KiB per dispatch,
# scaled by what the same counter reads for a plain copy of known size: x2.0 / x1.0).
# Measured offline (a benchmark run cannot collect counters on itself); keyed by (workload, kernel).
MEASURED_TRAFFIC_BYTES = {
    ("resnet18", "conv_patch_f32_kernel<float, 3, 3, 192, 0>"): (32886.5 * 2.0 + 46377.9) * 1024,
    ("winograd", "wino_fused_kernel<float, ...>"): ((16817.5 + 40712.4) / 2 * 2.0 + (25377.0 + 12838.6) / 2) * 1024,
    ("mobilenet", "depthwise3x3_kernel<float, 1>"): (27364.9 * 2.0 + 45795.7) * 1024,
}


def workload_layers(name):
    from dlprimitives_amd.workloads import MOBILENET_DEPTHWISE, MOBILENET_POINTWISE, RESNET18_CONVS, WINOGRAD_SHAPES, conv

    if name == "resnet18":
        return [dict(L, algo="gemm") for L in RESNET18_CONVS], "ResNet-18 conv stack forward: 20 convs, BN folded, fused ReLU, algo gemm"
    if name == "resnet50":
        from dlprimitives_amd.workloads import RESNET50_CONVS
        return [dict(L, algo="gemm") for L in RESNET50_CONVS], "ResNet-50 conv stack forward: 53 convs, BN folded, algo gemm"
    if name == "mobilenet":
        layers = []
        for (c, hw) in MOBILENET_DEPTHWISE:
            for s in (1, 2):
                layers.append(dict(conv("dw3x3s%d_c%d_at%d" % (s, c, hw), 3, s, 1, c, c, hw, groups=c, activation="relu6"),
                                   algo="depthwise_separable"))
        for (ci, co, hw) in MOBILENET_POINTWISE:
            layers.append(dict(conv("pw1x1_%dto%d_at%d" % (ci, co, hw), 1, 1, 0, ci, co, hw, activation="relu6"), algo="gemm"))
        return layers, "MobileNet-v2 style blocks: depthwise 3x3 stride 1 and 2 + 1x1 pointwise, ReLU6"
    if name in ("winograd", "winograd-gemm"):
        algo = "winograd" if name == "winograd" else "gemm"
        layers = [dict(conv("3x3_%dto%d_at%d" % (ci, co, hw), 3, 1, 1, ci, co, hw), algo=algo) for (_, ci, co, hw) in WINOGRAD_SHAPES]
        return layers, "Winograd configuration shapes (3x3 s1 p1), algo %s" % algo
    raise SystemExit("unknown workload " + name)


def build_layers(layer_list, batch, seed, bf16=False):
    import numpy as np
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA
    from dlprimitives_amd.workloads import conv_bytes, conv_flops

    rng = np.random.default_rng(seed)
    tdt = torch.bfloat16 if bf16 else torch.float32
    out = []
    for L in layer_list:
        cin_g = L["cin"] // L["groups"]
        x = torch.from_numpy(rng.uniform(-1, 1, (batch, L["cin"], L["hw"], L["hw"])).astype(np.float32)).cuda().to(tdt)
        w = torch.from_numpy((rng.standard_normal((L["cout"], cin_g, L["kernel"], L["kernel"])) *
                              np.sqrt(2.0 / (cin_g * L["kernel"] ** 2))).astype(np.float32)).cuda().to(tdt)
        b = torch.from_numpy(rng.uniform(-0.1, 0.1, L["cout"]).astype(np.float32)).cuda()
        y = torch.empty((batch, L["cout"], L["ohw"], L["ohw"]), dtype=tdt, device="cuda")
        st = dlp.Conv2DSettings(L["cin"], L["cout"], L["kernel"], L["stride"], 1, L["pad"], L["groups"], tuple(x.shape),
                                dtype=BFLOAT16_DATA if bf16 else FLOAT_DATA)
        op = dlp.Conv2DForward.create(st, True, L["activation"], L["algo"])
        assert op.algo() == L["algo"], (op.algo(), L["algo"])
        ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda")
        packed = torch.empty(max(op.packed_size(), 1), dtype=torch.uint8, device="cuda")
        op.pack(w, packed)  # used only with --prepacked
        out.append(dict(layer=L, op=op, x=x, w=w, b=b, y=y, ws=ws, packed=packed, flops=conv_flops(L, batch), bytes=conv_bytes(L, batch, 2 if bf16 else 4)))
    return out


def kernel_class(L, bf16=False):
    """Name of the kernel that does the layer's arithmetic, as a profiler lists it."""
    if L["algo"] == "depthwise_separable":
        return "depthwise3x3_kernel<%s, %d>" % ("bf16_t" if bf16 else "float", L["stride"])
    cin_g = L["cin"] // L["groups"]
    m = L["cout"] // L["groups"]
    if L["algo"] == "winograd":
        return "wino_fused_kernel<%s, ...>" % ("bf16_t" if bf16 else "float")
    small = L["kernel"] ** 2 <= 31
    if bf16 and L["activation"] not in ("tanh", "sigmoid"):
        order = 2 if (small and cin_g % 32 == 0) else 3  # one tap x 32 channels per K tile, or the per-element table
        tile = "128, 128, 2, 2" if m > 64 else "64, 256, 1, 4"
        hw = L["hw"] * L["hw"]
        same3 = L["kernel"] == 3 and L["stride"] == 1 and L["pad"] == 1 and L.get("dilate", 1) == 1
        if order == 2 and same3 and hw % 4 == 0 and hw >= (128 if m > 64 else 254):
            # stride-1 3x3: input patch through LDS (the library falls back to the gather when the patch does not fit)
            return "conv_patch_bf16_kernel<%s, %d, %d, 0>" % (tile, 320 if m > 64 else 448, 8 if hw % 8 == 0 else 4)
        pxl = 0
        if order == 2 and L["kernel"] == 1 and L["stride"] == 1 and L["pad"] == 0 and hw % 4 == 0:
            pxl = 8 if hw % 8 == 0 else 4  # dense loader: 8 or 4 pixels per load
        return "conv_gemm_bf16_kernel<%s, %d, 0, 2, %d>" % (tile, order, pxl)
    if (not bf16 and L["groups"] == 1 and L["cin"] == 3 and L["kernel"] == 7 and L["stride"] == 2 and L["pad"] <= 4 and m % 8 == 0
            and L["hw"] <= 232 and L.get("dilate", 1) == 1):
        return "conv_stem_f32_kernel<3, 7, 7, 2, 8, 240, true, false>"  # input rows of a band and the filter in LDS, no gather
    tile = "64, 64, 2, 2" if m > 32 else "32, 128, 1, 4"
    order = 1 if (small and cin_g % 16 == 0) else 0
    if (not bf16 and order == 1 and m > 32 and L["kernel"] == 3 and L["stride"] == 1 and L["pad"] == 1 and L.get("dilate", 1) == 1
            and L["hw"] * L["hw"] >= 32 and 64 + 2 * (L["hw"] + 1) < 192 and L["activation"] not in ("tanh", "sigmoid")):
        return "conv_patch_f32_kernel<float, 3, 3, 192, 0>"  # stride-1 3x3: input patch through LDS, stream-K
    mask = 1 if small else 2
    return "conv_gemm_f32_kernel<%s, %s, %d, %d, 0>" % ("bf16_t" if bf16 else "float", tile, order, mask)


def matrix_peak_tflops(kernel_name):
    return BF16_MATRIX_PEAK_TFLOPS if kernel_name.startswith(("conv_gemm_bf16_kernel", "conv_patch_bf16_kernel")) else FP32_MATRIX_PEAK_TFLOPS


MAIN_SECTION = {"gemm": "conv_gemm", "winograd": "winograd_fused", "depthwise_separable": "sep_conv"}


def cpu_baseline(layer_list, images, seed, threads=1):
    """Oracle (port of the reference CPU path), `images` images through all layers; threads = 1 is the reference's
    own single-threaded loop over the batch, more threads distribute the (independent) images over OpenMP threads."""
    import numpy as np

    import oracle
    from dlprimitives_amd.workloads import conv_flops

    rng = np.random.default_rng(seed)
    total = 0.0
    flops = 0.0
    for L in layer_list:
        cin_g = L["cin"] // L["groups"]
        x = rng.uniform(-1, 1, (images, L["cin"], L["hw"], L["hw"])).astype(np.float32)
        w = (rng.standard_normal((L["cout"], cin_g, L["kernel"], L["kernel"])) * np.sqrt(2.0 / (cin_g * L["kernel"] ** 2))).astype(np.float32)
        b = rng.uniform(-0.1, 0.1, L["cout"]).astype(np.float32)
        cfg = oracle.make_cfg(L["cin"], L["cout"], L["kernel"], L["stride"], 1, L["pad"], L["groups"])
        t0 = time.perf_counter()
        oracle.conv2d_forward(x, w, b, cfg, L["activation"], threads=threads)
        total += time.perf_counter() - t0
        flops += conv_flops(L, images)
    return dict(value=round(images / total, 3), unit="images/s", cores=threads, kind="port",
                sample="%d images through all %d layers of the workload, %s, %.1f s" % (
                    images, len(layer_list), "single thread" if threads == 1 else "%d OpenMP threads over the batch" % threads, total),
                gflops_per_s=round(flops / total / 1e9, 2))


def run_graph_workload(args):
    """Whole-network forward (convolutions + pooling + residual adds + global pooling + inner
    product) through the C-ABI operators; same JSON contract, no per-kernel roofline split."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd import graphs

    net = args.workload[:-len("-full")]
    ops = getattr(graphs, net)()
    params = graphs.random_parameters(ops, 2024)
    shape = (args.batch, 3, 224, 224)
    bf16 = args.dtype == "bf16"
    runner = graphs.GraphRunner(ops, params, shape, algo=args.algo, dtype="bfloat16" if bf16 else "float32")
    x = torch.rand(shape, device="cuda:0") * 2 - 1
    runner.t["data"].copy_(x)  # converts to the storage type
    for _ in range(args.warmup):
        runner.forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        runner.forward()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    dlp.timing_reset()
    dlp.timing_enable(True)
    runner.forward()
    torch.cuda.synchronize()
    dlp.timing_enable(False)
    sections = {}
    for (section, ms) in dlp.timing_records():
        sections[section] = round(sections.get(section, 0.0) + ms, 4)
    dlp.timing_reset()
    flops = runner.flops()
    conv_ms = sections.get("conv_gemm", 0.0) + sections.get("winograd_fused", 0.0)
    out = {
        "metric": BASELINE_METRIC, "value": round(args.batch / (ms_per_step * 1e-3), 1), "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32 arithmetic on bf16-stored tensors" if bf16 else "f32", "data": "synthetic",
        "config": {"workload": "%s full forward (conv + BN folded + ReLU, max pool, residual adds, global avg pool, inner product), "
                               "%s NCHW, batch %d, 224x224, conv algo '%s'" % (net, "bf16 storage" if bf16 else "fp32", args.batch,
                                                                                 args.algo or "auto"),
                   "batch": args.batch, "gflop_per_step": round(flops / 1e9, 1)},
        "gflops_per_s": round(flops / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_of_fp32_matrix_peak": round(flops / (ms_per_step * 1e-3) / 1e12 / FP32_MATRIX_PEAK_TFLOPS, 4),
        "kernel_ms_by_section": sections,
        "roofline": {"bound": "mfma", "kernel": "conv_gemm + wino_fused (all launches of one forward; direct-convolution flops)", "achieved": round(flops / (conv_ms * 1e-3) / 1e12, 2) if conv_ms else None,
                     "peak": FP32_MATRIX_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(flops / (conv_ms * 1e-3) / 1e12 / FP32_MATRIX_PEAK_TFLOPS, 4) if conv_ms else None,
                     "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(out))


def run_backward_workload(args):
    """Backward data + backward filter of every layer of the ResNet-18 convolution stack; same JSON
    contract; roofline for the backward-filter kernel (its flops = the forward convolution's)."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.workloads import RESNET18_CONVS, conv_flops

    torch.manual_seed(2024)
    layers = []
    for L in RESNET18_CONVS:
        st = dlp.Conv2DSettings(L["cin"], L["cout"], L["kernel"], L["stride"], 1, L["pad"], L["groups"], (args.batch, L["cin"], L["hw"], L["hw"]))
        osh = dlp.conv2d_output_shape(st, st.shape)
        e = dict(L=L, x=torch.randn(st.shape, device="cuda:0"),
                 w=torch.randn(L["cout"], L["cin"] // L["groups"], L["kernel"], L["kernel"], device="cuda:0"),
                 dy=torch.randn(osh, device="cuda:0"), bf=dlp.Conv2DBackwardFilter.create(st), bd=None if L["cin"] == 3 else dlp.Conv2DBackwardData.create(st))
        e["dx"], e["dw"] = torch.empty_like(e["x"]), torch.empty_like(e["w"])
        e["ws"] = torch.empty(max(e["bf"].workspace(), e["bd"].workspace() if e["bd"] else 0, 1), dtype=torch.uint8, device="cuda:0")
        layers.append(e)

    def step():
        for e in layers:
            e["bf"].enqueue(e["x"], e["dw"], e["dy"], e["ws"])
            if e["bd"]:
                e["bd"].enqueue(e["dx"], e["w"], e["dy"], e["ws"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    dlp.timing_reset()
    dlp.timing_enable(True)
    step()
    torch.cuda.synchronize()
    dlp.timing_enable(False)
    sections = {}
    for (section, ms) in dlp.timing_records():
        sections[section] = round(sections.get(section, 0.0) + ms, 4)
    dlp.timing_reset()
    flops_f = sum(conv_flops(e["L"], args.batch) for e in layers)
    flops_d = sum(conv_flops(e["L"], args.batch) for e in layers if e["bd"])
    wgrad_ms = sections.get("wgrad", 0.0)
    out = {
        "metric": BASELINE_METRIC, "value": round(args.batch / (ms_per_step * 1e-3), 1), "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "gradients of the ResNet-18 convolution stack: backward filter of 20 layers, backward data of 19 (not conv1), "
                               "fp32 NCHW, batch %d" % args.batch, "batch": args.batch,
                   "gflop_per_step": round((flops_f + flops_d) / 1e9, 1)},
        "gflops_per_s": round((flops_f + flops_d) / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_of_fp32_matrix_peak": round((flops_f + flops_d) / (ms_per_step * 1e-3) / 1e12 / FP32_MATRIX_PEAK_TFLOPS, 4),
        "kernel_ms_by_section": sections,
        "roofline": {"bound": "mfma", "kernel": "conv_wgrad_f32_kernel (20 launches)", "achieved": round(flops_f / (wgrad_ms * 1e-3) / 1e12, 2) if wgrad_ms else None,
                     "peak": FP32_MATRIX_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(flops_f / (wgrad_ms * 1e-3) / 1e12 / FP32_MATRIX_PEAK_TFLOPS, 4) if wgrad_ms else None, "traffic": None},
        "cpu_baseline": None,
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--workload", default="resnet18", choices=["resnet18", "resnet50", "mobilenet", "winograd", "winograd-gemm", "resnet18-full", "resnet50-full", "resnet18-backward"])
    ap.add_argument("--algo", default="gemm", help="conv algorithm of the -full workloads ('' = auto)")
    ap.add_argument("--dtype", default="f32", choices=["f32", "bf16"], help="storage type of the tensors (accumulation and epilogue are fp32 either way)")
    ap.add_argument("--cpu-images", type=int, default=8, help="images of the CPU baseline sample (0 = skip)")
    ap.add_argument("--layers", action="store_true", help="also print the per-layer table to stderr")
    ap.add_argument("--prepacked", action="store_true",
                    help="weights transformed once before the timed region (dlp_conv2d_fwd_pack / _enqueue_packed), as an inference "
                         "deployment does; the default transforms them in every step, as the reference's enqueue contract implies")
    ap.add_argument("--only", default="", help="profiling aid: keep only layers whose name contains this text")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; --gpus %d is not supported (the path shards over batch with no exchange)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch

    import dlprimitives_amd as dlp

    dlp.lib()  # fails loudly when the HIP library is missing
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.workload.endswith("-full"):
        run_graph_workload(args)
        return
    if args.workload == "resnet18-backward":
        run_backward_workload(args)
        return
    layer_list, description = workload_layers(args.workload)
    if args.only:
        layer_list = [L for L in layer_list if args.only in L["name"]]
        if not layer_list:
            print("bench.py: --only matches no layer", file=sys.stderr)
            sys.exit(2)
    bf16 = args.dtype == "bf16"
    layers = build_layers(layer_list, args.batch, 2024, bf16)
    stream = torch.cuda.current_stream()

    def step():
        if args.prepacked:
            for e in layers:
                e["op"].enqueue_packed(e["x"], e["w"], e["packed"], e["b"], e["y"], e["ws"], 0.0)
        else:
            for e in layers:
                e["op"].enqueue(e["x"], e["w"], e["b"], e["y"], e["ws"], 0.0)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    total_flops = sum(e["flops"] for e in layers)
    total_bytes = sum(e["bytes"] for e in layers)

    # second pass: the library's own per-kernel timing (a HIP event pair around every
    # kernel launch, on the launch stream); a layer = its main kernel + helper kernels
    nl = len(layers)
    dlp.timing_reset()
    dlp.timing_enable(True)
    spans = []
    for s in range(args.steps):
        for i, e in enumerate(layers):
            first = dlp.timing_count()
            if args.prepacked:
                e["op"].enqueue_packed(e["x"], e["w"], e["packed"], e["b"], e["y"], e["ws"], 0.0)
            else:
                e["op"].enqueue(e["x"], e["w"], e["b"], e["y"], e["ws"], 0.0)
            spans.append((i, first, dlp.timing_count()))
    torch.cuda.synchronize()
    dlp.timing_enable(False)
    records = dlp.timing_records()
    layer_ms = [0.0] * nl   # all kernels of the layer
    kernel_ms = [0.0] * nl  # the main kernel only
    for (i, first, last) in spans:
        main = MAIN_SECTION[layers[i]["layer"]["algo"]]
        for (section, ms) in records[first:last]:
            layer_ms[i] += ms / args.steps
            if section == main:
                kernel_ms[i] += ms / args.steps
    dlp.timing_reset()

    table = []
    classes = {}
    for e, ms, kms in zip(layers, layer_ms, kernel_ms):
        L = e["layer"]
        kname = kernel_class(L, bf16)
        peak = matrix_peak_tflops(kname) * 1e12
        ai = e["flops"] / e["bytes"]
        mfma_bound = ai * HBM_PEAK_GBS * 1e9 >= peak
        roof = min(peak, ai * HBM_PEAK_GBS * 1e9)
        ach = e["flops"] / (ms * 1e-3)
        table.append(dict(name=L["name"], ms=round(ms, 4), main_kernel_ms=round(kms, 4), tflops=round(ach / 1e12, 2), gbs=round(e["bytes"] / (ms * 1e-3) / 1e9, 1),
                          bound="mfma" if mfma_bound else "hbm", frac_of_roofline=round(ach / roof, 4), kernel=kname))
        c = classes.setdefault(kname, dict(ms=0.0, flops=0.0, bytes=0.0, launches=0, hbm=0))
        c["ms"] += kms
        # Winograd F(2x2,3x3) multiplies 16 values per 2x2 outputs instead of 36: the matrix-core
        # fraction is scored on the flops actually issued (direct / 2.25), so it cannot pass 100 %
        c["flops"] += e["flops"] / 2.25 if L["algo"] == "winograd" else e["flops"]
        c["bytes"] += e["bytes"]
        c["launches"] += 1
        c["hbm"] += 0 if mfma_bound else 1
    dom_name, dom = max(classes.items(), key=lambda kv: kv[1]["ms"])
    if dom["hbm"] * 2 > dom["launches"]:  # a bandwidth-bound kernel class: score achieved bytes/s
        achieved = dom["bytes"] / (dom["ms"] * 1e-3) / 1e9
        roofline = dict(bound="hbm", kernel=dom_name, launches_per_step=dom["launches"], avg_launch_ms=round(dom["ms"] / dom["launches"], 4),
                        bytes_per_launch=dom["bytes"] / dom["launches"], achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                        frac=round(achieved / HBM_PEAK_GBS, 4), traffic=None)
    else:
        achieved = dom["flops"] / (dom["ms"] * 1e-3) / 1e12
        peak_tf = matrix_peak_tflops(dom_name)
        roofline = dict(bound="mfma", kernel=dom_name, launches_per_step=dom["launches"], avg_launch_ms=round(dom["ms"] / dom["launches"], 4),
                        flops_per_launch=dom["flops"] / dom["launches"], bytes_per_launch=dom["bytes"] / dom["launches"],
                        achieved=round(achieved, 2), peak=peak_tf,
                        unit="TFLOP/s", frac=round(achieved / peak_tf, 4), traffic=None)
    if args.batch == 64 and not args.only:
        roofline["traffic"] = MEASURED_TRAFFIC_BYTES.get((args.workload, dom_name))
    if args.layers:
        for r in table:
            print(json.dumps(r), file=sys.stderr)

    cpu = cpu_baseline(layer_list, args.cpu_images, 2024) if args.cpu_images > 0 else None  # the fp32 reference path
    # the same arithmetic with the batch spread over the host's cores (what a reference build with a threaded BLAS
    # would approach); the box gives a GPU 16 cores whatever os.cpu_count() says
    cpu_mt = None
    if args.cpu_images > 0:
        nthreads = max(1, min(16, os.cpu_count() or 1))
        cpu_mt = cpu_baseline(layer_list, max(args.cpu_images, 2 * nthreads), 2024, threads=nthreads)

    out = {
        "metric": BASELINE_METRIC,
        "value": round(args.batch / (ms_per_step * 1e-3), 1),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16 storage, fp32 accumulate" if bf16 else "f32",
        "data": "synthetic",
        "config": {"workload": "%s%s, %s NCHW, batch %d" % (description, " (subset --only %s)" % args.only if args.only else "",
                                                            "bf16" if bf16 else "fp32", args.batch) +
                               (", weights packed once before the timed region" if args.prepacked else ""),
                   "batch": args.batch, "layers": nl, "gflop_per_step": round(total_flops / 1e9, 1),
                   "mbytes_per_step": round(total_bytes / 1e6, 1)},
        "gflops_per_s": round(total_flops / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_of_fp32_matrix_peak": round(total_flops / (ms_per_step * 1e-3) / 1e12 / FP32_MATRIX_PEAK_TFLOPS, 4),
        "kernel_ms_per_step": round(sum(layer_ms), 4),
        "roofline": roofline,
        "cpu_baseline": cpu,
        "cpu_baseline_all_cores": cpu_mt,
        "layers": table,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
