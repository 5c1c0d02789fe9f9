#!/usr/bin/env python3
"""Benchmark of the convolution forward hot path on one MI355X.

Default workload (the configuration the headline metric is quoted on): the 20
convolutions of the ResNet-18 conv stack, forward, fp32 NCHW, batch 64, BN folded
into weights + bias, fused ReLU, algorithm "gemm" (implicit GEMM on fp32 MFMA).
A step = one pass over all layers of the workload, launched back to back on one
stream, with every tensor already resident in HBM.  Synthetic data: inputs
uniform[-1,1], weights Kaiming-normal, bias uniform[-0.1,0.1], fixed seed.

Other workloads (same JSON contract, for the remaining configurations):
  --workload single         one 3x3 64->64 convolution at 56x56 (configuration 1 with --batch 16)
  --workload mobilenet      depthwise 3x3 stride 1/2 (HBM bound) + 1x1 pointwise, ReLU6
  --workload mobilenet-fused  the same layers with the depthwise -> pointwise pairs the library fuses run as one launch each
  --workload winograd       the two Winograd shapes, algo winograd
  --workload winograd-gemm  the same two shapes through the implicit GEMM
  --workload resnet18-full / resnet50-full   whole network forward incl. pooling, adds, GAP, IP
  --workload resnet18-backward   gradients of the 20 ResNet-18 convolutions (backward filter for all,
                            backward data for all but conv1, whose input needs none), fp32

The default run (no flags) also carries a `configs` object: the other four configurations of the baseline
(single layer at batch 16; the two Winograd shapes through "winograd" and through "gemm"; the MobileNet blocks with
every depthwise layer scored against 8 TB/s and against a plain streaming kernel on tensors of the same size;
the whole ResNet-50 forward in bf16 storage at batch 128), each with ms_per_step, its dominant kernel and that
kernel's roofline fraction, plus `measured_peak` (MFMA-only loops and streaming copies run on this device) next
to `vendor_peak`.  Kernel names come from the library's timing records (dlp_timing_get_kernel), not from this file.

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
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hbm_traffic_counters.txt")


def measured_traffic_bytes(workload, kernel):
    """HBM bytes per launch of `kernel` in `workload` at batch 64, from the hardware-counter summary kept under
    profiles/ (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, one counter per run, KiB per dispatch; a benchmark run
    cannot collect counters on itself).  Each counter is scaled by what it reads for the copy kernel of known size in
    the same file.  None when the file has no row for this kernel: a renamed or new kernel has no stale number."""
    try:
        lines = open(TRAFFIC_PROFILE).read().splitlines()
    except OSError:
        return None
    section, rows = None, {}
    for ln in lines:
        if ln.startswith("== "):
            section = ln[3:].split()[0]
            continue
        if section and " n=" in ln and "FETCH_SIZE" in ln and "WRITE_SIZE" in ln:
            name = ln[:ln.index(" n=")].strip()
            t = ln.split()
            rows.setdefault(section, []).append((name, float(t[t.index("FETCH_SIZE") + 1]), float(t[t.index("WRITE_SIZE") + 1])))
    copy = [r for r in rows.get("copy", []) if r[0].startswith(("copy_f4", "stream_kernel<1, 256, false>"))]
    if not copy or copy[0][1] <= 0 or copy[0][2] <= 0:
        return None
    copied_kib = 262144.0  # the calibration run copies 256 MiB per launch
    fetch_scale, write_scale = copied_kib / copy[0][1], copied_kib / copy[0][2]
    for (name, fetch, write) in rows.get(workload, []):
        if kernel == name or (len(name) >= 50 and kernel.startswith(name)):  # (older summaries cut names at 50 characters)
            return (fetch * fetch_scale + write * write_scale) * 1024
    return None


def workload_layers(name):
    from dlprimitives_amd.workloads import MOBILENET_DEPTHWISE, MOBILENET_POINTWISE, RESNET18_CONVS, WINOGRAD_SHAPES, conv

    if name == "single":
        return [dict(conv("3x3_64to64_at56", 3, 1, 1, 64, 64, 56), algo="gemm")], "single Conv2D 3x3 s1 p1 64->64 at 56x56, bias + ReLU, algo gemm"
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


def matrix_peak_tflops(kernel_name):
    return BF16_MATRIX_PEAK_TFLOPS if kernel_name.startswith(("conv_gemm_bf16_kernel", "conv_patch_bf16_kernel", "conv_stem_bf16_kernel")) else FP32_MATRIX_PEAK_TFLOPS


MAIN_SECTION = {"gemm": "conv_gemm", "winograd": "winograd_fused", "depthwise_separable": "sep_conv"}


def cpu_baseline(layer_list, images, seed, threads=1, runs=3):
    """Oracle (port of the reference CPU path), `images` images through all layers; threads = 1 is the reference's
    own single-threaded loop over the batch, more threads distribute the (independent) images over OpenMP threads.
    One untimed pass, then the mean of `runs` timed passes (std::chrono around forward in the reference's own flops tool,
    tools/flops.cpp:594-671; docs/benchmarks/methodology.md:3-6 warms up before it times)."""
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
        for run in range(-1, runs):
            t0 = time.perf_counter()
            oracle.conv2d_forward(x, w, b, cfg, L["activation"], threads=threads)
            if run >= 0:
                total += (time.perf_counter() - t0) / runs
        flops += conv_flops(L, images)
    return dict(value=round(images / total, 3), unit="images/s", cores=threads, kind="port",
                sample="%d images through all %d layers of the workload, %s, 1 untimed + %d timed passes of %.2f s" % (
                    images, len(layer_list), "single thread" if threads == 1 else "%d OpenMP threads over the batch" % threads, runs, total),
                gflops_per_s=round(flops / total / 1e9, 2))


def run_graph_workload(args):
    return graph_workload(args.workload[:-len("-full")], args.batch, args.algo, args.dtype == "bf16", args.steps, args.warmup, args.fuse_residual, args.prepacked,
                          args.channels_last, args.fuse_stem_pool)


def graph_workload(net, batch, algo, bf16, steps, warmup, fuse_residual=False, prepack=False, channels_last=False, fuse_stem_pool=False):
    """Whole-network forward (convolutions + pooling + residual adds + global pooling + inner
    product) through the C-ABI operators; same JSON contract, no per-kernel roofline split."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd import graphs

    ops = getattr(graphs, net)()
    params = graphs.random_parameters(ops, 2024)
    shape = (batch, 3, 224, 224)
    runner = graphs.GraphRunner(ops, params, shape, algo=algo, dtype="bfloat16" if bf16 else "float32", fuse_residual=fuse_residual, prepack=prepack,
                                channels_last=channels_last, fuse_stem_pool=fuse_stem_pool)
    pooled_inside = sum(1 for o in runner.ops if o.get("pool"))
    x = torch.rand(shape, device="cuda:0") * 2 - 1
    runner.t["data"].copy_(x)  # converts to the storage type
    for _ in range(warmup):
        runner.forward()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        runner.forward()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    dlp.timing_reset()
    dlp.timing_enable(True)
    runner.forward()
    torch.cuda.synchronize()
    dlp.timing_enable(False)
    sections, by_kernel = {}, {}
    for (section, ms, kname) in dlp.timing_records(kernels=True):
        sections[section] = round(sections.get(section, 0.0) + ms, 4)
        if section in ("conv_gemm", "winograd_fused"):
            by_kernel[kname] = by_kernel.get(kname, 0.0) + ms
    dlp.timing_reset()
    flops = runner.flops()
    conv_ms = sections.get("conv_gemm", 0.0) + sections.get("winograd_fused", 0.0)
    peak = BF16_MATRIX_PEAK_TFLOPS if bf16 else FP32_MATRIX_PEAK_TFLOPS
    dominant = max(by_kernel.items(), key=lambda kv: kv[1])[0] if by_kernel else ""
    return {
        "metric": BASELINE_METRIC, "value": round(batch / (ms_per_step * 1e-3), 1), "unit": "images/s", "n_gpus": 1,
        "steps": steps, "warmup": warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16 storage, fp32 accumulate" if bf16 else "f32", "data": "synthetic",
        "config": {"workload": "%s full forward (conv + BN folded + ReLU, max pool, residual adds%s, global avg pool, inner product), "
                               "%s NCHW, batch %d, 224x224, conv algo '%s'%s" % (net, " in the epilogue of the 1x1 convolution in front of them" if fuse_residual else "",
                                                                               "bf16 storage" if bf16 else "fp32", batch, algo or "auto",
                                                                               ", filters transformed once before the timed region" if prepack else "") +
                               ("; %d of the tensors between operators kept channels-last (input, logits and parameters as given)" % len(runner.cl) if runner.cl else "") +
                               ("; the stem's max pooling runs inside the stem's convolution kernel (its time counts as convolution time)" if pooled_inside else ""),
                   "batch": batch, "gflop_per_step": round(flops / 1e9, 1)},
        "gflops_per_s": round(flops / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_of_matrix_peak_whole_pass": round(flops / (ms_per_step * 1e-3) / 1e12 / peak, 4),
        "kernel_ms_by_section": sections,
        "roofline": {"bound": "mfma", "kernel": "all convolution launches of one forward (direct-convolution flops); largest share: " + dominant,
                     "achieved": round(flops / (conv_ms * 1e-3) / 1e12, 2) if conv_ms else None,
                     "peak": peak, "unit": "TFLOP/s", "frac": round(flops / (conv_ms * 1e-3) / 1e12 / peak, 4) if conv_ms else None,
                     "traffic": None},
        "cpu_baseline": None,
        "dominant_kernel": dominant,
    }


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


def run_conv_workload(workload, batch, bf16, steps, warmup, prepacked=False, only="", seed=2024, warm_seconds=0.0):
    """Times `steps` passes over the layers of a convolution workload (back to back on one stream, tensors resident),
    then a second pass with the library's per-kernel timing.  Returns the pieces of the JSON line.
    warm_seconds: keep running untimed passes after the `warmup` ones until this much time has gone by (the sub-millisecond
    configurations otherwise start their timed passes before the device has left its idle clocks)."""
    import torch

    import dlprimitives_amd as dlp

    layer_list, description = workload_layers(workload)
    if only:
        layer_list = [L for L in layer_list if only in L["name"]]
        if not layer_list:
            print("bench.py: --only matches no layer", file=sys.stderr)
            sys.exit(2)
    layers = build_layers(layer_list, batch, seed, bf16)

    def enqueue(e):
        if prepacked:
            e["op"].enqueue_packed(e["x"], e["w"], e["packed"], e["b"], e["y"], e["ws"], 0.0)
        else:
            e["op"].enqueue(e["x"], e["w"], e["b"], e["y"], e["ws"], 0.0)

    def step():
        for e in layers:
            enqueue(e)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < warm_seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    total_flops = sum(e["flops"] for e in layers)
    total_bytes = sum(e["bytes"] for e in layers)

    # second pass: the library's own per-kernel timing (a HIP event pair around every kernel launch, on the launch
    # stream); a layer = its main kernel + helper kernels.  The records also say which kernel ran.
    nl = len(layers)
    dlp.timing_reset()
    dlp.timing_enable(True)
    spans = []
    for _ in range(steps):
        for i, e in enumerate(layers):
            first = dlp.timing_count()
            enqueue(e)
            spans.append((i, first, dlp.timing_count()))
    torch.cuda.synchronize()
    dlp.timing_enable(False)
    records = dlp.timing_records(kernels=True)
    layer_ms = [0.0] * nl   # all kernels of the layer
    kernel_ms = [0.0] * nl  # the main kernel only
    kernel_name = [""] * nl
    for (i, first, last) in spans:
        main = MAIN_SECTION[layers[i]["layer"]["algo"]]
        for (section, ms, kname) in records[first:last]:
            layer_ms[i] += ms / steps
            if section == main:
                kernel_ms[i] += ms / steps
                kernel_name[i] = kname or section
    dlp.timing_reset()

    table = []
    classes = {}
    for e, ms, kms, kname in zip(layers, layer_ms, kernel_ms, kernel_name):
        L = e["layer"]
        peak = matrix_peak_tflops(kname) * 1e12
        ai = e["flops"] / e["bytes"]
        mfma_bound = ai * HBM_PEAK_GBS * 1e9 >= peak
        roof = min(peak, ai * HBM_PEAK_GBS * 1e9)
        # Winograd F(2x2,3x3) multiplies 16 values per 2x2 outputs instead of 36: against the matrix peak it is scored
        # on the flops it issues (direct / 2.25), so the fraction cannot pass 100 %; tflops stays direct-equivalent
        issued = e["flops"] / 2.25 if L["algo"] == "winograd" else e["flops"]
        row = dict(name=L["name"], ms=round(ms, 4), main_kernel_ms=round(kms, 4), tflops=round(e["flops"] / (ms * 1e-3) / 1e12, 2),
                   gbs=round(e["bytes"] / (ms * 1e-3) / 1e9, 1), bound="mfma" if mfma_bound else "hbm",
                   frac_of_roofline=round((issued if mfma_bound else e["flops"]) / (ms * 1e-3) / roof, 4), kernel=kname)
        if L["algo"] == "winograd":
            row["tflops_issued"] = round(issued / (ms * 1e-3) / 1e12, 2)
        table.append(row)
        c = classes.setdefault(kname, dict(ms=0.0, flops=0.0, bytes=0.0, launches=0, hbm=0))
        c["ms"] += kms
        c["flops"] += issued
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
    if batch == 64 and not only and not bf16:
        roofline["traffic"] = measured_traffic_bytes(workload, dom_name)
    return dict(layer_list=layer_list, description=description, ms_per_step=ms_per_step, total_flops=total_flops, total_bytes=total_bytes,
                kernel_ms_per_step=sum(layer_ms), roofline=roofline, table=table, nl=nl)


def isolated_layer_us(L, batch, bf16=False, ring_bytes=768 << 20, seed=7, warm_seconds=0.2, cached=False):
    """One layer alone: launches back to back, each on its own x / y pair out of a ring larger than the 256 MB last-level
    cache (every launch starts cold, as inside a network), ONE event pair around all of them.  An event between two
    launches makes the first write its part of the L2 back before it ends, which inflates short kernels by microseconds;
    this is how the streaming kernels of the probe (copy_at_size) are timed as well.
    cached=True: a ring of two pairs only, so x and y of every launch still sit in the last-level cache from the launch
    before last -- the state a small layer finds its input in when the preceding layer has just written it."""
    import torch

    import dlprimitives_amd as dlp
    from dlprimitives_amd.capi import BFLOAT16_DATA, FLOAT_DATA

    tdt = torch.bfloat16 if bf16 else torch.float32
    es = 2 if bf16 else 4
    cin_g = L["cin"] // L["groups"]
    xshape = (batch, L["cin"], L["hw"], L["hw"])
    yshape = (batch, L["cout"], L["ohw"], L["ohw"])
    pair = es * (batch * L["cin"] * L["hw"] ** 2 + batch * L["cout"] * L["ohw"] ** 2)
    ring = 2 if cached else max(3, min(48, ring_bytes // pair + 1))
    g = torch.Generator(device="cuda").manual_seed(seed)
    xs = [(torch.rand(xshape, device="cuda", generator=g) * 2 - 1).to(tdt) for _ in range(ring)]
    ys = [torch.empty(yshape, dtype=tdt, device="cuda") for _ in range(ring)]
    w = (torch.randn((L["cout"], cin_g, L["kernel"], L["kernel"]), device="cuda", generator=g) * (2.0 / (cin_g * L["kernel"] ** 2)) ** 0.5).to(tdt)
    b = torch.rand(L["cout"], device="cuda", generator=g) * 0.2 - 0.1
    st = dlp.Conv2DSettings(L["cin"], L["cout"], L["kernel"], L["stride"], 1, L["pad"], L["groups"], xshape, dtype=BFLOAT16_DATA if bf16 else FLOAT_DATA)
    op = dlp.Conv2DForward.create(st, True, L["activation"], L["algo"])
    ws = torch.empty(max(op.workspace(), 1), dtype=torch.uint8, device="cuda")
    reps = 60 if cached else 3 * ring
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < warm_seconds:  # untimed launches until the device runs at its working clocks
        for j in range(ring):
            op.enqueue(xs[j], w, b, ys[j], ws, 0.0)
        torch.cuda.synchronize()
    # One pass over the ring is recorded as a HIP graph and replayed: a launch of a few microseconds is shorter than the
    # host's path through the Python binding, and the layer would otherwise be timed at the host's launch rate.
    graph = None
    per_graph = max(ring, 24)  # launches per replay: a replay has a start-up cost of its own, which two launches would not amortise
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for j in range(per_graph):
                    op.enqueue(xs[j % ring], w, b, ys[j % ring], ws, 0.0)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
    except Exception:  # a layer whose enqueue cannot be captured is timed eagerly
        graph = None
        torch.cuda.synchronize()
    if graph is not None:
        passes = max(3, reps // per_graph)
        graph.replay()
        e0.record()
        for _ in range(passes):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e3 / (passes * per_graph)
    for r in range(-ring, reps):
        if r == 0:
            e0.record()
        j = r % ring
        op.enqueue(xs[j], w, b, ys[j], ws, 0.0)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def mobilenet_pairs(layer_list):
    """(index of a depthwise layer, index of the pointwise layer that can follow it): same channels, the depthwise
    layer's output size; every layer in at most one pair."""
    pairs, used = [], set()
    for i, d in enumerate(layer_list):
        if d["algo"] != "depthwise_separable":
            continue
        for j, p in enumerate(layer_list):
            if j not in used and p["kernel"] == 1 and p["groups"] == 1 and p["cin"] == d["cout"] and p["hw"] == d["ohw"]:
                pairs.append((i, j))
                used.add(j)
                break
    return pairs


def fused_pair_op(D, P, batch):
    """The depthwise layer D and the pointwise layer P as ONE operator (dlp_dwpw_fwd_*), or None where the library keeps them apart."""
    import dlprimitives_amd as dlp

    st = dlp.Conv2DSettings(D["cin"], D["cout"], 3, D["stride"], 1, 1, D["groups"], (batch, D["cin"], D["hw"], D["hw"]))
    if D["kernel"] != 3 or D["pad"] != 1 or not dlp.DepthwisePointwiseForward.supported(st, D["activation"], P["cout"], P["activation"]):
        return None
    return dlp.DepthwisePointwiseForward.create(st, True, D["activation"], P["cout"], True, P["activation"])


def isolated_fused_us(D, P, batch, ring_bytes=768 << 20, seed=7, warm_seconds=0.2):
    """isolated_layer_us for the fused depthwise + pointwise operator: x of the depthwise layer in, y of the pointwise layer out."""
    import torch

    op = fused_pair_op(D, P, batch)
    xshape = (batch, D["cin"], D["hw"], D["hw"])
    yshape = (batch, P["cout"], P["ohw"], P["ohw"])
    pair = 4 * (batch * D["cin"] * D["hw"] ** 2 + batch * P["cout"] * P["ohw"] ** 2)
    ring = max(3, min(48, ring_bytes // pair + 1))
    g = torch.Generator(device="cuda").manual_seed(seed)
    xs = [torch.rand(xshape, device="cuda", generator=g) * 2 - 1 for _ in range(ring)]
    ys = [torch.empty(yshape, device="cuda") for _ in range(ring)]
    wd = torch.randn((D["cout"], 1, 3, 3), device="cuda", generator=g) * (2.0 / 9) ** 0.5
    bd = torch.rand(D["cout"], device="cuda", generator=g) * 0.2 - 0.1
    wp = torch.randn((P["cout"], P["cin"], 1, 1), device="cuda", generator=g) * (2.0 / P["cin"]) ** 0.5
    bp = torch.rand(P["cout"], device="cuda", generator=g) * 0.2 - 0.1
    reps = 3 * ring
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < warm_seconds:
        for j in range(ring):
            op.enqueue(xs[j], wd, bd, wp, bp, ys[j])
        torch.cuda.synchronize()
    for r in range(-ring, reps):
        if r == 0:
            e0.record()
        op.enqueue(xs[r % ring], wd, bd, wp, bp, ys[r % ring])
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def mobilenet_fused_pass_ms(batch, steps, warmup, warm_seconds=0.3, seed=2024):
    """The mobilenet workload with every pair the library fuses run as one operator (the pointwise layer reads what the
    depthwise stage left on the chip); the other layers as in run_conv_workload.  Wall clock per pass."""
    import torch

    layer_list, _ = workload_layers("mobilenet")
    layers = build_layers(layer_list, batch, seed)
    fused, skip = {}, set()
    for (i, j) in mobilenet_pairs(layer_list):
        op = fused_pair_op(layer_list[i], layer_list[j], batch)
        if op is not None:
            fused[i] = (op, j)
            skip.add(j)

    def step():
        for i, e in enumerate(layers):
            if i in fused:
                op, j = fused[i]
                op.enqueue(e["x"], e["w"], e["b"], layers[j]["w"], layers[j]["b"], layers[j]["y"])
            elif i not in skip:
                e["op"].enqueue(e["x"], e["w"], e["b"], e["y"], e["ws"], 0.0)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t_warm = time.perf_counter()
    while time.perf_counter() - t_warm < warm_seconds:
        for _ in range(20):
            step()
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3, len(fused)


def compact(r, batch, extra=None):
    """One configuration as an entry of the `configs` object of the default line."""
    rf = r["roofline"]
    out = {"workload": r["description"], "batch": batch, "ms_per_step": round(r["ms_per_step"], 4),
           "images_per_s": round(batch / (r["ms_per_step"] * 1e-3), 1), "gflops_per_s": round(r["total_flops"] / (r["ms_per_step"] * 1e-3) / 1e9, 1),
           "kernel": rf["kernel"], "bound": rf["bound"], "achieved": rf["achieved"], "unit": rf["unit"], "frac": rf["frac"]}
    if extra:
        out.update(extra)
    return out


def other_configs(steps, warmup, peaks, with_cpu=True):
    """Configurations 1, 3, 4 and 5 of the baseline, each through the same timing as the headline (fewer steps)."""
    import torch

    from dlprimitives_amd import probe

    cfgs = {}
    # a pass of these two configurations lasts 40-250 us: 200 timed passes after 0.3 s of untimed ones, so that the
    # wall clock around them measures the kernels and not the wake-up of the device or the one synchronization
    small = dict(steps=max(steps, 200), warmup=warmup, warm_seconds=0.3)
    r = run_conv_workload("single", 16, False, **small)
    cfgs["config1_single_conv_b16"] = compact(r, 16, {"steps": small["steps"], "warm_seconds": 0.3})
    if with_cpu:  # the whole layer at its own batch, one thread: the reference's CPU path as it is built
        cfgs["config1_single_conv_b16"]["cpu_baseline"] = cpu_baseline(r["layer_list"], 16, 2024)
    # the headline's stack again as a caller with constant filters runs it (dlp_conv2d_fwd_pack once, _enqueue_packed per step):
    # what the packing launches inside the headline's timed step cost
    r = run_conv_workload("resnet18", 64, False, steps, warmup, prepacked=True, warm_seconds=0.3)
    cfgs["config2_filters_packed_once"] = compact(r, 64, {})
    for wl in ("winograd", "winograd-gemm"):
        r = run_conv_workload(wl, 64, False, **small)
        cfgs["config3_%s" % wl.replace("-", "_")] = compact(r, 64, {"layers": [
            {k: row[k] for k in ("name", "ms", "main_kernel_ms", "tflops", "tflops_issued", "frac_of_roofline", "kernel") if k in row} for row in r["table"]]})
        if with_cpu and wl == "winograd":  # both shapes, 16 of the 64 images each (images are independent), one thread
            cfgs["config3_winograd"]["cpu_baseline"] = cpu_baseline(r["layer_list"], 16, 2024)
    r = run_conv_workload("mobilenet", 64, False, max(steps, 100), warmup, warm_seconds=0.3)
    rows = []
    for L, row in zip(r["layer_list"], r["table"]):
        e = {k: row[k] for k in ("name", "kernel")}
        e["ms_in_sequence"] = row["ms"]  # inside the 16-layer pass, event pair per launch
        # the layer alone, launches back to back on cold tensors (see isolated_layer_us): what the fractions below use
        us = isolated_layer_us(L, 64)
        xb, yb = 4 * 64 * L["cin"] * L["hw"] ** 2, 4 * 64 * L["cout"] * L["ohw"] ** 2
        wb = 4 * L["cout"] * (L["cin"] // L["groups"]) * L["kernel"] ** 2
        flops = 2.0 * 64 * L["cout"] * L["ohw"] ** 2 * (L["cin"] // L["groups"]) * L["kernel"] ** 2
        e["us"] = round(us, 2)
        e["gbs"] = round((xb + yb + wb) / us / 1e3, 1)
        e["tflops"] = round(flops / us / 1e6, 2)
        if L["algo"] == "depthwise_separable":
            # bandwidth-bound: against the vendor's 8 TB/s, and against a plain streaming kernel that reads |X| and
            # writes |Y| of this very layer, timed the same way
            forms, best = probe.stream_forms(xb, yb)
            cus = forms[best]
            e["bound"] = "hbm"
            e["frac_of_hbm_peak"] = round(e["gbs"] / HBM_PEAK_GBS, 4)
            e["tuned_copy_us"] = round(cus, 2)
            e["tuned_copy_gbs"] = round((xb + yb) / cus / 1e3, 1)
            e["tuned_copy_form"] = best
            e["frac_of_tuned_copy"] = round(cus / us, 4)
            if xb + yb < 100e6:  # small tensors: also with x and y still in the last-level cache, as behind a producer
                e["us_tensors_in_last_level_cache"] = round(isolated_layer_us(L, 64, cached=True), 2)
        else:
            ai = flops / (xb + yb + wb)
            roof = min(FP32_MATRIX_PEAK_TFLOPS * 1e12, ai * HBM_PEAK_GBS * 1e9)
            e["bound"] = "mfma" if ai * HBM_PEAK_GBS * 1e9 >= FP32_MATRIX_PEAK_TFLOPS * 1e12 else "hbm"
            e["frac_of_roofline"] = round(flops / (us * 1e-6) / roof, 4)
            # what a launch of this size costs at the least on this chip: the tuned streaming kernel over the same |X| and |Y|
            gbs, cus = probe.copy_at_size(xb, yb)
            e["roofline_us"] = round(flops / roof * 1e6, 2)
            e["tuned_copy_us"] = round(cus, 2)
        rows.append(e)
    dw = [e for e in rows if "frac_of_hbm_peak" in e]
    pw = [e for e in rows if "frac_of_hbm_peak" not in e]
    # depthwise + pointwise pairs as one launch (the tensor between them never reaches memory): algorithmic bytes are
    # |x of the depthwise layer| + |y of the pointwise layer| + both filters; scored like the depthwise layers
    pairs = []
    LL = r["layer_list"]
    for (i, j) in mobilenet_pairs(LL):
        D, P = LL[i], LL[j]
        e = {"name": "%s+%s" % (D["name"], P["name"]), "separate_us": round(rows[i]["us"] + rows[j]["us"], 2)}
        if fused_pair_op(D, P, 64) is None:
            e["fused"] = False  # the library keeps this pair as two operators (faster there)
        else:
            us = isolated_fused_us(D, P, 64)
            xb, yb = 4 * 64 * D["cin"] * D["hw"] ** 2, 4 * 64 * P["cout"] * P["ohw"] ** 2
            wb = 4 * (D["cout"] * 9 + P["cout"] * P["cin"])
            gbs, cus = probe.copy_at_size(xb, yb)
            e.update({"fused": True, "kernel": "conv_dwpw_f32_kernel", "us": round(us, 2), "speedup": round(e["separate_us"] / us, 3), "bound": "hbm",
                      "gbs": round((xb + yb + wb) / us / 1e3, 1), "frac_of_hbm_peak": round((xb + yb + wb) / us / 1e3 / HBM_PEAK_GBS, 4),
                      "tuned_copy_us": round(cus, 2), "frac_of_tuned_copy": round(cus / us, 4)})
        pairs.append(e)
    fused_ms, nfused = mobilenet_fused_pass_ms(64, max(steps, 100), warmup)
    cfgs["config4_mobilenet_blocks_b64"] = compact(r, 64, {
        "depthwise_min_frac_of_hbm_peak": min(e["frac_of_hbm_peak"] for e in dw), "depthwise_min_frac_of_tuned_copy": min(e["frac_of_tuned_copy"] for e in dw),
        "pointwise_min_frac_of_roofline": min(e["frac_of_roofline"] for e in pw), "layers": rows,
        "ms_per_step_with_fused_pairs": round(fused_ms, 4), "fused_pairs_in_step": nfused, "fused_pairs": pairs})
    if with_cpu:  # all 16 layers, 16 of the 64 images, one thread
        cfgs["config4_mobilenet_blocks_b64"]["cpu_baseline"] = cpu_baseline(r["layer_list"], 16, 2024)
    del r
    torch.cuda.empty_cache()
    # an inference deployment, as dlprim::Net runs the same network: the residual sums run in the epilogue of the 1x1 convolution
    # that produces their later branch and the filters are transformed once (--workload resnet50-full --fuse-residual
    # --prepacked; without the flags the sums are operators of their own and every enqueue transforms its filter)
    # and the tensors between convolutions are kept channels-last where that is faster (the input, the logits and the parameters keep the
    # reference's layout); the same deployment on NCHW tensors throughout is timed next to it
    nchw = graph_workload("resnet50", 128, "gemm", True, max(3, steps // 2), max(2, warmup // 2), fuse_residual=True, prepack=True)
    torch.cuda.empty_cache()
    cfgs["config5_resnet50_full_bf16_b128"] = graph_workload("resnet50", 128, "gemm", True, max(3, steps // 2), max(2, warmup // 2), fuse_residual=True, prepack=True,
                                                             channels_last=True, fuse_stem_pool=True)
    cfgs["config5_resnet50_full_bf16_b128"]["nchw_between_layers"] = {"ms_per_step": nchw["ms_per_step"], "images_per_s": nchw["value"],
                                                                       "roofline_frac": nchw["roofline"]["frac"]}
    if with_cpu:
        # the fp32 reference path on the 53 convolutions of the network (99 % of its arithmetic), 16 of the 128 images
        # spread over the host cores the box gives a GPU
        from dlprimitives_amd.workloads import RESNET50_CONVS

        nthreads = max(1, min(16, os.cpu_count() or 1))
        cfgs["config5_resnet50_full_bf16_b128"]["cpu_baseline"] = cpu_baseline(RESNET50_CONVS, nthreads, 2024, threads=nthreads, runs=3)
    # HBM bytes per launch of the kernel with the largest share of the pass (from the tracked counter summary)
    cfgs["config5_resnet50_full_bf16_b128"]["roofline"]["traffic"] = measured_traffic_bytes("resnet50-bf16", cfgs["config5_resnet50_full_bf16_b128"].get("dominant_kernel", ""))
    return cfgs


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30,
                    help="untimed steps before the timed ones (the first ~50 steps of a process run 3-4 %% slower than the steady state)")
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--workload", default="resnet18", choices=["resnet18", "resnet50", "mobilenet", "mobilenet-fused", "winograd", "winograd-gemm", "single",
                                                                 "resnet18-full", "resnet50-full", "resnet18-backward"])
    ap.add_argument("--algo", default="gemm", help="conv algorithm of the -full workloads ('' = auto)")
    ap.add_argument("--dtype", default="f32", choices=["f32", "bf16"], help="storage type of the tensors (accumulation and epilogue are fp32 either way)")
    ap.add_argument("--cpu-images", type=int, default=8, help="images of the CPU baseline sample (0 = skip)")
    ap.add_argument("--layers", action="store_true", help="also print the per-layer table to stderr")
    ap.add_argument("--channels-last", action="store_true",
                    help="*-full workloads in bf16: tensors between convolutions are kept channels-last where the planner finds it faster")
    ap.add_argument("--fuse-stem-pool", action="store_true",
                    help="*-full workloads in bf16: the 3x3 stride-2 max pooling behind the 7x7 stem runs inside the stem's kernel (dlp_conv2d_fwd_fuse_max_pool)")
    ap.add_argument("--prepacked", action="store_true",
                    help="weights transformed once before the timed region (dlp_conv2d_fwd_pack / _enqueue_packed), as an inference "
                         "deployment does; the default transforms them in every step, as the reference's enqueue contract implies")
    ap.add_argument("--fuse-residual", action="store_true",
                    help="-full workloads: residual sums behind a 1x1 convolution run in that convolution's epilogue (dlp_conv2d_fwd_set_accumulate_first)")
    ap.add_argument("--only", default="", help="profiling aid: keep only layers whose name contains this text")
    ap.add_argument("--no-configs", action="store_true", help="default workload only: leave out the `configs` object (the other four configurations)")
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
        print(json.dumps(run_graph_workload(args)))
        return
    if args.workload == "resnet18-backward":
        run_backward_workload(args)
        return
    if args.workload == "mobilenet-fused":
        # the mobilenet workload with the depthwise -> pointwise pairs that the library fuses run as one launch each
        ms, nfused = mobilenet_fused_pass_ms(args.batch, args.steps, args.warmup)
        print(json.dumps({"metric": BASELINE_METRIC, "value": round(args.batch / (ms * 1e-3), 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
                          "warmup": args.warmup, "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32",
                          "data": "synthetic", "config": {"workload": "MobileNet-v2 style blocks, batch %d, %d depthwise + pointwise pairs as one launch each" %
                                                          (args.batch, nfused), "batch": args.batch}}))
        return
    bf16 = args.dtype == "bf16"
    r = run_conv_workload(args.workload, args.batch, bf16, args.steps, args.warmup, args.prepacked, args.only)
    ms_per_step = r["ms_per_step"]
    if args.layers:
        for row in r["table"]:
            print(json.dumps(row), file=sys.stderr)
    headline = args.workload == "resnet18" and args.batch == 64 and not bf16 and not args.only

    cpu = cpu_baseline(r["layer_list"], args.cpu_images, 2024) if args.cpu_images > 0 else None  # the fp32 reference path
    # the same arithmetic with the batch spread over the host's cores (what a reference build with a threaded BLAS
    # would approach); the box gives a GPU 16 cores whatever os.cpu_count() says
    cpu_mt = None
    if args.cpu_images > 0:
        nthreads = max(1, min(16, os.cpu_count() or 1))
        cpu_mt = cpu_baseline(r["layer_list"], max(args.cpu_images, 2 * nthreads), 2024, threads=nthreads)

    # what this chip reaches with no convolution around it (MFMA-only loops, streaming copies), next to the vendor peaks
    from dlprimitives_amd import probe

    peaks = probe.measured_peaks()
    rf = r["roofline"]
    measured = peaks["mfma_bf16_tflops" if rf["peak"] == BF16_MATRIX_PEAK_TFLOPS else "mfma_f32_tflops"] if rf["bound"] == "mfma" else peaks["copy_2048mib_gbs"]
    rf["measured_peak"] = measured
    rf["frac_of_measured_peak"] = round(rf["achieved"] / measured, 4)

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
        "config": {"workload": "%s%s, %s NCHW, batch %d" % (r["description"], " (subset --only %s)" % args.only if args.only else "",
                                                            "bf16" if bf16 else "fp32", args.batch) +
                               (", weights packed once before the timed region" if args.prepacked else ""),
                   "batch": args.batch, "layers": r["nl"], "gflop_per_step": round(r["total_flops"] / 1e9, 1),
                   "mbytes_per_step": round(r["total_bytes"] / 1e6, 1)},
        "gflops_per_s": round(r["total_flops"] / (ms_per_step * 1e-3) / 1e9, 1),
        "frac_of_fp32_matrix_peak": round(r["total_flops"] / (ms_per_step * 1e-3) / 1e12 / FP32_MATRIX_PEAK_TFLOPS, 4),
        "kernel_ms_per_step": round(r["kernel_ms_per_step"], 4),
        "roofline": rf,
        "cpu_baseline": cpu,
        "cpu_baseline_all_cores": cpu_mt,
        "vendor_peak": {"fp32_matrix_tflops": FP32_MATRIX_PEAK_TFLOPS, "bf16_matrix_tflops": BF16_MATRIX_PEAK_TFLOPS, "hbm_gbs": HBM_PEAK_GBS},
        "measured_peak": peaks,
        "layers": r["table"],
    }
    if headline and not args.no_configs:
        del r
        torch.cuda.empty_cache()
        out["configs"] = other_configs(max(5, args.steps // 2), max(2, args.warmup // 2), peaks, with_cpu=args.cpu_images > 0)
        out["configs"]["config2_resnet18_conv_stack_b64"] = "the headline of this line: value, ms_per_step, roofline, layers"
    print(json.dumps(out))


if __name__ == "__main__":
    main()
