"""Device peak probes: fp32 / bf16 MFMA throughput (no memory traffic) and streaming bandwidth, from libdlp_microbench.so.
They put the roofline fractions of the convolution kernels in context (nominal peaks: 157.3 TFLOP/s fp32 matrix, 2.5 PFLOP/s
bf16 matrix, 8 TB/s HBM) and give the hardware-counter runs a copy kernel of known size to be scaled by.

The streaming probe times several forms of a copy / read / write kernel (one 16-byte piece per thread, several pieces with
non-temporal accesses, 1024-thread workgroups, the untuned grid-stride loop, hipMemcpyAsync) on tensors of a given size, every
launch cold (a ring of buffers larger than the last-level cache), and reports the fastest kernel form: the "tuned copy".

    python -m dlprimitives_amd.probe [--copy-mb 256] [--no-mfma]
    python -m dlprimitives_amd.probe --tile-step
"""
import argparse
import ctypes
import json
import os


def _lib():
    lib = ctypes.CDLL(os.path.join(os.path.dirname(os.path.abspath(__file__)), "libdlp_microbench.so"))
    lib.dlp_probe_stream_forms.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_int)]
    lib.dlp_probe_stream_form_name.restype = ctypes.c_char_p
    return lib


def stream_forms(in_bytes, out_bytes):
    """{form name: microseconds per launch} of every streaming form that reads in_bytes and writes out_bytes, and the name of the
    fastest kernel form"""
    lib = _lib()
    n = lib.dlp_probe_stream_form_count()
    us = (ctypes.c_double * n)()
    best = ctypes.c_int(-1)
    if lib.dlp_probe_stream_forms(int(in_bytes), int(out_bytes), us, ctypes.byref(best)) != 0:
        raise RuntimeError("streaming probe failed")
    names = [lib.dlp_probe_stream_form_name(i).decode() for i in range(n)]
    return {names[i]: us[i] for i in range(n) if us[i] > 0}, names[best.value]


def copy_at_size(in_bytes, out_bytes):
    """(GB/s, microseconds per launch) of the tuned copy: the fastest streaming kernel form that reads in_bytes and writes
    out_bytes, launches back to back on cold tensors"""
    forms, best = stream_forms(in_bytes, out_bytes)
    us = forms[best]
    return (in_bytes + out_bytes) / us / 1e3, us


def tile_steps():
    """What LDS and the matrix pipe sustain together on one K step of a 128 x 128 x 32 bf16 tile in a four-wavefront workgroup, piece by
    piece (tile_step_kernel of csrc/microbench.hip): {form: {workgroups per CU: {"ns_per_step", "clocks_at_2.4GHz", "tflops"}}}, and the LDS
    rates that follow from the reads-only and stores-only forms."""
    lib = _lib()
    lib.dlp_probe_tile_step_name.restype = ctypes.c_char_p
    v = ctypes.c_double()
    out = {}
    for f in range(lib.dlp_probe_tile_step_count()):
        name = lib.dlp_probe_tile_step_name(f).decode()
        out[name] = {}
        for w in (1, 2, 3):
            if lib.dlp_probe_tile_step(f, w, ctypes.byref(v)) != 0:
                raise RuntimeError("tile step probe failed")
            ns = v.value
            row = {"ns_per_step": round(ns, 1), "clocks_at_2.4GHz": round(ns * 2.4)}
            if "alone" not in name:
                row["tflops"] = round(2.0 * 128 * 128 * 32 * 256 * w / (ns * 1e-9) / 1e12)
            out[name]["%d per CU" % w] = row
    rd = out["LDS reads + barrier alone (32 KB per step)"]["3 per CU"]["clocks_at_2.4GHz"] / 3.0
    wr = out["LDS stores + barrier alone (16 KB per step)"]["3 per CU"]["clocks_at_2.4GHz"] / 3.0
    out["lds_bytes_per_clock_and_cu"] = {"ds_read_b128": round(32768 / rd), "ds_write_b128": round(16384 / wr)}
    return out


def measured_peaks(big_mb=2048):
    """MFMA-only loops and streaming kernels on this device: what the chip reaches with no convolution around it."""
    lib = _lib()
    v = ctypes.c_double()
    out = {}
    for name, fn in (("mfma_f32_tflops", lib.dlp_probe_mfma_f32), ("mfma_bf16_tflops", lib.dlp_probe_mfma_bf16)):
        best = 0.0
        for waves in (1, 2):
            if fn(waves, ctypes.byref(v)) != 0:
                raise RuntimeError(name + " probe failed")
            best = max(best, v.value)
        out[name] = round(best, 1)
    for mb in (256, big_mb):
        if not mb:
            continue
        b = mb << 20
        gbs, _ = copy_at_size(b, b)
        out["copy_%dmib_gbs" % mb] = round(gbs, 1)
    b = (big_mb or 256) << 20
    out["read_%dmib_gbs" % (b >> 20)] = round(copy_at_size(b, 0)[0], 1)
    out["write_%dmib_gbs" % (b >> 20)] = round(copy_at_size(0, b)[0], 1)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--copy-mb", type=int, default=256, help="MiB per direction of the copy kernels")
    ap.add_argument("--no-mfma", action="store_true")
    ap.add_argument("--tile-step", action="store_true", help="only the K-step probe of a bf16 tile (LDS reads, LDS stores, matrix instructions together)")
    args = ap.parse_args()
    if args.tile_step:
        print(json.dumps(tile_steps(), indent=1))
        return
    lib = _lib()
    out = {}
    v = ctypes.c_double()
    if not args.no_mfma:
        for waves in (1, 2):
            if lib.dlp_probe_mfma_f32(waves, ctypes.byref(v)) != 0:
                raise SystemExit("MFMA probe failed")
            out["mfma_f32_tflops_%dwave_per_simd" % waves] = round(v.value, 1)
        for waves in (1, 2):
            if lib.dlp_probe_mfma_bf16(waves, ctypes.byref(v)) != 0:
                raise SystemExit("bf16 MFMA probe failed")
            out["mfma_bf16_tflops_%dwave_per_simd" % waves] = round(v.value, 1)
    b = args.copy_mb << 20

    def table(i, o):
        forms, best = stream_forms(i, o)
        return {"gbs": {k: round((i + o) / us / 1e3, 1) for k, us in forms.items()}, "best": best}

    out["copy_%dmib" % args.copy_mb] = table(b, b)
    if not args.no_mfma:
        big = 2048 << 20  # tensors far above the 256 MB last-level cache: what HBM itself sustains
        out["copy_2048mib"] = table(big, big)
        out["read_2048mib"] = table(big, 0)
        out["write_2048mib"] = table(0, big)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
