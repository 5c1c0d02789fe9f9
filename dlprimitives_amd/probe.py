"""Device peak probes: fp32 MFMA throughput (no memory traffic) and streaming-copy
bandwidth, from libdlp_microbench.so.  They put the roofline fractions of the
convolution kernels in context (nominal peaks: 157.3 TFLOP/s fp32 matrix, 8 TB/s HBM)
and give the hardware-counter runs a copy kernel of known size to be scaled by.

    python -m dlprimitives_amd.probe [--copy-mb 256] [--no-mfma]
"""
import argparse
import ctypes
import json
import os


def _lib():
    return ctypes.CDLL(os.path.join(os.path.dirname(os.path.abspath(__file__)), "libdlp_microbench.so"))


def measured_peaks(big_mb=2048):
    """MFMA-only loops and streaming copies on this device: what the chip reaches with no convolution around it."""
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
    if lib.dlp_probe_copy(256, ctypes.byref(v)) != 0:
        raise RuntimeError("copy probe failed")
    out["copy_256mib_gbs"] = round(v.value, 1)
    if big_mb and lib.dlp_probe_copy(big_mb, ctypes.byref(v)) == 0:
        out["copy_%dmib_gbs" % big_mb] = round(v.value, 1)
    return out


def copy_at_size(in_bytes, out_bytes):
    """(GB/s, microseconds per launch) of a plain streaming kernel that reads in_bytes and writes out_bytes, every launch
    timed by its own event pair and starting cold (a ring of buffers larger than the last-level cache)."""
    lib = _lib()
    lib.dlp_probe_copy_sized.argtypes = [ctypes.c_size_t, ctypes.c_size_t, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    gbs, us = ctypes.c_double(), ctypes.c_double()
    if lib.dlp_probe_copy_sized(int(in_bytes), int(out_bytes), ctypes.byref(gbs), ctypes.byref(us)) != 0:
        raise RuntimeError("sized copy probe failed")
    return gbs.value, us.value


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--copy-mb", type=int, default=256, help="MiB per direction of the copy kernel")
    ap.add_argument("--no-mfma", action="store_true")
    args = ap.parse_args()
    lib = ctypes.CDLL(os.path.join(os.path.dirname(os.path.abspath(__file__)), "libdlp_microbench.so"))
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
    if lib.dlp_probe_copy(args.copy_mb, ctypes.byref(v)) != 0:
        raise SystemExit("copy probe failed")
    out["copy_gbs_read_plus_write"] = round(v.value, 1)
    out["copy_bytes_per_launch_each_direction"] = args.copy_mb << 20
    if not args.no_mfma:
        # tensors far above the 256 MB last-level cache: what HBM itself sustains
        big = 2048
        if lib.dlp_probe_copy(big, ctypes.byref(v)) == 0:
            out["copy_gbs_%dmb" % big] = round(v.value, 1)
        if lib.dlp_probe_stream(big, 0, ctypes.byref(v)) == 0:
            out["read_gbs_%dmb" % big] = round(v.value, 1)
        if lib.dlp_probe_stream(big, 1, ctypes.byref(v)) == 0:
            out["write_gbs_%dmb" % big] = round(v.value, 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
