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
