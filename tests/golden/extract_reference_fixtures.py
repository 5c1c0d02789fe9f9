"""Extract the forward golden vectors the reference's own tests hold for this path.

Reads DATA files only (JSON written by the reference's PyTorch fixture generator):
  tests/test_case_inner_product.json  -> inner_product_fwd.json
  tests/test_case_activation.json     -> activation_fwd.json
  tests/test_case_pooling2d.json      -> pooling2d_fwd.json
  tests/test_case_global_pooling.json -> global_pooling_fwd.json
  tests/test_case_softmax.json        -> softmax_fwd.json       (cases of up to 1100 values)
  tests/test_case_log_softmax.json    -> log_softmax_fwd.json   (likewise)
  tests/test_case_interpolation.json  -> interpolation_fwd.json (cases of up to 200 values)
  tests/test_case_reduction.json      -> reduction_fwd.json     (cases of up to 800 values)
  tests/test_case_mse_loss.json, test_case_nll_loss.json, test_case_softmax_loss.json
                                      -> mse_loss_fwd.json, nll_loss_fwd.json, softmax_loss_fwd.json (up to 2000, 400, 1000 values)
  tests/test_case_abs.json, test_case_hardtanh.json, test_case_threshold.json, test_case_concat.json, test_case_slice.json
                                      -> abs_fwd.json, hardtanh_fwd.json, threshold_fwd.json, concat_fwd.json, slice_fwd.json
keeping options, parameters, inputs and expected forward outputs (gradients are
dropped: the path is forward only).  Run in the build container, where the
reference tree is mounted:  python tests/golden/extract_reference_fixtures.py
"""
import json
import os
import sys

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
HERE = os.path.dirname(os.path.abspath(__file__))


def extract(src, dst, max_values=None):
    with open(os.path.join(REF, "tests", src)) as f:
        doc = json.load(f)
    out = {"operator": doc["operator"], "source": "tests/" + src, "tests": []}
    for t in doc["tests"]:
        rec = {
            "options": t["options"],
            "setup_shapes": [s["shape"] for s in t["setup_tensors"]],
            "output_shapes": [s["shape"] for s in t["output_tensors"]],
            "param_shapes": [s["shape"] for s in t.get("param_specs", [])],
            "params": t.get("param_tensors", []),
            # cases without tensors are the reference's "compare with the CPU
            # operator on random inputs" cases: only their shapes are data
            "cases": [
                {
                    "in_shapes": c["in_shapes"],
                    "out_shapes": c["out_shapes"],
                    **({"in": c["in_tensors"], "out": c["out_tensors"]} if "in_tensors" in c else {"use_cpu_reference": True}),
                }
                for c in t["cases"]
                if max_values is None or all(len(v) <= max_values for v in c.get("in_tensors", []))
            ],
        }
        out["tests"].append(rec)
    with open(os.path.join(HERE, dst), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print(dst, len(out["tests"]), "tests", sum(len(t["cases"]) for t in out["tests"]), "cases")


if __name__ == "__main__":
    extract("test_case_inner_product.json", "inner_product_fwd.json")
    extract("test_case_activation.json", "activation_fwd.json")
    extract("test_case_pooling2d.json", "pooling2d_fwd.json")
    extract("test_case_global_pooling.json", "global_pooling_fwd.json")
    extract("test_case_softmax.json", "softmax_fwd.json", 1100)
    extract("test_case_log_softmax.json", "log_softmax_fwd.json", 1100)
    extract("test_case_interpolation.json", "interpolation_fwd.json", 200)
    extract("test_case_reduction.json", "reduction_fwd.json", 800)
    extract("test_case_mse_loss.json", "mse_loss_fwd.json", 2000)
    extract("test_case_nll_loss.json", "nll_loss_fwd.json", 400)
    extract("test_case_softmax_loss.json", "softmax_loss_fwd.json", 1000)
    for name in ("abs", "hardtanh", "threshold", "concat", "slice"):
        extract("test_case_%s.json" % name, name + "_fwd.json", 2000)
