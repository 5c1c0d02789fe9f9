"""Extract the forward golden vectors the reference's own tests hold for this path.

Reads DATA files only (JSON written by the reference's PyTorch fixture generator):
  tests/test_case_inner_product.json  -> inner_product_fwd.json
  tests/test_case_activation.json     -> activation_fwd.json
  tests/test_case_pooling2d.json      -> pooling2d_fwd.json
  tests/test_case_global_pooling.json -> global_pooling_fwd.json
  tests/test_case_softmax.json        -> softmax_fwd.json       (cases of up to 1100 values)
  tests/test_case_log_softmax.json    -> log_softmax_fwd.json   (likewise)
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
