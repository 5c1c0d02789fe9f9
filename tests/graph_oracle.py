"""CPU execution of a dlprimitives_amd.graphs graph with the oracle operators (test side only)."""
import numpy as np


def run_graph_on_oracle(orc, ops, params, x, keep=False):
    t = {"data": np.ascontiguousarray(x, dtype=np.float32)}
    for o in ops:
        if o["op"] == "conv":
            w, b = params[o["dst"]]
            cfg = orc.make_cfg(o["cin"], o["cout"], o["k"], o["s"], 1, o["p"], 1)
            t[o["dst"]] = orc.conv2d_forward(t[o["src"]], w, b, cfg, o["act"], threads=8)
        elif o["op"] == "maxpool":
            t[o["dst"]] = orc.pool2d_forward(t[o["src"]], o["k"], o["p"], o["s"], "max")
        elif o["op"] == "add":
            t[o["dst"]] = orc.eltwise_forward(t[o["src"][0]], t[o["src"][1]], "sum", 1.0, 1.0, o["act"])
        elif o["op"] == "gap":
            t[o["dst"]] = orc.global_pool_forward(t[o["src"]], "avg")
        elif o["op"] == "ip":
            w, b = params[o["dst"]]
            t[o["dst"]] = orc.ip_forward(t[o["src"]], w, b, "identity")
    return t if keep else t[ops[-1]["dst"]]
