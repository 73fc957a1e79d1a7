"""Turns an `.espdl` file (through the independent Python walker in tests/golden/espdl_reader.py) into a
zoo.GraphSpec, so that the CPU oracle's graph runner can execute exactly what the native loader hands to
dl::Model.  Test infrastructure."""
import importlib
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import espdl_reader  # noqa: E402


def _n_major(t, depthwise=False):
    """Blocked S3 / P4 filter order -> [N][spatial][C]; dims are [spatial..., C, N].  A depthwise filter
    ([spatial..., C, 1]) is blocked over its C filters of one input channel each."""
    dims, data, doc = list(t["dims"]), t["data"].ravel(), t["doc"] or ""
    block = 16 if "C16" in doc else (8 if "C8" in doc else 0)
    if not block:
        return data
    n, c = (dims[-2] * dims[-1], 1) if depthwise else (dims[-1], dims[-2])
    sp = int(np.prod(dims[:-2]))
    nb, tail = n // block, n % block
    out = np.zeros((n, sp, c), dtype=data.dtype)
    out[:nb * block] = data[:nb * block * sp * c].reshape(nb, sp, c, block).transpose(0, 3, 1, 2).reshape(-1, sp, c)
    if tail:
        out[nb * block:] = data[nb * block * sp * c:].reshape(tail, sp, c)  # remainder: plain filter-major
    if depthwise:  # [C][spatial][1] -> the c target's [spatial][C]
        out = out.reshape(n, sp).T
    return np.ascontiguousarray(out).ravel()


def spec_from_espdl(path):
    zoo = importlib.import_module("esp-dl_amd").zoo
    m = espdl_reader.read_espdl(path)
    g = zoo.GraphSpec(os.path.basename(path))
    depthwise = {n["input"][1] for n in m["nodes"]
                 if n["op_type"] == "Conv" and n["attrs"].get("group", 1) != 1 and len(n["input"]) > 1}
    for name, t in m["initializers"].items():
        if t["data"] is None:
            continue
        g.initializers[name] = (list(t["dims"]), t["dtype"], _n_major(t, name in depthwise),
                                [int(e) for e in t["exponents"]])
    for v in m["inputs"] + m["outputs"] + m["value_info"]:
        g.value_info[v["name"]] = (list(v["dims"]), v["dtype"] or zoo.INT8, int(v["exponents"][0]) if v["exponents"] else 0)
    g.inputs = [v["name"] for v in m["inputs"]]
    g.outputs = [v["name"] for v in m["outputs"]]
    for n in m["nodes"]:
        g.nodes.append({"name": n["name"], "op_type": n["op_type"], "inputs": list(n["input"]),
                        "outputs": list(n["output"]), "attrs": dict(n["attrs"])})
    return g, m
