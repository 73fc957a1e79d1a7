"""Extract the reference-held `c`-target Gemm known-answer vectors into gemm_c_fixtures.json.

Source (data files, read only in the build container):
  /root/reference/test_apps/esp-dl/models/c/Gemm/*.espdl
Each file holds one Gemm node, its int8 weight (declared shape [1,1,K,N]; bytes as stored),
int32 bias, per-tensor exponents, and the embedded test_inputs_value / test_outputs_value that
the reference's `Model::test()` compares bit-for-bit (esp-dl/dl/model/src/dl_model_base.cpp:442-519).

Run:  python tests/golden/make_gemm_fixtures.py
"""
import glob
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from espdl_reader import read_espdl  # noqa: E402

SRC = "/root/reference/test_apps/esp-dl/models/c/Gemm"


def main():
    cases = []
    for path in sorted(glob.glob(os.path.join(SRC, "*.espdl"))):
        m = read_espdl(path)
        assert m["meta"].get("target") == "c", path
        (node,) = m["nodes"]
        assert node["op_type"] == "Gemm"
        x_name, w_name, b_name = node["input"]
        (y_name,) = node["output"]
        w = m["initializers"][w_name]
        b = m["initializers"][b_name]
        x = m["test_inputs"][x_name]
        y = m["test_outputs"][y_name]
        cases.append({
            "file": os.path.relpath(path, "/root/reference"),
            "activation": node["attrs"]["activation"],
            "input_shape": x["dims"], "input_exponent": x["exponents"][0],
            "input": x["data"].ravel().tolist(),
            "filter_shape": w["dims"], "filter_exponents": w["exponents"],
            "filter_bytes": w["data"].ravel().tolist(),
            "bias_exponents": b["exponents"], "bias": b["data"].ravel().tolist(),
            "output_shape": y["dims"], "output_exponent": y["exponents"][0],
            "output": y["data"].ravel().tolist(),
        })
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gemm_c_fixtures.json")
    with open(out, "w") as f:
        json.dump(cases, f, separators=(",", ":"))
        f.write("\n")
    print(f"wrote {len(cases)} cases to {out}")


if __name__ == "__main__":
    main()
