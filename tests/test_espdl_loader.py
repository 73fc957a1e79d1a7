"""Native `.espdl` loader: parses the reference-held fixtures, re-lays blocked filters to N-major, and
refuses damaged files without crashing.  The independent check is tests/golden/espdl_reader.py (a
separate Python walker) plus the fact that the three targets of one fixture hold the same weights."""
import glob
import importlib
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "espdl", "*.espdl")))


def _model_mod():
    return importlib.import_module("esp-dl_amd").model


def _py_reader():
    import sys
    sys.path.insert(0, os.path.join(HERE, "golden"))
    import espdl_reader
    return espdl_reader


def _n_major(t):
    """Python restatement of the blocked layout -> [N][spatial][C] (dims are [spatial..., C, N])."""
    dims, data, doc = t["dims"], t["data"].ravel(), t["doc"] or ""
    if "16" not in doc:
        return data
    n, c = dims[-1], dims[-2]
    sp = int(np.prod(dims[:-2]))
    nb, tail = n // 16, n % 16
    out = np.zeros((n, sp, c), dtype=data.dtype)
    out[:nb * 16] = data[:nb * 16 * sp * c].reshape(nb, sp, c, 16).transpose(0, 3, 1, 2).reshape(nb * 16, sp, c)
    if tail:
        out[nb * 16:] = data[nb * 16 * sp * c:].reshape(sp, c, tail).transpose(2, 0, 1)
    return out.ravel()


def test_fixtures_are_present():
    assert len(FIXTURES) == 11


@pytest.mark.parametrize("path", FIXTURES, ids=os.path.basename)
def test_loader_matches_python_reader(path):
    ref = _py_reader().read_espdl(path)
    g = _model_mod().Graph.from_file(path)
    assert g.input_names() == [v["name"] for v in ref["inputs"]]
    assert g.output_names() == [v["name"] for v in ref["outputs"]]
    np_of = {3: np.int8, 5: np.int16, 6: np.int32, 7: np.int64, 1: np.float32}
    for name, t in ref["initializers"].items():
        got = g.initializer(name, np_of[t["dtype"]])
        np.testing.assert_array_equal(got, _n_major(t), err_msg=name)


def test_blocked_and_plain_targets_hold_the_same_filters():
    """The c target stores [N][K]; the S3 / P4 files of the same test store (N/16)HWC16.  After loading,
    all three are byte-identical, which pins the block re-layout on real exporter output."""
    base = os.path.join(HERE, "golden", "espdl")
    for shape in ("1_16_kshap_16_16", "1_31_kshap_32_31", "1_64_kshap_32_64"):
        graphs = [_model_mod().Graph.from_file(os.path.join(base, f"gemm_{t}_linear_ishap_{shape}_relu_s8.espdl"))
                  for t in ("c", "esp32s3", "esp32p4")]
        ref = _py_reader().read_espdl(os.path.join(base, f"gemm_c_linear_ishap_{shape}_relu_s8.espdl"))
        wname = [n for n, t in ref["initializers"].items() if t["dtype"] == 3][0]
        w = [g.initializer(wname) for g in graphs]
        np.testing.assert_array_equal(w[0], w[1])
        np.testing.assert_array_equal(w[0], w[2])


def test_damaged_files_are_refused_not_crashed_on():
    model = _model_mod()
    blob = open(FIXTURES[3], "rb").read()
    with pytest.raises(model.EspdlModelError):
        model.Graph.from_bytes(b"XXXX" + blob[4:])
    with pytest.raises(model.EspdlModelError):
        model.Graph.from_bytes(blob[:4] + (1).to_bytes(4, "little") + blob[8:])  # encrypted flag
    refused = 0
    for cut in range(8, len(blob), 97):  # truncations: every load either fails cleanly or yields a graph
        try:
            model.Graph.from_bytes(blob[:cut])
        except model.EspdlModelError:
            refused += 1
    assert refused > 10
    rng = np.random.default_rng(3)
    for _ in range(200):  # random byte damage inside the payload
        b = bytearray(blob)
        for pos in rng.integers(16, len(b), size=8):
            b[pos] = int(rng.integers(0, 256))
        try:
            model.Graph.from_bytes(bytes(b))
        except model.EspdlModelError:
            pass


def test_missing_file():
    with pytest.raises(_model_mod().EspdlModelError):
        _model_mod().Graph.from_file("/nonexistent/model.espdl")
