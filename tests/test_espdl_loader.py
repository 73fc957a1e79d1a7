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


def _spec(path):
    import sys
    sys.path.insert(0, HERE)
    import espdl_spec
    return espdl_spec.spec_from_espdl(path)[0]


def test_fixtures_are_present():
    assert len(FIXTURES) == 15


@pytest.mark.parametrize("path", FIXTURES, ids=os.path.basename)
def test_loader_matches_python_reader(path):
    ref = _py_reader().read_espdl(path)
    g = _model_mod().Graph.from_file(path)
    assert g.input_names() == [v["name"] for v in ref["inputs"]]
    assert g.output_names() == [v["name"] for v in ref["outputs"]]
    np_of = {3: np.int8, 5: np.int16, 6: np.int32, 7: np.int64, 1: np.float32}
    for name, (dims, dtype, data, _) in _spec(path).initializers.items():
        np.testing.assert_array_equal(g.initializer(name, np_of[dtype]), np.asarray(data).ravel(), err_msg=name)


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
    blob = open([f for f in FIXTURES if "gemm_chain_s3" in f][0], "rb").read()
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


REF = "/root/reference"
ZOO = [
    "models/imagenet_cls/models/p4/imagenet_cls_mobilenetv2_s8_v1.espdl",
    "models/imagenet_cls/models/s3/imagenet_cls_mobilenetv2_s8_v1.espdl",
    "models/human_face_detect/models/s3/human_face_detect_msr_s8_v1.espdl",
    "models/hand_gesture_recognition/models/p4/mobilenetv2_0_5_128_128_gesture.espdl",
]
needs_reference = pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not on this machine")


@needs_reference
@pytest.mark.parametrize("rel", ZOO, ids=os.path.basename)
def test_zoo_model_filters_match_python_relayout(rel):
    """Shipped models exercise what the Gemm fixtures do not: depthwise filters, filter counts that are
    not multiples of 16, 3x3 kernels.  The native loader and the Python walker must agree byte for byte."""
    sys_path_tests = os.path.dirname(os.path.abspath(__file__))
    import sys
    sys.path.insert(0, sys_path_tests)
    import espdl_spec
    path = os.path.join(REF, rel)
    spec, _ = espdl_spec.spec_from_espdl(path)
    g = _model_mod().Graph.from_file(path)
    np_of = {3: np.int8, 5: np.int16, 6: np.int32, 7: np.int64, 1: np.float32}
    checked = 0
    for name, (dims, dtype, data, _) in spec.initializers.items():
        np.testing.assert_array_equal(g.initializer(name, np_of[dtype]), np.asarray(data).ravel(), err_msg=name)
        checked += 1
    assert checked > 10
    assert all(_model_mod().is_registered(op) for op in g.op_types())


@needs_reference
def test_every_reference_espdl_file_loads():
    files = sorted(glob.glob(os.path.join(REF, "**", "*.espdl"), recursive=True))
    assert len(files) > 50
    for f in files:
        g = _model_mod().Graph.from_file(f)
        assert len(g.op_types()) > 0 and g.input_names() and g.output_names(), f


@needs_reference
@pytest.mark.parametrize("target,round_mode", [("p4", 1), ("s3", 0)])
def test_mobilenetv2_cat_known_answer(oracle, target, round_mode):
    """examples/mobilenetv2_cls/README.md lists the top-5 classes the reference prints for its cat.jpg:
    tabby, Egyptian_cat, Persian_cat, window_screen, lynx (ImageNet 281, 285, 283, 904, 287).  The shipped
    model, read with the layout rules of the loader and run on the oracle, must put tabby first and keep
    the cats on top; a wrong remainder or depthwise order gives window_screen or garbage instead.  (The
    JPEG decoder and resize differ from the firmware's, so logits are compared by rank, not value.)"""
    PIL = pytest.importorskip("PIL.Image")
    import sys
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    import espdl_spec
    import graph_runner
    spec, _ = espdl_spec.spec_from_espdl(os.path.join(REF, f"models/imagenet_cls/models/{target}/imagenet_cls_mobilenetv2_s8_v1.espdl"))
    img = np.asarray(PIL.open(os.path.join(REF, "examples/mobilenetv2_cls/main/cat.jpg")).convert("RGB"), dtype=np.float32)
    idx = (np.arange(224) * np.float32(img.shape[0] / 224)).astype(int)
    img = img[idx][:, idx]
    mean = np.array([123.675, 116.28, 103.53], dtype=np.float32)  # models/imagenet_cls/imagenet_cls.cpp:26
    std = np.array([58.395, 57.12, 57.375], dtype=np.float32)
    v = (img - mean) * (np.float32(1) / std)
    q = np.clip(np.floor(v * np.float32(2.0 ** -spec.exponent(spec.inputs[0])) + np.float32(0.5)), -128, 127).astype(np.int8)
    logits = graph_runner.run(spec, {spec.inputs[0]: q[None]}, round_mode, keep_all=False)[spec.outputs[0]][0].astype(int)
    top5 = set(int(i) for i in np.argsort(-logits, kind="stable")[:5])
    assert int(np.argmax(logits)) == 281
    assert len(top5 & {281, 285, 283, 904, 287}) >= 4
