"""The C-ABI library loads on a machine without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    with open(os.path.join(ROOT, "include", header)) as f:
        text = re.sub(r"/\*.*?\*/", "", f.read(), flags=re.S)
    return sorted(set(re.findall(r"\b(espdl_\w+)\s*\(", text)))


def test_libespdl_hip_exports_header_symbols():
    path = os.path.join(ROOT, "esp-dl_amd", "lib", "libespdl_hip.so")
    assert os.path.exists(path), "run `python esp-dl_amd/build.py` (or __graft_entry__.build()) first"
    lib = ctypes.CDLL(path)
    names = _declared("espdl_hip.h")
    assert len(names) >= 12
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in include/espdl_hip.h but not exported"


def test_validation_needs_no_gpu():
    import importlib
    m = importlib.import_module("esp-dl_amd")
    d = m.capi.make_desc((1, 56, 56, 64), 64, (3, 3), pads=(1, 1, 1, 1))
    assert m.conv_out_shape(d) == (56, 56)
    d = m.capi.make_desc((1, 100, 50, 3), 16, (3, 3), stride=(2, 2))
    assert m.conv_out_shape(d) == (49, 24)
    d.group = 5
    try:
        m.conv_out_shape(d)
        assert False
    except m.EspdlHipError as e:
        assert "group" in str(e)
