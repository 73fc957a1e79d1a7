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


def test_requantized_residual_is_refused_for_misaligned_operands():
    """A block whose shape alone passes for the workgroup-per-tile kernel but whose input is only 4-byte aligned
    falls to kernels that add the residual operand as it is: with residual_shift != 0 the call must fail with
    ESPDL_HIP_ENOTSUP before anything is launched (no GPU needed: the pointers are never followed)."""
    import ctypes as C
    import importlib
    m = importlib.import_module("esp-dl_amd")
    d = m.capi.MbconvDesc(1, 14, 14, 96, 576, 96, 1, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0, 1, 1, 1)
    d.residual_shift = 2
    assert m.lib().espdl_hip_mbconv_s8_supported(C.byref(d)) == 5
    base = 1 << 20  # a fake device address, 256-byte aligned
    w = m.capi.MbconvWeights(base * 3, None, base * 4, base * 5, None, base * 6, base * 7, None, base * 8)
    rc = m.lib().espdl_hip_mbconv_s8(C.byref(d), C.c_void_p(base + 4), C.byref(w), C.c_void_p(base * 9), C.c_void_p(base * 10), None)
    assert rc == -95, m.lib().espdl_hip_last_error()
    assert b"residual_shift" in m.lib().espdl_hip_last_error()
