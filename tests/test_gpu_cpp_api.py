"""The C++ host layer used from C++: tests/cpp/api_check.cpp (built by esp-dl_amd/build.py into
esp-dl_amd/lib/espdl_api_check) loads a reference `.espdl` fixture with fbs::FbsLoader, runs
dl::Model::test() and a manual run-and-compare, and exits 0 when everything matches."""
import glob
import os
import subprocess

import pytest

from gpu_util import announce

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(os.path.dirname(HERE), "esp-dl_amd", "lib", "espdl_api_check")
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "espdl", "*.espdl")))


@pytest.mark.parametrize("path", [p for p in FIXTURES if ("chain" in p or "conv1d" in p or "gemm_c_" in p) and "streaming" not in p],
                         ids=os.path.basename)
def test_cpp_program_runs_fixture(path):
    if not os.path.exists(BIN):
        pytest.skip("esp-dl_amd/lib/espdl_api_check is not built (python esp-dl_amd/build.py builds it)")
    announce("C++ api_check " + os.path.basename(path))
    round_mode = "1" if "p4" in os.path.basename(path) else "0"
    r = subprocess.run([BIN, path, round_mode], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok" in r.stdout
