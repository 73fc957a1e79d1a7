"""The loader-free host-layer interface, exercised from C++ by tests/cpp/module_api_check.cpp (built by
esp-dl_amd/build.py into esp-dl_amd/lib/espdl_module_api_check) the way the reference's API tests do
(test_apps/esp-dl/main/test_dl_api.cpp:20-335): Module::run on bare tensors, StreamingCache::reset,
Model::run(stage_num, stage_index), Model::reset; plus the Reshape / Squeeze output-shape rules, which
need no device."""
import os
import subprocess

import pytest

from gpu_util import announce

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(os.path.dirname(HERE), "esp-dl_amd", "lib", "espdl_module_api_check")


def _run(*args):
    if not os.path.exists(BIN):
        pytest.skip("esp-dl_amd/lib/espdl_module_api_check is not built (python esp-dl_amd/build.py builds it)")
    r = subprocess.run([BIN, *args], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ok" in r.stdout


def test_reshape_and_squeeze_shape_rules():
    _run("shapes")


@pytest.mark.gpu
def test_module_run_and_model_stages_on_device():
    announce("C++ module_api_check device")
    _run("device", os.path.join(HERE, "golden", "espdl", "gemm_chain_s3.espdl"))
