"""The reference's own `.espdl` fixtures (exported by esp-ppq, with embedded inputs and expected
outputs) loaded by the native loader and run on the GPU: dl::Model::test() compares every tensor the
file lists, as the reference's Model::test does (esp-dl/dl/model/src/dl_model_base.cpp)."""
import glob
import importlib
import os
import sys

import numpy as np
import pytest

from gpu_util import announce

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "espdl", "*.espdl")))


def _round_mode(path):
    # ESP32-P4 builds of the reference round half to even, the others half up
    return 1 if "p4" in os.path.basename(path) else 0


@pytest.mark.parametrize("path", FIXTURES, ids=os.path.basename)
def test_reference_fixture_passes_model_test(path):
    announce("espdl fixture " + os.path.basename(path))
    model = importlib.import_module("esp-dl_amd").model
    g = model.Graph.from_file(path)
    mdl = model.Model(g, 1, round_mode=_round_mode(path))
    assert mdl.test()
    mdl.close()


@pytest.mark.parametrize("path", [p for p in FIXTURES if "chain" in p or "1_64" in p], ids=os.path.basename)
def test_reference_fixture_batched(path):
    """The same known answers with the fixture's input repeated over a batch of 5."""
    announce("espdl fixture batched " + os.path.basename(path))
    sys.path.insert(0, os.path.join(HERE, "golden"))
    import espdl_reader
    ref = espdl_reader.read_espdl(path)
    model = importlib.import_module("esp-dl_amd").model
    g = model.Graph.from_file(path)
    mdl = model.Model(g, 5, round_mode=_round_mode(path))
    (in_name, tin), = ref["test_inputs"].items()
    x = np.repeat(tin["data"].reshape(tin["dims"]), 5, axis=0)
    mdl.set_input(in_name, x)
    mdl.run()
    for name, tout in ref["test_outputs"].items():
        want = np.repeat(tout["data"].reshape(tout["dims"]), 5, axis=0)
        np.testing.assert_array_equal(mdl.get_tensor(name).reshape(want.shape), want, err_msg=name)
    mdl.close()
