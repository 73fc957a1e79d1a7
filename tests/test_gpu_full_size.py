"""GPU parity at the sizes the benchmark configurations are quoted on: config 2 and 3 at batch 256,
config 4 at 640 x 640 batch 64 (all six outputs, int16 head included), config 5 at batch 512.
Kernel and tile selection depend on batch x pixels, so these are the code paths the benchmark times.
Every graph output is compared bit for bit with the CPU oracle run on the same seeded batch (the
oracle is called in chunks of images to bound host memory), eagerly and under HIP-graph replay."""
import importlib

import numpy as np
import pytest

from gpu_util import announce

pytestmark = pytest.mark.gpu


def _np_dtype(spec, name):
    return np.int16 if spec.dtype(name) == 5 else np.int8


def _oracle_outputs(spec, x, chunk, half_even=False):
    import espdl_oracle as oracle
    import graph_runner
    parts = {name: [] for name in spec.outputs}
    for i in range(0, x.shape[0], chunk):
        got = graph_runner.run(spec, {spec.inputs[0]: x[i:i + chunk]},
                               oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP, keep_all=False)
        for name in spec.outputs:
            parts[name].append(got[name])
    return {name: np.concatenate(v, axis=0) for name, v in parts.items()}


def _full_size(spec, batch, seed, chunk, half_even=False):
    pkg = importlib.import_module("esp-dl_amd")
    x = spec.make_input(np.random.default_rng(seed), batch)
    want = _oracle_outputs(spec, x, chunk, half_even)
    mdl = pkg.model.Model(pkg.model.Graph.from_spec(spec), batch, round_mode=1 if half_even else 0)
    mdl.set_input(spec.inputs[0], x)
    mdl.run()
    for name in spec.outputs:
        got = mdl.get_tensor(name, _np_dtype(spec, name))
        np.testing.assert_array_equal(got.reshape(want[name].shape), want[name], err_msg="eager " + name)
        assert want[name].min() < want[name].max(), name  # not a degenerate (saturated) tensor
    assert mdl.enable_graph()
    for rep in range(2):
        mdl.run()
        for name in spec.outputs:
            got = mdl.get_tensor(name, _np_dtype(spec, name))
            np.testing.assert_array_equal(got.reshape(want[name].shape), want[name],
                                          err_msg="graph replay %d %s" % (rep, name))
    mdl.close()


def test_config2_block_batch256(oracle):
    announce("full size: config2 batch 256")
    zoo = importlib.import_module("esp-dl_amd").zoo
    _full_size(zoo.config2_mbv2_block(), 256, 0xF2, 64)


def test_config3_mobilenetv2_224_batch256(oracle):
    announce("full size: config3 224x224 batch 256")
    zoo = importlib.import_module("esp-dl_amd").zoo
    _full_size(zoo.config3_mobilenetv2(), 256, 0xF3, 64)


def test_config3_mobilenetv2_224_batch256_round_half_even(oracle):
    """The rounding mode of ESP32-P4 exports: its own builds of the single-launch block kernels."""
    announce("full size: config3 224x224 batch 256, round half even")
    zoo = importlib.import_module("esp-dl_amd").zoo
    _full_size(zoo.config3_mobilenetv2(), 256, 0xF6, 64, half_even=True)


def test_config4_yolo_style_640_batch64(oracle):
    announce("full size: config4 640x640 batch 64")
    zoo = importlib.import_module("esp-dl_amd").zoo
    spec = zoo.config4_yolo_style()
    assert spec.shape(spec.inputs[0])[1:3] == [640, 640] and len(spec.outputs) == 6
    _full_size(spec, 64, 0xF4, 8)


def test_config5_ocr_style_batch512(oracle):
    announce("full size: config5 batch 512")
    zoo = importlib.import_module("esp-dl_amd").zoo
    _full_size(zoo.config5_ocr_style(), 512, 0xF5, 64)
