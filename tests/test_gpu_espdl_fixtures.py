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


# the streaming exports carry no embedded vectors: they are checked step by step against the oracle below
WITH_VECTORS = [p for p in FIXTURES if "streaming" not in os.path.basename(p)]


@pytest.mark.parametrize("path", [p for p in FIXTURES if "streaming" in os.path.basename(p)], ids=os.path.basename)
def test_streaming_model_carries_frames_between_calls(path):
    """StreamingCache: five consecutive chunks through one dl::Model (eager, then HIP-graph replays) against
    the oracle's graph runner keeping the same state; every image of the batch has its own history."""
    announce("espdl streaming " + os.path.basename(path))
    sys.path.insert(0, HERE)
    import espdl_spec
    import graph_runner
    import espdl_oracle as oracle
    spec, _ = espdl_spec.spec_from_espdl(path)
    model = importlib.import_module("esp-dl_amd").model
    rm = _round_mode(path)
    batch = 3
    rng = np.random.default_rng(78)
    mdl = model.Model(model.Graph.from_file(path), batch, round_mode=rm)
    state = {}
    outs = []
    for step in range(5):
        if step == 2:
            assert mdl.enable_graph()
        if step == 4:
            mdl.profile(repeats=2)  # timing passes must leave the carried frames alone
        x = spec.make_input(rng, batch)
        want = graph_runner.run(spec, {spec.inputs[0]: x}, oracle.ROUND_HALF_EVEN if rm else oracle.ROUND_HALF_UP,
                                keep_all=False, state=state)
        mdl.set_input(spec.inputs[0], x)
        mdl.run()
        for name in spec.outputs:
            np.testing.assert_array_equal(mdl.get_tensor(name).reshape(want[name].shape), want[name],
                                          err_msg=f"{name} step {step}")
        outs.append(want[spec.outputs[0]].copy())
    # the history matters: the same chunk gives another result once earlier frames are in the caches
    x = spec.make_input(np.random.default_rng(79), batch)
    fresh = graph_runner.run(spec, {spec.inputs[0]: x}, keep_all=False, state={})
    carried = graph_runner.run(spec, {spec.inputs[0]: x}, keep_all=False, state=state)
    assert not np.array_equal(fresh[spec.outputs[0]], carried[spec.outputs[0]])
    mdl.close()


@pytest.mark.parametrize("path", WITH_VECTORS, ids=os.path.basename)
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


def _extra_models():
    """More `.espdl` files (e.g. the reference's model zoo) can be named through ESPDL_EXTRA_MODELS, a
    directory; they are too large to keep as fixtures, so without the variable only the committed
    files run."""
    d = os.environ.get("ESPDL_EXTRA_MODELS")
    return sorted(glob.glob(os.path.join(d, "*.espdl"))) if d else []


@pytest.mark.parametrize("path", FIXTURES + _extra_models(), ids=os.path.basename)
def test_loaded_graph_matches_oracle_on_random_input(path):
    """Native loader -> dl::Model on the GPU against Python walker -> GraphSpec -> CPU oracle, on a seeded
    random batch: every graph output bit-exact (covers graphs whose files carry no test vectors)."""
    announce("espdl graph vs oracle " + os.path.basename(path))
    sys.path.insert(0, HERE)
    import espdl_spec
    import graph_runner
    import espdl_oracle as oracle
    spec, _ = espdl_spec.spec_from_espdl(path)
    model = importlib.import_module("esp-dl_amd").model
    unsupported = sorted({n["op_type"] for n in spec.nodes if not model.is_registered(n["op_type"])})
    if unsupported:
        pytest.skip("operators without a module in this build: " + ", ".join(unsupported))
    rm = _round_mode(path)
    batch = 3
    x = spec.make_input(np.random.default_rng(77), batch)
    try:
        want = graph_runner.run(spec, {spec.inputs[0]: x}, oracle.ROUND_HALF_EVEN if rm else oracle.ROUND_HALF_UP,
                                keep_all=False)
    except NotImplementedError as e:
        pytest.skip("the oracle's graph runner does not cover this graph: %s" % e)
    g = model.Graph.from_file(path)
    for fuse in (True, False):
        mdl = model.Model(g, batch, round_mode=rm, fuse_lut=fuse, fuse_blocks=fuse)
        mdl.set_input(spec.inputs[0], x)
        mdl.run()
        for name in spec.outputs:
            dt = np.int16 if spec.dtype(name) == 5 else np.int8
            got = mdl.get_tensor(name, dt)
            np.testing.assert_array_equal(got.reshape(want[name].shape), want[name], err_msg=f"{name} fuse={fuse}")
        mdl.close()
    # not a comparison of constants (single score maps of some detectors do saturate on noise)
    assert any(want[name].min() < want[name].max() for name in spec.outputs)
