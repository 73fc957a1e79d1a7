"""GPU parity of the dl::Model executor: the five benchmark configurations, built from the same
GraphSpec on both sides, every intermediate tensor compared bit-for-bit with the CPU oracle."""
import importlib

import numpy as np
import pytest

from gpu_util import announce

pytestmark = pytest.mark.gpu


def _mods():
    m = importlib.import_module("esp-dl_amd")
    import graph_runner
    return m, m.zoo, m.model, graph_runner


def _np_dtype(spec, name):
    return np.int16 if spec.dtype(name) == 5 else np.int8


def _check_all(spec, mdl, want, skip_missing=True):
    checked = 0
    for name, ref in want.items():
        try:
            got = mdl.get_tensor(name, _np_dtype(spec, name))
        except KeyError:
            assert skip_missing
            continue
        if name not in spec.outputs and name in getattr(mdl, "_may_alias", ()):
            continue
        np.testing.assert_array_equal(got.reshape(ref.shape), ref, err_msg=name)
        checked += 1
    return checked


def _run_config(spec, batch, seed, round_mode=0, fuse_lut=True, graph=False, fuse_blocks=True, fuse_add=True,
                fuse_gap=True, channel_slices=True):
    m, zoo, model, runner = _mods()
    import espdl_oracle as oracle
    rng = np.random.default_rng(seed)
    x = spec.make_input(rng, batch)
    want = runner.run(spec, {spec.inputs[0]: x}, oracle.ROUND_HALF_EVEN if round_mode else oracle.ROUND_HALF_UP)
    g = model.Graph.from_spec(spec)
    mdl = model.Model(g, batch, round_mode=round_mode, fuse_lut=fuse_lut, fuse_blocks=fuse_blocks, fuse_add=fuse_add,
                      fuse_gap=fuse_gap, channel_slices=channel_slices)
    mdl.set_input(spec.inputs[0], x)
    if graph:
        assert mdl.enable_graph()
    mdl.run()
    return mdl, want, x


def test_config1_single_conv(oracle):
    announce("model config1")
    _, zoo, _, _ = _mods()
    spec = zoo.config1_single_conv()
    mdl, want, _ = _run_config(spec, 1, 1)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name])
    assert mdl.shape(spec.outputs[0]) == [1, 56, 56, 64]
    assert mdl.exponent(spec.outputs[0]) == -6
    mdl.close()


@pytest.mark.parametrize("batch", [1, 5])
def test_config2_mbv2_block(oracle, batch):
    announce(f"model config2 batch={batch}")
    _, zoo, _, _ = _mods()
    spec = zoo.config2_mbv2_block()
    mdl, want, _ = _run_config(spec, batch, 2)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
    mdl.close()


def test_config2_every_intermediate_with_test_vectors(oracle):
    """Model::test(): every tensor of the block carries a known answer (from the oracle)."""
    announce("model config2 Model::test")
    m, zoo, model, runner = _mods()
    spec = zoo.config2_mbv2_block()
    x = spec.make_input(np.random.default_rng(3), 2)
    want = runner.run(spec, {"input": x})
    outs = {k: v for k, v in want.items() if k != "input"}
    g = model.Graph.from_spec(spec, test_input={"input": x}, test_outputs=outs)
    mdl = model.Model(g, 2)
    assert mdl.test()
    # a corrupted expectation must be caught
    bad = dict(outs)
    bad["dw_out"] = outs["dw_out"].copy()
    bad["dw_out"].ravel()[12345] ^= 1
    g2 = model.Graph.from_spec(spec, test_input={"input": x}, test_outputs=bad)
    mdl2 = model.Model(g2, 2)
    assert not mdl2.test()
    mdl.close()
    mdl2.close()


def test_config3_mobilenetv2_full_resolution(oracle):
    """Full MobileNetV2-224 topology, batch 2; every layer output compared."""
    announce("model config3 224 batch 2")
    _, zoo, _, _ = _mods()
    spec = zoo.config3_mobilenetv2()
    mdl, want, _ = _run_config(spec, 2, 4)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
    assert mdl.shape(spec.outputs[0]) == [2, 1000]
    logits = want[spec.outputs[0]]
    assert logits.min() < 0 < logits.max() and len(np.unique(logits)) > 50  # not degenerate
    # every inverted-residual block is one module (the stem inside the first), the two RequantizeLinear nodes
    # that only align a residual operand's exponent ride in their block's launch, and the head convolution
    # pools its own output: 17 blocks + head convolution with GlobalAveragePool + the view + Gemm
    n_requant = sum(1 for n in spec.nodes if n["op_type"] == "RequantizeLinear")
    assert n_requant == 2 and mdl.module_count() == 20
    mdl.close()


def test_config3_mobilenetv2_all_intermediates(oracle):
    """Test vectors on every tensor of the 75-node graph (Model::test, module by module)."""
    announce("model config3 96px all intermediates")
    m, zoo, model, runner = _mods()
    spec = zoo.config3_mobilenetv2(resolution=96)
    x = spec.make_input(np.random.default_rng(5), 3)
    want = runner.run(spec, {"input": x})
    outs = {k: v for k, v in want.items() if k != "input"}
    g = model.Graph.from_spec(spec, test_input={"input": x}, test_outputs=outs)
    mdl = model.Model(g, 3)
    assert mdl.test()
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_mobilenetv2_requantized_residuals_at_other_exponents(oracle, round_mode):
    """The pattern of the reference's exported MobileNetV2 files: the residual operand goes through a
    RequantizeLinear (scale as a constant second input) to an exponent that differs from the project convolution's,
    and the Add sums the stored integers.  Each such node rides in its block's launch (residual_shift = its input
    exponent - its output exponent); same logits as the node-by-node run of the oracle."""
    announce(f"model config3 224px with relabelled residual RequantizeLinear, round mode {round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.config3_mobilenetv2(num_classes=100, relabel_residual=True)
    n_requant = sum(1 for n in spec.nodes if n["op_type"] == "RequantizeLinear")
    assert n_requant >= 5
    mdl, want, _ = _run_config(spec, 2, 23, round_mode=round_mode)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
    assert mdl.module_count() == 20  # 17 blocks, head convolution, the view, Gemm: no RequantizeLinear module left
    mdl.close()


def test_config3_half_even(oracle):
    announce("model config3 96px half-even")
    _, zoo, _, _ = _mods()
    spec = zoo.config3_mobilenetv2(resolution=96)
    mdl, want, _ = _run_config(spec, 2, 6, round_mode=1)
    np.testing.assert_array_equal(mdl.get_tensor(spec.outputs[0]), want[spec.outputs[0]])
    mdl.close()


def test_config3_hip_graph_replays(oracle):
    """The captured plan must reproduce the eager result on every replay, with new inputs in between."""
    announce("model config3 96px HIP graph")
    m, zoo, model, runner = _mods()
    spec = zoo.config3_mobilenetv2(resolution=96)
    g = model.Graph.from_spec(spec)
    mdl = model.Model(g, 4)
    rng = np.random.default_rng(7)
    x0 = spec.make_input(rng, 4)
    mdl.set_input("input", x0)
    mdl.run()
    eager0 = mdl.get_tensor(spec.outputs[0])
    assert mdl.enable_graph()
    for rep in range(4):
        x = x0 if rep % 2 == 0 else spec.make_input(rng, 4)
        mdl.set_input("input", x)
        mdl.run()
        got = mdl.get_tensor(spec.outputs[0])
        want = runner.run(spec, {"input": x}, keep_all=False)[spec.outputs[0]]
        np.testing.assert_array_equal(got, want, err_msg=f"replay {rep}")
        if rep % 2 == 0:
            np.testing.assert_array_equal(got, eager0)
    mdl.disable_graph()
    mdl.run()
    mdl.close()


@pytest.mark.parametrize("fuse", [True, False], ids=["fused_lut", "separate_lut"])
def test_config4_yolo_style(oracle, fuse):
    """Mixed precision: int8 conv + SiLU LUT trunk, int16 head (int64 accumulation)."""
    announce(f"model config4 160px fuse={fuse}")
    _, zoo, _, _ = _mods()
    spec = zoo.config4_yolo_style(resolution=160)
    mdl, want, _ = _run_config(spec, 2, 8, fuse_lut=fuse, fuse_blocks=fuse, fuse_add=fuse)
    assert len(spec.outputs) == 6
    for name in spec.outputs:
        got = mdl.get_tensor(name, _np_dtype(spec, name))
        np.testing.assert_array_equal(got, want[name], err_msg=name)
        assert want[name].min() < want[name].max()
    if fuse:
        assert mdl.module_count() < len(spec.nodes)  # Conv -> LUT pairs were folded
    else:
        assert mdl.module_count() == len(spec.nodes)
    mdl.close()


def test_first_block_with_requantized_residual_from_the_graph_input(oracle):
    """The very first modules of the plan form a block whose residual is the graph input behind a
    RequantizeLinear: absorbing that node must not end the scan, so the second block fuses as well."""
    announce("model two blocks, first residual requantized from the graph input")
    _, zoo, model, runner = _mods()
    g = zoo.GraphSpec("first_block_requantized_residual")
    b = zoo.Builder(g, 0xE5F1, per_channel=True, w_exp_range=None)
    x = b.input("input", [1, 14, 14, 32], -5)
    cur = x
    for i in range(2):
        h = b.conv(cur, 192, k=1, relu=True, name="b%d_expand" % i)
        h = b.conv(h, None, k=3, depthwise=True, relu=True, name="b%d_dw" % i)
        p = b.conv(h, 32, k=1, out_exp=-4, name="b%d_project" % i)
        cur = b.add(cur, p, name="b%d_add" % i)  # the first operand is at -5: requantized to -4 in front of the Add
    b.output(cur)
    assert sum(1 for n in g.nodes if n["op_type"] == "RequantizeLinear") == 1
    mdl, want, _ = _run_config(g, 3, 47)
    np.testing.assert_array_equal(mdl.get_tensor(g.outputs[0]), want[g.outputs[0]])
    assert mdl.module_count() == 2
    mdl.close()


def test_channel_slices_every_case(oracle):
    """Split outputs left inside the Split's input and Concat inputs written in place, case by case: which
    tensors become slices (by their pitch), every tensor against the oracle, twice (the slices must survive a
    second pass over the same arena), then under a captured graph."""
    announce("model channel_slices")
    _, zoo, _, runner = _mods()
    spec = zoo.channel_slices()
    batch = 3
    mdl, want, x = _run_config(spec, batch, 41)
    pitch = {n: mdl.channel_pitch(n) for n in want if n not in spec.inputs}
    dense = lambda n: pitch[n] == want[n].shape[-1]  # noqa: E731
    # block 1: the pieces stay in s1_cv1's output (48 wide) except the one Relu reads; the bottleneck's result
    # (conv + folded Add) is written into the Concat (68 wide); s1_cv1's output itself cannot move
    assert pitch["s1_split_out0"] == 48 and pitch["s1_split_out1"] == 48 and dense("s1_split_out2")
    assert pitch["s1_add_out"] == 68 and dense("s1_relu_out") and dense("s1_cv1_out")
    # block 2: all pieces of the Split go into the Concat -> the Split's input lives inside the Concat (48 wide)
    assert pitch["s2_cv1_out"] == 48 and pitch["s2_split_out0"] == 48 and pitch["s2_split_out1"] == 48
    assert pitch["s2_m_out"] == 48
    # a tensor that appears twice in one Concat is copied there; it is in place in the later Concat (24 wide)
    assert pitch["s3_y_out"] == 24 and pitch["s3_z_out"] == 48 and dense("s4_out_out")
    assert pitch["s5_split_out0"] == 24 and dense("s5_split_out1")  # the depthwise Conv takes no pitch
    assert pitch["s5_strided_out"] == 24 and dense("s5_dw_out")
    # the requantized and the upsampled input of the last Concat are written in their places (40 wide)
    assert pitch["s6_cat_rq0_out"] == 40 and pitch["s6_up_out"] == 40 and dense("s6_fine_out")
    # (intermediate tensors share arena space: only the graph outputs, which every slice feeds, outlive a pass)
    for rep in range(2):
        for name in spec.outputs:
            np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=f"{name} pass {rep}")
            assert want[name].min() < want[name].max()
        mdl.run()
    assert mdl.enable_graph()
    x2 = spec.make_input(np.random.default_rng(42), batch)
    mdl.set_input(spec.inputs[0], x2)
    mdl.run()
    want2 = runner.run(spec, {spec.inputs[0]: x2}, keep_all=False)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want2[name], err_msg=name)
    mdl.close()
    # and with the slices switched off: everything dense, same results
    mdl, want, _ = _run_config(spec, batch, 41, channel_slices=False)
    for name, ref in want.items():
        if name not in spec.inputs:
            assert mdl.channel_pitch(name) in (ref.shape[-1], -1)  # -1: folded into a Conv, no tensor of its own
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
    mdl.close()


def test_channel_slices_pinned_tensors_stay_dense(oracle):
    """Tensors with test vectors stay dense and alive: with every Split / Concat / Conv output of the slices
    graph pinned, each equals the oracle's and nothing is a slice."""
    announce("model channel_slices pinned")
    m, zoo, model, runner = _mods()
    spec = zoo.channel_slices()
    batch = 2
    x = spec.make_input(np.random.default_rng(43), batch)
    want = runner.run(spec, {spec.inputs[0]: x})
    names = [o for n in spec.nodes for o in n["outputs"]]
    g = model.Graph.from_spec(spec, test_outputs={n: want[n][:1] for n in names})
    mdl = model.Model(g, batch)
    mdl.set_input(spec.inputs[0], x)
    mdl.run()
    for n in names:
        assert mdl.channel_pitch(n) == want[n].shape[-1], n
        np.testing.assert_array_equal(mdl.get_tensor(n), want[n], err_msg=n)
    mdl.close()
    # pin only the Concat outputs and the Split inputs: their slices are still made, and must be right
    keep = [o for n in spec.nodes if n["op_type"] == "Concat" for o in n["outputs"]] + ["s1_cv1_out"]
    g = model.Graph.from_spec(spec, test_outputs={n: want[n][:1] for n in keep})
    mdl = model.Model(g, batch)
    mdl.set_input(spec.inputs[0], x)
    mdl.run()
    assert mdl.channel_pitch("s1_split_out0") == 48 and mdl.channel_pitch("s2_m_out") == 48
    for n in keep:
        np.testing.assert_array_equal(mdl.get_tensor(n), want[n], err_msg=n)
    # the pieces of s1_cv1's output are views of a tensor that is still alive
    np.testing.assert_array_equal(mdl.get_tensor("s1_split_out0"), want["s1_split_out0"])
    np.testing.assert_array_equal(mdl.get_tensor("s1_split_out1"), want["s1_split_out1"])
    mdl.close()


@pytest.mark.parametrize("slices", [True, False], ids=["in_place", "copied"])
def test_config4_channel_slices(oracle, slices):
    """The detector graph with its C3k2 Splits / Concats in place and copied: every tensor equals the oracle's,
    and the device arena is no larger in place."""
    announce(f"model config4 160px channel_slices={slices}")
    _, zoo, _, _ = _mods()
    spec = zoo.config4_yolo_style(resolution=160)
    mdl, want, _ = _run_config(spec, 2, 9, channel_slices=slices)
    if slices:
        assert mdl.channel_pitch("c2_split_out0") == 96 and mdl.channel_pitch("c2_cv1_act_out") == 96
    else:
        assert mdl.channel_pitch("c2_split_out0") == 32
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name, _np_dtype(spec, name)), want[name], err_msg=name)
    mdl.close()


def test_config4_neck_data_movement_tensors(oracle):
    """Every Split / Concat / MaxPool / Resize / Transpose output of the detector graph, kept alive as
    test outputs, equals the oracle's (C3k2 split+concat, SPPF pool chain, FPN upsample+concat)."""
    announce("model config4 160px neck tensors")
    m, zoo, model, runner = _mods()
    import espdl_oracle as oracle_mod
    spec = zoo.config4_yolo_style(resolution=160)
    batch = 3
    x = spec.make_input(np.random.default_rng(12), batch)
    want = runner.run(spec, {spec.inputs[0]: x}, oracle_mod.ROUND_HALF_UP)
    names = [o for n in spec.nodes if n["op_type"] in ("Split", "Concat", "MaxPool", "Resize", "Transpose")
             for o in n["outputs"]]
    assert len(names) >= 25
    g = model.Graph.from_spec(spec, test_outputs={n: want[n][:1] for n in names})
    mdl = model.Model(g, batch)
    mdl.set_input(spec.inputs[0], x)
    mdl.run()
    for n in names:
        np.testing.assert_array_equal(mdl.get_tensor(n, _np_dtype(spec, n)), want[n], err_msg=n)
    # under a captured graph as well
    assert mdl.enable_graph()
    mdl.run()
    for n in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(n, _np_dtype(spec, n)), want[n], err_msg=n)
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_gated_block_with_mul(oracle, round_mode):
    """Sigmoid LUT + Mul gates (same-shape and broadcast over H x W), both rounding modes."""
    announce(f"model gated_block round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.gated_block()
    mdl, want, _ = _run_config(spec, 4, 21, round_mode=round_mode)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
        assert want[name].min() < want[name].max()
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_pooled_embedding_tail(oracle, round_mode):
    """AveragePool, ReduceMean and Reshape whose axes / shape arrive as initializer operands, then Gemm."""
    announce(f"model pooled_embedding round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.pooled_embedding()
    mdl, want, _ = _run_config(spec, 5, 33, round_mode=round_mode)
    got = mdl.get_tensor(spec.outputs[0])
    assert got.shape == (5, 64)
    np.testing.assert_array_equal(got, want[spec.outputs[0]])
    assert want[spec.outputs[0]].min() < want[spec.outputs[0]].max()
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_attention_block(oracle, round_mode):
    """MatMul of two activations, Mul by a constant, Softmax to float32, QuantizeLinear back to int8."""
    announce(f"model attention_block round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.attention_block()
    mdl, want, _ = _run_config(spec, 3, 35, round_mode=round_mode)
    got = mdl.get_tensor(spec.outputs[0])
    np.testing.assert_array_equal(got, want[spec.outputs[0]])
    assert want[spec.outputs[0]].min() < want[spec.outputs[0]].max()
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_int16_tail(oracle, round_mode):
    """int16 table, Add, Mul by a constant, AveragePool and ReduceMean behind an int8 -> int16 requantize."""
    announce(f"model int16_tail round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.int16_tail()
    mdl, want, _ = _run_config(spec, 3, 37, round_mode=round_mode)
    got = mdl.get_tensor(spec.outputs[0], np.int16)
    np.testing.assert_array_equal(got, want[spec.outputs[0]])
    assert want[spec.outputs[0]].min() < want[spec.outputs[0]].max()
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_centered_ratio(oracle, round_mode):
    """int8 Sub (broadcast) and Div in its loop and both table forms, through dl::Model."""
    announce(f"model centered_ratio round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.centered_ratio()
    mdl, want, _ = _run_config(spec, 3, 39, round_mode=round_mode)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name])
        assert len(np.unique(want[name])) > 8
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
@pytest.mark.parametrize("s16", [False, True], ids=["s8", "s16"])
def test_activation_chain(oracle, s16, round_mode):
    """Sigmoid, Tanh, HardSwish, Elu, LeakyRelu, Swish, HardSigmoid, Neg, Exp, Sqrt, Log and Identity nodes
    without tables in the file: the module evaluates the reference's float32 expression per possible input."""
    announce(f"model activation_chain s16={s16} round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.activation_chain(s16=s16)
    mdl, want, _ = _run_config(spec, 3, 41, round_mode=round_mode)
    for name in spec.outputs:
        got = mdl.get_tensor(name, np.int16) if s16 else mdl.get_tensor(name)
        np.testing.assert_array_equal(got, want[name], err_msg=name)
        assert len(np.unique(want[name])) > 20, name
    mdl.close()


def test_padded_convs(oracle):
    """Pad nodes (reflect, edge, constant with a value) in front of unpadded convolutions."""
    announce("model padded_convs")
    _, zoo, _, _ = _mods()
    spec = zoo.padded_convs()
    mdl, want, _ = _run_config(spec, 3, 43)
    got = mdl.get_tensor(spec.outputs[0])
    np.testing.assert_array_equal(got, want[spec.outputs[0]])
    assert len(np.unique(want[spec.outputs[0]])) > 20
    mdl.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
@pytest.mark.parametrize("s16", [False, True], ids=["s8", "s16"])
def test_reduce_heads(oracle, s16, round_mode):
    """ReduceMax, ReduceMin and ReduceSum nodes through dl::Model."""
    announce(f"model reduce_heads s16={s16} round_mode={round_mode}")
    _, zoo, _, _ = _mods()
    spec = zoo.reduce_heads(s16=s16)
    mdl, want, _ = _run_config(spec, 3, 45, round_mode=round_mode)
    for name in spec.outputs:
        got = mdl.get_tensor(name, np.int16) if s16 else mdl.get_tensor(name)
        np.testing.assert_array_equal(got, want[name], err_msg=name)
        assert len(np.unique(want[name])) > 8, name
    mdl.close()


def test_pixel_shuffle(oracle):
    """SpaceToDepth and DepthToSpace (CRD and DCR) nodes through dl::Model."""
    announce("model pixel_shuffle")
    _, zoo, _, _ = _mods()
    spec = zoo.pixel_shuffle()
    mdl, want, _ = _run_config(spec, 3, 47)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
        assert len(np.unique(want[name])) > 20, name
    assert not np.array_equal(want[spec.outputs[0]], want[spec.outputs[1]])
    mdl.close()


def test_gathered_rows(oracle):
    """Gather with constant indices (single index, repeats, a 2-D index tensor) through dl::Model."""
    announce("model gathered_rows")
    _, zoo, _, _ = _mods()
    spec = zoo.gathered_rows()
    mdl, want, _ = _run_config(spec, 3, 49)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
        assert len(np.unique(want[name])) > 20, name
    mdl.close()


def test_config5_ocr_style(oracle):
    announce("model config5 batch 3")
    _, zoo, _, _ = _mods()
    spec = zoo.config5_ocr_style()
    mdl, want, _ = _run_config(spec, 3, 9)
    got = mdl.get_tensor(spec.outputs[0])
    assert got.shape == (3, 40, 6625)
    np.testing.assert_array_equal(got, want[spec.outputs[0]])
    mdl.close()


def test_profile_reports_every_module():
    announce("model profile")
    _, zoo, model, _ = _mods()
    spec = zoo.config2_mbv2_block()
    mdl = model.Model(model.Graph.from_spec(spec), 4)
    info = mdl.profile(repeats=2)
    assert len(info) == mdl.module_count()
    convs = [i for i in info if "Conv" in i["type"]]  # "Conv", or "Conv>DepthwiseConv>Conv:wave" for a fused block
    assert sum(i["macs"] for i in convs) == 4 * spec.conv_macs_per_image
    assert all(i["latency_us"] > 0 for i in info)
    mdl.close()


def test_unknown_operator_fails_to_load():
    announce("model unknown op")
    _, zoo, model, _ = _mods()
    spec = zoo.config1_single_conv()
    spec.nodes[0]["op_type"] = "NoSuchOp"
    with pytest.raises(model.EspdlModelError):
        model.Model(model.Graph.from_spec(spec), 1)


@pytest.mark.parametrize("fuse_blocks", [True, False], ids=["fused_blocks", "separate_modules"])
def test_mobilenetv2_block_fusion(oracle, fuse_blocks):
    """depthwise -> project [-> Add] chains run as one module or as separate ones: same logits, and the
    fused plan is shorter (only blocks with at most 256 expanded channels fuse)."""
    announce(f"model config3 96px fuse_blocks={fuse_blocks}")
    _, zoo, _, _ = _mods()
    spec = zoo.config3_mobilenetv2(resolution=96, num_classes=100)
    mdl, want, _ = _run_config(spec, 3, 21, fuse_blocks=fuse_blocks, fuse_add=fuse_blocks, fuse_gap=fuse_blocks)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
    if fuse_blocks:
        assert mdl.module_count() < len(spec.nodes)
    else:
        assert mdl.module_count() == len(spec.nodes)
    mdl.close()


def test_mobilenetv2_conv_add_fusion(oracle):
    """Residual Adds folded into the project convolutions' epilogues, and not: same logits."""
    announce("model config3 96px fuse_add")
    _, zoo, _, _ = _mods()
    spec = zoo.config3_mobilenetv2(resolution=96, num_classes=100)
    mdl, want, _ = _run_config(spec, 3, 22, fuse_add=True)
    plain, _, _ = _run_config(spec, 3, 22, fuse_add=False)
    for name in spec.outputs:
        np.testing.assert_array_equal(mdl.get_tensor(name), want[name], err_msg=name)
        np.testing.assert_array_equal(plain.get_tensor(name), want[name], err_msg=name)
    assert mdl.module_count() < plain.module_count()
    mdl.close()
    plain.close()


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
def test_activation_modules_prelu_relu_nodes(oracle, round_mode):
    """PRelu and Relu as graph nodes of their own (dl::module::PRelu::forward, dl::module::Relu::forward
    through dl::Model), every tensor compared; also under HIP-graph replay."""
    announce(f"model activation_modules round_mode={round_mode}")
    m, zoo, model, runner = _mods()
    spec = zoo.activation_modules()
    assert [n["op_type"] for n in spec.nodes].count("PRelu") == 2 and "Relu" in [n["op_type"] for n in spec.nodes]
    batch = 5
    x = spec.make_input(np.random.default_rng(31), batch)
    import espdl_oracle as oracle_mod
    want = runner.run(spec, {"input": x}, oracle_mod.ROUND_HALF_EVEN if round_mode else oracle_mod.ROUND_HALF_UP)
    outs = {k: v for k, v in want.items() if k != "input"}
    g = model.Graph.from_spec(spec, test_input={"input": x}, test_outputs=outs)
    mdl = model.Model(g, batch, round_mode=round_mode)
    assert mdl.test()  # module by module, every tensor
    mdl.set_input("input", x)
    assert mdl.enable_graph()
    for _ in range(2):
        mdl.run()
        np.testing.assert_array_equal(mdl.get_tensor(spec.outputs[0]), want[spec.outputs[0]])
    assert (want["c1_prelu_out"] < 0).any() and (want["c2_relu_out"] == 0).any()
    mdl.close()


def test_failed_forward_is_reported(oracle):
    """A module whose launch is rejected on the host (a Conv with an activation no kernel fuses) makes
    run() fail instead of returning stale bytes, and its plan is not captured into a HIP graph."""
    announce("model run reports a rejected module")
    m, zoo, model, runner = _mods()
    spec = zoo.config1_single_conv()
    spec.nodes[0]["attrs"]["activation"] = "LeakyRelu"
    mdl = model.Model(model.Graph.from_spec(spec), 1)
    mdl.set_input("input", spec.make_input(np.random.default_rng(1), 1))
    with pytest.raises(model.EspdlModelError):
        mdl.run()
    assert not mdl.enable_graph()
    with pytest.raises(model.EspdlModelError):
        mdl.run()
    mdl.close()
    # the same graph with a supported activation runs
    spec = zoo.config1_single_conv()
    mdl = model.Model(model.Graph.from_spec(spec), 1)
    mdl.set_input("input", spec.make_input(np.random.default_rng(1), 1))
    mdl.run()
    mdl.close()
