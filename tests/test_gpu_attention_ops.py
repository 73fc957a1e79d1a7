"""Softmax (int8 -> float32), QuantizeLinear / DequantizeLinear and activation x activation MatMul on the GPU
against the CPU oracle.  Integer results are bit-exact.  The float32 softmax is compared bit for bit too: both
sides build the 256-entry table with the host C library's expf, add the row in index order in float32 and
divide once per element in IEEE float32."""
import numpy as np
import pytest

from gpu_util import announce, espdl, to_dev, to_host

pytestmark = pytest.mark.gpu


def _rand(rng, shape, dtype=np.int8):
    info = np.iinfo(dtype)
    return rng.integers(info.min, info.max + 1, size=shape).astype(dtype)


SOFTMAX_CASES = [
    # (shape, axis, in_exp)
    ((2, 2, 400, 400), -1, -3),   # the attention map of the exported YOLO11n graphs at 640 x 640
    ((3, 2, 100, 100), -1, -3),
    ((5, 7, 33), -1, -4),         # odd row length
    ((300, 1), -1, -2),           # rows of one element
    ((2, 1000, 6), -1, -5),       # many short rows
    ((4, 3000), -1, -4),          # rows longer than one staging buffer line
    ((2, 40000), -1, -6),         # rows too long for LDS staging: strided path with inner == 1
    ((2, 16, 20, 20), 1, -3),     # softmax over channels of an NCHW map (DFL-style)
    ((3, 9, 5), 0, -4),
    ((2, 5, 7, 3), 2, -4),
]


@pytest.mark.parametrize("case", SOFTMAX_CASES, ids=lambda c: f"{c[0]}_ax{c[1]}")
def test_softmax_s8(oracle, case):
    shape, axis, in_exp = case
    announce(f"softmax_s8 {case}")
    x = _rand(np.random.default_rng(41), shape)
    got = to_host(espdl().softmax_s8(to_dev(x), axis, in_exp))
    want = oracle.softmax_s8(x, axis, in_exp)
    assert got.dtype == np.float32
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_softmax_empty():
    announce("softmax_s8 empty")
    import torch
    out = espdl().softmax_s8(torch.empty((0, 8), dtype=torch.int8, device="cuda"), -1, -3)
    assert tuple(out.shape) == (0, 8)


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("out_exp", [-9, -7, 0, 3])
def test_quantize_f32(oracle, dtype, out_exp):
    announce(f"quantize_f32 {dtype.__name__} exp {out_exp}")
    import torch
    rng = np.random.default_rng(42)
    info = np.iinfo(dtype)
    scale = 2.0 ** out_exp
    x = np.concatenate([(rng.standard_normal(100003) * info.max * scale * 0.7).astype(np.float32),
                        ((np.arange(-300, 300) + 0.5) * scale).astype(np.float32),
                        rng.random(5000, dtype=np.float32)])
    got = to_host(espdl().quantize_f32(to_dev(x), out_exp, torch.int8 if dtype == np.int8 else torch.int16))
    np.testing.assert_array_equal(got, oracle.quantize_f32(x, out_exp, dtype))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
def test_dequantize_f32(oracle, dtype):
    announce(f"dequantize_f32 {dtype.__name__}")
    x = _rand(np.random.default_rng(43), (7, 1001), dtype)
    for e in (-12, -3, 0, 4):
        got = to_host(espdl().dequantize_f32(to_dev(x), e))
        np.testing.assert_array_equal(got.view(np.uint32), oracle.dequantize_f32(x, e).view(np.uint32))


def test_softmax_then_quantize_matches_reference_chain(oracle):
    """Softmax -> QuantizeLinear as the exported attention blocks chain them."""
    announce("softmax + quantize chain")
    x = _rand(np.random.default_rng(44), (2, 2, 400, 400))
    m = espdl()
    got = to_host(m.quantize_f32(m.softmax_s8(to_dev(x), -1, -3), -9))
    np.testing.assert_array_equal(got, oracle.quantize_f32(oracle.softmax_s8(x, -1, -3), -9))
    assert got.max() > 0


MATMUL_CASES = [
    # (a shape, b shape, shift)
    ((2, 2, 400, 32), (2, 2, 32, 400), 9),     # q^T x k of the exported attention block
    ((2, 2, 64, 400), (2, 2, 400, 400), 8),    # v x attn^T
    ((3, 1, 5, 7), (1, 4, 7, 3), 6),           # both leading dims broadcast, tiles mostly empty
    ((2, 65, 33), (2, 33, 130), 7),            # rank 3, extents just past one tile / chunk
    ((4, 9, 64), (1, 64, 64), 9),              # rank 3, right operand broadcast
    ((17, 100), (100, 19), 8),                 # plain matrices
    ((1, 1, 1, 1), (1, 1, 1, 1), 1),
    ((2, 3, 8, 16), (2, 3, 16, 8), 0),         # shift 0: saturation only
    ((2, 3, 8, 16), (2, 3, 16, 8), -2),        # left shift
]


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
@pytest.mark.parametrize("case", MATMUL_CASES, ids=lambda c: f"{c[0]}x{c[1]}_s{c[2]}")
def test_matmul_s8(oracle, case, round_mode):
    sa, sb, shift = case
    announce(f"matmul_s8 {case} round_mode={round_mode}")
    rng = np.random.default_rng(45)
    a, b = _rand(rng, sa), _rand(rng, sb)
    for act in (oracle.LINEAR, oracle.RELU):
        got = to_host(espdl().matmul_s8(to_dev(a), to_dev(b), shift, act, round_mode))
        want = oracle.matmul_s8(a, b, shift, act, round_mode)
        np.testing.assert_array_equal(got, want.reshape(got.shape))


def test_matmul_rounding_ties(oracle):
    """Accumulators that sit exactly on .5 after the shift: the two rounding modes differ there."""
    announce("matmul_s8 ties")
    a = np.zeros((1, 1, 64, 4), dtype=np.int8)
    a[0, 0, :, 0] = np.arange(-32, 32)
    b = np.zeros((1, 1, 4, 64), dtype=np.int8)
    b[0, 0, 0, :] = 1
    up = to_host(espdl().matmul_s8(to_dev(a), to_dev(b), 1, 0, 0))
    even = to_host(espdl().matmul_s8(to_dev(a), to_dev(b), 1, 0, 1))
    np.testing.assert_array_equal(up, oracle.matmul_s8(a, b, 1, 0, 0))
    np.testing.assert_array_equal(even, oracle.matmul_s8(a, b, 1, 0, 1))
    assert not np.array_equal(up, even)


def test_matmul_rejects_bad_arguments():
    announce("matmul_s8 argument checks")
    import ctypes
    import torch
    m = espdl()
    a = torch.zeros((2, 4), dtype=torch.int8, device="cuda")
    lead = (ctypes.c_int32 * 2)(70000, 1)
    z = (ctypes.c_int64 * 2)(0, 0)
    rc = m.lib().espdl_hip_matmul_s8(a.data_ptr(), a.data_ptr(), 2, 4, 2, lead, z, z, 7, 0, 0, a.data_ptr(), None)
    assert rc != 0 and b"65535" in m.lib().espdl_hip_last_error()
    lead = (ctypes.c_int32 * 2)(1, 1)
    assert m.lib().espdl_hip_matmul_s8(a.data_ptr(), a.data_ptr(), 2, 4, 2, lead, z, z, 7, 5, 0, a.data_ptr(), None) != 0
    assert m.lib().espdl_hip_matmul_s8(a.data_ptr(), None, 2, 4, 2, lead, z, z, 7, 0, 0, a.data_ptr(), None) != 0


@pytest.mark.parametrize("round_mode", [0, 1], ids=["ties_up", "ties_even"])
@pytest.mark.parametrize("entries", [65536, 65537, 32769, 2049, 257, 3])
def test_lut_s16(oracle, entries, round_mode):
    announce(f"lut_s16 entries={entries} round_mode={round_mode}")
    rng = np.random.default_rng(46)
    table = _rand(rng, (entries,), np.int16)
    x = np.concatenate([np.arange(-32768, 32768, dtype=np.int16), _rand(rng, (100003,), np.int16)])
    got = to_host(espdl().lut_s16(to_dev(x), to_dev(table), round_mode))
    np.testing.assert_array_equal(got, oracle.lut_s16(x, table, round_mode == 1))


def test_lut_s16_rejects_odd_table_sizes():
    announce("lut_s16 argument checks")
    import torch
    m = espdl()
    x = torch.zeros(8, dtype=torch.int16, device="cuda")
    with pytest.raises(m.EspdlHipError):
        m.lut_s16(x, torch.zeros(1000, dtype=torch.int16, device="cuda"))


def test_add_s16(oracle):
    announce("add_s16")
    rng = np.random.default_rng(60)
    a, b = _rand(rng, (3, 7, 33), np.int16), _rand(rng, (3, 7, 33), np.int16)
    np.testing.assert_array_equal(to_host(espdl().add_s16(to_dev(a), to_dev(b))), oracle.add_s16(a, b))
    # broadcast over the last axis
    c = _rand(rng, (3, 7, 1), np.int16)
    want = np.clip(a.astype(np.int32) + c.astype(np.int32), -32768, 32767).astype(np.int16)
    np.testing.assert_array_equal(to_host(espdl().add_s16(to_dev(a), to_dev(c))), want)


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
@pytest.mark.parametrize("shift", [0, 7, 13, 15, 22])
def test_mul_s16(oracle, shift, round_mode):
    announce(f"mul_s16 shift={shift} round_mode={round_mode}")
    rng = np.random.default_rng(61)
    a, b = _rand(rng, (50021,), np.int16), _rand(rng, (50021,), np.int16)
    a[:4], b[:4] = [-32768, 32767, -32768, 4097], [-32768, 32767, 32767, 4099]
    got = to_host(espdl().mul_s16(to_dev(a), to_dev(b), shift, round_mode))
    np.testing.assert_array_equal(got, oracle.mul_s16(a, b, shift, round_mode))
    s = _rand(rng, (1,), np.int16)
    got = to_host(espdl().mul_s16(to_dev(a), to_dev(s), shift, round_mode))
    np.testing.assert_array_equal(got, oracle.mul_s16(a, s, shift, round_mode))


def test_avg_pool_and_reduce_mean_s16(oracle):
    announce("avg_pool_s16 / reduce_mean_s16")
    rng = np.random.default_rng(62)
    x = _rand(rng, (3, 12, 9, 20), np.int16)
    for k, st, pads, ei, eo in (((3, 3), (2, 2), (1, 1, 1, 1), -10, -9), ((2, 2), (2, 2), (0, 0, 0, 0), -12, -12),
                                ((1, 9), (1, 1), (0, 0, 0, 0), -8, -11)):
        got = to_host(espdl().avg_pool_s16(to_dev(x), k, st, pads, ei, eo))
        np.testing.assert_array_equal(got, oracle.avg_pool_s16(x, k, st, pads, ei, eo))
    for axes, keep in (([1, 2], True), ([3], False), ([0, 2], True), ([], True)):
        got = to_host(espdl().reduce_mean_s16(to_dev(x), axes, keep, -10, -12))
        np.testing.assert_array_equal(got, oracle.reduce_mean_s16(x, axes, keep, -10, -12))


# int16 means over long runs of neighbouring axes (the pooling of a speaker-embedding or text-recognition graph):
# inner sizes of one 16-byte piece, several slabs, odd (single-element loads), 1; extreme inputs.
@pytest.mark.parametrize("shape,axes,keepdims", [
    ((4, 300, 8), [1], False), ((2, 40, 50, 520), [1, 2], True), ((3, 97, 1, 37), [1, 2], True), ((6, 1500), [1], True),
    ((2, 3, 200, 24), [2], False),
])
def test_reduce_mean_s16_long_runs(oracle, shape, axes, keepdims):
    announce(f"reduce_mean_s16 long runs {shape} axes {axes}")
    rng = np.random.default_rng(63)
    for x in (_rand(rng, shape, np.int16), np.full(shape, 32767, np.int16), np.full(shape, -32768, np.int16)):
        got = to_host(espdl().reduce_mean_s16(to_dev(x), axes, keepdims, -10, -12))
        np.testing.assert_array_equal(got, oracle.reduce_mean_s16(x, axes, keepdims, -10, -12))


# int16 Add / Mul / Sub and int8 Sub where the innermost axis is dense or constant in each operand and a multiple of
# a 16-byte piece long (8 int16, 16 int8): the 16-bytes-per-thread form, dense and with broadcasting.
@pytest.mark.parametrize("sa,sb", [((3, 20, 20, 64), (3, 1, 1, 64)), ((3, 1, 1, 64), (3, 20, 20, 64)), ((2, 75, 40), (2, 75, 40)),
                                   ((4, 7, 32), (1, 7, 1)), ((2, 9, 16), (16,)), ((6, 1, 5, 32), (1, 4, 1, 1))],
                         ids=lambda s: "x".join(map(str, s)))
def test_binary_s16_and_sub_s8_wide_form(oracle, sa, sb):
    announce(f"binary s16 / sub s8 wide form {sa} {sb}")
    rng = np.random.default_rng(66)
    a, b = _rand(rng, sa, np.int16), _rand(rng, sb, np.int16)
    a.reshape(-1)[:2], b.reshape(-1)[:2] = [-32768, 32767], [32767, -32768]
    wide = lambda t: t.astype(np.int64)  # noqa: E731
    np.testing.assert_array_equal(to_host(espdl().add_s16(to_dev(a), to_dev(b))),
                                  np.clip(wide(a) + wide(b), -32768, 32767).astype(np.int16))
    np.testing.assert_array_equal(to_host(espdl().sub_s16(to_dev(a), to_dev(b))),
                                  np.clip(wide(a) - wide(b), -32768, 32767).astype(np.int16))
    af, bf = (np.ascontiguousarray(t) for t in np.broadcast_arrays(a, b))  # the oracle multiplies equal shapes
    for shift, rm in ((14, 0), (15, 1), (3, 1)):
        np.testing.assert_array_equal(to_host(espdl().mul_s16(to_dev(a), to_dev(b), shift, rm)), oracle.mul_s16(af, bf, shift, rm))
    a8, b8 = _rand(rng, sa, np.int8), _rand(rng, sb, np.int8)
    np.testing.assert_array_equal(to_host(espdl().sub_s8(to_dev(a8), to_dev(b8))),
                                  np.clip(wide(a8) - wide(b8), -128, 127).astype(np.int8))


def test_sub_s16(oracle):
    announce("sub_s16")
    rng = np.random.default_rng(63)
    a, b = _rand(rng, (2, 286, 800), np.int16), _rand(rng, (2, 1, 800), np.int16)
    want = np.clip(a.astype(np.int32) - b.astype(np.int32), -32768, 32767).astype(np.int16)
    np.testing.assert_array_equal(to_host(espdl().sub_s16(to_dev(a), to_dev(b))), want)
    np.testing.assert_array_equal(to_host(espdl().sub_s16(to_dev(a), to_dev(a))), oracle.sub_s16(a, a))


@pytest.mark.parametrize("shapes", [((4, 3000), (4, 3000)), ((2, 800), (1,)), ((4, 300), (4, 1)), ((1,), (4, 300)),
                                    ((4, 1), (4, 300))], ids=str)
@pytest.mark.parametrize("shift", [-3, 0, 3, 9])
def test_div_s16(oracle, shapes, shift):
    announce(f"div_s16 {shapes} shift={shift}")
    rng = np.random.default_rng(64)
    a, b = _rand(rng, shapes[0], np.int16), _rand(rng, shapes[1], np.int16)
    a.flat[0] = 0
    b.flat[-1] = 0
    got = to_host(espdl().div_s16(to_dev(a), to_dev(b), shift))
    np.testing.assert_array_equal(got, oracle.div_s16(a, b, shift))


def test_sub_s8(oracle):
    announce("sub_s8")
    rng = np.random.default_rng(65)
    a, b = _rand(rng, (2, 286, 800), np.int8), _rand(rng, (2, 1, 800), np.int8)
    want = np.clip(a.astype(np.int32) - b.astype(np.int32), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(to_host(espdl().sub_s8(to_dev(a), to_dev(b))), want)
    np.testing.assert_array_equal(to_host(espdl().sub_s8(to_dev(a), to_dev(a))), oracle.sub_s8(a, a))


@pytest.mark.parametrize("shapes", [((4, 3000), (4, 3000)), ((2, 800), (1,)), ((4, 300), (4, 1)), ((1,), (4, 300)),
                                    ((4, 1), (4, 300)), ((1, 1), (1,))], ids=str)
@pytest.mark.parametrize("shift", [-3, 0, 3, 6])
def test_div_s8(oracle, shapes, shift):
    """Loop forms and both table forms of the reference, zero operands included (a one-element divisor of zero is
    undefined there and left out)."""
    announce(f"div_s8 {shapes} shift={shift}")
    rng = np.random.default_rng(66)
    for scalar0 in (0, 1):
        a, b = _rand(rng, shapes[0], np.int8), _rand(rng, shapes[1], np.int8)
        a.flat[0] = 0 if scalar0 == 0 else 37
        b.flat[-1] = 0
        if b.size == 1:
            b.flat[0] = -5
        b.flat[0] = 0 if b.size > 1 else b.flat[0]
        got = to_host(espdl().div_s8(to_dev(a), to_dev(b), shift))
        np.testing.assert_array_equal(got, oracle.div_s8(a, b, shift))


def test_div_s8_one_element_operands(oracle):
    announce("div_s8 one-element operands")
    zero = np.array([0], np.int8)
    got = to_host(espdl().div_s8(to_dev(zero), to_dev(zero), 0))
    np.testing.assert_array_equal(got, oracle.div_s8(zero, zero, 0))
    assert got[0] == -128
    z16 = np.array([0], np.int16)
    assert to_host(espdl().div_s16(to_dev(z16), to_dev(z16), 0))[0] == 0
