"""Pins the oracle's Softmax (int8 -> float32), QuantizeLinear / DequantizeLinear and activation x activation
MatMul against library routines and exact arithmetic.  No GPU needed."""
from fractions import Fraction

import numpy as np
import pytest
from scipy import special


def _rand(rng, shape, dtype=np.int8):
    info = np.iinfo(dtype)
    return rng.integers(info.min, info.max + 1, size=shape).astype(dtype)


@pytest.mark.parametrize("axis", [-1, 0, 1, 2])
@pytest.mark.parametrize("in_exp", [-5, -3, 0])
def test_softmax_is_scipy_softmax_within_float32(oracle, axis, in_exp):
    """Closed form: the real softmax of the dequantized values.  The reference subtracts no maximum on its
    int8 path, so at exponent 0 float32 overflows above e^88 and underflows below e^-87; the inputs stay
    inside that range here."""
    rng = np.random.default_rng(31)
    x = _rand(rng, (3, 4, 9, 6))
    if in_exp == 0:
        x = np.clip(x, -60, 60).astype(np.int8)
    got = oracle.softmax_s8(x, axis, in_exp)
    want = special.softmax(x.astype(np.float64) * 2.0 ** in_exp, axis=axis)
    assert got.dtype == np.float32 and got.shape == x.shape
    np.testing.assert_allclose(got, want, rtol=2e-6, atol=1e-30)  # float32 underflows below ~1e-38
    np.testing.assert_allclose(got.sum(axis=axis), 1.0, atol=1e-5)


def test_softmax_sums_in_index_order_in_float32(oracle):
    """The order of the float32 additions is part of the result.  numpy's cumsum adds strictly left to
    right, so its last element is the reference's row sum; a pairwise or float64 sum differs in the low
    bits on rows this long.  The table entries come from the C library's expf called directly."""
    import ctypes
    import ctypes.util
    libm = ctypes.CDLL(ctypes.util.find_library("m"))
    libm.expf.restype = ctypes.c_float
    libm.expf.argtypes = [ctypes.c_float]
    scale = np.float32(2.0 ** -3)
    table = np.array([libm.expf(float(scale * np.float32(q))) for q in range(-128, 128)], dtype=np.float32)
    rng = np.random.default_rng(32)
    x = _rand(rng, (64, 400))
    e = table[x.astype(np.int32) + 128]
    row_sum = np.cumsum(e, axis=1, dtype=np.float32)[:, -1:]
    np.testing.assert_array_equal(oracle.softmax_s8(x, -1, -3), e / row_sum)
    # the check above has teeth: a float64 row sum gives different float32 quotients somewhere
    assert not np.array_equal(e / e.sum(axis=1, dtype=np.float64, keepdims=True).astype(np.float32), e / row_sum)


def test_softmax_axis_views_agree(oracle):
    """Softmax along a middle axis equals softmax along the last axis of the transposed tensor, bit for bit."""
    rng = np.random.default_rng(33)
    x = _rand(rng, (2, 5, 7, 3))
    a = oracle.softmax_s8(x, 1, -4)
    b = oracle.softmax_s8(np.ascontiguousarray(np.moveaxis(x, 1, -1)), -1, -4)
    np.testing.assert_array_equal(a, np.moveaxis(b, -1, 1))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("out_exp", [-9, -7, 0, 2])
def test_quantize_is_round_half_up_of_the_scaled_value(oracle, dtype, out_exp):
    rng = np.random.default_rng(34)
    info = np.iinfo(dtype)
    scale = 2.0 ** out_exp
    x = (rng.standard_normal(4000) * info.max * scale * 0.7).astype(np.float32)
    # exact ties and the saturation edges
    ties = ((np.arange(-40, 40) + 0.5) * scale).astype(np.float32)
    edges = np.array([info.max + 0.49, info.max + 0.5, info.min - 0.5, info.min - 0.51, 3e4, -3e4], dtype=np.float64) * scale
    x = np.concatenate([x, ties, edges.astype(np.float32)])
    got = oracle.quantize_f32(x, out_exp, dtype)
    want = [min(max(int(np.floor(Fraction(float(v)) / Fraction(scale) + Fraction(1, 2))), info.min), info.max) for v in x]
    np.testing.assert_array_equal(got, np.array(want, dtype=dtype))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
def test_dequantize_is_exact_scaling(oracle, dtype):
    rng = np.random.default_rng(35)
    x = _rand(rng, (5, 33), dtype)
    for e in (-12, -3, 0, 4):
        np.testing.assert_array_equal(oracle.dequantize_f32(x, e), (x.astype(np.float64) * 2.0 ** e).astype(np.float32))


def _shift_round(v, shift, half_even):
    v = np.asarray(v, dtype=np.int64)
    if shift <= 0:
        return v << -shift
    q, r = v >> shift, v & ((1 << shift) - 1)
    h = 1 << (shift - 1)
    up = (r > h) | ((r == h) & ((q & 1) == 1)) if half_even else (r >= h)
    return q + up


@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
@pytest.mark.parametrize("shapes", [((2, 3, 5, 8), (2, 3, 8, 6)), ((1, 3, 5, 8), (2, 1, 8, 6)), ((4, 5, 16), (4, 16, 3)),
                                    ((7, 9), (9, 2))], ids=str)
def test_matmul_is_numpy_matmul_then_shift_round(oracle, shapes, round_mode):
    rng = np.random.default_rng(36)
    a, b = _rand(rng, shapes[0]), _rand(rng, shapes[1])
    exact = a.astype(np.int64) @ b.astype(np.int64)
    for shift, act in ((7, oracle.LINEAR), (10, oracle.RELU), (1, oracle.LINEAR), (13, oracle.LINEAR)):
        got = oracle.matmul_s8(a, b, shift, act, round_mode)
        want = _shift_round(exact, shift, round_mode == 1)
        if act == oracle.RELU:
            want = np.maximum(want, 0)
        np.testing.assert_array_equal(got, np.clip(want, -128, 127).astype(np.int8))
    assert got.shape == exact.shape


def test_matmul_transposed_operand_is_not_confused(oracle):
    """a x b differs from a x b^T for a square b: guards against reading the second operand [n][k]."""
    rng = np.random.default_rng(37)
    a, b = _rand(rng, (6, 6)), _rand(rng, (6, 6))
    got = oracle.matmul_s8(a, b, 8)
    np.testing.assert_array_equal(got, np.clip(_shift_round(a.astype(np.int64) @ b.astype(np.int64), 8, False), -128, 127))
    assert not np.array_equal(got, np.clip(_shift_round(a.astype(np.int64) @ b.T.astype(np.int64), 8, False), -128, 127))


@pytest.mark.parametrize("p4_ties", [False, True], ids=["ties_up", "ties_even"])
@pytest.mark.parametrize("entries", [65536, 65537, 2049, 257, 3])
def test_lut_s16_takes_the_nearest_sample(oracle, entries, p4_ties):
    """All 65536 inputs against exact rational arithmetic: index = round((x + 32768) / step)."""
    rng = np.random.default_rng(38)
    table = _rand(rng, (entries,), np.int16)
    x = np.arange(-32768, 32768, dtype=np.int16)
    step = 65536 // (entries - 1)
    want = np.empty(65536, dtype=np.int16)
    for i, v in enumerate(range(65536)):
        q = Fraction(v, step)
        idx = int(np.floor(q))
        frac = q - idx
        if frac > Fraction(1, 2) or (frac == Fraction(1, 2) and (idx % 2 == 1 if p4_ties else True)):
            idx += 1
        want[i] = table[idx]
    np.testing.assert_array_equal(oracle.lut_s16(x, table, p4_ties), want)


def test_lut_s16_rejects_odd_table_sizes(oracle):
    with pytest.raises(AssertionError):
        oracle.lut_s16(np.zeros(4, dtype=np.int16), np.zeros(1000, dtype=np.int16))


def test_add_s16_saturates(oracle):
    rng = np.random.default_rng(50)
    a, b = _rand(rng, (3, 1000), np.int16), _rand(rng, (3, 1000), np.int16)
    want = np.clip(a.astype(np.int32) + b.astype(np.int32), -32768, 32767).astype(np.int16)
    np.testing.assert_array_equal(oracle.add_s16(a, b), want)
    np.testing.assert_array_equal(oracle.add_s16(a, b[:1, :1]), np.clip(a.astype(np.int32) + int(b[0, 0]), -32768, 32767))


@pytest.mark.parametrize("shift", [0, 7, 12, 15, 20])
def test_mul_s16_goes_through_float32(oracle, shift):
    """Half up: the product passes through float32 (numpy's int64 -> float32 conversion rounds to nearest
    even, as the C conversion does), is scaled by an exact power of two and rounded half up in exact
    rationals.  Half even: integer shift-round of the exact product."""
    rng = np.random.default_rng(51)
    a, b = _rand(rng, (20000,), np.int16), _rand(rng, (20000,), np.int16)
    a[:4], b[:4] = [-32768, 32767, -32768, 4097], [-32768, 32767, 32767, 4099]
    prod = a.astype(np.int64) * b.astype(np.int64)
    as_f32 = prod.astype(np.float32)
    want = [min(max(int(np.floor(Fraction(float(v)) / (1 << shift) + Fraction(1, 2))), -32768), 32767) for v in as_f32]
    np.testing.assert_array_equal(oracle.mul_s16(a, b, shift, oracle.ROUND_HALF_UP), np.array(want, dtype=np.int16))
    if shift > 0:
        even = np.clip(_shift_round(prod, shift, True), -32768, 32767).astype(np.int16)
        np.testing.assert_array_equal(oracle.mul_s16(a, b, shift, oracle.ROUND_HALF_EVEN), even)
    if shift == 0:  # above 2^24 the float32 detour is visible: some products change
        assert np.any(as_f32.astype(np.int64) != prod)


def test_avg_pool_and_reduce_mean_s16_are_exact_means_away_from_ties(oracle):
    rng = np.random.default_rng(52)
    x = _rand(rng, (2, 9, 8, 5), np.int16)
    got = oracle.avg_pool_s16(x, (3, 3), (2, 2), (1, 1, 1, 1), -10, -9)
    pad = np.pad(x.astype(np.int64), ((0, 0), (1, 1), (1, 1), (0, 0)))
    checked = 0
    for oy in range(got.shape[1]):
        for ox in range(got.shape[2]):
            s = pad[:, 2 * oy:2 * oy + 3, 2 * ox:2 * ox + 3].sum(axis=(1, 2))
            for n in range(2):
                for c in range(5):
                    exact = Fraction(int(s[n, c]), 9) / 2  # 2^-10 / 2^-9
                    if abs((exact - np.floor(exact)) - Fraction(1, 2)) > Fraction(1, 1000):
                        assert got[n, oy, ox, c] == min(max(int(np.floor(exact + Fraction(1, 2))), -32768), 32767)
                        checked += 1
    assert checked > 150
    r = oracle.reduce_mean_s16(x, [1, 2], True, -10, -12)
    s = x.astype(np.int64).sum(axis=(1, 2))
    for n in range(2):
        for c in range(5):
            exact = Fraction(int(s[n, c]), 72) * 4
            if abs((exact - np.floor(exact)) - Fraction(1, 2)) > Fraction(1, 1000):
                assert r[n, 0, 0, c] == min(max(int(np.floor(exact + Fraction(1, 2))), -32768), 32767)


def test_sub_s16_saturates(oracle):
    rng = np.random.default_rng(53)
    a, b = _rand(rng, (3, 1000), np.int16), _rand(rng, (3, 1000), np.int16)
    want = np.clip(a.astype(np.int32) - b.astype(np.int32), -32768, 32767).astype(np.int16)
    np.testing.assert_array_equal(oracle.sub_s16(a, b), want)


@pytest.mark.parametrize("shapes,form", [(((4, 300), (4, 300)), 0), (((4, 300), (1,)), 1), (((4, 300), (4, 1)), 1),
                                         (((1,), (4, 300)), 2), (((4, 1), (4, 300)), 2)], ids=str)
@pytest.mark.parametrize("shift", [-3, 0, 5])
def test_div_s16_is_float32_arithmetic_in_the_reference_order(oracle, shapes, form, shift):
    """IEEE float32 operations in numpy, in the order of the loop that the broadcast selects; and within one
    unit of the exact quotient, which a wrong shift sign or swapped operands would miss by far."""
    rng = np.random.default_rng(54)
    a, b = _rand(rng, shapes[0], np.int16), _rand(rng, shapes[1], np.int16)
    a.flat[0] = 0
    b.flat[-1] = 0
    assert oracle.div_form(shapes[0], shapes[1]) == form
    got = oracle.div_s16(a, b, shift)
    af, bf = np.broadcast_arrays(a.astype(np.float32), b.astype(np.float32))
    r = np.float32(2.0 ** -shift)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = af * (r / bf) if form == 1 else ((af * r) / bf if form == 2 else af * r / bf)
    q = np.floor(v.astype(np.float64) + 0.5)
    want = np.clip(np.nan_to_num(q, nan=0.0, posinf=32767, neginf=-32768), -32768, 32767).astype(np.int16)
    want = np.where(af == 0, 0, np.where(bf == 0, np.where(af > 0, 32767, -32768), want)).astype(np.int16)
    np.testing.assert_array_equal(got, want)
    ok = (af != 0) & (bf != 0)
    exact = af[ok].astype(np.float64) * 2.0 ** -shift / bf[ok].astype(np.float64)
    inside = np.abs(exact) < 32000
    assert np.all(np.abs(got[ok][inside] - exact[inside]) <= 1.0)


def test_sub_s8_saturates(oracle):
    rng = np.random.default_rng(55)
    a, b = _rand(rng, (3, 1000), np.int8), _rand(rng, (3, 1000), np.int8)
    want = np.clip(a.astype(np.int32) - b.astype(np.int32), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(oracle.sub_s8(a, b), want)
    np.testing.assert_array_equal(oracle.sub_s8(a, np.array([-128], np.int8)),
                                  np.clip(a.astype(np.int32) + 128, -128, 127).astype(np.int8))


@pytest.mark.parametrize("shapes,form", [(((4, 300), (4, 300)), 0), (((4, 300), (4, 1)), 1), (((4, 1), (4, 300)), 2)],
                         ids=str)
@pytest.mark.parametrize("shift", [-3, 0, 4])
def test_div_s8_loop_forms_are_float32_arithmetic_in_the_reference_order(oracle, shapes, form, shift):
    """No one-element operand, so the reference runs its loops (dl_base_div.cpp:92-112, 141-163, 175-195): IEEE
    float32 operations in numpy in the same order, and within one unit of the exact quotient."""
    rng = np.random.default_rng(56)
    a, b = _rand(rng, shapes[0], np.int8), _rand(rng, shapes[1], np.int8)
    a.flat[0] = 0
    b.flat[-1] = 0
    got = oracle.div_s8(a, b, shift)
    af, bf = np.broadcast_arrays(a.astype(np.float32), b.astype(np.float32))
    r = np.float32(2.0 ** -shift)
    with np.errstate(divide="ignore", invalid="ignore"):
        v = af * (r / bf) if form == 1 else ((af * r) / bf if form == 2 else af * r / bf)
    q = np.floor(v.astype(np.float64) + 0.5)
    want = np.clip(np.nan_to_num(q, nan=0.0, posinf=127, neginf=-128), -128, 127).astype(np.int8)
    want = np.where(af == 0, 0, np.where(bf == 0, np.where(af > 0, 127, -128), want)).astype(np.int8)
    np.testing.assert_array_equal(got, want)
    ok = (af != 0) & (bf != 0)
    exact = af[ok].astype(np.float64) * 2.0 ** -shift / bf[ok].astype(np.float64)
    inside = np.abs(exact) < 120
    assert np.all(np.abs(got[ok][inside] - exact[inside]) <= 1.0)


@pytest.mark.parametrize("shift", [-3, 0, 2, 5])
@pytest.mark.parametrize("scalar", [-128, -77, -1, 0, 1, 5, 127])
def test_div_s8_table_forms_follow_create_div_lut(oracle, scalar, shift):
    """A one-element operand makes the reference read a table (dl_base_div.cpp:8-46): rebuilt here entry by entry
    in numpy float32 from its two expressions, over all 256 values of the other operand."""
    r = np.float32(2.0 ** -shift)
    other = np.arange(-128, 128, dtype=np.int8).reshape(2, 128)
    i = other.astype(np.float32)
    one = np.array([scalar], np.int8)

    def rounded(v):
        return np.clip(np.floor(v.astype(np.float64) + 0.5), -128, 127).astype(np.int8)

    # one-element dividend: table[i] = round((in0 * rescale) / i), entry 0 by the sign of in0 * rescale
    in0_float = np.float32(scalar) * r
    with np.errstate(divide="ignore", invalid="ignore"):
        want = rounded(np.where(other == 0, np.float32(1), in0_float / i))
    want = np.where(other == 0, 127 if in0_float > 0 else -128, want).astype(np.int8)
    np.testing.assert_array_equal(oracle.div_s8(one, other, shift), want)
    # one-element divisor: table[i] = round(i * (rescale / in1)), entry 0 is 0
    if scalar != 0:
        want = rounded(i * (r / np.float32(scalar)))
        want = np.where(other == 0, 0, want).astype(np.int8)
        np.testing.assert_array_equal(oracle.div_s8(other, one, shift), want)


def test_div_s8_one_element_result_uses_the_dividend_table(oracle):
    # both operands have one element: create_div_lut and elemwise_div test the dividend first
    assert oracle.div_s8(np.array([0], np.int8), np.array([0], np.int8), 0)[0] == -128
    assert oracle.div_s8(np.array([[0]], np.int8), np.array([[0, 3]], np.int8), 0).tolist() == [[-128, 0]]
    assert oracle.div_s8(np.array([[0, 3]], np.int8), np.array([[0, 3]], np.int8), 0).tolist() == [[0, 1]]
    assert oracle.div_form((1,), (1,), all_ones=2) == 2 and oracle.div_form((1,), (1,)) == 1
