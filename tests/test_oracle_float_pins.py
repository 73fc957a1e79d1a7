"""Pins of the oracle functions that the reference defines through float32 arithmetic: GlobalAveragePool,
AveragePool and ReduceMean (int8 and int16), and the per-element activation functions.

The float32 sequence of the reference is IEEE-deterministic step by step, so it can be replayed with numpy
scalars of the same widths, operation by operation, in the reference's order:

  pooling     scale = (DL_SCALE(in) * (1.f / area)) * DL_RESCALE(out), one float32 multiply of the integer
              sum converted to float32, then tool::round = floorf(float(double(v) + 0.5))
              (esp-dl/dl/base/dl_base_avg_pool2d.cpp:34-35, 50-53; esp-dl/dl/tool/src/dl_tool.cpp:72-75)
  ReduceMean  ((float(sum) * DL_SCALE(in)) / float(count)) * DL_RESCALE(out), the same rounding
              (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:38-42)

Every reachable sum is enumerated for int8 (|sum| <= 128 * area) and a dense sample plus every multiple
of area / 2 (the exact ties and their neighbours) for int16, ties and near-ties included.  The same sums are
also rounded in exact rational arithmetic; the places where float32 and exact rounding disagree are counted
and must all sit within float32 rounding error of a tie (that is the only thing float32 can change)."""
import ctypes
import ctypes.util
import math
from fractions import Fraction

import numpy as np
import pytest

F = np.float32


def dl_scale(e):
    return F(1 << e) if e > 0 else F(1.0) / F(1 << -e)


def dl_rescale(e):
    return F(1.0) / F(1 << e) if e > 0 else F(1 << -e)


def tool_round_f32(v):
    """tool::round(float): value + 0.5 is a double addition, floorf takes it back as a float."""
    v = np.asarray(v, dtype=np.float32)
    return np.floor((v.astype(np.float64) + 0.5).astype(np.float32)).astype(np.int64)


def pool_f32(sums, area, in_exp, out_exp, lo, hi):
    scale = F(F(dl_scale(in_exp) * F(F(1.0) / F(area))) * dl_rescale(out_exp))
    v = sums.astype(np.float32) * scale
    return np.clip(tool_round_f32(v), lo, hi)


def mean_f32(sums, count, in_exp, out_exp, lo, hi):
    v = sums.astype(np.float32) * dl_scale(in_exp)
    v = (v / F(count)).astype(np.float32)
    v = v * dl_rescale(out_exp)
    return np.clip(tool_round_f32(v), lo, hi)


def exact_half_up(sums, area, in_exp, out_exp, lo, hi):
    """floor(sum * 2^(in - out) / area + 1/2) in exact integers."""
    d = in_exp - out_exp
    num = sums.astype(object) * (2 ** d if d >= 0 else 1)
    den = area * (1 if d >= 0 else 2 ** -d)
    out = np.array([(2 * int(n) + den) // (2 * den) for n in num], dtype=np.int64)
    return np.clip(out, lo, hi)


def tie_distance(sums, area, in_exp, out_exp):
    """|frac(sum * 2^(in - out) / area) - 1/2| as floats (only used to describe where disagreements sit)."""
    v = sums.astype(np.float64) * 2.0 ** (in_exp - out_exp) / area
    return np.abs(v - np.floor(v) - 0.5)


def spread_s8(sums, area):
    """int8 values, `area` per sum, that add up to each sum: shape [area, len(sums)]."""
    base = np.floor_divide(sums, area)
    rem = sums - base * area
    x = np.repeat(base[None, :], area, axis=0) + (np.arange(area)[:, None] < rem[None, :])
    assert x.min() >= -128 and x.max() <= 127 and np.array_equal(x.sum(axis=0), sums)
    return x.astype(np.int8)


def spread_s16(sums, area):
    base = np.floor_divide(sums, area)
    rem = sums - base * area
    x = np.repeat(base[None, :], area, axis=0) + (np.arange(area)[:, None] < rem[None, :])
    assert x.min() >= -32768 and x.max() <= 32767 and np.array_equal(x.sum(axis=0), sums)
    return x.astype(np.int16)


EXP_PAIRS = [(-5, -5 - d) for d in range(-4, 5)] + [(2, 0), (0, 3), (-7, -3)]
AREAS = [(7, 7), (3, 3), (2, 3), (2, 2), (1, 2), (10, 10), (14, 14), (5, 1)]

# Filled by the tests and printed with `pytest -s`: (function, area, in_exp, out_exp) -> number of sums on
# which float32 rounding and exact-rational rounding differ.  The assertions bound them.
DISAGREE = {}


@pytest.mark.parametrize("hw", AREAS, ids=lambda v: "%dx%d" % v)
def test_global_avg_pool_s8_every_sum(oracle, hw):
    """Every reachable channel sum, ties and near-ties included, for nine exponent differences."""
    h, w = hw
    area = h * w
    sums = np.arange(-128 * area, 127 * area + 1, dtype=np.int64)
    x = spread_s8(sums, area).reshape(1, h, w, len(sums))
    for in_exp, out_exp in EXP_PAIRS:
        got = oracle.global_avg_pool_s8(x, in_exp, out_exp).reshape(-1).astype(np.int64)
        want = pool_f32(sums, area, in_exp, out_exp, -128, 127)
        np.testing.assert_array_equal(got, want, err_msg="area %d exps %d %d" % (area, in_exp, out_exp))
        exact = exact_half_up(sums, area, in_exp, out_exp, -128, 127)
        diff = got != exact
        DISAGREE[("gap_s8", area, in_exp, out_exp)] = int(diff.sum())
        if diff.any():
            # float32 can only move a result that sits within its rounding error of a tie, and by one unit
            assert np.abs(got - exact)[diff].max() == 1
            assert tie_distance(sums[diff], area, in_exp, out_exp).max() < 2e-5 * max(1.0, 2.0 ** (in_exp - out_exp) * 128)
        assert len(np.unique(got)) > 16 or in_exp - out_exp <= -3


def test_global_avg_pool_s8_exact_ties_round_up(oracle):
    """Exact ties that float32 represents exactly (power-of-two areas): half goes up, also for negatives."""
    sums = np.arange(-128 * 4, 127 * 4 + 1, dtype=np.int64)
    x = spread_s8(sums, 4).reshape(1, 2, 2, -1)
    got = oracle.global_avg_pool_s8(x, -5, -5).reshape(-1)
    np.testing.assert_array_equal(got, np.floor(sums / 4.0 + 0.5))
    assert got[sums == -2][0] == 0 and got[sums == 2][0] == 1 and got[sums == -6][0] == -1


@pytest.mark.parametrize("k", [(2, 2), (3, 3), (2, 3), (1, 2), (7, 7)], ids=lambda v: "%dx%d" % v)
def test_avg_pool_s8_every_sum(oracle, k):
    """The pooling form: one window per output position, every reachable window sum."""
    area = k[0] * k[1]
    sums = np.arange(-128 * area, 127 * area + 1, dtype=np.int64)
    x = spread_s8(sums, area).reshape(1, k[0], k[1], len(sums))
    for in_exp, out_exp in EXP_PAIRS:
        got = oracle.avg_pool_s8(x, k, (1, 1), (0, 0, 0, 0), in_exp, out_exp).reshape(-1).astype(np.int64)
        np.testing.assert_array_equal(got, pool_f32(sums, area, in_exp, out_exp, -128, 127))
    # a clipped window keeps the divisor k_h * k_w on this path (dl_base_pool2d.hpp:132): pad one side
    if k[1] > 1:
        got = oracle.avg_pool_s8(x, k, (1, 1), (0, 0, 0, k[1] - 1), -5, -5)[0, 0, -1].astype(np.int64)
        last_column = x[0, :, -1:, :].astype(np.int64).sum(axis=(0, 1))
        np.testing.assert_array_equal(got, pool_f32(last_column, area, -5, -5, -128, 127))


@pytest.mark.parametrize("count", [49, 9, 6, 4, 2, 100, 40, 3])
def test_reduce_mean_s8_every_sum(oracle, count):
    sums = np.arange(-128 * count, 127 * count + 1, dtype=np.int64)
    x = spread_s8(sums, count).T.copy()  # [n_sums, count]: reduce the last axis
    for in_exp, out_exp in EXP_PAIRS:
        got = oracle.reduce_mean_s8(x, [1], False, in_exp, out_exp).reshape(-1).astype(np.int64)
        want = mean_f32(sums, count, in_exp, out_exp, -128, 127)
        np.testing.assert_array_equal(got, want, err_msg="count %d exps %d %d" % (count, in_exp, out_exp))
        exact = exact_half_up(sums, count, in_exp, out_exp, -128, 127)
        diff = got != exact
        DISAGREE[("reduce_mean_s8", count, in_exp, out_exp)] = int(diff.sum())
        if diff.any():
            assert np.abs(got - exact)[diff].max() == 1
            assert tie_distance(sums[diff], count, in_exp, out_exp).max() < 2e-5 * max(1.0, 2.0 ** (in_exp - out_exp) * 128)


def _s16_sums(area, rng):
    lim_lo, lim_hi = -32768 * area, 32767 * area
    dense = rng.integers(lim_lo, lim_hi + 1, size=60000)
    # every exact tie of sum / area for the unit exponent difference is an odd multiple of area / 2;
    # take those multiples that exist and their neighbours
    step = area if area % 2 else area // 2
    ties = np.arange(lim_lo // step, lim_hi // step + 1, max(1, (lim_hi - lim_lo) // step // 40000)) * step
    near = np.concatenate([ties - 1, ties, ties + 1])
    s = np.unique(np.concatenate([dense, near, [lim_lo, lim_hi, 0, -1, 1]]))
    return s[(s >= lim_lo) & (s <= lim_hi)].astype(np.int64)


@pytest.mark.parametrize("k", [(2, 2), (3, 3), (2, 3), (7, 7), (1, 2)], ids=lambda v: "%dx%d" % v)
def test_avg_pool_s16_dense_sums_and_all_tie_multiples(oracle, k):
    area = k[0] * k[1]
    sums = _s16_sums(area, np.random.default_rng(area))
    x = spread_s16(sums, area).reshape(1, k[0], k[1], len(sums))
    for in_exp, out_exp in EXP_PAIRS:
        got = oracle.avg_pool_s16(x, k, (1, 1), (0, 0, 0, 0), in_exp, out_exp).reshape(-1).astype(np.int64)
        want = pool_f32(sums, area, in_exp, out_exp, -32768, 32767)
        np.testing.assert_array_equal(got, want, err_msg="area %d exps %d %d" % (area, in_exp, out_exp))
        exact = exact_half_up(sums, area, in_exp, out_exp, -32768, 32767)
        diff = got != exact
        DISAGREE[("avg_pool_s16", area, in_exp, out_exp)] = int(diff.sum())
        # int16 sums need up to 21 bits and the scale is rounded to 24: a unit of difference is possible
        # anywhere the scaled value exceeds 2^23 ulps of precision near a tie, never more than one unit
        if diff.any():
            assert np.abs(got - exact)[diff].max() == 1


@pytest.mark.parametrize("count", [4, 9, 49, 40, 6])
def test_reduce_mean_s16_dense_sums_and_all_tie_multiples(oracle, count):
    sums = _s16_sums(count, np.random.default_rng(100 + count))
    x = spread_s16(sums, count).T.copy()
    for in_exp, out_exp in EXP_PAIRS:
        got = oracle.reduce_mean_s16(x, [1], False, in_exp, out_exp).reshape(-1).astype(np.int64)
        want = mean_f32(sums, count, in_exp, out_exp, -32768, 32767)
        np.testing.assert_array_equal(got, want, err_msg="count %d exps %d %d" % (count, in_exp, out_exp))
        exact = exact_half_up(sums, count, in_exp, out_exp, -32768, 32767)
        diff = got != exact
        DISAGREE[("reduce_mean_s16", count, in_exp, out_exp)] = int(diff.sum())
        if diff.any():
            assert np.abs(got - exact)[diff].max() == 1


def test_where_float32_and_exact_rounding_differ(oracle):
    """The summary the design notes quote.  On the GlobalAveragePool of MobileNetV2 (7 x 7, equal
    exponents) float32 rounding and exact rounding agree on every reachable sum."""
    sums = np.arange(-128 * 49, 127 * 49 + 1, dtype=np.int64)
    x = spread_s8(sums, 49).reshape(1, 7, 7, -1)
    for d in range(-4, 5):
        got = oracle.global_avg_pool_s8(x, -5, -5 - d).reshape(-1).astype(np.int64)
        exact = exact_half_up(sums, 49, -5, -5 - d, -128, 127)
        n = int((got != exact).sum())
        print("gap 7x7 exponent difference %+d: %d of %d sums differ from exact rounding %s"
              % (d, n, len(sums), sums[got != exact][:8].tolist()))
        if d <= 0:
            assert n == 0  # an odd divisor has no exact tie and nothing lands within float32 error of one


# ------------------------------------------------------------------------------------------------------
# activation functions evaluated in float32 per element
# ------------------------------------------------------------------------------------------------------
_libm = ctypes.CDLL(ctypes.util.find_library("m"))
for _n in ("expf", "logf", "sqrtf"):
    getattr(_libm, _n).restype = ctypes.c_float
    getattr(_libm, _n).argtypes = [ctypes.c_float]


def _libm_map(name, x):
    fn = getattr(_libm, name)
    with np.errstate(all="ignore"):
        return np.array([fn(float(v)) for v in x], dtype=np.float32)


def _sigmoid_f32(x):
    """1.0 / (1.0 + expf(-x)) evaluated in double, returned as float (esp-dl/dl/math/include/dl_math.hpp:200-203)."""
    e = _libm_map("expf", -x)
    with np.errstate(all="ignore"):
        return (1.0 / (1.0 + e.astype(np.float64))).astype(np.float32)


def unary_f32(op, q, in_exp, out_exp, alpha, beta):
    """The reference's expression per operator with numpy scalars of the same widths; transcendental
    functions from the C library (the only part that is not IEEE-defined)."""
    x = q.astype(np.float32) * dl_scale(in_exp)
    out_scale = dl_rescale(out_exp)
    a, b = F(alpha), F(beta)
    with np.errstate(all="ignore"):
        if op == "Sigmoid":
            v = _sigmoid_f32(x) * out_scale
        elif op == "Tanh":
            t = (2 * _sigmoid_f32(F(2) * x).astype(np.float64) - 1).astype(np.float32)
            v = t * out_scale
        elif op == "HardSwish":
            gate = np.clip(0.166667 * x.astype(np.float64) + 0.5, 0, 1)
            v = (gate * x.astype(np.float64)).astype(np.float32) * out_scale
        elif op == "Elu":
            neg = ((a * (_libm_map("expf", x) - F(1))).astype(np.float32) * out_scale).astype(np.float32)
            v = np.where(x >= 0, x * out_scale, neg)
        elif op == "Exp":
            v = _libm_map("expf", x) * out_scale
        elif op == "Log":
            v = _libm_map("logf", x) * out_scale
        elif op == "Sqrt":
            v = _libm_map("sqrtf", x) * out_scale
        elif op == "LeakyRelu":
            v = np.where(x >= 0, x * out_scale, ((x * out_scale).astype(np.float32) * a).astype(np.float32))
        elif op == "Swish":
            v = (_sigmoid_f32(x) * x).astype(np.float32) * out_scale
        elif op == "HardSigmoid":
            v = np.clip((a * x).astype(np.float32) + b, F(0), F(1)).astype(np.float32) * out_scale
        else:
            raise KeyError(op)
    return np.asarray(v, dtype=np.float32)


UNARY_CASES = [("Sigmoid", -5, -7, None, None), ("Sigmoid", -4, -7, None, None), ("Tanh", -6, -7, None, None),
               ("HardSwish", -4, -4, None, None), ("Elu", -5, -5, 0.75, None), ("Elu", -4, -4, None, None),
               ("Exp", -6, -5, None, None), ("Log", -4, -5, None, None), ("Sqrt", -3, -4, None, None),
               ("LeakyRelu", -3, -3, 0.1, None), ("LeakyRelu", -3, -4, None, None), ("Swish", -5, -5, None, None),
               ("HardSigmoid", -5, -7, 0.25, 0.5), ("HardSigmoid", -4, -7, None, None)]
LIBM_OPS = ("Sigmoid", "Tanh", "Elu", "Exp", "Log", "Sqrt", "Swish")

# int16 table entries whose exact value lies within 4 float32 ulps of a rounding tie: what a C library whose
# expf / logf differs from this host's in the last places could move by one unit.  Nothing else is open.
OPEN_S16 = {("Sigmoid", -13, -15): 1009, ("Sigmoid", -12, -15): 992, ("Tanh", -14, -15): 4012,
            ("Elu", -13, -13): 187, ("Elu", -12, -12): 136, ("Exp", -14, -13): 535, ("Log", -12, -13): 330,
            ("Sqrt", -11, -12): 350, ("Swish", -13, -13): 515}


def _closed_form(op, x, alpha, beta):
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    with np.errstate(all="ignore"):
        return {"Sigmoid": lambda: sig(x), "Tanh": lambda: np.tanh(x),
                "HardSwish": lambda: np.clip(0.166667 * x + 0.5, 0, 1) * x,
                "Elu": lambda: np.where(x >= 0, x, alpha * (np.exp(x) - 1)), "Exp": lambda: np.exp(x),
                "Log": lambda: np.log(x), "Sqrt": lambda: np.sqrt(x),
                "LeakyRelu": lambda: np.where(x >= 0, x, alpha * x), "Swish": lambda: x * sig(x),
                "HardSigmoid": lambda: np.clip(alpha * x + beta, 0, 1)}[op]()


@pytest.mark.parametrize("bits", [8, 16])
@pytest.mark.parametrize("op,in_exp,out_exp,alpha,beta", UNARY_CASES, ids=lambda v: str(v))
def test_unary_every_entry_in_reference_widths(oracle, op, in_exp, out_exp, alpha, beta, bits):
    """Every table entry equals the float32 / double sequence of the reference replayed in numpy; the entries
    that a different C library could move (within 4 ulps of a tie) are counted: none for int8, the listed
    numbers for int16; every other entry also equals the float64 closed form rounded half up."""
    dt, lo, hi = (np.int8, -128, 127) if bits == 8 else (np.int16, -32768, 32767)
    if bits == 16:
        in_exp, out_exp = in_exp - 8, out_exp - 8
    q = np.arange(lo, hi + 1, dtype=dt)
    da, db = oracle.UNARY_DEFAULTS.get(op, (0.0, 0.0))
    al, be = (da if alpha is None else alpha), (db if beta is None else beta)
    got = oracle.unary(op, q, in_exp, out_exp, alpha, beta).astype(np.int64)
    v = unary_f32(op, q, in_exp, out_exp, al, be)
    ok = np.isfinite(v)
    want = np.clip(tool_round_f32(np.where(ok, v, 0)), lo, hi)
    np.testing.assert_array_equal(got[ok], want[ok])
    # the open set: distance of the exact value from a tie below 4 float32 ulps, inside the output range
    x = q.astype(np.float64) * 2.0 ** in_exp
    exact = _closed_form(op, x, al, be) * 2.0 ** -out_exp
    fin = np.isfinite(exact)
    e = exact[fin]
    dist = np.abs(e - np.floor(e) - 0.5)
    # float32 error model: 4 ulps of the result, or of the operands of the one cancelling subtraction some
    # forms contain (2 * sigmoid(2x) - 1 for Tanh, expf(x) - 1 for Elu), scaled to output units
    cancel = {"Tanh": 2.0, "Elu": abs(al)}.get(op, 0.0) * 2.0 ** -out_exp
    open_ = (dist <= np.maximum(np.maximum(np.abs(e), 1.0), cancel) * 2.0 ** -21) & (np.abs(e) < hi + 1)
    if op in LIBM_OPS:
        if bits == 8:
            assert open_.sum() == 0, q[fin][open_]
        else:
            print("open entries", op, in_exp, out_exp, int(open_.sum()))
            assert open_.sum() == OPEN_S16[(op, in_exp, out_exp)]
    # all other entries: the closed form decides
    clear = ~open_
    np.testing.assert_array_equal(got[fin][clear], np.clip(np.floor(e[clear] + 0.5), lo, hi))


def test_zz_float32_rounding_equals_exact_rounding_on_everything_enumerated():
    """After the tests above have filled the table: on every enumerated sum (all reachable int8 sums for the
    areas and exponent pairs above, the dense int16 samples with all tie multiples) the float32 sequence
    gives the same result as exact-rational round-half-up.  The float32 definition therefore changes no
    result; what the tests above pin is that the oracle follows it operation by operation."""
    if not DISAGREE:
        pytest.skip("run together with the enumeration tests of this file")
    nonzero = {k: v for k, v in DISAGREE.items() if v}
    for k in sorted(nonzero):
        print("float32 != exact:", k, nonzero[k])
    assert not nonzero


def test_int8_results_do_not_depend_on_the_float_evaluation_order():
    """The reference is compiled with -ffast-math (esp-dl/CMakeLists.txt:143), which lets a compiler
    re-associate the scale product or turn the division by `count` into a multiplication.  For int8 that
    cannot change a result except on an exact tie: a sum that is not an exact tie is at least
    1 / (2 * area * 2^max(0, out - in)) away from one, far more than the error of any float32 evaluation
    order (a few ulps of a value that matters only below 129).  Exact ties exist only for even areas; for power-of-two areas
    every order computes them exactly, so the open cases are the exact ties of areas such as 6, 40, 100, 196,
    where this oracle follows the order as written in the source.  The 7 x 7 GlobalAveragePool of
    MobileNetV2 has no exact tie at any exponent difference."""
    for area in sorted({h * w for h, w in AREAS} | {49, 9, 6, 4, 2, 100, 40, 3}):
        for d in range(-4, 5):
            den = area * 2 ** max(0, -d)
            vmax = min(128 * 2.0 ** d, 129.0)  # anything larger saturates whatever its last bits are
            assert 1.0 / (2 * den) > 16 * 2.0 ** -24 * max(vmax, 1.0), (area, d)
            sums = np.arange(-128 * area, 127 * area + 1, dtype=np.int64)
            num = sums * 2 ** max(0, d)
            ties = (2 * num) % (2 * den) == den
            if area % 2 == 1 and d >= -0:
                assert not ties.any()
            if area == 49:
                assert not ties[np.abs(sums) > 0].any() or d < 0
