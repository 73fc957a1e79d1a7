"""Pins of the oracle's float32-per-element activation functions (Sigmoid, Tanh, HardSwish, Elu, Exp, Log, Sqrt,
LeakyRelu, Swish, HardSigmoid, Neg) against their closed forms over every possible input."""
import ctypes
import ctypes.util
import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parents[1]
sys.path.insert(0, str(ROOT / "oracle"))


@pytest.fixture(scope="module")
def oracle():
    import espdl_oracle
    espdl_oracle.lib()
    return espdl_oracle


def _closed_form(op, x, alpha, beta):
    sig = lambda v: 1.0 / (1.0 + np.exp(-v))
    with np.errstate(all="ignore"):
        return {
            "Sigmoid": lambda: sig(x),
            "Tanh": lambda: np.tanh(x),
            "HardSwish": lambda: np.clip(0.166667 * x + 0.5, 0, 1) * x,
            "Elu": lambda: np.where(x >= 0, x, alpha * (np.exp(x) - 1)),
            "Exp": lambda: np.exp(x),
            "Log": lambda: np.log(x),
            "Sqrt": lambda: np.sqrt(x),
            "LeakyRelu": lambda: np.where(x >= 0, x, alpha * x),
            "Swish": lambda: x * sig(x),
            "HardSigmoid": lambda: np.clip(alpha * x + beta, 0, 1),
        }[op]()


CASES = [("Sigmoid", -5, -7, None, None), ("Sigmoid", -4, -7, None, None), ("Tanh", -6, -7, None, None),
         ("HardSwish", -4, -4, None, None), ("Elu", -5, -5, 0.75, None), ("Elu", -4, -4, None, None),
         ("Exp", -6, -5, None, None), ("Log", -4, -5, None, None), ("Sqrt", -3, -4, None, None),
         ("LeakyRelu", -3, -3, 0.1, None), ("LeakyRelu", -3, -4, None, None), ("Swish", -5, -5, None, None),
         ("HardSigmoid", -5, -7, 0.25, 0.5), ("HardSigmoid", -4, -7, None, None)]


@pytest.mark.parametrize("bits", [8, 16])
@pytest.mark.parametrize("round_mode", [0, 1], ids=["half_up", "half_even"])
@pytest.mark.parametrize("op,in_exp,out_exp,alpha,beta", CASES, ids=lambda v: str(v))
def test_unary_matches_the_closed_form_on_every_input(oracle, op, in_exp, out_exp, alpha, beta, round_mode, bits):
    """float64 closed form, scaled: the result is within one unit everywhere the function is defined, and equal
    wherever the scaled value is not within 1e-3 of a rounding tie (float32 evaluation error is far below that for
    int8; int16 keeps the one-unit bound only, since float32 has 24 bits for a 16-bit result)."""
    dt, lo, hi = (np.int8, -128, 127) if bits == 8 else (np.int16, -32768, 32767)
    if bits == 16:  # keep the real-valued range of the int8 case
        in_exp, out_exp = in_exp - 8, out_exp - 8
    q = np.arange(lo, hi + 1, dtype=dt)
    da, db = oracle.UNARY_DEFAULTS.get(op, (0.0, 0.0))
    got = oracle.unary(op, q, in_exp, out_exp, alpha, beta, round_mode).astype(np.int64)
    x = q.astype(np.float64) * 2.0 ** in_exp
    exact = _closed_form(op, x, da if alpha is None else alpha, db if beta is None else beta) * 2.0 ** -out_exp
    ok = np.isfinite(exact)
    assert ok.sum() > (hi - lo) // 3
    want = np.clip(exact[ok], lo, hi)
    assert np.all(np.abs(got[ok] - want) <= 1.0 + 1e-9)
    if bits == 8:
        frac = exact[ok] - np.floor(exact[ok])
        clear = np.abs(frac - 0.5) > 1e-3
        np.testing.assert_array_equal(got[ok][clear], np.clip(np.floor(exact[ok][clear] + 0.5), lo, hi))
    assert len(np.unique(got[ok])) > 20


def test_unary_undefined_inputs_are_pinned_to_the_documented_stand_in(oracle):
    q = np.array([-128, -1, 0, 1], np.int8)
    assert oracle.unary("Sqrt", q, -3, -4).tolist()[:2] == [0, 0]          # NaN -> 0
    assert oracle.unary("Log", q, -3, -4).tolist()[:3] == [0, 0, -128]     # NaN -> 0, -inf saturates
    assert oracle.unary("Exp", np.array([32767], np.int16), 0, -15)[0] == 32767  # +inf saturates


def test_neg_saturates_the_minimum(oracle):
    q8 = np.arange(-128, 128, dtype=np.int8)
    np.testing.assert_array_equal(oracle.unary("Neg", q8, -3, -3), np.clip(-q8.astype(np.int32), -128, 127))
    q16 = np.arange(-32768, 32768, dtype=np.int16)
    np.testing.assert_array_equal(oracle.unary("Neg", q16, 0, 0), np.clip(-q16.astype(np.int32), -32768, 32767))


def test_sigmoid_and_hard_swish_promotions(oracle):
    """sigmoid is 1.0 / (1.0 + expf(-x)) in double, stored to float; HardSwish's gate is double until the product
    is stored (dl_math.hpp:200-203, dl_module_hard_swish.hpp:73-75): the same widths in numpy, with the C
    library's expf, give every entry exactly."""
    libm = ctypes.CDLL(ctypes.util.find_library("m"))
    libm.expf.restype = ctypes.c_float
    libm.expf.argtypes = [ctypes.c_float]
    q = np.arange(-32768, 32768, dtype=np.int16)
    in_scale, out_scale = np.float32(2.0 ** -12), np.float32(2.0 ** 15)
    x = q.astype(np.float32) * in_scale
    e = np.array([libm.expf(float(-v)) for v in x], dtype=np.float32)
    sig = (1.0 / (1.0 + e.astype(np.float64))).astype(np.float32)
    want = np.clip(np.floor((sig * out_scale).astype(np.float64) + 0.5).astype(np.float32), -32768, 32767)
    np.testing.assert_array_equal(oracle.unary("Sigmoid", q, -12, -15), want.astype(np.int16))
    gate = np.clip(0.166667 * x.astype(np.float64) + 0.5, 0, 1)
    hs = (gate * x.astype(np.float64)).astype(np.float32)
    want = np.clip(np.floor((hs * np.float32(2.0 ** 12)).astype(np.float64) + 0.5), -32768, 32767)
    np.testing.assert_array_equal(oracle.unary("HardSwish", q, -12, -12), want.astype(np.int16))


def test_half_even_differs_from_half_up_only_on_ties(oracle):
    q = np.arange(-128, 128, dtype=np.int8)
    up = oracle.unary("LeakyRelu", q, 0, 1, 1.0, None, 0)       # q / 2: every odd q is a tie
    even = oracle.unary("LeakyRelu", q, 0, 1, 1.0, None, 1)
    np.testing.assert_array_equal(up, np.floor(q / 2 + 0.5))
    np.testing.assert_array_equal(even, np.round(q / 2))         # numpy rounds half to even
    assert (up != even).sum() == 64
