"""Pins the CPU oracle: reference-held known answers, exact-rational rounding, brute force on the
reference's own shape matrix, and structural invariants.  No GPU needed."""
import json
import os

import numpy as np
import pytest

import bruteforce as bf
from cases import CONFIG1, CONV_CASES, DW_CASES, GEMM_CASES, rng_int8, typical_shift

HERE = os.path.dirname(os.path.abspath(__file__))


# --------------------------------------------------------------------------- rounding helpers
def test_shift_round_half_up_exhaustive_int16(oracle):
    for s in range(1, 21):
        for v in range(-32768, 32768, 1 if s <= 4 else 7):
            assert oracle.shift_round_s32(v, s) == bf.round_half_up_exact(v, s), (v, s)


def test_shift_round_ties_table(oracle):
    # value/2^s in {+-0.5, +-1.5, +-2.5}: half-up goes toward +inf, half-even to the even neighbour
    for s in (1, 3, 9):
        h = 1 << (s - 1)
        for k, up, even in ((1, 1, 0), (-1, 0, 0), (3, 2, 2), (-3, -1, -2), (5, 3, 2), (-5, -2, -2)):
            assert oracle.shift_round_s32(k * h, s, oracle.ROUND_HALF_UP) == up
            assert oracle.shift_round_s32(k * h, s, oracle.ROUND_HALF_EVEN) == even
            assert oracle.shift_round_s64(k * h, s, oracle.ROUND_HALF_UP) == up
            assert oracle.shift_round_s64(k * h, s, oracle.ROUND_HALF_EVEN) == even


def test_shift_round_random_wide(oracle):
    rng = np.random.default_rng(1)
    for v in list(rng.integers(-2**31, 2**31, size=4000)) + [2**31 - 1, -2**31, 0, -1, 1]:
        for s in (1, 2, 7, 15, 24, 31):
            v = int(v)
            assert oracle.shift_round_s32(v, s) == bf.round_half_up_exact(v, s)
            assert oracle.shift_round_s32(v, s, oracle.ROUND_HALF_EVEN) == bf.round_half_even_exact(v, s)
    for v in rng.integers(-2**46, 2**46, size=2000):
        for s in (1, 9, 18, 24, 33):
            v = int(v)
            assert oracle.shift_round_s64(v, s) == bf.round_half_up_exact(v, s)
            assert oracle.shift_round_s64(v, s, oracle.ROUND_HALF_EVEN) == bf.round_half_even_exact(v, s)


def test_shift_round_left_shift_saturates(oracle):
    assert oracle.shift_round_s32(5, 0) == 5
    assert oracle.shift_round_s32(-5, -3) == -40
    assert oracle.shift_round_s32(2**30, -4) == 2**31 - 1
    assert oracle.shift_round_s32(-2**30, -4) == -2**31
    assert oracle.shift_round_s64(-5, -3) == -40


# --------------------------------------------------------------------------- reference goldens
def _load_gemm_fixtures():
    with open(os.path.join(HERE, "golden", "gemm_c_fixtures.json")) as f:
        return json.load(f)


@pytest.mark.parametrize("case", _load_gemm_fixtures(), ids=lambda c: os.path.basename(c["file"]))
def test_gemm_reference_known_answers(oracle, case):
    """The three `c`-target Gemm models the reference ships with embedded test vectors."""
    _, _, k, n = case["filter_shape"]
    x = np.array(case["input"], dtype=np.int8).reshape(case["input_shape"])
    w = np.array(case["filter_bytes"], dtype=np.int8)  # bytes as stored: N-major [N][K]
    bias = np.array(case["bias"], dtype=np.int32)
    want = np.array(case["output"], dtype=np.int8).reshape(case["output_shape"])
    (w_exp,) = case["filter_exponents"]
    assert case["bias_exponents"] == [case["input_exponent"] + w_exp]
    shift = case["output_exponent"] - w_exp - case["input_exponent"]
    act = oracle.RELU if case["activation"] == "Relu" else oracle.LINEAR
    got = oracle.gemm_s8(x, w, bias, shift, activation=act)
    np.testing.assert_array_equal(got, want)


def test_gemm_known_answers_discriminate(oracle):
    """A K-major reading of the filter bytes, flooring instead of rounding, or shifting before
    the bias is added must each fail to reproduce at least one reference vector."""
    wrong = {"layout": 0, "floor": 0, "bias_after_shift": 0}
    for case in _load_gemm_fixtures():
        _, _, k, n = case["filter_shape"]
        x = np.array(case["input"], dtype=np.int8).reshape(1, k)
        w = np.array(case["filter_bytes"], dtype=np.int8)
        bias = np.array(case["bias"], dtype=np.int64)
        want = np.array(case["output"], dtype=np.int64)
        (w_exp,) = case["filter_exponents"]
        shift = case["output_exponent"] - w_exp - case["input_exponent"]
        relu = case["activation"] == "Relu"
        fin = lambda v: np.clip(np.maximum(v, 0) if relu else v, -128, 127)  # noqa: E731
        acc = x.astype(np.int64) @ w.reshape(n, k).astype(np.int64).T
        acc_kmajor = x.astype(np.int64) @ w.reshape(k, n).astype(np.int64)
        half = 1 << (shift - 1)
        assert np.array_equal(fin((acc + bias + half) >> shift).ravel(), want)
        wrong["layout"] += not np.array_equal(fin((acc_kmajor + bias + half) >> shift).ravel(), want)
        wrong["floor"] += not np.array_equal(fin((acc + bias) >> shift).ravel(), want)
        wrong["bias_after_shift"] += not np.array_equal(fin(((acc + half) >> shift) + (bias >> shift)).ravel(), want)
    assert all(v >= 1 for v in wrong.values()), wrong


def test_gemm_fixture_covers_saturation_and_linear():
    cases = _load_gemm_fixtures()
    assert any(c["activation"] == "Linear" and min(c["output"]) < 0 for c in cases)
    assert any(127 in c["output"] for c in cases)


# --------------------------------------------------------------------------- brute force
def _conv_inputs(case, seed, n=1, per_channel=False, dtype=np.int8):
    name, (h, w, c), oc, k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(seed)
    if dtype == np.int8:
        x = rng_int8(rng, (n, h, w, c))
        f = rng_int8(rng, (oc, k[0], k[1], c))
        bias = rng.integers(-4096, 4097, size=oc).astype(np.int32) if has_bias else None
        base = typical_shift(k[0] * k[1] * c)
    else:
        x = rng.integers(-32768, 32768, size=(n, h, w, c)).astype(np.int16)
        f = rng.integers(-32768, 32768, size=(oc, k[0], k[1], c)).astype(np.int16)
        bias = rng.integers(-2**28, 2**28, size=oc).astype(np.int64) if has_bias else None
        base = typical_shift(k[0] * k[1] * c) + 16
    shift = (base + rng.integers(-2, 3, size=oc)).astype(np.int32) if per_channel else np.int32(base)
    return x, f, bias, shift, k, stride, dil, pads, relu


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("per_channel", [False, True], ids=["per_tensor", "per_channel"])
def test_conv2d_s8_vs_bruteforce(oracle, case, per_channel):
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 11, n=2, per_channel=per_channel)
    got = oracle.conv2d_s8(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR)
    want = bf.conv2d_ref(x, f, bias, shift, stride, dil, pads, relu)
    np.testing.assert_array_equal(got, want)
    assert got.min() < got.max()  # not degenerate (all-saturated outputs would hide errors)


def test_conv2d_s8_config1(oracle):
    x, f, bias, _, k, stride, dil, pads, relu = _conv_inputs(CONFIG1, 0xE5D1)
    got = oracle.conv2d_s8(x, f, bias, 9, k, stride, dil, pads, oracle.RELU)
    want = bf.conv2d_ref(x, f, bias, 9, stride, dil, pads, True)
    assert got.shape == (1, 56, 56, 64)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("shift", [-1, 0, 1])
def test_conv2d_s8_small_and_negative_shift(oracle, shift):
    rng = np.random.default_rng(5)
    x = rng.integers(-3, 4, size=(1, 6, 6, 4)).astype(np.int8)
    f = rng.integers(-3, 4, size=(5, 1, 1, 4)).astype(np.int8)
    bias = rng.integers(-20, 21, size=5).astype(np.int32)
    got = oracle.conv2d_s8(x, f, bias, shift, (1, 1))
    want = bf.conv2d_ref(x, f, bias, shift, (1, 1), (1, 1), (0, 0, 0, 0), False)
    np.testing.assert_array_equal(got, want)


def test_conv2d_s8_half_even(oracle):
    case = CONV_CASES[5]
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 3, per_channel=True)
    got = oracle.conv2d_s8(x, f, bias, shift, k, stride, dil, pads, oracle.LINEAR, oracle.ROUND_HALF_EVEN)
    want = bf.conv2d_ref(x, f, bias, shift, stride, dil, pads, False, half_even=True)
    np.testing.assert_array_equal(got, want)
    up = oracle.conv2d_s8(x, f, bias, shift, k, stride, dil, pads, oracle.LINEAR, oracle.ROUND_HALF_UP)
    assert np.abs(up.astype(int) - got.astype(int)).max() <= 1


@pytest.mark.parametrize("case", DW_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("per_channel", [False, True], ids=["per_tensor", "per_channel"])
def test_depthwise_s8_vs_bruteforce(oracle, case, per_channel):
    name, (h, w, c), k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(13)
    x = rng_int8(rng, (2, h, w, c))
    f = rng_int8(rng, (k[0], k[1], c))
    bias = rng.integers(-4096, 4097, size=c).astype(np.int32) if has_bias else None
    base = typical_shift(k[0] * k[1])
    shift = (base + rng.integers(-2, 3, size=c)).astype(np.int32) if per_channel else np.int32(base)
    got = oracle.depthwise_s8(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR)
    want = bf.depthwise_ref(x, f, bias, shift, stride, dil, pads, relu)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", [CONV_CASES[1], CONV_CASES[4], CONV_CASES[5], CONV_CASES[7], CONV_CASES[12]],
                         ids=lambda c: c[0])
def test_conv2d_s16_vs_bruteforce(oracle, case):
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 17, per_channel=True, dtype=np.int16)
    got = oracle.conv2d_s16(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR)
    want = bf.conv2d_ref(x, f, bias, shift, stride, dil, pads, relu, bits=16)
    np.testing.assert_array_equal(got, want)
    assert got.min() < got.max()


@pytest.mark.parametrize("case", [DW_CASES[1], DW_CASES[2], DW_CASES[5], DW_CASES[10]], ids=lambda c: c[0])
def test_depthwise_s16_vs_bruteforce(oracle, case):
    name, (h, w, c), k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(19)
    x = rng.integers(-32768, 32768, size=(2, h, w, c)).astype(np.int16)
    f = rng.integers(-32768, 32768, size=(k[0], k[1], c)).astype(np.int16)
    bias = rng.integers(-2**28, 2**28, size=c).astype(np.int64) if has_bias else None
    shift = (typical_shift(k[0] * k[1]) + 16 + rng.integers(-2, 3, size=c)).astype(np.int32)
    got = oracle.depthwise_s16(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR)
    want = bf.depthwise_ref(x, f, bias, shift, stride, dil, pads, relu, bits=16)
    np.testing.assert_array_equal(got, want)


# --------------------------------------------------------------------------- invariants
@pytest.mark.parametrize("m,k,n,has_bias,relu", GEMM_CASES)
def test_gemm_is_matmul(oracle, m, k, n, has_bias, relu):
    rng = np.random.default_rng(23)
    x = rng_int8(rng, (m, k))
    w = rng_int8(rng, (n, k))
    bias = rng.integers(-4096, 4097, size=n).astype(np.int32) if has_bias else None
    shift = (typical_shift(k) + rng.integers(-1, 2, size=n)).astype(np.int32)
    got = oracle.gemm_s8(x, w, bias, shift, activation=oracle.RELU if relu else oracle.LINEAR)
    acc = x.astype(np.int64) @ w.astype(np.int64).T
    if has_bias:
        acc = acc + bias
    want = bf.requant_vec(acc, shift, relu, -128, 127).astype(np.int8)
    np.testing.assert_array_equal(got, want)


def test_padding_equals_explicit_zero_padding(oracle):
    rng = np.random.default_rng(29)
    x = rng_int8(rng, (1, 9, 7, 6))
    f = rng_int8(rng, (10, 3, 5, 6))
    bias = rng.integers(-500, 500, size=10).astype(np.int32)
    pads = (2, 1, 3, 2)
    a = oracle.conv2d_s8(x, f, bias, 8, (3, 5), (2, 1), (1, 1), pads, oracle.RELU)
    b = oracle.conv2d_s8(bf.pad_nhwc(x, pads), f, bias, 8, (3, 5), (2, 1), (1, 1), (0, 0, 0, 0), oracle.RELU)
    np.testing.assert_array_equal(a, b)


def test_depthwise_equals_block_diagonal_dense(oracle):
    rng = np.random.default_rng(31)
    c = 6
    x = rng_int8(rng, (2, 8, 9, c))
    f = rng_int8(rng, (3, 3, c))
    bias = rng.integers(-500, 500, size=c).astype(np.int32)
    shift = np.array([5, 6, 7, 5, 6, 4], dtype=np.int32)
    dense = np.zeros((c, 3, 3, c), dtype=np.int8)
    for ch in range(c):
        dense[ch, :, :, ch] = f[:, :, ch]
    a = oracle.depthwise_s8(x, f, bias, shift, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1))
    b = oracle.conv2d_s8(x, dense, bias, shift, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1))
    np.testing.assert_array_equal(a, b)


def test_per_channel_is_per_tensor_on_channel_slices(oracle):
    """Definition of the per-channel mode: the per-tensor C formula, one output channel at a time."""
    rng = np.random.default_rng(37)
    x = rng_int8(rng, (1, 7, 7, 12))
    f = rng_int8(rng, (9, 3, 3, 12))
    bias = rng.integers(-4096, 4097, size=9).astype(np.int32)
    shift = rng.integers(6, 11, size=9).astype(np.int32)
    full = oracle.conv2d_s8(x, f, bias, shift, (3, 3), pads=(1, 1, 1, 1), activation=oracle.RELU)
    for oc in range(9):
        one = oracle.conv2d_s8(x, f[oc:oc + 1], bias[oc:oc + 1], int(shift[oc]), (3, 3), pads=(1, 1, 1, 1),
                               activation=oracle.RELU)
        np.testing.assert_array_equal(full[..., oc:oc + 1], one)


def test_batch_is_independent_images(oracle):
    rng = np.random.default_rng(41)
    x = rng_int8(rng, (3, 6, 6, 8))
    f = rng_int8(rng, (4, 3, 3, 8))
    full = oracle.conv2d_s8(x, f, None, 7, (3, 3), pads=(1, 1, 1, 1))
    for n in range(3):
        np.testing.assert_array_equal(full[n:n + 1], oracle.conv2d_s8(x[n:n + 1], f, None, 7, (3, 3), pads=(1, 1, 1, 1)))


def test_bad_geometry_is_rejected(oracle):
    x = np.zeros((1, 2, 2, 4), dtype=np.int8)
    with pytest.raises(ValueError):
        oracle.conv2d_s8(x, np.zeros((4, 5, 5, 4), dtype=np.int8), None, 3, (5, 5))


# --------------------------------------------------------------------------- elementwise
def test_lut_known_answer_pattern(oracle):
    """Pattern of test_apps/dl_pie_func/main/test_lut.cpp:104-150."""
    table = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
    edge = np.array([-128, -127, -1, 0, 1, 126, 127], dtype=np.int8)
    for size in (1, 7, 8, 15, 16, 63, 64, 1011, 1024):
        rng = np.random.default_rng(size)
        x = rng_int8(rng, (size,))
        x[:min(size, edge.size)] = edge[:min(size, edge.size)]
        got = oracle.lut_s8(x, table)
        want = table[x.astype(np.int32) + 128]
        np.testing.assert_array_equal(got, want)
    ident = np.arange(-128, 128).astype(np.int8)
    x = rng_int8(np.random.default_rng(0), (300,))
    np.testing.assert_array_equal(oracle.lut_s8(x, ident), x)


@pytest.mark.parametrize("shift", [-1, 0, 3, 6, 7])
def test_prelu_exhaustive(oracle, shift):
    xs, alphas = np.meshgrid(np.arange(-128, 128), np.arange(-128, 128), indexing="ij")
    x = xs.astype(np.int8)  # [256 pixels][256 channels], channel c has alpha c-128
    alpha = np.arange(-128, 128).astype(np.int8)
    got = oracle.prelu_s8(x, alpha, shift)
    want = np.empty_like(x)
    for i in range(256):
        for j in range(256):
            xv, av = int(xs[i, j]), int(alphas[i, j])
            if xv >= 0:
                want[i, j] = xv
            else:
                p = xv * av
                t = (p >> shift) if shift > 0 else (p << -shift)  # floor shift, exact integers
                t = ((t + 32768) % 65536) - 32768  # int16 temporary of the reference
                want[i, j] = max(-128, min(127, t))
    np.testing.assert_array_equal(got, want)


def test_add_exhaustive_and_broadcast(oracle):
    a, b = np.meshgrid(np.arange(-128, 128), np.arange(-128, 128), indexing="ij")
    got = oracle.add_s8(a.astype(np.int8), b.astype(np.int8))
    np.testing.assert_array_equal(got, np.clip(a + b, -128, 127).astype(np.int8))
    v = np.arange(-128, 128).astype(np.int8)
    s = np.array([100], dtype=np.int8)
    np.testing.assert_array_equal(oracle.add_s8(v, s), np.clip(v.astype(int) + 100, -128, 127).astype(np.int8))
    np.testing.assert_array_equal(oracle.add_s8(s, v), np.clip(v.astype(int) + 100, -128, 127).astype(np.int8))


def test_relu_clip_requantize_exact(oracle):
    x = np.arange(-128, 128).astype(np.int8)
    np.testing.assert_array_equal(oracle.relu_s8(x), np.maximum(x, 0))
    for in_exp, out_exp in ((-6, -5), (-5, -7), (-4, -4), (-7, -3), (-3, -6)):
        s = out_exp - in_exp
        exact = np.array([bf.round_half_up_exact(int(v), s) for v in x])
        np.testing.assert_array_equal(oracle.requantize_s8(x, in_exp, out_exp), np.clip(exact, -128, 127).astype(np.int8))
        np.testing.assert_array_equal(oracle.relu_s8(x, in_exp, out_exp),
                                      np.clip(np.where(x >= 0, exact, 0), -128, 127).astype(np.int8))
        lo, hi = 0, 96
        exact_c = np.array([bf.round_half_up_exact(int(min(max(v, lo), hi)), s) for v in x])
        np.testing.assert_array_equal(oracle.clip_s8(x, lo, hi, in_exp, out_exp),
                                      np.clip(exact_c, -128, 127).astype(np.int8))


def test_global_avg_pool_non_ties(oracle):
    """Exact rational mean, checked wherever float32 rounding cannot matter (distance from a tie > 1e-3)."""
    from fractions import Fraction
    import math
    rng = np.random.default_rng(43)
    x = rng_int8(rng, (3, 7, 7, 40))
    for in_exp, out_exp in ((-4, -5), (-5, -5), (-3, -6), (-6, -4)):
        got = oracle.global_avg_pool_s8(x, in_exp, out_exp).reshape(3, 40)
        sums = x.astype(np.int64).sum(axis=(1, 2))
        checked = 0
        for n in range(3):
            for c in range(40):
                val = Fraction(int(sums[n, c]), 49) * Fraction(2) ** (in_exp - out_exp)
                frac = val + Fraction(1, 2)
                if abs(frac - round(frac)) < Fraction(1, 1000):
                    continue
                assert got[n, c] == max(-128, min(127, math.floor(frac)))
                checked += 1
        assert checked > 100


def test_mul_s8_exhaustive(oracle):
    """All int8 operand pairs, shifts -4..14: round-half-up of the exact product (half-even table for the
    ESP32-P4 rounding), clamped; the float expression of the reference is exact for these operands."""
    a = np.repeat(np.arange(-128, 128, dtype=np.int8), 256)
    b = np.tile(np.arange(-128, 128, dtype=np.int8), 256)
    prod = a.astype(np.int64) * b.astype(np.int64)
    for shift in range(-4, 15):
        got = oracle.mul_s8(a, b, shift).astype(np.int64)
        if shift > 0:
            want = (prod + (1 << (shift - 1))) >> shift  # floor(p / 2^s + 1/2) in exact integers
        else:
            want = prod << -shift
        np.testing.assert_array_equal(got, np.clip(want, -128, 127), err_msg=f"shift {shift}")
        if shift > 0:
            he = oracle.mul_s8(a, b, shift, oracle.ROUND_HALF_EVEN).astype(np.int64)
            q, r = prod >> shift, prod & ((1 << shift) - 1)
            h = 1 << (shift - 1)
            want_he = q + ((r > h) | ((r == h) & ((q & 1) == 1)))
            np.testing.assert_array_equal(he, np.clip(want_he, -128, 127), err_msg=f"half-even shift {shift}")
    # scalar operand
    np.testing.assert_array_equal(oracle.mul_s8(a[:512], np.array([3], dtype=np.int8), 1),
                                  np.clip((a[:512].astype(np.int64) * 3 + 1) >> 1, -128, 127))
