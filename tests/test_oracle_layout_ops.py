"""Pins the oracle's data-movement operators (Concat, Split, Transpose, Resize-nearest, MaxPool) against
library routines and exact arithmetic.  No GPU needed."""
from fractions import Fraction

import numpy as np
import pytest
from scipy import ndimage

import bruteforce as bf


def _rand(rng, shape, dtype=np.int8):
    info = np.iinfo(dtype)
    return rng.integers(info.min, info.max + 1, size=shape).astype(dtype)


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("axis", [0, 1, 2, 3, -1])
def test_concat_is_numpy_concatenate(oracle, dtype, axis):
    rng = np.random.default_rng(5)
    base = [2, 3, 5, 7]
    arrays = []
    for extent in (4, 1, 9):
        shape = list(base)
        shape[axis] = extent
        arrays.append(_rand(rng, shape, dtype))
    np.testing.assert_array_equal(oracle.concat(arrays, axis), np.concatenate(arrays, axis=axis))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("axis,sizes", [(3, [16, 16]), (3, [5, 20, 7]), (1, [1, 2]), (0, [2]), (-2, [3, 1, 1])])
def test_split_is_numpy_split(oracle, dtype, axis, sizes):
    rng = np.random.default_rng(6)
    shape = [2, 3, 5, 32]
    shape[axis] = sum(sizes)
    x = _rand(rng, shape, dtype)
    want = np.split(x, np.cumsum(sizes)[:-1], axis=axis)
    got = oracle.split(x, axis, sizes)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g, w)


@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.int32])
@pytest.mark.parametrize("shape,perm", [
    ((2, 3, 4, 5), (0, 3, 1, 2)), ((2, 3, 4, 5), (0, 2, 3, 1)), ((2, 3, 4, 5), None), ((7, 9), (1, 0)),
    ((3, 1, 1, 8), (0, 3, 1, 2)), ((2, 3, 4), (-1, 0, 1)), ((2, 2, 3, 2, 5), (4, 0, 3, 1, 2)), ((6,), (0,)),
])
def test_transpose_is_numpy_transpose(oracle, dtype, shape, perm):
    rng = np.random.default_rng(7)
    x = _rand(rng, shape, dtype)
    np.testing.assert_array_equal(oracle.transpose(x, perm), np.transpose(x, perm))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("kernel,strides,pads", [
    ((5, 5), (1, 1), (2, 2, 2, 2)), ((2, 2), (2, 2), (0, 0, 0, 0)), ((3, 3), (2, 2), (1, 1, 1, 1)),
    ((3, 2), (1, 2), (1, 0, 0, 1)), ((1, 1), (1, 1), (0, 0, 0, 0)), ((3, 3), (1, 1), (0, 0, 0, 0)),
])
def test_max_pool_matches_brute_force(oracle, dtype, kernel, strides, pads):
    rng = np.random.default_rng(8)
    x = _rand(rng, (2, 9, 8, 5), dtype)
    got = oracle.max_pool(x, kernel, strides, pads)
    pt, pb, pl, pr = pads
    lo = np.iinfo(dtype).min
    padded = np.full((2, 9 + pt + pb, 8 + pl + pr, 5), lo, dtype=dtype)  # clipped window == minimum-value padding
    padded[:, pt:pt + 9, pl:pl + 8, :] = x
    oh = (9 + pt + pb - kernel[0]) // strides[0] + 1
    ow = (8 + pl + pr - kernel[1]) // strides[1] + 1
    want = np.empty((2, oh, ow, 5), dtype=dtype)
    for oy in range(oh):
        for ox in range(ow):
            win = padded[:, oy * strides[0]:oy * strides[0] + kernel[0], ox * strides[1]:ox * strides[1] + kernel[1], :]
            want[:, oy, ox, :] = win.max(axis=(1, 2))
    np.testing.assert_array_equal(got, want)


def test_max_pool_5x5_same_is_scipy_maximum_filter(oracle):
    """The SPPF pooling (5x5, stride 1, pad 2) is a maximum filter with a minimum-value border."""
    rng = np.random.default_rng(9)
    x = _rand(rng, (3, 20, 20, 6))
    want = ndimage.maximum_filter(x, size=(1, 5, 5, 1), mode="constant", cval=-128)
    np.testing.assert_array_equal(oracle.max_pool(x, (5, 5), (1, 1), (2, 2, 2, 2)), want)


def test_resize_nearest_integer_scales_are_numpy_repeat(oracle):
    rng = np.random.default_rng(10)
    x = _rand(rng, (2, 5, 7, 6))
    for sh, sw in ((2, 2), (1, 2), (3, 1), (2, 4), (1, 1)):
        want = np.repeat(np.repeat(x, sh, axis=1), sw, axis=2)
        np.testing.assert_array_equal(oracle.resize_nearest_s8(x, sh, sw), want)


@pytest.mark.parametrize("scale_h,scale_w", [(1.5, 2.5), (0.5, 0.5), (0.75, 1.25), (2.0, 3.0)])
def test_resize_nearest_coordinates_are_floor_of_exact_quotient(oracle, scale_h, scale_w):
    """Scales with an exact binary reciprocal or small numerators: float32 (int)(o * (1 / s)) equals
    floor(o / s) computed in rationals, clipped to the last row / column."""
    rng = np.random.default_rng(11)
    x = _rand(rng, (1, 8, 12, 3))
    got = oracle.resize_nearest_s8(x, scale_h, scale_w)
    oh, ow = int(8 * scale_h), int(12 * scale_w)
    assert got.shape == (1, oh, ow, 3)
    for oy in range(oh):
        iy = min(int(Fraction(oy) / Fraction(scale_h)), 7)
        for ox in range(ow):
            ix = min(int(Fraction(ox) / Fraction(scale_w)), 11)
            np.testing.assert_array_equal(got[0, oy, ox], x[0, iy, ix])


def test_resize_nearest_values_exhaustive(oracle):
    """All 256 int8 inputs: a larger output exponent is the round-half-up shift (pinned separately);
    a smaller one multiplies by 2^k and wraps to int8, as the reference's unsaturated store does."""
    x = np.arange(-128, 128, dtype=np.int8).reshape(1, 16, 16, 1)
    for d in range(0, 8):
        got = oracle.resize_nearest_s8(x, 1, 1, in_exp=-5, out_exp=-5 + d).ravel()
        want = [bf.round_half_up_exact(int(v), d) if d > 0 else int(v) for v in x.ravel()]
        np.testing.assert_array_equal(got, np.array(want, dtype=np.int64).astype(np.int8))
    for d in range(1, 4):
        got = oracle.resize_nearest_s8(x, 1, 1, in_exp=-5, out_exp=-5 - d).ravel()
        want = ((x.ravel().astype(np.int64) << d) & 0xff).astype(np.uint8).view(np.int8)
        np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("sl", [
    (np.s_[:, :, -3:], [-3], [2 ** 63 - 1], [2], [1]), (np.s_[:, 1:4:2], [1], [4], [1], [2]),
    (np.s_[0:1, :, 2:9:3, 1:], [0, 2, 1], [1, 9, 100], [0, 2, 3], [1, 3, 1]), (np.s_[:, :, :, ::4], [0], [64], [-1], [4]),
])
@pytest.mark.parametrize("dtype", [np.int8, np.int16])
def test_slice_is_numpy_slicing(oracle, sl, dtype):
    idx, starts, ends, axes, steps = sl
    x = _rand(np.random.default_rng(12), (2, 5, 10, 8), dtype)
    np.testing.assert_array_equal(oracle.slice_(x, starts, ends, axes, steps), x[idx])


@pytest.mark.parametrize("kernel,strides,pads,exps", [
    ((1, 3), (1, 1), (0, 0, 2, 0), (-6, -7)), ((3, 3), (1, 1), (1, 1, 1, 1), (-5, -5)), ((2, 2), (2, 2), (0, 0, 0, 0), (-4, -5)),
    ((7, 7), (1, 1), (0, 0, 0, 0), (-3, -4)), ((3, 2), (2, 1), (1, 0, 0, 1), (-5, -3)),
])
def test_avg_pool_matches_exact_mean_away_from_ties(oracle, kernel, strides, pads, exps):
    """Clipped-window sum divided by the FULL window area, scaled by 2^(in_exp - out_exp), rounded half up:
    the exact rational value decides every output that is not within float32 error of a tie."""
    rng = np.random.default_rng(13)
    x = _rand(rng, (2, 9, 11, 5))
    got = oracle.avg_pool_s8(x, kernel, strides, pads, exps[0], exps[1]).astype(int)
    pt, pb, pl, pr = pads
    padded = np.zeros((2, 9 + pt + pb, 11 + pl + pr, 5), dtype=np.int64)
    padded[:, pt:pt + 9, pl:pl + 11] = x
    oh, ow = got.shape[1], got.shape[2]
    area = kernel[0] * kernel[1]
    checked = 0
    for oy in range(oh):
        for ox in range(ow):
            win = padded[:, oy * strides[0]:oy * strides[0] + kernel[0], ox * strides[1]:ox * strides[1] + kernel[1]]
            sums = win.sum(axis=(1, 2))
            for n in range(2):
                for k in range(5):
                    exact = Fraction(int(sums[n, k]), area) * Fraction(2) ** (exps[0] - exps[1])
                    frac = exact - (exact.numerator // exact.denominator)
                    if abs(frac - Fraction(1, 2)) < Fraction(1, 10000):
                        continue  # a (near-)tie: float32 may fall either way
                    want = min(127, max(-128, (exact + Fraction(1, 2)).__floor__()))
                    assert got[n, oy, ox, k] == want, (n, oy, ox, k)
                    checked += 1
    assert checked > 50


@pytest.mark.parametrize("shape,axes,keepdims,exps", [
    ((2, 7, 7, 16), [1, 2], True, (-4, -5)), ((3, 5, 8), [-1], True, (-5, -5)), ((2, 3, 4, 5), [0, 2], False, (-3, -4)),
    ((4, 9), [], True, (-6, -6)), ((2, 6, 10), [1], False, (-5, -7)),
])
def test_reduce_mean_matches_exact_mean_away_from_ties(oracle, shape, axes, keepdims, exps):
    x = _rand(np.random.default_rng(14), shape)
    got = oracle.reduce_mean_s8(x, axes, keepdims, exps[0], exps[1])
    nd = len(shape)
    ax = tuple(a % nd for a in axes) if axes else tuple(range(nd))
    sums = x.astype(np.int64).sum(axis=ax, keepdims=keepdims)
    count = int(np.prod([shape[a] for a in ax]))
    assert got.shape == (sums.shape if sums.shape else (1,))
    checked = 0
    for g, sm in zip(got.ravel(), sums.ravel()):
        exact = Fraction(int(sm), count) * Fraction(2) ** (exps[0] - exps[1])
        frac = exact - (exact.numerator // exact.denominator)
        if abs(frac - Fraction(1, 2)) < Fraction(1, 10000):
            continue
        assert int(g) == min(127, max(-128, (exact + Fraction(1, 2)).__floor__()))
        checked += 1
    assert checked > 0


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("stride,pad", [((2, 2), (0, 0)), ((3, 1), (1, 0)), ((1, 1), (0, 2)), ((2, 4), (1, 3))])
def test_insert_zeros_is_strided_assignment(oracle, dtype, stride, pad):
    """numpy statement of the operator: zeros, then out[:, ::sh, ::sw] = x; equivalently the adjoint of a
    strided slice, which is how a transposed convolution's input is prepared."""
    rng = np.random.default_rng(39)
    x = _rand(rng, (2, 5, 4, 3), dtype)
    got = oracle.insert_zeros(x, stride, pad)
    oh = 5 + (stride[0] - 1) * 4 + pad[0]
    ow = 4 + (stride[1] - 1) * 3 + pad[1]
    want = np.zeros((2, oh, ow, 3), dtype=dtype)
    want[:, :(5 - 1) * stride[0] + 1:stride[0], :(4 - 1) * stride[1] + 1:stride[1]] = x
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got[:, ::stride[0], ::stride[1]][:, :5, :4], x)


@pytest.mark.parametrize("mode", ["constant", "edge", "reflect"])
@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.int32])
def test_pad_is_numpy_pad(oracle, mode, dtype):
    """numpy.pad is the textbook routine for all three modes; random ranks 1..5, unequal sides, zero pads."""
    rng = np.random.default_rng(71)
    for _ in range(30):
        nd = int(rng.integers(1, 6))
        shape = [int(rng.integers(2, 7)) for _ in range(nd)]
        info = np.iinfo(dtype)
        x = rng.integers(info.min, info.max, size=shape, dtype=dtype, endpoint=True)
        before = [int(rng.integers(0, s if mode == "reflect" else 4)) for s in shape]
        after = [int(rng.integers(0, s if mode == "reflect" else 4)) for s in shape]
        value = int(rng.integers(-100, 100))
        kw = {"constant_values": value} if mode == "constant" else {}
        want = np.pad(x, list(zip(before, after)), mode=mode, **kw)
        np.testing.assert_array_equal(oracle.pad(x, before + after, mode, value), want)


def test_pad_of_an_empty_axis_is_all_constant(oracle):
    x = np.zeros((2, 0, 3), np.int8)
    got = oracle.pad(x, [0, 2, 0, 0, 1, 0], "constant", 7)
    assert got.shape == (2, 3, 3) and np.all(got == 7)


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("op", ["ReduceMax", "ReduceMin", "ReduceSum", "ReduceL1", "ReduceSumSquare"])
def test_reduce_int_is_numpy(oracle, op, dtype):
    """numpy max / min / sum over the same axes; the sum then takes the pinned shift-round and saturates."""
    rng = np.random.default_rng(73)
    info = np.iinfo(dtype)
    for axes, keep in [([1, 2], True), ([3], False), ([0, 2], True), ([], True), ([-1], True), ([1], False)]:
        x = rng.integers(info.min, info.max, size=(2, 5, 6, 7), dtype=dtype, endpoint=True)
        ax = tuple(a % 4 for a in axes) if axes else None
        if op in ("ReduceSum", "ReduceL1", "ReduceSumSquare"):
            wide = x.astype(np.int64)
            terms = wide if op == "ReduceSum" else (np.abs(wide) if op == "ReduceL1" else wide * wide)
            for shift in ((-1, 0, 3, 6) if op != "ReduceSumSquare" else (0, 9, 14, 22)):
                for rm in (0, 1):
                    s = terms.sum(axis=ax, keepdims=keep)
                    if shift <= 0:
                        q = s << -shift
                    elif rm == 0:
                        q = (s + (1 << (shift - 1))) >> shift          # floor((s + half) / 2^shift)
                    else:
                        q = np.round(s / 2.0 ** shift).astype(np.int64)  # exact in float64; numpy rounds half to even
                    want = np.clip(q, info.min, info.max).astype(dtype)
                    got = oracle.reduce_int(op, x, axes, keep, shift, rm)
                    np.testing.assert_array_equal(got.reshape(want.shape), want)
        else:
            want = (x.max if op == "ReduceMax" else x.min)(axis=ax, keepdims=keep)
            got = oracle.reduce_int(op, x, axes, keep)
            np.testing.assert_array_equal(got.reshape(np.shape(want)), want)


@pytest.mark.parametrize("b", [2, 3])
def test_space_to_depth_and_depth_to_space_are_the_onnx_permutations(oracle, b):
    """The ONNX operator definitions are reshape / transpose recipes (NCHW there, NHWC here); the oracle scatters
    with the reference's index arithmetic.  CRD DepthToSpace inverts SpaceToDepth."""
    rng = np.random.default_rng(75)
    for c in (1, 4, 5):
        x = rng.integers(-128, 128, size=(2, 2 * b, 3 * b, c), dtype=np.int8)
        n, h, w, _ = x.shape
        want = x.reshape(n, h // b, b, w // b, b, c).transpose(0, 1, 3, 5, 2, 4).reshape(n, h // b, w // b, c * b * b)
        got = oracle.space_to_depth(x, b)
        np.testing.assert_array_equal(got, want)
        np.testing.assert_array_equal(oracle.depth_to_space(got, b, "CRD"), x)
    for oc in (1, b, 5):
        x = rng.integers(-128, 128, size=(2, 3, 4, oc * b * b), dtype=np.int16)
        n, h, w, _ = x.shape
        crd = x.reshape(n, h, w, oc, b, b).transpose(0, 1, 4, 2, 5, 3).reshape(n, h * b, w * b, oc)
        dcr = x.reshape(n, h, w, b, b, oc).transpose(0, 1, 3, 2, 4, 5).reshape(n, h * b, w * b, oc)
        np.testing.assert_array_equal(oracle.depth_to_space(x, b, "CRD"), crd)
        np.testing.assert_array_equal(oracle.depth_to_space(x, b, "DCR"), dcr)


def test_depth_to_space_dcr_is_the_reference_loop_when_it_is_a_permutation(oracle):
    """dl_module_depth_to_space.hpp:45-67 with C' == b: out channel c % b, row offset c // b^2, column offset
    (c % b^2) // b, replayed element by element."""
    rng = np.random.default_rng(76)
    b = 2
    x = rng.integers(-128, 128, size=(1, 3, 2, b * b * b), dtype=np.int8)
    want = np.zeros((1, 3 * b, 2 * b, b), dtype=np.int8)
    for h in range(3):
        for w in range(2):
            for c in range(b * b * b):
                want[0, h * b + c // (b * b), w * b + (c % (b * b)) // b, c % b] = x[0, h, w, c]
    np.testing.assert_array_equal(oracle.depth_to_space(x, b, "DCR"), want)


def test_gather_is_numpy_take(oracle):
    rng = np.random.default_rng(77)
    x = rng.integers(-128, 128, size=(3, 5, 6, 7), dtype=np.int8)
    for axis, idx in [(0, [2]), (1, [4, 0, 0, 3]), (-1, [[0, 6], [3, 3]]), (2, list(range(6)))]:
        np.testing.assert_array_equal(oracle.gather(x, idx, axis), np.take(x, np.asarray(idx), axis=axis))
    x16 = rng.integers(-32768, 32767, size=(4, 9), dtype=np.int16)
    np.testing.assert_array_equal(oracle.gather(x16, [8, 1], 1), np.take(x16, [8, 1], axis=1))
