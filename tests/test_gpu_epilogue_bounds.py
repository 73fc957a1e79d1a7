"""The short requantization forms of the kernels are chosen by range checks (|bias + 2^(s-1)| + K * 2^14 must
fit int32 also after the left shift by max(0, 8 - s)).  Uniform random operands never come near those bounds:
these cases do.  Every output channel carries its own (shift, bias, filter sign) combination, operands sit at the
int8 extremes, reductions are long, and both rounding modes run - on every kernel route, against the oracle,
whose shift_and_round widens to 64 bits as esp-dl/dl/tool/src/dl_tool.cpp:121-136 does."""
import itertools

import numpy as np
import pytest

from gpu_util import announce, espdl, to_dev, to_host

pytestmark = pytest.mark.gpu

SHIFTS = [1, 7, 8, 24, 31]
BIASES = [-(1 << 20), 1 << 20, -((1 << 30) - 1), (1 << 30) - 1]


def _channels(n_min=1):
    """(shift, bias, filter value) per output channel: every combination, repeated to a multiple of 64."""
    combos = list(itertools.product(SHIFTS, BIASES, [-128, 127]))
    while len(combos) % 64 or len(combos) < n_min:
        combos.append(combos[len(combos) % 40])
    shift = np.array([c[0] for c in combos], dtype=np.int32)
    bias = np.array([c[1] for c in combos], dtype=np.int32)
    wval = np.array([c[2] for c in combos], dtype=np.int8)
    return shift, bias, wval


def _dense(oracle, x, k, stride, pads, he, route):
    m = espdl()
    shift, bias, wval = _channels()
    oc = len(shift)
    c = x.shape[-1]
    f = np.broadcast_to(wval[:, None, None, None], (oc, k[0], k[1], c)).copy()
    # a few taps of the other sign so that sums are not all at +-K * 2^14
    f[:, 0, 0, ::7] = np.where(f[:, 0, 0, ::7] == 127, -128, 127)
    rm_g = m.capi.ROUND_HALF_EVEN if he else m.capi.ROUND_HALF_UP
    rm_o = oracle.ROUND_HALF_EVEN if he else oracle.ROUND_HALF_UP
    want = oracle.conv2d_s8(x, f, bias, shift, k, stride, (1, 1), pads, oracle.LINEAR, rm_o)
    got = m.conv2d(to_dev(x), to_dev(f), to_dev(bias), to_dev(shift), k, stride, (1, 1), pads, round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got), want, err_msg=route)
    assert len(np.unique(want)) > 2


@pytest.mark.parametrize("he", [False, True], ids=["half_up", "half_even"])
@pytest.mark.parametrize("xval", [-128, 127])
@pytest.mark.parametrize("k_total", [576, 1280, 2304])
def test_pointwise_routes_at_the_bounds(oracle, k_total, xval, he):
    """Flat 1x1 convolutions of reduction length K: a handful of rows (one wavefront per tile), a few hundred
    (tiled GEMM through LDS), strided (the implicit-GEMM kernel with operands from global memory)."""
    announce(f"epilogue bounds pointwise K={k_total} x={xval} he={he}")
    for route, shape, stride in (("rows", (1, 1, 16, k_total), (1, 1)), ("pwgemm", (1, 8, 8, k_total), (1, 1)),
                                 ("direct", (1, 9, 9, k_total), (2, 2))):
        x = np.full(shape, xval, dtype=np.int8)
        x[..., ::5] = 127 if xval == -128 else -128  # mixed signs along the reduction
        _dense(oracle, x, (1, 1), stride, (0, 0, 0, 0), he, route)


@pytest.mark.parametrize("he", [False, True], ids=["half_up", "half_even"])
@pytest.mark.parametrize("xval", [-128, 127])
@pytest.mark.parametrize("in_c", [64, 128, 256])
def test_lds_tiled_conv_at_the_bounds(oracle, in_c, xval, he):
    """3x3 convolutions of 64 / 128 / 256 channels (K = 576 / 1152 / 2304) through the LDS-tiled kernel (the
    last one through the direct kernel where the filters do not fit)."""
    announce(f"epilogue bounds 3x3 in_c={in_c} x={xval} he={he}")
    x = np.full((1, 9, 11, in_c), xval, dtype=np.int8)
    x[..., ::3] = 127 if xval == -128 else -128
    _dense(oracle, x, (3, 3), (1, 1), (1, 1, 1, 1), he, "tiled")


@pytest.mark.parametrize("he", [False, True], ids=["half_up", "half_even"])
@pytest.mark.parametrize("xval", [-128, 127])
def test_depthwise_at_the_bounds(oracle, xval, he):
    announce(f"epilogue bounds depthwise x={xval} he={he}")
    m = espdl()
    shift, bias, wval = _channels()
    c = len(shift)
    x = np.full((2, 12, 12, c), xval, dtype=np.int8)
    f = np.broadcast_to(wval[None, None, :], (3, 3, c)).copy()
    f[1, 1, ::2] = np.where(f[1, 1, ::2] == 127, -128, 127)
    rm_g = m.capi.ROUND_HALF_EVEN if he else m.capi.ROUND_HALF_UP
    rm_o = oracle.ROUND_HALF_EVEN if he else oracle.ROUND_HALF_UP
    want = oracle.depthwise_s8(x, f, bias, shift, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), oracle.LINEAR, rm_o)
    got = m.conv2d(to_dev(x), to_dev(f), to_dev(bias), to_dev(shift), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), depthwise=True,
                   round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got), want)


@pytest.mark.parametrize("he", [False, True], ids=["half_up", "half_even"])
@pytest.mark.parametrize("xval", [-128, 127])
@pytest.mark.parametrize("k_total", [576, 1280, 2304])
def test_conv_gap_at_the_bounds(oracle, k_total, xval, he):
    announce(f"epilogue bounds conv+GAP K={k_total} x={xval} he={he}")
    m = espdl()
    shift, bias, wval = _channels()
    oc = len(shift)
    x = np.full((3, 7, 7, k_total), xval, dtype=np.int8)
    x[..., ::5] = 127 if xval == -128 else -128
    f = np.broadcast_to(wval[:, None], (oc, k_total)).copy()
    f[:, ::9] = 3
    rm_g = m.capi.ROUND_HALF_EVEN if he else m.capi.ROUND_HALF_UP
    rm_o = oracle.ROUND_HALF_EVEN if he else oracle.ROUND_HALF_UP
    conv = oracle.conv2d_s8(x, f.reshape(oc, 1, 1, k_total), bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, rm_o)
    want = oracle.global_avg_pool_s8(conv, -4, -3)
    got = m.conv2d_gap_s8(to_dev(x), to_dev(f), to_dev(bias), to_dev(shift), -4, -3, round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got).reshape(want.shape), want)


# (name, block input, expanded channels, output channels, stride): one-wavefront-per-tile kernel (guard-free and
# guarded builds) and workgroup-per-tile kernel; the project stage reduces over up to 960 channels
MB_ROUTES = [
    ("wave_56x56_24_144_24", (2, 56, 56, 24), 144, 24, (1, 1)),
    ("wave_guarded_19x23_32_80_48", (2, 19, 23, 32), 80, 48, (1, 1)),
    ("group_14x14_64_384_64", (2, 14, 14, 64), 384, 64, (1, 1)),
    ("group_7x7_160_960_160", (3, 7, 7, 160), 960, 160, (1, 1)),
]


@pytest.mark.parametrize("he", [False, True], ids=["half_up", "half_even"])
@pytest.mark.parametrize("xval", [-128, 127])
@pytest.mark.parametrize("case", MB_ROUTES, ids=lambda c: c[0])
def test_fused_blocks_at_the_bounds(oracle, case, xval, he):
    """Every stage of a fused block with per-channel (shift, bias, filter sign) combinations at the bounds."""
    name, shape, ce, cout, stride = case
    announce(f"epilogue bounds {name} x={xval} he={he}")
    m = espdl()
    n, h, w, cin = shape
    rm_g = m.capi.ROUND_HALF_EVEN if he else m.capi.ROUND_HALF_UP
    rm_o = oracle.ROUND_HALF_EVEN if he else oracle.ROUND_HALF_UP
    rng = np.random.default_rng(len(name))

    def stage(oc, fshape, axis):
        shift, bias, wval = _channels(oc)
        pick = rng.permutation(len(shift))[:oc]
        sh = [1] * len(fshape)
        sh[axis] = oc
        f = np.broadcast_to(wval[pick].reshape(sh), fshape).copy()
        flip = rng.random(fshape) < 0.2
        f[flip] = np.where(f[flip] == 127, -128, 127)
        return f, bias[pick].copy(), shift[pick].copy()

    x = np.full(shape, xval, dtype=np.int8)
    x[..., ::3] = 127 if xval == -128 else -128
    ex = stage(ce, (ce, 1, 1, cin), 0)
    cur = oracle.conv2d_s8(x, ex[0], ex[1], ex[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU, rm_o)
    dw = stage(ce, (3, 3, ce), 2)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), stride, (1, 1), (1, 1, 1, 1), oracle.RELU, rm_o)
    pj = stage(cout, (cout, 1, 1, ce), 0)
    cur = oracle.conv2d_s8(cur, pj[0], pj[1], pj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, rm_o)
    res = np.full(cur.shape, 100, dtype=np.int8)
    cur = oracle.add_s8(cur, res)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    got = m.mbconv_s8(to_dev(x), dev(ex), dev(dw), dev(pj), (3, 3), stride, (1, 1), (1, 1, 1, 1), (True, True, False),
                      residual=to_dev(res), round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got), cur)


@pytest.mark.parametrize("k_total", [35984, 36000, 36016])
@pytest.mark.parametrize("value", [-32768, 32767])
def test_conv2d_s16_digit_form_guard(oracle, k_total, value):
    """int16 convolution as signed-byte products on the int8 matrix pipe: its int32 sums stay exact well beyond
    the reductions of at most 36000 it accepts; one case just under that guard and at it, one above it (which
    takes the 64-bit multiply-add kernel), all operands at one extreme - the largest byte sums there are."""
    announce(f"conv2d_s16 K={k_total} value={value}")
    m = espdl()
    x = np.full((1, 2, 3, k_total), value, dtype=np.int16)
    f = np.full((16, 1, 1, k_total), value, dtype=np.int16)
    f[1::2] = -32768 if value == 32767 else 32767
    bias = np.array([(-1) ** i * (1 << 44) for i in range(16)], dtype=np.int64)
    shift = np.full(16, 31, dtype=np.int32)
    want = oracle.conv2d_s16(x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, oracle.ROUND_HALF_UP)
    got = m.conv2d(to_dev(x), to_dev(f), to_dev(bias), to_dev(shift), (1, 1), (1, 1), (1, 1), (0, 0, 0, 0))
    np.testing.assert_array_equal(to_host(got), want)
    assert len(np.unique(want)) > 1
