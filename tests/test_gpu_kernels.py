"""GPU parity: every C-ABI entry point against the CPU oracle on the same seeded inputs.
Bit-exact equality is the bar for all of them (integer / byte work)."""
import ctypes

import numpy as np
import pytest

from cases import CONFIG1, CONV_CASES, DW_CASES, GEMM_CASES, POINTWISE_MANY_PIXELS, WIDE_ROWS, WINDOW_GEMM_CASES, TILED_MANY_PIXELS, STEM_CASES, TILED_CASES, every_sum_image, rng_int8, typical_shift
from gpu_util import announce, espdl, to_dev, to_host

pytestmark = pytest.mark.gpu


def _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, depthwise=False, half_even=False, lut=None,
                 residual_seed=None):
    m = espdl()
    act = m.capi.RELU if relu else m.capi.LINEAR
    rm = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP
    shift = np.atleast_1d(np.asarray(shift, dtype=np.int32))
    fn = oracle.depthwise_s8 if depthwise else oracle.conv2d_s8
    want = fn(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR,
              oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP)
    if lut is not None:
        want = oracle.lut_s8(want, lut)
    residual = None
    if residual_seed is not None:  # Conv -> Add in one launch
        residual = rng_int8(np.random.default_rng(residual_seed), want.shape)
        want = oracle.add_s8(want, residual)
    got = m.conv2d(to_dev(x), to_dev(f), to_dev(bias), to_dev(shift), k, stride, dil, pads, depthwise=depthwise,
                   activation=act, round_mode=rm, lut=to_dev(lut), residual=to_dev(residual))
    return to_host(got), want


def _conv_inputs(case, seed, n, per_channel):
    name, (h, w, c), oc, k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(seed)
    x = rng_int8(rng, (n, h, w, c))
    f = rng_int8(rng, (oc, k[0], k[1], c))
    bias = rng.integers(-4096, 4097, size=oc).astype(np.int32) if has_bias else None
    base = typical_shift(k[0] * k[1] * c)
    shift = (base + rng.integers(-2, 3, size=oc)).astype(np.int32) if per_channel else np.int32(base)
    return x, f, bias, shift, k, stride, dil, pads, relu


@pytest.mark.parametrize("case", CONV_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("per_channel", [False, True], ids=["per_tensor", "per_channel"])
def test_conv2d_s8(oracle, case, per_channel):
    announce(f"conv2d_s8 {case[0]} per_channel={per_channel}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 101, 3, per_channel)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", [CONV_CASES[1], CONV_CASES[2], CONV_CASES[4], CONV_CASES[5], CONV_CASES[11], CONFIG1],
                         ids=lambda c: c[0])
def test_conv2d_s8_residual(oracle, case):
    """Conv followed by a saturating Add of a tensor of the output's shape, in the conv's epilogue:
    16-byte, 4-byte and byte store paths, direct and LDS-staged output."""
    announce(f"conv2d_s8 + residual {case[0]}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 131, 3, True)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, residual_seed=5)
    np.testing.assert_array_equal(got, want)


def test_conv2d_s8_config1(oracle):
    """BASELINE config 1: 1x56x56x64 -> 64, 3x3, s1, p1, bias in [-2^12, 2^12], ReLU, shift 9."""
    announce("conv2d_s8 config1")
    x, f, bias, _, k, stride, dil, pads, relu = _conv_inputs(CONFIG1, 0xE5D1, 1, False)
    got, want = _run_conv_s8(oracle, x, f, bias, 9, k, stride, dil, pads, True)
    assert got.shape == (1, 56, 56, 64)
    np.testing.assert_array_equal(got, want)


def test_conv2d_s8_config1_batched(oracle):
    announce("conv2d_s8 config1 batch 16")
    x, f, bias, _, k, stride, dil, pads, relu = _conv_inputs(CONFIG1, 0xE5D2, 16, False)
    got, want = _run_conv_s8(oracle, x, f, bias, 9, k, stride, dil, pads, True)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", TILED_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("flavour", ["per_tensor", "per_channel", "half_even", "lut_residual", "general_epilogue"])
def test_conv2d_s8_lds_tiled(oracle, case, flavour):
    """Windowed convolutions with a multiple of 16 channels (input tile and filters staged in LDS): both exponent
    forms, round-half-even, table + residual in the epilogue, and shifts outside 1..31 mixed with large biases
    (the general shift-and-round form)."""
    announce(f"conv2d_s8 lds-tiled {case[0]} {flavour}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 211, 3, flavour != "per_tensor")
    kw = {}
    if flavour == "half_even":
        kw["half_even"] = True
    if flavour == "lut_residual":
        kw["lut"] = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
        kw["residual_seed"] = 9
        relu = False
    if flavour == "general_epilogue":
        shift = np.array(shift, dtype=np.int32)
        shift[::3] = 0
        shift[1::5] = 33
        if bias is not None:
            bias = bias.copy()
            bias[::2] = (1 << 30) - 7
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, **kw)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", STEM_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("flavour", ["per_tensor", "per_channel", "half_even", "lut", "general_epilogue"])
def test_conv2d_s8_first_layer(oracle, case, flavour):
    """Few-channel images through the one-MFMA-step kernel: both exponent forms, round-half-even, a table in the
    epilogue, and shifts outside 1..31 mixed with large biases (the general shift-and-round form)."""
    announce(f"conv2d_s8 first layer {case[0]} {flavour}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 223, 3, flavour != "per_tensor")
    kw = {}
    if flavour == "half_even":
        kw["half_even"] = True
    if flavour == "lut":
        kw["lut"] = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
        relu = False
    if flavour == "general_epilogue":
        shift = np.array(shift, dtype=np.int32)
        shift[::3] = 0
        shift[1::5] = 33
        if bias is not None:
            bias = bias.copy()
            bias[::2] = (1 << 30) - 7
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, **kw)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", POINTWISE_MANY_PIXELS, ids=lambda c: c[0])
@pytest.mark.parametrize("flavour", ["per_tensor", "per_channel", "half_even", "lut", "general_epilogue"])
def test_conv2d_s8_pointwise_short_reduction(oracle, case, flavour):
    """Pointwise products over many pixels with at most 128 input channels: both exponent forms, round-half-even,
    a table in the epilogue, the general shift-and-round form."""
    announce(f"conv2d_s8 pointwise short reduction {case[0]} {flavour}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 227, 3, flavour != "per_tensor")
    kw = {}
    if flavour == "half_even":
        kw["half_even"] = True
    if flavour == "lut":
        kw["lut"] = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
        relu = False
    if flavour == "general_epilogue":
        shift = np.array(shift, dtype=np.int32)
        shift[::3] = 0
        shift[1::5] = 33
        if bias is not None:
            bias = bias.copy()
            bias[::2] = (1 << 30) - 7
    oracle.set_threads(16)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, **kw)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", TILED_MANY_PIXELS, ids=lambda c: c[0])
@pytest.mark.parametrize("flavour", ["per_channel", "half_even", "residual"])
def test_conv2d_s8_window_on_many_pixels(oracle, case, flavour):
    """Stride-1 windows over 64 channels or more at a batch that puts them above 128 K output pixels."""
    announce(f"conv2d_s8 window on many pixels {case[0]} {flavour}")
    h, w = case[1][0], case[1][1]
    n = (128 * 1024) // (h * w) + 2
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 257, n, True)
    kw = {}
    if flavour == "half_even":
        kw["half_even"] = True
    if flavour == "residual":
        kw["residual_seed"] = 11
    oracle.set_threads(16)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, **kw)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", WINDOW_GEMM_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("flavour", ["per_tensor", "per_channel", "half_even", "lut", "residual", "general_epilogue"])
def test_conv2d_s8_strided_window_on_few_pixels(oracle, case, flavour):
    """Strided windows over many channels on few pixels (the downsampling convolutions deep in a detector): both
    exponent forms, round-half-even, a table and a residual Add in the epilogue, the general shift-and-round form."""
    announce(f"conv2d_s8 strided window {case[0]} {flavour}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 241, 5, flavour != "per_tensor")
    kw = {}
    if flavour == "half_even":
        kw["half_even"] = True
    if flavour == "lut":
        kw["lut"] = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
        relu = False
    if flavour == "residual":
        kw["residual_seed"] = 7
    if flavour == "general_epilogue":
        shift = np.array(shift, dtype=np.int32)
        shift[::3] = 0
        shift[1::5] = 33
        if bias is not None:
            bias = bias.copy()
            bias[::2] = (1 << 30) - 7
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, **kw)
    np.testing.assert_array_equal(got, want)


def test_conv2d_s8_strided_window_channel_slices(oracle):
    """The same route reading a channel slice of a wider tensor and writing into one (the operands of a Concat)."""
    import torch
    announce("conv2d_s8 strided window channel slices")
    m = espdl()
    rng = np.random.default_rng(251)
    n, h, w, c, oc = 4, 30, 34, 128, 96
    x = rng_int8(rng, (n, h, w, c))
    f = rng_int8(rng, (oc, 3, 3, c))
    bias = rng.integers(-4096, 4097, size=oc).astype(np.int32)
    shift = (typical_shift(9 * c) + rng.integers(-2, 3, size=oc)).astype(np.int32)
    want = oracle.conv2d_s8(x, f, bias, shift, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), oracle.RELU, oracle.ROUND_HALF_UP)
    wide_in = torch.full((n, h, w, c + 64), 55, dtype=torch.int8, device="cuda")
    wide_in[..., 32:32 + c].copy_(torch.from_numpy(x))
    wide_out = torch.full((n, want.shape[1], want.shape[2], oc + 48), 66, dtype=torch.int8, device="cuda")
    m.conv2d(wide_in[..., 32:32 + c], to_dev(f), to_dev(bias), to_dev(shift), (3, 3), (2, 2), (1, 1), (1, 1, 1, 1),
             activation=m.capi.RELU, out=wide_out[..., 16:16 + oc])
    got = to_host(wide_out)
    np.testing.assert_array_equal(got[..., 16:16 + oc], want)
    assert (got[..., :16] == 66).all() and (got[..., 16 + oc:] == 66).all()


@pytest.mark.parametrize("case", WIDE_ROWS, ids=lambda c: c[0])
@pytest.mark.parametrize("flavour", ["per_tensor", "per_channel", "half_even", "lut", "general_epilogue", "mixed_epilogue"])
def test_conv2d_s8_wide_rows(oracle, case, flavour):
    """Short reduction under thousands of filters over many rows (a recognizer's classifier): both exponent forms,
    round-half-even, a table in the epilogue, the general shift-and-round form for every group of 64 filters and for
    some of them only."""
    announce(f"conv2d_s8 wide rows {case[0]} {flavour}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 233, 3, flavour != "per_tensor")
    kw = {}
    if flavour == "half_even":
        kw["half_even"] = True
    if flavour == "lut":
        kw["lut"] = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
        relu = False
    if flavour in ("general_epilogue", "mixed_epilogue"):
        lim = len(shift) if flavour == "general_epilogue" else 700
        shift = np.array(shift, dtype=np.int32)
        shift[:lim:3] = 0
        shift[1:lim:5] = 33
        if bias is not None:
            bias = bias.copy()
            bias[:lim:2] = (1 << 30) - 7
    oracle.set_threads(16)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, **kw)
    np.testing.assert_array_equal(got, want)


def test_conv2d_s8_wide_rows_views(oracle):
    """The same product with an output that starts at an odd address, an input that is a channel slice of a wider
    tensor, and the recognizer's own shape (120 -> 6625) at a sequence count that is not a multiple of 64."""
    import torch
    announce("conv2d_s8 wide rows views")
    m = espdl()
    rng = np.random.default_rng(239)
    rows, c, oc = 16 * 4 * 256 + 37, 120, 6625
    x = rng_int8(rng, (1, 1, rows, c))
    f = rng_int8(rng, (oc, 1, 1, c))
    bias = rng.integers(-4096, 4097, size=oc).astype(np.int32)
    shift = (typical_shift(c) + rng.integers(-2, 3, size=oc)).astype(np.int32)
    oracle.set_threads(16)
    want = oracle.conv2d_s8(x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, oracle.ROUND_HALF_UP)
    wide = torch.zeros((1, 1, rows, c + 24), dtype=torch.int8, device="cuda")
    wide[..., 8:8 + c].copy_(torch.from_numpy(x))
    for offset in (0, 1, 7, 13):
        buf = torch.full((rows * oc + 64,), 77, dtype=torch.int8, device="cuda")
        out = buf[offset:offset + rows * oc].view(1, 1, rows, oc)
        m.conv2d(wide[..., 8:8 + c], to_dev(f), to_dev(bias), to_dev(shift), (1, 1), out=out)
        np.testing.assert_array_equal(to_host(out), want)
        # nothing outside the tensor was written
        assert bool((buf[:offset] == 77).all()) and bool((buf[offset + rows * oc:] == 77).all())


def test_conv2d_s8_first_layer_at_the_tensor_end(oracle):
    """The last pixels of the last row of the last image: their 16-byte reads would end behind the tensor, so
    they are assembled byte by byte.  The input sits at the very end of its allocation."""
    import torch
    announce("conv2d_s8 first layer tensor end")
    m = espdl()
    rng = np.random.default_rng(229)
    n, h, w, c, oc = 2, 33, 47, 3, 16
    x = rng_int8(rng, (n, h, w, c))
    f = rng_int8(rng, (oc, 3, 3, c))
    bias = rng.integers(-4096, 4097, size=oc).astype(np.int32)
    shift = np.full(oc, 9, dtype=np.int32)
    want = oracle.conv2d_s8(x, f, bias, shift, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), oracle.RELU, oracle.ROUND_HALF_UP)
    # a buffer that ends exactly with the tensor (torch rounds allocations up, so the slice ends inside one; what
    # matters is that the kernel never needs the bytes behind)
    buf = torch.empty(x.size + 4096, dtype=torch.int8, device="cuda")
    xd = buf[4096:].view(n, h, w, c)
    xd.copy_(torch.from_numpy(x))
    got = m.conv2d(xd, to_dev(f), to_dev(bias), to_dev(shift), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), activation=m.capi.RELU)
    np.testing.assert_array_equal(to_host(got), want)


# Operands that are channel slices of wider NHWC tensors (what a Conv reads from a Split output and writes into its
# part of a Concat result), on every dense route: (name, (N, H, W), in_c, out_c, k, stride, pads,
# (input offset, input width), (output offset, output width), (residual offset, residual width) or None, lut)
PITCH_CASES = [
    ("pw_few_pixels_64_64", (2, 7, 9), 64, 64, (1, 1), (1, 1), (0, 0, 0, 0), (32, 128), (64, 192), None, False),
    ("pw_few_pixels_120_48_unaligned", (2, 5, 8), 120, 48, (1, 1), (1, 1), (0, 0, 0, 0), (8, 136), (5, 61), (3, 55), False),
    ("pw_rows_64_32", (1, 1, 16), 64, 32, (1, 1), (1, 1), (0, 0, 0, 0), (64, 128), (32, 96), None, False),
    ("pw_many_pixels_32_32", (2, 150, 160), 32, 32, (1, 1), (1, 1), (0, 0, 0, 0), (16, 64), (0, 96), (32, 64), True),
    ("c3_tiled_32_32_residual", (2, 40, 40), 32, 32, (3, 3), (1, 1), (1, 1, 1, 1), (32, 64), (64, 96), (32, 64), True),
    ("c3_tiled_64_64", (3, 30, 30), 64, 64, (3, 3), (1, 1), (1, 1, 1, 1), (0, 128), (64, 128), None, False),
    ("c3s2_tiled_16_40", (2, 33, 35), 16, 40, (3, 3), (2, 2), (1, 1, 1, 1), (16, 48), (8, 56), (0, 40), False),
    ("c3_gather_22_33", (2, 19, 23), 22, 33, (3, 3), (1, 1), (1, 1, 1, 1), (5, 40), (7, 47), (1, 34), False),
    ("c3_direct_256_64", (1, 12, 12), 256, 64, (3, 3), (1, 1), (1, 1, 1, 1), (256, 512), (64, 192), None, True),
]


@pytest.mark.parametrize("case", PITCH_CASES, ids=lambda c: c[0])
def test_conv2d_s8_channel_slices(oracle, case):
    announce(f"conv2d_s8 on channel slices: {case[0]}")
    name, (n, h, w), cin, cout, k, stride, pads, (io, iw), (oo, ow_), res, with_lut = case
    m = espdl()
    import torch
    rng = np.random.default_rng(0x517C + len(name))
    wide_in = rng_int8(rng, (n, h, w, iw))
    x = np.ascontiguousarray(wide_in[..., io:io + cin])
    f = rng_int8(rng, (cout, k[0], k[1], cin))
    bias = rng.integers(-4096, 4097, size=cout).astype(np.int32)
    shift = (typical_shift(k[0] * k[1] * cin) + rng.integers(-2, 3, size=cout)).astype(np.int32)
    want = oracle.conv2d_s8(x, f, bias, shift, k, stride, (1, 1), pads, oracle.RELU, oracle.ROUND_HALF_UP)
    lut = None
    if with_lut:
        lut = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
        want = oracle.lut_s8(want, lut)
    wide_res = None
    if res is not None:
        wide_res = rng_int8(rng, want.shape[:3] + (res[1],))
        want = oracle.add_s8(want, np.ascontiguousarray(wide_res[..., res[0]:res[0] + cout]))
    before = rng_int8(rng, want.shape[:3] + (ow_,))
    d_in, d_out = to_dev(wide_in), to_dev(before)
    d_res = to_dev(wide_res)
    m.conv2d(d_in[..., io:io + cin], to_dev(f), to_dev(bias), to_dev(shift), k, stride, (1, 1), pads, activation=m.capi.RELU,
             lut=to_dev(lut), out=d_out[..., oo:oo + cout], residual=None if res is None else d_res[..., res[0]:res[0] + cout])
    got = to_host(d_out)
    np.testing.assert_array_equal(got[..., oo:oo + cout], want)
    # nothing outside the slice was touched
    keep = np.ones(ow_, dtype=bool)
    keep[oo:oo + cout] = False
    np.testing.assert_array_equal(got[..., keep], before[..., keep])


@pytest.mark.parametrize("shift", [-3, -1, 0, 1, 31, 33])
def test_conv2d_s8_shift_range(oracle, shift):
    announce(f"conv2d_s8 shift={shift}")
    rng = np.random.default_rng(7)
    x = rng.integers(-6, 7, size=(2, 5, 5, 8)).astype(np.int8)
    f = rng.integers(-6, 7, size=(12, 1, 1, 8)).astype(np.int8)
    bias = rng.integers(-50, 51, size=12).astype(np.int32)
    if shift > 8:
        bias = (bias.astype(np.int64) << 24).astype(np.int32)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", [CONV_CASES[5], CONV_CASES[13]], ids=lambda c: c[0])
def test_conv2d_s8_half_even(oracle, case):
    announce(f"conv2d_s8 half-even {case[0]}")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(case, 103, 2, True)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, half_even=True)
    np.testing.assert_array_equal(got, want)


def test_conv2d_s8_fused_lut(oracle):
    announce("conv2d_s8 + LUT epilogue")
    x, f, bias, shift, k, stride, dil, pads, relu = _conv_inputs(CONV_CASES[16], 105, 2, True)
    lut = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, False, lut=lut)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("k_total,oc", [(1280, 1000), (2304, 80), (960, 160), (576, 96)])
def test_conv2d_s8_large_k(oracle, k_total, oc):
    """Reduction lengths that exceed one LDS-resident filter chunk, and 1000 filters (not a multiple of 16)."""
    announce(f"conv2d_s8 large K={k_total} oc={oc}")
    rng = np.random.default_rng(k_total)
    x = rng_int8(rng, (1, 1, 37, k_total))
    f = rng_int8(rng, (oc, 1, 1, k_total))
    bias = rng.integers(-4096, 4097, size=oc).astype(np.int32)
    shift = (typical_shift(k_total) + rng.integers(-1, 2, size=oc)).astype(np.int32)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False)
    np.testing.assert_array_equal(got, want)


# Pointwise layers with few pixels and K % 16 == 0, K >= 64, N >= 32 take the tiled-GEMM kernel:
# (pixels (n, h, w), K, N): pixel tails (M % 128), filter tails (N % 128, % 16, % 4, odd), K tails (K % 64),
# many k steps, one k step.
PWGEMM_CASES = [
    ((2, 14, 14), 64, 384), ((3, 7, 7), 960, 160), ((1, 7, 7), 960, 320), ((2, 14, 14), 576, 96),
    ((1, 1, 256), 1280, 1000), ((1, 5, 9), 80, 40), ((2, 3, 5), 112, 33), ((1, 1, 1), 64, 32),
    ((1, 13, 11), 144, 200), ((4, 14, 14), 96, 576), ((1, 7, 7), 320, 1280),
]


@pytest.mark.parametrize("case", PWGEMM_CASES, ids=lambda c: "x".join(map(str, c[0])) + f"_k{c[1]}_n{c[2]}")
@pytest.mark.parametrize("variant", ["plain", "relu_pc", "half_even", "lut", "residual", "low_shift"])
def test_conv2d_s8_pointwise_tiled_gemm(oracle, case, variant):
    (n, h, w), kk, oc = case
    announce(f"conv2d_s8 pointwise tiled gemm {case} {variant}")
    rng = np.random.default_rng(4242 + kk + oc)
    x = rng_int8(rng, (n, h, w, kk))
    f = rng_int8(rng, (oc, 1, 1, kk))
    bias = rng.integers(-4096, 4097, size=oc).astype(np.int32) if variant != "plain" else None
    base = typical_shift(kk)
    shift = np.int32(base)
    if variant in ("relu_pc", "residual", "half_even"):
        shift = (base + rng.integers(-2, 3, size=oc)).astype(np.int32)
    if variant == "low_shift":  # some shifts below 8 (left-shift form) and one outside 1..31 (general form)
        shift = rng.integers(3, 12, size=oc).astype(np.int32)
        if oc > 40:
            shift[37] = 0
    lut = rng_int8(rng, (256,)) if variant == "lut" else None
    got, want = _run_conv_s8(oracle, x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), variant == "relu_pc",
                             half_even=variant == "half_even", lut=lut,
                             residual_seed=77 if variant == "residual" else None)
    np.testing.assert_array_equal(got, want)


# Round-half-even differs from half-up only at exact ties; small operands and small shifts make ties
# frequent (a quarter to a half of all outputs), on every kernel route that has the short epilogue.
@pytest.mark.parametrize("route", ["dense3x3", "pointwise_tiled", "pointwise_large", "depthwise", "depthwise_s2", "depthwise_5x5"])
@pytest.mark.parametrize("shift_lo,shift_hi", [(1, 3), (2, 9), (8, 10)])
def test_half_even_ties(oracle, route, shift_lo, shift_hi):
    announce(f"half-even ties {route} shifts {shift_lo}..{shift_hi}")
    rng = np.random.default_rng(900 + shift_lo)
    dw = route.startswith("depthwise")
    if route == "dense3x3":
        shape, oc, k, stride, pads = (2, 12, 12, 16), 32, (3, 3), (1, 1), (1, 1, 1, 1)
    elif route == "pointwise_tiled":
        shape, oc, k, stride, pads = (2, 9, 9, 64), 48, (1, 1), (1, 1), (0, 0, 0, 0)
    elif route == "pointwise_large":
        shape, oc, k, stride, pads = (2, 9, 9, 24), 40, (1, 1), (1, 1), (0, 0, 0, 0)
    elif route == "depthwise_5x5":
        shape, oc, k, stride, pads = (2, 18, 18, 32), 32, (5, 5), (1, 1), (2, 2, 2, 2)
    elif route == "depthwise":
        shape, oc, k, stride, pads = (2, 14, 14, 32), 32, (3, 3), (1, 1), (1, 1, 1, 1)
    else:
        shape, oc, k, stride, pads = (2, 15, 15, 48), 48, (3, 3), (2, 2), (1, 1, 1, 1)
    x = rng.integers(-4, 5, size=shape).astype(np.int8)
    f = rng.integers(-4, 5, size=(k[0], k[1], shape[3]) if dw else (oc, k[0], k[1], shape[3])).astype(np.int8)
    bias = rng.integers(-8, 9, size=oc).astype(np.int32)
    shift = rng.integers(shift_lo, shift_hi + 1, size=oc).astype(np.int32)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, (1, 1), pads, False, depthwise=dw, half_even=True)
    np.testing.assert_array_equal(got, want)
    up, _ = _run_conv_s8(oracle, x, f, bias, shift, k, stride, (1, 1), pads, False, depthwise=dw, half_even=False)
    if shift_hi <= 9:
        assert (up != got).mean() > 0.01  # the two modes really differ on this input


@pytest.mark.parametrize("m,k,n,has_bias,relu", GEMM_CASES)
def test_gemm_s8(oracle, m, k, n, has_bias, relu):
    announce(f"gemm_s8 M={m} K={k} N={n}")
    rng = np.random.default_rng(107)
    x = rng_int8(rng, (1, 1, m, k))
    f = rng_int8(rng, (n, 1, 1, k))
    bias = rng.integers(-4096, 4097, size=n).astype(np.int32) if has_bias else None
    shift = (typical_shift(k) + rng.integers(-1, 2, size=n)).astype(np.int32)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), relu)
    np.testing.assert_array_equal(got, want)


# Products with so few rows that the tiled kernels would leave most of the device idle go to a kernel with one
# wavefront per 16 x 16 tile: ragged row and filter counts, byte stores (N not a multiple of 4), one shift for all
# filters, shifts outside 1..31, both roundings.
@pytest.mark.parametrize("m,k,n", [(256, 1280, 1000), (1, 1280, 1000), (70, 64, 37), (33, 576, 129), (512, 128, 32),
                                   (32, 1280, 8), (5, 64, 1), (40, 128, 20)])
@pytest.mark.parametrize("variant", ["per_channel", "per_tensor", "half_even", "wide_shifts"])
def test_conv2d_s8_few_rows(oracle, m, k, n, variant):
    announce(f"conv2d_s8 few rows M={m} K={k} N={n} {variant}")
    rng = np.random.default_rng(0xF3 + m + n)
    x = rng_int8(rng, (m, 1, 1, k))
    f = rng_int8(rng, (n, 1, 1, k))
    bias = rng.integers(-4096, 4097, size=n).astype(np.int32)
    if variant == "per_tensor":
        shift = np.full(1, typical_shift(k), np.int32)
    elif variant == "wide_shifts":
        shift = rng.choice(np.array([-2, 0, 1, 5, typical_shift(k), 20, 31, 33], np.int32), size=n)
    else:
        shift = (typical_shift(k) + rng.integers(-2, 3, size=n)).astype(np.int32)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), variant == "per_tensor",
                             half_even=variant == "half_even")
    np.testing.assert_array_equal(got, want)


def test_gemm_reference_known_answers_on_gpu():
    """The reference-held Gemm vectors, straight through the C ABI."""
    import json
    import os
    announce("gemm reference fixtures")
    m = espdl()
    with open(os.path.join(os.path.dirname(__file__), "golden", "gemm_c_fixtures.json")) as f:
        cases = json.load(f)
    for case in cases:
        _, _, k, n = case["filter_shape"]
        x = np.array(case["input"], dtype=np.int8).reshape(1, 1, 1, k)
        w = np.array(case["filter_bytes"], dtype=np.int8)
        bias = np.array(case["bias"], dtype=np.int32)
        shift = np.array([case["output_exponent"] - case["filter_exponents"][0] - case["input_exponent"]], np.int32)
        act = m.capi.RELU if case["activation"] == "Relu" else m.capi.LINEAR
        got = m.conv2d(to_dev(x), to_dev(w), to_dev(bias), to_dev(shift), (1, 1), activation=act)
        np.testing.assert_array_equal(to_host(got).ravel(), np.array(case["output"], dtype=np.int8))


@pytest.mark.parametrize("case", DW_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("per_channel", [False, True], ids=["per_tensor", "per_channel"])
def test_depthwise_s8(oracle, case, per_channel):
    announce(f"depthwise_s8 {case[0]} per_channel={per_channel}")
    name, (h, w, c), k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(109)
    x = rng_int8(rng, (3, h, w, c))
    f = rng_int8(rng, (k[0], k[1], c))
    bias = rng.integers(-4096, 4097, size=c).astype(np.int32) if has_bias else None
    base = typical_shift(k[0] * k[1])
    shift = (base + rng.integers(-2, 3, size=c)).astype(np.int32) if per_channel else np.int32(base)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, depthwise=True)
    np.testing.assert_array_equal(got, want)


def test_depthwise_s8_config2_shape(oracle):
    announce("depthwise_s8 56x56x144 batch 4")
    rng = np.random.default_rng(111)
    x = rng_int8(rng, (4, 56, 56, 144))
    f = rng_int8(rng, (3, 3, 144))
    bias = rng.integers(-4096, 4097, size=144).astype(np.int32)
    shift = rng.integers(6, 11, size=144).astype(np.int32)
    got, want = _run_conv_s8(oracle, x, f, bias, shift, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, depthwise=True)
    np.testing.assert_array_equal(got, want)


# Geometries aimed at the LDS-tile depthwise kernel: tiles that do not divide the image, channel
# counts whose 16-channel groups split unevenly over workgroups, every tap count up to 12, dilation,
# asymmetric padding, shifts below 8 (left-shift form of the short epilogue), the general epilogue
# (half-even, shift 0 / 32), a fused LUT, per-tensor shift.
# Fields: (name, (N, H, W, C), (kh, kw), stride, dilation, pads, bias, relu, shift_lo, shift_hi, half_even, lut, per_tensor)
DW_TILE_CASES = [
    ("n3_61x45x48_k3p1", (3, 61, 45, 48), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 7, 11, False, False, False),
    ("n2_31x29x32_k3s2p1", (2, 31, 29, 32), (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, False, 8, 12, False, False, False),
    ("n2_33x37x272_k3p1", (2, 33, 37, 272), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 6, 10, False, False, False),
    ("n5_14x14x512_k3p1", (5, 14, 14, 512), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 9, 12, False, False, False),
    ("n9_7x7x960_k3p1", (9, 7, 7, 960), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 9, 12, False, False, False),
    ("n2_40x24x64_k3d2p2", (2, 40, 24, 64), (3, 3), (1, 1), (2, 2), (2, 2, 2, 2), True, True, 8, 11, False, False, False),
    ("n2_25x40x16_k2x2_tailpad", (2, 25, 40, 16), (2, 2), (1, 1), (1, 1), (0, 1, 0, 1), False, False, 5, 9, False, False, False),
    ("n2_20x33x80_k3x4_s12", (2, 20, 33, 80), (3, 4), (1, 2), (1, 1), (1, 1, 2, 1), True, True, 8, 12, False, False, False),
    ("n2_1x100x48_k1x3p1", (2, 1, 100, 48), (1, 3), (1, 1), (1, 1), (0, 0, 1, 1), True, False, 6, 9, False, False, False),
    ("n2_19x19x96_k3p1_halfeven", (2, 19, 19, 96), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 7, 11, True, False, False),
    ("n2_19x19x96_k3p1_wide_shifts", (2, 19, 19, 96), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False, 0, 33, False, False, False),
    ("n2_28x28x192_k3s2p1_lut", (2, 28, 28, 192), (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True, 8, 11, False, True, False),
    ("n2_56x56x144_k3p1_per_tensor", (2, 56, 56, 144), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 9, 9, False, False, True),
    ("n1_112x112x32_k3p1", (1, 112, 112, 32), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 8, 11, False, False, False),
    ("n1_112x112x96_k3s2_tailpad", (1, 112, 112, 96), (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), True, True, 8, 11, False, False, False),
    # more tiles than resident workgroups: a workgroup walks several tiles, the next patch in flight over the
    # current tile's stores
    ("n80_56x56x144_k3p1_many_tiles", (80, 56, 56, 144), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True, 8, 11, False, False, False),
    ("n80_56x56x144_k3p1_many_tiles_halfeven", (80, 56, 56, 144), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False, 6, 11, True, False, False),
    ("n96_57x57x48_k3s2_many_tiles", (96, 57, 57, 48), (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True, 8, 11, False, False, False),
    ("n64_30x30x80_k5p2_many_tiles", (64, 30, 30, 80), (5, 5), (1, 1), (1, 1), (2, 2, 2, 2), True, True, 9, 12, False, False, False),
]


S16_MFMA_CASES = [
    # (name, (n, h, w, c), out_c, k, stride, dil, pads, relu, half_even, values)
    ("pw_80x80_96_64", (2, 40, 40, 96), 64, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False, "random"),
    ("c3_20x20_256_16", (2, 20, 20, 256), 16, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False, "random"),
    ("c3_13x11_16_16", (3, 13, 11, 16), 16, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), False, True, "random"),
    ("pw_7x9_80_80", (2, 7, 9, 80), 80, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False, False, "random"),
    ("pw_9x5_16_4", (2, 9, 5, 16), 4, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False, False, "random"),
    ("c3s2_17x15_32_70", (2, 17, 15, 32), 70, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), True, False, "random"),
    ("c3d2_12x12_48_33", (1, 12, 12, 48), 33, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2), False, True, "random"),
    ("pw_6x6_384_256", (2, 6, 6, 384), 256, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False, "random"),
    # every byte of the operands at its extremes: all -32768, all 32767, and the byte boundaries
    ("extremes_min", (1, 5, 5, 64), 32, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), False, False, "min"),
    ("extremes_max", (1, 5, 5, 64), 32, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), False, False, "max"),
    ("extremes_edges", (1, 6, 6, 32), 16, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False, False, "edges"),
]


@pytest.mark.parametrize("case", S16_MFMA_CASES, ids=lambda c: c[0])
def test_conv2d_s16_matrix_pipe(oracle, case):
    """int16 convolutions whose input channels are a multiple of 16 run as products of signed bytes (high byte,
    low byte - 128) on the int8 MFMA; the 64-bit sums must come out exact whatever the bytes are."""
    announce(f"conv2d_s16 mfma {case[0]}")
    name, (n, h, w, c), oc, k, stride, dil, pads, relu, half_even, values = case
    rng = np.random.default_rng(0x516 + len(name))
    if values == "random":
        x = rng.integers(-32768, 32768, size=(n, h, w, c)).astype(np.int16)
        f = rng.integers(-32768, 32768, size=(oc, k[0], k[1], c)).astype(np.int16)
    else:
        pool = {"min": [-32768], "max": [32767],
                "edges": [-32768, -32513, -32512, -16385, -16384, -257, -256, -255, -129, -128, -127, -1, 0, 1, 127, 128,
                          255, 256, 16383, 16384, 32511, 32512, 32639, 32640, 32767]}[values]
        x = rng.choice(pool, size=(n, h, w, c)).astype(np.int16)
        f = rng.choice(pool, size=(oc, k[0], k[1], c)).astype(np.int16)
    bias = rng.integers(-2**40, 2**40, size=oc).astype(np.int64)
    shift = (typical_shift(k[0] * k[1] * c) + 16 + rng.integers(-2, 3, size=oc)).astype(np.int32)
    m = espdl()
    rm_g = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP
    rm_o = oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP
    got = m.conv2d(to_dev(x), to_dev(f), to_dev(bias), to_dev(shift), k, stride, dil, pads,
                   activation=m.capi.RELU if relu else m.capi.LINEAR, round_mode=rm_g)
    want = oracle.conv2d_s16(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR, rm_o)
    np.testing.assert_array_equal(to_host(got), want)
    assert want.min() < want.max()


@pytest.mark.parametrize("case", DW_TILE_CASES, ids=lambda c: c[0])
def test_depthwise_s8_tiles(oracle, case):
    announce(f"depthwise_s8 tiles {case[0]}")
    name, (n, h, w, c), k, stride, dil, pads, has_bias, relu, s_lo, s_hi, half_even, with_lut, per_tensor = case
    rng = np.random.default_rng(0xD3 + len(name))
    x = rng_int8(rng, (n, h, w, c))
    f = rng_int8(rng, (k[0], k[1], c))
    bias = rng.integers(-4096, 4097, size=c).astype(np.int32) if has_bias else None
    shift = np.int32(s_lo) if per_tensor else rng.integers(s_lo, s_hi + 1, size=c).astype(np.int32)
    lut = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8) if with_lut else None
    got, want = _run_conv_s8(oracle, x, f, bias, shift, k, stride, dil, pads, relu, depthwise=True,
                             half_even=half_even, lut=lut)
    np.testing.assert_array_equal(got, want)


def _run_conv_s16(oracle, x, f, bias, shift, k, stride, dil, pads, relu, depthwise):
    m = espdl()
    act = m.capi.RELU if relu else m.capi.LINEAR
    got = m.conv2d(to_dev(x), to_dev(f), to_dev(bias), to_dev(np.atleast_1d(shift).astype(np.int32)), k, stride, dil,
                   pads, depthwise=depthwise, activation=act)
    fn = oracle.depthwise_s16 if depthwise else oracle.conv2d_s16
    want = fn(x, f, bias, shift, k, stride, dil, pads, oracle.RELU if relu else oracle.LINEAR)
    return to_host(got), want


@pytest.mark.parametrize("case", [CONV_CASES[1], CONV_CASES[4], CONV_CASES[5], CONV_CASES[7], CONV_CASES[12]],
                         ids=lambda c: c[0])
def test_conv2d_s16(oracle, case):
    announce(f"conv2d_s16 {case[0]}")
    name, (h, w, c), oc, k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(113)
    x = rng.integers(-32768, 32768, size=(2, h, w, c)).astype(np.int16)
    f = rng.integers(-32768, 32768, size=(oc, k[0], k[1], c)).astype(np.int16)
    bias = rng.integers(-2**28, 2**28, size=oc).astype(np.int64) if has_bias else None
    shift = (typical_shift(k[0] * k[1] * c) + 16 + rng.integers(-2, 3, size=oc)).astype(np.int32)
    got, want = _run_conv_s16(oracle, x, f, bias, shift, k, stride, dil, pads, relu, False)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", [DW_CASES[1], DW_CASES[2], DW_CASES[5], DW_CASES[10]], ids=lambda c: c[0])
def test_depthwise_s16(oracle, case):
    announce(f"depthwise_s16 {case[0]}")
    name, (h, w, c), k, stride, dil, pads, has_bias, relu = case
    rng = np.random.default_rng(115)
    x = rng.integers(-32768, 32768, size=(2, h, w, c)).astype(np.int16)
    f = rng.integers(-32768, 32768, size=(k[0], k[1], c)).astype(np.int16)
    bias = rng.integers(-2**28, 2**28, size=c).astype(np.int64) if has_bias else None
    shift = (typical_shift(k[0] * k[1]) + 16 + rng.integers(-2, 3, size=c)).astype(np.int32)
    got, want = _run_conv_s16(oracle, x, f, bias, shift, k, stride, dil, pads, relu, True)
    np.testing.assert_array_equal(got, want)


# --------------------------------------------------------------------------- elementwise
SIZES = [1, 7, 8, 15, 16, 63, 64, 1011, 1024, 100003]


@pytest.mark.parametrize("size", SIZES)
def test_lut_s8(oracle, size):
    announce(f"lut_s8 size={size}")
    m = espdl()
    table = np.array([(i * 109 + 37) & 0xFF for i in range(256)], dtype=np.uint8).view(np.int8)
    rng = np.random.default_rng(size)
    x = rng_int8(rng, (size,))
    edge = np.array([-128, -127, -1, 0, 1, 126, 127], dtype=np.int8)
    x[:min(size, 7)] = edge[:min(size, 7)]
    got = to_host(m.lut_s8(to_dev(x), to_dev(table)))
    np.testing.assert_array_equal(got, oracle.lut_s8(x, table))
    # in place, and from an address that is not 16-byte aligned
    import torch
    buf = torch.zeros(size + 3, dtype=torch.int8, device="cuda")
    view = buf[3:]
    view.copy_(torch.from_numpy(x))
    m.lut_s8(view, to_dev(table), out=view)
    np.testing.assert_array_equal(to_host(view), oracle.lut_s8(x, table))


@pytest.mark.parametrize("shift", [-1, 0, 3, 6])
def test_prelu_s8(oracle, shift):
    announce(f"prelu_s8 shift={shift}")
    m = espdl()
    xs, _ = np.meshgrid(np.arange(-128, 128), np.arange(-128, 128), indexing="ij")
    x = xs.astype(np.int8).reshape(1, 16, 16, 256)
    alpha = np.arange(-128, 128).astype(np.int8)
    got = to_host(m.prelu_s8(to_dev(x), to_dev(alpha), shift))
    np.testing.assert_array_equal(got, oracle.prelu_s8(x, alpha, shift))
    rng = np.random.default_rng(3)
    # 20 channels: the per-byte form; 48 and 256: 16 consecutive channels per thread
    for shape in ((1, 20, 20, 20), (3, 9, 11, 48), (2, 5, 5, 256)):
        x = rng_int8(rng, shape)
        alpha = rng_int8(rng, (shape[-1],))
        got = to_host(m.prelu_s8(to_dev(x), to_dev(alpha), shift))
        np.testing.assert_array_equal(got, oracle.prelu_s8(x, alpha, shift))


def test_relu_clip_requantize_s8(oracle):
    announce("relu/clip/requantize")
    m = espdl()
    rng = np.random.default_rng(5)
    x = np.concatenate([np.arange(-128, 128).astype(np.int8), rng_int8(rng, (5000,))])
    xd = to_dev(x)
    np.testing.assert_array_equal(to_host(m.relu_s8(xd)), oracle.relu_s8(x))
    for in_exp, out_exp in ((-6, -5), (-5, -7), (-4, -4), (-7, -3), (-3, -6)):
        np.testing.assert_array_equal(to_host(m.relu_s8(xd, in_exp, out_exp)), oracle.relu_s8(x, in_exp, out_exp))
        np.testing.assert_array_equal(to_host(m.clip_s8(xd, 0, 96, in_exp, out_exp)),
                                      oracle.clip_s8(x, 0, 96, in_exp, out_exp))
        np.testing.assert_array_equal(to_host(m.clip_s8(xd, -100, 127, in_exp, out_exp)),
                                      oracle.clip_s8(x, -100, 127, in_exp, out_exp))
        np.testing.assert_array_equal(to_host(m.requantize_s8(xd, in_exp, out_exp)),
                                      oracle.requantize_s8(x, in_exp, out_exp))


def test_requantize_s8_every_byte_every_shift(oracle):
    """int8 -> int8 for every byte value and every exponent difference from -9 to 9: differences up to 7 take the
    packed-int16 form, larger ones the float expression; sizes with and without a tail of single bytes."""
    announce("requantize_s8 every byte, every shift")
    m = espdl()
    rng = np.random.default_rng(55)
    for size in (256, 256 + 16 * 7 + 5, 4096 + 3):
        x = np.concatenate([np.arange(-128, 128), rng.integers(-128, 128, size=size - 256)]).astype(np.int8)
        xd = to_dev(x)
        for d in range(-9, 10):
            got = to_host(m.requantize_s8(xd, -6, -6 - d))
            np.testing.assert_array_equal(got, oracle.requantize_s8(x, -6, -6 - d), err_msg=f"size {size} d {d}")


@pytest.mark.parametrize("src,dst", [("s8", "s16"), ("s16", "s8"), ("s16", "s16")])
def test_requantize_across_widths(oracle, src, dst):
    """TensorBase::assign between int8 and int16 tensors: same exponent widens / saturates, different
    exponents go through quantize(dequantize(x)) in float32 (oracle/graph_runner.requantize)."""
    import torch
    import graph_runner
    announce(f"requantize {src} -> {dst}")
    m = espdl()
    rng = np.random.default_rng(6)
    if src == "s8":
        x = np.concatenate([np.arange(-128, 128).astype(np.int8), rng_int8(rng, (4099,))])
    else:
        x = np.concatenate([np.arange(-32768, 32768, 7), rng.integers(-32768, 32768, size=4099)]).astype(np.int16)
    code = 5 if dst == "s16" else 3
    tdt = torch.int16 if dst == "s16" else torch.int8
    for in_exp, out_exp in ((-6, -6), (-6, -14), (-14, -6), (-7, -3), (-3, -9), (-12, -13)):
        want = graph_runner.requantize(x, in_exp, out_exp, code)
        got = to_host(m.requantize(to_dev(x), in_exp, out_exp, out_dtype=tdt))
        np.testing.assert_array_equal(got, want, err_msg=f"{in_exp}->{out_exp}")


ADD_SHAPES = [
    ((1, 96, 5, 48), (1, 96, 5, 48)), ((1, 96, 5, 48), (1, 96, 5, 1)), ((1, 96, 5, 1), (1, 96, 5, 48)),
    ((1, 5, 5, 31), (1, 1, 1, 31)), ((2, 3, 4, 5), (1, 1, 1, 1)), ((1, 1, 4, 5), (2, 3, 4, 5)),
    ((1, 1, 4, 5), (2, 3, 1, 1)), ((10, 1, 5, 5), (1, 1, 5, 5)), ((1, 512, 7, 7), (1, 512, 7, 7)),
    ((5,), (1,)), ((2, 5), (2, 1)), ((8, 2, 5), (2, 1)), ((1, 96, 5, 49), (1, 96, 5, 49)),
    ((4, 56, 56, 24), (4, 56, 56, 24)),
    # innermost axis dense or constant in each operand, a multiple of 16 long: 16 bytes per thread
    ((3, 20, 20, 64), (3, 1, 1, 64)), ((3, 1, 1, 64), (3, 20, 20, 64)), ((2, 286, 800), (2, 1, 800)),
    ((4, 7, 32), (1, 7, 1)), ((5, 3, 9, 48), (1, 3, 1, 48)), ((2, 9, 16), (16,)), ((6, 1, 5, 32), (1, 4, 1, 1)),
]


@pytest.mark.parametrize("sa,sb", ADD_SHAPES)
def test_add_s8(oracle, sa, sb):
    announce(f"add_s8 {sa} + {sb}")
    m = espdl()
    rng = np.random.default_rng(len(sa) * 100 + len(sb))
    a, b = rng_int8(rng, sa), rng_int8(rng, sb)
    got = to_host(m.add_s8(to_dev(a), to_dev(b)))
    want = np.clip(a.astype(np.int32) + b.astype(np.int32), -128, 127).astype(np.int8)
    np.testing.assert_array_equal(got, want)
    if a.size == b.size or a.size == 1 or b.size == 1:
        np.testing.assert_array_equal(got.ravel(), oracle.add_s8(a, b).ravel())


@pytest.mark.parametrize("sa,sb", ADD_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("shift,half_even", [(7, False), (7, True), (1, True), (0, False), (-2, False), (12, False)])
def test_mul_s8(oracle, sa, sb, shift, half_even):
    announce(f"mul_s8 {sa} * {sb} shift {shift} half_even={half_even}")
    m = espdl()
    rng = np.random.default_rng(31)
    a, b = rng_int8(rng, sa), rng_int8(rng, sb)
    ab, bb = np.broadcast_arrays(a, b)
    want = oracle.mul_s8(np.ascontiguousarray(ab), np.ascontiguousarray(bb), shift,
                         oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP)
    got = to_host(m.mul_s8(to_dev(a), to_dev(b), shift, m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP))
    np.testing.assert_array_equal(got, want)


def test_global_avg_pool_s8(oracle):
    announce("global_avg_pool_s8")
    m = espdl()
    rng = np.random.default_rng(9)
    for shape in ((3, 7, 7, 1280), (2, 5, 3, 33), (1, 1, 1, 8)):
        x = rng_int8(rng, shape)
        for in_exp, out_exp in ((-4, -5), (-5, -5), (-3, -6), (-6, -4)):
            got = to_host(m.global_avg_pool_s8(to_dev(x), in_exp, out_exp))
            np.testing.assert_array_equal(got, oracle.global_avg_pool_s8(x, in_exp, out_exp))
    x = np.full((1, 7, 7, 64), 127, dtype=np.int8)
    x[..., ::2] = -128
    got = to_host(m.global_avg_pool_s8(to_dev(x), -4, -4))
    np.testing.assert_array_equal(got, oracle.global_avg_pool_s8(x, -4, -4))


@pytest.mark.parametrize("hw", [(3, 3), (7, 7), (2, 5)], ids=["3x3", "7x7", "2x5"])
def test_global_avg_pool_s8_every_sum(oracle, hw):
    """Every sum an image can have, ties included: the operator is float(sum) * scale rounded in float and THEN
    given to round(), so a product that rounds to k + 0.5 in float must not be fused with the + 0.5 (sum -18 over
    3 x 3 at exponents -5 -> -3: the float product is exactly -0.5 and the result 0; a fused multiply-add gives -1)."""
    announce(f"global_avg_pool_s8 every sum {hw}")
    m = espdl()
    x = every_sum_image(*hw)
    for in_exp, out_exp in ((-5, -3), (-4, -4), (-4, -5), (-6, -3), (-3, -6)):
        got = to_host(m.global_avg_pool_s8(to_dev(x), in_exp, out_exp))
        np.testing.assert_array_equal(got, oracle.global_avg_pool_s8(x, in_exp, out_exp), err_msg=f"{in_exp} -> {out_exp}")


def test_bad_arguments_are_rejected():
    announce("argument validation")
    m = espdl()
    import torch
    x = torch.zeros((1, 2, 2, 4), dtype=torch.int8, device="cuda")
    f = torch.zeros((4, 5, 5, 4), dtype=torch.int8, device="cuda")
    s = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(m.EspdlHipError):
        m.conv2d(x, f, None, s, (5, 5))  # window larger than the input
    with pytest.raises(m.EspdlHipError):
        m.conv2d(x, f, None, torch.zeros(3, dtype=torch.int32, device="cuda"), (1, 1))  # n_shift neither 1 nor out_c
    empty = torch.zeros((0, 2, 2, 4), dtype=torch.int8, device="cuda")
    assert m.conv2d(empty, torch.zeros((4, 1, 1, 4), dtype=torch.int8, device="cuda"), None, s, (1, 1)).shape[0] == 0


# --------------------------------------------------------------------------- fused inverted-residual block
# (name, (N, H, W, Cin), Ce (None = no expand stage), Cout, k, stride, pads, residual, half_even, per_tensor)
MBCONV_CASES = [
    ("b8_14x14_64_384_64_res", (3, 14, 14, 64), 384, 64, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    ("b3_56x56_32_144_24_res", (2, 56, 56, 32), 144, 24, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    ("b2_40x40_16_96_24_s2", (2, 40, 40, 16), 96, 24, (3, 3), (2, 2), (1, 1, 1, 1), False, False, False),
    ("b1_30x30_32_noexp_16", (2, 30, 30, 32), None, 16, (3, 3), (1, 1), (1, 1, 1, 1), False, False, False),
    ("b17_7x7_160_960_320", (5, 7, 7, 160), 960, 320, (3, 3), (1, 1), (1, 1, 1, 1), False, False, False),
    ("b14_14x14_96_576_160_s2", (3, 14, 14, 96), 576, 160, (3, 3), (2, 2), (1, 1, 1, 1), False, False, False),
    ("ragged_19x23_32_80_48_res", (2, 19, 23, 32), 80, 48, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    ("tailpad_17x17_32_96_32_s2", (2, 17, 17, 32), 96, 32, (3, 3), (2, 2), (0, 1, 0, 1), False, False, False),
    ("halfeven_14x14_32_192_32_res", (2, 14, 14, 32), 192, 32, (3, 3), (1, 1), (1, 1, 1, 1), True, True, False),
    ("pertensor_28x28_32_192_64", (2, 28, 28, 32), 192, 64, (3, 3), (1, 1), (1, 1, 1, 1), False, False, True),
    # expand -> depthwise -> project [-> Add] inside the LDS-tile depthwise kernel (block input <= 64 channels,
    # at most 256 expanded channels): 24 input channels (one and a half 16-byte units), 64 (four units),
    # 4 (a quarter unit), 48 expanded channels in a 20-channel-wide ragged image
    ("edp_56x56_24_144_24_res", (2, 56, 56, 24), 144, 24, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    ("edp_56x56_24_144_32_s2", (2, 56, 56, 24), 144, 32, (3, 3), (2, 2), (0, 1, 0, 1), False, False, False),
    ("edp_112x112_16_96_24_s2", (1, 112, 112, 16), 96, 24, (3, 3), (2, 2), (0, 1, 0, 1), False, False, False),
    ("edp_14x14_64_256_64_res_halfeven", (3, 14, 14, 64), 256, 64, (3, 3), (1, 1), (1, 1, 1, 1), True, True, False),
    ("edp_9x11_4_16_8", (2, 9, 11, 4), 16, 8, (3, 3), (1, 1), (1, 1, 1, 1), False, False, True),
    ("edp_13x20_20_48_20_res", (2, 13, 20, 20), 48, 20, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    # no expand stage: depthwise -> project [-> Add] inside the LDS-tile depthwise kernel
    ("dwp_56x56_144_24_res", (2, 56, 56, 144), None, 24, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    ("dwp_57x41_96_24_s2", (2, 57, 41, 96), None, 24, (3, 3), (2, 2), (1, 1, 1, 1), False, False, False),
    ("dwp_28x28_192_64_s2", (3, 28, 28, 192), None, 64, (3, 3), (2, 2), (0, 1, 0, 1), False, False, False),
    ("dwp_20x20_256_48_res_halfeven", (2, 20, 20, 256), None, 48, (3, 3), (1, 1), (1, 1, 1, 1), True, True, False),
    ("dwp_112x112_32_16", (1, 112, 112, 32), None, 16, (3, 3), (1, 1), (1, 1, 1, 1), False, False, True),
    # the same form with more tiles than resident workgroups (several tiles per workgroup)
    ("dwp_56x56_144_24_res_many_tiles", (80, 56, 56, 144), None, 24, (3, 3), (1, 1), (1, 1, 1, 1), True, False, False),
    ("dwp_57x41_96_24_s2_many_tiles_halfeven", (96, 57, 41, 96), None, 24, (3, 3), (2, 2), (1, 1, 1, 1), False, True, False),
]


@pytest.mark.parametrize("case", MBCONV_CASES, ids=lambda c: c[0])
def test_mbconv_s8_fused(oracle, case):
    announce(f"mbconv_s8 {case[0]}")
    name, (n, h, w, cin), ce, cout, k, stride, pads, with_res, half_even, per_tensor = case
    m = espdl()
    rng = np.random.default_rng(0xB10C + len(name))
    rm_o = oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP
    rm_g = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP

    def stage(oc, kk, fshape):
        f = rng_int8(rng, fshape)
        b = rng.integers(-4096, 4097, size=oc).astype(np.int32)
        base = typical_shift(kk)
        s = np.full(1, base, np.int32) if per_tensor else (base + rng.integers(-2, 3, size=oc)).astype(np.int32)
        return f, b, s

    x = rng_int8(rng, (n, h, w, cin))
    cur = x
    expand = None
    e = cin
    if ce is not None:
        e = ce
        expand = stage(e, cin, (e, 1, 1, cin))
        cur = oracle.conv2d_s8(cur, expand[0], expand[1], expand[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU, rm_o)
    dw = stage(e, k[0] * k[1], (k[0], k[1], e))
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], k, stride, (1, 1), pads, oracle.RELU, rm_o)
    proj = stage(cout, e, (cout, 1, 1, e))
    cur = oracle.conv2d_s8(cur, proj[0], proj[1], proj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, rm_o)
    res = None
    if with_res:
        res = rng_int8(rng, cur.shape)
        cur = oracle.add_s8(cur, res)
    dev = lambda t: None if t is None else tuple(to_dev(a) for a in t)  # noqa: E731
    got = m.mbconv_s8(to_dev(x), dev(expand), dev(dw), dev(proj), k, stride, (1, 1), pads, (True, True, False),
                      residual=to_dev(res), round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got), cur)


# A Clip with equal exponents between the stages (ReLU6 exported as Clip), inside the launch: the block shapes of
# MobileNetV2 that the one-wavefront-per-tile kernel covers, linear convolutions followed by clamps with a lower
# bound of 0 / below 0 / above 0, one clamp only, a ragged last tile, a requantized residual operand.
# (name, (N, H, W, Cin), Ce, Cout, stride, clip_expand, clip_dw, relus, residual, residual_shift)
CLIP_CASES = [
    ("c2_56x56_24_144_24_relu6", (3, 56, 56, 24), 144, 24, (1, 1), (0, 48), (0, 96), (False, False, False), True, 0),
    ("c2_56x56_24_144_24_relu6_rq", (2, 56, 56, 24), 144, 24, (1, 1), (0, 48), (0, 96), (False, False, False), True, -1),
    ("b2_112x112_16_96_24_s2", (1, 112, 112, 16), 96, 24, (2, 2), (-20, 100), (5, 90), (False, False, False), False, 0),
    ("b4_56x56_24_144_32_s2", (2, 56, 56, 24), 144, 32, (2, 2), (0, 127), None, (True, True, False), False, 0),
    ("b5_28x28_32_192_32_only_dw", (2, 28, 28, 32), 192, 32, (1, 1), None, (-128, 20), (True, False, False), True, 0),
    ("b7_28x28_32_192_64_s2", (3, 28, 28, 32), 192, 64, (2, 2), (0, 31), (0, 31), (False, False, False), False, 0),
    ("ragged_50x56_24_144_24", (2, 50, 56, 24), 144, 24, (1, 1), (0, 48), (0, 96), (False, False, False), True, 0),
]


@pytest.mark.parametrize("staged", [False, True], ids=["single_launch", "staged"])
@pytest.mark.parametrize("case", CLIP_CASES, ids=lambda c: c[0])
def test_mbconv_s8_clip_between_stages(oracle, case, staged):
    announce(f"mbconv_s8 with Clip between the stages: {case[0]} staged={staged}")
    name, (n, h, w, cin), ce, cout, stride, clip_e, clip_d, relus, with_res, res_shift = case
    if staged and res_shift != 0:
        pytest.skip("the staged form adds the residual operand as it is")
    m = espdl()
    import torch
    rng = np.random.default_rng(0xC11F + len(name))

    def stage(oc, kk, fshape):
        f = rng_int8(rng, fshape)
        b = rng.integers(-4096, 4097, size=oc).astype(np.int32)
        s = (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32)
        return f, b, s

    act = lambda r: oracle.RELU if r else oracle.LINEAR  # noqa: E731
    x = rng_int8(rng, (n, h, w, cin))
    expand = stage(ce, cin, (ce, 1, 1, cin))
    cur = oracle.conv2d_s8(x, expand[0], expand[1], expand[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), act(relus[0]))
    if clip_e is not None:
        cur = oracle.clip_s8(cur, clip_e[0], clip_e[1], 0, 0)
    dw = stage(ce, 9, (3, 3, ce))
    pads = (1, 1, 1, 1) if stride == (1, 1) else (0, 1, 0, 1)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), stride, (1, 1), pads, act(relus[1]))
    if clip_d is not None:
        cur = oracle.clip_s8(cur, clip_d[0], clip_d[1], 0, 0)
    proj = stage(cout, ce, (cout, 1, 1, ce))
    cur = oracle.conv2d_s8(cur, proj[0], proj[1], proj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), act(relus[2]))
    res = None
    if with_res:
        res = rng_int8(rng, cur.shape)
        cur = oracle.add_s8(cur, oracle.requantize_s8(res, res_shift, 0) if res_shift else res)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    out = torch.empty(cur.shape, dtype=torch.int8, device="cuda")
    got = m.mbconv_s8(to_dev(x), dev(expand), dev(dw), dev(proj), (3, 3), stride, (1, 1), pads, relus,
                      residual=to_dev(res), residual_shift=res_shift, clip_expand=clip_e, clip_dw=clip_d, out=out,
                      staged=staged)
    np.testing.assert_array_equal(to_host(got), cur)


def test_mbconv_s8_clip_is_refused_where_not_covered():
    """Shapes without a guard-free build of the one-wavefront-per-tile kernel, and round half even, answer 0 /
    ESPDL_HIP_ENOTSUP when a Clip sits between the stages."""
    m = espdl()
    import torch
    for shape, ce, cout, rm in (((1, 14, 14, 96), 576, 96, m.capi.ROUND_HALF_UP), ((1, 50, 50, 24), 144, 40, m.capi.ROUND_HALF_UP),
                                ((1, 56, 56, 24), 144, 24, m.capi.ROUND_HALF_EVEN)):
        n, h, w, c = shape
        d = m.capi.MbconvDesc(n, h, w, c, ce, cout, 1, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0, 0, 0, rm, 1, 1, 1)
        d.clip_expand, d.clip_expand_min, d.clip_expand_max = 1, 0, 48
        assert m.lib().espdl_hip_mbconv_s8_supported(ctypes.byref(d)) == 0, shape
        x = torch.zeros(shape, dtype=torch.int8, device="cuda")
        z = lambda *s: torch.zeros(s, dtype=torch.int8, device="cuda")  # noqa: E731
        sh = torch.full((1,), 8, dtype=torch.int32, device="cuda")
        with pytest.raises(m.EspdlHipError, match="Clip"):
            m.mbconv_s8(x, (z(ce, c), None, sh), (z(3, 3, ce), None, sh), (z(cout, ce), None, sh), (3, 3), (1, 1), (1, 1),
                        (1, 1, 1, 1), (False, False, False), round_mode=rm, clip_expand=(0, 48))


# Expand stage with a window: a stem convolution in front of the first depthwise stage, in the block's launch.
# (name, (N, H, W, Cin), expand (kernel, stride, pads), Ce, Cout, depthwise stride, depthwise pads, residual, half_even)
ROWCONV_CASES = [
    ("stem_64x64_rgb_s2_32_16", (2, 64, 64, 3), ((3, 3), (2, 2), (1, 1, 1, 1)), 32, 16, (1, 1), (1, 1, 1, 1), False, False),
    ("stem_224x224_rgb_s2_32_16", (1, 224, 224, 3), ((3, 3), (2, 2), (1, 1, 1, 1)), 32, 16, (1, 1), (1, 1, 1, 1), False, False),
    ("stem_tailpad_65x47_rgb_s2", (2, 65, 47, 3), ((3, 3), (2, 2), (0, 1, 0, 1)), 32, 24, (1, 1), (1, 1, 1, 1), False, False),
    ("stem_gray_33x40_s1_16_8", (2, 33, 40, 1), ((3, 3), (1, 1), (1, 1, 1, 1)), 16, 8, (2, 2), (0, 1, 0, 1), False, False),
    ("stem_2ch_4x2window_30x31", (3, 30, 31, 2), ((4, 2), (2, 1), (1, 2, 0, 1)), 48, 48, (1, 1), (1, 1, 1, 1), True, False),
    ("stem_halfeven_50x50_rgb_s2", (2, 50, 50, 3), ((3, 3), (2, 2), (1, 1, 1, 1)), 32, 16, (1, 1), (1, 1, 1, 1), False, True),
    ("stem_nopad_21x21_rgb_s1_res", (2, 21, 21, 3), ((2, 3), (1, 1), (0, 0, 0, 0)), 32, 32, (1, 1), (1, 1, 1, 1), True, False),
    ("stem_tiny_5x5_rgb", (3, 5, 5, 3), ((3, 3), (2, 2), (1, 1, 1, 1)), 16, 4, (1, 1), (1, 1, 1, 1), False, False),
    # at most 16 project filters at depthwise stride 1: the build that copies the image rows under a tile's windows
    # into LDS one tile ahead (other channel counts, windows, strides, paddings and odd image sizes than the stem's)
    ("rows_gray_40x44_s1_16_8", (2, 40, 44, 1), ((3, 3), (1, 1), (1, 1, 1, 1)), 16, 8, (1, 1), (1, 1, 1, 1), False, False),
    ("rows_2ch_4x2window_50x37_res", (2, 50, 37, 2), ((4, 2), (2, 1), (1, 2, 0, 1)), 32, 16, (1, 1), (1, 1, 1, 1), True, False),
    ("rows_nopad_67x61_rgb_s2_halfeven", (2, 67, 61, 3), ((3, 3), (2, 2), (0, 0, 0, 0)), 32, 16, (1, 1), (1, 1, 1, 1), False, True),
    ("rows_4ch_3x2window_36x36", (1, 36, 36, 4), ((3, 2), (1, 1), (1, 1, 0, 1)), 48, 12, (1, 1), (1, 1, 1, 1), False, False),
    ("rows_odd_image_bytes_33x35_rgb_s2", (5, 33, 35, 3), ((3, 3), (2, 2), (1, 1, 1, 1)), 32, 16, (1, 1), (1, 1, 1, 1), False, False),
    ("rows_many_tiles_130x126_rgb_s2", (3, 130, 126, 3), ((3, 3), (2, 2), (1, 1, 1, 1)), 32, 16, (1, 1), (1, 1, 1, 1), False, False),
]


@pytest.mark.parametrize("staged", [False, True], ids=["single_launch", "staged"])
@pytest.mark.parametrize("case", ROWCONV_CASES, ids=lambda c: c[0])
def test_mbconv_s8_expand_with_window(oracle, case, staged):
    announce(f"mbconv_s8 expand stage with a window: {case[0]} staged={staged}")
    name, (n, h, w, cin), (ek, es, ep), ce, cout, stride, pads, with_res, half_even = case
    m = espdl()
    import torch
    rng = np.random.default_rng(0x57E4 + len(name))
    rm_o = oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP
    rm_g = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP

    def stage(oc, kk, fshape):
        f = rng_int8(rng, fshape)
        b = rng.integers(-4096, 4097, size=oc).astype(np.int32)
        s = (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32)
        return f, b, s

    x = rng_int8(rng, (n, h, w, cin))
    x[:, 0, :, :] = 127   # make the borders count: a wrongly placed or unmasked byte changes the result
    x[:, :, 0, :] = -128
    expand = stage(ce, ek[0] * ek[1] * cin, (ce, ek[0], ek[1], cin))
    cur = oracle.conv2d_s8(x, expand[0], expand[1], expand[2], ek, es, (1, 1), ep, oracle.RELU, rm_o)
    dw = stage(ce, 9, (3, 3, ce))
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), stride, (1, 1), pads, oracle.RELU, rm_o)
    proj = stage(cout, ce, (cout, 1, 1, ce))
    cur = oracle.conv2d_s8(cur, proj[0], proj[1], proj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, rm_o)
    res = None
    if with_res:
        res = rng_int8(rng, cur.shape)
        cur = oracle.add_s8(cur, res)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    out = torch.empty(cur.shape, dtype=torch.int8, device="cuda")
    got = m.mbconv_s8(to_dev(x), dev(expand), dev(dw), dev(proj), (3, 3), stride, (1, 1), pads, (True, True, False),
                      residual=to_dev(res), round_mode=rm_g, out=out, staged=staged, expand_conv=(ek, es, ep))
    np.testing.assert_array_equal(to_host(got), cur)


def test_mbconv_s8_expand_with_window_unaligned_images(oracle):
    """Image sizes whose byte count is not a multiple of four: every image but the first starts at an odd address."""
    announce("mbconv_s8 expand stage with a window, images at unaligned addresses")
    m = espdl()
    rng = np.random.default_rng(0xA11)
    n, h, w, cin, ce, cout = 5, 9, 7, 3, 16, 8
    x = rng_int8(rng, (n, h, w, cin))
    f = lambda oc, kk, shape: (rng_int8(rng, shape), rng.integers(-999, 999, size=oc).astype(np.int32),  # noqa: E731
                               (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32))
    ex, dw, pj = f(ce, 27, (ce, 3, 3, cin)), f(ce, 9, (3, 3, ce)), f(cout, ce, (cout, 1, 1, ce))
    cur = oracle.conv2d_s8(x, ex[0], ex[1], ex[2], (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), oracle.RELU)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), oracle.RELU)
    want = oracle.conv2d_s8(cur, pj[0], pj[1], pj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    got = m.mbconv_s8(to_dev(x), dev(ex), dev(dw), dev(pj), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), (True, True, False),
                      expand_conv=((3, 3), (1, 1), (1, 1, 1, 1)))
    np.testing.assert_array_equal(to_host(got), want)


def test_mbconv_s8_expand_with_window_is_refused_where_not_covered():
    announce("mbconv_s8 expand stage with a window: unsupported shapes are refused")
    m = espdl()
    d = m.capi.MbconvDesc()
    d.batch, d.in_h, d.in_w, d.in_c, d.exp_c, d.out_c, d.has_expand = 2, 32, 32, 8, 32, 16, 1
    d.k_h = d.k_w = 3
    d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
    d.pad_top = d.pad_bottom = d.pad_left = d.pad_right = 1
    d.n_shift_expand = d.n_shift_dw = d.n_shift_project = 1
    d.exp_k_h = d.exp_k_w = 3
    d.exp_stride_h = d.exp_stride_w = 2
    d.exp_pad_top = d.exp_pad_bottom = d.exp_pad_left = d.exp_pad_right = 1
    assert m.capi.lib().espdl_hip_mbconv_s8_supported(ctypes.byref(d)) == 0  # filter rows of 24 bytes
    d.in_c = 3
    assert m.capi.lib().espdl_hip_mbconv_s8_supported(ctypes.byref(d)) == 4
    d.has_expand = 0
    d.exp_c = 3
    assert m.capi.lib().espdl_hip_mbconv_s8_supported(ctypes.byref(d)) == 0  # a window without an expand stage


# The guard-free builds are picked at batches that fill the device; here with image sizes that leave ragged
# last tiles in both directions (rows computed and not stored, columns masked).
# The eight-wavefront kernel (answer 5 of espdl_hip_mbconv_s8_supported) has builds for one count of project pixel
# tiles per wavefront (MobileNetV2's output channel counts) and builds for any count: other output channel
# counts below, and a 13 x 13 image whose second tile has six rows.
# (name, (N, H, W, Cin), Ce, Cout, stride, residual, half_even, answer of espdl_hip_mbconv_s8_supported)
GUARD_FREE_RAGGED = [
    ("pack4_110x110_16_96_24_s2", (80, 110, 110, 16), 96, 24, 2, False, False, 4),
    ("pack2_54x54_24_144_24_s1_res", (80, 54, 54, 24), 144, 24, 1, True, False, 4),
    ("pack2_54x54_24_144_32_s2_halfeven", (96, 54, 54, 24), 144, 32, 2, False, True, 4),
    ("pack2_27x27_32_192_32_s1_res", (300, 27, 27, 32), 192, 32, 1, True, False, 4),
    ("group_13x13_64_384_64_s1_res", (70, 13, 13, 64), 384, 64, 1, True, False, 5),
    ("group_14x14_64_384_32_s1", (66, 14, 14, 64), 384, 32, 1, False, False, 5),
    ("group_14x14_96_576_64_s1_halfeven", (66, 14, 14, 96), 576, 64, 1, False, True, 5),
    ("group_13x13_96_576_96_s1_res", (40, 13, 13, 96), 576, 96, 1, True, False, 5),
    ("group_14x14_96_576_48_s2", (70, 14, 14, 96), 576, 48, 2, False, False, 5),
    ("group_7x7_160_960_64_s1", (130, 7, 7, 160), 960, 64, 1, False, False, 5),
    ("group_7x7_160_960_96_s1_halfeven", (130, 7, 7, 160), 960, 96, 1, False, True, 5),
    # image sizes of MobileNetV2 at 192 and 160 pixels and a 50 x 50 block: tile plans rounded up to the widths
    # and heights the guard-free builds are made for (14 or 7 columns, 8 / 7 / 4 rows)
    ("wave_96x96_16_96_24_s2", (8, 96, 96, 16), 96, 24, 2, False, False, 4),
    ("wave_48x48_24_144_24_s1_res", (12, 48, 48, 24), 144, 24, 1, True, False, 4),
    ("wave_50x50_24_144_24_s1_res", (12, 50, 50, 24), 144, 24, 1, True, True, 4),
    ("wave_40x40_24_144_32_s2", (12, 40, 40, 24), 144, 32, 2, False, False, 4),
    ("wave_24x24_32_192_32_s1_res", (30, 24, 24, 32), 192, 32, 1, True, False, 4),
    ("wave_20x20_32_192_64_s2", (30, 20, 20, 32), 192, 64, 2, False, False, 4),
    ("group_12x12_64_384_64_s1_res", (40, 12, 12, 64), 384, 64, 1, True, False, 5),
    ("group_10x10_96_576_96_s1_res_halfeven", (40, 10, 10, 96), 576, 96, 1, True, True, 5),
    ("group_12x12_96_576_160_s2", (40, 12, 12, 96), 576, 160, 2, False, False, 5),
    ("group_10x10_96_576_160_s2", (40, 10, 10, 96), 576, 160, 2, False, False, 5),
    ("group_6x6_160_960_160_s1_res", (60, 6, 6, 160), 960, 160, 1, True, False, 5),
    ("group_5x5_160_960_320_s1", (60, 5, 5, 160), 960, 320, 1, False, False, 5),
]


@pytest.mark.parametrize("case", GUARD_FREE_RAGGED, ids=lambda c: c[0])
def test_mbconv_s8_guard_free_builds_ragged_tiles(oracle, case):
    announce(f"mbconv_s8 guard-free build, ragged tiles: {case[0]}")
    name, (n, h, w, cin), ce, cout, stride, with_res, half_even, answer = case
    m = espdl()
    d = _block_desc(m, n, h, cin, ce, cout, stride, half_even)
    assert m.capi.lib().espdl_hip_mbconv_s8_supported(ctypes.byref(d)) == answer
    rng = np.random.default_rng(0x9A6 + len(name))
    rm_o = oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP
    rm_g = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP
    oracle.set_threads(16)

    def stage(oc, kk, fshape):
        return (rng_int8(rng, fshape), rng.integers(-4096, 4097, size=oc).astype(np.int32),
                (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32))

    x = rng_int8(rng, (n, h, w, cin))
    ex, dw, pj = stage(ce, cin, (ce, 1, 1, cin)), stage(ce, 9, (3, 3, ce)), stage(cout, ce, (cout, 1, 1, ce))
    pads = (1, 1, 1, 1)
    cur = oracle.conv2d_s8(x, ex[0], ex[1], ex[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU, rm_o)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), (stride, stride), (1, 1), pads, oracle.RELU, rm_o)
    cur = oracle.conv2d_s8(cur, pj[0], pj[1], pj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, rm_o)
    res = None
    if with_res:
        res = rng_int8(rng, cur.shape)
        cur = oracle.add_s8(cur, res)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    got = m.mbconv_s8(to_dev(x), dev(ex), dev(dw), dev(pj), (3, 3), (stride, stride), (1, 1), pads, (True, True, False),
                      residual=to_dev(res), round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got), cur)


# 1x1 convolution followed by GlobalAveragePool in one launch against the two operators of the oracle: the head of
# MobileNetV2 (7 x 7 x 320 -> 1280), an image of 64 pixels, one of 1 pixel, a filter count that is no multiple of
# 64, both rounding modes, a linear convolution, shifts outside the short epilogue's range, and a batch large
# enough for the build that takes two images per workgroup (odd, so that the last workgroup has one).
GAP_CASES = [
    ("head_7x7_320_1280", (37, 7, 7, 320), 1280, True, False, 0),
    ("head_two_images_per_group_odd_batch", (53, 7, 7, 320), 1280, True, False, 0),
    ("full_8x8_64_96", (5, 8, 8, 64), 96, True, False, 0),
    ("one_pixel_128_40", (9, 1, 1, 128), 40, False, False, 0),
    ("half_even_5x5_80_100", (6, 5, 5, 80), 100, True, True, 0),
    ("general_shifts_3x3_64_64", (4, 3, 3, 64), 64, False, False, 1),
    # enough images for four per workgroup, the last workgroup holding three
    ("four_images_per_group_7x7_64_1280", (207, 7, 7, 64), 1280, True, False, 0),
    ("four_images_per_group_half_even_6x6_128_1300", (210, 6, 6, 128), 1300, False, True, 0),
    ("four_images_per_group_general_shifts_8x8", (206, 8, 8, 64), 1290, True, False, 1),
]


@pytest.mark.parametrize("case", GAP_CASES, ids=lambda c: c[0])
@pytest.mark.parametrize("exps", [(-4, -4), (-5, -3), (-3, -6)], ids=["same_exp", "coarser", "finer"])
def test_conv2d_gap_s8(oracle, case, exps):
    announce(f"conv2d_gap_s8 {case[0]} exponents {exps}")
    name, (n, h, w, cin), cout, relu, half_even, odd_shifts = case
    m = espdl()
    rng = np.random.default_rng(0x6A9 + len(name) + exps[1])
    x = rng_int8(rng, (n, h, w, cin))
    f = rng_int8(rng, (cout, 1, 1, cin))
    b = rng.integers(-4096, 4097, size=cout).astype(np.int32)
    s = (typical_shift(cin) + rng.integers(-2, 3, size=cout)).astype(np.int32)
    if odd_shifts:
        s[::5] = 0
        s[2::9] = 33
    rm_o = oracle.ROUND_HALF_EVEN if half_even else oracle.ROUND_HALF_UP
    rm_g = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP
    conv = oracle.conv2d_s8(x, f, b, s, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU if relu else oracle.LINEAR, rm_o)
    want = oracle.global_avg_pool_s8(conv, exps[0], exps[1]).reshape(n, cout)
    got = m.conv2d_gap_s8(to_dev(x), to_dev(f), to_dev(b), to_dev(s), exps[0], exps[1],
                          activation=m.capi.RELU if relu else m.capi.LINEAR, round_mode=rm_g)
    np.testing.assert_array_equal(to_host(got), want)
    assert len(np.unique(want)) > 3  # not degenerate


# A residual operand at another exponent than the block output: the kernels requantize it in registers, as the
# RequantizeLinear node in front of the Add would (every shift the descriptor allows; wave and group kernels).
@pytest.mark.parametrize("shape", [(40, 28, 28, 32, 192, 32), (40, 14, 14, 64, 384, 64), (3, 20, 20, 8, 48, 8)],
                         ids=["wave_28x28", "group_14x14", "wave_guarded_20x20"])
@pytest.mark.parametrize("shift", [-7, -3, -1, 1, 2, 7])
def test_mbconv_s8_requantized_residual(oracle, shape, shift):
    announce(f"mbconv_s8 residual requantized by 2^{shift}, {shape}")
    n, h, w, cin, ce, cout = shape
    m = espdl()
    rng = np.random.default_rng(0x5E51 + shift + h)
    oracle.set_threads(16)

    def stage(oc, kk, fshape):
        return (rng_int8(rng, fshape), rng.integers(-4096, 4097, size=oc).astype(np.int32),
                (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32))

    x = rng_int8(rng, (n, h, w, cin))
    ex, dw, pj = stage(ce, cin, (ce, 1, 1, cin)), stage(ce, 9, (3, 3, ce)), stage(cout, ce, (cout, 1, 1, ce))
    pads = (1, 1, 1, 1)
    cur = oracle.conv2d_s8(x, ex[0], ex[1], ex[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), (1, 1), (1, 1), pads, oracle.RELU)
    cur = oracle.conv2d_s8(cur, pj[0], pj[1], pj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR)
    res = rng_int8(rng, cur.shape)
    res[0, 0, 0, :8] = [-128, -127, -1, 0, 1, 63, 64, 127][:min(8, cout)]
    want = oracle.add_s8(cur, oracle.requantize_s8(res, shift, 0))
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    got = m.mbconv_s8(to_dev(x), dev(ex), dev(dw), dev(pj), (3, 3), (1, 1), (1, 1), pads, (True, True, False),
                      residual=to_dev(res), residual_shift=shift)
    np.testing.assert_array_equal(to_host(got), want)


# Half-even in the block kernels: small operands and small shifts put exact ties in a large share of the outputs of
# every stage; shifts below 8 take the epilogue form with the left shift, a range across 8 mixes both in one stage.
@pytest.mark.parametrize("shape", [(3, 28, 28, 32, 192, 32), (3, 14, 14, 64, 384, 64), (2, 7, 7, 160, 960, 160)],
                         ids=["wave_28x28", "group_14x14", "group_7x7"])
@pytest.mark.parametrize("shift_lo,shift_hi", [(1, 3), (2, 9)])
def test_mbconv_s8_half_even_ties(oracle, shape, shift_lo, shift_hi):
    announce(f"mbconv_s8 half-even ties {shape} shifts {shift_lo}..{shift_hi}")
    n, h, w, cin, ce, cout = shape
    m = espdl()
    rng = np.random.default_rng(0x71E5 + shift_lo + h)

    def stage(oc, fshape):
        return (rng.integers(-2, 3, size=fshape).astype(np.int8), rng.integers(-8, 9, size=oc).astype(np.int32),
                rng.integers(shift_lo, shift_hi + 1, size=oc).astype(np.int32))

    x = rng.integers(-6, 7, size=(n, h, w, cin)).astype(np.int8)
    ex, dw, pj = stage(ce, (ce, 1, 1, cin)), stage(ce, (3, 3, ce)), stage(cout, (cout, 1, 1, ce))
    res = rng.integers(-6, 7, size=(n, h, w, cout)).astype(np.int8)
    pads = (1, 1, 1, 1)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    results = {}
    for name, rm_o, rm_g in (("even", oracle.ROUND_HALF_EVEN, m.capi.ROUND_HALF_EVEN),
                             ("up", oracle.ROUND_HALF_UP, m.capi.ROUND_HALF_UP)):
        cur = oracle.conv2d_s8(x, ex[0], ex[1], ex[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU, rm_o)
        cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), (1, 1), (1, 1), pads, oracle.RELU, rm_o)
        cur = oracle.conv2d_s8(cur, pj[0], pj[1], pj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR, rm_o)
        want = oracle.add_s8(cur, res)
        got = m.mbconv_s8(to_dev(x), dev(ex), dev(dw), dev(pj), (3, 3), (1, 1), (1, 1), pads, (True, True, False),
                          residual=to_dev(res), round_mode=rm_g)
        np.testing.assert_array_equal(to_host(got), want)
        results[name] = want
    assert (results["even"] != results["up"]).mean() > 0.01  # the two modes really differ on this input


def _block_desc(m, batch, hw, cin, ce, cout, stride, half_even=False):
    d = m.capi.MbconvDesc()
    d.batch, d.in_h, d.in_w, d.in_c, d.exp_c, d.out_c, d.has_expand = batch, hw, hw, cin, ce, cout, 1
    d.k_h = d.k_w = 3
    d.stride_h = d.stride_w = stride
    d.dil_h = d.dil_w = 1
    d.pad_top = d.pad_bottom = d.pad_left = d.pad_right = 1
    d.act_expand = d.act_dw = m.capi.RELU
    d.round_mode = m.capi.ROUND_HALF_EVEN if half_even else m.capi.ROUND_HALF_UP
    d.n_shift_expand, d.n_shift_dw, d.n_shift_project = ce, ce, cout
    return d


def test_mbconv_s8_preferred_follows_the_fast_builds():
    """dl::Model fuses a block where espdl_hip_mbconv_s8_preferred says so: yes for MobileNetV2's block shapes
    in both rounding modes, at a batch that fills the device and at a small one (the tile plan keeps the height
    that has a guard-free build), and for the same blocks at other image sizes (their tiles are rounded up to the
    ones the builds are made for); no for a shape that only the guarded builds take (they cover it, but the
    separate launches are as fast)."""
    announce("mbconv_s8_preferred")
    m = espdl()
    L = m.capi.lib()
    pref = lambda d: L.espdl_hip_mbconv_s8_preferred(ctypes.byref(d))  # noqa: E731
    kind = lambda d: L.espdl_hip_mbconv_s8_supported(ctypes.byref(d))  # noqa: E731
    blocks = [(112, 16, 96, 24, 2, 4), (56, 24, 144, 24, 1, 4), (56, 24, 144, 32, 2, 4), (28, 32, 192, 32, 1, 4),
              (28, 32, 192, 64, 2, 4), (14, 64, 384, 64, 1, 5), (14, 96, 576, 96, 1, 5), (14, 96, 576, 160, 2, 5),
              (7, 160, 960, 160, 1, 5), (7, 160, 960, 320, 1, 5)]
    for hw, cin, ce, cout, stride, want_kind in blocks:
        for he in (False, True):
            d = _block_desc(m, 256, hw, cin, ce, cout, stride, he)
            assert kind(d) == want_kind, (hw, cin, ce, cout, stride)
            assert pref(d) == 1, (hw, cin, ce, cout, stride, he)
        for small in (1, 4, 64):
            assert pref(_block_desc(m, small, hw, cin, ce, cout, stride)) == 1, (small, hw, cin, ce, cout, stride)
    # other image sizes are rounded up to the tiles the guard-free builds are made for: a 50 x 50 block, and the
    # blocks of MobileNetV2 at 192 and 160 pixels
    for hw, cin, ce, cout, stride, want_kind in [(50, 24, 144, 24, 1, 4), (96, 16, 96, 24, 2, 4), (48, 24, 144, 24, 1, 4),
                                                 (48, 24, 144, 32, 2, 4), (24, 32, 192, 32, 1, 4), (24, 32, 192, 64, 2, 4),
                                                 (12, 64, 384, 64, 1, 5), (12, 96, 576, 96, 1, 5), (12, 96, 576, 160, 2, 5),
                                                 (6, 160, 960, 160, 1, 5), (80, 16, 96, 24, 2, 4), (40, 24, 144, 24, 1, 4),
                                                 (20, 32, 192, 32, 1, 4), (10, 64, 384, 96, 1, 5), (5, 160, 960, 320, 1, 5)]:
        for he in (False, True):
            d = _block_desc(m, 256, hw, cin, ce, cout, stride, he)
            assert kind(d) == want_kind and pref(d) == 1, (hw, cin, ce, cout, stride, he)
    odd = _block_desc(m, 256, 50, 24, 144, 40, 1)  # three project row tiles: no guard-free build has them
    assert kind(odd) == 4 and pref(odd) == 0


@pytest.mark.parametrize("ce", [320, 192], ids=["e320_block_kernel", "e192_lds_tile_kernel"])
@pytest.mark.parametrize("general_stage", [0, 1, 2], ids=["expand_general", "dw_general", "project_general"])
def test_mbconv_s8_mixed_epilogues(oracle, general_stage, ce):
    """One stage has shifts outside 1..31 (general shift_and_round form), the other two take the
    short epilogue: the per-stage choice must not leak between stages."""
    announce(f"mbconv_s8 mixed epilogues, general stage {general_stage}, {ce} expanded channels")
    m = espdl()
    rng = np.random.default_rng(77 + general_stage)
    n, h, w, cin, cout = 2, 14, 14, 32, 48
    x = rng_int8(rng, (n, h, w, cin))

    def stage(idx, oc, kk, fshape):
        f = rng_int8(rng, fshape)
        b = rng.integers(-4096, 4097, size=oc).astype(np.int32)
        s = (typical_shift(kk) + rng.integers(-2, 3, size=oc)).astype(np.int32)
        if idx == general_stage:
            s[::7] = 0
            s[3::11] = 33
        return f, b, s

    ex = stage(0, ce, cin, (ce, 1, 1, cin))
    dw = stage(1, ce, 9, (3, 3, ce))
    pj = stage(2, cout, ce, (cout, 1, 1, ce))
    cur = oracle.conv2d_s8(x, ex[0], ex[1], ex[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.RELU)
    cur = oracle.depthwise_s8(cur, dw[0], dw[1], dw[2], (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), oracle.RELU)
    want = oracle.conv2d_s8(cur, pj[0], pj[1], pj[2], (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), oracle.LINEAR)
    dev = lambda t: tuple(to_dev(a) for a in t)  # noqa: E731
    got = m.mbconv_s8(to_dev(x), dev(ex), dev(dw), dev(pj), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), (True, True, False))
    np.testing.assert_array_equal(to_host(got), want)
