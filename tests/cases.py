"""Shape matrix shared by the oracle tests and the GPU parity tests.

CONV_CASES / DW_CASES restate tools/ops_test/config/op_cfg.toml:14-400 of the reference in NHWC
terms (aligned, unaligned 22->33 / 27 / 25 channels, filter larger than the input, stride 2,
asymmetric stride, dilation 3 with padding 12), plus BASELINE config 1 and a few geometries the
reference shell treats specially (tail-only padding, negative shift).
Fields: (name, (H, W, C), OC, (kh, kw), stride, dilation, pads(t,b,l,r), bias, relu)
"""

CONV_CASES = [
    ("c3_100x50_k3s2_relu", (100, 50, 3), 16, (3, 3), (2, 2), (1, 1), (0, 0, 0, 0), True, True),
    ("c16_20x20_k1", (20, 20, 16), 32, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("c16_100x50_k1", (100, 50, 16), 32, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("c16_22x22_k5s2p2_relu", (22, 22, 16), 32, (5, 5), (2, 2), (1, 1), (2, 2, 2, 2), True, True),
    ("c32_19x23_k3s2p1", (19, 23, 32), 16, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, False),
    ("c22_19x23_k3p1_oc33", (19, 23, 22), 33, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("c16_3x3_k3p1_nobias", (3, 3, 16), 16, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), False, False),
    ("c27_3x3_k5p2_nobias", (3, 3, 27), 27, (5, 5), (1, 1), (1, 1), (2, 2, 2, 2), False, False),
    # Conv1D rows of the matrix, as H = 1 images
    ("c3_1x50_k3s2_relu", (1, 50, 3), 16, (1, 3), (1, 2), (1, 1), (0, 0, 0, 0), True, True),
    ("c16_1x32_k5s2p2_relu", (1, 32, 16), 32, (1, 5), (1, 2), (1, 1), (0, 0, 2, 2), True, True),
    ("c22_1x29_k3p1_oc33", (1, 29, 22), 33, (1, 3), (1, 1), (1, 1), (0, 0, 1, 1), True, False),
    # extra geometries
    ("c8_9x11_k3s2_tailpad", (9, 11, 8), 12, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), False, False),
    ("c5_12x12_k3d2p2", (12, 12, 5), 7, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2), True, True),
    ("c64_14x14_k1_oc96", (14, 14, 64), 96, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("c24_8x8_k1_oc144", (8, 8, 24), 144, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("c64_8x8_k1s2", (8, 8, 64), 32, (1, 1), (2, 2), (1, 1), (0, 0, 0, 0), True, False),
    ("c32_10x10_k3p1_oc64_relu", (10, 10, 32), 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
]

# Convolutions whose window rows are at most 16 contiguous bytes (k_w * C <= 16) with at most 4 rows and 64 filters:
# the first-layer kernel that does the whole reduction in one MFMA step.  RGB / grey / RGBA / 5 and 8 channels, a
# 1 x 2 window over 8 channels, 7 to 64 filters (1 to 4 filter tiles, ragged ones), strides 1 to 3, dilated
# rows, padding on both / one / no side, rows longer than one 64-pixel unit, a one-row image.
STEM_CASES = [
    ("s3_64x96_k3s2p1_oc16", (64, 96, 3), 16, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True),
    ("s3_50x70_k3s1p1_oc32", (50, 70, 3), 32, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("s1_40x130_k4s2_oc8", (40, 130, 1), 8, (4, 4), (2, 2), (1, 1), (1, 2, 1, 2), True, True),
    ("s4_33x65_k3s2p1_oc24", (33, 65, 4), 24, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), False, False),
    ("s5_30x40_k3dh2_oc48", (30, 40, 5), 48, (3, 3), (1, 1), (2, 1), (2, 2, 1, 1), True, True),
    ("s8_40x40_k1x2_oc64", (40, 40, 8), 64, (1, 2), (1, 1), (1, 1), (0, 0, 0, 1), True, False),
    ("s8_37x41_k2s2_oc20_tailpad", (37, 41, 8), 20, (2, 2), (2, 2), (1, 1), (0, 1, 0, 1), True, True),
    ("s3_20x200_k3s2_nopad_oc16", (20, 200, 3), 16, (3, 3), (2, 2), (1, 1), (0, 0, 0, 0), True, True),
    ("s2_24x24_k3s3p2_oc7", (24, 24, 2), 7, (3, 3), (3, 3), (1, 1), (2, 2, 2, 2), True, False),
    ("s3_1x700_k3s2_oc16", (1, 700, 3), 16, (1, 3), (1, 2), (1, 1), (0, 0, 1, 1), True, True),
]

# Pointwise products with at most 128 input channels over enough pixels to fill the device (3 x 80 x 80: the routes
# the dispatcher takes for many pixels, which the small cases above never reach).  One and two reduction steps,
# reductions that end inside a step (72, 100, 120), filter counts that are no multiple of 64 / 16 / 4, many filters.
POINTWISE_MANY_PIXELS = [
    ("p16_32", (80, 80, 16), 32, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("p32_64", (80, 80, 32), 64, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("p48_40", (80, 80, 48), 40, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False, True),
    ("p64_120", (80, 80, 64), 120, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("p72_33", (80, 80, 72), 33, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("p96_64", (80, 80, 96), 64, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("p100_70", (80, 80, 100), 70, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("p120_1100", (80, 80, 120), 1100, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("p128_128", (80, 80, 128), 128, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
]

# Gemm-like products with a short reduction axis under a thousand or more filters over many rows (a recognizer's
# classifier), the output too large for the caches.  Row lengths that are odd (every output row starts at another
# alignment), even but not a multiple of 4, a multiple of 64; reduction lengths that are and are not multiples of
# 16, with one and two steps of 64; a last group of a single filter; row counts that are not a multiple of 64.
WIDE_ROWS = [
    ("w120_2049", (80, 81, 120), 2049, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("w128_1792", (80, 80, 128), 1792, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("w64_2050", (80, 81, 64), 2050, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), False, True),
    ("w40_1801", (83, 80, 40), 1801, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
    ("w100_1777", (80, 80, 100), 1777, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("w16_1900", (81, 81, 16), 1900, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), True, False),
]

# Windowed convolutions whose channel count is a multiple of 16: the kernel that stages the input tile and the
# filters in LDS.  Strides 1 to 3, dilation, reduction steps that span several taps (16, 32, 48 channels), several
# groups of 64 filters in one and in several chunks, filter counts that are not a multiple of 64 / 16 / 4, images
# wider than one column tile, ragged last tiles, padding on one side only, a window larger than the image.
TILED_CASES = [
    ("t64_30x30_k3p1_oc64", (30, 30, 64), 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
    ("t16_37x41_k3p1_oc16", (37, 41, 16), 16, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("t32_33x35_k3s2p1_oc64", (33, 35, 32), 64, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True),
    ("t48_20x20_k3p1_oc40", (20, 20, 48), 40, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("t128_18x18_k3p1_oc128", (18, 18, 128), 128, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
    ("t64_24x24_k3p1_oc160", (24, 24, 64), 160, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("t16_21x300_k3s2p1_oc32", (21, 300, 16), 32, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True),
    ("t32_40x40_k5d2p4_oc33", (40, 40, 32), 33, (5, 5), (1, 1), (2, 2), (4, 4, 4, 4), True, False),
    ("t16_26x26_k3s3_oc7", (26, 26, 16), 7, (3, 3), (3, 3), (1, 1), (0, 0, 0, 0), False, False),
    ("t32_9x70_k1x7p3_oc64", (9, 70, 32), 64, (1, 7), (1, 1), (1, 1), (0, 0, 3, 3), True, True),
    ("t64_5x5_k7p3_oc64", (5, 5, 64), 64, (7, 7), (1, 1), (1, 1), (3, 3, 3, 3), True, False),
    ("t32_17x19_k3s2_tailpad_oc20", (17, 19, 32), 20, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), True, True),
    ("t256_12x12_k3p1_oc64", (12, 12, 256), 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("t16_64x200_k3p1_oc16", (64, 200, 16), 16, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
]

# BASELINE config 1: 1x56x56x64 -> 64, 3x3, s1, p1, bias, ReLU, shift 9
# Strided windows over 64 channels or more on few pixels: rows gathered from under the window for the pointwise
# GEMM kernel.  Strides 2, 3 and mixed, 3 x 3 / 5 x 5 / 2 x 4 windows, dilation, asymmetric padding, windows that
# hang over every border, 64 / 128 / 192 / 320 channels, filter counts that are not a multiple of 64 / 16 / 4, pixel
# counts that are not a multiple of 64 or 128.
WINDOW_GEMM_CASES = [
    ("g64_40x40_k3s2p1_oc64", (40, 40, 64), 64, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True),
    ("g128_33x35_k3s2p1_oc128", (33, 35, 128), 128, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, True),
    ("g128_20x20_k3s2p1_oc256", (20, 20, 128), 256, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, False),
    ("g192_17x19_k3s2_tailpad_oc70", (17, 19, 192), 70, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), True, True),
    ("g64_31x29_k5s2p2_oc65", (31, 29, 64), 65, (5, 5), (2, 2), (1, 1), (2, 2, 2, 2), False, True),
    ("g64_26x26_k3s3_oc130", (26, 26, 64), 130, (3, 3), (3, 3), (1, 1), (0, 0, 0, 0), True, False),
    ("g64_30x44_k3s12d2p2_oc64", (30, 44, 64), 64, (3, 3), (1, 2), (2, 2), (2, 2, 2, 2), True, True),
    ("g320_9x9_k3s2p1_oc96", (9, 9, 320), 96, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, False),
    ("g128_12x50_k24s21p0312_oc64", (12, 50, 128), 64, (2, 4), (2, 1), (1, 1), (0, 3, 1, 2), True, True),
]

# Stride-1 windows over 64 and 128 channels on more than 128 K output pixels (with the batch the test gives them):
# the shapes that stay with the LDS-tiled kernel when the few-pixel route takes the smaller ones.
TILED_MANY_PIXELS = [
    ("tm64_56x56_k3p1_oc64", (56, 56, 64), 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
    ("tm128_40x44_k3p1_oc96", (40, 44, 128), 96, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, False),
    ("tm64_50x60_k3d2p2_oc72", (50, 60, 64), 72, (3, 3), (1, 1), (2, 2), (2, 2, 2, 2), False, True),
]

CONFIG1 = ("config1_56x56x64_k3p1_relu", (56, 56, 64), 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True)

DW_CASES = [
    ("dw16_3x3_k3p1_relu", (3, 3, 16), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
    ("dw16_20x20_k5s12p2_relu", (20, 20, 16), (5, 5), (1, 2), (1, 1), (2, 2, 2, 2), True, True),
    ("dw25_20x20_k7s12p2_relu", (20, 20, 25), (7, 7), (1, 2), (1, 1), (2, 2, 2, 2), True, True),
    ("dw32_100x50_k3_relu", (100, 50, 32), (3, 3), (1, 1), (1, 1), (0, 0, 0, 0), True, True),
    ("dw16_3x3_k5p2_nobias", (3, 3, 16), (5, 5), (1, 1), (1, 1), (2, 2, 2, 2), False, False),
    ("dw16_9x9_k5d3p12_nobias", (9, 9, 16), (5, 5), (1, 1), (3, 3), (12, 12, 12, 12), False, False),
    ("dw27_3x3_k5p2_nobias", (3, 3, 27), (5, 5), (1, 1), (1, 1), (2, 2, 2, 2), False, False),
    ("dw30_1x20_k7s2p2_relu", (1, 20, 30), (1, 7), (1, 2), (1, 1), (0, 0, 2, 2), True, True),
    ("dw144_14x14_k3p1_relu", (14, 14, 144), (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), True, True),
    ("dw96_15x15_k3s2p1", (15, 15, 96), (3, 3), (2, 2), (1, 1), (1, 1, 1, 1), True, False),
    ("dw8_7x9_k3s2_tailpad", (7, 9, 8), (3, 3), (2, 2), (1, 1), (0, 1, 0, 1), True, False),
    # windows of 13 to 28 taps (5 x 5 and others): the matrix-pipe depthwise kernel's build with seven k steps of taps
    ("dw64_60x60_k5p2_relu", (60, 60, 64), (5, 5), (1, 1), (1, 1), (2, 2, 2, 2), True, True),
    ("dw32_31x29_k5s2p2", (31, 29, 32), (5, 5), (2, 2), (1, 1), (2, 2, 2, 2), True, False),
    ("dw48_20x20_k4x6", (20, 20, 48), (4, 6), (1, 1), (1, 1), (1, 2, 2, 3), True, True),
    ("dw16_12x40_k1x25", (12, 40, 16), (1, 25), (1, 1), (1, 1), (0, 0, 12, 12), True, False),
    ("dw80_17x17_k7x4_nobias", (17, 17, 80), (7, 4), (1, 1), (1, 1), (3, 3, 1, 2), False, False),
]

GEMM_CASES = [  # (M, K, N, bias, relu)
    (1, 16, 16, True, True), (1, 31, 32, True, True), (1, 64, 32, True, False),
    (3, 10, 9, False, False), (32, 10, 35, False, False), (40, 120, 480, True, False),
    (7, 1280, 1000, True, False), (5, 33, 1, True, True),
]


def rng_int8(rng, shape):
    import numpy as np
    return rng.integers(-128, 128, size=shape, dtype=np.int64).astype(np.int8)


def typical_shift(k_total):
    """A requantization shift that keeps outputs spread over the int8 range for uniform int8 operands."""
    import math
    return max(1, int(round(math.log2(5461 * math.sqrt(k_total) / 40))))


def every_sum_image(h, w):
    """int8 [1, h, w, C]: channel i sums to the i-th of all the sums h * w int8 values can have (C padded to a
    multiple of 4 with zeros) - for the operators that average in float, where a tie in the rounding of
    float(sum) * scale is a single value of the sum."""
    import numpy as np
    area = h * w
    sums = np.arange(-128 * area, 127 * area + 1)
    c = (len(sums) + 3) // 4 * 4
    x = np.zeros((1, area, c), dtype=np.int64)
    for i, t in enumerate(sums):
        q, r = divmod(int(t), area)
        x[0, :, i] = q
        x[0, :r, i] += 1
    assert x.min() >= -128 and x.max() <= 127
    return x.reshape(1, h, w, c).astype(np.int8)
