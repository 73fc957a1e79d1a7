"""Concat / Split / Transpose / Resize-nearest / MaxPool on the GPU against the CPU oracle (bit-exact)."""
import numpy as np
import pytest

from gpu_util import announce, espdl, to_dev, to_host

pytestmark = pytest.mark.gpu


def _rand(rng, shape, dtype=np.int8):
    info = np.iinfo(dtype)
    return rng.integers(info.min, info.max + 1, size=shape).astype(dtype)


CONCAT_CASES = [
    # (base shape, axis, extents along the axis)
    ((2, 20, 20, 0), 3, [64, 64, 64, 64]),      # SPPF: four 16-byte aligned runs
    ((2, 40, 40, 0), 3, [128, 64]),              # FPN: upsampled + skip
    ((3, 7, 5, 0), 3, [5, 11, 16]),              # byte paths
    ((2, 0, 9, 8), 1, [3, 1, 6]),                # an outer axis
    ((0, 4, 4, 16), 0, [1, 2]),                  # batch axis: one run per input
    ((1, 4, 4, 0), -1, [4] * 11),                # more inputs than one launch takes
]


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("case", CONCAT_CASES, ids=lambda c: f"{c[0]}_ax{c[1]}")
def test_concat(oracle, case, dtype):
    base, axis, extents = case
    announce(f"concat {case} {dtype.__name__}")
    rng = np.random.default_rng(21)
    arrays = []
    for e in extents:
        shape = list(base)
        shape[axis] = e
        arrays.append(_rand(rng, shape, dtype))
    got = to_host(espdl().concat([to_dev(a) for a in arrays], axis))
    np.testing.assert_array_equal(got, oracle.concat(arrays, axis))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("shape,axis,sizes", [
    ((2, 20, 20, 128), 3, [64, 64]), ((2, 9, 9, 48), 3, [5, 20, 23]), ((4, 6, 5, 8), 1, [1, 2, 3]),
    ((5, 3, 3, 4), 0, [2, 3]), ((1, 1, 1, 32), -1, [16, 16]), ((3, 7, 11, 160), 3, [32, 16, 64, 48]),
    ((2, 5, 5, 144), 3, [16] * 9), ((3, 4, 64, 16), 1, [1, 3]),
])
def test_split(oracle, shape, axis, sizes, dtype):
    announce(f"split {shape} axis {axis} {sizes} {dtype.__name__}")
    x = _rand(np.random.default_rng(22), shape, dtype)
    got = espdl().split(to_dev(x), axis, sizes)
    want = oracle.split(x, axis, sizes)
    assert len(got) == len(want)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(to_host(g), w)


def test_split_skips_pieces_without_a_destination(oracle):
    """A NULL output is a piece the caller reads in place: the others are written, nothing else is touched."""
    import torch
    announce("split with a skipped piece")
    m = espdl()
    x = _rand(np.random.default_rng(30), (2, 6, 7, 96))
    a = torch.full((2, 6, 7, 32), 55, dtype=torch.int8, device="cuda")
    c = torch.full((2, 6, 7, 48), 55, dtype=torch.int8, device="cuda")
    m.split(to_dev(x), 3, [32, 16, 48], outs=[a, None, c])
    np.testing.assert_array_equal(to_host(a), x[..., :32])
    np.testing.assert_array_equal(to_host(c), x[..., 48:])


@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.int32])
@pytest.mark.parametrize("shape,perm", [
    ((2, 20, 20, 64), (0, 3, 1, 2)), ((2, 64, 20, 20), (0, 2, 3, 1)), ((3, 5, 7, 9), None), ((37, 65), (1, 0)),
    ((4, 1, 1, 1280), (0, 3, 1, 2)), ((2, 3, 4, 5), (0, 1, 2, 3)), ((2, 3, 4, 5), (1, 0, 2, 3)),
    ((2, 2, 3, 2, 5), (4, 0, 3, 1, 2)), ((2, 3, 33, 40), (0, 1, 3, 2)), ((6,), (0,)), ((2, 3, 4), (-1, 0, 1)),
    # the innermost axis stays innermost: its runs move in pieces of 16, 8, 4 or 2 bytes, by length and address
    ((2, 6, 10, 16), (0, 2, 1, 3)), ((3, 4, 5, 24), (0, 2, 1, 3)), ((2, 5, 7, 12), (1, 0, 2, 3)), ((2, 2, 25, 40, 16), (0, 1, 3, 2, 4)),
    ((2, 9, 3, 6), (2, 0, 1, 3)),
])
def test_transpose(oracle, shape, perm, dtype):
    announce(f"transpose {shape} {perm} {dtype.__name__}")
    x = _rand(np.random.default_rng(23), shape, dtype)
    got = to_host(espdl().transpose(to_dev(x), perm))
    np.testing.assert_array_equal(got, oracle.transpose(x, perm))


@pytest.mark.parametrize("shape,scales,exps", [
    ((2, 20, 20, 128), (2, 2), (-4, -4)), ((2, 10, 10, 64), (2, 2), (-4, -3)), ((1, 7, 5, 3), (2, 2), (-4, -4)),
    ((2, 8, 12, 16), (1.5, 2.5), (-4, -4)), ((2, 8, 12, 5), (0.5, 0.5), (-5, -3)), ((1, 6, 6, 32), (3, 1), (-4, -6)),
    ((1, 9, 9, 16), (1, 1), (0, 2)),
])
def test_resize_nearest_s8(oracle, shape, scales, exps):
    announce(f"resize nearest {shape} x{scales} exps {exps}")
    x = _rand(np.random.default_rng(24), shape)
    got = to_host(espdl().resize_nearest_s8(to_dev(x), scales[0], scales[1], exps[0], exps[1]))
    np.testing.assert_array_equal(got, oracle.resize_nearest_s8(x, scales[0], scales[1], exps[0], exps[1]))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("shape,kernel,strides,pads", [
    ((2, 20, 20, 128), (5, 5), (1, 1), (2, 2, 2, 2)), ((2, 16, 16, 24), (2, 2), (2, 2), (0, 0, 0, 0)),
    ((3, 9, 8, 5), (3, 3), (2, 2), (1, 1, 1, 1)), ((1, 11, 7, 16), (3, 2), (1, 2), (1, 0, 0, 1)),
    ((2, 5, 5, 8), (5, 5), (1, 1), (0, 0, 0, 0)), ((1, 1, 30, 40), (1, 3), (1, 1), (0, 0, 1, 1)),
])
def test_max_pool(oracle, shape, kernel, strides, pads, dtype):
    announce(f"max_pool {shape} k{kernel} s{strides} p{pads} {dtype.__name__}")
    x = _rand(np.random.default_rng(25), shape, dtype)
    got = to_host(espdl().max_pool(to_dev(x), kernel, strides, pads))
    np.testing.assert_array_equal(got, oracle.max_pool(x, kernel, strides, pads))


@pytest.mark.parametrize("shape,kernel,strides,pads,exps", [
    ((2, 1, 24, 32), (1, 3), (1, 1), (0, 0, 2, 0), (-6, -7)), ((2, 14, 14, 64), (3, 3), (1, 1), (1, 1, 1, 1), (-5, -5)),
    ((3, 16, 16, 24), (2, 2), (2, 2), (0, 0, 0, 0), (-4, -5)), ((2, 7, 7, 1280), (7, 7), (1, 1), (0, 0, 0, 0), (-3, -4)),
    ((1, 9, 11, 5), (3, 2), (2, 1), (1, 0, 0, 1), (-5, -3)),
])
def test_avg_pool_s8(oracle, shape, kernel, strides, pads, exps):
    announce(f"avg_pool {shape} k{kernel} s{strides} p{pads} exps {exps}")
    x = _rand(np.random.default_rng(26), shape)
    got = to_host(espdl().avg_pool_s8(to_dev(x), kernel, strides, pads, exps[0], exps[1]))
    np.testing.assert_array_equal(got, oracle.avg_pool_s8(x, kernel, strides, pads, exps[0], exps[1]))


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("shape,starts,ends,axes,steps", [
    ((2, 16, 24), [-3], [2 ** 63 - 1], [2], [1]), ((2, 5, 10, 8), [1], [4], [1], [2]),
    ((2, 5, 10, 8), [0, 2, 1], [1, 9, 100], [0, 2, 3], [1, 3, 1]), ((3, 4, 4, 64), [0], [64], [-1], [4]),
    ((6,), [2], [5], None, None),
])
def test_slice(oracle, shape, starts, ends, axes, steps, dtype):
    announce(f"slice {shape} {starts}:{ends} axes {axes} steps {steps} {dtype.__name__}")
    x = _rand(np.random.default_rng(27), shape, dtype)
    want = oracle.slice_(x, starts, ends, axes, steps)
    start, step, out_shape = oracle.normalize_slice(x.shape, starts, ends, axes, steps)
    got = to_host(espdl().slice_(to_dev(x), start, step, out_shape))
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("shape,axes,keepdims,exps", [
    ((4, 7, 7, 64), [1, 2], True, (-4, -5)), ((3, 40, 120), [-1], True, (-5, -5)), ((2, 3, 4, 5), [0, 2], False, (-3, -4)),
    ((4, 9), [], True, (-6, -6)), ((2, 6, 10), [1], False, (-5, -7)), ((2, 1, 40, 96), [2], True, (-4, -4)),
])
def test_reduce_mean_s8(oracle, shape, axes, keepdims, exps):
    announce(f"reduce_mean {shape} axes {axes} keepdims {keepdims} exps {exps}")
    x = _rand(np.random.default_rng(28), shape)
    got = to_host(espdl().reduce_mean_s8(to_dev(x), axes, keepdims, exps[0], exps[1]))
    np.testing.assert_array_equal(got, oracle.reduce_mean_s8(x, axes, keepdims, exps[0], exps[1]))


# Reductions over a run of neighbouring axes with many elements per output go through the kernel that sums the
# middle axis of an [outer][R][inner] view: inner sizes that are one 16-byte piece, several slabs with a ragged
# last one, not a multiple of 16 (single-element loads), 1 (a mean over the last axis); R not a multiple of the
# positions in flight; a reduced run split by an axis of length 1; extreme inputs (the largest sums).
@pytest.mark.parametrize("shape,axes,keepdims,exps", [
    ((2, 50, 60, 96), [1, 2], True, (-4, -5)), ((3, 33, 31, 20), [1, 2], False, (-5, -5)),
    ((2, 19, 23, 1040), [1, 2], True, (-3, -4)), ((5, 301, 16), [1], False, (-6, -6)),
    ((7, 1000), [1], True, (-4, -4)), ((3, 257, 1, 48), [1, 2], True, (-5, -6)), ((4, 6, 13, 1, 11, 24), [2, 3, 4], False, (-5, -5)),
])
def test_reduce_mean_s8_long_runs(oracle, shape, axes, keepdims, exps):
    announce(f"reduce_mean long runs {shape} axes {axes}")
    rng = np.random.default_rng(281)
    for x in (_rand(rng, shape), np.full(shape, 127, np.int8), np.full(shape, -128, np.int8)):
        got = to_host(espdl().reduce_mean_s8(to_dev(x), axes, keepdims, exps[0], exps[1]))
        np.testing.assert_array_equal(got, oracle.reduce_mean_s8(x, axes, keepdims, exps[0], exps[1]))


@pytest.mark.parametrize("shape", [(2, 50, 60, 96), (3, 33, 31, 20), (2, 19, 23, 1040), (1, 120, 160, 16), (4, 9, 9, 8),
                                   (2, 131, 127, 64)],  # few workgroups and a long sum: eight loads in flight per thread
                         ids=lambda s: "x".join(map(str, s)))
def test_global_avg_pool_s8_large_images(oracle, shape):
    announce(f"global_avg_pool_s8 large image {shape}")
    rng = np.random.default_rng(282)
    for x in (_rand(rng, shape), np.full(shape, 127, np.int8), np.full(shape, -128, np.int8)):
        for exps in ((-4, -5), (-5, -3)):
            got = to_host(espdl().global_avg_pool_s8(to_dev(x), exps[0], exps[1]))
            np.testing.assert_array_equal(got, oracle.global_avg_pool_s8(x, exps[0], exps[1]))


@pytest.mark.parametrize("hw", [(3, 3), (2, 5)], ids=["3x3", "2x5"])
def test_avg_pool_and_reduce_mean_s8_every_sum(oracle, hw):
    """Every sum a window can have, exponent pairs with and without ties: float(sum) * scale is rounded to float
    before round() adds its 0.5 (no fused multiply-add on the device)."""
    from cases import every_sum_image
    announce(f"avg_pool / reduce_mean every sum {hw}")
    x = every_sum_image(*hw)
    m = espdl()
    for exps in ((-5, -3), (-4, -4), (-4, -5), (-6, -3)):
        got = to_host(m.avg_pool_s8(to_dev(x), hw, (1, 1), (0, 0, 0, 0), exps[0], exps[1]))
        np.testing.assert_array_equal(got, oracle.avg_pool_s8(x, hw, (1, 1), (0, 0, 0, 0), exps[0], exps[1]), err_msg=str(exps))
        got = to_host(m.reduce_mean_s8(to_dev(x), [1, 2], True, exps[0], exps[1]))
        np.testing.assert_array_equal(got, oracle.reduce_mean_s8(x, [1, 2], True, exps[0], exps[1]), err_msg=str(exps))


@pytest.mark.parametrize("shape,k,pads", [
    # the stride-1 window kernel (channels in multiples of 8): odd and even widths, images smaller than the
    # window, one-sided padding, more rows than one strip, windows of 2 / 3 / 5
    ((2, 20, 20, 128), 5, (2, 2, 2, 2)), ((3, 7, 9, 16), 5, (2, 2, 2, 2)), ((1, 3, 2, 32), 5, (2, 2, 2, 2)),
    ((2, 1, 1, 16), 5, (2, 2, 2, 2)), ((1, 45, 13, 48), 5, (2, 2, 2, 2)), ((2, 9, 10, 16), 5, (4, 0, 0, 4)),
    ((2, 12, 11, 32), 5, (0, 0, 0, 0)), ((2, 11, 12, 16), 3, (1, 1, 1, 1)), ((2, 8, 7, 64), 3, (0, 2, 2, 0)),
    ((3, 6, 5, 16), 2, (0, 1, 0, 1)), ((1, 80, 80, 16), 5, (2, 2, 2, 2)), ((70, 20, 20, 16), 5, (2, 2, 2, 2)),
    ((2, 9, 9, 8), 5, (2, 2, 2, 2)), ((2, 10, 7, 24), 3, (1, 1, 1, 1)),
])
@pytest.mark.parametrize("fill", ["random", "extremes", "low"])
def test_max_pool_window_kernel(oracle, shape, k, pads, fill):
    """Packed-int16 maxima must order bytes exactly like signed bytes: random data, only -128 / 127 / -1 / 0 (the
    values where a wrong sign or a carry between neighbouring bytes shows), and all-low data (-128 / -127, where
    the out-of-image fill value could win by mistake)."""
    announce(f"max_pool window {shape} k{k} p{pads} {fill}")
    rng = np.random.default_rng(26)
    if fill == "random":
        x = _rand(rng, shape)
    elif fill == "extremes":
        x = rng.choice(np.array([-128, 127, -1, 0, 1], dtype=np.int8), size=shape)
    else:
        x = rng.choice(np.array([-128, -127], dtype=np.int8), size=shape, p=[0.9, 0.1])
    got = to_host(espdl().max_pool(to_dev(x), (k, k), (1, 1), pads))
    np.testing.assert_array_equal(got, oracle.max_pool(x, (k, k), (1, 1), pads))


@pytest.mark.parametrize("c,wide_in,wide_out,at", [(16, 64, 48, 16), (32, 32, 128, 96), (16, 40, 16, 0), (24, 72, 48, 24)])
def test_max_pool_channel_slices(oracle, c, wide_in, wide_out, at):
    """Input and output as channel slices of wider tensors (pitches that are and are not multiples of 16 bytes);
    the bytes of the wide output outside the slice stay as they were."""
    import torch
    announce(f"max_pool slices c={c} in={wide_in} out={wide_out} at={at}")
    m = espdl()
    rng = np.random.default_rng(27)
    xin = _rand(rng, (3, 13, 10, wide_in))
    lo = min(at, wide_in - c)
    x = np.ascontiguousarray(xin[..., lo:lo + c])
    want = oracle.max_pool(x, (5, 5), (1, 1), (2, 2, 2, 2))
    wide = to_dev(xin)
    out_wide = torch.full((3, 13, 10, wide_out), 77, dtype=torch.int8, device="cuda")
    m.max_pool(wide[..., lo:lo + c], (5, 5), (1, 1), (2, 2, 2, 2), out=out_wide[..., at:at + c])
    got = to_host(out_wide)
    np.testing.assert_array_equal(got[..., at:at + c], want)
    rest = np.delete(got, np.s_[at:at + c], axis=3)
    assert (rest == 77).all()


@pytest.mark.parametrize("c,wide_in,wide_out,at,exps", [(16, 64, 48, 16, (-4, -4)), (32, 32, 128, 96, (-4, -3)), (24, 72, 48, 24, (-5, -3)),
                                                        (16, 16, 40, 8, (-4, -4))])
def test_resize_nearest_channel_slices(oracle, c, wide_in, wide_out, at, exps):
    import torch
    announce(f"resize slices c={c} in={wide_in} out={wide_out} at={at} exps={exps}")
    m = espdl()
    rng = np.random.default_rng(28)
    xin = _rand(rng, (2, 9, 7, wide_in))
    lo = min(at, wide_in - c)
    x = np.ascontiguousarray(xin[..., lo:lo + c])
    want = oracle.resize_nearest_s8(x, 2, 2, exps[0], exps[1])
    wide = to_dev(xin)
    out_wide = torch.full((2, 18, 14, wide_out), 77, dtype=torch.int8, device="cuda")
    m.resize_nearest_s8(wide[..., lo:lo + c], 2, 2, exps[0], exps[1], out=out_wide[..., at:at + c])
    got = to_host(out_wide)
    np.testing.assert_array_equal(got[..., at:at + c], want)
    assert (np.delete(got, np.s_[at:at + c], axis=3) == 77).all()


@pytest.mark.parametrize("c,wide_in,wide_out,at", [(16, 64, 48, 16), (32, 32, 128, 96), (24, 72, 48, 24), (20, 33, 41, 7)])
@pytest.mark.parametrize("exps", [(-4, -5), (-3, -6), (-6, -4), (-2, -12), (-4, -4)])
def test_requantize_s8_channel_slices(oracle, c, wide_in, wide_out, at, exps):
    """int8 -> int8 between exponents on rows with pitches: 16-byte units, bytes, shifts beyond 7, a plain copy."""
    import torch
    announce(f"requantize slices c={c} in={wide_in} out={wide_out} at={at} exps={exps}")
    m = espdl()
    rng = np.random.default_rng(29)
    xin = _rand(rng, (3, 5, 11, wide_in))
    lo = min(at, wide_in - c)
    x = np.ascontiguousarray(xin[..., lo:lo + c])
    want = oracle.requantize_s8(x, exps[0], exps[1])
    wide = to_dev(xin)
    out_wide = torch.full((3, 5, 11, wide_out), 77, dtype=torch.int8, device="cuda")
    m.requantize_s8(wide[..., lo:lo + c], exps[0], exps[1], out=out_wide[..., at:at + c])
    got = to_host(out_wide)
    np.testing.assert_array_equal(got[..., at:at + c], want)
    assert (np.delete(got, np.s_[at:at + c], axis=3) == 77).all()


def test_sppf_pool_chain_idempotence():
    """Size-independent property at full batch: three chained 5x5/1 pools equal one 13x13/1 pool, and
    pooling is monotone (output >= input)."""
    import torch
    m = espdl()
    announce("max_pool chain 256x20x20x128")
    x = torch.randint(-128, 128, (256, 20, 20, 128), dtype=torch.int8, device="cuda")
    p1 = m.max_pool(x, (5, 5), (1, 1), (2, 2, 2, 2))
    p3 = m.max_pool(m.max_pool(p1, (5, 5), (1, 1), (2, 2, 2, 2)), (5, 5), (1, 1), (2, 2, 2, 2))
    big = m.max_pool(x, (13, 13), (1, 1), (6, 6, 6, 6))
    assert torch.equal(p3, big)
    assert bool((p1 >= x).all())


def test_bad_layout_arguments_are_rejected():
    import torch
    m = espdl()
    x = torch.zeros((1, 4, 4, 8), dtype=torch.int8, device="cuda")
    with pytest.raises(m.EspdlHipError):
        m.transpose(x, (0, 1, 1, 2))
    with pytest.raises(m.EspdlHipError):
        m.max_pool(x, (7, 7))
    with pytest.raises(m.EspdlHipError):
        m.resize_nearest_s8(x, 0.0, 2.0, out_hw=(4, 8))


INSERT_ZEROS_CASES = [
    # (shape, stride, output_padding)
    ((2, 80, 80, 64), (2, 2), (0, 0)),     # the mask branch of the exported segmentation graphs
    ((1, 23, 17, 16), (2, 2), (0, 0)),
    ((3, 5, 4, 3), (3, 1), (1, 0)),        # byte path, mixed strides, output padding
    ((2, 7, 9, 6), (2, 4), (1, 3)),        # 4-byte path for int16
    ((2, 6, 6, 8), (1, 1), (0, 0)),        # stride 1: a copy
    ((0, 4, 4, 16), (2, 2), (0, 0)),
]


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("case", INSERT_ZEROS_CASES, ids=lambda c: f"{c[0]}_s{c[1]}_p{c[2]}")
def test_insert_zeros(oracle, case, dtype):
    shape, stride, pad = case
    announce(f"insert_zeros {case} {dtype.__name__}")
    x = _rand(np.random.default_rng(29), shape, dtype)
    got = to_host(espdl().insert_zeros(to_dev(x), stride, pad))
    np.testing.assert_array_equal(got, oracle.insert_zeros(x, stride, pad))


def test_insert_zeros_one_spatial_dim(oracle):
    announce("insert_zeros NWC")
    x = _rand(np.random.default_rng(30), (3, 11, 5))
    got = to_host(espdl().insert_zeros(to_dev(x), (3,), (2,)))
    np.testing.assert_array_equal(got, oracle.insert_zeros(x[:, :, None], (3, 1), (2, 0))[:, :, 0])


@pytest.mark.parametrize("mode", ["constant", "edge", "reflect"])
@pytest.mark.parametrize("dtype", [np.int8, np.int16, np.int32])
def test_pad(oracle, mode, dtype):
    announce(f"pad {mode} {np.dtype(dtype).name}")
    rng = np.random.default_rng(72)
    shapes = [(37,), (5, 9), (2, 7, 11), (3, 14, 14, 32), (2, 3, 4, 5, 6), (1, 56, 56, 24)]
    for shape in shapes:
        nd = len(shape)
        info = np.iinfo(dtype)
        x = rng.integers(info.min, info.max, size=shape, dtype=dtype, endpoint=True)
        before = [int(rng.integers(0, min(s, 4))) for s in shape]
        after = [int(rng.integers(0, min(s, 4))) for s in shape]
        value = int(rng.integers(-100, 100))
        got = to_host(espdl().pad(to_dev(x), before + after, mode, value))
        np.testing.assert_array_equal(got, oracle.pad(x, before + after, mode, value))
        kw = {"constant_values": value} if mode == "constant" else {}
        np.testing.assert_array_equal(got, np.pad(x, list(zip(before, after)), mode=mode, **kw))


def test_pad_rejects_what_the_reference_cannot_do(oracle):
    announce("pad error paths")
    import torch
    x = torch.zeros((2, 3), dtype=torch.int8, device="cuda")
    with pytest.raises(espdl().EspdlHipError):
        espdl().pad(x, [0, 3, 0, 0], "reflect")          # reflected pad as long as the axis
    with pytest.raises(espdl().EspdlHipError):
        espdl().pad(x, [0, -1, 0, 0], "constant")
    empty = torch.zeros((2, 0), dtype=torch.int8, device="cuda")
    with pytest.raises(espdl().EspdlHipError):
        espdl().pad(empty, [0, 1, 0, 0], "edge")
    got = espdl().pad(empty, [0, 1, 0, 2], "constant", 5)
    assert got.shape == (2, 3) and bool((got == 5).all())


@pytest.mark.parametrize("dtype", [np.int8, np.int16])
@pytest.mark.parametrize("op", ["ReduceMax", "ReduceMin", "ReduceSum", "ReduceL1", "ReduceSumSquare"])
def test_reduce_int(oracle, op, dtype):
    announce(f"reduce_int {op} {np.dtype(dtype).name}")
    rng = np.random.default_rng(74)
    info = np.iinfo(dtype)
    cases = [((3, 14, 14, 32), [1, 2], True), ((3, 14, 14, 32), [3], True), ((2, 40, 97), [-1], False),
             ((2, 5, 6, 7), [], True), ((4, 300), [0], False), ((2, 3, 4, 5, 6), [1, 3], True)]
    for shape, axes, keep in cases:
        x = rng.integers(info.min, info.max, size=shape, dtype=dtype, endpoint=True)
        shifts = {"ReduceSum": [(-1, 0), (0, 0), (4, 0), (4, 1), (7, 1)], "ReduceL1": [(0, 0), (5, 0), (9, 1)],
                  "ReduceSumSquare": [(0, 0), (12, 0), (15, 1), (24, 0), (27, 1)]}.get(op, [(0, 0)])
        for shift, rm in shifts:
            got = to_host(espdl().reduce_int(op, to_dev(x), axes, keep, shift, rm))
            np.testing.assert_array_equal(got, oracle.reduce_int(op, x, axes, keep, shift, rm))
