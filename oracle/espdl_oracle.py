"""ctypes binding of the CPU oracle (oracle/libespdl_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline
leg.  The shipped library never loads it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libespdl_oracle.so")

ROUND_HALF_UP = 0
ROUND_HALF_EVEN = 1
LINEAR = 0
RELU = 1


class ConvGeom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "batch", "in_h", "in_w", "in_c", "out_c", "k_h", "k_w", "stride_h", "stride_w", "dil_h", "dil_w",
        "pad_top", "pad_bottom", "pad_left", "pad_right", "activation", "round_mode", "n_shift")]


def build():
    """Compile the oracle with gcc (make -C oracle)."""
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        src_time = max(os.path.getmtime(os.path.join(_HERE, f)) for f in ("espdl_oracle.c", "espdl_oracle.h"))
        if not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < src_time:
            build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64
        gp = ctypes.POINTER(ConvGeom)
        L.espdl_oracle_shift_round_s32.restype = ctypes.c_int32
        L.espdl_oracle_shift_round_s32.argtypes = [ctypes.c_int32, i32, i32]
        L.espdl_oracle_shift_round_s64.restype = ctypes.c_int64
        L.espdl_oracle_shift_round_s64.argtypes = [ctypes.c_int64, i32, i32]
        for name in ("conv_out_h", "conv_out_w"):
            f = getattr(L, "espdl_oracle_" + name)
            f.restype, f.argtypes = i32, [gp]
        for name in ("conv2d_s8", "depthwise_s8", "conv2d_s16", "depthwise_s16"):
            f = getattr(L, "espdl_oracle_" + name)
            f.restype, f.argtypes = i32, [gp, vp, vp, vp, vp, vp]
        L.espdl_oracle_lut_s8.argtypes = [vp, i64, vp, vp]
        L.espdl_oracle_prelu_s8.argtypes = [vp, i64, i32, vp, i32, vp]
        L.espdl_oracle_relu_s8.argtypes = [vp, i64, i32, i32, vp]
        L.espdl_oracle_clip_s8.argtypes = [vp, i64, i32, i32, i32, i32, vp]
        L.espdl_oracle_add_s8.argtypes = [vp, i64, vp, i64, i64, vp]
        L.espdl_oracle_global_avg_pool_s8.argtypes = [vp, i32, i32, i32, i32, i32, i32, vp]
        L.espdl_oracle_requantize_s8.argtypes = [vp, i64, i32, i32, vp]
        L.espdl_oracle_mul_s8.argtypes = [vp, i64, vp, i64, i64, i32, i32, vp]
        L.espdl_oracle_avg_pool_s8.argtypes = [vp] + [i32] * 14 + [vp]
        L.espdl_oracle_reduce_mean_s8.restype = i32
        L.espdl_oracle_reduce_mean_s8.argtypes = [vp, vp, i32, vp, i32, i32, vp]
        L.espdl_oracle_add_s16.restype = None
        L.espdl_oracle_add_s16.argtypes = [vp, i64, vp, i64, i64, vp]
        L.espdl_oracle_mul_s16.restype = None
        L.espdl_oracle_mul_s16.argtypes = [vp, i64, vp, i64, i64, i32, i32, vp]
        L.espdl_oracle_sub_s16.restype = None
        L.espdl_oracle_sub_s16.argtypes = [vp, i64, vp, i64, i64, vp]
        L.espdl_oracle_div_s16.restype = None
        L.espdl_oracle_unary_s8.restype = None
        L.espdl_oracle_unary_s8.argtypes = [i32, vp, i64, i32, i32, ctypes.c_float, ctypes.c_float, i32, vp]
        L.espdl_oracle_unary_s16.restype = None
        L.espdl_oracle_unary_s16.argtypes = [i32, vp, i64, i32, i32, ctypes.c_float, ctypes.c_float, i32, vp]
        L.espdl_oracle_reduce_int.restype = ctypes.c_int
        L.espdl_oracle_reduce_int.argtypes = [vp, i32, vp, i32, vp, i32, i32, i32, vp]
        L.espdl_oracle_pad.restype = None
        L.espdl_oracle_pad.argtypes = [vp, vp, i32, vp, i32, i32, i32, vp]
        L.espdl_oracle_sub_s8.restype = None
        L.espdl_oracle_sub_s8.argtypes = [vp, i64, vp, i64, i64, vp]
        L.espdl_oracle_div_s8.restype = None
        L.espdl_oracle_div_s8.argtypes = [vp, vp, i64, i32, i32, i32, vp]
        L.espdl_oracle_div_s16.argtypes = [vp, vp, i64, i32, i32, vp]
        L.espdl_oracle_avg_pool_s16.restype = None
        L.espdl_oracle_avg_pool_s16.argtypes = [vp] + [i32] * 14 + [vp]
        L.espdl_oracle_reduce_mean_s16.restype = i32
        L.espdl_oracle_reduce_mean_s16.argtypes = [vp, vp, i32, vp, i32, i32, vp]
        L.espdl_oracle_insert_zeros.restype = None
        L.espdl_oracle_insert_zeros.argtypes = [vp] + [i32] * 9 + [vp]
        L.espdl_oracle_lut_s16.restype = i32
        L.espdl_oracle_lut_s16.argtypes = [vp, i64, vp, i32, i32, vp]
        L.espdl_oracle_softmax_s8.restype = None
        L.espdl_oracle_softmax_s8.argtypes = [vp, i64, i64, i64, i32, vp]
        L.espdl_oracle_quantize_f32.restype = None
        L.espdl_oracle_quantize_f32.argtypes = [vp, i64, i32, i32, vp]
        L.espdl_oracle_dequantize_f32.restype = None
        L.espdl_oracle_dequantize_f32.argtypes = [vp, i64, i32, i32, vp]
        L.espdl_oracle_slice.restype = i32
        L.espdl_oracle_slice.argtypes = [vp, vp, i32, vp, vp, vp, i32, vp]
        L.espdl_oracle_concat.argtypes = [vp, i32, vp, i64, i32, vp]
        L.espdl_oracle_split_slice.argtypes = [vp, i64, i64, i64, i64, i64, i32, vp]
        L.espdl_oracle_transpose.restype = i32
        L.espdl_oracle_transpose.argtypes = [vp, vp, i32, vp, i32, vp]
        L.espdl_oracle_resize_nearest_s8.argtypes = [vp, i32, i32, i32, i32, i32, i32, ctypes.c_float, ctypes.c_float,
                                                     i32, i32, vp]
        L.espdl_oracle_max_pool.restype = i32
        L.espdl_oracle_max_pool.argtypes = [vp, i32] + [i32] * 12 + [vp]
        L.espdl_oracle_max_threads.restype = i32
        L.espdl_oracle_set_threads.argtypes = [i32]
        for name in ("lut_s8", "prelu_s8", "relu_s8", "clip_s8", "add_s8", "global_avg_pool_s8",
                     "requantize_s8", "set_threads"):
            getattr(L, "espdl_oracle_" + name).restype = None
        _lib = L
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _c(a, dtype):
    return None if a is None else np.ascontiguousarray(a, dtype=dtype)


def set_threads(n):
    lib().espdl_oracle_set_threads(int(n))


def max_threads():
    return lib().espdl_oracle_max_threads()


def shift_round_s32(v, shift, round_mode=ROUND_HALF_UP):
    return lib().espdl_oracle_shift_round_s32(int(v), int(shift), int(round_mode))


def shift_round_s64(v, shift, round_mode=ROUND_HALF_UP):
    return lib().espdl_oracle_shift_round_s64(int(v), int(shift), int(round_mode))


def conv_geom(x_shape, out_c, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), activation=LINEAR,
              round_mode=ROUND_HALF_UP, n_shift=1):
    """pads = (top, bottom, left, right), the order ConvOpArgs takes (dl_base.hpp:201-204)."""
    n, h, w, c = x_shape
    return ConvGeom(n, h, w, c, out_c, k[0], k[1], stride[0], stride[1], dilation[0], dilation[1],
                    pads[0], pads[1], pads[2], pads[3], activation, round_mode, n_shift)


def out_hw(g):
    return lib().espdl_oracle_conv_out_h(ctypes.byref(g)), lib().espdl_oracle_conv_out_w(ctypes.byref(g))


def _conv(fn, act_dtype, bias_dtype, x, filt, bias, shift, k, stride, dilation, pads, activation, round_mode,
          depthwise):
    x = _c(x, act_dtype)
    assert x.ndim == 4
    filt = _c(filt, act_dtype)
    shift = np.atleast_1d(_c(shift, np.int32))
    out_c = x.shape[3] if depthwise else filt.size // (k[0] * k[1] * x.shape[3])
    bias = _c(bias, bias_dtype)
    g = conv_geom(x.shape, out_c, k, stride, dilation, pads, activation, round_mode, shift.size)
    oh, ow = out_hw(g)
    out = np.empty((x.shape[0], oh, ow, out_c), dtype=act_dtype)
    rc = fn(ctypes.byref(g), _ptr(x), _ptr(filt), _ptr(bias), _ptr(shift), _ptr(out))
    if rc != 0:
        raise ValueError("oracle rejected the convolution geometry")
    return out


def conv2d_s8(x, filt, bias, shift, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), activation=LINEAR,
              round_mode=ROUND_HALF_UP):
    """x [N,H,W,C] int8, filt memory [OC][kH][kW][C] int8, bias [OC] int32 or None, shift scalar or [OC]."""
    return _conv(lib().espdl_oracle_conv2d_s8, np.int8, np.int32, x, filt, bias, shift, k, stride, dilation, pads,
                 activation, round_mode, False)


def depthwise_s8(x, filt, bias, shift, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), activation=LINEAR,
                 round_mode=ROUND_HALF_UP):
    """filt memory [kH][kW][C]."""
    return _conv(lib().espdl_oracle_depthwise_s8, np.int8, np.int32, x, filt, bias, shift, k, stride, dilation,
                 pads, activation, round_mode, True)


def conv2d_s16(x, filt, bias, shift, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), activation=LINEAR,
               round_mode=ROUND_HALF_UP):
    return _conv(lib().espdl_oracle_conv2d_s16, np.int16, np.int64, x, filt, bias, shift, k, stride, dilation,
                 pads, activation, round_mode, False)


def depthwise_s16(x, filt, bias, shift, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), activation=LINEAR,
                  round_mode=ROUND_HALF_UP):
    return _conv(lib().espdl_oracle_depthwise_s16, np.int16, np.int64, x, filt, bias, shift, k, stride, dilation,
                 pads, activation, round_mode, True)


def gemm_s8(x, filt, bias, shift, activation=LINEAR, round_mode=ROUND_HALF_UP):
    """Gemm / MatMul as the reference runs it: input viewed as {1,1,M,K}, 1x1 conv
    (esp-dl/dl/module/include/dl_module_gemm.hpp:86-123).  filt memory [N][K]."""
    x = _c(x, np.int8)
    k = x.shape[-1]
    m = x.size // k
    y = conv2d_s8(x.reshape(1, 1, m, k), filt, bias, shift, (1, 1), activation=activation, round_mode=round_mode)
    return y.reshape(x.shape[:-1] + (y.shape[-1],))


def matmul_s8(a, b, shift, activation=LINEAR, round_mode=ROUND_HALF_UP):
    """MatMul of two activations: every [M,K] x [K,N] pair of the broadcast leading dims runs as a 1x1
    convolution whose filter is the second operand (esp-dl/dl/module/include/dl_module_matmul.hpp: the
    batched branches build {1,1,K,N} filter views and call base::conv2d per matrix); one shift for all."""
    a, b = _c(a, np.int8), _c(b, np.int8)
    assert a.ndim >= 2 and b.ndim >= 2 and a.shape[-1] == b.shape[-2]
    lead = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    m, k, n = a.shape[-2], a.shape[-1], b.shape[-1]
    ab = np.broadcast_to(a, lead + (m, k)).reshape(-1, m, k)
    bb = np.broadcast_to(b, lead + (k, n)).reshape(-1, k, n)
    out = np.empty((ab.shape[0], m, n), dtype=np.int8)
    sh = np.array([shift], dtype=np.int32)
    for i in range(ab.shape[0]):
        out[i] = gemm_s8(ab[i], np.ascontiguousarray(bb[i].T), None, sh, activation=activation, round_mode=round_mode)
    return out.reshape(lead + (m, n))


def softmax_s8(x, axis=-1, in_exp=0):
    x = _c(x, np.int8)
    axis = axis % x.ndim
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    out = np.empty(x.shape, dtype=np.float32)
    lib().espdl_oracle_softmax_s8(_ptr(x), outer, x.shape[axis], inner, int(in_exp), _ptr(out))
    return out


def quantize_f32(x, out_exp, dtype=np.int8):
    x = _c(x, np.float32)
    out = np.empty(x.shape, dtype=dtype)
    lib().espdl_oracle_quantize_f32(_ptr(x), x.size, int(out_exp), out.itemsize, _ptr(out))
    return out


def dequantize_f32(x, in_exp):
    x = np.ascontiguousarray(x)
    assert x.dtype in (np.int8, np.int16)
    out = np.empty(x.shape, dtype=np.float32)
    lib().espdl_oracle_dequantize_f32(_ptr(x), x.size, int(in_exp), x.itemsize, _ptr(out))
    return out


def lut_s8(x, table):
    x = _c(x, np.int8)
    table = _c(table, np.int8)
    assert table.size == 256
    out = np.empty_like(x)
    lib().espdl_oracle_lut_s8(_ptr(x), x.size, _ptr(table), _ptr(out))
    return out


def insert_zeros(x, stride, output_padding=(0, 0)):
    x = np.ascontiguousarray(x)
    n, h, w, c = x.shape
    oh = h + (stride[0] - 1) * (h - 1) + output_padding[0]
    ow = w + (stride[1] - 1) * (w - 1) + output_padding[1]
    out = np.empty((n, oh, ow, c), dtype=x.dtype)
    lib().espdl_oracle_insert_zeros(_ptr(x), x.itemsize, n, h, w, c, stride[0], stride[1], oh, ow, _ptr(out))
    return out


def lut_s16(x, table, p4_ties=False):
    x = _c(x, np.int16)
    table = _c(table, np.int16)
    out = np.empty_like(x)
    rc = lib().espdl_oracle_lut_s16(_ptr(x), x.size, _ptr(table), table.size, 1 if p4_ties else 0, _ptr(out))
    assert rc == 0, "table size must be 65536 / 2^n + 1 (or 65536)"
    return out


def prelu_s8(x, alpha, shift):
    x = _c(x, np.int8)
    alpha = _c(alpha, np.int8)
    c = x.shape[-1]
    assert alpha.size == c
    out = np.empty_like(x)
    lib().espdl_oracle_prelu_s8(_ptr(x), x.size // c, c, _ptr(alpha), int(shift), _ptr(out))
    return out


def relu_s8(x, in_exp=0, out_exp=0):
    x = _c(x, np.int8)
    out = np.empty_like(x)
    lib().espdl_oracle_relu_s8(_ptr(x), x.size, in_exp, out_exp, _ptr(out))
    return out


def clip_s8(x, min_q, max_q, in_exp=0, out_exp=0):
    x = _c(x, np.int8)
    out = np.empty_like(x)
    lib().espdl_oracle_clip_s8(_ptr(x), x.size, int(min_q), int(max_q), in_exp, out_exp, _ptr(out))
    return out


def add_s8(a, b):
    a = _c(a, np.int8)
    b = _c(b, np.int8)
    size = max(a.size, b.size)
    assert a.size in (1, size) and b.size in (1, size)
    out = np.empty(a.shape if a.size == size else b.shape, dtype=np.int8)
    lib().espdl_oracle_add_s8(_ptr(a), a.size, _ptr(b), b.size, size, _ptr(out))
    return out


def mul_s8(a, b, shift, round_mode=ROUND_HALF_UP):
    """Element-wise product; a scalar operand broadcasts.  shift = out_exp - a_exp - b_exp."""
    a = _c(a, np.int8)
    b = _c(b, np.int8)
    size = max(a.size, b.size)
    assert a.size in (1, size) and b.size in (1, size)
    out = np.empty(a.shape if a.size == size else b.shape, dtype=np.int8)
    lib().espdl_oracle_mul_s8(_ptr(a), a.size, _ptr(b), b.size, size, int(shift), int(round_mode), _ptr(out))
    return out


def add_s16(a, b):
    a = _c(a, np.int16)
    b = _c(b, np.int16)
    size = max(a.size, b.size)
    assert a.size in (1, size) and b.size in (1, size)
    out = np.empty(a.shape if a.size == size else b.shape, dtype=np.int16)
    lib().espdl_oracle_add_s16(_ptr(a), a.size, _ptr(b), b.size, size, _ptr(out))
    return out


def sub_s16(a, b):
    a = _c(a, np.int16)
    b = _c(b, np.int16)
    size = max(a.size, b.size)
    assert a.size in (1, size) and b.size in (1, size)
    out = np.empty(a.shape if a.size == size else b.shape, dtype=np.int16)
    lib().espdl_oracle_sub_s16(_ptr(a), a.size, _ptr(b), b.size, size, _ptr(out))
    return out


def div_form(shape_a, shape_b, all_ones=1):
    """Which of the reference's three loops runs: 1 if the divisor is constant along the innermost axis of the
    result that is longer than 1, 2 if the dividend is, else 0.  A result of one element takes `all_ones`: the
    int16 dispatcher tests the divisor first, the int8 one the dividend."""
    out = np.broadcast_shapes(tuple(shape_a), tuple(shape_b))
    rank = len(out)
    pa = (1,) * (rank - len(shape_a)) + tuple(shape_a)
    pb = (1,) * (rank - len(shape_b)) + tuple(shape_b)
    for d in range(rank - 1, -1, -1):
        if out[d] > 1:
            return 1 if pb[d] == 1 else (2 if pa[d] == 1 else 0)
    return all_ones


UNARY_KINDS = {"Sigmoid": 0, "Tanh": 1, "HardSwish": 2, "Elu": 3, "Exp": 4, "Log": 5, "Sqrt": 6, "LeakyRelu": 7,
               "Neg": 8, "Swish": 9, "HardSigmoid": 10}
# default attribute values of the reference's deserializers (dl_module_elu.hpp:92, dl_module_leaky_relu.hpp:99,
# dl_module_hard_sigmoid.hpp: alpha 0.2, beta 0.5)
UNARY_DEFAULTS = {"Elu": (1.0, 0.0), "LeakyRelu": (0.01, 0.0), "HardSigmoid": (0.2, 0.5)}


def unary(op_type, x, in_exp, out_exp, alpha=None, beta=None, round_mode=ROUND_HALF_UP):
    """The float32-per-element activation modules and Neg, int8 or int16 by the dtype of x."""
    x = np.ascontiguousarray(x)
    assert x.dtype in (np.int8, np.int16)
    da, db = UNARY_DEFAULTS.get(op_type, (0.0, 0.0))
    alpha = da if alpha is None else alpha
    beta = db if beta is None else beta
    out = np.empty_like(x)
    fn = lib().espdl_oracle_unary_s8 if x.dtype == np.int8 else lib().espdl_oracle_unary_s16
    fn(UNARY_KINDS[op_type], _ptr(x), x.size, int(in_exp), int(out_exp), float(alpha), float(beta), int(round_mode),
       _ptr(out))
    return out


def gather(x, indices, axis=0):
    """Gather with constant indices as the reference copies it
    (esp-dl/dl/module/include/dl_module_gather.hpp:56-66): per outer index, one inner row per index, in order."""
    x = np.ascontiguousarray(x)
    indices = np.asarray(indices, dtype=np.int64)
    axis = axis + x.ndim if axis < 0 else axis
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    extent = x.shape[axis]
    flat_in = x.reshape(outer, extent, inner)
    flat_idx = indices.ravel()
    assert flat_idx.size == 0 or (flat_idx.min() >= 0 and flat_idx.max() < extent)
    out = np.empty((outer, flat_idx.size, inner), dtype=x.dtype)
    for o in range(outer):
        for i, idx in enumerate(flat_idx):
            out[o, i] = flat_in[o, int(idx)]
    return out.reshape(list(x.shape[:axis]) + list(indices.shape) + list(x.shape[axis + 1:]))


def space_to_depth(x, blocksize):
    """SpaceToDepth on NHWC as the reference's loop scatters it
    (esp-dl/dl/module/include/dl_module_space_to_depth.hpp:17-44): input element (n, h, w, c) lands at
    (n, h // b, w // b, c * b^2 + (h % b) * b + w % b)."""
    x = np.ascontiguousarray(x)
    n, h, w, c = x.shape
    b = int(blocksize)
    out = np.empty((n, h // b, w // b, c * b * b), dtype=x.dtype)
    hh, ww, cc = np.meshgrid(np.arange(h), np.arange(w), np.arange(c), indexing="ij")
    out[:, hh // b, ww // b, cc * b * b + (hh % b) * b + ww % b] = x[:, hh, ww, cc]
    return out


def depth_to_space(x, blocksize, mode="DCR"):
    """DepthToSpace on NHWC, a scatter like the reference's loops
    (esp-dl/dl/module/include/dl_module_depth_to_space.hpp:17-67).  CRD: channel c goes to out channel c // b^2 at
    row offset (c % b^2) // b and column offset c % b.  DCR: the reference takes out channel c % b, row offset
    c // b^2, column offset (c % b^2) // b, which is a permutation only when the output has b channels; the ONNX
    definition c = (row * b + col) * C' + out_c agrees with it there and is used for every C'."""
    x = np.ascontiguousarray(x)
    n, h, w, c = x.shape
    b = int(blocksize)
    oc = c // (b * b)
    out = np.empty((n, h * b, w * b, oc), dtype=x.dtype)
    hh, ww, cc = np.meshgrid(np.arange(h), np.arange(w), np.arange(c), indexing="ij")
    if mode == "CRD":
        k, row, col = cc // (b * b), (cc % (b * b)) // b, cc % b
    else:
        k, row, col = cc % oc, cc // (b * oc), (cc // oc) % b
    out[:, hh * b + row, ww * b + col, k] = x[:, hh, ww, cc]
    return out


REDUCE_OPS = {"ReduceMax": 0, "ReduceMin": 1, "ReduceSum": 2, "ReduceL1": 3, "ReduceSumSquare": 4}


def reduce_int(op_type, x, axes, keepdims=True, shift=0, round_mode=ROUND_HALF_UP):
    """ReduceMax / ReduceMin / ReduceSum of an int8 or int16 tensor; shift = out_exp - in_exp (sum only)."""
    x = np.ascontiguousarray(x)
    assert x.dtype in (np.int8, np.int16)
    nd = x.ndim
    axes = [a + nd if a < 0 else a for a in (axes if len(axes) else range(nd))]
    flags = np.array([1 if i in axes else 0 for i in range(nd)], dtype=np.int32)
    kept = [x.shape[i] for i in range(nd) if not flags[i]]
    out = np.empty(kept if kept else [1], dtype=x.dtype)
    shape = np.array(x.shape, dtype=np.int32)
    rc = lib().espdl_oracle_reduce_int(_ptr(x), 8 * x.dtype.itemsize, _ptr(shape), nd, _ptr(flags), REDUCE_OPS[op_type],
                                       int(shift), int(round_mode), _ptr(out))
    assert rc == 0
    if keepdims:
        out = out.reshape([1 if flags[i] else x.shape[i] for i in range(nd)])
    return out


PAD_MODES = {"constant": 0, "edge": 1, "reflect": 2}


def pad(x, pads, mode="constant", value=0):
    """pads: the leading pad of every axis, then the trailing pad of every axis."""
    x = np.ascontiguousarray(x)
    nd = x.ndim
    assert len(pads) == 2 * nd and x.dtype.itemsize in (1, 2, 4)
    shape = np.asarray(x.shape, dtype=np.int32)
    p = np.asarray(pads, dtype=np.int32)
    out = np.empty([x.shape[i] + int(p[i]) + int(p[i + nd]) for i in range(nd)], dtype=x.dtype)
    lib().espdl_oracle_pad(_ptr(x), _ptr(shape), nd, _ptr(p), PAD_MODES[mode], int(value), x.dtype.itemsize, _ptr(out))
    return out


def sub_s8(a, b):
    a = _c(a, np.int8)
    b = _c(b, np.int8)
    size = max(a.size, b.size)
    assert a.size in (1, size) and b.size in (1, size)
    out = np.empty(a.shape if a.size == size else b.shape, dtype=np.int8)
    lib().espdl_oracle_sub_s8(_ptr(a), a.size, _ptr(b), b.size, size, _ptr(out))
    return out


def div_s8(a, b, shift):
    """numpy-broadcast quotient; shift = out_exp - a_exp + b_exp.  A one-element operand selects the reference's
    table form, the dividend first (esp-dl/dl/base/dl_base_div.cpp:17, 33, 212-224)."""
    a, b = np.asarray(a, dtype=np.int8), np.asarray(b, dtype=np.int8)
    table_operand = 1 if a.size == 1 else (2 if b.size == 1 else 0)
    form = div_form(a.shape, b.shape, all_ones=2)
    a, b = np.broadcast_arrays(a, b)
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    out = np.empty(a.shape, dtype=np.int8)
    lib().espdl_oracle_div_s8(_ptr(a), _ptr(b), a.size, int(shift), form, table_operand, _ptr(out))
    return out


def div_s16(a, b, shift):
    """numpy-broadcast quotient; shift = out_exp - a_exp + b_exp."""
    form = div_form(np.shape(a), np.shape(b))
    a, b = np.broadcast_arrays(np.asarray(a, dtype=np.int16), np.asarray(b, dtype=np.int16))
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    out = np.empty(a.shape, dtype=np.int16)
    lib().espdl_oracle_div_s16(_ptr(a), _ptr(b), a.size, int(shift), form, _ptr(out))
    return out


def mul_s16(a, b, shift, round_mode=ROUND_HALF_UP):
    a = _c(a, np.int16)
    b = _c(b, np.int16)
    size = max(a.size, b.size)
    assert a.size in (1, size) and b.size in (1, size)
    out = np.empty(a.shape if a.size == size else b.shape, dtype=np.int16)
    lib().espdl_oracle_mul_s16(_ptr(a), a.size, _ptr(b), b.size, size, int(shift), int(round_mode), _ptr(out))
    return out


def global_avg_pool_s8(x, in_exp, out_exp):
    x = _c(x, np.int8)
    n, h, w, c = x.shape
    out = np.empty((n, 1, 1, c), dtype=np.int8)
    lib().espdl_oracle_global_avg_pool_s8(_ptr(x), n, h, w, c, in_exp, out_exp, _ptr(out))
    return out


def requantize_s8(x, in_exp, out_exp):
    x = _c(x, np.int8)
    out = np.empty_like(x)
    lib().espdl_oracle_requantize_s8(_ptr(x), x.size, in_exp, out_exp, _ptr(out))
    return out


def concat(arrays, axis):
    """Concat as the reference runs it: per outer index, one contiguous run from each input
    (esp-dl/dl/module/include/dl_module_concat.hpp:56-108)."""
    arrays = [np.ascontiguousarray(a) for a in arrays]
    dt = arrays[0].dtype
    nd = arrays[0].ndim
    axis = axis + nd if axis < 0 else axis
    loop_times = int(np.prod(arrays[0].shape[:axis], dtype=np.int64))
    copy_nums = np.array([int(np.prod(a.shape[axis:], dtype=np.int64)) for a in arrays], dtype=np.int64)
    shape = list(arrays[0].shape)
    shape[axis] = sum(a.shape[axis] for a in arrays)
    out = np.empty(shape, dtype=dt)
    ptrs = (ctypes.c_void_p * len(arrays))(*[a.ctypes.data for a in arrays])
    lib().espdl_oracle_concat(ptrs, len(arrays), _ptr(copy_nums), loop_times, dt.itemsize, _ptr(out))
    return out


def split(x, axis, sizes):
    """Split into consecutive pieces of the given sizes along axis
    (esp-dl/dl/module/include/dl_module_split.hpp:84-152)."""
    x = np.ascontiguousarray(x)
    axis = axis + x.ndim if axis < 0 else axis
    num_slices = int(np.prod(x.shape[:axis], dtype=np.int64))
    slice_size = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    outs, start = [], 0
    for sz in sizes:
        shape = list(x.shape)
        shape[axis] = int(sz)
        out = np.empty(shape, dtype=x.dtype)
        lib().espdl_oracle_split_slice(_ptr(x), start, num_slices, slice_size, x.shape[axis], int(sz), x.dtype.itemsize,
                                       _ptr(out))
        outs.append(out)
        start += int(sz)
    return outs


def transpose(x, perm=None):
    x = np.ascontiguousarray(x)
    perm = list(range(x.ndim - 1, -1, -1)) if not perm else [p + x.ndim if p < 0 else p for p in perm]
    out = np.empty([x.shape[p] for p in perm], dtype=x.dtype)
    shape = np.array(x.shape, dtype=np.int32)
    permv = np.array(perm, dtype=np.int32)
    rc = lib().espdl_oracle_transpose(_ptr(x), _ptr(shape), x.ndim, _ptr(permv), x.dtype.itemsize, _ptr(out))
    assert rc == 0
    return out


def resize_out_hw(h, w, scale_h, scale_w):
    """Output size as esp-dl/dl/module/include/dl_module_resize.hpp:66-70 computes it from scales."""
    return int(h * np.float32(scale_h)), int(w * np.float32(scale_w))


def resize_nearest_s8(x, scale_h, scale_w, in_exp=0, out_exp=0, out_hw=None):
    x = _c(x, np.int8)
    n, h, w, c = x.shape
    oh, ow = out_hw if out_hw is not None else resize_out_hw(h, w, scale_h, scale_w)
    out = np.empty((n, oh, ow, c), dtype=np.int8)
    lib().espdl_oracle_resize_nearest_s8(_ptr(x), n, h, w, c, oh, ow, float(scale_h), float(scale_w), in_exp, out_exp,
                                         _ptr(out))
    return out


def max_pool(x, kernel, strides=(1, 1), pads=(0, 0, 0, 0)):
    """pads = (top, bottom, left, right).  int8 or int16 NHWC."""
    x = np.ascontiguousarray(x)
    assert x.dtype in (np.int8, np.int16)
    n, h, w, c = x.shape
    pt, pb, pl, pr = pads
    oh = (h + pt + pb - kernel[0]) // strides[0] + 1
    ow = (w + pl + pr - kernel[1]) // strides[1] + 1
    out = np.empty((n, oh, ow, c), dtype=x.dtype)
    rc = lib().espdl_oracle_max_pool(_ptr(x), x.dtype.itemsize, n, h, w, c, kernel[0], kernel[1], strides[0], strides[1],
                                     pt, pb, pl, pr, _ptr(out))
    assert rc == 0
    return out


def avg_pool_s8(x, kernel, strides=(1, 1), pads=(0, 0, 0, 0), in_exp=0, out_exp=0):
    """pads = (top, bottom, left, right).  int8 NHWC."""
    x = _c(x, np.int8)
    n, h, w, c = x.shape
    pt, pb, pl, pr = pads
    oh = (h + pt + pb - kernel[0]) // strides[0] + 1
    ow = (w + pl + pr - kernel[1]) // strides[1] + 1
    out = np.empty((n, oh, ow, c), dtype=np.int8)
    lib().espdl_oracle_avg_pool_s8(_ptr(x), n, h, w, c, kernel[0], kernel[1], strides[0], strides[1], pt, pb, pl, pr,
                                   in_exp, out_exp, _ptr(out))
    return out


def avg_pool_s16(x, kernel, strides=(1, 1), pads=(0, 0, 0, 0), in_exp=0, out_exp=0):
    x = _c(x, np.int16)
    n, h, w, c = x.shape
    pt, pb, pl, pr = pads
    oh = (h + pt + pb - kernel[0]) // strides[0] + 1
    ow = (w + pl + pr - kernel[1]) // strides[1] + 1
    out = np.empty((n, oh, ow, c), dtype=np.int16)
    lib().espdl_oracle_avg_pool_s16(_ptr(x), n, h, w, c, kernel[0], kernel[1], strides[0], strides[1], pt, pb, pl, pr,
                                    in_exp, out_exp, _ptr(out))
    return out


def reduce_mean_s16(x, axes, keepdims=True, in_exp=0, out_exp=0):
    x = _c(x, np.int16)
    nd = x.ndim
    axes = [a + nd if a < 0 else a for a in (axes if len(axes) else range(nd))]
    flags = np.array([1 if i in axes else 0 for i in range(nd)], dtype=np.int32)
    kept = [x.shape[i] for i in range(nd) if not flags[i]]
    out = np.empty(kept if kept else [1], dtype=np.int16)
    shape = np.array(x.shape, dtype=np.int32)
    rc = lib().espdl_oracle_reduce_mean_s16(_ptr(x), _ptr(shape), nd, _ptr(flags), in_exp, out_exp, _ptr(out))
    assert rc == 0
    if keepdims:
        out = out.reshape([1 if flags[i] else x.shape[i] for i in range(nd)])
    return out


def normalize_slice(shape, starts, ends, axes=None, steps=None):
    """ONNX Slice bookkeeping for positive steps -> (start, step, out_shape) per dim."""
    nd = len(shape)
    start, step, out_shape = [0] * nd, [1] * nd, list(shape)
    for i in range(len(starts)):
        ax = i if axes is None or len(axes) == 0 else (int(axes[i]) + nd) % nd
        st = 1 if steps is None or len(steps) == 0 else int(steps[i])
        assert st >= 1, "negative steps are not part of this build"
        dim = shape[ax]
        s, e = int(starts[i]), int(ends[i])
        s = s + dim if s < 0 else s
        e = e + dim if e < 0 else e
        s, e = min(max(s, 0), dim), min(max(e, 0), dim)
        start[ax], step[ax], out_shape[ax] = s, st, max(0, -(-(e - s) // st))
    return start, step, out_shape


def slice_(x, starts, ends, axes=None, steps=None):
    x = np.ascontiguousarray(x)
    start, step, out_shape = normalize_slice(x.shape, starts, ends, axes, steps)
    out = np.empty(out_shape, dtype=x.dtype)
    i32 = lambda v: np.array(v, dtype=np.int32)  # noqa: E731
    sh, st, sp, os_ = i32(x.shape), i32(start), i32(step), i32(out_shape)
    rc = lib().espdl_oracle_slice(_ptr(x), _ptr(sh), x.ndim, _ptr(st), _ptr(sp), _ptr(os_), x.dtype.itemsize, _ptr(out))
    assert rc == 0
    return out


def reduce_mean_s8(x, axes, keepdims=True, in_exp=0, out_exp=0):
    x = _c(x, np.int8)
    nd = x.ndim
    axes = [a + nd if a < 0 else a for a in (axes if len(axes) else range(nd))]
    flags = np.array([1 if i in axes else 0 for i in range(nd)], dtype=np.int32)
    kept = [x.shape[i] for i in range(nd) if not flags[i]]
    out = np.empty(kept if kept else [1], dtype=np.int8)
    shape = np.array(x.shape, dtype=np.int32)
    rc = lib().espdl_oracle_reduce_mean_s8(_ptr(x), _ptr(shape), nd, _ptr(flags), in_exp, out_exp, _ptr(out))
    assert rc == 0
    if keepdims:
        out = out.reshape([1 if flags[i] else x.shape[i] for i in range(nd)])
    return out
