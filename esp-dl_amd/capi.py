"""ctypes binding of include/espdl_hip.h (lib/libespdl_hip.so).

Tensors are torch CUDA tensors used as plain device buffers (`data_ptr()`); kernels are enqueued on
torch's current stream unless another raw stream handle is given.  There is no CPU fallback: if the
library is missing, `lib()` raises.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libespdl_hip.so")

S8, S16 = 8, 16
LINEAR, RELU = 0, 1
ROUND_HALF_UP, ROUND_HALF_EVEN = 0, 1


class EspdlHipError(RuntimeError):
    pass


class ConvDesc(ctypes.Structure):
    """espdl_hip_conv_desc"""
    _fields_ = [(n, ctypes.c_int32) for n in (
        "dtype", "batch", "in_h", "in_w", "in_c", "out_c", "k_h", "k_w", "stride_h", "stride_w", "dil_h", "dil_w",
        "pad_top", "pad_bottom", "pad_left", "pad_right", "group", "activation", "round_mode", "n_shift",
        "in_pitch", "out_pitch", "res_pitch")]


class MbconvDesc(ctypes.Structure):
    """espdl_hip_mbconv_desc"""
    _fields_ = [(n, ctypes.c_int32) for n in (
        "batch", "in_h", "in_w", "in_c", "exp_c", "out_c", "has_expand", "k_h", "k_w", "stride_h", "stride_w",
        "dil_h", "dil_w", "pad_top", "pad_bottom", "pad_left", "pad_right", "act_expand", "act_dw", "act_project",
        "round_mode", "n_shift_expand", "n_shift_dw", "n_shift_project",
        "exp_k_h", "exp_k_w", "exp_stride_h", "exp_stride_w", "exp_pad_top", "exp_pad_bottom", "exp_pad_left",
        "exp_pad_right", "residual_shift", "clip_expand", "clip_expand_min", "clip_expand_max", "clip_dw",
        "clip_dw_min", "clip_dw_max")]


class MbconvWeights(ctypes.Structure):
    """espdl_hip_mbconv_weights"""
    _fields_ = [(n, ctypes.c_void_p) for n in (
        "w_expand", "b_expand", "s_expand", "w_dw", "b_dw", "s_dw", "w_project", "b_project", "s_project")]


_lib = None


def torch_device_first():
    """PyTorch wheels carry their own copy of the HIP runtime.  The copy that initializes first owns the device for
    the process, and the buffers handed to this library come from torch: so before the library makes its first
    HIP call, torch's runtime is brought up (nothing happens without torch or without a GPU)."""
    try:
        import torch
    except ImportError:
        return
    if torch.cuda.is_available():
        torch.cuda.init()


def lib():
    """Load libespdl_hip.so; fails loudly when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise EspdlHipError(
                f"{LIB_PATH} is missing: build it with `python esp-dl_amd/build.py` (no CPU fallback exists)")
        torch_device_first()
        L = ctypes.CDLL(LIB_PATH)
        vp, i32, i64 = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64
        dp = ctypes.POINTER(ConvDesc)
        L.espdl_hip_conv_out_shape.argtypes = [dp, ctypes.POINTER(i32), ctypes.POINTER(i32)]
        L.espdl_hip_conv2d.argtypes = [dp, vp, vp, vp, vp, vp, vp, vp]
        L.espdl_hip_conv2d_add.argtypes = [dp, vp, vp, vp, vp, vp, vp, vp, vp]
        L.espdl_hip_conv2d_add.restype = ctypes.c_int
        L.espdl_hip_conv2d_gap_s8.argtypes = [dp, vp, vp, vp, vp, i32, i32, vp, vp]
        L.espdl_hip_conv2d_gap_s8.restype = ctypes.c_int
        L.espdl_hip_conv2d_gap_s8_supported.argtypes = [dp]
        L.espdl_hip_conv2d_gap_s8_supported.restype = ctypes.c_int
        L.espdl_hip_lut_s8.argtypes = [vp, i64, vp, vp, vp]
        L.espdl_hip_prelu_s8.argtypes = [vp, i64, i32, vp, i32, vp, vp]
        L.espdl_hip_relu_s8.argtypes = [vp, i64, i32, i32, vp, vp]
        L.espdl_hip_clip_s8.argtypes = [vp, i64, i32, i32, i32, i32, vp, vp]
        L.espdl_hip_add_s8.argtypes = [ctypes.POINTER(i32 * 4), ctypes.POINTER(i64 * 4), ctypes.POINTER(i64 * 4),
                                       vp, vp, vp, vp]
        L.espdl_hip_mul_s8.argtypes = [ctypes.POINTER(i32 * 4), ctypes.POINTER(i64 * 4), ctypes.POINTER(i64 * 4),
                                       vp, vp, i32, i32, vp, vp]
        L.espdl_hip_mul_s8.restype = ctypes.c_int
        L.espdl_hip_global_avg_pool_s8.argtypes = [vp, i32, i32, i32, i32, i32, i32, vp, vp]
        L.espdl_hip_requantize_s8.argtypes = [vp, i64, i32, i32, vp, vp]
        L.espdl_hip_split.argtypes = [vp, i64, i32, ctypes.POINTER(vp), ctypes.POINTER(i64), i64, vp]
        L.espdl_hip_requantize_s8_rows.argtypes = [vp, i64, vp, i64, i64, i64, i32, i32, vp]
        L.espdl_hip_requantize.argtypes = [vp, i32, i64, i32, i32, vp, i32, vp]
        f32 = ctypes.c_float
        L.espdl_hip_concat.argtypes = [i32, vp, vp, i64, vp, vp]
        L.espdl_hip_copy_rows.argtypes = [vp, i64, vp, i64, i64, i64, vp]
        L.espdl_hip_transpose.argtypes = [vp, vp, i32, vp, i32, i32, vp, vp]
        L.espdl_hip_resize_nearest_s8.argtypes = [vp, i32, i32, i32, i32, i32, i32, f32, f32, i32, i32, vp, vp]
        L.espdl_hip_resize_nearest_s8_pitched.argtypes = [vp, i32, i32, i32, i32, i32, i32, f32, f32, i32, i32, i32, i32, vp, vp]
        L.espdl_hip_max_pool.argtypes = [vp, i32] + [i32] * 12 + [vp, vp]
        L.espdl_hip_max_pool_pitched.argtypes = [vp, i32] + [i32] * 14 + [vp, vp]
        L.espdl_hip_avg_pool_s8.argtypes = [vp] + [i32] * 14 + [vp, vp]
        L.espdl_hip_slice.argtypes = [vp, vp, i32, vp, vp, vp, i32, vp, vp]
        L.espdl_hip_reduce_mean_s8.argtypes = [vp, vp, i32, vp, i32, i32, vp, vp]
        L.espdl_hip_add_s16.argtypes = [vp, vp, vp, vp, vp, vp, vp]
        L.espdl_hip_mul_s16.argtypes = [vp, vp, vp, vp, vp, i32, i32, vp, vp]
        L.espdl_hip_avg_pool_s16.argtypes = [vp] + [i32] * 14 + [vp, vp]
        L.espdl_hip_reduce_mean_s16.argtypes = [vp, vp, i32, vp, i32, i32, vp, vp]
        L.espdl_hip_sub_s16.argtypes = [vp, vp, vp, vp, vp, vp, vp]
        L.espdl_hip_div_s16.argtypes = [vp, vp, vp, vp, vp, i32, vp, vp]
        L.espdl_hip_sub_s8.argtypes = [vp, vp, vp, vp, vp, vp, vp]
        L.espdl_hip_div_s8.argtypes = [vp, vp, vp, vp, vp, i32, vp, vp]
        for name in ("add_s16", "mul_s16", "sub_s16", "div_s16", "avg_pool_s16", "reduce_mean_s16", "sub_s8", "div_s8"):
            getattr(L, "espdl_hip_" + name).restype = ctypes.c_int
        L.espdl_hip_insert_zeros.argtypes = [vp] + [i32] * 9 + [vp, vp]
        L.espdl_hip_insert_zeros.restype = ctypes.c_int
        L.espdl_hip_pad.argtypes = [vp, vp, i32, vp, i32, i32, i32, vp, vp]
        L.espdl_hip_pad.restype = ctypes.c_int
        L.espdl_hip_reduce_int.argtypes = [vp, i32, vp, i32, vp, i32, i32, i32, vp, vp]
        L.espdl_hip_reduce_int.restype = ctypes.c_int
        L.espdl_hip_lut_s16.argtypes = [vp, i64, vp, i32, i32, vp, vp]
        L.espdl_hip_lut_s16.restype = ctypes.c_int
        L.espdl_hip_softmax_s8.argtypes = [vp, i64, i64, i64, i32, vp, vp]
        L.espdl_hip_quantize_f32.argtypes = [vp, i64, i32, i32, vp, vp]
        L.espdl_hip_dequantize_f32.argtypes = [vp, i64, i32, i32, vp, vp]
        L.espdl_hip_matmul_s8.argtypes = [vp, vp, i32, i32, i32, vp, vp, vp, i32, i32, i32, vp, vp]
        for name in ("concat", "copy_rows", "transpose", "resize_nearest_s8", "max_pool", "avg_pool_s8", "slice",
                     "reduce_mean_s8", "softmax_s8", "quantize_f32", "dequantize_f32", "matmul_s8"):
            getattr(L, "espdl_hip_" + name).restype = ctypes.c_int
        mp = ctypes.POINTER(MbconvDesc)
        L.espdl_hip_mbconv_out_shape.argtypes = [mp, ctypes.POINTER(i32), ctypes.POINTER(i32)]
        L.espdl_hip_mbconv_s8_supported.argtypes = [mp]
        L.espdl_hip_mbconv_s8.argtypes = [mp, vp, ctypes.POINTER(MbconvWeights), vp, vp, vp]
        L.espdl_hip_mbconv_s8_staged.argtypes = L.espdl_hip_mbconv_s8.argtypes
        L.espdl_hip_mbconv_s8_preferred.argtypes = [mp]
        for name in ("mbconv_out_shape", "mbconv_s8_supported", "mbconv_s8_preferred", "mbconv_s8", "mbconv_s8_staged"):
            getattr(L, "espdl_hip_" + name).restype = ctypes.c_int
        for name in ("conv_out_shape", "conv2d", "lut_s8", "prelu_s8", "relu_s8", "clip_s8", "add_s8",
                     "global_avg_pool_s8", "requantize_s8", "requantize", "device_cu_count"):
            getattr(L, "espdl_hip_" + name).restype = ctypes.c_int
        L.espdl_hip_last_error.restype = ctypes.c_char_p
        L.espdl_hip_version.restype = ctypes.c_char_p
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise EspdlHipError(f"espdl_hip error {rc}: {lib().espdl_hip_last_error().decode()}")


def _stream(stream):
    if stream is not None:
        return ctypes.c_void_p(stream)
    import torch
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def make_desc(x_shape, out_c, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), group=1, activation=LINEAR,
              round_mode=ROUND_HALF_UP, n_shift=1, dtype=S8):
    n, h, w, c = x_shape
    return ConvDesc(dtype, n, h, w, c, out_c, k[0], k[1], stride[0], stride[1], dilation[0], dilation[1],
                    pads[0], pads[1], pads[2], pads[3], group, activation, round_mode, n_shift)


def conv_out_shape(desc):
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    _check(lib().espdl_hip_conv_out_shape(ctypes.byref(desc), ctypes.byref(oh), ctypes.byref(ow)))
    return oh.value, ow.value


def _channel_pitch(t):
    """0 for a dense NHWC tensor; the pixel pitch for a channel slice t = wide[..., a:b] of a dense tensor."""
    if t is None or t.is_contiguous():
        return 0
    n, h, w, c = t.shape
    st = t.stride()
    if st[3] != 1 or st[1] != w * st[2] or st[0] != h * st[1] or st[2] < c:
        raise ValueError("only channel slices of dense NHWC tensors can be passed without a copy")
    return st[2]


def conv2d(x, filt, bias, shift, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), depthwise=False,
           activation=LINEAR, round_mode=ROUND_HALF_UP, lut=None, out=None, stream=None, residual=None):
    """x [N,H,W,C] int8|int16 CUDA tensor; filt dense [OC][kH][kW][C] or depthwise [kH][kW][C];
    bias int32|int64 [OC] or None; shift int32 tensor with 1 or OC entries (device).  x, out and residual may be
    channel slices of wider NHWC tensors (wide[..., a:b]): they are read / written in place through the
    descriptor's pitches."""
    import torch
    dtype = S8 if x.dtype == torch.int8 else S16
    n, h, w, c = x.shape
    out_c = c if depthwise else filt.numel() // (k[0] * k[1] * c)
    desc = make_desc(x.shape, out_c, k, stride, dilation, pads, c if depthwise else 1, activation, round_mode,
                     shift.numel(), dtype)
    desc.in_pitch, desc.out_pitch, desc.res_pitch = _channel_pitch(x), _channel_pitch(out), _channel_pitch(residual)
    oh, ow = conv_out_shape(desc)
    if out is None:
        out = torch.empty((n, oh, ow, out_c), dtype=x.dtype, device=x.device)
    _check(lib().espdl_hip_conv2d_add(ctypes.byref(desc), _p(x), _p(filt), _p(bias), _p(shift), _p(lut), _p(residual),
                                      _p(out), _stream(stream)))
    return out


def conv2d_gap_s8(x, filt, bias, shift, conv_out_exp, pool_out_exp, activation=LINEAR, round_mode=ROUND_HALF_UP,
                  out=None, stream=None):
    """1x1 convolution followed by GlobalAveragePool in one launch: x [N,H,W,C] int8 with H*W <= 64, filt [OC][C];
    returns the pooled [N][OC] int8 tensor (espdl_hip_conv2d_gap_s8)."""
    import torch
    n, h, w, c = x.shape
    out_c = filt.numel() // c
    desc = make_desc(x.shape, out_c, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), 1, activation, round_mode, shift.numel(), S8)
    if out is None:
        out = torch.empty((n, out_c), dtype=torch.int8, device=x.device)
    _check(lib().espdl_hip_conv2d_gap_s8(ctypes.byref(desc), _p(x), _p(filt), _p(bias), _p(shift), conv_out_exp,
                                         pool_out_exp, _p(out), _stream(stream)))
    return out


def mbconv_s8(x, expand, dw, project, k, stride=(1, 1), dilation=(1, 1), pads=(0, 0, 0, 0), relus=(True, True, False),
              residual=None, round_mode=ROUND_HALF_UP, out=None, stream=None, staged=False, expand_conv=None,
              residual_shift=0, clip_expand=None, clip_dw=None):
    """Fused inverted-residual block (staged=True: espdl_hip_mbconv_s8_staged, the separate stages with the
    intermediates in the library's own device array; `out` must then be given, nothing is allocated).  expand / dw / project are (filter, bias, shift) triples of CUDA
    tensors (expand may be None); filters as for conv2d: [E][C], [kH][kW][E], [OC][E].
    expand_conv = (kernel, stride, pads) makes the expand stage a dense convolution with a window over the
    block input (filter [E][kH][kW][C]); the depthwise stage then works on that convolution's output."""
    import torch
    n, h, w, c = x.shape
    wd, bd, sd = dw
    wp, bp, sp = project
    exp_c = wd.numel() // (k[0] * k[1])
    out_c = wp.numel() // exp_c
    we, be, se = expand if expand is not None else (None, None, None)
    desc = MbconvDesc(n, h, w, c, exp_c, out_c, 0 if expand is None else 1, k[0], k[1], stride[0], stride[1],
                      dilation[0], dilation[1], pads[0], pads[1], pads[2], pads[3],
                      RELU if relus[0] else LINEAR, RELU if relus[1] else LINEAR, RELU if relus[2] else LINEAR,
                      round_mode, 1 if se is None else se.numel(), sd.numel(), sp.numel())
    if expand_conv is not None:
        ek, es, ep = expand_conv
        (desc.exp_k_h, desc.exp_k_w, desc.exp_stride_h, desc.exp_stride_w) = (ek[0], ek[1], es[0], es[1])
        (desc.exp_pad_top, desc.exp_pad_bottom, desc.exp_pad_left, desc.exp_pad_right) = ep
    desc.residual_shift = residual_shift
    if clip_expand is not None:  # (min, max): Clip with equal exponents behind the expand stage
        desc.clip_expand, desc.clip_expand_min, desc.clip_expand_max = 1, clip_expand[0], clip_expand[1]
    if clip_dw is not None:
        desc.clip_dw, desc.clip_dw_min, desc.clip_dw_max = 1, clip_dw[0], clip_dw[1]
    oh, ow = ctypes.c_int32(), ctypes.c_int32()
    _check(lib().espdl_hip_mbconv_out_shape(ctypes.byref(desc), ctypes.byref(oh), ctypes.byref(ow)))
    if out is None:
        out = torch.empty((n, oh.value, ow.value, out_c), dtype=torch.int8, device=x.device)
    wts = MbconvWeights(_p(we), _p(be), _p(se), _p(wd), _p(bd), _p(sd), _p(wp), _p(bp), _p(sp))
    fn = lib().espdl_hip_mbconv_s8_staged if staged else lib().espdl_hip_mbconv_s8
    _check(fn(ctypes.byref(desc), _p(x), ctypes.byref(wts), _p(residual), _p(out), _stream(stream)))
    return out


def lut_s8(x, table, out=None, stream=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    _check(lib().espdl_hip_lut_s8(_p(x), x.numel(), _p(table), _p(out), _stream(stream)))
    return out


def prelu_s8(x, alpha, shift, out=None, stream=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    c = x.shape[-1]
    _check(lib().espdl_hip_prelu_s8(_p(x), x.numel() // c, c, _p(alpha), shift, _p(out), _stream(stream)))
    return out


def relu_s8(x, in_exp=0, out_exp=0, out=None, stream=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    _check(lib().espdl_hip_relu_s8(_p(x), x.numel(), in_exp, out_exp, _p(out), _stream(stream)))
    return out


def clip_s8(x, min_q, max_q, in_exp=0, out_exp=0, out=None, stream=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    _check(lib().espdl_hip_clip_s8(_p(x), x.numel(), min_q, max_q, in_exp, out_exp, _p(out), _stream(stream)))
    return out


def _pad4(shape):
    shape = list(shape)
    if len(shape) > 4:
        raise EspdlHipError("add_s8 handles up to 4 dims")
    return [1] * (4 - len(shape)) + shape


def _broadcast(a, b, out):
    import torch
    sa, sb = _pad4(a.shape), _pad4(b.shape)
    so = [max(x, y) for x, y in zip(sa, sb)]

    def strides(s):
        st, acc = [0] * 4, 1
        for i in range(3, -1, -1):
            st[i] = acc if s[i] != 1 else 0
            acc *= s[i]
        return st

    rank = max(a.dim(), b.dim())
    if out is None:
        out = torch.empty(so[4 - rank:] if rank else [], dtype=torch.int8, device=a.device)
    return (ctypes.c_int32 * 4)(*so), (ctypes.c_int64 * 4)(*strides(sa)), (ctypes.c_int64 * 4)(*strides(sb)), out


def add_s8(a, b, out=None, stream=None):
    """numpy-style broadcasting add of two contiguous tensors (up to 4 dims)."""
    dims, s0, s1, out = _broadcast(a, b, out)
    _check(lib().espdl_hip_add_s8(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), _p(out),
                                  _stream(stream)))
    return out


def mul_s8(a, b, shift, round_mode=ROUND_HALF_UP, out=None, stream=None):
    """numpy-style broadcasting product; shift = out_exp - a_exp - b_exp."""
    dims, s0, s1, out = _broadcast(a, b, out)
    _check(lib().espdl_hip_mul_s8(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), int(shift),
                                  round_mode, _p(out), _stream(stream)))
    return out


def global_avg_pool_s8(x, in_exp, out_exp, out=None, stream=None):
    import torch
    n, h, w, c = x.shape
    out = torch.empty((n, 1, 1, c), dtype=torch.int8, device=x.device) if out is None else out
    _check(lib().espdl_hip_global_avg_pool_s8(_p(x), n, h, w, c, in_exp, out_exp, _p(out), _stream(stream)))
    return out


def requantize_s8(x, in_exp, out_exp, out=None, stream=None):
    """x and out may be channel slices of wider NHWC tensors (wide[..., a:b])."""
    import torch
    out = torch.empty(x.shape, dtype=torch.int8, device=x.device) if out is None else out
    if x.dim() == 4 and (_channel_pitch(x) or _channel_pitch(out)):
        c = x.shape[3]
        _check(lib().espdl_hip_requantize_s8_rows(_p(x), _channel_pitch(x) or c, _p(out), _channel_pitch(out) or c, c,
                                                  x.numel() // c, in_exp, out_exp, _stream(stream)))
        return out
    _check(lib().espdl_hip_requantize_s8(_p(x), x.numel(), in_exp, out_exp, _p(out), _stream(stream)))
    return out


def requantize(x, in_exp, out_exp, out_dtype=None, out=None, stream=None):
    """int8 / int16 -> int8 / int16 across exponents (TensorBase::assign)."""
    import torch
    out_dtype = x.dtype if out_dtype is None else out_dtype
    out = torch.empty(x.shape, dtype=out_dtype, device=x.device) if out is None else out
    bits = lambda d: S16 if d == torch.int16 else S8  # noqa: E731
    _check(lib().espdl_hip_requantize(_p(x), bits(x.dtype), x.numel(), in_exp, out_exp, _p(out), bits(out.dtype),
                                      _stream(stream)))
    return out


def _prod(xs):
    n = 1
    for x in xs:
        n *= int(x)
    return n


def concat(tensors, axis, out=None, stream=None):
    """Concat of contiguous device tensors along axis (any element type)."""
    import torch
    nd = tensors[0].dim()
    axis = axis + nd if axis < 0 else axis
    esize = tensors[0].element_size()
    shape = list(tensors[0].shape)
    shape[axis] = sum(int(t.shape[axis]) for t in tensors)
    out = torch.empty(shape, dtype=tensors[0].dtype, device=tensors[0].device) if out is None else out
    n = len(tensors)
    ptrs = (ctypes.c_void_p * n)(*[t.data_ptr() for t in tensors])
    nbytes = (ctypes.c_int64 * n)(*[_prod(t.shape[axis:]) * esize for t in tensors])
    _check(lib().espdl_hip_concat(n, ptrs, nbytes, _prod(shape[:axis]), _p(out), _stream(stream)))
    return out


def split(x, axis, sizes, stream=None, outs=None):
    """Consecutive pieces of the given sizes along axis, each a new contiguous tensor (or the tensors of `outs`;
    a None entry there skips that piece), in one pass over x (espdl_hip_split)."""
    import torch
    axis = axis + x.dim() if axis < 0 else axis
    esize = x.element_size()
    num_slices, slice_size = _prod(x.shape[:axis]), _prod(x.shape[axis + 1:])
    results = []
    for j, sz in enumerate(sizes):
        shape = list(x.shape)
        shape[axis] = int(sz)
        if outs is not None:
            results.append(outs[j])
        else:
            results.append(torch.empty(shape, dtype=x.dtype, device=x.device))
    n = len(sizes)
    ptrs = (ctypes.c_void_p * n)(*[None if t is None else t.data_ptr() for t in results])
    sizes_b = (ctypes.c_int64 * n)(*[slice_size * int(sz) * esize for sz in sizes])
    _check(lib().espdl_hip_split(_p(x), slice_size * int(x.shape[axis]) * esize, n, ptrs, sizes_b, num_slices, _stream(stream)))
    return results


def transpose(x, perm=None, out=None, stream=None):
    import torch
    nd = x.dim()
    perm = list(perm) if perm else []
    full = [p + nd if p < 0 else p for p in perm] if perm else list(range(nd - 1, -1, -1))
    out = torch.empty([x.shape[p] for p in full], dtype=x.dtype, device=x.device) if out is None else out
    shape = (ctypes.c_int32 * nd)(*x.shape)
    pv = (ctypes.c_int32 * max(1, len(perm)))(*perm) if perm else None
    _check(lib().espdl_hip_transpose(_p(x), shape, nd, pv, len(perm), x.element_size(), _p(out), _stream(stream)))
    return out


def resize_nearest_s8(x, scale_h, scale_w, in_exp=0, out_exp=0, out_hw=None, out=None, stream=None):
    import numpy as np
    import torch
    n, h, w, c = x.shape
    oh, ow = out_hw if out_hw is not None else (int(h * np.float32(scale_h)), int(w * np.float32(scale_w)))
    out = torch.empty((n, oh, ow, c), dtype=torch.int8, device=x.device) if out is None else out
    ip, op = _channel_pitch(x), _channel_pitch(out)
    if ip or op:  # channel slices of wider NHWC tensors
        _check(lib().espdl_hip_resize_nearest_s8_pitched(_p(x), n, h, w, c, oh, ow, float(scale_h), float(scale_w), in_exp,
                                                         out_exp, ip, op, _p(out), _stream(stream)))
        return out
    _check(lib().espdl_hip_resize_nearest_s8(_p(x), n, h, w, c, oh, ow, float(scale_h), float(scale_w), in_exp, out_exp,
                                             _p(out), _stream(stream)))
    return out


def max_pool(x, kernel, strides=(1, 1), pads=(0, 0, 0, 0), out=None, stream=None):
    """pads = (top, bottom, left, right); x int8 or int16 NHWC.  x and out may be channel slices of wider
    NHWC tensors (wide[..., a:b])."""
    import torch
    n, h, w, c = x.shape
    pt, pb, pl, pr = pads
    oh = (h + pt + pb - kernel[0]) // strides[0] + 1
    ow = (w + pl + pr - kernel[1]) // strides[1] + 1
    out = torch.empty((n, max(oh, 0), max(ow, 0), c), dtype=x.dtype, device=x.device) if out is None else out
    ip, op = _channel_pitch(x), _channel_pitch(out)
    if ip or op:
        _check(lib().espdl_hip_max_pool_pitched(_p(x), S16 if x.dtype == torch.int16 else S8, n, h, w, c, kernel[0],
                                                kernel[1], strides[0], strides[1], pt, pb, pl, pr, ip, op, _p(out),
                                                _stream(stream)))
        return out
    _check(lib().espdl_hip_max_pool(_p(x), S16 if x.dtype == torch.int16 else S8, n, h, w, c, kernel[0], kernel[1],
                                    strides[0], strides[1], pt, pb, pl, pr, _p(out), _stream(stream)))
    return out


def avg_pool_s8(x, kernel, strides=(1, 1), pads=(0, 0, 0, 0), in_exp=0, out_exp=0, out=None, stream=None):
    """pads = (top, bottom, left, right); x int8 NHWC."""
    import torch
    n, h, w, c = x.shape
    pt, pb, pl, pr = pads
    oh = (h + pt + pb - kernel[0]) // strides[0] + 1
    ow = (w + pl + pr - kernel[1]) // strides[1] + 1
    out = torch.empty((n, max(oh, 0), max(ow, 0), c), dtype=torch.int8, device=x.device) if out is None else out
    _check(lib().espdl_hip_avg_pool_s8(_p(x), n, h, w, c, kernel[0], kernel[1], strides[0], strides[1], pt, pb, pl, pr,
                                       in_exp, out_exp, _p(out), _stream(stream)))
    return out


def slice_(x, start, step, out_shape, out=None, stream=None):
    """out[i...] = x[start + i * step ...]; start / step / out_shape have one entry per dim of x."""
    import torch
    nd = x.dim()
    out = torch.empty(list(out_shape), dtype=x.dtype, device=x.device) if out is None else out
    arr = lambda v: (ctypes.c_int32 * nd)(*[int(t) for t in v])  # noqa: E731
    _check(lib().espdl_hip_slice(_p(x), arr(x.shape), nd, arr(start), arr(step), arr(out_shape), x.element_size(),
                                 _p(out), _stream(stream)))
    return out


def reduce_mean_s8(x, axes, keepdims=True, in_exp=0, out_exp=0, stream=None):
    import torch
    nd = x.dim()
    axes = [a + nd if a < 0 else a for a in (axes if len(axes) else range(nd))]
    flags = [1 if i in axes else 0 for i in range(nd)]
    kept = [int(x.shape[i]) for i in range(nd) if not flags[i]]
    out = torch.empty(kept if kept else [1], dtype=torch.int8, device=x.device)
    _check(lib().espdl_hip_reduce_mean_s8(_p(x), (ctypes.c_int32 * nd)(*x.shape), nd, (ctypes.c_int32 * nd)(*flags),
                                          in_exp, out_exp, _p(out), _stream(stream)))
    return out.reshape([1 if flags[i] else int(x.shape[i]) for i in range(nd)]) if keepdims else out


def softmax_s8(x, axis=-1, in_exp=0, stream=None):
    """int8 tensor -> float32 softmax along `axis` (espdl_hip_softmax_s8)."""
    import torch
    import math
    axis = axis % x.dim()
    outer = math.prod(int(d) for d in x.shape[:axis])
    inner = math.prod(int(d) for d in x.shape[axis + 1:])
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _check(lib().espdl_hip_softmax_s8(_p(x), outer, int(x.shape[axis]), inner, in_exp, _p(out), _stream(stream)))
    return out


def quantize_f32(x, out_exp, dtype=None, stream=None):
    import torch
    dtype = dtype or torch.int8
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    _check(lib().espdl_hip_quantize_f32(_p(x), x.numel(), out_exp, out.element_size(), _p(out), _stream(stream)))
    return out


def dequantize_f32(x, in_exp, stream=None):
    import torch
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _check(lib().espdl_hip_dequantize_f32(_p(x), x.numel(), in_exp, x.element_size(), _p(out), _stream(stream)))
    return out


def matmul_s8(a, b, shift, activation=0, round_mode=0, stream=None):
    """a [..., M, K] x b [..., K, N] with up to two broadcast leading dims (espdl_hip_matmul_s8)."""
    import torch
    assert a.dim() >= 2 and b.dim() >= 2 and a.dim() <= 4 and b.dim() <= 4 and a.shape[-1] == b.shape[-2]
    la = [1] * (4 - a.dim()) + [int(d) for d in a.shape[:-2]]
    lb = [1] * (4 - b.dim()) + [int(d) for d in b.shape[:-2]]
    lead = [max(la[0], lb[0]), max(la[1], lb[1])]
    m, k, n = int(a.shape[-2]), int(a.shape[-1]), int(b.shape[-1])

    def strides(l, mat):
        return [0 if l[0] == 1 else l[1] * mat, 0 if l[1] == 1 else mat]

    rank = max(a.dim(), b.dim())
    out = torch.empty(lead[4 - rank:] + [m, n] if rank > 2 else [m, n], dtype=torch.int8, device=a.device)
    _check(lib().espdl_hip_matmul_s8(_p(a), _p(b), m, k, n, (ctypes.c_int32 * 2)(*lead),
                                     (ctypes.c_int64 * 2)(*strides(la, m * k)), (ctypes.c_int64 * 2)(*strides(lb, k * n)),
                                     shift, activation, round_mode, _p(out), _stream(stream)))
    return out


def lut_s16(x, table, round_mode=0, stream=None):
    import torch
    out = torch.empty_like(x)
    _check(lib().espdl_hip_lut_s16(_p(x), x.numel(), _p(table), table.numel(), round_mode, _p(out), _stream(stream)))
    return out


def insert_zeros(x, stride, output_padding=(0, 0), stream=None):
    """x [N, H, W, C] (or [N, L, C]) -> zeros with x at every stride-th position (espdl_hip_insert_zeros)."""
    import torch
    one_d = x.dim() == 3
    n, h, w, c = (int(x.shape[0]), int(x.shape[1]), 1, int(x.shape[2])) if one_d else [int(d) for d in x.shape]
    sh, sw = (stride[0], 1) if one_d else stride
    ph, pw = (output_padding[0], 0) if one_d else output_padding
    oh = max(0, h + (sh - 1) * (h - 1) + ph) if h else 0
    ow = max(0, w + (sw - 1) * (w - 1) + pw) if w else 0
    out = torch.empty([n, oh, c] if one_d else [n, oh, ow, c], dtype=x.dtype, device=x.device)
    _check(lib().espdl_hip_insert_zeros(_p(x), x.element_size(), n, h, w, c, sh, sw, ph, pw, _p(out), _stream(stream)))
    return out


def _broadcast16(a, b, dtype=None):
    import torch
    dims, s0, s1, _ = _broadcast(a, b, a)  # strides only; the result is allocated below
    rank = max(a.dim(), b.dim())
    so = [int(d) for d in dims]
    return dims, s0, s1, torch.empty(so[4 - rank:] if rank else [], dtype=dtype or torch.int16, device=a.device)


def add_s16(a, b, stream=None):
    dims, s0, s1, out = _broadcast16(a, b)
    _check(lib().espdl_hip_add_s16(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), _p(out),
                                   _stream(stream)))
    return out


def mul_s16(a, b, shift, round_mode=ROUND_HALF_UP, stream=None):
    dims, s0, s1, out = _broadcast16(a, b)
    _check(lib().espdl_hip_mul_s16(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), int(shift),
                                   round_mode, _p(out), _stream(stream)))
    return out


def avg_pool_s16(x, kernel, strides=(1, 1), pads=(0, 0, 0, 0), in_exp=0, out_exp=0, stream=None):
    import torch
    n, h, w, c = x.shape
    pt, pb, pl, pr = pads
    oh = (h + pt + pb - kernel[0]) // strides[0] + 1
    ow = (w + pl + pr - kernel[1]) // strides[1] + 1
    out = torch.empty((n, max(oh, 0), max(ow, 0), c), dtype=torch.int16, device=x.device)
    _check(lib().espdl_hip_avg_pool_s16(_p(x), n, h, w, c, kernel[0], kernel[1], strides[0], strides[1], pt, pb, pl, pr,
                                        in_exp, out_exp, _p(out), _stream(stream)))
    return out


def reduce_mean_s16(x, axes, keepdims=True, in_exp=0, out_exp=0, stream=None):
    import torch
    nd = x.dim()
    axes = [a + nd if a < 0 else a for a in (axes if len(axes) else range(nd))]
    flags = [1 if i in axes else 0 for i in range(nd)]
    kept = [int(x.shape[i]) for i in range(nd) if not flags[i]]
    out = torch.empty(kept if kept else [1], dtype=torch.int16, device=x.device)
    _check(lib().espdl_hip_reduce_mean_s16(_p(x), (ctypes.c_int32 * nd)(*x.shape), nd, (ctypes.c_int32 * nd)(*flags),
                                           in_exp, out_exp, _p(out), _stream(stream)))
    return out.reshape([1 if flags[i] else int(x.shape[i]) for i in range(nd)]) if keepdims else out


def sub_s16(a, b, stream=None):
    dims, s0, s1, out = _broadcast16(a, b)
    _check(lib().espdl_hip_sub_s16(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), _p(out),
                                   _stream(stream)))
    return out


REDUCE_OPS = {"ReduceMax": 0, "ReduceMin": 1, "ReduceSum": 2, "ReduceL1": 3, "ReduceSumSquare": 4}


def reduce_int(op_type, x, axes, keepdims=True, shift=0, round_mode=ROUND_HALF_UP, stream=None):
    """ReduceMax / ReduceMin / ReduceSum of an int8 or int16 tensor (espdl_hip_reduce_int); shift = out_exp - in_exp."""
    import torch
    nd = x.dim()
    axes = [a + nd if a < 0 else a for a in (axes if len(axes) else range(nd))]
    flags = [1 if i in axes else 0 for i in range(nd)]
    kept = [int(x.shape[i]) for i in range(nd) if not flags[i]]
    out = torch.empty(kept if kept else [1], dtype=x.dtype, device=x.device)
    _check(lib().espdl_hip_reduce_int(_p(x), S8 if x.dtype == torch.int8 else S16, (ctypes.c_int32 * nd)(*x.shape), nd,
                                      (ctypes.c_int32 * nd)(*flags), REDUCE_OPS[op_type], int(shift), round_mode, _p(out),
                                      _stream(stream)))
    return out.reshape([1 if flags[i] else int(x.shape[i]) for i in range(nd)]) if keepdims else out


PAD_MODES = {"constant": 0, "edge": 1, "reflect": 2}


def pad(x, pads, mode="constant", value=0, stream=None):
    """pads: the leading pad of every axis, then the trailing pad of every axis (espdl_hip_pad)."""
    import torch
    nd = x.dim()
    assert len(pads) == 2 * nd
    out = torch.empty([int(x.shape[i]) + int(pads[i]) + int(pads[i + nd]) for i in range(nd)], dtype=x.dtype,
                      device=x.device)
    _check(lib().espdl_hip_pad(_p(x), (ctypes.c_int32 * nd)(*x.shape), nd, (ctypes.c_int32 * (2 * nd))(*pads),
                               PAD_MODES[mode], int(value), x.element_size(), _p(out), _stream(stream)))
    return out


def sub_s8(a, b, stream=None):
    import torch
    dims, s0, s1, out = _broadcast16(a, b, torch.int8)
    _check(lib().espdl_hip_sub_s8(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), _p(out),
                                  _stream(stream)))
    return out


def div_s8(a, b, shift, stream=None):
    """shift = out_exp - a_exp + b_exp."""
    import torch
    dims, s0, s1, out = _broadcast16(a, b, torch.int8)
    _check(lib().espdl_hip_div_s8(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), int(shift),
                                  _p(out), _stream(stream)))
    return out


def div_s16(a, b, shift, stream=None):
    """shift = out_exp - a_exp + b_exp."""
    dims, s0, s1, out = _broadcast16(a, b)
    _check(lib().espdl_hip_div_s16(ctypes.byref(dims), ctypes.byref(s0), ctypes.byref(s1), _p(a), _p(b), int(shift),
                                   _p(out), _stream(stream)))
    return out
