"""esp-dl_amd: ESP-DL's quantized operator hot path on AMD MI355X (gfx950).

The product is native: `lib/libespdl_hip.so` (HIP kernels behind the C ABI of include/espdl_hip.h)
and `lib/libespdl_dl.so` (the C++ `dl::` host layer: TensorBase, Module, Model).  This Python
package is only a thin ctypes driver for tests and benchmarks; PyTorch supplies device memory and
streams, nothing else.  The directory name is not a Python identifier: import it with
`importlib.import_module("esp-dl_amd")`.
"""
from . import capi  # noqa: F401
from .capi import (  # noqa: F401
    ConvDesc, EspdlHipError, LIB_PATH, add_s16, add_s8, avg_pool_s16, div_s16, div_s8, sub_s8, pad, reduce_int, mul_s16, reduce_mean_s16, sub_s16, avg_pool_s8, clip_s8, concat, conv2d, conv2d_gap_s8, conv_out_shape, global_avg_pool_s8, insert_zeros, lib, lut_s16, lut_s8,
    dequantize_f32, matmul_s8, max_pool, mbconv_s8, mul_s8, quantize_f32, softmax_s8, prelu_s8, reduce_mean_s8, relu_s8, requantize, requantize_s8, resize_nearest_s8, slice_, split, transpose,
)
from . import model, zoo  # noqa: F401,E402
