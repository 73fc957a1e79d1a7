/*
 * espdl_hip.h — C ABI of the MI355X (gfx950) kernels for ESP-DL's quantized operator path.
 *
 * Every entry point replaces one kernel-level interface of the reference's portable C path
 * (esp-dl/dl/base); the reference file:line each one stands in for is cited at its declaration.
 *
 * Conventions
 *   - All data pointers are DEVICE pointers (HBM).  Descriptors are host structs passed by pointer.
 *   - Activations are NHWC with a leading batch dimension; the reference is batch-1, so a batch of
 *     N is N independent reference calls on the N images.
 *   - Dense filter memory is [out_c][k_h][k_w][in_c]; depthwise filter memory is [k_h][k_w][c]
 *     (the reference's `c`-target layouts, dl_base_conv2d.cpp:23,64,140;
 *     dl_base_depthwise_conv2d.cpp:46-65).
 *   - `shift` is int32[n_shift] on the device, n_shift = 1 (per-tensor) or out_c (per-channel);
 *     shift[i] = out_exponent - filter_exponent[i] - in_exponent (dl_base.hpp:260).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls are
 *     asynchronous on that stream and allocate nothing.
 *   - Return value: ESPDL_HIP_OK (0) or a negative error code; nothing throws.  The message of the
 *     last error of the calling thread is available from espdl_hip_last_error().
 *   - Results are bit-exact with the reference's portable C path.  Supported shift range: int8
 *     paths -31..62 (half-up) / -31..30 (half-even); int16 paths -15..62 (half-up) / -15..62.
 */
#ifndef ESPDL_HIP_H
#define ESPDL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ESPDL_HIP_OK 0
#define ESPDL_HIP_EINVAL (-22)   /* bad descriptor / null pointer / unsupported geometry */
#define ESPDL_HIP_ENOTSUP (-95)  /* valid request the library does not implement          */
#define ESPDL_HIP_EDEVICE (-5)   /* HIP runtime reported an error at launch                */

/* element type of activations and filters: quant_type_t of the reference (dl_define.hpp:94-100) */
#define ESPDL_HIP_S8 8
#define ESPDL_HIP_S16 16

/* activation_type_t of the reference (dl_define.hpp:102-108).  The portable C path fuses only
 * Linear and ReLU into Conv/Gemm (dl_base_conv2d.cpp:1299-1329). */
#define ESPDL_HIP_LINEAR 0
#define ESPDL_HIP_RELU 1

/* tool::shift_and_round flavour (dl_tool.cpp:95-146).  HALF_UP is the portable C path;
 * HALF_EVEN is what ESP32-P4 builds select (dl_define_private.hpp:44-48). */
#define ESPDL_HIP_ROUND_HALF_UP 0
#define ESPDL_HIP_ROUND_HALF_EVEN 1

/*
 * Convolution descriptor: the fields base::ConvOpArgs<T> derives from its tensors and attributes
 * (esp-dl/dl/base/dl_base.hpp:133-262), plus the batch size.
 */
typedef struct espdl_hip_conv_desc {
    int32_t dtype; /* ESPDL_HIP_S8 or ESPDL_HIP_S16 */
    int32_t batch, in_h, in_w, in_c;
    int32_t out_c; /* dense: number of filters; depthwise: must equal in_c */
    int32_t k_h, k_w;
    int32_t stride_h, stride_w;
    int32_t dil_h, dil_w;
    int32_t pad_top, pad_bottom, pad_left, pad_right; /* ConvOpArgs padding order {t,b,l,r} */
    int32_t group;      /* 1 = dense conv / Gemm / MatMul; in_c = depthwise (dl_module_conv.hpp:104-119) */
    int32_t activation; /* ESPDL_HIP_LINEAR / ESPDL_HIP_RELU */
    int32_t round_mode; /* ESPDL_HIP_ROUND_HALF_UP / ESPDL_HIP_ROUND_HALF_EVEN */
    int32_t n_shift;    /* 1 or out_c */
    /* Channel pitches, in elements; 0 = dense (the tensor's own channel count).  A pitch larger than the channel
     * count means the operand is a channel slice of a wider NHWC tensor: `in` / `out` / `residual` point at the
     * slice's first channel of the first pixel and consecutive pixels lie pitch elements apart.  This is how a
     * Conv reads one output of a Split (esp-dl/dl/module/include/dl_module_split.hpp:84-152) or writes its part
     * of a Concat result (dl_module_concat.hpp:86-108) without the copy those operators make.  Dense int8
     * convolutions (group 1) only; ESPDL_HIP_ENOTSUP elsewhere. */
    int32_t in_pitch, out_pitch, res_pitch;
} espdl_hip_conv_desc;

/* Output spatial size, Conv::get_output_shape (esp-dl/dl/module/include/dl_module_conv.hpp:81-102). */
int espdl_hip_conv_out_shape(const espdl_hip_conv_desc *desc, int32_t *out_h, int32_t *out_w);

/*
 * Conv2D / DepthwiseConv2D / Gemm / MatMul with fused bias, shift-round, ReLU, saturation and an
 * optional 256-entry int8 LUT applied to the stored value.
 * Replaces base::conv2d<int8_t,int32_t,int32_t>, base::conv2d<int16_t,int32_t,int64_t>
 * (esp-dl/dl/base/dl_base_conv2d.hpp:15-16; dl_base_conv2d.cpp:912-939, 1383-1411) and
 * base::depthwise_conv2d<...> (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:495-519, 854-880)
 * together with conv_operation_shell / dwconv_operation_shell (dl_base.hpp:382-1196, 1209-2107)
 * and the n_wise epilogues (dl_base_activate_buffer.hpp:10-74, 162-212).
 *   bias : int32[out_c] (S8) or int64[out_c] (S16), or NULL
 *   lut  : int8[256] or NULL; S8 only.  out = lut[q + 128] as base::lut_s8 would compute on the
 *          conv output (dl_base_lut.cpp:10-15), i.e. Conv followed by a LUT module in one pass.
 * Gemm / MatMul: describe the input as {1, 1, M, K} with a 1x1 filter, as the reference does
 * (esp-dl/dl/module/include/dl_module_gemm.hpp:86-123).
 */
int espdl_hip_conv2d(const espdl_hip_conv_desc *desc, const void *in, const void *filter, const void *bias,
                     const int32_t *shift, const int8_t *lut, void *out, void *stream);

/*
 * espdl_hip_conv2d followed by base::elemwise_add of `residual` (esp-dl/dl/base/dl_base_add.cpp:34-44) in
 * the same launch: out = clamp_int8(conv_result + residual), where conv_result is the int8 value
 * espdl_hip_conv2d would have stored (after the optional LUT) and residual has the output's shape.
 * Dense int8 convolutions only (group 1); residual == NULL is plain espdl_hip_conv2d.
 */
int espdl_hip_conv2d_add(const espdl_hip_conv_desc *desc, const void *in, const void *filter, const void *bias,
                         const int32_t *shift, const int8_t *lut, const int8_t *residual, void *out, void *stream);

/* base::lut_s8 (esp-dl/dl/base/dl_base_lut.cpp:10-48): out[i] = table[(uint8)in[i] ^ 0x80]. In-place allowed. */
int espdl_hip_lut_s8(const int8_t *in, int64_t size, const int8_t *table, int8_t *out, void *stream);

/* base::prelu<int8_t> (esp-dl/dl/base/dl_base_prelu.cpp:7-21, args dl_base.hpp:2165-2168):
 * alpha is int8[channels]; shift = out_exp - in_exp - alpha_exp.  In-place allowed. */
int espdl_hip_prelu_s8(const int8_t *in, int64_t pixels, int32_t channels, const int8_t *alpha, int32_t shift,
                       int8_t *out, void *stream);

/* module::Relu::forward_template (esp-dl/dl/module/include/dl_module_relu.hpp:65-93). In-place allowed. */
int espdl_hip_relu_s8(const int8_t *in, int64_t size, int32_t in_exp, int32_t out_exp, int8_t *out, void *stream);

/* module::Clip::forward_template (esp-dl/dl/module/include/dl_module_clip.hpp:78-90); min_q / max_q
 * are the quantized scalar bounds.  In-place allowed. */
int espdl_hip_clip_s8(const int8_t *in, int64_t size, int32_t min_q, int32_t max_q, int32_t in_exp,
                      int32_t out_exp, int8_t *out, void *stream);

/*
 * base::elemwise_add for int8 (esp-dl/dl/base/dl_base_add.cpp:8-44, 80-153) with the broadcast
 * description of base::elemwiseArgsType (esp-dl/dl/base/dl_base_elemwise.hpp:19-52): the output is a
 * dense tensor of up to 4 dims `out_dims` (outermost first, unused leading dims = 1); each input is
 * addressed with element strides per output dim (0 = broadcast along that dim).
 * out = clamp(in0 + in1); exponents are not consulted (the exporter matches them).
 */
int espdl_hip_add_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int8_t *out, void *stream);

/*
 * base::elemwise_mul for int8 (esp-dl/dl/base/dl_base_mul.cpp:33-46, 83-160), same broadcast description
 * as espdl_hip_add_s8.  mul_shift = out_exp - in0_exp - in1_exp (elemwiseArgsType::mul_shift,
 * dl_base_elemwise.cpp:167): out = clamp(round(in0 * in1 / 2^mul_shift)); a negative shift multiplies.
 * ESPDL_HIP_ROUND_HALF_UP is the portable C path; ESPDL_HIP_ROUND_HALF_EVEN is how the ESP32-P4 kernels
 * of the reference round this operator.
 */
int espdl_hip_mul_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int32_t mul_shift, int32_t round_mode, int8_t *out,
                     void *stream);

/* A 1x1 stride-1 module::Conv followed by GlobalAveragePool in one launch (the head of a classification network:
 * Conv::forward, esp-dl/dl/module/include/dl_module_conv.hpp, then the pooling of
 * esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54 over the whole image): the convolution's int8 results - at exponent
 * conv_out_exp, activation applied, exactly what espdl_hip_conv2d would store - are summed per image and filter
 * inside the kernel and only the pooled tensor out[batch][out_c] (exponent pool_out_exp) is written.  desc as for
 * espdl_hip_conv2d (ESPDL_HIP_S8, group 1, ESPDL_HIP_LINEAR / _RELU); images of at most 64 pixels, in_c a
 * multiple of 16 and at least 64, at least 32 filters, in and filter 16-byte aligned; ESPDL_HIP_ENOTSUP otherwise
 * (espdl_hip_conv2d_gap_s8_supported answers 1 / 0 for a descriptor). */
int espdl_hip_conv2d_gap_s8_supported(const espdl_hip_conv_desc *desc);
int espdl_hip_conv2d_gap_s8(const espdl_hip_conv_desc *desc, const int8_t *in, const int8_t *filter, const int32_t *bias,
                            const int32_t *shift, int32_t conv_out_exp, int32_t pool_out_exp, int8_t *out, void *stream);

/* GlobalAveragePool over H x W per image and channel: base::avgpool2d_hwc with the filter covering
 * the whole image (esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54). out is [batch][1][1][c]. */
int espdl_hip_global_avg_pool_s8(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t in_exp,
                                 int32_t out_exp, int8_t *out, void *stream);

/* TensorBase::assign int8 -> int8 across exponents (esp-dl/dl/tensor/src/dl_tensor_base.cpp:362-371),
 * which is what a RequantizeLinear node runs. */
int espdl_hip_requantize_s8(const int8_t *in, int64_t size, int32_t in_exp, int32_t out_exp, int8_t *out,
                            void *stream);

/* int8 -> int8 requantization (TensorBase::assign, esp-dl/dl/tensor/src/dl_tensor_base.cpp:223-401) of `rows` runs
 * of row_bytes values that lie in_pitch / out_pitch bytes apart: the channels of one tensor when it, or its
 * destination, is a channel slice of a wider NHWC tensor (rows = pixels, row_bytes = channels). */
int espdl_hip_requantize_s8_rows(const int8_t *in, int64_t in_pitch, int8_t *out, int64_t out_pitch, int64_t row_bytes,
                                 int64_t rows, int32_t in_exp, int32_t out_exp, void *stream);

/* TensorBase::assign between int8 / int16 tensors of any two exponents
 * (esp-dl/dl/tensor/src/dl_tensor_base.cpp:321-392): same exponent widens (int8 -> int16) or saturates
 * (int16 -> int8); different exponents run quantize(dequantize(x)) in float32 with round-half-up.
 * in_dtype / out_dtype are ESPDL_HIP_S8 or ESPDL_HIP_S16.  This is the int8 <-> int16 boundary of a
 * mixed-precision graph. */
int espdl_hip_requantize(const void *in, int32_t in_dtype, int64_t size, int32_t in_exp, int32_t out_exp, void *out,
                         int32_t out_dtype, void *stream);

/*
 * module::Concat::forward_template (esp-dl/dl/module/include/dl_module_concat.hpp:86-108): for each of
 * the loop_times outer positions (product of the dims before the axis) one contiguous run from every
 * input in turn; copy_bytes[j] = bytes input j contributes per position (product of its dims from the
 * axis on, times the element size).  `inputs` and `copy_bytes` are host arrays of n_inputs entries read
 * during the call; inputs[j] are device pointers.  Any element type.
 */
int espdl_hip_concat(int32_t n_inputs, const void *const *inputs, const int64_t *copy_bytes, int64_t loop_times,
                     void *out, void *stream);

/* `rows` runs of row_bytes bytes, run r from src + r * src_pitch to dst + r * dst_pitch.  One output of
 * module::Split (esp-dl/dl/module/include/dl_module_split.hpp:84-93) is this with rows = num_slices,
 * row_bytes = slice_size * out_axis * sizeof(T), src_pitch = slice_size * in_axis * sizeof(T),
 * src = input + slice_index * slice_size * sizeof(T), dst_pitch = row_bytes. */
int espdl_hip_copy_rows(const void *src, int64_t src_pitch, void *dst, int64_t dst_pitch, int64_t row_bytes,
                        int64_t rows, void *stream);

/* All outputs of module::Split (esp-dl/dl/module/include/dl_module_split.hpp:84-152) in one pass over the input:
 * `rows` runs (num_slices) that lie in_pitch bytes apart are cut into n_outputs consecutive pieces of copy_bytes[j]
 * bytes (slice_size * out_axis_j * sizeof(T)); piece j of run r goes to outputs[j] + r * copy_bytes[j].  A NULL
 * output is skipped (a piece the caller reads in place).  `outputs` and `copy_bytes` are host arrays read during
 * the call. */
int espdl_hip_split(const void *in, int64_t in_pitch, int32_t n_outputs, void *const *outputs, const int64_t *copy_bytes,
                    int64_t rows, void *stream);

/* TensorBase::transpose (esp-dl/dl/tensor/src/dl_tensor_base.cpp:722-812): out.shape[i] =
 * shape[perm[i]].  1..8 dims, elem_size 1, 2 or 4 bytes; perm entries may be negative (counted from
 * the end) and n_perm = 0 reverses the dims.  shape and perm are host arrays. */
int espdl_hip_transpose(const void *in, const int32_t *shape, int32_t dims, const int32_t *perm, int32_t n_perm,
                        int32_t elem_size, void *out, void *stream);

/* base::resize<int8_t> in nearest mode (esp-dl/dl/base/dl_base_resize.cpp:7-34, 236-268; arguments
 * esp-dl/dl/base/dl_base_resize.hpp:37-92) on [batch][h][w][c] -> [batch][out_h][out_w][c].
 * scale_h / scale_w are the module's float scales (output / input); exactly 2 x 2 replicates pixels,
 * any other scale maps coordinates with in = min((int)(out * (1 / scale)), len - 1).  A different
 * output exponent rescales with round-half-up and, like the reference, without saturation. */
int espdl_hip_resize_nearest_s8(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t out_h,
                                int32_t out_w, float scale_h, float scale_w, int32_t in_exp, int32_t out_exp,
                                int8_t *out, void *stream);
/* The same on channel slices of wider NHWC tensors (in_pitch / out_pitch: elements from pixel to pixel, 0 = c), so
 * that the upsampling of a top-down path writes its part of the Concat behind it (dl_module_concat.hpp:86-108). */
int espdl_hip_resize_nearest_s8_pitched(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t out_h,
                                        int32_t out_w, float scale_h, float scale_w, int32_t in_exp, int32_t out_exp,
                                        int32_t in_pitch, int32_t out_pitch, int8_t *out, void *stream);

/* base::max_pool2d (esp-dl/dl/base/dl_base_max_pool2d.cpp:9-29) over the window clipped to the image;
 * output size (h + pad_top + pad_bottom - k_h) / stride_h + 1 and likewise for the width
 * (esp-dl/dl/module/include/dl_module_max_pool.hpp:42-49).  dtype ESPDL_HIP_S8 or ESPDL_HIP_S16; the
 * exponent is unchanged.  out is [batch][out_h][out_w][c]. */
int espdl_hip_max_pool(const void *in, int32_t dtype, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h,
                       int32_t k_w, int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom,
                       int32_t pad_left, int32_t pad_right, void *out, void *stream);
/* The same on channel slices of wider NHWC tensors: in_pitch / out_pitch are the elements from one pixel to
 * the next at `in` / `out` (0 = dense, c), as in espdl_hip_conv_desc.  This is how the chained pools of an
 * SPPF block (MaxPool -> MaxPool -> MaxPool -> Concat of all, dl_module_concat.hpp:86-108) write their parts
 * of the Concat result directly. */
int espdl_hip_max_pool_pitched(const void *in, int32_t dtype, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h,
                               int32_t k_w, int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom,
                               int32_t pad_left, int32_t pad_right, int32_t in_pitch, int32_t out_pitch, void *out,
                               void *stream);

/* base::avg_pool2d<int8_t> on the portable C path (esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54 under the
 * shell of dl_base_pool2d.hpp:439-560): sum over the window clipped to the image, times
 * 2^in_exp * (1 / (k_h * k_w)) * 2^-out_exp in float32 (the divisor is the full window also at the borders),
 * round half up, clamp.  Output size as espdl_hip_max_pool. */
int espdl_hip_avg_pool_s8(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h, int32_t k_w,
                          int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom, int32_t pad_left,
                          int32_t pad_right, int32_t in_exp, int32_t out_exp, int8_t *out, void *stream);

/* module::ReduceMean for int8 (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:16-45): mean over the
 * axes whose reduce_flag is non-zero, out = clamp(round(sum * 2^in_exp / count * 2^-out_exp)) in float32.
 * `out` holds the kept axes in order (keepdims changes only the shape).  shape and reduce_flag are host
 * arrays of `dims` entries, 1..8 dims. */
int espdl_hip_reduce_mean_s8(const int8_t *in, const int32_t *shape, int32_t dims, const int32_t *reduce_flag,
                             int32_t in_exp, int32_t out_exp, int8_t *out, void *stream);

/* int16 forms.  espdl_hip_add_s16: c_impl_add_n_n<int16_t> (esp-dl/dl/base/dl_base_add.cpp:33-44), saturating
 * add.  espdl_hip_mul_s16: c_impl_mul_n_n<int16_t> (esp-dl/dl/base/dl_base_mul.cpp:33-46): the int32 product is
 * converted to float32, scaled by 2^-mul_shift and rounded half up (ESPDL_HIP_ROUND_HALF_UP), or shifted and
 * rounded half to even as an integer (ESPDL_HIP_ROUND_HALF_EVEN, the ESP32-P4 kernels).  Broadcast description
 * as espdl_hip_add_s8.  espdl_hip_avg_pool_s16: avgpool2d_hwc<int16_t, int32_t> (dl_base_avg_pool2d.cpp:28-54,
 * :87), arguments as espdl_hip_avg_pool_s8.  espdl_hip_reduce_mean_s16: reduce<int64_t, int16_t>
 * (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:18-56), arguments as espdl_hip_reduce_mean_s8. */
int espdl_hip_add_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int16_t *out, void *stream);
int espdl_hip_mul_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int32_t mul_shift, int32_t round_mode, int16_t *out,
                      void *stream);
/* base::elemwise_sub for int16 (esp-dl/dl/base/dl_base_sub.cpp:33-43): saturating in0 - in1. */
int espdl_hip_sub_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int16_t *out, void *stream);
/* base::elemwise_div for int16 (esp-dl/dl/base/dl_base_div.cpp:66-68, 92-112, 141-163, 175-195, 244-252): float32,
 * div_shift = out_exp - in0_exp + in1_exp; out = round(in0 * 2^-div_shift / in1), evaluated in the order of the
 * reference loop that matches the broadcast (divisor constant along the innermost axis: in0 * (2^-s / in1);
 * dividend constant: (in0 * 2^-s) / in1); in0 == 0 gives 0, in1 == 0 the int16 extreme of in0's sign. */
int espdl_hip_div_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int32_t div_shift, int16_t *out, void *stream);
/* base::elemwise_sub and base::elemwise_div for int8 (esp-dl/dl/base/dl_base_sub.cpp:33-43;
 * esp-dl/dl/base/dl_base_div.cpp:8-46, 66-70, 92-130, 141-175, 208-224).  Sub saturates in0 - in1 to int8.  Div is
 * the float32 arithmetic of espdl_hip_div_s16 with int8 limits; where an operand is a one-element tensor the
 * reference reads a 256-entry table built from the same expressions, which differs in one entry only: a
 * one-element dividend of 0 over a divisor of 0 gives -128.  A one-element divisor of 0 is undefined in the
 * reference (a float infinity converted to int); here it gives the int8 extreme of in0's sign, 0 for in0 == 0. */
int espdl_hip_sub_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int8_t *out, void *stream);
int espdl_hip_div_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int32_t div_shift, int8_t *out, void *stream);
int espdl_hip_avg_pool_s16(const int16_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h, int32_t k_w,
                           int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom, int32_t pad_left,
                           int32_t pad_right, int32_t in_exp, int32_t out_exp, int16_t *out, void *stream);
int espdl_hip_reduce_mean_s16(const int16_t *in, const int32_t *shape, int32_t dims, const int32_t *reduce_flag,
                              int32_t in_exp, int32_t out_exp, int16_t *out, void *stream);

/* module::InsertZeros (esp-dl/dl/module/include/dl_module_insert_zeros.hpp; the exporter places it in front of
 * a Conv to express a transposed convolution): in is [batch][h][w][c] of elem_size-byte elements, out is
 * [batch][out_h][out_w][c] with out_h = h + (stride_h - 1) * (h - 1) + output_padding_h (same for w);
 * out[n][y * stride_h][x * stride_w] = in[n][y][x], every other element 0.  1-D tensors pass w = 1. */
int espdl_hip_insert_zeros(const void *in, int32_t elem_size, int32_t batch, int32_t h, int32_t w, int32_t c,
                           int32_t stride_h, int32_t stride_w, int32_t output_padding_h, int32_t output_padding_w,
                           void *out, void *stream);

/* module::ReduceMax, ReduceMin, ReduceSum for int8 / int16 (esp-dl/dl/module/include/dl_module_reduce_max.hpp:14-52,
 * dl_module_reduce_min.hpp:15-53, dl_module_reduce_sum.hpp:13-56; loop nest dl_module_reduce_base.hpp).  dtype is
 * ESPDL_HIP_S8 or ESPDL_HIP_S16; shape / reduce_flag as espdl_hip_reduce_mean_s8.  Max and min return stored
 * integers and ignore shift; the sum (int32 for int8, int64 for int16) is shift_and_round(sum, shift) with
 * shift = out_exp - in_exp, then saturated.  ReduceL1 and ReduceSumSquare (dl_module_reduce_l1.hpp:14-50,
 * dl_module_reduce_sum_square.hpp:14-46) sum |x| and x * x the same way, the latter with
 * shift = out_exp - 2 * in_exp.  An empty reduction gives the identity (type minimum, maximum, 0). */
enum {
    ESPDL_HIP_REDUCE_MAX = 0,
    ESPDL_HIP_REDUCE_MIN = 1,
    ESPDL_HIP_REDUCE_SUM = 2,
    ESPDL_HIP_REDUCE_L1 = 3,        /* sum of |x|, shift = out_exp - in_exp */
    ESPDL_HIP_REDUCE_SUM_SQUARE = 4 /* sum of x * x, shift = out_exp - 2 * in_exp */
};
int espdl_hip_reduce_int(const void *in, int32_t dtype, const int32_t *shape, int32_t dims, const int32_t *reduce_flag,
                         int32_t op, int32_t shift, int32_t round_mode, void *out, void *stream);

/* module::Pad = TensorBase::pad (esp-dl/dl/module/include/dl_module_pad.hpp:33-40;
 * esp-dl/dl/tensor/src/dl_tensor_base.cpp:1225-1299; base::pad1D..pad4D, esp-dl/dl/base/dl_base_pad.cpp:19-260).
 * `shape` has `dims` (1..8) extents, `pads` 2 * dims entries: the leading pad of every axis, then the trailing pad
 * of every axis (the ONNX order the reference keeps).  out has extents shape[i] + pads[i] + pads[i + dims].
 * ESPDL_HIP_PAD_CONSTANT fills with constant_value (converted to the element type), ESPDL_HIP_PAD_EDGE repeats
 * the border element, ESPDL_HIP_PAD_REFLECT mirrors about it (pads shorter than the axis).  elem_size 1, 2, 4. */
enum { ESPDL_HIP_PAD_CONSTANT = 0, ESPDL_HIP_PAD_EDGE = 1, ESPDL_HIP_PAD_REFLECT = 2 };
int espdl_hip_pad(const void *in, const int32_t *shape, int32_t dims, const int32_t *pads, int32_t mode,
                  int32_t constant_value, int32_t elem_size, void *out, void *stream);

/* module::LUT for int16 (esp-dl/dl/module/include/dl_module_lut.hpp:61-74; base::lut_s16_nearest_neighbor and
 * lut_index, esp-dl/dl/base/dl_base_lut.cpp:49-77): `table` (device) holds table_size = 65536 / step + 1
 * entries, step a power of two, or 65536 entries; out = table[round((in + 32768) / step)].  Ties go up with
 * ESPDL_HIP_ROUND_HALF_UP (portable C path) and to the even index with ESPDL_HIP_ROUND_HALF_EVEN (the
 * ESP32-P4 build). */
int espdl_hip_lut_s16(const int16_t *in, int64_t size, const int16_t *table, int32_t table_size, int32_t round_mode,
                      int16_t *out, void *stream);

/* module::Softmax on an int8 tensor (Softmax::forward_lut, esp-dl/dl/module/include/dl_module_softmax.hpp:148-217):
 * the tensor is viewed as [outer][len][inner] and normalized along len; out is float32 of the same
 * layout, out = T[q] / sum_i T[q_i] with T[q] = expf(2^in_exp * q), the sum taken in float32 in index
 * order.  No maximum is subtracted, as in the reference's int8 path. */
int espdl_hip_softmax_s8(const int8_t *in, int64_t outer, int64_t len, int64_t inner, int32_t in_exp, float *out,
                         void *stream);

/* QuantizeLinear: TensorBase::assign from float32 (esp-dl/dl/tensor/src/dl_tensor_base.cpp:251-268):
 * out = clamp(round_half_up(in * 2^-out_exp)).  elem_size 1 writes int8, 2 writes int16. */
int espdl_hip_quantize_f32(const float *in, int64_t size, int32_t out_exp, int32_t elem_size, void *out, void *stream);

/* DequantizeLinear: TensorBase::assign into float32 (dl_tensor_base.cpp:286-299): out = in * 2^in_exp.
 * elem_size 1 reads int8, 2 reads int16. */
int espdl_hip_dequantize_f32(const void *in, int64_t size, int32_t in_exp, int32_t elem_size, float *out, void *stream);

/* module::MatMul with two int8 activations (batched branches of MatMul::forward_template,
 * esp-dl/dl/module/include/dl_module_matmul.hpp): for each of lead[0] x lead[1] leading index pairs
 * out[z0][z1] = a[z0][z1] ([m][k]) x b[z0][z1] ([k][n]), each run as the reference's 1x1 convolution with
 * one shift = out_exp - a_exp - b_exp, ESPDL_HIP_LINEAR / _RELU and the given round mode.  a_stride and
 * b_stride give each operand's element stride per leading dim (0 broadcasts that operand); out is dense
 * [lead[0]][lead[1]][m][n].  lead[0] * lead[1] <= 65535. */
int espdl_hip_matmul_s8(const int8_t *a, const int8_t *b, int32_t m, int32_t k, int32_t n, const int32_t lead[2],
                        const int64_t a_stride[2], const int64_t b_stride[2], int32_t shift, int32_t activation,
                        int32_t round_mode, int8_t *out, void *stream);

/* TensorBase::slice for positive steps (esp-dl/dl/base/dl_base_shape.cpp:68-120 gives the shape rule):
 * out[i0, i1, ...] = in[start[0] + i0 * step[0], start[1] + i1 * step[1], ...].  The caller passes
 * normalized values per dim (0 <= start, step >= 1, out_shape) for all `dims` dims of the input;
 * host arrays.  1..8 dims, elem_size 1, 2 or 4. */
int espdl_hip_slice(const void *in, const int32_t *shape, int32_t dims, const int32_t *start, const int32_t *step,
                    const int32_t *out_shape, int32_t elem_size, void *out, void *stream);

/*
 * Inverted-residual block in one launch: [1x1 Conv] -> depthwise Conv -> 1x1 Conv [-> Add].
 * No single reference function does this; it runs the same sequence of module::Conv::forward
 * (esp-dl/dl/module/include/dl_module_conv.hpp:121-162) and module::Add::forward
 * (esp-dl/dl/base/dl_base_add.cpp:34-44) calls as the separate entry points above, with the int8 result
 * of every stage formed exactly as espdl_hip_conv2d forms it, but keeps the expanded activation in
 * on-chip memory.  Results are bit-identical to the separate calls.
 *   has_expand = 0: the block starts at the depthwise stage and exp_c must equal in_c.
 *   Filters use the layouts of espdl_hip_conv2d: expand [exp_c][in_c], depthwise [k_h][k_w][exp_c],
 *   project [out_c][exp_c]; biases int32 or NULL; shifts int32[1 or channels] per stage.
 *   residual: int8 tensor of the output's shape added with saturation after the project stage, or NULL.
 * Needs exp_c % 16 == 0, in_c % 16 == 0, out_c % 4 == 0, at most 12 depthwise taps, in_c <= 192,
 * exp_c <= 1024, out_c <= 384, 16-byte aligned input and filters; espdl_hip_mbconv_s8_supported() answers for a descriptor: 0 = no, 1 = yes (general
 * fused kernel), 2 = yes, through the depthwise+project kernel (no expand stage, at most 256
 * channels), 3 = yes, expand stage inside the LDS-tile depthwise kernel, 4 = yes, one wavefront per tile
 * (3x3 depthwise stage, at most 64 block-input channels and 64 project filters), 5 = yes, a workgroup of
 * wavefronts per tile of a small image (output at most 16 pixels wide, block-input channels a multiple of
 * 16 and at most 192).  An expand stage with a window (exp_k_h, exp_k_w not 1: at most 4 rows of at most
 * 9 bytes, i.e. exp_k_w * in_c <= 9) is taken by the one-wavefront-per-tile kernel only.
 * espdl_hip_mbconv_s8 returns ESPDL_HIP_ENOTSUP where it does not apply.
 */
typedef struct espdl_hip_mbconv_desc {
    int32_t batch, in_h, in_w, in_c;
    int32_t exp_c, out_c;
    int32_t has_expand;
    int32_t k_h, k_w, stride_h, stride_w, dil_h, dil_w;               /* depthwise stage */
    int32_t pad_top, pad_bottom, pad_left, pad_right;                 /* depthwise stage */
    int32_t act_expand, act_dw, act_project;                          /* ESPDL_HIP_LINEAR / ESPDL_HIP_RELU */
    int32_t round_mode;
    int32_t n_shift_expand, n_shift_dw, n_shift_project;              /* 1 or channels of the stage */
    /* Expand stage other than a 1x1 convolution (a stem convolution in front of the first depthwise stage):
     * window, stride and padding of a dense convolution over the block input; in_h / in_w are then the
     * extents of the block input and the depthwise stage works on that convolution's output.  All eight
     * zero: the 1x1 stride-1 convolution.  Filter layout [exp_c][exp_k_h][exp_k_w][in_c]. */
    int32_t exp_k_h, exp_k_w, exp_stride_h, exp_stride_w;
    int32_t exp_pad_top, exp_pad_bottom, exp_pad_left, exp_pad_right;
    /* The residual operand stands at another exponent than the block output: it is requantized by
     * 2^residual_shift first (residual exponent - output exponent, -7 .. 7; round half up and saturate, as
     * TensorBase::assign does for the RequantizeLinear node that an exporter puts in front of such an Add,
     * esp-dl/dl/tensor/src/dl_tensor_base.cpp:362-371).  0: the operand is added as it is.  Taken by the
     * single-launch kernels of answers 4 and 5 only; espdl_hip_mbconv_s8_supported answers 0 elsewhere. */
    int32_t residual_shift;
    /* A Clip between two stages whose input and output exponents are equal (module::Clip::forward,
     * esp-dl/dl/module/include/dl_module_clip.hpp:78-90: the rescale factor is 1 and the operator is a clamp of
     * the stored int8 value; a ReLU6 exported as Clip): clip_expand != 0 clamps the expand stage's int8 result
     * to [clip_expand_min, clip_expand_max] before the depthwise stage reads it (the zero padding of the
     * depthwise window pads the CLAMPED activation, as with separate operators), clip_dw != 0 the depthwise
     * stage's result before the project stage.  Bounds in -128 .. 127, min <= max.  Taken by the
     * one-wavefront-per-tile kernel (answer 4) where its tile plan has a guard-free build, round half up;
     * espdl_hip_mbconv_s8_supported answers 0 elsewhere. */
    int32_t clip_expand, clip_expand_min, clip_expand_max;
    int32_t clip_dw, clip_dw_min, clip_dw_max;
} espdl_hip_mbconv_desc;

typedef struct espdl_hip_mbconv_weights {
    const int8_t *w_expand;
    const int32_t *b_expand, *s_expand;
    const int8_t *w_dw;
    const int32_t *b_dw, *s_dw;
    const int8_t *w_project;
    const int32_t *b_project, *s_project;
} espdl_hip_mbconv_weights;

int espdl_hip_mbconv_out_shape(const espdl_hip_mbconv_desc *desc, int32_t *out_h, int32_t *out_w);
int espdl_hip_mbconv_s8_supported(const espdl_hip_mbconv_desc *desc);
/* 1 when the single launch is expected to be faster than the separate launches for this descriptor,
 * rounding mode included (the rule follows measurements on MI355X at batch sizes from 1 to 512: the
 * one-wavefront-per-tile kernel, answer 4 of espdl_hip_mbconv_s8_supported, and the workgroup-per-tile kernel,
 * answer 5, where the tile plan has one of the guard-free builds, which exist for the block shapes of
 * MobileNetV2-style networks in both rounding modes; the depthwise+project form, answer 2, always); 0
 * otherwise.  dl::Model fuses blocks by this answer. */
int espdl_hip_mbconv_s8_preferred(const espdl_hip_mbconv_desc *desc);
int espdl_hip_mbconv_s8(const espdl_hip_mbconv_desc *desc, const int8_t *in, const espdl_hip_mbconv_weights *weights,
                        const int8_t *residual, int8_t *out, void *stream);

/*
 * The same block as espdl_hip_mbconv_s8, run as its separate stages ([1x1 Conv] -> depthwise Conv ->
 * 1x1 Conv [+ Add]: espdl_hip_conv2d, espdl_hip_conv2d, espdl_hip_conv2d_add on `stream`) with the two
 * intermediate activations in device memory that belongs to the library.  It has no counterpart in the
 * reference; it exists for callers that cannot allocate device memory and whose block shape the
 * single-launch kernels do not cover (espdl_hip_mbconv_s8_supported() == 0): code under HIP-graph
 * capture, serving loops, harnesses that forbid hipMalloc.  It allocates nothing and accepts every shape
 * espdl_hip_conv2d accepts, with or without Clips between the stages; a requantized residual operand
 * (residual_shift != 0) is refused with ESPDL_HIP_ENOTSUP (requantize it first).  Results are bit-identical to
 * espdl_hip_mbconv_s8 and to the separate calls.
 * The first call on a device looks up the array's address, which must not happen while `stream` records a
 * graph: call espdl_hip_mbconv_s8_staged_init() (or the entry point itself) once per device outside capture;
 * a first call under capture returns ESPDL_HIP_ENOTSUP.
 * The intermediates (batch*in_h*in_w*exp_c bytes when has_expand, plus batch*out_h*out_w*exp_c bytes, each
 * rounded up to 256) must fit ESPDL_HIP_MBCONV_STAGED_MAX_BYTES, else ESPDL_HIP_ENOTSUP: split the batch.
 * Every call on a device uses the same array: calls that overlap on one device (two streams, two threads)
 * race; calls ordered on one stream are safe.  The array stays allocated on every device the library
 * has been used on until the process ends.
 */
#define ESPDL_HIP_MBCONV_STAGED_MAX_BYTES (64u << 20)
int espdl_hip_mbconv_s8_staged(const espdl_hip_mbconv_desc *desc, const int8_t *in,
                               const espdl_hip_mbconv_weights *weights, const int8_t *residual, int8_t *out,
                               void *stream);
/* Set-up of espdl_hip_mbconv_s8_staged on the current device (address of the library's array); allocates
 * nothing, launches nothing.  No counterpart in the reference. */
int espdl_hip_mbconv_s8_staged_init(void);

/* Library / device information. */
const char *espdl_hip_last_error(void);
const char *espdl_hip_version(void);
/* Number of compute units of the current device (0 if none can be queried). */
int espdl_hip_device_cu_count(void);

#ifdef __cplusplus
}
#endif
#endif /* ESPDL_HIP_H */
