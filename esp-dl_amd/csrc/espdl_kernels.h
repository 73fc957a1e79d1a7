// Internal launch interface between the C ABI (espdl_hip_api.hip) and the kernel files.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace espdl {

// Sets the calling thread's espdl_hip_last_error() text; returns `code` (defined in espdl_hip_api.hip).
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Geometry every convolution kernel works from (derived once on the host by the C ABI).
struct ConvGeom {
    int batch, in_h, in_w, in_c;
    int out_c, out_h, out_w;
    int k_h, k_w, stride_h, stride_w, dil_h, dil_w, pad_top, pad_left;
    int relu, half_even, n_shift;
    // channel pitches of input, output and residual operand in elements (>= the channel count; equal: dense)
    int in_pitch, out_pitch, res_pitch;
};
inline bool conv_is_dense(const ConvGeom &g)
{
    return g.in_pitch == g.in_c && g.out_pitch == g.out_c && g.res_pitch == g.out_c;
}

// Dense int8 convolution / Gemm as an implicit GEMM on v_mfma_i32_16x16x64_i8.
hipError_t launch_conv2d_s8_mfma(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                 const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                 int cu_count, hipStream_t stream);

// Pointwise int8 convolution / Gemm as a tiled GEMM with both operands streamed through LDS; for layers
// with few pixels per compute unit, where the implicit-GEMM kernel's filter staging dominates.
bool conv2d_s8_pwgemm_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count);
bool conv2d_s8_rows_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count);
hipError_t launch_conv2d_s8_pwgemm(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                   const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                   int cu_count, hipStream_t stream);
// A convolution with a window through the pointwise GEMM kernel, rows gathered from under the window (channels a
// multiple of 64, few output pixels per compute unit, a long reduction axis).
bool conv2d_s8_wingemm_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count);
hipError_t launch_conv2d_s8_wingemm(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                    const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                    int cu_count, hipStream_t stream);
// Dense int8 convolution with a window, input tile and filters staged in LDS (conv2d_s8_tiled.hip): channel
// count a multiple of 16, 16-byte aligned input and filter.
bool conv2d_s8_tiled_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count);
hipError_t launch_conv2d_s8_tiled(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                  const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                  int cu_count, hipStream_t stream);
// The pointwise convolution followed by GlobalAveragePool, writing only the pooled [batch][out_c] tensor (images
// of at most 64 pixels); gap_scale from global_avg_pool_scale.
bool conv2d_gap_s8_supports(const ConvGeom &g, const void *in, const void *filter);
hipError_t launch_conv2d_gap_s8(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                const int32_t *shift, float gap_scale, int8_t *out, int cu_count, hipStream_t stream);
float global_avg_pool_scale(int h, int w, int in_exp, int out_exp);

hipError_t launch_depthwise_s8(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                               const int32_t *shift, const int8_t *lut, int8_t *out, hipStream_t stream);

// Depthwise on the matrix pipe with a diagonal operand A (up to 12 taps, channels % 16 == 0).
bool depthwise_s8_mfma_supports(const ConvGeom &g, const void *in, const void *out);
hipError_t launch_depthwise_s8_mfma(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                    const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count,
                                    hipStream_t stream);

// 1x1 project convolution (+ saturating residual Add) fused behind a depthwise convolution.
struct DwProject {
    const int8_t *w; // [out_c][channels of the depthwise stage]
    const int32_t *bias, *shift;
    int n_shift, relu, out_c;
    const int8_t *residual; // shape of out, or nullptr
    int8_t *out;
};

// 1x1 expand convolution fused in front of a depthwise convolution: the depthwise kernel computes its input
// patch from `x` ([batch][in_h][in_w][c0], c0 <= 64 and a multiple of 4) instead of reading it.
struct DwExpand {
    const int8_t *x;
    const int8_t *w; // [depthwise channels][c0]
    const int32_t *bias, *shift;
    int n_shift, relu, c0;
};

// Depthwise with the input tile staged in LDS (contiguous global reads and writes) and the products
// on the matrix pipe; same shape limits as the direct form.
bool depthwise_s8_lds_supports(const ConvGeom &g, const void *in, const void *out);
hipError_t launch_depthwise_s8_lds(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                   const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count,
                                   hipStream_t stream);

// Inverted-residual block as one kernel: [1x1 expand conv] -> depthwise conv -> 1x1 project conv
// [-> saturating Add of `residual`].  w_expand == nullptr means there is no expand stage
// (exp_c == in_c).  Filters are in the layouts of the separate kernels; every shift array has 1 or
// <channels> entries.
struct MbconvParams {
    const int8_t *in;
    const int8_t *residual; // same shape as out, or nullptr
    int8_t *out;
    const int8_t *w_expand; // [exp_c][in_c]
    const int32_t *b_expand, *s_expand;
    const int8_t *w_dw; // [k_h][k_w][exp_c]
    const int32_t *b_dw, *s_dw;
    const int8_t *w_project; // [out_c][exp_c]
    const int32_t *b_project, *s_project;
    int n_s_expand, n_s_dw, n_s_project;
    int batch, in_h, in_w, in_c, exp_c, out_c, out_h, out_w;
    int k_h, k_w, stride_h, stride_w, dil_h, dil_w, pad_top, pad_left;
    int relu_expand, relu_dw, relu_project, half_even;
    // Expand stage with a window (ek_h x ek_w not 1 x 1, or a stride, or padding): in_h / in_w above stay the
    // extents of the DEPTHWISE stage's input (the expand convolution's output), img_h / img_w are those of
    // the block input, w_expand is [exp_c][ek_h][ek_w][in_c].  For the 1x1 expand img == in and ek == es == 1.
    int img_h, img_w, ek_h, ek_w, es_h, es_w, epad_top, epad_left;
    // The residual operand is requantized by 2^residual_shift (round half up, saturated) before the Add:
    // a RequantizeLinear between two int8 exponents in front of the Add.  -7 .. 7; only the one-wavefront-per-tile
    // and the workgroup-per-tile kernels take a value other than 0.
    int residual_shift;
    // Clamp of a stage's int8 result before the next stage reads it (a Clip with equal exponents between the
    // stages); only the guard-free builds of the one-wavefront-per-tile kernel take it.
    int clip_e, clip_e_lo, clip_e_hi, clip_d, clip_d_lo, clip_d_hi;
};
inline bool mbconv_has_clip(const MbconvParams &p)
{
    return p.clip_e != 0 || p.clip_d != 0;
}
inline bool mbconv_expand_is_pointwise(const MbconvParams &p)
{
    return p.ek_h == 1 && p.ek_w == 1 && p.es_h == 1 && p.es_w == 1 && p.epad_top == 0 && p.epad_left == 0 &&
        p.img_h == p.in_h && p.img_w == p.in_w;
}
bool mbconv_s8_fused_supports(const MbconvParams &p);
hipError_t launch_mbconv_s8_fused(const MbconvParams &p, int cu_count, hipStream_t stream);

// The same block with one wavefront per output tile and no workgroup barriers (mbconv_s8_wave.hip): 3x3
// depthwise stage with stride 1 or 2, at most 64 block-input channels and 64 project filters.
bool mbconv_s8_wave_supports(const MbconvParams &p);
// Does the launch take one of the guard-free builds (compiled for the tile plans of MobileNetV2-style blocks)?
// The guarded builds cover every supported shape but do not beat the separate launches.
bool mbconv_s8_wave_has_fast_build(const MbconvParams &p);
hipError_t launch_mbconv_s8_wave(const MbconvParams &p, int cu_count, hipStream_t stream);

// The same block for small images (output at most 16 pixels wide): a workgroup of eight wavefronts per tile
// splits the expanded channels (mbconv_s8_group.hip); block-input channels a multiple of 16, at most 192.
bool mbconv_s8_group_supports(const MbconvParams &p);
bool mbconv_s8_group_has_fast_build(const MbconvParams &p);
hipError_t launch_mbconv_s8_group(const MbconvParams &p, int cu_count, hipStream_t stream);

// Depthwise -> 1x1 project [-> Add] in one launch of the LDS-tile depthwise kernel: the depthwise
// result never leaves LDS.  Needs at most 256 depthwise channels.
bool depthwise_project_s8_supports(const ConvGeom &g, const void *in, const DwProject &pj);
hipError_t launch_depthwise_project_s8(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                       const int32_t *shift, const DwProject &pj, int cu_count, hipStream_t stream);

// 1x1 expand -> depthwise -> 1x1 project [-> Add] in one launch of the same kernel: neither the expanded
// tensor nor the depthwise result exists in memory.  Needs at most 256 expanded channels and c0 <= 64.
bool expand_depthwise_project_s8_supports(const ConvGeom &g, const DwExpand &ex, const DwProject &pj);
hipError_t launch_expand_depthwise_project_s8(const ConvGeom &g, const DwExpand &ex, const int8_t *filter,
                                              const int32_t *bias, const int32_t *shift, const DwProject &pj,
                                              int cu_count, hipStream_t stream);

// Dense int8 convolution whose window rows are at most 16 contiguous bytes (k_w * in_c <= 16, k_h <= 4, at most
// 64 filters): the first layer of a network on RGB / grey images, one MFMA step per 16 pixels (conv2d_s8_stem.hip).
bool conv2d_s8_stem_supports(const ConvGeom &g, const void *residual);
hipError_t launch_conv2d_s8_stem(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                 const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count, hipStream_t stream);

// Dense int16 convolution on the int8 matrix pipe (two signed bytes per operand); in_c % 16 == 0, reduction length <= 36000.
bool conv2d_s16_mfma_supports(const ConvGeom &g, const void *in, const void *filter, const void *out);
hipError_t launch_conv2d_s16_mfma(const ConvGeom &g, const int16_t *in, const int16_t *filter, const int64_t *bias,
                                  const int32_t *shift, int16_t *out, int cu_count, hipStream_t stream);
hipError_t launch_conv2d_s16(const ConvGeom &g, const int16_t *in, const int16_t *filter, const int64_t *bias,
                             const int32_t *shift, int16_t *out, hipStream_t stream);
hipError_t launch_depthwise_s16(const ConvGeom &g, const int16_t *in, const int16_t *filter, const int64_t *bias,
                                const int32_t *shift, int16_t *out, hipStream_t stream);

hipError_t launch_lut_s8(const int8_t *in, int64_t size, const int8_t *table, int8_t *out, hipStream_t stream);
hipError_t launch_prelu_s8(const int8_t *in, int64_t pixels, int channels, const int8_t *alpha, int shift,
                           int8_t *out, hipStream_t stream);
hipError_t launch_relu_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out, hipStream_t stream);
hipError_t launch_clip_s8(const int8_t *in, int64_t size, int min_q, int max_q, int in_exp, int out_exp, int8_t *out,
                          hipStream_t stream);
hipError_t launch_add_s8(const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                         const int8_t *in1, int8_t *out, hipStream_t stream);
hipError_t launch_mul_s8(const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                         const int8_t *in1, int shift, int half_even, int8_t *out, hipStream_t stream);
hipError_t launch_global_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int in_exp, int out_exp,
                                     int8_t *out, hipStream_t stream);
// rows of row_bytes int8 values that lie in_pitch / out_pitch bytes apart (channel slices of wider tensors)
hipError_t launch_requantize_s8_rows(const int8_t *in, int64_t in_pitch, int8_t *out, int64_t out_pitch, int64_t row_bytes,
                                     int64_t rows, int in_exp, int out_exp, hipStream_t stream);
hipError_t launch_requantize_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out,
                                hipStream_t stream);

hipError_t launch_requantize_any(const void *in, int in_bits, int64_t size, int in_exp, int out_exp, void *out,
                                 int out_bits, hipStream_t stream);

// Data-movement operators (layout_ops.hip).
// Split: `rows` runs of the input, in_pitch bytes apart, cut into n_outputs consecutive pieces of copy_bytes[j] bytes;
// piece j of run r goes to outputs[j] + r * copy_bytes[j] (a null output is skipped).  One pass in input order.
hipError_t launch_split(const void *in, long long in_pitch, int n_outputs, void *const *outputs, const long long *copy_bytes,
                        long long rows, int cu_count, hipStream_t stream);
hipError_t launch_copy_rows(const void *src, long long src_pitch, void *dst, long long dst_pitch, long long row_bytes,
                            long long rows, int cu_count, hipStream_t stream);
hipError_t launch_concat(int n_inputs, const void *const *inputs, const long long *copy_bytes, long long loop_times,
                         void *out, int cu_count, hipStream_t stream);
hipError_t launch_transpose(const void *in, const int *shape, int dims, const int *perm, int elem_size, void *out,
                            int cu_count, hipStream_t stream);
hipError_t launch_resize_nearest_s8(const int8_t *in, int batch, int h, int w, int c, int out_h, int out_w, float scale_h,
                                    float scale_w, int in_exp, int out_exp, long long in_pitch, long long out_pitch,
                                    int8_t *out, int cu_count, hipStream_t stream);
// in_pitch / out_pitch: elements from pixel to pixel (c for dense tensors, more for channel slices)
hipError_t launch_max_pool(const void *in, int elem_size, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                           int stride_w, int pad_top, int pad_left, int out_h, int out_w, long long in_pitch,
                           long long out_pitch, void *out, int cu_count, hipStream_t stream);
// int8, square windows of 2 / 3 / 5 at stride 1, channels and pitches in multiples of 16 (max_pool_s8.hip)
bool max_pool_s8_window_supports(const void *in, int h, int w, int c, int k_h, int k_w, int stride_h, int stride_w,
                                 int pad_top, int pad_left, int out_h, int out_w, long long in_pitch, long long out_pitch,
                                 const void *out);
hipError_t launch_max_pool_s8_window(const void *in, int batch, int h, int w, int c, int k, int pad_top, int pad_left,
                                     int out_h, int out_w, long long in_pitch, long long out_pitch, void *out,
                                     int cu_count, hipStream_t stream);

hipError_t launch_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                              int stride_w, int pad_top, int pad_left, int out_h, int out_w, int in_exp, int out_exp,
                              int8_t *out, int cu_count, hipStream_t stream);
hipError_t launch_pad(const void *in, const int *shape, int dims, const int *pads, int mode, int value, int elem_size,
                      void *out, int cu_count, hipStream_t stream);
hipError_t launch_slice(const void *in, const int *shape, int dims, const int *start, const int *step, const int *out_shape,
                        int elem_size, void *out, int cu_count, hipStream_t stream);

hipError_t launch_reduce_mean_s8(const int8_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                 int out_exp, int8_t *out, int cu_count, hipStream_t stream);

hipError_t launch_insert_zeros(const void *in, int elem_size, int batch, int h, int w, int c, int stride_h, int stride_w,
                               int out_h, int out_w, void *out, int cu_count, hipStream_t stream);

// elementwise_s16.hip
hipError_t launch_binary_s16(int op, const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int16_t *in0,
                             const int16_t *in1, int shift, bool half_even, int16_t *out, int cu_count, hipStream_t stream);
hipError_t launch_subdiv_s8(bool div, const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                            const int8_t *in1, int shift, int8_t *out, int cu_count, hipStream_t stream);
hipError_t launch_reduce_int(const void *in, int bits, const int *shape, int dims, const int *reduce_flag, int op,
                             int shift, bool half_even, void *out, int cu_count, hipStream_t stream);
hipError_t launch_avg_pool_s16(const int16_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                               int stride_w, int pad_top, int pad_left, int out_h, int out_w, int in_exp, int out_exp,
                               int16_t *out, int cu_count, hipStream_t stream);
hipError_t launch_reduce_mean_s16(const int16_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                  int out_exp, int16_t *out, int cu_count, hipStream_t stream);

// attention_ops.hip
hipError_t launch_softmax_s8(const int8_t *in, long long outer, long long len, long long inner, int in_exp, float *out,
                             int cu_count, hipStream_t stream);
hipError_t launch_quantize_f32(const float *in, long long size, int out_exp, int elem_size, void *out, int cu_count,
                               hipStream_t stream);
hipError_t launch_dequantize_f32(const void *in, long long size, int in_exp, int elem_size, float *out, int cu_count,
                                 hipStream_t stream);
hipError_t launch_lut_s16(const int16_t *in, long long size, const int16_t *table, int table_size, int shift, bool p4_ties,
                          int16_t *out, int cu_count, hipStream_t stream);
hipError_t launch_matmul_s8(const int8_t *a, const int8_t *b, int m, int k, int n, const int lead[2],
                            const long long a_stride[2], const long long b_stride[2], int shift, bool relu, bool half_even,
                            int8_t *out, hipStream_t stream);

} // namespace espdl
