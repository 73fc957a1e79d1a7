// extern "C" entry points of libespdl_hip.so (declared in include/espdl_hip.h): argument
// validation, geometry derivation and kernel dispatch.  No allocation, no synchronization.
#include "../../include/espdl_hip.h"

#include <climits>
#include <cstdarg>
#include <cstdio>

#include "espdl_kernels.h"
#include <vector>

namespace {
thread_local char g_last_error[256] = "";
}

// Records the message espdl_hip_last_error() returns on this thread and hands `code` back.
int espdl::set_error(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

#define fail(...) espdl::set_error(__VA_ARGS__)

namespace {

int device_status(hipError_t e, const char *what)
{
    if (e == hipSuccess)
        return ESPDL_HIP_OK;
    return fail(ESPDL_HIP_EDEVICE, "%s: %s", what, hipGetErrorString(e));
}

int cu_count_cached()
{
    static thread_local int cached_dev = -1;
    static thread_local int cached_cus = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError(); // a failed query must not surface as the error of a later launch
        return 0;
    }
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) {
            (void)hipGetLastError();
            return 0; // not remembered: the next call asks again
        }
        cached_dev = dev;
        cached_cus = cus;
    }
    return cached_cus;
}

// Conv::get_output_shape (esp-dl/dl/module/include/dl_module_conv.hpp:90-98)
int derive_geometry(const espdl_hip_conv_desc *d, espdl::ConvGeom *g)
{
    if (d == nullptr)
        return fail(ESPDL_HIP_EINVAL, "conv descriptor is NULL");
    if (d->dtype != ESPDL_HIP_S8 && d->dtype != ESPDL_HIP_S16)
        return fail(ESPDL_HIP_EINVAL, "dtype %d is neither ESPDL_HIP_S8 nor ESPDL_HIP_S16", d->dtype);
    if (d->batch < 0 || d->in_h <= 0 || d->in_w <= 0 || d->in_c <= 0 || d->out_c <= 0)
        return fail(ESPDL_HIP_EINVAL, "bad tensor extents: batch %d in %dx%dx%d out_c %d", d->batch, d->in_h, d->in_w,
                    d->in_c, d->out_c);
    if (d->k_h <= 0 || d->k_w <= 0 || d->stride_h <= 0 || d->stride_w <= 0 || d->dil_h <= 0 || d->dil_w <= 0)
        return fail(ESPDL_HIP_EINVAL, "filter size, stride and dilation must be positive");
    if (d->pad_top < 0 || d->pad_bottom < 0 || d->pad_left < 0 || d->pad_right < 0)
        return fail(ESPDL_HIP_EINVAL, "negative padding");
    if (d->group != 1 && !(d->group == d->in_c && d->out_c == d->in_c))
        return fail(ESPDL_HIP_ENOTSUP, "group %d: only 1 (dense) or in_c with out_c == in_c (depthwise) are supported",
                    d->group);
    if (d->activation != ESPDL_HIP_LINEAR && d->activation != ESPDL_HIP_RELU)
        return fail(ESPDL_HIP_ENOTSUP, "fused activation %d: only Linear and ReLU exist on this path", d->activation);
    if (d->round_mode != ESPDL_HIP_ROUND_HALF_UP && d->round_mode != ESPDL_HIP_ROUND_HALF_EVEN)
        return fail(ESPDL_HIP_EINVAL, "unknown round_mode %d", d->round_mode);
    if (d->n_shift != 1 && d->n_shift != d->out_c)
        return fail(ESPDL_HIP_EINVAL, "n_shift %d must be 1 or out_c (%d)", d->n_shift, d->out_c);
    const long long span_h = (long long)d->in_h + d->pad_top + d->pad_bottom - (long long)d->dil_h * (d->k_h - 1) - 1;
    const long long span_w = (long long)d->in_w + d->pad_left + d->pad_right - (long long)d->dil_w * (d->k_w - 1) - 1;
    if (span_h < 0 || span_w < 0)
        return fail(ESPDL_HIP_EINVAL, "filter window is larger than the padded input");
    const long long oh = span_h / d->stride_h + 1, ow = span_w / d->stride_w + 1;
    const long long k_total = (long long)d->k_h * d->k_w * d->in_c;
    const long long in_elems = (long long)d->batch * d->in_h * d->in_w * d->in_c;
    const long long out_elems = (long long)d->batch * oh * ow * d->out_c;
    if (k_total > (1 << 24) || in_elems > (1ll << 40) || out_elems > (1ll << 40) || oh > INT_MAX || ow > INT_MAX ||
        (long long)d->batch * oh * ow > INT_MAX - 65536 || oh * ow > INT_MAX / 2)
        return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    g->batch = d->batch;
    g->in_h = d->in_h;
    g->in_w = d->in_w;
    g->in_c = d->in_c;
    g->out_c = d->out_c;
    g->out_h = (int)oh;
    g->out_w = (int)ow;
    g->k_h = d->k_h;
    g->k_w = d->k_w;
    g->stride_h = d->stride_h;
    g->stride_w = d->stride_w;
    g->dil_h = d->dil_h;
    g->dil_w = d->dil_w;
    g->pad_top = d->pad_top;
    g->pad_left = d->pad_left;
    g->relu = d->activation == ESPDL_HIP_RELU;
    g->half_even = d->round_mode == ESPDL_HIP_ROUND_HALF_EVEN;
    g->n_shift = d->n_shift;
    if (d->in_pitch < 0 || d->out_pitch < 0 || d->res_pitch < 0 || (d->in_pitch != 0 && d->in_pitch < d->in_c) ||
        (d->out_pitch != 0 && d->out_pitch < d->out_c) || (d->res_pitch != 0 && d->res_pitch < d->out_c))
        return fail(ESPDL_HIP_EINVAL, "channel pitches %d / %d / %d must be 0 or at least the channel counts", d->in_pitch,
                    d->out_pitch, d->res_pitch);
    g->in_pitch = d->in_pitch != 0 ? d->in_pitch : d->in_c;
    g->out_pitch = d->out_pitch != 0 ? d->out_pitch : d->out_c;
    g->res_pitch = d->res_pitch != 0 ? d->res_pitch : d->out_c;
    if ((long long)d->batch * d->in_h * d->in_w * g->in_pitch > (1ll << 40) || (long long)d->batch * oh * ow * g->out_pitch > (1ll << 40))
        return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    return ESPDL_HIP_OK;
}

bool misaligned(const void *p, uintptr_t a)
{
    return (reinterpret_cast<uintptr_t>(p) & (a - 1)) != 0;
}

} // namespace

extern "C" {

const char *espdl_hip_last_error(void)
{
    return g_last_error;
}

const char *espdl_hip_version(void)
{
    return "espdl_hip 0.1 (gfx950)";
}

int espdl_hip_device_cu_count(void)
{
    return cu_count_cached();
}

int espdl_hip_conv_out_shape(const espdl_hip_conv_desc *desc, int32_t *out_h, int32_t *out_w)
{
    espdl::ConvGeom g;
    const int rc = derive_geometry(desc, &g);
    if (rc != ESPDL_HIP_OK)
        return rc;
    if (out_h)
        *out_h = g.out_h;
    if (out_w)
        *out_w = g.out_w;
    return ESPDL_HIP_OK;
}

int espdl_hip_conv2d(const espdl_hip_conv_desc *desc, const void *in, const void *filter, const void *bias,
                     const int32_t *shift, const int8_t *lut, void *out, void *stream)
{
    return espdl_hip_conv2d_add(desc, in, filter, bias, shift, lut, nullptr, out, stream);
}

int espdl_hip_conv2d_add(const espdl_hip_conv_desc *desc, const void *in, const void *filter, const void *bias,
                         const int32_t *shift, const int8_t *lut, const int8_t *residual, void *out, void *stream)
{
    espdl::ConvGeom g;
    const int rc = derive_geometry(desc, &g);
    if (rc != ESPDL_HIP_OK)
        return rc;
    if (g.batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || filter == nullptr || shift == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in, filter, shift and out must not be NULL");
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    const bool depthwise = desc->group != 1;
    if (!espdl::conv_is_dense(g) && (depthwise || desc->dtype != ESPDL_HIP_S8))
        return fail(ESPDL_HIP_ENOTSUP, "channel pitches exist for dense int8 convolutions (group 1) only");
    if (desc->dtype == ESPDL_HIP_S8) {
        if (misaligned(bias, 4) || misaligned(shift, 4))
            return fail(ESPDL_HIP_EINVAL, "bias and shift must be 4-byte aligned");
        const int8_t *i8 = static_cast<const int8_t *>(in);
        const int8_t *f8 = static_cast<const int8_t *>(filter);
        const int32_t *b32 = static_cast<const int32_t *>(bias);
        int8_t *o8 = static_cast<int8_t *>(out);
        if (residual != nullptr && depthwise)
            return fail(ESPDL_HIP_ENOTSUP, "the fused residual Add exists for dense int8 convolutions only");
        if (depthwise) {
            if (espdl::depthwise_s8_lds_supports(g, in, out))
                return device_status(espdl::launch_depthwise_s8_lds(g, i8, f8, b32, shift, lut, o8, cu_count_cached(), s),
                                     "depthwise_s8_lds");
            if (espdl::depthwise_s8_mfma_supports(g, in, out))
                return device_status(espdl::launch_depthwise_s8_mfma(g, i8, f8, b32, shift, lut, o8, cu_count_cached(), s),
                                     "depthwise_s8_mfma");
            return device_status(espdl::launch_depthwise_s8(g, i8, f8, b32, shift, lut, o8, s), "depthwise_s8");
        }
        if (espdl::conv2d_s8_stem_supports(g, residual))
            return device_status(espdl::launch_conv2d_s8_stem(g, i8, f8, b32, shift, lut, o8, cu_count_cached(), s),
                                 "conv2d_s8_stem");
        // (the second test admits products with fewer than 32 filters, which only the few-rows kernel inside takes)
        if (espdl::conv2d_s8_pwgemm_supports(g, in, filter, cu_count_cached()) ||
            (lut == nullptr && residual == nullptr && espdl::conv2d_s8_rows_supports(g, in, filter, cu_count_cached())))
            return device_status(espdl::launch_conv2d_s8_pwgemm(g, i8, f8, b32, shift, lut, residual, o8, cu_count_cached(), s),
                                 "conv2d_s8_pwgemm");
        // Windows over 64 channels or more on few pixels: the pointwise GEMM kernel over gathered rows.  Strided
        // windows (80 x 80 x 128 -> 128 at stride 2, batch 64: 91 -> 41 us); at stride 1 up to 128 K output pixels
        // (40 x 40 x 128 -> 64, batch 64: 26 -> 22 us; 20 x 20 x 256 -> 256: 93 -> 38 us) or with a reduction axis of
        // 2048 or more, whose filters the LDS-tiled kernel below cannot keep resident (80 x 80 x 256 -> 256: 732 ->
        // 472 us); with more pixels and fewer channels that kernel is faster (80 x 80 x 64 -> 64: 30 against 41 us).
        const bool few_pixels = (long long)g.batch * g.out_h * g.out_w <= 128 * 1024;
        if ((g.stride_h != 1 || g.stride_w != 1 || few_pixels || g.k_h * g.k_w * g.in_c >= 2048) &&
            espdl::conv2d_s8_wingemm_supports(g, in, filter, cu_count_cached()))
            return device_status(espdl::launch_conv2d_s8_wingemm(g, i8, f8, b32, shift, lut, residual, o8, cu_count_cached(), s),
                                 "conv2d_s8_wingemm");
        if (espdl::conv2d_s8_tiled_supports(g, in, filter, cu_count_cached()))
            return device_status(espdl::launch_conv2d_s8_tiled(g, i8, f8, b32, shift, lut, residual, o8, cu_count_cached(), s),
                                 "conv2d_s8_tiled");
        return device_status(espdl::launch_conv2d_s8_mfma(g, i8, f8, b32, shift, lut, residual, o8, cu_count_cached(), s),
                             "conv2d_s8");
    }
    if (lut != nullptr || residual != nullptr)
        return fail(ESPDL_HIP_ENOTSUP, "the fused LUT / residual epilogues exist for ESPDL_HIP_S8 only");
    if (misaligned(in, 2) || misaligned(filter, 2) || misaligned(out, 2) || misaligned(bias, 8) || misaligned(shift, 4))
        return fail(ESPDL_HIP_EINVAL, "int16 tensors must be 2-byte aligned, int64 bias 8-byte aligned");
    const int16_t *i16 = static_cast<const int16_t *>(in);
    const int16_t *f16 = static_cast<const int16_t *>(filter);
    const int64_t *b64 = static_cast<const int64_t *>(bias);
    int16_t *o16 = static_cast<int16_t *>(out);
    if (depthwise)
        return device_status(espdl::launch_depthwise_s16(g, i16, f16, b64, shift, o16, s), "depthwise_s16");
    if (espdl::conv2d_s16_mfma_supports(g, i16, f16, o16))
        return device_status(espdl::launch_conv2d_s16_mfma(g, i16, f16, b64, shift, o16, cu_count_cached(), s),
                             "conv2d_s16_mfma");
    return device_status(espdl::launch_conv2d_s16(g, i16, f16, b64, shift, o16, s), "conv2d_s16");
}

static int check_exps(int32_t in_exp, int32_t out_exp);

int espdl_hip_conv2d_gap_s8_supported(const espdl_hip_conv_desc *desc)
{
    espdl::ConvGeom g;
    if (desc == nullptr || desc->dtype != ESPDL_HIP_S8 || desc->group != 1 || derive_geometry(desc, &g) != ESPDL_HIP_OK)
        return 0;
    static const int8_t *const aligned = reinterpret_cast<const int8_t *>(uintptr_t(256));
    return espdl::conv2d_gap_s8_supports(g, aligned, aligned) ? 1 : 0;
}

int espdl_hip_conv2d_gap_s8(const espdl_hip_conv_desc *desc, const int8_t *in, const int8_t *filter, const int32_t *bias,
                            const int32_t *shift, int32_t conv_out_exp, int32_t pool_out_exp, int8_t *out, void *stream)
{
    espdl::ConvGeom g;
    const int rc = derive_geometry(desc, &g);
    if (rc != ESPDL_HIP_OK)
        return rc;
    if (desc->dtype != ESPDL_HIP_S8 || desc->group != 1)
        return fail(ESPDL_HIP_ENOTSUP, "the pooled form exists for dense int8 convolutions only");
    if (check_exps(conv_out_exp, pool_out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (g.batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || filter == nullptr || shift == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in, filter, shift and out must not be NULL");
    if (misaligned(bias, 4) || misaligned(shift, 4))
        return fail(ESPDL_HIP_EINVAL, "bias and shift must be 4-byte aligned");
    if (!espdl::conv2d_gap_s8_supports(g, in, filter))
        return fail(ESPDL_HIP_ENOTSUP, "the pooled form takes 1x1 stride-1 convolutions over images of at most 64 pixels, "
                                       "input channels a multiple of 16 (at least 64), 16-byte aligned input and filter");
    const float scale = espdl::global_avg_pool_scale(g.out_h, g.out_w, conv_out_exp, pool_out_exp);
    return device_status(espdl::launch_conv2d_gap_s8(g, in, filter, bias, shift, scale, out, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         "conv2d_gap_s8");
}

int espdl_hip_lut_s8(const int8_t *in, int64_t size, const int8_t *table, int8_t *out, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || table == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in, table and out must not be NULL");
    return device_status(espdl::launch_lut_s8(in, size, table, out, reinterpret_cast<hipStream_t>(stream)), "lut_s8");
}

int espdl_hip_prelu_s8(const int8_t *in, int64_t pixels, int32_t channels, const int8_t *alpha, int32_t shift,
                       int8_t *out, void *stream)
{
    if (pixels < 0 || channels <= 0)
        return fail(ESPDL_HIP_EINVAL, "bad extents: pixels %lld channels %d", (long long)pixels, channels);
    if (pixels == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || alpha == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in, alpha and out must not be NULL");
    if (shift < -15 || shift > 31)
        return fail(ESPDL_HIP_EINVAL, "prelu shift %d outside [-15, 31]", shift);
    return device_status(
        espdl::launch_prelu_s8(in, pixels, channels, alpha, shift, out, reinterpret_cast<hipStream_t>(stream)),
        "prelu_s8");
}

static int check_exps(int32_t in_exp, int32_t out_exp)
{
    if (in_exp < -30 || in_exp > 30 || out_exp < -30 || out_exp > 30)
        return fail(ESPDL_HIP_EINVAL, "exponents %d / %d outside [-30, 30]", in_exp, out_exp);
    return ESPDL_HIP_OK;
}

int espdl_hip_relu_s8(const int8_t *in, int64_t size, int32_t in_exp, int32_t out_exp, int8_t *out, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_relu_s8(in, size, in_exp, out_exp, out, reinterpret_cast<hipStream_t>(stream)),
                         "relu_s8");
}

int espdl_hip_clip_s8(const int8_t *in, int64_t size, int32_t min_q, int32_t max_q, int32_t in_exp, int32_t out_exp,
                      int8_t *out, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (min_q < -128 || max_q > 127)
        return fail(ESPDL_HIP_EINVAL, "clip bounds [%d, %d] are not int8 values", min_q, max_q);
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(
        espdl::launch_clip_s8(in, size, min_q, max_q, in_exp, out_exp, out, reinterpret_cast<hipStream_t>(stream)),
        "clip_s8");
}

int espdl_hip_add_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int8_t *out, void *stream)
{
    if (out_dims == nullptr || in0_strides == nullptr || in1_strides == nullptr)
        return fail(ESPDL_HIP_EINVAL, "dims and strides must not be NULL");
    long long size = 1;
    for (int i = 0; i < 4; i++) {
        if (out_dims[i] < 0 || in0_strides[i] < 0 || in1_strides[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent or stride in dim %d", i);
        size *= out_dims[i];
        if (size > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in0 == nullptr || in1 == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in0, in1 and out must not be NULL");
    return device_status(
        espdl::launch_add_s8(out_dims, in0_strides, in1_strides, in0, in1, out, reinterpret_cast<hipStream_t>(stream)),
        "add_s8");
}

int espdl_hip_mul_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int32_t mul_shift, int32_t round_mode, int8_t *out,
                     void *stream)
{
    if (out_dims == nullptr || in0_strides == nullptr || in1_strides == nullptr)
        return fail(ESPDL_HIP_EINVAL, "dims and strides must not be NULL");
    if (mul_shift < -60 || mul_shift > 60)
        return fail(ESPDL_HIP_EINVAL, "mul_shift %d outside [-60, 60]", mul_shift);
    if (round_mode != ESPDL_HIP_ROUND_HALF_UP && round_mode != ESPDL_HIP_ROUND_HALF_EVEN)
        return fail(ESPDL_HIP_EINVAL, "bad round_mode %d", round_mode);
    long long size = 1;
    for (int i = 0; i < 4; i++) {
        if (out_dims[i] < 0 || in0_strides[i] < 0 || in1_strides[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent or stride in dim %d", i);
        size *= out_dims[i];
        if (size > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in0 == nullptr || in1 == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in0, in1 and out must not be NULL");
    return device_status(espdl::launch_mul_s8(out_dims, in0_strides, in1_strides, in0, in1, mul_shift,
                                              round_mode == ESPDL_HIP_ROUND_HALF_EVEN, out,
                                              reinterpret_cast<hipStream_t>(stream)),
                         "mul_s8");
}

int espdl_hip_global_avg_pool_s8(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t in_exp,
                                 int32_t out_exp, int8_t *out, void *stream)
{
    if (batch < 0 || h <= 0 || w <= 0 || c <= 0 || (long long)h * w > (1 << 23) || batch > 65535)
        return fail(ESPDL_HIP_EINVAL, "bad extents: batch %d, %dx%dx%d", batch, h, w, c);
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_global_avg_pool_s8(in, batch, h, w, c, in_exp, out_exp, out,
                                                          reinterpret_cast<hipStream_t>(stream)),
                         "global_avg_pool_s8");
}

int espdl_hip_requantize_s8(const int8_t *in, int64_t size, int32_t in_exp, int32_t out_exp, int8_t *out,
                            void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(
        espdl::launch_requantize_s8(in, size, in_exp, out_exp, out, reinterpret_cast<hipStream_t>(stream)),
        "requantize_s8");
}

int espdl_hip_requantize_s8_rows(const int8_t *in, int64_t in_pitch, int8_t *out, int64_t out_pitch, int64_t row_bytes,
                                 int64_t rows, int32_t in_exp, int32_t out_exp, void *stream)
{
    if (rows < 0 || row_bytes < 0 || in_pitch < row_bytes || out_pitch < row_bytes)
        return fail(ESPDL_HIP_EINVAL, "rows of %lld bytes need pitches of at least that (got %lld / %lld) and a count >= 0",
                    (long long)row_bytes, (long long)in_pitch, (long long)out_pitch);
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (rows == 0 || row_bytes == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    if (in_exp == out_exp)
        return espdl_hip_copy_rows(in, in_pitch, out, out_pitch, row_bytes, rows, stream);
    return device_status(espdl::launch_requantize_s8_rows(in, in_pitch, out, out_pitch, row_bytes, rows, in_exp, out_exp,
                                                          reinterpret_cast<hipStream_t>(stream)),
                         "requantize_s8_rows");
}

int espdl_hip_requantize(const void *in, int32_t in_dtype, int64_t size, int32_t in_exp, int32_t out_exp, void *out,
                         int32_t out_dtype, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if ((in_dtype != ESPDL_HIP_S8 && in_dtype != ESPDL_HIP_S16) || (out_dtype != ESPDL_HIP_S8 && out_dtype != ESPDL_HIP_S16))
        return fail(ESPDL_HIP_EINVAL, "dtypes must be ESPDL_HIP_S8 or ESPDL_HIP_S16");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    if ((in_dtype == ESPDL_HIP_S16 && misaligned(in, 2)) || (out_dtype == ESPDL_HIP_S16 && misaligned(out, 2)))
        return fail(ESPDL_HIP_EINVAL, "int16 tensors must be 2-byte aligned");
    if (in_dtype == ESPDL_HIP_S8 && out_dtype == ESPDL_HIP_S8)
        return espdl_hip_requantize_s8(static_cast<const int8_t *>(in), size, in_exp, out_exp,
                                       static_cast<int8_t *>(out), stream);
    return device_status(espdl::launch_requantize_any(in, in_dtype, size, in_exp, out_exp, out, out_dtype,
                                                      reinterpret_cast<hipStream_t>(stream)),
                         "requantize");
}

int espdl_hip_concat(int32_t n_inputs, const void *const *inputs, const int64_t *copy_bytes, int64_t loop_times,
                     void *out, void *stream)
{
    if (n_inputs < 0 || loop_times < 0 || (n_inputs > 0 && (inputs == nullptr || copy_bytes == nullptr)))
        return fail(ESPDL_HIP_EINVAL, "bad concat arguments");
    std::vector<long long> bytes((size_t)n_inputs);
    long long total = 0;
    for (int j = 0; j < n_inputs; j++) {
        if (copy_bytes[j] < 0 || (copy_bytes[j] > 0 && inputs[j] == nullptr))
            return fail(ESPDL_HIP_EINVAL, "concat input %d: null pointer or negative size", j);
        bytes[(size_t)j] = copy_bytes[j];
        total += copy_bytes[j];
    }
    if (total == 0 || loop_times == 0)
        return ESPDL_HIP_OK;
    if (out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "out must not be NULL");
    return device_status(espdl::launch_concat(n_inputs, inputs, bytes.data(), loop_times, out, cu_count_cached(),
                                              reinterpret_cast<hipStream_t>(stream)),
                         "concat");
}

int espdl_hip_copy_rows(const void *src, int64_t src_pitch, void *dst, int64_t dst_pitch, int64_t row_bytes,
                        int64_t rows, void *stream)
{
    if (rows < 0 || row_bytes < 0 || src_pitch < 0 || dst_pitch < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size or pitch");
    if (rows == 0 || row_bytes == 0)
        return ESPDL_HIP_OK;
    if (src == nullptr || dst == nullptr)
        return fail(ESPDL_HIP_EINVAL, "src and dst must not be NULL");
    if (rows > 1 && (src_pitch < row_bytes || dst_pitch < row_bytes))
        return fail(ESPDL_HIP_EINVAL, "pitches must be at least row_bytes");
    return device_status(espdl::launch_copy_rows(src, src_pitch, dst, dst_pitch, row_bytes, rows, cu_count_cached(),
                                                 reinterpret_cast<hipStream_t>(stream)),
                         "copy_rows");
}

int espdl_hip_split(const void *in, int64_t in_pitch, int32_t n_outputs, void *const *outputs, const int64_t *copy_bytes,
                    int64_t rows, void *stream)
{
    if (n_outputs < 1 || outputs == nullptr || copy_bytes == nullptr || rows < 0 || in_pitch < 0)
        return fail(ESPDL_HIP_EINVAL, "split needs at least one output, sizes and a row count >= 0");
    long long total = 0;
    std::vector<long long> bytes((size_t)n_outputs);
    for (int j = 0; j < n_outputs; j++) {
        if (copy_bytes[j] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative size of output %d", j);
        bytes[(size_t)j] = copy_bytes[j];
        total += copy_bytes[j];
    }
    if (rows == 0 || total == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in must not be NULL");
    if (rows > 1 && in_pitch < total)
        return fail(ESPDL_HIP_EINVAL, "the input pitch %lld is smaller than the pieces together (%lld)", (long long)in_pitch,
                    total);
    return device_status(espdl::launch_split(in, in_pitch, n_outputs, outputs, bytes.data(), rows, cu_count_cached(),
                                             reinterpret_cast<hipStream_t>(stream)),
                         "split");
}

int espdl_hip_transpose(const void *in, const int32_t *shape, int32_t dims, const int32_t *perm, int32_t n_perm,
                        int32_t elem_size, void *out, void *stream)
{
    if (dims < 1 || dims > 8 || shape == nullptr)
        return fail(ESPDL_HIP_EINVAL, "transpose handles 1..8 dims");
    if (elem_size != 1 && elem_size != 2 && elem_size != 4)
        return fail(ESPDL_HIP_EINVAL, "elem_size must be 1, 2 or 4");
    if (n_perm != 0 && (n_perm != dims || perm == nullptr))
        return fail(ESPDL_HIP_EINVAL, "perm must have one entry per dim (or none)");
    int p[8], sh[8];
    bool seen[8] = {false, false, false, false, false, false, false, false};
    long long total = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent");
        sh[i] = shape[i];
        total *= shape[i];
        int v = n_perm == 0 ? dims - 1 - i : perm[i];
        if (v < 0)
            v += dims;
        if (v < 0 || v >= dims || seen[v])
            return fail(ESPDL_HIP_EINVAL, "perm is not a permutation of the dims");
        seen[v] = true;
        p[i] = v;
    }
    if (total == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    if (misaligned(in, (size_t)elem_size) || misaligned(out, (size_t)elem_size))
        return fail(ESPDL_HIP_EINVAL, "tensors must be aligned to the element size");
    return device_status(espdl::launch_transpose(in, sh, dims, p, elem_size, out, cu_count_cached(),
                                                 reinterpret_cast<hipStream_t>(stream)),
                         "transpose");
}

int espdl_hip_resize_nearest_s8_pitched(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t out_h,
                                        int32_t out_w, float scale_h, float scale_w, int32_t in_exp, int32_t out_exp,
                                        int32_t in_pitch, int32_t out_pitch, int8_t *out, void *stream)
{
    if (batch < 0 || h <= 0 || w <= 0 || c <= 0 || out_h < 0 || out_w < 0 || !(scale_h > 0) || !(scale_w > 0))
        return fail(ESPDL_HIP_EINVAL, "bad resize geometry");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (out_exp - in_exp > 30 || in_exp - out_exp > 30)
        return fail(ESPDL_HIP_EINVAL, "exponent difference out of range");
    if (in_pitch < 0 || out_pitch < 0 || (in_pitch != 0 && in_pitch < c) || (out_pitch != 0 && out_pitch < c))
        return fail(ESPDL_HIP_EINVAL, "channel pitches %d / %d must be 0 or at least the channel count %d", in_pitch, out_pitch,
                    c);
    if ((long long)batch * out_h * out_w == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_resize_nearest_s8(in, batch, h, w, c, out_h, out_w, scale_h, scale_w, in_exp,
                                                         out_exp, in_pitch != 0 ? in_pitch : c, out_pitch != 0 ? out_pitch : c,
                                                         out, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         "resize_nearest_s8");
}

int espdl_hip_resize_nearest_s8(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t out_h,
                                int32_t out_w, float scale_h, float scale_w, int32_t in_exp, int32_t out_exp,
                                int8_t *out, void *stream)
{
    return espdl_hip_resize_nearest_s8_pitched(in, batch, h, w, c, out_h, out_w, scale_h, scale_w, in_exp, out_exp, 0, 0, out,
                                               stream);
}

int espdl_hip_max_pool_pitched(const void *in, int32_t dtype, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h,
                               int32_t k_w, int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom,
                               int32_t pad_left, int32_t pad_right, int32_t in_pitch, int32_t out_pitch, void *out,
                               void *stream)
{
    if (dtype != ESPDL_HIP_S8 && dtype != ESPDL_HIP_S16)
        return fail(ESPDL_HIP_EINVAL, "dtype must be ESPDL_HIP_S8 or ESPDL_HIP_S16");
    if (batch < 0 || h <= 0 || w <= 0 || c <= 0 || k_h <= 0 || k_w <= 0 || stride_h <= 0 || stride_w <= 0 || pad_top < 0 ||
        pad_bottom < 0 || pad_left < 0 || pad_right < 0)
        return fail(ESPDL_HIP_EINVAL, "bad max_pool geometry");
    if (h + pad_top + pad_bottom < k_h || w + pad_left + pad_right < k_w)
        return fail(ESPDL_HIP_EINVAL, "window larger than the padded image");
    if (in_pitch < 0 || out_pitch < 0 || (in_pitch != 0 && in_pitch < c) || (out_pitch != 0 && out_pitch < c))
        return fail(ESPDL_HIP_EINVAL, "channel pitches %d / %d must be 0 or at least the channel count %d", in_pitch, out_pitch,
                    c);
    const int out_h = (h + pad_top + pad_bottom - k_h) / stride_h + 1, out_w = (w + pad_left + pad_right - k_w) / stride_w + 1;
    if (batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    const int esize = dtype == ESPDL_HIP_S8 ? 1 : 2;
    if (misaligned(in, (size_t)esize) || misaligned(out, (size_t)esize))
        return fail(ESPDL_HIP_EINVAL, "int16 tensors must be 2-byte aligned");
    return device_status(espdl::launch_max_pool(in, esize, batch, h, w, c, k_h, k_w, stride_h, stride_w, pad_top, pad_left,
                                                out_h, out_w, in_pitch != 0 ? in_pitch : c, out_pitch != 0 ? out_pitch : c,
                                                out, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         "max_pool");
}

int espdl_hip_max_pool(const void *in, int32_t dtype, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h,
                       int32_t k_w, int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom,
                       int32_t pad_left, int32_t pad_right, void *out, void *stream)
{
    return espdl_hip_max_pool_pitched(in, dtype, batch, h, w, c, k_h, k_w, stride_h, stride_w, pad_top, pad_bottom, pad_left,
                                      pad_right, 0, 0, out, stream);
}

int espdl_hip_avg_pool_s8(const int8_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h, int32_t k_w,
                          int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom, int32_t pad_left,
                          int32_t pad_right, int32_t in_exp, int32_t out_exp, int8_t *out, void *stream)
{
    if (batch < 0 || h <= 0 || w <= 0 || c <= 0 || k_h <= 0 || k_w <= 0 || stride_h <= 0 || stride_w <= 0 || pad_top < 0 ||
        pad_bottom < 0 || pad_left < 0 || pad_right < 0 || (long long)k_h * k_w > (1 << 23))
        return fail(ESPDL_HIP_EINVAL, "bad avg_pool geometry");
    if (h + pad_top + pad_bottom < k_h || w + pad_left + pad_right < k_w)
        return fail(ESPDL_HIP_EINVAL, "window larger than the padded image");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    const int out_h = (h + pad_top + pad_bottom - k_h) / stride_h + 1, out_w = (w + pad_left + pad_right - k_w) / stride_w + 1;
    if (batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_avg_pool_s8(in, batch, h, w, c, k_h, k_w, stride_h, stride_w, pad_top, pad_left,
                                                   out_h, out_w, in_exp, out_exp, out, cu_count_cached(),
                                                   reinterpret_cast<hipStream_t>(stream)),
                         "avg_pool_s8");
}

int espdl_hip_slice(const void *in, const int32_t *shape, int32_t dims, const int32_t *start, const int32_t *step,
                    const int32_t *out_shape, int32_t elem_size, void *out, void *stream)
{
    if (dims < 1 || dims > 8 || shape == nullptr || start == nullptr || step == nullptr || out_shape == nullptr)
        return fail(ESPDL_HIP_EINVAL, "slice handles 1..8 dims");
    if (elem_size != 1 && elem_size != 2 && elem_size != 4)
        return fail(ESPDL_HIP_EINVAL, "elem_size must be 1, 2 or 4");
    int sh[8], st[8], sp[8], os[8];
    long long total = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0 || out_shape[i] < 0 || step[i] < 1 || start[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "dim %d: negative extent or start, or step below 1", i);
        if (out_shape[i] > 0 && (long long)start[i] + (long long)(out_shape[i] - 1) * step[i] >= shape[i])
            return fail(ESPDL_HIP_EINVAL, "dim %d: the slice leaves the tensor", i);
        sh[i] = shape[i];
        st[i] = start[i];
        sp[i] = step[i];
        os[i] = out_shape[i];
        total *= out_shape[i];
    }
    if (total == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    if (misaligned(in, (size_t)elem_size) || misaligned(out, (size_t)elem_size))
        return fail(ESPDL_HIP_EINVAL, "tensors must be aligned to the element size");
    return device_status(espdl::launch_slice(in, sh, dims, st, sp, os, elem_size, out, cu_count_cached(),
                                             reinterpret_cast<hipStream_t>(stream)),
                         "slice");
}

int espdl_hip_reduce_int(const void *in, int32_t dtype, const int32_t *shape, int32_t dims, const int32_t *reduce_flag,
                         int32_t op, int32_t shift, int32_t round_mode, void *out, void *stream)
{
    if (dtype != ESPDL_HIP_S8 && dtype != ESPDL_HIP_S16)
        return fail(ESPDL_HIP_EINVAL, "dtype must be ESPDL_HIP_S8 or ESPDL_HIP_S16");
    if (dims < 1 || dims > 8 || shape == nullptr || reduce_flag == nullptr)
        return fail(ESPDL_HIP_EINVAL, "reduce handles 1..8 dims");
    if (op < ESPDL_HIP_REDUCE_MAX || op > ESPDL_HIP_REDUCE_SUM_SQUARE)
        return fail(ESPDL_HIP_EINVAL, "unknown reduce op %d", op);
    if (round_mode != ESPDL_HIP_ROUND_HALF_UP && round_mode != ESPDL_HIP_ROUND_HALF_EVEN)
        return fail(ESPDL_HIP_EINVAL, "bad round_mode %d", round_mode);
    if (shift < -30 || shift > 62)
        return fail(ESPDL_HIP_EINVAL, "shift %d outside [-30, 62]", shift);
    int sh[8], fl[8];
    long long n_out = 1, count = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent in dim %d", i);
        sh[i] = shape[i];
        fl[i] = reduce_flag[i] ? 1 : 0;
        if (fl[i])
            count *= shape[i];
        else
            n_out *= shape[i];
        if (n_out > (1ll << 40) || count > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (n_out == 0)
        return ESPDL_HIP_OK;
    if (dtype == ESPDL_HIP_S8 && op >= ESPDL_HIP_REDUCE_SUM &&
        count > (op == ESPDL_HIP_REDUCE_SUM_SQUARE ? (1ll << 17) - 1 : (1ll << 24) - 1))
        return fail(ESPDL_HIP_ENOTSUP, "this int8 sum can leave the reference's int32 accumulator");
    if (out == nullptr || (in == nullptr && count > 0))
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    if (dtype == ESPDL_HIP_S16 && (misaligned(in, 2) || misaligned(out, 2)))
        return fail(ESPDL_HIP_EINVAL, "int16 tensors must be 2-byte aligned");
    return device_status(espdl::launch_reduce_int(in, dtype == ESPDL_HIP_S8 ? 8 : 16, sh, dims, fl, op, shift,
                                                  round_mode == ESPDL_HIP_ROUND_HALF_EVEN, out, cu_count_cached(),
                                                  reinterpret_cast<hipStream_t>(stream)),
                         "reduce_int");
}

int espdl_hip_pad(const void *in, const int32_t *shape, int32_t dims, const int32_t *pads, int32_t mode,
                  int32_t constant_value, int32_t elem_size, void *out, void *stream)
{
    if (dims < 1 || dims > 8 || shape == nullptr || pads == nullptr)
        return fail(ESPDL_HIP_EINVAL, "pad handles 1..8 dims");
    if (elem_size != 1 && elem_size != 2 && elem_size != 4)
        return fail(ESPDL_HIP_EINVAL, "elem_size must be 1, 2 or 4");
    if (mode != ESPDL_HIP_PAD_CONSTANT && mode != ESPDL_HIP_PAD_EDGE && mode != ESPDL_HIP_PAD_REFLECT)
        return fail(ESPDL_HIP_EINVAL, "unknown pad mode %d", mode);
    int sh[8], pd[16];
    long long total = 1, in_total = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0 || pads[i] < 0 || pads[i + dims] < 0)
            return fail(ESPDL_HIP_EINVAL, "dim %d: negative extent or pad", i);
        if (mode == ESPDL_HIP_PAD_REFLECT && (pads[i] > shape[i] - 1 || pads[i + dims] > shape[i] - 1) &&
            (pads[i] || pads[i + dims]))
            return fail(ESPDL_HIP_EINVAL, "dim %d: a reflected pad must be shorter than the axis", i);
        if (mode == ESPDL_HIP_PAD_EDGE && shape[i] == 0 && (pads[i] || pads[i + dims]))
            return fail(ESPDL_HIP_EINVAL, "dim %d: no edge to repeat on an empty axis", i);
        sh[i] = shape[i];
        pd[i] = pads[i];
        pd[i + dims] = pads[i + dims];
        in_total *= shape[i];
        total *= (long long)shape[i] + pads[i] + pads[i + dims];
        if (total > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (total == 0)
        return ESPDL_HIP_OK;
    if (out == nullptr || (in == nullptr && in_total > 0))
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    if (in_total == 0 && mode != ESPDL_HIP_PAD_CONSTANT)
        return fail(ESPDL_HIP_EINVAL, "only a constant pad can fill from an empty tensor");
    if (misaligned(in, (size_t)elem_size) || misaligned(out, (size_t)elem_size))
        return fail(ESPDL_HIP_EINVAL, "tensors must be aligned to the element size");
    return device_status(espdl::launch_pad(in, sh, dims, pd, mode, constant_value, elem_size, out, cu_count_cached(),
                                           reinterpret_cast<hipStream_t>(stream)),
                         "pad");
}

int espdl_hip_reduce_mean_s8(const int8_t *in, const int32_t *shape, int32_t dims, const int32_t *reduce_flag,
                             int32_t in_exp, int32_t out_exp, int8_t *out, void *stream)
{
    if (dims < 1 || dims > 8 || shape == nullptr || reduce_flag == nullptr)
        return fail(ESPDL_HIP_EINVAL, "reduce_mean handles 1..8 dims");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    int sh[8], fl[8];
    long long total = 1, count = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent");
        sh[i] = shape[i];
        fl[i] = reduce_flag[i] != 0;
        total *= shape[i];
        if (fl[i])
            count *= shape[i];
        if (total > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (total == 0)
        return ESPDL_HIP_OK;
    if (count > (1 << 23))
        return fail(ESPDL_HIP_ENOTSUP, "more than 2^23 elements per mean: the int32 sum could overflow");
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_reduce_mean_s8(in, sh, dims, fl, in_exp, out_exp, out, cu_count_cached(),
                                                      reinterpret_cast<hipStream_t>(stream)),
                         "reduce_mean_s8");
}

} // extern "C"

namespace {

// Fills the geometry part of MbconvParams; pointers are set by the caller.
int mbconv_geometry(const espdl_hip_mbconv_desc *d, espdl::MbconvParams *p)
{
    if (d == nullptr)
        return fail(ESPDL_HIP_EINVAL, "null descriptor");
    if (d->batch < 0 || d->in_h <= 0 || d->in_w <= 0 || d->in_c <= 0 || d->exp_c <= 0 || d->out_c <= 0 || d->k_h <= 0 ||
        d->k_w <= 0 || d->stride_h <= 0 || d->stride_w <= 0 || d->dil_h <= 0 || d->dil_w <= 0 || d->pad_top < 0 ||
        d->pad_bottom < 0 || d->pad_left < 0 || d->pad_right < 0)
        return fail(ESPDL_HIP_EINVAL, "bad mbconv geometry");
    if (!d->has_expand && d->exp_c != d->in_c)
        return fail(ESPDL_HIP_EINVAL, "without an expand stage exp_c must equal in_c");
    // expand stage with a window: the depthwise stage reads that convolution's output
    const bool windowed = d->exp_k_h != 0 || d->exp_k_w != 0 || d->exp_stride_h != 0 || d->exp_stride_w != 0 ||
        d->exp_pad_top != 0 || d->exp_pad_bottom != 0 || d->exp_pad_left != 0 || d->exp_pad_right != 0;
    int mid_h = d->in_h, mid_w = d->in_w;
    if (windowed) {
        if (!d->has_expand)
            return fail(ESPDL_HIP_EINVAL, "exp_k_* / exp_stride_* / exp_pad_* describe the expand stage: has_expand must be set");
        if (d->exp_k_h <= 0 || d->exp_k_w <= 0 || d->exp_stride_h <= 0 || d->exp_stride_w <= 0 || d->exp_pad_top < 0 ||
            d->exp_pad_bottom < 0 || d->exp_pad_left < 0 || d->exp_pad_right < 0)
            return fail(ESPDL_HIP_EINVAL, "bad expand-stage geometry");
        const int eh = d->in_h + d->exp_pad_top + d->exp_pad_bottom - d->exp_k_h;
        const int ew = d->in_w + d->exp_pad_left + d->exp_pad_right - d->exp_k_w;
        if (eh < 0 || ew < 0)
            return fail(ESPDL_HIP_EINVAL, "expand filter larger than the padded input");
        mid_h = eh / d->exp_stride_h + 1;
        mid_w = ew / d->exp_stride_w + 1;
    }
    const int eff_h = (d->k_h - 1) * d->dil_h + 1, eff_w = (d->k_w - 1) * d->dil_w + 1;
    const int span_h = mid_h + d->pad_top + d->pad_bottom - eff_h, span_w = mid_w + d->pad_left + d->pad_right - eff_w;
    if (span_h < 0 || span_w < 0)
        return fail(ESPDL_HIP_EINVAL, "depthwise filter larger than the padded input");
    if ((d->has_expand && d->n_shift_expand != 1 && d->n_shift_expand != d->exp_c) ||
        (d->n_shift_dw != 1 && d->n_shift_dw != d->exp_c) || (d->n_shift_project != 1 && d->n_shift_project != d->out_c))
        return fail(ESPDL_HIP_EINVAL, "n_shift_* must be 1 or the channel count of the stage");
    p->batch = d->batch;
    p->in_h = mid_h;
    p->in_w = mid_w;
    p->img_h = d->in_h;
    p->img_w = d->in_w;
    p->ek_h = windowed ? d->exp_k_h : 1;
    p->ek_w = windowed ? d->exp_k_w : 1;
    p->es_h = windowed ? d->exp_stride_h : 1;
    p->es_w = windowed ? d->exp_stride_w : 1;
    p->epad_top = d->exp_pad_top;
    p->epad_left = d->exp_pad_left;
    p->in_c = d->in_c;
    p->exp_c = d->exp_c;
    p->out_c = d->out_c;
    p->out_h = span_h / d->stride_h + 1;
    p->out_w = span_w / d->stride_w + 1;
    p->k_h = d->k_h;
    p->k_w = d->k_w;
    p->stride_h = d->stride_h;
    p->stride_w = d->stride_w;
    p->dil_h = d->dil_h;
    p->dil_w = d->dil_w;
    p->pad_top = d->pad_top;
    p->pad_left = d->pad_left;
    p->relu_expand = d->act_expand == ESPDL_HIP_RELU;
    p->relu_dw = d->act_dw == ESPDL_HIP_RELU;
    p->relu_project = d->act_project == ESPDL_HIP_RELU;
    p->half_even = d->round_mode == ESPDL_HIP_ROUND_HALF_EVEN;
    p->n_s_expand = d->n_shift_expand;
    p->n_s_dw = d->n_shift_dw;
    p->n_s_project = d->n_shift_project;
    if (d->residual_shift < -7 || d->residual_shift > 7)
        return fail(ESPDL_HIP_EINVAL, "residual_shift %d outside [-7, 7]", d->residual_shift);
    p->residual_shift = d->residual_shift;
    for (int st = 0; st < 2; st++) {
        const int on = st == 0 ? d->clip_expand : d->clip_dw;
        const int lo = st == 0 ? d->clip_expand_min : d->clip_dw_min, hi = st == 0 ? d->clip_expand_max : d->clip_dw_max;
        if (on != 0 && (lo < -128 || hi > 127 || lo > hi))
            return fail(ESPDL_HIP_EINVAL, "clip bounds [%d, %d] of the %s stage outside int8 or empty", lo, hi,
                        st == 0 ? "expand" : "depthwise");
    }
    if (d->clip_expand != 0 && !d->has_expand)
        return fail(ESPDL_HIP_EINVAL, "clip_expand without an expand stage");
    p->clip_e = d->clip_expand != 0;
    p->clip_e_lo = d->clip_expand_min;
    p->clip_e_hi = d->clip_expand_max;
    p->clip_d = d->clip_dw != 0;
    p->clip_d_lo = d->clip_dw_min;
    p->clip_d_hi = d->clip_dw_max;
    if ((long long)p->batch * p->out_h * p->out_w > 0x7fffffffll - 65536)
        return fail(ESPDL_HIP_EINVAL, "too many output pixels");
    return ESPDL_HIP_OK;
}

// Only the one-wavefront-per-tile kernel takes an expand stage with a window; every other form reads the
// block input as the depthwise stage's input grid.
bool pointwise_expand(const espdl::MbconvParams &p)
{
    return espdl::mbconv_expand_is_pointwise(p);
}

// Depthwise geometry and project description of a block without expand stage.
void dwproject_from(const espdl::MbconvParams &p, espdl::ConvGeom *g, espdl::DwProject *pj)
{
    g->batch = p.batch;
    g->in_h = p.in_h;
    g->in_w = p.in_w;
    g->in_c = p.in_c;
    g->out_c = p.in_c;
    g->out_h = p.out_h;
    g->out_w = p.out_w;
    g->k_h = p.k_h;
    g->k_w = p.k_w;
    g->stride_h = p.stride_h;
    g->stride_w = p.stride_w;
    g->dil_h = p.dil_h;
    g->dil_w = p.dil_w;
    g->pad_top = p.pad_top;
    g->pad_left = p.pad_left;
    g->relu = p.relu_dw;
    g->half_even = p.half_even;
    g->n_shift = p.n_s_dw;
    g->in_pitch = g->in_c;
    g->out_pitch = g->res_pitch = g->out_c;
    pj->w = p.w_project;
    pj->bias = p.b_project;
    pj->shift = p.s_project;
    pj->n_shift = p.n_s_project;
    pj->relu = p.relu_project;
    pj->out_c = p.out_c;
    pj->residual = p.residual;
    pj->out = p.out;
}

// The same for a block with expand stage: the depthwise stage works on exp_c channels.
void expand_dwproject_from(const espdl::MbconvParams &p, espdl::ConvGeom *g, espdl::DwProject *pj, espdl::DwExpand *ex)
{
    dwproject_from(p, g, pj);
    g->in_c = p.exp_c;
    g->out_c = p.exp_c;
    g->in_pitch = g->out_pitch = g->res_pitch = p.exp_c;
    ex->x = p.in;
    ex->w = p.w_expand;
    ex->bias = p.b_expand;
    ex->shift = p.s_expand;
    ex->n_shift = p.n_s_expand;
    ex->relu = p.relu_expand;
    ex->c0 = p.in_c;
}

} // namespace

extern "C" {

int espdl_hip_mbconv_out_shape(const espdl_hip_mbconv_desc *desc, int32_t *out_h, int32_t *out_w)
{
    espdl::MbconvParams p = {};
    const int rc = mbconv_geometry(desc, &p);
    if (rc != ESPDL_HIP_OK)
        return rc;
    if (out_h)
        *out_h = p.out_h;
    if (out_w)
        *out_w = p.out_w;
    return ESPDL_HIP_OK;
}

static int mbconv_kernel_choice(const espdl_hip_mbconv_desc *desc);

int espdl_hip_mbconv_s8_supported(const espdl_hip_mbconv_desc *desc)
{
    const int kind = mbconv_kernel_choice(desc);
    // a requantized residual operand is built into the two kernels that carry MobileNetV2-style networks
    if (kind != 0 && desc->residual_shift != 0 && kind != 4 && kind != 5)
        return 0;
    return kind;
}

// Blocks on large images go to the one-wavefront-per-tile kernel, small ones to the workgroup-per-tile kernel -
// unless only the former has a guard-free build for the shape (a third of the time of a guarded one).
static bool wave_before_group(const espdl::MbconvParams &p)
{
    if (!espdl::mbconv_s8_wave_supports(p))
        return false;
    if (p.in_h >= 28)
        return true;
    return espdl::mbconv_s8_wave_has_fast_build(p) &&
        !(espdl::mbconv_s8_group_supports(p) && espdl::mbconv_s8_group_has_fast_build(p));
}

static int mbconv_kernel_choice(const espdl_hip_mbconv_desc *desc)
{
    espdl::MbconvParams p = {};
    if (mbconv_geometry(desc, &p) != ESPDL_HIP_OK)
        return 0;
    // any 16-byte aligned non-null value stands for the pointers the plan looks at
    static const int8_t *const aligned = reinterpret_cast<const int8_t *>(uintptr_t(256));
    p.in = aligned;
    p.out = const_cast<int8_t *>(aligned);
    p.w_expand = desc->has_expand ? aligned : nullptr;
    p.w_dw = aligned;
    p.w_project = aligned;
    // a clamp between the stages: the guard-free builds of the one-wavefront-per-tile kernel only
    if (espdl::mbconv_has_clip(p))
        return (desc->has_expand && espdl::mbconv_s8_wave_has_fast_build(p)) ? 4 : 0;
    if (!desc->has_expand) {
        espdl::ConvGeom g;
        espdl::DwProject pj;
        dwproject_from(p, &g, &pj);
        if (espdl::depthwise_project_s8_supports(g, p.in, pj))
            return 2;
    }
    if (desc->has_expand && !pointwise_expand(p))
        return espdl::mbconv_s8_wave_supports(p) ? 4 : 0;
    if (desc->has_expand && wave_before_group(p))
        return 4;
    if (desc->has_expand && espdl::mbconv_s8_group_supports(p))
        return 5;
    if (desc->has_expand && espdl::mbconv_s8_wave_supports(p))
        return 4;
    if (desc->has_expand) {
        espdl::ConvGeom g;
        espdl::DwProject pj;
        espdl::DwExpand ex;
        expand_dwproject_from(p, &g, &pj, &ex);
        if (espdl::expand_depthwise_project_s8_supports(g, ex, pj))
            return 3;
    }
    return espdl::mbconv_s8_fused_supports(p) ? 1 : 0;
}

int espdl_hip_mbconv_s8_preferred(const espdl_hip_mbconv_desc *desc)
{
    const int kind = espdl_hip_mbconv_s8_supported(desc);
    if (kind == 2)
        return 1;
    if (kind != 4 && kind != 5)
        return 0;
    espdl::MbconvParams p = {};
    if (mbconv_geometry(desc, &p) != ESPDL_HIP_OK)
        return 0;
    static const int8_t *const aligned = reinterpret_cast<const int8_t *>(uintptr_t(256));
    p.in = aligned;
    p.w_expand = aligned;
    // Both single-launch kernels win with their guard-free builds (one per tile plan of MobileNetV2-style blocks)
    // and then at every batch size, from one image (fewer launches, no round trip of the expanded tensor) to
    // several rounds over the device; the guarded builds cover every shape but are no faster than the separate
    // launches.
    return (kind == 5 ? espdl::mbconv_s8_group_has_fast_build(p) : espdl::mbconv_s8_wave_has_fast_build(p)) ? 1 : 0;
}

int espdl_hip_mbconv_s8(const espdl_hip_mbconv_desc *desc, const int8_t *in, const espdl_hip_mbconv_weights *w,
                        const int8_t *residual, int8_t *out, void *stream)
{
    espdl::MbconvParams p = {};
    const int rc = mbconv_geometry(desc, &p);
    if (rc != ESPDL_HIP_OK)
        return rc;
    if (p.batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr || w == nullptr || w->w_dw == nullptr || w->s_dw == nullptr ||
        w->w_project == nullptr || w->s_project == nullptr || (desc->has_expand && (w->w_expand == nullptr || w->s_expand == nullptr)))
        return fail(ESPDL_HIP_EINVAL, "in, out, filters and shifts must not be NULL");
    if (misaligned(in, 4) || misaligned(out, 4) || misaligned(residual, 4) || misaligned(w->w_project, 16) ||
        misaligned(w->w_expand, 4) || misaligned(w->b_expand, 4) || misaligned(w->s_expand, 4) || misaligned(w->b_dw, 4) ||
        misaligned(w->s_dw, 4) || misaligned(w->b_project, 4) || misaligned(w->s_project, 4))
        return fail(ESPDL_HIP_EINVAL, "activations, expand filter, biases and shifts must be 4-byte aligned, the project filter 16-byte aligned");
    p.in = in;
    p.residual = residual;
    p.out = out;
    p.w_expand = desc->has_expand ? w->w_expand : nullptr;
    p.b_expand = w->b_expand;
    p.s_expand = w->s_expand;
    p.w_dw = w->w_dw;
    p.b_dw = w->b_dw;
    p.s_dw = w->s_dw;
    p.w_project = w->w_project;
    p.b_project = w->b_project;
    p.s_project = w->s_project;
    if (espdl::mbconv_has_clip(p)) {
        if (!desc->has_expand || !espdl::mbconv_s8_wave_has_fast_build(p))
            return fail(ESPDL_HIP_ENOTSUP, "a Clip between the stages is covered for the block shapes with a guard-free build of the one-wavefront-per-tile kernel, round half up");
        return device_status(espdl::launch_mbconv_s8_wave(p, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                             "mbconv_s8_wave");
    }
    if (!desc->has_expand) {
        espdl::ConvGeom g;
        espdl::DwProject pj;
        dwproject_from(p, &g, &pj);
        if (p.residual_shift == 0 && espdl::depthwise_project_s8_supports(g, p.in, pj))
            return device_status(espdl::launch_depthwise_project_s8(g, p.in, p.w_dw, p.b_dw, p.s_dw, pj, cu_count_cached(),
                                                                    reinterpret_cast<hipStream_t>(stream)),
                                 "depthwise_project_s8");
    }
    if (desc->has_expand && !pointwise_expand(p)) {
        if (!espdl::mbconv_s8_wave_supports(p))
            return fail(ESPDL_HIP_ENOTSUP, "an expand stage with a window needs a 3x3 depthwise stage, at most 4 filter rows of at most 9 bytes (exp_k_w * in_c) and at most 64 project filters");
        return device_status(espdl::launch_mbconv_s8_wave(p, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                             "mbconv_s8_wave");
    }
    if (desc->has_expand && !wave_before_group(p) && espdl::mbconv_s8_group_supports(p))
        return device_status(espdl::launch_mbconv_s8_group(p, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                             "mbconv_s8_group");
    if (desc->has_expand && espdl::mbconv_s8_wave_supports(p))
        return device_status(espdl::launch_mbconv_s8_wave(p, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                             "mbconv_s8_wave");
    // Only the two kernels above requantize the residual operand.  The answer comes from the real pointers: a
    // block whose operands are merely 4-byte aligned can be refused by both although the shape alone passes.
    if (p.residual_shift != 0)
        return fail(ESPDL_HIP_ENOTSUP, "a requantized residual operand (residual_shift %d) is not covered for this block shape and operand alignment",
                    p.residual_shift);
    if (desc->has_expand) {
        espdl::ConvGeom g;
        espdl::DwProject pj;
        espdl::DwExpand ex;
        expand_dwproject_from(p, &g, &pj, &ex);
        if (espdl::expand_depthwise_project_s8_supports(g, ex, pj))
            return device_status(espdl::launch_expand_depthwise_project_s8(g, ex, p.w_dw, p.b_dw, p.s_dw, pj, cu_count_cached(),
                                                                           reinterpret_cast<hipStream_t>(stream)),
                                 "expand_depthwise_project_s8");
    }
    if (!espdl::mbconv_s8_fused_supports(p))
        return fail(ESPDL_HIP_ENOTSUP, "this block shape is not covered by the fused kernel");
    return device_status(espdl::launch_mbconv_s8_fused(p, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         "mbconv_s8_fused");
}

static int binary_s16(int op, const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int32_t mul_shift, int32_t round_mode, int16_t *out,
                      void *stream)
{
    if (out_dims == nullptr || in0_strides == nullptr || in1_strides == nullptr)
        return fail(ESPDL_HIP_EINVAL, "dims and strides must not be NULL");
    if (mul_shift < -30 || mul_shift > 30)
        return fail(ESPDL_HIP_EINVAL, "mul_shift %d outside [-30, 30]", mul_shift);
    if (round_mode != ESPDL_HIP_ROUND_HALF_UP && round_mode != ESPDL_HIP_ROUND_HALF_EVEN)
        return fail(ESPDL_HIP_EINVAL, "bad round_mode %d", round_mode);
    long long size = 1;
    for (int i = 0; i < 4; i++) {
        if (out_dims[i] < 0 || in0_strides[i] < 0 || in1_strides[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent or stride in dim %d", i);
        size *= out_dims[i];
        if (size > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in0 == nullptr || in1 == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in0, in1 and out must not be NULL");
    static const char *const names[4] = {"add_s16", "mul_s16", "sub_s16", "div_s16"};
    return device_status(espdl::launch_binary_s16(op, out_dims, in0_strides, in1_strides, in0, in1, mul_shift,
                                                  round_mode == ESPDL_HIP_ROUND_HALF_EVEN, out, cu_count_cached(),
                                                  reinterpret_cast<hipStream_t>(stream)),
                         names[op & 3]);
}

int espdl_hip_add_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int16_t *out, void *stream)
{
    return binary_s16(0, out_dims, in0_strides, in1_strides, in0, in1, 0, ESPDL_HIP_ROUND_HALF_UP, out, stream);
}

int espdl_hip_mul_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int32_t mul_shift, int32_t round_mode, int16_t *out,
                      void *stream)
{
    return binary_s16(1, out_dims, in0_strides, in1_strides, in0, in1, mul_shift, round_mode, out, stream);
}

int espdl_hip_sub_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int16_t *out, void *stream)
{
    return binary_s16(2, out_dims, in0_strides, in1_strides, in0, in1, 0, ESPDL_HIP_ROUND_HALF_UP, out, stream);
}

int espdl_hip_div_s16(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                      const int16_t *in0, const int16_t *in1, int32_t div_shift, int16_t *out, void *stream)
{
    return binary_s16(3, out_dims, in0_strides, in1_strides, in0, in1, div_shift, ESPDL_HIP_ROUND_HALF_UP, out, stream);
}

static int subdiv_s8(bool div, const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int32_t div_shift, int8_t *out, void *stream)
{
    if (out_dims == nullptr || in0_strides == nullptr || in1_strides == nullptr)
        return fail(ESPDL_HIP_EINVAL, "dims and strides must not be NULL");
    if (div_shift < -30 || div_shift > 30)
        return fail(ESPDL_HIP_EINVAL, "div_shift %d outside [-30, 30]", div_shift);
    long long size = 1;
    for (int i = 0; i < 4; i++) {
        if (out_dims[i] < 0 || in0_strides[i] < 0 || in1_strides[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent or stride in dim %d", i);
        size *= out_dims[i];
        if (size > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in0 == nullptr || in1 == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in0, in1 and out must not be NULL");
    return device_status(espdl::launch_subdiv_s8(div, out_dims, in0_strides, in1_strides, in0, in1, div_shift, out,
                                                 cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         div ? "div_s8" : "sub_s8");
}

int espdl_hip_sub_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int8_t *out, void *stream)
{
    return subdiv_s8(false, out_dims, in0_strides, in1_strides, in0, in1, 0, out, stream);
}

int espdl_hip_div_s8(const int32_t out_dims[4], const int64_t in0_strides[4], const int64_t in1_strides[4],
                     const int8_t *in0, const int8_t *in1, int32_t div_shift, int8_t *out, void *stream)
{
    return subdiv_s8(true, out_dims, in0_strides, in1_strides, in0, in1, div_shift, out, stream);
}

int espdl_hip_avg_pool_s16(const int16_t *in, int32_t batch, int32_t h, int32_t w, int32_t c, int32_t k_h, int32_t k_w,
                           int32_t stride_h, int32_t stride_w, int32_t pad_top, int32_t pad_bottom, int32_t pad_left,
                           int32_t pad_right, int32_t in_exp, int32_t out_exp, int16_t *out, void *stream)
{
    if (batch < 0 || h <= 0 || w <= 0 || c <= 0 || k_h <= 0 || k_w <= 0 || stride_h <= 0 || stride_w <= 0 || pad_top < 0 ||
        pad_bottom < 0 || pad_left < 0 || pad_right < 0 || (long long)k_h * k_w > (1 << 15))
        return fail(ESPDL_HIP_EINVAL, "bad avg_pool geometry");
    if (h + pad_top + pad_bottom < k_h || w + pad_left + pad_right < k_w)
        return fail(ESPDL_HIP_EINVAL, "window larger than the padded image");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    const int out_h = (h + pad_top + pad_bottom - k_h) / stride_h + 1, out_w = (w + pad_left + pad_right - k_w) / stride_w + 1;
    if (batch == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_avg_pool_s16(in, batch, h, w, c, k_h, k_w, stride_h, stride_w, pad_top, pad_left,
                                                    out_h, out_w, in_exp, out_exp, out, cu_count_cached(),
                                                    reinterpret_cast<hipStream_t>(stream)),
                         "avg_pool_s16");
}

int espdl_hip_reduce_mean_s16(const int16_t *in, const int32_t *shape, int32_t dims, const int32_t *reduce_flag,
                              int32_t in_exp, int32_t out_exp, int16_t *out, void *stream)
{
    if (dims < 1 || dims > 8 || shape == nullptr || reduce_flag == nullptr)
        return fail(ESPDL_HIP_EINVAL, "reduce_mean handles 1..8 dims");
    if (check_exps(in_exp, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    int sh[8], fl[8];
    long long total = 1;
    for (int i = 0; i < dims; i++) {
        if (shape[i] < 0)
            return fail(ESPDL_HIP_EINVAL, "negative extent");
        sh[i] = shape[i];
        fl[i] = reduce_flag[i] != 0;
        total *= shape[i];
        if (total > (1ll << 40))
            return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    }
    if (total == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_reduce_mean_s16(in, sh, dims, fl, in_exp, out_exp, out, cu_count_cached(),
                                                       reinterpret_cast<hipStream_t>(stream)),
                         "reduce_mean_s16");
}

int espdl_hip_insert_zeros(const void *in, int32_t elem_size, int32_t batch, int32_t h, int32_t w, int32_t c,
                           int32_t stride_h, int32_t stride_w, int32_t output_padding_h, int32_t output_padding_w,
                           void *out, void *stream)
{
    if (elem_size != 1 && elem_size != 2 && elem_size != 4)
        return fail(ESPDL_HIP_EINVAL, "elem_size must be 1, 2 or 4");
    if (batch < 0 || h < 0 || w < 0 || c < 0)
        return fail(ESPDL_HIP_EINVAL, "negative extent");
    if (stride_h < 1 || stride_w < 1 || output_padding_h < 0 || output_padding_w < 0)
        return fail(ESPDL_HIP_EINVAL, "strides must be >= 1 and output paddings >= 0");
    if (batch == 0 || h == 0 || w == 0 || c == 0)
        return ESPDL_HIP_OK;
    const long long out_h = h + (long long)(stride_h - 1) * (h - 1) + output_padding_h;
    const long long out_w = w + (long long)(stride_w - 1) * (w - 1) + output_padding_w;
    if (out_h > 0x7fffffffll || out_w > 0x7fffffffll || (long long)batch * out_h > 0x7fffffffll / out_w ||
        (long long)batch * out_h * out_w > 0x7fffffffll / ((long long)c * elem_size))
        return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_insert_zeros(in, elem_size, batch, h, w, c, stride_h, stride_w, (int)out_h, (int)out_w,
                                                    out, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         "insert_zeros");
}

int espdl_hip_lut_s16(const int16_t *in, int64_t size, const int16_t *table, int32_t table_size, int32_t round_mode,
                      int16_t *out, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (round_mode != ESPDL_HIP_ROUND_HALF_UP && round_mode != ESPDL_HIP_ROUND_HALF_EVEN)
        return fail(ESPDL_HIP_EINVAL, "unknown round mode %d", round_mode);
    int shift = -1;
    if (table_size == 65536)
        shift = 0;
    for (int s = 0; s <= 15 && shift < 0; s++)
        if (table_size == (65536 >> s) + 1)
            shift = s;
    if (shift < 0)
        return fail(ESPDL_HIP_EINVAL, "table of %d entries: need 65536 / 2^n + 1 (n = 0..15) or 65536", table_size);
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr || table == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in, table and out must not be NULL");
    return device_status(espdl::launch_lut_s16(in, size, table, table_size, shift, round_mode == ESPDL_HIP_ROUND_HALF_EVEN,
                                               out, cu_count_cached(), reinterpret_cast<hipStream_t>(stream)),
                         "lut_s16");
}

int espdl_hip_softmax_s8(const int8_t *in, int64_t outer, int64_t len, int64_t inner, int32_t in_exp, float *out,
                         void *stream)
{
    if (outer < 0 || len < 0 || inner < 0)
        return fail(ESPDL_HIP_EINVAL, "negative extent");
    if (check_exps(in_exp, 0) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (outer == 0 || len == 0 || inner == 0)
        return ESPDL_HIP_OK;
    if (outer > (1ll << 40) / len || outer * len > (1ll << 40) / inner)
        return fail(ESPDL_HIP_ENOTSUP, "tensor too large for this build");
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_softmax_s8(in, outer, len, inner, in_exp, out, cu_count_cached(),
                                                  reinterpret_cast<hipStream_t>(stream)),
                         "softmax_s8");
}

int espdl_hip_quantize_f32(const float *in, int64_t size, int32_t out_exp, int32_t elem_size, void *out, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (elem_size != 1 && elem_size != 2)
        return fail(ESPDL_HIP_EINVAL, "elem_size must be 1 (int8) or 2 (int16)");
    if (check_exps(0, out_exp) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_quantize_f32(in, size, out_exp, elem_size, out, cu_count_cached(),
                                                    reinterpret_cast<hipStream_t>(stream)),
                         "quantize_f32");
}

int espdl_hip_dequantize_f32(const void *in, int64_t size, int32_t in_exp, int32_t elem_size, float *out, void *stream)
{
    if (size < 0)
        return fail(ESPDL_HIP_EINVAL, "negative size");
    if (elem_size != 1 && elem_size != 2)
        return fail(ESPDL_HIP_EINVAL, "elem_size must be 1 (int8) or 2 (int16)");
    if (check_exps(in_exp, 0) != ESPDL_HIP_OK)
        return ESPDL_HIP_EINVAL;
    if (size == 0)
        return ESPDL_HIP_OK;
    if (in == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "in and out must not be NULL");
    return device_status(espdl::launch_dequantize_f32(in, size, in_exp, elem_size, out, cu_count_cached(),
                                                      reinterpret_cast<hipStream_t>(stream)),
                         "dequantize_f32");
}

int espdl_hip_matmul_s8(const int8_t *a, const int8_t *b, int32_t m, int32_t k, int32_t n, const int32_t lead[2],
                        const int64_t a_stride[2], const int64_t b_stride[2], int32_t shift, int32_t activation,
                        int32_t round_mode, int8_t *out, void *stream)
{
    if (lead == nullptr || a_stride == nullptr || b_stride == nullptr)
        return fail(ESPDL_HIP_EINVAL, "lead, a_stride and b_stride must not be NULL");
    if (m < 0 || k < 0 || n < 0 || lead[0] < 0 || lead[1] < 0 || a_stride[0] < 0 || a_stride[1] < 0 || b_stride[0] < 0 ||
        b_stride[1] < 0)
        return fail(ESPDL_HIP_EINVAL, "negative extent or stride");
    if (activation != ESPDL_HIP_LINEAR && activation != ESPDL_HIP_RELU)
        return fail(ESPDL_HIP_EINVAL, "activation must be ESPDL_HIP_LINEAR or ESPDL_HIP_RELU");
    if (round_mode != ESPDL_HIP_ROUND_HALF_UP && round_mode != ESPDL_HIP_ROUND_HALF_EVEN)
        return fail(ESPDL_HIP_EINVAL, "unknown round mode %d", round_mode);
    if (shift < -31 || shift > 62)
        return fail(ESPDL_HIP_EINVAL, "shift %d outside [-31, 62]", shift);
    if (m == 0 || n == 0 || lead[0] == 0 || lead[1] == 0)
        return ESPDL_HIP_OK;
    if ((long long)lead[0] * lead[1] > 65535)
        return fail(ESPDL_HIP_ENOTSUP, "more than 65535 matrix pairs in one call");
    if (k > (1 << 16))
        return fail(ESPDL_HIP_ENOTSUP, "k above 65536: the int32 accumulator could overflow");
    if ((long long)m * n > 0x7fffffffll || (long long)m * k > 0x7fffffffll || (long long)k * n > 0x7fffffffll)
        return fail(ESPDL_HIP_ENOTSUP, "matrix too large for this build");
    if (a == nullptr || b == nullptr || out == nullptr)
        return fail(ESPDL_HIP_EINVAL, "a, b and out must not be NULL");
    const int ld[2] = {lead[0], lead[1]};
    const long long as[2] = {a_stride[0], a_stride[1]}, bs[2] = {b_stride[0], b_stride[1]};
    return device_status(espdl::launch_matmul_s8(a, b, m, k, n, ld, as, bs, shift, activation == ESPDL_HIP_RELU,
                                                 round_mode == ESPDL_HIP_ROUND_HALF_EVEN, out,
                                                 reinterpret_cast<hipStream_t>(stream)),
                         "matmul_s8");
}

} // extern "C"
