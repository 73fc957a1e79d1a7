/*
 * CPU oracle for ESP-DL's quantized operator path.  TEST INFRASTRUCTURE ONLY: see espdl_oracle.h
 * for who may use it and for the pinning status of every function.
 *
 * Each function cites the reference lines it restates (paths relative to the reference tree).
 */
#include "espdl_oracle.h"

#include <limits.h>
#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 0; /* 0 = leave OpenMP's default */

int espdl_oracle_max_threads(void)
{
#ifdef _OPENMP
    return g_threads > 0 ? g_threads : omp_get_max_threads();
#else
    return 1;
#endif
}

void espdl_oracle_set_threads(int n)
{
    g_threads = n;
#ifdef _OPENMP
    if (n > 0)
        omp_set_num_threads(n);
#endif
}

/* ---------------------------------------------------------------------------------------------
 * Integer helpers.
 * tool::truncate = clamp to the destination type (esp-dl/dl/tool/include/dl_tool.hpp:225-254).
 * ------------------------------------------------------------------------------------------- */
static inline int64_t clamp_i64(int64_t v, int64_t lo, int64_t hi)
{
    return v < lo ? lo : (v > hi ? hi : v);
}

/*
 * tool::shift_and_round<int32_t>  (esp-dl/dl/tool/src/dl_tool.cpp:95-146).
 * half-up:   shift > 0: (int64(v) + 2^(shift-1)) >> shift, arithmetic shift; the sum is formed in
 *            64 bits (`half` is int64_t there) and narrowed back to T.
 *            shift <= 0: int64(v) << -shift, saturated to T.
 * half-even: shift > 0: q = v >> shift, r = v & (2^shift - 1) (computed in T), bump q when
 *            r > half, or r == half and q is odd.
 */
int32_t espdl_oracle_shift_round_s32(int32_t value, int shift, int round_mode)
{
    if (shift <= 0) {
        /* multiply instead of shifting a negative number: same value, no undefined behaviour */
        int64_t shifted = (int64_t)value * ((int64_t)1 << -shift);
        return (int32_t)clamp_i64(shifted, INT32_MIN, INT32_MAX);
    }
    if (round_mode == ESPDL_ORACLE_ROUND_HALF_EVEN) {
        int32_t q = value >> shift;
        int32_t rem = value & (int32_t)(((uint32_t)1 << shift) - 1u);
        int32_t half = (int32_t)((uint32_t)1 << (shift - 1));
        if (rem > half || (rem == half && (q & 1)))
            q += 1;
        return q;
    }
    int64_t half = (int64_t)1 << (shift - 1);
    return (int32_t)(((int64_t)value + half) >> shift);
}

/* tool::shift_and_round<int64_t>: same text with T = int64_t (no widening is available). */
int64_t espdl_oracle_shift_round_s64(int64_t value, int shift, int round_mode)
{
    if (shift <= 0) {
        return (int64_t)((uint64_t)value << -shift); /* truncate(int64, int64) is the identity */
    }
    if (round_mode == ESPDL_ORACLE_ROUND_HALF_EVEN) {
        int64_t q = value >> shift;
        int64_t rem = value & (int64_t)(((uint64_t)1 << shift) - 1u);
        int64_t half = (int64_t)((uint64_t)1 << (shift - 1));
        if (rem > half || (rem == half && (q & 1)))
            q += 1;
        return q;
    }
    int64_t half = (int64_t)1 << (shift - 1);
    return (int64_t)((uint64_t)value + (uint64_t)half) >> shift;
}

/* Conv::get_output_shape (esp-dl/dl/module/include/dl_module_conv.hpp:90-98). */
int espdl_oracle_conv_out_h(const espdl_oracle_conv_t *g)
{
    return (g->in_h + g->pad_top + g->pad_bottom - g->dil_h * (g->k_h - 1) - 1) / g->stride_h + 1;
}

int espdl_oracle_conv_out_w(const espdl_oracle_conv_t *g)
{
    return (g->in_w + g->pad_left + g->pad_right - g->dil_w * (g->k_w - 1) - 1) / g->stride_w + 1;
}

static int geometry_ok(const espdl_oracle_conv_t *g, int depthwise)
{
    if (g->batch < 0 || g->in_h <= 0 || g->in_w <= 0 || g->in_c <= 0 || g->out_c <= 0)
        return 0;
    if (g->k_h <= 0 || g->k_w <= 0 || g->stride_h <= 0 || g->stride_w <= 0 || g->dil_h <= 0 || g->dil_w <= 0)
        return 0;
    if (g->pad_top < 0 || g->pad_bottom < 0 || g->pad_left < 0 || g->pad_right < 0)
        return 0;
    if (g->n_shift != 1 && g->n_shift != g->out_c)
        return 0;
    if (depthwise && g->out_c != g->in_c)
        return 0;
    if (g->in_h + g->pad_top + g->pad_bottom - g->dil_h * (g->k_h - 1) - 1 < 0)
        return 0;
    if (g->in_w + g->pad_left + g->pad_right - g->dil_w * (g->k_w - 1) - 1 < 0)
        return 0;
    return 1;
}

/*
 * The reference walks output pixels and, at padded borders, shrinks the filter window to the taps
 * that fall inside the image (esp-dl/dl/base/dl_base.hpp:951-1138; valid padding :1172-1191), so a
 * tap outside the image contributes nothing: zero padding.  [k0, k1) below is that in-image tap
 * range along one axis for the output coordinate `o`.
 */
static inline void tap_range(int o, int stride, int pad_head, int dil, int k, int in_size, int *k0, int *k1)
{
    int origin = o * stride - pad_head; /* input coordinate of tap 0 */
    int lo = 0, hi = k;
    if (origin < 0)
        lo = (-origin + dil - 1) / dil;
    /* last tap with origin + t*dil <= in_size - 1 */
    if (origin + (k - 1) * dil > in_size - 1) {
        int room = in_size - 1 - origin;
        hi = room < 0 ? 0 : room / dil + 1;
    }
    if (lo > hi)
        lo = hi;
    *k0 = lo;
    *k1 = hi;
}

/* ---------------------------------------------------------------------------------------------
 * Dense convolution, int8.
 *   MAC      conv2d_11cn / conv2d_33cn / conv2d_hwcn  (esp-dl/dl/base/dl_base_conv2d.cpp:9-163):
 *            int8 * int8 products accumulated in int32, filter [Cout][kH][kW][Cin].
 *   epilogue buffer_bias_linear/_relu, buffer_0000_linear/_relu
 *            (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210):
 *            acc += bias (int32) -> shift_and_round(acc, mac_shift) -> ReLU -> truncate to int8.
 *   mac_shift = out_exp - filter_exp - in_exp (esp-dl/dl/base/dl_base.hpp:260); with a shift per
 *            output channel the same formula is applied channel-wise.
 * ------------------------------------------------------------------------------------------- */
int espdl_oracle_conv2d_s8(const espdl_oracle_conv_t *g, const int8_t *in, const int8_t *filter,
                           const int32_t *bias, const int32_t *shift, int8_t *out)
{
    if (!geometry_ok(g, 0))
        return -1;
    const int oh = espdl_oracle_conv_out_h(g), ow = espdl_oracle_conv_out_w(g);
    const int C = g->in_c, OC = g->out_c, KH = g->k_h, KW = g->k_w;
    const int64_t in_img = (int64_t)g->in_h * g->in_w * C;
    const int64_t out_img = (int64_t)oh * ow * OC;
    const int64_t rows = (int64_t)g->batch * oh;

#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; row++) {
        const int n = (int)(row / oh), oy = (int)(row % oh);
        const int8_t *img = in + n * in_img;
        int8_t *dst = out + n * out_img + (int64_t)oy * ow * OC;
        int ky0, ky1;
        tap_range(oy, g->stride_h, g->pad_top, g->dil_h, KH, g->in_h, &ky0, &ky1);
        for (int ox = 0; ox < ow; ox++) {
            int kx0, kx1;
            tap_range(ox, g->stride_w, g->pad_left, g->dil_w, KW, g->in_w, &kx0, &kx1);
            for (int oc = 0; oc < OC; oc++) {
                const int8_t *f_oc = filter + (int64_t)oc * KH * KW * C;
                int32_t acc = 0;
                for (int ky = ky0; ky < ky1; ky++) {
                    const int iy = oy * g->stride_h - g->pad_top + ky * g->dil_h;
                    for (int kx = kx0; kx < kx1; kx++) {
                        const int ix = ox * g->stride_w - g->pad_left + kx * g->dil_w;
                        const int8_t *px = img + ((int64_t)iy * g->in_w + ix) * C;
                        const int8_t *fw = f_oc + ((int64_t)ky * KW + kx) * C;
                        int32_t s = 0;
                        for (int c = 0; c < C; c++)
                            s += (int32_t)px[c] * (int32_t)fw[c];
                        acc += s;
                    }
                }
                if (bias)
                    acc = (int32_t)((uint32_t)acc + (uint32_t)bias[oc]); /* int32 += int32 */
                int32_t v = espdl_oracle_shift_round_s32(acc, shift[g->n_shift == 1 ? 0 : oc], g->round_mode);
                if (g->activation == ESPDL_ORACLE_RELU && v < 0)
                    v = 0;
                dst[(int64_t)ox * OC + oc] = (int8_t)clamp_i64(v, INT8_MIN, INT8_MAX);
            }
        }
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Depthwise convolution, int8.
 *   MAC      depthwise_conv2d_11c1 / _33c1 / _hwc1
 *            (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:9-65): acc[c] += in[iy][ix][c] * f[ky][kx][c].
 *   epilogue the same n_wise functions as the dense path
 *            (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:760-805), shift indexed by channel.
 * ------------------------------------------------------------------------------------------- */
int espdl_oracle_depthwise_s8(const espdl_oracle_conv_t *g, const int8_t *in, const int8_t *filter,
                              const int32_t *bias, const int32_t *shift, int8_t *out)
{
    if (!geometry_ok(g, 1))
        return -1;
    const int oh = espdl_oracle_conv_out_h(g), ow = espdl_oracle_conv_out_w(g);
    const int C = g->in_c, KH = g->k_h, KW = g->k_w;
    const int64_t in_img = (int64_t)g->in_h * g->in_w * C;
    const int64_t out_img = (int64_t)oh * ow * C;
    const int64_t rows = (int64_t)g->batch * oh;

#pragma omp parallel
    {
        int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)C);
#pragma omp for schedule(static)
        for (int64_t row = 0; row < rows; row++) {
            const int n = (int)(row / oh), oy = (int)(row % oh);
            const int8_t *img = in + n * in_img;
            int8_t *dst = out + n * out_img + (int64_t)oy * ow * C;
            int ky0, ky1;
            tap_range(oy, g->stride_h, g->pad_top, g->dil_h, KH, g->in_h, &ky0, &ky1);
            for (int ox = 0; ox < ow; ox++) {
                int kx0, kx1;
                tap_range(ox, g->stride_w, g->pad_left, g->dil_w, KW, g->in_w, &kx0, &kx1);
                memset(acc, 0, sizeof(int32_t) * (size_t)C);
                for (int ky = ky0; ky < ky1; ky++) {
                    const int iy = oy * g->stride_h - g->pad_top + ky * g->dil_h;
                    for (int kx = kx0; kx < kx1; kx++) {
                        const int ix = ox * g->stride_w - g->pad_left + kx * g->dil_w;
                        const int8_t *px = img + ((int64_t)iy * g->in_w + ix) * C;
                        const int8_t *fw = filter + ((int64_t)ky * KW + kx) * C;
                        for (int c = 0; c < C; c++)
                            acc[c] += (int32_t)px[c] * (int32_t)fw[c];
                    }
                }
                for (int c = 0; c < C; c++) {
                    int32_t a = acc[c];
                    if (bias)
                        a = (int32_t)((uint32_t)a + (uint32_t)bias[c]);
                    int32_t v = espdl_oracle_shift_round_s32(a, shift[g->n_shift == 1 ? 0 : c], g->round_mode);
                    if (g->activation == ESPDL_ORACLE_RELU && v < 0)
                        v = 0;
                    dst[(int64_t)ox * C + c] = (int8_t)clamp_i64(v, INT8_MIN, INT8_MAX);
                }
            }
        }
        free(acc);
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * int16 paths: products are int16*int16 (formed as `int`), accumulator / bias / shift_and_round in
 * int64 (DL_S16_BUFFER_TYPE, esp-dl/dl/dl_define_private.hpp:15-17;
 * esp-dl/dl/base/dl_base_conv2d.cpp:875-897, 912-939; dl_base_depthwise_conv2d.cpp:495-519),
 * output clamped to the int16 range.
 * ------------------------------------------------------------------------------------------- */
int espdl_oracle_conv2d_s16(const espdl_oracle_conv_t *g, const int16_t *in, const int16_t *filter,
                            const int64_t *bias, const int32_t *shift, int16_t *out)
{
    if (!geometry_ok(g, 0))
        return -1;
    const int oh = espdl_oracle_conv_out_h(g), ow = espdl_oracle_conv_out_w(g);
    const int C = g->in_c, OC = g->out_c, KH = g->k_h, KW = g->k_w;
    const int64_t in_img = (int64_t)g->in_h * g->in_w * C;
    const int64_t out_img = (int64_t)oh * ow * OC;
    const int64_t rows = (int64_t)g->batch * oh;

#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; row++) {
        const int n = (int)(row / oh), oy = (int)(row % oh);
        const int16_t *img = in + n * in_img;
        int16_t *dst = out + n * out_img + (int64_t)oy * ow * OC;
        int ky0, ky1;
        tap_range(oy, g->stride_h, g->pad_top, g->dil_h, KH, g->in_h, &ky0, &ky1);
        for (int ox = 0; ox < ow; ox++) {
            int kx0, kx1;
            tap_range(ox, g->stride_w, g->pad_left, g->dil_w, KW, g->in_w, &kx0, &kx1);
            for (int oc = 0; oc < OC; oc++) {
                const int16_t *f_oc = filter + (int64_t)oc * KH * KW * C;
                int64_t acc = 0;
                for (int ky = ky0; ky < ky1; ky++) {
                    const int iy = oy * g->stride_h - g->pad_top + ky * g->dil_h;
                    for (int kx = kx0; kx < kx1; kx++) {
                        const int ix = ox * g->stride_w - g->pad_left + kx * g->dil_w;
                        const int16_t *px = img + ((int64_t)iy * g->in_w + ix) * C;
                        const int16_t *fw = f_oc + ((int64_t)ky * KW + kx) * C;
                        for (int c = 0; c < C; c++)
                            acc += (int64_t)((int32_t)px[c] * (int32_t)fw[c]);
                    }
                }
                if (bias)
                    acc += bias[oc];
                int64_t v = espdl_oracle_shift_round_s64(acc, shift[g->n_shift == 1 ? 0 : oc], g->round_mode);
                if (g->activation == ESPDL_ORACLE_RELU && v < 0)
                    v = 0;
                dst[(int64_t)ox * OC + oc] = (int16_t)clamp_i64(v, INT16_MIN, INT16_MAX);
            }
        }
    }
    return 0;
}

int espdl_oracle_depthwise_s16(const espdl_oracle_conv_t *g, const int16_t *in, const int16_t *filter,
                               const int64_t *bias, const int32_t *shift, int16_t *out)
{
    if (!geometry_ok(g, 1))
        return -1;
    const int oh = espdl_oracle_conv_out_h(g), ow = espdl_oracle_conv_out_w(g);
    const int C = g->in_c, KH = g->k_h, KW = g->k_w;
    const int64_t in_img = (int64_t)g->in_h * g->in_w * C;
    const int64_t out_img = (int64_t)oh * ow * C;
    const int64_t rows = (int64_t)g->batch * oh;

#pragma omp parallel for schedule(static)
    for (int64_t row = 0; row < rows; row++) {
        const int n = (int)(row / oh), oy = (int)(row % oh);
        const int16_t *img = in + n * in_img;
        int16_t *dst = out + n * out_img + (int64_t)oy * ow * C;
        int ky0, ky1;
        tap_range(oy, g->stride_h, g->pad_top, g->dil_h, KH, g->in_h, &ky0, &ky1);
        for (int ox = 0; ox < ow; ox++) {
            int kx0, kx1;
            tap_range(ox, g->stride_w, g->pad_left, g->dil_w, KW, g->in_w, &kx0, &kx1);
            for (int c = 0; c < C; c++) {
                int64_t acc = 0;
                for (int ky = ky0; ky < ky1; ky++) {
                    const int iy = oy * g->stride_h - g->pad_top + ky * g->dil_h;
                    for (int kx = kx0; kx < kx1; kx++) {
                        const int ix = ox * g->stride_w - g->pad_left + kx * g->dil_w;
                        acc += (int64_t)((int32_t)img[((int64_t)iy * g->in_w + ix) * C + c] *
                                         (int32_t)filter[((int64_t)ky * KW + kx) * C + c]);
                    }
                }
                if (bias)
                    acc += bias[c];
                int64_t v = espdl_oracle_shift_round_s64(acc, shift[g->n_shift == 1 ? 0 : c], g->round_mode);
                if (g->activation == ESPDL_ORACLE_RELU && v < 0)
                    v = 0;
                dst[(int64_t)ox * C + c] = (int16_t)clamp_i64(v, INT16_MIN, INT16_MAX);
            }
        }
    }
    return 0;
}

/* lut_s8_c (esp-dl/dl/base/dl_base_lut.cpp:10-15): out = table[(uint8)in ^ 0x80]. */
void espdl_oracle_lut_s8(const int8_t *in, int64_t size, const int8_t *table, int8_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < size; i++)
        out[i] = table[(uint8_t)in[i] ^ 0x80u];
}

/*
 * prelu_11c<int8_t, int16_t> (esp-dl/dl/base/dl_base_prelu.cpp:7-21): for x < 0 the product
 * int16(x) * int16(alpha[c]) is formed as `int`, shifted with DL_RIGHT_SHIFT (arithmetic right
 * shift for shift > 0, left shift otherwise; esp-dl/dl/dl_define.hpp:67-69), stored into an int16
 * temporary, then clamped to int8.  shift comes from get_activation_args
 * (esp-dl/dl/base/dl_base.hpp:2165-2168).
 */
void espdl_oracle_prelu_s8(const int8_t *in, int64_t pixels, int channels, const int8_t *alpha, int shift,
                           int8_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t p = 0; p < pixels; p++) {
        const int8_t *src = in + p * channels;
        int8_t *dst = out + p * channels;
        for (int c = 0; c < channels; c++) {
            int8_t x = src[c];
            if (x < 0) {
                int prod = (int)(int16_t)x * (int)(int16_t)alpha[c];
                int shifted = shift > 0 ? (prod >> shift) : (int)((unsigned)prod << -shift);
                int16_t temp = (int16_t)shifted;
                x = (int8_t)clamp_i64(temp, INT8_MIN, INT8_MAX);
            }
            dst[c] = x;
        }
    }
}

/* tool::round(float) = (int)floorf(value + 0.5) with a double literal (esp-dl/dl/tool/src/dl_tool.cpp:72-75). */
static inline int round_half_up_f32(float v)
{
    return (int)floorf((float)((double)v + 0.5));
}

/* DL_SCALE / DL_RESCALE (esp-dl/dl/dl_define.hpp:75-81) */
static inline float dl_scale(int e)
{
    return e > 0 ? (float)(1 << e) : 1.0f / (float)(1 << -e);
}
static inline float dl_rescale(int e)
{
    return e > 0 ? 1.0f / (float)(1 << e) : (float)(1 << -e);
}

/* Relu::forward_template (esp-dl/dl/module/include/dl_module_relu.hpp:65-93). */
void espdl_oracle_relu_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out)
{
    if (in_exp == out_exp) {
        for (int64_t i = 0; i < size; i++)
            out[i] = in[i] >= 0 ? in[i] : 0;
        return;
    }
    const float input_scale = dl_scale(in_exp), output_scale = dl_rescale(out_exp);
    for (int64_t i = 0; i < size; i++) {
        float temp = (float)in[i] * input_scale;
        out[i] = temp >= 0 ? (int8_t)clamp_i64(round_half_up_f32(temp * output_scale), INT8_MIN, INT8_MAX) : 0;
    }
}

/* Clip::forward_template (esp-dl/dl/module/include/dl_module_clip.hpp:78-90); min/max are quantized scalars. */
void espdl_oracle_clip_s8(const int8_t *in, int64_t size, int min_q, int max_q, int in_exp, int out_exp,
                          int8_t *out)
{
    const float rescale = dl_scale(in_exp) * dl_rescale(out_exp);
    for (int64_t i = 0; i < size; i++) {
        int8_t t = in[i] < min_q ? (int8_t)min_q : (in[i] > max_q ? (int8_t)max_q : in[i]);
        out[i] = (int8_t)clamp_i64(round_half_up_f32((float)t * rescale), INT8_MIN, INT8_MAX);
    }
}

/* c_impl_add_n_n / _n_1 / _1_n (esp-dl/dl/base/dl_base_add.cpp:8-44): clamp(a + b), no exponent handling. */
void espdl_oracle_add_s8(const int8_t *in0, int64_t len0, const int8_t *in1, int64_t len1, int64_t size,
                         int8_t *out)
{
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < size; i++) {
        int32_t a = in0[len0 == 1 ? 0 : i], b = in1[len1 == 1 ? 0 : i];
        out[i] = (int8_t)clamp_i64(a + b, INT8_MIN, INT8_MAX);
    }
}

/*
 * Mul, int8 (esp-dl/dl/base/dl_base_mul.cpp:9-46, 130-141; scales dl_base_elemwise.cpp:167-171):
 * out = truncate(round(float(a * b) * rescale)), rescale = DL_SCALE(e0) * DL_SCALE(e1) * DL_RESCALE(eout),
 * a product of powers of two, passed here as shift = eout - e0 - e1 (rescale = 2^-shift).  The portable C
 * path rounds half up (tool::round).  round_mode half-even restates what the ESP32-P4 kernels do for this
 * operator (they configure the hardware rounding, dl_base_mul.cpp:90): shift_and_round half-even of the
 * integer product.  len0 / len1 are `size` or 1 (scalar operand).
 */
void espdl_oracle_mul_s8(const int8_t *in0, int64_t len0, const int8_t *in1, int64_t len1, int64_t size, int shift,
                         int round_mode, int8_t *out)
{
    const float rescale = dl_rescale(shift); /* 2^-shift */
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < size; i++) {
        const int32_t a = in0[len0 == 1 ? 0 : i], b = in1[len1 == 1 ? 0 : i];
        const int32_t prod = a * b;
        int64_t q;
        if (round_mode == ESPDL_ORACLE_ROUND_HALF_EVEN && shift > 0)
            q = espdl_oracle_shift_round_s32(prod, shift, ESPDL_ORACLE_ROUND_HALF_EVEN);
        else
            q = (int64_t)floorf((float)prod * rescale + 0.5f);
        out[i] = (int8_t)clamp_i64(q, INT8_MIN, INT8_MAX);
    }
}

/*
 * GlobalAveragePool = avgpool2d_hwc over the whole image (esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54):
 * int32 sum per channel, then truncate(round(float(sum) * scale)),
 * scale = DL_SCALE(in_exp) * (1.f / area) * DL_RESCALE(out_exp) evaluated left to right in float32.
 */
void espdl_oracle_global_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int in_exp, int out_exp,
                                     int8_t *out)
{
    const float area_inv = 1.f / (float)(h * w);
    const float scale = dl_scale(in_exp) * area_inv * dl_rescale(out_exp);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < batch; n++) {
        const int8_t *img = in + (int64_t)n * h * w * c;
        for (int ch = 0; ch < c; ch++) {
            int32_t sum = 0;
            for (int p = 0; p < h * w; p++)
                sum += img[(int64_t)p * c + ch];
            out[(int64_t)n * c + ch] = (int8_t)clamp_i64(round_half_up_f32((float)sum * scale), INT8_MIN, INT8_MAX);
        }
    }
}

/*
 * AveragePool, int8 NHWC (esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54 under the pool shell of
 * dl_base_pool2d.hpp:439-560): int32 sum over the window clipped to the image, then
 * truncate(round(float(sum) * scale)) with scale = DL_SCALE(in_exp) * (1.f / area) * DL_RESCALE(out_exp)
 * evaluated left to right in float32.  On the portable C path `area` stays k_h * k_w for every window,
 * clipped or not (args.avg_pool_area is set once, dl_base_pool2d.hpp:132).  Output size as MaxPool.
 */
void espdl_oracle_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                              int stride_w, int pad_top, int pad_bottom, int pad_left, int pad_right, int in_exp,
                              int out_exp, int8_t *out)
{
    const int out_h = (h + pad_top + pad_bottom - k_h) / stride_h + 1;
    const int out_w = (w + pad_left + pad_right - k_w) / stride_w + 1;
    const float area_inv = 1.f / (float)(k_h * k_w);
    const float scale = dl_scale(in_exp) * area_inv * dl_rescale(out_exp);
#pragma omp parallel for schedule(static)
    for (int n = 0; n < batch; n++)
        for (int oy = 0; oy < out_h; oy++)
            for (int ox = 0; ox < out_w; ox++)
                for (int k = 0; k < c; k++) {
                    int32_t sum = 0;
                    for (int ky = 0; ky < k_h; ky++) {
                        const int iy = oy * stride_h - pad_top + ky;
                        if (iy < 0 || iy >= h)
                            continue;
                        for (int kx = 0; kx < k_w; kx++) {
                            const int ix = ox * stride_w - pad_left + kx;
                            if (ix < 0 || ix >= w)
                                continue;
                            sum += in[(((int64_t)n * h + iy) * w + ix) * c + k];
                        }
                    }
                    out[(((int64_t)n * out_h + oy) * out_w + ox) * c + k] =
                        (int8_t)clamp_i64(round_half_up_f32((float)sum * scale), INT8_MIN, INT8_MAX);
                }
}

/*
 * ReduceMean, int8 (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:16-45 over the loops of
 * dl_module_reduce_base.hpp:121-260): int32 sum over the flagged axes, then
 * truncate(round(sum * DL_SCALE(in_exp) / count * DL_RESCALE(out_exp))) in float32, left to right,
 * count = number of summed elements.  `out` holds the kept axes in order (keepdims only changes the
 * shape, not the bytes).  Up to 8 dims.
 */
int espdl_oracle_reduce_mean_s8(const int8_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                int out_exp, int8_t *out)
{
    if (dims < 1 || dims > 8)
        return -1;
    int64_t stride[8], total = 1, count = 1;
    stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        stride[i] = stride[i + 1] * shape[i + 1];
    for (int i = 0; i < dims; i++) {
        total *= shape[i];
        if (reduce_flag[i])
            count *= shape[i];
    }
    if (total == 0)
        return 0;
    const int64_t n_out = total / count;
    int32_t *sums = (int32_t *)calloc((size_t)n_out, sizeof(int32_t));
    if (!sums)
        return -1;
    int64_t idx[8] = {0};
    for (int64_t e = 0; e < total; e++) {
        int64_t o = 0;
        for (int i = 0; i < dims; i++)
            if (!reduce_flag[i])
                o = o * shape[i] + idx[i];
        sums[o] += in[e];
        for (int i = dims - 1; i >= 0; i--) {
            if (++idx[i] < shape[i])
                break;
            idx[i] = 0;
        }
    }
    const float input_scale = dl_scale(in_exp), output_scale = dl_rescale(out_exp);
    for (int64_t o = 0; o < n_out; o++)
        out[o] = (int8_t)clamp_i64(round_half_up_f32((float)sums[o] * input_scale / (float)count * output_scale),
                                   INT8_MIN, INT8_MAX);
    free(sums);
    (void)stride;
    return 0;
}

/*
 * Slice with ONNX semantics (what base::get_slice_shape, esp-dl/dl/base/dl_base_shape.cpp:68-120, and
 * TensorBase::slice compute for positive steps): per listed axis take indices start, start + step, ...
 * below end.  starts / ends / steps here are already normalized to 0 <= start < dim, step >= 1 and the
 * output extent out_shape[axis]; every other axis is copied whole.  Up to 8 dims.
 */
int espdl_oracle_slice(const void *in, const int *shape, int dims, const int *start, const int *step,
                       const int *out_shape, int elem_size, void *out)
{
    if (dims < 1 || dims > 8)
        return -1;
    int64_t in_stride[8], total = 1;
    in_stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        in_stride[i] = in_stride[i + 1] * shape[i + 1];
    for (int i = 0; i < dims; i++)
        total *= out_shape[i];
    int64_t idx[8] = {0};
    for (int64_t e = 0; e < total; e++) {
        int64_t src = 0;
        for (int i = 0; i < dims; i++)
            src += ((int64_t)start[i] + idx[i] * step[i]) * in_stride[i];
        memcpy((char *)out + e * elem_size, (const char *)in + src * elem_size, (size_t)elem_size);
        for (int i = dims - 1; i >= 0; i--) {
            if (++idx[i] < out_shape[i])
                break;
            idx[i] = 0;
        }
    }
    return 0;
}

/*
 * TensorBase::assign, int8 -> int8 with different exponents
 * (esp-dl/dl/tensor/src/dl_tensor_base.cpp:362-371; quantize/dequantize :18-42):
 * quantize(dequantize(x, DL_SCALE(in_exp)), 1.0 / DL_SCALE(out_exp)).
 */
void espdl_oracle_requantize_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out)
{
    if (in_exp == out_exp) {
        memmove(out, in, (size_t)size);
        return;
    }
    const float src_scale = dl_scale(in_exp);
    const float inv_scale = (float)(1.0 / (double)dl_scale(out_exp));
    for (int64_t i = 0; i < size; i++) {
        float tmp = (float)in[i] * src_scale;
        out[i] = (int8_t)clamp_i64(round_half_up_f32(tmp * inv_scale), INT8_MIN, INT8_MAX);
    }
}

/*
 * Softmax on an int8 tensor, float32 result (Softmax::forward_lut,
 * esp-dl/dl/module/include/dl_module_softmax.hpp:148-217): a 256-entry table
 * expf(DL_SCALE(in_exp) * (i - 128)) (tool::gen_lut_8bit, esp-dl/dl/tool/src/dl_tool.cpp:258-268), the
 * row sum accumulated in float32 in index order, then one division per element.  No maximum is
 * subtracted on this path.  The tensor is viewed as [outer][len][inner], softmax along len.
 */
void espdl_oracle_softmax_s8(const int8_t *in, int64_t outer, int64_t len, int64_t inner, int in_exp, float *out)
{
    float table[256];
    const float scale = dl_scale(in_exp);
    for (int i = 0; i < 256; i++)
        table[i] = expf(scale * (float)(i - 128));
    for (int64_t o = 0; o < outer; o++)
        for (int64_t k = 0; k < inner; k++) {
            const int8_t *src = in + o * len * inner + k;
            float *dst = out + o * len * inner + k;
            float sum = 0.f;
            for (int64_t i = 0; i < len; i++) {
                dst[i * inner] = table[(int)src[i * inner] + 128];
                sum += dst[i * inner];
            }
            for (int64_t i = 0; i < len; i++)
                dst[i * inner] = dst[i * inner] / sum;
        }
}

/*
 * QuantizeLinear = TensorBase::assign from a float32 tensor
 * (esp-dl/dl/tensor/src/dl_tensor_base.cpp:251-268, quantize :17-29): clip(round(v * DL_RESCALE(out_exp))).
 * elem_size 1 writes int8, 2 writes int16.
 */
void espdl_oracle_quantize_f32(const float *in, int64_t size, int out_exp, int elem_size, void *out)
{
    const float inv_scale = dl_rescale(out_exp);
    for (int64_t i = 0; i < size; i++) {
        const int q = round_half_up_f32(in[i] * inv_scale);
        if (elem_size == 1)
            ((int8_t *)out)[i] = (int8_t)clamp_i64(q, INT8_MIN, INT8_MAX);
        else
            ((int16_t *)out)[i] = (int16_t)clamp_i64(q, INT16_MIN, INT16_MAX);
    }
}

/* DequantizeLinear = TensorBase::assign into a float32 tensor (dl_tensor_base.cpp:286-299): v * DL_SCALE(in_exp). */
void espdl_oracle_dequantize_f32(const void *in, int64_t size, int in_exp, int elem_size, float *out)
{
    const float scale = dl_scale(in_exp);
    for (int64_t i = 0; i < size; i++)
        out[i] = (elem_size == 1 ? (float)((const int8_t *)in)[i] : (float)((const int16_t *)in)[i]) * scale;
}

/* ---------------------------------------------------------------------------------------------
 * int16 forms of the element-wise and pooling operators (the int16 PP-OCR recognizer uses them).
 * ------------------------------------------------------------------------------------------- */

/* Add, int16 (c_impl_add_n_n<int16_t>, esp-dl/dl/base/dl_base_add.cpp:33-44): saturating integer add. */
void espdl_oracle_add_s16(const int16_t *in0, int64_t len0, const int16_t *in1, int64_t len1, int64_t size,
                          int16_t *out)
{
    for (int64_t i = 0; i < size; i++) {
        const int32_t a = in0[len0 == 1 ? 0 : i], b = in1[len1 == 1 ? 0 : i];
        out[i] = (int16_t)clamp_i64(a + b, INT16_MIN, INT16_MAX);
    }
}

/*
 * Mul, int16 (c_impl_mul_n_n<int16_t>, esp-dl/dl/base/dl_base_mul.cpp:33-46): the int32 product is
 * converted to float32 (rounding to nearest even above 2^24), scaled by 2^-shift and rounded with
 * tool::round.  Half-even mode restates the ESP32-P4 kernels as for int8: shift_and_round half-even of
 * the exact product.
 */
void espdl_oracle_mul_s16(const int16_t *in0, int64_t len0, const int16_t *in1, int64_t len1, int64_t size, int shift,
                          int round_mode, int16_t *out)
{
    const float rescale = dl_rescale(shift);
    for (int64_t i = 0; i < size; i++) {
        const int32_t a = in0[len0 == 1 ? 0 : i], b = in1[len1 == 1 ? 0 : i];
        const int32_t prod = a * b; /* at most 2^30 in magnitude */
        int64_t q;
        if (round_mode == ESPDL_ORACLE_ROUND_HALF_EVEN && shift > 0)
            q = espdl_oracle_shift_round_s32(prod, shift, ESPDL_ORACLE_ROUND_HALF_EVEN);
        else
            q = round_half_up_f32((float)prod * rescale);
        out[i] = (int16_t)clamp_i64(q, INT16_MIN, INT16_MAX);
    }
}

/* Sub, int16 (c_impl_sub_n_n<int16_t>, esp-dl/dl/base/dl_base_sub.cpp:33-43): saturating integer subtraction. */
void espdl_oracle_sub_s16(const int16_t *in0, int64_t len0, const int16_t *in1, int64_t len1, int64_t size,
                          int16_t *out)
{
    for (int64_t i = 0; i < size; i++) {
        const int32_t a = in0[len0 == 1 ? 0 : i], b = in1[len1 == 1 ? 0 : i];
        out[i] = (int16_t)clamp_i64(a - b, INT16_MIN, INT16_MAX);
    }
}

/*
 * Div, int16 (esp-dl/dl/base/dl_base_div.cpp:66-68, 92-112, 141-163, 175-195): float32 arithmetic whose
 * order depends on which operand is constant along the innermost axis.  rescale = 2^-shift with
 * shift = out_exp - in0_exp + in1_exp.  form 0 (both vary): round(a * rescale / b); form 1 (divisor
 * constant): round(a * (rescale / b)); form 2 (dividend constant): round((a * rescale) / b).  a == 0 gives
 * 0, b == 0 gives the int16 extreme of a's sign.  Operands are passed already broadcast to `size`.
 */
void espdl_oracle_div_s16(const int16_t *in0, const int16_t *in1, int64_t size, int shift, int form, int16_t *out)
{
    const float rescale = dl_rescale(shift);
    for (int64_t i = 0; i < size; i++) {
        const int16_t a = in0[i], b = in1[i];
        if (a == 0) {
            out[i] = 0;
        } else if (b == 0) {
            out[i] = a > 0 ? INT16_MAX : INT16_MIN;
        } else {
            float v;
            if (form == 1) {
                const float r = rescale / (float)b;
                v = (float)a * r;
            } else if (form == 2) {
                const float r = (float)a * rescale;
                v = r / (float)b;
            } else {
                v = (float)a * rescale / (float)b;
            }
            out[i] = (int16_t)clamp_i64(round_half_up_f32(v), INT16_MIN, INT16_MAX);
        }
    }
}

/*
 * ReduceMax, ReduceMin, ReduceSum for int8 / int16 (esp-dl/dl/module/include/dl_module_reduce_max.hpp:14-52,
 * dl_module_reduce_min.hpp:15-53, dl_module_reduce_sum.hpp:13-56): max and min of the stored integers from the
 * type's minimum / maximum; the sum is accumulated in int32 (int8) or int64 (int16), then
 * shift_and_round(sum, out_exp - in_exp) and truncate.  Written as one walk over the input that folds every
 * element into its output slot.  ReduceL1 and ReduceSumSquare (dl_module_reduce_l1.hpp:14-50,
 * dl_module_reduce_sum_square.hpp:14-46) accumulate |x| and x * x the same way; the caller passes
 * shift = out_exp - 2 * in_exp for the squares.  op: 0 max, 1 min, 2 sum, 3 L1, 4 sum of squares.
 */
int espdl_oracle_reduce_int(const void *in, int bits, const int32_t *shape, int dims, const int32_t *reduce_flag, int op,
                            int shift, int round_mode, void *out)
{
    if (dims < 1 || dims > 8 || (bits != 8 && bits != 16))
        return -1;
    const int lo = bits == 8 ? INT8_MIN : INT16_MIN, hi = bits == 8 ? INT8_MAX : INT16_MAX;
    int64_t out_stride[8], n_out = 1, total = 1;
    for (int d = dims - 1; d >= 0; d--) {
        out_stride[d] = reduce_flag[d] ? 0 : n_out;
        if (!reduce_flag[d])
            n_out *= shape[d];
        total *= shape[d];
    }
    int64_t *acc = (int64_t *)malloc(sizeof(int64_t) * (size_t)(n_out > 0 ? n_out : 1));
    for (int64_t o = 0; o < n_out; o++)
        acc[o] = op == 0 ? lo : (op == 1 ? hi : 0);
    int32_t idx[8] = {0};
    for (int64_t i = 0; i < total; i++) {
        int64_t o = 0;
        for (int d = 0; d < dims; d++)
            o += idx[d] * out_stride[d];
        const int64_t v = bits == 8 ? ((const int8_t *)in)[i] : ((const int16_t *)in)[i];
        if (op == 0)
            acc[o] = v > acc[o] ? v : acc[o];
        else if (op == 1)
            acc[o] = v < acc[o] ? v : acc[o];
        else if (op == 2)
            acc[o] += v;
        else if (op == 3)
            acc[o] += v < 0 ? -v : v;
        else
            acc[o] += v * v;
        for (int d = dims - 1; d >= 0; d--) {
            if (++idx[d] < shape[d])
                break;
            idx[d] = 0;
        }
    }
    for (int64_t o = 0; o < n_out; o++) {
        int64_t r = acc[o];
        if (op >= 2) {
            r = bits == 8 ? (int64_t)espdl_oracle_shift_round_s32((int32_t)r, shift, round_mode)
                          : espdl_oracle_shift_round_s64(r, shift, round_mode);
            r = clamp_i64(r, lo, hi);
        }
        if (bits == 8)
            ((int8_t *)out)[o] = (int8_t)r;
        else
            ((int16_t *)out)[o] = (int16_t)r;
    }
    free(acc);
    return 0;
}

/*
 * Pad (TensorBase::pad, esp-dl/dl/tensor/src/dl_tensor_base.cpp:1225-1299; base::pad1D and pad_head_and_tail,
 * esp-dl/dl/base/dl_base_pad.cpp:19-64, 108-183): the innermost axis is padded row by row, then every outer axis
 * copies whole padded slabs, so each axis maps on its own.  mode 0 constant, 1 edge, 2 reflect.  Written here the
 * way the reference works, axis by axis from the innermost outwards on a growing buffer.
 */
void espdl_oracle_pad(const void *in, const int32_t *shape, int dims, const int32_t *pads, int mode, int32_t value,
                      int elem_size, void *out)
{
    int64_t cur_shape[8];
    int64_t total = 1;
    for (int d = 0; d < dims; d++) {
        cur_shape[d] = shape[d];
        total *= shape[d];
    }
    unsigned char *cur = (unsigned char *)malloc((size_t)(total > 0 ? total : 1) * elem_size);
    memcpy(cur, in, (size_t)total * elem_size);
    for (int axis = dims - 1; axis >= 0; axis--) {
        const int64_t before = pads[axis], after = pads[axis + dims], n = cur_shape[axis], m = n + before + after;
        int64_t outer = 1, inner = elem_size;
        for (int d = 0; d < axis; d++)
            outer *= cur_shape[d];
        for (int d = axis + 1; d < dims; d++)
            inner *= cur_shape[d];
        unsigned char *next = (unsigned char *)malloc((size_t)(outer * m * inner > 0 ? outer * m * inner : 1));
        for (int64_t o = 0; o < outer; o++) {
            const unsigned char *src = cur + o * n * inner;
            unsigned char *dst = next + o * m * inner;
            memcpy(dst + before * inner, src, (size_t)(n * inner));
            for (int64_t i = 0; i < before + after; i++) {
                const int64_t pos = i < before ? i : n + i;      /* position in the padded axis */
                unsigned char *line = dst + pos * inner;
                if (mode == 0) {
                    for (int64_t k = 0; k < inner; k += elem_size)
                        memcpy(line + k, &value, (size_t)elem_size); /* little endian: the low bytes */
                } else {
                    int64_t from;
                    if (mode == 1)
                        from = i < before ? 0 : n - 1;
                    else
                        from = i < before ? before - i : n - 2 - (i - before);
                    memcpy(line, src + from * inner, (size_t)inner);
                }
            }
        }
        free(cur);
        cur = next;
        cur_shape[axis] = m;
    }
    total = elem_size;
    for (int d = 0; d < dims; d++)
        total *= cur_shape[d];
    memcpy(out, cur, (size_t)total);
    free(cur);
}

/* Sub, int8 (c_impl_sub_n_n<int8_t>, esp-dl/dl/base/dl_base_sub.cpp:33-43): saturating integer subtraction. */
void espdl_oracle_sub_s8(const int8_t *in0, int64_t len0, const int8_t *in1, int64_t len1, int64_t size, int8_t *out)
{
    for (int64_t i = 0; i < size; i++) {
        const int32_t a = in0[len0 == 1 ? 0 : i], b = in1[len1 == 1 ? 0 : i];
        out[i] = (int8_t)clamp_i64(a - b, INT8_MIN, INT8_MAX);
    }
}

/*
 * Div, int8 (esp-dl/dl/base/dl_base_div.cpp:8-46, 66-70, 92-130, 141-175, 208-224).  The three loops are those
 * of the int16 form with int8 limits.  When an operand tensor has one element the reference reads a 256-entry
 * table instead (create_div_lut); this function builds that table the way the reference does and reads it
 * (table_operand: 0 no table, 1 the dividend is the one element, 2 the divisor is).  A one-element divisor of 0
 * makes the reference convert an infinity to int, which is undefined; here that entry follows the loop form
 * (the int8 extreme of the dividend's sign).  Operands are passed already broadcast to `size`.
 */
void espdl_oracle_div_s8(const int8_t *in0, const int8_t *in1, int64_t size, int shift, int form, int table_operand,
                         int8_t *out)
{
    const float rescale = dl_rescale(shift);
    if (table_operand && size > 0) {
        int8_t table[256];
        if (table_operand == 1) {
            const float in0_float = (float)in0[0] * rescale;
            for (int i = -128; i <= 127; i++) {
                if (i == 0)
                    table[i + 128] = in0_float > 0 ? INT8_MAX : INT8_MIN;
                else
                    table[i + 128] = (int8_t)clamp_i64(round_half_up_f32(in0_float / (float)i), INT8_MIN, INT8_MAX);
            }
            for (int64_t i = 0; i < size; i++)
                out[i] = table[in1[i] + 128];
        } else {
            if (in1[0] == 0) {
                for (int i = -128; i <= 127; i++)
                    table[i + 128] = i == 0 ? 0 : (i > 0 ? INT8_MAX : INT8_MIN);
            } else {
                const float scale = rescale / (float)in1[0];
                for (int i = -128; i <= 127; i++)
                    table[i + 128] =
                        i == 0 ? 0 : (int8_t)clamp_i64(round_half_up_f32((float)i * scale), INT8_MIN, INT8_MAX);
            }
            for (int64_t i = 0; i < size; i++)
                out[i] = table[in0[i] + 128];
        }
        return;
    }
    for (int64_t i = 0; i < size; i++) {
        const int8_t a = in0[i], b = in1[i];
        if (a == 0) {
            out[i] = 0;
        } else if (b == 0) {
            out[i] = a > 0 ? INT8_MAX : INT8_MIN;
        } else {
            float v;
            if (form == 1) {
                const float r = rescale / (float)b;
                v = (float)a * r;
            } else if (form == 2) {
                const float r = (float)a * rescale;
                v = r / (float)b;
            } else {
                v = (float)a * rescale / (float)b;
            }
            out[i] = (int8_t)clamp_i64(round_half_up_f32(v), INT8_MIN, INT8_MAX);
        }
    }
}

/*
 * The activation modules that compute in float32 per element: Sigmoid, Tanh, HardSwish, Elu, Exp, Log, Sqrt,
 * LeakyRelu, Swish, HardSigmoid, and the integer Neg.  All of them (int8 and int16 alike) are
 *     out = truncate(tool::round(f(q * DL_SCALE(in_exp)) * DL_RESCALE(out_exp)))
 * with f written exactly as the module writes it, float / double promotions included:
 *   sigmoid(x) = (float)(1.0 / (1.0 + expf(-x)))            esp-dl/dl/math/include/dl_math.hpp:200-203
 *   tanh(x)    = 2 * sigmoid(2 * x) - 1                      dl_math.hpp:205-208
 *   Sigmoid    dl_module_sigmoid.hpp:33-52                   Tanh       dl_module_tanh.hpp:47-66
 *   HardSwish  max(0, min(1, 0.166667 * x + 0.5)) * x in double, stored to float   dl_module_hard_swish.hpp:66-76
 *   Elu        x >= 0 ? x : alpha * (expf(x) - 1)            dl_module_elu.hpp:68-82
 *   Exp, Log, Sqrt   expf / logf / sqrtf                     dl_module_exp.hpp:62-72, _log.hpp:61-71, _sqrt.hpp:61-71
 *   LeakyRelu  x >= 0 ? x * rescale : x * rescale * alpha    dl_module_leaky_relu.hpp:74-87
 *   Swish      sigmoid(x) * x                                dl_module_swish.hpp:66-76
 *   HardSigmoid max(0, min(1, alpha * x + beta)) in float    dl_module_hard_sigmoid.hpp:74-84
 *   Neg        -q, the minimum maps to the maximum           dl_module_neg.hpp:57-86
 * tool::round is floorf(v + 0.5) in the portable build and round_half_even((double)v) in the ESP32-P4 build
 * (esp-dl/dl/tool/src/dl_tool.cpp:50-91).  Where f is not a number (Log or Sqrt of a negative input) or infinite
 * the reference converts it to int, which is undefined: this restatement gives 0 for NaN and saturates infinities.
 */
static int round_half_even_f64(double value)
{
    const double rounded = value < 0 ? value - 0.5 : value + 0.5;
    int int_part = (int)rounded;
    if (fabs(rounded - int_part) < 1e-6 && (int_part & 1) != 0)
        int_part += value < 0 ? 1 : -1;
    return int_part;
}

static float oracle_sigmoid(float x)
{
    return 1.0 / (1.0 + expf(-x));
}

static int64_t unary_value(int kind, int q, float in_scale, float out_scale, float alpha, float beta, int round_mode,
                           int lo, int hi)
{
    float temp = (float)q * in_scale, v;
    switch (kind) {
    case ESPDL_ORACLE_UNARY_SIGMOID:
        v = oracle_sigmoid(temp) * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_TANH:
        temp = 2 * oracle_sigmoid(2 * temp) - 1;
        v = temp * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_HARD_SWISH: {
        const double gate = 0.166667 * temp + 0.5;
        const double clipped = gate > 1 ? 1 : (gate < 0 ? 0 : gate);
        temp = clipped * temp;
        v = temp * out_scale;
        break;
    }
    case ESPDL_ORACLE_UNARY_ELU:
        v = temp >= 0 ? temp * out_scale : alpha * (expf(temp) - 1) * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_EXP:
        v = expf(temp) * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_LOG:
        v = logf(temp) * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_SQRT:
        v = sqrtf(temp) * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_LEAKY_RELU:
        v = temp >= 0 ? temp * out_scale : temp * out_scale * alpha;
        break;
    case ESPDL_ORACLE_UNARY_SWISH:
        temp = oracle_sigmoid(temp) * temp;
        v = temp * out_scale;
        break;
    case ESPDL_ORACLE_UNARY_HARD_SIGMOID: {
        const float gate = alpha * temp + beta;
        temp = gate > 1 ? 1 : (gate < 0 ? 0 : gate);
        v = temp * out_scale;
        break;
    }
    case ESPDL_ORACLE_UNARY_NEG:
        return q == lo ? hi : -q;
    default:
        return 0;
    }
    if (isnan(v))
        return 0;
    if (v >= 2147483520.f)
        return hi;
    if (v <= -2147483520.f)
        return lo;
    const int r = round_mode == ESPDL_ORACLE_ROUND_HALF_EVEN ? round_half_even_f64((double)v) : round_half_up_f32(v);
    return clamp_i64(r, lo, hi);
}

void espdl_oracle_unary_s8(int kind, const int8_t *in, int64_t size, int in_exp, int out_exp, float alpha, float beta,
                           int round_mode, int8_t *out)
{
    const float in_scale = dl_scale(in_exp), out_scale = dl_rescale(out_exp);
    for (int64_t i = 0; i < size; i++)
        out[i] = (int8_t)unary_value(kind, in[i], in_scale, out_scale, alpha, beta, round_mode, INT8_MIN, INT8_MAX);
}

void espdl_oracle_unary_s16(int kind, const int16_t *in, int64_t size, int in_exp, int out_exp, float alpha, float beta,
                            int round_mode, int16_t *out)
{
    const float in_scale = dl_scale(in_exp), out_scale = dl_rescale(out_exp);
    for (int64_t i = 0; i < size; i++)
        out[i] = (int16_t)unary_value(kind, in[i], in_scale, out_scale, alpha, beta, round_mode, INT16_MIN, INT16_MAX);
}

/* AveragePool, int16 (avgpool2d_hwc<int16_t, int32_t>, esp-dl/dl/base/dl_base_avg_pool2d.cpp:28-54, :87). */
void espdl_oracle_avg_pool_s16(const int16_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                               int stride_w, int pad_top, int pad_bottom, int pad_left, int pad_right, int in_exp,
                               int out_exp, int16_t *out)
{
    const int out_h = (h + pad_top + pad_bottom - k_h) / stride_h + 1;
    const int out_w = (w + pad_left + pad_right - k_w) / stride_w + 1;
    const float area_inv = 1.f / (float)(k_h * k_w);
    const float scale = dl_scale(in_exp) * area_inv * dl_rescale(out_exp);
    for (int n = 0; n < batch; n++)
        for (int oy = 0; oy < out_h; oy++)
            for (int ox = 0; ox < out_w; ox++)
                for (int k = 0; k < c; k++) {
                    int32_t sum = 0;
                    for (int ky = 0; ky < k_h; ky++) {
                        const int iy = oy * stride_h - pad_top + ky;
                        if (iy < 0 || iy >= h)
                            continue;
                        for (int kx = 0; kx < k_w; kx++) {
                            const int ix = ox * stride_w - pad_left + kx;
                            if (ix < 0 || ix >= w)
                                continue;
                            sum += in[(((int64_t)n * h + iy) * w + ix) * c + k];
                        }
                    }
                    out[(((int64_t)n * out_h + oy) * out_w + ox) * c + k] =
                        (int16_t)clamp_i64(round_half_up_f32((float)sum * scale), INT16_MIN, INT16_MAX);
                }
}

/* ReduceMean, int16 (reduce<int64_t, int16_t>, esp-dl/dl/module/include/dl_module_reduce_mean.hpp:18-45, :54-56). */
int espdl_oracle_reduce_mean_s16(const int16_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                 int out_exp, int16_t *out)
{
    if (dims < 1 || dims > 8)
        return -1;
    int64_t total = 1, count = 1;
    for (int i = 0; i < dims; i++) {
        total *= shape[i];
        if (reduce_flag[i])
            count *= shape[i];
    }
    if (total == 0)
        return 0;
    const int64_t n_out = total / count;
    int64_t *sums = (int64_t *)calloc((size_t)n_out, sizeof(int64_t));
    if (!sums)
        return -1;
    int64_t idx[8] = {0};
    for (int64_t e = 0; e < total; e++) {
        int64_t o = 0;
        for (int i = 0; i < dims; i++)
            if (!reduce_flag[i])
                o = o * shape[i] + idx[i];
        sums[o] += in[e];
        for (int i = dims - 1; i >= 0; i--) {
            if (++idx[i] < shape[i])
                break;
            idx[i] = 0;
        }
    }
    const float input_scale = dl_scale(in_exp), output_scale = dl_rescale(out_exp);
    for (int64_t o = 0; o < n_out; o++)
        out[o] = (int16_t)clamp_i64(round_half_up_f32((float)sums[o] * input_scale / (float)count * output_scale),
                                    INT16_MIN, INT16_MAX);
    free(sums);
    return 0;
}

/*
 * InsertZeros::forward_template (esp-dl/dl/module/include/dl_module_insert_zeros.hpp): the output is cleared,
 * then input pixel (h, w) is copied to output pixel (h * stride_h, w * stride_w).
 */
void espdl_oracle_insert_zeros(const void *in, int elem_size, int batch, int h, int w, int c, int stride_h, int stride_w,
                               int out_h, int out_w, void *out)
{
    const size_t px = (size_t)c * (size_t)elem_size;
    memset(out, 0, (size_t)batch * out_h * out_w * px);
    for (int n = 0; n < batch; n++)
        for (int y = 0; y < h; y++)
            for (int x = 0; x < w; x++)
                memcpy((char *)out + (((size_t)n * out_h + (size_t)y * stride_h) * out_w + (size_t)x * stride_w) * px,
                       (const char *)in + (((size_t)n * h + y) * w + x) * px, px);
}

/*
 * LUT on int16 (LUT::forward, esp-dl/dl/module/include/dl_module_lut.hpp:61-74, with
 * base::lut_s16_nearest_neighbor and lut_index, esp-dl/dl/base/dl_base_lut.cpp:49-77): the table holds
 * table_size = 65536 / step + 1 entries (step a power of two), or 65536 entries for step 1.  The input is
 * biased to 0..65535, divided by step and rounded to the nearest entry: ties go up on the portable C path
 * and to the even index when p4_ties is set (the ESP32-P4 build).
 */
int espdl_oracle_lut_s16(const int16_t *in, int64_t size, const int16_t *table, int table_size, int p4_ties,
                         int16_t *out)
{
    if (table_size < 2)
        return -1;
    const int step = 65536 / (table_size - 1);
    if (step < 1 || (step & (step - 1)) != 0)
        return -1;
    if (step == 1) {
        for (int64_t i = 0; i < size; i++)
            out[i] = table[(int)in[i] + 32768];
        return 0;
    }
    int shift = 0;
    while ((1 << shift) < step)
        shift++;
    for (int64_t i = 0; i < size; i++) {
        const uint32_t value = (uint32_t)(uint16_t)in[i] ^ 0x8000u;
        uint32_t index = value >> shift;
        const uint32_t remainder = value & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (p4_ties ? (remainder > half || (remainder == half && (index & 1u))) : (remainder >= half))
            index++;
        out[i] = table[index];
    }
    return 0;
}

/* ---------------------------------------------------------------------------------------------
 * Data-movement operators of the detection necks (Concat, Split, Transpose, Resize, MaxPool).
 * ------------------------------------------------------------------------------------------- */

/* Concat along an axis (esp-dl/dl/module/include/dl_module_concat.hpp:56-108): loop_times =
 * product of the dims before the axis; input j contributes copy_nums[j] = product of its dims
 * from the axis on, per loop.  elem_size in bytes. */
void espdl_oracle_concat(const void *const *inputs, int n_inputs, const int64_t *copy_nums, int64_t loop_times,
                         int elem_size, void *out)
{
    char *o = (char *)out;
    for (int64_t i = 0; i < loop_times; i++)
        for (int j = 0; j < n_inputs; j++) {
            const int64_t bytes = copy_nums[j] * elem_size;
            memcpy(o, (const char *)inputs[j] + i * bytes, (size_t)bytes);
            o += bytes;
        }
}

/* One output of Split (esp-dl/dl/module/include/dl_module_split.hpp:84-93): for each of the
 * num_slices outer positions copy out_axis * slice_size elements that start at element
 * (n * in_axis + slice_index) * slice_size. */
void espdl_oracle_split_slice(const void *in, int64_t slice_index, int64_t num_slices, int64_t slice_size,
                              int64_t in_axis, int64_t out_axis, int elem_size, void *out)
{
    for (int64_t n = 0; n < num_slices; n++) {
        const int64_t in_off = (n * in_axis + slice_index) * slice_size;
        const int64_t out_off = n * out_axis * slice_size;
        memcpy((char *)out + out_off * elem_size, (const char *)in + in_off * elem_size,
               (size_t)(slice_size * out_axis * elem_size));
    }
}

/* Transpose (esp-dl/dl/tensor/src/dl_tensor_base.cpp:722-812): out.shape[i] = in.shape[perm[i]],
 * out[index permuted] = in[index].  Up to 8 dims; perm entries already non-negative. */
int espdl_oracle_transpose(const void *in, const int *shape, int dims, const int *perm, int elem_size, void *out)
{
    if (dims < 1 || dims > 8)
        return -1;
    int64_t in_stride[8], out_stride[8], out_shape[8], total = 1;
    in_stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        in_stride[i] = in_stride[i + 1] * shape[i + 1];
    for (int i = 0; i < dims; i++) {
        if (perm[i] < 0 || perm[i] >= dims)
            return -1;
        out_shape[i] = shape[perm[i]];
        total *= shape[i];
    }
    out_stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        out_stride[i] = out_stride[i + 1] * out_shape[i + 1];
    int64_t idx[8] = {0};
    for (int64_t e = 0; e < total; e++) { /* e walks the input in memory order */
        int64_t o = 0;
        for (int i = 0; i < dims; i++)
            o += idx[perm[i]] * out_stride[i];
        memcpy((char *)out + o * elem_size, (const char *)in + e * elem_size, (size_t)elem_size);
        for (int i = dims - 1; i >= 0; i--) {
            if (++idx[i] < shape[i])
                break;
            idx[i] = 0;
        }
    }
    (void)in_stride;
    return 0;
}

/* Resize, nearest, int8 NHWC (esp-dl/dl/base/dl_base_resize.cpp:7-34 per pixel, :236-268 the
 * coordinate loops, esp-dl/dl/base/dl_base_resize.hpp:37-92 the arguments).  scale_h / scale_w are
 * the float32 scales of the module; the exact-2x path replicates each input pixel into a 2x2 block,
 * every other scale uses in = min((int)(out * (1 / scale)), len - 1) in float32 ("asymmetric").
 * Value: round((float)x * output_scale / (1 << output_shift)) with round = floorf(v + 0.5), stored
 * to int8 by C conversion (no saturation in the reference: wraps when the exponent shrinks). */
void espdl_oracle_resize_nearest_s8(const int8_t *in, int batch, int h, int w, int c, int out_h, int out_w,
                                    float scale_h, float scale_w, int in_exp, int out_exp, int8_t *out)
{
    int output_shift = out_exp - in_exp, output_scale = 1;
    if (output_shift < 0) {
        output_scale = 1 << (-output_shift);
        output_shift = 0;
    }
    const float scale_h_inv = 1 / scale_h, scale_w_inv = 1 / scale_w;
    const int exact2 = scale_h == 2 && scale_w == 2;
    for (int n = 0; n < batch; n++) {
        const int8_t *img = in + (int64_t)n * h * w * c;
        int8_t *oimg = out + (int64_t)n * out_h * out_w * c;
        for (int y = 0; y < out_h; y++) {
            int in_y = exact2 ? y / 2 : (int)(y * scale_h_inv);
            if (in_y > h - 1)
                in_y = h - 1;
            for (int x = 0; x < out_w; x++) {
                int in_x = exact2 ? x / 2 : (int)(x * scale_w_inv);
                if (in_x > w - 1)
                    in_x = w - 1;
                const int8_t *src = img + ((int64_t)in_y * w + in_x) * c;
                int8_t *dst = oimg + ((int64_t)y * out_w + x) * c;
                for (int k = 0; k < c; k++) {
                    const float v = (float)src[k] * (float)output_scale / (float)(1 << output_shift);
                    dst[k] = (int8_t)(int)floorf(v + 0.5f);
                }
            }
        }
    }
}

/* MaxPool, NHWC (esp-dl/dl/base/dl_base_max_pool2d.cpp:9-29 on the window clipped to the image as
 * the pool shell does; output size esp-dl/dl/module/include/dl_module_max_pool.hpp:42-49).  No
 * rescale: output exponent = input exponent.  elem_size 1 (int8) or 2 (int16). */
int espdl_oracle_max_pool(const void *in, int elem_size, int batch, int h, int w, int c, int k_h, int k_w,
                          int stride_h, int stride_w, int pad_top, int pad_bottom, int pad_left, int pad_right,
                          void *out)
{
    const int out_h = (h + pad_top + pad_bottom - k_h) / stride_h + 1;
    const int out_w = (w + pad_left + pad_right - k_w) / stride_w + 1;
    if (elem_size != 1 && elem_size != 2)
        return -1;
    for (int n = 0; n < batch; n++)
        for (int oy = 0; oy < out_h; oy++)
            for (int ox = 0; ox < out_w; ox++)
                for (int k = 0; k < c; k++) {
                    int best = 0, have = 0;
                    for (int ky = 0; ky < k_h; ky++) {
                        const int iy = oy * stride_h - pad_top + ky;
                        if (iy < 0 || iy >= h)
                            continue;
                        for (int kx = 0; kx < k_w; kx++) {
                            const int ix = ox * stride_w - pad_left + kx;
                            if (ix < 0 || ix >= w)
                                continue;
                            const int64_t off = (((int64_t)n * h + iy) * w + ix) * c + k;
                            const int v = elem_size == 1 ? ((const int8_t *)in)[off] : ((const int16_t *)in)[off];
                            if (!have || v > best)
                                best = v;
                            have = 1;
                        }
                    }
                    const int64_t ooff = (((int64_t)n * out_h + oy) * out_w + ox) * c + k;
                    if (elem_size == 1)
                        ((int8_t *)out)[ooff] = (int8_t)best;
                    else
                        ((int16_t *)out)[ooff] = (int16_t)best;
                }
    return 0;
}
