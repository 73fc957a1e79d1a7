/*
 * CPU oracle for ESP-DL's quantized operator path (portable C, non-PIE).
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's arithmetic, used
 * by tests/, by __graft_entry__.smoke() and by bench.py's cpu_baseline leg as the checker and the
 * timed CPU baseline.  Nothing in the shipped library links, loads or calls it.
 *
 * Conventions (as in the reference): activations NHWC, one image = one reference call (the
 * reference is batch-1; a batch of N is N independent images); conv filter memory is
 * [Cout][kH][kW][Cin] (esp-dl/dl/base/dl_base_conv2d.cpp:23,64,140), depthwise filter memory is
 * [kH][kW][C] (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:46-65); real = q * 2^exponent.
 *
 * Pinning status of each function (what fixes its behaviour besides re-reading the reference):
 *   espdl_oracle_shift_round_*   exhaustive comparison with floor(v/2^s + 1/2) in exact rationals
 *                                and the half-even ties table                            PINNED
 *   espdl_oracle_conv2d_s8       reference-held Gemm known answers (c target, 3 files) for the
 *                                1x1 path, N-major filter layout, bias-before-shift, rounding,
 *                                ReLU, saturation; brute force + padding/stride/dilation
 *                                invariants for the windowed path                         PINNED
 *   espdl_oracle_depthwise_s8    brute force; equality with a grouped conv written as a
 *                                block-diagonal espdl_oracle_conv2d_s8                    PINNED
 *   espdl_oracle_conv2d_s16 /
 *   espdl_oracle_depthwise_s16   brute force in arbitrary-precision integers              PINNED
 *   per-channel shift            by definition the per-tensor formula applied per output
 *                                channel (the reference C branch for it is dead code and the
 *                                shipping semantics live in ESP32-P4 assembly,
 *                                esp-dl/dl/base/isa/esp32p4/dl_esp32p4_s8.S:57-65); checked as
 *                                equality with per-tensor runs on single-channel slices   PINNED (to that definition)
 *   espdl_oracle_lut_s8          known-answer pattern of test_apps/dl_pie_func/main/test_lut.cpp:104-150,
 *                                identity table                                           PINNED
 *   espdl_oracle_prelu_s8, _relu_s8, _add_s8   exhaustive over all int8 operand pairs against
 *                                closed forms in exact integers                           PINNED
 *   espdl_oracle_clip_s8, _relu_s8 (exponent change), _requantize_s8   float32-defined in the reference
 *                                (floorf(x * 2^k + 0.5)); for int8/int16 x and power-of-two
 *                                scales every intermediate is exactly representable, so the
 *                                result is fixed by the mathematics: checked exhaustively
 *                                against round-half-up in exact rationals                 PINNED
 *   espdl_oracle_global_avg_pool_s8, _avg_pool_s8, _avg_pool_s16   float32-defined in the reference:
 *                                (DL_SCALE(in) * (1.f / area)) * DL_RESCALE(out), one multiply of float(sum),
 *                                tool::round.  Every reachable int8 sum for areas 49, 9, 6, 4, 2, 100, 196, 5 (a
 *                                dense sample plus all tie multiples for int16) x twelve exponent pairs, ties and
 *                                near-ties included, against the same IEEE float32 sequence replayed operation by
 *                                operation with numpy scalars, and against round-half-up in exact rationals (no
 *                                enumerated sum differs between the two).  The reference itself cannot be built
 *                                here (every translation unit needs ESP-IDF headers that are absent); it is
 *                                compiled with -ffast-math, which for int8 can only matter on exact ties of areas
 *                                that are not powers of two, where the order as written is followed   PINNED
 *   espdl_oracle_mul_s8          exhaustive over all int8 operand pairs and shifts -4..14 against round-half-up
 *                                (and the half-even table) of the exact product in rationals        PINNED
 *   espdl_oracle_reduce_mean_s8, _s16   ((float(sum) * DL_SCALE(in)) / float(count)) * DL_RESCALE(out): every
 *                                reachable int8 sum for counts 49, 9, 6, 4, 2, 100, 40, 3 (dense + tie multiples
 *                                for int16) against the numpy float32 replay and exact rationals, as above; the
 *                                reference's streaming-model fixtures pass through AveragePool        PINNED
 *   espdl_oracle_slice           equality with numpy basic slicing                                   PINNED
 *   espdl_oracle_softmax_s8      float32: within 2e-6 relative of scipy.special.softmax of the dequantized values;
 *                                the order-sensitive part (the float32 row sum in index order, one IEEE division
 *                                per element) bit for bit against numpy.cumsum / numpy division on the table the
 *                                host C library's expf gives.  The device the reference targets computes that
 *                                table with its own libm (newlib), whose expf may differ from glibc's in the last
 *                                place, so against that device the claim is the tolerance, not the bits
 *                                                                                   PINNED (to float32 tolerance)
 *   espdl_oracle_quantize_f32, _dequantize_f32   exact rational round-half-up of v * 2^-e incl. ties and the
 *                                saturation edges; exact scaling                                     PINNED
 *   matmul_s8 (espdl_oracle.py)  built from espdl_oracle_conv2d_s8 exactly as the reference builds it from
 *                                base::conv2d; checked against numpy integer matmul with broadcasting followed by
 *                                the pinned shift-round, and against the transposed-operand mistake   PINNED
 *   espdl_oracle_lut_s16         all 65536 inputs against round((x + 32768) / step) in exact rationals for both tie
 *                                rules and five table sizes                                          PINNED
 *   espdl_oracle_insert_zeros    equality with numpy strided assignment into zeros                   PINNED
 *   espdl_oracle_add_s16         numpy saturating add                                               PINNED
 *   espdl_oracle_mul_s16         numpy: int64 product -> float32 (round to nearest even) -> exact power-of-two
 *                                scaling -> exact rational round half up; half-even mode against the pinned
 *                                integer shift-round                                                  PINNED
 *   espdl_oracle_sub_s16         numpy saturating subtraction                                        PINNED
 *   espdl_oracle_div_s16         numpy float32 arithmetic in the same order for each of the three forms (IEEE
 *                                operations, so the order is the whole content), and within one unit of the exact
 *                                rational quotient                                                   PINNED
 *   espdl_oracle_unary_s8, _s16  every table entry (256 / 65536) of every function against the reference's
 *                                float / double sequence replayed with numpy scalars of the same widths and the
 *                                host C library's expf / logf / sqrtf, and against the float64 closed form rounded
 *                                half up on every entry that is not within 4 float32 ulps of a tie.  int8: no entry
 *                                of a libm-dependent function is that close to a tie, so any C library decides the
 *                                same table.  int16: 123 to 4012 of 65536 entries per libm-dependent function are
 *                                (counted in tests/test_oracle_float_pins.py); on those a C library that differs
 *                                from this host's in the last places of expf / logf could move the entry by one
 *                                unit, which no restatement can settle             PINNED (int16: to the host libm)
 *   espdl_oracle_reduce_int      numpy max / min / sum over the same axes; the sum followed by the pinned
 *                                shift-round and saturation                                          PINNED
 *   espdl_oracle_pad             equality with numpy.pad (constant / edge / reflect) on random shapes, ranks 1-5,
 *                                all three element sizes                                             PINNED
 *   espdl_oracle_sub_s8          numpy saturating subtraction                                        PINNED
 *   espdl_oracle_div_s8          as _div_s16 for the three loop forms; the table forms against a table built in
 *                                numpy float32 from the reference's two expressions, entry by entry   PINNED
 *   espdl_oracle_concat, _split_slice, _transpose   pure copies: equality with numpy.concatenate /
 *                                numpy.split / numpy.transpose on random shapes           PINNED
 *   espdl_oracle_max_pool        equality with scipy.ndimage.maximum_filter (minimum-value border)
 *                                sampled at the window centres, and brute force            PINNED
 *   espdl_oracle_resize_nearest_s8   coordinates: numpy.repeat for integer scales, exact rational
 *                                floor(o / scale) for the others where float32 is exact; values:
 *                                the already pinned round-half-up shift for a growing exponent,
 *                                x * 2^k wrapped to int8 for a shrinking one               PINNED
 */
#ifndef ESPDL_ORACLE_H
#define ESPDL_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { ESPDL_ORACLE_ROUND_HALF_UP = 0, ESPDL_ORACLE_ROUND_HALF_EVEN = 1 };
enum { ESPDL_ORACLE_LINEAR = 0, ESPDL_ORACLE_RELU = 1 };

/* Geometry of one convolution; shared by the s8/s16, dense/depthwise entry points. */
typedef struct {
    int batch, in_h, in_w, in_c; /* input  [batch][in_h][in_w][in_c]                      */
    int out_c;                   /* dense: filters; depthwise: must equal in_c            */
    int k_h, k_w;
    int stride_h, stride_w;
    int dil_h, dil_w;
    int pad_top, pad_bottom, pad_left, pad_right;
    int activation; /* ESPDL_ORACLE_LINEAR / ESPDL_ORACLE_RELU                            */
    int round_mode; /* ESPDL_ORACLE_ROUND_HALF_UP is the portable C path                   */
    int n_shift;    /* 1 = per-tensor, out_c = one shift per output channel               */
} espdl_oracle_conv_t;

int32_t espdl_oracle_shift_round_s32(int32_t value, int shift, int round_mode);
int64_t espdl_oracle_shift_round_s64(int64_t value, int shift, int round_mode);

int espdl_oracle_conv_out_h(const espdl_oracle_conv_t *g);
int espdl_oracle_conv_out_w(const espdl_oracle_conv_t *g);

/* bias may be NULL.  shift[i] = out_exp - filter_exp[i] - in_exp.  Returns 0, or -1 on bad geometry. */
int espdl_oracle_conv2d_s8(const espdl_oracle_conv_t *g, const int8_t *in, const int8_t *filter,
                           const int32_t *bias, const int32_t *shift, int8_t *out);
int espdl_oracle_depthwise_s8(const espdl_oracle_conv_t *g, const int8_t *in, const int8_t *filter,
                              const int32_t *bias, const int32_t *shift, int8_t *out);
int espdl_oracle_conv2d_s16(const espdl_oracle_conv_t *g, const int16_t *in, const int16_t *filter,
                            const int64_t *bias, const int32_t *shift, int16_t *out);
int espdl_oracle_depthwise_s16(const espdl_oracle_conv_t *g, const int16_t *in, const int16_t *filter,
                               const int64_t *bias, const int32_t *shift, int16_t *out);

void espdl_oracle_lut_s8(const int8_t *in, int64_t size, const int8_t *table, int8_t *out);
/* alpha has `channels` entries; shift = out_exp - in_exp - alpha_exp. */
void espdl_oracle_prelu_s8(const int8_t *in, int64_t pixels, int channels, const int8_t *alpha, int shift,
                           int8_t *out);
void espdl_oracle_relu_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out);
void espdl_oracle_clip_s8(const int8_t *in, int64_t size, int min_q, int max_q, int in_exp, int out_exp,
                          int8_t *out);
/* Broadcast add: len0 / len1 are `size` or 1 (scalar operand). */
void espdl_oracle_add_s8(const int8_t *in0, int64_t len0, const int8_t *in1, int64_t len1, int64_t size,
                         int8_t *out);
/* shift = out_exp - in0_exp - in1_exp; operands broadcast as in espdl_oracle_add_s8. */
void espdl_oracle_mul_s8(const int8_t *in0, int64_t len0, const int8_t *in1, int64_t len1, int64_t size, int shift,
                         int round_mode, int8_t *out);
void espdl_oracle_global_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int in_exp, int out_exp,
                                     int8_t *out);
void espdl_oracle_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                              int stride_w, int pad_top, int pad_bottom, int pad_left, int pad_right, int in_exp,
                              int out_exp, int8_t *out);
int espdl_oracle_reduce_mean_s8(const int8_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                int out_exp, int8_t *out);
int espdl_oracle_slice(const void *in, const int *shape, int dims, const int *start, const int *step,
                       const int *out_shape, int elem_size, void *out);
void espdl_oracle_requantize_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out);
void espdl_oracle_add_s16(const int16_t *in0, int64_t len0, const int16_t *in1, int64_t len1, int64_t size,
                          int16_t *out);
void espdl_oracle_mul_s16(const int16_t *in0, int64_t len0, const int16_t *in1, int64_t len1, int64_t size, int shift,
                          int round_mode, int16_t *out);
void espdl_oracle_sub_s16(const int16_t *in0, int64_t len0, const int16_t *in1, int64_t len1, int64_t size,
                          int16_t *out);
void espdl_oracle_div_s16(const int16_t *in0, const int16_t *in1, int64_t size, int shift, int form, int16_t *out);
enum {
    ESPDL_ORACLE_UNARY_SIGMOID = 0,
    ESPDL_ORACLE_UNARY_TANH = 1,
    ESPDL_ORACLE_UNARY_HARD_SWISH = 2,
    ESPDL_ORACLE_UNARY_ELU = 3,
    ESPDL_ORACLE_UNARY_EXP = 4,
    ESPDL_ORACLE_UNARY_LOG = 5,
    ESPDL_ORACLE_UNARY_SQRT = 6,
    ESPDL_ORACLE_UNARY_LEAKY_RELU = 7,
    ESPDL_ORACLE_UNARY_NEG = 8,
    ESPDL_ORACLE_UNARY_SWISH = 9,
    ESPDL_ORACLE_UNARY_HARD_SIGMOID = 10
};
void espdl_oracle_unary_s8(int kind, const int8_t *in, int64_t size, int in_exp, int out_exp, float alpha, float beta,
                           int round_mode, int8_t *out);
void espdl_oracle_unary_s16(int kind, const int16_t *in, int64_t size, int in_exp, int out_exp, float alpha, float beta,
                            int round_mode, int16_t *out);
int espdl_oracle_reduce_int(const void *in, int bits, const int32_t *shape, int dims, const int32_t *reduce_flag, int op,
                            int shift, int round_mode, void *out);
void espdl_oracle_pad(const void *in, const int32_t *shape, int dims, const int32_t *pads, int mode, int32_t value,
                      int elem_size, void *out);
void espdl_oracle_sub_s8(const int8_t *in0, int64_t len0, const int8_t *in1, int64_t len1, int64_t size, int8_t *out);
void espdl_oracle_div_s8(const int8_t *in0, const int8_t *in1, int64_t size, int shift, int form, int table_operand,
                         int8_t *out);
void espdl_oracle_avg_pool_s16(const int16_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                               int stride_w, int pad_top, int pad_bottom, int pad_left, int pad_right, int in_exp,
                               int out_exp, int16_t *out);
int espdl_oracle_reduce_mean_s16(const int16_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                 int out_exp, int16_t *out);
void espdl_oracle_insert_zeros(const void *in, int elem_size, int batch, int h, int w, int c, int stride_h, int stride_w,
                               int out_h, int out_w, void *out);
int espdl_oracle_lut_s16(const int16_t *in, int64_t size, const int16_t *table, int table_size, int p4_ties,
                         int16_t *out);
void espdl_oracle_softmax_s8(const int8_t *in, int64_t outer, int64_t len, int64_t inner, int in_exp, float *out);
void espdl_oracle_quantize_f32(const float *in, int64_t size, int out_exp, int elem_size, void *out);
void espdl_oracle_dequantize_f32(const void *in, int64_t size, int in_exp, int elem_size, float *out);

/* Data-movement operators (see the .c file for the reference lines each one follows). */
void espdl_oracle_concat(const void *const *inputs, int n_inputs, const int64_t *copy_nums, int64_t loop_times,
                         int elem_size, void *out);
void espdl_oracle_split_slice(const void *in, int64_t slice_index, int64_t num_slices, int64_t slice_size,
                              int64_t in_axis, int64_t out_axis, int elem_size, void *out);
int espdl_oracle_transpose(const void *in, const int *shape, int dims, const int *perm, int elem_size, void *out);
void espdl_oracle_resize_nearest_s8(const int8_t *in, int batch, int h, int w, int c, int out_h, int out_w,
                                    float scale_h, float scale_w, int in_exp, int out_exp, int8_t *out);
int espdl_oracle_max_pool(const void *in, int elem_size, int batch, int h, int w, int c, int k_h, int k_w,
                          int stride_h, int stride_w, int pad_top, int pad_bottom, int pad_left, int pad_right,
                          void *out);

/* Number of worker threads the batch loops use (1 unless built with OpenMP). */
int espdl_oracle_max_threads(void);
void espdl_oracle_set_threads(int n);

#ifdef __cplusplus
}
#endif
#endif
