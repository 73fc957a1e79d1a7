// int16 forms of Add, Mul, AveragePool and ReduceMean, and Sub / Div for int8 and int16, for gfx950.  They serve
// the int16 heads and the int16 text recognizer of the reference's model files: small tensors, so one element per
// lane and plain loops.
//
// Add: c_impl_add_n_n<int16_t> (esp-dl/dl/base/dl_base_add.cpp:33-44), saturating integer add.
// Mul: c_impl_mul_n_n<int16_t> (esp-dl/dl/base/dl_base_mul.cpp:33-46): the int32 product goes through
//      float32, is scaled by 2^-shift and rounded half up; with ESP32-P4 semantics the exact product is
//      shifted and rounded half to even.
// Sub: c_impl_sub_n_n<feature_t> (esp-dl/dl/base/dl_base_sub.cpp:33-43).  Div: esp-dl/dl/base/dl_base_div.cpp, float32;
//      the int8 form with a single-element operand goes through a 256-entry table there (create_div_lut, :8-46),
//      whose entries are the same float32 expressions except for 0 / 0 with a single-element dividend (-128).
// AveragePool: avgpool2d_hwc<int16_t, int32_t> (esp-dl/dl/base/dl_base_avg_pool2d.cpp:28-54).
// ReduceMean: reduce<int64_t, int16_t> (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:18-56).
#include "espdl_device.h"
#include "espdl_kernels.h"
#include "binary_vec.h"
#include "reduce_mid.h"

namespace espdl {
namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ int clamp_s16(int v)
{
    return min(max(v, -32768), 32767);
}

template <typename T>
struct BinaryArgs {
    const T *in0, *in1;
    T *out;
    int dims[4];
    long long s0[4], s1[4];
    long long total;
    int shift, half_even, zero_by_zero;
    float rescale;
};

// OP: 0 add, 1 mul, 2 sub, 3 div.  Add and Mul are instantiated for int16 only (int8 has kernels of its own).
template <typename T, int OP>
__global__ __launch_bounds__(kThreads) void binary_kernel(const BinaryArgs<T> a)
{
    constexpr int lo = sizeof(T) == 1 ? -128 : -32768, hi = sizeof(T) == 1 ? 127 : 32767;
    for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < a.total; i += (long long)gridDim.x * kThreads) {
        long long rem = i, o0 = 0, o1 = 0;
#pragma unroll
        for (int d = 3; d >= 0; d--) {
            const long long q = rem / a.dims[d];
            const long long idx = rem - q * a.dims[d];
            o0 += idx * a.s0[d];
            o1 += idx * a.s1[d];
            rem = q;
        }
        const int x = a.in0[o0], y = a.in1[o1];
        int r;
        if (OP == 3) {
            // c_impl_div_n_n / _n_1 / _1_n (esp-dl/dl/base/dl_base_div.cpp:92-112, 141-163, 175-195): float32, the
            // order of the two operations depends on which operand is constant along the innermost axis
            if (x == 0) {
                r = y == 0 ? a.zero_by_zero : 0;
            } else if (y == 0) {
                r = x > 0 ? hi : lo;
            } else {
                float v;
                if (a.shift == 1) {
                    const float q = a.rescale / (float)y;
                    v = (float)x * q;
                } else if (a.shift == 2) {
                    const float q = (float)x * a.rescale;
                    v = q / (float)y;
                } else {
                    v = (float)x * a.rescale / (float)y;
                }
                r = min(max(round_half_up_f32(v), lo), hi);
            }
        } else if (OP == 2) {
            r = min(max(x - y, lo), hi);
        } else if (OP == 1) {
            const int prod = x * y; // at most 2^30 in magnitude
            if (a.half_even && a.shift > 0) {
                const long long q = (long long)prod >> a.shift;
                const long long frac = (long long)prod & ((1ll << a.shift) - 1), half = 1ll << (a.shift - 1);
                r = (int)min(max(q + ((frac > half || (frac == half && (q & 1))) ? 1 : 0), -32768ll), 32767ll);
            } else {
                r = clamp_s16(round_half_up_f32((float)prod * a.rescale));
            }
        } else {
            r = clamp_s16(x + y);
        }
        a.out[i] = (T)r;
    }
}

struct Pool16Args {
    const int16_t *in;
    int16_t *out;
    int h, w, c, out_h, out_w, k_h, k_w, stride_h, stride_w, pad_top, pad_left;
    long long total;
    float scale;
};

__global__ __launch_bounds__(kThreads) void avg_pool_s16_kernel(const Pool16Args a)
{
    for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < a.total; i += (long long)gridDim.x * kThreads) {
        const long long pix = i / a.c;
        const int ch = (int)(i - pix * a.c);
        const long long row = pix / a.out_w;
        const int x = (int)(pix - row * a.out_w);
        const long long n = row / a.out_h;
        const int y = (int)(row - n * a.out_h);
        const int iy0 = y * a.stride_h - a.pad_top, ix0 = x * a.stride_w - a.pad_left;
        int sum = 0;
        for (int ky = max(0, -iy0); ky < min(a.k_h, a.h - iy0); ky++)
            for (int kx = max(0, -ix0); kx < min(a.k_w, a.w - ix0); kx++)
                sum += a.in[((n * a.h + iy0 + ky) * a.w + ix0 + kx) * a.c + ch];
        a.out[i] = (int16_t)clamp_s16(round_half_up_f32((float)sum * a.scale));
    }
}

struct Reduce16Args {
    const int16_t *in;
    int16_t *out;
    int n_kept, n_red;
    int kept_shape[8], red_shape[8];
    long long kept_stride[8], red_stride[8];
    long long n_out, count;
    float input_scale, output_scale;
};

__global__ __launch_bounds__(kThreads) void reduce_mean_s16_kernel(const Reduce16Args a)
{
    for (long long o = (long long)blockIdx.x * kThreads + threadIdx.x; o < a.n_out; o += (long long)gridDim.x * kThreads) {
        long long rem = o, base = 0;
        for (int d = a.n_kept - 1; d >= 0; d--) {
            const long long q = rem / a.kept_shape[d];
            base += (rem - q * a.kept_shape[d]) * a.kept_stride[d];
            rem = q;
        }
        long long sum = 0;
        for (long long r = 0; r < a.count; r++) {
            long long rr = r, off = base;
            for (int d = a.n_red - 1; d >= 0; d--) {
                const long long q = rr / a.red_shape[d];
                off += (rr - q * a.red_shape[d]) * a.red_stride[d];
                rr = q;
            }
            sum += a.in[off];
        }
        const float v = (float)sum * a.input_scale / (float)a.count * a.output_scale;
        a.out[o] = (int16_t)clamp_s16(round_half_up_f32(v));
    }
}

// ReduceMax / ReduceMin / ReduceSum (esp-dl/dl/module/include/dl_module_reduce_max.hpp:14-52,
// dl_module_reduce_min.hpp:15-53, dl_module_reduce_sum.hpp:13-56): max and min return the stored integer, the sum
// (int32 for int8, int64 for int16) goes through shift_and_round(sum, out_exp - in_exp) and truncate.  ReduceL1 and
// ReduceSumSquare (dl_module_reduce_l1.hpp:14-50, dl_module_reduce_sum_square.hpp:14-46) sum |x| and x * x the same way.
template <typename T>
struct ReduceIntArgs {
    const T *in;
    T *out;
    int n_kept, n_red;
    int kept_shape[8], red_shape[8];
    long long kept_stride[8], red_stride[8];
    long long n_out, count;
    int shift, half_even;
};

// OP: 0 max, 1 min, 2 sum, 3 sum of magnitudes (ReduceL1), 4 sum of squares (ReduceSumSquare)
template <typename T, int OP>
__global__ __launch_bounds__(kThreads) void reduce_int_kernel(const ReduceIntArgs<T> a)
{
    constexpr int lo = sizeof(T) == 1 ? -128 : -32768, hi = sizeof(T) == 1 ? 127 : 32767;
    for (long long o = (long long)blockIdx.x * kThreads + threadIdx.x; o < a.n_out; o += (long long)gridDim.x * kThreads) {
        long long rem = o, base = 0;
        for (int d = a.n_kept - 1; d >= 0; d--) {
            const long long q = rem / a.kept_shape[d];
            base += (rem - q * a.kept_shape[d]) * a.kept_stride[d];
            rem = q;
        }
        long long acc = OP == 0 ? lo : (OP == 1 ? hi : 0);
        for (long long r = 0; r < a.count; r++) {
            long long rr = r, off = base;
            for (int d = a.n_red - 1; d >= 0; d--) {
                const long long q = rr / a.red_shape[d];
                off += (rr - q * a.red_shape[d]) * a.red_stride[d];
                rr = q;
            }
            const long long v = a.in[off];
            acc = OP == 0 ? max(acc, v) : (OP == 1 ? min(acc, v) : (OP == 2 ? acc + v : (OP == 3 ? acc + (v < 0 ? -v : v) : acc + v * v)));
        }
        if (OP >= 2)
            acc = sizeof(T) == 1 ? requant_s8((int)acc, a.shift, false, a.half_even)
                                 : requant_s16(acc, a.shift, false, a.half_even);
        a.out[o] = (T)acc;
    }
}

unsigned blocks_for(long long total, int cu_count)
{
    return (unsigned)max(1ll, min((total + kThreads - 1) / kThreads, (long long)max(1, cu_count) * 16));
}

} // namespace

namespace {

// The element operations of binary_kernel as functors for the 16-bytes-per-thread form (Div stays element-wise).
struct Add16 {
    __device__ __forceinline__ int apply(int x, int y) const { return clamp_s16(x + y); }
};
template <typename T>
struct SubOp {
    __device__ __forceinline__ int apply(int x, int y) const
    {
        constexpr int lo = sizeof(T) == 1 ? -128 : -32768, hi = sizeof(T) == 1 ? 127 : 32767;
        return min(max(x - y, lo), hi);
    }
};
struct Mul16 {
    int shift, half_even;
    float rescale;
    __device__ __forceinline__ int apply(int x, int y) const
    {
        const int prod = x * y; // at most 2^30 in magnitude
        if (half_even && shift > 0) {
            const long long q = (long long)prod >> shift;
            const long long frac = (long long)prod & ((1ll << shift) - 1), half = 1ll << (shift - 1);
            return (int)min(max(q + ((frac > half || (frac == half && (q & 1))) ? 1 : 0), -32768ll), 32767ll);
        }
        return clamp_s16(round_half_up_f32((float)prod * rescale));
    }
};

template <typename T>
hipError_t launch_binary(int op, const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const T *in0, const T *in1,
                         int shift, bool half_even, T *out, int cu_count, hipStream_t stream)
{
    if (binary_vec::Args va; op != 3 && binary_vec::plan(dims, s0, s1, in0, in1, out, &va)) {
        if (op == 2)
            return binary_vec::launch(in0, in1, out, va, SubOp<T>{}, cu_count, stream);
        if constexpr (sizeof(T) == 2) {
            if (op == 1)
                return binary_vec::launch(in0, in1, out, va, Mul16{shift, half_even ? 1 : 0, dl_rescale(shift)}, cu_count, stream);
            return binary_vec::launch(in0, in1, out, va, Add16{}, cu_count, stream);
        }
    }
    BinaryArgs<T> a = {};
    a.in0 = in0;
    a.in1 = in1;
    a.out = out;
    a.total = 1;
    for (int i = 0; i < 4; i++) {
        a.dims[i] = dims[i];
        a.s0[i] = s0[i];
        a.s1[i] = s1[i];
        a.total *= dims[i];
    }
    if (a.total <= 0)
        return hipSuccess;
    a.shift = shift;
    a.half_even = half_even;
    a.rescale = dl_rescale(shift);
    const dim3 grid(blocks_for(a.total, cu_count));
    if (op == 3) {
        // the loop form: 1 = divisor constant along the innermost axis longer than 1, 2 = dividend constant.  With
        // every axis of length 1 the reference tests the divisor first for int16 (dl_base_div.cpp:248-252) and the
        // dividend first for int8 (:212-224).
        int form = sizeof(T) == 1 ? 2 : 1;
        bool single_dividend = true;
        for (int d = 3; d >= 0; d--)
            if (dims[d] > 1) {
                form = s1[d] == 0 ? 1 : (s0[d] == 0 ? 2 : 0);
                break;
            }
        for (int d = 0; d < 4; d++)
            single_dividend = single_dividend && (dims[d] == 1 || s0[d] == 0);
        a.shift = form;
        // int8, one-element dividend: entry 128 of the reference's table (dl_base_div.cpp:19-24) is -128 for 0 / 0
        a.zero_by_zero = (sizeof(T) == 1 && single_dividend) ? -128 : 0;
        binary_kernel<T, 3><<<grid, dim3(kThreads), 0, stream>>>(a);
    } else if (op == 2) {
        binary_kernel<T, 2><<<grid, dim3(kThreads), 0, stream>>>(a);
    } else if constexpr (sizeof(T) == 2) {
        if (op == 1)
            binary_kernel<T, 1><<<grid, dim3(kThreads), 0, stream>>>(a);
        else
            binary_kernel<T, 0><<<grid, dim3(kThreads), 0, stream>>>(a);
    } else {
        return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

} // namespace

hipError_t launch_binary_s16(int op, const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int16_t *in0,
                             const int16_t *in1, int shift, bool half_even, int16_t *out, int cu_count, hipStream_t stream)
{
    return launch_binary<int16_t>(op, dims, s0, s1, in0, in1, shift, half_even, out, cu_count, stream);
}

hipError_t launch_subdiv_s8(bool div, const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                            const int8_t *in1, int shift, int8_t *out, int cu_count, hipStream_t stream)
{
    return launch_binary<int8_t>(div ? 3 : 2, dims, s0, s1, in0, in1, shift, false, out, cu_count, stream);
}

hipError_t launch_avg_pool_s16(const int16_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                               int stride_w, int pad_top, int pad_left, int out_h, int out_w, int in_exp, int out_exp,
                               int16_t *out, int cu_count, hipStream_t stream)
{
    Pool16Args a = {};
    a.in = in;
    a.out = out;
    a.h = h;
    a.w = w;
    a.c = c;
    a.out_h = out_h;
    a.out_w = out_w;
    a.k_h = k_h;
    a.k_w = k_w;
    a.stride_h = stride_h;
    a.stride_w = stride_w;
    a.pad_top = pad_top;
    a.pad_left = pad_left;
    a.total = (long long)batch * out_h * out_w * c;
    if (a.total <= 0)
        return hipSuccess;
    const float area_inv = 1.f / (float)(k_h * k_w);
    a.scale = dl_scale(in_exp) * area_inv * dl_rescale(out_exp);
    avg_pool_s16_kernel<<<dim3(blocks_for(a.total, cu_count)), dim3(kThreads), 0, stream>>>(a);
    return hipGetLastError();
}

namespace {
// ReduceMean's float expression on the integer sum, left to right as in the reference
struct MeanFinish16 {
    int16_t *out;
    float input_scale, count, output_scale;
    __device__ void operator()(long long o, int total) const
    {
        out[o] = (int16_t)clamp_s16(round_half_up_f32((float)total * input_scale / count * output_scale));
    }
};
} // namespace

hipError_t launch_reduce_mean_s16(const int16_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                  int out_exp, int16_t *out, int cu_count, hipStream_t stream)
{
    Reduce16Args a = {};
    a.in = in;
    a.out = out;
    long long stride[8];
    stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        stride[i] = stride[i + 1] * shape[i + 1];
    a.n_out = 1;
    a.count = 1;
    for (int i = 0; i < dims; i++) {
        if (reduce_flag[i]) {
            a.red_shape[a.n_red] = shape[i];
            a.red_stride[a.n_red++] = stride[i];
            a.count *= shape[i];
        } else {
            a.kept_shape[a.n_kept] = shape[i];
            a.kept_stride[a.n_kept++] = stride[i];
            a.n_out *= shape[i];
        }
    }
    if (a.n_out <= 0 || a.count <= 0)
        return hipSuccess;
    a.input_scale = dl_scale(in_exp);
    a.output_scale = dl_rescale(out_exp);
    // the reduced axes are neighbours and the sum fits int32: contiguous loads, every lane busy
    long long outer, r_count, inner;
    if (reduce_mid::mid_view(shape, dims, reduce_flag, &outer, &r_count, &inner) && r_count >= 8 &&
        reduce_mid::fits<int16_t>(outer, r_count, inner))
        return reduce_mid::launch(in, outer, r_count, inner, MeanFinish16{out, a.input_scale, (float)a.count, a.output_scale}, stream);
    reduce_mean_s16_kernel<<<dim3(blocks_for(a.n_out, cu_count)), dim3(kThreads), 0, stream>>>(a);
    return hipGetLastError();
}

namespace {

template <typename T>
hipError_t launch_reduce_int_t(const T *in, const int *shape, int dims, const int *reduce_flag, int op, int shift,
                               bool half_even, T *out, int cu_count, hipStream_t stream)
{
    ReduceIntArgs<T> a = {};
    a.in = in;
    a.out = out;
    long long stride[8];
    stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        stride[i] = stride[i + 1] * shape[i + 1];
    a.n_out = 1;
    a.count = 1;
    for (int i = 0; i < dims; i++) {
        if (reduce_flag[i]) {
            a.red_shape[a.n_red] = shape[i];
            a.red_stride[a.n_red++] = stride[i];
            a.count *= shape[i];
        } else {
            a.kept_shape[a.n_kept] = shape[i];
            a.kept_stride[a.n_kept++] = stride[i];
            a.n_out *= shape[i];
        }
    }
    if (a.n_out <= 0)
        return hipSuccess;
    a.shift = shift;
    a.half_even = half_even;
    const dim3 grid(blocks_for(a.n_out, cu_count)), block(kThreads);
    if (op == 0)
        reduce_int_kernel<T, 0><<<grid, block, 0, stream>>>(a);
    else if (op == 1)
        reduce_int_kernel<T, 1><<<grid, block, 0, stream>>>(a);
    else if (op == 2)
        reduce_int_kernel<T, 2><<<grid, block, 0, stream>>>(a);
    else if (op == 3)
        reduce_int_kernel<T, 3><<<grid, block, 0, stream>>>(a);
    else
        reduce_int_kernel<T, 4><<<grid, block, 0, stream>>>(a);
    return hipGetLastError();
}

} // namespace

hipError_t launch_reduce_int(const void *in, int bits, const int *shape, int dims, const int *reduce_flag, int op,
                             int shift, bool half_even, void *out, int cu_count, hipStream_t stream)
{
    if (bits == 8)
        return launch_reduce_int_t<int8_t>(static_cast<const int8_t *>(in), shape, dims, reduce_flag, op, shift, half_even,
                                           static_cast<int8_t *>(out), cu_count, stream);
    return launch_reduce_int_t<int16_t>(static_cast<const int16_t *>(in), shape, dims, reduce_flag, op, shift, half_even,
                                        static_cast<int16_t *>(out), cu_count, stream);
}

} // namespace espdl
