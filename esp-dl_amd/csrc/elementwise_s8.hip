// Bandwidth-bound int8 element-wise operators for gfx950: LUT, PReLU, ReLU, Clip, Add,
// GlobalAveragePool, requantize.  Each thread moves 16 bytes per load/store when the tensors are
// 16-byte aligned; a byte tail (and unaligned tensors) take the scalar path of the same kernel.
#include "espdl_device.h"
#include "espdl_kernels.h"
#include "binary_vec.h"
#include "reduce_mid.h"

namespace espdl {

namespace {

constexpr int kBlock = 256;

// Launch helper: `vecs` 16-byte vectors handled by the vector path, the remaining `size - 16*vecs`
// bytes by the scalar path of the first threads.
inline dim3 grid_for(int64_t size, bool vec_ok, int64_t *vecs)
{
    *vecs = vec_ok ? size / 16 : 0;
    const int64_t tail = size - *vecs * 16;
    const int64_t threads = (*vecs > tail ? *vecs : tail);
    return dim3((unsigned)((threads + kBlock - 1) / kBlock));
}

inline bool aligned16(const void *a, const void *b)
{
    return ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15) == 0;
}

// A per-byte functor applied over a flat tensor.
template <typename F>
__global__ __launch_bounds__(kBlock) void map_s8_kernel(const int8_t *in, int8_t *out, int64_t size, int64_t vecs, F f)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    f.prepare();
    if (i < vecs) {
        const v4i v = reinterpret_cast<const v4i *>(in)[i];
        v4i r;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const int word = v[w];
            int o = 0;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                const int x = (int)(int8_t)(word >> (8 * b));
                o |= (f(x, i * 16 + w * 4 + b) & 0xff) << (8 * b);
            }
            r[w] = o;
        }
        reinterpret_cast<v4i *>(out)[i] = r;
    }
    const int64_t t = vecs * 16 + i;
    if (t < size)
        out[t] = (int8_t)f((int)in[t], t);
}

// base::lut_s8_c (esp-dl/dl/base/dl_base_lut.cpp:10-15); the table is copied to LDS once per workgroup.
struct LutFn {
    const int8_t *table;
    __device__ void prepare()
    {
        __shared__ int8_t tab[256];
        tab[threadIdx.x] = table[threadIdx.x];
        __syncthreads();
        lds = tab;
    }
    __device__ int operator()(int x, int64_t) const { return lds[x + 128]; }
    const int8_t *lds;
};

// module::Relu (esp-dl/dl/module/include/dl_module_relu.hpp:65-93)
struct ReluFn {
    int same_exp;
    float in_scale, out_scale;
    __device__ void prepare() {}
    __device__ int operator()(int x, int64_t) const
    {
        if (same_exp)
            return x >= 0 ? x : 0;
        const float temp = (float)x * in_scale;
        return temp >= 0 ? clamp_s8(round_half_up_f32(temp * out_scale)) : 0;
    }
};

// module::Clip (esp-dl/dl/module/include/dl_module_clip.hpp:78-90)
struct ClipFn {
    int lo, hi;
    float rescale;
    __device__ void prepare() {}
    __device__ int operator()(int x, int64_t) const
    {
        const int t = x < lo ? lo : (x > hi ? hi : x);
        return clamp_s8(round_half_up_f32((float)t * rescale));
    }
};

// TensorBase::assign int8 -> int8 (esp-dl/dl/tensor/src/dl_tensor_base.cpp:362-371, 18-42)
struct RequantFn {
    float src_scale, inv_scale;
    __device__ void prepare() {}
    __device__ int operator()(int x, int64_t) const
    {
        const float tmp = (float)x * src_scale;
        return clamp_s8(round_half_up_f32(tmp * inv_scale));
    }
};

// prelu_11c<int8_t, int16_t> (esp-dl/dl/base/dl_base_prelu.cpp:7-21)
struct PreluFn {
    const int8_t *alpha;
    int channels, shift;
    __device__ void prepare() {}
    __device__ __forceinline__ int one(int x, int slope) const
    {
        if (x >= 0)
            return x;
        const int prod = x * slope;
        const int shifted = shift > 0 ? (prod >> shift) : (int)((unsigned)prod << -shift);
        return clamp_s8((int)(int16_t)shifted);
    }
    __device__ int operator()(int x, int64_t idx) const { return x >= 0 ? x : one(x, (int)alpha[idx % channels]); }
};

template <typename F>
hipError_t launch_map(const int8_t *in, int8_t *out, int64_t size, F f, hipStream_t stream)
{
    if (size <= 0)
        return hipSuccess;
    int64_t vecs;
    const dim3 grid = grid_for(size, aligned16(in, out), &vecs);
    hipLaunchKernelGGL(map_s8_kernel<F>, grid, dim3(kBlock), 0, stream, in, out, size, vecs, f);
    return hipGetLastError();
}

// c_impl_add_n_n / _n_1 / _1_n (esp-dl/dl/base/dl_base_add.cpp:8-44): clamp(a + b).
// Binary element-wise operators on two int8 tensors: Op::apply(a, b) per element.
//   AddOp  elemwise_add, c_impl_add_n_n (esp-dl/dl/base/dl_base_add.cpp:8-44): clamp(a + b)
//   MulOp  elemwise_mul, c_impl_mul_n_n (esp-dl/dl/base/dl_base_mul.cpp:33-46): the product rescaled by
//          2^-(out_exp - e0 - e1) with round-half-up (the float expression there is exact for these
//          operands) or, for the ESP32-P4 behaviour, round-half-even; then clamped
struct AddOp {
    __device__ __forceinline__ int apply(int a, int b) const { return clamp_s8(a + b); }
};
struct MulOp {
    int shift;
    bool half_even;
    __device__ __forceinline__ int apply(int a, int b) const { return requant_s8(a * b, shift, false, half_even); }
};

template <typename Op>
__global__ __launch_bounds__(kBlock) void binary_s8_dense_kernel(const int8_t *in0, const int8_t *in1, int8_t *out,
                                                                 int64_t size, int64_t vecs, Op op)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < vecs) {
        const v4i a = reinterpret_cast<const v4i *>(in0)[i];
        const v4i b = reinterpret_cast<const v4i *>(in1)[i];
        v4i r;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            int o = 0;
#pragma unroll
            for (int k = 0; k < 4; k++)
                o |= (op.apply((int)(int8_t)(a[w] >> (8 * k)), (int)(int8_t)(b[w] >> (8 * k))) & 0xff) << (8 * k);
            r[w] = o;
        }
        reinterpret_cast<v4i *>(out)[i] = r;
    }
    const int64_t t = vecs * 16 + i;
    if (t < size)
        out[t] = (int8_t)op.apply((int)in0[t], (int)in1[t]);
}

struct BroadcastArgs {
    int d[4];
    long long s0[4], s1[4];
};

template <typename Op>
__global__ __launch_bounds__(kBlock) void binary_s8_broadcast_kernel(const int8_t *in0, const int8_t *in1, int8_t *out,
                                                                     int64_t size, BroadcastArgs a, Op op)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= size)
        return;
    int64_t rest = i;
    const int i3 = (int)(rest % a.d[3]);
    rest /= a.d[3];
    const int i2 = (int)(rest % a.d[2]);
    rest /= a.d[2];
    const int i1 = (int)(rest % a.d[1]);
    const int i0 = (int)(rest / a.d[1]);
    const long long o0 = i0 * a.s0[0] + i1 * a.s0[1] + i2 * a.s0[2] + i3 * a.s0[3];
    const long long o1 = i0 * a.s1[0] + i1 * a.s1[1] + i2 * a.s1[2] + i3 * a.s1[3];
    out[i] = (int8_t)op.apply((int)in0[o0], (int)in1[o1]);
}

template <typename Op>
hipError_t launch_binary_s8(const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                            const int8_t *in1, int8_t *out, Op op, hipStream_t stream)
{
    const int64_t size = (int64_t)dims[0] * dims[1] * dims[2] * dims[3];
    if (size <= 0)
        return hipSuccess;
    // dense strides of the output shape
    int64_t dense[4];
    dense[3] = 1;
    for (int i = 2; i >= 0; i--)
        dense[i] = dense[i + 1] * dims[i + 1];
    bool both_dense = true;
    for (int i = 0; i < 4; i++)
        if (dims[i] > 1 && (s0[i] != dense[i] || s1[i] != dense[i]))
            both_dense = false;
    if (both_dense) {
        const bool vec_ok = aligned16(in0, in1) && aligned16(out, out);
        int64_t vecs;
        const dim3 grid = grid_for(size, vec_ok, &vecs);
        hipLaunchKernelGGL(binary_s8_dense_kernel<Op>, grid, dim3(kBlock), 0, stream, in0, in1, out, size, vecs, op);
    } else if (binary_vec::Args va; binary_vec::plan(dims, s0, s1, in0, in1, out, &va)) {
        // innermost axis dense or constant in each operand (a channel-wise scale, a per-row offset): 16 bytes per thread
        return binary_vec::launch(in0, in1, out, va, op, 0, stream);
    } else {
        BroadcastArgs a;
        for (int i = 0; i < 4; i++) {
            a.d[i] = dims[i];
            a.s0[i] = dims[i] > 1 ? s0[i] : 0;
            a.s1[i] = dims[i] > 1 ? s1[i] : 0;
        }
        hipLaunchKernelGGL(binary_s8_broadcast_kernel<Op>, dim3((unsigned)((size + kBlock - 1) / kBlock)), dim3(kBlock), 0,
                           stream, in0, in1, out, size, a, op);
    }
    return hipGetLastError();
}

// GlobalAveragePool: avgpool2d_hwc with the window covering the image
// (esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54).  One workgroup per (image, slab of 64 x VEC channels):
// lane l owns VEC consecutive channels (one VEC-byte load per pixel, adjacent lanes adjacent bytes, so a
// wavefront reads whole contiguous runs of a pixel row), the 4 wavefronts split the pixels, int32
// partial sums meet in LDS.  VEC = 16 when the channel count and pointers allow, else 1.
template <int VEC>
__global__ __launch_bounds__(kBlock) void global_avg_pool_s8_kernel(const int8_t *in, int8_t *out, int hw, int c,
                                                                    float scale)
{
    __shared__ int partial[4][64 * VEC];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int ch = (blockIdx.x * 64 + lane) * VEC;
    const int8_t *img = in + (long long)blockIdx.y * hw * c;
    int sum[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++)
        sum[k] = 0;
    if (ch < c) {
        for (int p = wave; p < hw; p += 4) {
            if (VEC == 16) {
                const v4i v = *reinterpret_cast<const v4i *>(img + (long long)p * c + ch);
#pragma unroll
                for (int k = 0; k < VEC; k++)
                    sum[k] += (int)(int8_t)(v[k >> 2] >> (8 * (k & 3)));
            } else {
                sum[0] += img[(long long)p * c + ch];
            }
        }
    }
#pragma unroll
    for (int k = 0; k < VEC; k++)
        partial[wave][lane * VEC + k] = sum[k];
    __syncthreads();
    // 256 threads finish 64 * VEC channels
    for (int e = threadIdx.x; e < 64 * VEC; e += kBlock) {
        const int oc = blockIdx.x * 64 * VEC + e;
        if (oc < c) {
            const int total = partial[0][e] + partial[1][e] + partial[2][e] + partial[3][e];
            out[(long long)blockIdx.y * c + oc] = (int8_t)clamp_s8(round_half_up_f32((float)total * scale));
        }
    }
}

// The same operator for small windows (hw <= 64: a 7 x 7 head): one lane owns FOUR consecutive channels of one
// image and walks all pixels itself (one 4-byte load per pixel, adjacent lanes adjacent dwords, every load
// requested before the first is used), so there is no exchange between lanes at all.
__global__ __launch_bounds__(kBlock) void global_avg_pool_s8_small_kernel(const int8_t *in, int8_t *out, int hw, int c,
                                                                          float scale)
{
    const int ch = (blockIdx.x * kBlock + threadIdx.x) * 4;
    if (ch >= c)
        return;
    const int8_t *img = in + (long long)blockIdx.y * hw * c + ch;
    int sum[4] = {0, 0, 0, 0};
    constexpr int kStep = 16; // loads in flight per lane
    for (int p0 = 0; p0 < hw; p0 += kStep) {
        int v[kStep];
#pragma unroll
        for (int j = 0; j < kStep; j++)
            v[j] = *reinterpret_cast<const int *>(img + (size_t)(unsigned)(min(p0 + j, hw - 1) * c));
#pragma unroll
        for (int j = 0; j < kStep; j++) {
            if (p0 + j < hw) { // uniform
#pragma unroll
                for (int k = 0; k < 4; k++)
                    sum[k] += (int)(int8_t)(v[j] >> (8 * k));
            }
        }
    }
    int q[4];
#pragma unroll
    for (int k = 0; k < 4; k++)
        q[k] = clamp_s8(round_half_up_f32((float)sum[k] * scale));
    *reinterpret_cast<int *>(out + (long long)blockIdx.y * c + ch) = pack4_s8(q[0], q[1], q[2], q[3]);
}

} // namespace

hipError_t launch_lut_s8(const int8_t *in, int64_t size, const int8_t *table, int8_t *out, hipStream_t stream)
{
    return launch_map(in, out, size, LutFn{table, nullptr}, stream);
}

namespace {
// PReLU with a channel count that is a multiple of 16 and 16-byte aligned tensors: a thread's 16 bytes are 16
// consecutive channels of one pixel, so the slopes are one 16-byte load and the channel index is one division per
// thread (the per-byte functor form divides a 64-bit index for every byte).
__global__ __launch_bounds__(kBlock) void prelu_s8_vec_kernel(const int8_t *in, const int8_t *alpha, int8_t *out, int64_t vecs,
                                                              unsigned vecs_per_pixel, int shift)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= vecs)
        return;
    const unsigned cv = (unsigned)((uint64_t)i % vecs_per_pixel);
    const v4i x = reinterpret_cast<const v4i *>(in)[i];
    const v4i s = reinterpret_cast<const v4i *>(alpha)[cv];
    const PreluFn f{nullptr, 1, shift};
    v4i r;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        int o = 0;
#pragma unroll
        for (int b = 0; b < 4; b++)
            o |= (f.one((int)(int8_t)(x[w] >> (8 * b)), (int)(int8_t)(s[w] >> (8 * b))) & 0xff) << (8 * b);
        r[w] = o;
    }
    reinterpret_cast<v4i *>(out)[i] = r;
}
} // namespace

hipError_t launch_prelu_s8(const int8_t *in, int64_t pixels, int channels, const int8_t *alpha, int shift,
                           int8_t *out, hipStream_t stream)
{
    if (pixels > 0 && channels > 0 && (channels & 15) == 0 && aligned16(in, out) && aligned16(alpha, alpha)) {
        const int64_t vecs = pixels * (channels / 16);
        hipLaunchKernelGGL(prelu_s8_vec_kernel, dim3((unsigned)((vecs + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream, in, alpha,
                           out, vecs, (unsigned)(channels / 16), shift);
        return hipGetLastError();
    }
    return launch_map(in, out, pixels * channels, PreluFn{alpha, channels, shift}, stream);
}

hipError_t launch_relu_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out, hipStream_t stream)
{
    return launch_map(in, out, size, ReluFn{in_exp == out_exp, dl_scale(in_exp), dl_rescale(out_exp)}, stream);
}

namespace {
// Clip between equal exponents: the rescale factor is 1 and the operator is a clamp of the stored value.  Four
// bytes per packed-int16 sequence: the bytes go to the high bytes of two int16 pairs (x * 256), one packed
// maximum and minimum against (lo << 8) and (hi << 8) | 0xff, the high bytes are gathered again.
__global__ __launch_bounds__(kBlock) void clamp_s8_kernel(const int8_t *in, int8_t *out, int64_t size, int64_t vecs, int lo,
                                                          int hi)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const v2s lo2 = __builtin_bit_cast(v2s, ((lo << 8) & 0xffff) * 0x10001);
    const v2s hi2 = __builtin_bit_cast(v2s, (((hi << 8) | 0xff) & 0xffff) * 0x10001);
    if (i < vecs) {
        const v4i v = reinterpret_cast<const v4i *>(in)[i];
        v4i r;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            v2s p01 = __builtin_bit_cast(v2s, (int)__builtin_amdgcn_perm(0u, (unsigned)v[w], 0x010c000cu));
            v2s p23 = __builtin_bit_cast(v2s, (int)__builtin_amdgcn_perm(0u, (unsigned)v[w], 0x030c020cu));
            p01 = __builtin_elementwise_min(__builtin_elementwise_max(p01, lo2), hi2);
            p23 = __builtin_elementwise_min(__builtin_elementwise_max(p23, lo2), hi2);
            r[w] = (int)__builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, p23), (unsigned)__builtin_bit_cast(int, p01),
                                              0x07050301u);
        }
        reinterpret_cast<v4i *>(out)[i] = r;
    }
    const int64_t t = vecs * 16 + i;
    if (t < size)
        out[t] = (int8_t)min(max((int)in[t], lo), hi);
}
} // namespace

hipError_t launch_clip_s8(const int8_t *in, int64_t size, int min_q, int max_q, int in_exp, int out_exp, int8_t *out,
                          hipStream_t stream)
{
    const bool aligned = ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    if (in_exp == out_exp && aligned && min_q >= -128 && max_q <= 127 && min_q <= max_q) {
        const int64_t vecs = size / 16;
        const int64_t work = std::max<int64_t>(vecs, size - vecs * 16);
        if (work <= 0)
            return hipSuccess;
        hipLaunchKernelGGL(clamp_s8_kernel, dim3((unsigned)((work + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream, in, out,
                           size, vecs, min_q, max_q);
        return hipGetLastError();
    }
    return launch_map(in, out, size, ClipFn{min_q, max_q, dl_scale(in_exp) * dl_rescale(out_exp)}, stream);
}

namespace {
// int8 -> int8 between exponents at most 7 apart: four values per packed-int16 sequence (requant4_s8: round half
// up of x * 2^d, saturated - what RequantFn computes in float, where both scales are powers of two and every step
// is exact); bytes past the last 16-byte vector take RequantFn itself.
__global__ __launch_bounds__(kBlock) void requantize_pow2_s8_kernel(const int8_t *in, int8_t *out, int64_t size, int64_t vecs,
                                                                    int d, RequantFn tail)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const Requant4 q = make_requant4(d);
    if (i < vecs) {
        const v4i v = reinterpret_cast<const v4i *>(in)[i];
        v4i r;
#pragma unroll
        for (int w = 0; w < 4; w++)
            r[w] = requant4_s8(v[w], q);
        reinterpret_cast<v4i *>(out)[i] = r;
    }
    const int64_t t = vecs * 16 + i;
    if (t < size)
        out[t] = (int8_t)tail((int)in[t], t);
}
} // namespace

hipError_t launch_requantize_s8(const int8_t *in, int64_t size, int in_exp, int out_exp, int8_t *out,
                                hipStream_t stream)
{
    if (in_exp == out_exp) {
        if (in == out || size <= 0)
            return hipSuccess;
        return hipMemcpyAsync(out, in, (size_t)size, hipMemcpyDeviceToDevice, stream);
    }
    const float inv = (float)(1.0 / (double)dl_scale(out_exp));
    const int d = in_exp - out_exp;
    if (d >= -7 && d <= 7 && aligned16(in, out) && size >= 16) {
        int64_t vecs;
        const dim3 grid = grid_for(size, true, &vecs);
        hipLaunchKernelGGL(requantize_pow2_s8_kernel, grid, dim3(kBlock), 0, stream, in, out, size, vecs, d,
                           RequantFn{dl_scale(in_exp), inv});
        return hipGetLastError();
    }
    return launch_map(in, out, size, RequantFn{dl_scale(in_exp), inv}, stream);
}

namespace {
// The same on rows that lie `in_pitch` / `out_pitch` bytes apart (channel slices of wider NHWC tensors): a thread
// takes one 16-byte unit of a row (VEC) or one byte of it.
template <bool VEC>
__global__ __launch_bounds__(kBlock) void requantize_s8_rows_kernel(const int8_t *in, int64_t in_pitch, int8_t *out,
                                                                   int64_t out_pitch, FastDiv per_row, int64_t total, int d,
                                                                   RequantFn f)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= total)
        return;
    const unsigned row = fastdiv((unsigned)i, per_row);
    const unsigned u = (unsigned)i - row * per_row.d;
    if constexpr (VEC) {
        const Requant4 q = make_requant4(d);
        const v4i v = *reinterpret_cast<const v4i *>(in + (int64_t)row * in_pitch + 16 * (int64_t)u);
        v4i r;
#pragma unroll
        for (int w = 0; w < 4; w++)
            r[w] = requant4_s8(v[w], q);
        *reinterpret_cast<v4i *>(out + (int64_t)row * out_pitch + 16 * (int64_t)u) = r;
    } else {
        out[(int64_t)row * out_pitch + u] = (int8_t)f((int)in[(int64_t)row * in_pitch + u], 0);
    }
}
} // namespace

hipError_t launch_requantize_s8_rows(const int8_t *in, int64_t in_pitch, int8_t *out, int64_t out_pitch, int64_t row_bytes,
                                     int64_t rows, int in_exp, int out_exp, hipStream_t stream)
{
    if (rows <= 0 || row_bytes <= 0)
        return hipSuccess;
    const int d = in_exp - out_exp;
    const RequantFn f{dl_scale(in_exp), (float)(1.0 / (double)dl_scale(out_exp))};
    const bool vec = d >= -7 && d <= 7 && (row_bytes & 15) == 0 && (in_pitch & 15) == 0 && (out_pitch & 15) == 0 &&
        aligned16(in, out);
    const int64_t per_row = vec ? row_bytes / 16 : row_bytes;
    const int64_t total = rows * per_row;
    if (total > 0x7fffffffll || per_row > 0x7fffffffll)
        return hipErrorInvalidValue;
    const dim3 grid((unsigned)((total + kBlock - 1) / kBlock));
    if (vec)
        hipLaunchKernelGGL(requantize_s8_rows_kernel<true>, grid, dim3(kBlock), 0, stream, in, in_pitch, out, out_pitch,
                           make_fastdiv((unsigned)per_row), total, d, f);
    else
        hipLaunchKernelGGL(requantize_s8_rows_kernel<false>, grid, dim3(kBlock), 0, stream, in, in_pitch, out, out_pitch,
                           make_fastdiv((unsigned)per_row), total, d, f);
    return hipGetLastError();
}

// TensorBase::assign between int8 / int16 (esp-dl/dl/tensor/src/dl_tensor_base.cpp:321-392).
// Eight elements per thread (one 8- or 16-byte access each way) when both pointers allow; the last size % 8 elements,
// or everything when a pointer is unaligned, one element per thread.
template <typename T>
struct alignas(8 * sizeof(T)) Eight {
    T v[8];
};

template <typename ST, typename DT>
__device__ __forceinline__ DT requantize_one(ST x, int same_exp, float src_scale, float inv_scale)
{
    const int lo = sizeof(DT) == 1 ? -128 : -32768, hi = sizeof(DT) == 1 ? 127 : 32767;
    int q;
    if (same_exp) {
        q = (int)x;
    } else {
        const float tmp = (float)x * src_scale;
        q = round_half_up_f32(tmp * inv_scale);
    }
    return (DT)min(max(q, lo), hi);
}

template <typename ST, typename DT>
__global__ __launch_bounds__(kBlock) void requantize_any_kernel(const ST *in, DT *out, int64_t size, int64_t vecs, int same_exp,
                                                                float src_scale, float inv_scale)
{
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < vecs) {
        const Eight<ST> x = reinterpret_cast<const Eight<ST> *>(in)[i];
        Eight<DT> r;
#pragma unroll
        for (int k = 0; k < 8; k++)
            r.v[k] = requantize_one<ST, DT>(x.v[k], same_exp, src_scale, inv_scale);
        reinterpret_cast<Eight<DT> *>(out)[i] = r;
    }
    const int64_t t = vecs * 8 + i;
    if (t < size)
        out[t] = requantize_one<ST, DT>(in[t], same_exp, src_scale, inv_scale);
}

template <typename ST, typename DT>
hipError_t launch_requantize_any_t(const void *in, void *out, int64_t size, int same, float src, float inv, hipStream_t stream)
{
    const bool vec_ok = (reinterpret_cast<uintptr_t>(in) % (8 * sizeof(ST))) == 0 && (reinterpret_cast<uintptr_t>(out) % (8 * sizeof(DT))) == 0;
    const int64_t vecs = vec_ok ? size / 8 : 0;
    const int64_t tail = size - vecs * 8;
    const int64_t threads = vecs > tail ? vecs : tail;
    hipLaunchKernelGGL((requantize_any_kernel<ST, DT>), dim3((unsigned)((threads + kBlock - 1) / kBlock)), dim3(kBlock), 0, stream,
                       static_cast<const ST *>(in), static_cast<DT *>(out), size, vecs, same, src, inv);
    return hipGetLastError();
}

hipError_t launch_requantize_any(const void *in, int in_bits, int64_t size, int in_exp, int out_exp, void *out,
                                 int out_bits, hipStream_t stream)
{
    if (size <= 0)
        return hipSuccess;
    const int same = in_exp == out_exp;
    const float src = dl_scale(in_exp), inv = (float)(1.0 / (double)dl_scale(out_exp));
    if (in_bits == 8 && out_bits == 16)
        return launch_requantize_any_t<int8_t, int16_t>(in, out, size, same, src, inv, stream);
    if (in_bits == 16 && out_bits == 8)
        return launch_requantize_any_t<int16_t, int8_t>(in, out, size, same, src, inv, stream);
    if (in_bits == 16 && out_bits == 16)
        return launch_requantize_any_t<int16_t, int16_t>(in, out, size, same, src, inv, stream);
    return launch_requantize_any_t<int8_t, int8_t>(in, out, size, same, src, inv, stream);
}

hipError_t launch_add_s8(const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                         const int8_t *in1, int8_t *out, hipStream_t stream)
{
    return launch_binary_s8(dims, s0, s1, in0, in1, out, AddOp{}, stream);
}

hipError_t launch_mul_s8(const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const int8_t *in0,
                         const int8_t *in1, int shift, int half_even, int8_t *out, hipStream_t stream)
{
    return launch_binary_s8(dims, s0, s1, in0, in1, out, MulOp{shift, half_even != 0}, stream);
}

// the float factor of the pooling operator, formed as the reference forms it
float global_avg_pool_scale(int h, int w, int in_exp, int out_exp)
{
    const float area_inv = 1.f / (float)(h * w);
    return dl_scale(in_exp) * area_inv * dl_rescale(out_exp);
}

namespace {
// what GlobalAveragePool does with the sum of an image's pixels
struct GapFinish {
    int8_t *out;
    float scale;
    __device__ void operator()(long long o, int total) const
    {
        out[o] = (int8_t)clamp_s8(round_half_up_f32((float)total * scale));
    }
};
} // namespace

hipError_t launch_global_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int in_exp, int out_exp,
                                     int8_t *out, hipStream_t stream)
{
    if (batch <= 0)
        return hipSuccess;
    const float scale = global_avg_pool_scale(h, w, in_exp, out_exp);
    if ((c & 3) == 0 && h * w <= 64 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 3) == 0)
        hipLaunchKernelGGL(global_avg_pool_s8_small_kernel, dim3((unsigned)((c / 4 + kBlock - 1) / kBlock), (unsigned)batch),
                           dim3(kBlock), 0, stream, in, out, h * w, c, scale);
    else if (reduce_mid::fits<int8_t>(batch, (long long)h * w, c)) // every lane busy whatever the channel count
        return reduce_mid::launch(in, batch, (long long)h * w, c, GapFinish{out, scale}, stream);
    else if ((c & 15) == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0)
        hipLaunchKernelGGL(global_avg_pool_s8_kernel<16>, dim3((unsigned)((c + 1023) / 1024), (unsigned)batch), dim3(kBlock),
                           0, stream, in, out, h * w, c, scale);
    else
        hipLaunchKernelGGL(global_avg_pool_s8_kernel<1>, dim3((unsigned)((c + 63) / 64), (unsigned)batch), dim3(kBlock), 0,
                           stream, in, out, h * w, c, scale);
    return hipGetLastError();
}

} // namespace espdl
