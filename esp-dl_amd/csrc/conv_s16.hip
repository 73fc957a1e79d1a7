// int16 convolutions for gfx950: exact int16 x int16 products accumulated in int64 on the VALU.
//
// Restates conv2d_hwcn<int16_t, int64_t> (esp-dl/dl/base/dl_base_conv2d.cpp:116-163, selected at
// :875-897) and depthwise_conv2d_hwc1<int16_t, int64_t> (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:46-65)
// with the int64 epilogue (bias int64, shift_and_round<int64_t>, clamp to int16;
// esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72).
//
// Dense: a thread owns one output pixel and 4 consecutive filters; the reduction runs over the
// in-image taps only.  Products are formed in 32 bits (|int16 * int16| <= 2^30) and added to a
// 64-bit accumulator, as the reference does.
#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

struct S16Args {
    const int16_t *in;
    const int16_t *w;
    const int64_t *bias;
    const int32_t *shift;
    int16_t *out;
    ConvGeom g;
    int oc_quads;
    long long n_items;
    int vec8; // channels % 8 == 0 and 16-byte aligned tensors: 16-byte loads
};

__global__ __launch_bounds__(256) void conv2d_s16_kernel(const S16Args a)
{
    const ConvGeom &g = a.g;
    const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (item >= a.n_items)
        return;
    const int oq = (int)(item % a.oc_quads);
    long long rest = item / a.oc_quads;
    const int ox = (int)(rest % g.out_w);
    rest /= g.out_w;
    const int oy = (int)(rest % g.out_h);
    const int n = (int)(rest / g.out_h);
    const int C = g.in_c, OC = g.out_c;
    const int oc0 = oq * 4;
    const long long ftap = (long long)g.k_h * g.k_w * C; // elements per filter
    const int16_t *img = a.in + (long long)n * g.in_h * g.in_w * C;

    long long acc[4] = {0, 0, 0, 0};
    for (int ky = 0; ky < g.k_h; ky++) {
        const int iy = oy * g.stride_h - g.pad_top + ky * g.dil_h;
        if ((unsigned)iy >= (unsigned)g.in_h)
            continue;
        for (int kx = 0; kx < g.k_w; kx++) {
            const int ix = ox * g.stride_w - g.pad_left + kx * g.dil_w;
            if ((unsigned)ix >= (unsigned)g.in_w)
                continue;
            const int16_t *px = img + ((long long)iy * g.in_w + ix) * C;
            const int16_t *fw = a.w + (long long)oc0 * ftap + ((long long)ky * g.k_w + kx) * C;
            int c = 0;
            if (a.vec8 && oc0 + 3 < OC) {
                // eight channels per 16-byte load of the pixel and of each of the four filters; every product
                // goes into the 64-bit accumulator with one multiply-add
                for (; c + 8 <= C; c += 8) {
                    const v4i xv = *reinterpret_cast<const v4i *>(px + c);
                    v4i wv[4];
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        wv[r] = *reinterpret_cast<const v4i *>(fw + r * ftap + c);
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        const long long x0 = (short)xv[d], x1 = xv[d] >> 16;
#pragma unroll
                        for (int r = 0; r < 4; r++) {
                            acc[r] += x0 * (long long)(short)wv[r][d];
                            acc[r] += x1 * (long long)(wv[r][d] >> 16);
                        }
                    }
                }
            }
            for (; c < C; c++) {
                const int v = px[c];
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (oc0 + r < OC)
                        acc[r] += (long long)(v * (int)fw[r * ftap + c]);
            }
        }
    }
    int16_t *dst = a.out + (((long long)n * g.out_h + oy) * g.out_w + ox) * OC + oc0;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        if (oc0 + r < OC) {
            long long v = acc[r];
            if (a.bias != nullptr)
                v += a.bias[oc0 + r];
            dst[r] = (int16_t)requant_s16(v, a.shift[g.n_shift == 1 ? 0 : oc0 + r], g.relu != 0, g.half_even != 0);
        }
    }
}

__global__ __launch_bounds__(256) void depthwise_s16_kernel(const S16Args a)
{
    const ConvGeom &g = a.g;
    const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (item >= a.n_items)
        return;
    const int C = g.in_c;
    const int c = (int)(item % C);
    long long rest = item / C;
    const int ox = (int)(rest % g.out_w);
    rest /= g.out_w;
    const int oy = (int)(rest % g.out_h);
    const int n = (int)(rest / g.out_h);
    const int16_t *img = a.in + (long long)n * g.in_h * g.in_w * C + c;
    long long acc = 0;
    for (int ky = 0; ky < g.k_h; ky++) {
        const int iy = oy * g.stride_h - g.pad_top + ky * g.dil_h;
        if ((unsigned)iy >= (unsigned)g.in_h)
            continue;
        for (int kx = 0; kx < g.k_w; kx++) {
            const int ix = ox * g.stride_w - g.pad_left + kx * g.dil_w;
            if ((unsigned)ix < (unsigned)g.in_w)
                acc += (long long)((int)img[((long long)iy * g.in_w + ix) * C] *
                                   (int)a.w[((long long)ky * g.k_w + kx) * C + c]);
        }
    }
    if (a.bias != nullptr)
        acc += a.bias[c];
    a.out[item] = (int16_t)requant_s16(acc, a.shift[g.n_shift == 1 ? 0 : c], g.relu != 0, g.half_even != 0);
}

// Eight channels per lane with 16-byte loads (channels % 8 == 0, 16-byte aligned tensors).
__global__ __launch_bounds__(256) void depthwise_s16_vec8_kernel(const S16Args a)
{
    const ConvGeom &g = a.g;
    const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (item >= a.n_items)
        return;
    const int C = g.in_c, C8 = C / 8;
    const int c = (int)(item % C8) * 8;
    long long rest = item / C8;
    const int ox = (int)(rest % g.out_w);
    rest /= g.out_w;
    const int oy = (int)(rest % g.out_h);
    const int n = (int)(rest / g.out_h);
    const int16_t *img = a.in + (long long)n * g.in_h * g.in_w * C + c;
    long long acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int ky = 0; ky < g.k_h; ky++) {
        const int iy = oy * g.stride_h - g.pad_top + ky * g.dil_h;
        if ((unsigned)iy >= (unsigned)g.in_h)
            continue;
        for (int kx = 0; kx < g.k_w; kx++) {
            const int ix = ox * g.stride_w - g.pad_left + kx * g.dil_w;
            if ((unsigned)ix >= (unsigned)g.in_w)
                continue;
            const v4i xv = *reinterpret_cast<const v4i *>(img + ((long long)iy * g.in_w + ix) * C);
            const v4i wv = *reinterpret_cast<const v4i *>(a.w + ((long long)ky * g.k_w + kx) * C + c);
#pragma unroll
            for (int d = 0; d < 4; d++) {
                acc[2 * d] += (long long)(short)xv[d] * (long long)(short)wv[d];
                acc[2 * d + 1] += (long long)(xv[d] >> 16) * (long long)(wv[d] >> 16);
            }
        }
    }
    int q[8];
#pragma unroll
    for (int r = 0; r < 8; r++) {
        long long v = acc[r];
        if (a.bias != nullptr)
            v += a.bias[c + r];
        q[r] = requant_s16(v, a.shift[g.n_shift == 1 ? 0 : c + r], g.relu != 0, g.half_even != 0) & 0xffff;
    }
    *reinterpret_cast<v4i *>(a.out + (((long long)n * g.out_h + oy) * g.out_w + ox) * C + c) =
        v4i{q[0] | (q[1] << 16), q[2] | (q[3] << 16), q[4] | (q[5] << 16), q[6] | (q[7] << 16)};
}

} // namespace

hipError_t launch_conv2d_s16(const ConvGeom &g, const int16_t *in, const int16_t *filter, const int64_t *bias,
                             const int32_t *shift, int16_t *out, hipStream_t stream)
{
    S16Args a{in, filter, bias, shift, out, g, (g.out_c + 3) / 4, 0, 0};
    a.n_items = (long long)g.batch * g.out_h * g.out_w * a.oc_quads;
    a.vec8 = (g.in_c % 8) == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter)) & 15) == 0;
    if (a.n_items == 0)
        return hipSuccess;
    hipLaunchKernelGGL(conv2d_s16_kernel, dim3((unsigned)((a.n_items + 255) / 256)), dim3(256), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_depthwise_s16(const ConvGeom &g, const int16_t *in, const int16_t *filter, const int64_t *bias,
                                const int32_t *shift, int16_t *out, hipStream_t stream)
{
    S16Args a{in, filter, bias, shift, out, g, 0, 0, 0};
    a.n_items = (long long)g.batch * g.out_h * g.out_w * g.in_c;
    if (a.n_items == 0)
        return hipSuccess;
    if ((g.in_c % 8) == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter) |
                                reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        a.n_items /= 8;
        hipLaunchKernelGGL(depthwise_s16_vec8_kernel, dim3((unsigned)((a.n_items + 255) / 256)), dim3(256), 0, stream, a);
        return hipGetLastError();
    }
    hipLaunchKernelGGL(depthwise_s16_kernel, dim3((unsigned)((a.n_items + 255) / 256)), dim3(256), 0, stream, a);
    return hipGetLastError();
}

} // namespace espdl
