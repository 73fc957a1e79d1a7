// Depthwise int8 convolution for gfx950.  HBM-bound: no MFMA, coalesced loads along the NHWC
// channel axis, one accumulator per channel.
//
// Restates depthwise_conv2d_11c1 / _33c1 / _hwc1 (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:9-65)
// under dwconv_operation_shell's window clipping (esp-dl/dl/base/dl_base.hpp:1852-2102) and the shared
// n_wise epilogue (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210).
// Filter memory is [k_h][k_w][c].
//
// DW_VEC4: channels % 4 == 0.  A thread owns 4 channels (one dword) of XT consecutive output columns.
// Each 4-channel MAC is done with v_dot4_i32_i8 against the filter dword masked down to one byte, so
// a MAC costs one VALU instruction and no unpacking.  Adjacent threads take adjacent channel quads:
// a wavefront reads and writes contiguous NHWC bytes.
// DW_BYTE: any channel count, one thread per (pixel, channel).
#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

struct DwArgs {
    const int8_t *in;
    const int8_t *w;
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
    int8_t *out;
    ConvGeom g;
    int cq;            // channel quads (c / 4)
    int xt_per_row;    // ceil(out_w / XT)
    long long n_items; // work items
};

template <int XT>
__global__ __launch_bounds__(256) void depthwise_s8_vec4_kernel(const DwArgs a)
{
    const ConvGeom &g = a.g;
    const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (item >= a.n_items)
        return;
    const int q = (int)(item % a.cq);
    long long rest = item / a.cq;
    const int xs = (int)(rest % a.xt_per_row);
    rest /= a.xt_per_row;
    const int oy = (int)(rest % g.out_h);
    const int n = (int)(rest / g.out_h);
    const int C = g.in_c, c0 = q * 4;
    const int ox0 = xs * XT;

    int acc[XT][4];
#pragma unroll
    for (int x = 0; x < XT; x++)
#pragma unroll
        for (int r = 0; r < 4; r++)
            acc[x][r] = 0;

    const int8_t *img = a.in + (long long)n * g.in_h * g.in_w * C + c0;
    for (int ky = 0; ky < g.k_h; ky++) {
        const int iy = oy * g.stride_h - g.pad_top + ky * g.dil_h;
        if ((unsigned)iy >= (unsigned)g.in_h)
            continue;
        const int8_t *row = img + (long long)iy * g.in_w * C;
        for (int kx = 0; kx < g.k_w; kx++) {
            const int wq = *reinterpret_cast<const int *>(a.w + ((long long)ky * g.k_w + kx) * C + c0);
            const int w0 = wq & 0x000000ff, w1 = wq & 0x0000ff00, w2 = wq & 0x00ff0000, w3 = wq & (int)0xff000000;
#pragma unroll
            for (int x = 0; x < XT; x++) {
                const int ix = (ox0 + x) * g.stride_w - g.pad_left + kx * g.dil_w;
                if ((unsigned)ix < (unsigned)g.in_w) {
                    const int v = *reinterpret_cast<const int *>(row + (long long)ix * C);
                    acc[x][0] = __builtin_amdgcn_sdot4(v, w0, acc[x][0], false);
                    acc[x][1] = __builtin_amdgcn_sdot4(v, w1, acc[x][1], false);
                    acc[x][2] = __builtin_amdgcn_sdot4(v, w2, acc[x][2], false);
                    acc[x][3] = __builtin_amdgcn_sdot4(v, w3, acc[x][3], false);
                }
            }
        }
    }

    v4i bb = {0, 0, 0, 0};
    if (a.bias != nullptr)
        bb = *reinterpret_cast<const v4i *>(a.bias + c0);
    v4i ss;
    if (g.n_shift == 1) {
        const int s = a.shift[0];
        ss = v4i{s, s, s, s};
    } else {
        ss = *reinterpret_cast<const v4i *>(a.shift + c0);
    }
    const bool relu = g.relu != 0, half_even = g.half_even != 0;
    int8_t *dst = a.out + (((long long)n * g.out_h + oy) * g.out_w + ox0) * C + c0;
#pragma unroll
    for (int x = 0; x < XT; x++) {
        if (ox0 + x < g.out_w) {
            int qv[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                qv[r] = requant_s8(acc[x][r] + bb[r], ss[r], relu, half_even);
                if (a.lut != nullptr)
                    qv[r] = a.lut[qv[r] + 128];
            }
            *reinterpret_cast<int *>(dst + (long long)x * C) = pack4_s8(qv[0], qv[1], qv[2], qv[3]);
        }
    }
}

__global__ __launch_bounds__(256) void depthwise_s8_byte_kernel(const DwArgs a)
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
    const int8_t *img = a.in + (long long)n * g.in_h * g.in_w * C + c;
    int acc = 0;
    for (int ky = 0; ky < g.k_h; ky++) {
        const int iy = oy * g.stride_h - g.pad_top + ky * g.dil_h;
        if ((unsigned)iy >= (unsigned)g.in_h)
            continue;
        for (int kx = 0; kx < g.k_w; kx++) {
            const int ix = ox * g.stride_w - g.pad_left + kx * g.dil_w;
            if ((unsigned)ix < (unsigned)g.in_w)
                acc += (int)img[((long long)iy * g.in_w + ix) * C] * (int)a.w[((long long)ky * g.k_w + kx) * C + c];
        }
    }
    if (a.bias != nullptr)
        acc += a.bias[c];
    int qv = requant_s8(acc, a.shift[g.n_shift == 1 ? 0 : c], g.relu != 0, g.half_even != 0);
    if (a.lut != nullptr)
        qv = a.lut[qv + 128];
    a.out[item] = (int8_t)qv;
}

} // namespace

hipError_t launch_depthwise_s8(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                               const int32_t *shift, const int8_t *lut, int8_t *out, hipStream_t stream)
{
    DwArgs a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.out = out;
    a.g = g;
    const long long npix = (long long)g.batch * g.out_h * g.out_w;
    if (npix == 0)
        return hipSuccess;
    const uintptr_t align = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter) |
        reinterpret_cast<uintptr_t>(out);
    const bool bias_ok = bias == nullptr || (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
    const bool shift_ok = g.n_shift == 1 || (reinterpret_cast<uintptr_t>(shift) & 15) == 0;
    if ((g.in_c & 3) == 0 && (align & 3) == 0 && bias_ok && shift_ok) {
        constexpr int XT = 4;
        a.cq = g.in_c / 4;
        a.xt_per_row = (g.out_w + XT - 1) / XT;
        a.n_items = (long long)g.batch * g.out_h * a.xt_per_row * a.cq;
        const unsigned blocks = (unsigned)((a.n_items + 255) / 256);
        hipLaunchKernelGGL(depthwise_s8_vec4_kernel<XT>, dim3(blocks), dim3(256), 0, stream, a);
    } else {
        a.cq = 0;
        a.xt_per_row = 0;
        a.n_items = npix * g.in_c;
        const unsigned blocks = (unsigned)((a.n_items + 255) / 256);
        hipLaunchKernelGGL(depthwise_s8_byte_kernel, dim3(blocks), dim3(256), 0, stream, a);
    }
    return hipGetLastError();
}

} // namespace espdl
