// Depthwise int8 convolution for gfx950.  HBM-bound: no MFMA, coalesced loads along the NHWC
// channel axis, one accumulator per channel.
//
// Restates depthwise_conv2d_11c1 / _33c1 / _hwc1 (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:9-65)
// under dwconv_operation_shell's window clipping (esp-dl/dl/base/dl_base.hpp:1852-2102) and the shared
// n_wise epilogue (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210).
// Filter memory is [k_h][k_w][c].
//
// dw3x3_vec16: the common case (3x3, dilation 1, channels % 16 == 0).  A thread owns 16 channels (one
// 16-byte vector) of YT vertically adjacent output pixels; threads of a wavefront run along the
// channel vectors and then along x, so every load and store instruction of a wavefront covers one
// contiguous span of the NHWC row.  Per filter row the 3 x 16 weights are masked once into
// single-byte dwords and reused for the YT outputs.  When every shift of the thread's channels lies in
// 1..31 and nothing can overflow, accumulators start at bias + 2^(s-1) and the epilogue is the short
// shift / v_cvt_pk_i16_i32 / v_perm_b32 sequence; otherwise the general shift_and_round restatement.
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


template <int YT>
__global__ __launch_bounds__(256) void depthwise_s8_3x3_vec16_kernel(const DwArgs a)
{
    const ConvGeom &g = a.g;
    const long long item = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (item >= a.n_items)
        return;
    const int cv = (int)(item % a.cq); // 16-channel vector
    long long rest = item / a.cq;
    const int ox = (int)(rest % g.out_w);
    rest /= g.out_w;
    const int ys = (int)(rest % a.xt_per_row); // strip of YT output rows
    const int n = (int)(rest / a.xt_per_row);
    const int C = g.in_c, c0 = cv * 16;
    const int oy0 = ys * YT;
    const bool relu = g.relu != 0, half_even = g.half_even != 0;

    // per-channel epilogue constants
    int init[16], sh[16];
    bool fast = !half_even;
#pragma unroll
    for (int w = 0; w < 4; w++) {
        v4i bb = {0, 0, 0, 0};
        if (a.bias != nullptr)
            bb = *reinterpret_cast<const v4i *>(a.bias + c0 + 4 * w);
        v4i ss;
        if (g.n_shift == 1) {
            const int s = a.shift[0];
            ss = v4i{s, s, s, s};
        } else {
            ss = *reinterpret_cast<const v4i *>(a.shift + c0 + 4 * w);
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
            init[4 * w + r] = bb[r];
            sh[4 * w + r] = ss[r];
            const int s = ss[r];
            if (s < 1 || s > 31) {
                fast = false;
            } else {
                const long long start = (long long)bb[r] + (1ll << (s - 1));
                const long long mag = (start < 0 ? -start : start) + 9ll * 16384;
                if (mag >= (1ll << (31 - max(0, 8 - s))))
                    fast = false;
            }
        }
    }
    if (fast) {
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const int s = sh[i];
            init[i] += 1 << (s - 1);
            sh[i] = max(0, 8 - s) | (max(0, s - 8) << 8);
        }
    }

    int acc[YT][16];
#pragma unroll
    for (int y = 0; y < YT; y++)
#pragma unroll
        for (int i = 0; i < 16; i++)
            acc[y][i] = init[i];

    const int8_t *img = a.in + (long long)n * g.in_h * g.in_w * C + c0;
    const int ixl = ox * g.stride_w - g.pad_left; // input column of kx = 0
#pragma unroll
    for (int ky = 0; ky < 3; ky++) {
        // weights of this filter row, each dword masked down to one byte per accumulator
        int wm[3][16];
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const v4i wq = *reinterpret_cast<const v4i *>(a.w + (ky * 3 + kx) * C + c0);
#pragma unroll
            for (int w = 0; w < 4; w++) {
                wm[kx][4 * w + 0] = wq[w] & 0x000000ff;
                wm[kx][4 * w + 1] = wq[w] & 0x0000ff00;
                wm[kx][4 * w + 2] = wq[w] & 0x00ff0000;
                wm[kx][4 * w + 3] = wq[w] & (int)0xff000000;
            }
        }
#pragma unroll
        for (int y = 0; y < YT; y++) {
            const int iy = (oy0 + y) * g.stride_h - g.pad_top + ky;
            if ((unsigned)iy >= (unsigned)g.in_h || oy0 + y >= g.out_h)
                continue;
            const int8_t *row = img + (long long)iy * g.in_w * C;
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                const int ix = ixl + kx;
                if ((unsigned)ix >= (unsigned)g.in_w)
                    continue;
                const v4i v = *reinterpret_cast<const v4i *>(row + (long long)ix * C);
#pragma unroll
                for (int w = 0; w < 4; w++)
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        acc[y][4 * w + r] = __builtin_amdgcn_sdot4(v[w], wm[kx][4 * w + r], acc[y][4 * w + r], false);
            }
        }
    }

#pragma unroll
    for (int y = 0; y < YT; y++) {
        if (oy0 + y >= g.out_h)
            continue;
        v4i out;
#pragma unroll
        for (int w = 0; w < 4; w++) {
            int word;
            if (fast) {
                int tv[4];
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const int s2 = sh[4 * w + r];
                    const int v = (int)((unsigned)acc[y][4 * w + r] << (s2 & 31)) >> (s2 >> 8);
                    tv[r] = relu ? max(v, 0) : v;
                }
                const int p01 = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(tv[0], tv[1]));
                const int p23 = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(tv[2], tv[3]));
                word = (int)__builtin_amdgcn_perm((unsigned)p23, (unsigned)p01, 0x07050301u);
            } else {
                int q[4];
#pragma unroll
                for (int r = 0; r < 4; r++)
                    q[r] = requant_s8(acc[y][4 * w + r], sh[4 * w + r], relu, half_even);
                word = pack4_s8(q[0], q[1], q[2], q[3]);
            }
            if (a.lut != nullptr)
                word = pack4_s8(a.lut[(int)(int8_t)word + 128], a.lut[(int)(int8_t)(word >> 8) + 128],
                                a.lut[(int)(int8_t)(word >> 16) + 128], a.lut[(word >> 24) + 128]);
            out[w] = word;
        }
        *reinterpret_cast<v4i *>(a.out + (((long long)n * g.out_h + oy0 + y) * g.out_w + ox) * C + c0) = out;
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
    if (g.k_h == 3 && g.k_w == 3 && g.dil_h == 1 && g.dil_w == 1 && (g.in_c & 15) == 0 && (align & 15) == 0 && bias_ok &&
        shift_ok) {
        constexpr int YT = 4;
        a.cq = g.in_c / 16;
        a.xt_per_row = (g.out_h + YT - 1) / YT; // strips of YT output rows per image
        a.n_items = (long long)g.batch * a.xt_per_row * g.out_w * a.cq;
        const unsigned blocks = (unsigned)((a.n_items + 255) / 256);
        hipLaunchKernelGGL(depthwise_s8_3x3_vec16_kernel<YT>, dim3(blocks), dim3(256), 0, stream, a);
    } else if ((g.in_c & 3) == 0 && (align & 3) == 0 && bias_ok && shift_ok) {
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
