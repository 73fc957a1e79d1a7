// Depthwise int8 convolution (up to 12 filter taps, channels % 16 == 0) for gfx950, with the matrix
// pipe doing the byte multiply-accumulates.
//
// What it computes is depthwise_conv2d_33c1 / _hwc1 (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:19-65)
// under dwconv_operation_shell's window clipping (esp-dl/dl/base/dl_base.hpp:1852-2102) and the n_wise
// epilogue (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210).
//
// The operator is bandwidth-bound (about 7 operations per byte), but one multiply-accumulate per
// channel on the vector ALU costs more instruction issue than the memory system leaves time for:
// measured, the VALU form of this kernel was instruction-bound at a quarter of HBM speed.  So the
// products go to v_mfma_i32_16x16x64_i8 with a *diagonal* operand A: for a tile of 16 channels the
// reduction axis is (tap, channel), A[i][(tap, c)] = w[tap][i] when c == i and 0 otherwise, and
// operand B is simply the 16-byte NHWC vector of the tap's input pixel.  15/16 of the MFMA's
// products are zeros, which is free: three MFMAs finish 16 pixels x 16 channels x 9 taps, and the
// vector ALU is left with address arithmetic and the three-instruction epilogue.
//
// A wavefront owns 16 consecutive output pixels and one block of 16*NT channels (NT <= 4).  Lane
// (pixel j, quad g) loads, for k step ks, the NT vectors of tap 4*ks + g; its dwords are regrouped
// (register renaming only) so that tile t holds channels 4*NT*q + 4*t + r, which makes every lane end
// up with 4*NT consecutive output channels: one 16-byte store per lane, 64 contiguous bytes per
// pixel.  Operand A, start values (bias + rounding constant) and shifts sit in LDS, written once per
// persistent workgroup; the loads of the next pixel set are in flight while the current one is in the
// MFMA / epilogue phase.
#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

constexpr int kThreads = 256;
constexpr int kKs = 3; // k steps of 4 taps: up to 12 taps

struct DwMfmaArgs {
    const int8_t *in;
    const int8_t *w;
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
    int8_t *out;
    ConvGeom g;
    int taps;     // k_h * k_w
    int n_cblk;   // channel blocks of 64 (the last one may be narrower)
    int n_sets;   // pixel sets of 64 pixels (4 waves x 16)
    long long npix;
    FastDiv fd_out_hw, fd_out_w, fd_k_w;
};

struct DwPixel {
    unsigned int pix;
    long long base; // byte offset of input pixel (iy0, ix0), may point outside the image
    int iy0, ix0;
    bool valid;
};

__device__ __forceinline__ void dw_decode(const DwMfmaArgs &a, int set, int wave, int col, DwPixel &px)
{
    const ConvGeom &g = a.g;
    const unsigned int pix = ((unsigned)set * 4u + (unsigned)wave) * 16u + col;
    px.pix = pix;
    px.valid = (long long)pix < a.npix;
    const unsigned int pc = px.valid ? pix : 0u;
    const unsigned int n = fastdiv(pc, a.fd_out_hw);
    const unsigned int rem = pc - n * a.fd_out_hw.d;
    const unsigned int oy = fastdiv(rem, a.fd_out_w);
    const unsigned int ox = rem - oy * a.fd_out_w.d;
    px.iy0 = (int)oy * g.stride_h - g.pad_top;
    px.ix0 = (int)ox * g.stride_w - g.pad_left;
    px.base = ((long long)n * g.in_h * g.in_w + (long long)px.iy0 * g.in_w + px.ix0) * g.in_c;
}

// Operand B of all k steps for one lane: NT vectors per step, zeros outside the image.
template <int NT>
__device__ __forceinline__ void dw_load(const DwMfmaArgs &a, const DwPixel &px, int cb, const int (&dy)[kKs],
                                        const int (&dx)[kKs], v4i (&b)[kKs][NT])
{
    const ConvGeom &g = a.g;
#pragma unroll
    for (int ks = 0; ks < kKs; ks++) {
        const int iy = px.iy0 + dy[ks], ix = px.ix0 + dx[ks];
        const bool ok = px.valid && dy[ks] >= 0 && (unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w;
        const int8_t *src = a.in + px.base + ((long long)dy[ks] * g.in_w + dx[ks]) * g.in_c + cb;
#pragma unroll
        for (int q = 0; q < NT; q++)
            b[ks][q] = ok ? *reinterpret_cast<const v4i *>(src + 16 * q) : v4i{0, 0, 0, 0};
    }
}

template <int NT>
__device__ __forceinline__ void dw_block(const DwMfmaArgs &a, unsigned char *smem, int cb)
{
    // LDS: operand A [kKs][NT][64 lanes] x 16 B, then start values and shifts for 16*NT channels
    v4i *a_l = reinterpret_cast<v4i *>(smem);
    int *init_l = reinterpret_cast<int *>(smem + kKs * NT * 1024);
    int *shift_l = init_l + 16 * NT;
    int *lsh_l = shift_l + 16 * NT;
    int8_t *lut_l = reinterpret_cast<int8_t *>(lsh_l + 16 * NT);

    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int C = g.in_c;
    const bool relu = g.relu != 0, half_even = g.half_even != 0, has_lut = a.lut != nullptr;

    // taps handled by this lane's quad in each k step
    int dy[kKs], dx[kKs];
#pragma unroll
    for (int ks = 0; ks < kKs; ks++) {
        const int tap = 4 * ks + quad;
        if (tap < a.taps) {
            const int ky = (int)fastdiv((unsigned)tap, a.fd_k_w), kx = tap - ky * g.k_w;
            dy[ks] = ky * g.dil_h;
            dx[ks] = kx * g.dil_w;
        } else {
            dy[ks] = -1; // marks "no tap"
            dx[ks] = 0;
        }
    }

    const TileSeq seq = xcd_tile_sequence(a.n_sets);
    int set = seq.first;
    DwPixel px;
    v4i b[kKs][NT];
    if (set < seq.end) {
        dw_decode(a, set, wave, col, px);
        dw_load<NT>(a, px, cb, dy, dx, b);
    }

    // diagonal operand A: unit (ks, t, lane = (i, gk)) has one non-zero byte, position i, value
    // w[tap 4*ks + gk][channel 4*NT*(i/4) + 4*t + i%4]
    for (int u = tid; u < kKs * NT * 64; u += kThreads) {
        const int l = u & 63, t = (u >> 6) % NT, ks = u / (64 * NT);
        const int i = l & 15, gk = l >> 4;
        const int tap = 4 * ks + gk;
        int words[4] = {0, 0, 0, 0};
        if (tap < a.taps) {
            const int ch = cb + 4 * NT * (i >> 2) + 4 * t + (i & 3);
            const int wv = (unsigned char)a.w[(long long)tap * C + ch];
            words[i >> 2] = wv << (8 * (i & 3));
        }
        a_l[u] = v4i{words[0], words[1], words[2], words[3]};
    }
    // epilogue constants; the short form needs every shift in 1..31 and no possible overflow
    const long long mac_bound = (long long)a.taps * 16384;
    int ok_local = 1;
    for (int c = tid; c < 16 * NT; c += kThreads) {
        const int s = a.shift[g.n_shift == 1 ? 0 : cb + c];
        const long long bv = a.bias != nullptr ? (long long)a.bias[cb + c] : 0;
        if (s < 1 || s > 31) {
            ok_local = 0;
        } else {
            const long long start = bv + (1ll << (s - 1));
            if ((start < 0 ? -start : start) + mac_bound >= (1ll << (31 - max(0, 8 - s))))
                ok_local = 0;
        }
    }
    if (has_lut)
        lut_l[tid] = a.lut[tid];
    const bool fast = __syncthreads_and(ok_local) != 0;
    for (int c = tid; c < 16 * NT; c += kThreads) {
        const int s = a.shift[g.n_shift == 1 ? 0 : cb + c];
        const int bv = a.bias != nullptr ? a.bias[cb + c] : 0;
        init_l[c] = fast ? bv + (1 << (s - 1)) - (half_even ? 1 : 0) : bv; // pack_fast4<5> starts one lower
        shift_l[c] = fast ? max(0, s - 8) : s;
        lsh_l[c] = fast ? max(0, 8 - s) : 0;
    }
    __syncthreads();
    const int floor_pk = relu ? 0 : (int)0x80008000u;

    // this lane's 4*NT consecutive channels: cb + 4*NT*quad + [0, 4*NT)
    v4i init[NT], ss[NT], ls[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        init[t] = *reinterpret_cast<const v4i *>(init_l + 4 * NT * quad + 4 * t);
        ss[t] = *reinterpret_cast<const v4i *>(shift_l + 4 * NT * quad + 4 * t);
        ls[t] = *reinterpret_cast<const v4i *>(lsh_l + 4 * NT * quad + 4 * t);
    }

    for (; set < seq.end; set += seq.step) {
        DwPixel px_next;
        v4i bn[kKs][NT];
        const int set_next = set + seq.step;
        if (set_next < seq.end) {
            dw_decode(a, set_next, wave, col, px_next);
            dw_load<NT>(a, px_next, cb, dy, dx, bn);
        }

        v4i acc[NT];
#pragma unroll
        for (int t = 0; t < NT; t++)
            acc[t] = init[t];
#pragma unroll
        for (int ks = 0; ks < kKs; ks++) {
            if (4 * ks < a.taps) {
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    // tile t reads dword NT*q + t of the lane's 4*NT loaded dwords, q = 0..3
                    v4i bop;
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int d = NT * q + t; // compile-time after unrolling
                        bop[q] = b[ks][d >> 2][d & 3];
                    }
                    const v4i aop = a_l[(ks * NT + t) * 64 + lane];
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, bop, acc[t], 0, 0, 0);
                }
            }
        }

        if (px.valid) {
            int words[NT];
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if (fast) {
                    words[t] = half_even ? pack_fast4<5>(acc[t], ls[t], ss[t], floor_pk) : pack_fast4<1>(acc[t], ls[t], ss[t], floor_pk);
                } else {
                    int q[4];
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        q[r] = requant_s8(acc[t][r], ss[t][r], relu, half_even);
                    words[t] = pack4_s8(q[0], q[1], q[2], q[3]);
                }
                if (has_lut) {
                    const int w = words[t];
                    words[t] = pack4_s8(lut_l[(int)(int8_t)w + 128], lut_l[(int)(int8_t)(w >> 8) + 128],
                                        lut_l[(int)(int8_t)(w >> 16) + 128], lut_l[(w >> 24) + 128]);
                }
            }
            int8_t *dst = a.out + (long long)px.pix * C + cb + 4 * NT * quad;
            if (NT == 4) {
                *reinterpret_cast<v4i *>(dst) = v4i{words[0], words[NT > 1 ? 1 : 0], words[NT > 2 ? 2 : 0], words[NT > 3 ? 3 : 0]};
            } else {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    *reinterpret_cast<int *>(dst + 4 * t) = words[t];
            }
        }

        px = px_next;
#pragma unroll
        for (int ks = 0; ks < kKs; ks++)
#pragma unroll
            for (int q = 0; q < NT; q++)
                b[ks][q] = bn[ks][q];
    }
}

__global__ __launch_bounds__(kThreads) void depthwise_s8_mfma_kernel(const DwMfmaArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int cb = blockIdx.y * 64;
    const int nt = min(4, (a.g.in_c - cb) >> 4);
    switch (nt) { // uniform per workgroup
    case 4:
        dw_block<4>(a, smem, cb);
        break;
    case 3:
        dw_block<3>(a, smem, cb);
        break;
    case 2:
        dw_block<2>(a, smem, cb);
        break;
    default:
        dw_block<1>(a, smem, cb);
        break;
    }
}

} // namespace

bool depthwise_s8_mfma_supports(const ConvGeom &g, const void *in, const void *out)
{
    return (g.in_c & 15) == 0 && g.k_h * g.k_w <= 4 * kKs &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
}

hipError_t launch_depthwise_s8_mfma(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                    const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count,
                                    hipStream_t stream)
{
    DwMfmaArgs a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.out = out;
    a.g = g;
    a.taps = g.k_h * g.k_w;
    a.npix = (long long)g.batch * g.out_h * g.out_w;
    if (a.npix == 0)
        return hipSuccess;
    a.n_cblk = (g.in_c + 63) / 64;
    a.n_sets = (int)((a.npix + 63) / 64);
    a.fd_out_hw = make_fastdiv((unsigned)g.out_h * (unsigned)g.out_w);
    a.fd_out_w = make_fastdiv((unsigned)g.out_w);
    a.fd_k_w = make_fastdiv((unsigned)g.k_w);
    const int cus = cu_count > 0 ? cu_count : 256;
    // persistent: as many workgroups as are resident at once, over all channel blocks; x a multiple of 8 so that
    // blockIdx.x % 8 is the XCD of a workgroup (see xcd_tile_sequence)
    const size_t lds = (size_t)kKs * 4 * 1024 + 3 * 64 * sizeof(int) + 256;
    const int per_cu = resident_workgroups_per_cu(depthwise_s8_mfma_kernel, kThreads, lds);
    int gx = max(1, (cus * per_cu) / a.n_cblk);
    if (gx > a.n_sets)
        gx = a.n_sets;
    if (gx >= 8)
        gx &= ~7;
    hipLaunchKernelGGL(depthwise_s8_mfma_kernel, dim3((unsigned)gx, (unsigned)a.n_cblk), dim3(kThreads), lds, stream, a);
    return hipGetLastError();
}

} // namespace espdl
