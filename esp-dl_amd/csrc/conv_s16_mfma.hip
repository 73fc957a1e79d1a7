// Dense int16 convolution / Gemm for gfx950 on the int8 matrix pipe.
//
// What it computes is conv2d_11cn / _33cn / _hwcn for int16 (esp-dl/dl/base/dl_base_conv2d.cpp:9-163 with
// feature_t = int16_t, buffer_t = int64_t) under conv_operation_shell's window clipping: an exact 64-bit sum
// of int16 x int16 products, plus the int64 bias, shifted and rounded, saturated to int16.
//
// There is no int16 MFMA, so both operands are cut into two signed bytes that the int8 MFMA multiplies exactly.
// With h = the high byte of a 16-bit value v (signed) and l = its low byte xor 0x80 (signed, the low byte minus
// 128):  v = 256 h + l + 128.  For a pixel x = A + 128 and a weight w = B + 128 (A = 256 xh + xl, B = 256 wh + wl):
//   sum_k x w = sum_k A B + 128 sum_k A + 128 sum_k B + 16384 K
//             = 65536 HH + 256 (HL + LH) + LL  +  128 (256 sum_k xh + sum_k xl)  +  128 sum_k w
// with HH = sum_k xh wh and so on: four MFMA products per step into three int32 accumulators (HL and LH share
// one; none can overflow for K < 65536), the window sums of the pixel's own bytes (two dot-product instructions
// per loaded dword, summed over the four k slices of a tile at the end), and a per-filter constant.  Taps outside
// the image are x = 0, i.e. bytes (0, -128), which the same formula covers; k positions that pad the last step
// are zero bytes on both sides and add nothing.
//
// Layout of the work: a workgroup owns up to 64 filters, whose two byte planes it builds once in LDS in
// MFMA operand-A order for the whole reduction axis; each of its wavefronts then walks 16-pixel tiles,
// loading its lane's 16 channels of one tap (32 contiguous bytes) per k step straight from memory, sorting
// them into the two byte operands with two permutes and one xor per dword pair and issuing four MFMAs per
// 16 filters.
#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {
namespace {

constexpr int kThreads = 256; // per workgroup, or twice that (see the launch)
constexpr int kMaxRowTiles = 4;
constexpr size_t kLdsBudget = 140 * 1024;

struct S16MfmaArgs {
    const int16_t *in, *w;
    const int64_t *bias;
    const int32_t *shift;
    int16_t *out;
    ConvGeom g;
    int units_per_tap; // in_c / 16
    int n_units;       // taps * units_per_tap: 16-channel pieces of the reduction axis
    int ksteps;        // ceil(n_units / 4)
    int row_tiles;     // 16-filter tiles per workgroup
    int n_pixel_tiles; // ceil(batch * out_h * out_w / 16)
    int vec_out;       // out_c % 4 == 0 and out 8-byte aligned: four channels per store
    FastDiv fd_upt, fd_kw, fd_ow, fd_ohw;
};

// the high bytes / the low bytes of the four int16 held in two dwords, as one dword of four consecutive k
__device__ __forceinline__ int high_bytes(int m0, int m1)
{
    return (int)__builtin_amdgcn_perm((unsigned)m1, (unsigned)m0, 0x07050301u);
}
__device__ __forceinline__ int low_bytes(int m0, int m1)
{
    return (int)__builtin_amdgcn_perm((unsigned)m1, (unsigned)m0, 0x06040200u);
}

template <int THREADS>
__global__ __launch_bounds__(THREADS) void conv2d_s16_mfma_kernel(const S16MfmaArgs a)
{
    constexpr int kThreads = THREADS;
    extern __shared__ __align__(16) unsigned char smem[];
    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int OC = g.out_c, C = g.in_c;
    const int f0 = blockIdx.y * a.row_tiles * 16; // first filter of this workgroup
    const int n_f = a.row_tiles * 16;
    const long long ftap = (long long)g.k_h * g.k_w * C;

    // LDS: byte planes [row tile][high, low][k step][lane] x 16 bytes, then per filter: constant (int64), shift
    v4i *planes = reinterpret_cast<v4i *>(smem);
    const size_t plane_bytes = (size_t)a.row_tiles * 2 * a.ksteps * 64 * 16;
    long long *cst = reinterpret_cast<long long *>(smem + plane_bytes);
    int *shf = reinterpret_cast<int *>(cst + n_f);

    // per-filter sum of the weights, gathered while the planes are built (|sum| < 36000 * 2^15 fits int32)
    int *wsum = shf + n_f;
    for (int f = tid; f < n_f; f += kThreads)
        wsum[f] = 0;
    __syncthreads();
    // build the planes: one (row tile, k step, lane) slot of 16 weights at a time
    const int n_slots = a.row_tiles * a.ksteps * 64;
    for (int s = tid; s < n_slots; s += kThreads) {
        const int l = s & 63, ks = (s >> 6) % a.ksteps, rt = (s >> 6) / a.ksteps;
        const int f = f0 + 16 * rt + (l & 15);
        const int u = 4 * ks + (l >> 4);
        int wh[4] = {0, 0, 0, 0}, wl[4] = {0, 0, 0, 0};
        int part = 0;
        if (f < OC && u < a.n_units) {
            const int16_t *src = a.w + (long long)f * ftap + (long long)u * 16;
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const int v = src[e];
                wh[e >> 2] |= ((v >> 8) & 255) << (8 * (e & 3));
                wl[e >> 2] |= ((v & 255) ^ 128) << (8 * (e & 3));
                part += v;
            }
            atomicAdd(&wsum[16 * rt + (l & 15)], part);
        }
        const int base = ((rt * 2) * a.ksteps + ks) * 64 + l;
        planes[base] = v4i{wh[0], wh[1], wh[2], wh[3]};
        planes[base + a.ksteps * 64] = v4i{wl[0], wl[1], wl[2], wl[3]};
    }
    __syncthreads();
    // per filter: bias + 128 * (sum of its weights), and its shift
    for (int f = tid; f < n_f; f += kThreads) {
        long long c = 0;
        int sh = 0;
        if (f0 + f < OC) {
            c = (a.bias != nullptr ? a.bias[f0 + f] : 0) + 128ll * (long long)wsum[f];
            sh = a.shift[g.n_shift == 1 ? 0 : f0 + f];
        }
        cst[f] = c;
        shf[f] = sh;
    }
    __syncthreads();

    const long long n_pix = (long long)g.batch * g.out_h * g.out_w;
    const bool relu = g.relu != 0, half_even = g.half_even != 0;
    const int waves_total = gridDim.x * (kThreads / 64);
    for (int tile = blockIdx.x * (kThreads / 64) + wave; tile < a.n_pixel_tiles; tile += waves_total) {
        const long long pix = (long long)tile * 16 + col;
        const bool pix_ok = pix < n_pix;
        const unsigned up = pix_ok ? (unsigned)pix : 0u;
        const unsigned n = fastdiv(up, a.fd_ohw);
        const unsigned rem = up - n * a.fd_ohw.d;
        const unsigned oy = fastdiv(rem, a.fd_ow);
        const unsigned ox = rem - oy * a.fd_ow.d;
        const int iy0 = (int)oy * g.stride_h - g.pad_top, ix0 = (int)ox * g.stride_w - g.pad_left;
        const int16_t *img = a.in + (long long)n * g.in_h * g.in_w * C;

        v4i acc[kMaxRowTiles][3]; // HH, HL + LH, LL
#pragma unroll
        for (int rt = 0; rt < kMaxRowTiles; rt++)
#pragma unroll
            for (int s = 0; s < 3; s++)
                acc[rt][s] = v4i{0, 0, 0, 0};
        int sum_h = 0, sum_l = 0; // this lane's part of sum_k xh and sum_k xl of its pixel

        for (int ks = 0; ks < a.ksteps; ks++) {
            // this lane's 16 channels of one tap as high bytes and low bytes - 128
            const int u = 4 * ks + quad;
            v4i xh = {0, 0, 0, 0}, xl = {0, 0, 0, 0};
            if (u < a.n_units) {
                const unsigned tap = fastdiv((unsigned)u, a.fd_upt);
                const unsigned c16 = (unsigned)u - tap * a.fd_upt.d;
                const unsigned ky = fastdiv(tap, a.fd_kw);
                const unsigned kx = tap - ky * a.fd_kw.d;
                const int iy = iy0 + (int)ky * g.dil_h, ix = ix0 + (int)kx * g.dil_w;
                v4i lo = {0, 0, 0, 0}, hi = {0, 0, 0, 0};
                if (pix_ok && (unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w) {
                    const v4i *src = reinterpret_cast<const v4i *>(img + ((long long)iy * g.in_w + ix) * C + c16 * 16);
                    lo = src[0];
                    hi = src[1];
                }
                const int d[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    xh[q] = high_bytes(d[2 * q], d[2 * q + 1]);
                    xl[q] = low_bytes(d[2 * q], d[2 * q + 1]) ^ (int)0x80808080u;
                    sum_h = __builtin_amdgcn_sdot4(xh[q], 0x01010101, sum_h, false);
                    sum_l = __builtin_amdgcn_sdot4(xl[q], 0x01010101, sum_l, false);
                }
            }
#pragma unroll
            for (int rt = 0; rt < kMaxRowTiles; rt++) {
                if (rt < a.row_tiles) { // uniform
                    const int base = ((rt * 2) * a.ksteps + ks) * 64 + lane;
                    const v4i wh = planes[base], wl = planes[base + a.ksteps * 64];
                    acc[rt][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wh, xh, acc[rt][0], 0, 0, 0);
                    acc[rt][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wl, xh, acc[rt][1], 0, 0, 0);
                    acc[rt][1] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wh, xl, acc[rt][1], 0, 0, 0);
                    acc[rt][2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wl, xl, acc[rt][2], 0, 0, 0);
                }
            }
        }
        // the four k slices of the tile (lanes col, col + 16, col + 32, col + 48) together hold the pixel's sums
        sum_h += __shfl_xor(sum_h, 16);
        sum_l += __shfl_xor(sum_l, 16);
        sum_h += __shfl_xor(sum_h, 32);
        sum_l += __shfl_xor(sum_l, 32);
        const long long pixel_term = 128ll * (256ll * sum_h + sum_l);

        // this lane: filters f0 + 16 rt + 4 quad + r of pixel `pix`
        if (pix_ok) {
#pragma unroll
            for (int rt = 0; rt < kMaxRowTiles; rt++) {
                if (rt < a.row_tiles) {
                    const int fl = 16 * rt + 4 * quad;
                    short q[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        long long v = cst[fl + r] + pixel_term;
                        v += ((long long)acc[rt][0][r] << 16) + ((long long)acc[rt][1][r] << 8) + (long long)acc[rt][2][r];
                        q[r] = (short)requant_s16(v, shf[fl + r], relu, half_even);
                    }
                    int16_t *dst = a.out + pix * OC + f0 + fl;
                    if (a.vec_out && f0 + fl + 3 < OC) {
                        int2 pk;
                        pk.x = (int)(unsigned short)q[0] | ((int)(unsigned short)q[1] << 16);
                        pk.y = (int)(unsigned short)q[2] | ((int)(unsigned short)q[3] << 16);
                        *reinterpret_cast<int2 *>(dst) = pk;
                    } else {
#pragma unroll
                        for (int r = 0; r < 4; r++)
                            if (f0 + fl + r < OC)
                                dst[r] = q[r];
                    }
                }
            }
        }
    }
}

struct S16Plan {
    bool ok;
    int row_tiles, ksteps, n_units;
    size_t lds;
};

S16Plan plan_s16(const ConvGeom &g)
{
    S16Plan p = {};
    if (g.in_c % 16 != 0)
        return p;
    const long long k = (long long)g.k_h * g.k_w * g.in_c;
    if (k > 36000) // the int32 accumulators stay exact up to 65535; longer reductions are rare enough to leave
        return p;  // to the 64-bit multiply-add kernel from here on

    p.n_units = (int)(k / 16);
    p.ksteps = (p.n_units + 3) / 4;
    int rt = min(kMaxRowTiles, (g.out_c + 15) / 16);
    for (; rt >= 1; rt--) {
        p.lds = (size_t)rt * 2 * p.ksteps * 64 * 16 + (size_t)rt * 16 * 16;
        if (p.lds <= kLdsBudget)
            break;
    }
    if (rt < 1)
        return p;
    p.row_tiles = rt;
    p.ok = true;
    return p;
}

} // namespace

bool conv2d_s16_mfma_supports(const ConvGeom &g, const void *in, const void *filter, const void *out)
{
    if ((reinterpret_cast<uintptr_t>(in) & 15) != 0 || (reinterpret_cast<uintptr_t>(filter) & 1) != 0 ||
        (reinterpret_cast<uintptr_t>(out) & 1) != 0)
        return false;
    if ((long long)g.batch * g.out_h * g.out_w >= (1ll << 31) - 16 || (long long)g.in_h * g.in_w * g.in_c >= (1ll << 31))
        return false;
    return plan_s16(g).ok;
}

hipError_t launch_conv2d_s16_mfma(const ConvGeom &g, const int16_t *in, const int16_t *filter, const int64_t *bias,
                                  const int32_t *shift, int16_t *out, int cu_count, hipStream_t stream)
{
    const long long n_pix = (long long)g.batch * g.out_h * g.out_w;
    if (n_pix == 0 || g.out_c == 0)
        return hipSuccess;
    const S16Plan p = plan_s16(g);
    if (!p.ok)
        return hipErrorInvalidValue;
    S16MfmaArgs a = {};
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.out = out;
    a.g = g;
    a.units_per_tap = g.in_c / 16;
    a.n_units = p.n_units;
    a.ksteps = p.ksteps;
    a.row_tiles = p.row_tiles;
    a.n_pixel_tiles = (int)((n_pix + 15) / 16);
    a.vec_out = (g.out_c % 4) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0;
    a.fd_upt = make_fastdiv((unsigned)a.units_per_tap);
    a.fd_kw = make_fastdiv((unsigned)g.k_w);
    a.fd_ow = make_fastdiv((unsigned)g.out_w);
    a.fd_ohw = make_fastdiv((unsigned)(g.out_h * g.out_w));
    static const hipError_t lds_opt_in = [] {
        const hipError_t e0 = hipFuncSetAttribute(reinterpret_cast<const void *>(conv2d_s16_mfma_kernel<kThreads>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBudget);
        const hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void *>(conv2d_s16_mfma_kernel<2 * kThreads>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLdsBudget);
        return e0 != hipSuccess ? e0 : e1;
    }();
    if (lds_opt_in != hipSuccess)
        return lds_opt_in;
    const int gy = (g.out_c + p.row_tiles * 16 - 1) / (p.row_tiles * 16);
    const int cus = cu_count > 0 ? cu_count : 256;
    const size_t fit = (size_t)(160 * 1024) / (p.lds > 0 ? p.lds : 1);
    const int per_cu = fit < 1 ? 1 : (fit > 4 ? 4 : (int)fit);
    int gx = max(1, (cus * per_cu) / gy);
    // Filter planes of a long reduction axis (72 KB for 3 x 3 x 64 channels) leave room for two workgroups per
    // compute unit; eight wavefronts each then keep the vector ALU, which sorts the pixels' bytes, busy where four
    // leave it idle half of the time (80 x 80 x 64 -> 64, 3 x 3, batch 64: 123 -> 88 us).
    const bool wide = per_cu <= 2;
    const int waves = (wide ? 2 * kThreads : kThreads) / 64;
    gx = min(gx, (a.n_pixel_tiles + waves - 1) / waves);
    if (wide)
        conv2d_s16_mfma_kernel<2 * kThreads><<<dim3((unsigned)gx, (unsigned)gy), dim3(2 * kThreads), p.lds, stream>>>(a);
    else
        conv2d_s16_mfma_kernel<kThreads><<<dim3((unsigned)gx, (unsigned)gy), dim3(kThreads), p.lds, stream>>>(a);
    return hipGetLastError();
}

} // namespace espdl
