// Inverted-residual block (1x1 expand conv -> depthwise conv -> 1x1 project conv [-> Add]) for int8 on
// gfx950 as ONE kernel: the expanded activation, which is 6x the size of the block's input and output
// and is what the three separate kernels spend their time writing to and reading from memory, lives
// only in LDS.
//
// Every stage computes exactly what the separate operators compute, in the same integer arithmetic,
// with the int8 result of each stage materialized (in LDS) before the next one reads it:
//   expand / project  conv2d_11cn + n_wise epilogue (esp-dl/dl/base/dl_base_conv2d.cpp:9-33;
//                     esp-dl/dl/base/dl_base_activate_buffer.hpp:10-74, 162-212)
//   depthwise         depthwise_conv2d_33c1 / _hwc1 under dwconv_operation_shell's window clipping
//                     (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:19-65; esp-dl/dl/base/dl_base.hpp:1852-2102)
//   Add               saturating int8 add without rescale (esp-dl/dl/base/dl_base_add.cpp:34-44)
// so a fused block is bit-identical to running Conv, Conv, Conv, Add modules one after the other.
//
// A workgroup (8 wavefronts) owns a th x tw tile of the block's output in one image and walks the
// expanded channels in chunks of 64:
//   1. the input patch (tile + filter halo, all input channels) is copied to LDS once;
//   2. per chunk: the chunk's expand filters and project filter columns are staged in LDS in MFMA
//      operand order (the next chunk's are already in flight in registers);
//      expand   = MFMA GEMM  [64 filters] x [patch pixels] over the input channels -> E (LDS, int8);
//                 positions outside the image are forced to zero: the depthwise zero padding pads the
//                 *expanded* activation;
//      depthwise= MFMA with a diagonal operand A, operand B straight from E            -> D (LDS, int8);
//      project  = MFMA GEMM  [out_c filters] x [tile pixels], K = the chunk's 64 channels, accumulated
//                 over the chunks in registers;
//   3. project epilogue -> LDS -> (+ residual read from global) -> contiguous 16-byte global stores.
// Without an expand stage (first block of MobileNetV2) the depthwise stage reads the input patch.
#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / 64;
constexpr int kKsDw = 3;    // depthwise k steps of 4 taps
constexpr int kMaxKse = 4;  // expand k steps of 64 input channels (in_c <= 256)
constexpr int kMaxAcc = 10; // project accumulator tiles per wavefront
constexpr int kMaxWe = 2;   // 16-byte expand-filter units per thread and chunk
constexpr int kMaxWp = 3;   // 16-byte project-filter units per thread and chunk
constexpr int kEs = 80;     // pixel stride of E and D in LDS: 64 channels + 16 (odd number of 16-byte units)

struct MbArgs {
    MbconvParams p;
    int has_expand;
    int taps;
    int th, tw, ph, pw;
    int p_in, p_out;       // pixels of the patch / of the tile
    int nct_in, nct_out;   // column tiles of 16 pixels
    int xs;                // LDS pixel stride of the input patch, bytes
    int kse;               // expand k steps
    int n_chunks;          // chunks of 64 expanded channels
    int nrt;               // project row tiles of 16 filters
    int n_acc;             // nrt * nct_out
    int os;                // LDS pixel stride of the output tile, bytes
    int out_vec;           // bytes per output store piece: 16 or 4
    int in_vec;            // bytes per input load piece: 16 or 4
    int tiles_x, tiles_y, n_units;
    FastDiv fd_tiles_x, fd_tiles_yx, fd_pw, fd_tw, fd_nct_out, fd_in_vecs, fd_out_vecs;
    int in_vecs, out_vecs; // pieces per pixel
    // LDS layout (byte offsets)
    int off_x, off_e, off_d, off_out, off_we, off_wp, off_wd, off_ce, off_cd, off_cp, off_pixtab, off_rctab, off_slottab;
};

struct TilePos {
    int n, y0, x0;
};

__device__ __forceinline__ TilePos mb_tile(const MbArgs &a, int unit)
{
    TilePos u;
    const unsigned n = fastdiv((unsigned)unit, a.fd_tiles_yx);
    const unsigned rem = (unsigned)unit - n * a.fd_tiles_yx.d;
    const unsigned ty = fastdiv(rem, a.fd_tiles_x);
    u.n = (int)n;
    u.y0 = (int)ty * a.th;
    u.x0 = (int)(rem - ty * a.fd_tiles_x.d) * a.tw;
    return u;
}

// Requantize four accumulators of one lane (channels c..c+3) to a packed dword.
__device__ __forceinline__ int mb_pack(const v4i &acc, const int *cst, int stride, int c, bool fast, bool relu,
                                       bool half_even, int floor_pk)
{
    // cst: [init | shift | lsh] arrays of `stride` ints each
    const v4i ss = *reinterpret_cast<const v4i *>(cst + stride + c);
    if (fast) {
        const v4i ls = *reinterpret_cast<const v4i *>(cst + 2 * stride + c);
        return pack_fast4<true>(acc, ls, ss, floor_pk);
    }
    int q[4];
#pragma unroll
    for (int r = 0; r < 4; r++)
        q[r] = requant_s8(acc[r], ss[r], relu, half_even);
    return pack4_s8(q[0], q[1], q[2], q[3]);
}

// Fill one stage's constant table [init | shift | lsh] for `n` channels (padded to `stride`), and
// decide whether the short epilogue is valid for all of them.  Returns the flag; contains barriers.
__device__ __forceinline__ bool mb_fill_consts(int *cst, int stride, int n, const int32_t *bias, const int32_t *shift,
                                               int n_shift, long long mac_bound, bool half_even, int tid)
{
    int ok_local = half_even ? 0 : 1;
    for (int c = tid; c < n; c += kThreads) {
        const int s = shift[n_shift == 1 ? 0 : c];
        const long long bv = bias != nullptr ? (long long)bias[c] : 0;
        if (s < 1 || s > 31) {
            ok_local = 0;
        } else {
            const long long start = bv + (1ll << (s - 1));
            if ((start < 0 ? -start : start) + mac_bound >= (1ll << (31 - max(0, 8 - s))))
                ok_local = 0;
        }
    }
    const bool fast = __syncthreads_and(ok_local) != 0;
    for (int c = tid; c < stride; c += kThreads) {
        int s = 0, bv = 0;
        if (c < n) {
            s = shift[n_shift == 1 ? 0 : c];
            bv = bias != nullptr ? bias[c] : 0;
        }
        cst[c] = (fast && c < n) ? bv + (1 << (s - 1)) : bv;
        cst[stride + c] = fast ? max(0, s - 8) : s;
        cst[2 * stride + c] = fast ? max(0, 8 - s) : 0;
    }
    return fast;
}

// Filter units of one chunk: global -> registers.
__device__ __forceinline__ void mb_fetch_weights(const MbArgs &a, int chunk, int tid, v4i (&we)[kMaxWe],
                                                 v4i (&wp)[kMaxWp])
{
    const MbconvParams &p = a.p;
    const int e0 = chunk * 64;
    const int ng = min(4, (p.exp_c - e0) >> 4);
    if (a.has_expand) {
        // unit u = (ks * ng + t) * 64 + lane: row i of tile t is channel e0 + 4*ng*(i/4) + 4*t + i%4,
        // the lane's 16 k positions are input channels 64*ks + 16*gk ...
#pragma unroll
        for (int j = 0; j < kMaxWe; j++) {
            const int u = tid + j * kThreads;
            we[j] = v4i{0, 0, 0, 0};
            if (u < a.kse * ng * 64) {
                const int lane = u & 63, t = (u >> 6) % ng, ks = (u >> 6) / ng;
                const int i = lane & 15, gk = lane >> 4;
                const int ch = e0 + 4 * ng * (i >> 2) + 4 * t + (i & 3);
                const int k0 = 64 * ks + 16 * gk;
                const int8_t *src = p.w_expand + (long long)ch * p.in_c + k0;
                if (a.in_vec == 16) {
                    if (k0 < p.in_c)
                        we[j] = *reinterpret_cast<const v4i *>(src);
                } else {
#pragma unroll
                    for (int d = 0; d < 4; d++)
                        if (k0 + 4 * d < p.in_c)
                            we[j][d] = *reinterpret_cast<const int *>(src + 4 * d);
                }
            }
        }
    }
    // project: unit u = rt * 64 + lane: row i is filter 16*rt + i, k positions are expanded channels
    // e0 + 16*gk ... (zeros past exp_c and past out_c)
#pragma unroll
    for (int j = 0; j < kMaxWp; j++) {
        const int u = tid + j * kThreads;
        wp[j] = v4i{0, 0, 0, 0};
        if (u < a.nrt * 64) {
            const int lane = u & 63, rt = u >> 6;
            const int f = 16 * rt + (lane & 15), e = e0 + 16 * (lane >> 4);
            if (f < p.out_c && e < p.exp_c)
                wp[j] = *reinterpret_cast<const v4i *>(p.w_project + (long long)f * p.exp_c + e);
        }
    }
}

__device__ __forceinline__ void mb_store_weights(const MbArgs &a, int chunk, int tid, unsigned char *smem,
                                                 const v4i (&we)[kMaxWe], const v4i (&wp)[kMaxWp])
{
    const int ng = min(4, (a.p.exp_c - chunk * 64) >> 4);
    if (a.has_expand) {
#pragma unroll
        for (int j = 0; j < kMaxWe; j++) {
            const int u = tid + j * kThreads;
            if (u < a.kse * ng * 64)
                *reinterpret_cast<v4i *>(smem + a.off_we + 16 * u) = we[j];
        }
    }
#pragma unroll
    for (int j = 0; j < kMaxWp; j++) {
        const int u = tid + j * kThreads;
        if (u < a.nrt * 64)
            *reinterpret_cast<v4i *>(smem + a.off_wp + 16 * u) = wp[j];
    }
}

// Requantize four accumulators with the stage constants held in registers.
__device__ __forceinline__ int mb_pack_r(const v4i &acc, const v4i &ss, const v4i &ls, bool fast, bool relu,
                                         bool half_even, int floor_pk)
{
    if (fast)
        return pack_fast4<true>(acc, ls, ss, floor_pk);
    int q[4];
#pragma unroll
    for (int r = 0; r < 4; r++)
        q[r] = requant_s8(acc[r], ss[r], relu, half_even);
    return pack4_s8(q[0], q[1], q[2], q[3]);
}

constexpr int kMaxCtE = 12; // expand column tiles per wavefront (two wavefronts share a row tile)
constexpr int kMaxCtD = 8;  // depthwise column tiles per wavefront (two wavefronts share a channel group)
constexpr int kAccBatch = 5;

__global__ __launch_bounds__(kThreads, 2) void mbconv_s8_fused_kernel(const MbArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const MbconvParams &p = a.p;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int sub = wave & 3, half = wave >> 2; // row tile / channel group of this wavefront, and which half of the columns
    const bool half_even = p.half_even != 0;
    const int ec_pad = a.n_chunks * 64; // expanded channels padded to whole chunks
    const int oc_pad = a.nrt * 16;

    int *cst_e = reinterpret_cast<int *>(smem + a.off_ce); // [3][ec_pad]
    int *cst_d = reinterpret_cast<int *>(smem + a.off_cd); // [3][ec_pad]
    int *cst_p = reinterpret_cast<int *>(smem + a.off_cp); // [3][oc_pad]
    int *pixtab = reinterpret_cast<int *>(smem + a.off_pixtab);
    unsigned char *x_l = smem + a.off_x;
    unsigned char *e_l = smem + a.off_e;
    unsigned char *d_l = smem + a.off_d;
    unsigned char *out_l = smem + a.off_out;

    // ---- once per workgroup: constants of the three stages, depthwise filter, pixel table
    bool fast_e = false;
    if (a.has_expand)
        fast_e = mb_fill_consts(cst_e, ec_pad, p.exp_c, p.b_expand, p.s_expand, p.n_s_expand,
                                (long long)p.in_c * 16384, half_even, tid);
    const bool fast_d = mb_fill_consts(cst_d, ec_pad, p.exp_c, p.b_dw, p.s_dw, p.n_s_dw, (long long)a.taps * 16384,
                                       half_even, tid);
    const bool fast_p = mb_fill_consts(cst_p, oc_pad, p.out_c, p.b_project, p.s_project, p.n_s_project,
                                       (long long)p.exp_c * 16384, half_even, tid);
    for (int i = tid; i < a.taps * p.exp_c; i += kThreads)
        smem[a.off_wd + i] = (unsigned char)p.w_dw[i];
    // the depthwise stage reads from E (stride kEs) or, without expand, from the input patch (stride xs)
    const int dw_stride = a.has_expand ? kEs : a.xs;
    for (int q = tid; q < a.nct_out * 16; q += kThreads) {
        int off = 0;
        if (q < a.p_out) {
            const unsigned qy = fastdiv((unsigned)q, a.fd_tw);
            const unsigned qx = (unsigned)q - qy * a.fd_tw.d;
            off = (int)((qy * p.stride_h * a.pw + qx * p.stride_w) * dw_stride);
        }
        pixtab[q] = off;
    }
    // project accumulator tile t -> (row tile | column tile << 8); read back inside the loops so that
    // the per-tile addresses are formed where they are used instead of living in registers throughout
    int *slottab = reinterpret_cast<int *>(smem + a.off_slottab);
    for (int t = tid; t < kMaxAcc * kWaves; t += kThreads) {
        const int rt = (int)fastdiv((unsigned)t, a.fd_nct_out);
        slottab[t] = t < a.n_acc ? (rt | ((t - rt * a.nct_out) << 8)) : 0;
    }
    // (row | col << 16) of every patch pixel, -1 past the patch
    int *rctab = reinterpret_cast<int *>(smem + a.off_rctab);
    for (int q = tid; q < a.nct_in * 16; q += kThreads) {
        int rc = -1;
        if (q < a.p_in) {
            const unsigned py = fastdiv((unsigned)q, a.fd_pw);
            rc = (int)(py | (((unsigned)q - py * a.fd_pw.d) << 16));
        }
        rctab[q] = rc;
    }
    int tapoff[kKsDw];
#pragma unroll
    for (int ks = 0; ks < kKsDw; ks++) {
        const int tap = 4 * ks + quad;
        tapoff[ks] = 0;
        if (tap < a.taps) {
            const int ky = tap / p.k_w, kx = tap - ky * p.k_w;
            tapoff[ks] = (ky * p.dil_h * a.pw + kx * p.dil_w) * dw_stride;
        }
    }
    const int floor_e = p.relu_expand ? 0 : (int)0x80008000u;
    const int floor_d = p.relu_dw ? 0 : (int)0x80008000u;
    const int floor_p = p.relu_project ? 0 : (int)0x80008000u;
    __syncthreads();
    // patch pixel (row | col << 16) of this lane in each of the wavefront's expand column tiles
    // is recomputed per tile into a bit mask of the pixels that lie inside the image

    const TileSeq seq = xcd_tile_sequence(a.n_units);
    for (int unit = seq.first; unit < seq.end; unit += seq.step) {
        const TilePos u = mb_tile(a, unit);
        const int iy0 = u.y0 * p.stride_h - p.pad_top, ix0 = u.x0 * p.stride_w - p.pad_left;

        // ---- filters of chunk 0 on their way while the patch is copied
        v4i we_r[kMaxWe], wp_r[kMaxWp];
        mb_fetch_weights(a, 0, tid, we_r, wp_r);

        // ---- 1. input patch -> LDS (zeros outside the image)
        {
            const int8_t *base = p.in + (((long long)u.n * p.in_h + iy0) * p.in_w + ix0) * p.in_c;
            const int n_vec = a.p_in * a.in_vecs;
            for (int k = tid; k < n_vec; k += kThreads) {
                const unsigned pix = fastdiv((unsigned)k, a.fd_in_vecs);
                const unsigned v = (unsigned)k - pix * a.fd_in_vecs.d;
                const unsigned py = fastdiv(pix, a.fd_pw);
                const unsigned px = pix - py * a.fd_pw.d;
                const int iy = iy0 + (int)py, ix = ix0 + (int)px;
                const bool ok = (unsigned)iy < (unsigned)p.in_h && (unsigned)ix < (unsigned)p.in_w;
                const int8_t *src = base + ((long long)py * p.in_w + px) * p.in_c + v * a.in_vec;
                unsigned char *dst = x_l + pix * a.xs + v * a.in_vec;
                if (a.in_vec == 16)
                    *reinterpret_cast<v4i *>(dst) = ok ? *reinterpret_cast<const v4i *>(src) : v4i{0, 0, 0, 0};
                else
                    *reinterpret_cast<int *>(dst) = ok ? *reinterpret_cast<const int *>(src) : 0;
            }
        }
        // ---- project accumulators start at bias (+ rounding constant)
        v4i acc[kMaxAcc];
#pragma unroll
        for (int s = 0; s < kMaxAcc; s++) {
            const int t = wave + s * kWaves;
            if (t < a.n_acc) {
                const int rt = slottab[t] & 0xff;
                acc[s] = *reinterpret_cast<const v4i *>(cst_p + 16 * rt + 4 * quad);
            }
        }

        for (int chunk = 0; chunk < a.n_chunks; chunk++) {
            const int e0 = chunk * 64;
            const int ng = min(4, (p.exp_c - e0) >> 4);
            // the previous chunk's project reads of D and of the filters, and (chunk 0) the previous
            // tile's output copy, are finished before the filters are overwritten
            __syncthreads();
            mb_store_weights(a, chunk, tid, smem, we_r, wp_r);
            __syncthreads();
            if (chunk + 1 < a.n_chunks)
                mb_fetch_weights(a, chunk + 1, tid, we_r, wp_r); // in flight during this chunk's stages

            // ---- 2a. expand: this wavefront owns row tile `sub` (channels e0 + 4*ng*q + 4*sub + r of
            // lane quad q) and every second column tile; E[patch pixel][4*ng*q + 4*sub + r]
            if (a.has_expand) {
                if (sub < ng) {
                    const int c = e0 + 4 * ng * quad + 4 * sub;
                    const v4i init = *reinterpret_cast<const v4i *>(cst_e + c);
                    const v4i ss = *reinterpret_cast<const v4i *>(cst_e + ec_pad + c);
                    const v4i ls = *reinterpret_cast<const v4i *>(cst_e + 2 * ec_pad + c);
                    v4i aop[kMaxKse];
#pragma unroll
                    for (int ks = 0; ks < kMaxKse; ks++)
                        if (ks < a.kse)
                            aop[ks] = *reinterpret_cast<const v4i *>(smem + a.off_we + 16 * ((ks * ng + sub) * 64 + lane));
                    const unsigned char *bsrc = x_l + col * a.xs + 16 * quad;
                    unsigned char *dst = e_l + col * kEs + 4 * ng * quad + 4 * sub;
                    v4i b[kMaxKse];
#pragma unroll
                    for (int ks = 0; ks < kMaxKse; ks++)
                        if (ks < a.kse)
                            b[ks] = *reinterpret_cast<const v4i *>(bsrc + half * 16 * a.xs + 64 * ks);
#pragma unroll 1
                    for (int s = 0; s < kMaxCtE; s++) {
                        const int ct = half + 2 * s;
                        if (ct >= a.nct_in) // uniform per wavefront
                            break;
                        {
                            v4i r = init;
#pragma unroll
                            for (int ks = 0; ks < kMaxKse; ks++)
                                if (ks < a.kse)
                                    r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], b[ks], r, 0, 0, 0);
                            if (ct + 2 < a.nct_in) {
#pragma unroll
                                for (int ks = 0; ks < kMaxKse; ks++)
                                    if (ks < a.kse)
                                        b[ks] = *reinterpret_cast<const v4i *>(bsrc + (ct + 2) * 16 * a.xs + 64 * ks);
                            }
                            const int word = mb_pack_r(r, ss, ls, fast_e, p.relu_expand != 0, half_even, floor_e);
                            // outside the image the expanded activation is the depthwise zero padding
                            const int rc = rctab[ct * 16 + col];
                            const int iy = iy0 + (rc & 0xffff), ix = ix0 + (rc >> 16);
                            const bool inside = rc >= 0 && (unsigned)iy < (unsigned)p.in_h && (unsigned)ix < (unsigned)p.in_w;
                            *reinterpret_cast<int *>(dst + ct * 16 * kEs) = inside ? word : 0;
                        }
                    }
                }
                __syncthreads();
            }

            // ---- 2b. depthwise: this wavefront owns channel group `sub` and every second column tile;
            // D[tile pixel][16*sub + 4*q + r]
            {
                if (sub < ng) {
                    const unsigned char *src_l = (a.has_expand ? e_l : x_l + e0) + 16 * sub;
                    const int sel = col >> 2;
                    v4i aop[kKsDw];
#pragma unroll
                    for (int ks = 0; ks < kKsDw; ks++) {
                        const int tap = 4 * ks + quad;
                        int d = 0;
                        if (tap < a.taps)
                            d = (int)smem[a.off_wd + tap * p.exp_c + e0 + 16 * sub + col] << (8 * (col & 3));
                        aop[ks] = v4i{sel == 0 ? d : 0, sel == 1 ? d : 0, sel == 2 ? d : 0, sel == 3 ? d : 0};
                    }
                    const int c = e0 + 16 * sub + 4 * quad;
                    const v4i init = *reinterpret_cast<const v4i *>(cst_d + c);
                    const v4i ss = *reinterpret_cast<const v4i *>(cst_d + ec_pad + c);
                    const v4i ls = *reinterpret_cast<const v4i *>(cst_d + 2 * ec_pad + c);
                    unsigned char *dst = d_l + col * kEs + 16 * sub + 4 * quad;
                    v4i b[kKsDw];
                    {
                        const int po = pixtab[min(half, a.nct_out - 1) * 16 + col];
#pragma unroll
                        for (int ks = 0; ks < kKsDw; ks++)
                            b[ks] = *reinterpret_cast<const v4i *>(src_l + po + tapoff[ks]);
                    }
                    // patch offset of the lane's pixel in the column tile after this one (two ahead of the reads)
                    int po_next = pixtab[min(half + 2, a.nct_out - 1) * 16 + col];
#pragma unroll 1
                    for (int s = 0; s < kMaxCtD; s++) {
                        const int ct = half + 2 * s;
                        if (ct >= a.nct_out) // uniform per wavefront
                            break;
                        {
                            v4i r = init;
#pragma unroll
                            for (int ks = 0; ks < kKsDw; ks++)
                                if (4 * ks < a.taps)
                                    r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], b[ks], r, 0, 0, 0);
                            if (ct + 2 < a.nct_out) {
#pragma unroll
                                for (int ks = 0; ks < kKsDw; ks++)
                                    b[ks] = *reinterpret_cast<const v4i *>(src_l + po_next + tapoff[ks]);
                                po_next = pixtab[min(ct + 4, a.nct_out - 1) * 16 + col];
                            }
                            const int word = mb_pack_r(r, ss, ls, fast_d, p.relu_dw != 0, half_even, floor_d);
                            *reinterpret_cast<int *>(dst + ct * 16 * kEs) = word;
                        }
                    }
                }
                __syncthreads();
            }

            // ---- 2c. project: acc[rt][ct] += Wp[rt][chunk] x D[ct]; operands of a batch of tiles are
            // all requested before the first MFMA of the batch
#pragma unroll
            for (int s0 = 0; s0 < kMaxAcc; s0 += kAccBatch) {
                if (wave + s0 * kWaves < a.n_acc) { // uniform per wavefront
                    v4i aop[kAccBatch], b[kAccBatch];
#pragma unroll
                    for (int j = 0; j < kAccBatch; j++) {
                        const int t = wave + (s0 + j) * kWaves;
                        if (t < a.n_acc) {
                            const int e = slottab[t];
                            const int rt = e & 0xff, ct = e >> 8;
                            aop[j] = *reinterpret_cast<const v4i *>(smem + a.off_wp + 16 * (rt * 64 + lane));
                            b[j] = *reinterpret_cast<const v4i *>(d_l + (ct * 16 + col) * kEs + 16 * quad);
                        }
                    }
#pragma unroll
                    for (int j = 0; j < kAccBatch; j++)
                        if (wave + (s0 + j) * kWaves < a.n_acc)
                            acc[s0 + j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[j], b[j], acc[s0 + j], 0, 0, 0);
                }
            }
        }

        // ---- 3. project epilogue -> LDS tile (aliases the patch / E / D area) -> global
        __syncthreads();
#pragma unroll
        for (int s = 0; s < kMaxAcc; s++) {
            const int t = wave + s * kWaves;
            if (t < a.n_acc) {
                const int e = slottab[t];
                const int rt = e & 0xff, ct = e >> 8;
                const int c = 16 * rt + 4 * quad;
                const int word = mb_pack(acc[s], cst_p, oc_pad, c, fast_p, p.relu_project != 0, half_even, floor_p);
                *reinterpret_cast<int *>(out_l + (ct * 16 + col) * a.os + c) = word;
            }
        }
        __syncthreads();
        {
            const int rows = min(a.th, p.out_h - u.y0), cols = min(a.tw, p.out_w - u.x0);
            const long long obase = (((long long)u.n * p.out_h + u.y0) * p.out_w + u.x0) * p.out_c;
            const int n_vec = a.p_out * a.out_vecs;
            for (int k = tid; k < n_vec; k += kThreads) {
                const unsigned q = fastdiv((unsigned)k, a.fd_out_vecs);
                const unsigned v = (unsigned)k - q * a.fd_out_vecs.d;
                const unsigned qy = fastdiv(q, a.fd_tw);
                const unsigned qx = q - qy * a.fd_tw.d;
                if ((int)qy < rows && (int)qx < cols) {
                    const long long g = obase + ((long long)qy * p.out_w + qx) * p.out_c + v * a.out_vec;
                    const unsigned char *src = out_l + q * a.os + v * a.out_vec;
                    if (a.out_vec == 16) {
                        v4i w = *reinterpret_cast<const v4i *>(src);
                        if (p.residual != nullptr) {
                            const v4i r = *reinterpret_cast<const v4i *>(p.residual + g);
#pragma unroll
                            for (int d = 0; d < 4; d++)
                                w[d] = sat_add4_s8(w[d], r[d]);
                        }
                        *reinterpret_cast<v4i *>(p.out + g) = w;
                    } else {
                        int w = *reinterpret_cast<const int *>(src);
                        if (p.residual != nullptr)
                            w = sat_add4_s8(w, *reinterpret_cast<const int *>(p.residual + g));
                        *reinterpret_cast<int *>(p.out + g) = w;
                    }
                }
            }
        }
        // the output tile aliases the patch area: its reads finish before the next patch copy
        __syncthreads();
    }
}

struct MbPlan {
    bool ok;
    MbArgs a;
    size_t lds;
};

// LDS a workgroup of this kernel may use: the largest size the runtime accepts as the kernel's
// dynamic LDS limit (tried once, from the device's per-workgroup maximum downwards).
size_t lds_limit()
{
    static const size_t limit = [] {
        int dev = 0, v = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess || v <= 0)
            v = 64 * 1024;
        (void)hipGetLastError();
        const bool trace = getenv("ESPDL_HIP_TRACE") != nullptr;
        for (int sz : {std::min(v, 160 * 1024), 128 * 1024, 96 * 1024, 80 * 1024, 64 * 1024}) {
            if (sz > v)
                continue;
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(mbconv_s8_fused_kernel),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, sz);
            if (trace)
                fprintf(stderr, "mbconv_s8_fused: dynamic LDS limit %d: %s\n", sz, hipGetErrorString(e));
            if (e == hipSuccess)
                return (size_t)sz;
            (void)hipGetLastError();
        }
        return (size_t)(48 * 1024);
    }();
    return limit;
}

inline int odd16(int bytes) // round up to an odd number of 16-byte units
{
    int u = (bytes + 15) / 16;
    if ((u & 1) == 0)
        u++;
    return 16 * u;
}

MbPlan mb_plan(const MbconvParams &p)
{
    MbPlan best;
    best.ok = false;
    const bool has_expand = p.w_expand != nullptr;
    if ((p.exp_c & 15) != 0 || (p.in_c & 3) != 0 || (p.out_c & 3) != 0 || p.k_h * p.k_w > 4 * kKsDw)
        return best;
    if (!has_expand && (p.in_c != p.exp_c))
        return best;
    if (has_expand && p.in_c > 64 * kMaxKse)
        return best;
    const int halo_h = (p.k_h - 1) * p.dil_h + 1, halo_w = (p.k_w - 1) * p.dil_w + 1;
    double best_cost = 1e30;
    static const int sizes[] = {1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 14, 16};
    for (int th : sizes) {
        if (th > p.out_h && th != 1)
            continue;
        for (int tw : sizes) {
            if (tw > p.out_w && tw != 1)
                continue;
            MbArgs a;
            a.p = p;
            a.has_expand = has_expand ? 1 : 0;
            a.taps = p.k_h * p.k_w;
            a.th = std::min(th, p.out_h);
            a.tw = std::min(tw, p.out_w);
            a.ph = (a.th - 1) * p.stride_h + halo_h;
            a.pw = (a.tw - 1) * p.stride_w + halo_w;
            a.p_in = a.ph * a.pw;
            a.p_out = a.th * a.tw;
            a.nct_in = (a.p_in + 15) / 16;
            a.nct_out = (a.p_out + 15) / 16;
            a.in_vec = (p.in_c & 15) == 0 && (reinterpret_cast<uintptr_t>(p.in) & 15) == 0 &&
                    (!has_expand || (reinterpret_cast<uintptr_t>(p.w_expand) & 15) == 0) ? 16 : 4;
            a.out_vec = (p.out_c & 15) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0 &&
                    (p.residual == nullptr || (reinterpret_cast<uintptr_t>(p.residual) & 15) == 0) ? 16 : 4;
            a.in_vecs = p.in_c / a.in_vec;
            a.out_vecs = p.out_c / a.out_vec;
            a.xs = odd16(p.in_c);
            a.kse = has_expand ? (p.in_c + 63) / 64 : 0;
            a.n_chunks = (p.exp_c + 63) / 64;
            a.nrt = (p.out_c + 15) / 16;
            a.n_acc = a.nrt * a.nct_out;
            a.os = odd16(a.nrt * 16);
            if (a.nct_in > 2 * kMaxCtE || a.nct_out > 2 * kMaxCtD || a.n_acc > kMaxAcc * kWaves)
                continue;
            if (a.kse * 4 * 64 > kMaxWe * kThreads || a.nrt * 64 > kMaxWp * kThreads)
                continue;
            // LDS: [patch | E | D] (the output tile aliases this area), filters, tables
            size_t off = 0;
            a.off_x = (int)off;
            off += (size_t)a.nct_in * 16 * a.xs + 64 * kMaxKse; // expand k padding may read past the last pixel
            a.off_e = (int)off;
            if (has_expand)
                off += (size_t)a.nct_in * 16 * kEs + 64;
            a.off_d = (int)off;
            off += (size_t)a.nct_out * 16 * kEs;
            a.off_out = 0;
            off = std::max(off, (size_t)a.nct_out * 16 * a.os);
            off = (off + 15) & ~(size_t)15;
            a.off_we = (int)off;
            off += (size_t)a.kse * 4 * 64 * 16;
            a.off_wp = (int)off;
            off += (size_t)a.nrt * 64 * 16;
            a.off_wd = (int)off;
            off += ((size_t)a.taps * p.exp_c + 15) & ~(size_t)15;
            a.off_ce = (int)off;
            if (has_expand)
                off += (size_t)3 * a.n_chunks * 64 * 4;
            a.off_cd = (int)off;
            off += (size_t)3 * a.n_chunks * 64 * 4;
            a.off_cp = (int)off;
            off += (size_t)3 * a.nrt * 16 * 4;
            a.off_pixtab = (int)off;
            off += (size_t)a.nct_out * 16 * 4;
            a.off_rctab = (int)off;
            off += (size_t)a.nct_in * 16 * 4;
            a.off_slottab = (int)off;
            off += (size_t)kMaxAcc * kWaves * 4;
            if (off > lds_limit())
                continue;
            const int per_cu = off <= 80 * 1024 ? 2 : 1;
            a.tiles_y = (p.out_h + a.th - 1) / a.th;
            a.tiles_x = (p.out_w + a.tw - 1) / a.tw;
            // cost per output pixel: expand work on the patch, depthwise and project on the padded
            // tile, per-chunk filter staging and barriers amortized over the tile, edge waste
            const double px = (double)a.p_out;
            double cost = (has_expand ? 1.0 * a.nct_in * 16 * a.kse : 0.0) + 3.0 * a.nct_out * 16 + 0.3 * a.nct_out * 16 * a.nrt;
            cost += 600.0; // barriers and filter staging per chunk, in the same unit
            cost /= px;
            cost *= per_cu == 2 ? 1.0 : 1.5;
            cost *= (double)(a.tiles_y * a.th) * (a.tiles_x * a.tw) / ((double)p.out_h * p.out_w);
            if (cost < best_cost) {
                best_cost = cost;
                best.ok = true;
                best.a = a;
                best.lds = off;
            }
        }
    }
    return best;
}

} // namespace

bool mbconv_s8_fused_supports(const MbconvParams &p)
{
    if ((long long)p.in_h * p.in_w * p.in_c >= (1ll << 30) || (long long)p.out_h * p.out_w * p.out_c >= (1ll << 30))
        return false;
    return mb_plan(p).ok;
}

hipError_t launch_mbconv_s8_fused(const MbconvParams &p, int cu_count, hipStream_t stream)
{
    if ((long long)p.batch * p.out_h * p.out_w == 0)
        return hipSuccess;
    MbPlan plan = mb_plan(p);
    if (!plan.ok)
        return hipErrorInvalidValue;
    MbArgs &a = plan.a;
    const long long units = (long long)p.batch * a.tiles_y * a.tiles_x;
    if (units > 0x7fffffff)
        return hipErrorInvalidValue;
    a.n_units = (int)units;
    a.fd_tiles_x = make_fastdiv((unsigned)a.tiles_x);
    a.fd_tiles_yx = make_fastdiv((unsigned)(a.tiles_y * a.tiles_x));
    a.fd_pw = make_fastdiv((unsigned)a.pw);
    a.fd_tw = make_fastdiv((unsigned)a.tw);
    a.fd_nct_out = make_fastdiv((unsigned)a.nct_out);
    a.fd_in_vecs = make_fastdiv((unsigned)a.in_vecs);
    a.fd_out_vecs = make_fastdiv((unsigned)a.out_vecs);
    static const bool trace = getenv("ESPDL_HIP_TRACE") != nullptr;
    const int cus = cu_count > 0 ? cu_count : 256;
    const int per_cu = resident_workgroups_per_cu(mbconv_s8_fused_kernel, kThreads, plan.lds);
    int gx = std::max(1, cus * per_cu);
    if (gx > a.n_units)
        gx = a.n_units;
    if (gx >= 8)
        gx &= ~7;
    if (trace)
        fprintf(stderr, "mbconv_s8_fused: lds limit %zu; %dx%d in %d exp %d out %d s%d tile %dx%d patch %dx%d chunks %d nrt %d n_acc %d lds %zu per_cu %d grid %d units %d\n",
                lds_limit(), p.in_h, p.in_w, p.in_c, p.exp_c, p.out_c, p.stride_h, a.th, a.tw, a.ph, a.pw, a.n_chunks, a.nrt, a.n_acc,
                plan.lds, per_cu, gx, a.n_units);
    hipLaunchKernelGGL(mbconv_s8_fused_kernel, dim3((unsigned)gx), dim3(kThreads), plan.lds, stream, a);
    return hipGetLastError();
}

} // namespace espdl
