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
// The kernel is built for blocks at small spatial sizes (14x14, 7x7 in MobileNetV2), where separate
// kernels are bound by launch and start-up latency, not by bandwidth.  A workgroup of 16 wavefronts
// owns a th x tw tile of the block's output in one image:
//   1. the input patch (tile + filter halo, all input channels) is copied to LDS;
//   2. the expanded channels are walked in chunks of 64:
//      expand    MFMA GEMM [64 filters] x [patch pixels] over the input channels -> E (LDS, int8, two
//                buffers); positions outside the image are forced to zero, because the depthwise zero
//                padding pads the *expanded* activation; operand A comes straight from the filter in
//                global memory (L2), requested one chunk ahead;
//      depthwise MFMA with a diagonal operand A, operand B straight from E -> D (LDS, int8, all chunks);
//      expand(c) and depthwise(c - 1) share one barrier;
//   3. project   MFMA GEMM [out_c filters] x [tile pixels] over all expanded channels from D, operand A
//                straight from the filter in global memory, one k step ahead;
//   4. epilogue -> LDS -> (+ residual read from global) -> contiguous global stores.
// Without an expand stage the depthwise stage reads the input patch.
#include <algorithm>
#include <cstdio>
#include <cstdlib>

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

constexpr int kThreads = 1024;
constexpr int kWaves = kThreads / 64;
constexpr int kParts = kWaves / 4; // wavefronts that share a row tile / channel group split the column tiles
constexpr int kKsDw = 3;           // depthwise k steps of 4 taps
constexpr int kMaxKse = 3;         // expand k steps of 64 input channels (in_c <= 192)
constexpr int kMaxAcc = 5;         // project accumulator tiles per wavefront
constexpr int kEs = 80;            // pixel stride of E in LDS: 64 channels + 16 (odd number of 16-byte units)

struct MbArgs {
    MbconvParams p;
    int has_expand;
    int taps;
    int th, tw, ph, pw;
    int p_in, p_out;     // pixels of the patch / of the tile
    int nct_in, nct_out; // column tiles of 16 pixels
    int xs;              // LDS pixel stride of the input patch, bytes
    int ds;              // LDS pixel stride of D, bytes
    int kse;             // expand k steps
    int ksp;             // project k steps (chunks of 64 expanded channels)
    int n_chunks;        // = ksp
    int nrt;             // project row tiles of 16 filters
    int n_acc;           // nrt * nct_out
    int os;              // LDS pixel stride of the output tile, bytes
    int out_vec;         // bytes per output store piece: 16 or 4
    int in_vec;          // bytes per input load piece: 16 or 4
    int in_vecs, out_vecs;
    int tiles_x, tiles_y, n_units;
    FastDiv fd_tiles_x, fd_tiles_yx, fd_pw, fd_tw, fd_nct_out, fd_in_vecs, fd_out_vecs;
    // LDS layout (byte offsets)
    int off_x, off_e, off_d, off_out, off_wd, off_ce, off_cd, off_cp, off_pixtab, off_rctab;
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

// Requantize four accumulators with the stage constants held in registers.
__device__ __forceinline__ int mb_pack_r(const v4i &acc, const v4i &ss, const v4i &ls, bool fast, bool relu,
                                         bool half_even, int floor_pk)
{
    if (fast)
        return half_even ? pack_fast4<5>(acc, ls, ss, floor_pk) : pack_fast4<1>(acc, ls, ss, floor_pk);
    int q[4];
#pragma unroll
    for (int r = 0; r < 4; r++)
        q[r] = requant_s8(acc[r], ss[r], relu, half_even);
    return pack4_s8(q[0], q[1], q[2], q[3]);
}

// Is the short epilogue valid for this channel?  (shift in 1..31, no overflow of the start value plus
// the largest possible sum of products, also after the left shift the short form may apply)
__device__ __forceinline__ bool mb_short_ok(int s, int bias, long long mac_bound)
{
    if (s < 1 || s > 31)
        return false;
    const long long start = (long long)bias + (1ll << (s - 1));
    return (start < 0 ? -start : start) + mac_bound < (1ll << (31 - max(0, 8 - s)));
}

// The half-even short form (pack_fast4<5>) starts one below the half-up rounding constant.
__device__ __forceinline__ void mb_put_consts(int *cst, int stride, int c, bool valid, bool fast, int s, int b, bool half_even)
{
    cst[c] = (fast && valid) ? b + (1 << (s - 1)) - (half_even ? 1 : 0) : b;
    cst[stride + c] = fast ? max(0, s - 8) : s;
    cst[2 * stride + c] = fast ? max(0, 8 - s) : 0;
}

// Operand A of the expand stage for one chunk, straight from the filter: row i of row tile `sub` is
// channel e0 + 4*ng*(i/4) + 4*sub + i%4 (so that a lane ends up with 4 consecutive channels per row
// tile and 4*ng consecutive channels over the row tiles); the lane's 16 k positions are input channels
// 64*ks + 16*gk ... (zeros past in_c).
__device__ __forceinline__ void mb_load_we(const MbArgs &a, int chunk, int sub, int lane, v4i (&aop)[kMaxKse])
{
    const MbconvParams &p = a.p;
    const int e0 = chunk * 64;
    const int ng = min(4, (p.exp_c - e0) >> 4);
    const int i = lane & 15, gk = lane >> 4;
#pragma unroll
    for (int ks = 0; ks < kMaxKse; ks++) {
        aop[ks] = v4i{0, 0, 0, 0};
        if (ks < a.kse && sub < ng) {
            const int ch = e0 + 4 * ng * (i >> 2) + 4 * sub + (i & 3);
            const int k0 = 64 * ks + 16 * gk;
            const int8_t *src = p.w_expand + (long long)ch * p.in_c + k0;
            if (k0 < p.in_c) // in_c % 16 == 0: the 16 positions are all inside or all outside
                aop[ks] = *reinterpret_cast<const v4i *>(src);
        }
    }
}

__global__ __launch_bounds__(kThreads) void mbconv_s8_fused_kernel(const MbArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const MbconvParams &p = a.p;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int quad = lane >> 4;
    const bool half_even = p.half_even != 0;
    const int ec_pad = a.n_chunks * 64;
    const int oc_pad = a.nrt * 16;

    int *cst_e = reinterpret_cast<int *>(smem + a.off_ce); // [3][ec_pad]
    int *cst_d = reinterpret_cast<int *>(smem + a.off_cd); // [3][ec_pad]
    int *cst_p = reinterpret_cast<int *>(smem + a.off_cp); // [3][oc_pad]
    int *pixtab = reinterpret_cast<int *>(smem + a.off_pixtab);
    int *rctab = reinterpret_cast<int *>(smem + a.off_rctab);
    unsigned char *x_l = smem + a.off_x;
    unsigned char *d_l = smem + a.off_d;
    unsigned char *out_l = smem + a.off_out;

    // ---- once per workgroup.  Every thread owns one expanded channel (exp_c <= 1024) and one output
    // channel: one round of global reads, then the three "short epilogue valid" votes.
    bool fast_e, fast_d, fast_p;
    {
        int s_e = 0, b_e = 0, s_d = 0, b_d = 0, s_p = 0, b_p = 0;
        int bad = 0;
        if (tid < p.exp_c) {
            if (a.has_expand) {
                s_e = p.s_expand[p.n_s_expand == 1 ? 0 : tid];
                b_e = p.b_expand != nullptr ? p.b_expand[tid] : 0;
            }
            s_d = p.s_dw[p.n_s_dw == 1 ? 0 : tid];
            b_d = p.b_dw != nullptr ? p.b_dw[tid] : 0;
        }
        if (tid < p.out_c) {
            s_p = p.s_project[p.n_s_project == 1 ? 0 : tid];
            b_p = p.b_project != nullptr ? p.b_project[tid] : 0;
        }
        for (int i = tid; i < a.taps * p.exp_c; i += kThreads)
            smem[a.off_wd + i] = (unsigned char)p.w_dw[i];
        if (tid < p.exp_c) {
            if (a.has_expand && !mb_short_ok(s_e, b_e, (long long)p.in_c * 16384))
                bad |= 1;
            if (!mb_short_ok(s_d, b_d, (long long)a.taps * 16384))
                bad |= 2;
        }
        if (tid < p.out_c && !mb_short_ok(s_p, b_p, (long long)p.exp_c * 16384))
            bad |= 4;
        // the vote is a logical OR of a predicate, so one vote per stage
        fast_e = __syncthreads_or(bad & 1) == 0;
        fast_d = __syncthreads_or(bad & 2) == 0;
        fast_p = __syncthreads_or(bad & 4) == 0;
        if (tid < ec_pad) {
            if (a.has_expand)
                mb_put_consts(cst_e, ec_pad, tid, tid < p.exp_c, fast_e, s_e, b_e, half_even);
            mb_put_consts(cst_d, ec_pad, tid, tid < p.exp_c, fast_d, s_d, b_d, half_even);
        }
        if (tid < oc_pad)
            mb_put_consts(cst_p, oc_pad, tid, tid < p.out_c, fast_p, s_p, b_p, half_even);
    }
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
    // (row | col << 16) of every patch pixel, -1 past the patch
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

    const TileSeq seq = xcd_tile_sequence(a.n_units);
    for (int unit = seq.first; unit < seq.end; unit += seq.step) {
        const TilePos u = mb_tile(a, unit);
        const int iy0 = u.y0 * p.stride_h - p.pad_top, ix0 = u.x0 * p.stride_w - p.pad_left;
        // Lane and wavefront ids pass through an opaque copy once per tile: everything derived from
        // them below (operand addresses, accumulator-tile assignment) is then formed where it is used
        // instead of being hoisted out of the tile loop and held in registers throughout.
        int lane_t = lane, wave_v = wave;
        asm volatile("" : "+v"(lane_t), "+v"(wave_v));
        const int wave = __builtin_amdgcn_readfirstlane(wave_v);
        const int lane = lane_t;
        const int col = lane & 15, quad = lane >> 4;
        const int sub = wave & 3, part = wave >> 2;

        // expand operands of chunk 0 are requested before the patch copy
        v4i we_cur[kMaxKse];
        if (a.has_expand)
            mb_load_we(a, 0, sub, lane, we_cur);

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
                *reinterpret_cast<v4i *>(dst) = ok ? *reinterpret_cast<const v4i *>(src) : v4i{0, 0, 0, 0};
            }
        }
        __syncthreads(); // patch (and, first tile, the tables) visible

        // ---- 2. chunks of 64 expanded channels.  Pipeline: iteration c runs expand(c) and
        // depthwise(c - 1), which touch different E buffers; one barrier per iteration.
        for (int chunk = 0; chunk <= a.n_chunks; chunk++) {
            if (a.has_expand && chunk < a.n_chunks) {
                const int e0 = chunk * 64;
                const int ng = min(4, (p.exp_c - e0) >> 4);
                v4i aop[kMaxKse];
#pragma unroll
                for (int ks = 0; ks < kMaxKse; ks++)
                    aop[ks] = we_cur[ks];
                if (chunk + 1 < a.n_chunks)
                    mb_load_we(a, chunk + 1, sub, lane, we_cur); // in flight during this chunk
                if (sub < ng) {
                    const int c = e0 + 4 * ng * quad + 4 * sub;
                    const v4i init = *reinterpret_cast<const v4i *>(cst_e + c);
                    const v4i ss = *reinterpret_cast<const v4i *>(cst_e + ec_pad + c);
                    const v4i ls = *reinterpret_cast<const v4i *>(cst_e + 2 * ec_pad + c);
                    const unsigned char *bsrc = x_l + col * a.xs + 16 * quad;
                    unsigned char *dst = smem + a.off_e + (chunk & 1) * (a.nct_in * 16 * kEs) + col * kEs + 4 * ng * quad + 4 * sub;
                    v4i b[kMaxKse];
                    int rc = -1;
                    if (part < a.nct_in) {
#pragma unroll
                        for (int ks = 0; ks < kMaxKse; ks++)
                            if (ks < a.kse)
                                b[ks] = *reinterpret_cast<const v4i *>(bsrc + part * 16 * a.xs + 64 * ks);
                        rc = rctab[part * 16 + col];
                    }
#pragma unroll 1
                    for (int ct = part; ct < a.nct_in; ct += kParts) {
                        v4i r = init;
#pragma unroll
                        for (int ks = 0; ks < kMaxKse; ks++)
                            if (ks < a.kse)
                                r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], b[ks], r, 0, 0, 0);
                        const int rc_cur = rc;
                        if (ct + kParts < a.nct_in) {
#pragma unroll
                            for (int ks = 0; ks < kMaxKse; ks++)
                                if (ks < a.kse)
                                    b[ks] = *reinterpret_cast<const v4i *>(bsrc + (ct + kParts) * 16 * a.xs + 64 * ks);
                            rc = rctab[(ct + kParts) * 16 + col];
                        }
                        const int word = mb_pack_r(r, ss, ls, fast_e, p.relu_expand != 0, half_even, floor_e);
                        // outside the image the expanded activation is the depthwise zero padding
                        const int iy = iy0 + (rc_cur & 0xffff), ix = ix0 + (rc_cur >> 16);
                        const bool inside = rc_cur >= 0 && (unsigned)iy < (unsigned)p.in_h && (unsigned)ix < (unsigned)p.in_w;
                        *reinterpret_cast<int *>(dst + ct * 16 * kEs) = inside ? word : 0;
                    }
                }
            }
            // depthwise of the previous chunk (with expand) / of this chunk (without)
            const int dchunk = a.has_expand ? chunk - 1 : chunk;
            if (dchunk >= 0 && dchunk < a.n_chunks) {
                const int e0 = dchunk * 64;
                const int ng = min(4, (p.exp_c - e0) >> 4);
                if (sub < ng && part < a.nct_out) {
                    const unsigned char *src_l = (a.has_expand ? smem + a.off_e + (dchunk & 1) * (a.nct_in * 16 * kEs)
                                                               : x_l + e0) + 16 * sub;
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
                    unsigned char *dst = d_l + col * a.ds + c;
                    v4i b[kKsDw];
                    {
                        const int po = pixtab[part * 16 + col];
#pragma unroll
                        for (int ks = 0; ks < kKsDw; ks++)
                            b[ks] = *reinterpret_cast<const v4i *>(src_l + po + tapoff[ks]);
                    }
                    int po_next = pixtab[min(part + kParts, a.nct_out - 1) * 16 + col];
#pragma unroll 1
                    for (int ct = part; ct < a.nct_out; ct += kParts) {
                        v4i r = init;
#pragma unroll
                        for (int ks = 0; ks < kKsDw; ks++)
                            if (4 * ks < a.taps)
                                r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], b[ks], r, 0, 0, 0);
                        if (ct + kParts < a.nct_out) {
#pragma unroll
                            for (int ks = 0; ks < kKsDw; ks++)
                                b[ks] = *reinterpret_cast<const v4i *>(src_l + po_next + tapoff[ks]);
                            po_next = pixtab[min(ct + 2 * kParts, a.nct_out - 1) * 16 + col];
                        }
                        const int word = mb_pack_r(r, ss, ls, fast_d, p.relu_dw != 0, half_even, floor_d);
                        *reinterpret_cast<int *>(dst + ct * 16 * a.ds) = word;
                    }
                }
            }
            __syncthreads();
        }

        // ---- 3. project: acc[rt][ct] = sum over all expanded channels, operand A from global memory,
        // one k step ahead
        {
            v4i acc[kMaxAcc];
            int arow[kMaxAcc], boff[kMaxAcc];
#pragma unroll
            for (int s = 0; s < kMaxAcc; s++) {
                const int t = min(wave + s * kWaves, a.n_acc - 1);
                const int rt = (int)fastdiv((unsigned)t, a.fd_nct_out);
                const int ct = t - rt * a.nct_out;
                arow[s] = 16 * rt + col; // filter of this lane's row
                boff[s] = (ct * 16 + col) * a.ds + 16 * quad;
                acc[s] = *reinterpret_cast<const v4i *>(cst_p + 16 * rt + 4 * quad);
            }
            auto load_wp = [&](int ks, v4i(&w)[kMaxAcc]) {
#pragma unroll
                for (int s = 0; s < kMaxAcc; s++) {
                    w[s] = v4i{0, 0, 0, 0};
                    const int e = 64 * ks + 16 * quad;
                    if (wave + s * kWaves < a.n_acc && arow[s] < p.out_c && e < p.exp_c)
                        w[s] = *reinterpret_cast<const v4i *>(p.w_project + (long long)arow[s] * p.exp_c + e);
                }
            };
            v4i wa[kMaxAcc], wb[kMaxAcc];
            load_wp(0, wa);
#pragma unroll 1
            for (int ks = 0; ks < a.ksp; ks += 2) {
                if (ks + 1 < a.ksp)
                    load_wp(ks + 1, wb);
#pragma unroll
                for (int s = 0; s < kMaxAcc; s++)
                    if (wave + s * kWaves < a.n_acc) {
                        const v4i b = *reinterpret_cast<const v4i *>(d_l + boff[s] + 64 * ks);
                        acc[s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[s], b, acc[s], 0, 0, 0);
                    }
                if (ks + 1 < a.ksp) {
                    if (ks + 2 < a.ksp)
                        load_wp(ks + 2, wa);
#pragma unroll
                    for (int s = 0; s < kMaxAcc; s++)
                        if (wave + s * kWaves < a.n_acc) {
                            const v4i b = *reinterpret_cast<const v4i *>(d_l + boff[s] + 64 * (ks + 1));
                            acc[s] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wb[s], b, acc[s], 0, 0, 0);
                        }
                }
            }
            // ---- 4. epilogue -> LDS tile.  It aliases the patch / E area, which nobody reads after the
            // last barrier of step 2.
#pragma unroll
            for (int s = 0; s < kMaxAcc; s++) {
                const int t = wave + s * kWaves;
                if (t < a.n_acc) {
                    const int rt = (int)fastdiv((unsigned)t, a.fd_nct_out);
                    const int ct = t - rt * a.nct_out;
                    const int c = 16 * rt + 4 * quad;
                    const v4i ss = *reinterpret_cast<const v4i *>(cst_p + oc_pad + c);
                    const v4i ls = *reinterpret_cast<const v4i *>(cst_p + 2 * oc_pad + c);
                    const int word = mb_pack_r(acc[s], ss, ls, fast_p, p.relu_project != 0, half_even, floor_p);
                    *reinterpret_cast<int *>(out_l + (ct * 16 + col) * a.os + c) = word;
                }
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
    if ((p.exp_c & 15) != 0 || (p.in_c & 15) != 0 || (p.out_c & 3) != 0 || p.k_h * p.k_w > 4 * kKsDw ||
        p.exp_c > kThreads || p.out_c > 384 || (reinterpret_cast<uintptr_t>(p.w_project) & 15) != 0)
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
            if ((reinterpret_cast<uintptr_t>(p.in) & 15) != 0 || (has_expand && (reinterpret_cast<uintptr_t>(p.w_expand) & 15) != 0))
                continue;
            a.in_vec = 16;
            a.out_vec = (p.out_c & 15) == 0 && (reinterpret_cast<uintptr_t>(p.out) & 15) == 0 &&
                    (p.residual == nullptr || (reinterpret_cast<uintptr_t>(p.residual) & 15) == 0) ? 16 : 4;
            a.in_vecs = p.in_c / a.in_vec;
            a.out_vecs = p.out_c / a.out_vec;
            a.xs = odd16(p.in_c);
            a.kse = has_expand ? (p.in_c + 63) / 64 : 0;
            a.n_chunks = (p.exp_c + 63) / 64;
            a.ksp = a.n_chunks;
            a.ds = odd16(a.n_chunks * 64);
            a.nrt = (p.out_c + 15) / 16;
            a.n_acc = a.nrt * a.nct_out;
            a.os = odd16(a.nrt * 16);
            if (a.n_acc > kMaxAcc * kWaves || a.ph > 0xffff || a.pw > 0x7fff)
                continue;
            // LDS: [patch | E (two buffers)] (the output tile aliases this area), D, tables
            size_t off = 0;
            a.off_x = (int)off;
            off += (size_t)a.nct_in * 16 * a.xs + 64 * kMaxKse; // expand k padding may read past the last pixel
            a.off_e = (int)off;
            if (has_expand)
                off += (size_t)2 * a.nct_in * 16 * kEs + 64;
            a.off_out = 0;
            off = std::max(off, (size_t)a.nct_out * 16 * a.os);
            off = (off + 15) & ~(size_t)15;
            a.off_d = (int)off;
            off += (size_t)a.nct_out * 16 * a.ds + 64;
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
            if (off > lds_limit())
                continue;
            a.tiles_y = (p.out_h + a.th - 1) / a.th;
            a.tiles_x = (p.out_w + a.tw - 1) / a.tw;
            // work per output pixel: expand on the patch, depthwise and project on the padded tile, a
            // fixed cost per chunk (barrier) and per tile, edge waste
            const double px = (double)a.p_out;
            double cost = (has_expand ? 1.0 * a.nct_in * 16 * a.kse : 0.0) + 3.0 * a.nct_out * 16 +
                0.3 * a.nct_out * 16 * a.nrt;
            cost = cost * a.n_chunks + 300.0 * a.n_chunks + 1500.0;
            cost /= px;
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
