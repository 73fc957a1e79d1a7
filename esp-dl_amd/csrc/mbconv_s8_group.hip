// Inverted-residual block (1x1 expand conv -> 3x3 depthwise conv -> 1x1 project conv [-> Add]) for int8
// on gfx950 at SMALL spatial sizes (14 x 14, 7 x 7 images with hundreds of expanded channels), where a
// batch has too few output tiles to give every SIMD a tile of its own: a workgroup of eight wavefronts
// shares one tile and splits the EXPANDED CHANNELS instead.
//
// The stages compute exactly what the separate operators compute (see mbconv_s8_stages.h for the reference
// functions), with the int8 result of every stage materialized before the next one reads it, so the block
// is bit-identical to running Conv, Conv, Conv, Add modules one after the other.
//
// Per tile (th x tw output pixels of one image, tw = whole image width):
//   phase 0  all lanes build the per-channel requantization tables of the expand and depthwise stages in
//            LDS; every wavefront loads the block-input patch of the tile into the registers that are
//            operand B of its expand products (lane = patch pixel x 16 input channels per k step);
//   phase 1  wavefront w takes the chunks of 16 expanded channels w, w + 8, ... and, on its own (no barrier,
//            private LDS area), runs expand -> depthwise for them as the one-wavefront-per-tile kernel does;
//            the depthwise result goes to an LDS tile [pixel][all expanded channels] shared by the group;
//   barrier
//   phase 2  the project product: (16 filters x 16 pixels) accumulator tiles are dealt to the wavefronts,
//            operand B straight from the shared depthwise tile, operand A straight from the filter in
//            global memory (L2); epilogue, residual add, stores.
// Two barriers per tile in all; between them eight independent instruction streams per workgroup keep the
// matrix pipe, the vector ALU and LDS busy.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "mbconv_s8_stages.h"

namespace espdl {

namespace {

using namespace mbstage;

constexpr int kGroupWaves = 8;
constexpr int kGroupThreads = 64 * kGroupWaves;
constexpr int kMaxT = 7; // project pixel tiles per wavefront and row tile

struct GroupArgs {
    MbconvParams p;
    int th, tw, ph, pw;
    int twp;   // pixel slots per output row in the shared depthwise tile: 8 or 16
    int n_xpt; // pixel tiles of 16 in the patch
    int kse;   // expand k steps of 64 block-input channels
    int tiles_y, n_tiles;
    int n_sub; // chunks of 16 expanded channels
    int rt;    // project row tiles of 16 filters
    int npt;   // project pixel tiles of 16 slots
    int wr, wp, nt; // phase 2: wavefront grid (row groups x pixel groups, wr * wp <= 8), pixel tiles per wavefront
    int ds;    // LDS pixel stride of the shared depthwise tile, bytes
    int exp_bytes; // private expand area per wavefront
    int off_tab, off_exp, off_dw;
    FastDiv fd_pw, fd_tiles_y;
};

// EXACT: the plan is exactly (NXPT patch pixel tiles, KSE k steps, PT rows): no guards in the stage loops.
// KSP > 0: the project stage has exactly KSP k steps of 64 expanded channels and a wavefront holds operand A of
// a whole row tile of filters in registers (KSP = 0: any count, operand A in blocks of eight k steps).
// NTX > 0: a wavefront holds exactly NTX project pixel tiles at a time (no code for other counts: fewer registers).
template <int NXPT, int KSE, int PT, int S, bool HE, bool EXACT, int KSP = 0, int NTX = 0>
__global__ __launch_bounds__(kGroupThreads, (KSE == 1 && EXACT) ? 4 : 2) void mbconv_s8_group_kernel(const GroupArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const MbconvParams &p = a.p;
    const int tid = threadIdx.x, lane = tid & 63, col = lane & 15, quad = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int *tab_e = reinterpret_cast<int *>(smem + a.off_tab);
    int *tab_d = tab_e + 3 * p.exp_c;
    unsigned char *exp_l = smem + a.off_exp + wave * a.exp_bytes;
    unsigned char *dw_l = smem + a.off_dw;

    int tile = blockIdx.x;
    if ((gridDim.x & 7u) == 0) {
        const int per = gridDim.x >> 3;
        tile = (int)(blockIdx.x & 7u) * per + (int)(blockIdx.x >> 3);
    }
    const unsigned n = fastdiv((unsigned)tile, a.fd_tiles_y);
    const int oy0 = (int)((unsigned)tile - n * a.fd_tiles_y.d) * a.th;
    const int iy0 = oy0 * S - p.pad_top, ix0 = -p.pad_left;
    const int th_real = min(a.th, p.out_h - oy0);
    const int th = EXACT ? PT : th_real;
    const int n_xpt = EXACT ? NXPT : a.n_xpt;
    const int kse = EXACT ? KSE : a.kse;
    const int c0 = p.in_c;

    // ---- phase 0: tables (all lanes of the group), block-input patch -> operand B registers (per wavefront)
    const unsigned bound_e = (unsigned)c0 * 16384u, bound_d = 9u * 16384u;

    v4i xb[NXPT * KSE];
    unsigned xmask = 0;
    {
        const int8_t *img = p.in + (long long)n * p.in_h * p.in_w * c0;
#pragma unroll
        for (int pt = 0; pt < NXPT; pt++) {
            const unsigned pp = (unsigned)(pt * 16 + col);
            const unsigned prow = fastdiv(pp, a.fd_pw);
            const int iy = iy0 + (int)prow, ix = ix0 + (int)(pp - prow * a.fd_pw.d);
            const bool valid = pt < n_xpt && (int)prow < a.ph && (unsigned)iy < (unsigned)p.in_h &&
                (unsigned)ix < (unsigned)p.in_w;
            xmask |= valid ? 1u << pt : 0u;
#pragma unroll
            for (int ks = 0; ks < KSE; ks++) {
                xb[pt * KSE + ks] = v4i{0, 0, 0, 0};
                if (EXACT || (pt < n_xpt && ks < kse)) { // uniform
                    // nothing is zeroed here: a pixel outside the image gets its expand OUTPUT zeroed through
                    // xmask, reduction positions past in_c (a multiple of 16) meet zeros in operand A; such
                    // lanes read the image's first bytes
                    const bool ok = valid && c0 - 64 * ks - 16 * quad >= 16;
                    xb[pt * KSE + ks] = *reinterpret_cast<const v4i *>(
                        img + (size_t)(ok ? (unsigned)((iy * p.in_w + ix) * c0 + 64 * ks + 16 * quad) : 0u));
                }
            }
        }
    }
    // filters of a chunk of 16 expanded channels, requested one chunk ahead
    struct ChunkW {
        v4i aop[KSE];
        int wd0[3], wd1[3];
    };
    auto load_chunk = [&](int sub) {
        ChunkW w;
        const int ch0 = 16 * sub;
#pragma unroll
        for (int ks = 0; ks < KSE; ks++) {
            w.aop[ks] = v4i{0, 0, 0, 0};
            if (EXACT || ks < kse) // uniform
                w.aop[ks] = load16_partial<true>(p.w_expand, (unsigned)((ch0 + col) * c0 + 64 * ks + 16 * quad),
                                                 c0 - 64 * ks - 16 * quad);
        }
        const unsigned wd = (unsigned)(ch0 + col);
#pragma unroll
        for (int kx = 0; kx < 3; kx++) {
            const int v0 = (int)p.w_dw[(size_t)(wd + (unsigned)((min(quad, 2) * 3 + kx) * p.exp_c))];
            w.wd0[kx] = quad < 3 ? v0 : 0;
            w.wd1[kx] = 0;
            if constexpr (S == 1) {
                const int v1 = (int)p.w_dw[(size_t)(wd + (unsigned)((max(quad - 1, 0) * 3 + kx) * p.exp_c))];
                w.wd1[kx] = quad >= 1 ? v1 : 0;
            }
        }
        return w;
    };

    int mode_e, mode_d, mode_p;
    int *tab_p = tab_d + 3 * p.exp_c; // 3 x 16 rt entries
    {
        StageTablesArgs t;
        t.tab_e = tab_e;
        t.tab_d = tab_d;
        t.tab_p = tab_p;
        t.votes = tab_p + 3 * 16 * a.rt;
        t.b_e = p.b_expand;
        t.s_e = p.s_expand;
        t.b_d = p.b_dw;
        t.s_d = p.s_dw;
        t.b_p = p.b_project;
        t.s_p = p.s_project;
        t.n_s_e = p.n_s_expand;
        t.n_s_d = p.n_s_dw;
        t.n_s_p = p.n_s_project;
        t.n_ch = p.exp_c;
        t.n_ch_p = p.out_c;
        t.n_pad_p = 16 * a.rt;
        t.bound_e = bound_e;
        t.bound_d = bound_d;
        t.bound_p = (unsigned)p.exp_c * 16384u;
        build_stage_tables(t, HE, tid, kGroupThreads, mode_e, mode_d, mode_p); // tables complete
    }

    // ---- phase 1: this wavefront's chunks of 16 expanded channels, expand -> depthwise, no barriers
    const int floor_e = p.relu_expand ? 0 : (int)0x80008000u;
    const int floor_d = p.relu_dw ? 0 : (int)0x80008000u;
    unsigned char *exp_dst = exp_l + col * 16 + 4 * quad;
    const unsigned char *exp_src = exp_l + (quad * a.pw + S * col) * 16;
    const int row_bytes = a.twp * a.ds;
    const bool write_ok = col < a.twp;

    if (wave < a.n_sub) {
        ChunkW cur = load_chunk(wave);
        for (int sub = wave; sub < a.n_sub; sub += kGroupWaves) {
            const ChunkW nxt = load_chunk(min(sub + kGroupWaves, a.n_sub - 1));
            {
                const StageConsts ce = read_stage_table(tab_e, p.exp_c, 16 * sub + 4 * quad, mode_e);
                if (!HE && ce.mode == 0) // a build meets the forms of its rounding mode only
                    expand_chunk<0, NXPT, EXACT, KSE>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst);
                else if (!HE && ce.mode == 1)
                    expand_chunk<1, NXPT, EXACT, KSE>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst);
                else if (HE && ce.mode == 6)
                    expand_chunk<6, NXPT, EXACT, KSE>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst);
                else if (HE && ce.mode == 5)
                    expand_chunk<5, NXPT, EXACT, KSE>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst);
                else
                    expand_chunk<-1, NXPT, EXACT, KSE>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst);
            }
            wave_lds_sync();
            {
                v4i a0[3], a1[3];
#pragma unroll
                for (int kx = 0; kx < 3; kx++) {
                    a0[kx] = diag_operand(cur.wd0[kx], col);
                    a1[kx] = diag_operand(cur.wd1[kx], col);
                }
                const StageConsts cd = read_stage_table(tab_d, p.exp_c, 16 * sub + 4 * quad, mode_d);
                unsigned char *dst = dw_l + col * a.ds + 16 * sub + 4 * quad;
                if (!HE && cd.mode == 0) // a build meets the forms of its rounding mode only
                    depthwise_chunk<0, PT, S, EXACT>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, row_bytes, write_ok);
                else if (!HE && cd.mode == 1)
                    depthwise_chunk<1, PT, S, EXACT>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, row_bytes, write_ok);
                else if (HE && cd.mode == 6)
                    depthwise_chunk<6, PT, S, EXACT>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, row_bytes, write_ok);
                else if (HE && cd.mode == 5)
                    depthwise_chunk<5, PT, S, EXACT>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, row_bytes, write_ok);
                else
                    depthwise_chunk<-1, PT, S, EXACT>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, row_bytes, write_ok);
            }
            wave_lds_sync();
            cur = nxt;
        }
    }
    // operand A of the first project step does not depend on this tile's data: requested before the barrier
    const int ksp = (p.exp_c + 63) / 64;
    const int wrow = wave / a.wp, wpix = wave - wrow * a.wp;
    auto load_a = [&](int rt, int k0, v4i(&ap)[8]) {
        const bool row_ok = rt < a.rt && 16 * rt + col < p.out_c;
        const unsigned a_off = (unsigned)((16 * rt + col) * p.exp_c + 16 * quad);
#pragma unroll
        for (int kk = 0; kk < 8; kk++) // lanes past the last channel read offset 0 and get zeros
            ap[kk] = load16_partial<true>(p.w_project, a_off + 64u * (unsigned)(k0 + kk),
                                          row_ok ? p.exp_c - 64 * (k0 + kk) - 16 * quad : 0);
    };
    // KSP builds take whole row tiles and whole k steps only (out_c a multiple of 16, exp_c of 64), so this load
    // needs no mask: nothing touches the value between the load and its product, and a request for a row tile
    // past the last one reads the last one again
    auto load_a_step = [&](int rt, int k) {
        return *reinterpret_cast<const v4i *>(
            p.w_project + (size_t)((unsigned)((16 * min(rt, a.rt - 1) + col) * p.exp_c + 16 * quad) + 64u * (unsigned)k));
    };
    // (the blocked form does not prefetch in the build that is held to 128 registers so that two workgroups
    // share a compute unit)
    constexpr bool kPrefetchA = !(KSE == 1 && EXACT);
    v4i ap_first[KSP > 0 ? KSP : 8];
    if constexpr (KSP > 0) {
        if (wrow < a.wr) { // uniform
#pragma unroll
            for (int kk = 0; kk < KSP; kk++)
                ap_first[kk] = load_a_step(wrow, kk);
        }
    } else if constexpr (kPrefetchA) {
        load_a(wrow, 0, ap_first);
    }
    __syncthreads(); // the shared depthwise tile is complete

    // ---- phase 2: project.  The (row tile of 16 filters) x (pixel tile of 16 slots) accumulator tiles are dealt
    // to the wavefronts as a grid of a.wr row groups x a.wp pixel groups (chosen on the host): a wavefront
    // walks the row tiles of its row group and holds nt = ceil(npt / wp) pixel tiles at a time.  nt is a compile-time count here, so the operand-B reads of a k step are issued together and the
    // products follow back to back; a pixel tile past the last one reads the last tile again and stores
    // nothing.  Eight k steps of operand A are requested together, which hides the latency of those loads.
    // Reduction positions past exp_c meet zeros in operand A, whatever operand B holds there.
    const int t0 = wpix * a.nt;
    const int floor_p = p.relu_project ? 0 : (int)0x80008000u;
    const Requant4 res_q = make_requant4(p.residual_shift);
    const long long img_off = (long long)n * p.out_h * p.out_w * p.out_c;
    const int8_t *res_img = p.residual != nullptr ? p.residual + img_off : nullptr;
    int8_t *out_img = p.out + img_off;
    auto project = [&](auto nt_tag) {
        constexpr int NT = decltype(nt_tag)::value;
        const unsigned char *bsrc[NT];
#pragma unroll
        for (int i = 0; i < NT; i++)
            bsrc[i] = dw_l + (min(t0 + i, a.npt - 1) * 16 + col) * a.ds + 16 * quad;
        v4i ap[KSP > 0 ? KSP : 8];
        if constexpr (KSP > 0 || kPrefetchA) {
#pragma unroll
            for (int kk = 0; kk < (KSP > 0 ? KSP : 8); kk++)
                ap[kk] = ap_first[kk];
        }
        for (int rt = wrow; rt < a.rt; rt += a.wr) {
            v4i accp[NT];
#pragma unroll
            for (int i = 0; i < NT; i++)
                accp[i] = v4i{0, 0, 0, 0};
            // the residual words of this row tile are requested now and used after the products
            const int c = 16 * rt + 4 * quad;
            bool live[NT];
            unsigned off[NT];
            int rv[NT];
#pragma unroll
            for (int i = 0; i < NT; i++) {
                // pixel slot -> (row, column) of the tile: twp slots per output row
                const int slot = (t0 + i) * 16 + col;
                const int oy = a.twp == 16 ? t0 + i : (slot >> 3), ox = a.twp == 16 ? col : (slot & 7);
                live[i] = t0 + i < a.npt && oy < th_real && ox < p.out_w && c < p.out_c;
                off[i] = (unsigned)(((oy0 + oy) * p.out_w + ox) * p.out_c + c);
                rv[i] = res_img != nullptr ? *reinterpret_cast<const int *>(res_img + (size_t)(live[i] ? off[i] : 0u)) : 0;
            }
            if constexpr (KSP > 0) {
                // operand A of the whole row tile is in registers; each register is requested again, for the
                // wavefront's next row tile, as soon as its products are issued (the compiler gives the new
                // values registers of their own, so this form is for short reductions)
                auto steps = [&](auto more_tag) {
#pragma unroll
                    for (int kk = 0; kk < KSP; kk++) {
                        v4i bv[NT];
#pragma unroll
                        for (int i = 0; i < NT; i++)
                            bv[i] = *reinterpret_cast<const v4i *>(bsrc[i] + 64 * kk);
#pragma unroll
                        for (int i = 0; i < NT; i++)
                            accp[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ap[kk], bv[i], accp[i], 0, 0, 0);
                        if constexpr (decltype(more_tag)::value)
                            ap[kk] = load_a_step(rt + a.wr, kk);
                    }
                };
                if (rt + a.wr < a.rt) // uniform
                    steps(std::true_type{});
                else
                    steps(std::false_type{});
            } else {
                for (int k0 = 0; k0 < ksp; k0 += 8) {
                    // the next block of operand A (the next k steps, or the first ones of the next row tile) is
                    // requested before this block's products
                    v4i an[8];
                    const bool more_k = k0 + 8 < ksp;
                    if constexpr (kPrefetchA)
                        load_a(more_k ? rt : rt + a.wr, more_k ? k0 + 8 : 0, an);
                    else
                        load_a(rt, k0, ap);
#pragma unroll
                    for (int kk = 0; kk < 8; kk++) {
                        if (k0 + kk < ksp) { // uniform
                            v4i bv[NT];
#pragma unroll
                            for (int i = 0; i < NT; i++)
                                bv[i] = *reinterpret_cast<const v4i *>(bsrc[i] + 64 * (k0 + kk));
#pragma unroll
                            for (int i = 0; i < NT; i++)
                                accp[i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ap[kk], bv[i], accp[i], 0, 0, 0);
                        }
                    }
                    if constexpr (kPrefetchA) {
#pragma unroll
                        for (int kk = 0; kk < 8; kk++)
                            ap[kk] = an[kk];
                    }
                }
            }
            const StageConsts cp = read_stage_table<false>(tab_p, 16 * a.rt, c, mode_p);
            // the uniform choices (epilogue form, residual or not) are made once per row tile, outside the loop
            // over the words
            auto words = [&](auto mode_tag, auto res_tag) {
                constexpr int MODE = decltype(mode_tag)::value;
                constexpr bool RES = decltype(res_tag)::value;
#pragma unroll
                for (int i = 0; i < NT; i++) {
                    v4i acc = accp[i];
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        acc[k] += cp.init[k];
                    int word;
                    if constexpr (RES) {
                        int res = rv[i];
                        if (p.residual_shift != 0) // uniform
                            res = requant4_s8(res, res_q);
                        if constexpr (MODE >= 0)
                            word = pack_fast4_add<MODE>(acc, cp.lsh, cp.rsh, floor_p, res);
                        else
                            word = sat_add4_s8(wave_pack<MODE>(acc, cp, floor_p, p.relu_project != 0, HE), res);
                    } else {
                        word = wave_pack<MODE>(acc, cp, floor_p, p.relu_project != 0, HE);
                    }
                    if (live[i])
                        *reinterpret_cast<int *>(out_img + (size_t)off[i]) = word;
                }
            };
            auto with_mode = [&](auto mode_tag) {
                if (res_img != nullptr)
                    words(mode_tag, std::true_type{});
                else
                    words(mode_tag, std::false_type{});
            };
            if (cp.mode == -1)
                with_mode(std::integral_constant<int, -1>{});
            else if (HE && cp.mode == 6)
                with_mode(std::integral_constant<int, 6>{});
            else if constexpr (HE)
                with_mode(std::integral_constant<int, 5>{});
            else if (cp.mode == 0)
                with_mode(std::integral_constant<int, 0>{});
            else
                with_mode(std::integral_constant<int, 1>{});
        }
    };
    if (wrow < a.wr) { // uniform: wavefronts beyond the grid have no share
        const auto run = [&](auto nt_tag) {
            if constexpr (NTX == 0 || decltype(nt_tag)::value == NTX)
                project(nt_tag);
        };
        switch (a.nt) {
        case 1: run(std::integral_constant<int, 1>{}); break;
        case 2: run(std::integral_constant<int, 2>{}); break;
        case 3: run(std::integral_constant<int, 3>{}); break;
        case 4: run(std::integral_constant<int, 4>{}); break;
        case 5: run(std::integral_constant<int, 5>{}); break;
        case 6: run(std::integral_constant<int, 6>{}); break;
        default: run(std::integral_constant<int, kMaxT>{}); break;
        }
    }
}

struct GroupPlan {
    bool ok;
    GroupArgs a;
    size_t lds;
};

constexpr int kGroupPtMax = 8;
constexpr size_t kGroupLdsMax = 156 * 1024;

// Whether a guard-free build exists for a plan (defined behind the builds).
bool group_plan_has_exact_build(const GroupPlan &plan);

GroupPlan group_plan(const MbconvParams &p)
{
    GroupPlan plan;
    plan.ok = false;
    if (p.w_expand == nullptr || p.k_h != 3 || p.k_w != 3 || p.dil_h != 1 || p.dil_w != 1 || p.stride_h != p.stride_w ||
        (p.stride_h != 1 && p.stride_h != 2))
        return plan;
    if (p.in_c % 16 != 0 || p.in_c > 192 || p.exp_c % 16 != 0 || p.exp_c >= 65536 || p.out_c % 4 != 0 || p.out_w > 16 ||
        (reinterpret_cast<uintptr_t>(p.in) & 15) != 0 || (reinterpret_cast<uintptr_t>(p.w_expand) & 15) != 0)
        return plan;
    if ((long long)p.in_h * p.in_w * p.in_c >= (1ll << 30) || (long long)p.out_h * p.out_w * p.out_c >= (1ll << 30) ||
        (long long)p.out_c * p.exp_c >= (1ll << 31))
        return plan;
    const int s = p.stride_h;
    // The tile a workgroup takes is the whole width and as many rows as fit.  The guard-free builds are made for
    // widths of 14 (7 at depthwise stride 2 and for images up to 7 wide) and 7 rows (4 at stride 2): a narrower
    // or lower image is first tried rounded up to that tile - the columns and rows that do not exist load as
    // padding and their stores are dropped - and keeps the rounded plan when a guard-free build takes it (a third
    // of the time of a guarded build, which more than pays for the idle part of the tile).
    const int tw_class = (p.out_w <= 7) ? 7 : (p.out_w <= 14 ? 14 : p.out_w);
    const int th_class = s == 1 ? 7 : 4;
    for (int attempt = 0; attempt < 2; attempt++) {
        const bool rounded = attempt == 0;
        if (rounded && tw_class == p.out_w && th_class <= p.out_h)
            continue; // nothing to round: the natural plan below is the same or better
        GroupArgs a = {};
        a.p = p;
        a.tw = rounded ? tw_class : p.out_w;
        a.pw = (a.tw - 1) * s + 3;
        a.twp = a.tw <= 8 ? 8 : 16;
        a.kse = (p.in_c + 63) / 64;
        a.n_sub = p.exp_c / 16;
        a.rt = (p.out_c + 15) / 16;
        // Pixel pitch of the depthwise result: twice an odd number of 16-byte units.  A 16-byte-per-lane LDS read is
        // served in groups of 8 consecutive pixels x 2 neighbouring 16-byte quarters; with such a pitch the 16 pieces
        // of a group fall into 16 different bank sets (an odd number of units, the earlier choice, leaves half of the
        // project stage's operand-B reads in two passes).  The 4-byte stores of the depthwise stage then take two
        // passes, but the project stage reads every piece once per wavefront: eight times as many LDS cycles.
        a.ds = p.exp_c + 16;
        while ((a.ds / 16) % 4 != 2)
            a.ds += 16;
        // rows per tile: as many as fit the register and LDS budgets (fewer tiles, less halo to expand)
        a.th = 0;
        const int th_max = rounded ? th_class : std::min(kGroupPtMax - 1, p.out_h);
        for (int th = rounded ? th_class : 1; th <= th_max; th++) {
            const int ph = (th - 1) * s + 3;
            const int n_xpt = (ph * a.pw + 15) / 16;
            if (n_xpt > 9)
                break;
            const int npt = (th * a.twp + 15) / 16;
            if (npt > kMaxT)
                break;
            const size_t exp_bytes = (size_t)((ph * a.pw + 48 + 15) & ~15) * 16;
            const size_t lds = (size_t)p.exp_c * 24 + (size_t)a.rt * 16 * 12 + kStageVoteBytes + kGroupWaves * std::max(exp_bytes, (size_t)((n_xpt + 3) & ~3) * 256) +
                (size_t)npt * 16 * a.ds + 64;
            if (lds > kGroupLdsMax)
                break;
            a.th = th;
        }
        if (a.th == 0)
            continue;
        a.ph = (a.th - 1) * s + 3;
        a.n_xpt = (a.ph * a.pw + 15) / 16;
        a.npt = (a.th * a.twp + 15) / 16;
        a.tiles_y = (p.out_h + a.th - 1) / a.th;
        a.exp_bytes = (int)std::max((size_t)((a.ph * a.pw + 48 + 15) & ~15) * 16, (size_t)((a.n_xpt + 3) & ~3) * 256);
        a.off_tab = 0;
        a.off_exp = p.exp_c * 24 + a.rt * 16 * 12 + kStageVoteBytes; // expand, depthwise and project tables, vote words
        a.off_dw = a.off_exp + kGroupWaves * a.exp_bytes;
        plan.lds = (size_t)a.off_dw + (size_t)a.npt * 16 * a.ds + 64; // k steps read whole 64-byte pieces
        // phase-2 grid: a row tile of filters belongs to one wavefront where there are at least eight of them
        // (operand A comes from global memory: loading it once per workgroup matters more than an even share);
        // with fewer row tiles 8 / rt wavefronts share one and split the pixel tiles
        if (a.rt >= kGroupWaves) {
            a.wr = kGroupWaves;
            a.wp = 1;
        } else {
            a.wr = a.rt;
            a.wp = kGroupWaves / a.rt;
        }
        a.nt = (a.npt + a.wp - 1) / a.wp;
        a.fd_pw = make_fastdiv((unsigned)a.pw);
        a.fd_tiles_y = make_fastdiv((unsigned)a.tiles_y);
        plan.a = a;
        plan.ok = true;
        if (!rounded || group_plan_has_exact_build(plan))
            return plan;
        plan.ok = false; // the rounded tile has no guard-free build: take the natural one
    }
    return plan;
}

template <int NXPT, int KSE, int PT, int S, bool HE, bool EXACT, int KSP = 0, int NTX = 0>
hipError_t launch_group_one(const GroupPlan &plan, hipStream_t stream)
{
    auto kernel = mbconv_s8_group_kernel<NXPT, KSE, PT, S, HE, EXACT, KSP, NTX>;
    static bool raised = false; // the dynamic LDS limit of a kernel is raised once per process
    if (!raised) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, (int)kGroupLdsMax);
        if (e != hipSuccess)
            return e;
        raised = true;
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)plan.a.n_tiles), dim3(kGroupThreads), plan.lds, stream, plan.a);
    return hipGetLastError();
}

// The guard-free builds: the tile plans of MobileNetV2's 14 x 14 and 7 x 7 blocks, in both rounding modes.
// Returns false when the plan has none; with `dry` nothing is launched.
template <bool HE>
bool launch_group_exact(const GroupPlan &plan, hipStream_t stream, bool dry, hipError_t *err)
{
    const GroupArgs &a = plan.a;
    const int s = a.p.stride_h;
    const int ksp = (a.p.exp_c + 63) / 64;
    // k_project / nt: the project stage's k steps and pixel tiles per wavefront the build is made for (0: any)
    const auto is = [&](int nxpt, int kse, int th, int stride, int k_project, int nt) {
        return a.n_xpt == nxpt && a.kse == kse && a.th == th && s == stride &&
            (k_project == 0 || (ksp == k_project && a.p.exp_c % 64 == 0 && a.p.out_c % 16 == 0)) && (nt == 0 || a.nt == nt);
    };
#define ESPDL_GROUP_EXACT(NXPT, KSE, PT, S, KSP, NTX)                                    \
    do {                                                                                 \
        if (is(NXPT, KSE, PT, S, KSP, NTX)) {                                            \
            if (!dry)                                                                    \
                *err = launch_group_one<NXPT, KSE, PT, S, HE, true, KSP, NTX>(plan, stream); \
            return true;                                                                 \
        }                                                                                \
    } while (0)
    // MobileNetV2-1.0's blocks, each with the one pixel-tile count and reduction length it has there ...
    ESPDL_GROUP_EXACT(9, 1, 7, 1, 0, 4); // 14 x 14, 64 -> 384 -> 64 (held to 128 registers: operand A in blocks)
    ESPDL_GROUP_EXACT(9, 1, 7, 1, 0, 7); // 14 x 14, 64 -> 384 -> 96
    ESPDL_GROUP_EXACT(9, 2, 7, 1, 9, 7); // 14 x 14, 96 -> 576 -> 96
    ESPDL_GROUP_EXACT(9, 2, 4, 2, 9, 2); // 14 x 14, 96 -> 576 -> 160, stride 2
    ESPDL_GROUP_EXACT(6, 3, 7, 1, 0, 4); // 7 x 7, 160 -> 960 -> 160 / 320 (several row tiles per wavefront:
                                         // operand A in blocks hides their loads better)
    // ... and the same tile plans with any output channel count
    ESPDL_GROUP_EXACT(9, 1, 7, 1, 0, 0);
    ESPDL_GROUP_EXACT(9, 2, 7, 1, 0, 0);
    ESPDL_GROUP_EXACT(6, 3, 7, 1, 0, 0);
    ESPDL_GROUP_EXACT(9, 2, 4, 2, 0, 0);
#undef ESPDL_GROUP_EXACT
    return false;
}

bool group_plan_has_exact_build(const GroupPlan &plan)
{
    hipError_t err = hipSuccess;
    return plan.a.p.half_even ? launch_group_exact<true>(plan, nullptr, true, &err)
                              : launch_group_exact<false>(plan, nullptr, true, &err);
}

} // namespace

bool mbconv_s8_group_supports(const MbconvParams &p)
{
    return group_plan(p).ok;
}

hipError_t launch_mbconv_s8_group(const MbconvParams &p, int cu_count, hipStream_t stream)
{
    (void)cu_count;
    if ((long long)p.batch * p.out_h * p.out_w == 0)
        return hipSuccess;
    GroupPlan plan = group_plan(p);
    if (!plan.ok)
        return hipErrorInvalidValue;
    const long long tiles = (long long)p.batch * plan.a.tiles_y;
    if (tiles > 0x7fffffff)
        return hipErrorInvalidValue;
    plan.a.n_tiles = (int)tiles;
    const GroupArgs &a = plan.a;
    static const bool trace = getenv("ESPDL_HIP_TRACE") != nullptr;
    if (trace)
        fprintf(stderr, "mbconv_s8_group: %dx%d in %d exp %d out %d s%d tile %dx%d patch %dx%d n_xpt %d kse %d rt %d npt %d lds %zu tiles %lld\n",
                p.in_h, p.in_w, p.in_c, p.exp_c, p.out_c, p.stride_h, a.th, a.tw, a.ph, a.pw, a.n_xpt, a.kse, a.rt, a.npt,
                plan.lds, tiles);
    const int s = p.stride_h;
    hipError_t err = hipSuccess;
    if (p.half_even ? launch_group_exact<true>(plan, stream, false, &err) : launch_group_exact<false>(plan, stream, false, &err))
        return err;
    if (!p.half_even)
        return s == 1 ? launch_group_one<9, 3, kGroupPtMax, 1, false, false>(plan, stream)
                      : launch_group_one<9, 3, kGroupPtMax, 2, false, false>(plan, stream);
    return s == 1 ? launch_group_one<9, 3, kGroupPtMax, 1, true, false>(plan, stream)
                  : launch_group_one<9, 3, kGroupPtMax, 2, true, false>(plan, stream);
}

bool mbconv_s8_group_has_fast_build(const MbconvParams &p)
{
    const GroupPlan plan = group_plan(p);
    hipError_t err = hipSuccess;
    return plan.ok &&
        (p.half_even ? launch_group_exact<true>(plan, nullptr, true, &err) : launch_group_exact<false>(plan, nullptr, true, &err));
}

} // namespace espdl
