// Depthwise int8 convolution for gfx950 with the input tile staged in LDS (channels % 16 == 0, up to
// 12 filter taps).
//
// What it computes is depthwise_conv2d_33c1 / _hwc1 (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:19-65)
// under dwconv_operation_shell's window clipping (esp-dl/dl/base/dl_base.hpp:1852-2102) and the n_wise
// epilogue (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210).
//
// The operator moves two bytes per nine multiply-accumulates, so it has to run at memory speed, and
// that decides the structure:
//   * Every input byte is read from global memory once per tile, as part of a contiguous run:
//     a workgroup copies the (th*s + halo) x (tw*s + halo) x (16*gc channels) input patch of its
//     output tile into LDS with 16-byte loads of consecutive addresses (a pixel's channel chunk is
//     contiguous, a patch row is contiguous when the chunk is the whole pixel).  Out-of-image
//     positions are written as zeros, which is the reference's window clipping.  The patch of the
//     next tile is in flight (in registers) while the current one is computed.
//   * The byte products run on v_mfma_i32_16x16x64_i8 with a diagonal operand A (rows = 16 channels,
//     reduction axis = (tap, channel), A[i][(tap, c)] = w[tap][i] if c == i): three MFMAs finish 16
//     pixels x 16 channels x up to 12 taps, and operand B is one 16-byte LDS read per lane and k
//     step, at patch offset (pixel) + (tap) + 16 * group.  The vector ALU is left with three adds
//     and the epilogue per MFMA tile.  Windows of three columns take one k step per window row (slots
//     kx 0, 1, 2 and 2 again with zero weights): lane groups that read LDS together then address pieces
//     one pixel pitch apart or the same piece, which is free of bank conflicts at an odd pitch.
//   * MFMA tiles are taken group-major and split evenly over the four wavefronts; a wavefront
//     rebuilds operand A and its per-channel constants only when the channel group changes.
//   * Results go to an LDS copy of the output tile and leave as 16-byte stores of consecutive
//     addresses.
//   * Optional stages around the depthwise one, all on the tile while it is in LDS: a 1x1 project
//     convolution (+ residual Add) behind it, and a 1x1 expand convolution in front of it that computes
//     the patch from a patch of the block input (at most 64 channels) instead of reading it.
// A workgroup is persistent over tiles; tiles of one XCD are contiguous in memory (xcd_tile_sequence).
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

constexpr int kThreads = 512; // 8 wavefronts share one patch: fewer chunks (registers) per thread
constexpr int kWaves = kThreads / 64;
constexpr int kKs = 3;     // k steps of 4 taps: windows of up to 12 taps (3 x 3) ...
constexpr int kKsWide = 7; // ... and of up to 28 (5 x 5), in builds of their own (plain depthwise only)
constexpr int kMaxIn = 5;  // 16-byte patch chunks per thread
constexpr int kMaxOut = 4; // 16-byte output chunks per thread
constexpr int kMaxX = 4;   // dwords of the expand stage's input patch per thread

struct DwLdsArgs {
    const int8_t *in;
    const int8_t *w;
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
    int8_t *out;
    ConvGeom g;
    int taps;
    int img_bytes;      // bytes of one image of the input tensor
    int row3;           // 1: windows of 3 columns and at most 3 rows take one k step per window row (slots kx 0, 1, 2, 2)
    int ks_used;        // k steps that hold taps
    int th, tw;         // output tile, pixels
    int ph, pw;         // input patch, pixels
    int gc;             // channel groups of 16 per workgroup (divides in_c / 16)
    int cs;             // LDS pixel stride of the patch, bytes (an odd number of 16-byte units)
    int cso;            // LDS pixel stride of the output tile, bytes
    int np;             // pixel tiles of 16 per output tile
    int tiles_x, tiles_y;
    int n_units;        // batch * tiles_y * tiles_x
    int n_in_chunks;    // ph * pw * gc
    int n_out_chunks;   // th * tw * gc
    int tiles_per_wave; // ceil(gc * np / kWaves)
    FastDiv fd_tiles_x, fd_tiles_yx, fd_pwgc, fd_gc, fd_tw, fd_np;
    // LDS layout, byte offsets
    int off_patch, off_out, off_a, off_init, off_ss, off_ls, off_pixtab, off_lut;
    // optional 1x1 project convolution (+ residual Add) applied to the depthwise result of the tile
    // while it is still in LDS; needs every channel in one workgroup (gc == in_c / 16)
    DwProject pj;
    int p_nrt;          // row tiles of 16 project filters
    int p_ks;           // k steps of 64 depthwise channels
    int p_os;           // LDS pixel stride of the project result, bytes
    int p_vec;          // bytes per store piece of the project result: 16 or 4
    int p_vecs;         // pieces per pixel
    int n_pout_chunks;  // th * tw * p_vecs
    FastDiv fd_pvecs;
    int off_wp, off_cp, off_pout;
    // optional 1x1 expand convolution in front: the patch is computed from a patch of the block input
    // (ex.c0 <= 64 channels) instead of being read, so the expanded tensor never exists in memory
    DwExpand ex;
    int xs;              // LDS pixel stride of the block-input patch, bytes (an odd number of 16-byte units)
    int x_units;         // 16-byte units of a pixel that hold data: ceil(c0 / 16)
    int n_x_dwords;      // ph * pw * c0 / 4
    int n_xpt;           // pixel tiles of 16 in the patch
    FastDiv fd_xdw, fd_pw, fd_nxg;
    int off_xin, off_xrc, off_we, off_ce;
};

struct UnitPos {
    int n, y0, x0; // image, first output row / column of the tile
};

__device__ __forceinline__ UnitPos dw_unit(const DwLdsArgs &a, int unit)
{
    UnitPos u;
    const unsigned n = fastdiv((unsigned)unit, a.fd_tiles_yx);
    const unsigned rem = (unsigned)unit - n * a.fd_tiles_yx.d;
    const unsigned ty = fastdiv(rem, a.fd_tiles_x);
    u.n = (int)n;
    u.y0 = (int)ty * a.th;
    u.x0 = (int)(rem - ty * a.fd_tiles_x.d) * a.tw;
    return u;
}

// Patch chunks of this thread for one tile: global -> registers (zeros outside the image).
//
// The loads and the wait for them (dw_settle) are written as instructions.  The chunks are used at the top of
// the next iteration of the tile loop, after this tile's stores; a wavefront's loads and stores share one
// counter, and the compiler, for which the two kinds may complete in any order, waits there for the counter to
// reach zero - for the stores just issued as well, so no tile's stores would overlap the next tile's work.
// dw_settle() waits in front of the stores instead (the loads have had the whole compute phase to arrive) and
// nothing waits where the chunks are used.  What the compiler does not know any more has to hold by
// construction:
//   * between dw_fetch and dw_settle nothing may read or move a chunk.  The compiler sees the chunks as values
//     defined here and used by the LDS writes at the top of the loop and has no reason to touch them; the build
//     checks in the generated code that it did not (build.py: check_hand_waited_loads);
//   * the loads go through a buffer descriptor of the tile's image, and a chunk outside the image gets an offset
//     past the descriptor's end and comes back as zeros: no branch around a load, no select behind it;
//   * the descriptor may have been moved into its scalar registers by vector instructions right before a load,
//     and a memory instruction may read such a register five wait states later at the earliest: the compiler
//     pads its own instructions, not the text of an asm statement, hence the s_nop.
__device__ __forceinline__ void dw_fetch(const DwLdsArgs &a, const UnitPos &u, int cc0, const int (&rel)[kMaxIn],
                                         const int (&rc)[kMaxIn], v4i (&pv)[kMaxIn])
{
    const ConvGeom &g = a.g;
    const int iy0 = u.y0 * g.stride_h - g.pad_top, ix0 = u.x0 * g.stride_w - g.pad_left;
    // buffer descriptor: base, stride 0, bytes, 32-bit raw format
    const __amdgpu_buffer_rsrc_t img = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t *>(a.in + (long long)u.n * a.img_bytes + cc0), (short)0, a.img_bytes - cc0, 0x00020000);
    const int org = (iy0 * g.in_w + ix0) * g.in_c;
#pragma unroll
    for (int i = 0; i < kMaxIn; i++) {
        if (i * kThreads < a.n_in_chunks) { // uniform
            const int iy = iy0 + (rc[i] & 0xffff), ix = ix0 + (rc[i] >> 16);
            const bool ok = rc[i] >= 0 && (unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w;
            const int off = ok ? org + rel[i] : (int)0x80000000u;
            asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(pv[i]) : "v"(off), "s"(img));
        }
    }
}

// Wait for the wavefront's outstanding vector-memory instructions, as an instruction of its own.
__device__ __forceinline__ void dw_settle()
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// Block-input patch dwords of this thread for one tile (expand form): global -> registers.
__device__ __forceinline__ void dw_fetch_x(const DwLdsArgs &a, const UnitPos &u, const int (&rel)[kMaxX],
                                           const int (&rc)[kMaxX], int (&xv)[kMaxX])
{
    const ConvGeom &g = a.g;
    const int iy0 = u.y0 * g.stride_h - g.pad_top, ix0 = u.x0 * g.stride_w - g.pad_left;
    const int8_t *base = a.ex.x + (((long long)u.n * g.in_h + iy0) * g.in_w + ix0) * a.ex.c0;
#pragma unroll
    for (int i = 0; i < kMaxX; i++) {
        if (i * kThreads < a.n_x_dwords) { // uniform
            const int iy = iy0 + (rc[i] & 0xffff), ix = ix0 + (rc[i] >> 16);
            const bool ok = rc[i] >= 0 && (unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w;
            xv[i] = ok ? *reinterpret_cast<const int *>(base + rel[i]) : 0;
        }
    }
}

// Expand stage of one tile: patch[pixel][channel] = act(requant(w_e[channel] . x[pixel] + bias)) for the
// pixels of the patch that lie inside the image, zero for the others (the depthwise stage's window
// clipping).  Rows = 16 expanded channels, columns = 16 patch pixels, one MFMA per tile (c0 <= 64).
// A wavefront takes units of four pixel tiles of one channel tile, so that four independent
// load -> MFMA -> requantize -> store chains are in flight.  INTERIOR: the whole patch lies inside the
// image, no per-pixel test (pixel slots past the patch fall into slack the patch area keeps for them).
template <int MODE, bool INTERIOR> // MODE: pack_fast4 mode, or -1 for the general epilogue
__device__ __forceinline__ void dw_expand(const DwLdsArgs &a, unsigned char *smem, int wave, int lane, const UnitPos &u,
                                          int floor_e)
{
    const ConvGeom &g = a.g;
    const int col = lane & 15, quad = lane >> 4;
    const int iy0 = u.y0 * g.stride_h - g.pad_top, ix0 = u.x0 * g.stride_w - g.pad_left;
    const int *xrc = reinterpret_cast<const int *>(smem + a.off_xrc);
    const int *ce = reinterpret_cast<const int *>(smem + a.off_ce);
    const unsigned char *xin = smem + a.off_xin + col * a.xs + 16 * quad;
    unsigned char *patch = smem + a.off_patch + col * a.cs + 4 * quad;
    const int cw = a.gc * 16;
    const int n_xg = (a.n_xpt + 3) >> 2;
    const int n_units = a.gc * n_xg;
    const bool has_k = quad < a.x_units;
    // the wavefront index is the same in every lane: say so, so that the unit walk and its guards are scalar
    for (int unit = __builtin_amdgcn_readfirstlane(wave); unit < n_units; unit += kWaves) {
        const int ct = (int)fastdiv((unsigned)unit, a.fd_nxg);
        const int pt0 = (unit - ct * n_xg) * 4;
        const int cnt = min(4, a.n_xpt - pt0); // uniform
        const v4i aop = *reinterpret_cast<const v4i *>(smem + a.off_we + 16 * (ct * 64 + lane));
        const int ch = 16 * ct + 4 * quad;
        const v4i init = *reinterpret_cast<const v4i *>(ce + ch);
        const v4i ss = *reinterpret_cast<const v4i *>(ce + cw + ch);
        const v4i ls = *reinterpret_cast<const v4i *>(ce + 2 * cw + ch);
        v4i b[4], acc[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            b[j] = v4i{0, 0, 0, 0};
            if (j < cnt && has_k)
                b[j] = *reinterpret_cast<const v4i *>(xin + (pt0 + j) * 16 * a.xs);
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (j < cnt)
                acc[j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, b[j], init, 0, 0, 0);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (j < cnt) {
                int word;
                if constexpr (MODE >= 0) {
                    word = pack_fast4<MODE>(acc[j], ls, ss, floor_e);
                } else {
                    int q[4];
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        q[r] = requant_s8(acc[j][r], ss[r], a.ex.relu != 0, g.half_even != 0);
                    word = pack4_s8(q[0], q[1], q[2], q[3]);
                }
                int *dst = reinterpret_cast<int *>(patch + (pt0 + j) * 16 * a.cs + 16 * ct);
                if constexpr (INTERIOR) {
                    *dst = word;
                } else {
                    const int prc = xrc[(pt0 + j) * 16 + col];
                    if (prc >= 0) {
                        const int iy = iy0 + (prc & 0xffff), ix = ix0 + (prc >> 16);
                        *dst = ((unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w) ? word : 0;
                    }
                }
            }
        }
    }
}

// Tap of k slot `slot` (k step slot / 4, lane group slot % 4), or -1 for a slot without one; `*twin` is the tap
// whose patch offset an empty slot reads (its weights are zero).  Lane groups 0 / 1 and 2 / 3 read LDS
// together: their pieces must lie an odd number of 16-byte units apart or coincide, or the read takes two
// passes.  With one k step per window row (3-column windows) the pairs are (kx 0, kx 1) and (kx 2, kx 2 again):
// one pixel pitch apart, and identical.
__device__ __forceinline__ int dw_slot_tap(const DwLdsArgs &a, int slot, int *twin)
{
    if (a.row3) {
        const int ky = slot >> 2, q = slot & 3;
        *twin = ky < a.g.k_h ? ky * 3 + min(q, 2) : 0;
        return (q < 3 && ky < a.g.k_h) ? ky * 3 + q : -1;
    }
    *twin = slot < a.taps ? slot : 0;
    return slot < a.taps ? slot : -1;
}

template <bool FAST, int USE_LSH, int KS>
__device__ __forceinline__ void dw_compute(const DwLdsArgs &a, unsigned char *smem, int wave, int lane,
                                           const int (&tapoff)[KS], int floor_pk)
{
    const ConvGeom &g = a.g;
    const int col = lane & 15, quad = lane >> 4;
    const bool relu = g.relu != 0, half_even = g.half_even != 0, has_lut = a.lut != nullptr;
    const int *a_l = reinterpret_cast<const int *>(smem + a.off_a);
    const int8_t *lut_l = reinterpret_cast<const int8_t *>(smem + a.off_lut);
    const unsigned char *patch = smem + a.off_patch;
    unsigned char *out_l = smem + a.off_out;
    const int *pixtab = reinterpret_cast<const int *>(smem + a.off_pixtab) + col;

    // this wavefront's run of tiles, group-major: [t, t_end) = tiles [p, ...) of group grp, then whole
    // groups, then the head of a last one.  Everything that steers the walk is wave-uniform.
    const int npt = a.np;
    const int t_end = min((wave + 1) * a.tiles_per_wave, a.gc * npt);
    int t = wave * a.tiles_per_wave;
    if (t >= t_end)
        return;
    int grp = (int)fastdiv((unsigned)t, a.fd_np);
    int p = t - grp * npt;
    const bool all_k = a.ks_used == KS; // the usual case: no test per k step

    const int sel = col >> 2; // dword of the 16-byte operand A vector that holds this row's weight
    const int out_lane = col * a.cso + 4 * quad;
    auto finish = [&](const v4i &acc, const v4i &ls, const v4i &ss, unsigned char *dst) {
        int word;
        if (FAST) {
            word = pack_fast4<USE_LSH>(acc, ls, ss, floor_pk);
        } else {
            int q[4];
#pragma unroll
            for (int r = 0; r < 4; r++)
                q[r] = requant_s8(acc[r], ss[r], relu, half_even);
            word = pack4_s8(q[0], q[1], q[2], q[3]);
        }
        if (has_lut)
            word = pack4_s8(lut_l[(int)(int8_t)word + 128], lut_l[(int)(int8_t)(word >> 8) + 128],
                            lut_l[(int)(int8_t)(word >> 16) + 128], lut_l[(word >> 24) + 128]);
        *reinterpret_cast<int *>(dst) = word;
    };
    while (t < t_end) {
        // constants of the channel group; they are waited for here, outside the tile loop, so that the loop's own
        // waits count only its operand reads
        v4i aop[KS], init, ss, ls;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
            const int d = a_l[(grp * KS + ks) * 64 + lane];
            aop[ks] = v4i{sel == 0 ? d : 0, sel == 1 ? d : 0, sel == 2 ? d : 0, sel == 3 ? d : 0};
        }
        const int ch = 16 * grp + 4 * quad;
        init = *reinterpret_cast<const v4i *>(smem + a.off_init + 4 * ch);
        ss = *reinterpret_cast<const v4i *>(smem + a.off_ss + 4 * ch);
        ls = *reinterpret_cast<const v4i *>(smem + a.off_ls + 4 * ch);
        const int p_end = min(npt, p + (t_end - t)); // uniform
        const unsigned char *pg = patch + 16 * grp;
        unsigned char *og = out_l + out_lane + 16 * grp;
        // operand B one tile ahead, its patch offset two tiles ahead
        int po = pixtab[p * 16];
        int po_next = pixtab[min(p + 1, npt - 1) * 16];
        v4i b[KS];
#pragma unroll
        for (int ks = 0; ks < KS; ks++)
            b[ks] = *reinterpret_cast<const v4i *>(pg + po + tapoff[ks]);
        t += p_end - p;
        for (; p < p_end; p++) {
            v4i acc = init;
            if (all_k) {
#pragma unroll
                for (int ks = 0; ks < KS; ks++)
                    acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], b[ks], acc, 0, 0, 0);
            } else {
#pragma unroll
                for (int ks = 0; ks < KS; ks++)
                    if (ks < a.ks_used)
                        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], b[ks], acc, 0, 0, 0);
            }
            // the next tile's operand B is read while this one is in the matrix pipe and the epilogue (past the
            // last tile of the run the reads repeat a valid offset and are dropped)
            po = po_next;
            po_next = pixtab[min(p + 2, npt - 1) * 16];
#pragma unroll
            for (int ks = 0; ks < KS; ks++)
                b[ks] = *reinterpret_cast<const v4i *>(pg + po + tapoff[ks]);
            finish(acc, ls, ss, og + p * 16 * a.cso);
        }
        p = 0;
        grp++;
    }
}

// HE: the round-half-even build (a separate kernel so that the half-up build keeps its register count).
// KS: k steps of 4 taps the build holds operands for (kKs, or kKsWide for windows of 13 to 28 taps).
template <bool PROJ, bool HE, bool EXP, int KS = kKs>
__global__ __launch_bounds__(kThreads, KS > kKs ? 2 : 4) void depthwise_s8_lds_kernel(const DwLdsArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6); // the same in every lane: loops over it are scalar
    const int quad = lane >> 4;
    const int C = g.in_c;
    const int cc0 = blockIdx.y * a.gc * 16; // first channel of this workgroup's chunk
    const int cw = a.gc * 16;
    const bool half_even = g.half_even != 0;

    // per-thread chunk descriptors: the tile geometry is the same for every tile
    int in_rel[kMaxIn], in_lds[kMaxIn], in_rc[kMaxIn];
#pragma unroll
    for (int i = 0; i < kMaxIn; i++) {
        const int k = tid + i * kThreads;
        if (k < a.n_in_chunks) {
            const unsigned prow = fastdiv((unsigned)k, a.fd_pwgc);
            const unsigned rem = (unsigned)k - prow * a.fd_pwgc.d;
            const unsigned pcol = fastdiv(rem, a.fd_gc);
            const unsigned c16 = rem - pcol * a.fd_gc.d;
            in_rel[i] = (int)((prow * g.in_w + pcol) * C + c16 * 16);
            in_lds[i] = (int)((prow * a.pw + pcol) * a.cs + c16 * 16);
            in_rc[i] = (int)(prow | (pcol << 16));
        } else {
            in_rel[i] = 0;
            in_lds[i] = -1;
            in_rc[i] = -1;
        }
    }
    int x_rel[kMaxX], x_lds[kMaxX], x_rc[kMaxX];
#pragma unroll
    for (int i = 0; i < kMaxX; i++) {
        const int k = tid + i * kThreads;
        if (EXP && k < a.n_x_dwords) {
            const unsigned q = fastdiv((unsigned)k, a.fd_xdw);
            const unsigned d = (unsigned)k - q * a.fd_xdw.d;
            const unsigned prow = fastdiv(q, a.fd_pw);
            const unsigned pcol = q - prow * a.fd_pw.d;
            x_rel[i] = (int)((prow * g.in_w + pcol) * a.ex.c0 + 4 * d);
            x_lds[i] = (int)(q * a.xs + 4 * d);
            x_rc[i] = (int)(prow | (pcol << 16));
        } else {
            x_rel[i] = 0;
            x_lds[i] = -1;
            x_rc[i] = -1;
        }
    }
    int out_rel[kMaxOut], out_lds[kMaxOut], out_rc[kMaxOut];
#pragma unroll
    for (int i = 0; i < kMaxOut; i++) {
        const int k = tid + i * kThreads;
        if (PROJ && k < a.n_pout_chunks) {
            const unsigned q = fastdiv((unsigned)k, a.fd_pvecs);
            const unsigned v = (unsigned)k - q * a.fd_pvecs.d;
            const unsigned py = fastdiv(q, a.fd_tw);
            const unsigned px = q - py * a.fd_tw.d;
            out_rel[i] = (int)((py * g.out_w + px) * a.pj.out_c + v * a.p_vec);
            out_lds[i] = (int)(q * a.p_os + v * a.p_vec);
            out_rc[i] = (int)(py | (px << 16));
        } else if (!PROJ && k < a.n_out_chunks) {
            const unsigned q = fastdiv((unsigned)k, a.fd_gc);
            const unsigned c16 = (unsigned)k - q * a.fd_gc.d;
            const unsigned py = fastdiv(q, a.fd_tw);
            const unsigned px = q - py * a.fd_tw.d;
            out_rel[i] = (int)((py * g.out_w + px) * C + c16 * 16);
            out_lds[i] = (int)(q * a.cso + c16 * 16);
            out_rc[i] = (int)(py | (px << 16));
        } else {
            out_rel[i] = 0;
            out_lds[i] = 0;
            out_rc[i] = -1;
        }
    }

    const TileSeq seq = xcd_tile_sequence(a.n_units);
    int unit = seq.first;
    v4i pv[kMaxIn];
    int xv[kMaxX];
    UnitPos u = {0, 0, 0};
    if (unit < seq.end) {
        u = dw_unit(a, unit);
        if (EXP)
            dw_fetch_x(a, u, x_rel, x_rc, xv);
        else
            dw_fetch(a, u, cc0, in_rel, in_rc, pv);
    }

    // tables: diagonal operand A as one dword per (group, k step, lane); start values and shifts;
    // patch offset of every output pixel of the tile; the LUT
    int *a_l = reinterpret_cast<int *>(smem + a.off_a);
    for (int e = tid; e < a.gc * KS * 64; e += kThreads) {
        const int l = e & 63, ks = (e >> 6) % KS, gi = e / (64 * KS);
        const int i = l & 15;
        int twin;
        const int tap = dw_slot_tap(a, 4 * ks + (l >> 4), &twin);
        int d = 0;
        if (tap >= 0)
            d = (int)(unsigned char)a.w[(long long)tap * C + cc0 + 16 * gi + i] << (8 * (i & 3));
        a_l[e] = d;
    }
    // start values and shifts: every thread owns at most one channel of the chunk (16 * gc <= 256)
    const long long mac_bound = (long long)a.taps * 16384;
    int ok_local = 1;
    int lsh_local = 0;
    int my_s = 0, my_b = 0;
    if (tid < cw) {
        my_s = a.shift[g.n_shift == 1 ? 0 : cc0 + tid];
        my_b = a.bias != nullptr ? a.bias[cc0 + tid] : 0;
        if (my_s < 1 || my_s > 31) {
            ok_local = 0;
        } else {
            const long long start = (long long)my_b + (1ll << (my_s - 1));
            if ((start < 0 ? -start : start) + mac_bound >= (1ll << (31 - max(0, 8 - my_s))))
                ok_local = 0;
            if (my_s < 8)
                lsh_local = 1;
        }
    }
    const bool fast = __syncthreads_and(ok_local) != 0;
    const bool use_lsh = __syncthreads_or(lsh_local) != 0;
    {
        if (tid < cw) {
            reinterpret_cast<int *>(smem + a.off_init)[tid] = fast ? my_b + (1 << (my_s - 1)) - (HE ? 1 : 0) : my_b; // half-even forms start one lower
            reinterpret_cast<int *>(smem + a.off_ss)[tid] = fast ? max(0, my_s - 8) : my_s;
            reinterpret_cast<int *>(smem + a.off_ls)[tid] = fast ? max(0, 8 - my_s) : 0;
        }
        int *pixtab = reinterpret_cast<int *>(smem + a.off_pixtab);
        for (int q = tid; q < a.np * 16; q += kThreads) {
            int off = 0;
            if (q < a.th * a.tw) {
                const unsigned py = fastdiv((unsigned)q, a.fd_tw);
                const unsigned px = (unsigned)q - py * a.fd_tw.d;
                off = (int)((py * g.stride_h * a.pw + px * g.stride_w) * a.cs);
            }
            pixtab[q] = off;
        }
        if (a.lut != nullptr && tid < 256)
            reinterpret_cast<int8_t *>(smem + a.off_lut)[tid] = a.lut[tid];
    }
    // tap offsets of this lane's quad inside the patch
    int tapoff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
        int twin; // empty slots read where a neighbour reads: no bank conflict, no read outside the patch
        (void)dw_slot_tap(a, 4 * ks + quad, &twin);
        const int ky = twin / g.k_w, kx = twin - ky * g.k_w;
        tapoff[ks] = (ky * g.dil_h * a.pw + kx * g.dil_w) * a.cs;
    }
    const int floor_pk = g.relu ? 0 : (int)0x80008000u;

    // project stage: filters in MFMA operand-A order (row i of row tile rt is filter 16*rt + i, the
    // lane's 16 k positions are depthwise channels 64*ks + 16*gk ...; zeros past out_c and past C),
    // and the stage's [start value | shift | left shift] table
    bool fast_p = false;
    int floor_p = 0;
    if (PROJ) {
        const DwProject &pj = a.pj;
        for (int e = tid; e < a.p_nrt * a.p_ks * 64; e += kThreads) {
            const int l = e & 63, ks = (e >> 6) % a.p_ks, rt = (e >> 6) / a.p_ks;
            const int f = 16 * rt + (l & 15), k0 = 64 * ks + 16 * (l >> 4);
            v4i w = {0, 0, 0, 0};
            if (f < pj.out_c && k0 < C)
                w = *reinterpret_cast<const v4i *>(pj.w + (long long)f * C + k0);
            *reinterpret_cast<v4i *>(smem + a.off_wp + 16 * e) = w;
        }
        const int ocp = a.p_nrt * 16;
        const long long bound = (long long)C * 16384;
        int okp = 1;
        int ps = 0, pb = 0;
        if (tid < pj.out_c) {
            ps = pj.shift[pj.n_shift == 1 ? 0 : tid];
            pb = pj.bias != nullptr ? pj.bias[tid] : 0;
            if (ps < 1 || ps > 31) {
                okp = 0;
            } else {
                const long long start = (long long)pb + (1ll << (ps - 1));
                if ((start < 0 ? -start : start) + bound >= (1ll << (31 - max(0, 8 - ps))))
                    okp = 0;
            }
        }
        fast_p = __syncthreads_and(okp) != 0;
        int *cp = reinterpret_cast<int *>(smem + a.off_cp);
        if (tid < ocp) {
            cp[tid] = (fast_p && tid < pj.out_c) ? pb + (1 << (ps - 1)) - (HE ? 1 : 0) : pb;
            cp[ocp + tid] = fast_p ? max(0, ps - 8) : ps;
            cp[2 * ocp + tid] = fast_p ? max(0, 8 - ps) : 0;
        }
        floor_p = pj.relu ? 0 : (int)0x80008000u;
    }

    // expand stage: filters in MFMA operand-A order (row i of channel tile ct is expanded channel
    // cc0 + 16*ct + i, the lane's 16 k positions are block-input channels 16*quad ...; zeros past c0), the
    // [start value | shift | left shift] table, the (row, column) of every patch pixel, and a cleared
    // block-input patch (its bytes past c0 stay zero)
    bool fast_e = false;
    int floor_e = 0;
    if (EXP) {
        const DwExpand &ex = a.ex;
        for (int e = tid; e < a.gc * 64 * 16; e += kThreads) {
            const int byte = e & 15, l = (e >> 4) & 63, ct = e >> 10;
            const int ch = cc0 + 16 * ct + (l & 15), k = 16 * (l >> 4) + byte;
            smem[a.off_we + e] = k < ex.c0 ? (unsigned char)ex.w[(long long)ch * ex.c0 + k] : (unsigned char)0;
        }
        const long long bound = (long long)ex.c0 * 16384;
        int oke = 1;
        int es = 0, eb = 0;
        if (tid < cw) {
            es = ex.shift[ex.n_shift == 1 ? 0 : cc0 + tid];
            eb = ex.bias != nullptr ? ex.bias[cc0 + tid] : 0;
            if (es < 1 || es > 31) {
                oke = 0;
            } else {
                const long long start = (long long)eb + (1ll << (es - 1));
                if ((start < 0 ? -start : start) + bound >= (1ll << (31 - max(0, 8 - es))))
                    oke = 0;
            }
        }
        fast_e = __syncthreads_and(oke) != 0;
        int *ce = reinterpret_cast<int *>(smem + a.off_ce);
        if (tid < cw) {
            ce[tid] = fast_e ? eb + (1 << (es - 1)) - (HE ? 1 : 0) : eb;
            ce[cw + tid] = fast_e ? max(0, es - 8) : es;
            ce[2 * cw + tid] = fast_e ? max(0, 8 - es) : 0;
        }
        int *xrc = reinterpret_cast<int *>(smem + a.off_xrc);
        for (int q = tid; q < a.n_xpt * 16; q += kThreads) {
            int v = -1;
            if (q < a.ph * a.pw) {
                const unsigned prow = fastdiv((unsigned)q, a.fd_pw);
                v = (int)(prow | (((unsigned)q - prow * a.fd_pw.d) << 16));
            }
            xrc[q] = v;
        }
        for (int e = tid; e < a.n_xpt * 16 * a.xs / 4; e += kThreads)
            reinterpret_cast<int *>(smem + a.off_xin)[e] = 0;
        floor_e = ex.relu ? 0 : (int)0x80008000u;
        __syncthreads(); // the cleared patch must not overtake the first tile's stores below
    }

    if (!EXP)
        dw_settle(); // the first patch
    for (; unit < seq.end; unit += seq.step) {
        // patch of this tile: registers -> LDS
        if (EXP) {
#pragma unroll
            for (int i = 0; i < kMaxX; i++)
                if (i * kThreads < a.n_x_dwords && x_lds[i] >= 0)
                    *reinterpret_cast<int *>(smem + a.off_xin + x_lds[i]) = xv[i];
        } else {
#pragma unroll
            for (int i = 0; i < kMaxIn; i++)
                if (i * kThreads < a.n_in_chunks && in_lds[i] >= 0)
                    *reinterpret_cast<v4i *>(smem + a.off_patch + in_lds[i]) = pv[i];
        }
        __syncthreads();
        const UnitPos u_cur = u;
        const int unit_next = unit + seq.step;
        if (unit_next < seq.end) {
            u = dw_unit(a, unit_next);
            if (EXP)
                dw_fetch_x(a, u, x_rel, x_rc, xv); // in flight during the compute phases
            else
                dw_fetch(a, u, cc0, in_rel, in_rc, pv);
        }
        if (EXP) {
            const int py0 = u_cur.y0 * g.stride_h - g.pad_top, px0 = u_cur.x0 * g.stride_w - g.pad_left;
            const bool interior = py0 >= 0 && px0 >= 0 && py0 + a.ph <= g.in_h && px0 + a.pw <= g.in_w;
            if (fast_e && interior)
                dw_expand<HE ? 5 : 1, true>(a, smem, wave, lane, u_cur, floor_e);
            else if (fast_e)
                dw_expand<HE ? 5 : 1, false>(a, smem, wave, lane, u_cur, floor_e);
            else
                dw_expand<-1, false>(a, smem, wave, lane, u_cur, floor_e);
            __syncthreads();
        }

        // epilogue mode of pack_fast4: 0 plain (every shift >= 8), 1 with the left shift, 5 the same with
        // round-half-even
        if (fast && HE)
            dw_compute<true, 5, KS>(a, smem, wave, lane, tapoff, floor_pk);
        else if (fast && !use_lsh)
            dw_compute<true, 0, KS>(a, smem, wave, lane, tapoff, floor_pk);
        else if (fast)
            dw_compute<true, 1, KS>(a, smem, wave, lane, tapoff, floor_pk);
        else
            dw_compute<false, 0, KS>(a, smem, wave, lane, tapoff, floor_pk);
        __syncthreads();

        if (PROJ) {
            // 1x1 project convolution of the tile: rows = filters, columns = tile pixels, reduction
            // over the depthwise channels, operand B straight from the depthwise result in LDS
            const DwProject &pj = a.pj;
            const int col = lane & 15;
            const int ocp = a.p_nrt * 16;
            const int *cp = reinterpret_cast<const int *>(smem + a.off_cp);
            const int n_t = a.p_nrt * a.np;
            for (int t = wave; t < n_t; t += kWaves) {
                const int rt = (int)fastdiv((unsigned)t, a.fd_np);
                const int ct = t - rt * a.np;
                const int c = 16 * rt + 4 * quad;
                v4i r = *reinterpret_cast<const v4i *>(cp + c);
                const unsigned char *bsrc = smem + a.off_out + (ct * 16 + col) * a.cso + 16 * quad;
                const unsigned char *asrc = smem + a.off_wp + 16 * (rt * a.p_ks * 64 + lane);
                for (int ks = 0; ks < a.p_ks; ks++) {
                    const v4i aop = *reinterpret_cast<const v4i *>(asrc + 1024 * ks);
                    const v4i b = *reinterpret_cast<const v4i *>(bsrc + 64 * ks);
                    r = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, b, r, 0, 0, 0);
                }
                const v4i ss = *reinterpret_cast<const v4i *>(cp + ocp + c);
                int word;
                if (fast_p) {
                    const v4i ls = *reinterpret_cast<const v4i *>(cp + 2 * ocp + c);
                    word = pack_fast4<HE ? 5 : 1>(r, ls, ss, floor_p);
                } else {
                    int q[4];
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        q[k] = requant_s8(r[k], ss[k], pj.relu != 0, half_even);
                    word = pack4_s8(q[0], q[1], q[2], q[3]);
                }
                *reinterpret_cast<int *>(smem + a.off_pout + (ct * 16 + col) * a.p_os + c) = word;
            }
            __syncthreads();
        }

        // result tile: LDS -> global, consecutive pieces; the next patch has arrived before the first store
        if (!EXP)
            dw_settle();
        const int rows = min(a.th, g.out_h - u_cur.y0), cols = min(a.tw, g.out_w - u_cur.x0);
        if (PROJ) {
            const DwProject &pj = a.pj;
            const long long gbase = (((long long)u_cur.n * g.out_h + u_cur.y0) * g.out_w + u_cur.x0) * pj.out_c;
#pragma unroll
            for (int i = 0; i < kMaxOut; i++) {
                if (i * kThreads < a.n_pout_chunks) { // uniform
                    const int py = out_rc[i] & 0xffff, px = out_rc[i] >> 16;
                    if (out_rc[i] >= 0 && py < rows && px < cols) {
                        const long long go = gbase + out_rel[i];
                        if (a.p_vec == 16) {
                            v4i w = *reinterpret_cast<const v4i *>(smem + a.off_pout + out_lds[i]);
                            if (pj.residual != nullptr) {
                                const v4i rv = *reinterpret_cast<const v4i *>(pj.residual + go);
#pragma unroll
                                for (int d = 0; d < 4; d++)
                                    w[d] = sat_add4_s8(w[d], rv[d]);
                            }
                            *reinterpret_cast<v4i *>(pj.out + go) = w;
                        } else {
                            int w = *reinterpret_cast<const int *>(smem + a.off_pout + out_lds[i]);
                            if (pj.residual != nullptr)
                                w = sat_add4_s8(w, *reinterpret_cast<const int *>(pj.residual + go));
                            *reinterpret_cast<int *>(pj.out + go) = w;
                        }
                    }
                }
            }
        } else {
            int8_t *obase = a.out + (((long long)u_cur.n * g.out_h + u_cur.y0) * g.out_w + u_cur.x0) * C + cc0;
#pragma unroll
            for (int i = 0; i < kMaxOut; i++) {
                if (i * kThreads < a.n_out_chunks) { // uniform
                    const int py = out_rc[i] & 0xffff, px = out_rc[i] >> 16;
                    if (out_rc[i] >= 0 && py < rows && px < cols)
                        *reinterpret_cast<v4i *>(obase + out_rel[i]) =
                            *reinterpret_cast<const v4i *>(smem + a.off_out + out_lds[i]);
                }
            }
        }
        // the next iteration's patch stores touch only the patch area; its stores to the result tiles
        // come after the barrier that follows them, by which time these reads have completed
    }
}

struct DwLdsPlan {
    bool ok;
    DwLdsArgs a;
    size_t lds;
    int n_cchunk;
};

constexpr int kLdsBudget = 80 * 1024; // two workgroups of 8 wavefronts per CU (160 KB of LDS)

// Tile choice: the cheapest (patch bytes read per output byte, with a penalty for tiles too small
// to amortize the per-tile barriers) among the candidates that fit the LDS and register budgets.
// pixel tiles of 16 in a patch when an expand stage fills it, else 0
int expand_n_xpt(int ph, int pw, const DwExpand *ex)
{
    return ex != nullptr && ex->w != nullptr ? (ph * pw + 15) / 16 : 0;
}

DwLdsPlan dw_lds_plan(const ConvGeom &g, const DwProject *pj = nullptr, const DwExpand *ex = nullptr)
{
    DwLdsPlan best;
    best.ok = false;
    const int G = g.in_c / 16;
    const int taps = g.k_h * g.k_w;
    const int ks_steps = taps > 4 * kKs ? kKsWide : kKs;
    const int halo_h = (g.k_h - 1) * g.dil_h + 1, halo_w = (g.k_w - 1) * g.dil_w + 1;
    double best_cost = 1e30;
    static const int sizes[] = {1, 2, 3, 4, 6, 7, 8, 12, 14, 16, 24, 28, 32, 56, 64, 112};
    std::vector<int> cand_h, cand_w;
    for (int v : sizes) {
        if (v < g.out_h)
            cand_h.push_back(v);
        if (v < g.out_w)
            cand_w.push_back(v);
    }
    cand_h.push_back(g.out_h);
    cand_w.push_back(g.out_w);
    if ((long long)g.in_h * g.in_w * g.in_c >= (1ll << 31)) // chunk offsets inside an image are 32-bit
        return best;
    const bool proj = pj != nullptr && pj->w != nullptr;
    int p_nrt = 0, p_ks = 0, p_os = 0, p_vec = 16, p_vecs = 0;
    if (proj) {
        if (G > 16 || pj->out_c > 384 || (pj->out_c & 3) != 0)
            return best;
        p_nrt = (pj->out_c + 15) / 16;
        p_ks = (g.in_c + 63) / 64;
        p_os = 16 * ((p_nrt & 1) ? p_nrt : p_nrt + 1);
        const bool al16 = (pj->out_c & 15) == 0 && (reinterpret_cast<uintptr_t>(pj->out) & 15) == 0 &&
            (pj->residual == nullptr || (reinterpret_cast<uintptr_t>(pj->residual) & 15) == 0);
        p_vec = al16 ? 16 : 4;
        p_vecs = pj->out_c / p_vec;
    }
    const bool expand = ex != nullptr && ex->w != nullptr;
    int x_units = 0, xs = 0;
    if (expand) {
        if (ex->c0 < 4 || ex->c0 > 64 || (ex->c0 & 3) != 0)
            return best;
        x_units = (ex->c0 + 15) / 16;
        xs = 16 * ((x_units & 1) ? x_units : x_units + 1);
    }
    for (int gc = 1; gc <= min(G, 16); gc++) {
        if (G % gc != 0 || (proj && gc != G))
            continue;
        const int cs = 16 * ((gc & 1) ? gc : gc + 1); // odd number of 16-byte units: conflict-free LDS reads
        const int cso = cs;
        for (int the : cand_h) {
            for (int twe : cand_w) {
                const int ph = (the - 1) * g.stride_h + halo_h, pw = (twe - 1) * g.stride_w + halo_w;
                const int np = (the * twe + 15) / 16;
                const long long n_in = (long long)ph * pw * gc, n_out = (long long)the * twe * gc;
                if ((!expand && n_in > kMaxIn * kThreads) || n_out > kMaxOut * kThreads || ph > 0xffff || pw > 0x7fff)
                    continue;
                const long long n_x = expand ? (long long)ph * pw * (ex->c0 / 4) : 0;
                const int n_xpt = expand ? (ph * pw + 15) / 16 : 0;
                if (n_x > kMaxX * kThreads)
                    continue;
                const size_t xbytes = expand ? (size_t)n_xpt * 16 * xs + (size_t)n_xpt * 16 * 4 + (size_t)gc * 1024 + (size_t)gc * 16 * 12 : 0;
                // reads of padded pixel slots stay inside; the expand stage also writes whole pixel tiles
                const size_t patch = (size_t)std::max(ph * pw, expand_n_xpt(ph, pw, ex) * 16) * cs + 16 * 16;
                // the project stage reads whole 64-channel k steps: slack after the last pixel
                const size_t outb = (size_t)np * 16 * cso + (proj ? 256 : 0);
                const size_t pbytes = proj ? (size_t)p_nrt * p_ks * 1024 + (size_t)3 * p_nrt * 64 + (size_t)np * 16 * p_os : 0;
                const long long n_pout = (long long)the * twe * p_vecs;
                if (proj && n_pout > kMaxOut * kThreads)
                    continue;
                const size_t tables = (size_t)gc * ks_steps * 64 * 4 + (size_t)gc * 16 * 12 + (size_t)np * 16 * 4 + 256;
                const size_t lds = patch + outb + tables + pbytes + xbytes + 64;
                if (lds > (size_t)kLdsBudget)
                    continue;
                const int per_cu = (int)std::min<size_t>(2, (size_t)(160 * 1024) / lds); // 2 x 8 wavefronts fill a CU
                const double mfma_tiles = (double)np * gc;
                // bytes through the memory system per output byte, relative
                double cost = (double)ph * pw / ((double)the * twe) + 1.0;
                cost *= (double)(np * 16) / (the * twe);           // idle MFMA columns also idle the LDS reads
                cost *= 1.0 + 12.0 / mfma_tiles;                    // barriers and table walks per tile
                cost *= per_cu >= 2 ? 1.0 : 1.6; // latency hiding needs co-resident tiles
                // a pixel's channel chunk should cover whole 128-byte lines unless it is the whole pixel
                if (gc < G && gc * 16 < 128)
                    cost *= 1.0 + 0.5 * (128.0 / (gc * 16) - 1.0);
                // partial tiles at the image edges
                const int ty = (g.out_h + the - 1) / the, tx = (g.out_w + twe - 1) / twe;
                cost *= (double)(ty * the) * (tx * twe) / ((double)g.out_h * g.out_w);
                if (cost < best_cost) {
                    best_cost = cost;
                    best.ok = true;
                    DwLdsArgs &a = best.a;
                    a.taps = taps;
                    a.img_bytes = g.in_h * g.in_w * g.in_c;
                    a.row3 = (g.k_w == 3 && g.k_h <= kKs && ks_steps == kKs) ? 1 : 0;
                    a.ks_used = a.row3 ? g.k_h : (taps + 3) / 4;
                    a.th = the;
                    a.tw = twe;
                    a.ph = ph;
                    a.pw = pw;
                    a.gc = gc;
                    a.cs = cs;
                    a.cso = cso;
                    a.np = np;
                    a.tiles_y = ty;
                    a.tiles_x = tx;
                    a.n_in_chunks = (int)n_in;
                    a.n_out_chunks = (int)n_out;
                    a.tiles_per_wave = (gc * np + kWaves - 1) / kWaves;
                    size_t off = 0;
                    a.off_patch = (int)off;
                    off += (patch + 15) & ~(size_t)15;
                    a.off_out = (int)off;
                    off += outb;
                    a.off_a = (int)off;
                    off += (size_t)gc * ks_steps * 64 * 4;
                    a.off_init = (int)off;
                    off += (size_t)gc * 16 * 4;
                    a.off_ss = (int)off;
                    off += (size_t)gc * 16 * 4;
                    a.off_ls = (int)off;
                    off += (size_t)gc * 16 * 4;
                    a.off_pixtab = (int)off;
                    off += (size_t)np * 16 * 4;
                    a.off_lut = (int)off;
                    off += 256;
                    a.p_nrt = p_nrt;
                    a.p_ks = p_ks;
                    a.p_os = p_os;
                    a.p_vec = p_vec;
                    a.p_vecs = p_vecs;
                    a.n_pout_chunks = (int)n_pout;
                    a.off_wp = (int)off;
                    off += (size_t)p_nrt * p_ks * 1024;
                    a.off_cp = (int)off;
                    off += (size_t)3 * p_nrt * 64;
                    a.off_pout = (int)off;
                    off += proj ? (size_t)np * 16 * p_os : 0;
                    off = (off + 15) & ~(size_t)15;
                    a.xs = xs;
                    a.x_units = x_units;
                    a.n_x_dwords = (int)n_x;
                    a.n_xpt = n_xpt;
                    a.off_xin = (int)off;
                    off += expand ? (size_t)n_xpt * 16 * xs : 0;
                    a.off_xrc = (int)off;
                    off += expand ? (size_t)n_xpt * 16 * 4 : 0;
                    a.off_we = (int)off;
                    off += expand ? (size_t)gc * 1024 : 0;
                    a.off_ce = (int)off;
                    off += expand ? (size_t)gc * 16 * 12 : 0;
                    best.lds = off;
                    best.n_cchunk = G / gc;
                }
            }
        }
    }
    return best;
}

} // namespace

bool depthwise_s8_lds_supports(const ConvGeom &g, const void *in, const void *out)
{
    if ((g.in_c & 15) != 0 || g.k_h * g.k_w > 4 * kKsWide ||
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) != 0)
        return false;
    // 32-bit offsets inside one image
    if ((long long)g.in_h * g.in_w * g.in_c >= (1ll << 30) || (long long)g.out_h * g.out_w * g.out_c >= (1ll << 30))
        return false;
    return dw_lds_plan(g).ok;
}

namespace {

template <bool PROJ, bool EXP = false, int KS = kKs>
hipError_t dw_lds_launch(DwLdsPlan &plan, int cu_count, hipStream_t stream)
{
    DwLdsArgs &a = plan.a;
    const ConvGeom &g = a.g;
    const long long units = (long long)g.batch * a.tiles_y * a.tiles_x;
    if (units > 0x7fffffff)
        return hipErrorInvalidValue;
    a.n_units = (int)units;
    a.fd_tiles_x = make_fastdiv((unsigned)a.tiles_x);
    a.fd_tiles_yx = make_fastdiv((unsigned)(a.tiles_y * a.tiles_x));
    a.fd_pwgc = make_fastdiv((unsigned)(a.pw * a.gc));
    a.fd_gc = make_fastdiv((unsigned)a.gc);
    a.fd_tw = make_fastdiv((unsigned)a.tw);
    a.fd_np = make_fastdiv((unsigned)a.np);
    a.fd_pvecs = make_fastdiv((unsigned)max(1, a.p_vecs));
    a.fd_xdw = make_fastdiv((unsigned)max(1, a.ex.c0 / 4));
    a.fd_pw = make_fastdiv((unsigned)a.pw);
    a.fd_nxg = make_fastdiv((unsigned)max(1, (a.n_xpt + 3) / 4));
    const int cus = cu_count > 0 ? cu_count : 256;
    static const hipError_t lds_opt_in = [] {
        const hipError_t e0 = hipFuncSetAttribute(reinterpret_cast<const void *>(depthwise_s8_lds_kernel<PROJ, false, EXP, KS>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
        const hipError_t e1 = hipFuncSetAttribute(reinterpret_cast<const void *>(depthwise_s8_lds_kernel<PROJ, true, EXP, KS>),
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget);
        return e0 != hipSuccess ? e0 : e1;
    }();
    if (lds_opt_in != hipSuccess)
        return lds_opt_in;
    const bool he = g.half_even != 0;
    const int per_cu = he ? resident_workgroups_per_cu(depthwise_s8_lds_kernel<PROJ, true, EXP, KS>, kThreads, plan.lds)
                          : resident_workgroups_per_cu(depthwise_s8_lds_kernel<PROJ, false, EXP, KS>, kThreads, plan.lds);
    int gx = max(1, (cus * per_cu) / plan.n_cchunk);
    if (gx > a.n_units)
        gx = a.n_units;
    if (gx >= 8)
        gx &= ~7;
    static const bool trace = getenv("ESPDL_HIP_TRACE") != nullptr;
    if (trace)
        fprintf(stderr, "depthwise_s8_lds%s%s: %dx%dx%d s%d tile %dx%d patch %dx%d gc %d np %d lds %zu per_cu %d grid %dx%d units %d\n",
                EXP ? "expand+" : "", PROJ ? "+project" : "", g.in_h, g.in_w, g.in_c, g.stride_h, a.th, a.tw, a.ph, a.pw, a.gc, a.np, plan.lds,
                per_cu, gx, plan.n_cchunk, a.n_units);
    if (he)
        hipLaunchKernelGGL((depthwise_s8_lds_kernel<PROJ, true, EXP, KS>), dim3((unsigned)gx, (unsigned)plan.n_cchunk),
                           dim3(kThreads), plan.lds, stream, a);
    else
        hipLaunchKernelGGL((depthwise_s8_lds_kernel<PROJ, false, EXP, KS>), dim3((unsigned)gx, (unsigned)plan.n_cchunk),
                           dim3(kThreads), plan.lds, stream, a);
    return hipGetLastError();
}

} // namespace

hipError_t launch_depthwise_s8_lds(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                   const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count,
                                   hipStream_t stream)
{
    if ((long long)g.batch * g.out_h * g.out_w == 0)
        return hipSuccess;
    DwLdsPlan plan = dw_lds_plan(g);
    if (!plan.ok)
        return hipErrorInvalidValue;
    DwLdsArgs &a = plan.a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.out = out;
    a.g = g;
    a.pj = DwProject{};
    a.ex = DwExpand{};
    if (a.taps > 4 * kKs) // a 5 x 5 window: the build with seven k steps of taps
        return dw_lds_launch<false, false, kKsWide>(plan, cu_count, stream);
    return dw_lds_launch<false>(plan, cu_count, stream);
}

bool depthwise_project_s8_supports(const ConvGeom &g, const void *in, const DwProject &pj)
{
    if ((g.in_c & 15) != 0 || g.k_h * g.k_w > 4 * kKs || pj.w == nullptr ||
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(pj.w)) & 15) != 0 ||
        ((reinterpret_cast<uintptr_t>(pj.out) | reinterpret_cast<uintptr_t>(pj.residual)) & 3) != 0)
        return false;
    if ((long long)g.in_h * g.in_w * g.in_c >= (1ll << 30) || (long long)g.out_h * g.out_w * pj.out_c >= (1ll << 30))
        return false;
    return dw_lds_plan(g, &pj).ok;
}

hipError_t launch_depthwise_project_s8(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                       const int32_t *shift, const DwProject &pj, int cu_count, hipStream_t stream)
{
    if ((long long)g.batch * g.out_h * g.out_w == 0)
        return hipSuccess;
    DwLdsPlan plan = dw_lds_plan(g, &pj);
    if (!plan.ok)
        return hipErrorInvalidValue;
    DwLdsArgs &a = plan.a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = nullptr;
    a.out = nullptr;
    a.g = g;
    a.pj = pj;
    a.ex = DwExpand{};
    return dw_lds_launch<true>(plan, cu_count, stream);
}

bool expand_depthwise_project_s8_supports(const ConvGeom &g, const DwExpand &ex, const DwProject &pj)
{
    if ((g.in_c & 15) != 0 || g.k_h * g.k_w > 4 * kKs || pj.w == nullptr || ex.w == nullptr || ex.x == nullptr ||
        (reinterpret_cast<uintptr_t>(pj.w) & 15) != 0 || (reinterpret_cast<uintptr_t>(ex.x) & 3) != 0 ||
        ((reinterpret_cast<uintptr_t>(pj.out) | reinterpret_cast<uintptr_t>(pj.residual)) & 3) != 0)
        return false;
    if ((long long)g.in_h * g.in_w * ex.c0 >= (1ll << 30) || (long long)g.out_h * g.out_w * pj.out_c >= (1ll << 30))
        return false;
    return dw_lds_plan(g, &pj, &ex).ok;
}

hipError_t launch_expand_depthwise_project_s8(const ConvGeom &g, const DwExpand &ex, const int8_t *filter,
                                              const int32_t *bias, const int32_t *shift, const DwProject &pj,
                                              int cu_count, hipStream_t stream)
{
    if ((long long)g.batch * g.out_h * g.out_w == 0)
        return hipSuccess;
    DwLdsPlan plan = dw_lds_plan(g, &pj, &ex);
    if (!plan.ok)
        return hipErrorInvalidValue;
    DwLdsArgs &a = plan.a;
    a.in = nullptr;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = nullptr;
    a.out = nullptr;
    a.g = g;
    a.pj = pj;
    a.ex = ex;
    return dw_lds_launch<true, true>(plan, cu_count, stream);
}

} // namespace espdl
