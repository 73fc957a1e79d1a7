// Inverted-residual block (1x1 expand conv -> 3x3 depthwise conv -> 1x1 project conv [-> Add]) for int8
// on gfx950 with ONE WAVEFRONT PER TILE and no workgroup barriers.
//
// Every stage computes exactly what the separate operators compute, in the same integer arithmetic,
// with the int8 result of each stage materialized before the next one reads it:
//   expand / project  conv2d_11cn + n_wise epilogue (esp-dl/dl/base/dl_base_conv2d.cpp:9-33;
//                     esp-dl/dl/base/dl_base_activate_buffer.hpp:10-74, 162-212)
//   depthwise         depthwise_conv2d_33c1 under dwconv_operation_shell's window clipping
//                     (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:19-65; esp-dl/dl/base/dl_base.hpp:1852-2102)
//   Add               saturating int8 add without rescale (esp-dl/dl/base/dl_base_add.cpp:34-44)
// so a fused block is bit-identical to running Conv, Conv, Conv, Add modules one after the other.
//
// Why one wavefront per tile: the block is a chain of small dependent stages (a matrix product, a
// requantization on the vector ALU, a trip through LDS, the next matrix product ...).  A workgroup that
// walks the chain with barriers between the stages leaves every pipe idle most of the time.  Here a
// wavefront owns a th x tw tile of the block's output in one image and runs the whole chain on its own,
// ordered only by its own LDS accesses; the wavefronts of a compute unit sit at different points of the
// chain, so the matrix pipe, the vector ALU, LDS and the memory pipeline of the unit are busy at once.
// Four wavefronts form a workgroup for one reason only: they share the per-channel requantization tables
// of the three stages, built once in LDS before the single barrier of the kernel.
//
// Per tile:
//   * the (th*s + 2) x (tw*s + 2) patch of the block input is loaded ONCE, straight into the registers
//     that are operand B of the expand products (lane = patch pixel x 16 input channels), and stays
//     there for all expanded channels;
//   * the expanded channels are walked in chunks of 16:
//       expand     v_mfma_i32_16x16x64_i8 (rows = 16 expanded channels, columns = 16 patch pixels), fused
//                  shift-round-saturate, zeros for patch pixels outside the image (the depthwise zero
//                  padding pads the EXPANDED activation), int8 result to LDS as [patch pixel][16 ch];
//       depthwise  the same instruction with a diagonal operand A whose reduction axis is
//                  (input row, channel): the four 16-lane groups of a wavefront hold four consecutive
//                  patch rows, so one set of three operand-B reads (kx = 0, 1, 2) serves TWO output rows
//                  through two operand-A sets (rows 0-2 and rows 1-3); result to LDS as [pixel][64 ch];
//     and after every 64 expanded channels the project product accumulates into registers
//     (rows = 16 project filters, columns = one output row of the tile);
//   * project epilogue (constants from the LDS table), residual add, stores.
// Filters are read from global memory (L2) as they are needed, one chunk ahead of their use: 16-byte pieces
// in operand order, no staging.
//
// ROWCONV builds: the expand stage is a dense convolution with a window (a network's stem in front of its
// first depthwise stage: conv2d_hwcn, esp-dl/dl/base/dl_base_conv2d.cpp:35-68) whose filter rows are at
// most 9 bytes (k_w * in_c) and at most 4.  The reduction axis of the expand product is then
// (filter row = 16-lane group, 16 bytes of that row): operand B of a patch pixel is the window's row as it
// lies in memory (k_w * in_c consecutive bytes, cut out of three aligned dwords with v_alignbyte_b32),
// operand A the filter row padded with zeros, prepared once per workgroup in LDS.  Everything behind the
// expand product is the same code.  These tiles are short (two chunks for a 32-filter stem), so a wavefront
// walks several consecutive tiles and the workgroup's set-up is paid once.
#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "mbconv_s8_stages.h"

namespace espdl {

namespace {

using namespace mbstage;

constexpr int kWavesPerGroup = 4;
constexpr int kRowRounds = 4; // ROWCONV guard-free builds: at most 64 * 4 16-byte pieces of copied image rows

struct WaveArgs {
    MbconvParams p;
    int th, tw, ph, pw;
    int n_xpt; // pixel tiles of 16 in the patch
    int tiles_x, tiles_y, n_tiles;
    int tpw; // ROWCONV: consecutive tiles per wavefront
    int n_sub; // chunks of 16 expanded channels
    int rt;    // project row tiles of 16 filters
    int x_vec16, we_vec16;
    int off_exp, off_dw, off_tab;
    int off_aop; // ROWCONV: operand A of the expand stage for every expanded channel, [exp_c][4 rows][16 bytes]
    int off_wd;  // ROWCONV: the depthwise weights as a lane wants them, [exp_c / 16][64 lanes][8 int32]
    int wave_bytes; // LDS of one wavefront (expanded patch + depthwise result); the tables are shared
    // ROWCONV guard-free builds: the image rows under the patch's windows, copied to the wavefront's LDS as
    // consecutive aligned 16-byte pieces (0: the plan has no room for them)
    int rows_n;      // image rows: (ph - 1) * es_h + ek_h
    int rows_ppr;    // 16-byte pieces per copied row
    int rows_rounds; // load instructions per copy: pieces / 64, rounded up
    int off_rows;    // offset of the copied rows inside the wavefront's LDS
    FastDiv fd_pw, fd_tiles_x, fd_tiles_yx, fd_rows_ppr;
};

// EXACT: the tile plan is exactly (NXPT pixel tiles, RT project row tiles, PT rows): no run-time guards in
// the stage loops, so each stage of a chunk is one straight-line block the scheduler can interleave.  Rows
// of a ragged last tile that do not exist are computed from whatever the patch area holds and never stored.
// A workgroup is kWavesPerGroup wavefronts with a tile each; all they share is the requantization tables of
// the expand and depthwise stages, which they build together (one barrier) before going their own ways.
// Everything a tile reads from memory up front (its block-input patch, the residual words it will add at the
// very end, the filters of its first chunk) is requested BEFORE the tables are built, so that one memory
// round trip covers all of it.
// Byte masks of three dwords from a 12-bit byte-validity mask (bit j: byte j is kept).
__device__ __forceinline__ void byte_masks3(unsigned bm, int (&m)[3])
{
#pragma unroll
    for (int k = 0; k < 3; k++) {
        int v = __builtin_amdgcn_sbfe((int)bm, 4 * k, 1) & 0xff;
        v |= __builtin_amdgcn_sbfe((int)bm, 4 * k + 1, 1) & 0xff00;
        v |= __builtin_amdgcn_sbfe((int)bm, 4 * k + 2, 1) & 0xff0000;
        v |= __builtin_amdgcn_sbfe((int)bm, 4 * k + 3, 1) & (int)0xff000000u;
        m[k] = v;
    }
}

// CLIP: a Clip with equal exponents sits behind the expand and / or the depthwise stage (a ReLU6 exported as
// Clip): the stage's int8 result is clamped to the Clip's bounds before it goes to LDS, one packed minimum
// per pair of values on top of the packed maximum the ReLU floor already costs.
template <int NXPT, int RT, int PT, int S, bool HE, bool VEC16, bool EXACT, bool ROWCONV = false, int PACK = 1, bool CLIP = false>
__global__ __launch_bounds__(64 * kWavesPerGroup, EXACT ? ((PACK > 1 && S == 2) ? 3 : 2) : 1) void mbconv_s8_wave_kernel(const WaveArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const MbconvParams &p = a.p;
    const int lane = threadIdx.x & 63, col = lane & 15, quad = lane >> 4;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    unsigned char *exp_l = smem + a.off_exp + wave * a.wave_bytes;
    unsigned char *dw_l = smem + a.off_dw + wave * a.wave_bytes;
    int *tab_e = reinterpret_cast<int *>(smem + a.off_tab);
    int *tab_d = tab_e + 3 * a.p.exp_c;
    int *tab_p = tab_d + 3 * a.p.exp_c; // 3 x 16 rt entries
    const int c0 = p.in_c;

    // tile of this wavefront; consecutive tiles of an image stay on one XCD (its L2 holds the shared halo rows).
    // A wavefront past the last tile works on the last tile again and stores nothing.
    int group = blockIdx.x;
    if ((gridDim.x & 7u) == 0) {
        const int per = gridDim.x >> 3;
        group = (int)(blockIdx.x & 7u) * per + (int)(blockIdx.x >> 3);
    }
    // ROWCONV builds: a wavefront takes a.tpw consecutive tiles (their tiles are short: two chunks of expanded
    // channels), so that the workgroup's set-up serves several tiles
    int mode_e = 0, mode_d = 0, mode_p = 0;
    const int tpw = ROWCONV ? a.tpw : 1;

    // ROWCONV guard-free builds: the image rows under the patch's windows are copied to the wavefront's LDS as
    // consecutive aligned 16-byte pieces, by loads that write LDS directly (no registers in between), one tile
    // ahead: the copy for tile it + 1 is requested behind the first expand stage of tile it and has the rest of
    // the tile to arrive; settle_rows() waits for it in front of the tile's stores (a wait behind them would
    // wait for the stores too: one counter).  Piece i of a copy = piece i % rows_ppr of row i / rows_ppr, at
    // 16 i in the wavefront's row area; a piece whose row lies outside the image, or that would start in front of
    // the tensor or end behind it, gets an offset past the descriptor's end and arrives as zeros.
    constexpr bool kRowCopy = ROWCONV && EXACT;
    struct RowPiece {
        int wy;        // image row
        int lo, hi;    // bytes [lo, hi) of the piece lie inside the image row
        int po;        // byte offset of the piece from the start of the tensor (the tensor has less than 2^30 bytes)
        bool in_row;   // the row exists and the piece has bytes of it
        bool loadable; // the piece lies inside the tensor as a whole
    };
    const int rc_img_bytes = p.img_h * p.img_w * c0;
    const int rc_total = p.batch * rc_img_bytes;
    const int rc_rowb = p.img_w * c0;
    // (everything per lane in 32 bits: u = offset of the first byte the tile's windows touch, the same in every lane)
    auto row_piece = [&](int u, int wy0, int wx0, int j, int lane_now) {
        RowPiece q;
        const unsigned i = (unsigned)(lane_now + 64 * j);
        const unsigned r = fastdiv(i, a.fd_rows_ppr);
        const int pi = (int)(i - r * a.fd_rows_ppr.d);
        q.wy = wy0 + (int)r;
        const int first = u + (int)r * rc_rowb;  // the first byte the windows touch in this row
        const int mis = (int)(((unsigned)reinterpret_cast<uintptr_t>(p.in) + (unsigned)first) & 15u);
        q.po = first - mis + 16 * pi;            // 16-byte aligned as an address
        q.lo = first - wx0 * c0 - q.po;          // the row's first byte, relative to the piece
        q.hi = q.lo + rc_rowb;
        q.in_row = (int)r < a.rows_n && (unsigned)q.wy < (unsigned)p.img_h && q.hi > 0 && q.lo < 16;
        q.loadable = q.po >= 0 && q.po + 16 <= rc_total;
        return q;
    };
    auto tile_origin = [&](int it_n, int &u, int &wy0, int &wx0) {
        const int tile_id = (group * kWavesPerGroup + wave) * tpw + it_n;
        const int tile = min(tile_id, a.n_tiles - 1);
        const unsigned n_img = fastdiv((unsigned)tile, a.fd_tiles_yx);
        const unsigned rem = (unsigned)tile - n_img * a.fd_tiles_yx.d;
        const unsigned ty = fastdiv(rem, a.fd_tiles_x);
        const int oy0 = (int)ty * a.th, ox0 = (int)(rem - ty * a.fd_tiles_x.d) * a.tw;
        wy0 = (oy0 * S - p.pad_top) * p.es_h - p.epad_top;
        wx0 = (ox0 * S - p.pad_left) * p.es_w - p.epad_left;
        u = (int)n_img * rc_img_bytes + wy0 * rc_rowb + wx0 * c0;
    };
    unsigned char *rows_l = smem + a.off_exp + wave * a.wave_bytes + a.off_rows;
    auto request_rows = [&](int it_n) {
        int u, wy0, wx0;
        tile_origin(it_n, u, wy0, wx0);
        const int lane_now = lane; // (what depends on the lane alone is computed once, in front of the tile loop)
        // buffer descriptor of the whole tensor: base, stride 0, bytes, 32-bit raw format
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.in), (short)0, rc_total, 0x00020000);
        const unsigned lds0 = (unsigned)reinterpret_cast<uintptr_t>(rows_l); // LDS address: the low half of the pointer
        // m0 holds the LDS address of lane 0's piece and is read when the data arrives, so it is written once per
        // copy, when no copy is in flight (a write to it waits for the loads that still need it), and left as it is:
        // nothing else in these kernels uses it (the build checks that).  The rounds of a copy differ in the
        // instruction's immediate offset, which counts for the LDS address and for the memory address alike.  The
        // s_nops are the wait states a memory instruction needs after a vector instruction wrote its scalar
        // operands, and after m0 was written.
        asm volatile("s_nop 4\n\ts_mov_b32 m0, %0\n\ts_nop 0" ::"s"(lds0) : "memory");
#pragma unroll
        for (int j = 0; j < kRowRounds; j++)
            if (j < a.rows_rounds) { // uniform
                const RowPiece q = row_piece(u, wy0, wx0, j, lane_now);
                const int off = ((q.in_row && q.loadable) ? q.po : (int)0x80000000u) - 1024 * j;
                asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, 0 offen offset:%2 lds" ::"v"(off), "s"(rsrc), "n"(1024 * j)
                             : "memory");
            }
    };
    auto settle_rows = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };
    // Pieces that hang over an end of their image row carry bytes of the neighbouring row (or lie partly outside
    // the tensor and arrived as zeros): what lies outside the row is the convolution's padding.  Only tiles at the
    // left or right border of the image have such pieces.
    auto fix_row_ends = [&](int u, int wy0, int wx0) {
        // (the lane index through an empty asm statement: what depends on it is computed here, on the few tiles
        // that come here, and not in front of the tile loop, where it would occupy registers over every tile - this
        // kernel has none to spare)
        int lane_now = lane;
        asm volatile("" : "+v"(lane_now));
#pragma unroll
        for (int j = 0; j < kRowRounds; j++)
            if (j < a.rows_rounds) { // uniform
                const RowPiece q = row_piece(u, wy0, wx0, j, lane_now);
                if (q.in_row && (q.lo > 0 || q.hi < 16 || !q.loadable)) {
                    v4i *slot = reinterpret_cast<v4i *>(rows_l + 16 * (lane_now + 64 * j));
                    v4i v = {0, 0, 0, 0};
                    if (q.loadable) {
                        v = *slot;
                    } else { // over an end of the tensor (first or last row of the batch only): byte by byte
#pragma unroll 1
                        for (int k = 0; k < 16; k++)
                            if (q.po + k >= 0 && q.po + k < rc_total)
                                v[k >> 2] |= (int)(unsigned char)p.in[q.po + k] << (8 * (k & 3));
                    }
#pragma unroll
                    for (int dd = 0; dd < 4; dd++) {
                        const int dl = min(max(q.lo - 4 * dd, 0), 4), dh = min(max(q.hi - 4 * dd, 0), 4);
                        const unsigned m_lo = dl >= 4 ? 0u : 0xffffffffu << (8 * dl);
                        const unsigned m_hi = dh >= 4 ? 0xffffffffu : (1u << (8 * dh)) - 1u;
                        v[dd] &= (int)(m_lo & m_hi);
                    }
                    *slot = v;
                }
            }
    };
    if constexpr (kRowCopy)
        request_rows(0);
    for (int it = 0; it < tpw; it++) {
    const int tile_id = (group * kWavesPerGroup + wave) * tpw + it;
    const bool has_tile = tile_id < a.n_tiles; // uniform
    const int tile = min(tile_id, a.n_tiles - 1);
    const unsigned n = fastdiv((unsigned)tile, a.fd_tiles_yx);
    const unsigned rem = (unsigned)tile - n * a.fd_tiles_yx.d;
    const unsigned ty = fastdiv(rem, a.fd_tiles_x);
    const int oy0 = (int)ty * a.th, ox0 = (int)(rem - ty * a.fd_tiles_x.d) * a.tw;
    const int iy0 = oy0 * S - p.pad_top, ix0 = ox0 * S - p.pad_left;
    const int th_real = min(a.th, p.out_h - oy0); // rows of this tile that exist
    const int th = EXACT ? PT : th_real;
    const int n_xpt = EXACT ? NXPT : a.n_xpt;
    const int n_rt = EXACT ? RT : a.rt;

    // block-input patch -> operand B registers of the expand stage; xmask: patch pixels inside the image
    v4i xb[(NXPT + PACK - 1) / PACK];
    unsigned xmask = 0;
    if constexpr (PACK > 1) {
        // at most 64 / PACK input channels: the 4 / PACK 16-lane groups `sub` of tile slot `tsel` of register set
        // g load the 16-byte pieces of patch pixel (PACK g + tsel) * 16 + col; the validity bits of all pixel
        // tiles of a column come from the wavefront's votes
        constexpr int kSubs = 4 / PACK;
        const int tsel = quad / kSubs, sub = quad % kSubs;
        const int8_t *img = p.in + (long long)n * p.in_h * p.in_w * c0;
#pragma unroll
        for (int g = 0; g < (NXPT + PACK - 1) / PACK; g++) {
            const int pt = PACK * g + tsel;
            const unsigned pp = (unsigned)(pt * 16 + col);
            const unsigned prow = fastdiv(pp, a.fd_pw);
            const int iy = iy0 + (int)prow, ix = ix0 + (int)(pp - prow * a.fd_pw.d);
            const bool valid = pt < NXPT && (int)prow < a.ph && (unsigned)iy < (unsigned)p.in_h && (unsigned)ix < (unsigned)p.in_w;
            xb[g] = load16_clamped<VEC16>(img, (unsigned)((iy * p.in_w + ix) * c0 + 16 * sub), valid ? c0 - 16 * sub : 0);
            const unsigned long long votes = __ballot(valid); // bit 16 quad + col
#pragma unroll
            for (int t = 0; t < PACK; t++)
                xmask |= (unsigned)((votes >> (16 * kSubs * t + col)) & 1ull) << (PACK * g + t);
        }
    } else if constexpr (!ROWCONV) {
        const int8_t *img = p.in + (long long)n * p.in_h * p.in_w * c0;
        if constexpr (EXACT && S == 1) {
            // guard-free builds at stride 1 have patches of exactly 16 columns: pixel tile = patch row and lane
            // column = patch column, so the column part of the address and of the validity test is formed once
            // and a patch row costs one addition (rows are uniform: one scalar bit mask)
            const int ix = ix0 + col;
            const bool col_valid = (unsigned)ix < (unsigned)p.in_w;
            const int o0 = (iy0 * p.in_w + ix) * c0 + 16 * quad, o_step = p.in_w * c0;
            unsigned rows = 0;
#pragma unroll
            for (int pt = 0; pt < NXPT; pt++)
                rows |= (unsigned)(iy0 + pt) < (unsigned)p.in_h ? 1u << pt : 0u;
            xmask = col_valid ? rows : 0u;
#pragma unroll
            for (int pt = 0; pt < NXPT; pt++)
                xb[pt] = load16_clamped<VEC16>(img, (unsigned)(o0 + pt * o_step), ((xmask >> pt) & 1u) ? c0 - 16 * quad : 0);
        } else {
#pragma unroll
            for (int pt = 0; pt < NXPT; pt++) {
                xb[pt] = v4i{0, 0, 0, 0};
                if (pt < n_xpt) { // uniform
                    const unsigned pp = (unsigned)(pt * 16 + col);
                    const unsigned prow = fastdiv(pp, a.fd_pw);
                    const int iy = iy0 + (int)prow, ix = ix0 + (int)(pp - prow * a.fd_pw.d);
                    const bool valid = (int)prow < a.ph && (unsigned)iy < (unsigned)p.in_h && (unsigned)ix < (unsigned)p.in_w;
                    xmask |= valid ? 1u << pt : 0u;
                    xb[pt] = load16_clamped<VEC16>(img, (unsigned)((iy * p.in_w + ix) * c0 + 16 * quad),
                                                   valid ? c0 - 16 * quad : 0);
                }
            }
        }
    } else {
        // Lane (col, quad) of pixel tile pt: row `quad` of the window of patch pixel pt * 16 + col, i.e. the
        // wb = ek_w * c0 bytes of input row ry from column rx on, as bytes 0 .. wb-1 of the lane's 16 (bytes
        // from wb on meet zero weights).  They are cut out of the three aligned dwords around them; dword
        // addresses are clamped to the image, bytes outside the image (the convolution's zero padding) and
        // whole rows that do not exist are masked.  A tile whose windows all lie inside the image skips the masks.
        const int rowb = p.img_w * c0;
        const long long img_bytes = (long long)p.img_h * rowb;
        const int8_t *img = p.in + (long long)n * img_bytes;
        const int delta = (int)(reinterpret_cast<uintptr_t>(img) & 3u);
        const int8_t *base = img - delta; // 4-byte aligned; offsets below are relative to it
        const int off_max = (delta + (int)img_bytes - 1) & ~3; // the dword that holds the image's last byte
        const int wy0 = iy0 * p.es_h - p.epad_top, wx0 = ix0 * p.es_w - p.epad_left;
        const bool interior = iy0 >= 0 && ix0 >= 0 && iy0 + a.ph <= p.in_h && ix0 + a.pw <= p.in_w && wy0 >= 0 && wx0 >= 0 &&
            wy0 + (a.ph - 1) * p.es_h + p.ek_h <= p.img_h && wx0 + (a.pw - 1) * p.es_w + p.ek_w <= p.img_w; // uniform
        // byte-validity mask of a window row that starts at input column rx: the columns inside the image
        auto x_bytes = [&](int rx) -> unsigned {
            const int lo = max(0, -rx) * c0, hi = max(0, min(p.ek_w, p.img_w - rx)) * c0;
            return hi > lo ? ((1u << hi) - 1u) & ~((1u << lo) - 1u) : 0u;
        };
        // phase 1: every load of the patch is requested before any of them is used
        int d[NXPT][3];
        unsigned shs = 0;   // two bits per pixel tile: where the row starts inside its first dword
        unsigned rowok = 0; // one bit per pixel tile: the lane's window row exists (filter row, image row, pixel)
        auto request = [&](int pt, int o) {
            const int ab = o & ~3;
            shs |= (unsigned)(o & 3) << (2 * pt);
#pragma unroll
            for (int k = 0; k < 3; k++)
                d[pt][k] = *reinterpret_cast<const int *>(base + (size_t)(unsigned)min(max(ab + 4 * k, 0), off_max));
        };
        int rx_lane = 0; // EXACT: the lane's window column, the same for every pixel tile
        if constexpr (EXACT) {
            // Guard-free builds have 16-pixel-wide patches: pixel tile = patch row, lane column = patch column.
            // The image rows under the windows are in the wavefront's LDS (request_rows, one tile ahead); a lane
            // cuts the window row of each of its patch pixels out of them with one unaligned 16-byte read.
            const int mx = ix0 + col;
            rx_lane = mx * p.es_w - p.epad_left;
            const bool col_valid = (unsigned)mx < (unsigned)p.in_w;
            unsigned rows = 0; // uniform: patch rows inside the depthwise stage's input
#pragma unroll
            for (int pt = 0; pt < NXPT; pt++)
                rows |= (pt < a.ph && (unsigned)(iy0 + pt) < (unsigned)p.in_h) ? 1u << pt : 0u;
            xmask = col_valid ? rows : 0u;
            if (it == 0)
                settle_rows(); // later copies are waited for in front of the previous tile's stores
            // does a piece hang over an end of its row?  (uniform)
            if (wx0 * c0 < 15 || wx0 * c0 + 16 * a.rows_ppr > rowb) {
                fix_row_ends((int)n * rc_img_bytes + wy0 * rowb + wx0 * c0, wy0, wx0);
                wave_lds_sync();
            }
            const int pitch = 16 * a.rows_ppr;
            // the lane's window row of patch pixel (pt, col): copied row pt * es_h + quad (rows past the filter's
            // meet zero weights: any row will do), from byte col * es_w * c0 + the row's skew against 16 bytes
            const unsigned skew0 = (unsigned)(reinterpret_cast<uintptr_t>(img) + (uintptr_t)((long long)wy0 * rowb + wx0 * c0));
            // (three aligned dwords and a funnel shift: neighbouring lanes read the same or neighbouring dwords, which
            // LDS serves in one pass; an unaligned 16-byte read per lane at a 6-byte lane pitch takes several)
#pragma unroll
            for (int pt = 0; pt < NXPT; pt++) {
                const int r = min(pt * p.es_h + quad, a.rows_n - 1);
                const int o = r * pitch + col * p.es_w * c0 + (int)((skew0 + (unsigned)(r * rowb)) & 15u);
                const int *src = reinterpret_cast<const int *>(rows_l + (o & ~3));
                const unsigned sh = (unsigned)o & 3u;
                const int d0 = src[0], d1 = src[1], d2 = src[2];
                xb[pt] = v4i{(int)__builtin_amdgcn_alignbyte((unsigned)d1, (unsigned)d0, sh),
                             (int)__builtin_amdgcn_alignbyte((unsigned)d2, (unsigned)d1, sh),
                             (int)__builtin_amdgcn_alignbyte(0u, (unsigned)d2, sh), 0};
            }
            wave_lds_sync(); // the next tile's copy comes after these reads
        } else {
#pragma unroll
            for (int pt = 0; pt < NXPT; pt++) {
#pragma unroll
                for (int k = 0; k < 3; k++)
                    d[pt][k] = 0;
                if (pt < n_xpt) { // uniform
                    const unsigned pp = (unsigned)(pt * 16 + col);
                    const unsigned prow = fastdiv(pp, a.fd_pw);
                    const int my = iy0 + (int)prow, mx = ix0 + (int)(pp - prow * a.fd_pw.d);
                    const bool valid = (int)prow < a.ph && (unsigned)my < (unsigned)p.in_h && (unsigned)mx < (unsigned)p.in_w;
                    xmask |= valid ? 1u << pt : 0u;
                    const int ry = my * p.es_h - p.epad_top + quad, rx = mx * p.es_w - p.epad_left;
                    request(pt, ry * rowb + rx * c0 + delta); // may lie outside the image; only masked bytes then
                    rowok |= (valid && quad < p.ek_h && (unsigned)ry < (unsigned)p.img_h) ? 1u << pt : 0u;
                }
            }
        }
        // phase 2: cut the rows out of their dwords; border tiles mask what lies outside the image
        int mx3[3] = {-1, -1, -1};
        if (EXACT && !interior)
            byte_masks3(x_bytes(rx_lane), mx3);
#pragma unroll
        for (int pt = 0; pt < (EXACT ? 0 : NXPT); pt++) {
            const unsigned sh = (shs >> (2 * pt)) & 3u;
            int r[3];
            r[0] = (int)__builtin_amdgcn_alignbyte((unsigned)d[pt][1], (unsigned)d[pt][0], sh);
            r[1] = (int)__builtin_amdgcn_alignbyte((unsigned)d[pt][2], (unsigned)d[pt][1], sh);
            r[2] = (int)__builtin_amdgcn_alignbyte(0u, (unsigned)d[pt][2], sh);
            if (!interior) { // uniform
                int m[3];
                if constexpr (EXACT) {
#pragma unroll
                    for (int k = 0; k < 3; k++)
                        m[k] = mx3[k];
                } else {
                    const unsigned pp = (unsigned)(pt * 16 + col);
                    const unsigned prow = fastdiv(pp, a.fd_pw);
                    const int mx = ix0 + (int)(pp - prow * a.fd_pw.d);
                    byte_masks3(x_bytes(mx * p.es_w - p.epad_left), m);
                }
                const int keep = __builtin_amdgcn_sbfe((int)rowok, pt, 1); // all ones or zero
#pragma unroll
                for (int k = 0; k < 3; k++)
                    r[k] &= m[k] & keep;
            }
            xb[pt] = v4i{r[0], r[1], r[2], 0};
        }
    }

    // output words of this lane: pixel (oy0 + t, ox0 + col), filters 16 r + 4 quad ...
    const int ox = ox0 + col;
    const bool col_ok = has_tile && col < a.tw && ox < p.out_w;
    const long long img_off = (long long)n * p.out_h * p.out_w * p.out_c;
    const int8_t *res_img = p.residual != nullptr ? p.residual + img_off : nullptr;
    int8_t *out_img = p.out + img_off;
    const unsigned off0 = (unsigned)((oy0 * p.out_w + ox) * p.out_c + 4 * quad);
    // The residual words (the guard-free builds have the registers for it) are requested now, with the patch,
    // and used after the last chunk: in the epilogue their round trip would be fully exposed.
    constexpr bool kEarlyResidual = EXACT;
    int resw[RT][PT];
    auto request_residual = [&]() {
#pragma unroll
        for (int r = 0; r < RT; r++)
#pragma unroll
            for (int t = 0; t < PT; t++) {
                resw[r][t] = 0;
                if (res_img != nullptr) { // uniform
                    const bool live = col_ok && t < th_real && 16 * r + 4 * quad < p.out_c;
                    resw[r][t] = *reinterpret_cast<const int *>(
                        res_img + (size_t)(live ? off0 + (unsigned)(t * p.out_w * p.out_c + 16 * r) : 0u));
                }
            }
    };
    if constexpr (kEarlyResidual)
        request_residual();
    // Filters of a chunk are requested one chunk ahead (ChunkW), the project filters of a group of four
    // chunks at the start of the group: their latency hides behind the chunk in between.
    struct ChunkW {
        v4i aop[PACK];
        int wd0[3], wd1[3];
    };
    auto load_chunk = [&](int sub) {
        ChunkW w;
        const int ch0 = 16 * sub;
        if constexpr (PACK > 1) {
            // the filter's bytes in every tile slot; copy t keeps them in the groups of slot t only
            constexpr int kSubs = 4 / PACK;
            const v4i wq = load16_partial<VEC16>(p.w_expand, (unsigned)((ch0 + col) * c0 + 16 * (quad % kSubs)),
                                                 c0 - 16 * (quad % kSubs));
#pragma unroll
            for (int t = 0; t < PACK; t++)
                w.aop[t] = quad / kSubs == t ? wq : v4i{0, 0, 0, 0};
        } else if constexpr (ROWCONV) {
            w.aop[0] = *reinterpret_cast<const v4i *>(smem + a.off_aop + ((ch0 + col) * 4 + quad) * 16);
        } else {
            w.aop[0] = load16_partial<VEC16>(p.w_expand, (unsigned)((ch0 + col) * c0 + 16 * quad), c0 - 16 * quad);
        }
        if constexpr (ROWCONV) {
            // (these builds walk several short tiles per wavefront: the weights come from the workgroup's LDS copy
            // and a tile starts without a round trip to memory for them)
            const v4i *wl = reinterpret_cast<const v4i *>(smem + a.off_wd + (sub * 64 + lane) * 32);
            const v4i w0 = wl[0], w1 = wl[1];
            w.wd0[0] = w0[0], w.wd0[1] = w0[1], w.wd0[2] = w0[2];
            w.wd1[0] = w0[3], w.wd1[1] = w1[0], w.wd1[2] = w1[1];
            return w;
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
    v4i ap[RT];
    // (through a buffer descriptor: a piece that does not exist gets an offset past the descriptor's end and comes
    // back as zeros.  With a plain load and a select behind it the wait for the load stands at the select, right
    // behind the request, and every group of four chunks paid a round trip for its project filters.)
    const __amdgpu_buffer_rsrc_t wp_rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(p.w_project), (short)0, p.out_c * p.exp_c, 0x00020000);
    auto load_project = [&](int sub) {
        const int kc = (sub & ~3) * 16;
        const int nk = p.exp_c - kc - 16 * quad; // valid bytes of this lane's 16 k positions
#pragma unroll
        for (int r = 0; r < RT; r++) {
            const bool ok = r < n_rt && 16 * r + col < p.out_c && nk >= 16;
            const int off = ok ? (16 * r + col) * p.exp_c + kc + 16 * quad : (int)0x80000000u;
            const auto v = __builtin_amdgcn_raw_buffer_load_b128(wp_rsrc, off, 0, 0);
            ap[r] = v4i{(int)v[0], (int)v[1], (int)v[2], (int)v[3]};
        }
    };
    ChunkW cur;
    if constexpr (!ROWCONV)
        cur = load_chunk(0);

    if (ROWCONV && it == 0) {
        // operand A of the expand stage: filter row `q` of expanded channel f, zero-padded to 16 bytes
        const int wb = p.ek_w * c0;
        for (int i = (int)threadIdx.x; i < p.exp_c * 4; i += 64 * kWavesPerGroup) {
            const int f = i >> 2, q = i & 3;
            const bool row = q < p.ek_h;
            const unsigned src = (unsigned)((f * p.ek_h + (row ? q : 0)) * wb);
            int w[3] = {0, 0, 0};
#pragma unroll
            for (int j = 0; j < 9; j++) {
                const bool ok = row && j < wb;
                const int v = (int)(unsigned char)p.w_expand[(size_t)(src + (unsigned)(ok ? j : 0))];
                w[j >> 2] |= ok ? v << (8 * (j & 3)) : 0;
            }
            *reinterpret_cast<v4i *>(smem + a.off_aop + i * 16) = v4i{w[0], w[1], w[2], 0};
        }
        // the depthwise weights of lane l for chunk `sub`: filter rows min(quad, 2) (none for quad 3) and, at
        // stride 1, quad - 1 (none for quad 0) of channel 16 sub + col
        for (int i = (int)threadIdx.x; i < (p.exp_c >> 4) * 64; i += 64 * kWavesPerGroup) {
            const int l = i & 63, l_col = l & 15, l_quad = l >> 4;
            const unsigned wd = (unsigned)(16 * (i >> 6) + l_col);
            int w0[3], w1[3];
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                const int v0 = (int)p.w_dw[(size_t)(wd + (unsigned)((min(l_quad, 2) * 3 + kx) * p.exp_c))];
                w0[kx] = l_quad < 3 ? v0 : 0;
                w1[kx] = 0;
                if constexpr (S == 1) {
                    const int v1 = (int)p.w_dw[(size_t)(wd + (unsigned)((max(l_quad - 1, 0) * 3 + kx) * p.exp_c))];
                    w1[kx] = l_quad >= 1 ? v1 : 0;
                }
            }
            v4i *wl = reinterpret_cast<v4i *>(smem + a.off_wd + i * 32);
            wl[0] = v4i{w0[0], w0[1], w0[2], w1[0]};
            wl[1] = v4i{w1[1], w1[2], 0, 0};
        }
    }

    // the stage tables, by the whole group
    const unsigned bound_e = (unsigned)(ROWCONV ? p.ek_h * p.ek_w * c0 : c0) * 16384u, bound_d = 9u * 16384u;
    if (it == 0) { // uniform over the workgroup: every wavefront is in its first tile
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
        build_stage_tables(t, HE, (int)threadIdx.x, 64 * kWavesPerGroup, mode_e, mode_d, mode_p);
    } else {
        wave_lds_sync(); // the previous tile's reads of the wavefront's LDS areas come before this tile's writes
    }
    // tables (and, in ROWCONV builds, the expand operands) complete; no barrier after this one
    if constexpr (ROWCONV)
        cur = load_chunk(0);

    v4i accp[RT][PT];
#pragma unroll
    for (int r = 0; r < RT; r++)
#pragma unroll
        for (int t = 0; t < PT; t++)
            accp[r][t] = v4i{0, 0, 0, 0};

    // lower / upper clamp of a stage as two int16 in the fixed-point form of the short epilogue: ReLU and a Clip's
    // lower bound share the packed maximum, a Clip's upper bound is the packed minimum of the CLIP builds
    const int lo_e = max(p.relu_expand ? 0 : -128, (CLIP && p.clip_e) ? p.clip_e_lo : -128);
    const int lo_d = max(p.relu_dw ? 0 : -128, (CLIP && p.clip_d) ? p.clip_d_lo : -128);
    const int floor_e = ((lo_e << 8) & 0xffff) * 0x10001;
    const int floor_d = ((lo_d << 8) & 0xffff) * 0x10001;
    const int ceil_e = (CLIP && p.clip_e) ? (((p.clip_e_hi << 8) | 0xff) & 0xffff) * 0x10001 : 0x7fff7fff;
    const int ceil_d = (CLIP && p.clip_d) ? (((p.clip_d_hi << 8) | 0xff) & 0xffff) * 0x10001 : 0x7fff7fff;
    unsigned char *exp_dst = exp_l + col * 16 + 4 * quad;
    const unsigned char *exp_src = exp_l + (quad * a.pw + S * col) * 16;

    for (int sub = 0; sub < a.n_sub; sub++) {
        if ((sub & 3) == 0)
            load_project(sub);
        const ChunkW nxt = load_chunk(min(sub + 1, a.n_sub - 1));
        // ---- expand: 16 channels x every patch pixel
        {
            const StageConsts ce = read_stage_table(tab_e, p.exp_c, 16 * sub + 4 * quad, mode_e);
            if (!HE && ce.mode == 0) // a build meets the forms of its rounding mode only
                expand_chunk<0, NXPT, EXACT, 1, true, PACK, CLIP>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst, ceil_e);
            else if (!HE && ce.mode == 1)
                expand_chunk<1, NXPT, EXACT, 1, true, PACK, CLIP>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst, ceil_e);
            else if (HE && ce.mode == 6)
                expand_chunk<6, NXPT, EXACT, 1, true, PACK, CLIP>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst, ceil_e);
            else if (HE && ce.mode == 5)
                expand_chunk<5, NXPT, EXACT, 1, true, PACK, CLIP>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst, ceil_e);
            else
                expand_chunk<-1, NXPT, EXACT, 1, true, PACK, CLIP>(xb, n_xpt, xmask, cur.aop, ce, floor_e, p.relu_expand != 0, HE, exp_dst, ceil_e);
        }
        wave_lds_sync();
        if constexpr (kRowCopy)
            if (sub == 0 && it + 1 < tpw) { // uniform
                // The compiler counts the loads it knows and waits with vmcnt(n) for all but its n youngest; the
                // copy's loads, which it does not know, would be among the youngest, and such a wait would wait
                // for them.  So the loads requested so far (filters, long under way) are waited for first: the
                // compiler's counts then never reach below what is really outstanding.
                settle_rows();
                request_rows(it + 1);
            }

        // ---- depthwise: diagonal operands for patch rows quad (a0) and quad - 1 (a1)
        {
            v4i a0[3], a1[3];
#pragma unroll
            for (int kx = 0; kx < 3; kx++) {
                a0[kx] = diag_operand(cur.wd0[kx], col);
                a1[kx] = diag_operand(cur.wd1[kx], col);
            }
            const StageConsts cd = read_stage_table(tab_d, p.exp_c, 16 * sub + 4 * quad, mode_d);
            unsigned char *dst = dw_l + col * kDws + 16 * (sub & 3) + 4 * quad;
            if (!HE && cd.mode == 0) // a build meets the forms of its rounding mode only
                depthwise_chunk<0, PT, S, EXACT, true, CLIP>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, 16 * kDws, true, ceil_d);
            else if (!HE && cd.mode == 1)
                depthwise_chunk<1, PT, S, EXACT, true, CLIP>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, 16 * kDws, true, ceil_d);
            else if (HE && cd.mode == 6)
                depthwise_chunk<6, PT, S, EXACT, true, CLIP>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, 16 * kDws, true, ceil_d);
            else if (HE && cd.mode == 5)
                depthwise_chunk<5, PT, S, EXACT, true, CLIP>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, 16 * kDws, true, ceil_d);
            else
                depthwise_chunk<-1, PT, S, EXACT, true, CLIP>(exp_src, th, a.pw, a0, a1, cd, floor_d, p.relu_dw != 0, HE, dst, 16 * kDws, true, ceil_d);
        }
        wave_lds_sync();

        // ---- project: accumulate over the 64 (or last few) expanded channels gathered so far
        if ((sub & 3) == 3 || sub == a.n_sub - 1) {
            const unsigned char *bsrc = dw_l + col * kDws + 16 * quad;
#pragma unroll
            for (int t = 0; t < PT; t++) {
                if (EXACT || t < th) { // uniform
                    const v4i b = *reinterpret_cast<const v4i *>(bsrc + t * 16 * kDws);
#pragma unroll
                    for (int r = 0; r < RT; r++)
                        if (EXACT || r < n_rt) // uniform
                            accp[r][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ap[r], b, accp[r][t], 0, 0, 0);
                }
            }
            wave_lds_sync();
        }
        cur = nxt;
    }

    // ---- project epilogue, residual Add, stores
    if constexpr (kRowCopy)
        settle_rows(); // the next tile's rows, before this tile's first store
    if constexpr (!kEarlyResidual)
        request_residual(); // every residual word is requested before the first is used
    // The uniform choices (epilogue form, residual or not) are made once, outside the loops over the words, and
    // a row of a ragged last tile that does not exist is a store that no lane takes: the words of a tile are
    // one straight-line block.
    const int floor_p = p.relu_project ? 0 : (int)0x80008000u;
    const Requant4 res_q = make_requant4(p.residual_shift);
    auto words = [&](auto mode_tag, auto res_tag) {
        constexpr int MODE = decltype(mode_tag)::value;
        constexpr bool RES = decltype(res_tag)::value;
#pragma unroll
        for (int r = 0; r < RT; r++) {
            if (EXACT || r < n_rt) { // uniform
                const int c = 16 * r + 4 * quad;
                const StageConsts cp = read_stage_table<false>(tab_p, 16 * a.rt, c, mode_p);
                const bool live = col_ok && c < p.out_c;
#pragma unroll
                for (int t = 0; t < PT; t++) {
                    v4i acc = accp[r][t];
#pragma unroll
                    for (int k = 0; k < 4; k++)
                        acc[k] += cp.init[k];
                    int word;
                    if constexpr (RES) {
                        int res = resw[r][t];
                        if (p.residual_shift != 0) // uniform
                            res = requant4_s8(res, res_q);
                        if constexpr (MODE >= 0)
                            word = pack_fast4_add<MODE>(acc, cp.lsh, cp.rsh, floor_p, res);
                        else
                            word = sat_add4_s8(wave_pack<MODE>(acc, cp, floor_p, p.relu_project != 0, HE), res);
                    } else {
                        word = wave_pack<MODE>(acc, cp, floor_p, p.relu_project != 0, HE);
                    }
                    if (live && t < th_real)
                        *reinterpret_cast<int *>(out_img + (size_t)(off0 + (unsigned)(t * p.out_w * p.out_c + 16 * r))) = word;
                }
            }
        }
    };
    auto with_mode = [&](auto mode_tag) {
        if (res_img != nullptr)
            words(mode_tag, std::true_type{});
        else
            words(mode_tag, std::false_type{});
    };
    if (mode_p == -1)
        with_mode(std::integral_constant<int, -1>{});
    else if (HE && mode_p == 6)
        with_mode(std::integral_constant<int, 6>{});
    else if constexpr (HE)
        with_mode(std::integral_constant<int, 5>{});
    else if (mode_p == 0)
        with_mode(std::integral_constant<int, 0>{});
    else
        with_mode(std::integral_constant<int, 1>{});
    } // tiles of this wavefront
}

struct WavePlan {
    bool ok;
    WaveArgs a;
    size_t lds;
    int cus; // compute units of the device the launch goes to
};

constexpr int kPtMax = 8;
constexpr int kPlanCus = 256; // compute units the tile plan is balanced for

// LDS layout: the tables (shared by the wavefronts of a group), then per wavefront the expanded patch of one
// chunk (16 bytes per pixel; the depthwise reads run up to one row and a few pixels past the patch, into
// products with zero weights or into discarded columns) and the depthwise result of 64 channels.
void wave_layout(WaveArgs &a, size_t *lds)
{
    const int exp_px = std::max(((a.n_xpt + 3) & ~3) * 16, (a.ph * a.pw + 48 + 15) & ~15);
    a.off_tab = 0; // two stages x [init | rsh | lsh] x int32
    a.off_aop = a.p.exp_c * 24 + a.rt * 16 * 12 + kStageVoteBytes; // expand, depthwise and project tables, vote words
    a.off_wd = a.off_aop + (mbconv_expand_is_pointwise(a.p) ? 0 : a.p.exp_c * 64);
    a.off_exp = a.off_wd + (mbconv_expand_is_pointwise(a.p) ? 0 : a.p.exp_c * 128);
    a.off_dw = a.off_exp + exp_px * 16;
    a.wave_bytes = exp_px * 16 + a.th * 16 * kDws;
    a.rows_n = a.rows_ppr = a.rows_rounds = a.off_rows = 0;
    if (!mbconv_expand_is_pointwise(a.p)) {
        // a lane reads 16 bytes from byte (column * es_w * c0 + skew) of a copied row, skew < 16
        const int rows_n = (a.ph - 1) * a.p.es_h + a.p.ek_h;
        const int ppr = ((a.pw - 1) * a.p.es_w * a.p.in_c + 15 + 16 + 15) / 16;
        const int rounds = (rows_n * ppr + 63) / 64;
        const long long total = (long long)a.p.batch * a.p.img_h * a.p.img_w * a.p.in_c;
        if (rounds <= kRowRounds && total < (1ll << 30) &&
            (size_t)a.off_exp + (size_t)kWavesPerGroup * (a.wave_bytes + rounds * 1024) <= 80 * 1024) {
            a.rows_n = rows_n;
            a.rows_ppr = ppr;
            a.rows_rounds = rounds;
            a.off_rows = a.wave_bytes;
            a.wave_bytes += rounds * 1024; // whole rounds: lanes past the last piece write zeros
        }
    }
    a.fd_rows_ppr = make_fastdiv((unsigned)std::max(1, a.rows_ppr));
    *lds = (size_t)a.off_exp + (size_t)kWavesPerGroup * a.wave_bytes;
}

// Whether a guard-free build exists for a plan (tile geometry, row tiles, alignment, rounding mode of a.p).
bool wave_plan_has_exact_build(const WaveArgs &a);

WavePlan wave_plan(const MbconvParams &p)
{
    WavePlan plan;
    plan.ok = false;
    if (p.w_expand == nullptr || p.k_h != 3 || p.k_w != 3 || p.dil_h != 1 || p.dil_w != 1 || p.stride_h != p.stride_w ||
        (p.stride_h != 1 && p.stride_h != 2))
        return plan;
    const bool rowconv = !mbconv_expand_is_pointwise(p);
    if (rowconv) {
        // filter rows of at most 9 bytes cut out of three aligned dwords, one 16-lane group per row
        if (p.ek_h < 1 || p.ek_h > 4 || p.ek_w < 1 || p.ek_w * p.in_c > 9 || p.es_h < 1 || p.es_w < 1 ||
            (long long)p.img_h * p.img_w * p.in_c >= (1ll << 30) || (reinterpret_cast<uintptr_t>(p.in) & 3) != 0)
            return plan;
    } else if (p.in_c % 4 != 0 || p.in_c > 64) {
        return plan;
    }
    if (p.exp_c % 16 != 0 || p.out_c % 4 != 0 || p.out_c > 64)
        return plan;
    if ((long long)p.in_h * p.in_w * p.in_c >= (1ll << 30) || (long long)p.out_h * p.out_w * p.out_c >= (1ll << 30) ||
        p.exp_c >= 65536)
        return plan;
    const int s = p.stride_h;
    WaveArgs a = {};
    a.p = p;
    // columns: the fewest column tiles and the narrowest tile that gives them (less halo to expand), or tiles of
    // 14 columns, the width every guard-free build is made for (patches of 16 columns at depthwise stride 1,
    // where the patch column of a lane does not change from pixel tile to pixel tile, and of 29 at stride 2).
    // A plan rounded up to that width computes columns that do not exist (their loads are masked, their stores
    // dropped) and still takes a third of the time of a guarded build.
    // rows: cheapest total of expand tiles (x 1.5: MFMA + the longer epilogue) and depthwise MFMAs.  A launch
    // that does not fill the device once (two resident workgroups per compute unit) takes one tile's time
    // whatever its tile count, so there a lower tile that brings more workgroups wins.  Heights whose plan has a
    // guard-free build come first: the guarded builds take about three times as long per tile, and a caller
    // that fuses by espdl_hip_mbconv_s8_preferred gets the same answer at every batch size.
    const int nxpt_limit = 17;
    const double slots = 2.0 * kPlanCus;
    a.n_sub = p.exp_c / 16;
    a.rt = (p.out_c + 15) / 16;
    a.x_vec16 = (p.in_c % 16 == 0 && (reinterpret_cast<uintptr_t>(p.in) & 15) == 0) ? 1 : 0;
    a.we_vec16 = (p.in_c % 16 == 0 && (reinterpret_cast<uintptr_t>(p.w_expand) & 15) == 0) ? 1 : 0;
    double best = 1e30;
    int best_th = 0, best_tw = 0;
    bool best_exact = false;
    const int n_cols16 = (p.out_w + 15) / 16;
    const int tw_narrow = (rowconv && s == 1 && p.out_w > 14) ? 14 : (p.out_w + n_cols16 - 1) / n_cols16;
    const int tw_candidates[2] = {tw_narrow, 14};
    for (int ci = 0; ci < (tw_narrow == 14 ? 1 : 2); ci++) {
        a.tw = tw_candidates[ci];
        a.pw = (a.tw - 1) * s + 3;
        a.tiles_x = (p.out_w + a.tw - 1) / a.tw;
        for (int th = 1; th <= kPtMax; th++) {
            a.th = th;
            a.ph = (th - 1) * s + 3;
            a.n_xpt = (a.ph * a.pw + 15) / 16;
            if (a.n_xpt > nxpt_limit)
                break;
            a.tiles_y = (p.out_h + th - 1) / th;
            size_t lds_unused;
            wave_layout(a, &lds_unused); // (the guard-free build of a windowed expand stage asks for its row copy)
            const bool exact = wave_plan_has_exact_build(a);
            const double tile_cost = 1.5 * a.n_xpt + 3.0 * th + 2.0;
            const double groups = std::ceil((double)std::max(1, p.batch) * a.tiles_y * a.tiles_x / kWavesPerGroup);
            const double rounds = groups / slots;
            const double cost = tile_cost * std::max(1.0, rounds);
            if ((exact && !best_exact) || (exact == best_exact && cost < best)) {
                best = cost;
                best_th = th;
                best_tw = a.tw;
                best_exact = exact;
            }
        }
    }
    if (best_th == 0)
        return plan;
    a.tw = best_tw;
    a.pw = (a.tw - 1) * s + 3;
    a.tiles_x = (p.out_w + a.tw - 1) / a.tw;
    a.th = best_th;
    a.ph = (a.th - 1) * s + 3;
    a.n_xpt = (a.ph * a.pw + 15) / 16;
    a.tiles_y = (p.out_h + a.th - 1) / a.th;
    wave_layout(a, &plan.lds);
    if (plan.lds > (a.rows_n > 0 ? 80 : 64) * 1024)
        return plan;
    a.fd_pw = make_fastdiv((unsigned)a.pw);
    a.fd_tiles_x = make_fastdiv((unsigned)a.tiles_x);
    a.fd_tiles_yx = make_fastdiv((unsigned)(a.tiles_y * a.tiles_x));
    plan.a = a;
    plan.ok = true;
    return plan;
}

template <int NXPT, int RT, int PT, int S, bool HE, bool VEC16, bool EXACT, bool ROWCONV = false, int PACK = 1, bool CLIP = false>
hipError_t launch_one(const WavePlan &plan, hipStream_t stream)
{
    WaveArgs a = plan.a;
    auto kernel = mbconv_s8_wave_kernel<NXPT, RT, PT, S, HE, VEC16, EXACT, ROWCONV, PACK, CLIP>;
    if (plan.lds > 64 * 1024) {
        // the dynamic LDS limit of a kernel is raised once per device (bit d: done on device d; setting it twice
        // from two threads does no harm)
        static std::atomic<unsigned long long> raised{0};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess)
            return e;
        const unsigned long long bit = 1ull << (dev & 63);
        if (dev >= 64 || !(raised.load(std::memory_order_relaxed) & bit)) {
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                    80 * 1024);
            if (e != hipSuccess)
                return e;
            if (dev < 64)
                raised.fetch_or(bit, std::memory_order_relaxed);
        }
    }
    a.tpw = 1;
    if (ROWCONV) {
        // Tiles per wavefront: these tiles are short (two chunks of expanded channels for a 32-filter stem), so
        // a workgroup's set-up weighs on them.  Up to 16 rounds over the device the launch becomes one round of
        // resident workgroups that walk ceil(tiles / resident wavefronts) tiles each (measured on MobileNetV2's
        // stem at batch 256: 14 tiles per wavefront 0.742 ms per step, 7: 0.746, 10: 0.765, 1: 0.777); beyond
        // that the rounds balance themselves and eight tiles per wavefront amortize the set-up.
        const long long resident = (long long)plan.cus * resident_workgroups_per_cu(kernel, 64 * kWavesPerGroup, plan.lds) *
            kWavesPerGroup;
        const long long per_wave = (a.n_tiles + resident - 1) / resident;
        a.tpw = per_wave <= 16 ? (int)std::max<long long>(1, per_wave) : 8;
    }
    const int per_group = kWavesPerGroup * a.tpw;
    const unsigned groups = (unsigned)((a.n_tiles + per_group - 1) / per_group);
    hipLaunchKernelGGL(kernel, dim3(groups), dim3(64 * kWavesPerGroup), plan.lds, stream, a);
    return hipGetLastError();
}

// Guarded builds that take any plan within (17 pixel tiles, 4 row tiles, 8 rows).
template <int S, bool HE>
hipError_t launch_generic(const WavePlan &plan, hipStream_t stream)
{
    return (plan.a.x_vec16 && plan.a.we_vec16) ? launch_one<17, 4, kPtMax, S, HE, true, false>(plan, stream)
                                               : launch_one<17, 4, kPtMax, S, HE, false, false>(plan, stream);
}

// The guard-free builds: one per tile plan of MobileNetV2-style blocks, in both rounding modes.  Returns
// false when the plan has none; with `dry` nothing is launched (the question is only whether one exists).
template <bool HE>
bool launch_exact(const WavePlan &plan, hipStream_t stream, bool dry, hipError_t *err)
{
    const WaveArgs &a = plan.a;
    const bool vec16 = a.x_vec16 && a.we_vec16;
    const int s = a.p.stride_h;
    // a Clip between the stages: the half-up builds exist with the clamp compiled in, nothing else takes it
    const bool clip = mbconv_has_clip(a.p);
    if (clip && HE)
        return false;
#define ESPDL_WAVE_EXACT(NXPT, RT, PT, S, V, ROWCONV)                                                 \
    do {                                                                                               \
        if constexpr (!HE) {                                                                           \
            if (clip) {                                                                                \
                if (!dry)                                                                              \
                    *err = launch_one<NXPT, RT, PT, S, false, V, true, ROWCONV, 1, true>(plan, stream); \
                return true;                                                                           \
            }                                                                                          \
        }                                                                                              \
        if (!dry)                                                                                      \
            *err = launch_one<NXPT, RT, PT, S, HE, V, true, ROWCONV>(plan, stream);                    \
        return true;                                                                                   \
    } while (0)
    if (!mbconv_expand_is_pointwise(a.p)) {
        // expand stage with a window: the stem + first block of MobileNetV2 at 224 x 224
        if (a.n_xpt == 10 && a.pw == 16 && a.rt == 1 && a.th == 8 && s == 1 && a.rows_n > 0)
            ESPDL_WAVE_EXACT(10, 1, 8, 1, false, true);
        return false;
    }
    const auto is = [&](int nxpt, int rt, int th, int stride, bool v) {
        return a.n_xpt == nxpt && a.rt == rt && a.th == th && s == stride && vec16 == v && (stride != 1 || a.pw == 16);
    };
    // block inputs of at most 16 / 32 channels: four / two pixel tiles per operand-B register set
#define ESPDL_WAVE_PACKED(NXPT, RT, PT, S, V, PACK)                                                       \
    do {                                                                                                   \
        if constexpr (!HE) {                                                                               \
            if (clip) {                                                                                    \
                if (!dry)                                                                                  \
                    *err = launch_one<NXPT, RT, PT, S, false, V, true, false, PACK, true>(plan, stream);   \
                return true;                                                                               \
            }                                                                                              \
        }                                                                                                  \
        if (!dry)                                                                                          \
            *err = launch_one<NXPT, RT, PT, S, HE, V, true, false, PACK>(plan, stream);                    \
        return true;                                                                                       \
    } while (0)
    const int c0 = a.p.in_c;
    if (is(17, 2, 4, 2, true) && c0 == 16)
        ESPDL_WAVE_PACKED(17, 2, 4, 2, true, 4);
    if (is(17, 2, 4, 2, false) && c0 <= 32)
        ESPDL_WAVE_PACKED(17, 2, 4, 2, false, 2);
    if (is(10, 2, 8, 1, false) && c0 <= 32)
        ESPDL_WAVE_PACKED(10, 2, 8, 1, false, 2);
    if (is(9, 2, 7, 1, true) && c0 == 32)
        ESPDL_WAVE_PACKED(9, 2, 7, 1, true, 2);
    if (is(10, 4, 2, 2, true) && c0 == 32)
        ESPDL_WAVE_PACKED(10, 4, 2, 2, true, 2);
#undef ESPDL_WAVE_PACKED
    if (is(17, 2, 4, 2, true))
        ESPDL_WAVE_EXACT(17, 2, 4, 2, true, false);
    if (is(17, 2, 4, 2, false))
        ESPDL_WAVE_EXACT(17, 2, 4, 2, false, false);
    if (is(10, 2, 8, 1, false))
        ESPDL_WAVE_EXACT(10, 2, 8, 1, false, false);
    if (is(10, 2, 8, 1, true))
        ESPDL_WAVE_EXACT(10, 2, 8, 1, true, false);
    if (is(9, 2, 7, 1, true))
        ESPDL_WAVE_EXACT(9, 2, 7, 1, true, false);
    if (is(10, 4, 2, 2, true))
        ESPDL_WAVE_EXACT(10, 4, 2, 2, true, false);
#undef ESPDL_WAVE_EXACT
    return false;
}

bool wave_plan_has_exact_build(const WaveArgs &a)
{
    WavePlan plan;
    plan.ok = true;
    plan.a = a;
    plan.lds = 0;
    plan.cus = kPlanCus;
    hipError_t err = hipSuccess;
    return a.p.half_even ? launch_exact<true>(plan, nullptr, true, &err) : launch_exact<false>(plan, nullptr, true, &err);
}

hipError_t launch_planned(WavePlan &plan, hipStream_t stream)
{
    WaveArgs &a = plan.a;
    const int s = a.p.stride_h;
    hipError_t err = hipSuccess;
    if (a.p.half_even ? launch_exact<true>(plan, stream, false, &err) : launch_exact<false>(plan, stream, false, &err))
        return err;
    if (mbconv_has_clip(a.p))
        return hipErrorInvalidValue; // the guarded builds have no clamp
    // guarded builds
    if (!mbconv_expand_is_pointwise(a.p)) {
        if (a.p.half_even)
            return s == 1 ? launch_one<17, 4, kPtMax, 1, true, false, false, true>(plan, stream)
                          : launch_one<17, 4, kPtMax, 2, true, false, false, true>(plan, stream);
        return s == 1 ? launch_one<17, 4, kPtMax, 1, false, false, false, true>(plan, stream)
                      : launch_one<17, 4, kPtMax, 2, false, false, false, true>(plan, stream);
    }
    if (!a.p.half_even)
        return s == 1 ? launch_generic<1, false>(plan, stream) : launch_generic<2, false>(plan, stream);
    return s == 1 ? launch_generic<1, true>(plan, stream) : launch_generic<2, true>(plan, stream);
}

} // namespace

bool mbconv_s8_wave_supports(const MbconvParams &p)
{
    return wave_plan(p).ok;
}

bool mbconv_s8_wave_has_fast_build(const MbconvParams &p)
{
    const WavePlan plan = wave_plan(p);
    return plan.ok && wave_plan_has_exact_build(plan.a);
}

hipError_t launch_mbconv_s8_wave(const MbconvParams &p, int cu_count, hipStream_t stream)
{
    if ((long long)p.batch * p.out_h * p.out_w == 0)
        return hipSuccess;
    WavePlan plan = wave_plan(p);
    if (!plan.ok)
        return hipErrorInvalidValue;
    const long long tiles = (long long)p.batch * plan.a.tiles_y * plan.a.tiles_x;
    if (tiles > 0x7fffffff)
        return hipErrorInvalidValue;
    plan.a.n_tiles = (int)tiles;
    plan.cus = cu_count > 0 ? cu_count : kPlanCus;
    static const bool trace = getenv("ESPDL_HIP_TRACE") != nullptr;
    if (trace)
        fprintf(stderr, "mbconv_s8_wave: %dx%d in %d exp %d out %d s%d tile %dx%d patch %dx%d n_xpt %d rt %d lds %zu tiles %lld\n",
                p.in_h, p.in_w, p.in_c, p.exp_c, p.out_c, p.stride_h, plan.a.th, plan.a.tw, plan.a.ph, plan.a.pw,
                plan.a.n_xpt, plan.a.rt, plan.lds, tiles);
    return launch_planned(plan, stream);
}

} // namespace espdl
