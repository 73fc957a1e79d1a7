// Dense int8 convolution with a window (3x3, 5x5, dilated ...) at stride 1 for gfx950: implicit GEMM on
// v_mfma_i32_16x16x64_i8 with the NHWC input tile AND the filters staged in LDS.
//
// It computes what conv2d_33cn / conv2d_hwcn compute (esp-dl/dl/base/dl_base_conv2d.cpp:35-163) for every
// output pixel conv_operation_shell visits (esp-dl/dl/base/dl_base.hpp:940-1191: taps outside the image are
// skipped, i.e. they contribute zero), followed by the n_wise epilogue
// (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210).  Integer sums do not depend on
// their order, so the result is bit-identical.
//
// Why a second kernel next to conv2d_s8_mfma_kernel.h: that one reads operand B (the pixels) straight from
// global memory, once per filter tap, so a 3x3 convolution fetches every input byte nine times from L2 and
// pays address arithmetic per tap and pixel.  Here a workgroup owns a th x tw tile of ONE image's output:
//   * the (th + (k-1)*d) x (tw + (k-1)*d) input patch with all channels is copied to LDS once, with
//     16-byte loads of consecutive addresses and zeros for positions outside the image; the copy of the
//     NEXT tile's patch is in flight in registers while the current tile is computed;
//   * the filters of the workgroup's chunk (up to all of them) sit in LDS in MFMA operand-A order for the
//     whole life of the persistent workgroup;
//   * a wavefront takes sets of PT pixel tiles (16 pixels each) and, per group of 64 filters, walks the
//     reduction axis (tap, channel) in steps of 64: PT + 4 operand reads of 16 bytes per lane from LDS feed
//     4 * PT matrix instructions, the operands of the next step being read while the current products run.
// LDS layout of the patch: [row][column][channels + pad], the pixel pitch twice an odd number of 16-byte units
// (the pitch at which 16-byte-per-lane reads of 16 neighbouring pixels meet no bank twice).  The kernel is for
// stride 1 (strided layers re-read little and measured as fast or faster through the direct kernel, so the
// planner refuses them): the "pixels" of a tile are 16 consecutive positions of the patch's flattened
// (row, column) space, a tap is then a constant offset, tiles run across row ends, and only the (k-1)*d positions
// per row that wrap are wasted instead of the padding of every row to a multiple of 16.
// The offset of reduction step ks for lane group q (tap and first channel of k = 64 ks + 16 q) comes from a
// small LDS table, so any channel count that is a multiple of 16 works, also when a step of 64 spans taps.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

constexpr int kLdsLimit = 156 * 1024;    // LDS a compute unit gives its workgroups (of 160 KB)
constexpr int kPlanCus = 256;

struct TiledArgs {
    const int8_t *in;
    const int8_t *w;
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
    const int8_t *res;
    int8_t *out;
    ConvGeom g;
    int K, ksteps;
    int n_groups, groups_per_chunk;
    int th, tw;          // output tile
    int ph, pw;          // patch rows and columns
    int cs;              // LDS bytes per patch pixel
    int cu16;            // in_c / 16
    int n_ptiles, n_sets;
    int tiles_x, tiles_y, n_tiles;
    int row_units;       // pw * cu16: 16-byte pieces of one patch row
    int row_par;         // patch rows the workgroup's threads copy at a time (threads / row_units)
    int row_groups;      // pieces per thread: patch rows / row_par, rounded up (the LDS patch holds that many rows)
    int src_row_step;    // bytes between the input rows of a thread's consecutive pieces (row_par rows)
    int lds_row_step;    // the same in the LDS patch
    int img_bytes;       // bytes of one image of the input tensor
    int off_tabs, off_koff, off_lut, off_pix, off_patch; // LDS offsets (filters at 0)
    int out_vec;
    int epi;             // epilogue form: 0 plain 16-byte stores, 1 the same with table / residual, 2 general
    int koff_pitch;      // ints per lane-group row of the step-offset table
    FastDiv fd_cu16, fd_pw, fd_tiles_x, fd_tiles_yx, fd_row_units;
};

__device__ __forceinline__ int group_tiles(int out_c, int gbase)
{
    const int rem = out_c - gbase;
    return rem >= 64 ? 4 : (rem + 15) >> 4;
}

struct TileRef {
    long long img_out, img_res; // byte offsets of the tile's image in the output and residual tensors
    int oy0, ox0, th_real, tw_real;
};

// Image and tile position of a tile index.
struct TilePos {
    int n, ty, tx;
};

__device__ __forceinline__ TilePos locate_tile(int tile, const FastDiv &fd_yx, const FastDiv &fd_x)
{
    TilePos t;
    t.n = (int)fastdiv((unsigned)tile, fd_yx);
    const int rem = tile - t.n * (int)fd_yx.d;
    t.ty = (int)fastdiv((unsigned)rem, fd_x);
    t.tx = rem - t.ty * (int)fd_x.d;
    return t;
}

typedef unsigned int v4u __attribute__((ext_vector_type(4)));

// Wait for the wavefront's outstanding vector-memory instructions, as an instruction of its own.
__device__ __forceinline__ void settle()
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

struct Ctx {
    const v4i *wts;
    const int *init_l, *shift_l, *lsh_l, *koff_l;
    const int8_t *lut_l;
    const unsigned char *patch;
    const v4i *pix_l; // per position of the flattened patch a set can cover: {patch offset, row, column, row * out_w + column}
    int lane, col, quad;
    bool relu, has_lut;
    int floor_pk;
};

// One set of PT pixel tiles x one group of NT filter tiles: the products over the whole reduction axis, then
// the epilogue and the stores.  MODE: pack_fast4 mode, or -1 for the general shift_and_round form.
// EPI: 0 - 64 filters, 16-byte stores, no table, no residual: nothing but the requantization between the last
// product and the store; 1 - 64 filters, 16-byte stores, table and / or residual; 2 - anything else.
template <int PT, int NT, int MODE, bool HE, int EPI>
__device__ __forceinline__ void run_set(const TiledArgs &a, const Ctx &c, int8_t *out_img, const int8_t *res_img,
                                        const int (&pixoff)[PT], const int (&opix)[PT], unsigned okmask, int gi, int gbase)
{
    const int OC = a.g.out_c;
    const int c_local = gi * 64 + 4 * NT * c.quad;
    const int ksteps = a.ksteps;
    v4i acc[PT][NT];
    v4i start[NT]; // bias + rounding constant: the C operand of the first reduction step
#pragma unroll
    for (int t = 0; t < NT; t++)
        start[t] = *reinterpret_cast<const v4i *>(c.init_l + c_local + 4 * t);
    const v4i *wbase = c.wts + (size_t)gi * ksteps * 256 + c.lane;
    v4i A[2][NT], B[2][PT];
    auto load = [&](int buf, int ks, int ko) {
#pragma unroll
        for (int p = 0; p < PT; p++)
            B[buf][p] = *reinterpret_cast<const v4i *>(c.patch + pixoff[p] + ko);
#pragma unroll
        for (int t = 0; t < NT; t++)
            A[buf][t] = wbase[(ks * 4 + t) * 64];
    };
    auto products = [&](int buf) {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int p = 0; p < PT; p++)
                acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[buf][t], B[buf][p], acc[p][t], 0, 0, 0);
    };
    // Offsets of the reduction steps come from the lane group's row of the table, two steps per read, one loop
    // iteration ahead of their use; operands are read one step ahead.  Every LDS read of the loop is
    // unconditional (entries past the last step repeat it), so the in-order wait counters stay exact and a
    // product waits for its own operands only.
    const int *kq = c.koff_l + c.quad * a.koff_pitch; // kq[0]: step 0; kq[2 + j]: step min(j + 1, last)
    const int last = ksteps - 1;
    auto first_products = [&]() {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int p = 0; p < PT; p++)
                acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[0][t], B[0][p], start[t], 0, 0, 0);
    };
    // The products run at a raised wavefront priority: the other wavefront of the SIMD is in another phase of its
    // tile most of the time, and its vector instructions then fill the issue slots between the matrix
    // instructions instead of alternating with them (56 x 56 x 64 -> 64 at batch 256: 41.6 -> 40.5 us).
    __builtin_amdgcn_s_setprio(3);
    v2i pair = *reinterpret_cast<const v2i *>(kq + 2);
    load(0, 0, kq[0]);
    if (ksteps == 1) {
        first_products();
    } else {
        v2i next_pair = *reinterpret_cast<const v2i *>(kq + 4);
        load(1, 1, pair[0]);
        first_products();
        load(0, min(2, last), pair[1]);
        products(1);
        pair = next_pair;
        int ks = 2;
        for (; ks + 1 < ksteps; ks += 2) {
            next_pair = *reinterpret_cast<const v2i *>(kq + 4 + ks);
            load(1, ks + 1, pair[0]);
            products(0);
            load(0, min(ks + 2, last), pair[1]);
            products(1);
            pair = next_pair;
        }
        if (ks < ksteps)
            products(0);
    }
    __builtin_amdgcn_s_setprio(0);
    settle(); // the pieces of the next patch, before the first store after their request
    // epilogue: this lane owns output channels [c_lane, c_lane + 4 * NT) of pixel p * 16 + col of the set
    const int c_lane = gbase + 4 * NT * c.quad;
    v4i ss[NT], ls[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        ss[t] = *reinterpret_cast<const v4i *>(c.shift_l + c_local + 4 * t);
        ls[t] = (MODE == 1 || MODE == 5) ? *reinterpret_cast<const v4i *>(c.lsh_l + c_local + 4 * t) : v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int p = 0; p < PT; p++) {
        int words[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            if constexpr (MODE >= 0) {
                words[t] = pack_fast4<MODE>(acc[p][t], ls[t], ss[t], c.floor_pk);
            } else {
                int q[4];
#pragma unroll
                for (int r = 0; r < 4; r++)
                    q[r] = requant_s8(acc[p][t][r], ss[t][r], c.relu, HE);
                words[t] = pack4_s8(q[0], q[1], q[2], q[3]);
            }
        }
        // pixel index inside the image times the channel pitch of the output (and of the residual operand, which
        // may be a channel slice of another tensor): below 2^31
        const unsigned go = (unsigned)(opix[p] * a.g.out_pitch + c_lane);
        const unsigned ro = (unsigned)(opix[p] * a.g.res_pitch + c_lane);
        const bool ok = (okmask >> p) & 1u;
        if constexpr (EPI == 0) {
            if (ok)
                *reinterpret_cast<v4i *>(out_img + (size_t)go) = v4i{words[0], words[NT > 1 ? 1 : 0], words[NT > 2 ? 2 : 0], words[NT > 3 ? 3 : 0]};
            continue;
        }
        if (c.has_lut) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int v = words[t];
                words[t] = pack4_s8(c.lut_l[(int)(int8_t)v + 128], c.lut_l[(int)(int8_t)(v >> 8) + 128],
                                    c.lut_l[(int)(int8_t)(v >> 16) + 128], c.lut_l[(v >> 24) + 128]);
            }
        }
        if (!ok)
            continue;
        int8_t *dst = out_img + (size_t)go;
        // the widest piece that exists, at any byte address: 16 bytes, else 4 per filter tile, bytes for a row's tail
        if (EPI == 1 || (NT == 4 && c_lane + 16 <= OC)) {
            v4i v = {words[0], words[NT > 1 ? 1 : 0], words[NT > 2 ? 2 : 0], words[NT > 3 ? 3 : 0]};
            if (res_img != nullptr) {
                const v4i r = *reinterpret_cast<const v4i_unaligned *>(res_img + (size_t)ro);
#pragma unroll
                for (int d = 0; d < 4; d++)
                    v[d] = sat_add4_s8(v[d], r[d]);
            }
            *reinterpret_cast<v4i_unaligned *>(dst) = v;
        } else if (NT == 2 && c_lane + 8 <= OC) {
            // two filter tiles: the lane's eight channels as one piece (half the store instructions of a layer with
            // 32 filters, which the memory pipeline serves lane by lane either way)
            v2i v = {words[0], words[NT > 1 ? 1 : 0]};
            if (res_img != nullptr) {
                const v2i r = *reinterpret_cast<const v2i_unaligned *>(res_img + (size_t)ro);
                v[0] = sat_add4_s8(v[0], r[0]);
                v[1] = sat_add4_s8(v[1], r[1]);
            }
            *reinterpret_cast<v2i_unaligned *>(dst) = v;
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if (c_lane + 4 * t + 4 <= OC) {
                    int v = words[t];
                    if (res_img != nullptr)
                        v = sat_add4_s8(v, *reinterpret_cast<const int_unaligned *>(res_img + (size_t)ro + 4 * t));
                    *reinterpret_cast<int_unaligned *>(dst + 4 * t) = v;
                } else {
                    for (int r = 0; r < 4; r++)
                        if (c_lane + 4 * t + r < OC) {
                            int v = (int)(int8_t)(words[t] >> (8 * r));
                            if (res_img != nullptr)
                                v = clamp_s8(v + (int)res_img[(size_t)ro + 4 * t + r]);
                            dst[4 * t + r] = (int8_t)v;
                        }
                }
            }
        }
    }
}

// All sets of a wavefront that has at least one (wave < n_sets) for one tile, with one epilogue form compiled in.
template <int PT, int MODE, bool HE, int EPI>
__device__ __forceinline__ void run_tile(const TiledArgs &a, const Ctx &c, const TileRef &tr, int wave, int n_waves,
                                         int g_first, int g_count)
{
    const ConvGeom &g = a.g;
    const int OC = g.out_c;
    int8_t *out_img = a.out + tr.img_out;
    const int8_t *res_img = a.res != nullptr ? a.res + tr.img_res : nullptr;
    const int org_out = tr.oy0 * g.out_w + tr.ox0; // in pixels
    int set = wave;
    do {
        // the pixels of a set: 16 consecutive positions of the flattened patch per pixel tile, from the table
        int pixoff[PT];
        int opix[PT];
        unsigned okmask = 0;
        const v4i *pix = c.pix_l + set * (PT * 16) + c.col;
#pragma unroll
        for (int p = 0; p < PT; p++) {
            const v4i e = pix[p * 16];
            pixoff[p] = e[0];
            const bool ok = e[1] < tr.th_real && e[2] < tr.tw_real; // (positions past the tile hold row 0x7fff)
            okmask |= ok ? 1u << p : 0u;
            opix[p] = org_out + e[3];
        }
        int gi = 0;
        do {
            const int gbase = (g_first + gi) * 64;
            if constexpr (EPI != 2) {
                run_set<PT, 4, MODE, HE, EPI>(a, c, out_img, res_img, pixoff, opix, okmask, gi, gbase);
            } else {
                switch (group_tiles(OC, gbase)) { // uniform
                case 4:
                    run_set<PT, 4, MODE, HE, 2>(a, c, out_img, res_img, pixoff, opix, okmask, gi, gbase);
                    break;
                case 3:
                    run_set<PT, 3, MODE, HE, 2>(a, c, out_img, res_img, pixoff, opix, okmask, gi, gbase);
                    break;
                case 2:
                    run_set<PT, 2, MODE, HE, 2>(a, c, out_img, res_img, pixoff, opix, okmask, gi, gbase);
                    break;
                default:
                    run_set<PT, 1, MODE, HE, 2>(a, c, out_img, res_img, pixoff, opix, okmask, gi, gbase);
                    break;
                }
            }
        } while (++gi < g_count); // g_count >= 1
        set += n_waves;
    } while (set < a.n_sets);
}

// A value in a scalar register of its own.  Kernel arguments arrive in groups of eight or sixteen registers, and
// a group that does not stay resident over the tile loop is fetched back whole for every use of one member.
template <typename T>
__device__ __forceinline__ T lone(T v)
{
    asm volatile("" : "+s"(v));
    return v;
}

// Copying a patch: a thread owns ONE 16-byte column piece (patch column px, channels 16 cu ...) and walks the
// patch rows r0, r0 + row_par, ...: row_groups pieces, the same count for every thread (the LDS patch is that
// many rows tall; rows past the patch are never read).  Everything about the column is computed once per kernel.
// The loads go through a buffer descriptor of the tile's image: a piece outside the image gets an offset past
// the descriptor's end and comes back as zeros (the reference's window clipping), so there is one form for inner
// and border tiles and nothing to patch up when the pieces are written to LDS.  The pieces of the NEXT tile are
// requested before the current tile is computed and written to LDS after it.
//
// The loads and the wait for them are written as instructions.  The pieces are used after the tile's stores; a
// wavefront's loads and stores share one counter, and the compiler, for which the two kinds may complete in
// any order, waits for that counter to reach zero where the pieces are written to LDS - for the stores just
// issued as well - or, when the set loop reuses a piece register, in front of that loop, right after the
// request (measured on 56 x 56 x 64 -> 64 at batch 256: 48.8 and 46.9 us per launch; this form 43.3 us).
// settle() waits before the first store that follows a request instead - by then the loads have had the
// products of a set to arrive - and nothing waits where the pieces are used.  What the compiler does not
// know any more has to hold by construction:
//   * between a request and settle() nothing may read or move a piece.  The compiler sees the pieces as
//     values defined by request() and used by deposit(), keeps them in their registers over the tile and has no
//     reason to touch them; the build checks in the generated code that it did not, and that the kernels have
//     no register spills (build.py: check_hand_waited_loads);
//   * the descriptor may have been moved into its scalar registers by vector instructions right before a load,
//     and a memory instruction may read such a register five wait states later at the earliest: the
//     compiler pads its own instructions, not the text of an asm statement, hence the s_nop.
template <int UMAX>
struct Stager {
    int r0, px;       // first patch row and patch column of the thread's pieces
    bool active;      // the thread has pieces
    int src0, dst0;   // byte offset of piece 0 from the patch origin in the image / in the LDS patch
    v4u pre[UMAX];

    __device__ __forceinline__ void init(const TiledArgs &a, int tid)
    {
        const ConvGeom &g = a.g;
        r0 = (int)fastdiv((unsigned)tid, a.fd_row_units);
        const int ru = tid - r0 * a.row_units;
        active = r0 < a.row_par;
        px = (int)fastdiv((unsigned)ru, a.fd_cu16);
        const int cu = ru - px * a.cu16;
        src0 = (r0 * g.in_w + px) * g.in_pitch + 16 * cu;
        dst0 = (r0 * a.pw + px) * a.cs + 16 * cu;
    }
    // Pieces of the patch whose first pixel is (iy0, ix0) of the image at `img`.  When all patch rows lie inside the
    // image, the row of a piece goes into the instruction's scalar offset and the pieces share one vector offset;
    // else a piece's offset is computed and tested per thread.  Offsets handed to the hardware are never negative
    // (a negative vector offset would not wrap against the scalar one: the unit adds them to a 48-bit base).
    // One asm statement per piece serves both forms, so that a piece has one register whatever the form.
    __device__ __forceinline__ void request(const int8_t *img, int img_bytes, int iy0, int ix0, int in_h, int in_w,
                                            int in_pitch, int row_groups, int row_par, int src_row_step)
    {
        // buffer descriptor: base, stride 0, bytes, 32-bit raw format
        const __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t *>(img), (short)0, img_bytes, 0x00020000);
        constexpr int kParked = (int)0x80000000u; // past the end of any image: the load returns zeros
        const int org = (iy0 * in_w + ix0) * in_pitch;
        const bool xok = active && (unsigned)(ix0 + px) < (unsigned)in_w;
        int off[UMAX];
        int sstep;
        if (iy0 >= 0 && iy0 + row_groups * row_par <= in_h) { // uniform
            const int voff = xok ? org + src0 : kParked;
#pragma unroll
            for (int j = 0; j < UMAX; j++)
                off[j] = voff;
            sstep = src_row_step;
        } else {
            const int row = iy0 + r0;
#pragma unroll
            for (int j = 0; j < UMAX; j++) {
                const bool ok = xok && (unsigned)(row + j * row_par) < (unsigned)in_h;
                off[j] = ok ? org + src0 + j * src_row_step : kParked;
            }
            sstep = 0;
        }
#pragma unroll
        for (int j = 0; j < UMAX; j++)
            if (j < row_groups) // uniform
                asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2, %3 offen"
                             : "=v"(pre[j])
                             : "v"(off[j]), "s"(rsrc), "s"(j * sstep));
    }
    __device__ __forceinline__ void deposit(unsigned char *patch, int row_groups, int lds_row_step) const
    {
        if (active) {
#pragma unroll
            for (int j = 0; j < UMAX; j++)
                if (j < row_groups) // uniform
                    *reinterpret_cast<v4u *>(patch + dst0 + j * lds_row_step) = pre[j];
        }
    }
};

// The tile loop of a workgroup.
template <int PT, int UMAX, bool HE>
__device__ __forceinline__ void tile_loop(const TiledArgs &a, const Ctx &c, Stager<UMAX> &st, unsigned char *patch,
                                          const TileSeq &seq, TilePos pos, int wave, int n_waves, int g_first, int g_count,
                                          bool fast, bool use_lsh)
{
    const ConvGeom &g = a.g;
    // every scalar the loop uses, in a register of its own
    const int8_t *const in = lone(a.in);
    const int img_bytes = lone(a.img_bytes);
    const int in_h = lone(g.in_h), in_w = lone(g.in_w), in_pitch = lone(g.in_pitch);
    const int pad_top = lone(g.pad_top), pad_left = lone(g.pad_left);
    const int th = lone(a.th), tw = lone(a.tw);
    const int row_groups = lone(a.row_groups), row_par = lone(a.row_par);
    const int src_row_step = lone(a.src_row_step), lds_row_step = lone(a.lds_row_step);
    const int n_tiles_yx = lone((int)a.fd_tiles_yx.d), n_tiles_x = lone((int)a.fd_tiles_x.d);
    const FastDiv fd_yx = {lone(a.fd_tiles_yx.m), lone(a.fd_tiles_yx.s), (unsigned)n_tiles_yx};
    const FastDiv fd_x = {lone(a.fd_tiles_x.m), lone(a.fd_tiles_x.s), (unsigned)n_tiles_x};
    const int step = lone(seq.step), end = lone(seq.end);
    int tile = lone(seq.first);
    const bool idle = wave >= a.n_sets; // a wavefront without a set in the tiles of this layer only copies
    const int epi = lone(a.epi);

    const auto request = [&](const TilePos &t) {
        st.request(in + (long long)t.n * img_bytes, img_bytes, t.ty * th - pad_top, t.tx * tw - pad_left, in_h, in_w,
                   in_pitch, row_groups, row_par, src_row_step);
    };
    settle(); // the first patch, requested before the set-up (and whatever the set-up left in flight)
    for (; tile < end; tile += step) {
        st.deposit(patch, row_groups, lds_row_step);
        __syncthreads(); // patch (and, the first time, filters and tables) complete
        TileRef now;
        now.img_out = (long long)pos.n * g.out_h * g.out_w * g.out_pitch;
        now.img_res = (long long)pos.n * g.out_h * g.out_w * g.res_pitch;
        now.oy0 = pos.ty * th;
        now.ox0 = pos.tx * tw;
        now.th_real = min(th, g.out_h - now.oy0);
        now.tw_real = min(tw, g.out_w - now.ox0);
        const int next = tile + step;
        if (next < end) {
            pos = locate_tile(next, fd_yx, fd_x);
            request(pos);
        }
        // every path to the end of the tile settles the request: a set does before its stores, a wavefront
        // without a set does here
        const auto go = [&](auto mode_tag) {
            constexpr int MODE = decltype(mode_tag)::value;
            if (epi == 0)
                run_tile<PT, MODE, HE, 0>(a, c, now, wave, n_waves, g_first, g_count);
            else if (epi == 1)
                run_tile<PT, MODE, HE, 1>(a, c, now, wave, n_waves, g_first, g_count);
            else
                run_tile<PT, MODE, HE, 2>(a, c, now, wave, n_waves, g_first, g_count);
        };
        if (idle)
            settle();
        else if (!fast)
            go(std::integral_constant<int, -1>{});
        else if (HE)
            use_lsh ? go(std::integral_constant<int, 5>{}) : go(std::integral_constant<int, 6>{});
        else
            use_lsh ? go(std::integral_constant<int, 1>{}) : go(std::integral_constant<int, 0>{});
        __syncthreads(); // every wavefront is done with the patch
    }
}

// PT: pixel tiles per set; UMAX: 16-byte pieces of the next patch a thread holds in registers; MAXT / MINB:
// largest workgroup and how many of them share a compute unit (which caps the registers of a wavefront).
template <int PT, int UMAX, int MAXT, int MINB, bool HE>
__global__ __launch_bounds__(MAXT, MINB) void conv2d_s8_tiled_kernel(const TiledArgs a)
{
    constexpr int kUnitsMax = UMAX;
    extern __shared__ __align__(16) unsigned char smem[];
    const ConvGeom &g = a.g;
    v4i *wts = reinterpret_cast<v4i *>(smem);
    int *init_l = reinterpret_cast<int *>(smem + a.off_tabs);
    const int gpc = a.groups_per_chunk;
    int *shift_l = init_l + gpc * 64;
    int *lsh_l = shift_l + gpc * 64;
    int *koff_l = reinterpret_cast<int *>(smem + a.off_koff);
    int8_t *lut_l = reinterpret_cast<int8_t *>(smem + a.off_lut);
    v4i *pix_l = reinterpret_cast<v4i *>(smem + a.off_pix);
    unsigned char *patch = smem + a.off_patch;

    const int tid = threadIdx.x, nthreads = blockDim.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), n_waves = nthreads >> 6;
    const int OC = g.out_c;
    const int g_first = blockIdx.y * gpc;
    const int g_count = min(gpc, a.n_groups - g_first);
    const bool has_lut = a.lut != nullptr;

    const TileSeq seq = xcd_tile_sequence(a.n_tiles);
    Stager<kUnitsMax> st;
    st.init(a, tid);
    TilePos first_pos = {0, 0, 0};
    if (seq.first < seq.end) { // in flight during the set-up
        first_pos = locate_tile(seq.first, a.fd_tiles_yx, a.fd_tiles_x);
        st.request(a.in + (long long)first_pos.n * a.img_bytes, a.img_bytes, first_pos.ty * a.th - g.pad_top,
                   first_pos.tx * a.tw - g.pad_left, g.in_h, g.in_w, g.in_pitch, a.row_groups, a.row_par, a.src_row_step);
    }

    // filters of this workgroup's chunk -> LDS in operand-A order: unit (group, k step, tile, lane) holds the 16
    // k positions [64 ks + 16 (lane / 16), +16) of filter row (lane % 16) of tile t; filter rows are permuted
    // (row i of tile t is filter 4 nt (i / 4) + 4 t + i % 4) so that a lane ends up with 4 nt consecutive channels
    {
        const int units = g_count * a.ksteps * 256;
        for (int u0 = tid; u0 < units; u0 += 4 * nthreads) {
            v4i val[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int u = u0 + j * nthreads;
                val[j] = v4i{0, 0, 0, 0};
                if (u < units) {
                    const int l = u & 63, t = (u >> 6) & 3, rest = u >> 8;
                    const int gi = rest / a.ksteps, ks = rest - gi * a.ksteps;
                    const int gbase = (g_first + gi) * 64;
                    const int nt = group_tiles(OC, gbase);
                    const int i = l & 15;
                    const int oc = gbase + 4 * nt * (i >> 2) + 4 * t + (i & 3);
                    const int k = ks * 64 + (l >> 4) * 16;
                    if (t < nt && oc < OC && k < a.K)
                        val[j] = *reinterpret_cast<const v4i *>(a.w + (size_t)oc * a.K + k);
                }
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (u0 + j * nthreads < units)
                    wts[u0 + j * nthreads] = val[j];
        }
    }
    // offsets of the reduction steps inside the patch, one row per lane group q: entry 0 is step 0, entry 2 + j
    // is step min(j + 1, last) (the layout the product loop reads in pairs)
    for (int e = tid; e < 4 * a.koff_pitch; e += nthreads) {
        const int q = e / a.koff_pitch, j = e - q * a.koff_pitch;
        const int ks = j == 0 ? 0 : min(max(j - 1, 0), a.ksteps - 1);
        const int k = ks * 64 + q * 16;
        int off = 0;
        if (k < a.K) {
            const int tap = k / g.in_c, c0 = k - tap * g.in_c;
            const int ky = tap / g.k_w, kx = tap - ky * g.k_w;
            off = (ky * g.dil_h * a.pw + kx * g.dil_w) * a.cs + c0;
        }
        koff_l[e] = off;
    }
    // positions of the flattened patch that the sets cover: patch offset, output row and column inside the tile
    // (0x7fff: not a pixel of any tile), pixel offset inside the image
    for (int q = tid; q < a.n_sets * PT * 16; q += nthreads) {
        const unsigned row = fastdiv((unsigned)q, a.fd_pw);
        const int ox_l = q - (int)row * a.pw;
        const bool live = q < a.n_ptiles * 16;
        pix_l[q] = v4i{live ? q * a.cs : 0, live ? (int)row : 0x7fff, ox_l, (int)row * g.out_w + ox_l};
    }
    // Can the chunk's filters take the short epilogue?  Every shift in 1..31, and bias + 2^(s-1) plus the
    // largest sum of products must fit int32 also after the left shift by max(0, 8 - s) of the short form.
    const long long mac_bound = (long long)g.k_h * g.k_w * g.in_c * 16384;
    int ok_local = 1, lsh_local = 0;
    for (int c = tid; c < g_count * 64; c += nthreads) {
        const int oc = g_first * 64 + c;
        if (oc < OC) {
            const int s = a.shift[g.n_shift == 1 ? 0 : oc];
            const long long b = a.bias != nullptr ? (long long)a.bias[oc] : 0;
            if (s < 8)
                lsh_local = 1;
            if (s < 1 || s > 31) {
                ok_local = 0;
            } else {
                const long long start = b + (1ll << (s - 1));
                const long long mag = (start < 0 ? -start : start) + mac_bound;
                if (mag >= (1ll << (31 - max(0, 8 - s))))
                    ok_local = 0;
            }
        }
    }
    if (has_lut)
        for (int i = tid; i < 256; i += nthreads)
            lut_l[i] = a.lut[i];
    // (the votes are the same in every lane; readfirstlane lets the compiler branch on them as scalars)
    const bool fast = __builtin_amdgcn_readfirstlane(__syncthreads_and(ok_local)) != 0;
    const bool use_lsh = __builtin_amdgcn_readfirstlane(__syncthreads_or(lsh_local)) != 0;
    for (int c = tid; c < g_count * 64; c += nthreads) {
        const int oc = g_first * 64 + c;
        int init = 0, sh = fast ? 8 : 0, lsh = 0;
        if (oc < OC) {
            const int s = a.shift[g.n_shift == 1 ? 0 : oc];
            const int b = a.bias != nullptr ? a.bias[oc] : 0;
            init = fast ? b + (1 << (s - 1)) - (HE ? 1 : 0) : b; // the half-even form starts one lower
            sh = fast ? max(0, s - 8) : s;
            lsh = fast ? max(0, 8 - s) : 0;
        }
        init_l[c] = init;
        shift_l[c] = sh;
        lsh_l[c] = lsh;
    }

    Ctx c;
    c.wts = wts;
    c.init_l = init_l;
    c.shift_l = shift_l;
    c.lsh_l = lsh_l;
    c.koff_l = koff_l;
    c.lut_l = lut_l;
    c.patch = patch;
    c.pix_l = pix_l;
    c.lane = lane;
    c.col = lane & 15;
    c.quad = lane >> 4;
    c.relu = g.relu != 0;
    c.has_lut = has_lut;
    c.floor_pk = c.relu ? 0 : (int)0x80008000u;

    tile_loop<PT, UMAX, HE>(a, c, st, patch, seq, first_pos, wave, n_waves, g_first, g_count, fast, use_lsh);
}

struct TiledPlan {
    bool ok;
    TiledArgs a;
    size_t lds;
    int threads;
    int variant;
    int per_cu;
    int n_chunks;
    int cus;
    double cost;
};

int round_up(int v, int m)
{
    return (v + m - 1) / m * m;
}

// Tile plan: the cheapest of the (th, tw, filter chunk, workgroup size) combinations that fit LDS.  The cost
// counts matrix-instruction slots of the slowest wavefront per tile, scaled by how much of the device the
// resident workgroups fill; filters and patch compete for LDS.
struct Variant {
    int pt, threads, max_per_cu, umax;
};
constexpr Variant kVariants[] = {
    {4, 256, 2, 8}, // 64 pixels x 64 filters per set, two workgroups of four wavefronts per compute unit
    {4, 512, 1, 8}, // the same with one workgroup of eight wavefronts (a patch up to twice the size)
};
constexpr int kNumVariants = sizeof(kVariants) / sizeof(kVariants[0]);

TiledPlan tiled_plan(const ConvGeom &g, const void *in, const void *filter, int cu_count)
{
    TiledPlan best;
    best.ok = false;
    best.cost = 1e300;
    if (g.k_h * g.k_w < 2 || g.in_c % 16 != 0 || g.in_c < 16 || g.out_c < 1)
        return best;
    if ((reinterpret_cast<uintptr_t>(in) & 15) != 0 || (reinterpret_cast<uintptr_t>(filter) & 15) != 0)
        return best;
    if ((long long)g.in_h * g.in_w * g.in_pitch >= (1ll << 31) || (long long)g.out_h * g.out_w * g.out_pitch >= (1ll << 31) ||
        (long long)g.out_h * g.out_w * g.res_pitch >= (1ll << 31) || (g.in_pitch & 15) != 0)
        return best;
    // Strided windows re-read little of the input, and the direct kernel (operands from global memory) is as
    // fast or faster there (batch 64: 160 x 160 x 64 -> 64 at stride 2 45 us direct against 64 us staged,
    // 320 x 320 x 16 -> 32 64 against 62 us): the staged form is for stride 1.
    if (g.stride_h != 1 || g.stride_w != 1)
        return best;
    const int cus = cu_count > 0 ? cu_count : kPlanCus;
    const int K = g.k_h * g.k_w * g.in_c;
    const int ksteps = (K + 63) / 64;
    const int n_groups = (g.out_c + 63) / 64;
    const int cu16 = g.in_c / 16;
    // LDS pixel pitch in 16-byte units: twice an odd number (or 1).  A 16-byte-per-lane LDS read is served in
    // groups of 8 consecutive columns x 2 neighbouring lane groups; with such a pitch the 16 pieces of a group
    // fall into 16 different bank sets.
    int cs_units = cu16;
    if (cu16 > 1)
        while (cs_units % 4 != 2)
            cs_units++;
    const int cs = 16 * cs_units;
    const int span_h = (g.k_h - 1) * g.dil_h, span_w = (g.k_w - 1) * g.dil_w;

    for (int chunks = 1; chunks <= n_groups; chunks++) {
        const int gpc = (n_groups + chunks - 1) / chunks;
        if ((n_groups + gpc - 1) / gpc != chunks)
            continue;
        // (filters in several chunks mean every chunk's workgroups copy the same patch again; that still beats
        // reading operand B from global memory tap by tap)
        const int w_bytes = gpc * ksteps * 4096;
        const int koff_pitch = round_up(ksteps + 4, 4);
        const int tab_bytes = gpc * 768 + koff_pitch * 16 + 256;
        if (w_bytes + tab_bytes + 4096 > kLdsLimit)
            continue;
        // column tiles: the whole width, or equal parts of it
        for (int ncol = 1; ncol <= 8; ncol++) {
            const int tw = (g.out_w + ncol - 1) / ncol;
            if (ncol > 1 && tw < 16)
                break;
            const int pw = tw + span_w;
            for (int th = 1; th <= g.out_h; th++) {
                const int ph = th + span_h;
                if ((long long)w_bytes + tab_bytes + (long long)(ph * pw + 16 + span_w + 1) * cs > kLdsLimit)
                    break;
                const int n_ptiles = (th * pw + 15) / 16;
                const int tiles_y = (g.out_h + th - 1) / th;
                const long long n_tiles = (long long)g.batch * tiles_y * ncol;
                const int row_units = pw * cu16;
                for (int vi = 0; vi < kNumVariants; vi++) {
                    const Variant &var = kVariants[vi];
                    const int PT = var.pt, threads = var.threads, kUnitsMax = var.umax;
                    const int n_sets = (n_ptiles + PT - 1) / PT;
                    const int waves = threads / 64;
                    if (row_units > threads)
                        continue;
                    const int row_par = std::min(threads / row_units, ph);
                    const int row_groups = (ph + row_par - 1) / row_par;
                    if (row_groups > kUnitsMax)
                        continue;
                    // the patch in LDS: every thread writes row_groups rows, and the pixel tiles of the flattened
                    // patch run up to 16 + span_w positions past its last row
                    const int px_alloc = std::max(row_groups * row_par, ph) * pw + 16 + span_w + 1;
                    const int pix_bytes = n_sets * PT * 256;
                    const long long lds = (long long)w_bytes + tab_bytes + pix_bytes + (long long)px_alloc * cs;
                    if (lds > kLdsLimit)
                        continue;
                    const int per_cu = std::min<long long>(var.max_per_cu, kLdsLimit / lds);
                    if (per_cu < 1)
                        continue;
                    // matrix-instruction time of a tile: the slowest wavefront's sets (k steps x 4 PT instructions
                    // per 64 filters), plus a per-set epilogue and a per-tile fixed cost (barriers, patch copy)
                    const int rounds = (n_sets + waves - 1) / waves;
                    const double set_cost = gpc * (ksteps * 4.0 * PT + 3.0 * PT * 4);
                    double tile_cost = rounds * set_cost + 40.0;
                    // waves of one SIMD share its matrix pipe
                    const double simd_waves = waves * per_cu / 4.0;
                    const double resident = (double)cus * per_cu;
                    const double tiles_total = (double)n_tiles * chunks;
                    const double rounds_dev = std::max(1.0, tiles_total / resident);
                    // a second wavefront on a SIMD hides the first one's epilogue and barriers, not its matrix work
                    const double overlap = simd_waves >= 2.0 ? 0.62 : 1.0;
                    // one workgroup per compute unit stalls all of its wavefronts at every barrier; two overlap
                    // each other's patch copies (measured: 7 to 11 % on 160 x 160 x 32 -> 32 and 80 x 80 x 64 -> 64)
                    const double alone = per_cu < 2 ? 1.12 : 1.0;
                    const double cost = rounds_dev * tile_cost * simd_waves * overlap * alone;
                    if (cost < best.cost) {
                        best.ok = true;
                        best.cost = cost;
                        TiledArgs a = {};
                        a.g = g;
                        a.K = K;
                        a.ksteps = ksteps;
                        a.n_groups = n_groups;
                        a.groups_per_chunk = gpc;
                        a.th = th;
                        a.tw = tw;
                        a.ph = ph;
                        a.pw = pw;
                        a.cs = cs;
                        a.cu16 = cu16;
                        a.n_ptiles = n_ptiles;
                        a.n_sets = n_sets;
                        a.tiles_x = ncol;
                        a.tiles_y = tiles_y;
                        a.n_tiles = (int)std::min<long long>(n_tiles, 0x7fffffff);
                        a.row_units = row_units;
                        a.row_par = row_par;
                        a.row_groups = row_groups;
                        a.src_row_step = row_par * g.in_w * g.in_pitch;
                        a.lds_row_step = row_par * pw * cs;
                        a.img_bytes = g.in_h * g.in_w * g.in_pitch;
                        a.off_tabs = w_bytes;
                        a.off_koff = w_bytes + gpc * 768;
                        a.off_lut = a.off_koff + koff_pitch * 16;
                        a.koff_pitch = koff_pitch;
                        a.off_pix = a.off_lut + 256;
                        a.off_patch = a.off_pix + pix_bytes;
                        best.a = a;
                        best.lds = (size_t)lds;
                        best.threads = threads;
                        best.variant = vi;
                        best.per_cu = per_cu;
                        best.n_chunks = chunks;
                        best.cus = cus;
                        if (n_tiles > 0x7fffffff)
                            best.ok = false;
                    }
                }
            }
        }
    }
    return best;
}

template <int PT, int UMAX, int MAXT, int MINB, bool HE>
hipError_t launch_tiled(const TiledPlan &plan, hipStream_t stream)
{
    auto kernel = conv2d_s8_tiled_kernel<PT, UMAX, MAXT, MINB, HE>;
    static bool raised = false; // the dynamic LDS limit of a kernel is raised once per process
    if (!raised) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, kLdsLimit);
        if (e != hipSuccess)
            return e;
        raised = true;
    }
    const TiledArgs &a = plan.a;
    int per_cu = resident_workgroups_per_cu(kernel, plan.threads, plan.lds);
    per_cu = std::min(per_cu, plan.per_cu);
    int gx = std::max(1, plan.cus * per_cu);
    if (gx > a.n_tiles)
        gx = a.n_tiles;
    if (gx >= 8)
        gx &= ~7; // blockIdx.x % 8 is then the XCD of a workgroup, for every blockIdx.y
    hipLaunchKernelGGL(kernel, dim3((unsigned)gx, (unsigned)plan.n_chunks), dim3((unsigned)plan.threads), plan.lds,
                       stream, a);
    return hipGetLastError();
}

template <bool HE>
hipError_t launch_variant(const TiledPlan &plan, hipStream_t stream)
{
    switch (plan.variant) {
    case 0:
        return launch_tiled<4, 8, 256, 2, HE>(plan, stream);
    default:
        return launch_tiled<4, 8, 512, 1, HE>(plan, stream);
    }
}

} // namespace


bool conv2d_s8_tiled_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count)
{
    return tiled_plan(g, in, filter, cu_count).ok;
}

hipError_t launch_conv2d_s8_tiled(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                  const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                  int cu_count, hipStream_t stream)
{
    if ((long long)g.batch * g.out_h * g.out_w == 0)
        return hipSuccess;
    TiledPlan plan = tiled_plan(g, in, filter, cu_count);
    if (!plan.ok)
        return hipErrorInvalidValue;
    TiledArgs &a = plan.a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.res = residual;
    a.out = out;
    const uintptr_t out_addr = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(residual);
    a.out_vec = ((g.out_c & 15) == 0 && (out_addr & 15) == 0) ? 16 : (((g.out_c & 3) == 0 && (out_addr & 3) == 0) ? 4 : 1);
    // the 16-byte-store forms need every store (and residual load) aligned: pitches of whole 16-byte pieces
    a.epi = (g.out_c % 64 == 0 && a.out_vec == 16 && (g.out_pitch & 15) == 0 && (g.res_pitch & 15) == 0)
        ? ((lut == nullptr && residual == nullptr) ? 0 : 1)
        : 2;
    a.fd_cu16 = make_fastdiv((unsigned)a.cu16);
    a.fd_row_units = make_fastdiv((unsigned)a.row_units);
    a.fd_pw = make_fastdiv((unsigned)a.pw);
    a.fd_tiles_x = make_fastdiv((unsigned)a.tiles_x);
    a.fd_tiles_yx = make_fastdiv((unsigned)(a.tiles_y * a.tiles_x));
    static const bool trace = getenv("ESPDL_HIP_TRACE") != nullptr;
    if (trace)
        fprintf(stderr, "conv2d_s8_tiled: %dx%dx%d -> %d k%dx%d s%d tile %dx%d patch %dx%d cs %d ptiles %d sets %d chunks %d gpc %d "
                        "variant %d threads %d lds %zu tiles %d row units %d x %d\n",
                g.in_h, g.in_w, g.in_c, g.out_c, g.k_h, g.k_w, g.stride_w, a.th, a.tw, a.ph, a.pw, a.cs, a.n_ptiles, a.n_sets,
                plan.n_chunks, a.groups_per_chunk, plan.variant, plan.threads, plan.lds, a.n_tiles, a.row_units, a.row_par);
    return g.half_even ? launch_variant<true>(plan, stream) : launch_variant<false>(plan, stream);
}

} // namespace espdl
