// Stage building blocks of the inverted-residual kernels that run expand -> depthwise -> project with
// wavefronts working on their own (mbconv_s8_wave.hip: one wavefront per tile; mbconv_s8_group.hip: a
// workgroup of wavefronts that split the expanded channels of one tile).  The arithmetic is that of the
// separate operators: conv2d_11cn + n_wise epilogue (esp-dl/dl/base/dl_base_conv2d.cpp:9-33;
// esp-dl/dl/base/dl_base_activate_buffer.hpp:10-74, 162-212), depthwise_conv2d_33c1 under the shell's
// window clipping (esp-dl/dl/base/dl_base_depthwise_conv2d.cpp:19-65; esp-dl/dl/base/dl_base.hpp:1852-2102).
#pragma once

#include <type_traits>

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {
namespace mbstage {

constexpr int kDws = 80; // LDS pixel stride of a 64-channel depthwise result: 64 + 16 (odd number of 16-byte units)

// 16 bytes at p + off of which the first `nvalid` exist (nvalid a multiple of 4, possibly <= 0); the rest
// are zeros.  Branch-free: a piece that does not exist is read from offset 0 of `p` instead (always a valid
// address) and replaced by zero, so that every lane issues the same loads and the wait counters of loads
// requested ahead of their use stay exact.  VEC16: p + off is 16-byte aligned whenever nvalid >= 16 and
// nvalid is then never in 1..15.
template <bool VEC16>
__device__ __forceinline__ v4i load16_partial(const int8_t *p, unsigned off, int nvalid)
{
    // `p` is the same in every lane and `off` is an unsigned 32-bit byte offset: one scalar base plus one
    // vector offset per load, no 64-bit address arithmetic on the vector ALU
    v4i r;
    if constexpr (VEC16) {
        const bool ok = nvalid >= 16;
        r = *reinterpret_cast<const v4i *>(p + (size_t)(ok ? off : 0u));
        r = ok ? r : v4i{0, 0, 0, 0};
    } else {
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const bool ok = 4 * d < nvalid;
            const int v = *reinterpret_cast<const int *>(p + (size_t)(ok ? off + 4u * d : 0u));
            r[d] = ok ? v : 0;
        }
    }
    return r;
}

// The same addresses, nothing zeroed: pieces that do not exist read the first bytes at `p` and keep them.  For
// operand B of the expand products, where such bytes never count: a pixel outside the image has its expand
// OUTPUT zeroed, and reduction positions past the last input channel meet zeros in operand A.  Without the
// select between a load and its product, the loads of a patch stay in flight behind the set-up that follows.
template <bool VEC16>
__device__ __forceinline__ v4i load16_clamped(const int8_t *p, unsigned off, int nvalid)
{
    v4i r;
    if constexpr (VEC16) {
        r = *reinterpret_cast<const v4i *>(p + (size_t)(nvalid >= 16 ? off : 0u));
    } else {
#pragma unroll
        for (int d = 0; d < 4; d++)
            r[d] = *reinterpret_cast<const int *>(p + (size_t)(4 * d < nvalid ? off + 4u * d : 0u));
    }
    return r;
}

// Orders the LDS accesses of the wavefront's lanes among each other.  LDS executes the instructions of one
// wavefront in order, so nothing has to be waited for; the compiler must not move accesses across.
__device__ __forceinline__ void wave_lds_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Is the short epilogue (pack_fast4) exact for this channel?  The shift must be in 1..31 and
// |bias| + 2^(s-1) + mac_bound (the largest magnitude the accumulator can reach) must stay below
// 2^(31 - max(0, 8 - s)), so that neither the accumulator nor its left-shifted form overflows.
// mac_bound < 2^30 (checked on the host); everything fits unsigned 32-bit arithmetic.
__device__ __forceinline__ bool short_ok(int s, int bias, unsigned mac_bound)
{
    if (s < 1 || s > 31)
        return false;
    const unsigned lim = 1u << (31 - max(0, 8 - s));
    const unsigned t = mac_bound + (1u << (s - 1));
    const unsigned ub = bias < 0 ? 0u - (unsigned)bias : (unsigned)bias;
    return t < lim && ub < lim - t;
}

// Requantization constants of four consecutive channels of one stage, and which epilogue the whole
// wavefront takes for them: pack_fast4 mode 0 (every shift >= 8), 1 (some shift below 8), 6 and 5 (the
// same two in half-even), or -1 for the general shift_and_round restatement (a shift outside 1..31, or an accumulator that could
// overflow the short form).
struct StageConsts {
    v4i init, rsh, lsh;
    int mode;
};

// Per-channel constants of a stage live in LDS as three rows of n_ch int32: [bias + rounding constant (2^(s-1), one less in half-even) |
// right shift | left shift] in the form the short epilogue wants, or [bias | shift | 0] for the general one.
// build_stage_tables fills the tables of the three stages (expand and depthwise: the same n_ch channels;
// project: see below) with ONE memory round trip and ONE workgroup vote, which is also the barrier after which the tables are complete: every lane writes
// the short-epilogue form of its channels straight away and the vote tells whether some channel of a stage
// cannot take it; only then (rare) that stage's table is rewritten with the plain bias and shift, behind a
// second barrier.  `votes` is one LDS word per wavefront of the workgroup (kStageVoteBytes in all; a wavefront
// stores the OR of its lanes' flags, every lane ORs the words after the barrier).  Every lane of the workgroup
// must call this.
constexpr int kStageVoteBytes = 64; // up to 16 wavefronts
// The project stage has its own table of n_pad_p channels (out_c rounded up to 16; channels that do not
// exist get bias 0 and shift 8), in the same three-row layout; its epilogue reads it with
// read_stage_table<false> (shift counts, not multipliers).
struct StageTablesArgs {
    int *votes, *tab_e, *tab_d, *tab_p;
    const int32_t *b_e, *s_e, *b_d, *s_d, *b_p, *s_p;
    int n_s_e, n_s_d, n_s_p;
    int n_ch, n_ch_p, n_pad_p;
    unsigned bound_e, bound_d, bound_p;
};
__device__ __forceinline__ void build_stage_tables(const StageTablesArgs &t, bool half_even, int tid, int nthreads,
                                                   int &mode_e, int &mode_d, int &mode_p)
{
    const unsigned step_e = t.n_s_e == 1 ? 0u : 1u, step_d = t.n_s_d == 1 ? 0u : 1u, step_p = t.n_s_p == 1 ? 0u : 1u;
    const int n_ch = t.n_ch;
    const int he1 = half_even ? 1 : 0; // the half-even forms start one below the half-up rounding constant
    // bits 0 / 1 / 2: expand / depthwise / project needs the general form; bits 3 / 4 / 5: a shift below 8
    int flags = 0;
    for (int c = tid; c < n_ch; c += nthreads) {
        const int be = t.b_e != nullptr ? t.b_e[(size_t)(unsigned)c] : 0;
        const int bd = t.b_d != nullptr ? t.b_d[(size_t)(unsigned)c] : 0;
        const int se = t.s_e[(size_t)(step_e * (unsigned)c)];
        const int sd = t.s_d[(size_t)(step_d * (unsigned)c)];
        flags |= short_ok(se, be, t.bound_e) ? 0 : 1;
        flags |= short_ok(sd, bd, t.bound_d) ? 0 : 2;
        flags |= se < 8 ? 8 : 0;
        flags |= sd < 8 ? 16 : 0;
        const int se1 = min(max(se, 1), 31), sd1 = min(max(sd, 1), 31); // defined shifts where the form does not apply
        t.tab_e[c] = be + (1 << (se1 - 1)) - he1;
        t.tab_e[n_ch + c] = max(0, se - 8);
        t.tab_e[2 * n_ch + c] = max(0, 8 - se);
        t.tab_d[c] = bd + (1 << (sd1 - 1)) - he1;
        t.tab_d[n_ch + c] = max(0, sd - 8);
        t.tab_d[2 * n_ch + c] = max(0, 8 - sd);
    }
    // the project channels are few: the last lanes of the workgroup take them, so that with up to
    // nthreads - n_pad_p expanded channels no lane does both
    for (int c = nthreads - 1 - tid; c < t.n_pad_p; c += nthreads) {
        const bool exists = c < t.n_ch_p;
        const int bp = (exists && t.b_p != nullptr) ? t.b_p[(size_t)(unsigned)c] : 0;
        const int sp = exists ? t.s_p[(size_t)(step_p * (unsigned)c)] : 8;
        flags |= short_ok(sp, bp, t.bound_p) ? 0 : 4;
        flags |= sp < 8 ? 32 : 0;
        const int sp1 = min(max(sp, 1), 31);
        t.tab_p[c] = bp + (1 << (sp1 - 1)) - he1;
        t.tab_p[t.n_pad_p + c] = max(0, sp - 8);
        t.tab_p[2 * t.n_pad_p + c] = max(0, 8 - sp);
    }
    {
        int wf = 0; // OR over the wavefront's lanes, bit by bit
#pragma unroll
        for (int b = 0; b < 6; b++)
            wf |= __any(flags & (1 << b)) ? 1 << b : 0;
        if ((tid & 63) == 0)
            t.votes[tid >> 6] = wf;
    }
    __syncthreads();
    int all = 0;
    for (int w = 0; w < (nthreads >> 6); w++)
        all |= t.votes[w];
    if (all & 7) { // uniform
        for (int c = tid; c < n_ch; c += nthreads) {
            if (all & 1) {
                t.tab_e[c] = t.b_e != nullptr ? t.b_e[(size_t)(unsigned)c] : 0;
                t.tab_e[n_ch + c] = t.s_e[(size_t)(step_e * (unsigned)c)];
                t.tab_e[2 * n_ch + c] = 0;
            }
            if (all & 2) {
                t.tab_d[c] = t.b_d != nullptr ? t.b_d[(size_t)(unsigned)c] : 0;
                t.tab_d[n_ch + c] = t.s_d[(size_t)(step_d * (unsigned)c)];
                t.tab_d[2 * n_ch + c] = 0;
            }
        }
        if (all & 4) {
            for (int c = tid; c < t.n_pad_p; c += nthreads) {
                const bool exists = c < t.n_ch_p;
                t.tab_p[c] = (exists && t.b_p != nullptr) ? t.b_p[(size_t)(unsigned)c] : 0;
                t.tab_p[t.n_pad_p + c] = exists ? t.s_p[(size_t)(step_p * (unsigned)c)] : 8;
                t.tab_p[2 * t.n_pad_p + c] = 0;
            }
        }
        __syncthreads();
    }
    mode_e = (all & 1) ? -1 : (half_even ? ((all & 8) ? 5 : 6) : ((all & 8) ? 1 : 0));
    mode_d = (all & 2) ? -1 : (half_even ? ((all & 16) ? 5 : 6) : ((all & 16) ? 1 : 0));
    mode_p = (all & 4) ? -1 : (half_even ? ((all & 32) ? 5 : 6) : ((all & 32) ? 1 : 0));
}

// MULTIPLIERS: in mode 1 turn the left-shift counts into the packed multipliers of pack_fast4<4>
// (wave_pack_tab); false leaves the counts (wave_pack, pack_fast4_add).
template <bool MULTIPLIERS = true>
__device__ __forceinline__ StageConsts read_stage_table(const int *tab, int n_ch, int ch, int mode)
{
    StageConsts c;
    c.init = *reinterpret_cast<const v4i *>(tab + ch);
    c.rsh = *reinterpret_cast<const v4i *>(tab + n_ch + ch);
    c.lsh = v4i{0, 0, 0, 0};
    if (mode == 1 || mode == 5)
        c.lsh = *reinterpret_cast<const v4i *>(tab + 2 * n_ch + ch);
    if (MULTIPLIERS && mode == 1) // the multiplier form of pack_fast4<4>: 2^lsh of the channel pairs as packed int16
        c.lsh = v4i{(1 << c.lsh[0]) | (65536 << c.lsh[1]), (1 << c.lsh[2]) | (65536 << c.lsh[3]), 0, 0};
    c.mode = mode;
    return c;
}

// CLIP: a Clip sits behind the stage; floor_pk / ceil_pk carry its bounds (see pack_fast4), the general form
// reads them back out of the packed words.
template <int MODE, bool CLIP = false>
__device__ __forceinline__ int wave_pack(const v4i &acc, const StageConsts &c, int floor_pk, bool relu, bool half_even,
                                         int ceil_pk = 0x7fff7fff)
{
    if constexpr (MODE >= 0) {
        return pack_fast4<MODE, CLIP>(acc, c.lsh, c.rsh, floor_pk, ceil_pk);
    } else {
        int q[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            q[r] = requant_s8(acc[r], c.rsh[r], relu, half_even);
            if constexpr (CLIP)
                q[r] = min(max(q[r], (int)(short)(floor_pk & 0xffff) >> 8), (int)(short)(ceil_pk & 0xffff) >> 8);
        }
        return pack4_s8(q[0], q[1], q[2], q[3]);
    }
}

// The same for constants that came from read_stage_table: in mode 1 they carry multipliers, not shift counts.
template <int MODE, bool CLIP = false>
__device__ __forceinline__ int wave_pack_tab(const v4i &acc, const StageConsts &c, int floor_pk, bool relu, bool half_even,
                                             int ceil_pk = 0x7fff7fff)
{
    if constexpr (MODE == 1)
        return pack_fast4<4, CLIP>(acc, c.lsh, c.rsh, floor_pk, ceil_pk);
    else
        return wave_pack<MODE, CLIP>(acc, c, floor_pk, relu, half_even, ceil_pk);
}

// Expand stage of one chunk of 16 channels: every patch pixel tile through one MFMA and the epilogue, four
// tiles at a time so that four independent MFMA -> requantize -> store chains are in flight (tiles past
// n_xpt inside the last group of four have zero operands and a zero mask and land in slack).
// PACK = 2 or 4 (block inputs of at most 32 / 16 channels): the four 16-lane groups of an operand-B register set
// hold PACK pixel tiles (tile PACK g + t in the groups t * 4 / PACK ...), so the patch takes 1 / PACK of the
// registers and of the loads; operand A comes in PACK copies, copy t holding the filter in the groups of tile t
// and zeros elsewhere, which picks tile t out of the reduction.
template <int MODE, int NXPT, bool EXACT, int KSE = 1, bool PIPE = false, int PACK = 1, bool CLIP = false>
__device__ __forceinline__ void expand_chunk(const v4i (&xb)[PACK > 1 ? (NXPT + PACK - 1) / PACK : NXPT * KSE], int n_xpt,
                                             unsigned xmask, const v4i (&aop)[PACK > 1 ? PACK : KSE], const StageConsts &c,
                                             int floor_pk, bool relu, bool half_even,
                                             unsigned char *dst /* exp_l + col * 16 + 4 * quad */, int ceil_pk = 0x7fff7fff)
{
    auto product = [&](int pt) -> v4i {
        v4i acc = c.init;
        if constexpr (PACK > 1) {
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[pt % PACK], xb[pt / PACK], acc, 0, 0, 0);
        } else {
#pragma unroll
            for (int ks = 0; ks < KSE; ks++)
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[ks], xb[pt * KSE + ks], acc, 0, 0, 0);
        }
        return acc;
    };
    auto finish = [&](const v4i &acc, int pt) {
        int word = wave_pack_tab<MODE, CLIP>(acc, c, floor_pk, relu, half_even, ceil_pk);
        word &= __builtin_amdgcn_sbfe((int)xmask, pt, 1); // all ones or zero
        *reinterpret_cast<int *>(dst + pt * 256) = word;
    };
    if constexpr (EXACT && PIPE) {
        // software pipeline: the matrix product of the next pixel tile is issued before the requantization of
        // the current one, so the matrix pipe works while the vector ALU requantizes (the scheduling barriers
        // keep the compiler from putting the two back in source order of dependence)
        v4i acc[2];
        acc[0] = product(0);
#pragma unroll
        for (int pt = 0; pt < NXPT; pt++) {
            if (pt + 1 < NXPT)
                acc[(pt + 1) & 1] = product(pt + 1);
            __builtin_amdgcn_sched_barrier(0);
            finish(acc[pt & 1], pt);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
#pragma unroll
        for (int g0 = 0; g0 < NXPT; g0 += 4) {
            if (EXACT || g0 < n_xpt) { // uniform
                v4i acc[4];
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (g0 + j < NXPT)
                        acc[j] = product(g0 + j);
#pragma unroll
                for (int j = 0; j < 4; j++)
                    if (g0 + j < NXPT)
                        finish(acc[j], g0 + j);
            }
        }
    }
}

// Depthwise stage of one chunk of 16 channels.  S == 1: output rows in pairs, four patch rows per read.
template <int MODE, int PT, int S, bool EXACT, bool PIPE = false, bool CLIP = false>
__device__ __forceinline__ void depthwise_chunk(const unsigned char *src /* exp_l + (quad * pw + S * col) * 16 */,
                                                int th, int pw, const v4i (&a0)[3], const v4i (&a1)[3],
                                                const StageConsts &c, int floor_pk, bool relu, bool half_even,
                                                unsigned char *dst /* lane's slot in output row 0 of the result */,
                                                int row_bytes = 16 * kDws, bool write_ok = true, int ceil_pk = 0x7fff7fff)
{
    if constexpr (EXACT && PIPE) {
        // software pipeline over units (S == 1: a pair of output rows, S == 2: one output row): operand-B
        // reads two units ahead, matrix products one unit ahead of the requantization
        constexpr int UNITS = S == 1 ? (PT + 1) / 2 : PT;
        constexpr int ROWS = S == 1 ? 2 : 1;
        v4i b[3][3], acc[2][2];
        auto read = [&](int u) {
            const unsigned char *sp = src + (S == 1 ? 2 * u : S * u) * pw * 16;
#pragma unroll
            for (int kx = 0; kx < 3; kx++)
                b[u % 3][kx] = *reinterpret_cast<const v4i *>(sp + 16 * kx);
        };
        auto products = [&](int u) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                if (ROWS * u + r < PT) {
                    const v4i(&aw)[3] = r == 0 ? a0 : a1;
                    v4i v = __builtin_amdgcn_mfma_i32_16x16x64_i8(aw[0], b[u % 3][0], c.init, 0, 0, 0);
                    v = __builtin_amdgcn_mfma_i32_16x16x64_i8(aw[1], b[u % 3][1], v, 0, 0, 0);
                    acc[u & 1][r] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aw[2], b[u % 3][2], v, 0, 0, 0);
                }
            }
        };
        auto finish = [&](int u) {
#pragma unroll
            for (int r = 0; r < ROWS; r++) {
                if (ROWS * u + r < PT) {
                    const int w = wave_pack_tab<MODE, CLIP>(acc[u & 1][r], c, floor_pk, relu, half_even, ceil_pk);
                    if (write_ok)
                        *reinterpret_cast<int *>(dst + (ROWS * u + r) * row_bytes) = w;
                }
            }
        };
        read(0);
        if (UNITS > 1)
            read(1);
        products(0);
#pragma unroll
        for (int u = 0; u < UNITS; u++) {
            if (u + 2 < UNITS)
                read(u + 2);
            if (u + 1 < UNITS)
                products(u + 1);
            __builtin_amdgcn_sched_barrier(0);
            finish(u);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else if constexpr (S == 1) {
#pragma unroll
        for (int j = 0; j < (PT + 1) / 2; j++) {
            if (EXACT || 2 * j < th) { // uniform
                const unsigned char *s = src + 2 * j * pw * 16;
                const v4i b0 = *reinterpret_cast<const v4i *>(s);
                const v4i b1 = *reinterpret_cast<const v4i *>(s + 16);
                const v4i b2 = *reinterpret_cast<const v4i *>(s + 32);
                v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[0], b0, c.init, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[1], b1, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[2], b2, acc, 0, 0, 0);
                const int w0 = wave_pack_tab<MODE, CLIP>(acc, c, floor_pk, relu, half_even, ceil_pk);
                if (write_ok)
                    *reinterpret_cast<int *>(dst + (2 * j) * row_bytes) = w0;
                if (EXACT ? 2 * j + 1 < PT : 2 * j + 1 < th) {
                    v4i acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[0], b0, c.init, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[1], b1, acc1, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1[2], b2, acc1, 0, 0, 0);
                    const int w1 = wave_pack_tab<MODE, CLIP>(acc1, c, floor_pk, relu, half_even, ceil_pk);
                    if (write_ok)
                        *reinterpret_cast<int *>(dst + (2 * j + 1) * row_bytes) = w1;
                }
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < PT; t++) {
            if (EXACT || t < th) { // uniform
                const unsigned char *s = src + S * t * pw * 16;
                const v4i b0 = *reinterpret_cast<const v4i *>(s);
                const v4i b1 = *reinterpret_cast<const v4i *>(s + 16);
                const v4i b2 = *reinterpret_cast<const v4i *>(s + 32);
                v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[0], b0, c.init, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[1], b1, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0[2], b2, acc, 0, 0, 0);
                const int w0 = wave_pack_tab<MODE, CLIP>(acc, c, floor_pk, relu, half_even, ceil_pk);
                if (write_ok)
                    *reinterpret_cast<int *>(dst + t * row_bytes) = w0;
            }
        }
    }
}

// One dword of a diagonal operand A: weight byte `w` of channel row i sits at byte i of the lane's 16.
__device__ __forceinline__ v4i diag_operand(int w, int i)
{
    const int d = (w & 0xff) << (8 * (i & 3));
    const int sel = i >> 2;
    return v4i{sel == 0 ? d : 0, sel == 1 ? d : 0, sel == 2 ? d : 0, sel == 3 ? d : 0};
}

} // namespace mbstage
} // namespace espdl
