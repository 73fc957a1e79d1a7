// Dense int8 convolution / Gemm / MatMul for gfx950 as an implicit GEMM on v_mfma_i32_16x16x64_i8.
//
// What it computes is the reference's conv2d_11cn / conv2d_33cn / conv2d_hwcn MAC
// (esp-dl/dl/base/dl_base_conv2d.cpp:9-163) over every output pixel that conv_operation_shell visits
// (esp-dl/dl/base/dl_base.hpp:940-1191), followed by the n_wise epilogue
// (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210).  Integer sums are
// order-independent, so the MFMA's accumulation order cannot change a result.
//
// Mapping.  GEMM rows (MFMA operand A) are filters, GEMM columns (operand B) are output pixels, the
// reduction axis is k = (ky, kx, c) in the filter's own memory order.  One wavefront owns 16*PT
// pixels; for each group of up to 64 filters it runs 4 MFMA tiles per 64-wide k step.  After the
// MFMA a lane holds 4 consecutive rows of one column, so the filter -> tile-row assignment is
// permuted (row i of tile t is filter 4*nt*(i/4) + 4*t + i%4 of the group, nt = tiles in the group):
// every lane then ends up with 4*nt *consecutive* output channels of one pixel and stores them with a
// single 16-byte (nt = 4) write; the four lanes of a pixel cover 64 contiguous bytes of the NHWC row.
//
// Weights are re-laid into LDS once per workgroup in exactly the order the MFMA reads operand A
// (one 16-byte unit per lane, units of a tile contiguous), zero-padded along k and along the
// filter axis; padded k positions multiply to zero whatever operand B holds there.  Operand B is
// read straight from global memory, 16 bytes per lane:
//   B_VEC16   in_c % 16 == 0: the 16 k positions of a lane lie inside one filter tap -> one
//             aligned 16-byte load, or zeros when the tap falls into the padding;
//   B_POINT   1x1 filter without padding: k is the channel index; one (possibly unaligned) 16-byte
//             load that may run past in_c into the next pixel (those positions meet zero weights);
//   B_ROWSEG  dilation_w == 1: the k_w * in_c bytes of one filter row are contiguous in the input, so
//             the reduction axis is re-ordered as (ky, j) with every row segment padded to a
//             multiple of 16; a lane's chunk is one unaligned 16-byte load, masked at the left and
//             right image borders (the 3-channel stem convolutions run this way);
//   B_GATHER  anything else: byte gather.
// Epilogue.  When every shift of the workgroup's filters lies in 1..31, rounding is half-up and
// |bias + 2^(s-1)| + K * 2^14 cannot overflow, the accumulator starts at bias + 2^(s-1) and a value
// costs about three VALU instructions: t = (acc << max(0, 8-s)) >> max(0, s-8) carries the result in
// bits 8.. of t, v_cvt_pk_i16_i32 saturates two of them to int16 (which saturates the int8 result
// held in the high byte), and one v_perm_b32 gathers four high bytes into the output dword.
// Otherwise the general shift_and_round restatement runs.
// A workgroup is persistent: it keeps its filter chunk in LDS and walks pixel sets with a grid
// stride.  While one pixel set is in the MFMA/epilogue phase the operand-B loads of the next set are
// already in flight (register double buffer), and when the whole reduction axis fits in registers
// (KSC k steps) all its loads are issued back to back, so a wavefront pays one memory latency per
// pixel set instead of one per k step.  If 64 filters x K do not fit the LDS budget, K is processed
// in chunks that are re-staged between barriers while the accumulators stay in registers.
#pragma once

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {
namespace mfma_conv {

enum { B_VEC16 = 0, B_POINT = 1, B_GATHER = 2, B_ROWSEG = 3 };

constexpr int kThreads = 256; // 4 wavefronts

struct MfmaConvArgs {
    const int8_t *in;
    const int8_t *w;
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
    const int8_t *res; // tensor of the output's shape added with saturation to the stored value, or nullptr
    int8_t *out;
    ConvGeom g;
    int K;                // length of the reduction axis as the MFMA sees it (k_h * seg_pad for B_ROWSEG)
    int seg_len;          // B_ROWSEG: k_w * in_c, bytes of one filter row
    int seg_pad;          // B_ROWSEG: seg_len rounded up to a multiple of 16
    int ksteps;           // ceil(K / 64)
    int ks_per_chunk;     // k steps resident in LDS at a time (== ksteps when everything fits)
    int n_kchunks;        // ceil(ksteps / ks_per_chunk)
    int n_groups;         // ceil(out_c / 64)
    int groups_per_chunk; // filter groups resident in LDS (1 when n_kchunks > 1)
    int n_sets;           // pixel sets of 64 * PT pixels
    long long npix;       // batch * out_h * out_w
    long long in_bytes;   // size of the input tensor
    int out_vec;          // widest store the output allows: 16, 4 or 1 bytes
    FastDiv fd_out_hw, fd_out_w, fd_in_c, fd_k_w, fd_seg_pad; // launch-invariant divisors
    int stage_out;        // 1: a wave collects its 16*PT x out_c outputs in LDS and writes them as one
                          //    contiguous block (needs every filter group resident, i.e. one chunk)
};

__device__ __forceinline__ int group_tiles(int out_c, int gbase)
{
    const int rem = out_c - gbase;
    return rem >= 64 ? 4 : (rem + 15) >> 4;
}

// One 16-byte unit of operand A: filters (tile t, row i) x 16 k positions, zero padded.
__device__ __forceinline__ v4i weight_unit(const MfmaConvArgs &a, int gbase, int t, int l, int k)
{
    const int OC = a.g.out_c, K = a.K;
    const int nt = group_tiles(OC, gbase);
    v4i val = {0, 0, 0, 0};
    if (t >= nt)
        return val;
    const int i = l & 15;
    const int oc = gbase + 4 * nt * (i >> 2) + 4 * t + (i & 3);
    if (oc >= OC || k >= K)
        return val;
    if (a.seg_pad > 0) {
        // (ky, j) ordering: filter row ky starts at k = ky * seg_pad and holds seg_len bytes
        const int ky = k / a.seg_pad, j0 = k - ky * a.seg_pad;
        const int8_t *src = a.w + ((size_t)oc * a.g.k_h + ky) * a.seg_len + j0;
        unsigned int words[4] = {0, 0, 0, 0};
        const int n = min(16, a.seg_len - j0);
        for (int b = 0; b < n; b++)
            words[b >> 2] |= (unsigned int)(unsigned char)src[b] << ((b & 3) * 8);
        return v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
    }
    const int8_t *src = a.w + (size_t)oc * K + k;
    if ((K & 15) == 0 && (reinterpret_cast<uintptr_t>(a.w) & 15) == 0)
        return *reinterpret_cast<const v4i *>(src);
    const int n = min(16, K - k);
    if ((long long)oc * K + k + 16 <= (long long)OC * K) {
        // 16 bytes from any address in one load; what lies past the filter's last position is cut off
        v4i v = *reinterpret_cast<const v4i_unaligned *>(src);
#pragma unroll
        for (int d = 0; d < 4; d++) {
            const int keep = min(max(n - 4 * d, 0), 4);
            v[d] = keep >= 4 ? v[d] : (int)((unsigned)v[d] & ((1u << (8 * keep)) - 1u));
        }
        return v;
    }
    unsigned int words[4] = {0, 0, 0, 0};
    for (int b = 0; b < n; b++)
        words[b >> 2] |= (unsigned int)(unsigned char)src[b] << ((b & 3) * 8);
    return v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
}

// Copy one K chunk of `g_count` filter groups into LDS in MFMA operand-A order.  Four units per
// thread are fetched before any is stored, so their global loads overlap.
__device__ __forceinline__ void stage_weights(const MfmaConvArgs &a, v4i *wts, int g_first, int g_count, int ks_begin,
                                              int ks_count)
{
    const int units = g_count * ks_count * 256;
    for (int u0 = threadIdx.x; u0 < units; u0 += 4 * kThreads) {
        v4i val[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int u = u0 + j * kThreads;
            val[j] = v4i{0, 0, 0, 0};
            if (u < units) {
                const int l = u & 63, t = (u >> 6) & 3, rest = u >> 8;
                const int gi = rest / ks_count, ks = rest - gi * ks_count;
                val[j] = weight_unit(a, (g_first + gi) * 64, t, l, (ks_begin + ks) * 64 + (l >> 4) * 16);
            }
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (u0 + j * kThreads < units)
                wts[u0 + j * kThreads] = val[j];
    }
}

// Operand B for one lane: the 16 k positions [k, k+16) of output pixel (img_off, iy0, ix0).
template <int BMODE>
__device__ __forceinline__ v4i load_b(const MfmaConvArgs &a, bool valid, long long img_off, int iy0, int ix0, int k)
{
    v4i r = {0, 0, 0, 0};
    const ConvGeom &g = a.g;
    if (!valid || k >= a.K)
        return r;
    if (BMODE == B_POINT) {
        // flat pointwise: img_off is the byte offset of the lane's input pixel
        const long long off = img_off + k;
        if (off + 16 <= a.in_bytes) {
            __builtin_memcpy(&r, a.in + off, 16); // one dwordx4 load; gfx950 global loads need no alignment
        } else {
            unsigned int words[4] = {0, 0, 0, 0};
            const int n = min(16, a.K - k);
            for (int b = 0; b < n; b++)
                words[b >> 2] |= (unsigned int)(unsigned char)a.in[off + b] << ((b & 3) * 8);
            r = v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
        }
        return r;
    }
    if (BMODE == B_VEC16) {
        const int tap = (int)fastdiv((unsigned)k, a.fd_in_c), c0 = k - tap * g.in_c;
        const int ky = (int)fastdiv((unsigned)tap, a.fd_k_w), kx = tap - ky * g.k_w;
        const int iy = iy0 + ky * g.dil_h, ix = ix0 + kx * g.dil_w;
        if ((unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w)
            r = *reinterpret_cast<const v4i *>(a.in + img_off + ((long long)iy * g.in_w + ix) * g.in_pitch + c0);
        return r;
    }
    if (BMODE == B_ROWSEG) {
        const int ky = (int)fastdiv((unsigned)k, a.fd_seg_pad), j0 = k - ky * a.seg_pad;
        const int iy = iy0 + ky * g.dil_h;
        if ((unsigned)iy >= (unsigned)g.in_h)
            return r;
        // valid bytes of this chunk: those whose input column lies inside the image
        const int row_lo = -ix0 * g.in_c, row_hi = (g.in_w - ix0) * g.in_c; // j range inside the image
        const int nlo = min(max(row_lo - j0, 0), 16), nhi = min(max(row_hi - j0, 0), 16);
        if (nlo >= nhi)
            return r;
        const long long off = img_off + ((long long)iy * g.in_w + ix0) * g.in_c + j0;
        if (off >= 0 && off + 16 <= a.in_bytes) {
            __builtin_memcpy(&r, a.in + off, 16);
            if (nlo > 0 || nhi < 16) {
#pragma unroll
                for (int w = 0; w < 4; w++) {
                    const int hi_n = min(max(nhi - 4 * w, 0), 4), lo_n = min(max(nlo - 4 * w, 0), 4);
                    const unsigned hi_m = hi_n >= 4 ? 0xffffffffu : ((1u << (8 * hi_n)) - 1u);
                    const unsigned lo_m = lo_n >= 4 ? 0xffffffffu : ((1u << (8 * lo_n)) - 1u);
                    r[w] = (int)((unsigned)r[w] & hi_m & ~lo_m);
                }
            }
        } else {
            unsigned int words[4] = {0, 0, 0, 0};
            const int stop = min(nhi, a.seg_len - j0);
            for (int b = nlo; b < stop; b++)
                words[b >> 2] |= (unsigned int)(unsigned char)a.in[off + b] << ((b & 3) * 8);
            r = v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
        }
        return r;
    }
    // B_GATHER
    unsigned int words[4] = {0, 0, 0, 0};
    int tap = (int)fastdiv((unsigned)k, a.fd_in_c), c = k - tap * g.in_c;
    int ky = (int)fastdiv((unsigned)tap, a.fd_k_w), kx = tap - ky * g.k_w;
    const int n = min(16, a.K - k);
    for (int b = 0; b < n; b++) {
        const int iy = iy0 + ky * g.dil_h, ix = ix0 + kx * g.dil_w;
        if ((unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w) {
            const unsigned char v = (unsigned char)a.in[img_off + ((long long)iy * g.in_w + ix) * g.in_pitch + c];
            words[b >> 2] |= (unsigned int)v << ((b & 3) * 8);
        }
        if (++c == g.in_c) {
            c = 0;
            if (++kx == g.k_w) {
                kx = 0;
                ++ky;
            }
        }
    }
    return v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
}

// Output pixel of one lane in one of the wave's pixel tiles.
struct PixelRef {
    unsigned int pix;
    long long img_off;
    int iy0, ix0;
    bool valid;
};

template <int BMODE, int PT>
__device__ __forceinline__ void decode_set(const MfmaConvArgs &a, int set, int wave, int col, PixelRef (&px)[PT])
{
    const ConvGeom &g = a.g;
    const long long img_bytes = (long long)g.in_h * g.in_w * g.in_pitch;
#pragma unroll
    for (int p = 0; p < PT; p++) {
        const unsigned int pix = ((unsigned)set * 4u + (unsigned)wave) * (16u * PT) + p * 16 + col;
        px[p].pix = pix;
        px[p].valid = (long long)pix < a.npix;
        if (BMODE == B_POINT) {
            // flat pointwise: output pixel i reads input pixel i, no coordinates needed
            px[p].img_off = (long long)pix * g.in_pitch;
            px[p].iy0 = px[p].ix0 = 0;
            continue;
        }
        const unsigned int pc = px[p].valid ? pix : 0u;
        const unsigned int n = fastdiv(pc, a.fd_out_hw);
        const unsigned int rem = pc - n * a.fd_out_hw.d;
        const unsigned int oy = fastdiv(rem, a.fd_out_w);
        const unsigned int ox = rem - oy * a.fd_out_w.d;
        px[p].img_off = (long long)n * img_bytes;
        px[p].iy0 = (int)oy * g.stride_h - g.pad_top;
        px[p].ix0 = (int)ox * g.stride_w - g.pad_left;
    }
}

template <int BMODE, int PT, int KSC>
__device__ __forceinline__ void load_all_b(const MfmaConvArgs &a, const PixelRef (&px)[PT], int quad,
                                           v4i (&bc)[PT][KSC > 0 ? KSC : 1])
{
#pragma unroll
    for (int ks = 0; ks < KSC; ks++)
#pragma unroll
        for (int p = 0; p < PT; p++)
            bc[p][ks] = load_b<BMODE>(a, px[p].valid && ks < a.ksteps, px[p].img_off, px[p].iy0, px[p].ix0,
                                      ks * 64 + quad * 16);
}

// Everything a wave needs while it walks pixel sets.
struct WaveCtx {
    const v4i *wts;
    const int *init_l, *shift_l, *lsh_l;
    const int8_t *lut_l;
    unsigned char *my_tile;
    int lane, col, quad;
    bool relu, half_even, has_lut, stage_out;
    int floor_pk; // lower clamp of the short epilogue as two int16: 0 (ReLU) or 0x80008000
};

// One group of NT filter tiles (16*NT filters) for the wave's PT pixel tiles: MFMA over the K steps
// resident in registers (KSC > 0) or streamed (KSC == 0), then the epilogue.  NT is a compile-time
// constant so that the tile loops carry no run-time tests.
template <int BMODE, int PT, int KSC, bool FAST, int USE_LSH, int NT>
__device__ __forceinline__ void run_group(const MfmaConvArgs &a, const WaveCtx &w, const PixelRef (&px)[PT],
                                          const v4i (&bc)[PT][KSC > 0 ? KSC : 1], int gi, int gbase, int g_first,
                                          int g_count)
{
    const int OC = a.g.out_c;
    const int c_local = gi * 64 + 4 * NT * w.quad;
    v4i acc[PT][NT];
    v4i start[NT];
#pragma unroll
    for (int t = 0; t < NT; t++)
        start[t] = *reinterpret_cast<const v4i *>(w.init_l + c_local + 4 * t);

    if constexpr (KSC > 0) {
        // k step 0 always exists: it takes the start vector as its C operand (no register copies)
        {
            const v4i *wt = w.wts + ((gi * a.ks_per_chunk) * 4) * 64 + w.lane;
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const v4i aop = wt[t * 64];
#pragma unroll
                for (int p = 0; p < PT; p++)
                    acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, bc[p][0], start[t], 0, 0, 0);
            }
        }
#pragma unroll
        for (int ks = 1; ks < KSC; ks++) {
            if (ks < a.ksteps) {
                const v4i *wt = w.wts + ((gi * a.ks_per_chunk + ks) * 4) * 64 + w.lane;
#pragma unroll
                for (int t = 0; t < NT; t++) {
                    const v4i aop = wt[t * 64];
#pragma unroll
                    for (int p = 0; p < PT; p++)
                        acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, bc[p][ks], acc[p][t], 0, 0, 0);
                }
            }
        }
    } else {
#pragma unroll
        for (int t = 0; t < NT; t++)
#pragma unroll
            for (int p = 0; p < PT; p++)
                acc[p][t] = start[t];
        for (int kc = 0; kc < a.n_kchunks; kc++) {
            const int ks_begin = kc * a.ks_per_chunk;
            const int ks_count = min(a.ks_per_chunk, a.ksteps - ks_begin);
            if (a.n_kchunks > 1) {
                __syncthreads(); // everyone is done with the previous chunk
                stage_weights(a, const_cast<v4i *>(w.wts), g_first, g_count, ks_begin, ks_count);
                __syncthreads();
            }
            const int ks_stride = a.n_kchunks > 1 ? ks_count : a.ks_per_chunk;
            for (int ks0 = 0; ks0 < ks_count; ks0 += 4) {
                v4i b[4][PT];
#pragma unroll
                for (int j = 0; j < 4; j++)
#pragma unroll
                    for (int p = 0; p < PT; p++)
                        b[j][p] = load_b<BMODE>(a, px[p].valid && ks0 + j < ks_count, px[p].img_off, px[p].iy0, px[p].ix0,
                                                (ks_begin + ks0 + j) * 64 + w.quad * 16);
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    if (ks0 + j < ks_count) {
                        const v4i *wt = w.wts + ((gi * ks_stride + ks0 + j) * 4) * 64 + w.lane;
#pragma unroll
                        for (int t = 0; t < NT; t++) {
                            const v4i aop = wt[t * 64];
#pragma unroll
                            for (int p = 0; p < PT; p++)
                                acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, b[j][p], acc[p][t], 0, 0, 0);
                        }
                    }
                }
            }
        }
    }

    // epilogue: this lane owns output channels [c_lane, c_lane + 4*NT) of pixel px[p].pix
    const int c_lane = gbase + 4 * NT * w.quad;
    v4i ss[NT], ls[NT];
#pragma unroll
    for (int t = 0; t < NT; t++) {
        ss[t] = *reinterpret_cast<const v4i *>(w.shift_l + c_local + 4 * t);
        ls[t] = USE_LSH ? *reinterpret_cast<const v4i *>(w.lsh_l + c_local + 4 * t) : v4i{0, 0, 0, 0};
    }
#pragma unroll
    for (int p = 0; p < PT; p++) {
        int words[NT];
#pragma unroll
        for (int t = 0; t < NT; t++) {
            if constexpr (FAST) {
                words[t] = pack_fast4<USE_LSH>(acc[p][t], ls[t], ss[t], w.floor_pk);
            } else {
                int q[4];
#pragma unroll
                for (int r = 0; r < 4; r++)
                    q[r] = requant_s8(acc[p][t][r], ss[t][r], w.relu, w.half_even);
                words[t] = pack4_s8(q[0], q[1], q[2], q[3]);
            }
        }
        if (w.has_lut) {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                const int v = words[t];
                words[t] = pack4_s8(w.lut_l[(int)(int8_t)v + 128], w.lut_l[(int)(int8_t)(v >> 8) + 128],
                                    w.lut_l[(int)(int8_t)(v >> 16) + 128], w.lut_l[(v >> 24) + 128]);
            }
        }
        if (w.stage_out) {
            // collect in LDS, laid out exactly like the global block the wave will write
            unsigned char *dst = w.my_tile + (p * 16 + w.col) * OC + c_lane;
            if (NT == 4 && a.out_vec == 16) {
                *reinterpret_cast<v4i *>(dst) = v4i{words[0], words[NT > 1 ? 1 : 0], words[NT > 2 ? 2 : 0], words[NT > 3 ? 3 : 0]};
            } else {
#pragma unroll
                for (int t = 0; t < NT; t++)
                    if (c_lane + 4 * t < OC)
                        *reinterpret_cast<int *>(dst + 4 * t) = words[t];
            }
            continue;
        }
        if (!px[p].valid)
            continue;
        const long long goff = (long long)px[p].pix * a.g.out_pitch + c_lane;  // output and residual operand may be
        const long long roff = (long long)px[p].pix * a.g.res_pitch + c_lane; // channel slices of wider tensors
        int8_t *dst = a.out + goff;
        // Stores (and residual loads) take the widest piece that exists: 16 bytes when the lane's 16 channels do,
        // else 4 bytes per filter tile, single bytes only for the last channels of a row.  No piece needs an
        // aligned address, so a channel count that is not a multiple of 4 costs nothing but the row tails.
        if (NT == 4 && c_lane + 16 <= OC) {
            v4i v = {words[0], words[NT > 1 ? 1 : 0], words[NT > 2 ? 2 : 0], words[NT > 3 ? 3 : 0]};
            if (a.res != nullptr) {
                const v4i r = *reinterpret_cast<const v4i_unaligned *>(a.res + roff);
#pragma unroll
                for (int d = 0; d < 4; d++)
                    v[d] = sat_add4_s8(v[d], r[d]);
            }
            *reinterpret_cast<v4i_unaligned *>(dst) = v;
        } else {
#pragma unroll
            for (int t = 0; t < NT; t++) {
                if (c_lane + 4 * t + 4 <= OC) {
                    int v = words[t];
                    if (a.res != nullptr)
                        v = sat_add4_s8(v, *reinterpret_cast<const int_unaligned *>(a.res + roff + 4 * t));
                    *reinterpret_cast<int_unaligned *>(dst + 4 * t) = v;
                } else {
                    for (int r = 0; r < 4; r++)
                        if (c_lane + 4 * t + r < OC) {
                            int v = (int)(int8_t)(words[t] >> (8 * r));
                            if (a.res != nullptr)
                                v = clamp_s8(v + (int)a.res[roff + 4 * t + r]);
                            dst[4 * t + r] = (int8_t)v;
                        }
                }
            }
        }
    }
}

// The persistent loop over pixel sets with one epilogue flavour compiled in.
template <int BMODE, int PT, int KSC, bool FAST, int USE_LSH>
__device__ __forceinline__ void run_sets(const MfmaConvArgs &a, const WaveCtx &w, int wave, int g_first, int g_count,
                                         const TileSeq &seq, PixelRef (&px)[PT], v4i (&bc)[PT][KSC > 0 ? KSC : 1])
{
    constexpr bool kDoubleBuffer = KSC > 0 && KSC * PT <= 16;
    const int OC = a.g.out_c;
    for (int set = seq.first; set < seq.end; set += seq.step) {
        if constexpr (KSC == 0)
            decode_set<BMODE, PT>(a, set, wave, w.col, px);
        // operands of the next pixel set: issued now, consumed in the next iteration
        PixelRef px_next[PT];
        v4i bn[PT][kDoubleBuffer ? KSC : 1];
        const int set_next = set + seq.step;
        if constexpr (kDoubleBuffer) {
            if (set_next < seq.end) {
                decode_set<BMODE, PT>(a, set_next, wave, w.col, px_next);
                load_all_b<BMODE, PT, KSC>(a, px_next, w.quad, bn);
            }
        }

        for (int gi = 0; gi < g_count; gi++) {
            const int gbase = (g_first + gi) * 64;
            switch (group_tiles(OC, gbase)) { // uniform
            case 4:
                run_group<BMODE, PT, KSC, FAST, USE_LSH, 4>(a, w, px, bc, gi, gbase, g_first, g_count);
                break;
            case 3:
                run_group<BMODE, PT, KSC, FAST, USE_LSH, 3>(a, w, px, bc, gi, gbase, g_first, g_count);
                break;
            case 2:
                run_group<BMODE, PT, KSC, FAST, USE_LSH, 2>(a, w, px, bc, gi, gbase, g_first, g_count);
                break;
            default:
                run_group<BMODE, PT, KSC, FAST, USE_LSH, 1>(a, w, px, bc, gi, gbase, g_first, g_count);
                break;
            }
        }

        if (w.stage_out) {
            // the wave's 16*PT pixels x out_c bytes are one contiguous block of the NHWC output
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const unsigned int pix0 = ((unsigned)set * 4u + (unsigned)wave) * (16u * PT);
            const long long first = (long long)pix0 * OC;
            const long long total = (long long)a.npix * OC;
            const int tile_bytes = 16 * PT * OC; // multiple of 16
            int8_t *gdst = a.out + first;
            for (int off = w.lane * 16; off < tile_bytes; off += 64 * 16) {
                if (first + off + 16 <= total) {
                    v4i v = *reinterpret_cast<const v4i *>(w.my_tile + off);
                    if (a.res != nullptr) {
                        const v4i r = *reinterpret_cast<const v4i *>(a.res + first + off);
#pragma unroll
                        for (int d = 0; d < 4; d++)
                            v[d] = sat_add4_s8(v[d], r[d]);
                    }
                    *reinterpret_cast<v4i *>(gdst + off) = v;
                } else {
                    for (int b = 0; b < 16; b++)
                        if (first + off + b < total) {
                            int v = (int)(int8_t)w.my_tile[off + b];
                            if (a.res != nullptr)
                                v = clamp_s8(v + (int)a.res[first + off + b]);
                            gdst[off + b] = (int8_t)v;
                        }
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }

        if constexpr (KSC > 0) {
            if constexpr (kDoubleBuffer) {
#pragma unroll
                for (int p = 0; p < PT; p++) {
                    px[p] = px_next[p];
#pragma unroll
                    for (int ks = 0; ks < KSC; ks++)
                        bc[p][ks] = bn[p][ks];
                }
            } else if (set_next < a.n_sets) {
                decode_set<BMODE, PT>(a, set_next, wave, w.col, px);
                load_all_b<BMODE, PT, KSC>(a, px, w.quad, bc);
            }
        }
    }
}

// KSC > 0: the whole reduction axis (at most KSC k steps) is held in registers per pixel tile.
// KSC == 0: k steps are streamed four at a time (any K, including K chunks re-staged in LDS).
// HE: the round-half-even build of the kernel.  A separate kernel, not one more branch of this one: the
// register allocation of a kernel is that of its heaviest branch, and the half-even epilogue would cost
// the half-up build a wavefront of occupancy.
template <int BMODE, int PT, int KSC, bool HE>
__global__ __launch_bounds__(kThreads) void conv2d_s8_mfma_kernel(const MfmaConvArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int gpc = a.groups_per_chunk;
    v4i *wts = reinterpret_cast<v4i *>(smem);
    int *init_l = reinterpret_cast<int *>(smem + (size_t)gpc * a.ks_per_chunk * 4096); // accumulator start value
    int *shift_l = init_l + gpc * 64; // short epilogue: right shift max(0, s-8); general epilogue: the raw shift
    int *lsh_l = shift_l + gpc * 64;  // short epilogue: left shift max(0, 8-s)
    int8_t *lut_l = reinterpret_cast<int8_t *>(lsh_l + gpc * 64);
    unsigned char *out_tiles = reinterpret_cast<unsigned char *>(lut_l + 256); // stage_out: 4 waves x 16*PT*out_c

    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int OC = g.out_c;
    const int g_first = blockIdx.y * gpc;
    const int g_count = min(gpc, a.n_groups - g_first);
    const bool half_even = g.half_even != 0, has_lut = a.lut != nullptr;

    // first pixel set: get its operand loads going before anything else
    PixelRef px[PT];
    v4i bc[PT][KSC > 0 ? KSC : 1];
    const TileSeq seq = xcd_tile_sequence(a.n_sets);
    const int set = seq.first;
    if constexpr (KSC > 0) {
        if (set < seq.end) {
            decode_set<BMODE, PT>(a, set, wave, col, px);
            load_all_b<BMODE, PT, KSC>(a, px, quad, bc);
        }
    }

    // Can this workgroup's filters take the short epilogue?  Every shift in 1..31, and the sum
    // bias + 2^(s-1) + (k_h*k_w*in_c products of at most 2^14) must fit int32 even after the left
    // shift by max(0, 8-s) that the short form applies.
    const long long mac_bound = (long long)g.k_h * g.k_w * g.in_c * 16384;
    int ok_local = 1;
    int lsh_local = 0;
    for (int c = tid; c < g_count * 64; c += kThreads) {
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
        lut_l[tid] = a.lut[tid];
    if (a.n_kchunks == 1)
        stage_weights(a, wts, g_first, g_count, 0, a.ksteps);
    const bool fast = __syncthreads_and(ok_local) != 0;
    const bool use_lsh = __syncthreads_or(lsh_local) != 0;
    for (int c = tid; c < g_count * 64; c += kThreads) {
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
    __syncthreads();

    WaveCtx w;
    w.wts = wts;
    w.init_l = init_l;
    w.shift_l = shift_l;
    w.lsh_l = lsh_l;
    w.lut_l = lut_l;
    w.my_tile = out_tiles + (size_t)wave * (16 * PT) * OC;
    w.lane = lane;
    w.col = col;
    w.quad = quad;
    w.relu = g.relu != 0;
    w.half_even = half_even;
    w.has_lut = has_lut;
    w.floor_pk = w.relu ? 0 : (int)0x80008000u;
    w.stage_out = a.stage_out != 0;
    // epilogue mode of pack_fast4: 0 plain (every shift >= 8), 1 with the left shift, 5 the same with
    // round-half-even
    if (HE) {
        if (fast)
            run_sets<BMODE, PT, KSC, true, 5>(a, w, wave, g_first, g_count, seq, px, bc);
        else
            run_sets<BMODE, PT, KSC, false, 0>(a, w, wave, g_first, g_count, seq, px, bc);
    } else {
        if (fast && !use_lsh)
            run_sets<BMODE, PT, KSC, true, 0>(a, w, wave, g_first, g_count, seq, px, bc);
        else if (fast)
            run_sets<BMODE, PT, KSC, true, 1>(a, w, wave, g_first, g_count, seq, px, bc);
        else
            run_sets<BMODE, PT, KSC, false, 0>(a, w, wave, g_first, g_count, seq, px, bc);
    }
}

// What the host planner knows; the grid itself is sized per kernel variant from the number of
// workgroups of that variant a CU can hold (registers and LDS), so that the persistent grid is
// resident all at once: a grid larger than that would run in rounds, the last one partly empty.
struct GridPlan {
    int cus;      // compute units of the device
    int n_chunks; // filter chunks = gridDim.y
};

template <int BMODE, int PT, int KSC, bool HE>
hipError_t launch_variant_he(const MfmaConvArgs &a, GridPlan plan, size_t lds, hipStream_t stream)
{
    const int per_cu = resident_workgroups_per_cu(conv2d_s8_mfma_kernel<BMODE, PT, KSC, HE>, kThreads, lds);
    int gx = max(1, (plan.cus * per_cu) / plan.n_chunks);
    if (gx > a.n_sets)
        gx = a.n_sets;
    if (gx >= 8)
        gx &= ~7; // blockIdx.x % 8 is then the XCD of a workgroup, for every blockIdx.y
    hipLaunchKernelGGL((conv2d_s8_mfma_kernel<BMODE, PT, KSC, HE>), dim3((unsigned)gx, (unsigned)plan.n_chunks),
                       dim3(kThreads), lds, stream, a);
    return hipGetLastError();
}

template <int BMODE, int PT, int KSC>
hipError_t launch_variant(const MfmaConvArgs &a, GridPlan plan, size_t lds, hipStream_t stream)
{
    return a.g.half_even ? launch_variant_he<BMODE, PT, KSC, true>(a, plan, lds, stream)
                         : launch_variant_he<BMODE, PT, KSC, false>(a, plan, lds, stream);
}

// Smallest register-resident variant that holds `ksteps` k steps (0 = streamed).
inline int pick_ksc(int ksteps)
{
    static const int sizes[] = {1, 2, 3, 4, 6, 9, 12, 16, 20};
    for (int s : sizes)
        if (ksteps <= s)
            return s;
    return 0;
}

template <int BMODE, int PT>
hipError_t launch_ksc(const MfmaConvArgs &a, int ksc, GridPlan grid, size_t lds, hipStream_t stream)
{
    switch (ksc) {
    case 1:
        return launch_variant<BMODE, PT, 1>(a, grid, lds, stream);
    case 2:
        return launch_variant<BMODE, PT, 2>(a, grid, lds, stream);
    case 3:
        return launch_variant<BMODE, PT, 3>(a, grid, lds, stream);
    case 4:
        return launch_variant<BMODE, PT, 4>(a, grid, lds, stream);
    case 6:
        return launch_variant<BMODE, PT, 6>(a, grid, lds, stream);
    case 9:
        return launch_variant<BMODE, PT, 9>(a, grid, lds, stream);
    case 12:
        return launch_variant<BMODE, PT, 12>(a, grid, lds, stream);
    case 16:
        return launch_variant<BMODE, PT, 16>(a, grid, lds, stream);
    case 20:
        return launch_variant<BMODE, PT, 20>(a, grid, lds, stream);
    default:
        return launch_variant<BMODE, PT, 0>(a, grid, lds, stream);
    }
}

// Per operand-B mode entry points, each compiled in its own translation unit.
hipError_t launch_vec16(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream);
hipError_t launch_point(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream);
hipError_t launch_rowseg(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream);
hipError_t launch_gather(const MfmaConvArgs &a, int pt, int ksc, GridPlan grid, size_t lds, hipStream_t stream);

} // namespace mfma_conv
} // namespace espdl
