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
// stride.  If 64 filters x K do not fit the LDS budget, K is processed in chunks that are re-staged
// between barriers while the accumulators stay in registers.
#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

enum { B_VEC16 = 0, B_POINT = 1, B_GATHER = 2, B_ROWSEG = 3 };

constexpr int kThreads = 256;            // 4 wavefronts
constexpr int kLdsSoftBudget = 64 * 1024; // two workgroups per CU
constexpr int kLdsHardBudget = 64 * 1024; // one K chunk of one filter group never needs more

struct MfmaConvArgs {
    const int8_t *in;
    const int8_t *w;
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
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
};

__device__ __forceinline__ int group_tiles(int out_c, int gbase)
{
    const int rem = out_c - gbase;
    return rem >= 64 ? 4 : (rem + 15) >> 4;
}

// Copy one K chunk of `g_count` filter groups into LDS in MFMA operand-A order.
__device__ __forceinline__ void stage_weights(const MfmaConvArgs &a, v4i *wts, int g_first, int g_count, int ks_begin,
                                              int ks_count)
{
    const int units = g_count * ks_count * 256;
    const int OC = a.g.out_c, K = a.K;
    for (int u = threadIdx.x; u < units; u += kThreads) {
        const int l = u & 63, t = (u >> 6) & 3, rest = u >> 8;
        const int ks = rest % ks_count, gi = rest / ks_count;
        const int gbase = (g_first + gi) * 64;
        const int nt = group_tiles(OC, gbase);
        v4i val = {0, 0, 0, 0};
        if (t < nt) {
            const int i = l & 15, gk = l >> 4;
            const int oc = gbase + 4 * nt * (i >> 2) + 4 * t + (i & 3);
            const int k = (ks_begin + ks) * 64 + gk * 16;
            if (oc < OC && k < K && a.seg_pad > 0) {
                // (ky, j) ordering: filter row ky starts at k = ky * seg_pad and holds seg_len bytes
                const int ky = k / a.seg_pad, j0 = k - ky * a.seg_pad;
                const int8_t *src = a.w + ((size_t)oc * a.g.k_h + ky) * a.seg_len + j0;
                unsigned int words[4] = {0, 0, 0, 0};
                const int n = min(16, a.seg_len - j0);
                for (int b = 0; b < n; b++)
                    words[b >> 2] |= (unsigned int)(unsigned char)src[b] << ((b & 3) * 8);
                val = v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
            } else if (oc < OC && k < K) {
                const int8_t *src = a.w + (size_t)oc * K + k;
                if ((K & 15) == 0 && (reinterpret_cast<uintptr_t>(a.w) & 15) == 0) {
                    val = *reinterpret_cast<const v4i *>(src);
                } else {
                    unsigned int words[4] = {0, 0, 0, 0};
                    const int n = min(16, K - k);
                    for (int b = 0; b < n; b++)
                        words[b >> 2] |= (unsigned int)(unsigned char)src[b] << ((b & 3) * 8);
                    val = v4i{(int)words[0], (int)words[1], (int)words[2], (int)words[3]};
                }
            }
        }
        wts[u] = val;
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
        // iy0 / ix0 are the input coordinates themselves (no padding, single tap)
        const long long off = img_off + ((long long)iy0 * g.in_w + ix0) * g.in_c + k;
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
        const int tap = k / g.in_c, c0 = k - tap * g.in_c;
        const int ky = tap / g.k_w, kx = tap - ky * g.k_w;
        const int iy = iy0 + ky * g.dil_h, ix = ix0 + kx * g.dil_w;
        if ((unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w)
            r = *reinterpret_cast<const v4i *>(a.in + img_off + ((long long)iy * g.in_w + ix) * g.in_c + c0);
        return r;
    }
    if (BMODE == B_ROWSEG) {
        const int ky = k / a.seg_pad, j0 = k - ky * a.seg_pad;
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
    int tap = k / g.in_c, c = k - tap * g.in_c;
    int ky = tap / g.k_w, kx = tap - ky * g.k_w;
    const int n = min(16, a.K - k);
    for (int b = 0; b < n; b++) {
        const int iy = iy0 + ky * g.dil_h, ix = ix0 + kx * g.dil_w;
        if ((unsigned)iy < (unsigned)g.in_h && (unsigned)ix < (unsigned)g.in_w) {
            const unsigned char v = (unsigned char)a.in[img_off + ((long long)iy * g.in_w + ix) * g.in_c + c];
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

template <int BMODE, int PT, int KSC>
__global__ __launch_bounds__(kThreads) void conv2d_s8_mfma_kernel(const MfmaConvArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int gpc = a.groups_per_chunk;
    v4i *wts = reinterpret_cast<v4i *>(smem);
    int *init_l = reinterpret_cast<int *>(smem + (size_t)gpc * a.ks_per_chunk * 4096); // accumulator start value
    int *shift_l = init_l + gpc * 64; // fast epilogue: lsh | rsh << 8; general epilogue: the raw shift
    int8_t *lut_l = reinterpret_cast<int8_t *>(shift_l + gpc * 64);

    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const int OC = g.out_c;
    const int g_first = blockIdx.y * gpc;
    const int g_count = min(gpc, a.n_groups - g_first);
    const bool relu = g.relu != 0, half_even = g.half_even != 0, has_lut = a.lut != nullptr;

    // Can this workgroup's filters take the short epilogue?  Every shift in 1..31, and the sum
    // bias + 2^(s-1) + (k_h*k_w*in_c products of at most 2^14) must fit int32 even after the left
    // shift by max(0, 8-s) that the short form applies.
    const long long mac_bound = (long long)g.k_h * g.k_w * g.in_c * 16384;
    int ok_local = half_even ? 0 : 1;
    for (int c = tid; c < g_count * 64; c += kThreads) {
        const int oc = g_first * 64 + c;
        if (oc < OC) {
            const int s = a.shift[g.n_shift == 1 ? 0 : oc];
            const long long b = a.bias != nullptr ? (long long)a.bias[oc] : 0;
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
    for (int c = tid; c < g_count * 64; c += kThreads) {
        const int oc = g_first * 64 + c;
        int init = 0, sh = fast ? (8 << 8) : 0;
        if (oc < OC) {
            const int s = a.shift[g.n_shift == 1 ? 0 : oc];
            const int b = a.bias != nullptr ? a.bias[oc] : 0;
            init = fast ? b + (1 << (s - 1)) : b;
            sh = fast ? (max(0, 8 - s) | (max(0, s - 8) << 8)) : s;
        }
        init_l[c] = init;
        shift_l[c] = sh;
    }
    __syncthreads();

    const long long out_hw = (long long)g.out_h * g.out_w;
    const long long img_bytes = (long long)g.in_h * g.in_w * g.in_c;

    for (int set = blockIdx.x; set < a.n_sets; set += gridDim.x) {
        // this lane's output pixel in each of the wave's PT pixel tiles
        long long pix[PT], img_off[PT];
        int iy0[PT], ix0[PT];
        bool pv[PT];
#pragma unroll
        for (int p = 0; p < PT; p++) {
            pix[p] = ((long long)set * 4 + wave) * (16 * PT) + p * 16 + col;
            pv[p] = pix[p] < a.npix;
            const long long pc = pv[p] ? pix[p] : 0;
            const int n = (int)(pc / out_hw);
            const int rem = (int)(pc - (long long)n * out_hw);
            const int oy = rem / g.out_w, ox = rem - oy * g.out_w;
            img_off[p] = (long long)n * img_bytes;
            iy0[p] = oy * g.stride_h - g.pad_top;
            ix0[p] = ox * g.stride_w - g.pad_left;
        }

        v4i bc[PT][KSC > 0 ? KSC : 1];
        if (KSC > 0) {
#pragma unroll
            for (int ks = 0; ks < KSC; ks++)
#pragma unroll
                for (int p = 0; p < PT; p++)
                    bc[p][ks] = load_b<BMODE>(a, pv[p] && ks < a.ksteps, img_off[p], iy0[p], ix0[p], ks * 64 + quad * 16);
        }

        for (int gi = 0; gi < g_count; gi++) {
            const int gbase = (g_first + gi) * 64;
            const int nt = group_tiles(OC, gbase);
            // accumulators start at bias (+ rounding constant on the short path): integer addition
            // wraps associatively, so adding it first or last gives the same 32-bit value
            const int c_local = gi * 64 + 4 * nt * quad;
            v4i acc[PT][4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const v4i start = t < nt ? *reinterpret_cast<const v4i *>(init_l + c_local + 4 * t) : v4i{0, 0, 0, 0};
#pragma unroll
                for (int p = 0; p < PT; p++)
                    acc[p][t] = start;
            }

            if (KSC > 0) {
#pragma unroll
                for (int ks = 0; ks < KSC; ks++) {
                    if (ks < a.ksteps) {
                        const v4i *wt = wts + ((gi * a.ks_per_chunk + ks) * 4) * 64 + lane;
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            if (t < nt) {
                                const v4i aop = wt[t * 64];
#pragma unroll
                                for (int p = 0; p < PT; p++)
                                    acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, bc[p][ks], acc[p][t], 0, 0, 0);
                            }
                        }
                    }
                }
            } else {
                for (int kc = 0; kc < a.n_kchunks; kc++) {
                    const int ks_begin = kc * a.ks_per_chunk;
                    const int ks_count = min(a.ks_per_chunk, a.ksteps - ks_begin);
                    if (a.n_kchunks > 1) {
                        __syncthreads(); // everyone is done with the previous chunk
                        stage_weights(a, wts, g_first, g_count, ks_begin, ks_count);
                        __syncthreads();
                    }
                    const int ks_stride = a.n_kchunks > 1 ? ks_count : a.ks_per_chunk;
                    for (int ks = 0; ks < ks_count; ks++) {
                        v4i b[PT];
#pragma unroll
                        for (int p = 0; p < PT; p++)
                            b[p] = load_b<BMODE>(a, pv[p], img_off[p], iy0[p], ix0[p], (ks_begin + ks) * 64 + quad * 16);
                        const v4i *wt = wts + ((gi * ks_stride + ks) * 4) * 64 + lane;
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            if (t < nt) {
                                const v4i aop = wt[t * 64];
#pragma unroll
                                for (int p = 0; p < PT; p++)
                                    acc[p][t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, b[p], acc[p][t], 0, 0, 0);
                            }
                        }
                    }
                }
            }

            // epilogue: this lane owns output channels [c_lane, c_lane + 4*nt) of pixel pix[p]
            const int c_lane = gbase + 4 * nt * quad;
            v4i ss[4];
#pragma unroll
            for (int t = 0; t < 4; t++)
                ss[t] = t < nt ? *reinterpret_cast<const v4i *>(shift_l + c_local + 4 * t) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int p = 0; p < PT; p++) {
                int words[4];
#pragma unroll
                for (int t = 0; t < 4; t++) {
                    words[t] = 0;
                    if (t < nt) {
                        if (fast) {
                            int tv[4];
#pragma unroll
                            for (int r = 0; r < 4; r++) {
                                const int sh = ss[t][r];
                                int v = (int)((unsigned)acc[p][t][r] << (sh & 31)) >> (sh >> 8);
                                tv[r] = relu ? max(v, 0) : v;
                            }
                            const int p01 = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(tv[0], tv[1]));
                            const int p23 = __builtin_bit_cast(int, __builtin_amdgcn_cvt_pk_i16(tv[2], tv[3]));
                            words[t] = (int)__builtin_amdgcn_perm((unsigned)p23, (unsigned)p01, 0x07050301u);
                        } else {
                            int q[4];
#pragma unroll
                            for (int r = 0; r < 4; r++)
                                q[r] = requant_s8(acc[p][t][r], ss[t][r], relu, half_even);
                            words[t] = pack4_s8(q[0], q[1], q[2], q[3]);
                        }
                        if (has_lut) {
                            const int w = words[t];
                            words[t] = pack4_s8(lut_l[(int)(int8_t)w + 128], lut_l[(int)(int8_t)(w >> 8) + 128],
                                                lut_l[(int)(int8_t)(w >> 16) + 128], lut_l[(w >> 24) + 128]);
                        }
                    }
                }
                if (!pv[p])
                    continue;
                int8_t *dst = a.out + pix[p] * OC + c_lane;
                if (nt == 4 && a.out_vec == 16) {
                    *reinterpret_cast<v4i *>(dst) = v4i{words[0], words[1], words[2], words[3]};
                } else if (a.out_vec >= 4) {
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        if (t < nt && c_lane + 4 * t < OC)
                            *reinterpret_cast<int *>(dst + 4 * t) = words[t];
                } else {
#pragma unroll
                    for (int t = 0; t < 4; t++)
                        if (t < nt)
                            for (int r = 0; r < 4; r++)
                                if (c_lane + 4 * t + r < OC)
                                    dst[4 * t + r] = (int8_t)(words[t] >> (8 * r));
                }
            }
        }
    }
}

template <int BMODE, int PT, int KSC>
hipError_t launch_variant(const MfmaConvArgs &a, dim3 grid, size_t lds, hipStream_t stream)
{
    hipLaunchKernelGGL((conv2d_s8_mfma_kernel<BMODE, PT, KSC>), grid, dim3(kThreads), lds, stream, a);
    return hipGetLastError();
}

template <int BMODE, int PT>
hipError_t launch_ksc(const MfmaConvArgs &a, int ksc, dim3 grid, size_t lds, hipStream_t stream)
{
    switch (ksc) {
    case 1:
        return launch_variant<BMODE, PT, 1>(a, grid, lds, stream);
    case 2:
        return launch_variant<BMODE, PT, 2>(a, grid, lds, stream);
    case 3:
        return launch_variant<BMODE, PT, 3>(a, grid, lds, stream);
    default:
        return launch_variant<BMODE, PT, 0>(a, grid, lds, stream);
    }
}

template <int BMODE>
hipError_t launch_pt(const MfmaConvArgs &a, int pt, int ksc, dim3 grid, size_t lds, hipStream_t stream)
{
    return pt == 2 ? launch_ksc<BMODE, 2>(a, ksc, grid, lds, stream) : launch_ksc<BMODE, 1>(a, ksc, grid, lds, stream);
}

} // namespace

int conv2d_s8_mfma_max_k()
{
    return 1 << 24;
}

hipError_t launch_conv2d_s8_mfma(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                 const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count,
                                 hipStream_t stream)
{
    MfmaConvArgs a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.out = out;
    a.g = g;
    const bool aligned16 = ((reinterpret_cast<uintptr_t>(in) & 15) == 0);
    int bmode = B_GATHER;
    if ((g.in_c & 15) == 0 && aligned16)
        bmode = B_VEC16;
    else if (g.k_h == 1 && g.k_w == 1 && g.pad_top == 0 && g.pad_left == 0 && (g.out_h - 1) * g.stride_h < g.in_h &&
             (g.out_w - 1) * g.stride_w < g.in_w)
        bmode = B_POINT;
    else if (g.dil_w == 1)
        bmode = B_ROWSEG;
    a.seg_len = a.seg_pad = 0;
    a.K = g.k_h * g.k_w * g.in_c;
    if (bmode == B_ROWSEG) {
        a.seg_len = g.k_w * g.in_c;
        a.seg_pad = (a.seg_len + 15) & ~15;
        a.K = g.k_h * a.seg_pad;
    }
    a.ksteps = (a.K + 63) / 64;
    a.n_groups = (g.out_c + 63) / 64;
    a.npix = (long long)g.batch * g.out_h * g.out_w;
    a.in_bytes = (long long)g.batch * g.in_h * g.in_w * g.in_c;
    if (a.npix == 0)
        return hipSuccess;
    const uintptr_t out_addr = reinterpret_cast<uintptr_t>(out);
    a.out_vec = ((g.out_c & 15) == 0 && (out_addr & 15) == 0) ? 16 : (((g.out_c & 3) == 0 && (out_addr & 3) == 0) ? 4 : 1);

    // LDS plan: per resident filter group ksteps * 4 KiB of weights + 512 B of bias/shift, + 256 B LUT
    const int fixed = 256;
    const int per_group_full = a.ksteps * 4096 + 512;
    if (per_group_full + fixed <= kLdsHardBudget) {
        a.ks_per_chunk = a.ksteps;
        a.n_kchunks = 1;
        a.groups_per_chunk = min(a.n_groups, max(1, (kLdsSoftBudget - fixed) / per_group_full));
    } else {
        a.ks_per_chunk = (kLdsHardBudget - fixed - 512) / 4096;
        a.n_kchunks = (a.ksteps + a.ks_per_chunk - 1) / a.ks_per_chunk;
        a.groups_per_chunk = 1;
    }
    const int n_chunks = (a.n_groups + a.groups_per_chunk - 1) / a.groups_per_chunk;
    const size_t lds = (size_t)a.groups_per_chunk * (a.ks_per_chunk * 4096 + 512) + fixed;

    // 32 pixels per wave once there is enough work to keep every CU busy with the wider tile
    const int cus = cu_count > 0 ? cu_count : 256;
    const int pt = a.npix >= (long long)cus * 8 * 128 ? 2 : 1;
    a.n_sets = (int)((a.npix + 64 * pt - 1) / (64 * pt));
    const int ksc = (a.n_kchunks == 1 && a.ksteps <= 3) ? a.ksteps : 0;

    // persistent grid: about 4 workgroups per CU in total, gridDim.x a multiple of 8 so that the
    // workgroups that share a pixel set (same x, different filter chunk) land on the same XCD
    int gx = max(1, (cus * 4) / n_chunks);
    if (gx > a.n_sets)
        gx = a.n_sets;
    if (gx >= 8)
        gx &= ~7;
    dim3 grid((unsigned)gx, (unsigned)n_chunks, 1);

    switch (bmode) {
    case B_VEC16:
        return launch_pt<B_VEC16>(a, pt, ksc, grid, lds, stream);
    case B_POINT:
        return launch_pt<B_POINT>(a, pt, ksc, grid, lds, stream);
    case B_ROWSEG:
        return launch_pt<B_ROWSEG>(a, pt, ksc, grid, lds, stream);
    default:
        return launch_pt<B_GATHER>(a, pt, ksc, grid, lds, stream);
    }
}

} // namespace espdl
