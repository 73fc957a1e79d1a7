// Pointwise (1x1, stride 1, unpadded) int8 convolution / Gemm as a tiled GEMM for layers with few
// pixels per compute unit.
//
// What it computes is conv2d_11cn (esp-dl/dl/base/dl_base_conv2d.cpp:9-33) with the n_wise epilogue
// (esp-dl/dl/base/dl_base_activate_buffer.hpp:27-36, 61-72, 173-181, 201-210), exactly as the
// implicit-GEMM kernel in conv2d_s8_mfma_kernel.h does.
//
// Why a second kernel: the implicit-GEMM kernel keeps a whole 64-filter group (K x 64 bytes) resident
// in LDS per workgroup and walks pixel sets under it, which is right when a workgroup sees thousands of
// pixels.  At 14x14 and 7x7 a workgroup sees one or two pixel sets, and its time is the latency of
// staging up to 60 KB of filters before the first MFMA.  Here both operands stream through LDS in
// k steps of 64 with a register/LDS double buffer, so the first MFMA starts after one k step:
//   workgroup tile = 64*PT pixels x 64*NG filters, 4 wavefronts, wavefront = 16*PT pixels x all filters;
//   per k step: 64*PT x 64 B of pixels and 64*NG x 64 B of filters go global -> registers (one step
//   ahead) -> LDS rows of 96 bytes (a 16-byte-per-lane read is served in groups of 8 rows x 2 neighbouring
//   quarters; with a row pitch of twice an odd number of 16-byte units the 16 pieces of a group fall into
//   different bank sets, which a pitch of 80 bytes does not achieve);
//   one barrier per k step; MFMA operands are plain 16-byte LDS reads.
// The filter -> tile-row permutation (row i of tile t is filter 16*(i/4) + 4*t + i%4 of the group)
// leaves every lane with 16 consecutive output channels per pixel: one 16-byte store.
#include <type_traits>

#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {

namespace {

constexpr int kThreads = 256;
// LDS row of a tile: 64 k bytes + padding.  96 where LDS capacity allows it (conflict-free operand reads, see the
// head of the file); 80 for the four-image pooled build, whose 256-row pixel tile would otherwise leave two
// workgroups per compute unit instead of three (measured: 16.5 us at 80, 26.9 us at 96 on MobileNetV2's head).
template <int PT> constexpr int row_pitch = PT >= 4 ? 80 : 96;

struct PwArgs {
    const int8_t *in;  // [M][K]
    const int8_t *w;   // [N][K]
    const int32_t *bias;
    const int32_t *shift;
    const int8_t *lut;
    const int8_t *res;
    int8_t *out;       // [M][N]
    long long M;
    int K, N;
    int in_pitch, out_pitch, res_pitch; // bytes between consecutive rows of in, out and res (K, N, N when dense)
    int ksteps;
    int relu, half_even, n_shift;
    int out_vec; // 16, 4 or 1
    // WIN builds: a convolution with a window as the same product over gathered rows (im2col on the fly): row m is
    // output pixel m, its k bytes [tap][channel] come from the input pixels under the window (zeros outside the image)
    int w_in_h, w_in_w, w_in_c, w_k_w, w_stride_h, w_stride_w, w_dil_h, w_dil_w, w_pad_top, w_pad_left;
    FastDiv fd_ohw, fd_ow, fd_inc, fd_kw;
    int hw;          // GAP builds: pixels per image (at most 64)
    float gap_scale; // GAP builds: 2^in_exp / (h w) * 2^-out_exp of the pooling operator
};

// GAP: the convolution is followed by a GlobalAveragePool (base::avgpool2d_hwc with the filter covering the whole
// image, esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54) and only the pooled tensor [image][filter] is written.  A
// workgroup's pixel tile is then PT images of at most 64 pixels, 64 tile rows each: the convolution's int8
// results (requantized, activation applied, exactly what the separate operator would have stored) are summed
// over the image's pixels - over the 16 lanes of a pixel tile by rotations inside the row, over the four
// wavefronts through LDS - and the sum goes through the pooling operator's float scale and rounding.
// WIN: rows are gathered from under a convolution window (channels a multiple of 64, so that a k step of 64 lies
// inside one tap): what conv2d_33cn / conv2d_hwcn compute (esp-dl/dl/base/dl_base_conv2d.cpp:35-163) under
// conv_operation_shell's window clipping (esp-dl/dl/base/dl_base.hpp:940-1191).  For layers with few output pixels
// and a long reduction axis (the strided 3 x 3 convolutions deep in a detector's backbone), where a workgroup of
// the other kernels spends its time staging filters it uses for a handful of pixel sets.
template <int NG, int PT, bool GAP = false, bool K16 = true, bool WIN = false>
__global__ __launch_bounds__(kThreads) void conv2d_s8_pwgemm_kernel(const PwArgs a)
{
    constexpr int TN = 64 * NG;
    constexpr int kRow = row_pitch<PT>;
    constexpr int kTileM = 64 * PT; // pixels per workgroup, 16 * PT per wavefront
    constexpr int kPiecesB = kTileM * 4 / kThreads; // 16-byte pieces of the pixel tile per thread and k step (2)
    constexpr int kPiecesA = TN * 4 / kThreads;     // ... of the filter tile (1 or 2)
    __shared__ __align__(16) unsigned char b_l[2][kTileM * kRow];
    __shared__ __align__(16) unsigned char a_l[2][TN * kRow];
    __shared__ int cst[3][TN]; // start value | shift | left shift
    __shared__ int8_t lut_l[256];
    __shared__ int pool_l[GAP ? 4 : 1][GAP ? TN : 1]; // [wavefront][filter]: the wavefront's share of its image's sum

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const long long m0 = (long long)blockIdx.x * kTileM;
    // tile row -> pixel of the flat [M][K] input, or -1.  Pooled form: rows 64 i .. 64 i + hw - 1 are image
    // PT * blockIdx.x + i.
    auto row_pixel = [&](int r) -> long long {
        if constexpr (GAP) {
            const long long img = (long long)blockIdx.x * PT + (r >> 6);
            const int pix = r & 63;
            return (pix < a.hw && img * a.hw < a.M) ? img * a.hw + pix : -1;
        } else {
            return m0 + r < a.M ? m0 + r : -1;
        }
    };
    const int n0 = blockIdx.y * TN;
    const bool relu = a.relu != 0, half_even = a.half_even != 0, has_lut = a.lut != nullptr;

    // piece p of a tile: row p / 4, 16-byte quarter p % 4 of the 64-byte k step.  Rows whose length is not a
    // multiple of 16 (a Gemm over 120 features) are read with loads that need no alignment; the one piece that
    // holds a row's last n < 16 bytes is read as the 16 bytes that END at the row's end and shifted down, so
    // that nothing past a row (and so nothing past the tensor) is touched and the piece ends in zeros.
    // (K16 builds: rows of whole 16-byte pieces at aligned addresses)
    auto piece = [&](const int8_t *row, int k) -> v4i {
        if constexpr (K16)
            return k < a.K ? *reinterpret_cast<const v4i *>(row + k) : v4i{0, 0, 0, 0};
        if (k >= a.K)
            return v4i{0, 0, 0, 0};
        if (k + 16 <= a.K)
            return *reinterpret_cast<const v4i_unaligned *>(row + k);
        const v4i v = *reinterpret_cast<const v4i_unaligned *>(row + a.K - 16);
        const int sh = 16 - (a.K & 15); // uniform: bytes to shift down, 1..15
        const int d = sh >> 2;
        const unsigned b = (unsigned)(sh & 3);
        const int w[8] = {v[0], v[1], v[2], v[3], 0, 0, 0, 0};
        v4i r;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            int lo = 0, hi = 0;
#pragma unroll
            for (int j = 0; j < 4; j++) { // d is uniform: these are scalar choices
                lo = d == j ? w[i + j] : lo;
                hi = d == j ? w[i + j + 1] : hi;
            }
            r[i] = (int)__builtin_amdgcn_alignbyte((unsigned)hi, (unsigned)lo, b);
        }
        return r;
    };
    // WIN: where the window of this thread's rows starts in the input (row of piece slot j: (tid + j * kThreads) / 4)
    long long win_base[WIN ? kPiecesB : 1];
    int win_iy[WIN ? kPiecesB : 1], win_ix[WIN ? kPiecesB : 1];
    if constexpr (WIN) {
#pragma unroll
        for (int j = 0; j < kPiecesB; j++) {
            const long long m = row_pixel((tid + j * kThreads) >> 2);
            win_iy[j] = -0x40000000; // a row past the last: every tap is outside
            win_ix[j] = 0;
            win_base[j] = 0;
            if (m >= 0) {
                const unsigned n = fastdiv((unsigned)m, a.fd_ohw);
                const unsigned rem = (unsigned)m - n * a.fd_ohw.d;
                const unsigned oy = fastdiv(rem, a.fd_ow);
                const unsigned ox = rem - oy * a.fd_ow.d;
                win_iy[j] = (int)oy * a.w_stride_h - a.w_pad_top;
                win_ix[j] = (int)ox * a.w_stride_w - a.w_pad_left;
                win_base[j] = (((long long)n * a.w_in_h + win_iy[j]) * a.w_in_w + win_ix[j]) * a.in_pitch;
            }
        }
    }
    auto fetch = [&](int ks, v4i(&pb)[kPiecesB], v4i(&pa)[kPiecesA]) {
        const int k0 = 64 * ks;
        if constexpr (WIN) {
            // the tap and first channel of this k step (uniform)
            const unsigned tap = fastdiv((unsigned)k0, a.fd_inc);
            const int c0 = k0 - (int)tap * a.w_in_c;
            const unsigned ky = fastdiv(tap, a.fd_kw);
            const int dy = (int)ky * a.w_dil_h, dx = (int)(tap - ky * a.fd_kw.d) * a.w_dil_w;
            const long long tap_off = ((long long)dy * a.w_in_w + dx) * a.in_pitch + c0;
#pragma unroll
            for (int j = 0; j < kPiecesB; j++) {
                const int p = tid + j * kThreads;
                const bool ok = (unsigned)(win_iy[j] + dy) < (unsigned)a.w_in_h && (unsigned)(win_ix[j] + dx) < (unsigned)a.w_in_w;
                pb[j] = ok ? *reinterpret_cast<const v4i *>(a.in + win_base[j] + tap_off + 16 * (p & 3)) : v4i{0, 0, 0, 0};
            }
        } else {
#pragma unroll
            for (int j = 0; j < kPiecesB; j++) {
                const int p = tid + j * kThreads;
                const long long m = row_pixel(p >> 2);
                pb[j] = m >= 0 ? piece(a.in + m * a.in_pitch, k0 + 16 * (p & 3)) : v4i{0, 0, 0, 0};
            }
        }
#pragma unroll
        for (int j = 0; j < kPiecesA; j++) {
            const int p = tid + j * kThreads;
            const int n = n0 + (p >> 2);
            pa[j] = n < a.N ? piece(a.w + (long long)n * a.K, k0 + 16 * (p & 3)) : v4i{0, 0, 0, 0};
        }
    };
    auto stash = [&](int buf, const v4i(&pb)[kPiecesB], const v4i(&pa)[kPiecesA]) {
#pragma unroll
        for (int j = 0; j < kPiecesB; j++) {
            const int p = tid + j * kThreads;
            *reinterpret_cast<v4i *>(&b_l[buf][(p >> 2) * kRow + 16 * (p & 3)]) = pb[j];
        }
#pragma unroll
        for (int j = 0; j < kPiecesA; j++) {
            const int p = tid + j * kThreads;
            *reinterpret_cast<v4i *>(&a_l[buf][(p >> 2) * kRow + 16 * (p & 3)]) = pa[j];
        }
    };

    // two register sets: the operands of k step s+2 are requested while step s computes and are stored to LDS
    // at the end of step s+1, so a load has a whole k step (not just one step's few products) to arrive
    v4i pb[kPiecesB], pa[kPiecesA], pb2[kPiecesB], pa2[kPiecesA];
    fetch(0, pb, pa);
    if (a.ksteps > 1)
        fetch(1, pb2, pa2);

    // epilogue constants of the workgroup's filters; the short form needs every shift in 1..31 and no
    // possible overflow of bias + 2^(s-1) + K products
    const long long mac_bound = (long long)a.K * 16384;
    int ok_local = 1;
    int my_s = 0, my_b = 0;
    if (tid < TN) {
        const int n = n0 + tid;
        if (n < a.N) {
            my_s = a.shift[a.n_shift == 1 ? 0 : n];
            my_b = a.bias != nullptr ? a.bias[n] : 0;
            if (my_s < 1 || my_s > 31) {
                ok_local = 0;
            } else {
                const long long start = (long long)my_b + (1ll << (my_s - 1));
                if ((start < 0 ? -start : start) + mac_bound >= (1ll << (31 - max(0, 8 - my_s))))
                    ok_local = 0;
            }
        }
    }
    if (has_lut)
        lut_l[tid] = a.lut[tid];
    const bool fast = __syncthreads_and(ok_local) != 0;
    if (tid < TN) {
        const bool valid = n0 + tid < a.N;
        cst[0][tid] = (fast && valid) ? my_b + (1 << (my_s - 1)) - (half_even ? 1 : 0) : my_b; // mode 5 starts one lower
        cst[1][tid] = fast ? max(0, my_s - 8) : my_s;
        cst[2][tid] = fast ? max(0, 8 - my_s) : 0;
    }
    stash(0, pb, pa);
    if (a.ksteps > 2)
        fetch(2, pb, pa);
    __syncthreads();

    // accumulators: 2 pixel tiles x 4*NG filter tiles, started at bias (+ rounding constant)
    v4i acc[PT][4 * NG];
#pragma unroll
    for (int g = 0; g < NG; g++)
#pragma unroll
        for (int t = 0; t < 4; t++) {
            // rows 4*quad .. 4*quad+3 of tile t are filters 64*g + 16*quad + 4*t + r
            v4i init = *reinterpret_cast<const v4i *>(&cst[0][64 * g + 16 * quad + 4 * t]);
            if constexpr (GAP) { // pooled form: the operands swap roles, a lane holds four pixels of ONE filter
                const int i1 = cst[0][64 * g + 16 * (col >> 2) + (col & 3) + 4 * t];
                init = v4i{i1, i1, i1, i1};
            }
#pragma unroll
            for (int c = 0; c < PT; c++)
                acc[c][4 * g + t] = init;
        }

    // operand A row of this lane in tile t of group g: filter 64*g + 16*(col/4) + 4*t + col%4
    const int a_row0 = 16 * (col >> 2) + (col & 3);
    auto products = [&](int buf) {
        v4i b[PT];
#pragma unroll
        for (int c = 0; c < PT; c++)
            b[c] = *reinterpret_cast<const v4i *>(&b_l[buf][(16 * PT * wave + 16 * c + col) * kRow + 16 * quad]);
#pragma unroll
        for (int g = 0; g < NG; g++)
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const v4i aop = *reinterpret_cast<const v4i *>(&a_l[buf][(64 * g + a_row0 + 4 * t) * kRow + 16 * quad]);
#pragma unroll
                for (int c = 0; c < PT; c++) {
                    if constexpr (GAP) // rows = pixels, columns = filters: the sum over pixels stays inside a lane
                        acc[c][4 * g + t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b[c], aop, acc[c][4 * g + t], 0, 0, 0);
                    else
                        acc[c][4 * g + t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop, b[c], acc[c][4 * g + t], 0, 0, 0);
                }
            }
    };
    // Step ks reads LDS buffer ks & 1.  At its end the operands of step ks + 1 (held in registers since step
    // ks - 1) go to the other buffer, which was last read in step ks - 1 (every wavefront finished that before
    // the barrier at its end), and the registers they leave take the request for step ks + 3 ... the loop is
    // unrolled by two so that the two register sets keep their names.
    for (int ks = 0; ks < a.ksteps; ks += 2) {
        products(0);
        if (ks + 1 < a.ksteps) {
            stash(1, pb2, pa2);
            if (ks + 3 < a.ksteps)
                fetch(ks + 3, pb2, pa2);
            __syncthreads();
            products(1);
            if (ks + 2 < a.ksteps) {
                stash(0, pb, pa);
                if (ks + 4 < a.ksteps)
                    fetch(ks + 4, pb, pa);
                __syncthreads();
            }
        }
    }

    // epilogue: lane (col, quad) holds, per pixel tile and group, filters 64*g + 16*quad + [0, 16)
    const int floor_pk = relu ? 0 : (int)0x80008000u;
    // one straight-line copy per rounding mode (pack_fast4 mode 1: half up, 5: half even)
    auto epilogue = [&](auto mode) {
    #pragma unroll
        for (int c = 0; c < PT; c++) {
            const long long m = m0 + 16 * PT * wave + 16 * c + col;
    #pragma unroll
            for (int g = 0; g < NG; g++) {
                const int n = n0 + 64 * g + 16 * quad;
                int words[4];
    #pragma unroll
                for (int t = 0; t < 4; t++) {
                    const v4i ss = *reinterpret_cast<const v4i *>(&cst[1][64 * g + 16 * quad + 4 * t]);
                    if (fast) {
                        const v4i ls = *reinterpret_cast<const v4i *>(&cst[2][64 * g + 16 * quad + 4 * t]);
                        words[t] = pack_fast4<decltype(mode)::value>(acc[c][4 * g + t], ls, ss, floor_pk);
                    } else {
                        int q[4];
    #pragma unroll
                        for (int r = 0; r < 4; r++)
                            q[r] = requant_s8(acc[c][4 * g + t][r], ss[r], relu, half_even);
                        words[t] = pack4_s8(q[0], q[1], q[2], q[3]);
                    }
                    if (has_lut) {
                        const int v = words[t];
                        words[t] = pack4_s8(lut_l[(int)(int8_t)v + 128], lut_l[(int)(int8_t)(v >> 8) + 128],
                                            lut_l[(int)(int8_t)(v >> 16) + 128], lut_l[(v >> 24) + 128]);
                    }
                }
                if (m >= a.M || n >= a.N)
                    continue;
                const long long goff = m * a.out_pitch + n, roff = m * a.res_pitch + n;
                // the widest piece that exists, at any byte address: 16 bytes, else 4 per filter tile, bytes for
                // the last channels of a row (a row length that is not a multiple of 4 costs only those)
                if (n + 16 <= a.N) {
                    v4i v = {words[0], words[1], words[2], words[3]};
                    if (a.res != nullptr) {
                        const v4i r = *reinterpret_cast<const v4i_unaligned *>(a.res + roff);
    #pragma unroll
                        for (int d = 0; d < 4; d++)
                            v[d] = sat_add4_s8(v[d], r[d]);
                    }
                    if (a.out_vec == 16)
                        __builtin_nontemporal_store(v, reinterpret_cast<v4i *>(a.out + goff));
                    else
                        *reinterpret_cast<v4i_unaligned *>(a.out + goff) = v;
                } else {
    #pragma unroll
                    for (int t = 0; t < 4; t++) {
                        if (n + 4 * t + 4 <= a.N) {
                            int v = words[t];
                            if (a.res != nullptr)
                                v = sat_add4_s8(v, *reinterpret_cast<const int_unaligned *>(a.res + roff + 4 * t));
                            *reinterpret_cast<int_unaligned *>(a.out + goff + 4 * t) = v;
                        } else {
                            for (int r = 0; r < 4; r++)
                                if (n + 4 * t + r < a.N) {
                                    int v = (int)(int8_t)(words[t] >> (8 * r));
                                    if (a.res != nullptr)
                                        v = clamp_s8(v + (int)a.res[roff + 4 * t + r]);
                                    a.out[goff + 4 * t + r] = (int8_t)v;
                                }
                        }
                    }
                }
            }
        }
    };
    // Pooled form: lane (col, quad) holds pixels 4 quad + [0, 4) of every pixel tile for filter a_row0 + 4 t of the
    // group.  The four results of a tile are requantized with the lane's one set of constants, brought down to
    // their int8 value inside the int16 pairs (packed shift by 8), masked where the tile row is past the image,
    // and summed as packed int16 (at most 8 PT values of magnitude <= 128 per half).
    auto pooled = [&](auto mode) {
        constexpr int MODE = decltype(mode)::value; // 1: half up, 5: half even, -1: the general epilogue
        const v2s floor2 = __builtin_bit_cast(v2s, floor_pk);
        const long long img = (long long)blockIdx.x * PT + ((16 * PT * wave) >> 6);
        const bool img_ok = img * a.hw < a.M;
        int sums[4 * NG];
#pragma unroll
        for (int t = 0; t < 4 * NG; t++)
            sums[t] = 0;
#pragma unroll
        for (int c = 0; c < PT; c++) {
            const int pix0 = (16 * PT * wave + 16 * c) & 63;
            const int rows = img_ok ? min(max(a.hw - pix0, 0), 16) : 0; // uniform: tile rows inside the image
            if (rows == 0)
                continue;
            const int mine = rows - 4 * quad; // this lane's rows r < mine count
            const int m01 = (mine > 0 ? 0xffff : 0) | (mine > 1 ? (int)0xffff0000u : 0);
            const int m23 = (mine > 2 ? 0xffff : 0) | (mine > 3 ? (int)0xffff0000u : 0);
#pragma unroll
            for (int t = 0; t < 4 * NG; t++) {
                const int f = 64 * (t >> 2) + a_row0 + 4 * (t & 3); // tile t = 4 g + t' holds filters of group g
                const int ss = cst[1][f], ls = cst[2][f];
                const v4i v = acc[c][t];
                if constexpr (MODE >= 0) {
                    int w[4];
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        int x = v[r];
                        if (MODE == 5)
                            x = half_even_add(x, ss + 8 - ls);
                        w[r] = (int)((unsigned)x << ls) >> ss;
                    }
                    v2s p01 = __builtin_elementwise_max(__builtin_amdgcn_cvt_pk_i16(w[0], w[1]), floor2);
                    v2s p23 = __builtin_elementwise_max(__builtin_amdgcn_cvt_pk_i16(w[2], w[3]), floor2);
                    int q01 = __builtin_bit_cast(int, p01 >> 8), q23 = __builtin_bit_cast(int, p23 >> 8);
                    if (rows < 16) { // uniform
                        q01 &= m01;
                        q23 &= m23;
                    }
                    const v2s both = __builtin_bit_cast(v2s, q01) + __builtin_bit_cast(v2s, q23);
                    sums[t] = __builtin_bit_cast(int, __builtin_bit_cast(v2s, sums[t]) + both);
                } else {
#pragma unroll
                    for (int r = 0; r < 4; r++)
                        sums[t] += r < mine ? requant_s8(v[r], ss, relu, half_even) : 0;
                }
            }
        }
#pragma unroll
        for (int t = 0; t < 4 * NG; t++) {
            int total = MODE >= 0 ? (int)(short)(sums[t] & 0xffff) + (sums[t] >> 16) : sums[t];
            total += __shfl_xor(total, 16);
            total += __shfl_xor(total, 32);
            if (quad == 0)
                pool_l[wave][64 * (t >> 2) + a_row0 + 4 * (t & 3)] = total;
        }
    };
    if constexpr (GAP) {
        if (!fast)
            pooled(std::integral_constant<int, -1>{});
        else if (half_even)
            pooled(std::integral_constant<int, 5>{});
        else
            pooled(std::integral_constant<int, 1>{});
    } else {
        if (half_even)
            epilogue(std::integral_constant<int, 5>{});
        else
            epilogue(std::integral_constant<int, 1>{});
    }
    if constexpr (GAP) {
        __syncthreads();
        const int img_l = tid >> 6, flt = tid & 63; // image of the tile, filter of the group
        const long long img = (long long)blockIdx.x * PT + img_l;
#pragma unroll
        for (int g = 0; g < NG; g++)
            if (img_l < PT && img * a.hw < a.M && n0 + 64 * g + flt < a.N) {
                int sum = 0;
#pragma unroll
                for (int w = 0; w < 4; w++) // wavefront w holds tile rows 16 PT w ..: image PT w / 4
                    sum += ((PT * w) >> 2) == img_l ? pool_l[w][64 * g + flt] : 0;
                a.out[img * a.N + n0 + 64 * g + flt] = (int8_t)clamp_s8(round_half_up_f32((float)sum * a.gap_scale));
            }
    }
}

// The same product for a handful of rows (a classifier Gemm over one batch: 256 x 1280 x 1000): the tiled kernel
// above would run on a few dozen compute units and spend its time in twenty barrier-separated k steps.  Here a
// wavefront owns a 16-row x 16-filter tile for the whole reduction and reads both operands straight from
// global memory / L2 in the MFMA operand layout (lane (col, quad): 16 bytes of row col at k = 64 step + 16 quad),
// G k steps per batch of loads, the next batch in flight under the current one's MFMAs; a workgroup is four row
// tiles under one filter tile, so N / 16 x M / 64 workgroups fill the device and a workgroup's time is a few memory
// round trips.  K must be a multiple of 64.  The epilogue is the general one (any shift, either rounding).
template <int G>
__global__ __launch_bounds__(kThreads) void conv2d_s8_rows_kernel(const PwArgs a)
{
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col = lane & 15, quad = lane >> 4;
    const long long m0 = ((long long)blockIdx.x * 4 + wave) * 16;
    const int n0 = blockIdx.y * 16;
    if (m0 >= a.M) // uniform per wavefront; the kernel has no barrier
        return;
    const long long row = min(m0 + col, a.M - 1);
    const int flt = min(n0 + col, a.N - 1);
    const v4i *pa = reinterpret_cast<const v4i *>(a.w + (long long)flt * a.K + 16 * quad);
    const v4i *pb = reinterpret_cast<const v4i *>(a.in + row * a.in_pitch + 16 * quad);
    v4i ca[G], cb[G], na[G], nb[G];
#pragma unroll
    for (int i = 0; i < G; i++) {
        const int ks = min(i, a.ksteps - 1);
        ca[i] = pa[4 * ks];
        cb[i] = pb[4 * ks];
    }
    v4i acc = {0, 0, 0, 0};
    for (int g0 = 0; g0 < a.ksteps; g0 += G) {
        const bool more = g0 + G < a.ksteps; // uniform
        if (more) {
#pragma unroll
            for (int i = 0; i < G; i++) {
                const int ks = min(g0 + G + i, a.ksteps - 1);
                na[i] = pa[4 * ks];
                nb[i] = pb[4 * ks];
            }
        }
#pragma unroll
        for (int i = 0; i < G; i++)
            if (g0 + i < a.ksteps) // uniform
                acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(ca[i], cb[i], acc, 0, 0, 0);
        if (more) {
#pragma unroll
            for (int i = 0; i < G; i++) {
                ca[i] = na[i];
                cb[i] = nb[i];
            }
        }
    }
    // lane (col, quad) holds filters n0 + 4 quad + [0, 4) of row m0 + col
    const long long m = m0 + col;
    const int n = n0 + 4 * quad;
    const bool relu = a.relu != 0, half_even = a.half_even != 0;
    int q[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        const int nn = min(n + r, a.N - 1);
        const int b = a.bias != nullptr ? a.bias[nn] : 0;
        q[r] = requant_s8(acc[r] + b, a.shift[a.n_shift == 1 ? 0 : nn], relu, half_even);
    }
    if (m >= a.M || n >= a.N)
        return;
    int8_t *dst = a.out + m * a.out_pitch + n;
    if (a.out_vec >= 4 && n + 4 <= a.N) {
        *reinterpret_cast<int *>(dst) = pack4_s8(q[0], q[1], q[2], q[3]);
    } else {
#pragma unroll
        for (int r = 0; r < 4; r++)
            if (n + r < a.N)
                dst[r] = (int8_t)q[r];
    }
}

} // namespace

// Flat pointwise geometry; worth it when a workgroup of the implicit-GEMM
// kernel would see only a few pixel sets.
bool conv2d_s8_pwgemm_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count)
{
    const bool flat = g.k_h == 1 && g.k_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
        g.pad_left == 0 && g.out_h == g.in_h && g.out_w == g.in_w;
    if (!flat || g.in_c < 64 || g.out_c < 32)
        return false;
    // rows of a multiple of 16 bytes are read with aligned loads; any other length with loads that need none
    if ((g.in_c & 15) == 0 && (g.in_pitch & 15) == 0 &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter)) & 15) != 0)
        return false;
    const long long npix = (long long)g.batch * g.out_h * g.out_w;
    const int cus = cu_count > 0 ? cu_count : 256;
    // A short reduction under thousands of filters (a recognizer's 120 -> 6625 classifier) is bound by writing
    // the output: the implicit-GEMM kernel, whose wavefronts keep their pixels' operands in registers and write
    // several hundred contiguous bytes per pixel, does that faster (76 against 112 us on 20480 x 120 x 6625).
    if (g.in_c <= 128 && g.out_c >= 2048 && npix >= 64ll * cus)
        return false;
    return npix > 0 && (npix + 63) / 64 < (long long)cus * 16 && (npix + 63) / 64 <= 0x7fffffffll;
}

// The one-wavefront-per-tile kernel on its own: any filter count (a classifier with a handful of classes), K a
// multiple of 64, fewer 64 x 64 tiles than compute units.
bool conv2d_s8_rows_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count)
{
    const bool flat = g.k_h == 1 && g.k_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
        g.pad_left == 0 && g.out_h == g.in_h && g.out_w == g.in_w;
    if (!flat || (g.in_c & 63) != 0 || g.out_c < 1 || (g.in_pitch & 15) != 0 ||
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter)) & 15) != 0)
        return false;
    const long long npix = (long long)g.batch * g.out_h * g.out_w;
    const int cus = cu_count > 0 ? cu_count : 256;
    return npix > 0 && (npix + 63) / 64 * ((g.out_c + 63) / 64) < cus;
}

hipError_t launch_conv2d_s8_pwgemm(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                   const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                   int cu_count, hipStream_t stream)
{
    PwArgs a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.res = residual;
    a.out = out;
    a.M = (long long)g.batch * g.out_h * g.out_w;
    a.K = g.in_c;
    a.N = g.out_c;
    a.in_pitch = g.in_pitch;
    a.out_pitch = g.out_pitch;
    a.res_pitch = g.res_pitch;
    a.ksteps = (a.K + 63) / 64;
    a.relu = g.relu;
    a.half_even = g.half_even;
    a.n_shift = g.n_shift;
    a.hw = 0;
    a.gap_scale = 0.f;
    const uintptr_t oaddr = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(residual);
    a.out_vec = ((a.N & 15) == 0 && (oaddr & 15) == 0 && (a.out_pitch & 15) == 0) ? 16
        : (((a.N & 3) == 0 && (oaddr & 3) == 0 && (a.out_pitch & 3) == 0) ? 4 : 1);
    if (a.M == 0)
        return hipSuccess;
    // 64-filter tiles: measured faster than 128 on every MobileNetV2 layer (more, shorter workgroups).
    // 128-pixel tiles unless that leaves fewer than 1.5 workgroups per compute unit.
    const unsigned gy = (unsigned)((a.N + 63) / 64);
    const long long tiles128 = (a.M + 127) / 128;
    const int cus = cu_count > 0 ? cu_count : 256;
    // fewer 64 x 64 tiles than compute units: one wavefront per 16 x 16 tile, operands straight from global memory
    if (lut == nullptr && residual == nullptr && (a.K & 63) == 0 && (a.in_pitch & 15) == 0 && (a.M + 63) / 64 * gy < cus) {
        hipLaunchKernelGGL((conv2d_s8_rows_kernel<10>), dim3((unsigned)((a.M + 63) / 64), (unsigned)((a.N + 15) / 16)),
                           dim3(kThreads), 0, stream, a);
        return hipGetLastError();
    }
    const bool k16 = (a.K & 15) == 0 && (a.in_pitch & 15) == 0;
    if (tiles128 * gy * 2 < 3ll * cus) {
        if (k16)
            hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 1>), dim3((unsigned)((a.M + 63) / 64), gy), dim3(kThreads), 0, stream, a);
        else
            hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 1, false, false>), dim3((unsigned)((a.M + 63) / 64), gy), dim3(kThreads), 0, stream, a);
    } else {
        if (k16)
            hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 2>), dim3((unsigned)tiles128, gy), dim3(kThreads), 0, stream, a);
        else
            hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 2, false, false>), dim3((unsigned)tiles128, gy), dim3(kThreads), 0, stream, a);
    }
    return hipGetLastError();
}

// A convolution with a window through the same kernel, rows gathered from under the window: channels a multiple of
// 64, few output pixels per compute unit and a long reduction axis.
bool conv2d_s8_wingemm_supports(const ConvGeom &g, const void *in, const void *filter, int cu_count)
{
    if (g.k_h * g.k_w < 2 || (g.in_c & 63) != 0 || (g.in_pitch & 15) != 0 || g.out_c < 64 ||
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter)) & 15) != 0)
        return false;
    const long long npix = (long long)g.batch * g.out_h * g.out_w;
    const int cus = cu_count > 0 ? cu_count : 256;
    // the workgroups of the other kernels stage a filter group for every few pixel sets here: at most sixteen
    // 64-pixel tiles per compute unit, and a reduction axis of nine k steps or more
    return npix > 0 && npix < 0x7fffffffll && (npix + 63) / 64 < (long long)cus * 32 && g.k_h * g.k_w * g.in_c >= 576;
}

hipError_t launch_conv2d_s8_wingemm(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                    const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                    int cu_count, hipStream_t stream)
{
    PwArgs a = {};
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.res = residual;
    a.out = out;
    a.M = (long long)g.batch * g.out_h * g.out_w;
    a.K = g.k_h * g.k_w * g.in_c;
    a.N = g.out_c;
    a.in_pitch = g.in_pitch;
    a.out_pitch = g.out_pitch;
    a.res_pitch = g.res_pitch;
    a.ksteps = a.K / 64;
    a.relu = g.relu;
    a.half_even = g.half_even;
    a.n_shift = g.n_shift;
    a.w_in_h = g.in_h;
    a.w_in_w = g.in_w;
    a.w_in_c = g.in_c;
    a.w_k_w = g.k_w;
    a.w_stride_h = g.stride_h;
    a.w_stride_w = g.stride_w;
    a.w_dil_h = g.dil_h;
    a.w_dil_w = g.dil_w;
    a.w_pad_top = g.pad_top;
    a.w_pad_left = g.pad_left;
    a.fd_ohw = make_fastdiv((unsigned)(g.out_h * g.out_w));
    a.fd_ow = make_fastdiv((unsigned)g.out_w);
    a.fd_inc = make_fastdiv((unsigned)g.in_c);
    a.fd_kw = make_fastdiv((unsigned)g.k_w);
    const uintptr_t oaddr = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(residual);
    a.out_vec = ((a.N & 15) == 0 && (oaddr & 15) == 0 && (a.out_pitch & 15) == 0) ? 16
        : (((a.N & 3) == 0 && (oaddr & 3) == 0 && (a.out_pitch & 3) == 0) ? 4 : 1);
    if (a.M == 0)
        return hipSuccess;
    const unsigned gy = (unsigned)((a.N + 63) / 64);
    const long long tiles128 = (a.M + 127) / 128;
    const int cus = cu_count > 0 ? cu_count : 256;
    if (tiles128 * gy * 2 < 3ll * cus)
        hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 1, false, true, true>), dim3((unsigned)((a.M + 63) / 64), gy), dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 2, false, true, true>), dim3((unsigned)tiles128, gy), dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

// The same convolution followed by GlobalAveragePool, pooled tensor only: images of at most 64 pixels.
bool conv2d_gap_s8_supports(const ConvGeom &g, const void *in, const void *filter)
{
    const bool flat = g.k_h == 1 && g.k_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
        g.pad_left == 0 && g.out_h == g.in_h && g.out_w == g.in_w;
    return flat && g.in_pitch == g.in_c && (g.in_c & 15) == 0 && g.in_c >= 64 && g.out_c >= 32 && g.out_h * g.out_w <= 64 && g.batch <= 0x7fffffff &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(filter)) & 15) == 0;
}

hipError_t launch_conv2d_gap_s8(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                const int32_t *shift, float gap_scale, int8_t *out, int cu_count, hipStream_t stream)
{
    const int cus = cu_count > 0 ? cu_count : 256;
    PwArgs a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = nullptr;
    a.res = nullptr;
    a.out = out;
    a.hw = g.out_h * g.out_w;
    a.M = (long long)g.batch * a.hw;
    a.K = g.in_c;
    a.N = g.out_c;
    a.in_pitch = g.in_c;
    a.out_pitch = a.res_pitch = g.out_c;
    a.ksteps = (a.K + 63) / 64;
    a.relu = g.relu;
    a.half_even = g.half_even;
    a.n_shift = g.n_shift;
    a.out_vec = 1;
    a.gap_scale = gap_scale;
    if (a.M == 0)
        return hipSuccess;
    // else two images per workgroup (each filter tile is then read half as often) unless that leaves compute units idle
    const unsigned gy = (unsigned)((a.N + 63) / 64);
    // four images per workgroup while that leaves four workgroups per compute unit: a wavefront then reads each
    // filter tile from LDS once for four pixel tiles (the kernel is bound by LDS reads, not by the matrix pipe)
    if ((long long)((g.batch + 3) / 4) * gy >= 4ll * cus)
        hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 4, true>), dim3((unsigned)((g.batch + 3) / 4), gy), dim3(kThreads), 0, stream, a);
    else     if ((long long)((g.batch + 1) / 2) * gy >= 2ll * cus)
        hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 2, true>), dim3((unsigned)((g.batch + 1) / 2), gy), dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((conv2d_s8_pwgemm_kernel<1, 1, true>), dim3((unsigned)g.batch, gy), dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

} // namespace espdl
