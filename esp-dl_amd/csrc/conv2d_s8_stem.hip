// Dense int8 convolution of images with a handful of channels (the first layer of a network: RGB or grey
// input, 3 x 3 window, stride 2, 16 or 32 filters) for gfx950.
//
// What it computes is conv2d_33cn / _hwcn for int8 (esp-dl/dl/base/dl_base_conv2d.cpp:9-163) under
// conv_operation_shell's window clipping (esp-dl/dl/base/dl_base.hpp:382-1196), with the n_wise epilogue
// (bias, shift-round, ReLU, saturation; dl_base_activate_buffer.hpp:10-74) and an optional 256-entry table on
// the stored value (dl_base_lut.cpp:10-15).
//
// Such a layer moves a lot of bytes for very little arithmetic (27 multiply-adds per output value), and the
// general implicit-GEMM kernels spend their time on per-tile address arithmetic: 0.007 of the matrix peak and
// a seventh of the HBM rate.  Here the whole reduction is ONE MFMA step:
//   - a window row is k_w * in_c <= 16 contiguous bytes of the input row, so lane (pixel, ky) loads the 16
//     bytes that start at its window row with one unaligned load; the bytes behind the window row meet zero
//     weights.  That is operand B for k = 16 ky + (kx * in_c + c), k_h <= 4 rows -> K = 64;
//   - operand A (the filters in the same k order, zero filled) stays in registers for the life of the wavefront;
//   - a wavefront walks units of 64 consecutive output pixels of one output row: the unit's image, row and
//     first column are wave-uniform, a lane's address is base + column * stride * in_c;
//   - pixels whose window hangs over the left or right border (or whose 16 bytes would end behind the tensor)
//     assemble their bytes one by one; these are the first and last pixels of a row only.
// Filters are assigned to MFMA rows so that a lane ends up with 4 * RT consecutive channels of its pixel
// (RT = filter tiles of 16): one store of 4, 8, 12 or 16 bytes per pixel and lane.
#include "espdl_device.h"
#include "espdl_kernels.h"

#include <type_traits>

namespace espdl {
namespace {

constexpr int kThreads = 256;
constexpr int kUnitTiles = 4; // 16-pixel tiles per unit

struct StemArgs {
    const int8_t *in, *w, *lut;
    const int32_t *bias, *shift;
    int8_t *out;
    ConvGeom g;
    int seg_len;       // k_w * in_c, at most 16
    int row_bytes;     // in_w * in_c
    long long in_bytes; // whole input tensor
    long long img_bytes; // one image of it
    int xblocks;       // units per output row
    int n_units;
    int out_vec;       // 1: a lane's 4 * RT channels go out as one (unaligned) store of dwords
    FastDiv fd_xblocks, fd_out_h;
};

template <int RT, int MODE, bool HE>
__device__ __forceinline__ void stem_units(const StemArgs &a, const v4i (&wa)[RT], const v4i (&init)[RT], const v4i (&rsh)[RT],
                                           const v4i (&lsh)[RT], const unsigned char *lut_l, int first_unit, int unit_step)
{
    const ConvGeom &g = a.g;
    const int lane = threadIdx.x & 63, col = lane & 15, quad = lane >> 4;
    const bool relu = g.relu != 0, has_lut = a.lut != nullptr;
    const int floor_pk = relu ? 0 : (int)0x80008000u;
    const int OC = g.out_c, C = g.in_c;
    const int c_lane = 4 * RT * quad; // first channel of this lane
    // what does not change from unit to unit: this lane's column inside a tile as input bytes and output bytes,
    // its window row, whether its channels go out as whole dwords
    const int lane_in = col * g.stride_w * C;
    const int lane_out = col * g.out_pitch + c_lane;
    const int lane_iy = quad * g.dil_h - g.pad_top;
    const bool dwords_out = a.out_vec != 0 && c_lane + 4 * RT <= OC;
    const int tile_in = 16 * g.stride_w * C; // input bytes from tile to tile

    // operand B of the unit's four tiles: this lane's window row of pixel 16 t + col.  The unit number is
    // wave-uniform, so image, row and first column are scalars and a lane adds 32-bit offsets to them.
    const auto load_unit = [&](int unit, v4i (&b)[kUnitTiles]) {
        const unsigned rowid = fastdiv((unsigned)unit, a.fd_xblocks);
        const int xb = unit - (int)rowid * a.xblocks;
        const unsigned n = fastdiv(rowid, a.fd_out_h);
        const int oy = (int)(rowid - n * a.fd_out_h.d);
        const int8_t *img = a.in + (long long)n * a.img_bytes;
        const long long img_left = a.in_bytes - (long long)n * a.img_bytes; // bytes from the image start to the tensor end
        const int iy = oy * g.stride_h + lane_iy;
        const bool row_ok = quad < g.k_h && iy >= 0 && iy < g.in_h;
        const int row_off = (row_ok ? iy : 0) * a.row_bytes;
        const int off0 = (xb * (16 * kUnitTiles) * g.stride_w - g.pad_left) * C + lane_in;
        const int px_left = g.out_w - xb * (16 * kUnitTiles) - col; // this lane's pixel of tile t exists while 16 t < px_left
#pragma unroll
        for (int t = 0; t < kUnitTiles; t++) {
            const int off = off0 + t * tile_in; // first byte of the window row inside the input row
            b[t] = v4i{0, 0, 0, 0};
            if (row_ok && 16 * t < px_left) {
                // one 16-byte load from the byte where the window row starts.  (The memory pipeline takes such
                // loads apart lane by lane whether the start is a dword boundary or not: measured, loading from the
                // dword below and shifting was slower.  Its address unit is what bounds this kernel: 80 % busy.)
                const bool whole = off >= 0 && off + a.seg_len <= a.row_bytes && (long long)(row_off + off) + 16 <= img_left;
                const int8_t *row = img + row_off;
                if (whole) {
                    b[t] = *reinterpret_cast<const v4i_unaligned *>(row + off);
                } else {
                    // a window over the border, or 16 bytes that would end behind the tensor: byte by byte, all
                    // sixteen loads issued together (a byte outside the row reads the row's first byte and is dropped)
                    int word[4] = {0, 0, 0, 0};
#pragma unroll
                    for (int j = 0; j < 16; j++) {
                        const int pos = off + j;
                        // byte j belongs to tap kx = j / C at column ix0 + kx: inside the row, or padding
                        const bool inside = j < a.seg_len && pos >= 0 && pos < a.row_bytes;
                        const int v = (int)(unsigned char)row[inside ? pos : 0];
                        word[j >> 2] |= (inside ? v : 0) << (8 * (j & 3));
                    }
                    b[t] = v4i{word[0], word[1], word[2], word[3]};
                }
            }
        }
    };

    int unit = __builtin_amdgcn_readfirstlane(first_unit);
    if (unit >= a.n_units)
        return;
    v4i b[kUnitTiles], ahead[kUnitTiles];
    load_unit(unit, ahead);
    for (; unit < a.n_units; unit += unit_step) {
#pragma unroll
        for (int t = 0; t < kUnitTiles; t++)
            b[t] = ahead[t];
        // the next unit's bytes are requested before this one is worked on
        if (unit + unit_step < a.n_units)
            load_unit(unit + unit_step, ahead);
        const unsigned rowid = fastdiv((unsigned)unit, a.fd_xblocks);
        const int xb = unit - (int)rowid * a.xblocks;
        int8_t *out_px = a.out + ((long long)rowid * g.out_w + (long long)xb * (16 * kUnitTiles)) * g.out_pitch;
        const int px_left = g.out_w - xb * (16 * kUnitTiles) - col;
#pragma unroll
        for (int t = 0; t < kUnitTiles; t++) {
            int words[RT];
#pragma unroll
            for (int r = 0; r < RT; r++) {
                const v4i acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(wa[r], b[t], init[r], 0, 0, 0);
                if constexpr (MODE >= 0) {
                    words[r] = pack_fast4<MODE>(acc, lsh[r], rsh[r], floor_pk);
                } else {
                    int q[4];
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        q[e] = requant_s8(acc[e], rsh[r][e], relu, HE);
                    words[r] = pack4_s8(q[0], q[1], q[2], q[3]);
                }
                if (has_lut) {
                    const int v = words[r];
                    words[r] = pack4_s8(lut_l[(int)(int8_t)v + 128], lut_l[(int)(int8_t)(v >> 8) + 128],
                                        lut_l[(int)(int8_t)(v >> 16) + 128], lut_l[(v >> 24) + 128]);
                }
            }
            if (16 * t >= px_left)
                continue;
            int8_t *dst = out_px + (16 * t * g.out_pitch + lane_out);
            if (dwords_out) {
                if constexpr (RT == 4)
                    *reinterpret_cast<v4i_unaligned *>(dst) = v4i{words[0], words[1], words[2], words[3]};
                else
#pragma unroll
                    for (int r = 0; r < RT; r++)
                        *reinterpret_cast<int_unaligned *>(dst + 4 * r) = words[r];
            } else {
#pragma unroll
                for (int r = 0; r < RT; r++)
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (c_lane + 4 * r + e < OC)
                            dst[4 * r + e] = (int8_t)(words[r] >> (8 * e));
            }
        }
    }
}

template <int RT, bool HE>
__global__ __launch_bounds__(kThreads) void conv2d_s8_stem_kernel(const StemArgs a)
{
    __shared__ unsigned char lut_l[256];
    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, col = lane & 15, quad = lane >> 4;
    const int OC = g.out_c;

    // Can the filters take the short epilogue?  Every shift in 1..31, and bias + 2^(s-1) plus the largest sum
    // of products must fit int32 also after the left shift by max(0, 8 - s) of the short form.
    const long long mac_bound = (long long)g.k_h * g.k_w * g.in_c * 16384;
    int ok_local = 1, lsh_local = 0;
    for (int oc = tid; oc < OC; oc += kThreads) {
        const int s = a.shift[g.n_shift == 1 ? 0 : oc];
        const long long bv = a.bias != nullptr ? (long long)a.bias[oc] : 0;
        if (s < 8)
            lsh_local = 1;
        if (s < 1 || s > 31) {
            ok_local = 0;
        } else {
            const long long start = bv + (1ll << (s - 1));
            const long long mag = (start < 0 ? -start : start) + mac_bound;
            if (mag >= (1ll << (31 - max(0, 8 - s))))
                ok_local = 0;
        }
    }
    if (a.lut != nullptr && tid < 256)
        lut_l[tid] = (unsigned char)a.lut[tid];
    const bool fast = __syncthreads_and(ok_local) != 0;
    const bool use_lsh = __syncthreads_or(lsh_local) != 0;

    // MFMA row i of filter tile t is filter 4 RT (i >> 2) + 4 t + (i & 3): a lane's accumulators of all tiles are
    // then 4 RT consecutive channels.  Operand A: this lane's filter, window row `quad`, zero behind the row.
    v4i wa[RT], init[RT], rsh[RT], lsh[RT];
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const int f = 4 * RT * (col >> 2) + 4 * t + (col & 3);
        int word[4] = {0, 0, 0, 0};
        if (f < OC && quad < g.k_h) {
            const int8_t *src = a.w + ((long long)f * g.k_h + quad) * a.seg_len;
            for (int j = 0; j < a.seg_len; j++)
                word[j >> 2] |= (int)(unsigned char)src[j] << (8 * (j & 3));
        }
        wa[t] = v4i{word[0], word[1], word[2], word[3]};
        // the accumulators of this lane: channels 4 RT quad + 4 t + e
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const int oc = 4 * RT * quad + 4 * t + e;
            int i0 = 0, sh = fast ? 8 : 0, ls = 0;
            if (oc < OC) {
                const int s = a.shift[g.n_shift == 1 ? 0 : oc];
                const int bv = a.bias != nullptr ? a.bias[oc] : 0;
                i0 = fast ? bv + (1 << (s - 1)) - (HE ? 1 : 0) : bv; // the half-even form starts one lower
                sh = fast ? max(0, s - 8) : s;
                ls = fast ? max(0, 8 - s) : 0;
            }
            init[t][e] = i0;
            rsh[t][e] = sh;
            lsh[t][e] = ls;
        }
    }

    const int waves = kThreads / 64;
    const int first = blockIdx.x * waves + (tid >> 6), step = gridDim.x * waves;
    if (!fast)
        stem_units<RT, -1, HE>(a, wa, init, rsh, lsh, lut_l, first, step);
    else if (HE)
        use_lsh ? stem_units<RT, 5, HE>(a, wa, init, rsh, lsh, lut_l, first, step)
                : stem_units<RT, 6, HE>(a, wa, init, rsh, lsh, lut_l, first, step);
    else
        use_lsh ? stem_units<RT, 1, HE>(a, wa, init, rsh, lsh, lut_l, first, step)
                : stem_units<RT, 0, HE>(a, wa, init, rsh, lsh, lut_l, first, step);
}

template <int RT>
hipError_t launch_rt(const StemArgs &a, int blocks, hipStream_t stream)
{
    if (a.g.half_even)
        hipLaunchKernelGGL((conv2d_s8_stem_kernel<RT, true>), dim3(blocks), dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((conv2d_s8_stem_kernel<RT, false>), dim3(blocks), dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

} // namespace

bool conv2d_s8_stem_supports(const ConvGeom &g, const void *residual)
{
    if (residual != nullptr || g.k_h > 4 || g.k_w * g.in_c > 16 || g.dil_w != 1 || g.out_c > 64)
        return false;
    if (g.in_pitch != g.in_c) // window rows must be contiguous bytes of the input row
        return false;
    // a lane adds 32-bit offsets to the start of its image and of its unit's first output pixel
    if ((long long)g.batch * g.in_h * g.in_w * g.in_c >= (1ll << 40) || (long long)g.in_h * g.in_w * g.in_c >= (1ll << 30) ||
        (long long)g.out_pitch * 64 >= (1ll << 30) || (long long)g.in_h * g.in_w * g.in_c < 16)
        return false;
    const long long units = (long long)g.batch * g.out_h * ((g.out_w + 16 * kUnitTiles - 1) / (16 * kUnitTiles));
    // one MFMA per 16 pixels whatever the window: only worth it for images (many pixels per filter)
    // pointwise products over 16 channels are better off in the GEMM kernels (a quarter of this one's MFMA rows
    // would carry data)
    if (g.k_h * g.k_w == 1)
        return false;
    return units < (1ll << 31) && (long long)g.batch * g.out_h * g.out_w >= 256;
}

hipError_t launch_conv2d_s8_stem(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                 const int32_t *shift, const int8_t *lut, int8_t *out, int cu_count, hipStream_t stream)
{
    StemArgs a = {};
    a.in = in;
    a.w = filter;
    a.lut = lut;
    a.bias = bias;
    a.shift = shift;
    a.out = out;
    a.g = g;
    a.seg_len = g.k_w * g.in_c;
    a.row_bytes = g.in_w * g.in_c;
    a.in_bytes = (long long)g.batch * g.in_h * g.in_w * g.in_c;
    a.img_bytes = (long long)g.in_h * g.in_w * g.in_c;
    a.xblocks = (g.out_w + 16 * kUnitTiles - 1) / (16 * kUnitTiles);
    a.n_units = (int)((long long)g.batch * g.out_h * a.xblocks);
    if (a.n_units == 0 || g.out_c == 0)
        return hipSuccess;
    a.out_vec = (g.out_c % 4) == 0 ? 1 : 0;
    a.fd_xblocks = make_fastdiv((unsigned)a.xblocks);
    a.fd_out_h = make_fastdiv((unsigned)g.out_h);
    const int rt = (g.out_c + 15) / 16;
    const int cus = cu_count > 0 ? cu_count : 256;
    // resident workgroups walk the units with a stride: eight per compute unit, fewer when there is less work
    const int waves = kThreads / 64;
    const int blocks = (int)std::min<long long>((long long)cus * 8, ((long long)a.n_units + waves - 1) / waves);
    switch (rt) {
    case 1:
        return launch_rt<1>(a, blocks, stream);
    case 2:
        return launch_rt<2>(a, blocks, stream);
    case 3:
        return launch_rt<3>(a, blocks, stream);
    default:
        return launch_rt<4>(a, blocks, stream);
    }
}

} // namespace espdl
