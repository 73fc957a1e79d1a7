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
//   - a window row is k_w * in_c <= 16 contiguous bytes of the input row: that is operand B of lane (pixel, ky)
//     for k = 16 ky + (kx * in_c + c), k_h <= 4 rows -> K = 64; the bytes behind the window row meet zero weights;
//   - operand A (the filters in the same k order, zero filled) stays in registers for the life of the wavefront;
//   - a wavefront walks units of 64 consecutive output pixels of one output row: the unit's image, row and
//     first column are wave-uniform;
//   - the unit's k_h input rows are copied into the wavefront's LDS rows as CONSECUTIVE aligned 16-byte pieces
//     (the next unit's pieces are in flight while this one is multiplied), bytes outside the image row become
//     zeros there (that is the window clipping), and a lane cuts its window row out of LDS with one unaligned
//     16-byte read.  Loading the window rows straight from memory - 16 bytes per lane from addresses
//     stride * in_c bytes apart - was bound by the memory pipeline's address unit: a vector memory instruction
//     whose lanes do not address consecutive pieces is taken apart lane by lane (64 cycles instead of 16);
//   - for the same reason the results leave through an LDS slab as 16-byte pieces in memory order when every
//     filter tile is full (out_c = 16, 32, 48, 64).
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
    int ppr;           // 16-byte pieces per copied row
    FastDiv fd_xblocks, fd_out_h, fd_ppr;
};

template <int RT, int MODE, bool HE>
__device__ __forceinline__ void stem_units(const StemArgs &a, const v4i (&wa)[RT], const v4i (&init)[RT], const v4i (&rsh)[RT],
                                           const v4i (&lsh)[RT], const unsigned char *lut_l, unsigned char *stage,
                                           unsigned char *rowbuf, int first_unit, int unit_step)
{
    const ConvGeom &g = a.g;
    const int lane = threadIdx.x & 63, col = lane & 15, quad = lane >> 4;
    const bool relu = g.relu != 0, has_lut = a.lut != nullptr;
    const int floor_pk = relu ? 0 : (int)0x80008000u;
    const int OC = g.out_c, C = g.in_c;
    const int c_lane = 4 * RT * quad; // first channel of this lane
    const int lds_pitch = 16 * a.ppr;
    // what does not change from unit to unit
    const int lane_out = col * g.out_pitch + c_lane;
    const bool dwords_out = a.out_vec != 0 && c_lane + 4 * RT <= OC;
    // every filter tile full: the unit's 64 pixels x OC bytes go through this wavefront's LDS slab and leave as
    // 16-byte pieces in memory order, consecutive lanes writing consecutive addresses
    const bool staged_out = OC == 16 * RT;
    // this lane's window row inside the copied rows: row `quad`, byte (16 t + col) * stride_w * C (+ the skew)
    const int cut_off = quad * lds_pitch + col * g.stride_w * C;
    const int tile_in = 16 * g.stride_w * C; // input bytes from tile to tile
    // the two 16-byte pieces of the copied rows this lane brings in: piece lane + 64 j = piece pc_j of row r_j
    int pr[2], pp[2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const unsigned i = (unsigned)(lane + 64 * j);
        const unsigned r = fastdiv(i, a.fd_ppr);
        pr[j] = (int)r;
        pp[j] = (int)(i - r * a.fd_ppr.d);
    }
    const int8_t *const in_end = a.in + a.in_bytes;

    // Request the unit's k_h input rows as consecutive aligned 16-byte pieces: first piece = the 16-byte address at
    // or below the first byte the unit's windows touch.  Bytes outside the image row are padding (zeros).
    const auto fetch_rows = [&](int unit, v4i (&pc)[2]) {
        const unsigned rowid = fastdiv((unsigned)unit, a.fd_xblocks);
        const int xb = unit - (int)rowid * a.xblocks;
        const unsigned n = fastdiv(rowid, a.fd_out_h);
        const int oy = (int)(rowid - n * a.fd_out_h.d);
        const int8_t *img = a.in + (long long)n * a.img_bytes;
        const int start_off = (xb * (16 * kUnitTiles) * g.stride_w - g.pad_left) * C;
        const int iy0 = oy * g.stride_h - g.pad_top;
#pragma unroll
        for (int j = 0; j < 2; j++) {
            const int iy = iy0 + pr[j] * g.dil_h;
            pc[j] = v4i{0, 0, 0, 0};
            if (pr[j] < g.k_h && iy >= 0 && iy < g.in_h) {
                const int8_t *row = img + (long long)iy * a.row_bytes;
                const int8_t *first = row + start_off;
                const int8_t *pa = first - (int)(reinterpret_cast<uintptr_t>(first) & 15) + 16 * pp[j];
                const int lo = (int)(row - pa), hi = lo + a.row_bytes; // bytes [lo, hi) of the piece lie in the row
                if (hi > 0 && lo < 16) {
                    v4i v = {0, 0, 0, 0};
                    if (pa >= a.in && pa + 16 <= in_end) {
                        v = *reinterpret_cast<const v4i *>(pa);
                    } else { // the piece hangs over an end of the tensor (first or last row only): byte by byte
#pragma unroll 1
                        for (int k = 0; k < 16; k++)
                            if (pa + k >= a.in && pa + k < in_end)
                                v[k >> 2] |= (int)(unsigned char)pa[k] << (8 * (k & 3));
                    }
                    if (lo > 0 || hi < 16) { // over the row's first or last byte: what lies outside is padding
#pragma unroll
                        for (int d = 0; d < 4; d++) {
                            const int dl = min(max(lo - 4 * d, 0), 4), dh = min(max(hi - 4 * d, 0), 4);
                            const unsigned m_lo = dl >= 4 ? 0u : 0xffffffffu << (8 * dl);
                            const unsigned m_hi = dh >= 4 ? 0xffffffffu : (1u << (8 * dh)) - 1u;
                            v[d] &= (int)(m_lo & m_hi);
                        }
                    }
                    pc[j] = v;
                }
            }
        }
    };

    int unit = __builtin_amdgcn_readfirstlane(first_unit);
    if (unit >= a.n_units)
        return;
    v4i pieces[2];
    fetch_rows(unit, pieces);
    // copied rows -> LDS.  The rows of the NEXT unit are written where this unit's results are about to leave (its
    // window rows were cut out long before): the wait for their loads then stands in front of this unit's stores
    // and not behind them, where it would wait for the stores as well.
    const auto rows_to_lds = [&]() {
#pragma unroll
        for (int j = 0; j < 2; j++)
            if (pr[j] < g.k_h)
                *reinterpret_cast<v4i *>(rowbuf + pr[j] * lds_pitch + 16 * pp[j]) = pieces[j];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    rows_to_lds();
    for (; unit < a.n_units; unit += unit_step) {
        // this lane's four window rows out of the copied rows (unaligned 16-byte reads)
        const unsigned rowid = fastdiv((unsigned)unit, a.fd_xblocks);
        const int xb = unit - (int)rowid * a.xblocks;
        v4i b[kUnitTiles];
        {
            const unsigned n = fastdiv(rowid, a.fd_out_h);
            const int oy = (int)(rowid - n * a.fd_out_h.d);
            const int iy = oy * g.stride_h - g.pad_top + quad * g.dil_h;
            const int8_t *first = a.in + (long long)n * a.img_bytes + (long long)iy * a.row_bytes +
                (xb * (16 * kUnitTiles) * g.stride_w - g.pad_left) * C;
            const int skew = (int)(reinterpret_cast<uintptr_t>(first) & 15);
            // (one unaligned 16-byte LDS read per tile; three aligned dword reads and a funnel shift were slower)
#pragma unroll
            for (int t = 0; t < kUnitTiles; t++)
                b[t] = quad < g.k_h ? *reinterpret_cast<const v4i_unaligned *>(rowbuf + cut_off + skew + t * tile_in)
                                    : v4i{0, 0, 0, 0};
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // the next unit's rows are requested before this one is worked on
        if (unit + unit_step < a.n_units)
            fetch_rows(unit + unit_step, pieces);
        int8_t *out_px = a.out + ((long long)rowid * g.out_w + (long long)xb * (16 * kUnitTiles)) * g.out_pitch;
        const int unit_px = g.out_w - xb * (16 * kUnitTiles); // pixels of this unit that exist (up to 64 count)
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
            if (staged_out) {
                // slab layout: [pixel of the unit][16 RT bytes]; this lane's 4 RT channels of pixel 16 t + col
                unsigned char *slot = stage + (16 * t + col) * (16 * RT) + c_lane;
                if constexpr (RT == 4)
                    *reinterpret_cast<v4i *>(slot) = v4i{words[0], words[1], words[2], words[3]};
                else
#pragma unroll
                    for (int r = 0; r < RT; r++)
                        *reinterpret_cast<int *>(slot + 4 * r) = words[r];
                continue;
            }
            if (16 * t + col >= unit_px)
                continue;
            int8_t *dst = out_px + (16 * t * g.out_pitch + lane_out);
            if (dwords_out) {
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
        rows_to_lds(); // (its barrier also orders the slab's writes before the reads below)
        if (staged_out) {
            // piece i = 16 bytes i of the slab = piece i % RT of pixel i / RT
#pragma unroll
            for (int j = 0; j < RT; j++) {
                const int i = lane + 64 * j;
                const int px = i / RT, piece = i - px * RT;
                const v4i v = *reinterpret_cast<const v4i *>(stage + 16 * i);
                if (px < unit_px)
                    *reinterpret_cast<v4i_unaligned *>(out_px + px * g.out_pitch + 16 * piece) = v;
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    }
}

template <int RT, bool HE>
__global__ __launch_bounds__(kThreads) void conv2d_s8_stem_kernel(const StemArgs a)
{
    __shared__ unsigned char lut_l[256];
    __shared__ __align__(16) unsigned char slabs[kThreads / 64][64 * 16 * RT]; // a wavefront's unit of output
    const ConvGeom &g = a.g;
    const int tid = threadIdx.x, lane = tid & 63, col = lane & 15, quad = lane >> 4;
    const int OC = g.out_c;
    unsigned char *stage = slabs[tid >> 6];
    extern __shared__ __align__(16) unsigned char row_lds[]; // per wavefront: k_h copied input rows (when used)
    unsigned char *rowbuf = row_lds + (tid >> 6) * (g.k_h * 16 * a.ppr);

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
        stem_units<RT, -1, HE>(a, wa, init, rsh, lsh, lut_l, stage, rowbuf, first, step);
    else if (HE)
        use_lsh ? stem_units<RT, 5, HE>(a, wa, init, rsh, lsh, lut_l, stage, rowbuf, first, step)
                : stem_units<RT, 6, HE>(a, wa, init, rsh, lsh, lut_l, stage, rowbuf, first, step);
    else
        use_lsh ? stem_units<RT, 1, HE>(a, wa, init, rsh, lsh, lut_l, stage, rowbuf, first, step)
                : stem_units<RT, 0, HE>(a, wa, init, rsh, lsh, lut_l, stage, rowbuf, first, step);
}

template <int RT>
hipError_t launch_rt(const StemArgs &a, int blocks, hipStream_t stream)
{
    const size_t lds = (size_t)(kThreads / 64) * a.g.k_h * 16 * a.ppr;
    if (a.g.half_even)
        hipLaunchKernelGGL((conv2d_s8_stem_kernel<RT, true>), dim3(blocks), dim3(kThreads), lds, stream, a);
    else
        hipLaunchKernelGGL((conv2d_s8_stem_kernel<RT, false>), dim3(blocks), dim3(kThreads), lds, stream, a);
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
    // a unit's k_h input rows must fit two 16-byte pieces per lane
    if (g.k_h * (((16 * kUnitTiles - 1) * g.stride_w * g.in_c + 16 + 15 + 15) / 16) > 128)
        return false;
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
    // copied rows: the bytes the unit's windows touch, plus up to 15 in front (pieces start on 16-byte addresses)
    a.ppr = ((16 * kUnitTiles - 1) * g.stride_w * g.in_c + 16 + 15 + 15) / 16;
    a.fd_ppr = make_fastdiv((unsigned)a.ppr);
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
