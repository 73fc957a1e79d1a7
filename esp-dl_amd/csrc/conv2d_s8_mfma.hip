// Host side of the int8 implicit-GEMM convolution: picks the operand-B mode, the LDS plan (how many
// 64-filter groups and k steps stay resident per workgroup), the pixel tile and the persistent grid,
// then dispatches to the kernel variant compiled in conv2d_s8_mfma_<mode>.hip.  The kernel itself is
// described in conv2d_s8_mfma_kernel.h.
#include "conv2d_s8_mfma_kernel.h"

namespace espdl {

using namespace mfma_conv;

namespace {
constexpr int kLdsPerWorkgroup = 64 * 1024; // dynamic LDS a workgroup may ask for without opting in
} // namespace

hipError_t launch_conv2d_s8_mfma(const ConvGeom &g, const int8_t *in, const int8_t *filter, const int32_t *bias,
                                 const int32_t *shift, const int8_t *lut, const int8_t *residual, int8_t *out,
                                 int cu_count, hipStream_t stream)
{
    MfmaConvArgs a;
    a.in = in;
    a.w = filter;
    a.bias = bias;
    a.shift = shift;
    a.lut = lut;
    a.res = residual;
    a.out = out;
    a.g = g;
    a.npix = (long long)g.batch * g.out_h * g.out_w;
    // bytes a load may touch: up to the last channel of the last pixel of the (possibly pitched) input
    a.in_bytes = ((long long)g.batch * g.in_h * g.in_w - 1) * g.in_pitch + g.in_c;
    if (a.npix == 0)
        return hipSuccess;

    // operand-B mode
    const bool aligned16 = ((reinterpret_cast<uintptr_t>(in) & 15) == 0);
    int bmode = B_GATHER;
    // flat pointwise: 1x1, stride 1, no padding -> output pixel i reads input pixel i
    const bool flat = g.k_h == 1 && g.k_w == 1 && g.stride_h == 1 && g.stride_w == 1 && g.pad_top == 0 &&
        g.pad_left == 0 && g.out_h == g.in_h && g.out_w == g.in_w;
    if (flat)
        bmode = B_POINT;
    else if ((g.in_c & 15) == 0 && (g.in_pitch & 15) == 0 && aligned16)
        bmode = B_VEC16;
    else if (g.dil_w == 1 && g.in_pitch == g.in_c) // a filter row's bytes are contiguous in a dense input only
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
    const uintptr_t out_addr = reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(residual);
    a.out_vec = ((g.out_c & 15) == 0 && (out_addr & 15) == 0) ? 16 : (((g.out_c & 3) == 0 && (out_addr & 3) == 0) ? 4 : 1);

    // LDS plan: per resident filter group ksteps * 4 KiB of weights + 512 B of start values / shifts,
    // plus 256 B for the LUT.  All groups of the layer stay resident when they fit; otherwise as many
    // as fit; if even one group does not fit, K is chunked.
    const int fixed = 256;
    const int per_group_full = a.ksteps * 4096 + 768;
    const int cus = cu_count > 0 ? cu_count : 256;
    // With few pixel sets per CU a workgroup lives for a handful of sets and the launch is bound by
    // the latency of staging its filters and of its first loads, not by bandwidth: then smaller filter
    // chunks (more, shorter-lived workgroups per CU; the input is re-read per chunk, from L2) win.
    const long long sets64 = (a.npix + 63) / 64;
    const int budget = sets64 < (long long)cus * 16 ? 40 * 1024 : kLdsPerWorkgroup;
    if (per_group_full + fixed <= kLdsPerWorkgroup) {
        a.ks_per_chunk = a.ksteps;
        a.n_kchunks = 1;
        int gpc = min(a.n_groups, max(1, (budget - fixed) / per_group_full));
        // equal chunks: the slowest chunk sets the time
        const int chunks = (a.n_groups + gpc - 1) / gpc;
        gpc = (a.n_groups + chunks - 1) / chunks;
        a.groups_per_chunk = gpc;
    } else {
        a.ks_per_chunk = (kLdsPerWorkgroup - fixed - 768) / 4096;
        a.n_kchunks = (a.ksteps + a.ks_per_chunk - 1) / a.ks_per_chunk;
        a.groups_per_chunk = 1;
    }
    const int n_chunks = (a.n_groups + a.groups_per_chunk - 1) / a.groups_per_chunk;
    size_t lds = (size_t)a.groups_per_chunk * (a.ks_per_chunk * 4096 + 768) + fixed;

    // register plan: hold the whole reduction axis when it is short enough; two pixel tiles per wave
    // (half the LDS traffic per MFMA) when there are enough pixels and registers
    int ksc = a.n_kchunks == 1 ? pick_ksc(a.ksteps) : 0;
    if (bmode == B_GATHER)
        ksc = 0;
    // (with six or more resident k steps two pixel tiles take every register and leave one wavefront per SIMD:
    // measured 2 to 4 % slower on whole YOLO11n graphs than one tile at two wavefronts per SIMD)
    const int pt = (a.npix >= (long long)cus * 8 * 128 && ksc < 6) ? 2 : 1;
    a.n_sets = (int)((a.npix + 64 * pt - 1) / (64 * pt));
    // contiguous output: needs every filter group in one chunk, 4-byte aligned rows and room in LDS
    const size_t out_tiles = (size_t)4 * 16 * pt * g.out_c;
    a.stage_out = (n_chunks == 1 && a.out_vec >= 4 && (out_addr & 15) == 0 && g.out_pitch == g.out_c && g.res_pitch == g.out_c &&
                   lds + out_tiles <= 40 * 1024) ? 1 : 0;
    if (a.stage_out)
        lds += out_tiles;
    a.fd_out_hw = make_fastdiv((unsigned)g.out_h * (unsigned)g.out_w);
    a.fd_out_w = make_fastdiv((unsigned)g.out_w);
    a.fd_in_c = make_fastdiv((unsigned)g.in_c);
    a.fd_k_w = make_fastdiv((unsigned)g.k_w);
    a.fd_seg_pad = make_fastdiv((unsigned)(a.seg_pad > 0 ? a.seg_pad : 1));

    // persistent grid: sized by launch_variant from the residency of the chosen kernel variant
    const GridPlan grid{cus, n_chunks};

    switch (bmode) {
    case B_VEC16:
        return launch_vec16(a, pt, ksc, grid, lds, stream);
    case B_POINT:
        return launch_point(a, pt, ksc, grid, lds, stream);
    case B_ROWSEG:
        return launch_rowseg(a, pt, ksc, grid, lds, stream);
    default:
        return launch_gather(a, pt, ksc, grid, lds, stream);
    }
}

} // namespace espdl
