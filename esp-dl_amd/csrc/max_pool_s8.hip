// int8 MaxPool over K x K windows at stride 1 (the pools of SPP / SPPF blocks: 5 x 5, stride 1, padding 2),
// base::max_pool2d of esp-dl/dl/base/dl_base_max_pool2d.cpp:9-29 over the window clipped to the image.
//
// The hardware has no byte-wise maximum, and widening every byte to 32 bits costs several vector-ALU
// operations per byte and window position, which is what bounds a straightforward kernel (a tenth of the
// HBM rate on 5 x 5 windows).  Here the maximum works on int16 pairs (v_pk_max_i16):
//   - of a loaded dword the raw bits serve as the "odd bytes" operand: each 16-bit half orders like its high
//     byte (a signed byte), the low byte below it only breaks ties between equal high bytes, and only the
//     high byte of the result is kept;
//   - the dword shifted left by 8 is the "even bytes" operand in the same way;
//   - one byte permute puts the two results together.
// That is one shift per loaded dword, two packed maxima per dword and window position, one permute per result.
//
// The window is separable: a thread owns two neighbouring output columns and one 16-byte channel vector, walks
// down a strip of output rows, takes the horizontal maxima of each input row once (K + 1 loaded pixels, K
// maxima for the two columns since their windows share K - 1 pixels), keeps the last K of them in registers
// (joined back into bytes, which halves their registers and lets a fourth wavefront onto each SIMD) and takes
// the vertical maximum for each output row.  Pixels outside the image count as -128, which never wins against
// a pixel inside (every window of a valid geometry holds at least one).  The walk is bound by the latency of
// its loads (each pixel is requested by three threads), not by the arithmetic: 0.60 of the HBM rate on large
// tensors against 0.10 for the byte-wise kernel.
// Input and output may be channel slices of wider tensors (pitches in bytes).
#include "espdl_kernels.h"
#include "espdl_device.h"

namespace espdl {

namespace {

constexpr int kThreads = 256;

struct WindowPoolArgs {
    const char *in;
    char *out;
    int h, w, out_h, out_w, pad_top, pad_left;
    int cv;     // channel vectors (of D dwords) per pixel
    int rows;   // output rows per strip
    int strips; // strips per image
    int xpairs; // column pairs per row
    long long in_pitch, out_pitch; // bytes from pixel to pixel
    FastDiv fd_cv, fd_xpairs, fd_strips;
    unsigned total; // threads
};

// D dwords of one pixel
template <int D>
struct Vec {
    int d[D];
};

template <int D>
__device__ __forceinline__ Vec<D> load_vec(const char *p)
{
    Vec<D> r;
    if constexpr (D == 4) {
        const v4i x = *reinterpret_cast<const v4i *>(p);
        r.d[0] = x[0], r.d[1] = x[1], r.d[2] = x[2], r.d[3] = x[3];
    } else {
        const v2i x = *reinterpret_cast<const v2i *>(p);
        r.d[0] = x[0], r.d[1] = x[1];
    }
    return r;
}

template <int D>
__device__ __forceinline__ void store_vec(char *p, const Vec<D> &r)
{
    if constexpr (D == 4)
        *reinterpret_cast<v4i *>(p) = v4i{r.d[0], r.d[1], r.d[2], r.d[3]};
    else
        *reinterpret_cast<v2i *>(p) = v2i{r.d[0], r.d[1]};
}

template <int D>
__device__ __forceinline__ Vec<D> pkmax(const Vec<D> &a, const Vec<D> &b)
{
    Vec<D> r;
#pragma unroll
    for (int i = 0; i < D; i++)
        r.d[i] = pk_max_i16(a.d[i], b.d[i]);
    return r;
}

// the bytes of each dword moved up by one: the even bytes where packed int16 maxima order by them
template <int D>
__device__ __forceinline__ Vec<D> shifted(const Vec<D> &a)
{
    Vec<D> r;
#pragma unroll
    for (int i = 0; i < D; i++)
        r.d[i] = a.d[i] << 8;
    return r;
}

// bytes [even.1, odd.1, even.3, odd.3] of each dword: the maxima of the odd-byte and even-byte operands as bytes
template <int D>
__device__ __forceinline__ Vec<D> join(const Vec<D> &odd, const Vec<D> &even)
{
    Vec<D> r;
#pragma unroll
    for (int i = 0; i < D; i++)
        r.d[i] = (int)__builtin_amdgcn_perm((unsigned)odd.d[i], (unsigned)even.d[i], 0x07030501u);
    return r;
}

// K x K window, D dwords of channels per thread
template <int K, int D>
__global__ __launch_bounds__(kThreads) void max_pool_s8_window_kernel(const WindowPoolArgs a)
{
    typedef Vec<D> V;
    const unsigned tid = blockIdx.x * kThreads + threadIdx.x;
    if (tid >= a.total)
        return;
    const unsigned q0 = fastdiv(tid, a.fd_cv);
    const unsigned v = tid - q0 * a.fd_cv.d;
    const unsigned q1 = fastdiv(q0, a.fd_xpairs);
    const unsigned xp = q0 - q1 * a.fd_xpairs.d;
    const unsigned n = fastdiv(q1, a.fd_strips);
    const unsigned strip = q1 - n * a.fd_strips.d;
    const int x0 = 2 * (int)xp, y0 = (int)strip * a.rows;
    const char *img_in = a.in + (long long)n * a.h * a.w * a.in_pitch + (long long)v * (4 * D);
    char *img_out = a.out + (long long)n * a.out_h * a.out_w * a.out_pitch + (long long)v * (4 * D);

    // the K + 1 input columns under the two windows
    long long col_off[K + 1];
    bool col_ok[K + 1];
#pragma unroll
    for (int c = 0; c <= K; c++) {
        const int ix = x0 - a.pad_left + c;
        col_ok[c] = ix >= 0 && ix < a.w;
        col_off[c] = (long long)ix * a.in_pitch;
    }
    const bool second = x0 + 1 < a.out_w;
    V outside;
#pragma unroll
    for (int i = 0; i < D; i++)
        outside.d[i] = (int)0x80808080;

    // the K + 1 pixels of input row `r` of the strip (rows and columns outside the image count as -128)
    auto load_row = [&](int r, V (&px)[K + 1]) {
        const int iy = y0 - a.pad_top + r;
        const bool row_ok = iy >= 0 && iy < a.h;
        const char *row = img_in + (long long)iy * a.w * a.in_pitch;
#pragma unroll
        for (int c = 0; c <= K; c++)
            px[c] = (row_ok && col_ok[c]) ? load_vec<D>(row + col_off[c]) : outside;
    };

    // horizontal maxima of the last K input rows, as bytes again: [row][column of the pair]
    V hist[K][2];
    const int nrows = a.rows + K - 1;
    for (int base = 0; base < nrows; base += K) {
#pragma unroll
        for (int j = 0; j < K; j++) {
            const int r = base + j;
            V odd[K + 1], even[K + 1];
            load_row(r, odd);
#pragma unroll
            for (int c = 0; c <= K; c++)
#pragma unroll
                for (int i = 0; i < D; i++)
                    even[c].d[i] = odd[c].d[i] << 8;
            // columns 1 .. K-1 are under both windows
            V both_odd = odd[1], both_even = even[1];
#pragma unroll
            for (int c = 2; c < K; c++) {
                both_odd = pkmax(both_odd, odd[c]);
                both_even = pkmax(both_even, even[c]);
            }
            hist[j][0] = join(pkmax(odd[0], both_odd), pkmax(even[0], both_even));
            hist[j][1] = join(pkmax(both_odd, odd[K]), pkmax(both_even, even[K]));
            const int y = y0 + r - (K - 1);
            if (r >= K - 1 && r < nrows && y < a.out_h) {
#pragma unroll
                for (int o = 0; o < 2; o++) {
                    V best_odd = hist[0][o], best_even = shifted(hist[0][o]);
#pragma unroll
                    for (int k = 1; k < K; k++) {
                        best_odd = pkmax(best_odd, hist[k][o]);
                        best_even = pkmax(best_even, shifted(hist[k][o]));
                    }
                    if (o == 0 || second)
                        store_vec<D>(img_out + ((long long)y * a.out_w + x0 + o) * a.out_pitch, join(best_odd, best_even));
                }
            }
        }
    }
}

template <int K>
hipError_t launch_window(const WindowPoolArgs &a, int dwords, hipStream_t stream)
{
    const dim3 grid((a.total + kThreads - 1) / kThreads);
    if (dwords == 4)
        hipLaunchKernelGGL((max_pool_s8_window_kernel<K, 4>), grid, dim3(kThreads), 0, stream, a);
    else
        hipLaunchKernelGGL((max_pool_s8_window_kernel<K, 2>), grid, dim3(kThreads), 0, stream, a);
    return hipGetLastError();
}

} // namespace

bool max_pool_s8_window_supports(const void *in, int h, int w, int c, int k_h, int k_w, int stride_h, int stride_w,
                                 int pad_top, int pad_left, int out_h, int out_w, long long in_pitch, long long out_pitch,
                                 const void *out)
{
    if (k_h != k_w || (k_h != 2 && k_h != 3 && k_h != 5) || stride_h != 1 || stride_w != 1)
        return false;
    if ((c & 7) != 0 || (in_pitch & 7) != 0 || (out_pitch & 7) != 0 ||
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 7) != 0)
        return false;
    // every window must hold a pixel of the image
    if (pad_top >= k_h || pad_left >= k_w || out_h - 1 - pad_top >= h || out_w - 1 - pad_left >= w)
        return false;
    return true;
}

hipError_t launch_max_pool_s8_window(const void *in, int batch, int h, int w, int c, int k, int pad_top, int pad_left,
                                     int out_h, int out_w, long long in_pitch, long long out_pitch, void *out,
                                     int cu_count, hipStream_t stream)
{
    WindowPoolArgs a;
    a.in = static_cast<const char *>(in);
    a.out = static_cast<char *>(out);
    a.h = h;
    a.w = w;
    a.out_h = out_h;
    a.out_w = out_w;
    a.pad_top = pad_top;
    a.pad_left = pad_left;
    // 16 bytes of channels per thread where addresses allow, else 8
    const int dwords = ((c & 15) == 0 && (in_pitch & 15) == 0 && (out_pitch & 15) == 0 &&
                        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) ? 4 : 2;
    a.cv = c / (4 * dwords);
    a.in_pitch = in_pitch;
    a.out_pitch = out_pitch;
    a.xpairs = (out_w + 1) / 2;
    // Strips per image.  Long strips read each input row once; a strip of `rows` rows reads k - 1 rows more
    // (mostly from cache, but the horizontal maxima are taken again).  Short strips give small tensors enough
    // wavefronts, and the count decides how evenly the last round of wavefronts fills the chip (about four
    // wavefronts fit a SIMD).  Measured on 327 images of 80 x 80 x 128: 0.60 of the HBM rate at 5 strips (two
    // full rounds), 0.57 at 4 (2.1 rounds in 3), 0.54 at 8.
    const long long per_row = (long long)batch * a.xpairs * a.cv;
    const double capacity = (double)(cu_count > 0 ? cu_count : 256) * 4 * 4;
    int best_strips = 1;
    double best_score = -1.0;
    for (int strips = 1; strips <= out_h; strips++) {
        const int rows = (out_h + strips - 1) / strips;
        if ((out_h + rows - 1) / rows != strips)
            continue; // the same strip height as a smaller count
        const double waves = (double)per_row * strips / 64.0;
        const double rounds = waves / capacity;
        const double fill = rounds / (double)(long long)(rounds + 0.999999);
        const double score = fill / (1.0 + 0.5 * (k - 1) / rows);
        if (score > best_score * 1.02) { // ties go to the longer strips
            best_score = score;
            best_strips = strips;
        }
    }
    a.strips = best_strips;
    a.rows = (out_h + best_strips - 1) / best_strips;
    const long long total = per_row * a.strips;
    if (total <= 0)
        return hipSuccess;
    if (total > 0x7fffffffll)
        return hipErrorInvalidValue;
    a.total = (unsigned)total;
    a.fd_cv = make_fastdiv((unsigned)a.cv);
    a.fd_xpairs = make_fastdiv((unsigned)a.xpairs);
    a.fd_strips = make_fastdiv((unsigned)a.strips);
    switch (k) {
    case 2:
        return launch_window<2>(a, dwords, stream);
    case 3:
        return launch_window<3>(a, dwords, stream);
    default:
        return launch_window<5>(a, dwords, stream);
    }
}

} // namespace espdl
