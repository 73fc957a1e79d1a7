// Data-movement operators of detection necks for gfx950: Concat, Split (row copies), Transpose,
// Resize (nearest) and MaxPool.  All are HBM-bound byte movers: every path moves 16 bytes per thread
// when pointers, pitches and channel counts allow, and falls back to narrower accesses otherwise.
//
// Reference behaviour:
//   Concat     esp-dl/dl/module/include/dl_module_concat.hpp:86-108  (loop_times x one run per input)
//   Split      esp-dl/dl/module/include/dl_module_split.hpp:84-93    (num_slices runs per output)
//   Transpose  esp-dl/dl/tensor/src/dl_tensor_base.cpp:722-812
//   Resize     esp-dl/dl/base/dl_base_resize.cpp:7-34, 236-268 (nearest; "asymmetric" coordinates)
//   MaxPool    esp-dl/dl/base/dl_base_max_pool2d.cpp:9-29 on the window clipped to the image
#include "espdl_device.h"
#include "espdl_kernels.h"
#include "reduce_mid.h"

namespace espdl {

namespace {

constexpr int kBlock = 256;
constexpr int kMaxSeg = 8;

// ------------------------------------------------------------------------------------------------
// Row copies: `rows` runs of `row_bytes` bytes, run r at src + r * src_pitch -> dst + r * dst_pitch.
// ------------------------------------------------------------------------------------------------
struct RowSeg {
    const char *src;
    char *dst;
    long long src_pitch, dst_pitch, row_bytes;
    int vec;        // bytes per access: 16, 4 or 1
    FastDiv per_row; // accesses per row
};
struct RowCopyArgs {
    RowSeg seg[kMaxSeg];
    long long rows;
};

// Four pieces per thread and pass: the four loads are requested before the first store, so that enough bytes are
// in flight to cover the memory latency (one piece per thread moved 4.3 TB/s, a plain copy's rate is above 6).
__global__ __launch_bounds__(kBlock) void copy_rows_kernel(const RowCopyArgs a)
{
    const RowSeg &s = a.seg[blockIdx.y];
    const long long total = a.rows * s.per_row.d;
    const long long stride = (long long)gridDim.x * kBlock;
    const bool small = total <= 0x7fffffffll; // range in which fastdiv is exact
    auto locate = [&](long long i, const char *&sp, char *&dp) {
        long long r;
        unsigned c;
        if (small) {
            r = fastdiv((unsigned)i, s.per_row);
            c = (unsigned)i - (unsigned)r * s.per_row.d;
        } else {
            r = i / s.per_row.d;
            c = (unsigned)(i - r * s.per_row.d);
        }
        sp = s.src + r * s.src_pitch + (long long)c * s.vec;
        dp = s.dst + r * s.dst_pitch + (long long)c * s.vec;
    };
    for (long long i0 = (long long)blockIdx.x * kBlock + threadIdx.x; i0 < total; i0 += 4 * stride) {
        if (s.vec == 16) {
            v4i v[4];
            char *dp[4];
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const long long i = i0 + j * stride;
                const char *sp;
                locate(i < total ? i : i0, sp, dp[j]);
                v[j] = *reinterpret_cast<const v4i *>(sp);
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (i0 + j * stride < total)
                    *reinterpret_cast<v4i *>(dp[j]) = v[j];
        } else {
            for (int j = 0; j < 4; j++) {
                const long long i = i0 + j * stride;
                if (i >= total)
                    break;
                const char *sp;
                char *dp;
                locate(i, sp, dp);
                if (s.vec == 4)
                    *reinterpret_cast<int *>(dp) = *reinterpret_cast<const int *>(sp);
                else
                    *dp = *sp;
            }
        }
    }
}

inline int widest_access(const void *a, const void *b, long long p0, long long p1, long long n)
{
    const uintptr_t m = reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | (uintptr_t)p0 | (uintptr_t)p1 |
        (uintptr_t)n;
    return (m & 15) == 0 ? 16 : ((m & 3) == 0 ? 4 : 1);
}

inline bool fill_seg(RowSeg &s, const void *src, long long src_pitch, void *dst, long long dst_pitch, long long row_bytes)
{
    s.src = static_cast<const char *>(src);
    s.dst = static_cast<char *>(dst);
    s.src_pitch = src_pitch;
    s.dst_pitch = dst_pitch;
    s.row_bytes = row_bytes;
    s.vec = widest_access(src, dst, src_pitch, dst_pitch, row_bytes);
    const long long per_row = row_bytes / s.vec;
    if (per_row > 0x7fffffffll)
        return false;
    s.per_row = make_fastdiv((unsigned)std::max<long long>(per_row, 1));
    return true;
}

inline unsigned blocks_for(long long work, int cu_count)
{
    const long long want = (work + 4 * kBlock - 1) / (4 * kBlock); // four pieces per thread and pass
    const long long cap = (long long)(cu_count > 0 ? cu_count : 256) * 32; // grid-stride beyond this
    return (unsigned)std::max<long long>(1, std::min(want, cap));
}

// ------------------------------------------------------------------------------------------------
// Transpose.  Dimensions are first simplified on the host (size-1 dims dropped, dims that stay
// adjacent merged).  If the innermost dim stays innermost the copy is a gather of contiguous runs
// (general kernel, coalesced on both sides); otherwise a 32x32 tile goes through LDS so that reads
// run along the input's innermost dim and writes along the output's.
// ------------------------------------------------------------------------------------------------
constexpr int kMaxDims = 8;
struct TransposeArgs {
    const char *in;
    char *out;
    int dims, esize;
    long long total;
    int out_shape[kMaxDims];       // output extents, outermost first
    long long in_stride[kMaxDims]; // element stride in the input of output dim i
    // tiled path: a = input innermost dim, b = the input dim that becomes the output's innermost
    int ext_a, ext_b;
    long long a_out_stride, b_in_stride;
    int n_batch_dims;
    int batch_shape[kMaxDims];
    long long batch_in_stride[kMaxDims], batch_out_stride[kMaxDims];
    int tiles_a, tiles_b;
};

template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_general_kernel(const TransposeArgs a)
{
    const T *in = reinterpret_cast<const T *>(a.in);
    T *out = reinterpret_cast<T *>(a.out);
    for (long long o = (long long)blockIdx.x * kBlock + threadIdx.x; o < a.total; o += (long long)gridDim.x * kBlock) {
        long long rem = o, src = 0;
        for (int d = a.dims - 1; d >= 0; d--) {
            const long long q = rem / a.out_shape[d];
            src += (rem - q * a.out_shape[d]) * a.in_stride[d];
            rem = q;
        }
        out[o] = in[src];
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void transpose_tiled_kernel(const TransposeArgs a)
{
    __shared__ T tile[32][33];
    const T *in = reinterpret_cast<const T *>(a.in);
    T *out = reinterpret_cast<T *>(a.out);
    long long blk = blockIdx.x;
    const int ta = (int)(blk % a.tiles_a);
    blk /= a.tiles_a;
    const int tb = (int)(blk % a.tiles_b);
    blk /= a.tiles_b;
    long long in_base = 0, out_base = 0;
    for (int d = a.n_batch_dims - 1; d >= 0; d--) {
        const long long q = blk / a.batch_shape[d];
        const long long i = blk - q * a.batch_shape[d];
        in_base += i * a.batch_in_stride[d];
        out_base += i * a.batch_out_stride[d];
        blk = q;
    }
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5; // 32 x 8 threads
    const int a0 = ta * 32, b0 = tb * 32;
#pragma unroll
    for (int r = ty; r < 32; r += 8)
        if (b0 + r < a.ext_b && a0 + tx < a.ext_a)
            tile[r][tx] = in[in_base + (long long)(b0 + r) * a.b_in_stride + (a0 + tx)];
    __syncthreads();
#pragma unroll
    for (int r = ty; r < 32; r += 8)
        if (a0 + r < a.ext_a && b0 + tx < a.ext_b)
            out[out_base + (long long)(a0 + r) * a.a_out_stride + (b0 + tx)] = tile[tx][r];
}

// ------------------------------------------------------------------------------------------------
// Resize (nearest) and MaxPool: one thread per (output pixel, channel vector).
// ------------------------------------------------------------------------------------------------
struct ResizeArgs {
    const int8_t *in;
    int8_t *out;
    int h, w, c, out_h, out_w;
    float scale_h_inv, scale_w_inv;
    int exact2;
    int rshift, lshift; // value = wrap8((x + round) >> rshift) or wrap8(x << lshift)
    int vec;            // channels per thread: 16 or 1
    FastDiv fd_cv, fd_ow, fd_oh;
    long long total;
    long long in_pitch, out_pitch; // elements from pixel to pixel (c when dense)
};

__device__ __forceinline__ int resize_value(int x, int rshift, int lshift)
{
    // round((float)x * 2^lshift / 2^rshift) with round = floor(v + 0.5): exact in integers
    return rshift > 0 ? (x + (1 << (rshift - 1))) >> rshift : x << lshift;
}

__global__ __launch_bounds__(kBlock) void resize_nearest_s8_kernel(const ResizeArgs a)
{
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < a.total; i += (long long)gridDim.x * kBlock) {
        // i = ((n * out_h + y) * out_w + x) * cv + v; the host refuses totals of 2^31 and more
        const unsigned pix = fastdiv((unsigned)i, a.fd_cv);
        const unsigned v = (unsigned)i - pix * a.fd_cv.d;
        const unsigned row = fastdiv(pix, a.fd_ow);
        const unsigned x = pix - row * a.fd_ow.d;
        const unsigned n = fastdiv(row, a.fd_oh);
        const unsigned y = row - n * a.fd_oh.d;
        int in_y = a.exact2 ? (int)(y >> 1) : (int)((float)y * a.scale_h_inv);
        int in_x = a.exact2 ? (int)(x >> 1) : (int)((float)x * a.scale_w_inv);
        in_y = min(in_y, a.h - 1);
        in_x = min(in_x, a.w - 1);
        const long long src = (((long long)n * a.h + in_y) * a.w + in_x) * a.in_pitch + (long long)v * a.vec;
        const long long dst = (long long)pix * a.out_pitch + (long long)v * a.vec;
        if (a.vec == 16) {
            v4i d = *reinterpret_cast<const v4i *>(a.in + src);
            if (a.rshift | a.lshift) {
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    int o = 0;
#pragma unroll
                    for (int b = 0; b < 4; b++)
                        o |= (resize_value((int)(int8_t)(d[k] >> (8 * b)), a.rshift, a.lshift) & 0xff) << (8 * b);
                    d[k] = o;
                }
            }
            *reinterpret_cast<v4i *>(a.out + dst) = d;
        } else {
            a.out[dst] = (int8_t)resize_value((int)a.in[src], a.rshift, a.lshift);
        }
    }
}

// Exactly 2 x 2 on 16-byte channel vectors: a thread reads one input piece and writes the four output pixels that
// replicate it (one load instead of four; the value is rescaled once).
__global__ __launch_bounds__(kBlock) void resize_nearest2x_s8_kernel(const ResizeArgs a)
{
    // a.total counts INPUT pieces here: i = ((n * h + y) * w + x) * cv + v
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < a.total; i += (long long)gridDim.x * kBlock) {
        const unsigned pix = fastdiv((unsigned)i, a.fd_cv);
        const unsigned v = (unsigned)i - pix * a.fd_cv.d;
        const unsigned row = fastdiv(pix, a.fd_ow); // fd_ow / fd_oh hold the INPUT width / height in this kernel
        const unsigned x = pix - row * a.fd_ow.d;
        const unsigned n = fastdiv(row, a.fd_oh);
        const unsigned y = row - n * a.fd_oh.d;
        v4i d = *reinterpret_cast<const v4i *>(a.in + (long long)pix * a.in_pitch + (long long)v * 16);
        if (a.rshift | a.lshift) {
#pragma unroll
            for (int k = 0; k < 4; k++) {
                int o = 0;
#pragma unroll
                for (int b = 0; b < 4; b++)
                    o |= (resize_value((int)(int8_t)(d[k] >> (8 * b)), a.rshift, a.lshift) & 0xff) << (8 * b);
                d[k] = o;
            }
        }
        int8_t *dst = a.out + (((long long)n * a.out_h + 2 * y) * a.out_w + 2 * x) * a.out_pitch + (long long)v * 16;
        const long long down = (long long)a.out_w * a.out_pitch;
        *reinterpret_cast<v4i *>(dst) = d;
        *reinterpret_cast<v4i *>(dst + a.out_pitch) = d;
        *reinterpret_cast<v4i *>(dst + down) = d;
        *reinterpret_cast<v4i *>(dst + down + a.out_pitch) = d;
    }
}

struct InsertZerosArgs {
    const char *in;
    char *out;
    int h, w, out_h, out_w, stride_h, stride_w;
    int pixel_bytes, vec; // bytes per pixel (channels * element size) and bytes per lane (16, 4 or 1)
    long long total;
    FastDiv fd_cv, fd_ow, fd_oh;
};

// InsertZeros::forward_template (esp-dl/dl/module/include/dl_module_insert_zeros.hpp): input pixel (h, w)
// lands on output pixel (h * stride_h, w * stride_w); every other output pixel is zero.  Written as a
// gather over the output so that each byte is stored once.
__global__ __launch_bounds__(kBlock) void insert_zeros_kernel(const InsertZerosArgs a)
{
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < a.total; i += (long long)gridDim.x * kBlock) {
        const unsigned pix = fastdiv((unsigned)i, a.fd_cv);
        const unsigned v = (unsigned)i - pix * a.fd_cv.d;
        const unsigned row = fastdiv(pix, a.fd_ow);
        const unsigned x = pix - row * a.fd_ow.d;
        const unsigned n = fastdiv(row, a.fd_oh);
        const unsigned y = row - n * a.fd_oh.d;
        const unsigned iy = y / (unsigned)a.stride_h, ix = x / (unsigned)a.stride_w;
        const bool hit = iy * a.stride_h == y && ix * a.stride_w == x && iy < (unsigned)a.h && ix < (unsigned)a.w;
        const long long src = (((long long)n * a.h + iy) * a.w + ix) * a.pixel_bytes + (long long)v * a.vec;
        const long long dst = (long long)pix * a.pixel_bytes + (long long)v * a.vec;
        if (a.vec == 16)
            *reinterpret_cast<v4i *>(a.out + dst) = hit ? *reinterpret_cast<const v4i *>(a.in + src) : v4i{0, 0, 0, 0};
        else if (a.vec == 4)
            *reinterpret_cast<int *>(a.out + dst) = hit ? *reinterpret_cast<const int *>(a.in + src) : 0;
        else
            a.out[dst] = hit ? a.in[src] : (char)0;
    }
}

struct PoolArgs {
    const char *in;
    char *out;
    int h, w, c, out_h, out_w;
    int k_h, k_w, stride_h, stride_w, pad_top, pad_left;
    int vec; // elements per thread: 16 / 8 (vector path) or 1
    FastDiv fd_cv, fd_ow, fd_oh;
    long long total;
    long long in_pitch, out_pitch; // elements from pixel to pixel (c when dense)
};

typedef signed char v16c __attribute__((ext_vector_type(16)));
typedef short v8s __attribute__((ext_vector_type(8)));

template <typename T, typename V>
__global__ __launch_bounds__(kBlock) void max_pool_kernel(const PoolArgs a)
{
    const T *in = reinterpret_cast<const T *>(a.in);
    T *out = reinterpret_cast<T *>(a.out);
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < a.total; i += (long long)gridDim.x * kBlock) {
        const unsigned pix = fastdiv((unsigned)i, a.fd_cv);
        const unsigned v = (unsigned)i - pix * a.fd_cv.d;
        const unsigned row = fastdiv(pix, a.fd_ow);
        const unsigned x = pix - row * a.fd_ow.d;
        const unsigned n = fastdiv(row, a.fd_oh);
        const unsigned y = row - n * a.fd_oh.d;
        const int iy0 = (int)y * a.stride_h - a.pad_top, ix0 = (int)x * a.stride_w - a.pad_left;
        const int ky0 = max(0, -iy0), ky1 = min(a.k_h, a.h - iy0);
        const int kx0 = max(0, -ix0), kx1 = min(a.k_w, a.w - ix0);
        const long long img = (long long)n * a.h * a.w;
        const long long dst = (long long)pix * a.out_pitch + (long long)v * a.vec;
        if (a.vec > 1 && sizeof(T) == 1) {
            // No byte-wise maximum exists: int16 pairs instead.  The raw dword orders like its odd bytes (the
            // low byte of each half only breaks ties), the dword shifted left by 8 like its even bytes.
            const v4i lowest = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
            v4i odd = lowest, even = lowest;
            bool have = false;
            for (int ky = ky0; ky < ky1; ky++)
                for (int kx = kx0; kx < kx1; kx++) {
                    const v4i cur = *reinterpret_cast<const v4i *>(in + (img + (long long)(iy0 + ky) * a.w + (ix0 + kx)) * a.in_pitch +
                                                                   (long long)v * a.vec);
#pragma unroll
                    for (int d = 0; d < 4; d++) {
                        odd[d] = pk_max_i16(odd[d], cur[d]);
                        even[d] = pk_max_i16(even[d], cur[d] << 8);
                    }
                    have = true;
                }
            v4i res;
#pragma unroll
            for (int d = 0; d < 4; d++) // an empty clipped window (pads >= kernel) stores zeros
                res[d] = have ? (int)__builtin_amdgcn_perm((unsigned)odd[d], (unsigned)even[d], 0x07030501u) : 0;
            *reinterpret_cast<v4i *>(out + dst) = res;
        } else if (a.vec > 1) {
            V best = {}; // an empty clipped window (pads >= kernel) stores zeros
            bool have = false;
            for (int ky = ky0; ky < ky1; ky++)
                for (int kx = kx0; kx < kx1; kx++) {
                    const V cur = *reinterpret_cast<const V *>(in + (img + (long long)(iy0 + ky) * a.w + (ix0 + kx)) * a.in_pitch +
                                                               (long long)v * a.vec);
                    best = have ? __builtin_elementwise_max(best, cur) : cur;
                    have = true;
                }
            *reinterpret_cast<V *>(out + dst) = best;
        } else {
            int best = 0;
            bool have = false;
            for (int ky = ky0; ky < ky1; ky++)
                for (int kx = kx0; kx < kx1; kx++) {
                    const int cur = in[(img + (long long)(iy0 + ky) * a.w + (ix0 + kx)) * a.in_pitch + v];
                    best = have ? max(best, cur) : cur;
                    have = true;
                }
            out[dst] = (T)best;
        }
    }
}

// AveragePool (esp-dl/dl/base/dl_base_avg_pool2d.cpp:28-54): int32 sums over the clipped window, one
// float multiply, round half up, clamp.  One thread per (output pixel, 16 channels) or per element.
struct AvgPoolArgs {
    PoolArgs p;
    float scale;
};

__global__ __launch_bounds__(kBlock) void avg_pool_s8_kernel(const AvgPoolArgs args)
{
    const PoolArgs &a = args.p;
    const int8_t *in = reinterpret_cast<const int8_t *>(a.in);
    int8_t *out = reinterpret_cast<int8_t *>(a.out);
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < a.total; i += (long long)gridDim.x * kBlock) {
        const unsigned pix = fastdiv((unsigned)i, a.fd_cv);
        const unsigned v = (unsigned)i - pix * a.fd_cv.d;
        const unsigned row = fastdiv(pix, a.fd_ow);
        const unsigned x = pix - row * a.fd_ow.d;
        const unsigned n = fastdiv(row, a.fd_oh);
        const unsigned y = row - n * a.fd_oh.d;
        const int iy0 = (int)y * a.stride_h - a.pad_top, ix0 = (int)x * a.stride_w - a.pad_left;
        const int ky0 = max(0, -iy0), ky1 = min(a.k_h, a.h - iy0);
        const int kx0 = max(0, -ix0), kx1 = min(a.k_w, a.w - ix0);
        const long long img = (long long)n * a.h * a.w;
        const long long dst = (long long)pix * a.c + (long long)v * a.vec;
        if (a.vec == 16) {
            int sum[16];
#pragma unroll
            for (int k = 0; k < 16; k++)
                sum[k] = 0;
            for (int ky = ky0; ky < ky1; ky++)
                for (int kx = kx0; kx < kx1; kx++) {
                    const v4i cur = *reinterpret_cast<const v4i *>(in + (img + (long long)(iy0 + ky) * a.w + (ix0 + kx)) * a.c +
                                                                   (long long)v * 16);
#pragma unroll
                    for (int k = 0; k < 16; k++)
                        sum[k] += (int)(int8_t)(cur[k >> 2] >> (8 * (k & 3)));
                }
            v4i r;
#pragma unroll
            for (int wd = 0; wd < 4; wd++) {
                int o = 0;
#pragma unroll
                for (int b = 0; b < 4; b++)
                    o |= (clamp_s8(round_half_up_f32((float)sum[4 * wd + b] * args.scale)) & 0xff) << (8 * b);
                r[wd] = o;
            }
            *reinterpret_cast<v4i *>(out + dst) = r;
        } else {
            int sum = 0;
            for (int ky = ky0; ky < ky1; ky++)
                for (int kx = kx0; kx < kx1; kx++)
                    sum += in[(img + (long long)(iy0 + ky) * a.w + (ix0 + kx)) * a.c + v];
            out[dst] = (int8_t)clamp_s8(round_half_up_f32((float)sum * args.scale));
        }
    }
}

// ReduceMean (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:16-45): one thread per output element
// walks the reduced axes; the float expression is the reference's, left to right.
struct ReduceArgs {
    const int8_t *in;
    int8_t *out;
    int n_kept, n_red;
    int kept_shape[kMaxDims], red_shape[kMaxDims];
    long long kept_stride[kMaxDims], red_stride[kMaxDims];
    long long n_out, count;
    int lanes; // lanes per output: a power of two, 1..64
    float input_scale, output_scale;
};

// Each output is summed by `a.lanes` lanes of one wavefront (a power of two up to 64): neighbouring lanes hold
// neighbouring outputs, the lanes of one output sit 64 / lanes apart and walk the reduced elements with that
// stride; integer partial sums are combined with cross-lane adds, so the order does not matter.
__global__ __launch_bounds__(kBlock) void reduce_mean_s8_kernel(const ReduceArgs a)
{
    const int per_wave = 64 / a.lanes; // outputs per wavefront
    const int lane = threadIdx.x & 63;
    const int o_local = lane % per_wave, part = lane / per_wave;
    const long long waves = ((long long)gridDim.x * kBlock) >> 6;
    const long long n_groups = (a.n_out + per_wave - 1) / per_wave;
    for (long long grp = ((long long)blockIdx.x * kBlock + threadIdx.x) >> 6; grp < n_groups; grp += waves) {
        const long long o = grp * per_wave + o_local;
        int sum = 0;
        if (o < a.n_out) {
            long long rem = o, base = 0;
            for (int d = a.n_kept - 1; d >= 0; d--) {
                const long long q = rem / a.kept_shape[d];
                base += (rem - q * a.kept_shape[d]) * a.kept_stride[d];
                rem = q;
            }
            for (long long r = part; r < a.count; r += a.lanes) {
                long long rr = r, off = base;
                for (int d = a.n_red - 1; d >= 0; d--) {
                    const long long q = rr / a.red_shape[d];
                    off += (rr - q * a.red_shape[d]) * a.red_stride[d];
                    rr = q;
                }
                sum += a.in[off];
            }
        }
        for (int step = 32; step >= per_wave; step >>= 1)
            sum += __shfl_xor(sum, step, 64);
        if (o < a.n_out && part == 0) {
            const float v = (float)sum * a.input_scale / (float)a.count * a.output_scale;
            a.out[o] = (int8_t)clamp_s8(round_half_up_f32(v));
        }
    }
}

} // namespace

hipError_t launch_copy_rows(const void *src, long long src_pitch, void *dst, long long dst_pitch, long long row_bytes,
                            long long rows, int cu_count, hipStream_t stream)
{
    if (rows <= 0 || row_bytes <= 0)
        return hipSuccess;
    RowCopyArgs a;
    a.rows = rows;
    if (!fill_seg(a.seg[0], src, src_pitch, dst, dst_pitch, row_bytes))
        return hipErrorInvalidValue;
    hipLaunchKernelGGL(copy_rows_kernel, dim3(blocks_for(rows * a.seg[0].per_row.d, cu_count), 1), dim3(kBlock), 0, stream,
                       a);
    return hipGetLastError();
}

namespace {
// Concat walked in OUTPUT order: piece o of the output (16 bytes) lies in row o / per_row at column o % per_row,
// and the column says which input it comes from.  Every store of a wavefront is then a run of whole cache lines;
// with one pass per input the two halves of a 128-byte line arrive from different workgroups at different times
// (measured on 64 + 64 channels: 4.2 TB/s per-input, see the table in the kernel list for this form).
struct ConcatArgs {
    const char *src[kMaxSeg];
    unsigned first[kMaxSeg + 1]; // first output piece (of a row) of input j; first[n] = pieces per row
    unsigned pieces[kMaxSeg];    // pieces per row of input j
    int n;
    char *dst;
    long long rows;
    FastDiv per_row;
};

__global__ __launch_bounds__(kBlock) void concat_rows_kernel(const ConcatArgs a)
{
    const long long total = a.rows * a.per_row.d; // below 2^31 (checked on the host)
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long i0 = (long long)blockIdx.x * kBlock + threadIdx.x; i0 < total; i0 += 4 * stride) {
        v4i v[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const long long i = i0 + j * stride < total ? i0 + j * stride : i0;
            const unsigned r = fastdiv((unsigned)i, a.per_row);
            const unsigned c = (unsigned)i - r * a.per_row.d;
            int seg = 0;
#pragma unroll
            for (int k = 1; k < kMaxSeg; k++)
                seg += (k < a.n && c >= a.first[k]) ? 1 : 0;
            v[j] = *reinterpret_cast<const v4i *>(a.src[seg] + ((long long)r * a.pieces[seg] + (c - a.first[seg])) * 16);
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            if (i0 + j * stride < total)
                reinterpret_cast<v4i *>(a.dst)[i0 + j * stride] = v[j];
    }
}

// Split walked in input order: the mirror image.  Piece i of the input (row r, column c) goes to the output the
// column belongs to; every load of a wavefront is a run of whole cache lines of the input, which one pass per
// output reads as half lines twice (measured on 128 -> 64 + 64 channels: 0.44 of the HBM rate per output).
struct SplitArgs {
    char *dst[kMaxSeg];
    unsigned first[kMaxSeg + 1]; // first input piece (of a row) of output j; first[n] = pieces per row
    unsigned pieces[kMaxSeg];    // pieces per row of output j
    int n;
    const char *src;
    long long src_pitch; // bytes from row to row of the input
    long long rows;
    FastDiv per_row;
};

__global__ __launch_bounds__(kBlock) void split_rows_kernel(const SplitArgs a)
{
    const long long total = a.rows * a.per_row.d; // below 2^31 (checked on the host)
    const long long stride = (long long)gridDim.x * kBlock;
    for (long long i0 = (long long)blockIdx.x * kBlock + threadIdx.x; i0 < total; i0 += 4 * stride) {
        v4i v[4];
        unsigned rr[4], cc[4];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const long long i = i0 + j * stride < total ? i0 + j * stride : i0;
            rr[j] = fastdiv((unsigned)i, a.per_row);
            cc[j] = (unsigned)i - rr[j] * a.per_row.d;
            v[j] = *reinterpret_cast<const v4i *>(a.src + (long long)rr[j] * a.src_pitch + (long long)cc[j] * 16);
        }
#pragma unroll
        for (int j = 0; j < 4; j++) {
            if (i0 + j * stride >= total)
                continue;
            int seg = 0;
#pragma unroll
            for (int k = 1; k < kMaxSeg; k++)
                seg += (k < a.n && cc[j] >= a.first[k]) ? 1 : 0;
            if (a.dst[seg] != nullptr) // an output that already lies in the input is not written
                *reinterpret_cast<v4i *>(a.dst[seg] + ((long long)rr[j] * a.pieces[seg] + (cc[j] - a.first[seg])) * 16) = v[j];
        }
    }
}
} // namespace

hipError_t launch_split(const void *in, long long in_pitch, int n_outputs, void *const *outputs, const long long *copy_bytes,
                        long long rows, int cu_count, hipStream_t stream)
{
    long long total = 0;
    for (int j = 0; j < n_outputs; j++)
        total += copy_bytes[j];
    if (rows <= 0 || total <= 0)
        return hipSuccess;
    // input-order form: up to kMaxSeg outputs, everything in whole aligned 16-byte pieces
    bool ok = n_outputs <= kMaxSeg && (reinterpret_cast<uintptr_t>(in) & 15) == 0 && (in_pitch & 15) == 0 &&
        rows * (total / 16) <= 0x7fffffffll;
    SplitArgs a = {};
    unsigned first = 0;
    for (int j = 0; ok && j < n_outputs; j++) {
        ok = (copy_bytes[j] & 15) == 0 && copy_bytes[j] > 0 && (reinterpret_cast<uintptr_t>(outputs[j]) & 15) == 0;
        a.dst[j] = static_cast<char *>(outputs[j]);
        a.first[j] = first;
        a.pieces[j] = (unsigned)(copy_bytes[j] / 16);
        first += a.pieces[j];
    }
    if (ok) {
        for (int k = n_outputs; k <= kMaxSeg; k++)
            a.first[k] = first;
        a.n = n_outputs;
        a.src = static_cast<const char *>(in);
        a.src_pitch = in_pitch;
        a.rows = rows;
        a.per_row = make_fastdiv(first);
        hipLaunchKernelGGL(split_rows_kernel, dim3(blocks_for(rows * first, cu_count)), dim3(kBlock), 0, stream, a);
        return hipGetLastError();
    }
    // one pass per output
    long long prefix = 0;
    for (int j = 0; j < n_outputs; j++) {
        if (outputs[j] != nullptr && copy_bytes[j] > 0) {
            const hipError_t e = launch_copy_rows(static_cast<const char *>(in) + prefix, in_pitch, outputs[j], copy_bytes[j],
                                                  copy_bytes[j], rows, cu_count, stream);
            if (e != hipSuccess)
                return e;
        }
        prefix += copy_bytes[j];
    }
    return hipSuccess;
}

hipError_t launch_concat(int n_inputs, const void *const *inputs, const long long *copy_bytes, long long loop_times,
                         void *out, int cu_count, hipStream_t stream)
{
    long long total = 0;
    for (int j = 0; j < n_inputs; j++)
        total += copy_bytes[j];
    if (loop_times <= 0 || total <= 0)
        return hipSuccess;
    {
        // output-order form: up to kMaxSeg inputs, everything in whole aligned 16-byte pieces
        bool ok = n_inputs <= kMaxSeg && (reinterpret_cast<uintptr_t>(out) & 15) == 0 && (total & 15) == 0 &&
            loop_times * (total / 16) <= 0x7fffffffll;
        ConcatArgs a = {};
        unsigned first = 0;
        int n = 0;
        for (int j = 0; ok && j < n_inputs; j++) {
            if (copy_bytes[j] == 0)
                continue;
            ok = (copy_bytes[j] & 15) == 0 && (reinterpret_cast<uintptr_t>(inputs[j]) & 15) == 0;
            a.src[n] = static_cast<const char *>(inputs[j]);
            a.first[n] = first;
            a.pieces[n] = (unsigned)(copy_bytes[j] / 16);
            first += a.pieces[n];
            n++;
        }
        if (ok && n > 0) {
            for (int k = n; k <= kMaxSeg; k++)
                a.first[k] = first;
            a.n = n;
            a.dst = static_cast<char *>(out);
            a.rows = loop_times;
            a.per_row = make_fastdiv(first);
            hipLaunchKernelGGL(concat_rows_kernel, dim3(blocks_for(loop_times * first, cu_count)), dim3(kBlock), 0, stream, a);
            return hipGetLastError();
        }
    }
    long long prefix = 0;
    for (int j0 = 0; j0 < n_inputs; j0 += kMaxSeg) {
        RowCopyArgs a;
        a.rows = loop_times;
        int n = 0;
        long long most = 0;
        for (int j = j0; j < n_inputs && n < kMaxSeg; j++) {
            if (copy_bytes[j] > 0) {
                if (!fill_seg(a.seg[n], inputs[j], copy_bytes[j], static_cast<char *>(out) + prefix, total, copy_bytes[j]))
                    return hipErrorInvalidValue;
                most = std::max<long long>(most, loop_times * a.seg[n].per_row.d);
                n++;
            }
            prefix += copy_bytes[j];
        }
        if (n > 0)
            hipLaunchKernelGGL(copy_rows_kernel, dim3(blocks_for(most, cu_count), (unsigned)n), dim3(kBlock), 0, stream, a);
    }
    return hipGetLastError();
}

hipError_t launch_transpose(const void *in, const int *shape, int dims, const int *perm, int elem_size, void *out,
                            int cu_count, hipStream_t stream)
{
    // simplify: drop extent-1 dims, then merge input dims that are adjacent and in order in the output
    int s_shape[kMaxDims], s_perm[kMaxDims], n = 0;
    {
        int keep[kMaxDims], newidx[kMaxDims];
        for (int i = 0; i < dims; i++) {
            keep[i] = shape[i] != 1;
            newidx[i] = keep[i] ? n : -1;
            if (keep[i])
                s_shape[n++] = shape[i];
        }
        int m = 0;
        for (int i = 0; i < dims; i++)
            if (keep[perm[i]])
                s_perm[m++] = newidx[perm[i]];
    }
    long long total = 1;
    for (int i = 0; i < dims; i++)
        total *= shape[i];
    if (total == 0)
        return hipSuccess;
    bool merged = true;
    while (merged && n > 1) {
        merged = false;
        for (int i = 0; i + 1 < n; i++)
            if (s_perm[i + 1] == s_perm[i] + 1) { // input dims p, p+1 stay adjacent: one dim
                const int p = s_perm[i];
                s_shape[p] *= s_shape[p + 1];
                for (int k = p + 1; k + 1 < n; k++)
                    s_shape[k] = s_shape[k + 1];
                for (int k = i + 1; k + 1 < n; k++)
                    s_perm[k] = s_perm[k + 1];
                n--;
                for (int k = 0; k < n; k++)
                    if (s_perm[k] > p)
                        s_perm[k]--;
                merged = true;
                break;
            }
    }
    if (n <= 1) // identity
        return hipMemcpyAsync(out, in, (size_t)(total * elem_size), hipMemcpyDeviceToDevice, stream);

    if (s_perm[n - 1] == n - 1) {
        // the innermost axis stays innermost: its runs move in the widest pieces their length and the addresses
        // allow (one index decomposition per 16 bytes instead of per element)
        const uintptr_t addr = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out);
        for (int wide = 16; wide > elem_size; wide >>= 1) {
            const long long run = (long long)s_shape[n - 1] * elem_size;
            if (run % wide == 0 && (addr & (uintptr_t)(wide - 1)) == 0) {
                s_shape[n - 1] = (int)(run / wide);
                total = total * elem_size / wide;
                elem_size = wide;
                break;
            }
        }
    }
    TransposeArgs a = {};
    a.in = static_cast<const char *>(in);
    a.out = static_cast<char *>(out);
    a.dims = n;
    a.esize = elem_size;
    a.total = total;
    long long in_stride[kMaxDims], out_stride[kMaxDims];
    in_stride[n - 1] = 1;
    for (int i = n - 2; i >= 0; i--)
        in_stride[i] = in_stride[i + 1] * s_shape[i + 1];
    for (int i = 0; i < n; i++) {
        a.out_shape[i] = s_shape[s_perm[i]];
        a.in_stride[i] = in_stride[s_perm[i]];
    }
    out_stride[n - 1] = 1;
    for (int i = n - 2; i >= 0; i--)
        out_stride[i] = out_stride[i + 1] * a.out_shape[i + 1];

    if (s_perm[n - 1] != n - 1) {
        // tiled path
        const int da = n - 1, db = s_perm[n - 1];
        int pos_a = 0;
        for (int i = 0; i < n; i++)
            if (s_perm[i] == da)
                pos_a = i;
        a.ext_a = s_shape[da];
        a.ext_b = s_shape[db];
        a.a_out_stride = out_stride[pos_a];
        a.b_in_stride = in_stride[db];
        a.tiles_a = (a.ext_a + 31) / 32;
        a.tiles_b = (a.ext_b + 31) / 32;
        long long blocks = (long long)a.tiles_a * a.tiles_b;
        for (int i = 0; i < n; i++) { // the other dims, in output order
            const int d = s_perm[i];
            if (d == da || d == db)
                continue;
            a.batch_shape[a.n_batch_dims] = s_shape[d];
            a.batch_in_stride[a.n_batch_dims] = in_stride[d];
            a.batch_out_stride[a.n_batch_dims] = out_stride[i];
            a.n_batch_dims++;
            blocks *= s_shape[d];
        }
        if (blocks > 0x7fffffffll)
            return hipErrorInvalidValue;
        const dim3 grid((unsigned)blocks);
        if (elem_size == 1)
            hipLaunchKernelGGL(transpose_tiled_kernel<int8_t>, grid, dim3(kBlock), 0, stream, a);
        else if (elem_size == 2)
            hipLaunchKernelGGL(transpose_tiled_kernel<int16_t>, grid, dim3(kBlock), 0, stream, a);
        else
            hipLaunchKernelGGL(transpose_tiled_kernel<int32_t>, grid, dim3(kBlock), 0, stream, a);
        return hipGetLastError();
    }
    const dim3 grid(blocks_for(total, cu_count));
    if (elem_size == 1)
        hipLaunchKernelGGL(transpose_general_kernel<int8_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 2)
        hipLaunchKernelGGL(transpose_general_kernel<int16_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 4)
        hipLaunchKernelGGL(transpose_general_kernel<int32_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 8)
        hipLaunchKernelGGL(transpose_general_kernel<long long>, grid, dim3(kBlock), 0, stream, a);
    else
        hipLaunchKernelGGL(transpose_general_kernel<v4i>, grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_resize_nearest_s8(const int8_t *in, int batch, int h, int w, int c, int out_h, int out_w, float scale_h,
                                    float scale_w, int in_exp, int out_exp, long long in_pitch, long long out_pitch,
                                    int8_t *out, int cu_count, hipStream_t stream)
{
    ResizeArgs a;
    a.in = in;
    a.out = out;
    a.in_pitch = in_pitch;
    a.out_pitch = out_pitch;
    a.h = h;
    a.w = w;
    a.c = c;
    a.out_h = out_h;
    a.out_w = out_w;
    a.scale_h_inv = 1 / scale_h;
    a.scale_w_inv = 1 / scale_w;
    a.exact2 = scale_h == 2 && scale_w == 2;
    const int d = out_exp - in_exp;
    a.rshift = d > 0 ? d : 0;
    a.lshift = d < 0 ? -d : 0;
    const bool vec_ok = (c & 15) == 0 && (in_pitch & 15) == 0 && (out_pitch & 15) == 0 &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    a.vec = vec_ok ? 16 : 1;
    const int cv = c / a.vec;
    a.total = (long long)batch * out_h * out_w * cv;
    if (a.total <= 0)
        return hipSuccess;
    if (a.total > 0x7fffffffll) // fastdiv range
        return hipErrorInvalidValue;
    a.fd_cv = make_fastdiv((unsigned)cv);
    if (a.exact2 && a.vec == 16 && out_h == 2 * h && out_w == 2 * w) {
        a.total = (long long)batch * h * w * cv;
        a.fd_ow = make_fastdiv((unsigned)w);
        a.fd_oh = make_fastdiv((unsigned)h);
        hipLaunchKernelGGL(resize_nearest2x_s8_kernel, dim3(blocks_for(a.total, cu_count)), dim3(kBlock), 0, stream, a);
        return hipGetLastError();
    }
    a.fd_ow = make_fastdiv((unsigned)out_w);
    a.fd_oh = make_fastdiv((unsigned)out_h);
    hipLaunchKernelGGL(resize_nearest_s8_kernel, dim3(blocks_for(a.total, cu_count)), dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_insert_zeros(const void *in, int elem_size, int batch, int h, int w, int c, int stride_h, int stride_w,
                               int out_h, int out_w, void *out, int cu_count, hipStream_t stream)
{
    InsertZerosArgs a;
    a.in = static_cast<const char *>(in);
    a.out = static_cast<char *>(out);
    a.h = h;
    a.w = w;
    a.out_h = out_h;
    a.out_w = out_w;
    a.stride_h = stride_h;
    a.stride_w = stride_w;
    a.pixel_bytes = c * elem_size;
    const uintptr_t align = reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out);
    a.vec = (a.pixel_bytes % 16 == 0 && (align & 15) == 0) ? 16 : ((a.pixel_bytes % 4 == 0 && (align & 3) == 0) ? 4 : 1);
    const int cv = a.pixel_bytes / a.vec;
    a.total = (long long)batch * out_h * out_w * cv;
    if (a.total <= 0)
        return hipSuccess;
    if (a.total > 0x7fffffffll) // fastdiv range
        return hipErrorInvalidValue;
    a.fd_cv = make_fastdiv((unsigned)cv);
    a.fd_ow = make_fastdiv((unsigned)out_w);
    a.fd_oh = make_fastdiv((unsigned)out_h);
    hipLaunchKernelGGL(insert_zeros_kernel, dim3(blocks_for(a.total, cu_count)), dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_max_pool(const void *in, int elem_size, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                           int stride_w, int pad_top, int pad_left, int out_h, int out_w, long long in_pitch,
                           long long out_pitch, void *out, int cu_count, hipStream_t stream)
{
    if (elem_size == 1 && max_pool_s8_window_supports(in, h, w, c, k_h, k_w, stride_h, stride_w, pad_top, pad_left, out_h,
                                                      out_w, in_pitch, out_pitch, out))
        return launch_max_pool_s8_window(in, batch, h, w, c, k_h, pad_top, pad_left, out_h, out_w, in_pitch, out_pitch, out,
                                         cu_count, stream);
    PoolArgs a;
    a.in = static_cast<const char *>(in);
    a.out = static_cast<char *>(out);
    a.h = h;
    a.w = w;
    a.c = c;
    a.out_h = out_h;
    a.out_w = out_w;
    a.k_h = k_h;
    a.k_w = k_w;
    a.stride_h = stride_h;
    a.stride_w = stride_w;
    a.pad_top = pad_top;
    a.pad_left = pad_left;
    a.in_pitch = in_pitch;
    a.out_pitch = out_pitch;
    const int per_vec = 16 / elem_size;
    const bool vec_ok = (c % per_vec) == 0 && (in_pitch % per_vec) == 0 && (out_pitch % per_vec) == 0 &&
        ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    a.vec = vec_ok ? per_vec : 1;
    const int cv = c / a.vec;
    a.total = (long long)batch * out_h * out_w * cv;
    if (a.total <= 0)
        return hipSuccess;
    if (a.total > 0x7fffffffll) // fastdiv range
        return hipErrorInvalidValue;
    a.fd_cv = make_fastdiv((unsigned)cv);
    a.fd_ow = make_fastdiv((unsigned)out_w);
    a.fd_oh = make_fastdiv((unsigned)out_h);
    const dim3 grid(blocks_for(a.total, cu_count));
    if (elem_size == 1)
        hipLaunchKernelGGL((max_pool_kernel<int8_t, v16c>), grid, dim3(kBlock), 0, stream, a);
    else
        hipLaunchKernelGGL((max_pool_kernel<int16_t, v8s>), grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

hipError_t launch_avg_pool_s8(const int8_t *in, int batch, int h, int w, int c, int k_h, int k_w, int stride_h,
                              int stride_w, int pad_top, int pad_left, int out_h, int out_w, int in_exp, int out_exp,
                              int8_t *out, int cu_count, hipStream_t stream)
{
    AvgPoolArgs args;
    PoolArgs &a = args.p;
    a.in = reinterpret_cast<const char *>(in);
    a.out = reinterpret_cast<char *>(out);
    a.h = h;
    a.w = w;
    a.c = c;
    a.out_h = out_h;
    a.out_w = out_w;
    a.k_h = k_h;
    a.k_w = k_w;
    a.stride_h = stride_h;
    a.stride_w = stride_w;
    a.pad_top = pad_top;
    a.pad_left = pad_left;
    const bool vec_ok = (c & 15) == 0 && ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0;
    a.vec = vec_ok ? 16 : 1;
    const int cv = c / a.vec;
    a.total = (long long)batch * out_h * out_w * cv;
    if (a.total <= 0)
        return hipSuccess;
    if (a.total > 0x7fffffffll) // fastdiv range
        return hipErrorInvalidValue;
    a.fd_cv = make_fastdiv((unsigned)cv);
    a.fd_ow = make_fastdiv((unsigned)out_w);
    a.fd_oh = make_fastdiv((unsigned)out_h);
    // the scale the reference forms, left to right in float32
    const float area_inv = 1.f / (float)(k_h * k_w);
    args.scale = dl_scale(in_exp) * area_inv * dl_rescale(out_exp);
    hipLaunchKernelGGL(avg_pool_s8_kernel, dim3(blocks_for(a.total, cu_count)), dim3(kBlock), 0, stream, args);
    return hipGetLastError();
}

// Slice with positive steps: a gather whose element strides are the input strides times the steps.
hipError_t launch_slice(const void *in, const int *shape, int dims, const int *start, const int *step, const int *out_shape,
                        int elem_size, void *out, int cu_count, hipStream_t stream)
{
    TransposeArgs a = {};
    long long in_stride[kMaxDims];
    in_stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        in_stride[i] = in_stride[i + 1] * shape[i + 1];
    long long base = 0, total = 1;
    for (int i = 0; i < dims; i++) {
        base += (long long)start[i] * in_stride[i];
        a.out_shape[i] = out_shape[i];
        a.in_stride[i] = in_stride[i] * step[i];
        total *= out_shape[i];
    }
    if (total <= 0)
        return hipSuccess;
    a.in = static_cast<const char *>(in) + base * elem_size;
    a.out = static_cast<char *>(out);
    a.dims = dims;
    a.esize = elem_size;
    a.total = total;
    const dim3 grid(blocks_for(total, cu_count));
    if (elem_size == 1)
        hipLaunchKernelGGL(transpose_general_kernel<int8_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 2)
        hipLaunchKernelGGL(transpose_general_kernel<int16_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 4)
        hipLaunchKernelGGL(transpose_general_kernel<int32_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 8)
        hipLaunchKernelGGL(transpose_general_kernel<long long>, grid, dim3(kBlock), 0, stream, a);
    else
        hipLaunchKernelGGL(transpose_general_kernel<v4i>, grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

// Pad (esp-dl/dl/base/dl_base_pad.cpp:19-260, TensorBase::pad esp-dl/dl/tensor/src/dl_tensor_base.cpp:1225-1299):
// every axis is padded on its own, so an output coordinate maps to an input coordinate axis by axis.
// mode 0 constant, 1 edge (clamp), 2 reflect (mirror without repeating the border element).
struct PadArgs {
    const char *in;
    char *out;
    int dims, mode, value;
    int out_shape[kMaxDims], in_shape[kMaxDims], before[kMaxDims];
    long long in_stride[kMaxDims];
    long long total;
};

template <typename T>
__global__ __launch_bounds__(kBlock) void pad_kernel(const PadArgs a)
{
    const T *in = reinterpret_cast<const T *>(a.in);
    T *out = reinterpret_cast<T *>(a.out);
    for (long long i = (long long)blockIdx.x * kBlock + threadIdx.x; i < a.total; i += (long long)gridDim.x * kBlock) {
        long long rem = i, off = 0;
        bool outside = false;
        for (int d = a.dims - 1; d >= 0; d--) {
            const long long q = rem / a.out_shape[d];
            int x = (int)(rem - q * a.out_shape[d]) - a.before[d];
            rem = q;
            const int n = a.in_shape[d];
            if (x < 0 || x >= n) {
                if (a.mode == 0)
                    outside = true;
                else if (a.mode == 1)
                    x = x < 0 ? 0 : n - 1;
                else
                    x = x < 0 ? -x : 2 * (n - 1) - x;
            }
            off += (long long)x * a.in_stride[d];
        }
        out[i] = outside ? (T)a.value : in[off];
    }
}

hipError_t launch_pad(const void *in, const int *shape, int dims, const int *pads, int mode, int value, int elem_size,
                      void *out, int cu_count, hipStream_t stream)
{
    PadArgs a = {};
    a.in = static_cast<const char *>(in);
    a.out = static_cast<char *>(out);
    a.dims = dims;
    a.mode = mode;
    a.value = value;
    a.total = 1;
    long long stride = 1;
    for (int d = dims - 1; d >= 0; d--) {
        a.in_shape[d] = shape[d];
        a.before[d] = pads[d];
        a.out_shape[d] = shape[d] + pads[d] + pads[d + dims];
        a.in_stride[d] = stride;
        stride *= shape[d];
        a.total *= a.out_shape[d];
    }
    if (a.total <= 0)
        return hipSuccess;
    const dim3 grid(blocks_for(a.total, cu_count));
    if (elem_size == 1)
        hipLaunchKernelGGL(pad_kernel<int8_t>, grid, dim3(kBlock), 0, stream, a);
    else if (elem_size == 2)
        hipLaunchKernelGGL(pad_kernel<int16_t>, grid, dim3(kBlock), 0, stream, a);
    else
        hipLaunchKernelGGL(pad_kernel<int32_t>, grid, dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

namespace {
// ReduceMean's float expression on the integer sum, left to right as in the reference
struct MeanFinish8 {
    int8_t *out;
    float input_scale, count, output_scale;
    __device__ void operator()(long long o, int total) const
    {
        out[o] = (int8_t)clamp_s8(round_half_up_f32((float)total * input_scale / count * output_scale));
    }
};
} // namespace

hipError_t launch_reduce_mean_s8(const int8_t *in, const int *shape, int dims, const int *reduce_flag, int in_exp,
                                 int out_exp, int8_t *out, int cu_count, hipStream_t stream)
{
    ReduceArgs a = {};
    long long stride[kMaxDims];
    stride[dims - 1] = 1;
    for (int i = dims - 2; i >= 0; i--)
        stride[i] = stride[i + 1] * shape[i + 1];
    a.n_out = 1;
    a.count = 1;
    for (int i = 0; i < dims; i++) {
        if (reduce_flag[i]) {
            a.red_shape[a.n_red] = shape[i];
            a.red_stride[a.n_red++] = stride[i];
            a.count *= shape[i];
        } else {
            a.kept_shape[a.n_kept] = shape[i];
            a.kept_stride[a.n_kept++] = stride[i];
            a.n_out *= shape[i];
        }
    }
    if (a.n_out <= 0 || a.count <= 0)
        return hipSuccess;
    a.in = in;
    a.out = out;
    a.input_scale = dl_scale(in_exp);
    a.output_scale = dl_rescale(out_exp);
    // the reduced axes are neighbours (a pooled embedding, a mean over time): contiguous loads, every lane busy
    long long outer, r_count, inner;
    if (reduce_mid::mid_view(shape, dims, reduce_flag, &outer, &r_count, &inner) && r_count >= 8 &&
        reduce_mid::fits<int8_t>(outer, r_count, inner))
        return reduce_mid::launch(in, outer, r_count, inner, MeanFinish8{out, a.input_scale, (float)a.count, a.output_scale}, stream);
    // enough lanes per output to occupy the device when there are few outputs and long sums
    a.lanes = 1;
    while (a.lanes < 64 && a.n_out * a.lanes < (long long)max(1, cu_count) * 2048 && a.count >= 4ll * a.lanes)
        a.lanes *= 2;
    hipLaunchKernelGGL(reduce_mean_s8_kernel, dim3(blocks_for(a.n_out * a.lanes, cu_count)), dim3(kBlock), 0, stream, a);
    return hipGetLastError();
}

} // namespace espdl
