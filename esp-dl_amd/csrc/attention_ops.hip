// Operators of the quantized attention blocks for gfx950: Softmax on int8 with a float32 result,
// QuantizeLinear (float32 -> int8 / int16) and the batched MatMul of two int8 activations.
//
// Softmax follows Softmax::forward_lut (esp-dl/dl/module/include/dl_module_softmax.hpp:148-217): a
// 256-entry float table of expf(scale * (q - 128)), the row sum accumulated in float32 in index order,
// one IEEE division per element.  The row sum is a serial chain by definition, so one lane owns one
// row; everything around it (loads, the divisions, the stores) is done cooperatively and coalesced.
//
// MatMul follows the batched branches of MatMul::forward_template
// (esp-dl/dl/module/include/dl_module_matmul.hpp): every [M,K] x [K,N] pair is a 1x1 convolution with
// one shift, so out = clamp(act(shift_round(sum_k a[m,k] * b[k,n], shift))).
#include "espdl_device.h"
#include "espdl_kernels.h"

namespace espdl {
namespace {

constexpr int kThreads = 256;

struct SoftmaxArgs {
    const int8_t *in;
    float *out;
    long long outer, len, inner;
    int rows_per_block; // rows staged per workgroup (softmax axis innermost)
    int row_stride;     // padded LDS bytes per row
    FastDiv fd_len;     // element (or dword, see vec4) index -> row, without an integer division per element
    int vec4;           // rows are whole dwords at dword-aligned addresses: staged and stored four elements at a time
    float table[256];
};

// Softmax axis innermost: a workgroup stages `rows_per_block` whole rows (one contiguous span of the
// input) in LDS, lane r sums row r in index order, then all lanes divide and store in memory order.
__global__ __launch_bounds__(kThreads) void softmax_s8_rows_kernel(const SoftmaxArgs a)
{
    extern __shared__ __align__(16) unsigned char smem[];
    float *table = reinterpret_cast<float *>(smem);
    float *sums = table + 256;
    int8_t *rows = reinterpret_cast<int8_t *>(sums + a.rows_per_block);
    const int tid = threadIdx.x;
    table[tid] = a.table[tid];
    const long long n_rows = a.outer;
    const int len = (int)a.len;
    for (long long row0 = (long long)blockIdx.x * a.rows_per_block; row0 < n_rows;
         row0 += (long long)gridDim.x * a.rows_per_block) {
        const int rows_here = (int)min((long long)a.rows_per_block, n_rows - row0);
        const int8_t *src = a.in + row0 * len;
        float *dst = a.out + row0 * len;
        __syncthreads(); // table ready / previous span consumed
        if (a.vec4) { // rows of whole dwords at dword-aligned addresses: four elements per access
            const int len4 = len >> 2;
            for (int e = tid; e < rows_here * len4; e += kThreads) {
                const int r = (int)fastdiv((unsigned)e, a.fd_len);
                *reinterpret_cast<int *>(rows + r * a.row_stride + 4 * (e - r * len4)) = reinterpret_cast<const int *>(src)[e];
            }
        } else {
            for (int e = tid; e < rows_here * len; e += kThreads) {
                const int r = (int)fastdiv((unsigned)e, a.fd_len);
                rows[r * a.row_stride + (e - r * len)] = src[e];
            }
        }
        __syncthreads();
        if (tid < rows_here) {
            // four values per LDS read, their table entries fetched together; only the additions form a chain,
            // and they stay in index order
            const int8_t *row = rows + tid * a.row_stride;
            const int *row4 = reinterpret_cast<const int *>(row);
            float sum = 0.f;
            int i = 0;
            for (; i + 4 <= len; i += 4) {
                const int q = row4[i >> 2];
                const float t0 = table[(int)(int8_t)q + 128], t1 = table[(int)(int8_t)(q >> 8) + 128];
                const float t2 = table[(int)(int8_t)(q >> 16) + 128], t3 = table[(q >> 24) + 128];
                sum += t0;
                sum += t1;
                sum += t2;
                sum += t3;
            }
            for (; i < len; i++)
                sum += table[(int)row[i] + 128];
            sums[tid] = sum;
        }
        __syncthreads();
        if (a.vec4) {
            const int len4 = len >> 2;
            for (int e = tid; e < rows_here * len4; e += kThreads) {
                const int r = (int)fastdiv((unsigned)e, a.fd_len);
                const int q = *reinterpret_cast<const int *>(rows + r * a.row_stride + 4 * (e - r * len4));
                const float s = sums[r];
                float4 o;
                o.x = table[(int)(int8_t)q + 128] / s;
                o.y = table[(int)(int8_t)(q >> 8) + 128] / s;
                o.z = table[(int)(int8_t)(q >> 16) + 128] / s;
                o.w = table[(q >> 24) + 128] / s;
                reinterpret_cast<float4 *>(dst)[e] = o;
            }
        } else {
            for (int e = tid; e < rows_here * len; e += kThreads) {
                const int r = (int)fastdiv((unsigned)e, a.fd_len);
                dst[e] = table[(int)rows[r * a.row_stride + (e - r * len)] + 128] / sums[r];
            }
        }
    }
}

// Softmax axis not innermost: lane = one (outer, inner) pair; neighbouring lanes read neighbouring
// addresses at every step of the walk along the axis.
__global__ __launch_bounds__(kThreads) void softmax_s8_strided_kernel(const SoftmaxArgs a)
{
    __shared__ float table[256];
    table[threadIdx.x] = a.table[threadIdx.x];
    __syncthreads();
    const long long n = a.outer * a.inner;
    for (long long t = (long long)blockIdx.x * kThreads + threadIdx.x; t < n; t += (long long)gridDim.x * kThreads) {
        const long long o = t / a.inner, k = t - o * a.inner;
        const int8_t *src = a.in + o * a.len * a.inner + k;
        float *dst = a.out + o * a.len * a.inner + k;
        float sum = 0.f;
        for (long long i = 0; i < a.len; i++)
            sum += table[(int)src[i * a.inner] + 128];
        for (long long i = 0; i < a.len; i++)
            dst[i * a.inner] = table[(int)src[i * a.inner] + 128] / sum;
    }
}

// tool::round(v * inv_scale) then saturate (esp-dl/dl/tensor/src/dl_tensor_base.cpp:17-29)
template <typename T>
__global__ __launch_bounds__(kThreads) void quantize_f32_kernel(const float *__restrict__ in, long long size, float inv_scale,
                                                                T *__restrict__ out)
{
    constexpr int lo = sizeof(T) == 1 ? -128 : -32768, hi = sizeof(T) == 1 ? 127 : 32767;
    for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < size; i += (long long)gridDim.x * kThreads) {
        const int q = round_half_up_f32(in[i] * inv_scale);
        out[i] = (T)min(max(q, lo), hi);
    }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void dequantize_f32_kernel(const T *__restrict__ in, long long size, float scale,
                                                                  float *__restrict__ out)
{
    for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < size; i += (long long)gridDim.x * kThreads)
        out[i] = (float)in[i] * scale;
}

// base::lut_s16_nearest_neighbor with lut_index (esp-dl/dl/base/dl_base_lut.cpp:49-77).  Tables of up to
// 8193 entries are copied to LDS once per workgroup; larger ones are read through the caches.
template <bool LDS_TABLE>
__global__ __launch_bounds__(kThreads) void lut_s16_kernel(const int16_t *__restrict__ in, long long size,
                                                           const int16_t *__restrict__ table, int table_size, int shift,
                                                           int p4_ties, int16_t *__restrict__ out)
{
    extern __shared__ __align__(16) unsigned char smem[];
    const int16_t *t = table;
    if (LDS_TABLE) {
        int16_t *tl = reinterpret_cast<int16_t *>(smem);
        for (int i = threadIdx.x; i < table_size; i += kThreads)
            tl[i] = table[i];
        __syncthreads();
        t = tl;
    }
    for (long long i = (long long)blockIdx.x * kThreads + threadIdx.x; i < size; i += (long long)gridDim.x * kThreads) {
        const unsigned value = (unsigned)(unsigned short)in[i] ^ 0x8000u;
        unsigned index = value >> shift;
        if (shift > 0) {
            const unsigned remainder = value & ((1u << shift) - 1u), half = 1u << (shift - 1);
            if (p4_ties ? (remainder > half || (remainder == half && (index & 1u))) : (remainder >= half))
                index++;
        }
        out[i] = t[index];
    }
}

struct MatMulArgs {
    const int8_t *a, *b;
    int8_t *out;
    int m, k, n;
    int lead[2];                 // broadcast leading extents of the result (outer, inner)
    long long a_stride[2], b_stride[2]; // element strides of each operand per leading dim (0 = broadcast)
    int shift, relu, half_even;
    int vec_a, vec_b; // rows of a (k long) / b (n long) can be read with 8- / 4-byte loads
};

constexpr int kTile = 64;  // output tile edge
constexpr int kChunk = 32; // k per staging step
constexpr int kPad = 4;

// 64 x 64 output tile per workgroup, 4 x 4 outputs per lane; both operands pass through LDS in
// 32-deep k chunks.  The second operand is stored [k][n] in memory; it is transposed while being
// staged so that both LDS tiles hold k innermost and a dword is four consecutive k.
__global__ __launch_bounds__(kThreads) void matmul_s8_kernel(const MatMulArgs p)
{
    __shared__ __align__(16) int8_t as[kTile][kChunk + kPad];
    __shared__ __align__(16) int8_t bs[kTile][kChunk + kPad];
    const int tid = threadIdx.x;
    const int tx = tid & 15, ty = tid >> 4;
    const int bz = blockIdx.z;
    const int z0 = bz / p.lead[1], z1 = bz - z0 * p.lead[1];
    const int8_t *A = p.a + z0 * p.a_stride[0] + z1 * p.a_stride[1];
    const int8_t *B = p.b + z0 * p.b_stride[0] + z1 * p.b_stride[1];
    int8_t *O = p.out + (long long)bz * p.m * p.n;
    const int m0 = blockIdx.y * kTile, n0 = blockIdx.x * kTile;

    int acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
            acc[i][j] = 0;

    for (int k0 = 0; k0 < p.k; k0 += kChunk) {
        __syncthreads();
        // A tile: 64 rows x 32 k, k fastest in memory; 8 consecutive k per lane (one 8-byte load when the
        // row length and the base allow it)
        {
            const int r = tid >> 2, kk = (tid & 3) * 8;
            const int gm = m0 + r;
            if (p.vec_a && gm < p.m && k0 + kk + 8 <= p.k) {
                const int2 v = *reinterpret_cast<const int2 *>(A + (long long)gm * p.k + k0 + kk);
                *reinterpret_cast<int *>(&as[r][kk]) = v.x; // LDS rows are 36 bytes apart: 4-byte aligned only
                *reinterpret_cast<int *>(&as[r][kk + 4]) = v.y;
            } else {
#pragma unroll
                for (int e = 0; e < 8; e++) {
                    const int gk = k0 + kk + e;
                    as[r][kk + e] = (gm < p.m && gk < p.k) ? A[(long long)gm * p.k + gk] : (int8_t)0;
                }
            }
        }
        // B tile: 32 k x 64 n, n fastest in memory; a lane loads four neighbouring n of one k row (or single
        // bytes at the edges) and stores them transposed
        for (int it = tid; it < kChunk * (kTile / 4); it += kThreads) {
            const int kk = it >> 4, c4 = (it & 15) * 4;
            const int gk = k0 + kk, gn = n0 + c4;
            int v = 0;
            if (gk < p.k) {
                if (p.vec_b && gn + 4 <= p.n) {
                    v = *reinterpret_cast<const int *>(B + (long long)gk * p.n + gn);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (gn + e < p.n)
                            v |= (int)(unsigned char)B[(long long)gk * p.n + gn + e] << (8 * e);
                }
            }
#pragma unroll
            for (int e = 0; e < 4; e++)
                bs[c4 + e][kk] = (int8_t)(v >> (8 * e));
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < kChunk; kk += 4) {
            int av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                av[i] = *reinterpret_cast<const int *>(&as[ty * 4 + i][kk]);
#pragma unroll
            for (int j = 0; j < 4; j++)
                bv[j] = *reinterpret_cast<const int *>(&bs[tx * 4 + j][kk]);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_sdot4(av[i], bv[j], acc[i][j], false);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int gm = m0 + ty * 4 + i;
        if (gm >= p.m)
            continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int gn = n0 + tx * 4 + j;
            if (gn < p.n)
                O[(long long)gm * p.n + gn] = (int8_t)requant_s8(acc[i][j], p.shift, p.relu != 0, p.half_even != 0);
        }
    }
}

} // namespace

hipError_t launch_softmax_s8(const int8_t *in, long long outer, long long len, long long inner, int in_exp, float *out,
                             int cu_count, hipStream_t stream)
{
    SoftmaxArgs a = {};
    a.in = in;
    a.out = out;
    a.outer = outer;
    a.len = len;
    a.inner = inner;
    const float scale = dl_scale(in_exp);
    for (int i = 0; i < 256; i++)
        a.table[i] = expf(scale * (float)(i - 128));
    // rows staged in LDS: padded so that neighbouring rows start in different banks
    int stride = (int)((len + 3) & ~3ll);
    if (((stride >> 2) & 1) == 0)
        stride += 4;
    const long long lds_budget = 96 * 1024;
    if (inner == 1 && (long long)stride * 8 <= lds_budget) {
        int rows = (int)min((long long)kThreads, lds_budget / stride);
        rows = (int)min((long long)rows, outer);
        // fewer rows per workgroup while that leaves under two workgroups per compute unit (down to one wavefront
        // of row sums): the staging and the divisions of several workgroups then overlap on a compute unit
        while (rows > 64 && (outer + rows - 1) / rows < 2ll * max(1, cu_count))
            rows = (rows + 1) / 2;
        a.rows_per_block = rows;
        a.row_stride = stride;
        a.vec4 = (len & 3) == 0 && (reinterpret_cast<uintptr_t>(in) & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
        a.fd_len = make_fastdiv((unsigned)(a.vec4 ? len / 4 : len));
        const size_t lds = 256 * sizeof(float) + (size_t)rows * sizeof(float) + (size_t)rows * stride;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(softmax_s8_rows_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess)
            return e;
        const long long blocks = min((outer + rows - 1) / rows, (long long)cu_count * 8);
        softmax_s8_rows_kernel<<<dim3((unsigned)blocks), dim3(kThreads), lds, stream>>>(a);
        return hipGetLastError();
    }
    const long long n = outer * inner;
    const long long blocks = min((n + kThreads - 1) / kThreads, (long long)cu_count * 16);
    softmax_s8_strided_kernel<<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(a);
    return hipGetLastError();
}

hipError_t launch_quantize_f32(const float *in, long long size, int out_exp, int elem_size, void *out, int cu_count,
                               hipStream_t stream)
{
    const long long blocks = min((size + kThreads - 1) / kThreads, (long long)cu_count * 16);
    const float inv_scale = dl_rescale(out_exp);
    if (elem_size == 1)
        quantize_f32_kernel<int8_t><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(in, size, inv_scale,
                                                                                            static_cast<int8_t *>(out));
    else
        quantize_f32_kernel<int16_t><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(in, size, inv_scale,
                                                                                             static_cast<int16_t *>(out));
    return hipGetLastError();
}

hipError_t launch_dequantize_f32(const void *in, long long size, int in_exp, int elem_size, float *out, int cu_count,
                                 hipStream_t stream)
{
    const long long blocks = min((size + kThreads - 1) / kThreads, (long long)cu_count * 16);
    const float scale = dl_scale(in_exp);
    if (elem_size == 1)
        dequantize_f32_kernel<int8_t><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(static_cast<const int8_t *>(in),
                                                                                              size, scale, out);
    else
        dequantize_f32_kernel<int16_t><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(
            static_cast<const int16_t *>(in), size, scale, out);
    return hipGetLastError();
}

hipError_t launch_lut_s16(const int16_t *in, long long size, const int16_t *table, int table_size, int shift, bool p4_ties,
                          int16_t *out, int cu_count, hipStream_t stream)
{
    const long long blocks = min((size + kThreads - 1) / kThreads, (long long)cu_count * 8);
    if (table_size <= 8193)
        lut_s16_kernel<true><<<dim3((unsigned)blocks), dim3(kThreads), (size_t)table_size * 2, stream>>>(
            in, size, table, table_size, shift, p4_ties ? 1 : 0, out);
    else
        lut_s16_kernel<false><<<dim3((unsigned)blocks), dim3(kThreads), 0, stream>>>(in, size, table, table_size, shift,
                                                                                      p4_ties ? 1 : 0, out);
    return hipGetLastError();
}

hipError_t launch_matmul_s8(const int8_t *a, const int8_t *b, int m, int k, int n, const int lead[2],
                            const long long a_stride[2], const long long b_stride[2], int shift, bool relu, bool half_even,
                            int8_t *out, hipStream_t stream)
{
    MatMulArgs p = {};
    p.a = a;
    p.b = b;
    p.out = out;
    p.m = m;
    p.k = k;
    p.n = n;
    for (int i = 0; i < 2; i++) {
        p.lead[i] = lead[i];
        p.a_stride[i] = a_stride[i];
        p.b_stride[i] = b_stride[i];
    }
    p.shift = shift;
    p.relu = relu;
    p.half_even = half_even;
    p.vec_a = (k % 8) == 0 && (reinterpret_cast<uintptr_t>(a) & 7) == 0 && (a_stride[0] % 8) == 0 && (a_stride[1] % 8) == 0;
    p.vec_b = (n % 4) == 0 && (reinterpret_cast<uintptr_t>(b) & 3) == 0 && (b_stride[0] % 4) == 0 && (b_stride[1] % 4) == 0;
    const dim3 grid((unsigned)((n + kTile - 1) / kTile), (unsigned)((m + kTile - 1) / kTile), (unsigned)(lead[0] * lead[1]));
    matmul_s8_kernel<<<grid, dim3(kThreads), 0, stream>>>(p);
    return hipGetLastError();
}

} // namespace espdl
