// Element-wise binary operators with broadcasting (elemwise_add / _mul / _sub: esp-dl/dl/base/dl_base_add.cpp:8-44,
// dl_base_mul.cpp:33-46, dl_base_sub.cpp), 16 bytes per thread: for operands whose innermost axis is either dense
// or constant (a channel-wise scale [N][1][1][C] against [N][H][W][C], a per-row offset, two dense tensors).  The
// output index is split once per 16-byte piece with 32-bit divisions; an operand that is constant along the
// innermost axis is loaded as one element and repeated.  What the operator does with a pair of elements is the
// caller's functor, the same one its element-at-a-time kernel uses.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace espdl {
namespace binary_vec {

constexpr int kThreads = 256;

struct Args {
    unsigned d1, d2, d3p; // output dims 1, 2 and the innermost one in pieces
    long long s0[4], s1[4]; // element strides; the innermost ones are 0 or 1
    unsigned long long pieces;
};

template <typename T, int V>
struct alignas(sizeof(T) * V) Piece {
    T v[V];
};

template <typename T, typename Op>
__global__ __launch_bounds__(kThreads) void kernel(const T *in0, const T *in1, T *out, const Args a, Op op)
{
    constexpr int V = 16 / (int)sizeof(T);
    using P = Piece<T, V>;
    for (unsigned long long i = (unsigned long long)blockIdx.x * kThreads + threadIdx.x; i < a.pieces;
         i += (unsigned long long)gridDim.x * kThreads) {
        unsigned rest = (unsigned)i;
        const unsigned i3 = rest % a.d3p;
        rest /= a.d3p;
        const unsigned i2 = rest % a.d2;
        rest /= a.d2;
        const unsigned i1 = rest % a.d1;
        const unsigned i0 = rest / a.d1;
        const T *p0 = in0 + (long long)i0 * a.s0[0] + (long long)i1 * a.s0[1] + (long long)i2 * a.s0[2];
        const T *p1 = in1 + (long long)i0 * a.s1[0] + (long long)i1 * a.s1[1] + (long long)i2 * a.s1[2];
        P x, y, r;
        if (a.s0[3] != 0) { // uniform
            x = *reinterpret_cast<const P *>(p0 + (long long)i3 * V);
        } else {
            const T e = *p0;
#pragma unroll
            for (int k = 0; k < V; k++)
                x.v[k] = e;
        }
        if (a.s1[3] != 0) { // uniform
            y = *reinterpret_cast<const P *>(p1 + (long long)i3 * V);
        } else {
            const T e = *p1;
#pragma unroll
            for (int k = 0; k < V; k++)
                y.v[k] = e;
        }
#pragma unroll
        for (int k = 0; k < V; k++)
            r.v[k] = (T)op.apply((int)x.v[k], (int)y.v[k]);
        *reinterpret_cast<P *>(out + i * V) = r;
    }
}

// Fills `a` when the form applies: innermost extent a multiple of the piece, innermost strides 0 or 1, dense
// operands 16-byte aligned with outer strides that keep the alignment, fewer than 2^32 pieces.
template <typename T>
inline bool plan(const int32_t dims[4], const int64_t s0[4], const int64_t s1[4], const T *in0, const T *in1, const T *out,
                 Args *a)
{
    constexpr int V = 16 / (int)sizeof(T);
    if (dims[3] % V != 0 || (reinterpret_cast<uintptr_t>(out) & 15) != 0)
        return false;
    const int64_t *strides[2] = {s0, s1};
    const void *base[2] = {in0, in1};
    long long *dst[2] = {a->s0, a->s1};
    for (int k = 0; k < 2; k++) {
        for (int d = 0; d < 4; d++)
            dst[k][d] = dims[d] > 1 ? strides[k][d] : 0;
        if (dims[3] == 1)
            dst[k][3] = 0;
        if (dst[k][3] == 1) {
            if ((reinterpret_cast<uintptr_t>(base[k]) & 15) != 0)
                return false;
            for (int d = 0; d < 3; d++)
                if (dst[k][d] % V != 0)
                    return false;
        } else if (dst[k][3] != 0) {
            return false;
        }
    }
    const unsigned long long pieces = (unsigned long long)dims[0] * dims[1] * dims[2] * (dims[3] / V);
    if (pieces == 0 || pieces >= (1ull << 32))
        return false;
    a->d1 = (unsigned)dims[1];
    a->d2 = (unsigned)dims[2];
    a->d3p = (unsigned)(dims[3] / V);
    a->pieces = pieces;
    return true;
}

template <typename T, typename Op>
inline hipError_t launch(const T *in0, const T *in1, T *out, const Args &a, Op op, int cu_count, hipStream_t stream)
{
    const unsigned long long want = (a.pieces + kThreads - 1) / kThreads;
    const unsigned long long cap = (unsigned long long)(cu_count > 0 ? cu_count : 256) * 32;
    hipLaunchKernelGGL((kernel<T, Op>), dim3((unsigned)(want < cap ? want : cap)), dim3(kThreads), 0, stream, in0, in1, out, a, op);
    return hipGetLastError();
}

} // namespace binary_vec
} // namespace espdl
