// Sum over the middle axis of a contiguous [outer][R][inner] tensor of int8 or int16, the shape GlobalAveragePool
// (NHWC: [N][H W][C], esp-dl/dl/base/dl_base_avg_pool2d.cpp:9-54) and ReduceMean over a run of neighbouring axes
// (esp-dl/dl/module/include/dl_module_reduce_mean.hpp:16-45) reduce to.  The integer sum is exact in any order, so
// the work is laid out for the memory system only; what the operator does with the sum (its float scaling and
// rounding) is the caller's functor, applied once per output.
//
// One workgroup per (outer index, slab of up to 64 groups of VEC consecutive inner elements).  Thread t owns group
// t % G of the slab and the reduced positions t / G, t / G + PS, ... (PS = 256 / G): consecutive threads read
// consecutive 16-byte pieces of one reduced position, then the next position, so a wavefront's loads are whole
// contiguous runs whatever the inner size is - 16 channels or 1024 - and every lane has work when R is large.
// Four loads are in flight per thread (eight where the grid is small and the sums long).  The partial sums of the PS position classes meet in LDS.  With few outer
// indices the slabs are made narrower (down to 8 pieces, one 128-byte line per position) until the grid has two
// workgroups per compute unit: more workgroups, and more position classes in each, so fewer loads in a row per thread.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace espdl {
namespace reduce_mid {

constexpr int kThreads = 256;
constexpr int kSlabGroups = 64; // widest slab, in pieces

template <typename T, int VEC>
struct alignas(sizeof(T) * VEC) Piece { // one load instruction: 16 bytes in the wide form
    T v[VEC];
};

// U: loads in flight per thread (4; 8 when the grid has fewer workgroups than compute units and each has far to go).
template <typename T, int VEC, int U, typename Fin>
__global__ __launch_bounds__(kThreads) void sum_mid_kernel(const T *in, long long r_count, long long inner, int slab, Fin fin)
{
    __shared__ int partial[kThreads * VEC];
    const int tid = threadIdx.x;
    const long long groups_total = inner / VEC;
    const int g_count = (int)min((long long)slab, groups_total - (long long)blockIdx.x * slab);
    const int ps = kThreads / g_count; // position classes
    const int g = tid % g_count, pl = tid / g_count;
    const long long e0 = ((long long)blockIdx.x * slab + g) * VEC; // first inner element of this thread
    const T *base = in + (long long)blockIdx.y * r_count * inner + e0;
    int sum[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++)
        sum[k] = 0;
    if (pl < ps) {
        using P = Piece<T, VEC>;
        for (long long r = pl; r < r_count; r += (long long)U * ps) {
            P p[U];
#pragma unroll
            for (int j = 0; j < U; j++) // a position past the end reads the last one again and is not added
                p[j] = *reinterpret_cast<const P *>(base + min(r + (long long)j * ps, r_count - 1) * inner);
#pragma unroll
            for (int j = 0; j < U; j++)
                if (r + (long long)j * ps < r_count) {
#pragma unroll
                    for (int k = 0; k < VEC; k++)
                        sum[k] += (int)p[j].v[k];
                }
        }
#pragma unroll
        for (int k = 0; k < VEC; k++)
            partial[(pl * g_count + g) * VEC + k] = sum[k];
    }
    __syncthreads();
    const int width = g_count * VEC; // outputs of this slab
    for (int e = tid; e < width; e += kThreads) {
        int total = 0;
        for (int c = 0; c < ps; c++)
            total += partial[c * width + e];
        fin((long long)blockIdx.y * inner + (long long)blockIdx.x * slab * VEC + e, total);
    }
}

// The int32 partial sums hold r_count elements of |x| <= 2^(bits-1); the grid's second axis holds `outer`.
template <typename T>
inline bool fits(long long outer, long long r_count, long long inner)
{
    const long long bound = sizeof(T) == 1 ? (1ll << 23) : (1ll << 15);
    return outer > 0 && outer <= 65535 && r_count > 0 && r_count < bound && inner > 0 &&
        (inner + kSlabGroups - 1) / kSlabGroups <= 0x7fffffffll;
}

// Launches the widest form the inner size and the address allow (16-byte pieces, else single elements).
template <typename T, typename Fin>
inline hipError_t launch(const T *in, long long outer, long long r_count, long long inner, Fin fin, hipStream_t stream,
                         int cu_count = 256)
{
    constexpr int kWide = 16 / (int)sizeof(T);
    const bool wide = inner % kWide == 0 && (reinterpret_cast<uintptr_t>(in) & 15) == 0;
    const long long groups = wide ? inner / kWide : inner;
    // narrower slabs while the grid is under two workgroups per compute unit; a slab keeps whole 128-byte lines
    int slab = kSlabGroups;
    const int narrowest = wide ? 8 : kSlabGroups;
    while (slab > narrowest && outer * ((groups + slab - 1) / slab) < 2ll * cu_count && groups > slab / 2)
        slab /= 2;
    const long long slabs = (groups + slab - 1) / slab;
    const dim3 grid((unsigned)slabs, (unsigned)outer);
    const bool deep = wide && outer * slabs < cu_count && r_count >= 64ll * kThreads; // few workgroups, long sums
    if (deep)
        hipLaunchKernelGGL((sum_mid_kernel<T, kWide, 8, Fin>), grid, dim3(kThreads), 0, stream, in, r_count, inner, slab, fin);
    else if (wide)
        hipLaunchKernelGGL((sum_mid_kernel<T, kWide, 4, Fin>), grid, dim3(kThreads), 0, stream, in, r_count, inner, slab, fin);
    else
        hipLaunchKernelGGL((sum_mid_kernel<T, 1, 4, Fin>), grid, dim3(kThreads), 0, stream, in, r_count, inner, slab, fin);
    return hipGetLastError();
}

// [outer][R][inner] view of a reduction over the axes flagged in `reduce_flag`, when the flagged axes longer than 1
// are neighbours; false otherwise (the caller keeps its general kernel for that).
inline bool mid_view(const int *shape, int dims, const int *reduce_flag, long long *outer, long long *r_count, long long *inner)
{
    *outer = *r_count = *inner = 1;
    int state = 0; // 0: before the reduced run, 1: inside it, 2: behind it
    for (int i = 0; i < dims; i++) {
        if (shape[i] == 1)
            continue;
        if (reduce_flag[i]) {
            if (state == 2)
                return false;
            state = 1;
            *r_count *= shape[i];
        } else if (state == 0) {
            *outer *= shape[i];
        } else {
            state = 2;
            *inner *= shape[i];
        }
    }
    return true;
}

} // namespace reduce_mid
} // namespace espdl
