// Device-side integer helpers shared by the gfx950 kernels.
//
// The arithmetic restates tool::shift_and_round / tool::truncate of the reference
// (esp-dl/dl/tool/src/dl_tool.cpp:95-146; esp-dl/dl/tool/include/dl_tool.hpp:225-254) in forms that
// need no 64-bit intermediate on the int8 path.
#pragma once

#include <hip/hip_runtime.h>
#include <mutex>
#include <vector>
#include <stdint.h>

namespace espdl {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
// The same values at any byte address: gfx950 global loads and stores need no alignment, one instruction each.
typedef v4i v4i_unaligned __attribute__((aligned(1)));
typedef v2i v2i_unaligned __attribute__((aligned(1)));
typedef int int_unaligned __attribute__((aligned(1)));

__device__ __forceinline__ int clamp_s8(int v)
{
    return min(max(v, -128), 127);
}

// shift_and_round<int32_t> followed by optional ReLU and truncate(int8_t&, .).
//   shift in 1..31 : floor((v + 2^(s-1)) / 2^s) == (v >> s) + bit(s-1) of v   (no overflow)
//   shift >= 32    : the 64-bit sum v + 2^(s-1) is non-negative and below 2^s  -> 0
//   shift <= 0     : saturate(int64(v) << -s); since the result is clamped to int8 afterwards,
//                    clamping first and shifting by min(-s, 8) gives the same value.
__device__ __forceinline__ int requant_s8(int v, int shift, bool relu, bool half_even)
{
    int q;
    if (shift > 0) {
        if (shift > 31) {
            q = 0;
        } else if (half_even) {
            const unsigned mask = (1u << shift) - 1u;
            const int rem = (int)((unsigned)v & mask);
            const int half = (int)(1u << (shift - 1));
            q = v >> shift;
            q += (rem > half || (rem == half && (q & 1))) ? 1 : 0;
        } else {
            q = (v >> shift) + ((v >> (shift - 1)) & 1);
        }
    } else {
        q = clamp_s8(v) << min(-shift, 8);
    }
    if (relu)
        q = max(q, 0);
    return clamp_s8(q);
}

// shift_and_round<int64_t> followed by optional ReLU and truncate(int16_t&, .).
__device__ __forceinline__ int requant_s16(long long v, int shift, bool relu, bool half_even)
{
    long long q;
    if (shift > 0) {
        if (half_even) {
            const unsigned long long mask = (1ull << shift) - 1ull;
            const long long rem = (long long)((unsigned long long)v & mask);
            const long long half = (long long)(1ull << (shift - 1));
            q = v >> shift;
            q += (rem > half || (rem == half && (q & 1))) ? 1 : 0;
        } else {
            q = (long long)((unsigned long long)v + (1ull << (shift - 1))) >> shift;
        }
    } else {
        q = (long long)((unsigned long long)v << -shift);
    }
    if (relu && q < 0)
        q = 0;
    q = q < -32768 ? -32768 : (q > 32767 ? 32767 : q);
    return (int)q;
}

// tool::round(float) of the portable build: (int)floorf(value + 0.5) where 0.5 is a double literal,
// so the sum is formed in double and narrowed to float by floorf's parameter
// (esp-dl/dl/tool/src/dl_tool.cpp:72-75).
__device__ __forceinline__ int round_half_up_f32(float v)
{
    return (int)floorf((float)((double)v + 0.5));
}

// DL_SCALE / DL_RESCALE (esp-dl/dl/dl_define.hpp:75-81)
__host__ __device__ __forceinline__ float dl_scale(int e)
{
    return e > 0 ? (float)(1 << e) : 1.0f / (float)(1 << -e);
}
__host__ __device__ __forceinline__ float dl_rescale(int e)
{
    return e > 0 ? 1.0f / (float)(1 << e) : (float)(1 << -e);
}

typedef short v2s __attribute__((ext_vector_type(2)));

// Short requantization of four accumulators that already hold bias + 2^(s-1): after the shifts the
// result q sits in bits 8.. of t; v_cvt_pk_i16_i32 saturates t to int16, which saturates q to int8
// in the high byte; ReLU is one packed max on the int16 pairs; v_perm_b32 gathers the four high bytes.
// MODE 0: every shift is at least 8, round half up.  MODE 1: some shift is below 8, so the value is
// first shifted left by max(0, 8-s).  MODES 4, 5 and 6 are described at pack_fast4.
// Saturating packed multiply of two int16 by two int16 (v_pk_mad_i16 with the clamp bit: the products are
// formed exactly and saturated to int16).
// Maximum of two int16 pairs held in dwords (v_pk_max_i16).  The operands arrive by value on purpose: a
// __builtin_bit_cast applied directly to an element of an ext_vector (x[d]) reads element 0 whatever d is.
__device__ __forceinline__ int pk_max_i16(int a, int b)
{
    return __builtin_bit_cast(int, __builtin_elementwise_max(__builtin_bit_cast(v2s, a), __builtin_bit_cast(v2s, b)));
}

__device__ __forceinline__ v2s pk_mul_sat_i16(v2s a, int m)
{
    int d;
    asm("v_pk_mad_i16 %0, %1, %2, 0 clamp" : "=v"(d) : "v"(__builtin_bit_cast(int, a)), "v"(m));
    return __builtin_bit_cast(v2s, d);
}

// Round half to even on an accumulator that holds v + 2^(s-1) - 1, one less than the round-half-up start value:
// adding bit s of that accumulator gives the value whose arithmetic shift by s is the half-even result (the rule
// of esp-dl/dl/tool/src/dl_tool.cpp:95-119).  With f the low s bits of v and q the bits above: if f <= 2^(s-1)
// the sum f + 2^(s-1) - 1 does not carry, bit s of the accumulator is the parity of q, and adding it carries into
// bit s exactly when f = 2^(s-1) and q is odd; if f > 2^(s-1) the sum has carried already and one more cannot
// carry again.  Two instructions per value (v_bfe_u32, v_add).
__device__ __forceinline__ int half_even_add(int acc, int s)
{
    return acc + (int)__builtin_amdgcn_ubfe((unsigned)acc, (unsigned)s, 1u);
}

// MODE 4 is MODE 1 with the left shifts moved behind the saturating convert, two values per instruction:
// lsh[0] and lsh[1] hold the multipliers 2^max(0, 8-s) of the channel pairs (0, 1) and (2, 3) as packed
// int16.  A channel has either a right shift (s > 8) or a multiplier (s < 8), never both.  Saturating
// acc to int16 first and the product to int16 again gives the same high byte as saturating acc * 2^l once:
// where the first saturation acts (|acc| >= 2^15, l >= 0) the second one does too.
// MODE 5: half-even for accumulators that hold bias + 2^(s-1) - 1 (half_even_add), with the left shift.
// MODE 6: the same where every shift is at least 8.
// CEIL: the int8 result is also clamped from above (a Clip between two stages): ceil_pk holds the upper bound
// twice as int16 in the same fixed-point form, (max << 8) | 0xff, one packed minimum per pair.  floor_pk is
// then (max(lower bound, 0 for ReLU) << 8) & 0xffff twice.
template <int MODE, bool CEIL = false>
__device__ __forceinline__ int pack_fast4(const v4i &acc, const v4i &lsh, const v4i &rsh, int floor_pk,
                                          int ceil_pk = 0x7fff7fff)
{
    if constexpr (MODE == 4) {
        const v2s floor2 = __builtin_bit_cast(v2s, floor_pk);
        v2s p01 = __builtin_amdgcn_cvt_pk_i16(acc[0] >> rsh[0], acc[1] >> rsh[1]);
        v2s p23 = __builtin_amdgcn_cvt_pk_i16(acc[2] >> rsh[2], acc[3] >> rsh[3]);
        p01 = __builtin_elementwise_max(pk_mul_sat_i16(p01, lsh[0]), floor2);
        p23 = __builtin_elementwise_max(pk_mul_sat_i16(p23, lsh[1]), floor2);
        if constexpr (CEIL) {
            p01 = __builtin_elementwise_min(p01, __builtin_bit_cast(v2s, ceil_pk));
            p23 = __builtin_elementwise_min(p23, __builtin_bit_cast(v2s, ceil_pk));
        }
        return (int)__builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, p23), (unsigned)__builtin_bit_cast(int, p01),
                                          0x07050301u);
    }
    int t[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        int a = acc[r];
        if (MODE == 5)
            a = half_even_add(a, rsh[r] + 8 - lsh[r]);
        if (MODE == 6)
            a = half_even_add(a, rsh[r] + 8);
        const int v = (MODE != 0 && MODE != 6) ? (int)((unsigned)a << lsh[r]) : a;
        t[r] = v >> rsh[r];
    }
    // floor_pk holds the lower clamp twice as int16: 0 for ReLU, -32768 (no effect) otherwise
    const v2s floor2 = __builtin_bit_cast(v2s, floor_pk);
    v2s p01 = __builtin_elementwise_max(__builtin_amdgcn_cvt_pk_i16(t[0], t[1]), floor2);
    v2s p23 = __builtin_elementwise_max(__builtin_amdgcn_cvt_pk_i16(t[2], t[3]), floor2);
    if constexpr (CEIL) {
        p01 = __builtin_elementwise_min(p01, __builtin_bit_cast(v2s, ceil_pk));
        p23 = __builtin_elementwise_min(p23, __builtin_bit_cast(v2s, ceil_pk));
    }
    return (int)__builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, p23), (unsigned)__builtin_bit_cast(int, p01),
                                      0x07050301u);
}

// pack_fast4 followed by the saturating int8 Add of `res` (four packed int8, esp-dl/dl/base/dl_base_add.cpp:34-44).
// The int16 pairs hold q_sat * 256 + fraction after the saturating convert (and the ReLU max), so adding
// res * 256 with int16 saturation leaves saturate_int8(q_sat + res) in the high byte: the fraction (0..255)
// cannot carry across a saturation bound.  Two byte permutes spread `res` into the high bytes.
template <int MODE>
__device__ __forceinline__ int pack_fast4_add(const v4i &acc, const v4i &lsh, const v4i &rsh, int floor_pk, int res)
{
    int t[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        int a = acc[r];
        if (MODE == 5)
            a = half_even_add(a, rsh[r] + 8 - lsh[r]);
        if (MODE == 6)
            a = half_even_add(a, rsh[r] + 8);
        const int v = (MODE != 0 && MODE != 6) ? (int)((unsigned)a << lsh[r]) : a;
        t[r] = v >> rsh[r];
    }
    const v2s floor2 = __builtin_bit_cast(v2s, floor_pk);
    const v2s r01 = __builtin_bit_cast(v2s, (int)__builtin_amdgcn_perm(0u, (unsigned)res, 0x010c000cu));
    const v2s r23 = __builtin_bit_cast(v2s, (int)__builtin_amdgcn_perm(0u, (unsigned)res, 0x030c020cu));
    v2s p01 = __builtin_elementwise_max(__builtin_amdgcn_cvt_pk_i16(t[0], t[1]), floor2);
    v2s p23 = __builtin_elementwise_max(__builtin_amdgcn_cvt_pk_i16(t[2], t[3]), floor2);
    p01 = __builtin_elementwise_add_sat(p01, r01);
    p23 = __builtin_elementwise_add_sat(p23, r23);
    return (int)__builtin_amdgcn_perm((unsigned)__builtin_bit_cast(int, p23), (unsigned)__builtin_bit_cast(int, p01),
                                      0x07050301u);
}

// Four packed int8 requantized by 2^d, d in [-7, 7]: what RequantizeLinear / TensorBase::assign does between two
// int8 exponents (esp-dl/dl/tensor/src/dl_tensor_base.cpp:362-371: round(x * 2^d) half up, saturated).  The
// bytes are spread into the high bytes of int16 pairs (x * 256).  d > 0: a saturating multiply by 2^d.  d < 0:
// x * 128 (one shift, so that the rounding constant cannot overflow), + 2^(6-d), arithmetic shift by -d - 1.
// The result's high bytes are the answer.
struct Requant4 {
    int mul, pre, rnd, sh;
};
__device__ __forceinline__ Requant4 make_requant4(int d)
{
    Requant4 q;
    q.mul = (1 << max(d, 0)) * 0x00010001;
    q.pre = d < 0 ? 1 : 0;
    q.rnd = d < 0 ? (1 << (6 - d)) * 0x00010001 : 0;
    q.sh = d < 0 ? -d - 1 : 0;
    return q;
}
__device__ __forceinline__ int requant4_s8(int word, const Requant4 &q)
{
    int out[2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int hi = (int)__builtin_amdgcn_perm(0u, (unsigned)word, h == 0 ? 0x010c000cu : 0x030c020cu);
        v2s v = pk_mul_sat_i16(__builtin_bit_cast(v2s, hi), q.mul);
        v = v >> (short)q.pre;
        v = v + __builtin_bit_cast(v2s, q.rnd);
        v = v >> (short)q.sh;
        out[h] = __builtin_bit_cast(int, v);
    }
    return (int)__builtin_amdgcn_perm((unsigned)out[1], (unsigned)out[0], 0x07050301u);
}

// int8 x 4 saturating add of two packed dwords
__device__ __forceinline__ int sat_add4_s8(int x, int y)
{
    int r = 0;
#pragma unroll
    for (int b = 0; b < 4; b++) {
        int s = (int)(int8_t)(x >> (8 * b)) + (int)(int8_t)(y >> (8 * b));
        s = s < -128 ? -128 : (s > 127 ? 127 : s);
        r |= (s & 0xff) << (8 * b);
    }
    return r;
}

// Division of a 31-bit unsigned number by a launch-invariant divisor: q = (mulhi(n, m) + n) >> s
// with m = floor(2^32 * (2^s - d) / d) + 1, s = ceil(log2 d)  (Granlund-Montgomery; exact for
// every n < 2^31).  The host fills the struct, the device spends three instructions.
struct FastDiv {
    unsigned int m, s, d;
};

inline FastDiv make_fastdiv(unsigned int d)
{
    FastDiv f;
    f.d = d;
    unsigned int s = 0;
    while ((1ull << s) < d)
        s++;
    f.s = s;
    f.m = (unsigned int)(((1ull << 32) * ((1ull << s) - d)) / d + 1);
    return f;
}

__device__ __forceinline__ unsigned int fastdiv(unsigned int n, const FastDiv &f)
{
    return (__umulhi(n, f.m) + n) >> f.s;
}

__device__ __forceinline__ int pack4_s8(int a, int b, int c, int d)
{
    return (a & 0xff) | ((b & 0xff) << 8) | ((c & 0xff) << 16) | ((d & 0xff) << 24);
}

// Tile sequence of one workgroup of a persistent grid.  The hardware deals workgroups to the eight
// XCDs round-robin by their linear id, and every XCD has its own L2.  Striding tiles by gridDim.x
// would therefore spread neighbouring tiles (which share input rows through the filter window) over
// all eight L2s and each of them would fetch those rows from memory again.  Instead XCD x owns the
// contiguous eighth [x * per, (x + 1) * per) of the tiles and its workgroups stride through that
// range, so rows shared between neighbouring tiles are found in the L2 that already holds them.
// Needs gridDim.x % 8 == 0 (gridDim.y slices then keep blockIdx.x % 8 as the XCD); otherwise the
// plain strided sequence is used.
struct TileSeq {
    int first, step, end;
};

__device__ __forceinline__ TileSeq xcd_tile_sequence(int n_tiles)
{
    TileSeq s;
    if ((gridDim.x & 7u) == 0) {
        const int per = (n_tiles + 7) >> 3;
        const int xcd = blockIdx.x & 7;
        s.first = xcd * per + (int)(blockIdx.x >> 3);
        s.step = (int)(gridDim.x >> 3);
        s.end = min(n_tiles, (xcd + 1) * per);
    } else {
        s.first = blockIdx.x;
        s.step = gridDim.x;
        s.end = n_tiles;
    }
    return s;
}

// Workgroups of `kernel` (block size `threads`, `lds` bytes of dynamic LDS) that fit on one CU at
// the same time, as the runtime computes it from the kernel's register and LDS use; clamped to
// [1, 8].  Host only.  Looked up once per (kernel, lds) and remembered.
template <typename Kernel>
inline int resident_workgroups_per_cu(Kernel kernel, int threads, size_t lds)
{
    struct Entry {
        const void *fn;
        size_t lds;
        int n;
    };
    static std::mutex mu;
    static std::vector<Entry> seen;
    const void *fn = reinterpret_cast<const void *>(kernel);
    {
        std::lock_guard<std::mutex> lock(mu);
        for (const Entry &e : seen)
            if (e.fn == fn && e.lds == lds)
                return e.n;
    }
    int n = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, kernel, threads, lds) != hipSuccess || n < 1) {
        (void)hipGetLastError();
        n = 1;
    }
    if (n > 8)
        n = 8;
    std::lock_guard<std::mutex> lock(mu);
    seen.push_back(Entry{fn, lds, n});
    return n;
}

} // namespace espdl
