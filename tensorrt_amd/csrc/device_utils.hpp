// Device-side helpers shared by the gfx950 kernels: vector types, wave64 reductions, Welford
// merging and the INT8 conversion rules of the reference (plugin/common/common.cuh:482-526).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace trtamd
{

typedef _Float16 f16;
typedef f16 f16x2 __attribute__((ext_vector_type(2)));
typedef f16 f16x4 __attribute__((ext_vector_type(4)));
typedef f16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef int32_t i32x2 __attribute__((ext_vector_type(2)));
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
typedef int32_t i32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWaveSize = 64;

// ---- wave64 reductions -------------------------------------------------------------------

__device__ inline float wave_sum(float v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
    {
        v += __shfl_xor(v, m, kWaveSize);
    }
    return v;
}

__device__ inline float wave_max(float v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
    {
        v = fmaxf(v, __shfl_xor(v, m, kWaveSize));
    }
    return v;
}

__device__ inline int wave_min_i32(int v)
{
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1)
    {
        v = min(v, __shfl_xor(v, m, kWaveSize));
    }
    return v;
}

// Running (count, mean, sum of squared deviations); merged pairwise with Chan's formula so the
// variance never goes through E[x^2] - mean^2.
struct Welford
{
    float n;
    float mean;
    float m2;
};

__device__ inline Welford welford_merge(Welford a, Welford b)
{
    float const n = a.n + b.n;
    float const w = n > 0.f ? __fdividef(b.n, n) : 0.f;
    float const delta = b.mean - a.mean;
    Welford r;
    r.n = n;
    r.mean = fmaf(delta, w, a.mean);
    r.m2 = a.m2 + b.m2 + delta * delta * a.n * w;
    return r;
}

// Butterfly over `span` adjacent lanes (span a power of two <= 64); every lane of the group ends
// with the group's statistics (taken from the group's first lane so all lanes agree bit for bit).
template <int SPAN>
__device__ inline Welford group_welford(Welford w)
{
#pragma unroll
    for (int m = SPAN / 2; m >= 1; m >>= 1)
    {
        Welford o;
        o.n = __shfl_xor(w.n, m, kWaveSize);
        o.mean = __shfl_xor(w.mean, m, kWaveSize);
        o.m2 = __shfl_xor(w.m2, m, kWaveSize);
        w = welford_merge(w, o);
    }
    int const lead = (threadIdx.x & (kWaveSize - 1)) & ~(SPAN - 1);
    w.mean = __shfl(w.mean, lead, kWaveSize);
    w.m2 = __shfl(w.m2, lead, kWaveSize);
    return w;
}

// ---- INT8 conversion ---------------------------------------------------------------------

// float4_to_char4 per element: round to nearest even, saturate to [-128,127]; NaN gives 0.
__device__ inline int sat8_rne(float v)
{
    int i = __float2int_rn(v);
    return max(-128, min(127, i));
}

// quantize(): round to nearest even, clip to [-127,127].
__device__ inline int clip127_rne(float v)
{
    int i = __float2int_rn(v);
    return max(-127, min(127, i));
}

__device__ inline uint32_t pack_i8x4(int a, int b, int c, int d)
{
    return (uint32_t) (a & 0xff) | ((uint32_t) (b & 0xff) << 8) | ((uint32_t) (c & 0xff) << 16)
        | ((uint32_t) d << 24);
}

// Sign-extended byte k of a dword as float.
__device__ inline float i8_to_f32(uint32_t w, int k)
{
    return (float) (int8_t) (w >> (8 * k));
}

// XCD-aware block remap: consecutive workgroup ids are dealt round-robin to the 8 XCDs, so work
// items that share data (the query tiles of one head) are renumbered to land on one XCD's L2.
__device__ inline uint32_t xcd_remap(uint32_t bid, uint32_t nblocks)
{
    constexpr uint32_t kXcds = 8;
    uint32_t const per = nblocks / kXcds;
    uint32_t const main = per * kXcds;
    if (bid >= main)
    {
        return bid; // tail that does not fill a round keeps its id
    }
    return (bid % kXcds) * per + bid / kXcds;
}

} // namespace trtamd
