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
// All cross-lane steps stay in the vector ALU: DPP inside a row of 16 lanes, v_permlane16_swap /
// v_permlane32_swap (gfx950) across rows.  ds_bpermute (what __shfl_xor compiles to) would send
// every step through the LDS crossbar.

template <typename To, typename From>
__device__ inline To bits_as(From v)
{
    static_assert(sizeof(To) == sizeof(From), "same size");
    return __builtin_bit_cast(To, v);
}

// One butterfly step: combines v with the value of a lane of the "other" M-lane group (the lane
// index differs in bit log2(M); lower bits may differ too, which is immaterial once the lower steps
// have been taken).  Steps must therefore be applied in the order M = 1, 2, 4, 8, 16, 32.
template <int M, typename T, typename Op>
__device__ inline T reduce_step(T v, Op op)
{
    static_assert(sizeof(T) == 4, "32-bit values");
    int const bits = bits_as<int>(v);
    if constexpr (M == 16)
    {
        auto const r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
        return op(bits_as<T>((int) r[0]), bits_as<T>((int) r[1]));
    }
    else if constexpr (M == 32)
    {
        auto const r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
        return op(bits_as<T>((int) r[0]), bits_as<T>((int) r[1]));
    }
    else
    {
        // quad_perm [1,0,3,2], quad_perm [2,3,0,1], row_half_mirror, row_mirror
        constexpr int ctrl = M == 1 ? 0xB1 : (M == 2 ? 0x4E : (M == 4 ? 0x141 : 0x140));
        static_assert(M == 1 || M == 2 || M == 4 || M == 8, "step");
        return op(v, bits_as<T>(__builtin_amdgcn_update_dpp(bits, bits, ctrl, 0xF, 0xF, false)));
    }
}

// The value held by the partner lane of step M (see reduce_step), for combinations that are not
// symmetric in their operands.
template <int M, typename T>
__device__ inline T lane_partner(T v)
{
    static_assert(sizeof(T) == 4, "32-bit values");
    int const bits = bits_as<int>(v);
    if constexpr (M == 16 || M == 32)
    {
        // the swap leaves (own, other) in the two results for even rows / the low half and
        // (other, own) for odd rows / the high half
        int r0, r1;
        if constexpr (M == 16)
        {
            auto const r = __builtin_amdgcn_permlane16_swap(bits, bits, false, false);
            r0 = (int) r[0];
            r1 = (int) r[1];
        }
        else
        {
            auto const r = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
            r0 = (int) r[0];
            r1 = (int) r[1];
        }
        return bits_as<T>((threadIdx.x & M) ? r0 : r1);
    }
    else
    {
        constexpr int ctrl = M == 1 ? 0xB1 : (M == 2 ? 0x4E : (M == 4 ? 0x141 : 0x140));
        static_assert(M == 1 || M == 2 || M == 4 || M == 8, "step");
        return bits_as<T>(__builtin_amdgcn_update_dpp(bits, bits, ctrl, 0xF, 0xF, false));
    }
}

// Butterfly over the SPAN lanes of a group (SPAN a power of two <= 64), starting at step FIRST.
template <int SPAN, typename T, typename Op, int FIRST = 1>
__device__ inline T group_allreduce(T v, Op op)
{
    if constexpr (FIRST < SPAN)
    {
        v = reduce_step<FIRST>(v, op);
        return group_allreduce<SPAN, T, Op, FIRST * 2>(v, op);
    }
    else
    {
        return v;
    }
}

__device__ inline float wave_sum(float v)
{
    return group_allreduce<kWaveSize>(v, [](float a, float b) { return a + b; });
}

__device__ inline int wave_sum_i32(int v)
{
    return group_allreduce<kWaveSize>(v, [](int a, int b) { return a + b; });
}

__device__ inline float wave_max(float v)
{
    return group_allreduce<kWaveSize>(v, [](float a, float b) { return fmaxf(a, b); });
}

__device__ inline int wave_min_i32(int v)
{
    return group_allreduce<kWaveSize>(v, [](int a, int b) { return min(a, b); });
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
template <int SPAN, int FIRST = 1>
__device__ inline Welford welford_butterfly(Welford w)
{
    if constexpr (FIRST < SPAN)
    {
        Welford o;
        o.n = lane_partner<FIRST>(w.n);
        o.mean = lane_partner<FIRST>(w.mean);
        o.m2 = lane_partner<FIRST>(w.m2);
        return welford_butterfly<SPAN, FIRST * 2>(welford_merge(w, o));
    }
    else
    {
        return w;
    }
}

template <int SPAN>
__device__ inline Welford group_welford(Welford w)
{
    w = welford_butterfly<SPAN>(w);
    if constexpr (SPAN == kWaveSize)
    {
        w.mean = bits_as<float>(__builtin_amdgcn_readfirstlane(bits_as<int>(w.mean)));
        w.m2 = bits_as<float>(__builtin_amdgcn_readfirstlane(bits_as<int>(w.m2)));
    }
    else
    {
        int const lead = (threadIdx.x & (kWaveSize - 1)) & ~(SPAN - 1);
        w.mean = __shfl(w.mean, lead, kWaveSize);
        w.m2 = __shfl(w.m2, lead, kWaveSize);
    }
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

// Global stores that write through the XCD's L2 (`sc1`, agent scope): the data leaves the L2 while the kernel runs
// instead of in the write-back at its end, and still allocates in the last-level cache, where the kernel of the next
// layer finds it (a non-temporal store does not).  Inline assembly, since no builtin sets this bit on a vector
// store; the s_nop covers the wait states the hardware asks for between a store of more than 8 bytes and an
// overwrite of its data registers, which the compiler cannot insert for an instruction it does not see.
template <typename V>
__device__ inline void store_through_l2(void* p, V const& v)
{
    static_assert(sizeof(V) == 16 || sizeof(V) == 8 || sizeof(V) == 4, "one dword, two or four");
    if constexpr (sizeof(V) == 16)
    {
        asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
    }
    else if constexpr (sizeof(V) == 8)
    {
        asm volatile("global_store_dwordx2 %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    }
    else
    {
        asm volatile("global_store_dword %0, %1, off sc1" ::"v"(p), "v"(v) : "memory");
    }
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

// Which unit of work and which of its `parts` a workgroup takes when several workgroups share a unit's data (the
// attention kernels: a (sequence, head) unit's K and V, read by every workgroup that takes some of its queries).
// Workgroup ids are dealt round-robin to the 8 XCDs, so ids 8 q m + 8 p + x take unit 8 m + x, part p: the parts of a
// unit sit on one XCD and find the unit's data in that L2, and units are still started in id order, which is what
// serving the longest sequences first relies on (a renumbering that gives each XCD one contiguous range of units
// starts the short sequences of the far end first: 80.7 against 60.5 us for the encoder's attention launch at two
// workgroups per unit).  Ids behind the last whole span of 8 q keep the plain order.
struct UnitPart
{
    uint32_t unit;
    int part;
};

__device__ inline UnitPart unit_of_workgroup(uint32_t bid, uint32_t nblocks, int parts)
{
    if (parts <= 1)
    {
        return {bid, 0};
    }
    uint32_t const q = (uint32_t) parts, span = 8u * q, m = bid / span, x = bid % span;
    if ((m + 1) * span <= nblocks)
    {
        return {m * 8u + x % 8u, (int) (x / 8u)};
    }
    return {bid / q, (int) (bid % q)};
}

// 16 bytes per lane from global memory straight into LDS (global_load_lds_dwordx4): lane i's bytes land at LDS byte
// address ldsAddr + 16 i, so one instruction of a wavefront fills 1 KB; ldsAddr is wave-uniform and travels in M0.
// The data never passes through vector registers, and completion is counted by vmcnt like any vector-memory load.
// Written as inline assembly on purpose: the compiler then neither counts these loads nor orders LDS reads behind
// them, and the kernel below places its own s_waitcnt where a stage must have landed.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm" // M0 is named as clobbered on purpose
__device__ __forceinline__ void load_to_lds16(void const* g, uint32_t ldsAddr)
{
    // readfirstlane: a value the compiler cannot prove wave-uniform would otherwise arrive in a vector register
    uint32_t const uniform = (uint32_t) __builtin_amdgcn_readfirstlane((int) ldsAddr);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(uniform) : "memory", "m0");
}

// The same with the address split into a wave-uniform 64-bit base (scalar registers) and a 32-bit lane offset, the
// form in which advancing the base from one load to the next is scalar arithmetic and costs the vector ALU nothing.
__device__ __forceinline__ void load_to_lds16_sbase(void const* base, uint32_t laneOffset, uint32_t ldsAddr)
{
    uint64_t const b = reinterpret_cast<uint64_t>(base);
    uint32_t const lo = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) b);
    uint32_t const hi = (uint32_t) __builtin_amdgcn_readfirstlane((int) (uint32_t) (b >> 32));
    uint64_t const ub = ((uint64_t) hi << 32) | lo;
    uint32_t const uniform = (uint32_t) __builtin_amdgcn_readfirstlane((int) ldsAddr);
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(laneOffset), "s"(ub), "s"(uniform)
                 : "memory", "m0");
}
#pragma clang diagnostic pop

// s_waitcnt vmcnt(N) alone (the other counters at their maxima): gfx9 encoding, vmcnt in bits 3:0 and 15:14
template <int N>
__device__ __forceinline__ void wait_vmcnt()
{
    static_assert(N >= 0 && N < 64, "6-bit counter");
    __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | (7 << 4) | (15 << 8));
}

} // namespace trtamd
