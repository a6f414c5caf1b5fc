// On-box instruction-rate microbenchmarks for gfx950 (libtrtamd_microbench.so, loaded by bench.py only): what the
// matrix and vector pipes of this GPU sustain for the instructions the attention and linear kernels are made of.
// Every kernel runs register-only loops of independent chains on every SIMD of the chip; the host function times
// a few launches with events and returns milliseconds per launch.  Not part of the plugin library.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int i32x4 __attribute__((ext_vector_type(4)));
typedef int i32x16 __attribute__((ext_vector_type(16)));

namespace
{

constexpr int kThreads = 256; // 4 wavefronts: one per SIMD of a CU

// A and B operands of one lane: zeros, or bytes from a buffer of random data (so the values cannot be folded)
__device__ inline i32x4 operand(int32_t const* src, int which)
{
    i32x4 v;
    for (int i = 0; i < 4; ++i)
    {
        v[i] = src[(which * 64 + (threadIdx.x & 63)) * 4 + i];
    }
    return v;
}

// CHAINS independent accumulators per wavefront, each updated once per iteration
template <int CHAINS>
__global__ __launch_bounds__(kThreads) void mfma_16x16x64_i8_kernel(int32_t const* src, int32_t* out, int iters)
{
    i32x4 const a = operand(src, 0), b = operand(src, 1);
    i32x4 acc[CHAINS];
    for (int c = 0; c < CHAINS; ++c)
    {
        acc[c] = i32x4{c, 0, 0, 0};
    }
    for (int it = 0; it < iters; ++it)
    {
        // inline assembly pins each accumulator to its own vector registers: left to the compiler, four or more
        // chains in a loop are shuffled through the accumulation registers with a dozen copies per iteration
#pragma unroll
        for (int c = 0; c < CHAINS; ++c)
        {
            asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a), "v"(b));
        }
    }
    int s = 0;
    for (int c = 0; c < CHAINS; ++c)
    {
        s += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
    }
    out[blockIdx.x * kThreads + threadIdx.x] = s;
}

template <int CHAINS>
__global__ __launch_bounds__(kThreads) void mfma_32x32x32_i8_kernel(int32_t const* src, int32_t* out, int iters)
{
    i32x4 const a = operand(src, 0), b = operand(src, 1);
    i32x16 acc[CHAINS];
    for (int c = 0; c < CHAINS; ++c)
    {
        for (int i = 0; i < 16; ++i)
        {
            acc[c][i] = c + i;
        }
    }
    for (int it = 0; it < iters; ++it)
    {
#pragma unroll
        for (int c = 0; c < CHAINS; ++c)
        {
            asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc[c]) : "v"(a), "v"(b));
        }
    }
    int s = 0;
    for (int c = 0; c < CHAINS; ++c)
    {
        for (int i = 0; i < 16; ++i)
        {
            s += acc[c][i];
        }
    }
    out[blockIdx.x * kThreads + threadIdx.x] = s;
}

// Eight independent chains of one vector-ALU instruction
enum ValuOp
{
    OP_FMA = 0,
    OP_EXP = 1,
    OP_ADD = 2,
    OP_PERM = 3,
    OP_MAX3 = 4,
    OP_CVT_PK_U8 = 5,
    OP_SOFTMAX_MIX = 6, // fma, exp, add, fma per element: the inner sequence of the attention kernel
    OP_MAX3_F32 = 7,
    OP_MAX_F32 = 8,
    OP_MUL = 9,
    OP_LSHL_OR = 10,
    OP_CVT_F32_I32 = 11,
    OP_CVT_F32_BYTE = 12, // v_cvt_f32_ubyte0
    OP_DOT4 = 13,         // v_dot4_i32_i8
    OP_RCP = 14,
    OP_MED3_F32 = 15,
    OP_ADD_U32 = 16,
};

template <int OP>
__global__ __launch_bounds__(kThreads) void valu_kernel(int32_t const* src, int32_t* out, int iters, int64_t* clocks)
{
    uint64_t const c0 = __builtin_readcyclecounter();
    uint64_t const w0 = wall_clock64();
    float const c = __int_as_float(src[0] & 0x007fffff | 0x3f800000) * 0.5f + 0.25f; // in [0.75, 1.25)
    float a[8];
    float sum = 0.f;
    for (int i = 0; i < 8; ++i)
    {
        a[i] = (float) (threadIdx.x & 63) * 0.001f + (float) i;
    }
    for (int it = 0; it < iters; ++it)
    {
#pragma unroll
        for (int i = 0; i < 8; ++i)
        {
            if (OP == OP_FMA)
            {
                a[i] = __builtin_fmaf(a[i], c, 0.5f);
            }
            else if (OP == OP_EXP)
            {
                a[i] = __builtin_amdgcn_exp2f(a[i]);
            }
            else if (OP == OP_ADD)
            {
                a[i] = a[i] + c;
            }
            else if (OP == OP_PERM)
            {
                a[i] = __uint_as_float(__builtin_amdgcn_perm(__float_as_uint(a[i]), __float_as_uint(a[(i + 1) & 7]),
                    0x05040100u));
            }
            else if (OP == OP_MAX3)
            {
                a[i] = __int_as_float(max(max(__float_as_int(a[i]), __float_as_int(a[(i + 1) & 7])),
                    __float_as_int(a[(i + 2) & 7])));
            }
            else if (OP == OP_CVT_PK_U8)
            {
                a[i] = __uint_as_float(__builtin_amdgcn_cvt_pk_u8_f32(a[i], 1, __float_as_uint(a[(i + 1) & 7])));
            }
            else if (OP == OP_MAX3_F32)
            {
                asm volatile("v_max3_f32 %0, %0, %1, %2" : "+v"(a[i]) : "v"(a[(i + 1) & 7]), "v"(a[(i + 2) & 7]));
            }
            else if (OP == OP_MAX_F32)
            {
                asm volatile("v_max_f32 %0, %0, %1" : "+v"(a[i]) : "v"(a[(i + 1) & 7]));
            }
            else if (OP == OP_MUL)
            {
                asm volatile("v_mul_f32 %0, %0, %1" : "+v"(a[i]) : "v"(c));
            }
            else if (OP == OP_LSHL_OR)
            {
                asm volatile("v_lshl_or_b32 %0, %0, 8, %1" : "+v"(a[i]) : "v"(a[(i + 1) & 7]));
            }
            else if (OP == OP_CVT_F32_I32)
            {
                asm volatile("v_cvt_f32_i32 %0, %0" : "+v"(a[i]));
            }
            else if (OP == OP_CVT_F32_BYTE)
            {
                asm volatile("v_cvt_f32_ubyte0 %0, %0" : "+v"(a[i]));
            }
            else if (OP == OP_DOT4)
            {
                asm volatile("v_dot4_i32_i8 %0, %1, %2, %0" : "+v"(a[i]) : "v"(a[(i + 1) & 7]), "v"(c));
            }
            else if (OP == OP_RCP)
            {
                asm volatile("v_rcp_f32 %0, %0" : "+v"(a[i]));
            }
            else if (OP == OP_MED3_F32)
            {
                asm volatile("v_med3_f32 %0, %0, %1, %2" : "+v"(a[i]) : "v"(c), "v"(a[(i + 1) & 7]));
            }
            else if (OP == OP_ADD_U32)
            {
                asm volatile("v_add_u32 %0, %0, %1" : "+v"(a[i]) : "v"(a[(i + 1) & 7]));
            }
            else
            {
                float const e = __builtin_amdgcn_exp2f(__builtin_fmaf(a[i], c, -1.0f));
                sum += e;
                a[i] = __builtin_fmaf(e, c, 12582912.f);
            }
        }
    }
    float s = sum;
    for (int i = 0; i < 8; ++i)
    {
        s += a[i];
    }
    out[blockIdx.x * kThreads + threadIdx.x] = __float_as_int(s);
    if (clocks && threadIdx.x == 0)
    {
        // shader-clock cycles and 100 MHz wall-clock ticks this workgroup's first wavefront spent in the loop
        clocks[2 * blockIdx.x] = (int64_t) (__builtin_readcyclecounter() - c0);
        clocks[2 * blockIdx.x + 1] = (int64_t) (wall_clock64() - w0);
    }
}

// One MFMA and NV independent vector-ALU instructions per step, in one wavefront's instruction stream: does the
// matrix pipe run beside the vector ALU (time = max of the two) or in its place (time = sum)?  KIND selects the vector
// instructions: 0 = v_fma_f32, 1 = v_exp_f32, 2 = the softmax group fma, exp, add, fma (NV counts instructions, so
// NV / 4 groups).  Sixteen independent chains, so the vector instructions never wait for each other.  WITH_MFMA = false
// is the control: the same stream without the MFMA.
template <int NV, int KIND, bool WITH_MFMA>
__global__ __launch_bounds__(kThreads) void mfma_valu_mix_kernel(int32_t const* src, int32_t* out, int iters)
{
    i32x4 const a = operand(src, 0), b = operand(src, 1);
    float const c = __int_as_float(src[0] & 0x007fffff | 0x3f800000) * 0.5f + 0.25f;
    i32x4 acc[4];
    float f[16];
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
    for (int i = 0; i < 4; ++i)
    {
        acc[i] = i32x4{i, 0, 0, 0};
    }
    for (int i = 0; i < 16; ++i)
    {
        f[i] = (float) (threadIdx.x & 63) * 0.001f + (float) i;
    }
    for (int it = 0; it < iters; ++it)
    {
#pragma unroll
        for (int m = 0; m < 4; ++m)
        {
            if (WITH_MFMA)
            {
                asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[m]) : "v"(a), "v"(b));
            }
            if (KIND == 2)
            {
#pragma unroll
                for (int v = 0; v < NV / 4; ++v)
                {
                    int const k = (m * (NV / 4) + v) & 15;
                    float e;
                    asm volatile("v_fma_f32 %0, %1, %2, -1.0" : "=v"(e) : "v"(f[k]), "v"(c));
                    asm volatile("v_exp_f32 %0, %0" : "+v"(e));
                    asm volatile("v_add_f32 %0, %0, %1" : "+v"(sum[k & 3]) : "v"(e));
                    asm volatile("v_fma_f32 %0, %1, %2, %2" : "=v"(f[k]) : "v"(e), "v"(c));
                }
            }
            else
            {
#pragma unroll
                for (int v = 0; v < NV; ++v)
                {
                    int const k = (m * NV + v) & 15;
                    if (KIND == 0)
                    {
                        asm volatile("v_fma_f32 %0, %0, %1, %0" : "+v"(f[k]) : "v"(c));
                    }
                    else
                    {
                        asm volatile("v_exp_f32 %0, %0" : "+v"(f[k]));
                    }
                }
            }
        }
    }
    int s = 0;
    for (int i = 0; i < 4; ++i)
    {
        s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    }
    float t = sum[0] + sum[1] + sum[2] + sum[3];
    for (int i = 0; i < 16; ++i)
    {
        t += f[i];
    }
    out[blockIdx.x * kThreads + threadIdx.x] = s + __float_as_int(t);
}

// The same question across wavefronts: a workgroup of eight wavefronts, two per SIMD (wavefronts w and w + 4 share
// one), of which the first four issue only MFMAs (4 per iteration, independent accumulators) and the last four only
// v_fma_f32 (NV per iteration on sixteen independent chains, fully unrolled, so that a vector wavefront alone issues
// at the rate of the ALU and is not waiting for its own results).  `roles` selects who works (1: MFMA wavefronts,
// 2: vector wavefronts, 3: both); if the two kinds of wavefront run beside each other, roles 3 takes the longer of
// the two times, not their sum.
template <int NV, int PAD>
__global__ __launch_bounds__(512) void mfma_valu_split_kernel(int32_t const* src, int32_t* out, int iters, int roles)
{
    int const wave = threadIdx.x >> 6;
    int result = 0;
    if (wave < 4)
    {
        if (roles & 1)
        {
            i32x4 const a = operand(src, 0), b = operand(src, 1);
            i32x4 acc[4];
            for (int i = 0; i < 4; ++i)
            {
                acc[i] = i32x4{i, 0, 0, 0};
            }
            for (int it = 0; it < iters; ++it)
            {
#pragma unroll
                for (int m = 0; m < 4; ++m)
                {
                    asm volatile("v_mfma_i32_16x16x64_i8 %0, %1, %2, %0" : "+v"(acc[m]) : "v"(a), "v"(b));
                    // PAD scalar no-ops (`s_nop 7`, ~13 ns each as measured; they do not use the vector issue port)
                    // behind every MFMA: with two or more, this wavefront's next MFMA arrives when the matrix pipe is
                    // free again
#pragma unroll
                    for (int p = 0; p < PAD; ++p)
                    {
                        asm volatile("s_nop 7");
                    }
                }
            }
            for (int i = 0; i < 4; ++i)
            {
                result += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
            }
        }
    }
    else if (roles & 2)
    {
        float const c = __int_as_float(src[0] & 0x007fffff | 0x3f800000) * 0.5f + 0.25f;
        float f[16];
        for (int i = 0; i < 16; ++i)
        {
            f[i] = (float) (threadIdx.x & 63) * 0.001f + (float) i;
        }
        for (int it = 0; it < iters; ++it)
        {
#pragma unroll
            for (int u = 0; u < NV; ++u)
            {
                asm volatile("v_fma_f32 %0, %0, %1, %0" : "+v"(f[u & 15]) : "v"(c));
            }
        }
        float t = 0.f;
        for (int i = 0; i < 16; ++i)
        {
            t += f[i];
        }
        result = __float_as_int(t);
    }
    out[blockIdx.x * 512 + threadIdx.x] = result;
}

// A kernel that does nothing: what a back-to-back launch of a given grid costs on this box.
__global__ void empty_kernel(int32_t* out)
{
    if (out == nullptr && threadIdx.x == 12345)
    {
        __builtin_trap(); // never: keeps the parameter alive
    }
}

template <typename Launch>
float time_launches(Launch launch, int reps)
{
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)
    {
        return -1.f;
    }
    launch();
    launch();
    (void) hipDeviceSynchronize();
    (void) hipEventRecord(e0, nullptr);
    for (int i = 0; i < reps; ++i)
    {
        launch();
    }
    (void) hipEventRecord(e1, nullptr);
    (void) hipEventSynchronize(e1);
    float ms = -1.f;
    (void) hipEventElapsedTime(&ms, e0, e1);
    (void) hipEventDestroy(e0);
    (void) hipEventDestroy(e1);
    return hipGetLastError() == hipSuccess ? ms / (float) reps : -1.f;
}

} // namespace

#define MB_API extern "C" __attribute__((visibility("default")))

// Milliseconds per launch of `blocks` workgroups of 4 wavefronts, each wavefront issuing iters * chains MFMAs.
// shape: 0 = v_mfma_i32_16x16x64_i8, 1 = v_mfma_i32_32x32x32_i8 (both 32768 integer operations per instruction
// and wavefront); chains: 1, 2, 4 or 8 independent accumulators; operands: 128 x 4 int32 of device memory.
MB_API float trtamd_microbench_mfma_i8(int shape, int chains, int blocks, int iters, int32_t const* operands, int32_t* out)
{
#define MB_CASE(S, C)                                                                                                  \
    if (shape == S && chains == C)                                                                                     \
    {                                                                                                                  \
        return time_launches(                                                                                          \
            [&] {                                                                                                      \
                if (S == 0)                                                                                            \
                    hipLaunchKernelGGL((mfma_16x16x64_i8_kernel<C>), dim3(blocks), dim3(kThreads), 0, nullptr,         \
                        operands, out, iters);                                                                         \
                else                                                                                                   \
                    hipLaunchKernelGGL((mfma_32x32x32_i8_kernel<C>), dim3(blocks), dim3(kThreads), 0, nullptr,         \
                        operands, out, iters);                                                                         \
            },                                                                                                         \
            5);                                                                                                        \
    }
    MB_CASE(0, 1) MB_CASE(0, 2) MB_CASE(0, 4) MB_CASE(0, 8) MB_CASE(1, 1) MB_CASE(1, 2) MB_CASE(1, 4) MB_CASE(1, 8)
#undef MB_CASE
    return -1.f;
}

// Milliseconds per launch of an empty kernel of `blocks` workgroups of `threads` threads, back to back.
MB_API float trtamd_microbench_empty(int blocks, int threads, int32_t* out)
{
    return time_launches([&] { hipLaunchKernelGGL(empty_kernel, dim3(blocks), dim3(threads), 0, nullptr, out); }, 200);
}

// Milliseconds per launch; every wavefront issues iters * 4 steps of (one v_mfma_i32_16x16x64_i8, nv vector
// instructions of `kind`: 0 = v_fma_f32, 1 = v_exp_f32, 2 = the group fma, exp, add, fma (nv a multiple of 4)).
// with_mfma = 0 leaves the MFMA out (the control for the same vector instructions alone).
MB_API float trtamd_microbench_mfma_valu(int nv, int kind, int with_mfma, int blocks, int iters, int32_t const* operands,
    int32_t* out)
{
#define MB_NV(V, K)                                                                                                    \
    if (nv == V && kind == K)                                                                                          \
    {                                                                                                                  \
        return time_launches(                                                                                          \
            [&] {                                                                                                      \
                if (with_mfma)                                                                                         \
                    hipLaunchKernelGGL((mfma_valu_mix_kernel<V, K, true>), dim3(blocks), dim3(kThreads), 0, nullptr,   \
                        operands, out, iters);                                                                         \
                else                                                                                                   \
                    hipLaunchKernelGGL((mfma_valu_mix_kernel<V, K, false>), dim3(blocks), dim3(kThreads), 0, nullptr,  \
                        operands, out, iters);                                                                         \
            },                                                                                                         \
            5);                                                                                                        \
    }
#define MB_NVS(K) MB_NV(0, K) MB_NV(4, K) MB_NV(8, K) MB_NV(12, K) MB_NV(16, K) MB_NV(24, K) MB_NV(32, K)
    MB_NVS(0) MB_NVS(1) MB_NVS(2) MB_NV(1, 0) MB_NV(2, 0) MB_NV(3, 0) MB_NV(6, 0) MB_NV(2, 1) MB_NV(6, 1)
#undef MB_NVS
#undef MB_NV
    return -1.f;
}

// Milliseconds per launch; every wavefront issues iters * 8 instructions of kind `op` (ValuOp; OP_SOFTMAX_MIX
// issues iters * 8 groups of four).
// clocks (optional): 2 x blocks int64, per workgroup the shader-clock cycles and the 100 MHz ticks of its loop.
MB_API float trtamd_microbench_valu(int op, int blocks, int iters, int32_t const* operands, int32_t* out, int64_t* clocks)
{
#define MB_OP(O)                                                                                                       \
    if (op == O)                                                                                                       \
    {                                                                                                                  \
        return time_launches(                                                                                          \
            [&] { hipLaunchKernelGGL((valu_kernel<O>), dim3(blocks), dim3(kThreads), 0, nullptr, operands, out, iters, clocks); }, \
            5);                                                                                                        \
    }
    MB_OP(OP_FMA) MB_OP(OP_EXP) MB_OP(OP_ADD) MB_OP(OP_PERM) MB_OP(OP_MAX3) MB_OP(OP_CVT_PK_U8) MB_OP(OP_SOFTMAX_MIX)
    MB_OP(OP_MAX3_F32) MB_OP(OP_MAX_F32) MB_OP(OP_MUL) MB_OP(OP_LSHL_OR) MB_OP(OP_CVT_F32_I32) MB_OP(OP_CVT_F32_BYTE)
    MB_OP(OP_DOT4) MB_OP(OP_RCP) MB_OP(OP_MED3_F32) MB_OP(OP_ADD_U32)
#undef MB_OP
    return -1.f;
}

// Milliseconds per launch of `blocks` workgroups of eight wavefronts: four that issue 4 * iters MFMAs each and four
// that issue nv * iters v_fma_f32 each (nv 32 or 64); roles 1, 2 or 3 as described at the kernel; pad = number of
// `s_nop 7` behind every MFMA (0 .. 4).
MB_API float trtamd_microbench_mfma_valu_split(int blocks, int iters, int nv, int pad, int roles, int32_t const* operands,
    int32_t* out)
{
#define MB_SPLIT(V, P)                                                                                                 \
    if (nv == V && pad == P)                                                                                           \
    {                                                                                                                  \
        return time_launches(                                                                                          \
            [&] {                                                                                                      \
                hipLaunchKernelGGL((mfma_valu_split_kernel<V, P>), dim3(blocks), dim3(512), 0, nullptr, operands, out, \
                    iters, roles);                                                                                     \
            },                                                                                                         \
            20);                                                                                                       \
    }
    MB_SPLIT(32, 0) MB_SPLIT(32, 1) MB_SPLIT(32, 2) MB_SPLIT(32, 3) MB_SPLIT(32, 4)
    MB_SPLIT(64, 0) MB_SPLIT(64, 1) MB_SPLIT(64, 2) MB_SPLIT(64, 3) MB_SPLIT(64, 4)
#undef MB_SPLIT
    return -1.f;
}
