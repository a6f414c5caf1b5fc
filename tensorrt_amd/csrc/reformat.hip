// Layout and quantisation reformats either side of the interleaved encoder plugins:
//   INT8 linear [T][C]        <-> INT8 32-interleaved [C/32][T][32]      (a permutation of bytes)
//   FP16 linear [T][C]         -> INT8 32-interleaved, q = sat8(rne(x / scale))
//   INT8 32-interleaved        -> FP16 linear, x = q * scale
// All four are pure HBM streaming.  A workgroup moves a tile of 32 tokens x 256 channels through LDS
// so that both sides see long contiguous runs: 256-byte (512 for FP16) row pieces on the linear side,
// 1 KB slabs (32 tokens x 32 channels) on the interleaved side.
#include "device_utils.hpp"
#include "host_utils.hpp"
#include "trtamd_encoder_ops.h"

namespace trtamd
{
namespace
{

constexpr int kTileTokens = 32;
constexpr int kTileChannels = 256;
constexpr int kSlabs = kTileChannels / 32;
constexpr int kSlabStride = 1024 + 32; // 32 tokens x 32 bytes, padded so the 8 slabs start in different banks

__device__ inline int tile_offset(int row, int col16)
{
    return (col16 >> 1) * kSlabStride + row * 32 + (col16 & 1) * 16;
}

// 16 binary16 values -> 16 INT8, IQuantizeLayer arithmetic: clamp(round_half_even(x / scale), -128, 127)
__device__ inline i32x4 quantize16(f16x8 lo, f16x8 hi, float scale)
{
    int b[16];
#pragma unroll
    for (int e = 0; e < 8; ++e)
    {
        b[e] = sat8_rne(__fdiv_rn((float) lo[e], scale));
        b[8 + e] = sat8_rne(__fdiv_rn((float) hi[e], scale));
    }
    i32x4 r;
#pragma unroll
    for (int d = 0; d < 4; ++d)
    {
        r[d] = (int) pack_i8x4(b[4 * d], b[4 * d + 1], b[4 * d + 2], b[4 * d + 3]);
    }
    return r;
}

template <bool FROM_HALF>
__global__ __launch_bounds__(256) void to_interleaved_kernel(
    void const* __restrict__ in, int8_t* __restrict__ out, int T, int C, float scale)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile[kSlabs * kSlabStride];
    int const t0 = blockIdx.x * kTileTokens;
    int const c0 = blockIdx.y * kTileChannels;
    int const col16 = threadIdx.x & 15;
    int const c = c0 + col16 * 16;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass)
    {
        int const row = (threadIdx.x >> 4) + 16 * pass;
        int const t = t0 + row;
        i32x4 v = {0, 0, 0, 0};
        if (t < T && c < C)
        {
            if constexpr (FROM_HALF)
            {
                f16 const* src = static_cast<f16 const*>(in) + (size_t) t * C + c;
                f16x8 const lo = *reinterpret_cast<f16x8 const*>(src);
                f16x8 const hi = *(reinterpret_cast<f16x8 const*>(src) + 1);
                v = quantize16(lo, hi, scale);
            }
            else
            {
                v = *reinterpret_cast<i32x4 const*>(static_cast<int8_t const*>(in) + (size_t) t * C + c);
            }
        }
        *reinterpret_cast<i32x4*>(tile + tile_offset(row, col16)) = v;
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 2; ++pass)
    {
        int const slab = (threadIdx.x >> 6) + 4 * pass;
        int const row = (threadIdx.x & 63) >> 1;
        int const half = threadIdx.x & 1;
        int const t = t0 + row;
        int const cs = c0 + slab * 32;
        if (t < T && cs < C)
        {
            i32x4 const v = *reinterpret_cast<i32x4 const*>(tile + slab * kSlabStride + row * 32 + half * 16);
            // 32 tokens x 32 bytes per wavefront, read next by a GEMM or a plugin: through the L2 like the
            // interleaved outputs of the other kernels
            store_through_l2(out + ((size_t) (cs >> 5) * T + t) * 32 + half * 16, v);
        }
    }
}

template <bool TO_HALF>
__global__ __launch_bounds__(256) void from_interleaved_kernel(
    int8_t const* __restrict__ in, void* __restrict__ out, int T, int C, float scale)
{
    __shared__ __attribute__((aligned(16))) uint8_t tile[kSlabs * kSlabStride];
    int const t0 = blockIdx.x * kTileTokens;
    int const c0 = blockIdx.y * kTileChannels;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass)
    {
        int const slab = (threadIdx.x >> 6) + 4 * pass;
        int const row = (threadIdx.x & 63) >> 1;
        int const half = threadIdx.x & 1;
        int const t = t0 + row;
        int const cs = c0 + slab * 32;
        i32x4 v = {0, 0, 0, 0};
        if (t < T && cs < C)
        {
            v = *reinterpret_cast<i32x4 const*>(in + ((size_t) (cs >> 5) * T + t) * 32 + half * 16);
        }
        *reinterpret_cast<i32x4*>(tile + slab * kSlabStride + row * 32 + half * 16) = v;
    }
    __syncthreads();
    int const col16 = threadIdx.x & 15;
    int const c = c0 + col16 * 16;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass)
    {
        int const row = (threadIdx.x >> 4) + 16 * pass;
        int const t = t0 + row;
        if (t >= T || c >= C)
        {
            continue;
        }
        i32x4 const v = *reinterpret_cast<i32x4 const*>(tile + tile_offset(row, col16));
        if constexpr (TO_HALF)
        {
            f16x8 lo, hi;
#pragma unroll
            for (int e = 0; e < 8; ++e)
            {
                lo[e] = (f16) (i8_to_f32((uint32_t) v[e >> 2], e & 3) * scale);
                hi[e] = (f16) (i8_to_f32((uint32_t) v[2 + (e >> 2)], e & 3) * scale);
            }
            f16* dst = static_cast<f16*>(out) + (size_t) t * C + c;
            *reinterpret_cast<f16x8*>(dst) = lo;
            *(reinterpret_cast<f16x8*>(dst) + 1) = hi;
        }
        else
        {
            *reinterpret_cast<i32x4*>(static_cast<int8_t*>(out) + (size_t) t * C + c) = v;
        }
    }
}

int check_args(char const* what, int T, int C, void const* in, void const* out)
{
    if (in == nullptr || out == nullptr)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "%s: null pointer", what);
    }
    if (T < 0 || C <= 0 || C % 32 != 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "%s: T=%d C=%d (C must be a positive multiple of 32)", what, T, C);
    }
    if (!aligned16(in) || !aligned16(out))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "%s: pointers must be 16-byte aligned", what);
    }
    return TRTAMD_STATUS_SUCCESS;
}

dim3 tile_grid(int T, int C)
{
    return dim3((unsigned) ceil_div(T, kTileTokens), (unsigned) ceil_div(C, kTileChannels));
}

} // namespace
} // namespace trtamd

using namespace trtamd;

extern "C" int trtamd_int8_linear_to_interleaved(trtamd_stream_t stream, int32_t T, int32_t C, int8_t const* in, int8_t* out)
{
    if (int const rc = check_args("int8_linear_to_interleaved", T, C, in, out))
    {
        return rc;
    }
    if (T == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    hipLaunchKernelGGL(to_interleaved_kernel<false>, tile_grid(T, C), dim3(256), 0, as_stream(stream), in, out, T, C, 1.f);
    return check_launch("to_interleaved_kernel");
}

extern "C" int trtamd_int8_interleaved_to_linear(trtamd_stream_t stream, int32_t T, int32_t C, int8_t const* in, int8_t* out)
{
    if (int const rc = check_args("int8_interleaved_to_linear", T, C, in, out))
    {
        return rc;
    }
    if (T == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    hipLaunchKernelGGL(
        from_interleaved_kernel<false>, tile_grid(T, C), dim3(256), 0, as_stream(stream), in, out, T, C, 1.f);
    return check_launch("from_interleaved_kernel");
}

extern "C" int trtamd_quantize_fp16_to_interleaved(
    trtamd_stream_t stream, int32_t T, int32_t C, trtamd_half_t const* in, float scale, int8_t* out)
{
    if (int const rc = check_args("quantize_fp16_to_interleaved", T, C, in, out))
    {
        return rc;
    }
    if (!(scale > 0.f))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "quantize_fp16_to_interleaved: scale must be positive");
    }
    if (T == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    hipLaunchKernelGGL(to_interleaved_kernel<true>, tile_grid(T, C), dim3(256), 0, as_stream(stream), in, out, T, C, scale);
    return check_launch("to_interleaved_kernel");
}

extern "C" int trtamd_dequantize_interleaved_to_fp16(
    trtamd_stream_t stream, int32_t T, int32_t C, int8_t const* in, float scale, trtamd_half_t* out)
{
    if (int const rc = check_args("dequantize_interleaved_to_fp16", T, C, in, out))
    {
        return rc;
    }
    if (T == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    hipLaunchKernelGGL(
        from_interleaved_kernel<true>, tile_grid(T, C), dim3(256), 0, as_stream(stream), in, out, T, C, scale);
    return check_launch("from_interleaved_kernel");
}
