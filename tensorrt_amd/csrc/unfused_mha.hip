// Score-materialising attention for the cases the fused kernels do not cover (FP32, any head
// size, any sequence length), its row softmax, and the head-size padding copy.
//
// Replaces UnfusedMHARunner::run (plugin/bertQKVToContextPlugin/mhaRunner.cu:527-601: two
// cuBLAS strided-batched GEMMs around a softmax kernel), computeScaledSoftmax /
// computeMaskedScaledSoftmax (same file :196-344, plugin/common/common.cuh:313-421) and
// zeroPadding2d (plugin/bertQKVToContextPlugin/zeroPadding2d.cu) of the reference.
#include "device_utils.hpp"
#include "host_utils.hpp"

#include <algorithm>
#include <mutex>

// Score matrices of trtamd_unfused_mha_static: device memory that belongs to the library instead of the caller.
// Every GPU the library runs on holds its own copy of this array, at its own address, until the process ends.  In
// host code the name below is only a stand-in for the symbol (it is not a device address): host code goes through
// the per-device pointer that static_scratch() obtains with hipGetSymbolAddress.
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace trtamd
{
namespace
{

constexpr int kMaxDevices = 64;

// Device address of `scratch` on the current device, looked up once per device (with that device current).
int static_scratch(void** out)
{
    static std::mutex mtx;
    static void* ptrs[kMaxDevices] = {};
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= kMaxDevices)
    {
        (void) hipGetLastError();
        return set_error(TRTAMD_STATUS_FAILURE, "unfused MHA (static scratch): no current device (%s)",
            hipGetErrorString(e));
    }
    std::lock_guard<std::mutex> lock(mtx);
    if (ptrs[dev] == nullptr)
    {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
        {
            (void) hipGetLastError();
            return set_error(TRTAMD_STATUS_FAILURE, "unfused MHA (static scratch): hipGetSymbolAddress failed on device %d: %s",
                dev, hipGetErrorString(e));
        }
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return TRTAMD_STATUS_SUCCESS;
}

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWaveSize;

// ------------------------------------------------------------------------------------------
// Row softmax: out[i] = exp((x[i]-max)*w) / sum for i < lastValid, exactly 0 beyond; one wave
// per row of ld scores, the row is read into registers once when it fits (ld <= 64*NR).
// ------------------------------------------------------------------------------------------
template <typename T, int NR>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(int const ld, int64_t const rows,
    int64_t const rowsPerBatch, float const w, int32_t const* __restrict__ maskIdx, T const* __restrict__ in,
    T* __restrict__ out)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    int64_t const row = (int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= rows)
    {
        return;
    }
    int lastValid = ld;
    if (maskIdx)
    {
        lastValid = min(ld, maskIdx[row / rowsPerBatch]);
    }
    T const* x = in + row * ld;
    T* y = out + row * ld;
    float const wl2 = w * 1.4426950408889634f;
    if constexpr (NR > 0)
    {
        float v[NR];
        float mx = -3.0e38f;
#pragma unroll
        for (int j = 0; j < NR; ++j)
        {
            int const i = lane + kWaveSize * j;
            v[j] = i < lastValid ? (float) x[i] : -3.0e38f;
            mx = fmaxf(mx, v[j]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NR; ++j)
        {
            int const i = lane + kWaveSize * j;
            v[j] = i < lastValid ? __builtin_amdgcn_exp2f((v[j] - mx) * wl2) : 0.f;
            sum += v[j];
        }
        sum = wave_sum(sum);
        float const rz = 1.f / sum;
#pragma unroll
        for (int j = 0; j < NR; ++j)
        {
            int const i = lane + kWaveSize * j;
            if (i < ld)
            {
                y[i] = (T) (i < lastValid ? v[j] * rz : 0.f);
            }
        }
    }
    else
    {
        float mx = -3.0e38f;
        for (int i = lane; i < lastValid; i += kWaveSize)
        {
            mx = fmaxf(mx, (float) x[i]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
        for (int i = lane; i < lastValid; i += kWaveSize)
        {
            sum += __builtin_amdgcn_exp2f(((float) x[i] - mx) * wl2);
        }
        sum = wave_sum(sum);
        float const rz = 1.f / sum;
        for (int i = lane; i < ld; i += kWaveSize)
        {
            y[i] = (T) (i < lastValid ? __builtin_amdgcn_exp2f(((float) x[i] - mx) * wl2) * rz : 0.f);
        }
    }
}

template <typename T>
int scaled_softmax(hipStream_t stream, int32_t ld, int32_t B, int32_t N, float w, int32_t const* maskIdx, T const* in,
    T* out)
{
    if (ld < 0 || B < 0 || N < 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "scaledSoftmax: negative size");
    }
    int64_t const rows = (int64_t) B * N * ld;
    if (rows == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!in || !out)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "scaledSoftmax: null pointer");
    }
    dim3 const grid((unsigned) ceil_div<int64_t>(rows, kWavesPerBlock));
    int64_t const rpb = (int64_t) N * ld;
    if (ld <= 128)
    {
        hipLaunchKernelGGL((softmax_rows_kernel<T, 2>), grid, dim3(kBlock), 0, stream, ld, rows, rpb, w, maskIdx, in, out);
    }
    else if (ld <= 512)
    {
        hipLaunchKernelGGL((softmax_rows_kernel<T, 8>), grid, dim3(kBlock), 0, stream, ld, rows, rpb, w, maskIdx, in, out);
    }
    else
    {
        hipLaunchKernelGGL((softmax_rows_kernel<T, 0>), grid, dim3(kBlock), 0, stream, ld, rows, rpb, w, maskIdx, in, out);
    }
    return check_launch("softmax_rows_kernel");
}

// ------------------------------------------------------------------------------------------
// Strided batched GEMM on the vector ALU, 64x64 output tile per workgroup, binary32
// accumulation: C[m,n] = sum_k A(m,k) * B(k,n), operands addressed by element strides so the
// same kernel serves Q K^T (B = K read along its rows) and P V.
// Batch index z = b*heads + h; operand base = b*batchStride + h*headStride.
// ------------------------------------------------------------------------------------------
struct GemmOperand
{
    int64_t batchStride, headStride, rowStride, colStride;
};

template <typename T>
__global__ __launch_bounds__(kBlock) void batched_gemm_kernel(int const M, int const N, int const K, int const heads,
    T const* __restrict__ A, GemmOperand const oa, T const* __restrict__ B, GemmOperand const ob, T* __restrict__ Cm,
    GemmOperand const oc)
{
    constexpr int TM = 64, TN = 64, TK = 16;
    __shared__ float sA[TK][TM + 1];
    __shared__ float sB[TK][TN + 1];
    int const z = blockIdx.z;
    int const b = z / heads, h = z % heads;
    T const* a = A + b * oa.batchStride + h * oa.headStride;
    T const* bb = B + b * ob.batchStride + h * ob.headStride;
    T* c = Cm + b * oc.batchStride + h * oc.headStride;
    int const m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
    int const tx = threadIdx.x % 16, ty = threadIdx.x / 16;
    float acc[4][4] = {};
    for (int k0 = 0; k0 < K; k0 += TK)
    {
        for (int i = threadIdx.x; i < TM * TK; i += kBlock)
        {
            // A tile: consecutive threads walk k (contiguous for Q and P)
            int const kk = i % TK, mm = i / TK;
            int const m = m0 + mm, k = k0 + kk;
            sA[kk][mm] = (m < M && k < K) ? (float) a[m * oa.rowStride + k * oa.colStride] : 0.f;
        }
        for (int i = threadIdx.x; i < TN * TK; i += kBlock)
        {
            // B(k,n): choose the walk so that the contiguous dimension varies fastest
            int kk, nn;
            if (ob.colStride == 1)
            {
                nn = i % TN;
                kk = i / TN;
            }
            else
            {
                kk = i % TK;
                nn = i / TK;
            }
            int const n = n0 + nn, k = k0 + kk;
            sB[kk][nn] = (n < N && k < K) ? (float) bb[k * ob.rowStride + n * ob.colStride] : 0.f;
        }
        __syncthreads();
#pragma unroll
        for (int kk = 0; kk < TK; ++kk)
        {
            float av[4], bv[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                av[i] = sA[kk][ty * 4 + i];
                bv[i] = sB[kk][tx * 4 + i];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    acc[i][j] = fmaf(av[i], bv[j], acc[i][j]);
                }
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
    {
        int const m = m0 + ty * 4 + i;
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            int const n = n0 + tx * 4 + j;
            if (m < M && n < N)
            {
                c[m * oc.rowStride + n * oc.colStride] = (T) acc[i][j];
            }
        }
    }
}

template <typename T>
int unfused_mha(hipStream_t stream, int32_t S, int32_t B, int32_t N, int32_t d, T const* qkv, int32_t const* maskIdx,
    T* output, void* workspace)
{
    // geometry of MHARunner::setup (mhaRunner.h:62-83)
    int64_t const ldQKV = (int64_t) 3 * B * N * d;
    int64_t const strideQKV = (int64_t) 3 * d;
    int64_t const ldOut = (int64_t) B * N * d;
    int64_t const omat = (int64_t) S * S;
    int64_t const numMats = (int64_t) B * N;
    T* qk = static_cast<T*>(workspace);
    T* pp = qk + omat * numMats;
    T const* q = qkv;
    T const* k = qkv + d;
    T const* v = qkv + 2 * d;
    // batch z = b*N + h: qkv offset (b*N + h)*3d, score matrix z*S*S, output (b*N + h)*d
    GemmOperand const oq{N * strideQKV, strideQKV, ldQKV, 1};
    GemmOperand const okT{N * strideQKV, strideQKV, 1, ldQKV};  // B(k=dim, n=key) = K[key][dim]
    GemmOperand const os{N * omat, omat, S, 1};
    GemmOperand const ov{N * strideQKV, strideQKV, ldQKV, 1};   // B(k=key, n=dim) = V[key][dim]
    GemmOperand const oo{(int64_t) N * d, d, ldOut, 1};
    dim3 const g1(ceil_div(S, 64), ceil_div(S, 64), (unsigned) numMats);
    hipLaunchKernelGGL((batched_gemm_kernel<T>), g1, dim3(kBlock), 0, stream, S, S, d, N, q, oq, k, okT, qk, os);
    int st = check_launch("batched_gemm_kernel(QK^T)");
    if (st != 0)
    {
        return st;
    }
    float const w = 1.f / sqrtf((float) d);
    st = scaled_softmax<T>(stream, S, B, N, w, maskIdx, qk, pp);
    if (st != 0)
    {
        return st;
    }
    dim3 const g2(ceil_div(d, 64), ceil_div(S, 64), (unsigned) numMats);
    hipLaunchKernelGGL((batched_gemm_kernel<T>), g2, dim3(kBlock), 0, stream, S, d, S, N, pp, os, v, ov, output, oo);
    return check_launch("batched_gemm_kernel(PV)");
}

// ------------------------------------------------------------------------------------------
// zeroPadding2d: rows of spitch bytes -> rows of dpitch bytes, in units of U bytes.
// ------------------------------------------------------------------------------------------
template <typename U>
__global__ __launch_bounds__(kBlock) void zero_padding_kernel(
    U const* __restrict__ src, int const spitch, U* __restrict__ dst, int const dpitch, int64_t const total)
{
    for (int64_t uid = (int64_t) blockIdx.x * kBlock + threadIdx.x; uid < total; uid += (int64_t) gridDim.x * kBlock)
    {
        int64_t const ty = uid / dpitch;
        int const tx = (int) (uid % dpitch);
        U val{};
        if (tx < spitch)
        {
            val = src[ty * spitch + tx];
        }
        dst[uid] = val;
    }
}

struct alignas(16) Bytes16
{
    uint32_t w[4];
};

} // namespace
} // namespace trtamd

using namespace trtamd;

extern "C" int trtamd_scaled_softmax_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t N,
    float rsqrtHeadSize, int32_t const* maskIdx, float const* input, float* output)
{
    return scaled_softmax<float>(as_stream(stream), ld, B, N, rsqrtHeadSize, maskIdx, input, output);
}

extern "C" int trtamd_scaled_softmax_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t N,
    float rsqrtHeadSize, int32_t const* maskIdx, trtamd_half_t const* input, trtamd_half_t* output)
{
    return scaled_softmax<f16>(as_stream(stream), ld, B, N, rsqrtHeadSize, maskIdx,
        reinterpret_cast<f16 const*>(input), reinterpret_cast<f16*>(output));
}

extern "C" size_t trtamd_unfused_mha_workspace_size(int32_t type, int32_t S, int32_t B, int32_t N)
{
    // UnfusedMHARunner::getWorkspaceSize: 2 * wordSize * S*S * B*N  (mhaRunner.cu:522-525)
    size_t const word = type == 0 ? 4 : (type == 1 ? 2 : 1);
    return 2UL * word * (size_t) S * (size_t) S * (size_t) B * (size_t) N;
}

extern "C" int trtamd_unfused_mha(trtamd_stream_t stream, int32_t type, int32_t S, int32_t B, int32_t N, int32_t d,
    void const* qkv, int32_t const* maskIdx, void* output, void* workspace)
{
    if (type != 0 && type != 1)
    {
        // UnfusedMHARunner::isValid is false for INT8 (mhaRunner.cu:603-606)
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: data type %d (only FP32=0 and FP16=1)", type);
    }
    if (S <= 0 || B <= 0 || N <= 0 || d <= 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA: bad dimensions S=%d B=%d N=%d d=%d", S, B, N, d);
    }
    if ((int64_t) B * N > 65535)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: B*N = %lld exceeds 65535", (long long) B * N);
    }
    if (!qkv || !output || !workspace)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA: null pointer (workspace is required)");
    }
    if (type == 0)
    {
        return unfused_mha<float>(as_stream(stream), S, B, N, d, static_cast<float const*>(qkv), maskIdx,
            static_cast<float*>(output), workspace);
    }
    return unfused_mha<f16>(as_stream(stream), S, B, N, d, static_cast<f16 const*>(qkv), maskIdx,
        static_cast<f16*>(output), workspace);
}

extern "C" size_t trtamd_unfused_mha_static_capacity(void)
{
    return kStaticScratchBytes;
}

extern "C" int trtamd_unfused_mha_static(trtamd_stream_t stream, int32_t type, int32_t S, int32_t B, int32_t N, int32_t d,
    void const* qkv, int32_t const* maskIdx, void* output)
{
    if (type != 0 && type != 1)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: data type %d (only FP32=0 and FP16=1)", type);
    }
    if (S <= 0 || B <= 0 || N <= 0 || d <= 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA: bad dimensions S=%d B=%d N=%d d=%d", S, B, N, d);
    }
    // 2 * wordSize * S*S * B*N in 128-bit arithmetic free of overflow: each factor is below 2^31
    double const need = 2.0 * (type == 0 ? 4.0 : 2.0) * (double) S * (double) S * (double) B * (double) N;
    if (need > (double) kStaticScratchBytes)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED,
            "unfused MHA (static scratch): S=%d B=%d N=%d needs %.0f bytes of score matrices, the library's array holds "
            "%zu; use trtamd_unfused_mha with a workspace",
            S, B, N, need, kStaticScratchBytes);
    }
    void* ws = nullptr;
    int const st = static_scratch(&ws);
    if (st != TRTAMD_STATUS_SUCCESS)
    {
        return st;
    }
    // every score the second and third kernel read was written by the kernel before it in this call: nothing in
    // the array has to start at zero, and what the previous call left there is never read
    return trtamd_unfused_mha(stream, type, S, B, N, d, qkv, maskIdx, output, ws);
}

extern "C" int trtamd_zero_padding_2d(
    void const* src, int32_t spitch, void* dst, int32_t dpitch, int32_t height, trtamd_stream_t stream)
{
    if (spitch < 0 || dpitch < 0 || height < 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "zeroPadding2d: negative size");
    }
    if (dpitch == 0 || height == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!src || !dst)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "zeroPadding2d: null pointer");
    }
    // widest unit that divides both pitches and both addresses (zeroPadding2d.cu:100-126)
    uintptr_t const bits = reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst) | (uintptr_t) spitch
        | (uintptr_t) dpitch;
    int shift = 0;
    while (shift < 4 && ((bits >> shift) & 1u) == 0)
    {
        ++shift;
    }
    int const sp = spitch >> shift, dp = dpitch >> shift;
    int64_t const total = (int64_t) dp * height;
    unsigned const grid = (unsigned) std::min<int64_t>(ceil_div<int64_t>(total, kBlock), 256 * 8);
    hipStream_t const s = as_stream(stream);
    switch (shift)
    {
    case 4:
        hipLaunchKernelGGL((zero_padding_kernel<Bytes16>), dim3(grid), dim3(kBlock), 0, s,
            static_cast<Bytes16 const*>(src), sp, static_cast<Bytes16*>(dst), dp, total);
        break;
    case 3:
        hipLaunchKernelGGL((zero_padding_kernel<uint64_t>), dim3(grid), dim3(kBlock), 0, s,
            static_cast<uint64_t const*>(src), sp, static_cast<uint64_t*>(dst), dp, total);
        break;
    case 2:
        hipLaunchKernelGGL((zero_padding_kernel<uint32_t>), dim3(grid), dim3(kBlock), 0, s,
            static_cast<uint32_t const*>(src), sp, static_cast<uint32_t*>(dst), dp, total);
        break;
    case 1:
        hipLaunchKernelGGL((zero_padding_kernel<uint16_t>), dim3(grid), dim3(kBlock), 0, s,
            static_cast<uint16_t const*>(src), sp, static_cast<uint16_t*>(dst), dp, total);
        break;
    default:
        hipLaunchKernelGGL((zero_padding_kernel<uint8_t>), dim3(grid), dim3(kBlock), 0, s,
            static_cast<uint8_t const*>(src), sp, static_cast<uint8_t*>(dst), dp, total);
        break;
    }
    return check_launch("zero_padding_kernel");
}
