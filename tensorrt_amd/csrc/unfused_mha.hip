// Attention for the cases the fused kernels do not cover (FP32, any head size, any sequence
// length) — in one launch with a query's scores in registers where they fit, through score
// matrices in a workspace otherwise —, the row softmax, and the head-size padding copy.
//
// Replaces UnfusedMHARunner::run (plugin/bertQKVToContextPlugin/mhaRunner.cu:527-601: two
// cuBLAS strided-batched GEMMs around a softmax kernel), computeScaledSoftmax /
// computeMaskedScaledSoftmax (same file :196-344, plugin/common/common.cuh:313-421) and
// zeroPadding2d (plugin/bertQKVToContextPlugin/zeroPadding2d.cu) of the reference.
#include "device_utils.hpp"
#include "host_utils.hpp"

#include <algorithm>
#include <cmath>
#include <cstdlib>
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

// The same for rows that are whole 16-byte pieces at 16-byte aligned addresses: LPR lanes share a row (64 / LPR rows
// per wavefront), each taking NV pieces of 16 bytes, piece j of a lane LPR pieces behind piece j - 1, so that every
// access of the wavefront covers whole 64-byte runs and a short row does not leave most of the lanes idle.
template <typename T, int LPR, int NV>
__global__ __launch_bounds__(kBlock) void softmax_rows_vec_kernel(int const ld, int64_t const rows,
    int64_t const rowsPerBatch, float const w, int32_t const* __restrict__ maskIdx, T const* __restrict__ in,
    T* __restrict__ out)
{
    constexpr int V = 16 / sizeof(T);              // elements per piece
    constexpr int kRowsPerWave = kWaveSize / LPR;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const sub = lane % LPR;
    int64_t const row
        = ((int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)) * kRowsPerWave + lane / LPR;
    bool const live = row < rows;
    int lastValid = 0;
    if (live)
    {
        lastValid = maskIdx ? min(ld, maskIdx[row / rowsPerBatch]) : ld;
    }
    T const* x = in + (live ? row : 0) * ld;
    float const wl2 = w * 1.4426950408889634f;
    float v[NV][V];
    float mx = -3.0e38f;
#pragma unroll
    for (int j = 0; j < NV; ++j)
    {
        int const i0 = (sub + LPR * j) * V;
        T raw[V];
        if (live && i0 < ld)
        {
            *reinterpret_cast<u32x4*>(raw) = *reinterpret_cast<u32x4 const*>(x + i0);
        }
#pragma unroll
        for (int e = 0; e < V; ++e)
        {
            v[j][e] = (live && i0 + e < lastValid) ? (float) raw[e] : -3.0e38f;
            mx = fmaxf(mx, v[j][e]);
        }
    }
#pragma unroll
    for (int d = 1; d < LPR; d *= 2)
    {
        mx = fmaxf(mx, __shfl_xor(mx, d));
    }
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j)
    {
        int const i0 = (sub + LPR * j) * V;
#pragma unroll
        for (int e = 0; e < V; ++e)
        {
            v[j][e] = i0 + e < lastValid ? __builtin_amdgcn_exp2f((v[j][e] - mx) * wl2) : 0.f;
            sum += v[j][e];
        }
    }
#pragma unroll
    for (int d = 1; d < LPR; d *= 2)
    {
        sum += __shfl_xor(sum, d);
    }
    float const rz = 1.f / sum;
    if (live)
    {
        T* y = out + row * ld;
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            int const i0 = (sub + LPR * j) * V;
            if (i0 < ld)
            {
                T res[V];
#pragma unroll
                for (int e = 0; e < V; ++e)
                {
                    res[e] = (T) (i0 + e < lastValid ? v[j][e] * rz : 0.f);
                }
                *reinterpret_cast<u32x4*>(y + i0) = *reinterpret_cast<u32x4 const*>(res);
            }
        }
    }
}

template <typename T, int LPR, int NV>
void launch_softmax_vec(hipStream_t stream, int32_t ld, int64_t rows, int64_t rpb, float w, int32_t const* maskIdx,
    T const* in, T* out)
{
    int64_t const rowsPerBlock = (int64_t) kWavesPerBlock * (kWaveSize / LPR);
    dim3 const grid((unsigned) ceil_div<int64_t>(rows, rowsPerBlock));
    hipLaunchKernelGGL((softmax_rows_vec_kernel<T, LPR, NV>), grid, dim3(kBlock), 0, stream, ld, rows, rpb, w, maskIdx, in,
        out);
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
    int64_t const rpb = (int64_t) N * ld;
    // rows of whole, aligned 16-byte pieces, up to 256 of them (2048 binary16 or 1024 binary32 scores, held in
    // registers between the read and the write): the vectorised kernel
    constexpr int V = 16 / (int) sizeof(T);
    if (ld % V == 0 && ld / V <= 256 && (reinterpret_cast<uintptr_t>(in) & 15) == 0
        && (reinterpret_cast<uintptr_t>(out) & 15) == 0)
    {
        int const pieces = ld / V;
        if (pieces <= 16)
        {
            launch_softmax_vec<T, 16, 1>(stream, ld, rows, rpb, w, maskIdx, in, out);
        }
        else if (pieces <= 32)
        {
            launch_softmax_vec<T, 32, 1>(stream, ld, rows, rpb, w, maskIdx, in, out);
        }
        else if (pieces <= 64)
        {
            launch_softmax_vec<T, 64, 1>(stream, ld, rows, rpb, w, maskIdx, in, out);
        }
        else if (pieces <= 128)
        {
            launch_softmax_vec<T, 64, 2>(stream, ld, rows, rpb, w, maskIdx, in, out);
        }
        else
        {
            launch_softmax_vec<T, 64, 4>(stream, ld, rows, rpb, w, maskIdx, in, out);
        }
        return check_launch("softmax_rows_vec_kernel");
    }
    dim3 const grid((unsigned) ceil_div<int64_t>(rows, kWavesPerBlock));
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
// Strided batched GEMM on the matrix cores, binary32 accumulation: C[m,n] = sum_k A(m,k) * B(k,n), operands
// addressed by element strides so the same kernel serves Q K^T (B = K read along its rows) and P V.
// A workgroup of four wavefronts owns a 64 x 64 tile of C, a wavefront a 32 x 32 quarter of it in one accumulator
// tile of v_mfma_f32_32x32x16_f16 (binary16 operands) or v_mfma_f32_32x32x2_f32 (binary32 operands: full IEEE
// multiplies).  k advances in chunks of 64 (binary16) or 32 (binary32) through LDS, both operands stored [row][k]
// there, so that a fragment is one 16-byte read (binary16) or one 4-byte read per instruction (binary32); rows and k beyond the matrix are
// zero in LDS, so any M, N, K is served.  Global reads take 16 bytes per lane along whichever dimension is
// contiguous when addresses and strides allow, single elements otherwise.
// Batch index z = b*heads + h; operand base = b*batchStride + h*headStride.
// ------------------------------------------------------------------------------------------
struct GemmOperand
{
    int64_t batchStride, headStride, rowStride, colStride;
};

constexpr int kGemmTile = 64; // rows and columns of C per workgroup

template <typename T>
struct GemmLds
{
    // row pitch in elements: 16-byte aligned rows for the binary16 fragment reads, an odd number of dwords for the
    // binary32 ones (consecutive rows then fall in consecutive banks)
    // k per LDS stage: the whole head size of 64 in one step for binary16 (one trip to memory and one barrier pair for
    // Q K^T), 32 for binary32, whose stage of 64 would take the LDS of half the resident workgroups
    static constexpr int kK = sizeof(T) == 2 ? 64 : 32;
    static constexpr int kPitch = sizeof(T) == 2 ? kK + 8 : kK + 1;
};

// One operand's stage (64 rows x one chunk of k) into LDS as [row][k].  rowStride / kStride are the element strides of the operand's
// row index (m or n) and of k in global memory; rows < rowsLeft and k < kLeft exist.
template <typename T>
__device__ inline void stage_operand(T const* __restrict__ g, int64_t const rowStride, int64_t const kStride,
    int const rowsLeft, int const kLeft, bool const vec, T* __restrict__ lds)
{
    constexpr int P = GemmLds<T>::kPitch;
    constexpr int kGemmK = GemmLds<T>::kK;
    constexpr int V = 16 / sizeof(T); // elements per 16-byte access
    if (vec && kStride == 1)
    {
        // 16 bytes along k: (64 rows) x (32 / V chunks)
        for (int c = threadIdx.x; c < kGemmTile * (kGemmK / V); c += kBlock)
        {
            int const row = c / (kGemmK / V), k0 = (c % (kGemmK / V)) * V;
            T tmp[V];
            if (row < rowsLeft && k0 + V <= kLeft)
            {
                *reinterpret_cast<u32x4*>(tmp) = *reinterpret_cast<u32x4 const*>(g + row * rowStride + k0);
            }
            else
            {
#pragma unroll
                for (int i = 0; i < V; ++i)
                {
                    tmp[i] = (row < rowsLeft && k0 + i < kLeft) ? g[row * rowStride + k0 + i] : (T) 0.f;
                }
            }
#pragma unroll
            for (int i = 0; i < V; ++i)
            {
                lds[row * P + k0 + i] = tmp[i];
            }
        }
    }
    else if (vec && rowStride == 1)
    {
        // 16 bytes along the row index (V rows of one k): transposed on the way into LDS
        for (int c = threadIdx.x; c < kGemmK * (kGemmTile / V); c += kBlock)
        {
            int const k = c / (kGemmTile / V), r0 = (c % (kGemmTile / V)) * V;
            T tmp[V];
            if (k < kLeft && r0 + V <= rowsLeft)
            {
                *reinterpret_cast<u32x4*>(tmp) = *reinterpret_cast<u32x4 const*>(g + k * kStride + r0);
            }
            else
            {
#pragma unroll
                for (int i = 0; i < V; ++i)
                {
                    tmp[i] = (k < kLeft && r0 + i < rowsLeft) ? g[k * kStride + r0 + i] : (T) 0.f;
                }
            }
#pragma unroll
            for (int i = 0; i < V; ++i)
            {
                lds[(r0 + i) * P + k] = tmp[i];
            }
        }
    }
    else
    {
        bool const kFastest = kStride <= rowStride;
        for (int c = threadIdx.x; c < kGemmTile * kGemmK; c += kBlock)
        {
            int const row = kFastest ? c / kGemmK : c % kGemmTile;
            int const k = kFastest ? c % kGemmK : c / kGemmTile;
            lds[row * P + k] = (row < rowsLeft && k < kLeft) ? g[row * rowStride + k * kStride] : (T) 0.f;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void batched_gemm_kernel(int const M, int const N, int const K, int const heads,
    T const* __restrict__ A, GemmOperand const oa, T const* __restrict__ B, GemmOperand const ob, T* __restrict__ Cm,
    GemmOperand const oc, int const vecA, int const vecB)
{
    constexpr int P = GemmLds<T>::kPitch;
    constexpr int kGemmK = GemmLds<T>::kK;
    __shared__ __attribute__((aligned(16))) T sA[kGemmTile * P];
    __shared__ __attribute__((aligned(16))) T sB[kGemmTile * P];
    int const z = blockIdx.z;
    int const b = z / heads, h = z % heads;
    T const* a = A + b * oa.batchStride + h * oa.headStride;
    T const* bb = B + b * ob.batchStride + h * ob.headStride;
    T* c = Cm + b * oc.batchStride + h * oc.headStride;
    int const m0 = blockIdx.y * kGemmTile, n0 = blockIdx.x * kGemmTile;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const wm = (wave >> 1) * 32, wn = (wave & 1) * 32; // this wavefront's quarter of the tile
    int const r = lane & 31, kh = lane >> 5;               // fragment row / column and k half
    f32x16 acc;
#pragma unroll
    for (int i = 0; i < 16; ++i)
    {
        acc[i] = 0.f;
    }
    for (int k0 = 0; k0 < K; k0 += kGemmK)
    {
        // A(m,k): row index m, B(k,n): row index n (stored [n][k])
        stage_operand<T>(a + m0 * oa.rowStride + k0 * oa.colStride, oa.rowStride, oa.colStride, M - m0, K - k0,
            vecA != 0, sA);
        stage_operand<T>(bb + k0 * ob.rowStride + n0 * ob.colStride, ob.colStride, ob.rowStride, N - n0, K - k0,
            vecB != 0, sB);
        __syncthreads();
        if constexpr (sizeof(T) == 2)
        {
#pragma unroll
            for (int ks = 0; ks < kGemmK; ks += 16)
            {
                f16x8 const fa = *reinterpret_cast<f16x8 const*>(&sA[(wm + r) * P + ks + kh * 8]);
                f16x8 const fb = *reinterpret_cast<f16x8 const*>(&sB[(wn + r) * P + ks + kh * 8]);
                acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa, fb, acc, 0, 0, 0);
            }
        }
        else
        {
#pragma unroll
            for (int ks = 0; ks < kGemmK; ks += 2)
            {
                float const fa = sA[(wm + r) * P + ks + kh];
                float const fb = sB[(wn + r) * P + ks + kh];
                acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fa, fb, acc, 0, 0, 0);
            }
        }
        __syncthreads();
    }
    // accumulator i of lane (r, kh): row 8 (i / 4) + 4 kh + i % 4, column r of the wavefront's quarter
#pragma unroll
    for (int i = 0; i < 16; ++i)
    {
        int const m = m0 + wm + 8 * (i >> 2) + 4 * kh + (i & 3);
        int const n = n0 + wn + r;
        if (m < M && n < N)
        {
            c[m * oc.rowStride + n * oc.colStride] = (T) acc[i];
        }
    }
}

// 16-byte accesses along the contiguous dimension are possible when the base, both strides that get multiplied and
// the batch / head strides keep every address 16-byte aligned.
template <typename T>
int can_vectorise(T const* base, GemmOperand const& o)
{
    constexpr int64_t V = 16 / sizeof(T);
    bool const contiguous = o.colStride == 1 || o.rowStride == 1;
    int64_t const other = o.colStride == 1 ? o.rowStride : o.colStride;
    return contiguous && (reinterpret_cast<uintptr_t>(base) & 15u) == 0 && other % V == 0 && o.batchStride % V == 0
        && o.headStride % V == 0;
}

// ------------------------------------------------------------------------------------------
// The same attention in one launch, for sequences whose scores fit in registers (S <= 512, head size <= 128): no
// score matrix goes to memory.  A workgroup of four wavefronts owns 64 queries of one (batch, head), a wavefront 16
// of them with ALL their keys, so the row maximum and sum need no exchange between wavefronts.  The matrix products
// are computed transposed, S^T = K Q^T and O^T = V^T P^T, with the 16 x 16 MFMA tiles: a lane then holds, for its
// one query, four consecutive keys per tile — the softmax reductions run inside the lane (plus two lane exchanges),
// and the probabilities are, as they stand in the accumulator registers, the B operand of the second product.  The
// order in which a lane's eight (binary16) or four (binary32) k positions of a step map to dimensions / keys is
// free as long as both operands use the same one; it is chosen so that every fragment is one or two whole LDS reads:
//   binary16  Q K^T step t: lane group g holds dimensions 32t + 8g .. +7;  P V step s of a chunk: keys
//             32s + 4g .. +3 and 32s + 16 + 4g .. +3 (accumulator tiles 2s and 2s + 1 of the chunk);
//   binary32  step (u, i): dimension 16u + 4g + i;  P V step (tile j, i): key 16j + 4g + i.
// K and V pass through one LDS stage of 64 keys, K as [key][dim]; binary32 V transposed to [dim][key] on the way in
// (lane = key, so that the transposing writes of a wavefront fall on consecutive addresses), binary16 V as
// [key][dim] with the transposition left to the fragment reads (ds_read_tr16_b64).  Numerics as the three-kernel
// path and the reference's chain of GEMM, softmax, GEMM: scores and probabilities are rounded to T where that chain
// stores them, accumulation is binary32.  Chunks of 64 keys that lie wholly beyond a batch's valid length are
// skipped (their probabilities are exactly 0).
// ------------------------------------------------------------------------------------------
constexpr int kRegQueries = 64; // queries per workgroup
constexpr int kRegKeys = 64;    // keys per LDS stage
constexpr int kRegMaxD = 128;

template <typename T, int DP>
struct RegLds
{
    static constexpr int V = 16 / sizeof(T);
    // [key][dim]: 16-byte fragment reads of eight consecutive keys fall in different banks
    static constexpr int kPitchK = sizeof(T) == 2 ? DP + 8 : DP + 4;
    // binary32 V is stored transposed, [dim][key], with a pitch that keeps the 16-byte reads along the keys apart;
    // binary16 V stays [key][dim] and the fragments come out of transposing reads (ds_read_tr16_b64: the 16 lanes of
    // a group address 4 keys x 16 dimensions as 8-byte pieces and lane i receives the 4 keys of dimension i), the
    // pitch of 32 bytes more than a row puts the 4 keys of a group in different banks
    static constexpr int kPitchV = sizeof(T) == 2 ? DP + 16 : kRegKeys + 4;
    static constexpr int kElemsV = sizeof(T) == 2 ? kRegKeys * kPitchV : DP * kPitchV;
    static constexpr int kElems = kRegKeys * kPitchK > kElemsV ? kRegKeys * kPitchK : kElemsV;
};

typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

template <typename T>
struct RegFrag;
template <>
struct RegFrag<f16>
{
    typedef f16x8 type;
};
template <>
struct RegFrag<float>
{
    typedef f32x4 type;
};

// V consecutive elements of a row starting at element e0, zero where the row or the element does not exist.
template <typename T>
__device__ inline typename RegFrag<T>::type load_piece(T const* __restrict__ row, int const e0, int const n,
    bool const rowExists, bool const vec)
{
    constexpr int V = 16 / sizeof(T);
    typename RegFrag<T>::type f;
    if (rowExists && vec && e0 + V <= n)
    {
        f = *reinterpret_cast<typename RegFrag<T>::type const*>(row + e0);
    }
    else
    {
#pragma unroll
        for (int i = 0; i < V; ++i)
        {
            f[i] = (rowExists && e0 + i < n) ? row[e0 + i] : (T) 0.f;
        }
    }
    return f;
}

// Wavefronts per SIMD the register allocation aims at: what the scores of a query (NT tiles of 4 registers) leave
// room for without spills.
template <typename T, int DP, int NT>
constexpr int reg_waves()
{
    constexpr bool big = DP > 64, bigF32 = big && sizeof(T) == 4;
    return NT <= 8 ? (big ? 3 : 4) : NT <= 16 ? (bigF32 ? 2 : 3) : 2;
}

template <typename T, int DP, int NT>
__global__ __launch_bounds__(kBlock, (reg_waves<T, DP, NT>())) void attention_in_registers_kernel(int const S, int const heads, int const d,
    int const strips, float const w, T const* __restrict__ qkv, int64_t const ldQKV,
    int32_t const* __restrict__ maskIdx, T* __restrict__ out, int64_t const ldOut, int const vecIn, int const vecOut)
{
    using L = RegLds<T, DP>;
    using Frag = typename RegFrag<T>::type;
    constexpr int V = L::V;
    constexpr int kPieces = DP / V;       // 16-byte pieces of a padded row
    constexpr int kSteps = DP / (4 * V);  // fragments of a query: 4 lane groups x V dimensions each
    constexpr int kChunks = NT / 4;       // LDS stages of 64 keys
    constexpr int kDimTiles = DP / 16;
    constexpr bool kHalf = sizeof(T) == 2;
    constexpr int NP = kRegKeys * kPieces / kBlock; // pieces of a stage per thread
    // stages requested ahead of the one being multiplied, held in registers until their turn in LDS: the binary16
    // products of a stage are far shorter than a trip to memory, the binary32 ones are not
    constexpr int D = kHalf ? (DP <= 64 ? 4 : 2) : 1;
    // binary16: two LDS stages in turn, so that a stage is written while the one before it is still being read and one
    // barrier per stage is enough; binary32 (long products per stage, three times the LDS) keeps one stage and two
    constexpr int kStages = kHalf ? 2 : 1;
    __shared__ __attribute__((aligned(16))) T ldsAll[kStages * L::kElems];

    // the strips of a (batch, head) unit read the same K and V: on one XCD, whose L2 then fetches them once
    // (S=384, B=32, N=12 in binary16: 49.2 -> 40.0 us)
    UnitPart const up = unit_of_workgroup(blockIdx.x, gridDim.x, strips);
    int const strip = up.part;
    int const z = (int) up.unit; // batch * heads + head
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const n = lane & 15, g = lane >> 4;
    int const query = strip * kRegQueries + wave * 16 + n;
    bool const vec = vecIn != 0;
    T const* const qp = qkv + (int64_t) z * 3 * d;
    T const* const kp = qp + d;
    T const* const vp = qp + 2 * d;
    int valid = S;
    if (maskIdx)
    {
        valid = max(0, min(S, maskIdx[z / heads]));
    }
    int const nChunks = (valid + kRegKeys - 1) / kRegKeys;

    // this lane's part of its query: the B operand of every Q K^T step
    Frag qf[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t)
    {
        qf[t] = load_piece<T>(qp + (int64_t) query * ldQKV, 4 * V * t + V * g, d, query < S, vec);
    }

    // ---- S^T = K Q^T: tile j of the accumulators holds keys 16 j + 4 g + i of query n ---------------------------
    Frag ring[D][NP];
    // K (and binary16 V): consecutive threads take the pieces of one key (whole rows per access); binary32 V:
    // consecutive threads take consecutive keys, so that the transposing LDS writes of a wavefront are consecutive
    auto fetch_k = [&](Frag(&dst)[NP], int const c)
    {
#pragma unroll
        for (int it = 0; it < NP; ++it)
        {
            int const p = threadIdx.x + it * kBlock;
            int const gk = c * kRegKeys + p / kPieces;
            dst[it] = load_piece<T>(kp + (int64_t) gk * ldQKV, (p % kPieces) * V, d, gk < S, vec);
        }
    };
    auto fetch_v = [&](Frag(&dst)[NP], int const c)
    {
#pragma unroll
        for (int it = 0; it < NP; ++it)
        {
            int const p = threadIdx.x + it * kBlock;
            int const gk = c * kRegKeys + (kHalf ? p / kPieces : p % kRegKeys);
            dst[it] = load_piece<T>(vp + (int64_t) gk * ldQKV, (kHalf ? p % kPieces : p / kRegKeys) * V, d, gk < S,
                vec);
        }
    };
#pragma unroll
    for (int c = 0; c < D; ++c)
    {
        if (c < nChunks)
        {
            fetch_k(ring[c], c);
        }
    }
    f32x4 acc[NT];
#pragma unroll
    for (int c = 0; c < kChunks; ++c)
    {
        if (c < nChunks)
        {
            T* const lds = ldsAll + (c % kStages) * L::kElems;
            if constexpr (kStages == 1)
            {
                __syncthreads();
            }
#pragma unroll
            for (int it = 0; it < NP; ++it)
            {
                int const p = threadIdx.x + it * kBlock;
                *reinterpret_cast<Frag*>(&lds[(p / kPieces) * L::kPitchK + (p % kPieces) * V]) = ring[c % D][it];
            }
            __syncthreads();
            if (c + D < kChunks && c + D < nChunks)
            {
                fetch_k(ring[c % D], c + D);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int t = 0; t < kSteps; ++t)
                {
                    if (4 * V * t < d)
                    {
                        Frag const kf
                            = *reinterpret_cast<Frag const*>(&lds[(16 * j + n) * L::kPitchK + 4 * V * t + V * g]);
                        if constexpr (kHalf)
                        {
                            s = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[t], s, 0, 0, 0);
                        }
                        else
                        {
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                            {
                                s = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[i], qf[t][i], s, 0, 0, 0);
                            }
                        }
                    }
                }
                acc[4 * c + j] = s;
            }
        }
    }

    // the first V stages are on their way while the softmax runs
#pragma unroll
    for (int c = 0; c < D; ++c)
    {
        if (c < nChunks)
        {
            fetch_v(ring[c], c);
        }
    }

    // ---- softmax over the keys of a query: in the lane, then across the four lane groups ------------------------
    float const wl2 = w * 1.4426950408889634f;
    float mx = -3.0e38f;
#pragma unroll
    for (int c = 0; c < kChunks; ++c)
    {
        if (c < nChunks)
        {
#pragma unroll
            for (int j = 4 * c; j < 4 * c + 4; ++j)
            {
                // the scores as the GEMM of the three-kernel path stores them
                f32x4 x = acc[j];
                if constexpr (kHalf)
                {
                    x = __builtin_convertvector(__builtin_convertvector(x, f16x4), f32x4);
                }
                if (16 * j + 16 > valid)
                {
                    // the ragged tile (uniform branch): a masked key gets the most negative score, whose
                    // exponential below is exactly 0
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        x[i] = 16 * j + 4 * g + i < valid ? x[i] : -3.0e38f;
                    }
                }
                acc[j] = x;
                mx = fmaxf(fmaxf(mx, fmaxf(x[0], x[1])), fmaxf(x[2], x[3]));
            }
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    // exp((x - max) w) as one fma per score, the way the reference's kernel forms it (x w - max w)
    float const nmx = -mx * wl2;
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < kChunks; ++c)
    {
        if (c < nChunks)
        {
#pragma unroll
            for (int j = 4 * c; j < 4 * c + 4; ++j)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    float const e = __builtin_amdgcn_exp2f(fmaf(acc[j][i], wl2, nmx));
                    acc[j][i] = e;
                    sum += e;
                }
            }
        }
    }
    sum += __shfl_xor(sum, 16);
    sum += __shfl_xor(sum, 32);
    float const rz = 1.f / sum;

    // ---- O^T = V^T P^T ------------------------------------------------------------------------------------------
    f32x4 o[kDimTiles];
#pragma unroll
    for (int dt = 0; dt < kDimTiles; ++dt)
    {
        o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int c = 0; c < kChunks; ++c)
    {
        if (c < nChunks)
        {
            // the probabilities of this chunk as the softmax of the three-kernel path stores them
            typedef T Tx4 __attribute__((ext_vector_type(4)));
            Tx4 pr[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                pr[j] = __builtin_convertvector(acc[4 * c + j] * rz, Tx4);
            }
            // the stages go on taking turns behind the last one of K
            T* const lds = ldsAll + ((nChunks + c) % kStages) * L::kElems;
            if constexpr (kStages == 1)
            {
                __syncthreads();
            }
#pragma unroll
            for (int it = 0; it < NP; ++it)
            {
                int const p = threadIdx.x + it * kBlock;
                if constexpr (kHalf)
                {
                    *reinterpret_cast<Frag*>(&lds[(p / kPieces) * L::kPitchV + (p % kPieces) * V]) = ring[c % D][it];
                }
                else
                {
#pragma unroll
                    for (int i = 0; i < V; ++i)
                    {
                        lds[((p / kRegKeys) * V + i) * L::kPitchV + p % kRegKeys] = ring[c % D][it][i];
                    }
                }
            }
            __syncthreads();
            if (c + D < kChunks && c + D < nChunks)
            {
                fetch_v(ring[c % D], c + D);
            }
#pragma unroll
            for (int dt = 0; dt < kDimTiles; ++dt)
            {
                if (16 * dt < d)
                {
                    T const* const vrow = &lds[(16 * dt + n) * L::kPitchV];
                    if constexpr (kHalf)
                    {
#pragma unroll
                        for (int s = 0; s < 2; ++s)
                        {
                            // this lane's address: key 32 s + 4 g + n / 4, dimensions 16 dt + 4 (n % 4) .. + 3;
                            // it receives keys 32 s + 4 g .. + 3 (and those 16 further) of dimension 16 dt + n
                            T const* const vb = &lds[(32 * s + 4 * g + (n >> 2)) * L::kPitchV + 16 * dt + 4 * (n & 3)];
                            i16x4 const lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) vb);
                            i16x4 const hi
                                = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) (vb + 16 * L::kPitchV));
                            f16x8 const vf = __builtin_bit_cast(
                                f16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                            f16x8 const pf = __builtin_shufflevector(pr[2 * s], pr[2 * s + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                            o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, o[dt], 0, 0, 0);
                        }
                    }
                    else
                    {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                        {
                            f32x4 const vf = *reinterpret_cast<f32x4 const*>(vrow + 16 * j + 4 * g);
#pragma unroll
                            for (int i = 0; i < 4; ++i)
                            {
                                o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[i], pr[j][i], o[dt], 0, 0, 0);
                            }
                        }
                    }
                }
            }
        }
    }

    // accumulator i of tile dt: dimension 16 dt + 4 g + i of query n
    if (query < S)
    {
        T* const orow = out + (int64_t) query * ldOut + (int64_t) z * d;
#pragma unroll
        for (int dt = 0; dt < kDimTiles; ++dt)
        {
            int const d0 = 16 * dt + 4 * g;
            T res[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                res[i] = (T) o[dt][i];
            }
            if (vecOut && d0 + 4 <= d)
            {
                typedef T Tx4 __attribute__((ext_vector_type(4)));
                *reinterpret_cast<Tx4*>(orow + d0) = Tx4{res[0], res[1], res[2], res[3]};
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    if (d0 + i < d)
                    {
                        orow[d0 + i] = res[i];
                    }
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// One launch for sequences beyond 512 keys (head size <= 128): the scores of a query no longer fit in registers, so
// the keys are walked twice in stages of 64.  The first pass computes the scores of a stage, keeps each lane's running
// maximum and the sum of exponentials relative to it (rescaled when the maximum moves) and drops the scores; the four
// lane groups of a query are combined at the end.  The second pass computes the scores again, forms the
// probabilities with the row's maximum and sum now known, rounds them to T as the softmax of the three-kernel path
// stores them, and multiplies them with V.  Same roundings as the kernel above (scores to T, probabilities to T,
// binary32 accumulation); the only difference to it is the order of the binary32 sum of exponentials.  K is read
// twice and the first product is computed twice; no score goes to memory.
// Work split, operand layouts in LDS and fragment orders are those of attention_in_registers_kernel; K and V each
// have one LDS stage and are fetched into registers D stages ahead.
// ------------------------------------------------------------------------------------------
template <typename T, int DP>
__global__ __launch_bounds__(kBlock, 2) void attention_two_pass_kernel(int const S, int const heads, int const d,
    int const strips, float const w, T const* __restrict__ qkv, int64_t const ldQKV,
    int32_t const* __restrict__ maskIdx, T* __restrict__ out, int64_t const ldOut, int const vecIn, int const vecOut)
{
    using L = RegLds<T, DP>;
    using Frag = typename RegFrag<T>::type;
    constexpr int V = L::V;
    constexpr int kPieces = DP / V;
    constexpr int kSteps = DP / (4 * V);
    constexpr int kDimTiles = DP / 16;
    constexpr bool kHalf = sizeof(T) == 2;
    constexpr int NP = kRegKeys * kPieces / kBlock;
    constexpr int D = kHalf ? (DP <= 64 ? 3 : 2) : 1; // stages in flight ahead of the one in LDS
    __shared__ __attribute__((aligned(16))) T ldsK[kRegKeys * L::kPitchK];
    __shared__ __attribute__((aligned(16))) T ldsV[L::kElemsV];

    UnitPart const up = unit_of_workgroup(blockIdx.x, gridDim.x, strips); // a unit's strips on one XCD
    int const strip = up.part;
    int const z = (int) up.unit;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const n = lane & 15, g = lane >> 4;
    int const query = strip * kRegQueries + wave * 16 + n;
    bool const vec = vecIn != 0;
    T const* const qp = qkv + (int64_t) z * 3 * d;
    T const* const kp = qp + d;
    T const* const vp = qp + 2 * d;
    int valid = S;
    if (maskIdx)
    {
        valid = max(0, min(S, maskIdx[z / heads]));
    }
    int const nChunks = (valid + kRegKeys - 1) / kRegKeys;

    Frag qf[kSteps];
#pragma unroll
    for (int t = 0; t < kSteps; ++t)
    {
        qf[t] = load_piece<T>(qp + (int64_t) query * ldQKV, 4 * V * t + V * g, d, query < S, vec);
    }
    auto fetch_k = [&](Frag(&dst)[NP], int const c)
    {
#pragma unroll
        for (int it = 0; it < NP; ++it)
        {
            int const p = threadIdx.x + it * kBlock;
            int const gk = c * kRegKeys + p / kPieces;
            dst[it] = load_piece<T>(kp + (int64_t) gk * ldQKV, (p % kPieces) * V, d, gk < S, vec);
        }
    };
    auto fetch_v = [&](Frag(&dst)[NP], int const c)
    {
#pragma unroll
        for (int it = 0; it < NP; ++it)
        {
            int const p = threadIdx.x + it * kBlock;
            int const gk = c * kRegKeys + (kHalf ? p / kPieces : p % kRegKeys);
            dst[it] = load_piece<T>(vp + (int64_t) gk * ldQKV, (kHalf ? p % kPieces : p / kRegKeys) * V, d, gk < S,
                vec);
        }
    };
    auto store_k = [&](Frag const(&src)[NP])
    {
#pragma unroll
        for (int it = 0; it < NP; ++it)
        {
            int const p = threadIdx.x + it * kBlock;
            *reinterpret_cast<Frag*>(&ldsK[(p / kPieces) * L::kPitchK + (p % kPieces) * V]) = src[it];
        }
    };
    auto store_v = [&](Frag const(&src)[NP])
    {
#pragma unroll
        for (int it = 0; it < NP; ++it)
        {
            int const p = threadIdx.x + it * kBlock;
            if constexpr (kHalf)
            {
                *reinterpret_cast<Frag*>(&ldsV[(p / kPieces) * L::kPitchV + (p % kPieces) * V]) = src[it];
            }
            else
            {
#pragma unroll
                for (int i = 0; i < V; ++i)
                {
                    ldsV[((p / kRegKeys) * V + i) * L::kPitchV + p % kRegKeys] = src[it][i];
                }
            }
        }
    };
    // the scores of the stage in ldsK, as the GEMM of the three-kernel path stores them; masked keys of the ragged
    // tile get the most negative score, whose exponential is exactly 0
    auto scores = [&](f32x4(&x)[4], int const c)
    {
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            f32x4 sc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int t = 0; t < kSteps; ++t)
            {
                if (4 * V * t < d)
                {
                    Frag const kf = *reinterpret_cast<Frag const*>(&ldsK[(16 * j + n) * L::kPitchK + 4 * V * t + V * g]);
                    if constexpr (kHalf)
                    {
                        sc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kf, qf[t], sc, 0, 0, 0);
                    }
                    else
                    {
#pragma unroll
                        for (int i = 0; i < 4; ++i)
                        {
                            sc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[i], qf[t][i], sc, 0, 0, 0);
                        }
                    }
                }
            }
            if constexpr (kHalf)
            {
                sc = __builtin_convertvector(__builtin_convertvector(sc, f16x4), f32x4);
            }
            int const key0 = c * kRegKeys + 16 * j;
            if (key0 + 16 > valid)
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    sc[i] = key0 + 4 * g + i < valid ? sc[i] : -3.0e38f;
                }
            }
            x[j] = sc;
        }
    };

    float const wl2 = w * 1.4426950408889634f;
    Frag ringK[D][NP];

    // ---- first pass: row maximum and sum of exponentials -------------------------------------------------------
    float mx = -3.0e38f, sum = 0.f;
#pragma unroll
    for (int u = 0; u < D; ++u)
    {
        if (u < nChunks)
        {
            fetch_k(ringK[u], u);
        }
    }
    for (int c0 = 0; c0 < nChunks; c0 += D)
    {
#pragma unroll
        for (int u = 0; u < D; ++u)
        {
            int const c = c0 + u;
            if (c < nChunks)
            {
                __syncthreads(); // the stage before this one has been read by everyone
                store_k(ringK[u]);
                __syncthreads();
                if (c + D < nChunks)
                {
                    fetch_k(ringK[u], c + D);
                }
                f32x4 x[4];
                scores(x, c);
                float cm = mx;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    cm = fmaxf(fmaxf(cm, fmaxf(x[j][0], x[j][1])), fmaxf(x[j][2], x[j][3]));
                }
                // the sum so far, relative to the new maximum (a factor of exactly 1 when it did not move)
                sum *= __builtin_amdgcn_exp2f((mx - cm) * wl2);
                mx = cm;
                float const nm = -cm * wl2;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        sum += __builtin_amdgcn_exp2f(fmaf(x[j][i], wl2, nm));
                    }
                }
            }
        }
    }
    // the four lane groups of a query hold disjoint keys: bring their sums to the common maximum and add them
    {
        float all = fmaxf(mx, __shfl_xor(mx, 16));
        all = fmaxf(all, __shfl_xor(all, 32));
        sum *= __builtin_amdgcn_exp2f((mx - all) * wl2);
        mx = all;
        sum += __shfl_xor(sum, 16);
        sum += __shfl_xor(sum, 32);
    }
    float const nmx = -mx * wl2;
    float const rz = 1.f / sum;

    // ---- second pass: the scores again, probabilities, O^T = V^T P^T ---------------------------------------------
    Frag ringV[D][NP];
#pragma unroll
    for (int u = 0; u < D; ++u)
    {
        if (u < nChunks)
        {
            fetch_k(ringK[u], u);
            fetch_v(ringV[u], u);
        }
    }
    f32x4 o[kDimTiles];
#pragma unroll
    for (int dt = 0; dt < kDimTiles; ++dt)
    {
        o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    for (int c0 = 0; c0 < nChunks; c0 += D)
    {
#pragma unroll
        for (int u = 0; u < D; ++u)
        {
            int const c = c0 + u;
            if (c < nChunks)
            {
                __syncthreads();
                store_k(ringK[u]);
                store_v(ringV[u]);
                __syncthreads();
                if (c + D < nChunks)
                {
                    fetch_k(ringK[u], c + D);
                    fetch_v(ringV[u], c + D);
                }
                f32x4 x[4];
                scores(x, c);
                typedef T Tx4 __attribute__((ext_vector_type(4)));
                Tx4 pr[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    f32x4 e;
#pragma unroll
                    for (int i = 0; i < 4; ++i)
                    {
                        e[i] = __builtin_amdgcn_exp2f(fmaf(x[j][i], wl2, nmx));
                    }
                    pr[j] = __builtin_convertvector(e * rz, Tx4);
                }
#pragma unroll
                for (int dt = 0; dt < kDimTiles; ++dt)
                {
                    if (16 * dt < d)
                    {
                        if constexpr (kHalf)
                        {
#pragma unroll
                            for (int s2 = 0; s2 < 2; ++s2)
                            {
                                T const* const vb
                                    = &ldsV[(32 * s2 + 4 * g + (n >> 2)) * L::kPitchV + 16 * dt + 4 * (n & 3)];
                                i16x4 const lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) vb);
                                i16x4 const hi
                                    = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) (vb + 16 * L::kPitchV));
                                f16x8 const vf = __builtin_bit_cast(
                                    f16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
                                f16x8 const pf
                                    = __builtin_shufflevector(pr[2 * s2], pr[2 * s2 + 1], 0, 1, 2, 3, 4, 5, 6, 7);
                                o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf, pf, o[dt], 0, 0, 0);
                            }
                        }
                        else
                        {
                            T const* const vrow = &ldsV[(16 * dt + n) * L::kPitchV];
#pragma unroll
                            for (int j = 0; j < 4; ++j)
                            {
                                f32x4 const vf = *reinterpret_cast<f32x4 const*>(vrow + 16 * j + 4 * g);
#pragma unroll
                                for (int i = 0; i < 4; ++i)
                                {
                                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[i], pr[j][i], o[dt], 0, 0, 0);
                                }
                            }
                        }
                    }
                }
            }
        }
    }

    if (query < S)
    {
        T* const orow = out + (int64_t) query * ldOut + (int64_t) z * d;
#pragma unroll
        for (int dt = 0; dt < kDimTiles; ++dt)
        {
            int const d0 = 16 * dt + 4 * g;
            T res[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
            {
                res[i] = (T) o[dt][i];
            }
            if (vecOut && d0 + 4 <= d)
            {
                typedef T Tx4 __attribute__((ext_vector_type(4)));
                *reinterpret_cast<Tx4*>(orow + d0) = Tx4{res[0], res[1], res[2], res[3]};
            }
            else
            {
#pragma unroll
                for (int i = 0; i < 4; ++i)
                {
                    if (d0 + i < d)
                    {
                        orow[d0 + i] = res[i];
                    }
                }
            }
        }
    }
}

template <typename T, int DP>
int launch_attention_in_registers(hipStream_t stream, int32_t S, int32_t B, int32_t N, int32_t d, T const* qkv,
    int32_t const* maskIdx, T* output)
{
    constexpr int64_t V = 16 / sizeof(T);
    int64_t const ldQKV = (int64_t) 3 * B * N * d;
    int64_t const ldOut = (int64_t) B * N * d;
    int const strips = ceil_div(S, kRegQueries);
    int64_t const groups = (int64_t) strips * B * N;
    if (groups * kBlock > 0xffffffffll) // a launch holds fewer than 2^32 threads
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: %lld workgroups exceed the grid", (long long) groups);
    }
    // 16-byte reads of a row's pieces: every row of Q, K and V starts at a multiple of d elements from the base
    int const vecIn = d % V == 0 && (reinterpret_cast<uintptr_t>(qkv) & 15u) == 0;
    int const vecOut = d % 4 == 0 && (reinterpret_cast<uintptr_t>(output) & (4 * sizeof(T) - 1)) == 0;
    float const w = 1.f / sqrtf((float) d);
    dim3 const grid((unsigned) groups), block(kBlock);
    int const tiles = ceil_div(S, 16);
#define TRTAMD_LAUNCH_REG(NT_)                                                                                        \
    hipLaunchKernelGGL((attention_in_registers_kernel<T, DP, NT_>), grid, block, 0, stream, S, N, d, strips, w, qkv,   \
        ldQKV, maskIdx, output, ldOut, vecIn, vecOut)
    if (tiles <= 8)
    {
        TRTAMD_LAUNCH_REG(8);
    }
    else if (tiles <= 16)
    {
        TRTAMD_LAUNCH_REG(16);
    }
    else if (tiles <= 24)
    {
        TRTAMD_LAUNCH_REG(24);
    }
    else if (tiles <= 32)
    {
        TRTAMD_LAUNCH_REG(32);
    }
    else
    {
        hipLaunchKernelGGL((attention_two_pass_kernel<T, DP>), grid, block, 0, stream, S, N, d, strips, w, qkv, ldQKV,
            maskIdx, output, ldOut, vecIn, vecOut);
        return check_launch("attention_two_pass_kernel");
    }
#undef TRTAMD_LAUNCH_REG
    return check_launch("attention_in_registers_kernel");
}

// Whether a shape runs in one of the one-launch kernels (and so needs no score matrices): every sequence length, head
// sizes up to 128.  The tuning switch
// TRTAMD_UNFUSED_SPLIT=1 keeps every shape on the three kernels with the score matrices in the workspace; an entry
// point asks once per call and hands the answer down.
bool runs_in_one_launch(int32_t S, int32_t d)
{
    return d <= kRegMaxD && tuning(Tuning::kUnfusedSplit) == 0;
}

template <typename T>
int unfused_mha(hipStream_t stream, int32_t S, int32_t B, int32_t N, int32_t d, T const* qkv, int32_t const* maskIdx,
    T* output, void* workspace, bool const inRegisters)
{
    if (inRegisters)
    {
        return d <= 64 ? launch_attention_in_registers<T, 64>(stream, S, B, N, d, qkv, maskIdx, output)
                       : launch_attention_in_registers<T, 128>(stream, S, B, N, d, qkv, maskIdx, output);
    }
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
    hipLaunchKernelGGL((batched_gemm_kernel<T>), g1, dim3(kBlock), 0, stream, S, S, d, N, q, oq, k, okT, qk, os,
        can_vectorise(q, oq), can_vectorise(k, okT));
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
    hipLaunchKernelGGL((batched_gemm_kernel<T>), g2, dim3(kBlock), 0, stream, S, d, S, N, pp, os, v, ov, output, oo,
        can_vectorise(pp, os), can_vectorise(v, ov));
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

namespace trtamd
{
namespace
{
// Both entry points of the unfused attention after their own checks; inRegisters: the caller's one reading of
// runs_in_one_launch for this call.
int run_unfused(trtamd_stream_t stream, int32_t type, int32_t S, int32_t B, int32_t N, int32_t d, void const* qkv,
    int32_t const* maskIdx, void* output, void* workspace, bool const inRegisters)
{
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
            static_cast<float*>(output), workspace, inRegisters);
    }
    return unfused_mha<f16>(as_stream(stream), S, B, N, d, static_cast<f16 const*>(qkv), maskIdx,
        static_cast<f16*>(output), workspace, inRegisters);
}
} // namespace
} // namespace trtamd

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
    return trtamd::run_unfused(stream, type, S, B, N, d, qkv, maskIdx, output, workspace,
        trtamd::runs_in_one_launch(S, d));
}

extern "C" int trtamd_unfused_mha_routed(trtamd_stream_t stream, int32_t route, int32_t type, int32_t S, int32_t B,
    int32_t N, int32_t d, void const* qkv, int32_t const* maskIdx, void* output, void* workspace)
{
    if (route == TRTAMD_UNFUSED_ROUTE_BY_SHAPE)
    {
        return trtamd_unfused_mha(stream, type, S, B, N, d, qkv, maskIdx, output, workspace);
    }
    if (route != TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH && route != TRTAMD_UNFUSED_ROUTE_THREE_LAUNCHES)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA: unknown route %d", route);
    }
    if (type != 0 && type != 1)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: data type %d (only FP32=0 and FP16=1)", type);
    }
    if (S <= 0 || B <= 0 || N <= 0 || d <= 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA: bad dimensions S=%d B=%d N=%d d=%d", S, B, N, d);
    }
    if (route == TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH && d > trtamd::kRegMaxD)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: no one-launch kernel for head size %d (limit %d)", d,
            trtamd::kRegMaxD);
    }
    return trtamd::run_unfused(stream, type, S, B, N, d, qkv, maskIdx, output, workspace,
        route == TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH);
}

extern "C" int trtamd_unfused_mha_tune(
    int32_t type, int32_t S, int32_t B, int32_t N, int32_t d, int32_t* route, float* microseconds)
{
    using namespace trtamd;
    if (route == nullptr)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA tuning: null route pointer");
    }
    *route = TRTAMD_UNFUSED_ROUTE_BY_SHAPE;
    float us[2] = {-1.f, -1.f};
    auto report = [&] {
        if (microseconds)
        {
            microseconds[0] = us[0];
            microseconds[1] = us[1];
        }
    };
    report();
    if (type != 0 && type != 1)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "unfused MHA: data type %d (only FP32=0 and FP16=1)", type);
    }
    if (S <= 0 || B <= 0 || N <= 0 || d <= 0 || (int64_t) B * N > 65535)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "unfused MHA: bad dimensions S=%d B=%d N=%d d=%d", S, B, N, d);
    }
    if (d > kRegMaxD)
    {
        *route = TRTAMD_UNFUSED_ROUTE_THREE_LAUNCHES; // the only route there is
        return TRTAMD_STATUS_SUCCESS;
    }
    // the timed problem: the configured one, with the batch halved until the score matrices fit 1 GiB
    constexpr size_t kMaxWorkspace = (size_t) 1 << 30;
    int32_t bt = B;
    while (bt > 1 && trtamd_unfused_mha_workspace_size(type, S, bt, N) > kMaxWorkspace)
    {
        bt = (bt + 1) / 2;
    }
    size_t const wsBytes = trtamd_unfused_mha_workspace_size(type, S, bt, N);
    if (wsBytes > kMaxWorkspace)
    {
        return TRTAMD_STATUS_SUCCESS; // by shape
    }
    size_t const word = type == 0 ? 4 : 2;
    size_t const outBytes = word * (size_t) S * (size_t) bt * (size_t) N * (size_t) d;
    void *qkv = nullptr, *out = nullptr, *ws = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t e0 = nullptr, e1 = nullptr;
    auto release = [&] {
        if (e0) (void) hipEventDestroy(e0);
        if (e1) (void) hipEventDestroy(e1);
        if (stream) (void) hipStreamDestroy(stream);
        if (qkv) (void) hipFree(qkv);
        if (out) (void) hipFree(out);
        if (ws) (void) hipFree(ws);
    };
    bool ok = hipMalloc(&qkv, 3 * outBytes) == hipSuccess && hipMalloc(&out, outBytes) == hipSuccess
        && hipMalloc(&ws, wsBytes) == hipSuccess && hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) == hipSuccess
        && hipEventCreate(&e0) == hipSuccess && hipEventCreate(&e1) == hipSuccess;
    // every element the same small positive number (0x3c3c... is 1.06 in binary16 and 0.0115 in binary32)
    ok = ok && hipMemsetAsync(qkv, 0x3c, 3 * outBytes, stream) == hipSuccess;
    if (!ok)
    {
        (void) hipGetLastError(); // best effort: without buffers the choice stays with the shape
        release();
        return TRTAMD_STATUS_SUCCESS;
    }
    constexpr int kWarm = 2, kTimed = 5;
    int status = TRTAMD_STATUS_SUCCESS;
    for (int r = 0; r < 2 && status == TRTAMD_STATUS_SUCCESS; ++r)
    {
        for (int i = 0; i < kWarm + kTimed && status == TRTAMD_STATUS_SUCCESS; ++i)
        {
            if (i == kWarm && hipEventRecord(e0, stream) != hipSuccess)
            {
                status = set_error(TRTAMD_STATUS_FAILURE, "unfused MHA tuning: event record failed");
                break;
            }
            status = run_unfused(stream, type, S, bt, N, d, qkv, nullptr, out, ws, r == TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH);
        }
        float ms = 0.f;
        if (status == TRTAMD_STATUS_SUCCESS
            && (hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess
                || hipEventElapsedTime(&ms, e0, e1) != hipSuccess))
        {
            status = set_error(TRTAMD_STATUS_FAILURE, "unfused MHA tuning: timing failed");
        }
        us[r] = ms * 1000.f / kTimed;
    }
    (void) hipStreamSynchronize(stream);
    release();
    if (status != TRTAMD_STATUS_SUCCESS)
    {
        return status;
    }
    *route = us[1] < us[0] ? TRTAMD_UNFUSED_ROUTE_THREE_LAUNCHES : TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH;
    report();
    return TRTAMD_STATUS_SUCCESS;
}

extern "C" size_t trtamd_unfused_mha_static_capacity(void)
{
    return kStaticScratchBytes;
}

extern "C" int trtamd_unfused_mha_static_prepare(void)
{
    void* ws = nullptr;
    return static_scratch(&ws);
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
    // Shapes of the one-launch kernels (head sizes up to 128) keep their scores in registers and touch nothing of the
    // array: no limit for them.  Otherwise 2 * wordSize * S*S * B*N bytes, in double arithmetic free of overflow (each factor is below 2^31).
    bool const inRegisters = trtamd::runs_in_one_launch(S, d);
    double const need = 2.0 * (type == 0 ? 4.0 : 2.0) * (double) S * (double) S * (double) B * (double) N;
    if (!inRegisters && need > (double) kStaticScratchBytes)
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
    return trtamd::run_unfused(stream, type, S, B, N, d, qkv, maskIdx, output, ws, inRegisters);
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
