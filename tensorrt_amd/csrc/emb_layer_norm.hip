// Embedding gather + LayerNorm, mask index and packed-mask kernels for gfx950.
//
// One wavefront per token: the word/segment ids are read once (wave-uniform), the three table
// rows are fetched with 16-byte loads, summed in T in the reference's order (word + tok) + pos,
// normalised from registers (Welford/Chan statistics in binary32) and written exactly once;
// the reference writes the sum, then re-reads and re-writes it from its LayerNorm helper.
//
// Replaces plugin/embLayerNormPlugin/embLayerNormKernel.cu,
// plugin/embLayerNormPlugin/embLayerNormVarSeqlenKernelHFace.cu and
// plugin/embLayerNormPlugin/embLayerNormVarSeqlenKernelMTron.cu of the reference.
#include "device_utils.hpp"
#include "host_utils.hpp"

namespace trtamd
{
namespace
{

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWaveSize;

enum EmbMode
{
    kFIXED = 0, // ids [S,B], token index s*B+b
    kHFACE = 1, // packed ids, cu_seqlens
    kMTRON = 2  // kHFACE + pre-LayerNorm sum as second output
};

template <typename T>
struct Vec16
{
    static constexpr int kN = 16 / sizeof(T);
    union
    {
        u32x4 u;
        T e[kN];
    };
};

// Token of this wave: fills tokenIdx (row of ids and of the output) and pos (row of the
// position table).  Returns false when the wave has nothing to do.
template <int MODE>
__device__ inline bool locate_token(int64_t wave, int B, int S, int32_t const* cu, int64_t& tokenIdx, int& pos)
{
    if (wave >= (int64_t) S * B)
    {
        return false;
    }
    if (MODE == kFIXED)
    {
        tokenIdx = wave;
        pos = (int) (wave / B);
        return true;
    }
    int const b = (int) (wave / S);
    int const s = (int) (wave % S);
    int const first = cu[b];
    int const len = cu[b + 1] - first;
    if (s >= len)
    {
        return false;
    }
    tokenIdx = (int64_t) first + s;
    pos = s;
    return true;
}

// TPW consecutive token slots per wavefront.  gamma and beta are fetched once per wavefront (converted to T and
// back, as the reference does per element) instead of once per token: at TPW = 1 they are two thirds of the
// bytes a token pulls through the vector cache.
template <typename T, int NV, int MODE, int TPW>
__global__ __launch_bounds__(kBlock) void embln_kernel(int const ld, int const B, int const S,
    int32_t const* __restrict__ inputIds, int32_t const* __restrict__ tokenIds, int32_t const* __restrict__ cuSeqlens,
    float const* __restrict__ beta, float const* __restrict__ gamma, T const* __restrict__ wordEmb,
    T const* __restrict__ posEmb, T const* __restrict__ tokEmb, int32_t const wordSize, int32_t const tokSize,
    T* __restrict__ output, T* __restrict__ skipOut)
{
    constexpr int VPT = Vec16<T>::kN;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int64_t const wave
        = __builtin_amdgcn_readfirstlane((int) ((int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)));
    int const nvec = ld / VPT;

    // gamma/beta take the output type first: `const R g(gamma[i])`, common.cuh:275-276
    float gk[NV][VPT], bk[NV][VPT];
#pragma unroll
    for (int j = 0; j < NV; ++j)
    {
        int const vi = lane + kWaveSize * j;
        bool const ok = vi < nvec;
#pragma unroll
        for (int q = 0; q < VPT / 4; ++q)
        {
            f32x4 const g4 = ok ? *reinterpret_cast<f32x4 const*>(gamma + vi * VPT + q * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
            f32x4 const b4 = ok ? *reinterpret_cast<f32x4 const*>(beta + vi * VPT + q * 4) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                gk[j][q * 4 + e] = (float) (T) g4[e];
                bk[j][q * 4 + e] = (float) (T) b4[e];
            }
        }
    }

#pragma unroll 1
    for (int it = 0; it < TPW; ++it)
    {
        int64_t tokenIdx;
        int pos;
        if (!locate_token<MODE>(wave * TPW + it, B, S, cuSeqlens, tokenIdx, pos))
        {
            continue;
        }
        int const wordId = __builtin_amdgcn_readfirstlane(inputIds[tokenIdx]);
        int const tokId = __builtin_amdgcn_readfirstlane(tokenIds[tokenIdx]);
        bool const inRange = wordId >= 0 && wordId < wordSize && tokId >= 0 && tokId < tokSize;

        Vec16<T> w[NV], t[NV], p[NV];
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            int const vi = lane + kWaveSize * j;
            bool const ok = vi < nvec && inRange;
            w[j].u = ok ? *reinterpret_cast<u32x4 const*>(wordEmb + (int64_t) wordId * ld + vi * VPT) : u32x4{0, 0, 0, 0};
            t[j].u = ok ? *reinterpret_cast<u32x4 const*>(tokEmb + (int64_t) tokId * ld + vi * VPT) : u32x4{0, 0, 0, 0};
            p[j].u = ok ? *reinterpret_cast<u32x4 const*>(posEmb + (int64_t) pos * ld + vi * VPT) : u32x4{0, 0, 0, 0};
        }

        float v[NV][VPT];
        float sum = 0.f, cnt = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            bool const ok = lane + kWaveSize * j < nvec;
            Vec16<T> pre;
#pragma unroll
            for (int k = 0; k < VPT; ++k)
            {
                T const s = (w[j].e[k] + t[j].e[k]) + p[j].e[k];
                pre.e[k] = s;
                v[j][k] = (float) s;
                sum += ok ? v[j][k] : 0.f;
            }
            cnt += ok ? (float) VPT : 0.f;
            if (MODE == kMTRON && ok)
            {
                store_through_l2(skipOut + tokenIdx * ld + (int64_t) (lane + kWaveSize * j) * VPT, pre.u);
            }
        }
        Welford st;
        st.n = cnt;
        st.mean = cnt > 0.f ? sum / cnt : 0.f;
        st.m2 = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            bool const ok = lane + kWaveSize * j < nvec;
#pragma unroll
            for (int k = 0; k < VPT; ++k)
            {
                float const dlt = v[j][k] - st.mean;
                st.m2 += ok ? dlt * dlt : 0.f;
            }
        }
        st = group_welford<kWaveSize>(st);
        float const mu = st.mean;
        // No epsilon (plugin/common/common.cuh:269).  Ids out of range leave the reference's row
        // undefined; here such a row is the LayerNorm of zeros with rsigma forced to 0, i.e. beta.
        float const rsigma = inRange ? rsqrtf(st.m2 / (float) ld) : 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            int const vi = lane + kWaveSize * j;
            if (vi < nvec)
            {
                Vec16<T> y;
#pragma unroll
                for (int k = 0; k < VPT; ++k)
                {
                    y.e[k] = (T) (gk[j][k] * (v[j][k] - mu) * rsigma + bk[j][k]);
                }
                store_through_l2(output + tokenIdx * ld + (int64_t) vi * VPT, y.u);
            }
        }
    }
}

// Any ld: scalar sweeps, one wave per token.
template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void embln_generic_kernel(int const ld, int const B, int const S,
    int32_t const* __restrict__ inputIds, int32_t const* __restrict__ tokenIds, int32_t const* __restrict__ cuSeqlens,
    float const* __restrict__ beta, float const* __restrict__ gamma, T const* __restrict__ wordEmb,
    T const* __restrict__ posEmb, T const* __restrict__ tokEmb, int32_t const wordSize, int32_t const tokSize,
    T* __restrict__ output, T* __restrict__ skipOut)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    int64_t const wave
        = __builtin_amdgcn_readfirstlane((int) ((int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6)));
    int64_t tokenIdx;
    int pos;
    if (!locate_token<MODE>(wave, B, S, cuSeqlens, tokenIdx, pos))
    {
        return;
    }
    int const wordId = __builtin_amdgcn_readfirstlane(inputIds[tokenIdx]);
    int const tokId = __builtin_amdgcn_readfirstlane(tokenIds[tokenIdx]);
    bool const inRange = wordId >= 0 && wordId < wordSize && tokId >= 0 && tokId < tokSize;
    auto value = [&](int i) -> T {
        if (!inRange)
        {
            return (T) 0.f;
        }
        return (wordEmb[(int64_t) wordId * ld + i] + tokEmb[(int64_t) tokId * ld + i]) + posEmb[(int64_t) pos * ld + i];
    };
    float sum = 0.f;
    for (int i = lane; i < ld; i += kWaveSize)
    {
        T const s = value(i);
        if (MODE == kMTRON)
        {
            skipOut[tokenIdx * ld + i] = s;
        }
        sum += (float) s;
    }
    float const mu = wave_sum(sum) / (float) ld;
    float m2 = 0.f;
    for (int i = lane; i < ld; i += kWaveSize)
    {
        float const dlt = (float) value(i) - mu;
        m2 += dlt * dlt;
    }
    float const rsigma = inRange ? rsqrtf(wave_sum(m2) / (float) ld) : 0.f;
    for (int i = lane; i < ld; i += kWaveSize)
    {
        float const gk = (float) (T) gamma[i];
        float const bk = (float) (T) beta[i];
        output[tokenIdx * ld + i] = (T) (gk * ((float) value(i) - mu) * rsigma + bk);
    }
}

template <typename T, int MODE>
int emb_layer_norm(hipStream_t stream, int32_t ld, int32_t B, int32_t S, int32_t const* inputIds,
    int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta, float const* gamma, T const* wordEmb,
    T const* posEmb, T const* tokEmb, int32_t wordSize, int32_t tokSize, T* output, T* skipOut)
{
    if (ld <= 0 || B < 0 || S < 0 || wordSize < 0 || tokSize < 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "EmbLayerNorm: negative size");
    }
    if (B == 0 || S == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!inputIds || !tokenIds || !beta || !gamma || !wordEmb || !posEmb || !tokEmb || !output
        || (MODE != kFIXED && !cuSeqlens) || (MODE == kMTRON && !skipOut))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "EmbLayerNorm: null tensor pointer");
    }
    if ((int64_t) S * B > 0x7fffffffLL)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "EmbLayerNorm: S*B exceeds 2^31-1");
    }
    constexpr int VPT = 16 / (int) sizeof(T);
    bool const vec_ok = ld % VPT == 0 && aligned16(wordEmb) && aligned16(posEmb) && aligned16(tokEmb)
        && aligned16(output) && aligned16(beta) && aligned16(gamma) && (MODE != kMTRON || aligned16(skipOut));
    int const nv = vec_ok ? ceil_div(ld / VPT, kWaveSize) : 0;
    dim3 const grid((unsigned) ceil_div<int64_t>((int64_t) S * B, kWavesPerBlock));
    // several tokens per wavefront once there are enough token slots to keep every SIMD busy anyway
    int64_t const slots = (int64_t) S * B;
    bool const multi = slots >= 65536;
    dim3 const grid4((unsigned) ceil_div<int64_t>(ceil_div<int64_t>(slots, 4), kWavesPerBlock));
#define TRTAMD_EMB_LAUNCH(NVV)                                                                                         \
    if (multi)                                                                                                         \
    {                                                                                                                  \
        hipLaunchKernelGGL((embln_kernel<T, NVV, MODE, 4>), grid4, dim3(kBlock), 0, stream, ld, B, S, inputIds,          \
            tokenIds, cuSeqlens, beta, gamma, wordEmb, posEmb, tokEmb, wordSize, tokSize, output, skipOut);            \
    }                                                                                                                  \
    else                                                                                                               \
    {                                                                                                                  \
        hipLaunchKernelGGL((embln_kernel<T, NVV, MODE, 1>), grid, dim3(kBlock), 0, stream, ld, B, S, inputIds,           \
            tokenIds, cuSeqlens, beta, gamma, wordEmb, posEmb, tokEmb, wordSize, tokSize, output, skipOut);            \
    }
    if (vec_ok && nv == 1)
    {
        TRTAMD_EMB_LAUNCH(1);
    }
    else if (vec_ok && nv == 2)
    {
        TRTAMD_EMB_LAUNCH(2);
    }
    else if (vec_ok && nv <= 4)
    {
        TRTAMD_EMB_LAUNCH(4);
    }
    else
    {
        hipLaunchKernelGGL((embln_generic_kernel<T, MODE>), grid, dim3(kBlock), 0, stream, ld, B, S, inputIds, tokenIds,
            cuSeqlens, beta, gamma, wordEmb, posEmb, tokEmb, wordSize, tokSize, output, skipOut);
    }
#undef TRTAMD_EMB_LAUNCH
    return check_launch("embln_kernel");
}

// maskIdx[b] = first s with mask[s,b] == 0, else S  (embLayerNormKernel.cu:98-183).
__global__ __launch_bounds__(kBlock) void mask_idx_kernel(
    int const S, int const B, int32_t const* __restrict__ mask, int32_t* __restrict__ maskIdx)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const b = blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (b >= B)
    {
        return;
    }
    int first = S;
    for (int s = lane; s < S; s += kWaveSize)
    {
        if (mask[(int64_t) s * B + b] == 0)
        {
            first = min(first, s);
        }
    }
    first = wave_min_i32(first);
    if (lane == 0)
    {
        maskIdx[b] = first;
    }
}

// Packed mask (embLayerNormKernel.cu:41-96): word (b, mi, tidx) holds, for each ni, the mask at
// columns off, off+1, off, off+1, off+8, off+9, off+8, off+9 with
// off = ni*16*warps_n + (tidx/32/warps_m)*16 + (tidx%4)*2; identical for every mi.
// Columns at or beyond S count as masked.
__global__ void convert_mask_kernel(uint32_t const warps_m, uint32_t const warps_n, uint32_t const S, uint32_t const B,
    uint32_t const xmmas_m, uint32_t const xmmas_n, int32_t const* __restrict__ maskSB, uint32_t* __restrict__ maskX)
{
    uint32_t const bi = blockIdx.x;
    uint32_t const threads = blockDim.x;
    uint32_t const tidx = threadIdx.x;
    uint32_t const warp_n = (tidx / 32) / warps_m;
    uint32_t const col = warp_n * 16 + (tidx % 4) * 2;
    auto at = [&](uint32_t k) -> uint32_t { return (k < S && maskSB[(int64_t) k * B + bi] == 1) ? 1u : 0u; };
    uint32_t word = 0;
    for (uint32_t ni = 0; ni < xmmas_n; ++ni)
    {
        uint32_t const off = ni * 16 * warps_n + col;
        uint32_t const m0 = at(off), m1 = at(off + 1), m8 = at(off + 8), m9 = at(off + 9);
        uint32_t const byte = m0 | (m1 << 1) | (m0 << 2) | (m1 << 3) | (m8 << 4) | (m9 << 5) | (m8 << 6) | (m9 << 7);
        word |= byte << (8 * ni);
    }
    for (uint32_t mi = 0; mi < xmmas_m; ++mi)
    {
        maskX[((int64_t) bi * xmmas_m + mi) * threads + tidx] = word;
    }
}

} // namespace
} // namespace trtamd

using namespace trtamd;

#define TRTAMD_HALF(p) reinterpret_cast<f16 const*>(p)

extern "C" int trtamd_emb_layer_norm_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, float const* beta, float const* gamma, float const* wordEmb,
    float const* posEmb, float const* tokEmb, int32_t wordSize, int32_t tokSize, float* output)
{
    return emb_layer_norm<float, kFIXED>(as_stream(stream), ld, B, S, inputIds, tokenIds, nullptr, beta, gamma, wordEmb,
        posEmb, tokEmb, wordSize, tokSize, output, nullptr);
}

extern "C" int trtamd_emb_layer_norm_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, float const* beta, float const* gamma,
    trtamd_half_t const* wordEmb, trtamd_half_t const* posEmb, trtamd_half_t const* tokEmb, int32_t wordSize,
    int32_t tokSize, trtamd_half_t* output)
{
    return emb_layer_norm<f16, kFIXED>(as_stream(stream), ld, B, S, inputIds, tokenIds, nullptr, beta, gamma,
        TRTAMD_HALF(wordEmb), TRTAMD_HALF(posEmb), TRTAMD_HALF(tokEmb), wordSize, tokSize,
        reinterpret_cast<f16*>(output), nullptr);
}

extern "C" int trtamd_emb_layer_norm_hface_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, float const* wordEmb, float const* posEmb, float const* tokEmb, int32_t wordSize,
    int32_t tokSize, float* output)
{
    return emb_layer_norm<float, kHFACE>(as_stream(stream), ld, B, S, inputIds, tokenIds, cuSeqlens, beta, gamma,
        wordEmb, posEmb, tokEmb, wordSize, tokSize, output, nullptr);
}

extern "C" int trtamd_emb_layer_norm_hface_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, trtamd_half_t const* wordEmb, trtamd_half_t const* posEmb, trtamd_half_t const* tokEmb,
    int32_t wordSize, int32_t tokSize, trtamd_half_t* output)
{
    return emb_layer_norm<f16, kHFACE>(as_stream(stream), ld, B, S, inputIds, tokenIds, cuSeqlens, beta, gamma,
        TRTAMD_HALF(wordEmb), TRTAMD_HALF(posEmb), TRTAMD_HALF(tokEmb), wordSize, tokSize,
        reinterpret_cast<f16*>(output), nullptr);
}

extern "C" int trtamd_emb_layer_norm_mtron_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, float const* wordEmb, float const* posEmb, float const* tokEmb, int32_t wordSize,
    int32_t tokSize, float* output, float* skip)
{
    return emb_layer_norm<float, kMTRON>(as_stream(stream), ld, B, S, inputIds, tokenIds, cuSeqlens, beta, gamma,
        wordEmb, posEmb, tokEmb, wordSize, tokSize, output, skip);
}

extern "C" int trtamd_emb_layer_norm_mtron_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, trtamd_half_t const* wordEmb, trtamd_half_t const* posEmb, trtamd_half_t const* tokEmb,
    int32_t wordSize, int32_t tokSize, trtamd_half_t* output, trtamd_half_t* skip)
{
    return emb_layer_norm<f16, kMTRON>(as_stream(stream), ld, B, S, inputIds, tokenIds, cuSeqlens, beta, gamma,
        TRTAMD_HALF(wordEmb), TRTAMD_HALF(posEmb), TRTAMD_HALF(tokEmb), wordSize, tokSize,
        reinterpret_cast<f16*>(output), reinterpret_cast<f16*>(skip));
}

extern "C" int trtamd_compute_mask_idx(
    trtamd_stream_t stream, int32_t S, int32_t B, int32_t const* mask, int32_t* maskIdx)
{
    if (S < 0 || B < 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "computeMaskIdx: negative size");
    }
    if (B == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!mask || !maskIdx)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "computeMaskIdx: null pointer");
    }
    hipLaunchKernelGGL(mask_idx_kernel, dim3((unsigned) ceil_div(B, kWavesPerBlock)), dim3(kBlock), 0,
        as_stream(stream), S, B, mask, maskIdx);
    return check_launch("mask_idx_kernel");
}

extern "C" int trtamd_convert_mask(uint32_t S, uint32_t B, uint32_t warps_m, uint32_t warps_n, uint32_t warps_k,
    int32_t const* inputMaskSB, uint32_t* inputMaskX, trtamd_stream_t stream)
{
    if (warps_m == 0 || warps_n == 0 || warps_k == 0 || S == 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "convertMask: zero geometry");
    }
    uint32_t const threads = warps_m * warps_n * warps_k * 32;
    uint32_t const xmmas_m = (S + 16 * warps_m - 1) / (16 * warps_m);
    uint32_t const xmmas_n = (S + 16 * warps_n - 1) / (16 * warps_n);
    if (threads > 1024 || xmmas_n > 4)
    {
        // one uint32 per thread holds 8 bits per xmma_n
        return set_error(TRTAMD_STATUS_BAD_PARAM, "convertMask: geometry does not fit a 32-bit word per thread");
    }
    if (B == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!inputMaskSB || !inputMaskX)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "convertMask: null pointer");
    }
    hipLaunchKernelGGL(convert_mask_kernel, dim3(B), dim3(threads), 0, as_stream(stream), warps_m, warps_n, S, B,
        xmmas_m, xmmas_n, inputMaskSB, inputMaskX);
    return check_launch("convert_mask_kernel");
}
