// SkipLayerNorm kernels for gfx950: residual (+bias) + LayerNorm on rows of `ld` elements.
//
// All variants are HBM-bound streams.  Common shape: one 64-lane wavefront owns whole rows (or,
// for the 32-interleaved INT8 layout, 8 adjacent tokens), keeps the row in registers between the
// statistics and the normalisation (one read, one write per element), reduces with lane shuffles
// only (no LDS, no barrier on the data path) and issues every global load of its rows before the
// first arithmetic so that several KB per wave are in flight.
//
// Replaces plugin/skipLayerNormPlugin/skipLayerNormKernel.cu,
// plugin/skipLayerNormPlugin/skipLayerNormInt8InterleavedKernelHFace.cu and
// plugin/skipLayerNormPlugin/skipLayerNormInt8InterleavedKernelMTron.cu of the reference.
#include "device_utils.hpp"
#include "host_utils.hpp"

#include <cstdlib>

namespace trtamd
{
namespace
{

constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWaveSize;

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

// ------------------------------------------------------------------------------------------
// FP32 / FP16 rows, ld a multiple of the 16-byte vector width: register-resident rows.
// The residual sum is formed in T like the reference (skipLayerNormKernel.cu:121-134);
// statistics are a Welford/Chan merge in binary32; epsilon is the caller's.
// ------------------------------------------------------------------------------------------
template <typename T, int NV, int R, bool HAS_BIAS>
__global__ __launch_bounds__(kBlock) void skipln_rows_kernel(int const ld, int64_t const rows, T const* __restrict__ in,
    T const* __restrict__ skip, T const* __restrict__ beta, T const* __restrict__ gamma, T const* __restrict__ bias,
    T* __restrict__ out, float const eps)
{
    constexpr int VPT = Vec16<T>::kN;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int64_t const wave = (int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    int64_t const row0 = wave * R;
    if (row0 >= rows)
    {
        return;
    }
    int const nvec = ld / VPT;

    Vec16<T> xin[R][NV], xsk[R][NV];
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            int const vi = lane + kWaveSize * j;
            bool const ok = vi < nvec && row0 + r < rows;
            int64_t const off = (row0 + r) * ld + (int64_t) vi * VPT;
            xin[r][j].u = ok ? *reinterpret_cast<u32x4 const*>(in + off) : u32x4{0, 0, 0, 0};
            xsk[r][j].u = ok ? *reinterpret_cast<u32x4 const*>(skip + off) : u32x4{0, 0, 0, 0};
        }
    }
    Vec16<T> g[NV], b[NV], bs[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j)
    {
        int const vi = lane + kWaveSize * j;
        bool const ok = vi < nvec;
        g[j].u = ok ? *reinterpret_cast<u32x4 const*>(gamma + vi * VPT) : u32x4{0, 0, 0, 0};
        b[j].u = ok ? *reinterpret_cast<u32x4 const*>(beta + vi * VPT) : u32x4{0, 0, 0, 0};
        if (HAS_BIAS)
        {
            bs[j].u = ok ? *reinterpret_cast<u32x4 const*>(bias + vi * VPT) : u32x4{0, 0, 0, 0};
        }
    }

    float const rld = 1.f / (float) ld;
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        if (row0 + r >= rows)
        {
            break; // wave-uniform
        }
        float v[NV][VPT];
        float sum = 0.f;
        float cnt = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            bool const ok = lane + kWaveSize * j < nvec;
#pragma unroll
            for (int k = 0; k < VPT; ++k)
            {
                T t = xin[r][j].e[k] + xsk[r][j].e[k];
                if (HAS_BIAS)
                {
                    t = t + bs[j].e[k];
                }
                v[j][k] = (float) t;
                sum += ok ? v[j][k] : 0.f;
            }
            cnt += ok ? (float) VPT : 0.f;
        }
        Welford w;
        w.n = cnt;
        w.mean = cnt > 0.f ? sum / cnt : 0.f;
        w.m2 = 0.f;
#pragma unroll
        for (int j = 0; j < NV; ++j)
        {
            bool const ok = lane + kWaveSize * j < nvec;
#pragma unroll
            for (int k = 0; k < VPT; ++k)
            {
                float const dlt = v[j][k] - w.mean;
                w.m2 += ok ? dlt * dlt : 0.f;
            }
        }
        w = group_welford<kWaveSize>(w);
        float const mu = w.mean;
        float const rsigma = rsqrtf(w.m2 * rld + eps);
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
                    y.e[k] = (T) ((float) g[j].e[k] * (v[j][k] - mu) * rsigma + (float) b[j].e[k]);
                }
                store_through_l2(out + (row0 + r) * ld + (int64_t) vi * VPT, y.u);
            }
        }
    }
}

// Any ld (odd sizes, ld <= 32, very long rows): one wave per row, three L2-resident sweeps.
template <typename T, bool HAS_BIAS>
__global__ __launch_bounds__(kBlock) void skipln_generic_kernel(int const ld, int64_t const rows,
    T const* __restrict__ in, T const* __restrict__ skip, T const* __restrict__ beta, T const* __restrict__ gamma,
    T const* __restrict__ bias, T* __restrict__ out, float const eps)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    int64_t const row = (int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (row >= rows)
    {
        return;
    }
    T const* pi = in + row * ld;
    T const* ps = skip + row * ld;
    auto value = [&](int i) -> float {
        T t = pi[i] + ps[i];
        if (HAS_BIAS)
        {
            t = t + bias[i];
        }
        return (float) t;
    };
    float sum = 0.f;
    for (int i = lane; i < ld; i += kWaveSize)
    {
        sum += value(i);
    }
    float const mu = wave_sum(sum) / (float) ld;
    float m2 = 0.f;
    for (int i = lane; i < ld; i += kWaveSize)
    {
        float const dlt = value(i) - mu;
        m2 += dlt * dlt;
    }
    float const rsigma = rsqrtf(wave_sum(m2) / (float) ld + eps);
    for (int i = lane; i < ld; i += kWaveSize)
    {
        out[row * ld + i] = (T) ((float) gamma[i] * (value(i) - mu) * rsigma + (float) beta[i]);
    }
}

template <typename T, int NV, int R>
int launch_rows(hipStream_t stream, int ld, int64_t rows, T const* in, T const* skip, T const* beta, T const* gamma,
    T const* bias, T* out, float eps)
{
    int64_t const waves = ceil_div<int64_t>(rows, R);
    dim3 const grid((unsigned) ceil_div<int64_t>(waves, kWavesPerBlock));
    if (bias)
    {
        hipLaunchKernelGGL((skipln_rows_kernel<T, NV, R, true>), grid, dim3(kBlock), 0, stream, ld, rows, in, skip, beta,
            gamma, bias, out, eps);
    }
    else
    {
        hipLaunchKernelGGL((skipln_rows_kernel<T, NV, R, false>), grid, dim3(kBlock), 0, stream, ld, rows, in, skip,
            beta, gamma, bias, out, eps);
    }
    return check_launch("skipln_rows_kernel");
}

template <typename T>
int skip_layer_norm(hipStream_t stream, int32_t ld, int64_t n, T const* in, T const* skip, T const* beta,
    T const* gamma, T* out, T const* bias, float epsT)
{
    if (ld <= 0 || n < 0 || n % ld != 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNorm: n (%lld) must be a multiple of ld (%d)",
            (long long) n, ld);
    }
    if (n == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!in || !skip || !beta || !gamma || !out)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNorm: null tensor pointer");
    }
    int64_t const rows = n / ld;
    // The reference adds numeric_limits<T>::epsilon() only in its vectorised kernel, which it
    // selects for ld in {768,1024} (skipLayerNormKernel.cu:267-276, 149).
    float const eps = (ld == 768 || ld == 1024) ? epsT : 0.f;
    constexpr int VPT = 16 / (int) sizeof(T);
    bool const vec_ok = ld % VPT == 0 && ld > 32 && aligned16(in) && aligned16(skip) && aligned16(out)
        && aligned16(beta) && aligned16(gamma) && (!bias || aligned16(bias));
    int const nv = vec_ok ? ceil_div(ld / VPT, kWaveSize) : 0;
    if (vec_ok && nv == 1)
    {
        return launch_rows<T, 1, 4>(stream, ld, rows, in, skip, beta, gamma, bias, out, eps);
    }
    if (vec_ok && nv == 2)
    {
        return launch_rows<T, 2, 2>(stream, ld, rows, in, skip, beta, gamma, bias, out, eps);
    }
    if (vec_ok && nv <= 4)
    {
        return launch_rows<T, 4, 1>(stream, ld, rows, in, skip, beta, gamma, bias, out, eps);
    }
    if (vec_ok && nv <= 8)
    {
        return launch_rows<T, 8, 1>(stream, ld, rows, in, skip, beta, gamma, bias, out, eps);
    }
    dim3 const grid((unsigned) ceil_div<int64_t>(rows, kWavesPerBlock));
    if (bias)
    {
        hipLaunchKernelGGL((skipln_generic_kernel<T, true>), grid, dim3(kBlock), 0, stream, ld, rows, in, skip, beta,
            gamma, bias, out, eps);
    }
    else
    {
        hipLaunchKernelGGL((skipln_generic_kernel<T, false>), grid, dim3(kBlock), 0, stream, ld, rows, in, skip, beta,
            gamma, bias, out, eps);
    }
    return check_launch("skipln_generic_kernel");
}

// ------------------------------------------------------------------------------------------
// INT8 rows, linear layout (skiplnDQQ, skipLayerNormKernel.cu:43-106): each lane owns 16
// consecutive channels of a row, a wave owns R rows.  v = dqIn*in + dqSkip*skip (+bias),
// epsilon 2^-10, out = sat8(rne(y * qScale)).  The statistics are exact: integer dot products of
// the bytes (v_dot4_i32_i8) summed over the wave, the bias terms as binary32 dot products, all
// combined in binary64.  gamma*qScale and beta*qScale of the lane's 16 channels stay in registers
// for all rows.  A signed byte becomes binary32 in one instruction (v_cvt_f32_i32 with a sign-extending
// byte select); a result becomes a byte in one more: v_cvt_pk_u8_f32 rounds to nearest even, saturates to
// [0, 255] and places the byte, so 128 is folded into beta and one XOR per dword returns to two's
// complement.  Loads are ordinary ones and stores write through the L2 (not non-temporal): in a network the
// tensors were just written by the layer before and are read by the layer after, and the last-level cache
// keeps them in between.
// ------------------------------------------------------------------------------------------
template <int R, bool HAS_BIAS>
__global__ __launch_bounds__(kBlock) void skipln_dqq_kernel(int const ld, int64_t const rows,
    int8_t const* __restrict__ in, int8_t const* __restrict__ skip, f16 const* __restrict__ beta,
    f16 const* __restrict__ gamma, f16 const* __restrict__ bias, int8_t* __restrict__ out, float const dqIn,
    float const dqSkip, float const qScale)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    int64_t const wave = (int64_t) blockIdx.x * kWavesPerBlock + (threadIdx.x >> 6);
    int64_t const row0 = wave * R;
    if (row0 >= rows)
    {
        return;
    }
    bool const lane_ok = lane * 16 < ld;
    int const ch = lane_ok ? lane * 16 : 0;
    u32x4 xi[R], xs[R];
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        // rows past the end re-read the last row (and store nothing); idle lanes contribute zeros
        int64_t const row = min(row0 + r, rows - 1);
        int64_t const off = row * ld + ch;
        xi[r] = *reinterpret_cast<u32x4 const*>(in + off);
        xs[r] = *reinterpret_cast<u32x4 const*>(skip + off);
        if (!lane_ok)
        {
            xi[r] = u32x4{0, 0, 0, 0};
            xs[r] = u32x4{0, 0, 0, 0};
        }
    }
    float gq[16], bq[16], bs[16];
    float biasSum = 0.f, biasSq = 0.f;
#pragma unroll
    for (int h = 0; h < 2; ++h)
    {
        Vec16<f16> g, b, c;
        g.u = *reinterpret_cast<u32x4 const*>(gamma + ch + h * 8);
        b.u = *reinterpret_cast<u32x4 const*>(beta + ch + h * 8);
        if (HAS_BIAS)
        {
            c.u = *reinterpret_cast<u32x4 const*>(bias + ch + h * 8);
        }
#pragma unroll
        for (int k = 0; k < 8; ++k)
        {
            gq[h * 8 + k] = (float) g.e[k] * qScale;
            bq[h * 8 + k] = (float) b.e[k] * qScale + 128.f; // results are formed as unsigned bytes
            if (HAS_BIAS)
            {
                float const v = lane_ok ? (float) c.e[k] : 0.f;
                bs[h * 8 + k] = v;
                biasSum += v;
                biasSq += v * v;
            }
        }
    }
    if (HAS_BIAS)
    {
        biasSum = wave_sum(biasSum);
        biasSq = wave_sum(biasSq);
    }
    double const dIn = (double) dqIn, dSk = (double) dqSkip;
    double const rld = 1.0 / (double) ld;
#pragma unroll
    for (int r = 0; r < R; ++r)
    {
        int sIn = 0, sSk = 0, sII = 0, sIS = 0, sSS = 0;
        float dotIn = 0.f, dotSk = 0.f; // sum bias*in, sum bias*skip
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            sIn = __builtin_amdgcn_sdot4((int) xi[r][q], 0x01010101, sIn, false);
            sSk = __builtin_amdgcn_sdot4((int) xs[r][q], 0x01010101, sSk, false);
            sII = __builtin_amdgcn_sdot4((int) xi[r][q], (int) xi[r][q], sII, false);
            sIS = __builtin_amdgcn_sdot4((int) xi[r][q], (int) xs[r][q], sIS, false);
            sSS = __builtin_amdgcn_sdot4((int) xs[r][q], (int) xs[r][q], sSS, false);
            if (HAS_BIAS)
            {
#pragma unroll
                for (int k = 0; k < 4; ++k)
                {
                    dotIn = fmaf(i8_to_f32(xi[r][q], k), bs[q * 4 + k], dotIn);
                    dotSk = fmaf(i8_to_f32(xs[r][q], k), bs[q * 4 + k], dotSk);
                }
            }
        }
        sIn = wave_sum_i32(sIn);
        sSk = wave_sum_i32(sSk);
        sII = wave_sum_i32(sII);
        sIS = wave_sum_i32(sIS);
        sSS = wave_sum_i32(sSS);
        double sum1 = dIn * sIn + dSk * sSk;
        double sum2 = dIn * dIn * sII + 2.0 * dIn * dSk * sIS + dSk * dSk * sSS;
        if (HAS_BIAS)
        {
            dotIn = wave_sum(dotIn);
            dotSk = wave_sum(dotSk);
            sum1 += (double) biasSum;
            sum2 += 2.0 * (dIn * (double) dotIn + dSk * (double) dotSk) + (double) biasSq;
        }
        double const mean = sum1 * rld;
        float const var = (float) (sum2 * rld - mean * mean);
        float const rsigma = rsqrtf(fmaxf(var, 0.f) + 0.0009765625f);
        float const a1 = dqIn * rsigma;
        float const a2 = dqSkip * rsigma;
        float const c1 = (float) (-mean * (double) rsigma);
        u32x4 o;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            uint32_t yw = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                float const fa = i8_to_f32(xi[r][q], k);
                float const fs = i8_to_f32(xs[r][q], k);
                float const c = HAS_BIAS ? fmaf(bs[q * 4 + k], rsigma, c1) : c1;
                float const nrm = fmaf(fa, a1, fmaf(fs, a2, c));
                yw = __builtin_amdgcn_cvt_pk_u8_f32(fmaf(gq[q * 4 + k], nrm, bq[q * 4 + k]), k, yw);
            }
            o[q] = yw ^ 0x80808080u;
        }
        if (lane_ok && row0 + r < rows)
        {
            store_through_l2(out + (row0 + r) * ld + ch, o);
        }
    }
}

// ------------------------------------------------------------------------------------------
// INT8, 32-interleaved layout [ld/32][total][32] (TensorFormat::kCHW32 of a [1,ld,total,1]
// tensor).  A wave owns 8 adjacent tokens: lane = (sub, tok, half) with sub = lane/16 selecting
// one of 4 channel groups per step, tok = (lane%16)/2, half = lane%2 selecting 16 of the group's
// 32 channels.  One 16-byte load per lane therefore covers 4 channel groups x 256 contiguous
// bytes.  Statistics come from exact integer dot products (sum in, sum skip, sum in^2, sum
// in*skip, sum skip^2) combined in binary64, so mean and variance carry no accumulation error.
// gamma*qScale and beta*qScale are staged once per workgroup in LDS as binary32.
// ------------------------------------------------------------------------------------------
// Which block of TOK consecutive tokens a workgroup takes.  Workgroup ids are dealt round-robin to the 8 XCDs, each
// with an L2 of its own, and neighbouring token blocks touch the same cache lines at their common border in all 32
// channel groups whenever a group's rows do not start on a line (32 bytes per token: any token count that is not a
// multiple of 4): in id order both neighbours fetch those lines from memory and write them back in halves.  Runs of 64
// consecutive blocks therefore go to one XCD (ids 512 m + 8 r + x -> block 512 m + 64 x + r), and what is left
// behind the last whole span of 512 is dealt the same way in shorter runs.  Measured at 33289 tokens x 1024 channels:
// 19.5 -> 17.8 us with the tensors in the last-level cache, unchanged from memory (longer runs, up to one run per
// XCD, lose 3 % there); 65536 tokens, whose group stride is a power of two, 52.9 -> 31.5 us.
__device__ inline uint32_t token_block_of_workgroup(uint32_t bid, uint32_t nblocks)
{
    constexpr uint32_t kXcds = 8, kRun = 64, kSpan = kXcds * kRun;
    uint32_t const first = bid / kSpan * kSpan; // first id of this workgroup's span
    uint32_t const x = bid - first;
    uint32_t const run = first + kSpan <= nblocks ? kRun : (nblocks - first) / kXcds;
    if (x >= run * kXcds)
    {
        return bid; // the last few ids of a short span keep their blocks
    }
    return first + (x % kXcds) * run + x / kXcds;
}

template <int G, int W, int TOK, bool PRELN, bool TAIL>
__global__ __launch_bounds__(W * kWaveSize) void skipln_interleaved_kernel(int const total,
    int8_t const* __restrict__ in, int8_t const* __restrict__ skip, f16 const* __restrict__ beta,
    f16 const* __restrict__ gamma, int8_t* __restrict__ out, int8_t* __restrict__ preln, float const dqIn,
    float const dqSkip, float const qScale, float const qSkipScale, float const eps, float const prelnMin)
{
    // A workgroup of W wavefronts owns TOK consecutive tokens.  Lane = (sub, token, half): one load
    // instruction of a wavefront reads SUBS channel groups x TOK tokens x 32 bytes, TOK*32 contiguous
    // bytes per group; the W wavefronts take interleaved sets of SUBS groups, NI sets each.
    constexpr int LD = G * 32;
    constexpr int THREADS = W * kWaveSize;
    constexpr int LPG = TOK * 2;               // lanes per channel group
    constexpr int SUBS = kWaveSize / LPG;      // channel groups per load instruction
    constexpr int NI = G / (SUBS * W);
    static_assert(G % (SUBS * W) == 0 && NI <= 8, "every lane keeps its part of the row in registers");
    __shared__ float sGamma[LD];
    __shared__ float sBeta[LD];
    __shared__ int sStat[W][TOK][5];

    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const sub = lane / LPG;
    int const tok = (lane % LPG) >> 1;
    int const hf = lane & 1;
    uint32_t const block = token_block_of_workgroup(blockIdx.x, gridDim.x);
    int64_t const tRaw = (int64_t) block * TOK + tok;
    bool const valid = tRaw < total;
    // lanes past the last token re-read the last token (and store nothing): no divergent loads
    int64_t const t = valid ? tRaw : (int64_t) total - 1;
    int64_t const groupStride = (int64_t) total * 32;
    int const g0 = wave * SUBS + sub;               // first channel group of this lane; then += SUBS*W
    int64_t const base = (int64_t) g0 * groupStride + t * 32 + hf * 16;
    constexpr int64_t kStep = SUBS * W;

    u32x4 xi[NI], xs[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i)
    {
        xi[i] = *reinterpret_cast<u32x4 const*>(in + base + i * kStep * groupStride);
        xs[i] = *reinterpret_cast<u32x4 const*>(skip + base + i * kStep * groupStride);
    }
    // TAIL: a launch of fewer workgroups than token blocks (launch_interleaved: token counts just above one round of
    // resident workgroups) leaves tokens behind the last block, and workgroup b also takes token gridDim.x * TOK + b.
    // Its first wavefront requests that token's two rows now, straight into LDS (lane = channel group x half; no
    // vector registers held), and normalises it after the block.
    constexpr int kExtraLoads = (G + 31) / 32; // load instructions per tensor: 32 channel groups x 2 halves each
    __shared__ __attribute__((aligned(16))) uint8_t sExtra[2][TAIL ? kExtraLoads * 1024 : 16];
    int64_t const extraTok = (int64_t) gridDim.x * TOK + block;
    bool const hasExtra = TAIL && extraTok < total; // the same for every lane of the workgroup
    if (TAIL && hasExtra && wave == 0)
    {
#pragma unroll
        for (int e = 0; e < kExtraLoads; ++e)
        {
            int const grp = e * 32 + (lane >> 1);
            if (grp < G)
            {
                int64_t const off = (int64_t) grp * groupStride + extraTok * 32 + hf * 16;
                load_to_lds16(in + off, (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) sExtra[0] + e * 1024);
                load_to_lds16(skip + off, (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) sExtra[1] + e * 1024);
            }
        }
    }
    // gamma/beta are staged after the tensor loads were issued, so their latency overlaps
    for (int i = threadIdx.x; i < LD; i += THREADS)
    {
        sGamma[i] = (float) gamma[i] * qScale;
        sBeta[i] = (float) beta[i] * qScale + 128.f; // results are formed as unsigned bytes
    }
    int sIn = 0, sSk = 0, sII = 0, sIS = 0, sSS = 0;
#pragma unroll
    for (int i = 0; i < NI; ++i)
    {
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            sIn = __builtin_amdgcn_sdot4((int) xi[i][q], 0x01010101, sIn, false);
            sSk = __builtin_amdgcn_sdot4((int) xs[i][q], 0x01010101, sSk, false);
            sII = __builtin_amdgcn_sdot4((int) xi[i][q], (int) xi[i][q], sII, false);
            sIS = __builtin_amdgcn_sdot4((int) xi[i][q], (int) xs[i][q], sIS, false);
            sSS = __builtin_amdgcn_sdot4((int) xs[i][q], (int) xs[i][q], sSS, false);
        }
    }
    // the lanes of a token differ in bit 0 (half) and in the sub bits above the token bits
    {
        auto const add = [](int x, int y) { return x + y; };
        auto const over_token = [&](int v) {
            v = reduce_step<1>(v, add);
            if constexpr (LPG <= 16)
            {
                v = reduce_step<16>(v, add);
            }
            if constexpr (LPG <= 32)
            {
                v = reduce_step<32>(v, add);
            }
            return v;
        };
        sIn = over_token(sIn);
        sSk = over_token(sSk);
        sII = over_token(sII);
        sIS = over_token(sIS);
        sSS = over_token(sSS);
    }
    if (W > 1)
    {
        if (sub == 0 && hf == 0)
        {
            sStat[wave][tok][0] = sIn;
            sStat[wave][tok][1] = sSk;
            sStat[wave][tok][2] = sII;
            sStat[wave][tok][3] = sIS;
            sStat[wave][tok][4] = sSS;
        }
    }
    if (TAIL && hasExtra && wave == 0)
    {
        // the block's rows have arrived (the statistics above consumed them), and so have the extra token's, requested
        // right behind them: this wait makes that explicit for loads the compiler does not see, and costs nothing here
        wait_vmcnt<0>();
    }
    __syncthreads();
    if (W > 1)
    {
        sIn = sSk = sII = sIS = sSS = 0;
#pragma unroll
        for (int w = 0; w < W; ++w)
        {
            sIn += sStat[w][tok][0];
            sSk += sStat[w][tok][1];
            sII += sStat[w][tok][2];
            sIS += sStat[w][tok][3];
            sSS += sStat[w][tok][4];
        }
    }
    double const dIn = (double) dqIn, dSk = (double) dqSkip;
    double const mean = (dIn * sIn + dSk * sSk) * (1.0 / LD);
    double const ex2 = (dIn * dIn * sII + 2.0 * dIn * dSk * sIS + dSk * dSk * sSS) * (1.0 / LD);
    float const var = (float) (ex2 - mean * mean);
    float const rsigma = rsqrtf(fmaxf(var, 0.f) + eps);
    // A signed byte becomes binary32 in one instruction (v_cvt_f32_i32 with a sign-extending byte select).  Results
    // are produced as unsigned bytes: v_cvt_pk_u8_f32 rounds to nearest even, saturates to [0, 255] and places the
    // byte, so with 128 folded into the additive term one instruction does the rounding, the clamp to [-128, 127]
    // and the packing, and one XOR per dword returns to two's complement.
    float const a1 = dqIn * rsigma;
    float const a2 = dqSkip * rsigma;
    float const c1 = (float) (-mean * (double) rsigma);
    float const p1 = dqIn * qSkipScale;
    float const p2 = dqSkip * qSkipScale;
    float const pc = 128.f;
    float const prelnLo = prelnMin + 128.f;

#pragma unroll
    for (int i = 0; i < NI; ++i)
    {
        u32x4 const a = xi[i], s = xs[i];
        int const ch = (g0 + i * (int) kStep) * 32 + hf * 16;
        u32x4 o, po;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            f32x4 const gq = *reinterpret_cast<f32x4 const*>(&sGamma[ch + q * 4]);
            f32x4 const bq = *reinterpret_cast<f32x4 const*>(&sBeta[ch + q * 4]);
            uint32_t yw = 0, pw = 0;
#pragma unroll
            for (int k = 0; k < 4; ++k)
            {
                float const fa = i8_to_f32(a[q], k);
                float const fs = i8_to_f32(s[q], k);
                float const nrm = fmaf(fa, a1, fmaf(fs, a2, c1));
                yw = __builtin_amdgcn_cvt_pk_u8_f32(fmaf(gq[k], nrm, bq[k]), k, yw);
                if (PRELN)
                {
                    float const pv = fmaf(fa, p1, fmaf(fs, p2, pc));
                    pw = __builtin_amdgcn_cvt_pk_u8_f32(fmaxf(pv, prelnLo), k, pw);
                }
            }
            o[q] = yw ^ 0x80808080u;
            if (PRELN)
            {
                po[q] = pw ^ 0x80808080u;
            }
        }
        if (valid)
        {
            store_through_l2(out + base + i * kStep * groupStride, o);
            if (PRELN)
            {
                store_through_l2(preln + base + i * kStep * groupStride, po);
            }
        }
    }
    if constexpr (TAIL)
    if (hasExtra && wave == 0)
    {
        // The extra token, once the block's registers are free: its rows have been in LDS since before the barrier.
        // Lane = (channel group, half) as it loaded; the whole wavefront is one token.
        int eIn = 0, eSk = 0, eII = 0, eIS = 0, eSS = 0;
        u32x4 ea[kExtraLoads], es[kExtraLoads];
#pragma unroll
        for (int e = 0; e < kExtraLoads; ++e)
        {
            bool const live = e * 32 + (lane >> 1) < G;
            ea[e] = live ? *reinterpret_cast<u32x4 const*>(sExtra[0] + e * 1024 + lane * 16) : u32x4{0, 0, 0, 0};
            es[e] = live ? *reinterpret_cast<u32x4 const*>(sExtra[1] + e * 1024 + lane * 16) : u32x4{0, 0, 0, 0};
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                eIn = __builtin_amdgcn_sdot4((int) ea[e][q], 0x01010101, eIn, false);
                eSk = __builtin_amdgcn_sdot4((int) es[e][q], 0x01010101, eSk, false);
                eII = __builtin_amdgcn_sdot4((int) ea[e][q], (int) ea[e][q], eII, false);
                eIS = __builtin_amdgcn_sdot4((int) ea[e][q], (int) es[e][q], eIS, false);
                eSS = __builtin_amdgcn_sdot4((int) es[e][q], (int) es[e][q], eSS, false);
            }
        }
        eIn = wave_sum_i32(eIn);
        eSk = wave_sum_i32(eSk);
        eII = wave_sum_i32(eII);
        eIS = wave_sum_i32(eIS);
        eSS = wave_sum_i32(eSS);
        // the two scales converted again from copies the compiler takes as new: kept from the block's statistics,
        // the binary64 values would hold four vector registers through the block's arithmetic and cost the kernel a
        // resident workgroup per CU
        float dqI = dqIn, dqS = dqSkip;
        asm volatile("" : "+s"(dqI), "+s"(dqS));
        double const xIn = (double) dqI, xSk = (double) dqS;
        double const eMean = (xIn * eIn + xSk * eSk) * (1.0 / LD);
        double const eEx2 = (xIn * xIn * eII + 2.0 * xIn * xSk * eIS + xSk * xSk * eSS) * (1.0 / LD);
        float const eRsigma = rsqrtf(fmaxf((float) (eEx2 - eMean * eMean), 0.f) + eps);
        float const e1 = dqI * eRsigma;
        float const e2 = dqS * eRsigma;
        float const ec = (float) (-eMean * (double) eRsigma);
#pragma unroll
        for (int e = 0; e < kExtraLoads; ++e)
        {
            int const grp = e * 32 + (lane >> 1);
            int const ch = grp * 32 + hf * 16;
            u32x4 o, po;
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                uint32_t yw = 0, pw = 0;
#pragma unroll
                for (int k = 0; k < 4; ++k)
                {
                    float const fa = i8_to_f32(ea[e][q], k);
                    float const fs = i8_to_f32(es[e][q], k);
                    float const nrm = fmaf(fa, e1, fmaf(fs, e2, ec));
                    int const c = grp < G ? ch + q * 4 + k : 0;
                    yw = __builtin_amdgcn_cvt_pk_u8_f32(fmaf(sGamma[c], nrm, sBeta[c]), k, yw);
                    if (PRELN)
                    {
                        float const pv = fmaf(fa, p1, fmaf(fs, p2, pc));
                        pw = __builtin_amdgcn_cvt_pk_u8_f32(fmaxf(pv, prelnLo), k, pw);
                    }
                }
                o[q] = yw ^ 0x80808080u;
                if (PRELN)
                {
                    po[q] = pw ^ 0x80808080u;
                }
            }
            if (grp < G)
            {
                int64_t const off = (int64_t) grp * groupStride + extraTok * 32 + hf * 16;
                store_through_l2(out + off, o);
                if (PRELN)
                {
                    store_through_l2(preln + off, po);
                }
            }
        }
    }
}

// Workgroups of this kernel that the current device holds at once (asked once per process and kernel; 0 when it
// cannot be asked).
template <int G, int W, int TOK, bool PRELN, bool TAIL>
int resident_workgroups()
{
    static int const n = [] {
        int perCu = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(
                &perCu, skipln_interleaved_kernel<G, W, TOK, PRELN, TAIL>, W * kWaveSize, 0)
                != hipSuccess
            || perCu <= 0)
        {
            (void) hipGetLastError();
            return 0;
        }
        return perCu * num_cus();
    }();
    return n;
}

template <int G, int W, int TOK, bool PRELN>
int launch_interleaved_as(hipStream_t stream, int32_t total, int8_t const* in, int8_t const* skip, f16 const* beta,
    f16 const* gamma, int8_t* out, int8_t* preln, float dqIn, float dqSkip, float qScale, float qSkipScale, float eps,
    float prelnMin)
{
    // One workgroup per block of TOK tokens.  When that is a few workgroups more than the chip holds at once, the
    // stragglers of a second round cost 1.4-1.7 us whatever their number (33280 tokens x 1024 channels: 18.7 us where
    // 32736 tokens take 17.0), so when one token more per workgroup lets a single round cover the tensor the launch is
    // that round, with the kernel's tail path.
    int const blocks = ceil_div(total, TOK);
    dim3 const block(W * kWaveSize);
    int const residentPlain = resident_workgroups<G, W, TOK, PRELN, false>();
    int const residentTail = resident_workgroups<G, W, TOK, PRELN, true>();
    if (residentPlain > 0 && blocks > residentPlain && residentTail > 0 && residentTail < blocks
        && (int64_t) residentTail * (TOK + 1) >= total)
    {
        hipLaunchKernelGGL((skipln_interleaved_kernel<G, W, TOK, PRELN, true>), dim3((unsigned) residentTail), block, 0,
            stream, total, in, skip, beta, gamma, out, preln, dqIn, dqSkip, qScale, qSkipScale, eps, prelnMin);
    }
    else
    {
        hipLaunchKernelGGL((skipln_interleaved_kernel<G, W, TOK, PRELN, false>), dim3((unsigned) blocks), block, 0, stream,
            total, in, skip, beta, gamma, out, preln, dqIn, dqSkip, qScale, qSkipScale, eps, prelnMin);
    }
    return check_launch("skipln_interleaved_kernel");
}

template <int G, int W, int TOK>
int launch_interleaved(hipStream_t stream, int32_t total, int8_t const* in, int8_t const* skip, f16 const* beta,
    f16 const* gamma, int8_t* out, int8_t* preln, float dqIn, float dqSkip, float qScale, float qSkipScale, float eps,
    float prelnMin)
{
    return preln ? launch_interleaved_as<G, W, TOK, true>(stream, total, in, skip, beta, gamma, out, preln, dqIn, dqSkip,
               qScale, qSkipScale, eps, prelnMin)
                 : launch_interleaved_as<G, W, TOK, false>(stream, total, in, skip, beta, gamma, out, preln, dqIn, dqSkip,
                     qScale, qSkipScale, eps, prelnMin);
}

// small: epsilon = binary16 epsilon, preln clipped to +-127; large: binary32 epsilon, preln
// saturated to [-128,127].  maxLdSet: which ld values the reference launcher accepts.
int skipln_interleaved(hipStream_t stream, bool large, bool mtron, int32_t ld, int32_t total, int8_t const* in,
    int8_t const* skip, f16 const* beta, f16 const* gamma, int8_t* out, int8_t* preln, float dqIn, float dqSkip,
    float qScale, float qSkipScale)
{
    bool const base_ok = ld == 768 || ld == 1024;
    bool const wide_ok = !large && mtron && (ld == 1536 || ld == 2048 || ld == 3072 || ld == 4096);
    if (!base_ok && !wide_ok)
    {
        return set_error(TRTAMD_STATUS_FAILURE, "SkipLayerNormDQQ - FATAL: unsupported hidden layer size: %d", ld);
    }
    if (total < 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNorm interleaved: negative token count");
    }
    if (total == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!in || !skip || !beta || !gamma || !out || (mtron && !preln))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNorm interleaved: null tensor pointer");
    }
    if (!aligned16(in) || !aligned16(skip) || !aligned16(out) || (mtron && !aligned16(preln)))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNorm interleaved: tensors must be 16-byte aligned");
    }
    float const eps = large ? 1.1920928955078125e-07f : 0.0009765625f;
    float const pmin = large ? -128.f : -127.f;
    int8_t* pre = mtron ? preln : nullptr;
    // 32 tokens per workgroup and enough wavefronts that a lane keeps at most 8 x 16 bytes per tensor; other
    // splits (8 or 16 tokens, 2 to 16 wavefronts) measured the same or slower at 4 k to 33 k tokens
#define TRTAMD_IL(G, W, TOK)                                                                                          \
    return launch_interleaved<G, W, TOK>(stream, total, in, skip, beta, gamma, out, pre, dqIn, dqSkip, qScale,         \
        qSkipScale, eps, pmin)
    switch (ld)
    {
    case 768:
        TRTAMD_IL(24, 6, 32);
    case 1024:
        TRTAMD_IL(32, 8, 32);
    case 1536: TRTAMD_IL(48, 8, 32);
    case 2048: TRTAMD_IL(64, 8, 32);
    case 3072: TRTAMD_IL(96, 16, 32);
    default: TRTAMD_IL(128, 16, 32);
    }
#undef TRTAMD_IL
}

} // namespace
} // namespace trtamd

using namespace trtamd;

extern "C" int trtamd_skip_layer_norm_fp32(trtamd_stream_t stream, int32_t ld, int64_t n, float const* input,
    float const* skip, float const* beta, float const* gamma, float* output, float const* bias)
{
    return skip_layer_norm<float>(as_stream(stream), ld, n, input, skip, beta, gamma, output, bias,
        1.1920928955078125e-07f);
}

extern "C" int trtamd_skip_layer_norm_fp16(trtamd_stream_t stream, int32_t ld, int64_t n, trtamd_half_t const* input,
    trtamd_half_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, trtamd_half_t* output,
    trtamd_half_t const* bias)
{
    return skip_layer_norm<f16>(as_stream(stream), ld, n, reinterpret_cast<f16 const*>(input),
        reinterpret_cast<f16 const*>(skip), reinterpret_cast<f16 const*>(beta), reinterpret_cast<f16 const*>(gamma),
        reinterpret_cast<f16*>(output), reinterpret_cast<f16 const*>(bias), 0.0009765625f);
}

extern "C" int trtamd_skip_layer_norm_dqq(trtamd_stream_t stream, int32_t ld, int64_t n, int8_t const* input,
    int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    trtamd_half_t const* bias, float dqScaleIn, float dqScaleSkip, float qScale)
{
    if (ld <= 0 || n < 0 || n % ld != 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNormDQQ: n (%lld) must be a multiple of ld (%d)",
            (long long) n, ld);
    }
    if (ld != 768 && ld != 1024)
    {
        return set_error(TRTAMD_STATUS_FAILURE, "SkipLayerNormDQQ - FATAL: unsupported hidden layer size: %d", ld);
    }
    if (n == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!input || !skip || !beta || !gamma || !output)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNormDQQ: null tensor pointer");
    }
    if (!aligned16(input) || !aligned16(skip) || !aligned16(output) || !aligned16(beta) || !aligned16(gamma)
        || (bias && !aligned16(bias)))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "SkipLayerNormDQQ: tensors must be 16-byte aligned");
    }
    constexpr int R = 4;
    int64_t const rows = n / ld;
    dim3 const grid((unsigned) ceil_div<int64_t>(ceil_div<int64_t>(rows, R), kWavesPerBlock));
    auto const* b = reinterpret_cast<f16 const*>(beta);
    auto const* g = reinterpret_cast<f16 const*>(gamma);
    auto const* bs = reinterpret_cast<f16 const*>(bias);
    if (bias)
    {
        hipLaunchKernelGGL((skipln_dqq_kernel<R, true>), grid, dim3(kBlock), 0, as_stream(stream), ld, rows, input,
            skip, b, g, bs, output, dqScaleIn, dqScaleSkip, qScale);
    }
    else
    {
        hipLaunchKernelGGL((skipln_dqq_kernel<R, false>), grid, dim3(kBlock), 0, as_stream(stream), ld, rows, input,
            skip, b, g, bs, output, dqScaleIn, dqScaleSkip, qScale);
    }
    return check_launch("skipln_dqq_kernel");
}

extern "C" int trtamd_skipln_interleaved_small_hface(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    float dqScaleIn, float dqScaleSkip, float qScale)
{
    return skipln_interleaved(as_stream(stream), false, false, ld, total, input, skip,
        reinterpret_cast<f16 const*>(beta), reinterpret_cast<f16 const*>(gamma), output, nullptr, dqScaleIn,
        dqScaleSkip, qScale, 0.f);
}

extern "C" int trtamd_skipln_interleaved_large_hface(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    float dqScaleIn, float dqScaleSkip, float qScale)
{
    return skipln_interleaved(as_stream(stream), true, false, ld, total, input, skip,
        reinterpret_cast<f16 const*>(beta), reinterpret_cast<f16 const*>(gamma), output, nullptr, dqScaleIn,
        dqScaleSkip, qScale, 0.f);
}

extern "C" int trtamd_skipln_interleaved_small_mtron(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    int8_t* preln, float dqScaleIn, float dqScaleSkip, float qScale, float qSkipScale)
{
    return skipln_interleaved(as_stream(stream), false, true, ld, total, input, skip,
        reinterpret_cast<f16 const*>(beta), reinterpret_cast<f16 const*>(gamma), output, preln, dqScaleIn, dqScaleSkip,
        qScale, qSkipScale);
}

extern "C" int trtamd_skipln_interleaved_large_mtron(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    int8_t* preln, float dqScaleIn, float dqScaleSkip, float qScale, float qSkipScale)
{
    return skipln_interleaved(as_stream(stream), true, true, ld, total, input, skip,
        reinterpret_cast<f16 const*>(beta), reinterpret_cast<f16 const*>(gamma), output, preln, dqScaleIn, dqScaleSkip,
        qScale, qSkipScale);
}
