// Fused multi-head attention for gfx950 (head size 64, sequence length <= 512), INT8 and FP16.
//
// Stands in for the precompiled fused_multihead_attention / fused_multihead_attention_v2 kernels
// the reference loads from cubins (plugin/bertQKVToContextPlugin/fused_multihead_attention*/):
// one launch computes softmax(Q K^T * scale) V for every (sequence, head).
//
// Work split: a workgroup of 4 wavefronts owns 64 query rows of one (sequence, head); each wave
// owns 16 of them and never talks to the others after the K/V tiles are staged.
//   1. K is staged in LDS row-major (rows padded by 16 bytes so 16-byte reads of consecutive
//      keys fall in different banks), V is staged transposed, [d][key], with the keys of each
//      64-key block permuted into the order in which the MFMA accumulator of step 2 holds them.
//   2. S^T = K Q^T with v_mfma_i32_16x16x64_i8 (v_mfma_f32_16x16x32_f16 for FP16): the
//      accumulator layout gives every lane 4 keys x 1 query per 16-key tile, which is exactly
//      the B-operand layout of step 4, so probabilities never leave registers.
//   3. Row softmax over the whole row (<= 512 keys) held in registers: max/sum need only two
//      cross-lane steps (the 4 lane groups that share a query).  INT8 accumulators are seeded
//      with the bit pattern of 1.5*2^23 so the integer result reads directly as a binary32
//      number (no int->float conversion); probabilities are quantised with one fused
//      multiply-add against the same constant (round-to-nearest-even lands in the low byte).
//   4. O^T = V^T P^T with the same MFMA, requantised (INT8) or normalised (FP16) on store.
// Queries beyond the sequence length are neither computed nor written.
#include "device_utils.hpp"
#include "host_utils.hpp"

#include <cstring>
#include <mutex>
#include <vector>

namespace trtamd
{
namespace
{

constexpr int kQPerWave = 16;
constexpr int kWavesI8 = 4;  // 64 query rows per workgroup
constexpr int kWavesF16 = 8; // 128 query rows per workgroup: FP16 K/V tiles take twice the LDS
constexpr int kHeadSize = 64;
constexpr int kMagicBits = 0x4B400000;         // bit pattern of 12582912.f = 1.5 * 2^23
constexpr float kMagic = 12582912.f;
constexpr int kMaskedBits = 0x4B000000;        // below every reachable biased accumulator
constexpr float kLog2e = 1.4426950408889634f;

struct FmhaArgs
{
    void const* qkv;
    void* out;
    int32_t const* cuSeqlens;    // var-seqlen: [B+1]; nullptr = fixed layout
    uint32_t const* packedMask;  // fixed layout: packed key mask or nullptr (all keys valid)
    int64_t tokStrideIn;         // bytes between consecutive tokens of one sequence
    int64_t tokStrideOut;
    int64_t seqStrideIn;         // fixed layout: bytes between sequences (b -> b+1)
    int64_t seqStrideOut;
    int64_t maskStrideWords;
    int32_t B, N, S;
    int32_t qTiles;              // ceil(S / query rows per workgroup)
    int32_t total;               // interleaved: total token count
    int32_t warpsM, warpsN;      // geometry of the packed mask
    float c;                     // scale_bmm1 * log2(e)
    float scaleSoftmax;
    float scaleBmm2;
    int32_t clampP;              // scale_softmax may push p beyond 127
    int32_t* dbgAcc1;            // optional [B][N][S][S] int32 (INT8) / float bits (FP16)
    int8_t* dbgP8;               // optional [B][N][S][S]
};

template <int ESIZE>
struct Lds
{
    // K rows of 64 elements padded by 16 bytes; V^T rows of (keys + pad) elements
    static constexpr int kKRow = kHeadSize * ESIZE + 16;
    static __host__ __device__ constexpr int vtRow(int kt)
    {
        return kt * 64 * ESIZE + 16;
    }
    static __host__ __device__ constexpr int kBytes(int kt)
    {
        return kt * 64 * kKRow;
    }
    static __host__ __device__ constexpr int total(int kt)
    {
        return kBytes(kt) + kHeadSize * vtRow(kt) + 16 * 4;
    }
};

// Position, inside its 64-key block, at which key kk is stored in a V^T row.  The accumulator of
// S^T gives lane group g the keys 16u + 4g + j (u = 16-key tile, j = 0..3) and the P^T operand is
// built from it without moving data, so V^T must present keys in that order:
//   INT8 (one MFMA per 64 keys, 16 slots per lane group): slot 4u + j   -> position 16g + 4u + j
//   FP16 (one MFMA per 32 keys,  8 slots per lane group): slot 4(u&1)+j -> position 32(u/2) + 8g + 4(u&1) + j
template <int ESIZE>
__device__ inline int vt_pos(int kk)
{
    int const u = kk >> 4, g = (kk >> 2) & 3, j = kk & 3;
    return ESIZE == 1 ? 16 * g + 4 * u + j : 32 * (u >> 1) + 8 * g + 4 * (u & 1) + j;
}

// Byte address of the 16-byte chunk `chunk` (16*ESIZE... elements) of matrix `mat` (0 Q, 1 K, 2 V)
// for head n, token `tok` of the sequence described by (base, tokStride).
template <int ESIZE, bool INTERLEAVED>
__device__ inline int64_t qkv_chunk_offset(
    FmhaArgs const& a, int64_t seqBase, int64_t firstTok, int tok, int n, int mat, int chunk)
{
    if (INTERLEAVED)
    {
        // [3][N][d/32][T][32] bytes; chunk = 16-byte unit of the 64-byte head row
        int64_t const grp = ((int64_t) mat * a.N + n) * 2 + (chunk >> 1);
        return (grp * a.total + firstTok + tok) * 32 + (chunk & 1) * 16;
    }
    return seqBase + (int64_t) tok * a.tokStrideIn + ((int64_t) n * 3 + mat) * kHeadSize * ESIZE + chunk * 16;
}

// Builds the 512-bit key-valid mask of sequence b in LDS (sMask[16]).
__device__ inline void build_key_mask(FmhaArgs const& a, int b, int nk, uint32_t* sMask)
{
    if (threadIdx.x < 16)
    {
        uint32_t w = 0;
        int const k0 = threadIdx.x * 32;
        if (a.packedMask == nullptr)
        {
            int const v = nk - k0;
            w = v >= 32 ? 0xffffffffu : (v <= 0 ? 0u : ((1u << v) - 1u));
        }
        else
        {
            uint32_t const* pm = a.packedMask + (int64_t) b * a.maskStrideWords;
            for (int i = 0; i < 32; ++i)
            {
                int const key = k0 + i;
                if (key < nk)
                {
                    int const span = 16 * a.warpsN;
                    int const ni = key / span;
                    int const r = key % span;
                    int const warpN = r >> 4;
                    int const r2 = r & 15;
                    int const tidx = warpN * a.warpsM * 32 + ((r2 & 7) >> 1);
                    int const bit = 8 * ni + (r2 & 1) + ((r2 & 8) ? 4 : 0);
                    w |= ((pm[tidx] >> bit) & 1u) << i;
                }
            }
        }
        sMask[threadIdx.x] = w;
    }
}

// Stage K (row-major, padded) and V (transposed, permuted) of one (sequence, head) into LDS.
// Rows at or beyond nk are zero.  ESIZE = bytes per element (1 INT8, 2 FP16).
template <int ESIZE, int KT, bool INTERLEAVED, int WAVES>
__device__ inline void stage_kv(
    FmhaArgs const& a, int64_t seqBase, int64_t firstTok, int n, int nk, int nkb, uint8_t* sK, uint8_t* sVT)
{
    constexpr int kChunks = kHeadSize * ESIZE / 16;     // 16-byte chunks per head row: 4 or 8
    constexpr int kRowsPerPass = WAVES * kWaveSize / kChunks;
    constexpr int kPasses = 64 / kRowsPerPass;          // passes per 64-key block
    constexpr int kVtRow = Lds<ESIZE>::vtRow(KT);
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);
    int const chunk = threadIdx.x % kChunks;
    int const rowInPass = threadIdx.x / kChunks;
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
            u32x4 kv[kPasses], vv[kPasses];
#pragma unroll
            for (int p = 0; p < kPasses; ++p)
            {
                int const key = kb * 64 + p * kRowsPerPass + rowInPass;
                kv[p] = u32x4{0, 0, 0, 0};
                vv[p] = u32x4{0, 0, 0, 0};
                if (key < nk)
                {
                    kv[p] = *reinterpret_cast<u32x4 const*>(
                        src + qkv_chunk_offset<ESIZE, INTERLEAVED>(a, seqBase, firstTok, key, n, 1, chunk));
                    vv[p] = *reinterpret_cast<u32x4 const*>(
                        src + qkv_chunk_offset<ESIZE, INTERLEAVED>(a, seqBase, firstTok, key, n, 2, chunk));
                }
            }
#pragma unroll
            for (int p = 0; p < kPasses; ++p)
            {
                int const kk = p * kRowsPerPass + rowInPass;
                int const key = kb * 64 + kk;
                *reinterpret_cast<u32x4*>(sK + key * Lds<ESIZE>::kKRow + chunk * 16) = kv[p];
                int const col = (kb * 64 + vt_pos<ESIZE>(kk)) * ESIZE;
                if (ESIZE == 1)
                {
#pragma unroll
                    for (int x = 0; x < 16; ++x)
                    {
                        sVT[(chunk * 16 + x) * kVtRow + col] = (uint8_t) (vv[p][x >> 2] >> (8 * (x & 3)));
                    }
                }
                else
                {
#pragma unroll
                    for (int x = 0; x < 8; ++x)
                    {
                        *reinterpret_cast<uint16_t*>(sVT + (chunk * 8 + x) * kVtRow + col)
                            = (uint16_t) (vv[p][x >> 1] >> (16 * (x & 1)));
                    }
                }
            }
        }
    }
}

struct SeqInfo
{
    int64_t seqBaseIn, seqBaseOut, firstTok;
    int nq, nk;
};

__device__ inline SeqInfo seq_info(FmhaArgs const& a, int b, int capacity)
{
    SeqInfo s;
    if (a.cuSeqlens)
    {
        int const first = a.cuSeqlens[b];
        int const len = min(max(a.cuSeqlens[b + 1] - first, 0), capacity);
        s.firstTok = first;
        s.seqBaseIn = (int64_t) first * a.tokStrideIn;
        s.seqBaseOut = (int64_t) first * a.tokStrideOut;
        s.nq = len;
        s.nk = len;
    }
    else
    {
        s.firstTok = 0;
        s.seqBaseIn = (int64_t) b * a.seqStrideIn;
        s.seqBaseOut = (int64_t) b * a.seqStrideOut;
        s.nq = min(a.S, capacity);
        s.nk = min(a.S, capacity);
    }
    return s;
}

// ------------------------------------------------------------------------------------------
// INT8
// ------------------------------------------------------------------------------------------
template <int KT, bool INTERLEAVED, bool DEBUG>
__global__ __launch_bounds__(kWavesI8* kWaveSize) void fmha_i8_kernel(FmhaArgs const a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sK = smem;
    uint8_t* sVT = smem + Lds<1>::kBytes(KT);
    uint32_t* sMask = reinterpret_cast<uint32_t*>(sVT + kHeadSize * Lds<1>::vtRow(KT));
    constexpr int kVtRow = Lds<1>::vtRow(KT);
    constexpr int kKRow = Lds<1>::kKRow;

    uint32_t const bid = xcd_remap(blockIdx.x, gridDim.x);
    int const qt = bid % a.qTiles;
    int const n = (bid / a.qTiles) % a.N;
    int const b = bid / (a.qTiles * a.N);
    SeqInfo const sq = seq_info(a, b, KT * 64);
    int const q0 = qt * (kWavesI8 * kQPerWave);
    if (q0 >= sq.nq)
    {
        return;
    }
    int const nkb = (sq.nk + 63) >> 6;
    build_key_mask(a, b, sq.nk, sMask);
    stage_kv<1, KT, INTERLEAVED, kWavesI8>(a, sq.seqBaseIn, sq.firstTok, n, sq.nk, nkb, sK, sVT);

    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const lq = lane & 15; // query (column of S^T / O^T)
    int const g = lane >> 4;  // lane group: 16-byte k-chunk of the operands, 4 rows of the accumulators
    int const q = q0 + wave * kQPerWave + lq;
    bool const qValid = q < sq.nq;

    // Q^T operand: 16 bytes d = 16g .. 16g+15 of query q
    i32x4 qreg = {0, 0, 0, 0};
    if (qValid)
    {
        qreg = *reinterpret_cast<i32x4 const*>(static_cast<uint8_t const*>(a.qkv)
            + qkv_chunk_offset<1, INTERLEAVED>(a, sq.seqBaseIn, sq.firstTok, q, n, 0, g));
    }
    __syncthreads();
    if (q0 + wave * kQPerWave >= sq.nq)
    {
        return; // this wave's 16 rows lie beyond the sequence (no barrier follows)
    }

    // ---- S^T = K Q^T, biased so that the int32 reads as binary32 12582912 + acc ------------
    i32x4 acc[KT * 4];
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                int const key = kb * 64 + u * 16 + lq;
                i32x4 const kreg = *reinterpret_cast<i32x4 const*>(sK + key * kKRow + g * 16);
                acc[kb * 4 + u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                    kreg, qreg, i32x4{kMagicBits, kMagicBits, kMagicBits, kMagicBits}, 0, 0, 0);
            }
        }
    }

    if (DEBUG && a.dbgAcc1 && qValid)
    {
#pragma unroll
        for (int kb = 0; kb < KT; ++kb)
        {
            if (kb < nkb)
            {
                for (int u = 0; u < 4; ++u)
                {
                    for (int j = 0; j < 4; ++j)
                    {
                        int const key = kb * 64 + u * 16 + g * 4 + j;
                        if (key < sq.nk)
                        {
                            a.dbgAcc1[(((int64_t) b * a.N + n) * a.S + q) * a.S + key] = acc[kb * 4 + u][j] - kMagicBits;
                        }
                    }
                }
            }
        }
    }

    // ---- mask + row max (on the biased integers: the bias is monotone) ---------------------
    int mx = kMaskedBits;
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
            uint32_t const w0 = __builtin_amdgcn_readfirstlane(sMask[kb * 2]);
            uint32_t const w1 = __builtin_amdgcn_readfirstlane(sMask[kb * 2 + 1]);
            bool const full = (w0 & w1) == 0xffffffffu;
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                if (!full)
                {
                    uint32_t const bits = ((u < 2 ? w0 : w1) >> ((u & 1) * 16 + g * 4)) & 0xfu;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        acc[kb * 4 + u][j] = (bits >> j) & 1u ? acc[kb * 4 + u][j] : kMaskedBits;
                    }
                }
                mx = max(mx, max(max(acc[kb * 4 + u][0], acc[kb * 4 + u][1]),
                                 max(acc[kb * 4 + u][2], acc[kb * 4 + u][3])));
            }
        }
    }
    mx = max(mx, __shfl_xor(mx, 16, kWaveSize));
    mx = max(mx, __shfl_xor(mx, 32, kWaveSize));

    // ---- e = 2^((acc - max) * c), row sum -----------------------------------------------------
    float const negK0 = -__int_as_float(mx) * a.c;
    float sum = 0.f;
    float e[KT * 4][4];
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
            uint32_t const w0 = __builtin_amdgcn_readfirstlane(sMask[kb * 2]);
            uint32_t const w1 = __builtin_amdgcn_readfirstlane(sMask[kb * 2 + 1]);
            bool const full = (w0 & w1) == 0xffffffffu;
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    float v = __builtin_amdgcn_exp2f(fmaf(__int_as_float(acc[kb * 4 + u][j]), a.c, negK0));
                    if (!full)
                    {
                        v = acc[kb * 4 + u][j] == kMaskedBits ? 0.f : v;
                    }
                    e[kb * 4 + u][j] = v;
                    sum += v;
                }
            }
        }
    }
    sum += __shfl_xor(sum, 16, kWaveSize);
    sum += __shfl_xor(sum, 32, kWaveSize);
    float const r = sum > 0.f ? a.scaleSoftmax / sum : 0.f;

    // ---- p8 = rne(e * r) packed four keys to a dword; O^T = V^T P^T ---------------------------
    i32x4 oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
    {
        oacc[dt] = i32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
            i32x4 preg;
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                uint32_t yb[4];
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    float y = e[kb * 4 + u][j] * r;
                    if (a.clampP)
                    {
                        y = fminf(y, 127.f);
                    }
                    yb[j] = __float_as_uint(y + kMagic);
                }
                uint32_t const lo = __builtin_amdgcn_perm(yb[1], yb[0], 0x0c0c0400u);
                uint32_t const hi = __builtin_amdgcn_perm(yb[3], yb[2], 0x0c0c0400u);
                preg[u] = (int) __builtin_amdgcn_perm(hi, lo, 0x05040100u);
            }
            if (DEBUG && a.dbgP8 && qValid)
            {
                for (int u = 0; u < 4; ++u)
                {
                    for (int j = 0; j < 4; ++j)
                    {
                        int const key = kb * 64 + u * 16 + g * 4 + j;
                        if (key < sq.nk)
                        {
                            a.dbgP8[(((int64_t) b * a.N + n) * a.S + q) * a.S + key]
                                = (int8_t) ((uint32_t) preg[u] >> (8 * j));
                        }
                    }
                }
            }
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
            {
                i32x4 const vreg
                    = *reinterpret_cast<i32x4 const*>(sVT + (dt * 16 + lq) * kVtRow + kb * 64 + g * 16);
                oacc[dt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(vreg, preg, oacc[dt], 0, 0, 0);
            }
        }
    }

    // ---- out8 = sat8(rne(acc2 * scale_bmm2)); lane holds d = 16dt + 4g .. +3 of query q ------
    if (qValid)
    {
        uint8_t* dst = static_cast<uint8_t*>(a.out);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
        {
            uint32_t yb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                float y = (float) oacc[dt][j] * a.scaleBmm2;
                y = __builtin_amdgcn_fmed3f(y, -128.f, 127.f);
                yb[j] = __float_as_uint(y + kMagic);
            }
            uint32_t const lo = __builtin_amdgcn_perm(yb[1], yb[0], 0x0c0c0400u);
            uint32_t const hi = __builtin_amdgcn_perm(yb[3], yb[2], 0x0c0c0400u);
            uint32_t const packed = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
            int const d0 = dt * 16 + g * 4;
            int64_t off;
            if (INTERLEAVED)
            {
                // [N][d/32][T][32]
                off = (((int64_t) n * 2 + (d0 >> 5)) * a.total + sq.firstTok + q) * 32 + (d0 & 31);
            }
            else
            {
                off = sq.seqBaseOut + (int64_t) q * a.tokStrideOut + (int64_t) n * kHeadSize + d0;
            }
            *reinterpret_cast<uint32_t*>(dst + off) = packed;
        }
    }
}

// ------------------------------------------------------------------------------------------
// FP16
// ------------------------------------------------------------------------------------------
template <int KT, bool DEBUG>
__global__ __launch_bounds__(kWavesF16* kWaveSize) void fmha_f16_kernel(FmhaArgs const a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sK = smem;
    uint8_t* sVT = smem + Lds<2>::kBytes(KT);
    uint32_t* sMask = reinterpret_cast<uint32_t*>(sVT + kHeadSize * Lds<2>::vtRow(KT));
    constexpr int kVtRow = Lds<2>::vtRow(KT);
    constexpr int kKRow = Lds<2>::kKRow;

    uint32_t const bid = xcd_remap(blockIdx.x, gridDim.x);
    int const qt = bid % a.qTiles;
    int const n = (bid / a.qTiles) % a.N;
    int const b = bid / (a.qTiles * a.N);
    SeqInfo const sq = seq_info(a, b, KT * 64);
    int const q0 = qt * (kWavesF16 * kQPerWave);
    if (q0 >= sq.nq)
    {
        return;
    }
    int const nkb = (sq.nk + 63) >> 6;
    build_key_mask(a, b, sq.nk, sMask);
    stage_kv<2, KT, false, kWavesF16>(a, sq.seqBaseIn, sq.firstTok, n, sq.nk, nkb, sK, sVT);

    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const lq = lane & 15;
    int const g = lane >> 4;
    int const q = q0 + wave * kQPerWave + lq;
    bool const qValid = q < sq.nq;

    // Q^T operands: MFMA h covers d = 32h + 8g .. +7
    f16x8 qreg[2];
#pragma unroll
    for (int h = 0; h < 2; ++h)
    {
        u32x4 raw = {0, 0, 0, 0};
        if (qValid)
        {
            raw = *reinterpret_cast<u32x4 const*>(static_cast<uint8_t const*>(a.qkv)
                + qkv_chunk_offset<2, false>(a, sq.seqBaseIn, sq.firstTok, q, n, 0, h * 4 + g));
        }
        qreg[h] = __builtin_bit_cast(f16x8, raw);
    }
    __syncthreads();
    if (q0 + wave * kQPerWave >= sq.nq)
    {
        return;
    }

    // ---- S^T = K Q^T (binary32 accumulation) ---------------------------------------------------
    f32x4 acc[KT * 4];
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                int const key = kb * 64 + u * 16 + lq;
                f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int h = 0; h < 2; ++h)
                {
                    f16x8 const kreg = *reinterpret_cast<f16x8 const*>(sK + key * kKRow + (h * 4 + g) * 16);
                    s = __builtin_amdgcn_mfma_f32_16x16x32_f16(kreg, qreg[h], s, 0, 0, 0);
                }
                acc[kb * 4 + u] = s;
            }
        }
    }

    if (DEBUG && a.dbgAcc1 && qValid)
    {
#pragma unroll
        for (int kb = 0; kb < KT; ++kb)
        {
            if (kb < nkb)
            {
                for (int u = 0; u < 4; ++u)
                {
                    for (int j = 0; j < 4; ++j)
                    {
                        int const key = kb * 64 + u * 16 + g * 4 + j;
                        if (key < sq.nk)
                        {
                            a.dbgAcc1[(((int64_t) b * a.N + n) * a.S + q) * a.S + key]
                                = __float_as_int(acc[kb * 4 + u][j]);
                        }
                    }
                }
            }
        }
    }

    // ---- mask + row max ------------------------------------------------------------------------
    constexpr float kNegBig = -3.0e38f;
    float mx = kNegBig;
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
            uint32_t const w0 = __builtin_amdgcn_readfirstlane(sMask[kb * 2]);
            uint32_t const w1 = __builtin_amdgcn_readfirstlane(sMask[kb * 2 + 1]);
            bool const full = (w0 & w1) == 0xffffffffu;
#pragma unroll
            for (int u = 0; u < 4; ++u)
            {
                if (!full)
                {
                    uint32_t const bits = ((u < 2 ? w0 : w1) >> ((u & 1) * 16 + g * 4)) & 0xfu;
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        acc[kb * 4 + u][j] = (bits >> j) & 1u ? acc[kb * 4 + u][j] : kNegBig;
                    }
                }
                mx = fmaxf(mx, fmaxf(fmaxf(acc[kb * 4 + u][0], acc[kb * 4 + u][1]),
                                     fmaxf(acc[kb * 4 + u][2], acc[kb * 4 + u][3])));
            }
        }
    }
    mx = fmaxf(mx, __shfl_xor(mx, 16, kWaveSize));
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWaveSize));

    // ---- p = 2^((s - max) * c) rounded to binary16; O^T = V^T P^T; the row sum is taken by the
    //      matrix unit as well (a tile of ones), so numerator and denominator see the same
    //      rounded probabilities -------------------------------------------------------------------
    float const negK0 = -mx * a.c;
    f32x4 oacc[4];
    f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
    {
        oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    f16x8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        ones[i] = (f16) 1.f;
    }
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
            uint32_t const w0 = __builtin_amdgcn_readfirstlane(sMask[kb * 2]);
            uint32_t const w1 = __builtin_amdgcn_readfirstlane(sMask[kb * 2 + 1]);
            bool const full = (w0 & w1) == 0xffffffffu;
#pragma unroll
            for (int hb = 0; hb < 2; ++hb) // 32-key half of the block
            {
                f16x8 preg;
#pragma unroll
                for (int w = 0; w < 2; ++w)
                {
                    int const t = kb * 4 + hb * 2 + w;
                    float p[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        float v = __builtin_amdgcn_exp2f(fmaf(acc[t][j], a.c, negK0));
                        if (!full)
                        {
                            v = acc[t][j] == kNegBig ? 0.f : v;
                        }
                        p[j] = v;
                    }
                    f16x2 const p01 = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(p[0], p[1]));
                    f16x2 const p23 = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(p[2], p[3]));
                    preg[w * 4 + 0] = p01[0];
                    preg[w * 4 + 1] = p01[1];
                    preg[w * 4 + 2] = p23[0];
                    preg[w * 4 + 3] = p23[1];
                }
                if (DEBUG && a.dbgP8)
                {
                    // not used for FP16
                }
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
                {
                    f16x8 const vreg = *reinterpret_cast<f16x8 const*>(
                        sVT + (dt * 16 + lq) * kVtRow + ((kb * 64 + hb * 32) + g * 8) * 2);
                    oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vreg, preg, oacc[dt], 0, 0, 0);
                }
                sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, preg, sacc, 0, 0, 0);
            }
        }
    }

    if (qValid)
    {
        float const rinv = sacc[0] > 0.f ? 1.f / sacc[0] : 0.f;
        uint8_t* dst = static_cast<uint8_t*>(a.out);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
        {
            f16x4 y;
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                y[j] = (f16) (oacc[dt][j] * rinv);
            }
            int const d0 = dt * 16 + g * 4;
            int64_t const off = sq.seqBaseOut + (int64_t) q * a.tokStrideOut + ((int64_t) n * kHeadSize + d0) * 2;
            *reinterpret_cast<u32x2*>(dst + off) = __builtin_bit_cast(u32x2, y);
        }
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------

template <typename K>
int launch_fmha(K kernel, char const* name, hipStream_t stream, FmhaArgs const& args, int ldsBytes, int waves)
{
    // Raising the dynamic LDS limit is a per-function attribute; set once per process.
    static std::mutex mtx;
    static std::vector<void const*> done;
    {
        std::lock_guard<std::mutex> lock(mtx);
        void const* key = reinterpret_cast<void const*>(kernel);
        bool found = false;
        for (void const* p : done)
        {
            found = found || p == key;
        }
        if (!found)
        {
            hipError_t const e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes);
            if (e != hipSuccess)
            {
                (void) hipGetLastError();
                return set_error(TRTAMD_STATUS_FAILURE, "%s: cannot reserve %d bytes of LDS: %s", name, ldsBytes,
                    hipGetErrorString(e));
            }
            done.push_back(key);
        }
    }
    unsigned const blocks = (unsigned) args.B * args.N * args.qTiles;
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(waves * kWaveSize), ldsBytes, stream, args);
    return check_launch(name);
}

int pick_kt(int s)
{
    for (int kt : {1, 2, 3, 4, 6, 8})
    {
        if (s <= kt * 64)
        {
            return kt;
        }
    }
    return 0;
}

template <bool DEBUG>
int run_i8(hipStream_t stream, FmhaArgs const& a, bool interleaved)
{
    int const kt = pick_kt(a.S);
#define TRTAMD_I8(KT)                                                                                                  \
    case KT:                                                                                                           \
        return interleaved ? launch_fmha(fmha_i8_kernel<KT, true, DEBUG>, "fmha_i8_interleaved", stream, a,           \
                   Lds<1>::total(KT), kWavesI8)                                                                        \
                           : launch_fmha(fmha_i8_kernel<KT, false, DEBUG>, "fmha_i8", stream, a, Lds<1>::total(KT),    \
                               kWavesI8)
    switch (kt)
    {
        TRTAMD_I8(1);
        TRTAMD_I8(2);
        TRTAMD_I8(3);
        TRTAMD_I8(4);
        TRTAMD_I8(6);
        TRTAMD_I8(8);
    default: break;
    }
#undef TRTAMD_I8
    return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fused MHA: sequence length %d exceeds 512", a.S);
}

template <bool DEBUG>
int run_f16(hipStream_t stream, FmhaArgs const& a)
{
    int const kt = pick_kt(a.S);
#define TRTAMD_F16(KT)                                                                                                 \
    case KT: return launch_fmha(fmha_f16_kernel<KT, DEBUG>, "fmha_f16", stream, a, Lds<2>::total(KT), kWavesF16)
    switch (kt)
    {
        TRTAMD_F16(1);
        TRTAMD_F16(2);
        TRTAMD_F16(3);
        TRTAMD_F16(4);
        TRTAMD_F16(6);
        TRTAMD_F16(8);
    default: break;
    }
#undef TRTAMD_F16
    return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fused MHA: sequence length %d exceeds 512", a.S);
}

float bits_to_float(uint32_t u)
{
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// binary16 (low half of a half2 bit pattern) to binary32
float half_bits_to_float(uint16_t h)
{
    uint32_t const sign = (uint32_t) (h & 0x8000u) << 16;
    uint32_t const exp = (h >> 10) & 0x1fu;
    uint32_t const man = h & 0x3ffu;
    if (exp == 0)
    {
        float const v = (float) man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    uint32_t const bits = exp == 31 ? (sign | 0x7f800000u | (man << 13)) : (sign | ((exp + 112u) << 23) | (man << 13));
    return bits_to_float(bits);
}

int fused_mha_run(hipStream_t stream, int32_t dataType, trtamd_fmha_params const* p, int32_t* dbgAcc1, int8_t* dbgP8)
{
    if (!p)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: null parameter block");
    }
    if (dataType != 1 && dataType != 2)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fused MHA: data type %d (only FP16=1 and INT8=2)", dataType);
    }
    if (p->d != kHeadSize)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fused MHA: head size %d (only 64)", p->d);
    }
    if (p->b < 0 || p->h <= 0 || p->s <= 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: bad dimensions b=%d h=%d s=%d", p->b, p->h, p->s);
    }
    if (p->s > 512)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fused MHA: sequence length %d exceeds 512", p->s);
    }
    if (p->b == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    if (!p->qkv_ptr || !p->o_ptr)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: null tensor pointer");
    }
    if (!aligned16(p->qkv_ptr) || (reinterpret_cast<uintptr_t>(p->o_ptr) & 7u) != 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: qkv must be 16-byte and output 8-byte aligned");
    }
    bool const interleaved = p->interleaved != 0;
    if (interleaved && (dataType != 2 || !p->cu_seqlens))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: interleaved layout needs INT8 and cu_seqlens");
    }
    int const esize = dataType == 2 ? 1 : 2;
    FmhaArgs a{};
    a.qkv = p->qkv_ptr;
    a.out = p->o_ptr;
    a.cuSeqlens = p->cu_seqlens;
    a.B = p->b;
    a.N = p->h;
    a.S = p->s;
    a.qTiles = ceil_div(p->s, (dataType == 2 ? kWavesI8 : kWavesF16) * kQPerWave);
    a.dbgAcc1 = dbgAcc1;
    a.dbgP8 = dbgP8;
    if (interleaved)
    {
        // strides carry the total token count (qkvToContextInt8InterleavedPlugin.cpp:280-281)
        if (p->qkv_stride_in_bytes <= 0 || p->qkv_stride_in_bytes != p->o_stride_in_bytes
            || p->qkv_stride_in_bytes > 0x7fffffffLL)
        {
            return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: interleaved strides must both equal the token count");
        }
        a.total = (int32_t) p->qkv_stride_in_bytes;
    }
    else
    {
        int64_t const rowIn = (int64_t) 3 * p->h * kHeadSize * esize;
        int64_t const rowOut = (int64_t) p->h * kHeadSize * esize;
        a.tokStrideIn = p->qkv_stride_in_bytes;
        a.tokStrideOut = p->o_stride_in_bytes;
        if (a.tokStrideIn < rowIn || a.tokStrideOut < rowOut || (a.tokStrideIn & 15) != 0 || (a.tokStrideOut & 7) != 0)
        {
            return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: strides %lld/%lld too small or misaligned",
                (long long) a.tokStrideIn, (long long) a.tokStrideOut);
        }
        if (!p->cu_seqlens)
        {
            // fixed [S,B,N,3,d]: the token stride spans B sequences (MHARunner::setup, mhaRunner.h:62-83)
            a.seqStrideIn = rowIn;
            a.seqStrideOut = rowOut;
            if (a.tokStrideIn < rowIn * p->b || a.tokStrideOut < rowOut * p->b)
            {
                return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: fixed layout strides do not span the batch");
            }
        }
    }
    if (!p->cu_seqlens && p->packed_mask_ptr)
    {
        int wm = p->warps_m, wn = p->warps_n;
        if (wm == 0 || wn == 0)
        {
            // FusedMHARunner{FP16,Int8}::mhaImpl::setup, mhaRunner.cu:676-692, 805-821
            if (p->s == 64 || p->s == 96 || p->s == 128)
            {
                wm = 2;
                wn = 2;
            }
            else if (p->s == 384)
            {
                wm = 1;
                wn = 8;
            }
            else
            {
                return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fused MHA: no packed-mask geometry for s=%d", p->s);
            }
        }
        a.packedMask = static_cast<uint32_t const*>(p->packed_mask_ptr);
        a.warpsM = wm;
        a.warpsN = wn;
        a.maskStrideWords = p->packed_mask_stride_in_bytes / 4;
        int const xn = ceil_div(p->s, 16 * wn);
        if (xn > 4 || a.maskStrideWords < (int64_t) wm * wn * 32)
        {
            return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA: packed mask geometry/stride inconsistent with s");
        }
    }
    if (dataType == 2)
    {
        float const s1 = bits_to_float(p->scale_bmm1);
        float const ss = bits_to_float(p->scale_softmax);
        float const s2 = bits_to_float(p->scale_bmm2);
        if (!(s1 > 0.f) || !(ss > 0.f) || !(s2 > 0.f))
        {
            return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA INT8: scales must be positive (%g, %g, %g)", s1, ss, s2);
        }
        a.c = s1 * kLog2e;
        a.scaleSoftmax = ss;
        a.scaleBmm2 = s2;
        a.clampP = ss > 127.f ? 1 : 0;
        return (dbgAcc1 || dbgP8) ? run_i8<true>(stream, a, interleaved) : run_i8<false>(stream, a, interleaved);
    }
    // FP16: scale_bmm1 is a half2 holding 1/sqrt(d) twice; softmax/bmm2 scales are 1 (mhaRunner.cu:694-701)
    float const s1 = half_bits_to_float((uint16_t) (p->scale_bmm1 & 0xffffu));
    if (!(s1 > 0.f))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fused MHA FP16: scale_bmm1 must be positive (%g)", s1);
    }
    a.c = s1 * kLog2e;
    a.scaleSoftmax = 1.f;
    a.scaleBmm2 = 1.f;
    return dbgAcc1 ? run_f16<true>(stream, a) : run_f16<false>(stream, a);
}

} // namespace
} // namespace trtamd

using namespace trtamd;

extern "C" int trtamd_fused_mha_run(trtamd_stream_t stream, int32_t data_type, trtamd_fmha_params const* params)
{
    return fused_mha_run(as_stream(stream), data_type, params, nullptr, nullptr);
}

// Test hook: same launch, additionally dumping the first GEMM's accumulators ([b][h][s][s],
// int32 for INT8, binary32 bit patterns for FP16) and, for INT8, the quantised probabilities.
extern "C" TRTAMD_API int trtamd_fused_mha_run_debug(trtamd_stream_t stream, int32_t data_type,
    trtamd_fmha_params const* params, int32_t* acc1, int8_t* p8)
{
    return fused_mha_run(as_stream(stream), data_type, params, acc1, p8);
}

extern "C" int trtamd_fused_mha_is_valid(int32_t data_type, int32_t d, int32_t s)
{
    return (data_type == 1 || data_type == 2) && d == kHeadSize && s > 0 && s <= 512;
}
