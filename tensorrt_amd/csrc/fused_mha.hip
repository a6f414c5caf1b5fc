// Fused multi-head attention for gfx950 (head size 64, sequence length <= 512), INT8 and FP16.
//
// Stands in for the precompiled fused_multihead_attention / fused_multihead_attention_v2 kernels
// the reference loads from cubins (plugin/bertQKVToContextPlugin/fused_multihead_attention*/):
// one launch computes softmax(Q K^T * scale) V for every (sequence, head).
//
// Work split: a workgroup stages K and V of one (sequence, head) in LDS once (both row-major, rows
// padded by 16 bytes so 16-byte reads of consecutive keys fall in different banks) and its
// wavefronts then walk the 16-row query tiles of that head round-robin; `qSplit` workgroups share
// one head when the batch is too small to fill the chip otherwise.  Per query tile a wave
//   1. computes S^T = K Q^T with v_mfma_i32_16x16x64_i8 (v_mfma_f32_16x16x32_f16 for FP16): the
//      accumulator layout gives every lane 4 keys x 1 query per 16-key tile, which is exactly the
//      B-operand layout of step 3, so probabilities never leave registers;
//   2. does the row softmax over the whole row (<= 512 keys) in registers: max/sum need only two
//      cross-lane steps (the 4 lane groups that share a query).  INT8 accumulators are seeded
//      with the bit pattern of 1.5*2^23 so the integer result reads directly as a binary32
//      number (no int->float conversion); probabilities are quantised with one fused
//      multiply-add against the same constant (round-to-nearest-even lands in the low byte);
//   3. computes O^T = V^T P^T with the same MFMA; the V^T operand (16 keys of one head-dim per
//      lane) is produced from row-major V by the LDS transpose reads ds_read_b64_tr_b8 /
//      ds_read_b64_tr_b16, so V is never transposed in memory;
//   4. requantises (INT8) or normalises (FP16) on store.
// Queries beyond the sequence length are neither computed nor written.
#include "device_utils.hpp"
#include "host_utils.hpp"
#include "trtamd_test_hooks.h"

#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <vector>

namespace trtamd
{
namespace
{

constexpr int kQPerWave = 16;
constexpr int kWavesI8 = 4;
constexpr int kWavesF16 = 8; // FP16 K/V take twice the LDS, so one (larger) workgroup per CU
constexpr int kHeadSize = 64;
constexpr int kMagicBits = 0x4B400000;         // bit pattern of 12582912.f = 1.5 * 2^23
constexpr float kMagic = 12582912.f;
constexpr float kLog2e = 1.4426950408889634f;

typedef __attribute__((address_space(3))) i32x2 lds_i32x2;
typedef short i16x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) i16x4 lds_i16x4;

// a * b rounded to binary32 on its own: the caller's following add must not absorb it into an fma
__device__ inline float mul_rounded(float a, float b)
{
#pragma clang fp contract(off)
    return a * b;
}

// The MFMAs of the cu_seqlens kernels (fmha_i8_prefix_kernel, fmha_f16_prefix_kernel) go through these wrappers.  A
// library built with -DTRTAMD_ABLATE_ATTENTION_MFMA (`python -m tensorrt_amd.build --ablation` writes it to
// lib/libtrtamd_ablation.so; `python -m tensorrt_amd.kernel_bench --ablation` times it; nothing else loads it) leaves
// the instruction out: the result registers keep what they held and every other instruction of the kernel stays, so
// the results are wrong and the launch takes what the kernel would take if its matrix work cost nothing.
__device__ __forceinline__ i32x4 attention_mfma_i8(i32x4 const a, i32x4 const b, i32x4 c)
{
#ifdef TRTAMD_ABLATE_ATTENTION_MFMA
    i32x4 d;
    asm volatile("; v_mfma_i32_16x16x64_i8 left out" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
#else
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
#endif
}

__device__ __forceinline__ f32x4 attention_mfma_f16(f16x8 const a, f16x8 const b, f32x4 c)
{
#ifdef TRTAMD_ABLATE_ATTENTION_MFMA
    f32x4 d;
    asm volatile("; v_mfma_f32_16x16x32_f16 left out" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
#else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
#endif
}

// x[dt] of the lane in 16-lane row g  ->  x[g'] = what row g' held in its x[g]: a 4 x 4 transpose over the four rows of
// a wavefront.  All 64 lanes must be active.  The attention kernels end with lane (g, query) holding a piece of each
// quarter dt of the query's output row; transposed, it holds the whole quarter dt = g and stores it in one piece.
__device__ inline void rows_transpose(uint32_t (&x)[4])
{
    // rows 0,1 keep x[0] / x[1] of their own and get the same from rows 2,3; rows 2,3 the other way round
    auto const s02 = __builtin_amdgcn_permlane32_swap(x[0], x[2], false, false);
    auto const s13 = __builtin_amdgcn_permlane32_swap(x[1], x[3], false, false);
    // even rows keep the first of a pair and get it from the odd row below them; odd rows the second
    auto const t01 = __builtin_amdgcn_permlane16_swap(s02[0], s13[0], false, false);
    auto const t23 = __builtin_amdgcn_permlane16_swap(s02[1], s13[1], false, false);
    x[0] = t01[0];
    x[1] = t01[1];
    x[2] = t23[0];
    x[3] = t23[1];
}

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
    int32_t qSplit;              // workgroups per (sequence, head)
    int32_t total;               // interleaved: total token count
    int32_t warpsM, warpsN;      // geometry of the packed mask
    float c;                     // scale_bmm1 * log2(e)
    float scaleSoftmax;
    float scaleBmm2;
    int32_t clampP;              // scale_softmax may push p beyond 127
    int32_t* dbgAcc1;            // optional [B][N][S][S] int32 (INT8) / float bits (FP16)
    int8_t* dbgP8;               // optional [B][N][S][S]
    int32_t ranked;              // serve the longest sequences first (pointless when one round holds every workgroup)
};

template <int ESIZE>
struct Lds
{
    // K and V rows of 64 elements, unpadded; the 16-byte chunks of a row are XOR-swizzled with
    // the row index (see swz) so that the 8 consecutive rows a 16-lane group reads fall in
    // different banks
    static constexpr int kRow = kHeadSize * ESIZE;
    static __host__ __device__ constexpr int matBytes(int kt)
    {
        return kt * 64 * kRow;
    }
    static __host__ __device__ constexpr int total(int kt)
    {
        return 2 * matBytes(kt) + 16 * 4;
    }
};

// LDS row, inside its 64-key block, at which V's key kk is stored.  The accumulator of S^T gives
// lane group g the keys 16u + 4g + j (u = 16-key tile, j = 0..3) and the P^T operand is built
// from it without moving data.  One INT8 transpose read returns 8 keys to each lane group, which
// must be 8 consecutive LDS rows: tiles (2h, 2h+1), keys 4g..4g+3 of each -> rows 32h + 8g + 4(u&1) + j.
// The FP16 transpose read returns 4 keys, already consecutive (16u + 4g + j): natural order.
template <int ESIZE>
__device__ inline int v_row(int kk)
{
    int const u = kk >> 4, g = (kk >> 2) & 3, j = kk & 3;
    return ESIZE == 1 ? 32 * (u >> 1) + 8 * g + 4 * (u & 1) + j : kk;
}

// Position of 16-byte chunk `chunk` inside LDS row `row`.  Rows are 64 (INT8) or 128 (FP16) bytes;
// consecutive rows advance by a quarter / a half of the 256-byte bank window, so rows 2 (INT8) or
// 1 (FP16) apart in the sense below would collide without the swizzle.
template <int ESIZE>
__device__ inline int swz(int row, int chunk)
{
    return ESIZE == 1 ? (chunk ^ ((row >> 1) & 3)) : (chunk ^ (row & 7));
}

// Byte address of the 16-byte chunk `chunk` of matrix `mat` (0 Q, 1 K, 2 V) for head n, token
// `tok` of the sequence described by (seqBase, firstTok).
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

// Builds the 512-bit key-valid mask of sequence b in LDS (sMask[16]): every thread takes one key (and one word of the
// packed mask, if there is one), a wavefront's 64 answers become two words of the mask.
__device__ inline void build_key_mask(FmhaArgs const& a, int b, int nk, uint32_t* sMask)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    for (int key = threadIdx.x; key < 512; key += blockDim.x)
    {
        bool valid = key < nk;
        if (valid && a.packedMask != nullptr)
        {
            // bit layout of fillSBSMaskKernel (plugin/embLayerNormPlugin/embLayerNormKernel.cu:41-85)
            uint32_t const* pm = a.packedMask + (int64_t) b * a.maskStrideWords;
            int const span = 16 * a.warpsN;
            int const ni = key / span;
            int const r = key % span;
            int const warpN = r >> 4;
            int const r2 = r & 15;
            int const tidx = warpN * a.warpsM * 32 + ((r2 & 7) >> 1);
            int const bit = 8 * ni + (r2 & 1) + ((r2 & 8) ? 4 : 0);
            valid = ((pm[tidx] >> bit) & 1u) != 0;
        }
        uint64_t const m = __ballot(valid);
        if (lane == 0)
        {
            sMask[key >> 5] = (uint32_t) m;
            sMask[(key >> 5) + 1] = (uint32_t) (m >> 32);
        }
    }
}

// One past the last key of the mask that takes part (0: none does).  Keys behind it have probability zero whatever
// their scores, so the kernels treat the sequence as that much shorter: whole blocks of masked keys at the end are
// neither loaded nor multiplied.  sMask must be complete (barrier) before the call; the result is wave-uniform.
__device__ inline int used_keys(uint32_t const* sMask, int nk)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    uint32_t const w = lane < 16 ? sMask[lane] : 0u;
    int end = w ? lane * 32 + 32 - __builtin_clz(w) : 0;
#pragma unroll
    for (int d = 1; d < 16; d *= 2)
    {
        end = max(end, __shfl_xor(end, d));
    }
    return min(__builtin_amdgcn_readfirstlane(end), nk);
}

// Stage K and V of one (sequence, head) into LDS, 16 bytes per lane per access.  Rows at or
// beyond nk are zero, and so are the K rows of masked keys: a masked key's score is then exactly
// the accumulator's seed, which the caller sets to -infinity (see mask_seed).  ESIZE = bytes per
// element (1 INT8, 2 FP16).  sMask must be complete (barrier) before the call.
template <int ESIZE, int KT, bool INTERLEAVED, int WAVES>
__device__ inline void stage_kv(FmhaArgs const& a, int64_t seqBase, int64_t firstTok, int n, int nk, int nkb,
    uint32_t const* sMask, uint8_t* sK, uint8_t* sV)
{
    constexpr int kChunks = kHeadSize * ESIZE / 16;     // 16-byte chunks per head row: 4 or 8
    constexpr int kRowsPerPass = WAVES * kWaveSize / kChunks;
    constexpr int kPasses = 64 / kRowsPerPass;          // passes per 64-key block
    constexpr int kRow = Lds<ESIZE>::kRow;
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);
    int const chunk = threadIdx.x % kChunks;
    int const rowInPass = threadIdx.x / kChunks;
    // every global load of the workgroup is issued before the first LDS write, so the loads of
    // all key blocks are in flight together
    u32x4 kv[KT][kPasses], vv[KT][kPasses];
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
#pragma unroll
        for (int p = 0; p < kPasses; ++p)
        {
            int const key = kb * 64 + p * kRowsPerPass + rowInPass;
            kv[kb][p] = u32x4{0, 0, 0, 0};
            vv[kb][p] = u32x4{0, 0, 0, 0};
            if (key < nk)
            {
                vv[kb][p] = *reinterpret_cast<u32x4 const*>(
                    src + qkv_chunk_offset<ESIZE, INTERLEAVED>(a, seqBase, firstTok, key, n, 2, chunk));
                if ((sMask[key >> 5] >> (key & 31)) & 1u)
                {
                    kv[kb][p] = *reinterpret_cast<u32x4 const*>(
                        src + qkv_chunk_offset<ESIZE, INTERLEAVED>(a, seqBase, firstTok, key, n, 1, chunk));
                }
            }
        }
    }
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
#pragma unroll
            for (int p = 0; p < kPasses; ++p)
            {
                int const kk = p * kRowsPerPass + rowInPass;
                int const kr = kb * 64 + kk;
                int const vr = kb * 64 + v_row<ESIZE>(kk);
                *reinterpret_cast<u32x4*>(sK + kr * kRow + swz<ESIZE>(kr, chunk) * 16) = kv[kb][p];
                *reinterpret_cast<u32x4*>(sV + vr * kRow + swz<ESIZE>(vr, chunk) * 16) = vv[kb][p];
            }
        }
    }
}

// Accumulator seed of the four keys 16u + 4g + j of a 16-key tile: `valid` for keys that take
// part, the bit pattern of -infinity for masked ones (their K rows are zero, so the seed is their
// score): the integer/float row maximum ignores it and 2^(-inf) = 0 removes it from the softmax
// without any per-score instruction.
constexpr int kNegInfBits = (int) 0xFF800000u;
__device__ inline i32x4 mask_seed(uint32_t w0, uint32_t w1, int u, int g, int valid)
{
    uint32_t const bits = ((u < 2 ? w0 : w1) >> ((u & 1) * 16 + g * 4)) & 0xfu;
    i32x4 seed;
#pragma unroll
    for (int j = 0; j < 4; ++j)
    {
        seed[j] = (bits >> j) & 1u ? valid : kNegInfBits;
    }
    return seed;
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

// Which sequence a workgroup serves.  Workgroups are dispatched in index order, so serving the
// longest sequences first (cost grows with the square of the length) lets the short ones fill the
// tail of the launch.  `rank` is the position in that order; every workgroup ranks the (at most
// kMaxRanked) sequence lengths itself with a counting sort in LDS: no state outside the launch.
constexpr int kMaxRanked = 1024;
template <int THREADS>
__device__ inline int pick_sequence(FmhaArgs const& a, int rank, int* sLens /* [kMaxRanked + 1] */)
{
    if (a.cuSeqlens == nullptr || a.B > kMaxRanked || a.B == 1)
    {
        return rank; // fixed layout (equal lengths) or too many sequences: natural order
    }
    for (int t = threadIdx.x; t < a.B; t += THREADS)
    {
        sLens[t] = a.cuSeqlens[t + 1] - a.cuSeqlens[t];
    }
    if (threadIdx.x == 0)
    {
        sLens[kMaxRanked] = rank;
    }
    __syncthreads();
    for (int t = threadIdx.x; t < a.B; t += THREADS)
    {
        int const mine = sLens[t];
        int before = 0; // sequences served before t: longer ones, ties by index
        for (int o = 0; o < a.B; ++o)
        {
            int const other = sLens[o];
            before += (other > mine || (other == mine && o < t)) ? 1 : 0;
        }
        if (before == rank)
        {
            sLens[kMaxRanked] = t;
        }
    }
    __syncthreads();
    return sLens[kMaxRanked];
}

// ------------------------------------------------------------------------------------------
// INT8
// ------------------------------------------------------------------------------------------
template <int KT, bool INTERLEAVED, bool DEBUG>
__global__ __launch_bounds__(kWavesI8* kWaveSize) __attribute__((amdgpu_waves_per_eu(KT <= 6 ? 3 : 2))) void fmha_i8_kernel(FmhaArgs const a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sK = smem;
    uint8_t* sV = smem + Lds<1>::matBytes(KT);
    uint32_t* sMask = reinterpret_cast<uint32_t*>(sV + Lds<1>::matBytes(KT));
    constexpr int kRow = Lds<1>::kRow;

    __shared__ int sLens[kMaxRanked + 1];
    UnitPart const up = unit_of_workgroup(blockIdx.x, gridDim.x, a.qSplit);
    int const part = up.part;
    int const n = up.unit % a.N;
    int const b = pick_sequence<kWavesI8 * kWaveSize>(a, up.unit / a.N, sLens);
    SeqInfo const sq = seq_info(a, b, KT * 64);
    int const nqt = (sq.nq + kQPerWave - 1) / kQPerWave;
    if (part * kWavesI8 >= nqt)
    {
        return; // no query tile for this workgroup
    }
    build_key_mask(a, b, sq.nk, sMask);
    __syncthreads();
    int const nkUsed = used_keys(sMask, sq.nk);
    int const nkb = (nkUsed + 63) >> 6;
    int const ntile = (nkUsed + 15) >> 4; // 16-key tiles that hold at least one key
    stage_kv<1, KT, INTERLEAVED, kWavesI8>(a, sq.seqBaseIn, sq.firstTok, n, nkUsed, nkb, sMask, sK, sV);
    __syncthreads();

    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const lq = lane & 15; // query (column of S^T / O^T)
    int const g = lane >> 4;  // lane group: 16-byte k-chunk of the operands, 4 rows of the accumulators
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);

    // Q^T operand of a tile: 16 bytes d = 16g .. 16g+15 of query 16*qt + lq (zero beyond the
    // sequence).  The next tile's operand is requested while the current tile is computed.
    auto load_q = [&](int qt) -> i32x4 {
        int const qq = qt * kQPerWave + lq;
        i32x4 v = {0, 0, 0, 0};
        if (qq < sq.nq)
        {
            v = *reinterpret_cast<i32x4 const*>(
                src + qkv_chunk_offset<1, INTERLEAVED>(a, sq.seqBaseIn, sq.firstTok, qq, n, 0, g));
        }
        return v;
    };
    int const qtStep = a.qSplit * kWavesI8;
    i32x4 qnext = load_q(part * kWavesI8 + wave);
    for (int qt = part * kWavesI8 + wave; qt < nqt; qt += qtStep)
    {
        int const q = qt * kQPerWave + lq;
        bool const qValid = q < sq.nq;
        i32x4 const qreg = qnext;
        qnext = load_q(qt + qtStep);

        // ---- S^T = K Q^T, biased so that the int32 reads as binary32 12582912 + acc --------
        i32x4 acc[KT * 4];
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
                    if (kb * 4 + u >= ntile)
                    {
                        break; // tiles wholly beyond the sequence are never touched
                    }
                    int const key = kb * 64 + u * 16 + lq;
                    i32x4 const kreg = *reinterpret_cast<i32x4 const*>(sK + key * kRow + swz<1>(key, g) * 16);
                    i32x4 seed = {kMagicBits, kMagicBits, kMagicBits, kMagicBits};
                    if (!full)
                    {
                        asm volatile("" ::: "memory"); // scalar branch, taken for the ragged last block only
                        seed = mask_seed(w0, w1, u, g, kMagicBits);
                    }
                    acc[kb * 4 + u] = __builtin_amdgcn_mfma_i32_16x16x64_i8(kreg, qreg, seed, 0, 0, 0);
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
                            if (key < nkUsed)
                            {
                                a.dbgAcc1[(((int64_t) b * a.N + n) * a.S + q) * a.S + key]
                                    = acc[kb * 4 + u][j] - kMagicBits;
                            }
                        }
                    }
                }
            }
        }

        // ---- row max on the biased integers (the bias is monotone; masked keys hold the
        //      negative pattern of -infinity) ------------------------------------------------------
        int mx = kNegInfBits;
#pragma unroll
        for (int kb = 0; kb < KT; ++kb)
        {
            if (kb < nkb)
            {
#pragma unroll
                for (int u = 0; u < 4; ++u)
                {
                    if (kb * 4 + u >= ntile)
                    {
                        break;
                    }
                    mx = max(mx, max(max(acc[kb * 4 + u][0], acc[kb * 4 + u][1]),
                                     max(acc[kb * 4 + u][2], acc[kb * 4 + u][3])));
                }
            }
        }
        mx = reduce_step<16>(mx, [](int x, int y) { return max(x, y); });
        mx = reduce_step<32>(mx, [](int x, int y) { return max(x, y); });

        // ---- e = 2^((acc - max) * c), row sum; a fully masked row has max = -inf -> all e = 0 --
        float const negK0 = mx == kNegInfBits ? 0.f : -__int_as_float(mx) * a.c;
        float sum = 0.f;
        // e overwrites the accumulators in place (as bit patterns) to keep one row in registers
#pragma unroll
        for (int kb = 0; kb < KT; ++kb)
        {
            if (kb < nkb)
            {
#pragma unroll
                for (int u = 0; u < 4; ++u)
                {
                    if (kb * 4 + u >= ntile)
                    {
                        break;
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        float const ev
                            = __builtin_amdgcn_exp2f(fmaf(__int_as_float(acc[kb * 4 + u][j]), a.c, negK0));
                        acc[kb * 4 + u][j] = __float_as_int(ev);
                        sum += ev;
                    }
                }
            }
        }
        sum = reduce_step<16>(sum, [](float x, float y) { return x + y; });
        sum = reduce_step<32>(sum, [](float x, float y) { return x + y; });
        float const r = sum > 0.f ? a.scaleSoftmax / sum : 0.f;
        // e * r <= scale_softmax: only a scale above 127 can leave the INT8 range; the row is then
        // pre-clamped through e <= 127 / r (one extra op per score on that rare path only)
        if (a.clampP)
        {
            asm volatile("" ::: "memory"); // keep this a scalar branch: the clamp must not be speculated
            float const emax = r > 0.f ? 127.f / r : 0.f;
#pragma unroll
            for (int kb = 0; kb < KT; ++kb)
            {
                if (kb < nkb)
                {
#pragma unroll
                    for (int u = 0; u < 4; ++u)
                    {
                        if (kb * 4 + u >= ntile)
                        {
                            break;
                        }
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                        {
                            acc[kb * 4 + u][j] = __float_as_int(fminf(__int_as_float(acc[kb * 4 + u][j]), emax));
                        }
                    }
                }
            }
        }

        // ---- p8 = rne(e * r) packed four keys to a dword; O^T = V^T P^T -----------------------
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
                i32x4 preg = {0, 0, 0, 0};
#pragma unroll
                for (int u = 0; u < 4; ++u)
                {
                    if (kb * 4 + u >= ntile)
                    {
                        break;
                    }
                    uint32_t yb[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        yb[j] = __float_as_uint(fmaf(__int_as_float(acc[kb * 4 + u][j]), r, kMagic));
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
                            if (key < nkUsed)
                            {
                                a.dbgP8[(((int64_t) b * a.N + n) * a.S + q) * a.S + key]
                                    = (int8_t) ((uint32_t) preg[u] >> (8 * j));
                            }
                        }
                    }
                }
                // V^T operand for head dims 16dt .. 16dt+15: lane r of a group addresses LDS row
                // (8 keys per read: r/2) at byte 16dt + 8(r%2); the transpose read hands lane i
                // the 8 keys of head dim 16dt + i.
                int const vrow = kb * 64 + 8 * g + (lq >> 1);
                uint8_t const* vbase = sV + vrow * kRow + 8 * (lq & 1);
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
                {
                    // rows vrow and vrow + 32 share (row >> 1) & 3, hence the swizzled chunk
                    int const sc = swz<1>(vrow, dt) * 16;
                    i32x2 const v0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*) (vbase + sc));
                    i32x2 const v1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*) (vbase + 32 * kRow + sc));
                    i32x4 const vreg = {v0[0], v0[1], v1[0], v1[1]};
                    oacc[dt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(vreg, preg, oacc[dt], 0, 0, 0);
                }
            }
        }

        // ---- out8 = sat8(rne(acc2 * scale_bmm2)); lane holds d = 16dt + 4g .. +3 of query q, after the transpose
        //      the whole quarter d = 16g .. 16g+15
        uint32_t pk[4];
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
            pk[dt] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
        }
        rows_transpose(pk);
        if (qValid)
        {
            uint8_t* dst = static_cast<uint8_t*>(a.out);
            int const d0 = g * 16;
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
            u32x4 const quarter = {pk[0], pk[1], pk[2], pk[3]};
            *reinterpret_cast<u32x4*>(dst + off) = quarter;
        }
    }
}

// Sequence selection for the var-seqlen kernels with a single trip to global memory: all B+1
// cu_seqlens values go to LDS, sequences are ordered longest first by 16-token bucket (ties by
// index) with a histogram, and the workgroup looks up the sequence at its own position.  Every
// workgroup computes the same order, so no state outside the launch is needed.
constexpr int kLenBuckets = 34; // (length + 15) / 16 for lengths 0 .. 512, and one for longer
struct PickLds
{
    int cu[kMaxRanked + 1];
    int hist[kLenBuckets];
};

__device__ inline int len_bucket(int len)
{
    return min(max(len + 15, 0) >> 4, kLenBuckets - 1);
}

template <int THREADS>
__device__ inline SeqInfo pick_sequence_info(FmhaArgs const& a, int rank, int capacity, PickLds& l, int& bOut)
{
    if (a.cuSeqlens == nullptr || a.B > kMaxRanked || !a.ranked)
    {
        bOut = rank; // fixed layout (equal lengths), too many sequences, or a launch of a single round: natural order
        return seq_info(a, rank, capacity);
    }
    if (threadIdx.x < kLenBuckets)
    {
        l.hist[threadIdx.x] = 0;
    }
    for (int t = threadIdx.x; t <= a.B; t += THREADS)
    {
        l.cu[t] = a.cuSeqlens[t];
    }
    __syncthreads();
    for (int t = threadIdx.x; t < a.B; t += THREADS)
    {
        atomicAdd(&l.hist[len_bucket(l.cu[t + 1] - l.cu[t])], 1);
    }
    __syncthreads();
    // bucket that holds position `rank` (longest bucket first) and the offset inside it: lane k of every wavefront
    // takes bucket k, a prefix sum over the lanes gives the number of sequences in longer buckets, and the bucket is
    // the first one with no more than `rank` sequences above it (one LDS read and a few cross-lane steps instead of
    // a chain of dependent reads, one per bucket)
    int k, off;
    {
        int const lane = threadIdx.x & (kWaveSize - 1);
        int const mine = lane < kLenBuckets ? l.hist[lane] : 0;
        int incl = mine;
#pragma unroll
        for (int d = 1; d < kWaveSize; d *= 2)
        {
            int const up = __shfl_up(incl, d);
            incl += lane >= d ? up : 0;
        }
        int const total = __builtin_amdgcn_readlane(incl, kWaveSize - 1);
        int const above = total - incl; // sequences in buckets longer than this lane's
        uint64_t const fits = __ballot(lane < kLenBuckets && above <= rank);
        k = fits ? (int) __builtin_ctzll(fits) : 0;
        off = rank - __builtin_amdgcn_readlane(above, k);
    }
    // the off-th sequence (by index) of bucket k: every wavefront scans on its own
    int b = a.B - 1;
    int const lane = threadIdx.x & (kWaveSize - 1);
    for (int t0 = 0; t0 < a.B; t0 += kWaveSize)
    {
        int const t = t0 + lane;
        bool const in = t < a.B && len_bucket(l.cu[t + 1] - l.cu[t]) == k;
        uint64_t const m = __ballot(in);
        int const c = __popcll(m);
        if (off < c)
        {
            int const before = __popcll(m & ((1ull << lane) - 1ull));
            uint64_t const hit = __ballot(in && before == off);
            b = t0 + (int) __builtin_ctzll(hit);
            break;
        }
        off -= c;
    }
    bOut = b;
    SeqInfo s;
    int const first = l.cu[b];
    int const len = min(max(l.cu[b + 1] - first, 0), capacity);
    s.firstTok = first;
    s.seqBaseIn = (int64_t) first * a.tokStrideIn;
    s.seqBaseOut = (int64_t) first * a.tokStrideOut;
    s.nq = len;
    s.nk = len;
    return s;
}

// ------------------------------------------------------------------------------------------
// INT8, prefix-valid keys (cu_seqlens or no mask at all): the usual case, specialised on the exact
// number of 64-key blocks so that a query tile is one straight-line instruction stream.
// ------------------------------------------------------------------------------------------

// Stage K and V of one (sequence, head): rows < nk from memory, the rest of the last block zero.
template <int KT, bool INTERLEAVED>
__device__ inline void stage_kv_prefix_i8(FmhaArgs const& a, int64_t seqBase, int64_t firstTok, int n, int nk, int nkb,
    uint8_t* sK, uint8_t* sV)
{
    constexpr int kRowsPerPass = kWavesI8 * kWaveSize / 4;   // 4 chunks of 16 bytes per 64-byte row
    constexpr int kPasses = 64 / kRowsPerPass;
    constexpr int kRow = Lds<1>::kRow;
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);
    int const chunk = threadIdx.x & 3;
    int const rowInPass = threadIdx.x >> 2;
    // one address per matrix for this lane's first row; every further row of the lane is a whole number of tokens
    // further on (the address arithmetic of a layout is done once, not once per load)
    uint8_t const* kSrc = src + qkv_chunk_offset<1, INTERLEAVED>(a, seqBase, firstTok, rowInPass, n, 1, chunk);
    uint8_t const* vSrc = src + qkv_chunk_offset<1, INTERLEAVED>(a, seqBase, firstTok, rowInPass, n, 2, chunk);
    int64_t const tokBytes = INTERLEAVED ? 32 : a.tokStrideIn;
    u32x4 kv[KT][kPasses], vv[KT][kPasses];
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
#pragma unroll
        for (int p = 0; p < kPasses; ++p)
        {
            int const key = kb * 64 + p * kRowsPerPass + rowInPass;
            kv[kb][p] = u32x4{0, 0, 0, 0};
            vv[kb][p] = u32x4{0, 0, 0, 0};
            if (key < nk)
            {
                int64_t const step = (int64_t) (kb * 64 + p * kRowsPerPass) * tokBytes;
                kv[kb][p] = *reinterpret_cast<u32x4 const*>(kSrc + step);
                vv[kb][p] = *reinterpret_cast<u32x4 const*>(vSrc + step);
            }
        }
    }
    // LDS positions: a block is 64 rows further on; the swizzle depends on the row inside the block only
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
#pragma unroll
            for (int p = 0; p < kPasses; ++p)
            {
                int const kk = p * kRowsPerPass + rowInPass;
                int const vk = v_row<1>(kk);
                *reinterpret_cast<u32x4*>(sK + kb * 64 * kRow + kk * kRow + swz<1>(kk, chunk) * 16) = kv[kb][p];
                *reinterpret_cast<u32x4*>(sV + kb * 64 * kRow + vk * kRow + swz<1>(vk, chunk) * 16) = vv[kb][p];
            }
        }
    }
}

// One 16-query tile of a sequence of exactly NKB key blocks (the last one ragged): query tile qt of the sequence sq,
// head n; qreg = the tile's Q^T operand (16 bytes d = 16g .. 16g+15 of query 16 qt + lane % 16, zero beyond the
// sequence).  sK / sV: the head's keys and values in LDS as stage_kv_prefix_i8 lays them out.
template <int NKB, bool INTERLEAVED, bool DEBUG>
__device__ __forceinline__ void tile_i8(FmhaArgs const& a, SeqInfo const& sq, int const b, int const n, int const qt,
    uint8_t const* sK, uint8_t const* sV, i32x4 const qreg)
{
    constexpr int kRow = Lds<1>::kRow;
    constexpr int NT = NKB * 4;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const lq = lane & 15;
    int const g = lane >> 4;

    // last block: keys 64(NKB-1) + 16u + 4g + j exist for (16u + 4g + j) < lastKeys
    int const lastKeys = sq.nk - (NKB - 1) * 64;
    int const lastTiles = (lastKeys + 15) >> 4;
    i32x4 const seedFull = {kMagicBits, kMagicBits, kMagicBits, kMagicBits};
    int const lastRel = lastKeys - 4 * g; // key 16u + j of this lane group exists iff 16u + j < lastRel

    int const q = qt * kQPerWave + lq;
    bool const qValid = q < sq.nq;

    // ---- S^T = K Q^T; the int32 result reads as binary32 12582912 + acc, -inf for absent keys
    i32x4 acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t)
    {
        int const key = t * 16 + lq;
        i32x4 const kreg = *reinterpret_cast<i32x4 const*>(sK + key * kRow + swz<1>(key, g) * 16);
        i32x4 seed = seedFull;
        if (t >= NT - 4)
        {
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                seed[j] = (16 * (t & 3) + j) < lastRel ? kMagicBits : kNegInfBits;
            }
        }
        acc[t] = attention_mfma_i8(kreg, qreg, seed);
    }
    __builtin_amdgcn_sched_barrier(0);

    if (DEBUG && a.dbgAcc1 && qValid)
    {
        for (int t = 0; t < NT; ++t)
        {
            for (int j = 0; j < 4; ++j)
            {
                int const key = t * 16 + g * 4 + j;
                if (key < sq.nk)
                {
                    a.dbgAcc1[(((int64_t) b * a.N + n) * a.S + q) * a.S + key] = acc[t][j] - kMagicBits;
                }
            }
        }
    }

    // ---- row max on the biased integers (monotone in the score; -inf is a negative pattern)
    // two chains of three-input maxima (v_max3_i32): one instruction per two scores
    int mxA = kNegInfBits, mxB = kNegInfBits;
#pragma unroll
    for (int t = 0; t < NT; ++t)
    {
        mxA = max(max(mxA, acc[t][0]), acc[t][1]);
        mxB = max(max(mxB, acc[t][2]), acc[t][3]);
    }
    int mx = max(mxA, mxB);
    mx = reduce_step<16>(mx, [](int x, int y) { return max(x, y); });
    mx = reduce_step<32>(mx, [](int x, int y) { return max(x, y); });
    __builtin_amdgcn_sched_barrier(0);

    // ---- e = 2^((acc - max) * c) in place, row sum
    float const negK0 = -__int_as_float(mx) * a.c;
    float sum0 = 0.f, sum1 = 0.f;
#pragma unroll
    for (int t = 0; t < NT; ++t)
    {
        if ((t & 3) == 0)
        {
            __builtin_amdgcn_sched_barrier(0); // bound the live temporaries to one key block
        }
        if (t >= NT - 4 && (t & 3) >= lastTiles)
        {
            continue; // tile without keys: its accumulators keep the -inf pattern (p8 = 0 below)
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            float const ev = __builtin_amdgcn_exp2f(fmaf(__int_as_float(acc[t][j]), a.c, negK0));
            acc[t][j] = __float_as_int(ev);
            if (j & 1)
            {
                sum1 += ev;
            }
            else
            {
                sum0 += ev;
            }
        }
    }
    float sum = sum0 + sum1;
    sum = reduce_step<16>(sum, [](float x, float y) { return x + y; });
    sum = reduce_step<32>(sum, [](float x, float y) { return x + y; });
    float const r = a.scaleSoftmax / sum;   // sum >= 1: the row maximum contributes 2^0

    // ---- p8 = rne(e * r), four keys to a dword; O^T = V^T P^T
    i32x4 oacc[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
    {
        oacc[dt] = i32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb)
    {
        __builtin_amdgcn_sched_barrier(0);
        i32x4 preg = {0, 0, 0, 0};
#pragma unroll
        for (int u = 0; u < 4; ++u)
        {
            if (kb == NKB - 1 && u >= lastTiles)
            {
                continue;
            }
            uint32_t yb[4];
#pragma unroll
            for (int j = 0; j < 4; ++j)
            {
                yb[j] = __float_as_uint(fmaf(__int_as_float(acc[kb * 4 + u][j]), r, kMagic));
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
        int const vrow = kb * 64 + 8 * g + (lq >> 1);
        uint8_t const* vbase = sV + vrow * kRow + 8 * (lq & 1);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
        {
            int const sc = swz<1>(vrow, dt) * 16;
            i32x2 const v0 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*) (vbase + sc));
            i32x2 const v1 = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_i32x2*) (vbase + 32 * kRow + sc));
            i32x4 const vreg = {v0[0], v0[1], v1[0], v1[1]};
            oacc[dt] = attention_mfma_i8(vreg, preg, oacc[dt]);
        }
    }

    // ---- out8 = sat8(rne(acc2 * scale_bmm2)): binary32 product (rounded on its own, not fused
    //      into the add), rounded to an integer through the magic constant, clamped on the bit
    //      patterns (monotone for the positive results; anything negative is below the range).
    //      Lane (g, query) then holds bytes 4g..4g+3 of each 16-byte quarter dt of the query's row; a 4 x 4
    //      transpose over the four rows of 16 lanes (v_permlane32_swap, v_permlane16_swap) leaves it with the
    //      whole quarter dt = g, which goes out as one 16-byte store.
    uint32_t pk[4];
#pragma unroll
    for (int dt = 0; dt < 4; ++dt)
    {
        uint32_t yb[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
        {
            int const bits = __float_as_int(mul_rounded((float) oacc[dt][j], a.scaleBmm2) + kMagic);
            yb[j] = (uint32_t) min(max(bits, kMagicBits - 128), kMagicBits + 127);
        }
        uint32_t const lo = __builtin_amdgcn_perm(yb[1], yb[0], 0x0c0c0400u);
        uint32_t const hi = __builtin_amdgcn_perm(yb[3], yb[2], 0x0c0c0400u);
        pk[dt] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
    }
    rows_transpose(pk);
    if (qValid)
    {
        uint8_t* dst = static_cast<uint8_t*>(a.out);
        int const d0 = g * 16;
        int64_t off;
        if (INTERLEAVED)
        {
            off = (((int64_t) n * 2 + (d0 >> 5)) * a.total + sq.firstTok + q) * 32 + (d0 & 31);
        }
        else
        {
            off = sq.seqBaseOut + (int64_t) q * a.tokStrideOut + (int64_t) n * kHeadSize + d0;
        }
        u32x4 const quarter = {pk[0], pk[1], pk[2], pk[3]};
        *reinterpret_cast<u32x4*>(dst + off) = quarter;
    }
}

// Q^T operand of query tile qt (see tile_i8).
template <bool INTERLEAVED>
__device__ __forceinline__ i32x4 load_q_i8(FmhaArgs const& a, SeqInfo const& sq, int const n, int const qt)
{
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const qq = qt * kQPerWave + (lane & 15);
    i32x4 v = {0, 0, 0, 0};
    if (qq < sq.nq)
    {
        v = *reinterpret_cast<i32x4 const*>(static_cast<uint8_t const*>(a.qkv)
            + qkv_chunk_offset<1, INTERLEAVED>(a, sq.seqBaseIn, sq.firstTok, qq, n, 0, lane >> 4));
    }
    return v;
}

// All query tiles of this wavefront for a sequence of exactly NKB key blocks.
template <int NKB, bool INTERLEAVED, bool DEBUG>
__device__ __forceinline__ void attend_i8(FmhaArgs const& a, SeqInfo const& sq, int const b, int const n,
    int const qtBegin, int const qtEnd, uint8_t const* sK, uint8_t const* sV, i32x4 const qFirst)
{
    int const wave = threadIdx.x >> 6;
    constexpr int qtStep = kWavesI8;
    i32x4 qnext = qFirst; // requested by the caller together with K and V
    for (int qt = qtBegin + wave; qt < qtEnd; qt += qtStep)
    {
        i32x4 const qreg = qnext;
        qnext = load_q_i8<INTERLEAVED>(a, sq, n, qt + qtStep);
        tile_i8<NKB, INTERLEAVED, DEBUG>(a, sq, b, n, qt, sK, sV, qreg);
    }
}

template <int KT, bool INTERLEAVED, bool DEBUG>
__global__ __launch_bounds__(kWavesI8* kWaveSize) __attribute__((amdgpu_waves_per_eu(KT <= 6 ? 3 : 2))) void fmha_i8_prefix_kernel(FmhaArgs const a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sK = smem;
    uint8_t* sV = smem + Lds<1>::matBytes(KT);
    __shared__ PickLds sPick;
    UnitPart up = unit_of_workgroup(blockIdx.x, gridDim.x, a.qSplit);
    if (!INTERLEAVED && a.qSplit == 1 && (a.N & 1) == 0)
    {
        // Linear layout ([token][head][Q K V][64 bytes]): V of head n and Q of head n + 1 lie in one 128-byte line, so
        // the two heads of a pair go to one XCD (18239 tokens x 16 heads: 36.2 -> 35.2 us)
        UnitPart const pair = unit_of_workgroup(blockIdx.x, gridDim.x, 2);
        up.unit = pair.unit * 2u + (uint32_t) pair.part;
    }
    int const part = up.part;
    int const n = up.unit % a.N;
    int b;
    SeqInfo const sq = pick_sequence_info<kWavesI8 * kWaveSize>(a, up.unit / a.N, KT * 64, sPick, b);
    // contiguous tile ranges, each a multiple of one round of the workgroup's wavefronts
    int const nqt = (sq.nq + kQPerWave - 1) / kQPerWave;
    int const per = kWavesI8 * ((nqt + kWavesI8 * a.qSplit - 1) / (kWavesI8 * a.qSplit));
    int const qtBegin = min(part * per, nqt);
    int const qtEnd = min(qtBegin + per, nqt);
    if (qtBegin >= qtEnd)
    {
        return; // no query tile for this workgroup (also: empty sequence)
    }
    int const nkb = (sq.nk + 63) >> 6;
    // the first query tile of this wavefront travels with K and V
    i32x4 qFirst = {0, 0, 0, 0};
    {
        int const qq = (qtBegin + (int) (threadIdx.x >> 6)) * kQPerWave + (int) (threadIdx.x & 15);
        if (qq < sq.nq && qtBegin + (int) (threadIdx.x >> 6) < qtEnd)
        {
            qFirst = *reinterpret_cast<i32x4 const*>(static_cast<uint8_t const*>(a.qkv)
                + qkv_chunk_offset<1, INTERLEAVED>(a, sq.seqBaseIn, sq.firstTok, qq, n, 0, (threadIdx.x & 63) >> 4));
        }
    }
    stage_kv_prefix_i8<KT, INTERLEAVED>(a, sq.seqBaseIn, sq.firstTok, n, sq.nk, nkb, sK, sV);
    __syncthreads();
    switch (nkb)
    {
    case 1: attend_i8<1, INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst); break;
    case 2:
        if (KT >= 2) attend_i8<(KT >= 2 ? 2 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    case 3:
        if (KT >= 3) attend_i8<(KT >= 3 ? 3 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    case 4:
        if (KT >= 4) attend_i8<(KT >= 4 ? 4 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    case 5:
        if (KT >= 5) attend_i8<(KT >= 5 ? 5 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    case 6:
        if (KT >= 6) attend_i8<(KT >= 6 ? 6 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    case 7:
        if (KT >= 7) attend_i8<(KT >= 7 ? 7 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    case 8:
        if (KT >= 8) attend_i8<(KT >= 8 ? 8 : 1), INTERLEAVED, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst);
        break;
    default: break;
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
    uint8_t* sV = smem + Lds<2>::matBytes(KT);
    uint32_t* sMask = reinterpret_cast<uint32_t*>(sV + Lds<2>::matBytes(KT));
    constexpr int kRow = Lds<2>::kRow;

    __shared__ int sLens[kMaxRanked + 1];
    UnitPart const up = unit_of_workgroup(blockIdx.x, gridDim.x, a.qSplit);
    int const part = up.part;
    int const n = up.unit % a.N;
    int const b = pick_sequence<kWavesF16 * kWaveSize>(a, up.unit / a.N, sLens);
    SeqInfo const sq = seq_info(a, b, KT * 64);
    int const nqt = (sq.nq + kQPerWave - 1) / kQPerWave;
    if (part * kWavesF16 >= nqt)
    {
        return;
    }
    build_key_mask(a, b, sq.nk, sMask);
    __syncthreads();
    int const nkUsed = used_keys(sMask, sq.nk);
    int const nkb = (nkUsed + 63) >> 6;
    stage_kv<2, KT, false, kWavesF16>(a, sq.seqBaseIn, sq.firstTok, n, nkUsed, nkb, sMask, sK, sV);
    __syncthreads();

    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const lq = lane & 15;
    int const g = lane >> 4;
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);
    f16x8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        ones[i] = (f16) 1.f;
    }

    // Q^T operands of a tile: MFMA h covers d = 32h + 8g .. +7 of query 16*qt + lq.  The next
    // tile's operands are requested while the current tile is computed.
    auto load_q = [&](int qt, int h) -> f16x8 {
        int const qq = qt * kQPerWave + lq;
        u32x4 raw = {0, 0, 0, 0};
        if (qq < sq.nq)
        {
            raw = *reinterpret_cast<u32x4 const*>(
                src + qkv_chunk_offset<2, false>(a, sq.seqBaseIn, sq.firstTok, qq, n, 0, h * 4 + g));
        }
        return __builtin_bit_cast(f16x8, raw);
    };
    int const qtStep = a.qSplit * kWavesF16;
    f16x8 qnext[2] = {load_q(part * kWavesF16 + wave, 0), load_q(part * kWavesF16 + wave, 1)};
    for (int qt = part * kWavesF16 + wave; qt < nqt; qt += qtStep)
    {
        int const q = qt * kQPerWave + lq;
        bool const qValid = q < sq.nq;
        f16x8 const qreg[2] = {qnext[0], qnext[1]};
        qnext[0] = load_q(qt + qtStep, 0);
        qnext[1] = load_q(qt + qtStep, 1);

        // ---- S^T = K Q^T (binary32 accumulation) -----------------------------------------------
        f32x4 acc[KT * 4];
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
                    int const key = kb * 64 + u * 16 + lq;
                    f32x4 s = {0.f, 0.f, 0.f, 0.f};
                    if (!full)
                    {
                        asm volatile("" ::: "memory"); // scalar branch, taken for the ragged last block only
                        s = __builtin_bit_cast(f32x4, mask_seed(w0, w1, u, g, 0));
                    }
#pragma unroll
                    for (int h = 0; h < 2; ++h)
                    {
                        f16x8 const kreg
                            = *reinterpret_cast<f16x8 const*>(sK + key * kRow + swz<2>(key, h * 4 + g) * 16);
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
                            if (key < nkUsed)
                            {
                                a.dbgAcc1[(((int64_t) b * a.N + n) * a.S + q) * a.S + key]
                                    = __float_as_int(acc[kb * 4 + u][j]);
                            }
                        }
                    }
                }
            }
        }

        // ---- row max (masked keys hold -infinity) ------------------------------------------------
        float mx = -__builtin_inff();
#pragma unroll
        for (int kb = 0; kb < KT; ++kb)
        {
            if (kb < nkb)
            {
#pragma unroll
                for (int u = 0; u < 4; ++u)
                {
                    mx = fmaxf(mx, fmaxf(fmaxf(acc[kb * 4 + u][0], acc[kb * 4 + u][1]),
                                         fmaxf(acc[kb * 4 + u][2], acc[kb * 4 + u][3])));
                }
            }
        }
        mx = reduce_step<16>(mx, [](float x, float y) { return fmaxf(x, y); });
        mx = reduce_step<32>(mx, [](float x, float y) { return fmaxf(x, y); });

        // ---- p = 2^((s - max) * c) rounded to binary16; O^T = V^T P^T; the row sum is taken by
        //      the matrix unit as well (a tile of ones), so numerator and denominator see the
        //      same rounded probabilities ---------------------------------------------------------
        float const negK0 = mx == -__builtin_inff() ? 0.f : -mx * a.c; // fully masked row: every p = 0
        f32x4 oacc[4];
        f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
        {
            oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int kb = 0; kb < KT; ++kb)
        {
            if (kb < nkb)
            {
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
                            p[j] = __builtin_amdgcn_exp2f(fmaf(acc[t][j], a.c, negK0));
                        }
                        f16x2 const p01 = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(p[0], p[1]));
                        f16x2 const p23 = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(p[2], p[3]));
                        preg[w * 4 + 0] = p01[0];
                        preg[w * 4 + 1] = p01[1];
                        preg[w * 4 + 2] = p23[0];
                        preg[w * 4 + 3] = p23[1];
                    }
                    // V^T operand: lane r of a group addresses LDS row (4 keys per read: r/4) at
                    // halfword 16dt + 4(r%4); the transpose read hands lane i the 4 keys of head
                    // dim 16dt + i.  Slots 0..3 = keys 16(2hb)+4g.., slots 4..7 = keys 16(2hb+1)+4g..
                    int const vrow = kb * 64 + hb * 32 + 4 * g + (lq >> 2);
                    uint8_t const* vbase = sV + vrow * kRow + 8 * (lq & 1);
#pragma unroll
                    for (int dt = 0; dt < 4; ++dt)
                    {
                        // rows vrow and vrow + 16 share row & 7, hence the swizzled chunk
                        int const sc = swz<2>(vrow, 2 * dt + ((lq >> 1) & 1)) * 16;
                        i16x4 const v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) (vbase + sc));
                        i16x4 const v1
                            = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) (vbase + 16 * kRow + sc));
                        typedef short i16x8 __attribute__((ext_vector_type(8)));
                        i16x8 const both = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                        oacc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            __builtin_bit_cast(f16x8, both), preg, oacc[dt], 0, 0, 0);
                    }
                    sacc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ones, preg, sacc, 0, 0, 0);
                }
            }
        }

        {
            float const rinv = sacc[0] > 0.f ? 1.f / sacc[0] : 0.f;
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
            {
                f16x4 y;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    y[j] = (f16) (oacc[dt][j] * rinv);
                }
                u32x2 const w = __builtin_bit_cast(u32x2, y);
                lo[dt] = w[0];
                hi[dt] = w[1];
            }
            rows_transpose(lo);
            rows_transpose(hi);
            if (qValid)
            {
                uint8_t* dst = static_cast<uint8_t*>(a.out);
                int64_t const off
                    = sq.seqBaseOut + (int64_t) q * a.tokStrideOut + ((int64_t) n * kHeadSize + g * 16) * 2;
                u32x4 const first = {lo[0], hi[0], lo[1], hi[1]};
                u32x4 const second = {lo[2], hi[2], lo[3], hi[3]};
                *reinterpret_cast<u32x4*>(dst + off) = first;
                *reinterpret_cast<u32x4*>(dst + off + 16) = second;
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// FP16, prefix-valid keys: same specialisation on the number of 64-key blocks as the INT8 kernel.
// ------------------------------------------------------------------------------------------

template <int KT>
__device__ inline void stage_kv_prefix_f16(FmhaArgs const& a, int64_t seqBase, int64_t firstTok, int n, int nk,
    int nkb, uint8_t* sK, uint8_t* sV)
{
    constexpr int kRowsPerPass = kWavesF16 * kWaveSize / 8;   // 8 chunks of 16 bytes per 128-byte row
    constexpr int kPasses = 64 / kRowsPerPass;
    constexpr int kRow = Lds<2>::kRow;
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);
    int const chunk = threadIdx.x & 7;
    int const rowInPass = threadIdx.x >> 3;
    u32x4 kv[KT][kPasses], vv[KT][kPasses];
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
#pragma unroll
        for (int p = 0; p < kPasses; ++p)
        {
            int const key = kb * 64 + p * kRowsPerPass + rowInPass;
            kv[kb][p] = u32x4{0, 0, 0, 0};
            vv[kb][p] = u32x4{0, 0, 0, 0};
            if (key < nk)
            {
                kv[kb][p] = *reinterpret_cast<u32x4 const*>(
                    src + qkv_chunk_offset<2, false>(a, seqBase, firstTok, key, n, 1, chunk));
                vv[kb][p] = *reinterpret_cast<u32x4 const*>(
                    src + qkv_chunk_offset<2, false>(a, seqBase, firstTok, key, n, 2, chunk));
            }
        }
    }
#pragma unroll
    for (int kb = 0; kb < KT; ++kb)
    {
        if (kb < nkb)
        {
#pragma unroll
            for (int p = 0; p < kPasses; ++p)
            {
                int const kk = p * kRowsPerPass + rowInPass;
                int const kr = kb * 64 + kk;
                int const vr = kb * 64 + v_row<2>(kk);
                *reinterpret_cast<u32x4*>(sK + kr * kRow + swz<2>(kr, chunk) * 16) = kv[kb][p];
                *reinterpret_cast<u32x4*>(sV + vr * kRow + swz<2>(vr, chunk) * 16) = vv[kb][p];
            }
        }
    }
}

template <int NKB, bool DEBUG>
__device__ __forceinline__ void attend_f16(FmhaArgs const& a, SeqInfo const& sq, int const b, int const n,
    int const qtBegin, int const qtEnd, uint8_t const* sK, uint8_t const* sV, f16x8 const qFirst0,
    f16x8 const qFirst1)
{
    constexpr int kRow = Lds<2>::kRow;
    constexpr int NT = NKB * 4;
    int const lane = threadIdx.x & (kWaveSize - 1);
    int const wave = threadIdx.x >> 6;
    int const lq = lane & 15;
    int const g = lane >> 4;
    uint8_t const* src = static_cast<uint8_t const*>(a.qkv);
    f16x8 ones;
#pragma unroll
    for (int i = 0; i < 8; ++i)
    {
        ones[i] = (f16) 1.f;
    }
    int const lastKeys = sq.nk - (NKB - 1) * 64;
    int const lastHalves = (lastKeys + 31) >> 5;   // 32-key halves of the last block that hold keys
    int const lastRel = lastKeys - 4 * g;          // key 16u + j of this lane group exists iff 16u + j < lastRel

    auto load_q = [&](int qt, int h) -> f16x8 {
        int const qq = qt * kQPerWave + lq;
        u32x4 raw = {0, 0, 0, 0};
        if (qq < sq.nq)
        {
            raw = *reinterpret_cast<u32x4 const*>(
                src + qkv_chunk_offset<2, false>(a, sq.seqBaseIn, sq.firstTok, qq, n, 0, h * 4 + g));
        }
        return __builtin_bit_cast(f16x8, raw);
    };
    f16x8 qnext[2] = {qFirst0, qFirst1};
    for (int qt = qtBegin + wave; qt < qtEnd; qt += kWavesF16)
    {
        int const q = qt * kQPerWave + lq;
        bool const qValid = q < sq.nq;
        f16x8 const qreg[2] = {qnext[0], qnext[1]};
        qnext[0] = load_q(qt + kWavesF16, 0);
        qnext[1] = load_q(qt + kWavesF16, 1);

        // ---- S^T = K Q^T (binary32 accumulation); absent keys start from -infinity
        f32x4 acc[NT];
#pragma unroll
        for (int t = 0; t < NT; ++t)
        {
            int const key = t * 16 + lq;
            f32x4 sd = {0.f, 0.f, 0.f, 0.f};
            if (t >= NT - 4)
            {
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    sd[j] = (16 * (t & 3) + j) < lastRel ? 0.f : -__builtin_inff();
                }
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
            {
                f16x8 const kreg = *reinterpret_cast<f16x8 const*>(sK + key * kRow + swz<2>(key, h * 4 + g) * 16);
                sd = attention_mfma_f16(kreg, qreg[h], sd);
            }
            acc[t] = sd;
        }
        __builtin_amdgcn_sched_barrier(0);

        if (DEBUG && a.dbgAcc1 && qValid)
        {
            for (int t = 0; t < NT; ++t)
            {
                for (int j = 0; j < 4; ++j)
                {
                    int const key = t * 16 + g * 4 + j;
                    if (key < sq.nk)
                    {
                        a.dbgAcc1[(((int64_t) b * a.N + n) * a.S + q) * a.S + key] = __float_as_int(acc[t][j]);
                    }
                }
            }
        }

        // ---- row max
        float mxA = -__builtin_inff(), mxB = -__builtin_inff();
#pragma unroll
        for (int t = 0; t < NT; ++t)
        {
            mxA = fmaxf(fmaxf(mxA, acc[t][0]), acc[t][1]);
            mxB = fmaxf(fmaxf(mxB, acc[t][2]), acc[t][3]);
        }
        float mx = fmaxf(mxA, mxB);
        mx = reduce_step<16>(mx, [](float x, float y) { return fmaxf(x, y); });
        mx = reduce_step<32>(mx, [](float x, float y) { return fmaxf(x, y); });
        __builtin_amdgcn_sched_barrier(0);

        // ---- p = 2^((s - max) * c) rounded to binary16; O^T = V^T P^T; row sum by a tile of ones
        float const negK0 = -mx * a.c; // nk >= 1: the maximum is finite
        f32x4 oacc[4];
        f32x4 sacc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
        {
            oacc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
        {
#pragma unroll
            for (int hb = 0; hb < 2; ++hb)
            {
                if (kb == NKB - 1 && hb >= lastHalves)
                {
                    continue; // no key in this half
                }
                __builtin_amdgcn_sched_barrier(0);
                f16x8 preg;
#pragma unroll
                for (int w = 0; w < 2; ++w)
                {
                    int const t = kb * 4 + hb * 2 + w;
                    float pr[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                    {
                        pr[j] = __builtin_amdgcn_exp2f(fmaf(acc[t][j], a.c, negK0));
                    }
                    f16x2 const p01 = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(pr[0], pr[1]));
                    f16x2 const p23 = __builtin_bit_cast(f16x2, __builtin_amdgcn_cvt_pkrtz(pr[2], pr[3]));
                    preg[w * 4 + 0] = p01[0];
                    preg[w * 4 + 1] = p01[1];
                    preg[w * 4 + 2] = p23[0];
                    preg[w * 4 + 3] = p23[1];
                }
                int const vrow = kb * 64 + hb * 32 + 4 * g + (lq >> 2);
                uint8_t const* vbase = sV + vrow * kRow + 8 * (lq & 1);
#pragma unroll
                for (int dt = 0; dt < 4; ++dt)
                {
                    int const sc = swz<2>(vrow, 2 * dt + ((lq >> 1) & 1)) * 16;
                    i16x4 const v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) (vbase + sc));
                    i16x4 const v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_i16x4*) (vbase + 16 * kRow + sc));
                    typedef short i16x8 __attribute__((ext_vector_type(8)));
                    i16x8 const both = {v0[0], v0[1], v0[2], v0[3], v1[0], v1[1], v1[2], v1[3]};
                    oacc[dt] = attention_mfma_f16(__builtin_bit_cast(f16x8, both), preg, oacc[dt]);
                }
                sacc = attention_mfma_f16(ones, preg, sacc);
            }
        }

        // Lane (g, query) holds 8 bytes of each 32-byte quarter dt of the query's 128-byte row; a 4 x 4 transpose over
        // the four rows of 16 lanes (v_permlane32_swap, v_permlane16_swap, once for each dword) leaves it with the
        // whole quarter dt = g, which goes out as two 16-byte stores.
        {
            float const rinv = 1.f / sacc[0];
            uint32_t lo[4], hi[4];
#pragma unroll
            for (int dt = 0; dt < 4; ++dt)
            {
                f16x4 y;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                {
                    y[j] = (f16) (oacc[dt][j] * rinv);
                }
                u32x2 const w = __builtin_bit_cast(u32x2, y);
                lo[dt] = w[0];
                hi[dt] = w[1];
            }
            rows_transpose(lo);
            rows_transpose(hi);
            if (qValid)
            {
                uint8_t* dst = static_cast<uint8_t*>(a.out);
                int64_t const off
                    = sq.seqBaseOut + (int64_t) q * a.tokStrideOut + ((int64_t) n * kHeadSize + g * 16) * 2;
                u32x4 const first = {lo[0], hi[0], lo[1], hi[1]};
                u32x4 const second = {lo[2], hi[2], lo[3], hi[3]};
                *reinterpret_cast<u32x4*>(dst + off) = first;
                *reinterpret_cast<u32x4*>(dst + off + 16) = second;
            }
        }
    }
}

template <int KT, bool DEBUG>
__global__ __launch_bounds__(kWavesF16* kWaveSize) void fmha_f16_prefix_kernel(FmhaArgs const a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    uint8_t* sK = smem;
    uint8_t* sV = smem + Lds<2>::matBytes(KT);
    __shared__ PickLds sPick;
    UnitPart const up = unit_of_workgroup(blockIdx.x, gridDim.x, a.qSplit);
    int const part = up.part;
    int const n = up.unit % a.N;
    int b;
    SeqInfo const sq = pick_sequence_info<kWavesF16 * kWaveSize>(a, up.unit / a.N, KT * 64, sPick, b);
    int const nqt = (sq.nq + kQPerWave - 1) / kQPerWave;
    int const per = kWavesF16 * ((nqt + kWavesF16 * a.qSplit - 1) / (kWavesF16 * a.qSplit));
    int const qtBegin = min(part * per, nqt);
    int const qtEnd = min(qtBegin + per, nqt);
    if (qtBegin >= qtEnd)
    {
        return;
    }
    int const nkb = (sq.nk + 63) >> 6;
    f16x8 qFirst[2];
    {
        int const qt = qtBegin + (int) (threadIdx.x >> 6);
        int const qq = qt * kQPerWave + (int) (threadIdx.x & 15);
#pragma unroll
        for (int h = 0; h < 2; ++h)
        {
            u32x4 raw = {0, 0, 0, 0};
            if (qq < sq.nq && qt < qtEnd)
            {
                raw = *reinterpret_cast<u32x4 const*>(static_cast<uint8_t const*>(a.qkv)
                    + qkv_chunk_offset<2, false>(a, sq.seqBaseIn, sq.firstTok, qq, n, 0,
                        h * 4 + (int) ((threadIdx.x & 63) >> 4)));
            }
            qFirst[h] = __builtin_bit_cast(f16x8, raw);
        }
    }
    stage_kv_prefix_f16<KT>(a, sq.seqBaseIn, sq.firstTok, n, sq.nk, nkb, sK, sV);
    __syncthreads();
    switch (nkb)
    {
    case 1: attend_f16<1, DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]); break;
    case 2:
        if (KT >= 2) attend_f16<(KT >= 2 ? 2 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    case 3:
        if (KT >= 3) attend_f16<(KT >= 3 ? 3 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    case 4:
        if (KT >= 4) attend_f16<(KT >= 4 ? 4 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    case 5:
        if (KT >= 5) attend_f16<(KT >= 5 ? 5 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    case 6:
        if (KT >= 6) attend_f16<(KT >= 6 ? 6 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    case 7:
        if (KT >= 7) attend_f16<(KT >= 7 ? 7 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    case 8:
        if (KT >= 8) attend_f16<(KT >= 8 ? 8 : 1), DEBUG>(a, sq, b, n, qtBegin, qtEnd, sK, sV, qFirst[0], qFirst[1]);
        break;
    default: break;
    }
}

// ------------------------------------------------------------------------------------------
// host side
// ------------------------------------------------------------------------------------------

// Raising the dynamic LDS limit is a per-function attribute, set once per process and kernel: at the first launch,
// or ahead of it by trtamd_fused_mha_prepare.
int ensure_lds(void const* key, char const* name, int ldsBytes)
{
    static std::mutex mtx;
    static std::vector<void const*> done;
    std::lock_guard<std::mutex> lock(mtx);
    for (void const* p : done)
    {
        if (p == key)
        {
            return TRTAMD_STATUS_SUCCESS;
        }
    }
    hipError_t const e = hipFuncSetAttribute(key, hipFuncAttributeMaxDynamicSharedMemorySize, ldsBytes);
    if (e != hipSuccess)
    {
        (void) hipGetLastError();
        return set_error(TRTAMD_STATUS_FAILURE, "%s: cannot reserve %d bytes of LDS: %s", name, ldsBytes,
            hipGetErrorString(e));
    }
    done.push_back(key);
    return TRTAMD_STATUS_SUCCESS;
}

template <typename K>
int launch_fmha(K kernel, char const* name, hipStream_t stream, FmhaArgs const& args, int ldsBytes, int waves)
{
    int const st = ensure_lds(reinterpret_cast<void const*>(kernel), name, ldsBytes);
    if (st != TRTAMD_STATUS_SUCCESS)
    {
        return st;
    }
    unsigned const blocks = (unsigned) args.B * args.N * args.qSplit;
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
    // keys are a valid prefix (cu_seqlens, or no mask) and probabilities cannot leave the INT8 range:
    // the kernel specialised on the number of key blocks serves the launch
    int const noFast = tuning(Tuning::kFmhaGeneric);
    if (a.packedMask == nullptr && !a.clampP && !noFast)
    {
#define TRTAMD_I8P(KT)                                                                                                 \
    case KT:                                                                                                           \
        return interleaved ? launch_fmha(fmha_i8_prefix_kernel<KT, true, DEBUG>, "fmha_i8_prefix_interleaved", stream, \
                   a, Lds<1>::total(KT), kWavesI8)                                                                     \
                           : launch_fmha(fmha_i8_prefix_kernel<KT, false, DEBUG>, "fmha_i8_prefix", stream, a,         \
                               Lds<1>::total(KT), kWavesI8)
        switch (kt)
        {
            TRTAMD_I8P(1);
            TRTAMD_I8P(2);
            TRTAMD_I8P(3);
            TRTAMD_I8P(4);
            TRTAMD_I8P(6);
            TRTAMD_I8P(8);
        default: break;
        }
#undef TRTAMD_I8P
    }
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
    int const noFast = tuning(Tuning::kFmhaGeneric);
    if (a.packedMask == nullptr && !noFast)
    {
#define TRTAMD_F16P(KT)                                                                                                \
    case KT:                                                                                                           \
        return launch_fmha(fmha_f16_prefix_kernel<KT, DEBUG>, "fmha_f16_prefix", stream, a, Lds<2>::total(KT), kWavesF16)
        switch (kt)
        {
            TRTAMD_F16P(1);
            TRTAMD_F16P(2);
            TRTAMD_F16P(3);
            TRTAMD_F16P(4);
            TRTAMD_F16P(6);
            TRTAMD_F16P(8);
        default: break;
        }
#undef TRTAMD_F16P
    }
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

// Every shipped kernel's LDS reservation, so that no later launch has anything to set up.
template <int KT>
int prepare_kt()
{
    int st = ensure_lds(reinterpret_cast<void const*>(fmha_i8_prefix_kernel<KT, true, false>), "fmha_i8_prefix_interleaved",
        Lds<1>::total(KT));

    st = st ? st : ensure_lds(reinterpret_cast<void const*>(fmha_i8_prefix_kernel<KT, false, false>), "fmha_i8_prefix",
                      Lds<1>::total(KT));
    st = st ? st : ensure_lds(reinterpret_cast<void const*>(fmha_i8_kernel<KT, true, false>), "fmha_i8_interleaved",
                      Lds<1>::total(KT));
    st = st ? st : ensure_lds(reinterpret_cast<void const*>(fmha_i8_kernel<KT, false, false>), "fmha_i8", Lds<1>::total(KT));
    st = st ? st : ensure_lds(reinterpret_cast<void const*>(fmha_f16_prefix_kernel<KT, false>), "fmha_f16_prefix",
                      Lds<2>::total(KT));
    st = st ? st : ensure_lds(reinterpret_cast<void const*>(fmha_f16_kernel<KT, false>), "fmha_f16", Lds<2>::total(KT));
    return st;
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
    {
        // Workgroups per (sequence, head).  Every extra workgroup stages K and V again, so a unit is only shared
        // while the launch would otherwise leave the chip partly idle or badly balanced.  INT8 (three workgroups per
        // CU, 768 places): below 896 units two workgroups per unit, which also evens out a single round of units of
        // very different lengths (768 units of 128-384 keys: 24.9 against 27.8 us; 512 units: 18.7 against 23.1 us;
        // 896 units: 29.1 against 28.1 us), and more of them only to reach one round (256 units: three, 12.6 us
        // against 13.1 with two and 17.4 with one; at most four).  FP16 (its K and V take most of a CU's LDS, one
        // workgroup per CU, and staging them is 40 % of a workgroup's time): only below 160 units (192 units of 192-384
        // keys: 15.3 us alone, 17.5 us shared by two; 144 units: 14.9 against 12.9 us).
        int const waves = dataType == 2 ? kWavesI8 : kWavesF16;
        int const maxSplit = std::max(1, ceil_div(ceil_div(p->s, kQPerWave), waves));
        int64_t const heads = (int64_t) p->b * p->h;
        int split = 1;
        if (dataType == 2)
        {
            split = heads >= 896 ? 1 : (int) std::max<int64_t>(2, std::min<int64_t>(4, ceil_div<int64_t>(768, heads)));
        }
        else
        {
            while (split < maxSplit && heads * split < 160)
            {
                split *= 2;
            }
        }
        a.qSplit = std::min(split, maxSplit);
        // tuning override: TRTAMD_FMHA_QSPLIT=<n> forces the number of workgroups per head
        int const forced = tuning(Tuning::kFmhaQsplit);
        if (forced > 0)
        {
            a.qSplit = std::min(forced, maxSplit);
        }
    }
    a.dbgAcc1 = dbgAcc1;
    a.dbgP8 = dbgP8;
    {
        // The order in which sequences are served matters when workgroups run in several rounds (the long ones
        // first, so that the short ones fill the tail).  When every workgroup of the launch is resident at once it
        // changes nothing, and the workgroups skip the ranking (a trip to LDS and two barriers before their loads).
        int const kt = pick_kt(p->s);
        int64_t const lds = dataType == 2 ? Lds<1>::total(kt) : Lds<2>::total(kt);
        int64_t const perCu = std::max<int64_t>(1, std::min<int64_t>(dataType == 2 ? 3 : 2, (160 * 1024) / std::max<int64_t>(lds, 1)));
        a.ranked = (int64_t) a.B * a.N * a.qSplit > perCu * 256 ? 1 : 0;
        // tuning override: TRTAMD_FMHA_RANKED=0 / 1 forces natural order / the longest-first order
        int const forcedRank = tuning(Tuning::kFmhaRanked);
        if (forcedRank >= 0)
        {
            a.ranked = forcedRank ? 1 : 0;
        }
    }
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

// Test hook (include/trtamd_test_hooks.h): same launch, additionally dumping the first GEMM's accumulators
// ([b][h][s][s], int32 for INT8, binary32 bit patterns for FP16) and, for INT8, the quantised probabilities.
extern "C" int trtamd_fused_mha_run_debug(trtamd_stream_t stream, int32_t data_type,
    trtamd_fmha_params const* params, int32_t* acc1, int8_t* p8)
{
    return fused_mha_run(as_stream(stream), data_type, params, acc1, p8);
}

extern "C" int trtamd_fused_mha_prepare(void)
{
    int st = prepare_kt<1>();
    st = st ? st : prepare_kt<2>();
    st = st ? st : prepare_kt<3>();
    st = st ? st : prepare_kt<4>();
    st = st ? st : prepare_kt<6>();
    st = st ? st : prepare_kt<8>();
    return st;
}

extern "C" int trtamd_fused_mha_is_valid(int32_t data_type, int32_t d, int32_t s)
{
    return (data_type == 1 || data_type == 2) && d == kHeadSize && s > 0 && s <= 512;
}
