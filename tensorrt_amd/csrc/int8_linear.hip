// INT8 linear layer for gfx950: out[t][n] = epilogue(sum_k a[t][k] * w[n][k]).
//
// The projections between the encoder plugins (QKV, attention output, the two feed-forward
// layers) are plain GEMMs whose operands are both contiguous along k, which is what the INT8 MFMA
// wants: a lane feeds 16 consecutive k-bytes of one row.  v_mfma_i32_32x32x32_i8 is used: it runs at
// the full INT8 rate of the matrix core (measured: 32768 MACs in 33 cycles per SIMD, as does
// v_mfma_i32_16x16x64_i8 with 16384 in 16.5) and needs half as many fragment reads per MAC as the
// 16 x 16 form.  The kernel computes the transposed
// product (output channels are the M dimension, tokens the N dimension) so that a lane ends up with
// groups of four consecutive channels of one token, which pack into the token-major INT8 output of
// either layout.
//
// Tiling: a workgroup owns BM channels x BN tokens, its waves a WM x WN grid of (MT*32) x (NT*32)
// sub-tiles kept in INT32 accumulators.  One stage is 64 bytes of k for the whole tile (two MFMA
// steps).  Global loads are 16 bytes per lane with consecutive lanes on consecutive addresses; a
// fragment sits in LDS row-major with a one-bit swizzle, so LDS writes and the 16-byte-per-lane
// fragment reads are both conflict-free.  Stages are double-buffered in LDS and the loads run two
// stages ahead of the multiplication through two register sets.
//
// Activations, weights and outputs may be in the linear layout [R][C] or in the 32-interleaved
// layout [C/32][R][32] that the interleaved encoder plugins use; the interleaved one makes every
// load unit 1 KB of contiguous memory.
#include "device_utils.hpp"
#include "host_utils.hpp"
#include "trtamd_encoder_ops.h"

#include <cstdlib>
#include <type_traits>

namespace trtamd
{
namespace
{

constexpr int kBigTile = 256; // channels and tokens of the large workgroup tile

enum Epilogue
{
    kAFFINE = TRTAMD_LINEAR_AFFINE,
    kGELU = TRTAMD_LINEAR_GELU,
    kRAW = TRTAMD_LINEAR_RAW_INT32,
    kHALF = TRTAMD_LINEAR_AFFINE_FP16,
    // FP16 operands (trtamd_fp16_linear): the same kernels with v_mfma_f32_32x32x16_f16 and binary32 accumulators
    kF16_AFFINE = 4,
    kF16_GELU = 5
};

// INT8 operands accumulate in INT32, FP16 operands in binary32.  Either way a lane feeds 16 bytes of a row per
// operand and MFMA step (16 INT8 or 8 FP16 values of k), a fragment is 32 rows x 32 bytes, and the result has the
// same 32 x 32 accumulator layout, so the tiling, the LDS layout and the load schedule are shared.
template <int EPI>
using AccT = std::conditional_t<(EPI >= kF16_AFFINE), f32x16, i32x16>;

template <int EPI>
__device__ __forceinline__ AccT<EPI> mma(i32x4 const a, i32x4 const b, AccT<EPI> const c)
{
    if constexpr (EPI >= kF16_AFFINE)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(bits_as<f16x8>(a), bits_as<f16x8>(b), c, 0, 0, 0);
    }
    else
    {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
    }
}

struct LinearArgs
{
    int8_t const* a;
    int8_t const* w;
    float const* alpha;
    float const* beta;
    void* out;
    int T, K, N; // K: bytes of k per row (elements for INT8, twice the elements for FP16)
    float qOut;
    int mainTiles; // workgroups that own a 256 x 256 tile
    int tokMain;   // rows of 256 tokens they cover
    int panel;     // channel tiles per panel of the tile numbering (divides the number of channel tiles)
    int persist;   // persistent kernel: workgroups that loop over the 256 x 256 tiles
    int pieces;    // direct-to-LDS kernel: the tokens behind the large tiles go in 64 x 64 pieces (see linear_piece64)
};

// gelu(y) = y * Phi(y) = max(y, 0) - |y| * Phi(-|y|).  log2(Phi(-a)) is smooth and nearly quadratic, so
// Phi(-a) = exp2(P(a)) with a cubic fitted to minimise the error of a * Phi(-a) on [0, 7]; the leading coefficient is
// negative, so the term vanishes for larger a as it should.  Measured against the binary64 erf form the absolute
// error of gelu is below 5.5e-5 for every binary32 |y| <= 40 (largest near |y| = 1.1): at the output scales of an
// INT8 feed-forward layer (20-40 steps per unit) that moves 0.04-0.1 % of the requantised values by one step, half
// of what the parity tests allow, and it is far inside the FP16 output's tolerance.  Three fma, one v_exp_f32, one
// max and one fma per value (a degree-5 fit, 6.4e-7 and two more fma, measured the same results to 0.001 %).
__device__ inline float gelu_erf(float y)
{
    float const a = fabsf(y);
    float p = fmaf(a, -2.488555945e-02f, -4.988203049e-01f);
    p = fmaf(p, a, -1.129245639e+00f);
    p = fmaf(p, a, -1.003531814e+00f);
    return fmaf(-a, __builtin_amdgcn_exp2f(p), fmaxf(y, 0.f));
}

// One operand fragment of v_mfma_i32_32x32x32_i8 is 32 rows x 32 k-bytes; lane l feeds row l%32,
// bytes 16*(l/32)..+15.  In LDS a fragment is 1 KB, row-major, with the two 16-byte halves of a row
// swapped for rows 8..15 and 24..31: a 16-lane group then reads 16 different 16-byte columns of the
// bank array, and so does a group that writes 8 whole rows.
__device__ inline int frag_offset(int row, int half)
{
    return row * 32 + ((half ^ ((row >> 3) & 1)) << 4);
}

// Epilogue of one 32 x 32 accumulator block whose first channel is c0 (sAlpha / sBeta point at that channel's
// entry) and first token tb.  Accumulator register v is token l%32, channel 8*(v/4) + 4*(l/32) + v%4: four groups
// of four consecutive channels.  For the INT8 outputs the two lanes that share a token trade two packed dwords
// (v_permlane32_swap), after which lane l holds the 16 consecutive channels 16*(l/32)..+15 and stores them with
// one 16-byte write.
// THROUGH: the store writes through the L2 (inline assembly, which the compiler's own vmcnt bookkeeping does not see:
// only for the kernel that places its waits itself, and only where a wavefront's store covers whole cache lines, the
// 32-interleaved INT8 output: 32 tokens x 32 bytes; narrower pieces are better merged in the L2 first).
template <bool THROUGH, typename V>
__device__ __forceinline__ void store_out(void* p, V const& v)
{
    if constexpr (THROUGH)
    {
        store_through_l2(p, v);
    }
    else
    {
        *static_cast<V*>(p) = v;
    }
}

// The 16 scale / offset pairs a lane needs for one 32-channel block (channels 8g + 4 (l/32) + e of the block), read
// from the tile's vectors in LDS.  For the affine INT8 epilogue the offsets already carry the 128 of the unsigned
// byte conversion.  A block's scales serve every token block of the same channels, so callers that walk several
// token blocks load them once.
struct BlockScales
{
    f32x4 al[4], be[4];
};

template <int EPI>
__device__ __forceinline__ BlockScales load_block_scales(float const* sAlpha, float const* sBeta)
{
    BlockScales s;
    if constexpr (EPI != kRAW)
    {
        int const hi = (threadIdx.x & 63) >> 5;
#pragma unroll
        for (int g = 0; g < 4; ++g)
        {
            s.al[g] = *reinterpret_cast<f32x4 const*>(sAlpha + 8 * g + 4 * hi);
            s.be[g] = *reinterpret_cast<f32x4 const*>(sBeta + 8 * g + 4 * hi);
            if constexpr (EPI == kAFFINE)
            {
#pragma unroll
                for (int e = 0; e < 4; ++e)
                {
                    s.be[g][e] += 128.f;
                }
            }
        }
    }
    return s;
}

template <bool IL_OUT, int EPI, bool FULL = false, bool THROUGH = false>
__device__ __forceinline__ void store_block_scaled(
    LinearArgs const& p, AccT<EPI> const& acc, int const c0, int const tb, BlockScales const& sc)
{
    int const lane = threadIdx.x & 63;
    int const hi = lane >> 5;
    int const t = tb + (lane & 31);
    bool const live = FULL || t < p.T; // FULL: the block lies inside the problem and is stored unconditionally
    f32x4 const(&al)[4] = sc.al;
    f32x4 const(&be)[4] = sc.be;
    if constexpr (EPI == kRAW)
    {
        if (live)
        {
#pragma unroll
            for (int g = 0; g < 4; ++g)
            {
                i32x4 const v = {acc[4 * g], acc[4 * g + 1], acc[4 * g + 2], acc[4 * g + 3]};
                store_out<THROUGH>(static_cast<int32_t*>(p.out) + (size_t) t * p.N + c0 + 8 * g + 4 * hi, v);
            }
        }
    }
    else if constexpr (EPI >= kF16_AFFINE || EPI == kHALF)
    {
        u32x2 w[4];
#pragma unroll
        for (int g = 0; g < 4; ++g)
        {
            f16x4 h;
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                float const y = fmaf((float) acc[4 * g + e], al[g][e], be[g][e]);
                h[e] = (f16) (EPI == kF16_GELU ? gelu_erf(y) : y);
            }
            w[g] = __builtin_bit_cast(u32x2, h);
        }
        // lanes l < 32 hold channels 8g..8g+3 of each group g, lanes l+32 the other four: after the swaps lane l has
        // groups 0 and 1 whole, lane l+32 groups 2 and 3: 16 consecutive channels, two 16-byte stores
        auto const a0 = __builtin_amdgcn_permlane32_swap(w[0][0], w[2][0], false, false);
        auto const a1 = __builtin_amdgcn_permlane32_swap(w[0][1], w[2][1], false, false);
        auto const b0 = __builtin_amdgcn_permlane32_swap(w[1][0], w[3][0], false, false);
        auto const b1 = __builtin_amdgcn_permlane32_swap(w[1][1], w[3][1], false, false);
        u32x4 const first = {a0[0], a1[0], a0[1], a1[1]};
        u32x4 const second = {b0[0], b1[0], b0[1], b1[1]};
        if (live)
        {
            f16* dst = static_cast<f16*>(p.out) + (size_t) t * p.N + c0 + 16 * hi;
            store_out<THROUGH>(dst, first);
            store_out<THROUGH>(dst + 8, second);
        }
    }
    else
    {
        // Results are formed as unsigned bytes, x + 128: v_cvt_pk_u8_f32 rounds to nearest even, saturates to
        // [0, 255] and places the byte in one instruction; one XOR per dword returns to two's complement.
        int d[4];
#pragma unroll
        for (int g = 0; g < 4; ++g)
        {
            uint32_t w = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e)
            {
                if constexpr (EPI == kGELU)
                {
                    float const y = fmaf((float) acc[4 * g + e], al[g][e], be[g][e]);
                    w = __builtin_amdgcn_cvt_pk_u8_f32(fmaf(gelu_erf(y), p.qOut, 128.f), e, w);
                }
                else
                {
                    w = __builtin_amdgcn_cvt_pk_u8_f32(fmaf((float) acc[4 * g + e], al[g][e], be[g][e]), e, w);
                }
            }
            d[g] = (int) (w ^ 0x80808080u);
        }
        // lanes l < 32 hold channels [0-3][8-11][16-19][24-27], lanes l+32 the gaps
        auto const s02 = __builtin_amdgcn_permlane32_swap(d[0], d[2], false, false);
        auto const s13 = __builtin_amdgcn_permlane32_swap(d[1], d[3], false, false);
        i32x4 const packed = {(int) s02[0], (int) s02[1], (int) s13[0], (int) s13[1]};
        if (live)
        {
            int const c = c0 + 16 * hi;
            size_t const o = IL_OUT ? ((size_t) (c >> 5) * p.T + t) * 32 + (c & 31) : (size_t) t * p.N + c;
            store_out<THROUGH>(static_cast<int8_t*>(p.out) + o, packed);
        }
    }
}

template <bool IL_OUT, int EPI, bool FULL = false, bool THROUGH = false>
__device__ __forceinline__ void store_block(
    LinearArgs const& p, AccT<EPI> const& acc, int const c0, int const tb, float const* sAlpha, float const* sBeta)
{
    store_block_scaled<IL_OUT, EPI, FULL, THROUGH>(p, acc, c0, tb, load_block_scales<EPI>(sAlpha, sBeta));
}

// Epilogue of one workgroup tile.
template <int WM, int WN, int MT, int NT, bool IL_OUT, int EPI>
__device__ __forceinline__ void store_tile(LinearArgs const& p, AccT<EPI> const (&acc)[MT][NT], int const n0, int const t0,
    float const* sAlpha, float const* sBeta)
{
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const wm = wave / WN;
    int const wn = wave % WN;
#pragma unroll
    for (int i = 0; i < MT; ++i)
    {
        int const cl = (wm * MT + i) * 32; // wave-uniform, and so is the guard: N is a multiple of 32
        if (n0 + cl >= p.N)
        {
            break;
        }
#pragma unroll
        for (int j = 0; j < NT; ++j)
        {
            store_block<IL_OUT, EPI>(p, acc[i][j], n0 + cl, t0 + (wn * NT + j) * 32, sAlpha + cl, sBeta + cl);
        }
    }
}

// One output tile of BM = WM*MT*32 channels x BN = WN*NT*32 tokens at (n0, t0), by the whole workgroup.
template <int WM, int WN, int MT, int NT, bool IL_W, bool IL_IN, bool IL_OUT, int EPI>
__device__ __forceinline__ void linear_tile(
    LinearArgs const& p, int const n0, int const t0, uint8_t* __restrict__ lds, float* sAlpha, float* sBeta)
{
    constexpr int NWAVES = WM * WN;
    constexpr int BM = WM * MT * 32;    // output channels per workgroup
    constexpr int BN = WN * NT * 32;    // tokens per workgroup
    constexpr int AF = (BM / 32) * 2;   // weight fragments per stage (64 bytes of k = two MFMA steps)
    constexpr int BF = (BN / 32) * 2;   // activation fragments per stage
    static_assert(AF % NWAVES == 0 && BF % NWAVES == 0, "load units divide evenly among the waves");
    constexpr int LA = AF / NWAVES;
    constexpr int LB = BF / NWAVES;
    constexpr int STAGE = (AF + BF) * 1024;

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const wm = wave / WN;
    int const wn = wave % WN;
    int const col32 = lane & 31;
    int const hi = lane >> 5;

    // A load unit is 1 KB that one wave fetches with one 16-byte load per lane, consecutive lanes
    // reading consecutive memory.  Interleaved operand [K/32][R][32]: unit (rb, ks) is the 32 rows of
    // row block rb in k-slab ks, contiguous in memory, and is exactly one fragment.  Linear operand
    // [R][K]: unit (rb, h) is rows 16h..16h+15 of the block, 64 bytes of k each, and lands in the two
    // fragments (rb, 0) and (rb, 1).
    auto unit_addressing = [&](bool interleaved, int unit, int row0, int R, uint32_t& gOff, int& lOff) {
        int const rb = unit >> 1, sel = unit & 1;
        if (interleaved)
        {
            int const r = lane >> 1, c = lane & 1;
            int const row = min(row0 + rb * 32 + r, R - 1);
            gOff = ((uint32_t) sel * (uint32_t) R + (uint32_t) row) * 32u + (uint32_t) c * 16u;
            lOff = (rb * 2 + sel) * 1024 + frag_offset(r, c);
        }
        else
        {
            int const r = sel * 16 + (lane >> 2), c = lane & 3;
            int const row = min(row0 + rb * 32 + r, R - 1);
            gOff = (uint32_t) row * (uint32_t) p.K + (uint32_t) c * 16u;
            lOff = (rb * 2 + (c >> 1)) * 1024 + frag_offset(r, c & 1);
        }
    };
    uint32_t offA[LA], offB[LB];
    int ldsA[LA], ldsB[LB];
#pragma unroll
    for (int q = 0; q < LA; ++q)
    {
        unit_addressing(IL_W, q * NWAVES + wave, n0, p.N, offA[q], ldsA[q]);
    }
#pragma unroll
    for (int q = 0; q < LB; ++q)
    {
        unit_addressing(IL_IN, q * NWAVES + wave, t0, p.T, offB[q], ldsB[q]);
        ldsB[q] += AF * 1024;
    }
    uint32_t const stepA = IL_W ? 2u * (uint32_t) p.N * 32u : 64u;
    uint32_t const stepB = IL_IN ? 2u * (uint32_t) p.T * 32u : 64u;

    // two register sets: the loads of stage s+2 are issued while stage s is multiplied, so a load has
    // two stages of MFMA work to hide behind before its data is moved to LDS
    i32x4 ga[2][LA], gb[2][LB];
    auto fetch = [&](auto set, int kt) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            ga[S][q] = *reinterpret_cast<i32x4 const*>(p.w + offA[q] + (uint32_t) kt * stepA);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            gb[S][q] = *reinterpret_cast<i32x4 const*>(p.a + offB[q] + (uint32_t) kt * stepB);
        }
    };
    auto stash = [&](auto set, int buf) {
        constexpr int S = decltype(set)::value;
        uint8_t* base = lds + buf * STAGE;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            *reinterpret_cast<i32x4*>(base + ldsA[q]) = ga[S][q];
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            *reinterpret_cast<i32x4*>(base + ldsB[q]) = gb[S][q];
        }
    };

    AccT<EPI> acc[MT][NT];
#pragma unroll
    for (int i = 0; i < MT; ++i)
    {
#pragma unroll
        for (int j = 0; j < NT; ++j)
        {
#pragma unroll
            for (int v = 0; v < 16; ++v)
            {
                acc[i][j][v] = 0;
            }
        }
    }
    int const readOff = frag_offset(col32, hi);
    auto multiply = [&](int buf) {
        uint8_t const* base = lds + buf * STAGE + readOff;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
        {
            i32x4 fa[MT], fb[NT];
#pragma unroll
            for (int i = 0; i < MT; ++i)
            {
                fa[i] = *reinterpret_cast<i32x4 const*>(base + ((wm * MT + i) * 2 + ks) * 1024);
            }
#pragma unroll
            for (int j = 0; j < NT; ++j)
            {
                fb[j] = *reinterpret_cast<i32x4 const*>(base + (AF + (wn * NT + j) * 2 + ks) * 1024);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
            {
#pragma unroll
                for (int j = 0; j < NT; ++j)
                {
                    acc[i][j] = mma<EPI>(fa[i], fb[j], acc[i][j]);
                }
            }
        }
    };
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;

    // per-channel scale and offset of the tile, staged once for the epilogue
    if constexpr (EPI != kRAW)
    {
        for (int c = threadIdx.x; c < BM; c += 64 * NWAVES)
        {
            int const n = min(n0 + c, p.N - 1);
            sAlpha[c] = p.alpha[n];
            sBeta[c] = p.beta[n];
        }
    }

    // Stage kt sits in LDS buffer kt&1 and arrived through register set kt&1.  The loop body has no
    // branches (loads past the last stage re-read the last stage and are never used), so the number of
    // loads in flight at every point is fixed and a stash waits for its own four loads only.
    int const nk = p.K / 64;
    fetch(Set0{}, 0);
    fetch(Set1{}, min(1, nk - 1));
    stash(Set0{}, 0);
    __syncthreads();
    int kt = 0;
    for (; kt + 1 < nk; kt += 2)
    {
        fetch(Set0{}, min(kt + 2, nk - 1));
        multiply(0);
        stash(Set1{}, 1);
        __syncthreads();
        fetch(Set1{}, min(kt + 3, nk - 1));
        multiply(1);
        stash(Set0{}, 0);
        __syncthreads();
    }
    if (kt < nk)
    {
        multiply(0);
    }

    store_tile<WM, WN, MT, NT, IL_OUT, EPI>(p, acc, n0, t0, sAlpha, sBeta);
}

// A run of `count` tiles by one persistent workgroup, K % 128 == 0.  The stage pipeline does not drain
// between tiles: the last two stages of a tile already fetch the first two stages of the next one, the
// epilogue runs while those loads are in flight, and the next tile's scale/offset vectors are picked up at
// the start of the current one.  `origin(j, n0, t0)` gives the j-th tile's corner.
template <int WM, int WN, int MT, int NT, bool IL_W, bool IL_IN, bool IL_OUT, int EPI, typename Origin>
__device__ __forceinline__ void linear_tile_run(
    LinearArgs const& p, int const count, Origin origin, uint8_t* __restrict__ lds, float* sScale)
{
    constexpr int NWAVES = WM * WN;
    constexpr int BM = WM * MT * 32;
    constexpr int BN = WN * NT * 32;
    constexpr int AF = (BM / 32) * 2;
    constexpr int BF = (BN / 32) * 2;
    static_assert(AF % NWAVES == 0 && BF % NWAVES == 0, "load units divide evenly among the waves");
    static_assert((BM & (BM - 1)) == 0 && BM <= kBigTile, "scale staging");
    constexpr int LA = AF / NWAVES;
    constexpr int LB = BF / NWAVES;
    constexpr int STAGE = (AF + BF) * 1024;

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const wm = wave / WN;
    int const wn = wave % WN;

    int ldsA[LA], ldsB[LB];
    auto address = [&](int n0, int t0, uint32_t(&oa)[LA], uint32_t(&ob)[LB]) {
        auto unit = [&](bool interleaved, int u, int row0, int R, uint32_t& gOff, int& lOff) {
            int const rb = u >> 1, sel = u & 1;
            if (interleaved)
            {
                int const r = lane >> 1, c = lane & 1;
                int const row = min(row0 + rb * 32 + r, R - 1);
                gOff = ((uint32_t) sel * (uint32_t) R + (uint32_t) row) * 32u + (uint32_t) c * 16u;
                lOff = (rb * 2 + sel) * 1024 + frag_offset(r, c);
            }
            else
            {
                int const r = sel * 16 + (lane >> 2), c = lane & 3;
                int const row = min(row0 + rb * 32 + r, R - 1);
                gOff = (uint32_t) row * (uint32_t) p.K + (uint32_t) c * 16u;
                lOff = (rb * 2 + (c >> 1)) * 1024 + frag_offset(r, c & 1);
            }
        };
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            unit(IL_W, q * NWAVES + wave, n0, p.N, oa[q], ldsA[q]);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            unit(IL_IN, q * NWAVES + wave, t0, p.T, ob[q], ldsB[q]);
            ldsB[q] += AF * 1024;
        }
    };
    uint32_t const stepA = IL_W ? 2u * (uint32_t) p.N * 32u : 64u;
    uint32_t const stepB = IL_IN ? 2u * (uint32_t) p.T * 32u : 64u;

    i32x4 ga[2][LA], gb[2][LB];
    auto fetch = [&](auto set, uint32_t const(&oa)[LA], uint32_t const(&ob)[LB], int kt) {
        constexpr int S = decltype(set)::value;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            ga[S][q] = *reinterpret_cast<i32x4 const*>(p.w + oa[q] + (uint32_t) kt * stepA);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            gb[S][q] = *reinterpret_cast<i32x4 const*>(p.a + ob[q] + (uint32_t) kt * stepB);
        }
    };
    auto stash = [&](auto set, int buf) {
        constexpr int S = decltype(set)::value;
        uint8_t* base = lds + buf * STAGE;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            *reinterpret_cast<i32x4*>(base + ldsA[q]) = ga[S][q];
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            *reinterpret_cast<i32x4*>(base + ldsB[q]) = gb[S][q];
        }
    };

    AccT<EPI> acc[MT][NT];
    int const readOff = frag_offset(lane & 31, lane >> 5);
    auto multiply = [&](int buf) {
        uint8_t const* base = lds + buf * STAGE + readOff;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
        {
            i32x4 fa[MT], fb[NT];
#pragma unroll
            for (int i = 0; i < MT; ++i)
            {
                fa[i] = *reinterpret_cast<i32x4 const*>(base + ((wm * MT + i) * 2 + ks) * 1024);
            }
#pragma unroll
            for (int j = 0; j < NT; ++j)
            {
                fb[j] = *reinterpret_cast<i32x4 const*>(base + (AF + (wn * NT + j) * 2 + ks) * 1024);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
            {
#pragma unroll
                for (int j = 0; j < NT; ++j)
                {
                    acc[i][j] = mma<EPI>(fa[i], fb[j], acc[i][j]);
                }
            }
        }
    };
    using Set0 = std::integral_constant<int, 0>;
    using Set1 = std::integral_constant<int, 1>;

    // scale/offset vectors: sScale[parity][alpha|beta][channel]; every thread copies channel tid % BM
    int const ch = threadIdx.x & (BM - 1);
    auto scales = [&](int parity, int which) { return sScale + (parity * 2 + which) * kBigTile; };

    int n0, t0;
    origin(0, n0, t0);
    uint32_t oaC[LA], obC[LB], oaN[LA], obN[LB];
    address(n0, t0, oaC, obC);
    if constexpr (EPI != kRAW)
    {
        int const n = min(n0 + ch, p.N - 1);
        scales(0, 0)[ch] = p.alpha[n];
        scales(0, 1)[ch] = p.beta[n];
    }
    int const nk = p.K / 64; // even, >= 2
    fetch(Set0{}, oaC, obC, 0);
    fetch(Set1{}, oaC, obC, 1);
    stash(Set0{}, 0);
    __syncthreads();
    for (int j = 0; j < count; ++j)
    {
        int n1 = n0, t1 = t0;
        if (j + 1 < count)
        {
            origin(j + 1, n1, t1);
        }
        address(n1, t1, oaN, obN);
        float nextAlpha = 0.f, nextBeta = 0.f;
        if constexpr (EPI != kRAW)
        {
            int const n = min(n1 + ch, p.N - 1);
            nextAlpha = p.alpha[n];
            nextBeta = p.beta[n];
        }
#pragma unroll
        for (int i = 0; i < MT; ++i)
        {
#pragma unroll
            for (int jj = 0; jj < NT; ++jj)
            {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                {
                    acc[i][jj][v] = 0;
                }
            }
        }
        for (int kt = 0; kt + 2 < nk; kt += 2)
        {
            fetch(Set0{}, oaC, obC, kt + 2);
            multiply(0);
            stash(Set1{}, 1);
            __syncthreads();
            fetch(Set1{}, oaC, obC, kt + 3);
            multiply(1);
            stash(Set0{}, 0);
            __syncthreads();
        }
        // last two stages of this tile; the loads are the next tile's first two stages
        fetch(Set0{}, oaN, obN, 0);
        multiply(0);
        stash(Set1{}, 1);
        __syncthreads();
        fetch(Set1{}, oaN, obN, 1);
        multiply(1);
        if constexpr (EPI != kRAW)
        {
            scales((j + 1) & 1, 0)[ch] = nextAlpha;
            scales((j + 1) & 1, 1)[ch] = nextBeta;
        }
        store_tile<WM, WN, MT, NT, IL_OUT, EPI>(p, acc, n0, t0, scales(j & 1, 0), scales(j & 1, 1));
        stash(Set0{}, 0);
        __syncthreads();
        n0 = n1;
        t0 = t1;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            oaC[q] = oaN[q];
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            obC[q] = obN[q];
        }
    }
}

// The persistent run of 256 x 256 tiles with the stages brought in by direct-to-LDS loads: a ring of four LDS stage
// buffers, stage k+3 requested while stage k is multiplied, no staging registers, no LDS-write instructions and
// nothing for a wavefront to wait for before the barrier except loads issued two steps earlier.  N a multiple of 256
// and K of 256 bytes (the ring index is then the stage index modulo 4 in every tile).  One instruction fills 1 KB of
// LDS with lane i's 16 bytes at offset 16 i, so the LDS swizzle is applied on the source side: lane i fetches the
// 16 bytes that belong there.
//   IL (both operands 32-interleaved): a load unit is one fragment, 32 rows x 32 bytes, contiguous in memory.
//   otherwise (both operands linear [R][K], also the FP16 layers): a load unit is 16 rows x 64 bytes (four lanes
//   per row, 64 contiguous bytes of it); in LDS the 16-byte chunk c of row r sits at chunk c ^ (r / 4), which makes
//   the fragment reads (16 rows x one chunk per 16 lanes) conflict-free; fragment (block, ks) takes chunks 2 ks and
//   2 ks + 1 of the block's two units.
template <bool IL, bool IL_OUT, int EPI, typename Origin>
__device__ __forceinline__ void linear_tile_run_dma(
    LinearArgs const& p, int const count, Origin origin, uint8_t* __restrict__ lds, float* sScale)
{
    constexpr int KS = 2; // k-halves of 32 bytes per stage
    constexpr int WN = 4, MT = 4, NT = 2, NWAVES = 8;
    constexpr int AF = (kBigTile / 32) * KS;   // 1 KB fragments per operand and stage: KS k-halves of 32 bytes per row block
    constexpr int BF = (kBigTile / 32) * KS;
    constexpr int LA = AF / NWAVES;
    constexpr int LB = BF / NWAVES;
    constexpr int STAGE = (AF + BF) * 1024;
    constexpr int kLoads = LA + LB;           // direct loads per wavefront and stage
    // global stores per wavefront in a tile's epilogue: one 16-byte store per accumulator block (INT8), two (FP16)
    constexpr int kStores = MT * NT * (EPI >= kF16_AFFINE ? 2 : 1);
    static_assert(EPI == kAFFINE || EPI == kGELU || EPI == kF16_AFFINE || EPI == kF16_GELU, "store count per block");

    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const wm = wave / WN;
    int const wn = wave % WN;
    uint32_t const ldsBase = (uint32_t) (size_t) (__attribute__((address_space(3))) uint8_t*) lds;
    uint32_t const scaleBase = (uint32_t) (size_t) (__attribute__((address_space(3))) float*) sScale;

    // Lane i of a unit's load supplies LDS offset 16 i of the unit.  Its address is a wave-uniform part (the unit's
    // first row, kept in scalar registers and advanced by scalar arithmetic) plus a lane part that is the same for
    // every unit, tile and stage: the loop spends no vector-ALU instruction on addresses.
    uint32_t laneOff;
    if constexpr (IL)
    {
        int const r = lane >> 1; // row of the fragment; the half that the swizzle puts at this offset
        uint32_t const half = (uint32_t) ((lane & 1) ^ ((r >> 3) & 1));
        laneOff = (uint32_t) r * 32u + half * 16u;
    }
    else
    {
        int const rr = lane >> 2; // row of the 16-row unit; the chunk that the swizzle puts at this offset
        uint32_t const chunk = (uint32_t) ((lane & 3) ^ (rr >> 2));
        laneOff = (uint32_t) rr * (uint32_t) p.K + chunk * 16u;
    }
    auto unit_base = [&](int u, int row0, int R) -> uint32_t {
        int const rb = u >> 1, sel = u & 1;
        uint32_t const b = IL ? ((uint32_t) sel * (uint32_t) R + (uint32_t) (row0 + rb * 32)) * 32u
                              : (uint32_t) (row0 + rb * 32 + sel * 16) * (uint32_t) p.K;
        return (uint32_t) __builtin_amdgcn_readfirstlane((int) b);
    };
    auto address = [&](int n0, int t0, uint32_t(&oa)[LA], uint32_t(&ob)[LB]) {
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            oa[q] = unit_base(q * NWAVES + wave, n0, p.N);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            ob[q] = unit_base(q * NWAVES + wave, t0, p.T);
        }
    };
    uint32_t const stepA = IL ? (uint32_t) KS * (uint32_t) p.N * 32u : 64u;
    uint32_t const stepB = IL ? (uint32_t) KS * (uint32_t) p.T * 32u : 64u;
    int const nk = p.K / (32 * KS); // a multiple of 4

    uint32_t oaC[LA], obC[LB], oaN[LA], obN[LB];
    // stage kt of the current tile (or stage kt - nk of the next one) into ring slot `slot`
    auto fetch = [&](int kt, int slot) {
        bool const next = kt >= nk;
        uint32_t const k = (uint32_t) (next ? kt - nk : kt);
        uint32_t const dst = ldsBase + (uint32_t) slot * STAGE;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            load_to_lds16_sbase(p.w + (uint64_t) (next ? oaN[q] : oaC[q]) + (uint64_t) k * stepA, laneOff,
                dst + (uint32_t) (q * NWAVES + wave) * 1024u);
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            load_to_lds16_sbase(p.a + (uint64_t) (next ? obN[q] : obC[q]) + (uint64_t) k * stepB, laneOff,
                dst + (uint32_t) (AF + q * NWAVES + wave) * 1024u);
        }
    };

    AccT<EPI> acc[MT][NT];
    // byte offset, inside a 32-row block's 2 KB, of this lane's 16 bytes of fragment ks
    int readOff[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
    {
        if constexpr (IL)
        {
            readOff[ks] = ks * 1024 + frag_offset(lane & 31, lane >> 5);
        }
        else
        {
            int const fr = lane & 31, rr = fr & 15;
            readOff[ks] = (fr >> 4) * 1024 + rr * 64 + (((ks * 2 + (lane >> 5)) ^ (rr >> 2)) << 4);
        }
    }
    auto multiply = [&](int slot) {
        uint8_t const* base = lds + slot * STAGE;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
        {
            i32x4 fa[MT], fb[NT];
#pragma unroll
            for (int i = 0; i < MT; ++i)
            {
                fa[i] = *reinterpret_cast<i32x4 const*>(base + (wm * MT + i) * (KS * 1024) + readOff[ks]);
            }
#pragma unroll
            for (int j = 0; j < NT; ++j)
            {
                fb[j] = *reinterpret_cast<i32x4 const*>(base + AF * 1024 + (wn * NT + j) * (KS * 1024) + readOff[ks]);
            }
#pragma unroll
            for (int i = 0; i < MT; ++i)
            {
#pragma unroll
                for (int j = 0; j < NT; ++j)
                {
                    acc[i][j] = mma<EPI>(fa[i], fb[j], acc[i][j]);
                }
            }
        }
    };
    // scale / offset vectors of a tile, 256 binary32 values each: one direct load by wave 0 and one by wave 1
    auto fetch_scales = [&](int n0, int parity) {
        if (wave < 2)
        {
            float const* src = (wave == 0 ? p.alpha : p.beta) + n0 + lane * 4;
            load_to_lds16(src, scaleBase + (uint32_t) ((parity * 2 + wave) * kBigTile) * 4u);
        }
    };
    auto scales = [&](int parity, int which) { return sScale + (parity * 2 + which) * kBigTile; };
    // one step: request stage k+3, multiply stage k, make sure this wavefront's part of stage k+1 has landed, meet
    // the others.  vmcnt counts the kLoads of stages k+2 and k+3 behind it, and `extra` operations known to sit
    // between (epilogue stores), which must not be waited for.
    auto step = [&](int k, auto slotTag, auto extraTag) {
        constexpr int SLOT = decltype(slotTag)::value;
        constexpr int EXTRA = decltype(extraTag)::value;
        fetch(k + 3, (SLOT + 3) & 3);
        multiply(SLOT);
        wait_vmcnt<2 * kLoads + EXTRA>();
        __syncthreads();
    };
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    using NoExtra = std::integral_constant<int, 0>;
    using Stores = std::integral_constant<int, kStores>;

    int n0, t0;
    origin(0, n0, t0);
    address(n0, t0, oaC, obC);
#pragma unroll
    for (int q = 0; q < LA; ++q)
    {
        oaN[q] = oaC[q];
    }
#pragma unroll
    for (int q = 0; q < LB; ++q)
    {
        obN[q] = obC[q];
    }
    fetch_scales(n0, 0);
    fetch(0, 0);
    fetch(1, 1);
    fetch(2, 2);
    wait_vmcnt<2 * kLoads>();
    __syncthreads();
    for (int j = 0; j < count; ++j)
    {
        int n1 = n0, t1 = t0;
        if (j + 1 < count)
        {
            origin(j + 1, n1, t1);
        }
        address(n1, t1, oaN, obN);
#pragma unroll
        for (int i = 0; i < MT; ++i)
        {
#pragma unroll
            for (int jj = 0; jj < NT; ++jj)
            {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                {
                    acc[i][jj][v] = 0;
                }
            }
        }
        // The first two steps after an epilogue have its stores between the stage they wait for and the newer loads.
        // The next tile's scale vectors go into the buffer the previous tile's epilogue read: only after the first
        // barrier of this tile has every wavefront left that epilogue.  (On the two wavefronts that fetch them the
        // waits below then count one operation too few, which only makes them wait for one more load.)
        if (j == 0)
        {
            step(0, S0{}, NoExtra{});
            fetch_scales(n1, (j + 1) & 1);
            step(1, S1{}, NoExtra{});
        }
        else
        {
            step(0, S0{}, Stores{});
            fetch_scales(n1, (j + 1) & 1);
            step(1, S1{}, Stores{});
        }
        step(2, S2{}, NoExtra{});
        step(3, S3{}, NoExtra{});
        for (int k = 4; k < nk; k += 4)
        {
            step(k, S0{}, NoExtra{});
            step(k + 1, S1{}, NoExtra{});
            step(k + 2, S2{}, NoExtra{});
            step(k + 3, S3{}, NoExtra{});
        }
        BlockScales blockScales;
#pragma unroll
        for (int i = 0; i < MT; ++i)
        {
#pragma unroll
            for (int jj = 0; jj < NT; ++jj)
            {
                int const cl = (wm * MT + i) * 32;
                if (jj == 0)
                {
                    blockScales = load_block_scales<EPI>(scales(j & 1, 0) + cl, scales(j & 1, 1) + cl);
                }
                store_block_scaled<IL_OUT, EPI, true, IL_OUT && (EPI == kAFFINE || EPI == kGELU)>(
                    p, acc[i][jj], n0 + cl, t0 + (wn * NT + jj) * 32, blockScales);
            }
        }
        n0 = n1;
        t0 = t1;
#pragma unroll
        for (int q = 0; q < LA; ++q)
        {
            oaC[q] = oaN[q];
        }
#pragma unroll
        for (int q = 0; q < LB; ++q)
        {
            obC[q] = obN[q];
        }
    }
    // the loads requested for a tile after the last one are still in flight: they must land before the LDS is released
    wait_vmcnt<0>();
}

// Tokens [0, 256*tokMain) are cut into 256 x 256 tiles (workgroups 0 .. mainTiles-1); what is left, which
// would otherwise be a last round of big tiles on a fraction of the CUs, is cut into 128 x 128 tiles that
// spread over all of them.
constexpr int kBig = kBigTile;
constexpr int kSmall = 128;

template <bool IL_W, bool IL_IN, bool IL_OUT, int EPI>
__global__ __launch_bounds__(512) void int8_linear_kernel(LinearArgs const p)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * 2 * (kBig / 32) * 2 * 1024];
    __shared__ __attribute__((aligned(16))) float sAlpha[kBig];
    __shared__ __attribute__((aligned(16))) float sBeta[kBig];
    if ((int) blockIdx.x < p.mainTiles)
    {
        // Each XCD (own 4 MB L2) works through a contiguous run of tile numbers.  Tiles are numbered
        // panel by panel, a panel being `panel` channel tiles wide: inside a panel the channel tile varies
        // fastest, then the token tile.  The 32 workgroups resident on an XCD then cover 32/panel token
        // tiles x panel channel tiles, and the next 32 reuse the same weights from L2.
        uint32_t const pw = (uint32_t) p.panel;
        uint32_t const perPanel = (uint32_t) p.tokMain * pw;
        uint32_t const tile = xcd_remap(blockIdx.x, (uint32_t) p.mainTiles);
        uint32_t const pan = tile / perPanel, rem = tile % perPanel;
        linear_tile<2, 4, 4, 2, IL_W, IL_IN, IL_OUT, EPI>(
            p, (int) (pan * pw + rem % pw) * kBig, (int) (rem / pw) * kBig, lds, sAlpha, sBeta);
    }
    else
    {
        uint32_t const nbm = (uint32_t) ((p.N + kSmall - 1) / kSmall);
        uint32_t const tile = blockIdx.x - (uint32_t) p.mainTiles;
        linear_tile<2, 4, 2, 1, IL_W, IL_IN, IL_OUT, EPI>(
            p, (int) (tile % nbm) * kSmall, p.tokMain * kBig + (int) (tile / nbm) * kSmall, lds, sAlpha, sBeta);
    }
}

// The same tile plan run by persistent workgroups (K % 128 == 0): workgroups 0 .. persist-1 take the
// 256 x 256 tiles b, b + persist, ... in the panel numbering, the workgroups after them one 128 x 128 tile each.
template <bool IL_W, bool IL_IN, bool IL_OUT, int EPI>
__global__ __launch_bounds__(512) void int8_linear_persistent_kernel(LinearArgs const p)
{
    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * 2 * (kBig / 32) * 2 * 1024];
    __shared__ __attribute__((aligned(16))) float sScale[2 * 2 * kBig];
    if ((int) blockIdx.x < p.persist)
    {
        uint32_t const pw = (uint32_t) p.panel;
        uint32_t const perPanel = (uint32_t) p.tokMain * pw;
        int const count = (p.mainTiles - (int) blockIdx.x + p.persist - 1) / p.persist;
        auto origin = [&](int j, int& n0, int& t0) {
            uint32_t const tile = xcd_remap(blockIdx.x + (uint32_t) j * (uint32_t) p.persist, (uint32_t) p.mainTiles);
            uint32_t const pan = tile / perPanel, rem = tile % perPanel;
            n0 = (int) (pan * pw + rem % pw) * kBig;
            t0 = (int) (rem / pw) * kBig;
        };
        linear_tile_run<2, 4, 4, 2, IL_W, IL_IN, IL_OUT, EPI>(p, count, origin, lds, sScale);
    }
    else
    {
        uint32_t const nbm = (uint32_t) ((p.N + kSmall - 1) / kSmall);
        uint32_t const tile = blockIdx.x - (uint32_t) p.persist;
        auto origin = [&](int, int& n0, int& t0) {
            n0 = (int) (tile % nbm) * kSmall;
            t0 = p.tokMain * kBig + (int) (tile / nbm) * kSmall;
        };
        linear_tile_run<2, 4, 2, 1, IL_W, IL_IN, IL_OUT, EPI>(p, 1, origin, lds, sScale);
    }
}

// A 64-channel x 64-token piece of the output for the tokens behind the large tiles, interleaved INT8 operands,
// when those tokens would make only a few 128 x 128 tiles (a long k loop on a few CUs while the others idle).
// The eight wavefronts split k, not the piece: wavefront w multiplies the k-slabs w, w + 8, ... of all four 32 x 32
// blocks.  In the interleaved layout a fragment (32 rows x 32 bytes of one k-slab) is 1 KB of consecutive memory in
// exactly the order the MFMA wants it from the lanes, so every fragment is one 16-byte load per lane straight into the
// operand registers: no LDS stage, no barrier in the loop, and no byte is fetched twice by the workgroup.  The eight
// partial accumulators meet in LDS (8 x 16 KB), four wavefronts add them up, one block each, and run the epilogue.
// Integer addition is exact, so the result is the bits of any other order.  K % 256 == 0, N % 64 == 0.
template <bool IL_OUT, int EPI>
__device__ __forceinline__ void linear_piece64(
    LinearArgs const& p, int const n0, int const t0, uint8_t* __restrict__ lds, float* sScale)
{
    static_assert(EPI == kAFFINE || EPI == kGELU, "INT8 outputs");
    constexpr int kDepth = 4; // k-slabs in flight per wavefront
    int const lane = threadIdx.x & 63;
    int const wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int const row = lane & 31, half = lane >> 5;
    // channel and token rows of this lane in the two row blocks of each operand; tokens beyond T re-read the last one
    uint32_t offA[2], offB[2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
    {
        offA[b] = (uint32_t) (n0 + 32 * b + row) * 32u + (uint32_t) half * 16u;
        offB[b] = (uint32_t) min(t0 + 32 * b + row, p.T - 1) * 32u + (uint32_t) half * 16u;
    }
    uint32_t const slabA = (uint32_t) p.N * 32u, slabB = (uint32_t) p.T * 32u;
    int const steps = p.K / 256; // k-slabs of this wavefront
    if (threadIdx.x < 64)
    {
        sScale[threadIdx.x] = p.alpha[n0 + threadIdx.x];
        sScale[kBigTile + threadIdx.x] = p.beta[n0 + threadIdx.x];
    }
    i32x4 fa[kDepth][2], fb[kDepth][2];
    auto fetch = [&](int slot, int step) {
        uint32_t const ks = (uint32_t) (min(step, steps - 1) * 8 + wave);
#pragma unroll
        for (int b = 0; b < 2; ++b)
        {
            fa[slot][b] = *reinterpret_cast<i32x4 const*>(p.w + (size_t) ks * slabA + offA[b]);
            fb[slot][b] = *reinterpret_cast<i32x4 const*>(p.a + (size_t) ks * slabB + offB[b]);
        }
    };
    AccT<EPI> acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
    {
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
#pragma unroll
            for (int v = 0; v < 16; ++v)
            {
                acc[i][j][v] = 0;
            }
        }
    }
#pragma unroll
    for (int d = 0; d < kDepth; ++d)
    {
        fetch(d, d);
    }
    for (int s0 = 0; s0 < steps; s0 += kDepth)
    {
#pragma unroll
        for (int d = 0; d < kDepth; ++d)
        {
            if (s0 + d < steps)
            {
#pragma unroll
                for (int i = 0; i < 2; ++i)
                {
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                    {
                        acc[i][j] = mma<EPI>(fa[d][i], fb[d][j], acc[i][j]);
                    }
                }
                fetch(d, s0 + d + kDepth); // loads behind the last slab re-read it and are never used
            }
        }
    }
    // partial accumulators: [wavefront][block][four registers][lane], 16 bytes per lane and access
    i32x4* const part = reinterpret_cast<i32x4*>(lds);
#pragma unroll
    for (int i = 0; i < 2; ++i)
    {
#pragma unroll
        for (int j = 0; j < 2; ++j)
        {
#pragma unroll
            for (int q = 0; q < 4; ++q)
            {
                part[(((wave * 4) + (i * 2 + j)) * 4 + q) * 64 + lane]
                    = i32x4{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
            }
        }
    }
    __syncthreads();
    if (wave < 4)
    {
        AccT<EPI> sum;
#pragma unroll
        for (int q = 0; q < 4; ++q)
        {
            i32x4 t = part[((wave) * 4 + q) * 64 + lane];
#pragma unroll
            for (int w = 1; w < 8; ++w)
            {
                t += part[(((w * 4) + wave) * 4 + q) * 64 + lane];
            }
            sum[4 * q] = t[0];
            sum[4 * q + 1] = t[1];
            sum[4 * q + 2] = t[2];
            sum[4 * q + 3] = t[3];
        }
        int const cb = (wave >> 1) * 32, tb = (wave & 1) * 32;
        store_block<IL_OUT, EPI>(p, sum, n0 + cb, t0 + tb, sScale + cb, sScale + kBigTile + cb);
    }
}

// The persistent tile plan with direct-to-LDS loads for the 256 x 256 tiles.
template <bool IL, bool IL_OUT, int EPI>
__global__ __launch_bounds__(512) void int8_linear_dma_kernel(LinearArgs const p)
{
    __shared__ __attribute__((aligned(1024))) uint8_t lds[4 * 2 * (kBig / 32) * 2 * 1024];
    __shared__ __attribute__((aligned(16))) float sScale[2 * 2 * kBig];
    if ((int) blockIdx.x < p.persist)
    {
        uint32_t const pw = (uint32_t) p.panel;
        uint32_t const perPanel = (uint32_t) p.tokMain * pw;
        int const count = (p.mainTiles - (int) blockIdx.x + p.persist - 1) / p.persist;
        auto origin = [&](int j, int& n0, int& t0) {
            uint32_t const tile = xcd_remap(blockIdx.x + (uint32_t) j * (uint32_t) p.persist, (uint32_t) p.mainTiles);
            uint32_t const pan = tile / perPanel, rem = tile % perPanel;
            n0 = (int) (pan * pw + rem % pw) * kBig;
            t0 = (int) (rem / pw) * kBig;
        };
        linear_tile_run_dma<IL, IL_OUT, EPI>(p, count, origin, lds, sScale);
    }
    else
    {
        uint32_t const tile = blockIdx.x - (uint32_t) p.persist;
        if constexpr (IL && (EPI == kAFFINE || EPI == kGELU))
        {
            if (p.pieces)
            {
                uint32_t const nbm = (uint32_t) p.N / 64u;
                linear_piece64<IL_OUT, EPI>(p, (int) (tile % nbm) * 64, p.tokMain * kBig + (int) (tile / nbm) * 64, lds,
                    sScale);
                return;
            }
        }
        uint32_t const nbm = (uint32_t) ((p.N + kSmall - 1) / kSmall);
        auto origin = [&](int, int& n0, int& t0) {
            n0 = (int) (tile % nbm) * kSmall;
            t0 = p.tokMain * kBig + (int) (tile / nbm) * kSmall;
        };
        linear_tile_run<2, 4, 2, 1, IL, IL, IL_OUT, EPI>(p, 1, origin, lds, sScale);
    }
}

template <bool IL_W, bool IL_IN, bool IL_OUT, int EPI>
int launch_shape(hipStream_t stream, LinearArgs a)
{
    // big tiles for as many whole token-tile rows as fit in full rounds of one workgroup per CU
    int const nbmBig = ceil_div(a.N, kBig);
    int64_t const bigTiles = (int64_t) nbmBig * (a.T / kBig);
    int const cus = num_cus();
    // ... plus a last partial round when it would occupy more than `partial` per cent of the CUs: in 128 x 128
    // tiles that remainder needs three rounds or more, which take longer than one round of large tiles
    int const partial = tuning(Tuning::kLinearPartialRound);
    int64_t roundedTiles = (bigTiles / cus) * cus;
    if ((bigTiles - roundedTiles) * 100 > (int64_t) partial * cus)
    {
        roundedTiles = bigTiles;
    }
    a.tokMain = (int) (roundedTiles / nbmBig);
    a.mainTiles = a.tokMain * nbmBig;
    constexpr int kMaxPanel = 8; // 8 x 256 channels x K = 1024 of weights is half of an XCD's 4 MB L2
    a.panel = 1;
    for (int w = 1; w <= kMaxPanel && w <= nbmBig; ++w)
    {
        if (nbmBig % w == 0)
        {
            a.panel = w;
        }
    }
    int const restTokens = a.T - a.tokMain * kBig;
    int64_t const grid = (int64_t) a.mainTiles + (int64_t) ceil_div(a.N, kSmall) * ceil_div(restTokens, kSmall);
    if (grid >= (int64_t) 1 << 31)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "int8_linear: too many tiles");
    }
    int const persistent = tuning(Tuning::kLinearPersistent);
    if (persistent && a.K % 128 == 0)
    {
        a.persist = a.mainTiles < cus ? a.mainTiles : cus;
        int64_t const pgrid = grid - a.mainTiles + a.persist;
        int const direct = tuning(Tuning::kLinearDirect);
        if constexpr (IL_W == IL_IN && (EPI == kAFFINE || EPI == kGELU || EPI == kF16_AFFINE || EPI == kF16_GELU))
        {
            if (direct && a.N % kBig == 0 && a.K % 256 == 0 && a.mainTiles > 0)
            {
                int64_t dgrid = pgrid;
                if constexpr (IL_W && (EPI == kAFFINE || EPI == kGELU))
                {
                    // few 128 x 128 tiles behind the large ones (no more than TRTAMD_LINEAR_PIECES per cent of the CUs
                    // busy with a long k loop each): the same tokens as 64 x 64 pieces whose wavefronts split k
                    // (linear_piece64)
                    int64_t const smallTiles = grid - a.mainTiles;
                    if (restTokens > 0 && smallTiles * 100 <= (int64_t) tuning(Tuning::kLinearPieces) * cus)
                    {
                        a.pieces = 1;
                        dgrid = (int64_t) a.persist + (int64_t) (a.N / 64) * ceil_div(restTokens, 64);
                    }
                }
                hipLaunchKernelGGL((int8_linear_dma_kernel<IL_W, IL_OUT, EPI>), dim3((uint32_t) dgrid), dim3(512), 0, stream,
                    a);
                return check_launch("int8_linear_dma_kernel");
            }
        }
        hipLaunchKernelGGL((int8_linear_persistent_kernel<IL_W, IL_IN, IL_OUT, EPI>), dim3((uint32_t) pgrid), dim3(512), 0,
            stream, a);
        return check_launch("int8_linear_persistent_kernel");
    }
    hipLaunchKernelGGL((int8_linear_kernel<IL_W, IL_IN, IL_OUT, EPI>), dim3((uint32_t) grid), dim3(512), 0, stream, a);
    return check_launch("int8_linear_kernel");
}

template <bool IL_W, bool IL_IN>
int launch_out(hipStream_t stream, LinearArgs const& a, int epilogue, bool ilOut)
{
    switch (epilogue)
    {
    case kAFFINE:
        return ilOut ? launch_shape<IL_W, IL_IN, true, kAFFINE>(stream, a)
                     : launch_shape<IL_W, IL_IN, false, kAFFINE>(stream, a);
    case kGELU:
        return ilOut ? launch_shape<IL_W, IL_IN, true, kGELU>(stream, a)
                     : launch_shape<IL_W, IL_IN, false, kGELU>(stream, a);
    case kRAW: return launch_shape<IL_W, IL_IN, false, kRAW>(stream, a);
    case kHALF: return launch_shape<IL_W, IL_IN, false, kHALF>(stream, a);
    default: return set_error(TRTAMD_STATUS_BAD_PARAM, "int8_linear: unknown epilogue %d", epilogue);
    }
}

} // namespace
} // namespace trtamd

extern "C" int trtamd_int8_linear(trtamd_stream_t stream, trtamd_int8_linear_params const* p)
{
    using namespace trtamd;
    if (p == nullptr || p->a == nullptr || p->w == nullptr || p->out == nullptr)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "int8_linear: null pointer");
    }
    if (p->T < 0 || p->K <= 0 || p->N <= 0 || p->K % 64 != 0 || p->N % 32 != 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "int8_linear: T=%d K=%d N=%d (K must be a multiple of 64, N of 32)",
            p->T, p->K, p->N);
    }
    if (p->epilogue != TRTAMD_LINEAR_RAW_INT32 && (p->alpha == nullptr || p->beta == nullptr))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "int8_linear: alpha and beta are required by this epilogue");
    }
    bool const wideOut = p->epilogue == TRTAMD_LINEAR_RAW_INT32 || p->epilogue == TRTAMD_LINEAR_AFFINE_FP16;
    if (wideOut && p->out_interleaved)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "int8_linear: INT32 and FP16 outputs are linear only");
    }
    if ((int64_t) p->T * p->K >= (int64_t) 1 << 31 || (int64_t) p->N * p->K >= (int64_t) 1 << 31)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "int8_linear: operand of 2 GiB or more");
    }
    if (!aligned16(p->a) || !aligned16(p->w) || !aligned16(p->out) || (p->alpha && !aligned16(p->alpha))
        || (p->beta && !aligned16(p->beta)))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "int8_linear: pointers must be 16-byte aligned");
    }
    if (p->T == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    LinearArgs a{p->a, p->w, p->alpha, p->beta, p->out, p->T, p->K, p->N, p->out_scale, 0, 0, 1, 0};
    bool const ilOut = p->out_interleaved != 0;
    hipStream_t const st = as_stream(stream);
    if (p->w_interleaved)
    {
        return p->a_interleaved ? launch_out<true, true>(st, a, p->epilogue, ilOut)
                                : launch_out<true, false>(st, a, p->epilogue, ilOut);
    }
    return p->a_interleaved ? launch_out<false, true>(st, a, p->epilogue, ilOut)
                            : launch_out<false, false>(st, a, p->epilogue, ilOut);
}

extern "C" int trtamd_fp16_linear(trtamd_stream_t stream, trtamd_fp16_linear_params const* p)
{
    using namespace trtamd;
    if (p == nullptr || p->a == nullptr || p->w == nullptr || p->out == nullptr || p->alpha == nullptr
        || p->beta == nullptr)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fp16_linear: null pointer");
    }
    if (p->T < 0 || p->K <= 0 || p->N <= 0 || p->K % 32 != 0 || p->N % 32 != 0)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fp16_linear: T=%d K=%d N=%d (K and N must be multiples of 32)", p->T,
            p->K, p->N);
    }
    if (p->epilogue != TRTAMD_LINEAR_AFFINE && p->epilogue != TRTAMD_LINEAR_GELU)
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fp16_linear: unknown epilogue %d", p->epilogue);
    }
    if ((int64_t) p->T * p->K >= (int64_t) 1 << 30 || (int64_t) p->N * p->K >= (int64_t) 1 << 30)
    {
        return set_error(TRTAMD_STATUS_NOT_SUPPORTED, "fp16_linear: operand of 2 GiB or more");
    }
    if (!aligned16(p->a) || !aligned16(p->w) || !aligned16(p->out) || !aligned16(p->alpha) || !aligned16(p->beta))
    {
        return set_error(TRTAMD_STATUS_BAD_PARAM, "fp16_linear: pointers must be 16-byte aligned");
    }
    if (p->T == 0)
    {
        return TRTAMD_STATUS_SUCCESS;
    }
    LinearArgs a{reinterpret_cast<int8_t const*>(p->a), reinterpret_cast<int8_t const*>(p->w), p->alpha, p->beta, p->out,
        p->T, 2 * p->K, p->N, 1.f, 0, 0, 1, 0};
    hipStream_t const st = as_stream(stream);
    return p->epilogue == TRTAMD_LINEAR_GELU ? launch_shape<false, false, false, kF16_GELU>(st, a)
                                             : launch_shape<false, false, false, kF16_AFFINE>(st, a);
}
