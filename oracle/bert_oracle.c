/*
 * CPU oracle for the BERT encoder plugin hot path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in scalar C, what each GPU kernel of the reference computes, with the
 * reference's intermediate data types (binary16 arithmetic is emulated by rounding a double
 * result to the nearest binary16 after every operation).  Nothing in the shipped library links
 * or calls it: only the tests, the smoke check and the CPU-baseline leg of the benchmark do.
 *
 * Each function cites the reference source it follows (paths relative to the reference root).
 *
 * What a CPU restatement cannot restate, and therefore leaves PARITY UNPINNED at bit level:
 *   - cub::BlockReduce lives in CCCL (v3.4.0-rc0, fetched at configure time by
 *     cmake/modules/FetchCCCL.cmake:22, absent from the checkout).  Its published default algorithm
 *     (BLOCK_REDUCE_WARP_REDUCTIONS) is restated in block_reduce_pair below: a shuffle-down tree
 *     inside every 32-lane warp, then lane 0 adds the warp aggregates in warp order.  Per-thread
 *     partial sums are formed exactly as the kernels form them.  Whether the installed CCCL build
 *     specialises differently for a given type is not checkable here, so binary16 LayerNorm
 *     statistics stay unpinned at bit level (they are pinned to float64 within binary16 accuracy).
 *     The binary32 softmax sums are added in index order (differences of a few ulp).
 *   - the inside of the fused-attention cubins (SASS only).  Rounding is fixed here as
 *     round-to-nearest-even with saturation to [-128,127], softmax in binary32.
 *   - cuBLAS binary16 GEMM accumulation order/width in the unfused path
 *     (plugin/bertQKVToContextPlugin/mhaRunner.cu:557-574).  binary32 accumulation, one rounding.
 * The closed-form / brute-force checks that pin everything else live in tests/test_oracle_*.py.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include <float.h>

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------ */
/* binary16 emulation                                                                          */
/* ------------------------------------------------------------------------------------------ */

static float h2f(uint16_t h)
{
    uint32_t sign = (uint32_t) (h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0)
    {
        if (man == 0)
        {
            bits = sign;
        }
        else
        {
            /* subnormal: value = man * 2^-24 */
            float v = (float) man * 5.9604644775390625e-08f;
            memcpy(&bits, &v, 4);
            bits |= sign;
        }
    }
    else if (exp == 31)
    {
        bits = sign | 0x7f800000u | (man << 13);
    }
    else
    {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* Round a double to the nearest binary16 (ties to even); return the bit pattern. */
static uint16_t d2h(double x)
{
    if (isnan(x))
    {
        return 0x7e00u;
    }
    uint16_t sign = signbit(x) ? 0x8000u : 0u;
    double a = fabs(x);
    if (a >= 65520.0) /* halfway between 65504 and 2^16 rounds to infinity */
    {
        return sign | 0x7c00u;
    }
    if (a < 6.103515625e-05) /* below the smallest normal: quantum 2^-24 */
    {
        double q = nearbyint(a * 16777216.0); /* default rounding mode = ties to even */
        return sign | (uint16_t) q;           /* q == 1024 yields the smallest normal */
    }
    int e;
    double m = frexp(a, &e); /* a = m * 2^e, m in [0.5,1) */
    /* 11 significant bits: scale m to [1024,2048) */
    double q = nearbyint(m * 2048.0);
    if (q >= 2048.0)
    {
        q = 1024.0;
        e += 1;
    }
    int be = e - 1 + 15; /* biased exponent of 1.xxx * 2^(e-1) */
    return sign | (uint16_t) (be << 10) | (uint16_t) ((int) q - 1024);
}

static float hr(double x)
{
    return h2f(d2h(x));
}

ORC_API void orc_f32_to_f16(float const* src, uint16_t* dst, int64_t n)
{
    for (int64_t i = 0; i < n; ++i)
    {
        dst[i] = d2h((double) src[i]);
    }
}

ORC_API void orc_f16_to_f32(uint16_t const* src, float* dst, int64_t n)
{
    for (int64_t i = 0; i < n; ++i)
    {
        dst[i] = h2f(src[i]);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* integer conversion helpers  (plugin/common/common.cuh:482-526)                              */
/* ------------------------------------------------------------------------------------------ */

/* cvt.rni.sat.s32.f32 followed by cvt.pack.sat.s8.s32: nearest-even, saturate to [-128,127].
 * NaN converts to 0 in cvt.rni.sat. */
static int8_t sat8_rne(float v)
{
    if (isnan(v))
    {
        return 0;
    }
    float r = nearbyintf(v);
    if (r > 127.f)
    {
        r = 127.f;
    }
    if (r < -128.f)
    {
        r = -128.f;
    }
    return (int8_t) r;
}

/* quantize(): __float2int_rn(qScale * x) clipped to [-127,127]  (common.cuh:506-511). */
static int8_t quantize127(float x, float qScale)
{
    float p = qScale * x;
    float r;
    if (isnan(p))
    {
        r = 0.f;
    }
    else
    {
        r = nearbyintf(p);
    }
    if (r > 127.f)
    {
        r = 127.f;
    }
    if (r < -127.f)
    {
        r = -127.f;
    }
    return (int8_t) r;
}

ORC_API void orc_float4_to_char4(float const* v, int8_t* out, int64_t n)
{
    for (int64_t i = 0; i < n; ++i)
    {
        out[i] = sat8_rne(v[i]);
    }
}

ORC_API void orc_quantize(float const* v, float qScale, int8_t* out, int64_t n)
{
    for (int64_t i = 0; i < n; ++i)
    {
        out[i] = quantize127(v[i], qScale);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* SkipLayerNorm, floating point  (plugin/skipLayerNormPlugin/skipLayerNormKernel.cu:108-302)   */
/* ------------------------------------------------------------------------------------------ */

/* Arithmetic in the kernel's type T: is_half selects binary16 (every op rounded) or binary32. */
static inline float t_add(int is_half, float a, float b)
{
    return is_half ? hr((double) a + (double) b) : a + b;
}
static inline float t_sub(int is_half, float a, float b)
{
    return is_half ? hr((double) a - (double) b) : a - b;
}
static inline float t_mul(int is_half, float a, float b)
{
    return is_half ? hr((double) a * (double) b) : a * b;
}
static inline float t_div(int is_half, float a, float b)
{
    return is_half ? hr((double) a / (double) b) : a / b;
}
static inline float t_rsqrt(int is_half, float a)
{
    return is_half ? hr(1.0 / sqrt((double) a)) : (float) (1.0 / sqrt((double) a));
}

/*
 * cub::BlockReduce<T, TPB>::Reduce with the default BLOCK_REDUCE_WARP_REDUCTIONS algorithm, for a
 * pair of values reduced together (kvp<T> / half2 with a component-wise sum), TPB a multiple of 32:
 *   inside each warp, for offset = 1, 2, 4, 8, 16: lane l adds the value lane l+offset held before
 *   the step (when l+offset < 32); lane 0 ends with the warp aggregate;
 *   thread 0 then adds the aggregates of warps 1, 2, ... to its own, in that order.
 */
static void block_reduce_pair(int is_half, int nthreads, float const* p1, float const* p2, float* o1, float* o2)
{
    float tot1 = 0.f, tot2 = 0.f;
    for (int w0 = 0; w0 < nthreads; w0 += 32)
    {
        float a[32], b[32];
        int nl = nthreads - w0 < 32 ? nthreads - w0 : 32;
        for (int l = 0; l < 32; ++l)
        {
            a[l] = l < nl ? p1[w0 + l] : 0.f;
            b[l] = l < nl ? p2[w0 + l] : 0.f;
        }
        for (int off = 1; off < 32; off <<= 1)
        {
            for (int l = 0; l + off < nl; ++l) /* ascending l reads lanes not yet updated in this step */
            {
                a[l] = t_add(is_half, a[l], a[l + off]);
                b[l] = t_add(is_half, b[l], b[l + off]);
            }
        }
        if (w0 == 0)
        {
            tot1 = a[0];
            tot2 = b[0];
        }
        else
        {
            tot1 = t_add(is_half, tot1, a[0]);
            tot2 = t_add(is_half, tot2, b[0]);
        }
    }
    *o1 = tot1;
    *o2 = tot2;
}

/*
 * One row of computeSkipLayerNorm<T,hasBias>.
 * Dispatch (skipLayerNormKernel.cu:261-282): ld<=32 -> skipLayerNormKernelSmall (one element per
 * thread, no epsilon); ld in {768,1024} -> skipln_vec (VPT = 16/sizeof(T) consecutive elements
 * per thread, epsilon = numeric_limits<T>::epsilon()); otherwise skipLayerNormKernel (thread t
 * owns elements t, t+256, ...; no epsilon).
 * v, the residual sum, is formed in T; mean and mean-of-squares accumulate rld*v and rld*v*v
 * in T; output = gamma*(v-mu)*rsigma + beta evaluated left to right in T.
 */
static void skipln_row(int is_half, int ld, float const* in, float const* skip, float const* beta, float const* gamma,
    float const* bias, float* out, float* vbuf, float* part1, float* part2)
{
    float const rld = t_div(is_half, 1.f, (float) (is_half ? hr((double) ld) : (float) ld));
    int vec = (ld == 768 || ld == 1024);
    int small = (ld <= 32);
    int vpt = is_half ? 8 : 4;
    int nthreads = vec ? ld / vpt : (small ? 32 : 256);
    for (int t = 0; t < nthreads; ++t)
    {
        part1[t] = 0.f;
        part2[t] = 0.f;
    }
    for (int i = 0; i < ld; ++i)
    {
        float v = t_add(is_half, in[i], skip[i]);
        if (bias)
        {
            v = t_add(is_half, v, bias[i]);
        }
        vbuf[i] = v;
    }
    if (vec)
    {
        for (int t = 0; t < nthreads; ++t)
        {
            for (int it = 0; it < vpt; ++it)
            {
                float v = vbuf[t * vpt + it];
                float tmp = t_mul(is_half, rld, v);
                part1[t] = t_add(is_half, part1[t], tmp);
                part2[t] = t_add(is_half, part2[t], t_mul(is_half, tmp, v));
            }
        }
    }
    else
    {
        for (int i = 0; i < ld; ++i)
        {
            int t = i % nthreads;
            float v = vbuf[i];
            float tmp = t_mul(is_half, rld, v);
            part1[t] = t_add(is_half, part1[t], tmp);
            part2[t] = t_add(is_half, part2[t], t_mul(is_half, tmp, v));
        }
    }
    float mu, m2;
    block_reduce_pair(is_half, nthreads, part1, part2, &mu, &m2);
    float var = t_sub(is_half, m2, t_mul(is_half, mu, mu));
    if (vec)
    {
        float eps = is_half ? 0.0009765625f : FLT_EPSILON;
        var = t_add(is_half, var, eps);
    }
    float rsigma = t_rsqrt(is_half, var);
    for (int i = 0; i < ld; ++i)
    {
        float y = t_mul(is_half, gamma[i], t_sub(is_half, vbuf[i], mu));
        y = t_mul(is_half, y, rsigma);
        out[i] = t_add(is_half, y, beta[i]);
    }
}

ORC_API int orc_skipln_f32(int ld, int64_t rows, float const* in, float const* skip, float const* beta,
    float const* gamma, float const* bias, float* out)
{
    float* vbuf = (float*) malloc(sizeof(float) * (size_t) ld);
    float part1[256], part2[256];
    for (int64_t r = 0; r < rows; ++r)
    {
        skipln_row(0, ld, in + r * ld, skip + r * ld, beta, gamma, bias, out + r * ld, vbuf, part1, part2);
    }
    free(vbuf);
    return 0;
}

ORC_API int orc_skipln_f16(int ld, int64_t rows, uint16_t const* in, uint16_t const* skip, uint16_t const* beta,
    uint16_t const* gamma, uint16_t const* bias, uint16_t* out)
{
    size_t n = (size_t) ld;
    float* buf = (float*) malloc(sizeof(float) * n * 7);
    float *fi = buf, *fs = buf + n, *fb = buf + 2 * n, *fg = buf + 3 * n, *fbias = buf + 4 * n, *fo = buf + 5 * n,
          *vbuf = buf + 6 * n;
    float part1[256], part2[256];
    orc_f16_to_f32(beta, fb, ld);
    orc_f16_to_f32(gamma, fg, ld);
    if (bias)
    {
        orc_f16_to_f32(bias, fbias, ld);
    }
    for (int64_t r = 0; r < rows; ++r)
    {
        orc_f16_to_f32(in + r * ld, fi, ld);
        orc_f16_to_f32(skip + r * ld, fs, ld);
        skipln_row(1, ld, fi, fs, fb, fg, bias ? fbias : NULL, fo, vbuf, part1, part2);
        for (int i = 0; i < ld; ++i)
        {
            out[r * ld + i] = d2h((double) fo[i]);
        }
    }
    free(buf);
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* SkipLayerNorm INT8, linear layout: skiplnDQQ  (skipLayerNormKernel.cu:43-106, 219-250)       */
/* ------------------------------------------------------------------------------------------ */

/* binary16 LN core shared by skiplnDQQ, skiplnDQQ_vec3 and skiplnDQQ_vec4: thread t owns 8
 * consecutive channels; per element: tmp = rld*v; (sum, sumsq) += (tmp, tmp*v) as one half2 add.
 * y = float(gamma*(v-mu)*rsigma + beta) with the product chain in binary16 (the reference's
 * expression has __half operands throughout, converted to float on assignment). */
static void dqq_half_core(int ld, float const* v /* binary16 values */, float const* beta, float const* gamma,
    int rsqrt_in_float, float* y)
{
    float const rld = hr(1.0 / (double) hr((double) ld));
    int nthreads = ld / 8;
    float part1[512], part2[512];
    for (int t = 0; t < nthreads; ++t)
    {
        float p1 = 0.f, p2 = 0.f;
        for (int it = 0; it < 8; ++it)
        {
            float x = v[t * 8 + it];
            float tmp = hr((double) rld * x);
            p1 = hr((double) p1 + tmp);
            p2 = hr((double) p2 + hr((double) tmp * x));
        }
        part1[t] = p1;
        part2[t] = p2;
    }
    float mu, m2;
    block_reduce_pair(1, nthreads, part1, part2, &mu, &m2);
    float var = hr((double) hr((double) m2 - hr((double) mu * mu)) + 0.0009765625);
    float rsigma;
    if (rsqrt_in_float)
    {
        /* rsqrtf(float(half)) assigned to a __half  (skipLayerNormInt8InterleavedKernelHFace.cu:314) */
        rsigma = hr((double) (float) (1.0 / sqrt((double) var)));
    }
    else
    {
        rsigma = hr(1.0 / sqrt((double) var));
    }
    for (int i = 0; i < ld; ++i)
    {
        float a = hr((double) gamma[i] * hr((double) v[i] - mu));
        a = hr((double) a * rsigma);
        y[i] = hr((double) a + beta[i]);
    }
}

ORC_API int orc_skipln_dqq(int ld, int64_t rows, int8_t const* in, int8_t const* skip, uint16_t const* beta,
    uint16_t const* gamma, uint16_t const* bias, int8_t* out, float dqScaleIn, float dqScaleSkip, float qScale)
{
    if (ld != 768 && ld != 1024)
    {
        return 1; /* "unsupported hidden layer size"  (skipLayerNormKernel.cu:244-246) */
    }
    size_t n = (size_t) ld;
    float* buf = (float*) malloc(sizeof(float) * n * 5);
    float *fb = buf, *fg = buf + n, *fbias = buf + 2 * n, *v = buf + 3 * n, *y = buf + 4 * n;
    orc_f16_to_f32(beta, fb, ld);
    orc_f16_to_f32(gamma, fg, ld);
    if (bias)
    {
        orc_f16_to_f32(bias, fbias, ld);
    }
    for (int64_t r = 0; r < rows; ++r)
    {
        for (int i = 0; i < ld; ++i)
        {
            /* float expression dqScaleIn*tmpIn + dqScaleSkip*tmpSkip assigned to a __half */
            float f = dqScaleIn * (float) in[r * ld + i] + dqScaleSkip * (float) skip[r * ld + i];
            float h = hr((double) f);
            if (bias)
            {
                h = hr((double) h + fbias[i]);
            }
            v[i] = h;
        }
        dqq_half_core(ld, v, fb, fg, 0, y);
        for (int i = 0; i < ld; ++i)
        {
            out[r * ld + i] = sat8_rne(y[i] * qScale);
        }
    }
    free(buf);
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* SkipLayerNorm INT8, 32-interleaved layout [ld/32][total][32]                                 */
/*   small: skiplnDQQ_vec3 / skiplnDQQ_vec4                                                     */
/*     (skipLayerNormInt8InterleavedKernelHFace.cu:261-359, ...MTron.cu:281-411)                */
/*   large: skipln_vec32_hface / skipln_vec32_mtron  (HFace.cu:47-259, MTron.cu:47-279)         */
/* ------------------------------------------------------------------------------------------ */

static inline int64_t il_index(int c, int64_t t, int64_t total)
{
    return (int64_t) (c / 32) * total * 32 + t * 32 + (c % 32);
}

/* variant: 0 = HFace (no preln), 1 = MTron (preln written).  The plugin picks the small kernel
 * when total < 4096 (skipLayerNormInt8InterleavedPlugin.cpp:301-307, 345-352); `force` overrides:
 * -1 follow the plugin rule, 0 small, 1 large. */
ORC_API int orc_skipln_interleaved(int variant, int force, int ld, int64_t total, int8_t const* in,
    int8_t const* skip, uint16_t const* beta, uint16_t const* gamma, int8_t* out, int8_t* preln, float dqScaleIn,
    float dqScaleSkip, float qScale, float qSkipScale)
{
    int large = force < 0 ? (total >= 4096) : force;
    if (large)
    {
        if (ld != 768 && ld != 1024)
        {
            return 1;
        }
    }
    else if (variant == 0)
    {
        if (ld != 768 && ld != 1024)
        {
            return 1;
        }
    }
    else
    {
        if (ld != 768 && ld != 1024 && ld != 1536 && ld != 2048 && ld != 3072 && ld != 4096)
        {
            return 1;
        }
    }
    size_t n = (size_t) ld;
    float* buf = (float*) malloc(sizeof(float) * n * 4);
    float *fb = buf, *fg = buf + n, *v = buf + 2 * n, *y = buf + 3 * n;
    orc_f16_to_f32(beta, fb, ld);
    orc_f16_to_f32(gamma, fg, ld);
    for (int64_t t = 0; t < total; ++t)
    {
        if (!large)
        {
            for (int c = 0; c < ld; ++c)
            {
                int64_t idx = il_index(c, t, total);
                float f = dqScaleIn * (float) in[idx] + dqScaleSkip * (float) skip[idx];
                v[c] = hr((double) f);
            }
            if (variant == 1)
            {
                for (int c = 0; c < ld; ++c)
                {
                    preln[il_index(c, t, total)] = quantize127(v[c], qSkipScale);
                }
            }
            dqq_half_core(ld, v, fb, fg, 1, y);
            for (int c = 0; c < ld; ++c)
            {
                out[il_index(c, t, total)] = sat8_rne(y[c] * qScale);
            }
        }
        else
        {
            /* Thread (row, half) owns, for ii in {0,1}, the 16 bytes of channel group
             * (ii*HEADS + row) starting at byte half*16.  Its partial is accumulated in half2 over
             * the 32 values in that order; partials of the two threads of a token position are
             * added (shfl xor 1), then the rows of a warp (xor 8, 16), then the warps. */
            float const rld = 1.f / (float) ld;
            int heads = ld / 64;
            int nrows = heads; /* kROWS_PER_LDG */
            for (int c = 0; c < ld; ++c)
            {
                int64_t idx = il_index(c, t, total);
                v[c] = (float) in[idx] * dqScaleIn + (float) skip[idx] * dqScaleSkip;
            }
            if (variant == 1)
            {
                for (int c = 0; c < ld; ++c)
                {
                    preln[il_index(c, t, total)] = sat8_rne(v[c] * qSkipScale);
                }
            }
            float row1[64][2], row2[64][2];
            for (int row = 0; row < nrows; ++row)
            {
                for (int hf = 0; hf < 2; ++hf)
                {
                    float p1 = 0.f, p2 = 0.f;
                    for (int ii = 0; ii < 2; ++ii)
                    {
                        for (int k = 0; k < 16; ++k)
                        {
                            int c = (ii * nrows + row) * 32 + hf * 16 + k;
                            float tmp = v[c] * rld;
                            p1 = hr((double) p1 + hr((double) tmp));
                            p2 = hr((double) p2 + hr((double) (tmp * v[c])));
                        }
                    }
                    row1[row][hf] = p1;
                    row2[row][hf] = p2;
                }
            }
            /* xor 1: the two halves; xor 8,16: the 4 rows of one warp (8 threads per row, 32 per
             * warp); then warp 0 adds warps 1.. in order. */
            int nwarps = nrows / 4;
            float mu = 0.f, m2 = 0.f;
            for (int w = 0; w < nwarps; ++w)
            {
                float a1[4], a2[4];
                for (int r = 0; r < 4; ++r)
                {
                    a1[r] = hr((double) row1[w * 4 + r][0] + row1[w * 4 + r][1]);
                    a2[r] = hr((double) row2[w * 4 + r][0] + row2[w * 4 + r][1]);
                }
                float b1 = hr((double) hr((double) a1[0] + a1[1]) + hr((double) a1[2] + a1[3]));
                float b2 = hr((double) hr((double) a2[0] + a2[1]) + hr((double) a2[2] + a2[3]));
                if (w == 0)
                {
                    mu = b1;
                    m2 = b2;
                }
                else
                {
                    mu = hr((double) mu + b1);
                    m2 = hr((double) m2 + b2);
                }
            }
            float rsigma = (float) (1.0 / sqrt((double) (m2 - mu * mu + FLT_EPSILON)));
            /* (mu, rsigma) travel through a half2 in shared memory */
            mu = hr((double) mu);
            rsigma = hr((double) rsigma);
            for (int c = 0; c < ld; ++c)
            {
                float yy = fg[c] * rsigma * (v[c] - mu) + fb[c];
                out[il_index(c, t, total)] = sat8_rne(yy * qScale);
            }
        }
    }
    free(buf);
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Embedding gather + LayerNorm                                                                 */
/*   fixed length : embLayerNormKernel       (plugin/embLayerNormPlugin/embLayerNormKernel.cu:185-258) */
/*   var-seqlen   : embLayerNormKernelHFace  (embLayerNormVarSeqlenKernelHFace.cu:38-126)        */
/*                  embLayerNormKernelMTron  (embLayerNormVarSeqlenKernelMTron.cu:38-127)        */
/*   LN core      : layerNorm<T,T,float,256> (plugin/common/common.cuh:253-281), no epsilon      */
/* ------------------------------------------------------------------------------------------ */

/* One token.  pre (may be NULL) receives v = (word + tok) + pos in T.  Returns 0 when the ids are
 * out of range: the reference then leaves the row's pre-LN values unwritten and normalises
 * whatever the output buffer held, which no restatement can follow; the oracle reports it. */
static int embln_token(int is_half, int ld, int32_t wordId, int32_t tokenId, int32_t pos, float const* beta,
    float const* gamma, float const* wordEmb, float const* posEmb, float const* tokEmb, int32_t wordSize,
    int32_t tokSize, float* out, float* pre)
{
    if (!(wordId >= 0 && wordId < wordSize && tokenId >= 0 && tokenId < tokSize))
    {
        return 0;
    }
    float const rld = t_div(is_half, 1.f, is_half ? hr((double) ld) : (float) ld);
    float part1[256], part2[256];
    for (int t = 0; t < 256; ++t)
    {
        part1[t] = 0.f;
        part2[t] = 0.f;
    }
    for (int i = 0; i < ld; ++i)
    {
        float w = wordEmb[(int64_t) wordId * ld + i];
        float tk = tokEmb[(int64_t) tokenId * ld + i];
        float p = posEmb[(int64_t) pos * ld + i];
        float v = t_add(is_half, t_add(is_half, w, tk), p);
        out[i] = v;
        if (pre)
        {
            pre[i] = v;
        }
        float rv = t_mul(is_half, rld, v);
        int t = i % 256;
        part1[t] = t_add(is_half, part1[t], rv);
        part2[t] = t_add(is_half, part2[t], t_mul(is_half, rv, v));
    }
    float mu, m2;
    block_reduce_pair(is_half, 256, part1, part2, &mu, &m2);
    float rsigma = t_rsqrt(is_half, t_sub(is_half, m2, t_mul(is_half, mu, mu)));
    for (int i = 0; i < ld; ++i)
    {
        float g = is_half ? hr((double) gamma[i]) : gamma[i];
        float b = is_half ? hr((double) beta[i]) : beta[i];
        float y = t_mul(is_half, g, t_sub(is_half, out[i], mu));
        y = t_mul(is_half, y, rsigma);
        out[i] = t_add(is_half, y, b);
    }
    return 1;
}

/*
 * mode 0: fixed [S,B] inputs (index s*B+b), output row s*B+b, position row s.
 * mode 1: HFace var-seqlen, token cu[b]+s for s < cu[b+1]-cu[b] and s < S, position row s.
 * mode 2: MTron = mode 1 + pre-LN sum written to `skipOut`.
 * Tables and outputs are binary32 arrays holding T values (the caller converts for binary16).
 * `valid` (one byte per output row, may be NULL) is set to 1 for rows the oracle defined.
 */
ORC_API int orc_embln(int mode, int is_half, int ld, int B, int S, int32_t const* inputIds,
    int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta, float const* gamma, float const* wordEmb,
    float const* posEmb, float const* tokEmb, int32_t wordSize, int32_t tokSize, float* out, float* skipOut,
    uint8_t* valid)
{
    for (int b = 0; b < B; ++b)
    {
        int len = S;
        int64_t base = 0;
        if (mode != 0)
        {
            base = cuSeqlens[b];
            len = cuSeqlens[b + 1] - cuSeqlens[b];
            if (len > S)
            {
                len = S; /* grid.x = S: positions beyond the bucket are never launched */
            }
        }
        for (int s = 0; s < len; ++s)
        {
            int64_t seqPos = (mode == 0) ? ((int64_t) s * B + b) : (base + s);
            float* pre = (mode == 2) ? (skipOut + seqPos * ld) : NULL;
            int ok = embln_token(is_half, ld, inputIds[seqPos], tokenIds[seqPos], s, beta, gamma, wordEmb, posEmb,
                tokEmb, wordSize, tokSize, out + seqPos * ld, pre);
            if (valid)
            {
                valid[seqPos] = (uint8_t) ok;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* maskIdx and packed mask  (plugin/embLayerNormPlugin/embLayerNormKernel.cu:41-183)            */
/* ------------------------------------------------------------------------------------------ */

ORC_API int orc_mask_idx(int S, int B, int32_t const* mask, int32_t* maskIdx)
{
    for (int b = 0; b < B; ++b)
    {
        int m = S;
        for (int s = 0; s < S; ++s)
        {
            if (mask[(int64_t) s * B + b] == 0 && s < m)
            {
                m = s;
            }
        }
        maskIdx[b] = m;
    }
    return 0;
}

/* The kernel stages S mask words of one batch in shared memory and reads shm_mask[offset+9]
 * with offset up to xmmas_n*16*warps_n - 16 + col; for S not a multiple of 16*warps_n it reads
 * past the staged words.  The oracle treats words at index >= S as 0 and reports that it did so
 * through the return value (count of such reads), so tests only pin sizes without over-read. */
ORC_API int64_t orc_convert_mask(uint32_t S, uint32_t B, uint32_t warps_m, uint32_t warps_n, uint32_t warps_k,
    int32_t const* inputMaskSB, uint32_t* inputMaskX)
{
    uint32_t xmmas_m = (S + 16 * warps_m - 1) / (16 * warps_m);
    uint32_t xmmas_n = (S + 16 * warps_n - 1) / (16 * warps_n);
    uint32_t threads = warps_m * warps_n * warps_k * 32;
    int64_t overreads = 0;
    for (uint32_t bi = 0; bi < B; ++bi)
    {
        for (uint32_t mi = 0; mi < xmmas_m; ++mi)
        {
            for (uint32_t tidx = 0; tidx < threads; ++tidx)
            {
                uint32_t warp = tidx / 32;
                uint32_t warp_n = warp / warps_m;
                uint32_t lane = tidx % 32;
                uint32_t col = warp_n * 16 + lane % 4 * 2;
                uint32_t mask = 0;
                for (uint32_t ni = 0; ni < xmmas_n; ++ni)
                {
                    uint32_t offset = ni * 16 * warps_n + col;
                    static int const delta[8] = {0, 1, 0, 1, 8, 9, 8, 9};
                    for (int bit = 0; bit < 8; ++bit)
                    {
                        uint32_t k = offset + (uint32_t) delta[bit];
                        int32_t m = 0;
                        if (k < S)
                        {
                            m = inputMaskSB[(int64_t) k * B + bi];
                        }
                        else
                        {
                            ++overreads;
                        }
                        mask |= (m == 1 ? 1u : 0u) << (8 * ni + bit);
                    }
                }
                inputMaskX[((int64_t) bi * xmmas_m + mi) * threads + tidx] = mask;
            }
        }
    }
    return overreads;
}

/* ------------------------------------------------------------------------------------------ */
/* Row softmax of the unfused path                                                              */
/*   scaledSoftmax{,Small}  (plugin/common/common.cuh:313-421)                                   */
/*   softmax / maskedSoftmax (plugin/bertQKVToContextPlugin/mhaRunner.cu:46-195)                 */
/* input/output [B,N,S,S] binary32 arrays holding T values; maskIdx may be NULL (all valid).    */
/* exp((x-max)*w), binary32, 1/Z multiply; positions >= lastValid are exactly 0.                */
/* ------------------------------------------------------------------------------------------ */

ORC_API int orc_scaled_softmax(int is_half, int ld, int B, int N, float rsqrtHeadSize, int32_t const* maskIdx,
    float const* input, float* output)
{
    for (int b = 0; b < B; ++b)
    {
        int lastValid = ld;
        if (maskIdx)
        {
            lastValid = maskIdx[b] < ld ? maskIdx[b] : ld;
        }
        for (int64_t r = 0; r < (int64_t) N * ld; ++r)
        {
            float const* x = input + ((int64_t) b * N * ld + r) * ld;
            float* y = output + ((int64_t) b * N * ld + r) * ld;
            float fmax = -FLT_MAX;
            for (int i = 0; i < lastValid; ++i)
            {
                fmax = x[i] > fmax ? x[i] : fmax;
            }
            float z = 0.f;
            for (int i = 0; i < lastValid; ++i)
            {
                z += expf((x[i] - fmax) * rsqrtHeadSize);
            }
            float rz = 1.f / z;
            for (int i = 0; i < ld; ++i)
            {
                float val = (i < lastValid) ? expf((x[i] - fmax) * rsqrtHeadSize) * rz : 0.f;
                y[i] = is_half ? hr((double) val) : val;
            }
        }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* Attention                                                                                    */
/* Addressing is by strides in ELEMENTS so one routine serves every layout:                     */
/*   fixed  [S,B,N,3,d]: token stride 3*B*N*d, sequence b starts at b*3*N*d, head stride 3*d,    */
/*                       Q/K/V at +0,+d,+2d  (mhaRunner.h:62-83, mhaRunner.cu:550-552)           */
/*   packed [T,N,3,d]  : token stride 3*N*d, sequence b starts at cu[b]*3*N*d                    */
/*                       (mhaRunner.cu:1006-1008, 1171-1172)                                     */
/* The 32-interleaved INT8 layout is converted by orc_interleave/orc_deinterleave.              */
/* ------------------------------------------------------------------------------------------ */

typedef struct
{
    int32_t B, N, d;
    int64_t tokStrideIn;  /* elements between consecutive tokens of one sequence, input */
    int64_t tokStrideOut; /* same, output */
    int64_t headStrideIn; /* 3*d */
    int64_t headStrideOut; /* d */
} orc_mha_geom;

/* per-sequence description: first-element offsets and number of query rows / valid keys */
typedef struct
{
    int64_t inBase;
    int64_t outBase;
    int32_t nq;   /* query rows computed and written */
    int32_t nk;   /* keys attended (prefix) */
} orc_mha_seq;

/*
 * Unfused attention, UnfusedMHARunner::run (mhaRunner.cu:527-601):
 *   A[q,k] = sum_d Q[q,d]*K[k,d] stored in T unscaled; P = softmax(A * rsqrt(d)) over k < nk,
 *   exactly 0 for k >= nk, stored in T; ctx[q,:] = sum_k P[q,k]*V[k,:] stored in T.
 * nkTotal is the score-row length S (all S keys enter the second GEMM, the masked ones with 0).
 */
ORC_API int orc_mha_unfused(int is_half, orc_mha_geom const* g, orc_mha_seq const* seqs, float const* qkv, float* out)
{
    int d = g->d;
    float const w = 1.f / sqrtf((float) d);
    for (int b = 0; b < g->B; ++b)
    {
        orc_mha_seq const* sq = &seqs[b];
        float* prob = (float*) malloc(sizeof(float) * (size_t) (sq->nk > 0 ? sq->nk : 1));
        for (int n = 0; n < g->N; ++n)
        {
            for (int q = 0; q < sq->nq; ++q)
            {
                float const* Q = qkv + sq->inBase + (int64_t) q * g->tokStrideIn + (int64_t) n * g->headStrideIn;
                float fmax = -FLT_MAX;
                for (int k = 0; k < sq->nk; ++k)
                {
                    float const* K
                        = qkv + sq->inBase + (int64_t) k * g->tokStrideIn + (int64_t) n * g->headStrideIn + d;
                    float acc = 0.f;
                    for (int j = 0; j < d; ++j)
                    {
                        acc += Q[j] * K[j];
                    }
                    if (is_half)
                    {
                        acc = hr((double) acc);
                    }
                    prob[k] = acc;
                    fmax = acc > fmax ? acc : fmax;
                }
                float z = 0.f;
                for (int k = 0; k < sq->nk; ++k)
                {
                    z += expf((prob[k] - fmax) * w);
                }
                float rz = 1.f / z;
                for (int k = 0; k < sq->nk; ++k)
                {
                    float p = expf((prob[k] - fmax) * w) * rz;
                    prob[k] = is_half ? hr((double) p) : p;
                }
                float* O = out + sq->outBase + (int64_t) q * g->tokStrideOut + (int64_t) n * g->headStrideOut;
                for (int j = 0; j < d; ++j)
                {
                    float acc = 0.f;
                    for (int k = 0; k < sq->nk; ++k)
                    {
                        float const* V = qkv + sq->inBase + (int64_t) k * g->tokStrideIn
                            + (int64_t) n * g->headStrideIn + 2 * d;
                        acc += prob[k] * V[j];
                    }
                    O[j] = is_half ? hr((double) acc) : acc;
                }
            }
        }
        free(prob);
    }
    return 0;
}

/*
 * Fused FP16 attention contract (host side: mhaRunner.cu:705-720, 989-996): scale_bmm1 = 1/sqrt(d)
 * as half2, scale_softmax = scale_bmm2 = 1.  Restated as: binary32 scores from binary16 inputs,
 * scaled by the binary16-rounded 1/sqrt(d), binary32 softmax, P rounded to binary16, binary32
 * accumulation of P*V, one rounding to binary16.
 */
ORC_API int orc_mha_fused_f16(orc_mha_geom const* g, orc_mha_seq const* seqs, float const* qkv, float* out)
{
    int d = g->d;
    float const w = hr(1.0 / sqrt((double) d));
    for (int b = 0; b < g->B; ++b)
    {
        orc_mha_seq const* sq = &seqs[b];
        float* prob = (float*) malloc(sizeof(float) * (size_t) (sq->nk > 0 ? sq->nk : 1));
        for (int n = 0; n < g->N; ++n)
        {
            for (int q = 0; q < sq->nq; ++q)
            {
                float const* Q = qkv + sq->inBase + (int64_t) q * g->tokStrideIn + (int64_t) n * g->headStrideIn;
                float* O = out + sq->outBase + (int64_t) q * g->tokStrideOut + (int64_t) n * g->headStrideOut;
                float fmax = -FLT_MAX;
                for (int k = 0; k < sq->nk; ++k)
                {
                    float const* K
                        = qkv + sq->inBase + (int64_t) k * g->tokStrideIn + (int64_t) n * g->headStrideIn + d;
                    float acc = 0.f;
                    for (int j = 0; j < d; ++j)
                    {
                        acc += Q[j] * K[j];
                    }
                    prob[k] = acc * w;
                    fmax = prob[k] > fmax ? prob[k] : fmax;
                }
                float z = 0.f;
                for (int k = 0; k < sq->nk; ++k)
                {
                    prob[k] = expf(prob[k] - fmax);
                    z += prob[k];
                }
                float rz = sq->nk > 0 ? 1.f / z : 0.f;
                for (int k = 0; k < sq->nk; ++k)
                {
                    prob[k] = hr((double) (prob[k] * rz));
                }
                for (int j = 0; j < d; ++j)
                {
                    float acc = 0.f;
                    for (int k = 0; k < sq->nk; ++k)
                    {
                        float const* V = qkv + sq->inBase + (int64_t) k * g->tokStrideIn
                            + (int64_t) n * g->headStrideIn + 2 * d;
                        acc += prob[k] * V[j];
                    }
                    O[j] = hr((double) acc);
                }
            }
        }
        free(prob);
    }
    return 0;
}

/*
 * Fused INT8 attention contract (mhaRunner.cu:838-850, 1178-1190;
 * qkvToContextInt8InterleavedPlugin.cpp:269-277):
 *   acc1[q,k] = sum_d Q*K                      (int32, exact)
 *   s = float(acc1) * scale_bmm1               (scale_bmm1 = sQ*sQ/sqrt(d))
 *   p = softmax_k(s)                            (binary32)
 *   p8 = sat8(rne(p * scale_softmax))          (scale_softmax = 1/dqProbs)
 *   acc2[q,j] = sum_k p8*V[k,j]                (int32, exact)
 *   out8 = sat8(rne(float(acc2) * scale_bmm2)) (scale_bmm2 = dqProbs*sQ/sCtx)
 * Optional outputs (may be NULL) expose the exact integers for the bit-exact checks:
 *   acc1Out [B][N][maxq][maxk] int32, p8Out same shape int8, acc2Out laid out like `out` int32.
 */
ORC_API int orc_mha_fused_i8(orc_mha_geom const* g, orc_mha_seq const* seqs, int8_t const* qkv, int8_t* out,
    float scale_bmm1, float scale_softmax, float scale_bmm2, int32_t maxq, int32_t maxk, int32_t* acc1Out,
    int8_t* p8Out, int32_t* acc2Out)
{
    int d = g->d;
#pragma omp parallel for schedule(dynamic)
    for (int b = 0; b < g->B; ++b)
    {
        orc_mha_seq const* sq = &seqs[b];
        size_t nk = (size_t) (sq->nk > 0 ? sq->nk : 1);
        int32_t* a1 = (int32_t*) malloc(sizeof(int32_t) * nk);
        float* prob = (float*) malloc(sizeof(float) * nk);
        int8_t* p8 = (int8_t*) malloc(nk);
        for (int n = 0; n < g->N; ++n)
        {
            for (int q = 0; q < sq->nq; ++q)
            {
                int8_t const* Q = qkv + sq->inBase + (int64_t) q * g->tokStrideIn + (int64_t) n * g->headStrideIn;
                float fmax = -FLT_MAX;
                for (int k = 0; k < sq->nk; ++k)
                {
                    int8_t const* K
                        = qkv + sq->inBase + (int64_t) k * g->tokStrideIn + (int64_t) n * g->headStrideIn + d;
                    int32_t acc = 0;
                    for (int j = 0; j < d; ++j)
                    {
                        acc += (int32_t) Q[j] * (int32_t) K[j];
                    }
                    a1[k] = acc;
                    prob[k] = (float) acc * scale_bmm1;
                    fmax = prob[k] > fmax ? prob[k] : fmax;
                }
                float z = 0.f;
                for (int k = 0; k < sq->nk; ++k)
                {
                    prob[k] = expf(prob[k] - fmax);
                    z += prob[k];
                }
                float rz = sq->nk > 0 ? 1.f / z : 0.f;
                for (int k = 0; k < sq->nk; ++k)
                {
                    p8[k] = sat8_rne(prob[k] * rz * scale_softmax);
                }
                if (acc1Out && q < maxq)
                {
                    int64_t o = (((int64_t) b * g->N + n) * maxq + q) * maxk;
                    for (int k = 0; k < sq->nk && k < maxk; ++k)
                    {
                        acc1Out[o + k] = a1[k];
                        if (p8Out)
                        {
                            p8Out[o + k] = p8[k];
                        }
                    }
                }
                int64_t oidx = sq->outBase + (int64_t) q * g->tokStrideOut + (int64_t) n * g->headStrideOut;
                for (int j = 0; j < d; ++j)
                {
                    int32_t acc = 0;
                    for (int k = 0; k < sq->nk; ++k)
                    {
                        int8_t const* V = qkv + sq->inBase + (int64_t) k * g->tokStrideIn
                            + (int64_t) n * g->headStrideIn + 2 * d;
                        acc += (int32_t) p8[k] * (int32_t) V[j];
                    }
                    if (acc2Out)
                    {
                        acc2Out[oidx + j] = acc;
                    }
                    out[oidx + j] = sat8_rne((float) acc * scale_bmm2);
                }
            }
        }
        free(a1);
        free(prob);
        free(p8);
    }
    return 0;
}

/* 32-interleaved <-> channel-major-per-token conversion for INT8 tensors.
 * Logical [1,C,T,1] in TensorFormat::kCHW32 is stored [C/32][T][32]
 * (qkvToContextInt8InterleavedPlugin.cpp:124-127, 280-281). */
ORC_API void orc_interleave(int8_t const* linearTC, int8_t* il, int64_t T, int C)
{
    for (int64_t t = 0; t < T; ++t)
    {
        for (int c = 0; c < C; ++c)
        {
            il[il_index(c, t, T)] = linearTC[t * C + c];
        }
    }
}

ORC_API void orc_deinterleave(int8_t const* il, int8_t* linearTC, int64_t T, int C)
{
    for (int64_t t = 0; t < T; ++t)
    {
        for (int c = 0; c < C; ++c)
        {
            linearTC[t * C + c] = il[il_index(c, t, T)];
        }
    }
}

/* zeroPadding2d (plugin/bertQKVToContextPlugin/zeroPadding2d.cu:34-88): copy a [rows, srcCols]
 * matrix into [rows, dstCols]; columns beyond srcCols are zero, columns beyond dstCols dropped.
 * Element size in bytes is a parameter (2 for binary16, 1 for INT8). */
ORC_API void orc_zero_padding_2d(void const* src, void* dst, int64_t rows, int srcCols, int dstCols, int elemSize)
{
    uint8_t const* s = (uint8_t const*) src;
    uint8_t* t = (uint8_t*) dst;
    for (int64_t r = 0; r < rows; ++r)
    {
        for (int c = 0; c < dstCols; ++c)
        {
            for (int e = 0; e < elemSize; ++e)
            {
                t[(r * dstCols + c) * elemSize + e] = c < srcCols ? s[(r * srcCols + c) * elemSize + e] : 0;
            }
        }
    }
}

/* INT8 linear layer between the plugins (QKV / output projection / feed-forward).  There is no open
 * reference source for it (TensorRT's closed core runs these layers; plugin/fcPlugin is the FP16/FP32
 * cuBLASLt stand-in, plugin/fcPlugin/README.md:41-45), so this states the arithmetic the library
 * documents in include/trtamd_encoder_ops.h:
 *   acc[t][n] = sum_k a[t][k] * w[n][k]                    exact INT32
 *   y         = fmaf((float) acc, alpha[n], beta[n])        one binary32 rounding
 *   epilogue 0: out8 = sat8(rne(y))
 *   epilogue 1: g = 0.5 * y * (1 + erf(y / sqrt 2)) evaluated in binary64 and rounded to binary32,
 *               out8 = sat8(rne(g * out_scale))
 *   epilogue 2: out32 = acc           epilogue 3: out16 = binary16(y)
 * Activations / INT8 outputs are linear [T][C] or 32-interleaved [C/32][T][32]
 * (layout of qkvToContextInt8InterleavedPlugin.cpp:124-127); weights are [N][K] with the QKV rows in
 * the [head][3][64] order of plugin/bertQKVToContextPlugin/README.md:27-30. */
ORC_API int orc_int8_linear(int64_t T, int K, int N, int8_t const* a, int aInterleaved, int8_t const* w,
    float const* alpha, float const* beta, int epilogue, float outScale, int outInterleaved, void* out)
{
    if (K <= 0 || N <= 0 || epilogue < 0 || epilogue > 3)
    {
        return 1;
    }
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t)
    {
        int8_t* row = (int8_t*) malloc((size_t) K);
        for (int k = 0; k < K; ++k)
        {
            row[k] = aInterleaved ? a[il_index(k, t, T)] : a[t * K + k];
        }
        for (int n = 0; n < N; ++n)
        {
            int8_t const* wr = w + (int64_t) n * K;
            int32_t acc = 0;
            for (int k = 0; k < K; ++k)
            {
                acc += (int32_t) row[k] * (int32_t) wr[k];
            }
            if (epilogue == 2)
            {
                ((int32_t*) out)[t * N + n] = acc;
                continue;
            }
            float const y = fmaf((float) acc, alpha[n], beta[n]);
            if (epilogue == 3)
            {
                ((uint16_t*) out)[t * N + n] = d2h((double) y);
                continue;
            }
            float r = y;
            if (epilogue == 1)
            {
                float const g = (float) (0.5 * (double) y * (1.0 + erf((double) y * 0.70710678118654752440)));
                r = g * outScale;
            }
            ((int8_t*) out)[outInterleaved ? il_index(n, t, T) : t * N + n] = sat8_rne(r);
        }
        free(row);
    }
    return 0;
}

/* IQuantizeLayer / IDequantizeLayer with a per-tensor scale, fused with the kCHW32 reformat that
 * TensorRT inserts around the interleaved plugins (include/NvInfer.h:5333-5345, 5493-5500):
 *   q = clamp(round_half_even(x / scale), -128, 127)       x = binary16(q * scale)
 * x is binary16 [T][C]; q is INT8 [C/32][T][32]. */
ORC_API void orc_quantize_f16_interleave(uint16_t const* x, float scale, int8_t* q, int64_t T, int C)
{
    for (int64_t t = 0; t < T; ++t)
    {
        for (int c = 0; c < C; ++c)
        {
            q[il_index(c, t, T)] = sat8_rne(h2f(x[t * C + c]) / scale);
        }
    }
}

ORC_API void orc_dequantize_deinterleave_f16(int8_t const* q, float scale, uint16_t* x, int64_t T, int C)
{
    for (int64_t t = 0; t < T; ++t)
    {
        for (int c = 0; c < C; ++c)
        {
            x[t * C + c] = d2h((double) ((float) q[il_index(c, t, T)] * scale));
        }
    }
}

/* FP16 linear layer (include/trtamd_encoder_ops.h, trtamd_fp16_linear): the arithmetic of a cuBLASLt FP16 GEMM
 * with binary32 accumulation as CustomFCPluginDynamic configures it (plugin/fcPlugin/fcPlugin.cpp, compute type
 * CUBLAS_COMPUTE_32F for DataType::kHALF), plus the bias / GELU TensorRT fuses after it:
 *   acc = sum_k a[t][k] * w[n][k] in binary32 (products of binary16 values are exact in binary32; the order of
 *   the additions is k = 0, 1, ... here and a tree on the GPU, hence the floating-point tolerance of the tests)
 *   y = fmaf(acc, alpha[n], beta[n]);  epilogue 1: y = 0.5 y (1 + erf(y / sqrt 2)) in binary64;  out = binary16(y). */
ORC_API int orc_fp16_linear(int64_t T, int K, int N, uint16_t const* a, uint16_t const* w, float const* alpha,
    float const* beta, int epilogue, uint16_t* out)
{
    if (K <= 0 || N <= 0 || epilogue < 0 || epilogue > 1)
    {
        return 1;
    }
    float* wf = (float*) malloc((size_t) N * K * sizeof(float));
    for (int64_t i = 0; i < (int64_t) N * K; ++i)
    {
        wf[i] = h2f(w[i]);
    }
#pragma omp parallel for schedule(static)
    for (int64_t t = 0; t < T; ++t)
    {
        float* row = (float*) malloc((size_t) K * sizeof(float));
        for (int k = 0; k < K; ++k)
        {
            row[k] = h2f(a[t * K + k]);
        }
        for (int n = 0; n < N; ++n)
        {
            float acc = 0.f;
            for (int k = 0; k < K; ++k)
            {
                acc += row[k] * wf[(int64_t) n * K + k];
            }
            double y = (double) fmaf(acc, alpha[n], beta[n]);
            if (epilogue == 1)
            {
                y = 0.5 * y * (1.0 + erf(y * 0.70710678118654752440));
            }
            out[t * N + n] = d2h(y);
        }
        free(row);
    }
    free(wf);
    return 0;
}
