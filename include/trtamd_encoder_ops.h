/*
 * C-ABI of the encoder operations that sit BETWEEN the BERT plugins in a TensorRT engine: the INT8
 * linear layers (QKV projection, attention output projection, the two feed-forward layers) and the
 * layout / quantisation reformats either side of the interleaved plugins.  In the reference these
 * are not plugin code: TensorRT's closed core executes them (the only open counterpart is the
 * deprecated cuBLASLt plugin plugin/fcPlugin, FP32/FP16 only, plugin/fcPlugin/README.md:41-45), so
 * the semantics below are this library's own statement of an INT8 fully-connected layer with
 * folded quantisation scales.  Same calling rules as trtamd_bert_kernels.h: plain device pointers,
 * asynchronous on the given stream, int status, nothing allocates or synchronises.
 */
#ifndef TRTAMD_ENCODER_OPS_H
#define TRTAMD_ENCODER_OPS_H

#include "trtamd_bert_kernels.h"

#ifdef __cplusplus
extern "C"
{
#endif

/* What happens to the INT32 accumulator acc[t][n] = sum_k a[t][k] * w[n][k] (exact). */
enum
{
    /* y = fmaf(float(acc), alpha[n], beta[n]);  out8 = sat8(rne(y)).  alpha = s_a * s_w[n] / s_out and
     * beta = bias[n] / s_out: the caller folds the output scale, as a TensorRT build does. */
    TRTAMD_LINEAR_AFFINE = 0,
    /* y as above with alpha = s_a * s_w[n], beta = bias[n];  g = 0.5 * y * (1 + erf(y / sqrt(2)));
     * out8 = sat8(rne(g * out_scale)), out_scale = 1 / s_out. */
    TRTAMD_LINEAR_GELU = 1,
    /* out32[t][n] = acc, linear layout: the accumulators themselves, for bit-exact checks. */
    TRTAMD_LINEAR_RAW_INT32 = 2,
    /* out16[t][n] = binary16(y), linear layout: the de-quantised result (e.g. the last layer). */
    TRTAMD_LINEAR_AFFINE_FP16 = 3
};

typedef struct trtamd_int8_linear_params
{
    int8_t const* a;    /* activations: linear [T][K], or 32-interleaved [K/32][T][32] */
    int8_t const* w;    /* weights: linear [N][K] (one row of K per output channel), or 32-interleaved
                           [K/32][N][32] (the faster one: a build step reformats constant weights once).  For the QKV
                           projection the rows are ordered [head][q|k|v][64], the packing
                           plugin/bertQKVToContextPlugin/README.md:27-30 asks for. */
    float const* alpha; /* [N] */
    float const* beta;  /* [N] */
    void* out;          /* int8 [T][N] or [N/32][T][32]; int32 / binary16 [T][N] */
    int32_t T, K, N;    /* K % 64 == 0, N % 32 == 0 */
    int32_t a_interleaved;
    int32_t w_interleaved;
    int32_t out_interleaved;
    int32_t epilogue;
    float out_scale;    /* TRTAMD_LINEAR_GELU only */
} trtamd_int8_linear_params;

/* Stands where TensorRT's own INT8 fully-connected / 1x1-convolution layer runs between the plugins
 * (closed source; engine-side placement described in plugin/bertQKVToContextPlugin/README.md:25-30). */
TRTAMD_API int trtamd_int8_linear(trtamd_stream_t stream, trtamd_int8_linear_params const* params);

/* FP16 linear layer for the FP16 encoder: out[t][n] = binary16(f(fmaf(acc, alpha[n], beta[n]))), acc = sum_k
 * a[t][k] * w[n][k] accumulated in binary32 on the FP16 matrix cores, f = identity (TRTAMD_LINEAR_AFFINE) or erf-GELU
 * (TRTAMD_LINEAR_GELU).  alpha = 1 and beta = bias give the usual fully-connected layer.  All tensors linear:
 * a [T][K], w [N][K], out [T][N]; K % 32 == 0, N % 32 == 0.  The open counterpart in the reference is the deprecated
 * cuBLASLt GEMM plugin CustomFCPluginDynamic (plugin/fcPlugin/README.md:20-45, FP16 without bias or activation);
 * bias and GELU are what TensorRT's core fuses onto it. */
typedef struct trtamd_fp16_linear_params
{
    trtamd_half_t const* a;
    trtamd_half_t const* w;
    float const* alpha; /* [N] */
    float const* beta;  /* [N] */
    trtamd_half_t* out;
    int32_t T, K, N;
    int32_t epilogue;   /* TRTAMD_LINEAR_AFFINE or TRTAMD_LINEAR_GELU */
} trtamd_fp16_linear_params;

TRTAMD_API int trtamd_fp16_linear(trtamd_stream_t stream, trtamd_fp16_linear_params const* params);

/* ------------------------------------------------------------------------------------------
 * Reformats either side of the interleaved plugins.  TensorRT inserts these itself when a plugin asks
 * for TensorFormat::kCHW32 (include/NvInferRuntime.h:1471; the INT8 interleaved plugins do:
 * plugin/bertQKVToContextPlugin/qkvToContextInt8InterleavedPlugin.cpp:124-127,
 * plugin/skipLayerNormPlugin/skipLayerNormInt8InterleavedPlugin.cpp supportsFormatCombination); here
 * they are explicit calls.  "linear" is [T][C] (token-major); "interleaved" is [C/32][T][32], the
 * memory image of a [1,C,T,1] kCHW32 tensor.  C % 32 == 0.
 * ------------------------------------------------------------------------------------------ */

/* Pure layout change of INT8 data (also used once per weight matrix: [N][K] -> [K/32][N][32]). */
TRTAMD_API int trtamd_int8_linear_to_interleaved(trtamd_stream_t stream, int32_t T, int32_t C, int8_t const* in,
    int8_t* out);
TRTAMD_API int trtamd_int8_interleaved_to_linear(trtamd_stream_t stream, int32_t T, int32_t C, int8_t const* in,
    int8_t* out);

/* IQuantizeLayer with a per-tensor scale (include/NvInfer.h:5333-5345): out = clamp(round_half_even(in / scale),
 * -128, 127), fused with the reformat to the interleaved layout. */
TRTAMD_API int trtamd_quantize_fp16_to_interleaved(trtamd_stream_t stream, int32_t T, int32_t C,
    trtamd_half_t const* in, float scale, int8_t* out);

/* IDequantizeLayer with a per-tensor scale (include/NvInfer.h:5493-5500): out = binary16(in * scale), fused with
 * the reformat back to the linear layout. */
TRTAMD_API int trtamd_dequantize_interleaved_to_fp16(trtamd_stream_t stream, int32_t T, int32_t C, int8_t const* in,
    float scale, trtamd_half_t* out);

#ifdef __cplusplus
}
#endif

#endif /* TRTAMD_ENCODER_OPS_H */
