/*
 * C-ABI kernel layer of the MI355X BERT-encoder plugin library (libtrtamd_bert_plugins.so).
 *
 * Every entry point takes plain device pointers, sizes, scales and a HIP stream, launches
 * hand-written gfx950 kernels asynchronously on that stream and returns an int status
 * (0 = success, non-zero = invalid argument / unsupported size / launch error; nothing is
 * thrown, nothing allocates, nothing synchronises).  The IPluginV3 host classes in the same
 * library call these functions from enqueue(); tests and benches call them through ctypes.
 *
 * Each declaration names the function of the reference plugin library it stands in for
 * (paths relative to the reference root), with the same argument order and meaning, so a
 * maintainer can bind it where the reference calls its own CUDA launcher.
 */
#ifndef TRTAMD_BERT_KERNELS_H
#define TRTAMD_BERT_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C"
{
#endif

#define TRTAMD_API __attribute__((visibility("default")))

/* hipStream_t, passed as an opaque pointer (ABI-identical to cudaStream_t in the reference). */
typedef void* trtamd_stream_t;
/* IEEE binary16 storage. */
typedef uint16_t trtamd_half_t;

enum
{
    TRTAMD_STATUS_SUCCESS = 0,         /* pluginStatus_t::STATUS_SUCCESS, plugin/common/plugin.h:34-41 */
    TRTAMD_STATUS_FAILURE = 1,         /* STATUS_FAILURE */
    TRTAMD_STATUS_BAD_PARAM = 2,       /* STATUS_BAD_PARAM */
    TRTAMD_STATUS_NOT_SUPPORTED = 3,   /* STATUS_NOT_SUPPORTED */
    TRTAMD_STATUS_NOT_INITIALIZED = 4  /* STATUS_NOT_INITIALIZED */
};

/* Library version and a human-readable description of the last error of the calling thread. */
TRTAMD_API int trtamd_version(void);
TRTAMD_API char const* trtamd_last_error(void);

/* ------------------------------------------------------------------------------------------
 * SkipLayerNorm: output = gamma * normalise(input + skip [+ bias]) + beta, row length ld,
 * n = total element count (n % ld == 0).  bias may be NULL (hasBias = false).
 * ------------------------------------------------------------------------------------------ */

/* computeSkipLayerNorm<float,hasBias>  plugin/skipLayerNormPlugin/skipLayerNormPlugin.h:42-44,
 * plugin/skipLayerNormPlugin/skipLayerNormKernel.cu:252-287 */
TRTAMD_API int trtamd_skip_layer_norm_fp32(trtamd_stream_t stream, int32_t ld, int64_t n, float const* input,
    float const* skip, float const* beta, float const* gamma, float* output, float const* bias);

/* computeSkipLayerNorm<half,hasBias>  same lines */
TRTAMD_API int trtamd_skip_layer_norm_fp16(trtamd_stream_t stream, int32_t ld, int64_t n, trtamd_half_t const* input,
    trtamd_half_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, trtamd_half_t* output,
    trtamd_half_t const* bias);

/* computeSkipLayerNormDQQ<hasBias>  plugin/skipLayerNormPlugin/skipLayerNormPlugin.h:37-40,
 * plugin/skipLayerNormPlugin/skipLayerNormKernel.cu:219-250.  INT8 rows, ld in {768,1024}. */
TRTAMD_API int trtamd_skip_layer_norm_dqq(trtamd_stream_t stream, int32_t ld, int64_t n, int8_t const* input,
    int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    trtamd_half_t const* bias, float dqScaleIn, float dqScaleSkip, float qScale);

/* launch_small_hface / launch_large_hface
 * plugin/skipLayerNormPlugin/skipLayerNormInt8InterleavedPlugin.h:35-41.
 * INT8 tensors in the 32-interleaved layout [ld/32][total][32].  One entry point per reference
 * launcher: "small" applies epsilon 2^-10 (the binary16 epsilon), "large" 2^-23 and supports
 * ld in {768,1024} only, as the reference launchers do. */
TRTAMD_API int trtamd_skipln_interleaved_small_hface(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    float dqScaleIn, float dqScaleSkip, float qScale);
TRTAMD_API int trtamd_skipln_interleaved_large_hface(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    float dqScaleIn, float dqScaleSkip, float qScale);

/* launch_small_mtron / launch_large_mtron
 * plugin/skipLayerNormPlugin/skipLayerNormInt8InterleavedPlugin.h:43-49.
 * As above plus preln = quantised (input + skip) with qSkipScale; the small variant clips preln
 * to [-127,127], the large one saturates to [-128,127], as the reference kernels do. */
TRTAMD_API int trtamd_skipln_interleaved_small_mtron(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    int8_t* preln, float dqScaleIn, float dqScaleSkip, float qScale, float qSkipScale);
TRTAMD_API int trtamd_skipln_interleaved_large_mtron(trtamd_stream_t stream, int32_t ld, int32_t total,
    int8_t const* input, int8_t const* skip, trtamd_half_t const* beta, trtamd_half_t const* gamma, int8_t* output,
    int8_t* preln, float dqScaleIn, float dqScaleSkip, float qScale, float qSkipScale);

/* ------------------------------------------------------------------------------------------
 * Embedding gather + LayerNorm.  beta/gamma are float; tables and outputs are T.
 * ------------------------------------------------------------------------------------------ */

/* embSkipLayerNorm<T>  plugin/embLayerNormPlugin/embLayerNormPlugin.h:40-43,
 * plugin/embLayerNormPlugin/embLayerNormKernel.cu:237-258.  ids/token_ids are [S,B]. */
TRTAMD_API int trtamd_emb_layer_norm_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, float const* beta, float const* gamma, float const* wordEmb,
    float const* posEmb, float const* tokEmb, int32_t wordSize, int32_t tokSize, float* output);
TRTAMD_API int trtamd_emb_layer_norm_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, float const* beta, float const* gamma,
    trtamd_half_t const* wordEmb, trtamd_half_t const* posEmb, trtamd_half_t const* tokEmb, int32_t wordSize,
    int32_t tokSize, trtamd_half_t* output);

/* embSkipLayerNormHFace<T>  plugin/embLayerNormPlugin/embLayerNormVarSeqlenPlugin.h:36-39.
 * Packed ids [T], cuSeqlens [B+1]; S is the maximum sequence length (grid bound). */
TRTAMD_API int trtamd_emb_layer_norm_hface_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, float const* wordEmb, float const* posEmb, float const* tokEmb, int32_t wordSize,
    int32_t tokSize, float* output);
TRTAMD_API int trtamd_emb_layer_norm_hface_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, trtamd_half_t const* wordEmb, trtamd_half_t const* posEmb, trtamd_half_t const* tokEmb,
    int32_t wordSize, int32_t tokSize, trtamd_half_t* output);

/* embSkipLayerNormMTron<T>  plugin/embLayerNormPlugin/embLayerNormVarSeqlenPlugin.h:41-44.
 * As HFace plus `skip` = the pre-LayerNorm embedding sum. */
TRTAMD_API int trtamd_emb_layer_norm_mtron_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, float const* wordEmb, float const* posEmb, float const* tokEmb, int32_t wordSize,
    int32_t tokSize, float* output, float* skip);
TRTAMD_API int trtamd_emb_layer_norm_mtron_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t S,
    int32_t const* inputIds, int32_t const* tokenIds, int32_t const* cuSeqlens, float const* beta,
    float const* gamma, trtamd_half_t const* wordEmb, trtamd_half_t const* posEmb, trtamd_half_t const* tokEmb,
    int32_t wordSize, int32_t tokSize, trtamd_half_t* output, trtamd_half_t* skip);

/* computeMaskIdx  plugin/embLayerNormPlugin/embLayerNormPlugin.h:38,
 * plugin/embLayerNormPlugin/embLayerNormKernel.cu:159-183.  mask [S,B] -> maskIdx [B]. */
TRTAMD_API int trtamd_compute_mask_idx(
    trtamd_stream_t stream, int32_t S, int32_t B, int32_t const* mask, int32_t* maskIdx);

/* convertMask  plugin/embLayerNormPlugin/embLayerNormPlugin.h:45-46,
 * plugin/embLayerNormPlugin/embLayerNormKernel.cu:41-96.  [S,B] int mask -> packed bit mask
 * [B][xmmas_m][warps_m*warps_n*warps_k*32] (argument order as in the reference: stream last). */
TRTAMD_API int trtamd_convert_mask(uint32_t S, uint32_t B, uint32_t warps_m, uint32_t warps_n, uint32_t warps_k,
    int32_t const* inputMaskSB, uint32_t* inputMaskX, trtamd_stream_t stream);

/* ------------------------------------------------------------------------------------------
 * Attention
 * ------------------------------------------------------------------------------------------ */

/* computeScaledSoftmax<T> / computeMaskedScaledSoftmax<T>
 * plugin/bertQKVToContextPlugin/mhaRunner.cu:196-344.  input/output [B,N,ld,ld];
 * maskIdx == NULL selects the unmasked form. */
TRTAMD_API int trtamd_scaled_softmax_fp32(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t N,
    float rsqrtHeadSize, int32_t const* maskIdx, float const* input, float* output);
TRTAMD_API int trtamd_scaled_softmax_fp16(trtamd_stream_t stream, int32_t ld, int32_t B, int32_t N,
    float rsqrtHeadSize, int32_t const* maskIdx, trtamd_half_t const* input, trtamd_half_t* output);

/* UnfusedMHARunner::run  plugin/bertQKVToContextPlugin/mhaRunner.cu:527-601 with the geometry of
 * MHARunner::setup (plugin/bertQKVToContextPlugin/mhaRunner.h:62-83): qkv [S,B,N,3,d], output
 * [S,B,N,d], maskIdx [B] or NULL, workspace of trtamd_unfused_mha_workspace_size bytes (the reference's two S x S
 * matrices per batch and head; required, and written only for head sizes d > 128 — other shapes run in one launch
 * that never stores a score: up to 512 keys a query's scores stay in registers, beyond that the keys are walked twice).
 * type: 0 = fp32, 1 = fp16 (nvinfer1::DataType values). */
TRTAMD_API size_t trtamd_unfused_mha_workspace_size(int32_t type, int32_t S, int32_t B, int32_t N);
TRTAMD_API int trtamd_unfused_mha(trtamd_stream_t stream, int32_t type, int32_t S, int32_t B, int32_t N, int32_t d,
    void const* qkv, int32_t const* maskIdx, void* output, void* workspace);

/* The algorithm choice of the unfused runner.  The reference times cuBLAS's batched-GEMM algorithms for the configured
 * shape once, when the runner is set up, keeps the two winners (mAlgoBatchedEx1 / mAlgoBatchedEx2) in its serialised
 * state and passes them to every later product (tuneBatchedGemm and UnfusedMHARunner::setup / serialize,
 * plugin/bertQKVToContextPlugin/mhaRunner.cu:346-444, 476-507, 527-601).  Here what there is to choose for a shape is
 * the route: one launch that stores no score, or the three launches with the score matrices in the workspace.
 * trtamd_unfused_mha_tune times the routes that exist for the shape on buffers of its own (allocated and freed inside
 * the call: it is for configuration time, not for enqueue; the batch is cut down for the timing when the workspace
 * would exceed 1 GiB) and returns the faster one in *route and, when `microseconds` is not NULL, the two times
 * (microseconds[0] one launch, [1] three launches; -1 for a route that does not exist or was not timed).  When nothing
 * can be timed (no device memory for the buffers) it returns TRTAMD_UNFUSED_ROUTE_BY_SHAPE, which is also the
 * reference's default algorithm value, so that a state that was never tuned, or was written by the reference, reads as
 * "choose by shape".  trtamd_unfused_mha_routed is trtamd_unfused_mha with the route given: BY_SHAPE behaves as
 * trtamd_unfused_mha does, ONE_LAUNCH is refused for head sizes above 128, any other value is a bad parameter.
 * The routes round at the same places and differ in the order of binary32 sums only. */
#define TRTAMD_UNFUSED_ROUTE_ONE_LAUNCH 0
#define TRTAMD_UNFUSED_ROUTE_THREE_LAUNCHES 1
#define TRTAMD_UNFUSED_ROUTE_BY_SHAPE 99
TRTAMD_API int trtamd_unfused_mha_tune(int32_t type, int32_t S, int32_t B, int32_t N, int32_t d, int32_t* route,
    float* microseconds);
TRTAMD_API int trtamd_unfused_mha_routed(trtamd_stream_t stream, int32_t route, int32_t type, int32_t S, int32_t B,
    int32_t N, int32_t d, void const* qkv, int32_t const* maskIdx, void* output, void* workspace);

/* trtamd_unfused_mha for callers that cannot allocate (code under graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference: the score matrices live in a device array that belongs to
 * the library (trtamd_unfused_mha_static_capacity() bytes, 32 MiB, held by every GPU the library runs on until the
 * process ends) instead of a caller workspace.  None of the calls allocates, frees or synchronises; the array's address
 * is looked up once per device, by trtamd_unfused_mha_static_prepare() (call it with that device current before a
 * stream of that device is put into capture: the look-up may load the library's code object) or else by the first
 * trtamd_unfused_mha_static on the device.  A problem whose trtamd_unfused_mha_workspace_size exceeds the capacity is
 * refused with TRTAMD_STATUS_NOT_SUPPORTED.  All calls on one GPU share the array: calls that overlap on one GPU
 * (different streams) race; calls on one stream, or ordered by events, are safe.  The array is used, and the limit
 * applies, for the shapes whose scores go through memory (head sizes d > 128); all others run in one launch that
 * stores no score, touch nothing of the array and are accepted at any size. */
TRTAMD_API size_t trtamd_unfused_mha_static_capacity(void);
TRTAMD_API int trtamd_unfused_mha_static_prepare(void);
TRTAMD_API int trtamd_unfused_mha_static(trtamd_stream_t stream, int32_t type, int32_t S, int32_t B, int32_t N,
    int32_t d, void const* qkv, int32_t const* maskIdx, void* output);

/* Parameter block of the fused kernels: the fields of Fused_multihead_attention_params_v2
 * (plugin/bertQKVToContextPlugin/fused_multihead_attention_v2/fused_multihead_attention_v2.h:31-101)
 * and Fused_multihead_attention_params
 * (plugin/bertQKVToContextPlugin/fused_multihead_attention/fused_multihead_attention.h:286-342)
 * that the runners fill (plugin/bertQKVToContextPlugin/mhaRunner.cu:705-720, 838-863, 989-1008, 1171-1203). */
typedef struct trtamd_fmha_params
{
    void const* qkv_ptr;              /* packed QKV */
    void const* packed_mask_ptr;      /* v1 only: [b][packed_mask_stride] uint32 bit mask, else NULL */
    void* o_ptr;                      /* context output */
    int64_t qkv_stride_in_bytes;      /* bytes between consecutive tokens of one sequence */
    int64_t packed_mask_stride_in_bytes;
    int64_t o_stride_in_bytes;
    int32_t b, h, s, d;               /* batch, heads, (maximum) sequence length, head size */
    uint32_t scale_bmm1;              /* bit patterns: binary32 for INT8, half2 for FP16 */
    uint32_t scale_softmax;
    uint32_t scale_bmm2;
    int32_t enable_i2f_trick;         /* accepted; has no numerical meaning in this implementation */
    int32_t const* cu_seqlens;        /* v2: [b+1] prefix sums; NULL selects the v1 fixed layout */
    int32_t interleaved;              /* v2 INT8 only: 32-interleaved layout, strides = total tokens */
    int32_t use_int8_scale_max;       /* accepted; a softmax shift, no effect on the result */
    int32_t warps_m, warps_n;         /* v1: geometry of the packed mask (0,0 = derive from s) */
} trtamd_fmha_params;

/* FusedMultiHeadAttentionXMMAKernel::run / FusedMultiHeadAttentionXMMAKernelV2::run
 * (plugin/bertQKVToContextPlugin/fused_multihead_attention/fused_multihead_attention.h:184-199,
 *  plugin/bertQKVToContextPlugin/fused_multihead_attention_v2/fused_multihead_attention_v2.h:1080-1241):
 * one launch computes softmax(Q K^T * scale) V for every (sequence, head).
 * data_type: 1 = FP16, 2 = INT8 (nvinfer1::DataType values). */
TRTAMD_API int trtamd_fused_mha_run(trtamd_stream_t stream, int32_t data_type, trtamd_fmha_params const* params);
/* TFusedMultiHeadAttentionXMMAKernel::loadXMMAKernels
 * (plugin/bertQKVToContextPlugin/fused_multihead_attention/fused_multihead_attention.h:63-147), which loads every
 * kernel and raises its dynamic shared-memory limit when a runner is created: reserves the LDS of every fused
 * kernel of this library on the current device, so that trtamd_fused_mha_run only ever launches (the first launch
 * of a kernel otherwise does its own reservation).  Needs a GPU; idempotent. */
TRTAMD_API int trtamd_fused_mha_prepare(void);
/* isValid(headSize, s) of the same classes: 1 when a fused kernel covers (d, s). */
TRTAMD_API int trtamd_fused_mha_is_valid(int32_t data_type, int32_t d, int32_t s);

/* zeroPadding2d  plugin/bertQKVToContextPlugin/zeroPadding2d.cu:90-150: copy `height` rows of
 * spitch bytes into rows of dpitch bytes, zero-filling (dpitch > spitch) or truncating. */
TRTAMD_API int trtamd_zero_padding_2d(
    void const* src, int32_t spitch, void* dst, int32_t dpitch, int32_t height, trtamd_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* TRTAMD_BERT_KERNELS_H */
