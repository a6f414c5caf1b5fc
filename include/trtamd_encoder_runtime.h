/*
 * Native runner of a built INT8 BERT encoder: the part of a TensorRT engine that executes this network.
 *
 * In the reference that role is TensorRT's closed runtime (IExecutionContext::enqueueV3 walking the engine's
 * layers and calling IPluginV3OneRuntime::enqueue on the plugin layers, include/NvInferRuntime.h:3570-3600 and
 * 1140-1176).  Here it is an object that owns what a deserialised engine owns — the runtime-phase plugin
 * objects (created through the registry from their serialised fields), the device copies of the weights and
 * the activation scales — and enqueues, on one stream and without allocating or synchronising:
 *
 *   EmbLayerNorm v4 -> quantise+kCHW32 -> L x [ QKV GEMM, QKV-to-context v6, projection GEMM, SkipLayerNorm v7,
 *   feed-forward GEMM + GELU, feed-forward GEMM, SkipLayerNorm v7 ] -> dequantise+linear FP16.
 *
 * The builder's work (quantising weights, calibrating activation scales, folding scales into alpha/beta) is
 * the caller's: tensorrt_amd/encoder.py does it and hands the result over through trtamd_encoder_set_layer.
 */
#ifndef TRTAMD_ENCODER_RUNTIME_H
#define TRTAMD_ENCODER_RUNTIME_H

#include "trtamd_encoder_ops.h"

#ifdef __cplusplus
extern "C"
{
#endif

typedef struct trtamd_encoder_config
{
    int32_t hidden, heads, ffn, layers;
    int32_t vocab, max_pos, type_vocab;
    int32_t max_seqlen; /* extent of the attention plugin's "maximum sequence length" input: 64..512 */
} trtamd_encoder_config;

/* All pointers are HOST pointers; the runner copies what it needs to the GPU during the call. */
typedef struct trtamd_encoder_embedding
{
    float const* beta;  /* [hidden] */
    float const* gamma; /* [hidden] */
    float const* word;  /* [vocab][hidden] */
    float const* tok;   /* [type_vocab][hidden] */
    float const* pos;   /* [max_pos][hidden] */
    float scale;        /* quantisation scale of the embedding output (layer 0's input) */
} trtamd_encoder_embedding;

typedef struct trtamd_encoder_linear
{
    int8_t const* w;    /* [N][K] row-major INT8 */
    float const* alpha; /* [N], scales folded (see trtamd_int8_linear) */
    float const* beta;  /* [N] */
} trtamd_encoder_linear;

typedef struct trtamd_encoder_layer
{
    trtamd_encoder_linear qkv;  /* [3*hidden][hidden], rows ordered [q|k|v][head][64] */
    trtamd_encoder_linear proj; /* [hidden][hidden] */
    trtamd_encoder_linear ffn1; /* [ffn][hidden], GELU epilogue */
    trtamd_encoder_linear ffn2; /* [hidden][ffn] */
    float ffn1_out_scale;       /* 1 / scale of the GELU output */
    trtamd_half_t const* ln1_gamma;
    trtamd_half_t const* ln1_beta;
    trtamd_half_t const* ln2_gamma;
    trtamd_half_t const* ln2_beta;
    /* per-tensor activation scales: layer input, QKV, context, projection output, LN1 output, FFN2 output, LN2 output */
    float s_x, s_qkv, s_ctx, s_ao, s_h, s_f, s_out;
} trtamd_encoder_layer;

typedef void* trtamd_encoder_t;

/* NULL on failure (trtamd_last_error() says why). */
TRTAMD_API trtamd_encoder_t trtamd_encoder_create(trtamd_encoder_config const* config);
TRTAMD_API void trtamd_encoder_destroy(trtamd_encoder_t encoder);
TRTAMD_API int trtamd_encoder_set_embedding(trtamd_encoder_t encoder, trtamd_encoder_embedding const* embedding);
TRTAMD_API int trtamd_encoder_set_layer(trtamd_encoder_t encoder, int32_t index, trtamd_encoder_layer const* layer);
/* Bytes of device scratch enqueue() needs for up to max_tokens packed tokens. */
TRTAMD_API size_t trtamd_encoder_workspace_size(trtamd_encoder_t encoder, int32_t max_tokens);
/* ids, segment_ids: device int32 [tokens]; cu_seqlens: device int32 [batch + 1]; out: device binary16
 * [tokens][hidden]; workspace: device, 256-byte aligned, at least trtamd_encoder_workspace_size(tokens) bytes. */
TRTAMD_API int trtamd_encoder_enqueue(trtamd_encoder_t encoder, int32_t const* ids, int32_t const* segment_ids,
    int32_t const* cu_seqlens, int32_t batch, int32_t tokens, void* workspace, trtamd_half_t* out,
    trtamd_stream_t stream);

/* One packed batch of an enqueue: the arguments of trtamd_encoder_enqueue. */
typedef struct trtamd_encoder_batch
{
    int32_t const* ids;
    int32_t const* segment_ids;
    int32_t const* cu_seqlens; /* [batch + 1], starting at 0 for this batch */
    int32_t batch, tokens;
    void* workspace;           /* this batch's own, trtamd_encoder_workspace_size(tokens) bytes */
    trtamd_half_t* out;        /* [tokens][hidden] */
} trtamd_encoder_batch;

/* Execution contexts, the counterpart of ICudaEngine::createExecutionContext (include/NvInferRuntime.h:3087-3091: an
 * engine serves several contexts at once, each with clones of the engine's plugin objects, IPluginV3::clone,
 * include/NvInferPluginBase.h:229-239).  After every
 * set_layer call: makes `count` contexts available (1..8; the encoder starts with one), with their plugin clones,
 * streams and events, so that no later call has anything to allocate. */
TRTAMD_API int trtamd_encoder_reserve_contexts(trtamd_encoder_t encoder, int32_t count);
/* Runs `count` independent batches (count <= reserved contexts) at the same time: part 0 on `stream`, the others on
 * streams of the runner's own that start behind the work `stream` already holds and that `stream` waits for before
 * whatever is enqueued next.  Launches and records only (capturable).  Splitting one batch into two halves this way
 * fills the compute units that the tail of every kernel of the other half leaves idle: the 24-layer BERT-large pass
 * of 128 sequences takes 11.7 ms as two halves against 12.7 ms as one batch, with the same output bits. */
TRTAMD_API int trtamd_encoder_enqueue_concurrent(trtamd_encoder_t encoder, trtamd_encoder_batch const* parts,
    int32_t count, trtamd_stream_t stream);

#ifdef __cplusplus
}
#endif

#endif /* TRTAMD_ENCODER_RUNTIME_H */
