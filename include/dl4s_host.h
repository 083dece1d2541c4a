/*
 * dl4s_host.h -- C entry points of libdl4s_host.so, the C++ host layer that mirrors DL4S's Tensor and
 * layer interfaces (dl4s_amd/host/dl4s_host.hpp) on top of libdl4s_hip.so.  They exist so that a test
 * or benchmark harness in any language can drive whole layers: every function uploads its host inputs,
 * runs the layer `iters` times on the GPU (when out_ms != NULL: `iters` untimed calls first, then `iters` calls timed
 * with the context's stream timer),
 * downloads the last result and returns 0, or -1 with the text in dl4s_host_last_error().
 *
 * `fused` selects the execution mode of the host layer: 0 issues exactly the engine primitive calls the
 * reference's tensor operators issue; 1 lets the layers use the backend's fused entry points; 2 is 1 with
 * DL4S_SDPA_STRICT on every attention call (no tile skipping: NaN / Inf in keys or values at blocked
 * positions then reach the output as in the reference); 3 is 0 with the fused attention call in
 * ScaledDotProductAttention only - what a DL4S checkout gets from the engine conformance plus the hook in
 * ScaledDotProductAttention.callAsFunction, every other layer untouched - and 4 is 3 with DL4S_SDPA_STRICT.
 * A mask pointer may be NULL (no mask); mshape/mdim describe the mask tensor handed to the layer
 * (float, 1 = blocked), which must be broadcastable to [B,H,Lq,Lk].
 */
#ifndef DL4S_HOST_H
#define DL4S_HOST_H

#include "dl4s_hip.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct dl4s_host_mha_params {
    const float *qDense, *kDense, *vDense, *fc; /* [D,H*dk], [D,H*dk], [D,H*dv], [H*dv,D] */
    const float *norm_scale, *norm_shift;       /* [D] */
} dl4s_host_mha_params;

typedef struct dl4s_host_ffn_params {
    const float *w1, *b1, *w2, *b2;       /* [D,F], [F], [F,D], [D] */
    const float *norm_scale, *norm_shift; /* [D] */
} dl4s_host_ffn_params;

const char *dl4s_host_last_error(void);

/* ScaledDotProductAttention(temperature)((q, k, v, mask)) -- NN/Models/Transformer/ScaledDotProductAttention.swift:43 */
int dl4s_host_sdpa(dl4s_hip_ctx *ctx, int fused, const float *q, const float *k, const float *v, const float *mask,
                   const int64_t *mshape, int mdim, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv,
                   float temperature, float *out, int iters, float *out_ms);
/* MultiHeadAttention(heads, hiddenDim, keyDim, valueDim)((q, k, v, mask)), dropout inactive -- MultiHeadAttention.swift:97 */
int dl4s_host_mha(dl4s_hip_ctx *ctx, int fused, const float *q, const float *k, const float *v, const float *mask,
                  const int64_t *mshape, int mdim, int64_t B, int64_t Lq, int64_t Lk, int64_t D, int64_t H, int64_t dk,
                  int64_t dv, const dl4s_host_mha_params *p, float *out, int iters, float *out_ms);
/* TransformerEncoderBlock((inputs, mask)) -- TransformerEncoderBlock.swift:58 */
int dl4s_host_encoder_block(dl4s_hip_ctx *ctx, int fused, const float *x, const float *mask, const int64_t *mshape, int mdim,
                            int64_t B, int64_t L, int64_t D, int64_t H, int64_t dk, int64_t dv, int64_t F,
                            const dl4s_host_mha_params *attn, const dl4s_host_ffn_params *ffn, float *out, int iters,
                            float *out_ms);
/* TransformerDecoderBlock((decoderInput, encoderOutput, encoderMask, decoderMask)) -- TransformerDecoderBlock.swift:61 */
int dl4s_host_decoder_block(dl4s_hip_ctx *ctx, int fused, const float *dec, const float *enc, const float *enc_mask,
                            const int64_t *emshape, int emdim, const float *dec_mask, const int64_t *dmshape, int dmdim,
                            int64_t B, int64_t Ld, int64_t Le, int64_t D, int64_t H, int64_t dk, int64_t dv, int64_t F,
                            const dl4s_host_mha_params *self_attn, const dl4s_host_mha_params *enc_attn,
                            const dl4s_host_ffn_params *ffn, float *out, int iters, float *out_ms);
/* makeEncoderMasks / makeDecoderMasks -- TransformerUtil.swift:29-50.  out may be NULL to query *out_len only;
 * encoder mask is [B,1,1,maxLen], decoder mask [B,1,maxLen,maxLen]. */
int dl4s_host_make_encoder_masks(dl4s_hip_ctx *ctx, const int64_t *lengths, int64_t B, float *out, int64_t *out_len);
int dl4s_host_make_decoder_masks(dl4s_hip_ctx *ctx, const int64_t *lengths, int64_t B, float *out, int64_t *out_len);

/* ---- the model wrapper: Transformer (NN/Models/Transformer/Transformer.swift:29-138), dropout inactive.
 * The object keeps its weights on the device between calls. */
typedef struct dl4s_host_transformer dl4s_host_transformer;
typedef struct dl4s_host_transformer_config {
    int64_t encoder_layers, decoder_layers, vocab_size, hidden_dim, heads, key_dim, value_dim, forward_dim;
} dl4s_host_transformer_config;
typedef struct dl4s_host_transformer_params {
    const float *embedding;   /* [vocab, hidden]: Embedding.embeddingMatrix, shared with the output projection */
    const float *output_bias; /* [vocab] */
    const dl4s_host_mha_params *encoder_attention; /* [encoder_layers] */
    const dl4s_host_ffn_params *encoder_ffn;       /* [encoder_layers] */
    const dl4s_host_mha_params *decoder_self_attention, *decoder_encoder_attention; /* [decoder_layers] each */
    const dl4s_host_ffn_params *decoder_ffn;       /* [decoder_layers] */
} dl4s_host_transformer_params;

int dl4s_host_transformer_create(dl4s_hip_ctx *ctx, const dl4s_host_transformer_config *config,
                                 const dl4s_host_transformer_params *params, dl4s_host_transformer **out);
void dl4s_host_transformer_destroy(dl4s_host_transformer *t);
/* callAsFunction((encoderInput, decoderInput, encoderInputLengths, decoderInputLengths)) -- Transformer.swift:101-115.
 * Tokens are [B, enc_len] / [B, dec_len] int32 with -1 as padding; out is [B, dec_len, vocab] log-probabilities. */
int dl4s_host_transformer_forward(dl4s_hip_ctx *ctx, int fused, dl4s_host_transformer *t, const int32_t *encoder_input,
                                  int64_t enc_len, const int32_t *decoder_input, int64_t dec_len, const int64_t *encoder_lengths,
                                  const int64_t *decoder_lengths, int64_t B, float *out, int iters, float *out_ms);
/* callAsFunction(inputSequence:startToken:endToken:maxLength:) -- Transformer.swift:118-137.  out_tokens holds up to
 * max_length tokens, *out_count how many were produced; out_logits (may be NULL) receives the [count, vocab] rows the
 * argmax was taken over; out_ms (may be NULL) the wall time of the whole decode in milliseconds. */
int dl4s_host_transformer_greedy(dl4s_hip_ctx *ctx, int fused, dl4s_host_transformer *t, const int32_t *input_sequence,
                                 int64_t n, int32_t start_token, int32_t end_token, int64_t max_length, int32_t *out_tokens,
                                 int64_t *out_count, float *out_logits, float *out_ms);
/* No counterpart in the reference.  per_token != 0 makes every MultiHeadAttention of the model normalise each token by
 * itself (its LayerNorm input viewed as [batch * length, hidden]) instead of over (length, hidden) jointly as
 * MultiHeadAttention.swift:123-124 with LayerNorm.swift:62-77 does: the conventional Transformer, the only form whose
 * decoding can be cached.  Applies to forward and greedy as well. */
int dl4s_host_transformer_set_norm_per_token(dl4s_host_transformer *t, int per_token);
/* No counterpart in the reference.  Greedy decoding with key / value caches: each step runs the decoder on the one new
 * position (dl4s_hip_sdpa_decode_step_at_f32 over the layer's cache, dl4s_hip_sdpa_decode_f32 over the encoder states'
 * projections) instead of re-running the prefix.  The step's token and position stay in device memory, so every step
 * issues the same calls: with recorded != 0 (and max_length of at least 16: recording costs a few steps) they are
 * recorded into a HIP graph at the second step and replayed from then on, with recorded == 0 issued one by one (same
 * results, bit for bit).  Other arguments as
 * dl4s_host_transformer_greedy.  Requires fused mode,
 * head dim 64 and a model set to normalise per token (error otherwise: with the reference's joint normalisation a cache
 * computes a different function).  For such a model it returns the tokens of dl4s_host_transformer_greedy, and the same
 * logits up to summation order. */
int dl4s_host_transformer_greedy_cached(dl4s_hip_ctx *ctx, int fused, dl4s_host_transformer *t, const int32_t *input_sequence,
                                        int64_t n, int32_t start_token, int32_t end_token, int64_t max_length, int recorded,
                                        int32_t *out_tokens, int64_t *out_count, float *out_logits, float *out_ms);
/* PositionalEncoding(hiddenSize)(maxLen) -> [maxLen, hiddenSize] -- PositionalEncoding.swift:52-69 */
int dl4s_host_positional_encoding(dl4s_hip_ctx *ctx, int fused, int64_t max_len, int64_t hidden, float *out);

/* Tensor: Codable (Tensor/TensorExt.swift:241-271) as Foundation's JSONEncoder writes it:
 * {"requiresGradient":Bool,"data":"<base64 of the little-endian fp32 elements>","shape":[Int]}.
 * encode: host values -> device tensor -> JSON text (out may be NULL to query *needed, which includes the NUL);
 * decode: JSON text -> device tensor -> host values (out_values / out_shape may be NULL to query *out_count, *out_dim). */
int dl4s_host_tensor_encode_json(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim, char *out, size_t capacity,
                                 size_t *needed);
int dl4s_host_tensor_decode_json(dl4s_hip_ctx *ctx, const char *json, float *out_values, int64_t *out_count, int64_t *out_shape,
                                 int *out_dim);

#ifdef __cplusplus
}
#endif
#endif
