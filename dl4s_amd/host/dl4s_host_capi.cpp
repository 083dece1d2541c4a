// C entry points over the C++ host layer (see include/dl4s_host.h).
#include "../../include/dl4s_host.h"

#include <cstdio>
#include <cstring>
#include <chrono>
#include <functional>

#include "dl4s_host.hpp"

using namespace dl4s;

namespace {

thread_local char g_err[512] = "";

int guarded(dl4s_hip_ctx *ctx, int fused, const std::function<void()> &body) {
    if (!ctx) {
        snprintf(g_err, sizeof(g_err), "ctx is NULL");
        return -1;
    }
    HIP::context() = ctx;
    HIP::fused() = fused == 1 || fused == 2;
    HIP::strictMasks() = fused == 2 || fused == 4;
    HIP::attentionHook() = fused == 3 || fused == 4;
    try {
        body();
        return 0;
    } catch (const std::exception &e) {
        snprintf(g_err, sizeof(g_err), "%s", e.what());
        return -1;
    }
}

std::optional<Tensor> mask_tensor(const float *mask, const int64_t *mshape, int mdim) {
    if (!mask) return std::nullopt;
    Shape s(mshape, mshape + mdim);
    return Tensor(mask, s);
}

void load(MultiHeadAttention &m, const dl4s_host_mha_params *p) {
    m.qDense = Tensor(p->qDense, m.qDense.shape);
    m.kDense = Tensor(p->kDense, m.kDense.shape);
    m.vDense = Tensor(p->vDense, m.vDense.shape);
    m.fc = Tensor(p->fc, m.fc.shape);
    m.norm.scale = Tensor(p->norm_scale, m.norm.scale.shape);
    m.norm.shift = Tensor(p->norm_shift, m.norm.shift.shape);
    m.dropout.isActive = false;
}

void load(PointwiseFeedForward &f, const dl4s_host_ffn_params *p) {
    f.dense1.weights = Tensor(p->w1, f.dense1.weights.shape);
    f.dense1.bias = Tensor(p->b1, f.dense1.bias.shape);
    f.dense2.weights = Tensor(p->w2, f.dense2.weights.shape);
    f.dense2.bias = Tensor(p->b2, f.dense2.bias.shape);
    f.norm.scale = Tensor(p->norm_scale, f.norm.scale.shape);
    f.norm.shift = Tensor(p->norm_shift, f.norm.shift.shape);
    f.dropout.isActive = false;
}

// runs fn `iters` times between the stream timer's begin/end and returns the last result; a timed run is preceded by as
// many untimed calls (allocations then come from the pool, and the GPU, which needs some 20 ms of load after the idle gap
// of the uploads to reach its clocks, is at speed when the timer starts)
Tensor timed(dl4s_hip_ctx *ctx, int iters, float *out_ms, const std::function<Tensor()> &fn) {
    if (iters < 1) iters = 1;
    Tensor r;
    if (out_ms) {
        for (int i = 0; i < iters; ++i) r = fn();
        HIP::check(dl4s_hip_timer_begin(ctx));
    }
    for (int i = 0; i < iters; ++i) r = fn();
    if (out_ms) {
        float ms = 0.f;
        HIP::check(dl4s_hip_timer_end(ctx, &ms));
        *out_ms = ms / iters;
    }
    return r;
}

}  // namespace

extern "C" {

const char *dl4s_host_last_error(void) { return g_err; }

int dl4s_host_sdpa(dl4s_hip_ctx *ctx, int fused, const float *q, const float *k, const float *v, const float *mask,
                   const int64_t *mshape, int mdim, int64_t B, int64_t H, int64_t Lq, int64_t Lk, int64_t dk, int64_t dv,
                   float temperature, float *out, int iters, float *out_ms) {
    return guarded(ctx, fused, [&] {
        Tensor tq(q, {B, H, Lq, dk}), tk(k, {B, H, Lk, dk}), tv(v, {B, H, Lk, dv});
        auto m = mask_tensor(mask, mshape, mdim);
        ScaledDotProductAttention layer(temperature);
        Tensor r = timed(ctx, iters, out_ms, [&] { return layer(tq, tk, tv, m ? &*m : nullptr); });
        HIP::Memory::assign(r.buffer(), out, r.count());
    });
}

int dl4s_host_mha(dl4s_hip_ctx *ctx, int fused, const float *q, const float *k, const float *v, const float *mask,
                  const int64_t *mshape, int mdim, int64_t B, int64_t Lq, int64_t Lk, int64_t D, int64_t H, int64_t dk,
                  int64_t dv, const dl4s_host_mha_params *p, float *out, int iters, float *out_ms) {
    return guarded(ctx, fused, [&] {
        Tensor tq(q, {B, Lq, D});
        // q, k and v may be the same host array (self-attention): share the tensor like the caller would
        Tensor tk = (k == q) ? tq : Tensor(k, {B, Lk, D});
        Tensor tv = (v == q) ? tq : (v == k ? tk : Tensor(v, {B, Lk, D}));
        auto m = mask_tensor(mask, mshape, mdim);
        MultiHeadAttention layer(H, D, dk, dv);
        load(layer, p);
        Tensor r = timed(ctx, iters, out_ms, [&] { return layer(tq, tk, tv, m ? &*m : nullptr); });
        HIP::Memory::assign(r.buffer(), out, r.count());
    });
}

int dl4s_host_encoder_block(dl4s_hip_ctx *ctx, int fused, const float *x, const float *mask, const int64_t *mshape, int mdim,
                            int64_t B, int64_t L, int64_t D, int64_t H, int64_t dk, int64_t dv, int64_t F,
                            const dl4s_host_mha_params *attn, const dl4s_host_ffn_params *ffn, float *out, int iters,
                            float *out_ms) {
    return guarded(ctx, fused, [&] {
        precondition(mask != nullptr, "TransformerEncoderBlock takes a mask");
        Tensor tx(x, {B, L, D});
        Tensor m(mask, Shape(mshape, mshape + mdim));
        TransformerEncoderBlock block(D, F, H, dk, dv, 0.1f);
        load(block.selfAttention, attn);
        load(block.pointwiseFeedForward, ffn);
        Tensor r = timed(ctx, iters, out_ms, [&] { return block(tx, m); });
        HIP::Memory::assign(r.buffer(), out, r.count());
    });
}

int dl4s_host_decoder_block(dl4s_hip_ctx *ctx, int fused, const float *dec, const float *enc, const float *enc_mask,
                            const int64_t *emshape, int emdim, const float *dec_mask, const int64_t *dmshape, int dmdim,
                            int64_t B, int64_t Ld, int64_t Le, int64_t D, int64_t H, int64_t dk, int64_t dv, int64_t F,
                            const dl4s_host_mha_params *self_attn, const dl4s_host_mha_params *enc_attn,
                            const dl4s_host_ffn_params *ffn, float *out, int iters, float *out_ms) {
    return guarded(ctx, fused, [&] {
        precondition(enc_mask && dec_mask, "TransformerDecoderBlock takes both masks");
        Tensor td(dec, {B, Ld, D}), te(enc, {B, Le, D});
        Tensor em(enc_mask, Shape(emshape, emshape + emdim)), dm(dec_mask, Shape(dmshape, dmshape + dmdim));
        TransformerDecoderBlock block(D, F, H, dk, dv, 0.1f);
        load(block.selfAttention, self_attn);
        load(block.encoderAttention, enc_attn);
        load(block.pointwiseFeedForward, ffn);
        Tensor r = timed(ctx, iters, out_ms, [&] { return block(td, te, em, dm); });
        HIP::Memory::assign(r.buffer(), out, r.count());
    });
}

int dl4s_host_make_encoder_masks(dl4s_hip_ctx *ctx, const int64_t *lengths, int64_t B, float *out, int64_t *out_len) {
    return guarded(ctx, 0, [&] {
        std::vector<int64_t> lens(lengths, lengths + B);
        int64_t L = 0;
        for (auto l : lens) L = std::max(L, l);
        if (out_len) *out_len = L;
        if (!out) return;
        Tensor m = makeEncoderMasks(lens);
        HIP::Memory::assign(m.buffer(), out, m.count());
    });
}

int dl4s_host_make_decoder_masks(dl4s_hip_ctx *ctx, const int64_t *lengths, int64_t B, float *out, int64_t *out_len) {
    return guarded(ctx, 0, [&] {
        std::vector<int64_t> lens(lengths, lengths + B);
        int64_t L = 0;
        for (auto l : lens) L = std::max(L, l);
        if (out_len) *out_len = L;
        if (!out) return;
        Tensor m = makeDecoderMasks(lens);
        HIP::Memory::assign(m.buffer(), out, m.count());
    });
}

struct dl4s_host_transformer {
    Transformer model;
    dl4s_hip_ctx *ctx;
};

int dl4s_host_transformer_create(dl4s_hip_ctx *ctx, const dl4s_host_transformer_config *c, const dl4s_host_transformer_params *p,
                                 dl4s_host_transformer **out) {
    if (out) *out = nullptr;
    return guarded(ctx, 1, [&] {
        precondition(c && p && out, "NULL argument");
        precondition(c->encoder_layers >= 0 && c->decoder_layers >= 0 && c->vocab_size > 0 && c->hidden_dim > 0 && c->heads > 0 &&
                         c->key_dim > 0 && c->value_dim > 0 && c->forward_dim > 0,
                     "bad transformer configuration");
        auto *t = new dl4s_host_transformer{Transformer(c->encoder_layers, c->decoder_layers, c->vocab_size, c->hidden_dim, c->heads,
                                                        c->key_dim, c->value_dim, c->forward_dim, 0.1f),
                                            ctx};
        try {
            Transformer &m = t->model;
            m.dropout.isActive = false;
            m.embedding.embeddingMatrix = Tensor(p->embedding, m.embedding.embeddingMatrix.shape);
            m.outputBias = Tensor(p->output_bias, m.outputBias.shape);
            for (int64_t i = 0; i < c->encoder_layers; ++i) {
                load(m.encoder.encoderLayers[i].selfAttention, &p->encoder_attention[i]);
                load(m.encoder.encoderLayers[i].pointwiseFeedForward, &p->encoder_ffn[i]);
            }
            for (int64_t i = 0; i < c->decoder_layers; ++i) {
                load(m.decoder.decoderLayers[i].selfAttention, &p->decoder_self_attention[i]);
                load(m.decoder.decoderLayers[i].encoderAttention, &p->decoder_encoder_attention[i]);
                load(m.decoder.decoderLayers[i].pointwiseFeedForward, &p->decoder_ffn[i]);
            }
        } catch (...) {
            delete t;
            throw;
        }
        *out = t;
    });
}

void dl4s_host_transformer_destroy(dl4s_host_transformer *t) {
    if (!t) return;
    HIP::context() = t->ctx;
    delete t;
}

int dl4s_host_transformer_forward(dl4s_hip_ctx *ctx, int fused, dl4s_host_transformer *t, const int32_t *encoder_input,
                                  int64_t enc_len, const int32_t *decoder_input, int64_t dec_len, const int64_t *encoder_lengths,
                                  const int64_t *decoder_lengths, int64_t B, float *out, int iters, float *out_ms) {
    return guarded(ctx, fused, [&] {
        precondition(t && encoder_input && decoder_input && encoder_lengths && decoder_lengths && out, "NULL argument");
        std::vector<int32_t> enc(encoder_input, encoder_input + B * enc_len), dec(decoder_input, decoder_input + B * dec_len);
        std::vector<int64_t> el(encoder_lengths, encoder_lengths + B), dl(decoder_lengths, decoder_lengths + B);
        // the masks are as long as the longest sequence (TransformerUtil.swift:30, :40): the token arrays must match
        precondition(*std::max_element(el.begin(), el.end()) == enc_len && *std::max_element(dl.begin(), dl.end()) == dec_len,
                     "the padded length must equal the longest sequence length");
        Tensor r = timed(ctx, iters, out_ms, [&] { return t->model(enc, enc_len, dec, dec_len, el, dl); });
        HIP::Memory::assign(r.buffer(), out, r.count());
    });
}

static int greedy_decode(dl4s_hip_ctx *ctx, int fused, bool cached, bool recorded, dl4s_host_transformer *t, const int32_t *input_sequence, int64_t n,
                         int32_t start_token, int32_t end_token, int64_t max_length, int32_t *out_tokens, int64_t *out_count,
                         float *out_logits, float *out_ms) {
    return guarded(ctx, fused, [&] {
        precondition(t && input_sequence && out_tokens && out_count && n > 0 && max_length >= 0, "bad argument");
        std::vector<int32_t> in(input_sequence, input_sequence + n);
        std::vector<float> logits;
        HIP::check(dl4s_hip_sync(ctx));
        const auto t0 = std::chrono::steady_clock::now();
        std::vector<int32_t> toks = cached ? t->model.greedyCached(in, start_token, end_token, max_length, out_logits ? &logits : nullptr, recorded)
                                           : t->model.greedy(in, start_token, end_token, max_length, out_logits ? &logits : nullptr);
        HIP::check(dl4s_hip_sync(ctx));
        if (out_ms) *out_ms = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
        *out_count = (int64_t)toks.size();
        std::copy(toks.begin(), toks.end(), out_tokens);
        if (out_logits) std::copy(logits.begin(), logits.end(), out_logits);
    });
}

int dl4s_host_transformer_greedy(dl4s_hip_ctx *ctx, int fused, dl4s_host_transformer *t, const int32_t *input_sequence, int64_t n,
                                 int32_t start_token, int32_t end_token, int64_t max_length, int32_t *out_tokens,
                                 int64_t *out_count, float *out_logits, float *out_ms) {
    return greedy_decode(ctx, fused, false, false, t, input_sequence, n, start_token, end_token, max_length, out_tokens, out_count, out_logits,
                         out_ms);
}

int dl4s_host_transformer_greedy_cached(dl4s_hip_ctx *ctx, int fused, dl4s_host_transformer *t, const int32_t *input_sequence,
                                        int64_t n, int32_t start_token, int32_t end_token, int64_t max_length, int recorded,
                                        int32_t *out_tokens, int64_t *out_count, float *out_logits, float *out_ms) {
    return greedy_decode(ctx, fused, true, recorded != 0, t, input_sequence, n, start_token, end_token, max_length, out_tokens, out_count, out_logits,
                         out_ms);
}

int dl4s_host_transformer_set_norm_per_token(dl4s_host_transformer *t, int per_token) {
    if (!t) return DL4S_HIP_EINVALID_ARG;
    t->model.setNormalizesPerToken(per_token != 0);
    return DL4S_HIP_OK;
}

int dl4s_host_positional_encoding(dl4s_hip_ctx *ctx, int fused, int64_t max_len, int64_t hidden, float *out) {
    return guarded(ctx, fused, [&] {
        precondition(out != nullptr && max_len >= 0, "bad argument");
        Tensor r = PositionalEncoding(hidden)(max_len);
        HIP::Memory::assign(r.buffer(), out, r.count());
    });
}

int dl4s_host_tensor_encode_json(dl4s_hip_ctx *ctx, const float *values, const int64_t *shape, int dim, char *out, size_t capacity,
                                 size_t *needed) {
    return guarded(ctx, 1, [&] {
        precondition((values || dim >= 0) && dim >= 0 && dim <= DL4S_HIP_MAX_DIM && (dim == 0 || shape), "bad argument");
        Tensor t(values, Shape(shape, shape + dim));
        const std::string js = encodeJSON(t);
        if (needed) *needed = js.size() + 1;
        if (out) {
            precondition(capacity >= js.size() + 1, "output buffer too small");
            std::memcpy(out, js.c_str(), js.size() + 1);
        }
    });
}

int dl4s_host_tensor_decode_json(dl4s_hip_ctx *ctx, const char *json, float *out_values, int64_t *out_count, int64_t *out_shape,
                                 int *out_dim) {
    return guarded(ctx, 1, [&] {
        precondition(json != nullptr, "bad argument");
        Tensor t = decodeJSON(json);
        if (out_count) *out_count = t.count();
        if (out_dim) *out_dim = t.dim();
        if (out_shape) std::copy(t.shape.begin(), t.shape.end(), out_shape);
        if (out_values) HIP::Memory::assign(t.buffer(), out_values, t.count());
    });
}

}  // extern "C"
