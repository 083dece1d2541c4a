"""TEST INFRASTRUCTURE, NOT PRODUCT CODE: the Transformer model wrapper of the reference, composed from the C oracle's
engine primitives and layers (oracle/binding.py) in the order the reference's tensor operators issue them.

  positional_encoding   NN/Models/Transformer/PositionalEncoding.swift:52-69
  prepare_inputs        NN/Models/Transformer/Transformer.swift:86-92
  log_softmax           Tensor/Operators/Unary.swift:198-204
  encoder, decoder      NN/Models/Transformer/TransformerEncoder.swift:61-70, TransformerDecoder.swift:47-61
  forward               NN/Models/Transformer/Transformer.swift:101-115
  greedy_decode         NN/Models/Transformer/Transformer.swift:118-137
  mha_per_token         not the reference's layer: the variant with per-token normalisation that cached decoding needs

params = {"embedding": [vocab, D], "output_bias": [vocab], "encoder": [{"attn": mha, "ffn": ffn}, ...],
          "decoder": [{"self": mha, "cross": mha, "ffn": ffn}, ...], "heads", "dk", "dv"} with mha / ffn dictionaries as
oracle.binding.mha / ffn take them.  Dropout is inactive (inference).
"""
import numpy as np

from . import binding as orc


def positional_encoding(max_len, hidden):
    assert hidden % 2 == 0, "Hidden size must be multiple of 2"
    input_range = np.arange(max_len, dtype=np.float32)
    hidden_range = np.arange(hidden // 2, dtype=np.float32)
    ratio = orc.broadcast("div", hidden_range, np.float32(hidden // 2))          # hiddenRange / Tensor(hiddenSize / 2)
    log_base = orc.log(np.array(10000.0, np.float32))                             # Tensor(10000).raised(toPowerOf:) =
    frequencies = orc.exp(orc.broadcast("mul", log_base, ratio))                  #   (log(10000) * power).exp()
    sample_points = orc.broadcast("div", input_range[:, None], frequencies[None, :])
    s, c = orc.sin(sample_points), orc.cos(sample_points)
    return np.stack([s, c], axis=2).reshape(max_len, hidden)                      # stacking along 2, view as [-1, hidden]


def prepare_inputs(params, tokens):
    tokens = np.asarray(tokens, np.int32)
    B, L = tokens.shape
    E = np.asarray(params["embedding"], np.float32)
    D = E.shape[1]
    embedded = orc.embedding(E, tokens.reshape(-1), -1).reshape(B, L, D)
    scale = orc.sqrt(np.array(float(D), np.float32))                              # Element(embedded.shape[2]).sqrt()
    return orc.broadcast("add", orc.broadcast("mul", embedded, scale), positional_encoding(L, D))


def log_softmax(x):
    x = np.asarray(x, np.float32)
    ax = x.ndim - 1
    norm = orc.broadcast("sub", x, np.expand_dims(orc.reduce_max(x, ax), ax))
    lse = orc.log(orc.reduce_sum(orc.exp(norm), [ax]))
    return orc.broadcast("sub", norm, np.expand_dims(lse, ax))


def mha_per_token(q, k, v, mask, p, heads, dk, dv):
    """MultiHeadAttention with every token normalised by itself - NOT the reference's layer, which normalises over
    (length, hidden) jointly (MultiHeadAttention.swift:123-124).  The oracle's attention output before the output
    projection, then the reference's remaining steps with the LayerNorm input viewed [batch * length, hidden]."""
    q = np.asarray(q, np.float32)
    B, Lq, D = q.shape
    _, attended = orc.mha(q, k, v, mask, p, heads, dk, dv, return_attn=True)            # [B, H, Lq, dv]
    merged = orc.permute(attended, [0, 2, 1, 3]).reshape(B, Lq, heads * dv)
    out = orc.bmm(merged, np.asarray(p["Wo"], np.float32)[None], False, False)
    summed = orc.broadcast("add", out, q)
    return orc.layernorm(summed.reshape(B * Lq, D), p["ln_scale"], p["ln_shift"]).reshape(B, Lq, D)


def encoder(params, x, lengths, norm_per_token=False):
    mask = orc.make_encoder_masks(lengths)
    for layer in params["encoder"]:
        if norm_per_token:
            x = orc.ffn(mha_per_token(x, x, x, mask, layer["attn"], params["heads"], params["dk"], params["dv"]), layer["ffn"])
        else:
            x = orc.encoder_block(x, mask, layer["attn"], layer["ffn"], params["heads"], params["dk"], params["dv"])
    return x


def decoder(params, dec_in, enc_states, enc_lengths, dec_lengths, norm_per_token=False):
    enc_mask = orc.make_encoder_masks(enc_lengths)
    dec_mask = orc.make_decoder_masks(dec_lengths)
    x = dec_in
    for layer in params["decoder"]:
        if norm_per_token:
            h, dk, dv = params["heads"], params["dk"], params["dv"]
            a = mha_per_token(x, x, x, dec_mask, layer["self"], h, dk, dv)
            x = orc.ffn(mha_per_token(a, enc_states, enc_states, enc_mask, layer["cross"], h, dk, dv), layer["ffn"])
        else:
            x = orc.decoder_block(x, enc_states, dec_mask, enc_mask, layer["self"], layer["cross"], layer["ffn"],
                                  params["heads"], params["dk"], params["dv"])
    return x


def forward(params, enc_tokens, dec_tokens, enc_lengths, dec_lengths, norm_per_token=False):
    enc_states = encoder(params, prepare_inputs(params, enc_tokens), enc_lengths, norm_per_token)
    decoded = decoder(params, prepare_inputs(params, dec_tokens), enc_states, enc_lengths, dec_lengths, norm_per_token)
    deembedded = orc.bmm(decoded, np.asarray(params["embedding"], np.float32), False, True)
    return log_softmax(orc.broadcast("add", deembedded, np.asarray(params["output_bias"], np.float32)))


def greedy_decode(params, input_sequence, start_token, end_token, max_length, return_logits=False, norm_per_token=False):
    n = len(input_sequence)
    encoded = encoder(params, prepare_inputs(params, [list(input_sequence)]), [n], norm_per_token)
    tokens, logits = [], []
    for _ in range(max_length):
        token_input = [[start_token] + tokens]
        out = decoder(params, prepare_inputs(params, token_input), encoded, [n], [len(token_input[0])], norm_per_token)
        deembedded = orc.bmm(out, np.asarray(params["embedding"], np.float32), False, True)
        nxt, _ = orc.argmax(deembedded[0, -1])
        logits.append(deembedded[0, -1].copy())
        tokens.append(nxt)
        if nxt == end_token:
            break
    return (tokens, logits) if return_logits else tokens
