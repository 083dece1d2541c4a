"""Independent fp64 model of the layers on the path (numpy + scipy, BLAS matmuls).  TEST INFRASTRUCTURE.

It shares no code with the C oracle: tests pin the oracle against it on small shapes, and use it as the
referee at sizes where the single-threaded oracle would take minutes."""
import numpy as np
import scipy.special


def f64(a):
    return np.asarray(a, np.float64)


def sdpa64(q, k, v, mask=None, temperature=None):
    q, k, v = f64(q), f64(k), f64(v)
    T = np.sqrt(q.shape[-1]) if temperature is None else temperature
    s = np.matmul(q, np.swapaxes(k, -1, -2)) / T
    if mask is not None:
        s = s - f64(mask) * 1e9
    return np.matmul(scipy.special.softmax(s, axis=-1), v)


def sdpa_backward64(q, k, v, mask, dout, temperature=None):
    """Gradients of sdpa64 with respect to q, k, v for an upstream gradient `dout`, in closed form:
    dv = p^T.dout, dp = dout.v^T, ds = p.(dp - rowsum(dp.p)), dq = ds.k / T, dk = ds^T.q / T.  The mask enters as the
    additive -1e9 penalty; a row with an unblocked key gives its blocked keys a weight of exactly 0 in fp64 as in fp32
    (rows with every key blocked are a rounding artefact of fp32 and are not modelled here)."""
    q, k, v, dout = f64(q), f64(k), f64(v), f64(dout)
    T = np.sqrt(q.shape[-1]) if temperature is None else temperature
    s = np.matmul(q, np.swapaxes(k, -1, -2)) / T
    if mask is not None:
        s = s - f64(mask) * 1e9
    p = scipy.special.softmax(s, axis=-1)
    dv = np.matmul(np.swapaxes(p, -1, -2), dout)
    dp = np.matmul(dout, np.swapaxes(v, -1, -2))
    ds = p * (dp - (dp * p).sum(axis=-1, keepdims=True))
    return np.matmul(ds, k) / T, np.matmul(np.swapaxes(ds, -1, -2), q) / T, dv


def layernorm64(x, scale, shift):
    """NN/Layer/LayerNorm.swift:62-77: statistics over all non-batch axes, eps outside the square root."""
    x = f64(x)
    axes = tuple(range(1, x.ndim))
    mean = x.mean(axis=axes, keepdims=True)
    std = np.sqrt((x * x).mean(axis=axes, keepdims=True) - mean ** 2)
    return (x - mean) / (std + 1e-5) * f64(scale) + f64(shift)


def mha64(q, k, v, mask, p, H, dk, dv):
    B, Lq, D = q.shape
    Lk = k.shape[1]
    qp = (f64(q) @ f64(p["Wq"])).reshape(B, Lq, H, dk).transpose(0, 2, 1, 3)
    kp = (f64(k) @ f64(p["Wk"])).reshape(B, Lk, H, dk).transpose(0, 2, 1, 3)
    vp = (f64(v) @ f64(p["Wv"])).reshape(B, Lk, H, dv).transpose(0, 2, 1, 3)
    a = sdpa64(qp, kp, vp, mask, np.sqrt(dk))
    o = a.transpose(0, 2, 1, 3).reshape(B, Lq, H * dv) @ f64(p["Wo"]) + f64(q)
    return layernorm64(o, p["ln_scale"], p["ln_shift"])


def ffn64(x, p):
    shape = np.shape(x)
    x2 = f64(x).reshape(-1, shape[-1])
    h = x2 @ f64(p["W1"]) + f64(p["b1"])
    g = h * scipy.special.expit(1.702 * h)
    o = g @ f64(p["W2"]) + f64(p["b2"]) + x2
    return layernorm64(o, p["ln_scale"], p["ln_shift"]).reshape(shape)


def encoder_block64(x, mask, attn, ffn, H, dk, dv):
    return ffn64(mha64(x, x, x, mask, attn, H, dk, dv), ffn)


def decoder_block64(dec, enc, dec_mask, enc_mask, self_p, cross_p, ffn, H, dk, dv):
    a = mha64(dec, dec, dec, dec_mask, self_p, H, dk, dv)
    c = mha64(a, enc, enc, enc_mask, cross_p, H, dk, dv)
    return ffn64(c, ffn)


def xavier_uniform(rng, fan_in, fan_out):
    a = np.sqrt(6.0 / (fan_in + fan_out))
    return rng.uniform(-a, a, (fan_in, fan_out)).astype(np.float32)


def make_params(rng, D, H, dk, dv, F, trivial_affine=False):
    """Xavier-uniform weights; LayerNorm scale/shift and biases are 1/0 (the reference's init) when trivial_affine."""
    def aff(n, centre):
        return np.full(n, centre, np.float32) if trivial_affine else (centre + 0.1 * rng.standard_normal(n)).astype(np.float32)
    mha = dict(Wq=xavier_uniform(rng, D, H * dk), Wk=xavier_uniform(rng, D, H * dk), Wv=xavier_uniform(rng, D, H * dv),
               Wo=xavier_uniform(rng, H * dv, D), ln_scale=aff(D, 1.0), ln_shift=aff(D, 0.0))
    ffn = dict(W1=xavier_uniform(rng, D, F), b1=aff(F, 0.0), W2=xavier_uniform(rng, F, D), b2=aff(D, 0.0),
               ln_scale=aff(D, 1.0), ln_shift=aff(D, 0.0))
    return mha, ffn


# ---- the Transformer wrapper, independently of the fp32 oracle (plain numpy, float64)
def positional_encoding64(max_len, hidden):
    pos = np.arange(max_len, dtype=np.float64)[:, None]
    i = np.arange(hidden // 2, dtype=np.float64)[None, :]
    angle = pos / np.power(10000.0, i / (hidden // 2))
    out = np.empty((max_len, hidden))
    out[:, 0::2], out[:, 1::2] = np.sin(angle), np.cos(angle)
    return out


def prepare_inputs64(params, tokens):
    tokens = np.asarray(tokens)
    E = f64(params["embedding"])
    emb = np.where((tokens == -1)[..., None], 0.0, E[np.clip(tokens, 0, E.shape[0] - 1)])
    return emb * np.sqrt(E.shape[1]) + positional_encoding64(tokens.shape[1], E.shape[1])


def _enc_mask(lengths):
    L = max(lengths)
    return (np.arange(L)[None, None, None, :] >= np.asarray(lengths)[:, None, None, None]).astype(np.float64)


def _dec_mask(lengths):
    L = max(lengths)
    i, j = np.indices((L, L))
    return np.maximum(_enc_mask(lengths), (j > i)[None, None].astype(np.float64))


def transformer64(params, enc_tokens, dec_tokens, enc_lengths, dec_lengths, log_probs=True):
    H, dk, dv = params["heads"], params["dk"], params["dv"]
    x = prepare_inputs64(params, enc_tokens)
    for layer in params["encoder"]:
        x = encoder_block64(x, _enc_mask(enc_lengths), layer["attn"], layer["ffn"], H, dk, dv)
    y = prepare_inputs64(params, dec_tokens)
    for layer in params["decoder"]:
        y = decoder_block64(y, x, _dec_mask(dec_lengths), _enc_mask(enc_lengths), layer["self"], layer["cross"], layer["ffn"], H, dk, dv)
    logits = y @ f64(params["embedding"]).T
    if not log_probs:
        return logits
    logits = logits + f64(params["output_bias"])
    m = logits.max(-1, keepdims=True)
    return logits - m - np.log(np.exp(logits - m).sum(-1, keepdims=True))


def make_transformer_params(rng, vocab, D, H, dk, dv, F, n_enc, n_dec):
    p = {"embedding": (rng.standard_normal((vocab, D)) * (1.0 / np.sqrt(D))).astype(np.float32),
         "output_bias": (rng.standard_normal(vocab) * 0.1).astype(np.float32), "heads": H, "dk": dk, "dv": dv,
         "encoder": [], "decoder": []}
    for _ in range(n_enc):
        a, f = make_params(rng, D, H, dk, dv, F)
        p["encoder"].append({"attn": a, "ffn": f})
    for _ in range(n_dec):
        a, f = make_params(rng, D, H, dk, dv, F)
        c, _ = make_params(rng, D, H, dk, dv, F)
        p["decoder"].append({"self": a, "cross": c, "ffn": f})
    return p
