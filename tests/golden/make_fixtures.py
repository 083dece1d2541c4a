"""Writes tests/golden/attention_fixtures.npz and tests/golden/model_fixtures.npz: small inputs and the CPU oracle's
outputs for them.

The vectors come from this repository's oracle (oracle/dl4s_oracle.c), never from the reference (which is Swift and
cannot run here); they freeze the oracle's behaviour so that a later change to it shows up, and give the GPU tests a
fixed set of edge cases.  Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import binding as orc  # noqa: E402
from oracle import fp64_model as m64  # noqa: E402


def main():
    rng = np.random.default_rng(20240)
    out = {}
    B, H, Lq, Lk, d = 1, 2, 5, 7, 4
    q, k, v = (rng.standard_normal(s).astype(np.float32) for s in [(B, H, Lq, d), (B, H, Lk, d), (B, H, Lk, d)])
    i, j = np.indices((Lq, Lk))
    masks = {"none": None, "dense": (rng.random((B, H, Lq, Lk)) < 0.35).astype(np.float32),
             "causal": (j > i).astype(np.float32), "lens": (np.arange(Lk)[None, None, None, :] >= 4).astype(np.float32)}
    blocked = np.zeros((Lq, Lk), np.float32)
    blocked[2, :] = 1
    masks["blocked_row"] = blocked
    out.update(sdpa_q=q, sdpa_k=k, sdpa_v=v)
    for name, m in masks.items():
        if m is not None:
            out["sdpa_mask_" + name] = m
        out["sdpa_out_" + name] = orc.sdpa(q, k, v, m)
    qn = q.copy()
    qn[0, 0, 1, 0] = np.nan
    qn[0, 1, 3, 2] = np.inf
    with np.errstate(all="ignore"):
        out.update(sdpa_q_nonfinite=qn, sdpa_out_nonfinite=orc.sdpa(qn, k, v, None))
    # the hyper-parameters of Tests/DL4STests/TransformerTests.swift:31 (hidden 16, heads 4, key/value dim 8, ffn 32)
    Bm, L, D, Hm, dk, F = 2, 6, 16, 4, 8, 32
    attn, ffn = m64.make_params(rng, D, Hm, dk, dk, F)
    x = rng.standard_normal((Bm, L, D)).astype(np.float32)
    pad = orc.make_encoder_masks([6, 3])
    for kname, val in list(attn.items()):
        out["mha_" + kname] = val
    for kname, val in list(ffn.items()):
        out["ffn_" + kname] = val
    out.update(layer_x=x, layer_mask=pad, mha_out=orc.mha(x, x, x, pad, attn, Hm, dk, dk),
               encoder_out=orc.encoder_block(x, pad, attn, ffn, Hm, dk, dk))
    # decode: cache capacity 12, append rows 9, 10, 11 and attend after each append
    Bd, Hd, dd, Tcap = 1, 2, 64, 12
    kc = rng.standard_normal((Bd, Hd, Tcap, dd)).astype(np.float32)
    vc = rng.standard_normal((Bd, Hd, Tcap, dd)).astype(np.float32)
    qs = rng.standard_normal((3, Bd, Hd, 1, dd)).astype(np.float32)
    out.update(dec_k=kc, dec_v=vc, dec_q=qs,
               dec_out=np.stack([orc.sdpa_decode(qs[t], kc, vc, 10 + t) for t in range(3)]))
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "attention_fixtures.npz"), **out)
    print("wrote %d arrays" % len(out))


def flatten_transformer(params):
    flat = {"embedding": params["embedding"], "output_bias": params["output_bias"]}
    for side, parts in (("encoder", ("attn", "ffn")), ("decoder", ("self", "cross", "ffn"))):
        for i, layer in enumerate(params[side]):
            for part in parts:
                for name, val in layer[part].items():
                    flat["%s%d_%s_%s" % (side, i, part, name)] = val
    return flat


def model_fixtures():
    """Gradients of attention on the tiny attention fixture, and the Transformer wrapper (forward log-probabilities and
    greedy decoding) at the hyper-parameters of Tests/DL4STests/TransformerTests.swift:31."""
    from oracle import transformer as orc_t
    fix = np.load(os.path.join(ROOT, "tests", "golden", "attention_fixtures.npz"))
    rng = np.random.default_rng(20241)
    out = {}
    q, k, v = fix["sdpa_q"], fix["sdpa_k"], fix["sdpa_v"]
    dout = rng.standard_normal(q.shape).astype(np.float32)
    out["bwd_dout"] = dout
    for name in ("none", "dense", "causal", "blocked_row"):
        m = None if name == "none" else fix["sdpa_mask_" + name]
        dq, dk, dv = orc.sdpa_backward(q, k, v, m, dout)
        out.update({"bwd_dq_" + name: dq, "bwd_dk_" + name: dk, "bwd_dv_" + name: dv})
    vocab = 13
    params = m64.make_transformer_params(rng, vocab, 16, 4, 8, 8, 32, 2, 2)
    for name, val in flatten_transformer(params).items():
        out["tf_" + name] = val
    enc_len, dec_len = [7, 4], [5, 3]
    enc, dec = np.full((2, 7), -1, np.int32), np.full((2, 5), -1, np.int32)
    for b in range(2):
        enc[b, :enc_len[b]] = rng.integers(0, vocab, enc_len[b])
        dec[b, :dec_len[b]] = rng.integers(0, vocab, dec_len[b])
    src = rng.integers(0, vocab, 6).astype(np.int32)
    toks, logits = orc_t.greedy_decode(params, [int(t) for t in src], 1, 2, 6, return_logits=True)
    out.update(tf_enc_tokens=enc, tf_dec_tokens=dec, tf_enc_lengths=np.array(enc_len), tf_dec_lengths=np.array(dec_len),
               tf_log_probs=orc_t.forward(params, enc, dec, enc_len, dec_len), tf_positions=orc_t.positional_encoding(9, 16),
               tf_greedy_source=src, tf_greedy_tokens=np.array(toks, np.int32), tf_greedy_logits=np.stack(logits))
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "model_fixtures.npz"), **out)
    print("wrote %d arrays" % len(out))


if __name__ == "__main__":
    main()
    model_fixtures()
