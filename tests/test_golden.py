"""Golden fixtures (tests/golden/attention_fixtures.npz and model_fixtures.npz, written by tests/golden/make_fixtures.py
from the CPU oracle): the oracle must still reproduce them bit for bit (CPU), and the HIP path must match them (GPU)."""
import os

import numpy as np
import pytest

from helpers import assert_parity

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_fixtures.npz"))
MASKS = ["none", "dense", "causal", "lens", "blocked_row"]
HM, DK = 4, 8


def _mask(name):
    return None if name == "none" else FIX["sdpa_mask_" + name]


def _params(prefix, names):
    return {n: FIX[prefix + n] for n in names}


ATTN = ("Wq", "Wk", "Wv", "Wo", "ln_scale", "ln_shift")
FFN = ("W1", "b1", "W2", "b2", "ln_scale", "ln_shift")


def test_oracle_reproduces_fixtures(orc):
    q, k, v = FIX["sdpa_q"], FIX["sdpa_k"], FIX["sdpa_v"]
    for name in MASKS:
        assert np.array_equal(orc.sdpa(q, k, v, _mask(name)), FIX["sdpa_out_" + name]), name
    with np.errstate(all="ignore"):
        assert np.array_equal(orc.sdpa(FIX["sdpa_q_nonfinite"], k, v, None), FIX["sdpa_out_nonfinite"], equal_nan=True)
    attn, ffn = _params("mha_", ATTN), _params("ffn_", FFN)
    x, pad = FIX["layer_x"], FIX["layer_mask"]
    assert np.array_equal(orc.mha(x, x, x, pad, attn, HM, DK, DK), FIX["mha_out"])
    assert np.array_equal(orc.encoder_block(x, pad, attn, ffn, HM, DK, DK), FIX["encoder_out"])
    for t in range(3):
        assert np.array_equal(orc.sdpa_decode(FIX["dec_q"][t], FIX["dec_k"], FIX["dec_v"], 10 + t), FIX["dec_out"][t])


def test_fixture_invariants():
    out = FIX["sdpa_out_blocked_row"]
    assert np.allclose(out[:, :, 2], FIX["sdpa_v"].mean(axis=2), atol=1e-6)        # fully blocked row = mean of V
    nf = FIX["sdpa_out_nonfinite"]
    assert np.isnan(nf[0, 0, 1]).all() and np.isnan(nf[0, 1, 3]).all() and np.isnan(nf).sum() == 2 * nf.shape[-1]
    assert np.allclose(FIX["sdpa_out_causal"][:, :, 0], FIX["sdpa_v"][:, :, 0], atol=1e-6)


@pytest.mark.gpu
def test_hip_matches_fixtures():
    from dl4s_amd import host_lib, lib
    ctx = lib.Context(0)
    try:
        q, k, v = FIX["sdpa_q"], FIX["sdpa_k"], FIX["sdpa_v"]
        for fused in (False, True):
            for name in MASKS:
                assert_parity(host_lib.sdpa(ctx, q, k, v, _mask(name), fused=fused), FIX["sdpa_out_" + name], name)
            assert_parity(host_lib.sdpa(ctx, FIX["sdpa_q_nonfinite"], k, v, None, fused=fused), FIX["sdpa_out_nonfinite"], "non-finite")
            attn, ffn = _params("mha_", ATTN), _params("ffn_", FFN)
            x, pad = FIX["layer_x"], FIX["layer_mask"]
            assert_parity(host_lib.mha(ctx, x, x, x, pad, attn, HM, DK, DK, fused=fused), FIX["mha_out"], "mha")
            assert_parity(host_lib.encoder_block(ctx, x, pad, attn, ffn, HM, DK, DK, fused=fused), FIX["encoder_out"], "encoder")
        # decode: rows 9..11 appended one by one into a cache that holds rows 0..8
        kc, vc = FIX["dec_k"].copy(), FIX["dec_v"].copy()
        newk, newv = kc[:, :, 9:12].copy(), vc[:, :, 9:12].copy()
        kc[:, :, 9:] = 0
        vc[:, :, 9:] = 0
        dk_, dv_ = ctx.to_device(kc), ctx.to_device(vc)
        for t in range(3):
            kn, vn = ctx.to_device(newk[:, :, t:t + 1]), ctx.to_device(newv[:, :, t:t + 1])
            dq, out = ctx.to_device(FIX["dec_q"][t]), ctx.empty((1, 2, 1, 64))
            ctx.sdpa_decode_step(dq, dk_, dv_, kn, vn, out, 1, 2, 9 + t, 12, 64, 0.125)
            assert_parity(out.numpy(), FIX["dec_out"][t], "decode step %d" % t)
        assert np.array_equal(dk_.numpy(), FIX["dec_k"]) and np.array_equal(dv_.numpy(), FIX["dec_v"])
    finally:
        ctx.close()


# ------------------------------------------------------------------ gradients and the Transformer wrapper
MFIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "model_fixtures.npz"))
BWD_MASKS = ["none", "dense", "causal", "blocked_row"]


def _transformer_params():
    p = {"embedding": MFIX["tf_embedding"], "output_bias": MFIX["tf_output_bias"], "heads": 4, "dk": 8, "dv": 8, "encoder": [], "decoder": []}
    for side, parts in (("encoder", ("attn", "ffn")), ("decoder", ("self", "cross", "ffn"))):
        for i in range(2):
            layer = {}
            for part in parts:
                pre = "tf_%s%d_%s_" % (side, i, part)
                layer[part] = {k[len(pre):]: MFIX[k] for k in MFIX.files if k.startswith(pre)}
            p[side].append(layer)
    return p


def test_oracle_reproduces_model_fixtures(orc):
    from oracle import transformer as T
    q, k, v = FIX["sdpa_q"], FIX["sdpa_k"], FIX["sdpa_v"]
    for name in BWD_MASKS:
        got = orc.sdpa_backward(q, k, v, _mask(name), MFIX["bwd_dout"])
        for g, key in zip(got, ("dq", "dk", "dv")):
            assert np.array_equal(g, MFIX["bwd_%s_%s" % (key, name)]), (key, name)
    params = _transformer_params()
    assert np.array_equal(T.positional_encoding(9, 16), MFIX["tf_positions"])
    lp = T.forward(params, MFIX["tf_enc_tokens"], MFIX["tf_dec_tokens"], list(MFIX["tf_enc_lengths"]), list(MFIX["tf_dec_lengths"]))
    assert np.array_equal(lp, MFIX["tf_log_probs"])
    toks, logits = T.greedy_decode(params, [int(t) for t in MFIX["tf_greedy_source"]], 1, 2, 6, return_logits=True)
    assert toks == list(MFIX["tf_greedy_tokens"]) and np.array_equal(np.stack(logits), MFIX["tf_greedy_logits"])


def test_model_fixture_invariants():
    # every softmax row sums to 1, so the value gradient sums to the upstream gradient, whatever the mask
    for name in BWD_MASKS:
        assert np.allclose(MFIX["bwd_dv_" + name].sum(2), MFIX["bwd_dout"].sum(2), atol=1e-5)
    assert np.allclose(np.exp(MFIX["tf_log_probs"].astype(np.float64)).sum(-1), 1.0, atol=1e-5)
    top2 = np.sort(MFIX["tf_greedy_logits"], axis=1)[:, -2:]
    assert (top2[:, 1] - top2[:, 0]).min() > 1e-3                  # the greedy fixture does not sit on a tie


@pytest.mark.gpu
def test_hip_matches_model_fixtures():
    from dl4s_amd import host_lib, lib
    ctx = lib.Context(0)
    try:
        q, k, v, dout = FIX["sdpa_q"], FIX["sdpa_k"], FIX["sdpa_v"], MFIX["bwd_dout"]
        B, H, Lq, d = q.shape
        Lk = k.shape[2]
        bufs = [ctx.to_device(x) for x in (q, k, v, dout)]
        out, dq, st = ctx.empty(q.shape), ctx.empty(q.shape), ctx.empty((B, H, Lq, 2))
        dk_, dv_ = ctx.empty(k.shape), ctx.empty(v.shape)
        for name in BWD_MASKS:
            desc, keep = None, None
            if name != "none":
                keep = ctx.to_device(_mask(name))
                desc = ctx.mask_desc(lib.MASK_DENSE, dense=keep)
            ctx.sdpa_fwd_stats(bufs[0], bufs[1], bufs[2], out, st, B, H, Lq, Lk, d, 0.5, desc, 0)
            ctx.sdpa_bwd(bufs[0], bufs[1], bufs[2], out, st, bufs[3], dq, dk_, dv_, B, H, Lq, Lk, d, 0.5, desc, 0)
            assert_parity(out.numpy(), FIX["sdpa_out_" + name], "forward " + name)
            for got, key in ((dq, "dq"), (dk_, "dk"), (dv_, "dv")):
                assert_parity(got.numpy(), MFIX["bwd_%s_%s" % (key, name)], key + " " + name)
        params = _transformer_params()
        model = host_lib.Transformer(ctx, params)
        for fused in (False, True):
            assert_parity(host_lib.positional_encoding(ctx, 9, 16, fused=fused), MFIX["tf_positions"], "positions")
            lp = model.forward(MFIX["tf_enc_tokens"], MFIX["tf_dec_tokens"], MFIX["tf_enc_lengths"], MFIX["tf_dec_lengths"], fused=fused)
            assert_parity(lp, MFIX["tf_log_probs"], "log-probabilities")
            toks, logits = model.greedy(MFIX["tf_greedy_source"], 1, 2, 6, fused=fused, return_logits=True)
            assert toks == list(MFIX["tf_greedy_tokens"])
            assert_parity(logits, MFIX["tf_greedy_logits"], "greedy logits")
        model.close()
    finally:
        ctx.close()
