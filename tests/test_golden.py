"""Golden fixtures (tests/golden/attention_fixtures.npz, written by tests/golden/make_fixtures.py from the CPU
oracle): the oracle must still reproduce them bit for bit (CPU), and the HIP path must match them (GPU)."""
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
