"""The layers of the path, run through the C++ host layer (libdl4s_host.so -> C ABI -> HIP kernels) in both
execution modes, against the CPU oracle (small and config-2 shapes) and the independent fp64 model (config 3).

mode "primitive": every tensor operator issues the engine calls the reference issues (drop-in behaviour);
mode "fused": ScaledDotProductAttention, batched matmul, residual+LayerNorm and bias+GELU use fused entries.
"""
import sys

import numpy as np
import pytest

from helpers import assert_parity, causal_mask
from oracle import fp64_model as m64

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from dl4s_amd import lib
    c = lib.Context(0)
    yield c
    c.close()


@pytest.fixture(scope="module")
def host():
    from dl4s_amd import host_lib
    host_lib.load()
    return host_lib


MODES = [pytest.param(False, id="primitive"), pytest.param(True, id="fused"), pytest.param(2, id="fused_strict"),
         pytest.param(3, id="attention_hook_only"), pytest.param(4, id="attention_hook_only_strict")]


def test_mask_builders_match_oracle_exactly(ctx, host, orc):
    lens = [3, 5, 1, 0, 5]
    assert np.array_equal(host.make_encoder_masks(ctx, lens), orc.make_encoder_masks(lens))
    assert np.array_equal(host.make_decoder_masks(ctx, lens), orc.make_decoder_masks(lens))


@pytest.mark.parametrize("fused", MODES)
@pytest.mark.parametrize("shape", [(1, 2, 5, 7, 4), (2, 3, 40, 50, 64)])
def test_sdpa_layer(ctx, host, orc, fused, shape):
    B, H, Lq, Lk, d = shape
    rng = np.random.default_rng(31)
    q, k, v = (rng.standard_normal(s).astype(np.float32) for s in [(B, H, Lq, d), (B, H, Lk, d), (B, H, Lk, d)])
    for mask in [None, causal_mask(Lq, Lk)]:
        assert_parity(host.sdpa(ctx, q, k, v, mask, fused=fused), orc.sdpa(q, k, v, mask), "SDPA layer")
    pad = (np.arange(Lk)[None, None, None, :] >= np.array([3, Lk, 1][:B])[:, None, None, None]).astype(np.float32)
    assert_parity(host.sdpa(ctx, q, k, v, pad, fused=fused), orc.sdpa(q, k, v, pad), "SDPA layer padding mask")


def test_nan_at_a_blocked_key_follows_the_mode(ctx, host, orc):
    """The reference multiplies a NaN value at a blocked key by its zero weight (NaN).  The primitive and fused-strict modes
    do the same; the fused mode skips key tiles its mask blocks entirely and documents that it differs there."""
    B, H, L, d = 1, 2, 128, 64
    rng = np.random.default_rng(33)
    q, k, v = (rng.standard_normal((B, H, L, d)).astype(np.float32) for _ in range(3))
    v[0, 1, 127, 3] = np.nan
    mask = causal_mask(L, L)
    with np.errstate(all="ignore"):
        ref = orc.sdpa(q, k, v, mask)
    assert np.isnan(ref[0, 1, :, 3]).all() and not np.isnan(ref[0, 0]).any()
    for mode in (False, 2):
        assert_parity(host.sdpa(ctx, q, k, v, mask, fused=mode), ref, "mode %s" % mode)
    got = host.sdpa(ctx, q, k, v, mask, fused=True)
    assert not np.isnan(got[0, 1, :96]).any()             # key 127 lies in a tile these rows never visit
    assert np.isnan(got[0, 1, 96:, 3]).all()              # rows of the last tile row read it (weight 0 times NaN)
    keep = ~np.isnan(ref)
    assert_parity(np.where(keep, got, 0), np.where(keep, ref, 0), "fused, finite part")


@pytest.mark.parametrize("fused", MODES)
def test_sdpa_layer_traps_on_a_mask_that_does_not_broadcast(ctx, host, fused):
    q = np.zeros((1, 2, 4, 8), np.float32)
    k = np.zeros((1, 2, 5, 8), np.float32)
    bad = np.zeros((3, 5), np.float32)          # 3 is neither 1 nor queryCount
    with pytest.raises(host.HostError):
        host.sdpa(ctx, q, k, k, bad, fused=fused)
    assert host.sdpa(ctx, q, k, k, np.zeros((1, 5), np.float32), fused=fused).shape == (1, 2, 4, 8)


@pytest.mark.parametrize("fused", MODES)
def test_tiny_transformer_layers(ctx, host, orc, fused):
    """Hyper-parameters of Tests/DL4STests/TransformerTests.swift:31: hidden 16, heads 4, key/value dim 8 -> here 4, ffn 32."""
    B, L, Le, D, H, dk, F = 2, 6, 5, 16, 4, 4, 32
    rng = np.random.default_rng(12)
    attn, ffn = m64.make_params(rng, D, H, dk, dk, F)
    attn2, _ = m64.make_params(rng, D, H, dk, dk, F)
    x = rng.standard_normal((B, L, D)).astype(np.float32)
    enc = rng.standard_normal((B, Le, D)).astype(np.float32)
    enc_mask = orc.make_encoder_masks([3, 5])
    dec_mask = orc.make_decoder_masks([6, 4])
    assert_parity(host.mha(ctx, x, enc, enc, enc_mask, attn, H, dk, dk, fused=fused),
                  orc.mha(x, enc, enc, enc_mask, attn, H, dk, dk), "MHA cross")
    assert_parity(host.mha(ctx, x, x, x, None, attn, H, dk, dk, fused=fused), orc.mha(x, x, x, None, attn, H, dk, dk), "MHA nil mask")
    pad = orc.make_encoder_masks([6, 2])
    assert_parity(host.encoder_block(ctx, x, pad, attn, ffn, H, dk, dk, fused=fused),
                  orc.encoder_block(x, pad, attn, ffn, H, dk, dk), "encoder block")
    assert_parity(host.decoder_block(ctx, x, enc, enc_mask, dec_mask, attn, attn2, ffn, H, dk, dk, fused=fused),
                  orc.decoder_block(x, enc, dec_mask, enc_mask, attn, attn2, ffn, H, dk, dk), "decoder block")


@pytest.mark.parametrize("fused", MODES)
@pytest.mark.parametrize("dk", [96, 128, 12, 192, 256, 140])
def test_mha_with_other_head_dims(ctx, host, orc, fused, dk):
    """Head dims other than 64: in fused mode the token-major attention kernels take every multiple of 4 up to 256 (the
    MFMA kernels of the next tile width with padding columns)."""
    B, L, Le, D, H = 2, 40, 50, 32, 2
    rng = np.random.default_rng(dk)
    attn, _ = m64.make_params(rng, D, H, dk, dk, 8)
    x = rng.standard_normal((B, L, D)).astype(np.float32)
    enc = rng.standard_normal((B, Le, D)).astype(np.float32)
    enc_mask = orc.make_encoder_masks([33, Le])
    assert_parity(host.mha(ctx, x, enc, enc, enc_mask, attn, H, dk, dk, fused=fused),
                  orc.mha(x, enc, enc, enc_mask, attn, H, dk, dk), "MHA cross dk=%d" % dk)
    cm = causal_mask(L, L)
    assert_parity(host.mha(ctx, x, x, x, cm, attn, H, dk, dk, fused=fused), orc.mha(x, x, x, cm, attn, H, dk, dk), "MHA self dk=%d" % dk)


def test_mha_with_a_query_far_from_zero_mean_in_strict_mode(ctx, host, orc):
    """The residual of MultiHeadAttention is its query input; ten standard deviations from zero the one-pass variance of
    the joint LayerNorm depends on the order of its sums beyond the parity gate.  The strict fused mode adds them in the
    reference's order and stays inside the gate."""
    B, L, D, H, dk = 2, 64, 64, 2, 32
    rng = np.random.default_rng(97)
    attn, _ = m64.make_params(rng, D, H, dk, dk, 8)
    x = rng.standard_normal((B, L, D)).astype(np.float32)
    q = (x + np.float32(10)).astype(np.float32)
    ref = orc.mha(q, x, x, None, attn, H, dk, dk)
    assert_parity(host.mha(ctx, q, x, x, None, attn, H, dk, dk, fused=2), ref, "MHA, query mean = 10 std, strict")


def _config2():
    B, L, D, H, dk = 4, 512, 512, 8, 64
    rng = np.random.Generator(np.random.PCG64(1002))
    x = rng.standard_normal((B, L, D), dtype=np.float32)
    attn, _ = m64.make_params(rng, D, H, dk, dk, 8, trivial_affine=True)
    return B, L, D, H, dk, x, attn, causal_mask(L, L)


@pytest.mark.parametrize("fused", MODES)
def test_config2_mha_layer_causal(ctx, host, orc, fused):
    """MultiHeadAttention fp32, B4 L512 D512 H8 (d 64), Xavier-uniform weights, N(0,1) input, causal mask."""
    B, L, D, H, dk, x, attn, mask = _config2()
    got = host.mha(ctx, x, x, x, mask, attn, H, dk, dk, fused=fused)
    ref = orc.mha(x, x, x, mask, attn, H, dk, dk)
    assert_parity(got, ref, "config 2")
    assert_parity(got, m64.mha64(x, x, x, mask, attn, H, dk, dk).astype(np.float32), "config 2 vs fp64")
    # decoder form of the same mask: [B,1,L,L] from makeDecoderMasks with full lengths
    dmask = host.make_decoder_masks(ctx, [L] * B)
    assert np.array_equal(dmask, np.broadcast_to(mask, (B, 1, L, L)))
    assert np.array_equal(host.mha(ctx, x, x, x, dmask, attn, H, dk, dk, fused=fused), got)


def test_repeated_layer_calls_on_one_mask_tensor(ctx, host):
    """In fused mode the mask tensor's tile classes are formed by the first attention call that receives it and serve the
    later ones: four calls of the layer on the same tensors give the bits of one call."""
    B, L, D, H, dk, x, attn, mask = _config2()
    for fused in (1, 2):
        once = host.mha(ctx, x, x, x, mask, attn, H, dk, dk, fused=fused)
        again, _ = host.mha(ctx, x, x, x, mask, attn, H, dk, dk, fused=fused, iters=3)
        assert np.array_equal(once, again)


def test_config3_encoder_block_padding_mask(ctx, host, orc):
    """TransformerEncoderBlock fp32, B8 L1024 D1024 H16 F4096, sigmoid-GELU, LayerNorm, key-length mask U[512,1024].
    The fused mode is checked against the fp64 model on the whole batch (the single-threaded oracle needs
    minutes at this size), the primitive mode against the fused mode on two batch items, and all three modes against
    the C oracle on one whole batch item."""
    B, L, D, H, dk, F = 8, 1024, 1024, 16, 64, 4096
    rng = np.random.Generator(np.random.PCG64(1003))
    x = rng.standard_normal((B, L, D), dtype=np.float32)
    attn, ffn = m64.make_params(rng, D, H, dk, dk, F, trivial_affine=True)
    lens = rng.integers(512, 1025, size=B)
    mask = (np.arange(L)[None, None, None, :] >= lens[:, None, None, None]).astype(np.float32)
    got = host.encoder_block(ctx, x, mask, attn, ffn, H, dk, dk, fused=True)
    ref = np.concatenate([m64.encoder_block64(x[b:b + 1], mask[b:b + 1], attn, ffn, H, dk, dk) for b in range(B)])
    assert_parity(got, ref.astype(np.float32), "config 3 vs fp64")
    prim = host.encoder_block(ctx, x[:2], mask[:2], attn, ffn, H, dk, dk, fused=False)
    assert_parity(prim, got[:2], "config 3 primitive vs fused")
    # One whole batch item against the C oracle.  MultiHeadAttention's LayerNorm runs over (L, D) of a batch item and the
    # feed-forward one over D of a token, so a batch item is a self-contained problem: the oracle on item b alone computes
    # what the reference computes for item b of the batch (about 90 s of single-threaded CPU at these widths).
    b = int(np.argmin(lens))
    sys.__stdout__.write("\n[config 3] CPU oracle on batch item %d (%d valid keys) ...\n" % (b, lens[b]))
    sys.__stdout__.flush()
    ref_b = orc.encoder_block(x[b:b + 1], mask[b:b + 1], attn, ffn, H, dk, dk)
    assert_parity(got[b:b + 1], ref_b, "config 3, batch item %d, fused vs oracle" % b)
    strict_b = host.encoder_block(ctx, x[b:b + 1], mask[b:b + 1], attn, ffn, H, dk, dk, fused=2)
    assert_parity(strict_b, ref_b, "config 3, batch item %d, fused strict vs oracle" % b)
    assert_parity(prim[b:b + 1] if b < 2 else host.encoder_block(ctx, x[b:b + 1], mask[b:b + 1], attn, ffn, H, dk, dk, fused=False),
                  ref_b, "config 3, batch item %d, primitive vs oracle" % b)
