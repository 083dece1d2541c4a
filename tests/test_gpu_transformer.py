"""The callers on either side of the attention path: the engine additions the Transformer wrapper needs, and the wrapper
itself (embedding, positional encoding, encoder / decoder stacks, log-softmax output, greedy decoding) through the C++
host layer, against the CPU oracle.  Gate as everywhere: |gpu - oracle| <= 1e-4 + 1e-4 |oracle|; integer results exact."""
import numpy as np
import pytest

from helpers import assert_parity

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from dl4s_amd import lib
    c = lib.Context(0)
    yield c
    c.close()


def test_log_sin_cos(ctx, orc):
    rng = np.random.default_rng(31)
    n = 50001
    x = (rng.random(n) * 600.0).astype(np.float32)
    p = (rng.random(n) * 1e4 + 1e-3).astype(np.float32)
    dx, dp, dy = ctx.to_device(x), ctx.to_device(p), ctx.empty((n,))
    ctx.sin(dx, dy, n)
    assert_parity(dy.numpy(), orc.sin(x), "sin")
    ctx.cos(dx, dy, n)
    assert_parity(dy.numpy(), orc.cos(x), "cos")
    ctx.log(dp, dy, n)
    assert_parity(dy.numpy(), orc.log(p), "log")
    for b in (dx, dp, dy):
        b.release()


@pytest.mark.parametrize("n", [1, 7, 1024, 1025, 100003])
def test_argmax_matches_the_reference_scan(ctx, orc, n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    if n > 6:
        x[[2, n - 3]] = x.max() + 1.0          # a tie far apart: the first wins
        x[n // 2] = np.nan                      # NaN is never selected
    d = ctx.to_device(x)
    assert ctx.argmax(d, n) == orc.argmax(x)
    d.release()


def test_argmax_nothing_selected(ctx, orc):
    for x in (np.array([np.nan, np.nan, np.nan], np.float32), np.full(2000, -np.inf, np.float32)):
        d = ctx.to_device(x)
        assert ctx.argmax(d, len(x)) == orc.argmax(x) == (0, -np.inf)
        d.release()
    d = ctx.empty((4,))
    assert ctx.argmax(d, 0) == (0, -np.inf)
    d.release()


def test_stack_along_inner_axis(ctx):
    rng = np.random.default_rng(32)
    a, b, c = (rng.standard_normal(s).astype(np.float32) for s in ((5, 3, 4), (5, 2, 4), (5, 1, 4)))
    da, db, dc, dy = ctx.to_device(a), ctx.to_device(b), ctx.to_device(c), ctx.empty((5, 6, 4))
    ctx.stack_axis([da, db, dc], [12, 8, 4], 5, dy)
    assert np.array_equal(dy.numpy(), np.concatenate([a, b, c], axis=1))
    for x in (da, db, dc, dy):
        x.release()


def test_embedding_with_scale_and_positions(ctx, orc):
    from oracle import transformer as T
    rng = np.random.default_rng(33)
    V, D, B, L = 29, 24, 3, 7
    E = rng.standard_normal((V, D)).astype(np.float32)
    tok = rng.integers(0, V, (B, L)).astype(np.int32)
    tok[1, 4:] = -1
    dE, dt, dy = ctx.to_device(E), ctx.to_device(tok, dtype=np.int32), ctx.empty((B, L, D))
    ctx.embed_positions(dE, V, D, dt, B, L, -1, None, None, dy)
    assert np.array_equal(dy.numpy(), orc.embedding(E, tok.reshape(-1), -1).reshape(B, L, D))
    pos = T.positional_encoding(L, D)
    dpos = ctx.to_device(pos)
    scale = float(np.sqrt(np.float32(D)))
    ctx.embed_positions(dE, V, D, dt, B, L, -1, scale, dpos, dy)
    assert np.array_equal(dy.numpy(), T.prepare_inputs({"embedding": E}, tok))     # same roundings, same bits
    for x in (dE, dt, dy, dpos):
        x.release()


def test_embedding_never_reads_the_table_for_a_token_out_of_range(ctx):
    """The reference's subscript traps on a token outside [0, vocab).  The kernel does not read the table for one: the
    token's row of the result is NaN and every other row is what it would be without it.  The table sits at the end of
    its own small allocation, so an unchecked index of 10**9 or -7 would read far outside it."""
    rng = np.random.default_rng(35)
    V, D, B, L = 11, 8, 2, 5
    E = rng.standard_normal((V, D)).astype(np.float32)
    tok = rng.integers(0, V, (B, L)).astype(np.int32)
    good = tok.copy()
    tok[0, 1], tok[1, 3], tok[1, 4] = V, -7, 10 ** 9
    pos = rng.standard_normal((L, D)).astype(np.float32)
    dE, dt, dg, dpos = ctx.to_device(E), ctx.to_device(tok, dtype=np.int32), ctx.to_device(good, dtype=np.int32), ctx.to_device(pos)
    dy, dyg = ctx.empty((B, L, D)), ctx.empty((B, L, D))
    for scale, dp in ((None, None), (3.0, dpos)):
        ctx.embed_positions(dE, V, D, dt, B, L, -1, scale, dp, dy)
        ctx.embed_positions(dE, V, D, dg, B, L, -1, scale, dp, dyg)
        got, want = dy.numpy(), dyg.numpy()
        bad = np.zeros((B, L), bool)
        bad[0, 1] = bad[1, 3] = bad[1, 4] = True
        assert np.isnan(got[bad]).all() and np.array_equal(got[~bad], want[~bad])
    for x in (dE, dt, dg, dpos, dy, dyg):
        x.release()


def test_log_softmax_rows(ctx):
    from oracle import transformer as T
    rng = np.random.default_rng(34)
    x = (rng.standard_normal((37, 1000)) * 5).astype(np.float32)
    x[3, 10] = 80.0
    dx, dy = ctx.to_device(x), ctx.empty(x.shape)
    ctx.log_softmax(dx, 37, 1000, dy)
    assert_parity(dy.numpy(), T.log_softmax(x), "logSoftmax")
    dx.release()
    dy.release()


def test_embedding_of_a_token_held_in_device_memory(ctx, orc):
    """dl4s_hip_embed_at_f32: token and position come from device memory; same rounding as the host-token entry point;
    a token outside the vocabulary embeds as zeros, a position outside the table adds nothing."""
    from oracle import transformer as T
    rng = np.random.default_rng(34)
    V, D, rows = 29, 24, 9
    E = rng.standard_normal((V, D)).astype(np.float32)
    pos = T.positional_encoding(rows, D)
    scale = float(np.sqrt(np.float32(D)))
    dE, dpos, dy = ctx.to_device(E), ctx.to_device(pos), ctx.empty((D,))
    for token, at in ((0, 0), (17, 5), (28, 8)):
        cur = ctx.to_device(np.array([token, at], np.int32), dtype=np.int32)
        ctx.embed_at(dE, V, D, cur, scale, dpos, rows, cur.offset(4), dy)
        want = orc.broadcast("add", orc.broadcast("mul", E[token], np.float32(scale)), pos[at])
        assert np.array_equal(dy.numpy(), want)
        ctx.embed_at(dE, V, D, cur, None, None, 0, None, dy)
        assert np.array_equal(dy.numpy(), E[token])
        cur.release()
    for token, at, want in ((-1, 2, pos[2]), (V, 2, pos[2]), (3, rows, E[3] * np.float32(scale)), (3, -1, E[3] * np.float32(scale))):
        cur = ctx.to_device(np.array([token, at], np.int32), dtype=np.int32)
        ctx.embed_at(dE, V, D, cur, scale, dpos, rows, cur.offset(4), dy)
        assert np.array_equal(dy.numpy(), want.astype(np.float32))
        cur.release()
    for b in (dE, dpos, dy):
        b.release()


@pytest.mark.parametrize("n", [1, 7, 1025, 100003])
def test_argmax_to_device_memory(ctx, orc, n):
    rng = np.random.default_rng(n + 1)
    x = rng.standard_normal(n).astype(np.float32)
    if n > 6:
        x[[2, n - 3]] = x.max() + 1.0
    d = ctx.to_device(x)
    cur = ctx.to_device(np.array([-7, 41], np.int32), dtype=np.int32)
    ctx.argmax_to(d, n, cur, cur.offset(4))
    assert list(cur.numpy()) == [orc.argmax(x)[0], 42]
    ctx.argmax_to(d, n, cur.offset(4))                  # no counter
    assert list(cur.numpy()) == [orc.argmax(x)[0]] * 2
    d.release()
    cur.release()


@pytest.mark.parametrize("fused", [False, True])
def test_positional_encoding_layer(ctx, fused):
    from dl4s_amd import host_lib
    from oracle import transformer as T
    got = host_lib.positional_encoding(ctx, 300, 64, fused=fused)
    assert_parity(got, T.positional_encoding(300, 64), "PositionalEncoding")


def _model(seed, vocab, D, H, dk, F, n_enc, n_dec):
    from oracle import fp64_model as m64
    rng = np.random.default_rng(seed)
    return m64.make_transformer_params(rng, vocab, D, H, dk, dk, F, n_enc, n_dec), rng


CONFIGS = {  # vocab, hidden, heads, key/value dim, ffn, encoder layers, decoder layers
    "transformer_tests_hyperparameters": (13, 16, 4, 8, 32, 2, 2),   # Tests/DL4STests/TransformerTests.swift:31
    "head_dim_64": (40, 128, 2, 64, 256, 2, 2),
}


@pytest.mark.parametrize("name", list(CONFIGS))
@pytest.mark.parametrize("fused", [False, True])
def test_transformer_forward(ctx, name, fused):
    from dl4s_amd import host_lib
    from oracle import transformer as T
    vocab = CONFIGS[name][0]
    params, rng = _model(41, *CONFIGS[name])
    enc_len, dec_len = [9, 5, 7], [6, 6, 2]
    enc = np.full((3, 9), -1, np.int32)
    dec = np.full((3, 6), -1, np.int32)
    for b in range(3):
        enc[b, :enc_len[b]] = rng.integers(0, vocab, enc_len[b])
        dec[b, :dec_len[b]] = rng.integers(0, vocab, dec_len[b])
    model = host_lib.Transformer(ctx, params)
    got = model.forward(enc, dec, enc_len, dec_len, fused=fused)
    model.close()
    ref = T.forward(params, enc, dec, enc_len, dec_len)
    assert_parity(got, ref, "Transformer forward %s fused=%s" % (name, fused))
    assert np.allclose(np.exp(got.astype(np.float64)).sum(-1), 1.0, atol=1e-4)


@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_decoding(ctx, name):
    """Same tokens as the oracle's decoding, logits within tolerance; fused mode (which keeps the encoder-side key / value
    projections across steps when the head size allows) and primitive mode agree."""
    from dl4s_amd import host_lib
    from oracle import transformer as T
    vocab = CONFIGS[name][0]
    params, rng = _model(43, *CONFIGS[name])
    src = [int(t) for t in rng.integers(0, vocab, 8)]
    ref_tokens, ref_logits = T.greedy_decode(params, src, 1, 2, 7, return_logits=True)
    top2 = np.sort(np.stack(ref_logits), axis=1)[:, -2:]
    assert (top2[:, 1] - top2[:, 0]).min() > 1e-3, "the fixture must not sit on an argmax tie"
    model = host_lib.Transformer(ctx, params)
    for fused in (True, False):
        toks, logits = model.greedy(src, 1, 2, 7, fused=fused, return_logits=True)
        assert toks == ref_tokens
        assert_parity(logits, np.stack(ref_logits), "greedy logits %s fused=%s" % (name, fused))
    model.close()


def test_cached_greedy_decoding(ctx):
    """Decoding with key / value caches (one new position per step through the decode kernels) against the oracle's
    prefix re-run of the same model.  Only a model that normalises per token can be cached: the reference's joint
    normalisation is refused, and the per-token model's uncached paths are checked against the oracle as well."""
    from dl4s_amd import host_lib
    from oracle import transformer as T
    name = "head_dim_64"
    vocab = CONFIGS[name][0]
    params, rng = _model(47, *CONFIGS[name])
    src = [int(t) for t in rng.integers(0, vocab, 11)]
    steps = 20          # long enough for the recorded step (decodes of 16 tokens or more)
    ref_tokens, ref_logits = T.greedy_decode(params, src, 1, -5, steps, return_logits=True, norm_per_token=True)
    assert len(ref_tokens) == steps
    top2 = np.sort(np.stack(ref_logits), axis=1)[:, -2:]
    assert (top2[:, 1] - top2[:, 0]).min() > 1e-3, "the fixture must not sit on an argmax tie"
    model = host_lib.Transformer(ctx, params)
    with pytest.raises(host_lib.HostError, match="normalise per token"):
        model.greedy(src, 1, -5, steps, cached=True)
    model.set_norm_per_token(True)
    for fused in (True, False):                      # the prefix re-run of the per-token model
        toks, logits = model.greedy(src, 1, -5, steps, fused=fused, return_logits=True)
        assert toks == ref_tokens
        assert_parity(logits, np.stack(ref_logits), "per-token greedy logits fused=%s" % fused)
    toks, logits = model.greedy(src, 1, -5, steps, cached=True, return_logits=True)
    assert toks == ref_tokens
    assert_parity(logits, np.stack(ref_logits), "cached greedy logits")
    # the recorded step replayed at every position computes what the same calls issued one by one compute, and a second
    # decode (a new recording, the pool holding the first one's blocks again) repeats the first
    toks_s, logits_s = model.greedy(src, 1, -5, steps, cached="stepwise", return_logits=True)
    assert toks_s == toks and np.array_equal(logits_s, logits)
    toks_2, logits_2 = model.greedy(src, 1, -5, steps, cached=True, return_logits=True)
    assert toks_2 == toks and np.array_equal(logits_2, logits)
    # stops at the end token like the uncached loop
    assert model.greedy(src, 1, ref_tokens[3], steps, cached=True) == ref_tokens[:ref_tokens.index(ref_tokens[3]) + 1]
    assert model.greedy(src, 1, -5, 0, cached=True) == []
    with pytest.raises(host_lib.HostError, match="fused mode"):
        model.greedy(src, 1, -5, steps, fused=False, cached=True)
    # forward pass of the per-token model, and back to the reference's normalisation
    enc = np.array([src[:9], src[:5] + [-1] * 4], np.int32)
    dec = np.array([[1, 4, 7, 9, 3, 2], [1, 5, -1, -1, -1, -1]], np.int32)
    assert_parity(model.forward(enc, dec, [9, 5], [6, 2]), T.forward(params, enc, dec, [9, 5], [6, 2], norm_per_token=True),
                  "per-token forward")
    model.set_norm_per_token(False)
    assert_parity(model.forward(enc, dec, [9, 5], [6, 2]), T.forward(params, enc, dec, [9, 5], [6, 2]), "joint forward")
    model.close()


def test_cached_decoding_with_the_reference_test_models_key_size(ctx):
    """Key / value dim 8 (Tests/DL4STests/TransformerTests.swift:31): the decode kernels take every multiple of 4 up to
    128, so the per-token variant of that model decodes with caches too - same tokens as the oracle's prefix re-run,
    logits inside the gate, replayed and issued call by call the same bits."""
    from dl4s_amd import host_lib
    from oracle import transformer as T
    name = "transformer_tests_hyperparameters"
    params, rng = _model(48, *CONFIGS[name])
    src = [int(t) for t in rng.integers(0, CONFIGS[name][0], 6)]
    steps = 18
    ref_tokens, ref_logits = T.greedy_decode(params, src, 1, -5, steps, return_logits=True, norm_per_token=True)
    top2 = np.sort(np.stack(ref_logits), axis=1)[:, -2:]
    assert (top2[:, 1] - top2[:, 0]).min() > 1e-3, "the fixture must not sit on an argmax tie"
    model = host_lib.Transformer(ctx, params)
    model.set_norm_per_token(True)
    toks, logits = model.greedy(src, 1, -5, steps, cached=True, return_logits=True)
    assert toks == ref_tokens
    assert_parity(logits, np.stack(ref_logits), "cached greedy logits, key size 8")
    toks_s, logits_s = model.greedy(src, 1, -5, steps, cached="stepwise", return_logits=True)
    assert toks_s == toks and np.array_equal(logits_s, logits)
    model.close()


def test_transformer_argument_errors(ctx):
    from dl4s_amd import host_lib
    params, rng = _model(44, *CONFIGS["transformer_tests_hyperparameters"])
    model = host_lib.Transformer(ctx, params)
    with pytest.raises(host_lib.HostError):       # token outside the vocabulary: the reference traps on the subscript
        model.forward([[99, 1]], [[1]], [2], [1])
    with pytest.raises(host_lib.HostError):       # padded length differs from the longest sequence
        model.forward([[3, 1, -1]], [[1]], [2], [1])
    model.close()


def test_tensor_codable_json_round_trip(ctx):
    """Tensor: Codable (Tensor/TensorExt.swift:241-271) as JSONEncoder writes it: requiresGradient, base64 data, shape."""
    import base64
    import json
    from dl4s_amd import host_lib
    rng = np.random.default_rng(51)
    x = rng.standard_normal((3, 5, 7)).astype(np.float32)
    x[0, 0, 0], x[1, 2, 3] = np.inf, -0.0
    text = host_lib.tensor_encode_json(ctx, x)
    obj = json.loads(text)
    assert obj["shape"] == [3, 5, 7] and obj["requiresGradient"] is False
    assert base64.b64decode(obj["data"]) == x.tobytes()
    assert np.array_equal(host_lib.tensor_decode_json(ctx, text), x)
    # a document written elsewhere: other key order, whitespace, Foundation's escaped slashes
    doc = json.dumps({"shape": [5, 21], "data": base64.b64encode(x.tobytes()).decode(), "requiresGradient": True}, indent=1)
    doc = doc.replace("/", "\\/")
    assert np.array_equal(host_lib.tensor_decode_json(ctx, doc), x.reshape(5, 21))
    for bad in ('{"shape":[2,2],"data":"AAAA","requiresGradient":false}', '{"data":"AAAA"}'):
        with pytest.raises(host_lib.HostError):
            host_lib.tensor_decode_json(ctx, bad)
    s = host_lib.tensor_decode_json(ctx, host_lib.tensor_encode_json(ctx, np.float32(2.5)))      # scalar: shape []
    assert s.shape == () and s == np.float32(2.5)
