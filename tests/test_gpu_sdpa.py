"""Parity of the fused HIP attention kernels (through the C ABI) against the CPU oracle.

Gate: |gpu - oracle| <= 1e-4 + 1e-4 * |oracle| element-wise (fp32), NaN/Inf at exactly the same
positions, structured masks bit-identical to the dense mask they describe, mask == nil bit-identical
to an all-zero mask.
"""
import zlib

import numpy as np
import pytest

from helpers import assert_parity, causal_mask, lengths_mask

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from dl4s_amd import lib
    c = lib.Context(0)
    yield c
    c.close()


def run_sdpa(ctx, q, k, v, mask=None, kind=None, lens=None, strict=False, temperature=None, token_major=False, no_split=None):
    from dl4s_amd import lib
    B, H, Lq, dk = q.shape
    Lk, dv = v.shape[2], v.shape[3]
    T = np.float32(np.sqrt(np.float32(dk))) if temperature is None else np.float32(temperature)
    rT = float(np.float32(1.0) / T)
    if token_major:     # hand the kernel [B,L,H,d] tensors and give the caller back [B,H,L,d]
        q, k, v = (np.ascontiguousarray(x.transpose(0, 2, 1, 3)) for x in (q, k, v))
    bufs = [ctx.to_device(q), ctx.to_device(k), ctx.to_device(v), ctx.empty((B, H, Lq, dv))]
    desc = None
    if kind is None:
        kind = lib.MASK_NONE if mask is None else lib.MASK_DENSE
    if kind == lib.MASK_DENSE:
        md = ctx.to_device(mask)
        bufs.append(md)
        desc = ctx.mask_desc(lib.MASK_DENSE, dense=md)
    elif kind in (lib.MASK_KEY_LENGTHS, lib.MASK_CAUSAL_OR_KEY_LENGTHS):
        ld = ctx.to_device(np.asarray(lens, np.int32), dtype=np.int32)
        bufs.append(ld)
        desc = ctx.mask_desc(kind, lengths=ld)
    elif kind == lib.MASK_CAUSAL:
        desc = ctx.mask_desc(lib.MASK_CAUSAL)
    if no_split is None:
        no_split = NO_SPLIT_DEFAULT[0]
    flags = (lib.SDPA_STRICT if strict else 0) | (lib.SDPA_TOKEN_MAJOR if token_major else 0) | (lib.SDPA_NO_KEY_SPLIT if no_split else 0)
    ctx.sdpa_fwd(bufs[0], bufs[1], bufs[2], bufs[3], B, H, Lq, Lk, dk, dv, rT, desc, flags)
    out = bufs[3].numpy()
    if token_major:
        out = np.ascontiguousarray(out.reshape(B, Lq, H, dv).transpose(0, 2, 1, 3))
    for b in bufs:
        b.release()
    return out


# Small launches run the key-split kernel unless DL4S_SDPA_NO_KEY_SPLIT is set; the module's tests run once per variant.
NO_SPLIT_DEFAULT = [False]


@pytest.fixture(autouse=True, params=["key_split_auto", "no_key_split"])
def kernel_variant(request):
    NO_SPLIT_DEFAULT[0] = request.param == "no_key_split"
    yield
    NO_SPLIT_DEFAULT[0] = False


def rand(rng, *shape, scale=1.0):
    return (rng.standard_normal(shape) * scale).astype(np.float32)


# ------------------------------------------------------------------ small shapes, every mask kind
SHAPES = [  # B, H, Lq, Lk, d
    (1, 2, 5, 7, 4),        # the golden-fixture shape: the 16-wide MFMA kernel with 12 padding columns
    (2, 3, 9, 11, 8),       # key size of Tests/DL4STests/TransformerTests.swift:31
    (2, 3, 9, 11, 6),       # not a multiple of 4: plain kernel
    (1, 2, 40, 50, 96),     # above 64: the 128-wide MFMA kernel with padding columns
    (2, 2, 200, 333, 128),
    (2, 3, 130, 70, 72),
    (1, 2, 100, 100, 100),
    (1, 2, 40, 50, 130),    # not a multiple of 4 / above 128: plain kernel
    (1, 1, 33, 40, 200),
    (2, 3, 130, 70, 16),    # the 16-wide kernels, every column used
    (1, 2, 100, 100, 12),   # the 16-wide kernels with padding columns
    (2, 2, 200, 333, 24),   # the 32-wide kernels with padding columns
    (2, 3, 130, 70, 32),    # the 32-wide kernels, ragged
    (2, 2, 200, 333, 40),
    (1, 2, 100, 100, 60),
    (1, 2, 5, 7, 64),       # MFMA kernel, ragged single tile
    (2, 3, 130, 70, 64),    # ragged: Lq and Lk cross tile edges
    (1, 2, 128, 128, 64),
    (2, 2, 200, 333, 64),
    (1, 1, 1, 1, 64),       # single query, single key
    (1, 1, 300, 1, 64),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("mk", ["none", "dense_qk", "dense_full", "dense_b11k", "causal", "lens", "causal_lens", "half"])
def test_sdpa_matches_oracle(ctx, orc, shape, mk):
    from dl4s_amd import lib
    B, H, Lq, Lk, d = shape
    rng = np.random.default_rng(zlib.crc32(repr((shape, mk)).encode()))   # the same inputs in every process
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(0, Lk + 1, size=B)
    lens[0] = max(1, Lk // 2)
    kind, mask, lens_arg = None, None, None
    if mk == "dense_qk":
        mask = (rng.random((Lq, Lk)) < 0.4).astype(np.float32)
    elif mk == "dense_full":
        mask = (rng.random((B, H, Lq, Lk)) < 0.4).astype(np.float32)
    elif mk == "dense_b11k":
        mask = lengths_mask(lens, Lk)
    elif mk == "half":
        mask = (causal_mask(Lq, Lk) * np.float32(0.5)).reshape(1, 1, Lq, Lk)   # non-binary: a -5e8 penalty
    elif mk == "causal":
        kind, mask = lib.MASK_CAUSAL, causal_mask(Lq, Lk)
    elif mk == "lens":
        kind, mask, lens_arg = lib.MASK_KEY_LENGTHS, lengths_mask(lens, Lk), lens
    elif mk == "causal_lens":
        kind, lens_arg = lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens
        mask = np.maximum(lengths_mask(lens, Lk), causal_mask(Lq, Lk)[None, None])
    ref = orc.sdpa(q, k, v, mask)
    got = run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg)
    assert_parity(got, ref, "sdpa %s %s" % (shape, mk))
    if kind is not None:
        # structured descriptor == the dense mask it stands for, bit for bit (strict visits the same tiles)
        dense = run_sdpa(ctx, q, k, v, mask, strict=True)
        strict = run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, strict=True)
        assert np.array_equal(strict, dense)
        assert_parity(got, dense, "skip vs dense")
    if mask is not None:
        # a dense mask without the strict flag skips the all-ones tiles of query blocks whose rows all keep a key:
        # zero weights either way, the same bits
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask), run_sdpa(ctx, q, k, v, mask, strict=True))


def test_different_key_and_value_dims(ctx, orc):
    rng = np.random.default_rng(77)
    for dk, dv in [(8, 16), (64, 32), (5, 70)]:
        q, k, v = rand(rng, 2, 2, 40, dk), rand(rng, 2, 2, 55, dk), rand(rng, 2, 2, 55, dv)
        mask = (rng.random((40, 55)) < 0.3).astype(np.float32)
        assert_parity(run_sdpa(ctx, q, k, v, mask), orc.sdpa(q, k, v, mask), "dk %d dv %d" % (dk, dv))


@pytest.mark.parametrize("dk,dv", [(70, 70), (6, 6), (40, 24), (5, 128), (100, 36)])
def test_head_dims_served_by_padded_copies(ctx, orc, dk, dv):
    """Key dim != value dim or not a multiple of 4, on problems large enough for the padded-copy route (the MFMA kernels
    on zero-padded copies of the operands): every mask kind against the oracle, the structured kinds bit-identical to the
    dense tensors they describe, NaN / Inf placement as in the oracle."""
    from dl4s_amd import lib
    rng = np.random.default_rng(dk * 131 + dv)
    B, H, Lq, Lk = 2, 3, 330, 420
    assert B * H * Lq * Lk * max(dk, dv) >= 1 << 24 or (dk, dv) == (6, 6)
    if (dk, dv) == (6, 6):
        B, H, Lq, Lk = 2, 4, 900, 800
    q, k, v = rand(rng, B, H, Lq, dk), rand(rng, B, H, Lk, dk), rand(rng, B, H, Lk, dv)
    lens = [Lk - 57, 31][:B]
    i, j = np.indices((Lq, Lk))
    causal = (j > i).astype(np.float32)
    pad = (np.arange(Lk)[None, None, None, :] >= np.asarray(lens)[:, None, None, None]).astype(np.float32)
    for name, mask, kind, lens_arg in (("none", None, None, None), ("causal", causal, lib.MASK_CAUSAL, None),
                                       ("lens", pad, lib.MASK_KEY_LENGTHS, lens)):
        sample = (slice(0, 1), slice(0, 2))          # the single-thread oracle on a sample of the pairs
        ref = orc.sdpa(q[sample], k[sample], v[sample], None if mask is None else (mask if mask.ndim == 2 else mask[:1]))
        got = run_sdpa(ctx, q, k, v, mask)
        assert_parity(got[sample], ref, "padded %s dk %d dv %d" % (name, dk, dv))
        assert np.isfinite(got).all()
        if kind is not None:
            assert np.array_equal(run_sdpa(ctx, q, k, v, kind=kind, lens=lens_arg, strict=True), run_sdpa(ctx, q, k, v, mask, strict=True))
    q2, k2 = q.copy(), k.copy()
    q2[0, 0, 5, 1] = np.nan
    k2[0, 1, 9, 0] = np.inf
    got = run_sdpa(ctx, q2, k2, v, causal)
    ref = orc.sdpa(q2[:1, :2], k2[:1, :2], v[:1, :2], causal)
    assert np.array_equal(np.isnan(got[:1, :2]), np.isnan(ref))
    assert_parity(np.nan_to_num(got[:1, :2]), np.nan_to_num(ref), "padded NaN / Inf dk %d dv %d" % (dk, dv))


def test_nil_mask_equals_zero_mask_bitwise(ctx):
    rng = np.random.default_rng(3)
    for d in (8, 10, 64, 128, 100):
        q, k, v = rand(rng, 2, 2, 70, d), rand(rng, 2, 2, 90, d), rand(rng, 2, 2, 90, d)
        a = run_sdpa(ctx, q, k, v, None)
        b = run_sdpa(ctx, q, k, v, np.zeros((70, 90), np.float32))
        assert np.array_equal(a, b)


@pytest.mark.parametrize("d", [8, 10, 64, 128, 88])
def test_blocked_keys_have_exactly_zero_weight_and_blocked_rows_are_uniform(ctx, orc, d):
    rng = np.random.default_rng(5)
    B, H, Lq, Lk = 1, 2, 70, 100
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    mask = np.zeros((Lq, Lk), np.float32)
    mask[:, 61:] = 1
    mask[33, :] = 1                      # fully blocked row
    base = run_sdpa(ctx, q, k, v, mask)
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 61:] = 7.0                  # finite changes at blocked keys must not move a single bit
    v2[:, :, 61:] = -321.0
    other = run_sdpa(ctx, q, k2, v2, mask)
    rows = [r for r in range(Lq) if r != 33]
    assert np.array_equal(base[:, :, rows], other[:, :, rows])
    ref = orc.sdpa(q, k, v, mask)
    assert_parity(base, ref, "blocked")
    assert np.allclose(base[:, :, 33], v.mean(axis=2), atol=1e-5)       # uniform 1/Lk, never NaN
    assert not np.isnan(base).any()


@pytest.mark.parametrize("d", [64, 8, 32, 128, 10, 16, 48, 80, 96, 160, 256])
@pytest.mark.parametrize("mk", ["dense", "dense_ones_tiles", "lens", "causal_lens"])
def test_fully_blocked_rows_with_large_scores_follow_the_reference_rounding(ctx, orc, d, mk):
    """A row whose every key is blocked: the reference's fl(s - 1e9) keeps a score only as its bucket on the grid of 64
    that floats have next to 1e9, so with scores beyond +-32 the row is not uniform - the keys of the highest bucket
    share it (ScaledDotProductAttention.swift:55-59).  Scores here reach +-150; the oracle does that arithmetic, the
    kernels have to land in the same buckets (MFMA kernels: d = 64, 8, 32, 128; plain kernel: d = 10)."""
    from dl4s_amd import lib
    rng = np.random.default_rng(zlib.crc32(repr(("blocked large", d, mk)).encode()))
    B, H, Lq, Lk = 2, 2, 70, 100
    if mk == "causal_lens":
        Lk = Lq
    q, k, v = rand(rng, B, H, Lq, d, scale=5.0), rand(rng, B, H, Lk, d, scale=5.0), rand(rng, B, H, Lk, d)
    kind, lens_arg, lens = None, None, np.array([0, Lk // 2])
    if mk == "dense":
        mask = (rng.random((B, 1, Lq, Lk)) < 0.5).astype(np.float32)
        mask[:, :, 5, :] = 1.0
        mask[:, :, 40:44, :] = 1.0
    elif mk == "dense_ones_tiles":
        mask = np.zeros((B, 1, Lq, Lk), np.float32)
        mask[:, :, 32:64, :] = 1.0           # a whole 32-row block blocked: tiles of ones only
    elif mk == "lens":
        kind, lens_arg, mask = lib.MASK_KEY_LENGTHS, lens, lengths_mask(lens, Lk)         # batch item 0 has no valid key
    else:
        kind, lens_arg = lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens
        mask = np.maximum(lengths_mask(lens, Lk), causal_mask(Lq, Lk)[None, None])
    blocked = np.broadcast_to(mask, (B, H, Lq, Lk)).min(axis=3) >= 1.0
    assert blocked.any()
    # In the blocked rows keep every score 0.05 away from a bucket edge (32 + 64 n), where the last bits of the kernel's
    # score - summed in another order than the oracle's - would decide the bucket: nudge the query rows until none is left.
    T = float(np.float32(np.sqrt(np.float32(d))))
    for _ in range(50):
        s = np.einsum("bhid,bhjd->bhij", q.astype(np.float64) / T, k.astype(np.float64))
        edge = np.abs(np.abs(s) - 32.0) % 64.0
        near = (np.minimum(edge, 64.0 - edge) < 0.05) & blocked[..., None]
        if not near.any():
            break
        for b, h, i in np.argwhere(near.any(axis=3)):
            q[b, h, i] *= np.float32(1.003)
    assert not near.any()
    ref = orc.sdpa(q, k, v, mask)
    b0, h0, i0 = np.argwhere(blocked)[0]
    assert not np.allclose(ref[b0, h0, i0], v[b0, h0].mean(axis=0), atol=1e-3)      # the reference's rows are not uniform here
    for strict in (False, True):
        got = run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, strict=strict)
        assert_parity(got, ref, "fully blocked rows, large scores, d=%d %s strict=%s" % (d, mk, strict))
    if kind is not None:
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, strict=True), run_sdpa(ctx, q, k, v, mask, strict=True))


@pytest.mark.parametrize("d", [8, 10, 64, 128, 88])
def test_nan_inf_placement_matches_oracle(ctx, orc, d):
    rng = np.random.default_rng(9)
    B, H, Lq, Lk = 1, 1, 40, 150
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    q[0, 0, 3, 0] = np.nan               # NaN scores in row 3     -> row NaN
    q[0, 0, 5, :] = 0
    q[0, 0, 5, 1] = np.inf               # +/-Inf scores in row 5  -> row NaN
    k[0, 0, 140, :] = 0
    k[0, 0, 140, 2] = 3e38               # huge finite key: q.k overflows for some rows only
    mask = np.zeros((Lq, Lk), np.float32)
    mask[7, :] = np.inf                  # every score of row 7 is -Inf -> row NaN
    mask[9, 100:] = np.inf               # -Inf on a suffix (whole later tiles) -> weights 0 there, row finite
    mask[11, :70] = np.inf               # -Inf on the leading tile -> still finite
    with np.errstate(all="ignore"):
        ref = orc.sdpa(q, k, v, mask)
    got = run_sdpa(ctx, q, k, v, mask)
    assert np.isnan(ref[0, 0, 3]).all() and np.isnan(ref[0, 0, 5]).all() and np.isnan(ref[0, 0, 7]).all()
    assert not np.isnan(ref[0, 0, 9]).any() and not np.isnan(ref[0, 0, 11]).any()
    assert_parity(got, ref, "nan/inf d=%d" % d)


@pytest.mark.parametrize("seed", range(40))
def test_random_non_finite_values_visiting_every_tile(ctx, orc, seed):
    """Seeded random extents, head dims, mask kinds (non-binary values among them) and layouts with NaN and infinities at
    random places of q, k, v and the mask, every tile visited (DL4S_SDPA_STRICT, the reference's behaviour): NaN and
    Inf at exactly the oracle's positions, everything else within the gate."""
    from dl4s_amd import lib
    rng = np.random.default_rng(70000 + seed)
    B, H = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    Lq, Lk = int(rng.integers(1, 200)), int(rng.integers(1, 200))
    kind_name = ["none", "dense", "dense_bcast", "lengths", "causal", "causal_lengths", "scaled"][int(rng.integers(0, 7))]
    if kind_name.startswith("causal"):
        Lk = Lq
    d = int(rng.choice([4, 8, 16, 24, 32, 40, 64, 64, 72, 96, 128, 10, 130]))
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(0, Lk + 1, size=B)
    kw, mask = {}, None
    if kind_name == "dense":
        mask = (rng.random((B, H, Lq, Lk)) < rng.choice([0.1, 0.5, 0.9])).astype(np.float32)
        kw = dict(mask=mask)
    elif kind_name == "scaled":
        mask = ((rng.random((Lq, Lk)) < 0.5) * rng.choice([0.5, 2.0, -1.0, 1e-9])).astype(np.float32)
        kw = dict(mask=mask)
    elif kind_name == "dense_bcast":
        mask = (rng.random((B, 1, 1, Lk)) < 0.5).astype(np.float32)
        kw = dict(mask=mask)
    elif kind_name == "lengths":
        mask, kw = lengths_mask(lens, Lk), dict(kind=lib.MASK_KEY_LENGTHS, lens=lens)
    elif kind_name == "causal":
        mask, kw = causal_mask(Lq, Lq), dict(kind=lib.MASK_CAUSAL)
    elif kind_name == "causal_lengths":
        mask = np.maximum(lengths_mask(lens, Lk), causal_mask(Lq, Lq)[None, None])
        kw = dict(kind=lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens=lens)
    specials = [np.nan, np.inf, -np.inf]
    for arr in (q, k, v):
        if rng.random() < 0.5:
            for _ in range(int(rng.integers(1, 4))):
                arr[tuple(int(rng.integers(0, n)) for n in arr.shape)] = specials[int(rng.integers(0, 3))]
    if kind_name in ("dense", "scaled") and rng.random() < 0.3:
        mask[tuple(int(rng.integers(0, n)) for n in mask.shape)] = specials[int(rng.integers(0, 3))]
    tm = bool(rng.integers(0, 2)) and d % 4 == 0 and d <= 128
    with np.errstate(all="ignore"):
        ref = orc.sdpa(q, k, v, mask)
    got = run_sdpa(ctx, q, k, v, strict=True, token_major=tm, **kw)
    assert_parity(got, ref, "seed %d: B%d H%d Lq%d Lk%d d%d %s token_major=%s" % (seed, B, H, Lq, Lk, d, kind_name, tm))


@pytest.mark.parametrize("d", [8, 10, 64, 128])
def test_mask_penalties_at_the_top_of_the_float_range(ctx, orc, d):
    """mask * 1e9 is finite up to a mask value of 3.4e29 (the reference then subtracts about 3e38 and the row, if every key
    has that value, comes out uniform); the kernels hold penalties in the base-2 exponent domain, where the same penalty
    times log2(e) would be infinite and the row NaN.  Beyond 3.4e29 the reference's product is infinite as well."""
    rng = np.random.default_rng(31)
    B, H, Lq, Lk = 1, 2, 40, 75
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    mask = (rng.random((Lq, Lk)) < 0.3).astype(np.float32)
    mask[3, :] = 3e29            # every key: uniform row
    mask[5, 10:] = 3e29          # some keys: weight zero there
    mask[7, :] = 2e29            # finite in both domains
    mask[9, :] = 3.5e29          # mask * 1e9 overflows in the reference too: -inf everywhere, NaN row
    mask[11, :] = -3e29          # a bonus of 3e38 on every key: uniform again
    mask[13, 40] = -3e29         # one key takes all the weight
    with np.errstate(all="ignore"):
        ref = orc.sdpa(q, k, v, mask)
    assert np.isnan(ref[:, :, 9]).all() and np.isnan(ref).sum() == B * H * d
    assert np.allclose(ref[:, :, 3], v.mean(axis=2), atol=1e-5) and np.array_equal(ref[:, :, 13], v[:, :, 40])
    for strict in (False, True):
        got = run_sdpa(ctx, q, k, v, mask, strict=strict)
        assert_parity(got, ref, "huge mask values d=%d strict=%d" % (d, strict))


def test_nan_in_v_at_blocked_key_reaches_output_only_in_strict_mode(ctx, orc):
    from dl4s_amd import lib
    rng = np.random.default_rng(10)
    B, H, L, d = 1, 1, 256, 64
    q, k, v = rand(rng, B, H, L, d), rand(rng, B, H, L, d), rand(rng, B, H, L, d)
    v[0, 0, 255, 5] = np.nan             # last key: blocked for every query but the last
    mask = causal_mask(L, L)
    with np.errstate(all="ignore"):
        ref = orc.sdpa(q, k, v, mask)    # 0 * NaN = NaN in column 5 of every row
    assert np.isnan(ref[0, 0, :, 5]).all()
    strict = run_sdpa(ctx, q, k, v, mask, kind=lib.MASK_CAUSAL, strict=True)
    assert_parity(strict, ref, "strict NaN")
    dense = run_sdpa(ctx, q, k, v, mask, strict=True)
    assert_parity(dense, ref, "dense NaN")
    fast = run_sdpa(ctx, q, k, v, mask, kind=lib.MASK_CAUSAL)
    assert not np.isnan(fast[0, 0, :128]).any()     # documented: skipped tiles do not propagate it
    fast_dense = run_sdpa(ctx, q, k, v, mask)       # the same for the all-ones tiles of a dense mask
    assert not np.isnan(fast_dense[0, 0, :128]).any()


def test_temperature_is_a_reciprocal_multiply_on_q(ctx, orc):
    rng = np.random.default_rng(12)
    q, k, v = rand(rng, 1, 2, 50, 64), rand(rng, 1, 2, 60, 64), rand(rng, 1, 2, 60, 64)
    got = run_sdpa(ctx, q, k, v, None, temperature=3.0)
    assert_parity(got, orc.sdpa(q, k, v, None, temperature=3.0), "T=3")


def test_error_paths(ctx):
    from dl4s_amd import lib
    q = ctx.empty((1, 1, 4, 64))
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.sdpa_fwd(q, q, q, q, 1, 1, 4, 0, 64, 64, 0.125)          # empty key axis
    assert e.value.code == -2
    bad = ctx.empty((3, 5))
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.sdpa_fwd(q, q, q, q, 1, 1, 4, 4, 64, 64, 0.125, ctx.mask_desc(lib.MASK_DENSE, dense=bad))
    assert e.value.code == -2
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.sdpa_fwd(q, q, q, q, 1, 1, 4, 4, 512, 512, 0.125)
    assert e.value.code == -5
    ctx.sdpa_fwd(q, q, q, q, 0, 1, 4, 4, 64, 64, 0.125)              # empty batch is a no-op
    q.release()
    bad.release()


# ------------------------------------------------------------------ the benchmark configurations
def test_config1_sdpa_b1_h8_l128_d64(ctx, orc):
    rng = np.random.Generator(np.random.PCG64(1001))
    q, k, v = (rng.standard_normal((1, 8, 128, 64), dtype=np.float32) for _ in range(3))
    ref = orc.sdpa(q, k, v, None)
    got = run_sdpa(ctx, q, k, v, None)
    err = assert_parity(got, ref, "config 1")
    assert err < 1e-5


def test_config4_long_causal_prefill_sampled_against_oracle(ctx, orc):
    """B8 H16 L2048 d64 causal, inputs 0.5*N(0,1).  The oracle is evaluated on sampled (batch, head)
    pairs and query rows (rows are independent), the full output is checked through invariants."""
    from dl4s_amd import lib
    B, H, L, d = 8, 16, 2048, 64
    rng = np.random.Generator(np.random.PCG64(1004))
    q, k, v = (rng.standard_normal((B, H, L, d), dtype=np.float32) * np.float32(0.5) for _ in range(3))
    got = run_sdpa(ctx, q, k, v, kind=lib.MASK_CAUSAL)
    assert np.isfinite(got).all()
    # row 0 attends to key 0 only
    assert np.allclose(got[:, :, 0], v[:, :, 0], atol=1e-6)
    # every output is a convex combination of the visible V rows
    vmax = np.maximum.accumulate(v, axis=2)
    vmin = np.minimum.accumulate(v, axis=2)
    assert (got <= vmax + 1e-5).all() and (got >= vmin - 1e-5).all()
    srng = np.random.default_rng(4)
    rows = np.unique(np.concatenate([[0, 1, 31, 32, 63, 64, 127, 128, 2047], srng.integers(0, L, 40)]))
    cm = causal_mask(L, L)[rows]
    for (b, h) in [(0, 0), (3, 7), (7, 15)]:
        ref = orc.sdpa(q[b:b + 1, h:h + 1, rows], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], cm)
        assert_parity(got[b:b + 1, h:h + 1, rows], ref, "config 4 (b=%d,h=%d)" % (b, h))


def test_paired_causal_blocks_with_an_odd_block_count(ctx, orc):
    """Large causal launches pair long and short 128-query blocks in one workgroup; 9 blocks leave the middle
    one unpaired.  B16 H16 L1152 d64, checked on sampled rows of every block."""
    from dl4s_amd import lib
    B, H, L, d = 16, 16, 1152, 64
    rng = np.random.default_rng(1152)
    q, k, v = (rng.standard_normal((B, H, L, d), dtype=np.float32) for _ in range(3))
    got = run_sdpa(ctx, q, k, v, kind=lib.MASK_CAUSAL)
    strict = run_sdpa(ctx, q, k, v, kind=lib.MASK_CAUSAL, strict=True)     # unpaired, visits every tile
    assert_parity(got, strict, "paired vs strict")
    rows = np.concatenate([np.arange(0, L, 128), np.arange(127, L, 128), [500, 640, 1151]])
    cm = causal_mask(L, L)[rows]
    for (b, h) in [(0, 0), (15, 15)]:
        ref = orc.sdpa(q[b:b + 1, h:h + 1, rows], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], cm)
        assert_parity(got[b:b + 1, h:h + 1, rows], ref, "paired (b=%d,h=%d)" % (b, h))


def test_config3_shape_padding_mask_sampled(ctx, orc):
    """SDPA core of the encoder block: B8 H16 L1024 d64, key-length mask U[512,1024]."""
    from dl4s_amd import lib
    B, H, L, d = 8, 16, 1024, 64
    rng = np.random.Generator(np.random.PCG64(1003))
    q, k, v = (rng.standard_normal((B, H, L, d), dtype=np.float32) for _ in range(3))
    lens = rng.integers(512, 1025, size=B)
    got = run_sdpa(ctx, q, k, v, kind=lib.MASK_KEY_LENGTHS, lens=lens)
    rows = np.array([0, 5, 511, 512, 777, 1023])
    for (b, h) in [(0, 0), (5, 9)]:
        m = np.broadcast_to(lengths_mask(lens, L)[b:b + 1], (1, 1, len(rows), L)).copy()
        ref = orc.sdpa(q[b:b + 1, h:h + 1, rows], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], m)
        assert_parity(got[b:b + 1, h:h + 1, rows], ref, "config 3 core (b=%d,h=%d)" % (b, h))


# ------------------------------------------------------------------ decode
def run_decode(ctx, q, kc, vc, T, lens=None):
    B, H, Tcap, d = kc.shape
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
    bufs = [ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc), ctx.empty((B, H, 1, d))]
    if lens is None:
        ctx.sdpa_decode(bufs[0], bufs[1], bufs[2], bufs[3], B, H, T, Tcap, d, rT)
    else:
        bufs.append(ctx.to_device(np.asarray(lens, np.int32), dtype=np.int32))
        ctx.sdpa_decode_lengths(bufs[0], bufs[1], bufs[2], bufs[3], B, H, T, Tcap, d, rT, bufs[4])
    out = bufs[3].numpy()
    for b in bufs:
        b.release()
    return out


@pytest.mark.parametrize("B,H,T,Tcap", [(1, 1, 1, 1), (2, 3, 9, 12), (2, 2, 128, 128), (2, 2, 129, 140), (2, 2, 256, 256),
                                        (1, 4, 257, 300), (1, 8, 512, 512), (1, 8, 513, 600), (3, 2, 1000, 1024),
                                        (2, 2, 4097, 4160)])
def test_decode_matches_oracle(ctx, orc, B, H, T, Tcap):
    rng = np.random.default_rng(T)
    q, kc, vc = rand(rng, B, H, 1, 64), rand(rng, B, H, Tcap, 64), rand(rng, B, H, Tcap, 64)
    kc[:, :, T:] = np.nan           # rows beyond T must never be read into the result
    vc[:, :, T:] = np.nan
    ref = orc.sdpa_decode(q, kc, vc, T)
    got = run_decode(ctx, q, kc, vc, T)
    assert_parity(got, ref, "decode T=%d" % T)
    # and it is the same function as the prefill kernel with one query
    pre = run_sdpa(ctx, q, np.ascontiguousarray(kc[:, :, :T]), np.ascontiguousarray(vc[:, :, :T]))
    assert_parity(got, pre, "decode vs prefill")


@pytest.mark.parametrize("d", [32, 128, 8, 4, 40, 96, 100, 70, 1, 3, 6, 33, 127, 256, 192, 130, 255, 80, 160])
@pytest.mark.parametrize("B,H,T,Tcap", [(1, 1, 1, 1), (2, 3, 9, 12), (2, 2, 129, 140), (1, 4, 257, 300), (1, 8, 513, 600),
                                        (3, 2, 1000, 1024), (2, 2, 4097, 4160)])
def test_decode_other_head_dims(ctx, orc, B, H, T, Tcap, d):
    """Cache rows of 32 and 128 floats (8 and 32 lanes per row), head dims that leave lanes idle, and head dims that are no
    multiple of 4 (rows off the 16-byte grid: one float per load)."""
    rng = np.random.default_rng(T * 1000 + d)
    q, kc, vc = rand(rng, B, H, 1, d), rand(rng, B, H, Tcap, d), rand(rng, B, H, Tcap, d)
    kc[:, :, T:] = np.nan
    vc[:, :, T:] = np.nan
    ref = orc.sdpa_decode(q, kc, vc, T)
    got = run_decode(ctx, q, kc, vc, T)
    assert_parity(got, ref, "decode T=%d d=%d" % (T, d))
    assert_parity(got, run_sdpa(ctx, q, np.ascontiguousarray(kc[:, :, :T]), np.ascontiguousarray(vc[:, :, :T])), "decode vs prefill")


@pytest.mark.parametrize("d", [64, 32, 128, 24, 70, 5, 96, 256, 200, 192, 80, 160])
@pytest.mark.parametrize("B,H,T,Tcap", [(4, 2, 9, 12), (5, 2, 300, 320), (6, 3, 1000, 1024), (4, 2, 4097, 4160)])
def test_decode_with_key_lengths(ctx, orc, B, H, T, Tcap, d):
    """dl4s_hip_sdpa_decode_lengths_f32 against the oracle's attention on the gathered tensors under the padding mask
    m[b,0,0,j] = (j >= lengths[b]): a length inside the cache, the whole cache, beyond it, one key, and zero (every key
    blocked: the row is uniform over all T keys, never NaN)."""
    rng = np.random.default_rng(T * 100 + d)
    q, kc, vc = rand(rng, B, H, 1, d), rand(rng, B, H, Tcap, d), rand(rng, B, H, Tcap, d)
    kc[:, :, T:] = np.nan
    vc[:, :, T:] = np.nan
    lens = rng.integers(1, T + 1, size=B)
    lens[0], lens[1], lens[2], lens[3] = T, 0, 1, T + 50
    mask = lengths_mask(lens, T)
    ref = orc.sdpa(q, np.ascontiguousarray(kc[:, :, :T]), np.ascontiguousarray(vc[:, :, :T]), mask)
    got = run_decode(ctx, q, kc, vc, T, lens=lens)
    assert_parity(got, ref, "decode with lengths T=%d d=%d" % (T, d))
    assert np.allclose(got[1], vc[1, :, :T].mean(axis=1, keepdims=True), atol=1e-5)      # length zero: uniform
    assert np.array_equal(got[2], vc[2, :, :1])                                           # one key
    assert np.array_equal(got[0], run_decode(ctx, q, kc, vc, T)[0])                        # nothing blocked: the plain entry's bits
    # and it is what the prefill kernel gives for one query under the key-length descriptor
    from dl4s_amd import lib
    pre = run_sdpa(ctx, q, np.ascontiguousarray(kc[:, :, :T]), np.ascontiguousarray(vc[:, :, :T]), kind=lib.MASK_KEY_LENGTHS,
                   lens=np.minimum(lens, T))
    assert_parity(got, pre, "decode with lengths vs prefill")


@pytest.mark.parametrize("shift", [1, 2])
@pytest.mark.parametrize("d", [64, 128, 20, 96, 256, 192, 80])
@pytest.mark.parametrize("T,Tcap", [(9, 12), (700, 701), (4100, 4100)])
def test_decode_on_operands_off_the_16_byte_grid(ctx, orc, T, Tcap, d, shift):
    """Every operand 4 or 8 bytes past a 16-byte boundary (a view into a larger buffer): the kernel reads 32 or 64 bits per
    load and gives the bits of the aligned call (the same kernel form); decode_step appends through the same path."""
    rng = np.random.default_rng(T + d)
    B, H = 2, 3
    q, kc, vc = rand(rng, B, H, 1, d), rand(rng, B, H, Tcap, d), rand(rng, B, H, Tcap, d)
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
    aligned = run_decode(ctx, q, kc, vc, T)
    pad = lambda x: np.concatenate([np.zeros(shift, np.float32), x.ravel()])
    dq, dk_, dv_ = ctx.to_device(pad(q)), ctx.to_device(pad(kc)), ctx.to_device(pad(vc))
    dout = ctx.empty((B * H * d + shift,))
    off = 4 * shift
    ctx.sdpa_decode(dq.offset(off), dk_.offset(off), dv_.offset(off), dout.offset(off), B, H, T, Tcap, d, rT)
    got = dout.numpy()[shift:].reshape(B, H, 1, d)
    if d not in (96, 192, 80, 160):     # aligned rows of exactly 96, 192, 80 or 160 floats run forms of their own (three pieces per lane): another summation order
        assert np.array_equal(got, aligned)
    assert_parity(got, orc.sdpa_decode(q, kc, vc, T), "decode, unaligned operands")
    if T < Tcap:
        kn, vn = rand(rng, B, H, 1, d), rand(rng, B, H, 1, d)
        dkn, dvn = ctx.to_device(pad(kn)), ctx.to_device(pad(vn))
        ctx.sdpa_decode_step(dq.offset(off), dk_.offset(off), dv_.offset(off), dkn.offset(off), dvn.offset(off), dout.offset(off), B, H, T, Tcap, d, rT)
        kc2, vc2 = kc.copy(), vc.copy()
        kc2[:, :, T], vc2[:, :, T] = kn[:, :, 0], vn[:, :, 0]
        assert np.array_equal(dk_.numpy()[shift:].reshape(kc.shape), kc2) and np.array_equal(dv_.numpy()[shift:].reshape(vc.shape), vc2)
        assert_parity(dout.numpy()[shift:].reshape(B, H, 1, d), orc.sdpa_decode(q, kc2, vc2, T + 1), "decode step, unaligned operands")
        dkn.release(); dvn.release()
    for b_ in (dq, dk_, dv_, dout):
        b_.release()


@pytest.mark.parametrize("B,H,T,Tcap,d", [(2, 4, 131072, 131072, 64), (1, 2, 1000001, 1000001, 32), (1, 3, 200000, 262144, 128), (2, 2, 70001, 70001, 70),
                                          (1, 2, 100000, 100000, 256)])
def test_decode_over_very_long_caches(ctx, B, H, T, Tcap, d):
    """Caches far longer than the oracle finishes: the decode (plain and with key lengths) against an fp64 model written
    from the definition."""
    rng = np.random.default_rng(T + d)
    q, kc, vc = rand(rng, B, H, 1, d), rand(rng, B, H, Tcap, d), rand(rng, B, H, Tcap, d)
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
    s = np.einsum("bhtd,bhd->bht", kc[:, :, :T].astype(np.float64), q[:, :, 0].astype(np.float64)) * rT

    def model(n_of_batch):
        ref = np.empty((B, H, 1, d))
        for b, n in enumerate(n_of_batch):
            p = np.exp(s[b, :, :n] - s[b, :, :n].max(-1, keepdims=True))
            p /= p.sum(-1, keepdims=True)
            ref[b, :, 0] = np.einsum("ht,htd->hd", p, vc[b, :, :n].astype(np.float64))
        return ref
    np.testing.assert_allclose(run_decode(ctx, q, kc, vc, T), model([T] * B), rtol=1e-4, atol=2e-6)
    lens = [T - 7] + [T // 3] * (B - 1)
    np.testing.assert_allclose(run_decode(ctx, q, kc, vc, T, lens=np.array(lens)), model(lens), rtol=1e-4, atol=2e-6)


def test_decode_nan_inf(ctx, orc):
    rng = np.random.default_rng(77)
    B, H, T = 2, 2, 600
    q, kc, vc = rand(rng, B, H, 1, 64), rand(rng, B, H, T, 64), rand(rng, B, H, T, 64)
    kc[0, 0, 300, 0] = np.nan       # (0,0): NaN score -> NaN output
    q[1, 1, 0, :] = 0
    q[1, 1, 0, 3] = np.inf          # (1,1): +/-Inf scores -> NaN output
    with np.errstate(all="ignore"):
        ref = orc.sdpa_decode(q, kc, vc, T)
    got = run_decode(ctx, q, kc, vc, T)
    assert np.isnan(ref[0, 0]).all() and np.isnan(ref[1, 1]).all() and not np.isnan(ref[0, 1]).any()
    assert_parity(got, ref, "decode nan/inf")


@pytest.mark.parametrize("T", [1, 9, 45, 300, 1000, 2077])      # none a multiple of 32: the last block has lanes past the end
def test_decode_non_finite_values_in_the_last_cached_row(ctx, orc, T):
    """Lanes past the end of the cache re-read row T-1 with weight zero; they must add nothing (0 * Inf would be NaN)."""
    rng = np.random.default_rng(T)
    B, H = 2, 3
    q, kc, vc = rand(rng, B, H, 1, 64), rand(rng, B, H, T + 5, 64), rand(rng, B, H, T + 5, 64)
    vc[0, 0, T - 1, 7] = np.inf          # a valid row: weight > 0 times Inf = Inf in that column, in the reference too
    vc[0, 1, T - 1, 9] = -np.inf
    vc[1, 2, T - 1, 11] = np.nan
    kc[1, 0, T - 1, :] = 0
    kc[1, 0, T - 1, 3] = 3e38            # the last row's score overflows for this pair
    with np.errstate(all="ignore"):
        ref = orc.sdpa_decode(q, kc, vc, T)
    assert np.isposinf(ref[0, 0, 0, 7]) and np.isneginf(ref[0, 1, 0, 9]) and np.isnan(ref[1, 2, 0, 11])
    assert np.isfinite(ref[0, 0, 0, :7]).all() and np.isfinite(ref[0, 2]).all()
    assert_parity(run_decode(ctx, q, kc, vc, T), ref, "decode, non-finite last row, T=%d" % T)


def test_config5_incremental_decode_append_then_attend(ctx, orc):
    """B16 H16 d64, cache of 4096 rows, 64 steps: step t appends row 4096+t and attends over 4097+t rows.
    Checked against the oracle at the first, a middle and the last step on sampled (b, h), and through
    the append invariant (the cache equals the concatenation) at the end."""
    B, H, d, T0, steps = 16, 16, 64, 4096, 64
    Tcap = T0 + steps
    rng = np.random.Generator(np.random.PCG64(1005))
    qs = rng.standard_normal((steps, B, H, 1, d), dtype=np.float32)
    kc = np.zeros((B, H, Tcap, d), np.float32)
    vc = np.zeros((B, H, Tcap, d), np.float32)
    kc[:, :, :T0] = rng.standard_normal((B, H, T0, d), dtype=np.float32)
    vc[:, :, :T0] = rng.standard_normal((B, H, T0, d), dtype=np.float32)
    kn = rng.standard_normal((steps, B, H, 1, d), dtype=np.float32)
    vn = rng.standard_normal((steps, B, H, 1, d), dtype=np.float32)
    dk_, dv_ = ctx.to_device(kc), ctx.to_device(vc)
    dq, dkn, dvn = ctx.to_device(qs), ctx.to_device(kn), ctx.to_device(vn)
    dout = ctx.empty((steps, B, H, 1, d))
    step_bytes = B * H * d * 4
    for t in range(steps):
        if t % 2 == 0:   # fused append+attend
            ctx.sdpa_decode_step(dq.offset(t * step_bytes), dk_, dv_, dkn.offset(t * step_bytes), dvn.offset(t * step_bytes),
                                 dout.offset(t * step_bytes), B, H, T0 + t, Tcap, d, 0.125)
        else:            # separate append, then attend
            ctx.kv_append(dk_, dv_, dkn.offset(t * step_bytes), dvn.offset(t * step_bytes), B, H, T0 + t, Tcap, d)
            ctx.sdpa_decode(dq.offset(t * step_bytes), dk_, dv_, dout.offset(t * step_bytes), B, H, T0 + t + 1, Tcap, d, 0.125)
    out = dout.numpy()
    kfin, vfin = dk_.numpy(), dv_.numpy()
    for t in range(steps):
        kc[:, :, T0 + t] = kn[t, :, :, 0]
        vc[:, :, T0 + t] = vn[t, :, :, 0]
    assert np.array_equal(kfin, kc) and np.array_equal(vfin, vc)
    assert np.isfinite(out).all()
    for t in (0, 1, 31, 62, 63):
        for (b, h) in [(0, 0), (9, 4), (15, 15)]:
            ref = orc.sdpa_decode(qs[t, b:b + 1, h:h + 1], kc[b:b + 1, h:h + 1], vc[b:b + 1, h:h + 1], T0 + t + 1)
            assert_parity(out[t, b:b + 1, h:h + 1], ref, "config 5 step %d (b=%d,h=%d)" % (t, b, h))
    for buf in (dk_, dv_, dq, dkn, dvn, dout):
        buf.release()


@pytest.mark.parametrize("d", [64, 30, 7, 96, 256, 132, 192, 80, 160])
@pytest.mark.parametrize("Tcap,steps", [(300, 260), (100, 90)])      # workgroups of 16 and of 4 wavefronts
def test_decode_step_with_the_position_in_device_memory(ctx, orc, Tcap, steps, d):
    """dl4s_hip_sdpa_decode_step_at_f32 reads the row to append from device memory: a sequence of steps driven by a
    device counter (advanced by dl4s_hip_argmax_to_f32, as cached decoding does) fills the cache and attends like the
    by-value entry point; a position outside the cache leaves cache and output alone."""
    B, H = 2, 3
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))      # 0.125 at d = 64
    rng = np.random.default_rng(5150)
    qs, kn, vn = (rng.standard_normal((steps, B, H, 1, d)).astype(np.float32) for _ in range(3))
    dq, dkn, dvn = ctx.to_device(qs), ctx.to_device(kn), ctx.to_device(vn)
    dk_, dv_ = ctx.empty((B, H, Tcap, d)), ctx.empty((B, H, Tcap, d))
    ctx.fill(float("nan"), dk_, B * H * Tcap * d)          # rows never appended must never be read
    ctx.fill(float("nan"), dv_, B * H * Tcap * d)
    dout = ctx.empty((steps, B, H, 1, d))
    cursor = ctx.to_device(np.zeros(2, np.int32), dtype=np.int32)      # [token (unused here), position]
    scores = ctx.to_device(np.arange(7, dtype=np.float32))
    step_bytes = B * H * d * 4
    for t in range(steps):
        ctx.sdpa_decode_step_at(dq.offset(t * step_bytes), dk_, dv_, dkn.offset(t * step_bytes), dvn.offset(t * step_bytes),
                                dout.offset(t * step_bytes), B, H, cursor.offset(4), Tcap, d, rT)
        ctx.argmax_to(scores, 7, cursor, cursor.offset(4))               # position += 1
    assert list(cursor.numpy()) == [6, steps]
    out, kfin, vfin = dout.numpy(), dk_.numpy(), dv_.numpy()
    assert np.array_equal(kfin[:, :, :steps], np.moveaxis(kn[:, :, :, 0], 0, 2)) and np.isnan(kfin[:, :, steps:]).all()
    assert np.array_equal(vfin[:, :, :steps], np.moveaxis(vn[:, :, :, 0], 0, 2))
    for t in sorted({0, 1, 31, 32, min(127, steps - 1), min(128, steps - 1), min(129, steps - 1), steps - 1}):
        ref = orc.sdpa_decode(qs[t], kfin, vfin, t + 1)
        assert_parity(out[t], ref, "decode step at device position %d" % t)
    # positions outside the cache: nothing is written
    before = dout.numpy().copy()
    for bad in (-1, Tcap, 1 << 20):
        cur = ctx.to_device(np.array([0, bad], np.int32), dtype=np.int32)
        ctx.sdpa_decode_step_at(dq, dk_, dv_, dkn, dvn, dout, B, H, cur.offset(4), Tcap, d, rT)
        assert np.array_equal(dout.numpy(), before, equal_nan=True) and np.array_equal(dk_.numpy(), kfin, equal_nan=True)
        cur.release()
    for buf in (dq, dkn, dvn, dk_, dv_, dout, cursor, scores):
        buf.release()


@pytest.mark.parametrize("d", [64, 8, 16, 28, 36, 128, 80])
@pytest.mark.parametrize("B,H,Lq,Lk", [(2, 3, 130, 70), (1, 2, 5, 7), (2, 4, 256, 256), (1, 5, 33, 161)])
def test_token_major_layout_is_bit_identical(ctx, B, H, Lq, Lk, d):
    """[B,L,H,d] operands (what the projections of MultiHeadAttention produce before its permutes,
    NN/Models/Transformer/MultiHeadAttention.swift:105-117) give the same bits as the permuted [B,H,L,d] ones."""
    from dl4s_amd import lib
    rng = np.random.default_rng(B * 1000 + Lq + d)
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(1, Lk + 1, size=B)
    dense = (rng.random((B, 1, Lq, Lk)) < 0.3).astype(np.float32)
    cases = [dict(), dict(mask=dense), dict(kind=lib.MASK_KEY_LENGTHS, lens=lens)]
    if Lq == Lk:
        cases += [dict(kind=lib.MASK_CAUSAL), dict(kind=lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens=lens), dict(kind=lib.MASK_CAUSAL, strict=True)]
    for kw in cases:
        a = run_sdpa(ctx, q, k, v, **kw)
        b = run_sdpa(ctx, q, k, v, token_major=True, **kw)
        assert np.array_equal(a, b), kw.keys()


@pytest.mark.parametrize("d", [96, 70])
@pytest.mark.parametrize("B,H,Lq,Lk", [(64, 16, 130, 5), (32, 16, 129, 33), (128, 8, 1, 64), (64, 8, 128, 31)])
@pytest.mark.parametrize("mk", ["none", "causal_lens"])
def test_96_wide_kernel_on_short_and_ragged_extents(ctx, orc, B, H, Lq, Lk, d, mk):
    """Many (batch, head) pairs with few queries and keys: single tiles, a single query row, extents one past or one short
    of a tile edge, with 128-bit (d = 96) and 64-bit (d = 70) staging."""
    from dl4s_amd import lib
    rng = np.random.default_rng(zlib.crc32(repr(("w96 short", B, H, Lq, Lk, d, mk)).encode()))
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(0, Lk + 1, size=B)
    lens[0] = max(1, Lk // 2)
    kind, mask, lens_arg = None, None, None
    if mk == "causal_lens":
        kind, lens_arg = lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens
        mask = np.maximum(lengths_mask(lens, Lk), causal_mask(Lq, Lk)[None, None])
    got = run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg)
    for b in (0, 1, B - 1):
        mb = None if mask is None else mask[b:b + 1]
        assert_parity(got[b:b + 1], orc.sdpa(q[b:b + 1], k[b:b + 1], v[b:b + 1], mb), "96-wide short d=%d b=%d" % (d, b))
    if mask is not None:
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, strict=True), run_sdpa(ctx, q, k, v, mask, strict=True))


@pytest.mark.parametrize("d", [96, 80, 68, 70, 66, 94, 48, 40, 36, 44])
@pytest.mark.parametrize("mk", ["none", "dense", "causal", "lens", "causal_lens"])
def test_head_dims_up_to_96_on_launches_that_fill_the_gpu(ctx, orc, d, mk):
    """Head dims above 64 up to 96 with at least two 128-query blocks per CU run the 96-wide kernel (its 80-column form up
    to 80): multiples of 4 with 128-bit staging, other even head dims as they are with 64-bit staging (no padded copies).
    Head dims 36 .. 48 run the 48-column form of the narrow kernel.  B16 H16, ragged extents, checked against the oracle on
    whole (batch, head) slices."""
    from dl4s_amd import lib
    B, H, Lq, Lk = 16, 16, 300, 300
    rng = np.random.default_rng(zlib.crc32(repr(("w96", d, mk)).encode()))
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(0, Lk + 1, size=B)
    lens[0], lens[1] = Lk // 2, 0        # batch item 1: no valid key, uniform rows
    kind, mask, lens_arg = None, None, None
    if mk == "dense":
        mask = (rng.random((B, 1, Lq, Lk)) < 0.4).astype(np.float32)
        mask[:, :, 64:160, 96:224] = 1.0          # whole tiles of ones and of zeros
        mask[:, :, 160:224, 0:96] = 0.0
    elif mk == "causal":
        kind, mask = lib.MASK_CAUSAL, causal_mask(Lq, Lk)
    elif mk == "lens":
        kind, mask, lens_arg = lib.MASK_KEY_LENGTHS, lengths_mask(lens, Lk), lens
    elif mk == "causal_lens":
        kind, lens_arg = lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens
        mask = np.maximum(lengths_mask(lens, Lk), causal_mask(Lq, Lk)[None, None])
    got = run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg)
    for (b, h) in [(0, 0), (1, 5), (15, 15)]:
        mb = None if mask is None else (mask if mask.ndim == 2 else mask[b:b + 1])
        ref = orc.sdpa(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], mb)
        assert_parity(got[b:b + 1, h:h + 1], ref, "96-wide d=%d %s (b=%d,h=%d)" % (d, mk, b, h))
    if kind is not None:    # descriptor == the dense mask it stands for, bit for bit, when both visit every tile
        dense = run_sdpa(ctx, q, k, v, mask, strict=True)
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, strict=True), dense)
        assert_parity(got, dense, "skip vs dense")
    if mask is not None:
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask), run_sdpa(ctx, q, k, v, mask, strict=True))
    if d % 4 == 0:
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, token_major=True), got)


@pytest.mark.parametrize("d", [192, 256, 132, 160, 200, 252])
@pytest.mark.parametrize("mk", ["none", "dense", "causal", "lens", "causal_lens"])
def test_head_dims_above_128_on_the_wide_kernels(ctx, orc, d, mk):
    """Head dims above 128 up to 256 (multiples of 4) run the 192- and 256-wide MFMA kernels in the forward call: ragged
    extents, every mask kind, checked against the oracle on whole (batch, head) slices; descriptors against the dense masks
    they stand for; the token-major layout bit for bit."""
    from dl4s_amd import lib
    B, H, Lq, Lk = 3, 4, 300, 333
    if mk in ("causal", "causal_lens"):
        Lk = Lq
    rng = np.random.default_rng(zlib.crc32(repr(("wide", d, mk)).encode()))
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(0, Lk + 1, size=B)
    lens[0], lens[1] = Lk // 2, 0        # batch item 1: no valid key, uniform rows
    kind, mask, lens_arg = None, None, None
    if mk == "dense":
        mask = (rng.random((B, 1, Lq, Lk)) < 0.4).astype(np.float32)
        mask[:, :, 64:160, 96:224] = 1.0          # whole tiles of ones and of zeros
        mask[:, :, 160:224, 0:96] = 0.0
    elif mk == "causal":
        kind, mask = lib.MASK_CAUSAL, causal_mask(Lq, Lk)
    elif mk == "lens":
        kind, mask, lens_arg = lib.MASK_KEY_LENGTHS, lengths_mask(lens, Lk), lens
    elif mk == "causal_lens":
        kind, lens_arg = lib.MASK_CAUSAL_OR_KEY_LENGTHS, lens
        mask = np.maximum(lengths_mask(lens, Lk), causal_mask(Lq, Lk)[None, None])
    got = run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg)
    for (b, h) in [(0, 0), (1, 2), (2, 3)]:
        mb = None if mask is None else (mask if mask.ndim == 2 else mask[b:b + 1])
        ref = orc.sdpa(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], mb)
        assert_parity(got[b:b + 1, h:h + 1], ref, "wide d=%d %s (b=%d,h=%d)" % (d, mk, b, h))
    if kind is not None:    # descriptor == the dense mask it stands for, bit for bit, when both visit every tile
        dense = run_sdpa(ctx, q, k, v, mask, strict=True)
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, strict=True), dense)
        assert_parity(got, dense, "skip vs dense")
    if mask is not None:
        assert np.array_equal(run_sdpa(ctx, q, k, v, mask), run_sdpa(ctx, q, k, v, mask, strict=True))
    assert np.array_equal(run_sdpa(ctx, q, k, v, mask, kind=kind, lens=lens_arg, token_major=True), got)


@pytest.mark.parametrize("d", [192, 256, 140])
@pytest.mark.parametrize("B,H,Lq,Lk", [(2, 3, 130, 5), (1, 2, 129, 33), (4, 2, 1, 64), (2, 2, 128, 31), (1, 1, 1, 1), (1, 1, 700, 900)])
def test_wide_kernels_on_short_and_ragged_extents(ctx, orc, B, H, Lq, Lk, d):
    rng = np.random.default_rng(zlib.crc32(repr(("wide short", B, H, Lq, Lk, d)).encode()))
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    lens = rng.integers(0, Lk + 1, size=B)
    lens[0] = max(1, Lk // 2)
    from dl4s_amd import lib
    assert_parity(run_sdpa(ctx, q, k, v), orc.sdpa(q, k, v, None), "wide short d=%d" % d)
    mask = lengths_mask(lens, Lk)
    assert_parity(run_sdpa(ctx, q, k, v, mask, kind=lib.MASK_KEY_LENGTHS, lens=lens), orc.sdpa(q, k, v, mask), "wide short lens d=%d" % d)
    # non-finite values: a NaN key row, an Inf value
    k2, v2 = k.copy(), v.copy()
    k2[0, 0, Lk // 2] = np.nan
    v2[-1, -1, 0, d - 1] = np.inf
    with np.errstate(all="ignore"):
        ref = orc.sdpa(q, k2, v2, None)
    assert_parity(run_sdpa(ctx, q, k2, v2), ref, "wide short non-finite d=%d" % d)


@pytest.mark.parametrize("dk,dv", [(200, 130), (130, 256), (150, 150), (255, 255), (64, 192)])
@pytest.mark.parametrize("mk", ["none", "causal"])
def test_head_dims_up_to_256_served_by_padded_copies(ctx, orc, dk, dv, mk):
    """Unequal or odd head dims above 128: the forward call runs the wide kernels on zero-padded copies."""
    from dl4s_amd import lib
    B, H, Lq, Lk = 2, 3, 260, 260
    rng = np.random.default_rng(zlib.crc32(repr(("wide padded", dk, dv, mk)).encode()))
    q, k, v = rand(rng, B, H, Lq, dk), rand(rng, B, H, Lk, dk), rand(rng, B, H, Lk, dv)
    kind, mask = (lib.MASK_CAUSAL, causal_mask(Lq, Lk)) if mk == "causal" else (None, None)
    got = run_sdpa(ctx, q, k, v, mask, kind=kind)
    assert_parity(got[1:2, 2:3], orc.sdpa(q[1:2, 2:3], k[1:2, 2:3], v[1:2, 2:3], mask), "padded wide dk=%d dv=%d" % (dk, dv))
    assert_parity(got[0:1, 0:1], orc.sdpa(q[0:1, 0:1], k[0:1, 0:1], v[0:1, 0:1], mask), "padded wide dk=%d dv=%d" % (dk, dv))


def test_token_major_rejected_for_other_head_dims_and_unknown_flags(ctx):
    from dl4s_amd import lib
    q = ctx.empty((1, 2, 4, 260))
    for d in (6, 130, 202, 260):     # not a multiple of 4 up to 256
        with pytest.raises(lib.Dl4sHipError):
            ctx.sdpa_fwd(q, q, q, q, 1, 2, 4, 4, d, d, 0.5, None, lib.SDPA_TOKEN_MAJOR)
    with pytest.raises(lib.Dl4sHipError):       # different key and value dims
        ctx.sdpa_fwd(q, q, q, q, 1, 2, 4, 4, 8, 16, 0.5, None, lib.SDPA_TOKEN_MAJOR)
    with pytest.raises(lib.Dl4sHipError):
        ctx.sdpa_fwd(q, q, q, q, 1, 2, 4, 4, 8, 8, 0.5, None, 64)
    q.release()


@pytest.mark.parametrize("mshape", ["full", "b1qk", "qk", "b11k", "k", "bh1k", "1hq1"])
def test_dense_mask_with_uniform_and_mixed_tiles(ctx, orc, mshape):
    """Dense masks whose 32 x 32 tiles are all zeros, all ones or mixed (the kernel reads mask values only in mixed
    tiles), on every broadcast shape the reference accepts."""
    B, H, Lq, Lk = 2, 3, 150, 200
    rng = np.random.default_rng(len(mshape) * 17 + 3)
    q, k, v = rand(rng, B, H, Lq, 64), rand(rng, B, H, Lk, 64), rand(rng, B, H, Lk, 64)
    shape = {"full": (B, H, Lq, Lk), "b1qk": (B, 1, Lq, Lk), "qk": (Lq, Lk), "b11k": (B, 1, 1, Lk), "k": (Lk,),
             "bh1k": (B, H, 1, Lk), "1hq1": (1, H, Lq, 1)}[mshape]
    full = np.broadcast_to(np.zeros(shape, np.float32), shape).copy()
    # block structure: tiles of 32 set to 0, 1, random 0/1, or a non-binary value
    m4 = full.reshape((1,) * (4 - full.ndim) + full.shape)
    for qi in range(0, m4.shape[2], 32):
        for ki in range(0, m4.shape[3], 32):
            for bb in range(m4.shape[0]):
                for hh in range(m4.shape[1]):
                    c = rng.integers(0, 4)
                    blk = m4[bb, hh, qi:qi + 32, ki:ki + 32]
                    if c == 1:
                        blk[...] = 1.0
                    elif c == 2:
                        blk[...] = (rng.random(blk.shape) < 0.5)
                    elif c == 3:
                        blk[...] = 0.5
    got = run_sdpa(ctx, q, k, v, full)
    ref = orc.sdpa(q, k, v, full, np.float32(8.0))
    assert_parity(got, ref, "dense mask tiles " + mshape)
    got_tm = run_sdpa(ctx, q, k, v, full, token_major=True)
    assert np.array_equal(got, got_tm)


@pytest.mark.parametrize("mshape", ["full", "b1qk", "qk", "b11k", "k", "1hq1"])
@pytest.mark.parametrize("d", [64, 32, 96, 128, 192])
def test_prepared_mask_classes_give_the_bits_of_the_call_that_classifies(ctx, mshape, d):
    """dl4s_hip_mask_classify_f32 once, then attention calls that take the classes from the descriptor: the same bits as
    calls that classify the mask themselves, with and without tile skipping, on every broadcast shape; after the mask
    changes, classifying again follows it."""
    from dl4s_amd import lib
    B, H, Lq, Lk = 2, 3, 150, 200
    rng = np.random.default_rng(zlib.crc32(repr(("classes", mshape, d)).encode()))
    q, k, v = rand(rng, B, H, Lq, d), rand(rng, B, H, Lk, d), rand(rng, B, H, Lk, d)
    shape = {"full": (B, H, Lq, Lk), "b1qk": (B, 1, Lq, Lk), "qk": (Lq, Lk), "b11k": (B, 1, 1, Lk), "k": (Lk,), "1hq1": (1, H, Lq, 1)}[mshape]

    def make_mask():
        m = np.zeros(shape, np.float32)
        m4 = m.reshape((1,) * (4 - m.ndim) + m.shape)
        for qi in range(0, m4.shape[2], 32):
            for ki in range(0, m4.shape[3], 32):
                c = rng.integers(0, 4)
                blk = m4[:, :, qi:qi + 32, ki:ki + 32]
                blk[...] = {0: 0.0, 1: 1.0, 3: 0.5}.get(int(c), 0.0)
                if c == 2:
                    blk[...] = rng.random(blk.shape) < 0.5
        return m

    bufs = [ctx.to_device(x) for x in (q, k, v)]
    out = ctx.empty((B, H, Lq, d))
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
    md = ctx.to_device(make_mask())
    for round_ in range(2):
        plain = ctx.mask_desc(lib.MASK_DENSE, dense=md)
        prepared = ctx.mask_desc(lib.MASK_DENSE, dense=md)
        classes = ctx.mask_classify(prepared, B, H, Lq, Lk)
        assert prepared.classes
        for flags in (0, lib.SDPA_STRICT):
            ctx.sdpa_fwd(bufs[0], bufs[1], bufs[2], out, B, H, Lq, Lk, d, d, rT, plain, flags)
            want = out.numpy()
            for _ in range(2):      # the classes serve any number of calls
                ctx.sdpa_fwd(bufs[0], bufs[1], bufs[2], out, B, H, Lq, Lk, d, d, rT, prepared, flags)
                assert np.array_equal(out.numpy(), want, equal_nan=True)
        classes.release()
        ctx.assign_h2d(md, make_mask())     # a new mask in the same buffer: its classes are formed again
    # descriptors that have no classes
    import ctypes
    n, causal = ctypes.c_size_t(), ctx.mask_desc(lib.MASK_CAUSAL)
    i64 = ctypes.c_int64
    assert ctx.lib.dl4s_hip_mask_classes_size(ctypes.byref(causal), i64(1), i64(1), i64(8), i64(8), ctypes.byref(n)) != 0
    for b in bufs + [out, md]:
        b.release()


DESCRIBE_CASES = [  # name, B, H, Lq, Lk, expected kind
    ("zeros_b11k", 3, 2, 40, 50, "none"), ("zeros_qk", 2, 3, 70, 90, "dense"),     # a query axis is only looked at under the causal rule
    ("lens_b11k", 4, 2, 130, 200, "lens"), ("lens_k", 2, 2, 33, 64, "lens"), ("lens_with_empty_and_full", 3, 2, 65, 65, "lens"),
    ("causal_qk", 2, 3, 150, 150, "causal"), ("causal_wide", 1, 2, 100, 260, "causal"), ("causal_tall", 1, 2, 260, 100, "causal"),
    ("causal_11qk", 2, 2, 64, 64, "causal"),
    ("decoder_b1qk", 4, 2, 130, 130, "causal_lens"), ("decoder_with_empty_sequence", 3, 2, 96, 96, "causal_lens"),
    ("random", 2, 2, 70, 90, "dense"), ("half_causal", 1, 2, 64, 64, "dense"), ("lens_not_monotone", 2, 2, 40, 50, "dense"),
    ("head_axis", 2, 3, 40, 50, "dense"), ("causal_shifted", 1, 2, 64, 64, "dense"), ("q_axis_only", 1, 2, 64, 64, "dense"),
]


@pytest.mark.parametrize("case", DESCRIBE_CASES, ids=[c[0] for c in DESCRIBE_CASES])
def test_dense_masks_described_as_structured_kinds(ctx, case):
    """dl4s_hip_mask_describe_f32 finds the structured kind whose values a dense mask holds exactly (the masks of
    makeEncoderMasks / makeDecoderMasks, TransformerUtil.swift:29-50) and leaves every other mask dense; the attention call
    gives the same bits under the descriptor it returns as under the mask tensor, with and without tile skipping."""
    from dl4s_amd import lib
    name, B, H, Lq, Lk, want = case
    rng = np.random.default_rng(zlib.crc32(repr(case).encode()))
    lens = rng.integers(1, Lk, size=B)
    want_lens = None
    if name.startswith("zeros"):
        mask = np.zeros((Lq, Lk) if name == "zeros_qk" else (B, 1, 1, Lk), np.float32)
    elif name == "lens_b11k":
        mask, want_lens = lengths_mask(lens, Lk), lens
    elif name == "lens_k":
        mask, want_lens = lengths_mask(lens[:1], Lk).reshape(Lk), np.full(B, lens[0])
    elif name == "lens_with_empty_and_full":
        lens = np.array([0, Lk, 7])
        mask, want_lens = lengths_mask(lens, Lk), lens
    elif name in ("causal_qk", "causal_wide", "causal_tall"):
        mask = causal_mask(Lq, Lk)
    elif name == "causal_11qk":
        mask = causal_mask(Lq, Lk).reshape(1, 1, Lq, Lk)
    elif name == "decoder_b1qk":
        lens[0] = Lk                                    # one full sequence: recorded as Lk
        mask, want_lens = np.maximum(causal_mask(Lq, Lk)[None, None], lengths_mask(lens, Lk)), lens
    elif name == "decoder_with_empty_sequence":
        lens = np.array([0, 50, Lk])
        mask, want_lens = np.maximum(causal_mask(Lq, Lk)[None, None], lengths_mask(lens, Lk)), lens
    elif name == "random":
        mask = (rng.random((B, 1, Lq, Lk)) < 0.3).astype(np.float32)
    elif name == "half_causal":
        mask = causal_mask(Lq, Lk) * np.float32(0.5)
    elif name == "lens_not_monotone":
        mask = lengths_mask(lens, Lk)
        mask[1, 0, 0, Lk - 1] = 0.0
    elif name == "head_axis":
        mask = np.broadcast_to(lengths_mask(lens, Lk), (B, H, 1, Lk)).copy()
    elif name == "causal_shifted":
        mask = np.triu(np.ones((Lq, Lk), np.float32), k=2)
    else:
        mask = np.zeros((Lq, 1), np.float32)
    md = ctx.to_device(mask)
    dense = ctx.mask_desc(lib.MASK_DENSE, dense=md)
    desc, lbuf = ctx.mask_describe(dense, B, H, Lq, Lk)
    kinds = {"none": lib.MASK_NONE, "lens": lib.MASK_KEY_LENGTHS, "causal": lib.MASK_CAUSAL, "causal_lens": lib.MASK_CAUSAL_OR_KEY_LENGTHS,
             "dense": lib.MASK_DENSE}
    assert desc.kind == kinds[want], (desc.kind, want)
    if want in ("lens", "causal_lens"):
        assert desc.lengths == lbuf.ptr
        assert np.array_equal(lbuf.numpy(), np.asarray(want_lens, np.int32))
    if want == "dense":
        assert desc.dense == md.ptr and tuple(desc.shape) == tuple(dense.shape)
    q, k, v = rand(rng, B, H, Lq, 64), rand(rng, B, H, Lk, 64), rand(rng, B, H, Lk, 64)
    bufs = [ctx.to_device(x) for x in (q, k, v)]
    out = ctx.empty((B, H, Lq, 64))
    for flags in (0, lib.SDPA_STRICT):
        ctx.sdpa_fwd(bufs[0], bufs[1], bufs[2], out, B, H, Lq, Lk, 64, 64, 0.125, dense, flags)
        ref = out.numpy()
        ctx.sdpa_fwd(bufs[0], bufs[1], bufs[2], out, B, H, Lq, Lk, 64, 64, 0.125, None if desc.kind == lib.MASK_NONE else desc, flags)
        assert np.array_equal(out.numpy(), ref, equal_nan=True)
    for b in bufs + [out, md, lbuf]:
        b.release()


def test_tensors_beyond_2_31_elements(ctx, orc):
    """32768 (batch, head) pairs of 1024 x 64: every tensor holds 2^31 elements (8 GiB), so any 32-bit element index in
    the kernels or their launch arithmetic would wrap.  The tensors are filled on the device from one 64-pair block
    (with the last pair made distinct); the first, a middle and the last pair are checked against the oracle, and the
    output of every block of 64 pairs but the last must repeat the first block bit for bit."""
    import ctypes as C
    from dl4s_amd import lib
    if NO_SPLIT_DEFAULT[0]:
        pytest.skip("one run is enough: the launch is far beyond the key-split range")
    B, H, L, d = 2048, 16, 1024, 64
    blk = 64                                     # pairs per host block
    rng = np.random.default_rng(99)
    hq, hk, hv = (rand(rng, blk, L, d) for _ in range(3))
    last = [rand(rng, 1, L, d) for _ in range(3)]
    nbytes_pair = L * d * 4
    bufs = [lib.DeviceBuffer(ctx, B * H * nbytes_pair, (B, H, L, d)) for _ in range(4)]
    for buf, host, tail in zip(bufs, (hq, hk, hv), last):
        for i in range(B * H // blk):
            lib._check(ctx.lib.dl4s_hip_assign_h2d(ctx.handle, C.c_void_p(buf.offset(i * blk * nbytes_pair)),
                                                   host.ctypes.data_as(C.c_void_p), C.c_size_t(host.nbytes)))
        lib._check(ctx.lib.dl4s_hip_assign_h2d(ctx.handle, C.c_void_p(buf.offset((B * H - 1) * nbytes_pair)),
                                               tail.ctypes.data_as(C.c_void_p), C.c_size_t(tail.nbytes)))
    ctx.sdpa_fwd(bufs[0], bufs[1], bufs[2], bufs[3], B, H, L, L, d, d, 0.125, ctx.mask_desc(lib.MASK_CAUSAL), 0)

    def pair(i):
        out = np.empty((1, 1, L, d), np.float32)
        lib._check(ctx.lib.dl4s_hip_assign_d2h(ctx.handle, out.ctypes.data_as(C.c_void_p), C.c_void_p(bufs[3].offset(i * nbytes_pair)),
                                               C.c_size_t(out.nbytes)))
        return out
    m = causal_mask(L, L)
    for i, (q_, k_, v_) in ((0, (hq[0], hk[0], hv[0])), (B * H // 2 + 5, (hq[5], hk[5], hv[5])), (B * H - 1, [t[0] for t in last])):
        assert_parity(pair(i), orc.sdpa(q_[None, None], k_[None, None], v_[None, None], m), "pair %d of %d" % (i, B * H))
    first = np.empty((blk, L, d), np.float32)
    other = np.empty_like(first)
    lib._check(ctx.lib.dl4s_hip_assign_d2h(ctx.handle, first.ctypes.data_as(C.c_void_p), C.c_void_p(bufs[3].ptr), C.c_size_t(first.nbytes)))
    for i in (1, 255, B * H // blk - 2):
        lib._check(ctx.lib.dl4s_hip_assign_d2h(ctx.handle, other.ctypes.data_as(C.c_void_p),
                                               C.c_void_p(bufs[3].offset(i * blk * nbytes_pair)), C.c_size_t(other.nbytes)))
        assert np.array_equal(first, other)
    for b in bufs:
        b.release()


def test_concurrent_callers_on_one_context(ctx, orc):
    """Four host threads issue dense-mask attention calls (which stage mask tile classes in the context's scratch block)
    on the same context at once; every result must be its own problem's."""
    import threading
    rng = np.random.default_rng(77)
    problems = []
    for i in range(4):
        Lq, Lk = 96 + 32 * i, 200 - 24 * i
        q, k, v = rand(rng, 1, 2, Lq, 64), rand(rng, 1, 2, Lk, 64), rand(rng, 1, 2, Lk, 64)
        mask = (rng.random((1, 1, Lq, Lk)) < 0.5).astype(np.float32)
        mask[..., : Lk // 2] = float(i % 2)          # uniform tiles of both kinds plus mixed ones
        problems.append((q, k, v, mask, orc.sdpa(q, k, v, mask)))
    results = [[] for _ in problems]

    def work(i):
        q, k, v, mask, _ = problems[i]
        for _ in range(10):
            results[i].append(run_sdpa(ctx, q, k, v, mask))
    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(problems))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for i, (_, _, _, _, ref) in enumerate(problems):
        for got in results[i]:
            assert_parity(got, ref, "thread %d" % i)
            assert np.array_equal(got, results[i][0])


@pytest.mark.parametrize("kind_name", ["lens", "causal_lens"])
def test_sequence_of_length_zero_gives_uniform_rows(ctx, orc, kind_name):
    """A valid length of 0 blocks every key of that batch item: all rows are uniform (the mean of V), exactly as with
    the dense mask; the other batch items are unaffected."""
    from dl4s_amd import lib
    rng = np.random.default_rng(123)
    B, H, L = 3, 2, 160
    q, k, v = rand(rng, B, H, L, 64), rand(rng, B, H, L, 64), rand(rng, B, H, L, 64)
    lens = np.array([0, 97, 160])
    kind = lib.MASK_KEY_LENGTHS if kind_name == "lens" else lib.MASK_CAUSAL_OR_KEY_LENGTHS
    mask = lengths_mask(lens, L)
    if kind_name == "causal_lens":
        mask = np.maximum(mask, causal_mask(L, L)[None, None])
    got = run_sdpa(ctx, q, k, v, kind=kind, lens=lens)
    assert_parity(got, orc.sdpa(q, k, v, mask), kind_name)
    assert np.allclose(got[0], v[0].mean(axis=1, keepdims=True), atol=1e-5)
    assert np.array_equal(got, run_sdpa(ctx, q, k, v, mask))
