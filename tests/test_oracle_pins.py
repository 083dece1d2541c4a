"""Pins the CPU oracle to things it did not compute itself: the reference's own known answers
(Tests/DL4STests/VecTests.swift:86-156), numpy/scipy/torch library routines in fp64, brute force
and invariants.  Each check is chosen so that a dropped term, wrong sign, wrong index or a
transposed operand fails it."""
import numpy as np
import pytest
import scipy.special

from helpers import negative_variance_pairs

RNG = np.random.default_rng(7)


# --------------------------------------------------------------------------- GEMM
def test_gemm_reference_known_answers(orc):
    # Tests/DL4STests/VecTests.swift:86-156
    a = np.array([[1, 2, 3]], np.float32)
    b = np.array([[4], [5], [6]], np.float32)
    assert orc.gemm(a, b)[0, 0] == 32                                   # testMMul1x1
    c = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    assert orc.gemm(c, a.T.copy()).ravel().tolist() == [14, 32]          # testMMul2x1
    d = np.array([[1, 2]], np.float32)
    assert orc.gemm(d, c).ravel().tolist() == [9, 12, 15]                # testMMul1x2
    ct = np.ascontiguousarray(c.T)
    assert orc.gemm(ct, c).tolist() == [[17, 22, 27], [22, 29, 36], [27, 36, 45]]   # testMMul2x2
    assert orc.gemm(c, ct).tolist() == [[14, 32], [32, 77]]              # testMMul2x2_2
    # the same products through the transpose flags (EngineV2Tests.swift:306-325 exercises them)
    assert orc.gemm(c, c, trans_a=True).tolist() == [[17, 22, 27], [22, 29, 36], [27, 36, 45]]
    assert orc.gemm(c, c, trans_b=True).tolist() == [[14, 32], [32, 77]]


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
def test_gemm_integer_exact_all_flags(orc, ta, tb):
    M, N, K = 5, 7, 6
    A = RNG.integers(-9, 10, size=(K, M) if ta else (M, K)).astype(np.float32)
    B = RNG.integers(-9, 10, size=(N, K) if tb else (K, N)).astype(np.float32)
    want = (A.T if ta else A).astype(np.float64) @ (B.T if tb else B).astype(np.float64)
    got = orc.gemm(A, B, ta, tb, alpha=3.0)
    assert np.array_equal(got.astype(np.float64), 3.0 * want)


def test_gemm_fp32_vs_fp64(orc):
    A = RNG.standard_normal((33, 65)).astype(np.float32)
    B = RNG.standard_normal((65, 17)).astype(np.float32)
    want = A.astype(np.float64) @ B.astype(np.float64)
    assert np.allclose(orc.gemm(A, B), want, rtol=0, atol=2e-5)


def test_gemm_beta_is_overwritten_like_generic_path(orc):
    # CPUGeneric.swift:201-253: C is pre-scaled by beta and then assigned alpha*tmp.
    A = np.eye(2, dtype=np.float32)
    C0 = np.full((2, 2), 5.0, np.float32)
    assert orc.gemm(A, A, beta=1.0, c=C0).tolist() == [[1, 0], [0, 1]]


def test_bmm_is_stack_of_slices_and_broadcasts(orc):
    # identity stated by EngineV2Tests.swift:192-210 and Matrix.swift:106-116
    a = RNG.integers(-4, 5, size=(2, 1, 3, 4)).astype(np.float32)
    b = RNG.integers(-4, 5, size=(1, 3, 4, 5)).astype(np.float32)
    got = orc.bmm(a, b)
    assert got.shape == (2, 3, 3, 5)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    assert np.array_equal(got, want.astype(np.float32))
    bt = np.ascontiguousarray(np.swapaxes(b, -1, -2))
    assert np.array_equal(orc.bmm(a, bt, trans_b=True), got)
    # lower-rank rhs is left-padded with ones
    w = RNG.integers(-4, 5, size=(4, 2)).astype(np.float32)
    assert np.array_equal(orc.bmm(a[:, 0], w), np.matmul(a[:, 0].astype(np.float64), w).astype(np.float32))


# ---------------------------------------------------------------------- broadcast
@pytest.mark.parametrize("op,fn", [("add", np.add), ("sub", np.subtract), ("mul", np.multiply), ("div", np.divide)])
@pytest.mark.parametrize("sa,sb", [((2, 3, 4), (4,)), ((2, 3, 4), (3, 1)), ((2, 3, 4), ()), ((), (2, 3)),
                                   ((2, 1, 4), (1, 3, 1)), ((2, 3, 4, 5), (2, 1, 1, 5)), ((3, 4), (3, 4)),
                                   ((2, 2, 3, 3), (3, 3)), ((4, 1), (1, 5)), ((1,), (6,))])
def test_broadcast_vs_numpy(orc, op, fn, sa, sb):
    a = RNG.integers(1, 9, size=sa).astype(np.float32)
    b = RNG.integers(1, 9, size=sb).astype(np.float32)
    got = orc.broadcast(op, a, b)
    want = fn(a.astype(np.float64), b.astype(np.float64))
    assert got.shape == want.shape
    if op == "div":
        assert np.allclose(got, want, rtol=2e-7, atol=0)     # x*(1/s) may differ from x/s by 1 ulp
    else:
        assert np.array_equal(got.astype(np.float64), want)


def test_broadcast_scalar_forms_round_like_reference(orc):
    # vector / scalar is x * fl(1/s)  (CPUEngine.swift:635); vector - scalar is x + (-s)
    x = RNG.standard_normal(1000).astype(np.float32)
    s = np.float32(3.0)
    got = orc.broadcast("div", x, np.array(s))
    assert np.array_equal(got, x * (np.float32(1.0) / s))
    assert not np.array_equal(got, x / s)                    # and that really is a different rounding
    assert np.array_equal(orc.broadcast("sub", x, np.array(s)), x - s)
    assert np.array_equal(orc.broadcast("sub", np.array(s), x), s - x)
    assert np.array_equal(orc.broadcast("div", np.array(s), x), s / x)


# --------------------------------------------------------------------- reductions
@pytest.mark.parametrize("shape,axes", [((3, 4, 5), [2]), ((3, 4, 5), [1, 2]), ((3, 4, 5), [0]), ((3, 4, 5), [0, 1]),
                                        ((3, 4, 5), [0, 2]), ((6,), [0]), ((2, 3, 4, 5), [3]), ((2, 3, 4, 5), [1, 3]),
                                        ((4, 5), [0, 1])])
def test_reduce_sum_vs_numpy(orc, shape, axes):
    x = RNG.integers(-50, 50, size=shape).astype(np.float32)
    assert np.array_equal(orc.reduce_sum(x, axes).astype(np.float64), x.astype(np.float64).sum(axis=tuple(axes)))
    y = RNG.standard_normal(shape).astype(np.float32)
    assert np.allclose(orc.reduce_sum(y, axes), y.astype(np.float64).sum(axis=tuple(axes)), atol=1e-5)


def test_reduce_sum_is_sequential_left_to_right(orc):
    # 1e8 + 1 + 1 ... : a sequential fp32 sum loses every +1, a pairwise/tree sum would not.
    x = np.ones(4097, np.float32)
    x[0] = 1e8
    assert orc.reduce_sum(x, [0]) == np.float32(1e8)


@pytest.mark.parametrize("shape,axis", [((3, 4, 5), 2), ((3, 4, 5), 1), ((3, 4, 5), 0), ((7,), 0)])
def test_reduce_max_vs_numpy(orc, shape, axis):
    x = RNG.standard_normal(shape).astype(np.float32)
    assert np.array_equal(orc.reduce_max(x, axis), x.max(axis=axis))


def test_reduce_max_skips_nan_and_starts_at_minus_inf(orc):
    # CPUFloat.swift:308-315: maxV = -inf; if v > maxV
    x = np.array([[np.nan, 1.0, -2.0], [np.nan, np.nan, np.nan], [-np.inf, -np.inf, -np.inf]], np.float32)
    got = orc.reduce_max(x, 1)
    assert got[0] == 1.0 and got[1] == -np.inf and got[2] == -np.inf


# ------------------------------------------------------------ permute, band, masks
def test_permute_scatter_convention(orc):
    x = RNG.standard_normal((2, 3, 4, 5)).astype(np.float32)
    for arr in [(0, 2, 1, 3), (1, 2, 3, 0), (3, 0, 1, 2), (0, 1, 2, 3), (2, 0, 3, 1)]:
        got = orc.permute(x, arr)
        inv = np.argsort(arr)                 # source axis i -> destination axis arr[i]
        assert np.array_equal(got, np.transpose(x, inv))
    # for a non-involution the scatter and gather conventions differ: make sure we have the right one
    assert orc.permute(x, (1, 2, 3, 0)).shape == (5, 2, 3, 4)
    y = RNG.standard_normal((3, 5)).astype(np.float32)
    assert np.array_equal(orc.permute(y, (1, 0)), y.T)


def test_band_matches_closed_form(orc):
    x = RNG.standard_normal((6, 8)).astype(np.float32)
    i, j = np.indices(x.shape)
    for below, above in [(-1, None), (0, 0), (None, 0), (1, 2), (None, None), (-3, None), (2, -1)]:
        lo = i - (below if below is not None else 8)
        hi = i + (above if above is not None else 8)
        want = np.where((j >= lo) & (j <= hi), x, 0)
        assert np.array_equal(orc.band(x, below, above), want), (below, above)


def test_mask_builders_brute_force(orc):
    lens = [3, 5, 1, 0, 5]
    enc = orc.make_encoder_masks(lens)
    dec = orc.make_decoder_masks(lens)
    L = max(lens)
    assert enc.shape == (5, 1, 1, L) and dec.shape == (5, 1, L, L)
    for b, n in enumerate(lens):
        for j in range(L):
            assert enc[b, 0, 0, j] == float(j >= n)
            for i in range(L):
                assert dec[b, 0, i, j] == float(j >= n or j > i)


# ------------------------------------------------------------------------ softmax
def test_softmax_vs_scipy_and_invariants(orc):
    x = (RNG.standard_normal((64, 257)) * 4).astype(np.float32)
    got = orc.softmax_last(x)
    want = scipy.special.softmax(x.astype(np.float64), axis=-1)
    assert np.allclose(got, want, rtol=0, atol=1e-6)
    assert np.allclose(got.sum(-1, dtype=np.float64), 1.0, atol=2e-6)
    assert np.allclose(orc.softmax_last(x + np.float32(8.0)), got, atol=1e-6)   # shift invariance
    one = orc.softmax_last(np.array([[3.25]], np.float32))
    assert one[0, 0] == 1.0
    eq = orc.softmax_last(np.full((1, 8), -1e9, np.float32))
    assert np.all(eq == np.float32(0.125))                                       # uniform, not NaN


def test_softmax_nan_inf_table(orc):
    inf, nan = np.inf, np.nan
    rows = np.array([[1.0, nan, 2.0, 0.0],          # NaN score  -> whole row NaN
                     [1.0, inf, 2.0, 0.0],          # +Inf score -> whole row NaN
                     [-inf, -inf, -inf, -inf],      # all -Inf   -> whole row NaN
                     [-inf, 0.0, -inf, 0.0],        # some -Inf  -> weights 0 there
                     [3e38, -3e38, 3e38, 0.0]],     # huge finite -> no overflow
                    np.float32)
    with np.errstate(all="ignore"):
        got = orc.softmax_last(rows)
    assert np.isnan(got[0]).all() and np.isnan(got[1]).all() and np.isnan(got[2]).all()
    assert got[3].tolist() == [0.0, 0.5, 0.0, 0.5]
    assert got[4].tolist() == [0.5, 0.0, 0.5, 0.0]


# --------------------------------------------------------------------------- SDPA
def _torch_sdpa64(q, k, v, mask):
    import torch
    t = lambda a: torch.from_numpy(np.asarray(a, np.float64))
    am = None if mask is None else t(np.broadcast_to(mask, q.shape[:3] + (k.shape[2],)).copy()) * -1e9
    return torch.nn.functional.scaled_dot_product_attention(t(q), t(k), t(v), attn_mask=am).numpy()


@pytest.mark.parametrize("mask_kind", ["none", "causal", "lens", "dense_bh", "half"])
def test_sdpa_vs_torch_fp64(orc, mask_kind):
    B, H, Lq, Lk, d = 2, 3, 9, 11, 8
    q = RNG.standard_normal((B, H, Lq, d)).astype(np.float32)
    k = RNG.standard_normal((B, H, Lk, d)).astype(np.float32)
    v = RNG.standard_normal((B, H, Lk, d)).astype(np.float32)
    i, j = np.indices((Lq, Lk))
    mask = {"none": None,
            "causal": (j > i).astype(np.float32),
            "lens": (np.arange(Lk)[None, None, None, :] >= np.array([4, 11])[:, None, None, None]).astype(np.float32),
            "dense_bh": (RNG.random((B, H, Lq, Lk)) < 0.3).astype(np.float32),
            "half": np.full((Lq, Lk), 0.5, np.float32) * (j > i)}[mask_kind]
    got = orc.sdpa(q, k, v, mask)
    want = _torch_sdpa64(q, k, v, mask)
    assert np.allclose(got, want, rtol=1e-5, atol=2e-6)


def test_sdpa_scale_is_applied_through_temperature(orc):
    q = RNG.standard_normal((1, 1, 4, 16)).astype(np.float32)
    k = RNG.standard_normal((1, 1, 6, 16)).astype(np.float32)
    v = RNG.standard_normal((1, 1, 6, 16)).astype(np.float32)
    a = orc.sdpa(q, k, v, None, temperature=2.0)
    b = orc.sdpa(q * np.float32(2.0), k, v, None, temperature=4.0)   # exact power-of-two rescale
    assert np.array_equal(a, b)
    assert not np.allclose(a, orc.sdpa(q, k, v, None, temperature=4.0), atol=1e-3)


def test_sdpa_mask_invariants(orc):
    B, H, Lq, Lk, d = 1, 2, 6, 10, 4
    q = RNG.standard_normal((B, H, Lq, d)).astype(np.float32)
    k = RNG.standard_normal((B, H, Lk, d)).astype(np.float32)
    v = RNG.standard_normal((B, H, Lk, d)).astype(np.float32)
    mask = np.zeros((Lq, Lk), np.float32)
    mask[:, 7:] = 1
    mask[2, :] = 1                                      # row 2 fully blocked
    base = orc.sdpa(q, k, v, mask)
    # blocked columns get weight exactly 0: finite changes to K/V there do not change a single bit
    k2, v2 = k.copy(), v.copy()
    k2[:, :, 7:] = 5.0
    v2[:, :, 7:] = -123.0
    other = orc.sdpa(q, k2, v2, mask)
    rows = [0, 1, 3, 4, 5]
    assert np.array_equal(base[:, :, rows], other[:, :, rows])
    # a fully blocked row is the plain mean of V (all scores collapse to -1e9 in fp32)
    assert np.allclose(base[:, :, 2], v.mean(axis=2), atol=1e-6)
    # mask == nil is bit-identical to an all-zero mask
    assert np.array_equal(orc.sdpa(q, k, v, None), orc.sdpa(q, k, v, np.zeros((Lq, Lk), np.float32)))
    # 0 * NaN = NaN: a NaN in V at a blocked key still poisons that value column for every query
    v3 = v.copy()
    v3[0, 0, 9, 1] = np.nan
    with np.errstate(all="ignore"):
        pois = orc.sdpa(q, k, v3, mask)
    assert np.isnan(pois[0, 0, :, 1]).all() and not np.isnan(pois[0, 0, :, 0]).any() and not np.isnan(pois[0, 1]).any()


def test_sdpa_decode_is_sdpa_on_cache_prefix(orc):
    B, H, T, Tcap, d = 2, 2, 9, 12, 8
    q = RNG.standard_normal((B, H, 1, d)).astype(np.float32)
    kc = RNG.standard_normal((B, H, Tcap, d)).astype(np.float32)
    vc = RNG.standard_normal((B, H, Tcap, d)).astype(np.float32)
    got = orc.sdpa_decode(q, kc, vc, T)
    assert np.array_equal(got, orc.sdpa(q, kc[:, :, :T], vc[:, :, :T]))
    assert np.allclose(got, _torch_sdpa64(q, kc[:, :, :T], vc[:, :, :T], None), atol=2e-6)


# ---------------------------------------------------------------- LayerNorm, GELU
def test_layernorm_vs_torch_and_closed_form(orc):
    import torch
    x = (RNG.standard_normal((3, 7, 16)) * 2 + 0.5).astype(np.float32)
    scale = RNG.standard_normal(16).astype(np.float32)
    shift = RNG.standard_normal(16).astype(np.float32)
    got = orc.layernorm(x, scale, shift)                       # joint over (7, 16)
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=(1, 2), keepdims=True)
    std = np.sqrt((x64 * x64).mean(axis=(1, 2), keepdims=True) - mean * mean)
    want = (x64 - mean) / (std + 1e-5) * scale + shift         # eps outside the sqrt
    assert np.allclose(got, want, rtol=1e-5, atol=1e-5)
    # library routine: layer_norm over the last two dims without affine, eps inside the sqrt; the two
    # placements differ by a relative O(1e-5), so the tolerance is 1e-4 on the un-affined result
    ones, zeros = np.ones(16, np.float32), np.zeros(16, np.float32)
    lib = torch.nn.functional.layer_norm(torch.from_numpy(x64), (7, 16), eps=0.0).numpy()
    assert np.allclose(orc.layernorm(x, ones, zeros), lib, rtol=1e-4, atol=1e-4)
    # per-token when the input is 2-D
    x2 = x.reshape(21, 16)
    lib2 = torch.nn.functional.layer_norm(torch.from_numpy(x2.astype(np.float64)), (16,), eps=0.0).numpy()
    assert np.allclose(orc.layernorm(x2, ones, zeros), lib2, rtol=1e-4, atol=1e-4)


def test_layernorm_eps_sits_outside_the_root(orc):
    """NN/Layer/LayerNorm.swift:75: (x - mean) / (sqrt(var) + eps).  On an input of standard deviation 1e-3 the two
    placements of eps differ by a factor of about three, so the wrong one cannot pass."""
    x = (RNG.standard_normal((3, 5, 64)) * 1e-3).astype(np.float32)
    ones, zeros = np.ones(64, np.float32), np.zeros(64, np.float32)
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=(1, 2), keepdims=True)
    var = (x64 * x64).mean(axis=(1, 2), keepdims=True) - mean * mean
    outside = (x64 - mean) / (np.sqrt(var) + 1e-5)
    inside = (x64 - mean) / np.sqrt(var + 1e-5)
    got = orc.layernorm(x, ones, zeros)
    assert np.allclose(got, outside, rtol=2e-4, atol=1e-6)
    assert np.abs(outside).max() > 2.5 * np.abs(inside).max()          # what the wrong placement would give
    # per token (2-D input), same rule
    x2 = x.reshape(15, 64)
    x264 = x2.astype(np.float64)
    m2 = x264.mean(axis=1, keepdims=True)
    v2 = (x264 * x264).mean(axis=1, keepdims=True) - m2 * m2
    assert np.allclose(orc.layernorm(x2, ones, zeros), (x264 - m2) / (np.sqrt(v2) + 1e-5), rtol=2e-4, atol=1e-6)


def test_layernorm_variance_is_the_biased_one(orc):
    """Tensor/Operators/Reduce.swift:106-110 divides by N, not N - 1: on four elements the two differ by 15 %."""
    x = np.array([[1.0, 2.0, 4.0, 9.0]], np.float32)
    got = orc.layernorm(x, np.ones(4, np.float32), np.zeros(4, np.float32))
    x64 = x.astype(np.float64)
    want = (x64 - x64.mean()) / (x64.std(ddof=0) + 1e-5)
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)
    assert np.abs(got - (x64 - x64.mean()) / (x64.std(ddof=1) + 1e-5)).max() > 0.1


def test_layernorm_variance_is_one_pass_and_can_go_negative(orc):
    """Reduce.swift:106-110: var = E[x^2] - E[x]^2, evaluated in fp32.  A variance formed from squared deviations is
    never negative; the one-pass form is, for some rows, and then sqrt gives NaN and the whole row is NaN.  Two-element
    rows fix the fp32 value whatever the summation order."""
    rows = negative_variance_pairs()
    ones, zeros = np.ones(2, np.float32), np.zeros(2, np.float32)
    with np.errstate(invalid="ignore"):
        got = orc.layernorm(rows, ones, zeros)                       # 2-D input: one row per token
    assert np.isnan(got).all()
    ok = np.array([[1.5, 2.5], [-3.0, 3.0]], np.float32)            # exact in fp32: var = 0.25 and 9
    want = np.array([[-1.0, 1.0], [-1.0, 1.0]]) / (1 + 1e-5 / np.array([[0.5], [3.0]]))
    assert np.allclose(orc.layernorm(ok, ones, zeros), want, rtol=1e-6)


def test_layernorm_far_from_zero_mean_depends_on_the_summation_order(orc):
    """With |mean| = 1000 standard deviations, E[x^2] and E[x]^2 agree to six digits and fp32 keeps seven: what is left
    of the variance is rounding noise of the sums.  The oracle (sequential sums, Engine/CPU/CPUEngine.swift:306-378,
    CPUFloat.swift:239-261) is therefore far from the exact result there, and the same formula with pairwise sums is far
    from both - no order-independent value exists to hold a GPU kernel to.  At |mean| <= 3 standard deviations the two
    orders agree well inside the parity gate."""
    f = np.float32
    ones, zeros = np.ones(1024, f), np.zeros(1024, f)

    def pairwise(x):
        s, ss = np.sum(x, axis=1, dtype=f), np.sum(x * x, axis=1, dtype=f)
        mean = s * f(1 / 1024)
        var = ss * f(1 / 1024) - mean * mean
        with np.errstate(invalid="ignore"):
            return (x + (-mean[:, None])) * (f(1) / (np.sqrt(var) + f(1e-5)))[:, None]

    def exact(x):
        x64 = x.astype(np.float64)
        return (x64 - x64.mean(axis=1, keepdims=True)) / (x64.std(axis=1, keepdims=True) + 1e-5)

    far = (RNG.standard_normal((16, 1024)) + 1000).astype(f)
    with np.errstate(invalid="ignore"):
        got = orc.layernorm(far, ones, zeros)
    assert np.nanmax(np.abs(got - exact(far))) > 0.1                    # a two-pass variance would be exact to 1e-6
    assert np.nanmax(np.abs(got - pairwise(far))) > 0.1
    near = (RNG.standard_normal((16, 1024)) + 3).astype(f)
    got = orc.layernorm(near, ones, zeros)
    assert np.abs(got - exact(near)).max() < 5e-5 and np.abs(got - pairwise(near)).max() < 5e-5


def test_gelu_is_sigmoid_approximation(orc):
    x = np.linspace(-8, 8, 1001).astype(np.float32)
    want = x.astype(np.float64) * scipy.special.expit(1.702 * x.astype(np.float64))
    assert np.allclose(orc.gelu(x), want, rtol=0, atol=2e-6)
    erf_gelu = x * 0.5 * (1 + scipy.special.erf(x / np.sqrt(2)))
    assert np.abs(orc.gelu(x) - erf_gelu).max() > 1e-3          # it is NOT the erf form


def test_unary_vs_numpy(orc):
    x = RNG.standard_normal(513).astype(np.float32) * 3
    assert np.allclose(orc.exp(x), np.exp(x.astype(np.float64)), rtol=2e-7)
    assert np.allclose(orc.tanh(x), np.tanh(x.astype(np.float64)), rtol=3e-7, atol=1e-7)
    assert np.array_equal(orc.sqrt(np.abs(x)), np.sqrt(np.abs(x)))
    assert np.array_equal(orc.relu(x), np.maximum(x, 0))


# ------------------------------------------------------------------- MHA and blocks
def _params(D, H, dk, dv, F, rng):
    xav = lambda fi, fo: rng.uniform(-np.sqrt(6 / (fi + fo)), np.sqrt(6 / (fi + fo)), (fi, fo)).astype(np.float32)
    mha = dict(Wq=xav(D, H * dk), Wk=xav(D, H * dk), Wv=xav(D, H * dv), Wo=xav(H * dv, D),
               ln_scale=(1 + 0.1 * rng.standard_normal(D)).astype(np.float32),
               ln_shift=(0.1 * rng.standard_normal(D)).astype(np.float32))
    ffn = dict(W1=xav(D, F), b1=(0.1 * rng.standard_normal(F)).astype(np.float32), W2=xav(F, D),
               b2=(0.1 * rng.standard_normal(D)).astype(np.float32),
               ln_scale=(1 + 0.1 * rng.standard_normal(D)).astype(np.float32),
               ln_shift=(0.1 * rng.standard_normal(D)).astype(np.float32))
    return mha, ffn


def test_mha_core_vs_torch_multi_head_attention_forward(orc):
    import torch
    B, L, D, H, dk = 2, 7, 16, 4, 4          # the hyper-parameters of TransformerTests.swift:31 (hidden 16, heads 4)
    rng = np.random.default_rng(11)
    mha, _ = _params(D, H, dk, dk, 32, rng)
    x = rng.standard_normal((B, L, D)).astype(np.float32)
    i, j = np.indices((L, L))
    causal = (j > i).astype(np.float32)
    _, attn = orc.mha(x, x, x, causal, mha, H, dk, dk, return_attn=True)
    t = lambda a: torch.from_numpy(np.asarray(a, np.float64))
    xt = t(x).transpose(0, 1)               # torch wants [L, B, D]
    out, _ = torch.nn.functional.multi_head_attention_forward(
        xt, xt, xt, D, H, None, None, None, None, False, 0.0, torch.eye(D, dtype=torch.float64), None,
        training=False, need_weights=False, attn_mask=t(causal) * -1e9, use_separate_proj_weight=True,
        q_proj_weight=t(mha["Wq"]).T, k_proj_weight=t(mha["Wk"]).T, v_proj_weight=t(mha["Wv"]).T)
    want = out.transpose(0, 1).numpy().reshape(B, L, H, dk).transpose(0, 2, 1, 3)   # merged heads -> [B,H,L,dk]
    assert np.allclose(attn, want, rtol=1e-5, atol=5e-6)


from oracle.fp64_model import ffn64 as _ffn64, mha64 as _mha64  # noqa: E402


def test_mha_ffn_blocks_vs_independent_fp64_model(orc):
    B, L, Le, D, H, dk, F = 2, 6, 5, 16, 4, 4, 32
    rng = np.random.default_rng(12)
    mha, ffn = _params(D, H, dk, dk, F, rng)
    mha2, _ = _params(D, H, dk, dk, F, rng)
    x = rng.standard_normal((B, L, D)).astype(np.float32)
    enc = rng.standard_normal((B, Le, D)).astype(np.float32)
    enc_mask = orc.make_encoder_masks([3, 5])
    dec_mask = orc.make_decoder_masks([6, 4])
    tol = dict(rtol=1e-4, atol=1e-5)
    assert np.allclose(orc.mha(x, enc, enc, enc_mask, mha, H, dk, dk), _mha64(x, enc, enc, enc_mask, mha, H, dk, dk), **tol)
    assert np.allclose(orc.ffn(x, ffn), _ffn64(x, ffn), **tol)
    pad = orc.make_encoder_masks([6, 2])
    assert np.allclose(orc.encoder_block(x, pad, mha, ffn, H, dk, dk),
                       _ffn64(_mha64(x, x, x, pad, mha, H, dk, dk), ffn), **tol)
    want = _ffn64(_mha64(_mha64(x, x, x, dec_mask, mha, H, dk, dk), enc, enc, enc_mask, mha2, H, dk, dk), ffn)
    assert np.allclose(orc.decoder_block(x, enc, dec_mask, enc_mask, mha, mha2, ffn, H, dk, dk), want, **tol)


def test_mha_residual_is_the_unprojected_query(orc):
    # MultiHeadAttention.swift:106,123: with Wo = 0 the layer is LayerNorm(q) over (L, D) jointly
    B, L, D, H, dk = 1, 5, 8, 2, 4
    rng = np.random.default_rng(13)
    mha, _ = _params(D, H, dk, dk, 8, rng)
    mha["Wo"] = np.zeros_like(mha["Wo"])
    q = rng.standard_normal((B, L, D)).astype(np.float32)
    kv = rng.standard_normal((B, 3, D)).astype(np.float32)
    got = orc.mha(q, kv, kv, None, mha, H, dk, dk)
    assert np.array_equal(got, orc.layernorm(q, mha["ln_scale"], mha["ln_shift"]))


from oracle import fp64_model as m64  # noqa: E402


def test_oracle_agrees_with_fp64_model_on_one_config3_token_block(orc):
    """Ties the referee used above to the oracle at the config-3 widths (D 1024, F 4096) on a short sequence."""
    B, L, D, H, dk, F = 1, 48, 1024, 16, 64, 4096
    rng = np.random.default_rng(33)
    x = rng.standard_normal((B, L, D)).astype(np.float32)
    attn, ffn = m64.make_params(rng, D, H, dk, dk, F, trivial_affine=True)
    mask = (np.arange(L)[None, None, None, :] >= 30).astype(np.float32)
    assert np.allclose(orc.encoder_block(x, mask, attn, ffn, H, dk, dk), m64.encoder_block64(x, mask, attn, ffn, H, dk, dk),
                       rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ the Transformer wrapper (oracle/transformer.py)
def test_log_sin_cos_against_numpy_fp64(orc):
    rng = np.random.default_rng(5)
    x = (rng.random(4096) * 600.0).astype(np.float32)
    assert np.allclose(orc.sin(x), np.sin(x.astype(np.float64)), atol=2e-6)
    assert np.allclose(orc.cos(x), np.cos(x.astype(np.float64)), atol=2e-6)
    p = (rng.random(4096) * 1e4 + 1e-3).astype(np.float32)
    assert np.allclose(orc.log(p), np.log(p.astype(np.float64)), rtol=1e-6, atol=1e-7)
    # Tests/DL4STests/VecTests.swift:242-258 checks log against Foundation.log to 1e-4 on 1...16
    v = np.arange(1, 17, dtype=np.float32)
    assert np.abs(orc.log(v) - np.log(np.arange(1, 17))).max() < 1e-4


def test_argmax_first_maximum_nan_and_empty(orc):
    rng = np.random.default_rng(6)
    x = rng.standard_normal(1000).astype(np.float32)
    assert orc.argmax(x) == (int(np.argmax(x)), float(x.max()))
    assert orc.argmax(np.array([1, 3, 3, 2], np.float32)) == (1, 3.0)                 # ties: the first
    assert orc.argmax(np.array([np.nan, -5, np.nan, -7], np.float32)) == (1, -5.0)    # NaN never selected
    i, v = orc.argmax(np.array([np.nan, np.nan], np.float32))
    assert i == 0 and v == -np.inf                                                     # nothing selected
    i, v = orc.argmax(np.zeros(0, np.float32))
    assert i == 0 and v == -np.inf


def test_embedding_is_table_indexing_with_zero_rows_for_ignore(orc):
    rng = np.random.default_rng(7)
    E = rng.standard_normal((11, 6)).astype(np.float32)
    tok = np.array([3, -1, 0, 10, 3], np.int32)
    out = orc.embedding(E, tok, -1)
    assert np.array_equal(out[[0, 2, 3, 4]], E[[3, 0, 10, 3]]) and not out[1].any()
    with pytest.raises(ValueError):
        orc.embedding(E, np.array([11], np.int32), -1)


def test_positional_encoding_closed_form():
    from oracle import transformer as T, fp64_model as m64
    pe = T.positional_encoding(50, 16)
    assert pe.shape == (50, 16) and pe.dtype == np.float32
    # Attention Is All You Need, 3.5, with sin and cos interleaved and the exponent i / (d/2)
    pos, i = np.arange(50)[:, None], np.arange(8)[None, :]
    angle = pos / 10000.0 ** (i / 8.0)
    assert np.allclose(pe[:, 0::2], np.sin(angle), atol=2e-5) and np.allclose(pe[:, 1::2], np.cos(angle), atol=2e-5)
    assert np.allclose(pe, m64.positional_encoding64(50, 16), atol=2e-5)
    assert np.array_equal(pe[0], np.tile([0.0, 1.0], 8).astype(np.float32))           # position 0: sin 0, cos 0


def test_log_softmax_against_scipy():
    import scipy.special
    from oracle import transformer as T
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((3, 5, 37)) * 4).astype(np.float32)
    got = T.log_softmax(x)
    assert np.allclose(got, scipy.special.log_softmax(x.astype(np.float64), axis=-1), atol=2e-6)
    assert np.allclose(np.exp(got.astype(np.float64)).sum(-1), 1.0, atol=1e-5)
    assert np.allclose(T.log_softmax(x + np.float32(3.0)), got, atol=2e-6)            # shift invariance


def _tiny_transformer(seed=9, vocab=13):
    from oracle import fp64_model as m64
    rng = np.random.default_rng(seed)
    # the hyper-parameters of Tests/DL4STests/TransformerTests.swift:31: hidden 16, heads 4, key/value dim 8, ffn 32
    return m64.make_transformer_params(rng, vocab, 16, 4, 8, 8, 32, 2, 2), rng


def test_transformer_forward_against_independent_fp64_model():
    from oracle import transformer as T, fp64_model as m64
    params, rng = _tiny_transformer()
    enc_len, dec_len = [7, 4, 6], [5, 3, 5]
    enc = np.full((3, 7), -1, np.int32)
    dec = np.full((3, 5), -1, np.int32)
    for b in range(3):
        enc[b, :enc_len[b]] = rng.integers(0, 13, enc_len[b])
        dec[b, :dec_len[b]] = rng.integers(0, 13, dec_len[b])
    got = T.forward(params, enc, dec, enc_len, dec_len)
    ref = m64.transformer64(params, enc, dec, enc_len, dec_len)
    assert got.shape == (3, 5, 13)
    assert np.abs(got - ref).max() < 2e-4
    assert np.allclose(np.exp(got.astype(np.float64)).sum(-1), 1.0, atol=1e-5)


def test_greedy_decode_is_consistent_with_the_forward_pass():
    """Token t of the greedy output is the argmax of the forward pass's distribution at the last position when the
    decoder is fed start + tokens[:t] (bias zero: greedy decoding leaves the output bias out, Transformer.swift:127-130)."""
    from oracle import transformer as T, fp64_model as m64
    params, rng = _tiny_transformer(seed=10)
    params["output_bias"] = np.zeros_like(params["output_bias"])
    src = [int(t) for t in rng.integers(0, 13, 6)]
    toks, logits = T.greedy_decode(params, src, 1, 2, 6, return_logits=True)
    assert 1 <= len(toks) <= 6 and (toks[-1] == 2 or len(toks) == 6) and 2 not in toks[:-1]
    for t, tok in enumerate(toks):
        prefix = [[1] + toks[:t]]
        lp = T.forward(params, [src], prefix, [len(src)], [t + 1])
        assert int(np.argmax(lp[0, -1])) == tok
        ref = m64.transformer64(params, np.array([src]), np.array(prefix), [len(src)], [t + 1], log_probs=False)
        assert np.abs(logits[t] - ref[0, -1]).max() < 2e-4


# ------------------------------------------------------------------ SDPA backward
@pytest.mark.parametrize("masked", [False, True])
def test_sdpa_backward_against_torch_autograd_fp64(orc, masked):
    import torch
    rng = np.random.default_rng(12)
    B, H, Lq, Lk, d = 2, 3, 9, 11, 8
    q, k, v = (rng.standard_normal(s).astype(np.float32) for s in ((B, H, Lq, d), (B, H, Lk, d), (B, H, Lk, d)))
    dout = rng.standard_normal((B, H, Lq, d)).astype(np.float32)
    mask = (rng.random((B, 1, Lq, Lk)) < 0.3).astype(np.float32) if masked else None
    if masked:
        mask[0, 0, 2, :] = 1.0          # a fully blocked row: uniform weights, gradient still defined
    dq, dk, dv = orc.sdpa_backward(q, k, v, mask, dout)
    tq, tk, tv = (torch.tensor(x, dtype=torch.float64, requires_grad=True) for x in (q, k, v))
    s = tq @ tk.transpose(-1, -2) / np.sqrt(d)
    if masked:
        # the value of a blocked score is what fp32 leaves of s - 1e9 (exactly -1e9 for |s| < 32, so a fully blocked row is
        # uniform), while the reference's closures pass the gradient through the subtraction unchanged
        collapsed = (s.detach().float() - torch.tensor(mask) * 1e9).double()
        s = s + (collapsed - s).detach()
    o = torch.softmax(s, dim=-1) @ tv
    o.backward(torch.tensor(dout, dtype=torch.float64))
    for got, ref, name in ((dq, tq.grad, "dq"), (dk, tk.grad, "dk"), (dv, tv.grad, "dv")):
        assert np.abs(got - ref.numpy()).max() < 2e-5, name


def test_sdpa_backward_against_finite_differences():
    """Directional derivative of sum(out * dout) along random directions, central differences in fp64 (independent model)."""
    from oracle import binding as orc, fp64_model as m64
    rng = np.random.default_rng(13)
    B, H, L, d = 1, 2, 6, 4
    q, k, v, dout = (rng.standard_normal((B, H, L, d)).astype(np.float32) for _ in range(4))
    i, j = np.indices((L, L))
    mask = (j > i).astype(np.float32)
    dq, dk, dv = orc.sdpa_backward(q, k, v, mask, dout)
    f = lambda q_, k_, v_: float((m64.sdpa64(q_, k_, v_, mask) * dout).sum())
    eps = 1e-6
    for grad, idx in ((dq, 0), (dk, 1), (dv, 2)):
        direction = rng.standard_normal((B, H, L, d))
        args_p = [x.astype(np.float64) for x in (q, k, v)]
        args_m = [x.astype(np.float64) for x in (q, k, v)]
        args_p[idx] = args_p[idx] + eps * direction
        args_m[idx] = args_m[idx] - eps * direction
        fd = (f(*args_p) - f(*args_m)) / (2 * eps)
        assert abs(fd - float((grad * direction).sum())) < 1e-4


def test_fp64_gradient_model_against_torch_autograd():
    """fp64_model.sdpa_backward64 (the referee where the fp32 oracle's own sums run out of precision) is the closed form
    of the gradients: torch autograd in fp64 on the same expression gives the same numbers to rounding."""
    import torch
    from oracle import fp64_model as m64
    rng = np.random.default_rng(14)
    q, dout = rng.standard_normal((2, 3, 9, 8)), rng.standard_normal((2, 3, 9, 8))
    k, v = rng.standard_normal((2, 3, 11, 8)), rng.standard_normal((2, 3, 11, 8))
    mask = (rng.random((9, 11)) < 0.3).astype(np.float64)
    mask[:, 0] = 0                                  # every row keeps a key
    tq, tk, tv = (torch.tensor(x, requires_grad=True) for x in (q, k, v))
    o = torch.softmax(tq @ tk.transpose(-1, -2) / np.sqrt(8) - torch.tensor(mask) * 1e9, -1) @ tv
    o.backward(torch.tensor(dout))
    for got, ref, name in zip(m64.sdpa_backward64(q, k, v, mask, dout), (tq, tk, tv), ("dq", "dk", "dv")):
        assert np.abs(got - ref.grad.numpy()).max() < 1e-13, name


def test_per_token_attention_variant_of_the_transformer_oracle(orc):
    """oracle.transformer.mha_per_token is not the reference's layer; it is pinned by two properties.  With a single
    position the joint normalisation and the per-token one are the same computation (bit for bit against the pinned
    layer).  And a decoder built from it is causal: its output at a position does not depend on later positions, bit for
    bit - which the reference's jointly normalised decoder is not, the reason its decoding cannot be cached."""
    from oracle import fp64_model as m64
    from oracle import transformer as T
    rng = np.random.default_rng(71)
    params = m64.make_transformer_params(rng, 13, 16, 4, 8, 8, 32, 2, 2)
    p = params["decoder"][0]["self"]
    x = rng.standard_normal((3, 1, 16)).astype(np.float32)
    kv = rng.standard_normal((3, 5, 16)).astype(np.float32)
    assert np.array_equal(T.mha_per_token(x, kv, kv, None, p, 4, 8, 8), orc.mha(x, kv, kv, None, p, 4, 8, 8))
    # several positions: each output row equals the jointly normalised layer applied to that row alone
    xs = rng.standard_normal((2, 4, 16)).astype(np.float32)
    whole = T.mha_per_token(xs, kv[:2], kv[:2], None, p, 4, 8, 8)
    for i in range(4):
        assert np.array_equal(whole[:, i:i + 1], orc.mha(xs[:, i:i + 1], kv[:2], kv[:2], None, p, 4, 8, 8))
    src = [3, 4, 5, 6]
    for per_token in (True, False):
        enc = T.encoder(params, T.prepare_inputs(params, [src]), [4], per_token)
        long = T.decoder(params, T.prepare_inputs(params, [[1, 3, 4, 5, 6]]), enc, [4], [5], per_token)
        short = T.decoder(params, T.prepare_inputs(params, [[1, 3, 4]]), enc, [4], [3], per_token)
        if per_token:
            assert np.array_equal(long[:, :3], short)
        else:
            assert np.abs(long[:, :3] - short).max() > 1e-3
