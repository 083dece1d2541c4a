import numpy as np

ATOL = 1e-4   # max-abs tolerance of the parity gate
RTOL = 1e-4   # max-rel tolerance of the parity gate


def assert_parity(got, ref, what=""):
    """|got - ref| <= ATOL + RTOL * |ref| element-wise, and NaN/Inf at exactly the same places."""
    got = np.asarray(got)
    ref = np.asarray(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    gn, rn = np.isnan(got), np.isnan(ref)
    assert np.array_equal(gn, rn), "%s: NaN placement differs (%d vs %d NaNs)" % (what, gn.sum(), rn.sum())
    gi, ri = np.isinf(got), np.isinf(ref)
    assert np.array_equal(gi, ri) and np.array_equal(got[gi], ref[ri]), "%s: Inf placement differs" % what
    ok = ~(rn | ri)
    d = np.abs(got[ok].astype(np.float64) - ref[ok].astype(np.float64))
    lim = ATOL + RTOL * np.abs(ref[ok].astype(np.float64))
    if d.size and not np.all(d <= lim):
        i = int(np.argmax(d - lim))
        raise AssertionError("%s: max |d|=%.3e (limit %.3e) at flat index %d; max-abs %.3e" % (what, d[i], lim[i], i, d.max()))
    return float(d.max()) if d.size else 0.0


def causal_mask(Lq, Lk):
    i, j = np.indices((Lq, Lk))
    return (j > i).astype(np.float32)


def lengths_mask(lens, Lk):
    return (np.arange(Lk)[None, None, None, :] >= np.asarray(lens)[:, None, None, None]).astype(np.float32)


def negative_variance_pairs(count=6):
    """Two-element rows [a, b] whose variance by the one-pass formula E[x^2] - E[x]^2 is negative in fp32.  With two
    elements every step has one possible order, so the fp32 value is fixed by the formula alone."""
    f = np.float32
    rng = np.random.default_rng(0)
    rows = []
    while len(rows) < count:
        a = f(rng.uniform(1, 2))
        b = f(a + f(rng.integers(-3, 4)) * np.spacing(a))
        mean = f(f(a + b) * f(0.5))
        var = f(f(f(f(a * a) + f(b * b)) * f(0.5)) - f(mean * mean))
        if var < 0:
            rows.append((a, b))
    return np.array(rows, f)
