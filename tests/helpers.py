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
