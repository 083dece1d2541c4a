"""dl4s_hip_sdpa_decode_noalloc_f32 (partial records in the library's fixed device block, no allocation) against
dl4s_hip_sdpa_decode_f32 through the C ABI: the two share their kernels, so the bar is bit equality, and both are
held to the oracle's parity gate.  Two calls in a row, the second on a smaller input (fewer records than the first
call left behind in the block)."""
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


def _case(ctx, orc, seed, B, H, T, Tcap, d=64):
    rng = np.random.default_rng(seed)
    q = rng.standard_normal((B, H, 1, d)).astype(np.float32)
    kc = rng.standard_normal((B, H, Tcap, d)).astype(np.float32)
    vc = rng.standard_normal((B, H, Tcap, d)).astype(np.float32)
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))     # 0.125 at d = 64
    kc[:, :, T:] = np.nan     # rows beyond T are never read
    vc[:, :, T:] = np.nan
    dq, dk, dv = ctx.to_device(q), ctx.to_device(kc), ctx.to_device(vc)
    out_a, out_b = ctx.empty((B, H, 1, d)), ctx.empty((B, H, 1, d))
    ctx.fill(float("nan"), out_a, B * H * d)
    ctx.fill(float("nan"), out_b, B * H * d)
    in_use, pooled = ctx.mem_stats()
    ctx.sdpa_decode_noalloc(dq, dk, dv, out_a, B, H, T, Tcap, d, rT)
    assert ctx.mem_stats() == (in_use, pooled)       # the pool was not touched
    ctx.sdpa_decode(dq, dk, dv, out_b, B, H, T, Tcap, d, rT)
    a, b = out_a.numpy(), out_b.numpy()
    for buf in (dq, dk, dv, out_a, out_b):
        buf.release()
    assert np.array_equal(a, b), "no-alloc decode differs from dl4s_hip_sdpa_decode_f32 (B%d H%d T%d)" % (B, H, T)
    assert_parity(a, orc.sdpa_decode(q, kc, vc, T), "no-alloc decode B%d H%d T%d" % (B, H, T))


def test_no_alloc_decode_two_calls_the_second_smaller(ctx, orc):
    _case(ctx, orc, 1, 2, 4, 3000, 3072)     # 8 pairs: split over many workgroups, records in the fixed block
    _case(ctx, orc, 2, 1, 2, 700, 700)       # fewer pairs, fewer splits: most of the block keeps the first call's records
    _case(ctx, orc, 3, 2, 2, 300, 320)       # a short cache: one workgroup per pair, the block is not used at all
    _case(ctx, orc, 4, 2, 4, 3000, 3072, d=256)     # the widest rows: the largest records
    _case(ctx, orc, 5, 1, 3, 900, 900, d=96)


def test_no_alloc_decode_error_paths(ctx):
    """The size limit of the fixed block cannot be reached on a 256-CU GPU (the split rule asks for at most about 2048
    records there), so what is checked here is that the entry point refuses like the one it is a variant of."""
    from dl4s_amd import lib
    q, kc, out = ctx.empty((1, 1, 1, 64)), ctx.empty((1, 1, 8, 64)), ctx.empty((1, 1, 1, 64))
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.sdpa_decode_noalloc(q, kc, kc, out, 1, 1, 9, 8, 64, 0.125)     # T beyond the capacity
    assert e.value.code == -2
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.sdpa_decode_noalloc(q, kc, kc, out, 1, 1, 8, 8, 300, 0.125)    # a head dim no decode kernel takes
    assert e.value.code == -5
    for buf in (q, kc, out):
        buf.release()


def test_no_alloc_decode_from_two_contexts_of_one_gpu(ctx):
    """Two contexts (two streams) share the GPU's one fixed block: calls on them, issued back to back without a wait in
    between, must not see each other's partial records."""
    from dl4s_amd import lib
    other = lib.Context(0)
    try:
        rng = np.random.default_rng(77)
        cases = []
        for c, (B, H, T) in zip((ctx, other, ctx, other), ((2, 4, 3000), (1, 6, 2500), (1, 3, 1800), (2, 4, 2900))):
            q = rng.standard_normal((B, H, 1, 64)).astype(np.float32)
            kc = rng.standard_normal((B, H, T, 64)).astype(np.float32)
            vc = rng.standard_normal((B, H, T, 64)).astype(np.float32)
            cases.append((c, q, kc, vc, c.to_device(q), c.to_device(kc), c.to_device(vc), c.empty((B, H, 1, 64)), c.empty((B, H, 1, 64))))
        ctx.sync()
        other.sync()
        for _ in range(3):
            for c, q, kc, vc, dq, dk, dv, out, _ in cases:       # alternating contexts, nothing waits
                B, H, T = kc.shape[:3]
                c.sdpa_decode_noalloc(dq, dk, dv, out, B, H, T, T, 64, 0.125)
        for c, q, kc, vc, dq, dk, dv, out, ref in cases:
            B, H, T = kc.shape[:3]
            c.sdpa_decode(dq, dk, dv, ref, B, H, T, T, 64, 0.125)
            assert np.array_equal(out.numpy(), ref.numpy()), "B%d H%d T%d" % (B, H, T)
            for buf in (dq, dk, dv, out, ref):
                buf.release()
    finally:
        other.close()
