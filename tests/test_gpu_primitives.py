"""Parity of the engine primitives (C ABI) against the CPU oracle: element-wise results bit-exact where the
arithmetic is a single IEEE operation, 1e-4 tolerance where summation order or libm differ."""
import zlib

import numpy as np
import pytest

from helpers import assert_parity, negative_variance_pairs

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx():
    from dl4s_amd import lib
    c = lib.Context(0)
    yield c
    c.close()


RNG = np.random.default_rng(21)


def rnd(*shape):
    return RNG.standard_normal(shape).astype(np.float32)


def test_pool_trim_returns_pooled_blocks_largest_first(ctx):
    a, b, c = ctx.empty((1 << 20,)), ctx.empty((1 << 16,)), ctx.empty((1 << 10,))
    ctx.fill(1.0, a, 1 << 20)
    for t in (a, b, c):
        t.release()
    _, pooled0 = ctx.mem_stats()
    assert pooled0 >= (4 << 20) + (4 << 16) + (4 << 10)
    ctx.pool_trim(pooled0 - (4 << 20))            # the 4 MiB block goes first
    used, pooled1 = ctx.mem_stats()
    assert pooled1 <= pooled0 - (4 << 20)
    ctx.pool_trim(0)
    assert ctx.mem_stats() == (used, 0)
    d = ctx.empty((1 << 20,))                     # the pool is empty: a fresh block, and everything still works
    ctx.fill(2.0, d, 1 << 20)
    assert d.numpy()[-1] == 2.0
    d.release()


def test_memory_roundtrip_views_and_stats(ctx):
    from dl4s_amd import lib
    import ctypes as C
    a = rnd(1000)
    d = ctx.to_device(a)
    assert np.array_equal(d.numpy(), a)
    # an offset view is pointer arithmetic; getSize reports what is left of the allocation
    sz = C.c_size_t()
    lib._check(ctx.lib.dl4s_hip_get_size(ctx.handle, C.c_void_p(d.offset(400)), C.byref(sz)))
    assert sz.value >= 3600
    v = C.c_float()
    lib._check(ctx.lib.dl4s_hip_get_value_f32(ctx.handle, C.c_void_p(d.offset(4 * 17)), C.byref(v)))
    assert v.value == a[17]
    lib._check(ctx.lib.dl4s_hip_set_pointee_f32(ctx.handle, C.c_void_p(d.offset(4 * 17)), C.c_float(2.5)))
    assert d.numpy()[17] == 2.5
    e = ctx.empty((1000,))
    lib._check(ctx.lib.dl4s_hip_assign_d2d(ctx.handle, C.c_void_p(e.ptr), C.c_void_p(d.ptr), C.c_size_t(4000)))
    assert e.numpy()[17] == 2.5
    used0, _ = ctx.mem_stats()
    d.release()
    e.release()
    used1, pooled = ctx.mem_stats()
    assert used1 < used0 and pooled > 0
    # freeing an offset view or freeing twice is an error, not a crash
    f = ctx.empty((16,))
    p = f.ptr
    assert ctx.lib.dl4s_hip_free(ctx.handle, C.c_void_p(f.offset(8))) == -1
    f.release()
    assert ctx.lib.dl4s_hip_free(ctx.handle, C.c_void_p(p)) == -1
    assert b"double free" in ctx.lib.dl4s_hip_last_error()
    assert ctx.lib.dl4s_hip_free(ctx.handle, None) == 0      # NULL is a no-op


def test_elementwise_bit_exact(ctx, orc):
    n = 100003
    a, b = rnd(n), np.abs(rnd(n)) + np.float32(0.5)      # b > 0: it is also the sqrt argument
    da, db, dy = ctx.to_device(a), ctx.to_device(b), ctx.empty((n,))
    for fn, ref in [(ctx.vadd, a + b), (ctx.vsub, a - b), (ctx.vmul, a * b), (ctx.vdiv, a / b)]:
        fn(da, db, dy, n)
        assert np.array_equal(dy.numpy(), ref)
    ctx.vneg(da, dy, n)
    assert np.array_equal(dy.numpy(), -a)
    ctx.relu(da, dy, n)
    assert np.array_equal(dy.numpy(), orc.relu(a))
    ctx.sqrt(db, dy, n)
    assert np.array_equal(dy.numpy(), orc.sqrt(b))
    ctx.exp(da, dy, n)
    assert_parity(dy.numpy(), orc.exp(a), "exp")
    ctx.tanh(da, dy, n)
    assert_parity(dy.numpy(), orc.tanh(a), "tanh")
    ctx.fill(1.5, dy, n)
    assert (dy.numpy() == 1.5).all()
    ctx.vadd(da, db, da, n)            # result may alias an input
    assert np.array_equal(da.numpy(), a + b)
    for x in (da, db, dy):
        x.release()


@pytest.mark.parametrize("ta", [False, True])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (5, 7, 6), (128, 128, 16), (130, 70, 33), (257, 129, 100), (64, 512, 512),
                                   (260, 132, 100), (516, 260, 36), (8, 4, 4), (1028, 1284, 520)])   # the last four: ragged tiles on the fast kernels
def test_gemm(ctx, orc, ta, tb, M, N, K):
    A = rnd(K, M) if ta else rnd(M, K)
    B = rnd(N, K) if tb else rnd(K, N)
    dA, dB, dC = ctx.to_device(A), ctx.to_device(B), ctx.empty((M, N))
    ctx.gemm(dA, A.shape, dB, B.shape, dC, 1.0, 0.0, ta, tb)
    ref = orc.gemm(A, B, ta, tb)
    assert_parity(dC.numpy(), ref, "gemm %s" % ((M, N, K, ta, tb),))
    # alpha, and beta = 0 must ignore whatever C held (NaN included)
    ctx.fill(float("nan"), dC, M * N)
    ctx.gemm(dA, A.shape, dB, B.shape, dC, 2.0, 0.0, ta, tb)
    assert_parity(dC.numpy(), orc.gemm(A, B, ta, tb, alpha=2.0), "gemm alpha")
    for x in (dA, dB, dC):
        x.release()


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("M,N,K", [(1, 512, 512), (5, 2048, 512), (32, 512, 2048), (33, 70, 64), (100, 8000, 512), (128, 33, 100),
                                   (17, 512, 68), (3, 5, 4096), (512, 64, 512), (300, 40, 100), (1000, 33, 64)])
def test_gemm_skinny_products(ctx, orc, M, N, K, tb):
    """Few rows against a whole weight matrix (the products of greedy decoding): the contraction is cut into slices over
    workgroups and added up in a fixed order.  Parity with the oracle, alpha / beta, and the same bits alone, batched and
    grouped."""
    A = rnd(M, K)
    B = (rnd(N, K) if tb else rnd(K, N)) * np.float32(0.2)     # weight-like magnitudes: two summation orders over 4096
    C0 = rnd(M, N)                                               # unit-variance terms differ by more than the gate
    dA, dB, dC = ctx.to_device(A), ctx.to_device(B), ctx.empty((M, N))
    ctx.gemm(dA, A.shape, dB, B.shape, dC, 1.0, 0.0, False, tb)
    ref = orc.gemm(A, B, False, tb)
    assert_parity(dC.numpy(), ref, "skinny gemm %s" % ((M, N, K, tb),))
    first = dC.numpy()
    ctx.gemm(dA, A.shape, dB, B.shape, dC, 1.0, 0.0, False, tb)
    assert np.array_equal(dC.numpy(), first)                      # no atomics: the same bits again
    dD = ctx.to_device(C0)
    ctx.gemm(dA, A.shape, dB, B.shape, dD, 2.0, 1.0, False, tb)  # beta accumulates
    assert_parity(dD.numpy(), 2.0 * ref + C0, "skinny alpha beta")
    # batched (shared right operand) and grouped launches give each product the bits of the single call
    A3 = np.stack([A, rnd(M, K), A])
    dA3, dC3 = ctx.to_device(A3), ctx.empty((3, M, N))
    ctx.gemm_batched(dA3, (M, K), M * K, dB, B.shape, 0, dC3, M * N, 3, 1.0, 0.0, False, tb)
    assert np.array_equal(dC3.numpy()[0], first) and np.array_equal(dC3.numpy()[2], first)
    assert_parity(dC3.numpy()[1], orc.gemm(A3[1], B, False, tb), "skinny batched")
    outs = [ctx.empty((M, N)) for _ in range(2)]
    ctx.gemm_grouped([dA, dA3.offset(M * K * 4)], A.shape, [dB, dB], B.shape, outs, 1.0, 0.0, False, tb)
    assert np.array_equal(outs[0].numpy(), first) and np.array_equal(outs[1].numpy(), dC3.numpy()[1])
    for x in [dA, dB, dC, dD, dA3, dC3] + outs:
        x.release()


@pytest.mark.parametrize("tb", [False, True])
def test_gemm_skinny_products_with_a_sliced_contraction(ctx, orc, tb):
    """K long enough that the skinny form also cuts the contraction over workgroups (partial blocks in scratch, added up
    by a second kernel): parity, and the bits of the single call when batched."""
    M, N, K, batch = 3, 70, 16400, 3
    A = rnd(batch, M, K)
    B = (rnd(N, K) if tb else rnd(K, N)) * np.float32(0.05)
    dA, dB, dC, d1 = ctx.to_device(A), ctx.to_device(B), ctx.empty((batch, M, N)), ctx.empty((M, N))
    ctx.gemm_batched(dA, (M, K), M * K, dB, B.shape, 0, dC, M * N, batch, 1.0, 0.0, False, tb)
    got = dC.numpy()
    for b in range(batch):
        ctx.gemm(dA.offset(b * M * K * 4), (M, K), dB, B.shape, d1, 1.0, 0.0, False, tb)
        assert np.array_equal(d1.numpy(), got[b])
        assert_parity(got[b], orc.gemm(A[b], B, False, tb), "sliced skinny %d" % b)
    for x in (dA, dB, dC, d1):
        x.release()


def test_gemm_known_answers_and_beta(ctx):
    # Tests/DL4STests/VecTests.swift:127-156
    c = np.array([[1, 2, 3], [4, 5, 6]], np.float32)
    dc, r33, r22 = ctx.to_device(c), ctx.empty((3, 3)), ctx.empty((2, 2))
    ctx.gemm(dc, c.shape, dc, c.shape, r33, 1.0, 0.0, True, False)
    assert r33.numpy().tolist() == [[17, 22, 27], [22, 29, 36], [27, 36, 45]]
    ctx.gemm(dc, c.shape, dc, c.shape, r22, 1.0, 0.0, False, True)
    assert r22.numpy().tolist() == [[14, 32], [32, 77]]
    ctx.gemm(dc, c.shape, dc, c.shape, r22, 1.0, 1.0, False, True)      # beta accumulates (cblas semantics)
    assert r22.numpy().tolist() == [[28, 64], [64, 154]]
    for x in (dc, r33, r22):
        x.release()


def test_gemm_shape_error(ctx):
    from dl4s_amd import lib
    a = ctx.empty((4, 4))
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.gemm(a, (2, 3), a, (2, 3), a)
    assert e.value.code == -2
    a.release()


def test_gemm_batched_equals_loop_and_stack(ctx, orc):
    B, M, N, K = 5, 70, 40, 64
    A, W = rnd(B, M, K), rnd(K, N)
    dA, dW, dC = ctx.to_device(A), ctx.to_device(W), ctx.empty((B, M, N))
    ctx.gemm_batched(dA, (M, K), M * K, dW, (K, N), 0, dC, M * N, B)
    assert_parity(dC.numpy(), orc.bmm(A, W), "batched gemm")
    # the reference's form: one gemm per slice into its own buffer, then stack
    parts = [ctx.empty((M, N)) for _ in range(B)]
    for b in range(B):
        ctx.gemm(dA.offset(b * M * K * 4), (M, K), dW, (K, N), parts[b])
    dS = ctx.empty((B, M, N))
    ctx.stack(parts, M * N, dS)
    assert np.array_equal(dS.numpy(), dC.numpy())
    for x in [dA, dW, dC, dS] + parts:
        x.release()


@pytest.mark.parametrize("M,N,K,ta,tb", [(256, 128, 64, False, False), (2048, 512, 512, False, False), (70, 40, 30, False, False),
                                          (128, 64, 96, True, False), (96, 200, 64, False, True), (5, 7, 3, True, True)])
@pytest.mark.parametrize("count", [1, 2, 3, 4])
def test_gemm_grouped_gives_the_bits_of_single_calls(ctx, orc, M, N, K, ta, tb, count):
    """The three projections of NN/Models/Transformer/MultiHeadAttention.swift:105-107 as one launch: same bits as one call
    each, whatever tile size either launch picks; operands may repeat within a group."""
    As = [rnd(K, M) if ta else rnd(M, K) for _ in range(count)]
    Bs = [rnd(N, K) if tb else rnd(K, N) for _ in range(count)]
    dA, dB = [ctx.to_device(a) for a in As], [ctx.to_device(b) for b in Bs]
    if count >= 3:
        dA[2], As[2] = dA[0], As[0]          # a shared left operand, like q = k = v
    single, grouped = [ctx.empty((M, N)) for _ in range(count)], [ctx.empty((M, N)) for _ in range(count)]
    for i in range(count):
        ctx.gemm(dA[i], As[i].shape, dB[i], Bs[i].shape, single[i], 1.0, 0.0, ta, tb)
    ctx.gemm_grouped(dA, As[0].shape, dB, Bs[0].shape, grouped, 1.0, 0.0, ta, tb)
    for i in range(count):
        assert np.array_equal(single[i].numpy(), grouped[i].numpy())
        assert_parity(grouped[i].numpy(), orc.gemm(As[i], Bs[i], ta, tb), "grouped gemm %d" % i)
    for x in set(dA) | set(dB) | set(single) | set(grouped):
        x.release()


@pytest.mark.parametrize("M,N,K,ta,tb", [(2048, 512, 512, False, False), (1000, 1000, 256, False, False), (1030, 900, 384, False, True),
                                          (1024, 1024, 1024, False, False), (512, 512, 256, True, False), (640, 320, 768, True, True)])
def test_gemm_products_summed_in_two_halves(ctx, orc, M, N, K, ta, tb):
    """Products of at most one 64 x 64 tile per CU whose K is a multiple of 128 (from 256 on) are summed as two halves
    (so that a launch of one such product can put two groups of wavefronts on every tile).  The order is a property of the
    product's shape: the call alone (two groups side by side), a batch that fills the GPU (one group, the first half set
    aside at the middle), a group of three and the product with an epilogue give the same bits; against an fp64 product."""
    rng = np.random.default_rng(zlib.crc32(repr(("halves", M, N, K, ta, tb)).encode()))
    count = 6
    As = [rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32) for _ in range(count)]
    Bm = (rng.standard_normal((N, K) if tb else (K, N)) * 0.1).astype(np.float32)
    dA, dB = ctx.to_device(np.stack(As)), ctx.to_device(Bm)
    single = [ctx.empty((M, N)) for _ in range(count)]
    for i in range(count):
        ctx.gemm(dA.offset(i * As[0].size * 4), As[0].shape, dB, Bm.shape, single[i], 1.0, 0.0, ta, tb)
    ref = (As[0].T if ta else As[0]).astype(np.float64) @ (Bm.T if tb else Bm).astype(np.float64)
    bound = 2e-6 * np.sqrt(K) * (np.abs(ref).max() + 1.0) + 1e-6
    assert np.abs(single[0].numpy() - ref).max() <= bound
    batched = ctx.empty((count, M, N))
    ctx.gemm_batched(dA, As[0].shape, As[0].size, dB, Bm.shape, 0, batched, M * N, count, 1.0, 0.0, ta, tb)
    got = batched.numpy()
    for i in range(count):
        assert np.array_equal(got[i], single[i].numpy()), "batch item %d" % i
    grouped = [ctx.empty((M, N)) for _ in range(3)]
    ctx.gemm_grouped([dA.offset(i * As[0].size * 4) for i in range(3)], As[0].shape, [dB] * 3, Bm.shape, grouped, 1.0, 0.0, ta, tb)
    for i in range(3):
        assert np.array_equal(grouped[i].numpy(), single[i].numpy()), "group entry %d" % i
    keep = [dA, dB, batched] + single + grouped
    if not ta and not tb:      # the epilogue forms: + 0 leaves the bits (no sum here is -0)
        zero, fused = ctx.to_device(np.zeros((M, N), np.float32)), ctx.empty((M, N))
        ctx.dense_fused(dA, M, K, dB, N, None, 0, zero, fused)
        assert np.array_equal(fused.numpy(), single[0].numpy())
        keep += [zero, fused]
    for x in keep:
        x.release()


def test_gemm_grouped_argument_errors(ctx):
    from dl4s_amd import lib
    a = ctx.empty((4, 4))
    with pytest.raises(lib.Dl4sHipError):
        ctx.gemm_grouped([a] * 5, (4, 4), [a] * 5, (4, 4), [a] * 5)
    with pytest.raises(lib.Dl4sHipError):
        ctx.gemm_grouped([a, 0], (4, 4), [a, a], (4, 4), [a, a])
    ctx.gemm_grouped([], (4, 4), [], (4, 4), [])
    a.release()


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
@pytest.mark.parametrize("sa,sb", [((2, 3, 4), (4,)), ((2, 3, 4), (3, 1)), ((2, 3, 4), ()), ((), (2, 3)), ((2, 1, 4), (1, 3, 1)),
                                   ((2, 3, 4, 5), (2, 1, 1, 5)), ((3, 4), (3, 4)), ((2, 2, 33, 33), (33, 33)), ((40, 1), (1, 50)),
                                   ((2, 3, 7, 9), (2, 3, 7, 1)),
                                   # 128-bit paths of the merged-axes kernel: inner group taken by both, by lhs only, by rhs only
                                   ((2, 3, 64, 64), (64, 64)), ((4, 8, 16), (4, 8, 1)), ((8, 1), (8, 12)), ((5, 16), (1, 16)),
                                   ((3, 1, 8), (1, 5, 1)), ((6, 40), ()),
                                   # more than three groups: the general kernel
                                   ((2, 3, 4, 5, 6), (2, 1, 4, 1, 6)), ((2, 1, 4, 1, 6), (2, 3, 1, 5, 1))])
def test_broadcast_bit_exact(ctx, orc, op, sa, sb):
    from dl4s_amd import lib
    a, b = rnd(*sa), rnd(*sb) + np.float32(2.5)
    ref = orc.broadcast(op, a, b)
    da, db, dy = ctx.to_device(a), ctx.to_device(b), ctx.empty(ref.shape)
    ctx.broadcast({"add": lib.OP_ADD, "sub": lib.OP_SUB, "mul": lib.OP_MUL, "div": lib.OP_DIV}[op], da, sa, db, sb, dy)
    assert np.array_equal(dy.numpy(), ref)          # includes x*(1/s) and x+(-s) roundings of the scalar forms
    for x in (da, db, dy):
        x.release()


def test_broadcast_on_operands_that_are_not_16_byte_aligned(ctx, orc):
    """Offset views (a row of a larger tensor starting at an odd element) take the element-wise path of the same kernel."""
    from dl4s_amd import lib
    a, b = rnd(3 * 64 + 1), rnd(64 + 3)
    da, db, dy = ctx.to_device(a), ctx.to_device(b), ctx.empty((3 * 64 + 1,))
    ctx.broadcast(lib.OP_SUB, da.offset(4), (3, 64), db.offset(12), (64,), dy.offset(4))
    assert np.array_equal(dy.numpy()[1:].reshape(3, 64), orc.broadcast("sub", a[1:].reshape(3, 64), b[3:]))
    ctx.broadcast(lib.OP_MUL, da, (3, 64), db.offset(12), (64,), dy)        # only rhs off the grid
    assert np.array_equal(dy.numpy()[:192].reshape(3, 64), orc.broadcast("mul", a[:192].reshape(3, 64), b[3:]))
    for x in (da, db, dy):
        x.release()


def test_broadcast_shape_error(ctx):
    from dl4s_amd import lib
    a = ctx.empty((12,))
    with pytest.raises(lib.Dl4sHipError) as e:
        ctx.broadcast(lib.OP_ADD, a, (3, 4), a, (2, 4), a)
    assert e.value.code == -2
    a.release()


@pytest.mark.parametrize("shape,axes", [((3, 4, 5), [2]), ((3, 4, 5), [1, 2]), ((3, 4, 5), [0]), ((2, 3, 4, 50), [3]),
                                        ((2, 300, 70), [1, 2]), ((6,), [0]), ((4, 5), [0, 1]), ((4, 512, 512), [1, 2]),
                                        ((3, 1, 7, 1, 5), [1, 2]), ((2, 3, 4, 5), [0, 2]), ((2, 3, 4, 5), [1, 3]), ((1, 1), [0]),
                                        ((700000,), [0]), ((2, 200, 1, 300), [1, 2, 3]),
                                        # many short contiguous rows: one wavefront per row
                                        ((4, 300, 70), [2]), ((2, 8, 128, 130), [3]), ((1200, 3, 5), [1, 2]), ((1025, 1), [1]),
                                        ((1100, 4096), [1])])
def test_reduce_sum(ctx, orc, shape, axes):
    x = rnd(*shape)
    ref = orc.reduce_sum(x, axes)
    dx, dy = ctx.to_device(x), ctx.empty(ref.shape if ref.shape else (1,))
    ctx.reduce_sum(dx, shape, axes, dy)
    assert_parity(dy.numpy().reshape(ref.shape), ref, "reduceSum")
    dx.release()
    dy.release()


@pytest.mark.parametrize("shape,axis", [((3, 4, 5), 2), ((3, 4, 5), 1), ((3, 4, 5), 0), ((2, 2, 9, 1000), 3),
                                        ((2, 8, 128, 130), 3), ((1100, 7), 1)])
def test_reduce_max_exact_and_nan_skipping(ctx, orc, shape, axis):
    x = rnd(*shape)
    x.flat[3] = np.nan
    ref = orc.reduce_max(x, axis)
    dx, dy = ctx.to_device(x), ctx.empty(ref.shape)
    ctx.reduce_max(dx, shape, axis, dy)
    assert np.array_equal(dy.numpy(), ref)
    dx.release()
    dy.release()


@pytest.mark.parametrize("shape,arr", [((2, 3, 4, 5), (0, 2, 1, 3)), ((2, 3, 4, 5), (1, 2, 3, 0)), ((2, 3, 4, 5), (3, 0, 1, 2)),
                                       ((7, 9), (1, 0)), ((4, 16, 8, 64), (0, 2, 1, 3))])
def test_permute_axes_scatter_convention(ctx, orc, shape, arr):
    x = rnd(*shape)
    ref = orc.permute(x, arr)
    dx, dy = ctx.to_device(x), ctx.empty(ref.shape)
    ctx.permute_axes(dx, shape, arr, dy)
    assert np.array_equal(dy.numpy(), ref)
    dx.release()
    dy.release()


def test_band_and_decoder_mask_recipe(ctx, orc):
    from dl4s_amd import lib
    L = 37
    ones = np.ones((L, L), np.float32)
    dx, dy = ctx.to_device(ones), ctx.empty((L, L))
    for below, above in [(-1, None), (0, 0), (None, 0), (2, 3), (None, None)]:
        ctx.fill(0.0, dy, L * L)                   # bandMatrix zero-fills first (UtilOps.swift:117-121)
        ctx.band(dx, dy, L, L, below, above)
        assert np.array_equal(dy.numpy(), orc.band(ones, below, above)), (below, above)
    dx.release()
    dy.release()


@pytest.mark.parametrize("B,rows,D", [(3, 7, 16), (5, 1, 1024), (4, 512, 512), (2, 1, 33), (3, 1, 4096), (2, 300, 68), (2, 2000, 33),
                                       (6, 1, 12), (2, 40, 1028), (1, 20, 512), (2, 16, 1024), (3, 150, 33), (1, 32, 512)])
# vector and scalar paths, short and long rows (one workgroup of 256 or of 1024 threads, or two kernels), D not dividing the stride
def test_layernorm(ctx, orc, B, rows, D):
    x, res = rnd(B, rows, D) * 2 + np.float32(0.3), rnd(B, rows, D)
    scale, shift = rnd(D), rnd(D)
    dx, dr, ds, dh, dy = ctx.to_device(x), ctx.to_device(res), ctx.to_device(scale), ctx.to_device(shift), ctx.empty((B, rows, D))
    ctx.layernorm(dx, None, ds, dh, dy, B, rows, D)
    assert_parity(dy.numpy(), orc.layernorm(x, scale, shift), "layernorm")
    ctx.layernorm(dx, dr, ds, dh, dy, B, rows, D)
    assert_parity(dy.numpy(), orc.layernorm(x + res, scale, shift), "layernorm+residual")
    for t in (dx, dr, ds, dh, dy):
        t.release()


SLICES = [   # shape, index as numpy would write it (int, slice or None = whole axis)
    ((5, 7), (2, None)),                      # a prefix index (the reference returns a view; the copy must agree)
    ((5, 7), (None, 3)),                      # a column: runs of one float
    ((4, 6, 8), (None, 2, None)),
    ((4, 6, 8), (1, None, 5)),
    ((4, 6, 8), (slice(1, 3), slice(0, 6), slice(4, 8))),     # ranges; 128-bit pieces
    ((4, 6, 8), (slice(1, 3), slice(2, 5), slice(1, 7))),
    ((3, 4, 5, 6), (None, slice(1, 2), None, slice(0, 6))),
    ((2, 3, 4, 5, 6), (1, None, slice(1, 4), 2, None)),
    ((64, 1024), (slice(3, 60), slice(128, 896))),
    ((7,), (slice(2, 2),)),                   # empty
    ((6, 5), ()),                             # everything
]


def test_log_of_exp_and_sigmoid_as_the_reference_tests_them(ctx):
    """Tests/DL4STests/VecTests.swift:158-168 (testLog: log(exp(x)) = x to 1e-4 on a 10 x 10 tensor uniform in [-5, 5]) and
    :242-258 (testSigmoid: 1 / (1 + exp(-a)) against the scalar formula to 1e-4), issued as the engine calls those
    tensor expressions make: exp, log; negate, exp, scalar + tensor, scalar / tensor."""
    from dl4s_amd import lib
    rng = np.random.default_rng(158)
    x = rng.uniform(-5, 5, (10, 10)).astype(np.float32)
    dx, dy = ctx.to_device(x), ctx.empty((10, 10))
    ctx.exp(dx, dy, 100)
    ctx.log(dy, dy, 100)
    assert np.abs(dy.numpy() - x).max() <= 1e-4
    a = rng.standard_normal(10).astype(np.float32)
    da, dt, one = ctx.to_device(a), ctx.empty((10,)), ctx.to_device(np.ones((), np.float32))
    ctx.vneg(da, dt, 10)
    ctx.exp(dt, dt, 10)
    ctx.broadcast(lib.OP_ADD, one, (), dt, (10,), dt)
    ctx.broadcast(lib.OP_DIV, one, (), dt, (10,), dt)
    ref = 1.0 / (1.0 + np.exp(-a.astype(np.float64)))
    assert np.abs(dt.numpy() - ref).max() <= 1e-4
    for t in (dx, dy, da, dt, one):
        t.release()


def test_subscript_known_answers_of_the_reference(ctx):
    """The reference's own slice tests, value for value (Tests/DL4STests/EngineV2Tests.swift:235-287, testSubscriptSlice
    and testSubscriptSliceWrite; the values 0 ... 8 are exact in fp32)."""
    a = np.arange(9, dtype=np.float32).reshape(3, 3)
    da = ctx.to_device(a)
    reads = [((0, 0), (3, 2), [[0, 1], [3, 4], [6, 7]]),          # a[nil, 0 ..< 2]
             ((0, 1), (3, 2), [[1, 2], [4, 5], [7, 8]]),          # a[nil, 1 ..< 3]
             ((0, 0), (2, 3), [[0, 1, 2], [3, 4, 5]]),            # a[0 ..< 2]
             ((1, 0), (2, 3), [[3, 4, 5], [6, 7, 8]])]            # a[1 ..< 3]
    for start, extent, expected in reads:
        dy = ctx.empty(extent)
        ctx.subscript_read(da, (3, 3), start, extent, dy)
        assert np.array_equal(dy.numpy(), np.array(expected, np.float32))
        dy.release()
    src = ctx.to_device(np.array([[0, 1], [3, 4], [6, 7]], np.float32))
    writes = [((0, 0), [[0, 1, 0], [3, 4, 0], [6, 7, 0]]),        # result[nil, 0 ..< 2] = src1
              ((0, 1), [[0, 0, 1], [0, 3, 4], [0, 6, 7]])]        # result[nil, 1 ..< 3] = src1
    for start, expected in writes:
        dr = ctx.to_device(np.zeros((3, 3), np.float32))
        ctx.subscript_write(src, dr, (3, 3), start, (3, 2))
        assert np.array_equal(dr.numpy(), np.array(expected, np.float32))
        dr.release()
    da.release()
    src.release()


@pytest.mark.parametrize("shape,index", SLICES)
def test_subscript_read_and_write_match_numpy_slicing(ctx, shape, index):
    """Engine/Engine.swift:493-500 and MemoryOperatorsType.get / set(slice:) (semantics Engine/CPU/CPU.swift:137-218): one
    launch per slice, bit-exact against numpy's slicing of the same tensor."""
    x = rnd(*shape)
    idx = tuple(index) + (None,) * (len(shape) - len(index))
    start = [i if isinstance(i, int) else (i.start if isinstance(i, slice) else 0) for i in idx]
    extent = [1 if isinstance(i, int) else ((i.stop - i.start) if isinstance(i, slice) else n) for i, n in zip(idx, shape)]
    box = tuple(slice(s, s + e) for s, e in zip(start, extent))
    want = x[box]                                   # the axes an integer index would drop are kept with extent 1
    dx, dy = ctx.to_device(x), ctx.empty(tuple(extent))
    ctx.fill(float("nan"), dy, int(np.prod(extent)))
    ctx.subscript_read(dx, shape, start, extent, dy)
    assert np.array_equal(dy.numpy(), want)
    # write: the box takes new values, every other element keeps its own
    new = rnd(*extent)
    dn = ctx.to_device(new)
    ctx.subscript_write(dn, dx, shape, start, extent)
    expect = x.copy()
    expect[box] = new
    assert np.array_equal(dx.numpy(), expect)
    for t in (dx, dy, dn):
        t.release()


def test_subscript_box_outside_the_tensor_is_refused(ctx):
    from dl4s_amd import lib
    dx, dy = ctx.empty((4, 6)), ctx.empty((4, 6))
    for start, extent in (([0, 3], [4, 4]), ([-1, 0], [2, 2]), ([4, 0], [1, 6])):
        with pytest.raises(lib.Dl4sHipError) as e:
            ctx.subscript_read(dx, (4, 6), start, extent, dy)
        assert e.value.code == -2
        with pytest.raises(lib.Dl4sHipError) as e:
            ctx.subscript_write(dy, dx, (4, 6), start, extent)
        assert e.value.code == -2
    dx.release()
    dy.release()


def _ln(ctx, x, scale, shift):
    B, rows, D = x.shape
    dx, ds, dh, dy = ctx.to_device(x), ctx.to_device(scale), ctx.to_device(shift), ctx.empty((B, rows, D))
    ctx.layernorm(dx, None, ds, dh, dy, B, rows, D)
    y = dy.numpy()
    for t in (dx, ds, dh, dy):
        t.release()
    return y


@pytest.mark.parametrize("B,rows,D", [(3, 5, 64), (15, 1, 64), (2, 300, 68), (4, 1, 1024), (2, 1, 33)])
def test_layernorm_low_variance_input(ctx, orc, B, rows, D):
    """Standard deviation 1e-3: eps = 1e-5 outside the root (NN/Layer/LayerNorm.swift:75) is 1 % of the denominator;
    inside the root it would be 3.2e-3, three times the standard deviation."""
    x = rnd(B, rows, D) * np.float32(1e-3)
    scale, shift = rnd(D), rnd(D)
    got = _ln(ctx, x, scale, shift)
    assert_parity(got, orc.layernorm(x, scale, shift), "layernorm, low variance")
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=(1, 2), keepdims=True)
    std = np.sqrt((x64 * x64).mean(axis=(1, 2), keepdims=True) - mean * mean)
    assert np.allclose(got, (x64 - mean) / (std + 1e-5) * scale + shift, rtol=1e-3, atol=1e-4)


def test_layernorm_negative_one_pass_variance_gives_nan_rows(ctx, orc):
    """var = E[x^2] - E[x]^2 in fp32 (Tensor/Operators/Reduce.swift:106-110) is negative for some rows, the root is NaN
    and so is the row.  On two-element rows every sum has one possible order, so the kernel must agree with the oracle on
    which rows those are."""
    bad = negative_variance_pairs(8)
    good = np.array([[1.5, 2.5], [-3.0, 3.0], [0.1, 0.7]], np.float32)
    x = np.concatenate([bad[:4], good, bad[4:]]).reshape(-1, 1, 2)
    scale, shift = np.array([2.0, -1.0], np.float32), np.array([0.5, 0.25], np.float32)
    with np.errstate(invalid="ignore"):
        ref = orc.layernorm(x, scale, shift)
    assert np.isnan(ref[:4]).all() and np.isnan(ref[7:]).all() and np.isfinite(ref[4:7]).all()
    assert_parity(_ln(ctx, x, scale, shift), ref, "layernorm, negative variance")


@pytest.mark.parametrize("rows,D", [(1, 1024), (64, 512)])
def test_layernorm_off_centre_input(ctx, orc, rows, D):
    """The one-pass variance loses (mean / std)^2 * 2^-24 of relative precision per rounding of the sums.  Up to a mean
    of 3 standard deviations the kernel's tree sums and the oracle's sequential sums agree inside the parity gate.  At
    1000 standard deviations the formula's fp32 value is rounding noise of whichever summation order is used (the
    oracle pins show the same formula with pairwise sums as far from the sequential sums as from the exact result), so
    only what every order shares is asserted: a row is NaN as a whole or not at all."""
    scale, shift = np.ones(D, np.float32), np.zeros(D, np.float32)
    near = rnd(8, rows, D) + np.float32(3)
    assert_parity(_ln(ctx, near, scale, shift), orc.layernorm(near, scale, shift), "layernorm, mean = 3 std")
    far = rnd(8, rows, D) + np.float32(1000)
    got = _ln(ctx, far, scale, shift)
    nan_rows = np.isnan(got).any(axis=(1, 2))
    assert np.array_equal(nan_rows, np.isnan(got).all(axis=(1, 2)))


def _ln_ref_order(ctx, x, scale, shift, res=None):
    B, rows, D = x.shape
    dx, ds, dh, dy = ctx.to_device(x), ctx.to_device(scale), ctx.to_device(shift), ctx.empty((B, rows, D))
    dr = ctx.to_device(res) if res is not None else None
    ctx.layernorm_reference_order(dx, dr, ds, dh, dy, B, rows, D)
    y = dy.numpy()
    for t in (dx, ds, dh, dy) + ((dr,) if dr is not None else ()):
        t.release()
    return y


def _same_bits(a, b):
    return np.array_equal(a.view(np.uint32), b.view(np.uint32)) or np.array_equal(a, b, equal_nan=True)


@pytest.mark.parametrize("B,rows,D", [(3, 5, 64), (15, 1, 64), (2, 300, 68), (4, 1, 1024), (2, 1, 33), (1, 130, 1), (70, 1, 7),
                                      (2, 64, 128), (3, 65, 63), (2, 512, 512), (1, 1024, 1024),
                                      (2, 8200, 260)])      # the last: enough rows for the 32-row form, a second column step of 4
def test_layernorm_in_the_reference_order_is_the_oracle_bit_for_bit(ctx, orc, B, rows, D):
    """The sums of dl4s_hip_layernorm_reference_order_f32 are the reference's sequential ones, every other step one
    correctly rounded operation: the result is the oracle's to the last bit, with and without the residual."""
    x, res = rnd(B, rows, D) * 2 + np.float32(0.3), rnd(B, rows, D)
    scale, shift = rnd(D), rnd(D)
    assert _same_bits(_ln_ref_order(ctx, x, scale, shift), orc.layernorm(x, scale, shift))
    assert _same_bits(_ln_ref_order(ctx, x, scale, shift, res), orc.layernorm(x + res, scale, shift))


@pytest.mark.parametrize("rows,D", [(1, 1024), (64, 512), (16, 256)])
@pytest.mark.parametrize("offset", [3.0, 10.0, 1000.0])
def test_layernorm_off_centre_input_in_the_reference_order(ctx, orc, rows, D, offset):
    """Far from a zero mean the one-pass variance is rounding noise of the summation order; in the reference's order the
    kernel gives the reference's numbers, NaN rows (a negative variance under the root) included."""
    scale, shift = rnd(D), rnd(D)
    x = rnd(8, rows, D) + np.float32(offset)
    with np.errstate(invalid="ignore"):
        ref = orc.layernorm(x, scale, shift)
    assert _same_bits(_ln_ref_order(ctx, x, scale, shift), ref)


@pytest.mark.parametrize("rows,D", [(1, 1024), (1, 512), (32, 256)])
def test_layernorm_negative_variance_at_full_row_length_in_the_reference_order(ctx, orc, rows, D):
    """Items whose elements sit within a few ulp of one value: the variance is zero up to the rounding of the two sums, so
    its sign - a finite item or a NaN item - is decided by the order of every single addition.  The tree-sum kernel cannot
    be held to the oracle here; this one must give NaN for exactly the oracle's items."""
    rng = np.random.default_rng(rows * 7919 + D)
    B = 64
    base = rng.uniform(1, 2, (B, 1, 1)).astype(np.float32)
    x = (base + rng.integers(-3, 4, (B, rows, D)).astype(np.float32) * np.spacing(base)).astype(np.float32)
    scale, shift = np.ones(D, np.float32), np.zeros(D, np.float32)
    with np.errstate(invalid="ignore"):
        ref = orc.layernorm(x, scale, shift)
    nan_items = np.isnan(ref).all(axis=(1, 2))
    assert 4 <= nan_items.sum() <= B - 4, "the input must mix NaN items and finite ones (%d of %d)" % (nan_items.sum(), B)
    assert _same_bits(_ln_ref_order(ctx, x, scale, shift), ref)


def test_bias_gelu(ctx, orc):
    rows, D = 50, 129
    x, bias = rnd(rows, D) * 3, rnd(D)
    dx, db, dy = ctx.to_device(x), ctx.to_device(bias), ctx.empty((rows, D))
    ctx.bias_gelu(dx, db, dy, rows, D)
    assert_parity(dy.numpy(), orc.gelu(x + bias), "bias+gelu")
    ctx.bias_gelu(dx, None, dy, rows, D)
    assert_parity(dy.numpy(), orc.gelu(x), "gelu")
    for t in (dx, db, dy):
        t.release()


@pytest.mark.parametrize("M,K,N", [(130, 64, 72), (256, 128, 256), (64, 512, 1024), (7, 5, 3), (300, 100, 260),
                                   (5, 512, 2048), (31, 2048, 512), (100, 68, 70)])      # the last three: skinny products
@pytest.mark.parametrize("act", [0, 1])
@pytest.mark.parametrize("with_bias,with_res", [(True, False), (False, True), (True, True)])
def test_dense_fused_equals_separate_engine_calls(ctx, orc, M, K, N, act, with_bias, with_res):
    """act(x.W + b) + r as one product with an epilogue: the same bits as gemm, then bias (+ GELU), then vAdd, and within
    tolerance of the oracle's Dense / gaussianErrorLinear / residual sequence."""
    from dl4s_amd import lib
    x, W, b, r = rnd(M, K), rnd(K, N) * np.float32(0.2), rnd(N), rnd(M, N)
    dx, dW, db, dr = ctx.to_device(x), ctx.to_device(W), ctx.to_device(b), ctx.to_device(r)
    fused, sep = ctx.empty((M, N)), ctx.empty((M, N))
    ctx.dense_fused(dx, M, K, dW, N, db if with_bias else None, act, dr if with_res else None, fused)
    ctx.gemm(dx, (M, K), dW, (K, N), sep)
    if act:
        ctx.bias_gelu(sep, db if with_bias else None, sep, M, N)
    elif with_bias:
        ctx.broadcast(lib.OP_ADD, sep, (M, N), db, (N,), sep)
    if with_res:
        ctx.vadd(sep, dr, sep, M * N)
    assert np.array_equal(fused.numpy(), sep.numpy())
    ref = orc.gemm(x, W, False, False)
    if with_bias:
        ref = ref + b
    if act:
        ref = orc.gelu(ref)
    if with_res:
        ref = ref + r
    assert_parity(fused.numpy(), ref, "dense fused")
    # the result may alias the residual
    if with_res:
        ctx.dense_fused(dx, M, K, dW, N, db if with_bias else None, act, dr, dr)
        assert np.array_equal(dr.numpy(), fused.numpy())
    for t in (dx, dW, db, dr, fused, sep):
        t.release()


@pytest.mark.parametrize("items,item_rows,K,N", [
    (4, 512, 512, 512),      # 64 x 64 tiles, 64 pairs per item: the tail of a config-2 attention layer
    (8, 1024, 64, 1024),     # 128 x 128 tiles, 64 pairs per item
    (2, 128, 64, 2048),      # 32 pairs per item
    (3, 64, 128, 260),       # a last column tile that is partly outside
    (5, 128, 4, 512),        # a contraction of one MFMA step
    (2, 100, 128, 256),      # items that are not whole tiles: two calls
    (600, 1, 128, 128),      # per-row statistics: two calls
    (2, 30, 512, 512),       # a skinny product: two calls
    (1, 8192, 64, 512),      # more pairs than the normalising pass sums: two calls
])
@pytest.mark.parametrize("with_bias,act,with_res", [(False, 0, True), (True, 1, False), (True, 0, True), (False, 0, False)])
def test_dense_layernorm_in_one_call(ctx, orc, items, item_rows, K, N, with_bias, act, with_res):
    """LayerNorm(act(x.W + b) + r) with the statistics taken from the product's epilogue: within the gate of the oracle's
    Dense / gaussianErrorLinear / residual / LayerNorm sequence, and within rounding of the two separate calls (same
    arithmetic per element, the sums added in another order)."""
    rng = np.random.default_rng(zlib.crc32(repr(("dln", items, item_rows, K, N, with_bias, act, with_res)).encode()))
    M = items * item_rows
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) * 0.2).astype(np.float32)
    b, r = rng.standard_normal(N).astype(np.float32), rng.standard_normal((M, N)).astype(np.float32)
    scale, shift = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32), (0.1 * rng.standard_normal(N)).astype(np.float32)
    dx, dW, db, dr, dsc, dsh = (ctx.to_device(a) for a in (x, W, b, r, scale, shift))
    one, two = ctx.empty((M, N)), ctx.empty((M, N))
    ctx.dense_layernorm(dx, M, K, dW, N, db if with_bias else None, act, dr if with_res else None, item_rows, dsc, dsh, one)
    ctx.dense_fused(dx, M, K, dW, N, db if with_bias else None, act, dr if with_res else None, two)
    ctx.layernorm(two, None, dsc, dsh, two, items, item_rows, N)
    got, sep = one.numpy(), two.numpy()
    assert np.allclose(got, sep, rtol=2e-5, atol=2e-5)
    sample = list(range(items)) if M * N * K <= (1 << 26) else [0, items - 1]
    for i in sample:
        rows = slice(i * item_rows, (i + 1) * item_rows)
        ref = orc.gemm(x[rows], W, False, False)
        if with_bias:
            ref = ref + b
        if act:
            ref = orc.gelu(ref)
        if with_res:
            ref = ref + r[rows]
        ref = orc.layernorm(ref.reshape(1, item_rows, N), scale, shift).reshape(item_rows, N)
        assert_parity(got[rows], ref, "dense + layernorm item %d" % i)
    if with_res:    # the result may alias the residual
        ctx.dense_layernorm(dx, M, K, dW, N, db if with_bias else None, act, dr, item_rows, dsc, dsh, dr)
        assert np.array_equal(dr.numpy(), got)
    for t in (dx, dW, db, dr, dsc, dsh, one, two):
        t.release()


@pytest.mark.parametrize("seed", range(30))
def test_dense_layernorm_random_shapes(ctx, orc, seed):
    """Seeded random item counts, item lengths, widths and epilogue terms (none of them included): whichever route the call
    takes - sums from the epilogue, or the two separate calls - the result is within the gate of the oracle's sequence."""
    rng = np.random.default_rng(90000 + seed)
    items, item_rows = int(rng.integers(1, 6)), int(rng.choice([1, 3, 32, 64, 100, 128, 256]))
    K, N = int(rng.choice([4, 64, 100, 256])), int(rng.choice([4, 8, 64, 132, 256, 512]))
    M = items * item_rows
    x = rng.standard_normal((M, K)).astype(np.float32)
    W = (rng.standard_normal((K, N)) * 0.2).astype(np.float32)
    bias, res = rng.standard_normal(N).astype(np.float32), rng.standard_normal((M, N)).astype(np.float32)
    scale, shift = (1 + 0.1 * rng.standard_normal(N)).astype(np.float32), (0.1 * rng.standard_normal(N)).astype(np.float32)
    act, with_bias, with_res = int(rng.integers(0, 2)), bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    dev = [ctx.to_device(a) for a in (x, W, bias, res, scale, shift)]
    y = ctx.empty((M, N))
    ctx.dense_layernorm(dev[0], M, K, dev[1], N, dev[2] if with_bias else None, act, dev[3] if with_res else None, item_rows, dev[4], dev[5], y)
    ref = orc.gemm(x, W, False, False)
    if with_bias:
        ref = ref + bias
    if act:
        ref = orc.gelu(ref)
    if with_res:
        ref = ref + res
    ref = orc.layernorm(ref.reshape(items, item_rows, N), scale, shift).reshape(M, N)
    assert_parity(y.numpy(), ref, "seed %d: items %d x %d rows, K %d, N %d, act %d bias %s residual %s" % (seed, items, item_rows, K, N, act, with_bias, with_res))
    for t in dev + [y]:
        t.release()


def test_dense_fused_errors(ctx):
    from dl4s_amd import lib
    a = ctx.empty((4, 4))
    with pytest.raises(lib.Dl4sHipError):
        ctx.dense_fused(a, 4, 4, a, 4, None, 7, None, a)
    with pytest.raises(lib.Dl4sHipError):
        ctx.dense_fused(a, -1, 4, a, 4, None, 0, None, a)
    a.release()


@pytest.mark.parametrize("nbuf,count", [(1, 5), (3, 1000), (70, 333), (130, 64), (65, 4099)])
def test_stack_many_buffers(ctx, nbuf, count):
    """Tensor(stacking:) along axis 0 (Tensor/Operators/Stack.swift:79-98): more buffers than one launch carries, counts
    that are not multiples of four, sources at unaligned offsets."""
    rng = np.random.default_rng(nbuf * 100 + count)
    parts = [rng.standard_normal(count + 1).astype(np.float32) for _ in range(nbuf)]
    dev = [ctx.to_device(p) for p in parts]
    dst = ctx.empty((nbuf, count))
    srcs = [d.offset(4) if i % 2 else d for i, d in enumerate(dev)]      # every other source starts one float in
    ctx.stack(srcs, count, dst)
    ref = np.stack([p[1:count + 1] if i % 2 else p[:count] for i, p in enumerate(parts)])
    assert np.array_equal(dst.numpy(), ref)
    for d in dev + [dst]:
        d.release()


@pytest.mark.parametrize("seed", range(40))
def test_gemm_random_shapes_and_forms(ctx, seed):
    """Seeded random extents around the boundaries between the tiled, skinny and scalar-load kernels, every transpose
    combination, alone / batched / grouped, against an fp64 product (the bound scales with the size of the sums)."""
    rng = np.random.default_rng(7000 + seed)
    pick = lambda: int(rng.choice([1, 3, 4, 8, 31, 32, 33, 64, 100, 128, 129, 260, 512, 1000]))
    M, N, K = pick(), pick(), int(rng.choice([1, 4, 6, 60, 64, 68, 100, 256, 516, 1028, 2048]))
    ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    form = ["single", "batched", "grouped"][int(rng.integers(0, 3))]
    count = 1 if form == "single" else int(rng.integers(2, 5))
    As = [(rng.standard_normal((K, M) if ta else (M, K))).astype(np.float32) for _ in range(count)]
    Bs = [(rng.standard_normal((N, K) if tb else (K, N)) * 0.1).astype(np.float32) for _ in range(count)]
    what = "seed %d: M%d N%d K%d ta%d tb%d %s x%d" % (seed, M, N, K, ta, tb, form, count)
    refs = [(a.T if ta else a).astype(np.float64) @ (b.T if tb else b).astype(np.float64) for a, b in zip(As, Bs)]
    outs = [ctx.empty((M, N)) for _ in range(count)]
    keep = []
    if form == "batched":
        dA, dB, dC = ctx.to_device(np.stack(As)), ctx.to_device(np.stack(Bs)), ctx.empty((count, M, N))
        keep = [dA, dB, dC]
        ctx.gemm_batched(dA, As[0].shape, As[0].size, dB, Bs[0].shape, Bs[0].size, dC, M * N, count, 1.0, 0.0, ta, tb)
        got = list(dC.numpy())
    else:
        dA, dB = [ctx.to_device(a) for a in As], [ctx.to_device(b) for b in Bs]
        keep = dA + dB
        if form == "grouped":
            ctx.gemm_grouped(dA, As[0].shape, dB, Bs[0].shape, outs, 1.0, 0.0, ta, tb)
        else:
            ctx.gemm(dA[0], As[0].shape, dB[0], Bs[0].shape, outs[0], 1.0, 0.0, ta, tb)
        got = [o.numpy() for o in outs]
    for g, r in zip(got, refs):
        bound = 2e-6 * np.sqrt(K) * (np.abs(r).max() + 1.0) + 1e-6
        assert np.abs(g - r).max() <= bound, "%s: max |d| %.3e > %.3e" % (what, np.abs(g - r).max(), bound)
    # every form gives the bits of the single call
    single = ctx.empty((M, N))
    a0, b0 = ctx.to_device(As[-1]), ctx.to_device(Bs[-1])
    ctx.gemm(a0, As[-1].shape, b0, Bs[-1].shape, single, 1.0, 0.0, ta, tb)
    assert np.array_equal(single.numpy(), got[-1]), what
    for x in keep + outs + [single, a0, b0]:
        x.release()
