"""Recorded call sequences (dl4s_hip_graph_*): a replay gives the bits of the same calls issued one by one, on every
replay, with other work and waits between the replays and with new data in the recorded buffers; calls that cannot be
recorded are refused without breaking the recording."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

B, L, D, H = 4, 64, 512, 8
HD = D // H


@pytest.fixture()
def ctx():
    from dl4s_amd import lib
    if not lib.graph_supported():
        pytest.skip("graph launches abort the queue under rocprofv3")
    c = lib.Context(0)
    yield c
    c.close()


def _attention_layer(ctx, lib, bufs):
    """One multi-head attention layer on fixed buffers: three projections in one launch, fused attention under a causal
    mask tensor (the mask classifier uses the library's scratch block), the output product with its residual, the joint
    layer norm, then a product with few rows and a long inner dimension (partial sums in the scratch block) and a copy."""
    x, wq, wk, wv, wfc, scale, shift, mask = (bufs[n] for n in ("x", "wq", "wk", "wv", "wfc", "scale", "shift", "mask"))
    ctx.gemm_grouped([x, x, x], (B * L, D), [wq, wk, wv], (D, D), [bufs["q"], bufs["k"], bufs["v"]])
    m = ctx.mask_desc(lib.MASK_DENSE, dense=mask)
    ctx.sdpa_fwd(bufs["q"], bufs["k"], bufs["v"], bufs["att"], B, H, L, L, HD, HD, 1.0 / np.sqrt(HD), mask=m,
                 flags=lib.SDPA_TOKEN_MAJOR)
    ctx.dense_fused(bufs["att"], B * L, D, wfc, D, None, lib.ACT_NONE, x, bufs["fc"])
    ctx.layernorm(bufs["fc"], None, scale, shift, bufs["ln"], B, L, D)
    ctx.gemm(bufs["ln"], (B, L * D), bufs["wlong"], (L * D, 96), bufs["head"])
    lib._check(ctx.lib.dl4s_hip_assign_d2d(ctx.handle, C.c_void_p(bufs["copy"].ptr), C.c_void_p(bufs["head"].ptr),
                                           C.c_size_t(B * 96 * 4)))


def _buffers(ctx, rng):
    r = lambda *s: ctx.to_device((rng.standard_normal(s) * 0.1).astype(np.float32))
    bufs = {"x": r(B * L, D), "wq": r(D, D), "wk": r(D, D), "wv": r(D, D), "wfc": r(D, D), "scale": r(L, D),
            "shift": r(L, D), "wlong": r(L * D, 96),
            "mask": ctx.to_device(np.triu(np.ones((L, L), np.float32), 1))}
    for n, shape in (("q", (B * L, D)), ("k", (B * L, D)), ("v", (B * L, D)), ("att", (B * L, D)), ("fc", (B * L, D)),
                     ("ln", (B * L, D)), ("head", (B, 96)), ("copy", (B, 96))):
        bufs[n] = ctx.empty(shape)
    return bufs


OUTPUTS = ("q", "att", "fc", "ln", "head", "copy")


def test_replays_match_the_calls_issued_one_by_one(ctx):
    from dl4s_amd import lib
    rng = np.random.default_rng(5)
    bufs = _buffers(ctx, rng)
    _attention_layer(ctx, lib, bufs)           # sizes the scratch block, and the result to compare with
    want = {n: bufs[n].numpy() for n in OUTPUTS}
    assert np.isfinite(want["copy"]).all() and np.abs(want["copy"]).max() > 0

    ctx.graph_begin()
    _attention_layer(ctx, lib, bufs)
    graph = ctx.graph_end()
    assert graph.nodes >= 7                    # classifier, three products, attention, layer norm, copy at least
    other_a = ctx.to_device(rng.standard_normal((256, 256)).astype(np.float32))
    other_y = ctx.empty((256, 256))
    for replay in range(4):
        for n in OUTPUTS:                      # a replay that did nothing would leave these zeros behind
            ctx.fill(0.0, bufs[n], int(np.prod(bufs[n].shape)))
        ctx.gemm(other_a, (256, 256), other_a, (256, 256), other_y)   # unrelated work between replays
        ctx.sync()
        graph.replay()
        got = {n: bufs[n].numpy() for n in OUTPUTS}
        for n in OUTPUTS:
            assert np.array_equal(got[n], want[n]), (replay, n)

    # the recorded buffers are read at replay time: new input, new result, again equal to the calls issued one by one
    x2 = (rng.standard_normal((B * L, D)) * 0.1).astype(np.float32)
    lib._check(ctx.lib.dl4s_hip_assign_h2d(ctx.handle, C.c_void_p(bufs["x"].ptr), x2.ctypes.data_as(C.c_void_p),
                                           C.c_size_t(x2.nbytes)))
    graph.replay()
    got2 = {n: bufs[n].numpy() for n in OUTPUTS}
    _attention_layer(ctx, lib, bufs)
    want2 = {n: bufs[n].numpy() for n in OUTPUTS}
    for n in OUTPUTS:
        assert np.array_equal(got2[n], want2[n]), n
    assert not np.array_equal(want2["copy"], want["copy"])
    graph.destroy()


def test_calls_that_cannot_be_recorded_are_refused(ctx):
    from dl4s_amd import lib
    a = ctx.to_device(np.arange(1024, dtype=np.float32))
    y = ctx.empty((1024,))
    host = np.zeros(1024, np.float32)
    ctx.graph_begin()
    with pytest.raises(lib.Dl4sHipError, match="being recorded already"):
        ctx.graph_begin()
    for call in (lambda: ctx.sync(), lambda: ctx.timer_begin(), lambda: ctx.argmax(a, 1024), lambda: a.numpy(),
                 lambda: ctx.to_device(host)):
        with pytest.raises(lib.Dl4sHipError, match="cannot be recorded|while a graph is being recorded"):
            call()
    # no pooled block of this size: the allocation would reach the driver
    with pytest.raises(lib.Dl4sHipError, match="while a graph is being recorded"):
        ctx.empty((3 * 1024 * 1024 + 17,))
    ctx.vneg(a, y, 1024)                       # the recording is still open and usable
    graph = ctx.graph_end()
    assert graph.nodes == 1
    ctx.fill(0.0, y, 1024)
    graph.replay()
    assert np.array_equal(y.numpy(), -np.arange(1024, dtype=np.float32))
    graph.destroy()
    with pytest.raises(lib.Dl4sHipError, match="no graph is being recorded"):
        ctx.graph_end()


def test_scratch_growth_is_refused_while_recording_and_outdates_graphs(ctx):
    from dl4s_amd import lib
    rng = np.random.default_rng(6)
    a = ctx.to_device((rng.standard_normal((4, 8192)) * 0.1).astype(np.float32))
    w = ctx.to_device((rng.standard_normal((8192, 64)) * 0.1).astype(np.float32))
    y = ctx.empty((4, 64))
    ctx.graph_begin()
    with pytest.raises(lib.Dl4sHipError, match="run the same calls once before recording"):
        ctx.gemm(a, (4, 8192), w, (8192, 64), y)          # partial sums need scratch that is not there yet
    ctx.graph_end(keep=False)
    ctx.gemm(a, (4, 8192), w, (8192, 64), y)
    want = y.numpy()
    ctx.graph_begin()
    ctx.gemm(a, (4, 8192), w, (8192, 64), y)
    graph = ctx.graph_end()
    ctx.fill(0.0, y, 4 * 64)
    graph.replay()
    assert np.array_equal(y.numpy(), want)
    # a later call that needs a larger scratch block moves it: the graph holds the old address and is refused
    a2 = ctx.to_device((rng.standard_normal((64, 32768)) * 0.1).astype(np.float32))
    w2 = ctx.to_device((rng.standard_normal((32768, 128)) * 0.1).astype(np.float32))
    y2 = ctx.empty((64, 128))
    ctx.gemm(a2, (64, 32768), w2, (32768, 128), y2)
    with pytest.raises(lib.Dl4sHipError, match="regrown"):
        graph.replay()
    graph.destroy()


def test_blocks_freed_while_recording_stay_reserved_for_the_graph(ctx):
    """A recorded sequence may allocate and free its temporaries as usual: the freed blocks serve later allocations of the
    same recording, are kept out of the pool while the graph lives (an allocation made afterwards must not alias what a
    replay overwrites) and return to the pool when the graph is destroyed."""
    n = 4096
    x = ctx.to_device(np.arange(n, dtype=np.float32))
    y = ctx.empty((n,))

    def calls():
        t1 = ctx.empty((n,))
        ctx.vneg(x, t1, n)
        t2 = ctx.empty((n,))
        ctx.vadd(t1, t1, t2, n)
        p1 = t1.ptr
        t1.release()
        t3 = ctx.empty((n,))              # takes the block t1 gave back, inside the recording as outside
        ctx.vmul(t2, t2, t3, n)
        ctx.vadd(t3, x, y, n)
        ptrs = (p1, t2.ptr, t3.ptr)
        t2.release()
        t3.release()
        return ptrs

    eager = calls()
    assert eager[0] == eager[2]
    want = y.numpy()
    assert np.array_equal(want, 4.0 * np.arange(n, dtype=np.float32) ** 2 + np.arange(n, dtype=np.float32))
    used0, pooled0 = ctx.mem_stats()
    ctx.graph_begin()
    rec = calls()
    graph = ctx.graph_end()
    assert rec[0] == rec[2]
    used1, pooled1 = ctx.mem_stats()
    assert used1 == used0 and pooled1 == pooled0 - 2 * n * 4       # two blocks of the pool now belong to the graph
    others = [ctx.empty((n,)) for _ in range(4)]                    # same size class: must come from elsewhere
    assert not {o.ptr for o in others} & set(rec)
    for o in others:
        ctx.fill(7.0, o, n)
    ctx.fill(0.0, y, n)
    graph.replay()
    assert np.array_equal(y.numpy(), want)
    for o in others:
        assert np.array_equal(o.numpy(), np.full(n, 7.0, np.float32))
        o.release()
    graph.destroy()
    _, pooled2 = ctx.mem_stats()
    assert pooled2 >= pooled0                                        # the graph's blocks are back (plus the four others)
