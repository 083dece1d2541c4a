#!/usr/bin/env python3
"""Benchmark of the attention forward hot path on one MI355X.

Headline workload (config.workload): long-context prefill, B=8 H=16 L=2048 d=64, causal mask,
q/k/v = 0.5*N(0,1), fp32 -- the configuration the metric's MFMA target is quoted on.  One step is one
fused attention call over that batch with the inputs already resident in HBM.  The decode workload
(B=16 H=16 d=64, 4096-row cache, 64 append+attend steps) is reported beside it in "decode".

Prints ONE JSON line.  `value` is algorithmic TFLOP/s (4*d flops per unblocked query-key pair) over the
wall time of the K timed steps; roofline.achieved uses the HIP-event time of the same K launches.
cpu_baseline times the CPU oracle (a restatement of the reference's generic CPU engine) on a bounded
sample of the same workload, single-threaded like the reference's engine.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0
# Memory traffic per launch of the two timed kernels on these exact workloads, in bytes: rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE (two separate runs of this script; KiB per dispatch), scaled by what the same counters read for a 1 GiB
# streaming kernel (--copy-calibration: x2.00 and x1.00).  The runs and their figures are summarised in
# profiles/bench_prefill_config4_decode_config5.md; they are constants here because a counter run cannot be part of
# the timed process.
PREFILL_TRAFFIC_BYTES = (407114 * 2.00 + 65536 * 1.00) * 1024      # L2 fills (K/V re-reads included) + writes
DECODE_TRAFFIC_BYTES = (264315 * 2.00 + 192 * 1.00) * 1024
PREHEAT_S = 0.25


def prefill(ctx, lib, steps, warmup):
    B, H, L, d = 8, 16, 2048, 64
    rng = np.random.Generator(np.random.PCG64(1004))
    q, k, v = (rng.standard_normal((B, H, L, d), dtype=np.float32) * np.float32(0.5) for _ in range(3))
    dq, dk, dv = ctx.to_device(q), ctx.to_device(k), ctx.to_device(v)
    out = ctx.empty((B, H, L, d))
    desc = ctx.mask_desc(lib.MASK_CAUSAL)
    flops = 4.0 * d * B * H * (L * (L + 1) // 2)
    # The GPU idled while the inputs were generated and copied, and its clocks need tens of milliseconds of load to
    # come back up: run the workload untimed for PREHEAT_S first, then the W warm-up steps, then time K steps.
    t_end = time.perf_counter() + PREHEAT_S
    while time.perf_counter() < t_end:
        for _ in range(10):
            ctx.sdpa_fwd(dq, dk, dv, out, B, H, L, L, d, d, 0.125, desc, 0)
        ctx.sync()
    for _ in range(warmup):
        ctx.sdpa_fwd(dq, dk, dv, out, B, H, L, L, d, d, 0.125, desc, 0)
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_begin()
    for _ in range(steps):
        ctx.sdpa_fwd(dq, dk, dv, out, B, H, L, L, d, d, 0.125, desc, 0)
    ev_ms = ctx.timer_end()
    ctx.sync()
    wall = time.perf_counter() - t0
    o = out.numpy()
    # The same call with DL4S_SDPA_STRICT: every key tile visited, so that NaN / Inf in K or V at blocked keys reach the
    # output as in the reference (0 x NaN).  Same bits as the default on finite inputs; reported beside the headline.
    strict_out = ctx.empty((B, H, L, d))
    nstrict = max(3, steps // 4)
    for _ in range(3):
        ctx.sdpa_fwd(dq, dk, dv, strict_out, B, H, L, L, d, d, 0.125, desc, lib.SDPA_STRICT)
    ctx.timer_begin()
    for _ in range(nstrict):
        ctx.sdpa_fwd(dq, dk, dv, strict_out, B, H, L, L, d, d, 0.125, desc, lib.SDPA_STRICT)
    strict_ms = ctx.timer_end() / nstrict
    strict_same = bool(np.array_equal(strict_out.numpy(), o))
    strict_out.release()
    if not (np.isfinite(o).all() and np.allclose(o[:, :, 0], v[:, :, 0], atol=1e-6)):
        raise RuntimeError("prefill output failed its sanity check")
    for b in (dq, dk, dv, out):
        b.release()
    return {"flops": flops, "wall_s": wall, "event_ms_per_launch": ev_ms / steps, "strict_ms_per_launch": strict_ms,
            "strict_bit_identical": strict_same,
            "shape": {"B": B, "H": H, "L": L, "d": d}, "inputs": (q, k, v), "output": o}


def decode(ctx, lib, repeats, d=64):
    B, H, T0, steps = 16, 16, 4096, 64
    rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
    Tcap = T0 + steps
    rng = np.random.Generator(np.random.PCG64(1005))
    kc = ctx.to_device(rng.standard_normal((B, H, Tcap, d), dtype=np.float32))
    vc = ctx.to_device(rng.standard_normal((B, H, Tcap, d), dtype=np.float32))
    qs = ctx.to_device(rng.standard_normal((steps, B, H, 1, d), dtype=np.float32))
    kn = ctx.to_device(rng.standard_normal((steps, B, H, 1, d), dtype=np.float32))
    vn = ctx.to_device(rng.standard_normal((steps, B, H, 1, d), dtype=np.float32))
    out = ctx.empty((steps, B, H, 1, d))
    sb = B * H * d * 4

    def run():
        for t in range(steps):
            ctx.sdpa_decode_step(qs.offset(t * sb), kc, vc, kn.offset(t * sb), vn.offset(t * sb), out.offset(t * sb),
                                 B, H, T0 + t, Tcap, d, rT)
    t_end = time.perf_counter() + PREHEAT_S
    while time.perf_counter() < t_end:      # clocks back up after the idle time spent filling the cache
        run()
        ctx.sync()
    per_step_us = []
    for _ in range(repeats):
        ctx.timer_begin()
        run()
        per_step_us.append(ctx.timer_end() * 1e3 / steps)
    # the distribution over single steps: every step of one more pass bracketed by its own pair of events
    single_us = []
    for t in range(steps):
        ctx.timer_begin()
        ctx.sdpa_decode_step(qs.offset(t * sb), kc, vc, kn.offset(t * sb), vn.offset(t * sb), out.offset(t * sb),
                             B, H, T0 + t, Tcap, d, rT)
        single_us.append(ctx.timer_end() * 1e3)
    o = out.numpy()
    if not np.isfinite(o).all():
        raise RuntimeError("decode output failed its sanity check")
    for b in (kc, vc, qs, kn, vn, out):
        b.release()
    us = float(np.median(per_step_us))
    # algorithmic bytes per step: K and V rows 0..T-1 read once, q read, out written, the new k/v row written
    Tavg = T0 + (steps + 1) / 2.0
    bytes_step = 2 * B * H * Tavg * d * 4 + 2 * B * H * d * 4 + 2 * B * H * d * 4
    return {"us_per_step": us, "us_per_step_min": float(np.min(per_step_us)), "tokens_per_s": B / (us * 1e-6),
            "single_step_us_p50": float(np.percentile(single_us, 50)), "single_step_us_p99": float(np.percentile(single_us, 99)),
            "bytes_per_step": bytes_step, "gbs": bytes_step / (us * 1e-6) / 1e9,
            "shape": {"B": B, "H": H, "d": d, "T0": T0, "steps": steps}}


def under_rocprof():
    """rocprofv3's queue interception aborts the queue on a HIP graph launch (HSA_STATUS_ERROR_INVALID_PACKET_FORMAT) and
    then does not exit: the sections that replay recorded calls are left out when the process runs under it."""
    from dl4s_amd import lib
    return not lib.graph_supported()


# What a DL4S checkout has to contain for each host mode of the layer rows (the Swift sources and patches under swift/).
PATCH_SETS = {
    "primitive": "HIP.swift + module map + Package.swift.patch: the reference's engine calls one by one",
    "attention_hook_only": "primitive + Engine.swift.patch + HIPFusedAttention.swift + ScaledDotProductAttention.swift.patch",
    "fused": "attention_hook_only + HIPFusedLayers.swift + MultiHeadAttention.swift.patch + PointwiseFeedForward.swift.patch, "
             "HIP.fusedLayers = true (forward only)",
    "fused_strict": "fused with HIP.strictMasks = true: every key tile visited, LayerNorm sums in the reference's order",
}


def other_configs(ctx, lib, cpu, only=None):
    """Configs 1-3 of the baseline: us/call, TFLOP/s on the algorithmic flops, fraction of the fp32 MFMA peak; the
    CPU oracle beside each (whole call for configs 1 and 2, one batch item of config 3), single thread."""
    from dl4s_amd import host_lib
    from oracle import fp64_model as m64
    if cpu:
        from oracle import binding as orc
    res = {}
    want = lambda name: only is None or name in only
    if want("config1"):
        # config 1: SDPA B1 H8 L128 d64, no mask
        rng = np.random.Generator(np.random.PCG64(1001))
        q, k, v = (rng.standard_normal((1, 8, 128, 64), dtype=np.float32) for _ in range(3))
        dq, dk, dv, out = ctx.to_device(q), ctx.to_device(k), ctx.to_device(v), ctx.empty((1, 8, 128, 64))
        for _ in range(5):
            ctx.sdpa_fwd(dq, dk, dv, out, 1, 8, 128, 128, 64, 64, 0.125, None, 0)
        ctx.sync()
        ctx.timer_begin()
        for _ in range(200):
            ctx.sdpa_fwd(dq, dk, dv, out, 1, 8, 128, 128, 64, 64, 0.125, None, 0)
        us = ctx.timer_end() * 1e3 / 200
        fl = 4.0 * 64 * 8 * 128 * 128
        res["config1_sdpa_B1_H8_L128_d64"] = {"us_per_call": us, "tflops": fl / us / 1e6, "frac_mfma_peak": fl / us / 1e6 / MFMA_FP32_PEAK_TFLOPS,
                                              "flops": fl, "note": "launch-latency bound (33.6 MFLOP)"}
        for b in (dq, dk, dv, out):
            b.release()
        if cpu:
            from oracle import binding as orc
            t0 = time.perf_counter()
            orc.sdpa(q, k, v, None)
            dt = time.perf_counter() - t0
            res["config1_sdpa_B1_H8_L128_d64"]["cpu_baseline"] = {"us_per_call": dt * 1e6, "tflops": fl / dt / 1e12, "cores": 1, "kind": "port"}
    if want("config2") or (only is not None and "config2_fused_only" in only):
        # config 2: MHA layer B4 L512 D512 H8 causal (dense mask tensor, as the layer receives it; "config2_fused_only": that
        # host mode alone)
        B, L, D, H, dk_ = 4, 512, 512, 8, 64
        rng = np.random.Generator(np.random.PCG64(1002))
        x = rng.standard_normal((B, L, D), dtype=np.float32)
        attn, _ = m64.make_params(rng, D, H, dk_, dk_, 8, trivial_affine=True)
        i, j = np.indices((L, L))
        mask = (j > i).astype(np.float32)
        fl = 4.0 * 64 * B * H * (L * (L + 1) // 2) + 4 * 2.0 * B * L * D * D
        # fused: tiles the mask blocks entirely are skipped; fused_strict: every tile visited (NaN / Inf at blocked keys as in
        # the reference); primitive: the reference's engine calls one by one; attention_hook_only: the primitive layer with the
        # one fused call inside ScaledDotProductAttention (a DL4S checkout with the five-line hook and nothing else)
        for mode, fused in (("fused", 1), ("fused_strict", 2), ("primitive", 0), ("attention_hook_only", 3)):
            if not want("config2") and mode != "fused":
                continue
            quick = fused in (1, 2)
            # the harness runs as many untimed calls as timed ones first (0.04 - 0.1 s: the clocks are up when the timer starts)
            _, ms = host_lib.mha(ctx, x, x, x, mask, attn, H, dk_, dk_, fused=fused, iters=1000 if quick else (300 if fused else 60))
            res["config2_mha_B4_L512_D512_H8_causal_" + mode] = {"us_per_call": ms * 1e3, "tflops": fl / ms / 1e9,
                                                                "frac_mfma_peak": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS, "flops": fl,
                                                                "swift_patch_set": PATCH_SETS[mode]}
        if cpu and want("config2"):
            t0 = time.perf_counter()
            orc.mha(x, x, x, mask, attn, H, dk_, dk_)
            dt = time.perf_counter() - t0
            res["config2_mha_B4_L512_D512_H8_causal_fused"]["cpu_baseline"] = {"us_per_call": dt * 1e6, "tflops": fl / dt / 1e12, "cores": 1, "kind": "port"}
    if want("recorded") and under_rocprof():
        res["recorded"] = "skipped under rocprofv3 (graph launches abort its intercepted queue)"
    elif want("recorded"):
        # Calls recorded into a HIP graph and replayed, against the same calls issued one by one.
        B, L, D, H, dk_ = 4, 512, 512, 8, 64
        rng = np.random.Generator(np.random.PCG64(1012))
        x = rng.standard_normal((B, L, D), dtype=np.float32)
        i, j = np.indices((L, L))
        mask = (j > i).astype(np.float32)
        fl = 4.0 * 64 * B * H * (L * (L + 1) // 2) + 4 * 2.0 * B * L * D * D
        # config 2's fused layer (projections in one launch, attention, output product + residual + layer norm) on
        # fixed buffers through the C ABI: issued one by one, and recorded once into a graph and replayed
        r = lambda *sh: ctx.to_device(rng.standard_normal(sh, dtype=np.float32) * np.float32(0.05))
        dx, dmask, w4 = ctx.to_device(x.reshape(B * L, D)), ctx.to_device(mask), [r(D, D) for _ in range(4)]
        dscale, dshift = r(L, D), r(L, D)
        t = [ctx.empty((B * L, D)) for _ in range(6)]
        md = ctx.mask_desc(lib.MASK_DENSE, dense=dmask)

        def layer_calls():
            ctx.gemm_grouped([dx, dx, dx], (B * L, D), w4[:3], (D, D), t[:3])
            ctx.sdpa_fwd(t[0], t[1], t[2], t[3], B, H, L, L, dk_, dk_, 0.125, mask=md, flags=lib.SDPA_TOKEN_MAJOR)
            ctx.dense_layernorm(t[3], B * L, D, w4[3], D, None, lib.ACT_NONE, dx, L, dscale, dshift, t[5])

        def timed(fn, n):
            for _ in range(n * 10):
                fn()
            ctx.sync()
            ctx.timer_begin()
            for _ in range(n):
                fn()
            return ctx.timer_end() / n

        ms_calls = timed(layer_calls, 100)
        y_calls = t[5].numpy()
        # the same calls with the mask handed over as a causal descriptor (what the host layer's model-level API does)
        # instead of the [L, L] tensor: no tile classification launch, no mask reads
        md_dense, md = md, ctx.mask_desc(lib.MASK_CAUSAL)
        ms_desc = timed(layer_calls, 100)
        same_desc = bool(np.array_equal(t[5].numpy(), y_calls))
        md = md_dense
        ctx.graph_begin()
        layer_calls()
        graph = ctx.graph_end()
        ctx.fill(0.0, t[5], B * L * D)
        ms_graph = timed(graph.replay, 100)
        same = bool(np.array_equal(t[5].numpy(), y_calls))
        res["config2_mha_B4_L512_D512_H8_causal_c_abi_calls_recorded"] = {
            "us_per_call_issued_one_by_one": ms_calls * 1e3, "us_per_call_replayed": ms_graph * 1e3, "graph_nodes": graph.nodes,
            "replay_equals_calls_bitwise": same, "us_per_call_with_causal_descriptor": ms_desc * 1e3,
            "causal_descriptor_equals_mask_tensor_bitwise": same_desc, "tflops": fl / ms_graph / 1e9,
            "frac_mfma_peak": fl / ms_graph / 1e9 / MFMA_FP32_PEAK_TFLOPS, "flops": fl}
        graph.destroy()
        for b_ in [dx, dmask, dscale, dshift] + w4 + t:
            b_.release()
        # a chain of 32 dependent element-wise calls on 4096 floats: nothing but launch latency
        n = 4096
        a_, b_ = ctx.empty((n,)), ctx.empty((n,))
        ctx.fill(1.0, a_, n)
        ctx.fill(0.0, b_, n)

        def chain():
            for _ in range(16):
                ctx.vadd(a_, b_, b_, n)
                ctx.vmul(a_, b_, b_, n)

        ms_calls = timed(chain, 50)
        ctx.graph_begin()
        chain()
        graph = ctx.graph_end()
        ms_graph = timed(graph.replay, 50)
        res["chain_of_32_dependent_small_kernels_recorded"] = {
            "us_per_kernel_issued_one_by_one": ms_calls * 1e3 / 32, "us_per_kernel_replayed": ms_graph * 1e3 / 32,
            "graph_nodes": graph.nodes}
        graph.destroy()
        a_.release()
        b_.release()
    if want("config3") or (only is not None and "config3_hook_only" in only):
        # config 3: encoder block B8 L1024 D1024 H16 F4096, key-length mask ("config3_hook_only": that host mode alone)
        B, L, D, H, F = 8, 1024, 1024, 16, 4096
        rng = np.random.Generator(np.random.PCG64(1003))
        x = rng.standard_normal((B, L, D), dtype=np.float32)
        attn, ffn = m64.make_params(rng, D, H, 64, 64, F, trivial_affine=True)
        lens = rng.integers(512, 1025, size=B)
        mask = (np.arange(L)[None, None, None, :] >= lens[:, None, None, None]).astype(np.float32)
        fl = 4.0 * 64 * H * L * float(lens.sum()) + 4 * 2.0 * B * L * D * D + 2 * 2.0 * B * L * D * F
        for mode, fused in (("fused", 1), ("fused_strict", 2), ("attention_hook_only", 3)):
            if not want("config3") and mode != "attention_hook_only":
                continue
            # the harness runs as many untimed calls as timed ones first (about 0.1 s: the clocks are up when the timer starts)
            _, ms = host_lib.encoder_block(ctx, x, mask, attn, ffn, H, 64, 64, fused=fused, iters=50 if fused < 3 else 30)
            res["config3_encoder_block_B8_L1024_D1024_H16_F4096_" + mode] = {"us_per_call": ms * 1e3, "tflops": fl / ms / 1e9,
                                                                             "frac_mfma_peak": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS, "flops": fl,
                                                                             "swift_patch_set": PATCH_SETS[mode]}
        if cpu and want("config3"):
            t0 = time.perf_counter()
            orc.encoder_block(x[:1, :256], mask[:1, :, :, :256], attn, ffn, H, 64, 64)
            dt = time.perf_counter() - t0
            fl1 = 4.0 * 64 * H * 256 * min(int(lens[0]), 256) + 4 * 2.0 * 256 * D * D + 2 * 2.0 * 256 * D * F
            res["config3_encoder_block_B8_L1024_D1024_H16_F4096_fused"]["cpu_baseline"] = {
                "tflops": fl1 / dt / 1e12, "cores": 1, "kind": "port",
                "sample": "one batch item cut to 256 tokens (%.1f s); extrapolated whole call %.0f s" % (dt, dt * fl / fl1)}
    if want("backward"):
        # gradients of the headline workload (config 4 shapes): forward with row statistics, then dq, dk, dv; head dim 64
        # (the 64-wide kernels), 128, 96 and 32 (the 128-, 96- and 32-wide ones)
        B, H, L = 8, 16, 2048
        rng = np.random.Generator(np.random.PCG64(1004))
        for d in (64, 128, 96, 32, 256):
            bufs = [ctx.to_device(rng.standard_normal((B, H, L, d), dtype=np.float32) * np.float32(0.5)) for _ in range(4)]
            outs = [ctx.empty((B, H, L, d)) for _ in range(4)]
            st = ctx.empty((B, H, L, 2))
            desc = ctx.mask_desc(lib.MASK_CAUSAL)
            rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
            ctx.sdpa_fwd_stats(bufs[0], bufs[1], bufs[2], outs[0], st, B, H, L, L, d, rT, desc, 0)
            bwd = lambda: ctx.sdpa_bwd(bufs[0], bufs[1], bufs[2], outs[0], st, bufs[3], outs[1], outs[2], outs[3], B, H, L, L, d, rT, desc, 0)
            reps = 20 if d <= 128 else 5
            for _ in range(reps):
                bwd()
            ctx.sync()
            ctx.timer_begin()
            for _ in range(reps):
                bwd()
            ms = ctx.timer_end() / reps
            fl = 10.0 * d * B * H * (L * (L + 1) // 2)          # five products: the recomputed scores, dp, dv, dk, dq
            name = "config4_attention_backward_B8_H16_L2048_causal" + ("" if d == 64 else "_head_dim_%d" % d)
            res[name] = {
                "us_per_call": ms * 1e3, "tflops": fl / ms / 1e9, "frac_mfma_peak": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS, "flops": fl,
                "note": ("algorithmic flops = the 5 products, which is what the two deterministic kernels issue: the dK/dV kernel "
                         "stores its dS tiles (2 GiB scratch from the pool at this shape) and the dQ kernel contracts them with K")
                        if d <= 128 else
                        "head dims above 128: the five products as batched GEMMs around one elementwise pass, the tiles "
                        "beyond the diagonal left out under the causal mask; TFLOP/s on the algorithmic flops"}
            if cpu and d == 64:
                from oracle import binding as orc
                hq, hk, hv, hg = (b_.numpy()[:1, :2] for b_ in bufs)
                i, j = np.indices((L, L))
                t0 = time.perf_counter()
                orc.sdpa_backward(hq, hk, hv, (j > i).astype(np.float32), hg)
                dt = time.perf_counter() - t0
                res[name]["cpu_baseline"] = {
                    "tflops": fl * 2 / (B * H) / dt / 1e12, "cores": 1, "kind": "port",
                    "sample": "2 of 128 (batch, head) slices, dense causal mask (%.1f s)" % dt}
            for b_ in bufs + outs + [st]:
                b_.release()
    if want("masks_and_head_dim"):
        # the headline shape with the mask as an unmodified DL4S passes it (a dense [L,L] tensor): all-ones tiles skipped
        # (default) and every tile visited (DL4S_SDPA_STRICT); the same shape with the causal descriptor at other head dims:
        # 128 (128-wide tiles), 96, 80 and 70 (96-wide tiles, their 80-column form for the latter two; 70 is staged with 64-bit accesses, no padded copies), 32 and 16
        # (32- and 16-wide tiles), 192 and 256 (192- and 256-wide tiles).  TFLOP/s on each shape's own flops.
        B, H, L = 8, 16, 2048
        rng = np.random.Generator(np.random.PCG64(1008))
        i, j = np.indices((L, L))
        dmask = ctx.to_device((j > i).astype(np.float32))
        for d, name in ((64, "config4_shape_dense_causal_mask_tensor"), (128, "config4_shape_head_dim_128_causal"),
                        (96, "config4_shape_head_dim_96_causal"), (80, "config4_shape_head_dim_80_causal"), (70, "config4_shape_head_dim_70_causal"),
                        (48, "config4_shape_head_dim_48_causal"), (32, "config4_shape_head_dim_32_causal"), (16, "config4_shape_head_dim_16_causal"),
                        (192, "config4_shape_head_dim_192_causal"), (256, "config4_shape_head_dim_256_causal")):
            qkv = [ctx.to_device(rng.standard_normal((B, H, L, d), dtype=np.float32) * np.float32(0.5)) for _ in range(3)]
            o = ctx.empty((B, H, L, d))
            rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
            fl = 4.0 * d * B * H * (L * (L + 1) // 2)
            entry = {"flops": fl}
            keep = []
            if d == 64:
                # the tensor as it is (classified on every call), with its tile classes prepared once, and looked at once
                # by dl4s_hip_mask_describe_f32 (what the Swift hook and the host layer do per mask tensor: it is recognised
                # as the causal kind); then every tile visited
                plain, prepared = ctx.mask_desc(lib.MASK_DENSE, dense=dmask), ctx.mask_desc(lib.MASK_DENSE, dense=dmask)
                keep.append(ctx.mask_classify(prepared, B, H, L, L))
                described, lengths = ctx.mask_describe(plain, B, H, L, L)
                keep.append(lengths)
                entry["described_as_kind"] = int(described.kind)
                variants = (("tile_skipping", plain, 0), ("tile_skipping_classes_prepared_once", prepared, 0),
                            ("tile_skipping_described_once", described, 0), ("strict", plain, lib.SDPA_STRICT))
            else:
                variants = (("causal_descriptor", ctx.mask_desc(lib.MASK_CAUSAL), 0),)
            for vname, desc, flags in variants:
                for _ in range(100):
                    ctx.sdpa_fwd(qkv[0], qkv[1], qkv[2], o, B, H, L, L, d, d, rT, desc, flags)
                ctx.sync()
                ctx.timer_begin()
                for _ in range(30):
                    ctx.sdpa_fwd(qkv[0], qkv[1], qkv[2], o, B, H, L, L, d, d, rT, desc, flags)
                ms = ctx.timer_end() / 30
                entry[vname] = {"us_per_call": ms * 1e3, "tflops": fl / ms / 1e9, "frac_mfma_peak": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS}
            res[name] = entry
            for b_ in qkv + [o] + keep:
                b_.release()
        dmask.release()
    if want("decode_head_dims"):
        # config 5's decode (B16 H16, 4096 cached rows + 64 steps) with cache rows of 128, 96 and 32 floats
        for d in (128, 96, 32):
            dec = decode(ctx, lib, 3, d)
            res["config5_shape_decode_head_dim_%d" % d] = {"us_per_step": dec["us_per_step"], "gbs": dec["gbs"], "frac_hbm_peak": dec["gbs"] / HBM_PEAK_GBS,
                                                            "bytes_per_step": dec["bytes_per_step"]}
    if want("greedy") or want("greedy_fused") or want("greedy_primitive") or want("greedy_cached") or want("greedy_cached_only"):
        # the caller of the blocks: Transformer greedy decoding (batch 1; every step re-runs the decoder on the prefix, as the
        # reference does).  6 + 6 layers, hidden 512, 8 heads of 64, ffn 2048, vocabulary 8000, 64 source tokens, 32 generated.
        rng = np.random.Generator(np.random.PCG64(1006))
        params = m64.make_transformer_params(rng, 8000, 512, 8, 64, 64, 2048, 6, 6)
        src = [int(t) for t in rng.integers(0, 8000, 64)]
        model = host_lib.Transformer(ctx, params)
        entry = {"workload": "Transformer greedy decode, 6+6 layers, hidden 512, 8 heads x 64, ffn 2048, vocab 8000, 64 source tokens, "
                             "32 generated tokens (prefix re-run every step)"}
        for mode, fused in (("fused", True), ("primitive", False)):
            if not (want("greedy") or want("greedy_" + mode)):
                continue
            model.greedy(src, 1, -5, 4, fused=fused)                       # warm the allocator pool
            toks, ms = model.greedy(src, 1, -5, 32, fused=fused, timing=True)
            entry["ms_per_token_" + mode] = ms / len(toks)
            entry["tokens_per_s_" + mode] = len(toks) / ms * 1e3
        if only is not None and "greedy_cached_only" in only:
            # the cached decode of 512 tokens alone, its calls issued one by one (for a kernel trace of just that loop)
            model.set_norm_per_token(True)
            model.greedy(src, 1, -5, 4, cached="stepwise")
            toks_c, ms_c = model.greedy(src, 1, -5, 512, cached="stepwise", timing=True)
            entry["per_token_normalisation"] = {"512_tokens": {"cached_calls_issued_one_by_one": ms_c / len(toks_c)}}
            model.set_norm_per_token(False)
        if want("greedy") or want("greedy_cached"):
            # The same model with per-token normalisation in its attention layers (not the reference's model: its joint
            # normalisation cannot be cached), decoded by re-running the prefix and with key / value caches, 32 and 512 tokens.
            model.set_norm_per_token(True)
            replay = "stepwise" if under_rocprof() else True
            model.greedy(src, 1, -5, 4, cached=replay)
            per_token = {"note": "attention layers normalise per token (not the reference's model); ms per generated token"}
            for count in (32, 512):
                toks_r, ms_r = model.greedy(src, 1, -5, count, timing=True)
                toks_c, ms_c = model.greedy(src, 1, -5, count, cached=replay, timing=True)
                toks_s, ms_s = model.greedy(src, 1, -5, count, cached="stepwise", timing=True)
                per_token["%d_tokens" % count] = {"prefix_rerun": ms_r / len(toks_r), "cached_step_recorded_and_replayed": ms_c / len(toks_c),
                                                  "cached_calls_issued_one_by_one": ms_s / len(toks_s),
                                                  "same_tokens": toks_r == toks_c == toks_s}
            entry["per_token_normalisation"] = per_token
            model.set_norm_per_token(False)
        model.close()
        if cpu:
            from oracle import transformer as orc_t
            t0 = time.perf_counter()
            n_cpu = len(orc_t.greedy_decode(params, src, 1, -5, 4))
            dt = time.perf_counter() - t0
            entry["cpu_baseline"] = {"ms_per_token": dt * 1e3 / n_cpu, "cores": 1, "kind": "port",
                                     "sample": "encoder pass + the first %d generated tokens (%.1f s)" % (n_cpu, dt)}
        res["transformer_greedy_decode"] = entry
    return res


def cpu_baseline_decode(steps_sample=1):
    """One decode step (B16 H16 d64, T=4097) on the CPU oracle, single thread."""
    from oracle import binding as orc
    B, H, d, T = 16, 16, 64, 4097
    rng = np.random.Generator(np.random.PCG64(1005))
    kc = rng.standard_normal((B, H, T, d), dtype=np.float32)
    vc = rng.standard_normal((B, H, T, d), dtype=np.float32)
    q = rng.standard_normal((B, H, 1, d), dtype=np.float32)
    t0 = time.perf_counter()
    for _ in range(steps_sample):
        orc.sdpa_decode(q, kc, vc, T)
    dt = (time.perf_counter() - t0) / steps_sample
    return {"us_per_step": dt * 1e6, "tokens_per_s": B / dt, "cores": 1, "kind": "port", "sample": "%d whole step(s) at T=4097" % steps_sample}


def cpu_baseline_prefill(q, k, v, pairs, gpu_out=None):
    """The CPU oracle timed on `pairs` (batch, head) slices of the headline workload, single thread; its results also
    check the GPU output of the same slices (raw maxima of the absolute and the relative difference)."""
    from oracle import binding as orc
    L, d = q.shape[2], q.shape[3]
    i, j = np.indices((L, L))
    mask = (j > i).astype(np.float32)
    orc.lib()
    dt, max_abs, max_ref = 0.0, 0.0, 0.0
    for p in range(pairs):
        b, h = divmod(p, q.shape[1])
        t0 = time.perf_counter()
        ref = orc.sdpa(q[b:b + 1, h:h + 1], k[b:b + 1, h:h + 1], v[b:b + 1, h:h + 1], mask)
        dt += time.perf_counter() - t0
        if gpu_out is not None:
            diff = np.abs(gpu_out[b:b + 1, h:h + 1].astype(np.float64) - ref.astype(np.float64))
            if not (diff <= 1e-4 + 1e-4 * np.abs(ref)).all():
                raise RuntimeError("prefill output differs from the CPU oracle on slice (%d, %d): max |d| = %g" % (b, h, diff.max()))
            max_abs = max(max_abs, float(diff.max()))
            max_ref = max(max_ref, float(np.abs(ref).max()))
    flops = 4.0 * d * pairs * (L * (L + 1) // 2)
    parity = {} if gpu_out is None else {"parity": {"gate": "|gpu - oracle| <= 1e-4 + 1e-4 |oracle| on every element of the sample",
                                                    "max_abs_diff": max_abs, "max_abs_oracle": max_ref,
                                                    "max_abs_diff_over_max_abs_oracle": max_abs / max(max_ref, 1e-30)}}
    return {**parity, "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": "%d of %d (batch, head) slices of the headline workload (L=%d, d=%d, dense causal mask), "
                      "%.1f s of single-thread CPU time; host has %d cores" % (pairs, q.shape[0] * q.shape[1], L, d, dt,
                                                                             os.cpu_count() or 0)}


def cpu_blas_proxy_prefill(q, k, v, pairs):
    """The same materialised-score structure with the products handed to the host's threaded BLAS (numpy): a stand-in for
    the reference built against MKL (-DMKL_ENABLE), NOT the reference binary and not the parity oracle."""
    L, d = q.shape[2], q.shape[3]
    i, j = np.indices((L, L))
    pen = (j > i).astype(np.float32) * np.float32(1e9)
    t0 = time.perf_counter()
    for p in range(pairs):
        b, h = divmod(p, q.shape[1])
        s = (q[b, h] * np.float32(0.125)) @ k[b, h].T - pen
        s -= s.max(axis=1, keepdims=True)
        np.exp(s, out=s)
        s *= np.float32(1.0) / s.sum(axis=1, keepdims=True)
        s @ v[b, h]
    dt = time.perf_counter() - t0
    flops = 4.0 * d * pairs * (L * (L + 1) // 2)
    return {"value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": os.cpu_count() or 0, "kind": "proxy (numpy + threaded BLAS)",
            "sample": "%d (batch, head) slices, %.1f s" % (pairs, dt)}


def kernel_sample(ctx, lib, iters):
    """A short fixed sequence of the kernels behind configs 3 and 4 that the headline run does not time one by one (the
    fused Dense products, the dense-mask attention of config 3, the attention gradients, forward and gradients at head dims
    128, 96, 32, 256, 80, 48 and 16), `iters` launches each, for
    counter runs of a profiler: no pre-heat loops, a few dozen launches in all.  Returns the mean event time of each."""
    rng = np.random.Generator(np.random.PCG64(1007))
    res = {}

    def timed(name, fn):
        fn()
        ctx.sync()
        ctx.timer_begin()
        for _ in range(iters):
            fn()
        res[name] = {"us_per_launch": ctx.timer_end() * 1e3 / iters}
    M, D, F = 8192, 1024, 4096
    x, h = ctx.to_device(rng.standard_normal((M, D), dtype=np.float32)), ctx.empty((M, F))
    w1, w2 = ctx.to_device(rng.standard_normal((D, F), dtype=np.float32) * 0.03), ctx.to_device(rng.standard_normal((F, D), dtype=np.float32) * 0.03)
    wq, b1, b2, y = ctx.to_device(rng.standard_normal((D, D), dtype=np.float32) * 0.03), ctx.empty((F,)), ctx.empty((D,)), ctx.empty((M, D))
    ctx.fill(0.0, b1, F)
    ctx.fill(0.0, b2, D)
    timed("projection_8192x1024x1024", lambda: ctx.gemm(x, (M, D), wq, (D, D), y))
    timed("ffn_up_gelu_8192x1024x4096", lambda: ctx.dense_fused(x, M, D, w1, F, b1, lib.ACT_GELU, None, h))
    timed("ffn_down_residual_8192x4096x1024", lambda: ctx.dense_fused(h, M, F, w2, D, b2, lib.ACT_NONE, x, y))
    timed("fc_residual_8192x1024x1024", lambda: ctx.dense_fused(x, M, D, wq, D, None, lib.ACT_NONE, x, y))
    timed("fc_residual_layernorm_8192x1024x1024", lambda: ctx.dense_layernorm(x, M, D, wq, D, None, lib.ACT_NONE, x, 1024, b2, b2, y))
    for b_ in (x, h, w1, w2, wq, b1, b2, y):
        b_.release()
    B, H, L = 8, 16, 1024
    q, k, v = (ctx.to_device(rng.standard_normal((B, L, H, 64), dtype=np.float32)) for _ in range(3))
    lens = rng.integers(512, 1025, size=B)
    mask = ctx.to_device((np.arange(L)[None, None, None, :] >= lens[:, None, None, None]).astype(np.float32))
    out = ctx.empty((B, L, H, 64))
    desc = ctx.mask_desc(lib.MASK_DENSE, dense=mask)
    timed("attention_config3_dense_padding_mask_token_major",
          lambda: ctx.sdpa_fwd(q, k, v, out, B, H, L, L, 64, 64, 0.125, desc, lib.SDPA_STRICT | lib.SDPA_TOKEN_MAJOR))
    for b_ in (q, k, v, mask, out):
        b_.release()
    B, H, L = 8, 16, 2048
    bufs = [ctx.to_device(rng.standard_normal((B, H, L, 64), dtype=np.float32) * np.float32(0.5)) for _ in range(4)]
    outs = [ctx.empty((B, H, L, 64)) for _ in range(4)]
    st = ctx.empty((B, H, L, 2))
    desc = ctx.mask_desc(lib.MASK_CAUSAL)
    ctx.sdpa_fwd_stats(bufs[0], bufs[1], bufs[2], outs[0], st, B, H, L, L, 64, 0.125, desc, 0)
    timed("attention_backward_config4_causal",
          lambda: ctx.sdpa_bwd(bufs[0], bufs[1], bufs[2], outs[0], st, bufs[3], outs[1], outs[2], outs[3], B, H, L, L, 64, 0.125, desc, 0))
    for b_ in bufs + outs + [st]:
        b_.release()
    # the same shape at other head dims: forward and gradients on the other tile widths
    for d in (128, 96, 32, 256, 80, 48, 16):
        bufs = [ctx.to_device(rng.standard_normal((B, H, L, d), dtype=np.float32) * np.float32(0.5)) for _ in range(4)]
        outs = [ctx.empty((B, H, L, d)) for _ in range(4)]
        st = ctx.empty((B, H, L, 2))
        rT = float(np.float32(1.0) / np.float32(np.sqrt(np.float32(d))))
        timed("attention_forward_config4_shape_head_dim_%d" % d,
              lambda: ctx.sdpa_fwd_stats(bufs[0], bufs[1], bufs[2], outs[0], st, B, H, L, L, d, rT, desc, 0))
        timed("attention_backward_config4_shape_head_dim_%d" % d,
              lambda: ctx.sdpa_bwd(bufs[0], bufs[1], bufs[2], outs[0], st, bufs[3], outs[1], outs[2], outs[3], B, H, L, L, d, rT, desc, 0))
        for b_ in bufs + outs + [st]:
            b_.release()
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-pairs", type=int, default=64, help="(batch, head) slices timed on the CPU oracle; 0 disables")
    ap.add_argument("--decode-repeats", type=int, default=5)
    ap.add_argument("--no-other-configs", dest="other_configs", action="store_false",
                    help="skip configs 1-3 (SDPA, MHA layer, encoder block) that are reported beside the headline")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one streaming kernel (negate, 1 GiB read + 1 GiB written) so that a counter run of "
                         "this command can scale FETCH_SIZE / WRITE_SIZE by a kernel of known traffic")
    ap.add_argument("--kernel-sample", type=int, default=0, metavar="N",
                    help="instead of the benchmark, launch the kernels behind configs 3 and 4 (fused Dense products, dense-mask "
                         "attention, attention gradients) N times each and print their mean event times: a short command for "
                         "profiler counter runs")
    ap.add_argument("--only", default="", metavar="NAMES",
                    help="instead of the benchmark, run only these of the workloads reported beside the headline (comma "
                         "separated: config1, config2, config2_fused_only, recorded, config3, config3_hook_only, backward, masks_and_head_dim, decode_head_dims, greedy, greedy_fused, greedy_primitive, greedy_cached, greedy_cached_only) and print their entries: "
                         "short commands for profiler runs")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (every attention problem fits one MI355X); --gpus %d is not "
              "supported" % args.gpus, file=sys.stderr)
        sys.exit(2)

    from dl4s_amd import lib
    ctx = lib.Context(0)
    info = ctx.device_info()
    if args.kernel_sample > 0:
        print(json.dumps({"kernel_sample": kernel_sample(ctx, lib, args.kernel_sample)}))
        ctx.close()
        return
    if args.only:
        print(json.dumps({"only": other_configs(ctx, lib, args.cpu_pairs > 0, set(args.only.split(",")))}))
        ctx.close()
        return
    pre = prefill(ctx, lib, args.steps, args.warmup)
    dec = decode(ctx, lib, args.decode_repeats) if args.decode_repeats > 0 else None
    if args.copy_calibration:
        n = 1 << 28
        x, y = ctx.empty((n,)), ctx.empty((n,))
        ctx.fill(1.0, x, n)
        ctx.vneg(x, y, n)
        ctx.sync()
        x.release()
        y.release()
    others = other_configs(ctx, lib, args.cpu_pairs > 0) if args.other_configs else None
    ctx.close()

    tflops = pre["flops"] * args.steps / pre["wall_s"] / 1e12
    ach = pre["flops"] / (pre["event_ms_per_launch"] * 1e-3) / 1e12
    line = {}
    if others is not None:
        line["other_configs"] = others      # first, so that the headline objects end the line
    line.update({
        "metric": "attention fwd TFLOP/s (fp32)",
        "value": tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": pre["wall_s"] / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "long-context prefill B=8 H=16 L=2048 d=64 causal, q/k/v=0.5*N(0,1) (benchmark config 4)",
                   "flops_per_step": pre["flops"], "device": info["name"], "cu_count": info["cu_count"]},
        "roofline": {"bound": "mfma", "achieved": ach, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": ach / MFMA_FP32_PEAK_TFLOPS, "traffic": PREFILL_TRAFFIC_BYTES,
                     "traffic_unit": "bytes per launch (L2 fills + writes, rocprofv3 --pmc)", "kernel": "sdpa_prefill_f32_d64",
                     "ms_per_launch": pre["event_ms_per_launch"]},
    })
    sh = pre["shape"]
    dense_flops = 4.0 * sh["d"] * sh["B"] * sh["H"] * sh["L"] * sh["L"]
    # strict mode issues the dense problem's MFMAs for the causal problem's algorithmic flops
    line["roofline"]["strict_mode"] = {
        "what": "same launch with DL4S_SDPA_STRICT (every key tile visited: the reference's NaN/Inf behaviour at blocked keys)",
        "ms_per_launch": pre["strict_ms_per_launch"],
        "achieved": pre["flops"] / (pre["strict_ms_per_launch"] * 1e-3) / 1e12,
        "frac": pre["flops"] / (pre["strict_ms_per_launch"] * 1e-3) / 1e12 / MFMA_FP32_PEAK_TFLOPS,
        "issued_tflops": dense_flops / (pre["strict_ms_per_launch"] * 1e-3) / 1e12,
        "bit_identical_to_default_on_these_inputs": pre["strict_bit_identical"]}
    if dec:
        line["roofline"]["decode"] = {"bound": "hbm", "kernel": "sdpa_decode_splitk_f32", "us_per_step": dec["us_per_step"],
                                      "achieved": dec["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dec["gbs"] / HBM_PEAK_GBS,
                                      "tokens_per_s": dec["tokens_per_s"], "traffic": DECODE_TRAFFIC_BYTES,
                                      "bytes_per_step": dec["bytes_per_step"]}
    if dec:
        line["decode"] = {"workload": "incremental decode B=16 H=16 d=64, KV cache 4096 rows + 64 append+attend steps "
                                      "(benchmark config 5)",
                          "us_per_step": dec["us_per_step"], "tokens_per_s": dec["tokens_per_s"],
                          "single_step_us_p50": dec["single_step_us_p50"], "single_step_us_p99": dec["single_step_us_p99"],
                          "roofline": {"bound": "hbm", "achieved": dec["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                       "frac": dec["gbs"] / HBM_PEAK_GBS, "traffic": DECODE_TRAFFIC_BYTES,
                                       "kernel": "sdpa_decode_splitk_f32", "bytes_per_step": dec["bytes_per_step"]}}
    if args.cpu_pairs > 0:
        q, k, v = pre["inputs"]
        line["cpu_baseline"] = cpu_baseline_prefill(q, k, v, args.cpu_pairs, pre["output"])
        line["cpu_blas_proxy"] = cpu_blas_proxy_prefill(q, k, v, min(32, q.shape[0] * q.shape[1]))
        if dec:
            line["decode"]["cpu_baseline"] = cpu_baseline_decode()
    print(json.dumps(line))


if __name__ == "__main__":
    main()
