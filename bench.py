#!/usr/bin/env python3
"""Benchmark of the decode hot path on one MI355X.

Headline (the JSON line's `value`): HBM GB/s of the fused TQ2_0 dequant matvec at M = 1 on
the MLP gate/up shape (N = 8192, K = 2048, fp32 activations and outputs), measured the way
the reference measures its own kernels (local-metal/src/kernels.rs:8883-9020): R distinct
weight sets totalling >= 1 GiB so nothing is served from cache, GB/s = algorithmic bytes /
elapsed.  One "step" is one pass over the R weight sets, issued as ONE grouped launch.
Everything is resident in HBM before the timed region.

Also measured and reported in the same line (`extra`): the Q4_0 matvec (N = K = 2048), the
TQ2_0 down-projection shape, one logits-sized matvec (262144 x 1536, a single ordinary
launch), the tq2 flash-decoding attention at 32k context (single query, and a batch of
independent sequences), the small-batch layer and the prefill matmul.

`roofline` describes the dominant kernel (matvec_tq2_mfma_kernel, the TQ2_0 matvec): its
algorithmic bytes per launch over its launch duration from HIP events on the library's
stream.  `cpu_baseline` times the CPU restatement of the reference's own path (block dequant
to f16 + sequential f32 dot) on the host cores, on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense f16/bf16 matrix peak

# HBM bytes per launch of the headline kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this command, scaled by
# the same counters on the library's plain copy kernel.  A run of bench.py cannot read hardware counters itself: the
# figure is carried over from the profile named beside it (`roofline.traffic_source`), taken with the current kernel.
MEASURED_TRAFFIC_BYTES = 1085517824   # 526048 KiB x 2.0 + 7980 KiB x 1.0
TRAFFIC_SOURCE = "profiles/matvec_tq2_mfma_grouped_8192x2048.md (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE; carried over, not measured by this run)"


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def distinct_replicas(pkg, ctx, raw, count, block_bytes):
    """`count` weight sets of the same shape at distinct addresses (one allocation), each a
    different rotation of the generated blocks so no two are byte-identical."""
    wb = raw.size
    big = pkg.Buffer.empty(ctx, wb * count)
    for i in range(count):
        big.copy_from_bytes(np.roll(raw, i * block_bytes * 7), i * wb)
    return big, [big.view(i * wb, wb) for i in range(count)]


SETTLE_MS = 150.0   # --settle-ms: untimed run of each measured callable before its warm-up steps


def settle(ctx, fn, ms=None):
    """Runs fn() back to back for about `ms` milliseconds of wall time, untimed.  The GPU raises its clocks only after
    some tens of milliseconds of continuous work (the same launch measures 15-20 % slower in the first few
    milliseconds after an idle period), and the quantity reported is the rate the kernel sustains."""
    ms = SETTLE_MS if ms is None else ms
    if ms <= 0:
        return
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(8):
            fn()
        ctx.synchronize()


def time_steps(pkg, ctx, fn, steps, warmup):
    """Wall-clock (sync on both sides) and HIP-event time of `steps` calls of fn(), after the settle phase and `warmup`
    untimed calls."""
    settle(ctx, fn)
    for _ in range(warmup):
        fn()
    ctx.synchronize()
    e0, e1 = pkg.Event(ctx), pkg.Event(ctx)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    ctx.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ev_ms = e0.elapsed_ms(e1)
    return wall_ms / steps, ev_ms / steps


def bound_call(fn, *args):
    """A zero-argument callable for one C-ABI call with its ctypes arguments converted once:
    keeps the per-launch host cost of the timing loops near the cost of the launch itself."""
    import ctypes as C
    conv = []
    for a in args:
        if hasattr(a, "_h"):
            conv.append(a._h)
        elif isinstance(a, int):
            conv.append(C.c_uint32(a))
        else:
            conv.append(a)
    conv = tuple(conv)

    def call():
        if fn(*conv) != 0:
            raise RuntimeError("library call failed inside a timing loop")
    return call


def matvec_alg_bytes(pkg, fmt, rows, cols):
    return pkg.synth.weight_bytes(fmt, rows, cols) + cols * 4 + rows * 4


def bench_matvec_grouped(pkg, ctx, K, fmt, rows, cols, steps, warmup, total_bytes=1 << 30):
    ty = pkg.Q4_0 if fmt == "q4_0" else pkg.TQ2_0
    g = pkg.synth.rng(1 if fmt == "q4_0" else 2, rows)
    raw = pkg.synth.weights(fmt, rows, cols, g)
    R = max(1, -(-total_bytes // raw.size))
    big, ws = distinct_replicas(pkg, ctx, raw, R, 18 if fmt == "q4_0" else 66)
    x = pkg.synth.activations(1, cols, g)[0]
    xb = pkg.Buffer.from_slice(ctx, x)
    yall = pkg.Buffer.empty(ctx, R * rows * 4)
    ys = [yall.view(i * rows * 4, rows * 4) for i in range(R)]
    xs = [xb] * R
    batch = pkg.CommandBatch(ctx)

    def step():
        K.matvec_quant_grouped_into(batch, ty, ws, xs, pkg.F32, ys, pkg.F32, rows, cols)

    wall, ev = time_steps(pkg, ctx, step, steps, warmup)
    alg = R * matvec_alg_bytes(pkg, fmt, rows, cols)
    return {"replicas": R, "ms_per_step_wall": wall, "ms_per_launch_events": ev, "alg_bytes_per_launch": alg,
            "gbs_wall": alg / wall * 1e-6, "gbs_events": alg / ev * 1e-6,
            "_state": (raw, x, ws, xb, ys, big, yall)}


def bench_matvec_single(pkg, ctx, K, fmt, rows, cols, steps, warmup):
    """One ordinary launch per step (no grouping); replicas rotate so the weights come from HBM."""
    ty = pkg.Q4_0 if fmt == "q4_0" else pkg.TQ2_0
    g = pkg.synth.rng(7, rows)
    raw = pkg.synth.weights(fmt, rows, cols, g)
    R = max(2, min(8, (1 << 30) // raw.size))
    big, ws = distinct_replicas(pkg, ctx, raw, R, 18 if fmt == "q4_0" else 66)
    xb = pkg.Buffer.from_slice(ctx, pkg.synth.activations(1, cols, g)[0])
    yb = pkg.Buffer.empty(ctx, rows * 4)
    batch = pkg.CommandBatch(ctx)
    import ctypes as C
    calls = [bound_call(pkg.lib().lh_matvec_quant_typed_into, batch, C.c_int(ty), w, xb, C.c_int(pkg.F32), yb, C.c_int(pkg.F32),
                        rows, cols) for w in ws]
    it = [0]

    def step():
        calls[it[0] % R]()
        it[0] += 1

    wall, ev = time_steps(pkg, ctx, step, steps, warmup)
    alg = matvec_alg_bytes(pkg, fmt, rows, cols)
    return {"us_per_launch": ev * 1e3, "gbs": alg / ev * 1e-6, "alg_bytes": alg}


def make_kv_pool(pkg, ctx, K, lanes, T, hd, nkv, bits):
    """By-lane KV pool [lanes * T] encoded on the GPU from f16 N(0,1) rows (distinct per lane)."""
    from local_ai_amd import kv_cache
    cb = kv_cache.code_bytes(hd, bits)
    levels = pkg.Buffer.from_slice(ctx, kv_cache.turboquant_levels(hd, bits))
    signs = pkg.Buffer.from_slice(ctx, kv_cache.turboquant_signs(hd))
    pool = [pkg.Buffer.empty(ctx, lanes * T * nkv * cb), pkg.Buffer.empty(ctx, lanes * T * nkv * 2),
            pkg.Buffer.empty(ctx, lanes * T * nkv * cb), pkg.Buffer.empty(ctx, lanes * T * nkv * 2)]
    g = pkg.synth.rng(5, T)
    batch = pkg.CommandBatch(ctx)
    chunk = 8192
    for which in (0, 2):                       # lane 0 is encoded from fresh f16 N(0,1) rows ...
        for t0 in range(0, T, chunk):
            n = min(chunk, T - t0)
            rows = pkg.Buffer.from_slice(ctx, pkg.synth.kv_rows(n, nkv, hd, g))
            K.encode_kv_turboquant_into(batch, rows, levels, signs, pool[which], pool[which + 1], hd, nkv, n, bits, t0, 0)
            batch.commit_and_wait()
    for l in range(1, lanes):                  # ... the others are rotations of it (distinct addresses and contents)
        r = (l * 997) % T
        for buf, unit in ((pool[0], nkv * cb), (pool[1], nkv * 2), (pool[2], nkv * cb), (pool[3], nkv * 2)):
            batch.blit_copy(buf, r * unit, buf, l * T * unit, (T - r) * unit)
            if r:
                batch.blit_copy(buf, 0, buf, (l * T + T - r) * unit, r * unit)
    batch.commit_and_wait()
    return pool, levels, signs


def lanes_for_one_gib(T, hd, nkv=1, bits=2):
    """Independent sequences whose caches together exceed 1 GiB (and so the 256 MB last-level cache, several times)."""
    per_seq = T * nkv * (2 * (hd * bits // 8) + 4)
    n = -(-(1 << 30) // per_seq)
    return -(-n // 32) * 32          # a multiple of 32, so that the workgroups of a launch fill whole CUs


def bench_attention(pkg, ctx, K, steps, warmup, T=32768, lanes=None, hd=256, keep_state=False):
    """`lanes` independent sequences of T cached positions in one batched launch (default: as many as make the caches
    exceed 1 GiB, so that the figure is an HBM figure), and single decode tokens rotating over those sequences."""
    nq, nkv, bits = 8, 1, 2
    if lanes is None:
        lanes = lanes_for_one_gib(T, hd, nkv, bits)
    pool, levels, signs = make_kv_pool(pkg, ctx, K, lanes, T, hd, nkv, bits)
    g = pkg.synth.rng(5, 1)
    q = g.standard_normal((lanes, nq, hd), dtype=np.float32).astype(np.float16)
    qb = pkg.Buffer.from_slice(ctx, q)
    rq = pkg.Buffer.empty(ctx, lanes * nq * hd * 4)
    out = pkg.Buffer.empty(ctx, lanes * nq * hd * 4)
    positions = pkg.Buffer.from_slice(ctx, np.full(lanes, T - 1, np.uint32))
    batch = pkg.CommandBatch(ctx)
    K.hadamard_rotate_hf_into(batch, qb, signs, rq, hd, lanes * nq, True, False)
    batch.commit_and_wait()
    per_pos = nkv * (2 * (hd * bits // 8) + 4)

    def step_batched():
        K.flash_attention_tq_batched_into(batch, rq, pool[0], pool[1], pool[2], pool[3], levels, out, positions, hd, T, nq, nkv,
                                          0, bits, lanes, 0)

    _, ev_b = time_steps(pkg, ctx, step_batched, steps, warmup)
    cb = hd * bits // 8
    views = [[pool[0].view(l * T * nkv * cb, T * nkv * cb), pool[1].view(l * T * nkv * 2, T * nkv * 2),
              pool[2].view(l * T * nkv * cb, T * nkv * cb), pool[3].view(l * T * nkv * 2, T * nkv * 2)]
             for l in range(0, lanes, max(1, lanes // 256))]   # at most ~256 sequences, spread over the pool
    it = [0]
    calls = [bound_call(pkg.lib().lh_flash_attention_tq_into, batch, rq, v[0], v[1], v[2], v[3], levels, out, hd, T, T - 1, nq, nkv,
                        0, bits, 0) for v in views]

    def step_single():   # one decode token of one sequence; sequences rotate so the cache comes from HBM
        calls[it[0] % len(calls)]()
        it[0] += 1

    _, ev_s = time_steps(pkg, ctx, step_single, max(steps, 20), warmup)
    state = None
    if keep_state:   # lane 0's cache and query, for the CPU leg
        state = {"q": q[0].astype(np.float32), "k_codes": pool[0].view(0, T * nkv * cb).as_array(np.uint8, T * nkv * cb).copy(),
                 "k_norms": pool[1].view(0, T * nkv * 2).as_array(np.uint16, T * nkv).copy(),
                 "v_codes": pool[2].view(0, T * nkv * cb).as_array(np.uint8, T * nkv * cb).copy(),
                 "v_norms": pool[3].view(0, T * nkv * 2).as_array(np.uint16, T * nkv).copy(),
                 "levels": levels.as_array(np.float32, 1 << bits).copy(), "signs": signs.as_array(np.float32, hd).copy(),
                 "hd": hd, "nq": nq, "nkv": nkv, "bits": bits, "T": T}
    return {"_state": state, "context": T, "bytes_per_position": per_pos, "cache_bytes": lanes * T * per_pos,
            "batched_lanes": lanes, "batched_us_per_launch": ev_b * 1e3,
            "batched_tokens_per_s": lanes / (ev_b * 1e-3), "batched_gbs": lanes * T * per_pos / ev_b * 1e-6,
            "single_us_per_token": ev_s * 1e3, "single_tokens_per_s": 1.0 / (ev_s * 1e-3),
            "single_gbs": T * per_pos / ev_s * 1e-6}


def bench_attention_prefill(pkg, ctx, K, steps, warmup, T=32768, rows=256):
    """The attention of the last `rows`-token chunk of a T-token prompt (the reference's MAX_PREFILL_CHUNK rows, each seeing
    T - rows + r + 1 cached positions): the tiled prefill entry, head_dim 256, 8 query heads over one KV head."""
    hd, nq, nkv, bits = 256, 8, 1, 2
    pool, levels, signs = make_kv_pool(pkg, ctx, K, 1, T, hd, nkv, bits)
    g = pkg.synth.rng(5, 3)
    rq = pkg.Buffer.from_slice(ctx, g.standard_normal((rows, nq, hd), dtype=np.float32))
    out = pkg.Buffer.empty(ctx, rows * nq * hd * 4)
    batch = pkg.CommandBatch(ctx)

    def step():
        K.flash_attention_tq_prefill_tiled_into(batch, rq, pool[0], pool[1], pool[2], pool[3], levels, out, hd, T, T - rows, rows, nq,
                                                nkv, 0, bits, 0)

    _, ev = time_steps(pkg, ctx, step, steps, warmup)
    macs = rows * nq * hd * 2 * (T - rows / 2)          # multiply-adds of q.k and w.v over the positions each row sees
    return {"rows": rows, "context": T, "us_per_chunk": ev * 1e3, "useful_tmac_per_s": macs / (ev * 1e-3) * 1e-12}


def bench_attention_sweep(pkg, ctx, K, steps, warmup):
    """Context sweep (single decode token, sequences rotating so the cache comes from HBM) and the
    sliding-window layer: window 512 over a 512-slot ring that has wrapped many times."""
    hd, nq, nkv, bits = 256, 8, 1, 2
    per_pos = nkv * (2 * (hd * bits // 8) + 4)
    res = {}
    for T in (4096, 16384, 131072):          # every point over more than 1 GiB of distinct caches
        r = bench_attention(pkg, ctx, K, steps, warmup, T=T)
        res[f"ctx_{T}"] = {"single_us_per_token": r["single_us_per_token"], "single_gbs": r["single_gbs"], "cache_bytes": r["cache_bytes"],
                           "batched_lanes": r["batched_lanes"], "batched_us_per_launch": r["batched_us_per_launch"],
                           "batched_gbs": r["batched_gbs"], "batched_frac_of_hbm_peak": r["batched_gbs"] / HBM_PEAK_GBS}
    # the reference model's full-attention layers: head_dim 512 (260 bytes per position)
    r = bench_attention(pkg, ctx, K, steps, warmup, T=32768, hd=512)
    res["ctx_32768_head_dim_512"] = {"single_us_per_token": r["single_us_per_token"], "single_gbs": r["single_gbs"], "cache_bytes": r["cache_bytes"],
                                     "batched_lanes": r["batched_lanes"], "batched_us_per_launch": r["batched_us_per_launch"],
                                     "batched_gbs": r["batched_gbs"], "batched_frac_of_hbm_peak": r["batched_gbs"] / HBM_PEAK_GBS}
    # sliding window: every lane is a 512-slot ring; logical position far beyond the ring size
    ring, lanes, pos = 512, 4096, 100000
    pool, levels, signs = make_kv_pool(pkg, ctx, K, lanes, ring, hd, nkv, bits)
    g = pkg.synth.rng(9, 1)
    rq = pkg.Buffer.from_slice(ctx, g.standard_normal((lanes, nq, hd), dtype=np.float32))
    out = pkg.Buffer.empty(ctx, lanes * nq * hd * 4)
    positions = pkg.Buffer.from_slice(ctx, np.full(lanes, pos, np.uint32))
    batch = pkg.CommandBatch(ctx)

    def step_batched():
        K.flash_attention_tq_batched_into(batch, rq, pool[0], pool[1], pool[2], pool[3], levels, out, positions, hd, ring, nq, nkv,
                                          ring, bits, lanes, ring)

    _, ev_b = time_steps(pkg, ctx, step_batched, steps, warmup)
    cb = hd * bits // 8
    views = [[pool[0].view(l * ring * nkv * cb, ring * nkv * cb), pool[1].view(l * ring * nkv * 2, ring * nkv * 2),
              pool[2].view(l * ring * nkv * cb, ring * nkv * cb), pool[3].view(l * ring * nkv * 2, ring * nkv * 2)] for l in range(64)]
    calls = [bound_call(pkg.lib().lh_flash_attention_tq_into, batch, rq, v[0], v[1], v[2], v[3], levels, out, hd, pos + 1, pos, nq, nkv,
                        ring, bits, ring) for v in views]
    it = [0]

    def step_single():
        calls[it[0] % len(calls)]()
        it[0] += 1

    _, ev_s = time_steps(pkg, ctx, step_single, max(steps, 50), warmup)
    res["swa_window512_ring512"] = {"batched_lanes": lanes, "batched_us_per_launch": ev_b * 1e3,
                                    "batched_tokens_per_s": lanes / (ev_b * 1e-3), "batched_gbs": lanes * ring * per_pos / ev_b * 1e-6,
                                    "single_us_per_token": ev_s * 1e3}
    return res


def bench_layer(pkg, ctx, K, steps, warmup):
    """Small-batch decode over one decoder layer's seven projections (mixed Q4_0 / TQ2_0)."""
    g = pkg.synth.rng(3)
    ws = []
    for name, fmt, n, k in pkg.synth.DECODER_LAYER:
        ws.append((pkg.QuantWeight.from_bytes(ctx, pkg.synth.weights(fmt, n, k, g), pkg.Q4_0 if fmt == "q4_0" else pkg.TQ2_0, n, k), n, k))
    wbytes = sum(w.device_bytes() for w, _, _ in ws)
    res = {"weight_bytes": wbytes}
    batch = pkg.CommandBatch(ctx)
    for m in (1, 4, 8, 16):
        a2k = pkg.Buffer.from_slice(ctx, pkg.synth.activations(m, 2048, g))
        a8k = pkg.Buffer.from_slice(ctx, pkg.synth.activations(m, 8192, g))
        outs = [pkg.Buffer.empty(ctx, m * n * 4) for _, n, _ in ws]
        import ctypes as C
        calls = [bound_call(pkg.lib().lh_matmul_nt_quant_typed_into, batch, C.c_int(w.ty), a2k if k == 2048 else a8k, C.c_int(pkg.F32),
                            w.buf, o, C.c_int(pkg.F32), m, k, n) for (w, n, k), o in zip(ws, outs)]

        def step():
            for c in calls:
                c()

        _, ev = time_steps(pkg, ctx, step, steps, warmup)
        res[f"m{m}_us_per_layer"] = ev * 1e3
        res[f"m{m}_gbs_hot"] = wbytes / ev * 1e-6       # weights stay in the 256 MB last-level cache here
    return res


def bench_layer_hbm(pkg, ctx, K, steps, warmup, total_bytes=1 << 30):
    """The same small-batch layer with the weights coming from HBM: enough distinct copies of the layer's seven
    projections (18.3 MB each set) to exceed 1 GiB, walked once per step, so that no weight is served from the 256 MB
    last-level cache.  GB/s = weight bytes of all sets / time of one walk."""
    g = pkg.synth.rng(3)
    protos = [(fmt, n, k, pkg.synth.weights(fmt, n, k, g)) for _, fmt, n, k in pkg.synth.DECODER_LAYER]
    set_bytes = sum(r.size for _, _, _, r in protos)
    sets = max(2, -(-total_bytes // set_bytes))
    stacks = []          # per projection: one allocation holding `sets` distinct copies
    for fmt, n, k, raw in protos:
        big = pkg.Buffer.empty(ctx, raw.size * sets)
        blk = 18 if fmt == "q4_0" else 66
        for i in range(sets):
            big.copy_from_bytes(np.roll(raw, i * blk * 7), i * raw.size)
        stacks.append((fmt, n, k, raw.size, big))
    res = {"layer_sets": sets, "weight_bytes": set_bytes * sets}
    batch = pkg.CommandBatch(ctx)
    import ctypes as C
    for m in (1, 4, 8, 16):
        a2k = pkg.Buffer.from_slice(ctx, pkg.synth.activations(m, 2048, g))
        a8k = pkg.Buffer.from_slice(ctx, pkg.synth.activations(m, 8192, g))
        calls, keep = [], []          # `keep`: the views and outputs must outlive the bound calls, which hold raw handles
        for i in range(sets):
            for fmt, n, k, wb, big in stacks:
                ty = pkg.Q4_0 if fmt == "q4_0" else pkg.TQ2_0
                out, w = pkg.Buffer.empty(ctx, m * n * 4), big.view(i * wb, wb)
                keep += [out, w]
                calls.append(bound_call(pkg.lib().lh_matmul_nt_quant_typed_into, batch, C.c_int(ty), a2k if k == 2048 else a8k,
                                        C.c_int(pkg.F32), w, out, C.c_int(pkg.F32), m, k, n))

        def step():
            for c in calls:
                c()

        _, ev = time_steps(pkg, ctx, step, max(3, steps // 4), 1)
        res[f"m{m}_us_per_layer"] = ev * 1e3 / sets
        res[f"m{m}_gbs"] = set_bytes * sets / ev * 1e-6
        res[f"m{m}_frac_of_hbm_peak"] = res[f"m{m}_gbs"] / HBM_PEAK_GBS
    return res


def bench_prefill(pkg, ctx, K, steps, warmup):
    m, k, n = 512, 2048, 8192
    res = {}
    batch = pkg.CommandBatch(ctx)
    for fmt in ("tq2_0", "q4_0"):
        g = pkg.synth.rng(4, 1 if fmt == "q4_0" else 2)
        w = pkg.QuantWeight.from_bytes(ctx, pkg.synth.weights(fmt, n, k, g), pkg.Q4_0 if fmt == "q4_0" else pkg.TQ2_0, n, k)
        ab = pkg.Buffer.from_slice(ctx, pkg.synth.f32_to_bf16_bits(pkg.synth.activations(m, k, g)))
        cb = pkg.Buffer.empty(ctx, m * n * 4)

        import ctypes as C
        step = bound_call(pkg.lib().lh_matmul_nt_quant_typed_into, batch, C.c_int(w.ty), ab, C.c_int(pkg.BF16), w.buf, cb,
                          C.c_int(pkg.F32), m, k, n)

        _, ev = time_steps(pkg, ctx, step, steps, warmup)
        tf = 2.0 * m * k * n / (ev * 1e-3) * 1e-12
        res[fmt] = {"us": ev * 1e3, "tflops": tf, "frac_of_f16_mfma_peak": tf / MFMA_F16_PEAK_TFLOPS}
        # the same product with f16 activations and an f16 result (what a layer hands from kernel to kernel): no conversion
        # in the staging and half the output bytes
        ah = pkg.Buffer.from_slice(ctx, pkg.synth.activations(m, k, g).astype(np.float16))
        ch = pkg.Buffer.empty(ctx, m * n * 2)
        step_h = bound_call(pkg.lib().lh_matmul_nt_quant_typed_into, batch, C.c_int(w.ty), ah, C.c_int(pkg.F16), w.buf, ch,
                            C.c_int(pkg.F16), m, k, n)
        _, ev_h = time_steps(pkg, ctx, step_h, steps, warmup)
        tf_h = 2.0 * m * k * n / (ev_h * 1e-3) * 1e-12
        res[fmt].update({"f16_io_us": ev_h * 1e3, "f16_io_tflops": tf_h, "f16_io_frac_of_f16_mfma_peak": tf_h / MFMA_F16_PEAK_TFLOPS})
    return res


def bench_glue(pkg, ctx, K, steps, warmup):
    """Decoder-layer glue kernels: latency at the decode shapes (one row of hidden 2048, 8 heads x 256, FFN 8192, the
    262144 logits) and streaming rate on a large batch of rows (algorithmic bytes = reads + writes)."""
    g = pkg.synth.rng(11, 1)
    res = {}
    batch = pkg.CommandBatch(ctx)

    def f16buf(n):
        return pkg.Buffer.from_slice(ctx, g.standard_normal(n, dtype=np.float32).astype(np.float16))

    dim, rows = 2048, 49152          # 201 MB per tensor: beyond the 256 MB last-level cache
    x, w, r, o = f16buf(rows * dim), f16buf(dim), f16buf(rows * dim), pkg.Buffer.empty(ctx, rows * dim * 2)
    _, ev = time_steps(pkg, ctx, lambda: K.rms_norm_add_into(batch, x, w, r, o, dim, 1, 1e-6), max(steps, 20), warmup)
    res["rms_norm_add_1x2048_us"] = ev * 1e3
    _, ev = time_steps(pkg, ctx, lambda: K.rms_norm_add_into(batch, x, w, r, o, dim, rows, 1e-6), steps, warmup)
    res["rms_norm_add_49152x2048_gbs"] = rows * dim * 2 * 3 / ev * 1e-6
    hd, nh = 256, 8
    q, qw = f16buf(nh * hd), f16buf(hd)
    _, ev = time_steps(pkg, ctx, lambda: K.qk_norm_rope_into(batch, q, q, qw, hd, nh, 1e-6, 1234, 1e6, 1.0), max(steps, 20), warmup)
    res["qk_norm_rope_8x256_us"] = ev * 1e3
    n, big = 8192, 1 << 26
    a, b, go = f16buf(big), f16buf(big), pkg.Buffer.empty(ctx, big * 2)
    _, ev = time_steps(pkg, ctx, lambda: K.gelu_mul_into(batch, a, b, go, n), max(steps, 20), warmup)
    res["gelu_mul_8192_us"] = ev * 1e3
    _, ev = time_steps(pkg, ctx, lambda: K.gelu_mul_into(batch, a, b, go, big), steps, warmup)
    res["gelu_mul_64M_gbs"] = big * 2 * 3 / ev * 1e-6
    # FP16-weight matvec (the QuantWeight fallback): 131072 x 2048 f16 = 537 MB streamed once
    frows, fcols = 131072, 2048
    fw = pkg.Buffer.empty(ctx, frows * fcols * 2)
    seed_rows = g.standard_normal(4096 * fcols, dtype=np.float32).astype(np.float16)
    for i in range(frows // 4096):
        fw.copy_from_bytes(seed_rows, i * 4096 * fcols * 2)
    fx, fy = f16buf(fcols), pkg.Buffer.empty(ctx, frows * 4)
    _, ev = time_steps(pkg, ctx, lambda: K.matvec_f32out_offset_into(batch, fw, 0, fx, fy, frows, fcols), steps, warmup)
    res["matvec_f16_131072x2048_gbs"] = (frows * fcols * 2 + fcols * 2 + frows * 4) / ev * 1e-6
    _, ev = time_steps(pkg, ctx, lambda: K.matvec_f32out_offset_into(batch, fw, 0, fx, fy, 2048, fcols), max(steps, 20), warmup)
    res["matvec_f16_2048x2048_us"] = ev * 1e3
    logits = pkg.Buffer.from_slice(ctx, g.standard_normal(262144, dtype=np.float32))
    _, ev = time_steps(pkg, ctx, lambda: K.logit_softcap_gpu_into(batch, logits, 30.0, 262144), max(steps, 20), warmup)
    res["logit_softcap_262144_us"] = ev * 1e3
    return res


def fill_kv(pkg, ctx, K, cache, lanes, T, g):
    """Fill a KV cache / lane pool ([lanes * T] rows) with TurboQuant codes: lane 0 encoded on the GPU from f16
    N(0, 1) rows, the other lanes rotations of it (distinct addresses and contents)."""
    hd, nkv, bits = cache.head_dim, cache.n_kv_heads, cache.bits
    cb = hd * bits // 8
    batch = pkg.CommandBatch(ctx)
    for codes, norms in ((cache.keys_q, cache.key_norms), (cache.values_q, cache.value_norms)):
        for t0 in range(0, T, 8192):
            n = min(8192, T - t0)
            rows = pkg.Buffer.from_slice(ctx, pkg.synth.kv_rows(n, nkv, hd, g))
            K.encode_kv_turboquant_into(batch, rows, cache.levels, cache.signs, codes, norms, hd, nkv, n, bits, t0, 0)
            batch.commit_and_wait()
    for l in range(1, lanes):
        r = (l * 997) % T
        for buf, unit in ((cache.keys_q, nkv * cb), (cache.key_norms, nkv * 2), (cache.values_q, nkv * cb),
                          (cache.value_norms, nkv * 2)):
            batch.blit_copy(buf, r * unit, buf, l * T * unit, (T - r) * unit)
            if r:
                batch.blit_copy(buf, 0, buf, (l * T + T - r) * unit, r * unit)
    batch.commit_and_wait()


def bench_decode_step(pkg, ctx, K, steps, warmup, which, T=32768, n_layers=12, lanes=64, lane_layers=3, graphs=True, defer=True, rotate_in_o=True):
    """Whole decoder layers end to end (norms, Q/K/V projections, RoPE, KV encode, attention over the tq2 cache,
    output projection, GeGLU feed-forward, per-layer input injection) at hidden 2048, FFN 8192, 8 query heads over
    1 KV head of 256, Q4_0 attention and TQ2_0 feed-forward weights, context T.  A step runs `n_layers` distinct
    layers back to back (18.9 MB of weights and a cache of their own each, so nothing is served from the last-level
    cache twice), the output of one feeding the next, as a model's decode step does.  `which`: "single" (one
    sequence, one token per step), "lanes" (continuous batching, one token of each of `lanes` sequences) and / or
    "chunk" (a 256-token prefill chunk through forward_batch)."""
    L = pkg.layer
    dims = dict(hidden_size=2048, intermediate_size=8192, num_attention_heads=8, num_key_value_heads=1, head_dim=256)
    pld = 256
    g = pkg.synth.rng(12, 0)

    def make_layer(i):
        t = pkg.synth.decoder_layer_tensors(2048, 8192, 8, 1, 256, pld, g)
        params = L.LayerParams(layer_idx=i, per_layer_dim=pld, rope_theta=1e6, **dims)
        return L.TransformerLayer(params, L.LayerWeights.from_host(ctx, t), fuse_rotation=rotate_in_o)

    res = {"context": T}
    scratch = L.ScratchBuffers(ctx, 2048, 8192, 8, 1, 256, pld)
    batch = pkg.CommandBatch(ctx)
    kv_bytes = T * (2 * 64 + 4)
    if "single" in which:
        res["single"] = _decode_single(pkg, ctx, K, steps, warmup, T, n_layers, make_layer, scratch, batch, g, kv_bytes, graphs, defer)
    if "chunk" in which:
        res["prefill_chunk"] = _prefill_chunk(pkg, ctx, K, steps, warmup, T, make_layer, scratch, batch, g)
    if "lanes" in which:
        res["lanes"] = _decode_lanes(pkg, ctx, K, steps, warmup, T, lanes, lane_layers, make_layer, scratch, batch, g,
                                     kv_bytes, graphs)
    return res


def _prefill_chunk(pkg, ctx, K, steps, warmup, T, make_layer, scratch, batch, g, rows=256, n_layers=4):
    """forward_batch over one prefill chunk (`rows` prompt tokens, the reference's MAX_PREFILL_CHUNK) through
    `n_layers` distinct layers: at the start of a prompt, and as the last chunk of a T-token prompt (attention over the
    whole cache)."""
    pld = 256
    layers = [make_layer(i) for i in range(n_layers)]
    caches = []
    for i in range(n_layers):
        c = pkg.QuantizedKvCache(ctx, 1, 256, T)
        fill_kv(pkg, ctx, K, c, 1, T, pkg.synth.rng(12, 300 + i))
        caches.append(c)
    bs = pkg.layer.BatchScratch(ctx, rows, 2048, 8192, 8, 1, 256, pld, n_layers)
    xin = pkg.Buffer.from_slice(ctx, g.standard_normal(rows * 2048, dtype=np.float32).astype(np.float16))
    ple_all = pkg.Buffer.from_slice(ctx, g.standard_normal(rows * n_layers * pld, dtype=np.float32).astype(np.float16))
    bufs = (bs.hidden_a, bs.hidden_b)
    res = {"rows": rows, "layers_per_step": n_layers}
    for name, start in (("first_chunk", 0), ("last_chunk_of_%d" % T, T - rows)):
        def step():
            batch.blit_copy(xin, 0, bs.hidden_a, 0, rows * 4096)
            for i, layer in enumerate(layers):   # as the pipeline chains them: a layer's last dispatch applies the next layer's input norm
                nxt = layers[i + 1].weights.attn_norm if i + 1 < n_layers else None
                layer.forward_batch(K, batch, rows, start, bufs[i & 1], bufs[(i + 1) & 1], bs, scratch.ones, caches[i],
                                    (ple_all, n_layers), i > 0, nxt)
        wall, ev = time_steps(pkg, ctx, step, steps, warmup)
        out = bufs[n_layers & 1].as_array(np.float16, rows * 2048).astype(np.float32)
        if not np.isfinite(out).all():
            raise RuntimeError("prefill chunk produced non-finite hidden state")
        res[name] = {"us_per_layer_events": ev * 1e3 / n_layers,
                     "prompt_tokens_per_s_35_layers": rows / (ev * 1e-3 / n_layers * 35)}
    return res


def bench_model(pkg, ctx, K, steps, warmup, T=32768, single=True, lanes=64, defer_tail=True, rotate_in_o=True):
    """End-to-end decode of a synthetic model with the geometry of the reference's Gemma 4 E2B configuration
    (local-core/src/config/gemma4_qat.rs:262-283: vocabulary 262144, hidden 1536, 35 layers in a sliding x4 / full
    pattern with head_dim 256 / 512, window 512, the last 20 layers sharing KV, per-layer inputs of 256; Q4_0
    attention and embedding tables, TQ2_0 feed-forward, 6144 wide and 12288 in the KV-shared layers) with T cached
    positions: embedding gather, per-layer inputs, 35 layers, output norm, 262144-row logits, soft cap -- one batch and
    one wait per token."""
    P = pkg.pipeline
    types = ["full_attention" if i % 5 == 4 else "sliding_attention" for i in range(35)]
    cfg = P.Gemma4QATConfig(vocab_size=262144, hidden_size=1536, num_hidden_layers=35, num_attention_heads=8,
                            num_key_value_heads=1, head_dim=256, global_head_dim=512, sliding_window=512,
                            num_kv_shared_layers=20, hidden_size_per_layer_input=256, layer_types=types,
                            sliding_rope_theta=10000.0, full_rope_theta=1000000.0, full_partial_rotary_factor=0.25)
    g = pkg.synth.rng(13, 0)
    # one generated tensor set per kind of layer, uploaded once per layer (distinct addresses, nothing shared in HBM)
    kinds = {}
    for full in (False, True):
        for shared in (False, True):
            kinds[(full, shared)] = pkg.synth.decoder_layer_tensors(1536, 12288 if shared else 6144, 8, 1, 512 if full else 256,
                                                                   256, g, kv_shared=shared)
    one = pkg.synth.decode_model_tensors(P.Gemma4QATConfig(vocab_size=262144, hidden_size=1536, num_hidden_layers=35,
                                                           num_attention_heads=8, num_key_value_heads=1, head_dim=256,
                                                           hidden_size_per_layer_input=256, layer_types=[]),
                                         g, 256, table_rows=2048)
    tensors = {k: v for k, v in one.items() if k != "layers"}
    tensors["layers"] = [kinds[(cfg.is_full_attention(i), cfg.is_kv_shared(i))] for i in range(35)]
    max_ctx = T + 256
    pipe = P.DecodePipeline.from_host(ctx, K, cfg, tensors, max_ctx)
    pipe.defer_layer_tails = defer_tail
    for layer in pipe.layers:
        layer.fuse_rotation = layer.fuse_rotation and rotate_in_o
    del tensors, one, kinds
    if single:
        for i, c in enumerate(pipe.kv_caches):
            fill_kv(pkg, ctx, K, c, 1, min(T, c.physical_positions), pkg.synth.rng(13, 10 + i))
    pipe.position = T - 1
    weight_bytes = sum(_layer_weight_bytes(pkg, l) for l in pipe.layers) + pipe.token_embd.device_bytes() \
        + pipe.per_layer_model_proj.device_bytes()
    def kv_read_bytes(kv_len):
        """Codes and norms the 35 layers' attention reads for one token at kv_len cached positions: the window of a
        sliding layer, everything for a full layer; KV-shared layers read their source layer's rows again."""
        total = 0
        for i in range(cfg.num_hidden_layers):
            c = pipe.kv_caches[pipe.kv_index_map[i]]
            span = kv_len if cfg.is_full_attention(i) else min(kv_len, cfg.sliding_window)
            total += span * c.n_kv_heads * (2 * c.code_bytes() + 4)
        return total

    kv_bytes = kv_read_bytes(T)
    res = {"context": T, "layers": 35}
    if single:
        tokens = [int(v) for v in g.integers(0, cfg.vocab_size, steps + warmup)]
        for t in tokens[:warmup]:
            pipe.decode_step(t)
        ctx.synchronize()
        t0 = time.perf_counter()
        for t in tokens[warmup:]:
            pipe.decode_step(t)
        dt = (time.perf_counter() - t0) / steps
        logits = pipe.logits()
        if not np.isfinite(logits).all() or np.abs(logits).max() > 30.001:
            raise RuntimeError("model decode produced logits outside the soft cap")
        res.update({"us_per_token_wall": dt * 1e6, "tokens_per_s": 1.0 / dt, "weight_bytes_read_per_token": weight_bytes,
                    "kv_bytes_read_per_token": kv_bytes, "gbs_wall": (weight_bytes + kv_bytes) / dt * 1e-9})
    if lanes:
        # continuous batching (local-engine/src/pipeline/batched.rs:271-478): `lanes` sequences, each with about T cached
        # positions in by-lane pools, one token each per step; logits of every lane stay in device memory
        state = pipe.new_batched_decode_state(lanes, max_ctx)
        for i, pool in enumerate(state.pools):
            fill_kv(pkg, ctx, K, pool, lanes, pool.lane_stride(), pkg.synth.rng(13, 40 + i))
        positions = [T - 1 - l for l in range(lanes)]
        lane_steps = max(steps // 2, 5)
        toks = g.integers(0, cfg.vocab_size, (lane_steps + warmup, lanes))
        for row in toks[:warmup]:
            pipe.decode_batch_step(state, [int(v) for v in row], [int(v) for v in row], positions, read_logits=False)
        ctx.synchronize()
        t0 = time.perf_counter()
        for row in toks[warmup:]:
            pipe.decode_batch_step(state, [int(v) for v in row], [int(v) for v in row], positions, read_logits=False)
        dl = (time.perf_counter() - t0) / lane_steps
        lg = state.logits(2)
        if not np.isfinite(lg).all() or np.abs(lg).max() > 30.001:
            raise RuntimeError("batched model decode produced logits outside the soft cap")
        lane_kv = sum(kv_read_bytes(p_ + 1) for p_ in positions)
        res["lanes"] = {"lanes": lanes, "ms_per_step_wall": dl * 1e3, "tokens_per_s": lanes / dl,
                        "kv_bytes_read_per_step": lane_kv, "weight_bytes_read_per_step": weight_bytes,
                        "gbs_wall": (lane_kv + weight_bytes) / dl * 1e-9}
    return res


def _layer_weight_bytes(pkg, layer):
    return sum(w.device_bytes() for w in vars(layer.weights).values() if isinstance(w, pkg.QuantWeight))


def _decode_single(pkg, ctx, K, steps, warmup, T, n_layers, make_layer, scratch, batch, g, kv_bytes, graphs, defer=True):
    pld = 256
    layers = [make_layer(i) for i in range(n_layers)]
    wbytes = _layer_weight_bytes(pkg, layers[0])
    caches = []
    for i in range(n_layers):
        c = pkg.QuantizedKvCache(ctx, 1, 256, T)
        fill_kv(pkg, ctx, K, c, 1, T, pkg.synth.rng(12, 100 + i))
        caches.append(c)
    hidden = [pkg.Buffer.from_slice(ctx, g.standard_normal(2048, dtype=np.float32).astype(np.float16)),
              pkg.Buffer.empty(ctx, 2048 * 2)]
    x0 = pkg.Buffer.from_slice(ctx, hidden[0].as_array(np.float16, 2048))
    ple = pkg.Buffer.from_slice(ctx, g.standard_normal(n_layers * pld, dtype=np.float32).astype(np.float16))

    final = {"buf": 0}

    def step_single():   # as DecodePipeline.forward_token_turbo chains its layers
        batch.blit_copy(x0, 0, hidden[0], 0, 4096)
        cur, pend = 0, None
        for i, layer in enumerate(layers):
            pend = layer.forward_decode(K, batch, hidden[cur], hidden[cur ^ 1], T - 1, scratch, caches[i], ple, n_layers,
                                        pending=pend, defer_tail=defer and i + 1 < len(layers))
            if pend is None:
                cur ^= 1
        final["buf"] = cur

    d0 = batch.dispatch_count()
    step_single()
    per_layer = (batch.dispatch_count() - d0 - 1) // n_layers
    wall, ev = time_steps(pkg, ctx, step_single, max(steps, 20), warmup)
    host = []                                    # host time to enqueue one step (the GPU idle when it starts)
    for _ in range(5):
        ctx.synchronize()
        t0 = time.perf_counter()
        step_single()
        host.append(time.perf_counter() - t0)
    ctx.synchronize()
    out = hidden[final["buf"]].as_array(np.float16, 2048).astype(np.float32)
    if not np.isfinite(out).all():
        raise RuntimeError("decode step produced non-finite hidden state")
    res = {"layers_per_step": n_layers, "us_per_layer_events": ev * 1e3 / n_layers, "us_per_layer_wall": wall * 1e3 / n_layers,
           "dispatches_per_layer": per_layer, "host_enqueue_us_per_layer": min(host) * 1e6 / n_layers,
           "weight_bytes_per_layer": wbytes, "kv_bytes_per_layer": kv_bytes,
           "gbs_events": (wbytes + kv_bytes) / (ev / n_layers) * 1e-6,
           "tokens_per_s_35_layers": 1.0 / (ev * 1e-3 / n_layers * 35)}
    if not graphs:
        return res
    # The same step through the position-in-a-buffer path (one lane of forward_decode_batch_turbo), recorded once into a
    # graph and replayed: one host call per step instead of one per dispatch.
    L = pkg.layer
    pools = []
    for i in range(n_layers):
        pool = pkg.QuantizedUnifiedKvPool(ctx, 1, T, 1, 256, 2, 0)
        for name in ("keys_q", "values_q", "key_norms", "value_norms"):
            src = getattr(caches[i], name)
            batch.blit_copy(src, 0, getattr(pool, name), 0, src.length())
        pools.append(pool)
    batch.commit_and_wait()
    bs = L.BatchScratch(ctx, 1, 2048, 8192, 8, 1, 256, pld, n_layers)
    positions = pkg.Buffer.from_slice(ctx, np.full(1, T - 1, np.uint32))
    gbufs = (bs.hidden_a, bs.hidden_b)

    def encode_lane_step(b):
        b.blit_copy(x0, 0, bs.hidden_a, 0, 4096)
        for i, layer in enumerate(layers):   # as the pipeline chains them: a layer's last dispatch applies the next layer's input norm
            nxt = layers[i + 1].weights.attn_norm if i + 1 < n_layers else None
            layer.forward_decode_batch_turbo(b, K, 1, positions, gbufs[i & 1], gbufs[(i + 1) & 1], bs, scratch.ones, pools[i],
                                             (ple, n_layers), i > 0, nxt)

    batch.begin_capture()
    encode_lane_step(batch)
    graph = batch.end_capture()
    gwall, gev = time_steps(pkg, ctx, graph.launch, max(steps, 20), warmup)
    gout = gbufs[n_layers & 1].as_array(np.float16, 2048).astype(np.float32)
    if not np.isfinite(gout).all() or np.abs(gout - out).max() > 0.05 * max(1.0, np.abs(out).max()):
        raise RuntimeError("graph replay of the decode step disagrees with the eager step")
    res.update({"graph_us_per_layer_events": gev * 1e3 / n_layers, "graph_us_per_layer_wall": gwall * 1e3 / n_layers,
                "graph_dispatches_per_layer": graph.dispatch_count() // n_layers,
                "graph_tokens_per_s_35_layers": 1.0 / (gev * 1e-3 / n_layers * 35)})
    return res


def _decode_lanes(pkg, ctx, K, steps, warmup, T, lanes, lane_layers, make_layer, scratch, batch, g, kv_bytes, graphs):
    pld = 256
    layers = [make_layer(i) for i in range(lane_layers)]
    wbytes = _layer_weight_bytes(pkg, layers[0])
    pools = []
    for i in range(lane_layers):
        pool = pkg.QuantizedUnifiedKvPool(ctx, lanes, T, 1, 256, 2, 0)
        fill_kv(pkg, ctx, K, pool, lanes, T, pkg.synth.rng(12, 200 + i))
        pools.append(pool)
    bs = pkg.layer.BatchScratch(ctx, lanes, 2048, 8192, 8, 1, 256, pld, lane_layers)
    xin = pkg.Buffer.from_slice(ctx, g.standard_normal(lanes * 2048, dtype=np.float32).astype(np.float16))
    ple_all = pkg.Buffer.from_slice(ctx, g.standard_normal(lanes * lane_layers * pld, dtype=np.float32).astype(np.float16))
    positions = pkg.Buffer.from_slice(ctx, np.full(lanes, T - 1, np.uint32))

    def step_lanes():
        batch.blit_copy(xin, 0, bs.hidden_a, 0, lanes * 4096)
        bufs = (bs.hidden_a, bs.hidden_b)
        for i, layer in enumerate(layers):   # as the pipeline chains them: a layer's last dispatch applies the next layer's input norm
            nxt = layers[i + 1].weights.attn_norm if i + 1 < lane_layers else None
            layer.forward_decode_batch_turbo(batch, K, lanes, positions, bufs[i & 1], bufs[(i + 1) & 1], bs, scratch.ones,
                                             pools[i], (ple_all, lane_layers), i > 0, nxt)

    wall, ev = time_steps(pkg, ctx, step_lanes, steps, warmup)
    out = (bs.hidden_a, bs.hidden_b)[lane_layers & 1].as_array(np.float16, lanes * 2048).astype(np.float32)
    if not np.isfinite(out).all():
        raise RuntimeError("batched decode step produced non-finite hidden state")
    res = {"lanes": lanes, "layers_per_step": lane_layers, "us_per_layer_events": ev * 1e3 / lane_layers,
           "us_per_layer_wall": wall * 1e3 / lane_layers, "kv_bytes_per_layer": lanes * kv_bytes,
           "gbs_events": (wbytes + lanes * kv_bytes) / (ev / lane_layers) * 1e-6,
           "tokens_per_s_35_layers": lanes / (ev * 1e-3 / lane_layers * 35)}
    if not graphs:
        return res
    batch.commit_and_wait()
    batch.begin_capture()
    step_lanes()
    graph = batch.end_capture()
    gwall, gev = time_steps(pkg, ctx, graph.launch, steps, warmup)
    gout = (bs.hidden_a, bs.hidden_b)[lane_layers & 1].as_array(np.float16, lanes * 2048).astype(np.float32)
    if not np.array_equal(gout, out):
        raise RuntimeError("graph replay of the batched decode step disagrees with the eager step")
    res.update({"graph_us_per_layer_events": gev * 1e3 / lane_layers,
                "graph_tokens_per_s_35_layers": lanes / (gev * 1e-3 / lane_layers * 35)})
    return res


def cpu_baseline(pkg, raw, x, rows, cols, target_s=12.0):
    """CPU restatement of the reference path on the host cores: bounded sample of the same workload."""
    from oracle import oracle as orc
    threads = min(orc.max_threads(), os.cpu_count() or 1)
    alg = matvec_alg_bytes(pkg, "tq2_0", rows, cols)
    t0 = time.perf_counter()
    orc.matvec_quant_ref("tq2_0", raw, x, rows, cols, threads=threads)
    one = time.perf_counter() - t0
    reps = int(max(1, min(2000, target_s / max(one, 1e-4))))
    t0 = time.perf_counter()
    for _ in range(reps):
        y = orc.matvec_quant_ref("tq2_0", raw, x, rows, cols, threads=threads)
    dt = time.perf_counter() - t0
    t1 = time.perf_counter()
    orc.matvec_quant_ref("tq2_0", raw, x, rows, cols, threads=1)
    single = time.perf_counter() - t1
    return {"value": alg * reps / dt * 1e-9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{reps} repetitions of one 8192x2048 TQ2_0 matvec ({dt:.1f} s, OpenMP over rows); "
                      f"single thread: {alg / single * 1e-9:.3f} GB/s"}, y


def cpu_baseline_q4_0(pkg, target_s=6.0):
    """The same CPU path on the Q4_0 configuration (N = K = 2048, fp32 x and y)."""
    from oracle import oracle as orc
    rows = cols = 2048
    g = pkg.synth.rng(1, rows)
    raw = pkg.synth.weights("q4_0", rows, cols, g)
    x = pkg.synth.activations(1, cols, g)[0]
    threads = min(orc.max_threads(), os.cpu_count() or 1)
    alg = matvec_alg_bytes(pkg, "q4_0", rows, cols)
    t0 = time.perf_counter()
    orc.matvec_quant_ref("q4_0", raw, x, rows, cols, threads=threads)
    one = time.perf_counter() - t0
    reps = int(max(1, min(4000, target_s / max(one, 1e-4))))
    t0 = time.perf_counter()
    for _ in range(reps):
        orc.matvec_quant_ref("q4_0", raw, x, rows, cols, threads=threads)
    dt = time.perf_counter() - t0
    t1 = time.perf_counter()
    for _ in range(3):
        orc.matvec_quant_ref("q4_0", raw, x, rows, cols, threads=1)
    single = (time.perf_counter() - t1) / 3
    return {"workload": "Q4_0 fused dequant-matvec, M=1, N=2048 x K=2048", "value": alg * reps / dt * 1e-9, "unit": "GB/s",
            "cores": threads, "kind": "port",
            "sample": f"{reps} repetitions of one 2048x2048 Q4_0 matvec ({dt:.1f} s, OpenMP over rows); "
                      f"single thread: {alg / single * 1e-9:.3f} GB/s"}


def cpu_baseline_attention(pkg, st, target_s=8.0):
    """The reference's CPU attention over a TurboQuant cache: TurboQuant::decode of every cached K and V row
    (local-engine/src/turboquant.rs:280-291), then f32 softmax(q . k) . v per query head (the pattern of
    local-metal/src/kernels.rs:8497-8528), on one sequence of the benchmark's caches.  Rates are quoted over the same
    132 bytes per position the GPU figure uses."""
    from oracle import oracle as orc
    threads = min(orc.max_threads(), os.cpu_count() or 1)
    T, hd, nq, nkv, bits = st["T"], st["hd"], st["nq"], st["nkv"], st["bits"]
    args = (st["q"], st["k_codes"], st["k_norms"], st["v_codes"], st["v_norms"], st["levels"], st["signs"], hd, T, T - 1, nq, nkv, 0, bits, 0)
    alg = T * nkv * (2 * (hd * bits // 8) + 4)
    t0 = time.perf_counter()
    orc.attention_tq_decode_then_attend(*args, threads=threads)
    one = time.perf_counter() - t0
    reps = int(max(1, min(200, target_s / max(one, 1e-4))))
    t0 = time.perf_counter()
    for _ in range(reps):
        orc.attention_tq_decode_then_attend(*args, threads=threads)
    dt = (time.perf_counter() - t0) / reps
    t1 = time.perf_counter()
    orc.attention_tq_decode_then_attend(*args, threads=1)
    single = time.perf_counter() - t1
    return {"workload": f"tq2 KV attention, one query token over {T} cached positions, 8 query heads / 1 KV head, head_dim {hd}",
            "value": 1.0 / dt, "unit": "tokens/s", "gbs": alg / dt * 1e-9, "cores": threads, "kind": "port",
            "sample": f"{reps} repetitions of one decode token at {T} positions ({dt * reps:.1f} s; decode of every K and V row, then "
                      f"f32 softmax . V; OpenMP over positions); single thread: {1.0 / single:.2f} tokens/s, {alg / single * 1e-9:.4f} GB/s"}


def main():
    global SETTLE_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="untimed milliseconds each measured call is run before its warm-up steps, so that the clocks have risen")
    ap.add_argument("--quick", action="store_true", help="headline measurement only")
    ap.add_argument("--no-graph", action="store_true", help="decode legs: skip the recorded-batch (HIP graph) replays")
    ap.add_argument("--no-defer-tail", action="store_true",
                    help="decode / model legs: every layer dispatches its own last step (default: it rides in the next layer's first dispatch)")
    ap.add_argument("--no-rotate-in-o", action="store_true",
                    help="decode / model legs: the rotation back out of code space as a dispatch of its own (default: in the output projection's staging)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--legs", default="matvec,attention,sweep,layer,prefill,glue,decode,lanes,chunk,model,model_lanes",
                    help="comma-separated extra measurements to run besides the headline (for profiling one kernel at a time); "
                         "model_few_lanes (2 .. 16 sequences at 8k context) is not in the default set")
    args = ap.parse_args()
    SETTLE_MS = args.settle_ms
    if args.gpus != 1:
        print("bench.py measures one MI355X: the hot path is a single-GPU kernel path and no multi-GPU "
              "figure exists for it; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import __graft_entry__ as ge
    pkg = ge.load_package()
    ctx = pkg.Context(0)
    K = pkg.Kernels(ctx)
    log("[bench] device:", ctx.device_name(), "CUs:", ctx.compute_units())

    # A plain copy of known size first: the reference point for the HBM traffic counters when this
    # command runs under rocprofv3 --pmc (256 MiB read + 256 MiB written by blit_copy16_kernel).
    cal_src, cal_dst = pkg.Buffer.empty(ctx, 256 << 20), pkg.Buffer.empty(ctx, 256 << 20)
    cal_batch = pkg.CommandBatch(ctx)
    cal_batch.blit_copy(cal_src, 0, cal_dst, 0, 256 << 20)
    cal_batch.commit_and_wait()
    cal_src.free(); cal_dst.free()

    rows, cols = 8192, 2048
    head = bench_matvec_grouped(pkg, ctx, K, "tq2_0", rows, cols, args.steps, args.warmup)
    raw, x, ws, xb, ys, _, _ = head.pop("_state")
    log(f"[bench] TQ2_0 {rows}x{cols} x{head['replicas']}: {head['gbs_wall']:.0f} GB/s wall, {head['gbs_events']:.0f} GB/s events")

    # parity of what was just timed: replica 0 against the CPU path
    extra = {}
    cpu = None
    if not args.no_cpu:
        cpu, y_cpu = cpu_baseline(pkg, raw, x, rows, cols)
        got = ys[0].as_array(np.float32, rows)
        err = float(np.max(np.abs(got - y_cpu) / np.maximum(np.abs(y_cpu), 1.0)))
        extra["parity_max_norm_err_vs_cpu_path"] = err
        log(f"[bench] CPU baseline {cpu['value']:.2f} GB/s on {cpu['cores']} threads; parity err {err:.2e}")
        if err > 1e-3:
            log("[bench] PARITY FAILURE: GPU result differs from the CPU path beyond 1e-3")
            sys.exit(1)

    legs = set() if args.quick else set(args.legs.split(","))
    del ws, ys
    cpu_others = []      # CPU baselines of the other measured configurations, reported inside `cpu_baseline`
    if "matvec" in legs and not args.no_cpu:
        cpu_others.append(cpu_baseline_q4_0(pkg))
        log(f"[bench] CPU Q4_0 baseline: {cpu_others[-1]['value']:.2f} GB/s on {cpu_others[-1]['cores']} threads")
    if "matvec" in legs:
        for fmt, r, c in (("q4_0", 2048, 2048), ("tq2_0", 2048, 8192)):
            res = bench_matvec_grouped(pkg, ctx, K, fmt, r, c, args.steps, args.warmup)
            res.pop("_state")
            extra[f"matvec_{fmt}_{r}x{c}_grouped"] = {k: res[k] for k in ("replicas", "ms_per_launch_events", "gbs_events")}
            extra[f"matvec_{fmt}_{r}x{c}_grouped"]["frac_of_hbm_peak"] = res["gbs_events"] / HBM_PEAK_GBS
            log(f"[bench] {fmt} {r}x{c} grouped: {res['gbs_events']:.0f} GB/s")
        for fmt, r, c in (("q4_0", 262144, 1536), ("tq2_0", 8192, 2048), ("q4_0", 2048, 2048)):
            res = bench_matvec_single(pkg, ctx, K, fmt, r, c, max(args.steps, 50), args.warmup)
            res["frac_of_hbm_peak"] = res["gbs"] / HBM_PEAK_GBS
            extra[f"matvec_{fmt}_{r}x{c}_single_launch"] = res
            log(f"[bench] {fmt} {r}x{c} single launch: {res['us_per_launch']:.1f} us, {res['gbs']:.0f} GB/s")
    if "attention" in legs:
        att = bench_attention(pkg, ctx, K, args.steps, args.warmup, keep_state=not args.no_cpu)
        att_state = att.pop("_state")
        att["batched_frac_of_hbm_peak"] = att["batched_gbs"] / HBM_PEAK_GBS
        extra["tq2_attention_32k"] = att
        if att_state is not None:
            cpu_others.append(cpu_baseline_attention(pkg, att_state))
            log(f"[bench] CPU attention baseline: {cpu_others[-1]['value']:.2f} tokens/s, {cpu_others[-1]['gbs']:.3f} GB/s on {cpu_others[-1]['cores']} threads")
        log(f"[bench] tq2 attention 32k: batched {att['batched_tokens_per_s']:.0f} tok/s ({att['batched_gbs']:.0f} GB/s), "
            f"single {att['single_us_per_token']:.1f} us/token")
    if "attention" in legs:
        extra["tq2_attention_prefill_256x32k"] = bench_attention_prefill(pkg, ctx, K, args.steps, args.warmup)
        log("[bench] tiled prefill attention:", extra["tq2_attention_prefill_256x32k"])
    if "sweep" in legs:
        extra["tq2_attention_sweep"] = bench_attention_sweep(pkg, ctx, K, args.steps, args.warmup)
        log("[bench] attention sweep:", extra["tq2_attention_sweep"])
    if "layer" in legs:
        extra["decoder_layer_small_batch"] = bench_layer(pkg, ctx, K, args.steps, args.warmup)
        log("[bench] layer:", extra["decoder_layer_small_batch"])
        extra["decoder_layer_small_batch_hbm"] = bench_layer_hbm(pkg, ctx, K, args.steps, args.warmup)
        log("[bench] layer, weights from HBM:", extra["decoder_layer_small_batch_hbm"])
    if "prefill" in legs:
        extra["prefill_matmul_512x2048x8192_bf16"] = bench_prefill(pkg, ctx, K, args.steps, args.warmup)
        log("[bench] prefill:", extra["prefill_matmul_512x2048x8192_bf16"])
    if "glue" in legs:
        extra["layer_glue_kernels"] = bench_glue(pkg, ctx, K, args.steps, args.warmup)
        log("[bench] glue:", extra["layer_glue_kernels"])

    if legs & {"decode", "lanes", "chunk"}:
        which = (["single"] if "decode" in legs else []) + (["lanes"] if "lanes" in legs else []) + \
            (["chunk"] if "chunk" in legs else [])
        extra["decode_step_end_to_end"] = bench_decode_step(pkg, ctx, K, args.steps, args.warmup, which, graphs=not args.no_graph, defer=not args.no_defer_tail,
                                                            rotate_in_o=not args.no_rotate_in_o)
        log("[bench] decode step:", extra["decode_step_end_to_end"])

    if "model_few_lanes" in legs:
        # not in the default set: the same model with 2 .. 16 sequences at 8192 cached positions, where the small-batch
        # routing of the quantised products (rows as matvecs / the decode-batch kernels) decides the step time
        extra["model_decode_few_lanes_8k"] = {
            str(n): bench_model(pkg, ctx, K, max(args.steps, 20), args.warmup, T=8192, single=False, lanes=n)["lanes"]
            for n in (2, 4, 8, 12, 16)}
        log(f"[bench] model decode, few lanes: {extra['model_decode_few_lanes_8k']}")
    if legs & {"model", "model_lanes"}:
        extra["model_decode_e2b_geometry"] = bench_model(pkg, ctx, K, max(args.steps, 20), args.warmup, single="model" in legs,
                                                         lanes=64 if "model_lanes" in legs else 0, defer_tail=not args.no_defer_tail,
                                                         rotate_in_o=not args.no_rotate_in_o)
        log("[bench] model decode:", extra["model_decode_e2b_geometry"])

    achieved = head["alg_bytes_per_launch"] / head["ms_per_launch_events"] * 1e-6
    # The other north-star kernels of this run, in the blocks a reader of the line keeps: their rooflines beside the
    # headline kernel's, and the second half of the metric (attention tokens/s at 32k) in `config`.
    roof_others = []
    for key, kernel in (("matvec_q4_0_2048x2048_grouped", "matvec_quant_kernel<Q4_0, staged form> (Q4_0 M=1, N=K=2048)"),
                        ("matvec_tq2_0_2048x8192_grouped", "matvec_tq2_mfma_kernel, long-row form (TQ2_0 M=1, N=2048 x K=8192)")):
        if key in extra:
            r = extra[key]
            roof_others.append({"kernel": kernel, "bound": "hbm", "achieved": r["gbs_events"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                "frac": r["gbs_events"] / HBM_PEAK_GBS, "launch_ms": r["ms_per_launch_events"], "replicas": r["replicas"]})
    attention_cfg = None
    if "tq2_attention_32k" in extra:
        a = extra["tq2_attention_32k"]
        roof_others.append({"kernel": "attention_tq_mfma_quad_kernel (tq2 KV flash decoding, 8 q heads / 1 KV head, head_dim 256, 32768 positions; four chunks of a sequence per workgroup, merged in the kernel)",
                            "bound": "hbm", "achieved": a["batched_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                            "frac": a["batched_gbs"] / HBM_PEAK_GBS, "launch_ms": a["batched_us_per_launch"] * 1e-3,
                            "alg_bytes_per_launch": a["cache_bytes"]})
        attention_cfg = {"context": a["context"], "sequences_per_launch": a["batched_lanes"], "tokens_per_s": a["batched_tokens_per_s"],
                         "gbs": a["batched_gbs"], "frac_of_hbm_peak": a["batched_gbs"] / HBM_PEAK_GBS,
                         "us_per_launch": a["batched_us_per_launch"], "single_sequence_us_per_token": a["single_us_per_token"],
                         "single_sequence_tokens_per_s": a["single_tokens_per_s"]}
    if cpu is not None and cpu_others:
        cpu["others"] = cpu_others
    line = {
        "metric": "Q4_0/TQ2_0 matvec HBM GB/s (% of peak) at M=1; tq2 KV attn tokens/s @32k",
        "value": head["gbs_wall"],
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": head["ms_per_step_wall"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",   # 2-bit codes x 8-bit activation limbs on v_mfma_i32_16x16x64_i8, f32 block scales
        "data": "synthetic",
        "config": {"workload": "TQ2_0 fused dequant-matvec, M=1, N=8192 x K=2048 (MLP gate/up), fp32 x and y",
                   "replicas_per_step": head["replicas"], "launches_per_step": 1,
                   "bytes_per_step": head["alg_bytes_per_launch"], "pct_of_hbm_peak": 100.0 * head["gbs_wall"] / HBM_PEAK_GBS,
                   "settle_ms_before_warmup": SETTLE_MS,
                   "x_shared_by_replicas": True,   # the replicas read one 8 KB activation vector (0.2 % of the bytes); weights and outputs are distinct
                   "tq2_attention_32k": attention_cfg},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC_BYTES, "traffic_source": TRAFFIC_SOURCE,
                     "kernel": "matvec_tq2_mfma_kernel<float, float, false, 256, true>", "alg_bytes_per_launch": head["alg_bytes_per_launch"],
                     "launch_ms": head["ms_per_launch_events"], "others": roof_others},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
