"""Decoder layer end to end on the GPU (local-engine/src/layer.rs:354-873) against the CPU composition
in oracle/layer.py, plus the reference's own consistency properties: the multi-row and multi-lane
paths agree with single-token decode (pipeline/batched.rs:530-760 checks the same on a real model),
and a ringed lane pool matches an absolute one after wrapping
(kv_cache/quant_unified_pool.rs:377-459, bit for bit).

How a step is checked.  Every intermediate is stored as f16 and the kernels sum in f32 in another
order than the oracle's float64, so single roundings differ by an f16 ulp.  A 2-bit KV code is a
discontinuous function of its input: a K or V coordinate one ulp from a quantiser boundary flips, and
one flipped code moves the attention output by several per cent.  So each step is checked in two
stages: (1) the K / V rows the GPU is about to encode (left in the scratch buffers) against the
oracle's own, to a few f16 ulps; (2) the oracle then encodes the GPU's rows, after which the codes in
the device cache must equal the oracle's bit for bit and the layer output is held to 3e-2 absolute at
worst and 4e-3 on average (hidden state O(1), f16 ulp 1e-3 to 2e-3)."""
import numpy as np
import pytest

from oracle import layer as OL

pytestmark = pytest.mark.gpu

WORST, MEAN = 3e-2, 4e-3
KV_WORST, KV_MEAN = 1e-2, 1e-3


def _dims(hd=256, n_head=4, n_kv=1, hidden=512, inter=1024):
    return dict(hidden_size=hidden, intermediate_size=inter, num_attention_heads=n_head, num_key_value_heads=n_kv,
                head_dim=hd)


def _make(pkg, gpu, g, dims, pld=0, n_layers=1, layer_idx=0, extra=None, **synth_kw):
    ctx, _ = gpu
    extra = extra or {}
    t = pkg.synth.decoder_layer_tensors(dims["hidden_size"], dims["intermediate_size"], dims["num_attention_heads"],
                                        dims["num_key_value_heads"], dims["head_dim"], pld, g, **synth_kw)
    params = pkg.layer.LayerParams(layer_idx=layer_idx, per_layer_dim=pld, is_kv_shared=synth_kw.get("kv_shared", False),
                                   **dims, **extra)
    dev = pkg.layer.TransformerLayer(params, pkg.layer.LayerWeights.from_host(ctx, t))
    ora = OL.Layer.from_host(t, layer_idx=layer_idx, per_layer_dim=pld, is_kv_shared=synth_kw.get("kv_shared", False),
                             **dims, **extra)
    return dev, ora, t


def _close(got, want, what, worst=WORST, mean=MEAN):
    d = np.abs(np.asarray(got, np.float32) - np.asarray(want, np.float32))
    assert np.isfinite(np.asarray(got, np.float32)).all(), what
    assert d.max() <= worst and d.mean() <= mean, f"{what}: worst {d.max():.4g} mean {d.mean():.4g}"


def _step(ora, x, pos, kv, got, k_gpu, v_gpu, what, ple=None):
    """Stage 1 and 2 of the module docstring for one row; `k_gpu` is None for a KV-shared layer."""
    tr = {}
    want = OL.decode_layer(ora, x, pos, kv, ple, kv_rows=None if k_gpu is None else (k_gpu, v_gpu), trace=tr)
    if k_gpu is not None:
        _close(k_gpu, tr["k"], what + ": K row", KV_WORST, KV_MEAN)
        _close(v_gpu, tr["v"], what + ": V row", KV_WORST, KV_MEAN)
    _close(got, want, what)


def _same_cache(dev_cache, kv, rows):
    """The first `rows` physical rows of the device cache hold the oracle's codes and norms."""
    cb = len(kv.k_codes) // len(kv.k_norms)
    for name, arr, dt, n in (("keys_q", kv.k_codes, np.uint8, rows * cb), ("values_q", kv.v_codes, np.uint8, rows * cb),
                             ("key_norms", kv.k_norms, np.uint16, rows), ("value_norms", kv.v_norms, np.uint16, rows)):
        assert np.array_equal(getattr(dev_cache, name).as_array(dt, n), arr[:n]), name


def _decode_steps(pkg, gpu, dev, ora, xs, cache, kv, ple=None, n_layers=1, start=0):
    ctx, kernels = gpu
    p = dev.params
    scratch = pkg.layer.ScratchBuffers(ctx, p.hidden_size, p.intermediate_size, p.num_attention_heads,
                                       p.num_key_value_heads, p.head_dim, p.per_layer_dim)
    out = pkg.Buffer.empty(ctx, p.hidden_size * 2)
    ple_buf = pkg.Buffer.from_slice(ctx, ple) if ple is not None else None
    outs = []
    for i, x in enumerate(xs):
        inp = pkg.Buffer.from_slice(ctx, x)
        batch = pkg.CommandBatch(ctx)
        dev.forward_decode(kernels, batch, inp, out, start + i, scratch, cache, ple_buf, n_layers)
        batch.commit_and_wait()
        got = out.as_array(np.float16, p.hidden_size)
        kv_elems = p.num_key_value_heads * p.head_dim
        _step(ora, x, start + i, kv, got, scratch.k.as_array(np.float16, kv_elems),
              scratch.v.as_array(np.float16, kv_elems), f"position {start + i}", ple)
        outs.append(got)
    return outs


CASES = ["plain", "ple_scale", "hd512_partial_rotary", "f16_weights", "gqa"]


@pytest.mark.parametrize("case", CASES)
def test_forward_decode_matches_oracle(pkg, gpu, oracle, case):
    ctx, kernels = gpu
    g = pkg.synth.rng(900, CASES.index(case))
    dims, pld, extra, kw, n_layers, layer_idx = _dims(), 0, {}, {}, 1, 0
    if case == "ple_scale":
        pld, n_layers, layer_idx, kw = 256, 3, 1, dict(output_scale=0.75)
    elif case == "hd512_partial_rotary":
        dims, extra = _dims(hd=512, n_head=2), dict(rope_theta=1e6, partial_rotary_factor=0.25)
    elif case == "f16_weights":
        kw = dict(attn_fmt="q4_0", ffn_fmt="q4_0")
    elif case == "gqa":
        dims = _dims(n_head=8, n_kv=2)
    dev, ora, t = _make(pkg, gpu, g, dims, pld, n_layers, layer_idx, extra, **kw)
    if case == "f16_weights":        # attention projections expanded to f16 rows, as a Q8_0 / F32 tensor would be
        for name in ("attn_q", "attn_k", "attn_v", "attn_output"):
            fmt, rows, cols, payload = t[name]
            t[name] = ("f16", rows, cols, oracle.dequant_q4_0(payload).view(np.float16))
        dev = pkg.layer.TransformerLayer(dev.params, pkg.layer.LayerWeights.from_host(ctx, t))
        ora = OL.Layer.from_host(t, **dims)
    steps = 40
    cache = pkg.kv_cache.QuantizedKvCache(ctx, dims["num_key_value_heads"], dims["head_dim"], 64)
    cache.reset()
    kv = OL.KvState(dims["num_key_value_heads"], dims["head_dim"], 2, 64)
    xs = g.standard_normal((steps, dims["hidden_size"]), dtype=np.float32).astype(np.float16)
    ple = g.standard_normal(n_layers * pld, dtype=np.float32).astype(np.float16) if pld else None
    _decode_steps(pkg, gpu, dev, ora, xs, cache, kv, ple, n_layers)
    _same_cache(cache, kv, steps * dims["num_key_value_heads"])


def test_forward_decode_sliding_window_ring_and_shared_kv(pkg, gpu, oracle):
    """A sliding-window layer on a ringed cache that wraps, followed by a KV-shared layer reading that cache."""
    ctx, kernels = gpu
    g = pkg.synth.rng(901, 0)
    dims, window = _dims(), 32
    cap = pkg.kv_cache.swa_ring_capacity(window, 4096)
    dev, ora, _ = _make(pkg, gpu, g, dims, extra=dict(sliding_window=window))
    shared_dev, shared_ora, _ = _make(pkg, gpu, g, dims, extra=dict(sliding_window=window), kv_shared=True)
    assert shared_dev.weights.attn_k is None
    cache = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, 4096, 2, cap, window)
    cache.reset()
    kv = OL.KvState(1, 256, 2, 4096, ring_capacity=cap)
    steps = cap + 9
    xs = g.standard_normal((steps, 512), dtype=np.float32).astype(np.float16)
    scratch = pkg.layer.ScratchBuffers(ctx, 512, 1024, 4, 1, 256, 0)
    out, out2 = pkg.Buffer.empty(ctx, 1024), pkg.Buffer.empty(ctx, 1024)
    for pos in range(steps):
        inp = pkg.Buffer.from_slice(ctx, xs[pos])
        batch = pkg.CommandBatch(ctx)
        dev.forward_decode(kernels, batch, inp, out, pos, scratch, cache)
        shared_dev.forward_decode(kernels, batch, out, out2, pos, scratch, cache)      # both layers in one batch
        batch.commit_and_wait()
        got1 = out.as_array(np.float16, 512)
        # the shared layer ran last, so scratch.k / scratch.v still hold the own-KV layer's rows
        _step(ora, xs[pos], pos, kv, got1, scratch.k.as_array(np.float16, 256), scratch.v.as_array(np.float16, 256),
              f"own-KV layer, position {pos}")
        _step(shared_ora, got1, pos, kv, out2.as_array(np.float16, 512), None, None, f"KV-shared layer, position {pos}")
    _same_cache(cache, kv, cap)


def test_grouped_and_fused_dispatches_change_nothing(pkg, gpu, oracle):
    """Grouped K/V and gate/up launches and the fused qk_norm_rope give the bits of the reference's one-kernel-per-op
    sequence.  (The staged-vector prologues may differ from it by an f16 ulp of the normalised vector -- the RMS sum
    runs in another order -- so they are held to the oracle instead, by every other test in this file.)"""
    ctx, kernels = gpu
    g = pkg.synth.rng(902, 0)
    dims = _dims()
    dev, _, _ = _make(pkg, gpu, g, dims)
    variants = [pkg.layer.TransformerLayer(dev.params, dev.weights, group_projections=a, fuse_norm_rope=b,
                                           fuse_prologues=False) for a, b in ((False, False), (True, True))]
    x = g.standard_normal(512, dtype=np.float32).astype(np.float16)
    res = []
    for layer in variants:
        cache = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, 8)
        cache.reset()
        scratch = pkg.layer.ScratchBuffers(ctx, 512, 1024, 4, 1, 256, 0)
        inp, out = pkg.Buffer.from_slice(ctx, x), pkg.Buffer.empty(ctx, 1024)
        batch = pkg.CommandBatch(ctx)
        layer.forward_decode(kernels, batch, inp, out, 5, scratch, cache)
        batch.commit_and_wait()
        res.append((out.as_array(np.uint16, 512), cache.keys_q.as_array(np.uint8), cache.values_q.as_array(np.uint8)))
    for a, b in zip(*res):
        assert np.array_equal(a, b)


def test_rotation_in_the_output_projection_changes_nothing(pkg, gpu, oracle):
    """A decoded token's rotation back out of code space (quant_cache.rs:590-598) rides in the staging of the output
    projection (layer.rs:440-446): never more dispatches (one fewer where the merge of many partial records and the
    rotation were two), the same bits, at a short and at a longer context."""
    ctx, kernels = gpu
    g = pkg.synth.rng(903, 0)
    dims = _dims()
    dev, _, _ = _make(pkg, gpu, g, dims)
    variants = [pkg.layer.TransformerLayer(dev.params, dev.weights, fuse_rotation=f) for f in (False, True)]
    x = g.standard_normal(512, dtype=np.float32).astype(np.float16)
    for position in (5, 3000):
        res, counts = [], []
        for layer in variants:
            cache = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, 4096)
            fill = pkg.synth.rng(904, position)   # random codes and norms near one, the same for both variants
            for codes, norms in ((cache.keys_q, cache.key_norms), (cache.values_q, cache.value_norms)):
                codes.copy_from_bytes(fill.integers(0, 256, codes.length(), dtype=np.uint8))
                norms.copy_from_bytes((0.5 + fill.random(norms.length() // 2)).astype(np.float16))
            scratch = pkg.layer.ScratchBuffers(ctx, 512, 1024, 4, 1, 256, 0)
            inp, out = pkg.Buffer.from_slice(ctx, x), pkg.Buffer.empty(ctx, 1024)
            batch = pkg.CommandBatch(ctx)
            layer.forward_decode(kernels, batch, inp, out, position, scratch, cache)
            counts.append(batch.dispatch_count())
            batch.commit_and_wait()
            res.append(out.as_array(np.uint16, 512))
        assert np.array_equal(res[0], res[1])
        assert counts[1] <= counts[0]


def test_forward_decode_one_kernel_per_op_matches_oracle(pkg, gpu, oracle):
    """The reference's literal dispatch sequence (no grouping, no fusion) with per-layer input and output scale."""
    ctx, kernels = gpu
    g = pkg.synth.rng(905, 0)
    dims, pld, n_layers = _dims(), 256, 2
    dev, ora, _ = _make(pkg, gpu, g, dims, pld, n_layers, 1, output_scale=0.5)
    dev = pkg.layer.TransformerLayer(dev.params, dev.weights, group_projections=False, fuse_norm_rope=False,
                                     fuse_prologues=False)
    cache = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, 16)
    cache.reset()
    kv = OL.KvState(1, 256, 2, 16)
    xs = g.standard_normal((12, 512), dtype=np.float32).astype(np.float16)
    ple = g.standard_normal(n_layers * pld, dtype=np.float32).astype(np.float16)
    _decode_steps(pkg, gpu, dev, ora, xs, cache, kv, ple, n_layers)
    _same_cache(cache, kv, 12)


@pytest.mark.parametrize("n_rows,start,fused", [(1, 0, True), (5, 0, True), (16, 7, True), (48, 20, True), (130, 3, True),
                                                (5, 0, False), (48, 20, False)])
def test_forward_batch_matches_decode_row_by_row(pkg, gpu, oracle, n_rows, start, fused):
    """layer.rs:542-718 over rows start..start+n equals n single-token steps (oracle) -- with per-layer input
    injection and the output scale on."""
    ctx, kernels = gpu
    g = pkg.synth.rng(903, n_rows)
    dims, pld, n_layers, layer_idx = _dims(), 256, 2, 1
    dev, ora, _ = _make(pkg, gpu, g, dims, pld, n_layers, layer_idx, output_scale=1.25)
    if not fused:    # the reference's literal sequence: one kernel per operation
        dev = pkg.layer.TransformerLayer(dev.params, dev.weights, group_projections=False, fuse_norm_rope=False,
                                         fuse_prologues=False)
    total = start + n_rows
    cache = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, 256)
    cache.reset()
    kv = OL.KvState(1, 256, 2, 256)
    xs = g.standard_normal((total, 512), dtype=np.float32).astype(np.float16)
    ple = g.standard_normal((total, n_layers * pld), dtype=np.float32).astype(np.float16)
    # history: the first `start` positions through single-token decode on both sides
    scratch = pkg.layer.ScratchBuffers(ctx, 512, 1024, 4, 1, 256, pld)
    out1 = pkg.Buffer.empty(ctx, 1024)
    for pos in range(start):
        batch = pkg.CommandBatch(ctx)
        dev.forward_decode(kernels, batch, pkg.Buffer.from_slice(ctx, xs[pos]), out1, pos, scratch, cache,
                           pkg.Buffer.from_slice(ctx, ple[pos]), n_layers)
        batch.commit_and_wait()
        OL.decode_layer(ora, xs[pos], pos, kv, ple[pos],
                        kv_rows=(scratch.k.as_array(np.float16, 256), scratch.v.as_array(np.float16, 256)))
    bs = pkg.layer.BatchScratch(ctx, n_rows, 512, 1024, 4, 1, 256, pld, n_layers)
    inp, out = pkg.Buffer.from_slice(ctx, xs[start:]), pkg.Buffer.empty(ctx, n_rows * 1024)
    ple_buf = pkg.Buffer.from_slice(ctx, ple[start:])
    batch = pkg.CommandBatch(ctx)
    dev.forward_batch(kernels, batch, n_rows, start, inp, out, bs, scratch.ones, cache, (ple_buf, n_layers))
    batch.commit_and_wait()
    got = out.as_array(np.float16, n_rows * 512).reshape(n_rows, 512)
    k_gpu = bs.k.as_array(np.float16, n_rows * 256).reshape(n_rows, 256)
    v_gpu = bs.v.as_array(np.float16, n_rows * 256).reshape(n_rows, 256)
    for r in range(n_rows):
        _step(ora, xs[start + r], start + r, kv, got[r], k_gpu[r], v_gpu[r], f"row {r}", ple[start + r])
    _same_cache(cache, kv, total)
    with pytest.raises(pkg.InvalidArgument):
        dev.forward_batch(kernels, pkg.CommandBatch(ctx), n_rows + 1, 0, inp, out, bs, scratch.ones, cache)


@pytest.mark.parametrize("window,fused", [(0, True), (32, True), (0, False), (32, False)])
def test_forward_decode_batch_turbo_matches_single_sequence(pkg, gpu, oracle, window, fused):
    """layer.rs:731-873: lanes at different positions, each equal to its own single-sequence decode
    (pipeline/batched.rs:649-735 checks the same over greedy steps on the real model)."""
    ctx, kernels = gpu
    g = pkg.synth.rng(904, window)
    dims, n_lanes, lane_cap = _dims(), 3, 1024 if window else 128
    ring = pkg.kv_cache.swa_ring_capacity(window, lane_cap) if window else 0
    assert ring in (0, 512)
    dev, ora, _ = _make(pkg, gpu, g, dims, extra=dict(sliding_window=window))
    if not fused:
        dev = pkg.layer.TransformerLayer(dev.params, dev.weights, group_projections=False, fuse_norm_rope=False,
                                         fuse_prologues=False)
    pool = pkg.kv_cache.QuantizedUnifiedKvPool(ctx, n_lanes, lane_cap, 1, 256, 2, ring)
    pool.reset()
    kvs = [OL.KvState(1, 256, 2, lane_cap, ring_capacity=ring) for _ in range(n_lanes)]
    # lane l starts with a prefill of `pre[l]` positions computed by single-sequence decode into a staging cache
    pre = [0, 11, 45 if not window else ring + 5]
    bs = pkg.layer.BatchScratch(ctx, n_lanes, 512, 1024, 4, 1, 256, 0, 1)
    scratch = pkg.layer.ScratchBuffers(ctx, 512, 1024, 4, 1, 256, 0)
    out1 = pkg.Buffer.empty(ctx, 1024)
    for lane, n in enumerate(pre):
        if ring:
            stage = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, lane_cap, 2, ring, window)
        else:
            stage = pkg.kv_cache.QuantizedKvCache(ctx, 1, 256, lane_cap)
        stage.reset()
        hist = g.standard_normal((n, 512), dtype=np.float32).astype(np.float16)
        for pos in range(n):
            batch = pkg.CommandBatch(ctx)
            dev.forward_decode(kernels, batch, pkg.Buffer.from_slice(ctx, hist[pos]), out1, pos, scratch, stage)
            batch.commit_and_wait()
            OL.decode_layer(ora, hist[pos], pos, kvs[lane],
                            kv_rows=(scratch.k.as_array(np.float16, 256), scratch.v.as_array(np.float16, 256)))
        batch = pkg.CommandBatch(ctx)
        pool.copy_prefill_from(batch, stage, lane, n)
        batch.commit_and_wait()
    positions = np.array(pre, np.uint32)
    pos_buf = pkg.Buffer.from_slice(ctx, positions)
    out = pkg.Buffer.empty(ctx, n_lanes * 1024)
    for step in range(6):
        xs = g.standard_normal((n_lanes, 512), dtype=np.float32).astype(np.float16)
        pos_buf.copy_from_bytes(positions)
        batch = pkg.CommandBatch(ctx)
        dev.forward_decode_batch_turbo(batch, kernels, n_lanes, pos_buf, pkg.Buffer.from_slice(ctx, xs), out, bs,
                                       scratch.ones, pool)
        batch.commit_and_wait()
        got = out.as_array(np.float16, n_lanes * 512).reshape(n_lanes, 512)
        k_gpu = bs.k.as_array(np.float16, n_lanes * 256).reshape(n_lanes, 256)
        v_gpu = bs.v.as_array(np.float16, n_lanes * 256).reshape(n_lanes, 256)
        for lane in range(n_lanes):
            _step(ora, xs[lane], int(positions[lane]), kvs[lane], got[lane], k_gpu[lane], v_gpu[lane],
                  f"step {step} lane {lane} at position {positions[lane]}")
        positions += 1
    stride = pool.lane_stride()
    for lane in range(n_lanes):          # lane l's region of the pool holds exactly the oracle's lane cache
        lane_view = type("LaneView", (), {})()
        for name, unit in (("keys_q", pool._cb), ("values_q", pool._cb), ("key_norms", 2), ("value_norms", 2)):
            setattr(lane_view, name, getattr(pool, name).view(lane * stride * unit, stride * unit))
        _same_cache(lane_view, kvs[lane], stride)


def _seeded_f16(n, seed):
    """The reference test's generator (quant_unified_pool.rs:360-371): splitmix64 -> [-0.5, 0.5) f16."""
    M = (1 << 64) - 1
    s, out = seed | 1, np.empty(n, np.float32)
    for i in range(n):
        s = (s + 0x9E3779B97F4A7C15) & M
        z = s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z ^= z >> 31
        out[i] = np.float32(z >> 40) / np.float32(1 << 24) - np.float32(0.5)
    return out.astype(np.float16)


def test_batched_ring_pool_matches_full_after_lane_wrap(pkg, gpu):
    """quant_unified_pool.rs:377-459, same sizes and seeds: 2 lanes, head_dim 128, 4-bit codes, window 64,
    each lane wrapped twice-plus; attention out of the ringed pool equals the absolute pool's bit for bit."""
    ctx, kernels = gpu
    n_lanes, n_kv, hd, n_q, window = 2, 1, 128, 2, 64
    cap = pkg.kv_cache.swa_ring_capacity(window, 4096)
    assert cap == 512          # max(2 * 64, 64 + 255) rounded up to a power of two (quant_cache.rs:48-54)
    total = cap * 2 + 11
    full = pkg.kv_cache.QuantizedUnifiedKvPool(ctx, n_lanes, 4096, n_kv, hd, 4, 0)
    ring = pkg.kv_cache.QuantizedUnifiedKvPool(ctx, n_lanes, 4096, n_kv, hd, 4, cap)
    full.reset()
    ring.reset()
    pos_buf = pkg.Buffer.empty(ctx, n_lanes * 4)
    for pos in range(total):
        k = np.concatenate([_seeded_f16(n_kv * hd, 1 + pos * 7 + lane) for lane in range(n_lanes)])
        v = np.concatenate([_seeded_f16(n_kv * hd, 9001 + pos * 7 + lane) for lane in range(n_lanes)])
        k_src, v_src = pkg.Buffer.from_slice(ctx, k), pkg.Buffer.from_slice(ctx, v)
        pos_buf.copy_from_bytes(np.full(n_lanes, pos, np.uint32))
        batch = pkg.CommandBatch(ctx)
        for pool in (full, ring):
            pool.write_kv_into(batch, kernels, k_src, v_src, pos_buf, n_lanes)
        batch.commit_and_wait()
    pos_buf.copy_from_bytes(np.full(n_lanes, total - 1, np.uint32))
    q = _seeded_f16(n_lanes * n_q * hd, 4242)

    def run(pool):
        q_buf = pkg.Buffer.from_slice(ctx, q)
        rq, vacc = pkg.Buffer.empty(ctx, q.size * 4), pkg.Buffer.empty(ctx, q.size * 4)
        out = pkg.Buffer.empty(ctx, q.size * 2)
        batch = pkg.CommandBatch(ctx)
        pool.attention_into(batch, kernels, q_buf, rq, vacc, out, pos_buf, n_q, window, n_lanes)
        batch.commit_and_wait()
        return out.as_array(np.uint16, q.size)

    a, b = run(full), run(ring)
    assert a.any()
    assert np.array_equal(a, b)
    ring.reset_lane(1)
    c = run(ring)
    # a cleared lane decodes to zero (of either sign); the other lane is untouched
    assert np.array_equal(c[:n_q * hd], a[:n_q * hd]) and not c[n_q * hd:].view(np.float16).any()
