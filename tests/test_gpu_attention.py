"""GPU parity of the fused TurboQuant attention kernels against the f64 code-space oracle.
Mirrors local-metal/src/kernels.rs:9936-10125 (fused vs dequant-then-flash), 10126-10456
(prefill vs per-row decode, tiled vs non-tiled), 10457 (batched) and
local-engine/src/kv_cache/quant_cache.rs:1047-1107 (ring == full)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ATTN_TOL = 2e-3   # max |delta| <= tol * max(max|ref|, 1e-3), kernels.rs:10105-10114


def build_cache(pkg, oracle, T, n_kv, hd, bits, seed, ring=0, scale=1.0):
    g = pkg.synth.rng(6, seed)
    k = (pkg.synth.kv_rows(T, n_kv, hd, g).astype(np.float32) * scale).astype(np.float16)
    v = pkg.synth.kv_rows(T, n_kv, hd, g)
    signs, levels = oracle.rotation_signs(hd, oracle.TQ_SEED), oracle.tq_levels(hd, bits)
    cb = oracle.tq_code_bytes(hd, bits)
    phys = ring if ring else T
    kc = np.zeros((phys, n_kv, cb), np.uint8); vc = np.zeros_like(kc)
    kn = np.zeros((phys, n_kv), np.uint16); vn = np.zeros_like(kn)
    oracle.tq_write_kv(k.view(np.uint16), n_kv, hd, bits, signs, levels, 0, ring, kc, kn)
    oracle.tq_write_kv(v.view(np.uint16), n_kv, hd, bits, signs, levels, 0, ring, vc, vn)
    return signs, levels, kc, kn, vc, vn


def check(got, ref, label, tol=ATTN_TOL):
    err = float(np.max(np.abs(got - ref)))
    scale = max(float(np.max(np.abs(ref))), 1e-3)
    assert err <= tol * scale, f"{label}: max|delta| {err:.3e} > {tol} * {scale:.3e}"
    return err / scale


def upload(pkg, ctx, *arrays):
    return [pkg.Buffer.from_slice(ctx, a) for a in arrays]


@pytest.mark.parametrize("hd,nq,nkv,T,bits,window,qscale", [
    (128, 4, 2, 24, 4, 0, 1.0),        # the reference's own fused-attention test shape
    (256, 8, 1, 300, 2, 0, 1.0),       # measured configuration, short context
    (256, 8, 1, 4096, 2, 0, 1.0),
    (256, 8, 1, 1000, 2, 512, 1.0),    # sliding window
    (256, 8, 1, 777, 3, 0, 0.3),
    (512, 8, 1, 200, 2, 0, 0.2),
    (64, 6, 3, 90, 4, 16, 0.5),
    (256, 16, 1, 100, 2, 0, 0.3),      # more than 8 query heads per KV head
    (128, 2, 2, 1, 2, 0, 1.0),         # one position
    (256, 8, 1, 1, 2, 0, 1.0),         # matrix-core path: one position
    (256, 8, 1, 255, 2, 0, 1.0),       # just under / at / over one 256-position block
    (256, 8, 1, 256, 2, 0, 1.0),
    (256, 8, 1, 257, 2, 0, 1.0),
    (256, 4, 1, 700, 2, 0, 1.0),       # fewer than 8 query heads per KV head (padded MFMA rows)
    (256, 8, 2, 1300, 2, 300, 1.0),    # two KV heads, window not aligned to the block size
    (256, 6, 3, 513, 2, 0, 0.5),
    (256, 8, 1, 20000, 2, 0, 0.25),    # long context, soft attention (many positions carry weight)
    (512, 8, 1, 1, 2, 0, 1.0),         # head_dim 512 (full-attention layers): two V waves per workgroup
    (512, 8, 1, 257, 2, 0, 0.3),
    (512, 8, 1, 2500, 2, 0, 0.3),
    (512, 8, 2, 1300, 2, 300, 0.3),
    (512, 4, 1, 700, 2, 512, 0.3),
    (512, 8, 1, 20000, 2, 0, 0.15),
])
def test_decode_attention_matches_oracle(pkg, gpu, oracle, hd, nq, nkv, T, bits, window, qscale):
    print(f"case hd={hd} nq={nq} nkv={nkv} T={T} bits={bits} window={window}", flush=True)
    ctx, K = gpu
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, T + bits)
    q = (pkg.synth.rng(6, 999).standard_normal((nq, hd), dtype=np.float32) * qscale).astype(np.float16)
    rq_ref = oracle.hadamard_rotate(q.astype(np.float32), signs, hd, nq, True, False)
    acc_ref = oracle.attention_tq_codespace(rq_ref, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, window, bits, 0)
    kcb, knb, vcb, vnb, lvb, sgb, qb = upload(pkg, ctx, kc, kn, vc, vn, levels, signs, q)
    rq, vacc = pkg.Buffer.empty(ctx, nq * hd * 4), pkg.Buffer.empty(ctx, nq * hd * 4)
    out = pkg.Buffer.empty(ctx, nq * hd * 4)
    batch = pkg.CommandBatch(ctx)
    K.hadamard_rotate_hf_into(batch, qb, sgb, rq, hd, nq, True, False)
    K.flash_attention_tq_into(batch, rq, kcb, knb, vcb, vnb, lvb, vacc, hd, T, T - 1, nq, nkv, window, bits, 0)
    K.hadamard_rotate_into(batch, vacc, sgb, out, hd, nq, False, True)
    batch.commit_and_wait()
    e1 = check(vacc.as_array(np.float32), acc_ref, "rotated-space accumulation")
    ref = oracle.hadamard_rotate(acc_ref, signs, hd, nq, False, True)
    e2 = check(out.as_array(np.float32), ref, "attention output")
    # element-wise form too: |g - w| <= tol * max(|w|, 1)
    assert np.max(np.abs(out.as_array(np.float32) - ref) / np.maximum(np.abs(ref), 1.0)) <= ATTN_TOL
    print(f"  err rotated {e1:.2e}, output {e2:.2e}")


@pytest.mark.parametrize("T", [300, 5000])
def test_decode_attention_with_asymmetric_levels(pkg, gpu, oracle, T):
    """A level table that is not affine in the code bits (L3 - L2 != L1 - L0) takes the third bit plane."""
    ctx, K = gpu
    hd, nq, nkv, bits = 256, 8, 1, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 31 + T)
    levels = (levels * np.array([1.0, 1.3, 0.8, 1.1], np.float32)).astype(np.float32)
    rq = pkg.synth.rng(6, 17).standard_normal(nq * hd, dtype=np.float32) * 0.5
    ref = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, 0, bits, 0)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    out = pkg.Buffer.empty(ctx, nq * hd * 4)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, T - 1, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    check(out.as_array(np.float32), ref, "asymmetric levels")


def test_decode_attention_vs_reference_cpu_path(pkg, gpu, oracle):
    """Against the CPU path the reference would run: TurboQuant::decode of every position, then
    f32 attention in the original space."""
    ctx, K = gpu
    hd, nq, nkv, T, bits = 256, 8, 1, 512, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 4242)
    q = pkg.synth.rng(6, 5).standard_normal((nq, hd), dtype=np.float32).astype(np.float16)
    cache = pkg.QuantizedKvCache(ctx, nkv, hd, T, bits)
    cache.keys_q.copy_from_bytes(kc); cache.key_norms.copy_from_bytes(kn)
    cache.values_q.copy_from_bytes(vc); cache.value_norms.copy_from_bytes(vn)
    qb = pkg.Buffer.from_slice(ctx, q)
    rq, vacc = pkg.Buffer.empty(ctx, nq * hd * 4), pkg.Buffer.empty(ctx, nq * hd * 4)
    out = pkg.Buffer.empty(ctx, nq * hd * 2)
    batch = pkg.CommandBatch(ctx)
    cache.fused_attention_into(batch, K, qb, rq, vacc, out, T, T - 1, nq, 0)
    batch.commit_and_wait()
    ref = oracle.attention_tq_decode_then_attend(q.astype(np.float32), kc, kn, vc, vn, levels, signs, hd, T, T - 1, nq, nkv,
                                                 0, bits, 0, threads=8)
    check(out.as_array(np.float16).astype(np.float32), ref, "fused vs decode-then-attend", tol=ATTN_TOL + 1e-3)  # + f16 store


@pytest.mark.parametrize("T,sink", [(4096, 0), (20000, 7000), (3000, 2999)])
def test_attention_sink_with_flat_tail(pkg, gpu, oracle, T, sink):
    """One position whose key is aligned with every query head (its weight ~ e^11 times a typical one) in a context
    whose other weights are nearly flat: the tail carries several per cent of the mass in weights of about half a
    fixed-point step of the sink's.  The value weights are scaled per head and 64 or 128 positions, so only the sink's
    own neighbours are measured against it."""
    print(f"case T={T} sink at {sink}", flush=True)
    ctx, K = gpu
    hd, nq, nkv, bits = 256, 8, 1, 2
    g = pkg.synth.rng(6, 77 + T)
    q = (g.standard_normal((nq, hd), dtype=np.float32) * 0.05).astype(np.float16)
    k = (pkg.synth.kv_rows(T, nkv, hd, g).astype(np.float32) * 0.5).astype(np.float16)
    v = pkg.synth.kv_rows(T, nkv, hd, g)
    qsum = q.astype(np.float32).sum(axis=0)
    k[sink, 0] = (qsum * (11.0 / max(float(np.min(q.astype(np.float32) @ qsum)), 1e-6))).astype(np.float16)   # q_h . k_sink >= 11 for every head
    signs, levels = oracle.rotation_signs(hd, oracle.TQ_SEED), oracle.tq_levels(hd, bits)
    cb = oracle.tq_code_bytes(hd, bits)
    kc = np.zeros((T, nkv, cb), np.uint8); vc = np.zeros_like(kc)
    kn = np.zeros((T, nkv), np.uint16); vn = np.zeros_like(kn)
    oracle.tq_write_kv(k.view(np.uint16), nkv, hd, bits, signs, levels, 0, 0, kc, kn)
    oracle.tq_write_kv(v.view(np.uint16), nkv, hd, bits, signs, levels, 0, 0, vc, vn)
    rq_ref = oracle.hadamard_rotate(q.astype(np.float32), signs, hd, nq, True, False)
    acc_ref = oracle.attention_tq_codespace(rq_ref, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, 0, bits, 0)
    kcb, knb, vcb, vnb, lvb, sgb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, signs, rq_ref)
    vacc, out = pkg.Buffer.empty(ctx, nq * hd * 4), pkg.Buffer.empty(ctx, nq * hd * 4)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rqb, kcb, knb, vcb, vnb, lvb, vacc, hd, T, T - 1, nq, nkv, 0, bits, 0)
    K.hadamard_rotate_into(batch, vacc, sgb, out, hd, nq, False, True)
    batch.commit_and_wait()
    e1 = check(vacc.as_array(np.float32), acc_ref, "rotated-space accumulation")
    ref = oracle.hadamard_rotate(acc_ref, signs, hd, nq, False, True)
    e2 = check(out.as_array(np.float32), ref, "attention output")
    print(f"  err rotated {e1:.2e}, output {e2:.2e}")


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_randomised_shapes_match_oracle(pkg, gpu, oracle, seed):
    """Sixty random shapes per seed -- decode, batched lanes and prefill rows; head_dim 256 / 512; 1, 4, 6 or 8 query heads
    per KV head over one or two KV heads; context lengths around the 64- and 128-position boundaries and up to 33000
    (long enough for the eight-wave workgroups of several chunks, with one-group and with pair hand-overs);
    windows, wrapped rings; peaked to nearly uniform queries; now and then a level table that needs the third bit plane --
    over caches of random code bytes and norms (any code bytes and positive f16 norms are a valid cache)."""
    ctx, K = gpu
    bits = 2
    worst = 0.0
    for case in range(60):
        g = np.random.default_rng(seed * 1000 + case)
        hd = int(g.choice([256, 256, 512]))
        nkv = int(g.choice([1, 1, 2]))
        nq = nkv * int(g.choice([8, 8, 4, 1, 6]))
        mode = int(g.choice([0, 0, 1, 2]))          # 0 decode, 1 batched, 2 prefill
        T = int(g.choice([1, 63, 64, 65, 127, 128, 129, 255, 300, 1000, 1025, 2049, 4096, 5000, 9000, 20000, 33000]))
        T = max(1, T + int(g.integers(-2, 3)))
        window = int(g.choice([0, 0, 64, 100, 512, 1024, 3000]))
        ring = 0
        if window and mode != 1 and g.random() < 0.5:
            ring = ((window + 63) // 64) * 64 * int(g.choice([1, 2]))
        qscale = float(g.choice([1.0, 0.3, 0.1, 0.02])) / 16
        cb = oracle.tq_code_bytes(hd, bits)
        levels = oracle.tq_levels(hd, bits)
        if g.random() < 0.15:
            levels = levels.copy(); levels[3] += 0.2
        lanes, cap = 1, 0
        if mode == 1:
            lanes = int(g.choice([1, 3, 5])); cap = T + int(g.integers(0, 70))
            positions = g.integers(0, T, lanes).astype(np.uint32); positions[0] = T - 1
        phys = lanes * cap if mode == 1 else (ring if ring else T)
        kc = g.integers(0, 256, (phys, nkv, cb), dtype=np.uint8); vc = g.integers(0, 256, (phys, nkv, cb), dtype=np.uint8)
        kn = (g.random((phys, nkv), dtype=np.float32) * 4 + 14).astype(np.float16).view(np.uint16)
        vn = (g.random((phys, nkv), dtype=np.float32) * 4 + 14).astype(np.float16).view(np.uint16)
        what = f"seed {seed} case {case}: mode={mode} hd={hd} nq={nq} nkv={nkv} T={T} window={window} ring={ring} lanes={lanes}"
        print(what, flush=True)
        batch = pkg.CommandBatch(ctx)
        if mode == 0:
            rq = g.standard_normal((1, nq * hd), dtype=np.float32) * qscale
            b = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
            out = pkg.Buffer.empty(ctx, rq.nbytes)
            K.flash_attention_tq_into(batch, b[5], b[0], b[1], b[2], b[3], b[4], out, hd, T, T - 1, nq, nkv, window, bits, ring)
            refs = [lambda: oracle.attention_tq_codespace(rq[0], kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, window, bits, ring)]
        elif mode == 1:
            rq = g.standard_normal((lanes, nq * hd), dtype=np.float32) * qscale
            b = upload(pkg, ctx, kc, kn, vc, vn, levels, rq, positions)
            out = pkg.Buffer.empty(ctx, rq.nbytes)
            K.flash_attention_tq_batched_into(batch, b[5], b[0], b[1], b[2], b[3], b[4], out, b[6], hd, cap, nq, nkv, window, bits,
                                              lanes, 0)
            refs = [lambda l=l: oracle.attention_tq_codespace(rq[l], kc, kn, vc, vn, levels, hd, int(positions[l]) + 1,
                                                              int(positions[l]), nq, nkv, window, bits, 0, lane_base=l * cap)
                    for l in range(lanes)]
        else:
            rows = int(min(T, g.choice([1, 3, 17])))
            start = T - rows
            rq = g.standard_normal((rows, nq * hd), dtype=np.float32) * qscale
            b = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
            out = pkg.Buffer.empty(ctx, rq.nbytes)
            K.flash_attention_tq_prefill_tiled_into(batch, b[5], b[0], b[1], b[2], b[3], b[4], out, hd, T, start, rows, nq, nkv,
                                                    window, bits, ring)
            refs = [lambda r=r: oracle.attention_tq_codespace(rq[r], kc, kn, vc, vn, levels, hd, T, start + r, nq, nkv, window,
                                                              bits, ring) for r in range(rows)]
        batch.commit_and_wait()
        got = out.as_array(np.float32).reshape(len(refs), nq * hd)
        for i, ref in enumerate(refs):
            worst = max(worst, check(got[i], ref(), what))
    print(f"worst error / scale {worst:.2e}")


def test_ring_matches_full_cache_bitwise(pkg, gpu, oracle):
    """quant_cache.rs:1047-1107: attention over a wrapped ring is bit-identical to the full cache."""
    ctx, K = gpu
    hd, nq, nkv, bits, T, window, ring = 256, 8, 1, 2, 1500, 512, 512
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 77)
    _, _, rkc, rkn, rvc, rvn = build_cache(pkg, oracle, T, nkv, hd, bits, 77, ring=ring)
    rq = pkg.synth.rng(6, 8).standard_normal(nq * hd, dtype=np.float32)
    lvb, rqb = upload(pkg, ctx, levels, rq)
    outs = []
    for (a, b, c, d, r) in ((kc, kn, vc, vn, 0), (rkc, rkn, rvc, rvn, ring)):
        ab, bb, cb_, db = upload(pkg, ctx, a, b, c, d)
        o = pkg.Buffer.empty(ctx, nq * hd * 4)
        batch = pkg.CommandBatch(ctx)
        K.flash_attention_tq_into(batch, rqb, ab, bb, cb_, db, lvb, o, hd, T, T - 1, nq, nkv, window, bits, r)
        batch.commit_and_wait()
        outs.append(o.as_array(np.float32))
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    ref = oracle.attention_tq_codespace(rq, rkc, rkn, rvc, rvn, levels, hd, T, T - 1, nq, nkv, window, bits, ring)
    check(outs[1], ref, "ring attention")


def test_empty_range_gives_zeros(pkg, gpu, oracle):
    ctx, K = gpu
    hd, nq, nkv, bits = 128, 4, 2, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, 4, nkv, hd, bits, 1)
    bufs = upload(pkg, ctx, kc, kn, vc, vn, levels)
    rq = pkg.Buffer.from_slice(ctx, np.ones(nq * hd, np.float32))
    out = pkg.Buffer.from_slice(ctx, np.full(nq * hd, 7.0, np.float32))
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rq, bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, hd, 0, 0, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    assert np.all(out.as_array(np.float32) == 0)


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("hd,nq,nkv,bits,start,rows,window", [(256, 8, 1, 2, 0, 37, 0), (256, 8, 1, 2, 100, 20, 64),
                                                              (128, 4, 2, 4, 5, 9, 0), (512, 8, 1, 2, 70, 11, 0)])
def test_prefill_matches_per_row_decode(pkg, gpu, oracle, tiled, hd, nq, nkv, bits, start, rows, window):
    """kernels.rs:10126, 10295: every prefill row equals the decode kernel at that position."""
    print(f"case tiled={tiled} hd={hd} rows={rows} start={start}", flush=True)
    ctx, K = gpu
    T = start + rows
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 31 + rows)
    rq = (pkg.synth.rng(6, 12).standard_normal((rows, nq, hd), dtype=np.float32) * 0.5).astype(np.float32)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    out = pkg.Buffer.empty(ctx, rq.nbytes)
    batch = pkg.CommandBatch(ctx)
    fn = K.flash_attention_tq_prefill_tiled_into if tiled else K.flash_attention_tq_prefill_into
    fn(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, start, rows, nq, nkv, window, bits, 0)
    batch.commit_and_wait()
    got = out.as_array(np.float32).reshape(rows, nq * hd)
    for r in range(rows):
        ref = oracle.attention_tq_codespace(rq[r], kc, kn, vc, vn, levels, hd, T, start + r, nq, nkv, window, bits, 0)
        check(got[r], ref, f"row {r}")


@pytest.mark.parametrize("nq,nkv,start,rows,window,ring,qscale", [
    (8, 1, 0, 256, 0, 0, 0.5),          # a whole first chunk: every row's range ends inside the tiles (causal masks everywhere)
    (8, 1, 1000, 61, 0, 0, 1.0),        # rows not a multiple of the sixteen a workgroup takes; chunk ends inside a tile
    (8, 1, 2000, 40, 512, 512, 0.5),    # sliding window over a wrapped 512-slot ring: both ends of the range move with the row
    (4, 2, 300, 19, 0, 0, 1.0),         # two KV heads, two query heads each (padded MFMA rows)
    (8, 1, 5, 9, 3, 0, 1.0),            # a window shorter than the rows per workgroup: rows that share no position
    (8, 1, 6000, 256, 0, 0, 1.0),       # large enough for the tiled kernel by default (256 rows over 6k positions)
    (8, 1, 777, 2, 0, 0, 0.05),         # two rows, nearly flat scores
])
def test_prefill_tiled_rows_share_a_pass(pkg, gpu, oracle, nq, nkv, start, rows, window, ring, qscale):
    """The tiled prefill entry (shaders/attention_flash_tq.metal:425-567): every row against the f64 code-space oracle at
    that row's position, the reference's own check of its tiled kernel against per-row decode (kernels.rs:10295) at the
    attention tolerance.  The output buffer is pre-filled and has guard words behind it.  By default the entry gives
    launches of this size to the per-row kernel; under LOCAL_HIP_ATTN_PREFILL=tiled (tests/test_gpu_switches.py) the same
    cases run on the kernel that shares a pass over the codes among sixteen rows."""
    print(f"case tiled prefill nq={nq} nkv={nkv} start={start} rows={rows} window={window} ring={ring}", flush=True)
    ctx, K = gpu
    hd, bits = 256, 2
    T = start + rows
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 77 + rows, ring=ring)
    rq = (pkg.synth.rng(6, 15 + rows).standard_normal((rows, nq, hd), dtype=np.float32) * np.float32(qscale)).astype(np.float32)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    guard = 64
    out = pkg.Buffer.from_slice(ctx, np.full(rows * nq * hd + guard, 7.5, np.float32))
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_prefill_tiled_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, start, rows, nq, nkv, window, bits, ring)
    batch.commit_and_wait()
    full = out.as_array(np.float32)
    assert (full[rows * nq * hd:] == 7.5).all()
    got = full[:rows * nq * hd].reshape(rows, nq * hd)
    worst = 0.0
    for r in range(rows):
        ref = oracle.attention_tq_codespace(rq[r], kc, kn, vc, vn, levels, hd, T, start + r, nq, nkv, window, bits, ring)
        worst = max(worst, check(got[r], ref, f"row {r}"))
    print(f"worst row: {worst:.2e} of max|ref|")


def test_prefill_randomised_shapes_match_oracle(pkg, gpu, oracle):
    """Forty random prefill launches at head_dim 256 over caches of random code bytes and norms: 2 .. 40 rows (whole and
    partial groups of sixteen, odd counts), 1, 4, 6 or 8 query heads per KV head over one or two KV heads, chunks that
    start at position 0 or deep in the context, ends on and off the 64-position tile boundaries, windows shorter and longer
    than the chunk, wrapped rings, peaked to nearly uniform queries, and now and then a level table with a third-plane
    term.  Every row against the f64 oracle.  (Launches of this size take the per-row kernel by default and the
    sixteen-row kernel under LOCAL_HIP_ATTN_PREFILL=tiled; tests/test_gpu_switches.py runs this test both ways.)"""
    ctx, K = gpu
    hd, bits = 256, 2
    worst = 0.0
    for case in range(40):
        g = np.random.default_rng(7000 + case)
        nkv = int(g.choice([1, 1, 2]))
        nq = nkv * int(g.choice([8, 8, 4, 1, 6]))
        rows = int(g.choice([2, 5, 15, 16, 17, 31, 33, 40]))
        T = rows + int(g.choice([0, 1, 47, 63, 64, 65, 200, 511, 700, 1500, 3000])) + int(g.integers(0, 3))
        start = T - rows
        window = int(g.choice([0, 0, 3, 64, 100, 512, 1024]))
        ring = 0
        if window and g.random() < 0.5:
            ring = ((window + rows + 63) // 64) * 64 * int(g.choice([1, 2]))     # a ring holds the window of every row of the chunk
        qscale = float(g.choice([1.0, 0.3, 0.1, 0.02])) / 16
        levels = oracle.tq_levels(hd, bits)
        if g.random() < 0.2:
            levels = levels.copy(); levels[3] += 0.2
        cb = oracle.tq_code_bytes(hd, bits)
        phys = ring if ring else T
        kc = g.integers(0, 256, (phys, nkv, cb), dtype=np.uint8); vc = g.integers(0, 256, (phys, nkv, cb), dtype=np.uint8)
        kn = (g.random((phys, nkv), dtype=np.float32) * 4 + 14).astype(np.float16).view(np.uint16)
        vn = (g.random((phys, nkv), dtype=np.float32) * 4 + 14).astype(np.float16).view(np.uint16)
        what = f"case {case}: rows={rows} nq={nq} nkv={nkv} T={T} window={window} ring={ring}"
        print(what, flush=True)
        rq = g.standard_normal((rows, nq * hd), dtype=np.float32) * qscale
        b = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
        out = pkg.Buffer.empty(ctx, rq.nbytes)
        batch = pkg.CommandBatch(ctx)
        K.flash_attention_tq_prefill_tiled_into(batch, b[5], b[0], b[1], b[2], b[3], b[4], out, hd, T, start, rows, nq, nkv, window,
                                                bits, ring)
        batch.commit_and_wait()
        got = out.as_array(np.float32).reshape(rows, nq * hd)
        for r in range(rows):
            ref = oracle.attention_tq_codespace(rq[r], kc, kn, vc, vn, levels, hd, T, start + r, nq, nkv, window, bits, ring)
            worst = max(worst, check(got[r], ref, f"{what}, row {r}"))
    print(f"worst error / scale {worst:.2e}")


def test_prefill_tiled_last_chunk_of_a_32k_prompt(pkg, gpu, oracle):
    """The measured prefill shape: the last 256 rows of a 32768-token prompt (each row sees 32513 .. 32768 positions).
    Sixteen rows spread over the chunk against the f64 oracle; all rows finite; and the rows the tiled kernel produced
    (a launch of this size takes it by default) against the single-query entry at each sampled row's position."""
    ctx, K = gpu
    hd, nq, nkv, bits, T, rows = 256, 8, 1, 2, 32768, 256
    start = T - rows
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 32769)
    rq = pkg.synth.rng(6, 16).standard_normal((rows, nq, hd), dtype=np.float32)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    out = pkg.Buffer.empty(ctx, rq.nbytes)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_prefill_tiled_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, start, rows, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    got = out.as_array(np.float32).reshape(rows, nq * hd)
    assert np.isfinite(got).all()
    one = pkg.Buffer.empty(ctx, nq * hd * 4)
    for r in list(range(0, rows, 17)) + [rows - 1]:
        print(f"case 32k prefill row {r}", flush=True)
        ref = oracle.attention_tq_codespace(rq[r], kc, kn, vc, vn, levels, hd, T, start + r, nq, nkv, 0, bits, 0)
        check(got[r], ref, f"row {r}")
        rq1 = pkg.Buffer.from_slice(ctx, rq[r])
        K.flash_attention_tq_into(batch, rq1, kcb, knb, vcb, vnb, lvb, one, hd, T, start + r, nq, nkv, 0, bits, 0)
        batch.commit_and_wait()
        check(got[r], one.as_array(np.float32), f"row {r} against the single-query kernel")


def test_prefill_with_a_level_table_that_is_not_affine(pkg, gpu, oracle):
    """A level table that is not affine in the code bits (the per-row kernel carries a third bit plane for it, the tiled
    kernel looks levels up in the table itself): both prefill entries must follow whatever table the buffer holds, also
    one that is written on the device after the upload."""
    ctx, K = gpu
    hd, nq, nkv, bits, start, rows = 256, 8, 1, 2, 50, 12
    T = start + rows
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 91)
    odd = levels.copy()
    odd[3] = np.float32(odd[3] * 1.3)
    rq = pkg.synth.rng(6, 17).standard_normal((rows, nq, hd), dtype=np.float32)
    kcb, knb, vcb, vnb, lvb, rqb, oddb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq, odd)
    out = pkg.Buffer.empty(ctx, rq.nbytes)
    batch = pkg.CommandBatch(ctx)

    def run_and_check(table_buf, what):
        for fn in (K.flash_attention_tq_prefill_tiled_into, K.flash_attention_tq_prefill_into):
            fn(batch, rqb, kcb, knb, vcb, vnb, table_buf, out, hd, T, start, rows, nq, nkv, 0, bits, 0)
            batch.commit_and_wait()
            got = out.as_array(np.float32).reshape(rows, nq * hd)
            for r in range(rows):
                ref = oracle.attention_tq_codespace(rq[r], kc, kn, vc, vn, odd, hd, T, start + r, nq, nkv, 0, bits, 0)
                check(got[r], ref, f"row {r}, {what}")

    run_and_check(oddb, "non-affine table as uploaded")
    batch.blit_copy(oddb, 0, lvb, 0, 16)      # an uploaded symmetric table overwritten on the device
    run_and_check(lvb, "table overwritten on the device")


@pytest.mark.parametrize("hd", [256, 512])
def test_batched_matches_independent_sequences(pkg, gpu, oracle, hd):
    """kernels.rs:10457: lanes at different positions in one dispatch == separate single-sequence calls."""
    ctx, K = gpu
    nq, nkv, bits, lanes, cap = 8, 1, 2, 4, 600
    cb = oracle.tq_code_bytes(hd, bits)
    positions = np.array([599, 0, 123, 300], np.uint32)
    pool_kc = np.zeros((lanes * cap, nkv, cb), np.uint8); pool_vc = np.zeros_like(pool_kc)
    pool_kn = np.zeros((lanes * cap, nkv), np.uint16); pool_vn = np.zeros_like(pool_kn)
    levels = None
    for l in range(lanes):
        n = int(positions[l]) + 1
        signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, n, nkv, hd, bits, 500 + l)
        pool_kc[l * cap:l * cap + n] = kc; pool_vc[l * cap:l * cap + n] = vc
        pool_kn[l * cap:l * cap + n] = kn; pool_vn[l * cap:l * cap + n] = vn
    rq = pkg.synth.rng(6, 13).standard_normal((lanes, nq * hd), dtype=np.float32)
    bufs = upload(pkg, ctx, pool_kc, pool_kn, pool_vc, pool_vn, levels, rq, positions)
    out = pkg.Buffer.empty(ctx, rq.nbytes)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_batched_into(batch, bufs[5], bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, bufs[6], hd, cap, nq,
                                      nkv, 0, bits, lanes, 0)
    batch.commit_and_wait()
    got = out.as_array(np.float32).reshape(lanes, nq * hd)
    for l in range(lanes):
        ref = oracle.attention_tq_codespace(rq[l], pool_kc, pool_kn, pool_vc, pool_vn, levels, hd, int(positions[l]) + 1,
                                            int(positions[l]), nq, nkv, 0, bits, 0, lane_base=l * cap)
        check(got[l], ref, f"lane {l}")


@pytest.mark.parametrize("lanes,cap", [(32, 32768), (256, 4096)])
def test_batched_long_lanes_merged_in_the_workgroup(pkg, gpu, oracle, lanes, cap):
    """Long chunks of many lanes in one dispatch: four consecutive chunks of a lane share a workgroup that merges them
    itself.  32 lanes of up to 32768 positions: 32 chunks per lane leave eight partial records instead of thirty-two;
    256 lanes of up to 4096: four chunks per lane leave the kernel as the final output, with no merge behind it.  The
    lanes stand at ragged positions -- some shorter than one chunk, one empty but for its first position -- so a
    workgroup holds chunks with different numbers of hand-overs and chunks with nothing in them.  Every checked lane
    against the f64 oracle."""
    print(f"case lanes={lanes} cap={cap}", flush=True)
    ctx, K = gpu
    hd, nq, nkv, bits = 256, 8, 1, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, cap, nkv, hd, bits, 4040)
    g = pkg.synth.rng(6, 40)
    positions = g.integers(cap // 10, cap, lanes).astype(np.uint32)
    positions[:8] = [cap - 1, 0, 63, 64, 130, 1500, cap // 2 + 1, cap - 700]
    pool_kc, pool_vc = np.tile(kc, (lanes, 1, 1)), np.tile(vc, (lanes, 1, 1))
    pool_kn, pool_vn = np.tile(kn, (lanes, 1)), np.tile(vn, (lanes, 1))
    rq = g.standard_normal((lanes, nq * hd), dtype=np.float32)
    rq[1::2] *= 0.15                                    # every other lane a soft distribution
    bufs = upload(pkg, ctx, pool_kc, pool_kn, pool_vc, pool_vn, levels, rq, positions)
    out = pkg.Buffer.empty(ctx, rq.nbytes)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_batched_into(batch, bufs[5], bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, bufs[6], hd, cap, nq,
                                      nkv, 0, bits, lanes, 0)
    batch.commit_and_wait()
    got = out.as_array(np.float32).reshape(lanes, nq * hd)
    assert np.isfinite(got).all()
    for l in list(range(8)) + [11, 24, lanes - 1]:
        print(f"lane {l} at {positions[l]}", flush=True)
        ref = oracle.attention_tq_codespace(rq[l], pool_kc, pool_kn, pool_vc, pool_vn, levels, hd, int(positions[l]) + 1,
                                            int(positions[l]), nq, nkv, 0, bits, 0, lane_base=l * cap)
        check(got[l], ref, f"lane {l} at {positions[l]}")


def test_batched_hand_over_that_gives_up_is_reported(pkg, gpu, oracle):
    """The K wave and the V wave of a chunk meet at their hand-overs through counters in LDS, with a bounded poll.  With the
    poll budget forced to zero from the host a wave that arrives early goes on at once: every wave still runs to the end of
    the kernel, and the wait on the batch must report it as a command-buffer error instead of returning outputs that may be
    wrong.  With the budget restored the same launch is clean and equals the launch made before the budget was touched,
    bit for bit, and the oracle."""
    import ctypes as C
    ctx, K = gpu
    hd, nq, nkv, bits, lanes, cap = 256, 8, 1, 2, 256, 4096     # four chunks of 1024 positions per lane, one workgroup per lane
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, cap, nkv, hd, bits, 5151)
    g = pkg.synth.rng(6, 51)
    positions = g.integers(cap // 2, cap, lanes).astype(np.uint32)
    pool_kc, pool_vc = np.tile(kc, (lanes, 1, 1)), np.tile(vc, (lanes, 1, 1))
    pool_kn, pool_vn = np.tile(kn, (lanes, 1)), np.tile(vn, (lanes, 1))
    rq = g.standard_normal((lanes, nq * hd), dtype=np.float32)
    bufs = upload(pkg, ctx, pool_kc, pool_kn, pool_vc, pool_vn, levels, rq, positions)
    out = pkg.Buffer.empty(ctx, rq.nbytes)
    batch = pkg.CommandBatch(ctx)

    def launch():
        K.flash_attention_tq_batched_into(batch, bufs[5], bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], out, bufs[6], hd, cap, nq,
                                          nkv, 0, bits, lanes, 0)
        batch.commit_and_wait()
        return out.as_array(np.float32).reshape(lanes, nq * hd).copy()

    before = launch()
    setter = pkg.lib().lh_debug_set_attention_pair_spin_limit
    setter.restype = None
    seen = False
    try:
        setter(C.c_uint32(0))
        for _ in range(5):
            try:
                launch()
            except pkg.CommandBuffer as e:
                assert "gave up waiting for its partner" in str(e)
                seen = True
                break
    finally:
        setter(C.c_uint32(1 << 22))
    assert seen, "no wave of 5 launches ever had to wait: the forced give-up path was not reached"
    after = launch()                 # clean again: the fault word was cleared when it was reported
    assert np.array_equal(before, after)
    for l in (0, lanes // 2, lanes - 1):
        ref = oracle.attention_tq_codespace(rq[l], pool_kc, pool_kn, pool_vc, pool_vn, levels, hd, int(positions[l]) + 1,
                                            int(positions[l]), nq, nkv, 0, bits, 0, lane_base=l * cap)
        check(after[l], ref, f"lane {l} after the budget was restored")


def test_split_invariance_at_32k(pkg, gpu, oracle):
    """Full-size configuration (32768 cached positions, 8 q heads / 1 kv head, hd 256, 2 bits):
    parity with the f64 oracle, and the SWA-ring configuration (window 512, ring 512, wrapped)."""
    ctx, K = gpu
    hd, nq, nkv, bits, T = 256, 8, 1, 2, 32768
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 32768)
    q = pkg.synth.rng(6, 14).standard_normal((nq, hd), dtype=np.float32).astype(np.float16)
    rq = oracle.hadamard_rotate(q.astype(np.float32), signs, hd, nq, True, False)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    out = pkg.Buffer.empty(ctx, nq * hd * 4)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, T - 1, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    ref = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, 0, bits, 0)
    e = check(out.as_array(np.float32), ref, "32k full attention")
    print(f"32k: {e:.2e}")
    _, _, rkc, rkn, rvc, rvn = build_cache(pkg, oracle, 3000, nkv, hd, bits, 3000, ring=512)
    bufs = upload(pkg, ctx, rkc, rkn, rvc, rvn)
    K.flash_attention_tq_into(batch, rqb, bufs[0], bufs[1], bufs[2], bufs[3], lvb, out, hd, 3000, 2999, nq, nkv, 512, bits, 512)
    batch.commit_and_wait()
    ref = oracle.attention_tq_codespace(rq, rkc, rkn, rvc, rvn, levels, hd, 3000, 2999, nq, nkv, 512, bits, 512)
    check(out.as_array(np.float32), ref, "SWA ring 512")


@pytest.mark.parametrize("T", [16384, 131072])
@pytest.mark.parametrize("qscale", [1.0, 0.15])
def test_context_sweep_long(pkg, gpu, oracle, T, qscale):
    """The long ends of the measured context sweep (8 q heads / 1 kv head, hd 256, 2 bits, one query, full attention):
    a peaked distribution (q from N(0, 1)) and a soft one (q * 0.15, thousands of positions carry weight, which is what
    stresses the 16-bit fixed-point value weights, scaled per head and 64 or 128 positions).  Rotated-space output against the f64
    code-space oracle, and the rotated-back f16 output of the one-call entry."""
    print(f"case T={T} qscale={qscale}", flush=True)
    ctx, K = gpu
    hd, nq, nkv, bits = 256, 8, 1, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, T + 3)
    q = (pkg.synth.rng(6, 21).standard_normal((nq, hd), dtype=np.float32) * qscale).astype(np.float16)
    rq = oracle.hadamard_rotate(q.astype(np.float32), signs, hd, nq, True, False)
    kcb, knb, vcb, vnb, lvb, rqb, sgb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq, signs)
    out, out2 = pkg.Buffer.empty(ctx, nq * hd * 4), pkg.Buffer.empty(ctx, nq * hd * 4)
    o16 = pkg.Buffer.empty(ctx, nq * hd * 2)
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, T - 1, nq, nkv, 0, bits, 0)
    K.flash_attention_tq_rotated_into(batch, rqb, kcb, knb, vcb, vnb, lvb, sgb, out2, o16, hd, T, T - 1, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    ref = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, 0, bits, 0)
    e = check(out.as_array(np.float32), ref, f"T={T} rotated space")
    back = oracle.hadamard_rotate(np.asarray(ref, np.float32).reshape(nq, hd), signs, hd, nq, False, True)
    e2 = check(o16.as_array(np.float16).astype(np.float32), np.asarray(back, np.float32).reshape(-1), f"T={T} output", 3e-3)
    print(f"  T={T} qscale={qscale}: err rotated {e:.2e}, f16 output {e2:.2e}")


@pytest.mark.parametrize("hd,T,window,ring", [(256, 700, 512, 512), (256, 40, 0, 0), (256, 1500, 0, 0), (512, 900, 0, 0),
                                              (256, 9000, 0, 0), (256, 3, 0, 0), (128, 300, 0, 0)])
def test_rotated_entry_equals_attention_then_rotation(pkg, gpu, oracle, hd, T, window, ring):
    """quant_cache.rs:571-598: attend, then rotate back.  The one-call form (merge and rotation in one kernel for 2..32
    splits, the separate kernels otherwise; head_dim 128 takes the vector-ALU attention) must give the f16 head outputs of
    the two calls bit for bit, and those must match the oracle's attention and rotation."""
    ctx, K = gpu
    nq, nkv, bits = 8, 1, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 900 + T, ring=ring)
    rq = pkg.synth.rng(6, 15).standard_normal((nq, hd), dtype=np.float32)
    kcb, knb, vcb, vnb, lvb, rqb, sgb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq, signs)
    acc = [pkg.Buffer.empty(ctx, nq * hd * 4) for _ in range(3)]
    o16 = [pkg.Buffer.from_slice(ctx, np.full(nq * hd + 32, 0x7BFF, np.uint16)) for _ in range(3)]
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rqb, kcb, knb, vcb, vnb, lvb, acc[0], hd, T, T - 1, nq, nkv, window, bits, ring)
    K.hadamard_rotate_fh_into(batch, acc[0], sgb, o16[0], hd, nq, False, True)
    K.flash_attention_tq_rotated_into(batch, rqb, kcb, knb, vcb, vnb, lvb, sgb, acc[1], o16[1], hd, T, T - 1, nq, nkv, window,
                                      bits, ring)
    d0 = batch.dispatch_count()
    rotated = K.flash_attention_tq_rotated_lazy_into(batch, rqb, kcb, knb, vcb, vnb, lvb, sgb, acc[2], o16[2], hd, T, T - 1, nq,
                                                     nkv, window, bits, ring)
    lazy_dispatches = batch.dispatch_count() - d0
    batch.commit_and_wait()
    two, one = o16[0].as_array(np.uint16), o16[1].as_array(np.uint16)
    assert (one[nq * hd:] == 0x7BFF).all()
    assert np.array_equal(one, two), f"{int((one != two).sum())} of {nq * hd} f16 outputs differ"
    # the lazy form: either the rotated heads (the rotation rode in the merge launch), or the f32 heads of the attend step
    # alone and nothing written to the f16 buffer -- never a rotation launch of its own
    assert lazy_dispatches <= 2
    if rotated:
        assert np.array_equal(o16[2].as_array(np.uint16), two)
    else:
        assert (o16[2].as_array(np.uint16) == 0x7BFF).all()
        assert np.array_equal(acc[2].as_array(np.uint32), acc[0].as_array(np.uint32))
    ref = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, window, bits, ring)
    ref = oracle.hadamard_rotate(np.asarray(ref, np.float32).reshape(nq, hd), signs, hd, nq, False, True)
    check(one[:nq * hd].view(np.float16).astype(np.float32), np.asarray(ref, np.float32).reshape(-1), "rotated attention", 3e-3)


@pytest.mark.parametrize("hd,lanes,cap", [(256, 5, 600), (512, 3, 700), (256, 40, 256)])
def test_batched_rotated_entry_equals_attention_then_rotation(pkg, gpu, oracle, hd, lanes, cap):
    """quant_unified_pool.rs:225-256 as one call: lanes at different positions (one of them at position 0, so some of its
    splits are empty), f16 head outputs equal to the two calls' bit for bit."""
    ctx, K = gpu
    nq, nkv, bits = 8, 1, 2
    cb = oracle.tq_code_bytes(hd, bits)
    g = pkg.synth.rng(6, 16)
    positions = g.integers(0, cap, lanes).astype(np.uint32)
    positions[0], positions[-1] = cap - 1, 0
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, lanes * cap, nkv, hd, bits, 77)
    rq = g.standard_normal((lanes, nq * hd), dtype=np.float32)
    bufs = upload(pkg, ctx, kc, kn, vc, vn, levels, rq, positions, signs)
    acc = [pkg.Buffer.empty(ctx, rq.nbytes) for _ in range(2)]
    o16 = [pkg.Buffer.empty(ctx, rq.nbytes // 2) for _ in range(2)]
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_batched_into(batch, bufs[5], bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], acc[0], bufs[6], hd, cap, nq,
                                      nkv, 0, bits, lanes, 0)
    K.hadamard_rotate_fh_into(batch, acc[0], bufs[7], o16[0], hd, lanes * nq, False, True)
    K.flash_attention_tq_batched_rotated_into(batch, bufs[5], bufs[0], bufs[1], bufs[2], bufs[3], bufs[4], bufs[7], acc[1],
                                              o16[1], bufs[6], hd, cap, nq, nkv, 0, bits, lanes, 0)
    batch.commit_and_wait()
    two, one = o16[0].as_array(np.uint16), o16[1].as_array(np.uint16)
    assert np.array_equal(one, two), f"{int((one != two).sum())} of {one.size} f16 outputs differ"
    l = lanes // 2
    ref = oracle.attention_tq_codespace(rq[l], kc, kn, vc, vn, levels, hd, int(positions[l]) + 1, int(positions[l]), nq, nkv,
                                        0, bits, 0, lane_base=l * cap)
    ref = oracle.hadamard_rotate(np.asarray(ref, np.float32).reshape(nq, hd), signs, hd, nq, False, True)
    got = one.reshape(lanes, nq * hd)[l].view(np.float16).astype(np.float32)
    check(got, np.asarray(ref, np.float32).reshape(-1), f"lane {l}", 3e-3)


def test_rotated_entry_arguments(pkg, gpu, oracle):
    """The one-call form checks the two extra buffers like the others."""
    ctx, K = gpu
    hd, nq, nkv, bits, T = 256, 8, 1, 2, 100
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 5)
    rq = np.zeros((nq, hd), np.float32)
    kcb, knb, vcb, vnb, lvb, rqb, sgb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq, signs)
    acc, o16 = pkg.Buffer.empty(ctx, nq * hd * 4), pkg.Buffer.empty(ctx, nq * hd * 2)
    batch = pkg.CommandBatch(ctx)
    with pytest.raises(pkg.InvalidArgument):
        K.flash_attention_tq_rotated_into(batch, rqb, kcb, knb, vcb, vnb, lvb, sgb, acc, pkg.Buffer.empty(ctx, nq * hd), hd, T,
                                          T - 1, nq, nkv, 0, bits, 0)
    with pytest.raises(pkg.InvalidArgument):
        K.flash_attention_tq_rotated_into(batch, rqb, kcb, knb, vcb, vnb, lvb, pkg.Buffer.empty(ctx, hd * 2), acc, o16, hd, T,
                                          T - 1, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
