"""GPU parity of the TurboQuant KV kernels against the CPU codec, through the C ABI.
Mirrors local-metal/src/kernels.rs:9823-9935 (encode vs CPU), 10714 (encode->decode),
10457 (batched == independent) and local-engine/src/kv_cache/quant_cache.rs:789-1107."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def codec(oracle, hd, bits):
    return oracle.rotation_signs(hd, oracle.TQ_SEED), oracle.tq_levels(hd, bits)


def cpu_cache(oracle, rows, n_kv, hd, bits, position, ring, phys):
    signs, levels = codec(oracle, hd, bits)
    cb = oracle.tq_code_bytes(hd, bits)
    codes = np.zeros((phys, n_kv, cb), np.uint8)
    norms = np.zeros((phys, n_kv), np.uint16)
    oracle.tq_write_kv(rows.view(np.uint16), n_kv, hd, bits, signs, levels, position, ring, codes, norms)
    return codes, norms


@pytest.mark.parametrize("hd,n_kv,tokens,bits", [(128, 4, 3, 4), (256, 1, 64, 2), (256, 2, 9, 3), (512, 1, 5, 2),
                                                 (64, 2, 7, 4), (512, 2, 3, 3), (256, 1, 300, 2)])
def test_encode_is_bit_exact(pkg, gpu, oracle, hd, n_kv, tokens, bits):
    """Codes and f16 norms equal the CPU encoder's byte for byte (the reference's own GPU test
    only asks for <2 % one-level flips, kernels.rs:9823-9935)."""
    print(f"case hd={hd} n_kv={n_kv} tokens={tokens} bits={bits}", flush=True)
    ctx, K = gpu
    g = pkg.synth.rng(5, hd * 1000 + tokens * 10 + bits)
    rows = pkg.synth.kv_rows(tokens, n_kv, hd, g)
    rows[0, 0, :] = 0                                        # zero vector -> norm 0 (turboquant.rs:439-450)
    if tokens > 2:
        rows[1] *= np.float16(1e-3)                          # tiny norms
        rows[2] *= np.float16(30.0)
    signs, levels = codec(oracle, hd, bits)
    cb = oracle.tq_code_bytes(hd, bits)
    want_c, want_n = cpu_cache(oracle, rows, n_kv, hd, bits, 0, 0, tokens)
    inp = pkg.Buffer.from_slice(ctx, rows)
    lv, sg = pkg.Buffer.from_slice(ctx, levels), pkg.Buffer.from_slice(ctx, signs)
    packed = pkg.Buffer.empty(ctx, tokens * n_kv * cb)
    norms = pkg.Buffer.empty(ctx, tokens * n_kv * 2)
    K.encode_kv_turboquant(ctx, inp, lv, sg, packed, norms, hd, n_kv, tokens, bits, 0, 0)
    assert np.array_equal(norms.as_array(np.uint16), want_n.reshape(-1))
    assert np.array_equal(packed.as_array(np.uint8), want_c.reshape(-1))


def test_encode_ring_and_position_offsets(pkg, gpu, oracle):
    """Slot = ((position + token) % ring) * n_kv + head (dequantize_kv.metal:236-246)."""
    ctx, K = gpu
    hd, n_kv, bits, ring = 128, 2, 2, 16
    cb = oracle.tq_code_bytes(hd, bits)
    signs, levels = codec(oracle, hd, bits)
    lv, sg = pkg.Buffer.from_slice(ctx, levels), pkg.Buffer.from_slice(ctx, signs)
    g = pkg.synth.rng(5, 77)
    packed = pkg.Buffer.empty(ctx, ring * n_kv * cb)
    norms = pkg.Buffer.empty(ctx, ring * n_kv * 2)
    want_c = np.zeros((ring, n_kv, cb), np.uint8)
    want_n = np.zeros((ring, n_kv), np.uint16)
    batch = pkg.CommandBatch(ctx)
    pos = 0
    for chunk in (5, 9, 7, 1, 12):                            # wraps the ring twice
        rows = pkg.synth.kv_rows(chunk, n_kv, hd, g)
        oracle.tq_write_kv(rows.view(np.uint16), n_kv, hd, bits, signs, levels, pos, ring, want_c, want_n)
        K.encode_kv_turboquant_into(batch, pkg.Buffer.from_slice(ctx, rows), lv, sg, packed, norms, hd, n_kv, chunk, bits,
                                    pos, ring)
        pos += chunk
    batch.commit_and_wait()
    assert np.array_equal(packed.as_array(np.uint8), want_c.reshape(-1))
    assert np.array_equal(norms.as_array(np.uint16), want_n.reshape(-1))


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_dequantize_is_bit_exact_and_windowed(pkg, gpu, oracle, bits):
    """dequantize_kv == f16(TurboQuant::decode) for every slot; token_start leaves earlier rows
    untouched; ring source slots give the same output as the absolute cache
    (quant_cache.rs:905, 990)."""
    ctx, K = gpu
    hd, n_kv, T = 256, 2, 40
    g = pkg.synth.rng(5, bits)
    rows = pkg.synth.kv_rows(T, n_kv, hd, g)
    signs, levels = codec(oracle, hd, bits)
    codes, norms = cpu_cache(oracle, rows, n_kv, hd, bits, 0, 0, T)
    want = np.stack([oracle.tq_decode(codes[t, h], norms[t, h], hd, bits, signs, levels)
                     for t in range(T) for h in range(n_kv)]).astype(np.float16).reshape(-1)
    lv, sg = pkg.Buffer.from_slice(ctx, levels), pkg.Buffer.from_slice(ctx, signs)
    cbuf, nbuf = pkg.Buffer.from_slice(ctx, codes), pkg.Buffer.from_slice(ctx, norms)
    out = pkg.Buffer.empty(ctx, T * n_kv * hd * 2)
    K.dequantize_kv_turboquant(ctx, cbuf, nbuf, lv, sg, out, hd, n_kv, T, bits, 0, 0)
    got = out.as_array(np.float16)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # windowed: only tokens >= 25 are written
    out2 = pkg.Buffer.empty(ctx, T * n_kv * hd * 2)
    K.dequantize_kv_turboquant(ctx, cbuf, nbuf, lv, sg, out2, hd, n_kv, T, bits, 25, 0)
    got2 = out2.as_array(np.float16).reshape(T, -1)
    assert np.all(got2[:25] == 0) and np.array_equal(got2[25:].view(np.uint16), got.reshape(T, -1)[25:].view(np.uint16))
    # ring of 16 holding the last 16 tokens
    ring = 16
    rc, rn = cpu_cache(oracle, rows, n_kv, hd, bits, 0, ring, ring)
    out3 = pkg.Buffer.empty(ctx, T * n_kv * hd * 2)
    K.dequantize_kv_turboquant(ctx, pkg.Buffer.from_slice(ctx, rc), pkg.Buffer.from_slice(ctx, rn), lv, sg, out3, hd, n_kv, T,
                               bits, T - ring, ring)
    got3 = out3.as_array(np.float16).reshape(T, -1)
    assert np.array_equal(got3[T - ring:].view(np.uint16), got.reshape(T, -1)[T - ring:].view(np.uint16))


def test_encode_then_decode_roundtrips(pkg, gpu, oracle):
    """kernels.rs:10714: GPU encode then GPU dequantize stays within the 2-bit distortion."""
    ctx, K = gpu
    hd, n_kv, T, bits = 256, 1, 32, 2
    g = pkg.synth.rng(5, 123)
    rows = pkg.synth.kv_rows(T, n_kv, hd, g)
    cache = pkg.QuantizedKvCache(ctx, n_kv, hd, T, bits)
    batch = pkg.CommandBatch(ctx)
    src = pkg.Buffer.from_slice(ctx, rows)
    cache.write_kv_gpu_into(batch, K, src, src, 0, T)
    batch.commit_and_wait()
    ko, vo = pkg.Buffer.empty(ctx, rows.nbytes), pkg.Buffer.empty(ctx, rows.nbytes)
    cache.dequantize_into(ctx, K, ko, vo, T, 0)
    kd = ko.as_array(np.float16).astype(np.float32).reshape(T, hd)
    x = rows.astype(np.float32).reshape(T, hd)
    rel = np.sqrt(np.sum((kd - x) ** 2, axis=1) / np.sum(x ** 2, axis=1))
    assert np.all(rel < 0.45) and 0.28 < rel.mean() < 0.40          # sqrt(0.1175) ~ 0.34
    assert np.array_equal(ko.as_array(np.uint16), vo.as_array(np.uint16))
    with pytest.raises(pkg.InvalidArgument, match="exceeds capacity"):
        cache.write_kv_gpu_into(batch, K, src, src, 1, T)               # quant_cache.rs:400-406


@pytest.mark.parametrize("hd,heads", [(256, 8), (128, 3), (512, 2), (64, 5), (32, 1), (16, 2), (8, 3)])
def test_hadamard_rotate_variants_bit_exact(pkg, gpu, oracle, hd, heads):
    ctx, K = gpu
    g = pkg.synth.rng(5, hd + heads)
    x = g.standard_normal(heads * hd, dtype=np.float32)
    signs = oracle.rotation_signs(hd, oracle.TQ_SEED)
    sg = pkg.Buffer.from_slice(ctx, signs)
    batch = pkg.CommandBatch(ctx)
    for pre, post in ((True, False), (False, True), (True, True), (False, False)):
        want = oracle.hadamard_rotate(x, signs, hd, heads, pre, post)
        out = pkg.Buffer.empty(ctx, x.nbytes)
        K.hadamard_rotate_into(batch, pkg.Buffer.from_slice(ctx, x), sg, out, hd, heads, pre, post)
        batch.commit_and_wait()
        assert np.array_equal(out.as_array(np.float32).view(np.uint32), want.view(np.uint32))
        x16 = x.astype(np.float16)
        want_hf = oracle.hadamard_rotate(x16.astype(np.float32), signs, hd, heads, pre, post)
        out_hf = pkg.Buffer.empty(ctx, x.nbytes)
        K.hadamard_rotate_hf_into(batch, pkg.Buffer.from_slice(ctx, x16), sg, out_hf, hd, heads, pre, post)
        out_fh = pkg.Buffer.empty(ctx, heads * hd * 2)
        K.hadamard_rotate_fh_into(batch, pkg.Buffer.from_slice(ctx, x), sg, out_fh, hd, heads, pre, post)
        batch.commit_and_wait()
        assert np.array_equal(out_hf.as_array(np.float32).view(np.uint32), want_hf.view(np.uint32))
        assert np.array_equal(out_fh.as_array(np.uint16), want.astype(np.float16).view(np.uint16))


def test_batched_encode_matches_independent(pkg, gpu, oracle):
    """kernels.rs:10457: per-lane encode into the by-lane pool is byte-equal to single-sequence encodes."""
    ctx, K = gpu
    hd, n_kv, bits, lanes, cap = 128, 2, 2, 5, 24
    cb = oracle.tq_code_bytes(hd, bits)
    signs, levels = codec(oracle, hd, bits)
    lv, sg = pkg.Buffer.from_slice(ctx, levels), pkg.Buffer.from_slice(ctx, signs)
    g = pkg.synth.rng(5, 31)
    rows = pkg.synth.kv_rows(lanes, n_kv, hd, g)
    positions = np.array([0, 7, 23, 3, 11], np.uint32)
    packed = pkg.Buffer.empty(ctx, lanes * cap * n_kv * cb)
    norms = pkg.Buffer.empty(ctx, lanes * cap * n_kv * 2)
    batch = pkg.CommandBatch(ctx)
    K.encode_kv_turboquant_batched_into(batch, pkg.Buffer.from_slice(ctx, rows), lv, sg, packed, norms,
                                        pkg.Buffer.from_slice(ctx, positions), hd, n_kv, cap, bits, lanes, 0)
    batch.commit_and_wait()
    want_c = np.zeros((lanes * cap, n_kv, cb), np.uint8)
    want_n = np.zeros((lanes * cap, n_kv), np.uint16)
    for l in range(lanes):
        oracle.tq_write_kv(rows[l:l + 1].view(np.uint16), n_kv, hd, bits, signs, levels, l * cap + int(positions[l]), 0,
                           want_c, want_n)
    assert np.array_equal(packed.as_array(np.uint8), want_c.reshape(-1))
    assert np.array_equal(norms.as_array(np.uint16), want_n.reshape(-1))


def test_bad_shapes_are_rejected(pkg, gpu):
    ctx, K = gpu
    b = pkg.Buffer.empty(ctx, 1 << 16)
    batch = pkg.CommandBatch(ctx)
    with pytest.raises(pkg.InvalidArgument, match="bits must be 2..=4"):
        K.encode_kv_turboquant_into(batch, b, b, b, b, b, 256, 1, 1, 5, 0, 0)
    with pytest.raises(pkg.InvalidArgument, match="power of two"):
        K.encode_kv_turboquant_into(batch, b, b, b, b, b, 96, 1, 1, 2, 0, 0)
    with pytest.raises(pkg.InvalidArgument, match="power of two"):
        K.hadamard_rotate_into(batch, b, b, b, 1024, 1, True, False)
    with pytest.raises(pkg.InvalidArgument):
        pkg.QuantizedKvCache(ctx, 1, 256, 100000, 2, physical_positions=600, sliding_window=512)   # ring too small
    assert batch.dispatch_count() == 0


@pytest.mark.parametrize("hd,n_q,n_kv,bits,prf,with_norms,ring", [(256, 8, 1, 2, 1.0, True, 0), (512, 4, 2, 2, 0.25, True, 0),
                                                                 (128, 4, 4, 4, 1.0, False, 0), (64, 2, 1, 3, 0.5, True, 0),
                                                                 (256, 8, 1, 2, 1.0, True, 512)])
def test_decode_qkv_prepare_equals_the_separate_kernels(pkg, gpu, oracle, hd, n_q, n_kv, bits, prf, with_norms, ring):
    """One dispatch for qk_norm + rope on Q and K, unit-weight rms_norm on V, both KV encodes and the query rotation.
    Checked stage by stage: q / k / v left behind against the glue oracle (f16 ulps), the codes and norms against the
    CPU encoder applied to exactly those k / v rows (bit for bit), rq against the oracle's rotation of that q; and the
    whole against the eight separate dispatches (q, k, v within an f16 ulp -- the RMS sums run in another order)."""
    from oracle import layer_glue as G
    ctx, K = gpu
    g = pkg.synth.rng(61, hd + n_q + bits)
    position, eps, theta = 777, 1e-6, 1e4
    cap = ring if ring else 1024
    q0 = (g.standard_normal(n_q * hd, dtype=np.float32) * 2).astype(np.float16)
    k0 = (g.standard_normal(n_kv * hd, dtype=np.float32) * 2).astype(np.float16)
    v0 = (g.standard_normal(n_kv * hd, dtype=np.float32) * 2).astype(np.float16)
    qw = (0.25 * (1 + 0.1 * g.standard_normal(hd, dtype=np.float32))).astype(np.float16)
    kw = (0.25 * (1 + 0.1 * g.standard_normal(hd, dtype=np.float32))).astype(np.float16)
    levels, signs = oracle.tq_levels(hd, bits), oracle.rotation_signs(hd)
    cb = oracle.tq_code_bytes(hd, bits)
    lv, sg = pkg.Buffer.from_slice(ctx, levels), pkg.Buffer.from_slice(ctx, signs)
    qwb, kwb = (pkg.Buffer.from_slice(ctx, qw), pkg.Buffer.from_slice(ctx, kw)) if with_norms else (None, None)

    def fresh():
        return dict(q=pkg.Buffer.from_slice(ctx, q0), k=pkg.Buffer.from_slice(ctx, k0), v=pkg.Buffer.from_slice(ctx, v0),
                    rq=pkg.Buffer.empty(ctx, n_q * hd * 4), kc=pkg.Buffer.empty(ctx, cap * n_kv * cb),
                    kn=pkg.Buffer.empty(ctx, cap * n_kv * 2), vc=pkg.Buffer.empty(ctx, cap * n_kv * cb),
                    vn=pkg.Buffer.empty(ctx, cap * n_kv * 2))

    a, b = fresh(), fresh()
    batch = pkg.CommandBatch(ctx)
    K.decode_qkv_prepare_into(batch, a["q"], a["k"], a["v"], qwb, kwb, lv, sg, a["rq"], a["kc"], a["kn"], a["vc"], a["vn"],
                              hd, n_q, n_kv, eps, position, theta, prf, bits, ring)
    assert batch.dispatch_count() == 1
    ones = pkg.Buffer.from_slice(ctx, np.ones(hd, np.float16))
    if with_norms:
        K.qk_norm_gpu_into(batch, b["q"], qwb, hd, n_q, eps)
        K.qk_norm_gpu_into(batch, b["k"], kwb, hd, n_kv, eps)
    K.rope_into(batch, b["q"], b["q"], hd, position, theta, prf, n_q)
    K.rope_into(batch, b["k"], b["k"], hd, position, theta, prf, n_kv)
    K.rms_norm_into(batch, b["v"], ones, b["v"], hd, n_kv, eps)
    K.encode_kv_turboquant_into(batch, b["k"], lv, sg, b["kc"], b["kn"], hd, n_kv, 1, bits, position, ring)
    K.encode_kv_turboquant_into(batch, b["v"], lv, sg, b["vc"], b["vn"], hd, n_kv, 1, bits, position, ring)
    K.hadamard_rotate_hf_into(batch, b["q"], sg, b["rq"], hd, n_q, True, False)
    batch.commit_and_wait()

    got = {n: a[n].as_array(np.float16) for n in ("q", "k", "v")}
    want_q = G.rope(G.qk_norm(q0, qw, hd, n_q, eps) if with_norms else q0, hd, position, theta, prf, n_q)
    want_k = G.rope(G.qk_norm(k0, kw, hd, n_kv, eps) if with_norms else k0, hd, position, theta, prf, n_kv)
    want_v = G.rms_norm(v0, np.ones(hd, np.float16), hd, n_kv, eps)
    for name, want in (("q", want_q), ("k", want_k), ("v", want_v)):
        d = np.abs(got[name].astype(np.float32) - want.astype(np.float32))
        assert d.max() <= 4e-3 * max(1.0, np.abs(want.astype(np.float32)).max()), (name, d.max())
        sep = b[name].as_array(np.float16).astype(np.float32)
        assert np.abs(got[name].astype(np.float32) - sep).max() <= 2e-3 * max(1.0, np.abs(sep).max()), name
    # encode: bit exact for the rows this kernel left in k / v
    slot = position % ring if ring else position
    for rows, codes, norms in ((got["k"], a["kc"], a["kn"]), (got["v"], a["vc"], a["vn"])):
        packed, nrm = np.zeros(cap * n_kv * cb, np.uint8), np.zeros(cap * n_kv, np.uint16)
        oracle.tq_write_kv(rows.view(np.uint16), n_kv, hd, bits, signs, levels, position, ring, packed, nrm)
        assert packed[slot * n_kv * cb:(slot + 1) * n_kv * cb].any()
        assert np.array_equal(codes.as_array(np.uint8, cap * n_kv * cb), packed)
        assert np.array_equal(norms.as_array(np.uint16, cap * n_kv), nrm)
    want_rq = oracle.hadamard_rotate(got["q"].astype(np.float32), signs, hd, n_q, True, False)
    assert np.abs(a["rq"].as_array(np.float32) - want_rq).max() <= 1e-5 * max(1.0, np.abs(want_rq).max())
    # query only (a layer that reads another layer's cache): caches untouched
    c = fresh()
    batch = pkg.CommandBatch(ctx)
    K.decode_qkv_prepare_into(batch, c["q"], None, None, qwb, None, lv, sg, c["rq"], None, None, None, None, hd, n_q, n_kv, eps,
                              position, theta, prf, bits, ring)
    batch.commit_and_wait()
    assert np.array_equal(c["q"].as_array(np.uint16), a["q"].as_array(np.uint16))
    assert np.array_equal(c["rq"].as_array(np.uint32), a["rq"].as_array(np.uint32))
    assert not c["kc"].as_array(np.uint8).any()


@pytest.mark.parametrize("lanes_mode", [False, True])
def test_decode_qkv_prepare_rows_equals_row_by_row(pkg, gpu, oracle, lanes_mode):
    """Several tokens in one dispatch -- consecutive positions of one sequence on a ring that wraps inside the call, or
    one token per lane at positions from a device table -- give the bits of one single-token call per row (the
    single-token form is checked against the oracle and the separate kernels above)."""
    ctx, K = gpu
    hd, n_q, n_kv, bits, rows, eps, theta, prf = 256, 4, 2, 2, 7, 1e-6, 1e4, 1.0
    g = pkg.synth.rng(62, int(lanes_mode))
    cb = oracle.tq_code_bytes(hd, bits)
    ring = 512
    lane_cap = 600 if lanes_mode else 0
    start = 509                                            # rows 509..515 wrap the 512-slot ring
    positions = np.array([3, 700, 511, 512, 0, 1023, 77], np.uint32)
    q0 = (g.standard_normal(rows * n_q * hd, dtype=np.float32) * 2).astype(np.float16)
    k0 = (g.standard_normal(rows * n_kv * hd, dtype=np.float32) * 2).astype(np.float16)
    v0 = (g.standard_normal(rows * n_kv * hd, dtype=np.float32) * 2).astype(np.float16)
    qw = (0.25 * (1 + 0.1 * g.standard_normal(hd, dtype=np.float32))).astype(np.float16)
    kw = (0.25 * (1 + 0.1 * g.standard_normal(hd, dtype=np.float32))).astype(np.float16)
    lv = pkg.Buffer.from_slice(ctx, oracle.tq_levels(hd, bits))
    sg = pkg.Buffer.from_slice(ctx, oracle.rotation_signs(hd))
    qwb, kwb = pkg.Buffer.from_slice(ctx, qw), pkg.Buffer.from_slice(ctx, kw)
    phys = rows * lane_cap if lanes_mode else ring

    def fresh():
        return dict(q=pkg.Buffer.from_slice(ctx, q0), k=pkg.Buffer.from_slice(ctx, k0), v=pkg.Buffer.from_slice(ctx, v0),
                    rq=pkg.Buffer.empty(ctx, rows * n_q * hd * 4), kc=pkg.Buffer.empty(ctx, phys * n_kv * cb),
                    kn=pkg.Buffer.empty(ctx, phys * n_kv * 2), vc=pkg.Buffer.empty(ctx, phys * n_kv * cb),
                    vn=pkg.Buffer.empty(ctx, phys * n_kv * 2))

    a, b = fresh(), fresh()
    pos_buf = pkg.Buffer.from_slice(ctx, positions) if lanes_mode else None
    batch = pkg.CommandBatch(ctx)
    K.decode_qkv_prepare_rows_into(batch, a["q"], a["k"], a["v"], qwb, kwb, lv, sg, a["rq"], a["kc"], a["kn"], a["vc"], a["vn"],
                                   pos_buf, hd, n_q, n_kv, rows, eps, 0 if lanes_mode else start, theta, prf, bits, ring, lane_cap)
    assert batch.dispatch_count() == 1
    for r in range(rows):
        pos = int(positions[r]) if lanes_mode else start + r
        lane_bytes = lane_cap * n_kv
        view = {n: b[n].view(r * w, w) for n, w in (("q", n_q * hd * 2), ("k", n_kv * hd * 2), ("v", n_kv * hd * 2),
                                                     ("rq", n_q * hd * 4))}
        if lanes_mode:                                     # lane r's own region of the pool, addressed like a one-lane cache
            caches = {n: b[n].view(r * lane_bytes * u, lane_bytes * u) for n, u in (("kc", cb), ("kn", 2), ("vc", cb), ("vn", 2))}
        else:
            caches = {n: b[n] for n in ("kc", "kn", "vc", "vn")}
        K.decode_qkv_prepare_into(batch, view["q"], view["k"], view["v"], qwb, kwb, lv, sg, view["rq"], caches["kc"], caches["kn"],
                                  caches["vc"], caches["vn"], hd, n_q, n_kv, eps, pos, theta, prf, bits, ring)
    batch.commit_and_wait()
    for n in ("q", "k", "v", "rq", "kc", "kn", "vc", "vn"):
        assert np.array_equal(a[n].as_array(np.uint8), b[n].as_array(np.uint8)), n
    assert a["kc"].as_array(np.uint8).any()
    with pytest.raises(pkg.InvalidArgument):               # a positions table needs a lane capacity and the reverse
        K.decode_qkv_prepare_rows_into(pkg.CommandBatch(ctx), a["q"], a["k"], a["v"], qwb, kwb, lv, sg, a["rq"], a["kc"], a["kn"],
                                       a["vc"], a["vn"], None if lanes_mode else pkg.Buffer.from_slice(ctx, positions), hd, n_q,
                                       n_kv, rows, eps, 0, theta, prf, bits, ring, lane_cap if lanes_mode else 0)


@pytest.mark.parametrize("fmt,rows,hd,n_q,n_kv,k_dim,lanes_mode", [
    ("q4_0", 64, 256, 8, 1, 2048, True),       # the 64-lane decode layer: k split, the preparation sums the tiles
    ("q4_0", 5, 256, 8, 1, 2048, True),        # a few lanes: the small-batch kernel's tiles
    ("q4_0", 200, 256, 8, 1, 2048, False),     # a prefill chunk of one sequence, several groups of 64 rows
    ("tq2_0", 33, 128, 4, 2, 2048, True),      # TQ2_0 weights, two KV heads, head_dim 128
    ("q4_0", 12, 64, 6, 1, 512, True),         # K and V narrower than a 128-column tile: runs as the two calls
    ("q4_0", 1, 256, 8, 1, 2048, True),        # one row: the product runs as matvecs, then the preparation
])
def test_qkv_product_and_prepare_as_one_step_equals_the_two_calls(pkg, gpu, oracle, fmt, rows, hd, n_q, n_kv, k_dim, lanes_mode):
    """lh_matmul_nt_qkv_prepare_rows_into against lh_matmul_nt_quant_grouped_into followed by
    lh_decode_qkv_prepare_rows_into on the same inputs: q / k / v, the rotated queries, codes and norms bit for bit (the
    two calls are checked against the oracle and the separate kernels above and in test_gpu_matmul.py)."""
    print(f"case {fmt} rows={rows} hd={hd} n_q={n_q} n_kv={n_kv} k={k_dim} lanes={lanes_mode}", flush=True)
    ctx, K = gpu
    bits, eps, theta, prf = 2, 1e-6, 1e4, 1.0
    ty = pkg.Q4_0 if fmt == "q4_0" else pkg.TQ2_0
    g = pkg.synth.rng(63, rows * 7 + hd)
    cb = oracle.tq_code_bytes(hd, bits)
    lane_cap = 300 if lanes_mode else 0
    start = 0 if lanes_mode else 41
    positions = g.integers(0, lane_cap, rows).astype(np.uint32) if lanes_mode else None
    phys = rows * lane_cap if lanes_mode else start + rows
    ns = [n_q * hd, n_kv * hd, n_kv * hd]
    ws = [pkg.Buffer.from_slice(ctx, pkg.synth.weights(fmt, n, k_dim, g)) for n in ns]
    x = pkg.Buffer.from_slice(ctx, pkg.synth.activations(rows, k_dim, g).astype(np.float16))
    qw = (0.25 * (1 + 0.1 * g.standard_normal(hd, dtype=np.float32))).astype(np.float16)
    kw = (0.25 * (1 + 0.1 * g.standard_normal(hd, dtype=np.float32))).astype(np.float16)
    lv = pkg.Buffer.from_slice(ctx, oracle.tq_levels(hd, bits))
    sg = pkg.Buffer.from_slice(ctx, oracle.rotation_signs(hd))
    qwb, kwb = pkg.Buffer.from_slice(ctx, qw), pkg.Buffer.from_slice(ctx, kw)
    pos_buf = pkg.Buffer.from_slice(ctx, positions) if lanes_mode else None

    def fresh():
        d = dict(q=pkg.Buffer.empty(ctx, rows * ns[0] * 2), k=pkg.Buffer.empty(ctx, rows * ns[1] * 2),
                 v=pkg.Buffer.empty(ctx, rows * ns[2] * 2), rq=pkg.Buffer.empty(ctx, rows * ns[0] * 4),
                 kc=pkg.Buffer.empty(ctx, phys * n_kv * cb), kn=pkg.Buffer.empty(ctx, phys * n_kv * 2),
                 vc=pkg.Buffer.empty(ctx, phys * n_kv * cb), vn=pkg.Buffer.empty(ctx, phys * n_kv * 2))
        for buf in d.values():
            buf.copy_from_bytes(np.zeros(buf.length(), np.uint8))
        return d

    a, b = fresh(), fresh()
    batch = pkg.CommandBatch(ctx)
    K.matmul_nt_qkv_prepare_rows_into(batch, ty, x, ws[0], ws[1], ws[2], k_dim, a["q"], a["k"], a["v"], qwb, kwb, lv, sg, a["rq"],
                                      a["kc"], a["kn"], a["vc"], a["vn"], pos_buf, hd, n_q, n_kv, rows, eps, start, theta, prf,
                                      bits, 0, lane_cap)
    batch.commit_and_wait()
    K.matmul_nt_quant_grouped_into(batch, ty, x, ws, [b["q"], b["k"], b["v"]], rows, k_dim, ns)
    K.decode_qkv_prepare_rows_into(batch, b["q"], b["k"], b["v"], qwb, kwb, lv, sg, b["rq"], b["kc"], b["kn"], b["vc"], b["vn"],
                                   pos_buf, hd, n_q, n_kv, rows, eps, start, theta, prf, bits, 0, lane_cap)
    batch.commit_and_wait()
    for n in ("q", "k", "v", "rq", "kc", "kn", "vc", "vn"):
        assert np.array_equal(a[n].as_array(np.uint8), b[n].as_array(np.uint8)), n
    assert a["kc"].as_array(np.uint8).any() and a["rq"].as_array(np.float32).any()
    with pytest.raises(pkg.InvalidArgument):               # a too-small output is refused before anything is launched
        K.matmul_nt_qkv_prepare_rows_into(pkg.CommandBatch(ctx), ty, x, ws[0], ws[1], ws[2], k_dim, a["q"], a["k"], a["v"], qwb, kwb,
                                          lv, sg, pkg.Buffer.empty(ctx, 64), a["kc"], a["kn"], a["vc"], a["vn"], pos_buf, hd, n_q,
                                          n_kv, rows, eps, start, theta, prf, bits, 0, lane_cap)
