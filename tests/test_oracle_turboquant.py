"""Pins the CPU oracle's TurboQuant codec (local-engine/src/turboquant.rs) with
the reference's own unit-test facts, closed forms, and brute force."""
import numpy as np
import pytest
import scipy.linalg

import refgen


def py_splitmix_signs(dim, seed):
    """Independent restatement of turboquant.rs:66-79 in pure Python ints."""
    M = (1 << 64) - 1
    state = (seed | 1) & M
    out = []
    for _ in range(dim):
        state = (state + 0x9E3779B97F4A7C15) & M
        z = state
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & M
        z ^= z >> 31
        out.append(1.0 if (z & 1) == 0 else -1.0)
    return np.array(out, np.float32)


def test_fwht_matches_hadamard_matrix_and_is_involution(oracle):
    # turboquant.rs:358-369
    v = np.array([1.0, -2.0, 3.0, 0.5, -1.0, 2.0, -0.5, 4.0], np.float32)
    h = oracle.fwht_normalized(v)
    assert abs(np.linalg.norm(h) - np.linalg.norm(v)) < 1e-4
    assert np.allclose(oracle.fwht_normalized(h), v, atol=1e-4)
    for n in (8, 256, 512):
        x = np.random.default_rng(n).standard_normal(n).astype(np.float32)
        want = scipy.linalg.hadamard(n).astype(np.float64) @ x.astype(np.float64) / np.sqrt(n)
        assert np.allclose(oracle.fwht_normalized(x), want, atol=1e-4)


def test_rotation_signs(oracle):
    s = oracle.rotation_signs(256, oracle.TQ_SEED)
    assert np.array_equal(s, py_splitmix_signs(256, oracle.TQ_SEED))
    first64 = "".join("+" if v > 0 else "-" for v in s[:64])
    assert first64 == "--++-+-++--+-++-+-+--++-+-++-+++++--++--+++-+--+--++--+-+-+++--+"
    assert int((s > 0).sum()) == 129
    for dim, seed in ((128, 3), (512, 42), (256, 0)):
        assert np.array_equal(oracle.rotation_signs(dim, seed), py_splitmix_signs(dim, seed))


def test_rotation_inverse_recovers_input(oracle):
    # turboquant.rs:371-381
    signs = oracle.rotation_signs(256, 42)
    x = refgen.seeded_vec(256, 7)
    y = oracle.hadamard_rotate(x, signs, 256, 1, True, False)
    z = oracle.hadamard_rotate(y, signs, 256, 1, False, True)
    assert np.max(np.abs(z - x)) < 1e-3
    # hadamard_rotate(pre) == Rotation::apply == fwht(sign * x)
    assert np.array_equal(y, oracle.fwht_normalized(x * signs))


def _lloyd_max_f64(bits, iters=100):
    """Independent float64 / vectorised restatement of the same discretised
    Lloyd iteration (8192 midpoints on [-6, 6], same start, same 100 rounds)."""
    n = 8192
    xs = (np.arange(n) + 0.5) * (12.0 / n) - 6.0
    w = np.exp(-0.5 * xs * xs) / np.sqrt(2 * np.pi)
    k = 1 << bits
    lv = 6.0 * ((np.arange(k) + 0.5) / k - 0.5)
    for _ in range(iters):
        best = np.argmin(np.abs(xs[:, None] - lv[None, :]), axis=1)
        for j in range(k):
            m = best == j
            if w[m].sum() > 1e-12:
                lv[j] = (w[m] * xs[m]).sum() / w[m].sum()
    return np.sort(lv)


def test_lloyd_max_levels(oracle):
    # turboquant.rs:383-400, the published Lloyd-Max quantizers for N(0,1)
    # (the 100-round discretised iteration lands within ~5e-3 of them), and an
    # independent float64 evaluation of the same iteration.
    tables = {
        2: [0.4528, 1.5104],
        3: [0.2451, 0.7560, 1.3439, 2.1520],
        4: [0.1284, 0.3881, 0.6568, 0.9424, 1.2562, 1.6180, 2.0690, 2.7326],
    }
    for bits, pos in tables.items():
        l = oracle.lloyd_max_gaussian(bits).astype(np.float64)
        assert l.size == 1 << bits
        assert np.all(np.diff(l) > 0)
        assert np.max(np.abs(l + l[::-1])) < 0.05
        want = np.array([-p for p in pos[::-1]] + pos)
        assert np.max(np.abs(l - want)) < (6e-3 if bits < 4 else 2e-2), (bits, l, want)
        assert np.max(np.abs(l - _lloyd_max_f64(bits))) < (1e-5 if bits < 4 else 2e-3)
    lv = oracle.tq_levels(256, 2)
    assert np.array_equal(lv, oracle.lloyd_max_gaussian(2) * np.float32(1.0 / np.sqrt(np.float32(256.0))))


def test_code_bytes(oracle):
    # turboquant.rs:467-472
    assert [oracle.tq_code_bytes(256, b) for b in (4, 3, 2)] == [128, 96, 64]


def brute_encode(x, bits, signs, levels):
    x = x.astype(np.float32)
    sq = np.float32(0.0)
    for v in x:
        sq = np.float32(sq + np.float32(v * v))
    norm = np.sqrt(sq, dtype=np.float32)
    r = x.copy()
    if norm > 0:
        r = r * np.float32(np.float32(1.0) / norm)
    r = r * signs
    n = r.size
    ln = 1
    while ln < n:  # butterflies in float32
        r = r.reshape(-1, 2, ln)
        a, b = r[:, 0, :].copy(), r[:, 1, :].copy()
        r[:, 0, :], r[:, 1, :] = a + b, a - b
        r = r.reshape(-1)
        ln *= 2
    r = r * np.float32(np.float32(1.0) / np.sqrt(np.float32(n)))
    dist = np.abs(r[:, None] - levels[None, :])
    codes = np.argmin(dist, axis=1)  # first minimum == lowest index on ties
    bitstream = 0
    for i, c in enumerate(codes):
        bitstream |= int(c) << (i * bits)
    nbytes = (n * bits + 7) // 8
    return np.frombuffer(bitstream.to_bytes(nbytes, "little"), np.uint8), norm, r


@pytest.mark.parametrize("bits", [2, 3, 4])
@pytest.mark.parametrize("dim", [128, 256, 512])
def test_encode_matches_brute_force(oracle, bits, dim):
    signs = oracle.rotation_signs(dim, 7)
    levels = oracle.tq_levels(dim, bits)
    for seed in (1, 42, 1000):
        x = refgen.seeded_vec(dim, seed)
        codes, norm, rot = oracle.tq_encode(x, bits, signs, levels)
        bc, bn, br = brute_encode(x, bits, signs, levels)
        assert np.array_equal(rot, br)
        assert np.array_equal(codes, bc)
        assert norm == np.float16(bn).view(np.uint16)


def test_encode_zero_vector_and_ties(oracle):
    # turboquant.rs:439-450: zero vector -> norm 0, every coordinate 0.0
    dim = 128
    signs = oracle.rotation_signs(dim, 3)
    levels = oracle.tq_levels(dim, 4)
    codes, norm, rot = oracle.tq_encode(np.zeros(dim, np.float32), 4, signs, levels)
    assert norm == 0 and np.all(rot == 0)
    # exact tie between two levels -> lowest index (strict '<', turboquant.rs:293-304)
    lv = np.array([-1.0, 0.0, 1.0, 2.0], np.float32)
    x = np.zeros(4, np.float32)
    # craft rotated == [0.5, ...]: use identity-like case dim=1 is not a power-of-two FWHT; use brute search
    c, _, r = oracle.tq_encode(np.array([1.0, 0, 0, 0], np.float32), 2, np.ones(4, np.float32), lv)
    assert np.all(r == 0.5)           # H4 e0 / 2 = 0.5 everywhere
    assert c[0] == 0b01010101         # tie between levels 1 (0.0) and 2 (1.0) -> index 1


def test_decode_roundtrip_bounds(oracle):
    # turboquant.rs:402-415 (4-bit rel err < 0.10) and 452-465 (inner product within 15 %)
    dim = 256
    signs, levels = oracle.rotation_signs(dim, 123), oracle.tq_levels(dim, 4)
    x = refgen.seeded_vec(dim, 99)
    codes, norm, _ = oracle.tq_encode(x, 4, signs, levels)
    assert codes.size == 128
    xh = oracle.tq_decode(codes, norm, dim, 4, signs, levels)
    rel = np.sqrt(np.sum((x - xh) ** 2) / np.sum(x ** 2))
    assert rel < 0.10
    signs, levels = oracle.rotation_signs(dim, 5), oracle.tq_levels(dim, 4)
    k, qy = refgen.seeded_vec(dim, 1), refgen.seeded_vec(dim, 2)
    c, n, _ = oracle.tq_encode(k, 4, signs, levels)
    kh = oracle.tq_decode(c, n, dim, 4, signs, levels)
    exact, approx = float(qy @ k), float(qy @ kh)
    assert abs(exact - approx) / max(abs(exact), 1e-3) < 0.15
    # 2-bit distortion of a Gaussian vector is close to the Lloyd-Max MSE (0.1175)
    signs, levels = oracle.rotation_signs(dim, oracle.TQ_SEED), oracle.tq_levels(dim, 2)
    g = np.random.default_rng(0).standard_normal((64, dim)).astype(np.float32)
    mse = []
    for row in g:
        c, n, _ = oracle.tq_encode(row, 2, signs, levels)
        d = oracle.tq_decode(c, n, dim, 2, signs, levels)
        mse.append(np.sum((row - d) ** 2) / np.sum(row ** 2))
    assert 0.09 < np.mean(mse) < 0.15


def test_ring_capacity(oracle):
    # quant_cache.rs:964-974
    assert oracle.swa_ring_capacity(512, 131072) == 1024
    assert oracle.swa_ring_capacity(512, 600) == 600


def _make_cache(oracle, T, n_kv, hd, bits, seed, ring=0, start=0):
    rng = np.random.default_rng(seed)
    signs, levels = oracle.rotation_signs(hd, oracle.TQ_SEED), oracle.tq_levels(hd, bits)
    cb = oracle.tq_code_bytes(hd, bits)
    phys = ring if ring else start + T
    kc = np.zeros((phys, n_kv, cb), np.uint8); vc = np.zeros_like(kc)
    kn = np.zeros((phys, n_kv), np.uint16); vn = np.zeros_like(kn)
    k = rng.standard_normal((T, n_kv, hd)).astype(np.float16)
    v = rng.standard_normal((T, n_kv, hd)).astype(np.float16)
    oracle.tq_write_kv(k.view(np.uint16), n_kv, hd, bits, signs, levels, start, ring, kc, kn)
    oracle.tq_write_kv(v.view(np.uint16), n_kv, hd, bits, signs, levels, start, ring, vc, vn)
    return signs, levels, kc, kn, vc, vn, k, v


@pytest.mark.parametrize("bits", [2, 3, 4])
def test_codespace_attention_equals_decode_then_attend(oracle, bits):
    """Two formulations (rotated code space in f64 vs. per-vector decode + f32
    attention in the original space) must agree: <q,k> = <Rq, Rk>."""
    hd, nq, nkv, T = 128, 4, 2, 40
    signs, levels, kc, kn, vc, vn, _, _ = _make_cache(oracle, T, nkv, hd, bits, 11)
    q = (np.random.default_rng(2).standard_normal((nq, hd)) * 0.3).astype(np.float16).astype(np.float32)
    for window in (0, 8):
        rq = oracle.hadamard_rotate(q, signs, hd, nq, True, False)
        acc = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, window, bits, 0)
        out = oracle.hadamard_rotate(acc, signs, hd, nq, False, True)
        ref = oracle.attention_tq_decode_then_attend(q, kc, kn, vc, vn, levels, signs, hd, T, T - 1, nq, nkv,
                                                     window, bits, 0)
        assert np.max(np.abs(out - ref)) <= 2e-4 * max(np.max(np.abs(ref)), 1e-3)
        ref3 = oracle.attention_tq_decode_then_attend(q, kc, kn, vc, vn, levels, signs, hd, T, T - 1, nq, nkv,
                                                      window, bits, 0, threads=3)
        assert np.array_equal(ref, ref3)


def test_attention_ring_equals_absolute_and_empty_range(oracle):
    """quant_cache.rs:1047-1107: a wrapped ring gives the same attention as the
    absolute cache holding the same rows; kv_len = 0 -> zeros."""
    hd, nq, nkv, bits = 64, 2, 1, 2
    T, window, ring = 50, 8, 16
    signs, levels, kc, kn, vc, vn, k, v = _make_cache(oracle, T, nkv, hd, bits, 5)
    cb = oracle.tq_code_bytes(hd, bits)
    rkc = np.zeros((ring, nkv, cb), np.uint8); rvc = np.zeros_like(rkc)
    rkn = np.zeros((ring, nkv), np.uint16); rvn = np.zeros_like(rkn)
    oracle.tq_write_kv(k.view(np.uint16), nkv, hd, bits, signs, levels, 0, ring, rkc, rkn)
    oracle.tq_write_kv(v.view(np.uint16), nkv, hd, bits, signs, levels, 0, ring, rvc, rvn)
    rq = np.random.default_rng(9).standard_normal(nq * hd).astype(np.float32)
    a = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, window, bits, 0)
    b = oracle.attention_tq_codespace(rq, rkc, rkn, rvc, rvn, levels, hd, T, T - 1, nq, nkv, window, bits, ring)
    assert np.array_equal(a, b)
    z = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, 0, 0, nq, nkv, 0, bits, 0)
    assert np.all(z == 0)


def test_attention_single_position_returns_value(oracle):
    """With one cached position softmax is 1, so the output is exactly
    norm_v * levels[Vcode] -- catches a swapped K/V operand or a dropped norm."""
    hd, bits = 64, 2
    signs, levels, kc, kn, vc, vn, _, _ = _make_cache(oracle, 1, 1, hd, bits, 3)
    rq = np.ones(hd, np.float32)
    out = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, 1, 0, 1, 1, 0, bits, 0)
    codes = np.array([(vc[0, 0, i // 4] >> (2 * (i % 4))) & 3 for i in range(hd)])
    want = levels[codes].astype(np.float64) * float(vn.view(np.float16)[0, 0])
    assert np.allclose(out, want, rtol=1e-6, atol=0)


def test_attention_f16_reference(oracle):
    rng = np.random.default_rng(4)
    hd, nq, nkv, T = 32, 4, 2, 20
    q = rng.standard_normal((nq, hd)).astype(np.float16)
    k = (rng.standard_normal((T, nkv, hd)) * 0.3).astype(np.float16)
    v = (rng.standard_normal((T, nkv, hd)) * 0.4).astype(np.float16)
    out = oracle.attention_f16(q.view(np.uint16), k.view(np.uint16), v.view(np.uint16), hd, T, T - 1, nq, nkv, 8)
    for h in range(nq):
        g = h // (nq // nkv)
        s = k[12:, g].astype(np.float64) @ q[h].astype(np.float64)
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(out[h * hd:(h + 1) * hd], p @ v[12:, g].astype(np.float64), atol=1e-6)
