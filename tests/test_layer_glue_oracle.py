"""Pins the numpy restatements of the layer glue kernels (oracle/layer_glue.py) to the reference's own
known-answer tests and to closed forms.  CPU only."""
import math

import numpy as np

from oracle import layer_glue as lg


def test_rms_norm_known_vector():
    """kernels.rs:7050-7073: [1,2,3,4] with unit weights -> x / sqrt(7.5), tolerance 0.02."""
    out = lg.rms_norm(np.array([1, 2, 3, 4], np.float16), np.ones(4, np.float16), 4, 1, 1e-6).astype(np.float32)
    assert np.abs(out - np.arange(1, 5) / math.sqrt(7.5)).max() < 2e-3
    # closed form: with unit weights the output row has mean square 1
    x = np.random.default_rng(1).standard_normal((3, 64)).astype(np.float16)
    y = lg.rms_norm(x, np.ones(64, np.float16), 64, 3, 0.0).astype(np.float64).reshape(3, 64)
    assert np.abs((y ** 2).mean(axis=1) - 1).max() < 2e-3
    # the fused form adds the residual after the product
    r = np.random.default_rng(2).standard_normal((3, 64)).astype(np.float16)
    w = np.linspace(0.5, 1.5, 64).astype(np.float16)
    plain = lg.rms_norm(x, w, 64, 3, 1e-6).astype(np.float32) + r.reshape(-1).astype(np.float32)
    fused = lg.rms_norm(x, w, 64, 3, 1e-6, residual=r).astype(np.float32)
    assert np.abs(plain - fused).max() <= 2e-3 * max(1.0, np.abs(plain).max())


def test_rope_identity_and_partial_rotary():
    """kernels.rs:7214-7288."""
    x = np.array([1, 2, 3, 4], np.float16)
    assert np.array_equal(lg.rope(x, 4, 0, 10000.0, 1.0, 1), x)
    assert np.abs(lg.rope(x, 4, 100, 10000.0, 1.0, 1).astype(np.float32) - x.astype(np.float32)).max() > 0.01
    vals = np.arange(1, 9).astype(np.float16)
    out = lg.rope(vals, 8, 100, 10000.0, 0.25, 1).astype(np.float32)
    s, c = math.sin(100.0), math.cos(100.0)
    assert abs(out[0] - (1 * c - 5 * s)) < 0.02 and abs(out[4] - (1 * s + 5 * c)) < 0.02
    for i in (1, 2, 3, 5, 6, 7):
        assert out[i] == float(vals[i])
    # a rotation keeps the norm of every pair
    x = np.random.default_rng(3).standard_normal(2 * 64).astype(np.float16)
    y = lg.rope(x, 64, 977, 1e6, 1.0, 2).astype(np.float64).reshape(2, 64)
    xx = x.astype(np.float64).reshape(2, 64)
    assert np.abs((y[:, :32] ** 2 + y[:, 32:] ** 2) - (xx[:, :32] ** 2 + xx[:, 32:] ** 2)).max() < 2e-2


def test_qk_norm_matches_sequential_f32_formula_and_fusion():
    """kernels.rs:7818-7870 (CPU formula, tolerance 0.01) and 7873-7925 (fused == separate, bit for bit)."""
    nh, hd, eps = 4, 64, 1e-6
    qk = np.sin(np.arange(nh * hd, dtype=np.float32) * np.float32(0.037)).astype(np.float16)
    w = (1.0 + np.arange(hd, dtype=np.float32) * np.float32(0.01)).astype(np.float16)
    want = qk.astype(np.float32).copy()
    for h in range(nh):
        ss = np.float32(0)
        for j in range(hd):
            ss += want[h * hd + j] * want[h * hd + j]
        rms = np.float32(1) / np.sqrt(ss / np.float32(hd) + np.float32(eps))
        want[h * hd:(h + 1) * hd] = want[h * hd:(h + 1) * hd] * rms * w.astype(np.float32)
    assert np.abs(lg.qk_norm(qk, w, hd, nh, eps).astype(np.float32) - want).max() < 2e-3
    for prf in (1.0, 0.5):
        fused = lg.qk_norm_rope(qk, w, hd, nh, eps, 137, 1e6, prf)
        sep = lg.rope(lg.qk_norm(qk, w, hd, nh, eps), hd, 137, 1e6, prf, nh)
        assert np.array_equal(fused.view(np.uint16), sep.view(np.uint16))


def test_gelu_mul_known_values():
    """kernels.rs:7076-7117 (gelu_tanh values; the multiply by b = 1 leaves them)."""
    vals = np.array([0.0, 1.0, -1.0, 2.0, 10.0, -10.0, 65000.0], np.float16)
    out = lg.gelu_mul(vals, np.ones_like(vals)).astype(np.float32)
    for got, want in zip(out[:4], (0.0, 0.8412, -0.1588, 1.9545)):
        assert abs(got - want) < 2e-3
    assert np.isfinite(out).all() and abs(out[4] - 10.0) < 0.1 and abs(out[5]) < 0.01
    b = np.array([2.0, -0.5], np.float16)
    assert np.allclose(lg.gelu_mul(np.array([1.0, 2.0], np.float16), b).astype(np.float32), [0.8412 * 2, 1.9545 * -0.5], atol=3e-3)


def test_elementwise_closed_forms():
    a = np.array([1.0, 65504.0, 1e-4, -3.5], np.float16)
    b = np.array([2.0, 6e-8, 1e-4, 3.5], np.float16)
    assert np.array_equal(lg.residual_add(a, b), np.array([3.0, 65504.0, 2e-4, 0.0], np.float16))
    assert np.array_equal(lg.scale_in_place(np.array([1.0, -2.0, 0.5], np.float16), 0.5), np.array([0.5, -1.0, 0.25], np.float16))
    # kernels.rs:7751-7787: layer 3 of a packed [5, 7, 4] iota
    src = np.arange(5 * 7 * 4, dtype=np.float32).astype(np.float16)
    got = lg.gather_strided_f16(src, 7 * 4, 3 * 4, 4, 5)
    assert np.array_equal(got, src.reshape(5, 7, 4)[:, 3, :].reshape(-1))
    # kernels.rs:7790-7815
    data = (np.arange(4096, dtype=np.float32) - 2048.0) * np.float32(0.05)
    out = lg.logit_softcap(data, 30.0)
    for i in (0, 1000, 2048, 2049, 4095):
        assert abs(out[i] - 30.0 * math.tanh(float(data[i]) / 30.0)) < 1e-4


def test_matvec_f16_known_products():
    """kernels.rs:7294-7360: identity x [5,7,9]; [[1,2],[3,4]] x [5,6] = [17,39]; [[1..4],[5..8]] x ones = [10,26]."""
    h = np.float16
    assert np.array_equal(lg.matvec_f16(np.eye(3, dtype=h), np.array([5, 7, 9], h), 3, 3), np.array([5, 7, 9], h))
    assert np.array_equal(lg.matvec_f16(np.array([1, 2, 3, 4], h), np.array([5, 6], h), 2, 2), np.array([17, 39], h))
    assert np.array_equal(lg.matvec_f16(np.arange(1, 9).astype(h), np.ones(4, h), 2, 4, out_f32=True), np.array([10, 26], np.float32))
    # linear in x, and rows are independent
    g = np.random.default_rng(5)
    w = g.standard_normal((6, 40)).astype(h)
    x1, x2 = g.standard_normal(40).astype(np.float32), g.standard_normal(40).astype(np.float32)
    y = lg.matvec_f16(w, x1 + x2, 6, 40, out_f32=True)
    assert np.allclose(y, lg.matvec_f16(w, x1, 6, 40, out_f32=True) + lg.matvec_f16(w, x2, 6, 40, out_f32=True), atol=1e-4)
    assert np.array_equal(lg.matvec_f16(w[2:3], x1, 1, 40, out_f32=True), lg.matvec_f16(w, x1, 6, 40, out_f32=True)[2:3])
