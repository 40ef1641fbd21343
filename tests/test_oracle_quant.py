"""Pins the CPU oracle's f16 conversion, Q4_0 / TQ2_0 dequant and dot products
against the reference's known-answer vectors and independent evaluations
(numpy.float16 is an independent IEEE binary16 implementation)."""
import numpy as np
import pytest

import refgen


def test_f16_to_f32_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rne_subnormals_and_ties(oracle):
    rng = np.random.default_rng(1)
    # random floats over the whole f16 range incl. subnormals and overflow
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 200000).astype(np.float32),
        # exact halfway points between neighbouring f16 values (ties-to-even)
        ((np.arange(65535, dtype=np.uint16)[:31743].view(np.float16).astype(np.float64)
          + np.arange(1, 31744, dtype=np.uint16).view(np.float16).astype(np.float64)) / 2).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -26, np.inf, -np.inf], np.float32),
    ])
    got = oracle.f32_to_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_q4_0_known_answers(oracle):
    # local-engine/src/pipeline/init_gemma4_qat.rs:241-265 and qat_recover.rs:243-249
    blk = np.zeros(18, np.uint8)
    blk[0:2] = np.array([0.5], np.float16).view(np.uint8)
    nib = np.full(32, 8, np.uint8)
    nib[0], nib[1] = 15, 0
    blk[2:] = (nib[:16] & 0xF) | (nib[16:] << 4)
    out = oracle.dequant_q4_0(blk).view(np.float16).astype(np.float32)
    assert out[0] == 3.5 and out[1] == -4.0 and np.all(out[2:] == 0.0)
    allzero = blk.copy(); allzero[2:] = 0x88
    assert np.all(oracle.dequant_q4_0(allzero).view(np.float16) == 0)
    # truncation to num_elements
    assert oracle.dequant_q4_0(np.tile(blk, 3), 40).size == 40


def test_tq2_0_known_answers(oracle):
    # local-engine/src/qat_recover.rs:199-240
    blk = np.zeros(66, np.uint8)
    blk[0] = 0b00011011
    blk[64:66] = np.array([2.0], np.float16).view(np.uint8)
    out = oracle.dequant_tq2_0(blk).view(np.float16).astype(np.float32)
    assert out[0] == 4.0 and out[32] == 2.0 and out[64] == 0.0 and out[96] == -2.0 and out[1] == -2.0
    assert out.size == 256
    assert oracle.dequant_tq2_0(blk, 100).size == 100


def test_q4_0_brute_force_all_scales(oracle):
    """Every f16 scale x every nibble against an independent numpy evaluation."""
    d_bits = np.arange(65536, dtype=np.uint16)
    d_bits = d_bits[~np.isnan(d_bits.view(np.float16))]
    blocks = np.zeros((d_bits.size, 18), np.uint8)
    blocks[:, 0:2] = d_bits.view(np.uint8).reshape(-1, 2)
    lo = np.arange(16, dtype=np.uint8)           # low nibbles 0..15 -> elements 0..15
    hi = (15 - np.arange(16)).astype(np.uint8)   # high nibbles 15..0 -> elements 16..31
    blocks[:, 2:] = lo | (hi << 4)
    got = oracle.dequant_q4_0(blocks.reshape(-1)).reshape(-1, 32)
    q = np.concatenate([lo, hi]).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        want = ((q[None, :] - np.float32(8.0)) * d_bits.view(np.float16).astype(np.float32)[:, None]).astype(np.float16)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want.view(np.uint16)[ok])


def test_tq2_0_brute_force_all_scales(oracle):
    d_bits = np.arange(65536, dtype=np.uint16)
    d_bits = np.ascontiguousarray(d_bits[~np.isnan(d_bits.view(np.float16))][::7])
    rng = np.random.default_rng(3)
    blocks = np.zeros((d_bits.size, 66), np.uint8)
    blocks[:, :64] = rng.integers(0, 256, (d_bits.size, 64), dtype=np.uint8)
    blocks[:, 64:] = d_bits.view(np.uint8).reshape(-1, 2)
    got = oracle.dequant_tq2_0(blocks.reshape(-1)).reshape(-1, 256)
    qs = blocks[:, :64]
    want = np.empty((d_bits.size, 256), np.float16)
    d = d_bits.view(np.float16).astype(np.float32)
    with np.errstate(over="ignore", invalid="ignore"):
        for j in range(64):
            for l in range(4):
                e = (j >> 5) * 128 + l * 32 + (j & 31)   # shaders/matvec_quant.metal:15-17
                want[:, e] = (d * (((qs[:, j] >> (2 * l)) & 3).astype(np.float32) - np.float32(1.0))).astype(np.float16)
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want.view(np.uint16)[ok])


@pytest.mark.parametrize("fmt,rows,cols", [("q4_0", 5, 96), ("q4_0", 7, 64), ("tq2_0", 4, 512), ("tq2_0", 6, 256)])
def test_expand_matches_dequant_and_matvec_invariants(oracle, fmt, rows, cols):
    raw = refgen.q4_0_payload(rows, cols, 77) if fmt == "q4_0" else refgen.tq2_0_payload(rows, cols, 77)
    expand = oracle.expand_q4_0_f32 if fmt == "q4_0" else oracle.expand_tq2_0_f32
    deq = oracle.dequant_q4_0 if fmt == "q4_0" else oracle.dequant_tq2_0
    dq = expand(raw, rows, cols)
    h = deq(raw).view(np.float16).astype(np.float32).reshape(rows, cols)
    # the f16-rounded dequant is the RNE of the unrounded expansion
    assert np.array_equal(dq.astype(np.float16).astype(np.float32), h)
    _, v = refgen.test_vector(cols)
    y = oracle.matvec_f32(dq, v)
    y64 = oracle.matvec_f64(dq, v)
    assert np.allclose(y, y64, rtol=0, atol=1e-4)
    assert np.allclose(y64, dq.astype(np.float64) @ v.astype(np.float64), rtol=1e-12, atol=1e-12)
    # sequential left fold, reproduced with an explicit python loop on row 0
    s = np.float32(0.0)
    for c in range(cols):
        s = np.float32(s + np.float32(dq[0, c] * v[c]))
    assert s == y[0]
    # row-permutation equivariance and M-row batch == M independent matvecs
    perm = np.random.default_rng(0).permutation(rows)
    assert np.array_equal(oracle.matvec_f32(dq[perm], v), y[perm])
    a = np.stack([v, v[::-1].copy()])
    c = oracle.matmul_nt_f32(a, dq)
    assert np.array_equal(c[0], y) and np.array_equal(c[1], oracle.matvec_f32(dq, v[::-1].copy()))
    # the full reference CPU path (dequant->f16->dot) on the same payload
    yr = oracle.matvec_quant_ref(fmt, raw, v, rows, cols)
    assert np.array_equal(yr, oracle.matvec_f32(h, v))
    assert np.array_equal(oracle.matvec_quant_ref(fmt, raw, v, rows, cols, threads=3), yr)


def test_tensor_byte_sizes(oracle):
    # local-engine/src/gguf.rs:272-311; asserted values from gguf.rs:524-528
    assert oracle.tensor_bytes("q4_0", 1024) == 32 * 18
    assert oracle.tensor_bytes("q8_0", 1024) == 32 * 34
    assert oracle.tensor_bytes("tq2_0", 257) == 2 * 66


def test_legacy_tq2_dequant_and_f16_matmul(oracle):
    rng = np.random.default_rng(5)
    packed = rng.integers(0, 256, 16, dtype=np.uint8)
    scales = rng.standard_normal(16).astype(np.float16)
    got = oracle.tq2_dequant_legacy(packed, scales.view(np.uint16), 64).view(np.float16)
    for i in range(64):
        want = np.float16(np.float32(scales[i // 4]) * np.float32((packed[i // 4] >> (2 * (i % 4))) & 3))
        assert got[i] == want
    a = rng.standard_normal((3, 40)).astype(np.float16)
    b = rng.standard_normal((5, 40)).astype(np.float16)
    c = oracle.matmul_f16_nt(a.view(np.uint16), b.view(np.uint16), 3, 40, 5)
    assert np.allclose(c, a.astype(np.float64) @ b.astype(np.float64).T, rtol=1e-6, atol=1e-6)
