"""The oracle and the product's host-side codec against the known-answer vectors the
reference's own tests hold (tests/golden/known_answers.json: data only)."""
import json
import os

import numpy as np

GOLD = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")))


def test_q4_0_block(oracle):
    g = GOLD["q4_0_block"]
    nib = np.full(32, g["nibbles_default"], np.uint8)
    for k, v in g["nibbles"].items():
        nib[int(k)] = v
    blk = np.zeros(18, np.uint8)
    blk[0:2] = np.array([g["d"]], np.float16).view(np.uint8)
    blk[2:] = (nib[:16] & 0xF) | (nib[16:] << 4)
    out = oracle.dequant_q4_0(blk).view(np.float16).astype(np.float32)
    want = np.full(32, g["expect_rest"], np.float32)
    for k, v in g["expect"].items():
        want[int(k)] = v
    assert np.array_equal(out, want)


def test_tq2_0_block(oracle):
    g = GOLD["tq2_0_block"]
    blk = np.zeros(66, np.uint8)
    for k, v in g["qs"].items():
        blk[int(k)] = v
    blk[64:66] = np.array([g["d"]], np.float16).view(np.uint8)
    out = oracle.dequant_tq2_0(blk).view(np.float16).astype(np.float32)
    for k, v in g["expect"].items():
        assert out[int(k)] == v
    assert oracle.dequant_tq2_0(blk, g["num_elements_truncate"]).size == g["num_elements_truncate"]


def test_sizes_and_capacities(oracle, pkg):
    for fmt, n, want in GOLD["tensor_bytes"]["cases"]:
        assert oracle.tensor_bytes(fmt, n) == want
    for dim, bits, want in GOLD["turboquant_code_bytes"]["cases"]:
        assert oracle.tq_code_bytes(dim, bits) == want
        assert pkg.kv_cache.code_bytes(dim, bits) == want
    for window, maxpos, want in GOLD["swa_ring_capacity"]["cases"]:
        assert oracle.swa_ring_capacity(window, maxpos) == want
        assert pkg.kv_cache.swa_ring_capacity(window, maxpos) == want


def test_fwht_vector(oracle):
    x = np.array(GOLD["fwht_vector"]["x"], np.float32)
    y = oracle.fwht_normalized(x.copy())
    assert abs(np.linalg.norm(y) - np.linalg.norm(x)) < 1e-5
    assert np.allclose(oracle.fwht_normalized(y.copy()), x, atol=1e-5)


def test_rotation_signs(oracle, pkg):
    g = GOLD["rotation_signs_tq_seed"]
    for s in (oracle.rotation_signs(256, oracle.TQ_SEED), pkg.kv_cache.turboquant_signs(256)):
        assert "".join("+" if v > 0 else "-" for v in s[:64]) == g["first64"]
        assert int((s > 0).sum()) == g["positive_of_256"]
