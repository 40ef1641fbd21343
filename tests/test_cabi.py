"""CPU-side checks of the C ABI: the library loads, exports every symbol the header
declares, and the host-side pieces (codec parameters, flags, error text) behave like the
reference. No GPU work is issued here."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "local_hip.h")).read()
    return sorted(set(re.findall(r"LH_API[^;(]*?\b(lh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg.lib()
    names = header_symbols()
    assert len(names) >= 60
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_constants_and_flags(pkg):
    lib = pkg.lib()
    # kernels.rs:6155, 6160, 6362
    assert (lib.lh_smallm_max_m(), lib.lh_batchm_max_m(), lib.lh_multivec_max_m()) == (8, 4, 16)
    assert pkg.Kernels.SMALLM_MAX_M == 8 and pkg.Kernels.BATCHM_MAX_M == 4 and pkg.Kernels.MULTIVEC_MAX_M == 16
    assert pkg.Kernels.batchm_enabled() in (True, False)
    # kernels.rs:1265-1278 flash_split_count = clamp(ceil(n/16), 1, 16)
    f = lib.lh_flash_split_count
    assert [f(0), f(1), f(16), f(17), f(255), f(256), f(100000)] == [1, 1, 1, 2, 16, 16, 16]


def test_codec_parameters_match_oracle(pkg, oracle):
    """The product's host codec (C++) and the oracle (C) restate turboquant.rs independently;
    they must agree bit for bit."""
    from local_ai_amd import kv_cache
    for dim in (64, 128, 256, 512):
        for bits in (2, 3, 4):
            assert np.array_equal(kv_cache.turboquant_levels(dim, bits).view(np.uint32),
                                  oracle.tq_levels(dim, bits).view(np.uint32))
            assert kv_cache.code_bytes(dim, bits) == oracle.tq_code_bytes(dim, bits)
        for seed in (oracle.TQ_SEED, 42, 0):
            assert np.array_equal(kv_cache.turboquant_signs(dim, seed), oracle.rotation_signs(dim, seed))
    assert kv_cache.swa_ring_capacity(512, 131072) == 1024 and kv_cache.swa_ring_capacity(512, 600) == 600
    assert kv_cache.TQ_SEED == 0x7459C0DE and kv_cache.DEFAULT_KV_BITS == 2


def test_kv_bits_from_env(pkg, monkeypatch):
    from local_ai_amd import kv_cache
    for val, want in (("tq3", 3), ("tq4", 4), ("tq2", 2), ("bogus", 2)):
        monkeypatch.setenv("LOCAL_AI_KV_QUANT", val)
        assert kv_cache.kv_bits_from_env() == want
    monkeypatch.delenv("LOCAL_AI_KV_QUANT")
    assert kv_cache.kv_bits_from_env() == 2


def test_no_device_error_is_reported_not_crashed(pkg):
    """Without a GPU the context cannot be created; the call must fail with a NoDevice /
    LibraryCreation error and a message, never fall back to a CPU path."""
    import subprocess
    import sys
    code = ("import __graft_entry__ as ge, sys\n"
            "p = ge.load_package()\n"
            "try:\n"
            "    p.Context(0)\n"
            "    print('HAS_DEVICE')\n"
            "except p.Error as e:\n"
            "    print('ERR', type(e).__name__, str(e))\n")
    out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert "HAS_DEVICE" in out.stdout or "ERR NoDevice" in out.stdout or "ERR LibraryCreation" in out.stdout, out.stdout


def test_quant_weight_validation(pkg):
    class FakeBuf:
        def length(self):
            return 0
    with pytest.raises(pkg.InvalidArgument):
        pkg.QuantWeight.quantized(FakeBuf(), pkg.Q4_0, 4, 100)
    with pytest.raises(pkg.InvalidArgument):
        pkg.QuantWeight.quantized(FakeBuf(), pkg.TQ2_0, 4, 128)
    with pytest.raises(pkg.InvalidArgument):
        pkg.QuantWeight.quantized(FakeBuf(), 7, 4, 256)
    w = pkg.QuantWeight.quantized(FakeBuf(), pkg.TQ2_0, 4, 512)
    assert w.row_bytes() == 132


def test_synth_generators_are_seeded_and_well_formed(pkg, oracle):
    s = pkg.synth
    a = s.weights("tq2_0", 8, 512, s.rng(2))
    b = s.weights("tq2_0", 8, 512, s.rng(2))
    assert np.array_equal(a, b) and a.size == 8 * 2 * 66
    blocks = a.reshape(-1, 66)
    codes = np.stack([(blocks[:, :64] >> (2 * l)) & 3 for l in range(4)])
    assert codes.max() == 2                                     # never the fourth code
    d = blocks[:, 64:].copy().view(np.float16)
    assert np.all(d >= 0)
    q = s.weights("q4_0", 8, 512, s.rng(1)).reshape(-1, 18)
    dq = q[:, :2].copy().view(np.float16).astype(np.float32)
    assert np.all(dq >= 0) and np.mean(dq) < 0.02 / 8 * 1.5
    x = np.array([1.0, -1.0, 3.14159, 1e-3, 65504.0], np.float32)
    bf = s.f32_to_bf16_bits(x)
    assert np.allclose(s.bf16_bits_to_f32(bf), x, rtol=2 ** -8)
