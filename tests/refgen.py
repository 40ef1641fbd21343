"""Input generators the reference's own kernel tests use, restated so the parity
tests run on the same payloads (local-metal/src/kernels.rs:8776-8863,
local-engine/src/turboquant.rs:343-354)."""
import numpy as np


def xorshift_bytes(seed: int, n: int) -> np.ndarray:
    """kernels.rs:8776-8786."""
    s = (seed | 1) & 0xFFFFFFFF
    out = np.empty(n, np.uint8)
    for i in range(n):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        out[i] = (s >> 8) & 0xFF
    return out


def q4_0_payload(rows: int, cols: int, seed: int) -> np.ndarray:
    """kernels.rs:8790-8810: d = f16(0.01 + b/2550), 16 raw quant bytes."""
    nb = cols // 32
    rnd = xorshift_bytes(seed, rows * nb * 17).reshape(rows * nb, 17)
    d = (np.float32(0.01) + rnd[:, 0].astype(np.float32) / np.float32(2550.0)).astype(np.float16)
    raw = np.empty((rows * nb, 18), np.uint8)
    raw[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    raw[:, 2:] = rnd[:, 1:]
    return raw.reshape(-1)


def tq2_0_payload(rows: int, cols: int, seed: int) -> np.ndarray:
    """kernels.rs:8814-8841: 64 raw bytes (codes include 3), d = f16(0.05 + b/1275)."""
    nb = cols // 256
    rnd = xorshift_bytes(seed, rows * nb * 65).reshape(rows * nb, 65)
    d = (np.float32(0.05) + rnd[:, 64].astype(np.float32) / np.float32(1275.0)).astype(np.float16)
    raw = np.empty((rows * nb, 66), np.uint8)
    raw[:, :64] = rnd[:, :64]
    raw[:, 64:] = d.view(np.uint8).reshape(-1, 2)
    return raw.reshape(-1)


def test_vector(cols: int):
    """kernels.rs:8857-8863: f16(sin(0.731 i)); returns (f16 array, f32 widened)."""
    i = np.arange(cols, dtype=np.float32)
    v16 = np.sin(i * np.float32(0.731), dtype=np.float32).astype(np.float16)
    return v16, v16.astype(np.float32)


def seeded_vec(n: int, seed: int) -> np.ndarray:
    """turboquant.rs:343-354 (note: only one multiply round, as written there)."""
    M = (1 << 64) - 1
    s = (seed | 1) & M
    out = np.empty(n, np.float32)
    for i in range(n):
        s = (s + 0x9E3779B97F4A7C15) & M
        z = s
        z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & M
        z ^= z >> 31
        out[i] = np.float32(np.float32(z >> 40) / np.float32(1 << 24)) - np.float32(0.5)
    return out


def assert_close(got, want, tol, label=""):
    """kernels.rs:8871-8880: |g - w| <= tol * max(|w|, 1)."""
    got = np.asarray(got, np.float64).reshape(-1)
    want = np.asarray(want, np.float64).reshape(-1)
    assert got.shape == want.shape, f"{label}: length"
    err = np.abs(got - want) / np.maximum(np.abs(want), 1.0)
    i = int(np.argmax(err))
    assert err[i] <= tol, f"{label}[{i}]: got {got[i]}, want {want[i]} (norm err {err[i]:.3e} > {tol})"
    return float(err[i])


def scaled_error(got, want):
    """max |g - w| / max |w|: the error relative to the output's own scale (no floor of 1)."""
    got = np.asarray(got, np.float64).reshape(-1)
    want = np.asarray(want, np.float64).reshape(-1)
    return float(np.max(np.abs(got - want)) / max(float(np.max(np.abs(want))), 1e-30))


def assert_close_both(got, want, tol, label=""):
    """Both gates: the reference's |g - w| <= tol * max(|w|, 1) per element, and the scale-aware
    max|g - w| <= tol * max|w| (which does not loosen when the outputs are smaller than 1).
    Returns (normalised error, scale-aware error) and prints them."""
    e_norm = assert_close(got, want, tol, label)
    e_scaled = scaled_error(got, want)
    print(f"{label}: err/max(|w|,1) {e_norm:.2e}, err/max|w| {e_scaled:.2e}")
    assert e_scaled <= tol, f"{label}: max|g-w| / max|w| = {e_scaled:.3e} > {tol}"
    return e_norm, e_scaled
