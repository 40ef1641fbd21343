"""Seeded synthetic inputs for the measured configurations.

Weights follow the GGUF block layouts byte for byte (Q4_0: f16 d + 16 quant bytes per 32
weights; TQ2_0: 64 code bytes + f16 d per 256 weights, shaders/matvec_quant.metal:11-17);
distributions: Q4_0 d = f16(|N(0, 0.02)| / 8) with uniform nibbles, TQ2_0 2-bit fields
uniform over {0, 1, 2} with d = f16(|N(0, 0.02)|), activations N(0, 1)."""
from __future__ import annotations

import numpy as np

BASE_SEED = 0x5EED


def rng(config_id: int, stream: int = 0) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64([BASE_SEED + config_id, stream]))


def q4_0_weights(rows: int, cols: int, g: np.random.Generator) -> np.ndarray:
    nb = rows * (cols // 32)
    raw = np.empty((nb, 18), np.uint8)
    d = (np.abs(g.standard_normal(nb, dtype=np.float32) * np.float32(0.02)) / np.float32(8.0)).astype(np.float16)
    raw[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
    raw[:, 2:] = g.integers(0, 256, (nb, 16), dtype=np.uint8)
    return raw.reshape(-1)


def tq2_0_weights(rows: int, cols: int, g: np.random.Generator) -> np.ndarray:
    nb = rows * (cols // 256)
    raw = np.empty((nb, 66), np.uint8)
    codes = g.integers(0, 3, (nb, 64, 4), dtype=np.uint8)          # four 2-bit fields per byte, never 3
    raw[:, :64] = codes[..., 0] | (codes[..., 1] << 2) | (codes[..., 2] << 4) | (codes[..., 3] << 6)
    d = np.abs(g.standard_normal(nb, dtype=np.float32) * np.float32(0.02)).astype(np.float16)
    raw[:, 64:] = d.view(np.uint8).reshape(nb, 2)
    return raw.reshape(-1)


def weights(fmt: str, rows: int, cols: int, g: np.random.Generator) -> np.ndarray:
    return q4_0_weights(rows, cols, g) if fmt == "q4_0" else tq2_0_weights(rows, cols, g)


def weight_bytes(fmt: str, rows: int, cols: int) -> int:
    return rows * (cols // 32) * 18 if fmt == "q4_0" else rows * (cols // 256) * 66


def activations(m: int, k: int, g: np.random.Generator) -> np.ndarray:
    return g.standard_normal((m, k), dtype=np.float32)


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even bf16 bit patterns of an f32 array."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    return ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


# One decoder layer's projections with the mixed layout of the small-batch configuration:
# (name, format, rows N, cols K)
DECODER_LAYER = (
    ("attn_q", "q4_0", 2048, 2048),
    ("attn_k", "q4_0", 256, 2048),
    ("attn_v", "q4_0", 256, 2048),
    ("attn_output", "q4_0", 2048, 2048),
    ("ffn_gate", "tq2_0", 8192, 2048),
    ("ffn_up", "tq2_0", 8192, 2048),
    ("ffn_down", "tq2_0", 2048, 8192),
)


def kv_rows(t: int, n_kv: int, head_dim: int, g: np.random.Generator) -> np.ndarray:
    """K or V rows [t, n_kv, head_dim] as f16 N(0, 1)."""
    return g.standard_normal((t, n_kv, head_dim), dtype=np.float32).astype(np.float16)
