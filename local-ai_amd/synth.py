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


def decoder_layer_tensors(hidden: int, inter: int, n_head: int, n_kv: int, head_dim: int, per_layer_dim: int,
                          g: np.random.Generator, attn_fmt: str = "q4_0", ffn_fmt: str = "tq2_0",
                          output_scale: float | None = None, kv_shared: bool = False) -> dict:
    """Every tensor of one decoder layer (names of local-engine/src/layer.rs:310-328): projections as
    ``(format, rows, cols, payload bytes)``, norm vectors as f16 arrays c * (1 + N(0, 0.1)) with c = 1 except
    for q_norm / k_norm, where c = head_dim^-1/4: normalised q and k then have length head_dim^1/4, so the
    unscaled scores q . k of attention are about N(0, 1) rather than N(0, head_dim)."""
    def proj(fmt, rows, cols):
        return (fmt, rows, cols, weights(fmt, rows, cols, g))

    def norm(n, c=1.0):
        return (np.float32(c) * (np.float32(1.0) + np.float32(0.1) * g.standard_normal(n, dtype=np.float32))) \
            .astype(np.float16)

    qk_scale = float(head_dim) ** -0.25

    t = {
        "attn_norm": norm(hidden), "attn_q": proj(attn_fmt, n_head * head_dim, hidden),
        "q_norm": norm(head_dim, qk_scale), "attn_output": proj(attn_fmt, hidden, n_head * head_dim),
        "attn_post_norm": norm(hidden), "ffn_norm": norm(hidden),
        "ffn_gate": proj(ffn_fmt, inter, hidden), "ffn_up": proj(ffn_fmt, inter, hidden),
        "ffn_down": proj(ffn_fmt, hidden, inter), "ffn_post_norm": norm(hidden),
    }
    if not kv_shared:
        t["attn_k"] = proj(attn_fmt, n_kv * head_dim, hidden)
        t["attn_v"] = proj(attn_fmt, n_kv * head_dim, hidden)
        t["k_norm"] = norm(head_dim, qk_scale)
    if per_layer_dim:
        t["per_layer_inp_gate"] = proj(attn_fmt, per_layer_dim, hidden)
        t["per_layer_proj"] = proj(attn_fmt, hidden, per_layer_dim)
        t["per_layer_post_norm"] = norm(hidden)
    if output_scale is not None:
        t["layer_output_scale"] = np.array([output_scale], np.float16)
    return t


def decode_model_tensors(config, g: np.random.Generator, intermediate_size, attn_fmt: str = "q4_0", ffn_fmt: str = "tq2_0",
                         table_rows: int | None = None) -> dict:
    """Every tensor of a decode stack shaped by `config` (a pipeline.Gemma4QATConfig): one dict of layer tensors per
    layer (head_dim and KV sharing by layer type; `intermediate_size` an int or one value per layer), the tied
    Q4_0 embedding table, the output norm and, when the configuration has per-layer inputs, their table, projection
    and norm.  `table_rows` distinct rows are generated for the two vocabulary-sized tables and repeated to
    vocab_size (the decode step reads one row of each, so the repetition is invisible to it)."""
    h, n_layer, pld, vocab = config.hidden_size, config.num_hidden_layers, config.hidden_size_per_layer_input, config.vocab_size
    inters = [intermediate_size] * n_layer if isinstance(intermediate_size, int) else list(intermediate_size)
    layers = [decoder_layer_tensors(h, inters[i], config.num_attention_heads, config.num_key_value_heads,
                                    config.attn_head_dim(i), pld, g, attn_fmt, ffn_fmt, kv_shared=config.is_kv_shared(i))
              for i in range(n_layer)]

    def table(cols):
        rows = min(table_rows or vocab, vocab)
        block = q4_0_weights(rows, cols, g).reshape(rows, -1)
        reps = -(-vocab // rows)
        return ("q4_0", vocab, cols, np.tile(block, (reps, 1))[:vocab].reshape(-1))

    t = {"layers": layers, "token_embd": table(h),
         "output_norm": (np.float32(1.0) + np.float32(0.1) * g.standard_normal(h, dtype=np.float32)).astype(np.float16)}
    if pld:
        t["ple_table"] = table(pld * n_layer)
        t["per_layer_model_proj"] = (attn_fmt, pld * n_layer, h, weights(attn_fmt, pld * n_layer, h, g))
        t["per_layer_proj_norm"] = (np.float32(1.0) + np.float32(0.1) * g.standard_normal(pld, dtype=np.float32)).astype(np.float16)
    return t
