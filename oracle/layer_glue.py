"""CPU restatements (numpy) of the reference's decoder-layer glue kernels.

Test infrastructure only, like the rest of ``oracle/``: imported by ``tests/`` as the checker of the
HIP kernels in ``local-ai_amd/csrc/layer_glue.hip``.  Each function follows the Metal kernel it
cites: f32 arithmetic, f16 storage, the same rounding points; reductions are summed in float64 (the
reference's own CPU checks sum sequentially in f32, kernels.rs:7847-7856; both orders agree far below
one f16 ulp of the outputs).

What pins them (tests/test_layer_glue_oracle.py): the reference's known-answer tests --
rms_norm [1,2,3,4] -> x / sqrt(7.5) (kernels.rs:7050-7073), rope identity at position 0 and the
proportional partial-rotary vector (7214-7288), gather of layer 3 from a [5,7,4] iota (7751-7787),
soft cap against math.tanh (7790-7815), gelu(0, 1, -1, 2, +-10) (7076-7117), qk_norm against the
sequential f32 formula (7818-7870), qk_norm_rope == qk_norm then rope bit for bit (7873-7925) --
and closed forms (norm of the normalised row, rotation preserves pair norms, exact f16 sums).
"""
from __future__ import annotations

import numpy as np

F16, F32 = np.float16, np.float32


def _h(x) -> np.ndarray:
    """f16 values as f32."""
    return np.asarray(x, F16).astype(F32)


def rms_norm(x, w, dim: int, rows: int, eps: float, residual=None) -> np.ndarray:
    """shaders/rms_norm.metal:4-46 (and 48-88 with `residual`): f16 out."""
    x = _h(x).reshape(rows, dim)
    ss = (x.astype(np.float64) ** 2).sum(axis=1)
    rms = (F32(1.0) / np.sqrt((ss / dim).astype(F32) + F32(eps))).astype(F32)
    y = x * rms[:, None] * _h(w)[None, :]
    if residual is not None:
        y = y + _h(residual).reshape(rows, dim)
    return y.astype(F16).reshape(-1)


def qk_norm(qk, w, head_dim: int, num_heads: int, eps: float) -> np.ndarray:
    """shaders/qk_norm.metal:6-56: per-head RMSNorm, f16 out."""
    return rms_norm(qk, w, head_dim, num_heads, eps)


def rope(x, head_dim: int, position: int, theta: float, partial_rotary_factor: float, num_heads: int) -> np.ndarray:
    """shaders/rope.metal:14-61: NEOX pairs (i, i + head_dim/2); the first uint(head_dim * prf) / 2 pairs
    rotate with freq = 1 / theta^(2i / head_dim) (f32), the rest pass through; f16 out."""
    xin = np.asarray(x, F16).reshape(num_heads, head_dim)
    x = xin.astype(F32)
    half = head_dim // 2
    rope_angles = int(F32(head_dim) * F32(partial_rotary_factor)) // 2
    out = xin.copy()
    i = np.arange(rope_angles, dtype=np.uint32)
    expo = (F32(2) * i.astype(F32)) / F32(head_dim)
    freq = (F32(1.0) / np.power(F32(theta), expo, dtype=F32)).astype(F32)
    angle = (F32(position) * freq).astype(F32)
    c, s = np.cos(angle.astype(np.float64)), np.sin(angle.astype(np.float64))
    x0, x1 = x[:, :rope_angles].astype(np.float64), x[:, half:half + rope_angles].astype(np.float64)
    out[:, :rope_angles] = (x0 * c - x1 * s).astype(F16)
    out[:, half:half + rope_angles] = (x0 * s + x1 * c).astype(F16)
    return out.reshape(-1)


def qk_norm_rope(x, w, head_dim, num_heads, eps, position, theta, partial_rotary_factor) -> np.ndarray:
    """shaders/qk_norm.metal:70-140: the normalised head is rounded to f16 before it is rotated."""
    return rope(qk_norm(x, w, head_dim, num_heads, eps), head_dim, position, theta, partial_rotary_factor, num_heads)


def gelu_mul(a, b) -> np.ndarray:
    """shaders/gelu.metal:23-41: 0.5 x (1 + tanh(clamp(0.79788456 (x + 0.044715 x^3), -10, 10))) * b, f16 out."""
    x = _h(a)
    inner = F32(0.7978845608) * (x + F32(0.044715) * (x * x * x))
    t = np.tanh(np.clip(inner, F32(-10.0), F32(10.0)).astype(np.float64)).astype(F32)
    g = F32(0.5) * x * (F32(1.0) + t)
    with np.errstate(over="ignore"):   # a product beyond the f16 range rounds to infinity, as half() does
        return (g * _h(b)).astype(F16)


def residual_add(a, b) -> np.ndarray:
    """shaders/residual_add.metal:5-15: f16 + f16, the exact sum rounded once."""
    return (np.asarray(a, F16).astype(np.float64) + np.asarray(b, F16).astype(np.float64)).astype(F16)


def scale_in_place(data, scalar: float) -> np.ndarray:
    """shaders/scale_in_place.metal:5-14: half(float(x) * scalar)."""
    return (_h(data) * F32(scalar)).astype(F16)


def gather_strided_f16(src, row_stride: int, base_off: int, pld: int, n_rows: int) -> np.ndarray:
    """shaders/scale_in_place.metal:21-35."""
    src = np.asarray(src, F16).reshape(-1)
    idx = (np.arange(n_rows)[:, None] * row_stride + base_off + np.arange(pld)[None, :]).reshape(-1)
    return src[idx]


def logit_softcap(data, cap: float) -> np.ndarray:
    """shaders/scale_in_place.metal:39-49: cap * tanh(x / cap) in f32."""
    x = np.asarray(data, F32)
    return (F32(cap) * np.tanh((x / F32(cap)).astype(np.float64))).astype(F32)


def matvec_f16(w, x, rows: int, cols: int, out_f32: bool = False) -> np.ndarray:
    """shaders/matvec_f16.metal:14-133: y = W . x with f16 weights, f16 or f32 x, f32 accumulation (summed here in
    float64), y rounded to f16 unless `out_f32`."""
    w = np.asarray(w, F16).reshape(rows, cols).astype(np.float64)
    xv = np.asarray(x).astype(np.float64).reshape(cols)
    y = w @ xv
    return y.astype(F32) if out_f32 else y.astype(F32).astype(F16)
