"""ctypes front-end for the CPU oracle (``oracle/liboracle.so``).

Test infrastructure only: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  The GPU library never touches it.
Every wrapper takes and returns numpy arrays; shapes follow the reference's
layouts (weights ``[rows, cols]`` as verbatim GGUF blocks, KV codes
``[positions, n_kv, code_bytes]``, norms ``[positions, n_kv]`` f16 bits).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

TQ_SEED = 0x7459C0DE  # local-engine/src/kv_cache/quant_cache.rs:30
DEFAULT_KV_BITS = 2  # local-engine/src/kv_cache/quant_cache.rs:37


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (see oracle/Makefile)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B" if force else "-s"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.orc_f16_to_f32.restype = C.c_float
        _lib.orc_f16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_f32_to_f16.restype = C.c_uint16
        _lib.orc_f32_to_f16.argtypes = [C.c_float]
        for name in ("orc_dequant_tq2_0", "orc_dequant_q4_0", "orc_dequant_q8_0"):
            f = getattr(_lib, name)
            f.restype = C.c_size_t
            f.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p]
        _lib.orc_tq_code_bytes.restype = C.c_size_t
        _lib.orc_tq_code_bytes.argtypes = [C.c_size_t, C.c_uint]
        _lib.orc_tq_encode.restype = C.c_uint16
        _lib.orc_swa_ring_capacity.restype = C.c_size_t
        _lib.orc_swa_ring_capacity.argtypes = [C.c_size_t, C.c_size_t]
        _lib.orc_max_threads.restype = C.c_int
    return _lib


def _p(a: np.ndarray) -> C.c_void_p:
    return C.c_void_p(a.ctypes.data)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def _sz(v) -> C.c_size_t:
    return C.c_size_t(int(v))


# ---------------------------------------------------------------- f16 ------
def f16_to_f32(bits: np.ndarray) -> np.ndarray:
    b = _c(bits, np.uint16)
    out = np.empty(b.shape, np.float32)
    lib().orc_f16_to_f32_array(_p(b), _p(out), _sz(b.size))
    return out


def f32_to_f16(x: np.ndarray) -> np.ndarray:
    a = _c(x, np.float32)
    out = np.empty(a.shape, np.uint16)
    lib().orc_f32_to_f16_array(_p(a), _p(out), _sz(a.size))
    return out


# ------------------------------------------------------------ dequant ------
def _dequant(fn: str, block_elems: int, block_bytes: int, data: np.ndarray, num_elements=None) -> np.ndarray:
    d = _c(data, np.uint8).reshape(-1)
    blocks = d.size // block_bytes
    if num_elements is None:
        num_elements = blocks * block_elems
    out = np.empty(min(num_elements, blocks * block_elems), np.uint16)
    n = getattr(lib(), fn)(_p(d), _sz(d.size), _sz(num_elements), _p(out))
    return out[:n]


def dequant_q4_0(data, num_elements=None) -> np.ndarray:
    """f16 bit patterns, local-engine/src/qat_recover.rs:64-97."""
    return _dequant("orc_dequant_q4_0", 32, 18, data, num_elements)


def dequant_tq2_0(data, num_elements=None) -> np.ndarray:
    """f16 bit patterns, local-engine/src/qat_recover.rs:23-52."""
    return _dequant("orc_dequant_tq2_0", 256, 66, data, num_elements)


def dequant_q8_0(data, num_elements=None) -> np.ndarray:
    return _dequant("orc_dequant_q8_0", 32, 34, data, num_elements)


def expand_q4_0_f32(data, rows, cols) -> np.ndarray:
    d = _c(data, np.uint8).reshape(-1)
    out = np.empty((rows, cols), np.float32)
    lib().orc_expand_q4_0_f32(_p(d), _sz(rows), _sz(cols), _p(out))
    return out


def expand_tq2_0_f32(data, rows, cols) -> np.ndarray:
    d = _c(data, np.uint8).reshape(-1)
    out = np.empty((rows, cols), np.float32)
    lib().orc_expand_tq2_0_f32(_p(d), _sz(rows), _sz(cols), _p(out))
    return out


# ---------------------------------------------------------------- dot ------
def matvec_f32(dq, v) -> np.ndarray:
    dq = _c(dq, np.float32)
    v = _c(v, np.float32)
    rows, cols = dq.shape
    y = np.empty(rows, np.float32)
    lib().orc_matvec_f32(_p(dq), _p(v), _sz(rows), _sz(cols), _p(y))
    return y


def matvec_f64(dq, v) -> np.ndarray:
    dq = _c(dq, np.float32)
    v = _c(v, np.float32)
    rows, cols = dq.shape
    y = np.empty(rows, np.float64)
    lib().orc_matvec_f64(_p(dq), _p(v), _sz(rows), _sz(cols), _p(y))
    return y


def matmul_nt_f32(a, dq) -> np.ndarray:
    a = _c(a, np.float32)
    dq = _c(dq, np.float32)
    m, k = a.shape
    n = dq.shape[0]
    c = np.empty((m, n), np.float32)
    lib().orc_matmul_nt_f32(_p(a), _p(dq), _sz(m), _sz(k), _sz(n), _p(c))
    return c


def matvec_quant_ref(fmt: str, data, x, rows, cols, threads=1) -> np.ndarray:
    """Reference CPU path: block dequant to f16, widen, sequential f32 dot."""
    d = _c(data, np.uint8).reshape(-1)
    x = _c(x, np.float32)
    y = np.empty(rows, np.float32)
    lib().orc_matvec_quant_ref(C.c_int(0 if fmt == "q4_0" else 1), _p(d), _p(x), _sz(rows), _sz(cols), _p(y),
                               C.c_int(threads))
    return y


# --------------------------------------------------------- TurboQuant ------
def fwht_normalized(v) -> np.ndarray:
    a = _c(v, np.float32).copy()
    lib().orc_fwht_normalized(_p(a), _sz(a.size))
    return a


def rotation_signs(dim: int, seed: int = TQ_SEED) -> np.ndarray:
    out = np.empty(dim, np.float32)
    lib().orc_rotation_signs(_sz(dim), C.c_uint64(seed), _p(out))
    return out


def lloyd_max_gaussian(bits: int) -> np.ndarray:
    out = np.empty(1 << bits, np.float32)
    lib().orc_lloyd_max_gaussian(C.c_uint(bits), _p(out))
    return out


def tq_levels(dim: int, bits: int) -> np.ndarray:
    out = np.empty(1 << bits, np.float32)
    lib().orc_tq_levels(_sz(dim), C.c_uint(bits), _p(out))
    return out


def tq_code_bytes(dim: int, bits: int) -> int:
    return int(lib().orc_tq_code_bytes(dim, bits))


def tq_encode(x, bits, signs, levels):
    """One vector -> (codes u8[code_bytes], norm f16 bits, rotated f32[dim])."""
    x = _c(x, np.float32)
    dim = x.size
    signs = _c(signs, np.float32)
    levels = _c(levels, np.float32)
    rot = np.empty(dim, np.float32)
    codes = np.empty(tq_code_bytes(dim, bits), np.uint8)
    norm = lib().orc_tq_encode(_p(x), _sz(dim), C.c_uint(bits), _p(signs), _p(levels), _p(rot), _p(codes))
    return codes, np.uint16(norm), rot


def tq_decode(codes, norm_bits, dim, bits, signs, levels) -> np.ndarray:
    codes = _c(codes, np.uint8)
    signs = _c(signs, np.float32)
    levels = _c(levels, np.float32)
    out = np.empty(dim, np.float32)
    lib().orc_tq_decode(_p(codes), C.c_uint16(int(norm_bits)), _sz(dim), C.c_uint(bits), _p(signs), _p(levels), _p(out))
    return out


def tq_write_kv(inp_f16_bits, n_kv, dim, bits, signs, levels, position, ring_capacity, packed, norms):
    """Encode [num_tokens, n_kv, dim] f16 rows into `packed` / `norms` in place."""
    inp = _c(inp_f16_bits, np.uint16)
    num_tokens = inp.size // (n_kv * dim)
    signs = _c(signs, np.float32)
    levels = _c(levels, np.float32)
    assert packed.dtype == np.uint8 and norms.dtype == np.uint16
    assert packed.flags.c_contiguous and norms.flags.c_contiguous
    lib().orc_tq_write_kv(_p(inp), _sz(num_tokens), _sz(n_kv), _sz(dim), C.c_uint(bits), _p(signs), _p(levels),
                          _sz(position), _sz(ring_capacity), _p(packed), _p(norms))


def hadamard_rotate(x, signs, head_dim, num_heads, pre_sign, post_sign) -> np.ndarray:
    x = _c(x, np.float32)
    signs = _c(signs, np.float32)
    out = np.empty(num_heads * head_dim, np.float32)
    lib().orc_hadamard_rotate(_p(x), _p(signs), _p(out), _sz(head_dim), _sz(num_heads), C.c_int(int(pre_sign)),
                              C.c_int(int(post_sign)))
    return out


def attention_tq_codespace(rq, k_codes, k_norms, v_codes, v_norms, levels, head_dim, kv_len, current_pos,
                           num_q_heads, num_kv_heads, window, bits, ring_capacity, lane_base=0) -> np.ndarray:
    rq = _c(rq, np.float32)
    levels = _c(levels, np.float32)
    out = np.empty(num_q_heads * head_dim, np.float32)
    lib().orc_attention_tq_codespace(_p(rq), _p(_c(k_codes, np.uint8)), _p(_c(k_norms, np.uint16)),
                                     _p(_c(v_codes, np.uint8)), _p(_c(v_norms, np.uint16)), _p(levels), _p(out),
                                     _sz(head_dim), _sz(kv_len), _sz(current_pos), _sz(num_q_heads),
                                     _sz(num_kv_heads), _sz(window), C.c_uint(bits), _sz(ring_capacity),
                                     _sz(lane_base))
    return out


def attention_tq_decode_then_attend(q, k_codes, k_norms, v_codes, v_norms, levels, signs, head_dim, kv_len,
                                    current_pos, num_q_heads, num_kv_heads, window, bits, ring_capacity,
                                    threads=1) -> np.ndarray:
    q = _c(q, np.float32)
    out = np.empty(num_q_heads * head_dim, np.float32)
    lib().orc_attention_tq_decode_then_attend(
        _p(q), _p(_c(k_codes, np.uint8)), _p(_c(k_norms, np.uint16)), _p(_c(v_codes, np.uint8)),
        _p(_c(v_norms, np.uint16)), _p(_c(levels, np.float32)), _p(_c(signs, np.float32)), _p(out), _sz(head_dim),
        _sz(kv_len), _sz(current_pos), _sz(num_q_heads), _sz(num_kv_heads), _sz(window), C.c_uint(bits),
        _sz(ring_capacity), C.c_int(threads))
    return out


def attention_f16(q_bits, k_bits, v_bits, head_dim, kv_len, current_pos, num_q_heads, num_kv_heads, window=0):
    out = np.empty(num_q_heads * head_dim, np.float32)
    lib().orc_attention_f16(_p(_c(q_bits, np.uint16)), _p(_c(k_bits, np.uint16)), _p(_c(v_bits, np.uint16)), _p(out),
                            _sz(head_dim), _sz(kv_len), _sz(current_pos), _sz(num_q_heads), _sz(num_kv_heads),
                            _sz(window))
    return out


def tq2_dequant_legacy(packed, scales_bits, n) -> np.ndarray:
    out = np.empty(n, np.uint16)
    lib().orc_tq2_dequant_legacy(_p(_c(packed, np.uint8)), _p(_c(scales_bits, np.uint16)), _p(out), _sz(n))
    return out


def matmul_f16_nt(a_bits, b_bits, m, k, n) -> np.ndarray:
    c = np.empty((m, n), np.float32)
    lib().orc_matmul_f16_nt(_p(_c(a_bits, np.uint16)), _p(_c(b_bits, np.uint16)), _p(c), _sz(m), _sz(k), _sz(n))
    return c


def tensor_bytes(fmt: str, n_elements: int) -> int:
    """Payload bytes of a GGUF tensor: ceil(n / block elements) * block bytes
    (local-engine/src/gguf.rs:247-311: Q4_0 32 -> 18, Q8_0 32 -> 34, TQ2_0 256 -> 66)."""
    elems, size = {"q4_0": (32, 18), "q8_0": (32, 34), "tq2_0": (256, 66)}[fmt]
    return -(-n_elements // elems) * size


def swa_ring_capacity(window: int, max_positions: int) -> int:
    return int(lib().orc_swa_ring_capacity(window, max_positions))


def max_threads() -> int:
    return int(lib().orc_max_threads())
