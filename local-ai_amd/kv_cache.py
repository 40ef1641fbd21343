"""``QuantizedKvCache`` (local-engine/src/kv_cache/quant_cache.rs:73-700): TurboQuant KV cache
in device memory with ring addressing for sliding-window layers."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import Buffer, InvalidArgument, Kernels, lib

TQ_SEED = 0x7459C0DE       # quant_cache.rs:30
DEFAULT_KV_BITS = 2        # quant_cache.rs:37
MAX_PREFILL_CHUNK = 256    # quant_cache.rs:43


def swa_ring_capacity(window: int, max_positions: int) -> int:
    """quant_cache.rs:48-54."""
    f = lib().lh_swa_ring_capacity
    f.restype = C.c_size_t
    return int(f(C.c_size_t(window), C.c_size_t(max_positions)))


def kv_bits_from_env() -> int:
    """quant_cache.rs:60-66 (LOCAL_AI_KV_QUANT = tq2 | tq3 | tq4)."""
    f = lib().lh_kv_bits_from_env
    f.restype = C.c_uint32
    return int(f())


def turboquant_levels(dim: int, bits: int) -> np.ndarray:
    out = np.empty(1 << bits, np.float32)
    rc = lib().lh_turboquant_levels(C.c_uint32(dim), C.c_uint32(bits), C.c_void_p(out.ctypes.data))
    if rc:
        raise InvalidArgument(lib().lh_last_error().decode())
    return out


def turboquant_signs(dim: int, seed: int = TQ_SEED) -> np.ndarray:
    out = np.empty(dim, np.float32)
    rc = lib().lh_turboquant_signs(C.c_uint32(dim), C.c_uint64(seed), C.c_void_p(out.ctypes.data))
    if rc:
        raise InvalidArgument(lib().lh_last_error().decode())
    return out


def code_bytes(dim: int, bits: int) -> int:
    f = lib().lh_turboquant_code_bytes
    f.restype = C.c_uint32
    return int(f(C.c_uint32(dim), C.c_uint32(bits)))


class QuantizedKvCache:
    def __init__(self, ctx, n_kv_heads: int, head_dim: int, max_positions: int, bits: int = DEFAULT_KV_BITS,
                 physical_positions: int | None = None, sliding_window: int = 0):
        """quant_cache.rs:182-229 new_with_bits_and_ring."""
        if not 2 <= bits <= 4:
            raise InvalidArgument(f"TurboQuant bits must be 2..=4, got {bits}")
        if head_dim & (head_dim - 1) or head_dim > 512 or head_dim == 0:
            raise InvalidArgument(f"TurboQuant head_dim must be a power of two <= 512, got {head_dim}")
        if physical_positions is None:
            physical_positions = max_positions
        physical_positions = max(min(physical_positions, max_positions), 1)
        if physical_positions < max_positions and physical_positions < sliding_window + MAX_PREFILL_CHUNK - 1:
            raise InvalidArgument(f"ring capacity {physical_positions} too small for window {sliding_window} "
                                  f"+ prefill slack {MAX_PREFILL_CHUNK - 1}")
        self.ctx = ctx
        self.n_kv_heads, self.head_dim, self.bits = n_kv_heads, head_dim, bits
        self.max_positions, self.physical_positions = max_positions, physical_positions
        self._cb = code_bytes(head_dim, bits)
        slots = physical_positions * n_kv_heads
        self.levels = Buffer.from_slice(ctx, turboquant_levels(head_dim, bits))
        self.signs = Buffer.from_slice(ctx, turboquant_signs(head_dim, TQ_SEED))
        self.keys_q = Buffer.empty(ctx, max(slots * self._cb, 1))
        self.values_q = Buffer.empty(ctx, max(slots * self._cb, 1))
        self.key_norms = Buffer.empty(ctx, max(slots, 1) * 2)
        self.value_norms = Buffer.empty(ctx, max(slots, 1) * 2)

    def is_ringed(self) -> bool:
        return self.physical_positions < self.max_positions

    def ring_capacity(self) -> int:
        """quant_cache.rs:258-264: physical rows for a ring, 0 for absolute addressing."""
        return self.physical_positions if self.is_ringed() else 0

    def code_bytes(self) -> int:
        return self._cb

    def reset(self) -> None:
        """quant_cache.rs:367-380."""
        for b in (self.keys_q, self.values_q, self.key_norms, self.value_norms):
            b.fill_zero()

    def write_kv_gpu_into(self, batch, kernels: Kernels, k_src: Buffer, v_src: Buffer, position: int, n_rows: int):
        """quant_cache.rs:391-444."""
        if position + n_rows > self.max_positions:
            raise InvalidArgument(f"KV write [{position}..{position + n_rows}) exceeds capacity {self.max_positions}")
        for src, codes, norms in ((k_src, self.keys_q, self.key_norms), (v_src, self.values_q, self.value_norms)):
            kernels.encode_kv_turboquant_into(batch, src, self.levels, self.signs, codes, norms, self.head_dim,
                                              self.n_kv_heads, n_rows, self.bits, position, self.ring_capacity())

    def dequantize_into(self, ctx, kernels: Kernels, k_out: Buffer, v_out: Buffer, seq_len: int, token_start: int):
        """quant_cache.rs:490-532."""
        for codes, norms, out in ((self.keys_q, self.key_norms, k_out), (self.values_q, self.value_norms, v_out)):
            kernels.dequantize_kv_turboquant(ctx, codes, norms, self.levels, self.signs, out, self.head_dim,
                                             self.n_kv_heads, seq_len, self.bits, token_start, self.ring_capacity())

    def fused_attention_into(self, batch, kernels: Kernels, q: Buffer, rq: Buffer, vacc: Buffer, attn_out: Buffer,
                             seq_len: int, current_pos: int, n_q_heads: int, window: int):
        """quant_cache.rs:548-598: rotate q, attend over codes, inverse-rotate to f16."""
        hd = self.head_dim
        kernels.hadamard_rotate_hf_into(batch, q, self.signs, rq, hd, n_q_heads, True, False)
        kernels.flash_attention_tq_rotated_into(batch, rq, self.keys_q, self.key_norms, self.values_q, self.value_norms,
                                                self.levels, self.signs, vacc, attn_out, hd, seq_len, current_pos,
                                                n_q_heads, self.n_kv_heads, window, self.bits, self.ring_capacity())

    def prepare_token_into(self, batch, kernels: Kernels, q: Buffer, k, v, q_norm, k_norm, rq: Buffer, position: int,
                           n_q_heads: int, eps: float, theta: float, partial_rotary_factor: float) -> None:
        """One dispatch for a decoded token's head norms, RoPE, V norm, ``write_kv_gpu_into`` (quant_cache.rs:391-444)
        and the query rotation that opens ``fused_attention_into`` (quant_cache.rs:560-570); ``k = v = None`` leaves
        the cache alone (a KV-shared layer)."""
        if k is not None and position + 1 > self.max_positions:
            raise InvalidArgument(f"KV write [{position}..{position + 1}) exceeds capacity {self.max_positions}")
        kernels.decode_qkv_prepare_into(batch, q, k, v, q_norm, k_norm, self.levels, self.signs, rq,
                                        self.keys_q, self.key_norms, self.values_q, self.value_norms, self.head_dim,
                                        n_q_heads, self.n_kv_heads, eps, position, theta, partial_rotary_factor, self.bits,
                                        self.ring_capacity())

    def attention_from_rotated_into(self, batch, kernels: Kernels, rq: Buffer, vacc: Buffer, attn_out: Buffer,
                                    seq_len: int, current_pos: int, n_q_heads: int, window: int) -> None:
        """quant_cache.rs:571-598: the attend and rotate-back steps of ``fused_attention_into`` for a query that
        ``prepare_token_into`` has already rotated."""
        hd = self.head_dim
        kernels.flash_attention_tq_rotated_into(batch, rq, self.keys_q, self.key_norms, self.values_q, self.value_norms,
                                                self.levels, self.signs, vacc, attn_out, hd, seq_len, current_pos,
                                                n_q_heads, self.n_kv_heads, window, self.bits, self.ring_capacity())

    def attention_from_rotated_lazy_into(self, batch, kernels: Kernels, rq: Buffer, vacc: Buffer, attn_out: Buffer,
                                         seq_len: int, current_pos: int, n_q_heads: int, window: int) -> bool:
        """quant_cache.rs:571-598 for a caller whose output projection can rotate its input itself: True when
        ``attn_out`` holds the rotated f16 heads (the rotation rode in the merge launch), False when the f32 heads in
        ``vacc`` are still in code space (quant_cache.rs:590-598 is left to the caller)."""
        return kernels.flash_attention_tq_rotated_lazy_into(batch, rq, self.keys_q, self.key_norms, self.values_q,
                                                            self.value_norms, self.levels, self.signs, vacc, attn_out,
                                                            self.head_dim, seq_len, current_pos, n_q_heads,
                                                            self.n_kv_heads, window, self.bits, self.ring_capacity())

    def prepare_rows_into(self, batch, kernels: Kernels, q: Buffer, k, v, q_norm, k_norm, rq: Buffer, start_pos: int,
                          n_rows: int, n_q_heads: int, eps: float, theta: float, partial_rotary_factor: float) -> None:
        """``prepare_token_into`` for the ``n_rows`` consecutive tokens of a prefill chunk."""
        if k is not None and start_pos + n_rows > self.max_positions:
            raise InvalidArgument(f"KV write [{start_pos}..{start_pos + n_rows}) exceeds capacity {self.max_positions}")
        kernels.decode_qkv_prepare_rows_into(batch, q, k, v, q_norm, k_norm, self.levels, self.signs, rq, self.keys_q,
                                             self.key_norms, self.values_q, self.value_norms, None, self.head_dim,
                                             n_q_heads, self.n_kv_heads, n_rows, eps, start_pos, theta,
                                             partial_rotary_factor, self.bits, self.ring_capacity(), 0)

    def project_and_prepare_rows_into(self, batch, kernels: Kernels, weight_type: int, x: Buffer, w_q: Buffer, w_k: Buffer,
                                      w_v: Buffer, k_dim: int, q: Buffer, k: Buffer, v: Buffer, q_norm, k_norm, rq: Buffer,
                                      start_pos: int, n_rows: int, n_q_heads: int, eps: float, theta: float,
                                      partial_rotary_factor: float) -> None:
        """The Q / K / V projections of a chunk's rows and ``prepare_rows_into`` on their outputs as one encoded step."""
        if start_pos + n_rows > self.max_positions:
            raise InvalidArgument(f"KV write [{start_pos}..{start_pos + n_rows}) exceeds capacity {self.max_positions}")
        kernels.matmul_nt_qkv_prepare_rows_into(batch, weight_type, x, w_q, w_k, w_v, k_dim, q, k, v, q_norm, k_norm,
                                                self.levels, self.signs, rq, self.keys_q, self.key_norms, self.values_q,
                                                self.value_norms, None, self.head_dim, n_q_heads, self.n_kv_heads, n_rows,
                                                eps, start_pos, theta, partial_rotary_factor, self.bits,
                                                self.ring_capacity(), 0)

    def attention_rows_from_rotated_into(self, batch, kernels: Kernels, rq: Buffer, vacc: Buffer, attn_out: Buffer,
                                         kv_len: int, start_pos: int, n_rows: int, n_q_heads: int, window: int) -> None:
        """quant_cache.rs:660-700: the attend and rotate-back steps of ``fused_attention_batch_into``."""
        hd = self.head_dim
        kernels.flash_attention_tq_prefill_tiled_into(batch, rq, self.keys_q, self.key_norms, self.values_q,
                                                      self.value_norms, self.levels, vacc, hd, kv_len, start_pos, n_rows,
                                                      n_q_heads, self.n_kv_heads, window, self.bits, self.ring_capacity())
        kernels.hadamard_rotate_fh_into(batch, vacc, self.signs, attn_out, hd, n_rows * n_q_heads, False, True)

    def fused_attention_batch_into(self, batch, kernels: Kernels, q: Buffer, rq: Buffer, vacc: Buffer,
                                   attn_out: Buffer, kv_len: int, start_pos: int, n_rows: int, n_q_heads: int,
                                   window: int, tiled: bool = True):
        """quant_cache.rs:620-700."""
        hd = self.head_dim
        vecs = n_rows * n_q_heads
        kernels.hadamard_rotate_hf_into(batch, q, self.signs, rq, hd, vecs, True, False)
        fn = kernels.flash_attention_tq_prefill_tiled_into if tiled else kernels.flash_attention_tq_prefill_into
        fn(batch, rq, self.keys_q, self.key_norms, self.values_q, self.value_norms, self.levels, vacc, hd, kv_len,
           start_pos, n_rows, n_q_heads, self.n_kv_heads, window, self.bits, self.ring_capacity())
        kernels.hadamard_rotate_fh_into(batch, vacc, self.signs, attn_out, hd, vecs, False, True)


class QuantizedUnifiedKvPool:
    """``QuantizedUnifiedKvPool`` (local-engine/src/kv_cache/quant_unified_pool.rs:33-345): one layer's
    TurboQuant KV for ``n_lanes`` independent sequences, laid out
    ``[n_lanes, lane rows, n_kv_heads, code_bytes]``; a device ``positions[n_lanes]`` u32 buffer carries
    every lane's current position so one encode launch and one attention launch serve all lanes."""

    def __init__(self, ctx, n_lanes: int, lane_capacity: int, n_kv_heads: int, head_dim: int, bits: int,
                 lane_ring_capacity: int = 0):
        """quant_unified_pool.rs:69-104: a ringed lane keeps only its first ``lane_ring_capacity`` rows."""
        if not 2 <= bits <= 4:
            raise InvalidArgument(f"TurboQuant bits must be 2..=4, got {bits}")
        lane_ring_capacity = min(lane_ring_capacity, lane_capacity)
        self.ctx = ctx
        self.n_lanes, self.lane_capacity, self.lane_ring_capacity = n_lanes, lane_capacity, lane_ring_capacity
        self.n_kv_heads, self.head_dim, self.bits = n_kv_heads, head_dim, bits
        self._cb = code_bytes(head_dim, bits)
        slots = max(n_lanes * self.lane_stride() * n_kv_heads, 1)
        self.levels = Buffer.from_slice(ctx, turboquant_levels(head_dim, bits))
        self.signs = Buffer.from_slice(ctx, turboquant_signs(head_dim, TQ_SEED))
        self.keys_q = Buffer.empty(ctx, slots * self._cb)
        self.values_q = Buffer.empty(ctx, slots * self._cb)
        self.key_norms = Buffer.empty(ctx, slots * 2)
        self.value_norms = Buffer.empty(ctx, slots * 2)

    def lane_stride(self) -> int:
        """quant_unified_pool.rs:116-122: physical rows per lane, the lane base stride of the batched kernels."""
        return self.lane_ring_capacity if self.lane_ring_capacity else self.lane_capacity

    def write_kv_into(self, batch, kernels: Kernels, k_src: Buffer, v_src: Buffer, positions: Buffer,
                      active_lanes: int) -> None:
        """quant_unified_pool.rs:138-181: encode one K and one V row per lane at ``positions[lane]``."""
        lanes = min(active_lanes, self.n_lanes)
        for src, codes, norms in ((k_src, self.keys_q, self.key_norms), (v_src, self.values_q, self.value_norms)):
            kernels.encode_kv_turboquant_batched_into(batch, src, self.levels, self.signs, codes, norms, positions,
                                                      self.head_dim, self.n_kv_heads, self.lane_stride(), self.bits,
                                                      lanes, self.lane_ring_capacity)

    def attention_into(self, batch, kernels: Kernels, q: Buffer, rq: Buffer, vacc: Buffer, attn_out: Buffer,
                       positions: Buffer, n_q_heads: int, window: int, active_lanes: int) -> None:
        """quant_unified_pool.rs:194-256: rotate every lane's query heads, attend over the lane's codes up to its
        own position, rotate back to f16."""
        hd = self.head_dim
        lanes = min(active_lanes, self.n_lanes)
        total_heads = lanes * n_q_heads
        kernels.hadamard_rotate_hf_into(batch, q, self.signs, rq, hd, total_heads, True, False)
        kernels.flash_attention_tq_batched_into(batch, rq, self.keys_q, self.key_norms, self.values_q,
                                                self.value_norms, self.levels, vacc, positions, hd, self.lane_stride(),
                                                n_q_heads, self.n_kv_heads, window, self.bits, lanes,
                                                self.lane_ring_capacity)
        kernels.hadamard_rotate_fh_into(batch, vacc, self.signs, attn_out, hd, total_heads, False, True)

    def prepare_lanes_into(self, batch, kernels: Kernels, q: Buffer, k, v, q_norm, k_norm, rq: Buffer, positions: Buffer,
                           active_lanes: int, n_q_heads: int, eps: float, theta: float,
                           partial_rotary_factor: float) -> None:
        """One dispatch for every lane's head norms, RoPE, V norm, ``write_kv_into`` and the query rotation that opens
        ``attention_into``; ``k = v = None`` leaves the pool alone (a KV-shared layer)."""
        lanes = min(active_lanes, self.n_lanes)
        kernels.decode_qkv_prepare_rows_into(batch, q, k, v, q_norm, k_norm, self.levels, self.signs, rq, self.keys_q,
                                             self.key_norms, self.values_q, self.value_norms, positions, self.head_dim,
                                             n_q_heads, self.n_kv_heads, lanes, eps, 0, theta, partial_rotary_factor,
                                             self.bits, self.lane_ring_capacity, self.lane_stride())

    def project_and_prepare_lanes_into(self, batch, kernels: Kernels, weight_type: int, x: Buffer, w_q: Buffer, w_k: Buffer,
                                       w_v: Buffer, k_dim: int, q: Buffer, k: Buffer, v: Buffer, q_norm, k_norm, rq: Buffer,
                                       positions: Buffer, active_lanes: int, n_q_heads: int, eps: float, theta: float,
                                       partial_rotary_factor: float) -> None:
        """The Q / K / V projections of every lane and ``prepare_lanes_into`` on their outputs as one encoded step."""
        lanes = min(active_lanes, self.n_lanes)
        kernels.matmul_nt_qkv_prepare_rows_into(batch, weight_type, x, w_q, w_k, w_v, k_dim, q, k, v, q_norm, k_norm,
                                                self.levels, self.signs, rq, self.keys_q, self.key_norms, self.values_q,
                                                self.value_norms, positions, self.head_dim, n_q_heads, self.n_kv_heads,
                                                lanes, eps, 0, theta, partial_rotary_factor, self.bits,
                                                self.lane_ring_capacity, self.lane_stride())

    def attention_from_rotated_into(self, batch, kernels: Kernels, rq: Buffer, vacc: Buffer, attn_out: Buffer,
                                    positions: Buffer, n_q_heads: int, window: int, active_lanes: int) -> None:
        """quant_unified_pool.rs:225-256: the attend and rotate-back steps of ``attention_into``."""
        hd = self.head_dim
        lanes = min(active_lanes, self.n_lanes)
        kernels.flash_attention_tq_batched_rotated_into(batch, rq, self.keys_q, self.key_norms, self.values_q,
                                                        self.value_norms, self.levels, self.signs, vacc, attn_out,
                                                        positions, hd, self.lane_stride(), n_q_heads, self.n_kv_heads,
                                                        window, self.bits, lanes, self.lane_ring_capacity)

    def copy_prefill_from(self, batch, cache: QuantizedKvCache, lane: int, positions: int) -> None:
        """quant_unified_pool.rs:269-315: seed ``lane`` with the first ``positions`` rows of a single-sequence
        cache that shares the codec (a ringed pair copies the whole physical ring once it has wrapped).  Both
        sides live in device memory here, so the four copies are device-to-device and ordered in ``batch``."""
        if positions > self.lane_capacity:
            raise InvalidArgument(f"prefill {positions} positions exceeds lane_capacity {self.lane_capacity}")
        if lane >= self.n_lanes or positions == 0:
            return
        if self.lane_ring_capacity and self.lane_ring_capacity != cache.physical_positions:
            raise InvalidArgument(f"pool ring {self.lane_ring_capacity} must match staging cache ring "
                                  f"{cache.physical_positions}")
        rows = (min(positions, self.lane_ring_capacity) if self.lane_ring_capacity else positions) * self.n_kv_heads
        lane_row0 = lane * self.lane_stride() * self.n_kv_heads
        for src, dst, stride in ((cache.keys_q, self.keys_q, self._cb), (cache.values_q, self.values_q, self._cb),
                                 (cache.key_norms, self.key_norms, 2), (cache.value_norms, self.value_norms, 2)):
            batch.blit_copy(src, 0, dst, lane_row0 * stride, rows * stride)

    def reset(self) -> None:
        """quant_unified_pool.rs:318-328: a zero norm annihilates whatever the codes say."""
        for b in (self.keys_q, self.values_q, self.key_norms, self.value_norms):
            b.fill_zero()

    def reset_lane(self, lane: int) -> None:
        """quant_unified_pool.rs:331-345."""
        if lane >= self.n_lanes:
            return
        rows = self.lane_stride() * self.n_kv_heads
        for b, stride in ((self.keys_q, self._cb), (self.values_q, self._cb), (self.key_norms, 2),
                          (self.value_norms, 2)):
            b.view(lane * rows * stride, rows * stride).fill_zero()
