"""local-hip: gfx950 (MI355X) decode hot path behind local-metal's kernel-dispatch API.

This package is a thin ctypes mirror of the reference's host-side interface
(``local_metal::{context::MetalContext, buffer::MetalBuffer,
batch::CommandBatch, kernels::Kernels, error::Error}``) on top of the C ABI in
``include/local_hip.h``.  All compute happens in ``liblocal_hip.so`` (hand-written
HIP kernels); there is no CPU or PyTorch fallback -- if the library is missing or
no gfx950 device is present the calls raise.

The directory name carries a hyphen, so load it with ``__graft_entry__.load_package()``
(registers it as ``local_ai_amd``) or ``importlib`` rather than a plain import.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liblocal_hip.so")

F16, F32, BF16 = 0, 1, 2
Q4_0, TQ2_0 = 0, 1
ROWS_F16 = 2          # lh_dequant_rows_into: a table of plain f16 rows
_DTYPE_SIZE = {F16: 2, F32: 4, BF16: 2}

SMALLM_MAX_M = 8      # local-metal/src/kernels.rs:6155
BATCHM_MAX_M = 4      # local-metal/src/kernels.rs:6160
MULTIVEC_MAX_M = 16   # local-metal/src/kernels.rs:6362


class Error(Exception):
    """Mirror of ``local_metal::Error`` (local-metal/src/error.rs:1-32)."""
    code = -1


class NoDevice(Error):
    code = 1


class NoCommandQueue(Error):
    code = 2


class BufferAllocation(Error):
    code = 3


class LibraryCreation(Error):
    code = 4


class PipelineCreation(Error):
    code = 5


class ShaderNotFound(Error):
    code = 6


class CommandBuffer(Error):
    code = 7


class InvalidArgument(Error):
    code = 8


class Io(Error):
    code = 9


_ERRORS = {c.code: c for c in (NoDevice, NoCommandQueue, BufferAllocation, LibraryCreation, PipelineCreation,
                               ShaderNotFound, CommandBuffer, InvalidArgument, Io)}

_lib = None


def lib() -> C.CDLL:
    """Load ``liblocal_hip.so``; raises ``LibraryCreation`` when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryCreation(f"{LIB_PATH} is missing: run __graft_entry__.build() (make -C local-ai_amd/csrc)")
        _lib = C.CDLL(LIB_PATH)
        _lib.lh_last_error.restype = C.c_char_p
        _lib.lh_version.restype = C.c_char_p
        _lib.lh_buffer_length.restype = C.c_size_t
        _lib.lh_buffer_device_ptr.restype = C.c_void_p
        _lib.lh_context_stream.restype = C.c_void_p
        for name in ("lh_smallm_max_m", "lh_batchm_max_m", "lh_multivec_max_m", "lh_batch_dispatch_count",
                     "lh_flash_split_count"):
            getattr(_lib, name).restype = C.c_uint32
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        msg = lib().lh_last_error().decode("utf-8", "replace")
        raise _ERRORS.get(rc, Error)(msg)


def _u32(v) -> C.c_uint32:
    return C.c_uint32(int(v))


class Context:
    """``MetalContext`` (local-metal/src/context.rs:31-98): device + one in-order stream."""

    def __init__(self, device_index: int = 0):
        self._h = C.c_void_p()
        _check(lib().lh_context_create(C.c_int(device_index), C.byref(self._h)))

    def device_name(self) -> str:
        buf = C.create_string_buffer(256)
        _check(lib().lh_context_device_name(self._h, buf, C.c_size_t(256)))
        return buf.value.decode()

    def compute_units(self) -> int:
        return int(lib().lh_context_compute_units(self._h))

    def stream(self) -> int:
        return int(lib().lh_context_stream(self._h) or 0)

    def synchronize(self) -> None:
        _check(lib().lh_context_synchronize(self._h))

    def close(self) -> None:
        if self._h:
            lib().lh_context_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Event:
    """HIP event on the context stream (device-side timing)."""

    def __init__(self, ctx: Context):
        self._h = C.c_void_p()
        _check(lib().lh_event_create(ctx._h, C.byref(self._h)))

    def record(self) -> None:
        _check(lib().lh_event_record(self._h))

    def elapsed_ms(self, stop: "Event") -> float:
        ms = C.c_float()
        _check(lib().lh_event_elapsed_ms(self._h, stop._h, C.byref(ms)))
        return float(ms.value)

    def __del__(self):
        try:
            if self._h:
                lib().lh_event_destroy(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass


class Buffer:
    """``MetalBuffer`` (local-metal/src/buffer.rs:17-141) in device memory.

    Host access is an explicit copy (``as_array`` / ``copy_from_bytes``), ordered
    after the work already enqueued on the context.
    """

    def __init__(self, handle, ctx, parent=None):
        self._h = handle
        self.ctx = ctx
        self._parent = parent  # keeps the owner of a view alive

    @classmethod
    def from_slice(cls, ctx: Context, data) -> "Buffer":
        a = np.ascontiguousarray(data)
        h = C.c_void_p()
        _check(lib().lh_buffer_from_bytes(ctx._h, C.c_void_p(a.ctypes.data), C.c_size_t(a.nbytes), C.byref(h)))
        return cls(h, ctx)

    @classmethod
    def empty(cls, ctx: Context, byte_len: int) -> "Buffer":
        h = C.c_void_p()
        _check(lib().lh_buffer_empty(ctx._h, C.c_size_t(byte_len), C.byref(h)))
        return cls(h, ctx)

    @classmethod
    def wrap(cls, ctx: Context, device_ptr: int, byte_len: int, owner=None) -> "Buffer":
        """Non-owning handle over device memory allocated elsewhere (e.g. a torch tensor)."""
        h = C.c_void_p()
        _check(lib().lh_buffer_wrap(ctx._h, C.c_void_p(device_ptr), C.c_size_t(byte_len), C.byref(h)))
        return cls(h, ctx, parent=owner)

    def view(self, offset: int, byte_len: int) -> "Buffer":
        h = C.c_void_p()
        _check(lib().lh_buffer_view(self._h, C.c_size_t(offset), C.c_size_t(byte_len), C.byref(h)))
        return Buffer(h, self.ctx, parent=self)

    def length(self) -> int:
        return int(lib().lh_buffer_length(self._h))

    def device_ptr(self) -> int:
        return int(lib().lh_buffer_device_ptr(self._h) or 0)

    def copy_from_bytes(self, src, offset: int = 0) -> None:
        a = np.ascontiguousarray(src)
        _check(lib().lh_buffer_write(self._h, C.c_size_t(offset), C.c_void_p(a.ctypes.data), C.c_size_t(a.nbytes)))

    def as_array(self, dtype, count: int | None = None, offset: int = 0) -> np.ndarray:
        dt = np.dtype(dtype)
        if count is None:
            count = (self.length() - offset) // dt.itemsize
        out = np.empty(count, dt)
        _check(lib().lh_buffer_read(self._h, C.c_size_t(offset), C.c_void_p(out.ctypes.data), C.c_size_t(out.nbytes)))
        return out

    def fill_zero(self) -> None:
        _check(lib().lh_buffer_fill_zero(self._h))

    def free(self) -> None:
        if self._h:
            lib().lh_buffer_free(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class CommandBatch:
    """``CommandBatch`` (local-metal/src/batch.rs:21-291): dispatches run in encode order."""

    def __init__(self, ctx: Context):
        self.ctx = ctx
        self._h = C.c_void_p()
        _check(lib().lh_batch_new(ctx._h, C.byref(self._h)))

    def dispatch_count(self) -> int:
        return int(lib().lh_batch_dispatch_count(self._h))

    def blit_copy(self, src: Buffer, src_offset: int, dst: Buffer, dst_offset: int, length: int) -> None:
        _check(lib().lh_batch_blit_copy(self._h, src._h, C.c_size_t(src_offset), dst._h, C.c_size_t(dst_offset),
                                        C.c_size_t(length)))

    def commit_and_wait(self) -> None:
        _check(lib().lh_batch_commit_and_wait(self._h))

    def submit_and_renew(self) -> None:
        _check(lib().lh_batch_submit_and_renew(self._h))

    def commit_and_renew(self) -> None:
        _check(lib().lh_batch_commit_and_renew(self._h))

    def begin_capture(self) -> None:
        """Record the following ``*_into`` calls into a graph instead of running them."""
        _check(lib().lh_batch_begin_capture(self._h))

    def end_capture(self) -> "Graph":
        h = C.c_void_p()
        _check(lib().lh_batch_end_capture(self._h, C.byref(h)))
        return Graph(h, self.ctx)

    def __del__(self):
        try:
            if self._h:
                lib().lh_batch_free(self._h)
                self._h = C.c_void_p()
        except Exception:
            pass


class Graph:
    """A recorded batch: ``launch()`` enqueues one replay of every dispatch captured between
    ``CommandBatch.begin_capture`` and ``end_capture``."""

    def __init__(self, handle, ctx):
        self._h, self.ctx = handle, ctx

    def launch(self) -> None:
        _check(lib().lh_graph_launch(self._h))

    def dispatch_count(self) -> int:
        lib().lh_graph_dispatch_count.restype = C.c_uint32
        return int(lib().lh_graph_dispatch_count(self._h))

    def free(self) -> None:
        if self._h:
            lib().lh_graph_free(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _handles(bufs):
    arr = (C.c_void_p * len(bufs))(*[b._h for b in bufs])
    return arr


class Kernels:
    """``Kernels`` (local-metal/src/kernels.rs): one method per hot-path dispatch, same
    names and argument order.  ``*_into`` methods encode into a batch; the others block."""

    SMALLM_MAX_M = SMALLM_MAX_M
    BATCHM_MAX_M = BATCHM_MAX_M
    MULTIVEC_MAX_M = MULTIVEC_MAX_M

    def __init__(self, ctx: Context):
        self.ctx = ctx
        self._l = lib()

    # -- flags (kernels.rs:6277-6304) --
    @staticmethod
    def batchm_enabled() -> bool:
        return bool(lib().lh_batchm_enabled())

    @staticmethod
    def mma_enabled() -> bool:
        return bool(lib().lh_mma_enabled())

    @staticmethod
    def smallm_enabled() -> bool:
        return bool(lib().lh_smallm_enabled())

    # -- M = 1 matvec (kernels.rs:5711-6038) --
    def matvec_q4_0(self, ctx, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_q4_0(ctx._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_q4_0_into(self, batch, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_q4_0_into(batch._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_q4_0_f32out(self, ctx, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_q4_0_f32out(ctx._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_q4_0_f32out_into(self, batch, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_q4_0_f32out_into(batch._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_tq2_0(self, ctx, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_tq2_0(ctx._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_tq2_0_into(self, batch, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_tq2_0_into(batch._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_tq2_0_f32out(self, ctx, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_tq2_0_f32out(ctx._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_tq2_0_f32out_into(self, batch, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec_tq2_0_f32out_into(batch._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_tq2_0_soa_into(self, batch, qs, scales, vector, output, rows, cols):
        _check(self._l.lh_matvec_tq2_0_soa_into(batch._h, qs._h, scales._h, vector._h, output._h, _u32(rows),
                                                _u32(cols)))

    def matvec_quant_typed_into(self, batch, fmt, matrix, vector, vector_dtype, output, output_dtype, rows, cols):
        _check(self._l.lh_matvec_quant_typed_into(batch._h, C.c_int(fmt), matrix._h, vector._h, C.c_int(vector_dtype),
                                                  output._h, C.c_int(output_dtype), _u32(rows), _u32(cols)))

    def matvec_quant_grouped_into(self, batch, fmt, matrices, vectors, vector_dtype, outputs, output_dtype, rows,
                                  cols):
        n = len(matrices)
        assert len(vectors) == n and len(outputs) == n
        _check(self._l.lh_matvec_quant_grouped_into(batch._h, C.c_int(fmt), _u32(n), _handles(matrices),
                                                    _handles(vectors), C.c_int(vector_dtype), _handles(outputs),
                                                    C.c_int(output_dtype), _u32(rows), _u32(cols)))

    PROLOGUE_RMS_NORM, PROLOGUE_GELU_MUL = 1, 2

    def matvec_quant_fused_into(self, batch, fmt, matrices, vector, prologue, aux, eps, outputs, rows, cols):
        """1..8 matvecs of one shape against one f16 vector transformed while it is staged: rms_norm(vector) * aux
        (PROLOGUE_RMS_NORM) or gelu(vector) * aux (PROLOGUE_GELU_MUL), rounded to f16 as the separate kernel would."""
        n = len(matrices)
        assert len(outputs) == n
        _check(self._l.lh_matvec_quant_fused_into(batch._h, C.c_int(fmt), _u32(n), _handles(matrices), vector._h,
                                                  C.c_int(prologue), aux._h, C.c_float(eps), _handles(outputs),
                                                  _u32(rows), _u32(cols)))

    def matvec_quant_norm_chain_into(self, batch, fmt, matrices, vector, weight, residual, next_weight, store, eps, outputs,
                                     rows, cols):
        """Matvecs against t = rms_norm(vector) * weight + residual (as rms_norm_add_into rounds it), or against
        rms_norm(t) * next_weight when that is given; `store` receives t.  `residual`, `next_weight`, `store` may be None."""
        def h(b):
            return b._h if b is not None else None
        _check(self._l.lh_matvec_quant_norm_chain_into(batch._h, C.c_int(fmt), _u32(len(matrices)), _handles(matrices),
                                                       vector._h, weight._h, h(residual), h(next_weight), h(store),
                                                       C.c_float(eps), _handles(outputs), _u32(rows), _u32(cols)))

    def matvec_quant_norm_chain_tail_into(self, batch, fmt, matrices, vector, weight, residual, scale, next_weight, store, eps,
                                          outputs, rows, cols):
        """Matvecs against the next layer's attention norm of t = (rms_norm(vector) * weight + residual) * scale, rounded as
        rms_norm_residual_scale_into rounds it (`scale` None: no scale step); `store` receives t (the layer output)."""
        _check(self._l.lh_matvec_quant_norm_chain_tail_into(
            batch._h, C.c_int(fmt), _u32(len(matrices)), _handles(matrices), vector._h, weight._h, residual._h,
            C.c_int(0 if scale is None else 1), C.c_float(1.0 if scale is None else scale),
            next_weight._h if next_weight is not None else None, store._h, C.c_float(eps), _handles(outputs), _u32(rows),
            _u32(cols)))

    def matvec_quant_rotated_into(self, batch, fmt, matrix, vector, signs, head_dim, output, rows, cols):
        """hadamard_rotate_fh_into(vector, signs, post-sign) followed by the matvec, in one dispatch: `vector` holds the
        attention kernel's f32 head outputs, the rotation back out of code space happens while it is staged."""
        _check(self._l.lh_matvec_quant_rotated_into(batch._h, C.c_int(fmt), matrix._h, vector._h, signs._h, _u32(head_dim),
                                                    output._h, _u32(rows), _u32(cols)))

    # -- small-M / prefill matmul (kernels.rs:6378-6563, 5517-5568) --
    def matmul_nt_q4_0_into(self, batch, input, weight, output, m, k, n):
        _check(self._l.lh_matmul_nt_q4_0_into(batch._h, input._h, weight._h, output._h, _u32(m), _u32(k), _u32(n)))

    def matmul_nt_tq2_0_into(self, batch, input, weight, output, m, k, n):
        _check(self._l.lh_matmul_nt_tq2_0_into(batch._h, input._h, weight._h, output._h, _u32(m), _u32(k), _u32(n)))

    def multivec_nt_q4_0_into(self, batch, input, weight, output, m, k, n):
        _check(self._l.lh_multivec_nt_q4_0_into(batch._h, input._h, weight._h, output._h, _u32(m), _u32(k), _u32(n)))

    def multivec_nt_tq2_0_into(self, batch, input, weight, output, m, k, n):
        _check(self._l.lh_multivec_nt_tq2_0_into(batch._h, input._h, weight._h, output._h, _u32(m), _u32(k), _u32(n)))

    def matmul_nt_quant_typed_into(self, batch, fmt, input, input_dtype, weight, output, output_dtype, m, k, n):
        _check(self._l.lh_matmul_nt_quant_typed_into(batch._h, C.c_int(fmt), input._h, C.c_int(input_dtype),
                                                     weight._h, output._h, C.c_int(output_dtype), _u32(m), _u32(k),
                                                     _u32(n)))

    def matmul_nt_quant_grouped_into(self, batch, fmt, input, weights, outputs, m, k, ns):
        """Up to four matrices of one format against the same activations in one launch; output i is [m, ns[i]] f16."""
        n = len(weights)
        assert len(outputs) == n and len(ns) == n
        _check(self._l.lh_matmul_nt_quant_grouped_into(batch._h, C.c_int(fmt), _u32(n), input._h, _handles(weights),
                                                       _handles(outputs), (C.c_uint32 * n)(*[int(v) for v in ns]),
                                                       _u32(m), _u32(k)))

    def matmul_nt_quant_gelu_mul_strided_into(self, batch, fmt, input, weight, m, k, n, gate_rows, row_stride, row_offset, output):
        """output[r, i] = gelu((input . weight^T)[r, i]) * gate_rows[r * row_stride + row_offset + i]: the per-layer-input
        gate (product, slice gather, gelu_mul) as one step."""
        _check(self._l.lh_matmul_nt_quant_gelu_mul_strided_into(batch._h, C.c_int(fmt), input._h, weight._h, _u32(m), _u32(k),
                                                                _u32(n), gate_rows._h, _u32(row_stride), _u32(row_offset),
                                                                output._h))

    def matmul_nt_quant_gelu_mul_into(self, batch, fmt, input, w_gate, w_up, output, m, k, n):
        """output[m, n] = gelu(input . w_gate^T) * (input . w_up^T): the two feed-forward products and gelu_mul as one step."""
        _check(self._l.lh_matmul_nt_quant_gelu_mul_into(batch._h, C.c_int(fmt), input._h, w_gate._h, w_up._h, output._h,
                                                        _u32(m), _u32(k), _u32(n)))

    def matmul_nt_quant_norm_into(self, batch, fmt, input, weight, m, k, n, norm_weight, residual, output, eps, scale=None,
                                  norm2_weight=None, output2=None):
        """matmul_nt -> rms_norm(_add) (-> scale_in_place) (-> rms_norm) of the multi-row layer paths as one step, bit for
        bit the separate kernels' result; `residual`, `scale`, `norm2_weight` / `output2` are optional."""
        _check(self._l.lh_matmul_nt_quant_norm_into(batch._h, C.c_int(fmt), input._h, weight._h, _u32(m), _u32(k), _u32(n),
                                                    norm_weight._h, residual._h if residual is not None else None, output._h,
                                                    C.c_float(eps), C.c_int(0 if scale is None else 1),
                                                    C.c_float(0.0 if scale is None else scale),
                                                    norm2_weight._h if norm2_weight is not None else None,
                                                    output2._h if output2 is not None else None))

    def matmul_nt_into(self, batch, input, weight, output, m, k, n):
        _check(self._l.lh_matmul_nt_into(batch._h, input._h, weight._h, output._h, _u32(m), _u32(k), _u32(n)))

    def clipped_linear_tiled_nt_into(self, batch, input, weight, bias, output, m, k, n, input_min, input_max,
                                     output_min, output_max):
        """kernels.rs:3244-3330: clamp(clamp(x) @ W^T + bias); `bias` may be None."""
        _check(self._l.lh_clipped_linear_tiled_nt_into(batch._h, input._h, weight._h, bias._h if bias is not None else None,
                                                       output._h, _u32(m), _u32(k), _u32(n), C.c_float(input_min),
                                                       C.c_float(input_max), C.c_float(output_min), C.c_float(output_max)))

    # -- FP16-weight matvec family (kernels.rs:582, 1710-1930) --
    def matvec(self, ctx, matrix, vector, output, rows, cols):
        _check(self._l.lh_matvec(ctx._h, matrix._h, vector._h, output._h, _u32(rows), _u32(cols)))

    def matvec_offset_into(self, batch, matrix, matrix_offset, vector, output, rows, cols):
        _check(self._l.lh_matvec_offset_into(batch._h, matrix._h, C.c_size_t(matrix_offset), vector._h, output._h, _u32(rows),
                                             _u32(cols)))

    def matvec_f32out_offset(self, ctx, matrix, matrix_offset, vector, output, rows, cols):
        _check(self._l.lh_matvec_f32out_offset(ctx._h, matrix._h, C.c_size_t(matrix_offset), vector._h, output._h, _u32(rows),
                                               _u32(cols)))

    def matvec_f32out_offset_into(self, batch, matrix, matrix_offset, vector, output, rows, cols):
        _check(self._l.lh_matvec_f32out_offset_into(batch._h, matrix._h, C.c_size_t(matrix_offset), vector._h, output._h,
                                                    _u32(rows), _u32(cols)))

    def matvec_f32in_offset(self, ctx, matrix, matrix_offset, vector, output, rows, cols):
        _check(self._l.lh_matvec_f32in_offset(ctx._h, matrix._h, C.c_size_t(matrix_offset), vector._h, output._h, _u32(rows),
                                              _u32(cols)))

    def matvec_f32in_offset_into(self, batch, matrix, matrix_offset, vector, output, rows, cols):
        _check(self._l.lh_matvec_f32in_offset_into(batch._h, matrix._h, C.c_size_t(matrix_offset), vector._h, output._h,
                                                   _u32(rows), _u32(cols)))

    # -- decoder-layer glue (kernels.rs:509, 2142-2392, 2592-2890, 6648-6673) --
    def rms_norm_into(self, batch, input, weight, output, dim, rows, eps):
        _check(self._l.lh_rms_norm_into(batch._h, input._h, weight._h, output._h, _u32(dim), _u32(rows), C.c_float(eps)))

    def rms_norm_add_into(self, batch, input, weight, residual, output, dim, rows, eps):
        _check(self._l.lh_rms_norm_add_into(batch._h, input._h, weight._h, residual._h, output._h, _u32(dim), _u32(rows),
                                            C.c_float(eps)))

    def rms_norm_residual_scale_into(self, batch, input, weight, residual, output, dim, rows, eps, scale=None):
        """rms_norm_into + residual_add_into (+ scale_in_place_gpu_into when `scale` is given) in one dispatch, with the
        f16 rounding after each step that the separate kernels apply."""
        _check(self._l.lh_rms_norm_residual_scale_into(batch._h, input._h, weight._h, residual._h, output._h, _u32(dim),
                                                       _u32(rows), C.c_float(eps), C.c_int(scale is not None),
                                                       C.c_float(scale if scale is not None else 1.0)))

    def qk_norm_gpu_into(self, batch, qk_data, weight, head_dim, num_heads, eps):
        _check(self._l.lh_qk_norm_gpu_into(batch._h, qk_data._h, weight._h, _u32(head_dim), _u32(num_heads), C.c_float(eps)))

    def qk_norm_offset_into(self, batch, qk_data, weight, weight_offset, head_dim, num_heads, eps):
        _check(self._l.lh_qk_norm_offset_into(batch._h, qk_data._h, weight._h, C.c_size_t(weight_offset), _u32(head_dim),
                                              _u32(num_heads), C.c_float(eps)))

    def qk_norm_rope_available(self, head_dim):
        return bool(self._l.lh_qk_norm_rope_available(_u32(head_dim)))

    def qk_norm_rope_into(self, batch, input, output, weight, head_dim, num_heads, eps, position, theta,
                          partial_rotary_factor):
        _check(self._l.lh_qk_norm_rope_into(batch._h, input._h, output._h, weight._h, _u32(head_dim), _u32(num_heads),
                                            C.c_float(eps), _u32(position), C.c_float(theta),
                                            C.c_float(partial_rotary_factor)))

    def rope_into(self, batch, input, output, head_dim, position, theta, partial_rotary_factor, num_heads):
        _check(self._l.lh_rope_into(batch._h, input._h, output._h, _u32(head_dim), _u32(position), C.c_float(theta),
                                    C.c_float(partial_rotary_factor), _u32(num_heads)))

    def rope_batch_into(self, batch, qk, start_pos, theta, head_dim, num_heads, seq_len, partial_rotary_factor):
        _check(self._l.lh_rope_batch_into(batch._h, qk._h, _u32(start_pos), C.c_float(theta), _u32(head_dim), _u32(num_heads),
                                          _u32(seq_len), C.c_float(partial_rotary_factor)))

    def rope_batch_decode_into(self, batch, qk, positions, theta, head_dim, num_heads, seq_len, partial_rotary_factor):
        _check(self._l.lh_rope_batch_decode_into(batch._h, qk._h, positions._h, C.c_float(theta), _u32(head_dim), _u32(num_heads),
                                                 _u32(seq_len), C.c_float(partial_rotary_factor)))

    def gelu_mul_into(self, batch, a, b, out, count):
        _check(self._l.lh_gelu_mul_into(batch._h, a._h, b._h, out._h, _u32(count)))

    def residual_add_into(self, batch, a, b, output, count):
        _check(self._l.lh_residual_add_into(batch._h, a._h, b._h, output._h, _u32(count)))

    def scale_in_place_gpu_into(self, batch, data, scalar, count):
        _check(self._l.lh_scale_in_place_gpu_into(batch._h, data._h, C.c_float(scalar), _u32(count)))

    def gather_strided_f16_into(self, batch, src, dst, row_stride, base_off, pld, n_rows):
        _check(self._l.lh_gather_strided_f16_into(batch._h, src._h, dst._h, _u32(row_stride), _u32(base_off), _u32(pld),
                                                  _u32(n_rows)))

    def gelu_mul_strided_into(self, batch, a, b, b_row_stride, b_offset, out, dim, rows):
        """gather_strided_f16 + gelu_mul in one dispatch: out[r, i] = gelu(a[r, i]) * b[r * b_row_stride + b_offset + i]."""
        _check(self._l.lh_gelu_mul_strided_into(batch._h, a._h, b._h, _u32(b_row_stride), _u32(b_offset), out._h, _u32(dim),
                                                _u32(rows)))

    def logit_softcap_gpu_into(self, batch, data, cap, count):
        _check(self._l.lh_logit_softcap_gpu_into(batch._h, data._h, C.c_float(cap), _u32(count)))

    # -- block dequant (qat_recover.rs:23-97) and legacy unpack (kernels.rs:6753-6802) --
    def dequant_q4_0_into(self, batch, data, byte_offset, output, num_elements):
        _check(self._l.lh_dequant_q4_0_into(batch._h, data._h, C.c_size_t(byte_offset), output._h,
                                            C.c_size_t(num_elements)))

    def dequant_tq2_0_into(self, batch, data, byte_offset, output, num_elements):
        _check(self._l.lh_dequant_tq2_0_into(batch._h, data._h, C.c_size_t(byte_offset), output._h,
                                             C.c_size_t(num_elements)))

    def dequant_rows_into(self, batch, fmt, table, table_rows, cols, rows, n_rows, output, scale=1.0):
        """Rows `rows[0 .. n_rows)` (device u32 indices, clamped to the last row) of a packed table as a dense f16
        [n_rows, cols] matrix; `fmt` is Q4_0, TQ2_0 or ROWS_F16."""
        _check(self._l.lh_dequant_rows_into(batch._h, C.c_int(fmt), table._h, _u32(table_rows), _u32(cols), rows._h,
                                            _u32(n_rows), C.c_float(scale), output._h))

    def tq2_dequant(self, ctx, packed, scales, output, num_elements):
        _check(self._l.lh_tq2_dequant(ctx._h, packed._h, scales._h, output._h, _u32(num_elements)))

    # -- TurboQuant KV (kernels.rs:4641-5506) --
    def encode_kv_turboquant(self, ctx, input, levels, signs, packed, norms, head_dim, n_kv_heads, num_tokens, bits,
                             position, ring_capacity):
        _check(self._l.lh_encode_kv_turboquant(ctx._h, input._h, levels._h, signs._h, packed._h, norms._h,
                                               _u32(head_dim), _u32(n_kv_heads), _u32(num_tokens), _u32(bits),
                                               _u32(position), _u32(ring_capacity)))

    def encode_kv_turboquant_into(self, batch, input, levels, signs, packed, norms, head_dim, n_kv_heads, num_tokens,
                                  bits, position, ring_capacity):
        _check(self._l.lh_encode_kv_turboquant_into(batch._h, input._h, levels._h, signs._h, packed._h, norms._h,
                                                    _u32(head_dim), _u32(n_kv_heads), _u32(num_tokens), _u32(bits),
                                                    _u32(position), _u32(ring_capacity)))

    def encode_kv_turboquant_batched_into(self, batch, input, levels, signs, packed, norms, positions, head_dim,
                                          n_kv_heads, lane_capacity, bits, n_lanes, ring_capacity):
        _check(self._l.lh_encode_kv_turboquant_batched_into(batch._h, input._h, levels._h, signs._h, packed._h,
                                                            norms._h, positions._h, _u32(head_dim), _u32(n_kv_heads),
                                                            _u32(lane_capacity), _u32(bits), _u32(n_lanes),
                                                            _u32(ring_capacity)))

    def dequantize_kv_turboquant(self, ctx, packed, norms, levels, signs, output, head_dim, n_kv_heads, num_tokens,
                                 bits, token_start, ring_capacity):
        _check(self._l.lh_dequantize_kv_turboquant(ctx._h, packed._h, norms._h, levels._h, signs._h, output._h,
                                                   _u32(head_dim), _u32(n_kv_heads), _u32(num_tokens), _u32(bits),
                                                   _u32(token_start), _u32(ring_capacity)))

    def dequantize_kv_turboquant_into(self, batch, packed, norms, levels, signs, output, head_dim, n_kv_heads,
                                      num_tokens, bits, token_start, ring_capacity):
        _check(self._l.lh_dequantize_kv_turboquant_into(batch._h, packed._h, norms._h, levels._h, signs._h, output._h,
                                                        _u32(head_dim), _u32(n_kv_heads), _u32(num_tokens), _u32(bits),
                                                        _u32(token_start), _u32(ring_capacity)))

    def decode_qkv_prepare_into(self, batch, q, k, v, q_norm, k_norm, levels, signs, rq, k_codes, k_norms, v_codes, v_norms,
                                head_dim, n_q_heads, n_kv_heads, eps, position, theta, partial_rotary_factor, bits,
                                ring_capacity):
        """Head norms, RoPE, unit-weight V norm, both KV encodes and the query rotation of one decoded token in one
        dispatch; k = v = None prepares the query only (a layer reading another layer's cache)."""
        def h(b):
            return b._h if b is not None else None
        _check(self._l.lh_decode_qkv_prepare_into(batch._h, q._h, h(k), h(v), h(q_norm), h(k_norm), levels._h, signs._h, rq._h,
                                                  h(k_codes), h(k_norms), h(v_codes), h(v_norms), _u32(head_dim),
                                                  _u32(n_q_heads), _u32(n_kv_heads), C.c_float(eps), _u32(position),
                                                  C.c_float(theta), C.c_float(partial_rotary_factor), _u32(bits),
                                                  _u32(ring_capacity)))

    def decode_qkv_prepare_rows_into(self, batch, q, k, v, q_norm, k_norm, levels, signs, rq, k_codes, k_norms, v_codes,
                                     v_norms, positions, head_dim, n_q_heads, n_kv_heads, rows, eps, start_position, theta,
                                     partial_rotary_factor, bits, ring_capacity, lane_capacity):
        """decode_qkv_prepare_into for `rows` tokens: consecutive positions of one sequence from `start_position`
        (positions None, lane_capacity 0), or one token per lane at the device table `positions`."""
        def h(b):
            return b._h if b is not None else None
        _check(self._l.lh_decode_qkv_prepare_rows_into(batch._h, q._h, h(k), h(v), h(q_norm), h(k_norm), levels._h, signs._h,
                                                       rq._h, h(k_codes), h(k_norms), h(v_codes), h(v_norms), h(positions),
                                                       _u32(head_dim), _u32(n_q_heads), _u32(n_kv_heads), _u32(rows),
                                                       C.c_float(eps), _u32(start_position), C.c_float(theta),
                                                       C.c_float(partial_rotary_factor), _u32(bits), _u32(ring_capacity),
                                                       _u32(lane_capacity)))

    def matmul_nt_qkv_prepare_rows_into(self, batch, weight_type, input, w_q, w_k, w_v, k_dim, q, k, v, q_norm, k_norm, levels,
                                        signs, rq, k_codes, k_norms, v_codes, v_norms, positions, head_dim, n_q_heads,
                                        n_kv_heads, rows, eps, start_position, theta, partial_rotary_factor, bits,
                                        ring_capacity, lane_capacity):
        """The grouped Q / K / V product and decode_qkv_prepare_rows_into on its outputs; the preparation sums the
        product's k-split tiles itself where the product leaves them (same results bit for bit)."""
        def h(b):
            return b._h if b is not None else None
        _check(self._l.lh_matmul_nt_qkv_prepare_rows_into(batch._h, C.c_int(weight_type), input._h, w_q._h, w_k._h, w_v._h,
                                                          _u32(k_dim), q._h, k._h, v._h, h(q_norm), h(k_norm), levels._h,
                                                          signs._h, rq._h, k_codes._h, k_norms._h, v_codes._h, v_norms._h,
                                                          h(positions), _u32(head_dim), _u32(n_q_heads), _u32(n_kv_heads),
                                                          _u32(rows), C.c_float(eps), _u32(start_position), C.c_float(theta),
                                                          C.c_float(partial_rotary_factor), _u32(bits), _u32(ring_capacity),
                                                          _u32(lane_capacity)))

    def hadamard_rotate_into(self, batch, input, signs, output, head_dim, num_heads, pre_sign, post_sign):
        _check(self._l.lh_hadamard_rotate_into(batch._h, input._h, signs._h, output._h, _u32(head_dim),
                                               _u32(num_heads), C.c_int(bool(pre_sign)), C.c_int(bool(post_sign))))

    def hadamard_rotate_hf_into(self, batch, input, signs, output, head_dim, num_heads, pre_sign, post_sign):
        _check(self._l.lh_hadamard_rotate_hf_into(batch._h, input._h, signs._h, output._h, _u32(head_dim),
                                                  _u32(num_heads), C.c_int(bool(pre_sign)), C.c_int(bool(post_sign))))

    def hadamard_rotate_fh_into(self, batch, input, signs, output, head_dim, num_heads, pre_sign, post_sign):
        _check(self._l.lh_hadamard_rotate_fh_into(batch._h, input._h, signs._h, output._h, _u32(head_dim),
                                                  _u32(num_heads), C.c_int(bool(pre_sign)), C.c_int(bool(post_sign))))

    def flash_attention_tq_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, head_dim, kv_len,
                                current_pos, num_q_heads, num_kv_heads, window, bits, ring_capacity):
        _check(self._l.lh_flash_attention_tq_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h, v_norms._h,
                                                  levels._h, out._h, _u32(head_dim), _u32(kv_len), _u32(current_pos),
                                                  _u32(num_q_heads), _u32(num_kv_heads), _u32(window), _u32(bits),
                                                  _u32(ring_capacity)))

    def flash_attention_tq_static_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, head_dim, kv_len,
                                       current_pos, num_q_heads, num_kv_heads, window, bits, ring_capacity):
        """flash_attention_tq_into for callers that may not allocate: the split partials live in a static device array."""
        _check(self._l.lh_flash_attention_tq_static_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h, v_norms._h,
                                                         levels._h, out._h, _u32(head_dim), _u32(kv_len), _u32(current_pos),
                                                         _u32(num_q_heads), _u32(num_kv_heads), _u32(window), _u32(bits),
                                                         _u32(ring_capacity)))

    def flash_attention_tq_prefill_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, head_dim,
                                        kv_len, start_pos, n_rows, num_q_heads, num_kv_heads, window, bits,
                                        ring_capacity):
        _check(self._l.lh_flash_attention_tq_prefill_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h,
                                                          v_norms._h, levels._h, out._h, _u32(head_dim), _u32(kv_len),
                                                          _u32(start_pos), _u32(n_rows), _u32(num_q_heads),
                                                          _u32(num_kv_heads), _u32(window), _u32(bits),
                                                          _u32(ring_capacity)))

    def flash_attention_tq_prefill_tiled_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out,
                                              head_dim, kv_len, start_pos, n_rows, num_q_heads, num_kv_heads, window,
                                              bits, ring_capacity):
        _check(self._l.lh_flash_attention_tq_prefill_tiled_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h,
                                                                v_norms._h, levels._h, out._h, _u32(head_dim),
                                                                _u32(kv_len), _u32(start_pos), _u32(n_rows),
                                                                _u32(num_q_heads), _u32(num_kv_heads), _u32(window),
                                                                _u32(bits), _u32(ring_capacity)))

    def flash_attention_tq_batched_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, positions,
                                        head_dim, lane_capacity, num_q_heads, num_kv_heads, window, bits, n_lanes,
                                        ring_capacity):
        _check(self._l.lh_flash_attention_tq_batched_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h,
                                                          v_norms._h, levels._h, out._h, positions._h, _u32(head_dim),
                                                          _u32(lane_capacity), _u32(num_q_heads), _u32(num_kv_heads),
                                                          _u32(window), _u32(bits), _u32(n_lanes),
                                                          _u32(ring_capacity)))

    def flash_attention_tq_rotated_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, signs, out, out_f16,
                                        head_dim, kv_len, current_pos, num_q_heads, num_kv_heads, window, bits,
                                        ring_capacity):
        """``flash_attention_tq_into`` into the f32 scratch ``out``, then the rotation back out of code space
        (``hadamard_rotate_fh_into`` with the post-sign) into ``out_f16``, as one call."""
        _check(self._l.lh_flash_attention_tq_rotated_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h,
                                                          v_norms._h, levels._h, signs._h, out._h, out_f16._h,
                                                          _u32(head_dim), _u32(kv_len), _u32(current_pos),
                                                          _u32(num_q_heads), _u32(num_kv_heads), _u32(window),
                                                          _u32(bits), _u32(ring_capacity)))

    def flash_attention_tq_rotated_lazy_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, signs, out, out_f16,
                                             head_dim, kv_len, current_pos, num_q_heads, num_kv_heads, window, bits,
                                             ring_capacity) -> bool:
        """``flash_attention_tq_rotated_into`` that rotates only where the rotation rides in the merge launch.  True:
        ``out_f16`` holds the rotated heads.  False: the f32 heads in ``out`` are still in code space and the caller's
        next kernel rotates them (``matvec_quant_rotated_into``)."""
        rotated = C.c_int(0)
        _check(self._l.lh_flash_attention_tq_rotated_lazy_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h,
                                                               v_norms._h, levels._h, signs._h, out._h, out_f16._h,
                                                               _u32(head_dim), _u32(kv_len), _u32(current_pos),
                                                               _u32(num_q_heads), _u32(num_kv_heads), _u32(window),
                                                               _u32(bits), _u32(ring_capacity), C.byref(rotated)))
        return bool(rotated.value)

    def flash_attention_tq_batched_rotated_into(self, batch, rq, k_codes, k_norms, v_codes, v_norms, levels, signs, out,
                                                out_f16, positions, head_dim, lane_capacity, num_q_heads, num_kv_heads,
                                                window, bits, n_lanes, ring_capacity):
        """``flash_attention_tq_batched_into`` and the rotation back of every lane's heads as one call."""
        _check(self._l.lh_flash_attention_tq_batched_rotated_into(batch._h, rq._h, k_codes._h, k_norms._h, v_codes._h,
                                                                  v_norms._h, levels._h, signs._h, out._h, out_f16._h,
                                                                  positions._h, _u32(head_dim), _u32(lane_capacity),
                                                                  _u32(num_q_heads), _u32(num_kv_heads), _u32(window),
                                                                  _u32(bits), _u32(n_lanes), _u32(ring_capacity)))

    # -- FP16-KV split-K decode (kernels.rs:1265-1557) --
    def flash_split_count(self, eff_seq_len: int) -> int:
        return int(self._l.lh_flash_split_count(_u32(eff_seq_len)))

    def flash_decoding_into(self, batch, q, k, v, output, head_dim, kv_len, current_pos, num_q_heads, num_kv_heads):
        _check(self._l.lh_flash_decoding_into(batch._h, q._h, k._h, v._h, output._h, _u32(head_dim), _u32(kv_len),
                                              _u32(current_pos), _u32(num_q_heads), _u32(num_kv_heads)))

    def flash_attention_windowed_split_into(self, batch, q, k, v, output, partial_max, partial_sum, partial_acc,
                                            head_dim, kv_len, current_pos, num_q_heads, num_kv_heads, window,
                                            num_splits):
        _check(self._l.lh_flash_attention_windowed_split_into(batch._h, q._h, k._h, v._h, output._h, partial_max._h,
                                                              partial_sum._h, partial_acc._h, _u32(head_dim),
                                                              _u32(kv_len), _u32(current_pos), _u32(num_q_heads),
                                                              _u32(num_kv_heads), _u32(window), _u32(num_splits)))


from . import synth  # noqa: E402  (synthetic inputs of the measured configurations)
from .quant_weight import QuantWeight  # noqa: E402
from .kv_cache import QuantizedKvCache, QuantizedUnifiedKvPool, swa_ring_capacity, kv_bits_from_env, TQ_SEED, DEFAULT_KV_BITS  # noqa: E402
from . import gguf, weights  # noqa: E402  (GGUF reader and weight loader: gguf.rs, init_gemma4_qat.rs)
from . import layer  # noqa: E402  (decoder layer: layer.rs)
from . import pipeline  # noqa: E402  (decode core of the token loop: pipeline.rs)
from .layer import LayerParams, LayerWeights, ScratchBuffers, BatchScratch, TransformerLayer  # noqa: E402
