"""``QuantWeight`` (local-engine/src/layer.rs:18-282): a format-tagged weight in device
memory that routes matvec / matmul calls to the kernel for its block format."""
from __future__ import annotations

import numpy as np

from . import Q4_0, TQ2_0, ROWS_F16, F16, F32, BF16, Buffer, InvalidArgument, Kernels

_BLOCK = {Q4_0: (32, 18), TQ2_0: (256, 66)}
W_F16 = "f16"   # GGUFType::F16: plain f16 rows, served by the FP16 matvec / matmul kernels (layer.rs:27-34)


class QuantWeight:
    def __init__(self, buf: Buffer, ty: int, rows: int, cols: int):
        self.buf, self.ty, self.rows, self.cols = buf, ty, rows, cols

    @classmethod
    def f16(cls, buf: Buffer, rows: int, cols: int) -> "QuantWeight":
        """layer.rs:27-34: an FP16 tensor (also what Q8_0 / F32 tensors are expanded to at load time)."""
        return cls(buf, W_F16, rows, cols)

    @classmethod
    def quantized(cls, buf: Buffer, ty: int, rows: int, cols: int) -> "QuantWeight":
        """layer.rs:42-66: only Q4_0 and TQ2_0 have device kernels; cols must be block aligned."""
        if ty not in _BLOCK:
            raise InvalidArgument(f"QuantWeight: no device kernel for {ty!r}")
        block = _BLOCK[ty][0]
        if cols % block != 0:
            raise InvalidArgument(f"QuantWeight: cols {cols} not a multiple of block {block}")
        return cls(buf, ty, rows, cols)

    @classmethod
    def from_bytes(cls, ctx, raw, ty: int, rows: int, cols: int) -> "QuantWeight":
        """Verbatim GGUF payload upload (local-engine/src/pipeline/init_gemma4_qat.rs:62-66)."""
        raw = np.ascontiguousarray(raw, np.uint8).reshape(-1)
        block, nbytes = _BLOCK[ty]
        if raw.size != rows * (cols // block) * nbytes:
            raise InvalidArgument(f"QuantWeight: payload of {raw.size} bytes does not match {rows}x{cols}")
        return cls.quantized(Buffer.from_slice(ctx, raw), ty, rows, cols)

    def device_bytes(self) -> int:
        return self.buf.length()

    def row_bytes(self) -> int:
        if self.ty == W_F16:
            return self.cols * 2
        block, nbytes = _BLOCK[self.ty]
        return (self.cols // block) * nbytes

    # layer.rs:120-161: out[rows] = self x x[cols]
    def matvec_into(self, batch, kernels: Kernels, x: Buffer, out: Buffer) -> None:
        if self.ty == Q4_0:
            kernels.matvec_q4_0_into(batch, self.buf, x, out, self.rows, self.cols)
        elif self.ty == TQ2_0:
            kernels.matvec_tq2_0_into(batch, self.buf, x, out, self.rows, self.cols)
        else:
            kernels.matvec_offset_into(batch, self.buf, 0, x, out, self.rows, self.cols)

    def matvec_f32out_into(self, batch, kernels: Kernels, x: Buffer, out: Buffer) -> None:
        if self.ty == Q4_0:
            kernels.matvec_q4_0_f32out_into(batch, self.buf, x, out, self.rows, self.cols)
        elif self.ty == TQ2_0:
            kernels.matvec_tq2_0_f32out_into(batch, self.buf, x, out, self.rows, self.cols)
        else:
            kernels.matvec_f32out_offset_into(batch, self.buf, 0, x, out, self.rows, self.cols)

    def matvec_typed_into(self, batch, kernels: Kernels, x: Buffer, x_dtype: int, out: Buffer, out_dtype: int) -> None:
        kernels.matvec_quant_typed_into(batch, self.ty, self.buf, x, x_dtype, out, out_dtype, self.rows, self.cols)

    # layer.rs:218-246: out[m, rows] = x[m, cols] . self^T
    def matmul_nt_into(self, batch, kernels: Kernels, x: Buffer, out: Buffer, m: int) -> None:
        if self.ty == Q4_0:
            kernels.matmul_nt_q4_0_into(batch, x, self.buf, out, m, self.cols, self.rows)
        elif self.ty == TQ2_0:
            kernels.matmul_nt_tq2_0_into(batch, x, self.buf, out, m, self.cols, self.rows)
        else:
            kernels.matmul_nt_into(batch, x, self.buf, out, m, self.cols, self.rows)

    def matmul_nt_typed_into(self, batch, kernels: Kernels, x: Buffer, x_dtype: int, out: Buffer, out_dtype: int,
                             m: int) -> None:
        kernels.matmul_nt_quant_typed_into(batch, self.ty, x, x_dtype, self.buf, out, out_dtype, m, self.cols,
                                           self.rows)

    # layer.rs:269-281: one row dequantised to f16 (embedding gather); row clamps to the last row
    def dequant_row_into(self, batch, kernels: Kernels, row: int, out: Buffer) -> None:
        row = min(row, self.rows - 1)
        off = row * self.row_bytes()
        if self.ty == Q4_0:
            kernels.dequant_q4_0_into(batch, self.buf, off, out, self.cols)
        elif self.ty == TQ2_0:
            kernels.dequant_tq2_0_into(batch, self.buf, off, out, self.cols)
        else:
            batch.blit_copy(self.buf, off, out, 0, self.cols * 2)   # an f16 row is its own dequantisation

    def dequant_rows_into(self, batch, kernels: Kernels, rows: Buffer, n_rows: int, out: Buffer, scale: float = 1.0) -> None:
        """The rows listed in the device u32 buffer `rows` as a dense f16 [n_rows, cols] matrix, optionally scaled: the
        embedding gather of a chunk or of a step over many lanes (local-engine/src/pipeline.rs:781-832) in one dispatch."""
        fmt = ROWS_F16 if self.ty == W_F16 else self.ty
        kernels.dequant_rows_into(batch, fmt, self.buf, self.rows, self.cols, rows, n_rows, out, scale)
