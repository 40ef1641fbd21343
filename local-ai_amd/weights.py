"""Weights from GGUF tensors (local-engine/src/pipeline/init_gemma4_qat.rs:14-238): verbatim upload of the
formats that have device kernels (Q4_0, TQ2_0), FP16 expansion of everything else, and the per-layer token
embedding table kept packed and dequantised a row at a time.

MI355X: every tensor, including the multi-gigabyte per-layer embedding table the reference keeps in host
memory and decodes on the CPU per token, is resident in HBM; rows are decoded by the device kernels."""
from __future__ import annotations

import os
import sys
from typing import Dict, Optional, Sequence

import numpy as np

from . import Buffer, CommandBatch, InvalidArgument, Kernels, Q4_0, TQ2_0
from .gguf import GGUFModel, GGUFType, InvalidFormat
from .quant_weight import QuantWeight, W_F16

PLE_TABLE_NAME = "per_layer_token_embd.weight"          # init_gemma4_qat.rs:76
_DEVICE_TY = {GGUFType.Q4_0: Q4_0, GGUFType.TQ2_0: TQ2_0}


def quant_weights_enabled() -> bool:
    """init_gemma4_qat.rs:21-24: LOCAL_AI_QWEIGHTS=0 expands every tensor to FP16."""
    return os.environ.get("LOCAL_AI_QWEIGHTS") != "0"


def keep_quantized(ty: GGUFType, shape: Sequence[int]) -> bool:
    """init_gemma4_qat.rs:28-31."""
    return len(shape) == 2 and ty in _DEVICE_TY


def weight_dims(shape: Sequence[int]):
    """init_gemma4_qat.rs:33-37: GGUF stores [cols, rows]."""
    cols = int(shape[0]) if len(shape) > 0 else 1
    rows = int(shape[1]) if len(shape) > 1 else 1
    return rows, cols


def _f32_to_f16(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return x.astype(np.float16)          # IEEE round to nearest even, as half::f16::from_f32


def decode_tensor_to_f16_host(raw: np.ndarray, ty: GGUFType, num_elements: int) -> np.ndarray:
    """init_gemma4_qat.rs:179-200 for the formats whose expansion is plain host arithmetic: F32, F16, BF16 and
    Q8_0 (qat_recover.rs:105-129: f16(q * d)).  Q4_0 / TQ2_0 go through the device dequant kernels instead."""
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1)
    if ty == GGUFType.F32:
        return _f32_to_f16(raw.view(np.float32)[:num_elements])
    if ty == GGUFType.F16:
        return raw.view(np.float16)[:num_elements].copy()
    if ty == GGUFType.BF16:
        return _f32_to_f16((raw.view(np.uint16)[:num_elements].astype(np.uint32) << 16).view(np.float32))
    if ty == GGUFType.Q8_0:
        blocks = raw[:raw.size // 34 * 34].reshape(-1, 34)
        d = blocks[:, :2].copy().view(np.float16).astype(np.float32)          # [blocks, 1]
        q = blocks[:, 2:].view(np.int8).astype(np.float32)
        return _f32_to_f16(q * d).reshape(-1)[:num_elements]
    raise InvalidArgument(f"dequant not implemented for {ty.name}")           # qat_recover.rs:160-162


def _dequant_on_device(ctx, kernels: Kernels, raw: np.ndarray, ty: GGUFType, num_elements: int) -> Buffer:
    src = Buffer.from_slice(ctx, np.ascontiguousarray(raw, np.uint8))
    out = Buffer.empty(ctx, num_elements * 2)
    batch = CommandBatch(ctx)
    if ty == GGUFType.Q4_0:
        kernels.dequant_q4_0_into(batch, src, 0, out, num_elements)
    else:
        kernels.dequant_tq2_0_into(batch, src, 0, out, num_elements)
    batch.commit_and_wait()
    return out


def weight_from_raw(ctx, kernels: Kernels, raw, ty: GGUFType, shape: Sequence[int], name: str, allow_quant: bool) -> QuantWeight:
    """init_gemma4_qat.rs:47-72."""
    rows, cols = weight_dims(shape)
    kept = allow_quant and keep_quantized(ty, shape)
    if os.environ.get("LOCAL_AI_WFMT") is not None:
        print(f"[wfmt] {name} ty={ty.name} rows={rows} cols={cols} kept={str(kept).lower()}", file=sys.stderr)
    raw = np.ascontiguousarray(raw, np.uint8).reshape(-1)
    if kept:
        return QuantWeight.quantized(Buffer.from_slice(ctx, raw), _DEVICE_TY[ty], rows, cols)
    num_elements = 1
    for d in shape:
        num_elements *= int(d)
    if ty in _DEVICE_TY:
        buf = _dequant_on_device(ctx, kernels, raw, ty, num_elements)
    else:
        buf = Buffer.from_slice(ctx, decode_tensor_to_f16_host(raw, ty, num_elements))
    return QuantWeight.f16(buf, rows, cols)


class QuantRowTable:
    """init_gemma4_qat.rs:84-160: a packed [rows, cols] table whose rows are dequantised on demand (the per-layer
    token embeddings).  Here the table lives in HBM; Q4_0 / TQ2_0 rows are decoded by the device kernels, F16 rows
    are copied, other formats are expanded to F16 once at construction."""

    def __init__(self, weight: QuantWeight, ty: GGUFType, payload_bytes: int):
        self._w, self.ty, self._bytes = weight, ty, payload_bytes

    @classmethod
    def new(cls, ctx, raw, ty: GGUFType, cols: int, rows: int) -> "QuantRowTable":
        block = ty.block_size()
        if block == 0 or cols % block != 0:
            raise InvalidFormat(f"QuantRowTable: cols {cols} not a multiple of {ty.name} block size {block}")
        row_bytes = ty.tensor_bytes(cols)
        raw = np.ascontiguousarray(raw, np.uint8).reshape(-1)
        if raw.size < rows * row_bytes:
            raise InvalidFormat(f"QuantRowTable: payload {raw.size} < rows*row_bytes {rows * row_bytes}")
        if ty in _DEVICE_TY:
            w = QuantWeight.quantized(Buffer.from_slice(ctx, raw[:rows * row_bytes]), _DEVICE_TY[ty], rows, cols)
        else:
            w = QuantWeight.f16(Buffer.from_slice(ctx, decode_tensor_to_f16_host(raw[:rows * row_bytes], ty, rows * cols)), rows, cols)
        return cls(w, ty, raw.size)

    def cols(self) -> int:
        return self._w.cols

    def bytes(self) -> int:
        return self._bytes

    def dequant_row_into(self, batch, kernels: Kernels, row: int, out: Buffer) -> None:
        """Row `row` (clamped to the last row, init_gemma4_qat.rs:152) as cols f16 values into `out`."""
        self._w.dequant_row_into(batch, kernels, row, out)

    def dequant_rows_into(self, batch, kernels: Kernels, rows: Buffer, n_rows: int, out: Buffer, scale: float = 1.0) -> None:
        """Rows listed in a device u32 buffer, decoded side by side (pipeline.rs:1011-1019 loops over the tokens)."""
        self._w.dequant_rows_into(batch, kernels, rows, n_rows, out, scale)

    def dequant_row(self, ctx, kernels: Kernels, row: int) -> np.ndarray:
        out = Buffer.empty(ctx, self._w.cols * 2)
        batch = CommandBatch(ctx)
        self.dequant_row_into(batch, kernels, row, out)
        batch.commit_and_wait()
        return out.as_array(np.float16)


class WeightMap:
    """init_gemma4_qat.rs:14-19."""

    def __init__(self, buffers: Dict[str, QuantWeight], ple_table: Optional[QuantRowTable]):
        self.buffers, self.ple_table = buffers, ple_table


def load_all_weights(gguf: GGUFModel, ctx, kernels: Kernels) -> WeightMap:
    """init_gemma4_qat.rs:202-232."""
    allow_quant = quant_weights_enabled()
    buffers: Dict[str, QuantWeight] = {}
    ple_table = None
    for name, info in gguf.tensors.items():
        raw = gguf.tensor_data(name)
        if raw is None:
            raise InvalidFormat(f"tensor {name} has no data")
        if name == PLE_TABLE_NAME and len(info.shape) == 2:
            ple_table = QuantRowTable.new(ctx, raw, info.ty, int(info.shape[0]), int(info.shape[1]))
            continue
        buffers[name] = weight_from_raw(ctx, kernels, raw, info.ty, info.shape, name, allow_quant)
    return WeightMap(buffers, ple_table)
