"""GGUF container reader (local-engine/src/gguf.rs:6-420): tensor directory, type table and byte sizes.

Same behaviour as the reference's `GGUFModel`: key/value metadata is skipped, tensor names lose trailing
NULs, unknown tensor types are treated as F16 with a warning, tensor offsets are relative to the data
section, which starts at the next multiple of 32 after the tensor directory.  Tensor payloads are
returned as read-only views of a memory map of the file (the reference re-reads the range per call)."""
from __future__ import annotations

import enum
import mmap
import os
import struct
import sys
from dataclasses import dataclass
from typing import Dict, List, Optional

import numpy as np

from . import Error, Io


class InvalidFormat(Error):
    """local-engine/src/error.rs: Error::InvalidFormat."""


class GGUFType(enum.IntEnum):
    """gguf.rs:6-42."""
    F32 = 0; F16 = 1; Q4_0 = 2; Q4_1 = 3; Q8_0 = 8; Q8_1 = 9; Q2_K = 10; Q3_K = 11; Q4_K = 12; Q5_K = 13
    Q6_K = 14; Q8_K = 15; IQ2_XXS = 16; IQ2_XS = 17; IQ3_XXS = 18; IQ1_S = 19; IQ4_NL = 20; IQ3_S = 21
    IQ2_S = 22; IQ4_XS = 23; I8 = 24; I16 = 25; I32 = 26; I64 = 27; F64 = 28; IQ1_M = 29; BF16 = 30
    Q4_0_4_4 = 31; Q4_0_4_8 = 32; Q4_0_8_8 = 33; TQ1_0 = 34; TQ2_0 = 35; MXFP4 = 39; NVFP4 = 40; Q1_0 = 41

    @classmethod
    def from_u32(cls, raw: int) -> Optional["GGUFType"]:
        """gguf.rs:200-240."""
        try:
            return cls(raw)
        except ValueError:
            return None

    def elem_size(self) -> int:
        """gguf.rs:243-249."""
        return {GGUFType.F32: 4, GGUFType.F16: 2}.get(self, 1)

    def block_size(self) -> int:
        """gguf.rs:252-274."""
        T = GGUFType
        if self in (T.Q4_0, T.Q4_1, T.Q8_0, T.Q8_1, T.Q4_0_4_4, T.Q4_0_4_8, T.Q4_0_8_8, T.MXFP4):
            return 32
        if self in (T.Q2_K, T.Q3_K, T.Q4_K, T.Q5_K, T.Q6_K, T.Q8_K, T.IQ2_XXS, T.IQ2_XS, T.IQ3_XXS, T.IQ1_S, T.IQ4_NL,
                    T.IQ3_S, T.IQ2_S, T.IQ4_XS, T.IQ1_M, T.TQ1_0, T.TQ2_0):
            return 256
        if self == T.Q1_0:
            return 128
        if self == T.NVFP4:
            return 64
        return 1

    def tensor_bytes(self, num_elements: int) -> int:
        """gguf.rs:277-312."""
        T = GGUFType
        b32, b256 = -(-num_elements // 32), -(-num_elements // 256)
        table = {
            T.Q4_0: b32 * 18, T.Q4_1: b32 * 20, T.Q8_0: b32 * 34, T.Q8_1: b32 * 36,
            T.Q2_K: b256 * (16 * 2 + 2 * 4 + 16 + 4), T.Q3_K: b256 * (16 * 3 + 2 * 6 + 2), T.Q4_K: b256 * (16 * 4 + 2 * 6 + 2),
            T.Q5_K: b256 * (16 * 5 + 2 * 6 + 2), T.Q6_K: b256 * (16 * 12 + 2 * 2), T.Q8_K: b256 * (32 * 8 + 16 * 2 + 8 + 4),
            T.IQ2_XXS: b256 * (256 // 4 * 2 + 256 // 16 * 2), T.IQ2_XS: b256 * (256 // 4 * 2 + 256 // 16 * 2),
            T.IQ2_S: b256 * (256 // 4 * 2 + 256 // 16 * 2), T.IQ3_XXS: b256 * (256 // 3 * 3 + 256 // 8 * 2),
            T.IQ3_S: b256 * (256 // 3 * 3 + 256 // 8 * 2), T.IQ1_S: b256 * 256, T.IQ1_M: b256 * 256,
            T.IQ4_NL: b256 * (256 // 2 + 256 // 16 * 2), T.IQ4_XS: b256 * (256 // 2 + 256 // 16 * 2),
            T.I8: num_elements, T.I16: num_elements * 2, T.I32: num_elements * 4, T.I64: num_elements * 8,
            T.F64: num_elements * 8, T.BF16: num_elements * 2, T.TQ1_0: b256 * (2 + 4 * 13), T.TQ2_0: b256 * (2 + 64),
        }
        return table.get(self, num_elements * self.elem_size())


@dataclass
class TensorInfo:
    """gguf.rs:44-75."""
    name: str
    ty: GGUFType
    shape: List[int]
    offset: int      # relative to the data section
    bytes: int

    def shape_usize(self) -> List[int]:
        return list(self.shape)

    def elem_bytes(self) -> int:
        return {GGUFType.F32: 4, GGUFType.F16: 2}.get(self.ty, 1)

    def compute_bytes(self) -> int:
        total = int(np.prod(self.shape, dtype=np.uint64)) if self.shape else 1
        if self.ty in (GGUFType.F32, GGUFType.F16):
            return total * self.elem_bytes()
        return self.ty.tensor_bytes(total)


def _read_string(raw, off: int):
    """gguf.rs:321-336."""
    if off + 8 > len(raw):
        raise InvalidFormat("GGUF truncated inside a string length")
    (n,) = struct.unpack_from("<Q", raw, off)
    off += 8
    if off + n > len(raw):
        raise InvalidFormat("GGUF truncated inside a string")
    try:
        s = bytes(raw[off:off + n]).decode("utf-8")
    except UnicodeDecodeError as e:
        raise InvalidFormat(f"utf8 {e}") from None
    return s, off + n


_SCALAR_BYTES = {0: 1, 1: 1, 7: 1, 2: 2, 3: 2, 4: 4, 5: 4, 6: 4, 10: 8, 11: 8, 12: 8}


def _skip_kv(raw, off: int) -> int:
    """gguf.rs:338-418: key, value tag, value (scalars, string, arrays of scalars or strings)."""
    _key, off = _read_string(raw, off)
    if off >= len(raw):
        return off
    (tag,) = struct.unpack_from("<I", raw, off)
    off += 4
    if tag in _SCALAR_BYTES:
        return off + _SCALAR_BYTES[tag]
    if tag == 8:
        (n,) = struct.unpack_from("<Q", raw, off)
        return off + 8 + n
    if tag == 9:
        elem_type, n = struct.unpack_from("<IQ", raw, off)
        off += 12
        if elem_type in _SCALAR_BYTES:
            return off + n * _SCALAR_BYTES[elem_type]
        if elem_type == 8:
            for _ in range(n):
                (slen,) = struct.unpack_from("<Q", raw, off)
                off += 8 + slen
            return off
        raise InvalidFormat(f"unsupported array element type {elem_type}")
    raise InvalidFormat(f"unknown KV tag {tag}")


class GGUFModel:
    """gguf.rs:77-196."""

    def __init__(self, version: int, tensors: Dict[str, TensorInfo], data_offset: int, path: str, raw):
        self.version, self.tensors, self.data_offset, self.path = version, tensors, data_offset, path
        self._raw = raw

    @classmethod
    def open(cls, path) -> "GGUFModel":
        path = os.fspath(path)
        try:
            with open(path, "rb") as f:
                size = os.fstat(f.fileno()).st_size
                raw = mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ) if size else b""
        except OSError as e:
            raise Io(str(e)) from None
        return cls.parse(raw, path)

    @classmethod
    def parse(cls, raw, path="") -> "GGUFModel":
        if len(raw) < 24:
            raise InvalidFormat("GGUF too short")
        if bytes(raw[0:4]) != b"GGUF":
            raise InvalidFormat("bad magic")
        version, tensor_count, kv_count = struct.unpack_from("<IQQ", raw, 4)
        off = 24
        try:
            for _ in range(kv_count):
                off = _skip_kv(raw, off)
            tensors: Dict[str, TensorInfo] = {}
            for _ in range(tensor_count):
                name, off = _read_string(raw, off)
                (n_dims,) = struct.unpack_from("<I", raw, off)
                off += 4
                shape = list(struct.unpack_from(f"<{n_dims}Q", raw, off))
                off += 8 * n_dims
                ty_raw, file_offset = struct.unpack_from("<IQ", raw, off)
                off += 12
                ty = GGUFType.from_u32(ty_raw)
                if ty is None:
                    print(f"warning: unknown GGUF tensor type {ty_raw} for tensor '{name}', treating as F16", file=sys.stderr)
                    ty = GGUFType.F16
                total = 1
                for d in shape:
                    total *= d
                name = name.rstrip("\0")
                tensors[name] = TensorInfo(name, ty, shape, file_offset, ty.tensor_bytes(total))
        except struct.error:
            raise InvalidFormat("GGUF truncated inside the header") from None
        data_offset = (off + 31) & ~31       # `general.alignment` default
        return cls(version, dict(sorted(tensors.items())), data_offset, path, raw)

    def tensor_info(self, name: str) -> Optional[TensorInfo]:
        return self.tensors.get(name)

    def tensor_data(self, name: str) -> Optional[np.ndarray]:
        """The tensor's payload as a read-only uint8 view of the file; None if absent or out of range."""
        info = self.tensor_info(name)
        if info is None:
            return None
        start = self.data_offset + info.offset
        end = start + info.bytes
        if end > len(self._raw):
            return None
        return np.frombuffer(self._raw, dtype=np.uint8, count=info.bytes, offset=start)
