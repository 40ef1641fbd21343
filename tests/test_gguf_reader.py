"""GGUF reader and type table (local-ai_amd/gguf.py) against the reference's own tests (gguf.rs:424-529) and the
format's layout.  CPU only: nothing here touches the GPU library."""
import struct

import numpy as np
import pytest

import __graft_entry__ as ge


@pytest.fixture(scope="module")
def gg():
    return ge.load_package().gguf


def s(x: str) -> bytes:
    b = x.encode()
    return struct.pack("<Q", len(b)) + b


def build(tensors, kvs=b"", kv_count=0, version=3):
    """tensors: (name, dims, type id, payload bytes).  Mirrors write_tensor_info / finalize_gguf (gguf.rs:433-476):
    names carry a trailing NUL, offsets are relative to the 32-byte aligned data section."""
    buf = bytearray(b"GGUF" + struct.pack("<IQQ", version, len(tensors), kv_count) + kvs)
    pos = []
    for name, dims, ty, data in tensors:
        buf += s(name + "\0") + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims) + struct.pack("<I", ty)
        pos.append(len(buf))
        buf += struct.pack("<Q", 0)
    buf += bytes((-len(buf)) % 32)
    rel = 0
    for p, (_, _, _, data) in zip(pos, tensors):
        buf[p:p + 8] = struct.pack("<Q", rel)
        rel += len(data)
    for _, _, _, data in tensors:
        buf += data
    return bytes(buf)


def test_read_minimal_and_multiple(gg, tmp_path):
    """gguf.rs:478-514."""
    f = tmp_path / "minimal.gguf"
    f.write_bytes(build([("embed", [256, 1000], 0, bytes(256 * 1000 * 4))]))
    m = gg.GGUFModel.open(f)
    info = m.tensor_info("embed")
    assert info.shape == [256, 1000] and info.ty == gg.GGUFType.F32 and m.version == 3
    assert m.tensor_data("embed").size == 256 * 1000 * 4 and info.compute_bytes() == 256 * 1000 * 4
    f2 = tmp_path / "multi.gguf"
    f2.write_bytes(build([("x", [10], 0, bytes(40)), ("y", [20], 0, bytes(range(80)))]))
    m = gg.GGUFModel.open(f2)
    assert m.tensor_info("x").shape == [10] and m.tensor_info("y").shape == [20]
    assert m.tensor_info("y").offset == 40 and m.data_offset % 32 == 0
    assert bytes(m.tensor_data("y")) == bytes(range(80))
    assert m.tensor_info("nope") is None and m.tensor_data("nope") is None


def test_tensor_byte_sizes_and_blocks(gg):
    """gguf.rs:516-528 and the table at 277-312."""
    T = gg.GGUFType
    assert T.Q2_K.tensor_bytes(1024) == 4 * 60 and T.Q2_K.tensor_bytes(256) == 60 and T.Q2_K.tensor_bytes(512) == 120
    assert T.Q4_0.tensor_bytes(1024) == 32 * 18 and T.Q8_0.tensor_bytes(1024) == 32 * 34
    assert T.TQ2_0.tensor_bytes(256) == 66 and T.TQ2_0.tensor_bytes(257) == 132 and T.TQ1_0.tensor_bytes(256) == 54
    assert T.F32.tensor_bytes(7) == 28 and T.F16.tensor_bytes(7) == 14 and T.BF16.tensor_bytes(7) == 14 and T.I64.tensor_bytes(3) == 24
    assert T.Q4_0.block_size() == 32 and T.TQ2_0.block_size() == 256 and T.Q1_0.block_size() == 128 and T.NVFP4.block_size() == 64
    assert T.F16.block_size() == 1 and T.from_u32(35) == T.TQ2_0 and T.from_u32(36) is None and T.from_u32(2) == T.Q4_0


def test_metadata_is_skipped_and_names_trimmed(gg, tmp_path, capsys):
    """gguf.rs:338-418: every scalar tag, strings, scalar and string arrays; unknown tensor types read as F16."""
    kvs = (s("a.u8") + struct.pack("<IB", 0, 1) + s("a.i16") + struct.pack("<Ih", 3, -2) + s("a.f32") + struct.pack("<If", 6, 1.5)
           + s("a.bool") + struct.pack("<IB", 7, 1) + s("a.str") + struct.pack("<I", 8) + s("hello") + s("a.u64") + struct.pack("<IQ", 10, 7)
           + s("a.arr") + struct.pack("<IIQ", 9, 4, 3) + struct.pack("<3I", 1, 2, 3)
           + s("a.sarr") + struct.pack("<IIQ", 9, 8, 2) + s("x") + s("yz"))
    raw = build([("blk.0.w", [256, 4], 35, bytes(4 * 66)), ("odd", [8], 77, bytes(16))], kvs=kvs, kv_count=8)
    f = tmp_path / "kv.gguf"
    f.write_bytes(raw)
    m = gg.GGUFModel.open(f)
    assert list(m.tensors) == ["blk.0.w", "odd"]                      # BTreeMap order, NULs trimmed
    assert m.tensor_info("blk.0.w").ty == gg.GGUFType.TQ2_0 and m.tensor_info("blk.0.w").bytes == 4 * 66
    assert m.tensor_info("odd").ty == gg.GGUFType.F16 and "unknown GGUF tensor type 77" in capsys.readouterr().err
    assert m.tensor_data("odd").size == 16


def test_malformed_files(gg, tmp_path):
    with pytest.raises(gg.InvalidFormat, match="too short"):
        gg.GGUFModel.parse(b"GGUF")
    with pytest.raises(gg.InvalidFormat, match="bad magic"):
        gg.GGUFModel.parse(b"GGML" + bytes(40))
    bad = b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + s("k") + struct.pack("<I", 99)
    with pytest.raises(gg.InvalidFormat, match="unknown KV tag 99"):
        gg.GGUFModel.parse(bad + bytes(16))
    with pytest.raises(Exception):
        gg.GGUFModel.open(tmp_path / "missing.gguf")
