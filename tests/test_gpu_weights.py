"""A synthetic GGUF file (Q4_0, TQ2_0, F16, F32, BF16, Q8_0 tensors and a per-layer embedding table) loaded with
load_all_weights and used through QuantWeight: quantised tensors are uploaded verbatim and match the CPU dequant
path, everything else is expanded to exactly the f16 values of the reference's decode_tensor_to_f16
(init_gemma4_qat.rs:47-72, 179-232; known answers 241-265)."""
import struct

import numpy as np
import pytest

import refgen
from test_gguf_reader import build

pytestmark = pytest.mark.gpu


def q8_0_payload(n_elems, seed):
    g = np.random.default_rng(seed)
    blocks = n_elems // 32
    d = (g.random(blocks).astype(np.float32) * 0.02 + 0.001).astype(np.float16)
    q = g.integers(-128, 128, (blocks, 32), dtype=np.int8)
    raw = np.concatenate([d.view(np.uint8).reshape(blocks, 2), q.view(np.uint8)], axis=1).reshape(-1)
    want = (q.astype(np.float32) * d.astype(np.float32)[:, None]).astype(np.float16).reshape(-1)
    return raw, want


def test_load_all_weights_from_gguf(pkg, gpu, oracle, tmp_path, monkeypatch):
    ctx, K = gpu
    T = pkg.gguf.GGUFType
    rows, cols = 48, 512
    q4 = refgen.q4_0_payload(rows, cols, 0x11)
    tq = refgen.tq2_0_payload(rows, cols, 0x22)
    g = np.random.default_rng(3)
    f16 = g.standard_normal((rows, cols)).astype(np.float16)
    f32 = (g.standard_normal((rows, cols)) * 3).astype(np.float32)
    bf = (g.standard_normal(cols).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    q8_raw, q8_want = q8_0_payload(rows * cols, 5)
    ple = refgen.tq2_0_payload(20, 256, 0x33)
    tensors = [("blk.0.attn_q.weight", [cols, rows], int(T.Q4_0), q4.tobytes()),
               ("blk.0.ffn_gate.weight", [cols, rows], int(T.TQ2_0), tq.tobytes()),
               ("blk.0.half.weight", [cols, rows], int(T.F16), f16.tobytes()),
               ("blk.0.single.weight", [cols, rows], int(T.F32), f32.tobytes()),
               ("blk.0.norm.weight", [cols], int(T.BF16), bf.tobytes()),
               ("blk.0.q8.weight", [cols, rows], int(T.Q8_0), q8_raw.tobytes()),
               (pkg.weights.PLE_TABLE_NAME, [256, 20], int(T.TQ2_0), ple.tobytes())]
    path = tmp_path / "model.gguf"
    path.write_bytes(build(tensors, kvs=struct.pack("<Q", 12) + b"general.name" + struct.pack("<I", 8) + struct.pack("<Q", 4) + b"test", kv_count=1))
    model = pkg.gguf.GGUFModel.open(path)
    wm = pkg.weights.load_all_weights(model, ctx, K)
    assert set(wm.buffers) == {t[0] for t in tensors[:-1]} and wm.ple_table is not None

    x = np.sin(np.arange(cols, dtype=np.float32) * np.float32(0.731)).astype(np.float16)
    xb = pkg.Buffer.from_slice(ctx, x)

    def matvec(name):
        w = wm.buffers[name]
        y = pkg.Buffer.empty(ctx, w.rows * 4)
        batch = pkg.CommandBatch(ctx)
        w.matvec_f32out_into(batch, K, xb, y)
        batch.commit_and_wait()
        return w, y.as_array(np.float32)

    w, y = matvec("blk.0.attn_q.weight")
    assert w.ty == pkg.Q4_0 and (w.rows, w.cols) == (rows, cols) and w.device_bytes() >= q4.size
    refgen.assert_close(y, oracle.matvec_f32(oracle.expand_q4_0_f32(q4, rows, cols), x.astype(np.float32)), 1e-3, "q4_0 from gguf")
    w, y = matvec("blk.0.ffn_gate.weight")
    assert w.ty == pkg.TQ2_0
    refgen.assert_close(y, oracle.matvec_f32(oracle.expand_tq2_0_f32(tq, rows, cols), x.astype(np.float32)), 1e-3, "tq2_0 from gguf")
    for name, want16 in (("blk.0.half.weight", f16), ("blk.0.single.weight", f32.astype(np.float16)), ("blk.0.q8.weight", q8_want.reshape(rows, cols))):
        w, y = matvec(name)
        assert w.ty == pkg.quant_weight.W_F16
        assert np.array_equal(w.buf.as_array(np.uint16)[:rows * cols], np.asarray(want16).reshape(-1).view(np.uint16)), name
        refgen.assert_close(y, (want16.astype(np.float64) @ x.astype(np.float64)).astype(np.float32), 1e-3, name)
    nw = wm.buffers["blk.0.norm.weight"]                       # 1-D: rows 1, bf16 -> f16
    assert (nw.rows, nw.cols) == (1, cols)
    want = (bf.astype(np.uint32) << 16).view(np.float32).astype(np.float16)
    assert np.array_equal(nw.buf.as_array(np.uint16)[:cols], want.view(np.uint16))

    # per-layer embedding table: rows decoded on the device equal the CPU dequant bit for bit; the row index clamps
    deq = oracle.dequant_tq2_0(ple).reshape(20, 256)
    assert wm.ple_table.cols() == 256 and wm.ple_table.bytes() == ple.size
    for r in (0, 7, 19, 1000):
        assert np.array_equal(wm.ple_table.dequant_row(ctx, K, r).view(np.uint16), deq[min(r, 19)])

    # LOCAL_AI_QWEIGHTS=0: quantised tensors are expanded to f16 too (by the device dequant kernels)
    monkeypatch.setenv("LOCAL_AI_QWEIGHTS", "0")
    wm2 = pkg.weights.load_all_weights(model, ctx, K)
    w = wm2.buffers["blk.0.attn_q.weight"]
    assert w.ty == pkg.quant_weight.W_F16
    assert np.array_equal(w.buf.as_array(np.uint16)[:rows * cols], oracle.dequant_q4_0(q4))


def test_weight_rules(pkg, gpu):
    """init_gemma4_qat.rs:28-37, 84-110 and the known Q4_0 block of 241-265 (d = 0.5: nibble 15 -> 3.5, 0 -> -4)."""
    ctx, K = gpu
    T = pkg.gguf.GGUFType
    W = pkg.weights
    assert W.keep_quantized(T.Q4_0, [32, 4]) and W.keep_quantized(T.TQ2_0, [256, 4])
    assert not W.keep_quantized(T.Q4_0, [32]) and not W.keep_quantized(T.Q8_0, [32, 4]) and not W.keep_quantized(T.F16, [32, 4])
    assert W.weight_dims([512, 48]) == (48, 512) and W.weight_dims([512]) == (1, 512) and W.weight_dims([]) == (1, 1)
    with pytest.raises(pkg.gguf.InvalidFormat):
        W.QuantRowTable.new(ctx, np.zeros(66, np.uint8), T.TQ2_0, 100, 1)
    with pytest.raises(pkg.gguf.InvalidFormat):
        W.QuantRowTable.new(ctx, np.zeros(66, np.uint8), T.TQ2_0, 256, 2)
    nib = np.zeros(32, np.uint8); nib[0] = 15; nib[1] = 0; nib[2:] = 8
    block = np.concatenate([np.array([0.5], np.float16).view(np.uint8), (nib[:16] & 0xF) | (nib[16:] << 4)]).astype(np.uint8)
    t = W.QuantRowTable.new(ctx, block, T.Q4_0, 32, 1)
    row = t.dequant_row(ctx, K, 5).astype(np.float32)
    assert row[0] == 3.5 and row[1] == -4.0 and not row[2:].any()
    with pytest.raises(pkg.InvalidArgument):
        W.decode_tensor_to_f16_host(np.zeros(84, np.uint8), T.Q4_K, 256)
