"""FP16-weight matvec family through the C ABI against the numpy restatement (oracle/layer_glue.py:matvec_f16):
the reference's known-answer vectors (kernels.rs:7294-7360) and seeded shapes incl. ragged cols (the one-element
path), cols beyond the LDS staging limit, a byte offset into the weight buffer, and the QuantWeight F16 variant."""
import numpy as np
import pytest

from oracle import layer_glue as lg
import refgen

pytestmark = pytest.mark.gpu


def test_known_answer_vectors(pkg, gpu):
    ctx, K = gpu
    for mat, vec, rows, cols, want in (([1, 0, 0, 0, 1, 0, 0, 0, 1], [5, 7, 9], 3, 3, [5, 7, 9]),
                                       ([1, 2, 3, 4], [5, 6], 2, 2, [17, 39]),
                                       ([1, 2, 3, 4, 5, 6, 7, 8], [1, 1, 1, 1], 2, 4, [10, 26])):
        m, v = pkg.Buffer.from_slice(ctx, np.array(mat, np.float16)), pkg.Buffer.from_slice(ctx, np.array(vec, np.float16))
        out = pkg.Buffer.empty(ctx, rows * 2)
        K.matvec(ctx, m, v, out, rows, cols)
        assert np.array_equal(out.as_array(np.float16).astype(np.float32), np.array(want, np.float32))
        assert np.array_equal(lg.matvec_f16(np.array(mat, np.float16), np.array(vec, np.float16), rows, cols).astype(np.float32),
                              np.array(want, np.float32))


# (the last four: rows long enough for the form that keeps a lane's activations in registers -- one pass per row, with
# and without lanes past the row's end, one / four / eight loads per lane)
@pytest.mark.parametrize("rows,cols", [(256, 1536), (1536, 256), (33, 100), (7, 16392), (4096, 2048), (5, 8),
                                       (32773, 512), (33001, 1536), (32768, 2048), (32808, 2600)])
def test_matvec_f16_family(pkg, gpu, rows, cols):
    ctx, K = gpu
    g = pkg.synth.rng(31, rows + cols)
    w = (g.standard_normal((rows, cols), dtype=np.float32) * 0.5).astype(np.float16)
    x16 = g.standard_normal(cols, dtype=np.float32).astype(np.float16)
    x32 = g.standard_normal(cols, dtype=np.float32)
    pad = 32   # bytes in front of the matrix: exercises the offset argument (and keeps 16-byte alignment)
    wb = pkg.Buffer.from_slice(ctx, np.concatenate([np.zeros(pad // 2, np.float16), w.reshape(-1)]))
    xb16, xb32 = pkg.Buffer.from_slice(ctx, x16), pkg.Buffer.from_slice(ctx, x32)
    y16, y32, y16b = pkg.Buffer.empty(ctx, rows * 2), pkg.Buffer.empty(ctx, rows * 4), pkg.Buffer.empty(ctx, rows * 2)
    batch = pkg.CommandBatch(ctx)
    K.matvec_offset_into(batch, wb, pad, xb16, y16, rows, cols)
    K.matvec_f32out_offset_into(batch, wb, pad, xb16, y32, rows, cols)
    K.matvec_f32in_offset_into(batch, wb, pad, xb32, y16b, rows, cols)
    batch.commit_and_wait()
    refgen.assert_close(y32.as_array(np.float32), lg.matvec_f16(w, x16, rows, cols, out_f32=True), 1e-3, "f32out")
    refgen.assert_close(y16.as_array(np.float16).astype(np.float32), lg.matvec_f16(w, x16, rows, cols).astype(np.float32), 2e-3, "f16")
    refgen.assert_close(y16b.as_array(np.float16).astype(np.float32), lg.matvec_f16(w, x32, rows, cols).astype(np.float32), 2e-3, "f32in")
    # one-shot forms (enqueue and wait)
    z = pkg.Buffer.empty(ctx, rows * 4)
    K.matvec_f32out_offset(ctx, wb, pad, xb16, z, rows, cols)
    assert np.array_equal(z.as_array(np.uint32), y32.as_array(np.uint32))


def test_quant_weight_f16_variant(pkg, gpu):
    """layer.rs:27-34, 120-246, 269-281: an F16 QuantWeight routes to the FP16 kernels; a row dequantises to itself."""
    ctx, K = gpu
    rows, cols, m = 96, 512, 5
    g = pkg.synth.rng(32, 1)
    w = (g.standard_normal((rows, cols), dtype=np.float32) * 0.5).astype(np.float16)
    x = g.standard_normal((m, cols), dtype=np.float32).astype(np.float16)
    qw = pkg.QuantWeight.f16(pkg.Buffer.from_slice(ctx, w), rows, cols)
    xb = pkg.Buffer.from_slice(ctx, x)
    y, y32, c, row = pkg.Buffer.empty(ctx, rows * 2), pkg.Buffer.empty(ctx, rows * 4), pkg.Buffer.empty(ctx, m * rows * 2), pkg.Buffer.empty(ctx, cols * 2)
    batch = pkg.CommandBatch(ctx)
    qw.matvec_into(batch, K, xb, y)
    qw.matvec_f32out_into(batch, K, xb, y32)
    qw.matmul_nt_into(batch, K, xb, c, m)
    qw.dequant_row_into(batch, K, 1000, row)
    batch.commit_and_wait()
    refgen.assert_close(y32.as_array(np.float32), lg.matvec_f16(w, x[0], rows, cols, out_f32=True), 1e-3, "qw f32out")
    refgen.assert_close(y.as_array(np.float16).astype(np.float32), lg.matvec_f16(w, x[0], rows, cols).astype(np.float32), 2e-3, "qw f16")
    want = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
    refgen.assert_close(c.as_array(np.float16).astype(np.float32), want, 2e-3, "qw matmul")
    assert np.array_equal(row.as_array(np.uint16), w[rows - 1].view(np.uint16))
    assert qw.device_bytes() >= rows * cols * 2 and qw.row_bytes() == cols * 2


def test_matvec_f16_argument_errors(pkg, gpu):
    ctx, K = gpu
    small = pkg.Buffer.empty(ctx, 64)
    batch = pkg.CommandBatch(ctx)
    with pytest.raises(pkg.InvalidArgument):
        K.matvec_offset_into(batch, small, 0, small, small, 64, 64)
    with pytest.raises(pkg.InvalidArgument):
        K.matvec_offset_into(batch, small, 1, small, small, 2, 2)
