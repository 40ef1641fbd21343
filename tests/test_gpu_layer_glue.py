"""Parity of the decoder-layer glue kernels (through the C ABI) with oracle/layer_glue.py.

Tolerances: f16 outputs of f32 math may differ by one f16 rounding where the device's rsqrt / pow /
cos / sin / tanh differ from libm in the last bits: |g - w| <= 2e-3 * max(|w|, 1) (the reference's own
tests allow 0.01-0.02, kernels.rs:7050-7288).  Copies, the f16 add and the f32 scale are bit-exact."""
import numpy as np
import pytest

from oracle import layer_glue as lg
import refgen

pytestmark = pytest.mark.gpu


def close(got, want, tol, label):
    refgen.assert_close(np.asarray(got, np.float32), np.asarray(want, np.float32), tol, label)


@pytest.mark.parametrize("dim,rows", [(4, 1), (1536, 1), (1536, 7), (2048, 16), (100, 3), (8192, 2)])
def test_rms_norm_and_fused_residual(pkg, gpu, dim, rows):
    """kernels.rs:7050 (known vector shape 4 x 1), 7650; decode rows of hidden 1536 / 2048 and ragged dims."""
    ctx, K = gpu
    g = pkg.synth.rng(21, dim + rows)
    x = (g.standard_normal((rows, dim), dtype=np.float32) * 2).astype(np.float16)
    if dim == 4:
        x[0] = [1, 2, 3, 4]
    w = (1.0 + 0.1 * g.standard_normal(dim, dtype=np.float32)).astype(np.float16)
    r = g.standard_normal((rows, dim), dtype=np.float32).astype(np.float16)
    xb, wb, rb = pkg.Buffer.from_slice(ctx, x), pkg.Buffer.from_slice(ctx, w), pkg.Buffer.from_slice(ctx, r)
    o1, o2 = pkg.Buffer.empty(ctx, x.nbytes), pkg.Buffer.empty(ctx, x.nbytes)
    batch = pkg.CommandBatch(ctx)
    K.rms_norm_into(batch, xb, wb, o1, dim, rows, 1e-6)
    K.rms_norm_add_into(batch, xb, wb, rb, o2, dim, rows, 1e-6)
    K.rms_norm_add_into(batch, xb, wb, rb, rb, dim, rows, 1e-6)   # output aliases the residual (layer.rs:443)
    batch.commit_and_wait()
    close(o1.as_array(np.float16), lg.rms_norm(x, w, dim, rows, 1e-6), 2e-3, f"rms_norm {rows}x{dim}")
    want = lg.rms_norm(x, w, dim, rows, 1e-6, residual=r)
    close(o2.as_array(np.float16), want, 2e-3, f"rms_norm_add {rows}x{dim}")
    assert np.array_equal(rb.as_array(np.uint16), o2.as_array(np.uint16))


@pytest.mark.parametrize("hd,nh,prf,pos,theta", [(64, 4, 1.0, 137, 1e4), (256, 8, 1.0, 137, 1e6), (256, 8, 0.5, 137, 1e6),
                                                 (512, 8, 0.25, 100000, 1e6), (8, 1, 0.25, 100, 1e4), (256, 1, 1.0, 0, 1e6)])
def test_qk_norm_rope_family(pkg, gpu, hd, nh, prf, pos, theta):
    """kernels.rs:7214-7288, 7818-7925: qk_norm, rope, and the fused kernel == the two in sequence, bit for bit,
    with input == output as the reference's test runs them."""
    ctx, K = gpu
    n = nh * hd
    data = (np.sin(np.arange(n, dtype=np.float32) * np.float32(0.013)) * np.float32(0.8)).astype(np.float16)
    w = (1.0 + np.cos(np.arange(hd, dtype=np.float32) * np.float32(0.005)) * np.float32(0.1)).astype(np.float16)
    wb = pkg.Buffer.from_slice(ctx, np.concatenate([np.zeros(16, np.float16), w]))   # weights behind a 32-byte offset
    w0 = pkg.Buffer.from_slice(ctx, w)
    sep, fused, normed, roped = (pkg.Buffer.from_slice(ctx, data) for _ in range(4))
    rope_out = pkg.Buffer.empty(ctx, n * 2)
    batch = pkg.CommandBatch(ctx)
    K.qk_norm_offset_into(batch, normed, wb, 32, hd, nh, 1e-6)
    K.rope_into(batch, roped, rope_out, hd, pos, theta, prf, nh)
    K.qk_norm_gpu_into(batch, sep, w0, hd, nh, 1e-6)
    K.rope_into(batch, sep, sep, hd, pos, theta, prf, nh)
    assert K.qk_norm_rope_available(hd)
    K.qk_norm_rope_into(batch, fused, fused, w0, hd, nh, 1e-6, pos, theta, prf)
    batch.commit_and_wait()
    # angle = position * freq is an f32 of magnitude up to `pos`: one ulp of it (pos * 2^-23 rad) is the floor of
    # the agreement between two correctly rounded implementations of pow / cos / sin
    tol = 2e-3 + 2.5e-7 * pos
    close(normed.as_array(np.float16), lg.qk_norm(data, w, hd, nh, 1e-6), 2e-3, "qk_norm")
    close(rope_out.as_array(np.float16), lg.rope(data, hd, pos, theta, prf, nh), tol, "rope")
    assert np.array_equal(fused.as_array(np.uint16), sep.as_array(np.uint16)), "fused qk_norm_rope != qk_norm + rope"
    close(fused.as_array(np.float16), lg.qk_norm_rope(data, w, hd, nh, 1e-6, pos, theta, prf), tol + 1e-3, "qk_norm_rope")
    if pos == 0:
        assert np.array_equal(rope_out.as_array(np.uint16), data.view(np.uint16))
    # pairs beyond the rotated prefix pass through untouched
    ra = int(np.float32(hd) * np.float32(prf)) // 2
    got = rope_out.as_array(np.uint16).reshape(nh, hd)
    src = data.view(np.uint16).reshape(nh, hd)
    assert np.array_equal(got[:, ra:hd // 2], src[:, ra:hd // 2]) and np.array_equal(got[:, hd // 2 + ra:], src[:, hd // 2 + ra:])


@pytest.mark.parametrize("hd,nh,rows,prf", [(256, 8, 5, 1.0), (512, 2, 3, 0.25), (64, 4, 17, 0.5)])
def test_rope_batch_forms(pkg, gpu, hd, nh, rows, prf):
    """kernels.rs:8079-8190: rope_batch == rope per row at consecutive positions (bit for bit: same rotation code),
    rope_batch_decode == rope_batch for contiguous positions and applies independent positions per row."""
    ctx, K = gpu
    n = rows * nh * hd
    data = (np.sin(np.arange(n, dtype=np.float32) * np.float32(0.017)) * np.float32(0.9)).astype(np.float16)
    start, theta = 731, 1e6
    per_row = pkg.Buffer.from_slice(ctx, data)
    batched, dec_contig, dec_indep = (pkg.Buffer.from_slice(ctx, data) for _ in range(3))
    pos_indep = np.array([(r * 7919 + 13) % 50000 for r in range(rows)], np.uint32)
    pc, pi = pkg.Buffer.from_slice(ctx, np.arange(start, start + rows, dtype=np.uint32)), pkg.Buffer.from_slice(ctx, pos_indep)
    batch = pkg.CommandBatch(ctx)
    for r in range(rows):
        v = per_row.view(r * nh * hd * 2, nh * hd * 2)
        K.rope_into(batch, v, v, hd, start + r, theta, prf, nh)
    K.rope_batch_into(batch, batched, start, theta, hd, nh, rows, prf)
    K.rope_batch_decode_into(batch, dec_contig, pc, theta, hd, nh, rows, prf)
    K.rope_batch_decode_into(batch, dec_indep, pi, theta, hd, nh, rows, prf)
    batch.commit_and_wait()
    assert np.array_equal(batched.as_array(np.uint16), per_row.as_array(np.uint16))
    assert np.array_equal(dec_contig.as_array(np.uint16), batched.as_array(np.uint16))
    got = dec_indep.as_array(np.float16).reshape(rows, nh * hd)
    for r in range(rows):
        want = lg.rope(data.reshape(rows, nh * hd)[r], hd, int(pos_indep[r]), theta, prf, nh)
        close(got[r], want, 2e-3 + 2.5e-7 * int(pos_indep[r]), f"rope_batch_decode row {r}")


@pytest.mark.parametrize("n", [8192 + 37, 8192, 8])
def test_elementwise_glue(pkg, gpu, n):
    """kernels.rs:7076-7117, 7693-7815: gelu_mul, residual_add, scale_in_place, gather_strided_f16, logit_softcap
    (counts that take the 8-wide and the one-element form)."""
    ctx, K = gpu
    g = pkg.synth.rng(22, 5)
    a = (g.standard_normal(n, dtype=np.float32) * 3).astype(np.float16)
    a[:8] = [0, 1, -1, 2, 10, -10, 19, 65000]
    b = g.standard_normal(n, dtype=np.float32).astype(np.float16)
    ab, bb = pkg.Buffer.from_slice(ctx, a), pkg.Buffer.from_slice(ctx, b)
    o_gelu, o_add = pkg.Buffer.empty(ctx, n * 2), pkg.Buffer.empty(ctx, n * 2)
    sc = pkg.Buffer.from_slice(ctx, a)
    src = np.arange(5 * 7 * 4, dtype=np.float32).astype(np.float16)
    srcb, dstb = pkg.Buffer.from_slice(ctx, src), pkg.Buffer.empty(ctx, 5 * 4 * 2)
    logits = ((np.arange(4096, dtype=np.float32) - 2048.0) * np.float32(0.05))
    lb = pkg.Buffer.from_slice(ctx, logits)
    batch = pkg.CommandBatch(ctx)
    K.gelu_mul_into(batch, ab, bb, o_gelu, n)
    K.residual_add_into(batch, ab, bb, o_add, n)
    K.scale_in_place_gpu_into(batch, sc, 0.3, n)
    K.gather_strided_f16_into(batch, srcb, dstb, 7 * 4, 3 * 4, 4, 5)
    K.logit_softcap_gpu_into(batch, lb, 30.0, 4096)
    batch.commit_and_wait()
    got = o_gelu.as_array(np.float16).astype(np.float32)
    want = lg.gelu_mul(a, b).astype(np.float32)
    assert np.isfinite(got[~np.isinf(want)]).all()
    fin = np.isfinite(want)
    close(got[fin], want[fin], 2e-3, "gelu_mul")
    assert np.array_equal(o_add.as_array(np.uint16), lg.residual_add(a, b).view(np.uint16))
    assert np.array_equal(sc.as_array(np.uint16), lg.scale_in_place(a, 0.3).view(np.uint16))
    assert np.array_equal(dstb.as_array(np.uint16), lg.gather_strided_f16(src, 28, 12, 4, 5).view(np.uint16))
    assert np.abs(lb.as_array(np.float32) - lg.logit_softcap(logits, 30.0)).max() < 1e-4


def test_glue_argument_errors(pkg, gpu):
    ctx, K = gpu
    small = pkg.Buffer.empty(ctx, 64)
    batch = pkg.CommandBatch(ctx)
    with pytest.raises(pkg.InvalidArgument):
        K.rms_norm_into(batch, small, small, small, 1536, 1, 1e-6)
    with pytest.raises(pkg.InvalidArgument):
        K.rope_into(batch, small, small, 7, 0, 1e4, 1.0, 1)
    with pytest.raises(pkg.InvalidArgument):
        K.logit_softcap_gpu_into(batch, small, 30.0, 17)


@pytest.mark.parametrize("dim,rows", [(2048, 1), (512, 3), (100, 2)])
@pytest.mark.parametrize("scale", [None, 0.75])
def test_rms_norm_residual_scale_equals_the_three_kernels(pkg, gpu, dim, rows, scale):
    """One dispatch for rms_norm_into -> residual_add_into (-> scale_in_place_gpu_into), layer.rs:507-520: the same
    bits as the separate kernels, which the tests above hold to the oracle."""
    ctx, K = gpu
    g = pkg.synth.rng(77, dim + rows)
    x = (g.standard_normal(rows * dim, dtype=np.float32) * 3).astype(np.float16)
    w = (1 + 0.1 * g.standard_normal(dim, dtype=np.float32)).astype(np.float16)
    r = g.standard_normal(rows * dim, dtype=np.float32).astype(np.float16)
    xb, wb, rb = (pkg.Buffer.from_slice(ctx, a) for a in (x, w, r))
    tmp, want, got = (pkg.Buffer.empty(ctx, rows * dim * 2) for _ in range(3))
    batch = pkg.CommandBatch(ctx)
    K.rms_norm_into(batch, xb, wb, tmp, dim, rows, 1e-6)
    K.residual_add_into(batch, rb, tmp, want, rows * dim)
    if scale is not None:
        K.scale_in_place_gpu_into(batch, want, scale, rows * dim)
    K.rms_norm_residual_scale_into(batch, xb, wb, rb, got, dim, rows, 1e-6, scale)
    K.rms_norm_residual_scale_into(batch, xb, wb, rb, rb, dim, rows, 1e-6, scale)      # in place over the residual
    batch.commit_and_wait()
    assert np.array_equal(got.as_array(np.uint16), want.as_array(np.uint16))
    assert np.array_equal(rb.as_array(np.uint16), want.as_array(np.uint16))


def test_gelu_mul_strided_equals_gather_then_gelu_mul(pkg, gpu):
    """gelu_mul_strided_into against gather_strided_f16_into + gelu_mul_into, bit for bit, on the vector and scalar paths."""
    ctx, K = gpu
    g = pkg.synth.rng(44, 1)
    for rows, dim, stride, off in ((64, 256, 35 * 256, 7 * 256), (5, 24, 100, 3), (1, 256, 256, 0), (33, 40, 48, 8)):
        a_host = (g.standard_normal((rows, dim), dtype=np.float32) * 2).astype(np.float16)
        b_host = g.standard_normal(rows * stride + dim, dtype=np.float32).astype(np.float16)
        a, b = pkg.Buffer.from_slice(ctx, a_host), pkg.Buffer.from_slice(ctx, b_host)
        sl, want, got = (pkg.Buffer.empty(ctx, rows * dim * 2) for _ in range(3))
        batch = pkg.CommandBatch(ctx)
        K.gather_strided_f16_into(batch, b, sl, stride, off, dim, rows)
        K.gelu_mul_into(batch, a, sl, want, rows * dim)
        K.gelu_mul_strided_into(batch, a, b, stride, off, got, dim, rows)
        K.gelu_mul_strided_into(batch, a, b, stride, off, a, dim, rows)          # in place
        batch.commit_and_wait()
        assert np.array_equal(got.as_array(np.uint16), want.as_array(np.uint16)), (rows, dim, stride, off)
        assert np.array_equal(a.as_array(np.uint16), want.as_array(np.uint16))
    with pytest.raises(pkg.InvalidArgument):
        K.gelu_mul_strided_into(pkg.CommandBatch(ctx), a, b, stride, off + 64, got, dim, rows)     # last row past the end of b
