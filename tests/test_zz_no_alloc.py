"""The attention entry that allocates nothing (lh_flash_attention_tq_static_into: split partials in a static device
array) against the ordinary entry (lh_flash_attention_tq_into: partials in the context workspace), through the C ABI:
two calls in a row, the second over a smaller input, so that records left behind by the first call lie in the array
while the second runs.  Same kernels and -- for these shapes -- the same split count, so the outputs must agree bit for
bit: the split count is chosen from the work and only lowered when the records would not fit, and the static array
(2 Mi floats) holds the 256 splits a single query gets at most here for 8 heads of 512 dims (256 x 8 x 516 floats), as
the workspace does.  Both are also held to the f64 code-space oracle at the attention tolerance.  A last test reads the
device's free memory around a series of calls: the entry must not allocate."""
import numpy as np
import pytest

from test_gpu_attention import ATTN_TOL, build_cache, check, upload

pytestmark = pytest.mark.gpu


def run_pair(pkg, gpu, oracle, hd, nq, nkv, T, bits, window, ring, seed):
    ctx, K = gpu
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, seed, ring=ring)
    rq = pkg.synth.rng(6, seed).standard_normal((nq, hd), dtype=np.float32) * np.float32(0.5)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    outs = [pkg.Buffer.from_slice(ctx, np.full(nq * hd, 7.0, np.float32)) for _ in range(2)]
    batch = pkg.CommandBatch(ctx)
    K.flash_attention_tq_into(batch, rqb, kcb, knb, vcb, vnb, lvb, outs[0], hd, T, T - 1, nq, nkv, window, bits, ring)
    K.flash_attention_tq_static_into(batch, rqb, kcb, knb, vcb, vnb, lvb, outs[1], hd, T, T - 1, nq, nkv, window, bits, ring)
    batch.commit_and_wait()
    a, b = outs[0].as_array(np.float32), outs[1].as_array(np.float32)
    ref = oracle.attention_tq_codespace(rq, kc, kn, vc, vn, levels, hd, T, T - 1, nq, nkv, window, bits, ring)
    check(b, ref, f"static entry T={T} hd={hd}")
    check(a, ref, f"ordinary entry T={T} hd={hd}")
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"T={T}: {int((a != b).sum())} of {a.size} outputs differ"


def test_static_entry_matches_ordinary_entry_twice(pkg, gpu, oracle):
    print("case static attention: 32768 positions, then 700", flush=True)
    run_pair(pkg, gpu, oracle, 256, 8, 1, 32768, 2, 0, 0, 11)      # many splits: fills a large part of the array
    run_pair(pkg, gpu, oracle, 256, 8, 1, 700, 2, 0, 0, 12)        # fewer, shorter splits over the same array
    run_pair(pkg, gpu, oracle, 256, 8, 1, 40, 2, 0, 0, 13)         # a single split: the array is not used at all
    run_pair(pkg, gpu, oracle, 128, 4, 2, 300, 4, 64, 0, 14)       # vector-ALU kernel, window
    run_pair(pkg, gpu, oracle, 512, 8, 1, 3000, 2, 512, 512, 15)   # head_dim 512 over a wrapped ring


def test_static_entry_rejects_oversized_shapes(pkg, gpu):
    ctx, K = gpu
    b = pkg.Buffer.empty(ctx, 1 << 20)
    batch = pkg.CommandBatch(ctx)
    with pytest.raises(pkg.InvalidArgument, match=r"flash_attention_tq_static: num_q_heads 32 x \(head_dim 512 \+ 4\) exceeds 8192"):
        K.flash_attention_tq_static_into(batch, b, b, b, b, b, b, b, 512, 16, 15, 32, 1, 0, 2, 0)
    assert batch.dispatch_count() == 0


def test_static_entry_allocates_nothing(pkg, gpu, oracle):
    """hipMemGetInfo's free bytes before and after twenty calls of the entry (after one warm-up call, which may load
    the kernels' code): unchanged."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    ctx, K = gpu
    hd, nq, nkv, T, bits = 256, 8, 1, 4096, 2
    signs, levels, kc, kn, vc, vn = build_cache(pkg, oracle, T, nkv, hd, bits, 21)
    rq = pkg.synth.rng(6, 21).standard_normal((nq, hd), dtype=np.float32)
    kcb, knb, vcb, vnb, lvb, rqb = upload(pkg, ctx, kc, kn, vc, vn, levels, rq)
    out = pkg.Buffer.empty(ctx, nq * hd * 4)
    batch = pkg.CommandBatch(ctx)

    def free_bytes():
        free, total = C.c_size_t(0), C.c_size_t(0)
        assert hip.hipMemGetInfo(C.byref(free), C.byref(total)) == 0
        return free.value

    K.flash_attention_tq_static_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, T - 1, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    before = free_bytes()
    for _ in range(20):
        K.flash_attention_tq_static_into(batch, rqb, kcb, knb, vcb, vnb, lvb, out, hd, T, T - 1, nq, nkv, 0, bits, 0)
    batch.commit_and_wait()
    assert free_bytes() == before
