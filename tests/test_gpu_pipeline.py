"""The decode core of the token loop (local-engine/src/pipeline.rs:714-953) end to end on the GPU -- embedding gather
and scale, per-layer inputs, a stack of sliding-window, full-attention and KV-shared layers over ringed and absolute
caches, output norm, tied-embedding logits, soft cap -- against the oracle's composition of the same steps.

After each token the cache rows the GPU wrote are handed to the oracle (a 2-bit code flips when its input sits within
an f16 ulp of a quantiser boundary); the oracle's own codes for that row may differ from them in at most 1 % of the
fields, and the logits -- O(10) before the soft cap at 30 -- are held to 0.08 absolute and 0.01 on average."""
import numpy as np
import pytest

from oracle import layer as OL

pytestmark = pytest.mark.gpu


def _config(pkg, pld, head_dims=(128, 256)):
    types = ["sliding_attention", "sliding_attention", "full_attention", "sliding_attention", "sliding_attention",
             "full_attention"]
    return pkg.pipeline.Gemma4QATConfig(vocab_size=640, hidden_size=512, num_hidden_layers=6, num_attention_heads=4,
                                        num_key_value_heads=1, head_dim=head_dims[0], global_head_dim=head_dims[1], sliding_window=16,
                                        num_kv_shared_layers=3, hidden_size_per_layer_input=pld, layer_types=types,
                                        sliding_rope_theta=10000.0, full_rope_theta=1000000.0,
                                        full_partial_rotary_factor=0.25)


@pytest.mark.parametrize("pld,fused,head_dims,defer", [
    (64, True, (128, 256), True), (0, True, (128, 256), True), (64, False, (128, 256), True),
    (64, True, (256, 512), True),      # the reference model's head dims
    (64, True, (128, 256), False)])    # every layer runs its own last step (by default it rides in the next layer's first dispatch)
def test_decode_steps_match_oracle(pkg, gpu, oracle, pld, fused, head_dims, defer):
    ctx, K = gpu
    cfg = _config(pkg, pld, head_dims)
    g = pkg.synth.rng(970, pld)
    inters = [512, 512, 512, 1024, 1024, 1024]          # later layers double-wide, as in the reference model
    t = pkg.synth.decode_model_tensors(cfg, g, inters)
    options = {} if fused else dict(group_projections=False, fuse_norm_rope=False, fuse_prologues=False, stack_qkv=False)
    max_ctx = 1024
    pipe = pkg.pipeline.DecodePipeline.from_host(ctx, K, cfg, t, max_ctx, **options)
    pipe.defer_layer_tails = defer
    assert pipe.kv_index_map == [0, 1, 2, 1, 1, 2] and len(pipe.kv_caches) == 3
    assert [c.is_ringed() for c in pipe.kv_caches] == [True, True, False]
    model = OL.model_from_host(cfg, t)
    assert model.kv_index_map == pipe.kv_index_map
    kvs = [OL.KvState(1, c.head_dim, 2, max_ctx, ring_capacity=c.ring_capacity()) for c in pipe.kv_caches]
    tokens = [int(v) for v in g.integers(0, cfg.vocab_size, 24)]
    greedy_agree = 0
    for pos, tok in enumerate(tokens):
        pipe.decode_step(tok)
        got = pipe.logits()
        assert pipe.position == pos + 1 and np.isfinite(got).all()
        rows = []
        for i in range(cfg.num_hidden_layers):
            if cfg.is_kv_shared(i):
                rows.append(None)
                continue
            cache, kv = pipe.kv_caches[pipe.kv_index_map[i]], kvs[pipe.kv_index_map[i]]
            cs, ns = kv.row_slices(pos)
            rows.append((cache.keys_q.as_array(np.uint8, cs.stop - cs.start, cs.start),
                         cache.key_norms.as_array(np.uint16, ns.stop - ns.start, ns.start * 2),
                         cache.values_q.as_array(np.uint8, cs.stop - cs.start, cs.start),
                         cache.value_norms.as_array(np.uint16, ns.stop - ns.start, ns.start * 2)))
        tr = {}
        want = OL.decode_token(model, tok, pos, kvs, rows, tr)
        assert max(tr["code_flips"]) <= 0.01, f"position {pos}: code flips {tr['code_flips']}"
        d = np.abs(got - want)
        assert d.max() <= 0.08 and d.mean() <= 0.01, f"position {pos}: worst {d.max():.4g} mean {d.mean():.4g}"
        assert np.abs(got).max() <= 30.0 + 1e-3                      # soft cap
        # the GPU's greedy token is the oracle's, or one the oracle ranks within twice the tolerance of its best
        assert want[int(np.argmax(got))] >= want.max() - 0.16
        greedy_agree += int(np.argmax(got)) == int(np.argmax(want))
    assert greedy_agree >= len(tokens) * 3 // 4
    pipe.reset()
    assert pipe.position == 0 and not pipe.kv_caches[0].keys_q.as_array(np.uint8).any()
    with pytest.raises(pkg.InvalidArgument):
        pipe.forward_token(1, max_ctx)
