"""Continuous batching end to end on the GPU (local-engine/src/pipeline/batched.rs:72-478): lanes prefilled through the
chunked batch path and copied into by-lane pools, then decoded together at their own positions, each lane against
the oracle's single-sequence composition of the same steps.

As in the single-sequence test the cache rows the GPU wrote are handed to the oracle after every token (a 2-bit code
flips when its input sits within an f16 ulp of a quantiser boundary), the oracle's own codes may differ from them in
at most 1 % of the fields, and the logits are held to 0.08 absolute and 0.01 on average.  The lane-isolation checks
follow batched.rs:604-637: lanes fed the same token give bit-identical logits, and reversing the lanes reverses the
results."""
import numpy as np
import pytest

from oracle import layer as OL

pytestmark = pytest.mark.gpu

WORST, MEAN = 0.08, 0.01


def _config(pkg, pld=64, head_dims=(128, 256)):
    types = ["sliding_attention", "sliding_attention", "full_attention", "sliding_attention", "sliding_attention",
             "full_attention"]
    return pkg.pipeline.Gemma4QATConfig(vocab_size=640, hidden_size=512, num_hidden_layers=6, num_attention_heads=4,
                                        num_key_value_heads=1, head_dim=head_dims[0], global_head_dim=head_dims[1], sliding_window=16,
                                        num_kv_shared_layers=3, hidden_size_per_layer_input=pld, layer_types=types,
                                        sliding_rope_theta=10000.0, full_rope_theta=1000000.0,
                                        full_partial_rotary_factor=0.25)


def _pipe(pkg, gpu, pld=64, seed=0, max_batch=8, max_ctx=1024, head_dims=(128, 256), **layer_options):
    ctx, K = gpu
    cfg = _config(pkg, pld, head_dims)
    g = pkg.synth.rng(981, seed)
    t = pkg.synth.decode_model_tensors(cfg, g, [512, 512, 512, 1024, 1024, 1024])
    pipe = pkg.pipeline.DecodePipeline.from_host(ctx, K, cfg, t, max_ctx, max_batch=max_batch, **layer_options)
    return cfg, g, pipe, OL.model_from_host(cfg, t)


def _pool_row(pool, kv, lane, pos):
    """The (K codes, K norms, V codes, V norms) the GPU holds for `lane` at `pos`."""
    cs, ns = kv.row_slices(pos)                       # within one lane; a lane starts lane_stride rows further on
    cb = (cs.stop - cs.start) // (ns.stop - ns.start)
    row0 = lane * pool.lane_stride() * pool.n_kv_heads
    c0, n0 = row0 * cb + cs.start, row0 + ns.start
    nc, nn = cs.stop - cs.start, ns.stop - ns.start
    return (pool.keys_q.as_array(np.uint8, nc, c0), pool.key_norms.as_array(np.uint16, nn, n0 * 2),
            pool.values_q.as_array(np.uint8, nc, c0), pool.value_norms.as_array(np.uint16, nn, n0 * 2))


def _oracle_token(cfg, pipe, state, model, kvs, lane, tok, pos, overwritten=lambda slot: False, max_flips=0.01):
    """The oracle's logits for `tok` at `pos` of `lane`, fed the cache rows the GPU wrote for that position (a slot for
    which `overwritten` holds no longer has them -- a ring that has wrapped past the position -- and the oracle keeps its own)."""
    rows = []
    for i in range(cfg.num_hidden_layers):
        slot = pipe.kv_index_map[i]
        gone = cfg.is_kv_shared(i) or overwritten(slot)
        rows.append(None if gone else _pool_row(state.pools[slot], kvs[slot], lane, pos))
    tr = {}
    want = OL.decode_token(model, tok, pos, kvs, rows, tr)
    assert max(tr["code_flips"], default=0.0) <= max_flips, f"lane {lane} position {pos}: code flips {tr['code_flips']}"
    return want


def _close(got, want, what):
    d = np.abs(got - want)
    assert np.isfinite(got).all() and d.max() <= WORST and d.mean() <= MEAN, f"{what}: worst {d.max():.4g} mean {d.mean():.4g}"
    assert want[int(np.argmax(got))] >= want.max() - 2 * WORST, what


@pytest.mark.parametrize("pld,n_lanes,head_dims", [(64, 4, (128, 256)), (0, 4, (128, 256)), (64, 24, (128, 256)), (64, 20, (256, 512))])
def test_prefilled_lanes_decode_together(pkg, gpu, oracle, pld, n_lanes, head_dims):
    """4 lanes: every product runs as matvecs over the rows (exact integer arithmetic, at most 1 % of a row's codes differ
    from the oracle's).  24 lanes: the decode-batch matrix-core kernel with its fused tail (f16-rounded weights and
    activations; up to 3 %).  Head dims 256 / 512 are the reference model's: both attention layer kinds then run on the
    matrix-core attention kernel (128 takes the vector-ALU one)."""
    few = n_lanes <= 8
    cfg, g, pipe, model = _pipe(pkg, gpu, pld, seed=pld + n_lanes, max_batch=8 if few else 32, head_dims=head_dims)
    lane_cap, flips = 1024, 0.01 if few else 0.03
    state = pipe.new_batched_decode_state(n_lanes, lane_cap)
    assert len(state.pools) == len(pipe.kv_caches) == 3
    assert [p.lane_ring_capacity for p in state.pools] == [c.physical_positions if c.is_ringed() else 0 for c in pipe.kv_caches]
    kvs = [[OL.KvState(1, c.head_dim, 2, lane_cap, ring_capacity=c.ring_capacity()) for c in pipe.kv_caches]
           for _ in range(n_lanes)]
    # the other lanes start empty; lane 1 holds a short prompt, lane 2 one longer than the sliding window
    prompts = {1: [int(v) for v in g.integers(0, cfg.vocab_size, 5)], 2: [int(v) for v in g.integers(0, cfg.vocab_size, 21)]}
    positions = [0] * n_lanes
    for lane, prompt in prompts.items():
        got = pipe.prefill_lane(state, lane, prompt)
        for pos, tok in enumerate(prompt):
            want = _oracle_token(cfg, pipe, state, model, kvs[lane], lane, tok, pos, max_flips=flips)
        _close(got, want, f"prefill of lane {lane}")
        positions[lane] = len(prompt)
    for step in range(6):
        tokens = [int(v) for v in g.integers(0, cfg.vocab_size, n_lanes)]
        got = pipe.decode_batch_step(state, tokens, tokens, positions)
        assert got.shape == (n_lanes, cfg.vocab_size) and np.abs(got).max() <= 30.0 + 1e-3
        for lane in range(n_lanes):
            want = _oracle_token(cfg, pipe, state, model, kvs[lane], lane, tokens[lane], positions[lane], max_flips=flips)
            _close(got[lane], want, f"step {step} lane {lane} position {positions[lane]}")
        positions = [p + 1 for p in positions]
    # a lane taken out of service and reused: its rows are cleared and it decodes like a fresh sequence
    state.reset_lane(2)
    kvs[2] = [OL.KvState(1, c.head_dim, 2, lane_cap, ring_capacity=c.ring_capacity()) for c in pipe.kv_caches]
    positions[2] = 0
    tokens = [int(v) for v in g.integers(0, cfg.vocab_size, 3)]
    got = pipe.decode_batch_step(state, tokens, tokens, positions[:3])          # fewer active lanes than the state holds
    for lane in range(3):
        want = _oracle_token(cfg, pipe, state, model, kvs[lane], lane, tokens[lane], positions[lane])
        _close(got[lane], want, f"after reset lane {lane}")


def test_prompt_longer_than_the_ring_then_lanes_decode(pkg, gpu, oracle):
    """A prompt longer than the sliding-window ring (512 slots for this window): the chunked prefill wraps the staging
    rings (pipeline.rs:1332-1367, quant_cache.rs:266-274), the wrapped rings are copied slot for slot into the lane
    (quant_unified_pool.rs:269-315) and batched steps carry on past them, next to a lane that starts empty.  Positions
    whose ring slot has been overwritten by the time the lane is read back are outside every later sliding window; the
    oracle keeps its own codes for them."""
    cfg, g, pipe, model = _pipe(pkg, gpu, 64, seed=21, max_batch=256)
    ring = pipe.kv_caches[0].physical_positions
    n_prompt, n_lanes, lane_cap = ring + 29, 2, 1024
    assert pipe.kv_caches[0].is_ringed() and not pipe.kv_caches[2].is_ringed()
    state = pipe.new_batched_decode_state(n_lanes, lane_cap)
    kvs = [[OL.KvState(1, c.head_dim, 2, lane_cap, ring_capacity=c.ring_capacity()) for c in pipe.kv_caches]
           for _ in range(n_lanes)]
    prompt = [int(v) for v in g.integers(0, cfg.vocab_size, n_prompt)]
    got = pipe.prefill_lane(state, 1, prompt)
    for pos, tok in enumerate(prompt):
        # 256-row chunks go through the f16 matrix-core products (f16-rounded weights and activations, where the matvec
        # kernels and the oracle keep f32): K and V sit a little further from the oracle's and up to 3 % of a row's
        # codes land on the other side of a quantiser boundary
        want = _oracle_token(cfg, pipe, state, model, kvs[1], 1, tok, pos, max_flips=0.03,
                             overwritten=lambda slot: pipe.kv_caches[slot].is_ringed() and pos + ring < n_prompt)
    _close(got, want, "prefill past the ring")
    positions = [0, n_prompt]
    for step in range(4):
        tokens = [int(v) for v in g.integers(0, cfg.vocab_size, n_lanes)]
        got = pipe.decode_batch_step(state, tokens, tokens, positions)
        for lane in range(n_lanes):
            want = _oracle_token(cfg, pipe, state, model, kvs[lane], lane, tokens[lane], positions[lane])
            _close(got[lane], want, f"step {step} lane {lane} position {positions[lane]}")
        positions = [p + 1 for p in positions]


def test_batched_step_matches_single_sequence_at_pos0(pkg, gpu):
    """batched.rs:530-640 with the single-sequence pipeline as the yardstick."""
    cfg, g, pipe, _ = _pipe(pkg, gpu, seed=3)
    tokens = [2, 100, 333, 639]
    single = []
    for tok in tokens:
        pipe.reset()
        pipe.decode_step(tok)
        single.append(pipe.logits().copy())
    state = pipe.new_batched_decode_state(len(tokens), 1024)
    zeros = [0] * len(tokens)
    got = pipe.decode_batch_step(state, tokens, tokens, zeros)
    for lane, want in enumerate(single):          # M = 1 kernels against the M = n kernels: same envelope as against the oracle
        _close(got[lane], want, f"lane {lane}")
    dup = pipe.decode_batch_step(state, [tokens[0]] * 4, [tokens[0]] * 4, zeros)
    for lane in range(1, 4):
        assert np.array_equal(dup[lane], dup[0]), f"lane {lane} differs from lane 0 on the same token"
    rev = pipe.decode_batch_step(state, tokens[::-1], tokens[::-1], zeros)
    for lane in range(4):                          # results follow the token, not the lane index
        assert np.array_equal(rev[lane], got[3 - lane])


@pytest.mark.parametrize("pld,lanes", [(64, 40), (0, 24), (64, 5)])
def test_fused_tail_equals_separate_kernels(pkg, gpu, pld, lanes):
    """The fused steps of the multi-row layer tail (product + norm + residual (+ scale) (+ the next layer's attention
    norm), the per-layer-input gate read in place) against the reference's kernel-by-kernel sequence: the same logits bit
    for bit, for a prefilled lane and for batched steps -- a decode batch whose products take the direct-to-MFMA kernel
    and one small enough to run as matvecs."""
    runs = []
    for fused in (True, False):
        cfg, g, pipe, _ = _pipe(pkg, gpu, pld, seed=11, max_batch=64, fuse_norm_chain=fused)
        state = pipe.new_batched_decode_state(lanes, 1024)
        out = [pipe.prefill_lane(state, 1, [int(v) for v in g.integers(0, cfg.vocab_size, 19)])]
        positions = [0] * lanes
        positions[1] = 19
        for _ in range(3):
            tokens = [int(v) for v in g.integers(0, cfg.vocab_size, lanes)]
            out.append(pipe.decode_batch_step(state, tokens, tokens, positions))
            positions = [p + 1 for p in positions]
        runs.append(out)
    for a, b in zip(*runs):
        assert np.array_equal(a, b)


def test_batched_step_arguments(pkg, gpu):
    cfg, g, pipe, _ = _pipe(pkg, gpu, seed=4)
    with pytest.raises(pkg.InvalidArgument):
        pipe.new_batched_decode_state(0, 1024)
    with pytest.raises(pkg.InvalidArgument):
        pipe.new_batched_decode_state(9, 1024)                     # more lanes than the batch scratch has rows
    with pytest.raises(pkg.InvalidArgument):
        pipe.new_batched_decode_state(2, 8)                        # below the sliding-window ring
    state = pipe.new_batched_decode_state(2, 600)
    with pytest.raises(pkg.InvalidArgument):
        pipe.decode_batch_step(state, [], [], [])
    with pytest.raises(pkg.InvalidArgument):
        pipe.decode_batch_step(state, [1, 2, 3], [1, 2, 3], [0, 0, 0])
    with pytest.raises(pkg.InvalidArgument):
        pipe.decode_batch_step(state, [1, 2], [1], [0, 0])
    with pytest.raises(pkg.InvalidArgument):
        pipe.decode_batch_step(state, [1, 2], [1, 2], [0, 600])
    with pytest.raises(pkg.InvalidArgument):
        pipe.prefill_lane(state, 2, [1])
    with pytest.raises(pkg.InvalidArgument):
        pipe.prefill_lane(state, 0, [])
    with pytest.raises(pkg.InvalidArgument):
        pipe.prefill_lane(state, 0, [1] * 601)
    with pytest.raises(pkg.InvalidArgument):
        pipe.forward_tokens_batch([1] * 9, 0)
