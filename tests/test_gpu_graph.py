"""Recorded batches: a decode step captured once into a HIP graph and replayed with new inputs and
positions must give, replay after replay, the bits of the same step issued eagerly."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _layer(pkg, ctx, g, pld=0, n_layers=1, idx=0, **kw):
    dims = dict(hidden_size=512, intermediate_size=1024, num_attention_heads=4, num_key_value_heads=1, head_dim=256)
    t = pkg.synth.decoder_layer_tensors(512, 1024, 4, 1, 256, pld, g, **kw)
    params = pkg.layer.LayerParams(layer_idx=idx, per_layer_dim=pld, **dims)
    return pkg.layer.TransformerLayer(params, pkg.layer.LayerWeights.from_host(ctx, t))


@pytest.mark.parametrize("n_lanes", [1, 3, 40])
def test_captured_decode_step_replays_like_eager(pkg, gpu, n_lanes):
    ctx, K = gpu
    g = pkg.synth.rng(950, n_lanes)
    pld, n_layers, lane_cap = 256, 2, 64
    layers = [_layer(pkg, ctx, g, pld, n_layers, i, output_scale=0.5 + 0.25 * i) for i in range(n_layers)]
    pools = [[pkg.QuantizedUnifiedKvPool(ctx, n_lanes, lane_cap, 1, 256, 2, 0) for _ in range(n_layers)] for _ in range(2)]
    for side in pools:
        for p in side:
            p.reset()
    bs = pkg.layer.BatchScratch(ctx, n_lanes, 512, 1024, 4, 1, 256, pld, n_layers)
    ones = pkg.Buffer.from_slice(ctx, np.ones(256, np.float16))
    xin = pkg.Buffer.empty(ctx, n_lanes * 1024)
    ple = pkg.Buffer.empty(ctx, n_lanes * n_layers * pld * 2)
    pos_buf = pkg.Buffer.empty(ctx, n_lanes * 4)
    outs = [pkg.Buffer.empty(ctx, n_lanes * 1024) for _ in range(2)]
    mids = [pkg.Buffer.empty(ctx, n_lanes * 1024) for _ in range(2)]

    def encode(batch, side):
        layers[0].forward_decode_batch_turbo(batch, K, n_lanes, pos_buf, xin, mids[side], bs, ones, pools[side][0], (ple, n_layers))
        layers[1].forward_decode_batch_turbo(batch, K, n_lanes, pos_buf, mids[side], outs[side], bs, ones, pools[side][1],
                                             (ple, n_layers))

    batch = pkg.CommandBatch(ctx)
    batch.begin_capture()
    encode(batch, 0)
    graph = batch.end_capture()
    assert graph.dispatch_count() >= 16          # two layers of 8 - 10 encoded steps each
    ctx.synchronize()
    assert not outs[0].as_array(np.uint16).any()          # recording runs nothing

    positions = (np.arange(n_lanes, dtype=np.uint32) * 5) % 23
    for step in range(7):
        xin.copy_from_bytes(g.standard_normal(n_lanes * 512, dtype=np.float32).astype(np.float16))
        ple.copy_from_bytes(g.standard_normal(n_lanes * n_layers * pld, dtype=np.float32).astype(np.float16))
        pos_buf.copy_from_bytes(positions)
        graph.launch()
        ctx.synchronize()
        got = outs[0].as_array(np.uint16)
        eager = pkg.CommandBatch(ctx)
        encode(eager, 1)
        eager.commit_and_wait()
        want = outs[1].as_array(np.uint16)
        assert np.isfinite(want.view(np.float16).astype(np.float32)).all() and want.any()
        assert np.array_equal(got, want), f"replay {step}"
        for a, b in zip(pools[0], pools[1]):
            assert np.array_equal(a.keys_q.as_array(np.uint8), b.keys_q.as_array(np.uint8))
            assert np.array_equal(a.value_norms.as_array(np.uint16), b.value_norms.as_array(np.uint16))
        positions += 1


def test_capture_refuses_what_a_graph_cannot_hold(pkg, gpu):
    ctx, K = gpu
    buf = pkg.Buffer.empty(ctx, 256)
    a, b = pkg.Buffer.from_slice(ctx, np.ones(64, np.float16)), pkg.Buffer.from_slice(ctx, np.ones(64, np.float16))
    batch = pkg.CommandBatch(ctx)
    batch.begin_capture()
    try:
        with pytest.raises(pkg.InvalidArgument):
            pkg.CommandBatch(ctx).begin_capture()
        with pytest.raises(pkg.InvalidArgument):
            pkg.Buffer.empty(ctx, 16)
        with pytest.raises(pkg.InvalidArgument):
            pkg.Buffer.from_slice(ctx, np.zeros(4, np.float32))
        with pytest.raises(pkg.InvalidArgument):
            buf.as_array(np.uint8)
        with pytest.raises(pkg.InvalidArgument):
            buf.copy_from_bytes(np.zeros(4, np.uint8))
        with pytest.raises(pkg.InvalidArgument):
            buf.fill_zero()
        with pytest.raises(pkg.InvalidArgument):
            batch.commit_and_wait()
        with pytest.raises(pkg.InvalidArgument):
            ctx.synchronize()
        K.residual_add_into(batch, a, b, buf, 64)
    finally:
        graph = batch.end_capture()
    with pytest.raises(pkg.InvalidArgument):
        batch.end_capture()
    assert graph.dispatch_count() == 1
    assert not buf.as_array(np.uint16, 64).any()
    graph.launch()
    ctx.synchronize()
    assert (buf.as_array(np.float16, 64) == 2.0).all()
    graph.free()
    assert pkg.Buffer.empty(ctx, 16).length() == 16       # the context is usable again


def test_buffer_released_during_capture_lives_as_long_as_the_graph(pkg, gpu):
    """A scratch buffer that a recorded dispatch writes and a later one reads is released by its owner while the
    capture is still open (as a Rust scope would drop it).  The graph keeps the allocation: several replays, with
    other allocations made in between (which would reuse a freed block), still give the right sums."""
    ctx, K = gpu
    n = 4096
    a = pkg.Buffer.from_slice(ctx, np.full(n, 1.5, np.float16))
    b = pkg.Buffer.from_slice(ctx, np.full(n, 2.0, np.float16))
    out = pkg.Buffer.empty(ctx, n * 2)
    scratch = pkg.Buffer.empty(ctx, n * 2)          # created before the capture: allocation is refused inside one
    batch = pkg.CommandBatch(ctx)
    batch.begin_capture()
    K.residual_add_into(batch, a, b, scratch, n)          # scratch = a + b
    K.residual_add_into(batch, scratch, b, out, n)        # out = scratch + b
    scratch.free()                                         # dropped while the capture is open
    graph = batch.end_capture()
    filler = []
    for step in range(4):
        # allocations of the same size between replays: a block freed too early would be handed out here and overwritten
        filler.append(pkg.Buffer.from_slice(ctx, np.full(n, 100.0 + step, np.float16)))
        a.copy_from_bytes(np.full(n, 1.5 + step, np.float16))
        out.fill_zero()
        graph.launch()
        ctx.synchronize()
        got = out.as_array(np.float16, n).astype(np.float32)
        assert (got == 1.5 + step + 4.0).all(), f"replay {step}: {got[:4]}"
    graph.free()
