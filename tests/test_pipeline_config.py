"""CPU checks of the decode pipeline's configuration helpers against the reference's own tests
(local-core/src/config/gemma4_qat.rs:262-345) and of the cache-slot map (local-engine/src/pipeline.rs:379-437)."""
import __graft_entry__ as ge


def _e2b(pkg):
    types = ["full_attention" if i % 5 == 4 else "sliding_attention" for i in range(35)]
    return pkg.pipeline.Gemma4QATConfig(vocab_size=262144, hidden_size=1536, num_hidden_layers=35, num_attention_heads=8,
                                        num_key_value_heads=1, head_dim=256, global_head_dim=512,
                                        max_position_embeddings=131072, rms_norm_eps=1e-6, sliding_window=512,
                                        num_kv_shared_layers=20, hidden_size_per_layer_input=256, layer_types=types,
                                        sliding_rope_theta=10000.0, full_rope_theta=1000000.0,
                                        full_partial_rotary_factor=0.25)


def test_kv_sharing_maps_shared_layers_to_same_type_source():
    """gemma4_qat.rs:285-305."""
    cfg = _e2b(ge.load_package())
    assert cfg.first_kv_shared_layer() == 15
    for i in range(15):
        assert not cfg.is_kv_shared(i) and cfg.kv_source_layer(i) is None
    for i in (19, 24, 29, 34):
        assert cfg.is_kv_shared(i) and cfg.kv_source_layer(i) == 14
    for i in (15, 16, 17, 18, 20, 23, 33):
        assert cfg.is_kv_shared(i) and cfg.kv_source_layer(i) == 13


def test_layer_geometry_by_attention_type():
    """gemma4_qat.rs:307-345: head dims, rope bases and the proportional partial rotary of full-attention layers."""
    cfg = _e2b(ge.load_package())
    assert cfg.is_full_attention(4) and not cfg.is_full_attention(0) and not cfg.is_full_attention(99)
    assert cfg.attn_head_dim(4) == 512 and cfg.attn_head_dim(0) == 256
    assert cfg.rope_theta(4) == 1000000.0 and cfg.rope_theta(0) == 10000.0
    assert abs(cfg.partial_rotary_factor(4) - 0.25) < 1e-6 and cfg.partial_rotary_factor(0) == 1.0
    plain = ge.load_package().pipeline.Gemma4QATConfig(vocab_size=8, hidden_size=8, num_hidden_layers=2, num_attention_heads=1,
                                                       num_key_value_heads=1, head_dim=64, layer_types=["full_attention"])
    assert plain.rope_theta(0) == 10000.0 and plain.partial_rotary_factor(0) == 1.0 and plain.attn_head_dim(0) == 64
    assert not plain.is_kv_shared(1)


def test_oracle_cache_slot_map_matches_sharing_rule():
    """The oracle's layer -> slot map (15 slots; shared layers point at layers 13 / 14's slots)."""
    import numpy as np
    from oracle import layer as OL
    pkg = ge.load_package()
    cfg = _e2b(pkg)
    small = pkg.pipeline.Gemma4QATConfig(vocab_size=64, hidden_size=256, num_hidden_layers=35, num_attention_heads=2,
                                         num_key_value_heads=1, head_dim=128, global_head_dim=256, sliding_window=16,
                                         num_kv_shared_layers=20, layer_types=cfg.layer_types)
    t = pkg.synth.decode_model_tensors(small, pkg.synth.rng(5, 5), 256, attn_fmt="q4_0", ffn_fmt="q4_0", table_rows=64)
    m = OL.model_from_host(small, t)
    assert m.kv_index_map[:15] == list(range(15))
    assert all(m.kv_index_map[i] == 14 for i in (19, 24, 29, 34))
    assert all(m.kv_index_map[i] == 13 for i in (15, 16, 17, 18, 20, 23, 33))
    assert [l.head_dim for l in m.layers[:5]] == [128, 128, 128, 128, 256]
    assert m.layers[19].is_kv_shared and m.layers[19].attn_k is None and m.layers[14].attn_k is not None
