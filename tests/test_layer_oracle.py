"""CPU pins of the decoder-layer composition in oracle/layer.py (local-engine/src/layer.rs:354-523):
closed-form consequences of the layer's wiring that a wrong residual, a skipped norm or a swapped
operand would break."""
import numpy as np
import pytest

from oracle import layer as OL
from oracle import layer_glue as G
from oracle import oracle as O

DIMS = dict(hidden_size=256, intermediate_size=512, num_attention_heads=2, num_key_value_heads=1, head_dim=128)


def _synth():
    import __graft_entry__ as ge
    return ge.load_package().synth


def _tensors(g, **kw):
    return _synth().decoder_layer_tensors(DIMS["hidden_size"], DIMS["intermediate_size"], DIMS["num_attention_heads"],
                                          DIMS["num_key_value_heads"], DIMS["head_dim"], kw.pop("per_layer_dim", 0), g,
                                          **kw)


def _zeroed(t):
    fmt, rows, cols, payload = t
    return (fmt, rows, cols, np.zeros_like(payload))      # all-zero blocks: d = 0, every weight 0


def _kv():
    return OL.KvState(n_kv=1, head_dim=128, bits=2, max_positions=16)


@pytest.fixture(scope="module")
def x(oracle):
    return _synth().rng(77, 0).standard_normal(256, dtype=np.float32).astype(np.float16)


def test_zero_output_and_down_projections_pass_the_input_through(oracle, x):
    """rms_norm(0) * w + residual = residual, twice: the layer returns its input bit for bit."""
    t = _tensors(_synth().rng(77, 1))
    t["attn_output"], t["ffn_down"] = _zeroed(t["attn_output"]), _zeroed(t["ffn_down"])
    out = OL.decode_layer(OL.Layer.from_host(t, **DIMS), x, 3, _kv())
    assert np.array_equal(out.view(np.uint16), x.view(np.uint16))


def test_zero_per_layer_projection_is_identity_and_scale_halves(oracle, x):
    g = _synth().rng(77, 2)
    t = _tensors(g, per_layer_dim=128)
    ple = g.standard_normal(4 * 128, dtype=np.float32).astype(np.float16)
    plain = {k: v for k, v in t.items() if not k.startswith("per_layer")}
    base = OL.decode_layer(OL.Layer.from_host(plain, **DIMS), x, 0, _kv())
    t0 = dict(t)
    t0["per_layer_proj"] = _zeroed(t["per_layer_proj"])
    same = OL.decode_layer(OL.Layer.from_host(t0, per_layer_dim=128, layer_idx=2, **DIMS), x, 0, _kv(), ple)
    assert np.array_equal(same.view(np.uint16), base.view(np.uint16))
    moved = OL.decode_layer(OL.Layer.from_host(t, per_layer_dim=128, layer_idx=2, **DIMS), x, 0, _kv(), ple)
    assert not np.array_equal(moved.view(np.uint16), base.view(np.uint16))
    # the injection reads layer 2's slice: another layer's slice gives another result
    other = OL.decode_layer(OL.Layer.from_host(t, per_layer_dim=128, layer_idx=1, **DIMS), x, 0, _kv(), ple)
    assert not np.array_equal(other.view(np.uint16), moved.view(np.uint16))
    plain["layer_output_scale"] = np.array([0.5], np.float16)
    halved = OL.decode_layer(OL.Layer.from_host(plain, **DIMS), x, 0, _kv())
    assert np.array_equal(halved.astype(np.float32), base.astype(np.float32) * np.float32(0.5))


def test_kv_rows_written_are_the_normalised_rotated_projections(oracle, x):
    """K = rope(qk_norm(Wk n)), V = rms_norm_1(Wv n) with n = rms_norm(x) * attn_norm, encoded at `position`."""
    t = _tensors(_synth().rng(77, 3))
    L = OL.Layer.from_host(t, **DIMS)
    kv, pos = _kv(), 5
    OL.decode_layer(L, x, pos, kv)
    n = G.rms_norm(x, t["attn_norm"], 256, 1, 1e-6)
    k = G.rope(G.qk_norm(L.attn_k.matvec(n), t["k_norm"], 128, 1, 1e-6), 128, pos, 10000.0, 1.0, 1)
    v = G.rms_norm(L.attn_v.matvec(n), np.ones(128, np.float16), 128, 1, 1e-6)
    want = _kv()
    want.write(k, v, pos)
    for name in ("k_codes", "v_codes", "k_norms", "v_norms"):
        assert np.array_equal(getattr(kv, name), getattr(want, name)), name
    cb = O.tq_code_bytes(128, 2)
    assert kv.k_codes[pos * cb:(pos + 1) * cb].any() and not kv.k_codes[:pos * cb].any()


def test_first_token_attends_only_itself(oracle, x):
    """At position 0 softmax over one key is 1, so attention returns V's decoded row whatever q is."""
    t = _tensors(_synth().rng(77, 4))
    L = OL.Layer.from_host(t, **DIMS)
    kv = _kv()
    OL.decode_layer(L, x, 0, kv)
    q = _synth().rng(77, 5).standard_normal(256, dtype=np.float32).astype(np.float16)
    got = kv.attend(q, 1, 0, 2, 0).astype(np.float32).reshape(2, 128)
    v0 = O.tq_decode(kv.v_codes[:O.tq_code_bytes(128, 2)], kv.v_norms[0], 128, 2, kv.signs, kv.levels)
    assert np.abs(got - v0[None, :]).max() < 2e-3
