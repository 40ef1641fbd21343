"""CPU restatement of one decoder layer's single-token step (local-engine/src/layer.rs:354-523),
composed from the other oracle functions.

Test infrastructure only, like the rest of ``oracle/``.  ``decode_layer`` walks the same sequence of
operations as the reference and rounds to f16 wherever the reference stores f16; every operation is
one of the functions pinned elsewhere in this package (quant dequantisation, TurboQuant encode,
code-space attention, layer glue).  The multi-row paths (layer.rs:542-718, 731-873) compute the same
function row by row -- row r of a batch attends positions <= its own -- so their oracle is this step
applied once per row.

What pins the composition itself (tests/test_layer_oracle.py): with zero output and down projections
both residual branches contribute rms_norm(0) * w = 0 and the step must return its input bit for
bit; with a zero per-layer projection the injection is the identity; a scale of 0.5 halves the
output exactly; and the KV rows the step writes equal ``tq_write_kv`` of the hand-built K / V.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional

import numpy as np

from . import layer_glue as G
from . import oracle as O

F16, F32 = np.float16, np.float32


@dataclass
class Weight:
    """A projection as the f32 expansion of its stored values, [rows, cols]."""
    dq: np.ndarray

    @classmethod
    def from_quant(cls, fmt: str, data, rows: int, cols: int) -> "Weight":
        fn = O.expand_q4_0_f32 if fmt == "q4_0" else O.expand_tq2_0_f32
        return cls(fn(data, rows, cols))

    @classmethod
    def from_f16(cls, w, rows: int, cols: int) -> "Weight":
        return cls(np.asarray(w, F16).reshape(rows, cols).astype(F32))

    def matvec(self, x) -> np.ndarray:
        """f16 in, f16 out, exact (float64) accumulation (matvec_q4_0.metal / matvec_tq2_0.metal /
        matvec_f16.metal all accumulate in f32 and store half)."""
        return O.matvec_f64(self.dq, np.asarray(x, F16).astype(F32)).astype(F32).astype(F16)


@dataclass
class KvState:
    """One layer's TurboQuant cache (quant_cache.rs:73-229) as host arrays."""
    n_kv: int
    head_dim: int
    bits: int
    max_positions: int
    ring_capacity: int = 0          # 0 = absolute addressing
    signs: np.ndarray = field(init=False)
    levels: np.ndarray = field(init=False)

    def __post_init__(self):
        rows = (self.ring_capacity or self.max_positions) * self.n_kv
        cb = O.tq_code_bytes(self.head_dim, self.bits)
        self.signs = O.rotation_signs(self.head_dim)
        self.levels = O.tq_levels(self.head_dim, self.bits)
        self.k_codes = np.zeros(rows * cb, np.uint8)
        self.v_codes = np.zeros(rows * cb, np.uint8)
        self.k_norms = np.zeros(rows, np.uint16)
        self.v_norms = np.zeros(rows, np.uint16)

    def write(self, k, v, position: int) -> None:
        """quant_cache.rs:391-444."""
        for src, codes, norms in ((k, self.k_codes, self.k_norms), (v, self.v_codes, self.v_norms)):
            O.tq_write_kv(np.asarray(src, F16).view(np.uint16), self.n_kv, self.head_dim, self.bits, self.signs,
                          self.levels, position, self.ring_capacity, codes, norms)

    def row_slices(self, position: int):
        """(code bytes, norm entries) of the cache row that holds `position`."""
        cb = len(self.k_codes) // len(self.k_norms)
        slot = position % self.ring_capacity if self.ring_capacity else position
        return slice(slot * self.n_kv * cb, (slot + 1) * self.n_kv * cb), slice(slot * self.n_kv, (slot + 1) * self.n_kv)

    def replace_row(self, position: int, k_codes, k_norms, v_codes, v_norms) -> float:
        """Overwrite the row of `position`; returns the fraction of its code fields (of the given bit width, byte
        aligned widths only) that differed from what was there."""
        cs, ns = self.row_slices(position)
        new_k, new_v = np.asarray(k_codes, np.uint8).reshape(-1), np.asarray(v_codes, np.uint8).reshape(-1)
        diff, fields = 0, 0
        if 8 % self.bits == 0:
            mask = (1 << self.bits) - 1
            for old, new in ((self.k_codes[cs], new_k), (self.v_codes[cs], new_v)):
                x = np.bitwise_xor(old, new)
                for sh in range(0, 8, self.bits):
                    diff += int((((x >> sh) & mask) != 0).sum())
                fields += x.size * (8 // self.bits)
        self.k_codes[cs], self.v_codes[cs] = new_k, new_v
        self.k_norms[ns], self.v_norms[ns] = np.asarray(k_norms, np.uint16).reshape(-1), np.asarray(v_norms, np.uint16).reshape(-1)
        return diff / fields if fields else 0.0

    def attend(self, q, seq_len: int, current_pos: int, n_q_heads: int, window: int) -> np.ndarray:
        """quant_cache.rs:548-598: rotate q (f16 -> f32), attend in code space, rotate back (f32 -> f16)."""
        hd = self.head_dim
        rq = O.hadamard_rotate(np.asarray(q, F16).astype(F32), self.signs, hd, n_q_heads, True, False)
        vacc = O.attention_tq_codespace(rq, self.k_codes, self.k_norms, self.v_codes, self.v_norms, self.levels, hd,
                                        seq_len, current_pos, n_q_heads, self.n_kv, window, self.bits,
                                        self.ring_capacity)
        return O.hadamard_rotate(vacc, self.signs, hd, n_q_heads, False, True).astype(F16)


@dataclass
class Layer:
    """Host-side weights of one layer; names follow layer.rs:310-328."""
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    attn_norm: np.ndarray
    attn_q: Weight
    attn_output: Weight
    attn_post_norm: np.ndarray
    ffn_norm: np.ndarray
    ffn_gate: Weight
    ffn_up: Weight
    ffn_down: Weight
    ffn_post_norm: np.ndarray
    attn_k: Optional[Weight] = None
    attn_v: Optional[Weight] = None
    q_norm: Optional[np.ndarray] = None
    k_norm: Optional[np.ndarray] = None
    per_layer_inp_gate: Optional[Weight] = None
    per_layer_proj: Optional[Weight] = None
    per_layer_post_norm: Optional[np.ndarray] = None
    layer_output_scale: Optional[float] = None
    layer_idx: int = 0
    per_layer_dim: int = 0
    rope_theta: float = 10000.0
    partial_rotary_factor: float = 1.0
    sliding_window: int = 0
    rms_norm_eps: float = 1e-6
    is_kv_shared: bool = False

    @classmethod
    def from_host(cls, tensors: dict, **dims) -> "Layer":
        """Host tensors keyed by field name: a projection is ``(format, rows, cols, payload)``, a norm vector an
        f16 array, ``layer_output_scale`` a one-element f16 array."""
        fields = {}
        for name, t in tensors.items():
            if isinstance(t, tuple):
                fmt, rows, cols, payload = t
                fields[name] = Weight.from_f16(payload, rows, cols) if fmt == "f16" else \
                    Weight.from_quant(fmt, payload, rows, cols)
            elif name == "layer_output_scale":
                fields[name] = float(np.asarray(t, F16).reshape(-1)[0])
            else:
                fields[name] = np.asarray(t, F16)
        return cls(**fields, **dims)


def decode_layer(L: Layer, x, position: int, kv: KvState, per_layer_input=None, kv_rows=None, trace=None,
                 kv_codes=None) -> np.ndarray:
    """layer.rs:354-523: hidden state [hidden_size] f16 in and out; ``kv`` is updated in place.

    ``trace``, a dict, receives the intermediates (normed, q, k, v, attn_out, attn_resid).  ``kv_rows = (k, v)``
    encodes those f16 rows into the cache in place of the layer's own (still computed and traced): a 2-bit
    code is a discontinuous function of its input, so a checker that wants tight bounds downstream of the
    cache compares k / v first and then continues from the rows of the implementation under test.  ``kv_codes =
    (k_codes, k_norms, v_codes, v_norms)`` (the cache row of this position as the implementation under test wrote it)
    does the same one stage later, for a checker that cannot see the rows: the layer's own codes are still computed,
    the fraction of 2-bit codes that differ goes to ``trace["code_flips"]``, and the given row replaces them."""
    trace = {} if trace is None else trace
    h, hd, n_head, n_kv, eps = L.hidden_size, L.head_dim, L.num_attention_heads, L.num_key_value_heads, L.rms_norm_eps
    x = np.asarray(x, F16).reshape(h)

    # 1. layer.rs:387-404
    normed = G.rms_norm(x, L.attn_norm, h, 1, eps)
    q = L.attn_q.matvec(normed)
    if L.q_norm is not None:
        q = G.qk_norm(q, L.q_norm, hd, n_head, eps)
    q = G.rope(q, hd, position, L.rope_theta, L.partial_rotary_factor, n_head)

    # 2. layer.rs:406-450
    if not L.is_kv_shared and L.attn_k is not None and L.attn_v is not None:
        k = L.attn_k.matvec(normed)
        v = L.attn_v.matvec(normed)
        if L.k_norm is not None:
            k = G.qk_norm(k, L.k_norm, hd, n_kv, eps)
        v = G.rms_norm(v, np.ones(hd, F16), hd, n_kv, eps)
        k = G.rope(k, hd, position, L.rope_theta, L.partial_rotary_factor, n_kv)
        trace["k"], trace["v"] = k, v
        if kv_rows is not None:
            k, v = kv_rows
        kv.write(k, v, position)
        if kv_codes is not None:
            trace["code_flips"] = kv.replace_row(position, *kv_codes)
    trace["normed"], trace["q"] = normed, q
    attn_out = kv.attend(q, position + 1, position, n_head, L.sliding_window)

    # 3. layer.rs:452-466
    proj = L.attn_output.matvec(attn_out)
    attn_resid = G.rms_norm(proj, L.attn_post_norm, h, 1, eps, residual=x)
    trace["attn_out"], trace["attn_resid"] = attn_out, attn_resid

    # 4. layer.rs:468-494
    normed = G.rms_norm(attn_resid, L.ffn_norm, h, 1, eps)
    gate = G.gelu_mul(L.ffn_gate.matvec(normed), L.ffn_up.matvec(normed))
    out = G.rms_norm(L.ffn_down.matvec(gate), L.ffn_post_norm, h, 1, eps, residual=attn_resid)

    # 5. layer.rs:496-521
    if (L.per_layer_inp_gate is not None and L.per_layer_proj is not None and L.per_layer_post_norm is not None
            and per_layer_input is not None):
        pld = L.per_layer_dim
        ple = np.asarray(per_layer_input, F16).reshape(-1)[L.layer_idx * pld:(L.layer_idx + 1) * pld]
        g = G.gelu_mul(L.per_layer_inp_gate.matvec(out), ple)
        inj = G.rms_norm(L.per_layer_proj.matvec(g), L.per_layer_post_norm, h, 1, eps)
        out = G.residual_add(out, inj)

    # 6. layer.rs:513-520
    if L.layer_output_scale is not None:
        out = G.scale_in_place(out, L.layer_output_scale)
    return out


@dataclass
class Model:
    """Host-side state of the decode core of the reference's Pipeline (local-engine/src/pipeline.rs:714-953)."""
    hidden_size: int
    vocab_size: int
    layers: list                      # [Layer]
    kv_index_map: list                # layer -> index into the list of KvState (pipeline.rs:379-437)
    token_embd: Weight                # [vocab, hidden]: the f16 values of the stored rows, as f32
    output_norm: np.ndarray
    per_layer_dim: int = 0
    ple_table: Optional[Weight] = None          # [vocab, n_layer * pld]
    per_layer_model_proj: Optional[Weight] = None
    per_layer_proj_norm: Optional[np.ndarray] = None
    rms_norm_eps: float = 1e-6
    logit_softcap: float = 30.0


def model_from_host(config, tensors: dict, logit_softcap: float = 30.0) -> Model:
    """The host tensors of ``synth.decode_model_tensors`` for a ``pipeline.Gemma4QATConfig``-shaped `config`, with the
    cache-slot map of pipeline.rs:379-437."""
    n_layer = config.num_hidden_layers
    layers = []
    for i, lt in enumerate(tensors["layers"]):
        inter = lt["ffn_gate"][1]
        layers.append(Layer.from_host(lt, hidden_size=config.hidden_size, intermediate_size=inter,
                                      num_attention_heads=config.num_attention_heads,
                                      num_key_value_heads=config.num_key_value_heads, head_dim=config.attn_head_dim(i),
                                      layer_idx=i, per_layer_dim=config.hidden_size_per_layer_input,
                                      rope_theta=config.rope_theta(i), partial_rotary_factor=config.partial_rotary_factor(i),
                                      sliding_window=0 if config.is_full_attention(i) else config.sliding_window,
                                      rms_norm_eps=config.rms_norm_eps, is_kv_shared=config.is_kv_shared(i)))
    slot_of, kv_index_map, n_slots = {}, [0] * n_layer, 0
    for i in range(n_layer):
        if config.is_kv_shared(i):
            kv_index_map[i] = slot_of[config.kv_source_layer(i)]
        else:
            slot_of[i] = kv_index_map[i] = n_slots
            n_slots += 1

    def weight(t):
        fmt, rows, cols, payload = t
        return Weight.from_quant(fmt, payload, rows, cols)

    m = Model(hidden_size=config.hidden_size, vocab_size=config.vocab_size, layers=layers, kv_index_map=kv_index_map,
              token_embd=weight(tensors["token_embd"]), output_norm=np.asarray(tensors["output_norm"], F16),
              per_layer_dim=config.hidden_size_per_layer_input, rms_norm_eps=config.rms_norm_eps, logit_softcap=logit_softcap)
    if "ple_table" in tensors:
        m.ple_table = weight(tensors["ple_table"])
        m.per_layer_model_proj = weight(tensors["per_layer_model_proj"])
        m.per_layer_proj_norm = np.asarray(tensors["per_layer_proj_norm"], F16)
    return m


def per_layer_inputs(M: Model, token: int, hidden) -> Optional[np.ndarray]:
    """pipeline.rs:725-776."""
    if M.ple_table is None or M.per_layer_model_proj is None or M.per_layer_proj_norm is None:
        return None
    pld, n_layer = M.per_layer_dim, len(M.layers)
    tok = G.scale_in_place(M.ple_table.dq[min(token, M.vocab_size - 1)].astype(F16), float(F32(np.sqrt(F32(pld)))))
    proj = G.scale_in_place(M.per_layer_model_proj.matvec(hidden), float(F32(1.0) / np.sqrt(F32(M.hidden_size))))
    proj = G.rms_norm(proj, M.per_layer_proj_norm, pld, n_layer, M.rms_norm_eps)
    return G.scale_in_place(G.residual_add(proj, tok), float(F32(np.sqrt(0.5))))


def decode_token(M: Model, token: int, position: int, kvs: list, layer_kv_codes=None, trace=None) -> np.ndarray:
    """pipeline.rs:834-953: the f32 logits of `token` at `position`; `kvs` are the KvStates of the cache slots.
    `layer_kv_codes[i]`, when given for a layer that owns its KV, is passed to decode_layer as `kv_codes`."""
    trace = {} if trace is None else trace
    hidden = M.token_embd.dq[min(token, M.vocab_size - 1)].astype(F16)
    hidden = G.scale_in_place(hidden, float(F32(np.sqrt(F32(M.hidden_size)))))
    ple = per_layer_inputs(M, token, hidden)
    flips = []
    for i, layer in enumerate(M.layers):
        tr = {}
        hidden = decode_layer(layer, hidden, position, kvs[M.kv_index_map[i]], ple, trace=tr,
                              kv_codes=None if layer_kv_codes is None else layer_kv_codes[i])
        if "code_flips" in tr:
            flips.append(tr["code_flips"])
    trace["code_flips"] = flips
    final = G.rms_norm(hidden, M.output_norm, M.hidden_size, 1, M.rms_norm_eps)
    logits = O.matvec_f64(M.token_embd.dq, final.astype(F32)).astype(F32)
    return G.logit_softcap(logits, M.logit_softcap) if M.logit_softcap > 0 else logits
