"""``TransformerLayer`` (local-engine/src/layer.rs:284-873): one Gemma decoder layer encoded into a
command batch -- single-token decode, multi-row prefill / batched decode over one sequence, and
continuous-batching decode over independent lanes -- plus its scratch arenas
(``ScratchBuffers`` layer.rs:951-1037, ``BatchScratch`` layer.rs:878-948).

Every dispatch is one of the HIP kernels behind the C ABI; this file only orders them the way the
reference does and owns no arithmetic.  One addition over the reference's call sequence: when two
projections read the same input and share format and shape (K/V, gate/up), the single-token path
launches them as one grouped matvec so both weight streams are in flight together; the results are
the same values the separate launches produce.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import numpy as np

from . import F16, Q4_0, TQ2_0, Buffer, InvalidArgument, Kernels
from .kv_cache import QuantizedKvCache, QuantizedUnifiedKvPool
from .quant_weight import W_F16, QuantWeight

MAX_FLASH_SPLITS = 16   # layer.rs:979


@dataclass
class LayerParams:
    """layer.rs:291-308."""
    layer_idx: int
    hidden_size: int
    intermediate_size: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    per_layer_dim: int = 0
    rope_theta: float = 10000.0
    partial_rotary_factor: float = 1.0
    sliding_window: int = 0
    rms_norm_eps: float = 1e-6
    is_kv_shared: bool = False


@dataclass
class LayerWeights:
    """layer.rs:310-328: norm vectors are f16 buffers, projections are ``QuantWeight``."""
    attn_norm: Buffer
    attn_q: QuantWeight
    attn_output: QuantWeight
    attn_post_norm: Buffer
    ffn_norm: Buffer
    ffn_gate: QuantWeight
    ffn_up: QuantWeight
    ffn_down: QuantWeight
    ffn_post_norm: Buffer
    attn_k: Optional[QuantWeight] = None
    attn_v: Optional[QuantWeight] = None
    q_norm: Optional[Buffer] = None
    k_norm: Optional[Buffer] = None
    per_layer_inp_gate: Optional[QuantWeight] = None
    per_layer_proj: Optional[QuantWeight] = None
    per_layer_post_norm: Optional[Buffer] = None
    layer_output_scale: Optional[Buffer] = None

    @classmethod
    def from_host(cls, ctx, tensors: dict) -> "LayerWeights":
        """Upload host tensors keyed by field name: a projection is ``(format, rows, cols, payload)`` with
        format "q4_0" / "tq2_0" (GGUF block bytes, uploaded verbatim) or "f16"; anything else is an f16 vector."""
        fields = {}
        for name, t in tensors.items():
            if isinstance(t, tuple):
                fmt, rows, cols, payload = t
                if fmt == "f16":
                    fields[name] = QuantWeight.f16(Buffer.from_slice(ctx, np.asarray(payload, np.float16)), rows, cols)
                else:
                    fields[name] = QuantWeight.from_bytes(ctx, payload, {"q4_0": Q4_0, "tq2_0": TQ2_0}[fmt], rows, cols)
            else:
                fields[name] = Buffer.from_slice(ctx, np.asarray(t, np.float16))
        return cls(**fields)


def _alloc_f16(ctx, elems: int) -> Buffer:
    return Buffer.empty(ctx, max(elems, 1) * 2)


def _alloc_f32(ctx, elems: int) -> Buffer:
    return Buffer.empty(ctx, max(elems, 1) * 4)


class ScratchBuffers:
    """layer.rs:951-1037: single-token scratch sized for the widest layer."""

    def __init__(self, ctx, hidden_size: int, intermediate_size: int, num_attention_heads: int,
                 num_key_value_heads: int, head_dim: int, per_layer_dim: int):
        q_elems = num_attention_heads * head_dim
        kv_elems = num_key_value_heads * head_dim
        self.normed = _alloc_f16(ctx, hidden_size)
        # q, k, v are consecutive pieces of one allocation: a layer whose three projections were stacked into one
        # matrix writes them with a single matvec (at that layer's own sizes, see TransformerLayer._qkv_views)
        self.qkv = _alloc_f16(ctx, q_elems + 2 * kv_elems)
        self.q = self.qkv.view(0, q_elems * 2)
        self.k = self.qkv.view(q_elems * 2, kv_elems * 2)
        self.v = self.qkv.view((q_elems + kv_elems) * 2, kv_elems * 2)
        self.rq = _alloc_f32(ctx, q_elems)
        self.vacc = _alloc_f32(ctx, q_elems)
        self.attn_out = _alloc_f16(ctx, q_elems)
        self.attn_resid = _alloc_f16(ctx, hidden_size)
        self.gate = _alloc_f16(ctx, intermediate_size)
        self.up = _alloc_f16(ctx, intermediate_size)
        self.ffn_out = _alloc_f16(ctx, hidden_size)
        self.ple = _alloc_f16(ctx, per_layer_dim)
        self.ple_h = _alloc_f16(ctx, hidden_size)
        self.ones = Buffer.from_slice(ctx, np.ones(head_dim, np.float16))
        self.fa_pmax = _alloc_f32(ctx, num_attention_heads * MAX_FLASH_SPLITS)
        self.fa_psum = _alloc_f32(ctx, num_attention_heads * MAX_FLASH_SPLITS)
        self.fa_pacc = _alloc_f32(ctx, num_attention_heads * MAX_FLASH_SPLITS * head_dim)


class BatchScratch:
    """layer.rs:878-948: multi-row scratch sized for ``max_batch`` rows at the widest layer."""

    def __init__(self, ctx, max_batch: int, hidden_size: int, intermediate_size: int, num_attention_heads: int,
                 num_key_value_heads: int, head_dim: int, per_layer_dim: int, num_layers: int):
        mb = max_batch
        ple_total = mb * num_layers * per_layer_dim
        self.max_batch = max_batch
        self.hidden_a = _alloc_f16(ctx, mb * hidden_size)
        self.hidden_b = _alloc_f16(ctx, mb * hidden_size)
        self.normed = _alloc_f16(ctx, mb * hidden_size)
        self.q = _alloc_f16(ctx, mb * num_attention_heads * head_dim)
        self.k = _alloc_f16(ctx, mb * num_key_value_heads * head_dim)
        self.v = _alloc_f16(ctx, mb * num_key_value_heads * head_dim)
        self.attn_out = _alloc_f16(ctx, mb * num_attention_heads * head_dim)
        self.rq = _alloc_f32(ctx, mb * num_attention_heads * head_dim)
        self.vacc = _alloc_f32(ctx, mb * num_attention_heads * head_dim)
        self.attn_resid = _alloc_f16(ctx, mb * hidden_size)
        self.gate = _alloc_f16(ctx, mb * intermediate_size)
        self.up = _alloc_f16(ctx, mb * intermediate_size)
        self.ffn_out = _alloc_f16(ctx, mb * hidden_size)
        self.ple_tok = _alloc_f16(ctx, ple_total)
        self.ple_proj = _alloc_f16(ctx, ple_total)
        self.ple_all = _alloc_f16(ctx, ple_total)
        self.ple_g = _alloc_f16(ctx, mb * max(per_layer_dim, 1))
        self.ple_slice = _alloc_f16(ctx, mb * max(per_layer_dim, 1))


def _groupable(a: Optional[QuantWeight], b: Optional[QuantWeight]) -> bool:
    return (a is not None and b is not None and a.ty == b.ty and a.ty != W_F16
            and a.rows == b.rows and a.cols == b.cols)


@dataclass
class PendingTail:
    """The last step of a decoded layer, left for the next layer's first dispatch:
    hidden = (rms_norm(x) * weight + residual) * scale  (layer.rs:503-520; ``scale`` None: no output scale)."""
    x: Buffer
    weight: Buffer
    residual: Buffer
    scale: Optional[float]


class TransformerLayer:
    """layer.rs:330-873."""

    def __init__(self, params: LayerParams, weights: LayerWeights, group_projections: bool = True,
                 fuse_norm_rope: bool = True, fuse_prologues: bool = True, fuse_norm_chain: bool = True,
                 stack_qkv: bool = True, fuse_rotation: bool = True):
        self.params, self.weights = params, weights
        self.group_projections, self.fuse_norm_rope = group_projections, fuse_norm_rope
        self.fuse_prologues, self.fuse_norm_chain = fuse_prologues, fuse_prologues and fuse_norm_chain
        # a decoded token's rotation back out of code space rides in the output projection's staging
        self.fuse_rotation = fuse_prologues and fuse_rotation
        # layer.rs:515-520 reads the scalar out of shared memory at every encode; the buffer lives in device
        # memory here, so it is fetched once.
        self._output_scale = None
        if weights.layer_output_scale is not None and weights.layer_output_scale.length() >= 2:
            self._output_scale = float(weights.layer_output_scale.as_array(np.float16, 1)[0])
        self._qkv = None
        if stack_qkv:
            self._stack_qkv()

    def _stack_qkv(self) -> None:
        """Q, K and V projections of one format over the same input become the row blocks of one matrix (one
        allocation, the three weights rebound to views of it), so a decoded token needs one matvec for all three."""
        w = self.weights
        q, k, v = w.attn_q, w.attn_k, w.attn_v
        if self.params.is_kv_shared or k is None or v is None or q.ty == W_F16:
            return
        if not (q.ty == k.ty == v.ty and q.cols == k.cols == v.cols and q.cols % 64 == 0):
            return
        ctx = q.buf.ctx
        sizes = [x.rows * x.row_bytes() for x in (q, k, v)]
        stacked = Buffer.empty(ctx, sum(sizes))
        from . import CommandBatch
        batch = CommandBatch(ctx)
        off = 0
        for x, n in zip((q, k, v), sizes):
            batch.blit_copy(x.buf, 0, stacked, off, n)
            off += n
        batch.commit_and_wait()
        off = 0
        for x, n in zip((q, k, v), sizes):
            x.buf = stacked.view(off, n)
            off += n
        self._qkv = QuantWeight.quantized(stacked, q.ty, q.rows + k.rows + v.rows, q.cols)

    def _qkv_views(self, scratch: "ScratchBuffers"):
        """(q, k, v) views of scratch.qkv at this layer's sizes, consecutive (cached per scratch object)."""
        cached = getattr(self, "_qkv_view_cache", None)
        if cached is None or cached[0] is not scratch:
            p = self.params
            nq, nkv = p.num_attention_heads * p.head_dim * 2, p.num_key_value_heads * p.head_dim * 2
            cached = (scratch, scratch.qkv.view(0, nq), scratch.qkv.view(nq, nkv), scratch.qkv.view(nq + nkv, nkv),
                      scratch.qkv.view(0, nq + 2 * nkv))
            self._qkv_view_cache = cached
        return cached[1:]

    # ------------------------------------------------------------------ helpers
    def _pair_matvec(self, batch, kernels: Kernels, wa: QuantWeight, wb: QuantWeight, x: Buffer, out_a: Buffer,
                     out_b: Buffer) -> None:
        if self.group_projections and _groupable(wa, wb):
            kernels.matvec_quant_grouped_into(batch, wa.ty, [wa.buf, wb.buf], [x, x], F16, [out_a, out_b], F16,
                                              wa.rows, wa.cols)
        else:
            wa.matvec_into(batch, kernels, x, out_a)
            wb.matvec_into(batch, kernels, x, out_b)

    def _ple_slice(self, per_layer_input: Buffer) -> Buffer:
        """This layer's [per_layer_dim] slice of the per-layer input buffer, as a view (cached per buffer)."""
        cached = getattr(self, "_ple_view", None)
        if cached is None or cached[0] is not per_layer_input:
            pld = self.params.per_layer_dim
            cached = (per_layer_input, per_layer_input.view(self.params.layer_idx * pld * 2, pld * 2))
            self._ple_view = cached
        return cached[1]

    def _matmuls(self, batch, kernels: Kernels, ws, x: Buffer, outs, rows: int) -> None:
        """out_i[rows, w_i.rows] = x . w_i^T for projections that read the same rows; weights of one quantized format
        and width go out as one launch."""
        if (self.group_projections and len(ws) > 1 and all(w.ty == ws[0].ty and w.cols == ws[0].cols for w in ws)
                and ws[0].ty != W_F16):
            kernels.matmul_nt_quant_grouped_into(batch, ws[0].ty, x, [w.buf for w in ws], list(outs), rows, ws[0].cols,
                                                 [w.rows for w in ws])
            return
        for w, out in zip(ws, outs):
            w.matmul_nt_into(batch, kernels, x, out, rows)

    def _qkv_as_one(self) -> bool:
        """Whether Q, K and V can go out as the grouped product that hands its tiles to the preparation."""
        q, k, v = self.weights.attn_q, self.weights.attn_k, self.weights.attn_v
        return (self.group_projections and self.fuse_norm_chain and q.ty != W_F16 and q.ty == k.ty == v.ty
                and q.cols == k.cols == v.cols)

    def _one_prepare(self) -> bool:
        hd = self.params.head_dim
        return self.fuse_prologues and 64 <= hd <= 512 and hd & (hd - 1) == 0

    def _fusable(self, *ws: Optional[QuantWeight]) -> bool:
        return self.fuse_prologues and all(w is not None and w.ty != W_F16 and w.cols % 64 == 0 for w in ws)

    def _fused_matvecs(self, batch, kernels: Kernels, prologue: int, x: Buffer, aux: Buffer, ws, outs) -> None:
        """Every weight in `ws` against prologue(x, aux); weights of one format and shape share a launch."""
        eps = self.params.rms_norm_eps
        if len(ws) == 2 and self.group_projections and _groupable(ws[0], ws[1]):
            kernels.matvec_quant_fused_into(batch, ws[0].ty, [w.buf for w in ws], x, prologue, aux, eps, list(outs),
                                            ws[0].rows, ws[0].cols)
            return
        for w, out in zip(ws, outs):
            kernels.matvec_quant_fused_into(batch, w.ty, [w.buf], x, prologue, aux, eps, [out], w.rows, w.cols)

    def _norm_rope(self, batch, kernels: Kernels, qk: Buffer, norm_w: Optional[Buffer], heads: int, pos: int) -> None:
        """layer.rs:393-404 / 415-428: per-head RMS norm (when the layer has one) then RoPE, in place."""
        p = self.params
        if norm_w is not None and self.fuse_norm_rope and kernels.qk_norm_rope_available(p.head_dim):
            kernels.qk_norm_rope_into(batch, qk, qk, norm_w, p.head_dim, heads, p.rms_norm_eps, pos, p.rope_theta,
                                      p.partial_rotary_factor)
            return
        if norm_w is not None:
            kernels.qk_norm_gpu_into(batch, qk, norm_w, p.head_dim, heads, p.rms_norm_eps)
        kernels.rope_into(batch, qk, qk, p.head_dim, pos, p.rope_theta, p.partial_rotary_factor, heads)

    def _scale_output(self, batch, kernels: Kernels, output: Buffer, count: int) -> None:
        if self._output_scale is not None:
            kernels.scale_in_place_gpu_into(batch, output, self._output_scale, count)

    # ----------------------------------------------------- single-token decode
    def forward_decode(self, kernels: Kernels, batch, input: Buffer, output: Buffer, position: int,
                       scratch: ScratchBuffers, kv_cache: QuantizedKvCache, per_layer_input: Optional[Buffer] = None,
                       n_layer_total: int = 0, pending: Optional["PendingTail"] = None,
                       defer_tail: bool = False) -> Optional["PendingTail"]:
        """layer.rs:354-523.  ``kv_cache`` is this layer's cache, or for a KV-shared layer the source layer's
        (already written earlier in the same step).

        Two layers can share a dispatch across their boundary: with ``defer_tail`` the last step of this layer (per-layer
        post-norm, residual #3, output scale: layer.rs:503-520) is not dispatched but returned as a ``PendingTail``; the
        caller hands it to the next layer as ``pending``, whose first matvec computes it while it stages its input and
        writes it to ``input`` (which must be neither ``pending.x`` nor ``pending.residual``).  None is returned when the
        layer ran its last step itself (then ``output`` holds the result)."""
        p, w, s = self.params, self.weights, scratch
        h, hd, n_head, n_kv, eps = p.hidden_size, p.head_dim, p.num_attention_heads, p.num_key_value_heads, p.rms_norm_eps
        pos, seq_len = position, position + 1

        # 1. input_layernorm -> Q projection -> q_norm -> RoPE
        own_kv = not p.is_kv_shared and w.attn_k is not None and w.attn_v is not None
        fused_in = self._fusable(w.attn_q) and (not own_kv or self._fusable(w.attn_k, w.attn_v))
        q_buf, k_buf, v_buf = s.q, s.k, s.v
        stacked = fused_in and own_kv and self._qkv is not None
        if pending is not None and not fused_in:   # nothing here can take it along: the previous layer's last step by itself
            kernels.rms_norm_residual_scale_into(batch, pending.x, pending.weight, pending.residual, input, h, 1, eps, pending.scale)
            pending = None
        if stacked:   # one matvec over the stacked [Wq; Wk; Wv] writes q | k | v side by side
            q_buf, k_buf, v_buf, qkv_out = self._qkv_views(s)
            if pending is not None:
                kernels.matvec_quant_norm_chain_tail_into(batch, self._qkv.ty, [self._qkv.buf], pending.x, pending.weight,
                                                          pending.residual, pending.scale, w.attn_norm, input, eps, [qkv_out],
                                                          self._qkv.rows, self._qkv.cols)
            else:
                self._fused_matvecs(batch, kernels, kernels.PROLOGUE_RMS_NORM, input, w.attn_norm, [self._qkv], [qkv_out])
        elif fused_in:
            if pending is not None:   # (the K / V launch below then finds `input` written)
                kernels.matvec_quant_norm_chain_tail_into(batch, w.attn_q.ty, [w.attn_q.buf], pending.x, pending.weight,
                                                          pending.residual, pending.scale, w.attn_norm, input, eps, [s.q],
                                                          w.attn_q.rows, w.attn_q.cols)
            else:
                self._fused_matvecs(batch, kernels, kernels.PROLOGUE_RMS_NORM, input, w.attn_norm, [w.attn_q], [s.q])
        else:
            kernels.rms_norm_into(batch, input, w.attn_norm, s.normed, h, 1, eps)
            w.attn_q.matvec_into(batch, kernels, s.normed, s.q)
        one_prepare = self._one_prepare()
        rotate_in_o = (one_prepare and self.fuse_rotation and self._fusable(w.attn_output)
                       and w.attn_output.cols == n_head * hd)
        if not one_prepare:
            self._norm_rope(batch, kernels, q_buf, w.q_norm, n_head, pos)

        # 2. own K/V into the TurboQuant cache, then attention over the codes
        if own_kv and not stacked:
            if fused_in:
                self._fused_matvecs(batch, kernels, kernels.PROLOGUE_RMS_NORM, input, w.attn_norm,
                                    [w.attn_k, w.attn_v], [s.k, s.v])
            else:
                self._pair_matvec(batch, kernels, w.attn_k, w.attn_v, s.normed, s.k, s.v)
        if one_prepare:   # head norms, RoPE, V norm, both encodes and the query rotation in one dispatch
            kv_cache.prepare_token_into(batch, kernels, q_buf, k_buf if own_kv else None, v_buf if own_kv else None,
                                        w.q_norm, w.k_norm, s.rq, position, n_head, eps, p.rope_theta,
                                        p.partial_rotary_factor)
            if rotate_in_o:   # where the rotation would be a launch of its own, step 3 does it while it stages the heads
                rotate_in_o = not kv_cache.attention_from_rotated_lazy_into(batch, kernels, s.rq, s.vacc, s.attn_out,
                                                                            seq_len, pos, n_head, p.sliding_window)
            else:
                kv_cache.attention_from_rotated_into(batch, kernels, s.rq, s.vacc, s.attn_out, seq_len, pos, n_head,
                                                     p.sliding_window)
        elif own_kv:
            kernels.rms_norm_into(batch, v_buf, s.ones, v_buf, hd, n_kv, eps)   # V: RMS norm with unit weight
            self._norm_rope(batch, kernels, k_buf, w.k_norm, n_kv, pos)
            kv_cache.write_kv_gpu_into(batch, kernels, k_buf, v_buf, position, 1)
        if not one_prepare:
            kv_cache.fused_attention_into(batch, kernels, q_buf, s.rq, s.vacc, s.attn_out, seq_len, pos, n_head,
                                          p.sliding_window)

        # 3. output projection -> post_attention_norm + residual #1
        if rotate_in_o:
            kernels.matvec_quant_rotated_into(batch, w.attn_output.ty, w.attn_output.buf, s.vacc, kv_cache.signs, hd,
                                              s.ffn_out, w.attn_output.rows, w.attn_output.cols)
        else:
            w.attn_output.matvec_into(batch, kernels, s.attn_out, s.ffn_out)
        chain_ffn = (self.fuse_norm_chain and self._fusable(w.ffn_gate, w.ffn_up) and self.group_projections
                     and _groupable(w.ffn_gate, w.ffn_up))
        if not chain_ffn:
            kernels.rms_norm_add_into(batch, s.ffn_out, w.attn_post_norm, input, s.attn_resid, h, 1, eps)

        # 4. GeGLU feed-forward -> post_feedforward_norm + residual #2
        inter = p.intermediate_size
        if chain_ffn:   # residual #1 and the feed-forward pre-norm while gate / up stage their input; attn_resid kept
            kernels.matvec_quant_norm_chain_into(batch, w.ffn_gate.ty, [w.ffn_gate.buf, w.ffn_up.buf], s.ffn_out,
                                                 w.attn_post_norm, input, w.ffn_norm, s.attn_resid, eps, [s.gate, s.up],
                                                 w.ffn_gate.rows, w.ffn_gate.cols)
        elif self._fusable(w.ffn_gate, w.ffn_up):
            self._fused_matvecs(batch, kernels, kernels.PROLOGUE_RMS_NORM, s.attn_resid, w.ffn_norm,
                                [w.ffn_gate, w.ffn_up], [s.gate, s.up])
        else:
            kernels.rms_norm_into(batch, s.attn_resid, w.ffn_norm, s.normed, h, 1, eps)
            self._pair_matvec(batch, kernels, w.ffn_gate, w.ffn_up, s.normed, s.gate, s.up)
        if self._fusable(w.ffn_down):
            self._fused_matvecs(batch, kernels, kernels.PROLOGUE_GELU_MUL, s.gate, s.up, [w.ffn_down], [s.ffn_out])
        else:
            kernels.gelu_mul_into(batch, s.gate, s.up, s.gate, inter)
            w.ffn_down.matvec_into(batch, kernels, s.gate, s.ffn_out)
        has_ple = (w.per_layer_inp_gate is not None and w.per_layer_proj is not None
                   and w.per_layer_post_norm is not None and per_layer_input is not None)
        chain_ple = self.fuse_norm_chain and has_ple and self._fusable(w.per_layer_inp_gate) and output is not s.ffn_out
        if not chain_ple:
            kernels.rms_norm_add_into(batch, s.ffn_out, w.ffn_post_norm, s.attn_resid, output, h, 1, eps)

        # 5. per-layer input injection -> residual #3
        if has_ple:
            pld = p.per_layer_dim
            if chain_ple:   # residual #2 while the per-layer gate stages its input; `output` written once by that kernel
                g = w.per_layer_inp_gate
                kernels.matvec_quant_norm_chain_into(batch, g.ty, [g.buf], s.ffn_out, w.ffn_post_norm, s.attn_resid, None,
                                                     output, eps, [s.ple_h], g.rows, g.cols)
            else:
                w.per_layer_inp_gate.matvec_into(batch, kernels, output, s.ple_h)
            if self._fusable(w.per_layer_proj):
                # this layer's slice is read in place (no copy into scratch) while the projection stages its input
                self._fused_matvecs(batch, kernels, kernels.PROLOGUE_GELU_MUL, s.ple_h, self._ple_slice(per_layer_input),
                                    [w.per_layer_proj], [s.ffn_out])
            else:
                batch.blit_copy(per_layer_input, p.layer_idx * pld * 2, s.ple, 0, pld * 2)
                kernels.gelu_mul_into(batch, s.ple_h, s.ple, s.ple_h, pld)
                w.per_layer_proj.matvec_into(batch, kernels, s.ple_h, s.ffn_out)
            if self.fuse_prologues:   # norm, residual #3 and the output scale (step 6) in one dispatch
                if defer_tail:        # ... or in the next layer's first one
                    return PendingTail(s.ffn_out, w.per_layer_post_norm, output, self._output_scale)
                kernels.rms_norm_residual_scale_into(batch, s.ffn_out, w.per_layer_post_norm, output, output, h, 1, eps,
                                                     self._output_scale)
                return None
            kernels.rms_norm_into(batch, s.ffn_out, w.per_layer_post_norm, s.normed, h, 1, eps)
            kernels.residual_add_into(batch, output, s.normed, output, h)

        # 6. per-layer output scale
        self._scale_output(batch, kernels, output, h)
        return None

    # ------------------------------------------------ shared multi-row tail
    def _attention_tail(self, kernels: Kernels, batch, rows: int, input: Buffer, output: Buffer, bs: BatchScratch,
                        ple_all, next_norm: Optional[Buffer] = None) -> None:
        """Everything after attention, identical in layer.rs:640-716 and layer.rs:808-870.  With ``next_norm`` (the next
        layer's attention-norm weight) the last step also leaves rms_norm(output, next_norm) in ``bs.normed``, which is
        that layer's first dispatch."""
        p, w = self.params, self.weights
        h, eps, inter = p.hidden_size, p.rms_norm_eps, p.intermediate_size
        has_ple = (w.per_layer_inp_gate is not None and w.per_layer_proj is not None
                   and w.per_layer_post_norm is not None and ple_all is not None)

        def product_norm(weight, x, norm_w, residual, out, scale=None, norm2_w=None, out2=None):
            """matmul_nt -> rms_norm_add (-> output scale) (-> rms_norm): one fused step where the weight format has
            one, the separate kernels otherwise (same result either way)."""
            if self.fuse_norm_chain and weight.ty != W_F16 and h % 8 == 0 and h <= 8192:
                kernels.matmul_nt_quant_norm_into(batch, weight.ty, x, weight.buf, rows, weight.cols, weight.rows, norm_w,
                                                  residual, out, eps, scale, norm2_w, out2)
                return
            weight.matmul_nt_into(batch, kernels, x, bs.ffn_out, rows)
            kernels.rms_norm_add_into(batch, bs.ffn_out, norm_w, residual, out, h, rows, eps)
            if scale is not None:
                kernels.scale_in_place_gpu_into(batch, out, scale, rows * h)
            if norm2_w is not None:
                kernels.rms_norm_into(batch, out, norm2_w, out2, h, rows, eps)

        product_norm(w.attn_output, bs.attn_out, w.attn_post_norm, input, bs.attn_resid, None, w.ffn_norm, bs.normed)
        if self.fuse_norm_chain and _groupable(w.ffn_gate, w.ffn_up):
            kernels.matmul_nt_quant_gelu_mul_into(batch, w.ffn_gate.ty, bs.normed, w.ffn_gate.buf, w.ffn_up.buf, bs.gate, rows,
                                                  w.ffn_gate.cols, inter)
        else:
            self._matmuls(batch, kernels, [w.ffn_gate, w.ffn_up], bs.normed, [bs.gate, bs.up], rows)
            kernels.gelu_mul_into(batch, bs.gate, bs.up, bs.gate, rows * inter)
        if has_ple:
            product_norm(w.ffn_down, bs.gate, w.ffn_post_norm, bs.attn_resid, output)
        else:
            product_norm(w.ffn_down, bs.gate, w.ffn_post_norm, bs.attn_resid, output, self._output_scale, next_norm,
                         bs.normed if next_norm is not None else None)
        if has_ple:
            ple_buf, n_layer_total = ple_all
            pld = p.per_layer_dim
            g = w.per_layer_inp_gate
            if self.fuse_norm_chain and g.ty != W_F16 and pld % 8 == 0:
                # product, slice (read in place out of every row's per-layer inputs) and GeGLU in one step
                kernels.matmul_nt_quant_gelu_mul_strided_into(batch, g.ty, output, g.buf, rows, g.cols, g.rows, ple_buf,
                                                              n_layer_total * pld, p.layer_idx * pld, bs.ple_g)
            elif self.fuse_norm_chain:
                g.matmul_nt_into(batch, kernels, output, bs.ple_g, rows)
                kernels.gelu_mul_strided_into(batch, bs.ple_g, ple_buf, n_layer_total * pld, p.layer_idx * pld, bs.ple_g, pld,
                                              rows)
            else:
                g.matmul_nt_into(batch, kernels, output, bs.ple_g, rows)
                kernels.gather_strided_f16_into(batch, ple_buf, bs.ple_slice, n_layer_total * pld, p.layer_idx * pld, pld,
                                                rows)
                kernels.gelu_mul_into(batch, bs.ple_g, bs.ple_slice, bs.ple_g, rows * pld)
            product_norm(w.per_layer_proj, bs.ple_g, w.per_layer_post_norm, output, output, self._output_scale,
                         next_norm, bs.normed if next_norm is not None else None)

    def _check_rows(self, rows: int, bs: BatchScratch) -> None:
        if rows == 0 or rows > bs.max_batch:
            raise InvalidArgument(f"rows {rows} outside 1..={bs.max_batch} (BatchScratch capacity)")

    # -------------------------------------- n consecutive rows of one sequence
    def forward_batch(self, kernels: Kernels, batch, n_rows: int, start_pos: int, input: Buffer, output: Buffer,
                      bs: BatchScratch, ones: Buffer, kv_cache: QuantizedKvCache, ple_all=None, prenormed: bool = False,
                      next_norm: Optional[Buffer] = None) -> None:
        """layer.rs:542-718: rows at positions ``start_pos .. start_pos + n_rows``; ``ple_all`` is
        ``(buffer [n_rows, n_layer_total, per_layer_dim] f16, n_layer_total)``.  ``prenormed``: ``bs.normed`` already
        holds this layer's attention norm of ``input`` (the previous layer was given this layer's norm weight as its
        ``next_norm``)."""
        self._check_rows(n_rows, bs)
        p, w = self.params, self.weights
        rows, h, hd, n_head, n_kv, eps = n_rows, p.hidden_size, p.head_dim, p.num_attention_heads, \
            p.num_key_value_heads, p.rms_norm_eps
        kv_len = start_pos + n_rows

        own_kv = not p.is_kv_shared and w.attn_k is not None and w.attn_v is not None
        one_prepare = self._one_prepare()
        if not prenormed:
            kernels.rms_norm_into(batch, input, w.attn_norm, bs.normed, h, rows, eps)
        if own_kv and one_prepare and self._qkv_as_one():
            # the three projections and the preparation as one step: the preparation sums the product's k-split tiles
            kv_cache.project_and_prepare_rows_into(batch, kernels, w.attn_q.ty, bs.normed, w.attn_q.buf, w.attn_k.buf,
                                                   w.attn_v.buf, w.attn_q.cols, bs.q, bs.k, bs.v, w.q_norm, w.k_norm, bs.rq,
                                                   start_pos, n_rows, n_head, eps, p.rope_theta, p.partial_rotary_factor)
            kv_cache.attention_rows_from_rotated_into(batch, kernels, bs.rq, bs.vacc, bs.attn_out, kv_len, start_pos, rows,
                                                      n_head, p.sliding_window)
            self._attention_tail(kernels, batch, rows, input, output, bs, ple_all, next_norm)
            return
        if own_kv:
            self._matmuls(batch, kernels, [w.attn_q, w.attn_k, w.attn_v], bs.normed, [bs.q, bs.k, bs.v], rows)
        else:
            w.attn_q.matmul_nt_into(batch, kernels, bs.normed, bs.q, rows)
        if one_prepare:   # head norms, RoPE, V norm, both encodes and the query rotation of all rows in one dispatch
            kv_cache.prepare_rows_into(batch, kernels, bs.q, bs.k if own_kv else None, bs.v if own_kv else None, w.q_norm,
                                       w.k_norm, bs.rq, start_pos, n_rows, n_head, eps, p.rope_theta,
                                       p.partial_rotary_factor)
            kv_cache.attention_rows_from_rotated_into(batch, kernels, bs.rq, bs.vacc, bs.attn_out, kv_len, start_pos, rows,
                                                      n_head, p.sliding_window)
        else:
            if w.q_norm is not None:
                kernels.qk_norm_gpu_into(batch, bs.q, w.q_norm, hd, rows * n_head, eps)
            kernels.rope_batch_into(batch, bs.q, start_pos, p.rope_theta, hd, n_head, rows, p.partial_rotary_factor)
            if own_kv:
                if w.k_norm is not None:
                    kernels.qk_norm_gpu_into(batch, bs.k, w.k_norm, hd, rows * n_kv, eps)
                kernels.rms_norm_into(batch, bs.v, ones, bs.v, hd, rows * n_kv, eps)
                kernels.rope_batch_into(batch, bs.k, start_pos, p.rope_theta, hd, n_kv, rows, p.partial_rotary_factor)
                kv_cache.write_kv_gpu_into(batch, kernels, bs.k, bs.v, start_pos, n_rows)
            kv_cache.fused_attention_batch_into(batch, kernels, bs.q, bs.rq, bs.vacc, bs.attn_out, kv_len, start_pos, rows,
                                                n_head, p.sliding_window)
        self._attention_tail(kernels, batch, rows, input, output, bs, ple_all, next_norm)

    # ---------------------------- one row per independent lane (continuous batching)
    def forward_decode_batch_turbo(self, batch, kernels: Kernels, n_lanes: int, positions: Buffer, input: Buffer,
                                   output: Buffer, bs: BatchScratch, ones: Buffer, pool: QuantizedUnifiedKvPool,
                                   ple_all=None, prenormed: bool = False, next_norm: Optional[Buffer] = None) -> None:
        """layer.rs:731-873: ``positions`` is a device ``[n_lanes]`` u32 buffer shared by rope, the KV scatter
        and attention; ``prenormed`` / ``next_norm`` as in ``forward_batch``."""
        self._check_rows(n_lanes, bs)
        p, w = self.params, self.weights
        rows, h, hd, n_head, n_kv, eps = n_lanes, p.hidden_size, p.head_dim, p.num_attention_heads, \
            p.num_key_value_heads, p.rms_norm_eps

        own_kv = not p.is_kv_shared and w.attn_k is not None and w.attn_v is not None
        one_prepare = self._one_prepare()
        if not prenormed:
            kernels.rms_norm_into(batch, input, w.attn_norm, bs.normed, h, rows, eps)
        if own_kv and one_prepare and self._qkv_as_one():
            # the three projections and the preparation as one step: the preparation sums the product's k-split tiles
            pool.project_and_prepare_lanes_into(batch, kernels, w.attn_q.ty, bs.normed, w.attn_q.buf, w.attn_k.buf,
                                                w.attn_v.buf, w.attn_q.cols, bs.q, bs.k, bs.v, w.q_norm, w.k_norm, bs.rq,
                                                positions, n_lanes, n_head, eps, p.rope_theta, p.partial_rotary_factor)
            pool.attention_from_rotated_into(batch, kernels, bs.rq, bs.vacc, bs.attn_out, positions, n_head,
                                             p.sliding_window, n_lanes)
            self._attention_tail(kernels, batch, rows, input, output, bs, ple_all, next_norm)
            return
        if own_kv:
            self._matmuls(batch, kernels, [w.attn_q, w.attn_k, w.attn_v], bs.normed, [bs.q, bs.k, bs.v], rows)
        else:
            w.attn_q.matmul_nt_into(batch, kernels, bs.normed, bs.q, rows)
        if one_prepare:   # every lane's head norms, RoPE, V norm, encodes and query rotation in one dispatch
            pool.prepare_lanes_into(batch, kernels, bs.q, bs.k if own_kv else None, bs.v if own_kv else None, w.q_norm,
                                    w.k_norm, bs.rq, positions, n_lanes, n_head, eps, p.rope_theta,
                                    p.partial_rotary_factor)
            pool.attention_from_rotated_into(batch, kernels, bs.rq, bs.vacc, bs.attn_out, positions, n_head,
                                             p.sliding_window, n_lanes)
        else:
            if w.q_norm is not None:
                kernels.qk_norm_gpu_into(batch, bs.q, w.q_norm, hd, rows * n_head, eps)
            kernels.rope_batch_decode_into(batch, bs.q, positions, p.rope_theta, hd, n_head, rows,
                                           p.partial_rotary_factor)
            if own_kv:
                if w.k_norm is not None:
                    kernels.qk_norm_gpu_into(batch, bs.k, w.k_norm, hd, rows * n_kv, eps)
                kernels.rms_norm_into(batch, bs.v, ones, bs.v, hd, rows * n_kv, eps)
                kernels.rope_batch_decode_into(batch, bs.k, positions, p.rope_theta, hd, n_kv, rows,
                                               p.partial_rotary_factor)
                pool.write_kv_into(batch, kernels, bs.k, bs.v, positions, n_lanes)
            pool.attention_into(batch, kernels, bs.q, bs.rq, bs.vacc, bs.attn_out, positions, n_head, p.sliding_window,
                                n_lanes)
        self._attention_tail(kernels, batch, rows, input, output, bs, ple_all, next_norm)
