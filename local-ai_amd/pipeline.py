"""The token-level decode loop around the layers: ``Gemma4QATConfig``'s per-layer geometry
(local-core/src/config/gemma4_qat.rs:170-252), the KV-cache slots with their sharing map
(local-engine/src/pipeline.rs:379-437) and the decode core of ``Pipeline`` -- embedding gather and
scale, per-layer inputs, the layer stack in one command batch, final norm + logits + soft cap
(pipeline.rs:714-953), chunked prompt prefill (pipeline.rs:969-1100, 1332-1367) and the continuous-batching
step over by-lane KV pools (local-engine/src/pipeline/batched.rs:72-478).  Tokenizer, sampling, prompt
caches and the multimodal front ends of the reference's ``Pipeline`` are not part of the hot path and
are not here.

Differences from the reference, all because buffers live in device memory: embedding rows are decoded
by the device dequant kernels instead of by the CPU out of shared memory; a token (set-up, layers,
logits tail) or a batched step is encoded into one batch with a single wait at the end; and the logits
of a batched step come from one [lanes, hidden] x table^T product that reads the embedding table once,
where the reference runs one matvec per lane.
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional

import numpy as np

from . import Buffer, CommandBatch, InvalidArgument, Kernels
from . import F16, F32
from .kv_cache import QuantizedKvCache, QuantizedUnifiedKvPool, kv_bits_from_env, swa_ring_capacity
from .layer import BatchScratch, ScratchBuffers, TransformerLayer
from .quant_weight import QuantWeight

DEFAULT_LOGIT_SOFTCAP = 30.0   # local-engine/src/sampler.rs:30
DEFAULT_MAX_BATCH = 256         # local-engine/src/pipeline.rs:620-622: rows of the shared multi-row scratch


@dataclass
class Gemma4QATConfig:
    """The fields of local-core/src/config/gemma4_qat.rs that shape the decode path."""
    vocab_size: int
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    global_head_dim: int = 0
    max_position_embeddings: int = 131072
    rms_norm_eps: float = 1e-6
    sliding_window: int = 512
    num_kv_shared_layers: int = 0
    hidden_size_per_layer_input: int = 0
    layer_types: List[str] = field(default_factory=list)        # "sliding_attention" | "full_attention"
    sliding_rope_theta: float = 10000.0
    full_rope_theta: Optional[float] = None                     # None: no rope_parameters entry -> 10000
    full_partial_rotary_factor: Optional[float] = None

    def is_full_attention(self, layer_idx: int) -> bool:
        """gemma4_qat.rs:170-185: a layer past the end of the list is a sliding-attention layer."""
        return layer_idx < len(self.layer_types) and self.layer_types[layer_idx] == "full_attention"

    def attn_head_dim(self, layer_idx: int) -> int:
        """gemma4_qat.rs:187-194."""
        return self.global_head_dim if self.is_full_attention(layer_idx) and self.global_head_dim > 0 else self.head_dim

    def rope_theta(self, layer_idx: int) -> float:
        """gemma4_qat.rs:196-208."""
        if self.is_full_attention(layer_idx):
            return self.full_rope_theta if self.full_rope_theta is not None else 10000.0
        return self.sliding_rope_theta

    def partial_rotary_factor(self, layer_idx: int) -> float:
        """gemma4_qat.rs:210-221."""
        if self.is_full_attention(layer_idx) and self.full_partial_rotary_factor is not None:
            return self.full_partial_rotary_factor
        return 1.0

    def first_kv_shared_layer(self) -> int:
        return max(self.num_hidden_layers - self.num_kv_shared_layers, 0)

    def is_kv_shared(self, layer_idx: int) -> bool:
        """gemma4_qat.rs:232-234."""
        return self.num_kv_shared_layers > 0 and layer_idx >= self.first_kv_shared_layer()

    def kv_source_layer(self, layer_idx: int) -> Optional[int]:
        """gemma4_qat.rs:240-248: the last layer of the same attention type that owns its KV."""
        if not self.is_kv_shared(layer_idx):
            return None
        want = self.is_full_attention(layer_idx)
        for j in range(self.first_kv_shared_layer() - 1, -1, -1):
            if self.is_full_attention(j) == want:
                return j
        return None


def build_kv_caches(config: Gemma4QATConfig, layers: List[TransformerLayer], ctx, max_context_length: int,
                    ring_enabled: bool = True):
    """pipeline.rs:379-437: one cache per layer that owns its KV (a ring for sliding-window layers), and the
    layer -> cache index map through which KV-shared layers read their source layer's cache."""
    bits = kv_bits_from_env()
    kv_index_map = [0] * config.num_hidden_layers
    slot_of: List[Optional[int]] = [None] * config.num_hidden_layers
    slots = []
    for layer_idx, layer in enumerate(layers):
        if config.is_kv_shared(layer_idx):
            src = config.kv_source_layer(layer_idx)
            if src is None or slot_of[src] is None:
                raise InvalidArgument(f"no KV source for shared layer {layer_idx}")
            kv_index_map[layer_idx] = slot_of[src]
        else:
            window = 0 if config.is_full_attention(layer_idx) else config.sliding_window
            slot_of[layer_idx] = len(slots)
            kv_index_map[layer_idx] = len(slots)
            slots.append((layer.params.head_dim, window))
    caches = []
    for head_dim, window in slots:
        if ring_enabled and window > 0:
            ring = swa_ring_capacity(window, max_context_length)
            caches.append(QuantizedKvCache(ctx, config.num_key_value_heads, head_dim, max_context_length, bits, ring, window))
        else:
            caches.append(QuantizedKvCache(ctx, config.num_key_value_heads, head_dim, max_context_length, bits))
    return caches, kv_index_map


class BatchedDecodeState:
    """batched.rs:25-60: one by-lane KV pool per cache slot, the lanes' device-resident positions and logits."""

    def __init__(self, ctx, pools: List[QuantizedUnifiedKvPool], n_lanes: int, lane_capacity: int, vocab_size: int):
        self.pools, self.n_lanes, self.lane_capacity = pools, n_lanes, lane_capacity
        self.pos_buf = Buffer.empty(ctx, n_lanes * 4)
        self.logits_buf = Buffer.empty(ctx, n_lanes * vocab_size * 4)   # [n_lanes, vocab] f32
        self._vocab = vocab_size

    def reset_lane(self, lane: int) -> None:
        """batched.rs:55-59."""
        for pool in self.pools:
            pool.reset_lane(lane)

    def logits(self, n: Optional[int] = None) -> np.ndarray:
        n = self.n_lanes if n is None else n
        return self.logits_buf.as_array(np.float32, n * self._vocab).reshape(n, self._vocab)


class DecodePipeline:
    """The decode core of ``Pipeline`` (pipeline.rs:714-953)."""

    def __init__(self, ctx, kernels: Kernels, config: Gemma4QATConfig, layers: List[TransformerLayer],
                 token_embd: QuantWeight, output_norm: Buffer, max_context_length: int, ple_table=None,
                 per_layer_model_proj: Optional[QuantWeight] = None, per_layer_proj_norm: Optional[Buffer] = None,
                 logit_softcap: float = DEFAULT_LOGIT_SOFTCAP, max_batch: int = DEFAULT_MAX_BATCH):
        if len(layers) != config.num_hidden_layers:
            raise InvalidArgument(f"{len(layers)} layers for a {config.num_hidden_layers}-layer configuration")
        if token_embd.rows != config.vocab_size or token_embd.cols != config.hidden_size:
            raise InvalidArgument("token_embd does not match vocab_size x hidden_size")
        self.ctx, self.kernels, self.config, self.layers = ctx, kernels, config, layers
        self.token_embd, self.output_norm, self.logit_softcap = token_embd, output_norm, logit_softcap
        self.ple_table, self.per_layer_model_proj, self.per_layer_proj_norm = ple_table, per_layer_model_proj, per_layer_proj_norm
        self.max_context = max_context_length
        self.kv_caches, self.kv_index_map = build_kv_caches(config, layers, ctx, max_context_length)
        h, pld = config.hidden_size, config.hidden_size_per_layer_input
        self.hidden_a, self.hidden_b = Buffer.empty(ctx, h * 2), Buffer.empty(ctx, h * 2)
        self.logits_buf = Buffer.empty(ctx, config.vocab_size * 4)
        self.scratch = ScratchBuffers(ctx, h, max(l.params.intermediate_size for l in layers), config.num_attention_heads,
                                      config.num_key_value_heads, max(l.params.head_dim for l in layers), pld)
        ple_total = pld * config.num_hidden_layers
        self.per_layer_input = self.ple_tok = self.ple_proj = None
        if ple_table is not None and per_layer_model_proj is not None and per_layer_proj_norm is not None:
            self.per_layer_input, self.ple_tok, self.ple_proj = (Buffer.empty(ctx, ple_total * 2) for _ in range(3))
        self.max_batch = max_batch
        self.defer_layer_tails = True   # single-token decode: a layer's last step rides in the next layer's first dispatch
        self._batch_scratch: Optional[BatchScratch] = None
        self._tokens_buf = self._ple_tokens_buf = None
        self.position = 0
        self.reset()

    @property
    def batch_scratch(self) -> BatchScratch:
        """pipeline.rs:619-630: the shared multi-row scratch of prefill chunks and batched steps (built on first use)."""
        if self._batch_scratch is None:
            cfg = self.config
            self._batch_scratch = BatchScratch(self.ctx, self.max_batch, cfg.hidden_size,
                                               max(l.params.intermediate_size for l in self.layers),
                                               cfg.num_attention_heads, cfg.num_key_value_heads,
                                               max(l.params.head_dim for l in self.layers),
                                               cfg.hidden_size_per_layer_input, cfg.num_hidden_layers)
            self._tokens_buf = Buffer.empty(self.ctx, self.max_batch * 4)
            self._ple_tokens_buf = Buffer.empty(self.ctx, self.max_batch * 4)
        return self._batch_scratch

    @classmethod
    def from_host(cls, ctx, kernels: Kernels, config: Gemma4QATConfig, tensors: dict, max_context_length: int,
                  logit_softcap: float = DEFAULT_LOGIT_SOFTCAP, max_batch: int = DEFAULT_MAX_BATCH,
                  **layer_options) -> "DecodePipeline":
        """Upload host tensors laid out as ``synth.decode_model_tensors`` returns them: ``layers`` (one dict of layer
        tensors each), ``token_embd`` / ``ple_table`` / ``per_layer_model_proj`` as ``(format, rows, cols, payload)``,
        the norms as f16 vectors."""
        from . import Q4_0, TQ2_0
        from .gguf import GGUFType
        from .layer import LayerParams, LayerWeights
        from .weights import QuantRowTable
        fmt_id = {"q4_0": Q4_0, "tq2_0": TQ2_0}
        layers = []
        for i, lt in enumerate(tensors["layers"]):
            w = LayerWeights.from_host(ctx, lt)
            params = LayerParams(layer_idx=i, hidden_size=config.hidden_size, intermediate_size=w.ffn_gate.rows,
                                 num_attention_heads=config.num_attention_heads,
                                 num_key_value_heads=config.num_key_value_heads, head_dim=config.attn_head_dim(i),
                                 per_layer_dim=config.hidden_size_per_layer_input, rope_theta=config.rope_theta(i),
                                 partial_rotary_factor=config.partial_rotary_factor(i),
                                 sliding_window=0 if config.is_full_attention(i) else config.sliding_window,
                                 rms_norm_eps=config.rms_norm_eps, is_kv_shared=config.is_kv_shared(i))
            layers.append(TransformerLayer(params, w, **layer_options))
        fmt, rows, cols, payload = tensors["token_embd"]
        token_embd = QuantWeight.from_bytes(ctx, payload, fmt_id[fmt], rows, cols)
        output_norm = Buffer.from_slice(ctx, np.asarray(tensors["output_norm"], np.float16))
        ple_table = model_proj = proj_norm = None
        if "ple_table" in tensors:
            fmt, rows, cols, payload = tensors["ple_table"]
            ple_table = QuantRowTable.new(ctx, payload, {"q4_0": GGUFType.Q4_0, "tq2_0": GGUFType.TQ2_0}[fmt], cols, rows)
            fmt, rows, cols, payload = tensors["per_layer_model_proj"]
            model_proj = QuantWeight.from_bytes(ctx, payload, fmt_id[fmt], rows, cols)
            proj_norm = Buffer.from_slice(ctx, np.asarray(tensors["per_layer_proj_norm"], np.float16))
        return cls(ctx, kernels, config, layers, token_embd, output_norm, max_context_length, ple_table, model_proj,
                   proj_norm, logit_softcap, max_batch)

    def reset(self) -> None:
        """pipeline.rs:714-717."""
        self.position = 0
        for c in self.kv_caches:
            c.reset()

    def compute_per_layer_inputs(self, batch, token: int) -> None:
        """pipeline.rs:725-776: per_layer_input = (rms_norm(model_proj . h / sqrt(hidden)) + table[token] * sqrt(pld))
        / sqrt(2), one [pld] slice per layer; reads the scaled embedding in hidden_a."""
        if self.per_layer_input is None:
            return
        K, cfg = self.kernels, self.config
        pld, n_layer = cfg.hidden_size_per_layer_input, cfg.num_hidden_layers
        total = pld * n_layer
        self.ple_table.dequant_row_into(batch, K, token, self.ple_tok)
        K.scale_in_place_gpu_into(batch, self.ple_tok, math.sqrt(pld), total)
        self.per_layer_model_proj.matvec_into(batch, K, self.hidden_a, self.ple_proj)
        K.scale_in_place_gpu_into(batch, self.ple_proj, 1.0 / math.sqrt(cfg.hidden_size), total)
        K.rms_norm_into(batch, self.ple_proj, self.per_layer_proj_norm, self.ple_proj, pld, n_layer, cfg.rms_norm_eps)
        K.residual_add_into(batch, self.ple_proj, self.ple_tok, self.per_layer_input, total)
        K.scale_in_place_gpu_into(batch, self.per_layer_input, math.sqrt(0.5), total)

    def gather_embedding(self, batch, token: int, dst: Buffer) -> None:
        """pipeline.rs:781-790 for one token: row `token` of the tied embedding table as hidden_size f16 values."""
        self.token_embd.dequant_row_into(batch, self.kernels, token, dst)

    def forward_token(self, token: int, position: int, ple_token: Optional[int] = None, batch=None) -> bool:
        """pipeline.rs:834-911: embed, scale by sqrt(hidden), per-layer inputs, all layers.  Returns True when the final
        hidden state is in hidden_a.  With `batch` given the work is only encoded (the caller commits)."""
        if position >= self.max_context:
            raise InvalidArgument(f"position {position} beyond the context of {self.max_context}")
        own = batch is None
        batch = batch or CommandBatch(self.ctx)
        cfg, K = self.config, self.kernels
        self.gather_embedding(batch, token, self.hidden_a)
        K.scale_in_place_gpu_into(batch, self.hidden_a, math.sqrt(cfg.hidden_size), cfg.hidden_size)
        self.compute_per_layer_inputs(batch, token if ple_token is None else ple_token)
        # A layer may leave its last step (post-norm, residual, output scale) to the next layer's first dispatch: its input
        # buffer is dead by then and receives the finished hidden state, so the two buffers keep their roles in that case.
        cur_in_a, pend, last = True, None, len(self.layers) - 1
        for i, layer in enumerate(self.layers):
            inp, out = (self.hidden_a, self.hidden_b) if cur_in_a else (self.hidden_b, self.hidden_a)
            pend = layer.forward_decode(K, batch, inp, out, position, self.scratch, self.kv_caches[self.kv_index_map[i]],
                                        self.per_layer_input, cfg.num_hidden_layers, pending=pend,
                                        defer_tail=self.defer_layer_tails and i < last)
            if pend is None:
                cur_in_a = not cur_in_a
        if own:
            batch.commit_and_wait()
        return cur_in_a

    def write_logits(self, final_in_a: bool, batch=None) -> None:
        """pipeline.rs:914-953: output norm, tied-embedding logits (f32), soft cap."""
        own = batch is None
        batch = batch or CommandBatch(self.ctx)
        cfg, K = self.config, self.kernels
        final_hidden = self.hidden_a if final_in_a else self.hidden_b
        # the reference norms into hidden_b even when hidden_b is the input (the kernel is safe in place)
        K.rms_norm_into(batch, final_hidden, self.output_norm, self.hidden_b, cfg.hidden_size, 1, cfg.rms_norm_eps)
        self.token_embd.matvec_f32out_into(batch, K, self.hidden_b, self.logits_buf)
        if self.logit_softcap > 0.0:
            K.logit_softcap_gpu_into(batch, self.logits_buf, self.logit_softcap, cfg.vocab_size)
        if own:
            batch.commit_and_wait()

    def decode_step(self, token: int) -> None:
        """One generated token: forward_token at the current position and the logits tail in one batch, one wait."""
        batch = CommandBatch(self.ctx)
        final_in_a = self.forward_token(token, self.position, batch=batch)
        self.write_logits(final_in_a, batch=batch)
        batch.commit_and_wait()
        self.position += 1

    def logits(self) -> np.ndarray:
        return self.logits_buf.as_array(np.float32, self.config.vocab_size)

    # ---- multi-row paths: prefill chunks and continuous batching ---------------------------------------------------

    def _next_norm(self, i: int) -> Optional[Buffer]:
        """Layer i + 1's attention-norm weight when layer i can apply it in its last dispatch (the norm is then layer
        i + 1's first step, layer.rs:556 / 745, moved across the layer boundary); None for the last layer."""
        if i + 1 < len(self.layers) and self.layers[i].fuse_norm_chain and self.layers[i + 1].fuse_norm_chain:
            return self.layers[i + 1].weights.attn_norm
        return None

    def _embed_rows(self, batch, tokens, ple_tokens) -> bool:
        """pipeline.rs:994-1060 / batched.rs:305-368: rows of the embedding table scaled by sqrt(hidden) into hidden_a,
        and the per-layer inputs of every row into ple_all.  Returns whether per-layer inputs exist."""
        cfg, K, bs = self.config, self.kernels, self.batch_scratch
        n, h = len(tokens), cfg.hidden_size
        self._tokens_buf.copy_from_bytes(np.asarray(tokens, np.uint32))
        self.token_embd.dequant_rows_into(batch, K, self._tokens_buf, n, bs.hidden_a, math.sqrt(h))
        if self.per_layer_input is None:
            return False
        pld, nl = cfg.hidden_size_per_layer_input, cfg.num_hidden_layers
        total = n * pld * nl
        self._ple_tokens_buf.copy_from_bytes(np.asarray(ple_tokens, np.uint32))
        self.ple_table.dequant_rows_into(batch, K, self._ple_tokens_buf, n, bs.ple_tok, math.sqrt(pld))
        self.per_layer_model_proj.matmul_nt_into(batch, K, bs.hidden_a, bs.ple_proj, n)
        K.scale_in_place_gpu_into(batch, bs.ple_proj, 1.0 / math.sqrt(h), total)
        K.rms_norm_into(batch, bs.ple_proj, self.per_layer_proj_norm, bs.ple_proj, pld, n * nl, cfg.rms_norm_eps)
        K.residual_add_into(batch, bs.ple_proj, bs.ple_tok, bs.ple_all, total)
        K.scale_in_place_gpu_into(batch, bs.ple_all, math.sqrt(0.5), total)
        return True

    def forward_tokens_batch(self, tokens, start_pos: int, ple_tokens=None, batch=None) -> bool:
        """pipeline.rs:969-1100: one prefill chunk, rows at positions start_pos .. start_pos + len(tokens), through every
        layer's batch path into the single-sequence caches.  Returns True when the result is in batch_scratch.hidden_a."""
        n = len(tokens)
        ple_tokens = tokens if ple_tokens is None else ple_tokens
        if len(ple_tokens) != n:
            raise InvalidArgument(f"PLE token count {len(ple_tokens)} does not match token count {n}")
        if n < 1 or n > self.max_batch:
            raise InvalidArgument(f"chunk of {n} rows must be in 1..={self.max_batch}")
        if start_pos + n > self.max_context:
            raise InvalidArgument(f"positions up to {start_pos + n} beyond the context of {self.max_context}")
        own = batch is None
        batch = batch or CommandBatch(self.ctx)
        bs = self.batch_scratch
        ple_arg = (bs.ple_all, self.config.num_hidden_layers) if self._embed_rows(batch, tokens, ple_tokens) else None
        cur_in_a, prenormed = True, False
        for i, layer in enumerate(self.layers):
            inp, out = (bs.hidden_a, bs.hidden_b) if cur_in_a else (bs.hidden_b, bs.hidden_a)
            next_norm = self._next_norm(i)
            layer.forward_batch(self.kernels, batch, n, start_pos, inp, out, bs, self.scratch.ones,
                                self.kv_caches[self.kv_index_map[i]], ple_arg, prenormed, next_norm)
            cur_in_a, prenormed = not cur_in_a, next_norm is not None
        if own:
            batch.commit_and_wait()
        return cur_in_a

    def prefill_prompt(self, tokens, chunk_len: Optional[int] = None) -> bool:
        """pipeline.rs:1332-1367 without the prompt cache: all tokens but the last in chunks of at most max_batch rows,
        the last through forward_token so that its hidden state is where write_logits reads it."""
        if len(tokens) == 0:
            raise InvalidArgument("prefill prompt is empty")
        chunk_len = min(chunk_len or self.max_batch, self.max_batch)
        last_idx = len(tokens) - 1
        pos = 0
        while pos < last_idx:
            chunk = tokens[pos:min(pos + chunk_len, last_idx)]
            self.forward_tokens_batch(chunk, pos)
            pos += len(chunk)
        self.position = last_idx
        return self.forward_token(tokens[last_idx], last_idx)

    def new_batched_decode_state(self, n_lanes: int, lane_capacity: int) -> BatchedDecodeState:
        """batched.rs:72-151: one pool per cache slot with the slot's head_dim; a sliding-window slot's lanes are rings of
        the staging cache's size so that a wrapped prefill copies slot for slot."""
        if n_lanes == 0:
            raise InvalidArgument("n_lanes must be >= 1")
        if n_lanes > self.max_batch:
            raise InvalidArgument(f"n_lanes {n_lanes} exceeds batch scratch capacity {self.max_batch}")
        bits = kv_bits_from_env()
        pools = []
        for staging in self.kv_caches:
            lane_ring = 0
            if staging.is_ringed():
                lane_ring = staging.physical_positions
                if lane_capacity < lane_ring:
                    raise InvalidArgument(f"lane_capacity {lane_capacity} below sliding-window ring {lane_ring}")
            pools.append(QuantizedUnifiedKvPool(self.ctx, n_lanes, lane_capacity, self.config.num_key_value_heads,
                                                staging.head_dim, bits, lane_ring))
        return BatchedDecodeState(self.ctx, pools, n_lanes, lane_capacity, self.config.vocab_size)

    def prefill_lane(self, state: BatchedDecodeState, lane: int, tokens) -> np.ndarray:
        """batched.rs:162-197: prefill on the single-sequence caches, keep the last token's logits, copy the encoded
        rows into the lane's region of every pool."""
        if len(tokens) == 0:
            raise InvalidArgument("prefill prompt is empty")
        if lane >= state.n_lanes:
            raise InvalidArgument(f"lane {lane} out of range (n_lanes {state.n_lanes})")
        if len(tokens) > state.lane_capacity:
            raise InvalidArgument(f"prompt length {len(tokens)} exceeds lane_capacity {state.lane_capacity}")
        self.reset()
        final_in_a = self.prefill_prompt(tokens)
        batch = CommandBatch(self.ctx)
        self.write_logits(final_in_a, batch=batch)
        for slot, pool in enumerate(state.pools):
            pool.copy_prefill_from(batch, self.kv_caches[slot], lane, len(tokens))
        batch.commit_and_wait()
        return self.logits().copy()

    def encode_batch_step(self, batch, state: BatchedDecodeState, n: int) -> None:
        """The device work of decode_batch_step for the tokens and positions already uploaded: layers at M = n over the
        lanes' pools (batched.rs:371-409), then output norm, logits and soft cap of every lane (batched.rs:411-455)."""
        cfg, K, bs = self.config, self.kernels, self.batch_scratch
        h = cfg.hidden_size
        ple_arg = (bs.ple_all, cfg.num_hidden_layers) if self.per_layer_input is not None else None
        cur_in_a, prenormed = True, False
        for i, layer in enumerate(self.layers):
            inp, out = (bs.hidden_a, bs.hidden_b) if cur_in_a else (bs.hidden_b, bs.hidden_a)
            next_norm = self._next_norm(i)
            layer.forward_decode_batch_turbo(batch, K, n, state.pos_buf, inp, out, bs, self.scratch.ones,
                                             state.pools[self.kv_index_map[i]], ple_arg, prenormed, next_norm)
            cur_in_a, prenormed = not cur_in_a, next_norm is not None
        final_hidden = bs.hidden_a if cur_in_a else bs.hidden_b
        K.rms_norm_into(batch, final_hidden, self.output_norm, bs.normed, h, n, cfg.rms_norm_eps)
        self.token_embd.matmul_nt_typed_into(batch, K, bs.normed, F16, state.logits_buf, F32, n)
        if self.logit_softcap > 0.0:
            K.logit_softcap_gpu_into(batch, state.logits_buf, self.logit_softcap, n * cfg.vocab_size)

    def decode_batch_step(self, state: BatchedDecodeState, tokens, ple_tokens, positions, read_logits: bool = True):
        """batched.rs:271-478: one token for each of len(tokens) active lanes (lane l is row l), lane l at
        positions[l]; returns the [n, vocab] logits (or leaves them in state.logits_buf with read_logits=False)."""
        n = len(tokens)
        if n == 0 or n > state.n_lanes:
            raise InvalidArgument(f"active lanes {n} must be in 1..={state.n_lanes}")
        if len(ple_tokens) != n or len(positions) != n:
            raise InvalidArgument("tokens, ple_tokens and positions must have equal length")
        for lane, pos in enumerate(positions):
            if pos >= state.lane_capacity:
                raise InvalidArgument(f"lane {lane} position {pos} exceeds capacity {state.lane_capacity}")
        state.pos_buf.copy_from_bytes(np.asarray(positions, np.uint32))
        batch = CommandBatch(self.ctx)
        self._embed_rows(batch, tokens, ple_tokens)
        self.encode_batch_step(batch, state, n)
        batch.commit_and_wait()
        return state.logits(n).copy() if read_logits else None
