/*
 * local_hip.h -- C ABI of the gfx950 (MI355X) decode hot-path library.
 *
 * The library replaces, for Q4_0 / TQ2_0 quantized weights and the TurboQuant
 * KV cache, the kernel-dispatch layer that local-engine calls on local-metal
 * (local-metal/src/kernels.rs `Kernels`, plus batch.rs / buffer.rs / context.rs /
 * error.rs).  Every entry point below names the reference interface it stands
 * in for.  Conventions:
 *
 *  - Opaque handles; plain integers by value; no C++ / torch types.
 *  - Every call returns an lh_status (0 = OK).  On failure the message is kept
 *    per thread and read with lh_last_error(); its text follows the Display
 *    form of local_metal::Error (local-metal/src/error.rs:1-32), e.g.
 *    "Invalid argument: matvec_q4_0: cols 100 not /32".
 *  - `*_into` calls enqueue work on the context's single in-order HIP stream
 *    (the stand-in for one serial MTLComputeCommandEncoder: later dispatches
 *    see earlier dispatches' results) and return immediately; the blocking
 *    forms without `_into` enqueue and wait, as the reference's do.
 *  - Arguments are validated on the host (alignment of `cols`, buffer sizes
 *    against the shapes) before anything is launched.
 *  - Matrices are [rows(N), cols(K)] row-major in verbatim GGUF block layout
 *    (local-engine/src/layer.rs:16-17, shaders/matvec_quant.metal:11-17).
 *  - One owner thread per context (local-engine/src/cli/serve.rs:3-11).
 */
#ifndef LOCAL_HIP_H
#define LOCAL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LH_API __attribute__((visibility("default")))

/* local-metal/src/error.rs:1-32 */
typedef enum lh_status {
    LH_OK = 0,
    LH_ERR_NO_DEVICE = 1,           /* NoMetalDevice / NoDevice */
    LH_ERR_NO_COMMAND_QUEUE = 2,    /* NoCommandQueue (stream creation failed) */
    LH_ERR_BUFFER_ALLOCATION = 3,   /* BufferAllocation{size,reason} */
    LH_ERR_LIBRARY_CREATION = 4,    /* LibraryCreation */
    LH_ERR_PIPELINE_CREATION = 5,   /* PipelineCreation (kernel unavailable) */
    LH_ERR_SHADER_NOT_FOUND = 6,    /* ShaderNotFound */
    LH_ERR_COMMAND_BUFFER = 7,      /* CommandBuffer("GPU error: ...") */
    LH_ERR_INVALID_ARGUMENT = 8,    /* InvalidArgument */
    LH_ERR_IO = 9                   /* Io */
} lh_status;

typedef struct lh_context lh_context;  /* local-metal/src/context.rs:31 MetalContext (device + queue) */
typedef struct lh_buffer lh_buffer;    /* local-metal/src/buffer.rs:17 MetalBuffer */
typedef struct lh_batch lh_batch;      /* local-metal/src/batch.rs:21 CommandBatch */

/* Element types of activation / output buffers for the typed entry points. */
typedef enum lh_dtype { LH_F16 = 0, LH_F32 = 1, LH_BF16 = 2 } lh_dtype;
/* Weight block formats (local-engine/src/gguf.rs:247-268 block_size). */
typedef enum lh_quant { LH_Q4_0 = 0, LH_TQ2_0 = 1 } lh_quant;

LH_API const char* lh_last_error(void);
LH_API const char* lh_version(void);

/* ---- context: MetalContext::new / device_name / caps (context.rs:38-86) ---- */
LH_API int lh_context_create(int device_index, lh_context** out);
/* Waits for the stream and drops the creator's handle.  Buffers, batches and events made from the
 * context keep its stream and workspace alive until the last of them is freed, so handles may be
 * released in any order (as Rust's drop order lets the reference's owners do); `ctx` itself must not
 * be passed to any call afterwards. */
LH_API void lh_context_destroy(lh_context* ctx);
LH_API int lh_context_device_name(const lh_context* ctx, char* dst, size_t dst_len);
LH_API int lh_context_compute_units(const lh_context* ctx);
LH_API void* lh_context_stream(const lh_context* ctx);          /* hipStream_t, for interop */
LH_API int lh_context_synchronize(lh_context* ctx);

/* ---- timing: HIP events recorded on the context's stream (stands in for the
 *      reference's LOCAL_AI_TIMING wall-clock timers, local-engine/src/pipeline.rs:124-127,
 *      with device-side time stamps). ---- */
typedef struct lh_event lh_event;
LH_API int lh_event_create(lh_context* ctx, lh_event** out);
LH_API void lh_event_destroy(lh_event* ev);
LH_API int lh_event_record(lh_event* ev);                       /* enqueue on the context stream */
LH_API int lh_event_elapsed_ms(lh_event* start, lh_event* stop, float* ms); /* waits for `stop` */

/* ---- buffers: MetalBuffer::{from_slice, empty, length, as_slice,
 *      copy_from_bytes} (buffer.rs:28-131).  Device memory is not host-mapped
 *      on a discrete GPU, so host access is an explicit copy, ordered after all
 *      work already enqueued on the context. ---- */
LH_API int lh_buffer_from_bytes(lh_context* ctx, const void* src, size_t len, lh_buffer** out);
LH_API int lh_buffer_empty(lh_context* ctx, size_t len, lh_buffer** out);      /* zero-filled */
LH_API int lh_buffer_view(lh_buffer* parent, size_t offset, size_t len, lh_buffer** out); /* non-owning */
LH_API int lh_buffer_wrap(lh_context* ctx, void* device_ptr, size_t len, lh_buffer** out); /* non-owning */
LH_API void lh_buffer_free(lh_buffer* buf);
LH_API size_t lh_buffer_length(const lh_buffer* buf);
LH_API void* lh_buffer_device_ptr(const lh_buffer* buf);
LH_API int lh_buffer_write(lh_buffer* buf, size_t offset, const void* src, size_t len);
LH_API int lh_buffer_read(const lh_buffer* buf, size_t offset, void* dst, size_t len);
LH_API int lh_buffer_fill_zero(lh_buffer* buf);                 /* quant_cache.rs:367-380 reset() */

/* ---- command batch: CommandBatch::{new, dispatch_count, blit_buffer_copies,
 *      commit_and_wait, submit_and_renew, commit_and_renew} (batch.rs:154-291) ---- */
LH_API int lh_batch_new(lh_context* ctx, lh_batch** out);
LH_API void lh_batch_free(lh_batch* batch);
LH_API uint32_t lh_batch_dispatch_count(const lh_batch* batch);
LH_API int lh_batch_blit_copy(lh_batch* batch, const lh_buffer* src, size_t src_offset, lh_buffer* dst,
                              size_t dst_offset, size_t len);
/* Waits for the stream.  Besides HIP errors this reports, as LH_ERR_COMMAND_BUFFER, a kernel of the batch that gave
 * up a bounded wait of its own (the split form of the TQ2_0 matvec polls an LDS word for the previous use of a ring
 * slot; were that ever to run out, the wave goes on so that the kernel still ends, stores a code in a word of pinned
 * host memory, and the outputs of the batch are not valid).  PendingCommandBuffer::wait, batch.rs:136-144. */
LH_API int lh_batch_commit_and_wait(lh_batch* batch);
/* Test hook, no counterpart in the reference: the number of polls the wait above is good for (default 2^20).  A
 * test sets it to 0 to see the error path taken without any kernel hanging, and restores it afterwards. */
LH_API void lh_debug_set_tq2_split_spin_limit(uint32_t polls);
/* The same for the attention kernels that work on several chunks of positions per workgroup: a chunk's two waves
 * meet at their hand-overs through counters in LDS, with a bounded poll (default 2^22) that reports in the same way. */
LH_API void lh_debug_set_attention_pair_spin_limit(uint32_t polls);
LH_API int lh_batch_submit_and_renew(lh_batch* batch);
LH_API int lh_batch_commit_and_renew(lh_batch* batch);

/* ---- recorded batches (no counterpart in the reference: a Metal command buffer is encoded anew for
 *      every commit, batch.rs:240-291).  A decode step is a fixed sequence of some hundreds of short
 *      dispatches, and issuing them one by one costs more host time than the GPU needs to run them; the
 *      sequence is recorded once into a HIP graph and replayed with one call per step.  Between
 *      begin_capture and end_capture every `*_into` call on the context is recorded instead of run; calls
 *      that wait, allocate, copy from host memory or clear a buffer return LH_ERR_INVALID_ARGUMENT (and so
 *      does a grouped matvec of more than two problems).  Whatever changes from step to step must live in
 *      device buffers the recorded kernels read (positions: rope_batch_decode, encode_kv_turboquant_batched,
 *      flash_attention_tq_batched; inputs: write them into the same buffers before each replay). ---- */
typedef struct lh_graph lh_graph;
LH_API int lh_batch_begin_capture(lh_batch* batch);
LH_API int lh_batch_end_capture(lh_batch* batch, lh_graph** out);
LH_API int lh_graph_launch(lh_graph* graph);                    /* enqueues one replay on the context stream */
LH_API uint32_t lh_graph_dispatch_count(const lh_graph* graph);
LH_API void lh_graph_free(lh_graph* graph);

/* ---- M = 1 fused dequant matvec: y[rows] = W[rows, cols] . x[cols] ----------
 * kernels.rs:5711-5838 matvec_q4_0{,_into,_f32out,_f32out_into};
 * kernels.rs:5848-6038 matvec_tq2_0{,_into,_f32out,_f32out_into};
 * shaders/matvec_quant.metal:65-155, 173-312.  x is f16; y f16 or f32.
 * cols % 32 (Q4_0) / % 256 (TQ2_0) != 0 -> LH_ERR_INVALID_ARGUMENT.
 * Numerics: x is taken to 16-bit fixed point per weight block (a block whose
 * maximum stands out from its other elements gets a second 16-bit level), the
 * integer products are exact, and the block sums are combined in f32: within
 * 1e-3 of the reference's f32 dot relative to the output's scale.  In the
 * reference tests' own form, |g - w| <= tol * max(|w|, 1), that holds as well
 * except for TQ2_0 rows of 8192 columns and more against a vector in which
 * EVERY block has one element just under 32 x the mean of its other elements
 * (the second level starts at 32): there the outputs are small (|y| ~ 10),
 * that form judges them absolutely, and the error reaches 1.2e-3 (1.4e-4 of
 * the output's scale).  A NaN or an
 * infinity in x makes every output row NaN (the f32 dot would give NaN, or an
 * infinity where no opposite one cancels it); it is never clamped to a finite
 * value. */
LH_API int lh_matvec_q4_0(lh_context* ctx, const lh_buffer* matrix, const lh_buffer* vector, lh_buffer* output,
                          uint32_t rows, uint32_t cols);
LH_API int lh_matvec_q4_0_into(lh_batch* batch, const lh_buffer* matrix, const lh_buffer* vector, lh_buffer* output,
                               uint32_t rows, uint32_t cols);
LH_API int lh_matvec_q4_0_f32out(lh_context* ctx, const lh_buffer* matrix, const lh_buffer* vector,
                                 lh_buffer* output, uint32_t rows, uint32_t cols);
LH_API int lh_matvec_q4_0_f32out_into(lh_batch* batch, const lh_buffer* matrix, const lh_buffer* vector,
                                      lh_buffer* output, uint32_t rows, uint32_t cols);
LH_API int lh_matvec_tq2_0(lh_context* ctx, const lh_buffer* matrix, const lh_buffer* vector, lh_buffer* output,
                           uint32_t rows, uint32_t cols);
LH_API int lh_matvec_tq2_0_into(lh_batch* batch, const lh_buffer* matrix, const lh_buffer* vector, lh_buffer* output,
                                uint32_t rows, uint32_t cols);
LH_API int lh_matvec_tq2_0_f32out(lh_context* ctx, const lh_buffer* matrix, const lh_buffer* vector,
                                  lh_buffer* output, uint32_t rows, uint32_t cols);
LH_API int lh_matvec_tq2_0_f32out_into(lh_batch* batch, const lh_buffer* matrix, const lh_buffer* vector,
                                       lh_buffer* output, uint32_t rows, uint32_t cols);
/* kernels.rs:5919-5971 matvec_tq2_0_soa_into: qs[rows*cols/256*64] u8 and
 * scales[rows*cols/256] f16 split out of the 66-byte blocks
 * (shaders/matvec_quant.metal:314-387). */
LH_API int lh_matvec_tq2_0_soa_into(lh_batch* batch, const lh_buffer* qs, const lh_buffer* scales,
                                    const lh_buffer* vector, lh_buffer* output, uint32_t rows, uint32_t cols);
/* Same matvec with the activation / output element type chosen by the caller
 * (fp32 x and fp32 y are what the measured configurations use; the reference's
 * GPU path is f16-only, its CPU path is f32).  No reference counterpart beyond
 * the four variants above. */
LH_API int lh_matvec_quant_typed_into(lh_batch* batch, lh_quant fmt, const lh_buffer* matrix,
                                      const lh_buffer* vector, lh_dtype vector_dtype, lh_buffer* output,
                                      lh_dtype output_dtype, uint32_t rows, uint32_t cols);
/* `count` independent matvecs of one shape in a single launch (what the
 * reference's decode loop issues back to back inside one command buffer,
 * kernels.rs:8883-9020: e.g. gate+up, or Q/K/V, which share x).  Arrays are
 * host arrays of buffer handles. */
LH_API int lh_matvec_quant_grouped_into(lh_batch* batch, lh_quant fmt, uint32_t count,
                                        const lh_buffer* const* matrices, const lh_buffer* const* vectors,
                                        lh_dtype vector_dtype, lh_buffer* const* outputs, lh_dtype output_dtype,
                                        uint32_t rows, uint32_t cols);
/* 1..8 matvecs of one shape against ONE f16 vector that is transformed while it is staged, so the
 * kernel that would have produced the transformed vector is not dispatched (a single-token decode
 * step is bound by the number of dispatches).  Replaces, in layer.rs:387-392 / 468-482,
 *   LH_PROLOGUE_RMS_NORM: rms_norm_into(x, aux = weight, eps) followed by matvec_*_into      (attn_norm -> Q, K, V;
 *                         ffn_norm -> gate, up)
 *   LH_PROLOGUE_GELU_MUL: gelu_mul_into(x = gate, aux = up) followed by matvec_*_into       (-> down)
 * The transformed value is rounded to f16 exactly where the separate kernel would have stored it.
 * f16 vector and outputs; cols a multiple of 64 and 16-byte aligned operands, else INVALID_ARGUMENT. */
typedef enum lh_prologue { LH_PROLOGUE_RMS_NORM = 1, LH_PROLOGUE_GELU_MUL = 2 } lh_prologue;
/* The same for the norm chain between two sub-blocks of a layer (layer.rs:452-475, 484-510): the staged vector is
 *   t = f16(rms_norm(vector) * weight + residual)           as rms_norm_add_into computes it (residual may be NULL),
 *   then, when `next_weight` is given, f16(rms_norm(t) * next_weight)   as the following rms_norm_into would;
 * `store` (optional) receives t, written once, for the later residual.  It may alias none of the other operands. */
LH_API int lh_matvec_quant_norm_chain_into(lh_batch* batch, lh_quant fmt, uint32_t count, const lh_buffer* const* matrices,
                                           const lh_buffer* vector, const lh_buffer* weight, const lh_buffer* residual,
                                           const lh_buffer* next_weight, lh_buffer* store, float eps,
                                           lh_buffer* const* outputs, uint32_t rows, uint32_t cols);
/* The chain across two layers (layer.rs:503-520 of one layer, 387-392 of the next): the staged vector is the layer
 * output that rms_norm_residual_scale_into would have written,
 *   t = f16(f16(f16(rms_norm(vector) * weight) + residual) * scale)     (the scale only with `apply_scale`),
 * stored once in `store` (required: it is the next layer's input and first residual), then
 * f16(rms_norm(t) * next_weight) as that layer's attention norm (or t itself when `next_weight` is NULL). */
LH_API int lh_matvec_quant_norm_chain_tail_into(lh_batch* batch, lh_quant fmt, uint32_t count, const lh_buffer* const* matrices,
                                                const lh_buffer* vector, const lh_buffer* weight, const lh_buffer* residual,
                                                int apply_scale, float scale, const lh_buffer* next_weight, lh_buffer* store,
                                                float eps, lh_buffer* const* outputs, uint32_t rows, uint32_t cols);
/* One matvec whose input is rotated out of TurboQuant code space while it is staged: replaces, in
 * quant_cache.rs:590-598 followed by layer.rs:440-446, hadamard_rotate_fh_into(vector, signs, pre_sign = false,
 * post_sign = true) followed by matvec_*_into(matrix, that f16 vector).  `vector` = f32[cols] head outputs of the
 * attention kernel, cols = heads x head_dim; the staged value is f16(H(x) / sqrt(head_dim) * signs) exactly as the
 * rotation kernel would have stored it.  f16 output; head_dim a power of two in 8..=512 that divides cols, cols a
 * multiple of 64, 16-byte aligned operands, else INVALID_ARGUMENT. */
LH_API int lh_matvec_quant_rotated_into(lh_batch* batch, lh_quant fmt, const lh_buffer* matrix, const lh_buffer* vector,
                                        const lh_buffer* signs, uint32_t head_dim, lh_buffer* output, uint32_t rows,
                                        uint32_t cols);
LH_API int lh_matvec_quant_fused_into(lh_batch* batch, lh_quant fmt, uint32_t count, const lh_buffer* const* matrices,
                                      const lh_buffer* vector, int prologue, const lh_buffer* aux, float eps,
                                      lh_buffer* const* outputs, uint32_t rows, uint32_t cols);

/* ---- small-M / prefill quantized matmul: C[m,n] = A[m,k] . W[n,k]^T ----------
 * kernels.rs:6459-6563 matmul_nt_{q4_0,tq2_0}_into (routes by m:
 * batchm / smallm / mma / scalar), kernels.rs:6378-6457 multivec_nt_*_into
 * (1 <= m <= 16), layer.rs:218-246.  A and C are f16 row-major. */
LH_API int lh_matmul_nt_q4_0_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight,
                                  lh_buffer* output, uint32_t m, uint32_t k, uint32_t n);
LH_API int lh_matmul_nt_tq2_0_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight,
                                   lh_buffer* output, uint32_t m, uint32_t k, uint32_t n);
LH_API int lh_multivec_nt_q4_0_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight,
                                    lh_buffer* output, uint32_t m, uint32_t k, uint32_t n);
LH_API int lh_multivec_nt_tq2_0_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight,
                                     lh_buffer* output, uint32_t m, uint32_t k, uint32_t n);
/* Typed form: A f16 / f32 / bf16, C f16 / f32 (the measured small-batch and
 * prefill configurations use f32 and bf16 activations).  Up to 16 rows of f32
 * activations run as rows of the matvec and stay f32; up to 32 rows (TQ2_0
 * from 10 rows on) enter the matrix cores as two f16 rows each, the rounded
 * value and the remainder, and keep about 22 bits (magnitudes up to 131008
 * stay finite: the first part of a value beyond the f16 range is held at
 * 65504; beyond that the outputs are non-finite).  Larger products multiply
 * in f16 like the reference's kernels, whose activations are f16
 * (kernels.rs:6459-6563): bf16 activations convert exactly (down to the f16
 * subnormals), f32 activations are rounded to f16 first, which costs up to
 * 3e-4 of the largest output in absolute terms. */
LH_API int lh_matmul_nt_quant_typed_into(lh_batch* batch, lh_quant fmt, const lh_buffer* input, lh_dtype input_dtype,
                                         const lh_buffer* weight, lh_buffer* output, lh_dtype output_dtype,
                                         uint32_t m, uint32_t k, uint32_t n);
/* The feed-forward gate and up projections and their gelu_mul as one encoded step:
 * out[m, n] = half(gelu(half(in . w_gate^T)) * half(in . w_up^T)) -- matmul_nt_into twice and gelu_mul_into of the
 * multi-row layer paths (local-engine/src/layer.rs:652-662), with their roundings, so the result is theirs bit for
 * bit.  For a decode batch or prefill chunk (17 .. 256 rows) whose pair needs no k split this is a single kernel that
 * pairs gate and up rows in one workgroup; other shapes run the grouped product into the workspace and gelu_mul. */
LH_API int lh_matmul_nt_quant_gelu_mul_into(lh_batch* batch, lh_quant fmt, const lh_buffer* input, const lh_buffer* w_gate,
                                            const lh_buffer* w_up, lh_buffer* output, uint32_t m, uint32_t k, uint32_t n);
/* The per-layer-input gate of the multi-row layer paths as one encoded step (local-engine/src/layer.rs:686-700:
 * matmul_nt_into, gather_strided_f16_into, gelu_mul_into):
 * out[r, i] = half(gelu(half((in . w^T)[r, i])) * gate_rows[r * row_stride + row_offset + i]), bit for bit the
 * separate kernels' result; for a decode batch the gelu kernel sums the product's k-split partial tiles itself.
 * n, row_stride and row_offset must be multiples of 8, the buffers 16-byte aligned. */
LH_API int lh_matmul_nt_quant_gelu_mul_strided_into(lh_batch* batch, lh_quant fmt, const lh_buffer* input,
                                                    const lh_buffer* weight, uint32_t m, uint32_t k, uint32_t n,
                                                    const lh_buffer* gate_rows, uint32_t row_stride,
                                                    uint32_t row_offset, lh_buffer* output);
/* A product followed by the row-wise norm that consumes it, as one encoded step: out = rms_norm(in[m, k] . w^T,
 * norm_weight) (+ residual) (* scale), and with norm2_weight also out2 = rms_norm(out, norm2_weight).  This is the
 * sequence matmul_nt_into -> rms_norm_add_into (-> scale_in_place_gpu_into) (-> rms_norm_into) of the multi-row layer
 * paths -- local-engine/src/layer.rs:640-652 (attention output, post-attention norm + residual, feed-forward norm),
 * 664-672 (down projection, post-feed-forward norm + residual), 699-716 (per-layer projection, its norm + residual,
 * the layer's output scale) -- with the roundings of the separate kernels, so the results are theirs bit for bit.  For
 * a decode batch or prefill chunk (17 .. 256 rows) the norm kernel sums the product's k-split partial tiles itself, which removes the
 * reduction pass as well.  residual / norm2_weight / out2 may be NULL; out may alias residual; n must be a multiple
 * of 8, at most 8192, and every buffer 16-byte aligned. */
LH_API int lh_matmul_nt_quant_norm_into(lh_batch* batch, lh_quant fmt, const lh_buffer* input, const lh_buffer* weight,
                                        uint32_t m, uint32_t k, uint32_t n, const lh_buffer* norm_weight,
                                        const lh_buffer* residual, lh_buffer* output, float eps, int apply_scale,
                                        float scale, const lh_buffer* norm2_weight, lh_buffer* output2);
/* Up to four weight matrices of one format and one k against the same activations as one launch (what layer.rs:570-590 /
 * 658-662 issue back to back: Q, K and V, or gate and up), f16 in and out; output i is [m, ns[i]].  Shapes the separate
 * calls would send to other kernels (m <= 16, or enough 128-row tiles to fill the chip) are issued as those calls. */
LH_API int lh_matmul_nt_quant_grouped_into(lh_batch* batch, lh_quant fmt, uint32_t count, const lh_buffer* input,
                                           const lh_buffer* const* weights, lh_buffer* const* outputs, const uint32_t* ns,
                                           uint32_t m, uint32_t k);
/* kernels.rs:5517-5568 matmul_nt_into: FP16 weights, shaders/matmul_f16.metal:74-114. */
LH_API int lh_matmul_nt_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight, lh_buffer* output,
                             uint32_t m, uint32_t k, uint32_t n);
/* kernels.rs:3244-3330 clipped_linear_tiled_nt_into (shaders/matmul_f16.metal:121-170):
 * output = clamp(clamp(input, input_min, input_max) . weight^T + bias, output_min, output_max), all f16,
 * input [m, k], weight [n, k], bias [n] or NULL. */
LH_API int lh_clipped_linear_tiled_nt_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight,
                                           const lh_buffer* bias, lh_buffer* output, uint32_t m, uint32_t k, uint32_t n,
                                           float input_min, float input_max, float output_min, float output_max);
/* ---- FP16-weight matvec family (shaders/matvec_f16.metal:14-133), the QuantWeight fallbacks for tensors kept as
 * F16 (layer.rs:134, 158, 182).  matrix [rows, cols] f16 starting matrix_offset bytes into its buffer; f32 accumulate. */
/* kernels.rs:582-640 matvec (f16 x, f16 y; enqueue and wait) and 1710-1764 matvec_offset_into */
LH_API int lh_matvec(lh_context* ctx, const lh_buffer* matrix, const lh_buffer* vector, lh_buffer* output,
                     uint32_t rows, uint32_t cols);
LH_API int lh_matvec_offset_into(lh_batch* batch, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector,
                                 lh_buffer* output, uint32_t rows, uint32_t cols);
/* kernels.rs:1766-1874 matvec_f32out_offset{,_into} (matvec_f16w_f32out: f16 x, f32 y) */
LH_API int lh_matvec_f32out_offset(lh_context* ctx, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector,
                                   lh_buffer* output, uint32_t rows, uint32_t cols);
LH_API int lh_matvec_f32out_offset_into(lh_batch* batch, const lh_buffer* matrix, size_t matrix_offset,
                                        const lh_buffer* vector, lh_buffer* output, uint32_t rows, uint32_t cols);
/* kernels.rs:1876-1930 matvec_f32in_offset (matvec_f16w_f32in: f32 x, f16 y); the _into form is this library's */
LH_API int lh_matvec_f32in_offset(lh_context* ctx, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector,
                                  lh_buffer* output, uint32_t rows, uint32_t cols);
LH_API int lh_matvec_f32in_offset_into(lh_batch* batch, const lh_buffer* matrix, size_t matrix_offset,
                                       const lh_buffer* vector, lh_buffer* output, uint32_t rows, uint32_t cols);

/* ---- decoder-layer glue around the hot path (TransformerLayer::forward_decode, layer.rs:354-523) ----
 * All tensors f16 unless stated; argument order follows the Kernels method named on each line. */
/* kernels.rs:2142-2152 rms_norm_into (shaders/rms_norm.metal:4-46): out[r] = in[r] * rsqrt(mean(in[r]^2) + eps) * weight */
LH_API int lh_rms_norm_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight, lh_buffer* output,
                            uint32_t dim, uint32_t rows, float eps);
/* kernels.rs:6663-6673 rms_norm_add_into (rms_norm.metal:48-88): the same plus residual[r] */
LH_API int lh_rms_norm_add_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight, const lh_buffer* residual,
                                lh_buffer* output, uint32_t dim, uint32_t rows, float eps);
/* The tail of the single-token layer step in one dispatch (layer.rs:507-520 issues rms_norm_into, residual_add_into and,
 * when the layer has an output scale, scale_in_place_gpu_into): out = f16(f16(f16(norm(in) * weight) + residual) * scale),
 * i.e. with the f16 rounding after each of the three steps that the separate kernels apply; `scale` is used only when
 * `apply_scale` is non-zero.  `output` may alias `residual`. */
LH_API int lh_rms_norm_residual_scale_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight,
                                           const lh_buffer* residual, lh_buffer* output, uint32_t dim, uint32_t rows,
                                           float eps, int apply_scale, float scale);
/* kernels.rs:2215-2280 qk_norm_gpu_into / qk_norm_offset_into (shaders/qk_norm.metal:6-56): per-head RMSNorm in place;
 * weight_offset in bytes into the weight buffer */
LH_API int lh_qk_norm_gpu_into(lh_batch* batch, lh_buffer* qk_data, const lh_buffer* weight, uint32_t head_dim,
                               uint32_t num_heads, float eps);
LH_API int lh_qk_norm_offset_into(lh_batch* batch, lh_buffer* qk_data, const lh_buffer* weight, size_t weight_offset,
                                  uint32_t head_dim, uint32_t num_heads, float eps);
/* kernels.rs:2282-2392 qk_norm_rope_available / qk_norm_rope_into (qk_norm.metal:70-140): fused norm + NEOX RoPE,
 * bit-identical to qk_norm followed by rope; input may be output.  Honours LOCAL_AI_NO_FUSE_QKROPE=1. */
LH_API int lh_qk_norm_rope_available(uint32_t head_dim);
LH_API int lh_qk_norm_rope_into(lh_batch* batch, const lh_buffer* input, lh_buffer* output, const lh_buffer* weight,
                                uint32_t head_dim, uint32_t num_heads, float eps, uint32_t position, float theta,
                                float partial_rotary_factor);
/* kernels.rs:509-580 rope_into (shaders/rope.metal:14-61): NEOX pairs (i, i + head_dim/2), proportional partial rotary;
 * input may be output */
LH_API int lh_rope_into(lh_batch* batch, const lh_buffer* input, lh_buffer* output, uint32_t head_dim, uint32_t position,
                        float theta, float partial_rotary_factor, uint32_t num_heads);
/* kernels.rs:4228-4300 rope_batch_into (rope.metal:105-150): in place over qk [seq_len, num_heads, head_dim], row r at
 * position start_pos + r; kernels.rs:4311-4385 rope_batch_decode_into (rope.metal:157-200): row r at positions[r] (u32) */
LH_API int lh_rope_batch_into(lh_batch* batch, lh_buffer* qk, uint32_t start_pos, float theta, uint32_t head_dim,
                              uint32_t num_heads, uint32_t seq_len, float partial_rotary_factor);
LH_API int lh_rope_batch_decode_into(lh_batch* batch, lh_buffer* qk, const lh_buffer* positions, float theta,
                                     uint32_t head_dim, uint32_t num_heads, uint32_t seq_len, float partial_rotary_factor);
/* kernels.rs:6648-6660 gelu_mul_into (shaders/gelu.metal:23-41): out = gelu_tanh(a) * b */
LH_API int lh_gelu_mul_into(lh_batch* batch, const lh_buffer* a, const lh_buffer* b, lh_buffer* out, uint32_t count);
/* kernels.rs:2592-2637 residual_add_into (shaders/residual_add.metal:5-15) */
LH_API int lh_residual_add_into(lh_batch* batch, const lh_buffer* a, const lh_buffer* b, lh_buffer* output, uint32_t count);
/* kernels.rs:2845-2890 scale_in_place_gpu_into (shaders/scale_in_place.metal:5-14) */
LH_API int lh_scale_in_place_gpu_into(lh_batch* batch, lh_buffer* data, float scalar, uint32_t count);
/* kernels.rs:2801-2843 gather_strided_f16_into (scale_in_place.metal:21-35): dst[i*pld + p] = src[i*row_stride + base_off + p] */
LH_API int lh_gather_strided_f16_into(lh_batch* batch, const lh_buffer* src, lh_buffer* dst, uint32_t row_stride,
                                      uint32_t base_off, uint32_t pld, uint32_t n_rows);
/* gather_strided_f16_into followed by gelu_mul_into on the gathered rows (the per-layer-input gate of the multi-row
 * layer paths, local-engine/src/layer.rs:690-700) as one dispatch without the gathered copy:
 * out[r*dim + i] = half(gelu(a[r*dim + i]) * b[r*b_row_stride + b_offset + i]); out may be a. */
LH_API int lh_gelu_mul_strided_into(lh_batch* batch, const lh_buffer* a, const lh_buffer* b, uint32_t b_row_stride,
                                    uint32_t b_offset, lh_buffer* out, uint32_t dim, uint32_t rows);
/* kernels.rs:2749-2799 logit_softcap_gpu_into (scale_in_place.metal:39-49): f32 data[i] = cap * tanh(data[i] / cap) */
LH_API int lh_logit_softcap_gpu_into(lh_batch* batch, lh_buffer* data, float cap, uint32_t count);

/* kernels.rs:6155, 6160, 6362 constants and 6277-6304 env-flag getters
 * (LOCAL_AI_BATCHM / LOCAL_AI_MMA / LOCAL_AI_SMALLM, read once per process). */
LH_API uint32_t lh_smallm_max_m(void);
LH_API uint32_t lh_batchm_max_m(void);
LH_API uint32_t lh_multivec_max_m(void);
LH_API int lh_batchm_enabled(void);
LH_API int lh_mma_enabled(void);
LH_API int lh_smallm_enabled(void);

/* ---- block dequant to f16 (bit-exact twin of the CPU path) ----------------
 * local-engine/src/qat_recover.rs:23-97 dequant_{tq2_0,q4_0}_into; used by
 * QuantWeight::dequant_row_into (layer.rs:269-281) for the embedding gather.
 * `byte_offset` selects where in `data` the blocks start (a row of a matrix). */
LH_API int lh_dequant_q4_0_into(lh_batch* batch, const lh_buffer* data, size_t byte_offset, lh_buffer* output,
                                size_t num_elements);
LH_API int lh_dequant_tq2_0_into(lh_batch* batch, const lh_buffer* data, size_t byte_offset, lh_buffer* output,
                                 size_t num_elements);
/* Rows `rows[0 .. n_rows)` (a device u32 list; an index past the end reads the last row, init_gemma4_qat.rs:152)
 * of a packed [table_rows, cols] table decoded to a dense f16 [n_rows, cols] matrix in one dispatch: the embedding
 * gather of local-engine/src/pipeline.rs:781-832 (gather_embeddings, which decodes on the CPU one row at a time)
 * and the per-layer-embedding rows of pipeline.rs:1011-1019.  `fmt` is an lh_quant value or LH_ROWS_F16 for a
 * table of plain f16 rows.  With scale != 1 every value is multiplied by it and rounded to f16 once more, exactly
 * what scale_in_place_gpu_into (pipeline.rs:999-1001) does to the gathered rows. */
#define LH_ROWS_F16 2
LH_API int lh_dequant_rows_into(lh_batch* batch, int fmt, const lh_buffer* table, uint32_t table_rows, uint32_t cols,
                                const lh_buffer* rows, uint32_t n_rows, float scale, lh_buffer* output);
/* kernels.rs:6753-6802 tq2_dequant (legacy 2-bit unpack, shaders/tq2_dequant.metal:4-16). */
LH_API int lh_tq2_dequant(lh_context* ctx, const lh_buffer* packed, const lh_buffer* scales, lh_buffer* output,
                          uint32_t num_elements);

/* ---- TurboQuant codec parameters (host side, no GPU work) --------------------
 * local-engine/src/turboquant.rs:66-79 Rotation::new (splitmix64 signs),
 * 114-166 lloyd_max_gaussian, 187-192 TurboQuant::new (levels / sqrt(dim)),
 * 202-204 code_bytes; local-engine/src/kv_cache/quant_cache.rs:30,37 (seed,
 * default bits), 48-54 swa_ring_capacity, 60-66 kv_bits_from_env.  `levels`
 * receives 1 << bits floats, `signs` receives dim floats. */
#define LH_TQ_SEED 0x7459C0DEull
#define LH_DEFAULT_KV_BITS 2
LH_API int lh_turboquant_levels(uint32_t dim, uint32_t bits, float* levels);
LH_API int lh_turboquant_signs(uint32_t dim, uint64_t seed, float* signs);
LH_API uint32_t lh_turboquant_code_bytes(uint32_t dim, uint32_t bits);
LH_API size_t lh_swa_ring_capacity(size_t window, size_t max_positions);
LH_API uint32_t lh_kv_bits_from_env(void);

/* ---- TurboQuant KV cache ----------------------------------------------------
 * kernels.rs:4819-4890 encode_kv_turboquant_into, 4988-5020 encode_kv_turboquant,
 * shaders/dequantize_kv.metal:216-318.  input [num_tokens, n_kv_heads, head_dim]
 * f16; slot g = ((position + token) % ring_capacity or absolute) * n_kv_heads +
 * head; codes LSB-first, ceil(head_dim*bits/8) bytes per slot; norms f16.
 * Codes and norms equal the CPU encoder's (turboquant.rs:241-276) bit for bit. */
LH_API int lh_encode_kv_turboquant(lh_context* ctx, const lh_buffer* input, const lh_buffer* levels,
                                   const lh_buffer* signs, lh_buffer* packed, lh_buffer* norms, uint32_t head_dim,
                                   uint32_t n_kv_heads, uint32_t num_tokens, uint32_t bits, uint32_t position,
                                   uint32_t ring_capacity);
LH_API int lh_encode_kv_turboquant_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* levels,
                                        const lh_buffer* signs, lh_buffer* packed, lh_buffer* norms,
                                        uint32_t head_dim, uint32_t n_kv_heads, uint32_t num_tokens, uint32_t bits,
                                        uint32_t position, uint32_t ring_capacity);
/* kernels.rs:4901-4979 encode_kv_turboquant_batched_into,
 * shaders/dequantize_kv.metal:327-407: slot (lane*lane_capacity +
 * positions[lane] % ring) * n_kv_heads + head; positions u32[n_lanes]. */
LH_API int lh_encode_kv_turboquant_batched_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* levels,
                                                const lh_buffer* signs, lh_buffer* packed, lh_buffer* norms,
                                                const lh_buffer* positions, uint32_t head_dim, uint32_t n_kv_heads,
                                                uint32_t lane_capacity, uint32_t bits, uint32_t n_lanes,
                                                uint32_t ring_capacity);
/* kernels.rs:4641-4804 dequantize_kv_turboquant{,_into},
 * shaders/dequantize_kv.metal:132-189: codes -> f16 [num_tokens, n_kv, head_dim]
 * for tokens [token_start, num_tokens). */
LH_API int lh_dequantize_kv_turboquant(lh_context* ctx, const lh_buffer* packed, const lh_buffer* norms,
                                       const lh_buffer* levels, const lh_buffer* signs, lh_buffer* output,
                                       uint32_t head_dim, uint32_t n_kv_heads, uint32_t num_tokens, uint32_t bits,
                                       uint32_t token_start, uint32_t ring_capacity);
LH_API int lh_dequantize_kv_turboquant_into(lh_batch* batch, const lh_buffer* packed, const lh_buffer* norms,
                                            const lh_buffer* levels, const lh_buffer* signs, lh_buffer* output,
                                            uint32_t head_dim, uint32_t n_kv_heads, uint32_t num_tokens,
                                            uint32_t bits, uint32_t token_start, uint32_t ring_capacity);
/* Single-token Q / K / V preparation in one dispatch (no single counterpart in the reference: it replaces the eight
 * dispatches of layer.rs:393-450 + quant_cache.rs:391-444, 560-570 -- qk_norm_gpu_into and rope_into on Q and on K,
 * rms_norm_into with unit weight on V, encode_kv_turboquant_into for K and for V, hadamard_rotate_hf_into on Q):
 *   q [n_q_heads, head_dim] f16, in place: per-head RMS norm (when `q_norm` is given), NEOX RoPE at `position`;
 *      rq [n_q_heads, head_dim] f32 = FWHT(signs * q) / sqrt(head_dim), the query of flash_attention_tq_into;
 *   k, v [n_kv_heads, head_dim] f16, in place: K as Q with `k_norm`, V RMS-normalised with unit weight; both encoded
 *      into the cache row of `position` (ring addressing as in encode_kv_turboquant_into).
 * Pass k = v = NULL for a layer that shares another layer's cache (only Q is prepared).  Values are rounded to f16
 * wherever the separate kernels store f16; codes and norms equal the CPU encoder's for the k / v rows left behind. */
LH_API int lh_decode_qkv_prepare_into(lh_batch* batch, lh_buffer* q, lh_buffer* k, lh_buffer* v, const lh_buffer* q_norm,
                                      const lh_buffer* k_norm, const lh_buffer* levels, const lh_buffer* signs, lh_buffer* rq,
                                      lh_buffer* k_codes, lh_buffer* k_norms, lh_buffer* v_codes, lh_buffer* v_norms,
                                      uint32_t head_dim, uint32_t n_q_heads, uint32_t n_kv_heads, float eps, uint32_t position,
                                      float theta, float partial_rotary_factor, uint32_t bits, uint32_t ring_capacity);
/* The same for `rows` tokens at once (the eight dispatches of layer.rs:568-616 / 763-800 + quant_cache.rs:620-660 /
 * quant_unified_pool.rs:138-230): q [rows, n_q_heads, head_dim], k / v [rows, n_kv_heads, head_dim], rq [rows, n_q_heads,
 * head_dim] f32.  With `positions` == NULL (and lane_capacity 0) row r is the token at start_position + r of one
 * sequence (rope_batch_into / encode_kv_turboquant_into addressing); with a device table `positions[rows]` row r is one
 * token of lane r at positions[r], written into the lane's region of `lane_capacity` rows (rope_batch_decode_into /
 * encode_kv_turboquant_batched_into addressing). */
LH_API int lh_decode_qkv_prepare_rows_into(lh_batch* batch, lh_buffer* q, lh_buffer* k, lh_buffer* v, const lh_buffer* q_norm,
                                           const lh_buffer* k_norm, const lh_buffer* levels, const lh_buffer* signs,
                                           lh_buffer* rq, lh_buffer* k_codes, lh_buffer* k_norms, lh_buffer* v_codes,
                                           lh_buffer* v_norms, const lh_buffer* positions, uint32_t head_dim,
                                           uint32_t n_q_heads, uint32_t n_kv_heads, uint32_t rows, float eps,
                                           uint32_t start_position, float theta, float partial_rotary_factor, uint32_t bits,
                                           uint32_t ring_capacity, uint32_t lane_capacity);
/* The Q, K and V projections of `rows` tokens followed by lh_decode_qkv_prepare_rows_into on their outputs, i.e.
 * lh_matmul_nt_quant_grouped_into(fmt, 3, input, {w_q, w_k, w_v}, {q, k, v}, rows, k_dim) and then the preparation
 * (layer.rs:570-616 / 749-800), with the same results bit for bit: q / k / v, rq, codes and norms.  Where the product
 * runs on the decode-batch kernel with its k range split (a few to some hundreds of rows), the preparation sums the
 * product's partial tiles itself and the product's own reduction pass falls away; every other shape runs as the two
 * calls.  input [rows, k_dim] f16; w_q [n_q_heads * head_dim, k_dim], w_k / w_v [n_kv_heads * head_dim, k_dim] in `fmt`.
 * All three projections are required (a layer that shares another layer's cache takes the separate entry points). */
LH_API int lh_matmul_nt_qkv_prepare_rows_into(lh_batch* batch, lh_quant fmt, const lh_buffer* input, const lh_buffer* w_q,
                                              const lh_buffer* w_k, const lh_buffer* w_v, uint32_t k_dim, lh_buffer* q,
                                              lh_buffer* k, lh_buffer* v, const lh_buffer* q_norm, const lh_buffer* k_norm,
                                              const lh_buffer* levels, const lh_buffer* signs, lh_buffer* rq,
                                              lh_buffer* k_codes, lh_buffer* k_norms, lh_buffer* v_codes, lh_buffer* v_norms,
                                              const lh_buffer* positions, uint32_t head_dim, uint32_t n_q_heads,
                                              uint32_t n_kv_heads, uint32_t rows, float eps, uint32_t start_position,
                                              float theta, float partial_rotary_factor, uint32_t bits, uint32_t ring_capacity,
                                              uint32_t lane_capacity);
/* kernels.rs:5032-5163 hadamard_rotate{,_hf,_fh}_into,
 * shaders/attention_flash_tq.metal:58-139: per head optional sign flip, FWHT,
 * 1/sqrt(d), optional sign flip.  f32->f32, f16->f32, f32->f16. */
LH_API int lh_hadamard_rotate_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs,
                                   lh_buffer* output, uint32_t head_dim, uint32_t num_heads, int pre_sign,
                                   int post_sign);
LH_API int lh_hadamard_rotate_hf_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs,
                                      lh_buffer* output, uint32_t head_dim, uint32_t num_heads, int pre_sign,
                                      int post_sign);
LH_API int lh_hadamard_rotate_fh_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs,
                                      lh_buffer* output, uint32_t head_dim, uint32_t num_heads, int pre_sign,
                                      int post_sign);
/* kernels.rs:5176-5243 flash_attention_tq_into,
 * shaders/attention_flash_tq.metal:154-274: single-query decode attention
 * straight from packed codes (no 1/sqrt(d) scale), rq / out [num_q_heads,
 * head_dim] f32 in rotated space.
 * Numerics of the tq entries for 2-bit codes at head_dim 256 / 512 with up to
 * 8 query heads per KV head (the matrix-core kernel; other shapes multiply
 * decoded floats): the rotated query enters as 16-bit fixed point relative to
 * each head's largest element, the softmax weight x value norm as 16-bit fixed
 * point relative to the head's largest one among the 64 or 128 positions it is
 * handed over with (round to nearest); sums are exact integers, softmax sums
 * and the final scaling f32.  Measured against the f64 oracle: 1e-4 .. 3e-4 of
 * max|out|; the bound for one weight among 127 of just under half a step of it
 * is 2e-3 of that group's share.  A head whose softmax sum is not a positive
 * number (an empty range, a NaN logit) gives zeros, as the reference's
 * `gsum > 0 ? 1 / gsum : 0` does (attention_flash_tq.metal:263). */
LH_API int lh_flash_attention_tq_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                      const lh_buffer* k_norms, const lh_buffer* v_codes, const lh_buffer* v_norms,
                                      const lh_buffer* levels, lh_buffer* out, uint32_t head_dim, uint32_t kv_len,
                                      uint32_t current_pos, uint32_t num_q_heads, uint32_t num_kv_heads,
                                      uint32_t window, uint32_t bits, uint32_t ring_capacity);
/* No counterpart in the reference.  For callers that cannot allocate device
 * memory (code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): lh_flash_attention_tq_into with the split-K partial
 * records kept in a static device array of 8 MiB instead of the context
 * workspace; the call itself allocates nothing.  Same arguments and results.
 * Limit: num_q_heads * (head_dim + 4) <= 8192 (256 split records of every
 * query head must fit), otherwise LH_ERR_INVALID_ARGUMENT.  All calls on one
 * GPU share that GPU's array: calls that overlap on one GPU (two contexts,
 * two streams) race; calls on one context are ordered by its stream. */
LH_API int lh_flash_attention_tq_static_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                             const lh_buffer* k_norms, const lh_buffer* v_codes,
                                             const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                                             uint32_t head_dim, uint32_t kv_len, uint32_t current_pos,
                                             uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t window,
                                             uint32_t bits, uint32_t ring_capacity);
/* kernels.rs:5259-5420 flash_attention_tq_prefill{,_tiled}_into,
 * shaders/attention_flash_tq.metal:290-556: n_rows causal query rows at
 * positions start_pos..start_pos+n_rows-1; rq / out [n_rows, num_q_heads, head_dim]. */
LH_API int lh_flash_attention_tq_prefill_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                              const lh_buffer* k_norms, const lh_buffer* v_codes,
                                              const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                                              uint32_t head_dim, uint32_t kv_len, uint32_t start_pos,
                                              uint32_t n_rows, uint32_t num_q_heads, uint32_t num_kv_heads,
                                              uint32_t window, uint32_t bits, uint32_t ring_capacity);
LH_API int lh_flash_attention_tq_prefill_tiled_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                                    const lh_buffer* k_norms, const lh_buffer* v_codes,
                                                    const lh_buffer* v_norms, const lh_buffer* levels,
                                                    lh_buffer* out, uint32_t head_dim, uint32_t kv_len,
                                                    uint32_t start_pos, uint32_t n_rows, uint32_t num_q_heads,
                                                    uint32_t num_kv_heads, uint32_t window, uint32_t bits,
                                                    uint32_t ring_capacity);
/* kernels.rs:5434-5506 flash_attention_tq_batched_into,
 * shaders/attention_flash_tq.metal:569-690: one query per lane over the by-lane
 * pool; rq / out [n_lanes, num_q_heads, head_dim]; positions u32[n_lanes]. */
LH_API int lh_flash_attention_tq_batched_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                              const lh_buffer* k_norms, const lh_buffer* v_codes,
                                              const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                                              const lh_buffer* positions, uint32_t head_dim,
                                              uint32_t lane_capacity, uint32_t num_q_heads, uint32_t num_kv_heads,
                                              uint32_t window, uint32_t bits, uint32_t n_lanes,
                                              uint32_t ring_capacity);
/* quant_cache.rs:571-598 (the attend and rotate-back steps of fused_attention_into)
 * and quant_unified_pool.rs:225-256 (attention_into) as one call each:
 * lh_flash_attention_tq_into / lh_flash_attention_tq_batched_into into `out`
 * (f32 scratch of the same shape, left undefined), then
 * lh_hadamard_rotate_fh_into(out, signs, out_f16, post-sign only).  With 2..32
 * splits the merge and the rotation run as one kernel; the f16 result equals
 * the two calls' bit for bit either way. */
LH_API int lh_flash_attention_tq_rotated_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                              const lh_buffer* k_norms, const lh_buffer* v_codes,
                                              const lh_buffer* v_norms, const lh_buffer* levels,
                                              const lh_buffer* signs, lh_buffer* out, lh_buffer* out_f16,
                                              uint32_t head_dim, uint32_t kv_len, uint32_t current_pos,
                                              uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t window,
                                              uint32_t bits, uint32_t ring_capacity);
/* lh_flash_attention_tq_rotated_into for a caller whose next kernel can do the rotation itself
 * (lh_matvec_quant_rotated_into): where the rotation rides in the merge launch (2..32 partial
 * records) it is done here, `out_f16` holds the rotated heads and *rotated is set to 1; otherwise
 * no rotation kernel is launched, the f32 heads stay in `out`, still in code space, and *rotated
 * is set to 0.  The choice depends on the shape arguments only, so it is the same at every call
 * with the same shape (a recorded batch replays the choice made while it was recorded). */
LH_API int lh_flash_attention_tq_rotated_lazy_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                                   const lh_buffer* k_norms, const lh_buffer* v_codes,
                                                   const lh_buffer* v_norms, const lh_buffer* levels,
                                                   const lh_buffer* signs, lh_buffer* out, lh_buffer* out_f16,
                                                   uint32_t head_dim, uint32_t kv_len, uint32_t current_pos,
                                                   uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t window,
                                                   uint32_t bits, uint32_t ring_capacity, int* rotated);
LH_API int lh_flash_attention_tq_batched_rotated_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes,
                                                      const lh_buffer* k_norms, const lh_buffer* v_codes,
                                                      const lh_buffer* v_norms, const lh_buffer* levels,
                                                      const lh_buffer* signs, lh_buffer* out, lh_buffer* out_f16,
                                                      const lh_buffer* positions, uint32_t head_dim,
                                                      uint32_t lane_capacity, uint32_t num_q_heads,
                                                      uint32_t num_kv_heads, uint32_t window, uint32_t bits,
                                                      uint32_t n_lanes, uint32_t ring_capacity);

/* ---- FP16-KV split-K decode attention ---------------------------------------
 * kernels.rs:1397-1557 flash_decoding_into, 1292-1392
 * flash_attention_windowed_split_into, 1265-1278 flash_split_count;
 * shaders/flash_decoding.metal:10-189.  q [H, hd], k/v [T, n_kv, hd], out [H, hd], all f16. */
LH_API int lh_flash_decoding_into(lh_batch* batch, const lh_buffer* q, const lh_buffer* k, const lh_buffer* v,
                                  lh_buffer* output, uint32_t head_dim, uint32_t kv_len, uint32_t current_pos,
                                  uint32_t num_q_heads, uint32_t num_kv_heads);
LH_API int lh_flash_attention_windowed_split_into(lh_batch* batch, const lh_buffer* q, const lh_buffer* k,
                                                  const lh_buffer* v, lh_buffer* output, lh_buffer* partial_max,
                                                  lh_buffer* partial_sum, lh_buffer* partial_acc, uint32_t head_dim,
                                                  uint32_t kv_len, uint32_t current_pos, uint32_t num_q_heads,
                                                  uint32_t num_kv_heads, uint32_t window, uint32_t num_splits);
LH_API uint32_t lh_flash_split_count(uint32_t eff_seq_len);

#ifdef __cplusplus
}
#endif
#endif /* LOCAL_HIP_H */
