// Shared between the two implementations of attention over packed TurboQuant codes
// (attention_tq.hip: any bits / head_dim on the vector ALU; attention_tq_mfma.hip: 2-bit codes,
// head_dim 256 or 512 on the matrix cores).
#pragma once
#include "common.hpp"

namespace lh_attn {

enum Mode : uint32_t { kSingle = 0, kPrefill = 1, kBatched = 2 };

struct AttnParams {
    uint32_t head_dim, bits, code_bytes;
    uint32_t num_q_heads, num_kv_heads;
    uint32_t kv_len;          // single / prefill
    uint32_t pos0;            // single: current_pos; prefill: start_pos
    uint32_t window, ring_capacity, lane_capacity;
    uint32_t mode, num_queries, num_splits;
    uint32_t pair_spin_limit = 1u << 22;   // polls a wave of the several-chunk kernels spends at one hand-over before it gives up
};

constexpr int kMaxSplits = 1024;

// Logical position range [lo, hi) of query `qi` and the first slot of its lane in a by-lane pool
// (shaders/attention_flash_tq.metal:175-190, 590-600).
__device__ __forceinline__ void query_range(const AttnParams& p, const uint32_t* positions, uint32_t qi, uint32_t& lo, uint32_t& hi,
                                            uint32_t& lane_base) {
    uint32_t pos, kv_len;
    if (p.mode == kBatched) { pos = positions[qi]; kv_len = pos + 1u; lane_base = qi * p.lane_capacity; }
    else { pos = p.pos0 + (p.mode == kPrefill ? qi : 0u); kv_len = p.kv_len; lane_base = 0; }
    hi = kv_len < pos + 1u ? kv_len : pos + 1u;
    lo = (p.window > 0u && pos + 1u > p.window) ? pos + 1u - p.window : 0u;
    if (lo > hi) lo = hi;
}

// Per (query, head, split) record in the workspace: [m (natural log), l, pad, pad, acc[head_dim]].
__host__ __device__ __forceinline__ size_t partial_record_floats(uint32_t head_dim) { return (size_t)head_dim + 4; }

struct AttnPointers {
    const float* rq;
    const uint8_t* k_codes;
    const uint16_t* k_norms;
    const uint8_t* v_codes;
    const uint16_t* v_norms;
    const float* levels;
    const uint32_t* positions;
    float* out;
    float* ws;
    uint32_t* fault = nullptr;   // where a kernel reports a bounded wait that ran out (the context's fault word)
};

// True when the matrix-core kernel can take this call (2-bit codes, head_dim 256 or 512, at most 8 query heads per
// KV head, ring absent or a multiple of 64 slots, 4-byte aligned code buffers).
bool mfma_supported(const AttnParams& p, const AttnPointers& a);
// Chooses p.num_splits (wave chunks per query and KV head) and launches the split kernel; the caller
// runs the merge kernel when p.num_splits > 1.
int launch_mfma(lh_context* ctx, const char* op, const AttnPointers& a, AttnParams& p, uint64_t max_span, size_t ws_floats);

// The tiled prefill kernel (attention_tq_prefill_tile.hip): sixteen query rows per workgroup share one pass over the codes,
// K and V levels as f16 through LDS, any level table.  Takes 2-bit codes, head_dim 256, at most 8 query heads per KV head,
// ring absent or a multiple of 64 slots, two rows or more.
bool prefill_tile_supported(const AttnParams& p, const AttnPointers& a);
int launch_prefill_tile(lh_context* ctx, const char* op, const AttnPointers& a, AttnParams& p, uint64_t max_span, size_t ws_floats);

}  // namespace lh_attn
