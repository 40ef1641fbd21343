// TurboQuant KV cache: codec parameters (host), GPU encode, GPU dequantize and the
// randomized-Hadamard rotations around the fused attention kernel.
//
// Stands in for shaders/dequantize_kv.metal:132-407 (dequantize_kv_turboquant,
// encode_kv_turboquant{,_batched}), shaders/attention_flash_tq.metal:58-139
// (hadamard_rotate{,_hf,_fh}) and their dispatch in local-metal/src/kernels.rs:
// 4641-5163, plus the host-side codec set-up of local-engine/src/turboquant.rs.
//
// Bit-exactness contract: codes and f16 norms written by the encode kernels equal
// the CPU encoder's (turboquant.rs:241-276) for the same levels / signs.  That fixes
//   - the squared norm as a left-to-right f32 sum of separately rounded squares,
//   - IEEE sqrt and 1/norm, two separate multiplies (1/norm, then sign),
//   - butterflies (a+b, a-b) per stage -- the pairing is fixed, so running a stage in
//     parallel gives the same bits as the sequential loop,
//   - 1/sqrt(d) computed on the host exactly as the CPU does and passed in,
//   - nearest level with strict '<' from index 0 (lowest index wins ties).
// This file is compiled with -ffp-contract=off: no product may be fused into a sum.
#include "common.hpp"
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <algorithm>

namespace {

constexpr int kMaxHeadDim = 512;

__device__ __forceinline__ uint32_t unpack_code(const uint8_t* codes, uint32_t d, uint32_t bits) {
    // LSB-first bit stream; a 3-bit code may straddle two bytes (attention_flash_tq.metal:33-47)
    const uint32_t bit_off = d * bits, byte = bit_off >> 3, shift = bit_off & 7u;
    uint32_t v = codes[byte];
    if (shift + bits > 8u) v |= (uint32_t)codes[byte + 1] << 8;
    return (v >> shift) & ((1u << bits) - 1u);
}

__device__ __forceinline__ void fwht_lds(float* sh, uint32_t d, uint32_t lane) { lh_fwht_lds(sh, d, lane); }

struct EncodeParams {
    uint32_t head_dim, n_kv_heads, bits, code_bytes;
    uint32_t position;        // first logical token (single-sequence form)
    uint32_t ring_capacity;   // 0 = absolute
    uint32_t lane_capacity;   // batched form: physical tokens per lane region
    float inv_sqrt_d;
};

// The 2^bits <= 16 codec levels as values, requested at the top of a kernel (uniform addresses: scalar loads), so that the
// level search at the end of an encode does not start a trip to memory of its own; entries past 2^bits are +inf and never win.
struct LevelTable { float v[16]; };
__device__ __forceinline__ LevelTable load_levels(const float* __restrict__ levels, uint32_t bits) {
    LevelTable t;
    const uint32_t k = 1u << bits;
#pragma unroll
    for (int i = 0; i < 16; i++) t.v[i] = (uint32_t)i < k ? levels[i] : INFINITY;
    return t;
}

// TurboQuant encode of one vector held one coordinate per thread (turboquant.rs:241-276): norm, unit vector, signs,
// FWHT, 1/sqrt(d), nearest level, bit packing.  `sh` and `code_sh` are workgroup arrays of at least d entries; the
// calling kernel runs d threads.  `sign` is the lane's entry of the sign vector and `lv` the level table, both loaded by
// the caller ahead of its own work: behind the barriers here each would cost a round trip to memory.
__device__ __forceinline__ void encode_vector(float xv, uint32_t lane, uint32_t d, float* sh, uint32_t* code_sh,
                                              const float sign, const LevelTable& lv, uint32_t bits,
                                              uint32_t code_bytes, float inv_sqrt_d, uint8_t* __restrict__ packed_slot,
                                              uint16_t* __restrict__ norm_slot) {
    // norm = sqrt(fold(+, x_i * x_i)) in index order: the first wave walks the LDS words (broadcast reads, so each of its
    // lanes holds the sum) and hands the sum over; the d dependent additions are issued once per vector, not once per wave
    // (they are most of what a bulk encode issues).
    sh[lane] = __fmul_rn(xv, xv);
    __syncthreads();
    float sq = 0.0f;
    if (lane < 64) {
        if (d >= 4) {
            for (uint32_t i = 0; i < d; i += 4) {
                const float4 q = *reinterpret_cast<const float4*>(&sh[i]);
                sq = __fadd_rn(sq, q.x); sq = __fadd_rn(sq, q.y); sq = __fadd_rn(sq, q.z); sq = __fadd_rn(sq, q.w);
            }
        } else {
            for (uint32_t i = 0; i < d; i++) sq = __fadd_rn(sq, sh[i]);
        }
    }
    if (d > 64) {   // uniform over the workgroup
        if (lane == 0) reinterpret_cast<float*>(code_sh)[0] = sq;
        __syncthreads();
        sq = reinterpret_cast<const float*>(code_sh)[0];
    }
    const float norm = __fsqrt_rn(sq);
    float v = xv;
    if (norm > 0.0f) v = __fmul_rn(v, __fdiv_rn(1.0f, norm));
    v = __fmul_rn(v, sign);
    __syncthreads();
    sh[lane] = v;
    fwht_lds(sh, d, lane);
    const float y = __fmul_rn(sh[lane], inv_sqrt_d);

    uint32_t best = 0;
    float bd = INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const float dd = fabsf(__fsub_rn(y, lv.v[i]));
        if (dd < bd) { bd = dd; best = i; }
    }
    code_sh[lane] = best;
    if (lane == 0) *norm_slot = lh_f2h_exact(norm);
    __syncthreads();
    if (lane < code_bytes) {     // one thread per output byte
        uint32_t byte_val = 0;
        for (uint32_t bitpos = 0; bitpos < 8; ++bitpos) {
            const uint32_t global_bit = lane * 8 + bitpos, code_idx = global_bit / bits;
            if (code_idx >= d) break;
            byte_val |= ((code_sh[code_idx] >> (global_bit - code_idx * bits)) & 1u) << bitpos;
        }
        packed_slot[lane] = (uint8_t)byte_val;
    }
}

// One workgroup (head_dim threads) per (token, head) vector.  BATCHED: group = (lane, head),
// slot from positions[lane] (dequantize_kv.metal:327-407); else group = (token, head)
// (dequantize_kv.metal:216-318).
template <bool BATCHED>
__global__ __launch_bounds__(kMaxHeadDim) void encode_kv_kernel(const uint16_t* __restrict__ input, const float* __restrict__ levels,
                                                               const float* __restrict__ signs, uint8_t* __restrict__ packed,
                                                               uint16_t* __restrict__ norms, const uint32_t* __restrict__ positions,
                                                               EncodeParams p) {
    __shared__ __align__(16) float sh[kMaxHeadDim];
    __shared__ uint32_t code_sh[kMaxHeadDim];
    const uint32_t d = p.head_dim, lane = threadIdx.x, group = blockIdx.x;
    const float xv = lh_h2f(input[(size_t)group * d + lane]), sign = signs[lane];
    const LevelTable lv = load_levels(levels, p.bits);
    const uint32_t tok = group / p.n_kv_heads, head = group - tok * p.n_kv_heads;
    uint32_t g;
    if (BATCHED) {
        const uint32_t pos = positions[tok];
        const uint32_t ppos = p.ring_capacity ? pos % p.ring_capacity : pos;
        g = (tok * p.lane_capacity + ppos) * p.n_kv_heads + head;
    } else {
        const uint32_t logical = p.position + tok;
        g = (p.ring_capacity ? logical % p.ring_capacity : logical) * p.n_kv_heads + head;
    }
    encode_vector(xv, lane, d, sh, code_sh, sign, lv, p.bits, p.code_bytes, p.inv_sqrt_d, packed + (size_t)g * p.code_bytes, norms + g);
}

// ---- single-token Q / K / V preparation in one dispatch ---------------------------------------------------------
// What layer.rs:393-450 issues as qk_norm (Q), rope (Q), qk_norm (K), rms_norm with unit weight (V), rope (K), two KV
// encodes and the query rotation of quant_cache.rs:560-570 -- eight dispatches of a few hundred bytes each -- as one
// kernel: workgroup b < n_q prepares query head b (norm, RoPE, f16 store, signs + FWHT -> f32 rq), the next n_kv
// workgroups one K head each (norm, RoPE, f16 store, encode into the cache slot), the last n_kv one V head each
// (unit-weight RMS norm, f16 store, encode).  Every value is rounded to f16 where the separate kernels store f16, and
// the encode is the same code as encode_kv_kernel, so the codes are exactly those of the CPU encoder for the f16 rows
// this kernel leaves in k / v.
// Several rows at once: row r is the token at position `position + r` of one sequence (lane_capacity == 0; a prefill
// chunk or a verify batch), or one token of lane r at positions[r], whose cache region starts lane_capacity rows
// after the previous lane's (continuous batching; the addressing of encode_kv_turboquant_batched).
struct PrepareParams {
    uint32_t head_dim, n_q_heads, n_kv_heads, bits, code_bytes, position, ring_capacity, write_kv, lane_capacity;
    float eps, theta, prf, inv_sqrt_d;
    // The heads as the f32 partial tiles of a k-split product [splits][rows][part_cols] (columns: the query heads, the key
    // heads, the value heads, side by side) instead of f16 rows in q / k / v; nullptr: the rows are read from q / k / v.
    const float* partial;
    uint32_t splits, part_cols, rows;
};

__global__ __launch_bounds__(kMaxHeadDim) void decode_qkv_prepare_kernel(uint16_t* __restrict__ q, uint16_t* __restrict__ k,
                                                                        uint16_t* __restrict__ v, const uint16_t* __restrict__ q_norm_w,
                                                                        const uint16_t* __restrict__ k_norm_w, const float* __restrict__ signs,
                                                                        const float* __restrict__ levels, float* __restrict__ rq,
                                                                        uint8_t* __restrict__ k_codes, uint16_t* __restrict__ k_norms,
                                                                        uint8_t* __restrict__ v_codes, uint16_t* __restrict__ v_norms,
                                                                        const uint32_t* __restrict__ positions, PrepareParams p) {
    __shared__ __align__(16) float sh[kMaxHeadDim];
    __shared__ uint32_t code_sh[kMaxHeadDim];
    __shared__ uint16_t hbuf[kMaxHeadDim];
    __shared__ float wsum[kMaxHeadDim / 64];
    const uint32_t d = p.head_dim, lane = threadIdx.x;
    const uint32_t per_row = p.n_q_heads + 2 * p.n_kv_heads;            // n_kv_heads is 0 when the cache is not written
    const uint32_t row = blockIdx.x / per_row, b = blockIdx.x - row * per_row;
    const uint32_t position = positions ? positions[row] : p.position + row;
    const bool is_q = b < p.n_q_heads, is_k = !is_q && b < p.n_q_heads + p.n_kv_heads;
    const uint32_t head = is_q ? b : (is_k ? b - p.n_q_heads : b - p.n_q_heads - p.n_kv_heads);
    uint16_t* vec = (is_q ? q : (is_k ? k : v)) + ((size_t)row * (is_q ? p.n_q_heads : p.n_kv_heads) + head) * d;
    const uint16_t* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
    const bool normalise = !(is_q || is_k) || norm_w != nullptr;          // V always (unit weight); Q / K when the layer has the weight

    // Everything the workgroup reads from memory is requested here, in one trip: behind the barriers below each load
    // would be a round trip of its own (the norm weight, the sign, the levels: three of them on the K and V path).
    uint16_t raw;
    if (p.partial) {
        // The sum the product's own reduction pass would have stored: the splits in order, in f32, rounded to f16.  Eight
        // splits are requested before the first is added.
        const size_t zstride = (size_t)p.rows * p.part_cols;
        const float* part = p.partial + (size_t)row * p.part_cols + (size_t)b * d + lane;
        float acc = 0.0f;
        for (uint32_t z0 = 0; z0 < p.splits; z0 += 8) {
            float t[8];
#pragma unroll
            for (uint32_t u = 0; u < 8; u++) t[u] = part[(size_t)(z0 + u < p.splits ? z0 + u : p.splits - 1) * zstride];
#pragma unroll
            for (uint32_t u = 0; u < 8; u++) if (z0 + u < p.splits) acc += t[u];
        }
        raw = lh_f2h(acc);
    } else {
        raw = vec[lane];
    }
    const float norm_weight = norm_w ? lh_h2f(norm_w[lane]) : 1.0f;
    const float sign = signs[lane];
    LevelTable lv;
    if (!is_q && p.write_kv) lv = load_levels(levels, p.bits);
    // The RoPE pair's cosine and sine depend on the lane and the position only: evaluated here, under the loads above.
    const uint32_t half_dim = d / 2, rope_angles = (uint32_t)((float)d * p.prf) / 2;
    float rope_c = 1.0f, rope_s = 0.0f;
    if ((is_q || is_k) && lane < rope_angles) lh_rope_cos_sin(lane, d, position, p.theta, rope_c, rope_s);
    uint16_t h = raw;
    if (normalise) {
        const float x = lh_h2f(raw);
        const float part = lh_group_sum(x * x, 64);
        if ((lane & 63) == 0) wsum[lane >> 6] = part;
        __syncthreads();
        float ss = 0.0f;
        for (uint32_t w = 0; w < d / 64; w++) ss += wsum[w];
        const float rms = rsqrtf(ss / (float)d + p.eps);
        h = lh_f2h_exact(lh_norm_product(x, rms, norm_weight));
    }
    if (is_q || is_k) {                                                    // NEOX RoPE on the f16-rounded head (rope.metal:14-61)
        hbuf[lane] = h;
        __syncthreads();
        if (lane < rope_angles) {
            uint16_t o0, o1;
            lh_rope_apply(lh_h2f(hbuf[lane]), lh_h2f(hbuf[lane + half_dim]), rope_c, rope_s, o0, o1);
            hbuf[lane] = o0;
            hbuf[lane + half_dim] = o1;
        }
        __syncthreads();
        h = hbuf[lane];
    }
    vec[lane] = h;
    const float xv = lh_h2f(h);
    if (is_q) {                                                            // hadamard_rotate_hf with pre-sign (attention_flash_tq.metal:58-90)
        sh[lane] = __fmul_rn(xv, sign);
        fwht_lds(sh, d, lane);
        rq[((size_t)row * p.n_q_heads + head) * d + lane] = __fmul_rn(sh[lane], p.inv_sqrt_d);
        return;
    }
    if (!p.write_kv) return;
    const uint32_t slot = p.ring_capacity ? position % p.ring_capacity : position;
    const uint32_t g = (row * p.lane_capacity + slot) * p.n_kv_heads + head;   // lane_capacity == 0: one sequence, slot alone
    encode_vector(xv, lane, d, sh, code_sh, sign, lv, p.bits, p.code_bytes, p.inv_sqrt_d,
                  (is_k ? k_codes : v_codes) + (size_t)g * p.code_bytes, (is_k ? k_norms : v_norms) + g);
}

struct DequantParams {
    uint32_t head_dim, n_kv_heads, bits, code_bytes, group_offset, ring_capacity;
    float inv_sqrt_d;
};

// dequantize_kv.metal:132-189: x^ = sign * (1/sqrt d) * H(levels[code]) * norm -> f16 at the logical slot.
__global__ __launch_bounds__(kMaxHeadDim) void dequantize_kv_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ norms,
                                                                   const float* __restrict__ levels, const float* __restrict__ signs,
                                                                   uint16_t* __restrict__ output, DequantParams p) {
    __shared__ __align__(16) float sh[kMaxHeadDim];
    const uint32_t d = p.head_dim, lane = threadIdx.x;
    const uint32_t g = blockIdx.x + p.group_offset;
    uint32_t src_g = g;
    if (p.ring_capacity) {
        const uint32_t token = g / p.n_kv_heads, head = g - token * p.n_kv_heads;
        src_g = (token % p.ring_capacity) * p.n_kv_heads + head;
    }
    const float sign = signs[lane], norm = lh_h2f(norms[src_g]);   // requested with the codes, not behind the transform's barriers
    sh[lane] = levels[unpack_code(packed + (size_t)src_g * p.code_bytes, lane, p.bits)];
    fwht_lds(sh, d, lane);
    float val = __fmul_rn(sh[lane], p.inv_sqrt_d);
    val = __fmul_rn(val, sign);
    val = __fmul_rn(val, norm);
    output[(size_t)g * d + lane] = lh_f2h_exact(val);
}

// attention_flash_tq.metal:58-90: optional pre-sign, FWHT, 1/sqrt(d), optional post-sign.
template <typename TIn, typename TOut>
__global__ __launch_bounds__(kMaxHeadDim) void hadamard_rotate_kernel(const TIn* __restrict__ input, const float* __restrict__ signs,
                                                                     TOut* __restrict__ output, uint32_t head_dim, float inv_sqrt_d,
                                                                     int pre_sign, int post_sign) {
    __shared__ __align__(16) float sh[kMaxHeadDim];
    const uint32_t d = head_dim, lane = threadIdx.x, head = blockIdx.x;
    const float x = lh_load_as_f32<TIn>(input, (size_t)head * d + lane);
    const float sign = (pre_sign || post_sign) ? signs[lane] : 1.0f;
    sh[lane] = pre_sign ? __fmul_rn(x, sign) : x;
    fwht_lds(sh, d, lane);
    float y = __fmul_rn(sh[lane], inv_sqrt_d);
    if (post_sign) y = __fmul_rn(y, sign);
    if constexpr (sizeof(TOut) == 2) output[(size_t)head * d + lane] = lh_f2h_exact(y);
    else output[(size_t)head * d + lane] = y;
}

int check_tq_shape(const char* op, uint32_t head_dim, uint32_t bits) {
    // quant_cache.rs:191-200 and the debug_assert at kernels.rs:4667
    if (bits < 2 || bits > 4) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: TurboQuant bits must be 2..=4, got %u", op, bits);
    if (head_dim == 0 || (head_dim & (head_dim - 1)) != 0 || head_dim > kMaxHeadDim)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: TurboQuant head_dim must be a power of two <= 512, got %u", op, head_dim);
    return LH_OK;
}

inline float host_inv_sqrt(uint32_t d) { return 1.0f / std::sqrt((float)d); }   // turboquant.rs:47

}  // namespace

// The rotate-back step of the attention entries that take f32 head outputs to f16 (no pre-sign, post-sign): the same
// launch as lh_hadamard_rotate_fh_into, for callers inside the library that have already checked their buffers.
int lh_launch_hadamard_fh(lh_context* ctx, const float* input, const float* signs, uint16_t* output, uint32_t head_dim, uint32_t num_heads) {
    hipLaunchKernelGGL((hadamard_rotate_kernel<float, uint16_t>), dim3(num_heads), dim3(head_dim), 0, ctx->stream, input, signs, output,
                       head_dim, host_inv_sqrt(head_dim), 0, 1);
    return lh_check_launch("hadamard_rotate_fh");
}

namespace {

template <typename TIn, typename TOut>
int hadamard_launch(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs, lh_buffer* output, uint32_t head_dim,
                    uint32_t num_heads, int pre_sign, int post_sign, const char* op) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    int r = check_tq_shape(op, head_dim, 2);
    if (r != LH_OK) return r;
    if (num_heads == 0) return LH_OK;
    LH_NEED(input, (size_t)num_heads * head_dim * sizeof(TIn), op, "input");
    LH_NEED(signs, (size_t)head_dim * 4, op, "signs");
    LH_NEED(output, (size_t)num_heads * head_dim * sizeof(TOut), op, "output");
    hipLaunchKernelGGL((hadamard_rotate_kernel<TIn, TOut>), dim3(num_heads), dim3(head_dim), 0, batch->ctx->stream,
                       (const TIn*)input->ptr, (const float*)signs->ptr, (TOut*)output->ptr, head_dim, host_inv_sqrt(head_dim),
                       pre_sign, post_sign);
    r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

// ---- host codec ----------------------------------------------------------------
// turboquant.rs:114-166, same operation order in f32 (mul_add -> fmaf).
void lloyd_max_gaussian(uint32_t bits, float* levels) {
    constexpr int N = 8192;
    const float LO = -6.0f, HI = 6.0f;
    const float FRAC_1_SQRT_2 = 0.707106781186547524400844362104849039f;
    const float FRAC_2_SQRT_PI = 1.12837916709551257389615890312154517f;
    const size_t k = (size_t)1 << bits;
    const float dx = (HI - LO) / (float)N;
    float* xs = (float*)malloc(N * sizeof(float));
    float* pdf = (float*)malloc(N * sizeof(float));
    for (int i = 0; i < N; i++) xs[i] = std::fmaf((float)i + 0.5f, dx, LO);
    for (int i = 0; i < N; i++) {
        const float x = xs[i];
        pdf[i] = std::exp(-0.5f * x * x) * FRAC_1_SQRT_2 * FRAC_2_SQRT_PI / 2.0f;
    }
    for (size_t i = 0; i < k; i++) {
        const float t = ((float)i + 0.5f) / (float)k;
        levels[i] = 6.0f * (t - 0.5f);
    }
    float sum[16], wsum[16];
    for (int it = 0; it < 100; it++) {
        for (size_t j = 0; j < k; j++) { sum[j] = 0.0f; wsum[j] = 0.0f; }
        for (int i = 0; i < N; i++) {
            const float x = xs[i], w = pdf[i];
            size_t best = 0;
            float bd = INFINITY;
            for (size_t j = 0; j < k; j++) {
                const float dist = std::fabs(x - levels[j]);
                if (dist < bd) { bd = dist; best = j; }
            }
            sum[best] = std::fmaf(w, x, sum[best]);
            wsum[best] += w;
        }
        for (size_t j = 0; j < k; j++)
            if (wsum[j] > 1e-12f) levels[j] = sum[j] / wsum[j];
    }
    std::sort(levels, levels + k);
    free(xs);
    free(pdf);
}

}  // namespace

extern "C" {

int lh_turboquant_levels(uint32_t dim, uint32_t bits, float* levels) {
    if (!levels) return lh_fail(LH_ERR_INVALID_ARGUMENT, "turboquant_levels: levels is null");
    if (bits < 1 || bits > 4 || dim == 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "turboquant_levels: bad dim %u / bits %u", dim, bits);
    lloyd_max_gaussian(bits, levels);
    const float scale = 1.0f / std::sqrt((float)dim);     // turboquant.rs:187-192
    for (uint32_t i = 0; i < (1u << bits); i++) levels[i] = levels[i] * scale;
    return LH_OK;
}

int lh_turboquant_signs(uint32_t dim, uint64_t seed, float* signs) {
    if (!signs) return lh_fail(LH_ERR_INVALID_ARGUMENT, "turboquant_signs: signs is null");
    uint64_t state = seed | 1u;                              // turboquant.rs:66-79
    for (uint32_t i = 0; i < dim; i++) {
        state += 0x9E3779B97F4A7C15ull;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        signs[i] = (z & 1u) == 0 ? 1.0f : -1.0f;
    }
    return LH_OK;
}

uint32_t lh_turboquant_code_bytes(uint32_t dim, uint32_t bits) { return (dim * bits + 7) / 8; }

size_t lh_swa_ring_capacity(size_t window, size_t max_positions) {   // quant_cache.rs:48-54
    const size_t min_safe = window + 256 - 1;
    size_t v = std::max(window * 2, min_safe), p = 1;
    while (p < v) p <<= 1;
    return std::min(p, max_positions);
}

uint32_t lh_kv_bits_from_env(void) {                                 // quant_cache.rs:60-66
    const char* v = getenv("LOCAL_AI_KV_QUANT");
    if (v && strcmp(v, "tq3") == 0) return 3;
    if (v && strcmp(v, "tq4") == 0) return 4;
    return LH_DEFAULT_KV_BITS;
}

int lh_encode_kv_turboquant_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* levels, const lh_buffer* signs,
                                 lh_buffer* packed, lh_buffer* norms, uint32_t head_dim, uint32_t n_kv_heads, uint32_t num_tokens,
                                 uint32_t bits, uint32_t position, uint32_t ring_capacity) {
    const char* op = "encode_kv_turboquant";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    int r = check_tq_shape(op, head_dim, bits);
    if (r != LH_OK) return r;
    const uint32_t groups = n_kv_heads * num_tokens;
    if (groups == 0) return LH_OK;
    const uint32_t cb = lh_turboquant_code_bytes(head_dim, bits);
    // highest physical slot written
    const uint64_t phys_tokens = ring_capacity ? std::min<uint64_t>(ring_capacity, (uint64_t)position + num_tokens)
                                               : (uint64_t)position + num_tokens;
    LH_NEED(input, (size_t)groups * head_dim * 2, op, "input");
    LH_NEED(levels, (size_t)4 << bits, op, "levels");
    LH_NEED(signs, (size_t)head_dim * 4, op, "signs");
    LH_NEED(packed, (size_t)phys_tokens * n_kv_heads * cb, op, "packed");
    LH_NEED(norms, (size_t)phys_tokens * n_kv_heads * 2, op, "norms");
    EncodeParams p{head_dim, n_kv_heads, bits, cb, position, ring_capacity, 0, host_inv_sqrt(head_dim)};
    hipLaunchKernelGGL((encode_kv_kernel<false>), dim3(groups), dim3(head_dim), 0, batch->ctx->stream, (const uint16_t*)input->ptr,
                       (const float*)levels->ptr, (const float*)signs->ptr, (uint8_t*)packed->ptr, (uint16_t*)norms->ptr,
                       (const uint32_t*)nullptr, p);
    r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

int lh_encode_kv_turboquant(lh_context* ctx, const lh_buffer* input, const lh_buffer* levels, const lh_buffer* signs, lh_buffer* packed,
                            lh_buffer* norms, uint32_t head_dim, uint32_t n_kv_heads, uint32_t num_tokens, uint32_t bits,
                            uint32_t position, uint32_t ring_capacity) {
    if (!ctx) return lh_fail(LH_ERR_INVALID_ARGUMENT, "encode_kv_turboquant: context is null");
    lh_batch b{ctx, 0};
    int r = lh_encode_kv_turboquant_into(&b, input, levels, signs, packed, norms, head_dim, n_kv_heads, num_tokens, bits, position,
                                         ring_capacity);
    return r != LH_OK ? r : lh_batch_commit_and_wait(&b);
}

int lh_encode_kv_turboquant_batched_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* levels, const lh_buffer* signs,
                                         lh_buffer* packed, lh_buffer* norms, const lh_buffer* positions, uint32_t head_dim,
                                         uint32_t n_kv_heads, uint32_t lane_capacity, uint32_t bits, uint32_t n_lanes,
                                         uint32_t ring_capacity) {
    const char* op = "encode_kv_turboquant_batched";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    int r = check_tq_shape(op, head_dim, bits);
    if (r != LH_OK) return r;
    const uint32_t groups = n_kv_heads * n_lanes;
    if (groups == 0) return LH_OK;
    LH_REQUIRE(ring_capacity <= lane_capacity, "%s: ring_capacity %u exceeds lane_capacity %u", op, ring_capacity, lane_capacity);
    const uint32_t cb = lh_turboquant_code_bytes(head_dim, bits);
    LH_NEED(input, (size_t)groups * head_dim * 2, op, "input");
    LH_NEED(levels, (size_t)4 << bits, op, "levels");
    LH_NEED(signs, (size_t)head_dim * 4, op, "signs");
    LH_NEED(positions, (size_t)n_lanes * 4, op, "positions");
    // positions live in device memory, so the slot range cannot be checked here beyond the pool size
    LH_NEED(packed, (size_t)n_lanes * lane_capacity * n_kv_heads * cb, op, "packed");
    LH_NEED(norms, (size_t)n_lanes * lane_capacity * n_kv_heads * 2, op, "norms");
    EncodeParams p{head_dim, n_kv_heads, bits, cb, 0, ring_capacity, lane_capacity, host_inv_sqrt(head_dim)};
    hipLaunchKernelGGL((encode_kv_kernel<true>), dim3(groups), dim3(head_dim), 0, batch->ctx->stream, (const uint16_t*)input->ptr,
                       (const float*)levels->ptr, (const float*)signs->ptr, (uint8_t*)packed->ptr, (uint16_t*)norms->ptr,
                       (const uint32_t*)positions->ptr, p);
    r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

int lh_decode_qkv_prepare_rows_into(lh_batch* batch, lh_buffer* q, lh_buffer* k, lh_buffer* v, const lh_buffer* q_norm,
                                    const lh_buffer* k_norm, const lh_buffer* levels, const lh_buffer* signs, lh_buffer* rq, lh_buffer* k_codes,
                                    lh_buffer* k_norms, lh_buffer* v_codes, lh_buffer* v_norms, const lh_buffer* positions, uint32_t head_dim,
                                    uint32_t n_q_heads, uint32_t n_kv_heads, uint32_t rows, float eps, uint32_t start_position, float theta,
                                    float partial_rotary_factor, uint32_t bits, uint32_t ring_capacity, uint32_t lane_capacity) {
    const LhPrepareRows a{q, k, v, q_norm, k_norm, levels, signs, rq, k_codes, k_norms, v_codes, v_norms, positions, head_dim, n_q_heads, n_kv_heads,
                          rows, eps, start_position, theta, partial_rotary_factor, bits, ring_capacity, lane_capacity};
    return lh_prepare_rows_launch(batch, a, nullptr, 0, 0);
}

}  // extern "C"

int lh_prepare_rows_launch(lh_batch* batch, const LhPrepareRows& a, const float* partial, uint32_t splits, uint32_t part_cols, bool check_only) {
    lh_buffer* const q = a.q; lh_buffer* const k = a.k; lh_buffer* const v = a.v;
    const lh_buffer* const q_norm = a.q_norm; const lh_buffer* const k_norm = a.k_norm; const lh_buffer* const levels = a.levels;
    const lh_buffer* const signs = a.signs; lh_buffer* const rq = a.rq; lh_buffer* const k_codes = a.k_codes; lh_buffer* const k_norms = a.k_norms;
    lh_buffer* const v_codes = a.v_codes; lh_buffer* const v_norms = a.v_norms; const lh_buffer* const positions = a.positions;
    const uint32_t head_dim = a.head_dim, n_q_heads = a.n_q_heads, n_kv_heads = a.n_kv_heads, rows = a.rows, start_position = a.start_position,
                   bits = a.bits, ring_capacity = a.ring_capacity, lane_capacity = a.lane_capacity;
    const float eps = a.eps, theta = a.theta, partial_rotary_factor = a.partial_rotary_factor;
    const char* op = "decode_qkv_prepare";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    int r = check_tq_shape(op, head_dim, bits);
    if (r != LH_OK) return r;
    LH_REQUIRE(head_dim >= 64, "%s: head_dim %u below 64", op, head_dim);
    if (n_q_heads == 0 || rows == 0) return LH_OK;
    LH_REQUIRE((positions != nullptr) == (lane_capacity != 0), "%s: a positions table and a lane capacity go together", op);
    LH_REQUIRE(ring_capacity <= lane_capacity || lane_capacity == 0, "%s: ring_capacity %u exceeds lane_capacity %u", op, ring_capacity, lane_capacity);
    const bool write_kv = k != nullptr && v != nullptr && n_kv_heads != 0;
    const uint32_t cb = lh_turboquant_code_bytes(head_dim, bits);
    LH_NEED(q, (size_t)rows * n_q_heads * head_dim * 2, op, "q");
    LH_NEED(rq, (size_t)rows * n_q_heads * head_dim * 4, op, "rq");
    LH_NEED(signs, (size_t)head_dim * 4, op, "signs");
    if (q_norm) LH_NEED(q_norm, (size_t)head_dim * 2, op, "q_norm");
    if (positions) LH_NEED(positions, (size_t)rows * 4, op, "positions");
    if (write_kv) {
        // one sequence: rows land at start_position .. + rows (modulo the ring); lanes: positions live in device memory,
        // so the slot range cannot be checked here beyond the pool size
        const uint64_t last = (uint64_t)start_position + rows;
        const uint64_t phys = lane_capacity ? (uint64_t)rows * lane_capacity : (ring_capacity ? std::min<uint64_t>(ring_capacity, last) : last);
        LH_NEED(k, (size_t)rows * n_kv_heads * head_dim * 2, op, "k");
        LH_NEED(v, (size_t)rows * n_kv_heads * head_dim * 2, op, "v");
        LH_NEED(levels, (size_t)4 << bits, op, "levels");
        if (k_norm) LH_NEED(k_norm, (size_t)head_dim * 2, op, "k_norm");
        LH_NEED(k_codes, (size_t)phys * n_kv_heads * cb, op, "k_codes");
        LH_NEED(v_codes, (size_t)phys * n_kv_heads * cb, op, "v_codes");
        LH_NEED(k_norms, (size_t)phys * n_kv_heads * 2, op, "k_norms");
        LH_NEED(v_norms, (size_t)phys * n_kv_heads * 2, op, "v_norms");
    }
    PrepareParams p{head_dim, n_q_heads, write_kv ? n_kv_heads : 0u, bits, cb, start_position, ring_capacity, write_kv ? 1u : 0u, lane_capacity,
                    eps, theta, partial_rotary_factor, host_inv_sqrt(head_dim), partial, splits, part_cols, rows};
    const uint64_t groups = (uint64_t)rows * (n_q_heads + (write_kv ? 2 * n_kv_heads : 0));
    LH_REQUIRE(groups <= 0x7FFFFFFFull, "%s: %u rows are too many for one launch", op, rows);
    if (partial) LH_REQUIRE(splits >= 1 && (uint64_t)(n_q_heads + (write_kv ? 2 * n_kv_heads : 0)) * head_dim <= part_cols,
                            "%s: partial tiles of %u columns do not hold the heads", op, part_cols);
    if (check_only) return LH_OK;
    hipLaunchKernelGGL(decode_qkv_prepare_kernel, dim3((uint32_t)groups), dim3(head_dim), 0, batch->ctx->stream, (uint16_t*)q->ptr,
                       write_kv ? (uint16_t*)k->ptr : nullptr, write_kv ? (uint16_t*)v->ptr : nullptr,
                       q_norm ? (const uint16_t*)q_norm->ptr : nullptr, (write_kv && k_norm) ? (const uint16_t*)k_norm->ptr : nullptr,
                       (const float*)signs->ptr, write_kv ? (const float*)levels->ptr : nullptr, (float*)rq->ptr,
                       write_kv ? (uint8_t*)k_codes->ptr : nullptr, write_kv ? (uint16_t*)k_norms->ptr : nullptr,
                       write_kv ? (uint8_t*)v_codes->ptr : nullptr, write_kv ? (uint16_t*)v_norms->ptr : nullptr,
                       positions ? (const uint32_t*)positions->ptr : nullptr, p);
    r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

extern "C" {

int lh_decode_qkv_prepare_into(lh_batch* batch, lh_buffer* q, lh_buffer* k, lh_buffer* v, const lh_buffer* q_norm, const lh_buffer* k_norm,
                               const lh_buffer* levels, const lh_buffer* signs, lh_buffer* rq, lh_buffer* k_codes, lh_buffer* k_norms,
                               lh_buffer* v_codes, lh_buffer* v_norms, uint32_t head_dim, uint32_t n_q_heads, uint32_t n_kv_heads, float eps,
                               uint32_t position, float theta, float partial_rotary_factor, uint32_t bits, uint32_t ring_capacity) {
    return lh_decode_qkv_prepare_rows_into(batch, q, k, v, q_norm, k_norm, levels, signs, rq, k_codes, k_norms, v_codes, v_norms, nullptr,
                                           head_dim, n_q_heads, n_kv_heads, 1, eps, position, theta, partial_rotary_factor, bits, ring_capacity, 0);
}

int lh_dequantize_kv_turboquant_into(lh_batch* batch, const lh_buffer* packed, const lh_buffer* norms, const lh_buffer* levels,
                                     const lh_buffer* signs, lh_buffer* output, uint32_t head_dim, uint32_t n_kv_heads,
                                     uint32_t num_tokens, uint32_t bits, uint32_t token_start, uint32_t ring_capacity) {
    const char* op = "dequantize_kv_turboquant";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    int r = check_tq_shape(op, head_dim, bits);
    if (r != LH_OK) return r;
    if (token_start > num_tokens) token_start = num_tokens;              // kernels.rs:4668
    const uint32_t groups = n_kv_heads * (num_tokens - token_start);
    if (groups == 0) return LH_OK;
    const uint32_t cb = lh_turboquant_code_bytes(head_dim, bits);
    const uint64_t phys_tokens = ring_capacity ? std::min<uint64_t>(ring_capacity, num_tokens) : num_tokens;
    LH_NEED(packed, (size_t)phys_tokens * n_kv_heads * cb, op, "packed");
    LH_NEED(norms, (size_t)phys_tokens * n_kv_heads * 2, op, "norms");
    LH_NEED(levels, (size_t)4 << bits, op, "levels");
    LH_NEED(signs, (size_t)head_dim * 4, op, "signs");
    LH_NEED(output, (size_t)num_tokens * n_kv_heads * head_dim * 2, op, "output");
    DequantParams p{head_dim, n_kv_heads, bits, cb, token_start * n_kv_heads, ring_capacity, host_inv_sqrt(head_dim)};
    hipLaunchKernelGGL(dequantize_kv_kernel, dim3(groups), dim3(head_dim), 0, batch->ctx->stream, (const uint8_t*)packed->ptr,
                       (const uint16_t*)norms->ptr, (const float*)levels->ptr, (const float*)signs->ptr, (uint16_t*)output->ptr, p);
    r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

int lh_dequantize_kv_turboquant(lh_context* ctx, const lh_buffer* packed, const lh_buffer* norms, const lh_buffer* levels,
                                const lh_buffer* signs, lh_buffer* output, uint32_t head_dim, uint32_t n_kv_heads, uint32_t num_tokens,
                                uint32_t bits, uint32_t token_start, uint32_t ring_capacity) {
    if (!ctx) return lh_fail(LH_ERR_INVALID_ARGUMENT, "dequantize_kv_turboquant: context is null");
    lh_batch b{ctx, 0};
    int r = lh_dequantize_kv_turboquant_into(&b, packed, norms, levels, signs, output, head_dim, n_kv_heads, num_tokens, bits,
                                             token_start, ring_capacity);
    return r != LH_OK ? r : lh_batch_commit_and_wait(&b);
}

int lh_hadamard_rotate_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs, lh_buffer* output, uint32_t head_dim,
                            uint32_t num_heads, int pre_sign, int post_sign) {
    return hadamard_launch<float, float>(batch, input, signs, output, head_dim, num_heads, pre_sign, post_sign, "hadamard_rotate");
}
int lh_hadamard_rotate_hf_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs, lh_buffer* output, uint32_t head_dim,
                               uint32_t num_heads, int pre_sign, int post_sign) {
    return hadamard_launch<uint16_t, float>(batch, input, signs, output, head_dim, num_heads, pre_sign, post_sign, "hadamard_rotate_hf");
}
int lh_hadamard_rotate_fh_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* signs, lh_buffer* output, uint32_t head_dim,
                               uint32_t num_heads, int pre_sign, int post_sign) {
    return hadamard_launch<float, uint16_t>(batch, input, signs, output, head_dim, num_heads, pre_sign, post_sign, "hadamard_rotate_fh");
}

}  // extern "C"
