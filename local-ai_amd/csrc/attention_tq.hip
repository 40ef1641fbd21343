// Fused flash-decoding attention straight from packed TurboQuant codes.
//
// Stands in for shaders/attention_flash_tq.metal:154-690 (flash_attention_tq,
// _prefill, _prefill_tiled, _batched) and their dispatch in
// local-metal/src/kernels.rs:5176-5506.
//
// Semantics kept from the reference: seq_len = min(kv_len, pos + 1); the window
// starts at pos + 1 - window when that is positive; logical position t lives in
// physical row t % ring_capacity when a ring is used; logit_t = f32(norm_k[t]) *
// sum_i rq_i * levels[Kcode_{t,i}] with no 1/sqrt(d) factor; the output is the
// softmax-weighted sum of f32(norm_v[t]) * levels[Vcode_{t,i}], normalised, in
// rotated space; an empty range gives zeros.
//
// Structure here (different from the reference's one-threadgroup-per-head scan):
//  * split-K: the position range of one query is cut into `num_splits` chunks, one
//    workgroup each; every workgroup serves ALL query heads that share the KV
//    head (GQA), so each cached position is read and decoded once, not once per
//    query head;
//  * per workgroup the partial (max, sum, acc[head_dim]) per head goes to a
//    workspace and a second small kernel does the log-sum-exp merge; with one
//    split the workgroup writes the final result itself.
#include "attention_tq.hpp"
#include <atomic>
#include <algorithm>
#include <cmath>

namespace {
using namespace lh_attn;

constexpr int kThreads = 256;
constexpr int kWavesPerWG = kThreads / 64;
constexpr int kMaxDpl = 8;        // head_dim 512 over 64 lanes
constexpr int kHeadsPerPass = 8;  // query heads served together from one decode of a position
constexpr int kPosBatch = 8;      // positions whose loads a wave keeps in flight together

// Split-K partial records of lh_flash_attention_tq_static_into: device memory that exists from the moment the code
// object is loaded, so that entry never allocates.  Every GPU the library runs on holds its own copy at its own address
// until the process ends; the name below is only a host-side handle, the address comes from hipGetSymbolAddress.
constexpr size_t kStaticScratchFloats = (size_t)2 << 20;          // 8 MiB
constexpr uint32_t kStaticMinSplits = 256;                        // split records that must fit for a call to be accepted
static __device__ __align__(256) float scratch[kStaticScratchFloats];
constexpr int kMaxDevices = 64;
static std::atomic<float*> g_scratch_ptr[kMaxDevices];            // per device, set by lh_attention_static_scratch_init (contexts may open on several threads)

// The lane's bit window of one code record: `dpl` codes starting at bit lane*dpl*bits.
__device__ __forceinline__ uint32_t load_window(const uint8_t* rec, uint32_t byte0, uint32_t nbytes) {
    uint32_t v = 0;
    for (uint32_t i = 0; i < nbytes; i++) v |= (uint32_t)rec[byte0 + i] << (8 * i);
    return v;
}

// Sum each of 8 per-lane values over the 64 lanes; lane l ends with the total of value (l & 7).
// (Halving butterfly: 7 exchanges instead of 8 full reductions.)
__device__ __forceinline__ float reduce8(const float (&v)[8], int lane) {
    float a[4];
    const bool b0 = lane & 1;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const float keep = b0 ? v[2 * j + 1] : v[2 * j];
        const float give = b0 ? v[2 * j] : v[2 * j + 1];
        a[j] = keep + lh_dpp_f<LH_DPP_QUAD_XOR1>(give);
    }
    float b[2];
    const bool b1 = lane & 2;
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const float keep = b1 ? a[2 * j + 1] : a[2 * j];
        const float give = b1 ? a[2 * j] : a[2 * j + 1];
        b[j] = keep + lh_dpp_f<LH_DPP_QUAD_XOR2>(give);
    }
    const bool b2 = lane & 4;
    const float keep = b2 ? b[1] : b[0];
    const float give = b2 ? b[0] : b[1];
    // row_half_mirror pairs lane i with 7-i: the partner's bit 2 differs and its low two bits are
    // complemented, so route through an xor-4 exchange instead.
    float c = keep + __shfl_xor(give, 4, 64);
    c += __shfl_xor(c, 8, 64);
    c += lh_swap16_f(c);
    c += lh_swap32_f(c);
    return c;   // total of value index ((lane&1) | (lane&2) | (lane&4)) -> lane & 7
}

__global__ __launch_bounds__(kThreads) void attention_tq_split_kernel(
    const float* __restrict__ rq, const uint8_t* __restrict__ k_codes, const uint16_t* __restrict__ k_norms,
    const uint8_t* __restrict__ v_codes, const uint16_t* __restrict__ v_norms, const float* __restrict__ levels,
    const uint32_t* __restrict__ positions, float* __restrict__ out, float* __restrict__ ws, AttnParams p) {
    __shared__ float lds_levels[16];
    __shared__ float lds_m[kWavesPerWG][kHeadsPerPass];
    __shared__ float lds_l[kWavesPerWG][kHeadsPerPass];
    extern __shared__ __align__(16) float lds_acc[];   // [wave][head][head_dim]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t split = blockIdx.x;
    const uint32_t qi = blockIdx.y / p.num_kv_heads, kvh = blockIdx.y - qi * p.num_kv_heads;
    const uint32_t hd = p.head_dim, bits = p.bits;
    const uint32_t group = p.num_q_heads / p.num_kv_heads;           // query heads per KV head
    const uint32_t dpl = hd >= 64 ? hd / 64 : 1;                     // dims per lane (contiguous)
    const bool lane_on = hd >= 64 || (uint32_t)lane < hd;
    const uint32_t d0 = lane * dpl;
    const uint32_t bit0 = d0 * bits, byte0 = bit0 >> 3, shift0 = bit0 & 7u;
    const uint32_t nbytes = lane_on ? (shift0 + dpl * bits + 7u) / 8u : 0u;
    const uint32_t cmask = (1u << bits) - 1u;

    if (threadIdx.x < (1u << bits)) lds_levels[threadIdx.x] = levels[threadIdx.x];
    __syncthreads();

    uint32_t lo, hi, lane_base;
    query_range(p, positions, qi, lo, hi, lane_base);
    const uint32_t n = hi - lo;
    const uint32_t chunk = (n + p.num_splits - 1) / p.num_splits;
    const uint32_t c_lo = lo + std::min(n, split * chunk);
    const uint32_t c_hi = lo + std::min(n, (split + 1) * chunk);

    for (uint32_t h0 = 0; h0 < group; h0 += kHeadsPerPass) {
        const uint32_t nh = std::min<uint32_t>(kHeadsPerPass, group - h0);
        const uint32_t qh0 = kvh * group + h0;
        float rqr[kHeadsPerPass][kMaxDpl], acc[kHeadsPerPass][kMaxDpl];
#pragma unroll
        for (int h = 0; h < kHeadsPerPass; h++)
#pragma unroll
            for (int i = 0; i < kMaxDpl; i++) {
                acc[h][i] = 0.0f;
                rqr[h][i] = ((uint32_t)h < nh && (uint32_t)i < dpl && lane_on)
                                ? rq[((size_t)qi * p.num_q_heads + qh0 + h) * hd + d0 + i] : 0.0f;
            }
        // lane l tracks the running max / sum of head (l & 7)
        float run_m = -INFINITY, run_l = 0.0f;

        // each wave takes batches of kPosBatch consecutive positions; all loads of a batch are
        // issued before any of it is consumed
        for (uint32_t tb = c_lo + wave * kPosBatch; tb < c_hi; tb += kWavesPerWG * kPosBatch) {
            uint32_t kw[kPosBatch], vw[kPosBatch];
            float kn[kPosBatch], vn[kPosBatch];
#pragma unroll
            for (int j = 0; j < kPosBatch; j++) {
                const uint32_t t = std::min(tb + j, c_hi - 1);          // past-the-end entries re-read the last one (unused)
                const uint32_t pt = p.ring_capacity ? t % p.ring_capacity : t;
                const size_t slot = (size_t)(lane_base + pt) * p.num_kv_heads + kvh;
                kw[j] = load_window(k_codes + slot * p.code_bytes, byte0, nbytes) >> shift0;
                vw[j] = load_window(v_codes + slot * p.code_bytes, byte0, nbytes) >> shift0;
                kn[j] = lh_h2f(k_norms[slot]);
                vn[j] = lh_h2f(v_norms[slot]);
            }
#pragma unroll
            for (int j = 0; j < kPosBatch; j++) {
                if (tb + j >= c_hi) break;
                float dot[kHeadsPerPass];
#pragma unroll
                for (int h = 0; h < kHeadsPerPass; h++) dot[h] = 0.0f;
#pragma unroll
                for (int i = 0; i < kMaxDpl; i++) {
                    if ((uint32_t)i < dpl) {
                        const float kv = lds_levels[(kw[j] >> (i * bits)) & cmask];
#pragma unroll
                        for (int h = 0; h < kHeadsPerPass; h++) dot[h] += rqr[h][i] * kv;
                    }
                }
                const float logit = reduce8(dot, lane) * kn[j];                 // head (lane & 7)
                const float new_m = fmaxf(run_m, logit);
                const float rescale = __expf(run_m - new_m);                    // exp(-inf) = 0 on the first position
                const float w = __expf(logit - new_m);
                run_l = run_l * rescale + w;
                run_m = new_m;
                const float wv = w * vn[j];
                float vv[kMaxDpl];
#pragma unroll
                for (int i = 0; i < kMaxDpl; i++) vv[i] = (uint32_t)i < dpl ? lds_levels[(vw[j] >> (i * bits)) & cmask] : 0.0f;
#pragma unroll
                for (int h = 0; h < kHeadsPerPass; h++) {
                    const float r_h = __shfl(rescale, h, 64), w_h = __shfl(wv, h, 64);
#pragma unroll
                    for (int i = 0; i < kMaxDpl; i++)
                        if ((uint32_t)i < dpl) acc[h][i] = acc[h][i] * r_h + w_h * vv[i];
                }
            }
        }

        // merge the four waves (log-sum-exp), then either finish or hand the partial to the reduce kernel
        __syncthreads();
        if (lane < kHeadsPerPass) { lds_m[wave][lane] = run_m; lds_l[wave][lane] = run_l; }
#pragma unroll
        for (int h = 0; h < kHeadsPerPass; h++)
#pragma unroll
            for (int i = 0; i < kMaxDpl; i++)
                if ((uint32_t)i < dpl && lane_on) lds_acc[((size_t)wave * kHeadsPerPass + h) * hd + d0 + i] = acc[h][i];
        __syncthreads();
        for (uint32_t idx = threadIdx.x; idx < nh * hd; idx += kThreads) {
            const uint32_t h = idx / hd, d = idx - h * hd;
            float gm = -INFINITY;
#pragma unroll
            for (int w = 0; w < kWavesPerWG; w++) gm = fmaxf(gm, lds_m[w][h]);
            float gl = 0.0f, o = 0.0f;
#pragma unroll
            for (int w = 0; w < kWavesPerWG; w++) {
                const float f = lds_m[w][h] == -INFINITY ? 0.0f : __expf(lds_m[w][h] - gm);
                gl += f * lds_l[w][h];
                o += f * lds_acc[((size_t)w * kHeadsPerPass + h) * hd + d];
            }
            const uint32_t qh = qh0 + h;
            if (p.num_splits == 1) {
                out[((size_t)qi * p.num_q_heads + qh) * hd + d] = gl > 0.0f ? o / gl : 0.0f;
            } else {
                // workspace: per (query, head, split): [m, l, pad, pad, acc[hd]]
                float* rec = ws + (((size_t)qi * p.num_q_heads + qh) * p.num_splits + split) * (hd + 4);
                if (d == 0) { rec[0] = gm; rec[1] = gl; }
                rec[4 + d] = o;
            }
        }
    }
}

// flash_decoding.metal:148-189 applied to the TQ partials: LSE merge over splits.  One workgroup per
// (query, head, slab of 32 output dims): the per-split factors exp(m_s - max) are computed once into LDS,
// then thread groups fold interleaved subsets of the splits (coalesced 128-byte row reads, a batch of
// them in flight per thread, the first batch requested before the factors are known) and are summed through LDS.
constexpr int kReduceDims = 32;     // dims per workgroup
constexpr int kReduceBatch = 16;    // records per thread whose loads are in flight together
// kReduceSlices thread groups fold interleaved subsets of the splits: 16 for many splits (one long query), 2 for few
// (many queries, each with its own small merge).
template <int kReduceSlices>
__global__ __launch_bounds__(kReduceDims * kReduceSlices) void attention_tq_reduce_kernel(const float* __restrict__ ws, float* __restrict__ out,
                                                                                          uint32_t head_dim, uint32_t num_splits) {
    constexpr int kThreads = kReduceDims * kReduceSlices, kWaves = kThreads / 64;
    constexpr int kMl = kMaxSplits / kThreads;   // (m, l) pairs per thread
    __shared__ float f_s[kMaxSplits];
    __shared__ float red[2 * kWaves];
    __shared__ float part[kReduceSlices][kReduceDims];
    const uint32_t qh = blockIdx.x;     // flattened (query, head)
    const size_t rec = partial_record_floats(head_dim);
    const float* base = ws + (size_t)qh * num_splits * rec;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t dl = threadIdx.x & (kReduceDims - 1), slice = threadIdx.x / kReduceDims;
    const uint32_t d = blockIdx.y * kReduceDims + dl;
    const bool d_ok = d < head_dim;

    // The first batch of accumulator rows does not depend on the split weights: request it before anything else.
    float v[kReduceBatch];
#pragma unroll
    for (int i = 0; i < kReduceBatch; i++) {
        const uint32_t sp = slice + kReduceSlices * i;
        v[i] = (d_ok && sp < num_splits) ? base[(size_t)sp * rec + 4 + d] : 0.0f;
    }
    // (m, l) of every split, kMl per thread
    float2 ml[kMl];
#pragma unroll
    for (int i = 0; i < kMl; i++) {
        const uint32_t sp = threadIdx.x + kThreads * i;
        ml[i] = sp < num_splits ? *reinterpret_cast<const float2*>(base + (size_t)sp * rec) : make_float2(-INFINITY, 0.0f);
    }
    float m_loc = -INFINITY;
#pragma unroll
    for (int i = 0; i < kMl; i++) m_loc = fmaxf(m_loc, ml[i].x);
    m_loc = lh_group_max(m_loc, 64);
    if (lane == 0) red[wave] = m_loc;
    __syncthreads();
    float gm = red[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) gm = fmaxf(gm, red[w]);
    float l_loc = 0.0f;
#pragma unroll
    for (int i = 0; i < kMl; i++) {
        const uint32_t sp = threadIdx.x + kThreads * i;
        const float f = ml[i].x == -INFINITY ? 0.0f : __expf(ml[i].x - gm);
        if (sp < num_splits) f_s[sp] = f;
        l_loc += f * ml[i].y;
    }
    l_loc = lh_group_sum(l_loc, 64);
    if (lane == 0) red[kWaves + wave] = l_loc;
    __syncthreads();
    float gl = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) gl += red[kWaves + w];
    const float inv = gl > 0.0f ? 1.0f / gl : 0.0f;

    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < kReduceBatch; i++) {
        const uint32_t sp = slice + kReduceSlices * i;
        if (sp < num_splits) o = __builtin_fmaf(f_s[sp], v[i], o);
    }
    for (uint32_t s0 = kReduceSlices * kReduceBatch; s0 < num_splits; s0 += kReduceSlices * kReduceBatch) {   // more than 256 splits
#pragma unroll
        for (int i = 0; i < kReduceBatch; i++) {
            const uint32_t sp = s0 + slice + kReduceSlices * i;
            v[i] = (d_ok && sp < num_splits) ? base[(size_t)sp * rec + 4 + d] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < kReduceBatch; i++) {
            const uint32_t sp = s0 + slice + kReduceSlices * i;
            if (sp < num_splits) o = __builtin_fmaf(f_s[sp], v[i], o);
        }
    }
    part[slice][dl] = o;
    __syncthreads();
    if (slice == 0 && d_ok) {
        float t = 0.0f;
#pragma unroll
        for (int i = 0; i < kReduceSlices; i++) t += part[i][dl];
        out[(size_t)qh * head_dim + d] = t * inv;
    }
}

// The merge for a few splits per query (a batch of sequences, each cut into a handful of chunks): one wave per
// (query, head), four of them in a workgroup, every lane a float4 of each partial row.  A launch of one small
// workgroup per 32 dims spends its time on scheduling workgroups (256 sequences x 8 heads x 4 splits: 10.5 us);
// this form reads the same records with a sixteenth of the workgroups.  The arithmetic is attention_tq_reduce_kernel<2>'s
// in its order: the factors and their sum with one split per lane, two interleaved fma chains per dim, added.
constexpr uint32_t kWaveMergeMaxSplits = 16;
__global__ __launch_bounds__(256) void attention_tq_reduce_wave_kernel(const float* __restrict__ ws, float* __restrict__ out, uint32_t head_dim,
                                                                       uint32_t num_splits, uint32_t num_qh) {
    const uint32_t lane = threadIdx.x & 63, qh = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (qh >= num_qh) return;
    const size_t rec = partial_record_floats(head_dim);
    const float* base = ws + (size_t)qh * num_splits * rec;
    const float2 ml = lane < num_splits ? *reinterpret_cast<const float2*>(base + (size_t)lane * rec) : make_float2(-INFINITY, 0.0f);
    const float gm = lh_group_max(ml.x, 64);
    const float f = ml.x == -INFINITY ? 0.0f : __expf(ml.x - gm);
    float l_loc = 0.0f;
    l_loc += f * ml.y;
    l_loc = lh_group_sum(l_loc, 64);
    float gl = 0.0f;
    gl += l_loc;
    const float inv = gl > 0.0f ? 1.0f / gl : 0.0f;
    float fs[kWaveMergeMaxSplits];
#pragma unroll
    for (uint32_t i = 0; i < kWaveMergeMaxSplits; i++) fs[i] = __shfl(f, (int)i, 64);
    for (uint32_t d4 = lane; d4 < head_dim / 4; d4 += 64) {
        float4 v[kWaveMergeMaxSplits];
#pragma unroll
        for (uint32_t i = 0; i < kWaveMergeMaxSplits; i++)
            v[i] = i < num_splits ? *reinterpret_cast<const float4*>(base + (size_t)i * rec + 4 + 4 * d4) : make_float4(0.f, 0.f, 0.f, 0.f);
        float o0[4] = {0.f, 0.f, 0.f, 0.f}, o1[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (uint32_t i = 0; i < kWaveMergeMaxSplits; i += 2) {
            if (i < num_splits) {
                o0[0] = __builtin_fmaf(fs[i], v[i].x, o0[0]); o0[1] = __builtin_fmaf(fs[i], v[i].y, o0[1]);
                o0[2] = __builtin_fmaf(fs[i], v[i].z, o0[2]); o0[3] = __builtin_fmaf(fs[i], v[i].w, o0[3]);
            }
            if (i + 1 < num_splits) {
                o1[0] = __builtin_fmaf(fs[i + 1], v[i + 1].x, o1[0]); o1[1] = __builtin_fmaf(fs[i + 1], v[i + 1].y, o1[1]);
                o1[2] = __builtin_fmaf(fs[i + 1], v[i + 1].z, o1[2]); o1[3] = __builtin_fmaf(fs[i + 1], v[i + 1].w, o1[3]);
            }
        }
        float r[4];
#pragma unroll
        for (int c = 0; c < 4; c++) { float t = 0.0f; t += o0[c]; t += o1[c]; r[c] = t * inv; }
        *reinterpret_cast<float4*>(out + (size_t)qh * head_dim + 4 * d4) = make_float4(r[0], r[1], r[2], r[3]);
    }
}

// The merge of up to 2 * kReduceBatch splits and the rotation back out of code space (attention_flash_tq.metal:58-90 with
// the post-sign) in one launch: one workgroup per (query, head), one thread per output dim.  The merge is
// attention_tq_reduce_kernel<2>'s arithmetic in its order (the split factors and their sum on the first wave with one
// split per lane, two interleaved fma chains per dim, added), the rotation hadamard_rotate_kernel's, so the f16 result
// equals the two launches' bit for bit.
__global__ __launch_bounds__(512) void attention_tq_reduce_rotate_kernel(const float* __restrict__ ws, const float* __restrict__ signs,
                                                                         uint16_t* __restrict__ out, uint32_t head_dim, uint32_t num_splits,
                                                                         float inv_sqrt_d) {
    __shared__ __align__(16) float sh[512];
    __shared__ float f_s[2 * kReduceBatch];
    __shared__ float gl_s;
    const uint32_t qh = blockIdx.x, d = threadIdx.x;
    const size_t rec = partial_record_floats(head_dim);
    const float* base = ws + (size_t)qh * num_splits * rec;
    const float sign = signs[d];   // requested with the records, not behind the transform's barriers
    float v[2 * kReduceBatch];
#pragma unroll
    for (int i = 0; i < 2 * kReduceBatch; i++) v[i] = (uint32_t)i < num_splits ? base[(size_t)i * rec + 4 + d] : 0.0f;
    if (d < 64) {
        const float2 ml = d < num_splits ? *reinterpret_cast<const float2*>(base + (size_t)d * rec) : make_float2(-INFINITY, 0.0f);
        float gm = lh_group_max(ml.x, 64);
        gm = __shfl(gm, 0, 64);
        const float f = ml.x == -INFINITY ? 0.0f : __expf(ml.x - gm);
        if (d < num_splits) f_s[d] = f;
        float l_loc = 0.0f;
        l_loc += f * ml.y;
        l_loc = lh_group_sum(l_loc, 64);
        if (d == 0) gl_s = l_loc;
    }
    __syncthreads();
    float gl = 0.0f;
    gl += gl_s;
    const float inv = gl > 0.0f ? 1.0f / gl : 0.0f;
    float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
    for (int i = 0; i < kReduceBatch; i++) {
        if ((uint32_t)(2 * i) < num_splits) o0 = __builtin_fmaf(f_s[2 * i], v[2 * i], o0);
        if ((uint32_t)(2 * i + 1) < num_splits) o1 = __builtin_fmaf(f_s[2 * i + 1], v[2 * i + 1], o1);
    }
    float t = 0.0f;
    t += o0;
    t += o1;
    sh[d] = t * inv;
    lh_fwht_lds(sh, head_dim, d);
    float y = __fmul_rn(sh[d], inv_sqrt_d);
    y = __fmul_rn(y, sign);
    out[(size_t)qh * head_dim + d] = lh_f2h_exact(y);
}

// Where the f16 head outputs go when an entry also rotates back out of code space.
struct RotateBack {
    const lh_buffer* signs;
    lh_buffer* out16;
    // Lazy: rotate only where it rides in the merge launch (2 .. 32 partial records); otherwise leave the f32 heads in `out`
    // unrotated and say so in *rotated, so that the caller's next kernel can rotate them while it stages them.
    int* rotated = nullptr;
};

int attention_dispatch(lh_batch* batch, const char* op, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                       const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                       const lh_buffer* positions, AttnParams p, uint64_t max_span, uint64_t phys_slots, const RotateBack* rot = nullptr,
                       float* ws_override = nullptr, size_t ws_override_floats = 0) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (p.bits < 2 || p.bits > 4) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: TurboQuant bits must be 2..=4, got %u", op, p.bits);
    if (p.head_dim == 0 || (p.head_dim & (p.head_dim - 1)) || p.head_dim > 512)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: TurboQuant head_dim must be a power of two <= 512, got %u", op, p.head_dim);
    if (p.num_kv_heads == 0 || p.num_q_heads % p.num_kv_heads != 0)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: num_q_heads %u is not a multiple of num_kv_heads %u", op, p.num_q_heads, p.num_kv_heads);
    if (p.num_queries == 0 || p.num_q_heads == 0) return LH_OK;
    lh_context* ctx = batch->ctx;
    p.code_bytes = (p.head_dim * p.bits + 7) / 8;
    const size_t qbytes = (size_t)p.num_queries * p.num_q_heads * p.head_dim * 4;
    LH_NEED(rq, qbytes, op, "rq");
    LH_NEED(out, qbytes, op, "out");
    LH_NEED(levels, (size_t)4 << p.bits, op, "levels");
    LH_NEED(k_codes, (size_t)phys_slots * p.code_bytes, op, "k_codes");
    LH_NEED(v_codes, (size_t)phys_slots * p.code_bytes, op, "v_codes");
    LH_NEED(k_norms, (size_t)phys_slots * 2, op, "k_norms");
    LH_NEED(v_norms, (size_t)phys_slots * 2, op, "v_norms");
    if (p.mode == kBatched) LH_NEED(positions, (size_t)p.num_queries * 4, op, "positions");
    if (rot) {
        if (p.head_dim < 64) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: the rotated form needs head_dim >= 64, got %u", op, p.head_dim);
        LH_NEED(rot->signs, (size_t)p.head_dim * 4, op, "signs");
        LH_NEED(rot->out16, qbytes / 2, op, "out_f16");
    }

    float* const ws = ws_override ? ws_override : (float*)ctx->workspace;
    const size_t ws_avail = ws_override ? ws_override_floats : (ctx->workspace_bytes / 2) / 4;   // floats; the lower half of the workspace
    const AttnPointers ptrs{(const float*)rq->ptr, (const uint8_t*)k_codes->ptr, (const uint16_t*)k_norms->ptr,
                            (const uint8_t*)v_codes->ptr, (const uint16_t*)v_norms->ptr, (const float*)levels->ptr,
                            positions ? (const uint32_t*)positions->ptr : nullptr, (float*)out->ptr, ws, ctx->fault_dev};
    // Prefill entries with more than one row.  Sixteen rows sharing a pass over the codes (the tiled kernel) pay when there
    // is enough work to keep its eight-wave workgroups busy: measured against one query row per workgroup it wins from about
    // 1.5 M (row, position) pairs on (256 rows over 8k positions: 50 against 60 us; over 32k: 118 against 192) and loses
    // below (64 rows over 8k: 36 against 28 us; 256 rows over a 512-position window: 35 against 21), where a launch is
    // latency and the per-row form has the shorter chain per workgroup.  LOCAL_HIP_ATTN_PREFILL=rows / =tiled take one
    // form for every launch it supports (each is validated against the oracle that way).
    static const int prefill_env = [] { const char* e = getenv("LOCAL_HIP_ATTN_PREFILL"); return !e ? 0 : e[0] == 'r' ? 1 : e[0] == 't' ? 2 : 0; }();
    const bool tiled_pays = (uint64_t)p.num_queries * max_span >= 1500000ull;
    if (max_span != 0 && prefill_env != 1 && (prefill_env == 2 || tiled_pays) && prefill_tile_supported(p, ptrs)) {
        const int rl = launch_prefill_tile(ctx, op, ptrs, p, max_span, ws_avail);
        if (rl != LH_OK) return rl;
    } else if (max_span == 0 || !mfma_supported(p, ptrs)) {
        // Enough workgroups to fill the chip (about two per CU), at least 32 positions per workgroup.
        const uint64_t per_query_wgs = std::max<uint64_t>(1, (uint64_t)ctx->cu_count * 2 / ((uint64_t)p.num_queries * p.num_kv_heads));
        uint64_t splits = std::min<uint64_t>(per_query_wgs, (max_span + 31) / 32);
        splits = std::min<uint64_t>(std::max<uint64_t>(splits, 1), kMaxSplits);
        const size_t rec = partial_record_floats(p.head_dim);
        while (splits > 1 && (size_t)p.num_queries * p.num_q_heads * splits * rec > ws_avail) splits--;
        p.num_splits = (uint32_t)splits;

        const size_t lds_bytes = (size_t)kWavesPerWG * kHeadsPerPass * p.head_dim * 4;
        if (lds_bytes > 48 * 1024) {
            const int rl = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_split_kernel, 72 * 1024, op);
            if (rl != LH_OK) return rl;
        }
        hipLaunchKernelGGL(attention_tq_split_kernel, dim3(p.num_splits, p.num_queries * p.num_kv_heads), dim3(kThreads), lds_bytes, ctx->stream,
                           ptrs.rq, ptrs.k_codes, ptrs.k_norms, ptrs.v_codes, ptrs.v_norms, ptrs.levels, ptrs.positions, ptrs.out, ptrs.ws, p);
    } else {
        const int rl = launch_mfma(ctx, op, ptrs, p, max_span, ws_avail);
        if (rl != LH_OK) return rl;
    }
    int r = lh_check_launch(op);
    if (r != LH_OK) return r;
    batch->dispatch_count++;
    if (rot && p.num_splits > 1 && p.num_splits <= 2 * kReduceBatch) {
        hipLaunchKernelGGL(attention_tq_reduce_rotate_kernel, dim3(p.num_queries * p.num_q_heads), dim3(p.head_dim), 0, ctx->stream,
                           (const float*)ws, (const float*)rot->signs->ptr, (uint16_t*)rot->out16->ptr, p.head_dim, p.num_splits,
                           1.0f / std::sqrt((float)p.head_dim));
        r = lh_check_launch(op);
        if (r == LH_OK) batch->dispatch_count++;
        if (rot->rotated) *rot->rotated = 1;
        return r;
    }
    if (p.num_splits > 1) {
        const dim3 rgrid(p.num_queries * p.num_q_heads, (p.head_dim + kReduceDims - 1) / kReduceDims);
        const uint32_t num_qh = p.num_queries * p.num_q_heads;
        if (p.num_splits <= kWaveMergeMaxSplits && p.head_dim % 4 == 0 && num_qh >= 64 && (((uintptr_t)out->ptr | (uintptr_t)ws) & 15) == 0)
            hipLaunchKernelGGL(attention_tq_reduce_wave_kernel, dim3((num_qh + 3) / 4), dim3(256), 0, ctx->stream, (const float*)ws,
                               (float*)out->ptr, p.head_dim, p.num_splits, num_qh);
        else if (p.num_splits <= 2 * kReduceBatch)
            hipLaunchKernelGGL(attention_tq_reduce_kernel<2>, rgrid, dim3(kReduceDims * 2), 0, ctx->stream, (const float*)ws,
                               (float*)out->ptr, p.head_dim, p.num_splits);
        else
            hipLaunchKernelGGL(attention_tq_reduce_kernel<16>, rgrid, dim3(kReduceDims * 16), 0, ctx->stream, (const float*)ws,
                               (float*)out->ptr, p.head_dim, p.num_splits);
        r = lh_check_launch(op);
        if (r == LH_OK) batch->dispatch_count++;
    }
    if (rot && rot->rotated) { *rot->rotated = 0; return r; }
    if (rot && r == LH_OK) {
        r = lh_launch_hadamard_fh(ctx, (const float*)out->ptr, (const float*)rot->signs->ptr, (uint16_t*)rot->out16->ptr, p.head_dim,
                                  p.num_queries * p.num_q_heads);
        if (r == LH_OK) batch->dispatch_count++;
    }
    return r;
}

}  // namespace

// Called by lh_context_create with `device` current: resolves this device's copy of the static scratch array once.
int lh_attention_static_scratch_init(int device) {
    if (device < 0 || device >= kMaxDevices) return LH_OK;            // such a device simply has no static entry
    if (g_scratch_ptr[device].load(std::memory_order_acquire)) return LH_OK;
    float* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    // Only the entry that allocates nothing needs the array: when its address cannot be resolved the pointer stays null, that
    // entry reports "no static scratch", and contexts open all the same.
    if (e != hipSuccess || !ptr) { (void)hipGetLastError(); return LH_OK; }
    g_scratch_ptr[device].store(ptr, std::memory_order_release);
    return LH_OK;
}

extern "C" {

int lh_flash_attention_tq_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                               const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                               uint32_t head_dim, uint32_t kv_len, uint32_t current_pos, uint32_t num_q_heads, uint32_t num_kv_heads,
                               uint32_t window, uint32_t bits, uint32_t ring_capacity) {
    AttnParams p{};
    p.head_dim = head_dim; p.bits = bits; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads; p.kv_len = kv_len;
    p.pos0 = current_pos; p.window = window; p.ring_capacity = ring_capacity; p.mode = kSingle; p.num_queries = 1;
    const uint64_t seq = std::min<uint64_t>(kv_len, (uint64_t)current_pos + 1);
    const uint64_t lo = (window > 0 && (uint64_t)current_pos + 1 > window) ? (uint64_t)current_pos + 1 - window : 0;
    const uint64_t span = seq > lo ? seq - lo : 0;
    const uint64_t phys = (ring_capacity ? std::min<uint64_t>(ring_capacity, seq) : seq) * num_kv_heads;
    return attention_dispatch(batch, "flash_attention_tq", rq, k_codes, k_norms, v_codes, v_norms, levels, out, nullptr, p, span, phys);
}

int lh_flash_attention_tq_static_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                      const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                                      uint32_t head_dim, uint32_t kv_len, uint32_t current_pos, uint32_t num_q_heads, uint32_t num_kv_heads,
                                      uint32_t window, uint32_t bits, uint32_t ring_capacity) {
    const char* op = "flash_attention_tq_static";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    const int dev = batch->ctx->device;
    float* ws = (dev >= 0 && dev < kMaxDevices) ? g_scratch_ptr[dev].load(std::memory_order_acquire) : nullptr;
    if (!ws) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: no static scratch on device %d (the context was not created by this library)", op, dev);
    // kStaticMinSplits records of every query head must fit: beyond that the call is refused rather than run with few splits
    const uint64_t need = (uint64_t)num_q_heads * partial_record_floats(head_dim) * kStaticMinSplits;
    if (head_dim <= 512 && need > kStaticScratchFloats)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: num_q_heads %u x (head_dim %u + 4) exceeds %zu, the most the static scratch (%zu bytes) holds",
                       op, num_q_heads, head_dim, kStaticScratchFloats / kStaticMinSplits, kStaticScratchFloats * sizeof(float));
    AttnParams p{};
    p.head_dim = head_dim; p.bits = bits; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads; p.kv_len = kv_len;
    p.pos0 = current_pos; p.window = window; p.ring_capacity = ring_capacity; p.mode = kSingle; p.num_queries = 1;
    const uint64_t seq = std::min<uint64_t>(kv_len, (uint64_t)current_pos + 1);
    const uint64_t lo = (window > 0 && (uint64_t)current_pos + 1 > window) ? (uint64_t)current_pos + 1 - window : 0;
    const uint64_t span = seq > lo ? seq - lo : 0;
    const uint64_t phys = (ring_capacity ? std::min<uint64_t>(ring_capacity, seq) : seq) * num_kv_heads;
    return attention_dispatch(batch, op, rq, k_codes, k_norms, v_codes, v_norms, levels, out, nullptr, p, span, phys, nullptr, ws,
                              kStaticScratchFloats);
}

int lh_flash_attention_tq_rotated_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                       const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, const lh_buffer* signs,
                                       lh_buffer* out, lh_buffer* out_f16, uint32_t head_dim, uint32_t kv_len, uint32_t current_pos,
                                       uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t window, uint32_t bits, uint32_t ring_capacity) {
    AttnParams p{};
    p.head_dim = head_dim; p.bits = bits; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads; p.kv_len = kv_len;
    p.pos0 = current_pos; p.window = window; p.ring_capacity = ring_capacity; p.mode = kSingle; p.num_queries = 1;
    const uint64_t seq = std::min<uint64_t>(kv_len, (uint64_t)current_pos + 1);
    const uint64_t lo = (window > 0 && (uint64_t)current_pos + 1 > window) ? (uint64_t)current_pos + 1 - window : 0;
    const uint64_t span = seq > lo ? seq - lo : 0;
    const uint64_t phys = (ring_capacity ? std::min<uint64_t>(ring_capacity, seq) : seq) * num_kv_heads;
    const RotateBack rot{signs, out_f16};
    return attention_dispatch(batch, "flash_attention_tq_rotated", rq, k_codes, k_norms, v_codes, v_norms, levels, out, nullptr, p, span, phys, &rot);
}

int lh_flash_attention_tq_rotated_lazy_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                            const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, const lh_buffer* signs,
                                            lh_buffer* out, lh_buffer* out_f16, uint32_t head_dim, uint32_t kv_len, uint32_t current_pos,
                                            uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t window, uint32_t bits, uint32_t ring_capacity,
                                            int* rotated) {
    if (!rotated) return lh_fail(LH_ERR_INVALID_ARGUMENT, "flash_attention_tq_rotated_lazy: rotated is null");
    *rotated = 0;
    AttnParams p{};
    p.head_dim = head_dim; p.bits = bits; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads; p.kv_len = kv_len;
    p.pos0 = current_pos; p.window = window; p.ring_capacity = ring_capacity; p.mode = kSingle; p.num_queries = 1;
    const uint64_t seq = std::min<uint64_t>(kv_len, (uint64_t)current_pos + 1);
    const uint64_t lo = (window > 0 && (uint64_t)current_pos + 1 > window) ? (uint64_t)current_pos + 1 - window : 0;
    const uint64_t span = seq > lo ? seq - lo : 0;
    const uint64_t phys = (ring_capacity ? std::min<uint64_t>(ring_capacity, seq) : seq) * num_kv_heads;
    RotateBack rot{signs, out_f16};
    rot.rotated = rotated;
    return attention_dispatch(batch, "flash_attention_tq_rotated_lazy", rq, k_codes, k_norms, v_codes, v_norms, levels, out, nullptr, p, span, phys, &rot);
}

static int prefill_common(const char* op, lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                          const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                          uint32_t head_dim, uint32_t kv_len, uint32_t start_pos, uint32_t n_rows, uint32_t num_q_heads,
                          uint32_t num_kv_heads, uint32_t window, uint32_t bits, uint32_t ring_capacity) {
    AttnParams p{};
    p.head_dim = head_dim; p.bits = bits; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads; p.kv_len = kv_len;
    p.pos0 = start_pos; p.window = window; p.ring_capacity = ring_capacity; p.mode = kPrefill; p.num_queries = n_rows;
    const uint64_t seq = std::min<uint64_t>(kv_len, (uint64_t)start_pos + n_rows);
    const uint64_t span = window ? std::min<uint64_t>(window, seq) : seq;
    const uint64_t phys = (ring_capacity ? std::min<uint64_t>(ring_capacity, seq) : seq) * num_kv_heads;
    return attention_dispatch(batch, op, rq, k_codes, k_norms, v_codes, v_norms, levels, out, nullptr, p, span, phys);
}

int lh_flash_attention_tq_prefill_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                       const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                                       uint32_t head_dim, uint32_t kv_len, uint32_t start_pos, uint32_t n_rows, uint32_t num_q_heads,
                                       uint32_t num_kv_heads, uint32_t window, uint32_t bits, uint32_t ring_capacity) {
    return prefill_common("flash_attention_tq_prefill", batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, head_dim, kv_len,
                          start_pos, n_rows, num_q_heads, num_kv_heads, window, bits, ring_capacity);
}

int lh_flash_attention_tq_prefill_tiled_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                             const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels,
                                             lh_buffer* out, uint32_t head_dim, uint32_t kv_len, uint32_t start_pos, uint32_t n_rows,
                                             uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t window, uint32_t bits,
                                             uint32_t ring_capacity) {
    return prefill_common("flash_attention_tq_prefill_tiled", batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, head_dim,
                          kv_len, start_pos, n_rows, num_q_heads, num_kv_heads, window, bits, ring_capacity);
}

static int batched_common(const char* op, lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                          const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                          const lh_buffer* positions, uint32_t head_dim, uint32_t lane_capacity, uint32_t num_q_heads,
                          uint32_t num_kv_heads, uint32_t window, uint32_t bits, uint32_t n_lanes, uint32_t ring_capacity,
                          const RotateBack* rot) {
    AttnParams p{};
    p.head_dim = head_dim; p.bits = bits; p.num_q_heads = num_q_heads; p.num_kv_heads = num_kv_heads;
    p.window = window; p.ring_capacity = ring_capacity; p.lane_capacity = lane_capacity; p.mode = kBatched; p.num_queries = n_lanes;
    if (ring_capacity > lane_capacity)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: ring_capacity %u exceeds lane_capacity %u", op, ring_capacity, lane_capacity);
    // positions are device data: size the split count for the largest possible span
    const uint64_t cap = ring_capacity ? ring_capacity : lane_capacity;
    const uint64_t span = window ? std::min<uint64_t>(window, cap) : cap;
    const uint64_t phys = (uint64_t)n_lanes * lane_capacity * num_kv_heads;
    return attention_dispatch(batch, op, rq, k_codes, k_norms, v_codes, v_norms, levels, out, positions, p, span, phys, rot);
}

int lh_flash_attention_tq_batched_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                       const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels, lh_buffer* out,
                                       const lh_buffer* positions, uint32_t head_dim, uint32_t lane_capacity, uint32_t num_q_heads,
                                       uint32_t num_kv_heads, uint32_t window, uint32_t bits, uint32_t n_lanes, uint32_t ring_capacity) {
    return batched_common("flash_attention_tq_batched", batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, positions, head_dim,
                          lane_capacity, num_q_heads, num_kv_heads, window, bits, n_lanes, ring_capacity, nullptr);
}

int lh_flash_attention_tq_batched_rotated_into(lh_batch* batch, const lh_buffer* rq, const lh_buffer* k_codes, const lh_buffer* k_norms,
                                               const lh_buffer* v_codes, const lh_buffer* v_norms, const lh_buffer* levels,
                                               const lh_buffer* signs, lh_buffer* out, lh_buffer* out_f16, const lh_buffer* positions,
                                               uint32_t head_dim, uint32_t lane_capacity, uint32_t num_q_heads, uint32_t num_kv_heads,
                                               uint32_t window, uint32_t bits, uint32_t n_lanes, uint32_t ring_capacity) {
    const RotateBack rot{signs, out_f16};
    return batched_common("flash_attention_tq_batched_rotated", batch, rq, k_codes, k_norms, v_codes, v_norms, levels, out, positions,
                          head_dim, lane_capacity, num_q_heads, num_kv_heads, window, bits, n_lanes, ring_capacity, &rot);
}

}  // extern "C"
