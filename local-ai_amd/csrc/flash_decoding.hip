// FP16-KV split-K decode attention and the log-sum-exp reduce.
//
// Stands in for shaders/flash_decoding.metal:10-189 (flash_decoding_split / _reduce),
// the windowed split kernel of shaders/attention_flash.metal:398 and their dispatch in
// local-metal/src/kernels.rs:1265-1557.  Softmax scale is 1.0 (no 1/sqrt(d)), as in the
// reference.  Partials: partial_max / partial_sum [q_head * num_splits + split],
// partial_acc [(q_head * num_splits + split) * head_dim + d], unnormalised.
#include "common.hpp"
#include <algorithm>

namespace {

constexpr int kThreads = 256, kWaves = 4, kMaxDpl = 8;

__global__ __launch_bounds__(kThreads) void fd_split_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ k,
                                                           const uint16_t* __restrict__ v, float* __restrict__ pmax,
                                                           float* __restrict__ psum, float* __restrict__ pacc, uint32_t hd,
                                                           uint32_t kv_len, uint32_t current_pos, uint32_t nq, uint32_t nkv,
                                                           uint32_t window, uint32_t num_splits) {
    __shared__ float lds_m[kWaves], lds_l[kWaves];
    __shared__ float lds_acc[kWaves][512];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t qh = blockIdx.x / num_splits, split = blockIdx.x % num_splits;
    const uint32_t kvh = qh / (nq / nkv);
    const uint32_t seq = std::min(kv_len, current_pos + 1u);
    const uint32_t win = (window > 0u && current_pos + 1u > window) ? current_pos + 1u - window : 0u;
    const uint32_t range = seq > win ? seq - win : 0u;
    const uint32_t chunk = (range + num_splits - 1) / num_splits;
    const uint32_t c_lo = win + std::min(range, split * chunk), c_hi = win + std::min(range, (split + 1) * chunk);
    const uint32_t dpl = hd >= 64 ? hd / 64 : 1;
    const bool on = hd >= 64 || (uint32_t)lane < hd;
    const uint32_t d0 = lane * dpl;
    float qr[kMaxDpl], acc[kMaxDpl];
#pragma unroll
    for (int i = 0; i < kMaxDpl; i++) { acc[i] = 0.0f; qr[i] = ((uint32_t)i < dpl && on) ? lh_h2f(q[(size_t)qh * hd + d0 + i]) : 0.0f; }
    float m = -INFINITY, l = 0.0f;
    for (uint32_t t = c_lo + wave; t < c_hi; t += kWaves) {
        const size_t base = ((size_t)t * nkv + kvh) * hd + d0;
        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < kMaxDpl; i++) if ((uint32_t)i < dpl && on) dot += qr[i] * lh_h2f(k[base + i]);
        dot = lh_group_sum(dot, 64);
        const float nm = fmaxf(m, dot), r = __expf(m - nm), w = __expf(dot - nm);
        l = l * r + w; m = nm;
#pragma unroll
        for (int i = 0; i < kMaxDpl; i++) if ((uint32_t)i < dpl && on) acc[i] = acc[i] * r + w * lh_h2f(v[base + i]);
    }
    if (lane == 0) { lds_m[wave] = m; lds_l[wave] = l; }
#pragma unroll
    for (int i = 0; i < kMaxDpl; i++) if ((uint32_t)i < dpl && on) lds_acc[wave][d0 + i] = acc[i];
    __syncthreads();
    float gm = -INFINITY;
#pragma unroll
    for (int w = 0; w < kWaves; w++) gm = fmaxf(gm, lds_m[w]);
    float f[kWaves], gl = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; w++) { f[w] = lds_m[w] == -INFINITY ? 0.0f : __expf(lds_m[w] - gm); gl += f[w] * lds_l[w]; }
    const size_t pidx = (size_t)qh * num_splits + split;
    if (threadIdx.x == 0) { pmax[pidx] = gm; psum[pidx] = gl; }       // empty split: (-inf, 0, zeros)
    for (uint32_t d = threadIdx.x; d < hd; d += kThreads) {
        float o = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; w++) o += f[w] * lds_acc[w][d];
        pacc[pidx * hd + d] = o;
    }
}

// flash_decoding.metal:148-189
__global__ __launch_bounds__(256) void fd_reduce_kernel(const float* __restrict__ pmax, const float* __restrict__ psum,
                                                       const float* __restrict__ pacc, uint16_t* __restrict__ out, uint32_t hd,
                                                       uint32_t num_splits) {
    const uint32_t qh = blockIdx.x;
    float gm = -INFINITY;
    for (uint32_t s = 0; s < num_splits; s++) gm = fmaxf(gm, pmax[(size_t)qh * num_splits + s]);
    float gs = 0.0f;
    for (uint32_t s = 0; s < num_splits; s++) {
        const float m = pmax[(size_t)qh * num_splits + s];
        gs += psum[(size_t)qh * num_splits + s] * (m == -INFINITY ? 0.0f : __expf(m - gm));
    }
    const float inv = gs > 0.0f ? 1.0f / gs : 0.0f;
    for (uint32_t d = threadIdx.x; d < hd; d += blockDim.x) {
        float val = 0.0f;
        for (uint32_t s = 0; s < num_splits; s++) {
            const float m = pmax[(size_t)qh * num_splits + s];
            val += pacc[((size_t)qh * num_splits + s) * hd + d] * (m == -INFINITY ? 0.0f : __expf(m - gm));
        }
        out[(size_t)qh * hd + d] = lh_f2h(val * inv);
    }
}

int fd_launch(lh_batch* batch, const char* op, const lh_buffer* q, const lh_buffer* k, const lh_buffer* v, lh_buffer* output,
              float* pmax, float* psum, float* pacc, uint32_t hd, uint32_t kv_len, uint32_t current_pos, uint32_t nq, uint32_t nkv,
              uint32_t window, uint32_t num_splits) {
    if (hd == 0 || (hd & (hd - 1)) || hd > 512) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: head_dim %u must be a power of two <= 512", op, hd);
    if (nkv == 0 || nq % nkv != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: num_q_heads %u is not a multiple of num_kv_heads %u", op, nq, nkv);
    if (nq == 0) return LH_OK;
    const uint64_t seq = std::min<uint64_t>(kv_len, (uint64_t)current_pos + 1);
    LH_NEED(q, (size_t)nq * hd * 2, op, "q");
    LH_NEED(k, (size_t)seq * nkv * hd * 2, op, "k");
    LH_NEED(v, (size_t)seq * nkv * hd * 2, op, "v");
    LH_NEED(output, (size_t)nq * hd * 2, op, "output");
    hipLaunchKernelGGL(fd_split_kernel, dim3(nq * num_splits), dim3(kThreads), 0, batch->ctx->stream, (const uint16_t*)q->ptr,
                       (const uint16_t*)k->ptr, (const uint16_t*)v->ptr, pmax, psum, pacc, hd, kv_len, current_pos, nq, nkv, window,
                       num_splits);
    int r = lh_check_launch(op);
    if (r != LH_OK) return r;
    batch->dispatch_count++;
    hipLaunchKernelGGL(fd_reduce_kernel, dim3(nq), dim3(256), 0, batch->ctx->stream, pmax, psum, pacc, (uint16_t*)output->ptr, hd, num_splits);
    r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

}  // namespace

extern "C" {

uint32_t lh_flash_split_count(uint32_t eff_seq_len) {   // kernels.rs:1265-1278
    const uint32_t s = (eff_seq_len + 15u) / 16u;
    return s < 1u ? 1u : (s > 16u ? 16u : s);
}

int lh_flash_decoding_into(lh_batch* batch, const lh_buffer* q, const lh_buffer* k, const lh_buffer* v, lh_buffer* output,
                           uint32_t head_dim, uint32_t kv_len, uint32_t current_pos, uint32_t num_q_heads, uint32_t num_kv_heads) {
    const char* op = "flash_decoding";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    const uint32_t seq = std::min(kv_len, current_pos + 1u);
    uint32_t splits = std::max(1u, (seq + 255u) / 256u);            // kernels.rs:1437: one split per 256 positions
    lh_context* ctx = batch->ctx;
    // partials live in the lower half of the context workspace (the reference allocates them per call)
    const size_t avail = ctx->workspace_bytes / 2 / 4;
    while (splits > 1 && (size_t)num_q_heads * splits * (head_dim + 2) > avail) splits = (splits + 1) / 2;
    float* pmax = (float*)ctx->workspace;
    float* psum = pmax + (size_t)num_q_heads * splits;
    float* pacc = psum + (size_t)num_q_heads * splits;
    return fd_launch(batch, op, q, k, v, output, pmax, psum, pacc, head_dim, kv_len, current_pos, num_q_heads, num_kv_heads, 0, splits);
}

int lh_flash_attention_windowed_split_into(lh_batch* batch, const lh_buffer* q, const lh_buffer* k, const lh_buffer* v,
                                           lh_buffer* output, lh_buffer* partial_max, lh_buffer* partial_sum, lh_buffer* partial_acc,
                                           uint32_t head_dim, uint32_t kv_len, uint32_t current_pos, uint32_t num_q_heads,
                                           uint32_t num_kv_heads, uint32_t window, uint32_t num_splits) {
    const char* op = "flash_attention_windowed_split";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (num_splits == 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: num_splits is 0", op);
    LH_NEED(partial_max, (size_t)num_q_heads * num_splits * 4, op, "partial_max");
    LH_NEED(partial_sum, (size_t)num_q_heads * num_splits * 4, op, "partial_sum");
    LH_NEED(partial_acc, (size_t)num_q_heads * num_splits * head_dim * 4, op, "partial_acc");
    return fd_launch(batch, op, q, k, v, output, (float*)partial_max->ptr, (float*)partial_sum->ptr, (float*)partial_acc->ptr,
                     head_dim, kv_len, current_pos, num_q_heads, num_kv_heads, window, num_splits);
}

}  // extern "C"
