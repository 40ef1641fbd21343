// Block dequant of GGUF Q4_0 / TQ2_0 payloads to f16 on the GPU, bit for bit what the
// reference's CPU path produces (local-engine/src/qat_recover.rs:23-97), plus the
// legacy 2-bit unpack of shaders/tq2_dequant.metal:4-16.
//
// The arithmetic is (f32(q) - zp) * d in f32 (exact: at most 4 integer bits times an
// 11-bit significand) followed by one round-to-nearest-even narrowing to f16, as
// f16::from_f32 does.  Compiled with -ffp-contract=off.
#include "common.hpp"

namespace {

__global__ __launch_bounds__(256) void dequant_q4_0_kernel(const uint8_t* __restrict__ data, uint16_t* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint8_t* bp = data + (i >> 5) * 18;
    const float d = lh_h2f((uint16_t)(bp[0] | (bp[1] << 8)));
    const uint32_t j = (uint32_t)i & 31u;
    const uint32_t q = bp[2 + (j & 15u)];
    const uint32_t nib = j < 16u ? (q & 0x0Fu) : (q >> 4);
    out[i] = lh_f2h_exact(__fmul_rn(__fsub_rn((float)nib, 8.0f), d));     // qat_recover.rs:84-93
}

__global__ __launch_bounds__(256) void dequant_tq2_0_kernel(const uint8_t* __restrict__ data, uint16_t* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint8_t* bp = data + (i >> 8) * 66;
    const float d = lh_h2f((uint16_t)(bp[64] | (bp[65] << 8)));
    const uint32_t r = (uint32_t)i & 255u;
    const uint32_t q = (bp[(r >> 7) * 32 + (r & 31u)] >> (2 * ((r >> 5) & 3u))) & 3u;   // qat_recover.rs:39-47
    out[i] = lh_f2h_exact(__fmul_rn(d, __fsub_rn((float)q, 1.0f)));
}

__global__ __launch_bounds__(256) void tq2_dequant_legacy_kernel(const uint8_t* __restrict__ packed, const uint16_t* __restrict__ scales,
                                                                uint16_t* __restrict__ out, uint32_t n) {
    const uint32_t tid = threadIdx.x;
    if (tid >= n) return;
    const uint32_t idx = tid / 4u, rem = tid % 4u;
    const uint32_t val = (packed[idx] >> (rem * 2u)) & 3u;
    out[tid] = lh_f2h_exact(__fmul_rn(lh_h2f(scales[idx]), (float)val));
}

int dequant_dispatch(lh_batch* batch, lh_quant fmt, const lh_buffer* data, size_t byte_offset, lh_buffer* output, size_t num_elements) {
    const char* op = fmt == LH_Q4_0 ? "dequant_q4_0" : "dequant_tq2_0";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (!data || !output) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null buffer", op);
    if (byte_offset > data->len) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: offset %zu beyond %zu bytes", op, byte_offset, data->len);
    const size_t elems = fmt == LH_Q4_0 ? 32 : 256, bytes = fmt == LH_Q4_0 ? 18 : 66;
    const size_t blocks = (data->len - byte_offset) / bytes;
    const size_t n = num_elements < blocks * elems ? num_elements : blocks * elems;   // output stops at the last whole block
    if (n == 0) return LH_OK;
    LH_NEED(output, n * 2, op, "output");
    const uint8_t* src = (const uint8_t*)data->ptr + byte_offset;
    const dim3 grid((unsigned)((n + 255) / 256));
    if (fmt == LH_Q4_0) hipLaunchKernelGGL(dequant_q4_0_kernel, grid, dim3(256), 0, batch->ctx->stream, src, (uint16_t*)output->ptr, n);
    else hipLaunchKernelGGL(dequant_tq2_0_kernel, grid, dim3(256), 0, batch->ctx->stream, src, (uint16_t*)output->ptr, n);
    int r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

}  // namespace

extern "C" {

int lh_dequant_q4_0_into(lh_batch* batch, const lh_buffer* data, size_t byte_offset, lh_buffer* output, size_t num_elements) {
    return dequant_dispatch(batch, LH_Q4_0, data, byte_offset, output, num_elements);
}
int lh_dequant_tq2_0_into(lh_batch* batch, const lh_buffer* data, size_t byte_offset, lh_buffer* output, size_t num_elements) {
    return dequant_dispatch(batch, LH_TQ2_0, data, byte_offset, output, num_elements);
}

int lh_tq2_dequant(lh_context* ctx, const lh_buffer* packed, const lh_buffer* scales, lh_buffer* output, uint32_t num_elements) {
    // kernels.rs:6785-6797 launches ONE threadgroup of at most 256 threads, so only the
    // first min(num_elements, 256) outputs are produced; kept as is (the entry has no caller).
    const char* op = "tq2_dequant";
    if (!ctx) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: context is null", op);
    const uint32_t n = num_elements < 256 ? num_elements : 256;
    if (n == 0) return LH_OK;
    LH_NEED(packed, (n + 3) / 4, op, "packed");
    LH_NEED(scales, (size_t)((n + 3) / 4) * 2, op, "scales");
    LH_NEED(output, (size_t)n * 2, op, "output");
    hipLaunchKernelGGL(tq2_dequant_legacy_kernel, dim3(1), dim3(256), 0, ctx->stream, (const uint8_t*)packed->ptr,
                       (const uint16_t*)scales->ptr, (uint16_t*)output->ptr, n);
    int r = lh_check_launch(op);
    if (r != LH_OK) return r;
    return lh_context_synchronize(ctx);
}

}  // extern "C"
