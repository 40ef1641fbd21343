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

// Rows picked by a device-resident index list out of a packed [table_rows, cols] table, decoded to f16 into a dense
// [n_rows, cols] matrix: the embedding gather of a prefill chunk or of a step over many lanes
// (local-engine/src/pipeline.rs:781-832 decodes the rows on the CPU, one call per token).  An index past the end reads the
// last row (init_gemma4_qat.rs:152).  With scale != 1 each value is multiplied and rounded once more, which is what
// scale_in_place.metal:5-14 would do to the decoded row.
template <int FMT>
__global__ __launch_bounds__(256) void dequant_rows_kernel(const uint8_t* __restrict__ table, const uint32_t* __restrict__ rows, uint16_t* __restrict__ out,
                                                          uint32_t table_rows, uint32_t cols, size_t row_bytes, float scale) {
    const uint32_t c = blockIdx.x * 256 + threadIdx.x;
    if (c >= cols) return;
    uint32_t row = rows[blockIdx.y];
    if (row >= table_rows) row = table_rows - 1;
    const uint8_t* rp = table + (size_t)row * row_bytes;
    uint16_t h;
    if constexpr (FMT == LH_Q4_0) {
        const uint8_t* bp = rp + (c >> 5) * 18;
        const float d = lh_h2f((uint16_t)(bp[0] | (bp[1] << 8)));
        const uint32_t j = c & 31u, q = bp[2 + (j & 15u)];
        const uint32_t nib = j < 16u ? (q & 0x0Fu) : (q >> 4);
        h = lh_f2h_exact(__fmul_rn(__fsub_rn((float)nib, 8.0f), d));
    } else if constexpr (FMT == LH_TQ2_0) {
        const uint8_t* bp = rp + (c >> 8) * 66;
        const float d = lh_h2f((uint16_t)(bp[64] | (bp[65] << 8)));
        const uint32_t r = c & 255u;
        const uint32_t q = (bp[(r >> 7) * 32 + (r & 31u)] >> (2 * ((r >> 5) & 3u))) & 3u;
        h = lh_f2h_exact(__fmul_rn(d, __fsub_rn((float)q, 1.0f)));
    } else {
        h = reinterpret_cast<const uint16_t*>(rp)[c];
    }
    if (scale != 1.0f) h = lh_f2h(lh_h2f(h) * scale);
    out[(size_t)blockIdx.y * cols + c] = h;
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

int lh_dequant_rows_into(lh_batch* batch, int fmt, const lh_buffer* table, uint32_t table_rows, uint32_t cols, const lh_buffer* rows,
                         uint32_t n_rows, float scale, lh_buffer* output) {
    const char* op = "dequant_rows";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0 && fmt != LH_ROWS_F16) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: unknown weight format %d", op, fmt);
    if (n_rows == 0 || cols == 0) return LH_OK;
    if (table_rows == 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: the table has no rows", op);
    const uint32_t block = fmt == LH_Q4_0 ? 32u : fmt == LH_TQ2_0 ? 256u : 1u;
    if (cols % block != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: cols %u is not a multiple of the block size %u", op, cols, block);
    if (n_rows > 65535u) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: %u rows in one call (at most 65535)", op, n_rows);
    const size_t row_bytes = fmt == LH_Q4_0 ? (size_t)(cols / 32) * 18 : fmt == LH_TQ2_0 ? (size_t)(cols / 256) * 66 : (size_t)cols * 2;
    LH_NEED(table, (size_t)table_rows * row_bytes, op, "table");
    LH_NEED(rows, (size_t)n_rows * 4, op, "rows");
    LH_NEED(output, (size_t)n_rows * cols * 2, op, "output");
    const dim3 grid((cols + 255) / 256, n_rows);
    const uint8_t* t = (const uint8_t*)table->ptr;
    const uint32_t* idx = (const uint32_t*)rows->ptr;
    uint16_t* o = (uint16_t*)output->ptr;
    hipStream_t st = batch->ctx->stream;
    if (fmt == LH_Q4_0) hipLaunchKernelGGL(dequant_rows_kernel<LH_Q4_0>, grid, dim3(256), 0, st, t, idx, o, table_rows, cols, row_bytes, scale);
    else if (fmt == LH_TQ2_0) hipLaunchKernelGGL(dequant_rows_kernel<LH_TQ2_0>, grid, dim3(256), 0, st, t, idx, o, table_rows, cols, row_bytes, scale);
    else hipLaunchKernelGGL(dequant_rows_kernel<LH_ROWS_F16>, grid, dim3(256), 0, st, t, idx, o, table_rows, cols, row_bytes, scale);
    int r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
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
