// FP16-weight matvec family: y[rows] = W[rows, cols] . x[cols], f32 accumulation; x and y f16 or f32.
// Stands in for shaders/matvec_f16.metal:14-133 (matvec_f16, matvec_f16w_f32out, matvec_f16w_f32in) and their
// dispatchers (local-metal/src/kernels.rs:582, 1710-1930), the fallbacks of QuantWeight for tensors that are kept
// as F16 (local-engine/src/layer.rs:134, 158, 182).  Pure weight streaming: 2 bytes per multiply-add, HBM-bound.
// One wave per row at a time, 16 bytes per lane and load, the activation vector staged once per workgroup in LDS
// as f32; rows are dealt to the waves of the whole grid round robin so that the grid reads one advancing window.
#include "common.hpp"
#include <cstdlib>
#include <algorithm>

namespace {

// Weights are read once per launch: a streaming (non-temporal) 16-byte load.
__device__ __forceinline__ uint4 lh_ld16_stream(const uint16_t* p) {
    typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
    const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}


constexpr int kMaxLdsCols = 12288;   // 48 KB of f32 activations

template <typename XT> __device__ __forceinline__ float x_at(const XT* x, uint32_t i);
template <> __device__ __forceinline__ float x_at<uint16_t>(const uint16_t* x, uint32_t i) { return lh_h2f(x[i]); }
template <> __device__ __forceinline__ float x_at<float>(const float* x, uint32_t i) { return x[i]; }

// NL: 16-byte loads per lane and pass of the vector form (a pass covers 512 * NL columns).  FULL: cols is a multiple of
// that, so no lane ever stands past the end of a row (no address clamps, no per-lane conditions in the loop).
// XREG: the row is one pass long, so a lane multiplies the same 8 * NL activations in every row and keeps them in
// registers (read from LDS at a stride of 32 bytes between lanes they cost a four-way bank conflict per 16-byte read, and
// those reads, not the weight stream, then bound the kernel: 131072 x 2048 at 4.6 TB/s).
template <typename XT, typename YT, bool VEC, bool XLDS, int NL = 8, bool FULL = false, bool XREG = false>
__global__ __launch_bounds__(256) void matvec_f16_kernel(const uint16_t* __restrict__ W, const XT* __restrict__ x, YT* __restrict__ y, uint32_t rows,
                                                        uint32_t cols) {
    extern __shared__ float xs[];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    if (XLDS && !XREG) {
        for (uint32_t i = threadIdx.x; i < cols; i += blockDim.x) xs[i] = x_at<XT>(x, i);
        __syncthreads();
    }
    auto xv = [&](uint32_t i) { return XLDS ? xs[i] : x_at<XT>(x, i); };
    [[maybe_unused]] float xr[XREG ? NL : 1][8];
    if constexpr (XREG) {
#pragma unroll
        for (int c = 0; c < NL; c++)
#pragma unroll
            for (int j = 0; j < 8; j++) {
                const uint32_t k = lane * 8 + 512 * c + j;
                xr[c][j] = (FULL || k < cols) ? x_at<XT>(x, k) : 0.0f;
            }
    }
    if constexpr (VEC) {
        // cols a multiple of 8 and 16-byte aligned rows.  A wave walks its rows in passes of 512 * NL columns, NL loads of
        // 16 bytes per lane; the loads of the next pass (the next row, for rows of one pass) are issued before the arithmetic
        // of the current one, so that a wave always has a pass on its way.  Addresses past the row's end are clamped (a load
        // under a condition is followed by a wait for everything outstanding) and their values never used.
        constexpr uint32_t kPass = 512u * NL;
        const uint32_t ppr = (cols + kPass - 1) / kPass, row_step = gridDim.x * nwaves;
        uint32_t row = blockIdx.x * nwaves + wave, pass = 0;
        auto issue = [&](uint4 (&v)[NL], uint32_t r, uint32_t ps) {
            const uint16_t* wr = W + (size_t)r * cols;
#pragma unroll
            for (int c = 0; c < NL; c++) {
                const uint32_t k = lane * 8 + ps * kPass + 512 * c;
                v[c] = lh_ld16_stream(wr + (FULL || k < cols ? k : cols - 8));
            }
        };
        float acc = 0.0f;
        auto consume = [&](const uint4 (&v)[NL], uint32_t r, uint32_t ps) {
#pragma unroll
            for (int c = 0; c < NL; c++) {
                const uint32_t k = lane * 8 + ps * kPass + 512 * c;
                if (!FULL && k >= cols) break;
                const uint32_t wv[4] = {v[c].x, v[c].y, v[c].z, v[c].w};
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    acc = __builtin_fmaf(lh_h2f((uint16_t)(wv[j] & 0xFFFF)), XREG ? xr[XREG ? c : 0][2 * j] : xv(k + 2 * j), acc);
                    acc = __builtin_fmaf(lh_h2f((uint16_t)(wv[j] >> 16)), XREG ? xr[XREG ? c : 0][2 * j + 1] : xv(k + 2 * j + 1), acc);
                }
            }
            if (ps + 1 == ppr) {
                const float total = lh_group_sum(acc, 64);
                if (lane == 0) lh_store_from_f32<YT>(y, r, total);
                acc = 0.0f;
            }
        };
        auto step = [&](const uint4 (&cur)[NL], uint4 (&nxt)[NL]) {   // false: that was the wave's last pass
            uint32_t nrow = row, npass = pass + 1;
            if (npass == ppr) { npass = 0; nrow = row + row_step; }
            const bool more = nrow < rows;
            if (more) issue(nxt, nrow, npass);
            consume(cur, row, pass);
            row = nrow; pass = npass;
            return more;
        };
        uint4 a[NL], b[NL];
        if (row < rows) {
            issue(a, row, 0);
            while (step(a, b) && step(b, a)) {}
        }
    } else {
        for (uint32_t row = blockIdx.x * nwaves + wave; row < rows; row += gridDim.x * nwaves) {
            const uint16_t* wr = W + (size_t)row * cols;
            float acc = 0.0f;
            for (uint32_t k = lane; k < cols; k += 64) acc = __builtin_fmaf(lh_h2f(wr[k]), xv(k), acc);
            acc = lh_group_sum(acc, 64);
            if (lane == 0) lh_store_from_f32<YT>(y, row, acc);
        }
    }
}

template <typename XT, typename YT>
int launch(lh_context* ctx, const uint16_t* W, const void* x, void* y, uint32_t rows, uint32_t cols) {
    const bool vec = (cols & 7) == 0 && ((uintptr_t)W & 15) == 0;
    const bool xlds = cols <= (uint32_t)kMaxLdsCols;
    const uint32_t waves = 4;
    const uint64_t want = ((uint64_t)rows + waves - 1) / waves;
    // Rows of one pass (up to 4096 columns) run with the activations in registers and stream best from two workgroups per CU
    // (131072 x 2048: 6.83 TB/s against 6.67 from three to eight); the LDS form measures alike from 3 to 12.
    const uint32_t per_cu = (vec && cols <= 4096) ? 2u : 8u;
    const uint32_t grid = (uint32_t)std::min<uint64_t>(want, (uint64_t)ctx->cu_count * per_cu);
    const size_t lds = xlds ? (size_t)cols * 4 : 0;
#define LH_F16MV(V, L, N, F) hipLaunchKernelGGL((matvec_f16_kernel<XT, YT, V, L, N, F>), dim3(grid), dim3(64 * waves), lds, ctx->stream, W, (const XT*)x, (YT*)y, rows, cols)
#define LH_F16MV_R(N, F) hipLaunchKernelGGL((matvec_f16_kernel<XT, YT, true, true, N, F, true>), dim3(grid), dim3(64 * waves), 0, ctx->stream, W, (const XT*)x, (YT*)y, rows, cols)
#define LH_F16MV_N(L, N)                                                       \
    do {                                                                       \
        if (cols <= 512u * N) {   /* one pass per row: x in registers */ \
            if (cols % (512u * N) == 0) LH_F16MV_R(N, true);                   \
            else LH_F16MV_R(N, false);                                         \
        } else if (cols % (512u * N) == 0) LH_F16MV(true, L, N, true);         \
        else LH_F16MV(true, L, N, false);                                      \
    } while (0)
#define LH_F16MV_VEC(L)                                       \
    do {                                                      \
        if (cols <= 512) LH_F16MV_N(L, 1);                    \
        else if (cols <= 1024) LH_F16MV_N(L, 2);              \
        else if (cols <= 2048) LH_F16MV_N(L, 4);              \
        else LH_F16MV_N(L, 8);                                \
    } while (0)
    if (vec && xlds) LH_F16MV_VEC(true);
    else if (vec) LH_F16MV_VEC(false);
    else if (xlds) LH_F16MV(false, true, 8, false);
    else LH_F16MV(false, false, 8, false);
#undef LH_F16MV_N
#undef LH_F16MV_R
#undef LH_F16MV_VEC
#undef LH_F16MV
    return LH_OK;
}

int matvec_f16_dispatch(lh_context* ctx, lh_batch* batch, const char* op, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector,
                        lh_buffer* output, uint32_t rows, uint32_t cols, bool x_f32, bool y_f32) {
    if (!ctx) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: context is null", op);
    if (rows == 0 || cols == 0) return LH_OK;
    LH_REQUIRE((matrix_offset & 1) == 0, "%s: matrix offset %zu is not 2-byte aligned", op, matrix_offset);
    LH_NEED(matrix, matrix_offset + (size_t)rows * cols * 2, op, "matrix");
    LH_NEED(vector, (size_t)cols * (x_f32 ? 4 : 2), op, "vector");
    LH_NEED(output, (size_t)rows * (y_f32 ? 4 : 2), op, "output");
    const uint16_t* W = (const uint16_t*)((const uint8_t*)matrix->ptr + matrix_offset);
    if (!x_f32 && !y_f32) launch<uint16_t, uint16_t>(ctx, W, vector->ptr, output->ptr, rows, cols);
    else if (!x_f32) launch<uint16_t, float>(ctx, W, vector->ptr, output->ptr, rows, cols);
    else if (!y_f32) launch<float, uint16_t>(ctx, W, vector->ptr, output->ptr, rows, cols);
    else launch<float, float>(ctx, W, vector->ptr, output->ptr, rows, cols);
    const int r = lh_check_launch(op);
    if (r != LH_OK) return r;
    if (batch) { batch->dispatch_count++; return LH_OK; }
    lh_batch one_shot{ctx, 1};
    return lh_batch_commit_and_wait(&one_shot);
}

}  // namespace

extern "C" {

// kernels.rs:582-640 matvec (one-shot: enqueue and wait)
int lh_matvec(lh_context* ctx, const lh_buffer* matrix, const lh_buffer* vector, lh_buffer* output, uint32_t rows, uint32_t cols) {
    return matvec_f16_dispatch(ctx, nullptr, "matvec", matrix, 0, vector, output, rows, cols, false, false);
}
int lh_matvec_offset_into(lh_batch* batch, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector, lh_buffer* output, uint32_t rows,
                          uint32_t cols) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec: batch is null");
    return matvec_f16_dispatch(batch->ctx, batch, "matvec", matrix, matrix_offset, vector, output, rows, cols, false, false);
}
int lh_matvec_f32out_offset(lh_context* ctx, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector, lh_buffer* output, uint32_t rows,
                            uint32_t cols) {
    return matvec_f16_dispatch(ctx, nullptr, "matvec_f32out", matrix, matrix_offset, vector, output, rows, cols, false, true);
}
int lh_matvec_f32out_offset_into(lh_batch* batch, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector, lh_buffer* output,
                                 uint32_t rows, uint32_t cols) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_f32out: batch is null");
    return matvec_f16_dispatch(batch->ctx, batch, "matvec_f32out", matrix, matrix_offset, vector, output, rows, cols, false, true);
}
int lh_matvec_f32in_offset(lh_context* ctx, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector, lh_buffer* output, uint32_t rows,
                           uint32_t cols) {
    return matvec_f16_dispatch(ctx, nullptr, "matvec_f32in", matrix, matrix_offset, vector, output, rows, cols, true, false);
}
int lh_matvec_f32in_offset_into(lh_batch* batch, const lh_buffer* matrix, size_t matrix_offset, const lh_buffer* vector, lh_buffer* output,
                                uint32_t rows, uint32_t cols) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_f32in: batch is null");
    return matvec_f16_dispatch(batch->ctx, batch, "matvec_f32in", matrix, matrix_offset, vector, output, rows, cols, true, false);
}

}  // extern "C"
