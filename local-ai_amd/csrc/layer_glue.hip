// Decoder-layer glue kernels around the matvec / attention hot path: RMSNorm (+ residual), per-head QK norm
// (+ RoPE), NEOX RoPE with proportional partial rotary, GeGLU elementwise, residual add, in-place scale,
// strided f16 gather, final-logit soft cap.  Stand in for shaders/rms_norm.metal:4-88, qk_norm.metal:6-140,
// rope.metal:14-61, gelu.metal:23-41, residual_add.metal:5-15, scale_in_place.metal:5-52 and their dispatchers
// in local-metal/src/kernels.rs.  At decode these touch a few KB per call: they are latency bound, one small
// workgroup per row / head, f32 math, f16 storage with the same rounding points as the reference kernels.
#include "common.hpp"
#include "xquant.hpp"
#include <cstdlib>

namespace {

__device__ __forceinline__ float h_at(const uint16_t* p, size_t i) { return lh_h2f(p[i]); }

// Sum over a workgroup of up to 256 threads (4 waves).
__device__ __forceinline__ float block_sum(float v, float* scratch) {
    v = lh_group_sum(v, 64);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
    if (lane == 0) scratch[wave] = v;
    __syncthreads();
    float t = 0.0f;
    for (int w = 0; w < nwaves; w++) t += scratch[w];
    __syncthreads();
    return t;
}

// rms_norm.metal:4-46 / 48-88: out[r, i] = in[r, i] * rsqrt(mean(in[r]^2) + eps) * w[i] (+ residual[r, i]).
// VEC = 8: 16-byte accesses (dim a multiple of 8, 16-byte aligned rows); VEC = 1 otherwise.
// ADD with `tail` != 0 is the three-kernel tail of the single-token layer in one dispatch (layer.rs:507-520: rms_norm,
// residual_add, scale_in_place): the normalised value is rounded to f16, added to the residual as an f16 addition, and,
// with tail == 2, scaled and rounded once more -- the roundings of the three separate kernels.
__device__ __forceinline__ float norm_tail(float normed, float res, uint32_t tail, float scale) { return lh_norm_tail(normed, res, tail, scale); }

// The arithmetic of one 8-element chunk, shared by every kernel that must reproduce the stand-alone norm bit for bit.
__device__ __forceinline__ void rms_sumsq8(const uint4& v, float& s) {
    const uint32_t wv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; j++) { const float a = lh_h2f((uint16_t)(wv[j] & 0xFFFF)), b = lh_h2f((uint16_t)(wv[j] >> 16)); s += a * a; s += b * b; }
}
template <bool ADD>
__device__ __forceinline__ uint4 rms_apply8(const uint4& v, const uint4& g, const uint4& r, float rms, uint32_t tail, float scale) {
    const uint32_t wv[4] = {v.x, v.y, v.z, v.w}, wg[4] = {g.x, g.y, g.z, g.w}, wr[4] = {r.x, r.y, r.z, r.w};
    uint32_t wo[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float lo = lh_norm_product(lh_h2f((uint16_t)(wv[j] & 0xFFFF)), rms, lh_h2f((uint16_t)(wg[j] & 0xFFFF)));
        float hi = lh_norm_product(lh_h2f((uint16_t)(wv[j] >> 16)), rms, lh_h2f((uint16_t)(wg[j] >> 16)));
        if (ADD) {
            const float rlo = lh_h2f((uint16_t)(wr[j] & 0xFFFF)), rhi = lh_h2f((uint16_t)(wr[j] >> 16));
            if (tail) { lo = norm_tail(lo, rlo, tail, scale); hi = norm_tail(hi, rhi, tail, scale); }
            else { lo += rlo; hi += rhi; }
        }
        wo[j] = (uint32_t)lh_f2h_exact(lo) | ((uint32_t)lh_f2h_exact(hi) << 16);
    }
    return make_uint4(wo[0], wo[1], wo[2], wo[3]);
}

template <bool ADD, int VEC>
__global__ __launch_bounds__(256) void rms_norm_kernel(const uint16_t* in, const uint16_t* __restrict__ w, const uint16_t* res, uint16_t* out,   // out may be in or res
                                                      uint32_t dim, float eps, uint32_t tail = 0, float scale = 1.0f) {
    __shared__ float scratch[4];
    const size_t row = (size_t)blockIdx.x * dim;
    float s = 0.0f;
    if constexpr (VEC == 8) {
        for (uint32_t i = threadIdx.x * 8; i < dim; i += blockDim.x * 8) {
            const uint4 v = *reinterpret_cast<const uint4*>(in + row + i);
            rms_sumsq8(v, s);
        }
    } else {
        for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) { const float v = h_at(in, row + i); s += v * v; }
    }
    const float rms = rsqrtf(block_sum(s, scratch) / (float)dim + eps);
    if constexpr (VEC == 8) {
        for (uint32_t i = threadIdx.x * 8; i < dim; i += blockDim.x * 8) {
            const uint4 v = *reinterpret_cast<const uint4*>(in + row + i), g = *reinterpret_cast<const uint4*>(w + i);
            uint4 r = v;
            if (ADD) r = *reinterpret_cast<const uint4*>(res + row + i);
            *reinterpret_cast<uint4*>(out + row + i) = rms_apply8<ADD>(v, g, r, rms, tail, scale);
        }
    } else {
        for (uint32_t i = threadIdx.x; i < dim; i += blockDim.x) {
            float v = lh_norm_product(h_at(in, row + i), rms, h_at(w, i));
            if (ADD) v = tail ? norm_tail(v, h_at(res, row + i), tail, scale) : v + h_at(res, row + i);
            out[row + i] = lh_f2h_exact(v);
        }
    }
}

template <bool ADD>
void launch_rms_norm(hipStream_t stream, const void* in, const void* w, const void* res, void* out, uint32_t dim, uint32_t rows, float eps,
                     uint32_t tail = 0, float scale = 1.0f) {
    const bool vec = (dim & 7) == 0 && (((uintptr_t)in | (uintptr_t)w | (uintptr_t)(res ? res : in) | (uintptr_t)out) & 15) == 0;
    const uint32_t threads = vec ? (dim >= 2048 ? 256u : (dim >= 1024 ? 128u : 64u)) : (dim >= 256 ? 256u : (dim > 64 ? 128u : 64u));
    if (vec) hipLaunchKernelGGL((rms_norm_kernel<ADD, 8>), dim3(rows), dim3(threads), 0, stream, (const uint16_t*)in, (const uint16_t*)w, (const uint16_t*)res, (uint16_t*)out, dim, eps, tail, scale);
    else hipLaunchKernelGGL((rms_norm_kernel<ADD, 1>), dim3(rows), dim3(threads), 0, stream, (const uint16_t*)in, (const uint16_t*)w, (const uint16_t*)res, (uint16_t*)out, dim, eps, tail, scale);
}

// rms_norm_kernel<ADD, 8> with its input taken either from f16 rows or from the f32 partial tiles of a k-split product
// (summed in split order and rounded to f16, which is what the product's own reduction would have stored), optionally
// followed by the output scale (scale_in_place.metal:5-14) and by a second plain norm of the row just produced
// (layer.rs:640-652: post-attention norm + residual, then the feed-forward norm): up to four dispatches of a decode
// batch's layer in one.  Same thread count, accumulation order and rounding points as the separate kernels, so the
// results are theirs bit for bit.  A thread keeps its (up to four) 8-element chunks in registers between the passes.
template <bool PART, bool ADD>
__global__ __launch_bounds__(256) void rms_norm_fused_kernel(const LhNormFused a) {
    __shared__ float scratch[4];
    const uint32_t dim = a.dim, rowi = blockIdx.x;
    const size_t row = (size_t)rowi * dim;
    uint4 x[4], o[4];
    // The norm weights, the residual and the second norm's weights are requested here, with the row itself: read where they
    // are used, each waits for memory again behind the barrier of the pass before.
    uint4 gw[4], rr[4], gw2[4];
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const uint32_t i = (threadIdx.x + it * blockDim.x) * 8;
        gw[it] = rr[it] = gw2[it] = make_uint4(0u, 0u, 0u, 0u);
        if (i >= dim) break;
        gw[it] = *reinterpret_cast<const uint4*>(a.w + i);
        if (ADD) rr[it] = *reinterpret_cast<const uint4*>(a.res + row + i);
        if (a.w2 != nullptr) gw2[it] = *reinterpret_cast<const uint4*>(a.w2 + i);
    }
    float s = 0.0f;
    if constexpr (PART) {
        // the splits of two chunks, eight at a time, are all requested before the first is added (in split order)
        const size_t zstride = (size_t)a.part_rows * a.part_cols;
#pragma unroll
        for (int it0 = 0; it0 < 4; it0 += 2) {
            float v[2][8];
#pragma unroll
            for (int c = 0; c < 2; c++)
#pragma unroll
                for (int e = 0; e < 8; e++) v[c][e] = 0.0f;
            const uint32_t i0 = (threadIdx.x + it0 * blockDim.x) * 8, i1 = (threadIdx.x + (it0 + 1) * blockDim.x) * 8;
            if (i0 >= dim) break;
            const bool two = i1 < dim;
            const float* p0 = a.partial + (size_t)rowi * a.part_cols + i0;
            const float* p1 = a.partial + (size_t)rowi * a.part_cols + (two ? i1 : i0);
            for (uint32_t z0 = 0; z0 < a.splits; z0 += 8) {
                float4 lo[2][8], hi[2][8];
#pragma unroll
                for (uint32_t u = 0; u < 8; u++) {
                    const size_t zo = (size_t)(z0 + u < a.splits ? z0 + u : a.splits - 1) * zstride;
                    lo[0][u] = *reinterpret_cast<const float4*>(p0 + zo); hi[0][u] = *reinterpret_cast<const float4*>(p0 + zo + 4);
                    lo[1][u] = *reinterpret_cast<const float4*>(p1 + zo); hi[1][u] = *reinterpret_cast<const float4*>(p1 + zo + 4);
                }
#pragma unroll
                for (uint32_t u = 0; u < 8; u++) {
                    if (z0 + u >= a.splits) break;
#pragma unroll
                    for (int c = 0; c < 2; c++) {
                        v[c][0] += lo[c][u].x; v[c][1] += lo[c][u].y; v[c][2] += lo[c][u].z; v[c][3] += lo[c][u].w;
                        v[c][4] += hi[c][u].x; v[c][5] += hi[c][u].y; v[c][6] += hi[c][u].z; v[c][7] += hi[c][u].w;
                    }
                }
            }
#pragma unroll
            for (int c = 0; c < 2; c++)
                x[it0 + c] = make_uint4((uint32_t)lh_f2h(v[c][0]) | ((uint32_t)lh_f2h(v[c][1]) << 16), (uint32_t)lh_f2h(v[c][2]) | ((uint32_t)lh_f2h(v[c][3]) << 16),
                                        (uint32_t)lh_f2h(v[c][4]) | ((uint32_t)lh_f2h(v[c][5]) << 16), (uint32_t)lh_f2h(v[c][6]) | ((uint32_t)lh_f2h(v[c][7]) << 16));
        }
    }
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const uint32_t i = (threadIdx.x + it * blockDim.x) * 8;
        if (i >= dim) break;
        if constexpr (!PART) x[it] = *reinterpret_cast<const uint4*>(a.in + row + i);
        rms_sumsq8(x[it], s);
    }
    const float rms = rsqrtf(block_sum(s, scratch) / (float)dim + a.eps);
    float s2 = 0.0f;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const uint32_t i = (threadIdx.x + it * blockDim.x) * 8;
        if (i >= dim) break;
        const uint4 g = gw[it];
        uint4 r = x[it];
        if (ADD) r = rr[it];
        uint4 w = rms_apply8<ADD>(x[it], g, r, rms, a.tail, 1.0f);
        if (a.apply_scale) {
            uint32_t ws[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
            for (int j = 0; j < 4; j++)
                ws[j] = (uint32_t)lh_f2h(lh_h2f((uint16_t)(ws[j] & 0xFFFF)) * a.scale) | ((uint32_t)lh_f2h(lh_h2f((uint16_t)(ws[j] >> 16)) * a.scale) << 16);
            w = make_uint4(ws[0], ws[1], ws[2], ws[3]);
        }
        o[it] = w;
        rms_sumsq8(w, s2);
        *reinterpret_cast<uint4*>(a.out + row + i) = w;
    }
    if (a.w2 == nullptr) return;
    const float rms2 = rsqrtf(block_sum(s2, scratch) / (float)dim + a.eps);
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const uint32_t i = (threadIdx.x + it * blockDim.x) * 8;
        if (i >= dim) break;
        *reinterpret_cast<uint4*>(a.out2 + row + i) = rms_apply8<false>(o[it], gw2[it], o[it], rms2, a.tail, 1.0f);
    }
}

// qk_norm.metal:6-56 (in place; head h of `qk`), and 70-140 with the NEOX rotation fused: the normalised values are
// rounded to f16 before they are rotated, exactly as when qk_norm and rope run as two kernels.
template <bool ROPE>
__global__ __launch_bounds__(256) void qk_norm_kernel(const uint16_t* in, uint16_t* out, const uint16_t* __restrict__ w,   // in may be out
                                                     uint32_t head_dim, float eps, uint32_t position, float theta, float prf) {
    __shared__ float scratch[4];
    __shared__ uint16_t normed[512];
    const size_t base = (size_t)blockIdx.x * head_dim;
    float s = 0.0f;
    for (uint32_t j = threadIdx.x; j < head_dim; j += blockDim.x) { const float v = h_at(in, base + j); s += v * v; }
    const float rms = rsqrtf(block_sum(s, scratch) / (float)head_dim + eps);
    if (!ROPE) {
        for (uint32_t j = threadIdx.x; j < head_dim; j += blockDim.x) out[base + j] = lh_f2h_exact(lh_norm_product(h_at(in, base + j), rms, h_at(w, j)));
        return;
    }
    for (uint32_t j = threadIdx.x; j < head_dim; j += blockDim.x) normed[j] = lh_f2h_exact(lh_norm_product(h_at(in, base + j), rms, h_at(w, j)));
    __syncthreads();
    const uint32_t half_dim = head_dim / 2;
    const uint32_t rope_angles = (uint32_t)((float)head_dim * prf) / 2;
    for (uint32_t i = threadIdx.x; i < half_dim; i += blockDim.x) {
        const float x0 = lh_h2f(normed[i]), x1 = lh_h2f(normed[i + half_dim]);
        if (i >= rope_angles) {
            out[base + i] = lh_f2h(x0);
            out[base + i + half_dim] = lh_f2h(x1);
        } else {
            uint16_t o0, o1;
            lh_rotate_pair(x0, x1, i, head_dim, position, theta, o0, o1);
            out[base + i] = o0;
            out[base + i + half_dim] = o1;
        }
    }
}

// rope.metal:14-61: NEOX pairing (i, i + head_dim / 2); only the first prf * head_dim / 2 pairs rotate, with the
// frequencies of the full head.
__global__ __launch_bounds__(256) void rope_kernel(const uint16_t* in, uint16_t* out, uint32_t head_dim, uint32_t position,   // in may be out
                                                  float theta, float prf, uint32_t num_heads) {
    const uint32_t half_dim = head_dim / 2;
    const uint32_t t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= half_dim * num_heads) return;
    const uint32_t head = t / half_dim, i = t - head * half_dim;
    const size_t idx0 = (size_t)head * head_dim + i, idx1 = idx0 + half_dim;
    const uint32_t rope_angles = (uint32_t)((float)head_dim * prf) / 2;
    if (i >= rope_angles) { out[idx0] = in[idx0]; out[idx1] = in[idx1]; return; }
    const float x0 = h_at(in, idx0), x1 = h_at(in, idx1);
    uint16_t o0, o1;
    lh_rotate_pair(x0, x1, i, head_dim, position, theta, o0, o1);
    out[idx0] = o0;
    out[idx1] = o1;
}

// rope.metal:105-200 rope_batch / rope_batch_decode: in place over qk [seq_len, num_heads, head_dim]; row r sits at
// position start_pos + r, or at positions[r] when a table is given (independent sequences of a batched decode).
__global__ __launch_bounds__(256) void rope_batch_kernel(uint16_t* qk, const uint32_t* __restrict__ positions, uint32_t start_pos, float theta, uint32_t head_dim,
                                                        uint32_t num_heads, uint32_t seq_len, float prf) {
    const uint32_t half_dim = head_dim / 2;
    const uint32_t rope_angles = (uint32_t)((float)head_dim * prf) / 2;
    const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (rope_angles == 0 || t >= (uint64_t)rope_angles * num_heads * seq_len) return;
    const uint32_t i = (uint32_t)(t % rope_angles);
    const uint32_t flat = (uint32_t)(t / rope_angles);          // (row, head), head fastest: rows of qk are contiguous
    const uint32_t seq_idx = flat / num_heads, head = flat - seq_idx * num_heads;
    const uint32_t position = positions ? positions[seq_idx] : start_pos + seq_idx;
    const size_t idx0 = ((size_t)seq_idx * num_heads + head) * head_dim + i, idx1 = idx0 + half_dim;
    uint16_t o0, o1;
    lh_rotate_pair(h_at(qk, idx0), h_at(qk, idx1), i, head_dim, position, theta, o0, o1);
    qk[idx0] = o0;
    qk[idx1] = o1;
}

// Elementwise f16 kernels: a thread takes 8 consecutive elements with 16-byte accesses; the launcher sends a
// count that is not a multiple of 8, or pointers that are not 16-byte aligned, to the one-element form (VEC = 1).

enum { kGeluMul = 0, kResidualAdd = 1, kScale = 2 };

// gelu.metal:23-41 (out = gelu(a) * b), residual_add.metal:5-15 (an f16 addition: one rounding of the exact sum),
// scale_in_place.metal:5-14 (out = half(float(a) * scalar), a may be out)
template <int OP>
__device__ __forceinline__ uint16_t elementwise_one(uint16_t a, uint16_t b, float scalar) {
    if constexpr (OP == kGeluMul) return lh_gelu_mul_h(a, b);
    else if constexpr (OP == kResidualAdd) return __builtin_bit_cast(uint16_t, (_Float16)(__builtin_bit_cast(_Float16, a) + __builtin_bit_cast(_Float16, b)));
    else return lh_f2h(lh_h2f(a) * scalar);
}

template <int OP, int VEC>
__global__ __launch_bounds__(256) void elementwise_kernel(const uint16_t* a, const uint16_t* b, uint16_t* out, float scalar, uint32_t count) {
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
    if (i >= count) return;
    if constexpr (VEC == 8) {
        const uint4 va = *reinterpret_cast<const uint4*>(a + i);
        uint4 vb = va;
        if constexpr (OP != kScale) vb = *reinterpret_cast<const uint4*>(b + i);
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
        uint32_t wo[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            wo[j] = (uint32_t)elementwise_one<OP>((uint16_t)(wa[j] & 0xFFFF), (uint16_t)(wb[j] & 0xFFFF), scalar) |
                    ((uint32_t)elementwise_one<OP>((uint16_t)(wa[j] >> 16), (uint16_t)(wb[j] >> 16), scalar) << 16);
        *reinterpret_cast<uint4*>(out + i) = make_uint4(wo[0], wo[1], wo[2], wo[3]);
    } else {
        out[i] = elementwise_one<OP>(a[i], OP != kScale ? b[i] : a[i], scalar);
    }
}

// gelu_mul whose second operand is read through gather_strided_f16's addressing (row r of `b` starts at
// r * b_row_stride + b_off): out[r, i] = half(gelu(a[r, i]) * b[r * b_row_stride + b_off + i]) -- the slice gather and the
// gate of the per-layer input (layer.rs:690-700) in one dispatch, without the gathered copy.
// With `part` the first operand is the sum of a product's k-split partial tiles (split z of row r at
// part.partial[(z * rows + r) * part.cols]), added in split order and rounded to f16 as the product's own reduction would.
struct GeluPartials { const float* partial; uint32_t splits, cols; };
template <int VEC>
__global__ __launch_bounds__(256) void gelu_mul_strided_kernel(const uint16_t* a, const uint16_t* __restrict__ b, uint16_t* out, uint32_t dim,
                                                              uint32_t rows, uint32_t b_row_stride, uint32_t b_off, GeluPartials part) {
    const uint32_t per_row = dim / VEC, idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per_row * rows) return;
    const uint32_t r = idx / per_row, i = (idx - r * per_row) * VEC;
    const size_t ia = (size_t)r * dim + i, ib = (size_t)r * b_row_stride + b_off + i;
    if constexpr (VEC == 8) {
        uint4 va;
        if (part.partial) {
            float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            const size_t zstride = (size_t)rows * part.cols;
            const float* p0 = part.partial + (size_t)r * part.cols + i;
            for (uint32_t z0 = 0; z0 < part.splits; z0 += 8) {
                float4 lo[8], hi[8];
#pragma unroll
                for (uint32_t u = 0; u < 8; u++) {
                    const size_t zo = (size_t)(z0 + u < part.splits ? z0 + u : part.splits - 1) * zstride;
                    lo[u] = *reinterpret_cast<const float4*>(p0 + zo); hi[u] = *reinterpret_cast<const float4*>(p0 + zo + 4);
                }
#pragma unroll
                for (uint32_t u = 0; u < 8; u++) {
                    if (z0 + u >= part.splits) break;
                    v[0] += lo[u].x; v[1] += lo[u].y; v[2] += lo[u].z; v[3] += lo[u].w; v[4] += hi[u].x; v[5] += hi[u].y; v[6] += hi[u].z; v[7] += hi[u].w;
                }
            }
            va = make_uint4((uint32_t)lh_f2h(v[0]) | ((uint32_t)lh_f2h(v[1]) << 16), (uint32_t)lh_f2h(v[2]) | ((uint32_t)lh_f2h(v[3]) << 16),
                            (uint32_t)lh_f2h(v[4]) | ((uint32_t)lh_f2h(v[5]) << 16), (uint32_t)lh_f2h(v[6]) | ((uint32_t)lh_f2h(v[7]) << 16));
        } else {
            va = *reinterpret_cast<const uint4*>(a + ia);
        }
        const uint4 vb = *reinterpret_cast<const uint4*>(b + ib);
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
        uint32_t wo[4];
#pragma unroll
        for (int j = 0; j < 4; j++)
            wo[j] = (uint32_t)elementwise_one<kGeluMul>((uint16_t)(wa[j] & 0xFFFF), (uint16_t)(wb[j] & 0xFFFF), 0.0f) |
                    ((uint32_t)elementwise_one<kGeluMul>((uint16_t)(wa[j] >> 16), (uint16_t)(wb[j] >> 16), 0.0f) << 16);
        *reinterpret_cast<uint4*>(out + ia) = make_uint4(wo[0], wo[1], wo[2], wo[3]);
    } else {
        out[ia] = elementwise_one<kGeluMul>(a[ia], b[ib], 0.0f);
    }
}

template <int OP>
void launch_elementwise(hipStream_t stream, const void* a, const void* b, void* out, float scalar, uint32_t count) {
    const bool vec = (count & 7) == 0 && (((uintptr_t)a | (uintptr_t)(b ? b : a) | (uintptr_t)out) & 15) == 0;
    if (vec) hipLaunchKernelGGL((elementwise_kernel<OP, 8>), dim3((count / 8 + 255) / 256), dim3(256), 0, stream, (const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, scalar, count);
    else hipLaunchKernelGGL((elementwise_kernel<OP, 1>), dim3((count + 255) / 256), dim3(256), 0, stream, (const uint16_t*)a, (const uint16_t*)b, (uint16_t*)out, scalar, count);
}

// scale_in_place.metal:21-35: dst[i * pld + p] = src[i * row_stride + base_off + p]
__global__ __launch_bounds__(256) void gather_strided_f16_kernel(const uint16_t* __restrict__ src, uint16_t* __restrict__ dst, uint32_t row_stride, uint32_t base_off,
                                                                uint32_t pld, uint32_t n_rows) {
    const uint32_t g = blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_rows * pld) return;
    const uint32_t i = g / pld, p = g - i * pld;
    dst[g] = src[(size_t)i * row_stride + base_off + p];
}

// scale_in_place.metal:39-49
__global__ __launch_bounds__(256) void logit_softcap_kernel(float* __restrict__ data, float cap, uint32_t count) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) data[i] = cap * tanhf(data[i] / cap);
}

inline uint32_t blocks_for(uint64_t n) { return (uint32_t)((n + 255) / 256); }
inline uint32_t norm_threads(uint32_t dim) { return dim >= 256 ? 256u : (dim > 64 ? 128u : 64u); }

int finish(lh_batch* batch, const char* op) {
    const int r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

}  // namespace

bool lh_norm_fused_supported(uint32_t dim) { return (dim & 7) == 0 && dim <= 8192; }

void lh_launch_gelu_mul(hipStream_t stream, const void* a, const void* b, void* out, uint32_t count) {
    launch_elementwise<kGeluMul>(stream, a, b, out, 0.0f, count);
}

void lh_launch_gelu_mul_strided(hipStream_t stream, const void* a, const float* partial, uint32_t splits, uint32_t part_cols, const void* b,
                                uint32_t b_row_stride, uint32_t b_off, void* out, uint32_t dim, uint32_t rows) {
    const uint32_t items = rows * (dim / 8);
    hipLaunchKernelGGL(gelu_mul_strided_kernel<8>, dim3((items + 255) / 256), dim3(256), 0, stream, (const uint16_t*)a, (const uint16_t*)b,
                       (uint16_t*)out, dim, rows, b_row_stride, b_off, GeluPartials{partial, splits, part_cols});
}

void lh_launch_norm_fused(hipStream_t stream, const LhNormFused& a) {
    // the thread count launch_rms_norm picks for 16-byte accesses: the partial sums of the squares add up in the same order
    const uint32_t threads = a.dim >= 2048 ? 256u : (a.dim >= 1024 ? 128u : 64u);
    const bool part = a.partial != nullptr, add = a.res != nullptr;
    if (part) {
        if (add) hipLaunchKernelGGL((rms_norm_fused_kernel<true, true>), dim3(a.rows), dim3(threads), 0, stream, a);
        else hipLaunchKernelGGL((rms_norm_fused_kernel<true, false>), dim3(a.rows), dim3(threads), 0, stream, a);
    } else {
        if (add) hipLaunchKernelGGL((rms_norm_fused_kernel<false, true>), dim3(a.rows), dim3(threads), 0, stream, a);
        else hipLaunchKernelGGL((rms_norm_fused_kernel<false, false>), dim3(a.rows), dim3(threads), 0, stream, a);
    }
}

extern "C" {

int lh_rms_norm_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight, lh_buffer* output, uint32_t dim, uint32_t rows, float eps) {
    const char* op = "rms_norm";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (dim == 0 || rows == 0) return LH_OK;
    LH_NEED(input, (size_t)rows * dim * 2, op, "input");
    LH_NEED(weight, (size_t)dim * 2, op, "weight");
    LH_NEED(output, (size_t)rows * dim * 2, op, "output");
    launch_rms_norm<false>(batch->ctx->stream, input->ptr, weight->ptr, nullptr, output->ptr, dim, rows, eps);
    return finish(batch, op);
}

int lh_rms_norm_add_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight, const lh_buffer* residual, lh_buffer* output,
                         uint32_t dim, uint32_t rows, float eps) {
    const char* op = "rms_norm_add";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (dim == 0 || rows == 0) return LH_OK;
    LH_NEED(input, (size_t)rows * dim * 2, op, "input");
    LH_NEED(weight, (size_t)dim * 2, op, "weight");
    LH_NEED(residual, (size_t)rows * dim * 2, op, "residual");
    LH_NEED(output, (size_t)rows * dim * 2, op, "output");
    launch_rms_norm<true>(batch->ctx->stream, input->ptr, weight->ptr, residual->ptr, output->ptr, dim, rows, eps);
    return finish(batch, op);
}

int lh_rms_norm_residual_scale_into(lh_batch* batch, const lh_buffer* input, const lh_buffer* weight, const lh_buffer* residual,
                                    lh_buffer* output, uint32_t dim, uint32_t rows, float eps, int apply_scale, float scale) {
    const char* op = "rms_norm_residual_scale";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (dim == 0 || rows == 0) return LH_OK;
    LH_NEED(input, (size_t)rows * dim * 2, op, "input");
    LH_NEED(weight, (size_t)dim * 2, op, "weight");
    LH_NEED(residual, (size_t)rows * dim * 2, op, "residual");
    LH_NEED(output, (size_t)rows * dim * 2, op, "output");
    launch_rms_norm<true>(batch->ctx->stream, input->ptr, weight->ptr, residual->ptr, output->ptr, dim, rows, eps, apply_scale ? 2u : 1u, scale);
    return finish(batch, op);
}

int lh_qk_norm_offset_into(lh_batch* batch, lh_buffer* qk_data, const lh_buffer* weight, size_t weight_offset, uint32_t head_dim,
                           uint32_t num_heads, float eps) {
    const char* op = "qk_norm";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (head_dim == 0 || num_heads == 0) return LH_OK;
    LH_REQUIRE((weight_offset & 1) == 0, "%s: weight offset %zu is not 2-byte aligned", op, weight_offset);
    LH_NEED(qk_data, (size_t)num_heads * head_dim * 2, op, "qk_data");
    LH_NEED(weight, weight_offset + (size_t)head_dim * 2, op, "weight");
    const uint16_t* w = (const uint16_t*)((const uint8_t*)weight->ptr + weight_offset);
    hipLaunchKernelGGL(qk_norm_kernel<false>, dim3(num_heads), dim3(norm_threads(head_dim)), 0, batch->ctx->stream, (const uint16_t*)qk_data->ptr,
                       (uint16_t*)qk_data->ptr, w, head_dim, eps, 0u, 0.0f, 0.0f);
    return finish(batch, op);
}

int lh_qk_norm_gpu_into(lh_batch* batch, lh_buffer* qk_data, const lh_buffer* weight, uint32_t head_dim, uint32_t num_heads, float eps) {
    return lh_qk_norm_offset_into(batch, qk_data, weight, 0, head_dim, num_heads, eps);
}

int lh_qk_norm_rope_available(uint32_t head_dim) {
    static const bool disabled = [] { const char* e = getenv("LOCAL_AI_NO_FUSE_QKROPE"); return e && e[0] == '1' && e[1] == 0; }();
    return (!disabled && head_dim <= 512) ? 1 : 0;
}

int lh_qk_norm_rope_into(lh_batch* batch, const lh_buffer* input, lh_buffer* output, const lh_buffer* weight, uint32_t head_dim,
                         uint32_t num_heads, float eps, uint32_t position, float theta, float partial_rotary_factor) {
    const char* op = "qk_norm_rope";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (head_dim == 0 || num_heads == 0) return LH_OK;
    LH_REQUIRE(head_dim <= 512 && (head_dim & 1) == 0, "%s: head_dim %u must be even and at most 512", op, head_dim);
    LH_NEED(input, (size_t)num_heads * head_dim * 2, op, "input");
    LH_NEED(output, (size_t)num_heads * head_dim * 2, op, "output");
    LH_NEED(weight, (size_t)head_dim * 2, op, "weight");
    hipLaunchKernelGGL(qk_norm_kernel<true>, dim3(num_heads), dim3(norm_threads(head_dim)), 0, batch->ctx->stream, (const uint16_t*)input->ptr,
                       (uint16_t*)output->ptr, (const uint16_t*)weight->ptr, head_dim, eps, position, theta, partial_rotary_factor);
    return finish(batch, op);
}

int lh_rope_into(lh_batch* batch, const lh_buffer* input, lh_buffer* output, uint32_t head_dim, uint32_t position, float theta,
                 float partial_rotary_factor, uint32_t num_heads) {
    const char* op = "rope";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (head_dim == 0 || num_heads == 0) return LH_OK;
    LH_REQUIRE((head_dim & 1) == 0, "%s: head_dim %u must be even", op, head_dim);
    LH_NEED(input, (size_t)num_heads * head_dim * 2, op, "input");
    LH_NEED(output, (size_t)num_heads * head_dim * 2, op, "output");
    hipLaunchKernelGGL(rope_kernel, dim3(blocks_for((uint64_t)num_heads * head_dim / 2)), dim3(256), 0, batch->ctx->stream, (const uint16_t*)input->ptr,
                       (uint16_t*)output->ptr, head_dim, position, theta, partial_rotary_factor, num_heads);
    return finish(batch, op);
}

static int rope_batch_common(const char* op, lh_batch* batch, lh_buffer* qk, const lh_buffer* positions, uint32_t start_pos, float theta, uint32_t head_dim,
                             uint32_t num_heads, uint32_t seq_len, float partial_rotary_factor) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (head_dim == 0 || num_heads == 0 || seq_len == 0) return LH_OK;
    LH_REQUIRE((head_dim & 1) == 0, "%s: head_dim %u must be even", op, head_dim);
    LH_NEED(qk, (size_t)seq_len * num_heads * head_dim * 2, op, "qk");
    if (positions) LH_NEED(positions, (size_t)seq_len * 4, op, "positions");
    const uint32_t rope_angles = (uint32_t)((float)head_dim * partial_rotary_factor) / 2;
    if (rope_angles == 0) return LH_OK;
    hipLaunchKernelGGL(rope_batch_kernel, dim3(blocks_for((uint64_t)rope_angles * num_heads * seq_len)), dim3(256), 0, batch->ctx->stream, (uint16_t*)qk->ptr,
                       positions ? (const uint32_t*)positions->ptr : nullptr, start_pos, theta, head_dim, num_heads, seq_len, partial_rotary_factor);
    return finish(batch, op);
}

int lh_rope_batch_into(lh_batch* batch, lh_buffer* qk, uint32_t start_pos, float theta, uint32_t head_dim, uint32_t num_heads, uint32_t seq_len,
                       float partial_rotary_factor) {
    return rope_batch_common("rope_batch", batch, qk, nullptr, start_pos, theta, head_dim, num_heads, seq_len, partial_rotary_factor);
}

int lh_rope_batch_decode_into(lh_batch* batch, lh_buffer* qk, const lh_buffer* positions, float theta, uint32_t head_dim, uint32_t num_heads,
                              uint32_t seq_len, float partial_rotary_factor) {
    if (!positions) return lh_fail(LH_ERR_INVALID_ARGUMENT, "rope_batch_decode: positions is null");
    return rope_batch_common("rope_batch_decode", batch, qk, positions, 0, theta, head_dim, num_heads, seq_len, partial_rotary_factor);
}

int lh_gelu_mul_into(lh_batch* batch, const lh_buffer* a, const lh_buffer* b, lh_buffer* out, uint32_t count) {
    const char* op = "gelu_mul";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (count == 0) return LH_OK;
    LH_NEED(a, (size_t)count * 2, op, "a");
    LH_NEED(b, (size_t)count * 2, op, "b");
    LH_NEED(out, (size_t)count * 2, op, "out");
    launch_elementwise<kGeluMul>(batch->ctx->stream, a->ptr, b->ptr, out->ptr, 0.0f, count);
    return finish(batch, op);
}

int lh_gelu_mul_strided_into(lh_batch* batch, const lh_buffer* a, const lh_buffer* b, uint32_t b_row_stride, uint32_t b_offset, lh_buffer* out,
                             uint32_t dim, uint32_t rows) {
    const char* op = "gelu_mul_strided";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (dim == 0 || rows == 0) return LH_OK;
    LH_NEED(a, (size_t)rows * dim * 2, op, "a");
    LH_NEED(b, ((size_t)(rows - 1) * b_row_stride + b_offset + dim) * 2, op, "b");
    LH_NEED(out, (size_t)rows * dim * 2, op, "out");
    const bool vec = ((dim | b_row_stride | b_offset) & 7) == 0 && (((uintptr_t)a->ptr | (uintptr_t)b->ptr | (uintptr_t)out->ptr) & 15) == 0;
    const uint32_t items = rows * (dim / (vec ? 8 : 1));
    if (vec) hipLaunchKernelGGL(gelu_mul_strided_kernel<8>, dim3((items + 255) / 256), dim3(256), 0, batch->ctx->stream, (const uint16_t*)a->ptr,
                                (const uint16_t*)b->ptr, (uint16_t*)out->ptr, dim, rows, b_row_stride, b_offset, GeluPartials{nullptr, 0, 0});
    else hipLaunchKernelGGL(gelu_mul_strided_kernel<1>, dim3((items + 255) / 256), dim3(256), 0, batch->ctx->stream, (const uint16_t*)a->ptr,
                            (const uint16_t*)b->ptr, (uint16_t*)out->ptr, dim, rows, b_row_stride, b_offset, GeluPartials{nullptr, 0, 0});
    return finish(batch, op);
}

int lh_residual_add_into(lh_batch* batch, const lh_buffer* a, const lh_buffer* b, lh_buffer* output, uint32_t count) {
    const char* op = "residual_add";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (count == 0) return LH_OK;
    LH_NEED(a, (size_t)count * 2, op, "a");
    LH_NEED(b, (size_t)count * 2, op, "b");
    LH_NEED(output, (size_t)count * 2, op, "output");
    launch_elementwise<kResidualAdd>(batch->ctx->stream, a->ptr, b->ptr, output->ptr, 0.0f, count);
    return finish(batch, op);
}

int lh_scale_in_place_gpu_into(lh_batch* batch, lh_buffer* data, float scalar, uint32_t count) {
    const char* op = "scale_in_place";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (count == 0) return LH_OK;
    LH_NEED(data, (size_t)count * 2, op, "data");
    launch_elementwise<kScale>(batch->ctx->stream, data->ptr, nullptr, data->ptr, scalar, count);
    return finish(batch, op);
}

int lh_gather_strided_f16_into(lh_batch* batch, const lh_buffer* src, lh_buffer* dst, uint32_t row_stride, uint32_t base_off, uint32_t pld,
                               uint32_t n_rows) {
    const char* op = "gather_strided_f16";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (pld == 0 || n_rows == 0) return LH_OK;
    LH_REQUIRE((uint64_t)n_rows * pld <= 0xFFFFFFFFull, "%s: %u rows x %u elements do not fit 32 bits", op, n_rows, pld);
    LH_NEED(src, ((size_t)(n_rows - 1) * row_stride + base_off + pld) * 2, op, "src");
    LH_NEED(dst, (size_t)n_rows * pld * 2, op, "dst");
    hipLaunchKernelGGL(gather_strided_f16_kernel, dim3(blocks_for((uint64_t)n_rows * pld)), dim3(256), 0, batch->ctx->stream, (const uint16_t*)src->ptr,
                       (uint16_t*)dst->ptr, row_stride, base_off, pld, n_rows);
    return finish(batch, op);
}

int lh_logit_softcap_gpu_into(lh_batch* batch, lh_buffer* data, float cap, uint32_t count) {
    const char* op = "logit_softcap";
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (count == 0) return LH_OK;
    LH_NEED(data, (size_t)count * 4, op, "data");
    hipLaunchKernelGGL(logit_softcap_kernel, dim3(blocks_for(count)), dim3(256), 0, batch->ctx->stream, (float*)data->ptr, cap, count);
    return finish(batch, op);
}

}  // extern "C"
