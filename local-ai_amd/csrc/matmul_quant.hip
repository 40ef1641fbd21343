// Quantized-weight matmul C[M,N] = A[M,K] . W[N,K]^T for small batches and prefill.
//
// Stands in for shaders/matvec_quant.metal:394-1038 (matmul_nt_*, *_mma, *_smallm,
// *_batchm, multivec_nt_*), shaders/matmul_f16.metal:74-114 (matmul_f16_nt) and the
// routing in local-metal/src/kernels.rs:6049-6563, 5517-5568.
//
// Two kernels:
//  * multivec (M <= 16): one wave per weight row; the row is dequantised once in
//    registers (d*(q-zp) in f32, the reference GPU arithmetic) and reused for all M
//    activation rows, fp32 accumulate, wave butterfly per output.
//  * MFMA (M > 16): 128x128x32 tiles; the weight tile is dequantised to f16 -- for
//    Q4_0 that is exactly the reference's CPU dequant value f16((q-8)*d), for TQ2_0
//    d*(q-1) is exact in f16 -- and staged in LDS next to the activation tile
//    (converted to f16), then v_mfma_f32_16x16x32_f16 with fp32 accumulate.
#include "common.hpp"

namespace {

enum WeightKind { kQ4 = LH_Q4_0, kTQ2 = LH_TQ2_0, kF16W = 2 };

template <int DT> struct ElemT;
template <> struct ElemT<LH_F16> { using type = uint16_t; };
template <> struct ElemT<LH_F32> { using type = float; };
template <> struct ElemT<LH_BF16> { using type = uint16_t; };

template <int DT> __device__ __forceinline__ float load_elem(const void* p, size_t i) {
    if constexpr (DT == LH_F32) return static_cast<const float*>(p)[i];
    else if constexpr (DT == LH_F16) return lh_h2f(static_cast<const uint16_t*>(p)[i]);
    else return lh_bf2f(static_cast<const uint16_t*>(p)[i]);
}
template <int DT> __device__ __forceinline__ void store_elem(void* p, size_t i, float v) {
    if constexpr (DT == LH_F32) static_cast<float*>(p)[i] = v;
    else static_cast<uint16_t*>(p)[i] = lh_f2h(v);
}

// ---------------------------------------------------------------- multivec ----
constexpr int kMaxMultivecM = 16;

template <int FMT, int ADT, int CDT>
__global__ __launch_bounds__(256) void multivec_kernel(const void* __restrict__ A, const uint8_t* __restrict__ W, void* __restrict__ C,
                                                      uint32_t M, uint32_t K, uint32_t N) {
    const int lane = threadIdx.x & 63;
    const uint32_t n = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (n >= N) return;
    float acc[kMaxMultivecM];
#pragma unroll
    for (int m = 0; m < kMaxMultivecM; m++) acc[m] = 0.0f;
    if constexpr (FMT == kQ4) {
        const uint32_t nb = K >> 5;
        const uint8_t* rp = W + (size_t)n * nb * 18;
        for (uint32_t i = lane; i < nb * 16; i += 64) {
            const uint32_t b = i >> 4, j = i & 15;
            const uint8_t* bp = rp + (size_t)b * 18;
            const float d = lh_h2f((uint16_t)(bp[0] | (bp[1] << 8)));
            const uint32_t q = bp[2 + j];
            const float w0 = d * ((float)(q & 15) - 8.0f), w1 = d * ((float)(q >> 4) - 8.0f);
#pragma unroll
            for (int m = 0; m < kMaxMultivecM; m++)
                if ((uint32_t)m < M)
                    acc[m] += w0 * load_elem<ADT>(A, (size_t)m * K + b * 32 + j) + w1 * load_elem<ADT>(A, (size_t)m * K + b * 32 + 16 + j);
        }
    } else {
        const uint32_t nb = K >> 8;
        const uint8_t* rp = W + (size_t)n * nb * 66;
        for (uint32_t i = lane; i < nb * 64; i += 64) {
            const uint32_t b = i >> 6, j = i & 63;
            const uint8_t* bp = rp + (size_t)b * 66;
            const float d = lh_h2f((uint16_t)(bp[64] | (bp[65] << 8)));
            const uint32_t q = bp[j];
            const uint32_t e = b * 256 + (j >> 5) * 128 + (j & 31);
            float w[4];
#pragma unroll
            for (int l = 0; l < 4; l++) w[l] = d * ((float)((q >> (2 * l)) & 3) - 1.0f);
#pragma unroll
            for (int m = 0; m < kMaxMultivecM; m++)
                if ((uint32_t)m < M) {
#pragma unroll
                    for (int l = 0; l < 4; l++) acc[m] += w[l] * load_elem<ADT>(A, (size_t)m * K + e + l * 32);
                }
        }
    }
#pragma unroll
    for (int m = 0; m < kMaxMultivecM; m++) {
        if ((uint32_t)m < M) {
            const float t = lh_group_sum(acc[m], 64);
            if (lane == 0) store_elem<CDT>(C, (size_t)m * N + n, t);
        }
    }
}

// -------------------------------------------------------------------- MFMA ----
constexpr int BM = 128, BN = 128, BK = 32, LDK = BK + 8;   // LDS row stride in f16 (80 bytes)
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

struct Frag16 { uint32_t w[8]; };   // 16 f16 values

__device__ __forceinline__ uint32_t pack_h2(float a, float b) { return (uint32_t)lh_f2h(a) | ((uint32_t)lh_f2h(b) << 16); }

// 16 consecutive activations of one row as f16 (zero past row M).
template <int ADT>
__device__ __forceinline__ void load_a16(Frag16& f, const void* A, uint32_t row, uint32_t M, uint32_t K, uint32_t k0) {
    if (row >= M) {
#pragma unroll
        for (int i = 0; i < 8; i++) f.w[i] = 0;
        return;
    }
    if constexpr (ADT == LH_F32) {
        const float4* p = reinterpret_cast<const float4*>(static_cast<const float*>(A) + (size_t)row * K + k0);
#pragma unroll
        for (int i = 0; i < 4; i++) { const float4 v = p[i]; f.w[2 * i] = pack_h2(v.x, v.y); f.w[2 * i + 1] = pack_h2(v.z, v.w); }
    } else {
        const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(A) + (size_t)row * K + k0);
        const uint4 a = p[0], b = p[1];
        const uint32_t r[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if constexpr (ADT == LH_F16) f.w[i] = r[i];
            else f.w[i] = pack_h2(lh_bf2f((uint16_t)(r[i] & 0xFFFF)), lh_bf2f((uint16_t)(r[i] >> 16)));   // bf16 -> f16
        }
    }
}

// 16 consecutive dequantised weights of one row: elements k0 + half*16 .. +16 of weight row `row`.
template <int FMT>
__device__ __forceinline__ void load_b16(Frag16& f, const uint8_t* W, uint32_t row, uint32_t K, uint32_t k0, uint32_t half) {
    if constexpr (FMT == kF16W) {
        const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(W) + (size_t)row * K + k0 + half * 16);
        const uint4 a = p[0], b = p[1];
        f.w[0] = a.x; f.w[1] = a.y; f.w[2] = a.z; f.w[3] = a.w; f.w[4] = b.x; f.w[5] = b.y; f.w[6] = b.z; f.w[7] = b.w;
    } else if constexpr (FMT == kQ4) {
        const uint8_t* bp = W + ((size_t)row * (K >> 5) + (k0 >> 5)) * 18;
        const float d = lh_h2f(*reinterpret_cast<const uint16_t*>(bp));
        uint4 qv; __builtin_memcpy(&qv, __builtin_assume_aligned(bp + 2, 2), 16);
        const uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
        const uint32_t sh = half * 4;    // low nibbles -> elements 0..15, high nibbles -> 16..31
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t v = q[i] >> sh;
            f.w[2 * i] = pack_h2(((float)(v & 15) - 8.0f) * d, ((float)((v >> 8) & 15) - 8.0f) * d);
            f.w[2 * i + 1] = pack_h2(((float)((v >> 16) & 15) - 8.0f) * d, ((float)((v >> 24) & 15) - 8.0f) * d);
        }
    } else {
        const uint32_t blk = k0 >> 8, s = (k0 >> 5) & 7;               // 32-element slice s of the block
        const uint8_t* bp = W + ((size_t)row * (K >> 8) + blk) * 66;
        const float d = lh_h2f(*reinterpret_cast<const uint16_t*>(bp + 64));
        uint4 qv; __builtin_memcpy(&qv, __builtin_assume_aligned(bp + (s >> 2) * 32 + half * 16, 2), 16);
        const uint32_t q[4] = {qv.x, qv.y, qv.z, qv.w};
        const uint32_t sh = (s & 3) * 2;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t v = q[i] >> sh;
            f.w[2 * i] = pack_h2(d * ((float)(v & 3) - 1.0f), d * ((float)((v >> 8) & 3) - 1.0f));
            f.w[2 * i + 1] = pack_h2(d * ((float)((v >> 16) & 3) - 1.0f), d * ((float)((v >> 24) & 3) - 1.0f));
        }
    }
}

__device__ __forceinline__ void store_frag(_Float16* dst, const Frag16& f) {
    *reinterpret_cast<uint4*>(dst) = make_uint4(f.w[0], f.w[1], f.w[2], f.w[3]);
    *reinterpret_cast<uint4*>(dst + 8) = make_uint4(f.w[4], f.w[5], f.w[6], f.w[7]);
}

template <int FMT, int ADT, int CDT>
__global__ __launch_bounds__(256) void matmul_mfma_kernel(const void* __restrict__ A, const uint8_t* __restrict__ W, void* __restrict__ C,
                                                         uint32_t M, uint32_t K, uint32_t N) {
    __shared__ __align__(16) _Float16 As[BM * LDK];
    __shared__ __align__(16) _Float16 Bs[BN * LDK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;                 // 2 x 2 waves, 64 x 64 each
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t ld_row = tid >> 1, ld_half = tid & 1;     // staging: one 16-element run per thread
    const uint32_t a_row = m0 + ld_row;
    const uint32_t b_row = n0 + ld_row < N ? n0 + ld_row : N - 1;   // past-the-end rows re-read the last (never stored)

    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    Frag16 ra, rb;
    load_a16<ADT>(ra, A, a_row, M, K, ld_half * 16);
    load_b16<FMT>(rb, W, b_row, K, 0, ld_half);
    const uint32_t nk = K / BK;
    for (uint32_t kt = 0; kt < nk; kt++) {
        store_frag(&As[ld_row * LDK + ld_half * 16], ra);
        store_frag(&Bs[ld_row * LDK + ld_half * 16], rb);
        __syncthreads();
        if (kt + 1 < nk) {      // next tile's global loads fly during the MFMAs
            load_a16<ADT>(ra, A, a_row, M, K, (kt + 1) * BK + ld_half * 16);
            load_b16<FMT>(rb, W, b_row, K, (kt + 1) * BK, ld_half);
        }
        f16x8 fa[4], fb[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            fa[i] = *reinterpret_cast<const f16x8*>(&As[(wm * 64 + i * 16 + (lane & 15)) * LDK + (lane >> 4) * 8]);
#pragma unroll
        for (int j = 0; j < 4; j++)
            fb[j] = *reinterpret_cast<const f16x8*>(&Bs[(wn * 64 + j * 16 + (lane & 15)) * LDK + (lane >> 4) * 8]);
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        __syncthreads();
    }
    // D tile: lane holds column (lane & 15), rows 4*(lane >> 4) .. +4
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t n = n0 + wn * 64 + j * 16 + (lane & 15);
            if (n >= N) continue;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t m = m0 + wm * 64 + i * 16 + (lane >> 4) * 4 + r;
                if (m < M) store_elem<CDT>(C, (size_t)m * N + n, acc[i][j][r]);
            }
        }
}

template <int FMT, int ADT>
int launch_by_out(bool mfma, hipStream_t s, const void* A, const uint8_t* W, void* C, lh_dtype ct, uint32_t m, uint32_t k, uint32_t n) {
    if (mfma) {
        const dim3 grid((n + BN - 1) / BN, (m + BM - 1) / BM);
        if (ct == LH_F32) hipLaunchKernelGGL((matmul_mfma_kernel<FMT, ADT, LH_F32>), grid, dim3(256), 0, s, A, W, C, m, k, n);
        else hipLaunchKernelGGL((matmul_mfma_kernel<FMT, ADT, LH_F16>), grid, dim3(256), 0, s, A, W, C, m, k, n);
    } else {
        if constexpr (FMT != kF16W) {
            const dim3 grid((n + 3) / 4);
            if (ct == LH_F32) hipLaunchKernelGGL((multivec_kernel<FMT, ADT, LH_F32>), grid, dim3(256), 0, s, A, W, C, m, k, n);
            else hipLaunchKernelGGL((multivec_kernel<FMT, ADT, LH_F16>), grid, dim3(256), 0, s, A, W, C, m, k, n);
        }
    }
    return LH_OK;
}

template <int FMT>
int launch_by_in(bool mfma, hipStream_t s, const void* A, lh_dtype at, const uint8_t* W, void* C, lh_dtype ct, uint32_t m, uint32_t k,
                 uint32_t n) {
    switch (at) {
        case LH_F32: return launch_by_out<FMT, LH_F32>(mfma, s, A, W, C, ct, m, k, n);
        case LH_BF16: return launch_by_out<FMT, LH_BF16>(mfma, s, A, W, C, ct, m, k, n);
        default: return launch_by_out<FMT, LH_F16>(mfma, s, A, W, C, ct, m, k, n);
    }
}

// kind: kQ4 / kTQ2 / kF16W. `force_multivec` is the multivec_nt_* entry (m <= 16 enforced by the caller).
int matmul_dispatch(lh_batch* batch, const char* op, int kind, const lh_buffer* input, lh_dtype at, const lh_buffer* weight,
                    lh_buffer* output, lh_dtype ct, uint32_t m, uint32_t k, uint32_t n, bool force_multivec) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (ct == LH_BF16) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: bf16 output is not supported", op);
    const uint32_t blk = kind == kQ4 ? 32 : (kind == kTQ2 ? 256 : 32);
    // kernels.rs:6469-6473, 6519-6523: block alignment of k is checked before anything is encoded
    if (kind != kF16W && k % blk != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: k %u not /%u", op, k, blk);
    if (kind == kF16W && k % 32 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: k %u not /32", op, k);
    if (m == 0 || n == 0 || k == 0) return LH_OK;
    const size_t wbytes = kind == kQ4 ? (size_t)n * (k / 32) * 18 : (kind == kTQ2 ? (size_t)n * (k / 256) * 66 : (size_t)n * k * 2);
    LH_NEED(input, (size_t)m * k * lh_dtype_size(at), op, "input");
    LH_NEED(weight, wbytes, op, "weight");
    LH_NEED(output, (size_t)m * n * lh_dtype_size(ct), op, "output");
    LH_REQUIRE(((uintptr_t)input->ptr & 15) == 0, "%s: input must be 16-byte aligned", op);
    LH_REQUIRE(((uintptr_t)weight->ptr & 1) == 0, "%s: weight must be 2-byte aligned", op);
    const bool mfma = kind == kF16W || (!force_multivec && m > (uint32_t)kMaxMultivecM);
    if (!mfma) {
        // up to 16 activation rows: m matvecs against the same matrix in one launch of the M = 1 kernels (the weights
        // of one call stay cache resident between the rows); shapes they do not take fall through to multivec_kernel
        const int rr = lh_matvec_rows(batch, kind == kQ4 ? LH_Q4_0 : LH_TQ2_0, m, weight, input, at, output, ct, n, k, op);
        if (rr != -1) {
            if (rr == LH_OK) batch->dispatch_count++;
            return rr;
        }
    }
    hipStream_t s = batch->ctx->stream;
    const uint8_t* W = (const uint8_t*)weight->ptr;
    if (kind == kQ4) launch_by_in<kQ4>(mfma, s, input->ptr, at, W, output->ptr, ct, m, k, n);
    else if (kind == kTQ2) launch_by_in<kTQ2>(mfma, s, input->ptr, at, W, output->ptr, ct, m, k, n);
    else launch_by_in<kF16W>(true, s, input->ptr, at, W, output->ptr, ct, m, k, n);
    int r = lh_check_launch(op);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

}  // namespace

extern "C" {

int lh_matmul_nt_q4_0_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    return matmul_dispatch(b, "matmul_nt_q4_0", kQ4, in, LH_F16, w, out, LH_F16, m, k, n, false);
}
int lh_matmul_nt_tq2_0_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    return matmul_dispatch(b, "matmul_nt_tq2_0", kTQ2, in, LH_F16, w, out, LH_F16, m, k, n, false);
}
int lh_multivec_nt_q4_0_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    // kernels.rs:6388-6398
    if (k % 32 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "multivec_nt_q4_0: k %u not /32", k);
    if (m == 0 || m > (uint32_t)kMaxMultivecM) return lh_fail(LH_ERR_INVALID_ARGUMENT, "multivec_nt_q4_0: m %u out of 1..=16", m);
    return matmul_dispatch(b, "multivec_nt_q4_0", kQ4, in, LH_F16, w, out, LH_F16, m, k, n, true);
}
int lh_multivec_nt_tq2_0_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    // kernels.rs:6429-6439
    if (k % 256 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "multivec_nt_tq2_0: k %u not /256", k);
    if (m == 0 || m > (uint32_t)kMaxMultivecM) return lh_fail(LH_ERR_INVALID_ARGUMENT, "multivec_nt_tq2_0: m %u out of 1..=16", m);
    return matmul_dispatch(b, "multivec_nt_tq2_0", kTQ2, in, LH_F16, w, out, LH_F16, m, k, n, true);
}
int lh_matmul_nt_quant_typed_into(lh_batch* b, lh_quant fmt, const lh_buffer* in, lh_dtype at, const lh_buffer* w, lh_buffer* out,
                                  lh_dtype ct, uint32_t m, uint32_t k, uint32_t n) {
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matmul_nt_quant: unknown weight format %d", (int)fmt);
    return matmul_dispatch(b, fmt == LH_Q4_0 ? "matmul_nt_q4_0" : "matmul_nt_tq2_0", fmt == LH_Q4_0 ? kQ4 : kTQ2, in, at, w, out, ct, m,
                           k, n, false);
}
int lh_matmul_nt_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    return matmul_dispatch(b, "matmul_nt", kF16W, in, LH_F16, w, out, LH_F16, m, k, n, false);
}

}  // extern "C"
