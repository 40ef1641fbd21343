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
#include "xquant.hpp"
#include <cstdlib>

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
// C[M, N] = A[M, K] . W[N, K]^T with f16 MFMA: BM x 128 output tile per workgroup (BM = 64 or 128), 128-wide k steps.
// Weight tiles are dequantised to exactly the f16 values of the CPU path (qat_recover.rs:23-97) with packed f16
// arithmetic -- (1024 + code) is built by a byte permute, then (x - 1025) * d for TQ2_0 or (x - 1032) * d for Q4_0,
// whose single rounding equals f16::from_f32 of the f32 product -- and staged through LDS together with the
// activations (converted to f16); the next step's global loads fly during the MFMAs.
constexpr int BN = 128, BK = 128, LDK = BK + 16;  // LDS row stride in f16: 288 bytes.  The fragment reads (16 rows x 16 bytes per quarter wave) are conflict-free at 288 and lose a third of their rate at 272 (measured with a stand-alone probe: 5.9 against 8.0 cycles per ds_read_b128 with four waves reading)
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t pack_h2(float a, float b) { return (uint32_t)lh_f2h(a) | ((uint32_t)lh_f2h(b) << 16); }
// two bf16 -> two f16, each rounded to nearest even like the scalar conversion (v_cvt_pk_f16_f32)
__device__ __forceinline__ uint32_t bf2_to_h2(uint32_t w) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {__builtin_bit_cast(float, w << 16), __builtin_bit_cast(float, w & 0xFFFF0000u)};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}
__device__ __forceinline__ uint32_t h2_sub_mul(uint32_t x, uint32_t bias, uint32_t d2) {
    const f16x2 r = (__builtin_bit_cast(f16x2, x) - __builtin_bit_cast(f16x2, bias)) * __builtin_bit_cast(f16x2, d2);
    return __builtin_bit_cast(uint32_t, r);
}

// Raw global data of one weight staging run (32 consecutive k of one row), kept in registers across two k steps so that the
// loads have two steps of MFMA work to arrive; converted to f16 words just before they go to LDS.
template <int FMT> struct RawB { uint4 q[FMT == kF16W ? 4 : (FMT == kQ4 ? 1 : 2)]; uint32_t d; };

// Activations are staged in chunks of 8 consecutive k: the 16 lanes that share a row read 256 contiguous bytes (f16 / bf16).
template <int ADT> struct RawA8 { uint4 v[ADT == LH_F32 ? 2 : 1]; };

// Branch-free (the compiler can then count the loads in flight instead of waiting for all of them): rows past the end
// re-read the last row (their products are never stored), chunks past the end of a row re-read its last chunk and are
// zeroed by convert_a8.
template <int ADT>
__device__ __forceinline__ void load_raw_a8(RawA8<ADT>& r, const void* A, uint32_t row, uint32_t M, uint32_t K, uint32_t k0) {
    constexpr int NV = ADT == LH_F32 ? 2 : 1;
    const uint32_t rc = row < M ? row : M - 1, kc = k0 < K ? k0 : K - 8;
    const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint8_t*>(A) + ((size_t)rc * K + kc) * (ADT == LH_F32 ? 4 : 2));
#pragma unroll
    for (int i = 0; i < NV; i++) r.v[i] = p[i];
}

template <int ADT>
__device__ __forceinline__ uint4 convert_a8(const RawA8<ADT>& r) {
    if constexpr (ADT == LH_F32) {
        return make_uint4(pack_h2(__builtin_bit_cast(float, r.v[0].x), __builtin_bit_cast(float, r.v[0].y)),
                          pack_h2(__builtin_bit_cast(float, r.v[0].z), __builtin_bit_cast(float, r.v[0].w)),
                          pack_h2(__builtin_bit_cast(float, r.v[1].x), __builtin_bit_cast(float, r.v[1].y)),
                          pack_h2(__builtin_bit_cast(float, r.v[1].z), __builtin_bit_cast(float, r.v[1].w)));
    } else if constexpr (ADT == LH_F16) {
        return r.v[0];
    } else {
        const uint32_t w[4] = {r.v[0].x, r.v[0].y, r.v[0].z, r.v[0].w};
        uint32_t f[4];
#pragma unroll
        for (int j = 0; j < 4; j++) f[j] = pack_h2(lh_bf2f((uint16_t)(w[j] & 0xFFFF)), lh_bf2f((uint16_t)(w[j] >> 16)));   // bf16 -> f16
        return make_uint4(f[0], f[1], f[2], f[3]);
    }
}

// TQ2_0 weights of one k step (128 k = half a block = 32 code bytes of a row): a thread takes 16 of the bytes, i.e.
// elements 32f + 16 * part + j (field f = 0..3, j = 0..15) of the half block.
struct RawBT { uint4 q; uint32_t d; };
__device__ __forceinline__ void load_raw_bt(RawBT& r, const uint8_t* W, uint32_t row, uint32_t K, uint32_t k0, uint32_t part) {
    if (k0 >= K) k0 = K - 128;   // a step past the end re-reads the last one; convert_bt zeroes it
    const uint8_t* bp = W + ((size_t)row * (K >> 8) + (k0 >> 8)) * 66;
    r.d = *reinterpret_cast<const uint16_t*>(bp + 64);
    __builtin_memcpy(&r.q, __builtin_assume_aligned(bp + ((k0 >> 7) & 1) * 32 + 16 * part, 2), 16);
}
// The four values a TQ2_0 code can take in a block of scale d, d * (c - 1) for c = 0 .. 3, as two byte tables for v_perm_b32
// (byte c of lo / hi = low / high byte of the f16 value).  The products of d with -1, 0, 1 and 2 are exact in f16 (or the
// infinity, NaN or signed zero the CPU path's f32 product rounds to: qat_recover.rs:39-47), so looking a code up gives the
// CPU path's dequantised weight bit for bit -- with six instructions per four codes where (1024 + c - 1025) * d takes eight.
struct Tq2Table { uint32_t lo, hi; };
__device__ __forceinline__ Tq2Table tq2_table(uint32_t d2) {   // d2: the f16 scale in both halves
    const f16x2 dd = __builtin_bit_cast(f16x2, d2);
    const uint32_t t01 = __builtin_bit_cast(uint32_t, dd * (f16x2){(_Float16)-1.0f, (_Float16)0.0f});
    const uint32_t t23 = __builtin_bit_cast(uint32_t, dd * (f16x2){(_Float16)1.0f, (_Float16)2.0f});
    return {__builtin_amdgcn_perm(t23, t01, 0x06040200u), __builtin_amdgcn_perm(t23, t01, 0x07050301u)};
}
// Four codes (one per byte of c, each 0 .. 3) -> their f16 values: bytes 0, 1 in w0, bytes 2, 3 in w1.
__device__ __forceinline__ void tq2_lookup(const Tq2Table& t, uint32_t c, uint32_t& w0, uint32_t& w1) {
    const uint32_t lo = __builtin_amdgcn_perm(0u, t.lo, c), hi = __builtin_amdgcn_perm(0u, t.hi, c);
    w0 = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
    w1 = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
}
// f16 values of field f: 16 consecutive k as 8 words
__device__ __forceinline__ void convert_bt(uint32_t (&w)[8], const RawBT& r, int f, bool valid) {
    const uint32_t d = valid ? r.d : 0u;
    const Tq2Table t = tq2_table((d & 0xFFFFu) | (d << 16));
    const uint32_t q[4] = {r.q.x, r.q.y, r.q.z, r.q.w};
#pragma unroll
    for (int i = 0; i < 4; i++) tq2_lookup(t, (q[i] >> (2 * f)) & 0x03030303u, w[2 * i], w[2 * i + 1]);
}

// Elements k0 .. k0 + 32 of weight row `row` (k0 a multiple of 32).
template <int FMT>
__device__ __forceinline__ void load_raw_b(RawB<FMT>& r, const uint8_t* W, uint32_t row, uint32_t K, uint32_t k0) {
    // Past the end of the row in the last k step the last run is read again; convert_b zeroes it.  Nothing here may
    // compute on a loaded value: that would wait for the load right where it is issued.
    if (k0 >= K) k0 = K - 32;
    if constexpr (FMT == kF16W) {
        const uint4* p = reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(W) + (size_t)row * K + k0);
#pragma unroll
        for (int i = 0; i < 4; i++) r.q[i] = p[i];
        r.d = 0;
    } else if constexpr (FMT == kQ4) {
        const uint8_t* bp = W + ((size_t)row * (K >> 5) + (k0 >> 5)) * 18;
        r.d = *reinterpret_cast<const uint16_t*>(bp);
        __builtin_memcpy(&r.q[0], __builtin_assume_aligned(bp + 2, 2), 16);
    } else {
        const uint32_t blk = k0 >> 8, s = (k0 >> 5) & 7;               // 32-element slice s of the block: bytes (s/4)*32.., field s%4
        const uint8_t* bp = W + ((size_t)row * (K >> 8) + blk) * 66;
        r.d = *reinterpret_cast<const uint16_t*>(bp + 64);
        __builtin_memcpy(&r.q[0], __builtin_assume_aligned(bp + (s >> 2) * 32, 2), 16);
        __builtin_memcpy(&r.q[1], __builtin_assume_aligned(bp + (s >> 2) * 32 + 16, 2), 16);
    }
}

// k0 = first element of the run; `valid` = false past the end of the row (the run becomes zeros).
template <int FMT>
__device__ __forceinline__ void convert_b(uint32_t (&f)[16], const RawB<FMT>& r, uint32_t k0, bool valid) {
    if constexpr (FMT == kF16W) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            f[4 * i] = valid ? r.q[i].x : 0u; f[4 * i + 1] = valid ? r.q[i].y : 0u; f[4 * i + 2] = valid ? r.q[i].z : 0u; f[4 * i + 3] = valid ? r.q[i].w : 0u;
        }
    } else if constexpr (FMT == kQ4) {
        const uint32_t d = valid ? r.d : 0u;
        const uint32_t d2 = (d & 0xFFFFu) | (d << 16);
        const uint32_t q[4] = {r.q[0].x, r.q[0].y, r.q[0].z, r.q[0].w};
        // byte j: low nibble = element j, high nibble = element 16 + j
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t lo = q[i] & 0x0F0F0F0Fu, hi = (q[i] >> 4) & 0x0F0F0F0Fu;
            f[2 * i] = h2_sub_mul(__builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u), 0x64086408u, d2);          // 1024 + q - 1032
            f[2 * i + 1] = h2_sub_mul(__builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u), 0x64086408u, d2);
            f[8 + 2 * i] = h2_sub_mul(__builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u), 0x64086408u, d2);
            f[8 + 2 * i + 1] = h2_sub_mul(__builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u), 0x64086408u, d2);
        }
    } else {
        const uint32_t d = valid ? r.d : 0u;
        const uint32_t sh = ((k0 >> 5) & 3) * 2;
        const Tq2Table t = tq2_table((d & 0xFFFFu) | (d << 16));
        const uint32_t q[8] = {r.q[0].x, r.q[0].y, r.q[0].z, r.q[0].w, r.q[1].x, r.q[1].y, r.q[1].z, r.q[1].w};
#pragma unroll
        for (int i = 0; i < 8; i++) tq2_lookup(t, (q[i] >> sh) & 0x03030303u, f[2 * i], f[2 * i + 1]);
    }
}

template <int NW>
__device__ __forceinline__ void store_words(_Float16* dst, const uint32_t (&f)[NW]) {
#pragma unroll
    for (int i = 0; i < NW / 4; i++) *reinterpret_cast<uint4*>(dst + 8 * i) = make_uint4(f[4 * i], f[4 * i + 1], f[4 * i + 2], f[4 * i + 3]);
}

// Up to four weight matrices of one format and one K that multiply the same activations (Q / K / V, gate / up) as one
// launch: their column tiles are laid side by side, tile0[i] being the first tile of matrix i (tile0[count] = all).
struct GroupArgs {
    const uint8_t* W[4];
    void* C[4];
    uint32_t N[4];
    uint32_t tile0[5];
    uint32_t count;          // 0: the single matrix of the kernel arguments
};
__device__ __forceinline__ uint32_t group_of_tile(const GroupArgs& g, uint32_t tile) {
    uint32_t i = 0;
#pragma unroll
    for (uint32_t j = 1; j < 4; j++) if (j < g.count && tile >= g.tile0[j]) i = j;
    return i;
}

// Optional fused clamp / bias of the clipped linear layer (shaders/matmul_f16.metal:121-170):
// C = clamp(clamp(A, in_lo, in_hi) . W^T + bias, out_lo, out_hi).  Inactive for every other entry point.
struct ClipArgs {
    const uint16_t* bias;   // f16 [N] or null
    float in_lo, in_hi, out_lo, out_hi;
    uint32_t enabled;
};

__device__ __forceinline__ uint32_t clamp_h2(uint32_t w, float lo, float hi) {
    const float a = fminf(fmaxf(lh_h2f((uint16_t)(w & 0xFFFF)), lo), hi), b = fminf(fmaxf(lh_h2f((uint16_t)(w >> 16)), lo), hi);
    return pack_h2(a, b);
}

template <int FMT, int ADT, int CDT, int BM>
__global__ __launch_bounds__(256) void matmul_mfma_kernel(const void* __restrict__ A, const uint8_t* __restrict__ W_one, void* __restrict__ C_one,
                                                         uint32_t M, uint32_t K, uint32_t N_one, ClipArgs clip,
                                                         float* __restrict__ partial, uint32_t steps_per_split, GroupArgs grp) {
    const uint8_t* __restrict__ W = W_one;
    void* __restrict__ C = C_one;
    uint32_t N = N_one, col_tile = blockIdx.x;
    if (grp.count) {   // uniform over the workgroup
        const uint32_t gi = group_of_tile(grp, col_tile);
        W = grp.W[gi]; C = grp.C[gi]; N = grp.N[gi];
        col_tile -= grp.tile0[gi];
    }
    constexpr int TI = BM / 32;                              // 16-row MFMA tiles per wave along M (2 x 2 waves)
    constexpr int NCH = BM / 16;                             // 8-element activation chunks staged per thread
    __shared__ __align__(16) _Float16 As[BM * LDK];
    __shared__ __align__(16) _Float16 Bs[BN * LDK];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const uint32_t m0 = blockIdx.y * BM, n0 = col_tile * BN;
    const uint32_t b_ld_row = tid >> 1, b_ld_k = (tid & 1) * 64;
    const uint32_t b_row = n0 + b_ld_row < N ? n0 + b_ld_row : N - 1;   // past-the-end rows re-read the last (never stored)

    // Split k (gridDim.z > 1, few output tiles): this workgroup multiplies k steps [kt_begin, kt_end) only and leaves
    // its f32 tile in `partial[z]`; splitk_reduce_kernel sums the splits.  Steps at or past Kend are staged as zeros.
    const uint32_t nk = (K + BK - 1) / BK;
    const uint32_t kt_begin = blockIdx.z * steps_per_split;
    const uint32_t kt_end = kt_begin + steps_per_split < nk ? kt_begin + steps_per_split : nk;
    const uint32_t Kend = kt_end * BK < K ? kt_end * BK : K;

    f32x4 acc[TI][4];
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};

    RawA8<ADT> ra[2][NCH];   // [k step parity][chunk]: chunk c = tid + 256 i is row c / 16, k offset 8 * (c % 16)
    RawB<FMT> rb[2][FMT == kTQ2 ? 1 : 2];
    RawBT rbt[2];
    auto load_step = [&](int set, uint32_t kt) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const uint32_t c = tid + 256 * i;
            load_raw_a8<ADT>(ra[set][i], A, m0 + (c >> 4), M, K, kt * BK + 8 * (c & 15));
        }
        if constexpr (FMT == kTQ2) {
            load_raw_bt(rbt[set], W, b_row, K, kt * BK, tid & 1);
        } else {
#pragma unroll
            for (int i = 0; i < 2; i++) load_raw_b<FMT>(rb[set][i], W, b_row, K, kt * BK + b_ld_k + 32 * i);
        }
    };
    auto stage_step = [&](int set, uint32_t kt) {
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const uint32_t c = tid + 256 * i;
            uint4 v = convert_a8<ADT>(ra[set][i]);
            if (clip.enabled) v = make_uint4(clamp_h2(v.x, clip.in_lo, clip.in_hi), clamp_h2(v.y, clip.in_lo, clip.in_hi),
                                             clamp_h2(v.z, clip.in_lo, clip.in_hi), clamp_h2(v.w, clip.in_lo, clip.in_hi));
            if (kt * BK + BK > Kend && kt * BK + 8 * (c & 15) >= Kend) v = make_uint4(0u, 0u, 0u, 0u);   // only past the last k step
            *reinterpret_cast<uint4*>(&As[(c >> 4) * LDK + 8 * (c & 15)]) = v;
        }
        if constexpr (FMT == kTQ2) {
#pragma unroll
            for (int f = 0; f < 4; f++) {
                uint32_t w[8];
                convert_bt(w, rbt[set], f, kt * BK < Kend);
                store_words<8>(&Bs[b_ld_row * LDK + 32 * f + 16 * (tid & 1)], w);
            }
        } else {
            uint32_t f[16];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                const uint32_t k0 = kt * BK + b_ld_k + 32 * i;
                convert_b<FMT>(f, rb[set][i], k0, k0 < Kend);
                store_words<16>(&Bs[b_ld_row * LDK + b_ld_k + 32 * i], f);
            }
        }
    };
    auto mfma_step = [&]() {
#pragma unroll
        for (int ks = 0; ks < BK / 32; ks++) {
            f16x8 fa[TI], fb[4];
#pragma unroll
            for (int i = 0; i < TI; i++)
                fa[i] = *reinterpret_cast<const f16x8*>(&As[(wm * (BM / 2) + i * 16 + (lane & 15)) * LDK + ks * 32 + (lane >> 4) * 8]);
#pragma unroll
            for (int j = 0; j < 4; j++)
                fb[j] = *reinterpret_cast<const f16x8*>(&Bs[(wn * 64 + j * 16 + (lane & 15)) * LDK + ks * 32 + (lane >> 4) * 8]);
#pragma unroll
            for (int i = 0; i < TI; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
    };
    // Two k steps per trip (the register sets alternate without copies).  Every trip issues the same loads in the same
    // order, also past the end of K (those re-read the last step and are staged as zeros): a fixed number of loads in
    // flight lets the waits before staging leave the newer set outstanding.
    load_step(0, kt_begin);
    load_step(1, kt_begin + 1);
    for (uint32_t kt = kt_begin; kt < kt_end; kt += 2) {
        stage_step(0, kt);
        __syncthreads();
        load_step(0, kt + 2);
        mfma_step();
        __syncthreads();
        stage_step(1, kt + 1);
        __syncthreads();
        load_step(1, kt + 3);
        mfma_step();
        __syncthreads();
    }
    // D tile: lane holds column (lane & 15), rows 4*(lane >> 4) .. +4
#pragma unroll
    for (int i = 0; i < TI; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t n = n0 + wn * 64 + j * 16 + (lane & 15);
            if (n >= N) continue;
            if (partial) {
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    const uint32_t m = m0 + wm * (BM / 2) + i * 16 + (lane >> 4) * 4 + r;
                    // partial tiles keep the launch's tile grid: row stride gridDim.x * BN, column = tile * BN + offset
                    if (m < M) partial[((size_t)blockIdx.z * M + m) * (gridDim.x * BN) + blockIdx.x * BN + (n - n0)] = acc[i][j][r];
                }
                continue;
            }
            const float bias = (clip.enabled && clip.bias) ? lh_h2f(clip.bias[n]) : 0.0f;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const uint32_t m = m0 + wm * (BM / 2) + i * 16 + (lane >> 4) * 4 + r;
                float v = acc[i][j][r];
                if (clip.enabled) v = fminf(fmaxf(v + bias, clip.out_lo), clip.out_hi);
                if (m < M) store_elem<CDT>(C, (size_t)m * N + n, v);
            }
        }
}

// Sum of the split-k partial tiles (laid out on the launch's tile grid, `tiles` column tiles wide), with the bias / clamp
// of the clipped linear layer, stored in the output type of the matrix the column belongs to.
template <int CDT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, void* __restrict__ C_one, uint32_t M, uint32_t N_one,
                                                           uint32_t tiles, uint32_t splits, ClipArgs clip, GroupArgs grp) {
    const size_t nv_total = (size_t)tiles * BN, total = (size_t)M * nv_total, i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const uint32_t m = (uint32_t)(i / nv_total), nv = (uint32_t)(i - (size_t)m * nv_total);
    void* C = C_one;
    uint32_t N = N_one, n = nv;
    if (grp.count) {
        const uint32_t gi = group_of_tile(grp, nv / BN);
        C = grp.C[gi]; N = grp.N[gi];
        n = nv - grp.tile0[gi] * BN;
    }
    if (n >= N) return;
    float v = 0.0f;
    for (uint32_t z = 0; z < splits; z++) v += partial[(size_t)z * total + i];
    if (clip.enabled) {
        const float bias = clip.bias ? lh_h2f(clip.bias[n]) : 0.0f;
        v = fminf(fmaxf(v + bias, clip.out_lo), clip.out_hi);
    }
    store_elem<CDT>(C, (size_t)m * N + n, v);
}

// ---- 128 x 128 tiles for large M: f16 activations (converted once by a pre-pass when they arrive as bf16 / f32),
//      double-buffered LDS (one barrier per k step), four staging waves next to four multiplying waves, global data two
//      steps ahead in registers, and load addresses formed as uniform base + constant lane offset so that a staging
//      step spends its vector ALU time on the dequantisation.  The LDS traffic per step (128 KB of fragment reads, 64 KB
//      of staging writes against 1024 MFMA cycles per SIMD) is what bounds this tile shape.
template <int ADT>
__global__ __launch_bounds__(256) void convert_to_f16_kernel(const void* __restrict__ src, uint16_t* __restrict__ dst, size_t n8) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;   // 8 elements each
    if (i >= n8) return;
    RawA8<ADT> r;
    const uint4* p = reinterpret_cast<const uint4*>(static_cast<const uint8_t*>(src) + i * 8 * (ADT == LH_F32 ? 4 : 2));
#pragma unroll
    for (int j = 0; j < (ADT == LH_F32 ? 2 : 1); j++) r.v[j] = p[j];
    reinterpret_cast<uint4*>(dst)[i] = convert_a8<ADT>(r);
}

// Global loads whose completion the kernel waits for itself: the two register sets in flight need "wait until only
// the newer set is outstanding", which the compiler's own wait insertion turns into a wait for everything.  The value
// of a destination is undefined until wait_loads<N>() has run and the destination has passed through settle().
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void async_load16(u32x4v& dst, const uint8_t* uniform_base, uint32_t lane_offset) {
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(dst) : "v"(lane_offset), "s"(uniform_base) : "memory");
}
__device__ __forceinline__ void async_load2(uint32_t& dst, const uint8_t* uniform_base, uint32_t lane_offset) {
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(dst) : "v"(lane_offset), "s"(uniform_base) : "memory");
}
template <int N> __device__ __forceinline__ void wait_loads() { asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory"); }
__device__ __forceinline__ void settle(u32x4v& v) { asm volatile("" : "+v"(v)); }
__device__ __forceinline__ void settle(uint32_t& v) { asm volatile("" : "+v"(v)); }

// ABF: the activations arrive as bf16 and are converted to f16 on their way into LDS (three vector instructions per pair,
// in every column tile), which costs less than a conversion pass of its own: that pass is a second dependent launch.
// PW: staging waves (4 or 8) next to the four multiplying waves.  Eight halve the load -> convert -> store chain of each
// staging wave and put three waves on every SIMD.
template <int FMT, int CDT, bool ABF = false, int PW = 4>
__global__ __launch_bounds__(256 + 64 * PW) void matmul_mfma128_kernel(const uint16_t* __restrict__ A, const uint8_t* __restrict__ W, void* __restrict__ C,
                                                            uint32_t M, uint32_t K, uint32_t N) {
    static_assert(FMT == kQ4 || FMT == kTQ2, "quantised weights only");
    constexpr int BM = 128, PT = 64 * PW, NCH = 2048 / PT;        // staging threads; 16-byte activation chunks per staging thread and step
    constexpr int NB = (FMT == kQ4 && PW == 4) ? 2 : 1;           // weight pieces per staging thread and step
    constexpr int kLoadsPerStep = NCH + 2 * NB;
    __shared__ __align__(16) _Float16 As[2][BM * LDK];
    __shared__ __align__(16) _Float16 Bs[2][BN * LDK];
    // Waves 0-3 multiply (2 x 2 waves, 64 x 64 outputs each), the other PW waves stage: every SIMD holds one multiplying wave
    // and one or two staging waves, so the staging waves' memory and LDS waits are filled by the other wave's MFMAs.  One
    // barrier per k step hands over a buffer.
    const bool producer = threadIdx.x >= 256;
    const int tid = producer ? (int)threadIdx.x - 256 : (int)threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t nk = K / BK;                                   // K is a multiple of 128 here

    if (producer) {
        const uint32_t row_bytes = FMT == kQ4 ? (K >> 5) * 18 : (K >> 8) * 66;
        // lane-constant byte offsets from the tile bases; rows past the end re-read the last row (their products are not stored)
        uint32_t a_off[NCH], a_lds[NCH];
#pragma unroll
        for (int i = 0; i < NCH; i++) {
            const uint32_t c = tid + PT * i, row = c >> 4, kc = c & 15;
            const uint32_t rc = m0 + row < M ? row : M - 1 - m0;
            a_off[i] = (rc * K + 8 * kc) * 2;
            a_lds[i] = row * LDK + 8 * kc;
        }
        // Four staging waves: two threads per weight row.  Q4_0: 4 blocks of 18 bytes per step and row, a thread takes
        // blocks 2 * part, 2 * part + 1.  TQ2_0: one 66-byte block per two steps and row, a thread takes 16 of the step's
        // 32 code bytes (all four fields).  Eight staging waves: four threads per row; Q4_0 one block each, TQ2_0 the
        // same 16 code bytes twice, fields 0, 1 on one thread and 2, 3 on the other.
        // (TQ2_0, eight waves: the eight lanes of one LDS store phase take rows r and r + 2 instead of r and r + 1 -- at 288
        // bytes per row the four 32-byte pieces of neighbouring rows meet on the same banks, those of rows two apart do not)
        const uint32_t b_ld_row = PW == 4 ? tid >> 1
                                : FMT == kTQ2 ? ((tid >> 4) << 2) + (((tid >> 2) & 1) << 1) + ((tid >> 3) & 1) : tid >> 2;
        const uint32_t part = PW == 4 ? tid & 1 : (FMT == kQ4 ? tid & 3 : (tid >> 1) & 1), fh = tid & 1;
        (void)fh;
        const uint32_t b_rc = n0 + b_ld_row < N ? b_ld_row : N - 1 - n0;
        const uint32_t b_off = b_rc * row_bytes + (FMT == kQ4 ? part * (PW == 4 ? 36 : 18) : part * 16);
        const uint8_t* a_tile = reinterpret_cast<const uint8_t*>(A) + (size_t)m0 * K * 2;
        const uint8_t* w_tile = W + (size_t)n0 * row_bytes;

        u32x4v ra[2][NCH], rq[2][NB];
        uint32_t rd[2][NB];
        auto load_step = [&](int set, uint32_t kt) {
            if (kt >= nk) kt = nk - 1;                            // over-issued steps re-read the last one (staged into a buffer that is not read again)
            const uint8_t* ab = a_tile + (size_t)kt * (BK * 2);
#pragma unroll
            for (int i = 0; i < NCH; i++) async_load16(ra[set][i], ab, a_off[i]);
            if constexpr (FMT == kQ4) {
                const uint8_t* wb = w_tile + (size_t)kt * 72;
#pragma unroll
                for (int i = 0; i < NB; i++) {
                    async_load2(rd[set][i], wb, b_off + 18 * i);
                    async_load16(rq[set][i], wb, b_off + 18 * i + 2);
                }
            } else {
                const uint8_t* wb = w_tile + (size_t)(kt >> 1) * 66;
                async_load2(rd[set][0], wb, b_rc * row_bytes + 64);
                async_load16(rq[set][0], wb + (kt & 1) * 32, b_off);
            }
        };
        auto stage_step = [&](int set, int buf) {
            wait_loads<kLoadsPerStep>();                          // everything but the newer set has arrived
#pragma unroll
            for (int i = 0; i < NCH; i++) settle(ra[set][i]);
#pragma unroll
            for (int i = 0; i < NB; i++) { settle(rq[set][i]); settle(rd[set][i]); }
#pragma unroll
            for (int i = 0; i < NCH; i++) {
                uint4 v = make_uint4(ra[set][i].x, ra[set][i].y, ra[set][i].z, ra[set][i].w);
                if constexpr (ABF) v = make_uint4(bf2_to_h2(v.x), bf2_to_h2(v.y), bf2_to_h2(v.z), bf2_to_h2(v.w));
                *reinterpret_cast<uint4*>(&As[buf][a_lds[i]]) = v;
            }
            if constexpr (FMT == kQ4) {
                uint32_t f[16];
#pragma unroll
                for (int i = 0; i < NB; i++) {
                    RawB<kQ4> r;
                    r.q[0] = make_uint4(rq[set][i].x, rq[set][i].y, rq[set][i].z, rq[set][i].w);
                    r.d = rd[set][i];
                    convert_b<kQ4>(f, r, 0, true);
                    store_words<16>(&Bs[buf][b_ld_row * LDK + (PW == 4 ? 64 : 32) * part + 32 * i], f);
                }
            } else {
                RawBT r;
                r.q = make_uint4(rq[set][0].x, rq[set][0].y, rq[set][0].z, rq[set][0].w);
                r.d = rd[set][0];
                if constexpr (PW == 4) {
#pragma unroll
                    for (int f = 0; f < 4; f++) {
                        uint32_t w[8];
                        convert_bt(w, r, f, true);
                        store_words<8>(&Bs[buf][b_ld_row * LDK + 32 * f + 16 * part], w);
                    }
                } else {
#pragma unroll
                    for (int f2 = 0; f2 < 2; f2++) {
                        const int f = 2 * (int)fh + f2;
                        uint32_t w[8];
                        convert_bt(w, r, f, true);
                        store_words<8>(&Bs[buf][b_ld_row * LDK + 32 * f + 16 * part], w);
                    }
                }
            }
        };
        // Step kt is multiplied from LDS buffer kt & 1 while step kt + 1 is staged into the other buffer from register
        // set (kt + 1) & 1, whose registers then take the loads of step kt + 3.  Every stage finds exactly two sets in
        // flight, the one it needs being the older.
        load_step(0, 0);
        load_step(1, 1);
        stage_step(0, 0);
        load_step(0, 2);
        __syncthreads();
        for (uint32_t kt = 0; kt < nk; kt += 2) {
            stage_step(1, 1);
            load_step(1, kt + 3);
            __syncthreads();
            if (kt + 1 < nk) {
                stage_step(0, 0);
                load_step(0, kt + 4);
                __syncthreads();
            }
        }
        wait_loads<0>();             // the over-issued loads must not outlive their destination registers
        return;
    }

    const int wm = wave >> 1, wn = wave & 1;
    // acc[i][j] holds the transposed 16 x 16 tile (weights as the MFMA row operand): lane = output row m (lane & 15) and
    // four consecutive output columns 4 * (lane >> 4) .. + 3, i.e. one 16-byte store per tile.
    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto mfma_step = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < BK / 32; ks++) {
            f16x8 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; i++)
                fa[i] = *reinterpret_cast<const f16x8*>(&As[buf][(wm * 64 + i * 16 + (lane & 15)) * LDK + ks * 32 + (lane >> 4) * 8]);
#pragma unroll
            for (int j = 0; j < 4; j++)
                fb[j] = *reinterpret_cast<const f16x8*>(&Bs[buf][(wn * 64 + j * 16 + (lane & 15)) * LDK + ks * 32 + (lane >> 4) * 8]);
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
        }
    };
    __syncthreads();
    for (uint32_t kt = 0; kt < nk; kt += 2) {
        mfma_step(0);
        __syncthreads();
        if (kt + 1 < nk) {
            mfma_step(1);
            __syncthreads();
        }
    }

    const bool vec_ok = (N & 3) == 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t m = m0 + wm * 64 + i * 16 + (lane & 15);
        if (m >= M) continue;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const uint32_t n = n0 + wn * 64 + j * 16 + (lane >> 4) * 4;
            const f32x4 v = acc[i][j];
            if (vec_ok && n + 3 < N) {
                // an f32 result (16 bytes per lane) goes out with streaming stores: measured 26.3 -> 24.7 us on 512 x 2048 x 8192;
                // the 8-byte stores of an f16 result are slower that way (21.7 -> 23.7 us) and stay plain
                if constexpr (CDT == LH_F32) __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(static_cast<float*>(C) + (size_t)m * N + n));
                else *reinterpret_cast<uint2*>(static_cast<uint16_t*>(C) + (size_t)m * N + n) = make_uint2(pack_h2(v[0], v[1]), pack_h2(v[2], v[3]));
            } else {
#pragma unroll
                for (int r = 0; r < 4; r++)
                    if (n + r < N) store_elem<CDT>(C, (size_t)m * N + n + r, v[r]);
            }
        }
    }
}

// ---- a decode batch of 17 .. 64 rows, a prefill chunk of up to 256: weights straight from global memory into MFMA operands ----
// At these row counts a product is a few microseconds of matrix-core time and what counts is latency, so this kernel
// has no workgroup-wide staging phase and one barrier.  A workgroup owns 64 weight rows (four 16-row MFMA tiles) and a
// k range; its four waves split that range in quarters, every wave multiplying all four tiles against all activation
// rows for its quarter (one B fragment feeds four MFMAs), and the four partial tiles are added through LDS at the end.
//
// A lane fetches the codes it turns into its own A fragments, 8 bytes at a time, one "unit" ahead:
//   Q4_0  unit = 2 blocks (64 k).  Lane (row r, g) reads qs bytes 8(g&1) .. +8 of block (g>>1): the low nibbles are
//         elements 8(g&1) .. +8 of that block (fragment 0), the high nibbles elements 16 + 8(g&1) .. +8 (fragment 1).
//   TQ2_0 unit = half a block (128 k).  Lane (r, g) reads bytes 8g .. +8 of the half: field f of those bytes is
//         elements 32 f + 8g .. +8 of the half (fragment f, 0 .. 3).
// A code byte c becomes the f16 value 1024 + c by byte permutation (0x6400 | c), the zero point is subtracted exactly
// and the result multiplied by the block scale in f16: the CPU path's dequantised weight f16((q - 8) d) / d (q - 1)
// (qat_recover.rs:39-47, 84-93) bit for bit, as in the LDS-tiled kernels.  The B fragment of a k step holds the
// activations of the same eight k indices; a wave brings them in row by row and re-reads them in fragment order from
// its own LDS area (see load_b / park_b).
template <int FMT> struct Skinny;
template <> struct Skinny<kQ4> { static constexpr int unit_k = 64, frags = 2; };
template <> struct Skinny<kTQ2> { static constexpr int unit_k = 128, frags = 4; };

struct SkinnyRaw { uint32_t w0, w1, d; };

__device__ __forceinline__ uint2 ld8_align2(const uint8_t* p) {
    typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
    typedef u32x2_t __attribute__((aligned(2))) u32x2_a2;
    const u32x2_t v = *reinterpret_cast<const u32x2_a2*>(p);
    return make_uint2(v.x, v.y);
}

template <int FMT>
__device__ __forceinline__ f16x8 skinny_fragment(const SkinnyRaw& raw, int f) {
    if constexpr (FMT == kTQ2) {   // the block's four values looked up (tq2_table): the same bits with fewer instructions
        const Tq2Table t = tq2_table(raw.d);
        uint32_t o[4];
        tq2_lookup(t, (raw.w0 >> (2 * f)) & 0x03030303u, o[0], o[1]);
        tq2_lookup(t, (raw.w1 >> (2 * f)) & 0x03030303u, o[2], o[3]);
        struct { uint32_t v[4]; } tt = {{o[0], o[1], o[2], o[3]}};
        return __builtin_bit_cast(f16x8, tt);
    }
    uint32_t c0, c1;
    f16x2 zp;
    if constexpr (FMT == kQ4) { c0 = (raw.w0 >> (4 * f)) & 0x0F0F0F0Fu; c1 = (raw.w1 >> (4 * f)) & 0x0F0F0F0Fu; zp = (f16x2){(_Float16)1032.0f, (_Float16)1032.0f}; }
    else { c0 = (raw.w0 >> (2 * f)) & 0x03030303u; c1 = (raw.w1 >> (2 * f)) & 0x03030303u; zp = (f16x2){(_Float16)1025.0f, (_Float16)1025.0f}; }
    const f16x2 dd = __builtin_bit_cast(f16x2, raw.d);
    const uint32_t p[4] = {__builtin_amdgcn_perm(0x64646464u, c0, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, c0, 0x04030402u),
                           __builtin_amdgcn_perm(0x64646464u, c1, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, c1, 0x04030402u)};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; i++) o[i] = __builtin_bit_cast(uint32_t, (__builtin_bit_cast(f16x2, p[i]) - zp) * dd);
    struct { uint32_t v[4]; } t = {{o[0], o[1], o[2], o[3]}};
    return __builtin_bit_cast(f16x8, t);
}

// PAIR: the feed-forward gate and up projections with their gelu_mul (layer.rs:652-662).  The workgroup's tiles 0, 1 are 32
// rows of grp.W[0] (gate), tiles 2, 3 the same 32 rows of grp.W[1] (up), so that both factors of an output meet in the
// reduction: out = half(gelu(half(gate)) * half(up)), the values the two products and gelu_mul would have stored.
// XF32: f32 activations, at most 32 rows.  A row enters as two f16 rows -- x rounded to f16 in activation group j (rows 16j ..
// 16j + 15, j = 0, 1) and the remainder x - f16(x), rounded to f16, in group j + 2 -- and the two outputs are added at the
// end: the product then carries about 22 bits of every activation instead of 11.
template <int FMT, int CDT, bool PAIR = false, bool XF32 = false>
__global__ __launch_bounds__(256, 2) void matmul_skinny_kernel(const uint16_t* __restrict__ X, const uint8_t* __restrict__ W_one, void* __restrict__ C_one,
                                                              uint32_t M, uint32_t K, uint32_t N_one, float* __restrict__ partial,
                                                              uint32_t units_per_wave, GroupArgs grp) {
    constexpr int UK = Skinny<FMT>::unit_k, NF = Skinny<FMT>::frags;
    // [wave][tile][activation group][lane] partial tiles at the end; before that each wave keeps the activations of its
    // current unit in its quarter of the same memory
    __shared__ float4 red[4][4][4][64];
    const uint8_t* __restrict__ W = W_one;
    void* __restrict__ C = C_one;
    uint32_t N = N_one, tile = blockIdx.x >> 1;               // blockIdx.x counts 64-row halves of the 128-row tile grid
    if (!PAIR && grp.count) {
        const uint32_t gi = group_of_tile(grp, tile);
        W = grp.W[gi]; C = grp.C[gi]; N = grp.N[gi];
        tile -= grp.tile0[gi];
    }
    const uint32_t n0 = PAIR ? blockIdx.x * 32 : tile * BN + (blockIdx.x & 1) * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t r = lane & 15, g = lane >> 4;
    const size_t row_bytes = FMT == kQ4 ? (size_t)(K >> 5) * 18 : (size_t)(K >> 8) * 66;
    const uint32_t k_begin = (blockIdx.z * 4 + wave) * units_per_wave * UK;
    const uint32_t m0 = blockIdx.y * 64;                      // more than 64 activation rows: one workgroup per 64 of them

    const uint8_t* wrow = W + (size_t)(n0 + r) * row_bytes;   // tile t starts 16 rows further on
    const size_t tile_bytes = 16 * row_bytes;
    const uint8_t* wrow_up = PAIR ? grp.W[1] + (size_t)(n0 + r) * row_bytes : nullptr;
    auto load_a = [&](SkinnyRaw (&raw)[4], uint32_t k0) {
        size_t off, doff;
        if constexpr (FMT == kQ4) { const size_t b = (k0 >> 5) + (g >> 1); doff = b * 18; off = doff + 2 + 8 * (g & 1); }
        else { const size_t b = k0 >> 8; doff = b * 66 + 64; off = b * 66 + 32 * ((k0 >> 7) & 1) + 8 * g; }
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint8_t* p = PAIR ? (t < 2 ? wrow : wrow_up) + (t & 1) * tile_bytes : wrow + t * tile_bytes;
            const uint2 w = ld8_align2(p + off);
            const uint32_t d = *reinterpret_cast<const uint16_t*>(p + doff);
            raw[t].w0 = w.x; raw[t].w1 = w.y; raw[t].d = d | (d << 16);
        }
    };
    // The activations of a unit (64 rows x UK columns) come in with coalesced loads -- a lane takes 16 bytes of one row,
    // CPR consecutive lanes one row's UK columns -- one unit ahead, and are parked in the wave's LDS area in fragment
    // order: block (f, j) holds the 64 cells of B fragment f of activation group j, cell 16g + (c ^ (g | 4 (f & 1))) being
    // row 16j + c, k group g: eight consecutive lanes read eight cells of one aligned 128-byte line, and the eight cells
    // of a row that eight consecutive lanes write fall into eight different bank groups.  Read straight from global memory
    // in fragment order the same bytes cost 16 half-used cache lines per instruction, which bounded the kernel.
    constexpr int CPR = UK / 8, RPI = 64 / CPR, NLD = 64 / RPI;          // 16-byte chunks per row, rows and loads per unit
    f32x4* stage = reinterpret_cast<f32x4*>(&red[wave][0][0][0]);        // NF * 4 blocks of 64 cells (at most 16 KB)
    const uint32_t ld_row = lane / CPR, ld_q = lane % CPR;
    uint32_t ld_f, ld_g;
    if constexpr (FMT == kQ4) { ld_g = 2 * (ld_q >> 2) + (ld_q & 1); ld_f = (ld_q & 3) >> 1; }
    else { ld_f = ld_q >> 2; ld_g = ld_q & 3; }
    auto load_b = [&](f32x4 (&raw)[NLD], uint32_t k0) {
        if constexpr (XF32) {   // rows 0 .. 31 only, eight f32 values = two registers of the set per row
            const float* X32 = reinterpret_cast<const float*>(X);
#pragma unroll
            for (int i = 0; i < NLD / 2; i++) {
                const uint32_t m = RPI * i + ld_row;
                const float* p = X32 + (size_t)(m < M ? m : M - 1) * K + k0 + 8 * ld_q;
                raw[2 * i] = *reinterpret_cast<const f32x4*>(p);
                raw[2 * i + 1] = *reinterpret_cast<const f32x4*>(p + 4);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NLD; i++) {
                const uint32_t m = m0 + RPI * i + ld_row;
                raw[i] = *reinterpret_cast<const f32x4*>(X + (size_t)(m < M ? m : M - 1) * K + k0 + 8 * ld_q);   // rows past M repeat the last one
            }
        }
    };
    auto park_b = [&](const f32x4 (&raw)[NLD]) {
        if constexpr (XF32) {
#pragma unroll
            for (int i = 0; i < NLD / 2; i++) {
                const uint32_t m = RPI * i + ld_row, j = m >> 4, c = m & 15;
                const float x[8] = {raw[2 * i][0], raw[2 * i][1], raw[2 * i][2], raw[2 * i][3],
                                    raw[2 * i + 1][0], raw[2 * i + 1][1], raw[2 * i + 1][2], raw[2 * i + 1][3]};
                struct { uint32_t v[4]; } hi, lo;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    // A finite value beyond the f16 range keeps a finite first part (the remainder then carries the rest, up to
                    // 131008 in all); left alone it would be inf with the remainder -inf, and the two products would add to NaN.
                    auto first_part = [](float v) {
                        const float a = __builtin_fabsf(v);
                        return lh_f2h((a > 65504.0f && a < INFINITY) ? __builtin_copysignf(65504.0f, v) : v);
                    };
                    const uint16_t h0 = first_part(x[2 * e]), h1 = first_part(x[2 * e + 1]);
                    hi.v[e] = (uint32_t)h0 | ((uint32_t)h1 << 16);
                    lo.v[e] = pack_h2(x[2 * e] - lh_h2f(h0), x[2 * e + 1] - lh_h2f(h1));
                }
                const uint32_t cell = ld_g * 16 + (c ^ (ld_g | ((ld_f & 1) << 2)));
                stage[(ld_f * 4 + j) * 64 + cell] = __builtin_bit_cast(f32x4, hi);
                stage[(ld_f * 4 + j + 2) * 64 + cell] = __builtin_bit_cast(f32x4, lo);
            }
        } else {
#pragma unroll
            for (int i = 0; i < NLD; i++) {
                const uint32_t m = RPI * i + ld_row, j = m >> 4, c = m & 15;
                stage[(ld_f * 4 + j) * 64 + ld_g * 16 + (c ^ (ld_g | ((ld_f & 1) << 2)))] = raw[i];
            }
        }
    };

    f32x4 acc[4][4];
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[t][j] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const SkinnyRaw (&raw)[4]) {
#pragma unroll
        for (int f = 0; f < NF; f++) {
            f16x8 bf[4];
#pragma unroll
            for (int j = 0; j < 4; j++) bf[j] = __builtin_bit_cast(f16x8, stage[(f * 4 + j) * 64 + g * 16 + (r ^ (g | ((f & 1) << 2)))]);
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const f16x8 a = skinny_fragment<FMT>(raw[t], f);
#pragma unroll
                for (int j = 0; j < 4; j++) acc[t][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, bf[j], acc[t][j], 0, 0, 0);
            }
        }
    };

    // two register sets for the codes, one for the activations, the unit after the one being multiplied always in flight;
    // the load past the end re-reads the last unit
    SkinnyRaw ra0[4], ra1[4];
    f32x4 rb[NLD];
    const uint32_t last = k_begin + (units_per_wave - 1) * UK;
    load_a(ra0, k_begin);
    load_b(rb, k_begin);
    park_b(rb);
    for (uint32_t u = 0; u < units_per_wave; u += 2) {
        const uint32_t k1 = k_begin + (u + 1) * UK, k2 = k_begin + (u + 2) * UK;
        load_a(ra1, k1 < last ? k1 : last);
        load_b(rb, k1 < last ? k1 : last);
        multiply(ra0);
        if (u + 1 < units_per_wave) {
            park_b(rb);
            load_a(ra0, k2 < last ? k2 : last);
            load_b(rb, k2 < last ? k2 : last);
            multiply(ra1);
            park_b(rb);
        }
    }
    // a wave's partial tiles go where its staging area was
#pragma unroll
    for (int t = 0; t < 4; t++)
#pragma unroll
        for (int j = 0; j < 4; j++) red[wave][t][j][lane] = make_float4(acc[t][j][0], acc[t][j][1], acc[t][j][2], acc[t][j][3]);
    __syncthreads();
    if constexpr (PAIR) {
        // wave w finishes gate tile (w & 1) with up tile (w & 1) + 2 for the activation groups 2 (w >> 1), 2 (w >> 1) + 1
        const int tp = wave & 1;
#pragma unroll
        for (int jj = 0; jj < 2; jj++) {
            const int j = (wave >> 1) * 2 + jj;
            float4 gt = red[0][tp][j][lane], up = red[0][tp + 2][j][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) {
                const float4 a = red[w][tp][j][lane], b = red[w][tp + 2][j][lane];
                gt.x += a.x; gt.y += a.y; gt.z += a.z; gt.w += a.w;
                up.x += b.x; up.y += b.y; up.z += b.z; up.w += b.w;
            }
            const uint32_t m = m0 + 16 * j + r;
            if (m >= M) continue;
            const float gv[4] = {gt.x, gt.y, gt.z, gt.w}, uv[4] = {up.x, up.y, up.z, up.w};
            uint16_t h[4];
#pragma unroll
            for (int i = 0; i < 4; i++) h[i] = lh_gelu_mul_h(lh_f2h(gv[i]), lh_f2h(uv[i]));
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(grp.C[0]) + (size_t)m * grp.N[0] + n0 + 16 * tp + 4 * g) =
                make_uint2((uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16));
        }
        return;
    }
    // wave w finishes tile w: D[row 4g + i][activation row r] of each group j
#pragma unroll
    for (int j = 0; j < (XF32 ? 2 : 4); j++) {
        float4 v = red[0][wave][j][lane];
#pragma unroll
        for (int w = 1; w < 4; w++) {
            const float4 o = red[w][wave][j][lane];
            v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
        }
        if constexpr (XF32) {   // the remainders' product
            float4 u = red[0][wave][j + 2][lane];
#pragma unroll
            for (int w = 1; w < 4; w++) {
                const float4 o = red[w][wave][j + 2][lane];
                u.x += o.x; u.y += o.y; u.z += o.z; u.w += o.w;
            }
            v.x += u.x; v.y += u.y; v.z += u.z; v.w += u.w;
        }
        const uint32_t m = m0 + 16 * j + r;
        if (m >= M) continue;
        const uint32_t nl = 16 * wave + 4 * g;
        if (partial) {
            const size_t cols = (size_t)gridDim.x * 64;
            *reinterpret_cast<float4*>(partial + ((size_t)blockIdx.z * M + m) * cols + (size_t)blockIdx.x * 64 + nl) = v;
        } else if constexpr (CDT == LH_F32) {
            *reinterpret_cast<float4*>(static_cast<float*>(C) + (size_t)m * N + n0 + nl) = v;
        } else {
            *reinterpret_cast<uint2*>(static_cast<uint16_t*>(C) + (size_t)m * N + n0 + nl) = make_uint2(pack_h2(v.x, v.y), pack_h2(v.z, v.w));
        }
    }
}

// Most activation rows the skinny kernel takes (256: a prefill chunk).  Beyond 64 rows
// every group of 64 gets workgroups of its own, which re-read the codes from L2 while the activation traffic grows with
// rows x weight rows; measured on a 256-row chunk of the layer bench: 197 -> 163 us per layer, no gain at 512 rows.
uint32_t skinny_max_m() {
    return 256u;
}

// ---- Q4_0, 2 .. 16 activation rows: the same workgroup shape with the operand roles swapped ----------------------------------------
// The reference's small-batch kernels multiply unrounded f32 weights (q - 8) d (matvec_quant.metal:595-798, 945-1038), so here
// the block scale stays out of the f16 operand: the weights enter as the B operand holding the exact integers q - 8 (columns
// = 16 weight rows), the activations as the A operand (rows = activation rows, read straight from global memory: they are
// shared by every tile and workgroup and stay in L1/L2), one MFMA covers exactly one 32-wide block, and its f32 sums are
// scaled by d and accumulated on the vector ALU.  A lane's D column is the weight row whose codes and scale it loaded itself,
// so no value crosses lanes.  Products (4-bit integer x f16) and block sums are exact to f32 rounding: closer to the
// reference's f32 arithmetic than the 16-bit activation fixed point of the matvec kernels.  Workgroup = 64 weight rows x a
// k range, four waves = quarters of the range, partial tiles added through LDS; same grid, split and partial-tile layout as
// matmul_skinny_kernel.
__device__ __forceinline__ uint32_t ld4_align2(const uint8_t* p) {
    typedef uint32_t __attribute__((aligned(2))) u32_a2;
    return *reinterpret_cast<const u32_a2*>(p);
}

template <int CDT>
__global__ __launch_bounds__(256, 2) void matmul_small_q4_kernel(const uint16_t* __restrict__ X, const uint8_t* __restrict__ W_one, void* __restrict__ C_one,
                                                                uint32_t M, uint32_t K, uint32_t N_one, float* __restrict__ partial,
                                                                uint32_t blocks_per_wave, GroupArgs grp) {
    __shared__ float4 red[4][4][64];                          // [wave][tile][lane]
    const uint8_t* __restrict__ W = W_one;
    void* __restrict__ C = C_one;
    uint32_t N = N_one, tile = blockIdx.x >> 1;
    if (grp.count) {
        const uint32_t gi = group_of_tile(grp, tile);
        W = grp.W[gi]; C = grp.C[gi]; N = grp.N[gi];
        tile -= grp.tile0[gi];
    }
    const uint32_t n0 = tile * BN + (blockIdx.x & 1) * 64;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t c = lane & 15, g = lane >> 4;
    const size_t row_bytes = (size_t)(K >> 5) * 18;
    const uint32_t b_begin = (blockIdx.z * 4 + wave) * blocks_per_wave;
    const uint8_t* wrow = W + (size_t)(n0 + c) * row_bytes + 4 * g;        // tile t starts 16 rows further on
    const size_t tile_bytes = 16 * row_bytes;
    const uint16_t* xrow = X + (size_t)(c < M ? c : M - 1) * K + 4 * g;    // rows past M repeat the last one and are never stored

    struct Raw { uint32_t w[4], d[4]; uint2 lo, hi; };
    auto load = [&](Raw& r, uint32_t b) {
        const size_t off = (size_t)b * 18;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint8_t* p = wrow + t * tile_bytes + off;
            r.w[t] = ld4_align2(p + 2);
            r.d[t] = *reinterpret_cast<const uint16_t*>(p - 4 * g);
        }
        r.lo = *reinterpret_cast<const uint2*>(xrow + (size_t)b * 32);
        r.hi = *reinterpret_cast<const uint2*>(xrow + (size_t)b * 32 + 16);
    };
    f32x4 acc[4];
#pragma unroll
    for (int t = 0; t < 4; t++) acc[t] = (f32x4){0.f, 0.f, 0.f, 0.f};
    auto multiply = [&](const Raw& r) {
        struct { uint32_t v[4]; } ax = {{r.lo.x, r.lo.y, r.hi.x, r.hi.y}};
        const f16x8 a = __builtin_bit_cast(f16x8, ax);
        const f16x2 zp = (f16x2){(_Float16)1032.0f, (_Float16)1032.0f};
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t lo = r.w[t] & 0x0F0F0F0Fu, hi = (r.w[t] >> 4) & 0x0F0F0F0Fu;
            const uint32_t p[4] = {__builtin_amdgcn_perm(0x64646464u, lo, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, lo, 0x04030402u),
                                   __builtin_amdgcn_perm(0x64646464u, hi, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, hi, 0x04030402u)};
            struct { uint32_t v[4]; } bx;
#pragma unroll
            for (int i = 0; i < 4; i++) bx.v[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(f16x2, p[i]) - zp);
            const f32x4 blk = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, __builtin_bit_cast(f16x8, bx), (f32x4){0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
            const float d = lh_h2f((uint16_t)r.d[t]);
#pragma unroll
            for (int i = 0; i < 4; i++) acc[t][i] = __builtin_fmaf(blk[i], d, acc[t][i]);
        }
    };
    Raw r0, r1;
    const uint32_t last = b_begin + blocks_per_wave - 1;
    load(r0, b_begin);
    for (uint32_t u = 0; u < blocks_per_wave; u += 2) {
        const uint32_t b1 = b_begin + u + 1, b2 = b_begin + u + 2;
        load(r1, b1 < last ? b1 : last);
        multiply(r0);
        if (u + 1 < blocks_per_wave) {
            load(r0, b2 < last ? b2 : last);
            multiply(r1);
        }
    }
#pragma unroll
    for (int t = 0; t < 4; t++) red[wave][t][lane] = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
    __syncthreads();
    // wave w finishes tile w: D[activation row 4g + i][weight row c]
    float4 v = red[0][wave][lane];
#pragma unroll
    for (int w = 1; w < 4; w++) {
        const float4 o = red[w][wave][lane];
        v.x += o.x; v.y += o.y; v.z += o.z; v.w += o.w;
    }
    const float vv[4] = {v.x, v.y, v.z, v.w};
    const uint32_t nl = 16 * wave + c;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const uint32_t m = 4 * g + i;
        if (m >= M) continue;
        if (partial) partial[((size_t)blockIdx.z * M + m) * ((size_t)gridDim.x * 64) + (size_t)blockIdx.x * 64 + nl] = vv[i];
        else store_elem<CDT>(C, (size_t)m * N + n0 + nl, vv[i]);
    }
}

// Fewest activation rows the skinny kernel takes; below it rows run as matvecs.  TQ2_0 from 2 rows:
// its f16 weights d (q - 1) are exact, so the results differ from the matvec kernels' only in the order of the f32 sums,
// and a 35-layer step over 16 lanes at 8k context went from 5.19 to 4.05 ms (8 lanes 4.14 to 3.59, 4 lanes 3.63 to 3.38).  Q4_0
// from 9 rows (the matvec kernels are as fast up to 8): up to 16 rows go to matmul_small_q4_kernel,
// which keeps the weights unrounded as the reference's small-batch kernels do (16 lanes 3.95 -> 3.80 ms); from 17 rows on
// the weights are the CPU path's f16 values, as in its matrix kernels.
// Fewest f32 activation rows the TQ2_0 skinny kernel takes; below it the rows run as matvecs.
// One layer's three TQ2_0 projections, weights cache resident: rows 34.3 / 42.2 / 47.4 us at 8 / 12 / 16 rows, this form
// 36.3 / 36.8 / 37.6 us.
uint32_t skinny_min_m_f32() {
    return 10u;
}
uint32_t skinny_min_m(int fmt) {
    return fmt == kTQ2 ? 2u : 9u;
}

// Most 64-row workgroups a launch of the skinny kernel may have (64 per CU).
uint32_t skinny_max_blocks(const lh_context* ctx) {
    return 64u * (uint32_t)ctx->cu_count;
}

// k splits of the skinny kernel over `workgroups` (64-row blocks x groups of 64 activation rows): enough workgroups for every CU, a whole number of units
// per wave, partial tiles within half the workspace.
uint32_t skinny_splits(const lh_context* ctx, uint32_t m, uint32_t workgroups, uint32_t units_per_wg) {
    uint32_t splits = 1;
    if (workgroups < (uint32_t)ctx->cu_count) {
        const uint32_t blocks = workgroups / ((m + 63) / 64);
        const uint64_t fit = (ctx->workspace_bytes / 2) / ((uint64_t)m * blocks * 64 * 4);
        const uint32_t want = (uint32_t)std::min<uint64_t>(((uint32_t)ctx->cu_count + workgroups - 1) / workgroups, fit);
        for (uint32_t c = 1; c <= want && c <= units_per_wg; c++) if (units_per_wg % c == 0) splits = c;
    }
    return splits;
}

// The skinny kernel when the shape allows it (f16 activations, 17 .. skinny_max_m() rows, whole 128-row tiles, at least one unit of k
// per wave; at most 64 workgroups per CU, far above any shape here); false
// leaves the launch to the LDS-tiled kernels.  With `keep` the f32 partial
// tiles (one split included) stay in the workspace for a consumer that sums them itself.
struct SkinnyPartials { const float* partial; uint32_t splits, cols; };
template <int FMT, int ADT>
bool try_skinny(lh_context* ctx, const void* A, const uint8_t* W, void* C, lh_dtype ct, uint32_t m, uint32_t k, uint32_t n, const ClipArgs& clip,
                const GroupArgs& grp, SkinnyPartials* keep = nullptr) {
    hipStream_t s = ctx->stream;
    const uint32_t tiles_n = grp.count ? grp.tile0[grp.count] : (n + BN - 1) / BN;
    if constexpr (FMT != kF16W && ADT == LH_F32) {
        // f32 activations as pairs of f16 rows: up to 32 rows.  TQ2_0 from skinny_min_m_f32() rows (below that the rows run as
        // matvecs); Q4_0 from 17 rows (up to 16 the matvec rows multiply unrounded weights, as the reference's kernels do).
        const uint32_t units = k / Skinny<FMT>::unit_k;
        const uint32_t min_m = FMT == kTQ2 ? skinny_min_m_f32() : (uint32_t)kMaxMultivecM + 1;
        if (!clip.enabled && !grp.count && !keep && m >= min_m && m <= 32 && n % BN == 0 && k % (4 * Skinny<FMT>::unit_k) == 0 &&
            2 * tiles_n <= skinny_max_blocks(ctx)) {
            const uint32_t blocks = 2 * tiles_n, per_wg = units / 4;
            const uint32_t splits = skinny_splits(ctx, m, blocks, per_wg);
            float* partial = splits > 1 ? static_cast<float*>(ctx->workspace) : nullptr;
            const dim3 grid(blocks, 1, splits);
            const uint16_t* X = static_cast<const uint16_t*>(A);
            if (ct == LH_F32) hipLaunchKernelGGL((matmul_skinny_kernel<FMT, LH_F32, false, true>), grid, dim3(256), 0, s, X, W, C, m, k, n, partial, per_wg / splits, grp);
            else hipLaunchKernelGGL((matmul_skinny_kernel<FMT, LH_F16, false, true>), grid, dim3(256), 0, s, X, W, C, m, k, n, partial, per_wg / splits, grp);
            if (splits > 1) {
                const uint32_t rgrid = (uint32_t)(((size_t)m * tiles_n * BN + 255) / 256);
                if (ct == LH_F32) hipLaunchKernelGGL((splitk_reduce_kernel<LH_F32>), dim3(rgrid), dim3(256), 0, s, partial, C, m, n, tiles_n, splits, clip, grp);
                else hipLaunchKernelGGL((splitk_reduce_kernel<LH_F16>), dim3(rgrid), dim3(256), 0, s, partial, C, m, n, tiles_n, splits, clip, grp);
            }
            return true;
        }
    }
    if constexpr (FMT != kF16W && ADT == LH_F16) {
        bool whole = grp.count ? true : n % BN == 0;          // every matrix fills its 128-row tiles
        for (uint32_t i = 0; i < grp.count; i++) whole = whole && grp.N[i] % BN == 0;
        const uint32_t units = k / Skinny<FMT>::unit_k;
        if (!clip.enabled && m >= skinny_min_m(FMT) && m <= skinny_max_m() && whole && k % (4 * Skinny<FMT>::unit_k) == 0 &&
            2 * tiles_n <= skinny_max_blocks(ctx) && (m <= 64 || 2 * tiles_n * ((m + 63) / 64) <= 8 * (uint32_t)ctx->cu_count)) {
            // k splits: enough workgroups for every CU, a whole number of units per wave, partial tiles within half the workspace
            const uint32_t blocks = 2 * tiles_n, per_wg = units / 4;
            const uint64_t fit = (ctx->workspace_bytes / 2) / ((uint64_t)m * blocks * 64 * 4);
            if (keep && fit == 0) return false;
            const uint32_t mgroups = (m + 63) / 64;
            const uint32_t splits = skinny_splits(ctx, m, blocks * mgroups, per_wg);
            float* partial = (splits > 1 || keep) ? static_cast<float*>(ctx->workspace) : nullptr;
            const dim3 grid(blocks, mgroups, splits);
            const uint16_t* X = static_cast<const uint16_t*>(A);
            if (FMT == kQ4 && m <= (uint32_t)kMaxMultivecM) {   // unrounded weights for the small batches (2 blocks per unit)
                if (ct == LH_F32) hipLaunchKernelGGL((matmul_small_q4_kernel<LH_F32>), grid, dim3(256), 0, s, X, W, C, m, k, n, partial, 2 * (per_wg / splits), grp);
                else hipLaunchKernelGGL((matmul_small_q4_kernel<LH_F16>), grid, dim3(256), 0, s, X, W, C, m, k, n, partial, 2 * (per_wg / splits), grp);
            } else if (ct == LH_F32) hipLaunchKernelGGL((matmul_skinny_kernel<FMT, LH_F32>), grid, dim3(256), 0, s, X, W, C, m, k, n, partial, per_wg / splits, grp);
            else hipLaunchKernelGGL((matmul_skinny_kernel<FMT, LH_F16>), grid, dim3(256), 0, s, X, W, C, m, k, n, partial, per_wg / splits, grp);
            if (keep) {
                *keep = SkinnyPartials{partial, splits, blocks * 64};
            } else if (splits > 1) {
                const uint32_t rgrid = (uint32_t)(((size_t)m * tiles_n * BN + 255) / 256);
                if (ct == LH_F32) hipLaunchKernelGGL((splitk_reduce_kernel<LH_F32>), dim3(rgrid), dim3(256), 0, s, partial, C, m, n, tiles_n, splits, clip, grp);
                else hipLaunchKernelGGL((splitk_reduce_kernel<LH_F16>), dim3(rgrid), dim3(256), 0, s, partial, C, m, n, tiles_n, splits, clip, grp);
            }
            return true;
        }
    }
    return false;
}

// The 64-row-tile kernel over `tiles_n` column tiles (one matrix, or the matrices of `grp` side by side).  Few output
// tiles (a decode batch of some tens of rows): k is split so that every CU gets a workgroup, at least two k steps per
// split, partial tiles within the lower half of the context workspace, summed by splitk_reduce_kernel.
template <int FMT, int ADT>
void launch_tiles64(lh_context* ctx, const void* A, const uint8_t* W, void* C, lh_dtype ct, uint32_t m, uint32_t k, uint32_t n, const ClipArgs& clip,
                    const GroupArgs& grp) {
    hipStream_t s = ctx->stream;
    const int cus = ctx->cu_count;
    const uint32_t nk = (k + BK - 1) / BK;
    const uint32_t tiles_n = grp.count ? grp.tile0[grp.count] : (n + BN - 1) / BN;
    if (try_skinny<FMT, ADT>(ctx, A, W, C, ct, m, k, n, clip, grp)) return;
    const uint64_t tiles64 = (uint64_t)tiles_n * ((m + 63) / 64);
    uint32_t splits = 1;
    if (tiles64 * 2 <= (uint64_t)cus && nk >= 4) {
        splits = (uint32_t)std::min<uint64_t>(nk / 2, ((uint64_t)cus + tiles64 - 1) / tiles64);
        const uint64_t fit = (ctx->workspace_bytes / 2) / ((uint64_t)m * tiles_n * BN * 4);
        splits = (uint32_t)std::min<uint64_t>(splits, fit);
    }
    const uint32_t steps = splits > 1 ? (nk + splits - 1) / splits : nk;
    if (splits > 1) splits = (nk + steps - 1) / steps;
    float* partial = splits > 1 ? static_cast<float*>(ctx->workspace) : nullptr;
    const dim3 grid(tiles_n, (m + 63) / 64, splits > 1 ? splits : 1);
    if (ct == LH_F32) hipLaunchKernelGGL((matmul_mfma_kernel<FMT, ADT, LH_F32, 64>), grid, dim3(256), 0, s, A, W, C, m, k, n, clip, partial, steps, grp);
    else hipLaunchKernelGGL((matmul_mfma_kernel<FMT, ADT, LH_F16, 64>), grid, dim3(256), 0, s, A, W, C, m, k, n, clip, partial, steps, grp);
    if (splits > 1) {
        const uint32_t rgrid = (uint32_t)(((size_t)m * tiles_n * BN + 255) / 256);
        if (ct == LH_F32) hipLaunchKernelGGL((splitk_reduce_kernel<LH_F32>), dim3(rgrid), dim3(256), 0, s, partial, C, m, n, tiles_n, splits, clip, grp);
        else hipLaunchKernelGGL((splitk_reduce_kernel<LH_F16>), dim3(rgrid), dim3(256), 0, s, partial, C, m, n, tiles_n, splits, clip, grp);
    }
}

template <int FMT, int ADT>
int launch_by_out(bool mfma, lh_context* ctx, const void* A, const uint8_t* W, void* C, lh_dtype ct, uint32_t m, uint32_t k, uint32_t n,
                  const ClipArgs& clip) {
    hipStream_t s = ctx->stream;
    const int cus = ctx->cu_count;
    if (mfma) {
        if (try_skinny<FMT, ADT>(ctx, A, W, C, ct, m, k, n, clip, GroupArgs{})) return LH_OK;
        // 128-row tiles reuse each dequantised weight tile twice as often; 64-row tiles when that would leave most CUs idle
        const uint64_t tiles128 = (uint64_t)((n + BN - 1) / BN) * ((m + 127) / 128);
        const bool big = m > 64 && tiles128 * 2 >= (uint64_t)cus;
        if constexpr (FMT != kF16W) {
            const size_t a16_bytes = (size_t)m * k * 2;
            if (big && k % BK == 0 && (ADT == LH_F16 || a16_bytes <= ctx->workspace_bytes)) {
                const uint16_t* a16 = static_cast<const uint16_t*>(A);
                const dim3 grid128((n + BN - 1) / BN, (m + 127) / 128);
                if constexpr (ADT == LH_BF16) {
                    // bf16 is converted by the staging waves on its way into LDS
                    if (ct == LH_F32) hipLaunchKernelGGL((matmul_mfma128_kernel<FMT, LH_F32, true, 8>), grid128, dim3(768), 0, s, a16, W, C, m, k, n);
                    else hipLaunchKernelGGL((matmul_mfma128_kernel<FMT, LH_F16, true, 8>), grid128, dim3(768), 0, s, a16, W, C, m, k, n);
                    return LH_OK;
                }
                if constexpr (ADT != LH_F16) {   // f32: one pass over the activations instead of a conversion in every column tile
                    const size_t n8 = (size_t)m * k / 8;
                    hipLaunchKernelGGL((convert_to_f16_kernel<ADT>), dim3((uint32_t)((n8 + 255) / 256)), dim3(256), 0, s, A, (uint16_t*)ctx->workspace, n8);
                    a16 = static_cast<const uint16_t*>(ctx->workspace);
                }
                if (ct == LH_F32) hipLaunchKernelGGL((matmul_mfma128_kernel<FMT, LH_F32, false, 8>), grid128, dim3(768), 0, s, a16, W, C, m, k, n);
                else hipLaunchKernelGGL((matmul_mfma128_kernel<FMT, LH_F16, false, 8>), grid128, dim3(768), 0, s, a16, W, C, m, k, n);
                return LH_OK;
            }
        }
        const uint32_t nk = (k + BK - 1) / BK;
        if (tiles128 >= 2ull * (uint64_t)cus) {
            const dim3 grid((n + BN - 1) / BN, (m + 127) / 128);
            if (ct == LH_F32) hipLaunchKernelGGL((matmul_mfma_kernel<FMT, ADT, LH_F32, 128>), grid, dim3(256), 0, s, A, W, C, m, k, n, clip, (float*)nullptr, nk, GroupArgs{});
            else hipLaunchKernelGGL((matmul_mfma_kernel<FMT, ADT, LH_F16, 128>), grid, dim3(256), 0, s, A, W, C, m, k, n, clip, (float*)nullptr, nk, GroupArgs{});
        } else {
            launch_tiles64<FMT, ADT>(ctx, A, W, C, ct, m, k, n, clip, GroupArgs{});
        }
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
int launch_by_in(bool mfma, lh_context* ctx, const void* A, lh_dtype at, const uint8_t* W, void* C, lh_dtype ct, uint32_t m, uint32_t k,
                 uint32_t n, const ClipArgs& clip) {
    switch (at) {
        case LH_F32: return launch_by_out<FMT, LH_F32>(mfma, ctx, A, W, C, ct, m, k, n, clip);
        case LH_BF16: return launch_by_out<FMT, LH_BF16>(mfma, ctx, A, W, C, ct, m, k, n, clip);
        default: return launch_by_out<FMT, LH_F16>(mfma, ctx, A, W, C, ct, m, k, n, clip);
    }
}

// kind: kQ4 / kTQ2 / kF16W. `force_multivec` is the multivec_nt_* entry (m <= 16 enforced by the caller).
int matmul_dispatch(lh_batch* batch, const char* op, int kind, const lh_buffer* input, lh_dtype at, const lh_buffer* weight,
                    lh_buffer* output, lh_dtype ct, uint32_t m, uint32_t k, uint32_t n, bool force_multivec,
                    const ClipArgs& clip = ClipArgs{nullptr, 0.f, 0.f, 0.f, 0.f, 0u}) {
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
    if (!mfma && !force_multivec && at == LH_F16 && m >= skinny_min_m(kind)) {   // a small batch the decode-batch kernel takes
        const uint8_t* Ws = (const uint8_t*)weight->ptr;
        const bool took = kind == kQ4 ? try_skinny<kQ4, LH_F16>(batch->ctx, input->ptr, Ws, output->ptr, ct, m, k, n, clip, GroupArgs{})
                                      : try_skinny<kTQ2, LH_F16>(batch->ctx, input->ptr, Ws, output->ptr, ct, m, k, n, clip, GroupArgs{});
        if (took) {
            int r = lh_check_launch(op);
            if (r == LH_OK) batch->dispatch_count++;
            return r;
        }
    }
    if (!mfma && !force_multivec && at == LH_F32 && kind == kTQ2 && m >= skinny_min_m_f32()) {   // f32 rows as pairs of f16 rows
        if (try_skinny<kTQ2, LH_F32>(batch->ctx, input->ptr, (const uint8_t*)weight->ptr, output->ptr, ct, m, k, n, clip, GroupArgs{})) {
            int r = lh_check_launch(op);
            if (r == LH_OK) batch->dispatch_count++;
            return r;
        }
    }
    if (!mfma) {
        // up to 16 activation rows: m matvecs against the same matrix in one launch of the M = 1 kernels (the weights
        // of one call stay cache resident between the rows); shapes they do not take fall through to multivec_kernel
        const int rr = lh_matvec_rows(batch, kind == kQ4 ? LH_Q4_0 : LH_TQ2_0, m, weight, input, at, output, ct, n, k, op);
        if (rr != -1) {
            if (rr == LH_OK) batch->dispatch_count++;
            return rr;
        }
    }
    const uint8_t* W = (const uint8_t*)weight->ptr;
    if (kind == kQ4) launch_by_in<kQ4>(mfma, batch->ctx, input->ptr, at, W, output->ptr, ct, m, k, n, clip);
    else if (kind == kTQ2) launch_by_in<kTQ2>(mfma, batch->ctx, input->ptr, at, W, output->ptr, ct, m, k, n, clip);
    else launch_by_in<kF16W>(true, batch->ctx, input->ptr, at, W, output->ptr, ct, m, k, n, clip);
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
int lh_matmul_nt_quant_norm_into(lh_batch* b, lh_quant fmt, const lh_buffer* in, const lh_buffer* w, uint32_t m, uint32_t k, uint32_t n,
                                 const lh_buffer* norm_weight, const lh_buffer* residual, lh_buffer* out, float eps, int apply_scale,
                                 float scale, const lh_buffer* norm2_weight, lh_buffer* out2) {
    const char* op = fmt == LH_Q4_0 ? "matmul_nt_q4_0 + rms_norm" : "matmul_nt_tq2_0 + rms_norm";
    if (!b) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matmul_nt_quant: unknown weight format %d", (int)fmt);
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256;
    if (k % blk != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: k %u not /%u", op, k, blk);
    if (m == 0 || n == 0 || k == 0) return LH_OK;
    if (!lh_norm_fused_supported(n)) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: n %u must be a multiple of 8, at most 8192", op, n);
    if ((norm2_weight == nullptr) != (out2 == nullptr)) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: the second norm needs both its weight and its output", op);
    lh_context* ctx = b->ctx;
    const size_t wbytes = fmt == LH_Q4_0 ? (size_t)n * (k / 32) * 18 : (size_t)n * (k / 256) * 66;
    LH_NEED(in, (size_t)m * k * 2, op, "input");
    LH_NEED(w, wbytes, op, "weight");
    LH_NEED(norm_weight, (size_t)n * 2, op, "norm weight");
    LH_NEED(out, (size_t)m * n * 2, op, "output");
    if (residual) LH_NEED(residual, (size_t)m * n * 2, op, "residual");
    if (norm2_weight) { LH_NEED(norm2_weight, (size_t)n * 2, op, "second norm weight"); LH_NEED(out2, (size_t)m * n * 2, op, "second output"); }
    const uintptr_t align = (uintptr_t)in->ptr | (uintptr_t)norm_weight->ptr | (uintptr_t)out->ptr | (uintptr_t)(residual ? residual->ptr : nullptr) |
                            (uintptr_t)(norm2_weight ? norm2_weight->ptr : nullptr) | (uintptr_t)(out2 ? out2->ptr : nullptr);
    LH_REQUIRE((align & 15) == 0, "%s: buffers must be 16-byte aligned", op);
    LH_REQUIRE(((uintptr_t)w->ptr & 1) == 0, "%s: weight must be 2-byte aligned", op);

    LhNormFused a{};
    a.w = (const uint16_t*)norm_weight->ptr; a.res = residual ? (const uint16_t*)residual->ptr : nullptr; a.out = (uint16_t*)out->ptr;
    a.dim = n; a.rows = m; a.eps = eps; a.apply_scale = apply_scale ? 1u : 0u; a.scale = scale;
    a.w2 = norm2_weight ? (const uint16_t*)norm2_weight->ptr : nullptr; a.out2 = out2 ? (uint16_t*)out2->ptr : nullptr;
    const ClipArgs none{nullptr, 0.f, 0.f, 0.f, 0.f, 0u};
    SkinnyPartials kept{nullptr, 0, 0};
    const uint8_t* W = (const uint8_t*)w->ptr;
    const bool skinny = fmt == LH_Q4_0 ? try_skinny<kQ4, LH_F16>(ctx, in->ptr, W, nullptr, LH_F16, m, k, n, none, GroupArgs{}, &kept)
                                       : try_skinny<kTQ2, LH_F16>(ctx, in->ptr, W, nullptr, LH_F16, m, k, n, none, GroupArgs{}, &kept);
    if (skinny) {
        a.partial = kept.partial; a.splits = kept.splits; a.part_rows = m; a.part_cols = kept.cols;
    } else {
        // any other shape: the product as matmul_nt_quant_typed_into computes it, into the third quarter of the workspace
        // (the lower half holds partial tiles, the top quarter descriptor tables), then the same norm kernel over those rows
        const size_t half = ctx->workspace_bytes / 2, quarter = ctx->workspace_bytes / 4;
        if ((size_t)m * n * 2 > quarter) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: %u x %u product exceeds the %zu-byte staging area", op, m, n, quarter);
        lh_buffer tmp{};
        tmp.ptr = static_cast<uint8_t*>(ctx->workspace) + half; tmp.len = quarter; tmp.ctx = ctx;
        const uint32_t d0 = b->dispatch_count;
        int r = matmul_dispatch(b, op, fmt == LH_Q4_0 ? kQ4 : kTQ2, in, LH_F16, w, &tmp, LH_F16, m, k, n, false);
        if (r != LH_OK) return r;
        b->dispatch_count = d0;
        a.in = (const uint16_t*)tmp.ptr;
    }
    lh_launch_norm_fused(ctx->stream, a);
    int r = lh_check_launch(op);
    if (r == LH_OK) b->dispatch_count++;
    return r;
}
int lh_matmul_nt_quant_gelu_mul_strided_into(lh_batch* b, lh_quant fmt, const lh_buffer* in, const lh_buffer* w, uint32_t m, uint32_t k, uint32_t n,
                                             const lh_buffer* gate_rows, uint32_t row_stride, uint32_t row_offset, lh_buffer* out) {
    const char* op = fmt == LH_Q4_0 ? "matmul_nt_q4_0 + gelu_mul_strided" : "matmul_nt_tq2_0 + gelu_mul_strided";
    if (!b) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matmul_nt_quant: unknown weight format %d", (int)fmt);
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256;
    if (k % blk != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: k %u not /%u", op, k, blk);
    if (m == 0 || n == 0 || k == 0) return LH_OK;
    if (((n | row_stride | row_offset) & 7) != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: n, row_stride and row_offset must be multiples of 8", op);
    lh_context* ctx = b->ctx;
    const size_t wbytes = fmt == LH_Q4_0 ? (size_t)n * (k / 32) * 18 : (size_t)n * (k / 256) * 66;
    LH_NEED(in, (size_t)m * k * 2, op, "input");
    LH_NEED(w, wbytes, op, "weight");
    LH_NEED(gate_rows, ((size_t)(m - 1) * row_stride + row_offset + n) * 2, op, "gate rows");
    LH_NEED(out, (size_t)m * n * 2, op, "output");
    LH_REQUIRE((((uintptr_t)in->ptr | (uintptr_t)gate_rows->ptr | (uintptr_t)out->ptr) & 15) == 0, "%s: buffers must be 16-byte aligned", op);
    LH_REQUIRE(((uintptr_t)w->ptr & 1) == 0, "%s: weight must be 2-byte aligned", op);
    const ClipArgs none{nullptr, 0.f, 0.f, 0.f, 0.f, 0u};
    SkinnyPartials kept{nullptr, 0, 0};
    const uint8_t* W = (const uint8_t*)w->ptr;
    const bool skinny = fmt == LH_Q4_0 ? try_skinny<kQ4, LH_F16>(ctx, in->ptr, W, nullptr, LH_F16, m, k, n, none, GroupArgs{}, &kept)
                                       : try_skinny<kTQ2, LH_F16>(ctx, in->ptr, W, nullptr, LH_F16, m, k, n, none, GroupArgs{}, &kept);
    if (skinny) {
        lh_launch_gelu_mul_strided(ctx->stream, nullptr, kept.partial, kept.splits, kept.cols, gate_rows->ptr, row_stride, row_offset, out->ptr, n, m);
    } else {
        const size_t half = ctx->workspace_bytes / 2, quarter = ctx->workspace_bytes / 4;
        if ((size_t)m * n * 2 > quarter) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: %u x %u product exceeds the %zu-byte staging area", op, m, n, quarter);
        lh_buffer tmp{};
        tmp.ptr = static_cast<uint8_t*>(ctx->workspace) + half; tmp.len = quarter; tmp.ctx = ctx;
        const uint32_t d0 = b->dispatch_count;
        int r = matmul_dispatch(b, op, fmt == LH_Q4_0 ? kQ4 : kTQ2, in, LH_F16, w, &tmp, LH_F16, m, k, n, false);
        if (r != LH_OK) return r;
        b->dispatch_count = d0;
        lh_launch_gelu_mul_strided(ctx->stream, tmp.ptr, nullptr, 0, 0, gate_rows->ptr, row_stride, row_offset, out->ptr, n, m);
    }
    int r = lh_check_launch(op);
    if (r == LH_OK) b->dispatch_count++;
    return r;
}
int lh_matmul_nt_quant_grouped_into(lh_batch* b, lh_quant fmt, uint32_t count, const lh_buffer* in, const lh_buffer* const* ws,
                                    lh_buffer* const* outs, const uint32_t* ns, uint32_t m, uint32_t k) {
    const char* op = fmt == LH_Q4_0 ? "matmul_nt_q4_0 (grouped)" : "matmul_nt_tq2_0 (grouped)";
    if (!b) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matmul_nt_quant: unknown weight format %d", (int)fmt);
    if (count == 0 || m == 0 || k == 0) return LH_OK;
    if (count > 4) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: at most 4 matrices share one launch, got %u", op, count);
    if (!in || !ws || !outs || !ns) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null argument", op);
    const int kind = fmt == LH_Q4_0 ? kQ4 : kTQ2;
    lh_context* ctx = b->ctx;
    // The shapes the 64-row-tile kernel takes (some tens to a few hundred rows, not enough 128-row tiles to fill the
    // chip) go out as one launch; everything else as the separate calls this entry point stands for.
    uint64_t tiles_n = 0;
    for (uint32_t i = 0; i < count; i++) tiles_n += (ns[i] + BN - 1) / BN;
    const uint64_t tiles128 = tiles_n * ((m + 127) / 128);
    const bool small = m <= (uint32_t)kMaxMultivecM;          // then only the decode-batch kernel may take the group as one launch
    const bool together = (!small || m >= skinny_min_m(kind)) && !(m > 64 && tiles128 * 2 >= (uint64_t)ctx->cu_count);
    if (!together) {
        for (uint32_t i = 0; i < count; i++) {
            int r = matmul_dispatch(b, op, kind, in, LH_F16, ws[i], outs[i], LH_F16, m, k, ns[i], false);
            if (r != LH_OK) return r;
        }
        return LH_OK;
    }
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256;
    if (k % blk != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: k %u not /%u", op, k, blk);
    LH_NEED(in, (size_t)m * k * 2, op, "input");
    LH_REQUIRE(((uintptr_t)in->ptr & 15) == 0, "%s: input must be 16-byte aligned", op);
    GroupArgs grp{};
    grp.count = count;
    uint32_t tile = 0;
    for (uint32_t i = 0; i < count; i++) {
        if (ns[i] == 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: matrix %u has no rows", op, i);
        const size_t wbytes = fmt == LH_Q4_0 ? (size_t)ns[i] * (k / 32) * 18 : (size_t)ns[i] * (k / 256) * 66;
        LH_NEED(ws[i], wbytes, op, "weight");
        LH_NEED(outs[i], (size_t)m * ns[i] * 2, op, "output");
        LH_REQUIRE(((uintptr_t)ws[i]->ptr & 1) == 0, "%s: weight must be 2-byte aligned", op);
        grp.W[i] = (const uint8_t*)ws[i]->ptr; grp.C[i] = outs[i]->ptr; grp.N[i] = ns[i];
        grp.tile0[i] = tile;
        tile += (ns[i] + BN - 1) / BN;
    }
    for (uint32_t i = count; i <= 4; i++) grp.tile0[i] = tile;
    const ClipArgs none{nullptr, 0.f, 0.f, 0.f, 0.f, 0u};
    if (small) {
        const bool took = fmt == LH_Q4_0 ? try_skinny<kQ4, LH_F16>(ctx, in->ptr, grp.W[0], grp.C[0], LH_F16, m, k, grp.N[0], none, grp)
                                         : try_skinny<kTQ2, LH_F16>(ctx, in->ptr, grp.W[0], grp.C[0], LH_F16, m, k, grp.N[0], none, grp);
        if (!took) {
            for (uint32_t i = 0; i < count; i++) {
                int r = matmul_dispatch(b, op, kind, in, LH_F16, ws[i], outs[i], LH_F16, m, k, ns[i], false);
                if (r != LH_OK) return r;
            }
            return LH_OK;
        }
    } else if (fmt == LH_Q4_0) launch_tiles64<kQ4, LH_F16>(ctx, in->ptr, grp.W[0], grp.C[0], LH_F16, m, k, grp.N[0], none, grp);
    else launch_tiles64<kTQ2, LH_F16>(ctx, in->ptr, grp.W[0], grp.C[0], LH_F16, m, k, grp.N[0], none, grp);
    int r = lh_check_launch(op);
    if (r == LH_OK) b->dispatch_count++;
    return r;
}

int lh_matmul_nt_qkv_prepare_rows_into(lh_batch* b, lh_quant fmt, const lh_buffer* in, const lh_buffer* w_q, const lh_buffer* w_k,
                                       const lh_buffer* w_v, uint32_t k_dim, lh_buffer* q, lh_buffer* k, lh_buffer* v, const lh_buffer* q_norm,
                                       const lh_buffer* k_norm, const lh_buffer* levels, const lh_buffer* signs, lh_buffer* rq, lh_buffer* k_codes,
                                       lh_buffer* k_norms, lh_buffer* v_codes, lh_buffer* v_norms, const lh_buffer* positions, uint32_t head_dim,
                                       uint32_t n_q_heads, uint32_t n_kv_heads, uint32_t rows, float eps, uint32_t start_position, float theta,
                                       float partial_rotary_factor, uint32_t bits, uint32_t ring_capacity, uint32_t lane_capacity) {
    const char* op = fmt == LH_Q4_0 ? "matmul_nt_q4_0 (Q, K, V) + decode_qkv_prepare" : "matmul_nt_tq2_0 (Q, K, V) + decode_qkv_prepare";
    if (!b) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matmul_nt_quant: unknown weight format %d", (int)fmt);
    if (!in || !w_q || !w_k || !w_v || !q || !k || !v || n_q_heads == 0 || n_kv_heads == 0)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: needs the query, key and value projections and their outputs (a layer that shares its cache "
                                                "takes the separate entry points)", op);
    const LhPrepareRows a{q, k, v, q_norm, k_norm, levels, signs, rq, k_codes, k_norms, v_codes, v_norms, positions, head_dim, n_q_heads, n_kv_heads,
                          rows, eps, start_position, theta, partial_rotary_factor, bits, ring_capacity, lane_capacity};
    int r = lh_prepare_rows_launch(b, a, nullptr, 0, 0, true);   // the second half's arguments, before anything is launched
    if (r != LH_OK) return r;
    if (rows == 0 || k_dim == 0) return LH_OK;
    const lh_buffer* const ws[3] = {w_q, w_k, w_v};
    lh_buffer* const outs[3] = {q, k, v};
    const uint32_t ns[3] = {n_q_heads * head_dim, n_kv_heads * head_dim, n_kv_heads * head_dim};
    lh_context* ctx = b->ctx;
    const int kind = fmt == LH_Q4_0 ? kQ4 : kTQ2;
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256, m = rows;
    // The shapes that lh_matmul_nt_quant_grouped_into sends to the decode-batch kernel as one launch can leave their partial
    // tiles to the preparation; every other shape runs as that entry point followed by the preparation.
    uint64_t tiles_n = 0;
    bool whole = true;
    for (uint32_t i = 0; i < 3; i++) { tiles_n += (ns[i] + BN - 1) / BN; whole = whole && ns[i] % BN == 0; }
    const uint64_t tiles128 = tiles_n * ((m + 127) / 128);
    const bool small = m <= (uint32_t)kMaxMultivecM;
    const bool together = (!small || m >= skinny_min_m(kind)) && !(m > 64 && tiles128 * 2 >= (uint64_t)ctx->cu_count);
    bool fused = false;
    SkinnyPartials kept{nullptr, 0, 0};
    if (together && whole && k_dim % blk == 0 && ((uintptr_t)in->ptr & 15) == 0 && in->len >= (size_t)m * k_dim * 2) {
        GroupArgs grp{};
        grp.count = 3;
        uint32_t tile = 0;
        bool fits = true;
        for (uint32_t i = 0; i < 3; i++) {
            const size_t wbytes = fmt == LH_Q4_0 ? (size_t)ns[i] * (k_dim / 32) * 18 : (size_t)ns[i] * (k_dim / 256) * 66;
            fits = fits && ws[i]->len >= wbytes && ((uintptr_t)ws[i]->ptr & 1) == 0;
            grp.W[i] = (const uint8_t*)ws[i]->ptr; grp.C[i] = outs[i]->ptr; grp.N[i] = ns[i];
            grp.tile0[i] = tile;
            tile += ns[i] / BN;
        }
        for (uint32_t i = 3; i <= 4; i++) grp.tile0[i] = tile;
        const ClipArgs none{nullptr, 0.f, 0.f, 0.f, 0.f, 0u};
        if (fits)
            fused = fmt == LH_Q4_0 ? try_skinny<kQ4, LH_F16>(ctx, in->ptr, grp.W[0], grp.C[0], LH_F16, m, k_dim, grp.N[0], none, grp, &kept)
                                   : try_skinny<kTQ2, LH_F16>(ctx, in->ptr, grp.W[0], grp.C[0], LH_F16, m, k_dim, grp.N[0], none, grp, &kept);
    }
    if (fused) {
        r = lh_check_launch(op);
        if (r != LH_OK) return r;
        return lh_prepare_rows_launch(b, a, kept.partial, kept.splits, kept.cols);
    }
    r = lh_matmul_nt_quant_grouped_into(b, fmt, 3, in, ws, outs, ns, rows, k_dim);   // reports what is wrong with the product's arguments
    return r != LH_OK ? r : lh_prepare_rows_launch(b, a, nullptr, 0, 0);
}

int lh_matmul_nt_quant_gelu_mul_into(lh_batch* b, lh_quant fmt, const lh_buffer* in, const lh_buffer* w_gate, const lh_buffer* w_up,
                                     lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    const char* op = fmt == LH_Q4_0 ? "matmul_nt_q4_0 + gelu_mul" : "matmul_nt_tq2_0 + gelu_mul";
    if (!b) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matmul_nt_quant: unknown weight format %d", (int)fmt);
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256;
    if (k % blk != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: k %u not /%u", op, k, blk);
    if (m == 0 || n == 0 || k == 0) return LH_OK;
    lh_context* ctx = b->ctx;
    const size_t wbytes = fmt == LH_Q4_0 ? (size_t)n * (k / 32) * 18 : (size_t)n * (k / 256) * 66;
    LH_NEED(in, (size_t)m * k * 2, op, "input");
    LH_NEED(w_gate, wbytes, op, "gate weight");
    LH_NEED(w_up, wbytes, op, "up weight");
    LH_NEED(out, (size_t)m * n * 2, op, "output");
    LH_REQUIRE(((uintptr_t)in->ptr & 15) == 0 && ((uintptr_t)out->ptr & 15) == 0, "%s: input and output must be 16-byte aligned", op);
    LH_REQUIRE((((uintptr_t)w_gate->ptr | (uintptr_t)w_up->ptr) & 1) == 0, "%s: weights must be 2-byte aligned", op);
    const uint32_t unit_k = fmt == LH_Q4_0 ? Skinny<kQ4>::unit_k : Skinny<kTQ2>::unit_k;
    const uint32_t blocks = n / 32;
    // one launch where the grouped product of the pair takes the skinny kernel without a k split (split products need
    // their sums before the gelu); the same workgroup count and k ranges, hence the same sums
    const uint32_t mgroups = (m + 63) / 64;
    if (m >= skinny_min_m(fmt == LH_Q4_0 ? kQ4 : kTQ2) && (fmt != LH_Q4_0 || m > (uint32_t)kMaxMultivecM) && m <= skinny_max_m() &&
        n % BN == 0 && k % (4 * unit_k) == 0 &&
        blocks <= skinny_max_blocks(ctx) && (m <= 64 || blocks * mgroups <= 8 * (uint32_t)ctx->cu_count) &&
        skinny_splits(ctx, m, blocks * mgroups, k / unit_k / 4) == 1) {
        GroupArgs grp{};
        grp.count = 2;
        grp.W[0] = (const uint8_t*)w_gate->ptr; grp.W[1] = (const uint8_t*)w_up->ptr;
        grp.C[0] = out->ptr; grp.N[0] = n;
        const uint16_t* X = static_cast<const uint16_t*>(in->ptr);
        const uint32_t per_wave = k / unit_k / 4;
        if (fmt == LH_Q4_0) hipLaunchKernelGGL((matmul_skinny_kernel<kQ4, LH_F16, true>), dim3(blocks, mgroups), dim3(256), 0, ctx->stream, X, grp.W[0], out->ptr, m, k, n, (float*)nullptr, per_wave, grp);
        else hipLaunchKernelGGL((matmul_skinny_kernel<kTQ2, LH_F16, true>), dim3(blocks, mgroups), dim3(256), 0, ctx->stream, X, grp.W[0], out->ptr, m, k, n, (float*)nullptr, per_wave, grp);
    } else {
        // any other shape: the two products as matmul_nt_quant_grouped_into computes them, staged in the third quarter of the
        // workspace, then gelu_mul
        const size_t half = ctx->workspace_bytes / 2, quarter = ctx->workspace_bytes / 4, each = (((size_t)m * n * 2) + 255) & ~(size_t)255;
        if (2 * each > quarter) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: two %u x %u products exceed the %zu-byte staging area", op, m, n, quarter);
        lh_buffer tg{}, tu{};
        tg.ptr = static_cast<uint8_t*>(ctx->workspace) + half; tg.len = each; tg.ctx = ctx;
        tu.ptr = static_cast<uint8_t*>(ctx->workspace) + half + each; tu.len = each; tu.ctx = ctx;
        const lh_buffer* ws[2] = {w_gate, w_up};
        lh_buffer* outs[2] = {&tg, &tu};
        const uint32_t ns[2] = {n, n};
        const uint32_t d0 = b->dispatch_count;
        int r = lh_matmul_nt_quant_grouped_into(b, fmt, 2, in, ws, outs, ns, m, k);
        if (r != LH_OK) return r;
        b->dispatch_count = d0;
        lh_launch_gelu_mul(ctx->stream, tg.ptr, tu.ptr, out->ptr, m * n);
    }
    int r = lh_check_launch(op);
    if (r == LH_OK) b->dispatch_count++;
    return r;
}

int lh_matmul_nt_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, lh_buffer* out, uint32_t m, uint32_t k, uint32_t n) {
    return matmul_dispatch(b, "matmul_nt", kF16W, in, LH_F16, w, out, LH_F16, m, k, n, false);
}
int lh_clipped_linear_tiled_nt_into(lh_batch* b, const lh_buffer* in, const lh_buffer* w, const lh_buffer* bias, lh_buffer* out, uint32_t m,
                                    uint32_t k, uint32_t n, float input_min, float input_max, float output_min, float output_max) {
    if (bias) LH_NEED(bias, (size_t)n * 2, "clipped_linear_tiled_nt", "bias");
    const ClipArgs clip{bias ? (const uint16_t*)bias->ptr : nullptr, input_min, input_max, output_min, output_max, 1u};
    return matmul_dispatch(b, "clipped_linear_tiled_nt", kF16W, in, LH_F16, w, out, LH_F16, m, k, n, false, clip);
}

}  // extern "C"
