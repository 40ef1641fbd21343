// Fused dequant matvec for GGUF Q4_0 / TQ2_0 weights at M = 1 (decode).
//
// Stands in for shaders/matvec_quant.metal:65-155 (matvec_q4_0*), 173-312
// (matvec_tq2_0*), 314-387 (matvec_tq2_0_soa) and their dispatch in
// local-metal/src/kernels.rs:5588-6038.
//
// Design (gfx950, wave64):
//  * The weight stream is the only HBM traffic that matters.  A "unit" is 64
//    weights: for TQ2_0 one 16-byte quarter of a 66-byte block, for Q4_0 a pair
//    of 18-byte blocks (36 bytes, dword aligned).  Each lane owns one unit
//    column of a row and loads it with 128-bit loads; consecutive lanes cover a
//    contiguous span, so a wave reads 1-2.3 KB of consecutive bytes per load.
//  * The activation vector is converted once per workgroup to block fixed point
//    (per weight block: a float scale and 16- or 24-bit integers split into
//    signed 8-bit limbs) and kept in registers for the lane's unit column, so
//    the inner product is exact integer arithmetic on v_dot4_i32_i8:
//        y = sum_blocks d_b * s_b * (sum_i q_i n_i  -  zp * sum_i n_i)
//    2-bit / 4-bit codes are isolated with one AND per four weights; no
//    per-weight shift, convert or float multiply.
//  * Row sums use DPP / swizzle butterflies inside the wave (fixed pairing
//    order, so results are bit-reproducible run to run).
#include "common.hpp"
#include "xquant.hpp"
#include <cstdlib>

namespace {

constexpr int kWG = 256;          // threads per workgroup (4 waves)
constexpr int kWaves = kWG / 64;
constexpr uint32_t kMaxFastCols = 16384;  // 4 unit columns per lane at most
constexpr size_t kMaxDynamicLds = 96 * 1024;   // what launch_typed raises a kernel's dynamic LDS limit to

struct MatvecProblem {
    const uint8_t* matrix;
    const void* vector;
    void* output;
};
// The problem that travels in the kernel arguments.  With a descriptor table absent and count > 1, problem i is this
// one with its vector and output advanced by i strides (the rows of a small activation batch against one matrix).
struct MatvecBase {
    MatvecProblem p;
    uint32_t xstride, ystride;   // bytes
    uint64_t mstride = 0;        // bytes between the matrices of consecutive problems (0: one matrix for all of them)
    // A pair of unrelated problems (K and V, gate and up) also travels here, so the common grouped launch
    // needs no descriptor upload ahead of it.
    MatvecProblem second = {nullptr, nullptr, nullptr};
    uint32_t pair = 0;
    XPrologue pro = {kXProNone, nullptr, 0.0f};   // applied to every problem's vector while it is staged
};

// ---- per-lane activation registers for one unit column -------------------------
template <int FMT, int L>
struct UnitX {
    uint32_t xl[L][4][4];   // [limb][run of 16 elements][dword of 4 elements]
    float scale[2];         // Q4_0: the unit's two blocks; TQ2_0: [0] only (pre-divided by 16)
    int nsum[2];            // zero-point term: Q4_0 8*sum(n) per block; TQ2_0 16*sum(n) of the unit
};

template <int FMT, int L>
__device__ __forceinline__ void load_unit_x(UnitX<FMT, L>& ux, uint32_t ucol, uint32_t K, const uint32_t* xq, const float* xs) {
    const uint32_t kq = K >> 2;
#pragma unroll
    for (int r = 0; r < 4; r++) {
        uint32_t eb;
        if constexpr (FMT == LH_TQ2_0) {
            const uint32_t b = ucol >> 2, a = ucol & 3;
            eb = b * 256 + (a >> 1) * 128 + r * 32 + (a & 1) * 16;   // shaders/matvec_quant.metal:15-17
        } else {
            eb = ucol * 64 + r * 16;                                   // low nibbles then high nibbles of each block
        }
#pragma unroll
        for (int l = 0; l < L; l++) {
            const uint4 q = *reinterpret_cast<const uint4*>(&xq[l * kq + (eb >> 2)]);
            ux.xl[l][r][0] = q.x; ux.xl[l][r][1] = q.y; ux.xl[l][r][2] = q.z; ux.xl[l][r][3] = q.w;
        }
    }
    int s[4];
#pragma unroll
    for (int r = 0; r < 4; r++) {
        int tot = 0;
#pragma unroll
        for (int l = L - 1; l >= 0; l--) {
            int t = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) t = __builtin_amdgcn_sdot4((int)ux.xl[l][r][k], 0x01010101, t, false);
            tot = (tot << 8) + t;
        }
        s[r] = tot;
    }
    if constexpr (FMT == LH_TQ2_0) {
        ux.scale[0] = xs[ucol >> 2] * 0.0625f;
        ux.scale[1] = 0.0f;
        ux.nsum[0] = (s[0] + s[1] + s[2] + s[3]) << 4;
        ux.nsum[1] = 0;
    } else {
        ux.scale[0] = xs[2 * ucol];
        ux.scale[1] = xs[2 * ucol + 1];
        ux.nsum[0] = (s[0] + s[1]) << 3;
        ux.nsum[1] = (s[2] + s[3]) << 3;
    }
}

// ---- weight unit in registers -----------------------------------------------------
template <int FMT> struct UnitW;
template <> struct UnitW<LH_TQ2_0> { uint4 q; uint32_t d; };
template <> struct UnitW<LH_Q4_0> { uint4 a, b; uint32_t c; };

// Weight bytes are read through pointers in the global address space (the
// problem descriptors are loaded from memory, so the compiler cannot infer it).
typedef const __attribute__((address_space(1))) uint8_t* gptr_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

__device__ __forceinline__ uint4 ld16_align2(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(2))) u32x4_a2;
    const u32x4_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a2*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 ld16_align4(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(4))) u32x4_a4;
    const u32x4_t v = *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a4*>(p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

// The caller passes an in-range (row, ucol) for every lane, so the loads are
// unconditional; lanes without work carry zero activations instead.
template <int FMT>
__device__ __forceinline__ void load_unit_w(UnitW<FMT>& w, gptr_t row, uint32_t ucol) {
    if constexpr (FMT == LH_TQ2_0) {
        gptr_t blk = row + (size_t)(ucol >> 2) * 66;
        w.q = ld16_align2(blk + (ucol & 3) * 16);
        // only quarter 0 needs d; the other three lanes re-read their own quarter's first half-word
        w.d = *reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>(blk + ((ucol & 3) == 0 ? 64 : (ucol & 3) * 16));
    } else {
        gptr_t p = row + (size_t)ucol * 36;
        w.a = ld16_align4(p); w.b = ld16_align4(p + 16);
        w.c = *reinterpret_cast<const __attribute__((address_space(1))) uint32_t*>(p + 32);
    }
}

template <int L>
__device__ __forceinline__ int combine_limbs(const int (&acc)[L]) {
    int t = acc[L - 1];
#pragma unroll
    for (int l = L - 2; l >= 0; l--) t = (t << 8) + acc[l];
    return t;
}

// Contribution of one unit to its row: d * s * (sum q n - zp sum n).
template <int FMT, int L>
__device__ __forceinline__ float unit_dot(const UnitW<FMT>& w, const UnitX<FMT, L>& ux) {
    if constexpr (FMT == LH_TQ2_0) {
        const uint32_t wv[4] = {w.q.x, w.q.y, w.q.z, w.q.w};
        int A[L], B[L], Cq[L];
#pragma unroll
        for (int l = 0; l < L; l++) A[l] = B[l] = Cq[l] = 0;
#pragma unroll
        for (int m = 0; m < 4; m++) {
            const uint32_t v = wv[m], t = v >> 2;
            const int f0 = (int)(v & 0x03030303u), f1 = (int)(t & 0x03030303u);
            const int f2 = (int)(t & 0x0C0C0C0Cu), f3 = (int)(t & 0x30303030u);   // 4x and 16x the code
#pragma unroll
            for (int l = 0; l < L; l++) {
                A[l] = __builtin_amdgcn_sdot4(f0, (int)ux.xl[l][0][m], A[l], false);
                A[l] = __builtin_amdgcn_sdot4(f1, (int)ux.xl[l][1][m], A[l], false);
                B[l] = __builtin_amdgcn_sdot4(f2, (int)ux.xl[l][2][m], B[l], false);
                Cq[l] = __builtin_amdgcn_sdot4(f3, (int)ux.xl[l][3][m], Cq[l], false);
            }
        }
        int T[L];
#pragma unroll
        for (int l = 0; l < L; l++) T[l] = (A[l] << 4) + (B[l] << 2) + Cq[l];   // 16 * sum(code * n)
        const int i16 = combine_limbs<L>(T) - ux.nsum[0];                          // 16 * sum((code-1) * n)
        const int dbits = __builtin_amdgcn_update_dpp(0, (int)w.d, 0x00, 0xF, 0xF, true);  // quad lane 0 holds d
        return (float)i16 * (lh_h2f((uint16_t)dbits) * ux.scale[0]);
    } else {
        const uint32_t r[9] = {w.a.x, w.a.y, w.a.z, w.a.w, w.b.x, w.b.y, w.b.z, w.b.w, w.c};
        // dwords: [d0|q0 q1] [q2..5] [q6..9] [q10..13] [q14 q15|d1] [16 quant bytes of block 1]
        uint32_t q[2][4];
#pragma unroll
        for (int k = 0; k < 4; k++) q[0][k] = __builtin_amdgcn_alignbyte(r[k + 1], r[k], 2);
#pragma unroll
        for (int k = 0; k < 4; k++) q[1][k] = r[5 + k];
        const float d[2] = {lh_h2f((uint16_t)(r[0] & 0xFFFF)), lh_h2f((uint16_t)(r[4] >> 16))};
        float p = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int acc[L];
#pragma unroll
            for (int l = 0; l < L; l++) acc[l] = 0;
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const int lo = (int)(q[h][k] & 0x0F0F0F0Fu), hi = (int)((q[h][k] >> 4) & 0x0F0F0F0Fu);
#pragma unroll
                for (int l = 0; l < L; l++) {
                    acc[l] = __builtin_amdgcn_sdot4(lo, (int)ux.xl[l][2 * h][k], acc[l], false);
                    acc[l] = __builtin_amdgcn_sdot4(hi, (int)ux.xl[l][2 * h + 1][k], acc[l], false);
                }
            }
            const int iq = combine_limbs<L>(acc) - ux.nsum[h];                     // sum((q-8) * n)
            p += (float)iq * (d[h] * ux.scale[h]);
        }
        return p;
    }
}

template <int FMT> __host__ __device__ constexpr int steps_in_flight(int npos) {
    return FMT == LH_TQ2_0 ? (npos == 1 ? 8 : (npos == 2 ? 4 : 2)) : (npos == 1 ? 4 : (npos == 2 ? 2 : 1));
}

// Staged form (IMG, Q4_0 only): the rows of a wave's step are consecutive in memory, so the step is fetched as one
// contiguous run of 16-byte chunks -- consecutive lanes, consecutive chunks, every byte requested once, one step ahead in
// registers -- parked in a wave-private LDS image, and each lane reads its 36-byte units back from there (dword reads at a
// 9-dword lane stride: conflict free).  Fetching the units straight from global memory makes every lane's three loads share
// cache lines with its neighbours' and triples the address work of the memory pipeline.
constexpr int kImgLoads = 9;                                   // a step is at most 9216 bytes = 576 chunks
constexpr uint32_t kImgBytes = kImgLoads * 1024 + 64;          // per wave

__device__ __forceinline__ u32x4_t ld16_stream(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(4))) u32x4_a4;
    return __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4_a4*>(p));
}

// One launch serves `count` problems of the same shape (count == 1 for the plain matvec).
template <int FMT, int L, int NPOS, typename XT, typename YT, bool IMG = false>
__global__ __launch_bounds__(kWG, 2) void matvec_quant_kernel(const MatvecProblem* __restrict__ problems, MatvecBase single,
                                                             uint32_t count, uint32_t rows, uint32_t K, uint32_t lpr_log2,
                                                             uint32_t steps_per_wg) {
    extern __shared__ __align__(16) uint8_t lds[];
    constexpr int G = FMT == LH_TQ2_0 ? 256 : 32;
    constexpr int U = steps_in_flight<FMT>(NPOS);
    // [xq: L limb planes][xs: K/G scales] and, with two limbs, the residual level behind them: [xq2: 2 planes][xs2]
    uint32_t* xq = reinterpret_cast<uint32_t*>(lds);
    float* xs = reinterpret_cast<float*>(lds + (size_t)L * K);
    uint32_t* xq2 = reinterpret_cast<uint32_t*>(xs + K / G);
    float* xs2 = reinterpret_cast<float*>(reinterpret_cast<uint8_t*>(xq2) + (size_t)2 * K);
    const XResidual resid{xq2, xs2, nullptr};
    bool any_coarse = false;   // a lane of this wave owns a unit column with a residual level
    // the staged form's wave-private image sits behind the activation area (which ends with xs2 when L == 2)
    const size_t x_area = (size_t)L * K + (size_t)(K / G) * 4 + (L == 2 ? (size_t)2 * K + (size_t)(K / G) * 4 + 16 : 0);
    uint8_t* image = lds + ((x_area + 15) & ~(size_t)15) + (size_t)(threadIdx.x >> 6) * kImgBytes;

    const uint32_t upr = K >> 6;                                  // unit columns per row
    const uint32_t row_bytes = FMT == LH_TQ2_0 ? (K >> 8) * 66 : (K >> 5) * 18;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // A row's unit columns are dealt to `lpr` lanes, NPOS of them to a lane (columns col0, col0 + lpr, ...): lpr * NPOS >= upr.
    const uint32_t lpr = 1u << lpr_log2;                          // lanes per row
    const uint32_t rpw = 64u >> lpr_log2;                         // rows per wave step
    const uint32_t rsub = (uint32_t)lane >> lpr_log2;
    const uint32_t col0 = (uint32_t)lane & (lpr - 1);
    const uint32_t steps_per_problem = (rows + rpw - 1) / rpw;
    const uint64_t total_steps = (uint64_t)steps_per_problem * count;
    // One problem and a long walk per workgroup: the batches of U steps are dealt to the waves of the whole grid in turn, so
    // that the grid reads one compact, advancing window of the matrix instead of one stream per workgroup (the
    // 262144 x 1536 logits product: 0.64 -> 0.67 of the HBM rate).  Several problems keep a contiguous share per
    // workgroup: a workgroup then stages one or two vectors, not one per batch.
    const bool grid_window = count == 1 && steps_per_wg >= 8u * kWaves * U;
    uint64_t g0 = grid_window ? 0 : (uint64_t)blockIdx.x * steps_per_wg;
    const uint64_t g1 = grid_window ? total_steps : (g0 + steps_per_wg < total_steps ? g0 + steps_per_wg : total_steps);

    UnitX<FMT, L> ux[NPOS];
    const void* staged_vector = nullptr;
    while (g0 < g1) {
        const uint32_t prob = (uint32_t)(g0 / steps_per_problem);
        const uint32_t s_begin = (uint32_t)(g0 - (uint64_t)prob * steps_per_problem);
        const uint64_t seg_end64 = (uint64_t)(prob + 1) * steps_per_problem;
        const uint32_t s_end = (uint32_t)((g1 < seg_end64 ? g1 : seg_end64) - (uint64_t)prob * steps_per_problem);
        const MatvecProblem pb = problems ? problems[prob]
                                 : (single.pair && prob == 1) ? single.second
                                          : MatvecProblem{single.p.matrix + (size_t)prob * single.mstride, (const char*)single.p.vector + (size_t)prob * single.xstride,
                                                          (char*)single.p.output + (size_t)prob * single.ystride};
        // The waves of a workgroup take the batches of U steps of the segment in turn, so that the workgroup reads one
        // advancing window (four separate streams per workgroup measured 0.78-0.79 of the HBM rate on the grouped
        // 2048 x 2048 launch against 0.80-0.81) and a segment of few steps is not loaded once per wave: a wave always
        // requests U steps' rows, and with a contiguous share of one step each the four waves of a small launch requested
        // the same rows four times (a single-token decode layer: 66.6 -> 64.5 us).
        uint32_t st = s_begin + (grid_window ? blockIdx.x * kWaves + wave : wave) * U;
        const uint32_t st_end = s_end;
        if (st > s_end) st = s_end;
        const uint32_t kStride = (grid_window ? gridDim.x * kWaves : kWaves) * U;

        YT* y = static_cast<YT*>(pb.output);
        gptr_t mat = (gptr_t)pb.matrix;
        const uint32_t last_row = rows - 1;
        const int red_width = (int)lpr;
        const bool writer = ((uint32_t)lane & (lpr - 1)) == 0;

        // ---- staged form: chunk c = lane + 64 i of the step's contiguous bytes
        [[maybe_unused]] u32x4_t pre[kImgLoads];
        [[maybe_unused]] const uint32_t step_bytes = U * rpw * row_bytes;
        [[maybe_unused]] const uint32_t step_chunks = (step_bytes + 15) >> 4;
        [[maybe_unused]] const size_t mat_bytes = (size_t)rows * row_bytes;   // chunks past the matrix read its first slack bytes (never used)
        [[maybe_unused]] auto prefetch = [&](uint32_t st_) {
            const size_t base = (size_t)st_ * rpw * row_bytes;
#pragma unroll
            for (int i = 0; i < kImgLoads; i++) {
                // no branch around a load (a conditionally loaded register forces a wait right behind the load):
                // surplus lanes repeat the step's last chunk, which is never parked
                uint32_t c = lane + 64 * i;
                c = c < step_chunks ? c : step_chunks - 1;
                size_t off = base + (size_t)c * 16;
                off = off < mat_bytes ? off : mat_bytes;
                pre[i] = ld16_stream(mat + off);
            }
        };
        if constexpr (IMG) { if (st < st_end) prefetch(st); }
        // The first step's weights are requested before the vector is staged: their trip to memory then runs under the
        // quantiser and its two barriers instead of behind them (a launch of a few steps per wave is mostly that latency).
        constexpr bool kEarly = !IMG && FMT == LH_Q4_0 && NPOS <= 2;   // (the other forms have no registers to spare)
        [[maybe_unused]] UnitW<FMT> w_first[kEarly ? U : 1][kEarly ? NPOS : 1];
        bool have_first = false;
        if constexpr (kEarly) {
            if (pb.vector != staged_vector && st < st_end) {
#pragma unroll
                for (int u = 0; u < U; u++) {
                    uint32_t row = (st + u) * rpw + rsub;
                    row = row < last_row ? row : last_row;
                    gptr_t rp = mat + (size_t)row * row_bytes;
#pragma unroll
                    for (int p = 0; p < NPOS; p++) {
                        const uint32_t ucol = col0 + lpr * p;
                        load_unit_w<FMT>(w_first[u][p], rp, ucol < upr ? ucol : 0u);
                    }
                }
                have_first = true;
            }
        }
        if (pb.vector != staged_vector) {
            __syncthreads();   // every wave is done reading the previous vector's limbs
            quantize_x_to_lds<L, G, XT>(static_cast<const XT*>(pb.vector), K, xq, xs, nullptr, kWG, single.pro, L == 2 ? &resid : nullptr);
            __syncthreads();
            if constexpr (L == 2) {
                bool mine = false;
#pragma unroll
                for (int p = 0; p < NPOS; p++) {
                    const uint32_t ucol = col0 + lpr * p;
                    if (ucol < upr) {
                        if constexpr (FMT == LH_TQ2_0) mine = mine || xs2[ucol >> 2] != 0.0f;
                        else mine = mine || xs2[2 * ucol] != 0.0f || xs2[2 * ucol + 1] != 0.0f;
                    }
                }
                any_coarse = __builtin_amdgcn_ballot_w64(mine) != 0;
            }
#pragma unroll
            for (int p = 0; p < NPOS; p++) {
                const uint32_t ucol = col0 + lpr * p;
                load_unit_x<FMT, L>(ux[p], ucol < upr ? ucol : 0u, K, xq, xs);
                if (ucol >= upr) {   // a lane without a unit column contributes exactly zero
#pragma unroll
                    for (int l = 0; l < L; l++)
#pragma unroll
                        for (int r = 0; r < 4; r++)
#pragma unroll
                            for (int k = 0; k < 4; k++) ux[p].xl[l][r][k] = 0;
                    ux[p].scale[0] = ux[p].scale[1] = 0.0f;
                    ux[p].nsum[0] = ux[p].nsum[1] = 0;
                }
            }
            staged_vector = pb.vector;
        }

        for (; st < st_end; st += kStride) {
            float part[U];
            if constexpr (IMG) {
                __builtin_amdgcn_s_setprio(0);        // (raised below, once the step's data is in the image)
                __builtin_amdgcn_wave_barrier();      // the units of the previous step have been read
#pragma unroll
                for (int i = 0; i < kImgLoads; i++)
                    if ((uint32_t)lane + 64 * i < step_chunks) *reinterpret_cast<u32x4_t*>(image + ((uint32_t)lane + 64 * i) * 16) = pre[i];
                __builtin_amdgcn_wave_barrier();
                if (st + kStride < st_end) prefetch(st + kStride);
                // The wave has what it needs for this step and runs it at a raised priority: of the waves of a SIMD the one
                // that can finish a step does, and reaches its next wait, and the loads behind it, sooner.
                __builtin_amdgcn_s_setprio(1);
#pragma unroll
                for (int u = 0; u < U; u++) {
                    part[u] = 0.0f;
#pragma unroll
                    for (int p = 0; p < NPOS; p++) {
                        const uint32_t ucol = col0 + lpr * p;
                        UnitW<FMT> w;
                        const uint32_t* src = reinterpret_cast<const uint32_t*>(image + ((uint32_t)u * rpw + rsub) * row_bytes + (ucol < upr ? ucol : 0u) * 36);
                        w.a = make_uint4(src[0], src[1], src[2], src[3]);
                        w.b = make_uint4(src[4], src[5], src[6], src[7]);
                        w.c = src[8];
                        part[u] += unit_dot<FMT, L>(w, ux[p]);
                        if constexpr (L == 2) {
                            if (any_coarse && ucol < upr) {   // rare: the residual level of this unit column, read from LDS
                                UnitX<FMT, 2> ur;
                                load_unit_x<FMT, 2>(ur, ucol, K, xq2, xs2);
                                part[u] += unit_dot<FMT, 2>(w, ur);
                            }
                        }
                    }
                }
            } else {
            UnitW<FMT> w[U][NPOS];
            if (have_first) {                           // requested before the vector was staged
                if constexpr (kEarly) {
#pragma unroll
                    for (int u = 0; u < U; u++)
#pragma unroll
                        for (int p = 0; p < NPOS; p++) w[u][p] = w_first[u][p];
                }
                have_first = false;
            } else {
#pragma unroll
            for (int u = 0; u < U; u++) {
                uint32_t row = (st + u) * rpw + rsub;     // steps past the end re-read the last row (result dropped)
                row = row < last_row ? row : last_row;
                gptr_t rp = mat + (size_t)row * row_bytes;
#pragma unroll
                for (int p = 0; p < NPOS; p++) {
                    const uint32_t ucol = col0 + lpr * p;
                    load_unit_w<FMT>(w[u][p], rp, ucol < upr ? ucol : 0u);
                }
            }
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                part[u] = 0.0f;
#pragma unroll
                for (int p = 0; p < NPOS; p++) part[u] += unit_dot<FMT, L>(w[u][p], ux[p]);
            }
            if constexpr (L == 2) {
                if (__builtin_expect(any_coarse, 0)) {   // uniform over the wave; rare: the residual level of the lane's unit columns, read from LDS
#pragma unroll
                    for (int p = 0; p < NPOS; p++) {
                        const uint32_t ucol = col0 + lpr * p;
                        if (ucol < upr) {
                            UnitX<FMT, 2> ur;
                            load_unit_x<FMT, 2>(ur, ucol, K, xq2, xs2);
#pragma unroll
                            for (int u = 0; u < U; u++) part[u] += unit_dot<FMT, 2>(w[u][p], ur);
                        }
                    }
                }
            }
            }   // !IMG
            // butterfly over the lanes of a row, all U rows per level
            if (red_width > 1) {
#pragma unroll
                for (int u = 0; u < U; u++) part[u] += lh_dpp_f<LH_DPP_QUAD_XOR1>(part[u]);
            }
            if (red_width > 2) {
#pragma unroll
                for (int u = 0; u < U; u++) part[u] += lh_dpp_f<LH_DPP_QUAD_XOR2>(part[u]);
            }
            if (red_width > 4) {
#pragma unroll
                for (int u = 0; u < U; u++) part[u] += lh_dpp_f<LH_DPP_HALF_MIRROR>(part[u]);
            }
            if (red_width > 8) {
#pragma unroll
                for (int u = 0; u < U; u++) part[u] += lh_dpp_f<LH_DPP_ROW_MIRROR>(part[u]);
            }
            if (red_width > 16) {
#pragma unroll
                for (int u = 0; u < U; u++) part[u] += lh_swap16_f(part[u]);
            }
            if (red_width > 32) {
#pragma unroll
                for (int u = 0; u < U; u++) part[u] += lh_swap32_f(part[u]);
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const uint32_t row = (st + u) * rpw + rsub;
                if (writer && (st + u) < st_end && row < rows) lh_store_from_f32<YT>(y, row, part[u]);
            }
        }
        g0 = (uint64_t)prob * steps_per_problem + s_end;
    }
}

// Fallback for shapes / alignments the fast path does not take (Q4_0 with an
// odd block count per row, cols > 16384, odd base addresses): one wave per
// row, byte loads, fp32 FMA on the dequantised value d*(q-zp).
template <int FMT, typename XT, typename YT>
__global__ __launch_bounds__(256) void matvec_quant_generic_kernel(const uint8_t* __restrict__ matrix, const XT* __restrict__ x,
                                                                  YT* __restrict__ y, uint32_t rows, uint32_t K) {
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    float acc = 0.0f;
    if constexpr (FMT == LH_Q4_0) {
        const uint32_t nb = K >> 5;
        const uint8_t* rp = matrix + (size_t)row * nb * 18;
        for (uint32_t i = lane; i < nb * 16; i += 64) {     // one quant byte (2 weights) per lane per trip
            const uint32_t b = i >> 4, j = i & 15;
            const uint8_t* bp = rp + (size_t)b * 18;
            const float d = lh_h2f((uint16_t)(bp[0] | (bp[1] << 8)));
            const uint32_t q = bp[2 + j];
            acc += d * ((float)(q & 15) - 8.0f) * lh_load_as_f32<XT>(x, b * 32 + j);
            acc += d * ((float)(q >> 4) - 8.0f) * lh_load_as_f32<XT>(x, b * 32 + 16 + j);
        }
    } else {
        const uint32_t nb = K >> 8;
        const uint8_t* rp = matrix + (size_t)row * nb * 66;
        for (uint32_t i = lane; i < nb * 64; i += 64) {     // one qs byte (4 weights) per lane per trip
            const uint32_t b = i >> 6, j = i & 63;
            const uint8_t* bp = rp + (size_t)b * 66;
            const float d = lh_h2f((uint16_t)(bp[64] | (bp[65] << 8)));
            const uint32_t q = bp[j];
            const uint32_t e = b * 256 + (j >> 5) * 128 + (j & 31);
#pragma unroll
            for (int l = 0; l < 4; l++)
                acc += d * ((float)((q >> (2 * l)) & 3) - 1.0f) * lh_load_as_f32<XT>(x, e + l * 32);
        }
    }
    acc = lh_group_sum(acc, 64);
    if (lane == 0) lh_store_from_f32<YT>(y, row, acc);
}

// SoA TQ2_0 (64-byte aligned qs rows + separate f16 scales): same arithmetic as
// the generic path with 16-byte loads.
template <typename XT, typename YT>
__global__ __launch_bounds__(256) void matvec_tq2_0_soa_kernel(const uint8_t* __restrict__ qs, const uint16_t* __restrict__ scales,
                                                              const XT* __restrict__ x, YT* __restrict__ y, uint32_t rows, uint32_t K) {
    const int lane = threadIdx.x & 63;
    const uint32_t row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const uint32_t nb = K >> 8;
    float acc = 0.0f;
    for (uint32_t u = lane; u < nb * 4; u += 64) {            // 16 qs bytes per lane per trip
        const uint32_t b = u >> 2, a = u & 3;
        const uint4 v = *reinterpret_cast<const uint4*>(qs + ((size_t)row * nb + b) * 64 + a * 16);
        const float d = lh_h2f(scales[(size_t)row * nb + b]);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
        const uint32_t e0 = b * 256 + (a >> 1) * 128 + (a & 1) * 16;
        float s = 0.0f;
#pragma unroll
        for (int m = 0; m < 4; m++)
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const uint32_t q = (w[m] >> (8 * k)) & 0xFF;
#pragma unroll
                for (int l = 0; l < 4; l++)
                    s += ((float)((q >> (2 * l)) & 3) - 1.0f) * lh_load_as_f32<XT>(x, e0 + l * 32 + m * 4 + k);
            }
        acc += d * s;
    }
    acc = lh_group_sum(acc, 64);
    if (lane == 0) lh_store_from_f32<YT>(y, row, acc);
}

// Activation limbs: two (16-bit block fixed point, with a second level for blocks that need one).
int x_limbs(lh_quant) { return 2; }

// LOCAL_HIP_TQ2_KERNEL=valu selects the vector-ALU (v_dot4) TQ2_0 kernel instead of the MFMA one.
bool tq2_on_matrix_cores() {
    static bool v = [] {
        const char* e = getenv("LOCAL_HIP_TQ2_KERNEL");
        return !(e && e[0] == 'v');
    }();
    return v;
}

int wg_per_cu() { return 2; }

struct LaunchGeom {
    uint32_t npos, lpr_log2, rpw, grid, steps_per_wg;
    size_t lds_bytes;
    bool img;   // staged form: Q4_0 with two limbs and at least 16 readable bytes behind every matrix
};

LaunchGeom plan(lh_quant fmt, uint32_t count, uint32_t rows, uint32_t K, int cu_count, int L, size_t min_slack = 0) {
    LaunchGeom g{};
    const uint32_t upr = K / 64;
    g.npos = (upr + 63) / 64;
    uint32_t lpr = 1; g.lpr_log2 = 0;
    if (g.npos == 1) { while (lpr < upr) { lpr <<= 1; g.lpr_log2++; } }
    else { lpr = 64; g.lpr_log2 = 6; }
    // Three times a power of two (1536, 3072 or 6144 columns): three unit columns per lane and a third of the lanes per row keep
    // every lane at work, where the next power of two would leave a quarter of them idle.  For launches that stream (the
    // 262144 x 1536 logits product: 46.8 -> 44.3 us); a launch of a few steps per wave is latency, and there one unit per
    // lane with four steps in flight is the faster form (a decoded token of the 1536-wide model: -1.5 % with this one).
    if (upr % 3 == 0 && upr / 3 <= 64 && ((upr / 3) & (upr / 3 - 1)) == 0 && (uint64_t)rows * count * K >= (64ull << 20)) {
        g.npos = 3;
        lpr = upr / 3;
        g.lpr_log2 = 0;
        while ((1u << g.lpr_log2) < lpr) g.lpr_log2++;
    }
    g.rpw = 64 / lpr;
    const uint64_t steps = (uint64_t)((rows + g.rpw - 1) / g.rpw) * count;
    // two workgroups per CU when there is enough work; never fewer than one step per wave
    uint64_t want = (steps + kWaves - 1) / kWaves;
    const uint64_t cap = (uint64_t)cu_count * wg_per_cu();
    if (want > cap) want = cap;
    if (want < 1) want = 1;
    g.steps_per_wg = (uint32_t)((steps + want - 1) / want);
    // Several workgroups per problem (the rows of a small activation batch): a share that divides a problem's steps keeps
    // every workgroup inside one problem, so none stages a second vector half way (7 rows against 2048 x 2048: 7.2 -> 5.4 us).
    const uint32_t spp = (rows + g.rpw - 1) / g.rpw;
    if (count > 1 && g.steps_per_wg * 2 <= spp && spp % g.steps_per_wg != 0) {
        uint32_t s = g.steps_per_wg;
        while (s < 2 * g.steps_per_wg && spp % s != 0) s++;
        if (spp % s == 0) g.steps_per_wg = s;
    }
    g.grid = (uint32_t)((steps + g.steps_per_wg - 1) / g.steps_per_wg);
    const uint32_t G = fmt == LH_TQ2_0 ? 256 : 32;
    g.lds_bytes = (size_t)L * K + (size_t)(K / G) * 4 + (L == 2 ? (size_t)2 * K + (size_t)(K / G) * 4 + 16 : 0);
    // the staged form pays off once a wave walks several steps (its first fetch is not overlapped with anything)
    const uint32_t in_flight = g.npos == 1 ? 4u : (g.npos == 2 ? 2u : 1u);        // steps_in_flight<LH_Q4_0>(npos)
    g.img = fmt == LH_Q4_0 && L == 2 && min_slack >= 16 && g.steps_per_wg >= 2u * kWaves * in_flight;
    // The images come on top of the activation area; rows long enough to push the sum past the raised limit keep direct loads.
    const size_t with_img = ((g.lds_bytes + 15) & ~(size_t)15) + (size_t)kWaves * kImgBytes;
    if (g.img && with_img > kMaxDynamicLds) g.img = false;
    if (g.img) g.lds_bytes = with_img;
    return g;
}

template <int FMT, int L, int NPOS>
int launch_typed(lh_context* ctx, const MatvecProblem* dev_problems, const MatvecBase& single, uint32_t count, lh_dtype xt,
                 lh_dtype yt, uint32_t rows, uint32_t K, const LaunchGeom& g) {
#define LH_LAUNCH_K(KERNEL)                                                                                                 \
    do {                                                                                                                    \
        if (g.lds_bytes > kMaxDynamicLds)                                                                                   \
            return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: %zu bytes of LDS needed, limit %zu", g.lds_bytes,        \
                           (size_t)kMaxDynamicLds);                                                                         \
        if (g.lds_bytes > 64 * 1024) {   /* long rows: more than the 64 KB a kernel gets without asking */                  \
            const int rl = lh_raise_dynamic_lds(ctx, (const void*)KERNEL, kMaxDynamicLds, "matvec_quant");                  \
            if (rl != LH_OK) return rl;                                                                                     \
        }                                                                                                                   \
        hipLaunchKernelGGL(KERNEL, dim3(g.grid), dim3(kWG), g.lds_bytes, ctx->stream,                                       \
                           dev_problems, single, count, rows, K, g.lpr_log2, g.steps_per_wg);                               \
    } while (0)
#define LH_LAUNCH(XT, YT)                                                                                                   \
    do {                                                                                                                    \
        if constexpr (FMT == LH_Q4_0 && L == 2) {                                                                           \
            if (g.img) LH_LAUNCH_K((matvec_quant_kernel<FMT, L, NPOS, XT, YT, true>));                                      \
            else LH_LAUNCH_K((matvec_quant_kernel<FMT, L, NPOS, XT, YT, false>));                                           \
        } else LH_LAUNCH_K((matvec_quant_kernel<FMT, L, NPOS, XT, YT, false>));                                             \
    } while (0)
    if (xt == LH_F32 && yt == LH_F32) LH_LAUNCH(float, float);
    else if (xt == LH_F16 && yt == LH_F16) LH_LAUNCH(uint16_t, uint16_t);
    else if (xt == LH_F16 && yt == LH_F32) LH_LAUNCH(uint16_t, float);
    else LH_LAUNCH(float, uint16_t);
#undef LH_LAUNCH
#undef LH_LAUNCH_K
    return lh_check_launch("matvec_quant");
}

template <int FMT, int L>
int launch_npos(lh_context* ctx, const MatvecProblem* p, const MatvecBase& single, uint32_t count, lh_dtype xt, lh_dtype yt,
                uint32_t rows, uint32_t K, const LaunchGeom& g) {
    switch (g.npos) {
        case 1: return launch_typed<FMT, L, 1>(ctx, p, single, count, xt, yt, rows, K, g);
        case 2: return launch_typed<FMT, L, 2>(ctx, p, single, count, xt, yt, rows, K, g);
        case 3: return launch_typed<FMT, L, 3>(ctx, p, single, count, xt, yt, rows, K, g);
        default: return launch_typed<FMT, L, 4>(ctx, p, single, count, xt, yt, rows, K, g);
    }
}

template <int FMT>
int launch_generic(lh_context* ctx, const uint8_t* m, const void* x, void* y, lh_dtype xt, lh_dtype yt, uint32_t rows, uint32_t K) {
    const dim3 grid((rows + 3) / 4), block(256);
#define LH_LAUNCH(XT, YT) \
    hipLaunchKernelGGL((matvec_quant_generic_kernel<FMT, XT, YT>), grid, block, 0, ctx->stream, m, (const XT*)x, (YT*)y, rows, K)
    if (xt == LH_F32 && yt == LH_F32) LH_LAUNCH(float, float);
    else if (xt == LH_F16 && yt == LH_F16) LH_LAUNCH(uint16_t, uint16_t);
    else if (xt == LH_F16 && yt == LH_F32) LH_LAUNCH(uint16_t, float);
    else LH_LAUNCH(float, uint16_t);
#undef LH_LAUNCH
    return lh_check_launch("matvec_quant_generic");
}

const char* op_name(lh_quant fmt) { return fmt == LH_Q4_0 ? "matvec_q4_0" : "matvec_tq2_0"; }

bool fast_path_ok(lh_quant fmt, const void* matrix, const void* vector, uint32_t K) {
    if (K > kMaxFastCols) return false;
    if (((uintptr_t)vector & 15) != 0) return false;
    if (fmt == LH_Q4_0) return (K % 64) == 0 && ((uintptr_t)matrix & 3) == 0;
    return ((uintptr_t)matrix & 1) == 0;
}

// Validates and launches `count` matvecs of one shape.
int matvec_dispatch(lh_batch* batch, lh_quant fmt, uint32_t count, const lh_buffer* const* matrices,
                    const lh_buffer* const* vectors, lh_dtype xt, lh_buffer* const* outputs, lh_dtype yt, uint32_t rows,
                    uint32_t cols, const char* op, const XPrologue& pro = XPrologue{kXProNone, nullptr, 0.0f}) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: batch is null", op);
    if (xt == LH_BF16 || yt == LH_BF16) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: bf16 vectors are not supported", op);
    // kernels.rs:5720-5724, 5857-5861: block alignment is checked before anything is encoded.
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256;
    if (cols % blk != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: cols %u not /%u", op, cols, blk);
    if (count == 0 || rows == 0 || cols == 0) return LH_OK;
    lh_context* ctx = batch->ctx;
    const size_t wbytes = (size_t)rows * (cols / blk) * (fmt == LH_Q4_0 ? 18 : 66);
    bool fast = true;
    size_t min_slack = ~(size_t)0;   // the staged TQ2_0 kernel reads whole 16-byte chunks: up to 14 bytes past a ragged row
    for (uint32_t i = 0; i < count; i++) {
        LH_NEED(matrices[i], wbytes, op, "matrix");
        LH_NEED(vectors[i], (size_t)cols * lh_dtype_size(xt), op, "vector");
        LH_NEED(outputs[i], (size_t)rows * lh_dtype_size(yt), op, "output");
        fast = fast && fast_path_ok(fmt, matrices[i]->ptr, vectors[i]->ptr, cols);
        const size_t sl = matrices[i]->len - wbytes + matrices[i]->slack;
        if (sl < min_slack) min_slack = sl;
    }
    if (!fast && pro.kind != kXProNone)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: a fused activation prologue needs 16-byte aligned vectors and cols a multiple of 64", op);
    if (!fast) {
        for (uint32_t i = 0; i < count; i++) {
            int r = fmt == LH_Q4_0
                        ? launch_generic<LH_Q4_0>(ctx, (const uint8_t*)matrices[i]->ptr, vectors[i]->ptr, outputs[i]->ptr, xt, yt, rows, cols)
                        : launch_generic<LH_TQ2_0>(ctx, (const uint8_t*)matrices[i]->ptr, vectors[i]->ptr, outputs[i]->ptr, xt, yt, rows, cols);
            if (r != LH_OK) return r;
            batch->dispatch_count++;
        }
        return LH_OK;
    }
    // Problems whose matrices, vectors and outputs are each evenly spaced (replicas or layers packed into one allocation,
    // one shared vector) need no descriptor table: problem i is problem 0 advanced by i strides, which travels in the
    // kernel arguments.  That saves the table's upload, which sits between two launches on the stream.
    uint64_t mstride = 0, xstride = 0, ystride = 0;
    bool regular = count > 2 && pro.kind == kXProNone;
    if (regular) {
        const char* m0 = (const char*)matrices[0]->ptr; const char* x0 = (const char*)vectors[0]->ptr; const char* y0 = (const char*)outputs[0]->ptr;
        const char* m1 = (const char*)matrices[1]->ptr; const char* x1 = (const char*)vectors[1]->ptr; const char* y1 = (const char*)outputs[1]->ptr;
        regular = m1 > m0 && x1 >= x0 && y1 > y0;
        if (regular) {
            mstride = (uint64_t)(m1 - m0); xstride = (uint64_t)(x1 - x0); ystride = (uint64_t)(y1 - y0);
            regular = xstride <= 0xFFFFFFFFull && ystride <= 0xFFFFFFFFull && (xstride & 15) == 0 && (mstride & 3) == 0;
            for (uint32_t i = 2; regular && i < count; i++)
                regular = (const char*)matrices[i]->ptr == m0 + (size_t)i * mstride && (const char*)vectors[i]->ptr == x0 + (size_t)i * xstride &&
                          (const char*)outputs[i]->ptr == y0 + (size_t)i * ystride;
        }
    }
    if (fmt == LH_TQ2_0 && tq2_on_matrix_cores() && cols <= 12288 && ((cols / 256) % 8 == 0 || min_slack >= 16)) {
        if (regular) {
            const void* pm1[1] = {matrices[0]->ptr}; const void* px1[1] = {vectors[0]->ptr}; void* py1[1] = {outputs[0]->ptr};
            int r = lh_launch_matvec_tq2_mfma(ctx, count, pm1, px1, py1, xt, yt, rows, cols, (uint32_t)xstride, (uint32_t)ystride, pro, mstride);
            if (r == LH_OK) batch->dispatch_count++;
            return r;
        }
        const void* stack_m[8]; const void* stack_x[8]; void* stack_y[8];
        const void** pm = count <= 8 ? stack_m : (const void**)malloc(sizeof(void*) * 3 * count);
        if (!pm) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", sizeof(void*) * 3 * (size_t)count);
        const void** px = count <= 8 ? stack_x : pm + count;
        void** py = count <= 8 ? stack_y : (void**)(pm + 2 * (size_t)count);
        for (uint32_t i = 0; i < count; i++) { pm[i] = matrices[i]->ptr; px[i] = vectors[i]->ptr; py[i] = outputs[i]->ptr; }
        int r = lh_launch_matvec_tq2_mfma(ctx, count, pm, px, py, xt, yt, rows, cols, 0, 0, pro);
        if (count > 8) free((void*)pm);
        if (r == LH_OK) batch->dispatch_count++;
        return r;
    }
    // One problem travels in the kernel arguments; several go through a descriptor array in the
    // top quarter of the context workspace (the copy is stream ordered, so it cannot overtake a
    // kernel that still reads the previous set).
    MatvecBase single{MatvecProblem{(const uint8_t*)matrices[0]->ptr, vectors[0]->ptr, outputs[0]->ptr}, 0, 0};
    single.pro = pro;
    MatvecProblem* dev_desc = nullptr;
    if (count == 2) {
        single.second = MatvecProblem{(const uint8_t*)matrices[1]->ptr, vectors[1]->ptr, outputs[1]->ptr};
        single.pair = 1;
    } else if (regular) {
        single.xstride = (uint32_t)xstride; single.ystride = (uint32_t)ystride; single.mstride = mstride;
    } else if (count > 2) {
        if (ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: more than two grouped problems need a descriptor upload, which a captured graph cannot hold", op);
        const size_t desc_bytes = (size_t)count * sizeof(MatvecProblem);
        if (desc_bytes > ctx->workspace_bytes / 4)
            return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: %u problems exceed the descriptor area", op, count);
        MatvecProblem* host_desc = (MatvecProblem*)malloc(desc_bytes);
        if (!host_desc) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", desc_bytes);
        for (uint32_t i = 0; i < count; i++) {
            host_desc[i].matrix = (const uint8_t*)matrices[i]->ptr;
            host_desc[i].vector = vectors[i]->ptr;
            host_desc[i].output = outputs[i]->ptr;
        }
        dev_desc = (MatvecProblem*)((char*)ctx->workspace + ctx->workspace_bytes - ctx->workspace_bytes / 4);
        const int ru = lh_upload_descriptors(ctx, host_desc, desc_bytes, dev_desc, op);
        free(host_desc);   // staged by the helper
        if (ru != LH_OK) return ru;
    }
    const int L = x_limbs(fmt);
    const LaunchGeom g = plan(fmt, count, rows, cols, ctx->cu_count, L, min_slack);
    int r;
    if (fmt == LH_Q4_0) r = launch_npos<LH_Q4_0, 2>(ctx, dev_desc, single, count, xt, yt, rows, cols, g);
    else r = launch_npos<LH_TQ2_0, 2>(ctx, dev_desc, single, count, xt, yt, rows, cols, g);
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

int matvec_one(lh_batch* batch, lh_quant fmt, const lh_buffer* m, const lh_buffer* x, lh_dtype xt, lh_buffer* y, lh_dtype yt,
               uint32_t rows, uint32_t cols) {
    const lh_buffer* ms[1] = {m};
    const lh_buffer* xs[1] = {x};
    lh_buffer* ys[1] = {y};
    return matvec_dispatch(batch, fmt, 1, ms, xs, xt, ys, yt, rows, cols, op_name(fmt));
}

int matvec_blocking(lh_context* ctx, lh_quant fmt, const lh_buffer* m, const lh_buffer* x, lh_dtype xt, lh_buffer* y, lh_dtype yt,
                    uint32_t rows, uint32_t cols) {
    if (!ctx) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: context is null", op_name(fmt));
    lh_batch b{ctx, 0};
    int r = matvec_one(&b, fmt, m, x, xt, y, yt, rows, cols);
    if (r != LH_OK) return r;
    return lh_batch_commit_and_wait(&b);
}


int matvec_rows_impl(lh_batch* batch, lh_quant fmt, uint32_t m, const lh_buffer* weight, const lh_buffer* input, lh_dtype at,
                     lh_buffer* output, lh_dtype ct, uint32_t n, uint32_t k, const char* op) {
    if (at == LH_BF16 || ct == LH_BF16) return -1;
    if (!fast_path_ok(fmt, weight->ptr, input->ptr, k)) return -1;
    const size_t xstride = (size_t)k * lh_dtype_size(at), ystride = (size_t)n * lh_dtype_size(ct);
    if ((xstride & 15) != 0 || xstride > 0xFFFFFFFFull || ystride > 0xFFFFFFFFull) return -1;
    lh_context* ctx = batch->ctx;
    const uint32_t blk = fmt == LH_Q4_0 ? 32 : 256;
    const size_t wbytes = (size_t)n * (k / blk) * (fmt == LH_Q4_0 ? 18 : 66);
    const size_t slack = weight->len - wbytes + weight->slack;
    int r;
    if (fmt == LH_TQ2_0 && tq2_on_matrix_cores() && k <= 12288 && ((k / 256) % 8 == 0 || slack >= 16)) {
        const void* pm[1] = {weight->ptr}; const void* px[1] = {input->ptr}; void* py[1] = {output->ptr};
        r = lh_launch_matvec_tq2_mfma(ctx, m, pm, px, py, at, ct, n, k, (uint32_t)xstride, (uint32_t)ystride);
    } else {
        MatvecBase single{MatvecProblem{(const uint8_t*)weight->ptr, input->ptr, output->ptr}, (uint32_t)xstride, (uint32_t)ystride};
        const int L = x_limbs(fmt);
        const LaunchGeom g = plan(fmt, m, n, k, ctx->cu_count, L, slack);
        if (fmt == LH_Q4_0) r = launch_npos<LH_Q4_0, 2>(ctx, nullptr, single, m, at, ct, n, k, g);
        else r = launch_npos<LH_TQ2_0, 2>(ctx, nullptr, single, m, at, ct, n, k, g);
    }
    (void)op;
    return r;
}

}  // namespace

int lh_matvec_rows(lh_batch* batch, lh_quant fmt, uint32_t m, const lh_buffer* weight, const lh_buffer* input, lh_dtype at,
                   lh_buffer* output, lh_dtype ct, uint32_t n, uint32_t k, const char* op) {
    return matvec_rows_impl(batch, fmt, m, weight, input, at, output, ct, n, k, op);
}

extern "C" {

int lh_matvec_q4_0(lh_context* ctx, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_blocking(ctx, LH_Q4_0, m, x, LH_F16, y, LH_F16, rows, cols);
}
int lh_matvec_q4_0_into(lh_batch* b, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_one(b, LH_Q4_0, m, x, LH_F16, y, LH_F16, rows, cols);
}
int lh_matvec_q4_0_f32out(lh_context* ctx, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_blocking(ctx, LH_Q4_0, m, x, LH_F16, y, LH_F32, rows, cols);
}
int lh_matvec_q4_0_f32out_into(lh_batch* b, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_one(b, LH_Q4_0, m, x, LH_F16, y, LH_F32, rows, cols);
}
int lh_matvec_tq2_0(lh_context* ctx, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_blocking(ctx, LH_TQ2_0, m, x, LH_F16, y, LH_F16, rows, cols);
}
int lh_matvec_tq2_0_into(lh_batch* b, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_one(b, LH_TQ2_0, m, x, LH_F16, y, LH_F16, rows, cols);
}
int lh_matvec_tq2_0_f32out(lh_context* ctx, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_blocking(ctx, LH_TQ2_0, m, x, LH_F16, y, LH_F32, rows, cols);
}
int lh_matvec_tq2_0_f32out_into(lh_batch* b, const lh_buffer* m, const lh_buffer* x, lh_buffer* y, uint32_t rows, uint32_t cols) {
    return matvec_one(b, LH_TQ2_0, m, x, LH_F16, y, LH_F32, rows, cols);
}

int lh_matvec_quant_typed_into(lh_batch* b, lh_quant fmt, const lh_buffer* m, const lh_buffer* x, lh_dtype xt, lh_buffer* y,
                               lh_dtype yt, uint32_t rows, uint32_t cols) {
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: unknown weight format %d", (int)fmt);
    return matvec_one(b, fmt, m, x, xt, y, yt, rows, cols);
}

int lh_matvec_quant_grouped_into(lh_batch* b, lh_quant fmt, uint32_t count, const lh_buffer* const* ms, const lh_buffer* const* xs,
                                 lh_dtype xt, lh_buffer* const* ys, lh_dtype yt, uint32_t rows, uint32_t cols) {
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: unknown weight format %d", (int)fmt);
    if (count && (!ms || !xs || !ys)) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null problem arrays", op_name(fmt));
    return matvec_dispatch(b, fmt, count, ms, xs, xt, ys, yt, rows, cols, op_name(fmt));
}

int lh_matvec_quant_fused_into(lh_batch* b, lh_quant fmt, uint32_t count, const lh_buffer* const* ms, const lh_buffer* x, int prologue,
                               const lh_buffer* aux, float eps, lh_buffer* const* ys, uint32_t rows, uint32_t cols) {
    const char* op = fmt == LH_Q4_0 ? "matvec_q4_0 (fused prologue)" : "matvec_tq2_0 (fused prologue)";
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: unknown weight format %d", (int)fmt);
    if (prologue != LH_PROLOGUE_RMS_NORM && prologue != LH_PROLOGUE_GELU_MUL)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: unknown prologue %d", op, prologue);
    if (count == 0 || rows == 0 || cols == 0) return LH_OK;
    if (count > 8) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: at most 8 matrices share one staged vector, got %u", op, count);
    if (!ms || !ys || !x) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null problem arrays", op);
    if (cols % 8 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: cols %u not /8", op, cols);
    LH_NEED(aux, (size_t)cols * 2, op, prologue == LH_PROLOGUE_RMS_NORM ? "norm weight" : "second factor");
    LH_REQUIRE(((uintptr_t)aux->ptr & 15) == 0, "%s: the prologue operand must be 16-byte aligned", op);
    const lh_buffer* xs[8];
    for (uint32_t i = 0; i < count; i++) xs[i] = x;
    const XPrologue pro{prologue == LH_PROLOGUE_RMS_NORM ? kXProRmsNorm : kXProGeluMul, (const uint16_t*)aux->ptr, eps};
    return matvec_dispatch(b, fmt, count, ms, xs, LH_F16, ys, LH_F16, rows, cols, op, pro);
}

int lh_matvec_quant_norm_chain_into(lh_batch* b, lh_quant fmt, uint32_t count, const lh_buffer* const* ms, const lh_buffer* x,
                                    const lh_buffer* weight, const lh_buffer* residual, const lh_buffer* next_weight, lh_buffer* store,
                                    float eps, lh_buffer* const* ys, uint32_t rows, uint32_t cols) {
    const char* op = fmt == LH_Q4_0 ? "matvec_q4_0 (norm chain)" : "matvec_tq2_0 (norm chain)";
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: unknown weight format %d", (int)fmt);
    if (count == 0 || rows == 0 || cols == 0) return LH_OK;
    if (count > 8) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: at most 8 matrices share one staged vector, got %u", op, count);
    if (!ms || !ys || !x) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null problem arrays", op);
    if (cols % 8 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: cols %u not /8", op, cols);
    const lh_buffer* vecs[4] = {weight, residual, next_weight, store};
    const char* names[4] = {"norm weight", "residual", "second norm weight", "stored vector"};
    for (int i = 0; i < 4; i++) {
        if (!vecs[i]) {
            if (i == 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: norm weight is null", op);
            continue;
        }
        LH_NEED(vecs[i], (size_t)cols * 2, op, names[i]);
        LH_REQUIRE(((uintptr_t)vecs[i]->ptr & 15) == 0, "%s: the %s must be 16-byte aligned", op, names[i]);
    }
    if (store) {
        LH_REQUIRE(store->ptr != x->ptr && (!residual || store->ptr != residual->ptr), "%s: the stored vector may not alias an input", op);
        for (uint32_t i = 0; i < count; i++) LH_REQUIRE(ys[i] && store->ptr != ys[i]->ptr, "%s: the stored vector may not alias an output", op);
    }
    const lh_buffer* xs[8];
    for (uint32_t i = 0; i < count; i++) xs[i] = x;
    XPrologue pro{kXProRmsNorm, (const uint16_t*)weight->ptr, eps};
    pro.res = residual ? (const uint16_t*)residual->ptr : nullptr;
    pro.aux2 = next_weight ? (const uint16_t*)next_weight->ptr : nullptr;
    pro.store = store ? (uint16_t*)store->ptr : nullptr;
    return matvec_dispatch(b, fmt, count, ms, xs, LH_F16, ys, LH_F16, rows, cols, op, pro);
}

int lh_matvec_quant_norm_chain_tail_into(lh_batch* b, lh_quant fmt, uint32_t count, const lh_buffer* const* ms, const lh_buffer* x,
                                         const lh_buffer* weight, const lh_buffer* residual, int apply_scale, float scale,
                                         const lh_buffer* next_weight, lh_buffer* store, float eps, lh_buffer* const* ys,
                                         uint32_t rows, uint32_t cols) {
    const char* op = fmt == LH_Q4_0 ? "matvec_q4_0 (layer tail chain)" : "matvec_tq2_0 (layer tail chain)";
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: unknown weight format %d", (int)fmt);
    if (count == 0 || rows == 0 || cols == 0) return LH_OK;
    if (count > 8) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: at most 8 matrices share one staged vector, got %u", op, count);
    if (!ms || !ys || !x) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null problem arrays", op);
    if (cols % 8 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: cols %u not /8", op, cols);
    if (!weight || !residual || !store) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: norm weight, residual and stored vector are required", op);
    const lh_buffer* vecs[4] = {weight, residual, next_weight, store};
    const char* names[4] = {"norm weight", "residual", "second norm weight", "stored vector"};
    for (int i = 0; i < 4; i++) {
        if (!vecs[i]) continue;
        LH_NEED(vecs[i], (size_t)cols * 2, op, names[i]);
        LH_REQUIRE(((uintptr_t)vecs[i]->ptr & 15) == 0, "%s: the %s must be 16-byte aligned", op, names[i]);
    }
    LH_REQUIRE(store->ptr != x->ptr && store->ptr != residual->ptr, "%s: the stored vector may not alias an input", op);
    for (uint32_t i = 0; i < count; i++) LH_REQUIRE(ys[i] && store->ptr != ys[i]->ptr, "%s: the stored vector may not alias an output", op);
    const lh_buffer* xs[8];
    for (uint32_t i = 0; i < count; i++) xs[i] = x;
    XPrologue pro{kXProRmsNorm, (const uint16_t*)weight->ptr, eps};
    pro.res = (const uint16_t*)residual->ptr;
    pro.aux2 = next_weight ? (const uint16_t*)next_weight->ptr : nullptr;
    pro.store = (uint16_t*)store->ptr;
    pro.tail = apply_scale ? 2u : 1u;
    pro.scale = scale;
    return matvec_dispatch(b, fmt, count, ms, xs, LH_F16, ys, LH_F16, rows, cols, op, pro);
}

int lh_matvec_quant_rotated_into(lh_batch* b, lh_quant fmt, const lh_buffer* m, const lh_buffer* x, const lh_buffer* signs,
                                 uint32_t head_dim, lh_buffer* y, uint32_t rows, uint32_t cols) {
    const char* op = fmt == LH_Q4_0 ? "matvec_q4_0 (rotated input)" : "matvec_tq2_0 (rotated input)";
    if (fmt != LH_Q4_0 && fmt != LH_TQ2_0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_quant: unknown weight format %d", (int)fmt);
    if (head_dim < 8 || head_dim > 512 || (head_dim & (head_dim - 1)) != 0)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: head_dim must be a power of two in 8..=512, got %u", op, head_dim);
    if (cols % head_dim != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: cols %u is not a multiple of head_dim %u", op, cols, head_dim);
    if (rows == 0 || cols == 0) return LH_OK;
    if (!m || !x || !y) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: null buffer", op);
    LH_NEED(signs, (size_t)head_dim * 4, op, "signs");
    LH_REQUIRE(((uintptr_t)signs->ptr & 15) == 0, "%s: the sign vector must be 16-byte aligned", op);
    const lh_buffer* ms[1] = {m};
    const lh_buffer* xs[1] = {x};
    lh_buffer* ys[1] = {y};
    XPrologue pro{kXProRotate, nullptr, 0.0f};
    pro.signs = (const float*)signs->ptr;
    pro.head_dim = head_dim;
    pro.scale = 1.0f / std::sqrt((float)head_dim);   // turboquant.rs:47
    return matvec_dispatch(b, fmt, 1, ms, xs, LH_F32, ys, LH_F16, rows, cols, op, pro);
}

int lh_matvec_tq2_0_soa_into(lh_batch* b, const lh_buffer* qs, const lh_buffer* scales, const lh_buffer* x, lh_buffer* y,
                             uint32_t rows, uint32_t cols) {
    // kernels.rs:5929-5933
    if (!b) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_tq2_0_soa: batch is null");
    if (cols % 256 != 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_tq2_0_soa: cols %u not /256", cols);
    if (rows == 0 || cols == 0) return LH_OK;
    const size_t nblk = (size_t)rows * (cols / 256);
    LH_NEED(qs, nblk * 64, "matvec_tq2_0_soa", "qs");
    LH_NEED(scales, nblk * 2, "matvec_tq2_0_soa", "scales");
    LH_NEED(x, (size_t)cols * 2, "matvec_tq2_0_soa", "vector");
    LH_NEED(y, (size_t)rows * 2, "matvec_tq2_0_soa", "output");
    LH_REQUIRE(((uintptr_t)qs->ptr & 15) == 0, "matvec_tq2_0_soa: qs must be 16-byte aligned");
    hipLaunchKernelGGL((matvec_tq2_0_soa_kernel<uint16_t, uint16_t>), dim3((rows + 3) / 4), dim3(256), 0, b->ctx->stream,
                       (const uint8_t*)qs->ptr, (const uint16_t*)scales->ptr, (const uint16_t*)x->ptr, (uint16_t*)y->ptr, rows, cols);
    int r = lh_check_launch("matvec_tq2_0_soa");
    if (r == LH_OK) b->dispatch_count++;
    return r;
}

}  // extern "C"
