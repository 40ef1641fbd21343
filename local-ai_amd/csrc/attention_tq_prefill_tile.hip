// Tiled prefill attention over packed 2-bit TurboQuant codes: sixteen query rows share one pass over the codes.
//
// Stands in for flash_attention_tq_prefill_tiled (shaders/attention_flash_tq.metal:425-567, chosen at
// local-engine/src/kv_cache/quant_cache.rs:641-667).  The rows of a prefill chunk attend to the same cache, so decoding a
// tile of K / V codes once and using it for many rows is what the tiling is for.  A workgroup is eight waves and sixteen
// query rows (128 queries with 8 heads); per tile of 64 positions:
//   stage    every wave turns an eighth of the tile's K codes into f16 levels (two v_perm_b32 look the level of each
//            2-bit field up in the table itself, two more interleave the bytes) and writes them to LDS in the order the
//            matrix cores read their B operand; its eight V code bytes of the 64 positions go to LDS as they are.
//   phase A  wave w owns rows 2w, 2w + 1: logits = Q x K^T with v_mfma_f32_16x16x32_f16, the 16 MFMA rows being the
//            8 heads of the two rows.  An f16 query alone is not enough (its 11 bits cost 3e-3 of the output on peaked
//            scores), so the rotated query is scaled by a power of two and split into f16(q) and f16(q - f16(q)), both
//            multiplied against the same K operand into one accumulator: 24 bits of the query for twice the MFMAs.
//            logit = norm_k * sum(rq * level), no 1/sqrt(d) factor (attention_flash_tq.metal:175-273).  Softmax weights
//            relative to a reference that follows the running maximum lazily, times the value norm, leave as f16 to LDS.
//   phase B  wave w owns output dims 32w .. 32w + 31 of all 128 queries: the V codes come back from LDS transposed
//            (ds_read_b64_tr_b8: one code byte over eight positions), the same look-up makes f16 levels of them and
//            v_mfma_f32_16x16x32_f16 accumulates weights x levels in f32.
// K levels, weights and V codes are double-buffered in LDS, so one workgroup barrier per tile orders everything: a
// wave stages tile t + 1 after its phase A of tile t, and runs phase B of tile t next to other waves' phase A of t + 1.
// Any level table works (nothing here assumes it is affine in the code bits).  Positions are split over gridDim.x
// workgroups per row tile; partials (R, l, acc) go to the workspace in the decode kernel's record layout and are merged
// by the same merge kernels.
#include "attention_tq.hpp"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace {
using namespace lh_attn;

typedef int v2i __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2_t;
typedef const __attribute__((address_space(1))) uint8_t* gptr_t;

constexpr int kRows = 16;              // query rows per workgroup
constexpr int kWaves = 8;
constexpr int kTile = 64;              // positions per step
constexpr int kHeads = 8;              // query heads per KV head served by the 16 MFMA rows of a row pair
constexpr int kHeadDim = 256, kCodeBytes = 64;
constexpr int kPwGroup = 16 * 16 + 16;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kHeadroom = 8.0f;      // log2 of how far a weight may exceed the softmax reference before that moves (f16 range)
constexpr float kNoRef = -1.0e30f;     // "no position seen yet": finite, so that exp2(logit - R) of a masked logit is 0, not NaN

__device__ __forceinline__ u32x2_t ld8(gptr_t p) {
    typedef u32x2_t __attribute__((aligned(4))) u32x2_a4;
    return *reinterpret_cast<const __attribute__((address_space(1))) u32x2_a4*>(p);
}
__device__ __forceinline__ float ld_norm(gptr_t p) {
    return lh_h2f(*reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>(p));
}

struct TileShared {
    uint8_t kt[2][4][8][64][16];           // [buffer][16-position tile][k step][lane]: K levels as f16, B operands as they are read
    uint8_t pw[2][kWaves][2][4][kPwGroup]; // [buffer][row pair][32-position half][k group]: [query of the pair][8 positions] weights as f16, + 16 bytes so that the packed stores spread over the banks
    uint8_t vt[4][kWaves][kTile][8];       // [tile % 4][wave][position]: the wave's eight V code bytes (a wave may stage tile t + 2 before its phase B of tile t)
    float fsc[2][kRows * kHeads];          // per query: factor for its output sums when its reference moved in this tile
    __attribute__((aligned(16))) uint32_t moved[2][kWaves];   // [row pair]: a reference moved in this tile
    float fin_l[kRows * kHeads], fin_r[kRows * kHeads];
};

struct RowRange { uint32_t lo, hi; };

template <bool ONE_KV>
__global__ __launch_bounds__(512, 2) void attention_tq_prefill_tile_kernel(AttnPointers a, AttnParams p) {
    __shared__ __align__(16) TileShared sh;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t pcol = lane & 15, g = lane >> 4;
    const uint32_t rt = blockIdx.y / p.num_kv_heads, kvh = blockIdx.y - rt * p.num_kv_heads;
    const uint32_t group = p.num_q_heads / p.num_kv_heads;
    const uint32_t row0 = rt * kRows;
    const uint32_t nrows = std::min<uint32_t>((uint32_t)kRows, p.num_queries - row0);
    const uint32_t n_pairs = (nrows + 1) >> 1;          // row pairs (MFMA row tiles) that hold a row of the chunk
    const bool pair_on = wave < n_pairs;                // this wave's phase A has rows to work on

    // the level table as two byte tables for v_perm_b32: byte c of tl / th = low / high byte of f16(L[c])
    uint32_t tl = 0, th = 0;
#pragma unroll
    for (int c = 0; c < 4; c++) {
        const uint32_t hbits = lh_f2h(a.levels[c]);
        tl |= (hbits & 0xFFu) << (8 * c);
        th |= (hbits >> 8) << (8 * c);
    }

    // ---- position ranges: row r of the tile is the query at position pos0 + row0 + r (attention_flash_tq.metal:300-330)
    auto row_range = [&](uint32_t r) {
        if (r >= nrows) r = nrows - 1;                 // rows past the end of the chunk mirror the last one (never stored)
        const uint32_t pos = p.pos0 + row0 + r;
        RowRange rr;
        rr.hi = p.kv_len < pos + 1u ? p.kv_len : pos + 1u;
        rr.lo = (p.window > 0u && pos + 1u > p.window) ? pos + 1u - p.window : 0u;
        if (rr.lo > rr.hi) rr.lo = rr.hi;
        return rr;
    };
    const RowRange first = row_range(0), last = row_range(nrows - 1);
    const uint32_t lo_min = first.lo, hi_max = last.hi;          // union of the rows' ranges (both ends grow with the row)
    const uint32_t lo_max = last.lo, hi_min = first.hi;          // positions every row sees: [lo_max, hi_min)
    const uint32_t n = hi_max - lo_min, nsplit = p.num_splits, split = blockIdx.x;
    const uint32_t chunk = (((n + nsplit - 1) / nsplit) + (kTile - 1)) & ~(uint32_t)(kTile - 1);
    const uint32_t c_lo = lo_min + (uint32_t)std::min<uint64_t>(n, (uint64_t)split * chunk);
    const uint32_t c_hi = lo_min + (uint32_t)std::min<uint64_t>(n, (uint64_t)(split + 1) * chunk);
    const bool any = c_hi > c_lo;
    const uint32_t g_first = c_lo >> 6, g_last = any ? (c_hi - 1) >> 6 : 0u;
    const uint32_t full_lo = std::max(c_lo, lo_max), full_hi = std::min(c_hi, hi_min);
    auto tile_full = [&](uint32_t G) { return (G << 6) >= full_lo && (G << 6) + kTile <= full_hi; };
    auto tile_slot = [&](uint32_t G) { const uint32_t s = G << 6; return p.ring_capacity ? s % p.ring_capacity : s; };

    const uint32_t stride = ONE_KV ? (uint32_t)kCodeBytes : p.num_kv_heads * kCodeBytes;
    const uint32_t nstride = ONE_KV ? 2u : p.num_kv_heads * 2;

    // ---- query operands of this wave's row pair, in registers.  MFMA row m = lane % 16 is (row 2 * wave + m / 8, head m % 8);
    //      k group g = lane / 16 covers dims 64g .. 64g + 63; element j of k step (word mw, field pair fp) is dim
    //      64g + 16mw + 4 * (j % 4) + 2fp + j / 4 -- the order in which stage() lays the K levels out.
    f16x8 ahi[8], alo[8];
    float cs;
    {
        const uint32_t q_rho = pcol >> 3, q_h = pcol & 7;
        const uint32_t q_row = std::min<uint32_t>(2 * wave + q_rho, nrows - 1);
        const bool q_on = q_h < group;
        const float* src = a.rq + ((size_t)(row0 + q_row) * p.num_q_heads + (size_t)kvh * group + (q_on ? q_h : 0)) * kHeadDim + 64 * g;
        float x[64];
#pragma unroll
        for (int k = 0; k < 16; k++) {
            const float4 v = *reinterpret_cast<const float4*>(src + 4 * k);
            x[4 * k] = v.x; x[4 * k + 1] = v.y; x[4 * k + 2] = v.z; x[4 * k + 3] = v.w;
        }
        float m = 0.0f;
#pragma unroll
        for (int k = 0; k < 64; k++) {
            if (!q_on) x[k] = 0.0f;
            m = fmaxf(m, fabsf(x[k]));
        }
        m = lh_group_max(m, 64);
        // one power-of-two scale for the pair's 16 queries that brings their largest element to [512, 1024): both f16 parts
        // stay normal numbers, and a query 2^-8 below the largest still keeps 16 bits
        const uint32_t eb = __float_as_uint(m) & 0x7F800000u;
        const bool finite = eb < (255u << 23), sized = eb >= (10u << 23);
        const float s = !finite ? 1.0f : (sized ? __uint_as_float((263u << 23) - eb) : 0.0f);
        cs = !finite ? 1.0f : (sized ? __uint_as_float(eb - (9u << 23)) : 0.0f);
#pragma unroll
        for (int mw = 0; mw < 4; mw++)
#pragma unroll
            for (int fp = 0; fp < 2; fp++)
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    const float v = x[16 * mw + 4 * (j & 3) + 2 * fp + (j >> 2)] * s;
                    const _Float16 h = (_Float16)v;
                    ahi[2 * mw + fp][j] = h;
                    alo[2 * mw + fp][j] = (_Float16)(v - (float)h);
                }
    }
    // ---- phase-A state: the lane's accumulator rows are queries 4g + i of the pair = (row 2 * wave + g / 2, head 4 * (g % 2) + i)
    float R[4], l_run[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        R[i] = kNoRef;
        l_run[i] = 0.0f;
    }
    const RowRange rr = row_range(2 * wave + (g >> 1));
    // ---- phase-B state: output sums of all 128 queries for dims 32 * wave + 4 * (pcol % 8) + 2 * (pcol / 8) + fp
    f32x4 O[kWaves][2];   // [row pair][fp]: queries 4g .. 4g + 3 of the pair
#pragma unroll
    for (int mt = 0; mt < kWaves; mt++) O[mt][0] = O[mt][1] = (f32x4){0.f, 0.f, 0.f, 0.f};

    if (tid < 2 * kWaves) sh.moved[tid >> 3][tid & 7] = 0u;   // row pairs without a row never set theirs
    float v_down = 1.0f, v_up = 1.0f;
    if (any) {
        gptr_t krec0 = (gptr_t)a.k_codes + (size_t)kvh * kCodeBytes + 16 * g + 8 * (wave & 1);
        gptr_t vrec0 = (gptr_t)a.v_codes + (size_t)kvh * kCodeBytes + 8 * wave;
        gptr_t kn0 = (gptr_t)a.k_norms + (size_t)kvh * 2, vn0 = (gptr_t)a.v_norms + (size_t)kvh * 2;
        typedef __attribute__((address_space(3))) uint8_t* lds8_t;
        typedef __attribute__((address_space(3))) v2i* lds_v2i_t;
        const uint32_t s1_q = wave >> 1, s1_half = wave & 1;     // stage(): this wave's 16 positions and half of each 16-byte chunk

        u32x2_t kw, vx;
        float nk_c = 0.0f, nv_c = 0.0f, nk_n, nv_n;
        // Loads of tile G.  Positions outside the chunk are replaced by the nearest one inside it: their logits are masked,
        // so what is loaded for them only has to be finite, and no load is conditional.
        auto load_tile = [&](uint32_t G) {
            const uint32_t t0 = G << 6, pb = tile_slot(G);
            const uint32_t lo_off = c_lo > t0 ? c_lo - t0 : 0u, hi_off = std::min<uint32_t>(c_hi - 1u - t0, 63u);
            const uint32_t ko = std::min(std::max(32 * (s1_q >> 1) + 2 * pcol + (s1_q & 1), lo_off), hi_off);
            const uint32_t vo = std::min(std::max(lane, lo_off), hi_off);
            kw = ld8(krec0 + (size_t)(pb + ko) * stride);
            vx = ld8(vrec0 + (size_t)(pb + vo) * stride);
            nk_n = ld_norm(kn0 + (size_t)(pb + vo) * nstride);
            nv_n = ld_norm(vn0 + (size_t)(pb + vo) * nstride);
        };
        // K codes in kw -> f16 levels in LDS, V codes in vx -> LDS
        auto stage = [&](uint32_t buf, uint32_t vbuf) {
            *reinterpret_cast<u32x2_t*>(&sh.vt[vbuf][wave][lane][0]) = vx;
            const uint32_t w2[2] = {kw.x, kw.y};
#pragma unroll
            for (int mm = 0; mm < 2; mm++) {
                uint32_t d[4][2];
#pragma unroll
                for (int f = 0; f < 4; f++) {
                    const uint32_t c = (w2[mm] >> (2 * f)) & 0x03030303u;
                    const uint32_t lo = __builtin_amdgcn_perm(0u, tl, c), hi = __builtin_amdgcn_perm(0u, th, c);
                    d[f][0] = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
                    d[f][1] = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
                }
#pragma unroll
                for (int fp = 0; fp < 2; fp++)
                    *reinterpret_cast<u32x4_t*>(&sh.kt[buf][s1_q][4 * s1_half + 2 * mm + fp][lane][0]) =
                        (u32x4_t){d[2 * fp][0], d[2 * fp][1], d[2 * fp + 1][0], d[2 * fp + 1][1]};
            }
        };

        // ================================================================= phase A: logits and weights of the wave's two rows
        auto phase_a = [&](uint32_t buf, uint32_t G, auto full_c) {
            constexpr bool full = decltype(full_c)::value;   // every position of the tile is seen by every row: no masks
            const uint32_t t0 = G << 6;
            // column pcol of 16-position tile q is position 32 * (q / 2) + 2 * pcol + q % 2: a lane's weights of tiles 2s and 2s + 1
            // are neighbours in the V-side operand and leave as one packed store
            float kq[4], nvq[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                const int src = 32 * (q >> 1) + 2 * (int)pcol + (q & 1);
                kq[q] = __shfl(nk_c, src, 64) * (kLog2e * cs);
                nvq[q] = fminf(__shfl(nv_c, src, 64) * v_down, 255.0f);   // weight x norm stays within f16 (weights reach 2^kHeadroom = 256)
            }
            f32x4 acc[4];
#pragma unroll
            for (int q = 0; q < 4; q++) acc[q] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < 8; kk++) {
                f16x8 b[4];
#pragma unroll
                for (int q = 0; q < 4; q++) b[q] = *reinterpret_cast<const f16x8*>(&sh.kt[buf][q][kk][lane][0]);
#pragma unroll
                for (int q = 0; q < 4; q++) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi[kk], b[q], acc[q], 0, 0, 0);
#pragma unroll
                for (int q = 0; q < 4; q++) acc[q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo[kk], b[q], acc[q], 0, 0, 0);
            }
            // d = logit - R per [16-position tile][query 4g + i]; the reference R follows the running maximum lazily
            bool seen[4] = {true, true, true, true};
            if constexpr (!full) {   // positions this lane's row does not see (causal end, window start, the chunk's ends)
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t t = t0 + 32 * (q >> 1) + 2 * pcol + (q & 1);
                    seen[q] = t >= rr.lo && t < rr.hi && t >= c_lo && t < c_hi;
                }
            }
            float d[4][4];
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int i = 0; i < 4; i++) d[q][i] = (full || seen[q]) ? __builtin_fmaf(acc[q][i], kq[q], -R[i]) : -INFINITY;
            float over = fmaxf(fmaxf(d[0][0], d[0][1]), fmaxf(d[0][2], d[0][3]));
#pragma unroll
            for (int q = 1; q < 4; q++) over = fmaxf(fmaxf(over, fmaxf(d[q][0], d[q][1])), fmaxf(d[q][2], d[q][3]));
            const bool move = __builtin_amdgcn_ballot_w64(over > kHeadroom) != 0;
            if (move) {   // (also the first tile: against the "nothing seen" reference every logit is far above)
                float fs[4];
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    float lgv[4], mq = -INFINITY;
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        lgv[q] = (full || seen[q]) ? acc[q][i] * kq[q] : -INFINITY;
                        mq = fmaxf(mq, lgv[q]);
                    }
                    const float rn = fmaxf(R[i], lh_group_max(mq, 16));
                    const float f = rn > R[i] ? __builtin_amdgcn_exp2f(R[i] - rn) : 1.0f;   // 0 at the first positions seen
                    R[i] = rn;
                    l_run[i] *= f;
                    fs[i] = f;
#pragma unroll
                    for (int q = 0; q < 4; q++) d[q][i] = lgv[q] - rn;
                }
                if (pcol == 0) {
#pragma unroll
                    for (int i = 0; i < 4; i++) sh.fsc[buf][wave * 16 + 4 * g + i] = fs[i];
                }
            }
            if (lane == 0) sh.moved[buf][wave] = move ? 1u : 0u;
#pragma unroll
            for (int sx = 0; sx < 2; sx++)
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float e0 = __builtin_amdgcn_exp2f(d[2 * sx][i]), e1 = __builtin_amdgcn_exp2f(d[2 * sx + 1][i]);
                    l_run[i] += e0 + e1;
                    // the weights carry the value norm; positions 2 * pcol and 2 * pcol + 1 of the half
                    const f16x2 pk = __builtin_convertvector((f32x2){e0 * nvq[2 * sx], e1 * nvq[2 * sx + 1]}, f16x2);
                    *reinterpret_cast<f16x2*>(&sh.pw[buf][wave][sx][pcol >> 2][(4 * g + i) * 16 + 4 * (pcol & 3)]) = pk;
                }
        };

        // ================================================================= phase B: weights x V levels, dims 32 * wave ..
        auto phase_b = [&](uint32_t buf, uint32_t vbuf) {
            const lds8_t vt = (lds8_t)&sh.vt[vbuf][wave][0][0];
            const uint32_t sh0 = 4 * (pcol >> 3);   // bit position of field 2 * (pcol / 8)
            // V levels of code byte 8 * wave + pcol % 8, fields 2 * (pcol / 8) + fp, positions 32s + 8g + j, j = 0 .. 7 (byte j of
            // the pair z): the lanes 2j and 2j + 1 of a block of 16 both name position j, so that the lanes below and from 8
            // receive the same bytes
            auto v_levels = [&](int s, f16x8 (&bop)[2]) {
                const v2i z = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_t)(vt + (32 * s + 8 * g + (pcol >> 1)) * 8));
#pragma unroll
                for (int fp = 0; fp < 2; fp++) {
                    uint32_t d[4];
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) {
                        const uint32_t c = ((uint32_t)z[hh] >> (sh0 + 2 * fp)) & 0x03030303u;
                        const uint32_t lo = __builtin_amdgcn_perm(0u, tl, c), hi = __builtin_amdgcn_perm(0u, th, c);
                        d[2 * hh] = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
                        d[2 * hh + 1] = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
                    }
                    bop[fp] = __builtin_bit_cast(f16x8, (u32x4_t){d[0], d[1], d[2], d[3]});
                }
            };
            {   // a reference of some row pair moved: its sums follow (rare after a chunk's first tiles; one look at all eight flags)
                const u32x4_t m0 = *reinterpret_cast<const u32x4_t*>(&sh.moved[buf][0]), m1 = *reinterpret_cast<const u32x4_t*>(&sh.moved[buf][4]);
                const uint32_t flags[kWaves] = {m0.x, m0.y, m0.z, m0.w, m1.x, m1.y, m1.z, m1.w};
                if ((m0.x | m0.y | m0.z | m0.w | m1.x | m1.y | m1.z | m1.w) != 0u) {
#pragma unroll
                    for (int mt = 0; mt < kWaves; mt++) {
                        if (flags[mt] != 0u) {
#pragma unroll
                            for (int i = 0; i < 4; i++) {
                                const float fq = sh.fsc[buf][mt * 16 + 4 * g + i];
                                O[mt][0][i] *= fq;
                                O[mt][1][i] *= fq;
                            }
                        }
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < 2; s++) {
                f16x8 bop[2];
                v_levels(s, bop);
#pragma unroll
                for (int mt = 0; mt < kWaves; mt++) {
                    // (row pairs past the end of the chunk multiply whatever their part of LDS holds: never stored)
                    const f16x8 aop = *reinterpret_cast<const f16x8*>(&sh.pw[buf][mt][s][g][pcol * 16]);
                    O[mt][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, bop[0], O[mt][0], 0, 0, 0);
                    O[mt][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, bop[1], O[mt][1], 0, 0, 0);
                }
            }
        };

        load_tile(g_first);
        {   // The weights leave as f16 with the value norm folded in.  So that neither small nor large norms cost them their
            // range, norms are taken relative to a power of two near the largest of the chunk's first tile (the same for
            // every wave: all of them load the same norms); the sums are brought back at the end.  Norms more than 2^8
            // above that one are held there (the outputs then saturate instead of turning into infinities).
            const uint32_t e = lh_group_max_u(__float_as_uint(fabsf(nv_n)), 64) & 0x7F800000u;
            const bool ok = e != 0u && e < (254u << 23);
            v_down = ok ? __uint_as_float((254u << 23) - e) : 1.0f;
            v_up = ok ? __uint_as_float(e) : 1.0f;
        }
        stage(0, 0);
        nk_c = nk_n; nv_c = nv_n;
        if (g_last > g_first) load_tile(g_first + 1);
        __syncthreads();
        // produce(G): weights of tile G, then tile G + 1 staged (its buffers were last read before the previous barrier)
        auto produce = [&](uint32_t G) {
            const uint32_t buf = (G - g_first) & 1;
            // Phase A runs at a raised wave priority: the SIMD's other wave is in phase B or staging meanwhile, and the
            // weights of phase A are what every wave's next phase B waits for behind the barrier (118 -> 113 us for 256 rows
            // over 32768 positions; the priority on phase B or on the staging changes nothing).
            __builtin_amdgcn_s_setprio(1);
            if (pair_on) {
                if (tile_full(G)) phase_a(buf, G, std::true_type{});
                else phase_a(buf, G, std::false_type{});
            }
            __builtin_amdgcn_s_setprio(0);
            if (G < g_last) {
                stage(buf ^ 1, (G + 1 - g_first) & 3);
                nk_c = nk_n; nv_c = nv_n;
                if (G + 1 < g_last) load_tile(G + 2);
            }
        };
        // Between two barriers a wave owes phase B of tile G and the production of tile G + 1, in either order (they touch
        // different buffers).  The upper four waves take them the other way round, so that the two waves of a SIMD are not
        // both in the same phase at the same time.
        const bool b_first = wave < 4;
        produce(g_first);
        __syncthreads();                        // levels of tile G + 1 and weights of tile G are in LDS
        for (uint32_t G = g_first; G <= g_last; G++) {
            const uint32_t buf = (G - g_first) & 1;
            if (b_first) {
                phase_b(buf, (G - g_first) & 3);
                if (G < g_last) produce(G + 1);
            } else {
                if (G < g_last) produce(G + 1);
                phase_b(buf, (G - g_first) & 3);
            }
            if (G < g_last) __syncthreads();
        }
    }

    // ---- totals of the phase-A owners, then every wave writes its 32 dims of all queries
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float l_tot = lh_group_sum(l_run[i], 16);
        if (pcol == 0) {
            const uint32_t qx = wave * 16 + 4 * g + i;
            sh.fin_l[qx] = l_tot;
            sh.fin_r[qx] = R[i] <= 0.5f * kNoRef ? -INFINITY : R[i];
        }
    }
    __syncthreads();
    const uint32_t d0 = 32 * wave + 4 * (pcol & 7) + 2 * (pcol >> 3);
#pragma unroll
    for (int mt = 0; mt < kWaves; mt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q16 = 4 * g + i, r = 2 * mt + (q16 >> 3), h = q16 & 7;
            if (r >= nrows || h >= group) continue;
            const uint32_t qx = mt * 16 + q16, qh = kvh * group + h;
            const float l_tot = sh.fin_l[qx];
            const float2 o = make_float2(O[mt][0][i] * v_up, O[mt][1][i] * v_up);
            if (nsplit == 1) {
                const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
                float* dst = a.out + ((size_t)(row0 + r) * p.num_q_heads + qh) * kHeadDim + d0;
                *reinterpret_cast<float2*>(dst) = make_float2(o.x * inv, o.y * inv);
            } else {
                float* rec = a.ws + (((size_t)(row0 + r) * p.num_q_heads + qh) * nsplit + split) * partial_record_floats(kHeadDim);
                if (wave == 0 && pcol == 0) { rec[0] = sh.fin_r[qx] * kLn2; rec[1] = l_tot; }
                *reinterpret_cast<float2*>(rec + 4 + d0) = o;
            }
        }
}

}  // namespace

namespace lh_attn {

bool prefill_tile_supported(const AttnParams& p, const AttnPointers& a) {
    if (p.mode != kPrefill || p.bits != 2 || p.head_dim != kHeadDim) return false;
    if (p.num_q_heads / p.num_kv_heads > (uint32_t)kHeads) return false;
    if (p.ring_capacity % kTile != 0) return false;
    if (p.num_queries < 2) return false;                                  // a single row is the decode kernel's job
    if (((uintptr_t)a.k_codes | (uintptr_t)a.v_codes) & 3) return false;
    if (((uintptr_t)a.k_norms | (uintptr_t)a.v_norms) & 1) return false;
    if (((uintptr_t)a.rq | (uintptr_t)a.out) & 15) return false;
    return true;
}

int launch_prefill_tile(lh_context* ctx, const char* op, const AttnPointers& a, AttnParams& p, uint64_t max_span, size_t ws_floats) {
    const uint64_t tiles = ((uint64_t)p.num_queries + kRows - 1) / kRows * p.num_kv_heads;
    // one eight-wave workgroup per CU over the whole launch, at least 256 positions per workgroup
    uint64_t splits = std::max<uint64_t>(1, (uint64_t)ctx->cu_count / tiles);
    splits = std::min<uint64_t>(splits, (max_span + 255) / 256);
    splits = std::min<uint64_t>(std::max<uint64_t>(splits, 1), kMaxSplits);
    const size_t rec = partial_record_floats(p.head_dim);
    while (splits > 1 && (size_t)p.num_queries * p.num_q_heads * splits * rec > ws_floats) splits--;
    p.num_splits = (uint32_t)splits;
    const dim3 grid((uint32_t)splits, (uint32_t)tiles);
    if (p.num_kv_heads == 1) hipLaunchKernelGGL(attention_tq_prefill_tile_kernel<true>, grid, dim3(512), 0, ctx->stream, a, p);
    else hipLaunchKernelGGL(attention_tq_prefill_tile_kernel<false>, grid, dim3(512), 0, ctx->stream, a, p);
    return lh_check_launch(op);
}

}  // namespace lh_attn
