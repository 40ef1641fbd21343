// Tiled prefill attention over packed 2-bit TurboQuant codes on the matrix cores.
//
// Stands in for flash_attention_tq_prefill_tiled (shaders/attention_flash_tq.metal:425-556, chosen at
// local-engine/src/kv_cache/quant_cache.rs:641-667): several query rows of a prefill chunk share one pass over a tile
// of K/V codes.  The per-query decode kernel (attention_tq_mfma.hip) spends most of its time on work that is per
// (query row, position) whatever the tiling -- turning softmax weights into integer limbs and its integer sums back
// into floats -- so this kernel keeps that kernel's K side and replaces its V side:
//   K side  exactly as in the decode kernel: the rotated queries of one row's 8 heads as 16-bit block fixed point in
//           two int8 limbs (16 MFMA rows), the K codes' bit planes isolated with one AND per four codes and fed to
//           v_mfma_i32_16x16x64_i8 as they are; the planes are isolated ONCE per tile and used by every row of the
//           workgroup.  logit = norm_k * (scale_h * int + alpha * sum(rq_h)), no 1/sqrt(d) factor
//           (attention_flash_tq.metal:175-273).
//   V side  softmax weights times the value norm leave as f16 (relative to a reference that follows the running maximum
//           lazily, so they stay within f16 range) and are the A operand of v_mfma_f32_16x16x32_f16: 16 rows = the 8
//           heads of two query rows, k = 32 positions.  The B operand is the level table itself: V codes pass through
//           LDS and come back transposed (ds_read_b64_tr_b8: one code byte over eight positions), two byte permutes
//           look the f16 level of each 2-bit field up, two more interleave the bytes.  The V tile is decoded once for
//           all rows of the workgroup and the sums accumulate in f32 registers: no limbs, no per-tile scales.
// A workgroup is four waves and eight query rows.  Per tile of 64 positions, phase A: wave w computes logits and
// weights of rows 2w, 2w + 1 (64 int8 MFMAs) and parks the weights in LDS; phase B: wave w multiplies the weights of
// all 64 queries with the V levels of code bytes 16w .. 16w + 15, i.e. 64 of the 256 output dims (32 f16 MFMAs).
// Positions are split over gridDim.x workgroups per row tile; partials (R, l, acc) go to the workspace in the decode
// kernel's record layout and are merged by the same merge kernels.
#include "attention_tq.hpp"
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace {
using namespace lh_attn;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef const __attribute__((address_space(1))) uint8_t* gptr_t;

constexpr int kRows = 8;               // query rows per workgroup
constexpr int kTile = 64;              // positions per step
constexpr int kHeads = 8;              // query heads per KV head served by the 16 MFMA rows
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kQmax = 32639.0f;      // 127 * 256 + 127
constexpr float kHeadroom = 8.0f;      // log2 of how far a weight may exceed the softmax reference before that moves (f16 range)
constexpr float kNoRef = -1.0e30f;     // "no position seen yet": finite, so that exp2(logit - R) of a masked logit is 0, not NaN

__device__ __forceinline__ u32x4_t ld16(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(4))) u32x4_a4;
    return *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a4*>(p);
}
__device__ __forceinline__ float ld_norm(gptr_t p) {
    return lh_h2f(*reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>(p));
}

struct PrefillShared {
    uint8_t rqop[kRows][8][64][16];    // K-side A operands per (row, plane * 4 + field) and lane
    uint8_t pw[4][2][4][16][16];       // weights as f16, [row pair][32-position half][k group][query of the pair][8 positions]
    uint8_t vt[4][kTile * 16];         // [wave]: its 16 code bytes of the tile's 64 positions, read back transposed
    float fsc[kRows * kHeads];         // per query: factor for its output sums when its reference moved in this tile
    uint32_t moved[4];                 // [wave]: a reference moved in this tile
    float maxabs[kRows][kHeads], sum[kRows][kHeads];
    float fin_l[kRows * kHeads], fin_r[kRows * kHeads];
};

struct RowRange { uint32_t lo, hi; };

template <bool ONE_KV>
__global__ __launch_bounds__(256, 2) void attention_tq_prefill_mfma_kernel(AttnPointers a, AttnParams p, uint32_t* fault) {
    __shared__ __align__(16) PrefillShared sh;
    constexpr int kHeadDim = 256, kCodeBytes = 64;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t pcol = lane & 15, g = lane >> 4;
    const uint32_t rt = blockIdx.y / p.num_kv_heads, kvh = blockIdx.y - rt * p.num_kv_heads;
    const uint32_t group = p.num_q_heads / p.num_kv_heads;
    const uint32_t row0 = rt * kRows;
    const uint32_t nrows = std::min<uint32_t>((uint32_t)kRows, p.num_queries - row0);

    // L[c] = alpha + beta*bit0 + gam*bit1 (the dispatcher only sends level tables that are affine in the code bits here)
    const float L0 = a.levels[0], L1 = a.levels[1], L2 = a.levels[2], L3 = a.levels[3];
    const float d_raw = (L3 - L2) - (L1 - L0);
    const float alpha = L0 - 0.25f * d_raw, beta = (L1 - L0) + 0.5f * d_raw, gam = (L2 - L0) + 0.5f * d_raw;
    const float cmax_k = fmaxf(fabsf(beta), fabsf(0.5f * gam));
    {   // the host chose this kernel by what was uploaded into the table's buffer; a table that is not affine in the code
        // bits after all is reported, and nothing is computed
        const float lmax = fmaxf(fmaxf(fabsf(L0), fabsf(L1)), fmaxf(fabsf(L2), fabsf(L3)));
        if (!(fabsf(d_raw) <= 1e-5f * lmax)) {
            if (threadIdx.x == 0 && blockIdx.x == 0 && blockIdx.y == 0 && fault)
                __hip_atomic_store(fault, (uint32_t)LH_FAULT_PREFILL_LEVELS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
            return;
        }
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

    // ---- per (row, head): max |rq| (quantisation scale) and sum(rq) (constant term of the level table)
    for (uint32_t rh = tid >> 5; rh < (uint32_t)(kRows * kHeads); rh += 8) {
        const uint32_t r = rh >> 3, h = rh & 7, sub = tid & 31;
        float m = 0.0f, s = 0.0f;
        if (r < nrows && h < group) {
            const float* src = a.rq + ((size_t)(row0 + r) * p.num_q_heads + (size_t)kvh * group + h) * kHeadDim + sub * 8;
            const float4 x0 = *reinterpret_cast<const float4*>(src), x1 = *reinterpret_cast<const float4*>(src + 4);
            const float v[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
            for (int i = 0; i < 8; i++) { m = fmaxf(m, fabsf(v[i])); s += v[i]; }
        }
        m = lh_group_max(m, 32);
        s = lh_group_sum(s, 32);
        if (sub == 0) { sh.maxabs[r][h] = m; sh.sum[r][h] = s; }
    }
    __syncthreads();

    // ---- K-side A operands.  MFMA row rr: head (rr / 4) + 4 * ((rr / 2) % 2), limb rr % 2; k slot (word m, byte e) of
    //      k group g is code byte 16g + 4m + e, i.e. dim 4 * (that byte) + f for the operand of field f.  The lanes pcol and
    //      pcol ^ 1 serve the two limbs of one head: each quantises half of the words and they swap.
    {
        const uint32_t h_op = (pcol >> 2) + 4 * ((pcol >> 1) & 1), limb_op = pcol & 1;
        for (uint32_t unit = wave; unit < (uint32_t)(kRows * 2); unit += 4) {   // (row, plane)
            const uint32_t r = unit >> 1, pl = unit & 1;
            const bool on = r < nrows && h_op < group;
            const float ma = sh.maxabs[r][h_op];
            const float inv = (on && ma > 0.0f && cmax_k > 0.0f) ? kQmax / (ma * cmax_k) : 0.0f;
            const float mul = (pl == 0 ? beta : 0.5f * gam) * inv;
            const float* src = a.rq + ((size_t)(row0 + (on ? r : 0)) * p.num_q_heads + (size_t)kvh * group + (on ? h_op : 0)) * kHeadDim;
            uint32_t wlo[4][2], whi[4][2];
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int mm = 0; mm < 2; mm++) wlo[f][mm] = whi[f][mm] = 0;
#pragma unroll
            for (int mm = 0; mm < 2; mm++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float4 x = *reinterpret_cast<const float4*>(src + 4 * (16 * g + 4 * (2 * limb_op + mm) + e));
                    const float xv[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
                    for (int f = 0; f < 4; f++) {
                        float q = __builtin_rintf(xv[f] * mul);
                        q = fminf(fmaxf(q, -kQmax), kQmax);
                        const int nq = (int)q;
                        const int lo = (int)(int8_t)(nq & 0xFF);
                        wlo[f][mm] |= (uint32_t)(lo & 0xFF) << (8 * e);
                        whi[f][mm] |= (uint32_t)(((nq - lo) >> 8) & 0xFF) << (8 * e);
                    }
                }
#pragma unroll
            for (int f = 0; f < 4; f++) {
                uint32_t words[4];
#pragma unroll
                for (int mm = 0; mm < 2; mm++) {
                    const uint32_t mine = limb_op ? whi[f][mm] : wlo[f][mm];
                    const uint32_t give = limb_op ? wlo[f][mm] : whi[f][mm];
                    const uint32_t got = (uint32_t)__builtin_amdgcn_mov_dpp((int)give, 0xB1, 0xF, 0xF, true);   // lane ^ 1
                    words[mm] = limb_op ? got : mine;        // words 0, 1 were quantised by the limb-0 lane
                    words[2 + mm] = limb_op ? mine : got;    // words 2, 3 by the limb-1 lane
                }
                *reinterpret_cast<u32x4_t*>(&sh.rqop[r][pl * 4 + f][lane][0]) = (u32x4_t){words[0], words[1], words[2], words[3]};
            }
        }
    }
    __syncthreads();

    // ---- phase-A state of this wave: rows 2 * wave + rho, heads g and g + 4 in the lane's two head sets
    float cs[2][2], ca[2][2], R[2][2], l_run[2][2];
    RowRange rr[2];
#pragma unroll
    for (int rho = 0; rho < 2; rho++) {
        rr[rho] = row_range(2 * wave + rho);
#pragma unroll
        for (int hs = 0; hs < 2; hs++) {
            const uint32_t h = g + 4 * hs;
            cs[rho][hs] = sh.maxabs[2 * wave + rho][h] * cmax_k * (0.25f / kQmax);
            ca[rho][hs] = alpha * sh.sum[2 * wave + rho][h];
            R[rho][hs] = kNoRef;
            l_run[rho][hs] = 0.0f;
        }
    }
    // ---- phase-B state: output sums of all 64 queries (4 row pairs x 16) for dims 64 * wave + 4 * pcol + f, f = 0..3
    f32x4 O[4][4];   // [row pair][field]: rows 4g .. 4g + 3 of the pair's 16 queries, column pcol = code byte 16 * wave + pcol
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int f = 0; f < 4; f++) O[mt][f] = (f32x4){0.f, 0.f, 0.f, 0.f};
    // the level table as two byte tables for v_perm_b32: byte c of tl / th = low / high byte of f16(L[c])
    uint32_t tl = 0, th = 0;
    {
        const float lv[4] = {L0, L1, L2, L3};
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const uint32_t hbits = lh_f2h(lv[c]);
            tl |= (hbits & 0xFFu) << (8 * c);
            th |= (hbits >> 8) << (8 * c);
        }
    }

    float v_down = 1.0f, v_up = 1.0f;
    if (any) {
        gptr_t krec0 = (gptr_t)a.k_codes + (size_t)kvh * kCodeBytes;
        gptr_t vrec0 = (gptr_t)a.v_codes + (size_t)kvh * kCodeBytes + 16 * wave;
        gptr_t kn0 = (gptr_t)a.k_norms + (size_t)kvh * 2, vn0 = (gptr_t)a.v_norms + (size_t)kvh * 2;
        const uint32_t klane = pcol * stride + 16 * g;
        typedef __attribute__((address_space(3))) uint8_t* lds8_t;
        typedef __attribute__((address_space(3))) v2i* lds_v2i_t;
        typedef __attribute__((address_space(3))) u32x4_t* lds_x4_t;
        const lds8_t vt = (lds8_t)&sh.vt[wave][0];

        u32x4_t kw[4], vx;
        float nk, nv;
        // loads of tile G: unconditional when the whole tile lies inside the chunk, else only the chunk's positions
        auto load_tile = [&](bool inside, uint32_t G) {
            const uint32_t pb = tile_slot(G), t0 = G << 6;
            gptr_t kb = krec0 + (size_t)pb * stride, vb = vrec0 + (size_t)pb * stride;
            gptr_t knb = kn0 + (size_t)pb * nstride, vnb = vn0 + (size_t)pb * nstride;
            if (inside) {
#pragma unroll
                for (int q = 0; q < 4; q++) kw[q] = ld16(kb + (size_t)(16 * q) * stride + klane);
                vx = ld16(vb + (size_t)lane * stride);
                nk = ld_norm(knb + lane * nstride);
                nv = ld_norm(vnb + lane * nstride);
            } else {
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    kw[q] = (u32x4_t){0u, 0u, 0u, 0u};
                    const uint32_t t = t0 + 16 * q + pcol;
                    if (t >= c_lo && t < c_hi) kw[q] = ld16(kb + (size_t)(16 * q) * stride + klane);
                }
                vx = (u32x4_t){0u, 0u, 0u, 0u};
                nk = nv = 0.0f;
                const uint32_t t = t0 + lane;
                if (t >= c_lo && t < c_hi) {
                    vx = ld16(vb + (size_t)lane * stride);
                    nk = ld_norm(knb + lane * nstride);
                    nv = ld_norm(vnb + lane * nstride);
                }
            }
        };
        auto tile_inside = [&](uint32_t G) { return (G << 6) >= c_lo && (G << 6) + kTile <= c_hi; };

        // One tile.  `full`: every position of the tile is seen by every row (no masks to apply).
        // `next`: 0 nothing follows, 1 the next tile lies inside the chunk (unconditional loads), 2 it may not.
        auto step = [&](bool full, uint32_t G, int next) {
            const uint32_t t0 = G << 6;
            // this wave's V codes of the tile go to its LDS area now: their registers take the next tile's below
            __builtin_amdgcn_wave_barrier();
            *(lds_x4_t)(vt + lane * 16) = vx;
            __builtin_amdgcn_wave_barrier();
            // ================================================================= phase A: logits and weights of two rows
            // (row by row: a row's eight operands stay in registers over the four 16-position tiles, and the bit planes
            // of a tile are isolated again for the second row -- 36 cheap instructions against 32 KB of LDS reads)
            float nkq[4], nvq[4];
#pragma unroll
            for (int q = 0; q < 4; q++) {
                nkq[q] = __shfl(nk, 16 * q + (int)pcol, 64) * kLog2e;
                nvq[q] = fminf(__shfl(nv, 16 * q + (int)pcol, 64) * v_down, 255.0f);   // weight x norm stays within f16 (weights reach 2^kHeadroom = 256)
            }
            bool moved_any = false;
            float fs[2][2] = {{1.0f, 1.0f}, {1.0f, 1.0f}};
#pragma unroll
            for (int rho = 0; rho < 2; rho++) {
                const v4i* rqo = reinterpret_cast<const v4i*>(&sh.rqop[2 * wave + rho][0][lane][0]);   // operand (pl, f) at rqo[64 * (4 * pl + f)]
                v4i aop[8];
#pragma unroll
                for (int o = 0; o < 8; o++) aop[o] = rqo[64 * o];
                // (opaque to the compiler on purpose: it would otherwise keep the first row's 128 plane registers for the second)
#pragma unroll
                for (int q = 0; q < 4; q++) asm volatile("" : "+v"(kw[q]));
                float lg[4][2];
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    const uint32_t w[4] = {kw[q].x, kw[q].y, kw[q].z, kw[q].w};
                    v4i b00, b10, b01, b11, b02, b12, b03, b13;   // b<plane><field>
#pragma unroll
                    for (int m = 0; m < 4; m++) {
                        const uint32_t u = w[m] >> 4;
                        b00[m] = (int)(w[m] & 0x01010101u); b10[m] = (int)(w[m] & 0x02020202u);
                        b01[m] = (int)(w[m] & 0x04040404u); b11[m] = (int)(w[m] & 0x08080808u);
                        b02[m] = (int)(u & 0x01010101u);    b12[m] = (int)(u & 0x02020202u);
                        b03[m] = (int)(u & 0x04040404u);    b13[m] = (int)(u & 0x08080808u);
                    }
                    v4i acc1, acc4;   // fields 0, 2 arrive x1, fields 1, 3 x4
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[0], b00, (v4i){0, 0, 0, 0}, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[1], b01, (v4i){0, 0, 0, 0}, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[4], b10, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[5], b11, acc4, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[2], b02, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[3], b03, acc4, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[6], b12, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(aop[7], b13, acc4, 0, 0, 0);
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        uint32_t t1 = ((uint32_t)acc1[2 * hs + 1] << 8) + (uint32_t)acc1[2 * hs];
                        uint32_t t4 = ((uint32_t)acc4[2 * hs + 1] << 8) + (uint32_t)acc4[2 * hs];
                        asm("" : "+v"(t1), "+v"(t4));
                        const float inner = (float)(int)((t1 << 2) + t4) * cs[rho][hs] + ca[rho][hs];
                        lg[q][hs] = nkq[q] * inner;
                    }
                }
                if (rho == 1 && next) load_tile(next == 1, G + 1);   // the code registers and norms are free
                if (!full) {   // positions this row does not see (causal end, window start, the chunk's ends)
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const uint32_t t = t0 + 16 * q + pcol;
                        const bool seen = t >= rr[rho].lo && t < rr[rho].hi && t >= c_lo && t < c_hi;
                        if (!seen) lg[q][0] = lg[q][1] = -INFINITY;
                    }
                }
                // softmax weights relative to the reference R, which follows the running maximum lazily
                float mq[2];
#pragma unroll
                for (int hs = 0; hs < 2; hs++) mq[hs] = fmaxf(fmaxf(lg[0][hs], lg[1][hs]), fmaxf(lg[2][hs], lg[3][hs]));
                const bool move = __builtin_amdgcn_ballot_w64(fmaxf(mq[0] - R[rho][0], mq[1] - R[rho][1]) > kHeadroom) != 0;
                if (move) {
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        const float rn = fmaxf(R[rho][hs], lh_group_max(mq[hs], 16));
                        const float fsc = rn > R[rho][hs] ? __builtin_amdgcn_exp2f(R[rho][hs] - rn) : 1.0f;   // 0 at the first positions seen
                        R[rho][hs] = rn;
                        l_run[rho][hs] *= fsc;
                        fs[rho][hs] = fsc;
                    }
                    moved_any = true;
                }
#pragma unroll
                for (int hs = 0; hs < 2; hs++) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const float ew = __builtin_amdgcn_exp2f(lg[q][hs] - R[rho][hs]);
                        l_run[rho][hs] += ew;
                        const uint32_t sx = q >> 1, kg = 2 * (q & 1) + (pcol >> 3);
                        *reinterpret_cast<uint16_t*>(&sh.pw[wave][sx][kg][rho * 8 + g + 4 * hs][2 * (pcol & 7)]) = lh_f2h(ew * nvq[q]);   // the weight carries the value norm
                    }
                }
            }
            if (moved_any && pcol == 0) {
#pragma unroll
                for (int rho = 0; rho < 2; rho++)
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) sh.fsc[(2 * wave + rho) * kHeads + g + 4 * hs] = fs[rho][hs];
            }
            if (lane == 0) sh.moved[wave] = moved_any ? 1u : 0u;
            __syncthreads();   // weights, factors and flags of all four waves are in LDS
            // ================================================================= phase B: weights x V levels, dims 64 * wave ..
#pragma unroll
            for (int mt = 0; mt < 4; mt++) {
                if (sh.moved[mt] != 0) {   // a reference of this row pair moved: its sums follow (uniform, and rare after a chunk's first tiles)
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float fq = sh.fsc[mt * 16 + 4 * g + i];
#pragma unroll
                        for (int f = 0; f < 4; f++) O[mt][f][i] *= fq;
                    }
                }
            }
#pragma unroll
            for (int s = 0; s < 2; s++) {
                // code byte 16 * wave + pcol of positions 32s + 8g + j, j = 0 .. 7 (byte j of the pair z)
                const v2i z = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_t)(vt + 512 * s + 8 * lane));
                f16x8 bop[4];
#pragma unroll
                for (int f = 0; f < 4; f++) {
                    uint32_t d[4];
#pragma unroll
                    for (int hh = 0; hh < 2; hh++) {
                        const uint32_t c = ((uint32_t)z[hh] >> (2 * f)) & 0x03030303u;
                        const uint32_t lo = __builtin_amdgcn_perm(0u, tl, c), hi = __builtin_amdgcn_perm(0u, th, c);
                        d[2 * hh] = __builtin_amdgcn_perm(hi, lo, 0x05010400u);
                        d[2 * hh + 1] = __builtin_amdgcn_perm(hi, lo, 0x07030602u);
                    }
                    bop[f] = __builtin_bit_cast(f16x8, (u32x4_t){d[0], d[1], d[2], d[3]});
                }
#pragma unroll
                for (int mt = 0; mt < 4; mt++) {
                    const f16x8 aop = *reinterpret_cast<const f16x8*>(&sh.pw[mt][s][g][pcol][0]);
#pragma unroll
                    for (int f = 0; f < 4; f++) O[mt][f] = __builtin_amdgcn_mfma_f32_16x16x32_f16(aop, bop[f], O[mt][f], 0, 0, 0);
                }
            }
            __syncthreads();   // every wave has read the weights: the next tile may overwrite them
        };
        load_tile(tile_inside(g_first), g_first);
        {   // The weights leave as f16 with the value norm folded in.  So that neither small nor large norms cost them their
            // range, norms are taken relative to a power of two near the largest of the chunk's first tile (the same for
            // every wave: all of them load the same norms); the sums are brought back at the end.  Norms more than 2^8
            // above that one are held there (the outputs then saturate instead of turning into infinities).
            const uint32_t e = lh_group_max_u(__float_as_uint(fabsf(nv)), 64) & 0x7F800000u;
            const bool ok = e != 0u && e < (254u << 23);
            v_down = ok ? __uint_as_float((254u << 23) - e) : 1.0f;
            v_up = ok ? __uint_as_float(e) : 1.0f;
        }
        for (uint32_t G = g_first; G <= g_last; G++) {
            const int next = G == g_last ? 0 : (tile_inside(G + 1) ? 1 : 2);
            step(tile_full(G), G, next);
        }
    }

    // ---- totals of the phase-A owners, then every wave writes its 64 dims of all queries
#pragma unroll
    for (int rho = 0; rho < 2; rho++)
#pragma unroll
        for (int hs = 0; hs < 2; hs++) {
            const float l_tot = lh_group_sum(l_run[rho][hs], 16);
            if (pcol == 0) {
                const uint32_t qx = (2 * wave + rho) * kHeads + g + 4 * hs;
                sh.fin_l[qx] = l_tot;
                sh.fin_r[qx] = R[rho][hs] <= 0.5f * kNoRef ? -INFINITY : R[rho][hs];
            }
        }
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < 4; mt++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t q16 = 4 * g + i, r = 2 * mt + (q16 >> 3), h = q16 & 7;
            if (r >= nrows || h >= group) continue;
            const uint32_t qx = r * kHeads + h, qh = kvh * group + h;
            const float l_tot = sh.fin_l[qx];
            const float4 o = make_float4(O[mt][0][i] * v_up, O[mt][1][i] * v_up, O[mt][2][i] * v_up, O[mt][3][i] * v_up);
            if (nsplit == 1) {
                const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
                float* dst = a.out + ((size_t)(row0 + r) * p.num_q_heads + qh) * kHeadDim + 64 * wave + 4 * pcol;
                *reinterpret_cast<float4*>(dst) = make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
            } else {
                float* rec = a.ws + (((size_t)(row0 + r) * p.num_q_heads + qh) * nsplit + split) * partial_record_floats(kHeadDim);
                if (wave == 0 && pcol == 0) { rec[0] = sh.fin_r[qx] * kLn2; rec[1] = l_tot; }
                *reinterpret_cast<float4*>(rec + 4 + 64 * wave + 4 * pcol) = o;
            }
        }
}

}  // namespace

namespace lh_attn {

bool prefill_mfma_supported(const AttnParams& p, const AttnPointers& a) {
    if (p.mode != kPrefill || p.bits != 2 || p.head_dim != 256) return false;
    if (p.num_q_heads / p.num_kv_heads > (uint32_t)kHeads) return false;
    if (p.ring_capacity % kTile != 0) return false;
    if (p.num_queries < 2) return false;                                  // a single row is the decode kernel's job
    if (((uintptr_t)a.k_codes | (uintptr_t)a.v_codes) & 3) return false;
    if (((uintptr_t)a.k_norms | (uintptr_t)a.v_norms) & 1) return false;
    if (((uintptr_t)a.rq | (uintptr_t)a.out) & 15) return false;
    return true;
}

int launch_prefill_mfma(lh_context* ctx, const char* op, const AttnPointers& a, AttnParams& p, uint64_t max_span, size_t ws_floats) {
    const uint64_t tiles = ((uint64_t)p.num_queries + kRows - 1) / kRows * p.num_kv_heads;
    // about two workgroups per CU over the whole launch, at least 256 positions per workgroup
    uint64_t splits = std::max<uint64_t>(1, (uint64_t)ctx->cu_count * 2 / tiles);
    splits = std::min<uint64_t>(splits, (max_span + 255) / 256);
    splits = std::min<uint64_t>(std::max<uint64_t>(splits, 1), kMaxSplits);
    const size_t rec = partial_record_floats(p.head_dim);
    while (splits > 1 && (size_t)p.num_queries * p.num_q_heads * splits * rec > ws_floats) splits--;
    p.num_splits = (uint32_t)splits;
    const dim3 grid((uint32_t)splits, (uint32_t)tiles);
    if (p.num_kv_heads == 1) hipLaunchKernelGGL(attention_tq_prefill_mfma_kernel<true>, grid, dim3(256), 0, ctx->stream, a, p, ctx->fault_dev);
    else hipLaunchKernelGGL(attention_tq_prefill_mfma_kernel<false>, grid, dim3(256), 0, ctx->stream, a, p, ctx->fault_dev);
    return lh_check_launch(op);
}

}  // namespace lh_attn
