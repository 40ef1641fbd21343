// Flash-decoding attention over packed 2-bit TurboQuant codes on the matrix cores.
//
// Same contract as attention_tq.hip (stands in for shaders/attention_flash_tq.metal:154-690); this
// kernel takes the common case -- 2-bit codes, head_dim 256 or 512, up to 8 query heads per KV head -- and
// runs at more than half of the HBM rate instead of at a hundredth of it.  Per cached position the path
// moves 132 bytes and needs 8192 multiply-adds (8 heads x 256 dims x {K, V}); decoding every code to a
// float and multiplying on the vector ALU costs ~40x more issue slots than the memory stream leaves free.
//
// The 2-bit level table is written as L[c] = a + b*bit0(c) + g*bit1(c) (+ d*bit0*bit1, which is zero for
// the symmetric Lloyd-Max tables and costs a third bit plane otherwise).  Bit planes are isolated with
// one AND per four codes and fed to v_mfma_i32_16x16x64_i8 as they are; what multiplies them is
// quantised to fixed point and split into signed 8-bit limbs, one MFMA row per (query head, limb):
//   K side:  rows = 8 heads x 2 limbs of b*rq and g/2*rq (16-bit block fixed point per head), columns =
//            16 positions, k = 64 code bytes;  logit = norm_k * (scale_h * int + a * sum(rq_h)).
//   V side:  rows = 8 heads x 2 limbs of w = exp2(logit - R_h) * norm_v in 16-bit fixed point relative to
//            the head's largest weight of the current hand-over (64 or 128 positions; a power-of-two scale,
//            round to nearest), columns = 16 code-byte columns (x 4 fields), k = 64 positions; the planes share
//            one accumulator because their coefficients are folded into w before quantisation, and they are
//            meant as centred bits (b - 1/2): the sum of the quantised weights is taken off at the end.  The
//            position-major codes become "one code byte over many positions" operands on their way through the
//            wave's LDS area: stored as loaded, read back with the transposing read ds_read_b64_tr_b8.
// One workgroup owns a chunk of positions and walks it in aligned groups of 64: the K wave produces the
// softmax weights of a group (or of an aligned pair of groups, for long chunks), a V wave per 256 output
// dims, one hand-over behind with one barrier per hand-over, turns them into limbs, multiplies and adds
// the integer sums to its float outputs with the hand-over's scale.  A scale per head and hand-over keeps
// the long tail of a soft distribution: a weight is only compared with the 63 or 127 around it, never with
// a maximum seen thousands of positions earlier.  The softmax reference R_h only keeps exp2 in range and
// follows the running maximum lazily.  Splitting the roles lets two waves share a SIMD and fill each
// other's stalls.  head_dim 512 has two K waves, one per 64-byte half of the K codes: the second runs a
// further hand-over ahead and passes its integer logit sums to the first.  Partials (R, l, acc) per chunk
// go to the workspace for the merge kernel.
#include "attention_tq.hpp"
#include <atomic>
#include <algorithm>
#include <cstdlib>
#include <type_traits>

namespace {
using namespace lh_attn;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef unsigned short us2_t __attribute__((ext_vector_type(2)));
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
typedef const __attribute__((address_space(1))) uint8_t* gptr_t;

constexpr int kGroup = 64;             // positions per loop step: 4 K-side MFMA tiles, one V-side MFMA k-step
constexpr int kMaxGroupHeads = 8;      // query heads per KV head served by the 16 MFMA rows
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;
constexpr float kQmax = 32639.0f;      // 127 * 256 + 127
constexpr float kHeadroom = 32.0f;     // log2 of how far a weight may exceed the softmax reference before that moves

__device__ __forceinline__ u32x4_t ld16(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(4))) u32x4_a4;
    return *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a4*>(p);
}
__device__ __forceinline__ uint32_t ld4(gptr_t p) { return *reinterpret_cast<const __attribute__((address_space(1))) uint32_t*>(p); }
__device__ __forceinline__ float ld_norm(gptr_t p) {
    return lh_h2f(*reinterpret_cast<const __attribute__((address_space(1))) uint16_t*>(p));
}

struct GroupGeom {
    uint32_t pb;        // physical slot of the group's first position
    uint32_t vlo, vhi;  // valid positions of the group: [vlo, vhi) within 0..64
    bool full;
};

// One workgroup = two waves on one chunk of positions: the "K wave" turns K codes into softmax weights, the "V wave"
// multiplies them with the V codes.  The K wave runs one hand-over ahead; one workgroup barrier per hand-over passes a
// double-buffered set of weights, their scales and the rare "reference moved" message.  A hand-over is one group of 64
// positions (PS = 1: short chunks, where the pipeline's fill and drain count) or an aligned pair of groups (PS = 2: long
// chunks, where halving the per-hand-over work -- scales, the integer sums' way into the float outputs -- counts).
// Several chunks per workgroup: a chunk's K wave and V wave meet at their hand-overs through counters in LDS, not at a
// workgroup barrier (256 sequences x 32768 positions: 0.627-0.631 -> 0.644-0.646 of the HBM rate in alternating runs).
constexpr bool kPairSync = true;
template <int NH, int PS>   // NH = 64-byte halves of a position's code (head_dim / 256) = number of V waves; PS = groups per hand-over
struct AttnShared {
    uint8_t rqop[12 * NH][64][16]; // K-side A operands per (code half, plane, field) and lane
    float4 norm[kGroup];           // K wave: (norm_k*log2e, mask bias, norm_v, -) per group position
    float4 ww[2][PS][2][64];       // [buffer][group of the pair][head set][lane]: the K wave's weights of tiles 0..3, for the V wave
    float2 wsc[2][kMaxGroupHeads]; // [buffer][head]: (scale that takes the head's weights of this pair into [-1, 1], value of one integer step)
    uint8_t wx[NH][3][1024];       // [V wave][plane]: that wave's A operands (weights as limbs)
    uint8_t vt[NH][kGroup * 64];   // [V wave]: a group's V codes (64 bytes per position, 16-byte chunks swizzled), read back transposed
    v4i tb[NH == 2 ? 2 : 1][PS][2][64]; // head_dim 512: [buffer][group of the pair][head set][lane]: the second K wave's integer logit sums of tiles 0..3 (code half 1)
    float fsc[2][kMaxGroupHeads];  // [buffer][head]: factor for the float outputs when the reference moved
    uint32_t moved[2];             // [buffer]: the reference moved within this pair: rescale the outputs
    float fin_l[kMaxGroupHeads], fin_w[kMaxGroupHeads], fin_r[kMaxGroupHeads];
    float maxabs[kMaxGroupHeads], sum[kMaxGroupHeads];
    uint32_t psync[2];             // several chunks per workgroup: hand-overs the K wave / the V wave of this chunk has reached
    uint32_t pair_spin_limit;      // polls a wave spends at one hand-over before it gives up (copied from the launch parameters)
};

// NPL = number of bit planes: 2 when the level table is affine in the code bits, 3 with the bit0*bit1 plane.
// HD = head_dim: 256 (one V wave) or 512 (two V waves, one per 64-byte half of a position's code).
// ONE_KV: a single KV head (the measured configuration and the reference model): the distance between positions is a
// compile-time constant, so the loads of a group take immediate offsets instead of per-load address arithmetic.
// NQ = chunks per workgroup: 1, or 2 or 4 (head_dim 256): four or eight waves, a K wave and a V wave per chunk, each
// pair of waves with a hand-over area of its own; the query set-up is done once, by all eight, and the four partial results
// are merged through LDS, so that a query cut into four chunks needs neither partial records nor a merge launch.  The
// hand-over barriers are workgroup barriers, so every wave executes as many as the chunk with the most hand-overs needs.
template <int NPL, int HD, bool ONE_KV, int PS, int NQ = 1>
__device__ __forceinline__ void attention_body(const AttnPointers& a, const AttnParams& p, AttnShared<(HD / 256), PS>* shs, float alpha, float beta,
                                               float gam, float delta) {
    static_assert(NQ == 1 || ((NQ == 2 || NQ == 4) && HD == 256), "several chunks per workgroup: head_dim 256 only");
    // The wave's index as a scalar: what follows from it -- the chunk, its groups, their ring slots, the roles -- is uniform
    // over the wave, and the compiler keeps it in scalar registers and scalar branches only if it can see that (per pair
    // hand-over 36 vector instructions fewer on the K wave and 116 on the V wave of a several-chunk workgroup).  That is
    // what the latency-bound launches want (one query over 32768 positions: 12.2-12.4 against 12.5-12.7 us; over 131072:
    // 16.0 against 16.6).  The several-chunk workgroups with pair hand-overs keep the index as it comes: with the scalar
    // form the 256 x 32768 launch measured 2.4 % SLOWER in alternating runs on one box (0.612-0.613 against 0.627), the
    // other batched points within their run-to-run spread; the cause was not found.
    const uint32_t wave_raw = threadIdx.x >> 6;
    const uint32_t wave_all = (NQ > 1 && PS == 2) ? wave_raw : (uint32_t)__builtin_amdgcn_readfirstlane((int)wave_raw);   // wave of the workgroup (the set-up is dealt over all of them)
    const uint32_t sub = NQ == 1 ? 0u : wave_all >> 1;            // which of the workgroup's chunks this wave works on
    auto& sh = shs[sub];
    auto& s_rqop = shs[0].rqop;
    auto& s_maxabs = shs[0].maxabs;
    auto& s_sum = shs[0].sum;
    constexpr int kHeadDim = HD, kCodeBytes = HD / 4, NH = HD / 256;   // NH: 64-byte halves of a code
    constexpr bool has_delta = NPL == 3;
    constexpr int nplanes = NPL;
    // The two-plane forms are only entered with a level table whose mean is zero to rounding (any symmetric table): the
    // constant term of the centred planes then vanishes and the exact sum of the weights is not needed.
    constexpr bool need_wsum = NPL == 3;
    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = NQ == 1 ? wave_all : wave_all & 1u, nwaves = blockDim.x >> 6;
    const uint32_t pcol = lane & 15, g = lane >> 4;               // MFMA column / row group of this lane
    const uint32_t qi = blockIdx.y / p.num_kv_heads, kvh = blockIdx.y - qi * p.num_kv_heads;
    const uint32_t group = p.num_q_heads / p.num_kv_heads;
    const float* rq_base = a.rq + ((size_t)qi * p.num_q_heads + (size_t)kvh * group) * kHeadDim;

    const float cmax_k = fmaxf(fmaxf(fabsf(beta), fabsf(0.5f * gam)), has_delta ? fabsf(delta) : 0.0f);
    const float cmax_v = cmax_k;   // the V side also takes plane 1 at its bit position 2f + 1, i.e. with gam / 2

    // ---- the workgroup's chunk of positions
    uint32_t lo, hi, lane_base;
    query_range(p, a.positions, qi, lo, hi, lane_base);
    const uint32_t n = hi - lo, nsplit = p.num_splits * NQ;       // p.num_splits counts partial records, i.e. workgroups per query
    const uint32_t split = blockIdx.x * NQ + sub;
    const uint32_t chunk = (((n + nsplit - 1) / nsplit) + (kGroup - 1)) & ~(uint32_t)(kGroup - 1);
    const uint32_t c_lo = lo + (uint32_t)std::min<uint64_t>(n, (uint64_t)split * chunk);
    const uint32_t c_hi = lo + (uint32_t)std::min<uint64_t>(n, (uint64_t)(split + 1) * chunk);
    const bool any = c_hi > c_lo;
    const uint32_t g_first = c_lo >> 6, g_last = any ? (c_hi - 1) >> 6 : 0u;
    // Several chunks per workgroup: hand-overs (groups, or aligned pairs of groups) of this chunk, and of the workgroup's longest.
    [[maybe_unused]] uint32_t my_handovers = 0, max_handovers = 0;
    if constexpr (NQ > 1) {
        for (uint32_t s = blockIdx.x * NQ; s < (blockIdx.x + 1) * NQ; s++) {
            const uint32_t s_lo = lo + (uint32_t)std::min<uint64_t>(n, (uint64_t)s * chunk);
            const uint32_t s_hi = lo + (uint32_t)std::min<uint64_t>(n, (uint64_t)(s + 1) * chunk);
            constexpr int kShift = PS == 2 ? 7 : 6;
            const uint32_t cnt = s_hi > s_lo ? ((s_hi - 1) >> kShift) - (s_lo >> kShift) + 1 : 0u;
            if (s == split) my_handovers = cnt;
            max_handovers = std::max(max_handovers, cnt);
        }
    }

    const uint32_t stride = ONE_KV ? (uint32_t)kCodeBytes : p.num_kv_heads * kCodeBytes;   // bytes between positions
    const uint32_t nstride = ONE_KV ? 2u : p.num_kv_heads * 2;
    auto geom = [&](uint32_t G) {
        GroupGeom gg;
        const uint32_t gstart = G << 6;
        gg.vlo = c_lo > gstart ? std::min<uint32_t>(c_lo - gstart, (uint32_t)kGroup) : 0u;   // a group outside the chunk comes out empty
        gg.vhi = c_hi > gstart ? std::min<uint32_t>(c_hi - gstart, (uint32_t)kGroup) : 0u;
        if (gg.vhi < gg.vlo) gg.vhi = gg.vlo;
        gg.pb = p.ring_capacity ? gstart % p.ring_capacity : gstart;
        gg.full = gg.vlo == 0 && gg.vhi == (uint32_t)kGroup;
        return gg;
    };
    // Partial groups (chunk ends) load only their valid positions; the others read as zero codes and their
    // weights are masked to zero.
    auto is_valid = [](const GroupGeom& gg, uint32_t idx) { return idx - gg.vlo < gg.vhi - gg.vlo; };
    const float inv_cmax_v = cmax_v > 0.0f ? 1.0f / cmax_v : 0.0f;
    const float v_unit = cmax_v * (1.0f / kQmax);   // value of one integer step of a weight limb pair at scale 1
    // Roles rotate with the workgroup index, so that the kinds of wave mix on every SIMD.
    // head_dim 256: a K wave and a V wave.  head_dim 512: a K wave per 64-byte half of the K codes -- the second one (role 3)
    // runs a group ahead and hands its integer logit sums to the first, which adds its own and does the softmax -- and a V wave
    // per half of the V codes.
    // (Several chunks per workgroup: waves w and w + 4 share a SIMD, so chunks 0, 1 and chunks 2, 3 take opposite orders.)
    // (Two chunks per workgroup: two workgroups share a CU, and their order of roles follows the workgroup index.)
    const uint32_t role = NQ == 4 ? ((wave ^ (sub >> 1)) & 1u) : NQ == 2 ? ((wave ^ blockIdx.x ^ blockIdx.y) & 1u) : NH == 1 ? ((wave ^ blockIdx.x) & 1u) : (wave + blockIdx.x) & 3u;   // 0: K wave; 1, 2: V wave of code half role - 1; 3: second K wave
    const bool k_role = role == 0 || role == 3;
    const bool kb_role = NH == 2 && role == 3;
    const uint32_t khalf = kb_role ? 1u : 0u;
    // Several chunks per workgroup: the K wave and the V wave of a chunk meet at a hand-over through two counters in the
    // chunk's LDS area instead of a workgroup barrier, so that the chunks of a workgroup do not wait for one another.  A
    // wave's LDS operations execute in issue order, so "data, then the counter" needs only a wait for the wave's own LDS
    // operations and a compiler barrier (a fence would also wait for the loads in flight).  The poll is bounded: a wave that
    // runs out of patience goes on (the kernel must end), and says so in the context's fault word.
    uint32_t pair_step = 0;
    auto pair_barrier = [&]() {
        pair_step++;
        const uint32_t me = k_role ? 0u : 1u;
        __builtin_amdgcn_s_waitcnt(0xC07F); asm volatile("" ::: "memory");
        if (lane == 0) __hip_atomic_store(&sh.psync[me], pair_step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        bool seen = __hip_atomic_load(&sh.psync[me ^ 1u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= pair_step;
        if (!seen) {   // the budget lives in LDS and is read only by a wave that has to wait: no register holds it in between
            const uint32_t limit = sh.pair_spin_limit;
            uint32_t spins = 0;
            while (!(seen = __hip_atomic_load(&sh.psync[me ^ 1u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) >= pair_step) && spins++ < limit)
                __builtin_amdgcn_s_sleep(1);
        }
        if (!seen && lane == 0 && a.fault) __hip_atomic_store(a.fault, (uint32_t)LH_FAULT_ATTN_PAIR_WAIT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
        __builtin_amdgcn_s_waitcnt(0xC07F); asm volatile("" ::: "memory");
    };
    const uint32_t vhalf = k_role ? khalf : role - 1u;

    // ---- touch the first group's codes (one 64-byte record per lane) so that they are on their way into the cache
    //      while the set-up below runs; the value is only consumed (and waited for) after the set-up
    uint32_t touched = 0;
    if (any) {
        const GroupGeom g0 = geom(g_first);
        const uint8_t* rec0 = (k_role ? a.k_codes : a.v_codes) + (((size_t)lane_base + g0.pb + lane) * p.num_kv_heads + kvh) * kCodeBytes + 64 * vhalf;
        if (is_valid(g0, lane)) touched = __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(rec0));
    }

    // ---- this lane's share of the rotated queries for the K-side operands, requested together with the values for
    //      the statistics (one round trip to memory instead of two).  The lanes pcol, pcol ^ 1 serve the two limbs of
    //      one head; each quantises half of the code bytes 16g .. 16g + 15 (words m = 2 * limb, 2 * limb + 1) and
    //      they swap the limb the other one needs.
    const uint32_t h_op = (pcol >> 2) + 4 * ((pcol >> 1) & 1), limb_op = pcol & 1;
    float4 xq[2][4];
    auto load_xq = [&](uint32_t half) {   // code bytes 64 * half + 16g + 4 * (2 * limb + mm) + e
#pragma unroll
        for (int mm = 0; mm < 2; mm++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                xq[mm][e] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (h_op < group)
                    xq[mm][e] = *reinterpret_cast<const float4*>(rq_base + (size_t)h_op * kHeadDim + 256 * half + 4 * (16 * g + 4 * (2 * limb_op + mm) + e));
            }
    };
    // Operand units (code half, plane) are dealt to the waves round robin; the first unit's queries are requested here.
    uint32_t xq_half = wave_all / (uint32_t)nplanes;
    if (wave_all < (uint32_t)(nplanes * NH)) load_xq(xq_half);

    // ---- per head: max |rq| (quantisation scale) and sum(rq) (constant term of the level table)
    for (uint32_t h = tid >> 5; h < (uint32_t)kMaxGroupHeads; h += blockDim.x >> 5) {
        const uint32_t sub = tid & 31;
        constexpr int NV = HD / 32;   // values per thread: 32 threads per head
        float v[NV];
#pragma unroll
        for (int i = 0; i < NV; i++) v[i] = 0.0f;
        if (h < group) {
#pragma unroll
            for (int i = 0; i < NV / 4; i++) {
                const float4 x = *reinterpret_cast<const float4*>(rq_base + (size_t)h * kHeadDim + sub * NV + 4 * i);
                v[4 * i] = x.x; v[4 * i + 1] = x.y; v[4 * i + 2] = x.z; v[4 * i + 3] = x.w;
            }
        }
        float m = 0.0f, s = 0.0f;
#pragma unroll
        for (int i = 0; i < NV; i++) { m = fmaxf(m, fabsf(v[i])); s += v[i]; }
        m = lh_group_max(m, 32);
        s = lh_group_sum(s, 32);
        if (sub == 0) { s_maxabs[h] = m; s_sum[h] = s; }
    }
    if constexpr (kPairSync && NQ > 1) {
        if (tid < 2u * NQ) shs[tid >> 1].psync[tid & 1u] = 0u;
        else if (tid < 3u * NQ) shs[tid - 2u * NQ].pair_spin_limit = p.pair_spin_limit;
    }
    __syncthreads();

    // ---- K-side A operands.  Row r of the MFMA: head (r / 4) + 4 * ((r / 2) % 2), limb r % 2, so that the lanes of
    //      row group g end up with heads g and g + 4 on both the K and the V side.  k slot (word m, byte e) of
    //      row group g is code byte j = 64 * half + 16g + 4m + e, i.e. dim 4j + f for the operand of field f.
    {
        const float ma = s_maxabs[h_op];
        const float inv = (ma > 0.0f && cmax_k > 0.0f) ? kQmax / (ma * cmax_k) : 0.0f;
        for (uint32_t unit = wave_all; unit < (uint32_t)(nplanes * NH); unit += nwaves) {
            const uint32_t half = unit / (uint32_t)nplanes, pl = unit - half * (uint32_t)nplanes;
            if (half != xq_half) { load_xq(half); xq_half = half; }
            const float mul = (pl == 0 ? beta : pl == 1 ? 0.5f * gam : delta) * inv;
            uint32_t wlo[4][2], whi[4][2];   // [field][word mm]: low / high limbs of this lane's half, byte e = code byte 4m + e
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int mm = 0; mm < 2; mm++) wlo[f][mm] = whi[f][mm] = 0;
#pragma unroll
            for (int mm = 0; mm < 2; mm++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float xv[4] = {xq[mm][e].x, xq[mm][e].y, xq[mm][e].z, xq[mm][e].w};
#pragma unroll
                    for (int f = 0; f < 4; f++) {
                        float r = __builtin_rintf(xv[f] * mul);
                        r = fminf(fmaxf(r, -kQmax), kQmax);
                        const int n = (int)r;
                        const int lo = (int)(int8_t)(n & 0xFF);
                        wlo[f][mm] |= (uint32_t)(lo & 0xFF) << (8 * e);
                        whi[f][mm] |= (uint32_t)(((n - lo) >> 8) & 0xFF) << (8 * e);
                    }
                }
            uint32_t words[4][4];
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int mm = 0; mm < 2; mm++) {
                    const uint32_t mine = limb_op ? whi[f][mm] : wlo[f][mm];
                    const uint32_t give = limb_op ? wlo[f][mm] : whi[f][mm];
                    const uint32_t got = (uint32_t)__builtin_amdgcn_mov_dpp((int)give, 0xB1, 0xF, 0xF, true);   // quad_perm [1,0,3,2]: lane ^ 1
                    words[f][mm] = limb_op ? got : mine;        // words 0, 1 were quantised by the limb-0 lane
                    words[f][2 + mm] = limb_op ? mine : got;    // words 2, 3 by the limb-1 lane
                }
#pragma unroll
            for (int f = 0; f < 4; f++)
                *reinterpret_cast<u32x4_t*>(&s_rqop[(half * nplanes + pl) * 4 + f][lane][0]) = (u32x4_t){words[f][0], words[f][1], words[f][2], words[f][3]};
        }
    }
    __syncthreads();
    asm volatile("" :: "v"(touched));

    if (k_role) {
        // The K waves of the long-chunk forms that step through workgroup barriers run at a raised priority: they produce
        // what the V waves of the next step wait for (256 x 32768 positions: +2-2.5 % in alternating runs; head_dim 512,
        // 128 x 32768: +2-4 %), and so do those of the eight-wave workgroups with one-group hand-overs (one query over a
        // 512-position window: 11.15 -> 10.67 us).  The two-wave workgroups of head_dim 256 lose with it (2016 x 4096: -8 %;
        // the batched 512-position window: -5 %; a raised priority for their V waves instead: -3 % and -4 %) and keep the
        // default.
        if constexpr (NQ > 1 || (PS == 2 && NH == 2)) __builtin_amdgcn_s_setprio(1);
        // =================================================================== K wave
        float cs[2], ca[2];   // logit (log2 domain) = norm_k*log2e * (cs * int + ca) for the lane's two heads g, g + 4
#pragma unroll
        for (int hs = 0; hs < 2; hs++) {
            const uint32_t h = g + 4 * hs;
            cs[hs] = s_maxabs[h] * cmax_k * (0.25f / kQmax);
            ca[hs] = alpha * s_sum[h];
        }
        gptr_t krec0 = (gptr_t)a.k_codes + ((size_t)lane_base * p.num_kv_heads + kvh) * kCodeBytes + 64 * khalf;   // this wave's half of the code
        gptr_t kn0 = (gptr_t)a.k_norms + ((size_t)lane_base * p.num_kv_heads + kvh) * 2;
        gptr_t vn0 = (gptr_t)a.v_norms + ((size_t)lane_base * p.num_kv_heads + kvh) * 2;
        // The reference starts at a finite "nothing yet": an empty group ahead of the first position (a pair whose first group
        // lies before the chunk) then gives exp2(-inf) = 0 instead of exp2(-inf + inf).
        constexpr float kNoRef = -1.0e30f;
        float R[2] = {kNoRef, kNoRef}, l_run[2] = {0.f, 0.f}, w_run[2] = {0.f, 0.f};

        if (any) {
            GroupGeom gg = geom(PS == 2 ? (g_first & ~1u) : g_first);   // pairs are walked whole: a group outside the chunk is an empty one
            // K codes and norms of the current group.  Those of the next group are requested into the same registers as soon
            // as a tile's codes have been taken apart (a step of prefetch distance, no second register set, no copies).
            // `KIND` says what follows the group: 0 nothing, 1 a group that is certainly complete (every group between the
            // first and the last of a chunk is), 2 a group that may be partial.
            u32x4_t kw[4];
            float nk, nv;
            const uint32_t klane = pcol * stride + 16 * g, nlane = lane * nstride;
            auto load_tile = [&](bool full, const GroupGeom& G_, int q) {
                gptr_t kb = krec0 + (size_t)G_.pb * stride;
                if (full) kw[q] = ld16(kb + (size_t)(16 * q) * stride + klane);
                else {
                    kw[q] = (u32x4_t){0u, 0u, 0u, 0u};
                    if (is_valid(G_, 16 * q + pcol)) kw[q] = ld16(kb + (size_t)(16 * q) * stride + klane);
                }
            };
            auto load_norms = [&](bool full, const GroupGeom& G_) {
                gptr_t knb = kn0 + (size_t)G_.pb * nstride, vnb = vn0 + (size_t)G_.pb * nstride;
                if (full) { nk = ld_norm(knb + nlane); nv = ld_norm(vnb + nlane); }
                else {
                    nk = nv = 0.0f;
                    if (is_valid(G_, lane)) { nk = ld_norm(knb + nlane); nv = ld_norm(vnb + nlane); }
                }
            };
#pragma unroll
            for (int q = 0; q < 4; q++) load_tile(gg.full, gg, q);
            if (!kb_role) load_norms(gg.full, gg);

            // Two groups of 64 positions (an aligned pair) share one fixed-point scale per head and one hand-over to the V wave.
            float ww[PS][4][2];             // [group of the pair][tile][head set]: the pair's weights
            float wm[2] = {0.0f, 0.0f};     // largest |weight| of the pair so far, per head set
            float fsc_acc[2] = {1.0f, 1.0f};   // by how much the reference has moved within the pair
            bool moved_any = false;

            // The integer logit sums of a group's 4 tiles x (this lane's column position, heads g and g + 4) over this wave's half
            // of the code, handed tile by tile to `post`; the next group's codes are requested into a tile's registers as soon
            // as it has been taken apart.
            auto k_tiles = [&](auto kind_tag, const GroupGeom& gnext, auto&& post) {
                constexpr int KIND = decltype(kind_tag)::value;
                const v4i* rqo = reinterpret_cast<const v4i*>(&s_rqop[khalf * nplanes * 4][lane][0]);   // operand (plane pl, field f) at rqo[64 * (4 * pl + f)]
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    v4i acc1 = (v4i){0, 0, 0, 0}, acc4 = (v4i){0, 0, 0, 0};   // by mask scale: fields 0, 2 arrive x1, fields 1, 3 x4
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
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 0], b00, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 1], b01, acc4, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 4], b10, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 5], b11, acc4, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 2], b02, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 3], b03, acc4, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 6], b12, acc1, 0, 0, 0);
                    acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 7], b13, acc4, 0, 0, 0);
                    if constexpr (has_delta) {   // third plane bit0 & bit1, one bit per field at the even bit positions
                        v4i d0, d1, d2, d3;
#pragma unroll
                        for (int m = 0; m < 4; m++) {
                            const uint32_t t = w[m] & (w[m] >> 1), u = t >> 4;
                            d0[m] = (int)(t & 0x01010101u); d1[m] = (int)(t & 0x04040404u);
                            d2[m] = (int)(u & 0x01010101u); d3[m] = (int)(u & 0x04040404u);
                        }
                        acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 8], d0, acc1, 0, 0, 0);
                        acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 9], d1, acc4, 0, 0, 0);
                        acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 10], d2, acc1, 0, 0, 0);
                        acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(rqo[64 * 11], d3, acc4, 0, 0, 0);
                    }
                    if constexpr (KIND != 0) load_tile(KIND == 1, gnext, q);   // the tile's code registers are free
                    int t[2];
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        // three shift-adds: limbs first, then the two field scales
                        uint32_t t1 = ((uint32_t)acc1[2 * hs + 1] << 8) + (uint32_t)acc1[2 * hs];
                        uint32_t t4 = ((uint32_t)acc4[2 * hs + 1] << 8) + (uint32_t)acc4[2 * hs];
                        asm("" : "+v"(t1), "+v"(t4));   // keeps the three shift-adds (left alone the compiler regroups them into four instructions)
                        t[hs] = (int)((t1 << 2) + t4);
                    }
                    post(q, t[0], t[1]);
                }
            };
            uint32_t tbuf = 0;   // head_dim 512: which buffer holds the second K wave's sums of the group at hand

            // One group: logits, reference check, weights into wout.  `second`: the pair's first group has been done (its
            // weights in ww[0] follow the reference if that moves now).  FULL: the group is complete and not the chunk's
            // first (no masks, and the reference is finite: logits are then formed relative to it in the same fma).
            auto group_core = [&](auto kind_tag, auto full_tag, uint32_t G, float (&wout)[4][2], bool second) {
                constexpr int KIND = decltype(kind_tag)::value;
                constexpr bool FULL = decltype(full_tag)::value;
                const GroupGeom gnext = geom(KIND ? G + 1 : G);
                if constexpr (NH == 2) tbuf = (PS == 2 ? (G >> 1) - (g_first >> 1) : G - g_first) & 1u;

                // ---- norms of the group -> LDS
                {
                    const bool valid = FULL || (lane >= gg.vlo && lane < gg.vhi);
                    __builtin_amdgcn_wave_barrier();
                    sh.norm[lane] = make_float4(nk * kLog2e, valid ? 0.0f : -INFINITY, valid ? nv : 0.0f, 0.0f);
                    __builtin_amdgcn_wave_barrier();
                    if constexpr (KIND != 0) load_norms(KIND == 1, gnext);
                }

                // ---- logits of 4 tiles x (this lane's column position, heads g and g + 4)
                float lg[4][2], vn[4];
                v4i tb0 = (v4i){0, 0, 0, 0}, tb1 = (v4i){0, 0, 0, 0};   // head_dim 512: the other code half's sums, from the second K wave
                if constexpr (NH == 2) { const uint32_t sub = (PS == 2 && second) ? 1u : 0u; tb0 = sh.tb[tbuf][sub][0][lane]; tb1 = sh.tb[tbuf][sub][1][lane]; }
                k_tiles(kind_tag, gnext, [&](int q, int t0, int t1) {
                    const float4 nrm = sh.norm[16 * q + pcol];
                    vn[q] = nrm.z;
                    const int tt[2] = {t0 + tb0[q], t1 + tb1[q]};
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        const float inner = (float)tt[hs] * cs[hs] + ca[hs];
                        lg[q][hs] = FULL ? __builtin_fmaf(nrm.x, inner, -R[hs]) : nrm.x * inner + nrm.y;
                    }
                });

                // ---- softmax weights relative to the reference R, which follows the running maximum lazily: it moves
                //      when a logit of the group exceeds it by more than kHeadroom (always in the first group)
                float mq[2];
#pragma unroll
                for (int hs = 0; hs < 2; hs++) mq[hs] = fmaxf(fmaxf(lg[0][hs], lg[1][hs]), fmaxf(lg[2][hs], lg[3][hs]));
                const bool move = __builtin_amdgcn_ballot_w64((FULL ? fmaxf(mq[0], mq[1]) : fmaxf(mq[0] - R[0], mq[1] - R[1])) > kHeadroom) != 0;   // uniform
                if (move) {
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        float fsc;
                        if constexpr (FULL) {   // lg and mq are relative to R
                            const float d = fmaxf(lh_group_max(mq[hs], 16), 0.0f);
                            fsc = __builtin_amdgcn_exp2f(-d);
                            R[hs] += d;
#pragma unroll
                            for (int q = 0; q < 4; q++) lg[q][hs] -= d;
                        } else {
                            const float rn = fmaxf(R[hs], lh_group_max(mq[hs], 16));
                            fsc = rn > R[hs] ? __builtin_amdgcn_exp2f(R[hs] - rn) : 1.0f;   // 0 for the first group
                            R[hs] = rn;
                        }
                        l_run[hs] *= fsc;
                        w_run[hs] *= fsc;
                        fsc_acc[hs] *= fsc;
                        wm[hs] *= fsc;
                        if (PS == 2 && second) {
#pragma unroll
                            for (int q = 0; q < 4; q++) ww[0][q][hs] *= fsc;
                        }
                    }
                    moved_any = true;
                }
#pragma unroll
                for (int hs = 0; hs < 2; hs++) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const float ew = __builtin_amdgcn_exp2f(FULL ? lg[q][hs] : lg[q][hs] - R[hs]);
                        wout[q][hs] = ew * vn[q];
                        l_run[hs] += ew;
                        if constexpr (need_wsum) w_run[hs] += wout[q][hs];
                        wm[hs] = fmaxf(wm[hs], fabsf(wout[q][hs]));
                    }
                }
                gg = gnext;
            };
            // The pair's scales and the hand-over.
            auto finish_pair = [&](uint32_t P) {
                const uint32_t buf = (P - (PS == 2 ? g_first >> 1 : g_first)) & 1u;
#pragma unroll
                for (int hs = 0; hs < 2; hs++) {
                    // The head's scale for this pair: the power of two that takes its largest weight into [0.5, 1).
                    // Nothing representable (zero, subnormal or non-finite maximum): scale and step 0, the pair adds
                    // nothing to the integer sums (a non-finite weight still reaches the output through w_run).
                    // (wm is non-negative or NaN: its bit pattern orders like an unsigned integer, NaN on top)
                    const uint32_t e = lh_group_max_u(__float_as_uint(wm[hs]), 16) & 0x7F800000u;
                    const bool ok = e != 0u && e < (253u << 23);
                    const float sc = ok ? __uint_as_float((253u << 23) - e) : 0.0f;
                    const float un = ok ? __uint_as_float(e + (1u << 23)) * v_unit : 0.0f;
                    if (pcol == 0) {
                        sh.wsc[buf][g + 4 * hs] = make_float2(sc, un);
                        if (moved_any) sh.fsc[buf][g + 4 * hs] = fsc_acc[hs];
                    }
                    wm[hs] = 0.0f;
                    fsc_acc[hs] = 1.0f;
                }
                if (lane == 0) sh.moved[buf] = moved_any ? 1u : 0u;
                moved_any = false;
#pragma unroll
                for (int sub = 0; sub < PS; sub++)
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) sh.ww[buf][sub][hs][lane] = make_float4(ww[sub][0][hs], ww[sub][1][hs], ww[sub][2][hs], ww[sub][3][hs]);
                if constexpr (kPairSync && NQ > 1) pair_barrier();
                else __syncthreads();   // hand-over of buffer `buf`; also: the V wave is done with the buffer written next
            };
            if (kb_role) {
                // head_dim 512, second K wave: its code half's sums of every group, one hand-over ahead of the first K wave
                auto kb_step = [&](auto kind_tag, uint32_t G) {
                    constexpr int KIND = decltype(kind_tag)::value;
                    const GroupGeom gnext = geom(KIND ? G + 1 : G);
                    int t0s[4], t1s[4];
                    k_tiles(kind_tag, gnext, [&](int q, int t0, int t1) { t0s[q] = t0; t1s[q] = t1; });
                    const uint32_t b = (PS == 2 ? (G >> 1) - (g_first >> 1) : G - g_first) & 1u, sub = PS == 2 ? (G & 1u) : 0u;
                    sh.tb[b][sub][0][lane] = (v4i){t0s[0], t0s[1], t0s[2], t0s[3]};
                    sh.tb[b][sub][1][lane] = (v4i){t1s[0], t1s[1], t1s[2], t1s[3]};
                    gg = gnext;
                    if (PS == 1 || (G & 1u)) __syncthreads();   // the hand-over is complete
                };
                if constexpr (PS == 2) {
                    for (uint32_t G = g_first & ~1u; G <= (g_last | 1u); G++) {
                        if (G + 1 > g_first && G + 1 < g_last) kb_step(std::integral_constant<int, 1>{}, G);   // a complete group follows
                        else kb_step(std::integral_constant<int, 2>{}, G);
                    }
                } else {
                    uint32_t G = g_first;
                    for (; G + 1 < g_last; G++) kb_step(std::integral_constant<int, 1>{}, G);
                    if (G < g_last) { kb_step(std::integral_constant<int, 2>{}, G); G++; }
                    kb_step(std::integral_constant<int, 0>{}, G);
                }
                __syncthreads();   // the first K wave's last hand-over
                __syncthreads();   // the V waves' last hand-over
            } else if constexpr (PS == 2) {
                if constexpr (NH == 2) __syncthreads();   // the second K wave's first hand-over
                // A pair at a chunk end: either group may be partial or empty, and so may the group after each.
                auto edge_pair = [&](uint32_t P) {
                    group_core(std::integral_constant<int, 2>{}, std::false_type{}, 2 * P, ww[0], false);
                    group_core(std::integral_constant<int, 2>{}, std::false_type{}, 2 * P + 1, ww[PS - 1], true);
                    finish_pair(P);
                };
                uint32_t P = g_first >> 1;
                edge_pair(P);                                            // holds the chunk's first group
                P++;
                for (; 2 * P + 2 < g_last; P++) {                        // both groups and the one after them complete
                    group_core(std::integral_constant<int, 1>{}, std::true_type{}, 2 * P, ww[0], false);
                    group_core(std::integral_constant<int, 1>{}, std::true_type{}, 2 * P + 1, ww[PS - 1], true);
                    finish_pair(P);
                }
                for (; P <= (g_last >> 1); P++) edge_pair(P);
                if constexpr (NH == 2) __syncthreads();   // the V waves' last hand-over
            } else {
                if constexpr (NH == 2) __syncthreads();   // the second K wave's first hand-over
                uint32_t G = g_first;
                if (G + 1 < g_last) { group_core(std::integral_constant<int, 1>{}, std::false_type{}, G, ww[0], false); finish_pair(G); G++; }
                for (; G + 1 < g_last; G++) { group_core(std::integral_constant<int, 1>{}, std::true_type{}, G, ww[0], false); finish_pair(G); }
                if (G < g_last) { group_core(std::integral_constant<int, 2>{}, std::false_type{}, G, ww[0], false); finish_pair(G); G++; }
                group_core(std::integral_constant<int, 0>{}, std::false_type{}, G, ww[0], false);
                finish_pair(G);
                if constexpr (NH == 2) __syncthreads();   // the V waves' last hand-over
            }
        }
        if constexpr (NQ > 1 && !kPairSync) {   // the hand-overs that only longer chunks of this workgroup have
            for (uint32_t i = my_handovers; i < max_handovers; i++) __syncthreads();
        }
#pragma unroll
        for (int hs = 0; hs < 2; hs++) {
            const float l_tot = lh_group_sum(l_run[hs], 16);
            const float w_tot = lh_group_sum(w_run[hs], 16);
            if (pcol == 0 && !kb_role) { sh.fin_l[g + 4 * hs] = l_tot; sh.fin_w[g + 4 * hs] = w_tot; sh.fin_r[g + 4 * hs] = R[hs] <= 0.5f * kNoRef ? -INFINITY : R[hs]; }
        }
        __syncthreads();
    } else {
        // =================================================================== V wave
        gptr_t vrec0 = (gptr_t)a.v_codes + ((size_t)lane_base * p.num_kv_heads + kvh) * kCodeBytes + 64 * vhalf;
        float outv[4][4][2];   // [chunk e][field f][head set]: dim 64e + 4*pcol + f of head g + 4 * set, relative to exp2(R)
#pragma unroll
        for (int e = 0; e < 4; e++)
#pragma unroll
            for (int f = 0; f < 4; f++)
#pragma unroll
                for (int hs = 0; hs < 2; hs++) outv[e][f][hs] = 0.0f;
        // The planes are summed as 0/1 bits, but what is meant is the centred bit b - 1/2 (plane 2: b0*b1 - 1/4): per head
        // and group one more MFMA per plane against constant bytes gives the sum of the quantised weights themselves, and
        // sctr collects (1/2, 1, 1/4) of them.  Taking that off the outputs (and only the rest of the table's constant
        // term times the exact sum of weights on) makes the rounding errors of the weights enter every output dim with
        // a random sign: a common offset of all dims would be gathered into single elements by the rotation that follows.
        float sctr[2] = {0.0f, 0.0f};
        // Plane coefficients relative to the largest one, times kQmax / 32767: a weight scaled into [-1, 1] times this,
        // converted to a signed normalised 16-bit number, is at most kQmax in magnitude and splits into two int8 limbs.
        float cfn[3];
#pragma unroll
        for (int pl = 0; pl < 3; pl++) cfn[pl] = (pl == 0 ? beta : pl == 1 ? 0.5f * gam : delta) * inv_cmax_v * (kQmax / 32767.0f);

        if (any) {
            GroupGeom gg = geom(PS == 2 ? (g_first & ~1u) : g_first);
            // A group's V codes: lane L fetches 16-byte chunk L % 4 of positions 16q + L / 4 (a load instruction covers 16 whole
            // positions, 1 KB contiguous for one KV head) and parks it in the wave's LDS area; the MFMA's B operand wants "one
            // code byte over 16 positions" per lane, which ds_read_b64_tr_b8 delivers: within 16 lanes, lane i names an 8-byte
            // row and lane l receives byte l % 8 of rows 2j + l / 8, j = 0 .. 7.  Rows 2j / 2j + 1 are the two halves of a
            // 16-byte chunk of one position, so the 16 lanes get the 16 code bytes of a chunk over 8 positions.  The chunk index
            // is XORed with q and the positions of a read are spread over p % 4, which keeps both directions free of bank
            // conflicts without padding.
            u32x4_t vx[4];
            const uint32_t vpos = lane >> 2, vchunk = lane & 3;
            const uint32_t vlane = vpos * stride + 16 * vchunk;
            auto load_v = [&](bool full, const GroupGeom& G_) {
                gptr_t vb = vrec0 + (size_t)G_.pb * stride;
#pragma unroll
                for (int q = 0; q < 4; q++) {
                    if (full) vx[q] = ld16(vb + (size_t)(16 * q) * stride + vlane);
                    else {
                        vx[q] = (u32x4_t){0u, 0u, 0u, 0u};
                        if (is_valid(G_, 16 * q + vpos)) vx[q] = ld16(vb + (size_t)(16 * q) * stride + vlane);
                    }
                }
            };
            typedef __attribute__((address_space(3))) uint8_t* lds8_t;
            typedef __attribute__((address_space(3))) v2i* lds_v2i_t;
            typedef __attribute__((address_space(3))) u32x4_t* lds_x4_t;
            const lds8_t vt = (lds8_t)&sh.vt[vhalf][0];
            uint32_t wr_off[4], rd_off[4][2];   // [q] / [16-byte chunk e][read t]
#pragma unroll
            for (int q = 0; q < 4; q++) wr_off[q] = (16 * q + vpos) * 64 + ((vchunk ^ q) & 3) * 16;
            {
                const uint32_t i = lane & 15, A_ = lane >> 4, j = i >> 1, qj = j & 3;
#pragma unroll
                for (int t = 0; t < 2; t++) {
                    const uint32_t B_ = 2 * t + (j >> 2);                           // word of the operand this row feeds
                    const uint32_t src = 16 * qj + 4 * A_ + ((B_ + 2 * A_) & 3);    // position (column position 4A + ..., tile qj)
#pragma unroll
                    for (int e = 0; e < 4; e++) rd_off[e][t] = src * 64 + ((e ^ qj) & 3) * 16 + 8 * (i & 1);
                }
            }
            load_v(gg.full, gg);

            v4i acc[4][4];      // [code byte e][field f]: the pair's integer sums, rows = heads g, g + 4 x 2 limbs
            v4i csum;           // 4 x the centre: 2 sum(plane 0 weights) + 4 sum(plane 1 weights, which are halved) + sum(plane 2 weights)
            float uf[2][4];     // [head set][field]: value of one integer step of the accumulators of this pair
            float cq[2][3];     // [head set][plane]: weight -> signed normalised 16-bit number at the pair's scale
            uint32_t buf = 0;

            // The K wave's hand-over of a pair: rescale if the reference moved, read the pair's scales.
            auto begin_pair = [&](uint32_t P) {
                buf = (P - (PS == 2 ? g_first >> 1 : g_first)) & 1u;
                if constexpr (kPairSync && NQ > 1) pair_barrier();
                else __syncthreads();   // the K wave's weights of this pair
                if (__builtin_amdgcn_readfirstlane(sh.moved[buf]) != 0) {   // rare: the reference moved
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        const float fsc = sh.fsc[buf][g + 4 * hs];
#pragma unroll
                        for (int e = 0; e < 4; e++)
#pragma unroll
                            for (int f = 0; f < 4; f++) outv[e][f][hs] *= fsc;
                        sctr[hs] *= fsc;
                    }
                }
#pragma unroll
                for (int hs = 0; hs < 2; hs++) {
                    const float2 ws = sh.wsc[buf][g + 4 * hs];
                    uf[hs][0] = ws.y; uf[hs][1] = ws.y * 0.25f; uf[hs][2] = uf[hs][3] = ws.y * 0.0625f;   // field 3 is read at field 2's place
#pragma unroll
                    for (int pl = 0; pl < nplanes; pl++) cq[hs][pl] = cfn[pl] * ws.x;
                }
            };
            // One group of the pair.  KIND as in the K wave: 0 nothing follows, 1 a complete group follows, 2 a group that may be
            // partial.  ZERO: the accumulators start at zero here (the first MFMA of each takes the constant as its C operand).
            auto group_core = [&](auto kind_tag, auto zero_tag, uint32_t G, uint32_t sub) {
                constexpr int KIND = decltype(kind_tag)::value;
                constexpr bool ZERO = decltype(zero_tag)::value;
                // ---- weights -> 16-bit fixed point at the head's scale of this pair, two signed limbs; a lane holds the
                //      weights of column position pcol of the four tiles, i.e. one k word of the MFMA's A operand:
                //      lane (column 4A+B, row group g) feeds rows 4g + 2 * set + limb of k-group A, word B.
                {
                    const uint32_t A_ = pcol >> 2, B_ = ((pcol & 3) + 2 * (pcol >> 2)) & 3;   // k group and word: where the V codes of positions 16q + pcol land
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int hs = 0; hs < 2; hs++) {
                        const float4 wv = sh.ww[buf][sub][hs][lane];
#pragma unroll
                        for (int pl = 0; pl < nplanes; pl++) {
                            const float c = cq[hs][pl];
                            const uint32_t p01 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pknorm_i16(wv.x * c, wv.y * c));
                            const uint32_t p23 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pknorm_i16(wv.z * c, wv.w * c));
                            // per 16-bit half: low byte = signed low limb, high byte = what is left of it
                            const uint32_t t01 = __builtin_bit_cast(uint32_t, (us2_t)(__builtin_bit_cast(us2_t, p01) + (us2_t){0x80, 0x80})) ^ 0x00800080u;
                            const uint32_t t23 = __builtin_bit_cast(uint32_t, (us2_t)(__builtin_bit_cast(us2_t, p23) + (us2_t){0x80, 0x80})) ^ 0x00800080u;
                            uint8_t* dst = &sh.wx[vhalf][pl][(16 * A_ + 4 * g + 2 * hs) * 16 + 4 * B_];
                            *reinterpret_cast<uint32_t*>(dst) = __builtin_amdgcn_perm(t23, t01, 0x06040200u);        // low limbs of tiles 0..3
                            *reinterpret_cast<uint32_t*>(dst + 16) = __builtin_amdgcn_perm(t23, t01, 0x07050301u);   // high limbs
                        }
                    }
                    __builtin_amdgcn_wave_barrier();
                }
                uint32_t y[4][4];   // [word m][chunk e]: code byte 16e + pcol of the four positions of operand word m
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int q = 0; q < 4; q++) *(lds_x4_t)(vt + wr_off[q]) = vx[q];
                __builtin_amdgcn_wave_barrier();
                if constexpr (KIND != 0) load_v(KIND == 1, geom(G + 1));   // the V registers are free
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int t = 0; t < 2; t++) {
                        const v2i r = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_t)(vt + rd_off[e][t]));
                        y[2 * t][e] = (uint32_t)r.x;
                        y[2 * t + 1][e] = (uint32_t)r.y;
                    }
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int pl = 0; pl < nplanes; pl++) {
                    const v4i wop = *reinterpret_cast<const v4i*>(&sh.wx[vhalf][pl][lane * 16]);
                    {
                        const int cb = pl == 0 ? 0x02020202 : pl == 1 ? 0x04040404 : 0x01010101;
                        csum = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop, (v4i){cb, cb, cb, cb}, (ZERO && pl == 0) ? (v4i){0, 0, 0, 0} : csum, 0, 0, 0);
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        // Plane 0 and the product plane sit at bit 2f of a field, plane 1 at bit 2f + 1 (its coefficient is
                        // halved).  Field 3 is taken two bits down, at field 2's place: 0x80 would be a negative int8.
                        uint32_t yp[4], yd[4];
#pragma unroll
                        for (int m = 0; m < 4; m++) {
                            yp[m] = pl == 2 ? y[m][e] & (y[m][e] >> 1) : y[m][e];
                            yd[m] = yp[m] >> 2;
                        }
#pragma unroll
                        for (int f = 0; f < 4; f++) {
                            const uint32_t mask = (pl == 1 ? 0x02020202u : 0x01010101u) << (f == 3 ? 4 : 2 * f);
                            v4i b;
#pragma unroll
                            for (int m = 0; m < 4; m++) b[m] = (int)((f == 3 ? yd[m] : yp[m]) & mask);
                            acc[e][f] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wop, b, (ZERO && pl == 0) ? (v4i){0, 0, 0, 0} : acc[e][f], 0, 0, 0);
                        }
                    }
                }
            };
            // The pair's sums into the float outputs.
            auto end_pair = [&]() {
#pragma unroll
                for (int e = 0; e < 4; e++)
#pragma unroll
                    for (int f = 0; f < 4; f++)
#pragma unroll
                        for (int hs = 0; hs < 2; hs++) {
                            const int t = (int)(((uint32_t)acc[e][f][2 * hs + 1] << 8) + (uint32_t)acc[e][f][2 * hs]);
                            outv[e][f][hs] = __builtin_fmaf((float)t, uf[hs][f], outv[e][f][hs]);
                        }
#pragma unroll
                for (int hs = 0; hs < 2; hs++) {
                    const int t = (int)(((uint32_t)csum[2 * hs + 1] << 8) + (uint32_t)csum[2 * hs]);
                    sctr[hs] = __builtin_fmaf((float)t, 0.25f * uf[hs][0], sctr[hs]);
                }
            };
            if constexpr (PS == 2) {
                // A pair at a chunk end: either group may be partial or empty, and so may the group after each.
                auto edge_pair = [&](uint32_t P) {
                    begin_pair(P);
                    group_core(std::integral_constant<int, 2>{}, std::true_type{}, 2 * P, 0u);
                    group_core(std::integral_constant<int, 2>{}, std::false_type{}, 2 * P + 1, 1u);
                    end_pair();
                };
                if constexpr (NH == 2) __syncthreads();   // the second K wave's first hand-over
                uint32_t P = g_first >> 1;
                edge_pair(P);                                            // holds the chunk's first group
                P++;
                for (; 2 * P + 2 < g_last; P++) {                        // both groups and the one after them complete
                    begin_pair(P);
                    group_core(std::integral_constant<int, 1>{}, std::true_type{}, 2 * P, 0u);
                    group_core(std::integral_constant<int, 1>{}, std::false_type{}, 2 * P + 1, 1u);
                    end_pair();
                }
                for (; P <= (g_last >> 1); P++) edge_pair(P);
                if constexpr (NH == 2) __syncthreads();   // pairs with the K waves' count of barriers
            } else {
                if constexpr (NH == 2) __syncthreads();   // the second K wave's first hand-over
                uint32_t G = g_first;
                for (; G + 1 < g_last; G++) { begin_pair(G); group_core(std::integral_constant<int, 1>{}, std::true_type{}, G, 0u); end_pair(); }
                if (G < g_last) { begin_pair(G); group_core(std::integral_constant<int, 2>{}, std::true_type{}, G, 0u); end_pair(); G++; }
                begin_pair(G);
                group_core(std::integral_constant<int, 0>{}, std::true_type{}, G, 0u);
                end_pair();
                if constexpr (NH == 2) __syncthreads();   // pairs with the K waves' count of barriers
            }
        }
        if constexpr (NQ > 1 && !kPairSync) {   // the hand-overs that only longer chunks of this workgroup have
            for (uint32_t i = my_handovers; i < max_handovers; i++) __syncthreads();
        }
        __syncthreads();   // the K wave's totals

        // ---- the workgroup's result: final output (one split) or a partial record for the merge kernel
#pragma unroll
        for (int hs = 0; hs < 2; hs++) {
            const uint32_t h = g + 4 * hs;
            if (h >= group) continue;
            const float l_tot = sh.fin_l[h], w_tot = sh.fin_w[h];
            const uint32_t qh = kvh * group + h;
            const float bias = need_wsum ? (alpha + 0.5f * (beta + gam) + 0.25f * delta) * w_tot - sctr[hs] : -sctr[hs];
            if constexpr (NQ > 1) {   // parked for the merge below, in this pair's operand area (every loop of the workgroup has ended)
                float* park = reinterpret_cast<float*>(&sh.rqop[0][0][0]) + h * kHeadDim + 4 * pcol;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    *reinterpret_cast<float4*>(park + 64 * e) =
                        make_float4(outv[e][0][hs] + bias, outv[e][1][hs] + bias, outv[e][2][hs] + bias, outv[e][3][hs] + bias);
            } else if (nsplit == 1) {
                float* dst = a.out + ((size_t)qi * p.num_q_heads + qh) * kHeadDim + 256 * vhalf + 4 * pcol;
                const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
#pragma unroll
                for (int e = 0; e < 4; e++)
                    *reinterpret_cast<float4*>(dst + 64 * e) = make_float4((outv[e][0][hs] + bias) * inv, (outv[e][1][hs] + bias) * inv,
                                                                          (outv[e][2][hs] + bias) * inv, (outv[e][3][hs] + bias) * inv);
            } else {
                float* rec = a.ws + (((size_t)qi * p.num_q_heads + qh) * nsplit + split) * partial_record_floats(kHeadDim);
                if (pcol == 0 && vhalf == 0) { rec[0] = sh.fin_r[h] * kLn2; rec[1] = l_tot; }
#pragma unroll
                for (int e = 0; e < 4; e++)
                    *reinterpret_cast<float4*>(rec + 4 + 256 * vhalf + 4 * pcol + 64 * e) =
                        make_float4(outv[e][0][hs] + bias, outv[e][1][hs] + bias, outv[e][2][hs] + bias, outv[e][3][hs] + bias);
            }
        }
    }
    if constexpr (NQ > 1) {
        // ---- the chunks' results merged: a wave takes head h (two heads where the workgroup has four waves), a lane four dims.  (R, l, acc) of a chunk are relative to
        //      exp2(R); the result goes out as the final output (one workgroup per query) or as one partial record.
        static_assert(sizeof(sh.rqop) >= (size_t)kMaxGroupHeads * kHeadDim * sizeof(float), "the parked sums fit the operand area");
        __syncthreads();   // every chunk's sums are parked
        for (uint32_t h = wave_all; h < group; h += 2 * NQ) {
            float Rq[NQ], gm = -INFINITY;
#pragma unroll
            for (int q = 0; q < NQ; q++) { Rq[q] = shs[q].fin_r[h]; gm = fmaxf(gm, Rq[q]); }
            float l_all = 0.0f;
            float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
            for (int q = 0; q < NQ; q++) {
                const float f = Rq[q] == -INFINITY ? 0.0f : exp2f(Rq[q] - gm);
                const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(&shs[q].rqop[0][0][0]) + h * kHeadDim + 4 * lane);
                l_all = __builtin_fmaf(f, shs[q].fin_l[h], l_all);
                o.x = __builtin_fmaf(f, v.x, o.x); o.y = __builtin_fmaf(f, v.y, o.y);
                o.z = __builtin_fmaf(f, v.z, o.z); o.w = __builtin_fmaf(f, v.w, o.w);
            }
            const uint32_t qh = kvh * group + h;
            if (p.num_splits == 1) {
                const float inv = l_all > 0.0f ? 1.0f / l_all : 0.0f;
                *reinterpret_cast<float4*>(a.out + ((size_t)qi * p.num_q_heads + qh) * kHeadDim + 4 * lane) =
                    make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
            } else {
                float* rec = a.ws + (((size_t)qi * p.num_q_heads + qh) * p.num_splits + blockIdx.x) * partial_record_floats(kHeadDim);
                if (lane == 0) { rec[0] = gm * kLn2; rec[1] = l_all; }
                *reinterpret_cast<float4*>(rec + 4 + 4 * lane) = o;
            }
        }
    }
}

template <int OCC, int HD, int PS>
__global__ __launch_bounds__(HD / 2, OCC) void attention_tq_mfma_kernel(AttnPointers a, AttnParams p) {   // 128 / 256 threads
    __shared__ __align__(16) AttnShared<HD / 256, PS> sh;
    // L[c] = alpha + beta*bit0 + gam*bit1 + delta*bit0*bit1.  A delta that is only float noise of a symmetric table
    // (|delta| <= 1e-5 max|L|) is spread by the least-squares affine fit bit0*bit1 ~ -1/4 + bit0/2 + bit1/2, which
    // leaves +-delta/4 per code; anything larger gets its own bit plane.
    const float L0 = a.levels[0], L1 = a.levels[1], L2 = a.levels[2], L3 = a.levels[3];
    const float d_raw = (L3 - L2) - (L1 - L0);
    const float lmax = fmaxf(fmaxf(fabsf(L0), fabsf(L1)), fmaxf(fabsf(L2), fabsf(L3)));
    // The constant term left over by the centred planes is mean(L) times the sum of the weights.
    const float l_mean = 0.25f * ((L0 + L3) + (L1 + L2));
    if (fabsf(d_raw) > 1e-5f * lmax || fabsf(l_mean) > 1e-6f * lmax) attention_body<3, HD, false, PS>(a, p, &sh, L0, L1 - L0, L2 - L0, d_raw);
    else if (p.num_kv_heads == 1) attention_body<2, HD, true, PS>(a, p, &sh, L0 - 0.25f * d_raw, (L1 - L0) + 0.5f * d_raw, (L2 - L0) + 0.5f * d_raw, 0.0f);
    else attention_body<2, HD, false, PS>(a, p, &sh, L0 - 0.25f * d_raw, (L1 - L0) + 0.5f * d_raw, (L2 - L0) + 0.5f * d_raw, 0.0f);
}

// Four (or two) chunks of a query per workgroup (head_dim 256): 512 (256) threads, the hand-over areas in dynamic LDS.
constexpr int kQuad = 4;
template <int PS, int NQ = kQuad> constexpr size_t quad_lds_bytes() { return NQ * sizeof(AttnShared<1, PS>); }
template <int PS, int NQ = kQuad>
__global__ __launch_bounds__(128 * NQ, 2) void attention_tq_mfma_quad_kernel(AttnPointers a, AttnParams p) {
    extern __shared__ __align__(16) uint8_t quad_lds[];
    auto* shs = reinterpret_cast<AttnShared<1, PS>*>(quad_lds);
    const float L0 = a.levels[0], L1 = a.levels[1], L2 = a.levels[2], L3 = a.levels[3];   // as in attention_tq_mfma_kernel
    const float d_raw = (L3 - L2) - (L1 - L0);
    const float lmax = fmaxf(fmaxf(fabsf(L0), fabsf(L1)), fmaxf(fabsf(L2), fabsf(L3)));
    const float l_mean = 0.25f * ((L0 + L3) + (L1 + L2));
    if (fabsf(d_raw) > 1e-5f * lmax || fabsf(l_mean) > 1e-6f * lmax) attention_body<3, 256, false, PS, NQ>(a, p, shs, L0, L1 - L0, L2 - L0, d_raw);
    else if (p.num_kv_heads == 1) attention_body<2, 256, true, PS, NQ>(a, p, shs, L0 - 0.25f * d_raw, (L1 - L0) + 0.5f * d_raw, (L2 - L0) + 0.5f * d_raw, 0.0f);
    else attention_body<2, 256, false, PS, NQ>(a, p, shs, L0 - 0.25f * d_raw, (L1 - L0) + 0.5f * d_raw, (L2 - L0) + 0.5f * d_raw, 0.0f);
}

}  // namespace

int lh_attention_kernels_init(lh_context* ctx) {
    int r = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_mfma_quad_kernel<1, kQuad>, quad_lds_bytes<1, kQuad>(), "context_create");
    if (r == LH_OK) r = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_mfma_quad_kernel<2, kQuad>, quad_lds_bytes<2, kQuad>(), "context_create");
    if (r == LH_OK) r = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_mfma_quad_kernel<2, 2>, quad_lds_bytes<2, 2>(), "context_create");
    return r;
}

namespace lh_attn {

bool mfma_supported(const AttnParams& p, const AttnPointers& a) {
    static const bool off = [] { const char* e = getenv("LOCAL_HIP_ATTN_KERNEL"); return e && e[0] == 'v'; }();   // "valu"
    if (off) return false;
    if (p.bits != 2 || (p.head_dim != 256 && p.head_dim != 512)) return false;
    if (p.num_q_heads / p.num_kv_heads > (uint32_t)kMaxGroupHeads) return false;
    if (p.ring_capacity % kGroup != 0) return false;                      // aligned groups must not wrap inside
    if (((uintptr_t)a.k_codes | (uintptr_t)a.v_codes) & 3) return false;
    if (((uintptr_t)a.k_norms | (uintptr_t)a.v_norms) & 1) return false;
    if (((uintptr_t)a.rq | (uintptr_t)a.out) & 15) return false;
    return true;
}

// Test aid: the poll budget of a hand-over between a chunk's two waves.  With 0 a wave that arrives early gives up at once,
// which the wait on the batch reports; nothing in the library changes it.
static std::atomic<uint32_t> g_pair_spin_limit{1u << 22};

int launch_mfma(lh_context* ctx, const char* op, const AttnPointers& a, AttnParams& p, uint64_t max_span, size_t ws_floats) {
    p.pair_spin_limit = g_pair_spin_limit.load(std::memory_order_relaxed);
    // One workgroup (a K wave and one V wave per 256 dims) per chunk of positions.  Short jobs (the chunks of one workgroup per CU
    // stay within 128 positions) are latency bound: they get chunks down to one group of 64 and never share a CU.
    // Everything else gets about two waves per SIMD over the whole launch (the registers allow no third) and at least 128
    // positions per chunk.
    constexpr uint32_t wps = 2;
    const uint64_t pairs = (uint64_t)p.num_queries * p.num_kv_heads;
    const uint32_t wg_waves = p.head_dim == 512 ? 4 : 2;
    const uint64_t wg_slots = (uint64_t)ctx->cu_count * std::max(1u, 4u * wps / wg_waves);
    const size_t rec = partial_record_floats(p.head_dim);
    static const int pair_env = [] { const char* e = getenv("LOCAL_HIP_ATTN_PAIR"); return e ? atoi(e) : -1; }();
    uint64_t splits = std::min<uint64_t>((max_span + 63) / 64, std::max<uint64_t>(1, (uint64_t)ctx->cu_count / pairs));
    // Short jobs of head_dim 256 in fours: an eight-wave workgroup per CU takes four chunks of a query, down to one group each,
    // and merges them itself -- twice the waves of the two-wave form at work on a latency-bound job and a quarter of the
    // partial records.  It pays where a two-wave workgroup per CU would walk more than one group (one query over 32768
    // positions: 12.5-12.9 us against 13.9; over 131072: 16.5 against 20.0); where every workgroup has one group anyway the
    // longer set-up and the merge of the eight-wave workgroup cost more than they save (4096 positions: 12.5 against 10.6 us).
    // A few queries over at most eight groups each (one token over a sliding window of 512): one workgroup per query, one or
    // two groups per pair of waves, and the kernel's output is final -- no records, no merge launch behind it.
    const uint64_t groups = (max_span + 63) / 64;
    const bool whole = pairs <= 8 && groups >= 2 && groups <= 2 * (uint64_t)kQuad;
    if (p.head_dim == 256 && pair_env <= 0 && (whole || (max_span + splits - 1) / splits > 64)) {
        uint64_t q = std::min<uint64_t>(groups, std::max<uint64_t>(1, (uint64_t)kQuad * ctx->cu_count / pairs));
        q -= q % kQuad;
        if (whole) q = kQuad;
        while (q > (uint64_t)kQuad && (size_t)p.num_queries * p.num_q_heads * (q / kQuad) * rec > ws_floats) q -= kQuad;
        if (q >= (uint64_t)kQuad && (((max_span + q - 1) / q + 63) & ~(uint64_t)63) <= 128 &&
            (q == (uint64_t)kQuad || (size_t)p.num_queries * p.num_q_heads * (q / kQuad) * rec <= ws_floats)) {
            const int rl = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_mfma_quad_kernel<1>, quad_lds_bytes<1>(), op);
            if (rl != LH_OK) return rl;
            p.num_splits = (uint32_t)(q / kQuad);
            hipLaunchKernelGGL(attention_tq_mfma_quad_kernel<1>, dim3(p.num_splits, (uint32_t)pairs), dim3(128 * kQuad), quad_lds_bytes<1>(), ctx->stream, a, p);
            return lh_check_launch(op);
        }
    }
    splits = std::max<uint64_t>(splits, 1);
    if ((max_span + splits - 1) / splits > 128) {
        splits = std::max<uint64_t>(1, wg_slots / pairs);
        splits = std::min<uint64_t>(splits, (max_span + 127) / 128);
    }
    // The merge takes 256 splits of a query in one round of loads and every further 256 in a dependent round of their own (about
    // 2 us each), so one or two long queries keep 256 splits until a chunk passes 1024 positions (131072 positions, one query:
    // 20.5 us with 256 splits, 21.7 with 512, 25.8 with 1024).
    if (splits > 256) splits = std::max<uint64_t>(256, std::min<uint64_t>(splits, (max_span + 1023) / 1024));
    splits = std::min<uint64_t>(std::max<uint64_t>(splits, 1), kMaxSplits);
    while (splits > 1 && (size_t)p.num_queries * p.num_q_heads * splits * rec > ws_floats) splits--;
    p.num_splits = (uint32_t)splits;
    // Hand-overs of two groups pay from about a thousand positions per workgroup on (-2 % at 4096 positions per workgroup, -5 % at
    // 8192, either head_dim); below that the longer fill and drain of the pipeline costs more (a 512-position window: +24 %).
    // LOCAL_HIP_ATTN_PAIR=1 / 0 forces one form onto every chunk length (a test aid: it puts missing and partial groups at both
    // ends of short chunks through the paired loops).
    constexpr uint64_t pair_min = 1024;
    const bool pair = pair_env >= 0 ? pair_env != 0 : (max_span + splits - 1) / splits >= pair_min;
    // Long chunks of head_dim 256 in fours: one eight-wave workgroup takes four consecutive chunks of a query and merges them
    // itself, so a query of four chunks leaves the kernel as its final output (no partial records, no merge launch) and one of
    // 4 k chunks as k records.  Other chunk counts keep a workgroup per chunk: the gain is the merge launch that four chunks no
    // longer need (256 x 32768 positions: 218 against 229 us); with records left to merge the forms measure alike.
    if (p.head_dim == 256 && pair && splits % kQuad == 0) {
        const int rl = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_mfma_quad_kernel<2>, quad_lds_bytes<2>(), op);
        if (rl != LH_OK) return rl;
        p.num_splits = (uint32_t)(splits / kQuad);
        hipLaunchKernelGGL(attention_tq_mfma_quad_kernel<2>, dim3(p.num_splits, (uint32_t)pairs), dim3(128 * kQuad), quad_lds_bytes<2>(), ctx->stream, a, p);
        return lh_check_launch(op);
    }
    // Two long chunks per query (512 sequences of 16384 positions): the same with two chunks per four-wave workgroup, two
    // workgroups to a CU -- the query leaves the kernel as its final output.
    if (p.head_dim == 256 && pair && splits == 2) {
        constexpr size_t lds2 = quad_lds_bytes<2, 2>();
        const int rl = lh_raise_dynamic_lds(ctx, (const void*)attention_tq_mfma_quad_kernel<2, 2>, lds2, op);
        if (rl != LH_OK) return rl;
        p.num_splits = 1;
        hipLaunchKernelGGL((attention_tq_mfma_quad_kernel<2, 2>), dim3(1, (uint32_t)pairs), dim3(256), lds2, ctx->stream, a, p);
        return lh_check_launch(op);
    }
    const dim3 grid((uint32_t)splits, (uint32_t)pairs);
    if (p.head_dim == 512 && pair) hipLaunchKernelGGL((attention_tq_mfma_kernel<2, 512, 2>), grid, dim3(256), 0, ctx->stream, a, p);
    else if (p.head_dim == 512) hipLaunchKernelGGL((attention_tq_mfma_kernel<2, 512, 1>), grid, dim3(256), 0, ctx->stream, a, p);
    else if (pair) hipLaunchKernelGGL((attention_tq_mfma_kernel<2, 256, 2>), grid, dim3(128), 0, ctx->stream, a, p);
    else hipLaunchKernelGGL((attention_tq_mfma_kernel<2, 256, 1>), grid, dim3(128), 0, ctx->stream, a, p);
    return lh_check_launch(op);
}

}  // namespace lh_attn

extern "C" void lh_debug_set_attention_pair_spin_limit(uint32_t polls) { lh_attn::g_pair_spin_limit.store(polls, std::memory_order_relaxed); }
