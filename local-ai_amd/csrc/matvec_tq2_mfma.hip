// TQ2_0 fused dequant matvec (M = 1) with the inner products on the matrix cores.
//
// Same contract as the TQ2_0 path of matvec_quant.hip (stands in for
// shaders/matvec_quant.metal:173-312).  At 3.9 weights per byte the 2-bit unpack plus
// v_dot4 arithmetic of the vector-ALU kernel costs more issue slots than the HBM stream
// leaves free; here the vector ALU only isolates the 2-bit codes and the integer dot
// products run as v_mfma_i32_16x16x64_i8.
//
// One wave works on tiles of 16 weight rows x (up to) 8 blocks = 2048 columns:
//   1. The tile's bytes (codes AND the f16 block scales, verbatim GGUF order) are
//      fetched with fully coalesced 128-bit loads -- consecutive lanes read consecutive
//      16-byte chunks of a row -- into registers one tile ahead, then parked in a
//      wave-private LDS image.  (Loading in MFMA operand order straight from global
//      memory makes every 4-lane group touch 4 different rows, and separate 2-byte
//      scale loads cost more than the whole code stream: both were measured.)
//   2. Lane (r = lane % 16, g = lane / 16) takes quarter g of block b of row r from the
//      image: two aligned ds_read_b128 plus a constant funnel shift (blocks start on
//      2-byte boundaries).  (codes >> 2f) & 0x03030303 for field f is the MFMA A
//      operand: 16 rows x 64 k.
//   3. The B operand holds the activation limbs (16-bit block fixed point, see
//      xquant.hpp) of those 64 elements in columns 2b (low limb) and 2b + 1 (high limb)
//      and zeros elsewhere, read from LDS (lanes of other columns read a zero line), so
//      one accumulator tile D[16 rows][16 cols] collects all 8 blocks x 2 limbs.
//   4. Per tile the dense accumulator is combined (limbs, zero point), multiplied by
//      d * s per (row, block) -- the scales come from the same LDS image -- and the 16
//      columns are summed with DPP.
#include "common.hpp"
#include "xquant.hpp"
#include <algorithm>
#include <atomic>
#include <cstdlib>

namespace {

constexpr int kL = 2;                        // activation limbs (16-bit block fixed point)
constexpr int kMaxChunksPerRow = 33;         // 8 blocks * 66 bytes = 528 bytes = 33 chunks of 16 bytes
constexpr int kStageLoads = 9;               // ceil(16 rows * 33 chunks / 64 lanes)
constexpr uint32_t kImageBytes = 16 * (kMaxChunksPerRow * 16 + 16) + 32;   // padded row stride + over-read margin
// Ring slots for the partial rows of a split tile: the waves of a tile may drift kRing - 1 tiles apart.  One slot: a wave
// delivers tile n only after tile n - 1 has been summed, so the waves of a tile stay within a tile of each other and fetch
// the neighbouring segments of the same rows close together in time; with four slots the shared cache lines were evicted
// in between and fetched again (1.09 x the bytes with plain loads against 1.03 x, 5.3 against 5.5 TB/s).
constexpr uint32_t kRing = 1;
constexpr uint32_t kMaxWavesPerWG = 12;       // the largest workgroup launched here
constexpr size_t kProWords = sizeof(XPrologue) / 4;   // the prologue's words, kept in LDS behind the split area (see cold_kernargs)
constexpr size_t kSplitAreaBytes = (size_t)kRing * kMaxWavesPerWG * 16 * 4 + (size_t)kMaxWavesPerWG * 2 * kRing * 4 + ((kProWords * 4 + 15) & ~(size_t)15);   // partial rows + arrival / generation words per tile of a slot + the prologue
constexpr size_t kMaxLdsBytes = 160 * 1024;   // most dynamic LDS a launch here asks for: all a CU has
typedef int v4i __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) uint8_t* gptr_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

// Bytes of the activation area at the head of the dynamic LDS: two limb planes for each of the two fixed-point levels,
// four per-block arrays (scale and integer sum of either level), padded so that the 128-byte zero line behind it starts
// 64 bytes into a 256-byte line.  The limb planes of a level are K + 16 bytes apart and the zero line sits on banks of its
// own: the lanes of one B-operand read (low limb, high limb, zeros) then never meet on an LDS bank.
__host__ __device__ constexpr uint32_t plane_bytes(uint32_t K) { return K + 16; }
__host__ __device__ constexpr size_t lds_head_bytes(uint32_t K) {
    const size_t raw = (size_t)2 * kL * plane_bytes(K) + (size_t)(K >> 8) * 16;
    return ((raw + 255 - 64) & ~(size_t)255) + 64;
}

struct Tq2Problem {
    const uint8_t* matrix;
    const void* vector;
    void* output;
};
// The problem that travels in the kernel arguments.  With a descriptor table absent and count > 1, problem i is this
// one with its vector and output advanced by i strides (the rows of a small activation batch against one matrix).
struct Tq2Base {
    Tq2Problem p;
    uint32_t xstride, ystride;   // bytes
    uint64_t mstride = 0;        // bytes between the matrices of consecutive problems (0: one matrix for all of them)
    uint32_t split_waves = 0;    // split form: waves that share the block groups of one tile (0: all waves of the workgroup)
    // A pair of unrelated problems (gate and up) also travels here, so the common grouped launch needs no
    // descriptor upload ahead of it.
    Tq2Problem second = {nullptr, nullptr, nullptr};
    uint32_t pair = 0;
    XPrologue pro = {kXProNone, nullptr, 0.0f};   // applied to every problem's vector while it is staged
    // Split form: how often a wave polls for the previous use of its ring slot before it gives up, and where it says so.
    uint32_t spin_limit = 1u << 20;
    uint32_t* fault = nullptr;
};

// The kernel's arguments as they lie in its argument segment.  The ones that only the staging of a vector and the bounded
// wait read (the prologue, the poll limit, the fault word) are not taken from the argument registers: held in scalar
// registers for the whole kernel they cost the main loop spills.  The prologue is copied to LDS at the head of the kernel
// and read back where a vector is staged; the other two are fetched from the segment on the path that never runs, through
// a pointer the compiler cannot see through.
struct Tq2KernArgs { const Tq2Problem* problems; Tq2Base single; uint32_t count, rows, K; };
typedef const __attribute__((address_space(4))) Tq2KernArgs* kernargs_t;
__device__ __forceinline__ kernargs_t cold_kernargs() {
    kernargs_t ka = (kernargs_t)__builtin_amdgcn_kernarg_segment_ptr();
    asm volatile("" : "+s"(ka));
    return ka;
}

__device__ __forceinline__ u32x4_t ld16_align2_cached(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(2))) u32x4_a2;
    return *reinterpret_cast<const __attribute__((address_space(1))) u32x4_a2*>(p);
}
__device__ __forceinline__ u32x4_t ld16_align2(gptr_t p) {
    typedef u32x4_t __attribute__((aligned(2))) u32x4_a2;
    // weights are read once per launch: a streaming load keeps them from displacing the activations in the caches
    return __builtin_nontemporal_load(reinterpret_cast<const __attribute__((address_space(1))) u32x4_a2*>(p));
}

// 16 bytes starting `SH` bytes into the 32-byte pair (c0, c1).
template <int SH>
__device__ __forceinline__ void take16(const u32x4_t& c0, const u32x4_t& c1, uint32_t (&out)[4]) {
    const uint32_t in[8] = {c0.x, c0.y, c0.z, c0.w, c1.x, c1.y, c1.z, c1.w};
    constexpr int q = SH >> 2, rem = SH & 3;
#pragma unroll
    for (int m = 0; m < 4; m++) out[m] = rem ? __builtin_amdgcn_alignbit(in[m + q + 1], in[m + q], 8 * rem) : in[m + q];
}

// STREAM: the weight loads carry the non-temporal hint.  Right when a tile's bytes are one contiguous run (one block group
// per row: every cache line is used once, by one instruction).  With several groups per row a tile is sixteen 528-byte
// segments whose first and last cache lines are shared with the neighbouring segment.  Where one wave walks the groups of
// its tile the neighbour is read an item later: the hint evicts those lines early and they come from HBM a second time
// (measured: 1.19 x the bytes), so such launches use plain loads.  The twelve-wave split form reads the neighbouring
// segments on neighbouring waves at about the same time (kRing below): there the shared lines still cost 1.10 x, but the
// hinted loads stream enough faster to win (5.6-5.7 against 5.5 TB/s on 2048 x 8192 weights).
template <typename XT, typename YT, bool SPLITK, int MAXT = 256, bool STREAM = false>
__global__ __launch_bounds__(MAXT, MAXT == 256 ? 2 : 1) void matvec_tq2_mfma_kernel(const Tq2Problem* __restrict__ problems, Tq2Base single,
                                                                uint32_t count, uint32_t rows, uint32_t K) {
    constexpr bool splitk = SPLITK;
    extern __shared__ __align__(16) uint8_t lds[];
    const uint32_t nb = K >> 8;                                     // blocks per row
    // [xq: 2 x K/4 limb words][xq2: the same for the residual level][xs nb][xn nb][xs2 nb][xn2 nb][pad]
    uint32_t* xq = reinterpret_cast<uint32_t*>(lds);                // [2][K/4] activation limbs
    uint32_t* xq2 = reinterpret_cast<uint32_t*>(lds + (size_t)kL * plane_bytes(K));
    float* xs = reinterpret_cast<float*>(lds + (size_t)2 * kL * plane_bytes(K)); // [nb] activation scales
    int* xn = reinterpret_cast<int*>(xs + nb);                      // [nb] sum of the block's integers
    const XResidual resid{xq2, xs + 2 * nb, xn + 2 * nb};
    const uint32_t kq = plane_bytes(K) >> 2;                        // dwords between the low-limb and the high-limb plane
    const uint32_t row_bytes = nb * 66;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)), nwaves = blockDim.x >> 6;
    const uint32_t r = lane & 15, g = lane >> 4;                    // A layout: row r, quarter g
    const uint32_t c = lane & 15;                                   // B / D layout: column c, k-group / row-group g
    const uint32_t cb = c >> 1, cl = c & 1;                         // column's block (within a group of 8) and limb
    const uint32_t lane_x_off = 4u * (cl * kq + (g >> 1) * 32u + (g & 1) * 4u);
    const uint32_t zero_off = (uint32_t)lds_head_bytes(K);                      // 128 bytes of zeros behind the activation area
    if (threadIdx.x < 32) reinterpret_cast<uint32_t*>(lds + zero_off)[threadIdx.x] = 0;
    uint32_t slot_seq = 0;                                                      // tiles this wave has completed (split form)
    uint8_t* image = lds + zero_off + 128 + (size_t)wave * kImageBytes;         // this wave's tile image

    // Work order: "slots" of nwaves consecutive tiles, dealt round-robin to the workgroups, so that at any moment
    // the whole grid reads one compact, advancing window of the weight stream.
    const uint32_t tiles_per_problem = (rows + 15) >> 4;
    // Normally a slot is nwaves consecutive tiles, one per wave, each wave walking all block groups of its tile.  With
    // `splitk` (few tiles, long rows) a slot is ONE tile whose block groups are dealt to the waves (nwaves divides their
    // number) and the waves' partial row sums are added through LDS in a fixed order.
    // A large workgroup in split form holds several such tiles at once: sw waves per tile, nwaves / sw consecutive tiles
    // per slot (wave w works on tile w / sw of the slot, block groups w % sw, w % sw + sw, ...).
    const uint32_t sw = splitk ? (single.split_waves ? single.split_waves : (uint32_t)nwaves) : 1u;   // waves per tile
    const uint32_t tps = splitk ? (uint32_t)nwaves / sw : (uint32_t)nwaves;                          // tiles per slot
    const uint32_t tsub = splitk ? (uint32_t)wave / sw : (uint32_t)wave;                             // this wave's tile of the slot
    const uint32_t slots_per_problem = (tiles_per_problem + tps - 1) / tps;
    const uint64_t total_slots = (uint64_t)slots_per_problem * count;
    const uint32_t ngroups = (nb + 7) >> 3;
    const uint64_t my_slots = blockIdx.x < total_slots ? (total_slots - blockIdx.x + gridDim.x - 1) / gridDim.x : 0;
    const uint32_t grp0 = splitk ? (uint32_t)wave % sw : 0u, grp_step = sw;
    const uint32_t nitems = (uint32_t)(my_slots * (ngroups / grp_step));   // one item = one (tile, block group); the host keeps a launch's total under 2^32

    // Chunk -> (row, chunk-in-row) of the lane's staging loads.  Full groups of 8 blocks (33 chunks per row): the global
    // offsets live in registers and the image offsets are linear in the chunk index.  The trailing group of nb % 8
    // blocks: both tables live in LDS (one per workgroup), read back when such a group comes up.
    const uint32_t nbg_tail = (nb & 7) ? (nb & 7) : 8;
    // (all three tables live in LDS, one copy per workgroup, read back when a tile's loads are issued: the nine offsets
    // of a full group in registers cost the third wave per SIMD)
    // (16-bit entries: row offsets stay below 15 * 3168 + 528 bytes for the widest row this kernel takes)
    uint16_t* tail_tab = reinterpret_cast<uint16_t*>(lds + zero_off + 128 + (size_t)nwaves * kImageBytes);   // [3][kStageLoads][64]
    uint16_t* full_tab = tail_tab + 2 * kStageLoads * 64;
    uint32_t* const sync_words = reinterpret_cast<uint32_t*>(reinterpret_cast<float*>(tail_tab + 3 * kStageLoads * 64) + kRing * kMaxWavesPerWG * 16);
    if (splitk && threadIdx.x < kMaxWavesPerWG * 2 * kRing) sync_words[threadIdx.x] = 0u;   // arrival counts and generations of the partial-sum rings
    uint32_t* const pro_words = sync_words + kMaxWavesPerWG * 2 * kRing;
    if (threadIdx.x < kProWords)
        pro_words[threadIdx.x] = reinterpret_cast<const __attribute__((address_space(4))) uint32_t*>(&cold_kernargs()->single.pro)[threadIdx.x];
    // Position in the work order, advanced incrementally (all scalar, no division in the loop).
    struct Item { uint32_t grp, sip, prob; };                       // block group, slot within the problem, problem
    const uint32_t step_prob = gridDim.x / slots_per_problem, step_sip = gridDim.x % slots_per_problem;
    auto advance = [&](Item it) {
        it.grp += grp_step;
        if (it.grp >= ngroups) {
            it.grp = grp0;
            it.sip += step_sip;
            it.prob += step_prob;
            if (it.sip >= slots_per_problem) { it.sip -= slots_per_problem; it.prob++; }
        }
        return it;
    };
    auto item_tile_base = [&](const Item& it, uint32_t& grp, uint32_t& tile, Tq2Problem& pb) {
        grp = it.grp;
        tile = it.sip * tps + tsub;
        if (problems) pb = problems[it.prob];
        else if (single.pair && it.prob == 1) pb = single.second;
        else pb = Tq2Problem{single.p.matrix + (size_t)it.prob * single.mstride, (const char*)single.p.vector + (size_t)it.prob * single.xstride,
                             (char*)single.p.output + (size_t)it.prob * single.ystride};
    };
    Item cur{grp0, blockIdx.x % slots_per_problem, blockIdx.x / slots_per_problem};

    u32x4_t pre[kStageLoads];
    // `offs`: the lane's nine chunk offsets of a full group, read from full_tab by the caller ahead of the call (at the top of
    // a loop iteration, so that the LDS round trip hides behind the wait for the previous tile's loads; keeping them in
    // registers for the whole loop costs the third wave per SIMD)
    auto prefetch = [&](const Item& it, const uint32_t (&offs)[kStageLoads]) {
        uint32_t grp, tile; Tq2Problem pb;
        item_tile_base(it, grp, tile, pb);
        const bool tail = grp + 1 == ngroups && (nb & 7);
        if ((tile << 4) + 16 <= rows) {                              // every row of the tile exists: precomputed offsets
            gptr_t base = (gptr_t)pb.matrix + (size_t)(tile << 4) * row_bytes + (size_t)grp * 528;
            if (!tail) {
#pragma unroll
                for (int i = 0; i < kStageLoads; i++) pre[i] = STREAM ? ld16_align2(base + offs[i]) : ld16_align2_cached(base + offs[i]);
            } else {
#pragma unroll
                for (int i = 0; i < kStageLoads; i++) pre[i] = ld16_align2(base + tail_tab[i * 64 + lane]);
            }
        } else {                                                     // last, partial tile (or a surplus wave): clamp the row
            const uint32_t nbg = tail ? nbg_tail : 8;
            const uint32_t nch = (nbg * 66 + 15) >> 4;
            gptr_t base = (gptr_t)pb.matrix + (size_t)grp * 528;
#pragma unroll
            for (int i = 0; i < kStageLoads; i++) {
                uint32_t ch = lane + 64 * i;
                if (ch >= 16 * nch) ch = 16 * nch - 1;
                const uint32_t row = ch / nch, j = ch - row * nch;
                uint32_t grow = (tile << 4) + row;
                if (grow >= rows) grow = rows - 1;                   // rows past the end re-read the last row (never stored)
                pre[i] = ld16_align2(base + (size_t)grow * row_bytes + j * 16);
            }
        }
    };

    // The first item's loads go out ahead of the tables where they need none (a full group of a full tile): the lane's nine
    // offsets are computed here once; the loop reads them from the table, which costs no registers.
    bool first_issued = false;
    if (nitems) {
        uint32_t grp, tile; Tq2Problem pb;
        item_tile_base(cur, grp, tile, pb);
        if (!(grp + 1 == ngroups && (nb & 7)) && (tile << 4) + 16 <= rows) {
            uint32_t offs[kStageLoads];
#pragma unroll
            for (int i = 0; i < kStageLoads; i++) {
                const uint32_t ch = lane + 64 * i, cf = ch < 16 * 33 ? ch : 16 * 33 - 1, rf = cf / 33, jf = cf - rf * 33;
                offs[i] = rf * row_bytes + jf * 16;
            }
            prefetch(cur, offs);
            first_issued = true;
        }
    }
    {   // every thread fills its share of the tables (one wave doing all nine rounds is a microsecond at the head of a launch)
        const uint32_t nch_t = (nbg_tail * 66 + 15) >> 4, ss_t = (nch_t | 1) * 16;
        for (uint32_t ch = threadIdx.x; ch < kStageLoads * 64; ch += blockDim.x) {
            const uint32_t cf = ch < 16 * 33 ? ch : 16 * 33 - 1, rf = cf / 33, jf = cf - rf * 33;
            full_tab[ch] = (uint16_t)(rf * row_bytes + jf * 16);
            const uint32_t ct = ch < 16 * nch_t ? ch : 16 * nch_t - 1, rt = ct / nch_t, jt = ct - rt * nch_t;
            tail_tab[ch] = (uint16_t)(rt * row_bytes + jt * 16);
            tail_tab[kStageLoads * 64 + ch] = ch < 16 * nch_t ? (uint16_t)(rt * ss_t + jt * 16) : (uint16_t)0xFFFFu;   // surplus lanes do not store
        }
    }
    __syncthreads();
    if (nitems && !first_issued) {
        uint32_t offs[kStageLoads];
#pragma unroll
        for (int i = 0; i < kStageLoads; i++) offs[i] = full_tab[i * 64 + lane];
        prefetch(cur, offs);
    }
    const void* staged = nullptr;
    float rowacc[4] = {0.f, 0.f, 0.f, 0.f};
    for (uint32_t n = 0; n < nitems; n++) {
        uint32_t grp, tile; Tq2Problem pb;
        item_tile_base(cur, grp, tile, pb);
        const Item nxt = advance(cur);
        if (pb.vector != staged) {                                   // uniform over the workgroup
            __syncthreads();
            struct ProWords { uint32_t w[kProWords]; } words;
#pragma unroll
            for (uint32_t i = 0; i < kProWords; i++) words.w[i] = (uint32_t)__builtin_amdgcn_readfirstlane((int)pro_words[i]);
            const XPrologue pro = __builtin_bit_cast(XPrologue, words);
            quantize_x_to_lds<kL, 256, XT>(static_cast<const XT*>(pb.vector), K, xq, xs, xn, blockDim.x, pro, &resid, kq);
            __syncthreads();
            staged = pb.vector;
        }
        const uint32_t b0 = grp << 3;
        const uint32_t nbg = nb - b0 < 8 ? nb - b0 : 8;
        const uint32_t nch = (nbg * 66 + 15) >> 4;
        const uint32_t seg_stride = (nch | 1) * 16;                  // odd number of 16-byte chunks: conflict-free row stride
        (void)nch;

        __builtin_amdgcn_s_setprio(0);   // (raised below, once the item's data is in the image)
        // ---- park the prefetched chunks in the wave's LDS image, then start the next item's loads
        uint32_t offs[kStageLoads];
#pragma unroll
        for (int i = 0; i < kStageLoads; i++) offs[i] = full_tab[i * 64 + lane];
        __builtin_amdgcn_wave_barrier();
        if (nbg == 8) {
#pragma unroll
            for (int i = 0; i < kStageLoads; i++)
                if (i < kStageLoads - 1 || lane < 16 * 33 - 64 * (kStageLoads - 1))   // 528 chunks: the last round is partial
                    *reinterpret_cast<u32x4_t*>(image + lane * 16 + 1024 * i) = pre[i];
        } else {
#pragma unroll
            for (int i = 0; i < kStageLoads; i++) {
                const uint32_t lo = tail_tab[(kStageLoads + i) * 64 + lane];
                if (lo != 0xFFFFu) *reinterpret_cast<u32x4_t*>(image + lo) = pre[i];
            }
        }
        __builtin_amdgcn_wave_barrier();
        if (n + 1 < nitems) prefetch(nxt, offs);
        // From here to the end of the item the wave has everything it needs: it runs at a raised priority, so that of the
        // waves of a SIMD the one that can finish an item does, and gets to its next wait -- and with it to the loads after
        // that -- sooner (8192 x 2048 grouped: 0.726-0.729 -> 0.744-0.752 of the HBM rate; 2048 x 8192: 0.69-0.70 ->
        // 0.71-0.72; raising it ahead of the loads instead changes nothing).
        __builtin_amdgcn_s_setprio(1);
        cur = nxt;

        // ---- column constants of this group
        const bool col_valid = b0 + cb < nb;
        const uint32_t dblk = col_valid ? b0 + cb : nb - 1;
        const uint8_t* arow = image + r * seg_stride + g * 16;
        // A second pass over the same image adds the residual level of the activations when a block of this group has one.
        uint32_t npass = 1;
        if (__builtin_amdgcn_ballot_w64(col_valid && xs[2 * nb + dblk] != 0.0f) != 0) npass = 2;
#pragma nounroll
        for (uint32_t pass = 0; pass < npass; pass++) {
        const float xscale16 = (col_valid && cl == 0) ? xs[pass * 2 * nb + dblk] * 0.0625f : 0.0f;   // high-limb columns and padding add nothing
        const int nsum16 = col_valid ? xn[pass * 2 * nb + dblk] << 4 : 0;
        const uint32_t my_off = col_valid ? lane_x_off + dblk * 256u + pass * (uint32_t)(kL * plane_bytes(K)) : zero_off;

        // accumulators by code scale: fields 0 and 1 arrive as code, field 2 as 4*code, field 3 as 16*code
        v4i acc1 = (v4i){0, 0, 0, 0}, acc4 = (v4i){0, 0, 0, 0}, acc16 = (v4i){0, 0, 0, 0};
#define LH_TQ2_BLOCK(B, GUARD)                                                                                         \
        if (!(GUARD) || (B) < nbg) {                                                                                        \
            constexpr int o = (B) * 66;                                                                         \
            const u32x4_t c0 = *reinterpret_cast<const u32x4_t*>(arow + (o & ~15));                             \
            const u32x4_t c1 = *reinterpret_cast<const u32x4_t*>(arow + (o & ~15) + 16);                        \
            uint32_t wv[4];                                                                                     \
            take16<(o & 15)>(c0, c1, wv);                                                                       \
            v4i a0, a1, a2, a3;                                                                                 \
            _Pragma("unroll") for (int m = 0; m < 4; m++) {                                                     \
                const uint32_t t = wv[m] >> 2;                                                                  \
                a0[m] = (int)(wv[m] & 0x03030303u);                                                             \
                a1[m] = (int)(t & 0x03030303u);                                                                 \
                a2[m] = (int)(t & 0x0C0C0C0Cu);                                                                 \
                a3[m] = (int)(t & 0x30303030u);                                                                 \
            }                                                                                                   \
            const uint8_t* bq = lds + (cb == (B) ? my_off : zero_off);                                          \
            const v4i x0 = *reinterpret_cast<const v4i*>(bq);                                                   \
            const v4i x1 = *reinterpret_cast<const v4i*>(bq + 32);                                              \
            const v4i x2 = *reinterpret_cast<const v4i*>(bq + 64);                                              \
            const v4i x3 = *reinterpret_cast<const v4i*>(bq + 96);                                              \
            acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a0, x0, acc1, 0, 0, 0);                                \
            acc1 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a1, x1, acc1, 0, 0, 0);                                \
            acc4 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a2, x2, acc4, 0, 0, 0);                                \
            acc16 = __builtin_amdgcn_mfma_i32_16x16x64_i8(a3, x3, acc16, 0, 0, 0);                              \
        }
        if (nbg == 8) {   // full group: no branches between the blocks, so their LDS reads and MFMAs interleave
            LH_TQ2_BLOCK(0, false) LH_TQ2_BLOCK(1, false) LH_TQ2_BLOCK(2, false) LH_TQ2_BLOCK(3, false)
            LH_TQ2_BLOCK(4, false) LH_TQ2_BLOCK(5, false) LH_TQ2_BLOCK(6, false) LH_TQ2_BLOCK(7, false)
        } else {
            LH_TQ2_BLOCK(0, true) LH_TQ2_BLOCK(1, true) LH_TQ2_BLOCK(2, true) LH_TQ2_BLOCK(3, true)
            LH_TQ2_BLOCK(4, true) LH_TQ2_BLOCK(5, true) LH_TQ2_BLOCK(6, true) LH_TQ2_BLOCK(7, true)
        }
#undef LH_TQ2_BLOCK

        // ---- epilogue on the dense accumulator: combine scales and limbs, zero point, block scales
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int t16 = (acc1[i] << 4) + (acc4[i] << 2) + acc16[i];                       // 16 * sum(code * limb)
            const int hi = __builtin_amdgcn_update_dpp(0, t16, 0xF5, 0xF, 0xF, true);         // quad_perm [1,1,3,3]: odd neighbour
            const int iq16 = t16 + (hi << 8) - nsum16;                                        // 16 * sum((code - 1) * n), even columns
            const uint16_t dbits = *reinterpret_cast<const uint16_t*>(image + (4 * g + i) * seg_stride + (col_valid ? cb : nbg - 1) * 66 + 64);
            rowacc[i] += (float)iq16 * (lh_h2f(dbits) * xscale16);
        }
        }   // pass

        if (grp + grp_step >= ngroups) {      // tile complete for this wave: sum the 16 columns of each row (4 rows per lane group)
            YT* y = static_cast<YT*>(pb.output);
            float* part = reinterpret_cast<float*>(tail_tab + 3 * kStageLoads * 64);   // [kRing][nwaves][16] partial rows (splitk); 4-byte aligned: 3456 bytes of tables
            float parts[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float v = rowacc[i];
                v += lh_dpp_f<LH_DPP_QUAD_XOR1>(v);
                v += lh_dpp_f<LH_DPP_QUAD_XOR2>(v);
                v += lh_dpp_f<LH_DPP_HALF_MIRROR>(v);
                v += lh_dpp_f<LH_DPP_ROW_MIRROR>(v);
                const uint32_t orow = (tile << 4) + 4 * g + i;
                if (!splitk) {
                    if (c == 0 && tile < tiles_per_problem && orow < rows) lh_store_from_f32<YT>(y, orow, v);
                }
                parts[i] = v;
                rowacc[i] = 0.0f;
            }
            if (splitk) {
                // Every wave of the workgroup reaches this point once per slot, in the same slot order, but not in step:
                // a wave parks its sixteen partial rows in a ring slot and counts itself in; whichever wave arrives last
                // sums the partials in wave order (so the result does not depend on the order of arrival), stores the
                // rows and opens the ring slot for its next use.  No workgroup barrier: a wave waits only when it is kRing
                // tiles ahead of the slowest wave of its tile.
                uint32_t* sync = reinterpret_cast<uint32_t*>(part + kRing * kMaxWavesPerWG * 16) + tsub * 2 * kRing;   // this tile's arrivals[kRing], generation[kRing]
                float* tpart = part + (size_t)tsub * sw * 16;                                  // ring slot r of this tile: tpart + r * nwaves * 16
                const uint32_t gw = (uint32_t)wave % sw;
                const uint32_t ring = slot_seq % kRing, gen = slot_seq / kRing;
                // Ordering: the LDS unit executes a wave's operations in issue order, so "partial rows, then the arrival
                // count" and "count reset, then the generation word" need no more than a wait for this wave's own LDS
                // operations (lgkmcnt) and a compiler barrier.  A fence of workgroup scope would also wait for the wave's
                // outstanding global loads -- the next tile's prefetch -- and is deliberately not used.
                auto lds_order = [] { __builtin_amdgcn_s_waitcnt(0xC07F); asm volatile("" ::: "memory"); };   // lgkmcnt(0) only
                if (gen) {   // the slot's previous use must have been summed (bounded wait: never expected to run out)
                    bool seen = __hip_atomic_load(&sync[kRing + ring], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == gen;
                    if (!seen) {
                        const kernargs_t ka = cold_kernargs();
                        const uint32_t spin_limit = ka->single.spin_limit;
                        uint32_t spins = 0;
                        while (!(seen = __hip_atomic_load(&sync[kRing + ring], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == gen) &&
                               spins++ < spin_limit)
                            __builtin_amdgcn_s_sleep(2);
                        // Out of patience: the wave goes on (every wave must reach the end of the kernel), the rows of this
                        // tile are not to be trusted, and the host learns of it at its next wait on the stream.
                        uint32_t* fault = ka->single.fault;
                        if (!seen && lane == 0 && fault)
                            __hip_atomic_store(fault, (uint32_t)LH_FAULT_TQ2_SPLIT_WAIT, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    }
                    lds_order();
                }
                if (c == 0) {
#pragma unroll
                    for (int i = 0; i < 4; i++) tpart[(ring * nwaves + gw) * 16 + 4 * g + i] = parts[i];
                }
                lds_order();
                uint32_t arrived = 0;
                if (lane == 0) arrived = __hip_atomic_fetch_add(&sync[ring], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                arrived = (uint32_t)__builtin_amdgcn_readfirstlane((int)arrived);
                if (arrived == sw - 1u) {
                    lds_order();
                    if (lane < 16) {
                        float v = tpart[(ring * nwaves) * 16 + lane];
                        for (uint32_t w = 1; w < sw; w++) v += tpart[(ring * nwaves + w) * 16 + lane];
                        const uint32_t orow = (tile << 4) + lane;
                        if (tile < tiles_per_problem && orow < rows) lh_store_from_f32<YT>(y, orow, v);
                    }
                    lds_order();
                    if (lane == 0) {
                        __hip_atomic_store(&sync[ring], 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                        lds_order();
                        __hip_atomic_store(&sync[kRing + ring], gen + 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                }
                slot_seq++;
            }
        }
    }
}

}  // namespace

static std::atomic<uint32_t> g_tq2_spin_limit{1u << 20};
extern "C" void lh_debug_set_tq2_split_spin_limit(uint32_t polls) { g_tq2_spin_limit.store(polls, std::memory_order_relaxed); }

// Entry used by matvec_quant.hip's dispatcher. Arrays are host arrays of device pointers.
int lh_launch_matvec_tq2_mfma(lh_context* ctx, uint32_t count, const void* const* matrices, const void* const* vectors,
                              void* const* outputs, lh_dtype xt, lh_dtype yt, uint32_t rows, uint32_t K, uint32_t xstride,
                              uint32_t ystride, const XPrologue& pro, uint64_t mstride) {
    const bool strided = xstride != 0 || ystride != 0 || mstride != 0;   // problem i = problem 0 advanced by i strides: no descriptor table
    const uint32_t nb = K >> 8;
    const uint64_t tiles = (uint64_t)((rows + 15) >> 4) * count;
    // small jobs: one wave per workgroup so the tiles spread over all CUs; large jobs: four waves share one
    // quantised activation vector; few tiles with long rows: the block groups of a tile are split over 2-4 waves
    const uint32_t ngroups = (nb + 7) >> 3;
    uint32_t split_waves = 1;
    if (tiles < (uint64_t)ctx->cu_count * 2) {
        for (uint32_t w = 4; w >= 2; w--) if (ngroups % w == 0) { split_waves = w; break; }
        // six groups of blocks (12288 columns, the down projection of the wide feed-forward layers): a wave per group,
        // and twice the threads for the activation staging (f16 in and out only: the decode path's types)
        const size_t lds6 = lds_head_bytes(K) + 128 + 6 * (size_t)kImageBytes + 3 * kStageLoads * 64 * 2 + kSplitAreaBytes;
        if (ngroups % 6 == 0 && xt == LH_F16 && yt == LH_F16 && lds6 <= kMaxLdsBytes) split_waves = 6;
    }
    const uint32_t splitk = split_waves > 1 ? 1u : 0u;
    constexpr int wg256_tiles_per_cu = 2, wg_cu = 3;
    auto lds_for = [&](uint32_t nwaves) { return lds_head_bytes(K) + 128 + (size_t)nwaves * kImageBytes + 3 * kStageLoads * 64 * 2 + kSplitAreaBytes; };
    uint32_t threads = splitk ? 64 * split_waves : (tiles >= (uint64_t)ctx->cu_count * wg256_tiles_per_cu ? 256 : 64);
    // Long rows make the activation area large: when fewer than three four-wave workgroups fit a CU's LDS, a large job runs
    // one twelve-wave workgroup per CU instead, which stages the activations once and keeps three waves on every SIMD
    // (four-wave workgroups measured 0.70 of the HBM rate on 2048 x 8192 weights where this form reaches 0.71).
    bool wide = false;
    uint32_t wide_split = 0;     // waves per tile when the twelve-wave workgroup runs in split form
    if (!splitk && threads == 256 && (160 * 1024) / lds_for(4) < 3 && lds_for(12) <= kMaxLdsBytes &&
        tiles >= (uint64_t)ctx->cu_count * 24) {
        wide = true;
        threads = 768;
        // the block groups of a tile on neighbouring waves: the segments of one row are then fetched close together in time
        if (ngroups > 1 && 12 % ngroups == 0) wide_split = ngroups;   // (one wave walking all groups of its tile: 0.65 against 0.71)
    }
    // Few tiles, split over four waves each, f16 in and out, an even number of tiles (the decode path's down projection over
    // 8192 columns): two tiles per workgroup of eight waves, so that twice the threads stage the activation vector and half
    // as many workgroups stage it at all (a single-token decode layer: 64.4 -> 63.5 us).
    bool pair_tiles = false;
    if (splitk && split_waves == 4 && xt == LH_F16 && yt == LH_F16 && count == 1 && (((rows + 15) >> 4) & 1) == 0 && lds_for(8) <= kMaxLdsBytes) {
        pair_tiles = true;
        threads = 512;
        wide_split = 4;
    }
    const uint32_t waves = threads / 64;
    const uint32_t tiles_per_slot = wide_split ? waves / wide_split : (splitk ? 1u : waves);
    const uint64_t slots = (uint64_t)(((rows + 15) >> 4) + tiles_per_slot - 1) / tiles_per_slot * count;
    const size_t lds_bytes = lds_for(waves);
    const int lds_fit = (int)std::max<size_t>(1, (160 * 1024) / lds_bytes);          // workgroups per CU that LDS allows
    const int wg_eff = wide ? 1 : (threads == 256 ? std::min(wg_cu, lds_fit) : 4 * wg_cu);
    const uint64_t cap = (uint64_t)ctx->cu_count * wg_eff;
    const uint32_t grid = (uint32_t)(slots < cap ? (slots ? slots : 1) : cap);
    if (lds_bytes > kMaxLdsBytes) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_tq2_0: cols %u need %zu bytes of LDS", K, lds_bytes);
    if ((slots / grid + 1) * ngroups > 0xFFFFFFFFull)   // the kernel counts a workgroup's (tile, block group) items in 32 bits
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_tq2_0: %u problems of %u rows are more than one launch takes", count, rows);
    const void* fn;
    if (pair_tiles) fn = (const void*)matvec_tq2_mfma_kernel<uint16_t, uint16_t, true, 512>;
    else if (split_waves == 6) fn = (const void*)matvec_tq2_mfma_kernel<uint16_t, uint16_t, true, 384>;
#define LH_FN(XT, YT) (wide_split ? (const void*)matvec_tq2_mfma_kernel<XT, YT, true, 768, true>                                       \
                            : wide ? (const void*)matvec_tq2_mfma_kernel<XT, YT, false, 768>                                      \
                            : splitk ? (const void*)matvec_tq2_mfma_kernel<XT, YT, true>                                          \
                            : ngroups == 1 ? (const void*)matvec_tq2_mfma_kernel<XT, YT, false, 256, true>                        \
                                           : (const void*)matvec_tq2_mfma_kernel<XT, YT, false>)
    else if (xt == LH_F32 && yt == LH_F32) fn = LH_FN(float, float);
    else if (xt == LH_F16 && yt == LH_F16) fn = LH_FN(uint16_t, uint16_t);
    else if (xt == LH_F16 && yt == LH_F32) fn = LH_FN(uint16_t, float);
    else fn = LH_FN(float, uint16_t);
#undef LH_FN
    if (lds_bytes > 64 * 1024) {   // more than the 64 KB a kernel gets without asking
        const int rl = lh_raise_dynamic_lds(ctx, fn, kMaxLdsBytes, "matvec_tq2_0");
        if (rl != LH_OK) return rl;
    }

    Tq2Base single{Tq2Problem{(const uint8_t*)matrices[0], vectors[0], outputs[0]}, xstride, ystride};
    single.mstride = mstride;
    single.split_waves = wide_split;
    single.pro = pro;
    single.spin_limit = g_tq2_spin_limit.load(std::memory_order_relaxed);
    single.fault = ctx->fault_dev;
    Tq2Problem* dev = nullptr;
    if (count == 2 && !strided) {
        single.second = Tq2Problem{(const uint8_t*)matrices[1], vectors[1], outputs[1]};
        single.pair = 1;
    } else if (count > 2 && !strided) {
        if (ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_tq2_0: more than two grouped problems need a descriptor upload, which a captured graph cannot hold");
        const size_t bytes = (size_t)count * sizeof(Tq2Problem);
        if (bytes > ctx->workspace_bytes / 4) return lh_fail(LH_ERR_INVALID_ARGUMENT, "matvec_tq2_0: %u problems exceed the descriptor area", count);
        Tq2Problem* host = (Tq2Problem*)malloc(bytes);
        if (!host) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", bytes);
        for (uint32_t i = 0; i < count; i++) host[i] = Tq2Problem{(const uint8_t*)matrices[i], vectors[i], outputs[i]};
        dev = (Tq2Problem*)((char*)ctx->workspace + ctx->workspace_bytes - ctx->workspace_bytes / 4);
        const int ru = lh_upload_descriptors(ctx, host, bytes, dev, "matvec_tq2_0");
        free(host);   // staged by the helper
        if (ru != LH_OK) return ru;
    }
    const Tq2Problem* dev_arg = dev;
    void* args[] = {(void*)&dev_arg, (void*)&single, (void*)&count, (void*)&rows, (void*)&K};
    hipError_t le = hipLaunchKernel(fn, dim3(grid), dim3(threads), args, lds_bytes, ctx->stream);
    if (le != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: matvec_tq2_0 launch failed: %s", hipGetErrorString(le));
    return lh_check_launch("matvec_tq2_0");
}
