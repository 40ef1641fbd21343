// Issue model of one gfx950 SIMD: do vector-ALU and matrix-core instructions overlap?
//
// The attention, TQ2_0 matvec and prefill kernels of this library all interleave v_mfma_i32_16x16x64_i8 (or its f16
// sibling) with a larger number of ordinary vector instructions, from one or several waves per SIMD.  Whether their
// speed is "the longer of the two streams" or "the sum of both" decides which optimisations are worth trying.  This
// probe times fixed mixes at 1 .. 4 waves per SIMD, with the two kinds of instruction in one wave (finely or coarsely
// interleaved) or on different waves of the same SIMD, and prints nanoseconds per iteration and the SIMD cycles per
// instruction that follow from the clock the device reports.  One workgroup per CU, so waves per SIMD = threads / 256.
//
//   hipcc -O3 --offload-arch=gfx950 -o issue_model_probe issue_model.hip && ./issue_model_probe
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

enum Mix { kValu = 0, kMfma, kFine, kCoarse, kSplitWaves, kPerm, kFma, kExp, kValuSgpr, kAndOnlyLit, kAndOnlySgpr,
           kAndVgpr, kMulLit, kMulVgpr, kShiftLit, kShlAdd, kCvt, kTileF16, kTileI8 };

// One iteration per wave: 160 (v_and_b32, v_add_u32) pairs = 320 vector instructions and / or 16 MFMAs (kFine: 80 pairs
// between 16 MFMAs; kSplitWaves: even waves the 160 pairs, odd waves the 16 MFMAs), or 160 instructions of one other kind.
// The instruction counts handed to run() are those of the compiled loop bodies (hipcc -S): the and-xor chains of the last two
// integer mixes compile to v_bitop3_b32 and v_xor_b32, 320 and 312 instructions.
template <int MIX, int MAXT>
__global__ __launch_bounds__(MAXT) void mix_kernel(int iters, int* out, unsigned mask, unsigned step) {
    unsigned x[8];
    float f[8];
    v4i acc[4];
    for (int i = 0; i < 8; i++) { x[i] = threadIdx.x * 2654435761u + i; f[i] = 1.0f + threadIdx.x * 1e-3f + i; }
    for (int i = 0; i < 4; i++) acc[i] = (v4i){0, 0, 0, 0};
    const v4i a = (v4i){(int)threadIdx.x, 1, 2, 3}, b = (v4i){4, 5, (int)threadIdx.x, 7};
    const bool odd_wave = (threadIdx.x >> 6) & 1;
    // state of the two "prefill tile step" mixes: float sums of 16 tiles, four row-tile and four column-tile operands
    v4f tc[16];
    v8h ha[4], hb[4];
    v4i ia[4], il[4], ih[4];
    if constexpr (MIX == kTileF16 || MIX == kTileI8) {
#pragma unroll
        for (int t = 0; t < 16; t++) tc[t] = (v4f){(float)t, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; q++) {
#pragma unroll
            for (int j = 0; j < 8; j++) { ha[q][j] = (_Float16)(f[j] + (float)q); hb[q][j] = (_Float16)(f[(j + q) & 7] - (float)q); }
            ia[q] = a + (v4i){q, 1, q, 3}; il[q] = b - (v4i){q, q, 2, 1}; ih[q] = b ^ (v4i){3, q, q, 7};
        }
    }
    for (int it = 0; it < iters; it++) {
        if constexpr (MIX == kValu || MIX == kCoarse) {
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) x[i] = (x[i] & 0x7f7f7f7fu) + 0x01010101u * (i + 1);   // v_and_b32 + v_add_u32, both with a 32-bit literal
        }
        if constexpr (MIX == kMfma || MIX == kCoarse) {
#pragma unroll
            for (int r = 0; r < 16; r++) acc[r & 3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[r & 3], 0, 0, 0);
        }
        if constexpr (MIX == kFine) {
#pragma unroll
            for (int r = 0; r < 16; r++) {
#pragma unroll
                for (int i = 0; i < 5; i++) x[i] = (x[i] & 0x7f7f7f7fu) + 0x01010101u * (i + 1);
                acc[r & 3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[r & 3], 0, 0, 0);
            }
        }
        if constexpr (MIX == kSplitWaves) {
            if (odd_wave) {
#pragma unroll
                for (int r = 0; r < 16; r++) acc[r & 3] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, acc[r & 3], 0, 0, 0);
            } else {
#pragma unroll
                for (int r = 0; r < 20; r++)
#pragma unroll
                    for (int i = 0; i < 8; i++) x[i] = (x[i] & 0x7f7f7f7fu) + 0x01010101u * (i + 1);
            }
        }
        if constexpr (MIX == kPerm) {
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) x[i] = __builtin_amdgcn_perm(x[i], x[(i + 1) & 7], 0x05010400u);
        }
        if constexpr (MIX == kFma) {
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) f[i] = __builtin_fmaf(f[i], 1.0001f, 0.5f);
        }
        if constexpr (MIX == kValuSgpr) {   // the same pairs with the mask and the addend in scalar registers (no 32-bit literals)
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) x[i] = (x[i] & mask) + step;
        }
        if constexpr (MIX == kAndOnlyLit) {   // an and-xor chain with a different 32-bit literal per element
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) x[i] = (x[(i + 1) & 7] & (0x7f7f7f7fu - 0x01010101u * (unsigned)i)) ^ x[i];
        }
        if constexpr (MIX == kAndOnlySgpr) {
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) x[i] = (x[(i + 1) & 7] & mask) ^ x[i];
        }
        // (the next six are written as single instructions: the compiler would regroup the C forms)
#define LH_PROBE_160(STMT)                                   \
        _Pragma("unroll") for (int r = 0; r < 20; r++)       \
            _Pragma("unroll") for (int i = 0; i < 8; i++) { STMT; }
        if constexpr (MIX == kAndVgpr) {   // both operands in vector registers
            LH_PROBE_160(asm volatile("v_and_b32 %0, %0, %1\n\tv_add_u32 %0, %0, %2" : "+v"(x[i]) : "v"(x[(i + 3) & 7]), "v"(x[(i + 5) & 7])))
        }
        if constexpr (MIX == kMulLit) {
            LH_PROBE_160(asm volatile("v_mul_f32 %0, 0x3f800347, %0" : "+v"(f[i])))
        }
        if constexpr (MIX == kMulVgpr) {
            LH_PROBE_160(asm volatile("v_mul_f32 %0, %0, %1" : "+v"(f[i]) : "v"(f[(i + 3) & 7])))
        }
        if constexpr (MIX == kShiftLit) {
            LH_PROBE_160(asm volatile("v_lshrrev_b32 %0, 3, %0\n\tv_xor_b32 %0, 0x5a5a5a5a, %0" : "+v"(x[i])))
        }
        if constexpr (MIX == kShlAdd) {
            LH_PROBE_160(asm volatile("v_lshl_add_u32 %0, %0, 2, %1" : "+v"(x[i]) : "v"(x[(i + 3) & 7])))
        }
        if constexpr (MIX == kCvt) {
            LH_PROBE_160(asm volatile("v_cvt_f32_i32 %0, %0" : "+v"(f[i])))
        }
#undef LH_PROBE_160
        // One 256-column weight block of a 64 x 64 output tile of a prefill matmul, as one multiplying wave issues it:
        // f16 form: 16 accumulator tiles x 8 k steps of v_mfma_f32_16x16x32_f16 into float sums that stay where they are.
        // int8 form with 16-bit activations in two limbs: 16 tiles x 4 k steps x 2 limbs of v_mfma_i32_16x16x64_i8 into
        // int32 sums, which have to leave the integers once per block -- per output (64 per lane) a shift-add of the
        // limbs, a conversion and a multiply-add with the block's scale product.
        if constexpr (MIX == kTileF16) {
#pragma unroll
            for (int k = 0; k < 8; k++)
#pragma unroll
                for (int t = 0; t < 16; t++) tc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ha[t >> 2], hb[t & 3], tc[t], 0, 0, 0);
        }
        if constexpr (MIX == kTileI8) {
            v4i lo[16], hi[16];
#pragma unroll
            for (int t = 0; t < 16; t++) lo[t] = hi[t] = (v4i){0, 0, 0, 0};
#pragma unroll
            for (int k = 0; k < 4; k++)
#pragma unroll
                for (int t = 0; t < 16; t++) {
                    lo[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ia[t >> 2], il[t & 3], lo[t], 0, 0, 0);
                    hi[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(ia[t >> 2], ih[t & 3], hi[t], 0, 0, 0);
                }
#pragma unroll
            for (int t = 0; t < 16; t++)
#pragma unroll
                for (int i = 0; i < 4; i++) tc[t][i] = __builtin_fmaf((float)((hi[t][i] << 8) + lo[t][i]), f[(t + i) & 7], tc[t][i]);
        }
        if constexpr (MIX == kExp) {
#pragma unroll
            for (int r = 0; r < 20; r++)
#pragma unroll
                for (int i = 0; i < 8; i++) f[i] = __builtin_amdgcn_exp2f(f[i]);
        }
    }
    if constexpr (MIX == kTileF16 || MIX == kTileI8) {
#pragma unroll
        for (int t = 0; t < 16; t++) f[t & 7] += tc[t][0] + tc[t][1] + tc[t][2] + tc[t][3];
    }
    unsigned s = 0;
    for (int i = 0; i < 8; i++) s ^= x[i] ^ __float_as_uint(f[i]);
    for (int i = 0; i < 4; i++) s ^= (unsigned)(acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3]);
    if (s == 0x12345u) out[0] = (int)s;   // keeps the work alive
}

static double g_ghz = 0.0;
static unsigned g_mask = 0x7f7f7f7fu, g_step = 0x01010101u;   // reach the kernels as arguments, i.e. in scalar registers

template <int MIX, int MAXT = 1024>
static void run(const char* name, int valu_per_wave, int mfma_per_wave, int* d) {
    hipEvent_t e0, e1;
    if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) { fprintf(stderr, "hipEventCreate failed\n"); exit(1); }
    const int iters = 4000;
    printf("%-44s", name);
    for (int wps = 1; wps <= 4; wps++) {
        if ((MIX == kSplitWaves && (wps & 1)) || 256 * wps > MAXT) { printf(" | %-27s", "-"); continue; }
        float ms = 0;
        for (int rep = 0; rep < 3; rep++) {   // the last repetition counts (clocks up, code resident)
            (void)hipEventRecord(e0);
            hipLaunchKernelGGL((mix_kernel<MIX, MAXT>), dim3(256), dim3(256 * wps), 0, 0, iters, d, g_mask, g_step);
            (void)hipEventRecord(e1);
            if (hipEventSynchronize(e1) != hipSuccess) { fprintf(stderr, "kernel failed\n"); exit(1); }
            (void)hipEventElapsedTime(&ms, e0, e1);
        }
        const double ns = ms * 1e6 / iters;
        // cycles one SIMD spends per iteration of ALL its waves, against 4 per vector instruction + 16 per MFMA if they add
        const int waves_v = MIX == kSplitWaves ? wps / 2 : wps, waves_m = MIX == kSplitWaves ? wps / 2 : wps;
        const double model = 4.0 * valu_per_wave * waves_v + 16.0 * mfma_per_wave * waves_m;
        printf(" | %7.1f ns %6.0f cyc (%4.2f)", ns, ns * g_ghz, ns * g_ghz / model);
    }
    printf("\n");
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
}

int main() {
    int* d = nullptr;
    if (hipMalloc(&d, 4) != hipSuccess) { fprintf(stderr, "no device\n"); return 1; }
    int khz = 0;
    (void)hipDeviceGetAttribute(&khz, hipDeviceAttributeClockRate, 0);
    g_ghz = khz * 1e-6;
    printf("clock reported by the device: %.2f GHz; columns: 1, 2, 3, 4 waves per SIMD; per column: time per iteration, SIMD cycles at\n"
           "that clock, and (ratio to the additive model: 4 cycles per vector instruction + 16 per MFMA, summed over the SIMD's waves)\n", g_ghz);
    run<kValu>("160 x (v_and + v_add), literal operands", 320, 0, d);
    run<kValuSgpr>("160 x (v_and + v_add), SGPR operands", 320, 0, d);
    run<kAndOnlyLit>("320 v_bitop3/v_xor, literal masks", 320, 0, d);
    run<kAndOnlySgpr>("312 v_bitop3/v_xor, SGPR mask", 312, 0, d);
    run<kAndVgpr>("160 x (v_and + v_add), two VGPR operands", 320, 0, d);
    run<kShiftLit>("160 x (v_lshrrev + v_xor), literal operands", 320, 0, d);
    run<kMulLit>("160 v_mul_f32, literal factor", 160, 0, d);
    run<kMulVgpr>("160 v_mul_f32, two VGPR operands", 160, 0, d);
    run<kShlAdd>("160 v_lshl_add_u32", 160, 0, d);
    run<kCvt>("160 v_cvt_f32_i32", 160, 0, d);
    run<kPerm>("160 v_perm_b32", 160, 0, d);
    run<kFma>("160 v_fma_f32", 160, 0, d);
    run<kExp>("160 v_exp_f32", 160, 0, d);
    run<kMfma>("16 MFMA", 0, 16, d);
    // (launched for at most two waves per SIMD: the int8 form's 32 accumulator tiles need more than 128 registers)
    run<kTileF16, 512>("prefill tile step, f16: 128 MFMA f16", 0, 128, d);
    run<kTileI8, 512>("prefill tile step, int8: 128 MFMA i8 + 192", 192, 128, d);
    run<kFine>("16 x (5 x (v_and + v_add) + 1 MFMA)", 160, 16, d);
    run<kCoarse>("160 x (v_and + v_add), then 16 MFMA", 320, 16, d);
    run<kSplitWaves>("even waves 160 x (and + add), odd 16 MFMA", 320, 16, d);
    (void)hipFree(d);
    return 0;
}
