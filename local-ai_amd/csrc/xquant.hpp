// Activation quantisation shared by the quantized-weight matvec kernels: x -> block fixed point.
// Per group of G elements (G = weight block size): a float scale s = max|x| / qmax and integers
// n_i = rint(x_i / s), split into L signed 8-bit limbs (n = sum_l limb_l * 256^l) so that dot
// products with small unsigned weight codes are exact in v_dot4_i32_i8 / MFMA i8 arithmetic.
#pragma once
#include "common.hpp"

template <int L> struct Limb;
template <> struct Limb<2> { static constexpr float qmax = 32639.0f; };     // 127*256 + 127
template <> struct Limb<3> { static constexpr float qmax = 8355711.0f; };   // 127*65536 + 127*256 + 127

// gelu.metal:31-35: 0.5 x (1 + tanh(clamp(0.79788456 (x + 0.044715 x^3), -10, 10))).  tanh(u) is evaluated as
// 1 - 2 / (1 + e^(2u)) with the hardware exponential and reciprocal (a handful of instructions instead of the library
// routine's several dozen; |u| <= 10 keeps e^(2u) finite): its absolute error of about 1e-7 disappears in 1 + tanh(u),
// far below the f16 result's rounding step.
__device__ __forceinline__ float lh_gelu_tanh_f32(float x) {
    // the two multiply-adds are written as fused operations and nothing else here is a product feeding a sum, so the
    // compiler's contraction has no choice left to make: the kernels that evaluate this (gelu_mul, the matvec
    // prologue, the product epilogue) agree bit for bit whatever code surrounds the call
    const float x3 = x * x * x;
    const float inner = fminf(fmaxf(0.7978845608f * __builtin_fmaf(0.044715f, x3, x), -10.0f), 10.0f);
    const float t = __builtin_fmaf(-2.0f, __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * inner)), 1.0f);
    return 0.5f * x * (1.0f + t);
}

// gelu.metal:37-40: half(gelu(float(a)) * float(b)).  The f32 product passes through an empty asm statement so that it is
// rounded to f32 before it is narrowed (left alone the compiler sometimes narrows the exact product in one mixed-
// precision instruction, sometimes not, and two kernels then disagree in the last bit once in ten thousand values).
__device__ __forceinline__ uint16_t lh_gelu_mul_h(uint16_t a, uint16_t b) {
    float p = lh_gelu_tanh_f32(lh_h2f(a)) * lh_h2f(b);
    asm volatile("" : "+v"(p));
    return lh_f2h(p);
}

// Elements e0 .. e0 + 8 of f16(x * rms * aux (+ res)) as four packed words: the arithmetic of rms_norm_kernel<ADD>, its
// tail forms (pro.tail) included.
// (`a`, `g`, `r`: the eight elements of the vector, the norm weight and -- with pro.res -- the residual, as loaded.)
__device__ __forceinline__ void xpro_norm_add8_regs(const uint4 a, const uint4 g, const uint4 r, const XPrologue& pro, float rms, uint32_t (&packed)[4]) {
    const uint32_t wa[4] = {a.x, a.y, a.z, a.w}, wg[4] = {g.x, g.y, g.z, g.w}, wr[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float lo = lh_norm_product(lh_h2f((uint16_t)(wa[j] & 0xFFFF)), rms, lh_h2f((uint16_t)(wg[j] & 0xFFFF)));
        float hi = lh_norm_product(lh_h2f((uint16_t)(wa[j] >> 16)), rms, lh_h2f((uint16_t)(wg[j] >> 16)));
        if (pro.res != nullptr) {
            const float rlo = lh_h2f((uint16_t)(wr[j] & 0xFFFF)), rhi = lh_h2f((uint16_t)(wr[j] >> 16));
            if (pro.tail) { lo = lh_norm_tail(lo, rlo, pro.tail, pro.scale); hi = lh_norm_tail(hi, rhi, pro.tail, pro.scale); }
            else { lo += rlo; hi += rhi; }
        }
        packed[j] = (uint32_t)lh_f2h_exact(lo) | ((uint32_t)lh_f2h_exact(hi) << 16);
    }
}
__device__ __forceinline__ void xpro_norm_add8(const void* xv, const XPrologue& pro, uint32_t e0, float rms, uint32_t (&packed)[4]) {
    const uint16_t* x = static_cast<const uint16_t*>(xv);
    const uint4 a = *reinterpret_cast<const uint4*>(x + e0), g = *reinterpret_cast<const uint4*>(pro.aux + e0);
    uint4 r = make_uint4(0u, 0u, 0u, 0u);
    if (pro.res != nullptr) r = *reinterpret_cast<const uint4*>(pro.res + e0);
    xpro_norm_add8_regs(a, g, r, pro, rms, packed);
}

// The eight consecutive elements e0 .. e0 + 8 of a head that a lane holds, through the head's Walsh-Hadamard transform,
// 1/sqrt(head_dim) and the sign vector, rounded to f16 once: what hadamard_rotate_kernel<float, f16> stores, bit for bit
// (the same butterflies in the same order of stages; a sum does not depend on which operand is named first).  Stages
// 1, 2, 4 pair elements of one lane, the others pair the lanes of a head, head_dim / 8 <= 64 consecutive lanes of a wave.
// Every lane of the wave calls it; lanes past the vector carry zeros.
__device__ __forceinline__ void xpro_rotate8(float (&v)[8], const XPrologue& pro, uint32_t e0) {
#pragma unroll
    for (int len = 1; len < 8; len <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i & len) continue;
            const float lo = v[i], hi = v[i | len];
            v[i] = __fadd_rn(lo, hi);
            v[i | len] = __fsub_rn(lo, hi);
        }
    }
    const uint32_t lane = threadIdx.x & 63;
    for (uint32_t m = 1; 8 * m < pro.head_dim; m <<= 1) {
        const bool upper = (lane & m) != 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const float other = __shfl_xor(v[i], (int)m, 64);
            v[i] = upper ? __fsub_rn(other, v[i]) : __fadd_rn(v[i], other);
        }
    }
    const uint32_t d0 = e0 & (pro.head_dim - 1);
    const float4 s0 = *reinterpret_cast<const float4*>(pro.signs + d0), s1 = *reinterpret_cast<const float4*>(pro.signs + d0 + 4);
    const float sg[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = lh_h2f(lh_f2h_exact(__fmul_rn(__fmul_rn(v[i], pro.scale), sg[i])));
}

// Second level of the fixed point, for blocks whose first-level step would be too coarse.  A block with max|x| = m has
// the step s = m / qmax; every element carries an absolute error of up to s / 2 whatever its own size, so one large
// element (ordinary in a residual stream) costs its neighbours their low bits.  The test is relative to the block itself:
// with r = mean |x| of the block's other elements, the block is left alone while m <= kXOutlier * r -- the error of an
// element then stays below kXOutlier / (2 qmax) = 4.9e-4 r, and if every block of a vector sat at that limit the error of
// a row sum would still be about 2e-4 of its scale (m / r is 3 .. 6 for Gaussian values of any scale and 9 .. 14 for
// GeGLU products, whose blocks exceed 32 two or three times in a thousand).  A block above the limit also gets the
// residual r_i = x_i - s n_i in 16-bit fixed point of its own (step s * 0.52 / qmax: about 2^-31 of m in all), which the
// kernels add in a second pass over blocks that have one (those with xs2 != 0).
struct XResidual {
    uint32_t* xq2;   // [2][K/4] residual limbs, laid out like xq (written for blocks with a second level only)
    float* xs2;      // [K/G] residual scale; 0 for a block whose first level suffices
    int* xn2;        // [K/G] sum of the residual integers (may be null)
};
constexpr float kXOutlier = 32.0f;

// ---- activation quantisation into LDS ----------------------------------------
// xq[l][K/4]: limb l of elements 4i..4i+3 packed into one dword (signed bytes);
// xs[K/G]: float scale of each group of G elements (G = weight block size).
// `xn` (optional) receives sum(n_i) per group; `nthreads` = workgroup size (multiple of 64).
// A group that holds a NaN or an infinity gets the scale NaN, so every row sum that includes it comes out NaN (the
// reference's f32 dot gives NaN or an infinity there; nothing is silently clamped).
// `resid` (optional, L == 2 only): see XResidual.  `plane_dwords` (optional): distance of the limb planes in dwords.
template <int L, int G, typename XT>
__device__ __forceinline__ void quantize_x_to_lds(const XT* __restrict__ x, uint32_t K, uint32_t* xq, float* xs, int* xn,
                                                  uint32_t nthreads, const XPrologue pro = XPrologue{kXProNone, nullptr, 0.0f},
                                                  const XResidual* resid = nullptr, uint32_t plane_dwords = 0) {
    const int tid = threadIdx.x;
    const uint32_t kq = plane_dwords ? plane_dwords : K >> 2;   // dwords between the limb planes (K / 4 unless the caller pads them)
    float rms = 1.0f, rms2 = 1.0f;
    [[maybe_unused]] bool one_round = false;          // the RMS-norm prologue has left the thread's normalised elements in one_packed
    [[maybe_unused]] uint32_t one_packed[4] = {0u, 0u, 0u, 0u};
    [[maybe_unused]] uint4 one_g2 = make_uint4(0u, 0u, 0u, 0u);

    if constexpr (sizeof(XT) == 2) {
        if (pro.kind == kXProRmsNorm) {   // uniform over the workgroup; xs doubles as the reduction scratch before it is filled
            auto block_total = [&](float s) {
                s = lh_group_sum(s, 64);
                if ((tid & 63) == 0) xs[tid >> 6] = s;
                __syncthreads();
                float t = 0.0f;
                for (uint32_t w = 0; w < nthreads / 64; w++) t += xs[w];
                __syncthreads();
                return t;
            };
            if (K <= nthreads * 8) {
                // One round covers the vector (uniform over the workgroup): everything a thread reads -- its eight elements,
                // their norm weights, the residual, the second norm's weights -- is requested here at once and the passes
                // below work from registers.  Read pass by pass, each pass waits for memory again behind the barriers of
                // the pass before (three trips where this is one); the arithmetic and its order are those of the loops.
                const uint32_t e0 = tid * 8;
                const bool valid = e0 < K;
                const uint4 zero4 = make_uint4(0u, 0u, 0u, 0u);
                uint4 a = zero4, g = zero4, r = zero4;
                one_g2 = zero4;
                if (valid) {
                    a = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(x) + e0);
                    g = *reinterpret_cast<const uint4*>(pro.aux + e0);
                    if (pro.res != nullptr) r = *reinterpret_cast<const uint4*>(pro.res + e0);
                    if (pro.aux2 != nullptr) one_g2 = *reinterpret_cast<const uint4*>(pro.aux2 + e0);
                }
                float s = 0.0f;
                if (valid) {
                    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float lo = lh_h2f((uint16_t)(w[i] & 0xFFFF)), hi = lh_h2f((uint16_t)(w[i] >> 16));
                        s += lo * lo;
                        s += hi * hi;
                    }
                }
                rms = rsqrtf(block_total(s) / (float)K + pro.eps);
                if (valid) xpro_norm_add8_regs(a, g, r, pro, rms, one_packed);
                if (pro.aux2 != nullptr || pro.store != nullptr) {
                    float s2 = 0.0f;
                    if (valid) {
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            const float lo = lh_h2f((uint16_t)(one_packed[i] & 0xFFFF)), hi = lh_h2f((uint16_t)(one_packed[i] >> 16));
                            s2 += lo * lo;
                            s2 += hi * hi;
                        }
                        if (pro.store != nullptr && blockIdx.x == 0)
                            *reinterpret_cast<uint4*>(pro.store + e0) = make_uint4(one_packed[0], one_packed[1], one_packed[2], one_packed[3]);
                    }
                    if (pro.aux2 != nullptr) rms2 = rsqrtf(block_total(s2) / (float)K + pro.eps);
                }
                one_round = true;
            } else {
            float s = 0.0f;
            for (uint32_t e0 = tid * 8; e0 < K; e0 += nthreads * 8) {
                const uint4 a = *reinterpret_cast<const uint4*>(x + e0);
                const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const float lo = lh_h2f((uint16_t)(w[i] & 0xFFFF)), hi = lh_h2f((uint16_t)(w[i] >> 16));
                    s += lo * lo;
                    s += hi * hi;
                }
            }
            rms = rsqrtf(block_total(s) / (float)K + pro.eps);
            if (pro.aux2 != nullptr || pro.store != nullptr) {   // the normalised (+ residual) vector: its mean square, and the one stored copy
                float s2 = 0.0f;
                for (uint32_t e0 = tid * 8; e0 < K; e0 += nthreads * 8) {
                    uint32_t packed[4];
                    xpro_norm_add8(x, pro, e0, rms, packed);
#pragma unroll
                    for (int i = 0; i < 4; i++) {
                        const float lo = lh_h2f((uint16_t)(packed[i] & 0xFFFF)), hi = lh_h2f((uint16_t)(packed[i] >> 16));
                        s2 += lo * lo;
                        s2 += hi * hi;
                    }
                    if (pro.store != nullptr && blockIdx.x == 0)
                        *reinterpret_cast<uint4*>(pro.store + e0) = make_uint4(packed[0], packed[1], packed[2], packed[3]);
                }
                if (pro.aux2 != nullptr) rms2 = rsqrtf(block_total(s2) / (float)K + pro.eps);
            }
            }
        }
    }
    for (uint32_t base = 0; base < K; base += nthreads * 8) {
        const uint32_t e0 = base + tid * 8;
        const bool valid = e0 < K;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = 0.0f;
        if (valid) {
            if constexpr (sizeof(XT) == 4) {
                const float4 a = *reinterpret_cast<const float4*>(x + e0);
                const float4 b = *reinterpret_cast<const float4*>(x + e0 + 4);
                v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
            } else if (one_round) {
                const uint32_t wg2[4] = {one_g2.x, one_g2.y, one_g2.z, one_g2.w};
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    const float t = lh_h2f((uint16_t)((one_packed[i >> 1] >> (16 * (i & 1))) & 0xFFFF));
                    if (pro.aux2 != nullptr) v[i] = lh_h2f(lh_f2h_exact(lh_norm_product(t, rms2, lh_h2f((uint16_t)((wg2[i >> 1] >> (16 * (i & 1))) & 0xFFFF)))));
                    else v[i] = t;
                }
            } else {
                const uint4 a = *reinterpret_cast<const uint4*>(x + e0);
                const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    v[2 * i] = lh_h2f((uint16_t)(w[i] & 0xFFFF));
                    v[2 * i + 1] = lh_h2f((uint16_t)(w[i] >> 16));
                }
                if (pro.kind == kXProRmsNorm) {
                    uint32_t packed[4];
                    xpro_norm_add8(x, pro, e0, rms, packed);
                    uint4 g2 = make_uint4(0u, 0u, 0u, 0u);
                    if (pro.aux2 != nullptr) g2 = *reinterpret_cast<const uint4*>(pro.aux2 + e0);
                    const uint32_t wg2[4] = {g2.x, g2.y, g2.z, g2.w};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const float t = lh_h2f((uint16_t)((packed[i >> 1] >> (16 * (i & 1))) & 0xFFFF));
                        if (pro.aux2 != nullptr) v[i] = lh_h2f(lh_f2h_exact(lh_norm_product(t, rms2, lh_h2f((uint16_t)((wg2[i >> 1] >> (16 * (i & 1))) & 0xFFFF)))));
                        else v[i] = t;
                    }
                } else if (pro.kind == kXProGeluMul) {
                    const uint4 b = *reinterpret_cast<const uint4*>(pro.aux + e0);
                    const uint32_t wb[4] = {b.x, b.y, b.z, b.w};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        v[i] = lh_h2f(lh_gelu_mul_h((uint16_t)((w[i >> 1] >> (16 * (i & 1))) & 0xFFFF),
                                                    (uint16_t)((wb[i >> 1] >> (16 * (i & 1))) & 0xFFFF)));
                    }
                }
            }
        }
        if constexpr (sizeof(XT) == 4) {
            if (pro.kind == kXProRotate) xpro_rotate8(v, pro, e0);   // uniform over the workgroup
        }
        // the maximum over the bit patterns of |v|: the order of non-negative floats, with NaN and infinity on top
        uint32_t mbits = 0u;
        float asum = 0.0f;                                    // sum of |v| over the block (second-level test)
#pragma unroll
        for (int i = 0; i < 8; i++) { mbits = max(mbits, __builtin_bit_cast(uint32_t, fabsf(v[i]))); asum += fabsf(v[i]); }
        mbits = lh_group_max_u(mbits, G / 8);
        const bool finite = mbits < 0x7F800000u;
        const float m = __builtin_bit_cast(float, mbits);
        const float inv = (finite && m > 0.0f) ? Limb<L>::qmax / m : 0.0f;
        const float sc = finite ? m * (1.0f / Limb<L>::qmax) : __builtin_nanf("");
        uint32_t packed[L][2];
        int nsum = 0;
#pragma unroll
        for (int l = 0; l < L; l++) packed[l][0] = packed[l][1] = 0;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float r = rintf(v[i] * inv);
            r = fminf(fmaxf(r, -Limb<L>::qmax), Limb<L>::qmax);
            int n = (int)r;
            nsum += n;
#pragma unroll
            for (int l = 0; l < L; l++) {
                int limb;
                if (l == L - 1) limb = n;                       // top limb: what is left, fits a signed byte
                else { limb = (int)(int8_t)(n & 0xFF); n = (n - limb) >> 8; }
                packed[l][i >> 2] |= (uint32_t)(limb & 0xFF) << (8 * (i & 3));
            }
        }
        if (valid) {
#pragma unroll
            for (int l = 0; l < L; l++)
                *reinterpret_cast<uint2*>(&xq[l * kq + (e0 >> 2)]) = make_uint2(packed[l][0], packed[l][1]);
            if ((e0 & (G - 1)) == 0) xs[e0 / G] = sc;
        }
        if (xn != nullptr) {
            nsum = lh_group_sum_i(nsum, G / 8);
            if (valid && (e0 & (G - 1)) == 0) xn[e0 / G] = nsum;
        }
        if constexpr (L == 2) {
            if (resid != nullptr) {
                asum = lh_group_sum(asum, G / 8);
                const bool coarse = finite && m * (float)(G - 1) > kXOutlier * (asum - m);   // uniform over the lanes of a group
                const float sc2 = sc * (0.52f / Limb<2>::qmax);       // |r| <= 0.5 sc up to rounding: 0.52 leaves headroom
                int nsum2 = 0;
                if (__builtin_amdgcn_ballot_w64(coarse) != 0) {      // rare: skipped by waves without such a block
                    const float inv2 = coarse ? 1.0f / sc2 : 0.0f;
                    uint32_t p2[2][2] = {{0u, 0u}, {0u, 0u}};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        const float n1 = fminf(fmaxf(rintf(v[i] * inv), -Limb<L>::qmax), Limb<L>::qmax);   // the first level's integer again
                        const float rr = __builtin_fmaf(-n1, sc, v[i]);
                        float q2 = rintf(rr * inv2);
                        q2 = fminf(fmaxf(q2, -Limb<2>::qmax), Limb<2>::qmax);
                        int n2 = (int)q2;
                        nsum2 += n2;
                        const int lo = (int)(int8_t)(n2 & 0xFF);
                        const int hi = (n2 - lo) >> 8;
                        p2[0][i >> 2] |= (uint32_t)(lo & 0xFF) << (8 * (i & 3));
                        p2[1][i >> 2] |= (uint32_t)(hi & 0xFF) << (8 * (i & 3));
                    }
                    if (valid && coarse) {
                        *reinterpret_cast<uint2*>(&resid->xq2[e0 >> 2]) = make_uint2(p2[0][0], p2[0][1]);
                        *reinterpret_cast<uint2*>(&resid->xq2[kq + (e0 >> 2)]) = make_uint2(p2[1][0], p2[1][1]);
                    }
                    if (resid->xn2 != nullptr) nsum2 = lh_group_sum_i(nsum2, G / 8);
                }
                if (valid && (e0 & (G - 1)) == 0) {
                    resid->xs2[e0 / G] = coarse ? sc2 : 0.0f;
                    if (resid->xn2 != nullptr) resid->xn2[e0 / G] = coarse ? nsum2 : 0;
                }
            }
        }
    }
}

