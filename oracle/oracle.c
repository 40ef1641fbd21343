/*
 * CPU oracle for the decode hot path (TEST INFRASTRUCTURE, not product code).
 *
 * A plain-C restatement of the reference's CPU algorithms for quantized-weight
 * dequant / dot products and the TurboQuant KV codec.  Only tests, the smoke
 * check and the benchmark's cpu_baseline leg may load this library; the GPU
 * library never links or calls it.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the reference repository root).  Build with -ffp-contract=off: the reference
 * is Rust, which never fuses a*b+c unless mul_add is written explicitly.
 *
 * Pinning status (what independent evidence fixes each function) is listed in
 * oracle/README.md; the only item that no test can pin without running the
 * reference's own build is the exact bit pattern of the Lloyd-Max levels
 * (depends on the platform libm expf) -- "parity unpinned" for those bits,
 * pinned to ~1e-3 by the textbook 2/3/4-bit Gaussian quantizer tables.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------ f16 -- */
/* IEEE binary16 <-> binary32, round-to-nearest-even, subnormals kept: the
 * semantics of half::f16::{from_f32,to_f32} (crate `half` 2.7.1, not vendored
 * in the reference; call sites local-engine/src/qat_recover.rs:38,46,82,93). */
ORC_API float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int e = -1;
            do { e++; man <<= 1; } while ((man & 0x400u) == 0);
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7F800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f; memcpy(&f, &bits, 4); return f;
}

ORC_API uint16_t orc_f32_to_f16(float f) {
    uint32_t x; memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xFFu;
    uint32_t man = x & 0x7FFFFFu;
    if (exp == 255) { /* inf / nan (keep a quiet payload bit) */
        return (uint16_t)(sign | 0x7C00u | (man ? (0x200u | (man >> 13)) : 0u));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u);          /* overflow -> inf */
    if (e <= 0) {                                             /* subnormal / zero */
        if (e < -10) return (uint16_t)sign;
        man |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);                  /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1u))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half_man = man >> 13;
    uint32_t rem = man & 0x1FFFu;
    uint16_t out = (uint16_t)(sign | ((uint32_t)e << 10) | half_man);
    if (rem > 0x1000u || (rem == 0x1000u && (half_man & 1u))) out++; /* carries into exp correctly */
    return out;
}

ORC_API float orc_bf16_to_f32(uint16_t b) {
    uint32_t bits = (uint32_t)b << 16; float f; memcpy(&f, &bits, 4); return f;
}

ORC_API void orc_f16_to_f32_array(const uint16_t* in, float* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = orc_f16_to_f32(in[i]);
}
ORC_API void orc_f32_to_f16_array(const float* in, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; i++) out[i] = orc_f32_to_f16(in[i]);
}

/* -------------------------------------------------------------- dequant -- */
/* local-engine/src/qat_recover.rs:23-52 dequant_tq2_0_into.
 * 66-byte blocks: 64 bytes qs then f16 d.  Order: for j in {0,32}: for l in
 * 0..4: for m in 0..32: q = (qs[j+m] >> 2l) & 3; out = f16(d * (q - 1)).
 * Returns the number of f16 values written (min(num_elements, blocks*256)). */
ORC_API size_t orc_dequant_tq2_0(const uint8_t* data, size_t nbytes, size_t num_elements, uint16_t* out) {
    size_t blocks = nbytes / 66, n = 0;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t* qs = data + b * 66;
        float d = orc_f16_to_f32((uint16_t)(qs[64] | ((uint16_t)qs[65] << 8)));
        for (int j = 0; j < 64; j += 32)
            for (int l = 0; l < 4; l++)
                for (int m = 0; m < 32; m++) {
                    if (n >= num_elements) return n;
                    uint8_t q = (uint8_t)((qs[j + m] >> (l * 2)) & 3);
                    out[n++] = orc_f32_to_f16(d * ((float)q - 1.0f));
                }
    }
    return n;
}

/* local-engine/src/qat_recover.rs:64-97 dequant_q4_0_into.
 * 18-byte blocks: f16 d then 16 bytes; byte j holds element j (low nibble) and
 * j+16 (high nibble); value = f16((nibble - 8) * d). */
ORC_API size_t orc_dequant_q4_0(const uint8_t* data, size_t nbytes, size_t num_elements, uint16_t* out) {
    size_t blocks = nbytes / 18, n = 0;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t* p = data + b * 18;
        float d = orc_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
        float block[32];
        for (int j = 0; j < 16; j++) {
            uint8_t q = p[2 + j];
            block[j] = ((float)(q & 0x0F) - 8.0f) * d;
            block[j + 16] = ((float)(q >> 4) - 8.0f) * d;
        }
        for (int j = 0; j < 32; j++) {
            if (n >= num_elements) return n;
            out[n++] = orc_f32_to_f16(block[j]);
        }
    }
    return n;
}

/* local-engine/src/qat_recover.rs:108-134 dequant_q8_0_into (34-byte blocks). */
ORC_API size_t orc_dequant_q8_0(const uint8_t* data, size_t nbytes, size_t num_elements, uint16_t* out) {
    size_t blocks = nbytes / 34, n = 0;
    for (size_t b = 0; b < blocks; b++) {
        const uint8_t* p = data + b * 34;
        float d = orc_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
        for (int j = 0; j < 32; j++) {
            if (n >= num_elements) return n;
            out[n++] = orc_f32_to_f16((float)(int8_t)p[2 + j] * d);
        }
    }
    return n;
}

/* Unrounded f32 expansion used by the reference's GPU-kernel tests:
 * local-metal/src/kernels.rs:8790-8810 (q4_0_payload dq) and 8814-8841
 * (tq2_0_payload dq): (q-8)*d and (q-1)*d kept in f32. */
ORC_API void orc_expand_q4_0_f32(const uint8_t* data, size_t rows, size_t cols, float* dq) {
    size_t nb = cols / 32;
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < nb; b++) {
            const uint8_t* p = data + (r * nb + b) * 18;
            float d = orc_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
            for (int i = 0; i < 16; i++) {
                uint8_t q = p[2 + i];
                dq[r * cols + b * 32 + i] = ((float)(q & 0x0F) - 8.0f) * d;
                dq[r * cols + b * 32 + 16 + i] = ((float)(q >> 4) - 8.0f) * d;
            }
        }
}
ORC_API void orc_expand_tq2_0_f32(const uint8_t* data, size_t rows, size_t cols, float* dq) {
    size_t nb = cols / 256;
    for (size_t r = 0; r < rows; r++)
        for (size_t b = 0; b < nb; b++) {
            const uint8_t* qs = data + (r * nb + b) * 66;
            float d = orc_f16_to_f32((uint16_t)(qs[64] | ((uint16_t)qs[65] << 8)));
            for (int j = 0; j < 64; j++) {
                size_t base = b * 256 + (size_t)(j >> 5) * 128 + (size_t)(j & 31);
                for (int l = 0; l < 4; l++)
                    dq[r * cols + base + (size_t)l * 32] = ((float)((qs[j] >> (2 * l)) & 3) - 1.0f) * d;
            }
        }
}

/* ------------------------------------------------------------------ dot -- */
/* local-metal/src/kernels.rs:8865-8869 cpu_matvec: per row a left-to-right
 * f32 fold of separately rounded products. */
ORC_API void orc_matvec_f32(const float* dq, const float* v, size_t rows, size_t cols, float* y) {
    for (size_t r = 0; r < rows; r++) {
        float s = 0.0f;
        const float* w = dq + r * cols;
        for (size_t c = 0; c < cols; c++) s += w[c] * v[c];
        y[r] = s;
    }
}
/* f64-accumulated variant, for attributing tolerance. */
ORC_API void orc_matvec_f64(const float* dq, const float* v, size_t rows, size_t cols, double* y) {
    for (size_t r = 0; r < rows; r++) {
        double s = 0.0;
        const float* w = dq + r * cols;
        for (size_t c = 0; c < cols; c++) s += (double)w[c] * (double)v[c];
        y[r] = s;
    }
}
/* local-metal/src/kernels.rs:9536-9544 cpu_matmul_nt: C[M,N] = A[M,K] . W[N,K]^T. */
ORC_API void orc_matmul_nt_f32(const float* a, const float* dq, size_t m, size_t k, size_t n, float* c) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            float s = 0.0f;
            for (size_t p = 0; p < k; p++) s += a[i * k + p] * dq[j * k + p];
            c[i * n + j] = s;
        }
}

/* The reference CPU path for one quantized matvec as it would run it: block
 * dequant to f16 (qat_recover.rs:23-97), widen, sequential f32 dot
 * (kernels.rs:8865-8869).  fmt: 0 = Q4_0, 1 = TQ2_0.  `threads` > 1 splits
 * rows over OpenMP threads (row results are unchanged by the split). */
ORC_API void orc_matvec_quant_ref(int fmt, const uint8_t* data, const float* x, size_t rows, size_t cols,
                                  float* y, int threads) {
    size_t bpr = fmt == 0 ? (cols / 32) * 18 : (cols / 256) * 66;
#ifdef _OPENMP
    if (threads < 1) threads = 1;
#pragma omp parallel num_threads(threads)
#endif
    {
        uint16_t* h = (uint16_t*)malloc(cols * sizeof(uint16_t));
#ifdef _OPENMP
#pragma omp for schedule(static)
#endif
        for (size_t r = 0; r < rows; r++) {
            if (fmt == 0) orc_dequant_q4_0(data + r * bpr, bpr, cols, h);
            else orc_dequant_tq2_0(data + r * bpr, bpr, cols, h);
            float s = 0.0f;
            for (size_t c = 0; c < cols; c++) s += orc_f16_to_f32(h[c]) * x[c];
            y[r] = s;
        }
        free(h);
    }
    (void)threads;
}

/* ----------------------------------------------------------- TurboQuant -- */
/* local-engine/src/turboquant.rs:30-51 fwht_normalized. */
static void fwht_butterflies(float* v, size_t n) {
    for (size_t len = 1; len < n; len <<= 1)
        for (size_t i = 0; i < n; i += len << 1)
            for (size_t j = i; j < i + len; j++) {
                float a = v[j], b = v[j + len];
                v[j] = a + b;
                v[j + len] = a - b;
            }
}
ORC_API void orc_fwht_normalized(float* v, size_t n) {
    fwht_butterflies(v, n);
    float inv = 1.0f / sqrtf((float)n);
    for (size_t i = 0; i < n; i++) v[i] *= inv;
}

/* local-engine/src/turboquant.rs:66-79 Rotation::new: splitmix64 from
 * state = seed | 1; sign +1 when the low bit of the mixed word is 0. */
ORC_API void orc_rotation_signs(size_t dim, uint64_t seed, float* signs) {
    uint64_t state = seed | 1u;
    for (size_t i = 0; i < dim; i++) {
        state += 0x9E3779B97F4A7C15ull;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        signs[i] = (z & 1u) == 0 ? 1.0f : -1.0f;
    }
}

static int cmp_float(const void* a, const void* b) {
    float x = *(const float*)a, y = *(const float*)b;
    return (x > y) - (x < y);
}

/* local-engine/src/turboquant.rs:114-166 lloyd_max_gaussian: 8192-point
 * midpoint grid on [-6,6], 100 Lloyd iterations, all in f32 with the same
 * operation order (mul_add -> fmaf). Writes 2^bits increasing levels. */
ORC_API void orc_lloyd_max_gaussian(unsigned bits, float* levels) {
    enum { N = 8192 };
    const float LO = -6.0f, HI = 6.0f;
    const float FRAC_1_SQRT_2 = 0.707106781186547524400844362104849039f;
    const float FRAC_2_SQRT_PI = 1.12837916709551257389615890312154517f;
    size_t k = (size_t)1 << bits;
    float dx = (HI - LO) / (float)N;
    float* xs = (float*)malloc(N * sizeof(float));
    float* pdf = (float*)malloc(N * sizeof(float));
    for (int i = 0; i < N; i++) xs[i] = fmaf((float)i + 0.5f, dx, LO);
    for (int i = 0; i < N; i++) {
        float x = xs[i];
        pdf[i] = expf(-0.5f * x * x) * FRAC_1_SQRT_2 * FRAC_2_SQRT_PI / 2.0f;
    }
    for (size_t i = 0; i < k; i++) {
        float t = ((float)i + 0.5f) / (float)k;
        levels[i] = 6.0f * (t - 0.5f);
    }
    float sum[16], wsum[16];
    for (int it = 0; it < 100; it++) {
        for (size_t j = 0; j < k; j++) { sum[j] = 0.0f; wsum[j] = 0.0f; }
        for (int i = 0; i < N; i++) {
            float x = xs[i], w = pdf[i];
            size_t best = 0; float bd = INFINITY;
            for (size_t j = 0; j < k; j++) {
                float d = fabsf(x - levels[j]);
                if (d < bd) { bd = d; best = j; }
            }
            sum[best] = fmaf(w, x, sum[best]);
            wsum[best] += w;
        }
        for (size_t j = 0; j < k; j++)
            if (wsum[j] > 1e-12f) levels[j] = sum[j] / wsum[j];
    }
    qsort(levels, k, sizeof(float), cmp_float);
    free(xs); free(pdf);
}

/* local-engine/src/turboquant.rs:187-192 TurboQuant::new: levels scaled by
 * 1/sqrt(dim). */
ORC_API void orc_tq_levels(size_t dim, unsigned bits, float* levels) {
    orc_lloyd_max_gaussian(bits, levels);
    float scale = 1.0f / sqrtf((float)dim);
    for (size_t i = 0; i < ((size_t)1 << bits); i++) levels[i] = levels[i] * scale;
}

ORC_API size_t orc_tq_code_bytes(size_t dim, unsigned bits) { /* turboquant.rs:202-204 */
    return (dim * bits + 7) / 8;
}

static uint32_t nearest_level(const float* levels, size_t k, float v) { /* turboquant.rs:293-304 */
    uint32_t best = 0; float bd = INFINITY;
    for (size_t i = 0; i < k; i++) {
        float d = fabsf(v - levels[i]);
        if (d < bd) { bd = d; best = (uint32_t)i; }
    }
    return best;
}

/* local-engine/src/turboquant.rs:241-276 encode_into.  x: dim f32; writes
 * code_bytes packed codes (LSB first) and returns the f16 norm bits.
 * `rotated` (dim floats) receives the rotated, normalised coordinates. */
ORC_API uint16_t orc_tq_encode(const float* x, size_t dim, unsigned bits, const float* signs,
                               const float* levels, float* rotated, uint8_t* codes) {
    float sq = 0.0f;
    for (size_t i = 0; i < dim; i++) sq += x[i] * x[i];
    float norm = sqrtf(sq);
    for (size_t i = 0; i < dim; i++) rotated[i] = x[i];
    if (norm > 0.0f) {
        float inv = 1.0f / norm;
        for (size_t i = 0; i < dim; i++) rotated[i] *= inv;
    }
    for (size_t i = 0; i < dim; i++) rotated[i] *= signs[i];      /* Rotation::apply, turboquant.rs:94-99 */
    orc_fwht_normalized(rotated, dim);
    size_t cb = orc_tq_code_bytes(dim, bits);
    memset(codes, 0, cb);
    uint32_t acc = 0, nbits = 0; size_t idx = 0;
    for (size_t i = 0; i < dim; i++) {
        acc |= nearest_level(levels, (size_t)1 << bits, rotated[i]) << nbits;
        nbits += bits;
        while (nbits >= 8) { codes[idx++] = (uint8_t)(acc & 0xFF); acc >>= 8; nbits -= 8; }
    }
    if (nbits > 0) codes[idx] = (uint8_t)(acc & 0xFF);
    return orc_f32_to_f16(norm);
}

/* LSB-first code read, local-engine/src/turboquant.rs:308-337 BitReader /
 * shaders/attention_flash_tq.metal:33-47 tq_unpack_code. */
static inline uint32_t unpack_code(const uint8_t* codes, size_t d, unsigned bits) {
    size_t bit_off = d * bits;
    size_t byte = bit_off >> 3; unsigned shift = (unsigned)(bit_off & 7);
    uint32_t v = codes[byte];
    if (shift + bits > 8) v |= (uint32_t)codes[byte + 1] << 8;
    return (v >> shift) & ((1u << bits) - 1u);
}

/* local-engine/src/turboquant.rs:280-291 decode: levels[code] -> FWHT ->
 * 1/sqrt(n) -> sign -> * f32(norm). */
ORC_API void orc_tq_decode(const uint8_t* codes, uint16_t norm, size_t dim, unsigned bits,
                           const float* signs, const float* levels, float* out) {
    for (size_t i = 0; i < dim; i++) out[i] = levels[unpack_code(codes, i, bits)];
    orc_fwht_normalized(out, dim);                                  /* Rotation::apply_inverse, 102-108 */
    for (size_t i = 0; i < dim; i++) out[i] *= signs[i];
    float r = orc_f16_to_f32(norm);
    for (size_t i = 0; i < dim; i++) out[i] *= r;
}

/* local-engine/src/kv_cache/quant_cache.rs:449-476 write_kv (one of K or V)
 * for `num_tokens` consecutive positions starting at `position`: input
 * [num_tokens, n_kv, dim] f16; slot = (pos % ring or pos) * n_kv + head
 * (quant_cache.rs:266-274). */
ORC_API void orc_tq_write_kv(const uint16_t* input, size_t num_tokens, size_t n_kv, size_t dim, unsigned bits,
                             const float* signs, const float* levels, size_t position, size_t ring_capacity,
                             uint8_t* packed, uint16_t* norms) {
    size_t cb = orc_tq_code_bytes(dim, bits);
    float* x = (float*)malloc(dim * sizeof(float));
    float* rot = (float*)malloc(dim * sizeof(float));
    for (size_t t = 0; t < num_tokens; t++) {
        size_t pos = position + t;
        size_t slot = ring_capacity ? pos % ring_capacity : pos;
        for (size_t h = 0; h < n_kv; h++) {
            const uint16_t* src = input + (t * n_kv + h) * dim;
            for (size_t i = 0; i < dim; i++) x[i] = orc_f16_to_f32(src[i]);   /* quantize_head, 115-125 */
            size_t g = slot * n_kv + h;
            norms[g] = orc_tq_encode(x, dim, bits, signs, levels, rot, packed + g * cb);
        }
    }
    free(x); free(rot);
}

/* shaders/attention_flash_tq.metal:58-90 hadamard_rotate_impl semantics on
 * f32: optional pre-sign, unnormalised butterflies, * 1/sqrt(d), optional
 * post-sign. (The CPU twin is Rotation::apply / apply_inverse,
 * turboquant.rs:94-108.) */
ORC_API void orc_hadamard_rotate(const float* in, const float* signs, float* out, size_t head_dim,
                                 size_t num_heads, int pre_sign, int post_sign) {
    float inv = 1.0f / sqrtf((float)head_dim);
    for (size_t h = 0; h < num_heads; h++) {
        float* o = out + h * head_dim;
        for (size_t i = 0; i < head_dim; i++) {
            float x = in[h * head_dim + i];
            o[i] = pre_sign ? x * signs[i] : x;
        }
        fwht_butterflies(o, head_dim);
        for (size_t i = 0; i < head_dim; i++) {
            float y = o[i] * inv;
            if (post_sign) y *= signs[i];
            o[i] = y;
        }
    }
}

/* Attention range semantics shared by every TQ attention kernel,
 * shaders/attention_flash_tq.metal:175-178. */
static void attn_range(size_t kv_len, size_t current_pos, size_t window, size_t* lo, size_t* hi) {
    size_t seq_len = kv_len < current_pos + 1 ? kv_len : current_pos + 1;
    size_t win_start = (window > 0 && current_pos + 1 > window) ? current_pos + 1 - window : 0;
    *lo = win_start; *hi = seq_len;
}

/* Code-space attention, the mathematics of flash_attention_tq
 * (shaders/attention_flash_tq.metal:154-274) evaluated in f64 with a two-pass
 * softmax: logit_t = f32(norm_k[t]) * sum_i rq_i*levels[Kcode_{t,i}] (no
 * 1/sqrt(d) scale), out_i = sum_t p_t * f32(norm_v[t]) * levels[Vcode_{t,i}],
 * rotated space, normalised; empty range -> zeros.  `lane_base` is the first
 * physical token of the lane's region (0 for the single-sequence cache;
 * lane*lane_capacity for the by-lane pool, attention_flash_tq.metal:606,632). */
ORC_API void orc_attention_tq_codespace(const float* rq, const uint8_t* k_codes, const uint16_t* k_norms,
                                        const uint8_t* v_codes, const uint16_t* v_norms, const float* levels,
                                        float* out, size_t head_dim, size_t kv_len, size_t current_pos,
                                        size_t num_q_heads, size_t num_kv_heads, size_t window, unsigned bits,
                                        size_t ring_capacity, size_t lane_base) {
    size_t cb = orc_tq_code_bytes(head_dim, bits), lo, hi;
    attn_range(kv_len, current_pos, window, &lo, &hi);
    size_t n = hi > lo ? hi - lo : 0;
    double* logit = (double*)malloc((n ? n : 1) * sizeof(double));
    double* acc = (double*)malloc(head_dim * sizeof(double));
    for (size_t h = 0; h < num_q_heads; h++) {
        size_t kvh = h / (num_q_heads / num_kv_heads);
        const float* q = rq + h * head_dim;
        double mx = -INFINITY;
        for (size_t t = lo; t < hi; t++) {
            size_t pt = ring_capacity ? t % ring_capacity : t;
            size_t slot = (lane_base + pt) * num_kv_heads + kvh;
            const uint8_t* c = k_codes + slot * cb;
            double dot = 0.0;
            for (size_t i = 0; i < head_dim; i++) dot += (double)q[i] * (double)levels[unpack_code(c, i, bits)];
            dot *= (double)orc_f16_to_f32(k_norms[slot]);
            logit[t - lo] = dot;
            if (dot > mx) mx = dot;
        }
        double sum = 0.0;
        for (size_t i = 0; i < head_dim; i++) acc[i] = 0.0;
        for (size_t t = lo; t < hi; t++) {
            size_t pt = ring_capacity ? t % ring_capacity : t;
            size_t slot = (lane_base + pt) * num_kv_heads + kvh;
            const uint8_t* c = v_codes + slot * cb;
            double w = exp(logit[t - lo] - mx);
            sum += w;
            double wn = w * (double)orc_f16_to_f32(v_norms[slot]);
            for (size_t i = 0; i < head_dim; i++) acc[i] += wn * (double)levels[unpack_code(c, i, bits)];
        }
        double inv = sum > 0.0 ? 1.0 / sum : 0.0;
        for (size_t i = 0; i < head_dim; i++) out[h * head_dim + i] = (float)(acc[i] * inv);
    }
    free(logit); free(acc);
}

/* The reference CPU attention path as it would run it: TurboQuant::decode of
 * every cached K/V vector (turboquant.rs:280-291) followed by the f32
 * attention of local-metal/src/kernels.rs:8497-8528 (scale 1.0: scores,
 * max, exp, sum, weighted V), on the un-rotated query q (f32).  Output is in
 * the original (un-rotated) space.  threads > 1 splits the decode and the
 * score pass over positions; the final sums stay sequential per head. */
ORC_API void orc_attention_tq_decode_then_attend(const float* q, const uint8_t* k_codes, const uint16_t* k_norms,
                                                 const uint8_t* v_codes, const uint16_t* v_norms,
                                                 const float* levels, const float* signs, float* out,
                                                 size_t head_dim, size_t kv_len, size_t current_pos,
                                                 size_t num_q_heads, size_t num_kv_heads, size_t window,
                                                 unsigned bits, size_t ring_capacity, int threads) {
    size_t cb = orc_tq_code_bytes(head_dim, bits), lo, hi;
    attn_range(kv_len, current_pos, window, &lo, &hi);
    size_t n = hi > lo ? hi - lo : 0;
    size_t nkv = num_kv_heads, hd = head_dim;
    float* kd = (float*)malloc((n ? n : 1) * nkv * hd * sizeof(float));
    float* vd = (float*)malloc((n ? n : 1) * nkv * hd * sizeof(float));
    if (threads < 1) threads = 1;
#pragma omp parallel for schedule(static) num_threads(threads)
    for (size_t t = lo; t < hi; t++) {
        size_t pt = ring_capacity ? t % ring_capacity : t;
        for (size_t g = 0; g < nkv; g++) {
            size_t slot = pt * nkv + g;
            orc_tq_decode(k_codes + slot * cb, k_norms[slot], hd, bits, signs, levels, kd + ((t - lo) * nkv + g) * hd);
            orc_tq_decode(v_codes + slot * cb, v_norms[slot], hd, bits, signs, levels, vd + ((t - lo) * nkv + g) * hd);
        }
    }
    float* scores = (float*)malloc((n ? n : 1) * sizeof(float));
    for (size_t h = 0; h < num_q_heads; h++) {
        size_t kvh = h / (num_q_heads / num_kv_heads);
#pragma omp parallel for schedule(static) num_threads(threads)
        for (size_t t = 0; t < n; t++) {
            const float* kk = kd + (t * nkv + kvh) * hd;
            float s = 0.0f;
            for (size_t d = 0; d < hd; d++) s += q[h * hd + d] * kk[d];
            scores[t] = s;
        }
        float mx = -INFINITY;
        for (size_t t = 0; t < n; t++) mx = fmaxf(mx, scores[t]);
        float sum = 0.0f;
        for (size_t t = 0; t < n; t++) { scores[t] = expf(scores[t] - mx); sum += scores[t]; }
        for (size_t d = 0; d < hd; d++) out[h * hd + d] = 0.0f;
        for (size_t t = 0; t < n; t++) {
            float w = scores[t] / sum;
            const float* vv = vd + (t * nkv + kvh) * hd;
            for (size_t d = 0; d < hd; d++) out[h * hd + d] += w * vv[d];
        }
    }
    free(kd); free(vd); free(scores);
}

/* FP16-KV attention, local-metal/src/kernels.rs:8497-8528 (scale 1.0), f64
 * accumulation: the checker for the FP16 flash-decoding kernels. */
ORC_API void orc_attention_f16(const uint16_t* q, const uint16_t* k, const uint16_t* v, float* out,
                               size_t head_dim, size_t kv_len, size_t current_pos, size_t num_q_heads,
                               size_t num_kv_heads, size_t window) {
    size_t lo, hi; attn_range(kv_len, current_pos, window, &lo, &hi);
    size_t n = hi > lo ? hi - lo : 0, hd = head_dim, nkv = num_kv_heads;
    double* sc = (double*)malloc((n ? n : 1) * sizeof(double));
    for (size_t h = 0; h < num_q_heads; h++) {
        size_t kvh = h / (num_q_heads / nkv);
        double mx = -INFINITY;
        for (size_t t = lo; t < hi; t++) {
            double s = 0.0;
            for (size_t d = 0; d < hd; d++)
                s += (double)orc_f16_to_f32(q[h * hd + d]) * (double)orc_f16_to_f32(k[(t * nkv + kvh) * hd + d]);
            sc[t - lo] = s; if (s > mx) mx = s;
        }
        double sum = 0.0;
        for (size_t t = 0; t < n; t++) { sc[t] = exp(sc[t] - mx); sum += sc[t]; }
        for (size_t d = 0; d < hd; d++) {
            double a = 0.0;
            for (size_t t = lo; t < hi; t++) a += sc[t - lo] * (double)orc_f16_to_f32(v[(t * nkv + kvh) * hd + d]);
            out[h * hd + d] = n ? (float)(a / sum) : 0.0f;
        }
    }
    free(sc);
}

/* shaders/tq2_dequant.metal:4-16 legacy unpack: out[i] = f16(f32(scale[i/4]) *
 * ((packed[i/4] >> 2*(i%4)) & 3)) -- no zero point, scale indexed per byte. */
ORC_API void orc_tq2_dequant_legacy(const uint8_t* packed, const uint16_t* scales, uint16_t* out, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float s = orc_f16_to_f32(scales[i / 4]);
        uint32_t code = (packed[i / 4] >> (2 * (i % 4))) & 3u;
        out[i] = orc_f32_to_f16(s * (float)code);
    }
}

/* shaders/matmul_f16.metal:74-114 matmul_f16_nt: C[M,N] = A[M,K] . B[N,K]^T,
 * f16 operands, fp32 accumulate (checker: f64 accumulate). */
ORC_API void orc_matmul_f16_nt(const uint16_t* a, const uint16_t* b, float* c, size_t m, size_t k, size_t n) {
#pragma omp parallel for schedule(static)
    for (size_t i = 0; i < m; i++)
        for (size_t j = 0; j < n; j++) {
            double s = 0.0;
            for (size_t p = 0; p < k; p++) s += (double)orc_f16_to_f32(a[i * k + p]) * (double)orc_f16_to_f32(b[j * k + p]);
            c[i * n + j] = (float)s;
        }
}

/* local-engine/src/kv_cache/quant_cache.rs:48-54 swa_ring_capacity. */
ORC_API size_t orc_swa_ring_capacity(size_t window, size_t max_positions) {
    size_t min_safe = window + 256 - 1;
    size_t v = window * 2 > min_safe ? window * 2 : min_safe;
    size_t p = 1; while (p < v) p <<= 1;
    return p < max_positions ? p : max_positions;
}

ORC_API int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
