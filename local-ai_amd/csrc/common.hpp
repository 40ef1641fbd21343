// Internal declarations shared by the HIP translation units of liblocal_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <atomic>
#include <vector>
#include "../../include/local_hip.h"

struct lh_context {
    int device;
    hipStream_t stream;
    int cu_count;
    char name[256];
    // Split-K partial results of the attention kernels: (max, sum, acc[head_dim])
    // per (query head, split). Allocated once with the context.
    void* workspace;
    size_t workspace_bytes;
    // The creator's handle plus one per live buffer, batch and event: the stream and the workspace are
    // released when the last of them goes, so handles may be freed in any order.
    std::atomic<int> refs;
    // True between lh_batch_begin_capture and lh_batch_end_capture: dispatches are recorded into a graph instead
    // of running, and calls that would wait, allocate, copy from host memory or record a memset are refused.
    bool capturing;
    // Owning buffers released while a capture is open.  A recorded dispatch may reference them, so they live as long as
    // the graph the capture produces (lh_graph_free releases them); when the capture fails they go when it ends.
    std::vector<void*> deferred_free;
    // Pinned staging for descriptor tables of grouped launches: a small ring of slots, each guarded by an event that is
    // recorded behind the slot's copy, so a slot is rewritten only after the copy that read it has run.
    static constexpr int kDescSlots = 4;
    static constexpr size_t kDescSlotBytes = 64 * 1024;
    void* desc_pinned;
    hipEvent_t desc_event[kDescSlots];
    bool desc_used[kDescSlots];
    unsigned desc_next;
    // One word of pinned host memory that kernels can reach: a kernel that had to give up a bounded wait stores a code
    // here, and the next wait on the stream (lh_batch_commit_and_wait, lh_context_synchronize) reports it.
    uint32_t* fault_host;
    uint32_t* fault_dev;   // the same word as the device addresses it
};
// Kernel-reported fault codes (lh_context::fault_host).
enum : uint32_t { LH_FAULT_TQ2_SPLIT_WAIT = 1, LH_FAULT_ATTN_PAIR_WAIT = 2 };
// Reads and clears the context's fault word after a completed wait; LH_OK when no kernel reported anything.
int lh_check_fault_word(lh_context* ctx);

struct lh_buffer {
    lh_context* ctx;
    void* ptr;
    size_t len;
    bool owns;
    size_t slack;   // readable bytes behind ptr + len (allocation padding, or the rest of a viewed parent)
};

struct lh_batch {
    lh_context* ctx;
    uint32_t dispatch_count;
};

// Records the error text for lh_last_error() and returns `code`.
int lh_fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// Post-launch check: converts a pending HIP launch error into LH_ERR_COMMAND_BUFFER.
int lh_check_launch(const char* what);

#define LH_HIP_TRY(expr, code, what)                                                        \
    do {                                                                                    \
        hipError_t e__ = (expr);                                                            \
        if (e__ != hipSuccess) return lh_fail((code), "%s: %s", (what), hipGetErrorString(e__)); \
    } while (0)

#define LH_REQUIRE(cond, ...)                                            \
    do {                                                                 \
        if (!(cond)) return lh_fail(LH_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
    } while (0)

static inline int lh_need(const lh_buffer* b, size_t bytes, const char* op, const char* name) {
    if (b == nullptr) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: %s buffer is null", op, name);
    if (b->len < bytes)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: %s buffer holds %zu bytes, needs %zu", op, name, b->len, bytes);
    return LH_OK;
}
#define LH_NEED(buf, bytes, op, name)                        \
    do {                                                     \
        int r__ = lh_need((buf), (bytes), (op), (name));     \
        if (r__ != LH_OK) return r__;                        \
    } while (0)

// Optional transform applied to an f16 activation vector while a matvec stages it (saves the dispatch of the kernel
// that would otherwise have produced it): the value that is quantised is the f16 the separate kernel would have stored.
//   kXProRmsNorm: t_i = x_i * rsqrt(mean(x^2) + eps) * aux_i (rms_norm.metal:4-46; aux = norm weight, f16[K]); with
//                 `res` the residual is added before the one rounding (rms_norm.metal:48-88), the workgroup with
//                 blockIdx.x == 0 stores that vector to `store` when given, and with `aux2` the staged vector is the
//                 RMS norm of it with weight aux2 -- post-norm + residual followed by the next pre-norm.
//   kXProGeluMul: gelu_tanh(x_i) * aux_i                 (gelu.metal:23-41; x = gate, aux = up, f16[K])
//   kXProRotate:  x = f32 head outputs in code space, K = heads x head_dim: per head the Walsh-Hadamard transform,
//                 x 1/sqrt(head_dim) (`scale`), x signs[dim], one rounding to f16 (attention_flash_tq.metal:58-90 with the
//                 post-sign, as hadamard_rotate_kernel<float, f16> computes it).
enum : uint32_t { kXProNone = 0, kXProRmsNorm = 1, kXProGeluMul = 2, kXProRotate = 3 };
struct XPrologue {
    uint32_t kind;
    const uint16_t* aux;
    float eps;
    const uint16_t* res = nullptr;
    const uint16_t* aux2 = nullptr;
    uint16_t* store = nullptr;
    uint32_t tail = 0;      // with `res`: 0 the residual joins the f32 product (rms_norm_add); 1, 2 see lh_norm_tail
    float scale = 1.0f;
    const float* signs = nullptr;   // kXProRotate: the codec's sign vector, f32[head_dim]
    uint32_t head_dim = 0;          // kXProRotate: a power of two, 8 .. 512, dividing K
};

// TQ2_0 matvec on the matrix cores (matvec_tq2_mfma.hip). Host arrays of device pointers; shapes validated by the caller.
// With a non-zero stride only entry 0 of the arrays is used: problem i is problem 0 with its matrix / vector / output
// advanced by i * mstride / i * xstride / i * ystride bytes.
int lh_launch_matvec_tq2_mfma(lh_context* ctx, uint32_t count, const void* const* matrices, const void* const* vectors,
                              void* const* outputs, lh_dtype xt, lh_dtype yt, uint32_t rows, uint32_t K, uint32_t xstride,
                              uint32_t ystride, const XPrologue& pro = XPrologue{kXProNone, nullptr, 0.0f}, uint64_t mstride = 0);
// The m rows of a small activation batch against one quantized matrix, as m matvecs in one launch (matvec_quant.hip).
// Returns LH_OK, an error, or -1 when the fast kernels do not take the shape (the caller then uses its own kernel).
int lh_matvec_rows(lh_batch* batch, lh_quant fmt, uint32_t m, const lh_buffer* weight, const lh_buffer* input, lh_dtype at,
                   lh_buffer* output, lh_dtype ct, uint32_t n, uint32_t k, const char* op);

// A row-wise RMS norm whose input is f16 rows (`in`) or the f32 partial tiles of a k-split product (`partial`: split z
// of row r starts at partial[(z * part_rows + r) * part_cols]), with the optional residual, output scale and second
// norm of a decoder layer's tail; defined beside the stand-alone norm kernels, launched by the fused product entry.
struct LhNormFused {
    const uint16_t* in;
    const float* partial;
    uint32_t splits, part_rows, part_cols;
    const uint16_t* w;
    const uint16_t* res;      // null: no residual
    uint16_t* out;
    uint32_t dim, rows;
    float eps;
    uint32_t apply_scale;
    float scale;
    uint32_t tail;            // 0 here: the residual is added in f32 (rms_norm_add); passed through to the shared chunk arithmetic
    const uint16_t* w2;       // null: no second norm
    uint16_t* out2;
};
bool lh_norm_fused_supported(uint32_t dim);
// gelu_mul_strided's 16-byte kernel with the first operand either f16 rows (`a`) or a product's partial tiles (`partial` not
// null); dim, b_row_stride and b_off multiples of 8, pointers 16-byte aligned
void lh_launch_gelu_mul_strided(hipStream_t stream, const void* a, const float* partial, uint32_t splits, uint32_t part_cols, const void* b,
                                uint32_t b_row_stride, uint32_t b_off, void* out, uint32_t dim, uint32_t rows);
void lh_launch_gelu_mul(hipStream_t stream, const void* a, const void* b, void* out, uint32_t count);   // gelu_mul_into's kernel
void lh_launch_norm_fused(hipStream_t stream, const LhNormFused& a);

// The arguments of lh_decode_qkv_prepare_rows_into, and its launch with the heads taken from the f32 partial tiles of a
// k-split product ([splits][rows][part_cols], the query, key and value heads side by side; nullptr: from q / k / v).
// Defined with the kernel (turboquant_kv.hip); the product that leaves its tiles behind calls it (matmul_quant.hip).
// check_only validates the arguments and launches nothing.
struct LhPrepareRows {
    lh_buffer *q, *k, *v;
    const lh_buffer *q_norm, *k_norm, *levels, *signs;
    lh_buffer *rq, *k_codes, *k_norms, *v_codes, *v_norms;
    const lh_buffer* positions;
    uint32_t head_dim, n_q_heads, n_kv_heads, rows;
    float eps;
    uint32_t start_position;
    float theta, partial_rotary_factor;
    uint32_t bits, ring_capacity, lane_capacity;
};
int lh_prepare_rows_launch(lh_batch* batch, const LhPrepareRows& a, const float* partial, uint32_t splits, uint32_t part_cols, bool check_only = false);
int lh_launch_hadamard_fh(lh_context* ctx, const float* input, const float* signs, uint16_t* output, uint32_t head_dim, uint32_t num_heads);

// Stream-ordered copy of a host-built descriptor table to device memory.  The host block may be freed as soon as this
// returns (it has been copied into pinned staging; tables larger than a staging slot are copied synchronously after a
// stream wait).  Not available while a graph is being captured.
int lh_upload_descriptors(lh_context* ctx, const void* host, size_t bytes, void* device_dst, const char* op);

// Raises a kernel's dynamic-LDS limit to `bytes` (hipFuncAttributeMaxDynamicSharedMemorySize), once per kernel and device.
int lh_raise_dynamic_lds(lh_context* ctx, const void* kernel, size_t bytes, const char* op);

// Resolves the calling device's copy of the attention kernels' static scratch array (attention_tq.hip); the device must be current.
int lh_attention_static_scratch_init(int device);
// Raises the dynamic-LDS limit of the attention kernels that need more than the default (attention_tq_mfma.hip); ctx's device must be current.
int lh_attention_kernels_init(lh_context* ctx);

static inline size_t lh_dtype_size(lh_dtype t) { return t == LH_F32 ? 4 : 2; }

// ---- device helpers -------------------------------------------------------
#define LH_DPP_QUAD_XOR1 0xB1   // quad_perm:[1,0,3,2]
#define LH_DPP_QUAD_XOR2 0x4E   // quad_perm:[2,3,0,1]
#define LH_DPP_HALF_MIRROR 0x141
#define LH_DPP_ROW_MIRROR 0x140

template <int CTRL>
__device__ __forceinline__ float lh_dpp_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
template <int CTRL>
__device__ __forceinline__ int lh_dpp_i(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
// Exchange with the lane 16 away (inside each group of 32) and 32 away.
__device__ __forceinline__ float lh_swap16_f(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x1F | (16 << 10)));
}
__device__ __forceinline__ float lh_swap32_f(float v) {
    return __shfl_xor(v, 32, 64);
}

// Sum over aligned groups of `width` lanes (power of two, 1..64); every lane of
// a group ends with the group's total. Fixed pairing order: deterministic.
__device__ __forceinline__ float lh_group_sum(float v, int width) {
    if (width > 1) v += lh_dpp_f<LH_DPP_QUAD_XOR1>(v);
    if (width > 2) v += lh_dpp_f<LH_DPP_QUAD_XOR2>(v);
    if (width > 4) v += lh_dpp_f<LH_DPP_HALF_MIRROR>(v);
    if (width > 8) v += lh_dpp_f<LH_DPP_ROW_MIRROR>(v);
    if (width > 16) v += lh_swap16_f(v);
    if (width > 32) v += lh_swap32_f(v);
    return v;
}
__device__ __forceinline__ float lh_group_max(float v, int width) {
    if (width > 1) v = fmaxf(v, lh_dpp_f<LH_DPP_QUAD_XOR1>(v));
    if (width > 2) v = fmaxf(v, lh_dpp_f<LH_DPP_QUAD_XOR2>(v));
    if (width > 4) v = fmaxf(v, lh_dpp_f<LH_DPP_HALF_MIRROR>(v));
    if (width > 8) v = fmaxf(v, lh_dpp_f<LH_DPP_ROW_MIRROR>(v));
    if (width > 16) v = fmaxf(v, lh_swap16_f(v));
    if (width > 32) v = fmaxf(v, lh_swap32_f(v));
    return v;
}
// Maximum of unsigned values (also of non-negative floats taken as bit patterns) over aligned groups of `width` lanes.
__device__ __forceinline__ uint32_t lh_group_max_u(uint32_t v, int width) {
    if (width > 1) v = max(v, (uint32_t)lh_dpp_i<LH_DPP_QUAD_XOR1>((int)v));
    if (width > 2) v = max(v, (uint32_t)lh_dpp_i<LH_DPP_QUAD_XOR2>((int)v));
    if (width > 4) v = max(v, (uint32_t)lh_dpp_i<LH_DPP_HALF_MIRROR>((int)v));
    if (width > 8) v = max(v, (uint32_t)lh_dpp_i<LH_DPP_ROW_MIRROR>((int)v));
    if (width > 16) v = max(v, (uint32_t)__builtin_amdgcn_ds_swizzle((int)v, 0x1F | (16 << 10)));
    if (width > 32) v = max(v, (uint32_t)__shfl_xor((int)v, 32, 64));
    return v;
}
__device__ __forceinline__ int lh_group_sum_i(int v, int width) {
    if (width > 1) v += lh_dpp_i<LH_DPP_QUAD_XOR1>(v);
    if (width > 2) v += lh_dpp_i<LH_DPP_QUAD_XOR2>(v);
    if (width > 4) v += lh_dpp_i<LH_DPP_HALF_MIRROR>(v);
    if (width > 8) v += lh_dpp_i<LH_DPP_ROW_MIRROR>(v);
    if (width > 16) v += __builtin_amdgcn_ds_swizzle(v, 0x1F | (16 << 10));
    if (width > 32) v += __shfl_xor(v, 32, 64);
    return v;
}

__device__ __forceinline__ float lh_h2f(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }
__device__ __forceinline__ uint16_t lh_f2h(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
// One NEOX pair at `position` (rope.metal:46-58).  The same instruction sequence serves the stand-alone and the fused
// kernel, so that qk_norm + rope and qk_norm_rope agree bit for bit (kernels.rs:7873).
// (In two halves, so that a kernel can evaluate the pair's cosine and sine -- which depend on no data -- while its loads are
// on their way; both halves together are the sequence above.)
__device__ __forceinline__ void lh_rope_cos_sin(uint32_t i, uint32_t head_dim, uint32_t position, float theta, float& c, float& sn) {
    const float freq = 1.0f / powf(theta, (float)(2 * i) / (float)head_dim);
    const float angle = (float)position * freq;
    c = cosf(angle);
    sn = sinf(angle);
}
__device__ __forceinline__ void lh_rope_apply(float x0, float x1, float c, float sn, uint16_t& o0, uint16_t& o1) {
    o0 = lh_f2h(__builtin_fmaf(x0, c, -(x1 * sn)));
    o1 = lh_f2h(__builtin_fmaf(x0, sn, x1 * c));
}
__device__ __forceinline__ void lh_rotate_pair(float x0, float x1, uint32_t i, uint32_t head_dim, uint32_t position, float theta, uint16_t& o0, uint16_t& o1) {
    float c, sn;
    lh_rope_cos_sin(i, head_dim, position, theta, c, sn);
    lh_rope_apply(x0, x1, c, sn, o0, o1);
}
// Narrowing of an already rounded f32 value, as f16::from_f32 does it. The empty asm keeps the
// compiler from folding a preceding multiply into v_fma_mixlo_f16, which rounds the exact
// product once (a different result in double-rounding cases) and turns -0 into +0.
__device__ __forceinline__ uint16_t lh_f2h_exact(float f) { asm volatile("" : "+v"(f)); return lh_f2h(f); }
// x * rms * w of a norm as a rounded f32 value in a register.  Every kernel that evaluates a norm -- stand-alone, as the
// prologue of a product or as its epilogue -- goes through this, so that none of them has the product contracted into a
// following addition or narrowed to f16 in one mixed-precision instruction while another has not (the results then
// differ in the last f16 bit about once in ten thousand values).
__device__ __forceinline__ float lh_norm_product(float x, float rms, float w) {
    float p = x * rms * w;
    asm volatile("" : "+v"(p));
    return p;
}

// The end of a per-layer input block as its three kernels round it (layer.rs:503-520: rms_norm, residual_add,
// scale_in_place): the normalised value is rounded to f16, added to the residual as an f16 addition, and, with tail == 2,
// scaled (the caller rounds once more).
__device__ __forceinline__ float lh_norm_tail(float normed, float res, uint32_t tail, float scale) {
    const _Float16 sum = (_Float16)normed + (_Float16)res;
    return tail == 2 ? (float)sum * scale : (float)sum;
}

// The value of the lane LEN away (lane ^ LEN; LEN a power of two below 64).
template <int LEN>
__device__ __forceinline__ float lh_lane_xor_f(float v) {
    if constexpr (LEN == 1) return lh_dpp_f<LH_DPP_QUAD_XOR1>(v);
    else if constexpr (LEN == 2) return lh_dpp_f<LH_DPP_QUAD_XOR2>(v);
    else if constexpr (LEN <= 16) return __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x1F | (LEN << 10)));
    else return __shfl_xor(v, 32, 64);
}
template <int LEN>
__device__ __forceinline__ float lh_fwht_lane_stage(float v, uint32_t lane) {
    const float other = lh_lane_xor_f<LEN>(v);
    return (lane & LEN) ? __fsub_rn(other, v) : __fadd_rn(v, other);
}

// In-place unnormalised fast Walsh-Hadamard transform over sh[0..d) in LDS with one thread per element (thread `lane`
// has just written sh[lane] itself); every thread of the workgroup calls it.  Sums and differences only, in a fixed order
// (pairs 1 apart first, then 2, 4, ...), so every kernel that uses it produces the same bits.  The stages that pair
// elements of one wave exchange them between lanes; only those 64 and more apart go through LDS and a barrier.
__device__ __forceinline__ void lh_fwht_lds(float* sh, uint32_t d, uint32_t lane) {
    float v = sh[lane];
    if (d > 1) v = lh_fwht_lane_stage<1>(v, lane);
    if (d > 2) v = lh_fwht_lane_stage<2>(v, lane);
    if (d > 4) v = lh_fwht_lane_stage<4>(v, lane);
    if (d > 8) v = lh_fwht_lane_stage<8>(v, lane);
    if (d > 16) v = lh_fwht_lane_stage<16>(v, lane);
    if (d > 32) v = lh_fwht_lane_stage<32>(v, lane);
    for (uint32_t len = 64; len < d; len <<= 1) {
        sh[lane] = v;
        __syncthreads();
        const float other_v = sh[lane ^ len];
        __syncthreads();
        v = (lane & len) ? __fsub_rn(other_v, v) : __fadd_rn(v, other_v);
    }
    sh[lane] = v;
    __syncthreads();
}
__device__ __forceinline__ float lh_bf2f(uint16_t b) { return __builtin_bit_cast(float, (uint32_t)b << 16); }

template <typename T> __device__ __forceinline__ float lh_load_as_f32(const T* p, size_t i);
template <> __device__ __forceinline__ float lh_load_as_f32<float>(const float* p, size_t i) { return p[i]; }
template <> __device__ __forceinline__ float lh_load_as_f32<uint16_t>(const uint16_t* p, size_t i) { return lh_h2f(p[i]); }

template <typename T> __device__ __forceinline__ void lh_store_from_f32(T* p, size_t i, float v);
template <> __device__ __forceinline__ void lh_store_from_f32<float>(float* p, size_t i, float v) { p[i] = v; }
template <> __device__ __forceinline__ void lh_store_from_f32<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = lh_f2h(v); }
