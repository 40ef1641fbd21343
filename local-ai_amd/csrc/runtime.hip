// Context, buffer and command-batch plumbing of the C ABI: the HIP stand-ins for
// local-metal/src/{context.rs, buffer.rs, batch.rs, error.rs}.
#include "common.hpp"
#include <cmath>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

static thread_local char g_last_error[512] = "";

// Plain device-to-device copy used by lh_batch_blit_copy: 16 bytes per lane when both
// ends are 16-byte aligned, single bytes otherwise.
__global__ __launch_bounds__(256) void blit_copy16_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, size_t n16) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}
__global__ __launch_bounds__(256) void blit_copy1_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, size_t n) {
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

static const char* status_prefix(int code) {
    switch (code) {  // Display strings of local_metal::Error (error.rs:1-32)
        case LH_ERR_NO_DEVICE: return "No Metal device found";
        case LH_ERR_NO_COMMAND_QUEUE: return "Failed to create command queue";
        case LH_ERR_BUFFER_ALLOCATION: return "Buffer allocation failed";
        case LH_ERR_LIBRARY_CREATION: return "Failed to create Metal library: ";
        case LH_ERR_PIPELINE_CREATION: return "Failed to create pipeline state: ";
        case LH_ERR_SHADER_NOT_FOUND: return "Shader function not found: ";
        case LH_ERR_COMMAND_BUFFER: return "Command buffer error: ";
        case LH_ERR_INVALID_ARGUMENT: return "Invalid argument: ";
        case LH_ERR_IO: return "I/O error: ";
        default: return "";
    }
}

int lh_fail(int code, const char* fmt, ...) {
    char msg[384];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(msg, sizeof msg, fmt, ap);
    va_end(ap);
    if (code == LH_ERR_NO_DEVICE) snprintf(g_last_error, sizeof g_last_error, "No HIP device found (%s)", msg);
    else if (code == LH_ERR_BUFFER_ALLOCATION) snprintf(g_last_error, sizeof g_last_error, "%s (%s)", status_prefix(code), msg);
    else snprintf(g_last_error, sizeof g_last_error, "%s%s", status_prefix(code), msg);
    return code;
}

int lh_check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: %s launch failed: %s", what, hipGetErrorString(e));
    return LH_OK;
}

// hipFuncSetAttribute is per device: remember (kernel, device) pairs already raised.  One owner thread per context, but
// contexts on different threads may race here, hence the lock.
int lh_raise_dynamic_lds(lh_context* ctx, const void* kernel, size_t bytes, const char* op) {
    struct Raised { const void* fn; int device; size_t bytes; };
    static std::mutex mu;
    static std::vector<Raised> done;
    std::lock_guard<std::mutex> lock(mu);
    for (const Raised& r : done)
        if (r.fn == kernel && r.device == ctx->device && r.bytes >= bytes) return LH_OK;
    hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
    if (e != hipSuccess) return lh_fail(LH_ERR_PIPELINE_CREATION, "%s: %s", op, hipGetErrorString(e));
    done.push_back(Raised{kernel, ctx->device, bytes});
    return LH_OK;
}

int lh_upload_descriptors(lh_context* ctx, const void* host, size_t bytes, void* device_dst, const char* op) {
    if (ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "%s: a descriptor upload cannot be recorded into a graph", op);
    if (bytes == 0) return LH_OK;
    hipError_t e;
    if (bytes <= lh_context::kDescSlotBytes) {
        const unsigned slot = ctx->desc_next++ % lh_context::kDescSlots;
        if (ctx->desc_used[slot]) {   // the copy that last read this slot must have run (it has, but for a very deep queue)
            e = hipEventSynchronize(ctx->desc_event[slot]);
            if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: %s: descriptor staging: %s", op, hipGetErrorString(e));
        }
        void* stage = static_cast<char*>(ctx->desc_pinned) + (size_t)slot * lh_context::kDescSlotBytes;
        memcpy(stage, host, bytes);
        e = hipMemcpyAsync(device_dst, stage, bytes, hipMemcpyHostToDevice, ctx->stream);
        if (e == hipSuccess) e = hipEventRecord(ctx->desc_event[slot], ctx->stream);
        ctx->desc_used[slot] = true;
    } else {   // larger than a slot: wait for the kernels that still read the previous table, then a blocking copy
        e = hipStreamSynchronize(ctx->stream);
        if (e == hipSuccess) e = hipMemcpy(device_dst, host, bytes, hipMemcpyHostToDevice);
    }
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: %s: descriptor upload: %s", op, hipGetErrorString(e));
    return LH_OK;
}

int lh_check_fault_word(lh_context* ctx) {
    volatile uint32_t* w = ctx->fault_host;
    const uint32_t code = w ? *w : 0u;
    if (code == 0) return LH_OK;
    *w = 0;
    if (code == LH_FAULT_TQ2_SPLIT_WAIT)
        return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: matvec_tq2_0: a wave gave up waiting for the partial rows of its tile; "
                                              "the outputs of this batch are not valid");
    if (code == LH_FAULT_ATTN_PAIR_WAIT)
        return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: flash_attention_tq: a wave gave up waiting for its partner at a hand-over; "
                                              "the outputs of this batch are not valid");
    return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: a kernel reported fault code %u", code);
}

extern "C" {

const char* lh_last_error(void) { return g_last_error; }
const char* lh_version(void) { return "local-hip 0.1 (gfx950)"; }

static void ctx_retain(lh_context* ctx) { ctx->refs.fetch_add(1, std::memory_order_relaxed); }

static void ctx_release(lh_context* ctx) {
    if (ctx->refs.fetch_sub(1, std::memory_order_acq_rel) != 1) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    (void)hipFree(ctx->workspace);
    for (int i = 0; i < lh_context::kDescSlots; i++) (void)hipEventDestroy(ctx->desc_event[i]);
    (void)hipHostFree(ctx->desc_pinned);
    (void)hipHostFree(ctx->fault_host);
    (void)hipStreamDestroy(ctx->stream);
    delete ctx;
}

void lh_context_destroy(lh_context* ctx);

int lh_context_create(int device_index, lh_context** out) {
    if (!out) return lh_fail(LH_ERR_INVALID_ARGUMENT, "context_create: out is null");
    *out = nullptr;
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess || n <= 0) return lh_fail(LH_ERR_NO_DEVICE, "hipGetDeviceCount found none");
    if (device_index < 0 || device_index >= n) return lh_fail(LH_ERR_NO_DEVICE, "device index %d of %d", device_index, n);
    LH_HIP_TRY(hipSetDevice(device_index), LH_ERR_NO_DEVICE, "hipSetDevice");
    hipDeviceProp_t prop;
    LH_HIP_TRY(hipGetDeviceProperties(&prop, device_index), LH_ERR_NO_DEVICE, "hipGetDeviceProperties");
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return lh_fail(LH_ERR_LIBRARY_CREATION, "kernels are built for gfx950 only, device is %s", prop.gcnArchName);
    {
        const int rs = lh_attention_static_scratch_init(device_index);
        if (rs != LH_OK) return rs;
    }
    lh_context* ctx = new (std::nothrow) lh_context();
    if (!ctx) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", sizeof(lh_context));
    ctx->device = device_index;
    ctx->refs.store(1, std::memory_order_relaxed);
    ctx->capturing = false;
    ctx->desc_pinned = nullptr;
    ctx->desc_next = 0;
    ctx->cu_count = prop.multiProcessorCount;
    snprintf(ctx->name, sizeof ctx->name, "%s (%s)", prop.name, prop.gcnArchName);
    if (hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking) != hipSuccess) {
        delete ctx;
        return lh_fail(LH_ERR_NO_COMMAND_QUEUE, "hipStreamCreate");
    }
    ctx->workspace_bytes = (size_t)128 << 20;
    if (hipMalloc(&ctx->workspace, ctx->workspace_bytes) != hipSuccess) {
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: attention workspace", ctx->workspace_bytes);
    }
    if (hipHostMalloc(&ctx->desc_pinned, lh_context::kDescSlots * lh_context::kDescSlotBytes, hipHostMallocDefault) != hipSuccess) {
        (void)hipFree(ctx->workspace);
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: pinned descriptor staging", lh_context::kDescSlots * lh_context::kDescSlotBytes);
    }
    ctx->fault_host = nullptr;
    ctx->fault_dev = nullptr;
    if (hipHostMalloc((void**)&ctx->fault_host, 64, hipHostMallocDefault) != hipSuccess ||
        hipHostGetDevicePointer((void**)&ctx->fault_dev, ctx->fault_host, 0) != hipSuccess) {
        if (ctx->fault_host) (void)hipHostFree(ctx->fault_host);
        (void)hipHostFree(ctx->desc_pinned);
        (void)hipFree(ctx->workspace);
        (void)hipStreamDestroy(ctx->stream);
        delete ctx;
        return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: pinned fault word", (size_t)64);
    }
    *ctx->fault_host = 0;
    for (int i = 0; i < lh_context::kDescSlots; i++) {
        ctx->desc_used[i] = false;
        if (hipEventCreateWithFlags(&ctx->desc_event[i], hipEventDisableTiming) != hipSuccess) {
            for (int j = 0; j < i; j++) (void)hipEventDestroy(ctx->desc_event[j]);
            (void)hipHostFree(ctx->fault_host);
            (void)hipHostFree(ctx->desc_pinned);
            (void)hipFree(ctx->workspace);
            (void)hipStreamDestroy(ctx->stream);
            delete ctx;
            return lh_fail(LH_ERR_NO_COMMAND_QUEUE, "hipEventCreate");
        }
    }
    // The attention kernels with hand-over areas in dynamic LDS get their limit raised here, so that no launch -- in
    // particular none inside a recorded batch or from the entry that may not allocate -- has to do it.
    {
        const int ra = lh_attention_kernels_init(ctx);
        if (ra != LH_OK) { lh_context_destroy(ctx); return ra; }
    }
    *out = ctx;
    return LH_OK;
}

void lh_context_destroy(lh_context* ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);
    ctx_release(ctx);
}

int lh_context_device_name(const lh_context* ctx, char* dst, size_t dst_len) {
    if (!ctx || !dst || dst_len == 0) return lh_fail(LH_ERR_INVALID_ARGUMENT, "device_name: null argument");
    snprintf(dst, dst_len, "%s", ctx->name);
    return LH_OK;
}
int lh_context_compute_units(const lh_context* ctx) { return ctx ? ctx->cu_count : 0; }
void* lh_context_stream(const lh_context* ctx) { return ctx ? (void*)ctx->stream : nullptr; }

int lh_context_synchronize(lh_context* ctx) {
    if (ctx && ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "context_synchronize: not while a graph is being captured");
    if (!ctx) return lh_fail(LH_ERR_INVALID_ARGUMENT, "synchronize: context is null");
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: %s", hipGetErrorString(e));
    return lh_check_fault_word(ctx);
}

// ---- events -----------------------------------------------------------------
struct lh_event { lh_context* ctx; hipEvent_t ev; };

int lh_event_create(lh_context* ctx, lh_event** out) {
    if (!ctx || !out) return lh_fail(LH_ERR_INVALID_ARGUMENT, "event_create: null argument");
    lh_event* e = new (std::nothrow) lh_event();
    if (!e) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", sizeof(lh_event));
    e->ctx = ctx;
    if (hipEventCreate(&e->ev) != hipSuccess) { delete e; return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: hipEventCreate"); }
    ctx_retain(ctx);
    *out = e;
    return LH_OK;
}
void lh_event_destroy(lh_event* ev) {
    if (!ev) return;
    (void)hipEventDestroy(ev->ev);
    ctx_release(ev->ctx);
    delete ev;
}
int lh_event_record(lh_event* ev) {
    if (!ev) return lh_fail(LH_ERR_INVALID_ARGUMENT, "event_record: event is null");
    hipError_t e = hipEventRecord(ev->ev, ev->ctx->stream);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: event_record: %s", hipGetErrorString(e));
    return LH_OK;
}
int lh_event_elapsed_ms(lh_event* start, lh_event* stop, float* ms) {
    if (!start || !stop || !ms) return lh_fail(LH_ERR_INVALID_ARGUMENT, "event_elapsed_ms: null argument");
    hipError_t e = hipEventSynchronize(stop->ev);
    if (e == hipSuccess) e = hipEventElapsedTime(ms, start->ev, stop->ev);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: event_elapsed_ms: %s", hipGetErrorString(e));
    return LH_OK;
}

// ---- buffers ----------------------------------------------------------------
static int new_buffer(lh_context* ctx, size_t len, lh_buffer** out) {
    if (!ctx || !out) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer: null argument");
    *out = nullptr;
    lh_buffer* b = new (std::nothrow) lh_buffer();
    if (!b) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", len);
    b->ctx = ctx; b->len = len; b->owns = true; b->ptr = nullptr; b->slack = 64;
    // Room for one 16-byte over-read past the end keeps vector loads of a
    // partly filled last unit inside the allocation.
    hipError_t e = hipMalloc(&b->ptr, (len ? len : 1) + 64);
    if (e != hipSuccess) { delete b; return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: %s", len, hipGetErrorString(e)); }
    ctx_retain(ctx);
    *out = b;
    return LH_OK;
}

int lh_buffer_empty(lh_context* ctx, size_t len, lh_buffer** out) {
    if (ctx && ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_empty: not while a graph is being captured");
    int r = new_buffer(ctx, len, out);
    if (r != LH_OK) return r;
    hipError_t e = hipMemsetAsync((*out)->ptr, 0, len + 64, ctx->stream);
    if (e != hipSuccess) { lh_buffer_free(*out); *out = nullptr; return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: %s", len, hipGetErrorString(e)); }
    return LH_OK;
}

int lh_buffer_from_bytes(lh_context* ctx, const void* src, size_t len, lh_buffer** out) {
    if (ctx && ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_from_bytes: not while a graph is being captured");
    if (!src && len) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_from_bytes: src is null");
    int r = new_buffer(ctx, len, out);
    if (r != LH_OK) return r;
    hipError_t e = hipMemsetAsync((char*)(*out)->ptr + len, 0, 64, ctx->stream);
    if (e == hipSuccess && len) e = hipMemcpyAsync((*out)->ptr, src, len, hipMemcpyHostToDevice, ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(ctx->stream);  // src may be freed by the caller on return
    if (e != hipSuccess) { lh_buffer_free(*out); *out = nullptr; return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: %s", len, hipGetErrorString(e)); }
    return LH_OK;
}

int lh_buffer_view(lh_buffer* parent, size_t offset, size_t len, lh_buffer** out) {
    if (!parent || !out) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_view: null argument");
    if (offset > parent->len || len > parent->len - offset)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_view: range %zu+%zu exceeds %zu", offset, len, parent->len);
    lh_buffer* b = new (std::nothrow) lh_buffer();
    if (!b) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", len);
    b->ctx = parent->ctx; b->ptr = (char*)parent->ptr + offset; b->len = len; b->owns = false;
    b->slack = parent->len - offset - len + parent->slack;
    ctx_retain(b->ctx);
    *out = b;
    return LH_OK;
}

int lh_buffer_wrap(lh_context* ctx, void* device_ptr, size_t len, lh_buffer** out) {
    if (!ctx || !out || (!device_ptr && len)) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_wrap: null argument");
    lh_buffer* b = new (std::nothrow) lh_buffer();
    if (!b) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", len);
    b->ctx = ctx; b->ptr = device_ptr; b->len = len; b->owns = false; b->slack = 0;
    ctx_retain(ctx);
    *out = b;
    return LH_OK;
}

void lh_buffer_free(lh_buffer* buf) {
    if (!buf) return;
    if (buf->owns && buf->ptr) {
        lh_context* ctx = buf->ctx;
        if (ctx->capturing) {
            ctx->deferred_free.push_back(buf->ptr);   // neither a wait nor a free may happen inside a capture
        } else {
            (void)hipStreamSynchronize(ctx->stream);
            (void)hipFree(buf->ptr);
        }
    }
    ctx_release(buf->ctx);
    delete buf;
}

size_t lh_buffer_length(const lh_buffer* buf) { return buf ? buf->len : 0; }
void* lh_buffer_device_ptr(const lh_buffer* buf) { return buf ? buf->ptr : nullptr; }

int lh_buffer_write(lh_buffer* buf, size_t offset, const void* src, size_t len) {
    if (!buf || (!src && len)) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_write: null argument");
    if (buf->ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_write: not while a graph is being captured");
    if (offset > buf->len || len > buf->len - offset)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_write: range %zu+%zu exceeds %zu", offset, len, buf->len);
    if (!len) return LH_OK;
    hipError_t e = hipMemcpyAsync((char*)buf->ptr + offset, src, len, hipMemcpyHostToDevice, buf->ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(buf->ctx->stream);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: buffer_write: %s", hipGetErrorString(e));
    return LH_OK;
}

int lh_buffer_read(const lh_buffer* buf, size_t offset, void* dst, size_t len) {
    if (!buf || (!dst && len)) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_read: null argument");
    if (buf->ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_read: not while a graph is being captured");
    if (offset > buf->len || len > buf->len - offset)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_read: range %zu+%zu exceeds %zu", offset, len, buf->len);
    if (!len) return LH_OK;
    hipError_t e = hipMemcpyAsync(dst, (const char*)buf->ptr + offset, len, hipMemcpyDeviceToHost, buf->ctx->stream);
    if (e == hipSuccess) e = hipStreamSynchronize(buf->ctx->stream);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: buffer_read: %s", hipGetErrorString(e));
    return LH_OK;
}

int lh_buffer_fill_zero(lh_buffer* buf) {
    if (!buf) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_fill_zero: buffer is null");
    if (!buf->len) return LH_OK;
    if (buf->ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "buffer_fill_zero: not while a graph is being captured");
    hipError_t e = hipMemsetAsync(buf->ptr, 0, buf->len, buf->ctx->stream);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: buffer_fill_zero: %s", hipGetErrorString(e));
    return LH_OK;
}

// ---- command batch ------------------------------------------------------------
int lh_batch_new(lh_context* ctx, lh_batch** out) {
    if (!ctx || !out) return lh_fail(LH_ERR_INVALID_ARGUMENT, "batch_new: null argument");
    lh_batch* b = new (std::nothrow) lh_batch();
    if (!b) return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", sizeof(lh_batch));
    b->ctx = ctx; b->dispatch_count = 0;
    ctx_retain(ctx);
    *out = b;
    return LH_OK;
}
void lh_batch_free(lh_batch* batch) {
    if (!batch) return;
    ctx_release(batch->ctx);
    delete batch;
}
uint32_t lh_batch_dispatch_count(const lh_batch* batch) { return batch ? batch->dispatch_count : 0; }

int lh_batch_blit_copy(lh_batch* batch, const lh_buffer* src, size_t src_offset, lh_buffer* dst, size_t dst_offset, size_t len) {
    // batch.rs:46-57: out-of-bounds ranges are rejected before encoding.
    if (!batch || !src || !dst) return lh_fail(LH_ERR_INVALID_ARGUMENT, "blit_copy: null argument");
    if (src_offset > src->len || len > src->len - src_offset || dst_offset > dst->len || len > dst->len - dst_offset)
        return lh_fail(LH_ERR_INVALID_ARGUMENT, "blit_copy: range out of bounds (src %zu+%zu of %zu, dst %zu+%zu of %zu)",
                       src_offset, len, src->len, dst_offset, len, dst->len);
    if (!len) return LH_OK;
    const uint8_t* s = (const uint8_t*)src->ptr + src_offset;
    uint8_t* d = (uint8_t*)dst->ptr + dst_offset;
    const int cus = batch->ctx->cu_count;
    if ((((uintptr_t)s | (uintptr_t)d) & 15) == 0 && len >= 16) {
        const size_t n16 = len / 16;
        const unsigned grid = (unsigned)((n16 + 255) / 256 < (size_t)cus * 8 ? (n16 + 255) / 256 : (size_t)cus * 8);
        hipLaunchKernelGGL(blit_copy16_kernel, dim3(grid), dim3(256), 0, batch->ctx->stream, (const uint4*)s, (uint4*)d, n16);
        const size_t tail = len - n16 * 16;
        if (tail) hipLaunchKernelGGL(blit_copy1_kernel, dim3(1), dim3(256), 0, batch->ctx->stream, s + n16 * 16, d + n16 * 16, tail);
    } else {
        const unsigned grid = (unsigned)((len + 255) / 256 < (size_t)cus * 8 ? (len + 255) / 256 : (size_t)cus * 8);
        hipLaunchKernelGGL(blit_copy1_kernel, dim3(grid), dim3(256), 0, batch->ctx->stream, s, d, len);
    }
    int r = lh_check_launch("blit_copy");
    if (r == LH_OK) batch->dispatch_count++;
    return r;
}

int lh_batch_commit_and_wait(lh_batch* batch) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "commit_and_wait: batch is null");
    if (batch->ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "commit_and_wait: not while a graph is being captured");
    hipError_t e = hipStreamSynchronize(batch->ctx->stream);
    batch->dispatch_count = 0;
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: %s", hipGetErrorString(e));
    return lh_check_fault_word(batch->ctx);   // a kernel that gave up a bounded wait says so here (batch.rs:136-144: GPU errors surface at the wait)
}
int lh_batch_submit_and_renew(lh_batch* batch) {
    // Work is already on the stream as it is encoded; nothing to flush.
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "submit_and_renew: batch is null");
    batch->dispatch_count = 0;
    return LH_OK;
}
int lh_batch_commit_and_renew(lh_batch* batch) { return lh_batch_commit_and_wait(batch); }

// ---- recorded batches ----------------------------------------------------------
struct lh_graph {
    lh_context* ctx; hipGraph_t graph; hipGraphExec_t exec; uint32_t dispatch_count;
    std::vector<void*> owned;   // allocations released while the graph was recorded: its dispatches may still use them
};

int lh_batch_begin_capture(lh_batch* batch) {
    if (!batch) return lh_fail(LH_ERR_INVALID_ARGUMENT, "begin_capture: batch is null");
    lh_context* ctx = batch->ctx;
    if (ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "begin_capture: a capture is already open on this context");
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: begin_capture: %s", hipGetErrorString(e));
    ctx->capturing = true;
    batch->dispatch_count = 0;
    return LH_OK;
}

int lh_batch_end_capture(lh_batch* batch, lh_graph** out) {
    if (!batch || !out) return lh_fail(LH_ERR_INVALID_ARGUMENT, "end_capture: null argument");
    *out = nullptr;
    lh_context* ctx = batch->ctx;
    if (!ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "end_capture: no capture is open on this context");
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    std::vector<void*> released;
    released.swap(ctx->deferred_free);
    auto drop_released = [&]() {   // no graph will replay: nothing can reference them once the stream is idle
        if (released.empty()) return;
        (void)hipStreamSynchronize(ctx->stream);
        for (void* p : released) (void)hipFree(p);
        released.clear();
    };
    if (e != hipSuccess || !graph) { drop_released(); return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: end_capture: %s", hipGetErrorString(e)); }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        drop_released();
        return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: graph instantiation: %s", hipGetErrorString(e));
    }
    lh_graph* g = new (std::nothrow) lh_graph();
    if (!g) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        drop_released();
        return lh_fail(LH_ERR_BUFFER_ALLOCATION, "size=%zu: host allocation", sizeof(lh_graph));
    }
    g->ctx = ctx; g->graph = graph; g->exec = exec; g->dispatch_count = batch->dispatch_count;
    g->owned.swap(released);
    ctx_retain(ctx);
    batch->dispatch_count = 0;
    *out = g;
    return LH_OK;
}

int lh_graph_launch(lh_graph* graph) {
    if (!graph) return lh_fail(LH_ERR_INVALID_ARGUMENT, "graph_launch: graph is null");
    if (graph->ctx->capturing) return lh_fail(LH_ERR_INVALID_ARGUMENT, "graph_launch: not while a graph is being captured");
    hipError_t e = hipGraphLaunch(graph->exec, graph->ctx->stream);
    if (e != hipSuccess) return lh_fail(LH_ERR_COMMAND_BUFFER, "GPU error: graph_launch: %s", hipGetErrorString(e));
    return LH_OK;
}

uint32_t lh_graph_dispatch_count(const lh_graph* graph) { return graph ? graph->dispatch_count : 0; }

void lh_graph_free(lh_graph* graph) {
    if (!graph) return;
    (void)hipStreamSynchronize(graph->ctx->stream);   // a replay may still be running
    (void)hipGraphExecDestroy(graph->exec);
    (void)hipGraphDestroy(graph->graph);
    for (void* p : graph->owned) (void)hipFree(p);
    ctx_release(graph->ctx);
    delete graph;
}

// kernels.rs:6155-6304
static int env_flag_default_on(const char* name) {
    const char* v = getenv(name);
    return !(v && strcmp(v, "0") == 0);
}
uint32_t lh_smallm_max_m(void) { return 8; }
uint32_t lh_batchm_max_m(void) { return 4; }
uint32_t lh_multivec_max_m(void) { return 16; }
int lh_batchm_enabled(void) { static int v = env_flag_default_on("LOCAL_AI_BATCHM"); return v; }
int lh_mma_enabled(void) { static int v = env_flag_default_on("LOCAL_AI_MMA"); return v; }
int lh_smallm_enabled(void) { static int v = env_flag_default_on("LOCAL_AI_SMALLM"); return v; }

}  // extern "C"
