// What it costs to make one kernel out of two dependent ones on this device: a launch that depends on the one before it,
// against a grid-wide barrier inside a kernel (every workgroup publishes 256 bytes, fences, adds itself to a device-scope
// counter and polls it -- a bounded number of times, so the kernel ends whatever happens -- then reads a neighbour's bytes).
// A stand-alone program, no part of the library; every workgroup of the barrier kernel is resident (at most one per CU).
//
//   ./grid_sync_probe
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
#define CK(x) do { hipError_t e = (x); if (e != hipSuccess) { printf("%s: %s\n", #x, hipGetErrorString(e)); return 1; } } while (0)

__global__ void tiny_kernel(float* p) { if (threadIdx.x == 0) p[blockIdx.x] += 1.0f; }

__global__ __launch_bounds__(256) void barrier_kernel(float* data, unsigned* counter, unsigned* fault, int rounds, unsigned spin_limit) {
    const unsigned G = gridDim.x;
    for (int r = 0; r < rounds; r++) {
        if (threadIdx.x < 64) data[blockIdx.x * 64 + threadIdx.x] += 1.0f;    // something to publish
        __syncthreads();
        if (threadIdx.x == 0) {
            __threadfence();
            atomicAdd(counter, 1u);
            const unsigned target = G * (unsigned)(r + 1);
            unsigned spins = 0;
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target && spins++ < spin_limit) __builtin_amdgcn_s_sleep(1);
            if (spins >= spin_limit) *fault = 1u;
            __threadfence();
        }
        __syncthreads();
        // read what a neighbour published
        if (threadIdx.x < 64) data[blockIdx.x * 64 + threadIdx.x] += 0.5f * __builtin_nontemporal_load(&data[((blockIdx.x + 1) % G) * 64 + threadIdx.x]);
    }
}

int main() {
    float* data; unsigned *counter, *fault;
    CK(hipMalloc(&data, 256 * 64 * 4)); CK(hipMalloc(&counter, 4)); CK(hipMalloc(&fault, 4));
    CK(hipMemset(data, 0, 256 * 64 * 4)); CK(hipMemset(fault, 0, 4));
    hipStream_t s; CK(hipStreamCreate(&s));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    const int N = 2000;
    for (int G : {32, 256}) {
        for (int rep = 0; rep < 3; rep++) {
            CK(hipEventRecord(e0, s));
            for (int i = 0; i < N; i++) hipLaunchKernelGGL(tiny_kernel, dim3(G), dim3(256), 0, s, data);
            CK(hipEventRecord(e1, s)); CK(hipEventSynchronize(e1));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1));
            if (rep == 2) printf("G=%3d: %d dependent launches of a tiny kernel: %.2f us each\n", G, N, ms * 1e3 / N);
        }
        for (int rep = 0; rep < 3; rep++) {
            CK(hipMemsetAsync(counter, 0, 4, s));
            CK(hipEventRecord(e0, s));
            hipLaunchKernelGGL(barrier_kernel, dim3(G), dim3(256), 0, s, data, counter, fault, N, 1u << 20);
            CK(hipEventRecord(e1, s)); CK(hipEventSynchronize(e1));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1));
            unsigned f; CK(hipMemcpy(&f, fault, 4, hipMemcpyDeviceToHost));
            if (rep == 2) printf("G=%3d: %d grid barriers in one kernel: %.2f us each (fault %u)\n", G, N, ms * 1e3 / N, f);
        }
    }
    return 0;
}
