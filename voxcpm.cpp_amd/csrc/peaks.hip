// peaks.hip -- what this GPU actually delivers, measured with the simplest kernels there are: a streaming
// read of a large buffer (HBM), a loop of independent matrix-core instructions (MFMA), and a barrier across
// all work-groups of a resident grid (what a kernel that stays on the chip for a whole layer would pay where
// launches now follow each other).  The benchmark reports its rooflines against the published peaks AND
// against these; nothing in the product path uses this file.  Built as its own small library (libvx_peaks.so).
#include <hip/hip_runtime.h>

#include <cstdint>

typedef float    f32x4 __attribute__((ext_vector_type(4)));
typedef float    f32x16 __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef int      i32x4 __attribute__((ext_vector_type(4)));

namespace {

// Every block streams a contiguous slice with 16-byte loads, UNROLL of them in flight per lane, and leaves one
// word so that the loads cannot be dropped.
template <int UNROLL>
__global__ __launch_bounds__(256) void stream_read_kernel(const i32x4 * __restrict__ src, size_t n_vec, int * __restrict__ sink) {
    const size_t per_block = (n_vec + gridDim.x - 1) / gridDim.x;
    const size_t begin = (size_t) blockIdx.x * per_block;
    const size_t end   = begin + per_block < n_vec ? begin + per_block : n_vec;
    i32x4 acc = { 0, 0, 0, 0 };
    size_t i = begin + threadIdx.x;
    for (; i + (size_t) (UNROLL - 1) * 256 < end; i += (size_t) UNROLL * 256) {
        i32x4 v[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) v[u] = __builtin_nontemporal_load(src + i + (size_t) u * 256);
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
    }
    for (; i < end; i += 256) acc ^= __builtin_nontemporal_load(src + i);
    const int x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (x == 0x5a5a5a5a) sink[blockIdx.x] = x; // practically never: the store only keeps the loads alive
}

// 8 independent accumulators per wave, `iters` rounds: nothing but v_mfma_f32_32x32x16_f16 in the loop
__global__ __launch_bounds__(256) void mfma_f16_kernel(int iters, float * __restrict__ sink) {
    f16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16) (0.001f * (float) ((threadIdx.x + i) & 7)); b[i] = (_Float16) (0.002f * (float) ((threadIdx.x + 3 * i) & 7)); }
    f32x16 acc[8];
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[k][i] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 8; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[k], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < 8; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) s += acc[k][i];
    if (s == 123.456f) sink[blockIdx.x * 256 + threadIdx.x] = s;
}

// `rounds` barriers over the whole grid, nothing else: lane 0 of every work-group adds 1 to a counter in device memory
// and polls it (sleeping between polls) until all work-groups of the round have arrived; the other lanes wait at the
// work-group barrier.  ORDERED = false: relaxed device-scope accesses, the bare cost of the round trip through L2.
// ORDERED = true: the arrival is a release and the last poll an acquire, as a barrier must be when the work-groups
// exchange data through memory (L2 write-back of what the work-group wrote, invalidation of what it cached).
// A work-group gives up after spin_limit polls in all, raises *failed and leaves, so the grid drains whatever happens;
// the launcher only accepts grids that are resident all at once.
template <bool ORDERED>
__global__ __launch_bounds__(256) void grid_barrier_kernel(unsigned * __restrict__ counter, int rounds, unsigned spin_limit, int * __restrict__ failed) {
    __shared__ int gave_up;
    if (threadIdx.x == 0) gave_up = 0;
    unsigned spins = 0; // polls of the whole kernel, not of a round: a grid that cannot meet is gone after spin_limit polls in all
    for (int r = 0; r < rounds; ++r) {
        __syncthreads();
        if (threadIdx.x == 0) {
            const unsigned target = (unsigned) (r + 1) * gridDim.x;
            __hip_atomic_fetch_add(counter, 1u, ORDERED ? __ATOMIC_RELEASE : __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            while (__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) < target) {
                __builtin_amdgcn_s_sleep(1);
                if (++spins > spin_limit) { *failed = 1; gave_up = 1; break; }
            }
            if (ORDERED) __atomic_thread_fence(__ATOMIC_ACQUIRE); // (device scope for global memory)
        }
        __syncthreads();
        if (gave_up) return;
    }
}

} // namespace

extern "C" {

// streams `bytes` (a multiple of 16) from src once; blocks = 0 picks 8 per CU
__attribute__((visibility("default"))) int vxp_stream_read(const void * src, size_t bytes, int * sink, int blocks, void * stream) {
    if (!src || !sink || bytes % 16) return 1;
    if (blocks <= 0) {
        int dev = 0, cus = 256;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) cus = p.multiProcessorCount;
        blocks = 8 * cus;
    }
    stream_read_kernel<8><<<dim3((unsigned) blocks), dim3(256), 0, (hipStream_t) stream>>>((const i32x4 *) src, bytes / 16, sink);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

// blocks x 4 waves x iters x 8 MFMAs of 32 x 32 x 16 (32768 flop each); sink: blocks * 256 floats
__attribute__((visibility("default"))) int vxp_mfma_f16(int blocks, int iters, float * sink, void * stream) {
    if (!sink || blocks <= 0 || iters <= 0) return 1;
    mfma_f16_kernel<<<dim3((unsigned) blocks), dim3(256), 0, (hipStream_t) stream>>>(iters, sink);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
__attribute__((visibility("default"))) double vxp_mfma_f16_flop(int blocks, int iters) {
    return (double) blocks * 4.0 * (double) iters * 8.0 * 32768.0;
}


// `rounds` grid-wide barriers of `blocks` work-groups of 256 lanes (at most 4 per compute unit, so that all are resident);
// *counter must be 0 at the start, *failed is raised if a work-group ever gave up waiting (2^22 polls)
__attribute__((visibility("default"))) int vxp_grid_barrier(int blocks, int rounds, int ordered, unsigned * counter, int * failed, void * stream) {
    if (!counter || !failed || blocks <= 0 || rounds <= 0) return 1;
    int dev = 0;
    hipDeviceProp_t p;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&p, dev) != hipSuccess) return 2;
    if (blocks > 4 * p.multiProcessorCount) return 1;
    if (ordered) grid_barrier_kernel<true><<<dim3((unsigned) blocks), dim3(256), 0, (hipStream_t) stream>>>(counter, rounds, 1u << 22, failed);
    else         grid_barrier_kernel<false><<<dim3((unsigned) blocks), dim3(256), 0, (hipStream_t) stream>>>(counter, rounds, 1u << 22, failed);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

} // extern "C"
