// peaks.hip -- what this GPU actually delivers, measured with the simplest kernels there are: a streaming
// read of a large buffer (HBM), a loop of independent matrix-core instructions (MFMA), a barrier across
// all work-groups of a resident grid (what a kernel that stays on the chip for a whole layer would pay where
// launches now follow each other), and pairs of instruction streams on one SIMD (whether matrix and vector
// work run side by side).  The benchmark reports its rooflines against the published peaks AND
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

// Do a SIMD's matrix core and its vector unit run side by side?  A work-group of 8 waves puts two waves on every SIMD;
// waves 0-3 run role_a, waves 4-7 role_b: 0 idle, 1 four independent v_mfma_f32_32x32x16_f16 per iteration (128 cycles of
// matrix work), 2 thirty-two v_fma_f32 in eight independent chains, 3 sixteen v_exp_f32 (each followed by a v_sub_f32 that
// keeps the argument in range).  Times of the pairs against the times of the roles alone answer the question.
__device__ __forceinline__ void coexec_mfma(int iters, float * sink) {
    f16x8 a, b;
#pragma unroll
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16) (0.001f * (float) ((threadIdx.x + i) & 7)); b[i] = (_Float16) (0.002f * (float) ((threadIdx.x + 3 * i) & 7)); }
    f32x16 acc[4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[k][i] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 4; ++k) acc[k] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[k], 0, 0, 0);
    }
    float s = 0.0f;
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
        for (int i = 0; i < 16; ++i) s += acc[k][i];
    if (s == 123.456f) sink[threadIdx.x] = s;
}
__device__ __forceinline__ void coexec_fma(int iters, float * sink) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = 0.5f + (float) threadIdx.x * 1e-3f + (float) i;
    const float m = 0.999f, c = 1e-3f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int i = 0; i < 8; ++i) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(v[i]) : "v"(m), "v"(c));
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += v[i];
    if (s == 123.456f) sink[threadIdx.x] = s;
}
__device__ __forceinline__ void coexec_exp(int iters, float * sink) {
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = -0.5f - (float) threadIdx.x * 1e-3f - (float) i;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int i = 0; i < 8; ++i) asm volatile("v_exp_f32 %0, %0\n\tv_sub_f32 %0, 0, %0" : "+v"(v[i]));
    }
    float s = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) s += v[i];
    if (s == 123.456f) sink[threadIdx.x] = s;
}
__global__ __launch_bounds__(512) void coexec_kernel(int role_a, int role_b, int iters, float * __restrict__ sink) {
    const int role = (threadIdx.x >> 8) ? role_b : role_a; // uniform per wave
    if (role == 1) coexec_mfma(iters, sink);
    else if (role == 2) coexec_fma(iters, sink);
    else if (role == 3) coexec_exp(iters, sink);
}

// LDS read rate of a compute unit: every wave of a work-group issues 16-byte reads at lane-contiguous addresses (or, with
// `same`, one address per 16 lanes) from a 64 KB array, eight per iteration; the address moves behind an opaque
// constraint so that the reads stay in the loop.
__global__ __launch_bounds__(1024) void lds_read_kernel(int iters, int same, float * __restrict__ sink) {
    __shared__ __attribute__((aligned(16))) char lds[65536];
    for (int i = threadIdx.x; i < 16384; i += blockDim.x) ((float *) lds)[i] = (float) i;
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int base = (wave * 4096 + (same ? (lane >> 4) * 16 : lane * 16)) & 65535;
    f32x4 acc = {0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
        asm volatile("" : "+v"(base));
#pragma unroll
        for (int u = 0; u < 8; ++u) acc += *(const f32x4 *) (lds + ((base + u * 1024) & 65535));
    }
    if (acc[0] + acc[1] + acc[2] + acc[3] == 123.456f) sink[threadIdx.x] = acc[0];
}

// Fill rate of a compute unit with every compute unit pulling: work-groups of 8 waves re-read a region of `region`
// bytes (2 MiB: an XCD's L2 holds it; 16 MiB: the memory-side cache does), each wave 1 KB per load, 8 loads in flight,
// the work-groups starting at scattered places.
__global__ __launch_bounds__(512) void fill_rate_kernel(const char * __restrict__ src, size_t region, size_t per_wg, int * __restrict__ sink) {
    const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
    const size_t per_wave = per_wg / 8;
    size_t pos = ((size_t) blockIdx.x * 7919 * 1024 + (size_t) wid * per_wave) % region;
    const int n_kb = (int) (per_wave / 1024);
    i32x4 acc = {0, 0, 0, 0};
    for (int i = 0; i < n_kb; i += 8) {
        i32x4 v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = *(const i32x4 *) (src + (pos + (size_t) u * 1024) % region + lane * 16);
#pragma unroll
        for (int u = 0; u < 8; ++u) acc ^= v[u];
        pos = (pos + 8 * 1024) % region;
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5a5a5a5a) sink[blockIdx.x] = acc[0];
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


// one work-group of 8 waves per compute unit slot (`blocks` of them), `iters` iterations of the two roles (see coexec_kernel);
// sink: 512 floats
__attribute__((visibility("default"))) int vxp_coexec(int blocks, int role_a, int role_b, int iters, float * sink, void * stream) {
    if (!sink || blocks <= 0 || iters <= 0 || role_a < 0 || role_a > 3 || role_b < 0 || role_b > 3) return 1;
    coexec_kernel<<<dim3((unsigned) blocks), dim3(512), 0, (hipStream_t) stream>>>(role_a, role_b, iters, sink);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}


// `blocks` work-groups of `waves` waves (1 .. 16), `iters` iterations of eight 16-byte LDS reads per wave; sink: 1024 floats
__attribute__((visibility("default"))) int vxp_lds_read(int blocks, int waves, int iters, int same, float * sink, void * stream) {
    if (!sink || blocks <= 0 || waves < 1 || waves > 16 || iters <= 0) return 1;
    lds_read_kernel<<<dim3((unsigned) blocks), dim3(64 * waves), 0, (hipStream_t) stream>>>(iters, same, sink);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}
// `blocks` work-groups of 8 waves each read `per_wg` bytes (a multiple of 64 KiB) of the first `region` bytes of src
// (region a multiple of 8 KiB, at most the buffer's size); sink: `blocks` ints
__attribute__((visibility("default"))) int vxp_fill_rate(const void * src, size_t region, size_t per_wg, int blocks, int * sink, void * stream) {
    if (!src || !sink || blocks <= 0 || region == 0 || region % 8192 || per_wg == 0 || per_wg % 65536) return 1;
    fill_rate_kernel<<<dim3((unsigned) blocks), dim3(512), 0, (hipStream_t) stream>>>((const char *) src, region, per_wg, sink);
    return hipGetLastError() == hipSuccess ? 0 : 2;
}

} // extern "C"
