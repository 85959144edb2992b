// vx_runtime.hip -- device discovery, memory, streams and the per-stream workspace.
#include "vx_common.hpp"

#include <cstring>
#include <mutex>
#include <unordered_map>

namespace {

thread_local char g_err[512] = "";

struct workspace {
    void * ptr   = nullptr;
    size_t bytes = 0;
};
std::mutex                                    g_ws_mutex;
std::unordered_map<unsigned long long, workspace> g_ws;  // key: device << 56 ^ stream handle
std::unordered_map<unsigned long long, workspace> g_cnt; // zero-initialised counters, same key

} // namespace

void vx_set_error(const char * fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
}

vx_status vx_fail(vx_status st, const char * fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return st;
}

vx_status vx_workspace(hipStream_t stream, size_t bytes, void ** ptr) {
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    const unsigned long long key = ((unsigned long long) dev << 56) ^ (unsigned long long) (uintptr_t) stream;
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    workspace & ws = g_ws[key];
    if (ws.bytes < bytes) {
        if (ws.ptr) {
            // work already queued on this stream may still read the old block
            VX_HIP(hipStreamSynchronize(stream));
            VX_HIP(hipFree(ws.ptr));
            ws.ptr   = nullptr;
            ws.bytes = 0;
        }
        size_t want = bytes < (size_t) (1u << 20) ? (size_t) (1u << 20) : bytes + bytes / 4;
        want        = (want + 255) & ~(size_t) 255;
        hipError_t e = hipMalloc(&ws.ptr, want);
        if (e != hipSuccess) {
            ws.ptr = nullptr;
            return vx_fail(VX_ERR_ALLOC, "workspace hipMalloc(%zu) failed: %s", want, hipGetErrorString(e));
        }
        ws.bytes = want;
    }
    *ptr = ws.ptr;
    return VX_OK;
}

vx_status vx_counters(hipStream_t stream, size_t count, void ** ptr) {
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    const unsigned long long key = ((unsigned long long) dev << 56) ^ (unsigned long long) (uintptr_t) stream;
    const size_t bytes = count * sizeof(int);
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    workspace & ws = g_cnt[key];
    if (ws.bytes < bytes) {
        if (ws.ptr) {
            VX_HIP(hipStreamSynchronize(stream));
            VX_HIP(hipFree(ws.ptr));
            ws.ptr   = nullptr;
            ws.bytes = 0;
        }
        size_t want = bytes < 4096 ? 4096 : 2 * bytes;
        hipError_t e = hipMalloc(&ws.ptr, want);
        if (e != hipSuccess) {
            ws.ptr = nullptr;
            return vx_fail(VX_ERR_ALLOC, "counter hipMalloc(%zu) failed: %s", want, hipGetErrorString(e));
        }
        ws.bytes = want;
        VX_HIP(hipMemsetAsync(ws.ptr, 0, want, stream));
    }
    *ptr = ws.ptr;
    return VX_OK;
}

extern "C" {

const char * vx_last_error(void) { return g_err; }

int vx_device_count(void) {
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) {
        (void) hipGetLastError();
        return 0;
    }
    int ok = 0;
    for (int i = 0; i < n; ++i) {
        hipDeviceProp_t p;
        if (hipGetDeviceProperties(&p, i) != hipSuccess) continue;
        if (strncmp(p.gcnArchName, "gfx950", 6) == 0) ++ok;
    }
    // devices are addressed by HIP ordinal; a box mixing architectures is not supported
    return ok == n ? n : 0;
}

vx_status vx_init(int device) {
    const int n = vx_device_count();
    if (n <= 0) return vx_fail(VX_ERR_NO_DEVICE, "no gfx950 device visible to HIP");
    if (device < 0 || device >= n) return vx_fail(VX_ERR_INVALID, "device %d out of range (0..%d)", device, n - 1);
    VX_HIP(hipSetDevice(device));
    return VX_OK;
}

vx_status vx_device_info(int device, char * name, size_t name_len, size_t * free_bytes, size_t * total_bytes,
                         int * compute_units) {
    hipDeviceProp_t p;
    VX_HIP(hipGetDeviceProperties(&p, device));
    if (name && name_len) snprintf(name, name_len, "%s (%s)", p.name, p.gcnArchName);
    if (compute_units) *compute_units = p.multiProcessorCount;
    if (free_bytes || total_bytes) {
        int cur = 0;
        VX_HIP(hipGetDevice(&cur));
        VX_HIP(hipSetDevice(device));
        size_t f = 0, t = 0;
        hipError_t e = hipMemGetInfo(&f, &t);
        (void) hipSetDevice(cur);
        if (e != hipSuccess) return vx_fail(VX_ERR_HIP, "hipMemGetInfo failed: %s", hipGetErrorString(e));
        if (free_bytes) *free_bytes = f;
        if (total_bytes) *total_bytes = t;
    }
    return VX_OK;
}

vx_status vx_malloc(void ** ptr, size_t bytes) {
    if (!ptr) return vx_fail(VX_ERR_INVALID, "vx_malloc: null out pointer");
    *ptr         = nullptr;
    hipError_t e = hipMalloc(ptr, bytes ? bytes : 1);
    if (e != hipSuccess) return vx_fail(VX_ERR_ALLOC, "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    return VX_OK;
}

vx_status vx_free(void * ptr) {
    if (ptr) VX_HIP(hipFree(ptr));
    return VX_OK;
}

vx_status vx_malloc_host(void ** ptr, size_t bytes) {
    if (!ptr) return vx_fail(VX_ERR_INVALID, "vx_malloc_host: null out pointer");
    *ptr         = nullptr;
    hipError_t e = hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault);
    if (e != hipSuccess) return vx_fail(VX_ERR_ALLOC, "hipHostMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
    return VX_OK;
}

vx_status vx_free_host(void * ptr) {
    if (ptr) VX_HIP(hipHostFree(ptr));
    return VX_OK;
}

vx_status vx_memcpy_h2d(void * dst, const void * src, size_t bytes, vx_stream stream) {
    if (bytes) VX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, (hipStream_t) stream));
    return VX_OK;
}
vx_status vx_memcpy_d2h(void * dst, const void * src, size_t bytes, vx_stream stream) {
    if (bytes) VX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, (hipStream_t) stream));
    return VX_OK;
}
vx_status vx_memcpy_d2d(void * dst, const void * src, size_t bytes, vx_stream stream) {
    if (bytes) VX_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t) stream));
    return VX_OK;
}
vx_status vx_memset(void * dst, int value, size_t bytes, vx_stream stream) {
    if (bytes) VX_HIP(hipMemsetAsync(dst, value, bytes, (hipStream_t) stream));
    return VX_OK;
}

vx_status vx_stream_create(vx_stream * stream) {
    if (!stream) return vx_fail(VX_ERR_INVALID, "vx_stream_create: null out pointer");
    hipStream_t s = nullptr;
    VX_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
    *stream = (vx_stream) s;
    return VX_OK;
}
vx_status vx_stream_destroy(vx_stream stream) {
    if (!stream) return VX_OK;
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    VX_HIP(hipStreamSynchronize((hipStream_t) stream));
    {   // the stream's scratch blocks go with it
        const unsigned long long key = ((unsigned long long) dev << 56) ^ (unsigned long long) (uintptr_t) stream;
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        for (auto * map : {&g_ws, &g_cnt}) {
            auto it = map->find(key);
            if (it == map->end()) continue;
            if (it->second.ptr) (void) hipFree(it->second.ptr);
            map->erase(it);
        }
    }
    VX_HIP(hipStreamDestroy((hipStream_t) stream));
    return VX_OK;
}
vx_status vx_stream_synchronize(vx_stream stream) {
    VX_HIP(hipStreamSynchronize((hipStream_t) stream));
    return VX_OK;
}

} // extern "C"
