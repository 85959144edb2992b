// vx_runtime.hip -- device discovery, memory, streams and the per-stream workspace.
#include "vx_common.hpp"
#include "ws_policy.hpp"

#include <cstring>
#include <mutex>
#include <unordered_map>

namespace {

thread_local char g_err[512] = "";

std::mutex                                      g_ws_mutex;
std::unordered_map<unsigned long long, vx_ws_state> g_ws; // key: device << 56 ^ stream handle

unsigned long long ws_key(int dev, hipStream_t stream) {
    return ((unsigned long long) dev << 56) ^ (unsigned long long) (uintptr_t) stream;
}

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
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    vx_ws_state & ws = g_ws[ws_key(dev, stream)];
    bool capturing = false;
    if (bytes > ws.cur.bytes) { // only a growing request needs to know
        hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(stream, &cs) != hipSuccess) (void) hipGetLastError();
        capturing = cs != hipStreamCaptureStatusNone;
    }
    hipError_t err = hipSuccess;
    const vx_ws_result r = vx_ws_request(ws, bytes, capturing, [&](size_t want) -> void * {
        void * p = nullptr;
        err      = hipMalloc(&p, want);
        return err == hipSuccess ? p : nullptr;
    }, ptr);
    if (r == VX_WS_CAPTURING)
        return vx_fail(VX_ERR_UNSUPPORTED, "the stream is being captured and the call needs %zu bytes of workspace but %zu are reserved: "
                       "call vx_workspace_reserve(stream, bytes) before the capture begins", bytes, ws.cur.bytes);
    if (r == VX_WS_ALLOC_FAILED)
        return vx_fail(VX_ERR_ALLOC, "workspace hipMalloc for %zu bytes failed: %s", bytes, hipGetErrorString(err));
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
    return vx_fattn_static_setup(); // the fixed scratch array's address on this device
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
    {   // the stream's scratch blocks, live and retired, go with it
        std::lock_guard<std::mutex> lock(g_ws_mutex);
        auto it = g_ws.find(ws_key(dev, (hipStream_t) stream));
        if (it != g_ws.end()) {
            vx_ws_release_all(it->second, [](void * p) { (void) hipFree(p); });
            g_ws.erase(it);
        }
    }
    VX_HIP(hipStreamDestroy((hipStream_t) stream));
    return VX_OK;
}
vx_status vx_workspace_reserve(vx_stream stream, size_t bytes) {
    void * p = nullptr;
    return vx_workspace((hipStream_t) stream, bytes, &p);
}
vx_status vx_workspace_info(vx_stream stream, void ** ptr, size_t * bytes, int * retired_blocks) {
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_ws.find(ws_key(dev, (hipStream_t) stream));
    if (ptr) *ptr = it == g_ws.end() ? nullptr : it->second.cur.ptr;
    if (bytes) *bytes = it == g_ws.end() ? 0 : it->second.cur.bytes;
    if (retired_blocks) *retired_blocks = it == g_ws.end() ? 0 : (int) it->second.retired.size();
    return VX_OK;
}
vx_status vx_graph_begin(vx_stream stream) {
    VX_HIP(hipStreamBeginCapture((hipStream_t) stream, hipStreamCaptureModeThreadLocal));
    return VX_OK;
}
vx_status vx_graph_end(vx_stream stream, vx_graph * graph) {
    if (!graph) return vx_fail(VX_ERR_INVALID, "vx_graph_end: null out pointer");
    *graph = nullptr;
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture((hipStream_t) stream, &g);
    if (e != hipSuccess || !g) { // an invalidated recording: the stream is usable again, nothing to replay
        (void) hipGetLastError();
        if (g) (void) hipGraphDestroy(g);
        return VX_OK;
    }
    hipGraphExec_t exec = nullptr;
    const hipError_t e2 = hipGraphInstantiate(&exec, g, nullptr, nullptr, 0);
    (void) hipGraphDestroy(g);
    if (e2 != hipSuccess || !exec) {
        (void) hipGetLastError();
        return VX_OK;
    }
    *graph = (vx_graph) exec;
    return VX_OK;
}
vx_status vx_graph_launch(vx_graph graph, vx_stream stream) {
    if (!graph) return vx_fail(VX_ERR_INVALID, "vx_graph_launch: null graph");
    VX_HIP(hipGraphLaunch((hipGraphExec_t) graph, (hipStream_t) stream));
    return VX_OK;
}
vx_status vx_graph_destroy(vx_graph graph) {
    if (graph) VX_HIP(hipGraphExecDestroy((hipGraphExec_t) graph));
    return VX_OK;
}
vx_status vx_stream_synchronize(vx_stream stream) {
    VX_HIP(hipStreamSynchronize((hipStream_t) stream));
    return VX_OK;
}

} // extern "C"
