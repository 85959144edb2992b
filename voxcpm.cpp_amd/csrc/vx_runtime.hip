// vx_runtime.hip -- device discovery, memory, streams and the per-stream workspace.
#include "vx_common.hpp"
#include "ws_policy.hpp"

#include <cstdlib>
#include <cstring>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace {

thread_local char g_err[512] = "";

std::mutex                                      g_ws_mutex;
std::unordered_map<unsigned long long, vx_ws_state> g_ws; // key: device << 56 ^ stream handle

unsigned long long ws_key(int dev, hipStream_t stream) {
    return ((unsigned long long) dev << 56) ^ (unsigned long long) (uintptr_t) stream;
}

// ---- recorded graphs ----------------------------------------------------------------------------------------------
// What a vx_graph handle points to: the instantiated HIP graph, and -- when every launch of the recording went through
// vx_launch and the captured graph's kernel nodes agree with them one for one -- the launches themselves, so that a
// later run of the same operators can be compared with the recording and the differences set on the graph's nodes.
struct launch_rec {
    const void * func;
    dim3         grid, block;
    unsigned     lds_bytes;
    unsigned     first_param, n_params; // into recorded_graph::params
};
struct param_rec { unsigned offset, size; }; // into recorded_graph::bytes
struct recorded_graph {
    hipGraphExec_t              exec = nullptr;
    hipGraph_t                  graph = nullptr; // kept while `nodes` are in use: they belong to it
    hipEvent_t                  done = nullptr;  // recorded after each launch of a patchable graph
    bool                        in_flight = false;
    std::vector<hipGraphNode_t> nodes;           // one per launch, in launch order; empty = replay only
    std::vector<launch_rec>     launches;
    std::vector<param_rec>      params;
    std::vector<char>           bytes;
};
thread_local recorded_graph * t_rec     = nullptr; // the recording being made (mode 1) or compared with (mode 2)
thread_local size_t           t_next    = 0;       // mode 2: the launch the next note is compared with
thread_local bool             t_differs = false;   // mode 2: another function, another count, or a node that would not take its arguments
thread_local int              t_patched = 0;

void destroy_recorded(recorded_graph * r) {
    if (!r) return;
    if (r->exec) (void) hipGraphExecDestroy(r->exec);
    if (r->graph) (void) hipGraphDestroy(r->graph);
    if (r->done) (void) hipEventDestroy(r->done);
    delete r;
}

// ---- pinned weights and what is derived from them -----------------------------------------------------------------
// A caller may declare ranges of device memory constant (vx_weights_pin).  For tensors inside such a range an operator
// may keep a re-laid-out copy from one call to the next (the pre-tiled Q8_0 weights of the large products) instead of
// producing it on every call; vx_weights_changed / vx_weights_unpin drop whatever was derived from the bytes they name.
struct pinned_range { int dev; uintptr_t lo, hi; };
struct derived_entry {
    vx_derived_key key;
    uintptr_t      src[2][2]; // the byte ranges it was derived from (second one empty for a single matrix)
    void *         ptr;
    size_t         bytes;
    hipEvent_t     ready;     // recorded behind the kernel that fills it
    hipStream_t    filled_on;
    bool           filled;
};
std::mutex                 g_pin_mutex;
std::vector<pinned_range>  g_pinned;
std::vector<derived_entry> g_derived;
size_t                     g_derived_bytes = 0;

bool same_key(const vx_derived_key & a, const vx_derived_key & b) {
    return a.dev == b.dev && a.kind == b.kind && a.w == b.w && a.w2 == b.w2 && a.K == b.K && a.M == b.M && a.nb01 == b.nb01;
}
bool inside_pinned(int dev, uintptr_t lo, uintptr_t hi) { // (g_pin_mutex held)
    for (const pinned_range & r : g_pinned) if (r.dev == dev && lo >= r.lo && hi <= r.hi) return true;
    return false;
}
void drop_derived_from(int dev, uintptr_t lo, uintptr_t hi) { // (g_pin_mutex held) hipFree waits for the kernels still reading
    for (size_t i = 0; i < g_derived.size();) {
        derived_entry & e = g_derived[i];
        bool hit = false;
        for (int k = 0; k < 2; ++k) hit = hit || (e.src[k][0] < e.src[k][1] && e.src[k][0] < hi && lo < e.src[k][1]);
        if (e.key.dev == dev && hit) {
            (void) hipFree(e.ptr);
            if (e.ready) (void) hipEventDestroy(e.ready);
            g_derived_bytes -= e.bytes;
            g_derived[i] = g_derived.back();
            g_derived.pop_back();
        } else ++i;
    }
}
size_t derived_cap() { // bytes this process may hold in derived copies (VX_DERIVED_WEIGHTS_MB, default 8192; 0 keeps none)
    static const size_t cap = [] { const char * e = getenv("VX_DERIVED_WEIGHTS_MB"); return (size_t) (e ? atoll(e) : 8192) << 20; }();
    return cap;
}

} // namespace

thread_local int vx_tl_launch_mode = 0;

void * vx_derived_get(const vx_derived_key & key, size_t bytes, hipStream_t stream, bool * fresh) {
    *fresh = false;
    // Not while launches are recorded, compared or captured: a fill would be recorded (or not run at all), a capture may
    // not allocate, and a recording must not hold the address of a copy that a later vx_weights_changed frees.
    if (vx_tl_launch_mode != 0) return nullptr;
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    if (g_pinned.empty()) return nullptr;
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &cs) != hipSuccess) { (void) hipGetLastError(); return nullptr; }
    if (cs != hipStreamCaptureStatusNone) return nullptr;
    for (derived_entry & e : g_derived)
        if (same_key(e.key, key) && e.bytes == bytes) {
            if (!e.filled) return nullptr; // (a fill that was never confirmed: not used)
            if (e.filled_on != stream && hipStreamWaitEvent(stream, e.ready, 0) != hipSuccess) { (void) hipGetLastError(); return nullptr; }
            return e.ptr;
        }
    const uintptr_t w = (uintptr_t) key.w, w2 = (uintptr_t) key.w2, span = (uintptr_t) key.M * key.nb01;
    if (!inside_pinned(key.dev, w, w + span) || (w2 && !inside_pinned(key.dev, w2, w2 + span))) return nullptr;
    if (g_derived_bytes + bytes > derived_cap()) return nullptr;
    derived_entry e = {};
    e.key = key;
    e.src[0][0] = w; e.src[0][1] = w + span;
    e.src[1][0] = w2; e.src[1][1] = w2 ? w2 + span : 0;
    e.bytes = bytes;
    if (hipMalloc(&e.ptr, bytes) != hipSuccess) { (void) hipGetLastError(); return nullptr; }
    if (hipEventCreateWithFlags(&e.ready, hipEventDisableTiming) != hipSuccess) { (void) hipGetLastError(); (void) hipFree(e.ptr); return nullptr; }
    e.filled_on = stream;
    e.filled = false;
    g_derived.push_back(e);
    g_derived_bytes += bytes;
    *fresh = true;
    return e.ptr;
}

void vx_derived_abandon(const vx_derived_key & key, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    for (size_t i = 0; i < g_derived.size(); ++i) {
        derived_entry & e = g_derived[i];
        if (same_key(e.key, key) && !e.filled && e.filled_on == stream) {
            (void) hipFree(e.ptr);
            (void) hipEventDestroy(e.ready);
            g_derived_bytes -= e.bytes;
            g_derived[i] = g_derived.back();
            g_derived.pop_back();
            return;
        }
    }
}

void vx_derived_filled(const vx_derived_key & key, hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    for (derived_entry & e : g_derived)
        if (same_key(e.key, key) && !e.filled && e.filled_on == stream) {
            if (hipEventRecord(e.ready, stream) == hipSuccess) e.filled = true;
            else (void) hipGetLastError();
            return;
        }
}

void vx_launch_note(const void * func, dim3 grid, dim3 block, size_t lds_bytes, void * const * params, const size_t * sizes, int n_params) {
    recorded_graph * r = t_rec;
    if (!r) return;
    if (vx_tl_launch_mode == 1) { // recording: keep the launch
        launch_rec l = { func, grid, block, (unsigned) lds_bytes, (unsigned) r->params.size(), (unsigned) n_params };
        for (int i = 0; i < n_params; ++i) {
            const size_t at = (r->bytes.size() + 15) & ~(size_t) 15;
            r->bytes.resize(at + sizes[i]);
            memcpy(r->bytes.data() + at, params[i], sizes[i]);
            r->params.push_back({ (unsigned) at, (unsigned) sizes[i] });
        }
        r->launches.push_back(l);
        return;
    }
    if (t_differs) return;
    if (t_next >= r->launches.size()) { t_differs = true; return; }
    launch_rec & l = r->launches[t_next];
    if (l.func != func || (int) l.n_params != n_params) { t_differs = true; return; }
    bool same = l.grid.x == grid.x && l.grid.y == grid.y && l.grid.z == grid.z && l.block.x == block.x && l.block.y == block.y &&
                l.block.z == block.z && l.lds_bytes == (unsigned) lds_bytes;
    for (int i = 0; i < n_params; ++i) {
        const param_rec & pr = r->params[l.first_param + i];
        if (pr.size != sizes[i]) { t_differs = true; return; }
        if (memcmp(r->bytes.data() + pr.offset, params[i], sizes[i]) != 0) {
            memcpy(r->bytes.data() + pr.offset, params[i], sizes[i]);
            same = false;
        }
    }
    if (!same) {
        constexpr int MAX_PARAMS = 16;
        void * ptrs[MAX_PARAMS];
        if (n_params > MAX_PARAMS) { t_differs = true; return; }
        for (int i = 0; i < n_params; ++i) ptrs[i] = r->bytes.data() + r->params[l.first_param + i].offset;
        l.grid = grid; l.block = block; l.lds_bytes = (unsigned) lds_bytes;
        hipKernelNodeParams kp = {};
        kp.func = const_cast<void *>(func);
        kp.gridDim = grid;
        kp.blockDim = block;
        kp.sharedMemBytes = (unsigned) lds_bytes;
        kp.kernelParams = ptrs;
        kp.extra = nullptr;
        if (hipGraphExecKernelNodeSetParams(r->exec, r->nodes[t_next], &kp) != hipSuccess) {
            (void) hipGetLastError();
            t_differs = true;
            return;
        }
        ++t_patched;
    }
    ++t_next;
}

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
    if (vx_tl_launch_mode != 0) return vx_fail(VX_ERR_INVALID, "vx_graph_begin: this thread is already recording or comparing");
    VX_HIP(hipStreamBeginCapture((hipStream_t) stream, hipStreamCaptureModeThreadLocal));
    t_rec = new recorded_graph;
    vx_tl_launch_mode = 1;
    return VX_OK;
}
vx_status vx_graph_end(vx_stream stream, vx_graph * graph) {
    recorded_graph * r = t_rec;
    t_rec = nullptr;
    if (vx_tl_launch_mode == 1) vx_tl_launch_mode = 0;
    hipGraph_t g = nullptr;
    const hipError_t e = hipStreamEndCapture((hipStream_t) stream, &g); // (whatever follows: the stream must not stay in its capture)
    if (!graph) {
        (void) hipGetLastError();
        if (g) (void) hipGraphDestroy(g);
        destroy_recorded(r);
        return vx_fail(VX_ERR_INVALID, "vx_graph_end: null out pointer");
    }
    *graph = nullptr;
    if (e != hipSuccess || !g) { // an invalidated recording: the stream is usable again, nothing to replay
        (void) hipGetLastError();
        if (g) (void) hipGraphDestroy(g);
        destroy_recorded(r);
        return VX_OK;
    }
    if (!r) r = new recorded_graph;
    r->graph = g;
    const hipError_t e2 = hipGraphInstantiate(&r->exec, g, nullptr, nullptr, 0);
    if (e2 != hipSuccess || !r->exec) {
        (void) hipGetLastError();
        r->exec = nullptr;
        destroy_recorded(r);
        return VX_OK;
    }
    // the graph's nodes against the noted launches: the same count, kernels all, the same functions and grids in the same
    // order (a capture of one stream is a chain, and hipGraphGetNodes lists it in the order of capture; anything else --
    // launches that did not go through vx_launch, another order -- leaves a graph that can be replayed but not patched)
    size_t n = 0;
    bool patchable = !r->launches.empty() && hipGraphGetNodes(g, nullptr, &n) == hipSuccess && n == r->launches.size();
    if (patchable) {
        r->nodes.resize(n);
        patchable = hipGraphGetNodes(g, r->nodes.data(), &n) == hipSuccess && n == r->launches.size();
    }
    for (size_t i = 0; patchable && i < n; ++i) {
        hipGraphNodeType type;
        hipKernelNodeParams kp;
        patchable = hipGraphNodeGetType(r->nodes[i], &type) == hipSuccess && type == hipGraphNodeTypeKernel &&
                    hipGraphKernelNodeGetParams(r->nodes[i], &kp) == hipSuccess && kp.func == r->launches[i].func &&
                    kp.gridDim.x == r->launches[i].grid.x && kp.gridDim.y == r->launches[i].grid.y && kp.gridDim.z == r->launches[i].grid.z;
    }
    if (patchable) patchable = hipEventCreateWithFlags(&r->done, hipEventDisableTiming) == hipSuccess;
    if (!patchable) {
        (void) hipGetLastError();
        r->nodes.clear(); r->launches.clear(); r->params.clear(); r->bytes.clear();
        (void) hipGraphDestroy(r->graph);
        r->graph = nullptr;
    }
    *graph = (vx_graph) r;
    return VX_OK;
}
vx_status vx_graph_launch(vx_graph graph, vx_stream stream) {
    recorded_graph * r = (recorded_graph *) graph;
    if (!r || !r->exec) return vx_fail(VX_ERR_INVALID, "vx_graph_launch: null graph");
    VX_HIP(hipGraphLaunch(r->exec, (hipStream_t) stream));
    if (r->done) {
        VX_HIP(hipEventRecord(r->done, (hipStream_t) stream));
        r->in_flight = true;
    }
    return VX_OK;
}
vx_status vx_graph_destroy(vx_graph graph) {
    recorded_graph * r = (recorded_graph *) graph;
    if (r && r == t_rec) { t_rec = nullptr; vx_tl_launch_mode = 0; }
    if (r && r->in_flight && r->done) (void) hipEventSynchronize(r->done);
    destroy_recorded(r);
    return VX_OK;
}
int vx_graph_patchable(vx_graph graph) {
    const recorded_graph * r = (const recorded_graph *) graph;
    return r && !r->nodes.empty();
}
vx_status vx_graph_patch_begin(vx_graph graph) {
    recorded_graph * r = (recorded_graph *) graph;
    if (!r || r->nodes.empty()) return vx_fail(VX_ERR_UNSUPPORTED, "vx_graph_patch_begin: this recording cannot be compared with");
    if (vx_tl_launch_mode != 0) return vx_fail(VX_ERR_INVALID, "vx_graph_patch_begin: this thread is already recording or comparing");
    if (r->in_flight) { // its last launch may still be reading the arguments that are about to change
        VX_HIP(hipEventSynchronize(r->done));
        r->in_flight = false;
    }
    t_rec = r;
    t_next = 0;
    t_differs = false;
    t_patched = 0;
    vx_tl_launch_mode = 2;
    return VX_OK;
}
vx_status vx_graph_patch_end(vx_graph graph, int * patched) {
    recorded_graph * r = (recorded_graph *) graph;
    if (vx_tl_launch_mode != 2 || r != t_rec) return vx_fail(VX_ERR_INVALID, "vx_graph_patch_end: no comparison with this graph is open");
    vx_tl_launch_mode = 0;
    t_rec = nullptr;
    if (patched) *patched = t_patched;
    if (t_differs || t_next != r->launches.size())
        return vx_fail(VX_ERR_UNSUPPORTED, "vx_graph_patch_end: the launches differ from the recording's (%zu of %zu matched)", t_next, r->launches.size());
    return VX_OK;
}
vx_status vx_weights_pin(const void * base, size_t bytes) {
    if (!base || !bytes) return vx_fail(VX_ERR_INVALID, "vx_weights_pin: empty range");
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    for (const pinned_range & r : g_pinned)
        if (r.dev == dev && r.lo == (uintptr_t) base) {
            if (r.hi == (uintptr_t) base + bytes) return VX_OK;
            return vx_fail(VX_ERR_INVALID, "vx_weights_pin: a range of another size is pinned at this address");
        }
    g_pinned.push_back({ dev, (uintptr_t) base, (uintptr_t) base + bytes });
    return VX_OK;
}
vx_status vx_weights_changed(const void * base, size_t bytes) {
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    if (!g_derived.empty()) drop_derived_from(dev, (uintptr_t) base, (uintptr_t) base + bytes);
    return VX_OK;
}
vx_status vx_weights_unpin(const void * base) {
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    for (size_t i = 0; i < g_pinned.size(); ++i)
        if (g_pinned[i].dev == dev && g_pinned[i].lo == (uintptr_t) base) {
            drop_derived_from(dev, g_pinned[i].lo, g_pinned[i].hi);
            g_pinned[i] = g_pinned.back();
            g_pinned.pop_back();
            return VX_OK;
        }
    return vx_fail(VX_ERR_INVALID, "vx_weights_unpin: no range is pinned at this address");
}
vx_status vx_weights_info(size_t * pinned_ranges, size_t * derived_copies, size_t * derived_bytes) {
    std::lock_guard<std::mutex> lock(g_pin_mutex);
    if (pinned_ranges) *pinned_ranges = g_pinned.size();
    if (derived_copies) *derived_copies = g_derived.size();
    if (derived_bytes) *derived_bytes = g_derived_bytes;
    return VX_OK;
}
vx_status vx_stream_synchronize(vx_stream stream) {
    VX_HIP(hipStreamSynchronize((hipStream_t) stream));
    return VX_OK;
}

} // extern "C"
