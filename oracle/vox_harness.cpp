// vox_harness.cpp -- a C-callable driver over the REFERENCE's own module layer: VoxCPMBackend, VoxCPMWeightStore,
// MiniCPMKVCache and MiniCPMModel, compiled from the read-only reference sources where they lie (src/backend.cpp,
// src/weight-store.cpp, src/context.cpp, src/minicpm.cpp, ... -- see oracle/Makefile) into oracle/_ref.
// TEST INFRASTRUCTURE ONLY.
//
// It exists so that the graphs the plugin is validated on are the graphs the reference's own builders emit
// (MiniCPMModel::forward / forward_step, src/minicpm.cpp:779-846), loaded through the reference's own GGUF loader
// (src/weight-store.cpp:58-122), not a restatement of them: a test writes a small synthetic GGUF with ggml's gguf API,
// loads it with VoxCPMWeightStore on ggml-cpu and on the plugin, and runs prefill + decode steps on both.
//
// The reference picks a GPU device by registry name ("cuda" / "vulkan", src/backend.cpp:75-105); the plugin answers to
// such a name when GGML_GFX950_REG_NAME is set, which is how an unpatched VoxCPM build finds it.
#include "voxcpm/backend.h"
#include "voxcpm/context.h"
#include "voxcpm/minicpm.h"
#include "voxcpm/weight-store.h"

#include <ggml-cpu.h>
#include <gguf.h>

#include <chrono>
#include <cstdio>
#include <cstring>
#include <memory>
#include <string>
#include <vector>

using namespace voxcpm;

namespace {

// ---- GGUF writer state
gguf_context * g_w_gguf = nullptr;
ggml_context * g_w_ctx  = nullptr;
std::string    g_w_path;

// ---- model state
std::unique_ptr<VoxCPMBackend>  g_backend;
std::unique_ptr<MiniCPMModel>   g_model;
std::unique_ptr<MiniCPMKVCache> g_cache;
std::shared_ptr<VoxCPMWeightStore> g_store;
std::string g_err;
int g_last_nodes = 0;

int fail(const std::string & what) {
    g_err = what;
    return 1;
}

} // namespace

extern "C" {

const char * vh_last_error(void) { return g_err.c_str(); }

// ---- writing a synthetic model file with the reference's gguf API (ggml/src/gguf.cpp) ----------------------------
int vh_gguf_begin(const char * path, size_t ctx_bytes) {
    if (g_w_gguf) return fail("a GGUF is already being written");
    ggml_init_params ip = { ctx_bytes, nullptr, false };
    g_w_ctx = ggml_init(ip);
    if (!g_w_ctx) return fail("ggml_init failed");
    g_w_gguf = gguf_init_empty();
    g_w_path = path;
    return 0;
}
int vh_gguf_u32(const char * key, uint32_t v) { if (!g_w_gguf) return 1; gguf_set_val_u32(g_w_gguf, key, v); return 0; }
int vh_gguf_f32(const char * key, float v) { if (!g_w_gguf) return 1; gguf_set_val_f32(g_w_gguf, key, v); return 0; }
int vh_gguf_str(const char * key, const char * v) { if (!g_w_gguf) return 1; gguf_set_val_str(g_w_gguf, key, v); return 0; }
int vh_gguf_f32_array(const char * key, const float * v, int n) {
    if (!g_w_gguf) return 1;
    gguf_set_arr_data(g_w_gguf, key, GGUF_TYPE_FLOAT32, v, (size_t) n);
    return 0;
}
// data: the tensor's bytes in ggml layout (Q8_0 rows as 34-byte blocks)
int vh_gguf_tensor(const char * name, int type, int64_t ne0, int64_t ne1, const void * data, size_t nbytes) {
    if (!g_w_gguf) return 1;
    ggml_tensor * t = ne1 > 0 ? ggml_new_tensor_2d(g_w_ctx, (ggml_type) type, ne0, ne1) : ggml_new_tensor_1d(g_w_ctx, (ggml_type) type, ne0);
    if (!t) return fail(std::string("out of context memory at ") + name);
    if (ggml_nbytes(t) != nbytes) return fail(std::string("size mismatch for ") + name);
    ggml_set_name(t, name);
    memcpy(t->data, data, nbytes);
    gguf_add_tensor(g_w_gguf, t);
    return 0;
}
int vh_gguf_end(void) {
    if (!g_w_gguf) return 1;
    const bool ok = gguf_write_to_file(g_w_gguf, g_w_path.c_str(), false);
    gguf_free(g_w_gguf);
    ggml_free(g_w_ctx);
    g_w_gguf = nullptr;
    g_w_ctx  = nullptr;
    return ok ? 0 : fail("gguf_write_to_file failed");
}

// ---- the reference's module layer ---------------------------------------------------------------------------------
int vh_load_plugin(const char * path) { return ggml_backend_load(path) ? 0 : 1; }

void vh_close(void) {
    g_cache.reset();
    g_model.reset();
    g_store.reset();
    g_backend.reset();
}

// backend: 0 = BackendType::CPU with n_threads, 1 = BackendType::CUDA (the reference's GPU selection, by registry name)
int vh_open(int backend, int n_threads) {
    vh_close();
    try {
        g_backend = std::make_unique<VoxCPMBackend>(backend == 0 ? BackendType::CPU : BackendType::CUDA, n_threads);
    } catch (const std::exception & e) {
        return fail(e.what());
    }
    return 0;
}

const char * vh_backend_name(void) { return g_backend ? ggml_backend_name(g_backend->raw_backend()) : ""; }
int vh_backend_is_gpu(void) { return g_backend && g_backend->is_gpu() ? 1 : 0; }

// VoxCPMWeightStore::load_from_file + MiniCPMModel::load_from_store for `prefix` ("", "residual_lm", "locdit", ...),
// and a KV cache of max_length positions
int vh_minicpm_load(const char * gguf_path, const char * prefix, int max_length) {
    if (!g_backend) return fail("no backend");
    try {
        g_store = std::make_shared<VoxCPMWeightStore>();
        if (!g_store->load_from_file(gguf_path, *g_backend)) return fail("VoxCPMWeightStore::load_from_file failed");
        g_model = std::make_unique<MiniCPMModel>();
        if (!g_model->load_from_store(g_store, prefix, *g_backend)) return fail("MiniCPMModel::load_from_store failed");
        const MiniCPMConfig & c = g_model->config();
        g_cache = std::make_unique<MiniCPMKVCache>(c.n_layer, c.n_kv_heads, max_length, c.head_dim());
        g_cache->init(*g_backend);
        g_cache->clear();
    } catch (const std::exception & e) {
        return fail(e.what());
    }
    return 0;
}

int vh_weights_on_host(void) { return g_store && g_store->buffer() && ggml_backend_buffer_is_host(g_store->buffer()) ? 1 : 0; }
size_t vh_weight_bytes(void) { return g_store ? g_store->buffer_size() : 0; }
int vh_n_layer(void) { return g_model ? g_model->config().n_layer : 0; }
int vh_last_graph_nodes(void) { return g_last_nodes; }

// MiniCPMModel::forward (n_tokens > 1 or position < 0: a prefill from position 0, causal, writing the cache) or
// MiniCPMModel::forward_step (one token at `position`).  x: [hidden, n_tokens] F32; out the same shape.
// seconds (may be NULL): wall time of the backend's compute call(s), mean over `reps` further runs when reps > 0.
int vh_minicpm_run(const float * x, int n_tokens, int position, float * out, int reps, double * seconds) {
    if (!g_model || !g_cache || !g_backend) return fail("no model");
    try {
        const MiniCPMConfig & c = g_model->config();
        VoxCPMContext graph_ctx(ContextType::Graph, 8192, 65536);
        ggml_tensor * input = graph_ctx.new_tensor_2d(GGML_TYPE_F32, c.hidden_size, n_tokens);
        ggml_set_input(input);
        ggml_tensor * output = position < 0 ? g_model->forward(graph_ctx, input, nullptr, *g_cache, true, true)
                                            : g_model->forward_step(graph_ctx, input, position, *g_cache, true, true);
        if (!output) return fail("graph construction failed");
        ggml_set_output(output);
        ggml_cgraph * graph = graph_ctx.new_graph();
        graph_ctx.build_forward(graph, output);
        g_last_nodes = ggml_graph_n_nodes(graph);
        g_backend->alloc_graph(graph);
        g_backend->tensor_set(input, x, 0, ggml_nbytes(input));
        auto t0 = std::chrono::steady_clock::now();
        if (g_backend->compute(graph) != GGML_STATUS_SUCCESS) return fail("compute failed");
        double dt = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (reps > 0) { // the allocator hands an input's memory on once its readers have run: set it again before every run
            dt = 0.0;
            for (int r = 0; r < reps; ++r) {
                g_backend->tensor_set(input, x, 0, ggml_nbytes(input));
                t0 = std::chrono::steady_clock::now();
                if (g_backend->compute(graph) != GGML_STATUS_SUCCESS) return fail("compute failed");
                dt += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
            }
            dt /= reps;
        }
        if (seconds) *seconds = dt;
        g_backend->tensor_get(output, out, 0, ggml_nbytes(output));
    } catch (const std::exception & e) {
        return fail(e.what());
    }
    return 0;
}

// one layer's K (which = 0) or V (1) cache as the reference allocated it: [head_dim, max_length, n_kv_heads] F32
int vh_cache_get(int layer, int which, float * out, size_t nbytes) {
    if (!g_cache || !g_backend) return 1;
    ggml_tensor * t = which == 0 ? g_cache->raw_k_cache(layer) : g_cache->raw_v_cache(layer);
    if (ggml_nbytes(t) != nbytes) return fail("cache size mismatch");
    g_backend->tensor_get(t, out, 0, nbytes);
    return 0;
}

} // extern "C"
