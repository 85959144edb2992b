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

// ---- weight placement -----------------------------------------------------------------------------------------------
// A model file loaded the way VoxCPMWeightStore::load_from_file does (gguf_init_from_file with no_alloc, one pass over
// the tensor data, src/weight-store.cpp:58-122), except that the tensors are allocated by the backend's own placement
// helper (reached through ggml_backend_reg_get_proc_address): the transformer stacks' weights in device memory, the
// AudioVAE's in pinned host memory.  Then a graph that uses one weight of each kind -- a Q8_0 projection of the stack
// and the AudioVAE's fc_mu projection + bias + GELU -- runs under ggml_backend_sched over {device, CPU}.
// use_placement = 0: everything in one buffer of `device` (what the reference does).
// flags[0] = splits of the scheduled graph, [1] = stack weight in host memory, [2] = audio_vae weight in host memory,
// [3] = device buffer bytes, [4] = host buffer bytes
int vh_placed_run(const char * gguf_path, const char * device, int use_placement, const char * w_stack, const char * w_vae,
                  const char * b_vae, const float * x, int n_tokens, float * out, int64_t * flags) {
    ggml_context * wctx = nullptr;
    gguf_init_params gp = { true, &wctx };
    gguf_context * gg = gguf_init_from_file(gguf_path, gp);
    if (!gg || !wctx) return fail("gguf_init_from_file failed");
    ggml_backend_dev_t dev = ggml_backend_dev_by_name(device);
    if (!dev) return fail("no such device");
    ggml_backend_t backend = ggml_backend_dev_init(dev, nullptr);
    ggml_backend_t cpu     = ggml_backend_init_by_type(GGML_BACKEND_DEVICE_TYPE_CPU, nullptr);
    if (!backend || !cpu) return fail("backend init failed");
    ggml_backend_cpu_set_n_threads(cpu, 8);
    ggml_backend_buffer_t dbuf = nullptr, hbuf = nullptr;
    int rc = 0;
    if (use_placement) {
        typedef bool (*alloc_fn)(ggml_context *, ggml_backend_t, ggml_backend_buffer_t *, ggml_backend_buffer_t *);
        alloc_fn fn = (alloc_fn) ggml_backend_reg_get_proc_address(ggml_backend_dev_backend_reg(dev), "ggml_backend_gfx950_alloc_weights");
        if (!fn) rc = fail("the backend exports no placement helper");
        else if (!fn(wctx, backend, &dbuf, &hbuf)) rc = fail("placement failed");
    } else {
        dbuf = ggml_backend_alloc_ctx_tensors(wctx, backend);
        if (!dbuf) rc = fail("allocation failed");
        else ggml_backend_buffer_set_usage(dbuf, GGML_BACKEND_BUFFER_USAGE_WEIGHTS);
    }
    if (!rc) { // one pass over the file
        FILE * f = fopen(gguf_path, "rb");
        std::vector<char> tmp;
        const size_t base = gguf_get_data_offset(gg);
        for (int64_t i = 0; f && i < gguf_get_n_tensors(gg); ++i) {
            ggml_tensor * t = ggml_get_tensor(wctx, gguf_get_tensor_name(gg, i));
            tmp.resize(ggml_nbytes(t));
            if (fseek(f, (long) (base + gguf_get_tensor_offset(gg, i)), SEEK_SET) != 0 || fread(tmp.data(), 1, tmp.size(), f) != tmp.size()) { rc = fail("short read"); break; }
            ggml_backend_tensor_set(t, tmp.data(), 0, tmp.size());
        }
        if (f) fclose(f); else rc = fail("cannot open the model file");
    }
    ggml_tensor * ws = rc ? nullptr : ggml_get_tensor(wctx, w_stack);
    ggml_tensor * wv = rc ? nullptr : ggml_get_tensor(wctx, w_vae);
    ggml_tensor * bv = rc ? nullptr : ggml_get_tensor(wctx, b_vae);
    if (!rc && (!ws || !wv || !bv)) rc = fail("tensor not found");
    if (!rc) {
        ggml_init_params ip = { ggml_tensor_overhead() * 32 + ggml_graph_overhead(), nullptr, true };
        ggml_context * c = ggml_init(ip);
        ggml_tensor * inp = ggml_new_tensor_2d(c, GGML_TYPE_F32, ws->ne[0], n_tokens);
        ggml_set_input(inp);
        ggml_tensor * y = ggml_mul_mat(c, ws, inp);                          // the stack's projection: device weight
        ggml_tensor * z = ggml_gelu(c, ggml_add(c, ggml_mul_mat(c, wv, y), bv)); // the AudioVAE side: host weights, GELU is not claimed
        ggml_set_output(z);
        ggml_cgraph * gf = ggml_new_graph(c);
        ggml_build_forward_expand(gf, z);
        ggml_backend_t backs[2] = { backend, cpu };
        const bool same = ggml_backend_dev_type(dev) == GGML_BACKEND_DEVICE_TYPE_CPU;
        ggml_backend_sched_t sched = ggml_backend_sched_new(same ? backs + 1 : backs, nullptr, same ? 1 : 2, 64, false, true);
        if (!sched || !ggml_backend_sched_alloc_graph(sched, gf)) rc = fail("scheduler allocation failed");
        if (!rc) {
            ggml_backend_tensor_set(inp, x, 0, ggml_nbytes(inp));
            if (ggml_backend_sched_graph_compute(sched, gf) != GGML_STATUS_SUCCESS) rc = fail("scheduled compute failed");
        }
        if (!rc) {
            ggml_backend_tensor_get(z, out, 0, ggml_nbytes(z));
            flags[0] = ggml_backend_sched_get_n_splits(sched);
            flags[1] = ggml_backend_buffer_is_host(ws->buffer) ? 1 : 0;
            flags[2] = ggml_backend_buffer_is_host(wv->buffer) ? 1 : 0;
            flags[3] = dbuf ? (int64_t) ggml_backend_buffer_get_size(dbuf) : 0;
            flags[4] = hbuf ? (int64_t) ggml_backend_buffer_get_size(hbuf) : 0;
        }
        if (sched) ggml_backend_sched_free(sched);
        ggml_free(c);
    }
    if (dbuf) ggml_backend_buffer_free(dbuf);
    if (hbuf) ggml_backend_buffer_free(hbuf);
    ggml_backend_free(cpu);
    ggml_backend_free(backend);
    gguf_free(gg);
    ggml_free(wctx);
    return rc;
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
