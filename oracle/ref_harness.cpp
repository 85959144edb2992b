// ref_harness.cpp -- a thin C-callable driver over the REFERENCE's own ggml library
// (built from the read-only reference checkout into oracle/_ref by oracle/Makefile).
// TEST INFRASTRUCTURE ONLY: it exists so that tests, the smoke test and the benchmark's
// cpu_baseline leg can run one ggml op (or a small graph) on ggml-cpu -- or on any ggml
// backend plugin loaded through ggml's registry -- from host arrays, and time it.
//
// Every op goes through ggml's public API exactly as VoxCPM.cpp's graph builders do
// (ggml_mul_mat / ggml_rope_ext / ggml_rms_norm / ggml_soft_max_ext / ggml_flash_attn_ext,
// src/minicpm.cpp:572-716), is allocated with ggml_backend_alloc_ctx_tensors, uploaded with
// ggml_backend_tensor_set and run with ggml_backend_graph_compute, so a plugin backend is
// exercised through the same buffer/stream vtables a real host uses.
#include <ggml.h>
#include <ggml-alloc.h>
#include <ggml-backend.h>
#include <ggml-cpu.h>

#include <chrono>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

extern "C" {

// same layout as orc_tensor (oracle/oracle.h) and vx_tensor (include/voxcpm_gfx950.h)
struct rh_tensor {
    int32_t  type;
    int32_t  _pad;
    int64_t  ne[4];
    uint64_t nb[4];
    void *   data;
};

} // extern "C"

namespace {

ggml_backend_t g_backend = nullptr;
std::string    g_backend_name;

size_t row_bytes(ggml_type type, int64_t ne0) { return ggml_row_size(type, ne0); }

size_t span_bytes(const rh_tensor * t) {
    size_t s = row_bytes((ggml_type) t->type, t->ne[0]);
    for (int i = 1; i < 4; ++i) s += (size_t) (t->ne[i] - 1) * t->nb[i];
    return s;
}

struct op_graph {
    ggml_context * ctx = nullptr;
    ggml_backend_buffer_t buf = nullptr;
    std::vector<std::pair<ggml_tensor *, const rh_tensor *>> uploads;

    op_graph() {
        ggml_init_params ip = { ggml_tensor_overhead() * 64 + ggml_graph_overhead(), nullptr, true };
        ctx = ggml_init(ip);
    }
    ~op_graph() {
        if (buf) ggml_backend_buffer_free(buf);
        if (ctx) ggml_free(ctx);
    }
    // a tensor of the caller's type/shape/strides laid over a byte buffer that holds the
    // caller's memory span verbatim
    ggml_tensor * input(const rh_tensor * t) {
        if (!t) return nullptr;
        ggml_tensor * base = ggml_new_tensor_1d(ctx, GGML_TYPE_I8, (int64_t) span_bytes(t));
        ggml_tensor * view = ggml_new_tensor_4d(ctx, (ggml_type) t->type, t->ne[0], t->ne[1], t->ne[2], t->ne[3]);
        for (int i = 0; i < 4; ++i) view->nb[i] = t->nb[i];
        view->view_src  = base;
        view->view_offs = 0;
        uploads.push_back({ base, t });
        return view;
    }
    int run(ggml_tensor * out, const rh_tensor * dst, int reps, double * seconds) {
        if (!g_backend) return 100;
        ggml_cgraph * gf = ggml_new_graph(ctx);
        ggml_build_forward_expand(gf, out);
        buf = ggml_backend_alloc_ctx_tensors(ctx, g_backend);
        if (!buf) return 101;
        for (auto & u : uploads) ggml_backend_tensor_set(u.first, u.second->data, 0, ggml_nbytes(u.first));
        if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) return 102;
        if (reps > 0 && seconds) {
            double best = 1e30, total = 0;
            for (int r = 0; r < reps; ++r) {
                auto t0 = std::chrono::steady_clock::now();
                if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) return 102;
                auto t1 = std::chrono::steady_clock::now();
                const double dt = std::chrono::duration<double>(t1 - t0).count();
                total += dt;
                if (dt < best) best = dt;
            }
            seconds[0] = total / reps;
            seconds[1] = best;
        }
        // dst must be dense in the result's own layout
        if (ggml_nbytes(out) != span_bytes(dst)) return 103;
        ggml_backend_tensor_get(out, dst->data, 0, ggml_nbytes(out));
        return 0;
    }
};

} // namespace

extern "C" {

// ---- backend selection ------------------------------------------------------------
int rh_load_plugin(const char * path) { return ggml_backend_load(path) ? 0 : 1; }

int rh_device_count(void) { return (int) ggml_backend_dev_count(); }

const char * rh_device_name(int i) {
    ggml_backend_dev_t dev = ggml_backend_dev_get((size_t) i);
    return dev ? ggml_backend_dev_name(dev) : "";
}

// name: a registry device name ("CPU", "GFX950_0", ...).  n_threads / use_ref apply to CPU.
int rh_use_device(const char * name, int n_threads, int use_ref) {
    if (g_backend) {
        ggml_backend_free(g_backend);
        g_backend = nullptr;
    }
    ggml_backend_dev_t dev = ggml_backend_dev_by_name(name);
    if (!dev) return 1;
    g_backend = ggml_backend_dev_init(dev, nullptr);
    if (!g_backend) return 2;
    g_backend_name = name;
    if (ggml_backend_dev_type(dev) == GGML_BACKEND_DEVICE_TYPE_CPU) {
        ggml_backend_cpu_set_n_threads(g_backend, n_threads > 0 ? n_threads : 1);
        ggml_backend_cpu_set_use_ref(g_backend, use_ref != 0);
    }
    return 0;
}

void rh_release(void) {
    if (g_backend) ggml_backend_free(g_backend);
    g_backend = nullptr;
}

// ---- conversions / quantization ------------------------------------------------------
void rh_fp32_to_fp16_row(const float * x, uint16_t * y, int64_t n) { ggml_fp32_to_fp16_row(x, (ggml_fp16_t *) y, n); }
void rh_fp16_to_fp32_row(const uint16_t * x, float * y, int64_t n) { ggml_fp16_to_fp32_row((const ggml_fp16_t *) x, y, n); }

// ggml_quantize_chunk(Q8_0) == quantize_row_q8_0_ref per row (ggml/src/ggml-quants.c:199-222)
size_t rh_quantize_q8_0(const float * x, void * y, int64_t nrows, int64_t n_per_row) {
    return ggml_quantize_chunk(GGML_TYPE_Q8_0, x, y, 0, nrows, n_per_row, nullptr);
}
void rh_dequantize_q8_0(const void * x, float * y, int64_t k) {
    ggml_get_type_traits(GGML_TYPE_Q8_0)->to_float(x, y, k);
}
// the activation quantizer ggml-cpu's MUL_MAT applies to src1 rows (x86 build)
void rh_quantize_q8_0_cpu(const float * x, void * y, int64_t k) {
    ggml_get_type_traits_cpu(GGML_TYPE_Q8_0)->from_float(x, y, k);
}
float rh_vec_dot_q8_0_q8_0(int64_t n, const void * x, const void * y) {
    float s = 0;
    ggml_get_type_traits_cpu(GGML_TYPE_Q8_0)->vec_dot((int) n, &s, 0, x, 0, y, 0, 1);
    return s;
}

// ---- single ops ------------------------------------------------------------------------
int rh_mul_mat(const rh_tensor * src0, const rh_tensor * src1, const rh_tensor * dst, int reps, double * seconds) {
    op_graph g;
    ggml_tensor * a = g.input(src0);
    ggml_tensor * b = g.input(src1);
    return g.run(ggml_mul_mat(g.ctx, a, b), dst, reps, seconds);
}

int rh_rms_norm(const rh_tensor * src, const rh_tensor * dst, float eps, int reps, double * seconds) {
    op_graph g;
    return g.run(ggml_rms_norm(g.ctx, g.input(src), eps), dst, reps, seconds);
}

int rh_rope(const rh_tensor * src, const int32_t * pos, const float * freq_factors, const rh_tensor * dst,
            int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor,
            float attn_factor, float beta_fast, float beta_slow, int reps, double * seconds) {
    op_graph g;
    const int64_t np = src->ne[2];
    rh_tensor tp = { GGML_TYPE_I32, 0, { np, 1, 1, 1 }, { 4, (uint64_t) np * 4, (uint64_t) np * 4, (uint64_t) np * 4 }, (void *) pos };
    const int64_t nf = n_dims / 2;
    rh_tensor tf = { GGML_TYPE_F32, 0, { nf, 1, 1, 1 }, { 4, (uint64_t) nf * 4, (uint64_t) nf * 4, (uint64_t) nf * 4 }, (void *) freq_factors };
    ggml_tensor * a = g.input(src);
    ggml_tensor * p = g.input(&tp);
    ggml_tensor * f = freq_factors ? g.input(&tf) : nullptr;
    ggml_tensor * out = ggml_rope_ext(g.ctx, a, p, f, n_dims, mode, n_ctx_orig, freq_base, freq_scale,
                                      ext_factor, attn_factor, beta_fast, beta_slow);
    return g.run(out, dst, reps, seconds);
}

int rh_soft_max(const rh_tensor * src, const rh_tensor * mask, const float * sinks, const rh_tensor * dst,
                float scale, float max_bias, int reps, double * seconds) {
    op_graph g;
    const int64_t nh = src->ne[2];
    rh_tensor ts = { GGML_TYPE_F32, 0, { nh, 1, 1, 1 }, { 4, (uint64_t) nh * 4, (uint64_t) nh * 4, (uint64_t) nh * 4 }, (void *) sinks };
    ggml_tensor * a = g.input(src);
    ggml_tensor * m = g.input(mask);
    ggml_tensor * out = ggml_soft_max_ext(g.ctx, a, m, scale, max_bias);
    if (sinks) ggml_soft_max_add_sinks(out, g.input(&ts));
    return g.run(out, dst, reps, seconds);
}

int rh_flash_attn_ext(const rh_tensor * q, const rh_tensor * k, const rh_tensor * v, const rh_tensor * mask,
                      const float * sinks, const rh_tensor * dst, float scale, float max_bias,
                      float logit_softcap, int reps, double * seconds) {
    op_graph g;
    const int64_t nh = q->ne[2];
    rh_tensor ts = { GGML_TYPE_F32, 0, { nh, 1, 1, 1 }, { 4, (uint64_t) nh * 4, (uint64_t) nh * 4, (uint64_t) nh * 4 }, (void *) sinks };
    ggml_tensor * tq = g.input(q);
    ggml_tensor * tk = g.input(k);
    ggml_tensor * tv = g.input(v);
    ggml_tensor * tm = g.input(mask);
    ggml_tensor * out = ggml_flash_attn_ext(g.ctx, tq, tk, tv, tm, scale, max_bias, logit_softcap);
    if (sinks) ggml_flash_attn_ext_add_sinks(out, g.input(&ts));
    return g.run(out, dst, reps, seconds);
}

} // extern "C"
