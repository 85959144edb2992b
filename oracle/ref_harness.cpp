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
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
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
bool g_out_after_reps = false; // fetch the result after the timed repeats instead of after the first run
std::vector<double> g_last_times; // seconds of every timed repeat of the most recent timed run (rh_last_times)

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
            g_last_times.clear();
            for (int r = 0; r < reps; ++r) {
                auto t0 = std::chrono::steady_clock::now();
                if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) return 102;
                auto t1 = std::chrono::steady_clock::now();
                const double dt = std::chrono::duration<double>(t1 - t0).count();
                g_last_times.push_back(dt);
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

// the seconds of each timed repeat of the most recent run that was given reps > 0; returns how many there are
void rh_out_after_reps(int on) { g_out_after_reps = on != 0; }
int rh_last_times(double * out, int max) {
    const int n = (int) g_last_times.size();
    for (int i = 0; i < n && i < max; ++i) out[i] = g_last_times[(size_t) i];
    return n;
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

// ---- MiniCPM backbone --------------------------------------------------------------------
// The decoder stack as the reference builds it (src/minicpm.cpp:572-846: rms_norm*weight,
// separate Q/K/V projections, NEOX rope with frequency factors, KV append through ggml_cpy into
// the cache's write view plus the sum*0 ordering trick, concat(past view, current), flash
// attention, output projection, muP residual scale, SwiGLU MLP), on whichever backend
// rh_use_device selected.  Independent sequences ride in ne[3] (batch); batch 1 is the
// reference's graph node for node.  Weights are Q8_0; norms, rope factors F32.
namespace {

struct bb_layer {
    ggml_tensor * w[7];       // q k v o gate up down
    ggml_tensor * ln[2];      // input_layernorm, post_layernorm
    ggml_tensor * kc, * vc;   // [D, max_len, Hkv, B]
    ggml_tensor * qkv = nullptr, * gate_up = nullptr; // row-fused copies (rh_bb_fuse_weights), as the reference makes for LocDiT
};

struct backbone {
    int n_layer, hidden, n_heads, n_kv, head_dim, ffn, max_len, batch;
    float eps, residual_scale;
    bool  use_mup, fused_glu;
    ggml_context *        wctx = nullptr;
    ggml_backend_buffer_t wbuf = nullptr;
    ggml_context *        cctx = nullptr; // the KV cache: a buffer of its own, as MiniCPMKVCache allocates it (src/minicpm.cpp:178-187)
    ggml_backend_buffer_t cbuf = nullptr;
    ggml_context *        fctx = nullptr;
    ggml_backend_buffer_t fbuf = nullptr;
    std::vector<bb_layer> layers;
    ggml_tensor *         final_norm = nullptr;
    ggml_tensor *         rope_factors = nullptr;
};

backbone * g_bb = nullptr;
// Test switches (rh_bb_options): run the stack through ggml_backend_sched over {device, CPU} instead of a direct
// graph_compute, and add per layer a small term computed by an operator no accelerator plugin here claims (GELU of
// the normalised hidden state), so that the scheduler cuts the graph and a value in the middle of the device's part
// is also read from the CPU's part.
bool g_bb_sched = false, g_bb_probe = false, g_bb_whole = false;

ggml_tensor * bb_norm(ggml_context * c, const backbone & m, ggml_tensor * x, ggml_tensor * w) {
    return ggml_mul(c, ggml_rms_norm(c, x, m.eps), w);
}

ggml_tensor * bb_rope(ggml_context * c, const backbone & m, ggml_tensor * x, ggml_tensor * pos) {
    return ggml_rope_ext(c, x, pos, m.rope_factors, m.head_dim, GGML_ROPE_TYPE_NEOX, 32768, 10000.0f, 1.0f, 0.0f, 1.0f, 32.0f, 1.0f);
}

ggml_tensor * bb_layer_forward(ggml_context * c, const backbone & m, const bb_layer & L, ggml_tensor * x, ggml_tensor * pos,
                               ggml_tensor * mask, int T, int n_past, bool write_kv, std::vector<ggml_tensor *> & roots) {
    const int D = m.head_dim, B = m.batch;
    ggml_tensor * cur = bb_norm(c, m, x, L.ln[0]);
    ggml_tensor * q, * k, * v;
    if (L.qkv) { // one product, three strided views of it (src/minicpm.cpp:644-668)
        ggml_tensor * qkv = ggml_mul_mat(c, L.qkv, cur);
        const size_t  es = qkv->nb[0], qrows = (size_t) m.n_heads * D, krows = (size_t) m.n_kv * D;
        q = ggml_view_4d(c, qkv, D, m.n_heads, T, B, D * es, qkv->nb[1], (size_t) T * qkv->nb[1], 0);
        k = ggml_view_4d(c, qkv, D, m.n_kv, T, B, D * es, qkv->nb[1], (size_t) T * qkv->nb[1], qrows * es);
        v = ggml_view_4d(c, qkv, D, m.n_kv, T, B, D * es, qkv->nb[1], (size_t) T * qkv->nb[1], (qrows + krows) * es);
    } else {
        q = ggml_reshape_4d(c, ggml_mul_mat(c, L.w[0], cur), D, m.n_heads, T, B);
        k = ggml_reshape_4d(c, ggml_mul_mat(c, L.w[1], cur), D, m.n_kv, T, B);
        v = ggml_reshape_4d(c, ggml_mul_mat(c, L.w[2], cur), D, m.n_kv, T, B);
    }
    q = bb_rope(c, m, q, pos);
    k = bb_rope(c, m, k, pos);

    ggml_tensor * kv_sync = nullptr;
    if (write_kv) {
        auto write_view = [&](ggml_tensor * cache) {
            return ggml_view_4d(c, cache, D, m.n_kv, T, B, cache->nb[2], cache->nb[1], cache->nb[3], (size_t) n_past * cache->nb[1]);
        };
        ggml_tensor * kw = ggml_cpy(c, k, write_view(L.kc));
        ggml_tensor * vw = ggml_cpy(c, v, write_view(L.vc));
        if (L.kc->type == GGML_TYPE_F32) {
            kv_sync = ggml_add(c, ggml_sum(c, ggml_cont(c, kw)), ggml_sum(c, ggml_cont(c, vw)));
        } else { // an F16 cache: SCALE and ADD1 are F32 operators in ggml, so the written slots are read back as F32 for the sums
            kv_sync = ggml_add(c, ggml_sum(c, ggml_cast(c, kw, GGML_TYPE_F32)), ggml_sum(c, ggml_cast(c, vw, GGML_TYPE_F32)));
        }
        kv_sync = ggml_scale(c, kv_sync, 0.0f);
        (void) roots;
    }
    ggml_tensor * k_all = ggml_permute(c, k, 0, 2, 1, 3);
    ggml_tensor * v_all = ggml_permute(c, v, 0, 2, 1, 3);
    if (n_past > 0) {
        auto past_view = [&](ggml_tensor * cache) {
            return ggml_view_4d(c, cache, D, n_past, m.n_kv, B, cache->nb[1], cache->nb[2], cache->nb[3], 0);
        };
        if (L.kc->type != GGML_TYPE_F32) { // an F16 cache: concat needs one type
            k_all = ggml_cast(c, k_all, L.kc->type);
            v_all = ggml_cast(c, v_all, L.vc->type);
        }
        k_all = ggml_concat(c, past_view(L.kc), k_all, 1);
        v_all = ggml_concat(c, past_view(L.vc), v_all, 1);
    }
    q = ggml_permute(c, q, 0, 2, 1, 3);
    ggml_tensor * attn = ggml_flash_attn_ext(c, q, k_all, v_all, mask, 1.0f / sqrtf((float) D), 0.0f, 0.0f);
    if (kv_sync) attn = ggml_add1(c, attn, kv_sync);
    attn = ggml_reshape_2d(c, attn, (int64_t) m.n_heads * D, (int64_t) T * B);
    ggml_tensor * attn_out = ggml_mul_mat(c, L.w[3], attn);
    if (m.use_mup) attn_out = ggml_scale(c, attn_out, m.residual_scale);
    ggml_tensor * h = ggml_add(c, x, attn_out);

    cur = bb_norm(c, m, h, L.ln[1]);
    ggml_tensor * gate, * up;
    bool glu = m.fused_glu;
    if (L.gate_up) { // one product, two views of it, always the fused GLU (src/minicpm.cpp:724-731)
        ggml_tensor * gu = ggml_mul_mat(c, L.gate_up, cur);
        gate = ggml_view_2d(c, gu, m.ffn, gu->ne[1], gu->nb[1], 0);
        up   = ggml_view_2d(c, gu, m.ffn, gu->ne[1], gu->nb[1], (size_t) m.ffn * gu->nb[0]);
        glu  = true;
    } else {
        gate = ggml_mul_mat(c, L.w[4], cur);
        up   = ggml_mul_mat(c, L.w[5], cur);
    }
    ggml_tensor * act  = glu ? ggml_swiglu_split(c, gate, up) : ggml_mul(c, ggml_silu(c, gate), up);
    ggml_tensor * down = ggml_mul_mat(c, L.w[6], act);
    if (m.use_mup) down = ggml_scale(c, down, m.residual_scale);
    ggml_tensor * res = ggml_add(c, h, down);
    if (g_bb_probe) res = ggml_add(c, res, ggml_scale(c, ggml_gelu(c, cur), 1e-2f)); // cur: the post-attention normalised state
    return res;
}

} // namespace

extern "C" {

void rh_bb_free(void) {
    if (!g_bb) return;
    if (g_bb->fbuf) ggml_backend_buffer_free(g_bb->fbuf);
    if (g_bb->fctx) ggml_free(g_bb->fctx);
    if (g_bb->cbuf) ggml_backend_buffer_free(g_bb->cbuf);
    if (g_bb->cctx) ggml_free(g_bb->cctx);
    if (g_bb->wbuf) ggml_backend_buffer_free(g_bb->wbuf);
    if (g_bb->wctx) ggml_free(g_bb->wctx);
    delete g_bb;
    g_bb = nullptr;
}

// kv_type: GGML_TYPE_F32 (0, the reference's cache, src/minicpm.cpp:182-183) or GGML_TYPE_F16 (1)
int rh_bb_create(int n_layer, int hidden, int n_heads, int n_kv, int head_dim, int ffn, int max_len, int batch,
                 float eps, int use_mup, float scale_depth, int kv_type) {
    if (!g_backend) return 100;
    rh_bb_free();
    backbone * m = new backbone;
    m->n_layer = n_layer; m->hidden = hidden; m->n_heads = n_heads; m->n_kv = n_kv; m->head_dim = head_dim;
    m->ffn = ffn; m->max_len = max_len; m->batch = batch; m->eps = eps; m->use_mup = use_mup != 0;
    m->residual_scale = use_mup ? scale_depth / sqrtf((float) (n_layer > 0 ? n_layer : 1)) : 1.0f;
    ggml_init_params ip = { ggml_tensor_overhead() * ((size_t) n_layer * 11 + 4), nullptr, true };
    m->wctx = ggml_init(ip);
    m->cctx = ggml_init(ip);
    const int64_t qd = (int64_t) n_heads * head_dim, kd = (int64_t) n_kv * head_dim;
    const int64_t shapes[7][2] = { { hidden, qd }, { hidden, kd }, { hidden, kd }, { qd, hidden }, { hidden, ffn }, { hidden, ffn }, { ffn, hidden } };
    m->layers.resize((size_t) n_layer);
    for (auto & L : m->layers) {
        for (int i = 0; i < 7; ++i) L.w[i] = ggml_new_tensor_2d(m->wctx, GGML_TYPE_Q8_0, shapes[i][0], shapes[i][1]);
        for (int i = 0; i < 2; ++i) L.ln[i] = ggml_new_tensor_1d(m->wctx, GGML_TYPE_F32, hidden);
        L.kc = ggml_new_tensor_4d(m->cctx, (ggml_type) kv_type, head_dim, max_len, n_kv, batch);
        L.vc = ggml_new_tensor_4d(m->cctx, (ggml_type) kv_type, head_dim, max_len, n_kv, batch);
    }
    m->final_norm   = ggml_new_tensor_1d(m->wctx, GGML_TYPE_F32, hidden);
    m->rope_factors = ggml_new_tensor_1d(m->wctx, GGML_TYPE_F32, head_dim / 2);
    m->wbuf = ggml_backend_alloc_ctx_tensors(m->wctx, g_backend);
    m->cbuf = ggml_backend_alloc_ctx_tensors(m->cctx, g_backend);
    if (!m->wbuf || !m->cbuf) { g_bb = m; rh_bb_free(); return 101; }
    ggml_backend_buffer_set_usage(m->wbuf, GGML_BACKEND_BUFFER_USAGE_WEIGHTS); // src/weight-store.cpp:86
    ggml_backend_buffer_clear(m->wbuf, 0);
    ggml_backend_buffer_clear(m->cbuf, 0);
    // mlp_forward fuses SwiGLU when the weights are not in host memory (src/minicpm.cpp:729-745)
    m->fused_glu = !ggml_backend_buffer_is_host(m->wbuf);
    g_bb = m;
    return 0;
}

void rh_bb_options(int use_sched, int probe) {
    g_bb_sched = use_sched != 0;
    g_bb_probe = probe != 0;
}

// When on, the graph also holds what the reference puts around the decoder stack: the causal mask is built from
// the position ids by the node chain of MiniCPMModel::create_causal_mask (src/minicpm.cpp:602-620: ARANGE, CAST,
// REPEAT x2, SUB, ADD1, STEP, SCALE, CAST + CONT) instead of being handed in, and the input rows go through a
// GET_ROWS (the embedding lookup of src/components.cpp:223, here over the input matrix with identity ids).
void rh_bb_whole_graph(int on) { g_bb_whole = on != 0; }

// Row-fused weight copies, as MiniCPMModel::load_from_store makes them for the LocDiT decoder on a GPU backend
// (src/minicpm.cpp:427-492): qkv_proj = rows of q, k, v; gate_up_proj = rows of gate, up.  Call after rh_bb_set.
int rh_bb_fuse_weights(void) {
    if (!g_bb || !g_backend || g_bb->fctx) return 100;
    backbone & m = *g_bb;
    ggml_init_params ip = { ggml_tensor_overhead() * ((size_t) m.n_layer * 2 + 2), nullptr, true };
    m.fctx = ggml_init(ip);
    for (auto & L : m.layers) {
        L.qkv     = ggml_new_tensor_2d(m.fctx, L.w[0]->type, L.w[0]->ne[0], L.w[0]->ne[1] + L.w[1]->ne[1] + L.w[2]->ne[1]);
        L.gate_up = ggml_new_tensor_2d(m.fctx, L.w[4]->type, L.w[4]->ne[0], L.w[4]->ne[1] + L.w[5]->ne[1]);
    }
    m.fbuf = ggml_backend_alloc_ctx_tensors(m.fctx, g_backend);
    if (!m.fbuf) return 101;
    ggml_backend_buffer_set_usage(m.fbuf, GGML_BACKEND_BUFFER_USAGE_WEIGHTS); // src/minicpm.cpp:472
    std::vector<uint8_t> scratch;
    auto copy_rows = [&](ggml_tensor * src, ggml_tensor * dst, int64_t row0) {
        scratch.resize(ggml_nbytes(src));
        ggml_backend_tensor_get(src, scratch.data(), 0, scratch.size());
        ggml_backend_tensor_set(dst, scratch.data(), (size_t) row0 * dst->nb[1], scratch.size());
    };
    for (auto & L : m.layers) {
        copy_rows(L.w[0], L.qkv, 0);
        copy_rows(L.w[1], L.qkv, L.w[0]->ne[1]);
        copy_rows(L.w[2], L.qkv, L.w[0]->ne[1] + L.w[1]->ne[1]);
        copy_rows(L.w[4], L.gate_up, 0);
        copy_rows(L.w[5], L.gate_up, L.w[4]->ne[1]);
    }
    return 0;
}

// which: 0..6 = q k v o gate up down (Q8_0 rows), 7 = input_layernorm, 8 = post_layernorm;
// layer -1: which 0 = final norm, 1 = rope frequency factors
int rh_bb_set(int layer, int which, const void * data, size_t nbytes) {
    if (!g_bb) return 100;
    ggml_tensor * t = nullptr;
    if (layer < 0) t = which == 0 ? g_bb->final_norm : g_bb->rope_factors;
    else if (layer < g_bb->n_layer) t = which < 7 ? g_bb->layers[(size_t) layer].w[which] : g_bb->layers[(size_t) layer].ln[which - 7];
    if (!t || ggml_nbytes(t) != nbytes) return 101;
    ggml_backend_tensor_set(t, data, 0, nbytes);
    return 0;
}

// Fills (or reads back) one layer's K (which = 0) or V (which = 1) cache, the whole tensor [head_dim, max_len, n_kv, batch]
// in the cache's own type: lets a test start a decode step from a long seeded past without running the prefill.
int rh_bb_cache_set(int layer, int which, const void * data, size_t nbytes) {
    if (!g_bb || layer < 0 || layer >= g_bb->n_layer) return 100;
    ggml_tensor * t = which == 0 ? g_bb->layers[(size_t) layer].kc : g_bb->layers[(size_t) layer].vc;
    if (ggml_nbytes(t) != nbytes) return 101;
    ggml_backend_tensor_set(t, data, 0, nbytes);
    return 0;
}
int rh_bb_cache_get(int layer, int which, void * data, size_t nbytes) {
    if (!g_bb || layer < 0 || layer >= g_bb->n_layer) return 100;
    ggml_tensor * t = which == 0 ? g_bb->layers[(size_t) layer].kc : g_bb->layers[(size_t) layer].vc;
    if (ggml_nbytes(t) != nbytes) return 101;
    ggml_backend_tensor_get(t, data, 0, nbytes);
    return 0;
}

// x: [hidden, n_tokens, batch] F32 (dense); mask: F16 [n_past + n_tokens, n_tokens] or NULL;
// out: [hidden, n_tokens, batch] after the final norm.  Graph and compute buffer are rebuilt on
// every call, as the reference does per step (src/voxcpm.cpp:489-495); only the graph_compute
// calls are timed.
int rh_bb_forward(const float * x, const uint16_t * mask, int n_tokens, int n_past, int write_kv, float * out,
                  int reps, double * seconds) {
    if (!g_bb || !g_backend) return 100;
    const backbone & m = *g_bb;
    const int T = n_tokens, B = m.batch;
    if (n_past + T > m.max_len) return 104;
    const size_t n_nodes = (size_t) m.n_layer * 64 + 64;
    ggml_init_params ip = { ggml_tensor_overhead() * n_nodes + ggml_graph_overhead_custom(n_nodes, false), nullptr, true };
    ggml_context * c = ggml_init(ip);
    ggml_tensor * inp = ggml_new_tensor_2d(c, GGML_TYPE_F32, m.hidden, (int64_t) T * B);
    ggml_tensor * pos = ggml_new_tensor_1d(c, GGML_TYPE_I32, T);
    const bool whole = g_bb_whole && !g_bb_sched;
    ggml_tensor * msk = mask ? ggml_new_tensor_2d(c, GGML_TYPE_F16, n_past + T, T) : nullptr;
    ggml_tensor * ids = whole ? ggml_new_tensor_1d(c, GGML_TYPE_I32, (int64_t) T * B) : nullptr;
    ggml_set_input(inp); ggml_set_input(pos);
    if (msk) ggml_set_input(msk);
    ggml_tensor * h = inp;
    if (whole) {
        ggml_set_input(ids);
        h = ggml_get_rows(c, inp, ids);
        if (mask) { // the mask values handed in are not used: the graph derives them from pos
            const int total = n_past + T;
            ggml_tensor * keys = ggml_reshape_2d(c, ggml_arange(c, 0.0f, (float) total, 1.0f), total, 1);
            ggml_tensor * qpos = ggml_reshape_2d(c, ggml_cast(c, pos, GGML_TYPE_F32), 1, T);
            ggml_tensor * target = ggml_new_tensor_2d(c, GGML_TYPE_F32, total, T);
            ggml_tensor * mk = ggml_sub(c, ggml_repeat(c, keys, target), ggml_repeat(c, qpos, target));
            mk = ggml_add1(c, mk, ggml_arange(c, -0.5f, 0.5f, 1.0f));
            mk = ggml_scale(c, ggml_step(c, mk), -1.0e9f);
            msk = ggml_cont(c, ggml_cast(c, mk, GGML_TYPE_F16));
        }
    }
    const bool mask_is_input = msk && !(whole && mask);
    std::vector<ggml_tensor *> roots;
    for (const auto & L : m.layers) h = bb_layer_forward(c, m, L, h, pos, msk, T, n_past, write_kv != 0, roots);
    h = bb_norm(c, m, h, m.final_norm);
    ggml_set_output(h);
    ggml_cgraph * gf = ggml_new_graph_custom(c, n_nodes, false);
    ggml_build_forward_expand(gf, h);
    for (ggml_tensor * r : roots) ggml_build_forward_expand(gf, r);
    if (g_bb_sched) { // the scheduler path VoxCPM takes with VOXCPM_ENABLE_SCHEDULER (src/backend.cpp:263-283)
        ggml_backend_t cpu = ggml_backend_init_by_type(GGML_BACKEND_DEVICE_TYPE_CPU, nullptr);
        if (!cpu) { ggml_free(c); return 105; }
        ggml_backend_cpu_set_n_threads(cpu, 8);
        ggml_backend_t backs[2] = { g_backend, cpu };
        const bool same = ggml_backend_dev_type(ggml_backend_get_device(g_backend)) == GGML_BACKEND_DEVICE_TYPE_CPU;
        ggml_backend_sched_t sched = ggml_backend_sched_new(same ? backs + 1 : backs, nullptr, same ? 1 : 2, n_nodes, false, true);
        int rcs = 0;
        if (!sched || !ggml_backend_sched_alloc_graph(sched, gf)) rcs = 101;
        if (!rcs) {
            ggml_backend_tensor_set(inp, x, 0, ggml_nbytes(inp));
            std::vector<int32_t> p((size_t) T);
            for (int i = 0; i < T; ++i) p[(size_t) i] = n_past + i;
            ggml_backend_tensor_set(pos, p.data(), 0, ggml_nbytes(pos));
            if (msk) ggml_backend_tensor_set(msk, mask, 0, ggml_nbytes(msk));
            if (ggml_backend_sched_graph_compute(sched, gf) != GGML_STATUS_SUCCESS) rcs = 102;
        }
        if (!rcs && out) ggml_backend_tensor_get(h, out, 0, ggml_nbytes(h));
        if (seconds) { seconds[0] = seconds[1] = 0.0; seconds[2] = sched ? (double) ggml_backend_sched_get_n_splits(sched) : 0.0; }
        if (sched) ggml_backend_sched_free(sched);
        ggml_backend_free(cpu);
        ggml_free(c);
        return rcs;
    }
    ggml_gallocr_t ga = ggml_gallocr_new(ggml_backend_get_default_buffer_type(g_backend));
    int rc = 0;
    if (!ggml_gallocr_alloc_graph(ga, gf)) rc = 101;
    auto upload = [&] { // the allocator hands an input's memory on once its readers have run: written before every run
        ggml_backend_tensor_set(inp, x, 0, ggml_nbytes(inp));
        std::vector<int32_t> p((size_t) T);
        for (int i = 0; i < T; ++i) p[(size_t) i] = n_past + i;
        ggml_backend_tensor_set(pos, p.data(), 0, ggml_nbytes(pos));
        if (mask_is_input) ggml_backend_tensor_set(msk, mask, 0, ggml_nbytes(msk));
        if (ids) {
            std::vector<int32_t> id((size_t) T * B);
            for (size_t i = 0; i < id.size(); ++i) id[i] = (int32_t) i;
            ggml_backend_tensor_set(ids, id.data(), 0, ggml_nbytes(ids));
        }
    };
    if (!rc) {
        upload();
        if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) rc = 102;
    }
    if (!rc && reps > 0 && seconds) {
        double best = 1e30, total = 0;
        g_last_times.clear();
        for (int r = 0; r < reps && !rc; ++r) {
            upload(); // not timed
            auto t0 = std::chrono::steady_clock::now();
            if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) rc = 102;
            auto t1 = std::chrono::steady_clock::now();
            const double dt = std::chrono::duration<double>(t1 - t0).count();
            g_last_times.push_back(dt);
            total += dt;
            if (dt < best) best = dt;
        }
        seconds[0] = total / reps;
        seconds[1] = best;
    }
    if (!rc && out) ggml_backend_tensor_get(h, out, 0, ggml_nbytes(h));
    if (seconds) seconds[2] = (double) ggml_graph_n_nodes(gf);
    if (getenv("RH_DUMP_GRAPH")) { // node order of the graph, for inspection
        for (int i = 0; i < ggml_graph_n_nodes(gf); ++i) {
            ggml_tensor * n = ggml_graph_node(gf, i);
            fprintf(stderr, "%3d %s\n", i, ggml_op_desc(n));
        }
    }
    ggml_gallocr_free(ga);
    ggml_free(c);
    return rc;
}

// A run of consecutive decode steps as the reference drives them (src/voxcpm.cpp:485-513, 1027-1128): every step gets
// a fresh context and a graph built for its own position (n_past is baked into the views of the cache), the graph
// is laid out by the one graph allocator the run keeps, the step's input and position are uploaded, the graph is
// computed and the hidden state fetched.  x: [hidden, 1, batch], the same input every step.  seconds[0] = wall
// time per step over the whole loop, [1] = the graph_compute calls' share per step (with overlap: compute and the
// next graph's construction together), [2] = nodes of the last graph, [3] = graph construction + layout per step,
// [4] = the share of nodes whose address differs from the previous step's.  The cache is written: steps n_past0 ..
// n_past0 + steps - 1.
int rh_bb_decode_loop(const float * x, int n_past0, int steps, int overlap, float * out, double * seconds) {
    if (!g_bb || !g_backend || steps < 1) return 100;
    const backbone & m = *g_bb;
    const int B = m.batch;
    if (n_past0 + steps > m.max_len) return 104;
    const size_t n_nodes = (size_t) m.n_layer * 64 + 64;
    // overlap = 1: the next step's graph is built and laid out while the device works on the current one (its shape
    // depends on the position only, not on the step's result): two contexts and two graph allocators take turns, the
    // graph is enqueued with ggml_backend_graph_compute_async and the host synchronises when it needs the hidden state
    ggml_gallocr_t ga[2] = { ggml_gallocr_new(ggml_backend_get_default_buffer_type(g_backend)),
                             overlap ? ggml_gallocr_new(ggml_backend_get_default_buffer_type(g_backend)) : nullptr };
    int rc = 0, last_nodes = 0;
    long long moved = 0, compared = 0;
    double t_compute = 0.0, t_build = 0.0;
    std::vector<float> hidden((size_t) m.hidden * B);
    std::vector<const void *> prev_addr;
    struct built { ggml_context * c = nullptr; ggml_cgraph * gf = nullptr; ggml_tensor * inp = nullptr, * pos = nullptr, * h = nullptr; };
    auto build = [&](int n_past, ggml_gallocr_t alloc) {
        const auto tb0 = std::chrono::steady_clock::now();
        built b;
        ggml_init_params ip = { ggml_tensor_overhead() * n_nodes + ggml_graph_overhead_custom(n_nodes, false), nullptr, true };
        b.c = ggml_init(ip);
        b.inp = ggml_new_tensor_2d(b.c, GGML_TYPE_F32, m.hidden, (int64_t) B);
        b.pos = ggml_new_tensor_1d(b.c, GGML_TYPE_I32, 1);
        ggml_set_input(b.inp); ggml_set_input(b.pos);
        ggml_tensor * h = b.inp;
        std::vector<ggml_tensor *> roots;
        for (const auto & L : m.layers) h = bb_layer_forward(b.c, m, L, h, b.pos, nullptr, 1, n_past, true, roots);
        h = bb_norm(b.c, m, h, m.final_norm);
        ggml_set_output(h);
        b.h = h;
        b.gf = ggml_new_graph_custom(b.c, n_nodes, false);
        ggml_build_forward_expand(b.gf, h);
        for (ggml_tensor * r : roots) ggml_build_forward_expand(b.gf, r);
        if (!ggml_gallocr_alloc_graph(alloc, b.gf)) rc = 101;
        t_build += std::chrono::duration<double>(std::chrono::steady_clock::now() - tb0).count();
        return b;
    };
    const auto t_loop = std::chrono::steady_clock::now();
    built cur = build(n_past0, ga[0]);
    for (int s = 0; s < steps && !rc; ++s) {
        const int n_past = n_past0 + s;
        ggml_backend_tensor_set(cur.inp, x, 0, ggml_nbytes(cur.inp));
        const int32_t p = n_past;
        ggml_backend_tensor_set(cur.pos, &p, 0, sizeof p);
        last_nodes = ggml_graph_n_nodes(cur.gf);
        if (!overlap) { // how many nodes lie at another address than in the step before (the graph is otherwise the same)
            if ((int) prev_addr.size() == last_nodes)
                for (int i = 0; i < last_nodes; ++i) { ++compared; if (prev_addr[(size_t) i] != ggml_graph_node(cur.gf, i)->data) ++moved; }
            prev_addr.resize((size_t) last_nodes);
            for (int i = 0; i < last_nodes; ++i) prev_addr[(size_t) i] = ggml_graph_node(cur.gf, i)->data;
        }
        const auto t0 = std::chrono::steady_clock::now();
        built next;
        if (overlap) {
            if (ggml_backend_graph_compute_async(g_backend, cur.gf) != GGML_STATUS_SUCCESS) rc = 102;
            if (!rc && s + 1 < steps) next = build(n_past + 1, ga[(s + 1) & 1]);
            ggml_backend_synchronize(g_backend);
        } else {
            if (ggml_backend_graph_compute(g_backend, cur.gf) != GGML_STATUS_SUCCESS) rc = 102;
        }
        t_compute += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        if (!rc) ggml_backend_tensor_get(cur.h, hidden.data(), 0, ggml_nbytes(cur.h));
        ggml_free(cur.c);
        cur = built{};
        if (!rc && s + 1 < steps) cur = overlap ? next : build(n_past + 1, ga[0]);
    }
    if (cur.c) ggml_free(cur.c);
    const double t_all = std::chrono::duration<double>(std::chrono::steady_clock::now() - t_loop).count();
    if (seconds) {
        seconds[0] = t_all / steps; seconds[1] = t_compute / steps; seconds[2] = (double) last_nodes; seconds[3] = t_build / steps;
        seconds[4] = compared ? (double) moved / (double) compared : 0.0;
    }
    if (!rc && out) memcpy(out, hidden.data(), hidden.size() * sizeof(float));
    ggml_gallocr_free(ga[0]);
    if (ga[1]) ggml_gallocr_free(ga[1]);
    return rc;
}

// ---- two dependent stages, with and without a trip through the host -----------------------------------------
// The reference's decode step runs the base LM's step graph, fetches its hidden state to the host, adds the step's
// embedding there and uploads the sum as the input of the residual LM's step graph (src/voxcpm.cpp:1067-1093): two
// synchronous copies and a host loop between two graphs.  resident = 0 does exactly that with two forward graphs of the
// stack made by rh_bb_create (T tokens, no cache): out = forward(forward(x) + x).  resident = 1 keeps everything on
// the backend's device: the input and the first stage's result live in tensors of a persistent backend buffer (like
// the KV cache does), the first graph ends in a CPY into that state, the second graph begins with the ADD -- no
// tensor_get / tensor_set between the stages, one synchronisation at the end.  Same nodes, same arithmetic: the two
// variants must agree bit for bit.  seconds: mean and best wall time of one two-stage step (uploads of x included in
// both variants), repeats >= 1.
int rh_bb_two_stage(const float * x, const uint16_t * mask, int n_tokens, int resident, float * out, int reps, double * seconds) {
    if (!g_bb || !g_backend || reps < 1) return 100;
    const backbone & m = *g_bb;
    const int T = n_tokens, B = m.batch;
    if (T > m.max_len) return 104;
    const int64_t n_tok = (int64_t) T * B;
    const size_t n_nodes = (size_t) m.n_layer * 64 + 64;
    // persistent state on the device: the step's input and the first stage's hidden state
    ggml_init_params sp = { ggml_tensor_overhead() * 8, nullptr, true };
    ggml_context * sc = ggml_init(sp);
    ggml_tensor * x_dev = ggml_new_tensor_2d(sc, GGML_TYPE_F32, m.hidden, n_tok);
    ggml_tensor * h_dev = ggml_new_tensor_2d(sc, GGML_TYPE_F32, m.hidden, n_tok);
    ggml_tensor * pos_d = ggml_new_tensor_1d(sc, GGML_TYPE_I32, T);
    ggml_tensor * msk_d = mask ? ggml_new_tensor_2d(sc, GGML_TYPE_F16, T, T) : nullptr;
    ggml_backend_buffer_t sbuf = ggml_backend_alloc_ctx_tensors(sc, g_backend);
    if (!sbuf) { ggml_free(sc); return 101; }
    std::vector<int32_t> p((size_t) T);
    for (int i = 0; i < T; ++i) p[(size_t) i] = i;
    ggml_backend_tensor_set(pos_d, p.data(), 0, ggml_nbytes(pos_d));
    if (msk_d) ggml_backend_tensor_set(msk_d, mask, 0, ggml_nbytes(msk_d));

    struct stage { ggml_context * c = nullptr; ggml_cgraph * g = nullptr; ggml_gallocr_t ga = nullptr; ggml_tensor * in = nullptr, * out = nullptr; };
    auto build = [&](int which) {
        stage st;
        ggml_init_params ip = { ggml_tensor_overhead() * n_nodes + ggml_graph_overhead_custom(n_nodes, false), nullptr, true };
        st.c = ggml_init(ip);
        ggml_tensor * h;
        if (resident) {
            h = which == 0 ? x_dev : ggml_add(st.c, h_dev, x_dev);
        } else {
            st.in = ggml_new_tensor_2d(st.c, GGML_TYPE_F32, m.hidden, n_tok);
            ggml_set_input(st.in);
            h = st.in;
        }
        std::vector<ggml_tensor *> roots;
        for (const auto & L : m.layers) h = bb_layer_forward(st.c, m, L, h, pos_d, msk_d, T, 0, false, roots);
        h = bb_norm(st.c, m, h, m.final_norm);
        if (resident && which == 0) h = ggml_cpy(st.c, h, h_dev); // the state the next stage reads
        ggml_set_output(h);
        st.out = h;
        st.g = ggml_new_graph_custom(st.c, n_nodes, false);
        ggml_build_forward_expand(st.g, h);
        st.ga = ggml_gallocr_new(ggml_backend_get_default_buffer_type(g_backend));
        return st;
    };
    stage s0 = build(0), s1 = build(1);
    int rc = 0;
    if (!ggml_gallocr_alloc_graph(s0.ga, s0.g) || !ggml_gallocr_alloc_graph(s1.ga, s1.g)) rc = 101;
    const size_t nbytes = (size_t) n_tok * m.hidden * sizeof(float);
    std::vector<float> h1((size_t) n_tok * m.hidden), r((size_t) n_tok * m.hidden);
    double best = 1e30, total = 0;
    for (int it = 0; it < reps + 1 && !rc; ++it) { // the first pass is a warm-up
        auto t0 = std::chrono::steady_clock::now();
        if (resident) {
            ggml_backend_tensor_set(x_dev, x, 0, nbytes);
            if (ggml_backend_graph_compute_async(g_backend, s0.g) != GGML_STATUS_SUCCESS) rc = 102;
            if (!rc && ggml_backend_graph_compute_async(g_backend, s1.g) != GGML_STATUS_SUCCESS) rc = 102;
            if (!rc) { // buffer transfers are not ordered behind a backend's asynchronous work: wait for it first
                ggml_backend_synchronize(g_backend);
                ggml_backend_tensor_get(s1.out, out, 0, nbytes);
            }
        } else {
            ggml_backend_tensor_set(s0.in, x, 0, nbytes);
            if (ggml_backend_graph_compute(g_backend, s0.g) != GGML_STATUS_SUCCESS) rc = 102;
            if (!rc) {
                ggml_backend_tensor_get(s0.out, h1.data(), 0, nbytes);
                for (size_t i = 0; i < r.size(); ++i) r[i] = h1[i] + x[i];
                ggml_backend_tensor_set(s1.in, r.data(), 0, nbytes);
                if (ggml_backend_graph_compute(g_backend, s1.g) != GGML_STATUS_SUCCESS) rc = 102;
            }
            if (!rc) ggml_backend_tensor_get(s1.out, out, 0, nbytes);
        }
        auto t1 = std::chrono::steady_clock::now();
        if (it > 0) {
            const double d = std::chrono::duration<double>(t1 - t0).count();
            total += d;
            if (d < best) best = d;
        }
    }
    if (seconds) { seconds[0] = total / reps; seconds[1] = best; }
    for (stage * st : { &s0, &s1 }) { ggml_gallocr_free(st->ga); ggml_free(st->c); }
    ggml_backend_buffer_free(sbuf);
    ggml_free(sc);
    return rc;
}

// ---- a whole CFM solve as one graph ---------------------------------------------------------------------------
// The graph UnifiedCFM::forward builds (src/unified_cfm.cpp:88-184) around the LocDiT estimator's CFG-pair pass
// (src/locdit.cpp:248-258, 401-464): per Euler step the noisy patches are projected to the hidden size, the
// conditioned and unconditioned branches ride as ONE sequence of 2 * (1 + prefix + patch) tokens through the
// decoder stack (block-diagonal mask, positions i mod branch length, no cache write), both branches are projected
// back, combined by classifier-free guidance (zero-star scale: SUM, MUL, DIV, REPEAT, ARANGE for eps) and x takes
// the step.  The decoder is the stack made by rh_bb_create (batch 1; call rh_bb_fuse_weights for the row-fused
// variant the reference uses on GPU backends); the estimator's own projections are Q8_0 like every matrix the
// reference's quantizer writes for a Q8_0 model file (src/quantize.cpp:411-428), their biases F32.
namespace {
struct cfm_extra {
    ggml_context *        ctx = nullptr;
    ggml_backend_buffer_t buf = nullptr;
    ggml_tensor * w[3] = { nullptr, nullptr, nullptr }; // in_proj, cond_proj [feat, hidden]; out_proj [hidden, feat]
    ggml_tensor * b[3] = { nullptr, nullptr, nullptr };
    // time_mlp and delta_time_mlp: linear1, linear2 (Q8_0 [hidden, hidden]) and their biases (rh_cfm_set_time_mlp)
    ggml_tensor * tw[4] = { nullptr, nullptr, nullptr, nullptr };
    ggml_tensor * tb[4] = { nullptr, nullptr, nullptr, nullptr };
    bool has_time_mlp = false;
    int feat = 0;
};
cfm_extra * g_cfm = nullptr;
} // namespace

void rh_cfm_free(void) {
    if (!g_cfm) return;
    if (g_cfm->buf) ggml_backend_buffer_free(g_cfm->buf);
    if (g_cfm->ctx) ggml_free(g_cfm->ctx);
    delete g_cfm;
    g_cfm = nullptr;
}

// weights as Q8_0 rows: in_w, cond_w [hidden][feat]; out_w [feat][hidden] (rows of ne0 = the input size); F32 biases
// hidden / hidden / feat
int rh_cfm_create(int feat, const void * in_w, const float * in_b, const void * cond_w, const float * cond_b,
                  const void * out_w, const float * out_b) {
    if (!g_bb || !g_backend) return 100;
    rh_cfm_free();
    cfm_extra * e = new cfm_extra;
    e->feat = feat;
    ggml_init_params ip = { ggml_tensor_overhead() * 16, nullptr, true };
    e->ctx = ggml_init(ip);
    const int64_t H = g_bb->hidden;
    for (int i = 0; i < 4; ++i) {
        e->tw[i] = ggml_new_tensor_2d(e->ctx, GGML_TYPE_Q8_0, H, H);
        e->tb[i] = ggml_new_tensor_1d(e->ctx, GGML_TYPE_F32, H);
    }
    e->w[0] = ggml_new_tensor_2d(e->ctx, GGML_TYPE_Q8_0, feat, H); e->b[0] = ggml_new_tensor_1d(e->ctx, GGML_TYPE_F32, H);
    e->w[1] = ggml_new_tensor_2d(e->ctx, GGML_TYPE_Q8_0, feat, H); e->b[1] = ggml_new_tensor_1d(e->ctx, GGML_TYPE_F32, H);
    e->w[2] = ggml_new_tensor_2d(e->ctx, GGML_TYPE_Q8_0, H, feat); e->b[2] = ggml_new_tensor_1d(e->ctx, GGML_TYPE_F32, feat);
    e->buf = ggml_backend_alloc_ctx_tensors(e->ctx, g_backend);
    g_cfm = e;
    if (!e->buf) { rh_cfm_free(); return 101; }
    const void *  ws[3] = { in_w, cond_w, out_w };
    const float * bs[3] = { in_b, cond_b, out_b };
    for (int i = 0; i < 3; ++i) {
        ggml_backend_tensor_set(e->w[i], ws[i], 0, ggml_nbytes(e->w[i]));
        ggml_backend_tensor_set(e->b[i], bs[i], 0, ggml_nbytes(e->b[i]));
    }
    return 0;
}

// The weights of LocDiT's two timestep MLPs (src/locdit.cpp:213-246): which 0, 1 = time_mlp linear1, linear2; 2, 3 =
// delta_time_mlp linear1, linear2; Q8_0 rows [hidden][hidden] and F32 bias.  With them set, rh_cfm_solve called without a
// time table computes the combined time embedding of every step in the graph, as UnifiedCFM::forward does when it was not
// handed a precomputed table: ARANGE(t), the sinusoidal embedding (ARANGE, SCALE, EXP, SCALE, REPEAT, MUL, SIN, COS, CONCAT),
// two MUL_MAT + ADD + SILU layers, plus the delta-time embedding of zero.
int rh_cfm_set_time_mlp(int which, const void * w, const float * b) {
    if (!g_cfm || which < 0 || which > 3) return 100;
    ggml_backend_tensor_set(g_cfm->tw[which], w, 0, ggml_nbytes(g_cfm->tw[which]));
    ggml_backend_tensor_set(g_cfm->tb[which], b, 0, ggml_nbytes(g_cfm->tb[which]));
    if (which == 3) g_cfm->has_time_mlp = true;
    return 0;
}

// z [feat, patch, n_req], mu [hidden, n_req], cond [feat, prefix, n_req] (request-major), time_table [hidden, n_steps] (the
// combined time embedding of every step, as LocDiTModel::precompute_cfg_time_table hands it over; all requests step
// together), t_span n_steps + 1 values, pair_pos / pair_mask the CFG-pair constants for a branch of 1 + prefix + patch
// tokens.  out [feat, patch, n_req].  seconds: mean, best, node count.
// n_req > 1 (the decoder stack must have been made with that batch): the requests ride in dim 2 / as further sequences of
// the decoder's token dimension -- products, assembly and update are the same nodes over one more dimension, the
// zero-star sums become SUM_ROWS over each request's values (the reference runs one graph per request,
// src/voxcpm.cpp:1067-1093; this is how its graph reads with ggml's own batching).
static int cfm_solve_n(const float * z, const float * mu, const float * cond, const float * time_table, const float * t_span,
                       int n_steps, int patch, int prefix, const int32_t * pair_pos, const uint16_t * pair_mask, float cfg_value,
                       int zero_star, int n_req, float * out, int reps, double * seconds) {
    if (!g_bb || !g_cfm || !g_backend || n_steps < 1 || prefix < 1 || n_req < 1) return 100;
    if (!time_table && !g_cfm->has_time_mlp) return 103;
    const backbone & m = *g_bb;
    const cfm_extra & e = *g_cfm;
    const int H = m.hidden, F = e.feat, L = 1 + prefix + patch, T = 2 * L, R = n_req;
    if (T > m.max_len || R != m.batch) return 104;
    const size_t n_nodes = (size_t) n_steps * ((size_t) m.n_layer * 64 + 192) + 128;
    ggml_init_params ip = { ggml_tensor_overhead() * n_nodes + ggml_graph_overhead_custom(n_nodes, false), nullptr, true };
    ggml_context * c = ggml_init(ip);
    // (one request: exactly the reference's tensors and nodes)
    ggml_tensor * zin  = R == 1 ? ggml_new_tensor_2d(c, GGML_TYPE_F32, F, patch) : ggml_new_tensor_3d(c, GGML_TYPE_F32, F, patch, R);
    ggml_tensor * muin = R == 1 ? ggml_new_tensor_1d(c, GGML_TYPE_F32, H) : ggml_new_tensor_3d(c, GGML_TYPE_F32, H, 1, R);
    ggml_tensor * cin  = R == 1 ? ggml_new_tensor_2d(c, GGML_TYPE_F32, F, prefix) : ggml_new_tensor_3d(c, GGML_TYPE_F32, F, prefix, R);
    ggml_tensor * tab  = ggml_new_tensor_1d(c, GGML_TYPE_F32, (int64_t) H * n_steps);
    ggml_tensor * pos  = ggml_new_tensor_1d(c, GGML_TYPE_I32, T);
    ggml_tensor * msk  = ggml_new_tensor_2d(c, GGML_TYPE_F16, T, T);
    for (ggml_tensor * t : { zin, muin, cin, tab, pos, msk }) ggml_set_input(t);

    std::vector<ggml_tensor *> roots;
    ggml_tensor * x = zin;
    ggml_tensor * cond_proj = ggml_add(c, ggml_mul_mat(c, e.w[1], cin), e.b[1]); // [H, prefix, R]
    // LocDiTModel::sinusoidal_embedding + timestep_mlp (src/locdit.cpp:186-232)
    auto time_embedding = [&](ggml_tensor * scalar, int mlp) {
        const int   half = H / 2;
        const float ev   = logf(10000.0f) / (float) (half - 1);
        ggml_tensor * emb = ggml_scale(c, ggml_exp(c, ggml_scale(c, ggml_arange(c, 0.0f, (float) half, 1.0f), -ev)), 1000.0f);
        emb = ggml_mul(c, emb, ggml_repeat(c, ggml_reshape_1d(c, scalar, 1), emb));
        ggml_tensor * sc = ggml_concat(c, ggml_sin(c, emb), ggml_cos(c, emb), 0);
        ggml_tensor * h1 = ggml_silu(c, ggml_add(c, ggml_mul_mat(c, e.tw[2 * mlp], sc), e.tb[2 * mlp]));
        return ggml_add(c, ggml_mul_mat(c, e.tw[2 * mlp + 1], h1), e.tb[2 * mlp + 1]);
    };
    ggml_tensor * delta_zero = time_table ? nullptr : time_embedding(ggml_arange(c, 0.0f, 1.0f, 1.0f), 1);
    float t = t_span[0], dt = t_span[0] - t_span[1];
    const int zero_init_steps = n_steps > 1 ? std::max(1, (int) ((float) (n_steps + 1) * 0.04f)) : 0;
    for (int step = 1; step <= n_steps; ++step) {
        ggml_tensor * dphi;
        if (zero_star && step <= zero_init_steps) {
            dphi = ggml_scale(c, x, 0.0f);
        } else {
            ggml_tensor * x_proj   = ggml_add(c, ggml_mul_mat(c, e.w[0], x), e.b[0]); // [H, patch, R]
            ggml_tensor * combined = time_table ? ggml_view_1d(c, tab, H, (size_t) (step - 1) * H * sizeof(float))
                                                : ggml_add(c, time_embedding(ggml_arange(c, t, t + 1.0f, 1.0f), 0), delta_zero);
            ggml_tensor * comb_c, * comb_u;
            if (R == 1) { // the reference's nodes (src/locdit.cpp:401-452)
                comb_c = ggml_reshape_2d(c, ggml_add(c, ggml_reshape_1d(c, combined, H), muin), H, 1);
                comb_u = ggml_reshape_2d(c, combined, H, 1);
            } else {
                ggml_tensor * comb1 = ggml_reshape_3d(c, combined, H, 1, 1);
                comb_c = ggml_add(c, muin, comb1);      // mu of every request + the step's embedding
                comb_u = ggml_repeat(c, comb1, muin);   // the embedding alone, once per request
            }
            ggml_tensor * seq_c    = ggml_concat(c, ggml_concat(c, comb_c, cond_proj, 1), x_proj, 1);
            ggml_tensor * seq_u    = ggml_concat(c, ggml_concat(c, comb_u, cond_proj, 1), x_proj, 1);
            ggml_tensor * h        = ggml_concat(c, seq_c, seq_u, 1);
            if (R > 1) h = ggml_reshape_2d(c, h, H, (int64_t) T * R); // request after request in the decoder's token dimension
            for (const auto & Lr : m.layers) h = bb_layer_forward(c, m, Lr, h, pos, msk, T, 0, false, roots);
            h = bb_norm(c, m, h, m.final_norm);
            const size_t tok = h->nb[1];
            ggml_tensor * hc = R == 1 ? ggml_view_2d(c, h, H, patch, tok, (size_t) (prefix + 1) * tok)
                                      : ggml_view_3d(c, h, H, patch, R, tok, (size_t) T * tok, (size_t) (prefix + 1) * tok);
            ggml_tensor * hu = R == 1 ? ggml_view_2d(c, h, H, patch, tok, (size_t) (L + prefix + 1) * tok)
                                      : ggml_view_3d(c, h, H, patch, R, tok, (size_t) T * tok, (size_t) (L + prefix + 1) * tok);
            ggml_tensor * vc = ggml_add(c, ggml_mul_mat(c, e.w[2], hc), e.b[2]); // [F, patch, R]
            ggml_tensor * vu = ggml_add(c, ggml_mul_mat(c, e.w[2], hu), e.b[2]);
            if (zero_star) {
                ggml_tensor * dot, * nrm;
                if (R == 1) {
                    dot = ggml_sum(c, ggml_mul(c, vc, vu));
                    nrm = ggml_sum(c, ggml_mul(c, vu, vu));
                } else { // one sum per request
                    dot = ggml_sum_rows(c, ggml_reshape_2d(c, ggml_mul(c, vc, vu), (int64_t) F * patch, R)); // [1, R]
                    nrm = ggml_sum_rows(c, ggml_reshape_2d(c, ggml_mul(c, vu, vu), (int64_t) F * patch, R));
                }
                ggml_tensor * st  = ggml_div(c, dot, ggml_add(c, nrm, ggml_arange(c, 1.0e-8f, 1.0e-8f + 1.0f, 1.0f)));
                ggml_tensor * us  = ggml_mul(c, vu, ggml_repeat(c, R == 1 ? st : ggml_reshape_3d(c, st, 1, 1, R), vu));
                dphi = ggml_add(c, us, ggml_scale(c, ggml_sub(c, vc, us), cfg_value));
            } else {
                dphi = ggml_add(c, vu, ggml_scale(c, ggml_sub(c, vc, vu), cfg_value));
            }
        }
        x = ggml_sub(c, x, ggml_scale(c, dphi, dt));
        t -= dt;
        if (step < n_steps) dt = t - t_span[step + 1];
    }
    ggml_set_output(x);
    ggml_cgraph * gf = ggml_new_graph_custom(c, n_nodes, false);
    ggml_build_forward_expand(gf, x);

    ggml_gallocr_t ga = ggml_gallocr_new(ggml_backend_get_default_buffer_type(g_backend));
    int rc = 0;
    if (!ggml_gallocr_alloc_graph(ga, gf)) rc = 101;
    auto upload = [&] { // inputs may share memory with later nodes of the graph: written before every run
        ggml_backend_tensor_set(zin, z, 0, ggml_nbytes(zin));
        ggml_backend_tensor_set(muin, mu, 0, ggml_nbytes(muin));
        ggml_backend_tensor_set(cin, cond, 0, ggml_nbytes(cin));
        if (time_table) ggml_backend_tensor_set(tab, time_table, 0, ggml_nbytes(tab));
        ggml_backend_tensor_set(pos, pair_pos, 0, ggml_nbytes(pos));
        ggml_backend_tensor_set(msk, pair_mask, 0, ggml_nbytes(msk));
    };
    if (!rc) {
        upload();
        if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) rc = 102;
    }
    if (!rc && out) ggml_backend_tensor_get(x, out, 0, ggml_nbytes(x));
    if (!rc && reps > 0 && seconds) {
        double best = 1e30, total = 0;
        g_last_times.clear();
        for (int r = 0; r < reps && !rc; ++r) {
            upload();
            auto t0 = std::chrono::steady_clock::now();
            if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) rc = 102;
            auto t1 = std::chrono::steady_clock::now();
            const double d = std::chrono::duration<double>(t1 - t0).count();
            g_last_times.push_back(d);
            total += d;
            if (d < best) best = d;
        }
        seconds[0] = total / reps;
        seconds[1] = best;
        if (!rc && out && g_out_after_reps) ggml_backend_tensor_get(x, out, 0, ggml_nbytes(x)); // the last repeat's result
    }
    if (seconds) seconds[2] = (double) ggml_graph_n_nodes(gf);
    ggml_gallocr_free(ga);
    ggml_free(c);
    return rc;
}

int rh_cfm_solve(const float * z, const float * mu, const float * cond, const float * time_table, const float * t_span,
                 int n_steps, int patch, int prefix, const int32_t * pair_pos, const uint16_t * pair_mask, float cfg_value,
                 int zero_star, float * out, int reps, double * seconds) {
    return cfm_solve_n(z, mu, cond, time_table, t_span, n_steps, patch, prefix, pair_pos, pair_mask, cfg_value, zero_star, 1, out, reps, seconds);
}
int rh_cfm_solve_requests(const float * z, const float * mu, const float * cond, const float * time_table, const float * t_span,
                          int n_steps, int patch, int prefix, const int32_t * pair_pos, const uint16_t * pair_mask, float cfg_value,
                          int zero_star, int n_req, float * out, int reps, double * seconds) {
    return cfm_solve_n(z, mu, cond, time_table, t_span, n_steps, patch, prefix, pair_pos, pair_mask, cfg_value, zero_star, n_req, out, reps, seconds);
}


// ---- a random graph of the small operators around the stacks ------------------------------------------------
// What the plugin decides per graph (runs of tiny nodes as one launch, values that live in LDS only, trees of CONCATs
// written from their leaves, pairs of nodes) depends on reader counts and on the memory ggml-alloc hands out -- and
// ggml-alloc reuses a dead tensor's block at once.  A seeded random DAG of the exact operators (ADD, SUB, MUL with ggml's
// broadcast, SCALE, SQR, NEG, CONT, REPEAT, CONCAT + a view back, SUM_ROWS, SUM, DIV on the small results) over a handful
// of inputs, allocated by ggml_gallocr and computed on the selected backend: the same seed gives the same graph on every
// backend, so ggml-cpu is the reference.  out receives the final [n, R] tensor; *n_nodes the graph's node count.
int rh_random_graph(uint64_t seed, int n_ops, float * out, int64_t out_cap, int64_t * out_n, int * n_nodes) {
    if (!g_backend) return 100;
    uint64_t st = seed * 6364136223846793005ull + 1442695040888963407ull;
    auto rnd = [&]() { st = st * 6364136223846793005ull + 1442695040888963407ull; return (uint32_t) (st >> 33); };
    auto pick = [&](int n) { return (int) (rnd() % (uint32_t) n); };
    auto unif = [&]() { return (float) (rnd() % 20001) / 10000.0f - 1.0f; };
    const int64_t ns[] = { 64, 100, 257, 1024, 4096 }, rs[] = { 1, 2, 3, 8 }; // (4096 x 8: beyond a small-graph run, every node its own launch or pair)
    const int64_t n = ns[pick(5)], R = rs[pick(4)];
    ggml_init_params ip = { ggml_tensor_overhead() * (size_t) (32 + 8 * n_ops) + ggml_graph_overhead_custom(1024, false), nullptr, true };
    ggml_context * ic = ggml_init(ip);   // inputs: their own buffer
    ggml_context * c  = ggml_init(ip);   // the graph: ggml_gallocr's memory
    std::vector<ggml_tensor *> full, cols, scal;
    std::vector<ggml_tensor *> inputs;
    for (int k = 0; k < 4; ++k) { ggml_tensor * t = ggml_new_tensor_2d(ic, GGML_TYPE_F32, n, R); inputs.push_back(t); full.push_back(t); }
    ggml_tensor * row = ggml_new_tensor_2d(ic, GGML_TYPE_F32, n, 1); inputs.push_back(row);
    { ggml_tensor * t = ggml_new_tensor_2d(ic, GGML_TYPE_F32, 1, R); inputs.push_back(t); cols.push_back(t); }
    { ggml_tensor * t = ggml_new_tensor_1d(ic, GGML_TYPE_F32, 1); inputs.push_back(t); scal.push_back(t); }
    ggml_backend_buffer_t ibuf = ggml_backend_alloc_ctx_tensors(ic, g_backend);
    if (!ibuf) { ggml_free(ic); ggml_free(c); return 101; }
    for (ggml_tensor * t : inputs) {
        std::vector<float> v((size_t) ggml_nelements(t));
        for (float & x : v) x = unif();
        if (ggml_nelements(t) <= R) for (float & x : v) x += 2.5f; // (divisors and scalars away from zero)
        ggml_backend_tensor_set(t, v.data(), 0, ggml_nbytes(t));
    }
    std::vector<int> uses(full.size(), 0);
    auto take = [&]() { const int k = pick((int) full.size()); ++uses[k]; return full[k]; };
    auto put  = [&](ggml_tensor * t) { full.push_back(t); uses.push_back(0); };
    for (int k = 0; k < n_ops; ++k) {
        switch (pick(14)) {
            case 0: put(ggml_add(c, take(), take())); break;
            case 1: put(ggml_sub(c, take(), take())); break;
            case 2: put(ggml_mul(c, take(), take())); break;
            case 3: put(ggml_add(c, take(), pick(2) ? row : (pick(2) ? cols[pick((int) cols.size())] : scal[pick((int) scal.size())]))); break;
            case 4: put(ggml_mul(c, take(), pick(2) ? row : (pick(2) ? cols[pick((int) cols.size())] : scal[pick((int) scal.size())]))); break;
            case 5: put(ggml_scale(c, take(), 0.25f + 0.5f * (float) pick(4))); break;
            case 6: put(pick(2) ? ggml_sqr(c, take()) : ggml_neg(c, take())); break;
            case 7: put(ggml_cont(c, take())); break;
            case 8: put(ggml_repeat(c, pick(2) ? row : (pick(2) ? cols[pick((int) cols.size())] : scal[pick((int) scal.size())]), full[0])); break;
            case 9: { // CONCAT of two along the row dimension (or of a CONCAT and a third), then one half back as a view
                ggml_tensor * cat = ggml_concat(c, take(), take(), 1);
                if (pick(2)) cat = ggml_concat(c, cat, take(), 1);
                const int64_t first = pick((int) (cat->ne[1] / R)) * R;
                put(ggml_cont(c, ggml_view_2d(c, cat, n, R, cat->nb[1], (size_t) first * cat->nb[1])));
            } break;
            case 10: cols.push_back(ggml_sum_rows(c, take())); break;
            case 11: scal.push_back(ggml_sum(c, take())); break;
            case 12: cols.push_back(ggml_div(c, cols[pick((int) cols.size())], cols[pick((int) cols.size())])); break;
            default: scal.push_back(ggml_scale(c, scal[pick((int) scal.size())], 0.5f)); break;
        }
    }
    // everything nobody read yet flows into the result, so that (nearly) every node is an ancestor of it
    ggml_tensor * res = full.back();
    for (size_t k = 4; k + 1 < full.size(); ++k) if (uses[k] == 0) res = ggml_add(c, res, full[k]);
    res = ggml_add(c, res, ggml_repeat(c, cols.back(), res));
    res = ggml_add(c, res, scal.back());
    ggml_set_output(res);
    ggml_cgraph * gf = ggml_new_graph_custom(c, 1024, false);
    ggml_build_forward_expand(gf, res);
    ggml_gallocr_t ga = ggml_gallocr_new(ggml_backend_get_default_buffer_type(g_backend));
    int rc = 0;
    if (!ggml_gallocr_alloc_graph(ga, gf)) rc = 101;
    for (int rep = 0; rep < 2 && !rc; ++rep) // twice: the second computation finds whatever the first left in reused blocks
        if (ggml_backend_graph_compute(g_backend, gf) != GGML_STATUS_SUCCESS) rc = 102;
    if (!rc && ggml_nelements(res) > out_cap) rc = 103;
    if (!rc) { ggml_backend_tensor_get(res, out, 0, ggml_nbytes(res)); *out_n = ggml_nelements(res); *n_nodes = ggml_graph_n_nodes(gf); }
    ggml_gallocr_free(ga);
    ggml_backend_buffer_free(ibuf);
    ggml_free(c);
    ggml_free(ic);
    return rc;
}

} // extern "C"
