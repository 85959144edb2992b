// ggml-gfx950.cpp -- a ggml backend for AMD MI355X (gfx950) that claims the operators of
// VoxCPM.cpp's attention hot path and nothing else:
//
//     GGML_OP_FLASH_ATTN_EXT, GGML_OP_ROPE, GGML_OP_SOFT_MAX, GGML_OP_RMS_NORM,
//     GGML_OP_MUL_MAT (Q8_0 / F16 / F32 weights, F32 activations)
//
// plus the glue between them in a decoder layer (ADD, SUB, MUL, DIV, ADD1, SCALE, CPY, CONT,
// DUP, CONCAT, SUM, UNARY silu & co, GLU swiglu), so that a MiniCPM layer needs no scheduler
// split, and the view ops every backend accepts.  Everything else is answered with
// supports_op() == false, so ggml's scheduler keeps it on ggml-cpu.  The file is host-only
// C++: it implements ggml's five backend vtables (ggml/src/ggml-backend-impl.h:17-204 of
// the reference checkout) and forwards every claimed node, unchanged, to the C ABI of
// libvoxcpm_gfx950.so (include/voxcpm_gfx950.h), where the hand-written HIP kernels live.
//
// It is built against the reference's ggml headers and loaded like any dynamically loaded
// ggml backend: ggml_backend_load("libggml-gfx950.so") or GGML_BACKEND_PATH
// (ggml/src/ggml-backend-reg.cpp:194-238, 561-565).  ggml's own symbols are resolved from
// the host process.  With no gfx950 device visible, ggml_backend_score() returns 0 and the
// registry reports zero devices; nothing aborts.
#include "ggml-backend-impl.h"
#include "ggml-backend.h"
#include "ggml-impl.h"
#include "ggml.h"

#include "ggml-alloc.h"
#include "ggml-gfx950.h"
#include "voxcpm_gfx950.h"

#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <cstdlib>
#include <chrono>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>

namespace {

constexpr size_t GFX950_ALIGNMENT = 256;

// ------------------------------------------------------------------ tensor descriptors
vx_tensor to_vx(const ggml_tensor * t) {
    vx_tensor v;
    v.type = (int32_t) t->type;
    v._pad = 0;
    for (int i = 0; i < 4; ++i) {
        v.ne[i] = t->ne[i];
        v.nb[i] = t->nb[i];
    }
    v.data = t->data;
    return v;
}

bool type_known(ggml_type t) {
    return t == GGML_TYPE_F32 || t == GGML_TYPE_F16 || t == GGML_TYPE_Q8_0 || t == GGML_TYPE_I32;
}

int binary_code(ggml_op op) {
    switch (op) {
        case GGML_OP_ADD: return VX_BIN_ADD;
        case GGML_OP_SUB: return VX_BIN_SUB;
        case GGML_OP_MUL: return VX_BIN_MUL;
        default:          return VX_BIN_DIV;
    }
}

// ggml's stand-alone elementwise ops that the library serves through vx_unary; -1 for any other op
int standalone_unary_code(ggml_op op) {
    switch (op) {
        case GGML_OP_SQR:  return VX_UNARY_SQR;
        case GGML_OP_SQRT: return VX_UNARY_SQRT;
        case GGML_OP_LOG:  return VX_UNARY_LOG;
        case GGML_OP_SIN:  return VX_UNARY_SIN;
        case GGML_OP_COS:  return VX_UNARY_COS;
        default:           return -1;
    }
}

// how activations enter a Q8_0 product: the environment's choice at load time, or a later ggml_backend_gfx950_set_mul_mat_act
int g_mul_mat_act = -1;
int mul_mat_act_mode() {
    if (g_mul_mat_act < 0) {
        const char * e = getenv("GGML_GFX950_MUL_MAT_ACT");
        g_mul_mat_act = (e && strcmp(e, "q8") == 0) ? VX_ACT_Q8 : VX_ACT_FLOAT;
    }
    return g_mul_mat_act;
}

// --------------------------------------------------------------------- per-device state
struct device_ctx {
    int         index;
    std::string name;
    std::string description;
};

// A graph this backend has run before, recognised by a fingerprint of everything a launch depends on (operators,
// parameters, shapes, strides and addresses of every node and operand): from its third identical run on, the recorded
// launches are replayed as one HIP graph instead of being analysed and issued again.
struct seen_graph {
    uint64_t cheap = 0;      // a quick signature; only graphs that agree on it are fingerprinted in full
    uint64_t fingerprint = 0;
    int      runs = 0;       // identical runs so far
    int      launches = 0;
    bool     no_replay = false; // recording failed once: keep launching it node by node
    vx_graph recorded = nullptr;
    uint64_t last_use = 0;
};

// Graphs that agree in their nodes' operators and types but not in addresses, extents or parameters: the steps of a
// decode loop, each with one key more than the one before.  Such a graph never comes back, but its launches are the
// previous step's with a few arguments changed: the node-by-node pass is then made against a recording (nothing is
// launched, the arguments that differ are set on the recorded HIP graph) and the graph is launched as one unit.  Two
// recordings are used in turn, so that one can be prepared while the other still runs.
struct step_family {
    uint64_t shape = 0;       // node count, operators and types
    int      sightings = 0;
    int      failures = 0;    // recordings that could not be made, or passes that made other launches than recorded
    vx_graph recorded[2] = { nullptr, nullptr };
    int      turn = 0;
    int      launches = 0;
    uint64_t last_use = 0;
};

struct backend_ctx {
    int       device;
    vx_stream stream;
    std::vector<seen_graph> seen;   // a handful of entries, least recently used one replaced
    std::vector<step_family> families;
    uint64_t  clock = 0;
    int       replays = 0;          // diagnostic: graph_compute calls served by a replay
};

struct buffer_ctx {
    int    device;
    void * base;
    bool   pinned = false; // declared constant to the library (vx_weights_pin): writes into it are reported
};

ggml_backend_buffer_type_t device_buffer_type(ggml_backend_dev_t dev);

// ------------------------------------------------------------------------------ buffers
void buffer_free(ggml_backend_buffer_t buffer) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    vx_init(ctx->device);
    if (ctx->pinned) vx_weights_unpin(ctx->base);
    vx_free(ctx->base);
    delete ctx;
}

// The caller's statement that a buffer holds weights (ggml_backend_buffer_set_usage(..., GGML_BACKEND_BUFFER_USAGE_WEIGHTS):
// the reference's src/weight-store.cpp:86, src/minicpm.cpp:472) is passed on to the library when a product first reads a
// weight from the buffer: the library may then keep re-laid-out copies of those weights between calls.  Every write into
// such a buffer -- through the buffer interface, the backend's asynchronous upload or a graph node -- is reported, which
// drops the copies made from the bytes written.
void pin_if_weights(ggml_backend_buffer_t buffer) {
    if (!buffer || buffer->usage != GGML_BACKEND_BUFFER_USAGE_WEIGHTS || buffer->iface.free_buffer != buffer_free) return;
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    if (!ctx->pinned && vx_weights_pin(ctx->base, buffer->size) == VX_OK) ctx->pinned = true;
}
void written_to(ggml_backend_buffer_t buffer, const void * p, size_t bytes) {
    if (!buffer || buffer->iface.free_buffer != buffer_free) return;
    if (((buffer_ctx *) buffer->context)->pinned) vx_weights_changed(p, bytes);
}

void * buffer_get_base(ggml_backend_buffer_t buffer) { return ((buffer_ctx *) buffer->context)->base; }

void buffer_memset_tensor(ggml_backend_buffer_t buffer, ggml_tensor * tensor, uint8_t value, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    vx_init(ctx->device);
    written_to(buffer, (char *) tensor->data + offset, size);
    if (vx_memset((char *) tensor->data + offset, value, size, nullptr) != VX_OK || vx_stream_synchronize(nullptr) != VX_OK)
        GGML_ABORT("ggml-gfx950: memset_tensor failed: %s", vx_last_error());
}

void buffer_set_tensor(ggml_backend_buffer_t buffer, ggml_tensor * tensor, const void * data, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    vx_init(ctx->device);
    written_to(buffer, (char *) tensor->data + offset, size);
    if (vx_memcpy_h2d((char *) tensor->data + offset, data, size, nullptr) != VX_OK || vx_stream_synchronize(nullptr) != VX_OK)
        GGML_ABORT("ggml-gfx950: set_tensor failed: %s", vx_last_error());
}

void buffer_get_tensor(ggml_backend_buffer_t buffer, const ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    vx_init(ctx->device);
    if (vx_memcpy_d2h(data, (const char *) tensor->data + offset, size, nullptr) != VX_OK || vx_stream_synchronize(nullptr) != VX_OK)
        GGML_ABORT("ggml-gfx950: get_tensor failed: %s", vx_last_error());
}

bool buffer_cpy_tensor(ggml_backend_buffer_t buffer, const ggml_tensor * src, ggml_tensor * dst) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    if (!ggml_is_contiguous(src) || !ggml_is_contiguous(dst) || ggml_nbytes(src) != ggml_nbytes(dst)) return false;
    vx_init(ctx->device);
    written_to(buffer, dst->data, ggml_nbytes(dst));
    vx_status rc;
    if (ggml_backend_buffer_is_host(src->buffer)) {
        rc = vx_memcpy_h2d(dst->data, src->data, ggml_nbytes(src), nullptr);
    } else if (src->buffer->buft == buffer->buft) {
        rc = vx_memcpy_d2d(dst->data, src->data, ggml_nbytes(src), nullptr);
    } else {
        return false;
    }
    if (rc == VX_OK) rc = vx_stream_synchronize(nullptr);
    if (rc != VX_OK) GGML_ABORT("ggml-gfx950: cpy_tensor failed: %s", vx_last_error());
    return true;
}

void buffer_clear(ggml_backend_buffer_t buffer, uint8_t value) {
    buffer_ctx * ctx = (buffer_ctx *) buffer->context;
    vx_init(ctx->device);
    written_to(buffer, ctx->base, buffer->size);
    if (vx_memset(ctx->base, value, buffer->size, nullptr) != VX_OK || vx_stream_synchronize(nullptr) != VX_OK)
        GGML_ABORT("ggml-gfx950: clear failed: %s", vx_last_error());
}

const ggml_backend_buffer_i buffer_iface = {
    /* .free_buffer   = */ buffer_free,
    /* .get_base      = */ buffer_get_base,
    /* .init_tensor   = */ nullptr,
    /* .memset_tensor = */ buffer_memset_tensor,
    /* .set_tensor    = */ buffer_set_tensor,
    /* .get_tensor    = */ buffer_get_tensor,
    /* .cpy_tensor    = */ buffer_cpy_tensor,
    /* .clear         = */ buffer_clear,
    /* .reset         = */ nullptr,
};

// -------------------------------------------------------------------- device buffer type
const char * buft_get_name(ggml_backend_buffer_type_t buft) {
    return ((device_ctx *) buft->device->context)->name.c_str();
}

ggml_backend_buffer_t buft_alloc_buffer(ggml_backend_buffer_type_t buft, size_t size) {
    device_ctx * dctx = (device_ctx *) buft->device->context;
    if (vx_init(dctx->index) != VX_OK) {
        GGML_LOG_ERROR("ggml-gfx950: %s\n", vx_last_error());
        return nullptr;
    }
    void * base = nullptr;
    if (vx_malloc(&base, size) != VX_OK) {
        GGML_LOG_ERROR("ggml-gfx950: allocating %zu bytes on %s failed: %s\n", size, dctx->name.c_str(), vx_last_error());
        return nullptr;
    }
    return ggml_backend_buffer_init(buft, buffer_iface, new buffer_ctx{ dctx->index, base }, size);
}

size_t buft_get_alignment(ggml_backend_buffer_type_t) { return GFX950_ALIGNMENT; }

bool buft_is_host(ggml_backend_buffer_type_t) { return false; }

// ---------------------------------------------------------------- pinned host buffer type
// System memory allocated with hipHostMalloc: when ggml's scheduler puts its CPU-side compute
// buffers here (as VoxCPM.cpp does for CUDA, src/backend.cpp:275-281), split copies are DMA
// from pinned memory.  Tensor access is ggml's own CPU buffer code.
void host_buffer_free(ggml_backend_buffer_t buffer) { vx_free_host(buffer->context); }

const char * host_buft_get_name(ggml_backend_buffer_type_t) { return "GFX950_Host"; }

ggml_backend_buffer_t host_buft_alloc_buffer(ggml_backend_buffer_type_t buft, size_t size) {
    void * ptr = nullptr;
    if (vx_malloc_host(&ptr, size) != VX_OK) {
        GGML_LOG_WARN("ggml-gfx950: pinned allocation of %zu bytes failed (%s), using pageable memory\n", size, vx_last_error());
        return ggml_backend_buft_alloc_buffer(ggml_backend_cpu_buffer_type(), size);
    }
    ggml_backend_buffer_t buffer = ggml_backend_cpu_buffer_from_ptr(ptr, size);
    buffer->buft              = buft;
    buffer->iface.free_buffer = host_buffer_free;
    return buffer;
}

size_t host_buft_get_alignment(ggml_backend_buffer_type_t) { return GFX950_ALIGNMENT; }
bool   host_buft_is_host(ggml_backend_buffer_type_t) { return true; }

// ----------------------------------------------------------------------------- supports_op
bool supports_op(ggml_backend_dev_t, const ggml_tensor * op) {
    for (int i = 0; i < GGML_MAX_SRC; ++i)
        if (op->src[i] && !type_known(op->src[i]->type)) return false;

    switch (op->op) {
        case GGML_OP_NONE:
        case GGML_OP_RESHAPE:
        case GGML_OP_VIEW:
        case GGML_OP_PERMUTE:
        case GGML_OP_TRANSPOSE:
            return true;
        case GGML_OP_RMS_NORM: {
            const vx_tensor s = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_rms_norm(&s, &d) != 0;
        }
        case GGML_OP_ROPE: {
            const int n_dims = ((const int32_t *) op->op_params)[1];
            const int mode   = ((const int32_t *) op->op_params)[2];
            if (op->src[1] == nullptr || op->src[1]->type != GGML_TYPE_I32) return false;
            if (op->src[2] && (op->src[2]->type != GGML_TYPE_F32 || op->src[2]->ne[0] < n_dims / 2)) return false;
            const vx_tensor s = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_rope(&s, &d, n_dims, mode) != 0;
        }
        case GGML_OP_SOFT_MAX: {
            const vx_tensor s = to_vx(op->src[0]), d = to_vx(op);
            vx_tensor m;
            if (op->src[1]) m = to_vx(op->src[1]);
            if (op->src[2] && (op->src[2]->type != GGML_TYPE_F32 || op->src[2]->ne[0] != op->src[0]->ne[2])) return false;
            return vx_supports_soft_max(&s, op->src[1] ? &m : nullptr, &d) != 0;
        }
        case GGML_OP_FLASH_ATTN_EXT: {
            const vx_tensor q = to_vx(op->src[0]), k = to_vx(op->src[1]), v = to_vx(op->src[2]), d = to_vx(op);
            vx_tensor m;
            if (op->src[3]) m = to_vx(op->src[3]);
            if (op->src[4] && (op->src[4]->type != GGML_TYPE_F32 || op->src[4]->ne[0] != op->src[0]->ne[2])) return false;
            return vx_supports_flash_attn_ext(&q, &k, &v, op->src[3] ? &m : nullptr, &d) != 0;
        }
        case GGML_OP_MUL_MAT: {
            const vx_tensor a = to_vx(op->src[0]), b = to_vx(op->src[1]), d = to_vx(op);
            return vx_supports_mul_mat(&a, &b, &d) != 0;
        }
        case GGML_OP_ADD:
        case GGML_OP_SUB:
        case GGML_OP_MUL:
        case GGML_OP_DIV: {
            const vx_tensor a = to_vx(op->src[0]), b = to_vx(op->src[1]), d = to_vx(op);
            return vx_supports_binary(binary_code(op->op), &a, &b, &d) != 0;
        }
        case GGML_OP_ADD1: {
            const vx_tensor a = to_vx(op->src[0]), b = to_vx(op->src[1]), d = to_vx(op);
            return vx_supports_add1(&a, &b, &d) != 0;
        }
        case GGML_OP_SCALE: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_unary_like(&a, &d) != 0;
        }
        case GGML_OP_UNARY: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_unary((int) ggml_get_unary_op(op), &a, &d) != 0;
        }
        case GGML_OP_GLU: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            vx_tensor b;
            if (op->src[1]) b = to_vx(op->src[1]);
            return vx_supports_glu((int) ggml_get_glu_op(op), &a, op->src[1] ? &b : nullptr, &d) != 0;
        }
        case GGML_OP_DUP:
        case GGML_OP_CPY:
        case GGML_OP_CONT: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_cpy(&a, &d) != 0;
        }
        case GGML_OP_CONCAT: {
            const vx_tensor a = to_vx(op->src[0]), b = to_vx(op->src[1]), d = to_vx(op);
            return vx_supports_concat(&a, &b, &d, ((const int32_t *) op->op_params)[0]) != 0;
        }
        case GGML_OP_SUM: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_sum(&a, &d) != 0;
        }
        case GGML_OP_SUM_ROWS: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_sum_rows(&a, &d) != 0;
        }
        case GGML_OP_SQR:
        case GGML_OP_SQRT:
        case GGML_OP_LOG:
        case GGML_OP_SIN:
        case GGML_OP_COS: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_unary(standalone_unary_code(op->op), &a, &d) != 0;
        }
        case GGML_OP_ARANGE: {
            const vx_tensor d = to_vx(op);
            return vx_supports_arange(&d) != 0;
        }
        case GGML_OP_REPEAT: {
            const vx_tensor a = to_vx(op->src[0]), d = to_vx(op);
            return vx_supports_repeat(&a, &d) != 0;
        }
        case GGML_OP_GET_ROWS: {
            const vx_tensor a = to_vx(op->src[0]), b = to_vx(op->src[1]), d = to_vx(op);
            return vx_supports_get_rows(&a, &b, &d) != 0;
        }
        default:
            return false;
    }
}

// --------------------------------------------------------------------------- graph_compute
vx_status compute_node(backend_ctx * ctx, ggml_tensor * node) {
    switch (node->op) {
        case GGML_OP_ADD:
        case GGML_OP_SUB:
        case GGML_OP_MUL:
        case GGML_OP_DIV: {
            const vx_tensor a = to_vx(node->src[0]), b = to_vx(node->src[1]), d = to_vx(node);
            return vx_binary(binary_code(node->op), &a, &b, &d, ctx->stream);
        }
        case GGML_OP_ADD1: {
            const vx_tensor a = to_vx(node->src[0]), b = to_vx(node->src[1]), d = to_vx(node);
            return vx_add1(&a, &b, &d, ctx->stream);
        }
        case GGML_OP_SCALE: {
            float sc, bias; // ggml.c: scale, bias
            memcpy(&sc, (const float *) node->op_params + 0, sizeof(float));
            memcpy(&bias, (const float *) node->op_params + 1, sizeof(float));
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_scale(&a, &d, sc, bias, ctx->stream);
        }
        case GGML_OP_UNARY: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_unary((int) ggml_get_unary_op(node), &a, &d, ctx->stream);
        }
        case GGML_OP_GLU: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            vx_tensor b;
            if (node->src[1]) b = to_vx(node->src[1]);
            return vx_glu((int) ggml_get_glu_op(node), &a, node->src[1] ? &b : nullptr, &d,
                          ((const int32_t *) node->op_params)[1], ctx->stream);
        }
        case GGML_OP_DUP:
        case GGML_OP_CPY:
        case GGML_OP_CONT: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_cpy(&a, &d, ctx->stream);
        }
        case GGML_OP_CONCAT: {
            const vx_tensor a = to_vx(node->src[0]), b = to_vx(node->src[1]), d = to_vx(node);
            return vx_concat(&a, &b, &d, ((const int32_t *) node->op_params)[0], ctx->stream);
        }
        case GGML_OP_SUM: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_sum(&a, &d, ctx->stream);
        }
        case GGML_OP_SUM_ROWS: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_sum_rows(&a, &d, ctx->stream);
        }
        case GGML_OP_SQR:
        case GGML_OP_SQRT:
        case GGML_OP_LOG:
        case GGML_OP_SIN:
        case GGML_OP_COS: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_unary(standalone_unary_code(node->op), &a, &d, ctx->stream);
        }
        case GGML_OP_ARANGE: {
            float start, step; // ggml.c: start, stop, step
            memcpy(&start, (const float *) node->op_params + 0, sizeof(float));
            memcpy(&step, (const float *) node->op_params + 2, sizeof(float));
            const vx_tensor d = to_vx(node);
            return vx_arange(&d, start, step, ctx->stream);
        }
        case GGML_OP_REPEAT: {
            const vx_tensor a = to_vx(node->src[0]), d = to_vx(node);
            return vx_repeat(&a, &d, ctx->stream);
        }
        case GGML_OP_GET_ROWS: {
            const vx_tensor a = to_vx(node->src[0]), b = to_vx(node->src[1]), d = to_vx(node);
            return vx_get_rows(&a, &b, &d, ctx->stream);
        }
        case GGML_OP_RMS_NORM: {
            float eps;
            memcpy(&eps, node->op_params, sizeof(float));
            const vx_tensor s = to_vx(node->src[0]), d = to_vx(node);
            return vx_rms_norm(&s, &d, eps, ctx->stream);
        }
        case GGML_OP_ROPE: {
            const int32_t * p = (const int32_t *) node->op_params; // ggml.c:4112-4123
            float f[6];
            memcpy(f, p + 5, sizeof(f));
            const vx_tensor s = to_vx(node->src[0]), d = to_vx(node);
            return vx_rope(&s, (const int32_t *) node->src[1]->data, node->src[2] ? (const float *) node->src[2]->data : nullptr,
                           &d, p[1], p[2], p[4], f[0], f[1], f[2], f[3], f[4], f[5], ctx->stream);
        }
        case GGML_OP_SOFT_MAX: {
            float scale, max_bias;
            memcpy(&scale, (const float *) node->op_params + 0, sizeof(float));
            memcpy(&max_bias, (const float *) node->op_params + 1, sizeof(float));
            const vx_tensor s = to_vx(node->src[0]), d = to_vx(node);
            vx_tensor m;
            if (node->src[1]) m = to_vx(node->src[1]);
            return vx_soft_max(&s, node->src[1] ? &m : nullptr, node->src[2] ? (const float *) node->src[2]->data : nullptr,
                               &d, scale, max_bias, ctx->stream);
        }
        case GGML_OP_FLASH_ATTN_EXT: {
            float scale, max_bias, softcap; // ggml.c:5312-5313
            memcpy(&scale, (const float *) node->op_params + 0, sizeof(float));
            memcpy(&max_bias, (const float *) node->op_params + 1, sizeof(float));
            memcpy(&softcap, (const float *) node->op_params + 2, sizeof(float));
            const vx_tensor q = to_vx(node->src[0]), k = to_vx(node->src[1]), v = to_vx(node->src[2]), d = to_vx(node);
            vx_tensor m;
            if (node->src[3]) m = to_vx(node->src[3]);
            return vx_flash_attn_ext(&q, &k, &v, node->src[3] ? &m : nullptr,
                                     node->src[4] ? (const float *) node->src[4]->data : nullptr, &d, scale, max_bias,
                                     softcap, ctx->stream);
        }
        case GGML_OP_MUL_MAT: {
            const vx_tensor a = to_vx(node->src[0]), b = to_vx(node->src[1]), d = to_vx(node);
            return vx_mul_mat(&a, &b, &d, mul_mat_act_mode(), ctx->stream);
        }
        default:
            return VX_ERR_UNSUPPORTED;
    }
}

const char * backend_get_name(ggml_backend_t backend) {
    return ((device_ctx *) backend->device->context)->name.c_str();
}

void backend_free(ggml_backend_t backend) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    vx_init(ctx->device);
    vx_stream_synchronize(ctx->stream);
    for (seen_graph & g : ctx->seen) if (g.recorded) vx_graph_destroy(g.recorded);
    for (step_family & f : ctx->families) for (vx_graph & r : f.recorded) if (r) vx_graph_destroy(r);
    vx_stream_destroy(ctx->stream);
    delete ctx;
    delete backend;
}

void backend_synchronize(ggml_backend_t backend) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    vx_init(ctx->device);
    if (vx_stream_synchronize(ctx->stream) != VX_OK) GGML_ABORT("ggml-gfx950: synchronize failed: %s", vx_last_error());
}

void backend_set_tensor_async(ggml_backend_t backend, ggml_tensor * tensor, const void * data, size_t offset, size_t size) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    vx_init(ctx->device);
    written_to(tensor->buffer, (char *) tensor->data + offset, size);
    if (vx_memcpy_h2d((char *) tensor->data + offset, data, size, ctx->stream) != VX_OK)
        GGML_ABORT("ggml-gfx950: set_tensor_async failed: %s", vx_last_error());
}

void backend_get_tensor_async(ggml_backend_t backend, const ggml_tensor * tensor, void * data, size_t offset, size_t size) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    vx_init(ctx->device);
    if (vx_memcpy_d2h(data, (const char *) tensor->data + offset, size, ctx->stream) != VX_OK)
        GGML_ABORT("ggml-gfx950: get_tensor_async failed: %s", vx_last_error());
}

// ggml-alloc hands a node's output the memory of tensors that died before it.  Run as separate
// launches that is harmless; one launch that covers several nodes writes the last node's output while
// it may still be reading an operand of the first, so every group checks where its output lies.
bool overlaps(const ggml_tensor * a, const ggml_tensor * b) {
    if (!a || !b || !a->data || !b->data) return false;
    const char * a0 = (const char *) a->data;
    const char * b0 = (const char *) b->data;
    return a0 < b0 + ggml_nbytes(b) && b0 < a0 + ggml_nbytes(a);
}
// operand that work-groups other than the one writing an output element read: must not touch dst
bool apart(const ggml_tensor * dst, const ggml_tensor * in) { return !overlaps(dst, in); }
// Two views that interleave in memory without sharing an element, like the cached keys [0, n_past) and the slot
// being written [n_past, n_past + n_tokens) of one KV cache tensor: every row of the small view is located in
// the regular lattice of the big one (rows of ne0 elements every nb1 bytes, ne1 of them every nb2, ...).
bool apart_rows(const ggml_tensor * small, const ggml_tensor * big) {
    if (!overlaps(small, big)) return true;
    const size_t es = ggml_type_size(big->type);
    if (ggml_is_quantized(big->type) || ggml_is_quantized(small->type) || small->nb[0] != ggml_type_size(small->type) || big->nb[0] != es) return false;
    const int64_t big_row = (int64_t) (es * big->ne[0]), len = (int64_t) (small->nb[0] * small->ne[0]);
    if ((int64_t) big->nb[1] < big_row || big->nb[2] < big->nb[1] * (size_t) big->ne[1] || big->nb[3] < big->nb[2] * (size_t) big->ne[2]) return false;
    if (small->ne[1] * small->ne[2] * small->ne[3] > 65536) return false;
    for (int64_t i3 = 0; i3 < small->ne[3]; ++i3)
        for (int64_t i2 = 0; i2 < small->ne[2]; ++i2)
            for (int64_t i1 = 0; i1 < small->ne[1]; ++i1) {
                const int64_t o = ((const char *) small->data + i1 * small->nb[1] + i2 * small->nb[2] + i3 * small->nb[3]) - (const char *) big->data;
                if (o + len <= 0) continue;
                if (o < 0) return false;
                const int64_t j3 = o / (int64_t) big->nb[3], r3 = o % (int64_t) big->nb[3];
                const int64_t j2 = r3 / (int64_t) big->nb[2], r2 = r3 % (int64_t) big->nb[2];
                const int64_t j1 = r2 / (int64_t) big->nb[1], rem = r2 % (int64_t) big->nb[1];
                if (rem + len > (int64_t) big->nb[1]) return false; // reaches into the next row: not worth deciding
                if (j3 < big->ne[3] && j2 < big->ne[2] && j1 < big->ne[1] && rem < big_row) return false;
            }
    return true;
}
// operand whose element i is read only by the thread that writes element i of dst: may also BE dst
bool apart_or_same(const ggml_tensor * dst, const ggml_tensor * in) {
    if (!overlaps(dst, in)) return true;
    if (dst->data != in->data) return false;
    for (int i = 0; i < GGML_MAX_DIMS; ++i)
        if (dst->ne[i] != in->ne[i] || dst->nb[i] != in->nb[i]) return false;
    return true;
}

// Two consecutive nodes as one launch, when the first one's value has no other reader (checked by
// the caller).  Returns false when the pair is not one of the known shapes; *rc is the launch status.
bool compute_pair(backend_ctx * ctx, ggml_tensor * node, ggml_tensor * next, vx_status * rc) {
    const vx_tensor d = to_vx(next);
    if (node->op == GGML_OP_RMS_NORM && next->op == GGML_OP_MUL && next->src[0] == node) {
        // MiniCPMModel::rms_norm: ggml_mul(ggml_rms_norm(x), weight)
        const vx_tensor s = to_vx(node->src[0]), w = to_vx(next->src[1]);
        if (!vx_supports_rms_norm_mul(&s, &w, &d) || !apart_or_same(next, node->src[0]) || !apart(next, next->src[1])) return false;
        float eps;
        memcpy(&eps, node->op_params, sizeof(float));
        *rc = vx_rms_norm_mul(&s, &w, &d, eps, ctx->stream);
        return true;
    }
    if (node->op == GGML_OP_SCALE && next->op == GGML_OP_ADD && next->src[1] == node && next->src[0] != node) {
        float sc, bias;
        memcpy(&sc, (const float *) node->op_params + 0, sizeof(float));
        memcpy(&bias, (const float *) node->op_params + 1, sizeof(float));
        const vx_tensor a = to_vx(next->src[0]), x = to_vx(node->src[0]);
        if (bias != 0.0f || !vx_supports_fused_pair(&a, &x, &d) || !apart_or_same(next, next->src[0]) || !apart_or_same(next, node->src[0])) return false;
        *rc = vx_scale_add(&a, &x, &d, sc, ctx->stream);
        return true;
    }
    if (node->op == GGML_OP_ADD && next->op == GGML_OP_SCALE && next->src[0] == node) {
        float sc, bias;
        memcpy(&sc, (const float *) next->op_params + 0, sizeof(float));
        memcpy(&bias, (const float *) next->op_params + 1, sizeof(float));
        const vx_tensor a = to_vx(node->src[0]), b = to_vx(node->src[1]);
        if (!vx_supports_fused_pair(&a, &b, &d) || !apart_or_same(next, node->src[0]) || !apart_or_same(next, node->src[1])) return false;
        *rc = vx_add_scale(&a, &b, &d, sc, bias, ctx->stream);
        return true;
    }
    if (node->op == GGML_OP_FLASH_ATTN_EXT && next->op == GGML_OP_ADD1 && next->src[0] == node && next->src[1] != node &&
        next->src[1]->type == GGML_TYPE_F32 && ggml_nelements(next->src[1]) == 1) {
        // attention_forward's ggml_add1(attn, kv_sync): the scalar is added in the attention kernel's epilogue
        const vx_tensor q = to_vx(node->src[0]), k = to_vx(node->src[1]), v = to_vx(node->src[2]);
        vx_tensor m;
        if (node->src[3]) m = to_vx(node->src[3]);
        if (node->src[4] && (node->src[4]->type != GGML_TYPE_F32 || node->src[4]->ne[0] != node->src[0]->ne[2])) return false;
        if (!vx_supports_flash_attn_ext(&q, &k, &v, node->src[3] ? &m : nullptr, &d)) return false;
        for (int k_ = 0; k_ < 5; ++k_) if (!apart(next, node->src[k_])) return false;
        if (!apart(next, next->src[1])) return false;
        float scale, max_bias, softcap;
        memcpy(&scale, (const float *) node->op_params + 0, sizeof(float));
        memcpy(&max_bias, (const float *) node->op_params + 1, sizeof(float));
        memcpy(&softcap, (const float *) node->op_params + 2, sizeof(float));
        *rc = vx_flash_attn_ext_add1(&q, &k, &v, node->src[3] ? &m : nullptr, node->src[4] ? (const float *) node->src[4]->data : nullptr,
                                     (const float *) next->src[1]->data, &d, scale, max_bias, softcap, ctx->stream);
        return true;
    }
    if (node->op == GGML_OP_CONT && next->op == GGML_OP_SUM && next->src[0] == node) {
        // the sum does not care where the elements lie: read them where they are
        const vx_tensor s = to_vx(node->src[0]);
        if (node->src[0]->type != GGML_TYPE_F32 || !vx_supports_sum(&s, &d) || !apart(next, node->src[0])) return false;
        *rc = vx_sum(&s, &d, ctx->stream);
        return true;
    }
    return false;
}

// tensor -> count, for the graph analysis that runs in front of the first launch of every graph_compute: a flat
// open-addressing table (a node-based map costs more than 100 us on a 1200-node graph, all of it latency of the call)
class reader_map {
  public:
    struct slot { const ggml_tensor * first; int second; };
    void reserve(size_t n) {
        size_t cap = 64;
        while (cap < 2 * n) cap <<= 1;
        if (cap <= slots_.size()) return;
        std::vector<slot> old;
        old.swap(slots_);
        slots_.assign(cap, slot{ nullptr, 0 });
        used_ = 0;
        for (const slot & o : old) if (o.first) (*this)[o.first] = o.second;
    }
    int & operator[](const ggml_tensor * key) {
        if (2 * (used_ + 1) > slots_.size()) reserve(slots_.empty() ? 32 : slots_.size());
        slot * s = probe(key);
        if (!s->first) { s->first = key; ++used_; }
        return s->second;
    }
    const slot * find(const ggml_tensor * key) const {
        if (slots_.empty()) return nullptr;
        const slot * s = const_cast<reader_map *>(this)->probe(key);
        return s->first ? s : nullptr;
    }
    const slot * end() const { return nullptr; }

  private:
    slot * probe(const ggml_tensor * key) {
        const size_t mask = slots_.size() - 1;
        size_t i = (size_t) ((((uintptr_t) key >> 4) * 0x9E3779B97F4A7C15ull) >> 32) & mask;
        while (slots_[i].first && slots_[i].first != key) i = (i + 1) & mask;
        return &slots_[i];
    }
    std::vector<slot> slots_;
    size_t            used_ = 0;
};

// a node whose value only the group's next member looks at, so it need not be stored
bool private_to_group(const reader_map & readers, const ggml_tensor * t) {
    const auto it = readers.find(t);
    return (t->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 && (t->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 && it != readers.end() && it->second == 1;
}

// the same for the result of ggml_cast, a CPY node that names itself as its second operand (one reader more)
bool private_cast_node(const reader_map & readers, const ggml_tensor * t) {
    const auto it = readers.find(t);
    return t->op == GGML_OP_CPY && t->src[1] == t && (t->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 && (t->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 &&
           it != readers.end() && it->second == 2;
}

// index of the next node that does work (views and empty tensors are skipped), or n_nodes
int next_real(const ggml_cgraph * g, int i) {
    int k = i + 1;
    while (k < g->n_nodes && (ggml_op_is_empty(g->nodes[k]->op) || ggml_is_empty(g->nodes[k]))) ++k;
    return k;
}

// attention_forward's cache write and ordering scalar (src/minicpm.cpp:682-713) at decode size:
//   CPY(k, slot) CONT SUM , CPY(v, slot) CONT SUM , ADD , SCALE , ADD1(attn, .)     -> one launch.
// Returns the index of the group's last node, or -1.
// the nine nodes from index i on, checked for shape and privacy; returns the index of the last one or -1
int match_kv_store_group(const ggml_cgraph * g, int i, const reader_map & readers, ggml_tensor * n[9]) {
    int idx = i;
    for (int k = 0; k < 9; ++k) {
        if (idx >= g->n_nodes) return -1;
        n[k] = g->nodes[idx];
        if ((n[k]->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) return -1;
        if (k < 8) idx = next_real(g, idx);
    }
    // (with an F16 cache the sums are typed F32 through a cast of the written slot, CPY to a new F32 tensor, where the F32
    // cache has its CONT)
    static const ggml_op want[9] = { GGML_OP_CPY, GGML_OP_CONT, GGML_OP_SUM, GGML_OP_CPY, GGML_OP_CONT, GGML_OP_SUM, GGML_OP_ADD, GGML_OP_SCALE, GGML_OP_ADD1 };
    for (int k = 0; k < 9; ++k) {
        const bool cast_back = (k == 1 || k == 4) && n[k]->op == GGML_OP_CPY && n[k - 1]->type == GGML_TYPE_F16 && n[k]->src[1] == n[k] &&
                               ggml_is_contiguous(n[k]);
        if (n[k]->op != want[k] && !cast_back) return -1;
    }
    if (n[1]->src[0] != n[0] || n[2]->src[0] != n[1] || n[4]->src[0] != n[3] || n[5]->src[0] != n[4]) return -1;
    if (!((n[6]->src[0] == n[2] && n[6]->src[1] == n[5]) || (n[6]->src[0] == n[5] && n[6]->src[1] == n[2]))) return -1;
    if (n[7]->src[0] != n[6] || n[8]->src[1] != n[7]) return -1;
    ggml_tensor * x = n[8]->src[0];
    for (int k = 0; k < 8; ++k) {
        const bool cast_back = (k == 1 || k == 4) && n[k]->op == GGML_OP_CPY;
        if (x == n[k] || !(cast_back ? private_cast_node(readers, n[k]) : private_to_group(readers, n[k]))) return -1;
    }
    // the copies must be plain F32 -> F32 / F16 writes into the cache (the CPY node is a view of its destination)
    for (int c = 0; c < 4; c += 3) {
        if (n[c]->src[0]->type != GGML_TYPE_F32 || (n[c]->type != GGML_TYPE_F32 && n[c]->type != GGML_TYPE_F16) || n[c]->src[1] == nullptr ||
            n[c]->data != n[c]->src[1]->data) return -1;
        if (n[c + 1]->type != GGML_TYPE_F32) return -1;
        if ((n[c]->type == GGML_TYPE_F16) != (n[c + 1]->op == GGML_OP_CPY)) return -1;
    }
    ggml_tensor * dst = n[8];
    if (!apart(dst, n[0]->src[0]) || !apart(dst, n[3]->src[0]) || !apart(dst, n[0]) || !apart(dst, n[3]) || !apart_or_same(dst, x)) return -1;
    if (!apart(n[0], x) || !apart(n[3], x) || !apart(n[0], n[3]->src[0]) || !apart(n[3], n[0]->src[0]) || !apart(n[0], n[3])) return -1;
    return idx;
}

int compute_kv_store_group(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers, vx_status * rc) {
    ggml_tensor * n[9];
    const int idx = match_kv_store_group(g, i, readers, n);
    if (idx < 0) return -1;
    ggml_tensor * x = n[8]->src[0];
    ggml_tensor * dst = n[8];
    const vx_tensor k = to_vx(n[0]->src[0]), ks = to_vx(n[0]), v = to_vx(n[3]->src[0]), vs = to_vx(n[3]), xx = to_vx(x), d = to_vx(dst);
    if (!vx_supports_kv_store_sync(&k, &ks, &v, &vs, &xx, &d)) return -1;
    float sc, bias;
    memcpy(&sc, (const float *) n[7]->op_params + 0, sizeof(float));
    memcpy(&bias, (const float *) n[7]->op_params + 1, sizeof(float));
    *rc = vx_kv_store_sync(&k, &ks, &v, &vs, &xx, &d, sc, bias, ctx->stream);
    return idx;
}

// A graph node as a node of vx_small_graph (tiny elementwise / copy / concat / repeat / sum / row-sum / arange work); t holds the
// descriptors the node points to.  False for every other operator and for tensors above the small-graph size.
bool small_node_of(const ggml_tensor * n, vx_small_node * out, vx_tensor (&t)[3]) {
    *out = vx_small_node{};
    t[2] = to_vx(n);
    out->dst = &t[2];
    if (n->src[0]) { t[0] = to_vx(n->src[0]); out->src0 = &t[0]; }
    bool two = false;
    switch (n->op) {
        case GGML_OP_ADD: case GGML_OP_SUB: case GGML_OP_MUL: case GGML_OP_DIV:
            out->op = VX_NODE_ADD + binary_code(n->op); two = true; break;
        case GGML_OP_ADD1:   out->op = VX_NODE_ADD1; two = true; break;
        case GGML_OP_SCALE:
            out->op = VX_NODE_SCALE;
            memcpy(&out->p0, (const float *) n->op_params + 0, sizeof(float));
            memcpy(&out->p1, (const float *) n->op_params + 1, sizeof(float));
            break;
        case GGML_OP_UNARY:  out->op = VX_NODE_UNARY; out->aux = (int) ggml_get_unary_op(n); break;
        case GGML_OP_SQR: case GGML_OP_SQRT: case GGML_OP_LOG: case GGML_OP_SIN: case GGML_OP_COS:
            out->op = VX_NODE_UNARY; out->aux = standalone_unary_code(n->op); break;
        case GGML_OP_DUP: case GGML_OP_CPY: case GGML_OP_CONT: out->op = VX_NODE_CPY; break;
        case GGML_OP_CONCAT: out->op = VX_NODE_CONCAT; out->aux = ((const int32_t *) n->op_params)[0]; two = true; break;
        case GGML_OP_REPEAT: out->op = VX_NODE_REPEAT; break;
        case GGML_OP_SUM:    out->op = VX_NODE_SUM; break;
        case GGML_OP_SUM_ROWS: out->op = VX_NODE_SUM_ROWS; break;
        case GGML_OP_ARANGE:
            out->op = VX_NODE_ARANGE;
            memcpy(&out->p0, (const float *) n->op_params + 0, sizeof(float));
            memcpy(&out->p1, (const float *) n->op_params + 2, sizeof(float));
            out->src0 = nullptr;
            break;
        default: return false;
    }
    if (n->op != GGML_OP_ARANGE && !n->src[0]) return false;
    if (two) {
        if (!n->src[1]) return false;
        t[1] = to_vx(n->src[1]);
        out->src1 = &t[1];
    }
    return vx_supports_small_node(out) != 0;
}

// The run of tiny nodes that starts at node i (at most 16, view nodes in between skipped) as ONE launch: the bias adds,
// sequence-assembling CONCATs, guidance arithmetic and Euler update around the LocDiT estimator (src/locdit.cpp:401-464,
// src/unified_cfm.cpp:30-149).  A node all of whose readers are members of the run (and which is no graph output) is
// marked private: the kernel may keep it in LDS only.  Every other node writes its own tensor, in graph order.
// The run stops in front of anything another group claims.  Returns the index of the run's last node, or -1 when fewer
// than two nodes qualify.
int compute_small_run(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers,
                      const std::unordered_map<const ggml_tensor *, const ggml_tensor *> & absorbed,
                      const std::unordered_set<const ggml_tensor *> & done, vx_status * rc) {
    constexpr int MAX_RUN = 16;
    vx_small_node nodes[MAX_RUN];
    vx_tensor     ts[MAX_RUN][3];
    int count = 0, last = -1;
    for (int j = i; j < g->n_nodes && count < MAX_RUN; ++j) {
        const ggml_tensor * n = g->nodes[j];
        if (ggml_op_is_empty(n->op) || ggml_is_empty(n)) continue;
        if ((n->flags & GGML_TENSOR_FLAG_COMPUTE) == 0 || absorbed.count(n) || done.count(n)) break;
        if (n->op == GGML_OP_CPY) { // the cache-write group has its own launch
            ggml_tensor * tmp[9];
            if (match_kv_store_group(g, j, readers, tmp) >= 0) break;
        }
        if (!small_node_of(n, &nodes[count], ts[count])) break;
        ++count;
        last = j;
    }
    if (count < 2) return -1;
    // readers inside the run, per member (a view of a member is a reader outside it: views are not members)
    const ggml_tensor * member[MAX_RUN];
    int inside[MAX_RUN] = {0};
    {
        int m = 0;
        for (int j = i; j <= last; ++j) {
            const ggml_tensor * n = g->nodes[j];
            if (ggml_op_is_empty(n->op) || ggml_is_empty(n)) continue;
            member[m++] = n;
        }
        for (int k = 0; k < count; ++k)
            for (int sidx = 0; sidx < GGML_MAX_SRC; ++sidx) {
                const ggml_tensor * src = member[k]->src[sidx];
                if (!src) continue;
                for (int q = 0; q < k; ++q) if (member[q] == src) ++inside[q];
            }
    }
    for (int k = 0; k + 1 < count; ++k) { // (the last member has no reader in the run)
        const auto it = readers.find(member[k]);
        const bool out = (member[k]->flags & GGML_TENSOR_FLAG_OUTPUT) != 0;
        if (!out && it != readers.end() && it->second == inside[k] && inside[k] > 0) nodes[k].flags |= VX_SMALL_DST_PRIVATE;
    }
    *rc = vx_small_graph(nodes, count, ctx->stream);
    return last;
}

// layer_forward's residual updates (src/minicpm.cpp:762-777) at decode size:
//   MUL_MAT(w, x) [SCALE] ADD(residual, .)   -> one launch.  Returns the index of the ADD, or -1.
int compute_mul_mat_residual_group(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers, vx_status * rc) {
    ggml_tensor * mm = g->nodes[i];
    if (mm->op != GGML_OP_MUL_MAT || !private_to_group(readers, mm) || i + 1 >= g->n_nodes) return -1;
    ggml_tensor * val = mm;
    float sc = 1.0f;
    int ia = i + 1;
    if (g->nodes[ia]->op == GGML_OP_SCALE) {
        ggml_tensor * scn = g->nodes[ia];
        float bias;
        memcpy(&sc, (const float *) scn->op_params + 0, sizeof(float));
        memcpy(&bias, (const float *) scn->op_params + 1, sizeof(float));
        if (scn->src[0] != mm || bias != 0.0f || !private_to_group(readers, scn)) return -1;
        val = scn;
        if (++ia >= g->n_nodes) return -1;
    }
    ggml_tensor * add = g->nodes[ia];
    if (add->op != GGML_OP_ADD || (add->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) return -1;
    ggml_tensor * residual = add->src[0] == val ? add->src[1] : add->src[0];
    if ((add->src[0] != val && add->src[1] != val) || residual == val || residual == mm) return -1;
    if (!apart(add, mm->src[0]) || !apart(add, mm->src[1]) || !apart_or_same(add, residual)) return -1;
    const vx_tensor w = to_vx(mm->src[0]), x = to_vx(mm->src[1]), r = to_vx(residual), d = to_vx(add);
    if (!vx_supports_mul_mat_scale_add(&w, &x, &r, &d)) return -1;
    *rc = vx_mul_mat_scale_add(&w, &x, &r, &d, sc, mul_mat_act_mode(), ctx->stream);
    return ia;
}

// attention_forward appends the step's keys and values to the cached ones with two CONCATs and hands
// the results to FLASH_ATTN_EXT (src/minicpm.cpp:694-706).  When nothing else reads the concatenated
// tensors, the attention kernel reads both segments where they lie and the CONCATs are never run.
// The CONCATs' operands must then still be intact when the attention node is reached: no node in
// between (nor the attention's own output) may have been given their memory.
// With an F16 cache the step's keys reach the CONCAT through a cast (CPY to a new F16 tensor).  When only the CONCAT
// reads the cast, the attention kernel reads the F32 source instead and rounds while it loads, and the cast is never run.
struct kv2_group {
    const ggml_tensor * kcat; const ggml_tensor * vcat;
    const ggml_tensor * kcur; const ggml_tensor * vcur; // the second segments as the kernel reads them
};

// the F32 source behind a private F32 -> F16 cast node, or null
const ggml_tensor * private_cast_source(const reader_map & readers, const ggml_tensor * t) {
    if (t->op != GGML_OP_CPY || t->src[1] != t || t->type != GGML_TYPE_F16 || !t->src[0] || t->src[0]->type != GGML_TYPE_F32) return nullptr;
    if (!private_cast_node(readers, t) || !ggml_are_same_shape(t, t->src[0])) return nullptr;
    return t->src[0];
}

void find_kv2_groups(const ggml_cgraph * g, const reader_map & readers, std::unordered_map<const ggml_tensor *, kv2_group> & by_fa,
                     std::unordered_map<const ggml_tensor *, const ggml_tensor *> & absorbed) {
    for (int i = 0; i < g->n_nodes; ++i) {
        const ggml_tensor * f = g->nodes[i];
        if (f->op != GGML_OP_FLASH_ATTN_EXT || (f->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) continue;
        const ggml_tensor * cat[2] = { f->src[1], f->src[2] };
        const ggml_tensor * cur[2] = { nullptr, nullptr };  // the second segment: the CONCAT's operand, or the source of its cast
        const ggml_tensor * cast[2] = { nullptr, nullptr };
        int at[2] = { -1, -1 };
        bool ok = true;
        for (int c = 0; c < 2 && ok; ++c) {
            ok = cat[c] && cat[c]->op == GGML_OP_CONCAT && ((const int32_t *) cat[c]->op_params)[0] == 1 && private_to_group(readers, cat[c]) &&
                 absorbed.find(cat[c]) == absorbed.end();
            if (!ok) break;
            cur[c] = cat[c]->src[1];
            const ggml_tensor * target = cat[c];
            if (const ggml_tensor * src = private_cast_source(readers, cur[c])) {
                if (absorbed.find(cur[c]) != absorbed.end()) { ok = false; break; }
                cast[c] = cur[c];
                cur[c]  = src;
                target  = cast[c];   // the F32 source must stay intact from the cast's position on
            }
            for (int k = i - 1; ok && k >= 0 && k >= i - 32; --k)
                if (g->nodes[k] == target) { at[c] = k; break; }
            ok = ok && at[c] >= 0;
        }
        if (!ok || cat[0] == cat[1] || (cast[0] == nullptr) != (cast[1] == nullptr)) continue;
        if (f->src[4] && (f->src[4]->type != GGML_TYPE_F32 || f->src[4]->ne[0] != f->src[0]->ne[2])) continue;
        const vx_tensor q = to_vx(f->src[0]), kp = to_vx(cat[0]->src[0]), kc = to_vx(cur[0]), vp = to_vx(cat[1]->src[0]),
                        vc = to_vx(cur[1]), d = to_vx(f);
        vx_tensor m;
        if (f->src[3]) m = to_vx(f->src[3]);
        if (!vx_supports_flash_attn_ext_kv2(&q, &kp, &kc, &vp, &vc, f->src[3] ? &m : nullptr, &d)) continue;
        for (int c = 0; c < 2 && ok; ++c)
            for (int k = at[c] + 1; k <= i && ok; ++k) {
                const ggml_tensor * n = g->nodes[k];
                if (n == cat[0] || n == cat[1] || n == cast[0] || n == cast[1] || ggml_op_is_empty(n->op) || ggml_is_empty(n) ||
                    (n->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) continue;
                ok = apart(n, cat[c]->src[0]) && apart(n, cur[c]);
            }
        if (!ok) continue;
        by_fa[f] = kv2_group{ cat[0], cat[1], cur[0], cur[1] };
        absorbed[cat[0]] = f;
        absorbed[cat[1]] = f;
        if (cast[0]) { absorbed[cast[0]] = f; absorbed[cast[1]] = f; }
    }
}

// LocDiT's sequence assembly for several requests at once (src/locdit.cpp:401-452 with a request dimension): CONCATs of
// CONCATs along one dimension, some leaves REPEATed to their slot first, every inner node read by its parent only.  Each
// inner node would copy its rows once more (a row reaches the pair through up to three copies); the tree's root is written
// from the leaves in one launch instead and the inner nodes are never run.  Only trees too large for a small-graph run
// (the one-request graph's assembly is a few KB and rides there).  The leaves are then read at the root's position, not at
// the inner nodes': no node run in between (nor the root itself) may have been given a leaf's memory.
struct concat_tree {
    std::vector<const ggml_tensor *> leaves;
    std::vector<int64_t>             extents;
    int                              dim;
};

void find_concat_trees(const ggml_cgraph * g, const reader_map & readers, std::unordered_map<const ggml_tensor *, concat_tree> & by_root,
                       std::unordered_map<const ggml_tensor *, const ggml_tensor *> & absorbed) {
    constexpr int64_t SMALL_GRAPH_ELEMENTS = 16384; // below this a CONCAT is a member of a small-graph run
    constexpr size_t  MAX_LEAVES = 8;
    std::unordered_map<const ggml_tensor *, int> pos;
    for (int i = 0; i < g->n_nodes; ++i) pos[g->nodes[i]] = i;
    const auto inner_ok = [&](const ggml_tensor * t) {
        return pos.count(t) && t->type == GGML_TYPE_F32 && !t->view_src && (t->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 &&
               private_to_group(readers, t) && absorbed.find(t) == absorbed.end();
    };
    for (int i = g->n_nodes - 1; i >= 0; --i) { // parents before children: a root is never a node some other root absorbs
        const ggml_tensor * root = g->nodes[i];
        if (root->op != GGML_OP_CONCAT || root->type != GGML_TYPE_F32 || (root->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) continue;
        if (absorbed.find(root) != absorbed.end() || ggml_nelements(root) <= SMALL_GRAPH_ELEMENTS) continue;
        const int dim = ((const int32_t *) root->op_params)[0];
        concat_tree tree;
        tree.dim = dim;
        std::vector<const ggml_tensor *> inner;
        bool ok = true;
        // leaves in order: depth first, first operand first
        std::vector<const ggml_tensor *> stack = { root->src[1], root->src[0] };
        while (!stack.empty() && ok) {
            const ggml_tensor * t = stack.back();
            stack.pop_back();
            if (!t) { ok = false; break; }
            if (t->op == GGML_OP_CONCAT && ((const int32_t *) t->op_params)[0] == dim && inner_ok(t)) {
                inner.push_back(t);
                stack.push_back(t->src[1]);
                stack.push_back(t->src[0]);
            } else if (t->op == GGML_OP_REPEAT && inner_ok(t) && t->src[0] && t->src[0]->type == GGML_TYPE_F32) {
                inner.push_back(t);
                tree.leaves.push_back(t->src[0]);
                tree.extents.push_back(t->ne[dim]);
            } else {
                tree.leaves.push_back(t);
                tree.extents.push_back(t->ne[dim]);
            }
            ok = tree.leaves.size() <= MAX_LEAVES;
        }
        if (!ok || inner.empty()) continue;
        std::vector<vx_tensor> ts(tree.leaves.size());
        std::vector<const vx_tensor *> tp(tree.leaves.size());
        for (size_t k = 0; k < ts.size(); ++k) { ts[k] = to_vx(tree.leaves[k]); tp[k] = &ts[k]; }
        const vx_tensor d = to_vx(root);
        if (!vx_supports_concat_many(tp.data(), tree.extents.data(), (int) tp.size(), dim, &d)) continue;
        int first = i;
        for (const ggml_tensor * t : inner) first = std::min(first, pos[t]);
        for (const ggml_tensor * leaf : tree.leaves) ok = ok && apart(root, leaf);
        for (int k = first + 1; k < i && ok; ++k) {
            const ggml_tensor * n = g->nodes[k];
            if (ggml_op_is_empty(n->op) || ggml_is_empty(n) || (n->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) continue;
            if (std::find(inner.begin(), inner.end(), n) != inner.end()) continue;
            for (const ggml_tensor * leaf : tree.leaves)
                if (n != leaf && n != leaf->view_src) ok = ok && apart(n, leaf);
        }
        if (!ok) continue;
        for (const ggml_tensor * t : inner) absorbed[t] = root;
        by_root[root] = std::move(tree);
    }
}

// FLASH_ATTN_EXT over absorbed CONCATs directly followed by the cache-write group on its result (the decode
// step of attention_forward): one call, the write rides on the kernel that merges the key-range partials.
// Returns the index of the group's last node, or -1.
int compute_kv2_attention_store(backend_ctx * ctx, const ggml_cgraph * g, int i, const kv2_group & grp, const reader_map & readers, vx_status * rc) {
    const ggml_tensor * f = g->nodes[i];
    const int j = next_real(g, i);
    if (j >= g->n_nodes || g->nodes[j]->op != GGML_OP_CPY || !private_to_group(readers, f)) return -1;
    ggml_tensor * n[9];
    const int last = match_kv_store_group(g, j, readers, n);
    if (last < 0 || n[8]->src[0] != f) return -1;
    const ggml_tensor * dst = n[8];
    const ggml_tensor * reads[] = { f->src[0], f->src[3], f->src[4], grp.kcat->src[0], grp.kcur, grp.vcat->src[0], grp.vcur };
    for (const ggml_tensor * r : reads)
        if (r && (!apart(dst, r) || !apart_rows(n[0], r) || !apart_rows(n[3], r))) return -1;
    float scale, max_bias, softcap, sc, bias;
    memcpy(&scale, (const float *) f->op_params + 0, sizeof(float));
    memcpy(&max_bias, (const float *) f->op_params + 1, sizeof(float));
    memcpy(&softcap, (const float *) f->op_params + 2, sizeof(float));
    memcpy(&sc, (const float *) n[7]->op_params + 0, sizeof(float));
    memcpy(&bias, (const float *) n[7]->op_params + 1, sizeof(float));
    const vx_tensor q = to_vx(f->src[0]), kp = to_vx(grp.kcat->src[0]), kc = to_vx(grp.kcur), vp = to_vx(grp.vcat->src[0]),
                    vc = to_vx(grp.vcur), ksrc = to_vx(n[0]->src[0]), ks = to_vx(n[0]), vsrc = to_vx(n[3]->src[0]), vs = to_vx(n[3]),
                    d = to_vx(dst);
    vx_tensor m;
    if (f->src[3]) m = to_vx(f->src[3]);
    if (!vx_supports_flash_attn_ext_kv2_store(&q, &kp, &kc, &vp, &vc, f->src[3] ? &m : nullptr, &ksrc, &ks, &vsrc, &vs, &d)) return -1;
    *rc = vx_flash_attn_ext_kv2_store(&q, &kp, &kc, &vp, &vc, f->src[3] ? &m : nullptr, f->src[4] ? (const float *) f->src[4]->data : nullptr,
                                      &ksrc, &ks, &vsrc, &vs, &d, scale, max_bias, softcap, sc, bias, ctx->stream);
    return last;
}

// FLASH_ATTN_EXT at prefill size directly followed by the cache-write group on its result: one call that launches the
// write and the ordering scalar first and lets the attention add the scalar as it stores.  The write moves in front of
// the attention, so its slots must lie apart from everything the attention reads.  Returns the index of the group's
// last node, or -1.
int compute_attention_store(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers, vx_status * rc) {
    const ggml_tensor * f = g->nodes[i];
    const int j = next_real(g, i);
    if (j >= g->n_nodes || g->nodes[j]->op != GGML_OP_CPY || !private_to_group(readers, f)) return -1;
    if (f->src[4] && (f->src[4]->type != GGML_TYPE_F32 || f->src[4]->ne[0] != f->src[0]->ne[2])) return -1;
    ggml_tensor * n[9];
    const int last = match_kv_store_group(g, j, readers, n);
    if (last < 0 || n[8]->src[0] != f) return -1;
    const ggml_tensor * dst = n[8];
    for (int k = 0; k < 5; ++k) {
        const ggml_tensor * r = f->src[k];
        if (r && (!apart(dst, r) || !apart(n[0], r) || !apart(n[3], r))) return -1;
    }
    float scale, max_bias, softcap, sc, bias;
    memcpy(&scale, (const float *) f->op_params + 0, sizeof(float));
    memcpy(&max_bias, (const float *) f->op_params + 1, sizeof(float));
    memcpy(&softcap, (const float *) f->op_params + 2, sizeof(float));
    memcpy(&sc, (const float *) n[7]->op_params + 0, sizeof(float));
    memcpy(&bias, (const float *) n[7]->op_params + 1, sizeof(float));
    const vx_tensor q = to_vx(f->src[0]), k = to_vx(f->src[1]), v = to_vx(f->src[2]), ksrc = to_vx(n[0]->src[0]), ks = to_vx(n[0]),
                    vsrc = to_vx(n[3]->src[0]), vs = to_vx(n[3]), d = to_vx(dst);
    vx_tensor m;
    if (f->src[3]) m = to_vx(f->src[3]);
    if (!vx_supports_flash_attn_ext_store(&q, &k, &v, f->src[3] ? &m : nullptr, &ksrc, &ks, &vsrc, &vs, &d, softcap)) return -1;
    {   // the o projection and its residual update behind the ADD1 (attention_forward's last two lines, layer_forward's update):
        //   RESHAPE(attn) MUL_MAT(o_proj, .) [SCALE] ADD(residual, .)
        // with the reshape the ADD1's only reader and the product its only one, the attention's result goes to the product
        // as its f16 activation tiles and is never stored
        int im = last + 1;
        const ggml_tensor * view = nullptr;
        while (im < g->n_nodes && (ggml_op_is_empty(g->nodes[im]->op) || ggml_is_empty(g->nodes[im]))) {
            if (g->nodes[im]->view_src == dst && g->nodes[im]->src[0] == dst && !view) view = g->nodes[im];
            ++im;
        }
        const auto rd = readers.find(dst);
        const ggml_tensor * mm = im < g->n_nodes ? g->nodes[im] : nullptr;
        if (view && mm && mm->op == GGML_OP_MUL_MAT && mm->src[1] == view && (dst->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 &&
            (view->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 && rd != readers.end() && rd->second == 2 && private_to_group(readers, view) &&
            view->view_offs == 0 && ggml_is_contiguous(view) && private_to_group(readers, mm) && im + 1 < g->n_nodes) {
            const ggml_tensor * val = mm;
            float rs = 1.0f;
            int ia = im + 1;
            bool ok = true;
            if (g->nodes[ia]->op == GGML_OP_SCALE) {
                const ggml_tensor * scn = g->nodes[ia];
                float sb;
                memcpy(&rs, (const float *) scn->op_params + 0, sizeof(float));
                memcpy(&sb, (const float *) scn->op_params + 1, sizeof(float));
                ok = scn->src[0] == mm && sb == 0.0f && private_to_group(readers, scn) && ia + 1 < g->n_nodes;
                val = scn;
                ++ia;
            }
            const ggml_tensor * add = ok ? g->nodes[ia] : nullptr;
            if (add && add->op == GGML_OP_ADD && (add->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 && (add->src[0] == val) != (add->src[1] == val)) {
                const ggml_tensor * residual = add->src[0] == val ? add->src[1] : add->src[0];
                // (the update is the call's last kernel: what the cache write and the attention read is done with by then, and the
                // update may well have been given the memory of q; the weights and the residual are what its kernel reads)
                ok = residual != mm && residual != dst && residual != view && apart(add, mm->src[0]) && apart_or_same(add, residual) &&
                     apart(n[0], residual) && apart(n[3], residual);
                const vx_tensor av = to_vx(view), wo = to_vx(mm->src[0]), r = to_vx(residual), od = to_vx(add);
                if (ok && vx_supports_flash_attn_ext_store_proj(&q, &k, &v, f->src[3] ? &m : nullptr, &ksrc, &ks, &vsrc, &vs, &av, &wo, &r, &od, softcap,
                                                                mul_mat_act_mode())) {
                    *rc = vx_flash_attn_ext_store_proj(&q, &k, &v, f->src[3] ? &m : nullptr, f->src[4] ? (const float *) f->src[4]->data : nullptr,
                                                       &ksrc, &ks, &vsrc, &vs, &av, &wo, &r, &od, scale, max_bias, softcap, sc, bias, rs,
                                                       mul_mat_act_mode(), ctx->stream);
                    return ia;
                }
            }
        }
    }
    *rc = vx_flash_attn_ext_store(&q, &k, &v, f->src[3] ? &m : nullptr, f->src[4] ? (const float *) f->src[4]->data : nullptr,
                                  &ksrc, &ks, &vsrc, &vs, &d, scale, max_bias, softcap, sc, bias, ctx->stream);
    return last;
}

vx_status compute_kv2_attention(backend_ctx * ctx, const ggml_tensor * f, const kv2_group & grp) {
    float scale, max_bias, softcap;
    memcpy(&scale, (const float *) f->op_params + 0, sizeof(float));
    memcpy(&max_bias, (const float *) f->op_params + 1, sizeof(float));
    memcpy(&softcap, (const float *) f->op_params + 2, sizeof(float));
    const vx_tensor q = to_vx(f->src[0]), kp = to_vx(grp.kcat->src[0]), kc = to_vx(grp.kcur), vp = to_vx(grp.vcat->src[0]),
                    vc = to_vx(grp.vcur), d = to_vx(f);
    vx_tensor m;
    if (f->src[3]) m = to_vx(f->src[3]);
    return vx_flash_attn_ext_kv2(&q, &kp, &kc, &vp, &vc, f->src[3] ? &m : nullptr, f->src[4] ? (const float *) f->src[4]->data : nullptr,
                                 &d, scale, max_bias, softcap, ctx->stream);
}

// attention_forward's three projections and the rotation of Q and K (src/minicpm.cpp:669-680) at decode size:
//   MUL_MAT(wq, x) RESHAPE ROPE  [views]  MUL_MAT(wk, x) RESHAPE ROPE  [views, absorbed CONCAT]  MUL_MAT(wv, x)
// -> one launch at the first node; the other four are marked done.  K's and V's outputs are written earlier
// than their nodes' turn, which is safe because every node in between that does work belongs to the group.
typedef std::unordered_map<const ggml_tensor *, const ggml_tensor *> absorbed_map;

const ggml_tensor * rope_of_projection(const ggml_cgraph * g, int & idx, const ggml_tensor * mm, const reader_map & readers,
                                       const absorbed_map & absorbed) {
    // the next node that does work must be a ROPE over (a reshape of) mm, and nothing else may read mm
    int k = idx + 1;
    while (k < g->n_nodes && (ggml_op_is_empty(g->nodes[k]->op) || ggml_is_empty(g->nodes[k]) || absorbed.count(g->nodes[k]))) ++k;
    if (k >= g->n_nodes) return nullptr;
    const ggml_tensor * r = g->nodes[k];
    if (r->op != GGML_OP_ROPE || (r->flags & GGML_TENSOR_FLAG_COMPUTE) == 0 || (mm->flags & GGML_TENSOR_FLAG_OUTPUT) != 0) return nullptr;
    const ggml_tensor * in = r->src[0];
    const auto rd = [&](const ggml_tensor * t) { const auto it = readers.find(t); return it == readers.end() ? 0 : it->second; };
    if (in == mm) {
        if (rd(mm) != 1) return nullptr;
    } else {
        if (in->op != GGML_OP_RESHAPE || in->src[0] != mm || in->view_src != mm || (in->flags & GGML_TENSOR_FLAG_OUTPUT) != 0) return nullptr;
        if (rd(mm) != 2 || rd(in) != 1) return nullptr; // mm: the reshape's operand and view source; the reshape: the rope
    }
    idx = k;
    return r;
}

// norm / scale: the RMS_NORM and norm-weight MUL nodes right in front of the group when the normalised tensor has no
// reader outside it (then i is the RMS_NORM's index and the group starts two nodes later), else null.
bool compute_qkv_group(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers, const absorbed_map & absorbed,
                       std::unordered_set<const ggml_tensor *> & done, vx_status * rc, const ggml_tensor * norm = nullptr,
                       const ggml_tensor * scale = nullptr) {
    if (norm) i += 2;
    if (i >= g->n_nodes || g->nodes[i]->op != GGML_OP_MUL_MAT) return false;
    const ggml_tensor * mq = g->nodes[i];
    int idx = i;
    const ggml_tensor * rq = rope_of_projection(g, idx, mq, readers, absorbed);
    if (!rq) return false;
    auto next_work = [&](int k) {
        ++k;
        while (k < g->n_nodes && (ggml_op_is_empty(g->nodes[k]->op) || ggml_is_empty(g->nodes[k]) || absorbed.count(g->nodes[k]))) ++k;
        return k;
    };
    idx = next_work(idx);
    if (idx >= g->n_nodes) return false;
    const ggml_tensor * mk = g->nodes[idx];
    if (mk->op != GGML_OP_MUL_MAT || mk->src[1] != mq->src[1] || (mk->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) return false;
    const ggml_tensor * rk = rope_of_projection(g, idx, mk, readers, absorbed);
    if (!rk) return false;
    idx = next_work(idx);
    if (idx >= g->n_nodes) return false;
    const ggml_tensor * mv = g->nodes[idx];
    if (mv->op != GGML_OP_MUL_MAT || mv->src[1] != mq->src[1] || (mv->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) return false;
    // one rotation for both: same positions, factors and parameters
    if (rq->src[1] != rk->src[1] || rq->src[2] != rk->src[2] || memcmp(rq->op_params, rk->op_params, 11 * sizeof(int32_t)) != 0) return false;
    if (!rq->src[1] || rq->src[1]->type != GGML_TYPE_I32 || rq->src[1]->ne[0] != rq->ne[2]) return false;
    if (rq->src[2] && (rq->src[2]->type != GGML_TYPE_F32 || rq->src[2]->ne[0] < rq->ne[0] / 2)) return false;
    const int32_t * ip = (const int32_t *) rq->op_params;
    const int n_dims = ip[1], mode = ip[2], n_ctx_orig = ip[4];
    float fp[6];
    memcpy(fp, ip + 5, sizeof(fp));
    if (norm && mq->src[1] != scale) return false;
    const ggml_tensor * x = norm ? norm->src[0] : mq->src[1];
    const ggml_tensor * outs[3] = { rq, rk, mv };
    for (int a = 0; a < 3; ++a) {
        if (!apart(outs[a], x)) return false;
        for (int b = a + 1; b < 3; ++b) if (!apart(outs[a], outs[b])) return false;
    }
    const vx_tensor wq = to_vx(mq->src[0]), wk = to_vx(mk->src[0]), wv = to_vx(mv->src[0]), xx = to_vx(x), dq = to_vx(rq), dk = to_vx(rk),
                    dv = to_vx(mv);
    const int32_t * posd = (const int32_t *) rq->src[1]->data;
    const float *   ffd  = rq->src[2] ? (const float *) rq->src[2]->data : nullptr;
    if (norm) {
        const vx_tensor nw = to_vx(scale->src[1]);
        float eps;
        memcpy(&eps, norm->op_params, sizeof(float));
        // (decode sizes: one launch of the streaming kernel; prefill sizes: the norm in the pre-tiled kernel's activation pass,
        // the three matrices as one product, the rotations behind it)
        if ((!vx_supports_norm_qkv_proj_rope(&xx, &nw, &wq, &wk, &wv, &dq, &dk, &dv, n_dims, mode) &&
             !vx_supports_norm_qkv_proj_rope_tiled(&xx, &nw, &wq, &wk, &wv, &dq, &dk, &dv, n_dims, mode, mul_mat_act_mode())) ||
            (uintptr_t) xx.data % 16 || (uintptr_t) nw.data % 16) return false;
        *rc = vx_norm_qkv_proj_rope(&xx, &nw, eps, &wq, &wk, &wv, posd, ffd, &dq, &dk, &dv, n_dims, mode, n_ctx_orig, fp[0], fp[1], fp[2], fp[3],
                                    fp[4], fp[5], mul_mat_act_mode(), ctx->stream);
        done.insert(scale); done.insert(mq);
    } else {
        if (!vx_supports_qkv_proj_rope(&wq, &wk, &wv, &xx, &dq, &dk, &dv, n_dims, mode)) return false;
        *rc = vx_qkv_proj_rope(&wq, &wk, &wv, &xx, posd, ffd, &dq, &dk, &dv, n_dims, mode, n_ctx_orig, fp[0], fp[1], fp[2], fp[3], fp[4], fp[5],
                               mul_mat_act_mode(), ctx->stream);
    }
    done.insert(rq); done.insert(mk); done.insert(rk); done.insert(mv);
    return true;
}

// The same for K and V alone, where q's product has left the streaming kernel (a prompt of 205 to 1024 tokens):
//   MUL_MAT(wk, x) RESHAPE ROPE  [views, absorbed CONCAT]  MUL_MAT(wv, x)      -> one launch at the first node
bool compute_kv_group(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers, const absorbed_map & absorbed,
                      std::unordered_set<const ggml_tensor *> & done, vx_status * rc) {
    const ggml_tensor * mk = g->nodes[i];
    if (mk->op != GGML_OP_MUL_MAT) return false;
    int idx = i;
    const ggml_tensor * rk = rope_of_projection(g, idx, mk, readers, absorbed);
    if (!rk) return false;
    ++idx;
    while (idx < g->n_nodes && (ggml_op_is_empty(g->nodes[idx]->op) || ggml_is_empty(g->nodes[idx]) || absorbed.count(g->nodes[idx]))) ++idx;
    if (idx >= g->n_nodes) return false;
    const ggml_tensor * mv = g->nodes[idx];
    if (mv->op != GGML_OP_MUL_MAT || mv->src[1] != mk->src[1] || (mv->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) return false;
    if (!rk->src[1] || rk->src[1]->type != GGML_TYPE_I32 || rk->src[1]->ne[0] != rk->ne[2]) return false;
    if (rk->src[2] && (rk->src[2]->type != GGML_TYPE_F32 || rk->src[2]->ne[0] < rk->ne[0] / 2)) return false;
    const int32_t * ip = (const int32_t *) rk->op_params;
    const int n_dims = ip[1], mode = ip[2], n_ctx_orig = ip[4];
    float fp[6];
    memcpy(fp, ip + 5, sizeof(fp));
    const ggml_tensor * x = mk->src[1];
    if (!apart(rk, x) || !apart(mv, x) || !apart(rk, mv)) return false;
    const vx_tensor wk = to_vx(mk->src[0]), wv = to_vx(mv->src[0]), xx = to_vx(x), dk = to_vx(rk), dv = to_vx(mv);
    if (!vx_supports_kv_proj_rope(&wk, &wv, &xx, &dk, &dv, n_dims, mode)) return false;
    *rc = vx_kv_proj_rope(&wk, &wv, &xx, (const int32_t *) rk->src[1]->data, rk->src[2] ? (const float *) rk->src[2]->data : nullptr, &dk, &dv,
                          n_dims, mode, n_ctx_orig, fp[0], fp[1], fp[2], fp[3], fp[4], fp[5], mul_mat_act_mode(), ctx->stream);
    done.insert(rk); done.insert(mv);
    return true;
}

// The reference's row-fused weights (MiniCPMModel::load_from_store makes them for the LocDiT decoder on a GPU backend,
// src/minicpm.cpp:427-492): one MUL_MAT over qkv_proj, strided views of it as q, k, v, ROPE on the q and k views
// (src/minicpm.cpp:644-680)
//   [RMS_NORM MUL] MUL_MAT(qkv_proj, x) VIEW ROPE [views] VIEW ROPE        -> one launch: the multi-matrix kernel walks
// three row ranges of the one matrix, writes the rotated q and k to the ROPE nodes' outputs and v where it lies in the
// product.  A row range of a matrix as a descriptor of its own:
vx_tensor row_range(const ggml_tensor * w, int64_t row0, int64_t rows) {
    vx_tensor t = to_vx(w);
    t.data  = (char *) w->data + (size_t) row0 * w->nb[1];
    t.ne[1] = rows;
    return t;
}

// view of the product mm covering rows [row0, row0 + rows) of every token, as [head_dim, heads, tokens, batch]
bool is_row_view(const ggml_tensor * v, const ggml_tensor * mm, int64_t * row0, int64_t * rows) {
    if (!v || v->op != GGML_OP_VIEW || v->view_src != mm || v->type != GGML_TYPE_F32 || mm->type != GGML_TYPE_F32) return false;
    const ptrdiff_t off = (const char *) v->data - (const char *) mm->data;
    if (off < 0 || off % 4 || (size_t) off >= mm->nb[1]) return false;
    *row0 = off / 4;
    *rows = v->ne[0] * v->ne[1];
    if (*row0 + *rows > mm->ne[0]) return false;
    if (v->nb[0] != 4 || v->nb[1] != (size_t) v->ne[0] * 4 || v->nb[2] != mm->nb[1]) return false;
    if (v->ne[3] > 1 && v->nb[3] != (size_t) v->ne[2] * mm->nb[1]) return false;
    return v->ne[2] * v->ne[3] == mm->ne[1] * mm->ne[2] * mm->ne[3] && mm->ne[2] == 1;
}

bool compute_fused_qkv_group(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers, const absorbed_map & absorbed,
                             std::unordered_set<const ggml_tensor *> & done, vx_status * rc, const ggml_tensor * norm = nullptr,
                             const ggml_tensor * scale = nullptr) {
    if (norm) i += 2;
    if (i >= g->n_nodes || g->nodes[i]->op != GGML_OP_MUL_MAT) return false;
    const ggml_tensor * mm = g->nodes[i];
    if ((mm->flags & GGML_TENSOR_FLAG_OUTPUT) != 0 || (norm && mm->src[1] != scale)) return false;
    const auto rd = [&](const ggml_tensor * t) { const auto it = readers.find(t); return it == readers.end() ? 0 : it->second; };
    // the next two nodes that do work: ROPE over row views of mm
    const ggml_tensor * rope[2] = { nullptr, nullptr };
    int k = i;
    for (int n = 0; n < 2; ++n) {
        ++k;
        while (k < g->n_nodes && (ggml_op_is_empty(g->nodes[k]->op) || ggml_is_empty(g->nodes[k]) || absorbed.count(g->nodes[k]))) ++k;
        if (k >= g->n_nodes || g->nodes[k]->op != GGML_OP_ROPE || (g->nodes[k]->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) return false;
        rope[n] = g->nodes[k];
    }
    const ggml_tensor * rq = rope[0], * rk = rope[1];
    int64_t q0, qn, k0, kn;
    if (!is_row_view(rq->src[0], mm, &q0, &qn) || !is_row_view(rk->src[0], mm, &k0, &kn)) return false;
    if (rd(rq->src[0]) != 1 || rd(rk->src[0]) != 1) return false;          // the un-rotated q and k rows are never stored
    const int64_t M = mm->ne[0], vn = M - qn - kn;
    if (q0 != 0 || k0 != qn || vn <= 0) return false;
    // everything else that looks at the product must look at the v rows only (views of views share view_src)
    for (int n = 0; n < g->n_nodes; ++n) {
        const ggml_tensor * t = g->nodes[n];
        if (t == rq->src[0] || t == rk->src[0]) continue;
        bool reads = t->view_src == mm;
        for (int s2 = 0; s2 < GGML_MAX_SRC && !reads; ++s2) reads = t->src[s2] == mm && !ggml_op_is_empty(t->op);
        if (!reads) continue;
        if (t->view_src != mm || !ggml_op_is_empty(t->op)) return false;
        const ptrdiff_t off = (const char *) t->data - (const char *) mm->data;
        if (off < 0 || (int64_t) ((size_t) off % mm->nb[1]) < (qn + kn) * 4) return false;
    }
    if (rq->src[1] != rk->src[1] || rq->src[2] != rk->src[2] || memcmp(rq->op_params, rk->op_params, 11 * sizeof(int32_t)) != 0) return false;
    if (!rq->src[1] || rq->src[1]->type != GGML_TYPE_I32 || rq->src[1]->ne[0] != rq->ne[2]) return false;
    if (rq->src[2] && (rq->src[2]->type != GGML_TYPE_F32 || rq->src[2]->ne[0] < rq->ne[0] / 2)) return false;
    const int32_t * ip = (const int32_t *) rq->op_params;
    const int n_dims = ip[1], mode = ip[2], n_ctx_orig = ip[4];
    float fp[6];
    memcpy(fp, ip + 5, sizeof(fp));
    const ggml_tensor * x = norm ? norm->src[0] : mm->src[1];
    if (!apart(rq, x) || !apart(rk, x) || !apart(mm, x) || !apart(rq, rk) || !apart(rq, mm) || !apart(rk, mm)) return false;
    const ggml_tensor * W = mm->src[0];
    {   // the row ranges must be summed as the one product over all rows would be
        const int64_t tokens = x->ne[1] * x->ne[2] * x->ne[3];
        const int order = vx_mul_mat_sum_order(W->ne[0], tokens, M);
        if (order <= 0 || vx_mul_mat_sum_order(W->ne[0], tokens, qn) != order || vx_mul_mat_sum_order(W->ne[0], tokens, kn) != order ||
            vx_mul_mat_sum_order(W->ne[0], tokens, vn) != order) return false;
    }
    const vx_tensor wq = row_range(W, 0, qn), wk = row_range(W, qn, kn), wv = row_range(W, qn + kn, vn), xx = to_vx(x), dq = to_vx(rq), dk = to_vx(rk);
    vx_tensor dv = to_vx(mm);                       // the v rows of the product, where they lie
    dv.data  = (char *) mm->data + (size_t) (qn + kn) * 4;
    dv.ne[0] = vn;
    const int32_t * posd = (const int32_t *) rq->src[1]->data;
    const float *   ffd  = rq->src[2] ? (const float *) rq->src[2]->data : nullptr;
    if (norm) {
        const vx_tensor nw = to_vx(scale->src[1]);
        float eps;
        memcpy(&eps, norm->op_params, sizeof(float));
        if (!vx_supports_norm_qkv_proj_rope(&xx, &nw, &wq, &wk, &wv, &dq, &dk, &dv, n_dims, mode) || (uintptr_t) xx.data % 16 || (uintptr_t) nw.data % 16) return false;
        *rc = vx_norm_qkv_proj_rope(&xx, &nw, eps, &wq, &wk, &wv, posd, ffd, &dq, &dk, &dv, n_dims, mode, n_ctx_orig, fp[0], fp[1], fp[2], fp[3],
                                    fp[4], fp[5], mul_mat_act_mode(), ctx->stream);
        done.insert(scale); done.insert(mm);
    } else {
        if (!vx_supports_qkv_proj_rope(&wq, &wk, &wv, &xx, &dq, &dk, &dv, n_dims, mode)) return false;
        *rc = vx_qkv_proj_rope(&wq, &wk, &wv, &xx, posd, ffd, &dq, &dk, &dv, n_dims, mode, n_ctx_orig, fp[0], fp[1], fp[2], fp[3], fp[4], fp[5],
                               mul_mat_act_mode(), ctx->stream);
    }
    done.insert(rq); done.insert(rk);
    return true;
}

//   [RMS_NORM MUL] MUL_MAT(gate_up_proj, x) VIEW VIEW GLU(SWIGLU split)   (src/minicpm.cpp:724-745)  -> one launch:
// the gate rows and the up rows of the one matrix share the MFMA columns of the SwiGLU kernel.
bool compute_fused_gate_up_group(backend_ctx * ctx, const ggml_cgraph * g, int i, const reader_map & readers,
                                 std::unordered_set<const ggml_tensor *> & done, vx_status * rc, const ggml_tensor * norm = nullptr,
                                 const ggml_tensor * scale = nullptr) {
    if (norm) i += 2;
    if (i >= g->n_nodes || g->nodes[i]->op != GGML_OP_MUL_MAT) return false;
    const ggml_tensor * mm = g->nodes[i];
    if ((mm->flags & GGML_TENSOR_FLAG_OUTPUT) != 0 || (norm && mm->src[1] != scale) || mm->ne[2] != 1 || mm->ne[3] != 1) return false;
    const auto rd = [&](const ggml_tensor * t) { const auto it = readers.find(t); return it == readers.end() ? 0 : it->second; };
    const int kg = next_real(g, i);
    if (kg >= g->n_nodes) return false;
    const ggml_tensor * glu = g->nodes[kg];
    if (glu->op != GGML_OP_GLU || (glu->flags & GGML_TENSOR_FLAG_COMPUTE) == 0 || ggml_get_glu_op(glu) != GGML_GLU_OP_SWIGLU ||
        ((const int32_t *) glu->op_params)[1] != 0 || !glu->src[1]) return false;
    const ggml_tensor * vg = glu->src[0], * vu = glu->src[1];
    const int64_t ffn = mm->ne[0] / 2;
    for (const ggml_tensor * v : { vg, vu }) {
        if (v->op != GGML_OP_VIEW || v->view_src != mm || rd(v) != 1 || v->ne[0] != ffn || v->ne[1] != mm->ne[1] || v->ne[2] != 1 || v->ne[3] != 1 ||
            v->nb[0] != 4 || v->nb[1] != mm->nb[1]) return false;
    }
    if (mm->ne[0] != 2 * ffn || rd(mm) != 4 || vg->data != mm->data || (const char *) vu->data != (const char *) mm->data + (size_t) ffn * 4) return false;
    const ggml_tensor * x = norm ? norm->src[0] : mm->src[1];
    if (!apart(glu, x)) return false;
    const ggml_tensor * W = mm->src[0];
    {   // the two halves must be summed as the one product over all rows would be
        const int64_t tokens = x->ne[1] * x->ne[2] * x->ne[3];
        const int order = vx_mul_mat_sum_order(W->ne[0], tokens, 2 * ffn);
        if (order <= 0 || vx_mul_mat_sum_order(W->ne[0], tokens, ffn) != order) return false;
    }
    const vx_tensor gw = row_range(W, 0, ffn), uw = row_range(W, ffn, ffn), xx = to_vx(x), d = to_vx(glu);
    if (norm) {
        const vx_tensor nw = to_vx(scale->src[1]);
        float eps;
        memcpy(&eps, norm->op_params, sizeof(float));
        if (!vx_supports_norm_mul_mat_swiglu(&xx, &nw, &gw, &uw, &d) || (uintptr_t) xx.data % 16 || (uintptr_t) nw.data % 16) return false;
        *rc = vx_norm_mul_mat_swiglu(&xx, &nw, eps, &gw, &uw, &d, mul_mat_act_mode(), ctx->stream);
        done.insert(scale); done.insert(mm);
    } else {
        if (!vx_supports_mul_mat_swiglu(&gw, &uw, &xx, &d) && !vx_supports_mul_mat_swiglu_tiled(&gw, &uw, &xx, &d, mul_mat_act_mode())) return false;
        *rc = vx_mul_mat_swiglu(&gw, &uw, &xx, &d, mul_mat_act_mode(), ctx->stream);
    }
    done.insert(glu);
    return true;
}

int g_last_launches = 0; // operator launches of the most recent graph_compute (diagnostic)
int g_replays = 0;       // graph_compute calls of this process that were served by replaying recorded launches
int g_fusion_on = -1;    // run groups of nodes as one launch (GGML_GFX950_NO_FUSION switches it off, ggml_backend_gfx950_set_fusion either way)
bool fusion_on() {
    if (g_fusion_on < 0) g_fusion_on = getenv("GGML_GFX950_NO_FUSION") == nullptr;
    return g_fusion_on != 0;
}
int g_replay_on = -1;    // recognise recurring graphs and replay them (GGML_GFX950_GRAPH_REPLAY, ggml_backend_gfx950_set_graph_replay)

// ---- recognising a graph ---------------------------------------------------------------------------------------------
inline uint64_t mix64(uint64_t h, uint64_t v) {
    h ^= v + 0x9E3779B97F4A7C15ull + (h << 6) + (h >> 2);
    return h * 0xff51afd7ed558ccdull;
}
// cheap: node count, and per node the operator, the output address and the two outer extents (what changes from one
// decode step to the next: the key count) -- a few hundred nanoseconds per thousand nodes
// `shape`, taken in the same pass: node count, operators and types only -- what the steps of a decode loop share
uint64_t graph_cheap_signature(const ggml_cgraph * g, uint64_t * shape) {
    // (the activation mode of the Q8_0 products is part of what a recording holds: a graph recorded under one mode is
    // another graph under the other)
    uint64_t h = (uint64_t) g->n_nodes ^ (((uint64_t) mul_mat_act_mode() << 40) ^ ((uint64_t) fusion_on() << 42));
    uint64_t s = h;
    for (int i = 0; i < g->n_nodes; ++i) {
        const ggml_tensor * n = g->nodes[i];
        h = mix64(h, (uint64_t) (uintptr_t) n->data ^ ((uint64_t) n->op << 56) ^ ((uint64_t) n->ne[1] << 20) ^ ((uint64_t) n->ne[2] << 40));
        s = (s ^ (((uint64_t) n->op << 8) ^ (uint64_t) n->type)) * 0x9E3779B97F4A7C15ull;
        s ^= s >> 31;
    }
    *shape = s | 1;
    return h | 1;
}
// full: everything a launch is derived from.  A thousand nodes are some 25 000 words, hashed on every graph_compute of a
// caller that waits for each step: four independent multiply-xor chains take the words in turn (a single chain is bound
// by the multiplier's latency: 40 us for a decode step's graph, a twentieth of the step itself).
struct fingerprint_state {
    uint64_t h[4] = { 0x243F6A8885A308D3ull, 0x13198A2E03707344ull, 0xA4093822299F31D0ull, 0x082EFA98EC4E6C89ull };
    unsigned n = 0;
    void add(uint64_t v) {
        uint64_t & x = h[n++ & 3];
        x = (x ^ v) * 0x9E3779B97F4A7C15ull;
        x ^= x >> 29;
    }
    uint64_t finish() const { return mix64(mix64(mix64(mix64((uint64_t) n, h[0]), h[1]), h[2]), h[3]); }
};
void fingerprint_tensor(fingerprint_state & f, const ggml_tensor * t) {
    f.add((uint64_t) (uintptr_t) t->data);
    f.add(((uint64_t) t->type << 32) ^ (uint64_t) t->op ^ ((uint64_t) t->flags << 48));
    for (int d = 0; d < GGML_MAX_DIMS; ++d) f.add((uint64_t) t->ne[d] ^ ((uint64_t) t->nb[d] << 24));
}
uint64_t graph_fingerprint(const ggml_cgraph * g) {
    fingerprint_state f;
    f.add((uint64_t) g->n_nodes ^ (((uint64_t) mul_mat_act_mode() << 40) ^ ((uint64_t) fusion_on() << 42)));
    for (int i = 0; i < g->n_nodes; ++i) {
        const ggml_tensor * n = g->nodes[i];
        fingerprint_tensor(f, n);
        const uint64_t * op = (const uint64_t *) n->op_params;
        for (size_t k = 0; k < GGML_MAX_OP_PARAMS / sizeof(uint64_t); ++k) f.add(op[k]);
        uint64_t present = 0; // which operand slots are in use, then the operands themselves
        for (int k = 0; k < GGML_MAX_SRC; ++k) if (n->src[k]) present |= (uint64_t) 1 << k;
        f.add(present);
        for (int k = 0; k < GGML_MAX_SRC; ++k) if (n->src[k]) fingerprint_tensor(f, n->src[k]);
        f.add((uint64_t) (uintptr_t) (n->view_src ? n->view_src->data : nullptr) ^ ((uint64_t) n->view_offs << 1));
    }
    return f.finish() | 1;
}

ggml_status graph_compute_eager(backend_ctx * ctx, ggml_cgraph * cgraph, int * launches_out);
// A node that fails while a recording is being made (a launch that would have to grow the workspace under the capture)
// is no error and is not logged: the recording is dropped and the graph is launched node by node.
bool g_trial_pass = false;
#define NODE_FAILED(...) do { if (!g_trial_pass) GGML_LOG_ERROR(__VA_ARGS__); } while (0)
int g_patch_on = -1;     // run a decode loop's steps as patched recordings (GGML_GFX950_GRAPH_PATCH, ggml_backend_gfx950_set_graph_patch)
int g_patched_replays = 0; // graph_compute calls served by a recording whose arguments were brought up to date first
int g_last_patched = 0;    // nodes whose arguments the most recent such call changed
bool patch_on() {
    // off unless asked for: the comparison pass takes the host a quarter of a millisecond for a 24-layer step before the
    // GPU gets anything to do, where node-by-node launches keep the GPU busy from the first launch on
    if (g_patch_on < 0) { const char * e = getenv("GGML_GFX950_GRAPH_PATCH"); g_patch_on = e && atoi(e) != 0; }
    return g_patch_on != 0;
}

// One more member of a family: true when the graph has been computed here (by a patched recording, or by a new one).
bool family_compute(backend_ctx * ctx, step_family & fam, ggml_cgraph * cgraph) {
    constexpr int MAX_FAILURES = 3;
    if (fam.failures >= MAX_FAILURES) return false;
    vx_graph & rec = fam.recorded[fam.turn];
    int launches = 0;
    if (rec) {
        if (vx_graph_patch_begin(rec) == VX_OK) {
            g_trial_pass = true;
            const ggml_status st = graph_compute_eager(ctx, cgraph, &launches); // compares, launches nothing
            g_trial_pass = false;
            int patched = 0;
            const bool same = vx_graph_patch_end(rec, &patched) == VX_OK;
            if (st == GGML_STATUS_SUCCESS && same && vx_graph_launch(rec, ctx->stream) == VX_OK) {
                fam.turn ^= 1;
                ++g_replays;
                ++g_patched_replays;
                g_last_patched = patched;
                g_last_launches = fam.launches;
                return true;
            }
        }
        vx_graph_destroy(rec); // other launches than recorded (another kernel for this key count, say): its arguments are a mixture now
        rec = nullptr;
        ++fam.failures;
        return false;
    }
    if (vx_graph_begin(ctx->stream) != VX_OK) { ++fam.failures; return false; }
    g_trial_pass = true;
    const ggml_status st = graph_compute_eager(ctx, cgraph, &launches);
    g_trial_pass = false;
    vx_graph made = nullptr;
    vx_graph_end(ctx->stream, &made);
    if (st == GGML_STATUS_SUCCESS && made && vx_graph_patchable(made) && vx_graph_launch(made, ctx->stream) == VX_OK) {
        rec = made;
        fam.launches = launches;
        fam.turn ^= 1;
        fam.failures = 0;
        ++g_replays;
        g_last_launches = launches;
        return true;
    }
    if (made) vx_graph_destroy(made);
    ++fam.failures; // e.g. a launch that must allocate
    return false;
}
long long g_host_ns[2] = { 0, 0 }; // the most recent node-by-node graph_compute: host time of the analysis, and of issuing the launches

// graph_optimize (ggml/src/ggml-backend-impl.h:118-119): ggml_backend_sched calls it once per split when it lays a graph
// out, before the tensors have addresses.  Nothing is reordered here, and nothing is remembered: a signature taken now
// could be matched to a graph object that was edited, or rebuilt at the same address, before it is computed.
void backend_graph_optimize(ggml_backend_t backend, ggml_cgraph * cgraph) {
    (void) backend;
    (void) cgraph;
}

ggml_status backend_graph_compute(ggml_backend_t backend, ggml_cgraph * cgraph) {
    backend_ctx * ctx = (backend_ctx *) backend->context;
    if (vx_init(ctx->device) != VX_OK) {
        GGML_LOG_ERROR("ggml-gfx950: %s\n", vx_last_error());
        return GGML_STATUS_FAILED;
    }
    // GGML_GFX950_GRAPH_REPLAY=0 switches the recognition off; test-backend-ops style one-node graphs never qualify
    if (g_replay_on < 0) { const char * e = getenv("GGML_GFX950_GRAPH_REPLAY"); g_replay_on = !(e && atoi(e) == 0); }
    int launches = 0;
    if (!g_replay_on || cgraph->n_nodes < 8) {
        const ggml_status st = graph_compute_eager(ctx, cgraph, &launches);
        g_last_launches = launches;
        return st;
    }
    uint64_t shape = 0;
    const uint64_t cheap = graph_cheap_signature(cgraph, &shape);
    seen_graph * entry = nullptr;
    for (seen_graph & g : ctx->seen) if (g.cheap == cheap) { entry = &g; break; }
    ++ctx->clock;
    if (!entry && patch_on()) { // never seen as it is: a further step of a loop that has been seen?
        step_family * fam = nullptr;
        for (step_family & f : ctx->families) if (f.shape == shape) { fam = &f; break; }
        if (!fam) {
            constexpr size_t MAX_FAMILIES = 4;
            if (ctx->families.size() < MAX_FAMILIES) { ctx->families.emplace_back(); fam = &ctx->families.back(); }
            else {
                fam = &ctx->families[0];
                for (step_family & f : ctx->families) if (f.last_use < fam->last_use) fam = &f;
                for (vx_graph & r : fam->recorded) if (r) vx_graph_destroy(r);
                *fam = step_family{};
            }
            fam->shape = shape;
        }
        fam->last_use = ctx->clock;
        if (++fam->sightings >= 2 && family_compute(ctx, *fam, cgraph)) return GGML_STATUS_SUCCESS;
    }
    if (!entry) { // first sight: remember the cheap signature only (a decode step's graph never comes back)
        constexpr size_t MAX_SEEN = 8;
        if (ctx->seen.size() < MAX_SEEN) { ctx->seen.emplace_back(); entry = &ctx->seen.back(); }
        else {
            entry = &ctx->seen[0];
            for (seen_graph & g : ctx->seen) if (g.last_use < entry->last_use) entry = &g;
            if (entry->recorded) vx_graph_destroy(entry->recorded);
            *entry = seen_graph{};
        }
        entry->cheap = cheap;
        entry->runs = 1;
        entry->last_use = ctx->clock;
        const ggml_status st = graph_compute_eager(ctx, cgraph, &launches);
        entry->launches = launches;
        g_last_launches = launches;
        return st;
    }
    entry->last_use = ctx->clock;
    const uint64_t fp = graph_fingerprint(cgraph);
    if (entry->fingerprint != fp) { // second sight (or a different graph with the same quick signature): start counting
        if (entry->recorded) vx_graph_destroy(entry->recorded);
        entry->recorded = nullptr;
        entry->fingerprint = fp;
        entry->runs = 1;
        entry->no_replay = false;
    }
    ++entry->runs;
    if (entry->recorded) {
        if (vx_graph_launch(entry->recorded, ctx->stream) == VX_OK) {
            ++g_replays;
            g_last_launches = entry->launches;
            return GGML_STATUS_SUCCESS;
        }
        vx_graph_destroy(entry->recorded);
        entry->recorded = nullptr;
        entry->no_replay = true;
    }
    if (entry->runs >= 3 && !entry->no_replay) { // the same graph for the third time: record its launches, then replay them
        if (vx_graph_begin(ctx->stream) == VX_OK) {
            g_trial_pass = true;
            const ggml_status st = graph_compute_eager(ctx, cgraph, &launches);
            g_trial_pass = false;
            vx_graph rec = nullptr;
            vx_graph_end(ctx->stream, &rec);
            if (st == GGML_STATUS_SUCCESS && rec && vx_graph_launch(rec, ctx->stream) == VX_OK) {
                entry->recorded = rec;
                entry->launches = launches;
                ++g_replays;
                g_last_launches = launches;
                return GGML_STATUS_SUCCESS;
            }
            if (rec) vx_graph_destroy(rec);
        }
        entry->no_replay = true; // e.g. a launch that must allocate: this graph stays with node-by-node launches
    }
    const ggml_status st = graph_compute_eager(ctx, cgraph, &launches);
    entry->launches = launches;
    g_last_launches = launches;
    return st;
}

ggml_status graph_compute_eager(backend_ctx * ctx, ggml_cgraph * cgraph, int * launches_out) {
    int launches = 0;
    const auto t_begin = std::chrono::steady_clock::now();
    // readers of every tensor in this graph (as an operand or as the source of a view): a pair of
    // nodes is only run as one launch when nothing else looks at the value between them
    const bool fusion = fusion_on();
    for (int i = 0; i < cgraph->n_nodes; ++i) { // weights buffers: pinned at their first product, writes into them reported
        const ggml_tensor * n = cgraph->nodes[i];
        if (n->op == GGML_OP_MUL_MAT && n->src[0]) pin_if_weights(n->src[0]->buffer);
        if (n->buffer && n->buffer->usage == GGML_BACKEND_BUFFER_USAGE_WEIGHTS && !ggml_op_is_empty(n->op)) written_to(n->buffer, n->data, ggml_nbytes(n));
    }
    reader_map readers;
    if (fusion && cgraph->n_nodes > 1) {
        readers.reserve((size_t) cgraph->n_nodes * 2);
        // Under ggml_backend_sched this graph is a window of a larger one (ggml_graph_view: no leafs of its own, the
        // whole graph's hash set and use counts): a node that is also read from another split must be stored like
        // an output.  Such nodes get a reader count no group accepts.  A whole graph needs none of this.
        const bool window = cgraph->leafs == nullptr && cgraph->use_counts && cgraph->visited_hash_set.keys && cgraph->visited_hash_set.size > 0;
        reader_map as_operand; // uses as src[] only, the quantity ggml's own use counts hold
        if (window) as_operand.reserve((size_t) cgraph->n_nodes * 2);
        for (int i = 0; i < cgraph->n_nodes; ++i) {
            const ggml_tensor * n = cgraph->nodes[i];
            for (int k = 0; k < GGML_MAX_SRC; ++k)
                if (n->src[k]) {
                    readers[n->src[k]]++;
                    if (window) as_operand[n->src[k]]++;
                }
            if (n->view_src) readers[n->view_src]++;
        }
        if (window) {
            for (int i = 0; i < cgraph->n_nodes; ++i) {
                const ggml_tensor * n = cgraph->nodes[i];
                const size_t pos = ggml_hash_find(&cgraph->visited_hash_set, n);
                if (pos == GGML_HASHSET_FULL || !ggml_bitset_get(cgraph->visited_hash_set.used, pos)) continue;
                const auto it = as_operand.find(n);
                if (cgraph->use_counts[pos] > (it == as_operand.end() ? 0 : it->second)) readers[n] += 1 << 20;
            }
        }
    }
    std::unordered_map<const ggml_tensor *, kv2_group> kv2_by_fa;
    std::unordered_map<const ggml_tensor *, const ggml_tensor *> kv2_absorbed;
    std::unordered_set<const ggml_tensor *> done;
    if (fusion && cgraph->n_nodes > 2) find_kv2_groups(cgraph, readers, kv2_by_fa, kv2_absorbed);
    std::unordered_map<const ggml_tensor *, concat_tree> cat_by_root;
    static const bool concat_trees = getenv("GGML_GFX950_NO_CONCAT_TREES") == nullptr;
    if (fusion && concat_trees && cgraph->n_nodes > 2) find_concat_trees(cgraph, readers, cat_by_root, kv2_absorbed); // (inner nodes are skipped like absorbed CONCATs)
    const auto t_analysed = std::chrono::steady_clock::now();
    for (int i = 0; i < cgraph->n_nodes; ++i) {
        ggml_tensor * node = cgraph->nodes[i];
        // the same two skips ggml-cpu applies (ggml/src/ggml-cpu/ggml-cpu.c:2956-2966)
        if (ggml_op_is_empty(node->op) || ggml_is_empty(node)) continue;
        if ((node->flags & GGML_TENSOR_FLAG_COMPUTE) == 0) continue;
        if (kv2_absorbed.count(node)) continue; // a CONCAT the attention node reads through
        if (done.count(node)) continue;         // computed ahead of its turn by a group
        vx_status rc = VX_ERR_UNSUPPORTED;
        bool fused = false;
        if (fusion && node->op == GGML_OP_RMS_NORM && i + 2 < cgraph->n_nodes) {
            // MiniCPMModel::rms_norm (RMS_NORM, MUL by the norm weight) whose value only the projections behind it read:
            // the normalisation joins their launch and the normalised tensor is never stored
            ggml_tensor * mul = cgraph->nodes[i + 1];
            const auto rd = [&](const ggml_tensor * t) { const auto it = readers.find(t); return it == readers.end() ? 0 : it->second; };
            const bool norm_pair = mul->op == GGML_OP_MUL && mul->src[0] == node && mul->src[1] != node && rd(node) == 1 &&
                                   (node->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 && (mul->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 &&
                                   (mul->flags & GGML_TENSOR_FLAG_COMPUTE) != 0;
            bool grouped = false;
            if (norm_pair && rd(mul) == 3) {
                grouped = compute_qkv_group(ctx, cgraph, i, readers, kv2_absorbed, done, &rc, node, mul);
            } else if (norm_pair && rd(mul) == 1) { // one product over row-fused weights behind the norm
                grouped = compute_fused_qkv_group(ctx, cgraph, i, readers, kv2_absorbed, done, &rc, node, mul) ||
                          compute_fused_gate_up_group(ctx, cgraph, i, readers, done, &rc, node, mul);
            } else if (norm_pair && rd(mul) == 2 && i + 4 < cgraph->n_nodes) {
                ggml_tensor * gate = cgraph->nodes[i + 2];
                ggml_tensor * up   = cgraph->nodes[i + 3];
                ggml_tensor * glu  = cgraph->nodes[i + 4];
                if (gate->op == GGML_OP_MUL_MAT && up->op == GGML_OP_MUL_MAT && glu->op == GGML_OP_GLU && gate->src[1] == mul && up->src[1] == mul &&
                    glu->src[0] == gate && glu->src[1] == up && ggml_get_glu_op(glu) == GGML_GLU_OP_SWIGLU && ((const int32_t *) glu->op_params)[1] == 0 &&
                    private_to_group(readers, gate) && private_to_group(readers, up) && (glu->flags & GGML_TENSOR_FLAG_COMPUTE) != 0) {
                    const vx_tensor x = to_vx(node->src[0]), nw = to_vx(mul->src[1]), gw = to_vx(gate->src[0]), uw = to_vx(up->src[0]), d = to_vx(glu);
                    float eps;
                    memcpy(&eps, node->op_params, sizeof(float));
                    // Prefill sizes, and the GLU's value read by the down projection alone (MUL_MAT [SCALE] ADD behind it): the
                    // whole of mlp_forward with its residual update as one call, the tokens x ffn tensor never stored
                    if (i + 6 < cgraph->n_nodes && private_to_group(readers, glu) && (glu->flags & GGML_TENSOR_FLAG_OUTPUT) == 0) {
                        ggml_tensor * down = cgraph->nodes[i + 5];
                        ggml_tensor * val = down;
                        float sc = 1.0f;
                        int ia = i + 6;
                        bool chain = down->op == GGML_OP_MUL_MAT && down->src[1] == glu && private_to_group(readers, down) &&
                                     (down->flags & GGML_TENSOR_FLAG_OUTPUT) == 0;
                        if (chain && cgraph->nodes[ia]->op == GGML_OP_SCALE) {
                            ggml_tensor * scn = cgraph->nodes[ia];
                            float bias;
                            memcpy(&sc, (const float *) scn->op_params + 0, sizeof(float));
                            memcpy(&bias, (const float *) scn->op_params + 1, sizeof(float));
                            chain = scn->src[0] == down && bias == 0.0f && private_to_group(readers, scn) && (scn->flags & GGML_TENSOR_FLAG_OUTPUT) == 0;
                            val = scn;
                            if (++ia >= cgraph->n_nodes) chain = false;
                        }
                        if (chain) {
                            ggml_tensor * add = cgraph->nodes[ia];
                            chain = add->op == GGML_OP_ADD && (add->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 && (add->src[0] == val) != (add->src[1] == val);
                            if (chain) {
                                ggml_tensor * residual = add->src[0] == val ? add->src[1] : add->src[0];
                                const vx_tensor dw = to_vx(down->src[0]), r = to_vx(residual), out = to_vx(add);
                                if (residual != down && residual != glu && apart(add, down->src[0]) && apart(add, gate->src[0]) && apart(add, up->src[0]) &&
                                    apart(add, mul->src[1]) && apart_or_same(add, residual) && apart_or_same(add, node->src[0]) &&
                                    (uintptr_t) x.data % 16 == 0 && (uintptr_t) nw.data % 16 == 0 &&
                                    vx_supports_mlp_tiled(&x, &nw, &gw, &uw, &dw, &r, &out, mul_mat_act_mode())) {
                                    rc = vx_mlp_tiled(&x, &nw, eps, &gw, &uw, &dw, &r, sc, &out, mul_mat_act_mode(), ctx->stream);
                                    done.insert(mul); done.insert(gate); done.insert(up); done.insert(glu); done.insert(down);
                                    if (val != down) done.insert(val);
                                    done.insert(add);
                                    grouped = true;
                                }
                            }
                        }
                    }
                    if (grouped) {} else
                    // (decode sizes on the streaming kernel, prefill sizes in the pre-tiled kernel's activation pass)
                    if ((vx_supports_norm_mul_mat_swiglu(&x, &nw, &gw, &uw, &d) || vx_supports_norm_mul_mat_swiglu_tiled(&x, &nw, &gw, &uw, &d, mul_mat_act_mode())) &&
                        (uintptr_t) x.data % 16 == 0 && (uintptr_t) nw.data % 16 == 0 &&
                        apart(glu, node->src[0])) {
                        rc = vx_norm_mul_mat_swiglu(&x, &nw, eps, &gw, &uw, &d, mul_mat_act_mode(), ctx->stream);
                        done.insert(mul); done.insert(gate); done.insert(up); done.insert(glu);
                        grouped = true;
                    }
                }
            }
            if (grouped) {
                ++launches;
                if (rc != VX_OK) {
                    NODE_FAILED("ggml-gfx950: node %d (%s, rms_norm + projections) failed with status %d: %s\n", i, node->name, (int) rc, vx_last_error());
                    return GGML_STATUS_FAILED;
                }
                continue;
            }
        }
        if (node->op == GGML_OP_CONCAT) {
            const auto it = cat_by_root.find(node);
            if (it != cat_by_root.end()) {
                const concat_tree & tree = it->second;
                vx_tensor ts[8];
                const vx_tensor * tp[8];
                for (size_t k = 0; k < tree.leaves.size(); ++k) { ts[k] = to_vx(tree.leaves[k]); tp[k] = &ts[k]; }
                const vx_tensor d = to_vx(node);
                rc = vx_concat_many(tp, tree.extents.data(), (int) tree.leaves.size(), tree.dim, &d, ctx->stream);
                ++launches;
                if (rc != VX_OK) {
                    NODE_FAILED("ggml-gfx950: node %d (%s, a tree of CONCATs) failed with status %d: %s\n", i, node->name, (int) rc, vx_last_error());
                    return GGML_STATUS_FAILED;
                }
                continue;
            }
        }
        if (fusion && node->op == GGML_OP_MUL_MAT &&
            (compute_qkv_group(ctx, cgraph, i, readers, kv2_absorbed, done, &rc) ||
             compute_kv_group(ctx, cgraph, i, readers, kv2_absorbed, done, &rc) ||
             compute_fused_qkv_group(ctx, cgraph, i, readers, kv2_absorbed, done, &rc) ||
             compute_fused_gate_up_group(ctx, cgraph, i, readers, done, &rc))) {
            ++launches;
            if (rc != VX_OK) {
                NODE_FAILED("ggml-gfx950: node %d (%s, q/k/v projections + rope) failed with status %d: %s\n", i, node->name, (int) rc, vx_last_error());
                return GGML_STATUS_FAILED;
            }
            continue;
        }
        if (node->op == GGML_OP_FLASH_ATTN_EXT) {
            const auto it = kv2_by_fa.find(node);
            if (it != kv2_by_fa.end()) {
                const int last = compute_kv2_attention_store(ctx, cgraph, i, it->second, readers, &rc);
                if (last >= 0) i = last;
                else rc = compute_kv2_attention(ctx, node, it->second);
                ++launches;
                if (rc != VX_OK) {
                    NODE_FAILED("ggml-gfx950: node %d (%s, two-segment attention) failed with status %d: %s\n", i, node->name, (int) rc, vx_last_error());
                    return GGML_STATUS_FAILED;
                }
                continue;
            }
            if (fusion) {
                const int last = compute_attention_store(ctx, cgraph, i, readers, &rc);
                if (last >= 0) {
                    ++launches;
                    if (rc != VX_OK) {
                        NODE_FAILED("ggml-gfx950: node %d (%s, attention + cache write) failed with status %d: %s\n", i, node->name, (int) rc, vx_last_error());
                        return GGML_STATUS_FAILED;
                    }
                    i = last;
                    continue;
                }
            }
        }
        if (fusion && i + 1 < cgraph->n_nodes) {
            int last = -1;
            if (node->op == GGML_OP_CPY) last = compute_kv_store_group(ctx, cgraph, i, readers, &rc);
            else if (node->op == GGML_OP_MUL_MAT) last = compute_mul_mat_residual_group(ctx, cgraph, i, readers, &rc);
            if (last < 0) last = compute_small_run(ctx, cgraph, i, readers, kv2_absorbed, done, &rc);
            if (last >= 0) {
                fused = true;
                i = last - 1; // the common increment below steps onto the group's last node
            }
        }
        if (!fused && fusion && i + 1 < cgraph->n_nodes) {
            ggml_tensor * next = cgraph->nodes[i + 1];
            const bool private_value = (node->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 && (next->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 &&
                                       readers[node] == 1;
            // mlp_forward's MUL_MAT(gate), MUL_MAT(up), SWIGLU(gate, up) at decode size: one launch
            if (private_value && i + 2 < cgraph->n_nodes && node->op == GGML_OP_MUL_MAT && next->op == GGML_OP_MUL_MAT) {
                ggml_tensor * glu = cgraph->nodes[i + 2];
                if (glu->op == GGML_OP_GLU && (glu->flags & GGML_TENSOR_FLAG_COMPUTE) != 0 && glu->src[0] == node && glu->src[1] == next &&
                    ggml_get_glu_op(glu) == GGML_GLU_OP_SWIGLU && ((const int32_t *) glu->op_params)[1] == 0 &&
                    next->src[1] == node->src[1] && (next->flags & GGML_TENSOR_FLAG_OUTPUT) == 0 && readers[next] == 1) {
                    const vx_tensor g = to_vx(node->src[0]), u = to_vx(next->src[0]), x = to_vx(node->src[1]), d = to_vx(glu);
                    if ((vx_supports_mul_mat_swiglu(&g, &u, &x, &d) || vx_supports_mul_mat_swiglu_tiled(&g, &u, &x, &d, mul_mat_act_mode())) &&
                        apart(glu, node->src[1])) {
                        rc = vx_mul_mat_swiglu(&g, &u, &x, &d, mul_mat_act_mode(), ctx->stream);
                        fused = true;
                        ++i; // one more node than a pair
                    }
                }
            }
            if (!fused && private_value) fused = compute_pair(ctx, node, next, &rc);
        }
        if (fused) ++i;
        else rc = compute_node(ctx, node);
        ++launches;
        if (rc != VX_OK) {
            NODE_FAILED("ggml-gfx950: node %d (%s, op %s) failed with status %d: %s\n", i, node->name,
                           ggml_op_name(node->op), (int) rc, rc == VX_ERR_UNSUPPORTED && !*vx_last_error() ? "operator not claimed by this backend" : vx_last_error());
            return GGML_STATUS_FAILED;
        }
    }
    *launches_out = launches;
    const auto t_end = std::chrono::steady_clock::now();
    g_host_ns[0] = std::chrono::duration_cast<std::chrono::nanoseconds>(t_analysed - t_begin).count();
    g_host_ns[1] = std::chrono::duration_cast<std::chrono::nanoseconds>(t_end - t_analysed).count();
    return GGML_STATUS_SUCCESS;
}

const ggml_backend_i backend_iface = {
    /* .get_name           = */ backend_get_name,
    /* .free               = */ backend_free,
    /* .set_tensor_async   = */ backend_set_tensor_async,
    /* .get_tensor_async   = */ backend_get_tensor_async,
    /* .cpy_tensor_async   = */ nullptr,
    /* .synchronize        = */ backend_synchronize,
    /* .graph_plan_create  = */ nullptr,
    /* .graph_plan_free    = */ nullptr,
    /* .graph_plan_update  = */ nullptr,
    /* .graph_plan_compute = */ nullptr,
    /* .graph_compute      = */ backend_graph_compute,
    /* .event_record       = */ nullptr,
    /* .event_wait         = */ nullptr,
    /* .graph_optimize     = */ backend_graph_optimize,
};

ggml_guid_t backend_guid() {
    static ggml_guid guid = { 0x67, 0x66, 0x78, 0x39, 0x35, 0x30, 0x2d, 0x76, 0x6f, 0x78, 0x63, 0x70, 0x6d, 0x2d, 0x30, 0x31 };
    return &guid;
}

// ---------------------------------------------------------------------------------- device
const char * dev_get_name(ggml_backend_dev_t dev) { return ((device_ctx *) dev->context)->name.c_str(); }
const char * dev_get_description(ggml_backend_dev_t dev) { return ((device_ctx *) dev->context)->description.c_str(); }

void dev_get_memory(ggml_backend_dev_t dev, size_t * free, size_t * total) {
    *free = *total = 0;
    vx_device_info(((device_ctx *) dev->context)->index, nullptr, 0, free, total, nullptr);
}

enum ggml_backend_dev_type dev_get_type(ggml_backend_dev_t) { return GGML_BACKEND_DEVICE_TYPE_GPU; }

void dev_get_props(ggml_backend_dev_t dev, ggml_backend_dev_props * props) {
    props->name        = dev_get_name(dev);
    props->description = dev_get_description(dev);
    props->type        = dev_get_type(dev);
    props->device_id   = nullptr;
    dev_get_memory(dev, &props->memory_free, &props->memory_total);
    props->caps = { /* async */ true, /* host_buffer */ true, /* buffer_from_host_ptr */ false, /* events */ false };
}

ggml_backend_t dev_init_backend(ggml_backend_dev_t dev, const char *) {
    device_ctx * dctx = (device_ctx *) dev->context;
    if (vx_init(dctx->index) != VX_OK) {
        GGML_LOG_ERROR("ggml-gfx950: %s\n", vx_last_error());
        return nullptr;
    }
    vx_stream stream = nullptr;
    if (vx_stream_create(&stream) != VX_OK) {
        GGML_LOG_ERROR("ggml-gfx950: %s\n", vx_last_error());
        return nullptr;
    }
    return new ggml_backend{ backend_guid(), backend_iface, dev, new backend_ctx{ dctx->index, stream } };
}

ggml_backend_buffer_type_t dev_get_host_buffer_type(ggml_backend_dev_t dev) {
    static ggml_backend_buffer_type host_buft = {
        /* .iface   = */ { host_buft_get_name, host_buft_alloc_buffer, host_buft_get_alignment, nullptr, nullptr, host_buft_is_host },
        /* .device  = */ nullptr,
        /* .context = */ nullptr,
    };
    host_buft.device = dev;
    return &host_buft;
}

bool dev_supports_buft(ggml_backend_dev_t dev, ggml_backend_buffer_type_t buft) { return buft == device_buffer_type(dev); }

const ggml_backend_device_i device_iface = {
    /* .get_name             = */ dev_get_name,
    /* .get_description      = */ dev_get_description,
    /* .get_memory           = */ dev_get_memory,
    /* .get_type             = */ dev_get_type,
    /* .get_props            = */ dev_get_props,
    /* .init_backend         = */ dev_init_backend,
    /* .get_buffer_type      = */ device_buffer_type,
    /* .get_host_buffer_type = */ dev_get_host_buffer_type,
    /* .buffer_from_host_ptr = */ nullptr,
    /* .supports_op          = */ supports_op,
    /* .supports_buft        = */ dev_supports_buft,
    /* .offload_op           = */ nullptr,
    /* .event_new            = */ nullptr,
    /* .event_free           = */ nullptr,
    /* .event_synchronize    = */ nullptr,
};

// --------------------------------------------------------------------------------- registry
struct reg_ctx {
    std::vector<ggml_backend_device *>      devices;
    std::vector<ggml_backend_buffer_type *> bufts;
};

reg_ctx * registry_state(ggml_backend_reg_t reg) {
    static reg_ctx ctx;
    static std::once_flag once;
    std::call_once(once, [reg] {
        const int n = vx_device_count();
        for (int i = 0; i < n; ++i) {
            char desc[256] = "";
            vx_device_info(i, desc, sizeof(desc), nullptr, nullptr, nullptr);
            device_ctx * dctx = new device_ctx{ i, "GFX950_" + std::to_string(i), desc };
            ggml_backend_device * dev = new ggml_backend_device{ device_iface, reg, dctx };
            ctx.devices.push_back(dev);
            ctx.bufts.push_back(new ggml_backend_buffer_type{
                { buft_get_name, buft_alloc_buffer, buft_get_alignment, nullptr, nullptr, buft_is_host }, dev, nullptr });
        }
    });
    return &ctx;
}

ggml_backend_buffer_type_t device_buffer_type(ggml_backend_dev_t dev) {
    return registry_state(dev->reg)->bufts[((device_ctx *) dev->context)->index];
}

// The registry name.  VoxCPM.cpp chooses its GPU device by this name -- it looks for "cuda" or "vulkan" in it
// (src/backend.cpp:75-105 of the reference) -- so an unpatched VoxCPM build finds this backend when the environment
// names an alias, e.g. GGML_GFX950_REG_NAME=CUDA-gfx950 with `--backend cuda`; device names stay GFX950_<i>.
const char * reg_get_name(ggml_backend_reg_t) {
    static const std::string name = [] {
        const char * e = getenv("GGML_GFX950_REG_NAME");
        return std::string(e && *e ? e : "GFX950");
    }();
    return name.c_str();
}
size_t       reg_get_device_count(ggml_backend_reg_t reg) { return registry_state(reg)->devices.size(); }

ggml_backend_dev_t reg_get_device(ggml_backend_reg_t reg, size_t index) {
    reg_ctx * ctx = registry_state(reg);
    GGML_ASSERT(index < ctx->devices.size());
    return ctx->devices[index];
}

void * reg_get_proc_address(ggml_backend_reg_t, const char * name) {
    if (!name) return nullptr;
    if (strcmp(name, "ggml_backend_gfx950_weight_on_device") == 0) return (void *) ggml_backend_gfx950_weight_on_device;
    if (strcmp(name, "ggml_backend_gfx950_alloc_weights") == 0) return (void *) ggml_backend_gfx950_alloc_weights;
    if (strcmp(name, "ggml_backend_gfx950_last_launches") == 0) return (void *) ggml_backend_gfx950_last_launches;
    if (strcmp(name, "ggml_backend_gfx950_replays") == 0) return (void *) ggml_backend_gfx950_replays;
    if (strcmp(name, "ggml_backend_gfx950_patched_replays") == 0) return (void *) ggml_backend_gfx950_patched_replays;
    if (strcmp(name, "ggml_backend_gfx950_set_graph_patch") == 0) return (void *) ggml_backend_gfx950_set_graph_patch;
    if (strcmp(name, "ggml_backend_gfx950_set_graph_replay") == 0) return (void *) ggml_backend_gfx950_set_graph_replay;
    if (strcmp(name, "ggml_backend_gfx950_set_mul_mat_act") == 0) return (void *) ggml_backend_gfx950_set_mul_mat_act;
    if (strcmp(name, "ggml_backend_gfx950_set_fusion") == 0) return (void *) ggml_backend_gfx950_set_fusion;
    return nullptr;
}

} // namespace

extern "C" {

GGML_BACKEND_API ggml_backend_reg_t ggml_backend_gfx950_reg(void) {
    static ggml_backend_reg reg = {
        /* .api_version = */ GGML_BACKEND_API_VERSION,
        /* .iface       = */ { reg_get_name, reg_get_device_count, reg_get_device, reg_get_proc_address },
        /* .context     = */ nullptr,
    };
    return &reg;
}

// entry points ggml's loader looks up (ggml/src/ggml-backend-impl.h:215-251)
GGML_BACKEND_API ggml_backend_reg_t ggml_backend_init(void) { return ggml_backend_gfx950_reg(); }
GGML_BACKEND_API int                ggml_backend_score(void) { return vx_device_count() > 0 ? 100 : 0; }

} // extern "C"

// Diagnostic: how many operator calls the most recent graph_compute of this process issued (an attention
// call counts once although it may launch a split and a merge kernel).
extern "C" int ggml_backend_gfx950_last_launches(void) { return g_last_launches; }
// Diagnostic: host nanoseconds the most recent node-by-node graph_compute spent (0) analysing the graph, (1) issuing launches
extern "C" long long ggml_backend_gfx950_host_ns(int which) { return which == 0 || which == 1 ? g_host_ns[which] : 0; }
// how many graph_compute calls of this process were served by replaying a recorded graph
extern "C" int ggml_backend_gfx950_replays(void) { return g_replays; }
// how many of them brought a recording's arguments up to date first (the steps of a decode loop)
extern "C" int ggml_backend_gfx950_patched_replays(void) { return g_patched_replays; }
// nodes whose arguments the most recent such call changed
extern "C" int ggml_backend_gfx950_last_patched(void) { return g_last_patched; }
extern "C" int ggml_backend_gfx950_set_graph_patch(int on) {
    const int before = patch_on();
    g_patch_on = on != 0;
    return before;
}
// switches the recognition of recurring graphs on (1) or off (0); returns the previous setting
extern "C" int ggml_backend_gfx950_set_graph_replay(int on) {
    if (g_replay_on < 0) { const char * e = getenv("GGML_GFX950_GRAPH_REPLAY"); g_replay_on = !(e && atoi(e) == 0); }
    const int before = g_replay_on;
    g_replay_on = on != 0;
    return before;
}

// switches the grouping of nodes into single launches on (1) or off (0: every node its own launch) for later graph_compute
// calls; returns the previous setting.  Results do not depend on it.
extern "C" int ggml_backend_gfx950_set_fusion(int on) {
    const int before = fusion_on();
    g_fusion_on = on != 0;
    return before;
}

// ---- weight placement (declared and explained in ggml-gfx950.h) ------------------------------------------------------
extern "C" int ggml_backend_gfx950_weight_on_device(const char * tensor_name) {
    if (!tensor_name) return 1;
    return strncmp(tensor_name, "audio_vae.", 10) == 0 ? 0 : 1;
}

extern "C" bool ggml_backend_gfx950_alloc_weights(struct ggml_context * ctx, ggml_backend_t backend, ggml_backend_buffer_t * device_buffer,
                                                  ggml_backend_buffer_t * host_buffer) {
    if (device_buffer) *device_buffer = nullptr;
    if (host_buffer) *host_buffer = nullptr;
    if (!ctx || !backend || !device_buffer || !host_buffer) return false;
    ggml_backend_dev_t dev = ggml_backend_get_device(backend);
    if (!dev) return false;
    ggml_backend_buffer_type_t host_buft = ggml_backend_dev_host_buffer_type(dev);
    ggml_backend_buffer_type_t dev_buft  = ggml_backend_dev_buffer_type(dev);
    if (!host_buft || !dev_buft) return false;
    // the host share first: its tensors are placed one after the other in one pinned block
    const size_t align = ggml_backend_buft_get_alignment(host_buft);
    size_t host_bytes = 0, n_host = 0, n_dev = 0;
    for (ggml_tensor * t = ggml_get_first_tensor(ctx); t; t = ggml_get_next_tensor(ctx, t)) {
        if (t->data || t->view_src) continue;
        if (ggml_backend_gfx950_weight_on_device(t->name)) { ++n_dev; continue; }
        host_bytes += GGML_PAD(ggml_backend_buft_get_alloc_size(host_buft, t), align);
        ++n_host;
    }
    if (n_host) {
        *host_buffer = ggml_backend_buft_alloc_buffer(host_buft, host_bytes);
        if (!*host_buffer) return false;
        ggml_backend_buffer_set_usage(*host_buffer, GGML_BACKEND_BUFFER_USAGE_WEIGHTS);
        ggml_tallocr talloc = ggml_tallocr_new(*host_buffer);
        for (ggml_tensor * t = ggml_get_first_tensor(ctx); t; t = ggml_get_next_tensor(ctx, t)) {
            if (t->data || t->view_src || ggml_backend_gfx950_weight_on_device(t->name)) continue;
            if (ggml_tallocr_alloc(&talloc, t) != GGML_STATUS_SUCCESS) {
                ggml_backend_buffer_free(*host_buffer);
                *host_buffer = nullptr;
                return false;
            }
        }
    }
    if (n_dev) { // ggml allocates whatever is still unallocated (views included) in one buffer of the device type
        *device_buffer = ggml_backend_alloc_ctx_tensors_from_buft(ctx, dev_buft);
        if (!*device_buffer) {
            if (*host_buffer) ggml_backend_buffer_free(*host_buffer);
            *host_buffer = nullptr;
            return false;
        }
        ggml_backend_buffer_set_usage(*device_buffer, GGML_BACKEND_BUFFER_USAGE_WEIGHTS);
    }
    return true;
}
// Selects VX_ACT_FLOAT (0) or VX_ACT_Q8 (1) for the Q8_0 products of later graph_compute calls; returns the previous
// mode.  The environment variable GGML_GFX950_MUL_MAT_ACT=q8 sets the initial one.
extern "C" int ggml_backend_gfx950_set_mul_mat_act(int mode) {
    const int before = mul_mat_act_mode();
    if (mode == VX_ACT_FLOAT || mode == VX_ACT_Q8) g_mul_mat_act = mode;
    return before;
}
