/*
 * voxcpm_gfx950.h -- C ABI of the MI355X (gfx950) kernels behind VoxCPM.cpp's attention
 * hot path.  One shared library, libvoxcpm_gfx950.so; plain pointers and sizes only.
 *
 * Each vx_<op> entry point computes exactly one ggml operator with ggml's semantics, so a
 * ggml backend's graph_compute can forward a node to it unchanged: the ggml backend plugin
 * in this repository (libggml-gfx950.so) is that caller, and the entry points below are
 * what its dispatch switch binds -- the counterpart, for this path, of the per-op
 * functions ggml-cpu reaches from ggml_compute_forward()
 * (third_party/ggml/src/ggml-cpu/ggml-cpu.c:1680-2089 in the reference).
 *
 * Tensors are described as ggml describes them: ne[0] is the fastest dimension, nb[] are
 * byte strides, `data` is a DEVICE pointer.  Types use ggml's numbering.  Every op
 * validates shapes, types and strides on the host before launching anything and returns a
 * vx_status; nothing here falls back to the CPU.
 *
 * Streams: `stream` is a hipStream_t passed as void* (NULL = the null stream).  All work
 * is enqueued asynchronously on it.  Ops that need scratch memory take it from a
 * per-stream workspace the library grows on demand with hipMalloc (see vx_workspace_reserve).
 */
#ifndef VOXCPM_GFX950_H
#define VOXCPM_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define VX_API __attribute__((visibility("default")))

/* enum ggml_type values (third_party/ggml/include/ggml.h:389-431) */
enum vx_type { VX_TYPE_F32 = 0, VX_TYPE_F16 = 1, VX_TYPE_Q8_0 = 8, VX_TYPE_I32 = 26 };

typedef enum vx_status {
    VX_OK = 0,
    VX_ERR_NO_DEVICE = 1,   /* no gfx950 device / HIP runtime unusable */
    VX_ERR_UNSUPPORTED = 2, /* shape / type / stride combination this build does not claim */
    VX_ERR_INVALID = 3,     /* arguments violate the operator's contract */
    VX_ERR_HIP = 4,         /* a HIP call failed; see vx_last_error() */
    VX_ERR_ALLOC = 5
} vx_status;

/* struct ggml_tensor's {type, ne, nb, data} (third_party/ggml/include/ggml.h:655-691) */
typedef struct vx_tensor {
    int32_t  type;
    int32_t  _pad;
    int64_t  ne[4];
    uint64_t nb[4];
    void *   data;
} vx_tensor;

typedef void * vx_stream;

/* ---- runtime --------------------------------------------------------------------------
 * Replaces what ggml_backend_reg/device/buffer entries need from a device runtime
 * (third_party/ggml/src/ggml-backend-impl.h:17-58, 140-182): count devices, describe
 * them, allocate, copy, fill, synchronise. */
VX_API int          vx_device_count(void);                 /* gfx950 devices visible; 0 if none */
VX_API vx_status    vx_init(int device);                   /* make `device` current for this thread */
VX_API const char * vx_last_error(void);                   /* thread-local message of the last failure */
VX_API vx_status    vx_device_info(int device, char * name, size_t name_len,
                                   size_t * free_bytes, size_t * total_bytes, int * compute_units);
VX_API vx_status    vx_malloc(void ** ptr, size_t bytes);
VX_API vx_status    vx_free(void * ptr);
VX_API vx_status    vx_malloc_host(void ** ptr, size_t bytes);   /* pinned host memory */
VX_API vx_status    vx_free_host(void * ptr);
VX_API vx_status    vx_memcpy_h2d(void * dst, const void * src, size_t bytes, vx_stream stream);
VX_API vx_status    vx_memcpy_d2h(void * dst, const void * src, size_t bytes, vx_stream stream);
VX_API vx_status    vx_memcpy_d2d(void * dst, const void * src, size_t bytes, vx_stream stream);
VX_API vx_status    vx_memset(void * dst, int value, size_t bytes, vx_stream stream);
VX_API vx_status    vx_stream_create(vx_stream * stream);
VX_API vx_status    vx_stream_destroy(vx_stream stream);
VX_API vx_status    vx_stream_synchronize(vx_stream stream);
/* The per-stream workspace (split-KV partials, split-K partials, block sums, mask classification).  It grows on
 * demand; a block that was handed out keeps its address and stays allocated until vx_stream_destroy, also after a
 * larger block has replaced it, so launches already queued and HIP graphs already captured from the stream stay
 * valid.  A call that would have to grow the workspace while the stream is being captured returns
 * VX_ERR_UNSUPPORTED: reserve the largest size first.  No counterpart in the reference (ggml-cpu takes its scratch
 * from the compute plan's work buffer, ggml/src/ggml-cpu/ggml-cpu.c:2700-2935). */
VX_API vx_status    vx_workspace_reserve(vx_stream stream, size_t bytes);
/* current block, its size and the number of superseded blocks still held for this stream (any out pointer may be NULL) */
VX_API vx_status    vx_workspace_info(vx_stream stream, void ** ptr, size_t * bytes, int * retired_blocks);

/* Constant weights.  ggml marks the buffers that hold a model's weights (ggml_backend_buffer_set_usage(...,
 * GGML_BACKEND_BUFFER_USAGE_WEIGHTS), the reference's src/weight-store.cpp:86 and src/minicpm.cpp:472); this is the same
 * statement for the C ABI.  For a tensor that lies wholly inside a pinned range an operator may keep a re-laid-out copy
 * between calls instead of producing it on every call (today: the tiles of the Q8_0 weights of products with 1024 tokens
 * or more, 2.1 bytes per weight, at most VX_DERIVED_WEIGHTS_MB megabytes per process, default 8192).  Results do not
 * depend on it.  The owner of the memory calls vx_weights_changed for every range it writes to afterwards (copies derived
 * from those bytes are dropped), and vx_weights_unpin(base) before it frees or reuses the memory.  Ranges are per device
 * (the current one); the calls are thread-safe.  vx_weights_info reports the ranges pinned and the copies held. */
VX_API vx_status    vx_weights_pin(const void * base, size_t bytes);
VX_API vx_status    vx_weights_changed(const void * base, size_t bytes);
VX_API vx_status    vx_weights_unpin(const void * base);
VX_API vx_status    vx_weights_info(size_t * pinned_ranges, size_t * derived_copies, size_t * derived_bytes);

/* Recording the launches of a stream and replaying them as one unit (a HIP graph).  The reference builds and launches
 * its step graph anew on every call (src/voxcpm.cpp:485-495); a backend that recognises a graph it has already run can
 * replay the recorded launches instead of issuing them one by one.  Between begin and end every vx_* call on `stream`
 * is recorded, not executed; a call that would have to grow the workspace fails (see vx_workspace_reserve) and the
 * caller should end the recording, discard it and run eagerly.  The pointers and shapes of the recorded calls are
 * baked in: replay only while they are all still valid.  No counterpart in ggml-cpu. */
typedef void * vx_graph;
VX_API vx_status    vx_graph_begin(vx_stream stream);
VX_API vx_status    vx_graph_end(vx_stream stream, vx_graph * graph);   /* *graph = NULL when nothing usable was recorded */
VX_API vx_status    vx_graph_launch(vx_graph graph, vx_stream stream);
VX_API vx_status    vx_graph_destroy(vx_graph graph);
/* Running a recording again with other arguments.  A decode step's graph differs from the previous step's only in what
 * follows from the position (the key count of the attention launches, the cache slot that is written: the reference's
 * src/minicpm.cpp:393-470 builds them from n_past), so its launches are the recorded ones with a few arguments changed.
 * Between patch_begin and patch_end every vx_* operator call of the calling thread launches nothing: each launch it
 * would have made is compared, in order, with the recording's, and where the grid, the block, the LDS size or the
 * argument bytes differ they are set on the recorded graph's node.  patch_end returns VX_OK when the calls made the same
 * kernels in the same order and number as the recording (*patched = how many nodes were changed): vx_graph_launch then
 * runs the graph with the new arguments.  VX_ERR_UNSUPPORTED means they did not: the graph's arguments are then a
 * mixture, destroy it and run the calls again normally.  patch_begin waits for the graph's previous launch to finish
 * (its arguments must not change under it): a caller that wants the host to run ahead of the GPU alternates between two
 * recordings.  vx_graph_patchable says whether a recording can be used this way (all of its launches are kernels of this
 * library).  No counterpart in ggml-cpu. */
VX_API int          vx_graph_patchable(vx_graph graph);
VX_API vx_status    vx_graph_patch_begin(vx_graph graph);
VX_API vx_status    vx_graph_patch_end(vx_graph graph, int * patched);

/* ---- GGML_OP_RMS_NORM -------------------------------------------------------------------
 * replaces ggml_compute_forward_rms_norm (ggml/src/ggml-cpu/ops.cpp:3710-3777).
 * src, dst F32, same shape, ne[0] dense; rows may be strided; dst may alias src. */
VX_API vx_status vx_rms_norm(const vx_tensor * src, const vx_tensor * dst, float eps, vx_stream stream);

/* ---- GGML_OP_ROPE ------------------------------------------------------------------------
 * replaces ggml_compute_forward_rope (ggml/src/ggml-cpu/ops.cpp:5589-5882) for F32 tensors,
 * mode 0 (NORMAL) and 2 (NEOX); argument meaning as ggml_rope_ext
 * (ggml/include/ggml.h:1767-1781).  pos: device int32[ne2]; freq_factors: device
 * float[>= n_dims/2] or NULL; dst may alias src. */
VX_API vx_status vx_rope(const vx_tensor * src, const int32_t * pos, const float * freq_factors,
                         const vx_tensor * dst, int n_dims, int mode, int n_ctx_orig,
                         float freq_base, float freq_scale, float ext_factor, float attn_factor,
                         float beta_fast, float beta_slow, vx_stream stream);

/* ---- GGML_OP_SOFT_MAX ----------------------------------------------------------------------
 * replaces ggml_compute_forward_soft_max (ggml/src/ggml-cpu/ops.cpp:5225-5353):
 * dst = softmax(scale*src + slope(head)*mask) with optional sinks.  src F32; mask F16|F32
 * [ne0, >=ne1, ne2 | 1.., ne3 | 1..] or NULL; sinks device float[ne2] or NULL; dst F32
 * contiguous, may alias src. */
VX_API vx_status vx_soft_max(const vx_tensor * src, const vx_tensor * mask, const float * sinks,
                             const vx_tensor * dst, float scale, float max_bias, vx_stream stream);

/* ---- GGML_OP_FLASH_ATTN_EXT ----------------------------------------------------------------
 * replaces ggml_compute_forward_flash_attn_ext (ggml/src/ggml-cpu/ops.cpp:8109-8853).
 * q [D, n_q, Hq, ne3] F32; k [D, n_kv, Hkv, ne3'] F16|F32; v like k; mask [n_kv, >=n_q,
 * ne32, ne33] F16 or NULL; sinks device float[Hq] or NULL; dst [D, Hq, n_q, ne3] F32
 * contiguous.  D (= DK = DV) in {64, 128}.  Row strides are free (permuted views and
 * KV-cache views are fine); the innermost dimension must be dense. */
VX_API vx_status vx_flash_attn_ext(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                   const vx_tensor * mask, const float * sinks, const vx_tensor * dst,
                                   float scale, float max_bias, float logit_softcap,
                                   vx_stream stream);

/* vx_flash_attn_ext for callers that must not allocate: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, same results as
 * vx_flash_attn_ext wherever that call takes the key-range (split-KV) kernels, i.e. decode and LocDiT-sized query
 * counts; long prefills run on the same kernels too (within the operator's 2e-3 tolerance of the LDS-tiled kernel
 * vx_flash_attn_ext would choose, and slower).  The partial results of the key ranges go to a fixed array of
 * VX_FLASH_ATTN_EXT_STATIC_SCRATCH_BYTES that is part of the loaded library on each GPU (held until the process ends)
 * instead of the per-stream workspace; the call performs no hipMalloc / hipFree.  A shape whose partials would not fit
 * is refused with VX_ERR_UNSUPPORTED.  All calls on one GPU share the array: calls that overlap in time on one GPU
 * (different streams, different threads) race; issue them on one stream or order them yourself.  Nothing in the
 * array needs clearing between calls (every partial that is read has been written by the same call). */
#define VX_FLASH_ATTN_EXT_STATIC_SCRATCH_BYTES ((size_t) 16 << 20)
VX_API vx_status vx_flash_attn_ext_static(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                          const vx_tensor * mask, const float * sinks, const vx_tensor * dst,
                                          float scale, float max_bias, float logit_softcap,
                                          vx_stream stream);

/* ---- GGML_OP_MUL_MAT -----------------------------------------------------------------------
 * replaces ggml_compute_forward_mul_mat (ggml/src/ggml-cpu/ggml-cpu.c:1139-1421):
 * dst[ne01, ne11, ne12, ne13] = src0[ne00, ne01, ne02, ne03]^T x src1[ne00, ne11, ne12, ne13],
 * src0 broadcast over dims 2,3.  src0 Q8_0 | F16 | F32 (rows dense), src1 F32, dst F32
 * contiguous.
 * act_mode selects how src1 enters the product for Q8_0 weights:
 *   VX_ACT_FLOAT -- weights dequantised on the fly (q*d exactly; with the environment variable
 *                   VX_GEMM_LDS=2 the tiled kernel for >= 64 tokens rounds q*d once to f16 instead),
 *                   activations as f16/f32
 *   VX_ACT_Q8    -- activations quantised to Q8_0 blocks first, integer block dots scaled
 *                   by d_w*d_x: the arithmetic ggml-cpu performs
 *                   (ggml/src/ggml-cpu/arch/x86/quants.c:290-386, 1012-1078). */
enum vx_act_mode { VX_ACT_FLOAT = 0, VX_ACT_Q8 = 1 };
VX_API vx_status vx_mul_mat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst,
                            int act_mode, vx_stream stream);

/* ---- supports queries ------------------------------------------------------------------------
 * what ggml_backend_device_i::supports_op asks (ggml/src/ggml-backend-impl.h:163-164):
 * 1 if the matching vx_<op> call would be accepted, 0 otherwise.  No device needed. */
VX_API int vx_supports_rms_norm(const vx_tensor * src, const vx_tensor * dst);
VX_API int vx_supports_rope(const vx_tensor * src, const vx_tensor * dst, int n_dims, int mode);
VX_API int vx_supports_soft_max(const vx_tensor * src, const vx_tensor * mask, const vx_tensor * dst);
VX_API int vx_supports_flash_attn_ext(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                      const vx_tensor * mask, const vx_tensor * dst);
VX_API int vx_supports_mul_mat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst);

/* ---- KV-cache helpers ----------------------------------------------------------------------
 * MiniCPMKVCache's views (src/minicpm.cpp:200-236) as descriptors over one device cache
 * tensor [head_dim, max_length, n_kv_heads] of element size `es`. */
VX_API vx_status vx_kv_read_view(const vx_tensor * cache, int seq_len, vx_tensor * view);
VX_API vx_status vx_kv_write_view(const vx_tensor * cache, int start, int n_tokens, vx_tensor * view);
/* ggml_cpy(cur, write view): rows of `src` F32 [D, Hkv, n_tokens] (any strides) stored into
 * `view` (F16 or F32), converting to the cache type with round-to-nearest-even -- what
 * ggml-cpu's CPY does for f32 -> f16 (ggml/src/ggml-cpu/ops.cpp:47-268, 526-565). */
VX_API vx_status vx_kv_store(const vx_tensor * src, const vx_tensor * view, vx_stream stream);

/* ---- glue operators of the decoder layer -----------------------------------------------------
 * The operators src/minicpm.cpp:572-775 puts between the projections and attention, so that a
 * whole layer can stay on the device.  F32 unless stated; any strides (16-byte accesses when
 * rows are dense and aligned); `op` arguments use ggml's enum values. */
enum { VX_BIN_ADD = 0, VX_BIN_SUB = 1, VX_BIN_MUL = 2, VX_BIN_DIV = 3 };
/* enum ggml_unary_op (third_party/ggml/include/ggml.h:578-603), the ones implemented */
enum { VX_UNARY_ABS = 0, VX_UNARY_SGN = 1, VX_UNARY_NEG = 2, VX_UNARY_STEP = 3, VX_UNARY_TANH = 4,
       VX_UNARY_RELU = 6, VX_UNARY_SIGMOID = 7, VX_UNARY_SILU = 10, VX_UNARY_EXP = 13,
       VX_UNARY_FLOOR = 18, VX_UNARY_CEIL = 19, VX_UNARY_ROUND = 20, VX_UNARY_TRUNC = 21,
       /* ggml's stand-alone elementwise ops (GGML_OP_SQR / SQRT / LOG / SIN / COS,
        * ggml/src/ggml-cpu/unary-ops.cpp:52-70), served by the same call; codes of this library */
       VX_UNARY_SQR = 100, VX_UNARY_SQRT = 101, VX_UNARY_LOG = 102, VX_UNARY_SIN = 103, VX_UNARY_COS = 104 };
/* enum ggml_glu_op (ggml.h:605-614) */
enum { VX_GLU_REGLU = 0, VX_GLU_SWIGLU = 2 };

/* GGML_OP_ADD / SUB / MUL / DIV: replaces apply_binary_op (ggml/src/ggml-cpu/binary-ops.cpp:50-112);
 * dst has src0's shape, src1 is repeated over it (ggml_can_repeat). */
VX_API vx_status vx_binary(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, vx_stream stream);
/* GGML_OP_ADD1: dst = src0 + src1[0] (ggml/src/ggml-cpu/ops.cpp:772-830) */
VX_API vx_status vx_add1(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, vx_stream stream);
/* GGML_OP_SCALE: dst = src * scale (+ bias, fused) (ops.cpp:4374-4424) */
VX_API vx_status vx_scale(const vx_tensor * src, const vx_tensor * dst, float scale, float bias, vx_stream stream);
/* GGML_OP_UNARY (ops.cpp:9617-9719; SILU = x / (1 + expf(-x)), vec.h:1061-1063) */
VX_API vx_status vx_unary(int op, const vx_tensor * src, const vx_tensor * dst, vx_stream stream);
/* GGML_OP_GLU: dst = act(a) * b; src1 == NULL means a, b are the halves of src0's rows
 * (swapped exchanges them) (ops.cpp:3127-3185, 9721-9760) */
VX_API vx_status vx_glu(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int swapped, vx_stream stream);
/* GGML_OP_CPY / CONT / DUP between F32 and F16 tensors holding the same number of elements:
 * element i of src (row-major over src's shape) lands in element i of dst
 * (ggml_compute_forward_dup, ops.cpp:526-565); F32 -> F16 rounds to nearest even.  Also I32 -> F32
 * (ggml_cast of position ids, src/minicpm.cpp:606), F32 -> I32 (C truncation) and I32 -> I32. */
VX_API vx_status vx_cpy(const vx_tensor * src, const vx_tensor * dst, vx_stream stream);
/* GGML_OP_CONCAT along `dim`, F32 / F16 / I32 (ops.cpp:1891-2095) */
VX_API vx_status vx_concat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int dim, vx_stream stream);
/* GGML_OP_SUM: every element summed in double, rounded once (ops.cpp:1275-1300) */
VX_API vx_status vx_sum(const vx_tensor * src, const vx_tensor * dst, vx_stream stream);
/* GGML_OP_SUM_ROWS: dst[0, i1, i2, i3] = the row's elements summed in double, rounded once
 * (ggml_compute_forward_sum_rows_f32, ops.cpp:1451-1482, ggml_vec_sum_f32, vec.h:1510-1520) */
VX_API vx_status vx_sum_rows(const vx_tensor * src, const vx_tensor * dst, vx_stream stream);
VX_API int vx_supports_sum_rows(const vx_tensor * src, const vx_tensor * dst);
/* GGML_OP_ARANGE: dst[i] = start + step * i over a contiguous F32 tensor, the product rounded before the sum
 * (ggml_compute_forward_arange_f32, ops.cpp:7881-7902); the element count is dst's (ggml fixes it at graph build) */
VX_API vx_status vx_arange(const vx_tensor * dst, float start, float step, vx_stream stream);
/* GGML_OP_REPEAT: src tiled over dst, every dst dim a whole multiple of src's; F32 / F16 / I32, any strides
 * (ggml_compute_forward_repeat, ops.cpp:1689-1810).  The reference builds its attention masks from ARANGE +
 * REPEAT (src/minicpm.cpp:602-620, src/locdit.cpp:283-305). */
VX_API vx_status vx_repeat(const vx_tensor * src, const vx_tensor * dst, vx_stream stream);

/* A tree of GGML_OP_CONCAT nodes along one dimension as one launch: dst is its 2 .. 8 leaves side by side along `dim`, leaf k
 * filling extents[k] indices.  A leaf smaller than its slot (in any dimension) is repeated as GGML_OP_REPEAT would have
 * repeated it in front of the CONCAT.  LocDiT's sequence assembly for several requests is such a tree: (mu + t | cond | x)
 * and (t repeated | cond | x) joined once more (src/locdit.cpp:401-452; with one request per graph the same nodes are a few
 * KB and ride in vx_small_graph).  The bytes written are those of the node-by-node sequence.  F32 / I32. */
VX_API vx_status vx_concat_many(const vx_tensor * const * srcs, const int64_t * extents, int n_src, int dim, const vx_tensor * dst,
                                vx_stream stream);
VX_API int vx_supports_concat_many(const vx_tensor * const * srcs, const int64_t * extents, int n_src, int dim, const vx_tensor * dst);
/* GGML_OP_GET_ROWS: dst[:, i, j, k] = row rows[i, j, k] of table matrix (j, k), as F32; table F32 / F16 / Q8_0
 * (dequantised exactly as dequantize_row_q8_0, ggml/src/ggml-quants.c:401-415) or I32 (dst I32); rows I32
 * (ggml_compute_forward_get_rows, ops.cpp:4653-4870; the token embedding, src/components.cpp:223).  An index
 * outside the table makes ggml-cpu abort; here it is clamped into the table. */
VX_API vx_status vx_get_rows(const vx_tensor * table, const vx_tensor * rows, const vx_tensor * dst, vx_stream stream);

/* ---- adjacent node pairs as one launch ----------------------------------------------------------
 * What a backend's graph_compute may substitute for two consecutive nodes whose intermediate has no
 * other reader; every rounding happens where the two separate nodes would round, so results are
 * bit-identical to running them one after the other.  No counterpart in ggml-cpu (it runs the nodes
 * separately: ops.cpp:3710-3777 + binary-ops.cpp:50-112, ops.cpp:4374-4424). */
/* RMS_NORM(src) -> MUL(., weight): weight one F32 row of src's ne[0] (MiniCPMModel::rms_norm, src/minicpm.cpp:572-580) */
VX_API vx_status vx_rms_norm_mul(const vx_tensor * src, const vx_tensor * weight, const vx_tensor * dst, float eps, vx_stream stream);
/* SCALE(x, scale) -> ADD(a, .): dst = a + x * scale (the muP residual, src/minicpm.cpp:765-775) */
VX_API vx_status vx_scale_add(const vx_tensor * a, const vx_tensor * x, const vx_tensor * dst, float scale, vx_stream stream);
/* ADD(a, b) -> SCALE(., scale, bias): dst = (a + b) * scale + bias (the kv_sync tail, src/minicpm.cpp:685-689) */
VX_API vx_status vx_add_scale(const vx_tensor * a, const vx_tensor * b, const vx_tensor * dst, float scale, float bias, vx_stream stream);
/* FLASH_ATTN_EXT(...) -> ADD1(., addend): the scalar the reference adds after attention to order its cache
 * write (src/minicpm.cpp:711-713); addend is a device F32 scalar, added after the normalisation */
VX_API vx_status vx_flash_attn_ext_add1(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                        const vx_tensor * mask, const float * sinks, const float * addend,
                                        const vx_tensor * dst, float scale, float max_bias, float logit_softcap,
                                        vx_stream stream);
/* CONCAT(k_past, k_cur, dim 1) , CONCAT(v_past, v_cur, dim 1) -> FLASH_ATTN_EXT: the reference appends the step's
 * keys and values to the cached ones before attention (attention_forward, src/minicpm.cpp:694-706).  Here the
 * kernel reads keys 0 .. ne1(k_past)-1 from k_past / v_past and the rest from k_cur / v_cur, so the
 * concatenated tensors are never written.  Both segments of one type -- or k_past / v_past F16 (an F16 cache) and
 * k_cur / v_cur F32 (the step's keys as the projections left them; head_dim 64): the kernel then rounds them to f16,
 * to nearest even, as it loads them, which is what a CPY node to an F16 tensor in front of the CONCAT stores --, same
 * head_dim, head and batch counts; mask over all keys.  Query counts the LDS-tiled prefill kernel would take are not supported (use CONCAT).
 * Result identical to vx_concat x2 + vx_flash_attn_ext. */
VX_API vx_status vx_flash_attn_ext_kv2(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                       const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                       const float * sinks, const vx_tensor * dst, float scale, float max_bias,
                                       float logit_softcap, vx_stream stream);
VX_API int vx_supports_flash_attn_ext_kv2(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                          const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                          const vx_tensor * dst);
/* The decode attention block of attention_forward (src/minicpm.cpp:682-713) as one call: vx_flash_attn_ext_kv2
 * followed by vx_kv_store_sync on its result, with the cache write and the ordering scalar folded into the kernel
 * that merges the key-range partials.  k_src / v_src are the CPY sources (the values of k_cur / v_cur in the shape
 * the reference copies them), k_slot / v_slot the cache views written; sync_scale / sync_bias the SCALE node's
 * parameters.  Needs more than 256 keys in all (the split path).  The slots may be F32 or F16; an F16 slot receives
 * the values rounded to nearest even and the ordering sums are taken over the rounded values (the slot read back as
 * F32).  Result and cache contents equal the two separate calls'. */
VX_API vx_status vx_flash_attn_ext_kv2_store(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                             const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                             const float * sinks, const vx_tensor * k_src, const vx_tensor * k_slot,
                                             const vx_tensor * v_src, const vx_tensor * v_slot, const vx_tensor * dst,
                                             float scale, float max_bias, float logit_softcap, float sync_scale,
                                             float sync_bias, vx_stream stream);
VX_API int vx_supports_flash_attn_ext_kv2_store(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                                const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                                const vx_tensor * k_src, const vx_tensor * k_slot, const vx_tensor * v_src,
                                                const vx_tensor * v_slot, const vx_tensor * dst);
/* The prefill attention block of attention_forward (src/minicpm.cpp:682-713) as one call: vx_flash_attn_ext over the
 * projections' own k / v, followed by vx_kv_store_sync on its result.  The cache write and the ordering scalar are
 * launched first and the scalar is added in the attention kernel's epilogue (as vx_flash_attn_ext_add1 adds one), so
 * the tokens x hidden result is stored once instead of stored, read and stored again.  For query counts the LDS-tiled
 * kernel takes (logit_softcap 0) and the two-launch cache writes vx_kv_store_sync takes (a prompt's or a prefill's); the
 * slots must not overlap anything the attention reads.  Result and cache contents equal the two separate calls'.
 * (vx_supports_flash_attn_ext_store says whether the call takes this form; shapes outside it run as the two calls.) */
VX_API vx_status vx_flash_attn_ext_store(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                         const float * sinks, const vx_tensor * k_src, const vx_tensor * k_slot,
                                         const vx_tensor * v_src, const vx_tensor * v_slot, const vx_tensor * dst,
                                         float scale, float max_bias, float logit_softcap, float sync_scale,
                                         float sync_bias, vx_stream stream);
VX_API int vx_supports_flash_attn_ext_store(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                            const vx_tensor * k_src, const vx_tensor * k_slot, const vx_tensor * v_src,
                                            const vx_tensor * v_slot, const vx_tensor * dst, float logit_softcap);
/* The same block with the output projection and the residual update behind it (attention_forward's o_proj product,
 * src/minicpm.cpp:714-715, and layer_forward's update, :762-768): vx_flash_attn_ext_store followed by
 * vx_mul_mat_scale_add(w_o, attn, residual) -> dst.  The attention kernel's epilogue rounds its result to f16 straight
 * into the activation tiles of the pre-tiled Q8_0 product, so the tokens x hidden attention output is neither stored in
 * fp32 nor read back and laid out again.  attn describes that output as the projection reads it ([hidden, tokens] with
 * the sequences one after the other, or [hidden, tokens, batch]; dense, the attention result's own memory order): its
 * memory is NOT written -- for callers whose only reader of it is the projection.  Where vx_flash_attn_ext_store applies
 * and the projection alone would run on the pre-tiled kernel (Q8_0, VX_ACT_FLOAT) -- what the supports function reports;
 * other shapes run as the separate calls, through attn's memory.  dst and the cache contents equal the separate calls'. */
VX_API vx_status vx_flash_attn_ext_store_proj(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                              const float * sinks, const vx_tensor * k_src, const vx_tensor * k_slot,
                                              const vx_tensor * v_src, const vx_tensor * v_slot, const vx_tensor * attn,
                                              const vx_tensor * w_o, const vx_tensor * residual, const vx_tensor * dst,
                                              float scale, float max_bias, float logit_softcap, float sync_scale,
                                              float sync_bias, float res_scale, int act_mode, vx_stream stream);
VX_API int vx_supports_flash_attn_ext_store_proj(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                                 const vx_tensor * k_src, const vx_tensor * k_slot, const vx_tensor * v_src,
                                                 const vx_tensor * v_slot, const vx_tensor * attn, const vx_tensor * w_o,
                                                 const vx_tensor * residual, const vx_tensor * dst, float logit_softcap,
                                                 int act_mode);
/* MUL_MAT(wq, x) RESHAPE ROPE , MUL_MAT(wk, x) RESHAPE ROPE , MUL_MAT(wv, x): the three projections of
 * attention_forward with apply_rope on Q and K (src/minicpm.cpp:669-680, 582-600) as one launch for few tokens
 * (as above).  x [K, tokens, 1, batch] or [K, tokens * batch] (sequence after sequence); q_dst / k_dst are the ROPE
 * outputs [head_dim, heads, tokens, batch], contiguous; v_dst the third product, shaped like x with rows for K (dense
 * rows, any row stride: it may be the v rows of one wider q/k/v product, the reference's fused qkv_proj layout, with
 * wq / wk / wv row ranges of that one matrix).  mode must be NEOX (2) with n_dims ==
 * head_dim; the remaining arguments are vx_rope's.  Results equal vx_mul_mat x3 + vx_rope x2 bit for bit. */
VX_API vx_status vx_qkv_proj_rope(const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x,
                                  const int32_t * pos, const float * freq_factors, const vx_tensor * q_dst,
                                  const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode, int n_ctx_orig,
                                  float freq_base, float freq_scale, float ext_factor, float attn_factor, float beta_fast,
                                  float beta_slow, int act_mode, vx_stream stream);
VX_API int vx_supports_qkv_proj_rope(const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x,
                                     const vx_tensor * q_dst, const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims,
                                     int mode);
/* K and V alone -- MUL_MAT(wk, x) RESHAPE ROPE , MUL_MAT(wv, x) (src/minicpm.cpp:671-680) -- as one launch of the same
 * kernel: for token counts where q's product is no longer one the streaming kernel runs (from 449 tokens at 1024 rows)
 * but those of k and v still are (up to 2048 tokens at 128 rows each).  Arguments and bits as in vx_qkv_proj_rope. */
VX_API vx_status vx_kv_proj_rope(const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x, const int32_t * pos,
                                 const float * freq_factors, const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims,
                                 int mode, int n_ctx_orig, float freq_base, float freq_scale, float ext_factor,
                                 float attn_factor, float beta_fast, float beta_slow, int act_mode, vx_stream stream);
VX_API int vx_supports_kv_proj_rope(const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x, const vx_tensor * k_dst,
                                    const vx_tensor * v_dst, int n_dims, int mode);
/* RMS_NORM(x) , MUL(., norm_w) in front of vx_qkv_proj_rope / vx_mul_mat_swiglu: MiniCPMModel::rms_norm
 * (src/minicpm.cpp:572-580) as layer_forward applies it before attention and before the MLP (:761, :770), joined to
 * the projections' launch.  x is the un-normalised hidden state, rows of at most 1024 floats, 16-byte aligned;
 * norm_w one F32 row.  The normalised tensor is not stored.  Results equal vx_rms_norm_mul followed by the
 * projection call, bit for bit. */
VX_API vx_status vx_norm_qkv_proj_rope(const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * wq,
                                       const vx_tensor * wk, const vx_tensor * wv, const int32_t * pos,
                                       const float * freq_factors, const vx_tensor * q_dst, const vx_tensor * k_dst,
                                       const vx_tensor * v_dst, int n_dims, int mode, int n_ctx_orig, float freq_base,
                                       float freq_scale, float ext_factor, float attn_factor, float beta_fast,
                                       float beta_slow, int act_mode, vx_stream stream);
VX_API int vx_supports_norm_qkv_proj_rope(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * wq,
                                          const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * q_dst,
                                          const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode);
/* the same call at prefill sizes (Q8_0 weights, VX_ACT_FLOAT, every product one that a tiled kernel runs with its K
 * whole): the norm in the pre-tiled kernel's activation pass, q, k and v as one product launch over those tiles, the two
 * rotations in that product's epilogue (heads of 64 rows: the angles come from a table filled in front of the product by
 * vx_rope's own arithmetic; VX_QKV_ROPE_EPILOGUE=0 or other head sizes: launches of their own, in place).  Same bits as
 * RMS_NORM, MUL, three MUL_MATs, two ROPEs. */
VX_API int vx_supports_norm_qkv_proj_rope_tiled(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * wq,
                                                const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * q_dst,
                                                const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode, int act_mode);
VX_API vx_status vx_norm_mul_mat_swiglu(const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * gate,
                                        const vx_tensor * up, const vx_tensor * dst, int act_mode, vx_stream stream);
VX_API int vx_supports_norm_mul_mat_swiglu(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate,
                                           const vx_tensor * up, const vx_tensor * dst);
/* the same call at prefill sizes (vx_supports_mul_mat_swiglu_tiled's shapes on the pre-tiled Q8_0 kernel, 1024 tokens or
 * more): the norm and its weight are applied by the pass that lays the activations out in tiles, x is read once and the
 * normalised tensor is never stored.  Same bits as RMS_NORM, MUL, then vx_mul_mat_swiglu. */
VX_API int vx_supports_norm_mul_mat_swiglu_tiled(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate,
                                                 const vx_tensor * up, const vx_tensor * dst, int act_mode);
/* mlp_forward and the residual update behind it at prefill sizes (src/minicpm.cpp:718-747, 775-786):
 *   dst = residual + scale * (down . (silu(gate . n) * (up . n))),  n = RMS_NORM(x) * norm_w
 * for the node chain RMS_NORM, MUL, MUL_MAT, MUL_MAT, GLU(SWIGLU), MUL_MAT, SCALE, ADD.  The pair's results go to the down
 * projection as f16 tiles; the [tokens x ffn] tensor between them is not stored.  Same bits as the separate calls
 * (vx_norm_mul_mat_swiglu, vx_mul_mat_scale_add).  Q8_0 weights, VX_ACT_FLOAT, shapes that the pre-tiled kernel takes. */
VX_API int vx_supports_mlp_tiled(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate, const vx_tensor * up,
                                 const vx_tensor * down, const vx_tensor * residual, const vx_tensor * dst, int act_mode);
VX_API vx_status vx_mlp_tiled(const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * gate,
                              const vx_tensor * up, const vx_tensor * down, const vx_tensor * residual, float scale,
                              const vx_tensor * dst, int act_mode, vx_stream stream);
/* MUL_MAT(gate, x), MUL_MAT(up, x) -> GLU(SWIGLU split): dst = silu(gate x) * (up x) for few tokens (16, or more while tokens x rows <= 256 Ki)
 * (MiniCPMModel::mlp_forward, src/minicpm.cpp:718-747); gate and up Q8_0 or F16 of one shape and layout */
VX_API vx_status vx_mul_mat_swiglu(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst,
                                   int act_mode, vx_stream stream);
VX_API int vx_supports_mul_mat_swiglu(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst);
/* The same group at prefill sizes (64 tokens or more, f16 activations): both products on the LDS-tiled kernel, whose
 * work-groups hold a tile of gate rows and the same rows of up and apply the GLU as they store -- the two F32 products
 * (tokens x 2 x rows x 4 bytes written and read again) never reach memory.  vx_mul_mat_swiglu takes these shapes too;
 * this predicate needs the activation mode because under VX_ACT_Q8 the tiled products run on kernels without that epilogue. */
VX_API int vx_supports_mul_mat_swiglu_tiled(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst,
                                            int act_mode);
/* MUL_MAT(w, x) -> SCALE(., scale) -> ADD(residual, .): dst = residual + scale * (w x) for few tokens (as above),
 * and for 64 or more tokens over a long K (>= 2048, a multiple of 128) when the product is fewer than 64 tiles of
 * 64 x 64 (the down-projection of a hundred tokens): there the K range is cut across work-groups and the kernel that
 * adds the partials applies the update.  At prefill sizes (more than 16 tokens, rows a multiple of 4, dst dense and 16-byte
 * aligned) the LDS-tiled kernels apply the update as they store their tile, which saves the pass over dst that the ADD node
 * is; where no such kernel takes the shape or the activation mode, the plain product is followed by that pass (through the
 * per-stream workspace when the residual is dst itself).  The residual updates of MiniCPMModel::layer_forward
 * (src/minicpm.cpp:762-777); w Q8_0 or F16, residual F32 of dst's shape (or a bias row).  Bit-equal to the three nodes. */
VX_API vx_status vx_mul_mat_scale_add(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * residual,
                                      const vx_tensor * dst, float scale, int act_mode, vx_stream stream);
VX_API int vx_supports_mul_mat_scale_add(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * residual,
                                         const vx_tensor * dst);
/* The reference's KV append with its write-ordering scalar (attention_forward, src/minicpm.cpp:682-713), nine graph
 * nodes as one launch:  CPY(k, k_slot) CONT SUM , CPY(v, v_slot) CONT SUM , ADD , SCALE(scale, bias) , ADD1(x, .)
 *   k_slot <- k ; v_slot <- v ; dst = x + ((sum(k_slot) + sum(v_slot)) * scale + bias)
 * k, v, x F32; a cache write of at most 16384 elements (decode-sized: one launch, two when x has more than 16384
 * elements), a prompt's -- both sums within vx_sum's one block of 1024 threads (16 Ki sum units: 4 elements of a
 * 16-byte aligned row, else one), every wave of that block a work-group of its own here -- or a prefill's -- both of
 * more than 16 Ki units, i.e. sums that vx_sum spreads over its 128 blocks --, the latter two as two launches (stores
 * and wave or block totals; totals, scalar and ADD1) in place of eight to eleven; k_slot / v_slot with dense rows, F32
 * or F16.  With F16 slots the node sequence is CPY(k, k_slot) CPY(k_slot -> F32) SUM ...: the values are
 * rounded to nearest even on the way in and the sums see the rounded values.  The sums are formed in vx_sum's order,
 * so dst equals what the separate nodes give. */
VX_API vx_status vx_kv_store_sync(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot,
                                  const vx_tensor * x, const vx_tensor * dst, float scale, float bias, vx_stream stream);
VX_API int vx_supports_kv_store_sync(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot,
                                     const vx_tensor * x, const vx_tensor * dst);
VX_API int vx_supports_rms_norm_mul(const vx_tensor * src, const vx_tensor * weight, const vx_tensor * dst);
VX_API int vx_supports_fused_pair(const vx_tensor * a, const vx_tensor * b, const vx_tensor * dst);

VX_API int vx_supports_binary(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst);
VX_API int vx_supports_add1(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst);
VX_API int vx_supports_unary_like(const vx_tensor * src, const vx_tensor * dst); /* SCALE */
VX_API int vx_supports_unary(int op, const vx_tensor * src, const vx_tensor * dst);
VX_API int vx_supports_glu(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst);
VX_API int vx_supports_cpy(const vx_tensor * src, const vx_tensor * dst);
VX_API int vx_supports_arange(const vx_tensor * dst);
/* The order in which vx_mul_mat and the groups built on it sum the K blocks of a product with few tokens, as an opaque
 * number: products with equal K, equal token count of the call and equal number are summed identically.  The number depends
 * on the row count M, so a backend that replaces one product over a row-fused matrix (the reference's qkv_proj /
 * gate_up_proj, src/minicpm.cpp:427-492) by products over its row ranges compares the two before it promises the same bits.
 * No counterpart in the reference. */
VX_API int vx_mul_mat_sum_order(int64_t K, int64_t tokens, int64_t M);

/* ---- a run of tiny nodes as one launch -------------------------------------------------------------
 * Around the decoder stacks the reference's graphs hold chains of operators over a few hundred values: bias adds,
 * the CONCATs that assemble LocDiT's CFG-pair sequence (src/locdit.cpp:401-464), the guidance arithmetic and the Euler
 * update of UnifiedCFM (src/unified_cfm.cpp:30-149).  vx_small_graph runs up to 16 such nodes, in the order given, in ONE
 * launch (one work-group, a barrier between nodes); every node writes its own dst as its separate call would, with the
 * same arithmetic and the same summation order, so the results are those of the separate calls.  Each tensor of a node
 * holds at most 16384 elements.  No counterpart in ggml-cpu, which runs the nodes one by one. */
enum { VX_NODE_ADD = 0, VX_NODE_SUB = 1, VX_NODE_MUL = 2, VX_NODE_DIV = 3,  /* vx_binary                        */
       VX_NODE_ADD1 = 4,                                                    /* vx_add1                          */
       VX_NODE_SCALE = 5,                                                   /* vx_scale: p0 = scale, p1 = bias  */
       VX_NODE_UNARY = 6,                                                   /* vx_unary: aux = VX_UNARY_*       */
       VX_NODE_CPY = 7,                                                     /* vx_cpy (CPY / CONT / DUP)        */
       VX_NODE_CONCAT = 8,                                                  /* vx_concat: aux = dim             */
       VX_NODE_REPEAT = 9,                                                  /* vx_repeat                        */
       VX_NODE_SUM = 10,                                                    /* vx_sum                           */
       VX_NODE_ARANGE = 11,                                                 /* vx_arange: p0 = start, p1 = step */
       VX_NODE_SUM_ROWS = 12 };                                             /* vx_sum_rows                      */
/* flags: VX_SMALL_DST_PRIVATE -- the caller knows that nothing but later nodes of the same run reads dst (the plugin: every
 * reader of the graph node is a member of the run and the node is no graph output).  Such a destination is then carried in
 * LDS only, when there is room for it, and its memory is left untouched; without room it is written like any other. */
#define VX_SMALL_DST_PRIVATE 1
typedef struct vx_small_node {
    int32_t op, aux;
    float   p0, p1;
    const vx_tensor * src0, * src1, * dst;   /* src1 NULL where the operator has one operand, src0 NULL for ARANGE */
    int32_t flags, reserved;
} vx_small_node;
VX_API vx_status vx_small_graph(const vx_small_node * nodes, int n_nodes, vx_stream stream);
VX_API int vx_supports_small_node(const vx_small_node * node);
VX_API int vx_supports_repeat(const vx_tensor * src, const vx_tensor * dst);
VX_API int vx_supports_get_rows(const vx_tensor * table, const vx_tensor * rows, const vx_tensor * dst);
VX_API int vx_supports_concat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int dim);
VX_API int vx_supports_sum(const vx_tensor * src, const vx_tensor * dst);

#ifdef __cplusplus
}
#endif
#endif
