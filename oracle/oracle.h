/*
 * oracle.h -- CPU restatement of the ggml-cpu algorithms on VoxCPM.cpp's attention
 * hot path.  TEST INFRASTRUCTURE ONLY: this library is the checker the parity tests,
 * the smoke test and the benchmark's cpu_baseline leg compare against.  Nothing the
 * product ships links, loads or calls it, and the product has no CPU fallback.
 *
 * Every function follows one piece of the reference (paths relative to the
 * reference checkout; ggml/ = third_party/ggml/) and says which.  How each one is
 * pinned (against the reference's own ggml-cpu built into oracle/_ref, closed forms,
 * brute force, invariants) is listed beside it; tests/test_oracle.py runs the pins.
 *
 * Tensors use ggml's conventions: ne[0] is the fastest dimension, nb[] are strides in
 * bytes, a Q8_0 row is ne[0]/32 blocks of {f16 d; int8 qs[32]} (34 bytes).
 */
#ifndef VOXCPM_ORACLE_H
#define VOXCPM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* same numbering as enum ggml_type (ggml/include/ggml.h:389-431) */
enum { ORC_F32 = 0, ORC_F16 = 1, ORC_Q8_0 = 8, ORC_I32 = 26 };

typedef struct orc_tensor {
    int32_t  type;
    int32_t  _pad;
    int64_t  ne[4];
    uint64_t nb[4];
    void *   data;
} orc_tensor;

/* ---- scalar conversions: IEEE binary16 <-> binary32, round-to-nearest-even
 * (what F16C does; GGML_CPU_FP32_TO_FP16, ggml/src/ggml-cpu/simd-mappings.h).
 * Pinned: all 65536 halves and random floats against numpy.float16. */
uint16_t orc_fp32_to_fp16(float f);
float    orc_fp16_to_fp32(uint16_t h);
void     orc_fp32_to_fp16_row(const float * x, uint16_t * y, int64_t n);
void     orc_fp16_to_fp32_row(const uint16_t * x, float * y, int64_t n);

/* ---- Q8_0: block {f16 d; int8 qs[32]} (ggml/src/ggml-common.h:219-224) */
/* weight quantizer, ggml/src/ggml-quants.c:199-222 (id = 1/d, roundf).
 * Pinned: bit-exact vs ggml_quantize_chunk in oracle/_ref; round-trip RMSE bound of
 * ggml/tests/test-quantize-fns.cpp:17-18. */
void orc_quantize_row_q8_0_ref(const float * x, void * y, int64_t k);
/* activation quantizer of the x86 build, ggml/src/ggml-cpu/arch/x86/quants.c:290-386
 * (id = 127/max, round-to-nearest-even).  Pinned: bit-exact vs ggml-cpu MUL_MAT's
 * intermediate through the Q8_0 dot below; brute force on ties. */
void orc_quantize_row_q8_0_x86(const float * x, void * y, int64_t k);
/* ggml/src/ggml-quants.c:401-415.  Pinned: bit-exact vs ggml's to_float in oracle/_ref. */
void orc_dequantize_row_q8_0(const void * x, float * y, int64_t k);
/* ggml/src/ggml-cpu/quants.c:305-333 (generic) -- integer sub-dot exact, blocks summed
 * in order in fp32. */
float orc_vec_dot_q8_0_q8_0(int64_t n, const void * x, const void * y);
/* ggml/src/ggml-cpu/arch/x86/quants.c:1012-1078 (AVX2 order: 8 fp32 lane accumulators
 * each fed by 4 products per block, fused multiply-add, then the hsum_float_8 tree). */
float orc_vec_dot_q8_0_q8_0_avx2(int64_t n, const void * x, const void * y);

/* ---- GGML_OP_MUL_MAT: dst[ne01, ne11, ne12, ne13] = src0[ne00, ne01, ne02, ne03]^T x
 * src1[ne10, ne11, ne12, ne13] with broadcast over dims 2,3
 * (ggml/src/ggml-cpu/ggml-cpu.c:1139-1421).  src0 Q8_0 | F16 | F32, src1 F32, dst F32
 * contiguous.  act_mode: 0 = what ggml-cpu does (src1 converted to src0's vec_dot_type:
 * Q8_0 blocks by the x86 quantizer / F16 / F32), 1 = src1 kept in fp32 and src0
 * dequantized (the "dequantize then multiply" form), both accumulated in fp32 in order.
 * Returns 0 on success. */
int orc_mul_mat(const orc_tensor * src0, const orc_tensor * src1, orc_tensor * dst, int act_mode);
/* fp64 dequantize-then-multiply reference of the same op. */
int orc_mul_mat_f64(const orc_tensor * src0, const orc_tensor * src1, orc_tensor * dst);

/* ---- GGML_OP_RMS_NORM (ggml/src/ggml-cpu/ops.cpp:3710-3759): fp64 sum of fp32 squares. */
int orc_rms_norm(const orc_tensor * src, orc_tensor * dst, float eps);

/* ---- GGML_OP_ROPE, modes NORMAL(0) and NEOX(2) (ggml/src/ggml-cpu/ops.cpp:5589-5860,
 * corr dims ggml/src/ggml.c:4280-4294).  pos: int32[ne2]; freq_factors may be NULL. */
int orc_rope(const orc_tensor * src, const int32_t * pos, const float * freq_factors,
             orc_tensor * dst, int n_dims, int mode, int n_ctx_orig, float freq_base,
             float freq_scale, float ext_factor, float attn_factor, float beta_fast,
             float beta_slow);

/* ---- GGML_OP_SOFT_MAX (ggml/src/ggml-cpu/ops.cpp:5225-5335); mask F16|F32|NULL,
 * sinks float[ne02] or NULL. */
int orc_soft_max(const orc_tensor * src, const orc_tensor * mask, const float * sinks,
                 orc_tensor * dst, float scale, float max_bias);

/* ---- GGML_OP_FLASH_ATTN_EXT (ggml/src/ggml-cpu/ops.cpp:8109-8853).
 * q [DK,n_q,Hq,ne3] F32; k [DK,n_kv,Hkv,*] F32|F16; v [DV,n_kv,Hkv,*]; mask
 * [n_kv,>=n_q,ne32,ne33] F16 or NULL; sinks float[Hq] or NULL; dst [DV,Hq,n_q,ne3] F32.
 * path: ORC_FA_AUTO picks what ggml-cpu's dispatcher picks for nth threads
 * (ops.cpp:8752-8835); the others force one. */
enum { ORC_FA_AUTO = 0, ORC_FA_VEC = 1, ORC_FA_TILED = 2, ORC_FA_SPLIT_KV = 3 };
int orc_flash_attn_ext(const orc_tensor * q, const orc_tensor * k, const orc_tensor * v,
                       const orc_tensor * mask, const float * sinks, orc_tensor * dst,
                       float scale, float max_bias, float logit_softcap, int path, int nth);
/* textbook softmax(scale*QK^T + mask)V in fp64 with the same tensor conventions. */
int orc_flash_attn_ext_f64(const orc_tensor * q, const orc_tensor * k, const orc_tensor * v,
                           const orc_tensor * mask, const float * sinks, orc_tensor * dst,
                           float scale, float max_bias, float logit_softcap);

/* ---- MiniCPMKVCache views (src/minicpm.cpp:200-236): cache tensor is
 * [head_dim, max_length, n_kv_heads] with element size es.  Each call fills ne[3], nb[3]
 * and the byte offset of the view.  Pinned by tests/test_minicpm.cpp:775-809. */
void orc_kv_read_view(int head_dim, int max_length, int n_kv_heads, int es, int seq_len,
                      int64_t ne[3], uint64_t nb[3], uint64_t * offset);
void orc_kv_write_view(int head_dim, int max_length, int n_kv_heads, int es, int start,
                       int n_tokens, int64_t ne[3], uint64_t nb[3], uint64_t * offset);

/* ---- create_causal_mask (src/minicpm.cpp:602-620): F16 [total_len, n_q], 0x8000 (-0.0)
 * where key <= query position, 0xFC00 (-inf) elsewhere. */
void orc_causal_mask(const int32_t * positions, int n_q, int total_len, uint16_t * mask);

/* ---- LocDiT CFG pair constants (src/locdit.cpp:63-130): positions i % branch_len and a
 * [2L,2L] F16 block-diagonal mask (0 on the two diagonal blocks, -inf elsewhere). */
void orc_cfg_pair_constants(int branch_len, int32_t * positions, uint16_t * mask);

/* ---- UnifiedCFM::compute_t_span (src/unified_cfm.cpp:18-41), pinned by the closed form
 * in tests/test_unified_cfm.cpp:155-164.  out has n_timesteps+1 entries. */
void orc_t_span(int n_timesteps, float sway_coef, float * out);

#ifdef __cplusplus
}
#endif
#endif
