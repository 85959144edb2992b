/*
 * oracle.c -- CPU restatement of ggml-cpu's algorithms for VoxCPM.cpp's attention hot
 * path.  TEST INFRASTRUCTURE ONLY (see oracle.h): it is the checker, never the product.
 *
 * Built with -ffp-contract=off so that every fused multiply-add in this file is an
 * explicit fmaf() placed where the reference's x86 build fuses, and nothing else fuses.
 *
 * Order of floating point sums: ggml-cpu's dot products run in SIMD lanes whose count
 * depends on the ISA of the build, so a restatement can match them to rounding only
 * (about 1e-6 relative), never bit for bit; the places where the order *is* fixed by the
 * source (the tiled GEMM micro-kernel, the Q8_0 AVX2 dot, every element-wise step) are
 * restated in that exact order.
 */
#include "oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define QK8_0 32
typedef struct { uint16_t d; int8_t qs[QK8_0]; } block_q8_0; /* ggml/src/ggml-common.h:219-224 */

#define MAXF(a, b) ((a) > (b) ? (a) : (b))
#define MINF(a, b) ((a) < (b) ? (a) : (b))

/* ------------------------------------------------------------------ fp16 <-> fp32 */

uint16_t orc_fp32_to_fp16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    const uint32_t sign = (x >> 16) & 0x8000u;
    const uint32_t absx = x & 0x7FFFFFFFu;
    if (absx > 0x7F800000u) { /* NaN: keep it quiet, keep top mantissa bits */
        return (uint16_t)(sign | 0x7E00u | ((absx >> 13) & 0x03FFu));
    }
    if (absx >= 0x477FF000u) { /* rounds to >= 65520 -> inf (also inf itself) */
        return (uint16_t)(sign | 0x7C00u);
    }
    if (absx < 0x33000001u) { /* <= 2^-25: rounds to zero (tie at 2^-25 goes to even = 0) */
        return (uint16_t)sign;
    }
    const int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t mant = (absx & 0x007FFFFFu) | 0x00800000u; /* 24-bit significand */
    uint32_t shift;
    uint32_t half_exp;
    if (e < -14) { /* subnormal half: value = mant * 2^(e-23), unit 2^-24 */
        shift = (uint32_t)(13 + (-14 - e));
        half_exp = 0;
    } else {
        shift = 13;
        half_exp = (uint32_t)(e + 15);
    }
    const uint32_t q = mant >> shift;
    const uint32_t rem = mant & ((1u << shift) - 1u);
    const uint32_t halfway = 1u << (shift - 1);
    uint32_t r = q;
    if (rem > halfway || (rem == halfway && (q & 1u))) {
        r += 1;
    }
    uint32_t out;
    if (half_exp == 0) {
        out = r; /* may carry into exponent 1: that is the right encoding */
    } else {
        out = ((half_exp - 1) << 10) + r; /* r carries the implicit bit (0x400..0x800) */
    }
    return (uint16_t)(sign | out);
}

float orc_fp16_to_fp32(uint16_t h) {
    const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    const uint32_t man = h & 0x3FFu;
    uint32_t x;
    if (exp == 0) {
        if (man == 0) {
            x = sign;
        } else { /* subnormal: man * 2^-24, exact in fp32 */
            float f = (float)man * 5.9604644775390625e-08f;
            memcpy(&x, &f, 4);
            x |= sign;
        }
    } else if (exp == 31) {
        x = sign | 0x7F800000u | (man << 13);
    } else {
        x = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &x, 4);
    return f;
}

void orc_fp32_to_fp16_row(const float * x, uint16_t * y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = orc_fp32_to_fp16(x[i]);
}
void orc_fp16_to_fp32_row(const uint16_t * x, float * y, int64_t n) {
    for (int64_t i = 0; i < n; ++i) y[i] = orc_fp16_to_fp32(x[i]);
}

/* ------------------------------------------------------------------------- Q8_0 */

void orc_quantize_row_q8_0_ref(const float * x, void * vy, int64_t k) {
    block_q8_0 * y = (block_q8_0 *)vy;
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; ++i) {
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; ++j) amax = MAXF(amax, fabsf(x[i * QK8_0 + j]));
        const float d = amax / 127;
        const float id = d ? 1.0f / d : 0.0f;
        y[i].d = orc_fp32_to_fp16(d);
        for (int j = 0; j < QK8_0; ++j) y[i].qs[j] = (int8_t)roundf(x[i * QK8_0 + j] * id);
    }
}

void orc_quantize_row_q8_0_x86(const float * x, void * vy, int64_t k) {
    block_q8_0 * y = (block_q8_0 *)vy;
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; ++i) {
        float amax = 0.0f;
        for (int j = 0; j < QK8_0; ++j) amax = MAXF(amax, fabsf(x[i * QK8_0 + j]));
        const float d = amax / 127.f;
        y[i].d = orc_fp32_to_fp16(d);
        const float id = (amax != 0.0f) ? 127.f / amax : 0.0f;
        for (int j = 0; j < QK8_0; ++j) {
            /* _mm256_round_ps(NEAREST) then cvtps_epi32: ties to even; the int32 -> int16
             * -> int8 packs saturate, which cannot trigger since |x*id| <= 127 + 1 ulp */
            float r = nearbyintf(x[i * QK8_0 + j] * id);
            if (r > 127.f) r = 127.f;
            if (r < -128.f) r = -128.f;
            y[i].qs[j] = (int8_t)r;
        }
    }
}

void orc_dequantize_row_q8_0(const void * vx, float * y, int64_t k) {
    const block_q8_0 * x = (const block_q8_0 *)vx;
    const int64_t nb = k / QK8_0;
    for (int64_t i = 0; i < nb; ++i) {
        const float d = orc_fp16_to_fp32(x[i].d);
        for (int j = 0; j < QK8_0; ++j) y[i * QK8_0 + j] = x[i].qs[j] * d;
    }
}

float orc_vec_dot_q8_0_q8_0(int64_t n, const void * vx, const void * vy) {
    const block_q8_0 * x = (const block_q8_0 *)vx;
    const block_q8_0 * y = (const block_q8_0 *)vy;
    const int64_t nb = n / QK8_0;
    float sumf = 0;
    for (int64_t ib = 0; ib < nb; ++ib) {
        int sumi = 0;
        for (int j = 0; j < QK8_0; ++j) sumi += x[ib].qs[j] * y[ib].qs[j];
        sumf += sumi * (orc_fp16_to_fp32(x[ib].d) * orc_fp16_to_fp32(y[ib].d));
    }
    return sumf;
}

float orc_vec_dot_q8_0_q8_0_avx2(int64_t n, const void * vx, const void * vy) {
    const block_q8_0 * x = (const block_q8_0 *)vx;
    const block_q8_0 * y = (const block_q8_0 *)vy;
    const int64_t nb = n / QK8_0;
    float acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int64_t ib = 0; ib < nb; ++ib) {
        const float d = orc_fp16_to_fp32(x[ib].d) * orc_fp16_to_fp32(y[ib].d);
        for (int l = 0; l < 8; ++l) {
            /* mul_sum_i8_pairs_float: lane l = sum of bytes 4l..4l+3 (exact int) -> float */
            int s = 0;
            for (int j = 0; j < 4; ++j) s += x[ib].qs[4 * l + j] * y[ib].qs[4 * l + j];
            acc[l] = fmaf(d, (float)s, acc[l]);
        }
    }
    /* hsum_float_8: (lo128 + hi128), then movehl add, then movehdup add */
    float r[4];
    for (int l = 0; l < 4; ++l) r[l] = acc[l] + acc[l + 4];
    const float a0 = r[0] + r[2];
    const float a1 = r[1] + r[3];
    return a0 + a1;
}

/* ---------------------------------------------------------------------- helpers */

static inline const char * tptr(const orc_tensor * t, int64_t i1, int64_t i2, int64_t i3) {
    return (const char *)t->data + i1 * t->nb[1] + i2 * t->nb[2] + i3 * t->nb[3];
}

static int is_contiguous_f32(const orc_tensor * t) {
    return t->type == ORC_F32 && t->nb[0] == 4 && t->nb[1] == (uint64_t)t->ne[0] * 4 &&
           t->nb[2] == t->nb[1] * (uint64_t)t->ne[1] && t->nb[3] == t->nb[2] * (uint64_t)t->ne[2];
}

/* ---------------------------------------------------------------------- MUL_MAT */

int orc_mul_mat(const orc_tensor * src0, const orc_tensor * src1, orc_tensor * dst, int act_mode) {
    const int64_t ne00 = src0->ne[0], ne01 = src0->ne[1], ne02 = src0->ne[2], ne03 = src0->ne[3];
    const int64_t ne10 = src1->ne[0], ne11 = src1->ne[1], ne12 = src1->ne[2], ne13 = src1->ne[3];
    if (ne00 != ne10 || src1->type != ORC_F32 || dst->type != ORC_F32) return 1;
    if (dst->ne[0] != ne01 || dst->ne[1] != ne11 || dst->ne[2] != ne12 || dst->ne[3] != ne13) return 2;
    if (ne12 % ne02 || ne13 % ne03) return 3;
    if (src1->nb[0] != 4 || dst->nb[0] != 4) return 4;
    if (src0->type == ORC_Q8_0 && ne00 % QK8_0) return 5;
    const int64_t r2 = ne12 / ne02, r3 = ne13 / ne03;

    float * wrow = (float *)malloc((size_t)ne00 * sizeof(float));           /* src0 row in fp32 */
    block_q8_0 * xq = (block_q8_0 *)malloc((size_t)(ne00 / QK8_0 + 1) * sizeof(block_q8_0));
    uint16_t * xh = (uint16_t *)malloc((size_t)ne00 * sizeof(uint16_t));
    if (!wrow || !xq || !xh) { free(wrow); free(xq); free(xh); return 6; }

    for (int64_t i13 = 0; i13 < ne13; ++i13)
    for (int64_t i12 = 0; i12 < ne12; ++i12)
    for (int64_t i11 = 0; i11 < ne11; ++i11) {
        const float * x = (const float *)tptr(src1, i11, i12, i13);
        float * out = (float *)((char *)dst->data + i11 * dst->nb[1] + i12 * dst->nb[2] + i13 * dst->nb[3]);
        const int64_t i02 = i12 / r2, i03 = i13 / r3;
        if (act_mode == 0) {
            /* ggml-cpu.c:1291-1325: src1 row converted to vec_dot_type of src0 */
            if (src0->type == ORC_Q8_0) orc_quantize_row_q8_0_x86(x, xq, ne00);
            else if (src0->type == ORC_F16) orc_fp32_to_fp16_row(x, xh, ne00);
        }
        for (int64_t i01 = 0; i01 < ne01; ++i01) {
            const char * w = tptr(src0, i01, i02, i03);
            float acc = 0.0f;
            if (act_mode == 0 && src0->type == ORC_Q8_0) {
                acc = orc_vec_dot_q8_0_q8_0_avx2(ne00, w, xq);
            } else if (act_mode == 0 && src0->type == ORC_F16) {
                const uint16_t * wh = (const uint16_t *)w;
                for (int64_t i = 0; i < ne00; ++i)
                    acc = fmaf(orc_fp16_to_fp32(wh[i]), orc_fp16_to_fp32(xh[i]), acc);
            } else {
                if (src0->type == ORC_Q8_0) orc_dequantize_row_q8_0(w, wrow, ne00);
                else if (src0->type == ORC_F16) orc_fp16_to_fp32_row((const uint16_t *)w, wrow, ne00);
                else memcpy(wrow, w, (size_t)ne00 * 4);
                for (int64_t i = 0; i < ne00; ++i) acc = fmaf(wrow[i], x[i], acc);
            }
            out[i01] = acc;
        }
    }
    free(wrow); free(xq); free(xh);
    return 0;
}

int orc_mul_mat_f64(const orc_tensor * src0, const orc_tensor * src1, orc_tensor * dst) {
    const int64_t ne00 = src0->ne[0], ne01 = src0->ne[1], ne02 = src0->ne[2], ne03 = src0->ne[3];
    const int64_t ne11 = src1->ne[1], ne12 = src1->ne[2], ne13 = src1->ne[3];
    if (ne00 != src1->ne[0] || src1->type != ORC_F32 || dst->type != ORC_F32) return 1;
    if (ne12 % ne02 || ne13 % ne03) return 3;
    const int64_t r2 = ne12 / ne02, r3 = ne13 / ne03;
    float * wrow = (float *)malloc((size_t)ne00 * sizeof(float));
    if (!wrow) return 6;
    for (int64_t i13 = 0; i13 < ne13; ++i13)
    for (int64_t i12 = 0; i12 < ne12; ++i12)
    for (int64_t i01 = 0; i01 < ne01; ++i01) {
        const char * w = tptr(src0, i01, i12 / r2, i13 / r3);
        if (src0->type == ORC_Q8_0) orc_dequantize_row_q8_0(w, wrow, ne00);
        else if (src0->type == ORC_F16) orc_fp16_to_fp32_row((const uint16_t *)w, wrow, ne00);
        else memcpy(wrow, w, (size_t)ne00 * 4);
        for (int64_t i11 = 0; i11 < ne11; ++i11) {
            const float * x = (const float *)tptr(src1, i11, i12, i13);
            double acc = 0.0;
            for (int64_t i = 0; i < ne00; ++i) acc += (double)wrow[i] * (double)x[i];
            float * out = (float *)((char *)dst->data + i11 * dst->nb[1] + i12 * dst->nb[2] + i13 * dst->nb[3]);
            out[i01] = (float)acc;
        }
    }
    free(wrow);
    return 0;
}

/* --------------------------------------------------------------------- RMS_NORM */

int orc_rms_norm(const orc_tensor * src, orc_tensor * dst, float eps) {
    if (src->type != ORC_F32 || dst->type != ORC_F32 || src->nb[0] != 4 || dst->nb[0] != 4) return 1;
    if (eps < 0.0f) return 2;
    const int64_t ne00 = src->ne[0];
    for (int64_t i3 = 0; i3 < src->ne[3]; ++i3)
    for (int64_t i2 = 0; i2 < src->ne[2]; ++i2)
    for (int64_t i1 = 0; i1 < src->ne[1]; ++i1) {
        const float * x = (const float *)tptr(src, i1, i2, i3);
        float * y = (float *)((char *)dst->data + i1 * dst->nb[1] + i2 * dst->nb[2] + i3 * dst->nb[3]);
        double sum = 0.0;
        for (int64_t i = 0; i < ne00; ++i) sum += (double)(x[i] * x[i]); /* fp32 square, fp64 add */
        const float mean = (float)(sum / ne00);
        const float scale = 1.0f / sqrtf(mean + eps);
        for (int64_t i = 0; i < ne00; ++i) y[i] = x[i] * scale;
    }
    return 0;
}

/* ------------------------------------------------------------------------- ROPE */

static float yarn_corr_dim(int n_dims, int n_ctx_orig, float n_rot, float base) {
    return n_dims * logf(n_ctx_orig / (n_rot * 2 * (float)M_PI)) / (2 * logf(base));
}

static float yarn_ramp(const float low, const float high, const int i0) {
    const float y = (i0 / 2 - low) / MAXF(0.001f, high - low);
    return 1 - MINF(1, MAXF(0, y));
}

int orc_rope(const orc_tensor * src, const int32_t * pos, const float * freq_factors,
             orc_tensor * dst, int n_dims, int mode, int n_ctx_orig, float freq_base,
             float freq_scale, float ext_factor, float attn_factor, float beta_fast,
             float beta_slow) {
    if (src->type != ORC_F32 || dst->type != ORC_F32 || src->nb[0] != 4 || dst->nb[0] != 4) return 1;
    if (mode != 0 && mode != 2) return 2;
    const int64_t ne0 = src->ne[0];
    if (n_dims > ne0 || n_dims % 2) return 3;

    const float theta_scale = powf(freq_base, -2.0f / n_dims);
    float corr_dims[2];
    {
        const float start = floorf(yarn_corr_dim(n_dims, n_ctx_orig, beta_fast, freq_base));
        const float end = ceilf(yarn_corr_dim(n_dims, n_ctx_orig, beta_slow, freq_base));
        corr_dims[0] = MAXF(0, start);
        corr_dims[1] = MINF(n_dims - 1, end);
    }
    float * cache = (float *)malloc((size_t)ne0 * sizeof(float));
    if (!cache) return 6;

    for (int64_t i3 = 0; i3 < src->ne[3]; ++i3)
    for (int64_t i2 = 0; i2 < src->ne[2]; ++i2) {
        /* ggml_rope_cache_init: theta starts at the position (int -> float) and is
         * multiplied by theta_scale once per pair, in fp32 */
        float theta = (float)(int64_t)pos[i2];
        for (int64_t i0 = 0; i0 < ne0; i0 += 2) {
            const float ff = freq_factors ? freq_factors[i0 / 2] : 1.0f;
            const float theta_extrap = theta / ff;
            const float theta_interp = freq_scale * theta_extrap;
            float th = theta_interp;
            float mscale = attn_factor;
            if (ext_factor != 0.0f) {
                const float ramp_mix = yarn_ramp(corr_dims[0], corr_dims[1], (int)i0) * ext_factor;
                /* the reference's x86 build contracts this sum into one fused multiply-add */
                th = fmaf(theta_interp, (1 - ramp_mix), theta_extrap * ramp_mix);
                mscale *= 1.0f + 0.1f * logf(1.0f / freq_scale);
            }
            cache[i0 + 0] = cosf(th) * mscale;
            cache[i0 + 1] = sinf(th) * mscale;
            theta *= theta_scale;
        }
        for (int64_t i1 = 0; i1 < src->ne[1]; ++i1) {
            const float * x = (const float *)tptr(src, i1, i2, i3);
            float * y = (float *)((char *)dst->data + i1 * dst->nb[1] + i2 * dst->nb[2] + i3 * dst->nb[3]);
            const int64_t n_off = (mode == 0) ? 1 : n_dims / 2;
            const int scale = (mode == 0) ? 1 : 2;
            for (int64_t i0 = 0; i0 < n_dims; i0 += 2) {
                const int64_t ic = i0 / scale;
                const float c = cache[i0 + 0], s = cache[i0 + 1];
                const float x0 = x[ic], x1 = x[ic + n_off];
                y[ic] = x0 * c - x1 * s;
                y[ic + n_off] = x0 * s + x1 * c;
            }
            for (int64_t i0 = n_dims; i0 < ne0; ++i0) y[i0] = x[i0];
        }
    }
    free(cache);
    return 0;
}

/* --------------------------------------------------------------------- SOFT_MAX */

static float alibi_slope(float max_bias, uint32_t h, uint32_t n_head) {
    if (!(max_bias > 0.0f)) return 1.0f;
    const uint32_t n_head_log2 = 1u << (uint32_t)floor(log2(n_head));
    const float m0 = powf(2.0f, -(max_bias) / n_head_log2);
    const float m1 = powf(2.0f, -(max_bias / 2.0f) / n_head_log2);
    return h < n_head_log2 ? powf(m0, h + 1) : powf(m1, 2 * (h - n_head_log2) + 1);
}

int orc_soft_max(const orc_tensor * src, const orc_tensor * mask, const float * sinks,
                 orc_tensor * dst, float scale, float max_bias) {
    if (src->type != ORC_F32 || !is_contiguous_f32(dst)) return 1;
    if (mask && mask->type != ORC_F16 && mask->type != ORC_F32) return 2;
    const int64_t ne00 = src->ne[0];
    float * wp = (float *)malloc((size_t)ne00 * sizeof(float));
    if (!wp) return 6;
    for (int64_t i3 = 0; i3 < src->ne[3]; ++i3)
    for (int64_t i2 = 0; i2 < src->ne[2]; ++i2)
    for (int64_t i1 = 0; i1 < src->ne[1]; ++i1) {
        const float slope = alibi_slope(max_bias, (uint32_t)i2, (uint32_t)src->ne[2]);
        const float * sp = (const float *)tptr(src, i1, i2, i3);
        float * dp = (float *)((char *)dst->data + i1 * dst->nb[1] + i2 * dst->nb[2] + i3 * dst->nb[3]);
        for (int64_t i = 0; i < ne00; ++i) wp[i] = sp[i] * scale;
        if (mask) {
            const char * mp = tptr(mask, i1, i2 % mask->ne[2], i3 % mask->ne[3]);
            for (int64_t i = 0; i < ne00; ++i) {
                const float m = mask->type == ORC_F16 ? orc_fp16_to_fp32(((const uint16_t *)mp)[i])
                                                      : ((const float *)mp)[i];
                wp[i] += slope * m;
            }
        }
        float max = -INFINITY;
        for (int64_t i = 0; i < ne00; ++i) max = MAXF(max, wp[i]);
        if (sinks) max = MAXF(max, sinks[i2]);
        double sum = 0.0;
        for (int64_t i = 0; i < ne00; ++i) {
            const float e = expf(wp[i] - max);
            dp[i] = e;
            sum += (double)e;
        }
        if (sinks) sum += (double)expf(sinks[i2] - max);
        sum = 1.0 / sum;
        for (int64_t i = 0; i < ne00; ++i) dp[i] *= (float)sum;
    }
    free(wp);
    return 0;
}

/* --------------------------------------------------------------- FLASH_ATTN_EXT */

typedef struct {
    const orc_tensor *q, *k, *v, *mask;
    const float * sinks;
    orc_tensor * dst;
    float scale, max_bias, logit_softcap;
    int64_t DK, DV;
} fa_ctx;

static inline float kv_elem(const orc_tensor * t, const char * row, int64_t d) {
    return t->type == ORC_F16 ? orc_fp16_to_fp32(((const uint16_t *)row)[d]) : ((const float *)row)[d];
}

/* one query row over keys [ic_start, ic_end): ops.cpp:8193-8344.  When partial != NULL
 * writes {M, S, VKQ[DV]} there (split-KV), else normalises and stores the row. */
static void fa_vec_row(const fa_ctx * c, int64_t iq1, int64_t iq2, int64_t iq3, int64_t ic_start,
                       int64_t ic_end, float * partial, float * VKQ32, uint16_t * VKQ16,
                       float * Qf) {
    const orc_tensor *q = c->q, *k = c->k, *v = c->v, *mask = c->mask;
    const int64_t DK = c->DK, DV = c->DV;
    const int64_t rk2 = q->ne[2] / k->ne[2], rk3 = q->ne[3] / k->ne[3];
    const int64_t rv2 = q->ne[2] / v->ne[2], rv3 = q->ne[3] / v->ne[3];
    const float slope = alibi_slope(c->max_bias, (uint32_t)iq2, (uint32_t)q->ne[2]);
    const int v_f16 = v->type == ORC_F16;

    float S = 0.0f, M = -INFINITY;
    if (v_f16) memset(VKQ16, 0, (size_t)DV * 2); else memset(VKQ32, 0, (size_t)DV * 4);

    const uint16_t * mp = mask ? (const uint16_t *)tptr(mask, iq1, iq2 % mask->ne[2], iq3 % mask->ne[3]) : NULL;
    const float * pq = (const float *)tptr(q, iq1, iq2, iq3);
    /* q_to_vec_dot: Q row converted to K's vec_dot_type (F16 for F16 K, F32 for F32 K) */
    for (int64_t d = 0; d < DK; ++d)
        Qf[d] = k->type == ORC_F16 ? orc_fp16_to_fp32(orc_fp32_to_fp16(pq[d])) : pq[d];

    for (int64_t ic = ic_start; ic < ic_end; ++ic) {
        const float mv = mp ? slope * orc_fp16_to_fp32(mp[ic]) : 0.0f;
        if (mv == -INFINITY) continue;
        const char * krow = tptr(k, ic, iq2 / rk2, iq3 / rk3);
        float s = 0.0f;
        for (int64_t d = 0; d < DK; ++d) s = fmaf(kv_elem(k, krow, d), Qf[d], s);
        s = s * c->scale;
        if (c->logit_softcap != 0.0f) s = c->logit_softcap * tanhf(s);
        s += mv;

        const float Mold = M;
        float ms = 1.0f, vs = 1.0f;
        const char * vrow = tptr(v, ic, iq2 / rv2, iq3 / rv3);
        if (s > M) { M = s; ms = expf(Mold - M); } else { vs = expf(s - M); }
        if (v_f16) {
            /* F16 accumulator: every step rounds to half (ops.cpp:8259-8273;
             * ggml_vec_scale_f16 / ggml_vec_mad_f16 in ggml/src/ggml-cpu/vec.h) */
            if (s > Mold) for (int64_t d = 0; d < DV; ++d)
                VKQ16[d] = orc_fp32_to_fp16(orc_fp16_to_fp32(VKQ16[d]) * ms);
            for (int64_t d = 0; d < DV; ++d)
                VKQ16[d] = orc_fp32_to_fp16(fmaf(orc_fp16_to_fp32(((const uint16_t *)vrow)[d]), vs,
                                                 orc_fp16_to_fp32(VKQ16[d])));
        } else {
            if (s > Mold) for (int64_t d = 0; d < DV; ++d) VKQ32[d] *= ms;
            for (int64_t d = 0; d < DV; ++d) VKQ32[d] = fmaf(((const float *)vrow)[d], vs, VKQ32[d]);
        }
        S = S * ms + vs;
    }
    if (v_f16) for (int64_t d = 0; d < DV; ++d) VKQ32[d] = orc_fp16_to_fp32(VKQ16[d]);

    if (c->sinks && ic_start == 0) {
        const float s = c->sinks[iq2];
        float ms = 1.0f, vs = 1.0f;
        if (s > M) { ms = expf(M - s); M = s; for (int64_t d = 0; d < DV; ++d) VKQ32[d] *= ms; }
        else vs = expf(s - M);
        S = S * ms + vs;
    }
    if (partial) {
        partial[0] = M;
        partial[1] = S;
        memcpy(partial + 2, VKQ32, (size_t)DV * 4);
    } else {
        const float S_inv = S == 0.0f ? 0.0f : 1.0f / S;
        float * out = (float *)((char *)c->dst->data +
                                (iq3 * c->dst->ne[2] * c->dst->ne[1] + iq2 + iq1 * c->dst->ne[1]) * c->dst->nb[1]);
        for (int64_t d = 0; d < DV; ++d) out[d] = VKQ32[d] * S_inv;
    }
}

/* C[M x N] += A[M x K] B[K x N], each element accumulated over k in order with a fused
 * multiply-add: the order of simd_gemm_ukernel (ggml/src/ggml-cpu/simd-gemm.h:24-58). */
static void gemm_fma(float * C, const float * A, const float * B, int M, int K, int N) {
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            float acc = C[i * N + j];
            for (int kk = 0; kk < K; ++kk) acc = fmaf(B[kk * N + j], A[i * K + kk], acc);
            C[i * N + j] = acc;
        }
}

#define FA_TQ 64 /* GGML_FA_TILE_Q,  ggml/src/ggml-cpu/common.h:9-10 */
#define FA_TK 64 /* GGML_FA_TILE_KV */

/* rows [ir0, ir1) of the flattened (iq3, iq2, iq1) index space: ops.cpp:8347-8633 */
static int fa_tiled(const fa_ctx * c, int64_t ir0, int64_t ir1) {
    const orc_tensor *q = c->q, *k = c->k, *v = c->v, *mask = c->mask;
    const int64_t DK = c->DK, DV = c->DV;
    const int64_t neq1 = q->ne[1], neq2 = q->ne[2], nek1 = k->ne[1];
    const int64_t rk2 = q->ne[2] / k->ne[2], rk3 = q->ne[3] / k->ne[3];
    const int64_t rv2 = q->ne[2] / v->ne[2], rv3 = q->ne[3] / v->ne[3];
    float * buf = (float *)malloc(sizeof(float) * (size_t)(FA_TQ * DK + 2 * FA_TQ * FA_TK + FA_TQ * DV + FA_TK * DV + FA_TK * DK));
    if (!buf) return 6;
    float * Qf = buf, *KQ = Qf + FA_TQ * DK, *mask32 = KQ + FA_TQ * FA_TK, *VKQ = mask32 + FA_TQ * FA_TK;
    float * V32 = VKQ + FA_TQ * DV, *Kf = V32 + FA_TK * DV;

    int64_t ir = ir0;
    while (ir < ir1) {
        const int64_t iq3 = ir / (neq2 * neq1);
        const int64_t iq2 = (ir - iq3 * neq2 * neq1) / neq1;
        const int64_t iq1 = ir - iq3 * neq2 * neq1 - iq2 * neq1;
        int tile_rows = FA_TQ;
        if (ir1 - ir < tile_rows) tile_rows = (int)(ir1 - ir);
        if (neq1 - iq1 < tile_rows) tile_rows = (int)(neq1 - iq1);
        const float slope = alibi_slope(c->max_bias, (uint32_t)iq2, (uint32_t)neq2);

        float S[FA_TQ], M[FA_TQ];
        for (int i = 0; i < FA_TQ; ++i) { S[i] = 0.f; M[i] = -INFINITY; }
        memset(VKQ, 0, sizeof(float) * FA_TQ * DV);
        memset(mask32, 0, sizeof(float) * FA_TQ * FA_TK);
        for (int tq = 0; tq < FA_TQ; ++tq) {
            if (tq < tile_rows) memcpy(Qf + tq * DK, tptr(q, iq1 + tq, iq2, iq3), (size_t)DK * 4);
            else memset(Qf + tq * DK, 0, (size_t)DK * 4);
        }
        memset(Kf, 0, sizeof(float) * DK * FA_TK);
        memset(V32, 0, sizeof(float) * FA_TK * DV);

        for (int64_t ic = 0; ic < nek1; ic += FA_TK) {
            const int kv_tile = (int)((nek1 - ic) < FA_TK ? (nek1 - ic) : FA_TK);
            if (mask) {
                int can_skip = 1;
                for (int tq = 0; tq < tile_rows; ++tq) {
                    const uint16_t * mrow = (const uint16_t *)tptr(mask, iq1 + tq, iq2 % mask->ne[2], iq3 % mask->ne[3]);
                    for (int tk = 0; tk < kv_tile; ++tk) {
                        mask32[tq * FA_TK + tk] = slope * orc_fp16_to_fp32(mrow[ic + tk]);
                        if (mask32[tq * FA_TK + tk] != -INFINITY) can_skip = 0;
                    }
                    for (int tk = kv_tile; tk < FA_TK; ++tk) mask32[tq * FA_TK + tk] = -INFINITY;
                }
                if (can_skip) continue;
            }
            for (int tk = 0; tk < kv_tile; ++tk) {
                const char * krow = tptr(k, ic + tk, iq2 / rk2, iq3 / rk3);
                for (int64_t d = 0; d < DK; ++d) Kf[d * FA_TK + tk] = kv_elem(k, krow, d);
            }
            memset(KQ, 0, sizeof(float) * FA_TQ * FA_TK);
            gemm_fma(KQ, Qf, Kf, FA_TQ, (int)DK, FA_TK);
            for (int i = 0; i < FA_TQ * FA_TK; ++i) KQ[i] *= c->scale;
            if (kv_tile < FA_TK)
                for (int tq = 0; tq < FA_TQ; ++tq)
                    for (int tk = kv_tile; tk < FA_TK; ++tk) KQ[tq * FA_TK + tk] = -INFINITY;
            if (c->logit_softcap != 0.0f)
                for (int i = 0; i < FA_TQ * FA_TK; ++i) KQ[i] = tanhf(KQ[i]) * c->logit_softcap;
            if (mask) for (int i = 0; i < tile_rows * FA_TK; ++i) KQ[i] += mask32[i];

            int skip[FA_TQ];
            for (int tq = 0; tq < FA_TQ; ++tq) {
                float * row = KQ + tq * FA_TK;
                skip[tq] = 0;
                float tmax = -INFINITY;
                for (int tk = 0; tk < FA_TK; ++tk) tmax = MAXF(tmax, row[tk]);
                if (tmax == -INFINITY) { skip[tq] = 1; continue; }
                const float Mold = M[tq], Mnew = fmaxf(Mold, tmax);
                if (Mnew > Mold) {
                    const float ms = expf(Mold - Mnew);
                    for (int64_t d = 0; d < DV; ++d) VKQ[tq * DV + d] *= ms;
                    S[tq] *= ms;
                }
                M[tq] = Mnew;
                double sum = 0.0; /* ggml_vec_soft_max_f32 returns a ggml_float (double) */
                for (int tk = 0; tk < FA_TK; ++tk) { row[tk] = expf(row[tk] - Mnew); sum += (double)row[tk]; }
                S[tq] += (float)sum;
            }
            for (int tk = 0; tk < kv_tile; ++tk) {
                const char * vrow = tptr(v, ic + tk, iq2 / rv2, iq3 / rv3);
                for (int64_t d = 0; d < DV; ++d) V32[tk * DV + d] = kv_elem(v, vrow, d);
            }
            for (int tq = 0; tq < FA_TQ; ++tq)
                if (skip[tq]) memset(KQ + tq * FA_TK, 0, sizeof(float) * FA_TK);
            gemm_fma(VKQ, KQ, V32, FA_TQ, FA_TK, (int)DV);
        }
        for (int tq = 0; tq < tile_rows; ++tq) {
            if (c->sinks) {
                const float s = c->sinks[iq2];
                float ms = 1.0f, vs = 1.0f;
                if (s > M[tq]) { ms = expf(M[tq] - s); for (int64_t d = 0; d < DV; ++d) VKQ[tq * DV + d] *= ms; }
                else vs = expf(s - M[tq]);
                S[tq] = S[tq] * ms + vs;
            }
            const float S_inv = S[tq] == 0.0f ? 0.0f : 1.0f / S[tq];
            float * out = (float *)((char *)c->dst->data +
                                    (iq3 * c->dst->ne[2] * c->dst->ne[1] + iq2 + (iq1 + tq) * c->dst->ne[1]) * c->dst->nb[1]);
            for (int64_t d = 0; d < DV; ++d) out[d] = VKQ[tq * DV + d] * S_inv;
        }
        ir += tile_rows;
    }
    free(buf);
    return 0;
}

static int fa_check(const orc_tensor * q, const orc_tensor * k, const orc_tensor * v,
                    const orc_tensor * mask, const orc_tensor * dst) {
    if (q->type != ORC_F32 || dst->type != ORC_F32) return 1;
    if ((k->type != ORC_F32 && k->type != ORC_F16) || (v->type != ORC_F32 && v->type != ORC_F16)) return 2;
    if (q->ne[0] != k->ne[0] || k->ne[1] != v->ne[1]) return 3;
    if (q->ne[2] % k->ne[2] || q->ne[3] % k->ne[3] || q->ne[2] % v->ne[2] || q->ne[3] % v->ne[3]) return 4;
    if (dst->ne[0] != v->ne[0] || dst->ne[1] != q->ne[2] || dst->ne[2] != q->ne[1] || dst->ne[3] != q->ne[3]) return 5;
    if (q->nb[0] != 4 || dst->nb[0] != 4) return 6;
    if (mask && (mask->type != ORC_F16 || mask->ne[0] != k->ne[1] || mask->ne[1] < q->ne[1])) return 7;
    return 0;
}

int orc_flash_attn_ext(const orc_tensor * q, const orc_tensor * k, const orc_tensor * v,
                       const orc_tensor * mask, const float * sinks, orc_tensor * dst,
                       float scale, float max_bias, float logit_softcap, int path, int nth) {
    int rc = fa_check(q, k, v, mask, dst);
    if (rc) return rc;
    fa_ctx c = { q, k, v, mask, sinks, dst, scale, max_bias, logit_softcap, k->ne[0], v->ne[0] };
    if (logit_softcap != 0.0f) c.scale /= logit_softcap;
    if (nth < 1) nth = 1;
    const int64_t neq1 = q->ne[1], neq2 = q->ne[2], neq3 = q->ne[3], nek1 = k->ne[1];

    if (path == ORC_FA_AUTO) { /* ops.cpp:8755-8756, 8813-8820 */
        if (neq1 == 1 && neq3 == 1 && k->type == v->type && nek1 >= 512) path = ORC_FA_SPLIT_KV;
        else if (k->type == v->type && neq1 >= FA_TQ && c.DV % 16 == 0) path = ORC_FA_TILED;
        else path = ORC_FA_VEC;
    }
    if (path == ORC_FA_TILED) {
        if (k->type != v->type) return 8;
        return fa_tiled(&c, 0, neq1 * neq2 * neq3);
    }
    float * VKQ32 = (float *)malloc((size_t)(2 * c.DV + c.DK) * sizeof(float));
    if (!VKQ32) return 6;
    uint16_t * VKQ16 = (uint16_t *)(VKQ32 + c.DV);
    float * Qf = VKQ32 + 2 * c.DV;

    if (path == ORC_FA_VEC) {
        for (int64_t iq3 = 0; iq3 < neq3; ++iq3)
        for (int64_t iq2 = 0; iq2 < neq2; ++iq2)
        for (int64_t iq1 = 0; iq1 < neq1; ++iq1)
            fa_vec_row(&c, iq1, iq2, iq3, 0, nek1, NULL, VKQ32, VKQ16, Qf);
    } else if (path == ORC_FA_SPLIT_KV) { /* ops.cpp:8758-8786 and 8637-8705 */
        if (neq1 != 1 || neq3 != 1) { free(VKQ32); return 9; }
        const int64_t chunk = (nek1 + nth - 1) / nth;
        const int64_t psz = 2 + c.DV;
        float * partials = (float *)malloc((size_t)(neq2 * nth * psz) * sizeof(float));
        if (!partials) { free(VKQ32); return 6; }
        for (int ith = 0; ith < nth; ++ith) {
            const int64_t s0 = ith * chunk, s1 = MINF(s0 + chunk, nek1);
            for (int64_t h = 0; h < neq2; ++h) {
                float * p = partials + (h * nth + ith) * psz;
                if (s0 < nek1) fa_vec_row(&c, 0, h, 0, s0, s1, p, VKQ32, VKQ16, Qf);
                else { p[0] = -INFINITY; p[1] = 0.0f; }
            }
        }
        for (int64_t h = 0; h < neq2; ++h) {
            float Mf = -INFINITY, Sf = 0.0f;
            float * acc = VKQ32;
            memset(acc, 0, (size_t)c.DV * 4);
            for (int ci = 0; ci < nth; ++ci) {
                if (ci * chunk >= nek1) continue;
                const float * p = partials + (h * nth + ci) * psz;
                if (p[1] == 0.0f) continue;
                const float Mn = fmaxf(Mf, p[0]);
                const float so = expf(Mf - Mn), sn = expf(p[0] - Mn);
                for (int64_t d = 0; d < c.DV; ++d) acc[d] = acc[d] * so + p[2 + d] * sn;
                Sf = Sf * so + p[1] * sn;
                Mf = Mn;
            }
            float * out = (float *)((char *)dst->data + h * dst->nb[1]);
            const float inv = Sf != 0.0f ? 1.0f / Sf : 1.0f;
            for (int64_t d = 0; d < c.DV; ++d) out[d] = acc[d] * inv;
        }
        free(partials);
    } else { free(VKQ32); return 10; }
    free(VKQ32);
    return 0;
}

int orc_flash_attn_ext_f64(const orc_tensor * q, const orc_tensor * k, const orc_tensor * v,
                           const orc_tensor * mask, const float * sinks, orc_tensor * dst,
                           float scale, float max_bias, float logit_softcap) {
    int rc = fa_check(q, k, v, mask, dst);
    if (rc) return rc;
    const int64_t DK = k->ne[0], DV = v->ne[0], nek1 = k->ne[1];
    const int64_t rk2 = q->ne[2] / k->ne[2], rk3 = q->ne[3] / k->ne[3];
    const int64_t rv2 = q->ne[2] / v->ne[2], rv3 = q->ne[3] / v->ne[3];
    double sc = scale;
    if (logit_softcap != 0.0f) sc /= logit_softcap;
    double * s = (double *)malloc((size_t)(nek1 + DV) * sizeof(double));
    if (!s) return 6;
    double * acc = s + nek1;
    for (int64_t iq3 = 0; iq3 < q->ne[3]; ++iq3)
    for (int64_t iq2 = 0; iq2 < q->ne[2]; ++iq2)
    for (int64_t iq1 = 0; iq1 < q->ne[1]; ++iq1) {
        const double slope = alibi_slope(max_bias, (uint32_t)iq2, (uint32_t)q->ne[2]);
        const float * pq = (const float *)tptr(q, iq1, iq2, iq3);
        const uint16_t * mp = mask ? (const uint16_t *)tptr(mask, iq1, iq2 % mask->ne[2], iq3 % mask->ne[3]) : NULL;
        double mx = -INFINITY;
        for (int64_t ic = 0; ic < nek1; ++ic) {
            const char * krow = tptr(k, ic, iq2 / rk2, iq3 / rk3);
            double d = 0.0;
            for (int64_t i = 0; i < DK; ++i) d += (double)pq[i] * (double)kv_elem(k, krow, i);
            d *= sc;
            if (logit_softcap != 0.0f) d = logit_softcap * tanh(d);
            if (mp) d += slope * (double)orc_fp16_to_fp32(mp[ic]);
            s[ic] = d;
            if (d > mx) mx = d;
        }
        if (sinks && sinks[iq2] > mx) mx = sinks[iq2];
        double sum = 0.0;
        for (int64_t d = 0; d < DV; ++d) acc[d] = 0.0;
        if (mx != -INFINITY) {
            for (int64_t ic = 0; ic < nek1; ++ic) {
                if (s[ic] == -INFINITY) continue;
                const double p = exp(s[ic] - mx);
                sum += p;
                const char * vrow = tptr(v, ic, iq2 / rv2, iq3 / rv3);
                for (int64_t d = 0; d < DV; ++d) acc[d] += p * (double)kv_elem(v, vrow, d);
            }
            if (sinks) sum += exp((double)sinks[iq2] - mx);
        }
        float * out = (float *)((char *)dst->data + (iq3 * dst->ne[2] * dst->ne[1] + iq2 + iq1 * dst->ne[1]) * dst->nb[1]);
        for (int64_t d = 0; d < DV; ++d) out[d] = sum > 0.0 ? (float)(acc[d] / sum) : 0.0f;
    }
    free(s);
    return 0;
}

/* --------------------------------------------------------- host-side index helpers */

void orc_kv_read_view(int head_dim, int max_length, int n_kv_heads, int es, int seq_len,
                      int64_t ne[3], uint64_t nb[3], uint64_t * offset) {
    /* cache tensor [head_dim, max_length, n_kv_heads]: nb1 = head_dim*es, nb2 = max_length*nb1 */
    const uint64_t cnb1 = (uint64_t)head_dim * (uint64_t)es, cnb2 = cnb1 * (uint64_t)max_length;
    ne[0] = head_dim; ne[1] = seq_len; ne[2] = n_kv_heads;
    nb[0] = (uint64_t)es; nb[1] = cnb1; nb[2] = cnb2;
    *offset = 0;
}

void orc_kv_write_view(int head_dim, int max_length, int n_kv_heads, int es, int start,
                       int n_tokens, int64_t ne[3], uint64_t nb[3], uint64_t * offset) {
    const uint64_t cnb1 = (uint64_t)head_dim * (uint64_t)es, cnb2 = cnb1 * (uint64_t)max_length;
    ne[0] = head_dim; ne[1] = n_kv_heads; ne[2] = n_tokens;
    nb[0] = (uint64_t)es; nb[1] = cnb2; nb[2] = cnb1;
    *offset = (uint64_t)start * cnb1;
}

void orc_causal_mask(const int32_t * positions, int n_q, int total_len, uint16_t * mask) {
    /* step(key - query - 0.5) * -1e9 cast to F16: visible entries are 0 * -1e9 = -0.0 */
    for (int r = 0; r < n_q; ++r)
        for (int cidx = 0; cidx < total_len; ++cidx) {
            const float t = (float)cidx - (float)positions[r] + -0.5f;
            const float st = t > 0.0f ? 1.0f : 0.0f;
            mask[(size_t)r * (size_t)total_len + (size_t)cidx] = orc_fp32_to_fp16(st * -1e9f);
        }
}

void orc_cfg_pair_constants(int branch_len, int32_t * positions, uint16_t * mask) {
    const int total = 2 * branch_len;
    for (int i = 0; i < total; ++i) positions[i] = i % branch_len;
    for (int r = 0; r < total; ++r)
        for (int cidx = 0; cidx < total; ++cidx)
            mask[(size_t)r * (size_t)total + (size_t)cidx] =
                orc_fp32_to_fp16((r / branch_len) == (cidx / branch_len) ? 0.0f : -1e9f);
}

void orc_t_span(int n_timesteps, float sway_coef, float * out) {
    for (int i = 0; i <= n_timesteps; ++i) {
        const float base = 1.0f - (float)i / (float)n_timesteps;
        out[i] = base + sway_coef * (cosf((float)M_PI_2 * base) - 1.0f + base);
    }
}
