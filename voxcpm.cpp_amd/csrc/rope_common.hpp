// rope_common.hpp -- the angle and rotation arithmetic of GGML_OP_ROPE, shared by the ROPE kernel and by
// the projection kernel that applies the rotation in its epilogue, so that both round identically.
#pragma once
#include "vx_common.hpp"

#include <cmath>

struct rope_params {
    int   n_dims;
    int   mode; // 0 NORMAL, 2 NEOX
    float theta_scale;
    float freq_scale;
    float ext_factor;
    float attn_factor;
    float corr_lo, corr_hi;
};

// cos and sin (times the YaRN magnitude scale) of pair ip at position pos.  ggml-cpu builds the angle as
// pos * theta_scale^ip by ip successive fp32 multiplications (ggml/src/ggml-cpu/ops.cpp:5613-5627); the
// chain is replayed, and nothing here may be contracted into a fused multiply-add the host did not use.
__device__ __forceinline__ void rope_cos_sin(const rope_params & p, float pos, int ip, float ff, float & c, float & sn) {
#pragma clang fp contract(off)
    float theta = pos;
    for (int k = 0; k < ip; ++k) theta *= p.theta_scale;
    const float theta_extrap = theta / ff;
    const float theta_interp = p.freq_scale * theta_extrap;
    float       th           = theta_interp;
    float       mscale       = p.attn_factor;
    if (p.ext_factor != 0.0f) {
        // rope_yarn_ramp takes i0/2 as an int and clamps in fp32 (ops.cpp:5589-5592)
        const float yv       = ((float) ip - p.corr_lo) / fmaxf(0.001f, p.corr_hi - p.corr_lo);
        const float ramp_mix = (1.0f - fminf(1.0f, fmaxf(0.0f, yv))) * p.ext_factor;
        // ggml-cpu's x86 build contracts this sum into one fused multiply-add
        th                   = fmaf(theta_interp, 1.0f - ramp_mix, theta_extrap * ramp_mix);
        mscale *= 1.0f + 0.1f * logf(1.0f / p.freq_scale);
    }
    c  = cosf(th) * mscale;
    sn = sinf(th) * mscale;
}

__device__ __forceinline__ void rope_rotate(float x0, float x1, float c, float sn, float & y0, float & y1) {
#pragma clang fp contract(off)
    y0 = x0 * c - x1 * sn;
    y1 = x0 * sn + x1 * c;
}

static inline float rope_yarn_corr_dim(int n_dims, int n_ctx_orig, float n_rot, float base) {
    return n_dims * logf(n_ctx_orig / (n_rot * 2 * (float) M_PI)) / (2 * logf(base));
}

static inline rope_params rope_make_params(int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                                           float ext_factor, float attn_factor, float beta_fast, float beta_slow) {
    rope_params p;
    p.n_dims      = n_dims;
    p.mode        = mode;
    p.theta_scale = powf(freq_base, -2.0f / n_dims); // host libm, as ggml-cpu (ops.cpp:5775)
    p.freq_scale  = freq_scale;
    p.ext_factor  = ext_factor;
    p.attn_factor = attn_factor;
    // ggml_rope_yarn_corr_dims (ggml/src/ggml.c:4280-4294)
    const float start = floorf(rope_yarn_corr_dim(n_dims, n_ctx_orig, beta_fast, freq_base));
    const float end   = ceilf(rope_yarn_corr_dim(n_dims, n_ctx_orig, beta_slow, freq_base));
    p.corr_lo = fmaxf(0.0f, start);
    p.corr_hi = fminf((float) (n_dims - 1), end);
    return p;
}
