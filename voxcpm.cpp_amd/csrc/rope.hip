// rope.hip -- GGML_OP_ROPE (F32, modes NORMAL and NEOX, optional frequency factors and
// YaRN mixing) on gfx950.
//
// ggml-cpu builds the angle of pair p as pos * theta_scale^p by p successive fp32
// multiplications (ggml/src/ggml-cpu/ops.cpp:5613-5627).  At position 8192 the rounding
// of that chain moves the angle by about 1e-3 rad relative to a closed form, so the
// kernel replays the chain (p dependent multiplies, at most n_dims/2 - 1 of them) and
// only cosf/sinf differ from the host's libm, by an ulp or two.
//
// One thread per (pair, row); a row is one (head, token, batch) vector.  HBM-bound at
// 8 bytes per element; in decode it is a handful of rows and purely launch latency.
#include "rope_common.hpp"

// the angle arithmetic must round like the host code it mirrors: no fused multiply-adds
#pragma clang fp contract(off)

namespace {

__global__ __launch_bounds__(256) void rope_kernel(const char * __restrict__ src, char * __restrict__ dst, vx_dims s,
                                                   vx_dims d, const int32_t * __restrict__ pos,
                                                   const float * __restrict__ freq_factors, rope_params p) {
    const int64_t half   = s.ne[0] / 2; // pairs per row, counting the pass-through tail
    const int64_t nrows  = s.ne[1] * s.ne[2] * s.ne[3];
    const int64_t gid    = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= nrows * half) return;
    const int64_t row = gid / half;
    const int     ip  = (int) (gid % half); // pair index within the row
    const int64_t i1  = row % s.ne[1];
    const int64_t i2  = (row / s.ne[1]) % s.ne[2];
    const int64_t i3  = row / (s.ne[1] * s.ne[2]);
    const float * x   = (const float *) (src + i1 * s.nb[1] + i2 * s.nb[2] + i3 * s.nb[3]);
    float *       y   = (float *) (dst + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]);

    const int npairs = p.n_dims / 2;
    if (ip >= npairs) { // channels beyond n_dims are copied
        const int i0 = 2 * ip;
        const float a = x[i0], b = x[i0 + 1];
        y[i0]     = a;
        y[i0 + 1] = b;
        return;
    }

    // every load is requested before the angle arithmetic, so one memory round trip covers them all
    const int ia = p.mode == 0 ? 2 * ip : ip;
    const int ib = p.mode == 0 ? 2 * ip + 1 : ip + npairs;
    const float x0 = x[ia], x1 = x[ib];
    const float ff = freq_factors ? freq_factors[ip] : 1.0f;

    float c, sn;
    rope_cos_sin(p, (float) pos[i2], ip, ff, c, sn);
    float y0, y1;
    rope_rotate(x0, x1, c, sn, y0, y1);
    y[ia] = y0;
    y[ib] = y1;
}

} // namespace

extern "C" int vx_supports_rope(const vx_tensor * src, const vx_tensor * dst, int n_dims, int mode) {
    if (!src || !dst) return 0;
    if (src->type != VX_TYPE_F32 || dst->type != VX_TYPE_F32) return 0;
    if (!vx_same_shape(src, dst) || !vx_positive(src)) return 0;
    if (src->nb[0] != 4 || dst->nb[0] != 4) return 0;
    if (mode != 0 && mode != 2) return 0;
    if (n_dims <= 0 || n_dims % 2 || n_dims > src->ne[0] || src->ne[0] % 2) return 0;
    if (vx_nelements(src) / 2 > (int64_t) 0x7fffffff * 256) return 0;
    return 1;
}

extern "C" vx_status vx_rope(const vx_tensor * src, const int32_t * pos, const float * freq_factors,
                             const vx_tensor * dst, int n_dims, int mode, int n_ctx_orig, float freq_base,
                             float freq_scale, float ext_factor, float attn_factor, float beta_fast,
                             float beta_slow, vx_stream stream) {
    if (!src || !dst || !src->data || !dst->data || !pos) return vx_fail(VX_ERR_INVALID, "rope: null argument");
    if (!vx_supports_rope(src, dst, n_dims, mode))
        return vx_fail(VX_ERR_UNSUPPORTED, "rope: needs F32 tensors of equal shape, dense rows, mode 0 or 2, even n_dims <= ne0");
    const rope_params p = rope_make_params(n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    const int64_t total = vx_nrows(src) * (src->ne[0] / 2);
    const unsigned grid = (unsigned) ((total + 255) / 256);
    vx_launch(rope_kernel, dim3(grid), dim3(256), 0, (hipStream_t) stream, (const char *) src->data, (char *) dst->data,
                                                                    vx_dims_of(src), vx_dims_of(dst), pos,
                                                                    freq_factors, p);
    VX_LAUNCH_CHECK();
    return VX_OK;
}
