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

#include <cstdlib>

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

// A prefill's rotation: every head of a token turns by the same angles, so a thread takes one (token, pair) and walks the
// heads with one cosine and sine -- the angle arithmetic (a power, a sine and a cosine per pair, YaRN's ramp) is most of the
// kernel above and is done ne1 times less often here.  Same device functions, same bits.  32-bit element offsets (checked
// by the launcher); the walk's loads are requested four heads at a time.
__global__ __launch_bounds__(256) void rope_heads_kernel(const char * __restrict__ src, char * __restrict__ dst, vx_dims s, vx_dims d,
                                                         const int32_t * __restrict__ pos, const float * __restrict__ freq_factors, rope_params p) {
    const uint32_t half  = (uint32_t) (s.ne[0] / 2);
    const uint32_t gid   = blockIdx.x * 256u + threadIdx.x; // (token of the flattened (i2, i3) order, pair)
    const uint32_t tok   = gid / half, ip = gid - tok * half;
    const uint32_t ntok  = (uint32_t) (s.ne[2] * s.ne[3]);
    if (tok >= ntok) return;
    const uint32_t i3 = tok / (uint32_t) s.ne[2], i2 = tok - i3 * (uint32_t) s.ne[2];
    const char * x = src + (uint64_t) i2 * s.nb[2] + (uint64_t) i3 * s.nb[3];
    char *       y = dst + (uint64_t) i2 * d.nb[2] + (uint64_t) i3 * d.nb[3];
    const uint32_t npairs = (uint32_t) (p.n_dims / 2), heads = (uint32_t) s.ne[1];
    const bool     turn = ip < npairs;
    const uint32_t ia = !turn || p.mode == 0 ? 2 * ip : ip, ib = !turn || p.mode == 0 ? 2 * ip + 1 : ip + npairs;
    float c = 1.0f, sn = 0.0f;
    if (turn) rope_cos_sin(p, (float) pos[i2], (int) ip, freq_factors ? freq_factors[ip] : 1.0f, c, sn);
    for (uint32_t h0 = 0; h0 < heads; h0 += 4) {
        float x0[4], x1[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t h = min(h0 + u, heads - 1);
            const float * xr = (const float *) (x + (uint64_t) h * s.nb[1]);
            x0[u] = __builtin_nontemporal_load(xr + ia);
            x1[u] = __builtin_nontemporal_load(xr + ib);
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            if (h0 + u >= heads) break;
            float * yr = (float *) (y + (uint64_t) (h0 + u) * d.nb[1]);
            float y0 = x0[u], y1 = x1[u];
            if (turn) rope_rotate(x0[u], x1[u], c, sn, y0, y1); // (channels beyond n_dims are copied)
            yr[ia] = y0;
            yr[ib] = y1;
        }
    }
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
    // many tokens of several heads: the kernel that forms a token's angles once for all of its heads (VX_ROPE_HEADS=0: off)
    static const bool heads_off = [] { const char * e = getenv("VX_ROPE_HEADS"); return e && atoi(e) == 0; }();
    const int64_t ntok = src->ne[2] * src->ne[3];
    // (from 1024 tokens on: below, its few work-groups walking sixteen heads each take 5.8 us where a thread per (row, pair) takes 3.6 to 4.3)
    if (!heads_off && src->ne[1] >= 2 && ntok >= 1024 && ntok * (src->ne[0] / 2) < ((int64_t) 1 << 31)) {
        const int64_t threads = ntok * (src->ne[0] / 2);
        vx_launch(rope_heads_kernel, dim3((unsigned) ((threads + 255) / 256)), dim3(256), 0, (hipStream_t) stream, (const char *) src->data,
                  (char *) dst->data, vx_dims_of(src), vx_dims_of(dst), pos, freq_factors, p);
        VX_LAUNCH_CHECK();
        return VX_OK;
    }
    const int64_t total = vx_nrows(src) * (src->ne[0] / 2);
    const unsigned grid = (unsigned) ((total + 255) / 256);
    vx_launch(rope_kernel, dim3(grid), dim3(256), 0, (hipStream_t) stream, (const char *) src->data, (char *) dst->data,
                                                                    vx_dims_of(src), vx_dims_of(dst), pos,
                                                                    freq_factors, p);
    VX_LAUNCH_CHECK();
    return VX_OK;
}
