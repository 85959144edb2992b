// soft_max.hip -- GGML_OP_SOFT_MAX on gfx950: dst = softmax(scale*x + slope(head)*mask),
// optional per-head sinks (ggml/src/ggml-cpu/ops.cpp:5225-5335).
//
// VoxCPM's graphs never emit this op (attention goes through FLASH_ATTN_EXT); it is claimed
// for generality.  One block per row: rows up to SM_LDS_FLOATS are staged once in LDS
// (read x and mask once, write dst once -- the HBM minimum); longer rows are recomputed
// from global memory in three passes.
#include "vx_common.hpp"

#include <cmath>

namespace {

constexpr int SM_BLOCK      = 256;
constexpr int SM_LDS_FLOATS = 8192;

struct sm_params {
    float    scale, max_bias, m0, m1;
    uint32_t n_head_log2;
    int      mask_f16;
};

__device__ __forceinline__ float block_max(float v, float * red) {
    v = vx_wave_max(v);
    if (threadIdx.x % VX_WAVE == 0) red[threadIdx.x / VX_WAVE] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < SM_BLOCK / VX_WAVE; ++w) r = fmaxf(r, red[w]);
    __syncthreads();
    return r;
}
__device__ __forceinline__ float block_sum(float v, float * red) {
    v = vx_wave_sum(v);
    if (threadIdx.x % VX_WAVE == 0) red[threadIdx.x / VX_WAVE] = v;
    __syncthreads();
    float r = red[0];
#pragma unroll
    for (int w = 1; w < SM_BLOCK / VX_WAVE; ++w) r += red[w];
    __syncthreads();
    return r;
}

__global__ __launch_bounds__(SM_BLOCK) void soft_max_kernel(const char * __restrict__ src, const char * __restrict__ mask,
                                                            const float * __restrict__ sinks, char * __restrict__ dst,
                                                            vx_dims s, vx_dims m, vx_dims d, sm_params p) {
    __shared__ float vals[SM_LDS_FLOATS];
    __shared__ float red[SM_BLOCK / VX_WAVE];

    const int64_t row = blockIdx.x;
    const int64_t i1  = row % s.ne[1];
    const int64_t i2  = (row / s.ne[1]) % s.ne[2];
    const int64_t i3  = row / (s.ne[1] * s.ne[2]);
    const int64_t n   = s.ne[0];
    const float * x   = (const float *) (src + i1 * s.nb[1] + i2 * s.nb[2] + i3 * s.nb[3]);
    float *       y   = (float *) (dst + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]);
    const char *  mp  = mask ? mask + i1 * m.nb[1] + (i2 % m.ne[2]) * m.nb[2] + (i3 % m.ne[3]) * m.nb[3] : nullptr;
    const float slope = vx_alibi_slope(p.max_bias, (uint32_t) i2, p.n_head_log2, p.m0, p.m1);
    const bool  in_lds = n <= SM_LDS_FLOATS;

    auto logit = [&](int64_t i) -> float {
        float v = x[i] * p.scale;
        if (mp) v += slope * (p.mask_f16 ? __half2float(((const __half *) mp)[i]) : ((const float *) mp)[i]);
        return v;
    };

    float mx = -INFINITY;
    for (int64_t i = threadIdx.x; i < n; i += SM_BLOCK) {
        const float v = logit(i);
        if (in_lds) vals[i] = v;
        mx = fmaxf(mx, v);
    }
    mx = block_max(mx, red);
    if (sinks) mx = fmaxf(mx, sinks[i2]);

    float sum = 0.0f;
    for (int64_t i = threadIdx.x; i < n; i += SM_BLOCK) {
        const float e = expf((in_lds ? vals[i] : logit(i)) - mx);
        if (in_lds) vals[i] = e;
        sum += e;
    }
    sum = block_sum(sum, red);
    if (sinks) sum += expf(sinks[i2] - mx);
    const float inv = 1.0f / sum;

    // dst may alias src: every element is read (above) and written by the same thread
    for (int64_t i = threadIdx.x; i < n; i += SM_BLOCK) {
        const float e = in_lds ? vals[i] : expf(logit(i) - mx);
        y[i] = e * inv;
    }
}

} // namespace

extern "C" int vx_supports_soft_max(const vx_tensor * src, const vx_tensor * mask, const vx_tensor * dst) {
    if (!src || !dst) return 0;
    if (src->type != VX_TYPE_F32 || dst->type != VX_TYPE_F32) return 0;
    if (!vx_same_shape(src, dst) || !vx_positive(src)) return 0;
    if (src->nb[0] != 4 || !vx_is_contiguous(dst)) return 0;
    if (vx_nrows(src) > 0x7fffffff) return 0;
    if (mask) {
        if (mask->type != VX_TYPE_F16 && mask->type != VX_TYPE_F32) return 0;
        if (mask->nb[0] != vx_type_size(mask->type)) return 0;
        if (mask->ne[0] != src->ne[0] || mask->ne[1] < src->ne[1]) return 0;
        if (mask->ne[2] <= 0 || mask->ne[3] <= 0 || src->ne[2] % mask->ne[2] || src->ne[3] % mask->ne[3]) return 0;
    }
    return 1;
}

extern "C" vx_status vx_soft_max(const vx_tensor * src, const vx_tensor * mask, const float * sinks,
                                 const vx_tensor * dst, float scale, float max_bias, vx_stream stream) {
    if (!src || !dst || !src->data || !dst->data || (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "soft_max: null tensor");
    if (!vx_supports_soft_max(src, mask, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "soft_max: needs F32 src/dst of equal shape, dense rows, F16/F32 mask broadcastable over dims 2,3");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "soft_max: max_bias > 0 requires a mask");
    sm_params p;
    p.scale       = scale;
    p.max_bias    = max_bias;
    p.n_head_log2 = 1u << (uint32_t) floor(log2((double) src->ne[2]));
    p.m0          = powf(2.0f, -(max_bias) / p.n_head_log2);
    p.m1          = powf(2.0f, -(max_bias / 2.0f) / p.n_head_log2);
    p.mask_f16    = mask && mask->type == VX_TYPE_F16;
    vx_dims md    = mask ? vx_dims_of(mask) : vx_dims_of(src);
    vx_launch(soft_max_kernel, dim3((unsigned) vx_nrows(src)), dim3(SM_BLOCK), 0, (hipStream_t) stream, 
        (const char *) src->data, mask ? (const char *) mask->data : nullptr, sinks, (char *) dst->data,
        vx_dims_of(src), md, vx_dims_of(dst), p);
    VX_LAUNCH_CHECK();
    return VX_OK;
}
