// rms_norm.hip -- GGML_OP_RMS_NORM on gfx950.
//
// y = x / sqrt(mean(x^2) + eps), one row at a time.  ggml-cpu squares in fp32 and sums
// the squares in fp64 (ggml/src/ggml-cpu/ops.cpp:3736-3741); the kernel does the same so
// that mean, and therefore every output element, rounds identically except when two fp64
// summation orders straddle an fp32 rounding boundary.
//
// HBM-bound: 8 bytes per element (read + write).  A row is read once into registers, the
// wave (short rows) or block (long rows) reduces, the same registers are scaled and stored.
#include "vx_common.hpp"

namespace {

constexpr int RN_MAX_VEC = 8; // float4 chunks cached per thread before falling back to re-reading

template <int BLOCK>
__global__ __launch_bounds__(BLOCK) void rms_norm_kernel(const char * __restrict__ src, char * __restrict__ dst,
                                                         vx_dims s, vx_dims d, float eps, int rows_per_block,
                                                         const float * __restrict__ w) {
    constexpr int WAVES = BLOCK / VX_WAVE;
    __shared__ double red[WAVES];

    const int64_t ne00  = s.ne[0];
    const int64_t nrows = s.ne[1] * s.ne[2] * s.ne[3];
    // short rows: one wave per row, several rows per block; long rows: whole block per row
    const bool    wave_rows = rows_per_block > 1;
    const int     lane_id   = wave_rows ? (threadIdx.x % VX_WAVE) : threadIdx.x;
    const int     nlanes    = wave_rows ? VX_WAVE : BLOCK;
    const int64_t row       = wave_rows ? (int64_t) blockIdx.x * rows_per_block + threadIdx.x / VX_WAVE : blockIdx.x;
    if (row >= nrows) return; // whole wave (wave_rows) or whole block exits together

    const int64_t i1 = row % s.ne[1];
    const int64_t i2 = (row / s.ne[1]) % s.ne[2];
    const int64_t i3 = row / (s.ne[1] * s.ne[2]);
    const float * x  = (const float *) (src + i1 * s.nb[1] + i2 * s.nb[2] + i3 * s.nb[3]);
    float *       y  = (float *) (dst + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]);

    const bool vec_ok = (ne00 % 4 == 0) && (((uintptr_t) x | (uintptr_t) y | (uintptr_t) w) % 16 == 0);
    const int64_t nvec = vec_ok ? ne00 / 4 : 0;

    float4 cache[RN_MAX_VEC];
    float4 gain[RN_MAX_VEC]; // the weight row is requested together with x, not after the reduction
    double sum = 0.0;
    if (vec_ok) {
#pragma unroll
        for (int c = 0; c < RN_MAX_VEC; ++c) {
            const int64_t iv = lane_id + (int64_t) c * nlanes;
            if (iv < nvec) {
                const float4 v = ((const float4 *) x)[iv];
                if (w) gain[c] = ((const float4 *) w)[iv];
                cache[c]       = v;
                sum += (double) (v.x * v.x);
                sum += (double) (v.y * v.y);
                sum += (double) (v.z * v.z);
                sum += (double) (v.w * v.w);
            }
        }
        for (int64_t iv = lane_id + (int64_t) RN_MAX_VEC * nlanes; iv < nvec; iv += nlanes) {
            const float4 v = ((const float4 *) x)[iv];
            sum += (double) (v.x * v.x);
            sum += (double) (v.y * v.y);
            sum += (double) (v.z * v.z);
            sum += (double) (v.w * v.w);
        }
    } else {
        for (int64_t i = lane_id; i < ne00; i += nlanes) {
            const float v = x[i];
            sum += (double) (v * v);
        }
    }

    sum = vx_wave_sum(sum);
    if (!wave_rows) {
        if (threadIdx.x % VX_WAVE == 0) red[threadIdx.x / VX_WAVE] = sum;
        __syncthreads();
        sum = 0.0;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) sum += red[w];
    }

    const float mean  = (float) (sum / (double) ne00);
    const float scale = 1.0f / sqrtf(mean + eps);

    if (vec_ok) {
#pragma unroll
        for (int c = 0; c < RN_MAX_VEC; ++c) {
            const int64_t iv = lane_id + (int64_t) c * nlanes;
            if (iv < nvec) {
                float4 v = cache[c];
                v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
                if (w) { const float4 g = gain[c]; v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w; }
                ((float4 *) y)[iv] = v;
            }
        }
        for (int64_t iv = lane_id + (int64_t) RN_MAX_VEC * nlanes; iv < nvec; iv += nlanes) {
            float4 v = ((const float4 *) x)[iv];
            v.x *= scale; v.y *= scale; v.z *= scale; v.w *= scale;
            if (w) { const float4 g = ((const float4 *) w)[iv]; v.x *= g.x; v.y *= g.y; v.z *= g.z; v.w *= g.w; }
            ((float4 *) y)[iv] = v;
        }
    } else {
        for (int64_t i = lane_id; i < ne00; i += nlanes) {
            float v = x[i] * scale; // rounded here, as the separate RMS_NORM node would store it
            if (w) v *= w[i];
            y[i] = v;
        }
    }
}

} // namespace

extern "C" int vx_supports_rms_norm(const vx_tensor * src, const vx_tensor * dst) {
    if (!src || !dst) return 0;
    if (src->type != VX_TYPE_F32 || dst->type != VX_TYPE_F32) return 0;
    if (!vx_same_shape(src, dst) || !vx_positive(src)) return 0;
    if (src->nb[0] != 4 || dst->nb[0] != 4) return 0;
    if (vx_nrows(src) > 0x7fffffff) return 0;
    return 1;
}

static vx_status rms_norm_launch(const vx_tensor * src, const vx_tensor * dst, float eps, const float * w, vx_stream stream) {
    const int64_t nrows = vx_nrows(src);
    const vx_dims s = vx_dims_of(src), d = vx_dims_of(dst);
    hipStream_t   st = (hipStream_t) stream;
    if (src->ne[0] <= 1024) {
        const int rpb = 4; // one wave per row
        vx_launch(rms_norm_kernel<256>, dim3((unsigned) ((nrows + rpb - 1) / rpb)), dim3(256), 0, st, 
            (const char *) src->data, (char *) dst->data, s, d, eps, rpb, w);
    } else {
        vx_launch(rms_norm_kernel<256>, dim3((unsigned) nrows), dim3(256), 0, st, 
            (const char *) src->data, (char *) dst->data, s, d, eps, 1, w);
    }
    VX_LAUNCH_CHECK();
    return VX_OK;
}

extern "C" vx_status vx_rms_norm(const vx_tensor * src, const vx_tensor * dst, float eps, vx_stream stream) {
    if (!src || !dst || !src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "rms_norm: null tensor");
    if (!vx_supports_rms_norm(src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "rms_norm: needs F32 tensors of equal shape with dense rows");
    if (!(eps >= 0.0f)) return vx_fail(VX_ERR_INVALID, "rms_norm: eps must be >= 0");
    return rms_norm_launch(src, dst, eps, nullptr, stream);
}

extern "C" int vx_supports_rms_norm_mul(const vx_tensor * src, const vx_tensor * weight, const vx_tensor * dst) {
    if (!vx_supports_rms_norm(src, dst) || !weight || weight->type != VX_TYPE_F32) return 0;
    return weight->ne[0] == src->ne[0] && weight->ne[1] == 1 && weight->ne[2] == 1 && weight->ne[3] == 1 && weight->nb[0] == 4;
}

extern "C" vx_status vx_rms_norm_mul(const vx_tensor * src, const vx_tensor * weight, const vx_tensor * dst, float eps,
                                     vx_stream stream) {
    if (!src || !dst || !weight || !src->data || !dst->data || !weight->data) return vx_fail(VX_ERR_INVALID, "rms_norm_mul: null tensor");
    if (!vx_supports_rms_norm_mul(src, weight, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "rms_norm_mul: needs F32 tensors of equal shape with dense rows and one weight row");
    if (!(eps >= 0.0f)) return vx_fail(VX_ERR_INVALID, "rms_norm_mul: eps must be >= 0");
    return rms_norm_launch(src, dst, eps, (const float *) weight->data, stream);
}
