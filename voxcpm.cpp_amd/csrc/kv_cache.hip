// kv_cache.hip -- MiniCPMKVCache's views and the token append, on the device.
//
// The cache of one layer is a tensor [head_dim, max_length, n_kv_heads] (F16 or F32).
//   read view  (src/minicpm.cpp:200-212): [head_dim, seq_len, n_kv_heads], same strides,
//               offset 0 -- what FLASH_ATTN_EXT consumes, no copy.
//   write view (src/minicpm.cpp:222-236): [head_dim, n_kv_heads, n_tokens] with nb1 = the
//               cache's head stride and nb2 = its token stride, offset start * token stride
//               -- what ggml_cpy(k_cur, view) fills.
// vx_kv_store is that ggml_cpy: F32 rows in, cache-typed rows out (F32 -> F16 rounds to
// nearest even, as ggml-cpu's conversion does).  Pure index arithmetic plus one rounding.
#include "vx_common.hpp"

namespace {

template <typename T>
__global__ __launch_bounds__(256) void kv_store_kernel(const char * __restrict__ src, char * __restrict__ dst,
                                                       vx_dims s, vx_dims d) {
    const int64_t n   = s.ne[0] * s.ne[1] * s.ne[2] * s.ne[3];
    const int64_t gid = (int64_t) blockIdx.x * blockDim.x + threadIdx.x;
    if (gid >= n) return;
    const int64_t i0 = gid % s.ne[0];
    const int64_t i1 = (gid / s.ne[0]) % s.ne[1];
    const int64_t i2 = (gid / (s.ne[0] * s.ne[1])) % s.ne[2];
    const int64_t i3 = gid / (s.ne[0] * s.ne[1] * s.ne[2]);
    const float   x  = *(const float *) (src + i0 * 4 + i1 * s.nb[1] + i2 * s.nb[2] + i3 * s.nb[3]);
    *(T *) (dst + i0 * sizeof(T) + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]) = (T) x;
}

bool is_cache(const vx_tensor * c) {
    return c && (c->type == VX_TYPE_F16 || c->type == VX_TYPE_F32) && c->ne[0] > 0 && c->ne[1] > 0 && c->ne[2] > 0 &&
           c->ne[3] == 1 && c->nb[0] == vx_type_size(c->type);
}

} // namespace

extern "C" vx_status vx_kv_read_view(const vx_tensor * cache, int seq_len, vx_tensor * view) {
    if (!is_cache(cache) || !view) return vx_fail(VX_ERR_INVALID, "kv_read_view: cache must be a 3-d F16/F32 tensor");
    if (seq_len < 0 || seq_len > cache->ne[1]) return vx_fail(VX_ERR_INVALID, "kv_read_view: seq_len %d outside 0..%lld", seq_len, (long long) cache->ne[1]);
    *view       = *cache;
    view->ne[1] = seq_len;
    return VX_OK;
}

extern "C" vx_status vx_kv_write_view(const vx_tensor * cache, int start, int n_tokens, vx_tensor * view) {
    if (!is_cache(cache) || !view) return vx_fail(VX_ERR_INVALID, "kv_write_view: cache must be a 3-d F16/F32 tensor");
    if (start < 0 || n_tokens < 0 || (int64_t) start + n_tokens > cache->ne[1])
        return vx_fail(VX_ERR_INVALID, "kv_write_view: tokens %d..%d outside the cache (max_length %lld)", start, start + n_tokens, (long long) cache->ne[1]);
    view->type  = cache->type;
    view->_pad  = 0;
    view->ne[0] = cache->ne[0];
    view->ne[1] = cache->ne[2];
    view->ne[2] = n_tokens;
    view->ne[3] = 1;
    view->nb[0] = cache->nb[0];
    view->nb[1] = cache->nb[2];
    view->nb[2] = cache->nb[1];
    view->nb[3] = cache->nb[1] * (uint64_t) n_tokens;
    view->data  = cache->data ? (char *) cache->data + (uint64_t) start * cache->nb[1] : nullptr;
    return VX_OK;
}

extern "C" vx_status vx_kv_store(const vx_tensor * src, const vx_tensor * view, vx_stream stream) {
    if (!src || !view || !src->data || !view->data) return vx_fail(VX_ERR_INVALID, "kv_store: null tensor");
    if (src->type != VX_TYPE_F32 || src->nb[0] != 4) return vx_fail(VX_ERR_UNSUPPORTED, "kv_store: src must be F32 with dense rows");
    if (view->type != VX_TYPE_F16 && view->type != VX_TYPE_F32) return vx_fail(VX_ERR_UNSUPPORTED, "kv_store: cache must be F16 or F32");
    if (!vx_same_shape(src, view)) return vx_fail(VX_ERR_INVALID, "kv_store: shapes differ");
    const int64_t n = vx_nelements(src);
    if (n == 0) return VX_OK;
    if (n < 0 || (n + 255) / 256 > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "kv_store: too many elements");
    const dim3 grid((unsigned) ((n + 255) / 256)), block(256);
    if (view->type == VX_TYPE_F16)
        vx_launch(kv_store_kernel<_Float16>, grid, block, 0, (hipStream_t) stream, (const char *) src->data, (char *) view->data, vx_dims_of(src), vx_dims_of(view));
    else
        vx_launch(kv_store_kernel<float>, grid, block, 0, (hipStream_t) stream, (const char *) src->data, (char *) view->data, vx_dims_of(src), vx_dims_of(view));
    VX_LAUNCH_CHECK();
    return VX_OK;
}
