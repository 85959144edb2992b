// vx_common.hpp -- shared host/device helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <tuple>
#include <utility>

#include "../../include/voxcpm_gfx950.h"

#define VX_WAVE 64
#define VX_QK8_0 32
#define VX_Q8_BLOCK 34 /* bytes: f16 d + 32 int8 */

// ---- error plumbing -------------------------------------------------------------------
void       vx_set_error(const char * fmt, ...) __attribute__((format(printf, 1, 2)));
vx_status  vx_fail(vx_status st, const char * fmt, ...) __attribute__((format(printf, 2, 3)));

#define VX_HIP(call)                                                                         \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess)                                                                \
            return vx_fail(VX_ERR_HIP, "%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), \
                           __FILE__, __LINE__);                                              \
    } while (0)

#define VX_LAUNCH_CHECK()                                                                    \
    do {                                                                                     \
        hipError_t e_ = hipGetLastError();                                                   \
        if (e_ != hipSuccess)                                                                \
            return vx_fail(VX_ERR_HIP, "kernel launch failed: %s (%s:%d)",                   \
                           hipGetErrorString(e_), __FILE__, __LINE__);                       \
    } while (0)

// ---- launching --------------------------------------------------------------------------------------------------------
// Every kernel of the operators goes to the GPU through vx_launch, so that a recording made between vx_graph_begin and
// vx_graph_end knows its launches one by one (function, grid, block, LDS bytes, argument bytes), and so that a later run
// of the same operators can be compared with it without launching anything (vx_graph_patch_begin): the launches whose
// arguments differ are then set on the recorded graph, and one hipGraphLaunch issues them all.
//   0  launch;   1  launch (into the capture) and note;   2  compare with the recording, launch nothing
extern thread_local int vx_tl_launch_mode;
void vx_launch_note(const void * func, dim3 grid, dim3 block, size_t lds_bytes, void * const * params, const size_t * sizes, int n_params);

template <typename... P, size_t... I>
inline void vx_launch_note_tuple(const void * func, dim3 grid, dim3 block, size_t lds_bytes, std::tuple<P...> & vals, std::index_sequence<I...>) {
    void * const        ptrs[]  = { (void *) &std::get<I>(vals)... };
    static const size_t sizes[] = { sizeof(P)... };
    vx_launch_note(func, grid, block, lds_bytes, ptrs, sizes, (int) sizeof...(P));
}
template <typename... P, typename... A>
inline void vx_launch(void (*kernel)(P...), dim3 grid, dim3 block, size_t lds_bytes, hipStream_t stream, const A &... args) {
    static_assert(sizeof...(P) == sizeof...(A) && sizeof...(P) > 0, "one argument per kernel parameter");
    if (__builtin_expect(vx_tl_launch_mode != 0, 0)) {
        std::tuple<P...> vals(args...); // converted to the kernel's own parameter types, as the launch would
        vx_launch_note_tuple((const void *) kernel, grid, block, lds_bytes, vals, std::index_sequence_for<P...>{});
        if (vx_tl_launch_mode == 2) return;
    }
    kernel<<<grid, block, lds_bytes, stream>>>(args...);
}

// per-stream scratch memory, grown on demand.  A block stays allocated at its address until the stream is
// destroyed, also after a larger one has replaced it (ws_policy.hpp), so launches already queued and graphs
// already captured keep valid arguments; growth during a stream capture is refused.
vx_status vx_workspace(hipStream_t stream, size_t bytes, void ** ptr);

// Copies derived from pinned weights (vx_weights_pin), kept from call to call.  vx_derived_get returns the copy for `key`
// (the calling stream is made to wait for the kernel that filled it, if that ran on another stream), or a new block of
// `bytes` with *fresh set -- the caller then fills it on `stream` and calls vx_derived_filled -- or null: the weights are
// not pinned, launches are being recorded or compared, the stream is under capture, or the budget is spent.
struct vx_derived_key {
    int          dev;
    int          kind;     // which layout (and variant of it)
    const void * w;
    const void * w2;       // second matrix of a pair, or null
    int64_t      K, M;
    uint64_t     nb01;
};
void * vx_derived_get(const vx_derived_key & key, size_t bytes, hipStream_t stream, bool * fresh);
void   vx_derived_filled(const vx_derived_key & key, hipStream_t stream);
void   vx_derived_abandon(const vx_derived_key & key, hipStream_t stream); // a fresh block that will not be filled after all

// vx_flash_attn_ext_static's fixed scratch array (fattn.hip): the per-device address lookup that vx_init performs
// so that the first call of the entry point does no set-up work
vx_status vx_fattn_static_setup(void);

// Work that a caller of vx_fattn_prefill wants launched in front of the attention's own kernels, with a piece of the
// call's workspace block to itself: `bytes` (a multiple of 256) at the front of the block, handed to `launch` once the
// block is known; the float at `addend_at` bytes into it is then the attention's addend.
struct vx_pf_front {
    size_t bytes, addend_at;
    vx_status (*launch)(void * front, void * ctx, hipStream_t stream);
    void * ctx;
    // optionally the result leaves as the pre-tiled product kernel's f16 activation tiles (k = head * 64 + d) at
    // tiles_at bytes into the front instead of being stored to dst: tile_tt 16-token tiles per k block; tile_bs tiles
    // per batch entry (0: the sequences are flattened into one token dimension, tile_ts tokens apart)
    bool     tiles;
    size_t   tiles_at;
    uint32_t tile_tt, tile_bs, tile_ts;
};

// LDS-tiled prefill kernel (fattn_prefill.hip); VX_ERR_UNSUPPORTED means "use the general kernel"
vx_status vx_fattn_prefill(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                           const float * sinks, const float * addend, const vx_tensor * dst, float scale, float max_bias,
                           float logit_softcap, hipStream_t stream, const vx_pf_front * front = nullptr);

// A Q8_0 projection with its residual update (vx_mul_mat_scale_add) over activations that a kernel in front of it left
// as the pre-tiled kernel's f16 tiles in the stream's workspace (mul_mat.hip).  x describes the F32 activations the
// separate call would read (only shape and strides are looked at).  _ok: the separate call would run on the pre-tiled
// kernel; it reports the tile geometry.  _run: tiles at `tiles`, the first ws_offset bytes of the workspace are the caller's.
bool      vx_proj_tiles_ok(const vx_tensor * w, const vx_tensor * x, const vx_tensor * residual, const vx_tensor * dst, int act_mode,
                           uint32_t * tile_tt, uint32_t * n_kb, size_t * tile_bytes, size_t * own_bytes);
vx_status vx_proj_tiles_run(const vx_tensor * w, const vx_tensor * x, const vx_tensor * residual, const vx_tensor * dst, float scale,
                            int act_mode, const void * tiles, size_t ws_offset, hipStream_t stream);

// vx_kv_store_sync's cache write and ordering scalar without the ADD1 (glue.hip): the scalar is left in *y_out
// (device memory), partials are 2 KiB of device memory
bool      vx_kv_store_scalar_ok(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot);
vx_status vx_kv_store_scalar(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot,
                             float scale, float bias, void * partials, float * y_out, hipStream_t stream);

// whether vx_fattn_prefill would take this shape (k describes all keys)
bool vx_fattn_prefill_accepts(const vx_tensor * q, const vx_tensor * k, float logit_softcap);

// ---- host-side tensor predicates ---------------------------------------------------------
static inline size_t vx_type_size(int type) {
    switch (type) {
        case VX_TYPE_F32: return 4;
        case VX_TYPE_F16: return 2;
        case VX_TYPE_I32: return 4;
        case VX_TYPE_Q8_0: return VX_Q8_BLOCK;
        default: return 0;
    }
}
static inline int64_t vx_blck(int type) { return type == VX_TYPE_Q8_0 ? VX_QK8_0 : 1; }
static inline size_t  vx_row_size(int type, int64_t ne0) { return vx_type_size(type) * (size_t)(ne0 / vx_blck(type)); }
static inline int64_t vx_nelements(const vx_tensor * t) { return t->ne[0] * t->ne[1] * t->ne[2] * t->ne[3]; }
static inline int64_t vx_nrows(const vx_tensor * t) { return t->ne[1] * t->ne[2] * t->ne[3]; }
static inline bool vx_same_shape(const vx_tensor * a, const vx_tensor * b) {
    return a->ne[0] == b->ne[0] && a->ne[1] == b->ne[1] && a->ne[2] == b->ne[2] && a->ne[3] == b->ne[3];
}
static inline bool vx_is_contiguous(const vx_tensor * t) {
    size_t nb = vx_type_size(t->type);
    if (t->nb[0] != nb) return false;
    nb = vx_row_size(t->type, t->ne[0]);
    for (int i = 1; i < 4; ++i) {
        if (t->ne[i] != 1 && t->nb[i] != nb) return false;
        nb *= (size_t) t->ne[i];
    }
    return true;
}
static inline bool vx_positive(const vx_tensor * t) {
    return t->ne[0] > 0 && t->ne[1] > 0 && t->ne[2] > 0 && t->ne[3] > 0;
}

// GGML_OP_SUM over at most this many units (a unit = 4 consecutive elements of a dense, 16-byte aligned row, else
// one element) is formed by ONE wave: lane l adds units l, l + 64, ... in fp64, then one xor butterfly.  Every
// kernel that forms such a sum (the SUM kernel, the cache-write group, the attention merge) uses this order.
#define VX_SUM_ONE_WAVE_UNITS 1024

// ---- device helpers ------------------------------------------------------------------------
#ifdef __HIPCC__

// 4-d strides passed to kernels by value
struct vx_dims {
    int64_t  ne[4];
    uint64_t nb[4];
};
static inline vx_dims vx_dims_of(const vx_tensor * t) {
    vx_dims d;
    for (int i = 0; i < 4; ++i) { d.ne[i] = t->ne[i]; d.nb[i] = t->nb[i]; }
    return d;
}

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef float    float4_t __attribute__((ext_vector_type(4)));
typedef float    float16_t __attribute__((ext_vector_type(16)));
typedef int      int4_t __attribute__((ext_vector_type(4)));

// The value of lane (i + N) mod 16 of the same row of 16 lanes, by a DPP move (a register read; a lane exchange through
// LDS hardware costs a round trip of a hundred cycles).  In a butterfly sum whose steps run 32, 16, 8, 4, 2, 1 the steps
// 8 .. 1 may take it in place of the xor partner: when step s is reached the values repeat every 2 s lanes, and i + s and
// i ^ s differ by 0 or 2 s -- the same bits are added in the same order.
template <int N>
__device__ __forceinline__ float vx_row_ror(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x120 + N, 0xf, 0xf, false));
}
template <int N>
__device__ __forceinline__ double vx_row_ror(double v) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), 0x120 + N, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), 0x120 + N, 0xf, 0xf, false);
    return __hiloint2double(hi, lo);
}
template <typename T>
__device__ __forceinline__ T vx_wave_sum_t(T v) {
    v += __shfl_xor(v, 32, 64);
    v += __shfl_xor(v, 16, 64);
    v += vx_row_ror<8>(v);
    v += vx_row_ror<4>(v);
    v += vx_row_ror<2>(v);
    v += vx_row_ror<1>(v);
    return v;
}
__device__ __forceinline__ float  vx_wave_sum(float v)  { return vx_wave_sum_t(v); }
__device__ __forceinline__ double vx_wave_sum(double v) { return vx_wave_sum_t(v); }
// 1 / rms of one dense, 16-byte aligned row of ne00 <= 2048 floats, by one wave, exactly as the RMS_NORM
// kernel's wave-per-row path forms it: fp32 squares, fp64 lane sums in float4 order, xor butterfly, one
// rounding of the mean to fp32.  The same value in every lane.
// The load and the arithmetic are separate so that a caller can request the row ahead of other traffic.
struct vx_rms_row { float4 v[8]; };
__device__ __forceinline__ void vx_rms_row_load(vx_rms_row & r, const float * x, int64_t ne00, int lane) {
    const int64_t nvec = ne00 / 4;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int64_t iv = lane + (int64_t) c * 64;
        r.v[c] = iv < nvec ? ((const float4 *) x)[iv] : float4{0.0f, 0.0f, 0.0f, 0.0f};
    }
}
__device__ __forceinline__ double vx_rms_row_lane_sum(const vx_rms_row & r, int64_t ne00, int lane) {
    const int64_t nvec = ne00 / 4;
    double sum = 0.0;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const int64_t iv = lane + (int64_t) c * 64;
        if (iv < nvec) {
            const float4 v = r.v[c];
            sum += (double) (v.x * v.x);
            sum += (double) (v.y * v.y);
            sum += (double) (v.z * v.z);
            sum += (double) (v.w * v.w);
        }
    }
    return sum;
}
__device__ __forceinline__ float vx_rms_finish(double sum, int64_t ne00, float eps) {
    // a row length that is a power of two (the usual case) divides by a change of exponent: the same quotient as the
    // division, which costs some forty fp64 instructions
    const bool  pow2 = (ne00 & (ne00 - 1)) == 0;
    const float mean = pow2 ? (float) ldexp(sum, -(63 - __clzll((long long) ne00))) : (float) (sum / (double) ne00);
    return 1.0f / sqrtf(mean + eps);
}
__device__ __forceinline__ float vx_rms_row_scale(const vx_rms_row & r, int64_t ne00, int lane, float eps) {
    return vx_rms_finish(vx_wave_sum(vx_rms_row_lane_sum(r, ne00, lane)), ne00, eps);
}
// two rows by one wave: the same arithmetic per row, the two cross-lane chains issued side by side
__device__ __forceinline__ void vx_rms_row_scale2(const vx_rms_row & r1, const vx_rms_row & r2, int64_t ne00, int lane, float eps,
                                                  float & s1, float & s2) {
    double a = vx_rms_row_lane_sum(r1, ne00, lane), b = vx_rms_row_lane_sum(r2, ne00, lane);
#pragma unroll
    for (int off = 32; off > 8; off >>= 1) {
        const double ta = __shfl_xor(a, off, 64), tb = __shfl_xor(b, off, 64);
        a += ta;
        b += tb;
    }
    { const double ta = vx_row_ror<8>(a), tb = vx_row_ror<8>(b); a += ta; b += tb; }
    { const double ta = vx_row_ror<4>(a), tb = vx_row_ror<4>(b); a += ta; b += tb; }
    { const double ta = vx_row_ror<2>(a), tb = vx_row_ror<2>(b); a += ta; b += tb; }
    { const double ta = vx_row_ror<1>(a), tb = vx_row_ror<1>(b); a += ta; b += tb; }
    s1 = vx_rms_finish(a, ne00, eps);
    s2 = vx_rms_finish(b, ne00, eps);
}
__device__ __forceinline__ float vx_rms_scale_wave(const float * x, int64_t ne00, int lane, float eps) {
    vx_rms_row r;
    vx_rms_row_load(r, x, ne00, lane);
    return vx_rms_row_scale(r, ne00, lane, eps);
}
__device__ __forceinline__ float vx_wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 8; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    v = fmaxf(v, vx_row_ror<8>(v));
    v = fmaxf(v, vx_row_ror<4>(v));
    v = fmaxf(v, vx_row_ror<2>(v));
    v = fmaxf(v, vx_row_ror<1>(v));
    return v;
}

// ALiBi slope of head h (ggml/src/ggml-cpu/ops.cpp:8177-8200); m0, m1 computed on the host
__device__ __forceinline__ float vx_alibi_slope(float max_bias, uint32_t h, uint32_t n_head_log2, float m0, float m1) {
    if (!(max_bias > 0.0f)) return 1.0f;
    return h < n_head_log2 ? powf(m0, (float)(h + 1)) : powf(m1, (float)(2 * (h - n_head_log2) + 1));
}

#endif // __HIPCC__
