// kvs_common.hpp -- the cache write of attention_forward with its ordering sums, shared by the one-block
// kernel that runs the whole nine-node group and by the attention merge kernel that folds the group in.
#pragma once
#include "vx_common.hpp"

// one cache write: source tensor (F32, any strides) -> slot view of the cache (F32 or F16, dense rows); element i
// of the source in its own row-major order goes to element i of the slot in the slot's.  With an F16 cache the value
// is rounded to nearest even on the way (what GGML_OP_CPY does) and the ordering sum adds the ROUNDED values in fp64:
// the sum of the slot read back as F32, i.e. of the node sequence CPY(k, slot) , CPY(slot -> F32) , SUM.
struct kvs_side {
    const char * s; char * d;
    int64_t  nes[4], ned[4];
    uint64_t nbs[4], nbd[4];
    int vec; // units of 4 elements: the test vx_sum applies to the tensor it sums (the slot view, or its dense F32 copy)
    int src_dense; // the source is contiguous in its own order (element i at byte 4 i) and 16-byte aligned
    int dst_f16;
};

// host side: what one cache write may look like, and its kernel argument
static inline bool kvs_side_ok(const vx_tensor * src, const vx_tensor * slot, int64_t max_elements = 16384) {
    if (!src || !slot || src->type != VX_TYPE_F32 || (slot->type != VX_TYPE_F32 && slot->type != VX_TYPE_F16) || !vx_positive(src)) return false;
    if (vx_nelements(src) != vx_nelements(slot) || vx_nelements(src) > max_elements) return false;
    for (int i = 0; i < 4; ++i) if (src->nb[i] % 4) return false;
    if (slot->type == VX_TYPE_F16) {
        // the sum is taken over a dense F32 copy of the slot (vx_sum's 4-element units need ne0 % 4 == 0 only); the
        // stores are 8 bytes wide
        if (slot->nb[0] != 2 || slot->ne[0] % 4 || (uintptr_t) slot->data % 8) return false;
        for (int i = 1; i < 4; ++i) if (slot->nb[i] % 8) return false;
        return true;
    }
    for (int i = 0; i < 4; ++i) if (slot->nb[i] % 4) return false;
    return slot->nb[0] == 4;
}
static inline void kvs_side_fill(kvs_side & o, const vx_tensor * src, const vx_tensor * slot) {
    o.s = (const char *) src->data; o.d = (char *) slot->data;
    for (int i = 0; i < 4; ++i) { o.nes[i] = src->ne[i]; o.ned[i] = slot->ne[i]; o.nbs[i] = src->nb[i]; o.nbd[i] = slot->nb[i]; }
    o.dst_f16 = slot->type == VX_TYPE_F16;
    o.vec = slot->ne[0] % 4 == 0 && (uintptr_t) slot->data % 16 == 0 && slot->nb[1] % 16 == 0 && slot->nb[2] % 16 == 0 && slot->nb[3] % 16 == 0;
    if (o.dst_f16) o.vec = 1; // kvs_side_ok has checked what the 8-byte stores need
    o.src_dense = vx_is_contiguous(src) && (uintptr_t) src->data % 16 == 0;
}

#ifdef __HIPCC__
// Unit e of the slot (4 consecutive elements when VEC, else one): fetch from the source, optionally store,
// add to acc in element order -- the inner step of GGML_OP_SUM's walk over the written slot.
// (fetch and the rest are separate so that a caller can have several units' loads in flight)
template <bool VEC>
__device__ __forceinline__ void kvs_fetch(const kvs_side & a, uint32_t e, float (&v)[VEC ? 4 : 1]) {
    constexpr int W = VEC ? 4 : 1;
    if (a.src_dense) { // no index arithmetic: unit e holds elements e W .. e W + W - 1 of the source
        const float * ps = (const float *) a.s + (size_t) e * W;
        if constexpr (VEC) { const float4_t t = *(const float4_t *) ps; v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3]; }
        else               { v[0] = *ps; }
    } else {
        const uint32_t s0n = (uint32_t) a.nes[0], s1n = (uint32_t) a.nes[1], s2n = (uint32_t) a.nes[2];
#pragma unroll
        for (int k = 0; k < W; ++k) { // element number e W + k of the source, in its own shape
            uint32_t r = e * W + k;
            const uint32_t j0 = r % s0n; r /= s0n;
            const uint32_t j1 = r % s1n; r /= s1n;
            const uint32_t j2 = r % s2n, j3 = r / s2n;
            v[k] = *(const float *) (a.s + j0 * a.nbs[0] + j1 * a.nbs[1] + j2 * a.nbs[2] + j3 * a.nbs[3]);
        }
    }
}
template <bool VEC>
__device__ __forceinline__ void kvs_apply(const kvs_side & a, uint32_t e, bool store, float (&v)[VEC ? 4 : 1], double & acc) {
    constexpr int W = VEC ? 4 : 1;
    const uint32_t ne0 = (uint32_t) a.ned[0], per_row = ne0 / W;
    _Float16 h[W];
    if (a.dst_f16) { // uniform: the slot holds halves; the sum below sees what a reader of the slot would
#pragma unroll
        for (int k = 0; k < W; ++k) { h[k] = (_Float16) v[k]; v[k] = (float) h[k]; }
    }
    if (store) {
        const uint32_t ne1 = (uint32_t) a.ned[1], ne2 = (uint32_t) a.ned[2];
        const uint32_t row = e / per_row, iv = e - row * per_row;
        const uint32_t i1 = row % ne1, r2 = row / ne1, i2 = r2 % ne2, i3 = r2 / ne2;
        if (a.dst_f16) {
            char * pd = a.d + (uint64_t) iv * (2 * W) + i1 * a.nbd[1] + i2 * a.nbd[2] + i3 * a.nbd[3];
            if constexpr (VEC) *(half4_t *) pd = half4_t{h[0], h[1], h[2], h[3]};
            else               *(_Float16 *) pd = h[0];
        } else {
            char * pd = a.d + (uint64_t) iv * (4 * W) + i1 * a.nbd[1] + i2 * a.nbd[2] + i3 * a.nbd[3];
            if constexpr (VEC) *(float4_t *) pd = float4_t{v[0], v[1], v[2], v[3]};
            else               *(float *) pd = v[0];
        }
    }
#pragma unroll
    for (int k = 0; k < W; ++k) acc += (double) v[k];
}
template <bool VEC>
__device__ __forceinline__ void kvs_unit(const kvs_side & a, uint32_t e, bool store, double & acc) {
    float v[VEC ? 4 : 1];
    kvs_fetch<VEC>(a, e, v);
    kvs_apply<VEC>(a, e, store, v, acc);
}

__device__ __forceinline__ uint32_t kvs_units(const kvs_side & a, bool vec) {
    return (uint32_t) (a.ned[0] / (vec ? 4 : 1)) * (uint32_t) (a.ned[1] * a.ned[2] * a.ned[3]);
}

// The sum of a cache write as GGML_OP_SUM's kernels form it, by one wave.  Small writes: the one-wave order itself.
// Larger ones: a 1024-thread block's order (thread t walks units t, t + 1024, ...; each wave reduces by xor
// butterfly; the 16 wave totals are added in order), replayed wave by wave: the same additions in the same order.
template <bool VEC>
__device__ __forceinline__ double kvs_wave_total(const kvs_side & a, int lane, bool store) {
    const uint32_t n = kvs_units(a, VEC);
    if (n <= VX_SUM_ONE_WAVE_UNITS) {
        double acc = 0.0;
        for (uint32_t e = lane; e < n; e += 64) kvs_unit<VEC>(a, e, store, acc);
        return vx_wave_sum(acc);
    }
    double total = 0.0;
    int w = 0;
    for (; w < 16; ++w) {
        if ((uint32_t) w * 64 >= n) break; // the remaining waves of the block would hold no unit
        double acc = 0.0;
        for (uint32_t e = (uint32_t) w * 64 + lane; e < n; e += 1024) kvs_unit<VEC>(a, e, store, acc);
        total += vx_wave_sum(acc);
    }
    if (w < 16) total += 0.0; // their zeros, added once (it only matters for the sign of a zero total)
    return total;
}

// both cache writes of a step at once: the two sides' loads are in flight together
template <bool VK, bool VV>
__device__ __forceinline__ void kvs_wave_totals(const kvs_side & k, const kvs_side & v, int lane, bool store, double & tk, double & tv) {
    const uint32_t nk = kvs_units(k, VK), nv = kvs_units(v, VV);
    if (nk <= VX_SUM_ONE_WAVE_UNITS && nv <= VX_SUM_ONE_WAVE_UNITS) { // both in the one-wave order, loads side by side
        double ak = 0.0, av = 0.0;
        const uint32_t nmax = nk > nv ? nk : nv;
        // eight units of each side requested together, then taken in order: a lane's units arrive in one trip instead
        // of one trip each (sixteen streams write 512 units per side: 8 per lane; a trip to values another XCD wrote is
        // 1.5 us here)
        constexpr int UB = 8;
        for (uint32_t base = lane; base < nmax; base += 64 * UB) {
            float fk[UB][VK ? 4 : 1], fv[UB][VV ? 4 : 1];
#pragma unroll
            for (int i = 0; i < UB; ++i) {
                const uint32_t e = base + 64 * i;
                if (e < nk) kvs_fetch<VK>(k, e, fk[i]);
                if (e < nv) kvs_fetch<VV>(v, e, fv[i]);
            }
#pragma unroll
            for (int i = 0; i < UB; ++i) {
                const uint32_t e = base + 64 * i;
                if (e < nk) kvs_apply<VK>(k, e, store, fk[i], ak);
                if (e < nv) kvs_apply<VV>(v, e, store, fv[i], av);
            }
        }
        tk = vx_wave_sum(ak);
        tv = vx_wave_sum(av);
        return;
    }
    if (nk <= VX_SUM_ONE_WAVE_UNITS || nv <= VX_SUM_ONE_WAVE_UNITS) { // mixed sizes: each side in its own order
        tk = kvs_wave_total<VK>(k, lane, store);
        tv = kvs_wave_total<VV>(v, lane, store);
        return;
    }
    tk = 0.0; tv = 0.0;
    int wk = 0, wv = 0;
    for (int w = 0; w < 16; ++w) {
        const bool dk = (uint32_t) w * 64 < nk, dv = (uint32_t) w * 64 < nv; // uniform
        if (!dk && !dv) break;
        double ak = 0.0, av = 0.0;
        if (dk) for (uint32_t e = (uint32_t) w * 64 + lane; e < nk; e += 1024) kvs_unit<VK>(k, e, store, ak);
        if (dv) for (uint32_t e = (uint32_t) w * 64 + lane; e < nv; e += 1024) kvs_unit<VV>(v, e, store, av);
        if (dk) { tk += vx_wave_sum(ak); ++wk; }
        if (dv) { tv += vx_wave_sum(av); ++wv; }
    }
    if (wk < 16) tk += 0.0; // the zeros of the block's idle waves, added once (sign of a zero total)
    if (wv < 16) tv += 0.0;
}

// the scalar the reference adds to the attention output: (sum(k_slot) + sum(v_slot)) * scale + bias
__device__ __forceinline__ float kvs_scalar(float sk, float sv, float scale, float bias) {
    const float t = sk + sv;                                       // the ADD node
    return bias == 0.0f ? t * scale : fmaf(t, scale, bias);        // the SCALE node
}
#endif
