// fattn.hip -- GGML_OP_FLASH_ATTN_EXT on gfx950: the column-packed wave kernel (decode,
// LocDiT-sized sequences, and the general fallback) plus the split-KV combine.
//
// Work decomposition.  For one batch element b and one KV head g, every (query row iq1,
// query head of the GQA group) pair is a *column*: col = iq1 * gqa + head_in_group.  A
// wavefront owns 16 consecutive columns -- in decode that is the 8 query heads sharing the
// KV head (x2 rows when n_q = 2), in LocDiT 2 rows x 8 heads -- and one contiguous range
// of keys (a split).  Everything a wave needs stays in its registers: there is no LDS and
// no barrier, so waves retire independently and occupancy alone hides HBM latency.
//
// MFMA formulation (v_mfma_f32_16x16x32_f16, lane = 16*j + c):
//   S^T = K * Q^T      A = K rows as they lie in memory (lane c = key, 8 consecutive d per
//                      k-slot), B = Q^T (lane c = column).  The result puts 4 consecutive
//                      keys of column c in lane (j, c): the softmax statistics of a column
//                      are lane-local plus two cross-lane steps (xor 16, xor 32).
//   O^T += V^T * P^T   B = P^T is fed straight from the S^T accumulator registers (keys
//                      4j..4j+3 of both 16-key halves = the 8 k-slots of lane-group j), so
//                      probabilities never leave registers.  A = V^T needs 8 *keys* of one
//                      d per lane while memory has 8 *d* of one key; the transpose is done
//                      by the matrix core itself: V (as it lies in memory) times a 0/1
//                      selection matrix lands V^T in accumulator layout, exactly, and a
//                      convert makes it the A operand.  Matrix throughput is ~6x what HBM
//                      can feed in this regime, so spending it on the transpose is free.
// Precision: Q, P (and K, V when they are F32) are split into f16 hi + lo parts and both
// parts multiplied, so the products carry ~22 bits; accumulation and softmax are fp32.
//
// Algorithmic HBM bytes: each K and V element is read once per 16-column tile; in decode
// (one tile per KV head) that is n_kv * D * 2 * sizeof(kv) per (b, g), the figure the
// benchmark divides by.
#include "vx_common.hpp"

#include <cmath>

namespace {

struct fa_args {
    const char * q; const char * k; const char * v; const char * mask;
    const float * sinks;
    float * dst;
    float * part_o;  // [gcol][split][D]
    float * part_ml; // [gcol][split][2]
    uint64_t nbq1, nbq2, nbq3, nbk1, nbk2, nbk3, nbv1, nbv2, nbv3, nbm1, nbm2, nbm3;
    int n_q, n_kv, Hq, Hkv, gqa, ne3, rk3, nem2, nem3;
    int n_col_tiles, n_splits, chunk;
    float scale, softcap, max_bias, m0, m1;
    uint32_t n_head_log2;
};

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// 8 consecutive elements -> f16 hi (+ lo) operand
template <bool F32> struct kv_load;
template <> struct kv_load<false> {
    static __device__ __forceinline__ void run(const char * p, half8_t & hi, half8_t & lo) {
        hi = *(const half8_t *) p;
        (void) lo;
    }
};
template <> struct kv_load<true> {
    static __device__ __forceinline__ void run(const char * p, half8_t & hi, half8_t & lo) {
        const float4_t a = ((const float4_t *) p)[0], b = ((const float4_t *) p)[1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            hi[i]     = (_Float16) a[i];
            lo[i]     = (_Float16) (a[i] - (float) hi[i]);
            hi[4 + i] = (_Float16) b[i];
            lo[4 + i] = (_Float16) (b[i] - (float) hi[4 + i]);
        }
    }
};

template <int D, bool KV_F32>
__global__ __launch_bounds__(64) void fattn_cols16_kernel(const fa_args a) {
    constexpr int NP  = D / 32;          // MFMAs along the head dimension
    constexpr int SEG = D / 4;           // elements of a row owned by lane-group j
    constexpr int ES  = KV_F32 ? 4 : 2;  // bytes per K/V element

    const int lane = threadIdx.x;
    const int j = lane >> 4, c = lane & 15;

    int w = blockIdx.x;
    const int ct = w % a.n_col_tiles; w /= a.n_col_tiles;
    const int sp = w % a.n_splits;    w /= a.n_splits;
    const int g  = w % a.Hkv;
    const int b  = w / a.Hkv;

    const int  ncols  = a.n_q * a.gqa;
    const int  col    = ct * 16 + c;
    const bool col_ok = col < ncols;
    const int  iq1    = col_ok ? col / a.gqa : 0;
    const int  head   = g * a.gqa + (col_ok ? col % a.gqa : 0);

    // ---- Q^T operand: column c, elements d = SEG*j + 8p + i, split into hi + lo
    half8_t qhi[NP], qlo[NP];
    {
        const float * qp = (const float *) (a.q + (uint64_t) iq1 * a.nbq1 + (uint64_t) head * a.nbq2 + (uint64_t) b * a.nbq3) + SEG * j;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            float4_t x0 = {0, 0, 0, 0}, x1 = {0, 0, 0, 0};
            if (col_ok) { x0 = ((const float4_t *) (qp + 8 * p))[0]; x1 = ((const float4_t *) (qp + 8 * p))[1]; }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qhi[p][i]     = (_Float16) x0[i];
                qlo[p][i]     = (_Float16) (x0[i] - (float) qhi[p][i]);
                qhi[p][4 + i] = (_Float16) x1[i];
                qlo[p][4 + i] = (_Float16) (x1[i] - (float) qhi[p][4 + i]);
            }
        }
    }

    // ---- selection matrices for the V transpose: SEL_u[k-slot (j,i)][n] = 1 iff
    //      j == 2u + n/8 and i == n%8, so column n of the product picks d = SEG*(2u+n/8) + 8p + n%8
    half8_t sel[2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int i = 0; i < 8; ++i) sel[u][i] = (j == 2 * u + (c >> 3) && i == (c & 7)) ? (_Float16) 1.0f : (_Float16) 0.0f;

    const float slope = vx_alibi_slope(a.max_bias, (uint32_t) head, a.n_head_log2, a.m0, a.m1);
    const char * mrow = a.mask ? a.mask + (uint64_t) iq1 * a.nbm1 + (uint64_t) (head % a.nem2) * a.nbm2 + (uint64_t) (b % a.nem3) * a.nbm3 : nullptr;

    const char * kbase = a.k + (uint64_t) g * a.nbk2 + (uint64_t) (b / a.rk3) * a.nbk3 + (uint64_t) (SEG * j) * ES;
    const char * vbase = a.v + (uint64_t) g * a.nbv2 + (uint64_t) (b / a.rk3) * a.nbv3 + (uint64_t) (SEG * j) * ES;

    const int kv0 = sp * a.chunk;
    const int kv1 = min(a.n_kv, kv0 + a.chunk);

    float4_t o[NP][2];
#pragma unroll
    for (int p = 0; p < NP; ++p) { o[p][0] = float4_t{0, 0, 0, 0}; o[p][1] = float4_t{0, 0, 0, 0}; }
    float m = -INFINITY; // running max of column c (identical in the 4 lanes of a column)
    float l = 0.0f;      // this lane's share of the running sum

    for (int kb = kv0; kb < kv1; kb += 32) {
        // rows this lane loads (as MFMA row c of each 16-key half); clamped, masked out below
        const int key0 = min(kb + c, a.n_kv - 1), key1 = min(kb + 16 + c, a.n_kv - 1);

        half8_t khi[2][NP], klo[2][NP], vhi[2][NP], vlo[2][NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            kv_load<KV_F32>::run(kbase + (uint64_t) key0 * a.nbk1 + p * 8 * ES, khi[0][p], klo[0][p]);
            kv_load<KV_F32>::run(kbase + (uint64_t) key1 * a.nbk1 + p * 8 * ES, khi[1][p], klo[1][p]);
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            kv_load<KV_F32>::run(vbase + (uint64_t) key0 * a.nbv1 + p * 8 * ES, vhi[0][p], vlo[0][p]);
            kv_load<KV_F32>::run(vbase + (uint64_t) key1 * a.nbv1 + p * 8 * ES, vhi[1][p], vlo[1][p]);
        }

        // ---- S^T for the two 16-key halves
        float4_t s[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            float4_t acc = {0, 0, 0, 0};
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                acc = mfma16(khi[h][p], qlo[p], acc);
                if constexpr (KV_F32) acc = mfma16(klo[h][p], qhi[p], acc);
                acc = mfma16(khi[h][p], qhi[p], acc);
            }
            s[h] = acc;
        }

        // ---- scale, soft cap, mask; keys of lane (j,c): kb + 16h + 4j + r
        float cmax = -INFINITY;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = kb + 16 * h + 4 * j + r;
                float x = s[h][r] * a.scale;
                if (a.softcap != 0.0f) x = a.softcap * tanhf(x);
                if (key < kv1) {
                    if (mrow) x += slope * __half2float(((const __half *) mrow)[key]);
                } else {
                    x = -INFINITY;
                }
                s[h][r] = x;
                cmax = fmaxf(cmax, x);
            }
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));

        const float m_new = fmaxf(m, cmax);
        if (__builtin_amdgcn_ballot_w64(m_new != -INFINITY) == 0) continue; // every column fully masked so far

        const float alpha = (m_new == -INFINITY) ? 1.0f : __expf(m - m_new); // m = -inf -> 0
        float psum = 0.0f;
        half8_t phi, plo;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float pv = (m_new == -INFINITY) ? 0.0f : __expf(s[h][r] - m_new);
                psum += pv;
                const _Float16 ph = (_Float16) pv;
                phi[4 * h + r] = ph;
                plo[4 * h + r] = (_Float16) (pv - (float) ph);
            }
        l = l * alpha + psum;
        m = m_new;
#pragma unroll
        for (int p = 0; p < NP; ++p) { o[p][0] *= alpha; o[p][1] *= alpha; }

        // ---- O^T += V^T P^T, V^T produced by the matrix core
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                float4_t t0 = mfma16(vhi[0][p], sel[u], float4_t{0, 0, 0, 0});
                float4_t t1 = mfma16(vhi[1][p], sel[u], float4_t{0, 0, 0, 0});
                if constexpr (KV_F32) { t0 = mfma16(vlo[0][p], sel[u], t0); t1 = mfma16(vlo[1][p], sel[u], t1); }
                half8_t vt;
#pragma unroll
                for (int r = 0; r < 4; ++r) { vt[r] = (_Float16) t0[r]; vt[4 + r] = (_Float16) t1[r]; }
                o[p][u] = mfma16(vt, plo, o[p][u]);
                o[p][u] = mfma16(vt, phi, o[p][u]);
                if constexpr (KV_F32) {
                    half8_t vl;
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        vl[r]     = (_Float16) (t0[r] - (float) vt[r]);
                        vl[4 + r] = (_Float16) (t1[r] - (float) vt[4 + r]);
                    }
                    o[p][u] = mfma16(vl, phi, o[p][u]);
                }
            }
    }

    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);

    // lane (j,c), tile (p,u), register r holds d = SEG*(2u + j/2) + 8p + 4*(j%2) + r of column c
    if (a.n_splits == 1) {
        if (a.sinks) { // ops.cpp:8306-8322
            const float sk = a.sinks[head];
            float ms = 1.0f, vs = 1.0f;
            if (sk > m) { ms = __expf(m - sk); } else { vs = __expf(sk - m); }
#pragma unroll
            for (int p = 0; p < NP; ++p) { o[p][0] *= ms; o[p][1] *= ms; }
            l = l * ms + vs;
        }
        const float inv = l == 0.0f ? 0.0f : 1.0f / l;
        if (col_ok) {
            float * out = a.dst + (((uint64_t) b * a.n_q + iq1) * a.Hq + head) * D;
#pragma unroll
            for (int p = 0; p < NP; ++p)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const int d0 = SEG * (2 * u + (j >> 1)) + 8 * p + 4 * (j & 1);
                    *(float4_t *) (out + d0) = o[p][u] * inv;
                }
        }
    } else if (col_ok) {
        const uint64_t gcol = ((uint64_t) b * a.Hkv + g) * ncols + col;
        float * po = a.part_o + (gcol * a.n_splits + sp) * D;
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int d0 = SEG * (2 * u + (j >> 1)) + 8 * p + 4 * (j & 1);
                *(float4_t *) (po + d0) = o[p][u];
            }
        if (j == 0) {
            float * pml = a.part_ml + (gcol * a.n_splits + sp) * 2;
            pml[0] = m;
            pml[1] = l;
        }
    }
}

// merges the split partials of one column: the arithmetic of
// ggml_flash_attn_ext_reduce_partials (ggml/src/ggml-cpu/ops.cpp:8637-8705) with the global
// maximum taken first.  One block of D threads per column.
template <int D>
__global__ __launch_bounds__(D) void fattn_combine_kernel(const fa_args a) {
    const int      ncols = a.n_q * a.gqa;
    const uint64_t gcol  = blockIdx.x;
    const int      col   = (int) (gcol % ncols);
    const int      bg    = (int) (gcol / ncols);
    const int      g = bg % a.Hkv, b = bg / a.Hkv;
    const int      iq1 = col / a.gqa, head = g * a.gqa + col % a.gqa;
    const int      d = threadIdx.x;

    const float * pml = a.part_ml + gcol * a.n_splits * 2;
    const float * po  = a.part_o + gcol * a.n_splits * D;
    float M = -INFINITY;
    for (int s = 0; s < a.n_splits; ++s) M = fmaxf(M, pml[2 * s]);
    float acc = 0.0f, L = 0.0f;
    if (M != -INFINITY) {
        for (int s = 0; s < a.n_splits; ++s) {
            const float ms = pml[2 * s];
            if (ms == -INFINITY) continue;
            const float wgt = __expf(ms - M);
            acc += wgt * po[(uint64_t) s * D + d];
            L += wgt * pml[2 * s + 1];
        }
    }
    if (a.sinks) {
        const float sk = a.sinks[head];
        float ms = 1.0f, vs = 1.0f;
        if (sk > M) { ms = __expf(M - sk); } else { vs = __expf(sk - M); }
        acc *= ms;
        L = L * ms + vs;
    }
    a.dst[(((uint64_t) b * a.n_q + iq1) * a.Hq + head) * D + d] = L == 0.0f ? 0.0f : acc / L;
}

int g_num_cus = 0;

int num_cus() {
    if (g_num_cus == 0) {
        int dev = 0;
        hipDeviceProp_t p;
        if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&p, dev) == hipSuccess) g_num_cus = p.multiProcessorCount;
        if (g_num_cus <= 0) g_num_cus = 256;
    }
    return g_num_cus;
}

bool aligned16(const vx_tensor * t) {
    return ((uintptr_t) t->data % 16 == 0) && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
}

} // namespace

extern "C" int vx_supports_flash_attn_ext(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                          const vx_tensor * mask, const vx_tensor * dst) {
    if (!q || !k || !v || !dst) return 0;
    if (q->type != VX_TYPE_F32 || dst->type != VX_TYPE_F32) return 0;
    if (k->type != v->type || (k->type != VX_TYPE_F16 && k->type != VX_TYPE_F32)) return 0;
    if (!vx_positive(q) || !vx_positive(k) || !vx_positive(v)) return 0;
    const int64_t D = q->ne[0];
    if (D != 64 && D != 128) return 0;
    if (k->ne[0] != D || v->ne[0] != D) return 0;
    if (k->ne[1] != v->ne[1] || k->ne[2] != v->ne[2] || k->ne[3] != v->ne[3]) return 0;
    if (q->ne[2] % k->ne[2] || q->ne[3] % k->ne[3]) return 0;
    if (q->nb[0] != 4 || k->nb[0] != vx_type_size(k->type) || v->nb[0] != vx_type_size(v->type)) return 0;
    // strides must keep 16-byte vector loads aligned; the data pointers are checked at launch
    for (int i = 1; i < 4; ++i)
        if (q->nb[i] % 16 || k->nb[i] % 16 || v->nb[i] % 16) return 0;
    if (dst->ne[0] != D || dst->ne[1] != q->ne[2] || dst->ne[2] != q->ne[1] || dst->ne[3] != q->ne[3]) return 0;
    if (!vx_is_contiguous(dst)) return 0;
    if (mask) {
        if (mask->type != VX_TYPE_F16 || mask->nb[0] != 2) return 0;
        if (mask->ne[0] != k->ne[1] || mask->ne[1] < q->ne[1]) return 0;
        if (mask->ne[2] <= 0 || mask->ne[3] <= 0 || q->ne[2] % mask->ne[2] || q->ne[3] % mask->ne[3]) return 0;
    }
    if (q->ne[1] * (q->ne[2] / k->ne[2]) > 0x3fffffff || k->ne[1] > 0x3fffffff) return 0;
    return 1;
}

extern "C" vx_status vx_flash_attn_ext(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                       const vx_tensor * mask, const float * sinks, const vx_tensor * dst,
                                       float scale, float max_bias, float logit_softcap, vx_stream stream) {
    if (!q || !k || !v || !dst || !q->data || !k->data || !v->data || !dst->data || (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext: null tensor");
    if (!vx_supports_flash_attn_ext(q, k, v, mask, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: needs q F32, k/v both F16 or both F32, D in {64,128}, dense rows, 16-byte aligned strides, contiguous dst, F16 mask");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (uintptr_t) dst->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: tensor data must be 16-byte aligned");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext: max_bias > 0 requires a mask");

    hipStream_t st = (hipStream_t) stream;
    fa_args a;
    a.q = (const char *) q->data; a.k = (const char *) k->data; a.v = (const char *) v->data;
    a.mask = mask ? (const char *) mask->data : nullptr;
    a.sinks = sinks;
    a.dst = (float *) dst->data;
    a.part_o = nullptr; a.part_ml = nullptr;
    a.nbq1 = q->nb[1]; a.nbq2 = q->nb[2]; a.nbq3 = q->nb[3];
    a.nbk1 = k->nb[1]; a.nbk2 = k->nb[2]; a.nbk3 = k->nb[3];
    a.nbv1 = v->nb[1]; a.nbv2 = v->nb[2]; a.nbv3 = v->nb[3];
    a.nbm1 = mask ? mask->nb[1] : 0; a.nbm2 = mask ? mask->nb[2] : 0; a.nbm3 = mask ? mask->nb[3] : 0;
    a.n_q = (int) q->ne[1]; a.n_kv = (int) k->ne[1]; a.Hq = (int) q->ne[2]; a.Hkv = (int) k->ne[2];
    a.gqa = a.Hq / a.Hkv; a.ne3 = (int) q->ne[3]; a.rk3 = (int) (q->ne[3] / k->ne[3]);
    a.nem2 = mask ? (int) mask->ne[2] : 1; a.nem3 = mask ? (int) mask->ne[3] : 1;
    a.scale = scale; a.softcap = logit_softcap; a.max_bias = max_bias;
    if (logit_softcap != 0.0f) a.scale /= logit_softcap; // ops.cpp:8173-8175
    a.n_head_log2 = 1u << (uint32_t) floor(log2((double) a.Hq));
    a.m0 = powf(2.0f, -(max_bias) / a.n_head_log2);
    a.m1 = powf(2.0f, -(max_bias / 2.0f) / a.n_head_log2);

    const int ncols = a.n_q * a.gqa;
    a.n_col_tiles   = (ncols + 15) / 16;
    const int64_t base_waves = (int64_t) a.ne3 * a.Hkv * a.n_col_tiles;

    // split the keys so that the launch has about 8 waves per CU, at least 64 keys each
    const int64_t target = (int64_t) 8 * num_cus();
    int64_t want = (target + base_waves - 1) / base_waves;
    const int64_t max_splits = (a.n_kv + 63) / 64;
    if (want > max_splits) want = max_splits;
    if (want < 1) want = 1;
    int chunk = (int) ((a.n_kv + want - 1) / want);
    chunk     = (chunk + 31) / 32 * 32;
    a.chunk    = chunk;
    a.n_splits = (a.n_kv + chunk - 1) / chunk;

    const int64_t nblocks = base_waves * a.n_splits;
    if (nblocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: launch too large");
    const int D = (int) q->ne[0];
    const int64_t gcols = (int64_t) a.ne3 * a.Hkv * ncols;

    if (a.n_splits > 1) {
        const size_t o_bytes = (size_t) gcols * a.n_splits * D * sizeof(float);
        const size_t ml_bytes = (size_t) gcols * a.n_splits * 2 * sizeof(float);
        void * ws = nullptr;
        vx_status rc = vx_workspace(st, o_bytes + ml_bytes, &ws);
        if (rc != VX_OK) return rc;
        a.part_o  = (float *) ws;
        a.part_ml = (float *) ((char *) ws + o_bytes);
    }

    const bool f32 = k->type == VX_TYPE_F32;
    const dim3 grid((unsigned) nblocks), block(64);
    if (D == 64) {
        if (f32) fattn_cols16_kernel<64, true><<<grid, block, 0, st>>>(a);
        else     fattn_cols16_kernel<64, false><<<grid, block, 0, st>>>(a);
    } else {
        if (f32) fattn_cols16_kernel<128, true><<<grid, block, 0, st>>>(a);
        else     fattn_cols16_kernel<128, false><<<grid, block, 0, st>>>(a);
    }
    VX_LAUNCH_CHECK();
    if (a.n_splits > 1) {
        if (D == 64) fattn_combine_kernel<64><<<dim3((unsigned) gcols), dim3(64), 0, st>>>(a);
        else         fattn_combine_kernel<128><<<dim3((unsigned) gcols), dim3(128), 0, st>>>(a);
        VX_LAUNCH_CHECK();
    }
    return VX_OK;
}
