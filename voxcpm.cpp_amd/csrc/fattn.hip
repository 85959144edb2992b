// fattn.hip -- GGML_OP_FLASH_ATTN_EXT on gfx950: the column-packed kernel used for decode,
// LocDiT-sized sequences and as the general path.
//
// Work decomposition.  For one batch element b and one KV head g, every (query row iq1,
// query head of the GQA group) pair is a *column*: col = iq1 * gqa + head_in_group.  A
// wavefront owns 16 consecutive columns -- in decode that is the 8 query heads sharing the
// KV head (x2 rows when n_q = 2), in LocDiT 2 rows x 8 heads -- and one contiguous range
// of keys.  Its K/V stream never touches LDS: operands are loaded from global memory
// straight into MFMA layout, one 32-key tile in flight ahead of the one being consumed.
// When there are too few columns to fill the chip the keys are cut further (flash-decoding):
// several waves take adjacent key ranges of the same columns and write (max, sum, O)
// partials that a second, small kernel merges.  (Merging inside the first kernel, by the
// last wave to arrive, needs device-scope release/acquire fences; on this multi-die part
// those write back and invalidate L2 and cost several times what the second launch does.)
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
//                      convert makes it the A operand.  Matrix throughput is several times
//                      what HBM can feed in this regime, so the transpose costs nothing.
// Precision: Q, P (and K, V when they are F32) are split into f16 hi + lo parts and both
// parts multiplied, so the products carry ~22 bits; accumulation and softmax are fp32.
//
// Algorithmic HBM bytes: each K and V element is read once per 16-column tile; in decode
// (one tile per KV head) that is n_kv * D * 2 * sizeof(kv) per (b, g), the figure the
// benchmark divides by.
#include <type_traits>
#include "vx_common.hpp"
#include "kvs_common.hpp"

#include <cmath>
#include <cstdlib>
#include <mutex>

namespace {

struct fa_args {
    const char * q; const char * k; const char * v; const char * mask;
    const float * sinks;
    const float * add1; // optional scalar added to every output element (a fused GGML_OP_ADD1)
    float * dst;
    float * part_o;   // [tile][split][16 columns][D]   split partials, un-normalised
    float * part_ml;  // [tile][split][16 columns][2]   running max, running sum
    uint64_t nbq1, nbq2, nbq3, nbk1, nbk2, nbk3, nbv1, nbv2, nbv3, nbm1, nbm2, nbm3;
    // keys n_kv1 .. n_kv-1 may lie in a second pair of tensors (the current step's K and V, which the
    // reference appends to the cached ones with GGML_OP_CONCAT before attention); null = one segment
    // the reference's cache write with its ordering scalar folded in (has_kvs): an extra block of the first kernel does it,
    // block 0 stores both slots, every block forms the two sums and adds the scalar to its column
    kvs_side kvs_k, kvs_v;
    float kvs_scale, kvs_bias;
    int has_kvs;
    float * kvs_out; // the scalar, written by the first kernel's extra block and read by every merge block
    const char * k2; const char * v2;
    uint64_t nbk1b, nbk2b, nbk3b, nbv1b, nbv2b, nbv3b;
    int n_kv1;
    int seg2_f32; // the second segment holds F32 values while the first is an F16 cache (rounded to f16 as they are loaded)
    int n_q, n_kv, Hq, Hkv, gqa, ne3, rk3, nem2, nem3;
    int n_col_tiles, n_splits, chunk;
    float inv_gqa, inv_hkv; // reciprocals for fa_div
    float scale, softcap, max_bias, m0, m1;
    uint32_t n_head_log2;
};

// x / d for 0 <= x < 2^22 with inv = 1 / d: half a step away from every multiple of d the rounding of the product cannot
// reach the next integer.  (An integer division costs a wave some thirty instructions; the index arithmetic at the top of
// these kernels stands between the launch and the first load.)
__device__ __forceinline__ int fa_div(int x, float inv) { return (int) (((float) x + 0.5f) * inv); }

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// two floats -> packed halves, round toward zero: one instruction.  Used where the value is
// exactly representable (transposed f16 data) or where a lo part picks up the remainder.
__device__ __forceinline__ void pk2(half8_t & dst, int i, float a, float b) {
    typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
    const fp16x2 v = __builtin_amdgcn_cvt_pkrtz(a, b);
    dst[i]     = (_Float16) v[0];
    dst[i + 1] = (_Float16) v[1];
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

// the K and V rows one wave consumes per iteration: 32 keys, as MFMA operands
template <int NP, bool KV_F32> struct kv_tile {
    half8_t khi[2][NP], klo[2][NP], vhi[2][NP], vlo[2][NP];
    __half  mk[2][4]; // the mask's entries for this lane's 8 keys, requested with the tile
};

// sinks (ops.cpp:8306-8322), normalisation and the permuted store of ggml's result for 4
// consecutive d of one column
// (the sink and the addend are read by the caller, once and before its first store: a load behind a store waits for the
// store's completion as well, the memory counter being one for both)
__device__ __forceinline__ void fa_finish(const fa_args & a, float4_t acc, float M, float L, int b, int iq1, int head,
                                          int D, int d0, bool has_sink, float sink, bool has_addend, float addend) {
#pragma clang fp contract(off) // the normalised value is rounded before the addend joins it, as two nodes would
    if (has_sink) {
        const float sk = sink * 1.44269504088896341f; // M is in the log2 domain
        float ms = 1.0f, vs = 1.0f;
        if (sk > M) { ms = __builtin_amdgcn_exp2f(M - sk); } else { vs = __builtin_amdgcn_exp2f(sk - M); }
        acc *= ms;
        L = L * ms + vs;
    }
    const float inv = L == 0.0f ? 0.0f : 1.0f / L;
    float4_t r = acc * inv;
    if (has_addend) r += addend; // rounded after the normalisation, as the separate ADD1 node would
    *(float4_t *) (a.dst + (((uint64_t) b * a.n_q + iq1) * a.Hq + head) * D + d0) = r;
}

// One wave (= one block) = 16 columns x one key range.
// TWO_SEG: 0 = K and V are one tensor each; 1 = keys from n_kv1 on lie in a second pair of tensors of the same type;
// 2 = the first pair is an F16 cache and the second pair F32 (the step's own keys and values, as the projections
// left them): they are rounded to f16, to nearest even, while they are loaded -- exactly what a CPY node to an F16
// tensor in front of a CONCAT would have stored.
// HALF: the whole key range is at most 16 keys (chosen by the host: one range, one pair of tensors).
template <int D, bool KV_F32, bool HAS_MASK, bool SOFTCAP, int TWO_SEG, bool HALF = false>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2))) void fattn_cols16_kernel(const fa_args a) {
    constexpr int NP  = D / 32;          // MFMAs along the head dimension
    constexpr int SEG = D / 4;           // elements of a row owned by lane-group j
    constexpr int ES  = KV_F32 ? 4 : 2;  // bytes per K/V element

    const int lane = threadIdx.x;
    const int j = lane >> 4, c = lane & 15;

    // With the cache write folded in, the grid has one more slice in front: its first wave forms the two sums and leaves
    // the scalar for the merge kernel, its other waves store the slots.  (One wave reads
    // the step's keys and values: when every merge block formed the sums itself, sixteen streams' 512 blocks asked the
    // same few cache lines at once and the merge took 9 us instead of 4.)
    if constexpr (TWO_SEG != 0) {
        if (a.has_kvs && blockIdx.z == 0) {
            if (blockIdx.x != 0) return;
            if (blockIdx.y == 0) { // the sums, in GGML_OP_SUM's order, by one wave (no stores: their index arithmetic is the others' work)
                double tk, tv;
                if (a.kvs_k.vec && a.kvs_v.vec) kvs_wave_totals<true, true>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
                else if (a.kvs_k.vec)           kvs_wave_totals<true, false>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
                else if (a.kvs_v.vec)           kvs_wave_totals<false, true>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
                else                            kvs_wave_totals<false, false>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
                if (lane == 0) *a.kvs_out = kvs_scalar((float) tk, (float) tv, a.kvs_scale, a.kvs_bias);
            } else { // the stores, dealt over the slice's other waves (there are n_splits - 1 >= 1 of them)
                const uint32_t first = (blockIdx.y - 1) * 64 + lane, step = (gridDim.y - 1) * 64;
                double unused = 0.0;
                const uint32_t nk = kvs_units(a.kvs_k, a.kvs_k.vec != 0), nv = kvs_units(a.kvs_v, a.kvs_v.vec != 0);
                if (a.kvs_k.vec) { for (uint32_t e = first; e < nk; e += step) kvs_unit<true>(a.kvs_k, e, true, unused); }
                else             { for (uint32_t e = first; e < nk; e += step) kvs_unit<false>(a.kvs_k, e, true, unused); }
                if (a.kvs_v.vec) { for (uint32_t e = first; e < nv; e += step) kvs_unit<true>(a.kvs_v, e, true, unused); }
                else             { for (uint32_t e = first; e < nv; e += step) kvs_unit<false>(a.kvs_v, e, true, unused); }
            }
            return;
        }
    }
    // the grid is (column tile, key range, batch entry x KV head): dispatched in the same order as one flat index
    const int ct = blockIdx.x, sp = blockIdx.y, bg = (int) blockIdx.z - ((TWO_SEG != 0 && a.has_kvs) ? 1 : 0);
    const int b  = fa_div(bg, a.inv_hkv);
    const int g  = bg - b * a.Hkv;
    const int tile = bg * a.n_col_tiles + ct;

    const int  ncols  = a.n_q * a.gqa;
    const int  col    = ct * 16 + c;
    const bool col_ok = col < ncols;
    const int  iq1    = col_ok ? fa_div(col, a.inv_gqa) : 0;
    const int  head   = g * a.gqa + (col_ok ? col - iq1 * a.gqa : 0);
    const int  bk     = a.rk3 == 1 ? b : b / a.rk3; // K / V broadcast over the batch dimension: rare

    const char * kbase = a.k + (uint64_t) g * a.nbk2 + (uint64_t) bk * a.nbk3 + (uint64_t) (SEG * j) * ES;
    const char * vbase = a.v + (uint64_t) g * a.nbv2 + (uint64_t) bk * a.nbv3 + (uint64_t) (SEG * j) * ES;

    const char * kbase2 = kbase;
    const char * vbase2 = vbase;
    if constexpr (TWO_SEG != 0) {
        constexpr int ES2 = TWO_SEG == 2 ? 4 : ES;
        kbase2 = a.k2 + (uint64_t) g * a.nbk2b + (uint64_t) bk * a.nbk3b + (uint64_t) (SEG * j) * ES2;
        vbase2 = a.v2 + (uint64_t) g * a.nbv2b + (uint64_t) bk * a.nbv3b + (uint64_t) (SEG * j) * ES2;
    }

    float slope = 1.0f;
    const __half * mrow = nullptr;
    if constexpr (HAS_MASK) {
        slope = vx_alibi_slope(a.max_bias, (uint32_t) head, a.n_head_log2, a.m0, a.m1) * 1.44269504088896341f;
        if (a.mask) mrow = (const __half *) (a.mask + (uint64_t) iq1 * a.nbm1 + (uint64_t) (a.nem2 == 1 ? 0 : head % a.nem2) * a.nbm2 + (uint64_t) (a.nem3 == 1 ? 0 : b % a.nem3) * a.nbm3);
    }

    const int kv0 = sp * a.chunk;
    const int kv1 = min(a.n_kv, kv0 + a.chunk);
    // Mixed types: 32-key tiles that lie wholly in the cache (tile starts below `pure`) stream through the pipelined
    // loop; the tile that straddles the boundary and any tile behind it -- one tile in all at decode -- are loaded
    // lane by lane from whichever tensor holds the key.  Key ranges start at multiples of 32, so tiles do too.
    const int pure   = TWO_SEG == 2 ? a.n_kv1 / 32 * 32 : 0;
    const int kv1p   = TWO_SEG == 2 ? min(kv1, pure) : kv1;  // end of the pipelined tiles
    const int kclamp = TWO_SEG == 2 ? a.n_kv1 - 1 : a.n_kv - 1;

    // the mask's entries of a tile's keys kb + 16h + 4j + r, requested behind the tile itself (clamped like the rows)
    auto load_mask = [&](int kb, kv_tile<NP, KV_F32> & t, int halves) {
        if constexpr (HAS_MASK) {
            if (SOFTCAP ? mrow != nullptr : true) { // (without a soft cap this kernel is only launched with a mask)
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (h < halves) t.mk[h][r] = mrow[min(kb + 16 * h + 4 * j + r, a.n_kv - 1)];
            }
        }
    };

    // rows this lane loads (MFMA row c of each 16-key half); clamped, masked out later
    auto load_tile = [&](int kb, kv_tile<NP, KV_F32> & t) {
        const int key0 = min(kb + c, kclamp), key1 = min(kb + 16 + c, kclamp);
        const char * k0p = kbase + (uint64_t) key0 * a.nbk1;
        const char * k1p = kbase + (uint64_t) key1 * a.nbk1;
        const char * v0p = vbase + (uint64_t) key0 * a.nbv1;
        const char * v1p = vbase + (uint64_t) key1 * a.nbv1;
        if constexpr (TWO_SEG == 1) {
            if (key0 >= a.n_kv1) { k0p = kbase2 + (uint64_t) (key0 - a.n_kv1) * a.nbk1b; v0p = vbase2 + (uint64_t) (key0 - a.n_kv1) * a.nbv1b; }
            if (key1 >= a.n_kv1) { k1p = kbase2 + (uint64_t) (key1 - a.n_kv1) * a.nbk1b; v1p = vbase2 + (uint64_t) (key1 - a.n_kv1) * a.nbv1b; }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            kv_load<KV_F32>::run(k0p + p * 8 * ES, t.khi[0][p], t.klo[0][p]);
            kv_load<KV_F32>::run(k1p + p * 8 * ES, t.khi[1][p], t.klo[1][p]);
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            kv_load<KV_F32>::run(v0p + p * 8 * ES, t.vhi[0][p], t.vlo[0][p]);
            kv_load<KV_F32>::run(v1p + p * 8 * ES, t.vhi[1][p], t.vlo[1][p]);
        }
        load_mask(kb, t, 2);
    };

    // the first 16 keys of a tile only: all a range of at most 16 keys needs
    auto load_half0 = [&](int kb, kv_tile<NP, KV_F32> & t) {
        const int key0 = min(kb + c, kclamp);
        const char * k0p = kbase + (uint64_t) key0 * a.nbk1;
        const char * v0p = vbase + (uint64_t) key0 * a.nbv1;
        if constexpr (TWO_SEG == 1) {
            if (key0 >= a.n_kv1) { k0p = kbase2 + (uint64_t) (key0 - a.n_kv1) * a.nbk1b; v0p = vbase2 + (uint64_t) (key0 - a.n_kv1) * a.nbv1b; }
        }
#pragma unroll
        for (int p = 0; p < NP; ++p) kv_load<KV_F32>::run(k0p + p * 8 * ES, t.khi[0][p], t.klo[0][p]);
#pragma unroll
        for (int p = 0; p < NP; ++p) kv_load<KV_F32>::run(v0p + p * 8 * ES, t.vhi[0][p], t.vlo[0][p]);
        load_mask(kb, t, 1);
    };

    // a tile at or behind the type boundary: each lane reads its two keys from the tensor that holds them
    auto load_mixed = [&](int kb, kv_tile<NP, KV_F32> & t) {
        load_mask(kb, t, 2);
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const int key = min(kb + 16 * h + c, a.n_kv - 1);
            if (key < a.n_kv1) {
                const char * kp = kbase + (uint64_t) key * a.nbk1;
                const char * vp = vbase + (uint64_t) key * a.nbv1;
#pragma unroll
                for (int p = 0; p < NP; ++p) {
                    kv_load<KV_F32>::run(kp + p * 8 * ES, t.khi[h][p], t.klo[h][p]);
                    kv_load<KV_F32>::run(vp + p * 8 * ES, t.vhi[h][p], t.vlo[h][p]);
                }
            } else {
                const char * kp = kbase2 + (uint64_t) (key - a.n_kv1) * a.nbk1b;
                const char * vp = vbase2 + (uint64_t) (key - a.n_kv1) * a.nbv1b;
#pragma unroll
                for (int p = 0; p < NP; ++p) {
                    const float4_t ka = ((const float4_t *) (kp + p * 32))[0], kb4 = ((const float4_t *) (kp + p * 32))[1];
                    const float4_t va = ((const float4_t *) (vp + p * 32))[0], vb4 = ((const float4_t *) (vp + p * 32))[1];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        t.khi[h][p][i] = (_Float16) ka[i]; t.khi[h][p][4 + i] = (_Float16) kb4[i];
                        t.vhi[h][p][i] = (_Float16) va[i]; t.vhi[h][p][4 + i] = (_Float16) vb4[i];
                    }
                }
            }
        }
    };

    // Q's values are requested first: the tile loads below sit in branches, F32 tiles are converted where they are
    // loaded, and whatever is requested behind a branch waits for that conversion's data.
    float4_t qraw[NP][2];
    {
        const float * qp = (const float *) (a.q + (uint64_t) iq1 * a.nbq1 + (uint64_t) head * a.nbq2 + (uint64_t) b * a.nbq3) + SEG * j;
#pragma unroll
        for (int p = 0; p < NP; ++p) { qraw[p][0] = ((const float4_t *) (qp + 8 * p))[0]; qraw[p][1] = ((const float4_t *) (qp + 8 * p))[1]; }
    }

    // two tiles alternate in registers: while one is consumed the other is in flight
    kv_tile<NP, KV_F32> t0, t1, t2;
    const int kmix = max(kv0, pure); // first tile of the lane-by-lane part (TWO_SEG == 2)
    // A range of at most 16 keys (LocDiT's 14-token sequence) is half a tile: the second half's loads, conversions and
    // products would all be of keys that are switched off.  (A kernel of its own, not a branch: tile loads in a branch
    // would hold back every request behind it until their conversions have their data.)
    static_assert(!HALF || TWO_SEG == 0, "the half-tile kernel reads one pair of tensors");
    if constexpr (TWO_SEG == 2) {
        if (kmix < kv1) load_mixed(kmix, t2);  // requested first, consumed last
        if (kv0 < kv1p) load_tile(kv0, t0);
    } else if constexpr (HALF) {
        load_half0(kv0, t0);
    } else {
        load_tile(kv0, t0);
    }

    // ---- Q^T operand: column c, elements d = SEG*j + 8p + i, split into hi + lo
    half8_t qhi[NP], qlo[NP];
    {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            float4_t x0 = qraw[p][0], x1 = qraw[p][1];
            if (!col_ok) { x0 = float4_t{0, 0, 0, 0}; x1 = float4_t{0, 0, 0, 0}; }
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


    float4_t o[NP][2];
#pragma unroll
    for (int p = 0; p < NP; ++p) { o[p][0] = float4_t{0, 0, 0, 0}; o[p][1] = float4_t{0, 0, 0, 0}; }
    float m = -INFINITY; // running max of column c (identical in the 4 lanes of a column)
    float l = 0.0f;      // this lane's share of the running sum

    auto consume = [&](const kv_tile<NP, KV_F32> & t, int kb, auto first_half_only) {
        constexpr int NH = decltype(first_half_only)::value ? 1 : 2; // 16-key halves that take part
        // additive mask of this lane's 8 keys (kb + 16h + 4j + r); loads are clamped, keys
        // past the end of the range (only in a wave's last tile) are switched off
        const bool tail = kb + 32 > kv1; // wave-uniform
        float mv[2][4];
        if (HAS_MASK || tail) {
#pragma unroll
            for (int h = 0; h < NH; ++h)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int key = kb + 16 * h + 4 * j + r;
                    float x = 0.0f;
                    if constexpr (HAS_MASK) { if (SOFTCAP ? mrow != nullptr : true) x = slope * __half2float(t.mk[h][r]); } // slope carries log2(e)
                    mv[h][r] = key < kv1 ? x : -INFINITY;
                }
        }

        // ---- S^T for the two 16-key halves
        float4_t s[2];
#pragma unroll
        for (int h = 0; h < NH; ++h) {
            float4_t acc = {0, 0, 0, 0};
#pragma unroll
            for (int p = 0; p < NP; ++p) {
                acc = mfma16(t.khi[h][p], qlo[p], acc);
                if constexpr (KV_F32) acc = mfma16(t.klo[h][p], qhi[p], acc);
                acc = mfma16(t.khi[h][p], qhi[p], acc);
            }
            s[h] = acc;
        }

        // ---- scale, soft cap, mask
        float cmax = -INFINITY;
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // a.scale carries log2(e) (the soft cap path applies it after tanh)
                float x = s[h][r] * a.scale;
                if constexpr (SOFTCAP) x = a.softcap * tanhf(x);
                if (HAS_MASK || tail) x += mv[h][r];
                s[h][r] = x;
                cmax = fmaxf(cmax, x);
            }
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));

        // a column whose keys are all masked so far keeps m = -inf; shifting by 0 instead
        // keeps exp(-inf - shift) = 0 without a branch
        const float m_new  = fmaxf(m, cmax);
        const float shift  = (m_new == -INFINITY) ? 0.0f : m_new;
        const float alpha  = __builtin_amdgcn_exp2f(m - shift); // m = -inf -> 0
        float psum = 0.0f;
        half8_t phi, plo;
        float pvv[8] = { 0, 0, 0, 0, 0, 0, 0, 0 }; // (the weights of a half that takes no part: exactly what its switched-off keys would get)
#pragma unroll
        for (int h = 0; h < NH; ++h)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pvv[4 * h + r] = __builtin_amdgcn_exp2f(s[h][r] - shift);
                psum += pvv[4 * h + r];
            }
#pragma unroll
        for (int i = 0; i < 8; i += 2) pk2(phi, i, pvv[i], pvv[i + 1]);
#pragma unroll
        for (int i = 0; i < 8; i += 2) pk2(plo, i, pvv[i] - (float) phi[i], pvv[i + 1] - (float) phi[i + 1]);
        l = l * alpha + psum;
        m = m_new;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) { // the maxima rarely move late in a row
#pragma unroll
            for (int p = 0; p < NP; ++p) { o[p][0] *= alpha; o[p][1] *= alpha; }
        }

        // ---- O^T += V^T P^T, V^T produced by the matrix core
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                float4_t t0 = mfma16(t.vhi[0][p], sel[u], float4_t{0, 0, 0, 0});
                float4_t t1 = float4_t{0, 0, 0, 0};
                if constexpr (NH == 2) t1 = mfma16(t.vhi[1][p], sel[u], t1);
                if constexpr (KV_F32) {
                    t0 = mfma16(t.vlo[0][p], sel[u], t0);
                    if constexpr (NH == 2) t1 = mfma16(t.vlo[1][p], sel[u], t1);
                }
                half8_t vt;
#pragma unroll
                for (int r = 0; r < 4; r += 2) { pk2(vt, r, t0[r], t0[r + 1]); pk2(vt, 4 + r, t1[r], t1[r + 1]); }
                o[p][u] = mfma16(vt, plo, o[p][u]);
                o[p][u] = mfma16(vt, phi, o[p][u]);
                if constexpr (KV_F32) {
                    half8_t vl;
#pragma unroll
                    for (int r = 0; r < 4; r += 2) {
                        pk2(vl, r, t0[r] - (float) vt[r], t0[r + 1] - (float) vt[r + 1]);
                        pk2(vl, 4 + r, t1[r] - (float) vt[4 + r], t1[r + 1] - (float) vt[4 + r + 1]);
                    }
                    o[p][u] = mfma16(vl, phi, o[p][u]);
                }
            }
    };

    // The prefetches are unconditional (the tile index is clamped to the wave's last tile, a
    // cache hit) so that the wait before each use counts a fixed number of younger loads; a
    // conditional prefetch forces the compiler to wait for everything and exposes the whole
    // memory latency in every iteration.
    const int klast = kv0 + ((kv1p - kv0 - 1) / 32) * 32;
    if constexpr (HALF) {
        consume(t0, kv0, std::true_type{});
    } else {
        for (int kb = kv0; kb < kv1p; kb += 64) {
            load_tile(min(kb + 32, klast), t1);
            consume(t0, kb, std::false_type{});
            if (kb + 32 >= kv1p) break;
            load_tile(min(kb + 64, klast), t0);
            consume(t1, kb + 32, std::false_type{});
        }
    }
    if constexpr (TWO_SEG == 2) {
        for (int kb = kmix; kb < kv1; kb += 32) {
            if (kb != kmix) load_mixed(kb, t2);
            consume(t2, kb, std::false_type{});
        }
    }

    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (!col_ok) return;

    // lane (j,c), tile (p,u), register r holds d = SEG*(2u + j/2) + 8p + 4*(j%2) + r of column c
    if (a.n_splits == 1) {
        const bool  has_sink = a.sinks != nullptr, has_addend = a.add1 != nullptr;
        const float sink = has_sink ? a.sinks[head] : 0.0f, addend = has_addend ? *a.add1 : 0.0f;
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int u = 0; u < 2; ++u)
                fa_finish(a, o[p][u], m, l, b, iq1, head, D, SEG * (2 * u + (j >> 1)) + 8 * p + 4 * (j & 1), has_sink, sink, has_addend, addend);
    } else {
        const uint64_t pbase = ((uint64_t) tile * a.n_splits + sp) * 16 + c;
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int u = 0; u < 2; ++u)
                *(float4_t *) (a.part_o + pbase * D + SEG * (2 * u + (j >> 1)) + 8 * p + 4 * (j & 1)) = o[p][u];
        if (j == 0) { a.part_ml[pbase * 2] = m; a.part_ml[pbase * 2 + 1] = l; }
    }
}

// Merges the split partials: the arithmetic of ggml_flash_attn_ext_reduce_partials
// (ggml/src/ggml-cpu/ops.cpp:8637-8705) with the global maximum taken first.  One wave per
// output column.  Lane = (split phase q, 4 consecutive d): the D/4 lanes of a phase read one
// split's row as one coalesced line, the 64/(D/4) phases take interleaved splits.  A lane reads
// the (max, sum) pairs of its own splits too; every load of the first 16 splits per phase is
// issued before anything waits, so the kernel costs one trip to memory, a few cross-lane steps
// between the phases and a store.
constexpr int FA_MERGE_MAX_SPLITS = 256;
template <int D>
__global__ __launch_bounds__(64) void fattn_merge_kernel(const fa_args a) {
    constexpr int DU = D / 4;       // lanes per row
    constexpr int PH = 64 / DU;     // split phases
    constexpr int NB = 16;          // rows a lane has in flight
    // the grid is (16 columns x column tile, batch entry x KV head): no division of a flat index
    const int c = blockIdx.x & 15, ct = blockIdx.x >> 4, bg = blockIdx.y;
    const int tile = bg * a.n_col_tiles + ct;
    const int b = fa_div(bg, a.inv_hkv), g = bg - b * a.Hkv;
    const int col = ct * 16 + c;
    if (col >= a.n_q * a.gqa) return; // whole block
    const int lane = threadIdx.x, q = lane / DU, d0 = 4 * (lane % DU);
    // (with the cache write folded in, the addend is the scalar that the first kernel's extra block left: when every
    // merge block formed the sums itself in a second wave, sixteen streams' 512 blocks asked the same few cache lines at
    // once and the merge took 9 us instead of 4)
    const float * addend_p   = a.has_kvs ? a.kvs_out : a.add1;
    const bool    has_addend = addend_p != nullptr;
    const float   addend     = has_addend ? *addend_p : 0.0f;
    const uint64_t tbase = (uint64_t) tile * a.n_splits * 16 + c; // + split * 16
    // A lane works on the splits of its phase only: q, q + PH, q + 2 PH, ...  It reads their (max, sum) pairs and rows itself
    // and forms their weights itself, so the only cross-lane traffic is between the PH phases (log2 PH steps for the maximum,
    // the sum and the accumulator) -- no broadcast of weights from other lanes.
    const int per = (a.n_splits + PH - 1) / PH; // splits per lane
    const float2 *   pml = (const float2 *) (a.part_ml + tbase * 2);           // + split * 16 pairs
    const float4_t * po  = (const float4_t *) (a.part_o + tbase * D + d0);     // + split * 4 * D float4
    float    mv[NB], lv[NB];
    float4_t rows[NB];
    auto load_batch = [&](int j0) { // every load of a batch is issued before anything waits
#pragma unroll
        for (int jj = 0; jj < NB; ++jj) {
            const int  s2 = q + PH * (j0 + jj);
            const bool ok = j0 + jj < per && s2 < a.n_splits;
            const float2 ml = ok ? pml[(uint64_t) s2 * 16] : float2{-INFINITY, 0.0f};
            mv[jj] = ml.x; lv[jj] = ml.y;
            rows[jj] = ok ? po[(uint64_t) s2 * 4 * D] : float4_t{0, 0, 0, 0};
        }
    };
    load_batch(0);
    float M = -INFINITY;
#pragma unroll
    for (int jj = 0; jj < NB; ++jj) M = fmaxf(M, mv[jj]);
    for (int j0 = NB; j0 < per; j0 += NB) { // more than NB splits per lane: their maxima in a pass of their own
#pragma unroll
        for (int jj = 0; jj < NB; ++jj) {
            const int s2 = q + PH * (j0 + jj);
            if (j0 + jj < per && s2 < a.n_splits) M = fmaxf(M, pml[(uint64_t) s2 * 16].x);
        }
    }
#pragma unroll
    for (int off = DU; off < 64; off <<= 1) M = fmaxf(M, __shfl_xor(M, off, 64));
    const float shift = (M == -INFINITY) ? 0.0f : M;

    float    L   = 0.0f;
    float4_t acc = {0, 0, 0, 0};
    for (int j0 = 0; j0 < per; j0 += NB) {
        if (j0) load_batch(j0);
#pragma unroll
        for (int jj = 0; jj < NB; ++jj) {
            const float wgt = __builtin_amdgcn_exp2f(mv[jj] - shift); // the split's weight (0 for a slot past the end: max = -inf)
            L   += lv[jj] * wgt;
            acc += rows[jj] * wgt;
        }
    }
#pragma unroll
    for (int off = DU; off < 64; off <<= 1) {
        L += __shfl_xor(L, off, 64);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += __shfl_xor(acc[r], off, 64);
    }
    if (q == 0) {
        const int  iq1 = fa_div(col, a.inv_gqa), head = g * a.gqa + (col - iq1 * a.gqa);
        const bool has_sink = a.sinks != nullptr;
        fa_finish(a, acc, M, L, b, iq1, head, D, d0, has_sink, has_sink ? a.sinks[head] : 0.0f, has_addend, addend);
    }
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

// Work split.  Enough 16-column tiles to fill the chip: one wave per tile over all keys.
// Otherwise cut the keys (flash-decoding) aiming at ~4 waves per CU, at least `min_chunk`
// keys per wave and at most `cap` ranges, and merge the partials with a second small kernel.
// One 32-key step per wave is the fastest cut of a short cache (640 keys: 20 ranges, decode step
// 0.96 -> 0.92 ms against 64-key ranges); beyond 64 ranges the merge costs more than the cut saves
// (4096 keys in 128 ranges: 14.6 us against 8.2 us in 64).
void fa_split_plan(int64_t tiles, int n_kv, int * n_splits, int * chunk_out) {
    static const int min_chunk = [] { const char * e = getenv("VX_FA_MIN_CHUNK"); const int v = e ? atoi(e) : 0; return v >= 32 ? v / 32 * 32 : 32; }();
    *n_splits  = 1;
    *chunk_out = (n_kv + 31) / 32 * 32;
    // Up to 256 keys one wave finishes (0.5 us per 32-key step) before a split plus the merge
    // launch would.
    static const int waves_per_cu = [] { const char * e = getenv("VX_FA_WAVES_PER_CU"); const int v = e ? atoi(e) : 0; return v >= 1 && v <= 32 ? v : 4; }();
    if (tiles < (int64_t) waves_per_cu * num_cus() && n_kv > 256) {
        int64_t want = ((int64_t) waves_per_cu * num_cus() + tiles - 1) / tiles;
        const int64_t max_splits = (n_kv + min_chunk - 1) / min_chunk;
        if (want > max_splits) want = max_splits;
        static const int cap = [] { const char * e = getenv("VX_FA_MAX_SPLITS"); const int v = e ? atoi(e) : 0; return v >= 1 && v <= FA_MERGE_MAX_SPLITS ? v : 64; }();
        if (want > cap) want = cap;
        if (want < 1) want = 1;
        int chunk  = (int) ((n_kv + want - 1) / want);
        chunk      = (chunk + 31) / 32 * 32;
        *chunk_out = chunk;
        *n_splits  = (n_kv + chunk - 1) / chunk;
    }
}

int64_t fa_tiles(const vx_tensor * q, const vx_tensor * k) {
    const int64_t gqa = q->ne[2] / k->ne[2];
    return q->ne[3] * k->ne[2] * ((q->ne[1] * gqa + 15) / 16);
}

// ---- the streaming kernel for an f16 cache at decode (head size 64, one pair of tensors, no mask, no soft cap) -------
// The same work split as above (a wave = 16 columns x one key range), built for the one thing that bounds a long
// cache: bytes in flight per instruction issued.  A 32-key tile of K and of V is 8 direct loads into LDS
// (global_load_lds_dwordx4: 1 KB each, no registers, no address arithmetic: a scalar base per 8 rows and one lane
// offset; non-temporal, which alone is worth a microsecond and a half on a 64 MiB call), three tiles deep; K rows are
// read back as the A operand of S^T = K Q^T (16-byte chunks xor-swizzled by the row, 8-row blocks 128 bytes apart:
// conflict-free), V^T comes from the row-major V tile through the transposing LDS read (ds_read_b64_tr_b16), so no
// matrix instruction and no conversion is spent on the transpose.  Q (pre-scaled by scale * log2 e) and P are single
// f16 operands, as in the prefill kernel: 8 matrix instructions a tile where the general kernel issues 24, and 8 exp2.
// Scores are taken relative to a lazily moved reference that enters as the accumulator's initial value, so the common
// tile has no cross-lane step at all.
//
// Merging the key ranges inside this kernel (four ranges to a work-group meeting in LDS, a ticket per work-group from a
// per-tile counter, the last work-group adding up what the others left, partials stored and loaded past L2 with
// device-scope accesses and no fence) was built and gives the same results, and is slower than the second launch:
// 20.0 us against 17.3 for the 64 MiB call, 11.6 against 7.4 us for a 4 MiB one -- a device-scope store, the ticket
// and the loads are three dependent trips across the dies at two microseconds each.
constexpr int DEC_STAGES = 3;
constexpr int DEC_KBLK   = 1152;           // 8 rows of K and 128 bytes
constexpr int DEC_KTILE  = 4 * DEC_KBLK;   // 32 keys
constexpr int DEC_VTILE  = 32 * 128;
constexpr float DEC_SUM_LIMIT = 2048.0f;   // a lane's 8 probabilities of a tile may add up to this before the reference moves

typedef __attribute__((address_space(3))) char fa_lds_char;

__device__ __forceinline__ void dec_dma16(const char * base, uint32_t off, uint32_t lds) {
    // 16 bytes per lane from global memory (uniform base + per-lane offset) straight into LDS at lds + 16 lane
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt" ::"v"(off), "s"(base), "s"(lds) : "memory");
}

__device__ __forceinline__ half8_t dec_tr8(const fa_lds_char * p) { // keys 4j .. 4j+3 and 16 + 4j .. of one d
    typedef short short4_t __attribute__((ext_vector_type(4)));
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3))) *) p);
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3))) *) (p + 16 * 128));
    return __builtin_bit_cast(half8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

__global__ __launch_bounds__(64) void fattn_dec64_kernel(const fa_args a) {
    constexpr int D = 64;
    __shared__ __attribute__((aligned(1024))) char k_lds[DEC_STAGES + 1][DEC_KTILE]; // (the last one: a tile with keys of the second pair)
    __shared__ __attribute__((aligned(1024))) char v_lds[DEC_STAGES + 1][DEC_VTILE];
    const int lane = threadIdx.x;
    const int j = lane >> 4, c = lane & 15;
    if (a.has_kvs && blockIdx.z == 0) { // the folded cache write: see fattn_cols16_kernel
        if (blockIdx.x != 0) return;
        if (blockIdx.y == 0) {
            double tk, tv;
            if (a.kvs_k.vec && a.kvs_v.vec) kvs_wave_totals<true, true>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
            else if (a.kvs_k.vec)           kvs_wave_totals<true, false>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
            else if (a.kvs_v.vec)           kvs_wave_totals<false, true>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
            else                            kvs_wave_totals<false, false>(a.kvs_k, a.kvs_v, lane, false, tk, tv);
            if (lane == 0) *a.kvs_out = kvs_scalar((float) tk, (float) tv, a.kvs_scale, a.kvs_bias);
        } else {
            const uint32_t first = (blockIdx.y - 1) * 64 + lane, step = (gridDim.y - 1) * 64;
            double unused = 0.0;
            const uint32_t nk = kvs_units(a.kvs_k, a.kvs_k.vec != 0), nv = kvs_units(a.kvs_v, a.kvs_v.vec != 0);
            if (a.kvs_k.vec) { for (uint32_t e = first; e < nk; e += step) kvs_unit<true>(a.kvs_k, e, true, unused); }
            else             { for (uint32_t e = first; e < nk; e += step) kvs_unit<false>(a.kvs_k, e, true, unused); }
            if (a.kvs_v.vec) { for (uint32_t e = first; e < nv; e += step) kvs_unit<true>(a.kvs_v, e, true, unused); }
            else             { for (uint32_t e = first; e < nv; e += step) kvs_unit<false>(a.kvs_v, e, true, unused); }
        }
        return;
    }
    const int ct = blockIdx.x, sp = blockIdx.y, bg = (int) blockIdx.z - (a.has_kvs ? 1 : 0);
    const int b  = fa_div(bg, a.inv_hkv);
    const int g  = bg - b * a.Hkv;
    const int tile = bg * a.n_col_tiles + ct;
    const int  ncols  = a.n_q * a.gqa;
    const int  col    = ct * 16 + c;
    const bool col_ok = col < ncols;
    const int  iq1    = col_ok ? fa_div(col, a.inv_gqa) : 0;
    const int  head   = g * a.gqa + (col_ok ? col - iq1 * a.gqa : 0);
    const int  bk     = a.rk3 == 1 ? b : b / a.rk3;

    float4_t qraw[2][2];
    {
        const float * qp = (const float *) (a.q + (uint64_t) iq1 * a.nbq1 + (uint64_t) head * a.nbq2 + (uint64_t) b * a.nbq3) + 16 * j;
#pragma unroll
        for (int p = 0; p < 2; ++p) { qraw[p][0] = ((const float4_t *) (qp + 8 * p))[0]; qraw[p][1] = ((const float4_t *) (qp + 8 * p))[1]; }
    }

    const int kv0 = sp * a.chunk, kv1 = min(a.n_kv, kv0 + a.chunk);
    const int ntile = (kv1 - kv0 + 31) / 32;
    // With a second pair of tensors (the step's own keys behind the cached ones) the tiles that lie wholly in the cache
    // stream as described; a tile with later keys is put together lane by lane -- each row from the tensor that holds
    // it, F32 rows rounded to f16 as a CAST node would round them -- into a buffer of its own, in the layout the direct
    // loads leave.  The first such tile is fetched before the walk begins and consumed in its turn (after the cached
    // tiles, as the one-tensor call consumes it: the results are the same bits); further ones are fetched as they come.
    const int ndma = a.k2 ? min(ntile, max(0, (a.n_kv1 - kv0) / 32)) : ntile;

    // ---- direct loads: an instruction copies 8 rows; lane = (row lane / 8, chunk position lane % 8), the chunk it
    //      fetches is the position un-swizzled
    const char * kg = a.k + (uint64_t) g * a.nbk2 + (uint64_t) bk * a.nbk3;
    const char * vg = a.v + (uint64_t) g * a.nbv2 + (uint64_t) bk * a.nbv3;
    const uint32_t k_base = (uint32_t) (uintptr_t) (fa_lds_char *) &k_lds[0][0];
    const uint32_t v_base = (uint32_t) (uintptr_t) (fa_lds_char *) &v_lds[0][0];
    const int dr = lane >> 3, dp = lane & 7;
    const uint32_t kch = (uint32_t) ((dp ^ dr) << 4), vch = (uint32_t) ((dp ^ (2 * (dr & 3))) << 4);
    const uint32_t kof = (uint32_t) dr * (uint32_t) a.nbk1 + kch, vof = (uint32_t) dr * (uint32_t) a.nbv1 + vch;
    // tiles are sent in order: the next tile's row pointers are kept and moved on by 8 rows per instruction
    const uint64_t k8 = 8 * a.nbk1, v8 = 8 * a.nbv1;
    const char * knext = kg + (uint64_t) kv0 * a.nbk1;
    const char * vnext = vg + (uint64_t) kv0 * a.nbv1;
    int kb_next = kv0;
    auto issue = [&](int stage) { // the next tile of this wave's range into `stage`: always 8 loads
        const uint32_t kl = k_base + stage * DEC_KTILE, vl = v_base + stage * DEC_VTILE;
        if (kb_next + 32 <= a.n_kv) { // wave-uniform
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                dec_dma16(knext, kof, kl + u * DEC_KBLK);
                dec_dma16(vnext, vof, vl + u * 1024);
                knext += k8;
                vnext += v8;
            }
        } else { // the cache's last rows: clamped (their scores are switched off)
            const int last = a.n_kv - 1 - kb_next;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int r = min(8 * u + dr, last);
                dec_dma16(knext, (uint32_t) r * (uint32_t) a.nbk1 + kch, kl + u * DEC_KBLK);
                dec_dma16(vnext, (uint32_t) r * (uint32_t) a.nbv1 + vch, vl + u * 1024);
            }
        }
        kb_next += 32;
    };
#pragma unroll
    for (int t = 0; t < DEC_STAGES; ++t)
        if (t < ndma) issue(t);
    const char * kg2 = nullptr, * vg2 = nullptr;
    if (a.k2) {
        kg2 = a.k2 + (uint64_t) g * a.nbk2b + (uint64_t) bk * a.nbk3b;
        vg2 = a.v2 + (uint64_t) g * a.nbv2b + (uint64_t) bk * a.nbv3b;
    }
    auto fill_mixed = [&](int kb) { // the 32 keys from kb on into the last buffer
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int key = min(kb + 8 * u + dr, a.n_kv - 1);
            const int ck = dp ^ dr, cv = dp ^ (2 * (dr & 3)); // the chunks this lane's positions hold
            half8_t kh, vh;
            if (key < a.n_kv1) {
                kh = *(const half8_t *) (kg + (uint64_t) key * a.nbk1 + ck * 16);
                vh = *(const half8_t *) (vg + (uint64_t) key * a.nbv1 + cv * 16);
            } else if (a.seg2_f32) {
                const float4_t * kp = (const float4_t *) (kg2 + (uint64_t) (key - a.n_kv1) * a.nbk1b + ck * 32);
                const float4_t * vp = (const float4_t *) (vg2 + (uint64_t) (key - a.n_kv1) * a.nbv1b + cv * 32);
                const float4_t k0 = kp[0], k1 = kp[1], v0 = vp[0], v1 = vp[1];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    kh[i] = (_Float16) k0[i]; kh[4 + i] = (_Float16) k1[i];
                    vh[i] = (_Float16) v0[i]; vh[4 + i] = (_Float16) v1[i];
                }
            } else {
                kh = *(const half8_t *) (kg2 + (uint64_t) (key - a.n_kv1) * a.nbk1b + ck * 16);
                vh = *(const half8_t *) (vg2 + (uint64_t) (key - a.n_kv1) * a.nbv1b + cv * 16);
            }
            *(half8_t *) &k_lds[DEC_STAGES][u * DEC_KBLK + lane * 16] = kh;
            *(half8_t *) &v_lds[DEC_STAGES][u * 1024 + lane * 16] = vh;
        }
    };
    if (ndma < ntile) fill_mixed(kv0 + 32 * ndma);

    // ---- Q^T operand: column c, d = 16 j + 8 p + i, pre-scaled (a.scale carries log2 e)
    half8_t qh[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        float4_t x0 = qraw[p][0] * a.scale, x1 = qraw[p][1] * a.scale;
        if (!col_ok) { x0 = float4_t{0, 0, 0, 0}; x1 = float4_t{0, 0, 0, 0}; }
#pragma unroll
        for (int i = 0; i < 4; ++i) { qh[p][i] = (_Float16) x0[i]; qh[p][4 + i] = (_Float16) x1[i]; }
    }

    // ---- operand addresses inside a stage
    uint32_t kad[2], vad[4];
    {
        const int r8 = c & 7;
#pragma unroll
        for (int p = 0; p < 2; ++p) kad[p] = (uint32_t) ((c >> 3) * DEC_KBLK + r8 * 128 + (((2 * j + p) ^ r8) << 4)); // + 2 DEC_KBLK for keys 16 ..
#pragma unroll
        for (int dt = 0; dt < 4; ++dt)
            vad[dt] = (uint32_t) ((4 * j + (c >> 2)) * 128 + (((2 * dt + ((c & 3) >> 1)) ^ (2 * (c >> 2))) << 4) + 8 * (c & 1));
    }
    const fa_lds_char * const k_lds0 = (const fa_lds_char *) &k_lds[0][0];
    const fa_lds_char * const v_lds0 = (const fa_lds_char *) &v_lds[0][0];

    float4_t o[4], negm = float4_t{0, 0, 0, 0};
#pragma unroll
    for (int dt = 0; dt < 4; ++dt) o[dt] = float4_t{0, 0, 0, 0};
    float l = 0.0f;
    bool  seen = false, all_seen = false;

    typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
    auto probs = [&](const float4_t (&s)[2], int4_t & pb, float & lt) {
        half2_t acc = half2_t{(_Float16) 0.0f, (_Float16) 0.0f};
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int r = 0; r < 4; r += 2) {
                const fp16x2 pr = __builtin_amdgcn_cvt_pkrtz(__builtin_amdgcn_exp2f(s[h][r]), __builtin_amdgcn_exp2f(s[h][r + 1]));
                pb[2 * h + (r >> 1)] = __builtin_bit_cast(int, pr);
                acc += __builtin_bit_cast(half2_t, pr);
            }
        lt = (float) acc[0] + (float) acc[1];
    };

    for (int t = 0; t < ntile; ++t) {
        const bool streamed = t < ndma; // wave-uniform
        const int stage = streamed ? t % DEC_STAGES : DEC_STAGES;
        const int kb = kv0 + 32 * t;
        if (streamed) {
            // this tile has landed once at most the younger tiles' loads are outstanding (8 each)
            const int younger = min(DEC_STAGES - 1, ndma - 1 - t);
            if (younger >= 2)      asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
            else if (younger == 1) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
            else                   asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else if (t > ndma) {
            fill_mixed(kb); // (the buffer's previous tile is in registers: the wait below)
        }
        half8_t kk[2][2], vv[4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int p = 0; p < 2; ++p) kk[h][p] = *(const __attribute__((address_space(3))) half8_t *) (k_lds0 + stage * DEC_KTILE + kad[p] + h * 2 * DEC_KBLK);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) vv[dt] = dec_tr8(v_lds0 + stage * DEC_VTILE + vad[dt]);
        __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0): the stage is in registers, the tile three ahead may overwrite it
        if (t + DEC_STAGES < ndma) issue(stage);

        float4_t s[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            s[h] = mfma16(kk[h][0], qh[0], negm);
            s[h] = mfma16(kk[h][1], qh[1], s[h]);
        }
        int4_t pb;
        float  lt;
        probs(s, pb, lt);
        const bool tail = kb + 32 > kv1; // wave-uniform
        if (tail || !all_seen || __builtin_amdgcn_ballot_w64(!(lt <= DEC_SUM_LIMIT)) != 0) {
            if (tail) {
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int r = 0; r < 4; ++r) s[h][r] = kb + 16 * h + 4 * j + r < kv1 ? s[h][r] : -INFINITY;
            }
            float cm = fmaxf(fmaxf(fmaxf(s[0][0], s[0][1]), fmaxf(s[0][2], s[0][3])), fmaxf(fmaxf(s[1][0], s[1][1]), fmaxf(s[1][2], s[1][3])));
            cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
            cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
            // move the reference: up to the new maximum, or (first visible key of the column) onto it wherever it lies
            const bool  vis   = cm != -INFINITY;
            const float delta = !vis ? 0.0f : (seen ? fmaxf(cm, 0.0f) : cm);
            seen = seen || vis;
            const float f = __builtin_amdgcn_exp2f(-delta);
            s[0] -= delta;
            s[1] -= delta;
            negm -= delta;
#pragma unroll
            for (int dt = 0; dt < 4; ++dt) o[dt] *= f;
            l *= f;
            probs(s, pb, lt);
            all_seen = __builtin_amdgcn_ballot_w64(!seen) == 0;
        }
        l += lt;
        const half8_t p8 = __builtin_bit_cast(half8_t, pb);
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) o[dt] = mfma16(vv[dt], p8, o[dt]);
    }

    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    const float m = seen ? -negm[0] : -INFINITY;

    // lane (j, c), tile dt, register r holds d = 16 dt + 4 j + r of column c
    if (!col_ok) return;
    if (a.n_splits == 1) {
        const bool  has_sink = a.sinks != nullptr, has_addend = a.add1 != nullptr;
        const float sink = has_sink ? a.sinks[head] : 0.0f, addend = has_addend ? *a.add1 : 0.0f;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) fa_finish(a, o[dt], m, l, b, iq1, head, D, 16 * dt + 4 * j, has_sink, sink, has_addend, addend);
    } else {
        const uint64_t pbase = ((uint64_t) tile * a.n_splits + sp) * 16 + c;
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) *(float4_t *) (a.part_o + pbase * D + 16 * dt + 4 * j) = o[dt];
        if (j == 0) { a.part_ml[pbase * 2] = m; a.part_ml[pbase * 2 + 1] = l; }
    }
}

// whether the streaming kernel takes this launch (decided from the arguments alone); VX_FA_DEC=0 keeps every launch on
// the general kernel
bool fa_dec64_takes(const fa_args & a, int D, bool kv_f32) {
    static const bool off = [] { const char * e = getenv("VX_FA_DEC"); return e && atoi(e) == 0; }();
    if (off) return false;
    return D == 64 && !kv_f32 && !a.mask && a.softcap == 0.0f && a.n_kv > 64 && a.nbk1 < (1u << 28) && a.nbv1 < (1u << 28);
}
void launch_dec64(const fa_args & a, hipStream_t st) {
    const dim3 grid((unsigned) a.n_col_tiles, (unsigned) a.n_splits, (unsigned) (a.ne3 * a.Hkv + (a.has_kvs ? 1 : 0)));
    vx_launch(fattn_dec64_kernel, grid, dim3(64), 0, st, a);
}

template <int D, bool KV_F32>
void launch_cols16(const fa_args & a, hipStream_t st) {
    const dim3 grid((unsigned) a.n_col_tiles, (unsigned) a.n_splits, (unsigned) (a.ne3 * a.Hkv + (a.has_kvs ? 1 : 0))), block(64);
    if constexpr (D == 64 && !KV_F32) {
        if (a.k2 && a.seg2_f32) { // an F16 cache and the step's F32 keys
            if (a.softcap != 0.0f) vx_launch(fattn_cols16_kernel<D, false, true, true, 2>, grid, block, 0, st, a);
            else if (a.mask)       vx_launch(fattn_cols16_kernel<D, false, true, false, 2>, grid, block, 0, st, a);
            else                   vx_launch(fattn_cols16_kernel<D, false, false, false, 2>, grid, block, 0, st, a);
            return;
        }
    }
    if (a.k2) {
        if (a.softcap != 0.0f) vx_launch(fattn_cols16_kernel<D, KV_F32, true, true, 1>, grid, block, 0, st, a);
        else if (a.mask)       vx_launch(fattn_cols16_kernel<D, KV_F32, true, false, 1>, grid, block, 0, st, a);
        else                   vx_launch(fattn_cols16_kernel<D, KV_F32, false, false, 1>, grid, block, 0, st, a);
        return;
    }
    if (a.softcap != 0.0f) { // rare: always take the masked variant
        vx_launch(fattn_cols16_kernel<D, KV_F32, true, true, 0>, grid, block, 0, st, a);
    } else if (a.n_kv <= 16 && a.n_splits == 1) {
        if (a.mask) vx_launch(fattn_cols16_kernel<D, KV_F32, true, false, 0, true>, grid, block, 0, st, a);
        else        vx_launch(fattn_cols16_kernel<D, KV_F32, false, false, 0, true>, grid, block, 0, st, a);
    } else if (a.mask) {
        vx_launch(fattn_cols16_kernel<D, KV_F32, true, false, 0>, grid, block, 0, st, a);
    } else {
        vx_launch(fattn_cols16_kernel<D, KV_F32, false, false, 0>, grid, block, 0, st, a);
    }
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
    if (q->ne[3] * k->ne[2] > 65534) return 0; // (batch entry x KV head is one dimension of the grid, plus one slice for a folded cache write)
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
    return vx_flash_attn_ext_add1(q, k, v, mask, sinks, nullptr, dst, scale, max_bias, logit_softcap, stream);
}

// K/V as one tensor each (k2 == v2 == null) or as two key segments: k, v hold keys 0 .. n_kv1-1 and
// k2, v2 the rest; kall / vall describe the whole (for the one-segment case they are k and v).
static vx_status fa_run(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * k2, const vx_tensor * v2,
                        const vx_tensor * kall, const vx_tensor * vall, const vx_tensor * mask, const float * sinks,
                        const float * addend, const vx_tensor * dst, float scale, float max_bias, float logit_softcap,
                        hipStream_t st, const vx_tensor * ks_src = nullptr, const vx_tensor * ks_slot = nullptr,
                        const vx_tensor * vs_src = nullptr, const vx_tensor * vs_slot = nullptr, float kvs_scale = 0.0f,
                        float kvs_bias = 0.0f, void * fixed_ws = nullptr, size_t fixed_ws_bytes = 0);

extern "C" vx_status vx_flash_attn_ext_add1(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                            const vx_tensor * mask, const float * sinks, const float * addend,
                                            const vx_tensor * dst, float scale, float max_bias, float logit_softcap,
                                            vx_stream stream) {
    if (!q || !k || !v || !dst || !q->data || !k->data || !v->data || !dst->data || (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext: null tensor");
    if (!vx_supports_flash_attn_ext(q, k, v, mask, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: needs q F32, k/v both F16 or both F32, D in {64,128}, dense rows, 16-byte aligned strides, contiguous dst, F16 mask");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (uintptr_t) dst->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: tensor data must be 16-byte aligned");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext: max_bias > 0 requires a mask");

    hipStream_t st = (hipStream_t) stream;
    {   // many query rows: the LDS-tiled kernel
        static const bool no_prefill = getenv("VX_FA_NO_PREFILL") != nullptr;
        if (!no_prefill) {
            const vx_status rc = vx_fattn_prefill(q, k, v, mask, sinks, addend, dst, scale, max_bias, logit_softcap, st);
            if (rc != VX_ERR_UNSUPPORTED) return rc;
        }
    }
    return fa_run(q, k, v, nullptr, nullptr, k, v, mask, sinks, addend, dst, scale, max_bias, logit_softcap, st);
}

// CONCAT(k_past, k_cur) , CONCAT(v_past, v_cur) , FLASH_ATTN_EXT as one launch that reads both segments
// where they lie.  The whole of K (V) has the first segment's shape with ne[1] = the two key counts added.
// The second segment may be F32 behind an F16 first one (head_dim 64): the step's keys as the projections left them.
static bool kv2_whole(const vx_tensor * a, const vx_tensor * b, vx_tensor * whole) {
    if (!a || !b || !vx_positive(a) || !vx_positive(b)) return false;
    if (a->type != b->type && !(a->type == VX_TYPE_F16 && b->type == VX_TYPE_F32 && a->ne[0] == 64)) return false;
    if (a->ne[0] != b->ne[0] || a->ne[2] != b->ne[2] || a->ne[3] != b->ne[3]) return false;
    if (b->nb[0] != vx_type_size(b->type)) return false;
    for (int i = 1; i < 4; ++i) if (b->nb[i] % 16) return false;
    *whole = *a;
    whole->ne[1] = a->ne[1] + b->ne[1];
    return true;
}

extern "C" int vx_supports_flash_attn_ext_kv2(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                              const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                              const vx_tensor * dst) {
    vx_tensor kall, vall;
    if (!q || !kv2_whole(k_past, k_cur, &kall) || !kv2_whole(v_past, v_cur, &vall)) return 0;
    if (k_past->ne[1] != v_past->ne[1] || k_cur->type != v_cur->type) return 0;
    if (!vx_supports_flash_attn_ext(q, &kall, &vall, mask, dst)) return 0;
    // a shape the LDS-tiled kernel would take as one tensor stays with it (same results either way)
    return vx_fattn_prefill_accepts(q, &kall, 0.0f) ? 0 : 1;
}

extern "C" vx_status vx_flash_attn_ext_kv2(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                           const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                           const float * sinks, const vx_tensor * dst, float scale, float max_bias,
                                           float logit_softcap, vx_stream stream) {
    if (!q || !k_past || !k_cur || !v_past || !v_cur || !dst || !q->data || !k_past->data || !k_cur->data || !v_past->data ||
        !v_cur->data || !dst->data || (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext_kv2: null tensor");
    if (!vx_supports_flash_attn_ext_kv2(q, k_past, k_cur, v_past, v_cur, mask, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_kv2: two K/V segments of one type and head layout, otherwise as flash_attn_ext; decode-sized query counts");
    if (!aligned16(q) || !aligned16(k_past) || !aligned16(v_past) || !aligned16(k_cur) || !aligned16(v_cur) || (uintptr_t) dst->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_kv2: tensor data must be 16-byte aligned");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext_kv2: max_bias > 0 requires a mask");
    vx_tensor kall, vall;
    kv2_whole(k_past, k_cur, &kall);
    kv2_whole(v_past, v_cur, &vall);
    return fa_run(q, k_past, v_past, k_cur, v_cur, &kall, &vall, mask, sinks, nullptr, dst, scale, max_bias, logit_softcap, (hipStream_t) stream);
}

// The reference's decode attention block in two kernels: attention over cached + current keys, with the cache
// write and its ordering scalar (CPY CONT SUM x2, ADD, SCALE, ADD1; src/minicpm.cpp:682-713) folded into the
// kernel that merges the key-range partials.  k_src / v_src are the CPY sources (the same values as k_cur /
// v_cur, in the shape the reference copies them), k_slot / v_slot the cache views they are written to.
extern "C" int vx_supports_flash_attn_ext_kv2_store(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                                    const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                                    const vx_tensor * k_src, const vx_tensor * k_slot, const vx_tensor * v_src,
                                                    const vx_tensor * v_slot, const vx_tensor * dst) {
    if (!vx_supports_flash_attn_ext_kv2(q, k_past, k_cur, v_past, v_cur, mask, dst)) return 0;
    if (!kvs_side_ok(k_src, k_slot) || !kvs_side_ok(v_src, v_slot)) return 0;
    vx_tensor kall;
    kv2_whole(k_past, k_cur, &kall);
    int n_splits, chunk;
    fa_split_plan(fa_tiles(q, &kall), (int) kall.ne[1], &n_splits, &chunk);
    return n_splits > 1; // the write rides on the merge kernel
}

extern "C" vx_status vx_flash_attn_ext_kv2_store(const vx_tensor * q, const vx_tensor * k_past, const vx_tensor * k_cur,
                                                 const vx_tensor * v_past, const vx_tensor * v_cur, const vx_tensor * mask,
                                                 const float * sinks, const vx_tensor * k_src, const vx_tensor * k_slot,
                                                 const vx_tensor * v_src, const vx_tensor * v_slot, const vx_tensor * dst, float scale,
                                                 float max_bias, float logit_softcap, float sync_scale, float sync_bias,
                                                 vx_stream stream) {
    if (!q || !k_past || !k_cur || !v_past || !v_cur || !k_src || !k_slot || !v_src || !v_slot || !dst || !q->data || !k_past->data ||
        !k_cur->data || !v_past->data || !v_cur->data || !k_src->data || !k_slot->data || !v_src->data || !v_slot->data || !dst->data ||
        (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext_kv2_store: null tensor");
    if (!vx_supports_flash_attn_ext_kv2_store(q, k_past, k_cur, v_past, v_cur, mask, k_src, k_slot, v_src, v_slot, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_kv2_store: as flash_attn_ext_kv2 with more than 256 keys, F32 cache writes of at most 16384 elements");
    if (!aligned16(q) || !aligned16(k_past) || !aligned16(v_past) || !aligned16(k_cur) || !aligned16(v_cur) || (uintptr_t) dst->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_kv2_store: tensor data must be 16-byte aligned");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext_kv2_store: max_bias > 0 requires a mask");
    vx_tensor kall, vall;
    kv2_whole(k_past, k_cur, &kall);
    kv2_whole(v_past, v_cur, &vall);
    return fa_run(q, k_past, v_past, k_cur, v_cur, &kall, &vall, mask, sinks, nullptr, dst, scale, max_bias, logit_softcap, (hipStream_t) stream,
                  k_src, k_slot, v_src, v_slot, sync_scale, sync_bias);
}

// attention_forward at prefill size (src/minicpm.cpp:682-713): FLASH_ATTN_EXT over the projections' own K/V, then the
// cache write, its two sums, the ordering scalar and the ADD1 on the attention's result.  The write and the scalar are
// launched first and the scalar joins the attention's epilogue, so the result is stored once.
struct pf_store_ctx {
    const vx_tensor * k_src, * k_slot, * v_src, * v_slot;
    float scale, bias;
};
constexpr size_t PF_STORE_FRONT = 4096, PF_STORE_ADDEND_AT = 2048; // 256 block totals, then the scalar

static vx_status pf_store_launch(void * front, void * ctx, hipStream_t st) {
    const pf_store_ctx * c = (const pf_store_ctx *) ctx;
    return vx_kv_store_scalar(c->k_src, c->k_slot, c->v_src, c->v_slot, c->scale, c->bias, front, (float *) ((char *) front + PF_STORE_ADDEND_AT), st);
}

extern "C" int vx_supports_flash_attn_ext_store(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                                const vx_tensor * k_src, const vx_tensor * k_slot, const vx_tensor * v_src,
                                                const vx_tensor * v_slot, const vx_tensor * dst, float logit_softcap) {
    static const bool off = getenv("VX_FA_NO_PREFILL") != nullptr;
    if (off || !vx_supports_flash_attn_ext(q, k, v, mask, dst)) return 0;
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (uintptr_t) dst->data % 16) return 0;
    if (!vx_fattn_prefill_accepts(q, k, logit_softcap)) return 0;
    return vx_kv_store_scalar_ok(k_src, k_slot, v_src, v_slot) ? 1 : 0;
}

extern "C" vx_status vx_flash_attn_ext_store(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                             const float * sinks, const vx_tensor * k_src, const vx_tensor * k_slot,
                                             const vx_tensor * v_src, const vx_tensor * v_slot, const vx_tensor * dst, float scale,
                                             float max_bias, float logit_softcap, float sync_scale, float sync_bias, vx_stream stream) {
    if (!q || !k || !v || !k_src || !k_slot || !v_src || !v_slot || !dst || !q->data || !k->data || !v->data || !k_src->data ||
        !k_slot->data || !v_src->data || !v_slot->data || !dst->data || (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext_store: null tensor");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext_store: max_bias > 0 requires a mask");
    if (!vx_supports_flash_attn_ext_store(q, k, v, mask, k_src, k_slot, v_src, v_slot, dst, logit_softcap)) {
        // not this form's shapes (or the LDS-tiled kernel switched off since the caller asked): the two calls it stands for
        if (!vx_supports_flash_attn_ext(q, k, v, mask, dst) || !vx_supports_kv_store_sync(k_src, k_slot, v_src, v_slot, dst, dst))
            return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_store: shapes that neither the one call nor flash_attn_ext followed by kv_store_sync takes");
        const vx_status rc = vx_flash_attn_ext(q, k, v, mask, sinks, dst, scale, max_bias, logit_softcap, stream);
        return rc != VX_OK ? rc : vx_kv_store_sync(k_src, k_slot, v_src, v_slot, dst, dst, sync_scale, sync_bias, stream);
    }
    pf_store_ctx c{ k_src, k_slot, v_src, v_slot, sync_scale, sync_bias };
    const vx_pf_front front{ PF_STORE_FRONT, PF_STORE_ADDEND_AT, pf_store_launch, &c };
    return vx_fattn_prefill(q, k, v, mask, sinks, nullptr, dst, scale, max_bias, logit_softcap, (hipStream_t) stream, &front);
}

// The same block with the o projection and its residual update behind it (src/minicpm.cpp:708-715, 762-768): the
// attention's epilogue rounds its result to f16 straight into the projection's activation tiles, so the tokens x hidden
// attention output is neither stored in fp32 nor read back and laid out again.
struct pf_store_proj_ctx {
    pf_store_ctx store;
    void *       front;
};

static vx_status pf_store_proj_launch(void * front, void * ctx, hipStream_t st) {
    pf_store_proj_ctx * c = (pf_store_proj_ctx *) ctx;
    c->front = front;
    return pf_store_launch(front, &c->store, st);
}

// the tensor attn describes, in the attention's own shape [head_dim, heads, tokens, batch] (the same dense memory order)
static vx_tensor pf_attn_shape(const vx_tensor * q, const vx_tensor * attn) {
    vx_tensor ad = *attn;
    ad.ne[0] = q->ne[0]; ad.ne[1] = q->ne[2]; ad.ne[2] = q->ne[1]; ad.ne[3] = q->ne[3];
    ad.nb[0] = 4; ad.nb[1] = (uint64_t) ad.ne[0] * 4; ad.nb[2] = ad.nb[1] * (uint64_t) ad.ne[1]; ad.nb[3] = ad.nb[2] * (uint64_t) ad.ne[2];
    return ad;
}

// attn: the attention's result as the projection reads it, [hidden, tokens (, batch)], dense; the same memory order as the
// attention's own [head_dim, heads, tokens, batch]
static bool pf_proj_geometry(const vx_tensor * q, const vx_tensor * attn, const vx_tensor * w_o, const vx_tensor * residual, const vx_tensor * dst,
                             int act_mode, vx_pf_front * front, size_t * proj_bytes) {
    if (!attn || !w_o || !residual || !dst || attn->type != VX_TYPE_F32 || !vx_is_contiguous(attn)) return false;
    const int64_t hidden = q->ne[0] * q->ne[2], T = q->ne[1], B = q->ne[3];
    if (attn->ne[0] != hidden || vx_nelements(attn) != hidden * T * B) return false;
    const bool flat = attn->ne[1] == T * B && attn->ne[2] == 1 && attn->ne[3] == 1;
    const bool by_batch = attn->ne[1] == T && attn->ne[2] * attn->ne[3] == B;
    if (!flat && !by_batch) return false;
    uint32_t tile_tt = 0, n_kb = 0;
    size_t   tile_bytes = 0;
    if (!vx_proj_tiles_ok(w_o, attn, residual, dst, act_mode, &tile_tt, &n_kb, &tile_bytes, proj_bytes)) return false;
    front->tiles = true; front->tiles_at = PF_STORE_FRONT;
    front->tile_tt = tile_tt;
    front->tile_bs = by_batch && !flat ? n_kb * tile_tt : 0;
    front->tile_ts = by_batch && !flat ? 0 : (uint32_t) T;
    front->bytes = PF_STORE_FRONT + tile_bytes;
    return (int64_t) B * T < ((int64_t) 1 << 31);
}

extern "C" int vx_supports_flash_attn_ext_store_proj(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                                     const vx_tensor * k_src, const vx_tensor * k_slot, const vx_tensor * v_src,
                                                     const vx_tensor * v_slot, const vx_tensor * attn, const vx_tensor * w_o,
                                                     const vx_tensor * residual, const vx_tensor * dst, float logit_softcap, int act_mode) {
    if (!attn || !q) return 0;
    const vx_tensor ad = pf_attn_shape(q, attn);
    if (!vx_supports_flash_attn_ext_store(q, k, v, mask, k_src, k_slot, v_src, v_slot, &ad, logit_softcap)) return 0;
    vx_pf_front front{};
    size_t proj_bytes = 0;
    return pf_proj_geometry(q, attn, w_o, residual, dst, act_mode, &front, &proj_bytes) ? 1 : 0;
}

extern "C" vx_status vx_flash_attn_ext_store_proj(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                                                  const float * sinks, const vx_tensor * k_src, const vx_tensor * k_slot,
                                                  const vx_tensor * v_src, const vx_tensor * v_slot, const vx_tensor * attn,
                                                  const vx_tensor * w_o, const vx_tensor * residual, const vx_tensor * dst, float scale,
                                                  float max_bias, float logit_softcap, float sync_scale, float sync_bias, float res_scale,
                                                  int act_mode, vx_stream stream) {
    if (!q || !k || !v || !k_src || !k_slot || !v_src || !v_slot || !attn || !w_o || !residual || !dst || !q->data || !k->data || !v->data ||
        !k_src->data || !k_slot->data || !v_src->data || !v_slot->data || !attn->data || !w_o->data || !residual->data || !dst->data ||
        (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext_store_proj: null tensor");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext_store_proj: max_bias > 0 requires a mask");
    if (!vx_supports_flash_attn_ext_store_proj(q, k, v, mask, k_src, k_slot, v_src, v_slot, attn, w_o, residual, dst, logit_softcap, act_mode)) {
        // not this form's shapes (or a kernel it needs switched off since the caller asked): the calls it stands for, through attn's memory
        if (attn->type != VX_TYPE_F32 || !vx_is_contiguous(attn) || vx_nelements(attn) != vx_nelements(q))
            return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_store_proj: attn must be the attention's dense F32 result");
        {   // (this route stores the attention's result in attn's memory and the projection reads it there: dst must lie apart)
            const char * a0 = (const char *) attn->data, * d0 = (const char *) dst->data;
            const size_t ab = (size_t) vx_nelements(attn) * 4, db = (size_t) ((dst->ne[1] - 1) * dst->nb[1] + (dst->ne[2] - 1) * dst->nb[2] + (dst->ne[3] - 1) * dst->nb[3]) + (size_t) dst->ne[0] * 4;
            if (a0 < d0 + db && d0 < a0 + ab) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_store_proj: dst overlaps attn and the shapes need attn's memory");
        }
        const vx_tensor ad = pf_attn_shape(q, attn);
        const vx_status rc = vx_flash_attn_ext_store(q, k, v, mask, sinks, k_src, k_slot, v_src, v_slot, &ad, scale, max_bias, logit_softcap, sync_scale,
                                                     sync_bias, stream);
        return rc != VX_OK ? rc : vx_mul_mat_scale_add(w_o, attn, residual, dst, res_scale, act_mode, stream);
    }
    pf_store_proj_ctx c{ { k_src, k_slot, v_src, v_slot, sync_scale, sync_bias }, nullptr };
    vx_pf_front front{ PF_STORE_FRONT, PF_STORE_ADDEND_AT, pf_store_proj_launch, &c };
    size_t proj_bytes = 0;
    if (!pf_proj_geometry(q, attn, w_o, residual, dst, act_mode, &front, &proj_bytes)) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_store_proj: tile geometry");
    hipStream_t st = (hipStream_t) stream;
    {   // one block for both phases: the projection's request must not find the block too small once the attention has run
        // (a request that grows the block moves it, and under a capture growth is refused)
        void * p = nullptr;
        const vx_status rc = vx_workspace(st, front.bytes + proj_bytes, &p);
        if (rc != VX_OK) return rc;
    }
    const vx_tensor ad = pf_attn_shape(q, attn); // (never written: the result leaves as tiles)
    vx_status rc = vx_fattn_prefill(q, k, v, mask, sinks, nullptr, &ad, scale, max_bias, logit_softcap, st, &front);
    if (rc != VX_OK) return rc == VX_ERR_UNSUPPORTED ? vx_fail(rc, "flash_attn_ext_store_proj: the LDS-tiled kernel declined") : rc;
    // the projection: its own needs go behind the front (a block that a larger request replaces stays valid)
    return vx_proj_tiles_run(w_o, attn, residual, dst, res_scale, act_mode, (const char *) c.front + PF_STORE_FRONT, front.bytes, st);
}

// ---- the entry point that allocates nothing ------------------------------------------------------------
// The key-range partials of vx_flash_attn_ext_static live in a fixed array in device memory that is part of the
// loaded code object: every GPU the library runs on holds its own copy, at its own address, until the process
// ends.  In host code the array's name is only a handle for hipGetSymbolAddress -- the address kernels must be
// given is looked up once per device and kept.
constexpr size_t FA_STATIC_SCRATCH_BYTES = VX_FLASH_ATTN_EXT_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[FA_STATIC_SCRATCH_BYTES];

constexpr int FA_MAX_DEVICES = 64;
static void *     g_scratch_ptr[FA_MAX_DEVICES];
static std::mutex g_scratch_mutex;

// the address of `scratch` on the current device, looked up on the first request
static vx_status fa_static_scratch(void ** ptr) {
    int dev = 0;
    VX_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= FA_MAX_DEVICES) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_static: device ordinal %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void * p = nullptr;
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p)
            return vx_fail(VX_ERR_HIP, "hipGetSymbolAddress(scratch) failed on device %d: %s", dev, hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return VX_OK;
}

vx_status vx_fattn_static_setup(void) {
    void * p = nullptr;
    return fa_static_scratch(&p);
}

extern "C" vx_status vx_flash_attn_ext_static(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v,
                                              const vx_tensor * mask, const float * sinks, const vx_tensor * dst,
                                              float scale, float max_bias, float logit_softcap, vx_stream stream) {
    if (!q || !k || !v || !dst || !q->data || !k->data || !v->data || !dst->data || (mask && !mask->data))
        return vx_fail(VX_ERR_INVALID, "flash_attn_ext_static: null tensor");
    if (!vx_supports_flash_attn_ext(q, k, v, mask, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_static: needs q F32, k/v both F16 or both F32, D in {64,128}, dense rows, 16-byte aligned strides, contiguous dst, F16 mask");
    if (!aligned16(q) || !aligned16(k) || !aligned16(v) || (uintptr_t) dst->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_static: tensor data must be 16-byte aligned");
    if (max_bias > 0.0f && !mask) return vx_fail(VX_ERR_INVALID, "flash_attn_ext_static: max_bias > 0 requires a mask");
    void * ws = nullptr;
    const vx_status rc = fa_static_scratch(&ws);
    if (rc != VX_OK) return rc;
    return fa_run(q, k, v, nullptr, nullptr, k, v, mask, sinks, nullptr, dst, scale, max_bias, logit_softcap, (hipStream_t) stream,
                  nullptr, nullptr, nullptr, nullptr, 0.0f, 0.0f, ws, FA_STATIC_SCRATCH_BYTES);
}

static vx_status fa_run(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * k2, const vx_tensor * v2,
                        const vx_tensor * kall, const vx_tensor * vall, const vx_tensor * mask, const float * sinks,
                        const float * addend, const vx_tensor * dst, float scale, float max_bias, float logit_softcap,
                        hipStream_t st, const vx_tensor * ks_src, const vx_tensor * ks_slot, const vx_tensor * vs_src,
                        const vx_tensor * vs_slot, float kvs_scale, float kvs_bias, void * fixed_ws, size_t fixed_ws_bytes) {
    (void) vall;
    fa_args a;
    a.has_kvs = 0; a.kvs_out = nullptr;
    a.k2 = k2 ? (const char *) k2->data : nullptr; a.v2 = v2 ? (const char *) v2->data : nullptr;
    a.nbk1b = k2 ? k2->nb[1] : 0; a.nbk2b = k2 ? k2->nb[2] : 0; a.nbk3b = k2 ? k2->nb[3] : 0;
    a.nbv1b = v2 ? v2->nb[1] : 0; a.nbv2b = v2 ? v2->nb[2] : 0; a.nbv3b = v2 ? v2->nb[3] : 0;
    a.n_kv1 = (int) k->ne[1];
    a.seg2_f32 = k2 && k2->type == VX_TYPE_F32 && k->type == VX_TYPE_F16;
    a.q = (const char *) q->data; a.k = (const char *) k->data; a.v = (const char *) v->data;
    a.mask = mask ? (const char *) mask->data : nullptr;
    a.sinks = sinks;
    a.add1 = addend;
    a.dst = (float *) dst->data;
    a.part_o = nullptr; a.part_ml = nullptr;
    a.nbq1 = q->nb[1]; a.nbq2 = q->nb[2]; a.nbq3 = q->nb[3];
    a.nbk1 = k->nb[1]; a.nbk2 = k->nb[2]; a.nbk3 = k->nb[3];
    a.nbv1 = v->nb[1]; a.nbv2 = v->nb[2]; a.nbv3 = v->nb[3];
    a.nbm1 = mask ? mask->nb[1] : 0; a.nbm2 = mask ? mask->nb[2] : 0; a.nbm3 = mask ? mask->nb[3] : 0;
    a.n_q = (int) q->ne[1]; a.n_kv = (int) kall->ne[1]; a.Hq = (int) q->ne[2]; a.Hkv = (int) k->ne[2];
    a.gqa = a.Hq / a.Hkv; a.ne3 = (int) q->ne[3]; a.rk3 = (int) (q->ne[3] / k->ne[3]);
    a.nem2 = mask ? (int) mask->ne[2] : 1; a.nem3 = mask ? (int) mask->ne[3] : 1;
    a.scale = scale; a.softcap = logit_softcap; a.max_bias = max_bias;
    // the kernels work in the log2 domain: p = 2^(x*log2(e) - m)
    const float LOG2E = 1.44269504088896341f;
    if (logit_softcap != 0.0f) { a.scale /= logit_softcap; a.softcap *= LOG2E; } // ops.cpp:8173-8175
    else                       { a.scale *= LOG2E; }
    a.n_head_log2 = 1u << (uint32_t) floor(log2((double) a.Hq));
    a.m0 = powf(2.0f, -(max_bias) / a.n_head_log2);
    a.m1 = powf(2.0f, -(max_bias / 2.0f) / a.n_head_log2);

    const int ncols = a.n_q * a.gqa;
    a.n_col_tiles   = (ncols + 15) / 16;
    a.inv_gqa = 1.0f / (float) a.gqa; a.inv_hkv = 1.0f / (float) a.Hkv;
    if (ncols >= (1 << 22) || (int64_t) a.ne3 * a.Hkv > 65534) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: launch too large");
    const int64_t tiles = (int64_t) a.ne3 * a.Hkv * a.n_col_tiles;

    fa_split_plan(tiles, a.n_kv, &a.n_splits, &a.chunk);
    if (ks_src) {
        if (a.n_splits == 1) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_kv2_store: needs a key count that is split across waves");
        kvs_side_fill(a.kvs_k, ks_src, ks_slot);
        kvs_side_fill(a.kvs_v, vs_src, vs_slot);
        a.kvs_scale = kvs_scale; a.kvs_bias = kvs_bias;
        a.has_kvs = 1;
    }

    const int64_t nblocks = tiles * a.n_splits;
    if (nblocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext: launch too large");
    const int D = (int) q->ne[0];
    const bool f32 = k->type == VX_TYPE_F32;

    const bool dec = fa_dec64_takes(a, D, f32);

    if (a.n_splits > 1) {
        const size_t o_bytes  = (size_t) nblocks * 16 * D * sizeof(float);
        const size_t ml_bytes = (size_t) nblocks * 16 * 2 * sizeof(float) + (a.has_kvs ? 16 : 0); // (+ the folded cache write's scalar)
        void * ws = fixed_ws;
        if (fixed_ws) { // the caller's fixed block: nothing is allocated, larger shapes are refused
            if (o_bytes + ml_bytes > fixed_ws_bytes)
                return vx_fail(VX_ERR_UNSUPPORTED, "flash_attn_ext_static: the key-range partials of this shape need %zu bytes, the fixed scratch holds %zu "
                               "(use vx_flash_attn_ext, which allocates)", o_bytes + ml_bytes, fixed_ws_bytes);
        } else {
            vx_status rc = vx_workspace(st, o_bytes + ml_bytes, &ws);
            if (rc != VX_OK) return rc;
        }
        a.part_o  = (float *) ws;
        a.part_ml = (float *) ((char *) ws + o_bytes);
        a.kvs_out = a.has_kvs ? (float *) ((char *) ws + o_bytes + ml_bytes - 16) : nullptr;
    }

    if (dec) launch_dec64(a, st);
    else if (D == 64) { if (f32) launch_cols16<64, true>(a, st); else launch_cols16<64, false>(a, st); }
    else         { if (f32) launch_cols16<128, true>(a, st); else launch_cols16<128, false>(a, st); }
    VX_LAUNCH_CHECK();
    if (a.n_splits > 1) {
        const dim3 grid((unsigned) (a.n_col_tiles * 16), (unsigned) (a.ne3 * a.Hkv));
        const dim3 mblock(64);
        if (D == 64) vx_launch(fattn_merge_kernel<64>, grid, mblock, 0, st, a);
        else         vx_launch(fattn_merge_kernel<128>, grid, mblock, 0, st, a);
        VX_LAUNCH_CHECK();
    }
    return VX_OK;
}
