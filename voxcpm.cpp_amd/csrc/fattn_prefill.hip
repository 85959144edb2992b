// fattn_prefill.hip -- GGML_OP_FLASH_ATTN_EXT for many query rows (prefill) on gfx950: a
// tiled flash-attention kernel on f16 MFMA with K/V tiles staged in LDS and the online
// softmax in fp32.
//
// A work-group (4 waves) owns 256 *columns* of one (batch, KV head): RB = 256 / gqa
// consecutive query rows times the gqa query heads that share the KV head, so one K/V tile
// in LDS serves all of them (the GQA reuse).  Each wave owns 64 columns as four 16-column
// MFMA tiles.  Keys are walked in tiles of 64:
//     S^T = K Q^T     A = K rows from LDS, B = Q^T resident in registers (pre-scaled by
//                     scale * log2 e, rounded to f16)
//     softmax         per column: lane-local over its 8 keys per half tile + xor 16 / 32
//     O^T += V^T P^T  A = V^T from LDS, B = P^T straight from the S^T accumulator registers
// V is transposed on its way into LDS (each thread scatters the 8 halves it loaded), with
// the keys of a tile stored in the order the S^T accumulator layout hands P^T back, so both
// operands are single 16-byte LDS reads.  K/V tiles are double-buffered: global loads for
// tile i+1 are issued before tile i is consumed and written to the other buffer after it.
//
// The mask is data, not a flag: a small pre-pass classifies every (row block, key tile) of it
// as all -inf (tile skipped: the causal upper triangle costs nothing), all zero (no mask
// arithmetic) or mixed (mask values are applied element-wise), so the result equals
// ggml-cpu's for any mask while a causal mask gets causal cost.
//
// Roofline: MFMA-bound in principle (4 * D flops per score); at D = 64 the exp and the
// row statistics (VALU, one instruction per 4 cycles per wave) cost more cycles per score
// than the matrix core does, so the kernel is VALU-bound below the MFMA peak.
#include "vx_common.hpp"

#include <cmath>

namespace {

constexpr int PF_WAVES = 4;
constexpr int PF_COLS  = 256; // columns per work-group
constexpr int PF_CT    = 4;   // 16-column tiles per wave
constexpr int PF_GRP   = 2;   // column tiles scored together before the softmax work
constexpr int PF_KT    = 64;  // keys per tile
constexpr int PF_ROW   = 72;  // LDS row length in halves (64 + 8 pad: 144 bytes, conflict-free b128 reads)
constexpr int PF_MAX_TILES = 1024;
constexpr float PF_LAZY = 8.0f; // log2 units a score may exceed its reference before it is moved

struct pf_args {
    const char * q; const char * k; const char * v; const char * mask;
    const float * sinks;
    const float * add1; // optional scalar added to every output element (a fused GGML_OP_ADD1)
    float * dst;
    const uint8_t * flags; // [nem3][nem2][n_rb][n_tiles]: 0 skip, 1 no mask, 2 apply mask
    uint64_t nbq1, nbq2, nbq3, nbk1, nbk2, nbk3, nbv1, nbv2, nbv3, nbm1, nbm2, nbm3;
    int n_q, n_kv, Hq, Hkv, gqa, ne3, rk3, nem2, nem3;
    int RB, n_rb, n_tiles, n_groups, xcd_map;
    float scale2, max_bias, m0, m1; // scale2 = scale * log2(e)
    uint32_t n_head_log2;
    int kv_f32;
};

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

__device__ __forceinline__ void pk2(half8_t & dst, int i, float a, float b) {
    typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
    const fp16x2 v = __builtin_amdgcn_cvt_pkrtz(a, b);
    dst[i]     = (_Float16) v[0];
    dst[i + 1] = (_Float16) v[1];
}

// "does any of these 8 scores exceed a positive bound" on the bit patterns: as signed integers,
// floats above a positive bound (and NaNs) compare above its pattern, everything negative below.
// Integer max needs none of the canonicalising self-max instructions fmaxf() gets in front of
// operands that come out of the matrix core.
__device__ __forceinline__ int imax8(const float4_t & x, const float4_t & y) {
    const int4_t a = __builtin_bit_cast(int4_t, x), b = __builtin_bit_cast(int4_t, y);
    return max(max(max(a[0], a[1]), max(a[2], a[3])), max(max(b[0], b[1]), max(b[2], b[3])));
}
__device__ __forceinline__ float fmax8(const float4_t & x, const float4_t & y) {
    return fmaxf(fmaxf(fmaxf(x[0], x[1]), fmaxf(x[2], x[3])), fmaxf(fmaxf(y[0], y[1]), fmaxf(y[2], y[3])));
}

// classifies mask tiles: one wave per (key tile, row block, mask batch).  A lane reads 8 keys
// (16 bytes) of a row, so the wave covers 8 rows of the 64-key tile per step.
__global__ __launch_bounds__(64) void pf_mask_flags_kernel(const char * mask, uint64_t nbm1, uint64_t nbm2, uint64_t nbm3,
                                                           int nem2, int n_q, int n_kv, int RB, int n_rb, int n_tiles,
                                                           int vec_ok, uint8_t * flags) {
    const int tile = blockIdx.x, rb = blockIdx.y, mb = blockIdx.z;
    const char * mp = mask + (uint64_t) (mb % nem2) * nbm2 + (uint64_t) (mb / nem2) * nbm3;
    const int r0 = rb * RB, r1 = min(n_q, (rb + 1) * RB);
    bool any_visible = false, any_nonzero = false;
    if (vec_ok && (tile + 1) * PF_KT <= n_kv) {
        const int sub = threadIdx.x >> 3, part = threadIdx.x & 7; // row within the step, 8-key group
        for (int r = r0 + sub; r < r1; r += 8) {
            const int4_t v = *(const int4_t *) (mp + (uint64_t) r * nbm1 + ((uint64_t) tile * PF_KT + part * 8) * 2);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = (uint32_t) v[i];
                any_visible |= (w & 0xFFFFu) != 0xFC00u || (w >> 16) != 0xFC00u;
                any_nonzero |= (w & 0x7FFF7FFFu) != 0;
            }
        }
    } else {
        const int key = tile * PF_KT + threadIdx.x;
        if (key < n_kv) {
            for (int r = r0; r < r1; ++r) {
                const uint16_t bits = ((const uint16_t *) (mp + (uint64_t) r * nbm1))[key];
                any_visible |= bits != 0xFC00u;
                any_nonzero |= (bits & 0x7FFFu) != 0;
            }
        }
    }
    const bool vis = __builtin_amdgcn_ballot_w64(any_visible) != 0;
    const bool nz  = __builtin_amdgcn_ballot_w64(any_nonzero) != 0;
    if (threadIdx.x == 0) flags[((uint64_t) mb * n_rb + rb) * n_tiles + tile] = !vis ? 0 : (nz ? 2 : 1);
}

// CT: 16-column tiles per wave.  PF_CT for large problems; half of it (work-groups of half as many columns, twice as many
// of them) when the grid would leave most of the chip idle.
template <bool KV_F32, int CT = PF_CT>
__global__ __launch_bounds__(64 * PF_WAVES) __attribute__((amdgpu_waves_per_eu(2))) void pf_kernel(const pf_args a) {
    constexpr int D = 64, NP = 2, SEG = 16;
    __shared__ __attribute__((aligned(16))) _Float16 k_lds[2][PF_KT][PF_ROW];
    __shared__ __attribute__((aligned(16))) _Float16 vt_lds[2][D][PF_ROW];
    // F32 values keep their low halves (v - f16(v), itself rounded to f16) in a second image, so that P V carries V to
    // about 22 bits: without it an output dominated by one key is off by half an f16 ulp of that value
    __shared__ __attribute__((aligned(16))) _Float16 vtl_lds[KV_F32 ? 2 : 1][KV_F32 ? D : 1][KV_F32 ? PF_ROW : 8];
    __shared__ uint16_t tile_list[PF_MAX_TILES];
    __shared__ uint8_t  tile_flag[PF_MAX_TILES];
    __shared__ int      n_active_s;

    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int j = lane >> 4, c = lane & 15;

    // ---- which (batch, kv head, row block): heavy (late) row blocks first; blocks of one
    //      (batch, kv head) stay on one XCD (work-groups are dealt round-robin to 8 XCDs)
    int grp, rb;
    {
        const int i = blockIdx.x;
        if (a.xcd_map) {
            const int xcd = i & 7, slot = i >> 3;
            grp = (slot / a.n_rb) * 8 + xcd;
            rb  = a.n_rb - 1 - slot % a.n_rb;
        } else {
            grp = i % a.n_groups;
            rb  = a.n_rb - 1 - i / a.n_groups;
        }
    }
    const int g = grp % a.Hkv, b = grp / a.Hkv;
    const int row0 = rb * a.RB;

    // ---- active key tiles of this row block
    {
        const int head0 = g * a.gqa; // the mask may differ per head only through nem2; rows of a block share flags per head
        (void) head0;
        if (wave == 0) {
            int base = 0;
            for (int t0 = 0; t0 < a.n_tiles; t0 += 64) {
                const int t = t0 + lane;
                uint8_t f = 0;
                if (t < a.n_tiles) {
                    if (a.flags) {
                        // a tile is active if any head of the group sees it; mixed if any head needs the mask
                        for (int hl = 0; hl < a.gqa; ++hl) {
                            const int mb = ((b % a.nem3) * a.nem2) + ((g * a.gqa + hl) % a.nem2);
                            const uint8_t ff = a.flags[((uint64_t) mb * a.n_rb + rb) * a.n_tiles + t];
                            f = ff > f ? ff : f;
                            if (a.nem2 == 1) break;
                        }
                        if (a.nem2 > 1 && f == 1) f = 2; // heads may disagree: let the element-wise path decide
                    } else {
                        f = 1;
                    }
                    if (f && (t + 1) * PF_KT > a.n_kv) f = 2; // partial tile: bounds are applied element-wise
                }
                const uint64_t bal = __builtin_amdgcn_ballot_w64(f != 0);
                const int pos = base + __builtin_popcountll(bal & ((1ull << lane) - 1));
                if (f) { tile_list[pos] = (uint16_t) t; tile_flag[pos] = f; }
                base += __builtin_popcountll(bal);
            }
            if (lane == 0) n_active_s = base;
        }
        __syncthreads();
    }
    const int n_active = n_active_s;

    // ---- this wave's columns
    const int ncols_blk = min(a.n_q - row0, a.RB) * a.gqa; // valid columns of the block
    half8_t qhi[CT][NP];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int  col = wave * (16 * CT) + ct * 16 + c;
        const bool ok  = col < ncols_blk;
        const int  row = row0 + (ok ? col / a.gqa : 0);
        const int  hd  = g * a.gqa + (ok ? col % a.gqa : 0);
        const float * qp = (const float *) (a.q + (uint64_t) row * a.nbq1 + (uint64_t) hd * a.nbq2 + (uint64_t) b * a.nbq3) + SEG * j;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            float4_t x0 = ((const float4_t *) (qp + 8 * p))[0], x1 = ((const float4_t *) (qp + 8 * p))[1];
            if (!ok) { x0 = float4_t{0, 0, 0, 0}; x1 = float4_t{0, 0, 0, 0}; }
            x0 *= a.scale2;
            x1 *= a.scale2;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qhi[ct][p][i]     = (_Float16) x0[i];
                qhi[ct][p][4 + i] = (_Float16) x1[i];
            }
        }
    }

    // row sums of the *rounded* probabilities come from the matrix core too: an A operand whose
    // row 0 is all ones makes row 0 of the product sum_k P~[k][col], so the normaliser matches
    // the f16 numerators exactly and costs no vector instructions
    half8_t ones;
#pragma unroll
    for (int i = 0; i < 8; ++i) ones[i] = c == 0 ? (_Float16) 1.0f : (_Float16) 0.0f;

    // Softmax bookkeeping.  Probabilities are taken relative to a per-column *reference*
    // m_ref that trails the running maximum: the S^T accumulator starts at -m_ref, so the MFMA
    // hands back s - m_ref and the common case is exp2 + convert, nothing else.  Only when some
    // score of the wave runs more than PF_LAZY above its reference (or the tile carries mask
    // values, or a column has not seen a key yet) does the slow block run: it moves m_ref up
    // and rescales O.  Values up to 2^PF_LAZY sit comfortably in f16 and fp32.
    float4_t o[CT][4], ol[CT], negm[CT];
    bool     seen[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        negm[ct] = float4_t{0, 0, 0, 0};
        seen[ct] = false;
        ol[ct] = float4_t{0, 0, 0, 0};
#pragma unroll
        for (int t = 0; t < 4; ++t) o[ct][t] = float4_t{0, 0, 0, 0};
    }
    bool all_seen = false; // wave-uniform

    if (n_active > 0) {
        // ---- global -> register staging: thread = (key = tid/8 (+32), 16-byte chunk = tid%8)
        const int ld_key = tid >> 3, ld_chunk = tid & 7;
        const char * kg = a.k + (uint64_t) g * a.nbk2 + (uint64_t) (b / a.rk3) * a.nbk3;
        const char * vg = a.v + (uint64_t) g * a.nbv2 + (uint64_t) (b / a.rk3) * a.nbv3;
        half8_t kreg[2], vreg[2], vlreg[2];
        // a thread's byte offsets inside a full tile never change: the tile's base is scalar arithmetic
        // and the loads take (scalar base, 32-bit lane offset); only a ragged last tile clamps per lane
        // (K and V share the offsets when their row strides agree, which every cache layout does)
        const uint32_t koff = (uint32_t) (ld_key * a.nbk1 + ld_chunk * 16);
        const bool off32_ok = !KV_F32 && a.nbk1 == a.nbv1 && (uint64_t) PF_KT * a.nbk1 < (1ull << 31);
        const uint32_t half_off = (uint32_t) (32 * a.nbk1); // scalar
        auto load_global = [&](int tile) {
            if (off32_ok && (tile + 1) * PF_KT <= a.n_kv) { // wave-uniform
                const char * kt = kg + (uint64_t) tile * PF_KT * a.nbk1;
                const char * vt = vg + (uint64_t) tile * PF_KT * a.nbv1;
#pragma unroll
                for (int hh = 0; hh < 2; ++hh) {
                    kreg[hh] = *(const half8_t *) (kt + hh * half_off + koff);
                    vreg[hh] = *(const half8_t *) (vt + hh * half_off + koff);
                }
                return;
            }
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int key = min(tile * PF_KT + hh * 32 + ld_key, a.n_kv - 1);
                if constexpr (KV_F32) {
                    const float4_t * kp = (const float4_t *) (kg + (uint64_t) key * a.nbk1 + ld_chunk * 32);
                    const float4_t * vp = (const float4_t *) (vg + (uint64_t) key * a.nbv1 + ld_chunk * 32);
                    const float4_t k0 = kp[0], k1 = kp[1], v0 = vp[0], v1 = vp[1];
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        kreg[hh][i] = (_Float16) k0[i]; kreg[hh][4 + i] = (_Float16) k1[i];
                        vreg[hh][i] = (_Float16) v0[i]; vreg[hh][4 + i] = (_Float16) v1[i];
                        vlreg[hh][i]     = (_Float16) (v0[i] - (float) vreg[hh][i]);
                        vlreg[hh][4 + i] = (_Float16) (v1[i] - (float) vreg[hh][4 + i]);
                    }
                } else {
                    kreg[hh] = *(const half8_t *) (kg + (uint64_t) key * a.nbk1 + ld_chunk * 16);
                    vreg[hh] = *(const half8_t *) (vg + (uint64_t) key * a.nbv1 + ld_chunk * 16);
                }
            }
        };
        auto store_lds = [&](int buf) {
#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                const int kl = hh * 32 + ld_key; // key within the tile
                *(half8_t *) &k_lds[buf][kl][ld_chunk * 8] = kreg[hh];
                // V^T, keys stored in P^T operand order: key 32hh + 16h + 4jj + r -> 32hh + 8jj + 4h + r
                const int k32 = ld_key, h = k32 >> 4, jj = (k32 >> 2) & 3, r = k32 & 3;
                const int grp8 = hh * 4 + jj, sub = 4 * h + r;
                // d = 8 * ld_chunk + i sits in physical row 8 * i + ld_chunk, key group xor-ed with i: the 8
                // chunks a wave writes at once land in 8 consecutive rows (distinct banks), and the 16 rows
                // an operand read touches spread over all banks as well
#pragma unroll
                for (int i = 0; i < 8; ++i) vt_lds[buf][8 * i + ld_chunk][((grp8 ^ i) << 3) + sub] = vreg[hh][i];
                if constexpr (KV_F32) {
#pragma unroll
                    for (int i = 0; i < 8; ++i) vtl_lds[buf][8 * i + ld_chunk][((grp8 ^ i) << 3) + sub] = vlreg[hh][i];
                }
            }
        };

        load_global(tile_list[0]);
        store_lds(0);
        __syncthreads();

        for (int it = 0; it < n_active; ++it) {
            const int buf = it & 1;
            const int tile = __builtin_amdgcn_readfirstlane(tile_list[it]);
            const bool mixed = tile_flag[it] == 2;
            load_global(__builtin_amdgcn_readfirstlane(tile_list[min(it + 1, n_active - 1)])); // unconditional: keeps the wait counts exact

#pragma unroll
            for (int hh = 0; hh < 2; ++hh) {
                // K operands of this 32-key half: lane (j,c) = key 16h + c, d = 16j + 8p ..
                half8_t ak[2][NP];
#pragma unroll
                for (int h = 0; h < 2; ++h)
#pragma unroll
                    for (int p = 0; p < NP; ++p) ak[h][p] = *(const half8_t *) &k_lds[buf][hh * 32 + h * 16 + c][SEG * j + 8 * p];
                half8_t av[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) av[t] = *(const half8_t *) &vt_lds[buf][(c & 7) * 8 + 2 * t + (c >> 3)][((hh * 4 + j) ^ (c & 7)) << 3];
                half8_t avl[4];
                if constexpr (KV_F32) {
#pragma unroll
                    for (int t = 0; t < 4; ++t) avl[t] = *(const half8_t *) &vtl_lds[buf][(c & 7) * 8 + 2 * t + (c >> 3)][((hh * 4 + j) ^ (c & 7)) << 3];
                }

#pragma unroll
                for (int cg = 0; cg < CT; cg += PF_GRP) {
                    // scores of PF_GRP column tiles, then ONE wave-uniform decision for the group, so
                    // the common path is straight-line code the scheduler can interleave
                    float4_t s[PF_GRP][2];
#pragma unroll
                    for (int u = 0; u < PF_GRP; ++u) {
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            float4_t acc = negm[cg + u];
#pragma unroll
                            for (int p = 0; p < NP; ++p) acc = mfma16(ak[h][p], qhi[cg + u][p], acc);
                            s[u][h] = acc; // = score * log2(e) - m_ref
                        }
                    }
                    int gmax = 0;
#pragma unroll
                    for (int u = 0; u < PF_GRP; ++u) gmax = max(gmax, imax8(s[u][0], s[u][1]));
                    if (mixed || !all_seen || __builtin_amdgcn_ballot_w64(gmax > __builtin_bit_cast(int, PF_LAZY)) != 0) {
#pragma unroll
                        for (int u = 0; u < PF_GRP; ++u) {
                            const int ct = cg + u;
                            if (mixed) { // element-wise mask / bounds (diagonal and tail tiles only)
                                const int col  = wave * (16 * CT) + ct * 16 + c;
                                const bool ok  = col < ncols_blk;
                                const int row  = row0 + (ok ? col / a.gqa : 0);
                                const int hd   = g * a.gqa + (ok ? col % a.gqa : 0);
                                const float slope = vx_alibi_slope(a.max_bias, (uint32_t) hd, a.n_head_log2, a.m0, a.m1) * 1.44269504088896341f;
                                const __half * mrow = a.mask ? (const __half *) (a.mask + (uint64_t) row * a.nbm1 + (uint64_t) (hd % a.nem2) * a.nbm2 + (uint64_t) (b % a.nem3) * a.nbm3) : nullptr;
#pragma unroll
                                for (int h = 0; h < 2; ++h)
#pragma unroll
                                    for (int r = 0; r < 4; ++r) {
                                        const int key = tile * PF_KT + hh * 32 + 16 * h + 4 * j + r;
                                        float x = 0.0f;
                                        if (mrow) x = slope * __half2float(mrow[min(key, a.n_kv - 1)]);
                                        s[u][h][r] += key < a.n_kv ? x : -INFINITY;
                                    }
                            }
                            float cm = fmax8(s[u][0], s[u][1]);
                            cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
                            cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
                            // move the reference: up to the new maximum, or (first visible key of the
                            // column) onto it wherever it lies
                            const bool  vis   = cm != -INFINITY;
                            const float delta = !vis ? 0.0f : (seen[ct] ? fmaxf(cm, 0.0f) : cm);
                            seen[ct] = seen[ct] || vis;
                            const float f = __builtin_amdgcn_exp2f(-delta);
#pragma unroll
                            for (int h = 0; h < 2; ++h) s[u][h] -= delta;
                            negm[ct] -= delta;
#pragma unroll
                            for (int t = 0; t < 4; ++t) o[ct][t] *= f;
                            ol[ct] *= f;
                        }
                    }
#pragma unroll
                    for (int u = 0; u < PF_GRP; ++u) {
                        const int ct = cg + u;
                        half8_t pb;
#pragma unroll
                        for (int h = 0; h < 2; ++h)
#pragma unroll
                            for (int r = 0; r < 4; r += 2)
                                pk2(pb, 4 * h + r, __builtin_amdgcn_exp2f(s[u][h][r]), __builtin_amdgcn_exp2f(s[u][h][r + 1]));
#pragma unroll
                        for (int t = 0; t < 4; ++t) o[ct][t] = mfma16(av[t], pb, o[ct][t]);
                        if constexpr (KV_F32) {
#pragma unroll
                            for (int t = 0; t < 4; ++t) o[ct][t] = mfma16(avl[t], pb, o[ct][t]);
                        }
                        ol[ct] = mfma16(ones, pb, ol[ct]);
                    }
                }
            }

            if (!all_seen) {
                bool every = true;
#pragma unroll
                for (int ct = 0; ct < CT; ++ct) every = every && seen[ct];
                all_seen = __builtin_amdgcn_ballot_w64(!every) == 0;
            }
            store_lds(buf ^ 1);
            __syncthreads();
        }
    }

    // ---- finish: lane (j,c), d-tile t, register r holds d = 16t + 4j + r of column c
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
        const int  col = wave * (16 * CT) + ct * 16 + c;
        const bool ok  = col < ncols_blk;
        const int  row = row0 + (ok ? col / a.gqa : 0);
        const int  hd  = g * a.gqa + (ok ? col % a.gqa : 0);
        float L = __shfl(ol[ct][0], c, 64); // row 0 of the ones product lives in lane (0, c), register 0
        float M = -negm[ct][0]; // the reference the sums are relative to
        float ms = 1.0f;
        if (a.sinks) { // ggml/src/ggml-cpu/ops.cpp:8598-8615, in the log2 domain
            const float sk = a.sinks[hd] * 1.44269504088896341f;
            float vs = 1.0f;
            if (sk > M) { ms = __builtin_amdgcn_exp2f(M - sk); } else { vs = __builtin_amdgcn_exp2f(sk - M); }
            L = L * ms + vs;
        }
        const float inv = L == 0.0f ? 0.0f : ms / L;
        if (ok) {
            float * out = a.dst + (((uint64_t) b * a.n_q + row) * a.Hq + hd) * D;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                float4_t r = o[ct][t] * inv;
                if (a.add1) r += *a.add1;
                *(float4_t *) (out + 16 * t + 4 * j) = r;
            }
        }
    }
}

} // namespace

// Called by vx_flash_attn_ext when the shape suits this kernel; returns VX_ERR_UNSUPPORTED
// (without touching the error string) when the caller should use the general kernel.
bool vx_fattn_prefill_accepts(const vx_tensor * q, const vx_tensor * k, float logit_softcap) {
    if (q->ne[0] != 64 || logit_softcap != 0.0f) return false;
    // F32 K/V (the reference's own cache type, and what a prefill sees: the keys straight from the projections) are
    // staged as f16 here -- K rounded like Q is, V as a high and a low half, so the result carries the same error as with
    // an f16 cache (the rounding of P, about 1.3e-3 on unit-scale data against the 2e-3 bar).  The general kernel keeps
    // hi + lo parts of everything (1e-6) and is 10 - 20 times slower on such shapes; VX_FA_F32_PREFILL=0 sends F32 K/V
    // there (read on every call).
    if (k->type == VX_TYPE_F32) {
        const char * e = getenv("VX_FA_F32_PREFILL");
        if (e && atoi(e) == 0) return false;
    } else if (k->type != VX_TYPE_F16) {
        return false;
    }
    const int Hq = (int) q->ne[2], Hkv = (int) k->ne[2], gqa = Hq / Hkv;
    if (gqa > PF_COLS / 2 || ((PF_COLS / 2) % gqa) != 0) return false;
    const int n_q = (int) q->ne[1], n_kv = (int) k->ne[1];
    const int RB = PF_COLS / gqa, n_rb = (n_q + RB - 1) / RB, n_tiles = (n_kv + PF_KT - 1) / PF_KT;
    const int n_groups = (int) q->ne[3] * Hkv;
    if (n_q * gqa < PF_COLS || n_tiles > PF_MAX_TILES) return false;
    // too few work-groups: the wave kernel spreads wider (one stream of 512 tokens, 32 blocks of 256 columns run as 64 of
    // 128: 19 us here against 28 us there; 256 tokens, 16 blocks: 15 us against 14 us)
    return (int64_t) n_rb * n_groups >= 32;
}

vx_status vx_fattn_prefill(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                           const float * sinks, const float * addend, const vx_tensor * dst, float scale, float max_bias,
                           float logit_softcap, hipStream_t st) {
    if (!vx_fattn_prefill_accepts(q, k, logit_softcap)) return VX_ERR_UNSUPPORTED;
    const int Hq = (int) q->ne[2], Hkv = (int) k->ne[2], gqa = Hq / Hkv;
    const int n_q = (int) q->ne[1], n_kv = (int) k->ne[1];
    const int n_groups = (int) q->ne[3] * Hkv;
    // work-groups of 256 columns; of 128 while 256 would put fewer than two work-groups on every CU
    const bool half_cols = (int64_t) ((n_q + PF_COLS / gqa - 1) / (PF_COLS / gqa)) * n_groups < 512;
    const int cols = half_cols ? PF_COLS / 2 : PF_COLS;
    const int RB = cols / gqa, n_rb = (n_q + RB - 1) / RB, n_tiles = (n_kv + PF_KT - 1) / PF_KT;

    pf_args a;
    a.q = (const char *) q->data; a.k = (const char *) k->data; a.v = (const char *) v->data;
    a.mask = mask ? (const char *) mask->data : nullptr;
    a.sinks = sinks;
    a.add1 = addend;
    a.dst = (float *) dst->data;
    a.flags = nullptr;
    a.nbq1 = q->nb[1]; a.nbq2 = q->nb[2]; a.nbq3 = q->nb[3];
    a.nbk1 = k->nb[1]; a.nbk2 = k->nb[2]; a.nbk3 = k->nb[3];
    a.nbv1 = v->nb[1]; a.nbv2 = v->nb[2]; a.nbv3 = v->nb[3];
    a.nbm1 = mask ? mask->nb[1] : 0; a.nbm2 = mask ? mask->nb[2] : 0; a.nbm3 = mask ? mask->nb[3] : 0;
    a.n_q = n_q; a.n_kv = n_kv; a.Hq = Hq; a.Hkv = Hkv; a.gqa = gqa;
    a.ne3 = (int) q->ne[3]; a.rk3 = (int) (q->ne[3] / k->ne[3]);
    a.nem2 = mask ? (int) mask->ne[2] : 1; a.nem3 = mask ? (int) mask->ne[3] : 1;
    a.RB = RB; a.n_rb = n_rb; a.n_tiles = n_tiles; a.n_groups = n_groups;
    a.xcd_map = (n_groups % 8 == 0);
    a.scale2 = scale * 1.44269504088896341f;
    a.max_bias = max_bias;
    a.n_head_log2 = 1u << (uint32_t) floor(log2((double) Hq));
    a.m0 = powf(2.0f, -(max_bias) / a.n_head_log2);
    a.m1 = powf(2.0f, -(max_bias / 2.0f) / a.n_head_log2);
    a.kv_f32 = k->type == VX_TYPE_F32;

    if (mask) {
        const int nmb = a.nem2 * a.nem3;
        void * ws = nullptr;
        vx_status rc = vx_workspace(st, (size_t) nmb * n_rb * n_tiles, &ws);
        if (rc != VX_OK) return rc;
        pf_mask_flags_kernel<<<dim3((unsigned) n_tiles, (unsigned) n_rb, (unsigned) nmb), dim3(64), 0, st>>>(
            a.mask, a.nbm1, a.nbm2, a.nbm3, a.nem2, n_q, n_kv, RB, n_rb, n_tiles,
            (int) ((uintptr_t) a.mask % 16 == 0 && a.nbm1 % 16 == 0 && a.nbm2 % 16 == 0 && a.nbm3 % 16 == 0), (uint8_t *) ws);
        VX_LAUNCH_CHECK();
        a.flags = (const uint8_t *) ws;
    }
    const dim3 grid((unsigned) (n_rb * n_groups)), block(64 * PF_WAVES);
    if (half_cols) {
        if (a.kv_f32) pf_kernel<true, PF_CT / 2><<<grid, block, 0, st>>>(a);
        else          pf_kernel<false, PF_CT / 2><<<grid, block, 0, st>>>(a);
    } else {
        if (a.kv_f32) pf_kernel<true><<<grid, block, 0, st>>>(a);
        else          pf_kernel<false><<<grid, block, 0, st>>>(a);
    }
    VX_LAUNCH_CHECK();
    return VX_OK;
}
