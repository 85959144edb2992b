// fattn_prefill.hip -- GGML_OP_FLASH_ATTN_EXT for many query rows (prefill) on gfx950: a
// tiled flash-attention kernel on f16 MFMA with K/V tiles staged in LDS and the online
// softmax in fp32.
//
// A work-group (4 waves) owns 256 (or 128) *columns* of one (batch, KV head): RB = 256 / gqa
// consecutive query rows times the gqa query heads that share the KV head, so one K/V tile
// in LDS serves all of them (the GQA reuse).  Keys are walked in tiles of 64.
//
// The mask is data, not a flag: a small pre-pass classifies every (row block, key tile) of it
// as all -inf (tile skipped: the causal upper triangle costs nothing), all zero (no mask
// arithmetic) or mixed (mask values are applied element-wise), so the result equals
// ggml-cpu's for any mask while a causal mask gets causal cost.
//
// Roofline: MFMA-bound in principle (4 * D flops per score); at D = 64 the exp, the rounding
// and the row sums of a score (VALU) need about as many issue cycles as its share of the
// matrix instructions, so the two pipes have to run side by side to come near the peak.
#include "vx_common.hpp"

#include <cmath>

namespace {

constexpr int PF_WAVES = 4;
constexpr int PF_COLS  = 256; // columns per work-group
constexpr int PF_KT    = 64;  // keys per tile
constexpr int PF_MAX_TILES = 1024;

struct pf_args {
    const char * q; const char * k; const char * v; const char * vl; const char * mask;
    const float * sinks;
    const float * add1; // optional scalar added to every output element (a fused GGML_OP_ADD1)
    _Float16 * tile_out; // optional: the result as f16 activation tiles of the product that follows, instead of dst
    uint32_t tile_tt, tile_bs, tile_ts;
    float * dst;
    const uint8_t * flags; // [nem3][nem2][n_rb][n_tiles]: 0 skip, 1 no mask, 2 apply mask values, 3 apply visibility bits
    const uint8_t * bits;  // [nem3][nem2][n_q][n_tiles] 8 bytes each: one bit per key of the tile (flag 3)
    uint64_t nbq1, nbq2, nbq3, nbk1, nbk2, nbk3, nbv1, nbv2, nbv3, nbm1, nbm2, nbm3;
    int n_q, n_kv, Hq, Hkv, gqa, ne3, rk3, nem2, nem3;
    int RB, n_rb, n_tiles, n_groups, xcd_map;
    int gqa_sh; // gqa divides 128: a power of two, gqa == 1 << gqa_sh
    float scale2, max_bias, m0, m1; // scale2 = scale * log2(e)
    uint32_t n_head_log2;
    int kv_f32;
};

// classifies mask tiles: one wave per (key tile, row block, mask batch).  A lane reads 8 keys
// (16 bytes) of a row, so the wave covers 8 rows of the 64-key tile per step.  Flags: 0 no key of the tile is visible to
// any row of the block; 1 every entry is zero; 2 some entry is a finite non-zero value; 3 zeros and -inf only.  For the
// last kind the rows' visibility is also left as one bit per key (bits[mask batch][row][tile], keys past n_kv cleared),
// so that the attention kernel applies such a tile -- a causal mask's diagonal -- from 8 bytes per row.
__global__ __launch_bounds__(64) void pf_mask_flags_kernel(const char * mask, uint64_t nbm1, uint64_t nbm2, uint64_t nbm3,
                                                           int nem2, int n_q, int n_kv, int RB, int n_rb, int n_tiles,
                                                           int vec_ok, uint8_t * flags, uint8_t * bits) {
    const int tile = blockIdx.x, rb = blockIdx.y, mb = blockIdx.z;
    const char * mp = mask + (uint64_t) (mb % nem2) * nbm2 + (uint64_t) (mb / nem2) * nbm3;
    const int r0 = rb * RB, r1 = min(n_q, (rb + 1) * RB);
    bool any_visible = false, any_nonzero = false, any_hidden = false;
    if (vec_ok && (tile + 1) * PF_KT <= n_kv) {
        const int sub = threadIdx.x >> 3, part = threadIdx.x & 7; // row within the step, 8-key group
        for (int r = r0 + sub; r < r1; r += 8) {
            const int4_t v = *(const int4_t *) (mp + (uint64_t) r * nbm1 + ((uint64_t) tile * PF_KT + part * 8) * 2);
            uint32_t byte = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = (uint32_t) v[i];
                const bool v0 = (w & 0xFFFFu) != 0xFC00u, v1 = (w >> 16) != 0xFC00u;
                byte |= (v0 ? 1u : 0u) << (2 * i) | (v1 ? 1u : 0u) << (2 * i + 1);
                any_nonzero |= (v0 && (w & 0x7FFFu) != 0) || (v1 && (w & 0x7FFF0000u) != 0);
            }
            any_visible |= byte != 0;
            any_hidden  |= byte != 0xFFu;
            bits[(((uint64_t) mb * n_q + r) * n_tiles + tile) * 8 + part] = (uint8_t) byte;
        }
    } else {
        const int key = tile * PF_KT + threadIdx.x;
        for (int r = r0; r < r1; ++r) {
            bool vis = false;
            if (key < n_kv) {
                const uint16_t h = ((const uint16_t *) (mp + (uint64_t) r * nbm1))[key];
                vis = h != 0xFC00u;
                any_nonzero |= vis && (h & 0x7FFFu) != 0;
            }
            any_visible |= vis;
            any_hidden  |= !vis;
            const uint64_t row_bits = __builtin_amdgcn_ballot_w64(vis);
            if (threadIdx.x == 0) *(uint64_t *) (bits + (((uint64_t) mb * n_q + r) * n_tiles + tile) * 8) = row_bits;
        }
    }
    const bool vis = __builtin_amdgcn_ballot_w64(any_visible) != 0;
    const bool nz  = __builtin_amdgcn_ballot_w64(any_nonzero) != 0;
    const bool hid = __builtin_amdgcn_ballot_w64(any_hidden) != 0;
    if (threadIdx.x == 0) flags[((uint64_t) mb * n_rb + rb) * n_tiles + tile] = !vis ? 0 : (nz ? 2 : (hid ? 3 : 1));
}

// ---- the tiled kernel ---------------------------------------------------------------------------------------------
// A work-group (4 waves) owns 128 * NCB columns of one (batch, KV head); a wave owns NCB blocks of 32 columns and walks
// 64-key tiles as two blocks of 32 keys with v_mfma_f32_32x32x16_f16:
//     S^T = K Q^T     A = 32 keys x 16 d from LDS (one 16-byte read), B = Q^T resident in registers, C = -reference, so the
//                     matrix core hands back score - reference and the common path is exp2, convert, nothing else
//     O^T += V^T P^T  A = 32 d x 16 keys, read from the row-major V tile with the transposing LDS read
//                     (ds_read_b64_tr_b16: a lane of a 16-lane group receives one d of four consecutive keys), B = P^T
//                     straight from the S^T accumulator registers: lane-half h of the S^T result holds keys 4h .. 4h+3 of
//                     every group of 8, which is the order the V^T reads are issued in
// K and V tiles never pass through registers: every wave copies its share of a tile into LDS with direct loads
// (global_load_lds_dwordx4, 64 lanes x 16 bytes = 8 rows per instruction), four tiles deep (three with a low image of
// V), one barrier per tile.  The 16-byte chunks of a row are stored xor-swizzled (the permutation is applied on the
// global address, the LDS side of a direct load is always lane-linear): K by the row's low three bits, 8-row blocks 128
// bytes apart, so the 32 rows of an A operand fall into different banks; V by twice the row's low two bits, so the
// 4 rows x 32 bytes a 16-lane group transposes do (the bank-conflict counter reads zero).  F32 K/V are converted by a
// pass of their own beforehand (K rounded to f16 as Q is; V as a high and a low f16 image whose products are both
// added, so a value is carried to about 22 bits).
// What bounds the walk is instruction issue, not the matrix core: a SIMD issues from its two waves about three
// quarters of the time, so every instruction that is not an exp2, a convert, a packed add or a matrix instruction
// is kept out of the steady state (no divisions, one LDS wait per step, no wait states behind transcendentals).
constexpr int PF_STAGES_MAX = 4;       // tiles in LDS: being read, landed, and two in flight (one with the low image of V)
constexpr int PF_KBLK    = 1152;            // bytes of an 8-row block of a K tile in LDS (8 x 128 + 128)
constexpr int PF_KSTAGE  = 8 * PF_KBLK;     // a 64-key K tile
constexpr int PF_VSTAGE  = 64 * 128;        // a 64-key V tile, rows back to back
constexpr float PF_SUM_LIMIT = 2048.0f;     // a lane's 16 probabilities of a block may add up to this before the reference moves

typedef __attribute__((address_space(3))) char lds_char;

__device__ __forceinline__ float16_t mfma32(half8_t a, half8_t b, float16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
}

// 16 bytes per lane from global memory (uniform base + per-lane 32-bit offset) straight into LDS: lane l's land at
// lds + 16 l (lds uniform).  M0 carries the LDS address.
__device__ __forceinline__ void pf_dma16(const char * base, uint32_t off, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds) : "memory");
}

__device__ __forceinline__ void pf_dma4(const char * base, uint32_t off, uint32_t lds) { // 4 bytes per lane, at lds + 4 l
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(off), "s"(base), "s"(lds) : "memory");
}

__device__ __forceinline__ half8_t pf_tr8(const lds_char * p) {
    typedef short short4_t __attribute__((ext_vector_type(4)));
    typedef short short8_t __attribute__((ext_vector_type(8)));
    const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3))) *) p);
    const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((short4_t __attribute__((address_space(3))) *) (p + 8 * 128));
    return __builtin_bit_cast(half8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

// F32 K and V of one (batch entry, KV head) as f16 planes [key][64]: K rounded, V as high and low halves
__global__ __launch_bounds__(256) void pf_convert_kernel(const char * k, const char * v, uint64_t nbk1, uint64_t nbk2, uint64_t nbk3,
                                                         uint64_t nbv1, uint64_t nbv2, uint64_t nbv3, int n_kv, int Hkv,
                                                         _Float16 * k16, _Float16 * vhi, _Float16 * vlo) {
    const int unit = blockIdx.x * 256 + threadIdx.x; // 8 values each
    const int key = unit >> 3, part = unit & 7, g = blockIdx.y, b = blockIdx.z;
    if (key >= n_kv) return;
    const float4_t * kp = (const float4_t *) (k + (uint64_t) key * nbk1 + (uint64_t) g * nbk2 + (uint64_t) b * nbk3) + 2 * part;
    const float4_t * vp = (const float4_t *) (v + (uint64_t) key * nbv1 + (uint64_t) g * nbv2 + (uint64_t) b * nbv3) + 2 * part;
    const float4_t k0 = kp[0], k1 = kp[1], v0 = vp[0], v1 = vp[1];
    half8_t kh, vh, vl;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        kh[i] = (_Float16) k0[i]; kh[4 + i] = (_Float16) k1[i];
        vh[i] = (_Float16) v0[i]; vh[4 + i] = (_Float16) v1[i];
        vl[i]     = (_Float16) (v0[i] - (float) vh[i]);
        vl[4 + i] = (_Float16) (v1[i] - (float) vh[4 + i]);
    }
    const uint64_t o = (((uint64_t) b * Hkv + g) * n_kv + key) * 64 + 8 * part;
    *(half8_t *) (k16 + o) = kh;
    *(half8_t *) (vhi + o) = vh;
    *(half8_t *) (vlo + o) = vl;
}

// VLO: V comes with a low-half image (a.vl).  NCB: 32-column blocks per wave.
template <bool VLO, int NCB>
__global__ __launch_bounds__(64 * PF_WAVES) __attribute__((amdgpu_waves_per_eu(2, 2))) void pf_kernel(const pf_args a) {
    constexpr int D = 64;
    constexpr int PF_STAGES = VLO ? 3 : PF_STAGES_MAX; // (three stages of K, V and V low leave room for two work-groups on a compute unit)
    constexpr int NL = VLO ? 6 : 4; // direct loads per wave and tile (a tile that needs its visibility bits has one more)
    __shared__ __attribute__((aligned(1024))) char k_lds[PF_STAGES][PF_KSTAGE];
    __shared__ __attribute__((aligned(1024))) char v_lds[PF_STAGES][PF_VSTAGE];
    __shared__ __attribute__((aligned(1024))) char vl_lds[VLO ? PF_STAGES : 1][VLO ? PF_VSTAGE : 16];
    __shared__ __attribute__((aligned(256))) uint32_t bits_lds[PF_STAGES][64]; // visibility bits of the block's rows: 8 bytes per row
    __shared__ uint16_t tile_list[PF_MAX_TILES];
    __shared__ uint8_t  tile_flag[PF_MAX_TILES];
    __shared__ int      n_active_s;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int hl = lane >> 5, cl = lane & 31;

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

    // ---- this wave's columns: lane (hl, cl) holds column cl of each block as the B operand's d = 16 kk + 8 hl .. + 7.
    //      The loads are issued before anything else (the tile list and the first tiles' copies are built while they fly).
    const int ncols_blk = min(a.n_q - row0, a.RB) * a.gqa; // valid columns of the block
    float4_t qraw[NCB][4][2];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int  col = wave * (32 * NCB) + cb * 32 + cl;
        const bool ok  = col < ncols_blk;
        const int  row = row0 + (ok ? (col >> a.gqa_sh) : 0);
        const int  hd  = g * a.gqa + (ok ? (col & (a.gqa - 1)) : 0);
        const float * qp = (const float *) (a.q + (uint64_t) row * a.nbq1 + (uint64_t) hd * a.nbq2 + (uint64_t) b * a.nbq3) + 8 * hl;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            qraw[cb][kk][0] = ((const float4_t *) (qp + 16 * kk))[0];
            qraw[cb][kk][1] = ((const float4_t *) (qp + 16 * kk))[1];
        }
    }

    // ---- active key tiles of this row block
    if (wave == 0) {
        int base = 0;
        for (int t0 = 0; t0 < a.n_tiles; t0 += 64) {
            const int t = t0 + lane;
            uint8_t f = 0;
            if (t < a.n_tiles) {
                if (a.flags) {
                    // a tile is active if any head of the group sees it; mixed if any head needs the mask
                    for (int hd = 0; hd < a.gqa; ++hd) {
                        const int mb = ((b % a.nem3) * a.nem2) + ((g * a.gqa + hd) % a.nem2);
                        const uint8_t ff = a.flags[((uint64_t) mb * a.n_rb + rb) * a.n_tiles + t];
                        f = ff > f ? ff : f;
                        if (a.nem2 == 1) break;
                    }
                    if (a.nem2 > 1 && f) f = 2; // heads may disagree: let the element-wise path decide
                } else {
                    f = 1;
                }
                if (f == 1 && (t + 1) * PF_KT > a.n_kv) f = 3; // partial tile: the bounds are visibility bits
            }
            const uint64_t bal = __builtin_amdgcn_ballot_w64(f != 0);
            const int pos = base + __builtin_popcountll(bal & ((1ull << lane) - 1));
            if (f) { tile_list[pos] = (uint16_t) t; tile_flag[pos] = f; }
            base += __builtin_popcountll(bal);
        }
        if (lane == 0) n_active_s = base;
    }
    __syncthreads();
    const int n_active = __builtin_amdgcn_readfirstlane(n_active_s);

    // Softmax bookkeeping.  Probabilities are taken relative to a per-column *reference* that trails the running maximum:
    // the S^T accumulator starts at -reference (the same value in a lane's 16 registers: a lane holds one column).  The
    // row sums are formed from the *rounded* probabilities, so numerator and denominator see the same values: the 16 of a
    // unit are added as packed halves (v_pk_add_f16: one instruction per pair; a dot2 or two fp32 additions per pair cost the
    // loop a fifth of its speed, measured), the two partial sums then join the fp32 total.  A unit's contribution doubles
    // as the test for "some score ran far above its reference": only then (or when the tile carries mask values, or a column has not seen a key yet) does the slow
    // block run, which moves the reference up, rescales O and forms the block's probabilities again.
    half8_t   qb[NCB][4];
    float16_t o[NCB][2], negm[NCB];
    float     l[NCB];
    bool      seen[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        l[cb] = 0.0f;
        seen[cb] = false;
#pragma unroll
        for (int r = 0; r < 16; ++r) { negm[cb][r] = 0.0f; o[cb][0][r] = 0.0f; o[cb][1][r] = 0.0f; }
    }
    bool all_seen = false; // wave-uniform

    if (n_active > 0) {
        const char * kg = a.k + (uint64_t) g * a.nbk2 + (uint64_t) (b / a.rk3) * a.nbk3;
        const char * vg = a.v + (uint64_t) g * a.nbv2 + (uint64_t) (b / a.rk3) * a.nbv3;
        const char * vlg = VLO ? a.vl + (uint64_t) g * a.nbv2 + (uint64_t) (b / a.rk3) * a.nbv3 : nullptr;
        const uint32_t k_base = (uint32_t) (uintptr_t) (lds_char *) &k_lds[0][0];
        const uint32_t v_base = (uint32_t) (uintptr_t) (lds_char *) &v_lds[0][0];
        const uint32_t vl_base = (uint32_t) (uintptr_t) (lds_char *) &vl_lds[0][0];
        const uint32_t bits_base = (uint32_t) (uintptr_t) (lds_char *) &bits_lds[0][0];
        // the rows' visibility bits of a tile (used when the tile's flag is 3): lane = (row lane / 2, dword lane % 2); every
        // wave fetches the block's 256 bytes (the same bytes to the same place), only for tiles that need them
        const char * bits_src = a.bits ? (const char *) a.bits + ((uint64_t) (b % a.nem3) * a.nem2 * a.n_q) * a.n_tiles * 8 : a.q;
        // (this lane's offset into them, worked out where it is used: see apply_mask)
        auto bits_row = [&]() {
            int ln = lane;
            asm volatile("" : "+v"(ln));
            return (uint32_t) min(row0 + (ln >> 1), a.n_q - 1) * (uint32_t) a.n_tiles * 8 + 4 * (ln & 1);
        };

        // ---- direct loads: this wave copies rows 16 wave .. 16 wave + 15 of a tile, 8 rows per instruction; lane = (row
        //      lane / 8, chunk position lane % 8), the chunk it fetches is the position un-swizzled
        const int dr = lane >> 3, dp = lane & 7;
        const uint32_t kch = (uint32_t) ((dp ^ dr) << 4), vch = (uint32_t) ((dp ^ (2 * (dr & 3))) << 4);
        uint32_t kof[2], vof[2]; // this lane's byte offsets inside a whole tile, per 8-row block
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            kof[u] = (uint32_t) (16 * wave + 8 * u + dr) * (uint32_t) a.nbk1 + kch;
            vof[u] = (uint32_t) (16 * wave + 8 * u + dr) * (uint32_t) a.nbv1 + vch;
        }
        // A tile's copy is NOPS instructions per wave (K and V, two 8-row blocks each; with VLO the low image too).  They are
        // not issued in one burst: the memory pipeline takes a hundred cycles and more to accept one when all eight waves of
        // a compute unit arrive together, and a wave waits in line.  issue_setup fixes the tile and its stage, issue_op(j)
        // sends instruction j; the steps of the walk send one or two each.
        constexpr int NOPS = VLO ? 6 : 4;
        const char * dma_kt = nullptr, * dma_vt = nullptr, * dma_vlt = nullptr;
        uint32_t dma_kl = 0, dma_vl = 0;
        int dma_last = 0, dma_stage = 0, dma_tile = 0;
        bool dma_bits = false;
        auto issue_setup = [&](int idx, int stage) {
            const int at = min(idx, n_active - 1);
            const int tile = __builtin_amdgcn_readfirstlane(tile_list[at]);
            dma_kt = kg + (uint64_t) tile * PF_KT * a.nbk1;
            dma_vt = vg + (uint64_t) tile * PF_KT * a.nbv1;
            dma_vlt = VLO ? vlg + (uint64_t) tile * PF_KT * a.nbv1 : nullptr;
            dma_kl = k_base + stage * PF_KSTAGE + 2 * wave * PF_KBLK;
            dma_vl = stage * PF_VSTAGE + 2 * wave * 1024;
            dma_last = a.n_kv - 1 - tile * PF_KT; // rows past it are clamped (their scores are masked by the bounds)
            dma_stage = stage;
            dma_tile = tile;
            dma_bits = a.bits && __builtin_amdgcn_readfirstlane(tile_flag[at]) == 3;
        };
        auto issue_op = [&](int j) {
            const int u = j & 1, what = j >> 1; // 0 K, 1 V, 2 V low
            uint32_t off = what == 0 ? kof[u] : vof[u];
            if (dma_last < PF_KT - 1) { // wave-uniform: a ragged last tile
                const int r = min(16 * wave + 8 * u + dr, dma_last);
                off = what == 0 ? (uint32_t) r * (uint32_t) a.nbk1 + kch : (uint32_t) r * (uint32_t) a.nbv1 + vch;
            }
            if (what == 0) pf_dma16(dma_kt, off, dma_kl + u * PF_KBLK);
            if (what == 1) pf_dma16(dma_vt, off, v_base + dma_vl + u * 1024);
            if (what == 2) pf_dma16(dma_vlt, off, vl_base + dma_vl + u * 1024);
            // the rows' visibility bits ride behind the first instruction of a tile that needs them (a further load only
            // makes the waits below more conservative: they count what may still be in flight)
            if (j == 0 && dma_bits) pf_dma4(bits_src + (uint64_t) ((uint32_t) dma_tile * 8u), bits_row(), bits_base + dma_stage * 256);
        };
        auto issue = [&](int idx, int stage) {
            issue_setup(idx, stage);
#pragma unroll
            for (int j = 0; j < NOPS; ++j) issue_op(j);
        };

        for (int t = 0; t < PF_STAGES - 1; ++t) issue(t, t);

        // ---- Q, pre-scaled by scale * log2(e) and rounded to f16
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            const bool ok = wave * (32 * NCB) + cb * 32 + cl < ncols_blk;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                float4_t x0 = qraw[cb][kk][0], x1 = qraw[cb][kk][1];
                if (!ok) { x0 = float4_t{0, 0, 0, 0}; x1 = float4_t{0, 0, 0, 0}; }
                x0 *= a.scale2;
                x1 *= a.scale2;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    qb[cb][kk][i]     = (_Float16) x0[i];
                    qb[cb][kk][4 + i] = (_Float16) x1[i];
                }
            }
        }

        // ---- operand addresses inside a stage
        uint32_t kad[4], vad[2];
        {
            const int r8 = cl & 7;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) kad[kk] = (uint32_t) ((cl >> 3) * PF_KBLK + r8 * 128 + (((2 * kk + hl) ^ r8) << 4));
            const int i = lane & 15, gg = (lane >> 4) & 1;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
                vad[dt] = (uint32_t) ((4 * hl + (i >> 2)) * 128 + (((4 * dt + 2 * gg + ((i & 3) >> 1)) ^ (2 * (i >> 2))) << 4) + 8 * (i & 1));
        }
        const lds_char * const k_lds0 = (const lds_char *) &k_lds[0][0];
        const lds_char * const v_lds0 = (const lds_char *) &v_lds[0][0];
        const lds_char * const vl_lds0 = (const lds_char *) &vl_lds[0][0];

        // The walk is a software pipeline over *units* (a 32-key block x one of the wave's 32-column blocks; 2 NCB per tile,
        // column blocks alternating).  A step handles unit u as 8 groups of { one matrix instruction; exp2, exp2, convert,
        // dot2 of two of u's scores }: the matrix instructions of a step are the 4 of S(u + 1) and the 4 of O += V^T P(u - 1),
        // neither of which depends on the vector work they run beside.  The K operands of a block are read right after the
        // last S instruction that needs the previous ones has issued, the V^T operands likewise behind the O instructions.
        constexpr int NU = 2 * NCB;            // units (steps) per tile
        constexpr int KBAR = NU - 2;           // the step that waits for the next tile (its tail reads that tile's K)
        float16_t sbuf[2];                     // scores of the current and of the next unit (alternating)
        int4_t    pbuf[2][2];                  // probabilities of the current and of the previous unit: [parity][16-key half]
        half8_t   ak[4], av[2][2], avl[2][2];
#pragma unroll
        for (int x = 0; x < 2; ++x)
#pragma unroll
            for (int y = 0; y < 2; ++y) {
                pbuf[x][y] = int4_t{0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < 8; ++i) { av[x][y][i] = (_Float16) 0.0f; avl[x][y][i] = (_Float16) 0.0f; }
            }

        auto load_ak = [&](int stage, int kb) {
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) ak[kk] = *(const __attribute__((address_space(3))) half8_t *) (k_lds0 + stage * PF_KSTAGE + kad[kk] + kb * 4 * PF_KBLK);
        };
        auto load_av = [&](int stage, int kb) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks)
#pragma unroll
                for (int dt = 0; dt < 2; ++dt) {
                    av[dt][ks] = pf_tr8(v_lds0 + stage * PF_VSTAGE + vad[dt] + (32 * kb + 16 * ks) * 128);
                    if constexpr (VLO) avl[dt][ks] = pf_tr8(vl_lds0 + stage * PF_VSTAGE + vad[dt] + (32 * kb + 16 * ks) * 128);
                }
        };
        // the slow block of unit (kb, cb) of `tile`: mask and bounds, the column maxima, the reference moved, O rescaled
        // the mask of unit (kb, cb) of `tile` applied to its scores (tiles flagged 2 or 3 only)
        auto apply_mask = [&](int tile, int stage, int flag, int kb, int cb, float16_t & s) {
            // (the column's row and head are worked out here, behind an opaque statement: hoisted out of the walk they would be
            // held in registers the walk does not have, i.e. spilled)
            int clo = cl;
            asm volatile("" : "+v"(clo));
            if (flag == 3) { // zeros and -inf only (a causal diagonal, a ragged last tile): one bit per key
                const int col = wave * (32 * NCB) + cb * 32 + clo;
                const int rl  = col < ncols_blk ? (col >> a.gqa_sh) : 0;
                uint32_t w;
                if (a.bits) {
                    w = bits_lds[stage][2 * rl + kb];
                } else { // no mask: the bounds
                    const int left = a.n_kv - tile * PF_KT - 32 * kb;
                    w = left >= 32 ? 0xFFFFFFFFu : (left <= 0 ? 0u : (1u << left) - 1u);
                }
                w >>= 4 * hl;
#pragma unroll
                for (int r = 0; r < 16; ++r) s[r] = ((w >> (8 * (r >> 2) + (r & 3))) & 1u) ? s[r] : -INFINITY;
            } else { // element-wise mask values / bounds
                const int col  = wave * (32 * NCB) + cb * 32 + clo;
                const bool ok  = col < ncols_blk;
                const int row  = row0 + (ok ? (col >> a.gqa_sh) : 0);
                const int hd   = g * a.gqa + (ok ? (col & (a.gqa - 1)) : 0);
                const float slope = vx_alibi_slope(a.max_bias, (uint32_t) hd, a.n_head_log2, a.m0, a.m1) * 1.44269504088896341f;
                const __half * mrow = a.mask ? (const __half *) (a.mask + (uint64_t) row * a.nbm1 + (uint64_t) (hd % a.nem2) * a.nbm2 + (uint64_t) (b % a.nem3) * a.nbm3) : nullptr;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int key = tile * PF_KT + 32 * kb + 8 * (r >> 2) + 4 * hl + (r & 3);
                    float x = 0.0f;
                    if (mrow) x = slope * __half2float(mrow[min(key, a.n_kv - 1)]);
                    s[r] += key < a.n_kv ? x : -INFINITY;
                }
            }
        };
        // the slow block: the column maxima of a unit's scores, the reference moved, O rescaled
        auto move_reference = [&](int cb, float16_t & s, float16_t & s_inflight, bool same_cb_inflight) {
            float cm = s[0];
#pragma unroll
            for (int r = 1; r < 16; ++r) cm = fmaxf(cm, s[r]);
            cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
            // move the reference: up to the new maximum, or (first visible key of the column) onto it wherever it lies
            const bool  vis   = cm != -INFINITY;
            const float delta = !vis ? 0.0f : (seen[cb] ? fmaxf(cm, 0.0f) : cm);
            seen[cb] = seen[cb] || vis;
            if (__builtin_amdgcn_ballot_w64(delta != 0.0f) == 0) return; // nothing moves (wave-uniform)
            const float f = __builtin_amdgcn_exp2f(-delta);
            s -= delta;
            if (same_cb_inflight) s_inflight -= delta; // scores already formed against the old reference
            negm[cb] -= delta;
            o[cb][0] *= f;
            o[cb][1] *= f;
            l[cb] *= f;
        };
        auto probs = [&](const float16_t & s, int4_t (&pb)[2], float & lt) {
            typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
            half2_t acc = half2_t{(_Float16) 0.0f, (_Float16) 0.0f};
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const fp16x2 pr = __builtin_amdgcn_cvt_pkrtz(__builtin_amdgcn_exp2f(s[2 * i]), __builtin_amdgcn_exp2f(s[2 * i + 1]));
                pb[i >> 2][i & 3] = __builtin_bit_cast(int, pr);
                acc += __builtin_bit_cast(half2_t, pr);
            }
            lt = (float) acc[0] + (float) acc[1];
        };
        // O += V^T P of one unit (outside the pipelined steps: the very last unit)
        auto pv_all = [&](int cb, const int4_t (&pb)[2]) {
#pragma unroll
            for (int ks = 0; ks < 2; ++ks) {
                const half8_t p = __builtin_bit_cast(half8_t, pb[ks]);
#pragma unroll
                for (int dt = 0; dt < 2; ++dt) {
                    o[cb][dt] = mfma32(av[dt][ks], p, o[cb][dt]);
                    if constexpr (VLO) o[cb][dt] = mfma32(avl[dt][ks], p, o[cb][dt]);
                }
            }
        };

        asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(NL * (PF_STAGES - 2)) : "memory"); // tile 0 has landed
        load_ak(0, 0);
        sbuf[0] = negm[0];
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) sbuf[0] = mfma32(ak[kk], qb[0][kk], sbuf[0]);
        if constexpr (NCB == 1) load_ak(0, 1); // the next unit is the tile's second block already

        for (int it = 0; it < n_active; ++it) {
            const int  stage  = it % PF_STAGES, stage1 = (it + 1) % PF_STAGES;
            const int  tile   = __builtin_amdgcn_readfirstlane(tile_list[it]);
            const int  flag   = __builtin_amdgcn_readfirstlane(tile_flag[it]); // 1 plain, 2 mask values, 3 visibility bits

#pragma unroll
            for (int k = 0; k < NU; ++k) {
                const int kb = k / NCB, cb = k % NCB;             // this step's unit
                const int cbn = (k + 1) % NCB;                    // the next unit's column block
                const int cbp = (k + NU - 1) % NCB;               // the previous unit's
                const int cur = k & 1, nxt = cur ^ 1;             // NU is even: parities line up across tiles
                if (k == KBAR) {
                    // the next tile has landed for everybody, and everybody is past the previous tile: its stage is refilled,
                    // the copy's instructions spread over this step and the NU - 1 that follow
                    asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(NL * (PF_STAGES - 3)) : "memory");
                    issue_setup(it + PF_STAGES - 1, (it + PF_STAGES - 1) % PF_STAGES);
                }
                {   // with four stages the copy has until the wait after next and spreads over a whole round of steps (those
                    // ahead of the first wait belong to a tile the prologue has sent); with three it must be under way before
                    // the next wait and takes the steps that are left of this round
                    constexpr int SPREAD = PF_STAGES >= 4 ? NU : NU - KBAR;
                    constexpr int PER = NOPS / SPREAD; // 4 or 6 instructions over 2 or 4 steps: 1, 2 or 3 a step
                    static_assert(PER * SPREAD == NOPS, "the copy's instructions must divide over its steps");
                    const int sl = (k - KBAR + NU) % NU; // which step of the copy this is
                    if (sl < SPREAD && (k >= KBAR || it > 0)) {
#pragma unroll
                        for (int j = PER * sl; j < PER * sl + PER; ++j) issue_op(j);
                    }
                }
                float lt = 0.0f;
                half2_t acc2 = half2_t{(_Float16) 0.0f, (_Float16) 0.0f};
                typedef __fp16 fp16x2 __attribute__((ext_vector_type(2)));
                // matrix instruction i of the step, and the operand reads that follow it
                auto mat = [&](int i) {
                    if (i < 4) {
                        sbuf[nxt] = mfma32(ak[i], qb[cbn][i], i == 0 ? negm[cbn] : sbuf[nxt]);
                    } else {
                        const int ks = (i - 4) >> 1, dt = (i - 4) & 1;
                        const half8_t p = __builtin_bit_cast(half8_t, pbuf[nxt][ks]); // the previous unit wrote the other parity
                        o[cbp][dt] = mfma32(av[dt][ks], p, o[cbp][dt]);
                        if constexpr (VLO) o[cbp][dt] = mfma32(avl[dt][ks], p, o[cbp][dt]);
                    }
                    if (i == 3) { // the K operands the S instructions after the next step's need
                        if (NCB == 2 && k == 0) load_ak(stage, 1);
                        if (NCB == 2 && k == 2) load_ak(stage1, 0);
                        if (NCB == 1 && k == 0) load_ak(stage1, 0);
                        if (NCB == 1 && k == 1) load_ak(stage1, 1);
                    }
                    // the V^T operands of this unit's block, for the O instructions of the next step (and the one after)
                    if (i == 7 && cb == 0) load_av(stage, kb);
                };
                // One path for every tile: on a masked tile, and while a column has not seen a key, the probabilities
                // formed here are thrown away (the slow block forms them again from the corrected scores), which keeps the
                // matrix instructions in one place; `lt` passes through an opaque statement so that the vector work stays
                // where it is written instead of being moved under the condition.
                // (everything a step's matrix instructions read from LDS was requested a step ago: one wait, stated here, in
                // place of one in front of every instruction; and a pair's conversion trails its exponentials by a group, so
                // that no wait state is needed between a transcendental and its reader)
                __builtin_amdgcn_s_waitcnt(0xC07F); // lgkmcnt(0)
                float ea = 0.0f, eb = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    mat(i);
                    const float na = __builtin_amdgcn_exp2f(sbuf[cur][2 * i]), nb = __builtin_amdgcn_exp2f(sbuf[cur][2 * i + 1]);
                    if (i > 0) {
                        const fp16x2 pr = __builtin_amdgcn_cvt_pkrtz(ea, eb);
                        pbuf[cur][(i - 1) >> 2][(i - 1) & 3] = __builtin_bit_cast(int, pr);
                        acc2 += __builtin_bit_cast(half2_t, pr);
                    }
                    ea = na;
                    eb = nb;
                    __builtin_amdgcn_sched_barrier(0);
                }
                {
                    const fp16x2 pr = __builtin_amdgcn_cvt_pkrtz(ea, eb);
                    pbuf[cur][1][3] = __builtin_bit_cast(int, pr);
                    acc2 += __builtin_bit_cast(half2_t, pr);
                }
                lt = (float) acc2[0] + (float) acc2[1];
                asm volatile("" : "+v"(lt));
                bool redo = !all_seen || __builtin_amdgcn_ballot_w64(!(lt <= PF_SUM_LIMIT)) != 0;
                if (flag != 1) { // a masked tile: what was formed above is void, the scores take the mask first
                    apply_mask(tile, stage, flag, kb, cb, sbuf[cur]);
                    redo = true;
                    if (all_seen) {
                        probs(sbuf[cur], pbuf[cur], lt);
                        redo = __builtin_amdgcn_ballot_w64(!(lt <= PF_SUM_LIMIT)) != 0;
                    }
                }
                if (redo) {
                    move_reference(cb, sbuf[cur], sbuf[nxt], NCB == 1);
                    probs(sbuf[cur], pbuf[cur], lt);
                    if (!all_seen) {
                        bool every = true;
#pragma unroll
                        for (int c2 = 0; c2 < NCB; ++c2) every = every && seen[c2];
                        all_seen = __builtin_amdgcn_ballot_w64(!every) == 0;
                    }
                }
                l[cb] += lt;
            }
        }
        pv_all(NCB - 1, pbuf[(NU - 1) & 1]); // the last unit's
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // the loads issued past the last tile
    }

    // ---- finish: lane (hl, cl), d block dt, register r holds d = 32 dt + 8 (r / 4) + 4 hl + r % 4 of column cl
    int lane_e = threadIdx.x & 63; // (worked out again rather than kept alive through the walk)
    asm volatile("" : "+v"(lane_e));
    const int hl_e = lane_e >> 5, cl_e = lane_e & 31;
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        const int  col = wave * (32 * NCB) + cb * 32 + cl_e;
        const bool ok  = col < ncols_blk;
        const int  row = row0 + (ok ? (col >> a.gqa_sh) : 0);
        const int  hd  = g * a.gqa + (ok ? (col & (a.gqa - 1)) : 0);
        float L = l[cb] + __shfl_xor(l[cb], 32, 64); // the two lanes of a column hold disjoint keys
        float M = -negm[cb][0]; // the reference the sums are relative to
        float ms = 1.0f;
        if (a.sinks) { // ggml/src/ggml-cpu/ops.cpp:8598-8615, in the log2 domain
            const float sk = a.sinks[hd] * 1.44269504088896341f;
            float vs = 1.0f;
            if (sk > M) { ms = __builtin_amdgcn_exp2f(M - sk); } else { vs = __builtin_amdgcn_exp2f(sk - M); }
            L = L * ms + vs;
        }
        const float inv = L == 0.0f ? 0.0f : ms / L;
        if (ok && a.tile_out) { // (uniform choice) rounded to f16 as the product's activation pass would round the stored value
            // k = hd * 64 + d: tile (k block 2 hd + dt, 16 tokens), slot (q4, token mod 16), halves 4 hl .. 4 hl + 3
            const uint32_t tokf = (uint32_t) b * a.tile_ts + (uint32_t) row;
            _Float16 * tb = a.tile_out + ((((uint64_t) b * a.tile_bs + (uint64_t) (2 * hd) * a.tile_tt + (tokf >> 4)) * 64 + (tokf & 15)) * 8 + 4 * hl_e);
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    float4_t r = float4_t{o[cb][dt][4 * q4], o[cb][dt][4 * q4 + 1], o[cb][dt][4 * q4 + 2], o[cb][dt][4 * q4 + 3]} * inv;
                    if (a.add1) r += *a.add1;
                    asm volatile("" : "+v"(r)); // the fp32 value the node holds, formed as such, then rounded
                    *(half4_t *) (tb + ((uint64_t) dt * a.tile_tt * 64 + 16 * q4) * 8) = half4_t{(_Float16) r[0], (_Float16) r[1], (_Float16) r[2], (_Float16) r[3]};
                }
        } else if (ok) {
            float * out = a.dst + (((uint64_t) b * a.n_q + row) * a.Hq + hd) * D;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
#pragma unroll
                for (int q4 = 0; q4 < 4; ++q4) {
                    float4_t r = float4_t{o[cb][dt][4 * q4], o[cb][dt][4 * q4 + 1], o[cb][dt][4 * q4 + 2], o[cb][dt][4 * q4 + 3]} * inv;
                    if (a.add1) r += *a.add1;
                    *(float4_t *) (out + 32 * dt + 8 * q4 + 4 * hl_e) = r;
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
    if (k->type == VX_TYPE_F16 && k->nb[1] >= (1u << 25)) return false; // a tile's rows are addressed by 32-bit offsets
    // too few work-groups: the wave kernel spreads wider (one stream of 512 tokens, 32 blocks of 256 columns run as 64 of
    // 128: 19 us here against 28 us there; 256 tokens, 16 blocks: 15 us against 14 us)
    return (int64_t) n_rb * n_groups >= 32;
}

vx_status vx_fattn_prefill(const vx_tensor * q, const vx_tensor * k, const vx_tensor * v, const vx_tensor * mask,
                           const float * sinks, const float * addend, const vx_tensor * dst, float scale, float max_bias,
                           float logit_softcap, hipStream_t st, const vx_pf_front * front) {
    if (!vx_fattn_prefill_accepts(q, k, logit_softcap)) return VX_ERR_UNSUPPORTED;
    const int Hq = (int) q->ne[2], Hkv = (int) k->ne[2], gqa = Hq / Hkv;
    const int n_q = (int) q->ne[1], n_kv = (int) k->ne[1];
    const int n_groups = (int) q->ne[3] * Hkv;
    // work-groups of 256 columns; of 128 while 256 would put fewer than two work-groups on every CU
    // (with the low image of V a wave of 64 columns does not fit two to a SIMD: F32 K/V always take the 128-column form)
    const bool half_cols = k->type == VX_TYPE_F32 || (int64_t) ((n_q + PF_COLS / gqa - 1) / (PF_COLS / gqa)) * n_groups < 512;
    const int cols = half_cols ? PF_COLS / 2 : PF_COLS;
    const int RB = cols / gqa, n_rb = (n_q + RB - 1) / RB, n_tiles = (n_kv + PF_KT - 1) / PF_KT;

    pf_args a;
    a.q = (const char *) q->data; a.k = (const char *) k->data; a.v = (const char *) v->data;
    a.mask = mask ? (const char *) mask->data : nullptr;
    a.sinks = sinks;
    a.add1 = addend;
    a.tile_out = nullptr; a.tile_tt = a.tile_bs = a.tile_ts = 0;
    a.dst = (float *) dst->data;
    a.flags = nullptr;
    a.bits = nullptr;
    a.nbq1 = q->nb[1]; a.nbq2 = q->nb[2]; a.nbq3 = q->nb[3];
    a.nbk1 = k->nb[1]; a.nbk2 = k->nb[2]; a.nbk3 = k->nb[3];
    a.nbv1 = v->nb[1]; a.nbv2 = v->nb[2]; a.nbv3 = v->nb[3];
    a.nbm1 = mask ? mask->nb[1] : 0; a.nbm2 = mask ? mask->nb[2] : 0; a.nbm3 = mask ? mask->nb[3] : 0;
    a.n_q = n_q; a.n_kv = n_kv; a.Hq = Hq; a.Hkv = Hkv; a.gqa = gqa;
    a.gqa_sh = 0;
    while ((1 << a.gqa_sh) < gqa) ++a.gqa_sh;
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
    a.vl = nullptr;

    // one workspace block: the mask's tile flags, then (F32 K/V) the f16 images of K, V high and V low
    const size_t bits_bytes = mask ? (size_t) a.nem2 * a.nem3 * n_q * n_tiles * 8 : 0;
    const size_t flag_bytes = mask ? ((bits_bytes + (size_t) a.nem2 * a.nem3 * n_rb * n_tiles + 255) & ~(size_t) 255) : 0;
    const size_t plane = a.kv_f32 ? (size_t) k->ne[3] * Hkv * n_kv * 64 * sizeof(_Float16) : 0;
    char * ws = nullptr;
    const size_t front_bytes = front ? front->bytes : 0;
    if (front_bytes + flag_bytes + 3 * plane) {
        void * p = nullptr;
        vx_status rc = vx_workspace(st, front_bytes + flag_bytes + 3 * plane, &p);
        if (rc != VX_OK) return rc;
        ws = (char *) p;
    }
    if (front) { // the caller's launches first: they own the front of the block, and leave the addend there
        const vx_status rc = front->launch(ws, front->ctx, st);
        if (rc != VX_OK) return rc;
        a.add1 = (const float *) (ws + front->addend_at);
        if (front->tiles) {
            a.tile_out = (_Float16 *) (ws + front->tiles_at);
            a.tile_tt = front->tile_tt; a.tile_bs = front->tile_bs; a.tile_ts = front->tile_ts;
        }
        ws += front_bytes;
    }
    if (mask) {
        vx_launch(pf_mask_flags_kernel, dim3((unsigned) n_tiles, (unsigned) n_rb, (unsigned) (a.nem2 * a.nem3)), dim3(64), 0, st,
            a.mask, a.nbm1, a.nbm2, a.nbm3, a.nem2, n_q, n_kv, RB, n_rb, n_tiles,
            (int) ((uintptr_t) a.mask % 16 == 0 && a.nbm1 % 16 == 0 && a.nbm2 % 16 == 0 && a.nbm3 % 16 == 0), (uint8_t *) ws + bits_bytes,
            (uint8_t *) ws);
        VX_LAUNCH_CHECK();
        a.bits = (const uint8_t *) ws;
        a.flags = (const uint8_t *) ws + bits_bytes;
    }
    if (a.kv_f32) {
        _Float16 * k16 = (_Float16 *) (ws + flag_bytes), * vhi = (_Float16 *) (ws + flag_bytes + plane), * vlo = (_Float16 *) (ws + flag_bytes + 2 * plane);
        vx_launch(pf_convert_kernel, dim3((unsigned) ((n_kv * 8 + 255) / 256), (unsigned) Hkv, (unsigned) k->ne[3]), dim3(256), 0, st,
            a.k, a.v, a.nbk1, a.nbk2, a.nbk3, a.nbv1, a.nbv2, a.nbv3, n_kv, Hkv, k16, vhi, vlo);
        VX_LAUNCH_CHECK();
        a.k = (const char *) k16; a.v = (const char *) vhi; a.vl = (const char *) vlo;
        a.nbk1 = a.nbv1 = 128; a.nbk2 = a.nbv2 = (uint64_t) n_kv * 128; a.nbk3 = a.nbv3 = (uint64_t) Hkv * n_kv * 128;
    }
    const dim3 grid((unsigned) (n_rb * n_groups)), block(64 * PF_WAVES);
    if (half_cols) {
        if (a.kv_f32) vx_launch(pf_kernel<true, 1>, grid, block, 0, st, a);
        else          vx_launch(pf_kernel<false, 1>, grid, block, 0, st, a);
    } else {
        vx_launch(pf_kernel<false, 2>, grid, block, 0, st, a);
    }
    VX_LAUNCH_CHECK();
    return VX_OK;
}
