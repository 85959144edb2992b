// mul_mat.hip -- GGML_OP_MUL_MAT on gfx950 for Q8_0 / F16 / F32 weights and F32 activations.
//
// dst[token][row] = sum_k x[token][k] * W[row][k], computed on the matrix cores as
// D[m = token][n = weight row] with v_mfma_f32_16x16x32_f16.  K = 32 of that instruction is
// exactly one Q8_0 block, so for quantised weights every MFMA yields the block's partial
// dot product with the weights still *integers* (int8 -> f16 is exact), and the block scale
// d is applied in fp32 afterwards: acc += d * partial.  The effective weight is q*d exactly,
// the value ggml's dequantize_row_q8_0 produces (ggml/src/ggml-quants.c:401-415).
//
// Operands (lane = 16*j + c):
//   B = W^T   lane c = weight row, k-slots 8j..8j+7 of the block: 8 bytes of a Q8_0 block
//             (2-byte aligned) turned into f16 with one xor, two byte permutes and two
//             packed subtracts per dword (bias trick: 0x6400|u is 1024+u in f16).
//   A = x     lane c = token; converted to f16 once per work-group and parked in LDS in
//             operand order, swizzled so both the staging writes and the operand reads
//             are bank-conflict free.
// With VX_ACT_Q8 the staging step quantises each 32-wide activation block the way
// ggml-cpu's x86 build does (id = 127/max, round half to even, d rounded to f16;
// ggml/src/ggml-cpu/arch/x86/quants.c:290-386): the MFMA then produces ggml-cpu's exact
// integer block dot and the scale is d_w * d_x.
//
// Tiling: a work-group is 4 waves.  GEMM shape (many tokens): 64 rows x 16*TT tokens, each
// wave 16 rows.  GEMV shape (<= 16 tokens): its own streaming kernel (gemv_kernel below); the
// staged K-split variant of the GEMM kernel remains for F32 weights and ragged K.
//
// Algorithmic HBM bytes: weights once (34 bytes per 32 weights) + activations + output.
#include "vx_common.hpp"
#include "rope_common.hpp"

#include <cstdlib>
#include <type_traits>

namespace {

constexpr int GV_MAX_SEG = 3;
struct gv_seg {
    const char * w; char * dst;
    int64_t  M;
    uint64_t nb01, nb1, nb2, nb3; // weight row stride; dst strides of token, ne2, ne3
    int wg0;                      // first work-group of this matrix
    int rope;                     // rotate (row d, row d + head_dim/2) pairs of every head before storing
};

struct mm_args {
    const char * w; const char * x; char * dst;
    int64_t K, M, N;
    uint64_t nb01, nb02, nb03, nb11, nb12, nb13, nb1, nb2, nb3;
    int ne12, r2, r3;
    int x_aligned; // src1 rows allow 16-byte vector loads
    int w_aligned; // Q8_0 rows start on dword boundaries
    int rows_wg;   // GEMV: weight rows per work-group (16, 8 or 4)
    const char * w2; // GEMV, fused gate/up + SwiGLU: the second weight matrix (same shape and strides), else null
    const char * res; // GEMV, fused residual update: dst = res + res_scale * (W x); null for a plain product
    uint64_t rnb1, rnb2, rnb3;
    float res_scale;
    // GEMV over several weight matrices that share the activations (the Q, K and V projections), each
    // with its own destination and optionally the NEOX rotation of GGML_OP_ROPE applied before the store
    gv_seg seg[GV_MAX_SEG];
    int nseg;
    const int32_t * pos; const float * ff;
    rope_params rp;
    int head_dim;
    int rope_T; // tokens per sequence: token n of the flattened (token, batch) order sits at position pos[n % rope_T]
    // tiled kernel, long K on a small grid: the K range is cut across ksplit work-groups that leave fp32 partials
    // [batch][split][token][row] for a second kernel to add in split order (ksplit <= 1: off)
    int ksplit;
    float * partial;
    size_t ws_offset; // bytes at the start of the stream's workspace that the caller keeps for itself: partials go behind them
    // pre-tiled kernel, mlp_forward as one call: the pair's epilogue writes silu(g) * u as the f16 activation tiles of the
    // product that follows (tile_out) instead of storing dst, and that product takes them as they are (tile_in) instead of
    // laying x out itself; tile_tt: 16-token tiles per k block in that buffer (whole 128-token tiles of the pair)
    void * tile_out; const void * tile_in; int tile_tt;
    // GEMV with RMS_NORM and the norm-weight MUL applied to the activations as they are staged
    // (x is then the un-normalised tensor): x[t][k] / rms(x[t]) * norm_w[k], rounded after each product
    const float * norm_w;
    float norm_eps;
    // GEMV prologue helpers, filled in by launch_gemv: everything a wave needs before it can request its weights is
    // kept free of integer divisions (a dependent chain of some thirty instructions each, ahead of the first load)
    int   nbatch;     // ne12 * ne13 of the activations; 1: no batch index arithmetic at all
    float inv_upr;    // 1 / (K / 8): (unit + 0.5) * inv_upr truncates to unit / (K / 8) exactly for every unit of a chunk
    int   half_shift; // log2(head_dim / 2) when that is a power of two, else -1
    int   exact;      // every wave's blocks fill its load rounds exactly: no clamping of block indices
    // gemv_dma_kernel: the weight rows of a work-group as an image in LDS
    int   w_lds_off;  // byte offset of the image in the work-group's dynamic LDS (a multiple of 16)
    int   w_slot;     // bytes between the images of consecutive MFMA columns: the row's bytes plus padding
};

// a + x * s with the product rounded before the sum, as a SCALE node followed by an ADD node rounds
__device__ __forceinline__ float scaled_residual(float x, float s, float a) {
#pragma clang fp contract(off)
    const float t = x * s;
    return a + t;
}

constexpr int WT_Q8 = 0, WT_F16 = 1, WT_F32 = 2;
constexpr int KC_BLOCKS = 4; // 32-wide k blocks staged per round

__device__ __forceinline__ float4_t mfma16(half8_t a, half8_t b, float4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}

// 8 int8 (two dwords) -> 8 f16, exactly
__device__ __forceinline__ half8_t q8_to_half8(uint32_t lo, uint32_t hi) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const uint32_t bias = 0x64646464u;
    lo ^= 0x80808080u;
    hi ^= 0x80808080u;
    u32x4 r;
    r[0] = __builtin_amdgcn_perm(bias, lo, 0x04010400u);
    r[1] = __builtin_amdgcn_perm(bias, lo, 0x04030402u);
    r[2] = __builtin_amdgcn_perm(bias, hi, 0x04010400u);
    r[3] = __builtin_amdgcn_perm(bias, hi, 0x04030402u);
    half8_t h = __builtin_bit_cast(half8_t, r);
    const _Float16 off = (_Float16) 1152.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] -= off;
    return h;
}

// The 8 quants lane-group j needs from Q8_0 block kb of a row: bytes 34*kb + 2 + 8j .. +8, which are
// only 2-byte aligned.  Vector loads that are not dword-aligned are served lane by lane and run
// several times slower, so when the row itself is dword-aligned (al4) the lane fetches the three
// aligned dwords that cover its bytes (never outside the block) and shifts them into place;
// whether a shift is needed depends only on the parity of kb.
struct q8_raw { uint32_t w0, w1, w2; };
__device__ __forceinline__ q8_raw q8_load(const char * wrow, int64_t kb, int j, bool al4) {
    q8_raw r;
    if (al4) {
        const char * p = (const char *) __builtin_assume_aligned(wrow + kb * VX_Q8_BLOCK + 8 * j - ((kb & 1) ? 2 : 0), 4);
        uint32_t v[3];
        __builtin_memcpy(v, p, 12);
        r.w0 = v[0]; r.w1 = v[1]; r.w2 = v[2];
    } else {
        uint32_t v[2];
        __builtin_memcpy(v, wrow + kb * VX_Q8_BLOCK + 2 + 8 * j, 8);
        r.w0 = 0; r.w1 = v[0]; r.w2 = v[1];
    }
    return r;
}
__device__ __forceinline__ half8_t q8_unpack(const q8_raw & r, int64_t kb, bool al4) {
    const bool shifted = al4 && !(kb & 1); // even blocks start on a dword: the quants sit 2 bytes in
    const uint32_t lo = shifted ? __builtin_amdgcn_alignbit(r.w1, r.w0, 16) : r.w1;
    const uint32_t hi = shifted ? __builtin_amdgcn_alignbit(r.w2, r.w1, 16) : r.w2;
    return q8_to_half8(lo, hi);
}

__device__ __forceinline__ int lds_slot(int kbl, int tt, int TT, int j, int c) {
    return ((kbl * TT + tt) * 4 + j) * 16 + ((c + 4 * kbl + j) & 15);
}

template <int WT, int TT, bool ACT_Q8, bool KSPLIT>
__global__ __launch_bounds__(256) void mm_kernel(const mm_args a) {
    __shared__ half8_t xs[KC_BLOCKS * TT * 64];
    __shared__ float   xd[ACT_Q8 ? KC_BLOCKS * TT * 16 : 1];
    __shared__ float4_t red[KSPLIT ? 3 * TT * 64 : 1];

    const int tid = threadIdx.x, wid = tid >> 6, lane = tid & 63;
    const int j = lane >> 4, c = lane & 15;

    const int     nsplit = (!KSPLIT && a.ksplit > 1) ? a.ksplit : 1; // uniform
    const int     batch = (int) blockIdx.z / nsplit, split = (int) blockIdx.z % nsplit;
    const int     i12 = batch % a.ne12, i13 = batch / a.ne12;
    const char *  wb  = a.w + (uint64_t) (i12 / a.r2) * a.nb02 + (uint64_t) (i13 / a.r3) * a.nb03;
    const char *  xb  = a.x + (uint64_t) i12 * a.nb12 + (uint64_t) i13 * a.nb13;
    char *        db  = a.dst + (uint64_t) i12 * a.nb2 + (uint64_t) i13 * a.nb3;
    uint64_t      dnb1 = a.nb1;
    if (nsplit > 1) { // this work-group's share goes to its slab of the partial buffer, dense [token][row]
        db   = (char *) (a.partial + ((uint64_t) batch * nsplit + split) * (uint64_t) a.N * a.M);
        dnb1 = (uint64_t) a.M * 4;
    }

    const int64_t tok0 = (int64_t) blockIdx.y * 16 * TT;
    const int64_t row0 = KSPLIT ? (int64_t) blockIdx.x * 16 : (int64_t) blockIdx.x * 64 + wid * 16;
    const int64_t row  = min(row0 + c, a.M - 1);
    const char *  wrow = wb + (uint64_t) row * a.nb01;

    float4_t acc[TT];
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) acc[tt] = float4_t{0, 0, 0, 0};

    const int64_t nkb_all = (a.K + 31) / 32;
    const int64_t per_split = ((nkb_all + nsplit - 1) / nsplit + KC_BLOCKS - 1) / KC_BLOCKS * KC_BLOCKS;
    const int64_t kb_first = (int64_t) split * per_split;
    const int64_t nkb = min(nkb_all, kb_first + per_split);
    for (int64_t kb0 = kb_first; kb0 < nkb; kb0 += KC_BLOCKS) {
        // ---- stage 16*TT tokens x 128 k of activations as f16 operands
#pragma unroll
        for (int it = 0; it < TT; ++it) {
            const int unit = tid + 256 * it;
            const int t = unit >> 4, u = unit & 15; // token within tile, 8-wide k unit
            const int kbl = u >> 2, uj = u & 3;
            const int64_t tok = tok0 + t;
            const int64_t k   = (kb0 + kbl) * 32 + uj * 8;
            float v[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = 0.0f;
            if (tok < a.N && k < a.K) {
                const float * xp = (const float *) (xb + (uint64_t) tok * a.nb11) + k;
                if (a.x_aligned && k + 8 <= a.K) {
                    const float4_t v0 = ((const float4_t *) xp)[0], v1 = ((const float4_t *) xp)[1];
#pragma unroll
                    for (int i = 0; i < 4; ++i) { v[i] = v0[i]; v[4 + i] = v1[i]; }
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) if (k + i < a.K) v[i] = xp[i];
                }
            }
            half8_t h;
            if constexpr (ACT_Q8) {
                float amax = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
                amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
                const float d  = amax / 127.f;
                const float id = amax != 0.0f ? 127.f / amax : 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = (_Float16) rintf(v[i] * id);
                if (uj == 0) xd[(kbl * TT + (t >> 4)) * 16 + (t & 15)] = (float) (_Float16) d;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = (_Float16) v[i];
            }
            xs[lds_slot(kbl, t >> 4, TT, uj, t & 15)] = h;
        }
        __syncthreads();

        // ---- multiply
#pragma unroll
        for (int kbl = 0; kbl < KC_BLOCKS; ++kbl) {
            if (KSPLIT && kbl != wid) continue;
            const int64_t kb = kb0 + kbl;
            if (kb >= nkb) break;
            half8_t bop;
            float   dw = 1.0f;
            if constexpr (WT == WT_Q8) {
                const char * bp = wrow + (uint64_t) kb * VX_Q8_BLOCK;
                dw = (float) *(const _Float16 *) bp;
                bop = q8_unpack(q8_load(wrow, kb, j, false), kb, false);
            } else if constexpr (WT == WT_F16) {
                const int64_t k = kb * 32 + 8 * j;
                if (k + 8 <= a.K) {
                    __builtin_memcpy(&bop, wrow + (uint64_t) k * 2, 16);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; ++i) bop[i] = k + i < a.K ? ((const _Float16 *) wrow)[k + i] : (_Float16) 0.0f;
                }
            } else {
                const int64_t k = kb * 32 + 8 * j;
#pragma unroll
                for (int i = 0; i < 8; ++i) bop[i] = k + i < a.K ? (_Float16) ((const float *) wrow)[k + i] : (_Float16) 0.0f;
            }
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                const half8_t aop = xs[lds_slot(kbl, tt, TT, j, c)];
                if constexpr (WT == WT_Q8) {
                    const float4_t blk = mfma16(aop, bop, float4_t{0, 0, 0, 0});
                    if constexpr (ACT_Q8) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[tt][r] += blk[r] * (dw * xd[(kbl * TT + tt) * 16 + 4 * j + r]);
                    } else {
                        acc[tt] += blk * dw;
                    }
                } else {
                    acc[tt] = mfma16(aop, bop, acc[tt]);
                }
            }
        }
        __syncthreads();
    }

    if constexpr (KSPLIT) {
        if (wid > 0) {
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) red[((wid - 1) * TT + tt) * 64 + lane] = acc[tt];
        }
        __syncthreads();
        if (wid > 0) return;
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
            for (int ww = 0; ww < 3; ++ww) acc[tt] += red[(ww * TT + tt) * 64 + lane];
    }

    // lane (j,c), register r: token tok0 + 16*tt + 4j + r, row row0 + c
    if (row0 + c < a.M) {
#pragma unroll
        for (int tt = 0; tt < TT; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t tok = tok0 + 16 * tt + 4 * j + r;
                if (tok < a.N) *(float *) (db + (uint64_t) tok * dnb1 + (uint64_t) (row0 + c) * 4) = acc[tt][r];
            }
    }
}

// adds the K-split partials in split order: one thread per 4 consecutive rows of one token
__global__ __launch_bounds__(256) void mm_splitk_reduce_kernel(const mm_args a) {
    const int64_t m4 = a.M / 4;
    const int64_t u = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (u >= a.N * m4) return;
    const int64_t tok = u / m4, r4 = (u % m4) * 4;
    const int     batch = blockIdx.z;
    const int     i12 = batch % a.ne12, i13 = batch / a.ne12;
    const float * p = a.partial + (uint64_t) batch * a.ksplit * (uint64_t) a.N * a.M + (uint64_t) tok * a.M + r4;
    float4_t acc = *(const float4_t *) p;
    for (int s = 1; s < a.ksplit; ++s) acc += *(const float4_t *) (p + (uint64_t) s * a.N * a.M);
    if (a.res) { // the fused residual update: dst = res + scale * (W x), rounded as the SCALE and the ADD node would
        const float * rp = (const float *) (a.res + (uint64_t) i12 * a.rnb2 + (uint64_t) i13 * a.rnb3 + (uint64_t) tok * a.rnb1 + (uint64_t) r4 * 4);
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = scaled_residual(acc[r], a.res_scale, rp[r]);
    }
    *(float4_t *) (a.dst + (uint64_t) i12 * a.nb2 + (uint64_t) i13 * a.nb3 + (uint64_t) tok * a.nb1 + (uint64_t) r4 * 4) = acc;
}


// ---- GEMV shape: few tokens (decode, LocDiT) --------------------------------------------------
// Pure weight streaming, so the kernel is built around memory-level parallelism: a work-group owns
// 16 weight rows, its NW waves take interleaved 32-wide k blocks of those rows, and every wave
// issues the loads of all its blocks (GV_UNROLL at a time, normally all of them) before anything
// else happens.  While they fly the work-group converts the few activation rows to f16 (or
// quantises them, VX_ACT_Q8) into LDS, [token][k].  Then one MFMA per block -- tokens that do not
// exist are zero lanes of the A operand -- and a fixed-order reduction of the waves' partial sums
// through LDS.  With K = 1024 and 4 waves, or K = 4096 and 16 waves, the whole matrix is requested
// in one round trip to HBM.
constexpr int GV_UNROLL = 8;

template <int WT, bool ACT_Q8, int NW, bool AL4, bool SEG, int UNR = GV_UNROLL>
__global__ __launch_bounds__(64 * NW) void gemv_kernel(const mm_args a) {
    extern __shared__ __attribute__((aligned(16))) char gv_smem[];
    const int nkb = (int) (a.K / 32);
    _Float16 * xs  = (_Float16 *) gv_smem;                                   // [N][K]
    const int NL = (int) (a.N < 16 ? a.N : 16);                              // tokens a work-group stages
    float *    xd  = (float *) (gv_smem + (size_t) NL * a.K * 2);            // [NL][K/32] (ACT_Q8)
    float4_t * red = (float4_t *) (gv_smem + (size_t) NL * a.K * 2 + (ACT_Q8 ? (size_t) NL * nkb * 4 : 0));
    float *    nsc = (float *) (red + (NW > 1 ? NW - 1 : 0) * 64); // [16] per-token 1 / rms (fused RMS_NORM)
    float2 *   rcs = (float2 *) (nsc + 16);                          // [4][64] cos / sin exchanged between waves (SEG)

    const int tid = threadIdx.x, wid = tid >> 6, lane = tid & 63;
    const int j = lane >> 4, c = lane & 15;
    const int     batch = blockIdx.z;
    // more than 16 tokens: blockIdx.y picks a chunk of 16; the chunks' work-groups stream the same weight
    // rows, which the first one pulls into L2
    const int     tok0 = 16 * (int) blockIdx.y;
    // batch offsets: all zero for the common single-sequence call, which then skips the divisions and the 64-bit products
    int           i12 = 0, i13 = 0;
    uint64_t      w_off = 0, x_off = 0, d_off = 0, r_off = 0;
    if (a.nbatch > 1) { // uniform
        i12 = batch % a.ne12; i13 = batch / a.ne12;
        w_off = (uint64_t) (i12 / a.r2) * a.nb02 + (uint64_t) (i13 / a.r3) * a.nb03;
        x_off = (uint64_t) i12 * a.nb12 + (uint64_t) i13 * a.nb13;
        d_off = (uint64_t) i12 * a.nb2 + (uint64_t) i13 * a.nb3;
        r_off = (uint64_t) i12 * a.rnb2 + (uint64_t) i13 * a.rnb3;
    }
    if (tok0) { x_off += (uint64_t) tok0 * a.nb11; r_off += (uint64_t) tok0 * a.rnb1; } // uniform
    const char *  xb  = a.x + x_off;
    const char *  wb  = a.w + w_off;
    char *        db  = a.dst + d_off;
    int           M = (int) a.M;
    uint64_t      nb01 = a.nb01, nb1 = a.nb1;
    int           wl = blockIdx.x; // work-group index within its matrix
    bool          rope = false;
    if constexpr (SEG) {
        int sg = 0;
        if (a.nseg > 1 && wl >= a.seg[1].wg0) sg = 1;
        if (a.nseg > 2 && wl >= a.seg[2].wg0) sg = 2;
        const gv_seg & S = a.seg[sg];
        wb = S.w; db = S.dst;
        if (a.nbatch > 1) db += (uint64_t) i12 * S.nb2 + (uint64_t) i13 * S.nb3;
        M = (int) S.M; nb01 = S.nb01; nb1 = S.nb1;
        wl -= S.wg0;
        rope = S.rope != 0;
    }
    // R = a.rows_wg (16, 8 or 4) of the 16 MFMA columns carry weight rows; fewer rows per work-group put a short
    // matrix on more CUs (a CU sustains only so many outstanding lines, so 64 work-groups cannot
    // pull what 256 can).  Lanes c >= R load nothing; their columns are never stored.
    // With a second matrix (SwiGLU: dst = silu(W x) * (W2 x)) the MFMA columns are split: the first half of
    // them carries rows of W, the second half the same rows of W2, and the epilogue pairs them up.
    const bool    dual = a.w2 != nullptr;                 // uniform
    const int     R  = a.rows_wg, Rr = dual ? R / 2 : R;   // MFMA columns in use, output rows per work-group (powers of two)
    // the weight row of MFMA column cc.  Plain: consecutive rows.  With the rotation the R columns hold R/2
    // pairs (d, d + head_dim/2) of one head, first elements in columns 0 .. R/2-1, partners in the rest.
    // Rows are counted in 32 bits (the host checks M < 2^31).
    const int     h2 = R >> 1, half_dim = a.head_dim >> 1;
    auto column = [&](int cc, int & row_, int & pair_, bool & ok_, const char *& wrow_) {
        const int cr = dual ? (cc & (Rr - 1)) : cc;
        row_  = wl * Rr + cr;
        pair_ = 0; // index of the pair within its head: the rotation's frequency index
        if (SEG && rope) {
            const unsigned f = (unsigned) (wl * h2 + (cc & (h2 - 1)));
            const unsigned head = a.half_shift >= 0 ? f >> a.half_shift : f / (unsigned) half_dim;
            pair_ = (int) (f - head * (unsigned) half_dim);
            row_  = (int) head * a.head_dim + pair_ + (cc >= h2 ? half_dim : 0);
        }
        ok_ = cc < R && row_ < M;
        const char * wsel = (dual && cc >= Rr) ? a.w2 + w_off : wb;
        wrow_ = wsel + (uint64_t) (unsigned) min(row_, M - 1) * nb01;
    };
    int           row;
    int           pair;
    bool          row_ok;
    const char *  wrow;
    column(c, row, pair, row_ok, wrow);
    // Fetching in MFMA layout -- lane (j,c) = chunk j of row c -- makes every 16-lane group of a load touch 16 rows,
    // 16 cache lines for 12 useful bytes each, and the CU's vector cache serves one line per cycle.  With dword-aligned
    // Q8_0 rows the fetch is therefore done in row-major lane order (lane l = chunk l & 3 of column l >> 2: four rows
    // per 16 lanes) and the dwords are handed to their MFMA lanes by a cross-lane permute once they have arrived;
    // the block scale rides in the first dword of chunk 0, so it needs no load of its own.
    constexpr bool PERM = WT == WT_Q8 && AL4;
    int           row_ld;
    int           pair_ld;
    bool          ld_ok = row_ok;
    const char *  wrow_ld = wrow;
    if constexpr (PERM) column(lane >> 2, row_ld, pair_ld, ld_ok, wrow_ld);
    const int     j_ld = PERM ? (lane & 3) : j;
    const int     perm_src = (4 * c + j) * 4, perm_src0 = (4 * c) * 4; // byte addresses of the source lanes
    const int     N = min(16, (int) a.N - tok0); // tokens of this chunk
    if (tok0) db += (uint64_t) tok0 * nb1;

    // ---- this wave's weight blocks: kb = wid + NW * i
    constexpr bool al4 = AL4;
    q8_raw   wq[UNR];
    half8_t  wh[UNR];
    _Float16 wdv[UNR];
    // Exact rounds (the usual shapes): block wid + NW * (i0 + u) of the lane's row sits at a compile-time distance from the
    // round's first block, and an even wave count keeps the parity of a wave's blocks fixed -- one base address per lane and
    // round, the loads take immediate offsets.  Otherwise block indices are clamped (a valid address, the result unused).
    auto load_blocks = [&](int i0) {
        if (!ld_ok) {
#pragma unroll
            for (int u = 0; u < UNR; ++u) { wq[u] = q8_raw{0, 0, 0}; wdv[u] = (_Float16) 0.0f; wh[u] = half8_t{0, 0, 0, 0, 0, 0, 0, 0}; }
            return;
        }
        if constexpr (WT == WT_Q8 && PERM && NW % 2 == 0) {
            if (a.exact) { // uniform
                const char * p0 = wrow_ld + (wid + NW * i0) * VX_Q8_BLOCK + 8 * j_ld - ((wid & 1) ? 2 : 0);
#pragma unroll
                for (int u = 0; u < UNR; ++u) {
                    uint32_t v[3];
                    __builtin_memcpy(v, (const char *) __builtin_assume_aligned(p0 + u * NW * VX_Q8_BLOCK, 4), 12);
                    wq[u] = q8_raw{v[0], v[1], v[2]};
                }
                return;
            }
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int kb = min(wid + NW * (i0 + u), nkb - 1);
            if constexpr (WT == WT_Q8) {
                if constexpr (!PERM) wdv[u] = *(const _Float16 *) (wrow_ld + (uint64_t) kb * VX_Q8_BLOCK);
                wq[u] = q8_load(wrow_ld, kb, j_ld, al4);
            } else {
                __builtin_memcpy(&wh[u], wrow + (uint64_t) (kb * 32 + 8 * j) * 2, 16);
            }
        }
    };
    // ---- activations -> LDS.  A thread's first unit (8 consecutive k of one token; usually its only
    // one) is requested before the weights: loads return in order, so its conversion then waits for
    // an L2 hit only, not for the weight stream behind it.
    const int upr = (int) (a.K / 8), units = N * upr;
    auto unit_token = [&](int unit) { return (int) (((float) unit + 0.5f) * a.inv_upr); }; // = unit / upr
    auto fetch = [&](int unit, float4_t & v0, float4_t & v1) {
        const int t = unit_token(unit), u = unit - t * upr;
        const float * xp = (const float *) (xb + (uint64_t) t * a.nb11) + 8 * u;
        if (a.x_aligned) {
            v0 = ((const float4_t *) xp)[0]; v1 = ((const float4_t *) xp)[1];
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) { v0[i] = xp[i]; v1[i] = xp[4 + i]; }
        }
    };
    auto stage = [&](int unit, const float4_t & v0, const float4_t & v1, const float4_t & g0, const float4_t & g1) {
        const int t = unit_token(unit), u = unit - t * upr;
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = v0[i]; v[4 + i] = v1[i]; }
        if (a.norm_w) { // RMS_NORM's product, then the MUL node's, each rounded as the separate kernels round them
            const float sc = nsc[t];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[i]     *= sc; v[i]     *= g0[i];
                v[4 + i] *= sc; v[4 + i] *= g1[i];
            }
        }
        half8_t h;
        if constexpr (ACT_Q8) { // 4 consecutive units = one 32-wide block (K/8 is a multiple of 4)
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
            amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
            const float d  = amax / 127.f;
            const float id = amax != 0.0f ? 127.f / amax : 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = (_Float16) rintf(v[i] * id);
            if ((u & 3) == 0) xd[t * nkb + (u >> 2)] = (float) (_Float16) d;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = (_Float16) v[i];
        }
        *(half8_t *) (xs + (size_t) t * a.K + 8 * u) = h;
    };
    float4_t f0 = {0, 0, 0, 0}, f1 = {0, 0, 0, 0}, g0 = {1, 1, 1, 1}, g1 = {1, 1, 1, 1};
    if (tid < units) fetch(tid, f0, f1);
    auto fetch_gain = [&](int unit, float4_t & a0, float4_t & a1) { // the norm weights of a unit's 8 columns (16-byte aligned)
        const float4_t * gp = (const float4_t *) (a.norm_w + 8 * (unit - unit_token(unit) * upr));
        a0 = gp[0]; a1 = gp[1];
    };
    if (a.norm_w && tid < units) fetch_gain(tid, g0, g1);
    // the row this wave normalises first (token wid), also requested ahead of the weights
    vx_rms_row nrow;
    if (a.norm_w && wid < N) vx_rms_row_load(nrow, (const float *) (xb + (uint64_t) wid * a.nb11), a.K, lane);
    vx_rms_row nrow2; // the wave's second token (more tokens than waves), requested up front as well
    if (a.norm_w && wid + NW < N) vx_rms_row_load(nrow2, (const float *) (xb + (uint64_t) (wid + NW) * a.nb11), a.K, lane);
    // the residual values the storing wave will need, requested ahead of the weight stream as well
    float resv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (a.res && wid == 0 && row_ok && c < Rr) {
        const char * rb = a.res + r_off + (uint64_t) row * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            if (4 * j + r < N) resv[r] = *(const float *) (rb + (uint64_t) (4 * j + r) * a.rnb1);
    }
    load_blocks(0);
    // the rotation's cos / sin for this lane's (token, pair) values: computed while the weights fly
    float rc[4] = {1.0f, 1.0f, 1.0f, 1.0f}, rs[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    // an angle costs a chain of multiplications and two accurate trigonometric evaluations: with four waves or more, wave r
    // computes token slot r of every lane and the storing wave collects the four through LDS
    constexpr bool ROPE_SPREAD = SEG && NW >= 4;
    if (SEG && rope && row_ok && (ROPE_SPREAD ? wid < 4 : wid == 0)) {
        const float ffv = a.ff ? a.ff[pair] : 1.0f;
        if constexpr (ROPE_SPREAD) {
            float cv = 1.0f, sv = 0.0f;
            if (4 * j + wid < N) rope_cos_sin(a.rp, (float) a.pos[(batch * (int) a.N + tok0 + 4 * j + wid) % a.rope_T], pair, ffv, cv, sv);
            rcs[wid * 64 + lane] = float2{cv, sv};
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (4 * j + r < N) rope_cos_sin(a.rp, (float) a.pos[(batch * (int) a.N + tok0 + 4 * j + r) % a.rope_T], pair, ffv, rc[r], rs[r]);
        }
    }
    if (a.norm_w) { // one wave per token, as the RMS_NORM kernel has it; a wave with several tokens takes two at a time
        for (int t = wid; t < N; t += 2 * NW) {
            if (t != wid) vx_rms_row_load(nrow, (const float *) (xb + (uint64_t) t * a.nb11), a.K, lane);
            if (t + NW < N) {
                if (t != wid) vx_rms_row_load(nrow2, (const float *) (xb + (uint64_t) (t + NW) * a.nb11), a.K, lane);
                float s1, s2;
                vx_rms_row_scale2(nrow, nrow2, a.K, lane, a.norm_eps, s1, s2);
                if (lane == 0) { nsc[t] = s1; nsc[t + NW] = s2; }
            } else {
                const float sc = vx_rms_row_scale(nrow, a.K, lane, a.norm_eps);
                if (lane == 0) nsc[t] = sc;
            }
        }
        __syncthreads();
    }
    if (tid < units) stage(tid, f0, f1, g0, g1);
    for (int unit = tid + 64 * NW; unit < units; unit += 64 * NW) {
        fetch(unit, f0, f1);
        if (a.norm_w) fetch_gain(unit, g0, g1);
        stage(unit, f0, f1, g0, g1);
    }
    __syncthreads();
    if constexpr (ROPE_SPREAD) {
        if (rope && row_ok && wid == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) { const float2 v = rcs[r * 64 + lane]; rc[r] = v.x; rs[r] = v.y; }
        }
    }
    float4_t acc = {0, 0, 0, 0};
    const int per = (nkb + NW - 1) / NW; // blocks per wave
    for (int i0 = 0; i0 < per; i0 += UNR) {
        if (i0) load_blocks(i0);
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
            const int kb = wid + NW * (i0 + u);
            if (kb >= nkb) break; // wave-uniform
            half8_t aop = {0, 0, 0, 0, 0, 0, 0, 0};
            if (c < N) aop = *(const half8_t *) (xs + (size_t) c * a.K + kb * 32 + 8 * j);
            if constexpr (WT == WT_Q8) {
                q8_raw raw = wq[u];
                float  dw;
                if constexpr (PERM) {
                    const uint32_t first = (uint32_t) __builtin_amdgcn_ds_bpermute(perm_src0, (int) raw.w0); // chunk 0 of this lane's row
                    raw.w0 = (uint32_t) __builtin_amdgcn_ds_bpermute(perm_src, (int) raw.w0);
                    raw.w1 = (uint32_t) __builtin_amdgcn_ds_bpermute(perm_src, (int) raw.w1);
                    raw.w2 = (uint32_t) __builtin_amdgcn_ds_bpermute(perm_src, (int) raw.w2);
                    // an even block starts on a dword with its scale in front; the fetch of an odd block starts 2 bytes early
                    dw = (float) __builtin_bit_cast(_Float16, (uint16_t) ((kb & 1) ? first >> 16 : first & 0xffffu));
                } else {
                    dw = (float) wdv[u];
                }
                const half8_t  bop = q8_unpack(raw, kb, al4);
                const float4_t blk = mfma16(aop, bop, float4_t{0, 0, 0, 0});
                if constexpr (ACT_Q8) {
#pragma unroll
                    for (int r = 0; r < 4; ++r) acc[r] += blk[r] * (dw * (4 * j + r < N ? xd[(4 * j + r) * nkb + kb] : 0.0f));
                } else {
                    acc += blk * dw;
                }
            } else {
                acc = mfma16(aop, wh[u], acc);
            }
        }
    }
    if constexpr (NW > 1) {
        if (wid > 0) red[(wid - 1) * 64 + lane] = acc;
        __syncthreads();
        if (wid > 0) return;
#pragma unroll
        for (int ww = 0; ww < NW - 1; ++ww) acc += red[ww * 64 + lane];
    }
    // lane (j,c), register r: token 4j + r, row row0 + c
    if (dual) { // lane c < Rr holds W's row, lane c + Rr the same row of W2: dst = silu(gate) * up
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float up = __shfl(acc[r], lane + Rr, 64);
            acc[r] = (acc[r] / (1.0f + expf(-acc[r]))) * up;
        }
    }
    if (a.res) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = scaled_residual(acc[r], a.res_scale, resv[r]);
    }
    if (SEG && rope) { // column c < R/2 holds x0 of its pair, column c + R/2 the partner x1
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float other = __shfl_xor(acc[r], h2, 64);
            const bool  first = c < h2;
            float y0, y1;
            rope_rotate(first ? acc[r] : other, first ? other : acc[r], rc[r], rs[r], y0, y1);
            acc[r] = first ? y0 : y1;
        }
    }
    if (row_ok && c < Rr) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tok = 4 * j + r;
            if (tok < N) *(float *) (db + (uint64_t) tok * nb1 + (uint64_t) row * 4) = acc[r];
        }
    }
}

// ---- GEMV shape, weights through LDS --------------------------------------------------------------------
// The same product as gemv_kernel -- same work-groups, same k blocks per wave, same order of every sum -- for the common
// case (Q8_0 rows and F32 activation rows on 16-byte boundaries, one batch entry, eight or sixteen waves), organised around
// two facts measured on this chip: a wave issues one instruction every four cycles or so, whatever the instruction, and a
// wave's loads return in order.  So
//   * the weight rows do not pass through registers: the first half of the waves copies them into LDS with direct loads
//     (64 lanes x 16 consecutive bytes of one row per instruction -- whole cache lines instead of 12-byte pieces of sixteen
//     rows), starts doing so a few dozen instructions after the kernel begins, and then only waits for them;
//   * the other half does everything on the activations' side (fetch, the fused norm, staging as f16 or Q8, the rotation's
//     angles): with no weight loads of their own in flight, they see their data after an L2 hit;
//   * after the barrier every wave takes its k blocks' bytes from the LDS image (each column's image padded so that the
//     sixteen columns fall into different banks), all reads of a round issued before the first is used.
// What is fused is a template parameter here, so that a wave executes no instruction of a path it does not take.
__device__ __forceinline__ void gv_dma16(const char * g, uint32_t lds_base) {
    // 16 bytes per lane from global memory straight into LDS: lane l's land at lds_base + 16 l (lds_base uniform).  M0 carries
    // the LDS address; the compiler keeps nothing in M0 across statements (it sets it right before each instruction that reads it).
    const uint32_t base = (uint32_t) __builtin_amdgcn_readfirstlane((int) lds_base);
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(base) : "memory");
}

enum gv_epilogue : int { GV_PLAIN = 0, GV_RES = 1, GV_SWIGLU = 2 };

// Four k blocks of one wave from the LDS images: blocks kb, kb + NW, kb + 2 NW, kb + 3 NW sit at compile-time distances, and
// with an even wave count they share their parity, so a round is straight-line code over three addresses: all reads first,
// then the four products, then the four scaled additions (in block order, as everywhere).
//   sp: this lane's column image at block kb (where the block's scale sits); xp: this lane's token at k = 32 kb + 8 j;
//   xdp (ACT_Q8): the activations' block scales of block kb, [block][16 tokens], at token 4 j
template <bool ACT_Q8, int NW, bool ODD>
__device__ __forceinline__ void gv_round4(const char * sp, int j, const _Float16 * xp, const float * xdp, float4_t & acc) {
    q8_raw   raw[4];
    _Float16 dwh[4];
    half8_t  aop[4];
    float4_t xdv[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const char * bp = sp + u * NW * VX_Q8_BLOCK;
        if constexpr (ODD) { // the block starts 2 bytes past a dword: its quants are dword-aligned
            const uint32_t * q = (const uint32_t *) (bp + 2 + 8 * j);
            raw[u] = q8_raw{ 0, q[0], q[1] };
        } else {             // the block starts on a dword: the quants sit 2 bytes in
            const uint32_t * q = (const uint32_t *) (bp + 8 * j);
            raw[u] = q8_raw{ q[0], q[1], q[2] };
        }
        dwh[u] = *(const _Float16 *) bp;
        aop[u] = *(const half8_t *) (xp + u * NW * 32);
        if constexpr (ACT_Q8) xdv[u] = *(const float4_t *) (xdp + u * NW * 16);
    }
    float4_t blk[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) blk[u] = mfma16(aop[u], q8_unpack(raw[u], ODD ? 1 : 0, true), float4_t{0, 0, 0, 0});
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const float dw = (float) dwh[u];
        if constexpr (ACT_Q8) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[r] += blk[u][r] * (dw * xdv[u][r]);
        } else {
            acc += blk[u] * dw;
        }
    }
}

template <bool ACT_Q8, int NW, bool SEG, bool NORM, int EPI, bool MANY>
__global__ __launch_bounds__(64 * NW) void gemv_dma_kernel(const mm_args a) {
    static_assert(NW == 4 || NW == 8 || NW == 16, "four, eight or sixteen waves");
    constexpr int  NWD = NW / 2, NA = NW - NWD; // waves 0 .. NWD-1 fetch the weights, the rest handle the activations
    constexpr bool dual = EPI == GV_SWIGLU;
    extern __shared__ __attribute__((aligned(16))) char gv_smem[];
    const int K = (int) a.K, nkb = K >> 5;
    const int KP = K + 8; // halfs between staged tokens; the padding spreads the tokens over the banks
    const int tok0 = 16 * (int) blockIdx.y;
    const int N  = min(16, (int) a.N - tok0); // tokens of this chunk
    const int NL = (int) (a.N < 16 ? a.N : 16);
    _Float16 * xs  = (_Float16 *) gv_smem;                                   // [N][KP]
    float *    xd  = (float *) (gv_smem + (size_t) NL * KP * 2);             // [K/32][16 tokens] (ACT_Q8): the activations' block scales
    // the waves' partial sums take the activations' place once every wave has walked its blocks (sixteen tokens of K = 4096
    // and the partials of sixteen waves do not fit a CU's LDS side by side); the region holds whichever is larger
    float4_t * red = (float4_t *) gv_smem;
    const size_t act_bytes = (size_t) NL * KP * 2 + (ACT_Q8 ? (size_t) 16 * nkb * 4 : 0), red_bytes = (size_t) (NW - 1) * 64 * 16;
    float *    nsc = (float *) (gv_smem + (act_bytes > red_bytes ? act_bytes : red_bytes)); // [16] (unused: kept for the layout)
    float2 *   rcs = (float2 *) (nsc + 16);                                  // [4][64] cos / sin of four token slots (SEG)
    const char * w_lds = gv_smem + a.w_lds_off;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wid = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane >> 4, c = lane & 15;

    // ---- which matrix, which rows
    int          wl = blockIdx.x; // work-group index within its matrix
    int          M = (int) a.M;
    const char * wb = a.w;
    char *       db = a.dst;
    uint64_t     nb01 = a.nb01, nb1 = a.nb1;
    bool         rope = false;
    if constexpr (SEG) {
        int sg = 0;
        if (a.nseg > 1 && wl >= a.seg[1].wg0) sg = 1;
        if (a.nseg > 2 && wl >= a.seg[2].wg0) sg = 2;
        const gv_seg & S = a.seg[sg];
        wb = S.w; db = S.dst; M = (int) S.M; nb01 = S.nb01; nb1 = S.nb1;
        wl -= S.wg0;
        rope = S.rope != 0;
    }
    const int R = a.rows_wg, Rr = dual ? R / 2 : R; // MFMA columns in use, output rows per work-group (powers of two)
    const int h2 = R >> 1, half_dim = a.head_dim >> 1;
    // the weight row of MFMA column cc, as gemv_kernel has it
    auto column = [&](int cc, int & row_, int & pair_, bool & ok_, const char *& wrow_) {
        const int cr = dual ? (cc & (Rr - 1)) : cc;
        row_  = wl * Rr + cr;
        pair_ = 0;
        if (SEG && rope) {
            const unsigned f = (unsigned) (wl * h2 + (cc & (h2 - 1)));
            const unsigned head = a.half_shift >= 0 ? f >> a.half_shift : f / (unsigned) half_dim;
            pair_ = (int) (f - head * (unsigned) half_dim);
            row_  = (int) head * a.head_dim + pair_ + (cc >= h2 ? half_dim : 0);
        }
        ok_ = cc < R && row_ < M;
        const char * wsel = (dual && cc >= Rr) ? a.w2 : wb;
        wrow_ = wsel + (uint64_t) (unsigned) min(row_, M - 1) * nb01;
    };

    const int upr = K >> 3, units = N * upr; // a unit: 8 consecutive k of one token
    auto unit_token = [&](int unit) { return (int) (((float) unit + 0.5f) * a.inv_upr); }; // = unit / upr
    const char * xb = a.x + (uint64_t) tok0 * a.nb11;
    float resv[4] = {0.0f, 0.0f, 0.0f, 0.0f};

    // ---- activations without a norm: units of 8 values, a thread's units UB at a time (requested together, then staged: a
    // round trip per unit would be paid a dozen times with sixteen tokens).  With many units the waves that fetch the weights
    // take a share once their requests are out -- until the rows land they have nothing else to do.
    auto fetch = [&](int unit, float4_t & v0, float4_t & v1) {
        const int t = unit_token(unit), u = unit - t * upr;
        const float4_t * xp = (const float4_t *) ((const float *) (xb + (uint64_t) t * a.nb11) + 8 * u);
        v0 = xp[0]; v1 = xp[1];
    };
    auto stage = [&](int unit, const float4_t & v0, const float4_t & v1) {
        const int t = unit_token(unit), u = unit - t * upr;
        float v[8];
#pragma unroll
        for (int i = 0; i < 4; ++i) { v[i] = v0[i]; v[4 + i] = v1[i]; }
        half8_t h;
        if constexpr (ACT_Q8) { // 4 consecutive units = one 32-wide block
            float amax = 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
            amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
            amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
            const float d  = amax / 127.f;
            const float id = amax != 0.0f ? 127.f / amax : 0.0f;
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = (_Float16) rintf(v[i] * id);
            if ((u & 3) == 0) xd[(u >> 2) * 16 + t] = (float) (_Float16) d;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] = (_Float16) v[i];
        }
        *(half8_t *) (xs + (size_t) t * KP + 8 * u) = h;
    };
    constexpr int  UB = MANY ? (NW == 16 ? 4 : 8) : 1;
    constexpr bool SHARE = MANY && !NORM;                 // the weight-fetching waves stage units too
    constexpr int  USTRIDE = 64 * (SHARE ? NW : NA);      // the staging threads' stride in units
    auto stage_rest = [&](int first) { // units first, first + USTRIDE, ... : UB requests together, then their staging
        float4_t f0[UB], f1[UB];
        for (int base = first; base < units; base += UB * USTRIDE) {
#pragma unroll
            for (int i = 0; i < UB; ++i) {
                const int unit = base + i * USTRIDE;
                if (unit < units) fetch(unit, f0[i], f1[i]);
            }
#pragma unroll
            for (int i = 0; i < UB; ++i) {
                const int unit = base + i * USTRIDE;
                if (unit < units) stage(unit, f0[i], f1[i]);
            }
        }
    };

    // ---- fused RMS_NORM: a token's row belongs to ONE wave, as in the RMS_NORM kernel: the wave reads the row once, sums its
    // squares, and stages the normalised row from the registers it already holds.  Lane l holds columns 4 (l + 64 c) .. + 3.
    // Tokens are dealt in pairs: the first 2 NA to the activation waves (t, t + NA), the next 2 NWD to the waves that fetch
    // the weights (they have nothing to do while their requests are under way), anything beyond to the activation waves again.
        const int nv = (int) (a.K >> 8); // 16-byte pieces of a row per lane (K is a multiple of 256 here)
        // the norm weights of this lane's columns: requested with the rows, in registers when the scale is known
        auto load_gains = [&](vx_rms_row & gn) {
#pragma unroll
            for (int cc = 0; cc < 8; ++cc)
                if (cc < nv) gn.v[cc] = ((const float4 *) a.norm_w)[lane + 64 * cc];
        };
        auto stage_row = [&](int t, const vx_rms_row & r, float sc, const vx_rms_row & gn) {
#pragma unroll
            for (int cc = 0; cc < 8; ++cc) {
                if (cc >= nv) break;
                const int    iv = lane + 64 * cc;
                const float4 g  = gn.v[cc];
                // RMS_NORM's product, then the MUL node's, each rounded as the separate kernels round them
                float v[4] = { r.v[cc].x, r.v[cc].y, r.v[cc].z, r.v[cc].w };
                const float gg[4] = { g.x, g.y, g.z, g.w };
#pragma unroll
                for (int i = 0; i < 4; ++i) { v[i] *= sc; v[i] *= gg[i]; }
                half4_t h;
                if constexpr (ACT_Q8) { // 8 consecutive lanes = one 32-wide block
                    float amax = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3])));
                    amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
                    amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
                    amax = fmaxf(amax, __shfl_xor(amax, 4, 64));
                    const float d  = amax / 127.f;
                    const float id = amax != 0.0f ? 127.f / amax : 0.0f;
#pragma unroll
                    for (int i = 0; i < 4; ++i) h[i] = (_Float16) rintf(v[i] * id);
                    if ((lane & 7) == 0) xd[(iv >> 3) * 16 + t] = (float) (_Float16) d;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) h[i] = (_Float16) v[i];
                }
                *(half4_t *) (xs + (size_t) t * KP + 4 * iv) = h;
            }
        };
    auto norm_pair = [&](int t, int stride) { // tokens t and t + stride (if there is one) by this wave
        vx_rms_row r1, r2, gn;
        vx_rms_row_load(r1, (const float *) (xb + (uint64_t) t * a.nb11), a.K, lane);
        if (t + stride < N) {
            vx_rms_row_load(r2, (const float *) (xb + (uint64_t) (t + stride) * a.nb11), a.K, lane);
            load_gains(gn);
            float s1, s2;
            vx_rms_row_scale2(r1, r2, a.K, lane, a.norm_eps, s1, s2);
            stage_row(t, r1, s1, gn);
            stage_row(t + stride, r2, s2, gn);
        } else {
            load_gains(gn);
            stage_row(t, r1, vx_rms_row_scale(r1, a.K, lane, a.norm_eps), gn);
        }
    };

    if (wid < NWD) {
        // ---- weight rows -> LDS.  These waves share their SIMDs with the activation waves: until the requests are out they go first
        __builtin_amdgcn_s_setprio(3);
        const uint32_t lds0 = (uint32_t) (uintptr_t) (__attribute__((address_space(3))) char *) gv_smem + (uint32_t) a.w_lds_off;
        const int units_row = (nkb * VX_Q8_BLOCK) >> 4;
        for (int cc = wid; cc < R; cc += NWD) { // a wave takes whole columns: one row address, then 1 KiB pieces of it
            int          row_t, pair_t;
            bool         ok_t;
            const char * wrow_t;
            column(cc, row_t, pair_t, ok_t, wrow_t);
            if (!ok_t) continue;
            const char * g   = wrow_t + (size_t) lane * 16;
            uint32_t     dst = lds0 + (uint32_t) (cc * a.w_slot);
            for (int u = lane; u < units_row; u += 64, g += 1024, dst += 1024) gv_dma16(g, dst);
        }
        __builtin_amdgcn_s_setprio(0);
        if constexpr (EPI == GV_RES) { // the residual values the storing wave will need: in flight with the weights
            int          row_c, pair_c;
            bool         ok_c;
            const char * wrow_c;
            column(c, row_c, pair_c, ok_c, wrow_c);
            if (wid == 0 && ok_c) {
                const char * rb = a.res + (uint64_t) tok0 * a.rnb1 + (uint64_t) row_c * 4;
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (4 * j + r < N) resv[r] = *(const float *) (rb + (uint64_t) (4 * j + r) * a.rnb1);
            }
        }
        if constexpr (SEG) { // the rotation's cos / sin, four token slots per lane: arithmetic that waits for nothing, done
                             // by these waves while their requests are under way (the other waves have the tokens' rows)
            if (rope && wid < 4) {
                int  row_c, pair_c;
                bool ok_c;
                const char * wrow_c;
                column(c, row_c, pair_c, ok_c, wrow_c);
                const float ffv = a.ff ? a.ff[pair_c] : 1.0f;
                for (int slot = wid; slot < 4; slot += NWD) {
                    float cv = 1.0f, sv = 0.0f;
                    if (ok_c && 4 * j + slot < N) rope_cos_sin(a.rp, (float) a.pos[(tok0 + 4 * j + slot) % a.rope_T], pair_c, ffv, cv, sv);
                    rcs[slot * 64 + lane] = float2{cv, sv};
                }
            }
        }
        if constexpr (NORM) { // (requested behind the weights, these rows arrive behind them)
            if (2 * NA + wid < N) norm_pair(2 * NA + wid, NWD);
        }
        if constexpr (SHARE) stage_rest(64 * NA + tid);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wave's direct loads have landed (they are not known to the compiler)
    } else {
        // ---- activations -> LDS as f16 (or quantised), [token][k]
        const int awid = wid - NWD, atid = tid - 64 * NWD;
        float4_t f0[UB], f1[UB]; // this thread's first UB units, requested before the other work of the wave
        if constexpr (!NORM) {
#pragma unroll
            for (int i = 0; i < UB; ++i) {
                const int unit = atid + i * USTRIDE;
                if (unit < units) fetch(unit, f0[i], f1[i]);
            }
        }
        // With a fused norm a token's row belongs to ONE wave, as in the RMS_NORM kernel: the wave reads the row once, sums
        // its squares, and stages the normalised row from the registers it already holds -- no second trip for the values,
        // no exchange of scales between the waves.  Lane l holds columns 4 (l + 64 c) .. + 3 of the row.
        vx_rms_row nrow, nrow2, ngain; // the tokens this wave normalises first (and the norm weights), requested up front
        if constexpr (NORM) {
            if (awid < N) vx_rms_row_load(nrow, (const float *) (xb + (uint64_t) awid * a.nb11), a.K, lane);
            if (awid + NA < N) vx_rms_row_load(nrow2, (const float *) (xb + (uint64_t) (awid + NA) * a.nb11), a.K, lane);
            if (awid < N) load_gains(ngain);
        }
        if constexpr (NORM) { // a wave with several tokens takes two at a time
            if (awid < N) { // the first pair: its rows were requested up front
                if (awid + NA < N) {
                    float s1, s2;
                    vx_rms_row_scale2(nrow, nrow2, a.K, lane, a.norm_eps, s1, s2);
                    stage_row(awid, nrow, s1, ngain);
                    stage_row(awid + NA, nrow2, s2, ngain);
                } else {
                    stage_row(awid, nrow, vx_rms_row_scale(nrow, a.K, lane, a.norm_eps), ngain);
                }
            }
            for (int t = 2 * NW + awid; t < N; t += 2 * NA) norm_pair(t, NA); // (more than 2 NW tokens: four-wave work-groups only)
        } else {
#pragma unroll
            for (int i = 0; i < UB; ++i) {
                const int unit = atid + i * USTRIDE;
                if (unit < units) stage(unit, f0[i], f1[i]);
            }
            stage_rest(atid + UB * USTRIDE);
        }
    }
    __syncthreads();

    // ---- this wave's k blocks: kb = wid + NW * i, the LDS reads of four blocks issued together
    float4_t acc = {0, 0, 0, 0};
    {
        const char *     wcol = w_lds + min(c, R - 1) * a.w_slot; // lanes past the last column read a valid image; never stored
        const _Float16 * xrow = xs + (size_t) min(c, N - 1) * KP + 8 * j; // rows past the last token likewise
        const int per = (nkb + NW - 1) / NW;
        if (a.exact) { // uniform: every wave has a whole number of four-block rounds
            const char *     sp  = wcol + wid * VX_Q8_BLOCK;
            const _Float16 * xp  = xrow + wid * 32;
            const float *    xdp = xd + wid * 16 + 4 * j;
            if (wid & 1) {
                for (int i0 = 0; i0 < per; i0 += 4, sp += 4 * NW * VX_Q8_BLOCK, xp += 4 * NW * 32, xdp += 4 * NW * 16)
                    gv_round4<ACT_Q8, NW, true>(sp, j, xp, xdp, acc);
            } else {
                for (int i0 = 0; i0 < per; i0 += 4, sp += 4 * NW * VX_Q8_BLOCK, xp += 4 * NW * 32, xdp += 4 * NW * 16)
                    gv_round4<ACT_Q8, NW, false>(sp, j, xp, xdp, acc);
            }
        } else {
            constexpr int PB = 4;
            for (int i0 = 0; i0 < per; i0 += PB) {
                q8_raw   raw[PB];
                _Float16 dwh[PB];
                half8_t  aop[PB];
#pragma unroll
                for (int u = 0; u < PB; ++u) {
                    const int kb = min(wid + NW * (i0 + u), nkb - 1); // clamped: a valid address, the result unused
                    const char *     blk_p = wcol + kb * VX_Q8_BLOCK;
                    const uint32_t * q     = (const uint32_t *) (blk_p + 8 * j - ((kb & 1) ? 2 : 0)); // dword-aligned, as q8_load has it
                    raw[u] = q8_raw{ q[0], q[1], q[2] };
                    dwh[u] = *(const _Float16 *) blk_p;
                    aop[u] = *(const half8_t *) (xrow + kb * 32);
                }
#pragma unroll
                for (int u = 0; u < PB; ++u) {
                    const int kb = wid + NW * (i0 + u);
                    if (kb >= nkb) break; // wave-uniform
                    const float    dw  = (float) dwh[u];
                    const half8_t  bop = q8_unpack(raw[u], kb, true);
                    const float4_t blk = mfma16(aop[u], bop, float4_t{0, 0, 0, 0});
                    if constexpr (ACT_Q8) {
#pragma unroll
                        for (int r = 0; r < 4; ++r) acc[r] += blk[r] * (dw * (4 * j + r < N ? xd[kb * 16 + 4 * j + r] : 0.0f));
                    } else {
                        acc += blk * dw;
                    }
                }
            }
        }
    }

    // ---- the waves' partial sums, added in wave order by wave 0, which also finishes and stores
    int          row, pair;
    bool         row_ok;
    const char * wrow;
    column(c, row, pair, row_ok, wrow);
    __syncthreads(); // every wave is done with the staged activations: their place takes the partial sums
    if (wid > 0) red[(wid - 1) * 64 + lane] = acc;
    __syncthreads();
    if (wid > 0) return;
#pragma unroll
    for (int ww = 0; ww < NW - 1; ++ww) acc += red[ww * 64 + lane];
    // lane (j,c), register r: token 4j + r, row of column c
    if constexpr (dual) { // lane c < Rr holds W's row, lane c + Rr the same row of W2: dst = silu(gate) * up
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float up = __shfl(acc[r], lane + Rr, 64);
            acc[r] = (acc[r] / (1.0f + expf(-acc[r]))) * up;
        }
    }
    if constexpr (EPI == GV_RES) {
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] = scaled_residual(acc[r], a.res_scale, resv[r]);
    }
    if constexpr (SEG) {
        if (rope) { // column c < R/2 holds x0 of its pair, column c + R/2 the partner x1
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float2 cs = rcs[r * 64 + lane];
                const float other = __shfl_xor(acc[r], h2, 64);
                const bool  first = c < h2;
                float y0, y1;
                rope_rotate(first ? acc[r] : other, first ? other : acc[r], cs.x, cs.y, y0, y1);
                acc[r] = first ? y0 : y1;
            }
        }
    }
    if (row_ok && c < Rr) {
        char * out = db + (uint64_t) tok0 * nb1 + (uint64_t) row * 4;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int tok = 4 * j + r;
            if (tok < N) *(float *) (out + (uint64_t) tok * nb1) = acc[r];
        }
    }
}


constexpr size_t GV_MAX_LDS  = 160 * 1024;    // what a gfx950 CU has
constexpr size_t GV_ROPE_LDS = 4 * 64 * 8;     // cos / sin of four token slots per lane, exchanged between waves

// Shapes the streaming kernel takes: up to 16 tokens always; more (in chunks of 16, the chunks re-reading
// the weight rows from L2) while tokens x rows stays small -- measured against the tiled kernels: 1024 rows win up
// to 448 tokens, 4096 rows up to 64.  VX_GEMV_MAX_TOKENS=16 restores the 16-token limit.
bool gemv_shape_ok(int64_t N, int64_t rows, int64_t K) {
    static const int64_t max_tokens = [] { const char * e = getenv("VX_GEMV_MAX_TOKENS"); const int n = e ? atoi(e) : 0; return n >= 16 ? (int64_t) n : (int64_t) 1 << 30; }();
    if (K % 32 || K < 32 || N < 1) return false;
    static const int64_t max_work = [] { const char * e = getenv("VX_GEMV_MAX_WORK"); const long n = e ? atol(e) : 0; return n > 0 ? (int64_t) n : (int64_t) 256 * 1024; }();
    // (up to 1024 rows the tiled kernels' 64-token tiles are under a work-group per compute unit until some 500 tokens, 14 to
    // 15 us whatever the count: the chunks win up to 448 tokens -- 9.2 us at 256, 11.2 at 384)
    static const bool wide = getenv("VX_GEMV_MAX_WORK") == nullptr;
    if (N > 16 && (N > max_tokens || (N * rows > max_work && !(wide && rows <= 1024 && N <= 448)))) return false;
    // chunks of 16 tokens each stage 16 x K activations: with a long K a work-group fills a CU's LDS alone and the chunks
    // queue up behind each other (1024 rows x K = 4096 at 112 tokens: 63 us against 26 us on the tiled kernel with its K cut)
    if (N > 16 && K > 2048) return false;
    const size_t nl = (size_t) (N < 16 ? N : 16);
    return nl * K * 2 + nl * (K / 32) * 4 + 15 * 64 * 16 + 16 * sizeof(float) + GV_ROPE_LDS <= GV_MAX_LDS;
}

size_t gemv_smem(const mm_args & a, bool act_q8, int nw, bool dma = false) {
    const size_t nl = (size_t) (a.N < 16 ? a.N : 16);
    const size_t act = nl * (a.K + (dma ? 8 : 0)) * 2 + (act_q8 ? (dma ? 16 : nl) * (a.K / 32) * 4 : 0), red = (size_t) (nw > 1 ? nw - 1 : 0) * 64 * 16;
    // (gemv_dma_kernel puts the partial sums where the activations were)
    return (dma ? (act > red ? act : red) : act + red) + 16 * sizeof(float) + (a.nseg > 0 ? GV_ROPE_LDS : 0);
}

// gemv_dma_kernel's weight image: bytes between consecutive columns.  The padding is chosen so that the dword reads of the
// sixteen columns (lane (j, c): dword c * slot / 4 + 2 j + const) spread over the 64 banks as evenly as they can.
int gemv_dma_slot(int64_t K) {
    const int row_bytes = (int) (K / 32) * VX_Q8_BLOCK;
    int best_pad = 16, best = 1 << 30;
    for (int pad = 16; pad <= 256; pad += 16) {
        const int sd = (row_bytes + pad) / 4;
        int worst = 0;
        for (int half = 0; half < 2; ++half) { // 32 lanes at a time
            int count[64] = {0};
            for (int l = 32 * half; l < 32 * half + 32; ++l) {
                const int n = ++count[((l & 15) * sd + 2 * (l >> 4)) & 63];
                worst = n > worst ? n : worst;
            }
        }
        if (worst < best) { best = worst; best_pad = pad; }
    }
    return row_bytes + best_pad;
}

// Everything gemv_dma_kernel asks of a call except room in LDS
bool gemv_dma_takes(const mm_args & a, int nbatch, int nw) {
    const char * env = getenv("VX_GEMV_DMA"); // read on every call; 0 keeps the weights on the register path of gemv_kernel
    if ((env && atoi(env) == 0) || nbatch != 1 || (nw != 4 && nw != 8 && nw != 16) || !a.x_aligned || !a.w_aligned || a.K % 256) return false;
    if (a.norm_w && a.K > 2048) return false;
    if (a.w2 && a.res) return false;
    if (a.nseg > 0 && (a.w2 || a.res)) return false;
    if (a.res && a.norm_w) return false;
    auto al16 = [](const void * p_, uint64_t stride) { return (uintptr_t) p_ % 16 == 0 && stride % 16 == 0; };
    if (a.nseg == 0 && (!al16(a.w, a.nb01) || (a.w2 && !al16(a.w2, 0)))) return false;
    for (int i = 0; i < a.nseg; ++i) if (!al16(a.seg[i].w, a.seg[i].nb01)) return false;
    return true;
}
size_t gemv_dma_lds(const mm_args & a, bool act_q8, int nw, int rows_wg) {
    return (gemv_smem(a, act_q8, nw, true) + 15) / 16 * 16 + (size_t) rows_wg * gemv_dma_slot(a.K);
}

// Launches gemv_dma_kernel if the call is one it takes (a: as launch_gemv has prepared it, rows_wg and the prologue
// helpers included; nw: the wave count every kernel uses for this shape).
template <bool ACT_Q8>
bool launch_gemv_dma(mm_args & a, int nbatch, int nw, dim3 grid, hipStream_t st) {
    if (!gemv_dma_takes(a, nbatch, nw)) return false;
    a.w_slot    = gemv_dma_slot(a.K);
    a.w_lds_off = (int) ((gemv_smem(a, ACT_Q8, nw, true) + 15) / 16 * 16);
    const size_t smem = (size_t) a.w_lds_off + (size_t) a.rows_wg * a.w_slot;
    if (smem > GV_MAX_LDS) return false;
    a.exact = (a.K / 32) % (4 * nw) == 0; // whole four-block rounds for every wave
    const dim3 block((unsigned) (64 * nw));
#define VX_DMA_GO(NW_, SEG_, NORM_, EPI_)                                                                              \
    do {                                                                                                               \
        auto kern = many ? gemv_dma_kernel<ACT_Q8, NW_, SEG_, NORM_, EPI_, true>                                       \
                         : gemv_dma_kernel<ACT_Q8, NW_, SEG_, NORM_, EPI_, false>;                                     \
        if (smem > 64 * 1024) { /* above 64 KiB of LDS a kernel has to be told once that it may be given that much */  \
            static bool raised[2] = { false, false };                                                                  \
            if (!raised[many]) {                                                                                       \
                if (hipFuncSetAttribute((const void *) kern, hipFuncAttributeMaxDynamicSharedMemorySize,               \
                                        (int) GV_MAX_LDS) != hipSuccess) { (void) hipGetLastError(); return false; }   \
                raised[many] = true;                                                                                   \
            }                                                                                                          \
        }                                                                                                              \
        vx_launch(kern, grid, block, smem, st, a);                                                                            \
        return true;                                                                                                   \
    } while (0)
#define VX_DMA_NW(SEG_, NORM_, EPI_)                                                                                   \
    do { if (nw == 4) VX_DMA_GO(4, SEG_, NORM_, EPI_); else if (nw == 8) VX_DMA_GO(8, SEG_, NORM_, EPI_); else VX_DMA_GO(16, SEG_, NORM_, EPI_); } while (0)
    const bool norm = a.norm_w != nullptr;
    const bool many = (a.N < 16 ? a.N : 16) * (a.K / 8) > 64 * (nw - nw / 2); // an activation thread stages more than one unit
    if (a.nseg > 0) { if (norm) VX_DMA_NW(true, true, GV_PLAIN); else VX_DMA_NW(true, false, GV_PLAIN); }
    if (a.w2)       { if (norm) VX_DMA_NW(false, true, GV_SWIGLU); else VX_DMA_NW(false, false, GV_SWIGLU); }
    if (a.res)      { if (norm) return false; VX_DMA_NW(false, false, GV_RES); }
    if (norm) VX_DMA_NW(false, true, GV_PLAIN);
    VX_DMA_NW(false, false, GV_PLAIN);
#undef VX_DMA_NW
#undef VX_DMA_GO
    return false;
}

// waves per work-group for a matrix of M rows: about 4 blocks per wave for one chunk of tokens (K = 1024: 8 waves; measured
// against 8 blocks per wave: decode step 1.03 -> 0.96 ms), 8 when chunks of 16 tokens multiply the work-groups; either way
// every load is issued up front.  More
// than a handful of tokens: the activations' work (staging, a fused RMS_NORM's wave-per-token sums in fp64, the rotation's
// angles) outweighs the K walk and a matrix of few rows spreads it over 16 waves (norm + q/k/v + rope at 14 tokens: 12.8 ->
// 9.8 us); a tall matrix already fills the CUs with work-groups and is slower with more waves (4096 x 2 rows: 9.3 -> 13.5 us
// with 8).  The count -- and with it the order in which a product's K blocks are summed -- depends on K, on all tokens of the
// call and on M, never on what is fused to the product.
int gemv_waves_for(int64_t K, int64_t tokens, int64_t M) {
    const int64_t nkb = K / 32;
    int nw = 1;
    const int bpw = tokens <= 16 ? 4 : GV_UNROLL; // blocks per wave aimed at
    while (nw < 16 && nkb > (int64_t) nw * bpw) nw *= 2;
    static const int many = [] { const char * e = getenv("VX_GEMV_MANY_TOKENS"); return e ? atoi(e) : 5; }();
    // (one chunk of tokens only: with several, 16-wave work-groups take a CU each and queue up -- since the waves that fetch
    // the weights share the tokens' work, the 4 waves of the rule above are faster there, several work-groups to a CU:
    // 8 concurrent CFM solves 3.03 ms with 16 waves, 2.95 with 8, 2.90 with 4)
    if (tokens >= many && tokens <= 16 && nkb >= 16 && M <= 2048) nw = 16;
    return nw;
}

// A launch over several matrices (the q / k / v segments, the gate / up pair) has one wave count: every matrix must get the
// count it would get in a launch of its own.  -1 when they disagree: such a shape is left to the separate launches.
int gemv_waves(const mm_args & a, int nbatch) {
    const int64_t tokens = a.N * nbatch;
    if (a.nseg == 0) return gemv_waves_for(a.K, tokens, a.M);
    const int nw = gemv_waves_for(a.K, tokens, a.seg[0].M);
    for (int i = 1; i < a.nseg; ++i) if (gemv_waves_for(a.K, tokens, a.seg[i].M) != nw) return -1;
    return nw;
}

template <int WT, bool ACT_Q8>
bool launch_gemv(const mm_args & a0, int nbatch, hipStream_t st) {
    mm_args a = a0;
    {
        // (several matrices in one launch: wherever each of them alone is this kernel's shape -- the launch then sums every
        // product as its own call would)
        if (a.nseg > 0) { for (int i = 0; i < a.nseg; ++i) if (!gemv_shape_ok(a.N, a.seg[i].M, a.K)) return false; }
        else if (!gemv_shape_ok(a.N, a.w2 ? 2 * a.M : a.M, a.K)) return false;
    }
    if (a.M >= ((int64_t) 1 << 31) || a.K >= ((int64_t) 1 << 31)) return false;
    a.rows_wg = 16;
    a.nbatch  = nbatch;
    a.inv_upr = 1.0f / (float) (a.K / 8);
    {
        const int half = a.head_dim / 2;
        a.half_shift = -1;
        if (half > 0 && (half & (half - 1)) == 0) { a.half_shift = 0; while ((1 << a.half_shift) < half) ++a.half_shift; }
    }
    const int split = a.w2 ? 2 : 1; // with two matrices a work-group's MFMA columns hold half as many output rows
    auto groups = [&](int rows_wg) { // work-groups per batch entry
        if (a.nseg == 0) return (a.M * split + rows_wg - 1) / rows_wg;
        int64_t n = 0;
        for (int i = 0; i < a.nseg; ++i) n += (a.seg[i].M + rows_wg - 1) / rows_wg;
        return n;
    };
    const int64_t nchunk = (a.N + 15) / 16;
    while (a.rows_wg > 4 && groups(a.rows_wg) * nbatch * nchunk < 128) a.rows_wg /= 2;
    const int nw = gemv_waves(a, nbatch);
    if (nw < 0) return false;
    const size_t smem = gemv_smem(a, ACT_Q8, nw);
    if (smem > GV_MAX_LDS) return false;
    if constexpr (WT == WT_Q8) { // the kernel that keeps a work-group's rows in LDS: fewer rows each when they would not fit
        if (gemv_dma_takes(a, nbatch, nw))
            while (a.rows_wg > 4 && gemv_dma_lds(a, ACT_Q8, nw, a.rows_wg) > GV_MAX_LDS) a.rows_wg /= 2;
    }
    int64_t nwg = groups(a.rows_wg);
    if (a.nseg > 0) {
        int wg0 = 0;
        for (int i = 0; i < a.nseg; ++i) { a.seg[i].wg0 = wg0; wg0 += (int) ((a.seg[i].M + a.rows_wg - 1) / a.rows_wg); }
    }
    const dim3 grid((unsigned) nwg, (unsigned) nchunk, (unsigned) nbatch);
    const dim3 block((unsigned) (64 * nw));
    if constexpr (WT == WT_Q8) { if (launch_gemv_dma<ACT_Q8>(a, nbatch, nw, grid, st)) return true; }
    // above 64 KiB of LDS a kernel has to be told once that it may be given that much
#define VX_GEMV_GO(...)                                                                                                \
    do {                                                                                                               \
        if (smem > 64 * 1024) {                                                                                        \
            static bool raised = false;                                                                                \
            if (!raised) {                                                                                             \
                if (hipFuncSetAttribute((const void *) __VA_ARGS__, hipFuncAttributeMaxDynamicSharedMemorySize,        \
                                        (int) GV_MAX_LDS) != hipSuccess) { (void) hipGetLastError(); return false; }   \
                raised = true;                                                                                         \
            }                                                                                                          \
        }                                                                                                              \
        vx_launch(__VA_ARGS__, grid, block, smem, st, a);                                                                     \
    } while (0)
#define VX_GEMV(NW_)                                                                                                   \
    do {                                                                                                               \
        if (a.nseg > 0) {                                                                                              \
            if (WT == WT_Q8 && a.w_aligned && few) VX_GEMV_GO(gemv_kernel<WT, ACT_Q8, NW_, true, true, 4>);            \
            else if (WT == WT_Q8 && a.w_aligned)   VX_GEMV_GO(gemv_kernel<WT, ACT_Q8, NW_, true, true>);               \
            else                            VX_GEMV_GO(gemv_kernel<WT, ACT_Q8, NW_, false, true>);                     \
        } else {                                                                                                       \
            if (WT == WT_Q8 && a.w_aligned && few) VX_GEMV_GO(gemv_kernel<WT, ACT_Q8, NW_, true, false, 4>);           \
            else if (WT == WT_Q8 && a.w_aligned)   VX_GEMV_GO(gemv_kernel<WT, ACT_Q8, NW_, true, false>);              \
            else                            VX_GEMV_GO(gemv_kernel<WT, ACT_Q8, NW_, false, false>);                    \
        }                                                                                                              \
    } while (0)
    // a wave with at most four blocks requests four: the loads past a wave's last block are clamped re-reads of it
    const bool few = (a.K / 32 + nw - 1) / nw <= 4;
    a.exact = (a.K / 32) % ((int64_t) nw * (few ? 4 : GV_UNROLL)) == 0;
    switch (nw) {
        case 1:  VX_GEMV(1); break;
        case 2:  VX_GEMV(2); break;
        case 4:  VX_GEMV(4); break;
        case 8:  VX_GEMV(8); break;
        default: VX_GEMV(16); break;
    }
#undef VX_GEMV
#undef VX_GEMV_GO
    return true;
}


// ---- GEMM shape: many tokens (prefill) --------------------------------------------------------------
// A work-group of 4 waves (2 x 2) owns 128 weight rows x 128 tokens, each wave 64 x 64 as 4 x 4 MFMA
// tiles, so an operand fetched from LDS (activations) or dequantised in registers (weights) feeds four
// MFMAs.  K is walked in rounds of GM_KC blocks.  Both streams are software-pipelined: the raw Q8_0
// bytes of round r+1 are requested right after round r's have been turned into operands, and the
// activations of round r+1 are requested before round r's MFMAs and converted into the other LDS
// buffer after them -- one barrier per round, no load waits in front of the matrix work.
constexpr int GM_KC = 2;

template <int WT, bool ACT_Q8, bool AL4>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void gemm128_kernel(const mm_args a) {
    constexpr int TT = 8; // 16-token tiles per work-group
    __shared__ half8_t xs[2][GM_KC * TT * 64];
    __shared__ float   xd[2][ACT_Q8 ? GM_KC * TT * 16 : 1];

    const int tid = threadIdx.x, wid = tid >> 6, lane = tid & 63;
    const int j = lane >> 4, c = lane & 15;
    const int wr = wid >> 1, wt = wid & 1;

    const int     batch = blockIdx.z;
    const int     i12 = batch % a.ne12, i13 = batch / a.ne12;
    const char *  wb  = a.w + (uint64_t) (i12 / a.r2) * a.nb02 + (uint64_t) (i13 / a.r3) * a.nb03;
    const char *  xb  = a.x + (uint64_t) i12 * a.nb12 + (uint64_t) i13 * a.nb13;
    char *        db  = a.dst + (uint64_t) i12 * a.nb2 + (uint64_t) i13 * a.nb3;

    // Tile order.  Work-groups are dealt to the 8 XCDs round-robin and each XCD has its own L2, so the
    // token tiles are partitioned over the XCDs (tile ty goes to XCD ty % 8) and inside an XCD the row
    // tiles of one token tile run side by side: its activations are fetched into that L2 once, and the
    // weights stream through it once per couple of token tiles instead of once per work-group.
    // (with fewer than 8 token tiles the row tiles are dealt over the XCDs instead: no XCD without work)
    const int64_t gx = (a.M + 127) / 128, gy = (a.N + 127) / 128;
    const int64_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    int64_t ty, tx;
    if (gy >= 8) { ty = (slot / gx) * 8 + xcd; tx = slot % gx; }
    else         { ty = slot % gy; tx = (slot / gy) * 8 + xcd; }
    if (ty >= gy || tx >= gx) return; // padding of the last group of 8 tiles (whole work-group)
    const int64_t tok0 = ty * 128;
    const int64_t row0 = tx * 128 + wr * 64;
    // addresses are (uniform base + uniform round offset) + a 32-bit lane offset that never changes, so the
    // loads take a scalar base and no per-load vector address arithmetic (the launcher checks the ranges)
    uint32_t woff[4];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) woff[rt] = (uint32_t) (min(row0 + 16 * rt + c, a.M - 1) * a.nb01);
    constexpr bool al4 = AL4;
    const int64_t nkb = a.K / 32, nround = (nkb + GM_KC - 1) / GM_KC;
    constexpr int WBLK = WT == WT_Q8 ? VX_Q8_BLOCK : 64; // bytes of one 32-wide block of a row

    // ---- weight stream: raw bytes of one round
    q8_raw   wq[GM_KC][4];
    _Float16 wdv[GM_KC][4];
    half8_t  wh[GM_KC][4];
    auto load_weights = [&](int64_t round) {
#pragma unroll
        for (int kbl = 0; kbl < GM_KC; ++kbl) {
            const int64_t kb = min(round * GM_KC + kbl, nkb - 1); // clamped: a valid address, result unused
            const char * wk = wb + (uint64_t) kb * WBLK;          // uniform
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                if constexpr (WT == WT_Q8) {
                    wdv[kbl][rt] = *(const _Float16 *) (wk + woff[rt]);
                    if constexpr (AL4) {
                        const bool odd = (kb & 1) != 0; // uniform
                        const char * p = (const char *) __builtin_assume_aligned(wk + (odd ? -2 : 0) + (woff[rt] + 8u * (uint32_t) j), 4);
                        uint32_t v[3];
                        __builtin_memcpy(v, p, 12);
                        wq[kbl][rt] = q8_raw{v[0], v[1], v[2]};
                    } else {
                        wq[kbl][rt] = q8_load(wk + woff[rt], 0, j, false);
                    }
                } else {
                    __builtin_memcpy(&wh[kbl][rt], wk + (woff[rt] + 16u * (uint32_t) j), 16);
                }
            }
        }
    };
    // ---- activation stream: a thread moves 4 units (8 consecutive k of one token) per round
    float4_t xr[4][2];
    uint32_t xoff[4];
#pragma unroll
    for (int it = 0; it < 4; ++it) {
        const int unit = tid + 256 * it;
        xoff[it] = (uint32_t) ((uint64_t) (unit >> 3) * a.nb11 + (uint64_t) (unit & 7) * 32);
    }
    const char * xtile = xb + (uint64_t) tok0 * a.nb11; // uniform
    auto load_acts = [&](int64_t round) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int unit = tid + 256 * it;
            const int t = unit >> 3, u = unit & 7;
            const int64_t tok = tok0 + t, k = (round * GM_KC) * 32 + u * 8;
            xr[it][0] = float4_t{0, 0, 0, 0}; xr[it][1] = float4_t{0, 0, 0, 0};
            if (tok < a.N && k < a.K) {
                const float * xp = (const float *) (xtile + (uint64_t) round * (GM_KC * 32 * 4) + xoff[it]);
                if (a.x_aligned) { xr[it][0] = ((const float4_t *) xp)[0]; xr[it][1] = ((const float4_t *) xp)[1]; }
                else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) { xr[it][0][i] = xp[i]; xr[it][1][i] = xp[4 + i]; }
                }
            }
        }
    };
    auto store_acts = [&](int buf) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int unit = tid + 256 * it;
            const int t = unit >> 3, u = unit & 7, kbl = u >> 2, uj = u & 3;
            float v[8];
#pragma unroll
            for (int i = 0; i < 4; ++i) { v[i] = xr[it][0][i]; v[4 + i] = xr[it][1][i]; }
            half8_t h;
            if constexpr (ACT_Q8) {
                float amax = 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) amax = fmaxf(amax, fabsf(v[i]));
                amax = fmaxf(amax, __shfl_xor(amax, 1, 64));
                amax = fmaxf(amax, __shfl_xor(amax, 2, 64));
                const float d  = amax / 127.f;
                const float id = amax != 0.0f ? 127.f / amax : 0.0f;
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = (_Float16) rintf(v[i] * id);
                if (uj == 0) xd[buf][(kbl * TT + (t >> 4)) * 16 + (t & 15)] = (float) (_Float16) d;
            } else {
#pragma unroll
                for (int i = 0; i < 8; ++i) h[i] = (_Float16) v[i];
            }
            xs[buf][lds_slot(kbl, t >> 4, TT, uj, t & 15)] = h;
        }
    };

    float4_t acc[4][4]; // [row tile][token tile]
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) acc[rt][tt] = float4_t{0, 0, 0, 0};

    load_weights(0);
    load_acts(0);
    store_acts(0);
    __syncthreads();

    for (int64_t round = 0; round < nround; ++round) {
        const int buf = (int) (round & 1);
        // this round's weights become operands; their registers take the next round's bytes
        half8_t bop[GM_KC][4];
        float   dw[GM_KC][4];
#pragma unroll
        for (int kbl = 0; kbl < GM_KC; ++kbl)
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                if constexpr (WT == WT_Q8) {
                    bop[kbl][rt] = q8_unpack(wq[kbl][rt], min(round * GM_KC + kbl, nkb - 1), al4);
                    dw[kbl][rt]  = (float) wdv[kbl][rt];
                } else {
                    bop[kbl][rt] = wh[kbl][rt];
                    dw[kbl][rt]  = 1.0f;
                }
            }
        const bool more = round + 1 < nround; // uniform
        if (more) { load_weights(round + 1); load_acts(round + 1); }

#pragma unroll
        for (int kbl = 0; kbl < GM_KC; ++kbl) {
            if (round * GM_KC + kbl >= nkb) break; // uniform: K holds an odd number of blocks
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
                const half8_t aop = xs[buf][lds_slot(kbl, wt * 4 + tt, TT, j, c)];
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) {
                    if constexpr (WT == WT_Q8) {
                        const float4_t blk = mfma16(aop, bop[kbl][rt], float4_t{0, 0, 0, 0});
                        if constexpr (ACT_Q8) {
#pragma unroll
                            for (int r = 0; r < 4; ++r) acc[rt][tt][r] += blk[r] * (dw[kbl][rt] * xd[buf][(kbl * TT + wt * 4 + tt) * 16 + 4 * j + r]);
                        } else {
                            acc[rt][tt] += blk * dw[kbl][rt];
                        }
                    } else {
                        acc[rt][tt] = mfma16(aop, bop[kbl][rt], acc[rt][tt]);
                    }
                }
            }
        }
        if (more) store_acts(buf ^ 1);
        __syncthreads();
    }

    // lane (j,c), tile (rt, tt), register r: token tok0 + 64 wt + 16 tt + 4j + r, row row0 + 16 rt + c
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const int64_t row = row0 + 16 * rt + c;
        if (row >= a.M) continue;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t tok = tok0 + 64 * wt + 16 * tt + 4 * j + r;
                if (tok < a.N) *(float *) (db + (uint64_t) tok * a.nb1 + (uint64_t) row * 4) = acc[rt][tt][r];
            }
    }
}

template <int WT, bool ACT_Q8>
bool launch_gemm128(const mm_args & a, int nbatch, hipStream_t st) {
    if (WT == WT_F32 || a.K % 32 || a.K < 32 || a.N < 128) return false;
    const int64_t gx = (a.M + 127) / 128, gy = (a.N + 127) / 128;
    if (gx * gy * nbatch < 192) return false; // small problems spread wider on the 64 x 64 tiles
    const int64_t blocks = gy >= 8 ? gx * ((gy + 7) / 8) * 8 : ((gx + 7) / 8) * 8 * gy; // (the kernel's two ways of dealing tiles to XCDs)
    if (blocks > 0x7fffffff) return false;
    // 32-bit lane offsets inside the kernel: rows of the weight matrix and the 128 tokens of a tile
    if ((uint64_t) a.M * a.nb01 >= (1ull << 32) || (uint64_t) 128 * a.nb11 + 256 >= (1ull << 32)) return false;
    const dim3 grid((unsigned) blocks, 1, (unsigned) nbatch);
    if (WT == WT_Q8 && a.w_aligned) vx_launch(gemm128_kernel<WT, ACT_Q8, true>, grid, dim3(256), 0, st, a);
    else                            vx_launch(gemm128_kernel<WT, ACT_Q8, false>, grid, dim3(256), 0, st, a);
    return true;
}

// ---- GEMM shape, both operands through LDS -----------------------------------------------------------
// Fetching the weights straight into the MFMA layout, as the kernels above do, makes every 16-lane group of a
// load touch 16 different rows, i.e. 16 cache lines for 12 useful bytes each, and the per-CU vector cache, which
// serves about one line per cycle, becomes the limit of the whole kernel.  Here a thread fetches (row, block,
// 8-quant group) units in row-major lane order, so that 16 lanes cover four 32-byte runs, turns its quants into
// f16 once for the work-group, and parks them in LDS in the operand layout; activations are fetched 256
// contiguous bytes per 16 lanes.  One barrier per round of GL_KC blocks; the global loads run two rounds ahead.
constexpr int    GL_KC   = 2;
// LDS of a work-group that owns 16 TR rows x 16 TC tokens: both operands double-buffered, and the block scales
constexpr size_t gl_lds(int TR, int TC) { return 2 * GL_KC * (TR + TC) * 64 * sizeof(half8_t) + 2 * GL_KC * 16 * TR * sizeof(float); }

// FOLD: the block scale is multiplied into the f16 weights as they are parked (q * d rounded to f16, relative
// error 2^-12 on average -- the size of the activations' own rounding) and the MFMAs accumulate across blocks;
// otherwise the weights stay the exact integers and each 32-wide partial product is scaled in fp32.
// A wave owns RT x CT MFMA tiles (16 rows x 16 tokens each), the work-group WR x WC waves.
// DUAL: two matrices of one layout (mlp_forward's gate and up, src/minicpm.cpp:724-731) and dst = silu(W x) * (W2 x), the
// GLU node's arithmetic.  The work-group's 16-row tiles alternate between the matrices -- tile 2p holds rows
// 16p .. 16p + 15 of W, tile 2p + 1 the same rows of W2 -- so that a wave (an even number of row tiles) holds both halves
// of every value it stores, and a wave's weight units (its index picks the tile's parity) come from one matrix only.
template <int WT, bool FOLD, int RT, int CT, int WR, int WC, bool DUAL = false>
__global__ __launch_bounds__(64 * WR * WC) __attribute__((amdgpu_waves_per_eu(RT * CT >= 16 ? 2 : 4))) void gemm_lds_kernel(const mm_args a) {
    static_assert(!DUAL || (RT % 2 == 0 && (WR * WC) % 2 == 0), "pairs of row tiles inside a wave, a matrix per wave parity");
    static_assert(GL_KC == 2, "the parity of a block inside a round is its index in the round");
    constexpr int  TR = WR * RT, TC = WC * CT; // 16-wide tiles per work-group: rows, tokens
    constexpr int  NT = 64 * WR * WC;          // threads
    constexpr int  WU = 16 * TR * 8 / NT, XU = 16 * TC * 16 / NT; // weight / activation units per thread and round
    static_assert(WU * NT == 16 * TR * 8 && XU * NT == 16 * TC * 16 && NT % 256 == 0 && WU % 2 == 0, "units divide evenly over the threads");
    constexpr int  ROWS = 16 * TR, TOKS = 16 * TC;
    constexpr bool POST = WT == WT_Q8 && !FOLD; // scale after the MFMA
    extern __shared__ __align__(16) char gl_smem[];
    constexpr int XOPS = GL_KC * TC * 64, WOPS = GL_KC * TR * 64;
    half8_t * xs = (half8_t *) gl_smem;                       // [2][XOPS] activations
    half8_t * ws = xs + 2 * XOPS;                             // [2][WOPS] weights
    float *   wd = (float *) (ws + 2 * WOPS);                 // [2][GL_KC * ROWS] block scales

    const int tid = threadIdx.x, wid = tid >> 6, lane = tid & 63;
    const int j = lane >> 4, c = lane & 15;
    const int wr = wid / WC, wt = wid % WC;

    // a long K on a grid of few tiles is cut across nsplit work-groups (blockIdx.z = batch x split): each leaves its share
    // in its slab of the partial buffer, dense [token][row], for mm_splitk_reduce_kernel to add in split order
    // (only the 64 x 64 tile is launched with a cut K: the larger tile keeps its registers for the accumulators)
    constexpr bool CUT = RT * CT <= 4 && !DUAL;
    const int     nsplit = CUT && a.ksplit > 1 ? a.ksplit : 1; // uniform
    const int     batch = (int) blockIdx.z / nsplit, split = (int) blockIdx.z % nsplit;
    const int     i12 = batch % a.ne12, i13 = batch / a.ne12;
    // (DUAL: odd waves fetch the second matrix -- unit idx of a thread lies in row tile idx / 64 = wave + waves * (it / 2))
    const char *  wsel = DUAL && (wid & 1) ? a.w2 : a.w; // uniform per wave
    const char *  wb  = wsel + (uint64_t) (i12 / a.r2) * a.nb02 + (uint64_t) (i13 / a.r3) * a.nb03;
    const char *  xb  = a.x + (uint64_t) i12 * a.nb12 + (uint64_t) i13 * a.nb13;
    char *        db  = a.dst + (uint64_t) i12 * a.nb2 + (uint64_t) i13 * a.nb3;
    uint64_t      dnb1 = a.nb1;
    if (nsplit > 1) {
        db   = (char *) (a.partial + ((uint64_t) batch * nsplit + split) * (uint64_t) a.N * a.M);
        dnb1 = (uint64_t) a.M * 4;
    }

    // token tiles partitioned over the XCDs, row tiles of one token tile side by side (see gemm128_kernel).  With fewer
    // than 8 token tiles that would leave XCDs without work (112 tokens are 2 tiles: a quarter of the chip, and three empty
    // blocks dispatched for every working one): then the ROW tiles are dealt over the XCDs and a row tile's few token tiles
    // sit side by side on one, where they share the weight rows in its L2.
    // (32-bit and uniform: the larger tile has no register to spare)
    const int64_t  MV = DUAL ? 2 * a.M : a.M; // rows of the tiled (virtual) matrix
    const uint32_t gx = (uint32_t) ((MV + ROWS - 1) / ROWS), gy = (uint32_t) ((a.N + TOKS - 1) / TOKS);
    const uint32_t xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const bool     by_tokens = gy >= 8;
    const uint32_t inner = by_tokens ? gx : gy, q = slot / inner, rem = slot - q * inner;
    const uint32_t ty = by_tokens ? q * 8 + xcd : rem, tx = by_tokens ? rem : q * 8 + xcd;
    if (ty >= gy || tx >= gx) return;
    const int64_t tok0 = (int64_t) ty * TOKS;
    const int64_t rowg = (int64_t) tx * ROWS;
    // the launcher takes whole rounds only; a split may hold an odd number of them (a round's register set and LDS buffer
    // are the parity of its index within the split, and the loop below guards the second round of each pair)
    const int64_t rounds_all = a.K / (32 * GL_KC), rbeg = rounds_all / nsplit * split, nround = rbeg + rounds_all / nsplit;

    // Loads never leave the operands: rows past M and tokens past N are clamped to the last one (their
    // products are computed and dropped), so no load carries a predicate.  They are buffer loads: a uniform
    // base in a resource descriptor, a 32-bit lane offset that never changes and a scalar offset per round
    // (the launcher checks the ranges), so a load costs no address arithmetic.
    const __amdgpu_buffer_rsrc_t wres = __builtin_amdgcn_make_buffer_rsrc((void *) wb, 0, -1, 0x00020000);
    // ---- weight stream: unit = (row, block of the round, group of 8 k), WU per thread and round.  Unit `it` of a
    // thread belongs to block it & 1, so a block's parity -- where its quants sit in the dwords -- is known at compile time.
    constexpr int WUNIT = WT == WT_Q8 ? 3 : 4; // dwords fetched per unit
    uint32_t wraw[2][WU][WUNIT]; // two register sets: the rounds after next and next
    uint32_t woff[WU / 2];       // block 0 of the pair; block 1 is 32 bytes on (Q8_0: 34 - 2) or 64 (F16)
    uint32_t wslot[WU];          // where a unit goes in LDS: the same place every round
#pragma unroll
    for (int it = 0; it < WU; ++it) {
        const int idx = tid + NT * (it >> 1), kbl = it & 1;
        const int row = idx >> 2, uj = idx & 3;
        const uint32_t wrow   = DUAL ? (uint32_t) (rowg >> 1) + 16 * (row >> 5) + (row & 15) : (uint32_t) rowg + row; // the row of its own matrix
        const uint64_t rowoff = (uint64_t) min(wrow, (uint32_t) a.M - 1) * a.nb01;
        if (kbl == 0) woff[it >> 1] = (uint32_t) (rowoff + (WT == WT_Q8 ? 8 : 16) * uj);
        wslot[it] = (uint32_t) lds_slot(kbl, row >> 4, TR, uj, row & 15);
    }
    constexpr int WROUND = GL_KC * (WT == WT_Q8 ? VX_Q8_BLOCK : 64); // bytes of a row walked per round
    auto load_weights = [&](int64_t round, auto SET) {
        constexpr int S = decltype(SET)::value;
        const int so = (int) (round * WROUND); // uniform
#pragma unroll
        for (int it = 0; it < WU; ++it) {
            const uint32_t vo = woff[it >> 1] + (it & 1) * (WT == WT_Q8 ? 32 : 64);
            if constexpr (WT == WT_Q8) {
                typedef uint32_t u32x3 __attribute__((ext_vector_type(3)));
                const u32x3 v = __builtin_amdgcn_raw_buffer_load_b96(wres, (int) vo, so, 0);
                wraw[S][it][0] = v[0]; wraw[S][it][1] = v[1]; wraw[S][it][2] = v[2];
            } else {
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(wres, (int) vo, so, 0);
                wraw[S][it][0] = v[0]; wraw[S][it][1] = v[1]; wraw[S][it][2] = v[2]; wraw[S][it][3] = v[3];
            }
        }
    };
    auto store_weights = [&](int buf, auto SET) {
        constexpr int S = decltype(SET)::value;
#pragma unroll
        for (int it = 0; it < WU; ++it) {
            const int idx = tid + NT * (it >> 1), kbl = it & 1;
            const int row = idx >> 2, uj = idx & 3;
            half8_t h;
            if constexpr (WT == WT_Q8) {
                // an even block starts on a dword with its scale in front; the fetch of an odd block starts 2 bytes early
                h = q8_unpack(q8_raw{wraw[S][it][0], wraw[S][it][1], wraw[S][it][2]}, kbl, true);
                const uint32_t bits = kbl ? wraw[S][it][0] >> 16 : wraw[S][it][0] & 0xffffu; // the scale, in the unit with uj == 0
                if constexpr (FOLD) {
                    // the four units of a block sit in four neighbouring lanes: take the scale from the first
                    const uint32_t b0 = (uint32_t) __builtin_amdgcn_update_dpp(0, (int) bits, 0x00 /* quad_perm 0,0,0,0 */, 0xf, 0xf, true);
                    const _Float16 d = __builtin_bit_cast(_Float16, (uint16_t) b0);
#pragma unroll
                    for (int i = 0; i < 8; ++i) h[i] *= d;
                } else {
                    if (uj == 0) wd[(buf * GL_KC + kbl) * ROWS + row] = (float) __builtin_bit_cast(_Float16, (uint16_t) bits);
                }
            } else {
                typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
                h = __builtin_bit_cast(half8_t, u32x4{wraw[S][it][0], wraw[S][it][1], wraw[S][it][2], wraw[S][it][3]});
            }
            ws[buf * WOPS + wslot[it]] = h;
        }
    };
    // ---- activation stream: unit = (token, 16-byte piece of its 256 bytes of the round), XU per thread and round
    float4_t xr[2][XU];
    const int xchunk = tid & 15;
    uint32_t xoff[XU];
#pragma unroll
    for (int i = 0; i < XU; ++i) {
        const int64_t tok = min(tok0 + (tid >> 4) + (NT / 16) * i, a.N - 1);
        xoff[i] = (uint32_t) ((uint64_t) (tok - tok0) * a.nb11 + (uint64_t) xchunk * 16);
    }
    const __amdgpu_buffer_rsrc_t xres = __builtin_amdgcn_make_buffer_rsrc((void *) (xb + (uint64_t) tok0 * a.nb11), 0, -1, 0x00020000);
    auto load_acts = [&](int64_t round, auto SET) {
        constexpr int S = decltype(SET)::value;
        const int so = (int) (round * (GL_KC * 128)); // uniform
#pragma unroll
        for (int i = 0; i < XU; ++i) {
            xr[S][i] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(xres, (int) xoff[i], so, 0));
        }
    };
    // byte offset of token (tid >> 4)'s piece in LDS; unit i is NT / 16 tokens = NT / 256 tiles of 64 slots further on
    const uint32_t xslot = (uint32_t) lds_slot(xchunk >> 3, tid >> 8, TC, (xchunk & 7) >> 1, (tid >> 4) & 15) * 16 + 8 * (xchunk & 1);
    auto store_acts = [&](int buf, auto SET) {
        constexpr int S = decltype(SET)::value;
        typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
#pragma unroll
        for (int i = 0; i < XU; ++i) {
            half4_t h;
#pragma unroll
            for (int e = 0; e < 4; ++e) h[e] = (_Float16) xr[S][i][e];
            *(half4_t *) ((char *) (xs + buf * XOPS + 64 * (NT / 256) * i) + xslot) = h;
        }
    };

    float4_t acc[RT][CT]; // [row tile][token tile]
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int tt = 0; tt < CT; ++tt) acc[rt][tt] = float4_t{0, 0, 0, 0};

    // operand slots of this lane for the two blocks of a round (tile 0; a tile is 64 slots)
    const int ra0 = lds_slot(0, 0, TC, j, c), ra1 = lds_slot(1, 0, TC, j, c);
    const int rb0 = lds_slot(0, 0, TR, j, c), rb1 = lds_slot(1, 0, TR, j, c);
    auto multiply_block = [&](int buf, int kbl) {
        const int ra = buf * XOPS + (kbl ? ra1 : ra0), rb = buf * WOPS + (kbl ? rb1 : rb0);
        half8_t bop[RT];
        float   dw[RT];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
            bop[rt] = ws[rb + 64 * (wr * RT + rt)];
            dw[rt]  = POST ? wd[(buf * GL_KC + kbl) * ROWS + wr * (16 * RT) + 16 * rt + c] : 1.0f;
        }
#pragma unroll
        for (int tt = 0; tt < CT; ++tt) {
            const half8_t aop = xs[ra + 64 * (wt * CT + tt)];
#pragma unroll
            for (int rt = 0; rt < RT; ++rt) {
                if constexpr (POST) {
                    const float4_t blk = mfma16(aop, bop[rt], float4_t{0, 0, 0, 0});
                    acc[rt][tt] += blk * dw[rt];
                } else {
                    acc[rt][tt] = mfma16(aop, bop[rt], acc[rt][tt]);
                }
            }
            if constexpr (POST) __builtin_amdgcn_sched_barrier(0); // keeps the live partial products to one token tile's
        }
    };

    // Round r's operands are in LDS buffer r & 1 while round r+1 waits in register set (r+1) & 1 and round
    // r+2 is being fetched into set r & 1: a fetch has a whole round (MFMAs, conversion, barrier) and the next
    // round's MFMAs to arrive before it is converted.
    using set0 = std::integral_constant<int, 0>;
    using set1 = std::integral_constant<int, 1>;
    load_weights(rbeg, set0{});
    load_acts(rbeg, set0{});
    if (rbeg + 1 < nround) { load_weights(rbeg + 1, set1{}); load_acts(rbeg + 1, set1{}); }
    store_weights(0, set0{});
    store_acts(0, set0{});
    __syncthreads();

    auto one_round = [&](int64_t round, auto SET) { // SET = round & 1
        using other = std::integral_constant<int, 1 - decltype(SET)::value>;
        const int buf = decltype(SET)::value;
        if (round + 2 < nround) { load_weights(round + 2, SET); load_acts(round + 2, SET); }
        if constexpr (POST) {
#pragma unroll 1 // unrolled, the two blocks' operand fetches are hoisted together and the kernel spills
            for (int kbl = 0; kbl < GL_KC; ++kbl) multiply_block(buf, kbl);
        } else {
            multiply_block(buf, 0);
            multiply_block(buf, 1);
        }
        if (round + 1 < nround) { store_weights(buf ^ 1, other{}); store_acts(buf ^ 1, other{}); }
        __syncthreads();
    };
    for (int64_t round = rbeg; round < nround; round += 2) {
        one_round(round, set0{});
        if (round + 1 < nround) one_round(round + 1, set1{});
    }

    // lane (j,c), tile (rt, tt), register r: token tok0 + 16 (CT wt + tt) + 4j + r, row rowg + 16 (RT wr + rt) + c
    // A fused residual update (dst = res + scale * (W x), rounded as the SCALE and the ADD node would) is applied here
    // unless K is cut: then the kernel that adds the partials applies it.  The residual may be dst itself: an element is
    // read by the lane that writes it.
    if constexpr (DUAL) {
        // lane (j,c), tile pair (2p, 2p + 1), register r: dst row rowg / 2 + 16 (RT wr / 2 + p) + c of token ... + 4j + r
#pragma unroll
        for (int p2 = 0; p2 < RT / 2; ++p2) {
            const int64_t row = (rowg >> 1) + 16 * ((RT * wr) / 2 + p2) + c;
            if (row >= a.M) continue;
#pragma unroll
            for (int tt = 0; tt < CT; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t tok = tok0 + 16 * (CT * wt + tt) + 4 * j + r;
                    const float g = acc[2 * p2][tt][r], u = acc[2 * p2 + 1][tt][r];
                    if (tok < a.N) *(float *) (db + (uint64_t) tok * dnb1 + (uint64_t) row * 4) = (g / (1.0f + expf(-g))) * u;
                }
        }
        return;
    }
    const bool    residual = a.res != nullptr && nsplit == 1; // uniform
    const char *  rbase    = residual ? a.res + (uint64_t) i12 * a.rnb2 + (uint64_t) i13 * a.rnb3 : nullptr;
    if (tok0 + TOKS <= a.N && rowg + ROWS <= a.M) { // uniform: a tile inside the matrix stores without tests,
        // at a uniform base plus one 32-bit lane offset (the launcher checks the range)
        char * tb = db + (uint64_t) tok0 * dnb1 + (uint64_t) rowg * 4;
        const uint32_t loff = (uint32_t) ((uint64_t) (16 * CT * wt + 4 * j) * dnb1 + (uint64_t) (16 * RT * wr + c) * 4);
        if (residual) {
            const char *   rb    = rbase + (uint64_t) tok0 * a.rnb1 + (uint64_t) rowg * 4;
            const uint32_t rloff = (uint32_t) ((uint64_t) (16 * CT * wt + 4 * j) * a.rnb1 + (uint64_t) (16 * RT * wr + c) * 4);
#pragma unroll
            for (int tt = 0; tt < CT; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const char * rr = rb + (uint64_t) (16 * tt + r) * a.rnb1; // uniform
#pragma unroll
                    for (int rt = 0; rt < RT; ++rt) acc[rt][tt][r] = scaled_residual(acc[rt][tt][r], a.res_scale, *(const float *) (rr + 64 * rt + rloff));
                }
        }
#pragma unroll
        for (int tt = 0; tt < CT; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                char * tr = tb + (uint64_t) (16 * tt + r) * dnb1; // uniform
#pragma unroll
                for (int rt = 0; rt < RT; ++rt) *(float *) (tr + 64 * rt + loff) = acc[rt][tt][r];
            }
        return;
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
        const int64_t row = rowg + 16 * (RT * wr + rt) + c;
        if (row >= a.M) continue;
#pragma unroll
        for (int tt = 0; tt < CT; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t tok = tok0 + 16 * (CT * wt + tt) + 4 * j + r;
                if (tok >= a.N) continue;
                float v = acc[rt][tt][r];
                if (residual) v = scaled_residual(v, a.res_scale, *(const float *) (rbase + (uint64_t) tok * a.rnb1 + (uint64_t) row * 4));
                *(float *) (db + (uint64_t) tok * dnb1 + (uint64_t) row * 4) = v;
            }
    }
}

template <int WT, bool FOLD, int RT, int CT, int WR, int WC, bool DUAL = false>
bool launch_gemm_lds_tile(const mm_args & a, int nbatch, hipStream_t st) {
    constexpr size_t lds = gl_lds(RT * WR, CT * WC);
    const int64_t gx = ((DUAL ? 2 : 1) * a.M + 16 * RT * WR - 1) / (16 * RT * WR), gy = (a.N + 16 * CT * WC - 1) / (16 * CT * WC);
    const int64_t blocks = gy >= 8 ? gx * ((gy + 7) / 8) * 8 : ((gx + 7) / 8) * 8 * gy; // (the kernel's two ways of dealing tiles to XCDs)
    if (blocks > 0x7fffffff) return false;
    static bool raised = false;
    if (!raised && lds > 48 * 1024) {
        if (hipFuncSetAttribute((const void *) gemm_lds_kernel<WT, FOLD, RT, CT, WR, WC, DUAL>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds) != hipSuccess) {
            (void) hipGetLastError();
            return false;
        }
        raised = true;
    }
    const int nsplit = a.ksplit > 1 ? a.ksplit : 1;
    vx_launch(gemm_lds_kernel<WT, FOLD, RT, CT, WR, WC, DUAL>, dim3((unsigned) blocks, 1, (unsigned) (nbatch * nsplit)), dim3(64 * WR * WC), lds, st, a);
    return true;
}

// VX_GEMM_LDS: 0 = off (the register-operand kernels), 1 (default) = block scale applied in fp32 after each MFMA, so
// that a weight enters the sum as exactly q * d; 2 = scale folded into the f16 weights (q * d rounded once to f16,
// 10-22 % faster).  Read on every call: a product of this size takes tens of microseconds.
int gemm_lds_mode() { const char * e = getenv("VX_GEMM_LDS"); return e ? atoi(e) : 1; }

// The cut of K for a product of 64 x 64 tiles, from its shape alone (the groups that promise a single product's bits ask it
// too).  Fewer than 64 tiles (the down-projection of a hundred tokens: 32 tiles, 64 rounds): cut so that some 256
// work-groups walk 8 or more rounds each.  Up to 256 tiles -- one work-group or less to a compute unit, whose rounds then
// follow each other with nothing to hide a load behind -- and 32 or more rounds (the down-projection of a thousand tokens:
// 256 tiles, 64 rounds, 51 us): halves or quarters, so that several work-groups share a compute unit.
int gemm_lds_cut(int64_t M, int64_t N, int64_t K, int64_t nbatch) {
    if (((M + 127) / 128) * ((N + 127) / 128) * nbatch >= 192) return 1;
    const int64_t tiles64 = ((M + 63) / 64) * ((N + 63) / 64) * nbatch, rounds = K / (32 * GL_KC);
    int ks = 1;
    if (tiles64 < 64) {
        while (ks < 16 && tiles64 * ks < 192 && rounds % (4 * ks) == 0 && rounds / (2 * ks) >= 4) ks *= 2;
    } else if (tiles64 <= 256 && rounds >= 32) {
        // (measured on 24 layers at 2 x 512 tokens, K = 4096: whole 4.98 ms, halves 4.67, quarters 4.62; the same cut for the
        // 16 rounds of K = 1024 costs more in partials than it hides: 4.68)
        ks = rounds >= 64 && rounds % 4 == 0 ? 4 : (rounds % 2 == 0 ? 2 : 1);
    }
    return ks;
}

// A cut product whose workspace request fails (a growing request on a stream under capture, or no memory) must not
// quietly become another kernel's product with another summation order: the launcher records the status here, every
// launcher after it stands back, and the entry point returns the status (thread-local: launches come from any thread).
thread_local vx_status t_ws_status = VX_OK;
bool ws_failed() { return t_ws_status != VX_OK; }
vx_status take_ws_status() { const vx_status rc = t_ws_status; t_ws_status = VX_OK; return rc; }

// ---- Q8_0 weights x many tokens, both operands laid out for the matrix cores beforehand -----------------------------
// At prefill sizes every weight is used by hundreds of token tiles and every activation by dozens of row tiles; the
// kernel above converts each of them (int8 -> f16, f32 -> f16) once per tile that uses it, and that conversion work, not
// the matrix cores, bounds it.  Here two small passes convert once: the weights into exact f16 integers with their block
// scales apart, the activations into f16 (to nearest even, as the kernel above rounds them), both written as the 1 KB
// operand tiles of v_mfma_f32_16x16x32_f16 -- [k block][16-row tile][lane (j, c): row c, k 8j .. 8j + 7] -- so that the
// product kernel brings a tile into LDS with one direct load (global_load_lds_dwordx4, no register, no address
// arithmetic) and reads an operand with one conflict-free 16-byte LDS load.  The arithmetic is the kernel above's: a 32-wide
// partial product per block from one MFMA, scaled by the block's d in fp32 and added -- the same bits.
//
// Work-group: 8 waves, 256 rows x 128 tokens (a wave: 64 x 64 = 4 x 4 MFMA tiles), two stages of one k block
// (16 KB of weights, 8 KB of activations, 1 KB of scales; a third stage measured 5 % slower), one barrier a block, two
// work-groups to a compute unit (50 KB of LDS and 128 registers each): everything a wave does besides its MFMAs -- issuing the direct loads (a hundred
// cycles apiece), the barrier, the operand reads, the 64 scaled additions of a block, the stores at the end -- was
// measured to add up unhidden with one work-group's waves in step; the second work-group's waves fill those gaps.
// The weights are the MFMA's column operand: lane c holds row c of every row tile and needs one scale per tile, which the
// weight pass lays out so that a lane's four come with one 16-byte LDS load.
// Work-groups are dealt to the XCDs in groups of 4 row tiles x 8 token tiles that run side by side on one XCD's 32
// compute units and share its L2.
// Measured on 4096 rows x K 1024 x 16384 tokens: 205 us with both passes (11 and 21 us) against 300 us for the kernel
// above; the kernel alone 167 us.  Per compute unit and block (two work-groups, 16 waves) that is 2600 cycles against
// 1024 of MFMAs and 1216 of scaled additions per SIMD (which do run side by side), 600 of LDS reads and some 1100 to
// bring 50 KB in from L2: no single unit bounds it; what is left is the waves of a work-group meeting at a barrier every
// block and the issue of the direct loads (a fifth of the time when they are taken out).
constexpr int QT_ROWS = 256, QT_TOKS = 128, QT_STAGES = 2;
constexpr int QT_STAGE_BYTES = (QT_ROWS + QT_TOKS) / 16 * 1024 + QT_ROWS * 4;
constexpr size_t QT_LDS = (size_t) QT_STAGES * QT_STAGE_BYTES;

struct qt_args {
    const char * w; const char * w2; // Q8_0 rows (w2: the second matrix of a gate/up pair, else null)
    const char * x; char * dst; const char * res;
    int64_t  K, M, N;                // M: rows of one matrix
    uint64_t nb01, nb11, nb12, nb13, nb1, nb2, nb3, rnb1, rnb2, rnb3;
    int      ne12;
    float    res_scale;
    half8_t * wt; float * wdt; half8_t * xt; // the operand tiles in the workspace
    int      n_rt, n_tt, n_kb;       // 16-row tiles (of the virtual matrix: gate and up tiles alternate), token tiles, k blocks
    int      w_al4;
    int      fold;                   // the block scale multiplied into the f16 weights by the weight pass (VX_GEMM_LDS=2)
    const float * norm_w; float norm_eps; // the activation pass applies RMS_NORM and the norm-weight MUL (x is the un-normalised tensor)
    _Float16 * tile_out; int out_tt;      // DUAL: the results leave as the next product's activation tiles (out_tt tiles per k block)
    // several matrices over the same activations as one virtual matrix (q, k and v): rows [seg_row[s], seg_row[s + 1]) are
    // matrix s (whole 64-row groups each), stored to its own destination
    int          nseg;
    int          seg_row[4];
    const char * seg_w[3]; uint64_t seg_nb01[3];
    char *       seg_dst[3]; uint64_t seg_nb1[3], seg_nb3[3];
    // the NEOX rotation of GGML_OP_ROPE on the first rope_segs matrices (heads of 64 rows, rotated whole), applied to the
    // accumulators before the store: (cos, sin) of (token of a batch entry, pair) from a table that a kernel in front of
    // the product fills with the ROPE kernel's own arithmetic
    const float2 * rope_tab; int rope_segs;
};

// (cos, sin) of every (position index, pair): what rope_heads_kernel forms per (token, pair), once per call
// (one wave a work-group: a thread's work is a chain of up to 31 multiplications and a sine and cosine of a large angle,
// so the kernel's time is one thread's latency and the waves are spread over every SIMD)
__global__ __launch_bounds__(64) void qt_rope_table_kernel(const int32_t * __restrict__ pos, const float * __restrict__ ff, rope_params p,
                                                           int N, int T, float2 * __restrict__ tab) {
    const uint32_t gid = blockIdx.x * 64u + threadIdx.x, tok = gid >> 5, ip = gid & 31;
    if (tok >= (uint32_t) N) return;
    float c, sn;
    rope_cos_sin(p, (float) pos[tok % (uint32_t) T], (int) ip, ff ? ff[ip] : 1.0f, c, sn);
    tab[gid] = make_float2(c, sn);
}

// one thread = 8 quants of a block: (virtual row, block, j)
__global__ __launch_bounds__(256) void qt_weights_kernel(const qt_args a) {
    const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
    const int     slot = (int) (idx & 63), c = slot & 15, j = slot >> 4;
    const int64_t t = idx >> 6;
    const int64_t kb = t % a.n_kb; // (neighbouring waves: neighbouring blocks of the same 16 rows, which share cache lines)
    const int64_t rt = t / a.n_kb;
    if (rt >= a.n_rt) return;
    const bool    dual = a.w2 != nullptr;
    int64_t       row  = dual ? 16 * (int64_t) (rt >> 1) + c : 16 * (int64_t) rt + c; // of its own matrix
    const char *  wsel = dual && (rt & 1) ? a.w2 : a.w;
    uint64_t      nb01 = a.nb01;
    int64_t       rows = a.M;
    if (a.nseg) { // (a 16-row tile lies in one matrix: they are whole 64-row groups)
        const int sg = row >= a.seg_row[2] ? 2 : row >= a.seg_row[1] ? 1 : 0;
        wsel = a.seg_w[sg]; nb01 = a.seg_nb01[sg]; rows = a.seg_row[sg + 1] - a.seg_row[sg];
        row -= a.seg_row[sg];
    }
    half8_t h = {0, 0, 0, 0, 0, 0, 0, 0};
    float   d = 0.0f;
    if (row < rows) {
        const char * wrow = wsel + (uint64_t) row * nb01;
        h = q8_unpack(q8_load(wrow, kb, j, a.w_al4 != 0), kb, a.w_al4 != 0);
        const _Float16 dh = *(const _Float16 *) (wrow + kb * VX_Q8_BLOCK);
        d = (float) dh;
        if (a.fold) { // q * d rounded once to f16, as gemm_lds_kernel's FOLD form parks it
#pragma unroll
            for (int i = 0; i < 8; ++i) h[i] *= dh;
        }
    }
    a.wt[(kb * a.n_rt + rt) * 64 + slot] = h;
    // (scales: within every 64 rows, row 16 t + c sits at 4 c + t, so that a lane of the product kernel reads the scales of
    // its row c in the wave's four row tiles with one 16-byte load)
    if (j == 0) a.wdt[kb * ((int64_t) ((a.n_rt + 3) & ~3) * 16) + 64 * (rt >> 2) + 4 * c + (rt & 3)] = d; // (a row of whole groups of 64)
}

// one thread = 8 consecutive k of a token in each of QT_ACT_UNROLL k blocks: (token, group of blocks, j); blockIdx.y =
// batch entry.  A wave reads 16 tokens x 128 bytes per block, all blocks' loads in flight together, and writes one 1 KB
// tile per block.
constexpr int QT_ACT_UNROLL = 4;
__global__ __launch_bounds__(256) void qt_acts_kernel(const qt_args a) {
    const int64_t idx = (int64_t) blockIdx.x * 256 + threadIdx.x;
    const int     slot = (int) (idx & 63), c = slot & 15, j = slot >> 4;
    const int64_t t = idx >> 6;
    const int     n_kg = (a.n_kb + QT_ACT_UNROLL - 1) / QT_ACT_UNROLL;
    const int     kb0 = (int) (t % n_kg) * QT_ACT_UNROLL;
    const int64_t tt = t / n_kg;
    if (tt >= a.n_tt) return;
    const int     batch = blockIdx.y, i12 = batch % a.ne12, i13 = batch / a.ne12;
    const int64_t tok = 16 * tt + c;
    float4_t lo[QT_ACT_UNROLL], hi[QT_ACT_UNROLL];
    const bool live = tok < a.N;
    const char * row = a.x + (uint64_t) i12 * a.nb12 + (uint64_t) i13 * a.nb13 + (uint64_t) (live ? tok : 0) * a.nb11;
#pragma unroll
    for (int u = 0; u < QT_ACT_UNROLL; ++u) {
        const int kb = min(kb0 + u, a.n_kb - 1);
        const float4_t * p = (const float4_t *) (row + (uint64_t) (32 * kb + 8 * j) * 4);
        lo[u] = __builtin_nontemporal_load(p);
        hi[u] = __builtin_nontemporal_load(p + 1);
    }
#pragma unroll
    for (int u = 0; u < QT_ACT_UNROLL; ++u) {
        const int kb = kb0 + u;
        if (kb >= a.n_kb) break;
        half8_t h = {0, 0, 0, 0, 0, 0, 0, 0};
        if (live) {
#pragma unroll
            for (int i = 0; i < 4; ++i) { h[i] = (_Float16) lo[u][i]; h[4 + i] = (_Float16) hi[u][i]; }
        }
        a.xt[(((int64_t) batch * a.n_kb + kb) * a.n_tt + tt) * 64 + slot] = h;
    }
}

// The same tiles from an un-normalised x: RMS_NORM and the norm-weight MUL on the way, rounded as the two separate kernels
// round them.  A work-group = one tile of 16 tokens, a wave = one token in the RMS_NORM kernel's wave-per-row order (rows
// of at most 1024 values: lane l holds columns 4 (l + 64 c) .. + 3); the sixteen rows meet in LDS as f16 and leave as the
// tile's k blocks, 1 KB each.  Against the norm kernel followed by the pass above that is one trip over x instead of two
// and the normalised tensor neither written nor read back.
__global__ __launch_bounds__(1024) void qt_acts_norm_kernel(const qt_args a) {
    constexpr int ROW = 1024 + 8; // halfs between the staged rows: the padding spreads the sixteen tokens over the banks
    __shared__ __attribute__((aligned(16))) _Float16 rows[16 * ROW];
    const int     lane = threadIdx.x & 63, wid = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    const int64_t tt = blockIdx.x;
    const int     batch = blockIdx.y, i12 = batch % a.ne12, i13 = batch / a.ne12;
    const int64_t tok = 16 * tt + wid;
    const int     nv = (int) ((a.K + 255) >> 8); // 16-byte pieces of a row per lane
    const int64_t nvec = a.K / 4;
    if (tok < a.N) { // (uniform per wave)
        vx_rms_row r, gn;
        vx_rms_row_load(r, (const float *) (a.x + (uint64_t) i12 * a.nb12 + (uint64_t) i13 * a.nb13 + (uint64_t) tok * a.nb11), a.K, lane);
#pragma unroll
        for (int cc = 0; cc < 4; ++cc)
            if (cc < nv && lane + 64 * cc < nvec) gn.v[cc] = ((const float4 *) a.norm_w)[lane + 64 * cc];
        const float sc = vx_rms_row_scale(r, a.K, lane, a.norm_eps);
#pragma unroll
        for (int cc = 0; cc < 4; ++cc) {
            if (cc >= nv || lane + 64 * cc >= nvec) break;
            float       v[4]  = { r.v[cc].x, r.v[cc].y, r.v[cc].z, r.v[cc].w };
            const float gg[4] = { gn.v[cc].x, gn.v[cc].y, gn.v[cc].z, gn.v[cc].w };
            half4_t h;
#pragma unroll
            for (int i = 0; i < 4; ++i) { v[i] *= sc; v[i] *= gg[i]; h[i] = (_Float16) v[i]; } // RMS_NORM's product, then the MUL node's
            *(half4_t *) &rows[wid * ROW + 4 * (lane + 64 * cc)] = h;
        }
    } else {
        for (int64_t e = lane; e < nvec; e += 64) *(half4_t *) &rows[wid * ROW + 4 * e] = half4_t{0, 0, 0, 0};
    }
    __syncthreads();
    const int j = lane >> 4, c = lane & 15;
    for (int kb = wid; kb < a.n_kb; kb += 16)
        a.xt[(((int64_t) batch * a.n_kb + kb) * a.n_tt + tt) * 64 + lane] = *(const half8_t *) &rows[c * ROW + 32 * kb + 8 * j];
}

__device__ __forceinline__ void qt_dma16(const void * base, uint32_t off, uint32_t lds) {
    // 16 bytes per lane from global memory (uniform base + lane offset) into LDS at lds + 16 lane
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(off), "s"(base), "s"(lds) : "memory");
}

template <bool DUAL, bool FOLD, bool SEGS = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) void gemm_q8t_kernel(const qt_args a) {
    extern __shared__ __align__(1024) char qt_smem[]; // per stage: 8 token tiles, 16 row tiles, 256 scales
    typedef __attribute__((address_space(3))) char lds_char;
    const int lane = threadIdx.x & 63, wid = __builtin_amdgcn_readfirstlane((int) (threadIdx.x >> 6));
    const int j = lane >> 4, c = lane & 15;
    const int wr = wid >> 1, wc = wid & 1;

    // which tile: groups of 4 row tiles x 8 token tiles, a group's 32 work-groups on one XCD
    const int gx = (a.n_rt + 15) / 16, gy = (a.n_tt + 7) / 8; // tiles of 256 rows / 128 tokens
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int group = (seq >> 5) * 8 + xcd, within = seq & 31;
    int tx, ty;
    if constexpr (SEGS) {
        // several matrices of few rows in all (q, k and v: 1280 rows, five row tiles): a group is ALL the row tiles of
        // 32 / gx token tiles, so that every token tile's activations are fetched into one XCD's L2 once and the small
        // matrices' tiles run beside the large one's (as a group of four row tiles plus a leftover group the last tile's
        // work-groups ran alone at the end, every one of them fetching its tokens from memory: 309 us against 200 for q alone)
        const int per = 32 / gx; // (the launcher takes this form for gx <= 8 only)
        if (within >= gx * per) return;
        const int wy = within / gx;
        tx = __builtin_amdgcn_readfirstlane(within - wy * gx);
        ty = __builtin_amdgcn_readfirstlane(group * per + wy);
    } else {
        const int Gx = (gx + 3) / 4, Gy = (gy + 7) / 8;
        if (group >= Gx * Gy) return;
        tx = (group % Gx) * 4 + (within & 3);
        ty = (group / Gx) * 8 + (within >> 2);
    }
    if (tx >= gx || ty >= gy) return;
    const int batch = blockIdx.y, i12 = batch % a.ne12, i13 = batch / a.ne12;

    // ---- direct loads of a stage: wave w brings row tiles 2w and 2w + 1 and token tile w; wave 0 the scales as well.
    // A tile past the operand's last one is not loaded (its products are dropped at the store).
    const int rt0 = 16 * tx, tt0 = 8 * ty;
    const uint32_t smem0 = (uint32_t) (uintptr_t) (lds_char *) qt_smem;
    const bool     have_w0 = rt0 + 2 * wid < a.n_rt, have_w1 = rt0 + 2 * wid + 1 < a.n_rt, have_x = tt0 + wid < a.n_tt;
    const half8_t * wsrc = a.wt + ((int64_t) rt0 + 2 * wid) * 64;
    const half8_t * xsrc = a.xt + ((int64_t) batch * a.n_kb * a.n_tt + tt0 + wid) * 64;
    const float *   dsrc = a.wdt + (int64_t) rt0 * 16;
    const uint32_t  loff = (uint32_t) lane * 16;
    const int       n_rt4 = (a.n_rt + 3) & ~3;                  // the scale rows hold whole groups of 64 rows
    const int       n_dsc = min(256, (n_rt4 - rt0) * 16) / 4;  // 16-byte pieces of the scale row that exist
    auto issue = [&](int kb) {
        const uint32_t st = smem0 + (uint32_t) (kb % QT_STAGES) * QT_STAGE_BYTES;
        if (have_x)  qt_dma16(xsrc + (int64_t) kb * a.n_tt * 64, loff, st + wid * 1024);
        if (have_w0) qt_dma16(wsrc + (int64_t) kb * a.n_rt * 64, loff, st + 8192 + 2 * wid * 1024);
        if (have_w1) qt_dma16(wsrc + (int64_t) kb * a.n_rt * 64 + 64, loff, st + 8192 + (2 * wid + 1) * 1024);
        if (wid == 0) qt_dma16(dsrc + (int64_t) kb * n_rt4 * 16, lane < n_dsc ? loff : 0u, st + 8192 + 16384);
    };
    // (a wave waits for its own loads, so it counts what it issued per stage)
    const int mine = (have_x ? 1 : 0) + (have_w0 ? 1 : 0) + (have_w1 ? 1 : 0) + (wid == 0 ? 1 : 0);

    float4_t acc[4][4]; // [row tile][token tile]
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) acc[rt][tt] = float4_t{0, 0, 0, 0};

    const int nkb = a.n_kb;
    auto wait_stage = [&](int kb) { // stage kb has landed once only the younger stages' loads of this wave are outstanding
        const int younger = min(QT_STAGES - 2, nkb - 1 - kb) * mine;
        if (younger >= 8)      asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        else if (younger == 6) asm volatile("s_waitcnt vmcnt(6)" ::: "memory");
        else if (younger == 4) asm volatile("s_waitcnt vmcnt(4)" ::: "memory");
        else if (younger == 3) asm volatile("s_waitcnt vmcnt(3)" ::: "memory");
        else if (younger == 2) asm volatile("s_waitcnt vmcnt(2)" ::: "memory");
        else                   asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    };
    // 16 MFMAs and their 64 scaled additions: the additions of a product follow the MFMA two further on, so that matrix
    // instructions are in flight while the vector unit scales an earlier one
    auto multiply = [&](int kb) {
        const lds_char * st = (const lds_char *) qt_smem + (kb % QT_STAGES) * QT_STAGE_BYTES;
        half8_t bop[4];
#pragma unroll
        for (int rt = 0; rt < 4; ++rt) bop[rt] = *(const __attribute__((address_space(3))) half8_t *) (st + 8192 + (4 * wr + rt) * 1024 + lane * 16);
        // the scales of row c in the wave's four row tiles: one load (LDS reads, counted at their full 64 lanes x 16 bytes
        // whatever they broadcast, are what bounds this loop: four loads here were a quarter of its time)
        const float4_t dw = *(const __attribute__((address_space(3))) float4_t *) (st + 8192 + 16384 + (64 * wr + 4 * c) * 4);
        half8_t aop[2];
        aop[0] = *(const __attribute__((address_space(3))) half8_t *) (st + (4 * wc) * 1024 + lane * 16);
        if constexpr (FOLD) { // the scale is in the weights: the MFMAs accumulate across blocks
#pragma unroll
            for (int tt = 0; tt < 4; ++tt) {
                if (tt < 3) aop[(tt + 1) & 1] = *(const __attribute__((address_space(3))) half8_t *) (st + (4 * wc + tt + 1) * 1024 + lane * 16);
#pragma unroll
                for (int rt = 0; rt < 4; ++rt) acc[rt][tt] = mfma16(aop[tt & 1], bop[rt], acc[rt][tt]);
            }
            return;
        }
        float4_t blk[3];
#pragma unroll
        for (int i = 0; i < 18; ++i) {
            const int tt = i >> 2, rt = i & 3;
            if (i < 16) {
                if (rt == 0 && tt < 3) aop[(tt + 1) & 1] = *(const __attribute__((address_space(3))) half8_t *) (st + (4 * wc + tt + 1) * 1024 + lane * 16);
                blk[i % 3] = mfma16(aop[tt & 1], bop[rt], float4_t{0, 0, 0, 0});
                __builtin_amdgcn_sched_barrier(0); // (the MFMA first: the additions below belong to the one two before it)
            }
            if (i >= 2) {
                const int p = i - 2;
                acc[p & 3][p >> 2] += blk[p % 3] * dw[p & 3]; // (one scale per lane: the weights are the MFMA's column operand, lane c = row c)
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
#pragma unroll
    for (int s = 0; s < QT_STAGES - 1; ++s)
        if (s < nkb) issue(s);
    for (int kb = 0; kb < nkb; ++kb) {
        wait_stage(kb);
        __syncthreads(); // every wave's part of stage kb is in LDS, and every wave is done with stage kb - 1
        if (kb + QT_STAGES - 1 < nkb) issue(kb + QT_STAGES - 1);
        multiply(kb);
    }

    // lane (j, c), tile (rt, tt), register r: token tok0 + 16 tt + 4 j + r, virtual row 16 (rt0 + 4 wr + rt) + c
    const int64_t tok0 = (int64_t) ty * QT_TOKS + 64 * wc;
    char * db = a.dst + (uint64_t) i12 * a.nb2 + (uint64_t) i13 * a.nb3;
    if constexpr (SEGS) { // (a form of its own: in the common kernel the extra addresses cost the registers it has none to spare of)
        { // (uniform per wave) the wave's 64 rows belong to one matrix: its destination, its row numbers
            const int vrow = 16 * (rt0 + 4 * wr);
            if (vrow >= a.seg_row[3]) return;
            const int sg = vrow >= a.seg_row[2] ? 2 : vrow >= a.seg_row[1] ? 1 : 0;
            char *         sb  = a.seg_dst[sg] + (uint64_t) i13 * a.seg_nb3[sg];
            const uint64_t nb1 = a.seg_nb1[sg];
            const int      r0  = vrow - a.seg_row[sg];
            if (a.rope_tab && sg < a.rope_segs) { // (uniform) the wave's 64 rows are one head: pair (d, d + 32) is tiles (rt, rt + 2) of a lane
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int r2 = 0; r2 < 4; r2 += 2) {
                        float2 cs[2][2];
#pragma unroll
                        for (int r = 0; r < 2; ++r) {
                            uint32_t tok = min((uint32_t) tok0 + (uint32_t) (16 * tt + 4 * j + r2 + r), (uint32_t) a.N - 1u); // (a ragged tile's spare tokens: stores dropped below)
                            const uint32_t off = tok * 256u + (uint32_t) c * 8u; // (uniform base + 32-bit lane offset; the launcher checks the range)
                            cs[r][0] = *(const float2 *) ((const char *) a.rope_tab + off);
                            cs[r][1] = *(const float2 *) ((const char *) a.rope_tab + off + 128u);
                        }
#pragma unroll
                        for (int r = 0; r < 2; ++r)
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                float y0, y1;
                                rope_rotate(acc[h][tt][r2 + r], acc[h + 2][tt][r2 + r], cs[r][h].x, cs[r][h].y, y0, y1);
                                acc[h][tt][r2 + r] = y0; acc[h + 2][tt][r2 + r] = y1;
                            }
                        __builtin_amdgcn_sched_barrier(0); // (eight table values at a time: the accumulators leave few registers)
                    }
            }
            if ((int64_t) (ty + 1) * QT_TOKS <= a.N) { // (uniform) a whole token tile: a uniform base and one 32-bit lane offset, no tests
                char *         tb = sb + (uint64_t) tok0 * nb1 + (uint64_t) r0 * 4;
                const uint32_t lo = (uint32_t) ((uint64_t) (4 * j) * nb1 + (uint64_t) c * 4);
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        char * tr = tb + (uint64_t) (16 * tt + r) * nb1; // uniform
#pragma unroll
                        for (int rt = 0; rt < 4; ++rt) __builtin_nontemporal_store(acc[rt][tt][r], (float *) (tr + 64 * rt + lo));
                    }
                return;
            }
#pragma unroll
            for (int rt = 0; rt < 4; ++rt) {
                const int row = r0 + 16 * rt + c; // (inside the matrix: whole 64-row groups)
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int64_t tok = tok0 + 16 * tt + 4 * j + r;
                        if (tok < a.N) __builtin_nontemporal_store(acc[rt][tt][r], (float *) (sb + (uint64_t) tok * nb1 + (uint64_t) row * 4));
                    }
            }
            return;
        }
    }
    // A tile inside the matrix stores without tests, at a uniform base plus one 32-bit lane offset (the launcher checks the
    // range): computed per element in 64-bit arithmetic, the addresses of a tile's 64 stores per lane were a fifth of the
    // kernel's vector instructions.
    if constexpr (DUAL) {
        if (a.tile_out) { // (uniform) silu(g) * u rounded to f16, as the next product's activation pass would round it, straight
            // into that product's tiles: row = its k index.  Tile (k block, 16 tokens), slot (k / 8 mod 4, token mod 16), 8 halfs.
            const uint32_t n_kb2 = (uint32_t) (a.M >> 5);
#pragma unroll
            for (int p2 = 0; p2 < 2; ++p2) {
                const uint32_t row = 16u * ((uint32_t) (rt0 >> 1) + 2u * wr + p2) + c;
                if (row >= (uint32_t) a.M) continue;
                const uint32_t kb2 = row >> 5, slot_j = (row >> 3) & 3, e = row & 7;
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const uint32_t tok = (uint32_t) tok0 + 16u * tt + 4u * j + r;
                        const float g = acc[2 * p2][tt][r], u = acc[2 * p2 + 1][tt][r];
                        const uint64_t tile = ((uint64_t) batch * n_kb2 + kb2) * (uint32_t) a.out_tt + (tok >> 4);
                        float h = (g / (1.0f + expf(-g))) * u; // the fp32 value the GLU node holds ...
                        asm volatile("" : "+v"(h));             // ... formed as such, then rounded as the activation pass rounds it
                        a.tile_out[(tile * 64 + slot_j * 16 + (tok & 15)) * 8 + e] = (_Float16) h;
                    }
            }
            return;
        }
    }
    const bool inside = (int64_t) (ty + 1) * QT_TOKS <= a.N && (int64_t) (tx + 1) * QT_ROWS <= (DUAL ? 2 * a.M : a.M); // uniform
    if (inside) {
        const int64_t  row0 = DUAL ? 16 * ((int64_t) (rt0 >> 1) + 2 * wr) : 16 * ((int64_t) rt0 + 4 * wr);
        char *         tb   = db + (uint64_t) tok0 * a.nb1 + (uint64_t) row0 * 4;
        const uint32_t lo   = (uint32_t) ((uint64_t) (4 * j) * a.nb1 + (uint64_t) c * 4);
        if constexpr (DUAL) {
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    char * tr = tb + (uint64_t) (16 * tt + r) * a.nb1; // uniform
#pragma unroll
                    for (int p2 = 0; p2 < 2; ++p2) {
                        const float g = acc[2 * p2][tt][r], u = acc[2 * p2 + 1][tt][r];
                        __builtin_nontemporal_store((g / (1.0f + expf(-g))) * u, (float *) (tr + 64 * p2 + lo));
                    }
                }
            return;
        } else {
            if (a.res) {
                const char *   rb  = a.res + (uint64_t) i12 * a.rnb2 + (uint64_t) i13 * a.rnb3 + (uint64_t) tok0 * a.rnb1 + (uint64_t) row0 * 4;
                const uint32_t rlo = (uint32_t) ((uint64_t) (4 * j) * a.rnb1 + (uint64_t) c * 4);
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const char * rr = rb + (uint64_t) (16 * tt + r) * a.rnb1; // uniform
#pragma unroll
                        for (int rt = 0; rt < 4; ++rt) acc[rt][tt][r] = scaled_residual(acc[rt][tt][r], a.res_scale, *(const float *) (rr + 64 * rt + rlo));
                    }
            }
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    char * tr = tb + (uint64_t) (16 * tt + r) * a.nb1; // uniform
#pragma unroll
                    for (int rt = 0; rt < 4; ++rt) __builtin_nontemporal_store(acc[rt][tt][r], (float *) (tr + 64 * rt + lo));
                }
            return;
        }
    }
    if constexpr (DUAL) {
        // tile pair (2p, 2p + 1) holds gate and up of row 16 (rt0 / 2 + 2 wr + p) + c
#pragma unroll
        for (int p2 = 0; p2 < 2; ++p2) {
            const int64_t row = 16 * ((int64_t) (rt0 >> 1) + 2 * wr + p2) + c;
            if (row >= a.M) continue;
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t tok = tok0 + 16 * tt + 4 * j + r;
                    const float g = acc[2 * p2][tt][r], u = acc[2 * p2 + 1][tt][r];
                    if (tok < a.N) __builtin_nontemporal_store((g / (1.0f + expf(-g))) * u, (float *) (db + (uint64_t) tok * a.nb1 + (uint64_t) row * 4));
                }
        }
        return;
    }
    const bool   residual = a.res != nullptr; // uniform
    const char * rbase    = residual ? a.res + (uint64_t) i12 * a.rnb2 + (uint64_t) i13 * a.rnb3 : nullptr;
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) {
        const int64_t row = 16 * ((int64_t) rt0 + 4 * wr + rt) + c;
        if (row >= a.M) continue;
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t tok = tok0 + 16 * tt + 4 * j + r;
                if (tok >= a.N) continue;
                float v = acc[rt][tt][r];
                if (residual) v = scaled_residual(v, a.res_scale, *(const float *) (rbase + (uint64_t) tok * a.rnb1 + (uint64_t) row * 4));
                __builtin_nontemporal_store(v, (float *) (db + (uint64_t) tok * a.nb1 + (uint64_t) row * 4));
            }
    }
}

// VX_GEMM_Q8T=0 keeps these products on gemm_lds_kernel, 2 sends every shape the kernel can take to it, however few its
// tiles (read on every call: a product of this size takes a hundred microseconds, and a test compares the two kernels in
// one process)
int gemm_q8t_mode() { const char * e = getenv("VX_GEMM_Q8T"); return e ? atoi(e) : 1; }

// the shapes the pre-tiled kernel takes: one weight matrix for every batch entry, at least 1024 (virtual) rows and
// 1024 tokens -- below that the two passes in front cost more than they save -- and two tiles of 256 x 128 or more per
// compute unit (the 2 x 512-token prefill of a 24-layer stack is 32 to 256 such tiles a product: 4.6 ms on the smaller
// tiles of gemm_lds_kernel and its K cut, 7.2 ms here)
bool gemm_q8t_takes(const mm_args & a, int nbatch, bool dual) {
    const int64_t MV = dual ? 2 * a.M : a.M;
    if (a.norm_w && (a.K > 1024 || a.K % 8 || (uintptr_t) a.norm_w % 16)) return false; // (the norm's wave-per-row regime)
    const int mode = gemm_q8t_mode();
    const int64_t tiles = ((MV + QT_ROWS - 1) / QT_ROWS) * ((a.N + QT_TOKS - 1) / QT_TOKS) * nbatch;
    // (and a thousand tiles' worth of K = 1024: 1024 x 1024 x 16384 is 86 us here against 74, 4096 x 1024 x 4096 a tie, every
    // larger product 20 to 30 % faster here)
    if (mode == 0 || (mode != 2 && (tiles < 512 || tiles * a.K < 1024 * 1024))) return false;
    // (32-bit lane offsets inside a tile: the 128 tokens of dst and of a residual)
    if ((uint64_t) 128 * a.nb1 + 1024 >= (1ull << 32) || (a.res && (uint64_t) 128 * a.rnb1 + 1024 >= (1ull << 32))) return false;
    return a.K % 32 == 0 && (!dual || a.M % 16 == 0) && MV >= 1024 && a.N >= 1024 && a.x_aligned && (nbatch == 1 || (a.r2 == a.ne12 && a.r3 * a.ne12 == nbatch)) &&
           a.K < (1ll << 24) && nbatch <= 65535;
}

template <bool DUAL>
bool launch_gemm_q8t(const mm_args & a, int nbatch, hipStream_t st, bool fold) {
    qt_args q = {};
    q.w = a.w; q.w2 = DUAL ? a.w2 : nullptr; q.x = a.x; q.dst = a.dst; q.res = DUAL ? nullptr : a.res;
    q.K = a.K; q.M = a.M; q.N = a.N;
    q.nb01 = a.nb01; q.nb11 = a.nb11; q.nb12 = a.nb12; q.nb13 = a.nb13; q.nb1 = a.nb1; q.nb2 = a.nb2; q.nb3 = a.nb3;
    q.rnb1 = a.rnb1; q.rnb2 = a.rnb2; q.rnb3 = a.rnb3;
    q.ne12 = a.ne12; q.res_scale = a.res_scale;
    q.w_al4 = a.w_aligned;
    q.fold  = fold;
    const int64_t MV = DUAL ? 2 * a.M : a.M;
    q.n_rt = (int) ((MV + 15) / 16); q.n_tt = a.tile_in ? a.tile_tt : (int) ((a.N + 15) / 16); q.n_kb = (int) (a.K / 32);
    q.tile_out = DUAL ? (_Float16 *) a.tile_out : nullptr; q.out_tt = a.tile_tt;
    const bool segs = !DUAL && a.nseg > 0; // (the streaming kernel's segments: rotation is the caller's business here)
    if (segs) {
        if (a.nseg > 3 || a.res) return false;
        int at = 0;
        for (int i = 0; i < 3; ++i) {
            q.seg_row[i] = at;
            if (i < a.nseg) {
                if (a.seg[i].M % 64 || (uint64_t) 128 * a.seg[i].nb1 + 1024 >= (1ull << 32)) return false; // (whole 64-row groups; 32-bit lane offsets in a tile)
                q.seg_w[i] = a.seg[i].w; q.seg_nb01[i] = a.seg[i].nb01; q.seg_dst[i] = a.seg[i].dst; q.seg_nb1[i] = a.seg[i].nb1; q.seg_nb3[i] = a.seg[i].nb3;
                at += (int) a.seg[i].M;
            } else {
                q.seg_w[i] = nullptr; q.seg_nb01[i] = 0; q.seg_dst[i] = nullptr; q.seg_nb1[i] = 0; q.seg_nb3[i] = 0;
            }
        }
        q.seg_row[3] = at;
        q.nseg = a.nseg;
        if (at != a.M) return false;
    }
    const size_t wt_bytes = (size_t) q.n_kb * q.n_rt * 1024, wd_bytes = ((size_t) q.n_kb * ((q.n_rt + 3) & ~3) * 16 * 4 + 1023) / 1024 * 1024 + 1024; // (+ a scale row's worth: the last stage's 1 KB load of a ragged row tile count stays inside)
    const size_t xt_bytes = a.tile_in ? 0 : (size_t) nbatch * q.n_kb * q.n_tt * 1024;
    static bool raised = false;
    if (!raised) {
        if (hipFuncSetAttribute((const void *) gemm_q8t_kernel<false, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QT_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *) gemm_q8t_kernel<true, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QT_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *) gemm_q8t_kernel<false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QT_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *) gemm_q8t_kernel<true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QT_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *) gemm_q8t_kernel<false, false, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QT_LDS) != hipSuccess ||
            hipFuncSetAttribute((const void *) gemm_q8t_kernel<false, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int) QT_LDS) != hipSuccess) {
            (void) hipGetLastError();
            return false;
        }
        raised = true;
    }
    const int64_t wunits = (int64_t) q.n_kb * q.n_rt * 64, xunits = (int64_t) ((q.n_kb + QT_ACT_UNROLL - 1) / QT_ACT_UNROLL) * q.n_tt * 64;
    if ((wunits + 255) / 256 > 0x7fffffff || (xunits + 255) / 256 > 0x7fffffff) return false;
    const int gx = (q.n_rt + 15) / 16, gy = (q.n_tt + 7) / 8, Gx = (gx + 3) / 4, Gy = (gy + 7) / 8;
    if (segs && gx > 8) return false; // (the segment form's groups hold all the row tiles)
    // groups of 32 work-groups, dealt to the XCDs in turn: 4 row tiles x 8 token tiles, or (segments) all gx row tiles x 32 / gx token tiles
    const int64_t groups = segs ? ((int64_t) gy + 32 / gx - 1) / (32 / gx) : (int64_t) Gx * Gy;
    const int64_t blocks = (groups + 7) / 8 * 8 * 32;
    if (blocks > 0x7fffffff) return false;
    // the weights' tiles: kept from call to call when the caller has pinned the weights, else made in the workspace
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void) hipGetLastError(); return false; }
    const vx_derived_key key = { dev, fold ? 2 : 1, a.w, DUAL ? a.w2 : nullptr, a.K, a.M, a.nb01 };
    bool fresh = false;
    char * kept = segs ? nullptr : (char *) vx_derived_get(key, wt_bytes + wd_bytes, st, &fresh); // (three matrices: tiles made per call)
    void * ws = nullptr;
    // (segments with a rotation: the angle table behind the tiles)
    const bool   rotate = segs && a.pos != nullptr;
    // (token n of a batch entry sits at position index n % rope_T: sequences may be flattened into the token dimension)
    const size_t tab_bytes = rotate ? (size_t) a.N * 32 * sizeof(float2) : 0;
    if (rotate && (a.head_dim != 64 || a.rp.n_dims != 64 || a.rp.mode != 2 || a.rope_T <= 0 || a.N * 256 >= ((int64_t) 1 << 32))) return false;
    if ((t_ws_status = vx_workspace(st, a.ws_offset + (kept ? 0 : wt_bytes + wd_bytes) + xt_bytes + tab_bytes, &ws)) != VX_OK) {
        (void) hipGetLastError();
        if (fresh) vx_derived_abandon(key, st);
        return false;
    }
    char * base = (char *) ws + a.ws_offset;
    if (kept) { q.wt = (half8_t *) kept; q.wdt = (float *) (kept + wt_bytes); q.xt = (half8_t *) base; }
    else      { q.wt = (half8_t *) base; q.wdt = (float *) (base + wt_bytes); q.xt = (half8_t *) (base + wt_bytes + wd_bytes); }
    if (a.tile_in) q.xt = (half8_t *) const_cast<void *>(a.tile_in);
    if (!kept || fresh) vx_launch(qt_weights_kernel, dim3((unsigned) ((wunits + 255) / 256)), dim3(256), 0, st, q);
    if (fresh) vx_derived_filled(key, st);
    q.norm_w = a.norm_w; q.norm_eps = a.norm_eps;
    if (a.tile_in) {} // (the activations are the tiles the product before left)
    else if (a.norm_w) vx_launch(qt_acts_norm_kernel, dim3((unsigned) q.n_tt, (unsigned) nbatch), dim3(1024), 0, st, q);
    else          vx_launch(qt_acts_kernel, dim3((unsigned) ((xunits + 255) / 256), (unsigned) nbatch), dim3(256), 0, st, q);
    if constexpr (!DUAL) {
        if (segs) {
            if (rotate) {
                q.rope_tab = (const float2 *) (base + (kept ? 0 : wt_bytes + wd_bytes) + xt_bytes);
                q.rope_segs = 2;
                vx_launch(qt_rope_table_kernel, dim3((unsigned) ((a.N * 32 + 63) / 64)), dim3(64), 0, st, a.pos, a.ff, a.rp, (int) a.N, a.rope_T,
                          const_cast<float2 *>(q.rope_tab));
            }
            if (fold) vx_launch(gemm_q8t_kernel<false, true, true>, dim3((unsigned) blocks, (unsigned) nbatch), dim3(512), QT_LDS, st, q);
            else      vx_launch(gemm_q8t_kernel<false, false, true>, dim3((unsigned) blocks, (unsigned) nbatch), dim3(512), QT_LDS, st, q);
            return true;
        }
    }
    if (fold) vx_launch(gemm_q8t_kernel<DUAL, true>, dim3((unsigned) blocks, (unsigned) nbatch), dim3(512), QT_LDS, st, q);
    else      vx_launch(gemm_q8t_kernel<DUAL, false>, dim3((unsigned) blocks, (unsigned) nbatch), dim3(512), QT_LDS, st, q);
    return true;
}

template <int WT>
bool launch_gemm_lds(const mm_args & a, int nbatch, hipStream_t st) {
    const int mode = gemm_lds_mode();
    // (from 17 tokens on: what reaches this point with fewer than 64 is a product the streaming kernel has declined -- K beyond
    // 2048, or too many rows for its token chunks -- and the one ragged token tile with its K cut is 12 us where the older
    // kernels took 21 to 54)
    if (mode == 0 || WT == WT_F32 || a.K % (32 * GL_KC) || a.N <= 16 || !a.x_aligned) return false;
    if (WT == WT_Q8 && !a.w_aligned) return false;
    if (WT == WT_F16 && (((uintptr_t) a.w | a.nb01 | a.nb02 | a.nb03) % 16 != 0)) return false;
    // 32-bit lane offsets: rows of the weight matrix, the (up to 256) tokens of a tile
    if ((uint64_t) a.M * a.nb01 >= (1ull << 32) || (uint64_t) 256 * a.nb11 + 256 >= (1ull << 32) ||
        (uint64_t) 256 * a.nb1 + 1024 >= (1ull << 32) || a.K >= (1ll << 28)) return false;
    const bool fold = WT == WT_Q8 && mode == 2;
    if constexpr (WT == WT_Q8) {
        if (gemm_q8t_takes(a, nbatch, false)) return launch_gemm_q8t<false>(a, nbatch, st, fold);
    }
    // (a residual update is fused into the kernel that adds a cut K's partials, nowhere else here)
    // 128 x 128 tiles once they fill most of the chip, else 64 x 64
    const bool big = ((a.M + 127) / 128) * ((a.N + 127) / 128) * nbatch >= 192;
    const int64_t tiles64 = ((a.M + 63) / 64) * ((a.N + 63) / 64) * nbatch;
    const int  ks = gemm_lds_cut(a.M, a.N, a.K, nbatch);
    const bool cut_fits = !(a.M % 4 || (uintptr_t) a.dst % 16 || a.nb1 % 16 || a.nb2 % 16 || a.nb3 % 16 || (int64_t) nbatch * ks > 65535);
    if (!big && tiles64 < 64 && !(ks >= 2 && cut_fits)) return false; // (few tiles with K whole: the other kernels' shape)
    if (ks >= 2 && cut_fits) {
        // the K range is cut across ks work-groups per tile; a second kernel adds their partials in split order
        void * ws = nullptr;
        if ((t_ws_status = vx_workspace(st, a.ws_offset + (size_t) nbatch * ks * a.N * a.M * sizeof(float), &ws)) != VX_OK) { (void) hipGetLastError(); return false; }
        mm_args b = a;
        b.ksplit = ks; b.partial = (float *) ((char *) ws + a.ws_offset);
        const bool ok = WT == WT_Q8 && mode == 2 ? launch_gemm_lds_tile<WT, WT == WT_Q8, 2, 2, 2, 2>(b, nbatch, st) : launch_gemm_lds_tile<WT, false, 2, 2, 2, 2>(b, nbatch, st);
        if (!ok) return false;
        const int64_t units = a.N * (a.M / 4);
        vx_launch(mm_splitk_reduce_kernel, dim3((unsigned) ((units + 255) / 256), 1, (unsigned) nbatch), dim3(256), 0, st, b);
        return true;
    }
    if (a.res && (uint64_t) 256 * a.rnb1 + 1024 >= (1ull << 32)) return false; // (the residual's 32-bit lane offsets)
    // 128 x 128: 8 waves of 64 rows x 32 tokens (4 waves per SIMD with two work-groups per CU measured 5-10 % above
    // 4 waves of 64 x 64); 64 x 64: 4 waves of 32 x 32
    if constexpr (WT == WT_Q8) {
        if (fold) return big ? launch_gemm_lds_tile<WT, true, 4, 2, 2, 4>(a, nbatch, st) : launch_gemm_lds_tile<WT, true, 2, 2, 2, 2>(a, nbatch, st);
    }
    return big ? launch_gemm_lds_tile<WT, false, 4, 2, 2, 4>(a, nbatch, st) : launch_gemm_lds_tile<WT, false, 2, 2, 2, 2>(a, nbatch, st);
}

// gate and up of mlp_forward with the GLU node's arithmetic in the tile's epilogue (gemm_lds_kernel's DUAL form); the
// shapes are those of gemm_lds_swiglu_ok
template <int WT>
bool launch_gemm_lds_swiglu(const mm_args & a, int nbatch, hipStream_t st) {
    const bool fold = WT == WT_Q8 && gemm_lds_mode() == 2;
    if constexpr (WT == WT_Q8) {
        if (gemm_q8t_takes(a, nbatch, true)) return launch_gemm_q8t<true>(a, nbatch, st, fold);
    }
    if (a.norm_w) return false; // (a fused norm exists in the pre-tiled kernel's activation pass only)
    const bool big  = ((2 * a.M + 127) / 128) * ((a.N + 127) / 128) * nbatch >= 192;
    if constexpr (WT == WT_Q8) {
        if (fold) return big ? launch_gemm_lds_tile<WT, true, 4, 2, 2, 4, true>(a, nbatch, st) : launch_gemm_lds_tile<WT, true, 2, 2, 2, 2, true>(a, nbatch, st);
    }
    return big ? launch_gemm_lds_tile<WT, false, 4, 2, 2, 4, true>(a, nbatch, st) : launch_gemm_lds_tile<WT, false, 2, 2, 2, 2, true>(a, nbatch, st);
}

// A long K on a grid that leaves most CUs with one work-group is a chain of ~3 us rounds: cut K so that every split walks
// about 1024 of it, and add the partials in a second launch (which also applies a fused residual update).
template <int WT, bool ACT_Q8>
bool launch_mm_cut(const mm_args & a, int nbatch, hipStream_t st) {
    if (a.N <= 32) return false;
    const int64_t gx = (a.M + 63) / 64, gy = (a.N + 63) / 64;
    if (!(a.K >= 2048 && a.K % 128 == 0 && a.M % 4 == 0 && gx * gy * nbatch <= 512 && (uintptr_t) a.dst % 16 == 0 && a.nb1 % 16 == 0 &&
          a.nb2 % 16 == 0 && a.nb3 % 16 == 0)) return false;
    int ks = (int) (a.K / 1024);
    if (ks > 8) ks = 8;
    if (ks < 2 || (int64_t) nbatch * ks > 65535) return false;
    void * ws = nullptr;
    if ((t_ws_status = vx_workspace(st, a.ws_offset + (size_t) nbatch * ks * a.N * a.M * sizeof(float), &ws)) != VX_OK) { (void) hipGetLastError(); return false; }
    mm_args b = a;
    b.ksplit = ks; b.partial = (float *) ((char *) ws + a.ws_offset);
    vx_launch(mm_kernel<WT, 4, ACT_Q8, false>, dim3((unsigned) gx, (unsigned) gy, (unsigned) (nbatch * ks)), dim3(256), 0, st, b);
    const int64_t units = a.N * (a.M / 4);
    vx_launch(mm_splitk_reduce_kernel, dim3((unsigned) ((units + 255) / 256), 1, (unsigned) nbatch), dim3(256), 0, st, b);
    return true;
}

template <int WT, bool ACT_Q8>
void launch(const mm_args & a, int nbatch, hipStream_t st) {
    if constexpr (WT != WT_F32) { if (launch_gemv<WT, ACT_Q8>(a, nbatch, st)) return; }
    if constexpr (WT != WT_F32 && !ACT_Q8) { if (launch_gemm_lds<WT>(a, nbatch, st) || ws_failed()) return; }
    if constexpr (WT != WT_F32) { if (launch_gemm128<WT, ACT_Q8>(a, nbatch, st)) return; }
    if (a.N <= 16) {
        const dim3 grid((unsigned) ((a.M + 15) / 16), 1, (unsigned) nbatch);
        vx_launch(mm_kernel<WT, 1, ACT_Q8, true>, grid, dim3(256), 0, st, a);
    } else if (a.N <= 32) {
        const dim3 grid((unsigned) ((a.M + 63) / 64), 1, (unsigned) nbatch);
        vx_launch(mm_kernel<WT, 2, ACT_Q8, false>, grid, dim3(256), 0, st, a);
    } else {
        if (launch_mm_cut<WT, ACT_Q8>(a, nbatch, st) || ws_failed()) return;
        const int64_t gx = (a.M + 63) / 64, gy = (a.N + 63) / 64;
        const dim3 grid((unsigned) gx, (unsigned) gy, (unsigned) nbatch);
        vx_launch(mm_kernel<WT, 4, ACT_Q8, false>, grid, dim3(256), 0, st, a);
    }
}

} // namespace

extern "C" int vx_supports_mul_mat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst) {
    if (!src0 || !src1 || !dst) return 0;
    if (src0->type != VX_TYPE_Q8_0 && src0->type != VX_TYPE_F16 && src0->type != VX_TYPE_F32) return 0;
    if (src1->type != VX_TYPE_F32 || dst->type != VX_TYPE_F32) return 0;
    if (!vx_positive(src0) || !vx_positive(src1)) return 0;
    if (src0->ne[0] != src1->ne[0]) return 0;
    if (src0->type == VX_TYPE_Q8_0 && src0->ne[0] % VX_QK8_0) return 0;
    if (src1->ne[2] % src0->ne[2] || src1->ne[3] % src0->ne[3]) return 0;
    if (dst->ne[0] != src0->ne[1] || dst->ne[1] != src1->ne[1] || dst->ne[2] != src1->ne[2] || dst->ne[3] != src1->ne[3]) return 0;
    if (src0->nb[0] != vx_type_size(src0->type) || src1->nb[0] != 4 || dst->nb[0] != 4) return 0;
    // weight rows must not overlap or interleave (transposed views stay on the CPU)
    if (src0->nb[1] < vx_row_size(src0->type, src0->ne[0])) return 0;
    if (src0->type == VX_TYPE_F16 && (src0->nb[1] % 2 || src0->nb[2] % 2 || src0->nb[3] % 2)) return 0;
    if (src0->type == VX_TYPE_F32 && (src0->nb[1] % 4 || src0->nb[2] % 4 || src0->nb[3] % 4)) return 0;
    if (src1->nb[1] % 4 || src1->nb[2] % 4 || src1->nb[3] % 4) return 0;
    if (dst->nb[1] % 4 || dst->nb[2] % 4 || dst->nb[3] % 4 || dst->nb[1] < (uint64_t) dst->ne[0] * 4) return 0;
    if (src1->ne[2] * src1->ne[3] > 65535) return 0;
    if ((src1->ne[1] + 63) / 64 > 65535) return 0;
    return 1;
}

extern "C" vx_status vx_mul_mat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int act_mode,
                                vx_stream stream) {
    if (!src0 || !src1 || !dst || !src0->data || !src1->data || !dst->data)
        return vx_fail(VX_ERR_INVALID, "mul_mat: null tensor");
    if (!vx_supports_mul_mat(src0, src1, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat: needs src0 Q8_0/F16/F32 with dense rows, src1 F32, dst F32, matching shapes");
    if (act_mode != VX_ACT_FLOAT && act_mode != VX_ACT_Q8) return vx_fail(VX_ERR_INVALID, "mul_mat: bad act_mode");
    if (src0->type == VX_TYPE_F16 && (uintptr_t) src0->data % 2) return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat: F16 weights must be 2-byte aligned");
    if (src0->type == VX_TYPE_F32 && (uintptr_t) src0->data % 4) return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat: F32 weights must be 4-byte aligned");
    if ((uintptr_t) src1->data % 4 || (uintptr_t) dst->data % 4) return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat: F32 tensors must be 4-byte aligned");

    mm_args a = {};
    a.w = (const char *) src0->data; a.x = (const char *) src1->data; a.dst = (char *) dst->data;
    a.K = src0->ne[0]; a.M = src0->ne[1]; a.N = src1->ne[1];
    a.nb01 = src0->nb[1]; a.nb02 = src0->nb[2]; a.nb03 = src0->nb[3];
    a.nb11 = src1->nb[1]; a.nb12 = src1->nb[2]; a.nb13 = src1->nb[3];
    a.nb1 = dst->nb[1]; a.nb2 = dst->nb[2]; a.nb3 = dst->nb[3];
    a.ne12 = (int) src1->ne[2];
    a.r2 = (int) (src1->ne[2] / src0->ne[2]); a.r3 = (int) (src1->ne[3] / src0->ne[3]);
    a.rows_wg   = 16;
    a.w2        = nullptr;
    a.w_aligned = ((uintptr_t) src0->data % 4 == 0) && src0->nb[1] % 4 == 0 && src0->nb[2] % 4 == 0 && src0->nb[3] % 4 == 0;
    a.x_aligned = ((uintptr_t) src1->data % 16 == 0) && src1->nb[1] % 16 == 0 && src1->nb[2] % 16 == 0 && src1->nb[3] % 16 == 0;
    const int nbatch = (int) (src1->ne[2] * src1->ne[3]);
    hipStream_t st = (hipStream_t) stream;

    (void) take_ws_status();
    switch (src0->type) {
        case VX_TYPE_Q8_0:
            if (act_mode == VX_ACT_Q8) launch<WT_Q8, true>(a, nbatch, st);
            else                       launch<WT_Q8, false>(a, nbatch, st);
            break;
        case VX_TYPE_F16: launch<WT_F16, false>(a, nbatch, st); break;
        default:          launch<WT_F32, false>(a, nbatch, st); break;
    }
    if (ws_failed()) return take_ws_status();
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// MUL_MAT(gate) , MUL_MAT(up) , GLU(SWIGLU split) as one launch for decode-sized token counts
// (MiniCPMModel::mlp_forward, src/minicpm.cpp:718-747).  Both products are formed exactly as vx_mul_mat
// forms them (same block order, same reduction order), so the result equals the three separate nodes'.
extern "C" int vx_supports_mul_mat_swiglu(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst) {
    if (!vx_supports_mul_mat(gate, src1, dst) || !up) return 0;
    if (gate->type != VX_TYPE_Q8_0 && gate->type != VX_TYPE_F16) return 0;
    if (up->type != gate->type) return 0;
    for (int i = 0; i < 4; ++i) if (up->ne[i] != gate->ne[i] || up->nb[i] != gate->nb[i]) return 0;
    return gemv_shape_ok(src1->ne[1], 2 * gate->ne[1], gate->ne[0]);
}

// Prefill sizes: both products on the LDS-tiled kernel, the GLU in its epilogue (f16 activations only: under VX_ACT_Q8
// the tiled products run on other kernels, and the node-by-node sequence stays).
static bool gemm_lds_swiglu_ok(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst, int act_mode) {
    if (act_mode != VX_ACT_FLOAT || gemm_lds_mode() == 0) return false;
    const int64_t K = gate->ne[0], M = gate->ne[1], N = src1->ne[1], nbatch = src1->ne[2] * src1->ne[3];
    if (K % (32 * GL_KC) || N < 64 || K >= (1ll << 28)) return false;
    auto al = [](const vx_tensor * t, uint64_t m) { return (uintptr_t) t->data % m == 0 && t->nb[1] % m == 0 && t->nb[2] % m == 0 && t->nb[3] % m == 0; };
    if (!al(src1, 16)) return false;
    const uint64_t wm = gate->type == VX_TYPE_Q8_0 ? 4 : 16;
    if (!al(gate, wm) || !al(up, wm)) return false;
    if ((uint64_t) M * gate->nb[1] >= (1ull << 32) || (uint64_t) 256 * src1->nb[1] + 256 >= (1ull << 32) || (uint64_t) 256 * dst->nb[1] + 1024 >= (1ull << 32)) return false;
    // (each product on its own must be one that the tiled kernel walks with its K whole: a cut K is summed in another order)
    return ((M + 63) / 64) * ((N + 63) / 64) * nbatch >= 64 && gemm_lds_cut(M, N, K, nbatch) == 1;
}

extern "C" int vx_supports_mul_mat_swiglu_tiled(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst, int act_mode) {
    if (!vx_supports_mul_mat(gate, src1, dst) || !up) return 0;
    if (gate->type != VX_TYPE_Q8_0 && gate->type != VX_TYPE_F16) return 0;
    if (up->type != gate->type) return 0;
    for (int i = 0; i < 4; ++i) if (up->ne[i] != gate->ne[i] || up->nb[i] != gate->nb[i]) return 0;
    // (neither the pair nor one product on its own may be a shape of the streaming kernel: it sums the K blocks in another order)
    return !gemv_shape_ok(src1->ne[1], 2 * gate->ne[1], gate->ne[0]) && !gemv_shape_ok(src1->ne[1], gate->ne[1], gate->ne[0]) &&
           gemm_lds_swiglu_ok(gate, up, src1, dst, act_mode);
}

// whether the activations of a streaming-kernel launch can be normalised on the fly: rows of at most 1024
// floats (the RMS_NORM kernel's wave-per-row regime), everything 16-byte aligned, one F32 weight row
static bool norm_prologue_ok(const vx_tensor * x, const vx_tensor * norm_w) {
    if (!norm_w || norm_w->type != VX_TYPE_F32 || norm_w->nb[0] != 4) return false;
    if (norm_w->ne[0] != x->ne[0] || norm_w->ne[1] != 1 || norm_w->ne[2] != 1 || norm_w->ne[3] != 1) return false;
    if (x->ne[0] > 1024 || x->ne[0] % 8) return false;
    return x->nb[1] % 16 == 0 && x->nb[2] % 16 == 0 && x->nb[3] % 16 == 0;
}

static vx_status swiglu_run(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * norm_w, float eps,
                            const vx_tensor * dst, int act_mode, vx_stream stream);

extern "C" vx_status vx_mul_mat_swiglu(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * dst,
                                       int act_mode, vx_stream stream) {
    return swiglu_run(gate, up, src1, nullptr, 0.0f, dst, act_mode, stream);
}

// RMS_NORM , MUL(norm weight) , MUL_MAT(gate) , MUL_MAT(up) , GLU(SWIGLU): mlp_forward behind its rms_norm
// (src/minicpm.cpp:572-580, 718-747) as one launch; x is the un-normalised hidden state.
static void swiglu_fill(mm_args & a, const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * norm_w, float eps,
                        const vx_tensor * dst) {
    a.w = (const char *) gate->data; a.x = (const char *) src1->data; a.dst = (char *) dst->data;
    a.K = gate->ne[0]; a.M = gate->ne[1]; a.N = src1->ne[1];
    a.nb01 = gate->nb[1]; a.nb02 = gate->nb[2]; a.nb03 = gate->nb[3];
    a.nb11 = src1->nb[1]; a.nb12 = src1->nb[2]; a.nb13 = src1->nb[3];
    a.nb1 = dst->nb[1]; a.nb2 = dst->nb[2]; a.nb3 = dst->nb[3];
    a.ne12 = (int) src1->ne[2];
    a.r2 = (int) (src1->ne[2] / gate->ne[2]); a.r3 = (int) (src1->ne[3] / gate->ne[3]);
    a.rows_wg   = 16;
    a.w2        = (const char *) up->data;
    a.norm_w    = norm_w ? (const float *) norm_w->data : nullptr;
    a.norm_eps  = eps;
    a.w_aligned = (((uintptr_t) gate->data | (uintptr_t) up->data) % 4 == 0) && gate->nb[1] % 4 == 0 && gate->nb[2] % 4 == 0 && gate->nb[3] % 4 == 0;
    a.x_aligned = ((uintptr_t) src1->data % 16 == 0) && src1->nb[1] % 16 == 0 && src1->nb[2] % 16 == 0 && src1->nb[3] % 16 == 0;
}

// The same at prefill sizes: the pair on the pre-tiled kernel (vx_supports_mul_mat_swiglu_tiled, Q8_0 weights, a shape that
// kernel takes), the norm in its activation pass.
static bool norm_swiglu_tiled_ok(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate, const vx_tensor * up, const vx_tensor * dst,
                                 int act_mode) {
    if (!gate || gate->type != VX_TYPE_Q8_0 || !norm_prologue_ok(x, norm_w) || !norm_w->data || (uintptr_t) norm_w->data % 16 || !x->data ||
        (uintptr_t) x->data % 16) return false;
    if (!vx_supports_mul_mat_swiglu_tiled(gate, up, x, dst, act_mode)) return false;
    mm_args a = {};
    swiglu_fill(a, gate, up, x, norm_w, 0.0f, dst);
    return gemm_q8t_takes(a, (int) (x->ne[2] * x->ne[3]), true);
}
extern "C" int vx_supports_norm_mul_mat_swiglu_tiled(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate, const vx_tensor * up,
                                                     const vx_tensor * dst, int act_mode) {
    return x && norm_w && up && dst && norm_swiglu_tiled_ok(x, norm_w, gate, up, dst, act_mode);
}

extern "C" int vx_supports_norm_mul_mat_swiglu(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate, const vx_tensor * up,
                                               const vx_tensor * dst) {
    return vx_supports_mul_mat_swiglu(gate, up, x, dst) && norm_prologue_ok(x, norm_w);
}

extern "C" vx_status vx_norm_mul_mat_swiglu(const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * gate,
                                            const vx_tensor * up, const vx_tensor * dst, int act_mode, vx_stream stream) {
    if (!x || !norm_w || !gate || !up || !dst || !norm_w->data) return vx_fail(VX_ERR_INVALID, "norm_mul_mat_swiglu: null tensor");
    if ((!vx_supports_norm_mul_mat_swiglu(x, norm_w, gate, up, dst) && !norm_swiglu_tiled_ok(x, norm_w, gate, up, dst, act_mode)) ||
        (uintptr_t) x->data % 16 || (uintptr_t) norm_w->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "norm_mul_mat_swiglu: as mul_mat_swiglu, with 16-byte aligned rows of at most 1024 floats and one F32 norm weight row");
    if (!(eps >= 0.0f)) return vx_fail(VX_ERR_INVALID, "norm_mul_mat_swiglu: eps must be >= 0");
    return swiglu_run(gate, up, x, norm_w, eps, dst, act_mode, stream);
}

static vx_status swiglu_run(const vx_tensor * gate, const vx_tensor * up, const vx_tensor * src1, const vx_tensor * norm_w, float eps,
                            const vx_tensor * dst, int act_mode, vx_stream stream) {
    if (!gate || !up || !src1 || !dst || !gate->data || !up->data || !src1->data || !dst->data)
        return vx_fail(VX_ERR_INVALID, "mul_mat_swiglu: null tensor");
    if (act_mode != VX_ACT_FLOAT && act_mode != VX_ACT_Q8) return vx_fail(VX_ERR_INVALID, "mul_mat_swiglu: bad act_mode");
    const bool tiled = norm_w ? norm_swiglu_tiled_ok(src1, norm_w, gate, up, dst, act_mode) : vx_supports_mul_mat_swiglu_tiled(gate, up, src1, dst, act_mode) != 0;
    if (!tiled && !vx_supports_mul_mat_swiglu(gate, up, src1, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat_swiglu: two Q8_0/F16 matrices of one layout, a token count the streaming kernel takes "
                       "(or, with f16 activations, 64 tokens or more for the tiled kernel: vx_supports_mul_mat_swiglu_tiled)");
    if ((uintptr_t) src1->data % 4 || (uintptr_t) dst->data % 4 || (gate->type == VX_TYPE_F16 && (((uintptr_t) gate->data | (uintptr_t) up->data) % 2)))
        return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat_swiglu: misaligned tensor data");
    mm_args a = {};
    swiglu_fill(a, gate, up, src1, norm_w, eps, dst);
    const int nbatch = (int) (src1->ne[2] * src1->ne[3]);
    hipStream_t st = (hipStream_t) stream;
    bool ok;
    (void) take_ws_status();
    if (tiled)                           ok = gate->type == VX_TYPE_Q8_0 ? launch_gemm_lds_swiglu<WT_Q8>(a, nbatch, st) : launch_gemm_lds_swiglu<WT_F16>(a, nbatch, st);
    else if (gate->type == VX_TYPE_Q8_0) ok = act_mode == VX_ACT_Q8 ? launch_gemv<WT_Q8, true>(a, nbatch, st) : launch_gemv<WT_Q8, false>(a, nbatch, st);
    else                                 ok = launch_gemv<WT_F16, false>(a, nbatch, st);
    if (ws_failed()) return take_ws_status(); // (the pre-tiled kernel's workspace: never answered by another kernel)
    if (!ok) return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat_swiglu: shape outside the streaming and the tiled kernel");
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// MUL_MAT , SCALE , ADD as one launch for decode-sized token counts: dst = residual + scale * (W x)
// (MiniCPMModel::layer_forward's residual updates, src/minicpm.cpp:749-786).  The product is formed
// exactly as vx_mul_mat forms it and then rounded, scaled and added as the two separate nodes would.
extern "C" int vx_supports_mul_mat_scale_add(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * residual, const vx_tensor * dst) {
    if (!vx_supports_mul_mat(src0, src1, dst) || !residual) return 0;
    if (src0->type != VX_TYPE_Q8_0 && src0->type != VX_TYPE_F16) return 0;
    if (residual->type != VX_TYPE_F32 || residual->ne[0] != dst->ne[0] || residual->nb[0] != 4) return 0;
    // dst's shape, or one row / one matrix repeated over it (a bias: ggml_add repeats src1)
    for (int i = 1; i < 4; ++i) if (residual->ne[i] != dst->ne[i] && residual->ne[i] != 1) return 0;
    if (residual->nb[1] % 4 || residual->nb[2] % 4 || residual->nb[3] % 4) return 0;
    if (gemv_shape_ok(src1->ne[1], src0->ne[1], src0->ne[0])) return 1;
    // a long K over few tiles (the down-projection of a hundred tokens): the product's K range is cut across work-groups
    // and the kernel that adds the partials applies the update
    const int64_t M = src0->ne[1], K = src0->ne[0], N = src1->ne[1], nbatch = src1->ne[2] * src1->ne[3];
    if (N >= 64 && K >= 2048 && K % 128 == 0 && M % 4 == 0 && ((M + 63) / 64) * ((N + 63) / 64) * nbatch < 64 && nbatch * 16 <= 65535 &&
        (uintptr_t) dst->data % 16 == 0 && dst->nb[1] % 16 == 0 && dst->nb[2] % 16 == 0 && dst->nb[3] % 16 == 0) return 1;
    // prefill sizes: the LDS-tiled kernels apply the update as they store; a shape or activation mode that they do not
    // take gets the plain product and a second pass over dst, which must then be dense
    return N > 16 && M % 4 == 0 && (uintptr_t) dst->data % 16 == 0 && dst->nb[1] == (uint64_t) M * 4 &&
           (dst->ne[2] == 1 || dst->nb[2] == dst->nb[1] * (uint64_t) N) && (dst->ne[3] == 1 || dst->nb[3] == dst->nb[1] * (uint64_t) N * (uint64_t) dst->ne[2]);
}

extern "C" vx_status vx_mul_mat_scale_add(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * residual, const vx_tensor * dst,
                                          float scale, int act_mode, vx_stream stream) {
    if (!src0 || !src1 || !residual || !dst || !src0->data || !src1->data || !residual->data || !dst->data)
        return vx_fail(VX_ERR_INVALID, "mul_mat_scale_add: null tensor");
    if (!vx_supports_mul_mat_scale_add(src0, src1, residual, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat_scale_add: Q8_0/F16 weights, a token count the streaming kernel takes, F32 residual of dst's shape");
    if (act_mode != VX_ACT_FLOAT && act_mode != VX_ACT_Q8) return vx_fail(VX_ERR_INVALID, "mul_mat_scale_add: bad act_mode");
    if ((uintptr_t) src1->data % 4 || (uintptr_t) dst->data % 4 || (uintptr_t) residual->data % 4 || (src0->type == VX_TYPE_F16 && (uintptr_t) src0->data % 2))
        return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat_scale_add: misaligned tensor data");
    mm_args a = {};
    a.w = (const char *) src0->data; a.x = (const char *) src1->data; a.dst = (char *) dst->data;
    a.K = src0->ne[0]; a.M = src0->ne[1]; a.N = src1->ne[1];
    a.nb01 = src0->nb[1]; a.nb02 = src0->nb[2]; a.nb03 = src0->nb[3];
    a.nb11 = src1->nb[1]; a.nb12 = src1->nb[2]; a.nb13 = src1->nb[3];
    a.nb1 = dst->nb[1]; a.nb2 = dst->nb[2]; a.nb3 = dst->nb[3];
    a.ne12 = (int) src1->ne[2];
    a.r2 = (int) (src1->ne[2] / src0->ne[2]); a.r3 = (int) (src1->ne[3] / src0->ne[3]);
    a.rows_wg   = 16;
    a.res       = (const char *) residual->data;
    // a repeated dim of the residual (a bias row) is walked with stride 0
    a.rnb1 = residual->ne[1] == dst->ne[1] ? residual->nb[1] : 0;
    a.rnb2 = residual->ne[2] == dst->ne[2] ? residual->nb[2] : 0;
    a.rnb3 = residual->ne[3] == dst->ne[3] ? residual->nb[3] : 0;
    a.res_scale = scale;
    a.w_aligned = ((uintptr_t) src0->data % 4 == 0) && src0->nb[1] % 4 == 0 && src0->nb[2] % 4 == 0 && src0->nb[3] % 4 == 0;
    a.x_aligned = ((uintptr_t) src1->data % 16 == 0) && src1->nb[1] % 16 == 0 && src1->nb[2] % 16 == 0 && src1->nb[3] % 16 == 0;
    const int nbatch = (int) (src1->ne[2] * src1->ne[3]);
    hipStream_t st = (hipStream_t) stream;
    bool ok;
    (void) take_ws_status();
    if (src0->type == VX_TYPE_Q8_0) ok = act_mode == VX_ACT_Q8 ? launch_gemv<WT_Q8, true>(a, nbatch, st) : launch_gemv<WT_Q8, false>(a, nbatch, st);
    else                            ok = launch_gemv<WT_F16, false>(a, nbatch, st);
    if (!ok) { // not the streaming kernel's shape: the tiled kernels with K cut (see vx_supports_mul_mat_scale_add)
        if (src0->type == VX_TYPE_Q8_0) {
            if (act_mode == VX_ACT_Q8) ok = launch_mm_cut<WT_Q8, true>(a, nbatch, st);
            else                       ok = launch_gemm_lds<WT_Q8>(a, nbatch, st) || (!ws_failed() && launch_mm_cut<WT_Q8, false>(a, nbatch, st));
        } else {
            ok = launch_gemm_lds<WT_F16>(a, nbatch, st) || (!ws_failed() && launch_mm_cut<WT_F16, false>(a, nbatch, st));
        }
        if (ws_failed()) return take_ws_status();
    }
    if (!ok) { // the plain product, then the update in a pass of its own (dense dst: checked by vx_supports_mul_mat_scale_add)
        const size_t bytes = (size_t) nbatch * a.N * a.M * sizeof(float);
        const char * r0 = (const char *) residual->data, * d0 = (const char *) dst->data;
        const size_t rbytes = (size_t) ((residual->ne[1] - 1) * residual->nb[1] + (residual->ne[2] - 1) * residual->nb[2] + (residual->ne[3] - 1) * residual->nb[3]) +
                              (size_t) residual->ne[0] * 4;
        void * product = dst->data;
        if (r0 < d0 + bytes && d0 < r0 + rbytes) { // the residual is (in) dst: the product needs a place of its own
            const vx_status rc = vx_workspace(st, bytes, &product);
            if (rc != VX_OK) return rc;
        }
        mm_args p = a;
        p.res = nullptr; p.dst = (char *) product;
        // (a cut of this product puts its partials behind the product when that lies in the workspace; if the request
        // grows the workspace, the block with the product stays valid: retired blocks live as long as the stream)
        if (product != dst->data) p.ws_offset = (bytes + 255) & ~(size_t) 255;
        p.nb1 = (uint64_t) a.M * 4; p.nb2 = p.nb1 * (uint64_t) a.N; p.nb3 = p.nb2 * (uint64_t) a.ne12;
        if (src0->type == VX_TYPE_Q8_0) { if (act_mode == VX_ACT_Q8) launch<WT_Q8, true>(p, nbatch, st); else launch<WT_Q8, false>(p, nbatch, st); }
        else                            launch<WT_F16, false>(p, nbatch, st);
        if (ws_failed()) return take_ws_status();
        mm_args b = a;
        b.ksplit = 1; b.partial = (float *) product;
        const int64_t units = a.N * (a.M / 4);
        if ((units + 255) / 256 > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "mul_mat_scale_add: launch too large");
        vx_launch(mm_splitk_reduce_kernel, dim3((unsigned) ((units + 255) / 256), 1, (unsigned) nbatch), dim3(256), 0, st, b);
    }
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// mlp_forward and the residual update behind it at prefill sizes (src/minicpm.cpp:718-747, 775-786): RMS_NORM, MUL, gate, up,
// SwiGLU, down, SCALE, ADD.  Three launches on the pre-tiled kernel: the activation pass with the norm, the gate/up pair
// whose epilogue writes silu(g) * u as f16 tiles, and the down projection that takes those tiles as they are, with the
// update in its epilogue.  The intermediate [tokens x ffn] tensor is neither stored in fp32 nor read back and re-laid-out
// (at 65536 tokens x 4096: a gigabyte each way).  Every value is rounded where the separate calls round it: same bits.
static bool mlp_fill(mm_args & a, mm_args & b, const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * gate, const vx_tensor * up,
                     const vx_tensor * down, const vx_tensor * residual, float scale, const vx_tensor * dst, int act_mode) {
    if (!x || !norm_w || !gate || !up || !down || !residual || !dst) return false;
    if (down->type != VX_TYPE_Q8_0 || down->ne[2] != 1 || down->ne[3] != 1 || gate->ne[2] != 1 || gate->ne[3] != 1) return false;
    if (down->ne[0] != gate->ne[1] || gate->ne[1] % 32 || dst->ne[0] != down->ne[1] || dst->ne[1] != x->ne[1] || dst->ne[2] != x->ne[2] || dst->ne[3] != x->ne[3]) return false;
    if (dst->type != VX_TYPE_F32 || dst->nb[0] != 4 || residual->type != VX_TYPE_F32 || residual->nb[0] != 4 || !vx_same_shape(residual, dst)) return false;
    // the intermediate as the separate calls would see it: dense [ffn, tokens, batch]
    vx_tensor act = *dst;
    act.ne[0] = gate->ne[1];
    act.nb[1] = (uint64_t) act.ne[0] * 4; act.nb[2] = act.nb[1] * (uint64_t) act.ne[1]; act.nb[3] = act.nb[2] * (uint64_t) act.ne[2];
    act.data = x->data; // (only its alignment is looked at)
    if (!norm_swiglu_tiled_ok(x, norm_w, gate, up, &act, act_mode)) return false;
    if (!vx_supports_mul_mat_scale_add(down, &act, residual, dst)) return false;
    swiglu_fill(a, gate, up, x, norm_w, eps, &act);
    b = mm_args{};
    b.w = (const char *) down->data; b.x = (const char *) x->data; b.dst = (char *) dst->data;
    b.K = down->ne[0]; b.M = down->ne[1]; b.N = x->ne[1];
    b.nb01 = down->nb[1]; b.nb02 = down->nb[2]; b.nb03 = down->nb[3];
    b.nb11 = act.nb[1]; b.nb12 = act.nb[2]; b.nb13 = act.nb[3];
    b.nb1 = dst->nb[1]; b.nb2 = dst->nb[2]; b.nb3 = dst->nb[3];
    b.ne12 = (int) x->ne[2];
    b.r2 = (int) x->ne[2]; b.r3 = (int) x->ne[3];
    b.rows_wg = 16;
    b.res = (const char *) residual->data;
    b.rnb1 = residual->nb[1]; b.rnb2 = residual->nb[2]; b.rnb3 = residual->nb[3];
    b.res_scale = scale;
    b.w_aligned = ((uintptr_t) down->data % 4 == 0) && down->nb[1] % 4 == 0;
    b.x_aligned = 1;
    const int nbatch = (int) (x->ne[2] * x->ne[3]);
    // both products on the pre-tiled kernel, as the separate calls would run them
    return gemm_lds_mode() != 0 && b.w_aligned && (uintptr_t) dst->data % 4 == 0 && (uintptr_t) residual->data % 4 == 0 &&
           gemm_q8t_takes(a, nbatch, true) && gemm_q8t_takes(b, nbatch, false) && (uint64_t) 256 * b.rnb1 + 1024 < (1ull << 32);
}

extern "C" int vx_supports_mlp_tiled(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * gate, const vx_tensor * up, const vx_tensor * down,
                                     const vx_tensor * residual, const vx_tensor * dst, int act_mode) {
    mm_args a = {}, b = {};
    return mlp_fill(a, b, x, norm_w, 0.0f, gate, up, down, residual, 0.0f, dst, act_mode);
}

extern "C" vx_status vx_mlp_tiled(const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * gate, const vx_tensor * up,
                                  const vx_tensor * down, const vx_tensor * residual, float scale, const vx_tensor * dst, int act_mode, vx_stream stream) {
    mm_args a = {}, b = {};
    if (!mlp_fill(a, b, x, norm_w, eps, gate, up, down, residual, scale, dst, act_mode))
        return vx_fail(VX_ERR_UNSUPPORTED, "mlp_tiled: the shapes of vx_supports_norm_mul_mat_swiglu_tiled, a Q8_0 down projection that the pre-tiled kernel takes, "
                       "an F32 residual of dst's shape");
    if (!x->data || !norm_w->data || !gate->data || !up->data || !down->data || !residual->data || !dst->data) return vx_fail(VX_ERR_INVALID, "mlp_tiled: null data");
    if (!(eps >= 0.0f)) return vx_fail(VX_ERR_INVALID, "mlp_tiled: eps must be >= 0");
    const int nbatch = (int) (x->ne[2] * x->ne[3]);
    hipStream_t st = (hipStream_t) stream;
    // the tiles between the two products: whole 128-token tiles of the pair (it writes every token of its tiles), at the front of
    // the workspace; both products put what they need behind them (a block that a later, larger request replaces stays valid)
    const int    tile_tt = (int) ((a.N + QT_TOKS - 1) / QT_TOKS) * (QT_TOKS / 16);
    const size_t tiles   = ((size_t) nbatch * (size_t) (a.M / 32) * (size_t) tile_tt * 1024 + 255) & ~(size_t) 255;
    void * ws = nullptr;
    (void) take_ws_status();
    const vx_status rc = vx_workspace(st, tiles, &ws);
    if (rc != VX_OK) return rc;
    a.ws_offset = tiles; a.tile_out = ws; a.tile_tt = tile_tt;
    b.ws_offset = tiles; b.tile_in = ws;  b.tile_tt = tile_tt;
    const bool fold = gemm_lds_mode() == 2;
    if (!launch_gemm_q8t<true>(a, nbatch, st, fold)) return ws_failed() ? take_ws_status() : vx_fail(VX_ERR_UNSUPPORTED, "mlp_tiled: the gate/up product could not be launched");
    if (!launch_gemm_q8t<false>(b, nbatch, st, fold)) return ws_failed() ? take_ws_status() : vx_fail(VX_ERR_UNSUPPORTED, "mlp_tiled: the down projection could not be launched");
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// A projection with its residual update whose activations a kernel in front of it (the prefill attention's epilogue) has
// left as this kernel's f16 tiles: vx_mul_mat_scale_add without its activation pass.  Taken where the separate call runs
// on the pre-tiled kernel, so the bits are the same.
static bool proj_tiles_fill(mm_args & b, const vx_tensor * w, const vx_tensor * x, const vx_tensor * residual, const vx_tensor * dst, float scale, int act_mode) {
    if (!w || !x || !residual || !dst || act_mode != VX_ACT_FLOAT || gemm_lds_mode() == 0) return false;
    if (w->type != VX_TYPE_Q8_0 || w->ne[2] != 1 || w->ne[3] != 1 || x->type != VX_TYPE_F32 || !vx_is_contiguous(x)) return false;
    if (!vx_supports_mul_mat_scale_add(w, x, residual, dst) || !vx_same_shape(residual, dst) || residual->nb[0] != 4 || dst->nb[0] != 4) return false;
    b = mm_args{};
    b.w = (const char *) w->data; b.x = (const char *) x->data; b.dst = (char *) dst->data;
    b.K = w->ne[0]; b.M = w->ne[1]; b.N = x->ne[1];
    b.nb01 = w->nb[1]; b.nb02 = w->nb[2]; b.nb03 = w->nb[3];
    b.nb11 = x->nb[1]; b.nb12 = x->nb[2]; b.nb13 = x->nb[3];
    b.nb1 = dst->nb[1]; b.nb2 = dst->nb[2]; b.nb3 = dst->nb[3];
    b.ne12 = (int) x->ne[2];
    b.r2 = (int) x->ne[2]; b.r3 = (int) x->ne[3];
    b.rows_wg = 16;
    b.res = (const char *) residual->data;
    b.rnb1 = residual->nb[1]; b.rnb2 = residual->nb[2]; b.rnb3 = residual->nb[3];
    b.res_scale = scale;
    b.w_aligned = ((uintptr_t) w->data % 4 == 0) && w->nb[1] % 4 == 0;
    b.x_aligned = ((uintptr_t) x->data % 16 == 0) && x->nb[1] % 16 == 0 && x->nb[2] % 16 == 0 && x->nb[3] % 16 == 0;
    const int64_t nbatch = x->ne[2] * x->ne[3];
    // (what launch_gemm_lds asks for before it hands a product to the pre-tiled kernel)
    if ((uint64_t) b.M * b.nb01 >= (1ull << 32) || (uint64_t) 256 * b.nb11 + 256 >= (1ull << 32) || (uint64_t) 256 * b.nb1 + 1024 >= (1ull << 32) ||
        b.K >= (1ll << 28) || b.N <= 16) return false;
    return b.w_aligned && b.x_aligned && nbatch <= 65535 && (uintptr_t) dst->data % 4 == 0 && (uintptr_t) residual->data % 4 == 0 &&
           !gemv_shape_ok(b.N, b.M, b.K) && b.K % (32 * GL_KC) == 0 && gemm_q8t_takes(b, (int) nbatch, false) &&
           (uint64_t) 256 * b.rnb1 + 1024 < (1ull << 32);
}

bool vx_proj_tiles_ok(const vx_tensor * w, const vx_tensor * x, const vx_tensor * residual, const vx_tensor * dst, int act_mode,
                      uint32_t * tile_tt, uint32_t * n_kb, size_t * tile_bytes, size_t * own_bytes) {
    mm_args b;
    if (!proj_tiles_fill(b, w, x, residual, dst, 0.0f, act_mode)) return false;
    {   // what the product itself puts behind the tiles when the weights' tiles are not kept: as launch_gemm_q8t sizes them
        const size_t kb = (size_t) (b.K / 32), rt = (size_t) ((b.M + 15) / 16);
        *own_bytes = kb * rt * 1024 + (kb * ((rt + 3) & ~(size_t) 3) * 16 * 4 + 1023) / 1024 * 1024 + 1024;
    }
    const int64_t tt = (b.N + QT_TOKS - 1) / QT_TOKS * (QT_TOKS / 16), nbatch = x->ne[2] * x->ne[3];
    if (tt * (b.K / 32) * nbatch >= ((int64_t) 1 << 31)) return false;
    *tile_tt = (uint32_t) tt; *n_kb = (uint32_t) (b.K / 32);
    *tile_bytes = ((size_t) nbatch * (size_t) (b.K / 32) * (size_t) tt * 1024 + 255) & ~(size_t) 255;
    return true;
}

vx_status vx_proj_tiles_run(const vx_tensor * w, const vx_tensor * x, const vx_tensor * residual, const vx_tensor * dst, float scale,
                            int act_mode, const void * tiles, size_t ws_offset, hipStream_t st) {
    mm_args b;
    if (!proj_tiles_fill(b, w, x, residual, dst, scale, act_mode)) return vx_fail(VX_ERR_UNSUPPORTED, "projection over tiles: a shape outside the pre-tiled kernel");
    if (!w->data || !residual->data || !dst->data || !tiles) return vx_fail(VX_ERR_INVALID, "projection over tiles: null data");
    b.ws_offset = ws_offset; b.tile_in = tiles; b.tile_tt = (int) ((b.N + QT_TOKS - 1) / QT_TOKS * (QT_TOKS / 16));
    (void) take_ws_status();
    if (!launch_gemm_q8t<false>(b, (int) (x->ne[2] * x->ne[3]), st, gemm_lds_mode() == 2))
        return ws_failed() ? take_ws_status() : vx_fail(VX_ERR_UNSUPPORTED, "projection over tiles: the product could not be launched");
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// The Q, K and V projections of one attention block with the NEOX rotation of Q and K, one launch:
//   MUL_MAT(wq, x) RESHAPE ROPE , MUL_MAT(wk, x) RESHAPE ROPE , MUL_MAT(wv, x)
// (MiniCPMModel::attention_forward, src/minicpm.cpp:640-680).  q_dst and k_dst are the ROPE nodes'
// outputs [head_dim, heads, tokens, batch], v_dst is the third MUL_MAT's [rows, tokens, 1, batch]
// (or, like x, with the batch flattened into the token dimension).
// Every product is formed as vx_mul_mat forms it and rotated with vx_rope's arithmetic.
static bool qkv_rope_dst_ok(const vx_tensor * w, const vx_tensor * x, const vx_tensor * dst, int head_dim) {
    if (!dst || dst->type != VX_TYPE_F32 || !vx_is_contiguous(dst)) return false;
    if (dst->ne[0] != head_dim || dst->ne[0] * dst->ne[1] != w->ne[1]) return false;
    // x is [K, tokens, 1, batch] or, with every sequence's tokens flattened into dim 1, [K, tokens * batch, 1, 1]
    if (x->ne[3] == 1) return dst->ne[2] * dst->ne[3] == x->ne[1];
    return dst->ne[2] == x->ne[1] && dst->ne[3] == x->ne[3];
}

extern "C" int vx_supports_qkv_proj_rope(const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x,
                                         const vx_tensor * q_dst, const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode) {
    if (!wq || !wk || !wv || !x || !q_dst || !k_dst || !v_dst) return 0;
    if (wq->type != VX_TYPE_Q8_0 && wq->type != VX_TYPE_F16) return 0;
    const vx_tensor * ws[3] = { wq, wk, wv };
    for (const vx_tensor * w : ws) {
        if (w->type != wq->type || w->ne[0] != wq->ne[0] || w->ne[2] != 1 || w->ne[3] != 1 || !vx_positive(w)) return 0;
        if (w->nb[0] != vx_type_size(w->type) || w->nb[1] < vx_row_size(w->type, w->ne[0])) return 0;
        if (w->type == VX_TYPE_F16 && w->nb[1] % 2) return 0;
    }
    if (x->type != VX_TYPE_F32 || !vx_positive(x) || x->ne[0] != wq->ne[0] || x->ne[2] != 1 || x->nb[0] != 4) return 0;
    if (x->nb[1] % 4 || x->nb[3] % 4 || x->ne[3] > 65535) return 0;
    if (wq->ne[0] % 32 || wq->ne[0] < 32) return 0;
    if (mode != 2 || n_dims <= 0 || n_dims % 16) return 0; // NEOX over the whole head; pairs split evenly over work-groups
    if (!qkv_rope_dst_ok(wq, x, q_dst, n_dims) || !qkv_rope_dst_ok(wk, x, k_dst, n_dims)) return 0;
    // v_dst may be a row range of a wider tensor (the v rows of one fused q/k/v product): dense rows, any row stride
    if (v_dst->type != VX_TYPE_F32 || v_dst->nb[0] != 4 || v_dst->nb[1] % 4 || v_dst->nb[3] % 4) return 0;
    if (v_dst->nb[1] < (uint64_t) v_dst->ne[0] * 4 || (v_dst->ne[3] > 1 && v_dst->nb[3] < v_dst->nb[1] * (uint64_t) v_dst->ne[1])) return 0;
    if (v_dst->ne[0] != wv->ne[1] || v_dst->ne[1] != x->ne[1] || v_dst->ne[2] != 1 || v_dst->ne[3] != x->ne[3]) return 0;
    {
        const int64_t tokens = x->ne[1] * x->ne[2] * x->ne[3];
        const int nw = gemv_waves_for(wq->ne[0], tokens, wq->ne[1]);
        if (gemv_waves_for(wq->ne[0], tokens, wk->ne[1]) != nw || gemv_waves_for(wq->ne[0], tokens, wv->ne[1]) != nw) return 0;
    }
    return gemv_shape_ok(x->ne[1], wq->ne[1], wq->ne[0]) && gemv_shape_ok(x->ne[1], wk->ne[1], wq->ne[0]) && gemv_shape_ok(x->ne[1], wv->ne[1], wq->ne[0]);
}

// The order in which vx_mul_mat (and every group built on it) sums the K blocks of a product, as an opaque number: two
// products with equal K, token count of the call and number are summed identically.  It depends on the row count, so a backend
// that runs a product over a row range of a matrix in place of the product over the whole matrix (the reference's row-fused
// qkv_proj / gate_up_proj) compares the two before promising identical bits.
extern "C" int vx_mul_mat_sum_order(int64_t K, int64_t tokens, int64_t M) {
    if (K < 32 || K % 32 || tokens < 1 || M < 1) return 0;
    return gemv_waves_for(K, tokens, M);
}

static vx_status qkv_run(const vx_tensor * norm_w, float eps, const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv,
                         const vx_tensor * x, const int32_t * pos, const float * freq_factors, const vx_tensor * q_dst,
                         const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode, int n_ctx_orig, float freq_base,
                         float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow, int act_mode,
                         vx_stream stream);

// The same group at prefill sizes: RMS_NORM and the norm weight in the activation pass of the pre-tiled kernel, q, k and v
// as one virtual matrix over those tiles (one product launch instead of three, x laid out once), each stored to its own
// destination; the two rotations in the product's epilogue (heads of 64 rows) or as launches of their own, in place.  Taken when every piece is what the separate
// nodes would run -- each product on a tiled kernel with its K whole (the pre-tiled kernel and the LDS-operand kernel form
// and add a block's products identically) -- so the bits are those of RMS_NORM, MUL, three MUL_MATs and two ROPEs.
static bool qkv_tiled_fill(mm_args & a, const vx_tensor * norm_w, float eps, const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv,
                           const vx_tensor * x, const vx_tensor * q_dst, const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode, int act_mode) {
    if (!wq || !wk || !wv || !x || !norm_w || !q_dst || !k_dst || !v_dst || act_mode != VX_ACT_FLOAT || gemm_lds_mode() == 0) return false;
    const vx_tensor * ws[3] = { wq, wk, wv };
    const vx_tensor * ds[3] = { q_dst, k_dst, v_dst };
    if (!norm_prologue_ok(x, norm_w) || x->type != VX_TYPE_F32 || x->ne[2] != 1 || x->nb[0] != 4 || x->ne[3] > 65535) return false;
    if (mode != 2 || n_dims <= 0 || !qkv_rope_dst_ok(wq, x, q_dst, n_dims) || !qkv_rope_dst_ok(wk, x, k_dst, n_dims)) return false;
    if (v_dst->type != VX_TYPE_F32 || v_dst->nb[0] != 4 || v_dst->nb[1] % 4 || v_dst->nb[3] % 4 || v_dst->nb[1] < (uint64_t) v_dst->ne[0] * 4 ||
        (v_dst->ne[3] > 1 && v_dst->nb[3] < v_dst->nb[1] * (uint64_t) v_dst->ne[1])) return false;
    if (v_dst->ne[0] != wv->ne[1] || v_dst->ne[1] != x->ne[1] || v_dst->ne[2] != 1 || v_dst->ne[3] != x->ne[3]) return false;
    a = mm_args{};
    a.x = (const char *) x->data;
    a.K = wq->ne[0]; a.N = x->ne[1]; a.M = 0;
    a.nb11 = x->nb[1]; a.nb12 = x->nb[2]; a.nb13 = x->nb[3];
    a.ne12 = 1; a.r2 = 1; a.r3 = (int) x->ne[3];
    a.w_aligned = 1;
    a.nseg = 3;
    const int nbatch = (int) x->ne[3];
    for (int i = 0; i < 3; ++i) {
        const vx_tensor * w = ws[i];
        if (w->type != VX_TYPE_Q8_0 || w->ne[0] != wq->ne[0] || w->ne[2] != 1 || w->ne[3] != 1 || !vx_positive(w) || w->ne[1] % 64) return false;
        if (w->nb[0] != VX_Q8_BLOCK || w->nb[1] < vx_row_size(w->type, w->ne[0])) return false;
        gv_seg & sg = a.seg[i];
        sg.w = (const char *) w->data; sg.dst = (char *) ds[i]->data;
        sg.M = w->ne[1]; sg.nb01 = w->nb[1];
        sg.nb1 = (uint64_t) sg.M * 4; sg.nb2 = 0; sg.nb3 = (uint64_t) sg.M * 4 * x->ne[1];
        if (i == 2) { sg.nb1 = v_dst->nb[1]; sg.nb3 = v_dst->nb[3]; }
        a.w_aligned = a.w_aligned && ((uintptr_t) w->data % 4 == 0) && w->nb[1] % 4 == 0;
        a.M += sg.M;
        // the product on its own: a tiled kernel with its K whole (not the streaming kernel, no cut K, not the older kernels)
        const int64_t t64 = ((sg.M + 63) / 64) * ((a.N + 63) / 64) * nbatch;
        const bool    big = ((sg.M + 127) / 128) * ((a.N + 127) / 128) * nbatch >= 192;
        if (gemv_shape_ok(a.N, sg.M, a.K) || a.K % (32 * GL_KC) || gemm_lds_cut(sg.M, a.N, a.K, nbatch) != 1 || (!big && t64 < 64)) return false;
    }
    a.w = a.seg[0].w; a.dst = a.seg[0].dst; a.nb01 = a.seg[0].nb01; a.nb1 = a.seg[0].nb1; a.nb3 = a.seg[0].nb3;
    a.x_aligned = ((uintptr_t) x->data % 16 == 0) && x->nb[1] % 16 == 0 && x->nb[3] % 16 == 0;
    a.norm_w = (const float *) norm_w->data; a.norm_eps = eps;
    return a.w_aligned && a.x_aligned && norm_w->data && (uintptr_t) norm_w->data % 16 == 0 && gemm_q8t_takes(a, nbatch, false);
}

extern "C" int vx_supports_norm_qkv_proj_rope_tiled(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * wq, const vx_tensor * wk,
                                                    const vx_tensor * wv, const vx_tensor * q_dst, const vx_tensor * k_dst, const vx_tensor * v_dst,
                                                    int n_dims, int mode, int act_mode) {
    mm_args a;
    return qkv_tiled_fill(a, norm_w, 0.0f, wq, wk, wv, x, q_dst, k_dst, v_dst, n_dims, mode, act_mode) &&
           vx_supports_rope(q_dst, q_dst, n_dims, mode) && vx_supports_rope(k_dst, k_dst, n_dims, mode);
}

extern "C" vx_status vx_qkv_proj_rope(const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x,
                                      const int32_t * pos, const float * freq_factors, const vx_tensor * q_dst, const vx_tensor * k_dst,
                                      const vx_tensor * v_dst, int n_dims, int mode, int n_ctx_orig, float freq_base, float freq_scale,
                                      float ext_factor, float attn_factor, float beta_fast, float beta_slow, int act_mode,
                                      vx_stream stream) {
    return qkv_run(nullptr, 0.0f, wq, wk, wv, x, pos, freq_factors, q_dst, k_dst, v_dst, n_dims, mode, n_ctx_orig, freq_base, freq_scale,
                   ext_factor, attn_factor, beta_fast, beta_slow, act_mode, stream);
}

// K and V alone: MUL_MAT(wk, x) RESHAPE ROPE , MUL_MAT(wv, x).  From 449 tokens on the three-matrix launch above no longer
// applies (q's product leaves the streaming kernel there, and with it the order of its sums), but the two 128-row
// products stay on it up to 2048 tokens: one launch for the two of them and k's rotation instead of three.
extern "C" int vx_supports_kv_proj_rope(const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x, const vx_tensor * k_dst,
                                        const vx_tensor * v_dst, int n_dims, int mode) {
    if (!wk || !wv || !x || !k_dst || !v_dst) return 0;
    if (wk->type != VX_TYPE_Q8_0 && wk->type != VX_TYPE_F16) return 0;
    const vx_tensor * ws[2] = { wk, wv };
    for (const vx_tensor * w : ws) {
        if (w->type != wk->type || w->ne[0] != wk->ne[0] || w->ne[2] != 1 || w->ne[3] != 1 || !vx_positive(w)) return 0;
        if (w->nb[0] != vx_type_size(w->type) || w->nb[1] < vx_row_size(w->type, w->ne[0])) return 0;
        if (w->type == VX_TYPE_F16 && w->nb[1] % 2) return 0;
    }
    if (x->type != VX_TYPE_F32 || !vx_positive(x) || x->ne[0] != wk->ne[0] || x->ne[2] != 1 || x->nb[0] != 4) return 0;
    if (x->nb[1] % 4 || x->nb[3] % 4 || x->ne[3] > 65535) return 0;
    if (wk->ne[0] % 32 || wk->ne[0] < 32) return 0;
    if (mode != 2 || n_dims <= 0 || n_dims % 16) return 0;
    if (!qkv_rope_dst_ok(wk, x, k_dst, n_dims)) return 0;
    if (v_dst->type != VX_TYPE_F32 || v_dst->nb[0] != 4 || v_dst->nb[1] % 4 || v_dst->nb[3] % 4) return 0;
    if (v_dst->nb[1] < (uint64_t) v_dst->ne[0] * 4 || (v_dst->ne[3] > 1 && v_dst->nb[3] < v_dst->nb[1] * (uint64_t) v_dst->ne[1])) return 0;
    if (v_dst->ne[0] != wv->ne[1] || v_dst->ne[1] != x->ne[1] || v_dst->ne[2] != 1 || v_dst->ne[3] != x->ne[3]) return 0;
    const int64_t tokens = x->ne[1] * x->ne[2] * x->ne[3];
    if (gemv_waves_for(wk->ne[0], tokens, wk->ne[1]) != gemv_waves_for(wk->ne[0], tokens, wv->ne[1])) return 0;
    return gemv_shape_ok(x->ne[1], wk->ne[1], wk->ne[0]) && gemv_shape_ok(x->ne[1], wv->ne[1], wk->ne[0]);
}

extern "C" vx_status vx_kv_proj_rope(const vx_tensor * wk, const vx_tensor * wv, const vx_tensor * x, const int32_t * pos,
                                     const float * freq_factors, const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode,
                                     int n_ctx_orig, float freq_base, float freq_scale, float ext_factor, float attn_factor,
                                     float beta_fast, float beta_slow, int act_mode, vx_stream stream) {
    if (!vx_supports_kv_proj_rope(wk, wv, x, k_dst, v_dst, n_dims, mode))
        return vx_fail(VX_ERR_UNSUPPORTED, "kv_proj_rope: two Q8_0/F16 matrices over one activation tensor, a token count the streaming kernel takes, NEOX rotation over the whole head, contiguous k output");
    if (!pos || !wk->data || !wv->data || !x->data || !k_dst->data || !v_dst->data) return vx_fail(VX_ERR_INVALID, "kv_proj_rope: null data");
    if (act_mode != VX_ACT_FLOAT && act_mode != VX_ACT_Q8) return vx_fail(VX_ERR_INVALID, "kv_proj_rope: bad act_mode");
    const vx_tensor * ws[2] = { wk, wv };
    const vx_tensor * ds[2] = { k_dst, v_dst };
    if ((uintptr_t) x->data % 4) return vx_fail(VX_ERR_UNSUPPORTED, "kv_proj_rope: misaligned activations");
    mm_args a = {};
    a.x = (const char *) x->data;
    a.K = wk->ne[0]; a.N = x->ne[1];
    a.M = 0;
    a.nb11 = x->nb[1]; a.nb12 = x->nb[2]; a.nb13 = x->nb[3];
    a.ne12 = 1; a.r2 = 1; a.r3 = 1;
    a.rows_wg = 16;
    a.w_aligned = 1;
    a.nseg = 2;
    for (int i = 0; i < 2; ++i) {
        if ((uintptr_t) ds[i]->data % 4 || (ws[i]->type == VX_TYPE_F16 && (uintptr_t) ws[i]->data % 2))
            return vx_fail(VX_ERR_UNSUPPORTED, "kv_proj_rope: misaligned tensor data");
        gv_seg & sg = a.seg[i];
        sg.w = (const char *) ws[i]->data; sg.dst = (char *) ds[i]->data;
        sg.M = ws[i]->ne[1]; sg.nb01 = ws[i]->nb[1];
        sg.nb1 = (uint64_t) sg.M * 4; sg.nb2 = 0; sg.nb3 = (uint64_t) sg.M * 4 * x->ne[1];
        if (i == 1) { sg.nb1 = v_dst->nb[1]; sg.nb3 = v_dst->nb[3]; }
        sg.rope = i == 0;
        a.w_aligned = a.w_aligned && ((uintptr_t) ws[i]->data % 4 == 0) && ws[i]->nb[1] % 4 == 0;
        a.M += sg.M;
    }
    a.w = a.seg[0].w; a.dst = a.seg[0].dst;
    a.x_aligned = ((uintptr_t) x->data % 16 == 0) && x->nb[1] % 16 == 0 && x->nb[3] % 16 == 0;
    a.pos = pos; a.ff = freq_factors;
    a.rp = rope_make_params(n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    a.head_dim = n_dims;
    a.rope_T   = (int) k_dst->ne[2];
    const int nbatch = (int) x->ne[3];
    hipStream_t st = (hipStream_t) stream;
    bool ok;
    if (wk->type == VX_TYPE_Q8_0) ok = act_mode == VX_ACT_Q8 ? launch_gemv<WT_Q8, true>(a, nbatch, st) : launch_gemv<WT_Q8, false>(a, nbatch, st);
    else                          ok = launch_gemv<WT_F16, false>(a, nbatch, st);
    if (!ok) return vx_fail(VX_ERR_UNSUPPORTED, "kv_proj_rope: shape outside the streaming kernel");
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// RMS_NORM , MUL(norm weight) in front of the three projections: layer_forward's input rms_norm
// (src/minicpm.cpp:572-580, 761) joins the launch; x is the un-normalised hidden state.
extern "C" int vx_supports_norm_qkv_proj_rope(const vx_tensor * x, const vx_tensor * norm_w, const vx_tensor * wq, const vx_tensor * wk,
                                              const vx_tensor * wv, const vx_tensor * q_dst, const vx_tensor * k_dst, const vx_tensor * v_dst,
                                              int n_dims, int mode) {
    return vx_supports_qkv_proj_rope(wq, wk, wv, x, q_dst, k_dst, v_dst, n_dims, mode) && norm_prologue_ok(x, norm_w);
}

extern "C" vx_status vx_norm_qkv_proj_rope(const vx_tensor * x, const vx_tensor * norm_w, float eps, const vx_tensor * wq,
                                           const vx_tensor * wk, const vx_tensor * wv, const int32_t * pos, const float * freq_factors,
                                           const vx_tensor * q_dst, const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode,
                                           int n_ctx_orig, float freq_base, float freq_scale, float ext_factor, float attn_factor,
                                           float beta_fast, float beta_slow, int act_mode, vx_stream stream) {
    if (!x || !norm_w || !norm_w->data) return vx_fail(VX_ERR_INVALID, "norm_qkv_proj_rope: null tensor");
    if (!vx_supports_norm_qkv_proj_rope(x, norm_w, wq, wk, wv, q_dst, k_dst, v_dst, n_dims, mode) &&
        vx_supports_norm_qkv_proj_rope_tiled(x, norm_w, wq, wk, wv, q_dst, k_dst, v_dst, n_dims, mode, act_mode)) {
        // prefill sizes: the norm in the activation pass, one product launch for the three matrices, the rotations in place
        if (!pos || !x->data || !q_dst->data || !k_dst->data || !v_dst->data || !wq->data || !wk->data || !wv->data)
            return vx_fail(VX_ERR_INVALID, "norm_qkv_proj_rope: null data");
        if (!(eps >= 0.0f)) return vx_fail(VX_ERR_INVALID, "norm_qkv_proj_rope: eps must be >= 0");
        mm_args a;
        if (!qkv_tiled_fill(a, norm_w, eps, wq, wk, wv, x, q_dst, k_dst, v_dst, n_dims, mode, act_mode))
            return vx_fail(VX_ERR_UNSUPPORTED, "norm_qkv_proj_rope: shape outside the pre-tiled kernel");
        (void) take_ws_status();
        // heads of 64 rows: the rotations in the product's epilogue, from an angle table (VX_QKV_ROPE_EPILOGUE=0: as launches of their own)
        static const bool rope_apart = [] { const char * e = getenv("VX_QKV_ROPE_EPILOGUE"); return e && atoi(e) == 0; }();
        const bool in_epilogue = !rope_apart && n_dims == 64 && q_dst->ne[0] == 64 && k_dst->ne[0] == 64 && q_dst->ne[2] == k_dst->ne[2];
        if (in_epilogue) {
            a.pos = pos; a.ff = freq_factors;
            a.rp = rope_make_params(n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
            a.head_dim = 64;
            a.rope_T   = (int) q_dst->ne[2];
        }
        if (!launch_gemm_q8t<false>(a, (int) x->ne[3], (hipStream_t) stream, gemm_lds_mode() == 2))
            return ws_failed() ? take_ws_status() : vx_fail(VX_ERR_UNSUPPORTED, "norm_qkv_proj_rope: the product could not be launched");
        if (in_epilogue) return VX_OK;
        vx_status rc = vx_rope(q_dst, pos, freq_factors, q_dst, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow, stream);
        if (rc == VX_OK) rc = vx_rope(k_dst, pos, freq_factors, k_dst, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow, stream);
        return rc;
    }
    if (!vx_supports_norm_qkv_proj_rope(x, norm_w, wq, wk, wv, q_dst, k_dst, v_dst, n_dims, mode) || (uintptr_t) x->data % 16 ||
        (uintptr_t) norm_w->data % 16)
        return vx_fail(VX_ERR_UNSUPPORTED, "norm_qkv_proj_rope: as qkv_proj_rope, with 16-byte aligned rows of at most 1024 floats and one F32 norm weight row");
    if (!(eps >= 0.0f)) return vx_fail(VX_ERR_INVALID, "norm_qkv_proj_rope: eps must be >= 0");
    return qkv_run(norm_w, eps, wq, wk, wv, x, pos, freq_factors, q_dst, k_dst, v_dst, n_dims, mode, n_ctx_orig, freq_base, freq_scale,
                   ext_factor, attn_factor, beta_fast, beta_slow, act_mode, stream);
}

static vx_status qkv_run(const vx_tensor * norm_w, float eps, const vx_tensor * wq, const vx_tensor * wk, const vx_tensor * wv,
                         const vx_tensor * x, const int32_t * pos, const float * freq_factors, const vx_tensor * q_dst,
                         const vx_tensor * k_dst, const vx_tensor * v_dst, int n_dims, int mode, int n_ctx_orig, float freq_base,
                         float freq_scale, float ext_factor, float attn_factor, float beta_fast, float beta_slow, int act_mode,
                         vx_stream stream) {
    if (!vx_supports_qkv_proj_rope(wq, wk, wv, x, q_dst, k_dst, v_dst, n_dims, mode))
        return vx_fail(VX_ERR_UNSUPPORTED, "qkv_proj_rope: three Q8_0/F16 matrices over one activation tensor, a token count the streaming kernel takes, NEOX rotation over the whole head, contiguous outputs");
    if (!pos || !wq->data || !wk->data || !wv->data || !x->data || !q_dst->data || !k_dst->data || !v_dst->data)
        return vx_fail(VX_ERR_INVALID, "qkv_proj_rope: null data");
    if (act_mode != VX_ACT_FLOAT && act_mode != VX_ACT_Q8) return vx_fail(VX_ERR_INVALID, "qkv_proj_rope: bad act_mode");
    const vx_tensor * ws[3] = { wq, wk, wv };
    const vx_tensor * ds[3] = { q_dst, k_dst, v_dst };
    if ((uintptr_t) x->data % 4) return vx_fail(VX_ERR_UNSUPPORTED, "qkv_proj_rope: misaligned activations");
    mm_args a = {};
    a.x = (const char *) x->data;
    a.K = wq->ne[0]; a.N = x->ne[1];
    a.M = 0;
    a.nb11 = x->nb[1]; a.nb12 = x->nb[2]; a.nb13 = x->nb[3];
    a.ne12 = 1; a.r2 = 1; a.r3 = 1;
    a.rows_wg = 16;
    a.w_aligned = 1;
    a.nseg = 3;
    for (int i = 0; i < 3; ++i) {
        if ((uintptr_t) ds[i]->data % 4 || (ws[i]->type == VX_TYPE_F16 && (uintptr_t) ws[i]->data % 2))
            return vx_fail(VX_ERR_UNSUPPORTED, "qkv_proj_rope: misaligned tensor data");
        gv_seg & s = a.seg[i];
        s.w = (const char *) ws[i]->data; s.dst = (char *) ds[i]->data;
        s.M = ws[i]->ne[1]; s.nb01 = ws[i]->nb[1];
        s.nb1 = (uint64_t) s.M * 4; s.nb2 = 0; s.nb3 = (uint64_t) s.M * 4 * x->ne[1]; // the contiguous [rows, tokens, 1, batch] view of dst
        if (i == 2) { s.nb1 = v_dst->nb[1]; s.nb3 = v_dst->nb[3]; }
        s.rope = i < 2;
        a.w_aligned = a.w_aligned && ((uintptr_t) ws[i]->data % 4 == 0) && ws[i]->nb[1] % 4 == 0;
        a.M += s.M;
    }
    a.w = a.seg[0].w; a.dst = a.seg[0].dst;
    a.x_aligned = ((uintptr_t) x->data % 16 == 0) && x->nb[1] % 16 == 0 && x->nb[3] % 16 == 0;
    a.pos = pos; a.ff = freq_factors;
    a.rp = rope_make_params(n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow);
    a.head_dim = n_dims;
    a.rope_T   = (int) q_dst->ne[2];
    a.norm_w   = norm_w ? (const float *) norm_w->data : nullptr;
    a.norm_eps = eps;
    const int nbatch = (int) x->ne[3];
    hipStream_t st = (hipStream_t) stream;
    bool ok;
    if (wq->type == VX_TYPE_Q8_0) ok = act_mode == VX_ACT_Q8 ? launch_gemv<WT_Q8, true>(a, nbatch, st) : launch_gemv<WT_Q8, false>(a, nbatch, st);
    else                          ok = launch_gemv<WT_F16, false>(a, nbatch, st);
    if (!ok) return vx_fail(VX_ERR_UNSUPPORTED, "qkv_proj_rope: shape outside the streaming kernel");
    VX_LAUNCH_CHECK();
    return VX_OK;
}
