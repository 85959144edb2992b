// glue.hip -- the small operators between the projections and attention in the MiniCPM / LocDiT
// graphs (src/minicpm.cpp:572-775): residual ADD, norm-weight MUL, SCALE, ADD1, the KV append
// CPY / CONT, CONCAT of past and current keys, SUM (the reference's write-ordering trick),
// SILU and SWIGLU.  All of them move each byte once: they exist so that a whole decoder layer
// stays on the device and no scheduler split (with its blocking copy) falls between two
// claimed operators.
//
// One indexing scheme serves all of them: a thread owns VEC consecutive elements of one dst row;
// rows are flattened over (i1, i2, i3).  VEC = 4 (16-byte accesses) when every operand is dense
// and 16-byte aligned along dim 0, VEC = 1 otherwise (any strides, ggml's broadcast rules).
#include "vx_common.hpp"
#include "kvs_common.hpp"

#include <algorithm>
#include <cmath>
#include <type_traits>

namespace {

enum ew_op : int {
    EW_ADD, EW_SUB, EW_MUL, EW_DIV,   // dst = src0 (op) src1, src1 broadcast (ggml_can_repeat)
    EW_ADD1,                          // dst = src0 + src1[0]
    EW_SCALE,                         // dst = src0 * p0 (+ p1)
    EW_UNARY,                         // dst = f(src0), f = aux
    EW_GLU,                           // dst = act(a) * b, act = aux
    EW_SCALE_ADD,                     // dst = src0 + src1 * p0   (SCALE feeding ADD)
    EW_ADD_SCALE,                     // dst = (src0 + src1) * p0 (+ p1)   (ADD feeding SCALE)
};

struct ew_args {
    const char * s0; const char * s1; char * d;
    int64_t  ne[4];     // dst shape
    int64_t  ne1[4];    // src1 shape (broadcast)
    uint64_t nb0[4], nb1[4], nbd[4];
    float p0, p1;
    int aux;
    int64_t nchunk;     // blocks per row
};

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }

__device__ __forceinline__ float unary_f(int op, float x) {
    switch (op) {
        case VX_UNARY_ABS:     return fabsf(x);
        case VX_UNARY_SGN:     return x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : 0.0f);
        case VX_UNARY_NEG:     return -x;
        case VX_UNARY_STEP:    return x > 0.0f ? 1.0f : 0.0f;
        case VX_UNARY_TANH:    return tanhf(x);
        case VX_UNARY_RELU:    return x > 0.0f ? x : 0.0f;
        case VX_UNARY_SIGMOID: return 1.0f / (1.0f + expf(-x));
        case VX_UNARY_SILU:    return silu_f(x);
        case VX_UNARY_EXP:     return expf(x);
        case VX_UNARY_FLOOR:   return floorf(x);
        case VX_UNARY_CEIL:    return ceilf(x);
        case VX_UNARY_ROUND:   return roundf(x); // halves away from zero, as libm's
        case VX_UNARY_TRUNC:   return truncf(x);
        case VX_UNARY_SQR:     return x * x;
        case VX_UNARY_SQRT:    return sqrtf(x);
        case VX_UNARY_LOG:     return logf(x);
        case VX_UNARY_SIN:     return sinf(x);
        case VX_UNARY_COS:     return cosf(x);
        default:               return x;
    }
}

// a + x * s with the product rounded first, as a SCALE node followed by an ADD node rounds it
// (the compiler would otherwise contract the pair into one fused multiply-add)
__device__ __forceinline__ float mul_then_add(float x, float s, float a) {
#pragma clang fp contract(off)
    const float t = x * s;
    return a + t;
}

// p0, p1, aux: the node's parameters (scale and bias, the unary / GLU code)
template <int OP>
__device__ __forceinline__ float ew_apply(float p0, float p1, int aux, float x, float y) {
    if constexpr (OP == EW_ADD)   return x + y;
    if constexpr (OP == EW_SUB)   return x - y;
    if constexpr (OP == EW_MUL)   return x * y;
    if constexpr (OP == EW_DIV)   return x / y;
    if constexpr (OP == EW_ADD1)  return x + y;
    if constexpr (OP == EW_SCALE) return p1 == 0.0f ? x * p0 : fmaf(x, p0, p1); // vec_scale / vec_mad1
    if constexpr (OP == EW_UNARY) return unary_f(aux, x);
    if constexpr (OP == EW_GLU)   return (aux == VX_GLU_REGLU ? (x > 0.0f ? x : 0.0f) : silu_f(x)) * y;
    // the fused pairs round exactly where the two separate nodes would (no contraction)
    if constexpr (OP == EW_SCALE_ADD) return mul_then_add(y, p0, x);
    if constexpr (OP == EW_ADD_SCALE) { const float t = x + y; return p1 == 0.0f ? t * p0 : fmaf(t, p0, p1); }
    return x;
}

template <int OP> constexpr bool ew_has_src1() {
    return OP == EW_ADD || OP == EW_SUB || OP == EW_MUL || OP == EW_DIV || OP == EW_GLU || OP == EW_SCALE_ADD || OP == EW_ADD_SCALE;
}

template <int OP, int VEC>
__global__ __launch_bounds__(256) void ew_kernel(const ew_args a) {
    const int64_t row   = blockIdx.x / a.nchunk;
    const int64_t chunk = blockIdx.x % a.nchunk;
    const int64_t i0    = (chunk * 256 + threadIdx.x) * VEC;
    if (i0 >= a.ne[0]) return;
    const int64_t i1 = row % a.ne[1], i2 = (row / a.ne[1]) % a.ne[2], i3 = row / (a.ne[1] * a.ne[2]);
    const char * p0 = a.s0 + i1 * a.nb0[1] + i2 * a.nb0[2] + i3 * a.nb0[3];
    char *       pd = a.d + i1 * a.nbd[1] + i2 * a.nbd[2] + i3 * a.nbd[3];
    const char * p1 = nullptr;
    float yb = 0.0f;
    if constexpr (ew_has_src1<OP>()) p1 = a.s1 + (i1 % a.ne1[1]) * a.nb1[1] + (i2 % a.ne1[2]) * a.nb1[2] + (i3 % a.ne1[3]) * a.nb1[3];
    if constexpr (OP == EW_ADD1) yb = *(const float *) a.s1;

    if constexpr (VEC == 4) {
        const float4_t x = *(const float4_t *) (p0 + i0 * 4);
        float4_t y = {yb, yb, yb, yb};
        if constexpr (ew_has_src1<OP>()) y = *(const float4_t *) (p1 + i0 * 4);
        float4_t r;
#pragma unroll
        for (int k = 0; k < 4; ++k) r[k] = ew_apply<OP>(a.p0, a.p1, a.aux, x[k], y[k]);
        *(float4_t *) (pd + i0 * 4) = r;
    } else {
        const float x = *(const float *) (p0 + i0 * a.nb0[0]);
        float y = yb;
        if constexpr (ew_has_src1<OP>()) y = *(const float *) (p1 + (i0 % a.ne1[0]) * a.nb1[0]);
        *(float *) (pd + i0 * a.nbd[0]) = ew_apply<OP>(a.p0, a.p1, a.aux, x, y);
    }
}

bool al16(const void * p, const uint64_t * nb) {
    return (uintptr_t) p % 16 == 0 && nb[1] % 16 == 0 && nb[2] % 16 == 0 && nb[3] % 16 == 0;
}

template <int OP>
vx_status ew_launch(ew_args & a, hipStream_t st) {
    if (a.ne[0] <= 0 || a.ne[1] * a.ne[2] * a.ne[3] <= 0) return VX_OK;
    // A block walks one row.  Short rows that follow each other in memory in every operand (attention-shaped tensors:
    // 64 elements per row, 16384 rows at a 2 x 512-token prefill) are joined into long ones first, so that a block's
    // 256 threads all have an element.
    while (a.ne[0] < 1024 && a.ne[1] > 1 && a.nb0[0] == 4 && a.nbd[0] == 4 && a.nb0[1] == (uint64_t) a.ne[0] * 4 && a.nbd[1] == (uint64_t) a.ne[0] * 4 &&
           (!ew_has_src1<OP>() || (a.ne1[0] == a.ne[0] && a.ne1[1] == a.ne[1] && a.nb1[0] == 4 && a.nb1[1] == (uint64_t) a.ne[0] * 4))) {
        a.ne[0] *= a.ne[1];
        a.ne1[0] = ew_has_src1<OP>() ? a.ne[0] : a.ne1[0];
        for (int i = 1; i < 3; ++i) {
            a.ne[i] = a.ne[i + 1]; a.ne1[i] = a.ne1[i + 1];
            a.nb0[i] = a.nb0[i + 1]; a.nb1[i] = a.nb1[i + 1]; a.nbd[i] = a.nbd[i + 1];
        }
        a.ne[3] = 1; a.ne1[3] = 1;
        a.nb0[3] = a.nb0[2] * (uint64_t) a.ne[2]; a.nb1[3] = a.nb1[2] * (uint64_t) a.ne1[2]; a.nbd[3] = a.nbd[2] * (uint64_t) a.ne[2];
    }
    const int64_t rows = a.ne[1] * a.ne[2] * a.ne[3];
    bool vec = a.ne[0] % 4 == 0 && a.nb0[0] == 4 && a.nbd[0] == 4 && al16(a.s0, a.nb0) && al16(a.d, a.nbd);
    if (ew_has_src1<OP>()) vec = vec && a.ne1[0] == a.ne[0] && a.nb1[0] == 4 && al16(a.s1, a.nb1);
    const int V = vec ? 4 : 1;
    a.nchunk    = (a.ne[0] + 256 * V - 1) / (256 * V);
    const int64_t blocks = rows * a.nchunk;
    if (blocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "elementwise op: launch too large");
    if (vec) vx_launch(ew_kernel<OP, 4>, dim3((unsigned) blocks), dim3(256), 0, st, a);
    else     vx_launch(ew_kernel<OP, 1>, dim3((unsigned) blocks), dim3(256), 0, st, a);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

void ew_fill(ew_args & a, const vx_tensor * s0, const vx_tensor * s1, const vx_tensor * d) {
    a.s0 = (const char *) s0->data; a.s1 = s1 ? (const char *) s1->data : nullptr; a.d = (char *) d->data;
    for (int i = 0; i < 4; ++i) {
        a.ne[i] = d->ne[i]; a.nb0[i] = s0->nb[i]; a.nbd[i] = d->nb[i];
        a.ne1[i] = s1 ? s1->ne[i] : 1; a.nb1[i] = s1 ? s1->nb[i] : 0;
    }
    a.p0 = a.p1 = 0.0f; a.aux = 0; a.nchunk = 1;
}

bool f32(const vx_tensor * t) { return t && t->type == VX_TYPE_F32; }
bool can_repeat(const vx_tensor * small, const vx_tensor * big) {
    for (int i = 0; i < 4; ++i) if (small->ne[i] <= 0 || big->ne[i] % small->ne[i]) return false;
    return true;
}
bool fl_type(int t) { return t == VX_TYPE_F32 || t == VX_TYPE_F16; }
bool nb_multiple(const vx_tensor * t, uint64_t m) {
    return t->nb[0] % m == 0 && t->nb[1] % m == 0 && t->nb[2] % m == 0 && t->nb[3] % m == 0;
}

// ---- CPY / CONT / DUP -----------------------------------------------------------------------
// Element i of src (row-major order of src's shape) goes to element i of dst (row-major order of
// dst's shape): ggml_compute_forward_dup's rule; the shapes only have to hold the same count.
struct cpy_args {
    const char * s; char * d;
    int64_t  nes[4], ned[4];
    uint64_t nbs[4], nbd[4];
    int64_t  n;
};

// same type: the bits (integers above 2^24 and NaN payloads survive); otherwise through float, as
// ggml_compute_forward_dup_flt converts (ggml/src/ggml-cpu/common.h:34-40: I32 <-> F32 are C casts)
template <typename TS, typename TD>
__device__ __forceinline__ TD cpy_convert(TS x) {
    if constexpr (std::is_same<TS, TD>::value) return x;
    else                                       return (TD) (float) x;
}

template <typename TS, typename TD, int VEC>
__global__ __launch_bounds__(256) void cpy_kernel(const cpy_args a) {
    const int64_t e = ((int64_t) blockIdx.x * 256 + threadIdx.x) * VEC;
    if (e >= a.n) return;
    int64_t r = e;
    const int64_t s0 = r % a.nes[0]; r /= a.nes[0];
    const int64_t s1 = r % a.nes[1]; r /= a.nes[1];
    const int64_t s2 = r % a.nes[2]; const int64_t s3 = r / a.nes[2];
    const char * ps = a.s + s0 * a.nbs[0] + s1 * a.nbs[1] + s2 * a.nbs[2] + s3 * a.nbs[3];
    r = e;
    const int64_t d0 = r % a.ned[0]; r /= a.ned[0];
    const int64_t d1 = r % a.ned[1]; r /= a.ned[1];
    const int64_t d2 = r % a.ned[2]; const int64_t d3 = r / a.ned[2];
    char * pd = a.d + d0 * a.nbd[0] + d1 * a.nbd[1] + d2 * a.nbd[2] + d3 * a.nbd[3];
    if constexpr (VEC == 1) {
        *(TD *) pd = cpy_convert<TS, TD>(*(const TS *) ps);
    } else { // 4 consecutive elements of a dense run on both sides
        typedef TS vs_t __attribute__((ext_vector_type(4)));
        typedef TD vd_t __attribute__((ext_vector_type(4)));
        const vs_t x = *(const vs_t *) ps;
        vd_t y;
#pragma unroll
        for (int k = 0; k < 4; ++k) y[k] = cpy_convert<TS, TD>(x[k]);
        *(vd_t *) pd = y;
    }
}

template <typename TS, typename TD>
vx_status cpy_launch(const cpy_args & a, bool vec, hipStream_t st) {
    const int V = vec ? 4 : 1;
    const int64_t blocks = (a.n / V + 255) / 256;
    if (blocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "cpy: launch too large");
    if (vec) vx_launch(cpy_kernel<TS, TD, 4>, dim3((unsigned) blocks), dim3(256), 0, st, a);
    else     vx_launch(cpy_kernel<TS, TD, 1>, dim3((unsigned) blocks), dim3(256), 0, st, a);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// ---- CONCAT -----------------------------------------------------------------------------------
struct cat_args {
    const char * s0; const char * s1; char * d;
    int64_t  ne[4], ne0[4];   // dst shape, src0 shape
    uint64_t nb0[4], nb1[4], nbd[4];
    int dim;
    int64_t n;                 // dst units (elements, or 16-byte groups when VEC)
};

// UNIT = bytes moved per thread (element size, or 16 for a dense run along dim 0)
template <int UNIT, int ES>
__global__ __launch_bounds__(256) void concat_kernel(const cat_args a) {
    const int64_t u = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (u >= a.n) return;
    constexpr int EPU = UNIT / ES; // elements per unit
    const int64_t units0 = a.ne[0] / EPU;
    int64_t r = u;
    int64_t i[4];
    i[0] = (r % units0) * EPU; r /= units0;
    i[1] = r % a.ne[1]; r /= a.ne[1];
    i[2] = r % a.ne[2]; i[3] = r / a.ne[2];
    char * pd = a.d + i[0] * a.nbd[0] + i[1] * a.nbd[1] + i[2] * a.nbd[2] + i[3] * a.nbd[3];
    const char * ps;
    if (i[a.dim] < a.ne0[a.dim]) {
        ps = a.s0 + i[0] * a.nb0[0] + i[1] * a.nb0[1] + i[2] * a.nb0[2] + i[3] * a.nb0[3];
    } else {
        i[a.dim] -= a.ne0[a.dim];
        ps = a.s1 + i[0] * a.nb1[0] + i[1] * a.nb1[1] + i[2] * a.nb1[2] + i[3] * a.nb1[3];
    }
    if constexpr (UNIT == 16)     *(int4_t *) pd = *(const int4_t *) ps;
    else if constexpr (UNIT == 4) *(int32_t *) pd = *(const int32_t *) ps;
    else                          *(int16_t *) pd = *(const int16_t *) ps;
}

// A tree of CONCATs along one dimension written from its leaves: up to CATM_MAX sources side by side along `dim`, a
// source smaller than its slot is repeated (GGML_OP_REPEAT's index rule: the slot's index modulo the source's shape).
constexpr int CATM_MAX = 8;
struct catm_src { const char * p; uint32_t ne[4]; uint32_t end; uint32_t pad; uint64_t nb[4]; }; // end: one past its last index along dim
struct catm_args {
    catm_src s[CATM_MAX];
    char *   d;
    uint32_t ne[4];
    uint64_t nbd[4];
    int      dim, n_src;
    uint32_t n; // dst units
};
template <bool VEC>
__global__ __launch_bounds__(256) void concat_many_kernel(const catm_args a) {
    const uint32_t u = blockIdx.x * 256u + threadIdx.x;
    if (u >= a.n) return;
    const uint32_t units0 = VEC ? a.ne[0] / 4 : a.ne[0];
    uint32_t i[4], r = u;
    i[0] = (r % units0) * (VEC ? 4 : 1); r /= units0;
    i[1] = r % a.ne[1]; r /= a.ne[1];
    i[2] = r % a.ne[2]; i[3] = r / a.ne[2];
    char * pd = a.d + i[0] * a.nbd[0] + i[1] * a.nbd[1] + i[2] * a.nbd[2] + i[3] * a.nbd[3];
    const uint32_t at = i[a.dim];
    uint32_t begin = 0;
#pragma unroll
    for (int k = 0; k < CATM_MAX; ++k) { // (k is uniform: the sources stay in scalar registers)
        if (k < a.n_src) {
            const catm_src & sr = a.s[k];
            if (at >= begin && at < sr.end) {
                uint32_t j[4] = { i[0], i[1], i[2], i[3] };
                j[a.dim] = at - begin;
#pragma unroll
                for (int q = 0; q < 4; ++q) if (j[q] >= sr.ne[q]) j[q] %= sr.ne[q];
                const char * ps = sr.p + j[0] * sr.nb[0] + j[1] * sr.nb[1] + j[2] * sr.nb[2] + j[3] * sr.nb[3];
                if constexpr (VEC) *(int4_t *) pd = *(const int4_t *) ps;
                else               *(int32_t *) pd = *(const int32_t *) ps;
            }
            begin = sr.end;
        }
    }
}

// ---- ARANGE / REPEAT / GET_ROWS -----------------------------------------------------------------
// The ops the reference's graphs use around the decoder stacks: the causal and CFG-pair masks are
// built from ARANGE + REPEAT (src/minicpm.cpp:602-620, src/locdit.cpp:283-305), token embeddings are
// a GET_ROWS (src/components.cpp:223).  With them a whole forward graph stays on the device.
__device__ __forceinline__ float arange_value(float start, float step, int64_t i) {
#pragma clang fp contract(off)
    const float t = step * (float) i; // product rounded, then the sum: ops.cpp:7899
    return start + t;
}

__global__ __launch_bounds__(256) void arange_kernel(float * d, int64_t n, float start, float step) {
    const int64_t i = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    d[i] = arange_value(start, step, i);
}

struct rep_args {
    const char * s; char * d;
    int64_t  ne[4], nes[4];   // dst shape, src shape
    uint64_t nbs[4], nbd[4];
    int64_t  n;               // dst units
};

// UNIT bytes per thread: the element, or 16 when src rows are whole 16-byte groups
template <int UNIT, int ES>
__global__ __launch_bounds__(256) void repeat_kernel(const rep_args a) {
    const int64_t u = (int64_t) blockIdx.x * 256 + threadIdx.x;
    if (u >= a.n) return;
    constexpr int EPU = UNIT / ES;
    const int64_t units0 = a.ne[0] / EPU;
    int64_t r = u;
    const int64_t i0 = (r % units0) * EPU; r /= units0;
    const int64_t i1 = r % a.ne[1]; r /= a.ne[1];
    const int64_t i2 = r % a.ne[2]; const int64_t i3 = r / a.ne[2];
    char *       pd = a.d + i0 * a.nbd[0] + i1 * a.nbd[1] + i2 * a.nbd[2] + i3 * a.nbd[3];
    const char * ps = a.s + (i0 % a.nes[0]) * a.nbs[0] + (i1 % a.nes[1]) * a.nbs[1] + (i2 % a.nes[2]) * a.nbs[2] + (i3 % a.nes[3]) * a.nbs[3];
    if constexpr (UNIT == 16)     *(int4_t *) pd = *(const int4_t *) ps;
    else if constexpr (UNIT == 4) *(int32_t *) pd = *(const int32_t *) ps;
    else                          *(int16_t *) pd = *(const int16_t *) ps;
}

struct rows_args {
    const char * table; const char * idx; char * d;
    int64_t  nc, n_rows_table;       // row length, rows per table matrix
    int64_t  ne10, ne11, ne12;       // index tensor shape
    uint64_t nb01, nb02, nb03, nb10, nb11, nb12, nb1, nb2, nb3;
    int64_t  nchunk;
};

// one block per (index, 256 * VEC columns).  WT: 0 = 4-byte elements copied as bits (F32, I32),
// 1 = F16 widened, 2 = Q8_0 dequantised as dequantize_row_q8_0 does (quant * f16 scale, one rounding)
template <int WT>
__global__ __launch_bounds__(256) void get_rows_kernel(const rows_args a) {
    const int64_t r = blockIdx.x / a.nchunk, chunk = blockIdx.x % a.nchunk;
    const int64_t i10 = r % a.ne10, i11 = (r / a.ne10) % a.ne11, i12 = r / (a.ne10 * a.ne11);
    int64_t row = *(const int32_t *) (a.idx + i10 * a.nb10 + i11 * a.nb11 + i12 * a.nb12);
    // ggml-cpu aborts on an index outside the table (ops.cpp:4689); a kernel cannot, so it stays in bounds
    row = row < 0 ? 0 : (row >= a.n_rows_table ? a.n_rows_table - 1 : row);
    const char * src = a.table + row * a.nb01 + i11 * a.nb02 + i12 * a.nb03;
    char *       dst = a.d + i10 * a.nb1 + i11 * a.nb2 + i12 * a.nb3;
    const int64_t c = chunk * 256 + threadIdx.x;
    if (c >= a.nc) return;
    if constexpr (WT == 0) {
        *(int32_t *) (dst + c * 4) = *(const int32_t *) (src + c * 4);
    } else if constexpr (WT == 1) {
        *(float *) (dst + c * 4) = (float) *(const _Float16 *) (src + c * 2);
    } else {
        const char * blk = src + (c >> 5) * 34;
        const float  d   = (float) *(const _Float16 *) blk;
        *(float *) (dst + c * 4) = (float) *(const int8_t *) (blk + 2 + (c & 31)) * d;
    }
}

// ---- SUM ---------------------------------------------------------------------------------------
// ggml sums every element in double and rounds once (ops.cpp:1275-1300): fp64 lanes, a fixed reduction
// order.  Rows are dense (checked by the caller); 16-byte loads when VEC.  Small tensors (the ones
// the decode graphs sum) take one block; large ones take SUM_BLOCKS blocks that leave fp64 partials for
// a second, one-wave launch.
constexpr int SUM_BLOCKS = 128;

// the block's 1024 lane totals -> one double, the same value in every thread
__device__ __forceinline__ double block_total(double acc, double * part /* 16 doubles of LDS */) {
    acc = vx_wave_sum(acc);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    double t = 0.0;
    for (int w = 0; w < 16; ++w) t += part[w];
    __syncthreads(); // part may be written again
    return t;
}

// one lane's share of a sum: units first, first + step, ... (< n) added in that order in fp64
template <bool VEC>
__device__ __forceinline__ double sum_lane(const char * src, const vx_dims & s, uint32_t first, uint32_t step, uint32_t n) {
    constexpr int W = VEC ? 4 : 1;
    const uint32_t per_row = (uint32_t) (s.ne[0] / W);
    const uint32_t ne1 = (uint32_t) s.ne[1], ne2 = (uint32_t) s.ne[2];
    double acc = 0.0;
    for (uint32_t e = first; e < n; e += step) {
        const uint32_t row = e / per_row, iv = e - row * per_row;
        const uint32_t i1 = row % ne1, r2 = row / ne1, i2 = r2 % ne2, i3 = r2 / ne2;
        const char * p = src + (uint64_t) iv * (4 * W) + i1 * s.nb[1] + i2 * s.nb[2] + i3 * s.nb[3];
        if constexpr (VEC) {
            const float4_t v = *(const float4_t *) p;
            acc += (double) v[0]; acc += (double) v[1]; acc += (double) v[2]; acc += (double) v[3];
        } else {
            acc += (double) *(const float *) p;
        }
    }
    return acc;
}

template <bool VEC>
__global__ __launch_bounds__(1024) void sum_kernel(const char * src, vx_dims s, float * dst, double * partials) {
    __shared__ double part[16];
    const uint32_t n = (uint32_t) (s.ne[0] / (VEC ? 4 : 1)) * (uint32_t) (s.ne[1] * s.ne[2] * s.ne[3]); // < 2^24, checked by the caller
    const bool one_wave = n <= VX_SUM_ONE_WAVE_UNITS && gridDim.x == 1; // uniform
    if (one_wave && threadIdx.x >= 64) return;
    const uint32_t first = one_wave ? threadIdx.x : blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t step  = one_wave ? 64 : gridDim.x * blockDim.x;
    double acc = sum_lane<VEC>(src, s, first, step, n);
    if (one_wave) {
        acc = vx_wave_sum(acc);
        if (threadIdx.x == 0) *dst = (float) acc;
        return;
    }
    const double t = block_total(acc, part);
    if (threadIdx.x == 0) {
        if (partials) partials[blockIdx.x] = t;
        else          *dst = (float) t;
    }
}

// adds the blocks' partials in block order; they are fetched by as many lanes at once (one trip to memory, not n)
__global__ __launch_bounds__(SUM_BLOCKS) void sum_partials_kernel(const double * partials, int n, float * dst) {
    __shared__ double part[SUM_BLOCKS];
    if ((int) threadIdx.x < n) part[threadIdx.x] = partials[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < n; ++i) t += part[i];
        *dst = (float) t;
    }
}

// ---- a run of tiny nodes as one launch --------------------------------------------------------------
// Around the decoder stacks the reference's graphs hold chains of operators on a few hundred values (bias
// adds, the CONCATs that assemble LocDiT's 14-token sequence, the guidance arithmetic and the Euler update of
// UnifiedCFM, src/unified_cfm.cpp:30-149): a dependent launch each, microseconds for nothing.  One work-group
// of 1024 threads runs such a run node after node.  Every node writes its result to its own memory as its
// separate kernel would, with that kernel's arithmetic (the same device functions, sums in the same order), and
// also into a slot of LDS while there is room: a later node of the run whose operand is exactly that tensor reads
// the slot, so the common chain costs an LDS round trip per node instead of a trip through L2.  An operand that
// merely overlaps something written earlier in the run (a view of it) is read from memory after a full barrier.
constexpr int SG_MAX_NODES = 16;
constexpr int SG_MAX_ELEMS = 16384;
constexpr int SG_LDS_ELEMS = 38912; // 152 KiB of 4-byte slots at most (an F16 value sits in the low half of its slot); a run is given what it uses

enum sg_kind : int { SG_EW2 = 0, SG_ADD1, SG_SCALE, SG_UNARY, SG_CPY, SG_CONCAT, SG_REPEAT, SG_SUM, SG_ARANGE, SG_SUM_ROWS };

struct sg_shape {
    int32_t ne[4];
    int64_t nb[4];
};
struct sg_tensor {
    char *  p;
    int32_t ne[4];
    int64_t nb[4];
    int32_t type;
    int32_t lds;         // first LDS slot of this tensor's row-major image, or -1
};
struct sg_node {
    int32_t kind, aux;   // aux: binary / unary code, CONCAT dim, SUM's 16-byte-unit flag
    float   p0, p1;
    int32_t wait_memory; // an operand (or the destination) overlaps memory written earlier in the run without being that tensor
    int32_t flat;        // 1: element e of the destination takes element e (or the only element) of every operand, all of
                         // them dense or imaged in LDS -- no index arithmetic; 2: a CONCAT of such tensors along their outermost dim
    int32_t one0, one1;  // with flat: operand 0 / 1 is a single element
    // all a flat node needs of its tensors, together at the front (the kernel reads these 22 dwords of a node first and
    // the full descriptors only for the indexed forms): base, type and LDS slot of operand 0, operand 1, destination;
    // element counts of the destination and of operand 0
    char *   fp[3];
    int32_t  ftype[3], flds[3];
    uint32_t fn, fn0;
    sg_shape sh[3];      // shapes and strides of operand 0, operand 1, destination (the indexed forms)
};
constexpr int SG_HEAD_DWORDS = (int) (offsetof(sg_node, sh) / 4);
// Operands that the run only reads (dense 4-byte tensors that no node of the run writes) are brought into LDS images
// before the first node, all loads in flight together: read where they are used, each would cost the run a trip to
// memory of its own, one behind the other.
constexpr int SG_MAX_PRELOADS = 8;
struct sg_preload {
    const uint32_t * p;
    uint32_t         n;   // elements
    int32_t          lds; // first slot of the image
};
struct sg_head {
    int32_t    n, n_pre;
    uint32_t   pre_most, pad; // the largest preloaded tensor's elements
    sg_preload pre[SG_MAX_PRELOADS];
};
struct sg_args {
    sg_head h;
    sg_node node[SG_MAX_NODES];
};

// every thread of the work-group; the caller's next barrier publishes the images
__device__ __forceinline__ void sg_preload_images(const sg_head & h, uint32_t * lds) {
    const uint32_t nt = blockDim.x;
    for (uint32_t base = 0; base < h.pre_most; base += nt) {
        const uint32_t e = base + threadIdx.x;
        uint32_t v[SG_MAX_PRELOADS];
#pragma unroll
        for (int i = 0; i < SG_MAX_PRELOADS; ++i)
            if (i < h.n_pre && e < h.pre[i].n) v[i] = h.pre[i].p[e];
#pragma unroll
        for (int i = 0; i < SG_MAX_PRELOADS; ++i)
            if (i < h.n_pre && e < h.pre[i].n) lds[h.pre[i].lds + e] = v[i];
    }
}

__device__ __forceinline__ void sg_index(const sg_tensor & t, uint32_t e, uint32_t (&i)[4]) {
    i[0] = e % (uint32_t) t.ne[0]; e /= (uint32_t) t.ne[0];
    i[1] = e % (uint32_t) t.ne[1]; e /= (uint32_t) t.ne[1];
    i[2] = e % (uint32_t) t.ne[2]; i[3] = e / (uint32_t) t.ne[2];
}
__device__ __forceinline__ uint32_t sg_count(const sg_tensor & t) { return (uint32_t) (t.ne[0] * t.ne[1] * t.ne[2] * t.ne[3]); }

// the bits of element i of t (i taken modulo t's shape when REP: ggml's repeat rule), from its LDS image or from memory
template <bool REP>
__device__ __forceinline__ uint32_t sg_get(const sg_tensor & t, const uint32_t (&i)[4], const uint32_t * lds) {
    uint32_t j[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) j[q] = REP ? i[q] % (uint32_t) t.ne[q] : i[q];
    if (t.lds >= 0) return lds[(uint32_t) t.lds + ((j[3] * (uint32_t) t.ne[2] + j[2]) * (uint32_t) t.ne[1] + j[1]) * (uint32_t) t.ne[0] + j[0]];
    const char * p = t.p + j[0] * t.nb[0] + j[1] * t.nb[1] + j[2] * t.nb[2] + j[3] * t.nb[3];
    return t.type == VX_TYPE_F16 ? (uint32_t) *(const uint16_t *) p : *(const uint32_t *) p;
}
// element e (row-major) = index i of the destination: to memory, and to the LDS image when it has one
__device__ __forceinline__ void sg_put(const sg_tensor & t, uint32_t e, const uint32_t (&i)[4], uint32_t bits, uint32_t * lds) {
    if (t.p) { // (no memory behind a private destination that has its image)
        char * p = t.p + i[0] * t.nb[0] + i[1] * t.nb[1] + i[2] * t.nb[2] + i[3] * t.nb[3];
        if (t.type == VX_TYPE_F16) *(uint16_t *) p = (uint16_t) bits;
        else                       *(uint32_t *) p = bits;
    }
    if (t.lds >= 0) lds[(uint32_t) t.lds + e] = bits;
}
// the same for the flat case: element e in row-major order of a dense tensor (or its LDS image)
__device__ __forceinline__ uint32_t sg_get_flat(const sg_tensor & t, uint32_t e, const uint32_t * lds) {
    if (t.lds >= 0) return lds[(uint32_t) t.lds + e];
    return t.type == VX_TYPE_F16 ? (uint32_t) ((const uint16_t *) t.p)[e] : ((const uint32_t *) t.p)[e];
}
__device__ __forceinline__ void sg_put_flat(const sg_tensor & t, uint32_t e, uint32_t bits, uint32_t * lds) {
    if (t.type == VX_TYPE_F16) ((uint16_t *) t.p)[e] = (uint16_t) bits;
    else                       ((uint32_t *) t.p)[e] = bits;
    if (t.lds >= 0) lds[(uint32_t) t.lds + e] = bits;
}
__device__ __forceinline__ float    sg_f(uint32_t b) { return __builtin_bit_cast(float, b); }
__device__ __forceinline__ uint32_t sg_b(float f) { return __builtin_bit_cast(uint32_t, f); }

template <typename TS, typename TD>
__device__ __forceinline__ uint32_t sg_convert(uint32_t bits) {
    TS x;
    if constexpr (sizeof(TS) == 2) x = __builtin_bit_cast(TS, (uint16_t) bits); else x = __builtin_bit_cast(TS, bits);
    const TD y = cpy_convert<TS, TD>(x);
    if constexpr (sizeof(TD) == 2) return (uint32_t) __builtin_bit_cast(uint16_t, y); else return __builtin_bit_cast(uint32_t, y);
}

// one lane's share of a sum over an LDS image: the units of sum_lane (4 consecutive elements, or 1), same order
template <bool VEC>
__device__ __forceinline__ double sum_lane_lds(const uint32_t * img, uint32_t first, uint32_t step, uint32_t n) {
    constexpr int W = VEC ? 4 : 1;
    double acc = 0.0;
    for (uint32_t e = first; e < n; e += step)
#pragma unroll
        for (int q = 0; q < W; ++q) acc += (double) sg_f(img[e * W + q]);
    return acc;
}

__global__ __launch_bounds__(1024) void small_graph_kernel(const sg_args a0) {
    __shared__ double   part[16];
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[]; // the images: as many slots as the host counted
    // The node table is fetched ONCE, by all threads together, into LDS: read from the argument block where a field is
    // first needed, every cache line of every node is a trip to memory of its own.  A node's fields then become scalars,
    // once per node -- the head for every node, the full tensor descriptors only for the indexed forms.
    __shared__ __attribute__((aligned(16))) uint32_t table[(sizeof(sg_args) + 3) / 4];
    {
        typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
        static_assert(sizeof(sg_args) % 16 == 0 && sizeof(sg_args) <= 256 * 16, "16 bytes per thread of the smallest work-group");
        const uint32_t quads = (uint32_t) (offsetof(sg_args, node) + (size_t) a0.h.n * sizeof(sg_node) + 15) / 16;
        if (threadIdx.x < quads) ((u32x4 *) table)[threadIdx.x] = ((const u32x4 *) &a0)[threadIdx.x]; // one trip to memory for the whole table
    }
    sg_preload_images(a0.h, lds);
    __syncthreads();
    const uint32_t nt = blockDim.x; // the host sizes the work-group to the run: a run of 128-element nodes is two waves' work
    const int n_nodes = a0.h.n;
    // a node's head is read from the table one node ahead, so that its LDS latency passes under the node before it
    uint32_t head[SG_HEAD_DWORDS];
    auto read_head = [&](int k) {
        const uint32_t * src = table + (offsetof(sg_args, node) + (size_t) k * sizeof(sg_node)) / 4;
#pragma unroll
        for (int i = 0; i < SG_HEAD_DWORDS; ++i) head[i] = src[i];
    };
    read_head(0);
    for (int k = 0; k < n_nodes; ++k) { // uniform: every thread walks every node and meets every barrier
        sg_node nd;
        const uint32_t * nsrc = table + (offsetof(sg_args, node) + (size_t) k * sizeof(sg_node)) / 4;
        {
            uint32_t * dst = (uint32_t *) &nd;
#pragma unroll
            for (int i = 0; i < SG_HEAD_DWORDS; ++i) dst[i] = (uint32_t) __builtin_amdgcn_readfirstlane((int) head[i]);
        }
        if (k + 1 < n_nodes) read_head(k + 1);
        if (nd.flat == 0) {
            uint32_t * dst = (uint32_t *) &nd;
#pragma unroll
            for (int i = SG_HEAD_DWORDS; i < (int) (sizeof(sg_node) / 4); ++i) dst[i] = (uint32_t) __builtin_amdgcn_readfirstlane((int) nsrc[i]);
        }
        auto tensor_of = [&](int o) {
            sg_tensor t;
            t.p = nd.fp[o]; t.type = nd.ftype[o]; t.lds = nd.flds[o];
#pragma unroll
            for (int q = 0; q < 4; ++q) { t.ne[q] = nd.sh[o].ne[q]; t.nb[q] = nd.sh[o].nb[q]; }
            return t;
        };
        if (k > 0) {
            if (nd.wait_memory) {
                __syncthreads(); // earlier nodes' stores to memory are complete and visible to the work-group
            } else {             // only the LDS images carry values between the nodes: no wait for stores in flight
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
            }
        }
        const uint32_t n = nd.fn;
        // where each tensor's elements are, decided once: its LDS image, or memory as F32 / I32 or F16
        const uint32_t * img0 = nd.flds[0] >= 0 ? lds + nd.flds[0] : nullptr, * img1 = nd.flds[1] >= 0 ? lds + nd.flds[1] : nullptr;
        uint32_t *       imgd = nd.flds[2] >= 0 ? lds + nd.flds[2] : nullptr;
        auto get0 = [&](uint32_t e) -> uint32_t {
            if (img0) return img0[e];
            return nd.ftype[0] == VX_TYPE_F16 ? (uint32_t) ((const uint16_t *) nd.fp[0])[e] : ((const uint32_t *) nd.fp[0])[e];
        };
        auto get1 = [&](uint32_t e) -> uint32_t {
            if (img1) return img1[e];
            return nd.ftype[1] == VX_TYPE_F16 ? (uint32_t) ((const uint16_t *) nd.fp[1])[e] : ((const uint32_t *) nd.fp[1])[e];
        };
        auto put = [&](uint32_t e, uint32_t bits) { // (no memory behind a private destination that has its image)
            if (nd.fp[2]) {
                if (nd.ftype[2] == VX_TYPE_F16) ((uint16_t *) nd.fp[2])[e] = (uint16_t) bits;
                else                            ((uint32_t *) nd.fp[2])[e] = bits;
            }
            if (imgd) imgd[e] = bits;
        };
        if (nd.flat == 1) { // dense operands of the destination's shape (or single elements): no index arithmetic
#define SG_FLAT_LOOP(expr) for (uint32_t e = threadIdx.x; e < n; e += nt) put(e, (expr))
#define SG_X (sg_f(get0(nd.one0 ? 0 : e)))
#define SG_Y (sg_f(get1(nd.one1 ? 0 : e)))
            switch (nd.kind) {
                case SG_ARANGE: SG_FLAT_LOOP(sg_b(arange_value(nd.p0, nd.p1, (int64_t) e))); break;
                case SG_EW2:
                    switch (nd.aux) {
                        case VX_BIN_ADD: SG_FLAT_LOOP(sg_b(ew_apply<EW_ADD>(0, 0, 0, SG_X, SG_Y))); break;
                        case VX_BIN_SUB: SG_FLAT_LOOP(sg_b(ew_apply<EW_SUB>(0, 0, 0, SG_X, SG_Y))); break;
                        case VX_BIN_MUL: SG_FLAT_LOOP(sg_b(ew_apply<EW_MUL>(0, 0, 0, SG_X, SG_Y))); break;
                        default:         SG_FLAT_LOOP(sg_b(ew_apply<EW_DIV>(0, 0, 0, SG_X, SG_Y))); break;
                    }
                    break;
                case SG_ADD1: {
                    const float y = sg_f(get1(0));
                    SG_FLAT_LOOP(sg_b(ew_apply<EW_ADD1>(0, 0, 0, SG_X, y)));
                } break;
                case SG_SCALE: SG_FLAT_LOOP(sg_b(ew_apply<EW_SCALE>(nd.p0, nd.p1, 0, SG_X, 0.0f))); break;
                case SG_UNARY: SG_FLAT_LOOP(sg_b(ew_apply<EW_UNARY>(0, 0, nd.aux, SG_X, 0.0f))); break;
                default: // SG_CPY between dense tensors (element e to element e), SG_REPEAT of one value
#define SG_BITS (get0(nd.one0 ? 0 : e))
                    if (nd.ftype[0] == VX_TYPE_I32) {
                        if (nd.ftype[2] == VX_TYPE_I32) SG_FLAT_LOOP(SG_BITS); else SG_FLAT_LOOP((sg_convert<int32_t, float>(SG_BITS)));
                    } else if (nd.ftype[2] == VX_TYPE_I32) {
                        SG_FLAT_LOOP((sg_convert<float, int32_t>(SG_BITS)));
                    } else if (nd.ftype[0] == VX_TYPE_F32) {
                        if (nd.ftype[2] == VX_TYPE_F32) SG_FLAT_LOOP(SG_BITS); else SG_FLAT_LOOP((sg_convert<float, _Float16>(SG_BITS)));
                    } else {
                        if (nd.ftype[2] == VX_TYPE_F32) SG_FLAT_LOOP((sg_convert<_Float16, float>(SG_BITS))); else SG_FLAT_LOOP(SG_BITS);
                    }
#undef SG_BITS
                    break;
            }
#undef SG_X
#undef SG_Y
#undef SG_FLAT_LOOP
            continue;
        }
        if (nd.flat == 2) { // CONCAT along the outermost dim: the first operand's elements, then the second's
            const uint32_t n0 = nd.fn0;
            for (uint32_t e = threadIdx.x; e < n; e += nt) put(e, e < n0 ? get0(e) : get1(e - n0));
            continue;
        }
        const sg_tensor S0 = tensor_of(0), S1 = tensor_of(1), D = tensor_of(2); // only the indexed forms get here
        switch (nd.kind) {
            case SG_EW2:
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4];
                    sg_index(D, e, i);
                    const float x = sg_f(sg_get<false>(S0, i, lds)), y = sg_f(sg_get<true>(S1, i, lds));
                    float r;
                    switch (nd.aux) {
                        case VX_BIN_ADD: r = ew_apply<EW_ADD>(0, 0, 0, x, y); break;
                        case VX_BIN_SUB: r = ew_apply<EW_SUB>(0, 0, 0, x, y); break;
                        case VX_BIN_MUL: r = ew_apply<EW_MUL>(0, 0, 0, x, y); break;
                        default:         r = ew_apply<EW_DIV>(0, 0, 0, x, y); break;
                    }
                    sg_put(D, e, i, sg_b(r), lds);
                }
                break;
            case SG_ADD1: {
                const uint32_t zero[4] = { 0, 0, 0, 0 };
                const float y = sg_f(sg_get<false>(S1, zero, lds));
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4];
                    sg_index(D, e, i);
                    sg_put(D, e, i, sg_b(ew_apply<EW_ADD1>(0, 0, 0, sg_f(sg_get<false>(S0, i, lds)), y)), lds);
                }
            } break;
            case SG_SCALE:
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4];
                    sg_index(D, e, i);
                    sg_put(D, e, i, sg_b(ew_apply<EW_SCALE>(nd.p0, nd.p1, 0, sg_f(sg_get<false>(S0, i, lds)), 0.0f)), lds);
                }
                break;
            case SG_UNARY:
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4];
                    sg_index(D, e, i);
                    sg_put(D, e, i, sg_b(ew_apply<EW_UNARY>(0, 0, nd.aux, sg_f(sg_get<false>(S0, i, lds)), 0.0f)), lds);
                }
                break;
            case SG_CPY: // element e of the source shape -> element e of the destination shape
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t is[4], id[4];
                    sg_index(S0, e, is);
                    sg_index(D, e, id);
                    const uint32_t x = sg_get<false>(S0, is, lds);
                    uint32_t y;
                    if (S0.type == VX_TYPE_I32)      y = D.type == VX_TYPE_I32 ? x : sg_convert<int32_t, float>(x);
                    else if (D.type == VX_TYPE_I32)  y = sg_convert<float, int32_t>(x);
                    else if (S0.type == VX_TYPE_F32) y = D.type == VX_TYPE_F32 ? x : sg_convert<float, _Float16>(x);
                    else                                y = D.type == VX_TYPE_F32 ? sg_convert<_Float16, float>(x) : x;
                    sg_put(D, e, id, y, lds);
                }
                break;
            case SG_CONCAT:
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4], j[4];
                    sg_index(D, e, i);
#pragma unroll
                    for (int q = 0; q < 4; ++q) j[q] = i[q];
                    uint32_t off = 0;
#pragma unroll
                    for (int q = 0; q < 4; ++q) if (q == nd.aux) off = (uint32_t) S0.ne[q];
                    bool second = false;
#pragma unroll
                    for (int q = 0; q < 4; ++q) if (q == nd.aux && i[q] >= off) { j[q] = i[q] - off; second = true; }
                    sg_put(D, e, i, second ? sg_get<false>(S1, j, lds) : sg_get<false>(S0, j, lds), lds);
                }
                break;
            case SG_REPEAT:
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4];
                    sg_index(D, e, i);
                    sg_put(D, e, i, sg_get<true>(S0, i, lds), lds);
                }
                break;
            case SG_SUM: { // vx_sum's two single-block orders: one wave up to VX_SUM_ONE_WAVE_UNITS units, the block beyond
                vx_dims s;
                for (int q = 0; q < 4; ++q) { s.ne[q] = S0.ne[q]; s.nb[q] = (uint64_t) S0.nb[q]; }
                const uint32_t units = sg_count(S0) / (nd.aux ? 4 : 1);
                const bool one_wave = units <= VX_SUM_ONE_WAVE_UNITS;
                const uint32_t step = one_wave ? 64 : 1024; // (a sum over the whole block: the host launches 1024 threads for such a run)
                double acc = 0.0;
                if (!one_wave || threadIdx.x < 64) {
                    if (S0.lds >= 0) acc = nd.aux ? sum_lane_lds<true>(lds + S0.lds, threadIdx.x, step, units) : sum_lane_lds<false>(lds + S0.lds, threadIdx.x, step, units);
                    else                acc = nd.aux ? sum_lane<true>(S0.p, s, threadIdx.x, step, units) : sum_lane<false>(S0.p, s, threadIdx.x, step, units);
                }
                double t;
                if (one_wave) t = threadIdx.x < 64 ? vx_wave_sum(acc) : 0.0;
                else          t = block_total(acc, part);
                if (threadIdx.x == 0) {
                    const uint32_t zero[4] = { 0, 0, 0, 0 };
                    sg_put(D, 0, zero, sg_b((float) t), lds);
                }
            } break;
            case SG_ARANGE:
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    uint32_t i[4];
                    sg_index(D, e, i);
                    sg_put(D, e, i, sg_b(arange_value(nd.p0, nd.p1, (int64_t) e)), lds);
                }
                break;
            case SG_SUM_ROWS: { // vx_sum_rows' order: a wave per row, lane-strided in fp64, one butterfly
                const uint32_t ne0 = (uint32_t) S0.ne[0], rows = sg_count(S0) / ne0, lane = threadIdx.x & 63;
                for (uint32_t r = threadIdx.x >> 6; r < rows; r += nt >> 6) {
                    uint32_t i[4] = { 0, r % (uint32_t) S0.ne[1], 0, 0 };
                    const uint32_t r2 = r / (uint32_t) S0.ne[1];
                    i[2] = r2 % (uint32_t) S0.ne[2]; i[3] = r2 / (uint32_t) S0.ne[2];
                    double acc = 0.0;
                    for (uint32_t c0 = lane; c0 < ne0; c0 += 64) { i[0] = c0; acc += (double) sg_f(sg_get<false>(S0, i, lds)); }
                    acc = vx_wave_sum(acc);
                    i[0] = 0;
                    if (lane == 0) sg_put(D, r, i, sg_b((float) acc), lds);
                }
            } break;
            default: break;
        }
    }
}

// ---- the same run when every node is dense F32 -----------------------------------------------------------
// The interpreter above pays for its generality in instructions: ≈ 360 per node and wave for a chain of 128-element
// nodes, at the 4 cycles a wave needs per instruction.  When every node of a run is a dense F32 operator (element e of the
// destination from element e, or the only element, of each operand; a CONCAT along the outermost dimension; a sum in the
// one-wave order) the host resolves everything else beforehand into 16 dwords per node -- operator code, counts, where
// each operand lies (its LDS image or a global address) -- and the kernel only scalarises them (read one node ahead),
// meets the barrier and runs a loop of a handful of instructions.  Same device functions, same orders, same bits.
enum sgd_code : uint32_t { SGD_ADD = 0, SGD_SUB, SGD_MUL, SGD_DIV, SGD_ADD1, SGD_SCALE, SGD_UNARY, SGD_COPY, SGD_CONCAT, SGD_SUM4, SGD_SUM1, SGD_ARANGE,
                           SGD_COPY4, SGD_CONCAT4,   // these two: 16 bytes per thread, counts in quads
                           SGD_SUM_ROWS };           // n rows of n0 values each, a wave per row
// SGD_NO_BARRIER: every value this node reads from an image written since the last barrier was written by the reading
// thread itself (element e of a dense node is always thread e mod work-group size), and its destination is a fresh image
// SGD_BLK0 / SGD_MOD0 (a REPEAT as SGD_COPY): destination element e takes source element e / block (p0 = 1 / block: a value
// per request repeated over the request's elements) or e mod n0 (p0 = 1 / n0: a row repeated for every request)
constexpr uint32_t SGD_ONE0 = 1, SGD_ONE1 = 2, SGD_WAIT_MEMORY = 4, SGD_NO_BARRIER = 8, SGD_BLK0 = 16, SGD_MOD0 = 32,
                   SGD_MOD1 = 64, // a binary node whose second operand repeats every aux elements (p1 = 1 / aux: a row added to every request)
                   SGD_BLOCKS = 128; // a CONCAT below the outermost dimension (a sequence assembled per request): the destination is
                                     // blocks of aux elements (p0 = 1 / aux), each n0 of the first operand's followed by aux - n0 of the second's
struct sgd_op {
    uint32_t code, n, n0, flags; // n: destination elements (SUM: units of the source); n0: CONCAT's first operand
    float    p0, p1;
    int32_t  s0_lds, s1_lds, d_lds, aux; // first LDS slot of the operand's image, or -1 (then the global address below)
    const float * s0, * s1;
    float *       d;              // null: a private destination that lives in its image only
};
static_assert(sizeof(sgd_op) == 64, "16 dwords per node");
struct sgd_args {
    sg_head h;
    sgd_op  op[SG_MAX_NODES];
};

__global__ __launch_bounds__(1024) void small_graph_dense_kernel(const sgd_args a0) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) uint32_t lds[]; // the images
    __shared__ u32x4 table[sizeof(sgd_args) / 16];
    static_assert(sizeof(sgd_args) % 16 == 0 && sizeof(sgd_args) / 16 <= 256, "16 bytes per thread of the smallest work-group");
    const int n_nodes = a0.h.n;
    constexpr int OPS_AT = (int) (offsetof(sgd_args, op) / 16);
    static_assert(offsetof(sgd_args, op) % 16 == 0, "nodes on 16-byte boundaries");
    if (threadIdx.x < OPS_AT + 4 * (uint32_t) n_nodes) table[threadIdx.x] = ((const u32x4 *) &a0)[threadIdx.x]; // one trip for the whole table
    sg_preload_images(a0.h, lds);
    __syncthreads();
    const uint32_t nt = blockDim.x;
    const float *  ldsf = (const float *) lds;
    u32x4 nx[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) nx[q] = table[OPS_AT + q];
    for (int k = 0; k < n_nodes; ++k) { // uniform: every thread walks every node and meets every barrier
        sgd_op op;
        {
            uint32_t * w = (uint32_t *) &op;
#pragma unroll
            for (int q = 0; q < 4; ++q)
#pragma unroll
                for (int i = 0; i < 4; ++i) w[4 * q + i] = (uint32_t) __builtin_amdgcn_readfirstlane((int) nx[q][i]);
        }
        if (k + 1 < n_nodes) {
#pragma unroll
            for (int q = 0; q < 4; ++q) nx[q] = table[OPS_AT + 4 * (k + 1) + q];
        }
        if (k > 0 && !(op.flags & SGD_NO_BARRIER)) {
            if (op.flags & SGD_WAIT_MEMORY) {
                __syncthreads(); // earlier nodes' stores to memory are complete and visible to the work-group
            } else {             // only the LDS images carry values between the nodes: no wait for stores in flight
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
            }
        }
        const uint32_t n = op.n;
        const bool l0 = op.s0_lds >= 0, l1 = op.s1_lds >= 0, ld = op.d_lds >= 0, one0 = op.flags & SGD_ONE0, one1 = op.flags & SGD_ONE1;
        auto x_at = [&](uint32_t e) { return l0 ? ldsf[op.s0_lds + e] : op.s0[e]; };
        auto y_at = [&](uint32_t e) { return l1 ? ldsf[op.s1_lds + e] : op.s1[e]; };
        auto put = [&](uint32_t e, float r) {
            if (ld) lds[op.d_lds + e] = __builtin_bit_cast(uint32_t, r);
            if (op.d) op.d[e] = r;
        };
#define SGD_LOOP(expr) for (uint32_t e = threadIdx.x; e < n; e += nt) put(e, (expr))
#define SGD_X x_at(one0 ? 0 : e)
#define SGD_Y y_at(one1 ? 0 : e)
        switch (op.code) {
#define SGD_Y_TILED y_at(e - (uint32_t) (((float) e + 0.5f) * op.p1) * (uint32_t) op.aux)
#define SGD_BINARY(OP) if (op.flags & SGD_MOD1) SGD_LOOP(ew_apply<OP>(0, 0, 0, SGD_X, SGD_Y_TILED)); else SGD_LOOP(ew_apply<OP>(0, 0, 0, SGD_X, SGD_Y))
            case SGD_ADD:    SGD_BINARY(EW_ADD); break;
            case SGD_SUB:    SGD_BINARY(EW_SUB); break;
            case SGD_MUL:    SGD_BINARY(EW_MUL); break;
            case SGD_DIV:    SGD_BINARY(EW_DIV); break;
            case SGD_ADD1: { const float y = y_at(0); SGD_LOOP(ew_apply<EW_ADD1>(0, 0, 0, SGD_X, y)); } break;
            case SGD_SCALE:  SGD_LOOP(ew_apply<EW_SCALE>(op.p0, op.p1, 0, SGD_X, 0.0f)); break;
            case SGD_UNARY:  SGD_LOOP(ew_apply<EW_UNARY>(0, 0, op.aux, SGD_X, 0.0f)); break;
            case SGD_COPY:
                if (op.flags & (SGD_BLK0 | SGD_MOD0)) { // exact below 2^22 elements (a node holds at most 16384)
                    const bool blk = op.flags & SGD_BLK0;
                    for (uint32_t e = threadIdx.x; e < n; e += nt) {
                        const uint32_t q = (uint32_t) (((float) e + 0.5f) * op.p0);
                        put(e, x_at(blk ? q : e - q * op.n0));
                    }
                } else {
                    SGD_LOOP(SGD_X);
                }
                break;
            case SGD_CONCAT:
                if (op.flags & SGD_BLOCKS) { // (the quotient is exact below 2^22 elements)
                    const uint32_t inner = (uint32_t) op.aux, n1 = inner - op.n0;
                    for (uint32_t e = threadIdx.x; e < n; e += nt) {
                        const uint32_t b = (uint32_t) (((float) e + 0.5f) * op.p0), r = e - b * inner;
                        put(e, r < op.n0 ? x_at(b * op.n0 + r) : y_at(b * n1 + r - op.n0));
                    }
                } else {
                    SGD_LOOP(e < op.n0 ? x_at(e) : y_at(e - op.n0));
                }
                break;
            case SGD_ARANGE: SGD_LOOP(arange_value(op.p0, op.p1, (int64_t) e)); break;
            case SGD_COPY4: case SGD_CONCAT4: { // (a COPY4 has n0 == n)
                const u32x4 * g0 = (const u32x4 *) op.s0, * g1 = (const u32x4 *) op.s1;
                const u32x4 * i0 = (const u32x4 *) (lds + (l0 ? op.s0_lds : 0)), * i1 = (const u32x4 *) (lds + (l1 ? op.s1_lds : 0));
                u32x4 * gd = (u32x4 *) op.d, * id = (u32x4 *) (lds + (ld ? op.d_lds : 0));
                const bool     blocks = op.code == SGD_CONCAT4 && (op.flags & SGD_BLOCKS);
                const uint32_t inner = blocks ? (uint32_t) op.aux : n, n1 = inner - op.n0;
                for (uint32_t e = threadIdx.x; e < n; e += nt) {
                    const uint32_t b = blocks ? (uint32_t) (((float) e + 0.5f) * op.p0) : 0u, r = e - b * inner;
                    u32x4 v;
                    if (r < op.n0) v = l0 ? i0[b * op.n0 + r] : g0[b * op.n0 + r];
                    else           v = l1 ? i1[b * n1 + r - op.n0] : g1[b * n1 + r - op.n0];
                    if (ld) id[e] = v;
                    if (gd) gd[e] = v;
                }
            } break;
            case SGD_SUM_ROWS: { // vx_sum_rows' order: a wave per row, lane-strided in fp64, one butterfly
                const uint32_t lane = threadIdx.x & 63;
                for (uint32_t r = threadIdx.x >> 6; r < n; r += nt >> 6) {
                    double acc = 0.0;
                    for (uint32_t c0 = lane; c0 < op.n0; c0 += 64) acc += (double) x_at(r * op.n0 + c0);
                    acc = vx_wave_sum(acc);
                    if (lane == 0) put(r, (float) acc);
                }
            } break;
            default: { // SGD_SUM4 / SGD_SUM1: vx_sum's one-wave order -- lane-strided units in fp64, one butterfly
                if (threadIdx.x < 64) {
                    const int W = op.code == SGD_SUM4 ? 4 : 1;
                    double acc = 0.0;
                    for (uint32_t u = threadIdx.x; u < n; u += 64)
                        for (int q = 0; q < W; ++q) acc += (double) x_at(u * W + q);
                    const double t = vx_wave_sum(acc);
                    if (threadIdx.x == 0) put(0, (float) t);
                }
            } break;
        }
#undef SGD_LOOP
#undef SGD_X
#undef SGD_Y
#undef SGD_Y_TILED
#undef SGD_BINARY
    }
}

// ---- KV append + the reference's write-ordering scalar, one block ---------------------------------
// attention_forward (src/minicpm.cpp:682-713) copies the new keys and values into their cache slots,
// sums both copies, scales the total (by zero) and adds it to the attention output, so that the
// writes are ancestors of the graph's result:
//     CPY(k, k_slot) CONT SUM , CPY(v, v_slot) CONT SUM , ADD , SCALE , ADD1(x, .)
// Here the block stores both slots, forms the two sums in sum_kernel's order (so the scalar is the
// one the separate nodes produce, NaN and infinity included) and writes dst = x + scalar.
constexpr int KVS_PRE = 4; // x elements per thread requested before anything else

struct kvs_args {
    kvs_side k, v;
    const char * x; char * d;
    int64_t  ne[4];
    uint64_t nbx[4], nbd[4];
    float scale, bias;
    int dense4; // x and d are contiguous, 16-byte aligned, a multiple of 4 elements: the ADD1 walks them 16 bytes at a time
    double * defer; // kv_store_sync_kernel leaves the two sums here (in the layout of kv_store_large_kernel's block totals) and the
                    // ADD1 to kv_sync_add1_kernel: one work-group adding a scalar to a prompt's 64 x 1024 values took 40 us
};

// stores the slot and returns the sum of what was stored, the same value in every thread of the block
template <bool VEC>
__device__ __forceinline__ float store_and_sum(const kvs_side & a, double * part) {
    const uint32_t n = kvs_units(a, VEC);
    if (n <= VX_SUM_ONE_WAVE_UNITS) { // the one-wave order of small sums
        if (threadIdx.x < 64) {
            const double t = kvs_wave_total<VEC>(a, threadIdx.x, true);
            if (threadIdx.x == 0) part[0] = t;
        }
        __syncthreads();
        const float r = (float) part[0];
        __syncthreads();
        return r;
    }
    double acc = 0.0;
    for (uint32_t e = threadIdx.x; e < n; e += 1024) kvs_unit<VEC>(a, e, true, acc);
    return (float) block_total(acc, part);
}

__global__ __launch_bounds__(1024) void kv_store_sync_kernel(const kvs_args a) {
    __shared__ double part[16];
    const uint32_t n0 = (uint32_t) a.ne[0], n1 = (uint32_t) a.ne[1], n2 = (uint32_t) a.ne[2];
    const uint32_t nx = n0 * n1 * (uint32_t) (n2 * a.ne[3]);
    auto offsets = [&](uint32_t e, uint64_t & ox, uint64_t & od) {
        uint32_t r = e;
        const uint32_t i0 = r % n0; r /= n0;
        const uint32_t i1 = r % n1; r /= n1;
        const uint32_t i2 = r % n2, i3 = r / n2;
        ox = i0 * a.nbx[0] + i1 * a.nbx[1] + i2 * a.nbx[2] + i3 * a.nbx[3];
        od = i0 * a.nbd[0] + i1 * a.nbd[1] + i2 * a.nbd[2] + i3 * a.nbd[3];
    };
    if (a.defer) { // (uniform) the sums only: as floats, as the scalar takes them, in the first slot of each half
        const float sk = a.k.vec ? store_and_sum<true>(a.k, part) : store_and_sum<false>(a.k, part);
        const float sv = a.v.vec ? store_and_sum<true>(a.v, part) : store_and_sum<false>(a.v, part);
        if (threadIdx.x < 2 * SUM_BLOCKS) a.defer[threadIdx.x] = threadIdx.x == 0 ? (double) sk : threadIdx.x == SUM_BLOCKS ? (double) sv : 0.0;
        return;
    }
    float    xv[KVS_PRE];
    uint64_t xo[KVS_PRE];
#pragma unroll
    for (int p = 0; p < KVS_PRE; ++p) {
        const uint32_t e = threadIdx.x + 1024 * p;
        xv[p] = 0.0f; xo[p] = 0;
        if (e < nx) { uint64_t ox; offsets(e, ox, xo[p]); xv[p] = *(const float *) (a.x + ox); }
    }
    const float sk = a.k.vec ? store_and_sum<true>(a.k, part) : store_and_sum<false>(a.k, part);
    const float sv = a.v.vec ? store_and_sum<true>(a.v, part) : store_and_sum<false>(a.v, part);
    const float  y  = kvs_scalar(sk, sv, a.scale, a.bias);
#pragma unroll
    for (int p = 0; p < KVS_PRE; ++p)
        if (threadIdx.x + 1024 * p < nx) *(float *) (a.d + xo[p]) = xv[p] + y;  // the ADD1 node
    for (uint32_t e = threadIdx.x + 1024 * KVS_PRE; e < nx; e += 1024) {
        uint64_t ox, od; offsets(e, ox, od);
        *(float *) (a.d + od) = *(const float *) (a.x + ox) + y;
    }
}

// A prefill's cache write (tens of thousands of keys at once): the same nodes, of which the two SUMs are then the
// 128-block form of GGML_OP_SUM's kernel -- thread t of block b walks units b * 1024 + t, + 128 * 1024, ...; the
// blocks' fp64 totals are added in block order by a second kernel.  Here the first kernel also stores the slots (one
// grid half per cache), and the second, which adds the totals, forms the scalar and applies the ADD1 to x.
template <bool VK, bool VV>
__global__ __launch_bounds__(1024) void kv_store_large_kernel(const kvs_args a, double * partials) {
    __shared__ double part[16];
    const bool     second = blockIdx.x >= SUM_BLOCKS; // uniform
    const uint32_t b = blockIdx.x - (second ? SUM_BLOCKS : 0);
    double acc = 0.0;
    if (!second) { const uint32_t n = kvs_units(a.k, VK); for (uint32_t e = b * 1024 + threadIdx.x; e < n; e += SUM_BLOCKS * 1024) kvs_unit<VK>(a.k, e, true, acc); }
    else         { const uint32_t n = kvs_units(a.v, VV); for (uint32_t e = b * 1024 + threadIdx.x; e < n; e += SUM_BLOCKS * 1024) kvs_unit<VV>(a.v, e, true, acc); }
    const double t = block_total(acc, part);
    if (threadIdx.x == 0) partials[blockIdx.x] = t;
}

// A write between the two (a prompt of a few hundred tokens): each SUM is still GGML_OP_SUM's one block of 1024 threads
// -- thread t walks units t, t + 1024, ..., a wave adds its lanes by butterfly, the 16 wave totals are added in order --
// but one work-group storing and adding 2 x 64 Ki values is 17 us.  Here every wave of that block is a work-group of its
// own (16 per cache) and leaves its total where the kernel behind adds the block totals in order: the same additions in
// the same order, the zeros of the 112 further slots change nothing.
template <bool VEC>
__device__ __forceinline__ double kvs_mid_wave(const kvs_side & s, uint32_t w, uint32_t lane) {
    const uint32_t n = kvs_units(s, VEC);
    double acc = 0.0;
    if (n <= VX_SUM_ONE_WAVE_UNITS) { // (uniform) a sum of one wave's size: its order, by the first wave
        if (w) return 0.0;
        for (uint32_t e = lane; e < n; e += 64) kvs_unit<VEC>(s, e, true, acc);
        return vx_wave_sum(acc);
    }
    if (w * 64 >= n) return 0.0;
    for (uint32_t e = w * 64 + lane; e < n; e += 1024) kvs_unit<VEC>(s, e, true, acc);
    return vx_wave_sum(acc);
}

template <bool VK, bool VV>
__global__ __launch_bounds__(64) void kv_store_mid_kernel(const kvs_args a, double * partials) {
    const bool     second = blockIdx.x >= 16; // uniform
    const uint32_t w = blockIdx.x - (second ? 16 : 0);
    const double   t = second ? kvs_mid_wave<VV>(a.v, w, threadIdx.x) : kvs_mid_wave<VK>(a.k, w, threadIdx.x);
    double * half = partials + (second ? SUM_BLOCKS : 0);
    if (threadIdx.x == 0) half[w] = t;
    if (w == 0) for (int i = 16 + (int) threadIdx.x; i < SUM_BLOCKS; i += 64) half[i] = 0.0;
}

// the block totals of the two sums, added in block order, as the scalar of the SCALE node (256 threads)
__device__ __forceinline__ float kvs_scalar_of_totals(const kvs_args & a, const double * partials) {
    __shared__ double part[2 * SUM_BLOCKS];
    __shared__ float  y_s;
    static_assert(2 * SUM_BLOCKS == 256, "a partial per thread");
    part[threadIdx.x] = partials[threadIdx.x];
    __syncthreads();
    if (threadIdx.x == 0) {
        double tk = 0.0, tv = 0.0;
        for (int i = 0; i < SUM_BLOCKS; ++i) tk += part[i];               // (sum_partials_kernel's order)
        for (int i = 0; i < SUM_BLOCKS; ++i) tv += part[SUM_BLOCKS + i];
        y_s = kvs_scalar((float) tk, (float) tv, a.scale, a.bias);
    }
    __syncthreads();
    return y_s;
}

// the scalar alone, for a consumer that adds it itself (the prefill attention's epilogue)
__global__ __launch_bounds__(256) void kv_sync_scalar_kernel(const kvs_args a, const double * partials, float * y_out) {
    const float y = kvs_scalar_of_totals(a, partials);
    if (threadIdx.x == 0) *y_out = y;
}

__global__ __launch_bounds__(256) void kv_sync_add1_kernel(const kvs_args a, const double * partials) {
    const float y = kvs_scalar_of_totals(a, partials);
    const uint32_t n0 = (uint32_t) a.ne[0], n1 = (uint32_t) a.ne[1], n2 = (uint32_t) a.ne[2];
    const uint64_t nx = (uint64_t) n0 * n1 * (uint64_t) (n2 * a.ne[3]);
    if (a.dense4) { // (a prefill's attention output: 256 MiB at 16 x 4096 tokens; element by element with its index
        // arithmetic this pass took 228 us)
        const float4_t * px = (const float4_t *) a.x;
        float4_t *       pd = (float4_t *) a.d;
        for (uint64_t e = (uint64_t) blockIdx.x * 256 + threadIdx.x; e < nx / 4; e += (uint64_t) gridDim.x * 256) pd[e] = px[e] + y;
        return;
    }
    for (uint64_t e = (uint64_t) blockIdx.x * 256 + threadIdx.x; e < nx; e += (uint64_t) gridDim.x * 256) {
        uint64_t r = e;
        const uint32_t i0 = (uint32_t) (r % n0); r /= n0;
        const uint32_t i1 = (uint32_t) (r % n1); r /= n1;
        const uint32_t i2 = (uint32_t) (r % n2), i3 = (uint32_t) (r / n2);
        const uint64_t ox = i0 * a.nbx[0] + i1 * a.nbx[1] + i2 * a.nbx[2] + i3 * a.nbx[3];
        const uint64_t od = i0 * a.nbd[0] + i1 * a.nbd[1] + i2 * a.nbd[2] + i3 * a.nbd[3];
        *(float *) (a.d + od) = *(const float *) (a.x + ox) + y;  // the ADD1 node
    }
}

} // namespace

// ================================================================================== C ABI

extern "C" int vx_supports_binary(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst) {
    if (op < VX_BIN_ADD || op > VX_BIN_DIV) return 0;
    if (!f32(src0) || !f32(src1) || !f32(dst)) return 0;
    if (!vx_positive(src0) || !vx_same_shape(src0, dst) || !can_repeat(src1, src0)) return 0;
    return nb_multiple(src0, 4) && nb_multiple(src1, 4) && nb_multiple(dst, 4);
}

extern "C" vx_status vx_binary(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_binary(op, src0, src1, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "binary op %d: F32 operands, src1 repeatable over src0", op);
    if (!src0->data || !src1->data || !dst->data) return vx_fail(VX_ERR_INVALID, "binary op: null data");
    ew_args a; ew_fill(a, src0, src1, dst);
    switch (op) {
        case VX_BIN_ADD: return ew_launch<EW_ADD>(a, (hipStream_t) stream);
        case VX_BIN_SUB: return ew_launch<EW_SUB>(a, (hipStream_t) stream);
        case VX_BIN_MUL: return ew_launch<EW_MUL>(a, (hipStream_t) stream);
        default:         return ew_launch<EW_DIV>(a, (hipStream_t) stream);
    }
}

extern "C" int vx_supports_add1(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst) {
    if (!f32(src0) || !f32(src1) || !f32(dst)) return 0;
    if (!vx_positive(src0) || !vx_same_shape(src0, dst) || vx_nelements(src1) != 1) return 0;
    return nb_multiple(src0, 4) && nb_multiple(dst, 4);
}

extern "C" vx_status vx_add1(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_add1(src0, src1, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "add1: F32 tensor plus F32 scalar");
    if (!src0->data || !src1->data || !dst->data) return vx_fail(VX_ERR_INVALID, "add1: null data");
    ew_args a; ew_fill(a, src0, nullptr, dst);
    a.s1 = (const char *) src1->data;
    return ew_launch<EW_ADD1>(a, (hipStream_t) stream);
}

extern "C" int vx_supports_unary_like(const vx_tensor * src, const vx_tensor * dst) {
    if (!f32(src) || !f32(dst)) return 0;
    if (!vx_positive(src) || !vx_same_shape(src, dst)) return 0;
    return nb_multiple(src, 4) && nb_multiple(dst, 4);
}

extern "C" vx_status vx_scale(const vx_tensor * src, const vx_tensor * dst, float scale, float bias, vx_stream stream) {
    if (!vx_supports_unary_like(src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "scale: F32 tensors of one shape");
    if (!src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "scale: null data");
    ew_args a; ew_fill(a, src, nullptr, dst);
    a.p0 = scale; a.p1 = bias;
    return ew_launch<EW_SCALE>(a, (hipStream_t) stream);
}

// SCALE(x) feeding ADD(a, .) and ADD(a, b) feeding SCALE, as one launch each; a, b/x, dst of one shape
extern "C" int vx_supports_fused_pair(const vx_tensor * a, const vx_tensor * b, const vx_tensor * dst) {
    if (!f32(a) || !f32(b) || !f32(dst)) return 0;
    if (!vx_positive(a) || !vx_same_shape(a, dst) || !vx_same_shape(a, b)) return 0;
    return nb_multiple(a, 4) && nb_multiple(b, 4) && nb_multiple(dst, 4);
}

extern "C" vx_status vx_scale_add(const vx_tensor * a, const vx_tensor * x, const vx_tensor * dst, float scale, vx_stream stream) {
    if (!vx_supports_fused_pair(a, x, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "scale_add: F32 tensors of one shape");
    if (!a->data || !x->data || !dst->data) return vx_fail(VX_ERR_INVALID, "scale_add: null data");
    ew_args e; ew_fill(e, a, x, dst);
    e.p0 = scale;
    return ew_launch<EW_SCALE_ADD>(e, (hipStream_t) stream);
}

extern "C" vx_status vx_add_scale(const vx_tensor * a, const vx_tensor * b, const vx_tensor * dst, float scale, float bias,
                                  vx_stream stream) {
    if (!vx_supports_fused_pair(a, b, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "add_scale: F32 tensors of one shape");
    if (!a->data || !b->data || !dst->data) return vx_fail(VX_ERR_INVALID, "add_scale: null data");
    ew_args e; ew_fill(e, a, b, dst);
    e.p0 = scale; e.p1 = bias;
    return ew_launch<EW_ADD_SCALE>(e, (hipStream_t) stream);
}

extern "C" int vx_supports_unary(int op, const vx_tensor * src, const vx_tensor * dst) {
    switch (op) {
        case VX_UNARY_ABS: case VX_UNARY_SGN: case VX_UNARY_NEG: case VX_UNARY_STEP: case VX_UNARY_TANH:
        case VX_UNARY_RELU: case VX_UNARY_SIGMOID: case VX_UNARY_SILU: case VX_UNARY_EXP:
        case VX_UNARY_FLOOR: case VX_UNARY_CEIL: case VX_UNARY_ROUND: case VX_UNARY_TRUNC:
        case VX_UNARY_SQR: case VX_UNARY_SQRT: case VX_UNARY_LOG: case VX_UNARY_SIN: case VX_UNARY_COS: break;
        default: return 0;
    }
    return vx_supports_unary_like(src, dst);
}

extern "C" vx_status vx_unary(int op, const vx_tensor * src, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_unary(op, src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "unary op %d: F32 tensors of one shape", op);
    if (!src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "unary: null data");
    ew_args a; ew_fill(a, src, nullptr, dst);
    a.aux = op;
    return ew_launch<EW_UNARY>(a, (hipStream_t) stream);
}

extern "C" int vx_supports_glu(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst) {
    if (op != VX_GLU_SWIGLU && op != VX_GLU_REGLU) return 0;
    if (!f32(src0) || !f32(dst) || (src1 && !f32(src1))) return 0;
    if (!vx_positive(src0) || src0->nb[0] != 4 || dst->nb[0] != 4) return 0;
    if (src1) {
        if (!vx_same_shape(src0, src1) || !vx_same_shape(src0, dst) || src1->nb[0] != 4) return 0;
        if (!nb_multiple(src1, 4)) return 0;
    } else {
        if (src0->ne[0] % 2 || dst->ne[0] != src0->ne[0] / 2) return 0;
        for (int i = 1; i < 4; ++i) if (dst->ne[i] != src0->ne[i]) return 0;
    }
    return nb_multiple(src0, 4) && nb_multiple(dst, 4);
}

extern "C" vx_status vx_glu(int op, const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int swapped,
                            vx_stream stream) {
    if (!vx_supports_glu(op, src0, src1, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "glu op %d: F32 SWIGLU / REGLU with dense rows", op);
    if (!src0->data || !dst->data || (src1 && !src1->data)) return vx_fail(VX_ERR_INVALID, "glu: null data");
    // one tensor: the row's halves are the two operands (ops.cpp:3165-3168); `swapped` only
    // applies there.  x feeds the activation, y the gate.
    vx_tensor x = *src0, y = src1 ? *src1 : *src0;
    if (!src1) {
        const int64_t nc = src0->ne[0] / 2;
        x.ne[0] = y.ne[0] = nc;
        x.data = (char *) src0->data + (swapped ? nc * 4 : 0);
        y.data = (char *) src0->data + (swapped ? 0 : nc * 4);
    }
    ew_args a; ew_fill(a, &x, &y, dst);
    a.aux = op;
    return ew_launch<EW_GLU>(a, (hipStream_t) stream);
}

extern "C" int vx_supports_cpy(const vx_tensor * src, const vx_tensor * dst) {
    if (!src || !dst) return 0;
    // F32 / F16 in any combination; I32 to and from F32 (ggml_cast of position ids) and I32 to I32
    const bool ints = (src->type == VX_TYPE_I32 && (dst->type == VX_TYPE_F32 || dst->type == VX_TYPE_I32)) ||
                      (src->type == VX_TYPE_F32 && dst->type == VX_TYPE_I32);
    if (!ints && (!fl_type(src->type) || !fl_type(dst->type))) return 0;
    if (!vx_positive(src) || !vx_positive(dst) || vx_nelements(src) != vx_nelements(dst)) return 0;
    return nb_multiple(src, vx_type_size(src->type)) && nb_multiple(dst, vx_type_size(dst->type));
}

extern "C" vx_status vx_cpy(const vx_tensor * src, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_cpy(src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "cpy: F32/F16 (or I32 <-> F32) tensors holding the same number of elements");
    if (!src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "cpy: null data");
    cpy_args a;
    a.s = (const char *) src->data; a.d = (char *) dst->data; a.n = vx_nelements(src);
    for (int i = 0; i < 4; ++i) { a.nes[i] = src->ne[i]; a.ned[i] = dst->ne[i]; a.nbs[i] = src->nb[i]; a.nbd[i] = dst->nb[i]; }
    const size_t ss = vx_type_size(src->type), ds = vx_type_size(dst->type);
    const bool vec = src->ne[0] % 4 == 0 && dst->ne[0] % 4 == 0 && src->nb[0] == ss && dst->nb[0] == ds &&
                     (uintptr_t) src->data % (4 * ss) == 0 && (uintptr_t) dst->data % (4 * ds) == 0 &&
                     src->nb[1] % (4 * ss) == 0 && src->nb[2] % (4 * ss) == 0 && src->nb[3] % (4 * ss) == 0 &&
                     dst->nb[1] % (4 * ds) == 0 && dst->nb[2] % (4 * ds) == 0 && dst->nb[3] % (4 * ds) == 0;
    hipStream_t st = (hipStream_t) stream;
    if (src->type == VX_TYPE_I32) {
        return dst->type == VX_TYPE_I32 ? cpy_launch<int32_t, int32_t>(a, vec, st) : cpy_launch<int32_t, float>(a, vec, st);
    }
    if (dst->type == VX_TYPE_I32) return cpy_launch<float, int32_t>(a, vec, st);
    if (src->type == VX_TYPE_F32) {
        return dst->type == VX_TYPE_F32 ? cpy_launch<float, float>(a, vec, st) : cpy_launch<float, _Float16>(a, vec, st);
    }
    return dst->type == VX_TYPE_F32 ? cpy_launch<_Float16, float>(a, vec, st) : cpy_launch<_Float16, _Float16>(a, vec, st);
}

extern "C" int vx_supports_concat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int dim) {
    if (!src0 || !src1 || !dst || dim < 0 || dim > 3) return 0;
    if (src0->type != src1->type || src0->type != dst->type) return 0;
    if (src0->type != VX_TYPE_F32 && src0->type != VX_TYPE_F16 && src0->type != VX_TYPE_I32) return 0;
    if (!vx_positive(src0) || !vx_positive(src1)) return 0;
    for (int i = 0; i < 4; ++i) {
        if (i == dim) { if (dst->ne[i] != src0->ne[i] + src1->ne[i]) return 0; }
        else if (src0->ne[i] != src1->ne[i] || dst->ne[i] != src0->ne[i]) return 0;
    }
    const uint64_t es = vx_type_size(src0->type);
    return nb_multiple(src0, es) && nb_multiple(src1, es) && nb_multiple(dst, es);
}

extern "C" vx_status vx_concat(const vx_tensor * src0, const vx_tensor * src1, const vx_tensor * dst, int dim, vx_stream stream) {
    if (!vx_supports_concat(src0, src1, dst, dim)) return vx_fail(VX_ERR_UNSUPPORTED, "concat: F32/F16/I32 tensors equal outside dim %d", dim);
    if (!src0->data || !src1->data || !dst->data) return vx_fail(VX_ERR_INVALID, "concat: null data");
    cat_args a;
    a.s0 = (const char *) src0->data; a.s1 = (const char *) src1->data; a.d = (char *) dst->data; a.dim = dim;
    for (int i = 0; i < 4; ++i) {
        a.ne[i] = dst->ne[i]; a.ne0[i] = src0->ne[i];
        a.nb0[i] = src0->nb[i]; a.nb1[i] = src1->nb[i]; a.nbd[i] = dst->nb[i];
    }
    const int es = (int) vx_type_size(src0->type);
    const int epu = 16 / es;
    auto dense16 = [&](const vx_tensor * t) {
        return t->nb[0] == (uint64_t) es && (uintptr_t) t->data % 16 == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
    };
    const bool vec = dim != 0 && dst->ne[0] % epu == 0 && dense16(src0) && dense16(src1) && dense16(dst);
    const int64_t n_el = vx_nelements(dst);
    a.n = vec ? n_el / epu : n_el;
    const int64_t blocks = (a.n + 255) / 256;
    if (blocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "concat: launch too large");
    const dim3 grid((unsigned) blocks), block(256);
    hipStream_t st = (hipStream_t) stream;
    if (vec)          { if (es == 4) vx_launch(concat_kernel<16, 4>, grid, block, 0, st, a); else vx_launch(concat_kernel<16, 2>, grid, block, 0, st, a); }
    else if (es == 4) vx_launch(concat_kernel<4, 4>, grid, block, 0, st, a);
    else              vx_launch(concat_kernel<2, 2>, grid, block, 0, st, a);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

extern "C" int vx_supports_concat_many(const vx_tensor * const * srcs, const int64_t * extents, int n_src, int dim, const vx_tensor * dst) {
    if (!srcs || !extents || !dst || n_src < 2 || n_src > CATM_MAX || dim < 0 || dim > 3) return 0;
    if (dst->type != VX_TYPE_F32 && dst->type != VX_TYPE_I32) return 0;
    if (!vx_positive(dst) || vx_nelements(dst) >= ((int64_t) 1 << 31) || !nb_multiple(dst, 4) || dst->nb[0] != 4) return 0;
    int64_t total = 0;
    for (int k = 0; k < n_src; ++k) {
        const vx_tensor * t = srcs[k];
        if (!t || t->type != dst->type || !vx_positive(t) || t->nb[0] != 4 || !nb_multiple(t, 4)) return 0;
        for (int q = 0; q < 4; ++q) {
            const int64_t slot = q == dim ? extents[k] : dst->ne[q];
            if (slot <= 0 || slot % t->ne[q]) return 0;
        }
        total += extents[k];
    }
    return total == dst->ne[dim];
}

extern "C" vx_status vx_concat_many(const vx_tensor * const * srcs, const int64_t * extents, int n_src, int dim, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_concat_many(srcs, extents, n_src, dim, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "concat_many: 2 to %d F32 / I32 sources whose shapes divide their slots along dim %d", CATM_MAX, dim);
    if (!dst->data) return vx_fail(VX_ERR_INVALID, "concat_many: null data");
    catm_args a = {};
    auto dense16 = [](const vx_tensor * t) {
        return (uintptr_t) t->data % 16 == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
    };
    bool vec = dim != 0 && dst->ne[0] % 4 == 0 && dense16(dst);
    int64_t end = 0;
    for (int k = 0; k < n_src; ++k) {
        const vx_tensor * t = srcs[k];
        if (!t->data) return vx_fail(VX_ERR_INVALID, "concat_many: null data");
        a.s[k].p = (const char *) t->data;
        end += extents[k];
        a.s[k].end = (uint32_t) end;
        for (int q = 0; q < 4; ++q) { a.s[k].ne[q] = (uint32_t) t->ne[q]; a.s[k].nb[q] = t->nb[q]; }
        vec = vec && t->ne[0] == dst->ne[0] && dense16(t); // 16 bytes per thread: whole rows side by side
    }
    a.d = (char *) dst->data; a.dim = dim; a.n_src = n_src;
    for (int q = 0; q < 4; ++q) { a.ne[q] = (uint32_t) dst->ne[q]; a.nbd[q] = dst->nb[q]; }
    a.n = (uint32_t) (vec ? vx_nelements(dst) / 4 : vx_nelements(dst));
    const dim3 grid((a.n + 255) / 256), block(256);
    if (vec) vx_launch(concat_many_kernel<true>, grid, block, 0, (hipStream_t) stream, a);
    else     vx_launch(concat_many_kernel<false>, grid, block, 0, (hipStream_t) stream, a);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

extern "C" int vx_supports_arange(const vx_tensor * dst) {
    return f32(dst) && vx_positive(dst) && vx_is_contiguous(dst);
}

extern "C" vx_status vx_arange(const vx_tensor * dst, float start, float step, vx_stream stream) {
    if (!vx_supports_arange(dst)) return vx_fail(VX_ERR_UNSUPPORTED, "arange: a contiguous F32 tensor");
    if (!dst->data) return vx_fail(VX_ERR_INVALID, "arange: null data");
    const int64_t n = vx_nelements(dst), blocks = (n + 255) / 256;
    if (blocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "arange: launch too large");
    vx_launch(arange_kernel, dim3((unsigned) blocks), dim3(256), 0, (hipStream_t) stream, (float *) dst->data, n, start, step);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

extern "C" int vx_supports_repeat(const vx_tensor * src, const vx_tensor * dst) {
    if (!src || !dst || src->type != dst->type) return 0;
    if (src->type != VX_TYPE_F32 && src->type != VX_TYPE_F16 && src->type != VX_TYPE_I32) return 0;
    if (!vx_positive(src) || !vx_positive(dst) || !can_repeat(src, dst)) return 0;
    const uint64_t es = vx_type_size(src->type);
    return nb_multiple(src, es) && nb_multiple(dst, es);
}

extern "C" vx_status vx_repeat(const vx_tensor * src, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_repeat(src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "repeat: F32/F16/I32, dst a whole multiple of src in every dim");
    if (!src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "repeat: null data");
    rep_args a;
    a.s = (const char *) src->data; a.d = (char *) dst->data;
    for (int i = 0; i < 4; ++i) { a.ne[i] = dst->ne[i]; a.nes[i] = src->ne[i]; a.nbs[i] = src->nb[i]; a.nbd[i] = dst->nb[i]; }
    const int es = (int) vx_type_size(src->type), epu = 16 / es;
    auto dense16 = [&](const vx_tensor * t) {
        return t->nb[0] == (uint64_t) es && (uintptr_t) t->data % 16 == 0 && t->nb[1] % 16 == 0 && t->nb[2] % 16 == 0 && t->nb[3] % 16 == 0;
    };
    const bool vec = src->ne[0] % epu == 0 && dense16(src) && dense16(dst);
    const int64_t n_el = vx_nelements(dst);
    a.n = vec ? n_el / epu : n_el;
    const int64_t blocks = (a.n + 255) / 256;
    if (blocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "repeat: launch too large");
    const dim3 grid((unsigned) blocks), block(256);
    hipStream_t st = (hipStream_t) stream;
    if (vec)          { if (es == 4) vx_launch(repeat_kernel<16, 4>, grid, block, 0, st, a); else vx_launch(repeat_kernel<16, 2>, grid, block, 0, st, a); }
    else if (es == 4) vx_launch(repeat_kernel<4, 4>, grid, block, 0, st, a);
    else              vx_launch(repeat_kernel<2, 2>, grid, block, 0, st, a);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

extern "C" int vx_supports_get_rows(const vx_tensor * table, const vx_tensor * rows, const vx_tensor * dst) {
    if (!table || !rows || !dst || rows->type != VX_TYPE_I32) return 0;
    const int tt = table->type;
    if (tt != VX_TYPE_F32 && tt != VX_TYPE_F16 && tt != VX_TYPE_Q8_0 && tt != VX_TYPE_I32) return 0;
    if (dst->type != (tt == VX_TYPE_I32 ? VX_TYPE_I32 : VX_TYPE_F32)) return 0;
    if (!vx_positive(table) || !vx_positive(rows) || !vx_positive(dst)) return 0;
    if (tt == VX_TYPE_Q8_0 && table->ne[0] % 32) return 0;
    // ggml_get_rows (ggml.c): dst = [ne00, ne10, ne11, ne12]; table matrices are picked by (i11, i12)
    if (rows->ne[3] != 1 || table->ne[2] != rows->ne[1] || table->ne[3] != rows->ne[2]) return 0;
    if (dst->ne[0] != table->ne[0] || dst->ne[1] != rows->ne[0] || dst->ne[2] != rows->ne[1] || dst->ne[3] != rows->ne[2]) return 0;
    if (table->nb[0] != vx_type_size(tt) || dst->nb[0] != 4) return 0;
    const uint64_t ts = tt == VX_TYPE_F16 || tt == VX_TYPE_Q8_0 ? 2 : 4;
    return nb_multiple(rows, 4) && nb_multiple(dst, 4) && table->nb[1] % ts == 0 && table->nb[2] % ts == 0 && table->nb[3] % ts == 0;
}

extern "C" vx_status vx_get_rows(const vx_tensor * table, const vx_tensor * rows, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_get_rows(table, rows, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "get_rows: F32/F16/Q8_0/I32 table with dense rows, I32 indices");
    if (!table->data || !rows->data || !dst->data) return vx_fail(VX_ERR_INVALID, "get_rows: null data");
    rows_args a;
    a.table = (const char *) table->data; a.idx = (const char *) rows->data; a.d = (char *) dst->data;
    a.nc = table->ne[0]; a.n_rows_table = table->ne[1];
    a.ne10 = rows->ne[0]; a.ne11 = rows->ne[1]; a.ne12 = rows->ne[2];
    a.nb01 = table->nb[1]; a.nb02 = table->nb[2]; a.nb03 = table->nb[3];
    a.nb10 = rows->nb[0]; a.nb11 = rows->nb[1]; a.nb12 = rows->nb[2];
    a.nb1 = dst->nb[1]; a.nb2 = dst->nb[2]; a.nb3 = dst->nb[3];
    a.nchunk = (a.nc + 255) / 256;
    const int64_t blocks = vx_nelements(rows) * a.nchunk;
    if (blocks > 0x7fffffff) return vx_fail(VX_ERR_UNSUPPORTED, "get_rows: launch too large");
    const dim3 grid((unsigned) blocks), block(256);
    hipStream_t st = (hipStream_t) stream;
    if (table->type == VX_TYPE_F16)       vx_launch(get_rows_kernel<1>, grid, block, 0, st, a);
    else if (table->type == VX_TYPE_Q8_0) vx_launch(get_rows_kernel<2>, grid, block, 0, st, a);
    else                                  vx_launch(get_rows_kernel<0>, grid, block, 0, st, a);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// ---- vx_small_graph -------------------------------------------------------------------------------
static bool sg_fits(const vx_tensor * t) {
    if (!t || !vx_positive(t) || vx_nelements(t) > SG_MAX_ELEMS) return false;
    for (int i = 0; i < 4; ++i) if (t->nb[i] > ((uint64_t) 1 << 40)) return false;
    return true;
}

extern "C" int vx_supports_small_node(const vx_small_node * nd) {
    if (!nd || !nd->dst || !sg_fits(nd->dst)) return 0;
    const vx_tensor * a = nd->src0, * b = nd->src1, * d = nd->dst;
    switch (nd->op) {
        case VX_NODE_ADD: case VX_NODE_SUB: case VX_NODE_MUL: case VX_NODE_DIV:
            return sg_fits(a) && sg_fits(b) && vx_supports_binary(nd->op - VX_NODE_ADD, a, b, d);
        case VX_NODE_ADD1:   return sg_fits(a) && b && vx_supports_add1(a, b, d);
        case VX_NODE_SCALE:  return sg_fits(a) && vx_supports_unary_like(a, d);
        case VX_NODE_UNARY:  return sg_fits(a) && vx_supports_unary(nd->aux, a, d);
        case VX_NODE_CPY:    return sg_fits(a) && vx_supports_cpy(a, d);
        case VX_NODE_CONCAT: return sg_fits(a) && sg_fits(b) && vx_supports_concat(a, b, d, nd->aux);
        case VX_NODE_REPEAT: return sg_fits(a) && vx_supports_repeat(a, d);
        case VX_NODE_SUM:    return sg_fits(a) && vx_supports_sum(a, d);
        case VX_NODE_ARANGE: return vx_supports_arange(d);
        case VX_NODE_SUM_ROWS: return sg_fits(a) && vx_supports_sum_rows(a, d);
        default:             return 0;
    }
}

static sg_tensor sg_desc(const vx_tensor * t) {
    sg_tensor r = {};
    r.lds = -1;
    if (!t) return r;
    r.p = (char *) t->data; r.type = t->type;
    for (int i = 0; i < 4; ++i) { r.ne[i] = (int32_t) t->ne[i]; r.nb[i] = (int64_t) t->nb[i]; }
    return r;
}

namespace {
// what the host remembers of the run so far: which tensors have an LDS image, and which bytes were written
struct sg_span { uintptr_t lo, hi; };
sg_span sg_span_of(const vx_tensor * t) {
    uintptr_t hi = (uintptr_t) t->data + vx_type_size(t->type);
    for (int i = 0; i < 4; ++i) hi += (uintptr_t) (t->ne[i] - 1) * t->nb[i];
    return { (uintptr_t) t->data, hi };
}
bool sg_same(const vx_tensor * a, const vx_tensor * b) {
    if (a->data != b->data || a->type != b->type) return false;
    for (int i = 0; i < 4; ++i) if (a->ne[i] != b->ne[i] || a->nb[i] != b->nb[i]) return false;
    return true;
}
struct sg_image { vx_tensor t; int32_t off; bool valid; };
// an operand reads a tensor's image when it IS that tensor, or a reshape of it (both dense: the same elements in the same
// row-major order -- ggml's RESHAPE / VIEW of a whole contiguous tensor, e.g. the [F * patch, requests] view that SUM_ROWS sums)
bool sg_reads_image(const vx_tensor * img, const vx_tensor * op) {
    if (sg_same(img, op)) return true;
    return img->data == op->data && img->type == op->type && vx_nelements(img) == vx_nelements(op) && vx_is_contiguous(img) && vx_is_contiguous(op);
}
} // namespace

extern "C" vx_status vx_small_graph(const vx_small_node * nodes, int n_nodes, vx_stream stream) {
    if (!nodes || n_nodes < 1 || n_nodes > SG_MAX_NODES) return vx_fail(VX_ERR_UNSUPPORTED, "small graph: 1 to %d nodes", SG_MAX_NODES);
    sg_args a = {};
    a.h.n = n_nodes;
    sg_image images[SG_MAX_NODES + SG_MAX_PRELOADS];
    sg_span  written[SG_MAX_NODES];
    vx_tensor written_t[SG_MAX_NODES];
    int n_images = 0, n_written = 0;
    int32_t lds_used = 0;
    for (int k = 0; k < n_nodes; ++k) {
        const vx_small_node & nd = nodes[k];
        if (!vx_supports_small_node(&nd)) return vx_fail(VX_ERR_UNSUPPORTED, "small graph: node %d (op %d) is not a small elementwise / copy / sum node", k, nd.op);
        if (!nd.dst->data || (nd.src0 && !nd.src0->data) || (nd.src1 && !nd.src1->data)) return vx_fail(VX_ERR_INVALID, "small graph: null data in node %d", k);
    }
    // operands that the run only reads get their images first (at most half of the slots, so that the nodes' own
    // destinations keep theirs): dense F32 / I32 tensors that overlap no destination of the run
    static const bool preload_allowed = [] { const char * e = getenv("VX_SMALL_GRAPH_PRELOAD"); return !(e && e[0] == '0'); }();
    for (int k = 0; k < n_nodes && preload_allowed; ++k) {
        const vx_tensor * ops[2] = { nodes[k].op == VX_NODE_ARANGE ? nullptr : nodes[k].src0, nodes[k].src1 };
        for (int o = 0; o < 2; ++o) {
            const vx_tensor * t = ops[o];
            if (!t || a.h.n_pre == SG_MAX_PRELOADS || vx_type_size(t->type) != 4 || !vx_is_contiguous(t)) continue;
            const int32_t cnt = (int32_t) vx_nelements(t);
            if (lds_used + cnt > SG_LDS_ELEMS / 2) continue;
            const sg_span sp = sg_span_of(t);
            bool keep = true;
            for (int m = 0; m < n_nodes && keep; ++m) {
                const sg_span d = sg_span_of(nodes[m].dst);
                keep = !(sp.lo < d.hi && d.lo < sp.hi);
            }
            for (int m = 0; m < n_images && keep; ++m) keep = !sg_same(&images[m].t, t);
            if (!keep) continue;
            a.h.pre[a.h.n_pre++] = { (const uint32_t *) t->data, (uint32_t) cnt, lds_used };
            a.h.pre_most = std::max(a.h.pre_most, (uint32_t) cnt);
            images[n_images++] = { *t, lds_used, true };
            lds_used += (cnt + 3) & ~3; // images start on 16-byte boundaries
        }
    }
    for (int k = 0; k < n_nodes; ++k) {
        const vx_small_node & nd = nodes[k];
        sg_node & g = a.node[k];
        struct { sg_tensor s0, s1, d; } gt; // the three descriptors while the node is put together
        gt.s0 = sg_desc(nd.op == VX_NODE_ARANGE ? nullptr : nd.src0); gt.s1 = sg_desc(nd.src1); gt.d = sg_desc(nd.dst);
        g.p0 = nd.p0; g.p1 = nd.p1; g.aux = nd.aux;
        switch (nd.op) {
            case VX_NODE_ADD: case VX_NODE_SUB: case VX_NODE_MUL: case VX_NODE_DIV: g.kind = SG_EW2; g.aux = nd.op - VX_NODE_ADD; break;
            case VX_NODE_ADD1:   g.kind = SG_ADD1; break;
            case VX_NODE_SCALE:  g.kind = SG_SCALE; break;
            case VX_NODE_UNARY:  g.kind = SG_UNARY; break;
            case VX_NODE_CPY:    g.kind = SG_CPY; break;
            case VX_NODE_CONCAT: g.kind = SG_CONCAT; break;
            case VX_NODE_REPEAT: g.kind = SG_REPEAT; break;
            case VX_NODE_SUM:    g.kind = SG_SUM; g.aux = nd.src0->ne[0] % 4 == 0 && al16(nd.src0->data, nd.src0->nb); break; // vx_sum's unit rule
            case VX_NODE_SUM_ROWS: g.kind = SG_SUM_ROWS; break;
            default:             g.kind = SG_ARANGE; break;
        }
        // operands: the LDS image of exactly this tensor, else memory -- after a full barrier if the run wrote there
        const vx_tensor * ops[2] = { nd.op == VX_NODE_ARANGE ? nullptr : nd.src0, nd.src1 };
        sg_tensor * gops[2] = { &gt.s0, &gt.s1 };
        for (int o = 0; o < 2; ++o) {
            if (!ops[o]) continue;
            for (int m = 0; m < n_images; ++m)
                if (images[m].valid && sg_reads_image(&images[m].t, ops[o])) gops[o]->lds = images[m].off;
            if (gops[o]->lds >= 0) continue;
            const sg_span sp = sg_span_of(ops[o]);
            for (int m = 0; m < n_written; ++m) if (sp.lo < written[m].hi && written[m].lo < sp.hi) g.wait_memory = 1;
        }
        // destination: keeps its image when it is rewritten as the same tensor; any other overlap retires the image
        // and orders the stores through memory
        const sg_span dsp = sg_span_of(nd.dst);
        int mine = -1;
        for (int m = 0; m < n_images; ++m) {
            if (!images[m].valid) continue;
            if (sg_same(&images[m].t, nd.dst)) { mine = m; continue; }
            const sg_span sp = sg_span_of(&images[m].t);
            if (dsp.lo < sp.hi && sp.lo < dsp.hi) images[m].valid = false;
        }
        for (int m = 0; m < n_written; ++m)
            if (dsp.lo < written[m].hi && written[m].lo < dsp.hi && !sg_same(&written_t[m], nd.dst)) g.wait_memory = 1;
        const int32_t cnt = (int32_t) vx_nelements(nd.dst);
        if (mine >= 0) {
            gt.d.lds = images[mine].off;
        } else if (lds_used + cnt <= SG_LDS_ELEMS) {
            images[n_images] = { *nd.dst, lds_used, true };
            gt.d.lds = lds_used;
            lds_used += (cnt + 3) & ~3;
            ++n_images;
        }
        // a private destination with an image is not stored at all (and so leaves no bytes for later nodes to wait for)
        const bool in_lds_only = (nd.flags & VX_SMALL_DST_PRIVATE) && gt.d.lds >= 0;
        if (in_lds_only) gt.d.p = nullptr;
        else { written[n_written] = dsp; written_t[n_written] = *nd.dst; ++n_written; }
        const sg_tensor * gts[3] = { &gt.s0, &gt.s1, &gt.d };
        for (int o = 0; o < 3; ++o)
            for (int q = 0; q < 4; ++q) { g.sh[o].ne[q] = gts[o]->ne[q]; g.sh[o].nb[q] = gts[o]->nb[q]; }
        g.fp[0] = gt.s0.p; g.fp[1] = gt.s1.p; g.fp[2] = gt.d.p;
        g.ftype[0] = gt.s0.type; g.ftype[1] = gt.s1.type; g.ftype[2] = gt.d.type;
        g.flds[0] = gt.s0.lds; g.flds[1] = gt.s1.lds; g.flds[2] = gt.d.lds;
        g.fn = (uint32_t) vx_nelements(nd.dst); g.fn0 = ops[0] ? (uint32_t) vx_nelements(ops[0]) : 0;
        // the flat forms: dense row-major tensors (or LDS images) indexed by the destination's element number
        if (vx_is_contiguous(nd.dst)) {
            auto flat_operand = [&](const vx_tensor * t, const sg_tensor & gt, int32_t * one) {
                *one = 0;
                if (vx_nelements(t) == 1) { *one = 1; return true; }
                return vx_same_shape(t, nd.dst) && (gt.lds >= 0 || vx_is_contiguous(t));
            };
            const bool f0 = ops[0] ? flat_operand(ops[0], gt.s0, &g.one0) : true;
            const bool f1 = ops[1] ? flat_operand(ops[1], gt.s1, &g.one1) : true;
            switch (g.kind) {
                case SG_EW2: case SG_SCALE: case SG_UNARY: if (f0 && f1) g.flat = 1; break;
                case SG_ADD1:   if (f0) g.flat = 1; break;
                case SG_REPEAT: if (g.one0) g.flat = 1; break; // one value over the whole destination
                case SG_ARANGE: g.flat = 1; break;
                case SG_CPY:    if (gt.s0.lds >= 0 || vx_is_contiguous(ops[0])) g.flat = 1; break; // element e -> element e whatever the shapes
                case SG_CONCAT: {
                    bool outer = true;
                    for (int q = nd.aux + 1; q < 4; ++q) outer = outer && nd.dst->ne[q] == 1;
                    if (outer && (gt.s0.lds >= 0 || vx_is_contiguous(ops[0])) && (gt.s1.lds >= 0 || vx_is_contiguous(ops[1]))) g.flat = 2;
                } break;
                default: break;
            }
        }
    }
    // the work-group: a thread per element of the largest node, in whole waves; a sum that takes the whole block's order
    // (more than one wave's units) needs all 1024
    int64_t most = 64;
    bool    block_sum = false;
    for (int k = 0; k < n_nodes; ++k) {
        most = std::max(most, vx_nelements(nodes[k].dst));
        if (a.node[k].kind == SG_SUM && vx_nelements(nodes[k].src0) / (a.node[k].aux ? 4 : 1) > VX_SUM_ONE_WAVE_UNITS) block_sum = true;
    }
    const unsigned threads = block_sum ? 1024u : (unsigned) std::min<int64_t>(1024, std::max<int64_t>(256, (most + 63) / 64 * 64));
    static_assert(sizeof(sg_args) <= 4096, "the node table rides in the kernel's argument block");
    const size_t smem = (size_t) lds_used * 4;
    // a run of dense F32 nodes (and one-wave sums) goes to the kernel that has nothing left to decode
    static const bool dense_allowed = [] { const char * e = getenv("VX_SMALL_GRAPH_DENSE"); return !(e && e[0] == '0'); }();
    sgd_args da = {};
    da.h = a.h;
    bool dense = dense_allowed && !block_sum;
    struct { int32_t off; int writer; bool quads; } wrote[SG_MAX_NODES]; // images written by the run: by which node, in which thread order
    sg_span touched[3 * SG_MAX_NODES]; // memory that the nodes since the last barrier read or stored
    int     n_touched = 0;
    int n_wrote = 0, last_barrier = 0;
    for (int k = 0; k < n_nodes && dense; ++k) {
        const sg_node & g = a.node[k];
        const vx_small_node & nd = nodes[k];
        sgd_op & op = da.op[k];
        const bool has0 = nd.op != VX_NODE_ARANGE && nd.src0, has1 = nd.src1 != nullptr;
        if ((has0 && g.ftype[0] != VX_TYPE_F32) || (has1 && g.ftype[1] != VX_TYPE_F32) || g.ftype[2] != VX_TYPE_F32) { dense = false; break; }
        op.n = g.fn; op.n0 = g.fn0; op.p0 = g.p0; op.p1 = g.p1; op.aux = g.aux;
        op.flags = (g.one0 ? SGD_ONE0 : 0) | (g.one1 ? SGD_ONE1 : 0) | (g.wait_memory ? SGD_WAIT_MEMORY : 0);
        op.s0_lds = has0 ? g.flds[0] : -1; op.s1_lds = has1 ? g.flds[1] : -1; op.d_lds = g.flds[2];
        op.s0 = has0 ? (const float *) g.fp[0] : nullptr; op.s1 = has1 ? (const float *) g.fp[1] : nullptr; op.d = (float *) g.fp[2];
        if (g.kind == SG_SUM) {
            if (g.flds[0] < 0 && !vx_is_contiguous(nd.src0)) { dense = false; break; }
            op.code = g.aux ? SGD_SUM4 : SGD_SUM1;
            op.n = (uint32_t) (vx_nelements(nd.src0) / (g.aux ? 4 : 1));
        } else if (g.kind == SG_SUM_ROWS) {
            if ((g.flds[0] < 0 && !vx_is_contiguous(nd.src0)) || !vx_is_contiguous(nd.dst)) { dense = false; break; }
            op.code = SGD_SUM_ROWS;
            op.n0 = (uint32_t) nd.src0->ne[0];
            op.n  = (uint32_t) (vx_nelements(nd.src0) / nd.src0->ne[0]);
        } else if (g.kind == SG_REPEAT && g.flat == 0) {
            // a dense source repeated block-wise (its leading dims are 1) or tile-wise (its trailing dims are 1)
            const vx_tensor * sr = nd.src0, * ds = nd.dst;
            if ((g.flds[0] < 0 && !vx_is_contiguous(sr)) || !vx_is_contiguous(ds)) { dense = false; break; }
            int64_t lead = 1, ns = vx_nelements(sr);
            int d0 = 0;
            while (d0 < 4 && sr->ne[d0] == 1) { lead *= ds->ne[d0]; ++d0; }
            bool blk = true, mod = true;
            for (int q = d0; q < 4; ++q) blk = blk && sr->ne[q] == ds->ne[q];
            int d1 = 4;
            while (d1 > 0 && sr->ne[d1 - 1] == 1) --d1;
            for (int q = 0; q < d1; ++q) mod = mod && sr->ne[q] == ds->ne[q];
            if (blk)      { op.code = SGD_COPY; op.flags |= SGD_BLK0; op.p0 = 1.0f / (float) lead; }
            else if (mod) { op.code = SGD_COPY; op.flags |= SGD_MOD0; op.p0 = 1.0f / (float) ns; op.n0 = (uint32_t) ns; }
            else          { dense = false; break; }
        } else if (g.kind == SG_EW2 && g.flat == 0) {
            // a dense second operand whose trailing dims are 1, under a first operand of the destination's shape
            const vx_tensor * x = nd.src0, * y = nd.src1, * ds = nd.dst;
            const bool x_ok = g.one0 || (vx_same_shape(x, ds) && (g.flds[0] >= 0 || vx_is_contiguous(x)));
            if (!x_ok || !vx_is_contiguous(ds) || (g.flds[1] < 0 && !vx_is_contiguous(y))) { dense = false; break; }
            int d1 = 4;
            while (d1 > 0 && y->ne[d1 - 1] == 1) --d1;
            bool tiled = true;
            for (int q = 0; q < d1; ++q) tiled = tiled && y->ne[q] == ds->ne[q];
            if (!tiled) { dense = false; break; }
            op.code = SGD_ADD + (uint32_t) g.aux;
            op.flags |= SGD_MOD1;
            op.aux = (int32_t) vx_nelements(y);
            op.p1 = 1.0f / (float) op.aux;
        } else if (g.flat == 2) {
            op.code = SGD_CONCAT;
        } else if (g.kind == SG_CONCAT && g.flat == 0) {
            // dense operands joined below the outermost dimension: blocks of the destination, each the first operand's part
            // followed by the second's
            const vx_tensor * x = nd.src0, * y = nd.src1, * ds = nd.dst;
            if (!vx_is_contiguous(ds) || (g.flds[0] < 0 && !vx_is_contiguous(x)) || (g.flds[1] < 0 && !vx_is_contiguous(y))) { dense = false; break; }
            int64_t inner = 1, in0 = 1;
            for (int q = 0; q <= nd.aux; ++q) { inner *= ds->ne[q]; in0 *= x->ne[q]; }
            if (inner <= in0 || inner >= (1 << 22)) { dense = false; break; }
            op.code = SGD_CONCAT;
            op.flags |= SGD_BLOCKS;
            op.n0 = (uint32_t) in0;
            op.aux = (int32_t) inner;
            op.p0 = 1.0f / (float) inner;
        } else if (g.flat == 1) {
            switch (g.kind) {
                case SG_EW2:    op.code = SGD_ADD + (uint32_t) g.aux; break;
                case SG_ADD1:   op.code = SGD_ADD1; break;
                case SG_SCALE:  op.code = SGD_SCALE; break;
                case SG_UNARY:  op.code = SGD_UNARY; break;
                case SG_ARANGE: op.code = SGD_ARANGE; break;
                default:        op.code = SGD_COPY; break; // CPY of dense F32, REPEAT of one value
            }
        } else {
            dense = false;
        }
        if (!dense) break;
        // 16 bytes per thread for the plain moves
        auto al = [&](const void * ptr, int32_t off) { return off >= 0 ? off % 4 == 0 : (uintptr_t) ptr % 16 == 0; };
        if ((op.code == SGD_CONCAT || (op.code == SGD_COPY && !g.one0 && !(op.flags & (SGD_BLK0 | SGD_MOD0)))) && op.n % 4 == 0 && al(op.s0, op.s0_lds) && (op.d_lds < 0 || op.d_lds % 4 == 0) &&
            (uintptr_t) op.d % 16 == 0 && (op.code == SGD_COPY || (op.n0 % 4 == 0 && al(op.s1, op.s1_lds))) && (!(op.flags & SGD_BLOCKS) || op.aux % 4 == 0)) {
            op.n0 = op.code == SGD_COPY ? op.n / 4 : op.n0 / 4;
            op.n /= 4;
            if (op.flags & SGD_BLOCKS) { op.aux /= 4; op.p0 = 1.0f / (float) op.aux; }
            op.code = op.code == SGD_COPY ? SGD_COPY4 : SGD_CONCAT4;
        }
        // which barriers the run can do without
        // (quads: the destination's elements are not written by thread e mod size -- readers of such an image meet a barrier)
        const bool quads = op.code == SGD_COPY4 || op.code == SGD_CONCAT4 || op.code == SGD_SUM_ROWS;
        const bool own_elements = !quads && op.code != SGD_CONCAT && op.code != SGD_SUM4 && op.code != SGD_SUM1 &&
                                  !(op.flags & (SGD_BLK0 | SGD_MOD0 | SGD_MOD1)); // thread e mod size reads element e
        bool need = g.wait_memory != 0;
        const int32_t src_lds[2] = { op.s0_lds, op.s1_lds };
        const bool    single[2]  = { g.one0 != 0, g.one1 != 0 || op.code == SGD_ADD1 }; // every thread reads element 0
        for (int o = 0; o < 2 && !need; ++o) {
            if (src_lds[o] < 0) continue;
            for (int m = 0; m < n_wrote; ++m) {
                if (wrote[m].off != src_lds[o] || wrote[m].writer < last_barrier) continue; // (preloaded, or published by a later barrier)
                // element 0 is thread 0's: a node of one element reads what thread 0 wrote
                const bool same_thread = own_elements && !wrote[m].quads && (!single[o] || op.n == 1);
                if (!same_thread) need = true;
            }
        }
        int mine = -1;
        for (int m = 0; m < n_wrote; ++m) if (wrote[m].off == op.d_lds) mine = m;
        if (mine >= 0) need = true; // a rewritten image may still have readers
        if (op.d_lds >= 0) {
            if (mine < 0) mine = n_wrote++;
            wrote[mine] = { op.d_lds, k, quads };
        }
        // ... and through memory: a destination that is stored must not overlap anything that a node since the last barrier
        // read from memory (another thread may still be reading it: a sum walks its operand with one wave while the other
        // waves go on) or stored there (two stores of different threads to one address land in either order)
        if (op.d) {
            const sg_span dsp = sg_span_of(nd.dst);
            for (int m = 0; m < n_touched && !need; ++m) if (dsp.lo < touched[m].hi && touched[m].lo < dsp.hi) need = true;
        }
        if (k > 0 && !need) op.flags |= SGD_NO_BARRIER;
        else              { last_barrier = k; n_touched = 0; }
        if (has0 && op.s0_lds < 0) touched[n_touched++] = sg_span_of(nd.src0);
        if (has1 && op.s1_lds < 0) touched[n_touched++] = sg_span_of(nd.src1);
        if (op.d)                  touched[n_touched++] = sg_span_of(nd.dst);
    }
    // VX_SMALL_GRAPH_EXPLAIN=1: say on stderr which node kept a run from the resolved kernel
    static const bool explain = [] { const char * e = getenv("VX_SMALL_GRAPH_EXPLAIN"); return e && e[0] == '1'; }();
    if (explain && !dense) {
        int k = 0;
        while (k + 1 < n_nodes && da.op[k + 1].n != 0) ++k; // the nodes behind the one that failed were not looked at
        fprintf(stderr, "small graph of %d nodes: general kernel%s\n", n_nodes, block_sum ? " (a sum in the whole block's order)" : "");
        for (int q = 0; q < n_nodes; ++q) {
            const vx_small_node & nd = nodes[q];
            const vx_tensor * ts[3] = { nd.dst, nd.op == VX_NODE_ARANGE ? nullptr : nd.src0, nd.src1 };
            fprintf(stderr, "  node %d op %d aux %d flat %d%s:", q, nd.op, nd.aux, a.node[q].flat, q == k ? "  <- first unresolved" : "");
            for (const vx_tensor * t : ts)
                if (t) fprintf(stderr, " [%lld %lld %lld %lld | %llu %llu %llu %llu t%d]", (long long) t->ne[0], (long long) t->ne[1], (long long) t->ne[2],
                               (long long) t->ne[3], (unsigned long long) t->nb[0], (unsigned long long) t->nb[1], (unsigned long long) t->nb[2],
                               (unsigned long long) t->nb[3], t->type);
            fprintf(stderr, "\n");
        }
    }
    if (smem > 48 * 1024) { // a kernel has to be told once that it may be given more dynamic LDS than the default limit
        static bool raised[2] = { false, false };
        if (!raised[dense]) {
            const void * fn = dense ? (const void *) small_graph_dense_kernel : (const void *) small_graph_kernel;
            if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, SG_LDS_ELEMS * 4) != hipSuccess)
                return vx_fail(VX_ERR_HIP, "small graph: %s", hipGetErrorString(hipGetLastError()));
            raised[dense] = true;
        }
    }
    if (dense) {
        vx_launch(small_graph_dense_kernel, dim3(1), dim3(threads), smem, (hipStream_t) stream, da);
    } else {
        vx_launch(small_graph_kernel, dim3(1), dim3(threads), smem, (hipStream_t) stream, a);
    }
    VX_LAUNCH_CHECK();
    return VX_OK;
}

extern "C" int vx_supports_sum(const vx_tensor * src, const vx_tensor * dst) {
    if (!f32(src) || !f32(dst)) return 0;
    if (!vx_positive(src) || vx_nelements(dst) != 1) return 0;
    // rows must be dense: ggml-cpu asserts nb[0] == sizeof(float) (ops.cpp:1286) and reads rows as
    // contiguous regardless.  One block walks the tensor: meant for the small tensors the graphs sum.
    return src->nb[0] == 4 && vx_nelements(src) <= (int64_t) 1 << 24 && nb_multiple(src, 4);
}

extern "C" vx_status vx_sum(const vx_tensor * src, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_sum(src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "sum: F32 tensor of at most 2^24 elements to an F32 scalar");
    if (!src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "sum: null data");
    const bool vec = src->ne[0] % 4 == 0 && al16(src->data, src->nb);
    hipStream_t st = (hipStream_t) stream;
    const int64_t units = vx_nelements(src) / (vec ? 4 : 1);
    double * partials = nullptr;
    int blocks = 1;
    if (units > 16 * 1024) { // more than 16 units per thread of one block: spread the walk
        void * ws = nullptr;
        const vx_status rc = vx_workspace(st, SUM_BLOCKS * sizeof(double), &ws);
        if (rc != VX_OK) return rc;
        partials = (double *) ws; blocks = SUM_BLOCKS;
    }
    const dim3 block(units <= VX_SUM_ONE_WAVE_UNITS ? 64 : 1024); // small sums are one wave's work
    if (vec) vx_launch(sum_kernel<true>, dim3(blocks), block, 0, st, (const char *) src->data, vx_dims_of(src), (float *) dst->data, partials);
    else     vx_launch(sum_kernel<false>, dim3(blocks), block, 0, st, (const char *) src->data, vx_dims_of(src), (float *) dst->data, partials);
    if (partials) vx_launch(sum_partials_kernel, dim3(1), dim3(SUM_BLOCKS), 0, st, partials, blocks, (float *) dst->data);
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// ---- GGML_OP_SUM_ROWS: one wave per row ---------------------------------------------------------
namespace {
__global__ __launch_bounds__(64) void sum_rows_kernel(const char * src, vx_dims s, char * dst, vx_dims d) {
    const uint32_t row = blockIdx.x;
    const uint32_t i1 = row % (uint32_t) s.ne[1], r2 = row / (uint32_t) s.ne[1], i2 = r2 % (uint32_t) s.ne[2], i3 = r2 / (uint32_t) s.ne[2];
    const float * x = (const float *) (src + i1 * s.nb[1] + i2 * s.nb[2] + i3 * s.nb[3]);
    double acc = 0.0;
    for (int64_t i = threadIdx.x; i < s.ne[0]; i += 64) acc += (double) x[i];
    acc = vx_wave_sum(acc);
    if (threadIdx.x == 0) *(float *) (dst + i1 * d.nb[1] + i2 * d.nb[2] + i3 * d.nb[3]) = (float) acc;
}
} // namespace

extern "C" int vx_supports_sum_rows(const vx_tensor * src, const vx_tensor * dst) {
    if (!f32(src) || !f32(dst) || !vx_positive(src)) return 0;
    if (dst->ne[0] != 1 || dst->ne[1] != src->ne[1] || dst->ne[2] != src->ne[2] || dst->ne[3] != src->ne[3]) return 0;
    if (src->nb[0] != 4 || !nb_multiple(src, 4) || !nb_multiple(dst, 4)) return 0;
    return src->ne[1] * src->ne[2] * src->ne[3] <= 0x7fffffff;
}

extern "C" vx_status vx_sum_rows(const vx_tensor * src, const vx_tensor * dst, vx_stream stream) {
    if (!vx_supports_sum_rows(src, dst)) return vx_fail(VX_ERR_UNSUPPORTED, "sum_rows: F32 rows (nb0 == 4) to an F32 tensor of one element per row");
    if (!src->data || !dst->data) return vx_fail(VX_ERR_INVALID, "sum_rows: null data");
    const int64_t rows = src->ne[1] * src->ne[2] * src->ne[3];
    vx_launch(sum_rows_kernel, dim3((unsigned) rows), dim3(64), 0, (hipStream_t) stream, (const char *) src->data, vx_dims_of(src), (char *) dst->data, vx_dims_of(dst));
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// a prefill-sized write: both sums are ones that GGML_OP_SUM's kernel spreads over its 128 blocks (more than 16 Ki units)
static bool kvs_large(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot) {
    if (!kvs_side_ok(k, k_slot, (int64_t) 1 << 24) || !kvs_side_ok(v, v_slot, (int64_t) 1 << 24)) return false;
    kvs_side sk, sv;
    kvs_side_fill(sk, k, k_slot);
    kvs_side_fill(sv, v, v_slot);
    return vx_nelements(k) / (sk.vec ? 4 : 1) > 16 * 1024 && vx_nelements(v) / (sv.vec ? 4 : 1) > 16 * 1024;
}

// both sums are ones that GGML_OP_SUM's kernel forms in one block (at most 16 Ki units each), and at least one write is
// beyond what the one-launch form takes
static bool kvs_mid(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot) {
    if (!kvs_side_ok(k, k_slot, (int64_t) 1 << 24) || !kvs_side_ok(v, v_slot, (int64_t) 1 << 24)) return false;
    if (kvs_side_ok(k, k_slot) && kvs_side_ok(v, v_slot)) return false;
    kvs_side sk, sv;
    kvs_side_fill(sk, k, k_slot);
    kvs_side_fill(sv, v, v_slot);
    return vx_nelements(k) / (sk.vec ? 4 : 1) <= 16 * 1024 && vx_nelements(v) / (sv.vec ? 4 : 1) <= 16 * 1024;
}

extern "C" int vx_supports_kv_store_sync(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot,
                                         const vx_tensor * x, const vx_tensor * dst) {
    if (!k || !k_slot || !v || !v_slot || !x || !dst) return 0;
    if (!f32(x) || !f32(dst) || !vx_positive(x) || !vx_same_shape(x, dst) || !nb_multiple(x, 4) || !nb_multiple(dst, 4)) return 0;
    // (x of any size: beyond 16384 values the ADD1 is a launch of its own)
    return (kvs_side_ok(k, k_slot) && kvs_side_ok(v, v_slot)) || kvs_mid(k, k_slot, v, v_slot) || kvs_large(k, k_slot, v, v_slot)
               ? vx_nelements(x) < ((int64_t) 1 << 31) : 0;
}

// the launches of a mid-sized or prefill-sized write: stores and (wave or block) totals to partials
static void kvs_launch_store(const kvs_args & a, bool mid, double * partials, hipStream_t st) {
    if (mid) {
        const dim3 grid(32), block(64);
        if (a.k.vec && a.v.vec) vx_launch(kv_store_mid_kernel<true, true>, grid, block, 0, st, a, partials);
        else if (a.k.vec)       vx_launch(kv_store_mid_kernel<true, false>, grid, block, 0, st, a, partials);
        else if (a.v.vec)       vx_launch(kv_store_mid_kernel<false, true>, grid, block, 0, st, a, partials);
        else                    vx_launch(kv_store_mid_kernel<false, false>, grid, block, 0, st, a, partials);
        return;
    }
    const dim3 grid(2 * SUM_BLOCKS), block(1024);
    if (a.k.vec && a.v.vec) vx_launch(kv_store_large_kernel<true, true>, grid, block, 0, st, a, partials);
    else if (a.k.vec)       vx_launch(kv_store_large_kernel<true, false>, grid, block, 0, st, a, partials);
    else if (a.v.vec)       vx_launch(kv_store_large_kernel<false, true>, grid, block, 0, st, a, partials);
    else                    vx_launch(kv_store_large_kernel<false, false>, grid, block, 0, st, a, partials);
}

extern "C" vx_status vx_kv_store_sync(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot,
                                      const vx_tensor * x, const vx_tensor * dst, float scale, float bias, vx_stream stream) {
    if (!vx_supports_kv_store_sync(k, k_slot, v, v_slot, x, dst))
        return vx_fail(VX_ERR_UNSUPPORTED, "kv_store_sync: F32 tensors; both cache writes of at most 16 Ki units (of four elements where rows are 16-byte aligned), or both of more");
    if (!k->data || !k_slot->data || !v->data || !v_slot->data || !x->data || !dst->data) return vx_fail(VX_ERR_INVALID, "kv_store_sync: null data");
    kvs_args a;
    kvs_side_fill(a.k, k, k_slot);
    kvs_side_fill(a.v, v, v_slot);
    a.x = (const char *) x->data; a.d = (char *) dst->data;
    for (int i = 0; i < 4; ++i) { a.ne[i] = x->ne[i]; a.nbx[i] = x->nb[i]; a.nbd[i] = dst->nb[i]; }
    a.scale = scale; a.bias = bias;
    a.dense4 = vx_is_contiguous(x) && vx_is_contiguous(dst) && vx_nelements(x) % 4 == 0 && ((uintptr_t) x->data | (uintptr_t) dst->data) % 16 == 0;
    a.defer = nullptr;
    if (kvs_side_ok(k, k_slot) && kvs_side_ok(v, v_slot)) {
        // beyond a few thousand values of x the ADD1 is a launch of its own over many work-groups (the sums stay with the one
        // work-group whose order they are defined by); a workspace that cannot be had (a capture without a reservation)
        // leaves everything in the one launch
        void * ws = nullptr;
        if (vx_nelements(x) > 16384 && vx_workspace((hipStream_t) stream, 2 * SUM_BLOCKS * sizeof(double), &ws) == VX_OK) a.defer = (double *) ws;
        else (void) hipGetLastError();
        vx_launch(kv_store_sync_kernel, dim3(1), dim3(1024), 0, (hipStream_t) stream, a);
        if (a.defer) {
            const int64_t nx = vx_nelements(x);
            vx_launch(kv_sync_add1_kernel, dim3((unsigned) std::min<int64_t>((nx + 1023) / 1024, 4096)), dim3(256), 0, (hipStream_t) stream, a, (const double *) a.defer);
        }
    } else { // a prompt's or a prefill's write: stores and wave or block totals, then totals, scalar and ADD1
        void * ws = nullptr;
        const vx_status rc = vx_workspace((hipStream_t) stream, 2 * SUM_BLOCKS * sizeof(double), &ws);
        if (rc != VX_OK) return rc;
        hipStream_t st = (hipStream_t) stream;
        kvs_launch_store(a, kvs_mid(k, k_slot, v, v_slot), (double *) ws, st);
        const int64_t nx = vx_nelements(x);
        const unsigned blocks = (unsigned) std::min<int64_t>((nx + 1023) / 1024, 4096);
        vx_launch(kv_sync_add1_kernel, dim3(blocks), dim3(256), 0, st, a, (const double *) ws);
    }
    VX_LAUNCH_CHECK();
    return VX_OK;
}

// The cache write and the ordering scalar of vx_kv_store_sync without its ADD1: the scalar goes to y_out for a kernel
// launched behind this call on the same stream to add.  partials: 2 * SUM_BLOCKS doubles of device memory.
bool vx_kv_store_scalar_ok(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot) {
    // (a prompt's or a prefill's write: attention shapes with a smaller one do not reach the kernel that adds the scalar)
    return k && k_slot && v && v_slot && (kvs_mid(k, k_slot, v, v_slot) || kvs_large(k, k_slot, v, v_slot));
}

vx_status vx_kv_store_scalar(const vx_tensor * k, const vx_tensor * k_slot, const vx_tensor * v, const vx_tensor * v_slot,
                             float scale, float bias, void * partials, float * y_out, hipStream_t st) {
    if (!vx_kv_store_scalar_ok(k, k_slot, v, v_slot)) return vx_fail(VX_ERR_UNSUPPORTED, "kv_store_scalar: shapes vx_kv_store_sync does not take");
    kvs_args a;
    kvs_side_fill(a.k, k, k_slot);
    kvs_side_fill(a.v, v, v_slot);
    a.x = nullptr; a.d = nullptr;
    for (int i = 0; i < 4; ++i) { a.ne[i] = 0; a.nbx[i] = 0; a.nbd[i] = 0; }
    a.scale = scale; a.bias = bias;
    a.dense4 = 0;
    a.defer = nullptr;
    kvs_launch_store(a, kvs_mid(k, k_slot, v, v_slot), (double *) partials, st);
    vx_launch(kv_sync_scalar_kernel, dim3(1), dim3(256), 0, st, a, (const double *) partials, y_out);
    VX_LAUNCH_CHECK();
    return VX_OK;
}
