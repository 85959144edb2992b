"""Python-side plumbing over libvoxcpm_gfx950.so (the C ABI in include/voxcpm_gfx950.h).

The product is the shared library and the ggml backend plugin beside it; this package
only loads the library with ctypes and wraps torch tensors (used purely as device memory
and streams) into the library's tensor descriptors, for the parity tests and bench.py.
There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(_HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libvoxcpm_gfx950.so")
PLUGIN_PATH = os.path.join(LIB_DIR, "libggml-gfx950.so")

F32, F16, Q8_0, I32 = 0, 1, 8, 26
ACT_FLOAT, ACT_Q8 = 0, 1
QK8_0, Q8_BLOCK_BYTES = 32, 34


class VxError(RuntimeError):
    pass


class VxTensor(C.Structure):
    _fields_ = [
        ("type", C.c_int32),
        ("_pad", C.c_int32),
        ("ne", C.c_int64 * 4),
        ("nb", C.c_uint64 * 4),
        ("data", C.c_void_p),
    ]


class VxSmallNode(C.Structure):
    _fields_ = [
        ("op", C.c_int32),
        ("aux", C.c_int32),
        ("p0", C.c_float),
        ("p1", C.c_float),
        ("src0", C.POINTER(VxTensor)),
        ("src1", C.POINTER(VxTensor)),
        ("dst", C.POINTER(VxTensor)),
        ("flags", C.c_int32),
        ("reserved", C.c_int32),
    ]


SMALL_DST_PRIVATE = 1

EXPORTS = [
    "vx_device_count", "vx_init", "vx_last_error", "vx_device_info", "vx_malloc", "vx_free",
    "vx_malloc_host", "vx_free_host", "vx_memcpy_h2d", "vx_memcpy_d2h", "vx_memcpy_d2d", "vx_memset",
    "vx_stream_create", "vx_stream_destroy", "vx_stream_synchronize", "vx_workspace_reserve", "vx_workspace_info",
    "vx_graph_begin", "vx_graph_end", "vx_graph_launch", "vx_graph_destroy",
    "vx_graph_patchable", "vx_graph_patch_begin", "vx_graph_patch_end",
    "vx_weights_pin", "vx_weights_changed", "vx_weights_unpin", "vx_weights_info",
    "vx_rms_norm", "vx_rope", "vx_soft_max", "vx_flash_attn_ext", "vx_flash_attn_ext_static", "vx_mul_mat",
    "vx_supports_rms_norm", "vx_supports_rope", "vx_supports_soft_max", "vx_supports_flash_attn_ext",
    "vx_supports_mul_mat", "vx_kv_read_view", "vx_kv_write_view", "vx_kv_store",
    "vx_binary", "vx_add1", "vx_scale", "vx_unary", "vx_glu", "vx_cpy", "vx_concat", "vx_concat_many", "vx_supports_concat_many", "vx_sum", "vx_sum_rows", "vx_supports_sum_rows",
    "vx_supports_binary", "vx_supports_add1", "vx_supports_unary_like", "vx_supports_unary", "vx_supports_glu",
    "vx_supports_cpy", "vx_supports_concat", "vx_supports_sum",
    "vx_arange", "vx_repeat", "vx_get_rows", "vx_supports_arange", "vx_supports_repeat", "vx_supports_get_rows",
    "vx_small_graph", "vx_supports_small_node", "vx_mul_mat_sum_order",
    "vx_rms_norm_mul", "vx_scale_add", "vx_add_scale", "vx_flash_attn_ext_add1", "vx_mul_mat_swiglu", "vx_supports_mul_mat_swiglu", "vx_supports_mul_mat_swiglu_tiled", "vx_mul_mat_scale_add", "vx_supports_mul_mat_scale_add", "vx_kv_store_sync", "vx_supports_kv_store_sync", "vx_flash_attn_ext_kv2", "vx_supports_flash_attn_ext_kv2", "vx_flash_attn_ext_kv2_store", "vx_supports_flash_attn_ext_kv2_store", "vx_flash_attn_ext_store", "vx_supports_flash_attn_ext_store", "vx_flash_attn_ext_store_proj", "vx_supports_flash_attn_ext_store_proj", "vx_qkv_proj_rope", "vx_supports_qkv_proj_rope", "vx_kv_proj_rope", "vx_supports_kv_proj_rope", "vx_norm_qkv_proj_rope", "vx_supports_norm_qkv_proj_rope", "vx_norm_mul_mat_swiglu", "vx_supports_norm_qkv_proj_rope_tiled", "vx_supports_mlp_tiled", "vx_mlp_tiled", "vx_supports_norm_mul_mat_swiglu_tiled", "vx_supports_norm_mul_mat_swiglu", "vx_supports_rms_norm_mul", "vx_supports_fused_pair",
]

BIN_ADD, BIN_SUB, BIN_MUL, BIN_DIV = 0, 1, 2, 3
UNARY_ABS, UNARY_SGN, UNARY_NEG, UNARY_STEP, UNARY_TANH, UNARY_RELU, UNARY_SIGMOID, UNARY_SILU, UNARY_EXP = 0, 1, 2, 3, 4, 6, 7, 10, 13
UNARY_FLOOR, UNARY_CEIL, UNARY_ROUND, UNARY_TRUNC = 18, 19, 20, 21
UNARY_SQR, UNARY_SQRT, UNARY_LOG, UNARY_SIN, UNARY_COS = 100, 101, 102, 103, 104   # ggml's stand-alone ops
GLU_REGLU, GLU_SWIGLU = 0, 2
(NODE_ADD, NODE_SUB, NODE_MUL, NODE_DIV, NODE_ADD1, NODE_SCALE, NODE_UNARY, NODE_CPY, NODE_CONCAT, NODE_REPEAT, NODE_SUM,
 NODE_ARANGE, NODE_SUM_ROWS) = range(13)

_lib = None


def lib():
    """The loaded C library; raises VxError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise VxError(f"{LIB_PATH} is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                      "(or make -C voxcpm.cpp_amd/csrc) first")
    l = C.CDLL(LIB_PATH)
    TP = C.POINTER(VxTensor)
    vp, f32p, i32p = C.c_void_p, C.c_void_p, C.c_void_p  # device pointers travel as integers
    l.vx_last_error.restype = C.c_char_p
    l.vx_init.argtypes = [C.c_int]
    l.vx_device_info.argtypes = [C.c_int, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_int)]
    l.vx_malloc.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    l.vx_free.argtypes = [vp]
    l.vx_malloc_host.argtypes = [C.POINTER(C.c_void_p), C.c_size_t]
    l.vx_free_host.argtypes = [vp]
    for n in ("vx_memcpy_h2d", "vx_memcpy_d2h", "vx_memcpy_d2d"):
        getattr(l, n).argtypes = [vp, vp, C.c_size_t, vp]
    l.vx_memset.argtypes = [vp, C.c_int, C.c_size_t, vp]
    l.vx_stream_create.argtypes = [C.POINTER(C.c_void_p)]
    l.vx_stream_destroy.argtypes = [vp]
    l.vx_stream_synchronize.argtypes = [vp]
    l.vx_graph_begin.argtypes = [vp]
    l.vx_graph_end.argtypes = [vp, C.POINTER(C.c_void_p)]
    l.vx_graph_launch.argtypes = [vp, vp]
    l.vx_graph_destroy.argtypes = [vp]
    l.vx_graph_patchable.argtypes = [vp]
    l.vx_graph_patch_begin.argtypes = [vp]
    l.vx_graph_patch_end.argtypes = [vp, C.POINTER(C.c_int)]
    l.vx_weights_pin.argtypes = [vp, C.c_size_t]
    l.vx_weights_changed.argtypes = [vp, C.c_size_t]
    l.vx_weights_unpin.argtypes = [vp]
    l.vx_weights_info.argtypes = [C.POINTER(C.c_size_t)] * 3
    l.vx_workspace_reserve.argtypes = [vp, C.c_size_t]
    l.vx_workspace_info.argtypes = [vp, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.POINTER(C.c_int)]
    l.vx_rms_norm.argtypes = [TP, TP, C.c_float, vp]
    l.vx_rope.argtypes = [TP, i32p, f32p, TP, C.c_int, C.c_int, C.c_int] + [C.c_float] * 6 + [vp]
    l.vx_soft_max.argtypes = [TP, TP, f32p, TP, C.c_float, C.c_float, vp]
    l.vx_flash_attn_ext.argtypes = [TP, TP, TP, TP, f32p, TP, C.c_float, C.c_float, C.c_float, vp]
    l.vx_flash_attn_ext_static.argtypes = l.vx_flash_attn_ext.argtypes
    l.vx_mul_mat.argtypes = [TP, TP, TP, C.c_int, vp]
    l.vx_supports_rms_norm.argtypes = [TP, TP]
    l.vx_supports_rope.argtypes = [TP, TP, C.c_int, C.c_int]
    l.vx_supports_soft_max.argtypes = [TP, TP, TP]
    l.vx_supports_flash_attn_ext.argtypes = [TP, TP, TP, TP, TP]
    l.vx_supports_mul_mat.argtypes = [TP, TP, TP]
    l.vx_kv_read_view.argtypes = [TP, C.c_int, TP]
    l.vx_kv_write_view.argtypes = [TP, C.c_int, C.c_int, TP]
    l.vx_kv_store.argtypes = [TP, TP, vp]
    l.vx_binary.argtypes = [C.c_int, TP, TP, TP, vp]
    l.vx_add1.argtypes = [TP, TP, TP, vp]
    l.vx_scale.argtypes = [TP, TP, C.c_float, C.c_float, vp]
    l.vx_unary.argtypes = [C.c_int, TP, TP, vp]
    l.vx_glu.argtypes = [C.c_int, TP, TP, TP, C.c_int, vp]
    l.vx_cpy.argtypes = [TP, TP, vp]
    l.vx_concat.argtypes = [TP, TP, TP, C.c_int, vp]
    l.vx_concat_many.argtypes = [C.POINTER(TP), C.POINTER(C.c_int64), C.c_int, C.c_int, TP, vp]
    l.vx_supports_concat_many.argtypes = [C.POINTER(TP), C.POINTER(C.c_int64), C.c_int, C.c_int, TP]
    l.vx_sum.argtypes = [TP, TP, vp]
    l.vx_sum_rows.argtypes = [TP, TP, vp]
    l.vx_supports_sum_rows.argtypes = [TP, TP]
    l.vx_supports_binary.argtypes = [C.c_int, TP, TP, TP]
    l.vx_supports_add1.argtypes = [TP, TP, TP]
    l.vx_supports_unary_like.argtypes = [TP, TP]
    l.vx_supports_unary.argtypes = [C.c_int, TP, TP]
    l.vx_supports_glu.argtypes = [C.c_int, TP, TP, TP]
    l.vx_supports_cpy.argtypes = [TP, TP]
    l.vx_supports_concat.argtypes = [TP, TP, TP, C.c_int]
    l.vx_supports_sum.argtypes = [TP, TP]
    l.vx_arange.argtypes = [TP, C.c_float, C.c_float, vp]
    l.vx_repeat.argtypes = [TP, TP, vp]
    l.vx_get_rows.argtypes = [TP, TP, TP, vp]
    l.vx_supports_arange.argtypes = [TP]
    l.vx_supports_repeat.argtypes = [TP, TP]
    l.vx_supports_get_rows.argtypes = [TP, TP, TP]
    l.vx_small_graph.argtypes = [C.POINTER(VxSmallNode), C.c_int, vp]
    l.vx_supports_small_node.argtypes = [C.POINTER(VxSmallNode)]
    l.vx_mul_mat_sum_order.argtypes = [C.c_int64, C.c_int64, C.c_int64]
    l.vx_rms_norm_mul.argtypes = [TP, TP, TP, C.c_float, vp]
    l.vx_scale_add.argtypes = [TP, TP, TP, C.c_float, vp]
    l.vx_add_scale.argtypes = [TP, TP, TP, C.c_float, C.c_float, vp]
    l.vx_flash_attn_ext_add1.argtypes = [TP, TP, TP, TP, f32p, f32p, TP, C.c_float, C.c_float, C.c_float, vp]
    l.vx_mul_mat_swiglu.argtypes = [TP, TP, TP, TP, C.c_int, vp]
    l.vx_supports_mul_mat_swiglu.argtypes = [TP, TP, TP, TP]
    l.vx_supports_mul_mat_swiglu_tiled.argtypes = [TP, TP, TP, TP, C.c_int]
    l.vx_mul_mat_scale_add.argtypes = [TP, TP, TP, TP, C.c_float, C.c_int, vp]
    l.vx_supports_mul_mat_scale_add.argtypes = [TP, TP, TP, TP]
    l.vx_kv_store_sync.argtypes = [TP, TP, TP, TP, TP, TP, C.c_float, C.c_float, vp]
    l.vx_supports_kv_store_sync.argtypes = [TP, TP, TP, TP, TP, TP]
    l.vx_flash_attn_ext_kv2.argtypes = [TP, TP, TP, TP, TP, TP, f32p, TP, C.c_float, C.c_float, C.c_float, vp]
    l.vx_supports_flash_attn_ext_kv2.argtypes = [TP, TP, TP, TP, TP, TP, TP]
    l.vx_flash_attn_ext_kv2_store.argtypes = [TP, TP, TP, TP, TP, TP, f32p, TP, TP, TP, TP, TP] + [C.c_float] * 5 + [vp]
    l.vx_supports_flash_attn_ext_kv2_store.argtypes = [TP] * 11
    l.vx_flash_attn_ext_store.argtypes = [TP, TP, TP, TP, f32p, TP, TP, TP, TP, TP] + [C.c_float] * 5 + [vp]
    l.vx_supports_flash_attn_ext_store.argtypes = [TP] * 9 + [C.c_float]
    l.vx_flash_attn_ext_store_proj.argtypes = [TP, TP, TP, TP, f32p] + [TP] * 8 + [C.c_float] * 6 + [C.c_int, vp]
    l.vx_supports_flash_attn_ext_store_proj.argtypes = [TP] * 12 + [C.c_float, C.c_int]
    l.vx_qkv_proj_rope.argtypes = [TP, TP, TP, TP, i32p, f32p, TP, TP, TP, C.c_int, C.c_int, C.c_int] + [C.c_float] * 6 + [C.c_int, vp]
    l.vx_supports_qkv_proj_rope.argtypes = [TP, TP, TP, TP, TP, TP, TP, C.c_int, C.c_int]
    l.vx_kv_proj_rope.argtypes = [TP, TP, TP, i32p, f32p, TP, TP, C.c_int, C.c_int, C.c_int] + [C.c_float] * 6 + [C.c_int, vp]
    l.vx_supports_kv_proj_rope.argtypes = [TP, TP, TP, TP, TP, C.c_int, C.c_int]
    l.vx_norm_qkv_proj_rope.argtypes = [TP, TP, C.c_float, TP, TP, TP, i32p, f32p, TP, TP, TP, C.c_int, C.c_int, C.c_int] + [C.c_float] * 6 + [C.c_int, vp]
    l.vx_supports_norm_qkv_proj_rope.argtypes = [TP, TP, TP, TP, TP, TP, TP, TP, C.c_int, C.c_int]
    l.vx_supports_norm_qkv_proj_rope_tiled.argtypes = [TP, TP, TP, TP, TP, TP, TP, TP, C.c_int, C.c_int, C.c_int]
    l.vx_norm_mul_mat_swiglu.argtypes = [TP, TP, C.c_float, TP, TP, TP, C.c_int, vp]
    l.vx_supports_norm_mul_mat_swiglu.argtypes = [TP, TP, TP, TP, TP]
    l.vx_supports_norm_mul_mat_swiglu_tiled.argtypes = [TP, TP, TP, TP, TP, C.c_int]
    l.vx_supports_mlp_tiled.argtypes = [TP, TP, TP, TP, TP, TP, TP, C.c_int]
    l.vx_mlp_tiled.argtypes = [TP, TP, C.c_float, TP, TP, TP, TP, C.c_float, TP, C.c_int, vp]
    l.vx_supports_rms_norm_mul.argtypes = [TP, TP, TP]
    l.vx_supports_fused_pair.argtypes = [TP, TP, TP]
    _lib = l
    return l


def check(status, what=""):
    if status != 0:
        raise VxError(f"{what} failed with status {status}: {lib().vx_last_error().decode()}")


def make_desc(ttype, ne, nb, data):
    t = VxTensor()
    t.type = ttype
    for i in range(4):
        t.ne[i] = ne[i]
        t.nb[i] = nb[i]
    t.data = data
    return t


_TORCH_TYPES = None


def desc(t):
    """Descriptor of a torch tensor (<= 4 dims, any strides, last dim dense): numpy/torch
    shape (n3, n2, n1, n0) becomes ggml ne = [n0, n1, n2, n3]."""
    import torch
    global _TORCH_TYPES
    if _TORCH_TYPES is None:
        _TORCH_TYPES = {torch.float32: F32, torch.float16: F16, torch.int32: I32}
    if t is None:
        return None
    assert t.dim() <= 4
    es = t.element_size()
    shape = [1] * (4 - t.dim()) + list(t.shape)
    strides = [s * es for s in t.stride()]
    while len(strides) < 4:
        strides.insert(0, (strides[0] * shape[4 - len(strides)]) if strides else es)
    d = make_desc(_TORCH_TYPES[t.dtype], shape[::-1], strides[::-1], t.data_ptr())
    d._keep = t
    return d


def desc_q8(raw, ne0):
    """Descriptor of Q8_0 rows held in a contiguous uint8 torch tensor (..., rows, ne0/32*34)."""
    assert raw.is_contiguous() and raw.shape[-1] == ne0 // QK8_0 * Q8_BLOCK_BYTES
    shape = [1] * (4 - raw.dim()) + list(raw.shape)
    rowb = shape[3]
    d = make_desc(Q8_0, [ne0, shape[2], shape[1], shape[0]],
                  [Q8_BLOCK_BYTES, rowb, rowb * shape[2], rowb * shape[2] * shape[1]], raw.data_ptr())
    d._keep = raw
    return d


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _p(t):
    return None if t is None else t.data_ptr()


# ---- one function per ggml operator, same argument meaning as the ggml_* graph builders ----
def rms_norm(x, eps, out=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    check(lib().vx_rms_norm(desc(x), desc(out), eps, _stream()), "vx_rms_norm")
    return out


def rope_ext(x, pos, freq_factors, n_dims, mode, n_ctx_orig, freq_base, freq_scale, ext_factor,
             attn_factor, beta_fast, beta_slow, out=None):
    import torch
    out = torch.empty_like(x) if out is None else out
    check(lib().vx_rope(desc(x), _p(pos), _p(freq_factors), desc(out), n_dims, mode, n_ctx_orig, freq_base,
                        freq_scale, ext_factor, attn_factor, beta_fast, beta_slow, _stream()), "vx_rope")
    return out


def soft_max_ext(x, mask, scale, max_bias, sinks=None, out=None):
    import torch
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device) if out is None else out
    check(lib().vx_soft_max(desc(x), desc(mask), _p(sinks), desc(out), scale, max_bias, _stream()), "vx_soft_max")
    return out


def flash_attn_ext(q, k, v, mask, scale, max_bias=0.0, logit_softcap=0.0, sinks=None, out=None):
    """q (ne3, Hq, n_q, D) f32; k, v (ne3', Hkv, n_kv, D) f16|f32 (any row strides); mask
    (ne33, ne32, >=n_q, n_kv) f16 or None.  Returns (ne3, n_q, Hq, D) f32, ggml's permuted result."""
    import torch
    if out is None:
        out = torch.empty((q.shape[-4] if q.dim() == 4 else 1, q.shape[-2], q.shape[-3], v.shape[-1]),
                          dtype=torch.float32, device=q.device)
    check(lib().vx_flash_attn_ext(desc(q), desc(k), desc(v), desc(mask), _p(sinks), desc(out), scale, max_bias,
                                  logit_softcap, _stream()), "vx_flash_attn_ext")
    return out


def flash_attn_ext_static(q, k, v, mask, scale, max_bias=0.0, logit_softcap=0.0, sinks=None, out=None):
    """flash_attn_ext through the entry point that allocates nothing; `out` must be given by callers that
    may not allocate either."""
    import torch
    if out is None:
        out = torch.empty((q.shape[-4] if q.dim() == 4 else 1, q.shape[-2], q.shape[-3], v.shape[-1]),
                          dtype=torch.float32, device=q.device)
    check(lib().vx_flash_attn_ext_static(desc(q), desc(k), desc(v), desc(mask), _p(sinks), desc(out), scale, max_bias,
                                         logit_softcap, _stream()), "vx_flash_attn_ext_static")
    return out


def mul_mat(w, x, act_mode=ACT_FLOAT, w_ne0=None, out=None):
    """w: weights (ne03, ne02, rows, K) f16|f32, or Q8_0 bytes (.., rows, K/32*34) uint8 with
    w_ne0=K; x (ne13, ne12, tokens, K) f32.  Returns (ne13, ne12, tokens, rows) f32."""
    import torch
    wd = desc_q8(w, w_ne0) if w.dtype == torch.uint8 else desc(w)
    xd = desc(x)
    if out is None:
        shape = list(x.shape[:-1]) + [wd.ne[1]]
        out = torch.empty(shape, dtype=torch.float32, device=x.device)
    check(lib().vx_mul_mat(wd, xd, desc(out), act_mode, _stream()), "vx_mul_mat")
    return out


# ---- glue operators (torch dim d corresponds to ggml dim ndim-1-d) ----
def binary(op, a, b, out=None):
    import torch
    out = torch.empty_like(a) if out is None else out
    check(lib().vx_binary(op, desc(a), desc(b), desc(out), _stream()), "vx_binary")
    return out


def add1(a, b, out=None):
    import torch
    out = torch.empty_like(a) if out is None else out
    check(lib().vx_add1(desc(a), desc(b), desc(out), _stream()), "vx_add1")
    return out


def scale(a, s, bias=0.0, out=None):
    import torch
    out = torch.empty_like(a) if out is None else out
    check(lib().vx_scale(desc(a), desc(out), s, bias, _stream()), "vx_scale")
    return out


def unary(op, a, out=None):
    import torch
    out = torch.empty_like(a) if out is None else out
    check(lib().vx_unary(op, desc(a), desc(out), _stream()), "vx_unary")
    return out


def glu(op, a, b=None, swapped=False, out=None):
    import torch
    if out is None:
        shape = list(a.shape)
        if b is None:
            shape[-1] //= 2
        out = torch.empty(shape, dtype=torch.float32, device=a.device)
    check(lib().vx_glu(op, desc(a), desc(b), desc(out), int(swapped), _stream()), "vx_glu")
    return out


def cpy(src, dst):
    check(lib().vx_cpy(desc(src), desc(dst), _stream()), "vx_cpy")
    return dst


def concat(a, b, ggml_dim, out=None):
    import torch
    if out is None:
        shape = list(a.shape)
        shape[a.dim() - 1 - ggml_dim] += b.shape[b.dim() - 1 - ggml_dim]
        out = torch.empty(shape, dtype=a.dtype, device=a.device)
    check(lib().vx_concat(desc(a), desc(b), desc(out), ggml_dim, _stream()), "vx_concat")
    return out


def concat_many(srcs, extents, ggml_dim, out):
    """A tree of concatenations along one ggml dimension written from its leaves: source k fills extents[k] indices of
    `out` along that dimension and is repeated where it is smaller than its slot."""
    ds = [desc(t) for t in srcs]
    arr = (C.POINTER(VxTensor) * len(ds))(*[C.pointer(d) for d in ds])
    ext = (C.c_int64 * len(ds))(*extents)
    check(lib().vx_concat_many(arr, ext, len(ds), ggml_dim, desc(out), _stream()), "vx_concat_many")
    return out


def arange(start, stop, step, device="cuda"):
    """ggml_arange: ceil((stop - start) / step) values start + step * i."""
    import math
    import numpy as np
    import torch
    n = int(math.ceil((np.float32(stop) - np.float32(start)) / np.float32(step)))
    out = torch.empty((n,), dtype=torch.float32, device=device)
    check(lib().vx_arange(desc(out), start, step, _stream()), "vx_arange")
    return out


def repeat(a, shape, out=None):
    """ggml_repeat: `a` tiled to `shape` (torch order), each dim a whole multiple of a's."""
    import torch
    out = torch.empty(shape, dtype=a.dtype, device=a.device) if out is None else out
    check(lib().vx_repeat(desc(a), desc(out), _stream()), "vx_repeat")
    return out


def get_rows(table, rows, ne0=None, out=None):
    """ggml_get_rows: `table` a float / int32 torch tensor, or Q8_0 rows as uint8 with the row length `ne0`;
    `rows` int32 indices; result (..., rows, ne0) F32 (I32 for an I32 table)."""
    import torch
    td = desc_q8(table, ne0) if ne0 is not None else desc(table)
    nc = ne0 if ne0 is not None else table.shape[-1]
    if out is None:
        shape = list(rows.shape) + [nc]
        out = torch.empty(shape, dtype=torch.int32 if table.dtype == torch.int32 else torch.float32, device=rows.device)
    check(lib().vx_get_rows(td, desc(rows), desc(out), _stream()), "vx_get_rows")
    return out


def small_node(op, dst, src0=None, src1=None, aux=0, p0=0.0, p1=0.0, private=False):
    """One node of a small graph: tensors as descriptors (VxTensor) or torch tensors.  private: only later nodes of the
    same run read dst (it may then live in LDS only and its memory stay untouched)."""
    nd = VxSmallNode()
    nd.op, nd.aux, nd.p0, nd.p1 = op, aux, p0, p1
    nd.flags = SMALL_DST_PRIVATE if private else 0
    keep = []
    for name, t in (("src0", src0), ("src1", src1), ("dst", dst)):
        if t is None:
            continue
        d = t if isinstance(t, VxTensor) else desc(t)
        keep.append(d)
        setattr(nd, name, C.pointer(d))
    nd._keep = keep
    return nd


def small_graph(nodes):
    """Runs up to 16 tiny nodes (small_node) in the order given as one launch."""
    arr = (VxSmallNode * len(nodes))(*nodes)
    check(lib().vx_small_graph(arr, len(nodes), _stream()), "vx_small_graph")


def sum_rows(a, out=None):
    """GGML_OP_SUM_ROWS: every row (the innermost dimension) of an F32 tensor summed; shape (..., 1)."""
    import torch
    out = torch.empty(tuple(a.shape[:-1]) + (1,), dtype=torch.float32, device=a.device) if out is None else out
    check(lib().vx_sum_rows(desc(a), desc(out), _stream()), "vx_sum_rows")
    return out


def sum_all(a, out=None):
    import torch
    out = torch.empty((1,), dtype=torch.float32, device=a.device) if out is None else out
    check(lib().vx_sum(desc(a), desc(out), _stream()), "vx_sum")
    return out
