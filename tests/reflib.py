"""Test-side loaders and helpers for the two CPU checkers.

* ``oracle``  -- this repository's C restatement of the ggml-cpu algorithms
  (``oracle/liboracle.so``, built from ``oracle/oracle.c``).
* ``ref``     -- the reference's own ggml + ggml-cpu, compiled from the reference
  checkout into ``oracle/_ref/<isa>/`` and driven through ``oracle/ref_harness.cpp``.
  It exists only where it was prebuilt; tests that need it skip otherwise.

Tensors cross both C boundaries as a small descriptor (type, ne[4], nb[4] in bytes,
data pointer) in ggml's convention: ``ne[0]`` is the fastest dimension, so a numpy
array of shape ``(n3, n2, n1, n0)`` maps to ``ne = [n0, n1, n2, n3]``.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")

F32, F16, Q8_0, I32 = 0, 1, 8, 26
QK8_0 = 32
Q8_BLOCK_BYTES = 34


class Tensor(C.Structure):
    _fields_ = [
        ("type", C.c_int32),
        ("_pad", C.c_int32),
        ("ne", C.c_int64 * 4),
        ("nb", C.c_uint64 * 4),
        ("data", C.c_void_p),
    ]


_NP_TYPES = {np.dtype(np.float32): F32, np.dtype(np.float16): F16, np.dtype(np.int32): I32}


def desc(a, ttype=None):
    """Descriptor of a numpy array (any strides, at most 4 dims, last dim dense)."""
    assert a.ndim <= 4
    if ttype is None:
        ttype = _NP_TYPES[a.dtype]
    shape = (1,) * (4 - a.ndim) + tuple(a.shape)
    strides = list(a.strides)
    # leading broadcast dims get the stride ggml would give a dense tensor
    while len(strides) < 4:
        strides.insert(0, strides[0] * shape[4 - len(strides)] if strides else a.itemsize)
    t = Tensor()
    t.type = ttype
    for i in range(4):
        t.ne[i] = shape[3 - i]
        t.nb[i] = strides[3 - i]
    assert t.nb[0] == a.itemsize, "fastest dimension must be dense"
    t.data = a.ctypes.data
    t._keep = a
    return t


def desc_q8(raw, ne0):
    """Descriptor of a Q8_0 tensor held as uint8 rows: shape (..., rows, ne0/32*34)."""
    assert raw.dtype == np.uint8 and raw.flags.c_contiguous
    assert raw.shape[-1] == ne0 // QK8_0 * Q8_BLOCK_BYTES
    shape = (1,) * (4 - raw.ndim) + tuple(raw.shape)
    t = Tensor()
    t.type = Q8_0
    t.ne[0] = ne0
    t.ne[1], t.ne[2], t.ne[3] = shape[2], shape[1], shape[0]
    rowb = shape[3]
    t.nb[0] = Q8_BLOCK_BYTES
    t.nb[1] = rowb
    t.nb[2] = rowb * shape[2]
    t.nb[3] = rowb * shape[2] * shape[1]
    t.data = raw.ctypes.data
    t._keep = raw
    return t


def ptr(a, ctype):
    return None if a is None else a.ctypes.data_as(C.POINTER(ctype))


# ----------------------------------------------------------------------------- oracle
_oracle = None


def load_oracle():
    global _oracle
    if _oracle is not None:
        return _oracle
    path = os.path.join(ORACLE_DIR, "liboracle.so")
    if not os.path.exists(path):
        subprocess.check_call(["make", "-C", ORACLE_DIR, "oracle"], stdout=subprocess.DEVNULL)
    lib = C.CDLL(path)
    TP = C.POINTER(Tensor)
    f32p, i32p, u16p = C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_uint16)
    lib.orc_fp32_to_fp16.restype = C.c_uint16
    lib.orc_fp32_to_fp16.argtypes = [C.c_float]
    lib.orc_fp16_to_fp32.restype = C.c_float
    lib.orc_fp16_to_fp32.argtypes = [C.c_uint16]
    lib.orc_fp32_to_fp16_row.argtypes = [f32p, u16p, C.c_int64]
    lib.orc_fp16_to_fp32_row.argtypes = [u16p, f32p, C.c_int64]
    for name in ("orc_quantize_row_q8_0_ref", "orc_quantize_row_q8_0_x86"):
        getattr(lib, name).argtypes = [f32p, C.c_void_p, C.c_int64]
    lib.orc_dequantize_row_q8_0.argtypes = [C.c_void_p, f32p, C.c_int64]
    for name in ("orc_vec_dot_q8_0_q8_0", "orc_vec_dot_q8_0_q8_0_avx2"):
        getattr(lib, name).restype = C.c_float
        getattr(lib, name).argtypes = [C.c_int64, C.c_void_p, C.c_void_p]
    lib.orc_mul_mat.argtypes = [TP, TP, TP, C.c_int]
    lib.orc_mul_mat_f64.argtypes = [TP, TP, TP]
    lib.orc_rms_norm.argtypes = [TP, TP, C.c_float]
    lib.orc_rope.argtypes = [TP, i32p, f32p, TP, C.c_int, C.c_int, C.c_int] + [C.c_float] * 6
    lib.orc_soft_max.argtypes = [TP, TP, f32p, TP, C.c_float, C.c_float]
    lib.orc_flash_attn_ext.argtypes = [TP, TP, TP, TP, f32p, TP, C.c_float, C.c_float, C.c_float, C.c_int, C.c_int]
    lib.orc_flash_attn_ext_f64.argtypes = [TP, TP, TP, TP, f32p, TP, C.c_float, C.c_float, C.c_float]
    i64p, u64p = C.POINTER(C.c_int64), C.POINTER(C.c_uint64)
    lib.orc_kv_read_view.argtypes = [C.c_int] * 5 + [i64p, u64p, u64p]
    lib.orc_kv_write_view.argtypes = [C.c_int] * 6 + [i64p, u64p, u64p]
    lib.orc_causal_mask.argtypes = [i32p, C.c_int, C.c_int, u16p]
    lib.orc_cfg_pair_constants.argtypes = [C.c_int, i32p, u16p]
    lib.orc_t_span.argtypes = [C.c_int, C.c_float, f32p]
    _oracle = lib
    return lib


# -------------------------------------------------------------------------- reference
_ref = None
_ref_tried = False


def cpu_isa():
    try:
        flags = open("/proc/cpuinfo").read()
    except OSError:
        return "avx2"
    need = ("avx512f", "avx512bw", "avx512dq", "avx512vl", "avx512cd", "avx512_vnni")
    return "avx512" if all(f in flags for f in need) else "avx2"


def ref_dir():
    return os.path.join(ORACLE_DIR, "_ref", cpu_isa())


def load_ref():
    """The reference's ggml-cpu behind oracle/ref_harness.cpp, or None when not prebuilt."""
    global _ref, _ref_tried
    if _ref_tried:
        return _ref
    _ref_tried = True
    path = os.path.join(ref_dir(), "libref_harness.so")
    if not os.path.exists(path):
        return None
    C.CDLL(os.path.join(ref_dir(), "libggml-ref.so"), mode=C.RTLD_GLOBAL)
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    TP = C.POINTER(Tensor)
    f32p, i32p, u16p, f64p = C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_uint16), C.POINTER(C.c_double)
    lib.rh_load_plugin.argtypes = [C.c_char_p]
    lib.rh_device_name.restype = C.c_char_p
    lib.rh_device_name.argtypes = [C.c_int]
    lib.rh_use_device.argtypes = [C.c_char_p, C.c_int, C.c_int]
    lib.rh_fp32_to_fp16_row.argtypes = [f32p, u16p, C.c_int64]
    lib.rh_fp16_to_fp32_row.argtypes = [u16p, f32p, C.c_int64]
    lib.rh_quantize_q8_0.restype = C.c_size_t
    lib.rh_quantize_q8_0.argtypes = [f32p, C.c_void_p, C.c_int64, C.c_int64]
    lib.rh_dequantize_q8_0.argtypes = [C.c_void_p, f32p, C.c_int64]
    lib.rh_quantize_q8_0_cpu.argtypes = [f32p, C.c_void_p, C.c_int64]
    lib.rh_vec_dot_q8_0_q8_0.restype = C.c_float
    lib.rh_vec_dot_q8_0_q8_0.argtypes = [C.c_int64, C.c_void_p, C.c_void_p]
    lib.rh_mul_mat.argtypes = [TP, TP, TP, C.c_int, f64p]
    lib.rh_rms_norm.argtypes = [TP, TP, C.c_float, C.c_int, f64p]
    lib.rh_rope.argtypes = [TP, i32p, f32p, TP, C.c_int, C.c_int, C.c_int] + [C.c_float] * 6 + [C.c_int, f64p]
    lib.rh_soft_max.argtypes = [TP, TP, f32p, TP, C.c_float, C.c_float, C.c_int, f64p]
    lib.rh_flash_attn_ext.argtypes = [TP, TP, TP, TP, f32p, TP, C.c_float, C.c_float, C.c_float, C.c_int, f64p]
    lib.rh_bb_create.argtypes = [C.c_int] * 8 + [C.c_float, C.c_int, C.c_float, C.c_int]
    lib.rh_bb_set.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_size_t]
    lib.rh_last_times.argtypes = [f64p, C.c_int]
    lib.rh_out_after_reps.argtypes = [C.c_int]
    lib.rh_out_after_reps.restype = None
    lib.rh_bb_cache_set.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_size_t]
    lib.rh_bb_cache_get.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_size_t]
    lib.rh_bb_options.argtypes = [C.c_int, C.c_int]
    lib.rh_bb_options.restype = None
    lib.rh_bb_whole_graph.argtypes = [C.c_int]
    lib.rh_bb_whole_graph.restype = None
    f32p_, i32p_, u16p_ = C.POINTER(C.c_float), C.POINTER(C.c_int32), C.POINTER(C.c_uint16)
    lib.rh_cfm_create.argtypes = [C.c_int, C.c_void_p, f32p_, C.c_void_p, f32p_, C.c_void_p, f32p_]
    lib.rh_cfm_solve.argtypes = [f32p_, f32p_, f32p_, f32p_, f32p_, C.c_int, C.c_int, C.c_int, i32p_, u16p_, C.c_float, C.c_int,
                                 f32p_, C.c_int, C.POINTER(C.c_double)]
    lib.rh_bb_two_stage.argtypes = [f32p_, u16p_, C.c_int, C.c_int, f32p_, C.c_int, C.POINTER(C.c_double)]
    lib.rh_random_graph.argtypes = [C.c_uint64, C.c_int, C.POINTER(C.c_float), C.c_int64, C.POINTER(C.c_int64), C.POINTER(C.c_int)]
    lib.rh_cfm_solve_requests.argtypes = [f32p_, f32p_, f32p_, f32p_, f32p_, C.c_int, C.c_int, C.c_int, i32p_, u16p_, C.c_float, C.c_int, C.c_int,
                                          f32p_, C.c_int, C.POINTER(C.c_double)]
    lib.rh_cfm_set_time_mlp.argtypes = [C.c_int, C.c_void_p, f32p_]
    lib.rh_cfm_free.argtypes = []
    lib.rh_cfm_free.restype = None
    lib.rh_bb_fuse_weights.argtypes = []
    lib.rh_bb_forward.argtypes = [f32p, u16p, C.c_int, C.c_int, C.c_int, f32p, C.c_int, f64p]
    lib.rh_bb_decode_loop.argtypes = [f32p, C.c_int, C.c_int, C.c_int, f32p, f64p]
    assert lib.rh_use_device(b"CPU", min(8, os.cpu_count() or 1), 0) == 0
    _ref = lib
    return lib


# ------------------------------------------------------------------- seeded test data
def ref_last_times():
    """Seconds of every timed repeat of the harness's most recent timed run (numpy array)."""
    lib = load_ref()
    buf = np.zeros(1 << 16, np.float64)
    n = lib.rh_last_times(ptr(buf, C.c_double), buf.size)
    return buf[:min(n, buf.size)].copy()


def rng(*key):
    """A generator seeded by a readable key, e.g. rng("cfg1", "q")."""
    import zlib
    return np.random.default_rng(zlib.crc32("/".join(str(k) for k in key).encode()))


def quantize_q8_0(w):
    """Q8_0 rows (uint8, 34 bytes per 32 weights) with the oracle's weight quantizer."""
    lib = load_oracle()
    w = np.ascontiguousarray(w, dtype=np.float32)
    k = w.shape[-1]
    out = np.empty(w.shape[:-1] + (k // QK8_0 * Q8_BLOCK_BYTES,), dtype=np.uint8)
    lib.orc_quantize_row_q8_0_ref(ptr(w, C.c_float), out.ctypes.data, w.size)
    return out


def nmse(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    return float(((a - b) ** 2).sum() / max((a ** 2).sum(), 1e-300))


# --------------------------------------------------------- numpy-level op wrappers
ORC_FA_AUTO, ORC_FA_VEC, ORC_FA_TILED, ORC_FA_SPLIT_KV = 0, 1, 2, 3


def _as4(a):
    return a.reshape((1,) * (4 - a.ndim) + a.shape)


def fa_out_shape(q, v):
    q4, v4 = _as4(q), _as4(v)
    return (q4.shape[0], q4.shape[2], q4.shape[1], v4.shape[3])


def oracle_fa(q, k, v, mask=None, scale=0.125, max_bias=0.0, softcap=0.0, sinks=None, path=ORC_FA_VEC, nth=1,
              f64=False):
    """q (ne3,Hq,n_q,D) f32, k/v (ne3',Hkv,n_kv,D) f16|f32, mask (..,>=n_q,n_kv) f16 -> (ne3,n_q,Hq,D)."""
    lib = load_oracle()
    out = np.zeros(fa_out_shape(q, v), np.float32)
    md = desc(mask) if mask is not None else None
    sp = ptr(sinks, C.c_float)
    if f64:
        rc = lib.orc_flash_attn_ext_f64(desc(q), desc(k), desc(v), md, sp, desc(out), scale, max_bias, softcap)
    else:
        rc = lib.orc_flash_attn_ext(desc(q), desc(k), desc(v), md, sp, desc(out), scale, max_bias, softcap, path, nth)
    assert rc == 0, f"oracle flash_attn_ext rc={rc}"
    return out


def ref_fa(q, k, v, mask=None, scale=0.125, max_bias=0.0, softcap=0.0, sinks=None, reps=0):
    lib = load_ref()
    out = np.zeros(fa_out_shape(q, v), np.float32)
    sec = (C.c_double * 2)()
    rc = lib.rh_flash_attn_ext(desc(q), desc(k), desc(v), desc(mask) if mask is not None else None,
                               ptr(sinks, C.c_float), desc(out), scale, max_bias, softcap, reps, sec)
    assert rc == 0, f"reference flash_attn_ext rc={rc}"
    return (out, (sec[0], sec[1])) if reps else out


def oracle_rms_norm(x, eps):
    out = np.zeros(x.shape, np.float32)
    assert load_oracle().orc_rms_norm(desc(x), desc(out), eps) == 0
    return out


def ref_rms_norm(x, eps):
    out = np.zeros(x.shape, np.float32)
    assert load_ref().rh_rms_norm(desc(x), desc(out), eps, 0, None) == 0
    return out


def oracle_rope(x, pos, ff, n_dims, mode, n_ctx_orig=32768, freq_base=10000.0, freq_scale=1.0, ext_factor=0.0,
                attn_factor=1.0, beta_fast=32.0, beta_slow=1.0):
    out = np.zeros(x.shape, np.float32)
    rc = load_oracle().orc_rope(desc(x), ptr(pos, C.c_int32), ptr(ff, C.c_float), desc(out), n_dims, mode,
                                n_ctx_orig, freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow)
    assert rc == 0, rc
    return out


def ref_rope(x, pos, ff, n_dims, mode, n_ctx_orig=32768, freq_base=10000.0, freq_scale=1.0, ext_factor=0.0,
             attn_factor=1.0, beta_fast=32.0, beta_slow=1.0):
    out = np.zeros(x.shape, np.float32)
    rc = load_ref().rh_rope(desc(x), ptr(pos, C.c_int32), ptr(ff, C.c_float), desc(out), n_dims, mode, n_ctx_orig,
                            freq_base, freq_scale, ext_factor, attn_factor, beta_fast, beta_slow, 0, None)
    assert rc == 0, rc
    return out


def oracle_soft_max(x, mask, scale, max_bias, sinks=None):
    out = np.zeros(x.shape, np.float32)
    rc = load_oracle().orc_soft_max(desc(x), desc(mask) if mask is not None else None, ptr(sinks, C.c_float),
                                    desc(out), scale, max_bias)
    assert rc == 0, rc
    return out


def ref_soft_max(x, mask, scale, max_bias, sinks=None):
    out = np.zeros(x.shape, np.float32)
    rc = load_ref().rh_soft_max(desc(x), desc(mask) if mask is not None else None, ptr(sinks, C.c_float),
                                desc(out), scale, max_bias, 0, None)
    assert rc == 0, rc
    return out


def _w_desc(w, k):
    return desc_q8(w, k) if w.dtype == np.uint8 else desc(w)


def mm_out(w, x, k):
    wd = _w_desc(w, k)
    return np.zeros(tuple(x.shape[:-1]) + (wd.ne[1],), np.float32)


def oracle_mul_mat(w, x, k=None, act_mode=0, f64=False):
    """w: f16/f32 (.., rows, K) or Q8_0 bytes with k=K; x (.., tokens, K) f32 -> (.., tokens, rows)."""
    k = x.shape[-1] if k is None else k
    out = mm_out(w, x, k)
    lib = load_oracle()
    rc = lib.orc_mul_mat_f64(_w_desc(w, k), desc(x), desc(out)) if f64 else \
        lib.orc_mul_mat(_w_desc(w, k), desc(x), desc(out), act_mode)
    assert rc == 0, rc
    return out


def ref_mul_mat(w, x, k=None, reps=0):
    k = x.shape[-1] if k is None else k
    out = mm_out(w, x, k)
    sec = (C.c_double * 2)()
    rc = load_ref().rh_mul_mat(_w_desc(w, k), desc(x), desc(out), reps, sec)
    assert rc == 0, rc
    return (out, (sec[0], sec[1])) if reps else out


def causal_mask(n_q, n_kv, n_past=0):
    """create_causal_mask of the reference for query positions n_past..n_past+n_q-1."""
    pos = np.arange(n_past, n_past + n_q, dtype=np.int32)
    m = np.empty((n_q, n_kv), np.uint16)
    load_oracle().orc_causal_mask(ptr(pos, C.c_int32), n_q, n_kv, ptr(m, C.c_uint16))
    return m.view(np.float16)


# ------------------------------------------------------------------- MiniCPM backbone
BB_WEIGHTS = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")


def backbone_params(tag, n_layer, hidden=1024, n_heads=16, n_kv=2, head_dim=64, ffn=4096):
    """Seeded weights of BASELINE config 4: N(0, 0.02) quantised to Q8_0 with the reference's
    weight quantizer, norm weights near 1, rope frequency factors in [1, 2)."""
    qd, kd = n_heads * head_dim, n_kv * head_dim
    shapes = {"q_proj": (qd, hidden), "k_proj": (kd, hidden), "v_proj": (kd, hidden), "o_proj": (hidden, qd),
              "gate_proj": (ffn, hidden), "up_proj": (ffn, hidden), "down_proj": (hidden, ffn)}
    layers = []
    for li in range(n_layer):
        lw = {n: quantize_q8_0((rng(tag, li, n).standard_normal(shapes[n]) * 0.02).astype(np.float32)) for n in BB_WEIGHTS}
        for n in ("input_layernorm", "post_layernorm"):
            lw[n] = (1.0 + 0.1 * rng(tag, li, n).standard_normal(hidden)).astype(np.float32)
        layers.append(lw)
    final = (1.0 + 0.1 * rng(tag, "final").standard_normal(hidden)).astype(np.float32)
    factors = (1.0 + rng(tag, "rope").random(head_dim // 2)).astype(np.float32)
    return {"layers": layers, "final_norm": final, "rope_factors": factors, "shapes": shapes,
            "dims": dict(n_layer=n_layer, hidden=hidden, n_heads=n_heads, n_kv=n_kv, head_dim=head_dim, ffn=ffn)}


def ref_backbone_create(params, max_len, batch, use_mup=False, kv_f16=False, eps=1e-5, fused_weights=False):
    """Builds the decoder stack on the harness's current device (rh_use_device) and uploads params.
    fused_weights: the graph variant the reference uses for the LocDiT decoder on a GPU backend, one product
    over row-fused q/k/v (and gate/up) weights with strided views of it."""
    lib = load_ref()
    d = params["dims"]
    rc = lib.rh_bb_create(d["n_layer"], d["hidden"], d["n_heads"], d["n_kv"], d["head_dim"], d["ffn"], max_len, batch,
                          eps, int(use_mup), 1.4, 1 if kv_f16 else 0)
    assert rc == 0, rc
    ref_backbone_upload(params)
    if fused_weights:
        assert lib.rh_bb_fuse_weights() == 0


def ref_backbone_upload(params):
    """(Re-)uploads params into the decoder stack that exists: the same tensors at the same addresses."""
    lib = load_ref()
    for li, lw in enumerate(params["layers"]):
        for wi, n in enumerate(BB_WEIGHTS + ("input_layernorm", "post_layernorm")):
            a = np.ascontiguousarray(lw[n])
            assert lib.rh_bb_set(li, wi, a.ctypes.data, a.nbytes) == 0, (li, n)
    assert lib.rh_bb_set(-1, 0, params["final_norm"].ctypes.data, params["final_norm"].nbytes) == 0
    assert lib.rh_bb_set(-1, 1, params["rope_factors"].ctypes.data, params["rope_factors"].nbytes) == 0


def ref_backbone_forward(x, n_past, mask=None, write_kv=True, reps=0):
    """x: (batch, n_tokens, hidden) f32.  Returns (out, seconds[mean, best], n_nodes)."""
    lib = load_ref()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    sec = np.zeros(3, np.float64)
    m = None if mask is None else np.ascontiguousarray(mask).view(np.uint16)
    rc = lib.rh_bb_forward(ptr(x, C.c_float), None if m is None else ptr(m, C.c_uint16), x.shape[1], n_past, int(write_kv),
                           ptr(out, C.c_float), reps, ptr(sec, C.c_double))
    assert rc == 0, rc
    return out, sec[:2].copy(), int(sec[2])


def ref_backbone_decode_loop(x, n_past0, steps, overlap=False):
    """`steps` consecutive decode steps from cache length n_past0, each with a graph built for its own position as the
    reference builds them (src/voxcpm.cpp:485-513).  x: (batch, 1, hidden) f32, the same input every step.  Returns the
    last step's hidden state and a dict of per-step seconds (wall over the loop, graph_compute's share, graph
    construction + layout), the node count and the share of nodes that moved between steps.  overlap: the next step's
    graph is built while the device computes the current one."""
    lib = load_ref()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    sec = np.zeros(5, np.float64)
    rc = lib.rh_bb_decode_loop(ptr(x, C.c_float), n_past0, steps, int(overlap), ptr(out, C.c_float), ptr(sec, C.c_double))
    assert rc == 0, rc
    return out, {"wall": float(sec[0]), "graph_compute": float(sec[1]), "build": float(sec[3]), "n_nodes": int(sec[2]), "moved": float(sec[4])}


def cfm_params(tag, feat=64, hidden=1024):
    """Seeded weights of the LocDiT estimator's own projections (in_proj, cond_proj: feat -> hidden; out_proj:
    hidden -> feat; quantised to Q8_0 on upload), scaled so that activations stay O(1)."""
    g = lambda *k: rng(tag, *k)
    return {"feat": feat, "hidden": hidden,
            "in_w": (g("in_w").standard_normal((hidden, feat)) / np.sqrt(feat)).astype(np.float32),
            "in_b": (0.1 * g("in_b").standard_normal(hidden)).astype(np.float32),
            "cond_w": (g("cond_w").standard_normal((hidden, feat)) / np.sqrt(feat)).astype(np.float32),
            "cond_b": (0.1 * g("cond_b").standard_normal(hidden)).astype(np.float32),
            "out_w": (g("out_w").standard_normal((feat, hidden)) / np.sqrt(hidden)).astype(np.float32),
            "out_b": (0.1 * g("out_b").standard_normal(feat)).astype(np.float32),
            # time_mlp linear1 / linear2, delta_time_mlp linear1 / linear2 (src/locdit.cpp:213-246)
            "time_w": [(g("time_w", i).standard_normal((hidden, hidden)) / np.sqrt(hidden)).astype(np.float32) for i in range(4)],
            "time_b": [(0.1 * g("time_b", i).standard_normal(hidden)).astype(np.float32) for i in range(4)]}


def ref_backbone_two_stage(x, mask, resident, reps=1):
    """out = forward(forward(x) + x) on the stack made by ref_backbone_create, as two graphs: with the first stage's
    result fetched, added on the host and uploaded again (resident=False, the reference's decode step,
    src/voxcpm.cpp:1067-1093) or kept in a persistent device tensor (resident=True).  x (batch, T, hidden).
    Returns (out, seconds[mean, best])."""
    lib = load_ref()
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty_like(x)
    sec = np.zeros(2, np.float64)
    m = None if mask is None else np.ascontiguousarray(mask).view(np.uint16)
    rc = lib.rh_bb_two_stage(ptr(x, C.c_float), None if m is None else ptr(m, C.c_uint16), x.shape[1], int(resident),
                             ptr(out, C.c_float), reps, ptr(sec, C.c_double))
    assert rc == 0, rc
    return out, sec


def ref_cfm_create(p):
    """The estimator's projections beside the decoder stack made by ref_backbone_create (batch 1)."""
    lib = load_ref()
    f = lambda a: ptr(np.ascontiguousarray(a), C.c_float)
    q = {n: quantize_q8_0(p[n]) for n in ("in_w", "cond_w", "out_w")}   # Q8_0, as the reference's quantizer stores them
    rc = lib.rh_cfm_create(p["feat"], q["in_w"].ctypes.data, f(p["in_b"]), q["cond_w"].ctypes.data, f(p["cond_b"]),
                           q["out_w"].ctypes.data, f(p["out_b"]))
    assert rc == 0, rc
    for i in range(4):
        wq = quantize_q8_0(p["time_w"][i])
        assert lib.rh_cfm_set_time_mlp(i, wq.ctypes.data, f(p["time_b"][i])) == 0


def ref_cfm_solve(z, mu, cond, table, n_steps=10, sway=1.0, cfg_value=2.0, zero_star=True, reps=0):
    """One UnifiedCFM solve as a single graph on the harness's device.  z (patch, feat), mu (hidden,), cond (prefix, feat),
    table (n_steps, hidden).  Returns (x (patch, feat), seconds[mean, best], n_nodes).
    With a leading request dimension -- z (R, patch, feat), mu (R, hidden), cond (R, prefix, feat) -- the R requests are
    solved by ONE graph (the decoder stack must have been created with batch R)."""
    lib, orc = load_ref(), load_oracle()
    z, mu, cond = (np.ascontiguousarray(a, dtype=np.float32) for a in (z, mu, cond))
    table = None if table is None else np.ascontiguousarray(table, dtype=np.float32)   # None: the time embeddings are built in the graph
    n_req = z.shape[0] if z.ndim == 3 else 1
    patch, prefix = z.shape[-2], cond.shape[-2]
    L = 1 + prefix + patch
    t_span = np.zeros(n_steps + 1, np.float32)
    orc.orc_t_span(n_steps, sway, ptr(t_span, C.c_float))
    pos = np.zeros(2 * L, np.int32)
    mk = np.zeros((2 * L, 2 * L), np.uint16)
    orc.orc_cfg_pair_constants(L, ptr(pos, C.c_int32), ptr(mk, C.c_uint16))
    out = np.empty_like(z)
    sec = np.zeros(3, np.float64)
    if z.ndim == 3:
        rc = lib.rh_cfm_solve_requests(ptr(z, C.c_float), ptr(mu, C.c_float), ptr(cond, C.c_float), None if table is None else ptr(table, C.c_float),
                                       ptr(t_span, C.c_float), n_steps, patch, prefix, ptr(pos, C.c_int32), ptr(mk, C.c_uint16), cfg_value,
                                       int(zero_star), n_req, ptr(out, C.c_float), reps, ptr(sec, C.c_double))
    else:
        rc = lib.rh_cfm_solve(ptr(z, C.c_float), ptr(mu, C.c_float), ptr(cond, C.c_float), None if table is None else ptr(table, C.c_float), ptr(t_span, C.c_float),
                              n_steps, patch, prefix, ptr(pos, C.c_int32), ptr(mk, C.c_uint16), cfg_value, int(zero_star),
                              ptr(out, C.c_float), reps, ptr(sec, C.c_double))
    assert rc == 0, rc
    return out, sec[:2].copy(), int(sec[2])


# ------------------------------------------------- the reference's own module layer (oracle/vox_harness.cpp)
_vox = None


def load_vox():
    """libvox_harness.so: VoxCPMBackend / VoxCPMWeightStore / MiniCPMModel compiled from the reference's sources,
    or None when oracle/_ref was not prebuilt."""
    global _vox
    if _vox is not None:
        return _vox
    path = os.path.join(ref_dir(), "libvox_harness.so")
    if not os.path.exists(path):
        return None
    C.CDLL(os.path.join(ref_dir(), "libggml-ref.so"), mode=C.RTLD_GLOBAL)   # a plugin resolves ggml's symbols from the process
    lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
    lib.vh_last_error.restype = C.c_char_p
    lib.vh_backend_name.restype = C.c_char_p
    lib.vh_weight_bytes.restype = C.c_size_t
    lib.vh_gguf_begin.argtypes = [C.c_char_p, C.c_size_t]
    lib.vh_gguf_u32.argtypes = [C.c_char_p, C.c_uint32]
    lib.vh_gguf_f32.argtypes = [C.c_char_p, C.c_float]
    lib.vh_gguf_str.argtypes = [C.c_char_p, C.c_char_p]
    lib.vh_gguf_f32_array.argtypes = [C.c_char_p, C.c_void_p, C.c_int]
    lib.vh_gguf_tensor.argtypes = [C.c_char_p, C.c_int, C.c_int64, C.c_int64, C.c_void_p, C.c_size_t]
    lib.vh_load_plugin.argtypes = [C.c_char_p]
    lib.vh_open.argtypes = [C.c_int, C.c_int]
    lib.vh_minicpm_load.argtypes = [C.c_char_p, C.c_char_p, C.c_int]
    lib.vh_minicpm_run.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_double)]
    lib.vh_cache_get.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_size_t]
    lib.vh_placed_run.argtypes = [C.c_char_p, C.c_char_p, C.c_int, C.c_char_p, C.c_char_p, C.c_char_p, C.c_void_p, C.c_int, C.c_void_p,
                                  C.POINTER(C.c_int64)]
    _vox = lib
    return lib


GGML_TYPE_F32, GGML_TYPE_Q8_0 = 0, 8
GGUF_LAYER_NAMES = {"q_proj": "attn_q", "k_proj": "attn_k", "v_proj": "attn_v", "o_proj": "attn_output",
                    "gate_proj": "ffn_gate", "up_proj": "ffn_up", "down_proj": "ffn_down",
                    "input_layernorm": "attn_norm", "post_layernorm": "ffn_norm"}


def write_minicpm_gguf(path, params, prefix, max_len, use_mup=True, extra=()):
    """A synthetic model file for MiniCPMModel::load_from_store (src/minicpm.cpp:296-360, 522-570): the decoder stack of
    backbone_params() under `prefix` ("residual_lm" or "locdit"), written with the reference's gguf API."""
    lib = load_vox()
    d = params["dims"]
    total = sum(a.nbytes for lw in params["layers"] for a in lw.values()) + (64 << 20)
    ok = lambda rc: (_ for _ in ()).throw(AssertionError(lib.vh_last_error())) if rc else None
    ok(lib.vh_gguf_begin(path.encode(), total))
    for key, v in (("llama.embedding_length", d["hidden"]), ("llama.feed_forward_length", d["ffn"]),
                   ("llama.attention.head_count", d["n_heads"]), ("llama.attention.head_count_kv", d["n_kv"]),
                   ("llama.context_length", max_len), ("voxcpm_lm_config_use_mup", int(use_mup)),
                   ("voxcpm_lm_config_rope_scaling_original_max_position_embeddings", 32768),
                   ("voxcpm_residual_lm_num_layers", d["n_layer"]),
                   ("voxcpm_dit_config_hidden_dim", d["hidden"]), ("voxcpm_dit_config_ffn_dim", d["ffn"]),
                   ("voxcpm_dit_config_num_heads", d["n_heads"]), ("voxcpm_dit_config_num_layers", d["n_layer"])):
        ok(lib.vh_gguf_u32(key.encode(), v))
    for key, v in (("llama.attention.layer_norm_rms_epsilon", 1e-5), ("llama.rope.freq_base", 10000.0),
                   ("voxcpm_lm_config_scale_depth", 1.4)):
        ok(lib.vh_gguf_f32(key.encode(), v))
    ff = np.ascontiguousarray(params["rope_factors"], np.float32)
    for key in ("voxcpm_lm_config_rope_scaling_short_factor", "voxcpm_lm_config_rope_scaling_long_factor"):
        ok(lib.vh_gguf_f32_array(key.encode(), ff.ctypes.data, ff.size))
    pre = prefix + "." if prefix else ""
    fn = np.ascontiguousarray(params["final_norm"], np.float32)
    ok(lib.vh_gguf_tensor((pre + "output_norm.weight").encode(), GGML_TYPE_F32, fn.size, 0, fn.ctypes.data, fn.nbytes))
    for li, lw in enumerate(params["layers"]):
        for n, gname in GGUF_LAYER_NAMES.items():
            a = np.ascontiguousarray(lw[n])
            name = f"{pre}blk.{li}.{gname}.weight".encode()
            if n in params["shapes"]:
                rows, k = params["shapes"][n]
                ok(lib.vh_gguf_tensor(name, GGML_TYPE_Q8_0, k, rows, a.ctypes.data, a.nbytes))
            else:
                ok(lib.vh_gguf_tensor(name, GGML_TYPE_F32, a.size, 0, a.ctypes.data, a.nbytes))
    for name, a in extra:   # further F32 tensors (name, array of 1 or 2 dims)
        a = np.ascontiguousarray(a, np.float32)
        ok(lib.vh_gguf_tensor(name.encode(), GGML_TYPE_F32, a.shape[-1], a.shape[0] if a.ndim == 2 else 0, a.ctypes.data, a.nbytes))
    ok(lib.vh_gguf_end())
