"""Pins for the CPU oracle (oracle/oracle.c).  Each function is checked against something
that is *not* a retyping of its formula:

  * golden outputs of the reference's own ggml-cpu (tests/golden/ggml_cpu_golden.npz, made by
    tests/golden/make_golden.py from the reference build) -- always available;
  * that same ggml-cpu live (oracle/_ref) where it was prebuilt, on more shapes;
  * the fixtures the reference's own tests hold (KV-cache view shapes, compute_t_span closed
    form, Q8_0 round-trip bound);
  * mathematics: numpy float16 for the conversions, brute-force integer dots, fp64 closed
    forms, invariants (rows of a softmax sum to one, n_kv = 1, equal keys, key permutation,
    split-KV associativity, rotation norms).
"""
import ctypes as C
import os
import sys

import numpy as np
import pytest

import reflib
from reflib import desc, nmse, ptr, rng

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden"))
import make_golden  # noqa: E402

GOLD = {k: v for k, v in np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ggml_cpu_golden.npz")).items()}
IN = make_golden.inputs()


# ------------------------------------------------------------------------- fp16 <-> fp32
def test_fp16_to_fp32_all_halves(oracle):
    h = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    oracle.orc_fp16_to_fp32_row(ptr(h, C.c_uint16), ptr(out, C.c_float), 65536)
    want = h.view(np.float16).astype(np.float32)
    assert np.array_equal(out.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.isnan(out[np.isnan(want)]).all()


def test_fp32_to_fp16_matches_ieee_rne(oracle):
    r = rng("f16")
    x = np.concatenate([
        r.standard_normal(200000).astype(np.float32) * np.float32(3.0),
        (r.standard_normal(50000) * 1e-6).astype(np.float32),           # subnormal halves
        (r.standard_normal(50000) * 3e4).astype(np.float32),            # near overflow
        np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.9, 65520.0, 2.0 ** -24, 2.0 ** -25,
                  1.5 * 2.0 ** -25, 2049.0, 2051.0, -1e9, 1e-10], np.float32),
        np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32),  # round trip
    ])
    x = x[~np.isnan(x)]
    out = np.empty(x.size, np.uint16)
    oracle.orc_fp32_to_fp16_row(ptr(x, C.c_float), ptr(out, C.c_uint16), x.size)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(out, want)
    assert oracle.orc_fp32_to_fp16(C.c_float(-1e9)) == 0xFC00  # the mask constant becomes -inf
    assert oracle.orc_fp32_to_fp16(C.c_float(-0.0)) == 0x8000


# --------------------------------------------------------------------------------- Q8_0
def test_q8_0_weight_quantizer_golden(oracle):
    assert np.array_equal(reflib.quantize_q8_0(IN["w"]), GOLD["w_q8_0"])
    deq = np.empty((48, 256), np.float32)
    oracle.orc_dequantize_row_q8_0(GOLD["w_q8_0"].ctypes.data, ptr(deq, C.c_float), 48 * 256)
    assert np.array_equal(deq.view(np.uint32), GOLD["w_dequant"].view(np.uint32))
    # independent statement of the block layout: d = f16 at byte 0, 32 int8 after it
    raw = GOLD["w_q8_0"].reshape(48, 8, 34)
    d = raw[:, :, :2].copy().view(np.float16).astype(np.float32)
    q = raw[:, :, 2:].view(np.int8).astype(np.float32)
    assert np.array_equal((q * d).reshape(48, 256), deq)


def test_q8_0_roundtrip_bound(oracle):
    """ggml/tests/test-quantize-fns.cpp:17-18: round-trip RMSE of Q8_0 stays under 0.002 on its
    synthetic signal 0.1 + 2*cos(i + offset)."""
    n = 32 * 128
    x = (0.1 + 2.0 * np.cos(np.arange(n, dtype=np.float32) + np.float32(0.0))).astype(np.float32)
    q = reflib.quantize_q8_0(x[None, :])
    y = np.empty(n, np.float32)
    oracle.orc_dequantize_row_q8_0(q.ctypes.data, ptr(y, C.c_float), n)
    rmse = np.sqrt(((x - y) ** 2).sum()) / n
    assert rmse < 0.002


def test_q8_0_activation_quantizer_golden(oracle):
    xq = np.empty((5, 8 * 34), np.uint8)
    for i in range(5):
        oracle.orc_quantize_row_q8_0_x86(ptr(IN["x"][i], C.c_float), xq[i].ctypes.data, 256)
    assert np.array_equal(xq, GOLD["x_q8_0_cpu"])


def test_q8_0_quantizers_differ_on_ties_only_as_documented(oracle):
    """weights: roundf (ties away from zero) with id = 1/d; activations (x86): ties to even
    with id = 127/max.  amax = 127 makes d = id = 1 so the rounding rule alone decides."""
    x = np.zeros(32, np.float32)
    x[0], x[1], x[2], x[3], x[4] = 127.0, 0.5, 1.5, 2.5, -0.5
    a = np.empty(34, np.uint8)
    b = np.empty(34, np.uint8)
    oracle.orc_quantize_row_q8_0_ref(ptr(x, C.c_float), a.ctypes.data, 32)
    oracle.orc_quantize_row_q8_0_x86(ptr(x, C.c_float), b.ctypes.data, 32)
    assert list(a[2:7].view(np.int8)) == [127, 1, 2, 3, -1]
    assert list(b[2:7].view(np.int8)) == [127, 0, 2, 2, 0]
    z = np.zeros(32, np.float32)  # all-zero block: d = 0, quants 0, no NaN
    oracle.orc_quantize_row_q8_0_x86(ptr(z, C.c_float), b.ctypes.data, 32)
    assert not b.any()


def test_q8_0_dot_bruteforce(oracle):
    r = rng("dot")
    n = 32 * 9
    a = reflib.quantize_q8_0(r.standard_normal((1, n)).astype(np.float32))
    b = reflib.quantize_q8_0(r.standard_normal((1, n)).astype(np.float32))
    ra, rb = a.reshape(9, 34), b.reshape(9, 34)
    da = ra[:, :2].copy().view(np.float16).astype(np.float64)[:, 0]
    db = rb[:, :2].copy().view(np.float16).astype(np.float64)[:, 0]
    si = (ra[:, 2:].view(np.int8).astype(np.int64) * rb[:, 2:].view(np.int8).astype(np.int64)).sum(1)
    want = float((si * da * db).sum())
    for fn in (oracle.orc_vec_dot_q8_0_q8_0, oracle.orc_vec_dot_q8_0_q8_0_avx2):
        got = fn(n, a.ctypes.data, b.ctypes.data)
        assert abs(got - want) <= 1e-5 * abs(want) + 1e-6


# ------------------------------------------------------------------------------ MUL_MAT
def test_mul_mat_golden(oracle):
    got = reflib.oracle_mul_mat(GOLD["w_q8_0"], IN["x"], 256, act_mode=0)
    assert np.abs(got - GOLD["mul_mat_q8_0"]).max() <= 1e-6 * np.abs(GOLD["mul_mat_q8_0"]).max()
    got16 = reflib.oracle_mul_mat(IN["w"].astype(np.float16), IN["x"], act_mode=0)
    assert np.abs(got16 - GOLD["mul_mat_f16"]).max() <= 2e-6
    # fp64 dequantise-then-multiply equals numpy on the dequantised weights
    f64 = reflib.oracle_mul_mat(GOLD["w_q8_0"], IN["x"], 256, f64=True)
    want = (IN["x"].astype(np.float64) @ GOLD["w_dequant"].astype(np.float64).T).astype(np.float32)
    assert np.array_equal(f64, want)
    # ggml-cpu's int8 activation path sits ~3e-5 NMSE from the dequantised product
    assert 1e-6 < nmse(f64, GOLD["mul_mat_q8_0"]) < 5e-4
    fl = reflib.oracle_mul_mat(GOLD["w_q8_0"], IN["x"], 256, act_mode=1)
    assert nmse(f64, fl) < 1e-12


def test_mul_mat_vs_reference_live(oracle, ref):
    for M, K, N, batch in ((64, 1024, 3, ()), (130, 96, 17, ()), (32, 64, 4, (2, 3))):
        w = (rng("mm", M, K).standard_normal(batch + (M, K)) * 0.02).astype(np.float32)
        x = rng("mmx", N, K).standard_normal(batch + (N, K)).astype(np.float32)
        wq = reflib.quantize_q8_0(w)
        a, b = reflib.oracle_mul_mat(wq, x, K, 0), reflib.ref_mul_mat(wq, x, K)
        assert np.abs(a - b).max() <= 1e-6 * np.abs(b).max()
        for wt in (np.float16, np.float32):
            a, b = reflib.oracle_mul_mat(w.astype(wt), x, None, 0), reflib.ref_mul_mat(w.astype(wt), x)
            assert np.abs(a - b).max() <= 3e-6


# ----------------------------------------------------------------------------- RMS_NORM
def test_rms_norm(oracle):
    got = reflib.oracle_rms_norm(IN["rms_x"], 1e-5)
    assert np.array_equal(got, GOLD["rms"])
    x64 = IN["rms_x"].astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(-1, keepdims=True) + 1e-5)
    assert np.abs(got - want).max() <= 1e-6
    # strided rows
    base = rng("rmsv").standard_normal((4, 300)).astype(np.float32)
    v = base[:, :128]
    assert np.array_equal(reflib.oracle_rms_norm(v, 0.0), reflib.oracle_rms_norm(np.ascontiguousarray(v), 0.0))


# --------------------------------------------------------------------------------- ROPE
def rope_closed_form(x, pos, ff, n_dims, mode, base=10000.0):
    x = x.astype(np.float64)
    out = x.copy()
    i = np.arange(n_dims // 2)
    inv = base ** (-2.0 * i / n_dims) / (np.ones(n_dims // 2) if ff is None else ff.astype(np.float64))
    th = pos.astype(np.float64)[:, None] * inv[None, :]           # (tokens, pairs)
    c, s = np.cos(th)[None, :, None, :], np.sin(th)[None, :, None, :]
    if mode == 2:
        a, b = x[..., : n_dims // 2], x[..., n_dims // 2: n_dims]
        out[..., : n_dims // 2], out[..., n_dims // 2: n_dims] = a * c - b * s, a * s + b * c
    else:
        a, b = x[..., 0:n_dims:2], x[..., 1:n_dims:2]
        out[..., 0:n_dims:2], out[..., 1:n_dims:2] = a * c - b * s, a * s + b * c
    return out


def test_rope(oracle):
    x, pos, ff = IN["rope_x"], IN["rope_pos"], IN["rope_ff"]
    neox = reflib.oracle_rope(x, pos, ff, 64, 2)
    normal = reflib.oracle_rope(x, pos, None, 64, 0)
    # golden: libm sinf/cosf may differ by an ulp between builds, nothing more
    assert np.abs(neox - GOLD["rope_neox"]).max() <= 2e-6
    assert np.abs(normal - GOLD["rope_normal"]).max() <= 2e-6
    # closed form in fp64: tight at small positions, ~pos * 1e-7 further out (fp32 angle chain)
    small = pos < 300
    assert np.abs(neox[:, small] - rope_closed_form(x, pos, ff, 64, 2)[:, small]).max() <= 1e-4
    assert np.abs(normal[:, small] - rope_closed_form(x, pos, None, 64, 0)[:, small]).max() <= 1e-4
    assert np.abs(neox - rope_closed_form(x, pos, ff, 64, 2)).max() <= 5e-3
    # position 0 is the identity; partial rotation copies the tail
    assert np.array_equal(neox[:, 0], x[:, 0])
    part = reflib.oracle_rope(x, pos, None, 32, 2)
    assert np.array_equal(part[..., 32:], x[..., 32:])
    assert np.allclose((neox ** 2).sum(-1), (x ** 2).sum(-1), rtol=1e-5)


def test_rope_vs_reference_live(oracle, ref):
    x = rng("ropel").standard_normal((2, 9, 3, 128)).astype(np.float32)
    pos = (np.arange(9, dtype=np.int32) * 911) % 8192
    ff = (1.0 + rng("ropeff").random(64)).astype(np.float32)
    for mode in (0, 2):
        for kw in (dict(), dict(freq_scale=0.5, ext_factor=1.0, attn_factor=1.2, n_ctx_orig=4096), dict(attn_factor=0.7)):
            a = reflib.oracle_rope(x, pos, ff, 128, mode, **kw)
            b = reflib.ref_rope(x, pos, ff, 128, mode, **kw)
            assert np.abs(a - b).max() <= 3e-6


# ----------------------------------------------------------------------------- SOFT_MAX
def test_soft_max(oracle, request):
    got = reflib.oracle_soft_max(IN["sm_x"], IN["sm_mask"], 0.25, 8.0)
    assert np.abs(got - GOLD["soft_max"]).max() <= 1e-7
    assert np.allclose(got.sum(-1), 1.0, atol=1e-6)
    # closed form with ALiBi slopes m0^(h+1), m0 = 2^(-8/4)
    slopes = (2.0 ** (-8.0 / 4)) ** (np.arange(4) + 1.0)
    z = IN["sm_x"].astype(np.float64) * 0.25 + slopes[None, :, None, None] * IN["sm_mask"].astype(np.float64)
    e = np.exp(z - z.max(-1, keepdims=True))
    assert np.abs(got - e / e.sum(-1, keepdims=True)).max() <= 1e-6


# ------------------------------------------------------------------------ FLASH_ATTN_EXT
def numpy_attention(q, k, v, mask, scale):
    """Textbook softmax(scale * Q K^T + mask) V with GQA head h -> kv head h // (Hq/Hkv)."""
    q64, k64, v64 = q.astype(np.float64), k.astype(np.float64), v.astype(np.float64)
    rep = q.shape[1] // k.shape[1]
    k64, v64 = np.repeat(k64, rep, axis=1), np.repeat(v64, rep, axis=1)
    s = np.einsum("bhqd,bhkd->bhqk", q64, k64) * scale
    if mask is not None:
        s = s + mask.astype(np.float64)[None, None, : q.shape[2]]
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return np.einsum("bhqk,bhkd->bqhd", p, v64)


def test_flash_attn_golden_and_textbook(oracle):
    mask = reflib.causal_mask(70, 70)
    q, k, v = IN["q_pre"], IN["k_pre"], IN["v_pre"]
    want = numpy_attention(q, k, v, mask, 0.125)
    for path in (reflib.ORC_FA_TILED, reflib.ORC_FA_AUTO):
        got = reflib.oracle_fa(q, k, v, mask, path=path, nth=4)
        assert np.abs(got - GOLD["fa_prefill_f16"]).max() <= 2e-6
        assert np.abs(got - want).max() <= 2e-6
    assert np.abs(reflib.oracle_fa(q, k, v, mask, f64=True) - want).max() <= 1e-6
    # decode, F32-typed K/V (fp32 accumulation): the parity oracle of the GPU tests
    qd, kd, vd = IN["q_dec"], IN["k_dec"].astype(np.float32), IN["v_dec"].astype(np.float32)
    want = numpy_attention(qd, kd, vd, None, 0.125)
    for path, nth in ((reflib.ORC_FA_VEC, 1), (reflib.ORC_FA_SPLIT_KV, 4), (reflib.ORC_FA_AUTO, 4), (reflib.ORC_FA_SPLIT_KV, 7)):
        got = reflib.oracle_fa(qd, kd, vd, None, path=path, nth=nth)
        assert np.abs(got - GOLD["fa_decode_f32kv"]).max() <= 2e-6
        assert np.abs(got - want).max() <= 2e-6
    # decode, F16-typed K/V: ggml-cpu accumulates V*P in half precision; the restatement follows
    # it (1e-3 scale noise) and both sit ~1e-3 away from the exact result
    got16 = reflib.oracle_fa(IN["q_dec"], IN["k_dec"], IN["v_dec"], None, path=reflib.ORC_FA_AUTO, nth=4)
    assert np.abs(got16 - GOLD["fa_decode_f16kv"]).max() <= 3e-3
    assert 1e-5 < np.abs(GOLD["fa_decode_f16kv"] - want).max() < 1e-2


def test_flash_attn_invariants(oracle):
    r = rng("inv")
    q = r.standard_normal((2, 8, 5, 64)).astype(np.float32)
    k = r.standard_normal((2, 2, 90, 64)).astype(np.float32)
    v = r.standard_normal((2, 2, 90, 64)).astype(np.float32)
    base = reflib.oracle_fa(q, k, v)
    perm = r.permutation(90)
    assert np.abs(reflib.oracle_fa(q, k[:, :, perm].copy(), v[:, :, perm].copy()) - base).max() <= 1e-5
    one = reflib.oracle_fa(q, k[:, :, :1].copy(), v[:, :, :1].copy())
    for h in range(8):
        assert np.abs(one[:, :, h] - v[:, h // 4, 0][:, None]).max() <= 1e-7
    keq = np.repeat(k[:, :, :1], 90, axis=2).copy()
    eq = reflib.oracle_fa(q, keq, v)
    for h in range(8):
        assert np.abs(eq[:, :, h] - v[:, h // 4].mean(1)[:, None]).max() <= 1e-5
    mask = np.zeros((5, 90), np.float16)
    mask[3] = -np.inf
    assert not reflib.oracle_fa(q, k, v, mask)[:, 3].any()
    assert (base >= v.min() - 1e-6).all() and (base <= v.max() + 1e-6).all()
    # strided views (permuted q, cache-style k/v) give what the dense copies give
    qb = np.ascontiguousarray(q.transpose(0, 2, 1, 3))
    cache_k = np.zeros((2, 2, 128, 64), np.float32)
    cache_k[:, :, :90] = k
    assert np.array_equal(reflib.oracle_fa(qb.transpose(0, 2, 1, 3), cache_k[:, :, :90], v), base)


def test_flash_attn_vs_reference_live(oracle, ref):
    for (B, Hq, Hkv, nq, nkv, kvt) in ((1, 16, 2, 256, 256, np.float16), (2, 16, 2, 1, 2048, np.float32),
                                       (3, 8, 2, 5, 113, np.float32), (1, 4, 4, 64, 70, np.float32)):
        q = rng("fl", nq, nkv).standard_normal((B, Hq, nq, 64)).astype(np.float32)
        k = rng("flk", nq, nkv).standard_normal((B, Hkv, nkv, 64)).astype(kvt)
        v = rng("flv", nq, nkv).standard_normal((B, Hkv, nkv, 64)).astype(kvt)
        mask = reflib.causal_mask(nq, nkv, n_past=nkv - nq) if nq > 1 else None
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        a = reflib.oracle_fa(q, k, v, mask, path=reflib.ORC_FA_AUTO, nth=8)
        b = reflib.ref_fa(q, k, v, mask)
        assert np.abs(a - b).max() <= 3e-6, (nq, nkv)
    sinks = rng("sinks").standard_normal(8).astype(np.float32)
    q = rng("fs").standard_normal((1, 8, 3, 64)).astype(np.float32)
    k = rng("fsk").standard_normal((1, 2, 40, 64)).astype(np.float32)
    m = rng("fsm").standard_normal((1, 1, 3, 40)).astype(np.float16)
    for kw in (dict(sinks=sinks), dict(max_bias=8.0), dict(softcap=5.0)):
        assert np.abs(reflib.oracle_fa(q, k, k, m, **kw) - reflib.ref_fa(q, k, k, m, **kw)).max() <= 3e-6


# ------------------------------------------------------- host-side index helpers / masks
def test_kv_views_reference_fixture(oracle):
    """tests/test_minicpm.cpp:775-809 of the reference: MiniCPMKVCache(2 layers, 2 kv heads,
    max_length 16, head_dim 8)."""
    ne, nb, off = (C.c_int64 * 3)(), (C.c_uint64 * 3)(), C.c_uint64()
    oracle.orc_kv_read_view(8, 16, 2, 4, 4, ne, nb, C.byref(off))
    assert list(ne) == [8, 4, 2] and list(nb) == [4, 32, 512] and off.value == 0
    oracle.orc_kv_read_view(8, 16, 2, 4, 7, ne, nb, C.byref(off))
    assert list(ne) == [8, 7, 2]
    oracle.orc_kv_write_view(8, 16, 2, 4, 3, 1, ne, nb, C.byref(off))
    assert list(ne) == [8, 2, 1] and list(nb) == [4, 512, 32] and off.value == 96
    oracle.orc_kv_write_view(8, 16, 2, 4, 5, 2, ne, nb, C.byref(off))
    assert list(ne) == [8, 2, 2] and off.value == 160
    # writing token t through the write view and reading through the read view meet at the
    # same element: brute force over a numbered cache
    cache = np.arange(2 * 16 * 8, dtype=np.float32).reshape(2, 16, 8)  # [D, max_length, Hkv] in ggml order
    raw = cache.view(np.uint8).reshape(-1)
    for start in range(15):
        oracle.orc_kv_write_view(8, 16, 2, 4, start, 2, ne, nb, C.byref(off))
        for t in range(2):
            for h in range(2):
                for d in range(8):
                    o = off.value + d * nb[0] + h * nb[1] + t * nb[2]
                    assert raw[o:o + 4].view(np.float32)[0] == cache[h, start + t, d]


def test_causal_mask_and_cfg_pair(oracle):
    m = reflib.causal_mask(4, 6, n_past=2).view(np.uint16)
    for r in range(4):
        for c in range(6):
            assert m[r, c] == (0x8000 if c <= r + 2 else 0xFC00)
    L = 7
    pos = np.zeros(2 * L, np.int32)
    mk = np.zeros((2 * L, 2 * L), np.uint16)
    oracle.orc_cfg_pair_constants(L, ptr(pos, C.c_int32), ptr(mk, C.c_uint16))
    assert list(pos) == list(range(L)) * 2
    blk = mk.reshape(2, L, 2, L)
    assert (blk[0, :, 0] == 0).all() and (blk[1, :, 1] == 0).all()
    assert (blk[0, :, 1] == 0xFC00).all() and (blk[1, :, 0] == 0xFC00).all()


def test_t_span_reference_fixture(oracle):
    """tests/test_unified_cfm.cpp:155-164: compute_t_span(10, 1.0) against its closed form."""
    out = np.zeros(11, np.float32)
    oracle.orc_t_span(10, 1.0, ptr(out, C.c_float))
    base = 1.0 - np.arange(11) / 10.0
    want = base + 1.0 * (np.cos(np.pi / 2 * base) - 1.0 + base)
    assert np.abs(out - want).max() <= 1e-6
    assert out[0] == pytest.approx(1.0) and abs(out[10]) <= 1e-6
