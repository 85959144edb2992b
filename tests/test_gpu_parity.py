"""GPU parity: every claimed ggml op, called through the C ABI of libvoxcpm_gfx950.so on
cuda:0, against the CPU oracle (oracle/liboracle.so) on the same seeded inputs -- and, where
the reference's own ggml-cpu was prebuilt (oracle/_ref), against that as well.

Tolerances.  Attention: 2e-3 max-abs against the fp32-accumulating ggml-cpu arithmetic
(K/V handed to the oracle as F32 tensors holding the f16 cache values), the bar the task
states.  MUL_MAT: VX_ACT_Q8 reproduces ggml-cpu's integer block dots, so it is held to
1e-5 relative; VX_ACT_FLOAT (weights dequantised exactly, activations as f16) is held to
ggml's own backend-test bar, NMSE <= 5e-4 against ggml-cpu, and to 1e-5 NMSE against the
fp64 dequantise-then-multiply reference.  RMS_NORM / ROPE / SOFT_MAX: 1e-5 max-abs or better.
"""
import sys

import numpy as np
import pytest

import reflib
from reflib import nmse, rng

pytestmark = pytest.mark.gpu

FA_TOL = 2e-3


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def sync_np(t):
    import torch
    torch.cuda.synchronize()
    return t.cpu().numpy()


# ------------------------------------------------------------------------------ RMS_NORM
@pytest.mark.parametrize("shape", [(1, 1024), (2, 1024), (512, 1024), (3, 5, 64), (7, 1025), (2, 3, 4, 4096), (5, 10000)])
@pytest.mark.parametrize("eps", [1e-5, 0.0, 0.1])
def test_rms_norm(gpu, shape, eps):
    say(f"rms_norm shape={shape} eps={eps}")
    x = rng("rms", shape).standard_normal(shape).astype(np.float32)
    want = reflib.oracle_rms_norm(x, eps)
    got = sync_np(gpu.rms_norm(dev(x), eps))
    assert np.abs(got - want).max() <= 1e-6 * max(1.0, np.abs(want).max())
    # scale invariance: rms_norm(c*x) == rms_norm(x) when eps is negligible
    if eps == 0.0:
        got2 = sync_np(gpu.rms_norm(dev(x * np.float32(8.0)), eps))
        assert np.abs(got2 - got).max() <= 1e-6


def test_rms_norm_strided_and_inplace(gpu):
    import torch
    say("rms_norm strided view + in place")
    base = rng("rms", "strided").standard_normal((6, 2048)).astype(np.float32)
    xv = base[:, :1024]  # row stride 2048 floats
    want = reflib.oracle_rms_norm(np.ascontiguousarray(xv), 1e-5)
    t = dev(base)
    view = t[:, :1024]
    got = sync_np(gpu.rms_norm(view, 1e-5, out=torch.empty((6, 1024), device="cuda")))
    assert np.abs(got - want).max() <= 1e-6
    gpu.rms_norm(view, 1e-5, out=view)  # in place on the strided view
    after = sync_np(t)
    assert np.abs(after[:, :1024] - want).max() <= 1e-6
    assert np.array_equal(after[:, 1024:], base[:, 1024:])  # neighbours untouched


# ---------------------------------------------------------------------------------- ROPE
@pytest.mark.parametrize("mode", [0, 2])
@pytest.mark.parametrize("case", ["decode", "prefill", "long", "partial", "yarn", "prefill batch partial", "prefill yarn"])
def test_rope(gpu, mode, case):
    say(f"rope mode={mode} case={case}")
    if case == "prefill batch partial":   # many tokens: the kernel that walks a token's heads; 6 heads (a ragged group of four), a tail that is copied
        shape, pos = (4, 300, 6, 80), np.arange(300, dtype=np.int32) * 3 + 7
    elif case == "prefill yarn":
        shape, pos = (1, 1100, 5, 128), np.arange(1100, dtype=np.int32) * 7
    elif case == "decode":
        shape, pos = (2, 1, 16, 64), np.array([4095], np.int32)
    elif case == "prefill":
        shape, pos = (1, 256, 16, 64), np.arange(256, dtype=np.int32)
    elif case == "long":
        shape, pos = (1, 64, 2, 64), np.arange(8192 - 64, 8192, dtype=np.int32)
    elif case == "partial":
        shape, pos = (1, 9, 3, 80), np.arange(9, dtype=np.int32) * 37
    else:
        shape, pos = (1, 33, 4, 128), np.arange(33, dtype=np.int32) * 301
    x = rng("rope", case, mode).standard_normal(shape).astype(np.float32)
    n_dims = 64 if case in ("decode", "prefill", "long", "partial", "prefill batch partial") else 128
    ff = (1.0 + rng("rope", "ff").random(n_dims // 2)).astype(np.float32) if "partial" not in case else None
    kw = dict(n_ctx_orig=32768, freq_base=10000.0, freq_scale=1.0, ext_factor=0.0, attn_factor=1.0,
              beta_fast=32.0, beta_slow=1.0)
    if "yarn" in case:
        kw.update(freq_scale=0.25, ext_factor=1.0, attn_factor=1.3, n_ctx_orig=4096)
    want = reflib.oracle_rope(x, pos, ff, n_dims, mode, **kw)
    got = sync_np(gpu.rope_ext(dev(x), dev(pos), None if ff is None else dev(ff), n_dims, mode, kw["n_ctx_orig"],
                               kw["freq_base"], kw["freq_scale"], kw["ext_factor"], kw["attn_factor"],
                               kw["beta_fast"], kw["beta_slow"]))
    err = np.abs(got - want).max()
    say(f"   max-abs {err:.3e}")
    # only sinf/cosf differ from the host libm (the angle chain is replayed exactly)
    assert err <= 2e-5
    # each rotated pair keeps its norm (times attn_factor)
    if case == "prefill":
        h = n_dims // 2
        pairs_in = x[..., :h] ** 2 + x[..., h:] ** 2 if mode == 2 else x[..., 0::2] ** 2 + x[..., 1::2] ** 2
        pairs_out = got[..., :h] ** 2 + got[..., h:] ** 2 if mode == 2 else got[..., 0::2] ** 2 + got[..., 1::2] ** 2
        assert np.allclose(pairs_in, pairs_out, rtol=1e-4, atol=1e-5)


def test_rope_inplace_pos0(gpu):
    say("rope in place, position 0 is the identity")
    x = rng("rope", "id").standard_normal((1, 3, 16, 64)).astype(np.float32)
    t = dev(x)
    gpu.rope_ext(t, dev(np.zeros(3, np.int32)), None, 64, 2, 32768, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0, out=t)
    assert np.array_equal(sync_np(t), x)


# ------------------------------------------------------------------------------ SOFT_MAX
@pytest.mark.parametrize("ncols", [7, 64, 1000, 8192, 20000])
@pytest.mark.parametrize("mask_type", [None, np.float16, np.float32])
def test_soft_max(gpu, ncols, mask_type):
    say(f"soft_max ncols={ncols} mask={mask_type}")
    x = rng("sm", ncols).standard_normal((2, 4, 5, ncols)).astype(np.float32)
    mask = None if mask_type is None else rng("sm", "m", ncols).standard_normal((1, 1, 5, ncols)).astype(mask_type)
    max_bias = 8.0 if mask is not None else 0.0
    sinks = rng("sm", "sinks").standard_normal(4).astype(np.float32) if ncols == 64 else None
    want = reflib.oracle_soft_max(x, mask, 0.3, max_bias, sinks)
    got = sync_np(gpu.soft_max_ext(dev(x), None if mask is None else dev(mask), 0.3, max_bias,
                                   None if sinks is None else dev(sinks)))
    assert np.abs(got - want).max() <= 1e-6
    if sinks is None:
        assert np.allclose(got.sum(-1), 1.0, atol=1e-5)


# ------------------------------------------------------------------------ FLASH_ATTN_EXT
def fa_case(gpu, q, k, v, mask=None, scale=0.125, max_bias=0.0, softcap=0.0, sinks=None, tol=FA_TOL, name=""):
    """q, k, v, mask: numpy arrays (possibly strided views).  Returns the max-abs error."""
    import torch
    kf = np.ascontiguousarray(k).astype(np.float32)
    vf = np.ascontiguousarray(v).astype(np.float32)
    want = reflib.oracle_fa(np.ascontiguousarray(q), kf, vf, mask, scale, max_bias, softcap, sinks,
                            path=reflib.ORC_FA_VEC)

    def same_view(a):  # device tensor with the same shape and strides as the numpy view
        base = a
        while base.base is not None and isinstance(base.base, np.ndarray):
            base = base.base
        tb = torch.from_numpy(base).cuda()
        off = (a.__array_interface__["data"][0] - base.__array_interface__["data"][0]) // a.itemsize
        return torch.as_strided(tb.view(-1), a.shape, [s // a.itemsize for s in a.strides], off)

    got = sync_np(gpu.flash_attn_ext(same_view(q), same_view(k), same_view(v), None if mask is None else dev(mask),
                                     scale, max_bias, softcap, None if sinks is None else dev(sinks)))
    err = float(np.abs(got - want).max())
    say(f"   {name} max-abs vs oracle(fp32 acc) {err:.3e}")
    assert np.isfinite(got).all()
    assert err <= tol, (name, err)
    return got, want


def qkv(tag, B, Hq, Hkv, n_q, n_kv, D=64, kv_dtype=np.float16):
    q = rng(tag, "q").standard_normal((B, Hq, n_q, D)).astype(np.float32)
    k = rng(tag, "k").standard_normal((B, Hkv, n_kv, D)).astype(kv_dtype)
    v = rng(tag, "v").standard_normal((B, Hkv, n_kv, D)).astype(kv_dtype)
    return q, k, v


def test_fa_cfg1_prefill_causal(gpu):
    say("flash_attn cfg1: T=KV=256, 16/2 heads, D=64, f16 KV, causal mask")
    q, k, v = qkv("cfg1", 1, 16, 2, 256, 256)
    got, want = fa_case(gpu, q, k, v, reflib.causal_mask(256, 256), name="cfg1")
    if reflib.load_ref() is not None:
        r = reflib.ref_fa(q, k, v, reflib.causal_mask(256, 256))  # ggml-cpu tiled path (fp32)
        e = float(np.abs(got - r).max())
        say(f"   vs ggml-cpu (reference build) {e:.3e}")
        assert e <= FA_TOL


@pytest.mark.parametrize("L", [128, 512, 2048, 4096])
def test_fa_cfg2_decode(gpu, L):
    say(f"flash_attn cfg2 decode: B=2, 16/2 heads, D=64, f16 KV, L={L}")
    q, k, v = qkv(("cfg2", L), 2, 16, 2, 1, L)
    got, want = fa_case(gpu, q, k, v, None, name=f"decode L={L}")
    f64 = reflib.oracle_fa(q, k, v, f64=True)
    say(f"   vs fp64 brute force {np.abs(got - f64).max():.3e}")
    if reflib.load_ref() is not None:
        r16 = reflib.ref_fa(q, k, v)  # ggml-cpu with F16-typed K/V: accumulates in f16
        say(f"   raw diff vs ggml-cpu F16-typed path {np.abs(got - r16).max():.3e} "
            f"(that path itself is {np.abs(r16 - f64).max():.3e} from fp64)")
        r32 = reflib.ref_fa(q, k.astype(np.float32), v.astype(np.float32))
        assert np.abs(got - r32).max() <= FA_TOL


def test_fa_cfg3_locdit_cfg_pair(gpu):
    say("flash_attn cfg3 LocDiT: 8 requests x CFG pair of 7 tokens, 16/2 heads, block-diagonal mask")
    import ctypes as C
    L = 7
    pos = np.zeros(2 * L, np.int32)
    m = np.zeros((2 * L, 2 * L), np.uint16)
    reflib.load_oracle().orc_cfg_pair_constants(L, reflib.ptr(pos, C.c_int32), reflib.ptr(m, C.c_uint16))
    mask = m.view(np.float16)
    q, k, v = qkv("cfg3", 8, 16, 2, 2 * L, 2 * L, kv_dtype=np.float32)  # LocDiT K/V are F32 activations
    got, _ = fa_case(gpu, q, k, v, mask, name="locdit pair")
    # the pair equals two independent 7-token attentions
    for br in range(2):
        sl = slice(br * L, (br + 1) * L)
        solo = reflib.oracle_fa(np.ascontiguousarray(q[:, :, sl]), np.ascontiguousarray(k[:, :, sl]),
                                np.ascontiguousarray(v[:, :, sl]), None)
        assert np.abs(got[:, sl] - solo).max() <= FA_TOL


@pytest.mark.parametrize("n_q,n_kv", [(5, 5), (1, 1), (3, 113), (16, 512), (35, 1024), (75, 113), (2, 33)])
@pytest.mark.parametrize("masked", [False, True])
def test_fa_ragged(gpu, n_q, n_kv, masked):
    say(f"flash_attn ragged n_q={n_q} n_kv={n_kv} mask={masked}")
    q, k, v = qkv(("rag", n_q, n_kv), 3, 8, 2, n_q, n_kv)
    mask = None
    if masked:
        mm = rng("rag", "m", n_q, n_kv).standard_normal((1, 1, n_q, n_kv)).astype(np.float32)
        mm[rng("rag", "d", n_q, n_kv).random(mm.shape) < 0.3] = -np.inf
        mask = mm.astype(np.float16)
    fa_case(gpu, q, k, v, mask, name="ragged")


def test_fa_special_cases(gpu):
    say("flash_attn special cases: n_kv=1 -> out = v; equal keys -> mean(V); fully masked row -> 0")
    q, k, v = qkv("sp1", 1, 16, 2, 4, 1)
    got, _ = fa_case(gpu, q, k, v, None, name="n_kv=1")
    for h in range(16):
        assert np.abs(got[0, :, h] - v[0, h // 8, 0].astype(np.float32)).max() <= 1e-6
    q, k, v = qkv("sp2", 1, 16, 2, 3, 200)
    k[:] = k[:, :, :1]
    got, _ = fa_case(gpu, q, k, v, None, name="equal keys")
    mean_v = v.astype(np.float32).mean(axis=2)  # (1, Hkv, D)
    for h in range(16):
        assert np.abs(got[0, :, h] - mean_v[0, h // 8]).max() <= 1e-4
    q, k, v = qkv("sp3", 2, 16, 2, 6, 70)
    mask = np.zeros((1, 1, 6, 70), np.float16)
    mask[0, 0, 2, :] = -np.inf
    mask[0, 0, 4, 10:] = -np.inf
    got, _ = fa_case(gpu, q, k, v, mask, name="masked rows")
    assert np.array_equal(got[:, 2], np.zeros_like(got[:, 2]))
    # permuting the keys leaves the result unchanged
    perm = rng("sp4").permutation(70)
    got2, _ = fa_case(gpu, q, np.ascontiguousarray(k[:, :, perm]), np.ascontiguousarray(v[:, :, perm]),
                      np.ascontiguousarray(mask[..., perm]), name="permuted keys")
    assert np.abs(got - got2).max() <= 1e-5


def test_fa_graph_views(gpu):
    say("flash_attn on the strided views attention_forward builds: q/k/v permuted [D,T,H], KV-cache read view")
    T, Hq, Hkv, D, maxlen = 40, 16, 2, 64, 96
    qb = rng("views", "q").standard_normal((1, T, Hq, D)).astype(np.float32)    # [D, Hq, T] as produced by MUL_MAT
    q = qb.transpose(0, 2, 1, 3)                                                 # ggml_permute(q, 0, 2, 1, 3)
    cache_k = rng("views", "k").standard_normal((1, Hkv, maxlen, D)).astype(np.float16)
    cache_v = rng("views", "v").standard_normal((1, Hkv, maxlen, D)).astype(np.float16)
    k, v = cache_k[:, :, :T], cache_v[:, :, :T]                                  # get_k/get_v(seq_len = T)
    fa_case(gpu, q, k, v, reflib.causal_mask(T, T), name="views")


@pytest.mark.parametrize("kv_dtype", [np.float16, np.float32])
@pytest.mark.parametrize("D", [64, 128])
def test_fa_dtypes_and_head_sizes(gpu, kv_dtype, D):
    say(f"flash_attn D={D} kv={kv_dtype.__name__}")
    q, k, v = qkv(("dt", D, kv_dtype.__name__), 2, 8, 2, 9, 300, D=D, kv_dtype=kv_dtype)
    fa_case(gpu, q, k, v, reflib.causal_mask(9, 300, n_past=291), scale=1.0 / np.sqrt(D), name="dtype")


def test_fa_sinks_softcap_alibi(gpu):
    say("flash_attn with sinks, logit soft cap and ALiBi slopes")
    q, k, v = qkv("ext", 2, 12, 4, 4, 150)
    mask = rng("ext", "m").standard_normal((1, 1, 4, 150)).astype(np.float16)
    sinks = rng("ext", "s").standard_normal(12).astype(np.float32)
    fa_case(gpu, q, k, v, mask, max_bias=8.0, name="alibi")
    fa_case(gpu, q, k, v, mask, softcap=10.0, name="softcap")
    fa_case(gpu, q, k, v, mask, sinks=sinks, name="sinks")
    q, k, v = qkv("ext2", 1, 12, 4, 1, 2000)
    fa_case(gpu, q, k, v, None, sinks=sinks, name="sinks + split")


@pytest.mark.parametrize("seed", list(range(64)))
def test_fa_random_shapes(gpu, seed):
    """Random shapes around every boundary the kernels have (16-column tiles, 32-key tiles, the cut into key ranges, the
    half tile of at most 16 keys, the LDS-tiled prefill kernel's 64-key tiles): batch, GQA ratio, query rows, key count,
    head size, K/V type, mask with switched-off keys and whole switched-off rows per head or shared, ALiBi, soft cap, sinks --
    against the scalar oracle, with the tolerance of every other attention test."""
    r = rng("fa-random", seed)
    B, Hkv, gqa = int(r.choice([1, 2, 3])), int(r.choice([1, 2, 4])), int(r.choice([1, 2, 4, 8]))
    n_q = int(r.choice([1, 1, 2, 5, 16, 17, 40, 70]))
    n_kv = int(r.choice([1, 7, 16, 17, 31, 32, 33, 64, 100, 255, 256, 257, 300, 513, 777, 1024, 1300]))
    D = int(r.choice([64, 64, 128]))
    kv_dtype = np.float16 if r.integers(3) else np.float32
    q, k, v = qkv(("far", seed), B, Hkv * gqa, Hkv, n_q, n_kv, D=D, kv_dtype=kv_dtype)
    mask = None
    if r.integers(3):
        per = int(r.choice([1, Hkv * gqa])) if r.integers(2) else 1          # one mask for all heads, or one per head
        mm = r.standard_normal((int(r.choice([1, B])), per, n_q, n_kv)).astype(np.float32)
        mm[r.random(mm.shape) < 0.3] = -np.inf
        if n_q > 1 and r.integers(2): mm[:, :, int(r.integers(n_q))] = -np.inf   # a row that sees no key
        mask = mm.astype(np.float16)
    extra = int(r.integers(4))
    max_bias = 8.0 if extra == 1 and mask is not None else 0.0
    softcap = 10.0 if extra == 2 else 0.0
    sinks = r.standard_normal(Hkv * gqa).astype(np.float32) if extra == 3 else None
    say(f"flash_attn random seed={seed}: B={B} heads={Hkv * gqa}/{Hkv} n_q={n_q} n_kv={n_kv} D={D} kv={kv_dtype.__name__} "
        f"mask={None if mask is None else mask.shape} max_bias={max_bias} softcap={softcap} sinks={sinks is not None}")
    fa_case(gpu, q, k, v, mask, scale=1.0 / np.sqrt(D), max_bias=max_bias, softcap=softcap, sinks=sinks, name=f"random {seed}")


def test_fa_cfg5_shape_properties(gpu):
    """BASELINE config 5 decode shape (batch 16, L = 8192): too big for the scalar oracle in
    seconds, so check a sample of (batch, head) slices against it plus convexity everywhere."""
    import torch
    say("flash_attn cfg5 decode shape: B=16, L=8192, 16/2 heads")
    B, L = 16, 8192
    q, k, v = qkv("cfg5", B, 16, 2, 1, L)
    got = sync_np(gpu.flash_attn_ext(dev(q), dev(k), dev(v), None, 0.125))
    assert np.isfinite(got).all()
    vmin = v.astype(np.float32).min(axis=2)  # (B, Hkv, D)
    vmax = v.astype(np.float32).max(axis=2)
    for h in range(16):
        assert (got[:, 0, h] >= vmin[:, h // 8] - 1e-5).all() and (got[:, 0, h] <= vmax[:, h // 8] + 1e-5).all()
    for b in (0, 7, 15):
        want = reflib.oracle_fa(q[b:b + 1], k[b:b + 1].astype(np.float32), v[b:b + 1].astype(np.float32))
        err = np.abs(got[b:b + 1] - want).max()
        say(f"   batch {b}: max-abs {err:.3e}")
        assert err <= FA_TOL


def test_fa_full_size_invariants(gpu):
    """Properties that hold at any size, checked at BASELINE config 5's shapes where the scalar
    oracle is too slow: permuting the keys (K and V rows together) leaves decode attention
    unchanged; the output is linear in V; prefill attention without a mask equals the
    wave kernel's result on a sample of rows (two independent kernels, same arithmetic)."""
    import torch
    say("flash_attn full-size invariants: B=16, L=8192 decode; T=4096 prefill")
    B, L = 16, 8192
    q, k, v = qkv("cfg5inv", B, 16, 2, 1, L)
    qd, kd, vd = dev(q), dev(k), dev(v)
    base = gpu.flash_attn_ext(qd, kd, vd, None, 0.125).clone()
    perm = torch.from_numpy(rng("cfg5inv", "perm").permutation(L)).cuda()
    got = gpu.flash_attn_ext(qd, kd[:, :, perm].contiguous(), vd[:, :, perm].contiguous(), None, 0.125)
    e_perm = float((got - base).abs().max())
    v2 = dev(rng("cfg5inv", "v2").standard_normal(v.shape).astype(np.float16))
    o2 = gpu.flash_attn_ext(qd, kd, v2, None, 0.125).clone()
    vsum = (vd.float() + 2.0 * v2.float())  # F32 V: the sum is not f16-representable
    o12 = gpu.flash_attn_ext(qd, kd.float(), vsum, None, 0.125)
    e_lin = float((o12 - (base + 2.0 * o2)).abs().max())
    say(f"   key permutation: max-abs {e_perm:.3e};  linearity in V: max-abs {e_lin:.3e}")
    # the streaming kernel of an f16 cache rounds Q and the probabilities to f16 (the prefill kernel's arithmetic): the
    # order of the keys moves which probabilities share a reference, and the F32 comparison run keeps hi + lo parts of
    # everything; both stay two orders of magnitude inside the 2e-3 bar
    assert e_perm <= 2e-4
    assert e_lin <= 2e-4

    T = 4096
    q, k, v = qkv("cfg5pre", 1, 16, 2, T, T)
    mask = dev(reflib.causal_mask(T, T))
    qd, kd, vd = dev(q), dev(k), dev(v)
    full = gpu.flash_attn_ext(qd, kd, vd, mask, 0.125).clone()          # LDS-tiled kernel
    rows = [0, 1, 63, 64, 2047, 4095]
    for r in rows:                                                         # wave kernel: one row, keys 0..r
        one = gpu.flash_attn_ext(qd[:, :, r:r + 1].contiguous(), kd[:, :, :r + 1].contiguous(),
                                 vd[:, :, :r + 1].contiguous(), None, 0.125)
        err = float((one[0, 0] - full[0, r]).abs().max())
        say(f"   prefill row {r}: max-abs vs single-row decode {err:.3e}")
        assert err <= FA_TOL
    torch.cuda.synchronize()


def test_fa_prefill_kernel_for_f32_kv(gpu, monkeypatch):
    """F32 K/V (the reference's own cache type, and every prefill's keys) take the LDS-tiled kernel with K rounded to
    f16 like Q and V kept as a high and a low half: the 2e-3 bar holds as it does for an f16 cache, also for a row that
    sees one key only (its output is that key's V, which a V rounded to f16 would miss by half an f16 ulp).  With
    VX_FA_F32_PREFILL=0 they go to the hi/lo wave kernel (1e-6)."""
    say("flash_attn prefill kernel, F32 K/V: tiled kernel by default, the wave kernel on request")
    B, Hq, Hkv, T = 2, 16, 2, 1024
    q, k, v = qkv(("pf32", T), B, Hq, Hkv, T, T, kv_dtype=np.float32)
    v *= 4.0                                      # |v| up to ~18: half an f16 ulp would be 8e-3
    mask = reflib.causal_mask(T, T)
    monkeypatch.delenv("VX_FA_F32_PREFILL", raising=False)
    got, want = fa_case(gpu, q, k, v, mask, tol=4 * FA_TOL, name="F32 K/V, tiled kernel (values x4: bar x4)")
    assert np.abs(got[:, 0] - want[:, 0]).max() <= 1e-5          # row 0 sees key 0 only: V to full precision
    assert np.abs(got - want).max() > 2e-5                        # it did take the f16-P kernel
    monkeypatch.setenv("VX_FA_F32_PREFILL", "0")
    fa_case(gpu, q, k, v, mask, tol=1e-4, name="F32 K/V, wave kernel on request")


@pytest.mark.parametrize("case", ["causal", "wide", "past", "nomask", "f32kv", "random_mask", "mha", "sinks_alibi", "ragged"])
def test_fa_prefill_kernel(gpu, case):
    """Shapes large enough to take the LDS-tiled prefill kernel (>= 256 columns per KV head,
    >= 32 work-groups of 256 columns)."""
    say(f"flash_attn prefill kernel: {case}")
    B, Hq, Hkv, T, KV = 4, 16, 2, 512, 512
    mask, sinks, max_bias, kvt = None, None, 0.0, np.float16
    if case == "causal":          # 128 work-groups: the half-width (128-column) form
        mask = reflib.causal_mask(T, KV)
    elif case == "wide":          # 512 work-groups of 256 columns: the full-width form
        B = 16
        mask = reflib.causal_mask(T, KV)
    elif case == "past":
        T, KV = 300, 700
        mask = reflib.causal_mask(T, KV, n_past=KV - T)
    elif case == "f32kv":
        kvt = np.float32
        mask = reflib.causal_mask(T, KV)
    elif case == "random_mask":
        T, KV = 256, 333
        mm = rng("pf", "m").standard_normal((1, 1, T, KV)).astype(np.float32)
        mm[rng("pf", "d").random(mm.shape) < 0.4] = -np.inf
        mm[:, :, 17, :] = -np.inf
        mask = mm.astype(np.float16)
    elif case == "mha":
        B, Hq, Hkv, T, KV = 2, 4, 4, 2048, 128
        mask = None
    elif case == "sinks_alibi":
        T, KV = 256, 256
        mask = rng("pf", "am").standard_normal((1, 1, T, KV)).astype(np.float16)
        sinks = rng("pf", "s").standard_normal(Hq).astype(np.float32)
        max_bias = 8.0
    elif case == "ragged":
        B, T, KV = 5, 250, 999
        mask = reflib.causal_mask(T, KV, n_past=KV - T)
    q, k, v = qkv(("pf", case), B, Hq, Hkv, T, KV, kv_dtype=kvt)
    fa_case(gpu, q, k, v, mask, max_bias=max_bias, sinks=sinks, name=f"prefill {case}")


# ------------------------------------------------------------------------------- MUL_MAT
def mm_inputs(tag, M, K, N, batch=()):
    w = (rng(tag, "w").standard_normal(batch + (M, K)) * 0.02).astype(np.float32)
    x = rng(tag, "x").standard_normal(batch + (N, K)).astype(np.float32)
    return w, x


@pytest.mark.parametrize("M,K,N", [(1024, 1024, 1), (1024, 1024, 2), (128, 1024, 2), (4096, 1024, 2), (1024, 4096, 2),
                                   (1024, 1024, 5), (1024, 1024, 16), (1024, 1024, 17), (1000, 1024, 33),
                                   (3072, 1024, 112), (1024, 1024, 512), (70, 96, 130),
                                   # the 128 x 128 pipelined GEMM: full tiles, and ragged rows / tokens / odd block count
                                   (4096, 1024, 1024), (2000, 1056, 1700),
                                   # operands through LDS: ragged rows and tokens on 128 x 128 and 64 x 64 tiles, few rows
                                   (2000, 1024, 1700), (1000, 1024, 333), (64, 1024, 4100), (130, 2048, 9000),
                                   # a long K on a small grid: K cut across work-groups, partials added by a second kernel
                                   (1024, 4096, 600), (1000, 2176, 300),
                                   # 64 to 256 tiles of 64 x 64 with 68 and 34 rounds of K: quarters and halves of 17 rounds, an odd
                                   # number for the two-round loop of the LDS-operand kernel
                                   (1024, 4352, 1000), (1000, 2176, 600),
                                   # the same on the LDS-operand kernel when its 64 x 64 tiles are few (the down-projection of
                                   # 8 requests' 112 tokens): 8, 8 and 4 splits, ragged rows and tokens
                                   (1024, 4096, 112), (1000, 4096, 70), (512, 2048, 64),
                                   # 17 to 63 tokens behind a K beyond the streaming kernel's 2048: one ragged token tile of the
                                   # LDS-operand kernel with its K cut (a short prompt's down-projection)
                                   (1024, 4096, 17), (1024, 4096, 40), (1000, 2304, 63), (2048, 4096, 33)])
def test_mul_mat_q8_0(gpu, M, K, N):
    say(f"mul_mat Q8_0 M={M} K={K} N={N}")
    w, x = mm_inputs(("q8", M, K, N), M, K, N)
    wq = reflib.quantize_q8_0(w)
    cpu = reflib.oracle_mul_mat(wq, x, K, act_mode=0)          # ggml-cpu arithmetic (int8 x int8)
    f64 = reflib.oracle_mul_mat(wq, x, K, f64=True)            # dequantise, multiply in fp64
    got_q8 = sync_np(gpu.mul_mat(dev(wq), dev(x), gpu.ACT_Q8, w_ne0=K))
    got_fl = sync_np(gpu.mul_mat(dev(wq), dev(x), gpu.ACT_FLOAT, w_ne0=K))
    scale = np.abs(cpu).max()
    e_q8 = np.abs(got_q8 - cpu).max() / scale
    say(f"   ACT_Q8 vs ggml-cpu arithmetic: rel max {e_q8:.3e};  ACT_FLOAT: nmse vs cpu {nmse(cpu, got_fl):.3e}, "
        f"vs fp64 dequant {nmse(f64, got_fl):.3e}")
    assert e_q8 <= 1e-5
    assert nmse(cpu, got_fl) <= 5e-4
    assert nmse(f64, got_fl) <= 1e-5


def test_mul_mat_q8_0_full_size_prefill(gpu):
    """The gate/up product of a full-size prefill: 4096 rows, K = 1024, 16 sequences x 1024 tokens (the shape the Q8_0 GEMM
    is measured on).  Every token's row of the result depends on that token alone, so the oracle is run on a sample of 96
    tokens (the first and last tiles, and random ones) with test_mul_mat_q8_0's bars; the whole result is compared with
    ggml-cpu where its build is there."""
    M, K, N = 4096, 1024, 16384
    say(f"mul_mat Q8_0 M={M} K={K} N={N}")
    w, x = mm_inputs(("q8-full", M, K, N), M, K, N)
    wq = reflib.quantize_q8_0(w)
    wd, xd = dev(wq), dev(x)
    got_q8 = sync_np(gpu.mul_mat(wd, xd, gpu.ACT_Q8, w_ne0=K))
    got_fl = sync_np(gpu.mul_mat(wd, xd, gpu.ACT_FLOAT, w_ne0=K))
    pick = np.unique(np.concatenate([np.arange(32), np.arange(N - 32, N), rng("q8-full", "pick").integers(0, N, 32)]))
    xs = np.ascontiguousarray(x[pick])
    cpu = reflib.oracle_mul_mat(wq, xs, K, act_mode=0)
    f64 = reflib.oracle_mul_mat(wq, xs, K, f64=True)
    e_q8 = np.abs(got_q8[pick] - cpu).max() / np.abs(cpu).max()
    say(f"   {len(pick)} sampled tokens: ACT_Q8 vs ggml-cpu arithmetic rel max {e_q8:.3e};  ACT_FLOAT nmse vs cpu "
        f"{nmse(cpu, got_fl[pick]):.3e}, vs fp64 dequant {nmse(f64, got_fl[pick]):.3e}")
    assert e_q8 <= 1e-5
    assert nmse(cpu, got_fl[pick]) <= 5e-4
    assert nmse(f64, got_fl[pick]) <= 1e-5
    if reflib.load_ref() is not None:
        r = reflib.ref_mul_mat(wq, x, K)
        e = np.abs(got_q8 - r).max() / np.abs(r).max()
        say(f"   all {N} tokens vs ggml-cpu (reference build): ACT_Q8 rel max {e:.3e}, ACT_FLOAT nmse {nmse(r, got_fl):.3e}")
        assert e <= 1e-5
        assert nmse(r, got_fl) <= 5e-4


@pytest.mark.parametrize("M,K,N,batch", [(4096, 1024, 4096, 1), (1024, 4096, 2048, 1), (2000, 1056, 1700, 1), (1030, 1024, 1100, 1),
                                         (1024, 1024, 1024, 3), (1024, 2176, 1500, 2)])
@pytest.mark.parametrize("folded", [False, True])
def test_mul_mat_q8_0_pretiled_equals_the_lds_kernel(gpu, M, K, N, batch, folded, monkeypatch):
    """Products of 1024 rows and tokens or more take the kernel whose operands two passes lay out beforehand (weights as
    exact f16 integers with their scales apart, activations rounded to f16); VX_GEMM_Q8T=0 keeps them on the kernel that
    converts inside every tile.  Both form a block's partial product with the same matrix instruction and scale and add
    it in fp32 in the same order: the plain product, the fused residual update and the fused gate/up SwiGLU must be the
    same bits -- full and ragged tiles in both dimensions, K with an odd number of blocks, a batch of sequences.  folded:
    the opt-in form of both kernels (VX_GEMM_LDS=2) in which the block scale is multiplied into the f16 weights."""
    import torch
    L, d = gpu.lib(), gpu.desc
    say(f"pre-tiled Q8_0 product vs the LDS kernel M={M} K={K} N={N} batch={batch} folded={folded}")
    if folded:
        monkeypatch.setenv("VX_GEMM_LDS", "2")
    else:
        monkeypatch.delenv("VX_GEMM_LDS", raising=False)
    w = (rng("q8t", "w", M, K).standard_normal((M, K)) * 0.02).astype(np.float32)
    w2 = (rng("q8t", "w2", M, K).standard_normal((M, K)) * 0.02).astype(np.float32)
    x = rng("q8t", "x", N, K).standard_normal((batch, N, K) if batch > 1 else (N, K)).astype(np.float32)
    wq, wq2, xd = dev(reflib.quantize_q8_0(w)), dev(reflib.quantize_q8_0(w2)), dev(x)

    def both(fn):
        monkeypatch.setenv("VX_GEMM_Q8T", "2")   # (also where the launcher would find too few tiles for it)
        a = fn()
        monkeypatch.setenv("VX_GEMM_Q8T", "0")
        b = fn()
        monkeypatch.delenv("VX_GEMM_Q8T", raising=False)
        torch.cuda.synchronize()
        return a, b

    a, b = both(lambda: gpu.mul_mat(wq, xd, gpu.ACT_FLOAT, w_ne0=K))
    assert torch.equal(a, b), float((a - b).abs().max())
    cpu = reflib.oracle_mul_mat(reflib.quantize_q8_0(w), x[..., :64, :] if batch == 1 else x[0, :64], K, f64=True)
    got = a[:64] if batch == 1 else a[0, :64]
    assert nmse(cpu, got.cpu().numpy()) <= 1e-5
    res = dev(rng("q8t", "res", M, N).standard_normal(tuple(a.shape)).astype(np.float32))

    def scale_add():
        out = torch.empty_like(a)
        gpu.check(L.vx_mul_mat_scale_add(gpu.desc_q8(wq, K), d(xd), d(res), d(out), 0.2857738, gpu.ACT_FLOAT, None), "mul_mat_scale_add")
        return out

    def swiglu():
        out = torch.empty_like(a)
        gpu.check(L.vx_mul_mat_swiglu(gpu.desc_q8(wq, K), gpu.desc_q8(wq2, K), d(xd), d(out), gpu.ACT_FLOAT, None), "mul_mat_swiglu")
        return out

    if L.vx_supports_mul_mat_scale_add(gpu.desc_q8(wq, K), d(xd), d(res), d(a)):
        a2, b2 = both(scale_add)
        assert torch.equal(a2, b2), float((a2 - b2).abs().max())
    if L.vx_supports_mul_mat_swiglu_tiled(gpu.desc_q8(wq, K), gpu.desc_q8(wq2, K), d(xd), d(a), gpu.ACT_FLOAT):
        a3, b3 = both(swiglu)
        assert torch.equal(a3, b3), float((a3 - b3).abs().max())


@pytest.mark.parametrize("folded", [False, True])
def test_mul_mat_q8_0_pinned_weights_keep_their_tiles(gpu, folded, monkeypatch):
    """vx_weights_pin: the tiles of pinned Q8_0 weights are made once and kept; the product, the residual update and the
    gate/up SwiGLU give the same bits as with the tiles made on every call, on the stream that made the copy and on
    another one; vx_weights_changed drops the copies made from the bytes it names (the next call sees the new weights),
    vx_weights_unpin drops the rest; nothing is kept for weights outside a pinned range."""
    import ctypes as C
    import torch
    L, d = gpu.lib(), gpu.desc
    M, K, N = 2048, 1024, 1100
    monkeypatch.setenv("VX_GEMM_Q8T", "2")
    if folded:
        monkeypatch.setenv("VX_GEMM_LDS", "2")
    else:
        monkeypatch.delenv("VX_GEMM_LDS", raising=False)
    mk = lambda *tag: dev(reflib.quantize_q8_0((rng("pin", *tag).standard_normal((M, K)) * 0.02).astype(np.float32)))
    # one allocation for the two matrices of the pair and a third matrix outside the pinned part
    pool = torch.empty((3,) + tuple(mk("shape").shape), dtype=torch.uint8, device="cuda")
    pool[0], pool[1], pool[2] = mk("w"), mk("w2"), mk("w3")
    wq, wq2, wq3 = pool[0], pool[1], pool[2]
    xd = dev(rng("pin", "x").standard_normal((N, K)).astype(np.float32))
    res = dev(rng("pin", "res").standard_normal((N, M)).astype(np.float32))

    def info():
        v = [C.c_size_t() for _ in range(3)]
        gpu.check(L.vx_weights_info(*[C.byref(x) for x in v]), "info")
        return tuple(x.value for x in v)

    def three(w=wq):
        a = gpu.mul_mat(w, xd, gpu.ACT_FLOAT, w_ne0=K)
        b, c = torch.empty_like(a), torch.empty_like(a)
        gpu.check(L.vx_mul_mat_scale_add(gpu.desc_q8(w, K), d(xd), d(res), d(b), 0.2857738, gpu.ACT_FLOAT, gpu._stream()), "scale_add")
        gpu.check(L.vx_mul_mat_swiglu(gpu.desc_q8(w, K), gpu.desc_q8(wq2, K), d(xd), d(c), gpu.ACT_FLOAT, gpu._stream()), "swiglu")
        torch.cuda.synchronize()
        return a, b, c

    base = info()
    plain = three()
    assert info() == base, "a copy was kept for weights nobody pinned"
    say(f"pinned Q8_0 weights, folded={folded}")
    one = wq.numel()
    gpu.check(L.vx_weights_pin(pool.data_ptr(), 2 * one), "pin")
    try:
        first = three()                      # makes the copies (single matrix, pair)
        held = info()
        assert held[0] == base[0] + 1 and held[1] == base[1] + 2 and held[2] - base[2] >= 3 * 2 * M * K
        again = three()
        assert info() == held
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            other = three()                  # the copies were filled on another stream
        for want, a, b, c in zip(plain, first, again, other):
            assert torch.equal(want, a) and torch.equal(want, b) and torch.equal(want, c)
        p3 = three(wq3)                      # outside the pinned bytes: the pair (wq3, wq2) is not kept either
        assert info() == held
        # new weights at the same address
        wq.copy_(mk("w, rewritten"))
        gpu.check(L.vx_weights_changed(wq.data_ptr(), one), "changed")
        assert info()[1] == base[1]          # both copies held bytes of the first matrix
        monkeypatch.setenv("VX_GEMM_Q8T", "0")
        want = three()
        monkeypatch.setenv("VX_GEMM_Q8T", "2")
        got, got2 = three(), three()
        for w_, a, b in zip(want, got, got2):
            assert torch.equal(w_, a) and torch.equal(w_, b)
        assert not torch.equal(got[0], plain[0])
        assert info() == held
        # under a recording nothing is taken from the copies (a recording must not hold their addresses)
        g = torch.cuda.CUDAGraph()
        out = torch.empty_like(got[0])
        gpu.check(L.vx_workspace_reserve(side.cuda_stream, 64 << 20), "reserve")
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                gpu.mul_mat(wq, xd, gpu.ACT_FLOAT, w_ne0=K, out=out)
        gpu.check(L.vx_weights_unpin(pool.data_ptr()), "unpin")
        assert info() == base
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, got[0])
    finally:
        L.vx_weights_unpin(pool.data_ptr())
    assert L.vx_weights_unpin(pool.data_ptr()) == 3   # VX_ERR_INVALID: nothing is pinned there any more


@pytest.mark.parametrize("seed", list(range(48)))
def test_mul_mat_q8_0_random_shapes(gpu, seed):
    """Random row, column and token counts around every threshold the launcher has (streaming kernel up to 16 tokens and a
    work bound beyond, 64 x 64 and 128 x 128 tiles, the K cut of few tiles, K in whole rounds of 64 or not, rows that are
    no multiple of 4 or 16): both activation modes against the oracle with test_mul_mat_q8_0's bars."""
    r = rng("mm-random", seed)
    M = int(r.choice([1, 3, 16, 24, 64, 65, 130, 200, 512, 1000, 1024, 1030, 2048]))
    K = 32 * int(r.choice([1, 2, 3, 8, 16, 17, 32, 33, 64, 128]))
    N = int(r.choice([1, 2, 3, 5, 14, 16, 17, 31, 33, 63, 64, 65, 100, 112, 127, 128, 129, 200, 300, 520]))
    say(f"mul_mat Q8_0 random seed={seed}: M={M} K={K} N={N}")
    w, x = mm_inputs(("q8r", seed), M, K, N)
    wq = reflib.quantize_q8_0(w)
    cpu = reflib.oracle_mul_mat(wq, x, K, act_mode=0)
    f64 = reflib.oracle_mul_mat(wq, x, K, f64=True)
    got_q8 = sync_np(gpu.mul_mat(dev(wq), dev(x), gpu.ACT_Q8, w_ne0=K))
    got_fl = sync_np(gpu.mul_mat(dev(wq), dev(x), gpu.ACT_FLOAT, w_ne0=K))
    scale = np.abs(cpu).max()
    assert np.abs(got_q8 - cpu).max() / scale <= 1e-5
    assert nmse(cpu, got_fl) <= 5e-4
    assert nmse(f64, got_fl) <= 1e-5


@pytest.mark.parametrize("M,K,N", [(1024, 1024, 1), (1024, 1024, 2), (1000, 1024, 14), (1536, 1024, 16), (1024, 4096, 2), (1024, 4096, 14),
                                   (8192, 1024, 2), (200, 2048, 3), (64, 512, 2), (1024, 768, 5), (24, 1024, 2), (1024, 1024, 17),
                                   (1024, 1024, 40), (4096, 4096, 16)])
def test_gemv_weights_through_lds_equals_the_register_path(gpu, M, K, N, monkeypatch):
    """Products of up to 16 tokens per chunk take the kernel that brings the weight rows into LDS by direct loads when rows
    and activations sit on 16-byte boundaries (K a multiple of 256); VX_GEMV_DMA=0 keeps them on the kernel that loads
    the weights into registers.  Both walk the same k blocks per wave and add in the same order: bit-equal, in both
    activation modes; shapes: ragged rows, 4 / 8 / 16 rows per work-group, four, eight and sixteen waves, K with and
    without whole four-block rounds, several chunks of tokens."""
    say(f"gemv through LDS vs registers M={M} K={K} N={N}")
    w, x = mm_inputs(("dma", M, K, N), M, K, N)
    wq, xd = dev(reflib.quantize_q8_0(w)), dev(x)
    for mode in (gpu.ACT_FLOAT, gpu.ACT_Q8):
        monkeypatch.delenv("VX_GEMV_DMA", raising=False)
        a = sync_np(gpu.mul_mat(wq, xd, mode, w_ne0=K))
        monkeypatch.setenv("VX_GEMV_DMA", "0")
        b = sync_np(gpu.mul_mat(wq, xd, mode, w_ne0=K))
        assert np.array_equal(a, b), (mode, np.abs(a - b).max())
    monkeypatch.delenv("VX_GEMV_DMA", raising=False)
    cpu = reflib.oracle_mul_mat(reflib.quantize_q8_0(w), x, K, act_mode=0)
    assert np.abs(sync_np(gpu.mul_mat(wq, xd, gpu.ACT_Q8, w_ne0=K)) - cpu).max() / np.abs(cpu).max() <= 1e-5


@pytest.mark.parametrize("wtype", [np.float16, np.float32])
@pytest.mark.parametrize("M,K,N", [(1024, 1024, 2), (1024, 64, 14), (333, 256, 40), (64, 1024, 300), (2048, 256, 1600),
                                   (1000, 256, 3000), (200, 192, 700)])
def test_mul_mat_float_weights(gpu, wtype, M, K, N):
    say(f"mul_mat {wtype.__name__} weights M={M} K={K} N={N}")
    w, x = mm_inputs(("fw", M, K, N), M, K, N)
    w = w.astype(wtype)
    cpu = reflib.oracle_mul_mat(w, x, act_mode=0)
    f64 = reflib.oracle_mul_mat(w, x, f64=True)
    got = sync_np(gpu.mul_mat(dev(w), dev(x)))
    say(f"   nmse vs ggml-cpu arithmetic {nmse(cpu, got):.3e}, vs fp64 {nmse(f64, got):.3e}")
    assert nmse(cpu, got) <= 1e-6
    assert nmse(f64, got) <= 1e-6


def test_mul_mat_broadcast_and_views(gpu):
    say("mul_mat batch broadcast (ne12 = 4 over ne02 = 2) and a QKV row-slice view")
    w, _ = mm_inputs("bc", 96, 128, 1, batch=(1, 2))
    x = rng("bc", "x").standard_normal((1, 4, 9, 128)).astype(np.float32)
    wq = reflib.quantize_q8_0(w)
    cpu = reflib.oracle_mul_mat(wq, x, 128, act_mode=0)
    got = sync_np(gpu.mul_mat(dev(wq), dev(x), gpu.ACT_Q8, w_ne0=128))
    assert np.abs(got - cpu).max() <= 1e-5 * np.abs(cpu).max()
    # the same broadcast with enough tokens for the LDS-tiled kernel (one grid plane per batch entry)
    w, _ = mm_inputs("bc2", 192, 128, 1, batch=(1, 2))
    x = rng("bc2", "x").standard_normal((1, 4, 400, 128)).astype(np.float32)
    wq = reflib.quantize_q8_0(w)
    f64 = reflib.oracle_mul_mat(wq, x, 128, f64=True)
    got = sync_np(gpu.mul_mat(dev(wq), dev(x), gpu.ACT_FLOAT, w_ne0=128))
    assert got.shape == f64.shape and nmse(f64, got) <= 1e-6


def test_q8_0_dequant_is_exact(gpu):
    """x = unit vectors: the ACT_FLOAT product then *is* the dequantised weight, which must equal
    ggml's dequantize_row_q8_0 bit for bit."""
    import ctypes as C
    say("Q8_0 dequantisation exact: W x I == dequantize_row_q8_0(W)")
    K, M = 256, 80
    w = (rng("deq", "w").standard_normal((M, K)) * 0.05).astype(np.float32)
    wq = reflib.quantize_q8_0(w)
    deq = np.zeros((M, K), np.float32)
    reflib.load_oracle().orc_dequantize_row_q8_0(wq.ctypes.data, reflib.ptr(deq, C.c_float), M * K)
    eye = np.eye(K, dtype=np.float32)
    got = sync_np(gpu.mul_mat(dev(wq), dev(eye), gpu.ACT_FLOAT, w_ne0=K))  # (K tokens, M rows)
    assert np.array_equal(got.T, deq)


@pytest.mark.parametrize("M", [512, 2048])
def test_q8_0_dequant_on_the_tiled_gemm(gpu, M, monkeypatch):
    """The same unit-vector probe at shapes that run on the LDS-tiled GEMM (64 x 64 and 128 x 128 tiles).  With
    the default (VX_GEMM_LDS=1) the block scale is applied in fp32 and the product is the dequantised weight bit for
    bit; with VX_GEMM_LDS=2 the scale is folded into the f16 operand, i.e. the weight is q * d rounded once to f16."""
    import ctypes as C
    K = 1536
    say(f"Q8_0 dequantisation on the tiled GEMM, M={M}: exact scale mode, folded scale mode")
    w = (rng("deq2", M).standard_normal((M, K)) * 0.05).astype(np.float32)
    w[3, 64:96] *= 1e-4                              # a block whose products are f16 subnormals
    wq = reflib.quantize_q8_0(w)
    deq = np.zeros((M, K), np.float32)
    reflib.load_oracle().orc_dequantize_row_q8_0(wq.ctypes.data, reflib.ptr(deq, C.c_float), M * K)
    eye = np.eye(K, dtype=np.float32)
    monkeypatch.delenv("VX_GEMM_LDS", raising=False)
    got = sync_np(gpu.mul_mat(dev(wq), dev(eye), gpu.ACT_FLOAT, w_ne0=K))
    assert np.array_equal(got.T, deq)
    monkeypatch.setenv("VX_GEMM_LDS", "1")
    got = sync_np(gpu.mul_mat(dev(wq), dev(eye), gpu.ACT_FLOAT, w_ne0=K))
    assert np.array_equal(got.T, deq)
    monkeypatch.setenv("VX_GEMM_LDS", "2")
    got = sync_np(gpu.mul_mat(dev(wq), dev(eye), gpu.ACT_FLOAT, w_ne0=K))
    assert np.array_equal(got.T, deq.astype(np.float16).astype(np.float32))
    monkeypatch.setenv("VX_GEMM_LDS", "0")           # the register-operand kernels
    got = sync_np(gpu.mul_mat(dev(wq), dev(eye), gpu.ACT_FLOAT, w_ne0=K))
    assert np.array_equal(got.T, deq)


# ------------------------------------------------------------------------------ KV cache
@pytest.mark.parametrize("cache_dtype", [np.float16, np.float32])
def test_kv_cache_views_and_store(gpu, cache_dtype):
    import ctypes as C
    import torch
    say(f"kv cache views + store, cache {cache_dtype.__name__}")
    D, maxlen, Hkv = 64, 48, 2
    es = np.dtype(cache_dtype).itemsize
    orc = reflib.load_oracle()
    cache = torch.zeros((Hkv, maxlen, D), dtype=torch.float16 if es == 2 else torch.float32, device="cuda")
    cd = gpu.desc(cache)
    host = np.zeros((Hkv, maxlen, D), cache_dtype)
    start = 0
    for n_tok in (5, 1, 1, 7):
        cur = rng("kv", start).standard_normal((n_tok, Hkv, D)).astype(np.float32)  # [D, Hkv, n_tokens]
        wv = gpu.VxTensor()
        gpu.check(gpu.lib().vx_kv_write_view(cd, start, n_tok, wv), "kv_write_view")
        ne, nb, off = (C.c_int64 * 3)(), (C.c_uint64 * 3)(), C.c_uint64()
        orc.orc_kv_write_view(D, maxlen, Hkv, es, start, n_tok, ne, nb, C.byref(off))
        assert [wv.ne[i] for i in range(3)] == list(ne) and [wv.nb[i] for i in range(3)] == list(nb)
        assert wv.data - cache.data_ptr() == off.value
        gpu.check(gpu.lib().vx_kv_store(gpu.desc(dev(cur)), wv, torch.cuda.current_stream().cuda_stream), "kv_store")
        host[:, start:start + n_tok] = cur.transpose(1, 0, 2).astype(cache_dtype)
        start += n_tok
        rv = gpu.VxTensor()
        gpu.check(gpu.lib().vx_kv_read_view(cd, start, rv), "kv_read_view")
        orc.orc_kv_read_view(D, maxlen, Hkv, es, start, ne, nb, C.byref(off))
        assert [rv.ne[i] for i in range(3)] == list(ne) and [rv.nb[i] for i in range(3)] == list(nb) and off.value == 0
    got = sync_np(cache)
    assert np.array_equal(got.view(np.uint16 if es == 2 else np.uint32), host.view(np.uint16 if es == 2 else np.uint32))
    # attention over the read view equals attention over the dense copy
    q = rng("kv", "q").standard_normal((1, 16, 1, D)).astype(np.float32)
    other = torch.from_numpy(host.copy()).cuda()
    out = gpu.flash_attn_ext(dev(q), cache[None, :, :start], other[None, :, :start], None, 0.125)
    want = reflib.oracle_fa(q, host[None, :, :start].astype(np.float32), host[None, :, :start].astype(np.float32))
    assert np.abs(sync_np(out) - want).max() <= FA_TOL


# ------------------------------------------------------------------- glue ops of a decoder layer
def test_glue_binary_broadcast_and_views(gpu):
    """ADD/SUB/MUL/DIV are single IEEE operations: bit-exact against numpy, with ggml's
    broadcast (norm weight over tokens, bias column) and with strided operands."""
    import torch
    say("glue: binary ops")
    a = rng("glue", "a").standard_normal((2, 3, 5, 1024)).astype(np.float32)
    cases = {"same": a * 0.5 + 1, "row": rng("glue", "w").standard_normal((1024,)).astype(np.float32),
             "col": rng("glue", "c").standard_normal((2, 1, 5, 1)).astype(np.float32),
             "odd": rng("glue", "o").standard_normal((3, 1, 1024)).astype(np.float32)}
    fns = {gpu.BIN_ADD: np.add, gpu.BIN_SUB: np.subtract, gpu.BIN_MUL: np.multiply, gpu.BIN_DIV: np.divide}
    for name, b in cases.items():
        b4 = b.reshape((1,) * (4 - b.ndim) + b.shape)
        for op, fn in fns.items():
            got = sync_np(gpu.binary(op, dev(a), dev(b4)))
            assert np.array_equal(got, fn(a, b4)), (name, op)
    # odd row length (scalar path) and a permuted src0 / transposed src1
    x = rng("glue", "x").standard_normal((4, 7, 33)).astype(np.float32)
    y = rng("glue", "y").standard_normal((4, 33, 7)).astype(np.float32)
    got = sync_np(gpu.binary(gpu.BIN_ADD, dev(x), dev(y).transpose(1, 2)))
    assert np.array_equal(got, x + y.transpose(0, 2, 1))


def test_glue_scale_add1_unary_glu(gpu):
    import torch
    say("glue: scale / add1 / unary / glu")
    x = (rng("glue2", "x").standard_normal((3, 130, 1024)) * 3).astype(np.float32)
    got = sync_np(gpu.scale(dev(x), 0.37))
    assert np.array_equal(got, x * np.float32(0.37))
    got = sync_np(gpu.scale(dev(x), 0.37, 1.5))
    want = (x.astype(np.float64) * np.float64(np.float32(0.37)) + 1.5).astype(np.float32)  # fused multiply-add
    assert np.abs(got - want).max() <= 1e-6 and (got != want).mean() < 1e-3
    s = np.array([0.25], np.float32)
    assert np.array_equal(sync_np(gpu.add1(dev(x), dev(s))), x + s[0])
    x64 = x.astype(np.float64)
    silu = x64 / (1 + np.exp(-x64))
    got = sync_np(gpu.unary(gpu.UNARY_SILU, dev(x)))
    assert np.abs(got - silu).max() <= 2e-6
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_RELU, dev(x))), np.maximum(x, 0))
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_NEG, dev(x))), -x)
    up = rng("glue2", "up").standard_normal(x.shape).astype(np.float32)
    got = sync_np(gpu.glu(gpu.GLU_SWIGLU, dev(x), dev(up)))
    assert np.abs(got - silu * up).max() <= 1e-5
    # one-tensor form: halves of the row, and swapped
    gu = np.concatenate([x, up], axis=-1)
    assert np.array_equal(sync_np(gpu.glu(gpu.GLU_SWIGLU, dev(gu))), got)
    ug = np.concatenate([up, x], axis=-1)
    assert np.array_equal(sync_np(gpu.glu(gpu.GLU_SWIGLU, dev(ug), swapped=True)), got)
    # views of a fused gate|up projection, as mlp_forward builds them
    t = dev(gu)
    assert np.array_equal(sync_np(gpu.glu(gpu.GLU_SWIGLU, t[..., :1024], t[..., 1024:])), got)


@pytest.mark.parametrize("cache_dtype", [np.float16, np.float32])
def test_glue_cpy_cont_concat_sum(gpu, cache_dtype):
    """The KV append of attention_forward: CPY of the rotated keys into the cache's write view,
    CONT + SUM of that view, CONCAT of the past view with the current keys."""
    import torch
    say(f"glue: cpy / cont / concat / sum, cache {np.dtype(cache_dtype).name}")
    D, Hkv, maxlen, n_past, T = 64, 2, 96, 37, 5
    tt = torch.float16 if cache_dtype == np.float16 else torch.float32
    cache0 = rng("glue3", "cache").standard_normal((Hkv, maxlen, D)).astype(cache_dtype)
    kcur = rng("glue3", "k").standard_normal((T, Hkv, D)).astype(np.float32)
    cache = dev(cache0)
    wview = cache[:, n_past:n_past + T].transpose(0, 1)          # (T, Hkv, D): ggml [D, Hkv, T]
    gpu.cpy(dev(kcur), wview)
    want = cache0.copy()
    want[:, n_past:n_past + T] = kcur.transpose(1, 0, 2).astype(cache_dtype)
    assert np.array_equal(sync_np(cache), want)
    cont = torch.empty((T, Hkv, D), dtype=tt, device="cuda")
    gpu.cpy(wview, cont)
    assert np.array_equal(sync_np(cont), want[:, n_past:n_past + T].transpose(1, 0, 2))
    if cache_dtype == np.float32:
        got = float(sync_np(gpu.sum_all(wview))[0])
        assert got == np.float32(kcur.astype(np.float64).sum())
    # reshaping copy: same element count, different shapes (element i -> element i)
    flat = torch.empty((T * Hkv * D // 8, 8), dtype=torch.float32, device="cuda")
    gpu.cpy(wview, flat)
    assert np.array_equal(sync_np(flat).reshape(-1), want[:, n_past:n_past + T].transpose(1, 0, 2).astype(np.float32).reshape(-1))
    # concat(past view [D, n_past, Hkv], permuted current keys [D, T, Hkv]) along ggml dim 1
    past = cache[:, :n_past]
    cur = dev(kcur.astype(cache_dtype)).transpose(0, 1)          # (Hkv, T, D), strided
    got = sync_np(gpu.concat(past, cur, 1))
    assert np.array_equal(got, np.concatenate([want[:, :n_past], kcur.transpose(1, 0, 2).astype(cache_dtype)], axis=1))
    # other dims, odd sizes (element path)
    a = rng("glue3", "a").standard_normal((2, 3, 5, 7)).astype(cache_dtype)
    for gd in range(4):
        shp = list(a.shape); shp[3 - gd] += 2
        b = rng("glue3", "b", gd).standard_normal([2 if i == 3 - gd else n for i, n in enumerate(a.shape)]).astype(cache_dtype)
        assert np.array_equal(sync_np(gpu.concat(dev(a), dev(b), gd)), np.concatenate([a, b], axis=3 - gd))


# ------------------------------------------- the ops around the decoder stacks (masks, embeddings)
def test_glue_arange_repeat_and_the_mask_chains(gpu):
    """ARANGE / REPEAT are exact; chained with SUB, ADD1, STEP / ABS, SCALE and the F32 -> F16 cast
    they build the reference's causal mask (src/minicpm.cpp:602-620) and CFG-pair mask
    (src/locdit.cpp:283-305), compared here with the masks written down directly."""
    import torch
    say("glue: arange / repeat / mask chains")
    for start, stop, step in ((0.0, 10.0, 1.0), (-0.5, 0.5, 1.0), (0.3, 77.1, 0.7), (5.0, -3.0, -0.25)):
        got = sync_np(gpu.arange(start, stop, step))
        f = np.float32
        n = int(np.ceil((f(stop) - f(start)) / f(step)))
        want = (f(start) + (f(step) * np.arange(n, dtype=np.float32)).astype(np.float32)).astype(np.float32)
        assert got.shape == (n,) and np.array_equal(got, want), (start, stop, step)
    for dt in (np.float32, np.float16, np.int32):
        a = (rng("rep", str(dt)).standard_normal((2, 1, 3, 8)) * 100).astype(dt)
        for reps in ((1, 1, 1, 1), (1, 4, 1, 2), (3, 2, 2, 1), (2, 1, 1, 5)):
            shape = tuple(n * r for n, r in zip(a.shape, reps))
            assert np.array_equal(sync_np(gpu.repeat(dev(a), shape)), np.tile(a, reps)), (dt, reps)
        b = a[..., :5]                                            # odd rows, strided source
        assert np.array_equal(sync_np(gpu.repeat(dev(a)[..., :5], (2, 2, 3, 10))), np.tile(b, (1, 2, 1, 2)))
    # causal mask for 5 queries at positions 3..7 over 8 keys
    total, pos = 8, np.arange(3, 8, dtype=np.int32)
    keys = gpu.arange(0.0, float(total), 1.0).reshape(1, total)
    qpos = torch.empty((len(pos), 1), dtype=torch.float32, device="cuda")
    gpu.cpy(dev(pos).reshape(len(pos), 1), qpos)                  # ggml_cast I32 -> F32
    grid_k, grid_q = gpu.repeat(keys, (len(pos), total)), gpu.repeat(qpos, (len(pos), total))
    m = gpu.binary(gpu.BIN_SUB, grid_k, grid_q)
    m = gpu.add1(m, gpu.arange(-0.5, 0.5, 1.0))
    m = gpu.scale(gpu.unary(gpu.UNARY_STEP, m), -1e9)
    m16 = torch.empty(m.shape, dtype=torch.float16, device="cuda")
    gpu.cpy(m, m16)
    want = np.where(np.arange(total)[None, :] > pos[:, None], -np.inf, -0.0).astype(np.float16)
    assert np.array_equal(sync_np(m16).view(np.uint16), want.view(np.uint16))
    # CFG-pair mask: two branches of 7 tokens see only themselves
    L = 7
    ids = gpu.unary(gpu.UNARY_STEP, gpu.add1(gpu.arange(0.0, 2.0 * L, 1.0), gpu.arange(0.5 - L, 1.5 - L, 1.0)))
    kg, qg = gpu.repeat(ids.reshape(1, 2 * L), (2 * L, 2 * L)), gpu.repeat(ids.reshape(2 * L, 1), (2 * L, 2 * L))
    m = gpu.scale(gpu.unary(gpu.UNARY_ABS, gpu.binary(gpu.BIN_SUB, kg, qg)), -1e9)
    m16 = torch.empty(m.shape, dtype=torch.float16, device="cuda")
    gpu.cpy(m, m16)
    br = np.arange(2 * L) >= L
    want = np.where(br[None, :] != br[:, None], -np.inf, 0.0).astype(np.float16)
    assert np.array_equal(sync_np(m16), want)


@pytest.mark.parametrize("seed", list(range(48)))
def test_glue_random_shapes(gpu, seed):
    """Binary operators with ggml's broadcast rule, REPEAT, CONCAT along every dimension, a tree of CONCATs and copies
    between shapes, at random 4-d shapes with strided (sliced, permuted) operands: the results are fixed by IEEE arithmetic
    and by indexing alone, so numpy is the reference and the comparison is exact."""
    import torch
    r = rng("glue-random", seed)
    ne = [int(r.choice([1, 2, 3, 5])), int(r.choice([1, 2, 4, 7])), int(r.choice([1, 3, 14, 17])), int(r.choice([1, 4, 30, 64, 100, 257]))]   # torch order
    say(f"glue random seed={seed}: shape {ne}")
    a = r.standard_normal(ne).astype(np.float32)
    # src1 broadcast: every dim is 1 or the full extent
    nb_ = [n if r.integers(2) else 1 for n in ne]
    b = (r.standard_normal(nb_) + 3.0).astype(np.float32)
    A, Bt = dev(a), dev(b)
    for op, f in ((gpu.BIN_ADD, np.add), (gpu.BIN_SUB, np.subtract), (gpu.BIN_MUL, np.multiply), (gpu.BIN_DIV, np.divide)):
        got = sync_np(gpu.binary(op, A, Bt))
        assert np.array_equal(got, f(a, b).astype(np.float32)), ("binary", op)
    # a strided first operand: a slice of a wider tensor, and a permuted view
    wide = r.standard_normal(ne[:3] + [ne[3] + 5]).astype(np.float32)
    Wd = dev(wide)
    got = sync_np(gpu.binary(gpu.BIN_ADD, Wd[..., 2:2 + ne[3]], Bt))
    assert np.array_equal(got, wide[..., 2:2 + ne[3]] + b)
    perm = dev(np.ascontiguousarray(a.transpose(0, 2, 1, 3)))        # stored [n0, n2, n1, n3], viewed back as [n0, n1, n2, n3]
    out = torch.empty(ne, dtype=torch.float32, device="cuda")
    gpu.cpy(perm.permute(0, 2, 1, 3), out)
    assert np.array_equal(sync_np(out), a), "cpy of a permuted view"
    # REPEAT of the broadcast operand to the full shape
    assert np.array_equal(sync_np(gpu.repeat(Bt, tuple(ne))), np.broadcast_to(b, ne)), "repeat"
    # CONCAT along every ggml dimension (ggml dim d = torch dim 3 - d)
    for gd in range(4):
        td = 3 - gd
        other = list(ne); other[td] = int(r.choice([1, 2, 5]))
        c = r.standard_normal(other).astype(np.float32)
        assert np.array_equal(sync_np(gpu.concat(A, dev(c), gd)), np.concatenate([a, c], axis=td)), ("concat", gd)
    # a tree of CONCATs from its leaves, one leaf repeated, along ggml dim 1 and dim 0
    for gd in (1, 0):
        td = 3 - gd
        l1, l2 = list(ne), list(ne)
        l1[td], l2[td] = 3, 2
        small = [1 if i != 3 else ne[3] for i in range(4)] if gd == 1 else [1, 1, ne[2], 1]
        x1, x2, x3 = r.standard_normal(l1).astype(np.float32), r.standard_normal(l2).astype(np.float32), r.standard_normal(small).astype(np.float32)
        rep_shape = list(ne); rep_shape[td] = 4 if gd == 1 else 4 * small[3]
        want = np.concatenate([x1, np.broadcast_to(x3, rep_shape) if gd == 1 else np.tile(x3, [ne[0], ne[1], 1, 4]), x2], axis=td)
        out = torch.full(want.shape, float("nan"), dtype=torch.float32, device="cuda")
        gpu.concat_many([dev(x1), dev(x3), dev(x2)], [l1[td], rep_shape[td], l2[td]], gd, out)
        assert np.array_equal(sync_np(out), want), ("concat_many", gd)


def test_glue_get_rows(gpu):
    """GET_ROWS gathers exactly: F32 / I32 rows as bits, F16 widened, Q8_0 as quant * scale (one rounding,
    the oracle's dequantisation); batched tables and a strided index view as ggml's tests use them."""
    import torch
    say("glue: get_rows")
    n_vocab, nc = 517, 96
    idx = rng("gr", "idx").integers(0, n_vocab, size=(33,)).astype(np.int32)
    tab = rng("gr", "t").standard_normal((n_vocab, nc)).astype(np.float32)
    assert np.array_equal(sync_np(gpu.get_rows(dev(tab), dev(idx))), tab[idx])
    t16 = tab.astype(np.float16)
    assert np.array_equal(sync_np(gpu.get_rows(dev(t16), dev(idx))), t16[idx].astype(np.float32))
    ti = (tab * 1e8).astype(np.int32)
    got = sync_np(gpu.get_rows(dev(ti), dev(idx)))
    assert got.dtype == np.int32 and np.array_equal(got, ti[idx])
    raw = reflib.quantize_q8_0(tab)                               # (n_vocab, nc / 32 * 34) bytes
    blocks = raw.reshape(n_vocab, nc // 32, 34)
    d = blocks[:, :, :2].copy().view(np.float16).astype(np.float32)            # (n_vocab, nb, 1)
    q = blocks[:, :, 2:].view(np.int8).astype(np.float32)
    deq = (q * d).reshape(n_vocab, nc)
    got = sync_np(gpu.get_rows(dev(raw), dev(idx), ne0=nc))
    assert np.array_equal(got, deq[idx])
    # batched: table (2, 3, rows, nc), indices (2, 3, n): matrix (j, k) serves index column (j, k)
    tb = rng("gr", "tb").standard_normal((2, 3, 11, 40)).astype(np.float32)
    ib = rng("gr", "ib").integers(0, 11, size=(2, 3, 6)).astype(np.int32)
    want = np.take_along_axis(tb, ib[..., None].astype(np.int64), axis=2)
    assert np.array_equal(sync_np(gpu.get_rows(dev(tb), dev(ib))), want)
    # strided indices (every other entry) and a strided destination
    wide = torch.zeros((17, 2 * nc), dtype=torch.float32, device="cuda")
    gpu.get_rows(dev(tab), dev(idx)[::2], out=wide[:, :nc])
    assert np.array_equal(sync_np(wide)[:, :nc], tab[idx[::2]]) and not sync_np(wide)[:, nc:].any()
    # an index outside the table stays inside it (ggml-cpu aborts there)
    bad = np.array([-5, n_vocab + 3], np.int32)
    assert np.array_equal(sync_np(gpu.get_rows(dev(tab), dev(bad))), tab[[0, n_vocab - 1]])


def test_glue_rounding_unaries_and_integer_copies(gpu):
    """FLOOR / CEIL / ROUND / TRUNC / SQR / SQRT are single correctly rounded operations: bit-exact against
    numpy (ROUND rounds halves away from zero as roundf does); SIN / COS / LOG within 2 ulp-sized steps of
    the fp64 value (ggml-cpu calls libm's sinf / cosf / logf); I32 <-> F32 copies are C casts."""
    import torch
    say("glue: rounding unaries, sin / cos / log, integer copies")
    x = (rng("un", "x").standard_normal((3, 7, 130)) * 37).astype(np.float32)
    x[0, 0, :8] = [0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 0.0, -0.0]
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_FLOOR, dev(x))), np.floor(x))
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_CEIL, dev(x))), np.ceil(x))
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_TRUNC, dev(x))), np.trunc(x))
    away = (np.sign(x) * np.floor(np.abs(x.astype(np.float64)) + 0.5)).astype(np.float32)
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_ROUND, dev(x))), away)
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_SQR, dev(x))), x * x)
    assert np.array_equal(sync_np(gpu.unary(gpu.UNARY_SQRT, dev(np.abs(x)))), np.sqrt(np.abs(x)))
    x64 = x.astype(np.float64)
    for op, fn in ((gpu.UNARY_SIN, np.sin), (gpu.UNARY_COS, np.cos)):
        got = sync_np(gpu.unary(op, dev(x)))
        assert np.abs(got - fn(x64)).max() <= 2.5e-7
    xl = np.abs(x) + np.float32(1e-3)
    got = sync_np(gpu.unary(gpu.UNARY_LOG, dev(xl)))
    assert np.abs(got - np.log(xl.astype(np.float64))).max() <= 1e-6
    # the LocDiT timestep embedding's tail (src/locdit.cpp:198-212): sin / cos of t * exp(-k * i)
    i = gpu.arange(0.0, 128.0, 1.0)
    emb = gpu.scale(gpu.unary(gpu.UNARY_EXP, gpu.scale(i, -float(np.log(10000.0) / 127))), 1000.0 * 0.37)
    s = sync_np(gpu.unary(gpu.UNARY_SIN, emb))
    e64 = np.exp(np.arange(128) * -(np.log(10000.0) / 127)) * 370.0
    assert np.abs(s - np.sin(e64)).max() <= 5e-4                  # the argument (up to 370) carries its own fp32 roundings
    # integer copies
    ints = np.array([[0, 1, -1, 2**24 + 1, -(2**24) - 3, 2**31 - 1, -(2**31), 123456789]], np.int32)
    f = torch.empty(ints.shape, dtype=torch.float32, device="cuda")
    gpu.cpy(dev(ints), f)
    assert np.array_equal(sync_np(f), ints.astype(np.float32))
    ii = torch.empty(ints.shape, dtype=torch.int32, device="cuda")
    gpu.cpy(dev(ints), ii)
    assert np.array_equal(sync_np(ii), ints)                      # bits, not through float
    vals = np.array([[0.0, 0.9, -0.9, 7.5, -7.5, 16777217.0, -2.0e9, 1.9e9]], np.float32)
    gpu.cpy(dev(vals), ii)
    assert np.array_equal(sync_np(ii), vals.astype(np.int32))
    # transposing I32 -> F32 copy (strided source)
    grid = np.arange(35, dtype=np.int32).reshape(5, 7)
    ft = torch.empty((7, 5), dtype=torch.float32, device="cuda")
    gpu.cpy(dev(grid).t(), ft)
    assert np.array_equal(sync_np(ft), grid.T.astype(np.float32))
