"""GPU: every entry point that runs several adjacent graph nodes as one launch must give,
bit for bit, what the same nodes give when each is its own launch (the separate launches are
held to the CPU oracle and ggml-cpu in test_gpu_parity.py / test_gpu_ggml_backend.py).
Covered here: RMS_NORM+MUL, SCALE+ADD, ADD+SCALE, FLASH_ATTN_EXT+ADD1, MUL_MAT+MUL_MAT+SWIGLU,
MUL_MAT(+SCALE)+ADD, and the nine-node cache write with its ordering scalar.
"""
import sys

import numpy as np
import pytest

import reflib
from reflib import rng

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def q8_dev(w):
    return dev(reflib.quantize_q8_0(w)), w.shape[1]


def ok(pkg, rc, what):
    pkg.check(rc, what)


def same_bits(a, b):
    import torch
    return torch.equal(a.view(torch.int32), b.view(torch.int32))


@pytest.mark.parametrize("shape", [(2, 1024), (18, 1024), (3, 5, 4096), (7, 1025)])
def test_rms_norm_mul(pkg, gpu, shape):
    import torch
    say(f"fused rms_norm+mul {shape}")
    L, d = pkg.lib(), pkg.desc
    x = dev(rng("f-rms", shape).standard_normal(shape).astype(np.float32))
    w = dev((1 + 0.1 * rng("f-rms-w", shape).standard_normal(shape[-1])).astype(np.float32))
    a, b = torch.empty_like(x), torch.empty_like(x)
    ok(pkg, L.vx_rms_norm(d(x), d(a), 1e-5, None), "rms_norm")
    ok(pkg, L.vx_binary(pkg.BIN_MUL, d(a), d(w), d(a), None), "mul")
    ok(pkg, L.vx_rms_norm_mul(d(x), d(w), d(b), 1e-5, None), "rms_norm_mul")
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    # in place, as ggml-alloc may lay it out
    xc = x.clone()
    ok(pkg, L.vx_rms_norm_mul(d(xc), d(w), d(xc), 1e-5, None), "rms_norm_mul in place")
    torch.cuda.synchronize()
    assert torch.equal(a, xc)


@pytest.mark.parametrize("shape", [(2, 1024), (2, 3, 1030), (1, 1)])
def test_scale_add_and_add_scale(pkg, gpu, shape):
    import torch
    say(f"fused scale+add / add+scale {shape}")
    L, d = pkg.lib(), pkg.desc
    x = dev(rng("f-sa", shape).standard_normal(shape).astype(np.float32))
    y = dev(rng("f-sa-y", shape).standard_normal(shape).astype(np.float32))
    t, o1, o2 = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    for s in (0.2857738, 0.0, -3.0):
        ok(pkg, L.vx_scale(d(y), d(t), s, 0.0, None), "scale")
        ok(pkg, L.vx_binary(pkg.BIN_ADD, d(x), d(t), d(o1), None), "add")
        ok(pkg, L.vx_scale_add(d(x), d(y), d(o2), s, None), "scale_add")
        torch.cuda.synchronize()
        assert torch.equal(o1, o2)
        for bias in (0.0, 0.75):
            ok(pkg, L.vx_binary(pkg.BIN_ADD, d(x), d(y), d(t), None), "add")
            ok(pkg, L.vx_scale(d(t), d(o1), s, bias, None), "scale")
            ok(pkg, L.vx_add_scale(d(x), d(y), d(o2), s, bias, None), "add_scale")
            torch.cuda.synchronize()
            assert torch.equal(o1, o2)


@pytest.mark.parametrize("T,n_kv,kv_f16", [(1, 640, False), (1, 4096, True), (512, 512, True), (7, 300, False)])
def test_flash_attn_add1(pkg, gpu, T, n_kv, kv_f16):
    import torch
    say(f"fused flash_attn+add1 T={T} n_kv={n_kv} f16={kv_f16}")
    L, d = pkg.lib(), pkg.desc
    B, H, Hkv, D = 2, 16, 2, 64
    g = rng("f-fa", T, n_kv)
    q = dev(g.standard_normal((B, H, T, D)).astype(np.float32))
    kt = np.float16 if kv_f16 else np.float32
    k = dev(g.standard_normal((B, Hkv, n_kv, D)).astype(kt))
    v = dev(g.standard_normal((B, Hkv, n_kv, D)).astype(kt))
    mask = dev(reflib.causal_mask(T, n_kv, n_kv - T)) if T > 1 else None
    addend = dev(np.array([0.375], dtype=np.float32))
    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    ok(pkg, L.vx_flash_attn_ext(d(q), d(k), d(v), d(mask), None, d(a), 0.125, 0.0, 0.0, None), "fa")
    ok(pkg, L.vx_add1(d(a), d(addend), d(a), None), "add1")
    ok(pkg, L.vx_flash_attn_ext_add1(d(q), d(k), d(v), d(mask), None, addend.data_ptr(), d(b), 0.125, 0.0, 0.0, None), "fa_add1")
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("M,K,N,nb", [(4096, 1024, 1, 2), (4096, 1024, 2, 1), (1000, 512, 16, 1), (24, 4096, 3, 2), (1024, 1024, 40, 1), (512, 4096, 14, 2)])
@pytest.mark.parametrize("act", ["float", "q8"])
def test_mul_mat_swiglu(pkg, gpu, M, K, N, nb, act):
    import torch
    say(f"fused gate/up/swiglu M={M} K={K} N={N} batch={nb} act={act}")
    L, d = pkg.lib(), pkg.desc
    mode = pkg.ACT_Q8 if act == "q8" else pkg.ACT_FLOAT
    g = rng("f-swiglu", M, K, N)
    wg, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    wu, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    x = dev(g.standard_normal((nb, 1, N, K)).astype(np.float32))
    gate = torch.empty((nb, 1, N, M), dtype=torch.float32, device="cuda")
    up, a, b = torch.empty_like(gate), torch.empty_like(gate), torch.empty_like(gate)
    ok(pkg, L.vx_mul_mat(pkg.desc_q8(wg, K), d(x), d(gate), mode, None), "gate")
    ok(pkg, L.vx_mul_mat(pkg.desc_q8(wu, K), d(x), d(up), mode, None), "up")
    ok(pkg, L.vx_glu(pkg.GLU_SWIGLU, d(gate), d(up), d(a), 0, None), "glu")
    ok(pkg, L.vx_mul_mat_swiglu(pkg.desc_q8(wg, K), pkg.desc_q8(wu, K), d(x), d(b), mode, None), "mul_mat_swiglu")
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("M,K,N,nb", [(4096, 1024, 1024, 1), (4096, 1024, 112, 1), (1000, 1024, 500, 1), (520, 512, 600, 2), (2048, 4096, 128, 1),
                                      (2048, 4096, 576, 1)])
@pytest.mark.parametrize("wtype", ["q8", "f16"])
def test_mul_mat_swiglu_tiled(pkg, gpu, M, K, N, nb, wtype):
    """gate, up and the GLU at prefill sizes: the tiled kernel's work-groups hold a tile of gate rows and the same rows of up
    (mlp_forward, src/minicpm.cpp:724-731).  Whole and ragged tiles of both sizes, rows that are no multiple of 16, a batch;
    bit-equal to the two products and the GLU node.  Under VX_ACT_Q8 the shape is not announced and the call refuses it."""
    import torch
    say(f"tiled gate/up/swiglu M={M} K={K} N={N} batch={nb} weights={wtype}")
    L, d = pkg.lib(), pkg.desc
    g = rng("f-swiglu-t", M, K, N)
    wgf, wuf = (0.05 * g.standard_normal((M, K))).astype(np.float32), (0.05 * g.standard_normal((M, K))).astype(np.float32)
    if wtype == "q8":
        wg, _ = q8_dev(wgf); wu, _ = q8_dev(wuf)
        dg, du = pkg.desc_q8(wg, K), pkg.desc_q8(wu, K)
    else:
        wg, wu = dev(wgf.astype(np.float16)), dev(wuf.astype(np.float16))
        dg, du = d(wg), d(wu)
    x = dev(g.standard_normal((nb, 1, N, K)).astype(np.float32))
    gate = torch.empty((nb, 1, N, M), dtype=torch.float32, device="cuda")
    up, a, b = torch.empty_like(gate), torch.empty_like(gate), torch.full_like(gate, float("nan"))
    # one product on its own with 64..256 tiles of 64 x 64 and K of 2048 or more has its K cut (summed in another order than
    # the pair's whole K): such a pair is left to the separate launches
    tiles, big = -(-M // 64) * -(-N // 64) * nb, -(-M // 128) * -(-N // 128) * nb >= 192
    if not big and 64 <= tiles <= 256 and K >= 2048:
        assert L.vx_supports_mul_mat_swiglu_tiled(dg, du, d(x), d(b), pkg.ACT_FLOAT) == 0
        return
    assert L.vx_supports_mul_mat_swiglu_tiled(dg, du, d(x), d(b), pkg.ACT_FLOAT) == 1
    assert L.vx_supports_mul_mat_swiglu_tiled(dg, du, d(x), d(b), pkg.ACT_Q8) == 0
    ok(pkg, L.vx_mul_mat(dg, d(x), d(gate), pkg.ACT_FLOAT, None), "gate")
    ok(pkg, L.vx_mul_mat(du, d(x), d(up), pkg.ACT_FLOAT, None), "up")
    ok(pkg, L.vx_glu(pkg.GLU_SWIGLU, d(gate), d(up), d(a), 0, None), "glu")
    ok(pkg, L.vx_mul_mat_swiglu(dg, du, d(x), d(b), pkg.ACT_FLOAT, None), "mul_mat_swiglu")
    torch.cuda.synchronize()
    assert torch.equal(a, b)
    if not L.vx_supports_mul_mat_swiglu(dg, du, d(x), d(b)):
        assert L.vx_mul_mat_swiglu(dg, du, d(x), d(b), pkg.ACT_Q8, None) != 0


@pytest.mark.parametrize("M,K,N,nb", [(1024, 1024, 1, 2), (1024, 4096, 2, 1), (1000, 512, 16, 1), (20, 1024, 5, 3), (1024, 4096, 14, 1), (1024, 1024, 112, 1), (1024, 2048, 40, 2),
                                      # a long K over few tiles: the tiled kernels with K cut, the update in the kernel that adds the partials
                                      (1024, 4096, 112, 1), (1000, 4096, 70, 1),
                                      # prefill sizes: the update in the tiled kernels' epilogue (whole and ragged tiles of 64 and of 128),
                                      # or the plain product and a pass of its own (every shape under VX_ACT_Q8)
                                      (1024, 1024, 512, 1), (1024, 4096, 300, 1), (1000, 1024, 200, 2), (4096, 1024, 1024, 1),
                                      # 17 to 63 tokens behind a K the streaming kernel declines: one ragged token tile, K cut
                                      (1024, 4096, 17, 1), (1024, 4096, 40, 1), (1000, 2304, 63, 2)])
@pytest.mark.parametrize("act", ["float", "q8"])
def test_mul_mat_scale_add(pkg, gpu, M, K, N, nb, act):
    import torch
    say(f"fused mul_mat+scale+add M={M} K={K} N={N} batch={nb} act={act}")
    L, d = pkg.lib(), pkg.desc
    mode = pkg.ACT_Q8 if act == "q8" else pkg.ACT_FLOAT
    g = rng("f-mmsa", M, K, N)
    w, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    x = dev(g.standard_normal((nb, 1, N, K)).astype(np.float32))
    res_wide = dev(g.standard_normal((nb, 1, N, M + 8)).astype(np.float32))
    res = res_wide[..., :M]                      # a residual with its own row stride
    prod = torch.empty((nb, 1, N, M), dtype=torch.float32, device="cuda")
    a, b = torch.empty_like(prod), torch.empty_like(prod)
    for s in (0.2857738, 1.0):
        ok(pkg, L.vx_mul_mat(pkg.desc_q8(w, K), d(x), d(prod), mode, None), "mul_mat")
        ok(pkg, L.vx_scale(d(prod), d(prod), s, 0.0, None), "scale")
        ok(pkg, L.vx_binary(pkg.BIN_ADD, d(res), d(prod), d(a), None), "add")
        ok(pkg, L.vx_mul_mat_scale_add(pkg.desc_q8(w, K), d(x), d(res), d(b), s, mode, None), "mul_mat_scale_add")
        torch.cuda.synchronize()
        assert torch.equal(a, b)
    # in place on the residual, the layout ggml-alloc gives the reference's graph
    r2 = res.contiguous()
    ok(pkg, L.vx_mul_mat_scale_add(pkg.desc_q8(w, K), d(x), d(r2), d(r2), 1.0, mode, None), "mul_mat_scale_add in place")
    torch.cuda.synchronize()
    assert torch.equal(a, r2)
    # beyond the streaming kernel's token counts the destination has to be dense (the update may need a pass of its own)
    nbig = max(256 * 1024 // M + 17, 470)   # beyond tokens x rows <= 256 Ki, and beyond 448 tokens
    xl = dev(np.zeros((1, 1, nbig, K), dtype=np.float32))
    rl = torch.zeros((1, 1, nbig, M), dtype=torch.float32, device="cuda")
    dl = torch.zeros((1, 1, nbig, M + 8), dtype=torch.float32, device="cuda")[..., :M]
    assert L.vx_supports_mul_mat_scale_add(pkg.desc_q8(w, K), d(xl), d(rl), d(rl)) == (1 if M % 4 == 0 else 0)
    assert L.vx_supports_mul_mat_scale_add(pkg.desc_q8(w, K), d(xl), d(rl), d(dl)) == 0
    assert L.vx_mul_mat_scale_add(pkg.desc_q8(w, K), d(xl), d(rl), d(dl), 1.0, mode, None) != 0


@pytest.mark.parametrize("seed", list(range(120)))
def test_projection_groups_random_shapes(pkg, gpu, seed):  # (seed 29: one product alone is a streaming shape, the pair is not)
    """MUL_MAT + SCALE + ADD and MUL_MAT, MUL_MAT, GLU as one call each against their nodes at random row, column and token
    counts on both sides of every kernel choice (streaming, K cut, 64 x 64 and 128 x 128 tiles, the second pass), both
    activation modes.  Whatever the predicates announce must come out bit-equal; what they do not announce must be refused."""
    import torch
    L, d = pkg.lib(), pkg.desc
    r = rng("f-proj-random", seed)
    M = int(r.choice([16, 20, 64, 128, 200, 512, 1000, 1024, 2048]))
    K = 32 * int(r.choice([2, 8, 16, 32, 33, 64, 128]))
    N = int(r.choice([1, 2, 5, 14, 16, 17, 40, 63, 64, 65, 112, 128, 200, 300, 700]))
    nb = int(r.choice([1, 1, 2]))
    mode = pkg.ACT_Q8 if r.integers(2) else pkg.ACT_FLOAT
    say(f"projection groups random seed={seed}: M={M} K={K} N={N} batch={nb} act={'q8' if mode == pkg.ACT_Q8 else 'float'}")
    w, _ = q8_dev((0.05 * r.standard_normal((M, K))).astype(np.float32))
    w2, _ = q8_dev((0.05 * r.standard_normal((M, K))).astype(np.float32))
    x = dev(r.standard_normal((nb, 1, N, K)).astype(np.float32))
    res = dev(r.standard_normal((nb, 1, N, M)).astype(np.float32))
    prod = torch.empty((nb, 1, N, M), dtype=torch.float32, device="cuda")
    up, a, b = torch.empty_like(prod), torch.empty_like(prod), torch.full_like(prod, float("nan"))
    dw, dw2 = pkg.desc_q8(w, K), pkg.desc_q8(w2, K)
    # projection + scale + residual
    ok(pkg, L.vx_mul_mat(dw, d(x), d(prod), mode, None), "mul_mat")
    ok(pkg, L.vx_scale(d(prod), d(up), 0.2857738, 0.0, None), "scale")
    ok(pkg, L.vx_binary(pkg.BIN_ADD, d(res), d(up), d(a), None), "add")
    if L.vx_supports_mul_mat_scale_add(dw, d(x), d(res), d(b)):
        ok(pkg, L.vx_mul_mat_scale_add(dw, d(x), d(res), d(b), 0.2857738, mode, None), "mul_mat_scale_add")
        torch.cuda.synchronize()
        assert torch.equal(a, b), "projection + scale + residual"
        r2 = res.clone()
        ok(pkg, L.vx_mul_mat_scale_add(dw, d(x), d(r2), d(r2), 0.2857738, mode, None), "mul_mat_scale_add in place")
        torch.cuda.synchronize()
        assert torch.equal(a, r2), "in place on the residual"
    else:
        assert L.vx_mul_mat_scale_add(dw, d(x), d(res), d(b), 0.2857738, mode, None) != 0
    # gate, up, GLU
    ok(pkg, L.vx_mul_mat(dw2, d(x), d(up), mode, None), "up")
    ok(pkg, L.vx_glu(pkg.GLU_SWIGLU, d(prod), d(up), d(a), 0, None), "glu")
    b.fill_(float("nan"))
    if L.vx_supports_mul_mat_swiglu(dw, dw2, d(x), d(b)) or L.vx_supports_mul_mat_swiglu_tiled(dw, dw2, d(x), d(b), mode):
        ok(pkg, L.vx_mul_mat_swiglu(dw, dw2, d(x), d(b), mode, None), "mul_mat_swiglu")
        torch.cuda.synchronize()
        assert torch.equal(a, b), "gate, up, GLU"
    else:
        assert L.vx_mul_mat_swiglu(dw, dw2, d(x), d(b), mode, None) != 0


@pytest.mark.parametrize("B,T,Hkv,D,H", [(2, 1, 2, 64, 16), (1, 3, 2, 64, 16), (2, 4, 4, 128, 8), (3, 1, 1, 30, 2),
                                        # a short prompt's write: the sums in one work-group, the ADD1 over x a launch of its own
                                        (1, 48, 2, 64, 16), (1, 64, 2, 64, 16), (2, 20, 2, 64, 16), (1, 128, 2, 64, 16)])
@pytest.mark.parametrize("poison", [None, "nan", "inf"])
def test_kv_store_sync(pkg, gpu, B, T, Hkv, D, H, poison):
    import torch
    say(f"fused cache write + ordering scalar B={B} T={T} Hkv={Hkv} D={D} poison={poison}")
    L, d = pkg.lib(), pkg.desc
    g = rng("f-kvs", B, T, Hkv, D)
    max_len, n_past = 40 + T, 17
    k = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    if poison == "nan":
        k[0, 0, 0, 1] = float("nan")
    if poison == "inf":
        v[-1, -1, -1, -1] = float("inf")
    attn = dev(g.standard_normal((B, T, H, D)).astype(np.float32))
    caches = [torch.zeros((B, Hkv, max_len, D), dtype=torch.float32, device="cuda") for _ in range(4)]
    kc1, vc1, kc2, vc2 = caches

    def slot(c):  # the reference's write view [D, Hkv, T, B] of a cache [D, max_len, Hkv, B]
        return c[:, :, n_past:n_past + T].transpose(1, 2)

    for scale, bias in ((0.0, 0.0), (0.5, 0.0), (0.25, 1.5)):
        # separate nodes: CPY, CONT, SUM (twice), ADD, SCALE, ADD1
        cont = torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda")
        sk, sv, sync = (torch.empty(1, dtype=torch.float32, device="cuda") for _ in range(3))
        a = torch.empty_like(attn)
        for src, c, s in ((k, kc1, sk), (v, vc1, sv)):
            ok(pkg, L.vx_cpy(d(src), d(slot(c)), None), "cpy")
            ok(pkg, L.vx_cpy(d(slot(c)), d(cont), None), "cont")
            ok(pkg, L.vx_sum(d(cont), d(s), None), "sum")
        ok(pkg, L.vx_binary(pkg.BIN_ADD, d(sk), d(sv), d(sync), None), "add")
        ok(pkg, L.vx_scale(d(sync), d(sync), scale, bias, None), "scale")
        ok(pkg, L.vx_add1(d(attn), d(sync), d(a), None), "add1")
        # one launch
        b = torch.empty_like(attn)
        assert L.vx_supports_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(attn), d(b)) == 1
        ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(attn), d(b), scale, bias, None), "kv_store_sync")
        torch.cuda.synchronize()
        assert same_bits(kc1, kc2) and same_bits(vc1, vc2)
        assert torch.equal(torch.isnan(a), torch.isnan(b))
        assert torch.equal(a.nan_to_num(123.0), b.nan_to_num(123.0))
        if poison is None:
            assert torch.equal(kc2[:, :, n_past:n_past + T], k.transpose(1, 2))
        else:
            assert not bool(torch.isfinite(b).any())   # a NaN or infinity in the cache write poisons the output, as in the reference
    # in place on x, and a permuted source (ggml hands k over as a permuted view)
    kp = k.transpose(1, 2).contiguous().transpose(1, 2)
    x2 = attn.clone()
    ok(pkg, L.vx_kv_store_sync(d(kp), d(slot(kc2)), d(v), d(slot(vc2)), d(x2), d(x2), 0.25, 1.5, None), "kv_store_sync in place")
    torch.cuda.synchronize()
    assert torch.equal(b.nan_to_num(123.0), x2.nan_to_num(123.0)) and same_bits(kc1, kc2)


def test_kv_store_sync_limits(pkg, gpu):
    import torch
    say("fused cache write: one write whose sum is one block's beside one whose sum is spread over 128 blocks is refused")
    L, d = pkg.lib(), pkg.desc
    k = torch.zeros((2, 100, 2, 64), dtype=torch.float32, device="cuda")      # 25600 elements: 6400 units, one block's sum
    v = torch.zeros((2, 600, 2, 64), dtype=torch.float32, device="cuda")      # 153600 elements: 38400 units, 128 blocks
    c = torch.zeros((2, 2, 700, 64), dtype=torch.float32, device="cuda")
    x = torch.zeros((2, 100, 16, 64), dtype=torch.float32, device="cuda")
    s, s2 = c[:, :, :100].transpose(1, 2), c[:, :, :600].transpose(1, 2)
    assert L.vx_supports_kv_store_sync(d(k), d(s), d(k), d(s), d(x), d(x)) == 1
    assert L.vx_supports_kv_store_sync(d(k), d(s), d(v), d(s2), d(x), d(x)) == 0
    assert L.vx_kv_store_sync(d(k), d(s), d(v), d(s2), d(x), d(x), 0.0, 0.0, None) != 0


@pytest.mark.parametrize("B,T,Hkv,D,H", [(2, 512, 2, 64, 16), (16, 300, 2, 64, 16), (1, 1100, 1, 64, 4), (3, 600, 2, 30, 2),
                                        # a prompt's write: each sum one block's, its waves spread over work-groups
                                        (1, 129, 2, 64, 16), (1, 256, 2, 64, 16), (1, 512, 2, 64, 16), (2, 100, 2, 64, 16), (1, 300, 1, 64, 4)])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("poison", [None, "nan"])
def test_kv_store_sync_prefill_sized(pkg, gpu, B, T, Hkv, D, H, f16, poison):
    """The cache write of a prompt or a prefill (src/minicpm.cpp:682-690 with hundreds or thousands of tokens): CPY into
    the slot, CONT (the cast back from an F16 cache), SUM -- one block of 1024 threads up to 16 Ki units, beyond that the
    128-block form of the sum kernel and the kernel that adds its partials --, twice, ADD, SCALE, ADD1 over the attention
    output: eight to eleven launches against the two of vx_kv_store_sync, bit for bit, cache contents included.  Rows of
    64 and of 30 values (with and without 16-byte units)."""
    import torch
    say(f"prefill-sized cache write B={B} T={T} Hkv={Hkv} D={D} H={H} f16={f16} poison={poison}")
    if f16 and D % 4:
        pytest.skip("an F16 slot needs rows in whole 8-byte groups")
    L, d = pkg.lib(), pkg.desc
    g = rng("f-kvs-large", B, T, Hkv, D)
    n_past = 7
    k = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    if poison:
        v[B - 1, T // 2, 0, 3] = float("nan")
    attn = dev(g.standard_normal((B, T, H, D)).astype(np.float32))
    cdt = torch.float16 if f16 else torch.float32
    kc1, vc1, kc2, vc2 = (torch.zeros((B, Hkv, n_past + T + 5, D), dtype=cdt, device="cuda") for _ in range(4))
    slot = lambda c: c[:, :, n_past:n_past + T].transpose(1, 2)
    cont = torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda")
    sk, sv, sync = (torch.empty(1, dtype=torch.float32, device="cuda") for _ in range(3))
    a = torch.empty_like(attn)
    for src, c, s_ in ((k, kc1, sk), (v, vc1, sv)):
        ok(pkg, L.vx_cpy(d(src), d(slot(c)), None), "cpy")
        ok(pkg, L.vx_cpy(d(slot(c)), d(cont), None), "cont")
        ok(pkg, L.vx_sum(d(cont), d(s_), None), "sum")
    ok(pkg, L.vx_binary(pkg.BIN_ADD, d(sk), d(sv), d(sync), None), "add")
    ok(pkg, L.vx_scale(d(sync), d(sync), 0.25, 0.5, None), "scale")
    ok(pkg, L.vx_add1(d(attn), d(sync), d(a), None), "add1")
    b = torch.full_like(attn, 7.0)
    assert L.vx_supports_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(attn), d(b)) == 1
    ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(attn), d(b), 0.25, 0.5, None), "kv_store_sync")
    torch.cuda.synchronize()
    assert torch.equal(kc1.view(torch.uint8), kc2.view(torch.uint8)) and torch.equal(vc1.view(torch.uint8), vc2.view(torch.uint8))
    assert torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(a.nan_to_num(123.0), b.nan_to_num(123.0))
    if poison:
        assert not bool(torch.isfinite(b).any())
    # in place on the attention output
    x2 = attn.clone()
    ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(x2), d(x2), 0.25, 0.5, None), "in place")
    torch.cuda.synchronize()
    assert torch.equal(a.nan_to_num(123.0), x2.nan_to_num(123.0))


@pytest.mark.parametrize("B,T,Hkv,H", [(2, 512, 2, 16), (3, 600, 2, 16), (2, 1100, 1, 4), (16, 300, 2, 16), (1, 512, 2, 16), (2, 256, 2, 16)])
@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("poison", [None, "nan"])
def test_flash_attn_ext_store(pkg, gpu, B, T, Hkv, H, f16, poison):
    """The prefill attention block of attention_forward (src/minicpm.cpp:682-713) as one call: the cache write and its
    ordering scalar are launched first and the scalar joins the attention's epilogue.  Against vx_flash_attn_ext followed
    by vx_kv_store_sync, bit for bit, cache contents included; a NaN in the written values poisons the whole result,
    as it does through the reference's ADD1."""
    import torch
    say(f"prefill attention + cache write as one call B={B} T={T} Hkv={Hkv} H={H} f16 cache={f16} poison={poison}")
    L, d = pkg.lib(), pkg.desc
    D = 64
    g = rng("f-attn-store", B, T, Hkv, H)
    n_past = 5
    q = dev(g.standard_normal((B, T, H, D)).astype(np.float32))
    k = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    if poison:
        k[B - 1, T // 3, 0, 7] = float("nan")
    mask = torch.full((T, T), float("-inf"), dtype=torch.float16, device="cuda").triu(1).contiguous()
    qd, kd, vd = d(q.transpose(1, 2)), d(k.transpose(1, 2)), d(v.transpose(1, 2))
    cdt = torch.float16 if f16 else torch.float32
    kc1, vc1, kc2, vc2 = (torch.zeros((B, Hkv, n_past + T + 3, D), dtype=cdt, device="cuda") for _ in range(4))
    slot = lambda c: c[:, :, n_past:n_past + T].transpose(1, 2)
    scale = 1.0 / 8.0
    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    ok(pkg, L.vx_flash_attn_ext(qd, kd, vd, d(mask), None, d(a), scale, 0.0, 0.0, None), "flash_attn_ext")
    ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc1)), d(v), d(slot(vc1)), d(a), d(a), 0.25, 0.5, None), "kv_store_sync")
    b = torch.full_like(a, 7.0)
    assert L.vx_supports_flash_attn_ext_store(qd, kd, vd, d(mask), d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(b), 0.0) == 1
    ok(pkg, L.vx_flash_attn_ext_store(qd, kd, vd, d(mask), None, d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(b), scale, 0.0, 0.0,
                                      0.25, 0.5, None), "flash_attn_ext_store")
    torch.cuda.synchronize()
    assert torch.equal(kc1.view(torch.uint8), kc2.view(torch.uint8)) and torch.equal(vc1.view(torch.uint8), vc2.view(torch.uint8))
    assert torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(a.nan_to_num(123.0), b.nan_to_num(123.0))
    if poison:
        assert not bool(torch.isfinite(b).any())
    else:
        assert bool(torch.isfinite(b).all())
    # a second call on the same stream with another scalar: the workspace's front is written anew
    ok(pkg, L.vx_flash_attn_ext_store(qd, kd, vd, d(mask), None, d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(b), scale, 0.0, 0.0,
                                      0.0, 0.0, None), "flash_attn_ext_store again")
    ok(pkg, L.vx_flash_attn_ext(qd, kd, vd, d(mask), None, d(a), scale, 0.0, 0.0, None), "flash_attn_ext")
    ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc1)), d(v), d(slot(vc1)), d(a), d(a), 0.0, 0.0, None), "kv_store_sync")
    torch.cuda.synchronize()
    assert torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(a.nan_to_num(123.0), b.nan_to_num(123.0))


@pytest.mark.parametrize("B,T,flat", [(16, 2048, True), (8, 4100, True), (16, 2048, False), (5, 7000, True), (16, 1024, True), (2, 300, False)])
@pytest.mark.parametrize("f16", [False, True])
def test_flash_attn_ext_store_proj(pkg, gpu, B, T, flat, f16):
    """Prefill attention, cache write, o projection and residual update as one call: the attention's epilogue writes the
    projection's f16 activation tiles (the attention output is never stored).  Against vx_flash_attn_ext_store followed by
    vx_mul_mat_scale_add, bit for bit, cache contents included; the sequences flattened into one token dimension (ragged
    token tiles too) and as a batch."""
    import torch
    say(f"prefill attention + cache write + o projection as one call B={B} T={T} flat={flat} f16 cache={f16}")
    L, d = pkg.lib(), pkg.desc
    H, Hkv, D, hidden = 16, 2, 64, 1024
    g = rng("f-attn-store-proj", B, T)
    q = torch.randn((B, T, H, D), device="cuda", generator=torch.Generator(device="cuda").manual_seed(B * T))
    k = torch.randn((B, T, Hkv, D), device="cuda", generator=torch.Generator(device="cuda").manual_seed(B * T + 1))
    v = torch.randn((B, T, Hkv, D), device="cuda", generator=torch.Generator(device="cuda").manual_seed(B * T + 2))
    res = torch.randn((B, T, hidden), device="cuda", generator=torch.Generator(device="cuda").manual_seed(B * T + 3))
    w = q8_dev((0.05 * g.standard_normal((hidden, hidden))).astype(np.float32))[0]
    wd = pkg.desc_q8(w, hidden)
    mask = torch.full((T, T), float("-inf"), dtype=torch.float16, device="cuda").triu(1).contiguous()
    qd, kd, vd = d(q.transpose(1, 2)), d(k.transpose(1, 2)), d(v.transpose(1, 2))
    cdt = torch.float16 if f16 else torch.float32
    kc1, vc1, kc2, vc2 = (torch.zeros((B, Hkv, T + 3, D), dtype=cdt, device="cuda") for _ in range(4))
    slot = lambda c: c[:, :, 2:2 + T].transpose(1, 2)
    shape = (lambda t, rows: t.view(B * T, rows)) if flat else (lambda t, rows: t.view(B, T, rows))
    scale = 1.0 / 8.0
    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    o1 = torch.empty((B, T, hidden), dtype=torch.float32, device="cuda")
    ok(pkg, L.vx_flash_attn_ext_store(qd, kd, vd, d(mask), None, d(k), d(slot(kc1)), d(v), d(slot(vc1)), d(a), scale, 0.0, 0.0, 0.25, 0.5, None),
       "flash_attn_ext_store")
    ok(pkg, L.vx_mul_mat_scale_add(wd, d(shape(a, hidden)), d(shape(res, hidden)), d(shape(o1, hidden)), 0.7, pkg.ACT_FLOAT, None), "mul_mat_scale_add")
    b = torch.full_like(a, 7.0)
    o2 = torch.full_like(o1, float("nan"))
    args = (qd, kd, vd, d(mask))
    tail = (d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(shape(b, hidden)), wd, d(shape(res, hidden)), d(shape(o2, hidden)))
    one_pass = B * T >= 32768   # (from there on the projection alone is a product the pre-tiled kernel takes)
    assert L.vx_supports_flash_attn_ext_store_proj(*args, *tail, 0.0, pkg.ACT_FLOAT) == (1 if one_pass else 0)
    assert L.vx_supports_flash_attn_ext_store_proj(*args, *tail, 0.0, pkg.ACT_Q8) == 0
    ok(pkg, L.vx_flash_attn_ext_store_proj(*args, None, *tail, scale, 0.0, 0.0, 0.25, 0.5, 0.7, pkg.ACT_FLOAT, None), "flash_attn_ext_store_proj")
    torch.cuda.synchronize()
    assert torch.equal(kc1.view(torch.uint8), kc2.view(torch.uint8)) and torch.equal(vc1.view(torch.uint8), vc2.view(torch.uint8))
    assert bool(torch.isfinite(o2).all()) and torch.equal(o1, o2)
    if one_pass:
        assert bool((b == 7.0).all()), "the attention output is not stored"
    else:   # smaller shapes run as the calls the entry point stands for, through attn's memory
        assert torch.equal(a, b)
        assert L.vx_flash_attn_ext_store_proj(*args, None, *tail[:4], d(shape(o2, hidden)), *tail[5:], scale, 0.0, 0.0, 0.25, 0.5, 0.7, pkg.ACT_FLOAT, None) != 0, \
            "dst over attn's memory must be refused on this route"
    # in place on the residual, as layer_forward's update is laid out
    r2 = res.clone()
    ok(pkg, L.vx_flash_attn_ext_store_proj(*args, None, *tail[:6], d(shape(r2, hidden)), d(shape(r2, hidden)), scale, 0.0, 0.0, 0.25, 0.5, 0.7,
                                           pkg.ACT_FLOAT, None), "in place")
    torch.cuda.synchronize()
    assert torch.equal(o1, r2)


def test_flash_attn_ext_store_limits(pkg, gpu):
    import torch
    say("prefill attention + cache write: decode-sized and softcapped calls are refused")
    L, d = pkg.lib(), pkg.desc
    z = lambda *s: torch.zeros(s, dtype=torch.float32, device="cuda")
    q, k, c, o = z(2, 1, 16, 64), z(2, 1, 2, 64), z(2, 2, 64, 64), z(2, 1, 16, 64)
    s = c[:, :, :1].transpose(1, 2)
    assert L.vx_supports_flash_attn_ext_store(d(q.transpose(1, 2)), d(k.transpose(1, 2)), d(k.transpose(1, 2)), None, d(k), d(s), d(k), d(s), d(o), 0.0) == 0
    q, k, c, o = z(2, 512, 16, 64), z(2, 512, 2, 64), z(2, 2, 600, 64), z(2, 512, 16, 64)
    s = c[:, :, :512].transpose(1, 2)
    args = (d(q.transpose(1, 2)), d(k.transpose(1, 2)), d(k.transpose(1, 2)), None, d(k), d(s), d(k), d(s), d(o))
    assert L.vx_supports_flash_attn_ext_store(*args, 0.0) == 1
    assert L.vx_supports_flash_attn_ext_store(*args, 30.0) == 0
    # the call itself then runs the two calls it stands for
    ok(pkg, L.vx_flash_attn_ext_store(args[0], args[1], args[2], None, None, *args[4:], 0.125, 0.0, 30.0, 0.0, 0.0, None), "softcapped: two calls inside")
    torch.cuda.synchronize()
    assert bool((o == 0).all())   # (all-zero values)


@pytest.mark.parametrize("shape", [(8, 128), (1, 1), (3, 5, 7, 1000), (2, 4100), (16, 2, 64)])
def test_sum_rows_matches_ggml_cpu_arithmetic(gpu, shape):
    """GGML_OP_SUM_ROWS (ggml_compute_forward_sum_rows_f32, ops.cpp:1451-1482): a row's elements added in double and
    rounded once.  Checked against numpy's float64 row sums rounded to float32 (bit-equal whenever the double sum is
    exact, which it is for these magnitudes up to the order of the additions: at most one float32 ulp otherwise), on
    dense tensors and on a strided view."""
    say(f"sum_rows {shape}")
    x = rng("sumrows", shape).standard_normal(shape).astype(np.float32)
    import torch
    sync_np = lambda t: (torch.cuda.synchronize(), t.cpu().numpy())[1]
    got = sync_np(gpu.sum_rows(dev(x)))
    want = x.astype(np.float64).sum(axis=-1, keepdims=True).astype(np.float32)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= np.spacing(np.abs(want).max())
    if len(shape) >= 2 and shape[-2] > 1:   # rows of a view: every second row
        xv = dev(x)[..., ::2, :]
        got = sync_np(gpu.sum_rows(xv))
        want = x[..., ::2, :].astype(np.float64).sum(axis=-1, keepdims=True).astype(np.float32)
        assert np.abs(got - want).max() <= np.spacing(np.abs(want).max())


@pytest.mark.parametrize("shape", [(2, 512, 2, 64), (3, 70000), (1, 20000)])
def test_sum_large_matches_fp64(pkg, gpu, shape):
    import torch
    say(f"sum over {shape}: several blocks, fp64 partials")
    x = rng("f-sum", shape).standard_normal(shape).astype(np.float32)
    got = gpu.sum_all(dev(x))
    torch.cuda.synchronize()
    want = np.float32(x.astype(np.float64).sum())
    assert abs(float(got.cpu().numpy().reshape(-1)[0]) - float(want)) <= 2e-6 * max(1.0, abs(float(want)))


@pytest.mark.parametrize("T,n_past,kv_f16,D", [(1, 639, False, 64), (1, 4095, True, 64), (1, 100, True, 128), (2, 31, False, 64),
                                                (5, 1000, False, 128), (1, 1, True, 64), (40, 24, True, 64)])
def test_flash_attn_two_segments(pkg, gpu, T, n_past, kv_f16, D):
    import torch
    say(f"attention over cached + current keys T={T} n_past={n_past} f16={kv_f16} D={D}")
    L, d = pkg.lib(), pkg.desc
    B, H, Hkv = 2, 16, 2
    g = rng("f-kv2", T, n_past, D)
    kt = torch.float16 if kv_f16 else torch.float32
    q = dev(g.standard_normal((B, H, T, D)).astype(np.float32))
    cache_k = dev(g.standard_normal((B, Hkv, n_past + 7, D)).astype(np.float32)).to(kt)
    cache_v = dev(g.standard_normal((B, Hkv, n_past + 7, D)).astype(np.float32)).to(kt)
    kp, vp = cache_k[:, :, :n_past], cache_v[:, :, :n_past]          # views of a longer cache
    # the step's keys as the projection leaves them, [B, T, Hkv, D], seen through ggml_permute(0, 2, 1, 3)
    kc = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32)).to(kt).transpose(1, 2)
    vc = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32)).to(kt).transpose(1, 2)
    n_kv = n_past + T
    mask = dev(reflib.causal_mask(T, n_kv, n_past)) if T > 1 else None
    kall = torch.empty((B, Hkv, n_kv, D), dtype=kt, device="cuda")
    vall = torch.empty_like(kall)
    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    ok(pkg, L.vx_concat(d(kp), d(kc), d(kall), 1, None), "concat k")
    ok(pkg, L.vx_concat(d(vp), d(vc), d(vall), 1, None), "concat v")
    sc = 1.0 / np.sqrt(D)
    ok(pkg, L.vx_flash_attn_ext(d(q), d(kall), d(vall), d(mask), None, d(a), sc, 0.0, 0.0, None), "fa")
    assert L.vx_supports_flash_attn_ext_kv2(d(q), d(kp), d(kc), d(vp), d(vc), d(mask), d(b)) == 1
    ok(pkg, L.vx_flash_attn_ext_kv2(d(q), d(kp), d(kc), d(vp), d(vc), d(mask), None, d(b), sc, 0.0, 0.0, None), "fa_kv2")
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_flash_attn_two_segments_declines_prefill_shapes(pkg, gpu):
    import torch
    say("two-segment attention leaves prefill-sized f16 shapes to concat + the tiled kernel")
    L, d = pkg.lib(), pkg.desc
    B, H, Hkv, D, T, n_past = 2, 16, 2, 64, 512, 512
    q = torch.zeros((B, H, T, D), dtype=torch.float32, device="cuda")
    kp = torch.zeros((B, Hkv, n_past, D), dtype=torch.float16, device="cuda")
    kc = torch.zeros((B, Hkv, T, D), dtype=torch.float16, device="cuda")
    mask = dev(reflib.causal_mask(T, n_past + T, n_past))
    o = torch.zeros((B, T, H, D), dtype=torch.float32, device="cuda")
    assert L.vx_supports_flash_attn_ext_kv2(d(q), d(kp), d(kc), d(kp), d(kc), d(mask), d(o)) == 0
    assert L.vx_flash_attn_ext_kv2(d(q), d(kp), d(kc), d(kp), d(kc), d(mask), None, d(o), 0.125, 0.0, 0.0, None) != 0
    # an F32 cache with F16 current keys, and K / V segments of different kinds, are refused as well
    kc32 = kc[:, :, :1].float()
    q1 = q[:, :, :1].contiguous()
    o1 = torch.zeros((B, 1, H, D), dtype=torch.float32, device="cuda")
    assert L.vx_supports_flash_attn_ext_kv2(d(q1), d(kp.float()), d(kc[:, :, :1]), d(kp.float()), d(kc[:, :, :1]), None, d(o1)) == 0
    assert L.vx_supports_flash_attn_ext_kv2(d(q1), d(kp), d(kc32), d(kp), d(kc[:, :, :1]), None, d(o1)) == 0
    assert L.vx_supports_flash_attn_ext_kv2(d(q1), d(kp), d(kc32), d(kp), d(kc32), None, d(o1)) == 1   # F16 cache + the step's F32 keys


@pytest.mark.parametrize("T,n_past,B", [(1, 639, 2), (1, 4095, 2), (1, 8191, 16), (1, 1, 2), (1, 31, 2), (1, 32, 2), (1, 33, 1), (2, 62, 2),
                                        (5, 1000, 2), (40, 24, 2), (14, 300, 3)])
def test_flash_attn_two_segments_f16_cache_f32_step(pkg, gpu, T, n_past, B):
    """An F16 cache and the step's keys and values still in F32 (as the projections and the rotation left them): the
    kernel rounds them to f16 as it loads them, so the result must equal CPY(F32 -> F16) x2, CONCAT x2, FLASH_ATTN_EXT
    bit for bit."""
    import torch
    say(f"attention over an f16 cache + F32 current keys T={T} n_past={n_past} B={B}")
    L, d = pkg.lib(), pkg.desc
    H, Hkv, D = 16, 2, 64
    g = rng("f-kv2m", T, n_past, B)
    q = dev(g.standard_normal((B, H, T, D)).astype(np.float32))
    cache_k = dev(g.standard_normal((B, Hkv, n_past + 3, D)).astype(np.float16))
    cache_v = dev(g.standard_normal((B, Hkv, n_past + 3, D)).astype(np.float16))
    kp, vp = cache_k[:, :, :n_past], cache_v[:, :, :n_past]
    k32 = g.standard_normal((B, T, Hkv, D)).astype(np.float32)
    v32 = g.standard_normal((B, T, Hkv, D)).astype(np.float32)
    k32[0, 0, 0, :6] = [65504.0, 70000.0, 1e-8, 6.1e-5, -3.0e-8, 1.00048828125]   # f16 max, overflow, underflow, subnormals, a tie
    kc, vc = dev(k32).transpose(1, 2), dev(v32).transpose(1, 2)          # ggml_permute(0, 2, 1, 3) of [D, Hkv, T, B]
    n_kv = n_past + T
    mask = dev(reflib.causal_mask(T, n_kv, n_past)) if T > 1 else None
    k16 = torch.empty((B, Hkv, T, D), dtype=torch.float16, device="cuda")
    v16 = torch.empty_like(k16)
    kall = torch.empty((B, Hkv, n_kv, D), dtype=torch.float16, device="cuda")
    vall = torch.empty_like(kall)
    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    b = torch.full_like(a, 3.0)
    ok(pkg, L.vx_cpy(d(kc), d(k16), None), "cast k")
    ok(pkg, L.vx_cpy(d(vc), d(v16), None), "cast v")
    ok(pkg, L.vx_concat(d(kp), d(k16), d(kall), 1, None), "concat k")
    ok(pkg, L.vx_concat(d(vp), d(v16), d(vall), 1, None), "concat v")
    ok(pkg, L.vx_flash_attn_ext(d(q), d(kall), d(vall), d(mask), None, d(a), 0.125, 0.0, 0.0, None), "fa")
    assert L.vx_supports_flash_attn_ext_kv2(d(q), d(kp), d(kc), d(vp), d(vc), d(mask), d(b)) == 1
    ok(pkg, L.vx_flash_attn_ext_kv2(d(q), d(kp), d(kc), d(vp), d(vc), d(mask), None, d(b), 0.125, 0.0, 0.0, None), "fa_kv2 mixed")
    torch.cuda.synchronize()
    assert torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(a.nan_to_num(5.0), b.nan_to_num(5.0))


@pytest.mark.parametrize("T,n_past,B", [(1, 639, 2), (1, 300, 1), (1, 4100, 16), (3, 4000, 2), (1, 100, 2)])
@pytest.mark.parametrize("poison", [None, "nan"])
def test_f16_cache_write_with_ordering_scalar(pkg, gpu, T, n_past, B, poison):
    """The cache write of attention_forward into an F16 cache: CPY(k -> f16 slot), CPY(slot -> F32), SUM (twice), ADD,
    SCALE, ADD1 as separate nodes against vx_kv_store_sync, and -- with more than 256 keys -- against
    vx_flash_attn_ext_kv2_store, which also reads the F32 keys of the step in place."""
    import torch
    say(f"f16 cache write with the ordering scalar T={T} n_past={n_past} B={B} {poison}")
    L, d = pkg.lib(), pkg.desc
    H, Hkv, D = 16, 2, 64
    g = rng("f-kvs16", T, n_past, B)
    q = dev(g.standard_normal((B, H, T, D)).astype(np.float32))
    caches = [dev(g.standard_normal((B, Hkv, n_past + T + 5, D)).astype(np.float16)) for _ in range(2)]
    caches += [c.clone() for c in caches] + [c.clone() for c in caches]
    kc1, vc1, kc2, vc2, kc3, vc3 = caches
    k = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    if poison:
        v[0, 0, 0, 3] = float("nan")
    kcur, vcur = k.transpose(1, 2), v.transpose(1, 2)
    mask = dev(reflib.causal_mask(T, n_past + T, n_past)) if T > 1 else None

    def slot(c):
        return c[:, :, n_past:n_past + T].transpose(1, 2)

    for sync_scale, sync_bias in ((0.0, 0.0), (0.125, 0.5)):
        # node by node
        a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
        ok(pkg, L.vx_flash_attn_ext_kv2(d(q), d(kc1[:, :, :n_past]), d(kcur), d(vc1[:, :, :n_past]), d(vcur), d(mask), None, d(a), 0.125, 0.0, 0.0, None), "kv2")
        cont = torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda")
        sk, sv, sync = (torch.empty(1, dtype=torch.float32, device="cuda") for _ in range(3))
        a1 = torch.empty_like(a)
        for src, c, s_ in ((k, kc1, sk), (v, vc1, sv)):
            ok(pkg, L.vx_cpy(d(src), d(slot(c)), None), "cpy")
            ok(pkg, L.vx_cpy(d(slot(c)), d(cont), None), "cast back")
            ok(pkg, L.vx_sum(d(cont), d(s_), None), "sum")
        ok(pkg, L.vx_binary(pkg.BIN_ADD, d(sk), d(sv), d(sync), None), "add")
        ok(pkg, L.vx_scale(d(sync), d(sync), sync_scale, sync_bias, None), "scale")
        ok(pkg, L.vx_add1(d(a), d(sync), d(a1), None), "add1")
        # the write group as one launch
        b = torch.empty_like(a)
        assert L.vx_supports_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(a), d(b)) == 1
        ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(a), d(b), sync_scale, sync_bias, None), "kv_store_sync f16")
        torch.cuda.synchronize()
        assert same_bits(kc1, kc2) and same_bits(vc1, vc2)
        assert torch.equal(torch.isnan(a1), torch.isnan(b)) and torch.equal(a1.nan_to_num(7.0), b.nan_to_num(7.0))
        # attention + write as one call
        c_ = torch.empty_like(a)
        want = 1 if n_past + T > 256 else 0
        assert L.vx_supports_flash_attn_ext_kv2_store(d(q), d(kc3[:, :, :n_past]), d(kcur), d(vc3[:, :, :n_past]), d(vcur), d(mask),
                                                      d(k), d(slot(kc3)), d(v), d(slot(vc3)), d(c_)) == want
        if want:
            ok(pkg, L.vx_flash_attn_ext_kv2_store(d(q), d(kc3[:, :, :n_past]), d(kcur), d(vc3[:, :, :n_past]), d(vcur), d(mask), None,
                                                  d(k), d(slot(kc3)), d(v), d(slot(vc3)), d(c_), 0.125, 0.0, 0.0, sync_scale, sync_bias, None), "kv2_store f16")
            torch.cuda.synchronize()
            assert same_bits(kc1, kc3) and same_bits(vc1, vc3)
            assert torch.equal(torch.isnan(a1), torch.isnan(c_)) and torch.equal(a1.nan_to_num(7.0), c_.nan_to_num(7.0))
    if not poison:
        assert torch.equal(kc2[:, :, n_past:n_past + T], k.transpose(1, 2).to(torch.float16))


@pytest.mark.parametrize("seed", list(range(40)))
def test_decode_attention_groups_random_shapes(pkg, gpu, seed):
    """attention_forward's decode step (src/minicpm.cpp:682-713) at random shapes: cached keys + the step's keys read in
    place against CONCAT, CONCAT, FLASH_ATTN_EXT, and the cache write with its ordering scalar against its nodes, for F32
    and F16 caches, head sizes 64 and 128, past lengths on both sides of every tile and range boundary.  Bit for bit."""
    import torch
    L, d = pkg.lib(), pkg.desc
    r = rng("f-decode-random", seed)
    B, Hkv, gqa = int(r.choice([1, 2, 3, 16])), int(r.choice([1, 2, 4])), int(r.choice([1, 4, 8]))
    D, T = int(r.choice([64, 64, 128])), int(r.choice([1, 1, 1, 2, 3]))
    n_past = int(r.choice([1, 15, 16, 31, 32, 33, 63, 64, 65, 255, 256, 257, 300, 511, 640, 767, 1023, 1025, 2049, 4100]))
    f16 = bool(r.integers(2))
    H = Hkv * gqa
    say(f"decode groups random seed={seed}: B={B} heads={H}/{Hkv} D={D} T={T} n_past={n_past} cache={'f16' if f16 else 'f32'}")
    cdt = np.float16 if f16 else np.float32
    q = dev(r.standard_normal((B, H, T, D)).astype(np.float32))
    kc1, vc1 = (dev(r.standard_normal((B, Hkv, n_past + T + 3, D)).astype(cdt)) for _ in range(2))
    kc2, vc2 = kc1.clone(), vc1.clone()
    k = dev(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    v = dev(r.standard_normal((B, T, Hkv, D)).astype(np.float32))
    kcur, vcur = k.transpose(1, 2), v.transpose(1, 2)
    mask = dev(reflib.causal_mask(T, n_past + T, n_past)) if T > 1 else None
    scale = float(1.0 / np.sqrt(D))
    slot = lambda c: c[:, :, n_past:n_past + T].transpose(1, 2)
    # node by node: (cast,) CONCAT, CONCAT, attention; then the write and its scalar
    if f16:
        k16, v16 = torch.empty((B, Hkv, T, D), dtype=torch.float16, device="cuda"), torch.empty((B, Hkv, T, D), dtype=torch.float16, device="cuda")
        ok(pkg, L.vx_cpy(d(kcur), d(k16), None), "cast k"); ok(pkg, L.vx_cpy(d(vcur), d(v16), None), "cast v")
        kseg, vseg = k16, v16
    else:
        kseg, vseg = kcur, vcur
    kall = torch.empty((B, Hkv, n_past + T, D), dtype=kc1.dtype, device="cuda"); vall = torch.empty_like(kall)
    ok(pkg, L.vx_concat(d(kc1[:, :, :n_past]), d(kseg), d(kall), 1, None), "concat k")
    ok(pkg, L.vx_concat(d(vc1[:, :, :n_past]), d(vseg), d(vall), 1, None), "concat v")
    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    ok(pkg, L.vx_flash_attn_ext(d(q), d(kall), d(vall), d(mask), None, d(a), scale, 0.0, 0.0, None), "attention")
    cont = torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda")
    sk, sv, sync = (torch.empty(1, dtype=torch.float32, device="cuda") for _ in range(3))
    for src, c, s_ in ((k, kc1, sk), (v, vc1, sv)):
        ok(pkg, L.vx_cpy(d(src), d(slot(c)), None), "cpy")
        ok(pkg, L.vx_cpy(d(slot(c)), d(cont), None), "cont")
        ok(pkg, L.vx_sum(d(cont), d(s_), None), "sum")
    ok(pkg, L.vx_binary(pkg.BIN_ADD, d(sk), d(sv), d(sync), None), "add")
    ok(pkg, L.vx_scale(d(sync), d(sync), 0.25, 0.125, None), "scale")
    a1 = torch.empty_like(a)
    ok(pkg, L.vx_add1(d(a), d(sync), d(a1), None), "add1")
    # the groups
    args = (d(q), d(kc2[:, :, :n_past]), d(kcur), d(vc2[:, :, :n_past]), d(vcur), d(mask))
    if L.vx_supports_flash_attn_ext_kv2(*args, d(a)):
        b = torch.full_like(a, float("nan"))
        ok(pkg, L.vx_flash_attn_ext_kv2(*args, None, d(b), scale, 0.0, 0.0, None), "kv2")
        torch.cuda.synchronize()
        assert torch.equal(a, b), "two segments against CONCAT + attention"
    else:
        say("   (two-segment attention declines the shape)")
    if L.vx_supports_flash_attn_ext_kv2_store(*args, d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(a)):
        c_ = torch.full_like(a, float("nan"))
        ok(pkg, L.vx_flash_attn_ext_kv2_store(*args, None, d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(c_), scale, 0.0, 0.0, 0.25, 0.125, None), "kv2_store")
        torch.cuda.synchronize()
        assert torch.equal(a1, c_), "attention with the cache write against its nodes"
        assert same_bits(kc1, kc2) and same_bits(vc1, vc2)
    elif L.vx_supports_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(a), d(a)):
        c_ = torch.full_like(a, float("nan"))
        ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(a), d(c_), 0.25, 0.125, None), "kv_store_sync")
        torch.cuda.synchronize()
        assert torch.equal(a1, c_) and same_bits(kc1, kc2) and same_bits(vc1, vc2)


@pytest.mark.parametrize("T,B,H,Hkv,D,K", [(1, 2, 16, 2, 64, 1024), (1, 1, 16, 2, 64, 1024), (3, 2, 8, 8, 128, 512), (16, 1, 4, 1, 32, 256), (14, 8, 16, 2, 64, 1024), (21, 1, 16, 2, 64, 1024)])
@pytest.mark.parametrize("act", ["float", "q8"])
@pytest.mark.parametrize("yarn", [False, True])
def test_qkv_proj_rope(pkg, gpu, T, B, H, Hkv, D, K, act, yarn):
    import torch
    say(f"fused q/k/v projections + rope T={T} B={B} H={H}/{Hkv} D={D} K={K} act={act} yarn={yarn}")
    L, d = pkg.lib(), pkg.desc
    mode = pkg.ACT_Q8 if act == "q8" else pkg.ACT_FLOAT
    g = rng("f-qkv", T, B, H, D, K)
    wq, _ = q8_dev((0.05 * g.standard_normal((H * D, K))).astype(np.float32))
    wk, _ = q8_dev((0.05 * g.standard_normal((Hkv * D, K))).astype(np.float32))
    wv, _ = q8_dev((0.05 * g.standard_normal((Hkv * D, K))).astype(np.float32))
    x = dev(g.standard_normal((B, 1, T, K)).astype(np.float32))
    pos = torch.arange(700, 700 + T, dtype=torch.int32, device="cuda")
    ff = dev((1.0 + g.random(D // 2)).astype(np.float32))
    rope_args = (D, 2, 4096, 10000.0, 1.0, 0.0, 1.1, 32.0, 1.0) if not yarn else (D, 2, 512, 10000.0, 0.5, 1.0, 1.0, 32.0, 1.0)

    def outs():
        return (torch.empty((B, T, H, D), dtype=torch.float32, device="cuda"),
                torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda"),
                torch.empty((B, 1, T, Hkv * D), dtype=torch.float32, device="cuda"))

    q1, k1, v1 = outs()
    for w, o, M in ((wq, q1, H * D), (wk, k1, Hkv * D), (wv, v1, Hkv * D)):
        ok(pkg, L.vx_mul_mat(pkg.desc_q8(w, K), d(x), d(o.view(B, 1, T, M)), mode, None), "mul_mat")
    for o in (q1, k1):
        ok(pkg, L.vx_rope(d(o), pos.data_ptr(), ff.data_ptr(), d(o), *rope_args, None), "rope")
    q2, k2, v2 = outs()
    assert L.vx_supports_qkv_proj_rope(pkg.desc_q8(wq, K), pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), d(q2), d(k2), d(v2), D, 2) == 1
    ok(pkg, L.vx_qkv_proj_rope(pkg.desc_q8(wq, K), pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), pos.data_ptr(), ff.data_ptr(),
                               d(q2), d(k2), d(v2), *rope_args, mode, None), "qkv_proj_rope")
    torch.cuda.synchronize()
    assert torch.equal(v1, v2)
    assert torch.equal(k1, k2)
    assert torch.equal(q1, q2)
    # the same with every sequence's tokens flattened into one token dimension, as a 2-D activation tensor (all the
    # sequences' tokens are then one call's tokens: beyond the streaming kernel's work bound the flattened form is declined)
    q3, k3, v3 = outs()
    xf, vf = x.view(B * T, K), v3.view(B * T, Hkv * D)
    if L.vx_supports_qkv_proj_rope(pkg.desc_q8(wq, K), pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(xf), d(q3), d(k3), d(vf), D, 2):
        ok(pkg, L.vx_qkv_proj_rope(pkg.desc_q8(wq, K), pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(xf), pos.data_ptr(), ff.data_ptr(),
                                   d(q3), d(k3), d(vf), *rope_args, mode, None), "qkv_proj_rope flattened")
        torch.cuda.synchronize()
        assert torch.equal(q1, q3) and torch.equal(k1, k3) and torch.equal(v1, v3)
    # NORMAL-mode rotation and partial rotation are left to the separate operators
    assert L.vx_supports_qkv_proj_rope(pkg.desc_q8(wq, K), pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), d(q2), d(k2), d(v2), D, 0) == 0
    assert L.vx_supports_qkv_proj_rope(pkg.desc_q8(wq, K), pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), d(q2), d(k2), d(v2), D // 2, 2) == 0


@pytest.mark.parametrize("T,B,Hkv,D,K,flat", [(205, 1, 2, 64, 1024, False), (256, 1, 2, 64, 1024, True), (512, 2, 2, 64, 1024, True), (1024, 1, 2, 64, 1024, False),
                                              (700, 1, 2, 64, 1024, True), (300, 3, 2, 64, 1024, False), (333, 1, 1, 128, 512, True), (40, 2, 4, 64, 2048, False)])
@pytest.mark.parametrize("act", ["float", "q8"])
@pytest.mark.parametrize("yarn", [False, True])
def test_kv_proj_rope(pkg, gpu, T, B, Hkv, D, K, flat, act, yarn):
    """The k and v projections with k's rotation as one launch of the streaming kernel, at token counts beyond the
    three-matrix launch's (q's product is on a tiled kernel there): against two MUL_MATs and a ROPE, bit for bit, the
    sequences as a batch or flattened into one token dimension."""
    import torch
    say(f"k/v projections + rope as one launch T={T} B={B} Hkv={Hkv} D={D} K={K} flat={flat} act={act} yarn={yarn}")
    L, d = pkg.lib(), pkg.desc
    mode = pkg.ACT_Q8 if act == "q8" else pkg.ACT_FLOAT
    g = rng("f-kv", T, B, Hkv, D, K)
    wk, _ = q8_dev((0.05 * g.standard_normal((Hkv * D, K))).astype(np.float32))
    wv, _ = q8_dev((0.05 * g.standard_normal((Hkv * D, K))).astype(np.float32))
    x = dev(g.standard_normal((B * T, K) if flat else (B, 1, T, K)).astype(np.float32))
    pos = torch.arange(90, 90 + T, dtype=torch.int32, device="cuda")
    ff = dev((1.0 + g.random(D // 2)).astype(np.float32))
    rope_args = (D, 2, 4096, 10000.0, 1.0, 0.0, 1.1, 32.0, 1.0) if not yarn else (D, 2, 512, 10000.0, 0.5, 1.0, 1.0, 32.0, 1.0)
    shape = (lambda t: t.view(B * T, Hkv * D)) if flat else (lambda t: t.view(B, 1, T, Hkv * D))
    k1 = torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda")
    v1 = torch.empty((B, T, Hkv * D), dtype=torch.float32, device="cuda")
    ok(pkg, L.vx_mul_mat(pkg.desc_q8(wk, K), d(x), d(shape(k1)), mode, None), "k")
    ok(pkg, L.vx_mul_mat(pkg.desc_q8(wv, K), d(x), d(shape(v1)), mode, None), "v")
    ok(pkg, L.vx_rope(d(k1), pos.data_ptr(), ff.data_ptr(), d(k1), *rope_args, None), "rope")
    k2, v2 = torch.full_like(k1, float("nan")), torch.full_like(v1, float("nan"))
    if not L.vx_supports_kv_proj_rope(pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), d(k2), d(shape(v2)), D, 2):
        assert flat and B * T * 2 * Hkv * D > 256 * 1024   # (beyond the streaming kernel's work bound)
        assert L.vx_kv_proj_rope(pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), pos.data_ptr(), ff.data_ptr(), d(k2), d(shape(v2)), *rope_args, mode, None) != 0
        return
    ok(pkg, L.vx_kv_proj_rope(pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), pos.data_ptr(), ff.data_ptr(), d(k2), d(shape(v2)), *rope_args, mode, None),
       "kv_proj_rope")
    torch.cuda.synchronize()
    assert torch.equal(v1, v2) and torch.equal(k1, k2)
    assert L.vx_supports_kv_proj_rope(pkg.desc_q8(wk, K), pkg.desc_q8(wv, K), d(x), d(k2), d(shape(v2)), D, 0) == 0


@pytest.mark.parametrize("seed", list(range(40)))
def test_qkv_and_mlp_groups_random_shapes(pkg, gpu, seed):
    """The q/k/v + rope group, with and without the norm in front, and the norm + gate/up + SwiGLU group at random token
    counts, batches, head counts, head sizes and K (several chunks of 16 tokens, K with and without whole rounds, one to
    eight KV heads): whatever the predicates announce is run through the parametrised tests' own bodies, bit for bit."""
    import torch
    L, d = pkg.lib(), pkg.desc
    r = rng("f-qkv-random", seed)
    T, B = int(r.choice([1, 2, 3, 5, 14, 16, 17, 21, 40])), int(r.choice([1, 2, 8]))
    Hkv, gqa, D = int(r.choice([1, 2, 4, 8])), int(r.choice([1, 4, 8])), int(r.choice([32, 64, 128]))
    K = int(r.choice([256, 512, 768, 1024, 2048]))
    act, yarn = ("q8" if r.integers(2) else "float"), bool(r.integers(2))
    H = Hkv * gqa
    z = lambda rows: pkg.desc_q8(torch.zeros((rows, K // 32 * 34), dtype=torch.uint8, device="cuda"), K)
    x = torch.empty((B, 1, T, K), dtype=torch.float32, device="cuda")
    q, k, v = (torch.empty((B, T, H, D), dtype=torch.float32, device="cuda"), torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda"),
               torch.empty((B, 1, T, Hkv * D), dtype=torch.float32, device="cuda"))
    ran = []
    if L.vx_supports_qkv_proj_rope(z(H * D), z(Hkv * D), z(Hkv * D), d(x), d(q), d(k), d(v), D, 2):
        test_qkv_proj_rope(pkg, gpu, T, B, H, Hkv, D, K, act, yarn)
        ran.append("qkv")
        nw = torch.empty((K,), dtype=torch.float32, device="cuda")
        xf, vf = x.view(B * T, K), v.view(B * T, Hkv * D)   # (that test hands over the flattened form)
        if L.vx_supports_norm_qkv_proj_rope(d(xf), d(nw), z(H * D), z(Hkv * D), z(Hkv * D), d(q), d(k), d(vf), D, 2):
            test_norm_qkv_proj_rope(pkg, gpu, T, B, H, Hkv, D, K, act)
            ran.append("norm + qkv")
    M = int(r.choice([64, 1000, 2048, 4096]))
    nw = torch.empty((K,), dtype=torch.float32, device="cuda")
    act_out = torch.empty((B, 1, T, M), dtype=torch.float32, device="cuda")
    if L.vx_supports_norm_mul_mat_swiglu(d(x), d(nw), z(M), z(M), d(act_out)):
        test_norm_mul_mat_swiglu(pkg, gpu, T, B, K, M, act)
        ran.append("norm + gate/up")
    say(f"qkv / mlp groups random seed={seed}: T={T} B={B} heads={H}/{Hkv} D={D} K={K} M={M} act={act} yarn={yarn}: ran {ran}")


@pytest.mark.parametrize("T,B,K,M", [(1, 2, 1024, 4096), (2, 1, 1024, 4096), (16, 1, 512, 1000), (3, 2, 256, 64), (14, 1, 1024, 4096), (40, 1, 1024, 2048)])
@pytest.mark.parametrize("act", ["float", "q8"])
def test_norm_mul_mat_swiglu(pkg, gpu, T, B, K, M, act):
    import torch
    say(f"fused rms_norm+mul in front of gate/up/swiglu T={T} B={B} K={K} M={M} act={act}")
    L, d = pkg.lib(), pkg.desc
    mode = pkg.ACT_Q8 if act == "q8" else pkg.ACT_FLOAT
    g = rng("f-nswiglu", T, B, K, M)
    wg, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    wu, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    x = dev((3.0 * g.standard_normal((B, 1, T, K))).astype(np.float32))
    nw = dev((1 + 0.1 * g.standard_normal(K)).astype(np.float32))
    normed = torch.empty_like(x)
    a = torch.empty((B, 1, T, M), dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    ok(pkg, L.vx_rms_norm_mul(d(x), d(nw), d(normed), 1e-5, None), "rms_norm_mul")
    ok(pkg, L.vx_mul_mat_swiglu(pkg.desc_q8(wg, K), pkg.desc_q8(wu, K), d(normed), d(a), mode, None), "mul_mat_swiglu")
    assert L.vx_supports_norm_mul_mat_swiglu(d(x), d(nw), pkg.desc_q8(wg, K), pkg.desc_q8(wu, K), d(b)) == 1
    ok(pkg, L.vx_norm_mul_mat_swiglu(d(x), d(nw), 1e-5, pkg.desc_q8(wg, K), pkg.desc_q8(wu, K), d(b), mode, None), "norm_mul_mat_swiglu")
    torch.cuda.synchronize()
    assert torch.equal(a, b)


@pytest.mark.parametrize("T,B,K,M", [(2048, 1, 1024, 4096), (1100, 2, 1024, 2048), (1024, 1, 768, 1024), (1030, 1, 256, 1040)])
def test_norm_mul_mat_swiglu_at_prefill_sizes(pkg, gpu, T, B, K, M, monkeypatch):
    """RMS_NORM, MUL, gate, up, SwiGLU at prefill sizes: the norm and its weight applied by the pass that lays the
    activations out in tiles for the pre-tiled Q8_0 kernel (one trip over x, the normalised tensor never stored), against
    RMS_NORM+MUL followed by the tiled pair: the same bits -- whole and ragged token tiles, rows shorter than 1024, a batch."""
    import torch
    say(f"fused rms_norm+mul in front of the pre-tiled gate/up/swiglu T={T} B={B} K={K} M={M}")
    L, d = pkg.lib(), pkg.desc
    monkeypatch.setenv("VX_GEMM_Q8T", "2")   # (also where the launcher would find too few tiles for the pre-tiled kernel)
    g = rng("f-nswiglu-t", T, B, K, M)
    wg, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    wu, _ = q8_dev((0.05 * g.standard_normal((M, K))).astype(np.float32))
    x = dev((3.0 * g.standard_normal((B, T, K) if B > 1 else (T, K))).astype(np.float32))
    nw = dev((1 + 0.1 * g.standard_normal(K)).astype(np.float32))
    normed = torch.empty_like(x)
    a = torch.empty(tuple(x.shape[:-1]) + (M,), dtype=torch.float32, device="cuda")
    b = torch.full_like(a, float("nan"))
    dg, du = pkg.desc_q8(wg, K), pkg.desc_q8(wu, K)
    assert L.vx_supports_norm_mul_mat_swiglu(d(x), d(nw), dg, du, d(b)) == 0
    assert L.vx_supports_norm_mul_mat_swiglu_tiled(d(x), d(nw), dg, du, d(b), pkg.ACT_FLOAT) == 1
    assert L.vx_supports_norm_mul_mat_swiglu_tiled(d(x), d(nw), dg, du, d(b), pkg.ACT_Q8) == 0
    ok(pkg, L.vx_rms_norm_mul(d(x), d(nw), d(normed), 1e-5, None), "rms_norm_mul")
    ok(pkg, L.vx_mul_mat_swiglu(dg, du, d(normed), d(a), pkg.ACT_FLOAT, None), "mul_mat_swiglu")
    ok(pkg, L.vx_norm_mul_mat_swiglu(d(x), d(nw), 1e-5, dg, du, d(b), pkg.ACT_FLOAT, None), "norm_mul_mat_swiglu")
    torch.cuda.synchronize()
    assert torch.equal(a, b), float((a - b).abs().max())
    monkeypatch.setenv("VX_GEMM_Q8T", "0")   # without the pre-tiled kernel there is no fused form: said so, not answered otherwise
    assert L.vx_supports_norm_mul_mat_swiglu_tiled(d(x), d(nw), dg, du, d(b), pkg.ACT_FLOAT) == 0
    assert L.vx_norm_mul_mat_swiglu(d(x), d(nw), 1e-5, dg, du, d(b), pkg.ACT_FLOAT, None) != 0


@pytest.mark.parametrize("T,B,K,F", [(2048, 1, 1024, 4096), (1100, 2, 1024, 2048), (1024, 1, 1024, 1280), (1030, 3, 1024, 1088)])
@pytest.mark.parametrize("folded", [False, True])
def test_mlp_tiled(pkg, gpu, T, B, K, F, folded, monkeypatch):
    """mlp_forward and its residual update at prefill sizes as one call (RMS_NORM, MUL, gate, up, SwiGLU, down, SCALE, ADD):
    the pair's results reach the down projection as f16 tiles, the tokens x ffn tensor between them is never stored.  Against
    the three separate calls: the same bits -- whole and ragged token tiles, a batch, an ffn that is not a multiple of the
    row tile, the residual in place, the scale folded into the weights or not."""
    import torch
    say(f"fused mlp at prefill sizes T={T} B={B} K={K} ffn={F} folded={folded}")
    L, d = pkg.lib(), pkg.desc
    monkeypatch.setenv("VX_GEMM_Q8T", "2")
    if folded:
        monkeypatch.setenv("VX_GEMM_LDS", "2")
    else:
        monkeypatch.delenv("VX_GEMM_LDS", raising=False)
    g = rng("f-mlp-t", T, B, K, F)
    wg, _ = q8_dev((0.05 * g.standard_normal((F, K))).astype(np.float32))
    wu, _ = q8_dev((0.05 * g.standard_normal((F, K))).astype(np.float32))
    wd, _ = q8_dev((0.05 * g.standard_normal((K, F))).astype(np.float32))
    x = dev((3.0 * g.standard_normal((B, T, K) if B > 1 else (T, K))).astype(np.float32))
    nw = dev((1 + 0.1 * g.standard_normal(K)).astype(np.float32))
    normed, act = torch.empty_like(x), torch.empty(tuple(x.shape[:-1]) + (F,), dtype=torch.float32, device="cuda")
    a, b = torch.empty_like(x), torch.full_like(x, float("nan"))
    dg, du, dd = pkg.desc_q8(wg, K), pkg.desc_q8(wu, K), pkg.desc_q8(wd, F)
    scale = 0.2857738
    assert L.vx_supports_mlp_tiled(d(x), d(nw), dg, du, dd, d(x), d(b), pkg.ACT_FLOAT) == 1
    assert L.vx_supports_mlp_tiled(d(x), d(nw), dg, du, dd, d(x), d(b), pkg.ACT_Q8) == 0
    ok(pkg, L.vx_rms_norm_mul(d(x), d(nw), d(normed), 1e-5, None), "rms_norm_mul")
    ok(pkg, L.vx_mul_mat_swiglu(dg, du, d(normed), d(act), pkg.ACT_FLOAT, None), "mul_mat_swiglu")
    ok(pkg, L.vx_mul_mat_scale_add(dd, d(act), d(x), d(a), scale, pkg.ACT_FLOAT, None), "mul_mat_scale_add")
    ok(pkg, L.vx_mlp_tiled(d(x), d(nw), 1e-5, dg, du, dd, d(x), scale, d(b), pkg.ACT_FLOAT, None), "mlp_tiled")
    torch.cuda.synchronize()
    assert torch.equal(a, b), float((a - b).abs().max())
    x2 = x.clone()   # the update in place, as the graph's residual stream has it
    ok(pkg, L.vx_mlp_tiled(d(x2), d(nw), 1e-5, dg, du, dd, d(x2), scale, d(x2), pkg.ACT_FLOAT, None), "mlp_tiled in place")
    torch.cuda.synchronize()
    assert torch.equal(a, x2)
    monkeypatch.setenv("VX_GEMM_Q8T", "0")
    assert L.vx_supports_mlp_tiled(d(x), d(nw), dg, du, dd, d(x), d(b), pkg.ACT_FLOAT) == 0
    assert L.vx_mlp_tiled(d(x), d(nw), 1e-5, dg, du, dd, d(x), scale, d(b), pkg.ACT_FLOAT, None) != 0


def test_norm_prologue_limits(pkg, gpu):
    import torch
    say("norm prologue: rows beyond 1024 floats stay with the separate RMS_NORM")
    L, d = pkg.lib(), pkg.desc
    K, M = 2048, 64
    w, _ = q8_dev(np.zeros((M, K), dtype=np.float32))
    x = torch.zeros((1, 1, 1, K), dtype=torch.float32, device="cuda")
    nw = torch.ones(K, dtype=torch.float32, device="cuda")
    o = torch.zeros((1, 1, 1, M), dtype=torch.float32, device="cuda")
    assert L.vx_supports_norm_mul_mat_swiglu(d(x), d(nw), pkg.desc_q8(w, K), pkg.desc_q8(w, K), d(o)) == 0
    assert L.vx_norm_mul_mat_swiglu(d(x), d(nw), 1e-5, pkg.desc_q8(w, K), pkg.desc_q8(w, K), d(o), pkg.ACT_FLOAT, None) != 0


@pytest.mark.parametrize("T,B,H,Hkv,D,K", [(1, 2, 16, 2, 64, 1024), (4, 2, 8, 2, 64, 512), (1, 1, 4, 4, 128, 1024), (14, 8, 16, 2, 64, 1024)])
@pytest.mark.parametrize("act", ["float", "q8"])
def test_norm_qkv_proj_rope(pkg, gpu, T, B, H, Hkv, D, K, act):
    import torch
    say(f"fused rms_norm+mul in front of q/k/v projections + rope T={T} B={B} H={H}/{Hkv} D={D} K={K} act={act}")
    L, d = pkg.lib(), pkg.desc
    mode = pkg.ACT_Q8 if act == "q8" else pkg.ACT_FLOAT
    g = rng("f-nqkv", T, B, H, D, K)
    ws = [q8_dev((0.05 * g.standard_normal((n * D, K))).astype(np.float32))[0] for n in (H, Hkv, Hkv)]
    wd = [pkg.desc_q8(w, K) for w in ws]
    x = dev((2.0 * g.standard_normal((B * T, K))).astype(np.float32))
    nw = dev((1 + 0.1 * g.standard_normal(K)).astype(np.float32))
    pos = torch.arange(300, 300 + T, dtype=torch.int32, device="cuda")
    ff = dev((1.0 + g.random(D // 2)).astype(np.float32))
    rope_args = (D, 2, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0)

    def outs():
        return (torch.empty((B, T, H, D), dtype=torch.float32, device="cuda"),
                torch.empty((B, T, Hkv, D), dtype=torch.float32, device="cuda"),
                torch.empty((B * T, Hkv * D), dtype=torch.float32, device="cuda"))

    q1, k1, v1 = outs()
    normed = torch.empty_like(x)
    ok(pkg, L.vx_rms_norm_mul(d(x), d(nw), d(normed), 1e-5, None), "rms_norm_mul")
    ok(pkg, L.vx_qkv_proj_rope(*wd, d(normed), pos.data_ptr(), ff.data_ptr(), d(q1), d(k1), d(v1), *rope_args, mode, None), "qkv_proj_rope")
    q2, k2, v2 = outs()
    assert L.vx_supports_norm_qkv_proj_rope(d(x), d(nw), *wd, d(q2), d(k2), d(v2), D, 2) == 1
    ok(pkg, L.vx_norm_qkv_proj_rope(d(x), d(nw), 1e-5, *wd, pos.data_ptr(), ff.data_ptr(), d(q2), d(k2), d(v2), *rope_args, mode, None),
       "norm_qkv_proj_rope")
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2)


@pytest.mark.parametrize("T,B,H,Hkv,D,K,batched", [(2304, 1, 16, 2, 64, 1024, False), (1100, 2, 16, 2, 64, 1024, False), (2100, 2, 16, 2, 64, 1024, True),
                                                    (1030, 1, 8, 4, 128, 768, False)])
@pytest.mark.parametrize("yarn", [False, True])
def test_norm_qkv_proj_rope_at_prefill_sizes(pkg, gpu, T, B, H, Hkv, D, K, batched, yarn, monkeypatch):
    """RMS_NORM, MUL, the q, k and v projections and both rotations at prefill sizes as one call: the norm in the pre-tiled
    kernel's activation pass, the three matrices as one product over those tiles, the rotations in that product's epilogue
    from a table of angles (heads of 64 rows) or in place behind it (128).  Against the separate calls (RMS_NORM+MUL, three
    MUL_MATs, two ROPEs): the same bits -- the sequences flattened into one token dimension or as a batch, ragged token
    tiles, 64- and 128-wide heads, plain and YaRN-mixed angles with frequency factors."""
    import torch
    say(f"fused rms_norm+mul, q/k/v as one pre-tiled product, rope: T={T} B={B} H={H}/{Hkv} D={D} K={K} batched={batched} yarn={yarn}")
    L, d = pkg.lib(), pkg.desc
    monkeypatch.setenv("VX_GEMM_Q8T", "2")
    g = rng("f-nqkv-t", T, B, H, D, K)
    ws = [q8_dev((0.05 * g.standard_normal((n * D, K))).astype(np.float32))[0] for n in (H, Hkv, Hkv)]
    wd = [pkg.desc_q8(w, K) for w in ws]
    x = dev((2.0 * g.standard_normal((B, 1, T, K) if batched else (B * T, K))).astype(np.float32))
    nw = dev((1 + 0.1 * g.standard_normal(K)).astype(np.float32))
    pos = torch.arange(300, 300 + T, dtype=torch.int32, device="cuda")
    ff = dev((1.0 + g.random(D // 2)).astype(np.float32))
    rope_args = (D, 2, 4096, 10000.0, 0.5, 1.0, 1.1, 32.0, 1.0) if yarn else (D, 2, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0)

    def outs():
        return (torch.full((B, T, H, D), float("nan"), dtype=torch.float32, device="cuda"),
                torch.full((B, T, Hkv, D), float("nan"), dtype=torch.float32, device="cuda"),
                torch.full((B, 1, T, Hkv * D) if batched else (B * T, Hkv * D), float("nan"), dtype=torch.float32, device="cuda"))

    q1, k1, v1 = outs()
    normed = torch.empty_like(x)
    flat = (lambda t, rows: t.view(B, 1, T, rows)) if batched else (lambda t, rows: t.view(B * T, rows))
    ok(pkg, L.vx_rms_norm_mul(d(x), d(nw), d(normed), 1e-5, None), "rms_norm_mul")
    ok(pkg, L.vx_mul_mat(wd[0], d(normed), d(flat(q1, H * D)), pkg.ACT_FLOAT, None), "q")
    ok(pkg, L.vx_mul_mat(wd[1], d(normed), d(flat(k1, Hkv * D)), pkg.ACT_FLOAT, None), "k")
    ok(pkg, L.vx_mul_mat(wd[2], d(normed), d(v1), pkg.ACT_FLOAT, None), "v")
    for t in (q1, k1):
        ok(pkg, L.vx_rope(d(t), pos.data_ptr(), ff.data_ptr(), d(t), *rope_args, None), "rope")
    q2, k2, v2 = outs()
    assert L.vx_supports_norm_qkv_proj_rope(d(x), d(nw), *wd, d(q2), d(k2), d(v2), D, 2) == 0
    assert L.vx_supports_norm_qkv_proj_rope_tiled(d(x), d(nw), *wd, d(q2), d(k2), d(v2), D, 2, pkg.ACT_FLOAT) == 1
    assert L.vx_supports_norm_qkv_proj_rope_tiled(d(x), d(nw), *wd, d(q2), d(k2), d(v2), D, 2, pkg.ACT_Q8) == 0
    ok(pkg, L.vx_norm_qkv_proj_rope(d(x), d(nw), 1e-5, *wd, pos.data_ptr(), ff.data_ptr(), d(q2), d(k2), d(v2), *rope_args, pkg.ACT_FLOAT, None),
       "norm_qkv_proj_rope")
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2)
    assert bool(torch.isfinite(q2).all()) and bool(torch.isfinite(v2).all())


@pytest.mark.parametrize("T,n_past,B,Hkv,D", [(1, 639, 2, 2, 64), (1, 300, 1, 2, 64), (2, 1000, 2, 4, 128), (3, 4000, 2, 2, 64)])
@pytest.mark.parametrize("poison", [None, "nan"])
def test_flash_attn_two_segments_with_cache_write(pkg, gpu, T, n_past, B, Hkv, D, poison):
    import torch
    say(f"attention over cached + current keys with the cache write folded in T={T} n_past={n_past} B={B} Hkv={Hkv} D={D} {poison}")
    L, d = pkg.lib(), pkg.desc
    H = 8 * Hkv
    g = rng("f-kv2s", T, n_past, B, D)
    q = dev(g.standard_normal((B, H, T, D)).astype(np.float32))
    caches = [dev(g.standard_normal((B, Hkv, n_past + T + 5, D)).astype(np.float32)) for _ in range(2)]
    caches += [c.clone() for c in caches]
    kc1, vc1, kc2, vc2 = caches
    k = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))   # as the projection + rope leave them
    v = dev(g.standard_normal((B, T, Hkv, D)).astype(np.float32))
    if poison:
        v[0, 0, 0, 3] = float("nan")
    kcur, vcur = k.transpose(1, 2), v.transpose(1, 2)
    mask = dev(reflib.causal_mask(T, n_past + T, n_past)) if T > 1 else None
    sc = 1.0 / np.sqrt(D)

    def slot(c):
        return c[:, :, n_past:n_past + T].transpose(1, 2)

    a = torch.empty((B, T, H, D), dtype=torch.float32, device="cuda")
    b = torch.empty_like(a)
    for sync_scale, sync_bias in ((0.0, 0.0), (0.125, 0.5)):
        ok(pkg, L.vx_flash_attn_ext_kv2(d(q), d(kc1[:, :, :n_past]), d(kcur), d(vc1[:, :, :n_past]), d(vcur), d(mask), None, d(a), sc, 0.0, 0.0, None), "kv2")
        ok(pkg, L.vx_kv_store_sync(d(k), d(slot(kc1)), d(v), d(slot(vc1)), d(a), d(a), sync_scale, sync_bias, None), "kv_store_sync")
        assert L.vx_supports_flash_attn_ext_kv2_store(d(q), d(kc2[:, :, :n_past]), d(kcur), d(vc2[:, :, :n_past]), d(vcur), d(mask),
                                                      d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(b)) == 1
        ok(pkg, L.vx_flash_attn_ext_kv2_store(d(q), d(kc2[:, :, :n_past]), d(kcur), d(vc2[:, :, :n_past]), d(vcur), d(mask), None,
                                              d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(b), sc, 0.0, 0.0, sync_scale, sync_bias, None), "kv2_store")
        torch.cuda.synchronize()
        assert same_bits(kc1, kc2) and same_bits(vc1, vc2)
        assert torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(a.nan_to_num(7.0), b.nan_to_num(7.0))
        if poison:
            assert bool(torch.isnan(b).all())
    # too few keys for the split path: refused, the separate calls remain
    assert L.vx_supports_flash_attn_ext_kv2_store(d(q), d(kc2[:, :, :100]), d(kcur), d(vc2[:, :, :100]), d(vcur), None,
                                                  d(k), d(slot(kc2)), d(v), d(slot(vc2)), d(b)) == 0


@pytest.mark.parametrize("N", [2, 14, 40])
def test_groups_with_f16_weights(pkg, gpu, N):
    import torch
    say(f"node groups over F16 weight matrices, {N} tokens")
    L, d = pkg.lib(), pkg.desc
    H, Hkv, D, K, F = 4, 2, 64, 512, 768
    g = rng("f-f16", N)
    mk = lambda m: dev((0.05 * g.standard_normal((m, K))).astype(np.float16))
    wq, wk, wv, wg, wu = mk(H * D), mk(Hkv * D), mk(Hkv * D), mk(F), mk(F)
    wo = dev((0.05 * g.standard_normal((K, H * D))).astype(np.float16))
    x = dev(g.standard_normal((N, K)).astype(np.float32))
    nw = dev((1 + 0.1 * g.standard_normal(K)).astype(np.float32))
    pos = torch.arange(5, 5 + N, dtype=torch.int32, device="cuda")
    rope_args = (D, 2, 4096, 10000.0, 1.0, 0.0, 1.0, 32.0, 1.0)
    mode = pkg.ACT_FLOAT
    # rms_norm + q/k/v + rope
    normed = torch.empty_like(x)
    ok(pkg, L.vx_rms_norm_mul(d(x), d(nw), d(normed), 1e-5, None), "rms_norm_mul")
    q1 = torch.empty((1, N, H, D), dtype=torch.float32, device="cuda")
    k1 = torch.empty((1, N, Hkv, D), dtype=torch.float32, device="cuda")
    v1 = torch.empty((N, Hkv * D), dtype=torch.float32, device="cuda")
    for w, o, M in ((wq, q1, H * D), (wk, k1, Hkv * D), (wv, v1, Hkv * D)):
        ok(pkg, L.vx_mul_mat(d(w), d(normed), d(o.view(N, M)), mode, None), "mul_mat")
    for o in (q1, k1):
        ok(pkg, L.vx_rope(d(o), pos.data_ptr(), None, d(o), *rope_args, None), "rope")
    q2, k2, v2 = torch.empty_like(q1), torch.empty_like(k1), torch.empty_like(v1)
    assert L.vx_supports_norm_qkv_proj_rope(d(x), d(nw), d(wq), d(wk), d(wv), d(q2), d(k2), d(v2), D, 2) == 1
    ok(pkg, L.vx_norm_qkv_proj_rope(d(x), d(nw), 1e-5, d(wq), d(wk), d(wv), pos.data_ptr(), None, d(q2), d(k2), d(v2), *rope_args, mode, None), "norm_qkv")
    # rms_norm + gate/up + SwiGLU
    ga, up, a1, a2 = (torch.empty((N, F), dtype=torch.float32, device="cuda") for _ in range(4))
    ok(pkg, L.vx_mul_mat(d(wg), d(normed), d(ga), mode, None), "gate")
    ok(pkg, L.vx_mul_mat(d(wu), d(normed), d(up), mode, None), "up")
    ok(pkg, L.vx_glu(pkg.GLU_SWIGLU, d(ga), d(up), d(a1), 0, None), "glu")
    ok(pkg, L.vx_norm_mul_mat_swiglu(d(x), d(nw), 1e-5, d(wg), d(wu), d(a2), mode, None), "norm_swiglu")
    # projection + scale + residual
    attn = q1.view(N, H * D)
    prod, r1, r2 = (torch.empty((N, K), dtype=torch.float32, device="cuda") for _ in range(3))
    ok(pkg, L.vx_mul_mat(d(wo), d(attn), d(prod), mode, None), "o")
    ok(pkg, L.vx_scale(d(prod), d(prod), 0.3, 0.0, None), "scale")
    ok(pkg, L.vx_binary(pkg.BIN_ADD, d(x), d(prod), d(r1), None), "add")
    ok(pkg, L.vx_mul_mat_scale_add(d(wo), d(attn), d(x), d(r2), 0.3, mode, None), "mul_mat_scale_add")
    torch.cuda.synchronize()
    assert torch.equal(q1, q2) and torch.equal(k1, k2) and torch.equal(v1, v2)
    assert torch.equal(a1, a2)
    assert torch.equal(r1, r2)


# ------------------------------------------------------------------------- runs of tiny nodes
def _run_both(gpu, program, tensors):
    """program: list of (op, dst, src0, src1, aux, p0, p1) over names in `tensors` (name -> numpy array, the initial
    contents).  Runs it node by node through the separate entry points and as ONE vx_small_graph launch, each on its
    own copy of the tensors; returns both sets of device tensors."""
    import torch
    sets = []
    for mode in ("separate", "one launch"):
        T = {k: dev(v) for k, v in tensors.items()}
        g = lambda n: None if n is None else (T[n[0]][n[1]] if isinstance(n, tuple) else T[n])   # (name, index) = a view
        if mode == "separate":
            for op, dst, s0, s1, aux, p0, p1 in program:
                d, a, b = g(dst), g(s0), g(s1)
                if op <= gpu.NODE_DIV: gpu.binary(op, a, b, out=d)
                elif op == gpu.NODE_ADD1: gpu.add1(a, b, out=d)
                elif op == gpu.NODE_SCALE: gpu.scale(a, p0, p1, out=d)
                elif op == gpu.NODE_UNARY: gpu.unary(aux, a, out=d)
                elif op == gpu.NODE_CPY: gpu.cpy(a, d)
                elif op == gpu.NODE_CONCAT: gpu.concat(a, b, aux, out=d)
                elif op == gpu.NODE_REPEAT: gpu.repeat(a, None, out=d)
                elif op == gpu.NODE_SUM: gpu.sum_all(a, out=d)
                else: gpu.check(gpu.lib().vx_arange(gpu.desc(d), p0, p1, None), "arange")
        else:
            nodes = [gpu.small_node(op, g(dst), g(s0), g(s1), aux, p0, p1) for op, dst, s0, s1, aux, p0, p1 in program]
            for i in range(0, len(nodes), 16):
                gpu.small_graph(nodes[i:i + 16])
        torch.cuda.synchronize()
        sets.append(T)
    return sets


def _assert_same(sets, what):
    """Bit for bit, except that a NaN only has to be a NaN in both: which operand's sign and payload an arithmetic
    instruction hands on is the compiler's choice of operand order, in the separate kernels as much as in the run."""
    import torch
    a, b = sets
    for k in a:
        x, y = a[k].contiguous(), b[k].contiguous()
        if x.dtype in (torch.float32, torch.float16):
            nx, ny = torch.isnan(x), torch.isnan(y)
            assert torch.equal(nx, ny), (what, k, "NaN positions")
            x, y = torch.where(nx, torch.zeros_like(x), x), torch.where(ny, torch.zeros_like(y), y)
        assert torch.equal(x.view(torch.uint8), y.view(torch.uint8)), (what, k)


def test_small_graph_cfg_guidance_and_euler_update(gpu):
    """The node chain UnifiedCFM puts behind the estimator (src/unified_cfm.cpp:30-86, 146): zero-star scale from two
    SUMs, ARANGE for eps, DIV, REPEAT, the guidance combination and the Euler update of x -- 16 nodes, one launch, every
    intermediate and the result bit-identical to the separate launches; NaN / infinity in the velocities included."""
    say("small graph: CFG guidance + Euler update")
    N = gpu
    for poison in (None, np.nan, np.inf):
        t = {"vc": rng("sg", "vc").standard_normal((2, 64)).astype(np.float32), "vu": rng("sg", "vu").standard_normal((2, 64)).astype(np.float32),
             "x": rng("sg", "x").standard_normal((2, 64)).astype(np.float32), "bias": rng("sg", "b").standard_normal((64,)).astype(np.float32)}
        if poison is not None:
            t["vu"][1, 7] = poison
        for name in ("pc", "pu", "uu", "us", "rep", "diff", "cs", "dphi", "step", "xn", "vcb", "vub"):
            t[name] = np.zeros((2, 64), np.float32)
        for name in ("dot", "nrm", "eps", "den", "st"):
            t[name] = np.zeros((1,), np.float32)
        prog = [(N.NODE_ADD, "vcb", "vc", "bias", 0, 0, 0), (N.NODE_ADD, "vub", "vu", "bias", 0, 0, 0),
                (N.NODE_MUL, "pc", "vcb", "vub", 0, 0, 0), (N.NODE_SUM, "dot", "pc", None, 0, 0, 0),
                (N.NODE_MUL, "uu", "vub", "vub", 0, 0, 0), (N.NODE_SUM, "nrm", "uu", None, 0, 0, 0),
                (N.NODE_ARANGE, "eps", None, None, 0, 1e-8, 1.0), (N.NODE_ADD, "den", "nrm", "eps", 0, 0, 0),
                (N.NODE_DIV, "st", "dot", "den", 0, 0, 0), (N.NODE_REPEAT, "rep", "st", None, 0, 0, 0),
                (N.NODE_MUL, "us", "vub", "rep", 0, 0, 0), (N.NODE_SUB, "diff", "vcb", "us", 0, 0, 0),
                (N.NODE_SCALE, "cs", "diff", None, 0, 2.0, 0.0), (N.NODE_ADD, "dphi", "us", "cs", 0, 0, 0),
                (N.NODE_SCALE, "step", "dphi", None, 0, 0.0937, 0.0), (N.NODE_SUB, "xn", "x", "step", 0, 0, 0)]
        sets = _run_both(gpu, prog, t)
        _assert_same(sets, f"guidance poison={poison}")
        if poison is None:
            import torch
            xn = sets[1]["xn"].cpu().numpy().astype(np.float64)
            vc, vu = (t["vc"] + t["bias"]).astype(np.float64), (t["vu"] + t["bias"]).astype(np.float64)
            st = (vc * vu).sum() / ((vu * vu).sum() + 1e-8)
            want = t["x"] - 0.0937 * (st * vu + 2.0 * (vc - st * vu))
            assert np.abs(xn - want).max() <= 1e-5


def test_small_graph_sequence_assembly_copies_and_sums(gpu):
    """CONCATs that assemble LocDiT's 14-token CFG-pair sequence (src/locdit.cpp:441-452), casts, strided and in-place
    operands, and SUMs in each of vx_sum's single-block orders (one wave in 16-byte units, one wave element-wise on an
    odd row length, the 1024-thread block beyond 1024 units)."""
    import torch
    say("small graph: concat / cpy / repeat / sum orders")
    N = gpu
    H = 1024
    t = {"tok_c": rng("sg2", "tc").standard_normal((1, H)).astype(np.float32), "tok_u": rng("sg2", "tu").standard_normal((1, H)).astype(np.float32),
         "cond": rng("sg2", "c").standard_normal((4, H)).astype(np.float32), "xp": rng("sg2", "x").standard_normal((2, H)).astype(np.float32),
         "a5": np.zeros((5, H), np.float32), "b5": np.zeros((5, H), np.float32), "a7": np.zeros((7, H), np.float32), "b7": np.zeros((7, H), np.float32),
         "pair": np.zeros((14, H), np.float32), "pair16": np.zeros((14, H), np.float16), "back": np.zeros((14, H), np.float32),
         "ids": np.arange(14, dtype=np.int32), "idf": np.zeros((14,), np.float32), "idi": np.zeros((14,), np.int32),
         "odd": rng("sg2", "odd").standard_normal((3, 333)).astype(np.float32), "s_vec": np.zeros((1,), np.float32),
         "s_odd": np.zeros((1,), np.float32), "s_blk": np.zeros((1,), np.float32), "s_view": np.zeros((1,), np.float32),
         "tile": np.zeros((3, 2, 4, 8), np.float32), "seed": rng("sg2", "seed").standard_normal((1, 2, 1, 8)).astype(np.float32),
         "cat0": np.zeros((2, 2056), np.float32), "wide": rng("sg2", "w").standard_normal((2, 1028)).astype(np.float32)}
    prog = [(N.NODE_CONCAT, "a5", "tok_c", "cond", 1, 0, 0), (N.NODE_CONCAT, "a7", "a5", "xp", 1, 0, 0),
            (N.NODE_CONCAT, "b5", "tok_u", "cond", 1, 0, 0), (N.NODE_CONCAT, "b7", "b5", "xp", 1, 0, 0),
            (N.NODE_CONCAT, "pair", "a7", "b7", 1, 0, 0),
            (N.NODE_CPY, "pair16", "pair", None, 0, 0, 0), (N.NODE_CPY, "back", "pair16", None, 0, 0, 0),
            (N.NODE_CPY, "idf", "ids", None, 0, 0, 0), (N.NODE_CPY, "idi", "idf", None, 0, 0, 0),
            (N.NODE_SUM, "s_vec", "xp", None, 0, 0, 0),          # 512 units of 16 bytes: one wave
            (N.NODE_SUM, "s_odd", "odd", None, 0, 0, 0),         # 999 single elements: one wave, element order
            (N.NODE_SUM, "s_blk", "pair", None, 0, 0, 0),        # 3584 units: the 1024-thread block
            (N.NODE_SUM, "s_view", ("pair", slice(3, 7)), None, 0, 0, 0),   # rows 3..6 of the sequence: a view
            (N.NODE_REPEAT, "tile", "seed", None, 0, 0, 0),
            (N.NODE_CONCAT, "cat0", "wide", "wide", 0, 0, 0),    # along dim 0, rows of 1028
            (N.NODE_UNARY, "xp", "xp", None, N.UNARY_SILU, 0, 0),           # in place
            (N.NODE_ADD1, "cond", "cond", "s_vec", 0, 0, 0),     # in place, scalar from an earlier node of the run
            (N.NODE_SCALE, "back", "back", None, 0, 0.5, 1.25)]
    sets = _run_both(gpu, prog, t)
    _assert_same(sets, "assembly")
    got = sets[1]
    pair = np.concatenate([t["tok_c"], t["cond"], t["xp"], t["tok_u"], t["cond"], t["xp"]], axis=0)
    assert np.array_equal(got["pair"].cpu().numpy(), pair)
    assert float(got["s_blk"].cpu()[0]) == np.float32(pair.astype(np.float64).sum())
    assert np.array_equal(got["idi"].cpu().numpy(), np.arange(14, dtype=np.int32))
    assert np.array_equal(got["tile"].cpu().numpy(), np.tile(t["seed"], (3, 1, 4, 1)))


@pytest.mark.gpu
@pytest.mark.parametrize("H,R,prefix,patch", [(1024, 8, 4, 2), (1024, 3, 4, 2), (30, 5, 3, 1), (8, 2, 1, 1)])
def test_concat_tree_from_its_leaves(gpu, H, R, prefix, patch):
    """LocDiT's sequence assembly for R requests (src/locdit.cpp:401-452 with a request dimension): two sequences
    (t + mu | cond | x) and (t for every request | cond | x) joined along the token dimension, as one launch from the six
    leaves against the five CONCATs and the REPEAT node by node.  Rows of 16-byte multiples and not; dim 0 as well."""
    import torch
    say(f"concat tree: H={H} R={R} prefix={prefix} patch={patch}")
    g = lambda tag, *shape: dev(rng("cattree", tag, H, R).standard_normal(shape).astype(np.float32))
    comb_c, cond, x, t_row = g("c", R, 1, H), g("k", R, prefix, H), g("x", R, patch, H), g("t", 1, 1, H)
    # node by node
    comb_u = gpu.repeat(t_row, (R, 1, H))
    seq_c = gpu.concat(gpu.concat(comb_c, cond, 1), x, 1)
    seq_u = gpu.concat(gpu.concat(comb_u, cond, 1), x, 1)
    want = gpu.concat(seq_c, seq_u, 1)
    L = 1 + prefix + patch
    got = torch.full((R, 2 * L, H), float("nan"), dtype=torch.float32, device="cuda")
    gpu.concat_many([comb_c, cond, x, t_row, cond, x], [1, prefix, patch, 1, prefix, patch], 1, got)
    torch.cuda.synchronize()
    assert torch.equal(want.view(torch.int32), got.view(torch.int32))
    # along dim 0 (no 16-byte units), a strided source and a source repeated along the dimension itself
    a, b = g("a", R, 3, 5), g("b", R, 3, 7)
    wide = g("w", R, 3, 12)[:, :, 2:6]                       # a view: rows 48 bytes apart, 4 of them used
    pair = g("p", R, 3, 2)
    want0 = gpu.concat(gpu.concat(gpu.concat(a, b, 0), wide.contiguous(), 0), gpu.repeat(pair, (R, 3, 6)), 0)
    got0 = torch.full((R, 3, 22), float("nan"), dtype=torch.float32, device="cuda")
    gpu.concat_many([a, b, wide, pair], [5, 7, 4, 6], 0, got0)
    torch.cuda.synchronize()
    assert torch.equal(want0.view(torch.int32), got0.view(torch.int32))


@pytest.mark.gpu
@pytest.mark.parametrize("R,n", [(8, 128), (3, 100), (1, 64), (5, 1001)])
@pytest.mark.parametrize("private", [0, 1])
def test_small_graph_row_sums_and_repeats_per_request(gpu, R, n, private):
    """The guidance arithmetic of several requests at once (src/unified_cfm.cpp:100-140 with a request per row): row sums,
    a value per request repeated over the request's elements, a row repeated for every request, and a reshaped view of a
    tensor the run wrote read from where the run keeps it.  One launch against a launch per node, bit for bit."""
    import torch
    say(f"small graph: row sums R={R} n={n} private={private}")
    N = gpu
    t = {"vc": rng("sgr", "c", R, n).standard_normal((R, n)).astype(np.float32), "vu": rng("sgr", "u", R, n).standard_normal((R, n)).astype(np.float32),
         "row": rng("sgr", "r", n).standard_normal((1, n)).astype(np.float32)}
    for name in ("diff", "dot", "sq", "st", "fill", "tile", "out"):
        t[name] = np.zeros((R, n), np.float32)
    for name in ("sdot", "ssq", "eps", "den", "star"):
        t[name] = np.zeros((R, 1), np.float32)
    t["flat_sum"] = np.zeros((R,), np.float32)
    views = {"star_flat": ("star", (R,)), "ssq_flat": ("ssq", (R,))}
    prog = [(N.NODE_SUB, "diff", "vc", "vu", 0, 0, 0), (N.NODE_MUL, "dot", "vc", "vu", 0, 0, 0), (N.NODE_MUL, "sq", "vu", "vu", 0, 0, 0),
            (N.NODE_SUM_ROWS, "sdot", "dot", None, 0, 0, 0), (N.NODE_SUM_ROWS, "ssq", "sq", None, 0, 0, 0),
            (N.NODE_SCALE, "den", "ssq", None, 0, 1.0, 1e-8), (N.NODE_DIV, "star", "sdot", "den", 0, 0, 0),
            (N.NODE_REPEAT, "fill", "star", None, 0, 0, 0),                                                # a value per request
            (N.NODE_MUL, "st", "vu", "fill", 0, 0, 0),
            (N.NODE_REPEAT, "tile", "row", None, 0, 0, 0),                                                # the same row for every request
            (N.NODE_ADD, "flat_sum", "star_flat", "ssq_flat", 0, 0, 0),                                   # reshaped views of the run's own tensors
            (N.NODE_ADD, "out", "st", "tile", 0, 0, 0), (N.NODE_ADD, "out", "out", "diff", 0, 0, 0),
            (N.NODE_MUL, "out", "out", "row", 0, 0, 0)]                                                   # a row under every request, no REPEAT
    keep = {"out", "flat_sum", "star"} if private else None
    sets = []
    for mode in ("separate", "one launch"):
        T = {k: dev(v) for k, v in t.items()}
        for k, (base, shape) in views.items():
            T[k] = T[base].view(*shape)
        if mode == "separate":
            for op, dst, s0, s1, aux, p0, p1 in prog:
                d, a, b = T[dst], (None if s0 is None else T[s0]), (None if s1 is None else T[s1])
                if op <= N.NODE_DIV: N.binary(op, a, b, out=d)
                elif op == N.NODE_SCALE: N.scale(a, p0, p1, out=d)
                elif op == N.NODE_REPEAT: N.repeat(a, None, out=d)
                else: N.sum_rows(a, out=d)
        else:
            last = {dst: i for i, (_, dst, *_r) in enumerate(prog)}
            nodes = [N.small_node(op, T[dst], None if s0 is None else T[s0], None if s1 is None else T[s1], aux, p0, p1,
                                  private=bool(private and not (dst in keep and last[dst] == i)))
                     for i, (op, dst, s0, s1, aux, p0, p1) in enumerate(prog)]
            for nd in nodes:
                assert N.lib().vx_supports_small_node(nd) == 1
            N.small_graph(nodes)
        torch.cuda.synchronize()
        sets.append({k: v for k, v in T.items() if k not in views} if keep is None else {k: T[k] for k in keep})
    _assert_same(sets, f"row sums R={R} n={n} private={private}")
    assert float(sets[1]["out"].abs().sum()) > 0


@pytest.mark.gpu
@pytest.mark.parametrize("n", [64, 1001, 2700])
@pytest.mark.parametrize("private", [False, True])
def test_small_graph_dense_runs_barriers_and_wide_moves(gpu, n, private):
    """Runs of dense F32 nodes take the kernel that the host has resolved every operand for: operands the run only reads
    are in LDS before the first node, a node whose inputs were written by the reading thread itself meets no barrier,
    plain moves go 16 bytes per thread.  The cases that tests: rows longer than the work-group (several elements per
    thread), a value broadcast from a sum of the same run, an image rewritten in place after other threads read it,
    concatenations with and without 16-byte alignment, intermediates with and without memory behind them."""
    import torch
    say(f"small graph: dense run n={n} private={private}")
    N = gpu
    t = {"a": rng("sgd", "a", n).standard_normal((3, n)).astype(np.float32), "b": rng("sgd", "b", n).standard_normal((3, n)).astype(np.float32),
         "row": rng("sgd", "r", n).standard_normal((1, n)).astype(np.float32)}
    for name in ("p", "q", "r", "u", "out"):
        t[name] = np.zeros((3, n), np.float32)
    for name in ("s", "s2"):
        t[name] = np.zeros((1,), np.float32)
    t["cat"] = np.zeros((6, n), np.float32); t["cat1"] = np.zeros((4, n), np.float32)
    t["flat"] = np.zeros((3 * n,), np.float32); t["shift"] = np.zeros((3 * n + 3,), np.float32)
    t["three"] = np.array([1.0, 2.0, 3.0], np.float32)
    prog = [(N.NODE_MUL, "p", "a", "b", 0, 0, 0), (N.NODE_UNARY, "q", "p", None, N.UNARY_SILU, 0, 0),       # q from p: own elements
            (N.NODE_SUM, "s", "q", None, 0, 0, 0),                                                        # reads across threads
            (N.NODE_ADD1, "r", "q", "s", 0, 0, 0),                                                        # broadcast of the run's own scalar
            (N.NODE_SCALE, "q", "r", None, 0, 0.5, -1.0),                                                 # q rewritten after the sum read it
            (N.NODE_SUM, "s2", "q", None, 0, 0, 0), (N.NODE_DIV, "s2", "s2", "s", 0, 0, 0),               # scalars stay with thread 0
            (N.NODE_REPEAT, "u", "s2", None, 0, 0, 0), (N.NODE_SUB, "u", "u", "q", 0, 0, 0),
            (N.NODE_CONCAT, "cat", "u", "a", 1, 0, 0),                                                    # whole quads when n % 4 == 0
            (N.NODE_CONCAT, "cat1", "row", "r", 1, 0, 0),
            (N.NODE_CPY, "flat", "u", None, 0, 0, 0), (N.NODE_CONCAT, "shift", "three", "flat", 0, 0, 0),   # 3 elements first: no quads
            (N.NODE_CPY, "out", "u", None, 0, 0, 0), (N.NODE_ADD, "out", "out", "r", 0, 0, 0)]
    keep = {"out", "cat", "cat1", "s2", "shift"} if private else None
    sets = []
    for mode in ("separate", "one launch"):
        T = {k: dev(v) for k, v in t.items()}
        if mode == "separate":
            for op, dst, s0, s1, aux, p0, p1 in prog:
                d, a, b = T[dst], (None if s0 is None else T[s0]), (None if s1 is None else T[s1])
                if op <= N.NODE_DIV: N.binary(op, a, b, out=d)
                elif op == N.NODE_ADD1: N.add1(a, b, out=d)
                elif op == N.NODE_SCALE: N.scale(a, p0, p1, out=d)
                elif op == N.NODE_UNARY: N.unary(aux, a, out=d)
                elif op == N.NODE_CPY: N.cpy(a, d)
                elif op == N.NODE_CONCAT: N.concat(a, b, aux, out=d)
                elif op == N.NODE_REPEAT: N.repeat(a, None, out=d)
                else: N.sum_all(a, out=d)
        else:
            last = {dst: i for i, (_, dst, *_r) in enumerate(prog)}
            nodes = [N.small_node(op, T[dst], None if s0 is None else T[s0], None if s1 is None else T[s1], aux, p0, p1,
                                  private=bool(private and not (dst in keep and last[dst] == i)))
                     for i, (op, dst, s0, s1, aux, p0, p1) in enumerate(prog)]
            N.small_graph(nodes)
        torch.cuda.synchronize()
        sets.append(T if keep is None else {k: T[k] for k in keep})
    _assert_same(sets, f"dense n={n} private={private}")
    assert float(sets[1]["out"].abs().sum()) > 0


@pytest.mark.parametrize("seed", list(range(160)))
def test_small_graph_random_programs(gpu, seed):
    """Random runs of up to 16 nodes over a small pool of tensors -- results rewritten in place, values read again after
    their source changed, scalars and per-request columns produced inside the run and broadcast later, reshaped views of the
    run's own tensors, temporaries that are private to the run -- one launch against a launch per node, bit for bit.  What
    it is after: the host-side decisions of the dense kernel (which barriers a run can do without, which operands are
    brought into LDS beforehand, which image a view reads) and the general kernel's fallbacks for strided operands."""
    import torch
    N = gpu
    r = rng("sg-random", seed)
    R, n = int(r.choice([1, 2, 3, 5])), int(r.choice([64, 100, 257, 1024]))
    say(f"small graph: random program seed={seed} R={R} n={n}")
    init = {}
    for name in ("A0", "A1", "A2", "T0", "T1", "T2"):
        init[name] = r.standard_normal((R, n)).astype(np.float32)
    init["W"] = r.standard_normal((R, n + 8)).astype(np.float32)          # its first n columns: a strided operand
    init["row"] = r.standard_normal((1, n)).astype(np.float32)
    for name in ("c0", "ct"):
        init[name] = r.standard_normal((R, 1)).astype(np.float32)
    for name in ("s0", "st"):
        init[name] = r.standard_normal((1,)).astype(np.float32)
    init["cat"] = np.zeros((2 * R, n), np.float32)
    init["wide"] = np.zeros((R, 2 * n), np.float32)
    temps = {"T0", "T1", "T2", "ct", "st"}
    full, cols, scalars = ["A0", "A1", "A2", "T0", "T1", "T2"], ["c0", "ct"], ["s0", "st"]
    pick = lambda names: names[int(r.integers(len(names)))]
    prog = []
    for _ in range(int(r.integers(6, 17))):
        kind = pick(["ew", "ew", "ew", "bcast", "add1", "scale", "unary", "cpy", "repeat", "sum", "sum_rows", "concat", "colop", "strided", "flat"])
        if kind == "ew":        prog.append((pick([N.NODE_ADD, N.NODE_SUB, N.NODE_MUL]), pick(full), pick(full), pick(full), 0, 0.0, 0.0))
        elif kind == "bcast":   prog.append((pick([N.NODE_ADD, N.NODE_MUL]), pick(full), pick(full), pick(["row", "c0", "ct", "s0", "st"]), 0, 0.0, 0.0))
        elif kind == "add1":    prog.append((N.NODE_ADD1, pick(full), pick(full), pick(scalars), 0, 0.0, 0.0))
        elif kind == "scale":   prog.append((N.NODE_SCALE, pick(full + cols + scalars), None, None, 0, float(r.uniform(-1.5, 1.5)), float(r.uniform(-1, 1))))
        elif kind == "unary":   prog.append((N.NODE_UNARY, pick(full), pick(full), None, pick([N.UNARY_SILU, N.UNARY_NEG, N.UNARY_TANH]), 0.0, 0.0))
        elif kind == "cpy":     prog.append((N.NODE_CPY, pick(full), pick(full), None, 0, 0.0, 0.0))
        elif kind == "repeat":  prog.append((N.NODE_REPEAT, pick(full), pick(["row", "c0", "ct", "s0", "st"]), None, 0, 0.0, 0.0))
        elif kind == "sum":     prog.append((N.NODE_SUM, pick(scalars), pick(full), None, 0, 0.0, 0.0))
        elif kind == "sum_rows": prog.append((N.NODE_SUM_ROWS, pick(cols), pick(full), None, 0, 0.0, 0.0))
        elif kind == "concat":
            if r.integers(2): prog.append((N.NODE_CONCAT, "cat", pick(full), pick(full), 1, 0.0, 0.0))
            else:             prog.append((N.NODE_CONCAT, "wide", pick(full), pick(full), 0, 0.0, 0.0))
        elif kind == "colop":   prog.append((pick([N.NODE_ADD, N.NODE_MUL, N.NODE_DIV]), pick(cols), pick(cols), pick(cols + scalars), 0, 0.0, 0.0))
        elif kind == "strided": prog.append((pick([N.NODE_ADD, N.NODE_MUL]), pick(full), "Wv", pick(full), 0, 0.0, 0.0))
        else:                   prog.append((N.NODE_ADD, "A0f", pick(["A1f", "T0f"]), "A2f", 0, 0.0, 0.0))   # flat views of the run's tensors
    for i, p in enumerate(prog):                      # SCALE in place
        if p[0] == N.NODE_SCALE: prog[i] = (p[0], p[1], p[1], None, 0, p[5], p[6])
    base = lambda name: name[:-1] if name.endswith("f") else name
    sets = []
    for mode in ("separate", "one launch"):
        T = {k: dev(v) for k, v in init.items()}
        T["Wv"] = T["W"][:, :n]
        for k in ("A0", "A1", "A2", "T0"):
            T[k + "f"] = T[k].view(R * n)
        nodes = []
        for op, dst, s0, s1, aux, p0, p1 in prog:
            d, a, b = T[dst], (None if s0 is None else T[s0]), (None if s1 is None else T[s1])
            if mode == "separate":
                if op <= N.NODE_DIV: N.binary(op, a, b, out=d)
                elif op == N.NODE_ADD1: N.add1(a, b, out=d)
                elif op == N.NODE_SCALE: N.scale(a, p0, p1, out=d)
                elif op == N.NODE_UNARY: N.unary(aux, a, out=d)
                elif op == N.NODE_CPY: N.cpy(a, d)
                elif op == N.NODE_CONCAT: N.concat(a, b, aux, out=d)
                elif op == N.NODE_REPEAT: N.repeat(a, None, out=d)
                elif op == N.NODE_SUM: N.sum_all(a, out=d)
                else: N.sum_rows(a, out=d)
            else:
                nd = N.small_node(op, d, a, b, aux, p0, p1, private=base(dst) in temps)
                assert N.lib().vx_supports_small_node(nd) == 1, (op, dst, s0, s1)
                nodes.append(nd)
        if mode == "one launch":
            N.small_graph(nodes)
        torch.cuda.synchronize()
        sets.append({k: v for k, v in T.items() if base(k) not in temps and k in init})
    _assert_same(sets, f"random program seed={seed}: {prog}")


def test_small_graph_limits(gpu, pkg):
    """What a run may hold: at most 16 nodes, tensors of at most 16384 elements, only the tiny operators."""
    import torch
    L = pkg.lib()
    small = torch.zeros((4, 1024), dtype=torch.float32, device="cuda")
    big = torch.zeros((17, 1024), dtype=torch.float32, device="cuda")
    nd = gpu.small_node(gpu.NODE_ADD, small, small, small)
    assert L.vx_supports_small_node(nd) == 1
    assert L.vx_supports_small_node(gpu.small_node(gpu.NODE_ADD, big, big, big)) == 0
    assert L.vx_supports_small_node(gpu.small_node(13, small, small, small)) == 0                    # no such operator
    assert L.vx_supports_small_node(gpu.small_node(gpu.NODE_UNARY, small, small, aux=8)) == 0       # GELU
    arr = (pkg.VxSmallNode * 17)(*([nd] * 17))
    assert L.vx_small_graph(arr, 17, None) == 2   # VX_ERR_UNSUPPORTED
    assert L.vx_small_graph(arr, 0, None) == 2   # VX_ERR_UNSUPPORTED


@pytest.mark.gpu
@pytest.mark.parametrize("R,n", [(2, 512), (8, 64), (3, 30), (5, 101)])
@pytest.mark.parametrize("private", [0, 1])
def test_small_graph_sequence_assembly_per_request(gpu, R, n, private):
    """The CFG-pair sequence of several requests at once (src/locdit.cpp's CONCATs with the requests in the next dimension): a
    token row, the prefix rows and the patch rows joined along dim 1 for every request, a row repeated for every request and
    added -- CONCATs below the outermost dimension, whole 16-byte quads (n % 4 == 0) and single values.  One launch against a
    launch per node, bit for bit."""
    import torch
    say(f"small graph: per-request sequence assembly R={R} n={n} private={private}")
    N = gpu
    g = lambda tag, *shape: rng("sgq", tag, R, n).standard_normal(shape).astype(np.float32)
    t = {"tok": g("tok", R, 1, n), "cond": g("cond", R, 4, n), "xp": g("xp", R, 2, n), "row": g("row", 1, 1, n),
         "rep": np.zeros((R, 1, n), np.float32), "tokb": np.zeros((R, 1, n), np.float32),
         "a5": np.zeros((R, 5, n), np.float32), "a7": np.zeros((R, 7, n), np.float32), "b7": np.zeros((R, 7, n), np.float32),
         "pair": np.zeros((R, 14, n), np.float32), "out": np.zeros((R, 14, n), np.float32)}
    prog = [(N.NODE_REPEAT, "rep", "row", None, 0, 0, 0), (N.NODE_ADD, "tokb", "tok", "rep", 0, 0, 0),
            (N.NODE_CONCAT, "a5", "tokb", "cond", 1, 0, 0), (N.NODE_CONCAT, "a7", "a5", "xp", 1, 0, 0),
            (N.NODE_CONCAT, "b7", "a5", "xp", 1, 0, 0), (N.NODE_CONCAT, "pair", "a7", "b7", 1, 0, 0),
            (N.NODE_SCALE, "out", "pair", None, 0, 0.5, 0.25)]
    keep = {"out", "a7"} if private else None
    sets = []
    for mode in ("separate", "one launch"):
        T = {k: dev(v) for k, v in t.items()}
        if mode == "separate":
            for op, dst, s0, s1, aux, p0, p1 in prog:
                d, a, b = T[dst], T[s0], (None if s1 is None else T[s1])
                if op == N.NODE_ADD: N.binary(op, a, b, out=d)
                elif op == N.NODE_SCALE: N.scale(a, p0, p1, out=d)
                elif op == N.NODE_REPEAT: N.repeat(a, None, out=d)
                else: N.concat(a, b, aux, out=d)
        else:
            last = {dst: i for i, (_, dst, *_r) in enumerate(prog)}
            nodes = [N.small_node(op, T[dst], T[s0], None if s1 is None else T[s1], aux, p0, p1,
                                  private=bool(private and not (dst in keep and last[dst] == i)))
                     for i, (op, dst, s0, s1, aux, p0, p1) in enumerate(prog)]
            for nd in nodes:
                assert N.lib().vx_supports_small_node(nd) == 1
            N.small_graph(nodes)
        torch.cuda.synchronize()
        sets.append(dict(T) if keep is None else {k: T[k] for k in keep})
    _assert_same(sets, f"per-request assembly R={R} n={n} private={private}")
    want = np.concatenate([t["tok"] + t["row"], t["cond"], t["xp"]], axis=1)
    want = np.concatenate([want, want], axis=1) * 0.5 + 0.25
    assert np.array_equal(sets[1]["out"].cpu().numpy(), want.astype(np.float32))
