"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
header declares, refuses work without a device instead of falling back, the supports_*
truth table, and the ggml plugin's behaviour on a GPU-less host."""
import ctypes as C
import os
import re

import numpy as np
import pytest

import reflib

ROOT = reflib.ROOT


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "voxcpm_gfx950.h")).read()
    return sorted(set(re.findall(r"VX_API\s+[\w\s\*]+?\b(vx_\w+)\s*\(", text)))


def test_header_symbols_are_exported(pkg):
    lib = pkg.lib()
    names = declared_symbols()
    assert len(names) >= 25
    assert set(names) == set(pkg.EXPORTS)
    for n in names:
        assert hasattr(lib, n), n


def have_gpu(pkg):
    return pkg.lib().vx_device_count() > 0


def test_no_device_is_an_error_not_a_fallback(pkg):
    lib = pkg.lib()
    if have_gpu(pkg):
        pytest.skip("a GPU is present")
    assert lib.vx_device_count() == 0
    assert lib.vx_init(0) == 1  # VX_ERR_NO_DEVICE
    assert b"gfx950" in lib.vx_last_error()


def D(pkg, ttype, ne, nb, data=0x1000):
    return pkg.make_desc(ttype, ne, nb, data)


def f32(pkg, ne):
    nb = [4, 4 * ne[0], 4 * ne[0] * ne[1], 4 * ne[0] * ne[1] * ne[2]]
    return D(pkg, pkg.F32, ne, nb)


def f16(pkg, ne):
    nb = [2, 2 * ne[0], 2 * ne[0] * ne[1], 2 * ne[0] * ne[1] * ne[2]]
    return D(pkg, pkg.F16, ne, nb)


def q8(pkg, ne):
    rb = ne[0] // 32 * 34
    return D(pkg, pkg.Q8_0, ne, [34, rb, rb * ne[1], rb * ne[1] * ne[2]])


def test_supports_truth_table(pkg):
    lib = pkg.lib()
    # RMS_NORM: F32 only, equal shapes
    assert lib.vx_supports_rms_norm(f32(pkg, [1024, 7, 1, 1]), f32(pkg, [1024, 7, 1, 1])) == 1
    assert lib.vx_supports_rms_norm(f16(pkg, [1024, 7, 1, 1]), f16(pkg, [1024, 7, 1, 1])) == 0
    assert lib.vx_supports_rms_norm(f32(pkg, [1024, 7, 1, 1]), f32(pkg, [1024, 8, 1, 1])) == 0
    # ROPE: modes 0 (NORMAL) and 2 (NEOX) only
    x = f32(pkg, [64, 16, 5, 1])
    assert lib.vx_supports_rope(x, x, 64, 2) == 1 and lib.vx_supports_rope(x, x, 64, 0) == 1
    assert lib.vx_supports_rope(x, x, 64, 8) == 0 and lib.vx_supports_rope(x, x, 64, 24) == 0
    assert lib.vx_supports_rope(x, x, 66, 2) == 0 and lib.vx_supports_rope(x, x, 63, 2) == 0
    # FLASH_ATTN_EXT: D in {64,128}, K/V same type F16|F32, mask F16, GQA divisibility
    q, dst = f32(pkg, [64, 1, 16, 2]), f32(pkg, [64, 16, 1, 2])
    k = f16(pkg, [64, 4096, 2, 2])
    assert lib.vx_supports_flash_attn_ext(q, k, k, None, dst) == 1
    assert lib.vx_supports_flash_attn_ext(q, k, f32(pkg, [64, 4096, 2, 2]), None, dst) == 0
    assert lib.vx_supports_flash_attn_ext(q, f16(pkg, [64, 4096, 3, 2]), f16(pkg, [64, 4096, 3, 2]), None, dst) == 0
    q80, d80 = f32(pkg, [80, 1, 16, 2]), f32(pkg, [80, 16, 1, 2])
    assert lib.vx_supports_flash_attn_ext(q80, f16(pkg, [80, 64, 2, 2]), f16(pkg, [80, 64, 2, 2]), None, d80) == 0
    assert lib.vx_supports_flash_attn_ext(q, k, k, f16(pkg, [4096, 1, 1, 1]), dst) == 1
    assert lib.vx_supports_flash_attn_ext(q, k, k, f32(pkg, [4096, 1, 1, 1]), dst) == 0
    # MUL_MAT: Q8_0 / F16 / F32 weights x F32 activations
    x2, o2 = f32(pkg, [1024, 2, 1, 1]), f32(pkg, [4096, 2, 1, 1])
    assert lib.vx_supports_mul_mat(q8(pkg, [1024, 4096, 1, 1]), x2, o2) == 1
    assert lib.vx_supports_mul_mat(f16(pkg, [1024, 4096, 1, 1]), x2, o2) == 1
    assert lib.vx_supports_mul_mat(q8(pkg, [1024, 4096, 1, 1]), f16(pkg, [1024, 2, 1, 1]), o2) == 0
    assert lib.vx_supports_mul_mat(q8(pkg, [1024, 4096, 1, 1]), f32(pkg, [512, 2, 1, 1]), o2) == 0
    transposed = D(pkg, pkg.F32, [1024, 4096, 1, 1], [4 * 4096, 4, 4 * 1024 * 4096, 4 * 1024 * 4096])
    assert lib.vx_supports_mul_mat(transposed, x2, o2) == 0


def test_supports_truth_table_glue(pkg):
    """The glue operators of a decoder layer and the fused pairs: what supports_op will answer."""
    lib = pkg.lib()
    a = f32(pkg, [1024, 5, 3, 2])
    assert lib.vx_supports_binary(pkg.BIN_ADD, a, a, a) == 1
    assert lib.vx_supports_binary(pkg.BIN_MUL, a, f32(pkg, [1024, 1, 1, 1]), a) == 1      # norm weight over tokens
    assert lib.vx_supports_binary(pkg.BIN_MUL, a, f32(pkg, [1, 5, 1, 2]), a) == 1          # bias column
    assert lib.vx_supports_binary(pkg.BIN_ADD, a, f32(pkg, [1000, 5, 3, 2]), a) == 0       # not repeatable
    assert lib.vx_supports_binary(pkg.BIN_ADD, a, a, f32(pkg, [1024, 5, 3, 1])) == 0
    assert lib.vx_supports_binary(pkg.BIN_ADD, f16(pkg, [8, 1, 1, 1]), f16(pkg, [8, 1, 1, 1]), f16(pkg, [8, 1, 1, 1])) == 0
    assert lib.vx_supports_binary(7, a, a, a) == 0
    one = f32(pkg, [1, 1, 1, 1])
    assert lib.vx_supports_add1(a, one, a) == 1 and lib.vx_supports_add1(a, f32(pkg, [2, 1, 1, 1]), a) == 0
    assert lib.vx_supports_unary(pkg.UNARY_SILU, a, a) == 1
    assert lib.vx_supports_unary(8, a, a) == 0                                               # GELU: not claimed
    gu = f32(pkg, [8192, 2, 1, 1])
    half = f32(pkg, [4096, 2, 1, 1])
    assert lib.vx_supports_glu(pkg.GLU_SWIGLU, half, half, half) == 1
    assert lib.vx_supports_glu(pkg.GLU_SWIGLU, gu, None, half) == 1
    assert lib.vx_supports_glu(pkg.GLU_SWIGLU, gu, None, gu) == 0
    assert lib.vx_supports_glu(1, half, half, half) == 0                                     # GEGLU: not claimed
    # CPY: F32/F16 both ways, equal element counts, any shapes
    assert lib.vx_supports_cpy(f32(pkg, [64, 2, 5, 2]), f16(pkg, [64, 2, 5, 2])) == 1
    assert lib.vx_supports_cpy(f32(pkg, [64, 2, 5, 2]), f32(pkg, [128, 10, 1, 1])) == 1
    assert lib.vx_supports_cpy(f32(pkg, [64, 2, 5, 2]), f32(pkg, [64, 2, 5, 1])) == 0
    assert lib.vx_supports_cpy(q8(pkg, [64, 2, 1, 1]), f32(pkg, [64, 2, 1, 1])) == 0
    # CONCAT: same type, equal outside the dim
    past, cur, both = f32(pkg, [64, 37, 2, 2]), f32(pkg, [64, 1, 2, 2]), f32(pkg, [64, 38, 2, 2])
    assert lib.vx_supports_concat(past, cur, both, 1) == 1
    assert lib.vx_supports_concat(past, cur, both, 0) == 0
    assert lib.vx_supports_concat(past, f16(pkg, [64, 1, 2, 2]), both, 1) == 0
    # a tree of CONCATs from its leaves: 2 to 8 sources whose shapes divide their slots, the slots filling the dimension
    import ctypes as C
    def many(srcs, extents, dim, dst):
        arr = (C.POINTER(pkg.VxTensor) * len(srcs))(*[C.pointer(t) for t in srcs])
        return lib.vx_supports_concat_many(arr, (C.c_int64 * len(srcs))(*extents), len(srcs), dim, dst)
    tok, four, two, seq = f32(pkg, [1024, 1, 8, 1]), f32(pkg, [1024, 4, 8, 1]), f32(pkg, [1024, 2, 8, 1]), f32(pkg, [1024, 14, 8, 1])
    row = f32(pkg, [1024, 1, 1, 1])
    assert many([tok, four, two, row, four, two], [1, 4, 2, 1, 4, 2], 1, seq) == 1           # (t + mu | cond | x | t, once per request | cond | x)
    assert many([tok, four, two, row, four, two], [1, 4, 2, 1, 4, 3], 1, seq) == 0           # slots must fill the dimension
    assert many([tok, four], [1, 13], 1, seq) == 0                                           # 13 is no multiple of 4
    assert many([seq], [14], 1, seq) == 0 and many([tok] * 9, [1] * 9, 1, f32(pkg, [1024, 9, 8, 1])) == 0
    assert many([tok, f16(pkg, [1024, 13, 8, 1])], [1, 13], 1, seq) == 0
    # SUM: dense F32 rows to a scalar
    assert lib.vx_supports_sum(a, one) == 1 and lib.vx_supports_sum(a, f32(pkg, [2, 1, 1, 1])) == 0
    permuted = D(pkg, pkg.F32, [5, 1024, 1, 1], [4096, 4, 20480, 20480])
    assert lib.vx_supports_sum(permuted, one) == 0
    # the ops around the stacks: masks (ARANGE, REPEAT, I32 -> F32 cast), embeddings (GET_ROWS), rounding, sin / cos
    def i32(ne):
        return D(pkg, pkg.I32, ne, [4, 4 * ne[0], 4 * ne[0] * ne[1], 4 * ne[0] * ne[1] * ne[2]])
    assert lib.vx_supports_cpy(i32([5, 1, 1, 1]), f32(pkg, [5, 1, 1, 1])) == 1
    assert lib.vx_supports_cpy(f32(pkg, [5, 1, 1, 1]), i32([5, 1, 1, 1])) == 1
    assert lib.vx_supports_cpy(i32([5, 1, 1, 1]), i32([1, 5, 1, 1])) == 1
    assert lib.vx_supports_cpy(i32([5, 1, 1, 1]), f16(pkg, [5, 1, 1, 1])) == 0              # ggml-cpu has no such copy either
    assert lib.vx_supports_arange(f32(pkg, [4096, 1, 1, 1])) == 1
    assert lib.vx_supports_arange(f16(pkg, [8, 1, 1, 1])) == 0
    assert lib.vx_supports_arange(D(pkg, pkg.F32, [8, 1, 1, 1], [8, 64, 64, 64])) == 0      # ggml-cpu asserts dense elements
    assert lib.vx_supports_repeat(f32(pkg, [4096, 1, 1, 1]), f32(pkg, [4096, 512, 1, 1])) == 1  # key positions over queries
    assert lib.vx_supports_repeat(f32(pkg, [1, 512, 1, 1]), f32(pkg, [4096, 512, 1, 1])) == 1   # query positions over keys
    assert lib.vx_supports_repeat(f32(pkg, [3, 1, 1, 1]), f32(pkg, [4096, 1, 1, 1])) == 0       # not a whole multiple
    assert lib.vx_supports_repeat(f32(pkg, [8, 1, 1, 1]), f16(pkg, [16, 1, 1, 1])) == 0
    vocab = 73448
    for table in (f32(pkg, [1024, vocab, 1, 1]), f16(pkg, [1024, vocab, 1, 1]), q8(pkg, [1024, vocab, 1, 1])):
        assert lib.vx_supports_get_rows(table, i32([7, 1, 1, 1]), f32(pkg, [1024, 7, 1, 1])) == 1
        assert lib.vx_supports_get_rows(table, i32([7, 1, 1, 1]), f32(pkg, [1024, 8, 1, 1])) == 0
        assert lib.vx_supports_get_rows(table, f32(pkg, [7, 1, 1, 1]), f32(pkg, [1024, 7, 1, 1])) == 0   # indices must be I32
        assert lib.vx_supports_get_rows(table, i32([7, 2, 1, 1]), f32(pkg, [1024, 7, 2, 1])) == 0        # one table matrix per index column
    assert lib.vx_supports_get_rows(i32([16, 9, 1, 1]), i32([3, 1, 1, 1]), i32([16, 3, 1, 1])) == 1
    assert lib.vx_supports_get_rows(i32([16, 9, 1, 1]), i32([3, 1, 1, 1]), f32(pkg, [16, 3, 1, 1])) == 0
    for op in (pkg.UNARY_FLOOR, pkg.UNARY_CEIL, pkg.UNARY_ROUND, pkg.UNARY_TRUNC, pkg.UNARY_SQR, pkg.UNARY_SQRT,
               pkg.UNARY_LOG, pkg.UNARY_SIN, pkg.UNARY_COS):
        assert lib.vx_supports_unary(op, a, a) == 1, op
    assert lib.vx_supports_unary(105, a, a) == 0 and lib.vx_supports_unary(17, a, a) == 0
    # nodes of a one-launch run: the tiny operators, tensors of at most 16384 elements
    v, sc1 = f32(pkg, [64, 2, 1, 1]), f32(pkg, [1, 1, 1, 1])
    seq = f32(pkg, [1024, 14, 1, 1])
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_MUL, v, v, v)) == 1
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_SUM, sc1, v)) == 1
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_REPEAT, v, sc1)) == 1
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_ARANGE, sc1)) == 1
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_CONCAT, seq, f32(pkg, [1024, 7, 1, 1]), f32(pkg, [1024, 7, 1, 1]), aux=1)) == 1
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_ADD, a, a, a)) == 0            # 30720 elements: its own launch
    assert lib.vx_supports_small_node(pkg.small_node(pkg.NODE_UNARY, v, v, aux=8)) == 0      # GELU is not claimed at all
    assert lib.vx_supports_small_node(pkg.small_node(12, v, v, v)) == 0
    # fused pairs
    w = f32(pkg, [1024, 1, 1, 1])
    assert lib.vx_supports_rms_norm_mul(a, w, a) == 1
    assert lib.vx_supports_rms_norm_mul(a, f32(pkg, [1024, 5, 1, 1]), a) == 0
    assert lib.vx_supports_fused_pair(a, a, a) == 1 and lib.vx_supports_fused_pair(a, w, a) == 0


def test_supports_truth_table_node_groups(pkg):
    """The one-launch groups of a decoder layer: which shapes the plugin may hand to them."""
    lib = pkg.lib()
    K, H, Hkv, Dh = 1024, 16, 2, 64
    wq, wk, wo = q8(pkg, [K, H * Dh, 1, 1]), q8(pkg, [K, Hkv * Dh, 1, 1]), q8(pkg, [K, K, 1, 1])
    wdown = q8(pkg, [4096, K, 1, 1])

    def acts(n, k=K):
        return f32(pkg, [k, n, 1, 1])

    # projection + scale + residual: every token count; beyond the streaming kernel's (16, tokens x rows <= 256 Ki, or 448
    # tokens of at most 1024 rows) and the K-cut shapes only into a dense destination with rows in whole 16-byte groups
    for n, want in ((1, 1), (16, 1), (17, 1), (256, 1), (257, 1), (449, 1), (65536, 1)):
        assert lib.vx_supports_mul_mat_scale_add(wo, acts(n), acts(n), acts(n)) == want, n
    strided = D(pkg, pkg.F32, [K, 449, 1, 1], [4, 4 * (K + 8), 4 * (K + 8) * 449, 4 * (K + 8) * 449])
    assert lib.vx_supports_mul_mat_scale_add(wo, acts(449), acts(449), strided) == 0
    strided = D(pkg, pkg.F32, [K, 448, 1, 1], [4, 4 * (K + 8), 4 * (K + 8) * 448, 4 * (K + 8) * 448])
    assert lib.vx_supports_mul_mat_scale_add(wo, acts(448), acts(448), strided) == 1
    assert lib.vx_supports_mul_mat_scale_add(wo, acts(14), acts(14), D(pkg, pkg.F32, [K, 14, 1, 1], [4, 4 * (K + 8), 4 * (K + 8) * 14, 4 * (K + 8) * 14])) == 1
    odd = q8(pkg, [K, 1002, 1, 1])
    assert lib.vx_supports_mul_mat_scale_add(odd, acts(500), f32(pkg, [1002, 500, 1, 1]), f32(pkg, [1002, 500, 1, 1])) == 0
    assert lib.vx_supports_mul_mat_scale_add(wdown, acts(14, 4096), acts(14), acts(14)) == 1      # 16 x 4096 halves of LDS
    # gate + up + GLU on the tiled kernel: f16 activations, 64 tokens or more, shapes the streaming kernel does not take, and
    # products that the tiled kernel walks with K whole (at least 64 tiles of 64 x 64 each)
    wgate = q8(pkg, [K, 4096, 1, 1])
    ffn = lambda n: f32(pkg, [4096, n, 1, 1])
    tiled = lib.vx_supports_mul_mat_swiglu_tiled
    assert tiled(wgate, wgate, acts(1024), ffn(1024), pkg.ACT_FLOAT) == 1 and tiled(wgate, wgate, acts(1024), ffn(1024), pkg.ACT_Q8) == 0
    assert tiled(wgate, wgate, acts(112), ffn(112), pkg.ACT_FLOAT) == 1                        # 8 requests x 14 tokens
    assert tiled(wgate, wgate, acts(14), ffn(14), pkg.ACT_FLOAT) == 0 and lib.vx_supports_mul_mat_swiglu(wgate, wgate, acts(14), ffn(14)) == 1
    small = q8(pkg, [K, 1024, 1, 1])
    assert tiled(small, small, acts(128), acts(128), pkg.ACT_FLOAT) == 0                       # 32 tiles: its K would be cut
    assert tiled(wgate, q8(pkg, [K, 2048, 1, 1]), acts(1024), ffn(1024), pkg.ACT_FLOAT) == 0   # matrices of different shapes
    # 64..256 tiles with K of 2048 or more: one product on its own is cut in two or four, the pair is not
    long_k = q8(pkg, [4096, 2048, 1, 1])
    pair_out = lambda n: f32(pkg, [2048, n, 1, 1])
    assert tiled(long_k, long_k, acts(128, 4096), pair_out(128), pkg.ACT_FLOAT) == 0           # 64 tiles
    assert tiled(long_k, long_k, acts(512, 4096), pair_out(512), pkg.ACT_FLOAT) == 0           # 256 tiles
    assert tiled(long_k, long_k, acts(576, 4096), pair_out(576), pkg.ACT_FLOAT) == 1           # 288 tiles: K whole
    assert lib.vx_supports_mul_mat_scale_add(wo, acts(2), acts(3), acts(2)) == 0                  # residual of another shape
    assert lib.vx_supports_mul_mat_scale_add(wo, acts(14), acts(1), acts(14)) == 1                # a bias row, repeated over the tokens
    assert lib.vx_supports_mul_mat_scale_add(q8(pkg, [64, K, 1, 1]), acts(2, 64), acts(1), acts(2)) == 1   # LocDiT's in_proj + bias
    assert lib.vx_supports_mul_mat_scale_add(f32(pkg, [K, K, 1, 1]), acts(2), acts(2), acts(2)) == 0   # F32 weights
    # the order in which a product's K blocks are summed depends on its shape alone; what the plugin compares before it
    # replaces one product over a row-fused matrix by products over its row ranges
    order = lib.vx_mul_mat_sum_order
    assert order(K, 2, 1280) == order(K, 2, 1024) == order(K, 2, 128) > 0          # decode: q, k, v ranges of qkv_proj
    assert order(K, 14, 1280) == order(K, 14, 1024) == order(K, 14, 128)           # LocDiT's 14-token pair
    assert order(K, 14, 8192) == order(K, 14, 4096)                                # gate_up_proj and its halves
    assert order(K, 14, 1024) != order(K, 14, 4096)                                # few rows spread the token work over more waves
    assert order(K, 14, 1024) != order(K, 2, 1024)
    # one chunk of tokens aims at 4 blocks per wave, several chunks (which multiply the work-groups) at 8; the 16 waves of
    # few-row products are for one chunk only
    assert order(K, 2, 1024) == order(K, 16, 4096) == 8 and order(K, 17, 4096) == 4 and order(K, 112, 1024) == 4 and order(K, 14, 1024) == 16
    assert order(4096, 2, 1024) == order(4096, 112, 1024) == 16
    assert order(K, 0, 1024) == 0 and order(33, 2, 1024) == 0
    # gate / up / SwiGLU: both matrices count as rows
    wg = q8(pkg, [K, 4096, 1, 1])
    ffn = lambda n: f32(pkg, [4096, n, 1, 1])
    for n, want in ((2, 1), (16, 1), (32, 1), (33, 0)):
        assert lib.vx_supports_mul_mat_swiglu(wg, wg, acts(n), ffn(n)) == want, n
    assert lib.vx_supports_mul_mat_swiglu(wg, q8(pkg, [K, 2048, 1, 1]), acts(2), ffn(2)) == 0
    # q/k/v + rope: NEOX over the whole head only; batch in dim 3 or flattened into the token dimension
    q_dst, k_dst = f32(pkg, [Dh, H, 1, 2]), f32(pkg, [Dh, Hkv, 1, 2])
    xb, vb = f32(pkg, [K, 1, 1, 2]), f32(pkg, [Hkv * Dh, 1, 1, 2])
    assert lib.vx_supports_qkv_proj_rope(wq, wk, wk, xb, q_dst, k_dst, vb, Dh, 2) == 1
    assert lib.vx_supports_qkv_proj_rope(wq, wk, wk, acts(2), q_dst, k_dst, f32(pkg, [Hkv * Dh, 2, 1, 1]), Dh, 2) == 1
    assert lib.vx_supports_qkv_proj_rope(wq, wk, wk, xb, q_dst, k_dst, vb, Dh, 0) == 0            # NORMAL pairing
    assert lib.vx_supports_qkv_proj_rope(wq, wk, wk, xb, q_dst, k_dst, vb, Dh // 2, 2) == 0       # partial rotation
    assert lib.vx_supports_qkv_proj_rope(wq, wk, wk, acts(3), q_dst, k_dst, vb, Dh, 2) == 0       # token counts disagree
    assert lib.vx_supports_qkv_proj_rope(wq, wk, f32(pkg, [K, Hkv * Dh, 1, 1]), xb, q_dst, k_dst, vb, Dh, 2) == 0
    # rms_norm in front: rows of at most 1024 floats, one weight row
    nw = f32(pkg, [K, 1, 1, 1])
    assert lib.vx_supports_norm_qkv_proj_rope(xb, nw, wq, wk, wk, q_dst, k_dst, vb, Dh, 2) == 1
    assert lib.vx_supports_norm_qkv_proj_rope(xb, f32(pkg, [K, 2, 1, 1]), wq, wk, wk, q_dst, k_dst, vb, Dh, 2) == 0
    assert lib.vx_supports_norm_mul_mat_swiglu(acts(2), nw, wg, wg, ffn(2)) == 1
    w2k = q8(pkg, [2048, 64, 1, 1])
    assert lib.vx_supports_norm_mul_mat_swiglu(acts(1, 2048), f32(pkg, [2048, 1, 1, 1]), w2k, w2k, f32(pkg, [64, 1, 1, 1])) == 0
    # cache write + ordering scalar: F32, decode-sized
    k_src, slot = f32(pkg, [Dh, Hkv, 1, 2]), D(pkg, pkg.F32, [Dh, Hkv, 1, 2], [4, 4 * Dh * 768, 4 * Dh, 4 * Dh * 768 * Hkv])
    attn = f32(pkg, [Dh, H, 1, 2])
    assert lib.vx_supports_kv_store_sync(k_src, slot, k_src, slot, attn, attn) == 1
    slot16 = D(pkg, pkg.F16, [Dh, Hkv, 1, 2], [2, 2 * Dh * 768, 2 * Dh, 2 * Dh * 768 * Hkv])
    assert lib.vx_supports_kv_store_sync(k_src, slot16, k_src, slot16, attn, attn) == 1                         # F16 cache: rounded on the way
    assert lib.vx_supports_kv_store_sync(k_src, D(pkg, pkg.F16, [Dh, Hkv, 1, 2], [2, 2 * Dh * 768, 2 * Dh, 2 * Dh * 768 * Hkv], 0x1002),
                                         k_src, slot, attn, attn) == 0                                            # slot not 8-byte aligned
    assert lib.vx_supports_kv_store_sync(f16(pkg, [Dh, Hkv, 1, 2]), slot16, k_src, slot, attn, attn) == 0       # F16 source
    big, mid = f32(pkg, [Dh, Hkv, 512, 2]), f32(pkg, [Dh, Hkv, 100, 2])
    assert lib.vx_supports_kv_store_sync(big, big, big, big, attn, attn) == 1                                     # a prefill's write: sums over 128 blocks
    assert lib.vx_supports_kv_store_sync(mid, mid, mid, mid, attn, attn) == 1                                     # a prompt's: one block's sum each
    assert lib.vx_supports_kv_store_sync(mid, mid, big, big, attn, attn) == 0                                     # one of each
    assert lib.vx_supports_kv_store_sync(big, big, mid, mid, attn, attn) == 0
    # attention over cached + current keys
    q = f32(pkg, [Dh, 1, H, 2])
    past = D(pkg, pkg.F32, [Dh, 640, Hkv, 2], [4, 4 * Dh, 4 * Dh * 768, 4 * Dh * 768 * Hkv])
    cur = D(pkg, pkg.F32, [Dh, 1, Hkv, 2], [4, 4 * Dh * Hkv, 4 * Dh, 4 * Dh * Hkv])
    assert lib.vx_supports_flash_attn_ext_kv2(q, past, cur, past, cur, None, attn) == 1
    assert lib.vx_supports_flash_attn_ext_kv2(q, past, f16(pkg, [Dh, 1, Hkv, 2]), past, cur, None, attn) == 0   # segment types differ
    assert lib.vx_supports_flash_attn_ext_kv2(q, past, f32(pkg, [Dh, 1, 4, 2]), past, cur, None, attn) == 0      # head counts differ
    assert lib.vx_supports_flash_attn_ext_kv2_store(q, past, cur, past, cur, None, k_src, slot, k_src, slot, attn) == 1
    short = D(pkg, pkg.F32, [Dh, 100, Hkv, 2], [4, 4 * Dh, 4 * Dh * 768, 4 * Dh * 768 * Hkv])
    assert lib.vx_supports_flash_attn_ext_kv2(q, short, cur, short, cur, None, attn) == 1
    assert lib.vx_supports_flash_attn_ext_kv2_store(q, short, cur, short, cur, None, k_src, slot, k_src, slot, attn) == 0  # no merge kernel to ride on
    # a prefill's attention block: the cache write in front of the attention, the o projection behind it
    T = 4096
    qp, kp = f32(pkg, [Dh, T, H, 16]), f32(pkg, [Dh, T, Hkv, 16])
    ks_, slotp = f32(pkg, [Dh, Hkv, T, 16]), D(pkg, pkg.F16, [Dh, Hkv, T, 16], [2, 2 * Dh * (T + 8), 2 * Dh, 2 * Dh * (T + 8) * Hkv])
    outp = f32(pkg, [Dh, H, T, 16])
    assert lib.vx_supports_flash_attn_ext_store(qp, kp, kp, None, ks_, slotp, ks_, slotp, outp, 0.0) == 1
    assert lib.vx_supports_flash_attn_ext_store(qp, kp, kp, None, ks_, slotp, ks_, slotp, outp, 30.0) == 0          # soft cap: the general kernel
    assert lib.vx_supports_flash_attn_ext_store(q, f32(pkg, [Dh, 1, Hkv, 2]), f32(pkg, [Dh, 1, Hkv, 2]), None, k_src, slot, k_src, slot, attn, 0.0) == 0  # decode-sized
    flat, hid = f32(pkg, [K, 16 * T, 1, 1]), f32(pkg, [K, 16 * T, 1, 1])
    assert lib.vx_supports_flash_attn_ext_store_proj(qp, kp, kp, None, ks_, slotp, ks_, slotp, flat, wo, hid, hid, 0.0, pkg.ACT_FLOAT) == 1
    assert lib.vx_supports_flash_attn_ext_store_proj(qp, kp, kp, None, ks_, slotp, ks_, slotp, flat, wo, hid, hid, 0.0, pkg.ACT_Q8) == 0
    assert lib.vx_supports_flash_attn_ext_store_proj(qp, kp, kp, None, ks_, slotp, ks_, slotp, f32(pkg, [K, T, 16, 1]), wo,
                                                     f32(pkg, [K, T, 16, 1]), f32(pkg, [K, T, 16, 1]), 0.0, pkg.ACT_FLOAT) == 1   # as a batch
    assert lib.vx_supports_flash_attn_ext_store_proj(qp, kp, kp, None, ks_, slotp, ks_, slotp, f32(pkg, [K, 8 * T, 2, 1]), wo,
                                                     f32(pkg, [K, 8 * T, 2, 1]), f32(pkg, [K, 8 * T, 2, 1]), 0.0, pkg.ACT_FLOAT) == 0  # neither layout
    # k and v alone with k's rotation: while both are the streaming kernel's shapes
    for n, want in ((300, 1), (2048, 1), (2049, 0)):
        xn = f32(pkg, [K, n, 1, 1])
        assert lib.vx_supports_kv_proj_rope(wk, wk, xn, f32(pkg, [Dh, Hkv, n, 1]), f32(pkg, [Hkv * Dh, n, 1, 1]), Dh, 2) == want, n
    assert lib.vx_supports_kv_proj_rope(wk, wk, f32(pkg, [K, 300, 1, 1]), f32(pkg, [Dh, Hkv, 300, 1]), f32(pkg, [Hkv * Dh, 300, 1, 1]), Dh, 0) == 0
    # null operands are refused, not dereferenced
    assert lib.vx_supports_flash_attn_ext_store(qp, kp, kp, None, None, slotp, ks_, slotp, outp, 0.0) == 0
    assert lib.vx_supports_flash_attn_ext_store_proj(qp, kp, kp, None, ks_, slotp, ks_, slotp, flat, None, hid, hid, 0.0, pkg.ACT_FLOAT) == 0
    assert lib.vx_supports_kv_proj_rope(wk, None, xb, k_dst, vb, Dh, 2) == 0
    assert lib.vx_supports_flash_attn_ext_kv2(q, past, None, past, cur, None, attn) == 0
    assert lib.vx_supports_mul_mat_scale_add(wo, acts(2), None, acts(2)) == 0
    assert lib.vx_supports_kv_store_sync(k_src, slot, None, slot, attn, attn) == 0


def test_ops_validate_before_touching_the_device(pkg):
    """Contract violations are reported by status + message; nothing is launched."""
    lib = pkg.lib()
    x = f32(pkg, [64, 16, 5, 1])
    assert lib.vx_rms_norm(x, x, -1.0, None) == 3                       # VX_ERR_INVALID: eps < 0
    assert lib.vx_rms_norm(f16(pkg, [64, 1, 1, 1]), f16(pkg, [64, 1, 1, 1]), 1e-5, None) == 2  # UNSUPPORTED
    assert b"F32" in lib.vx_last_error()
    assert lib.vx_flash_attn_ext(None, None, None, None, None, None, 1.0, 0.0, 0.0, None) == 3
    q, dst = f32(pkg, [64, 1, 16, 2]), f32(pkg, [64, 16, 1, 2])
    k = f16(pkg, [64, 4096, 2, 2])
    assert lib.vx_flash_attn_ext(q, k, k, None, None, dst, 0.125, 8.0, 0.0, None) == 3  # max_bias needs a mask
    assert lib.vx_mul_mat(q8(pkg, [1024, 8, 1, 1]), f32(pkg, [1024, 2, 1, 1]), f32(pkg, [8, 2, 1, 1]), 7, None) == 3


def test_kv_views_match_reference_layout(pkg):
    """MiniCPMKVCache view shapes (reference tests/test_minicpm.cpp:775-809: cache (2 layers,
    2 kv heads, max_length 16, head_dim 8); get_k(seq 4) -> [8,4,2]; get_k_slot(3) -> [8,2,1];
    get_v_batch(5, 2) -> [8,2,2]) and the oracle's stride/offset formulas."""
    lib, orc = pkg.lib(), reflib.load_oracle()
    cache = pkg.make_desc(pkg.F32, [8, 16, 2, 1], [4, 32, 512, 1024], 0x10000)
    v = pkg.VxTensor()
    assert lib.vx_kv_read_view(cache, 4, v) == 0 and list(v.ne)[:3] == [8, 4, 2]
    assert lib.vx_kv_read_view(cache, 7, v) == 0 and list(v.ne)[:3] == [8, 7, 2]
    assert lib.vx_kv_write_view(cache, 3, 1, v) == 0 and list(v.ne)[:3] == [8, 2, 1]
    assert lib.vx_kv_write_view(cache, 5, 2, v) == 0 and list(v.ne)[:3] == [8, 2, 2]
    ne, nb, off = (C.c_int64 * 3)(), (C.c_uint64 * 3)(), C.c_uint64()
    orc.orc_kv_write_view(8, 16, 2, 4, 5, 2, ne, nb, C.byref(off))
    assert list(v.nb)[:3] == list(nb) and v.data - 0x10000 == off.value == 5 * 32
    assert lib.vx_kv_read_view(cache, 17, v) == 3 and lib.vx_kv_write_view(cache, 15, 2, v) == 3


def test_plugin_on_a_gpuless_host(pkg, ref):
    """ggml's loader must reject the plugin cleanly (score 0) when no gfx950 device exists,
    leaving ggml-cpu as the only device."""
    if have_gpu(pkg):
        pytest.skip("a GPU is present")
    if not os.path.exists(pkg.PLUGIN_PATH):
        pytest.skip("plugin not built")
    plug = C.CDLL(pkg.PLUGIN_PATH)
    assert plug.ggml_backend_score() == 0
    assert ref.rh_load_plugin(pkg.PLUGIN_PATH.encode()) != 0
    names = [ref.rh_device_name(i).decode() for i in range(ref.rh_device_count())]
    assert names == ["CPU"]


def test_workspace_growth_policy(tmp_path):
    """The per-stream workspace never frees or moves a block it has handed out (a captured HIP graph keeps the
    address), refuses to grow during a capture, and releases everything with the stream: the policy header,
    compiled for the host with a counting allocator."""
    import subprocess
    exe = str(tmp_path / "ws_policy_check")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-o", exe, os.path.join(ROOT, "tests", "ws_policy_check.cpp")])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr


def test_weight_placement_policy(pkg):
    """Which tensors of a VoxCPM model file the plugin's placement helper sends to device memory and which to pinned
    host memory, by the reference's GGUF tensor names (src/minicpm.cpp:522-570, src/locdit.cpp, src/audio-vae.cpp:164-303):
    what the claimed operators consume goes to the device, the AudioVAE's weights stay with ggml-cpu."""
    import ctypes
    if not os.path.exists(pkg.PLUGIN_PATH):
        pytest.skip("the ggml plugin was not built")
    # the plugin resolves ggml's symbols from the process, as every dynamically loaded ggml backend does
    ref_dir = reflib.ref_dir()
    if not os.path.exists(os.path.join(ref_dir, "libggml-ref.so")):
        pytest.skip("oracle/_ref was not prebuilt")
    ctypes.CDLL(os.path.join(ref_dir, "libggml-ref.so"), mode=ctypes.RTLD_GLOBAL)
    plugin = ctypes.CDLL(pkg.PLUGIN_PATH)
    on_device = lambda n: plugin.ggml_backend_gfx950_weight_on_device(n.encode())
    for name in ("token_embd.weight", "output_norm.weight", "blk.0.attn_q.weight", "blk.23.ffn_down.weight", "blk.3.attn_norm.weight",
                 "residual_lm.blk.5.attn_k.weight", "residual_lm.output_norm.weight", "locenc.in_proj.weight", "locenc.blk.0.ffn_up.weight",
                 "locdit.in_proj.weight", "locdit.cond_proj.bias", "locdit.time_mlp.linear_1.weight", "locdit.blk.3.attn_v.weight",
                 "fsq.in_proj.weight", "stop.stop_proj.weight", "stop.stop_head.weight"):
        assert on_device(name) == 1, name
    for name in ("audio_vae.encoder.block.0.weight", "audio_vae.encoder.fc_mu.weight", "audio_vae.encoder.fc_mu.bias",
                 "audio_vae.decoder.model.0.weight", "audio_vae.decoder.model.1.block.0.block.1.alpha", "audio_vae.decoder.model.7.bias"):
        assert on_device(name) == 0, name
    # every helper is also handed out by name, the way ggml exposes backend-specific functions
    reg = plugin.ggml_backend_gfx950_reg
    reg.restype = ctypes.c_void_p
    ggml = ctypes.CDLL(os.path.join(ref_dir, "libggml-ref.so"))
    ggml.ggml_backend_reg_get_proc_address.restype = ctypes.c_void_p
    ggml.ggml_backend_reg_get_proc_address.argtypes = [ctypes.c_void_p, ctypes.c_char_p]
    for fn in ("ggml_backend_gfx950_weight_on_device", "ggml_backend_gfx950_alloc_weights", "ggml_backend_gfx950_last_launches"):
        assert ggml.ggml_backend_reg_get_proc_address(reg(), fn.encode())
    assert not ggml.ggml_backend_reg_get_proc_address(reg(), b"no_such_function")


def test_index_division_by_reciprocal_is_exact():
    """The attention kernels divide small indices (column / heads per group, grid z / KV heads) as
    (int) ((x + 0.5f) * (1.0f / d)) in single precision; the matrix kernels divide a unit number by the units per row
    the same way.  Exact for every 0 <= x < 2^22 (the kernels refuse larger launches): checked here over the whole range
    for the divisors the path meets and for awkward ones, in the same float32 arithmetic."""
    x = np.arange(1 << 22, dtype=np.int64)
    xf = x.astype(np.float32) + np.float32(0.5)
    for d in (1, 2, 3, 5, 6, 7, 8, 12, 16, 24, 40, 64, 96, 127, 128, 512, 1000, 4099):
        inv = np.float32(1.0) / np.float32(d)
        got = (xf * inv).astype(np.int64)   # float32 product, truncated like the kernel's conversion
        assert np.array_equal(got, x // d), d


def test_row_rotations_reproduce_the_xor_butterfly():
    """A wave sum's steps 32, 16, 8, 4, 2, 1: the kernels take the last four as rotations within rows of 16 lanes
    (lane i reads lane (i + s) mod 16 of its row) instead of the xor partner i ^ s.  The same bits: when step s is reached
    the values repeat every 2 s lanes.  Simulated here in float64 and float32 on random and on badly conditioned values."""
    rng = np.random.default_rng(7)
    lanes = np.arange(64)
    for dtype in (np.float64, np.float32):
        for trial in range(50):
            v = rng.standard_normal(64).astype(dtype)
            if trial % 5 == 0:
                v = (v * dtype(10.0) ** rng.integers(-6, 7, 64).astype(dtype)).astype(dtype)
            a = v.copy()
            for s in (32, 16, 8, 4, 2, 1):
                a = (a + a[lanes ^ s]).astype(dtype)
            b = v.copy()
            for s in (32, 16):
                b = (b + b[lanes ^ s]).astype(dtype)
            for s in (8, 4, 2, 1):
                b = (b + b[(lanes & ~15) | ((lanes + s) & 15)]).astype(dtype)
            assert np.array_equal(a.view(np.uint8), b.view(np.uint8)), (dtype, trial)
            assert len(set(a.tolist())) == 1   # every lane holds the same total


def test_hot_kernels_do_not_spill():
    """The build keeps every kernel's resource remarks beside its object file.  The kernels on the timed paths must not
    use scratch memory: a few spilled registers cost the 128 x 128 GEMM tile a quarter of its speed once, and no parity
    test notices that.  (The F32-cache variants of the wave attention kernel do spill: they are listed, so that a new
    entry shows.)"""
    import glob, os, re
    files = sorted(glob.glob(os.path.join(os.path.dirname(__file__), "..", "voxcpm.cpp_amd", "lib", "obj", "*.resources.txt")))
    if not files:
        pytest.skip("no resource remarks: the library was not built on this machine")
    scratch = {}
    for f in files:
        text = open(f).read()
        names = re.findall(r"Function Name: (\S+)", text)
        sizes = re.findall(r"ScratchSize \[bytes/lane\]: (\d+)", text)
        assert len(names) == len(sizes), f
        scratch.update({n: int(s) for n, s in zip(names, sizes)})
    assert len(scratch) > 250
    hot = [r"gemm_q8t_kernel", r"qt_weights_kernel", r"qt_acts_kernel", r"qt_acts_norm_kernel", r"qt_rope_table_kernel", r"rope_heads_kernel", r"kv_sync_add1_kernel", r"kv_sync_scalar_kernel", r"kv_store_mid_kernel", "kv_sync_scalar_kernel", r"fattn_dec64_kernel", r"gemm_lds_kernel", r"gemv_dma_kernel", r"gemv_kernel", r"mm_kernel", r"mm_splitk_reduce_kernel", r"fattn_merge_kernel",
           r"fattn_cols16_kernelILi64ELb0", r"pf_kernel", r"small_graph_dense_kernel", r"small_graph_kernel", r"rms_norm_kernel",
           r"rope_kernel", r"concat_many_kernel"]
    known = [r"fattn_cols16_kernelILi(64|128)ELb1", r"fattn_cols16_kernelILi128ELb0ELb1ELb[01]ELi1", r"kv_store_sync_kernel",
             r"gemm128_kernelILi0ELb1ELb1E",
             r"gemm_lds_kernelILi0ELb0ELi4ELi2ELi2ELi4ELb1E"]  # gate + up with the GLU epilogue, 128 x 128 tile: 5 registers, one reload a round
    for name, size in scratch.items():
        if any(re.search(h, name) for h in hot) and not any(re.search(k, name) for k in known):
            assert size == 0, (name, size)
    for name, size in scratch.items():
        if size:
            assert any(re.search(k, name) for k in known), (name, size)
