"""vx_flash_attn_ext_static -- the attention entry point that allocates nothing -- against
vx_flash_attn_ext on the same inputs, through the C ABI.

Both calls take the same key-range kernels for these decode-sized shapes, so the results must be
bit-identical (tighter than the operator's 2e-3 bar against ggml-cpu, which the oracle check of the
first call also applies).  Two calls in a row share the library's fixed scratch array; the second is
smaller, so any partial it failed to overwrite would be a leftover of the first.
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


def make(B, Hq, Hkv, D, L, n_q, tag, kv_dtype=np.float16):
    q = rng("noalloc", tag, "q").standard_normal((B, Hq, n_q, D)).astype(np.float32)
    k = rng("noalloc", tag, "k").standard_normal((B, Hkv, L, D)).astype(kv_dtype)
    v = rng("noalloc", tag, "v").standard_normal((B, Hkv, L, D)).astype(kv_dtype)
    return q, k, v


def test_static_scratch_matches_the_allocating_call(gpu, oracle):
    import torch
    cases = [  # (B, Hq, Hkv, D, L, n_q): the second call is smaller than the first in every respect
        (16, 16, 2, 64, 8192, 1),
        (2, 16, 2, 64, 700, 1),
    ]
    outs = []
    for i, (B, Hq, Hkv, D, L, n_q) in enumerate(cases):
        say(f"no-alloc attention call {i}: B={B} Hq={Hq} Hkv={Hkv} D={D} L={L} n_q={n_q}")
        q, k, v = make(B, Hq, Hkv, D, L, n_q, i)
        tq, tk, tv = (torch.from_numpy(x).cuda() for x in (q, k, v))
        want = gpu.flash_attn_ext(tq, tk, tv, None, 0.125)
        got = torch.empty_like(want)
        torch.cuda.synchronize()
        before = torch.cuda.mem_get_info()[0]
        gpu.flash_attn_ext_static(tq, tk, tv, None, 0.125, out=got)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before, "the call changed the amount of free device memory"
        assert torch.equal(got, want), float((got - want).abs().max())
        outs.append((q, k, v, got.cpu().numpy()))
    # the smaller call against the oracle (the operator's own bar)
    q, k, v, got = outs[1]
    B, Hq, n_q, D = q.shape
    want = np.zeros((B, n_q, Hq, D), np.float32)
    rc = oracle.orc_flash_attn_ext(reflib.desc(q), reflib.desc(k.astype(np.float32)), reflib.desc(v.astype(np.float32)), None, None,
                                   reflib.desc(want), 0.125, 0.0, 0.0, 1, 1)
    assert rc == 0
    assert np.abs(got - want).max() <= 2e-3


def test_static_scratch_with_mask_and_f32_cache(gpu):
    """LocDiT-sized masked attention and an F32 cache: same kernels as the allocating call, same bits."""
    import torch
    say("no-alloc attention: masked 14-token sequences, then an F32 cache")
    q, k, v = make(16, 16, 16, 64, 14, 14, "locdit")
    mask = np.where(rng("noalloc", "mask").random((14, 14)) < 0.3, -np.inf, 0.0).astype(np.float16)
    mask[np.arange(14), np.arange(14)] = 0
    tq, tk, tv, tm = (torch.from_numpy(x).cuda() for x in (q, k, v, mask))
    want = gpu.flash_attn_ext(tq, tk, tv, tm, 0.125)
    got = gpu.flash_attn_ext_static(tq, tk, tv, tm, 0.125)
    assert torch.equal(got, want)
    q, k, v = make(2, 16, 2, 64, 1500, 1, "f32", np.float32)
    tq, tk, tv = (torch.from_numpy(x).cuda() for x in (q, k, v))
    want = gpu.flash_attn_ext(tq, tk, tv, None, 0.125)
    got = gpu.flash_attn_ext_static(tq, tk, tv, None, 0.125)
    assert torch.equal(got, want)


def test_static_scratch_refuses_what_does_not_fit(gpu):
    """A shape whose partials exceed the fixed array is refused before anything is launched.

    The largest partials come from the largest number of sixteen-column tiles that is still cut into key ranges: one
    less than the library's four waves per compute unit, cut in two.  The shape is therefore derived from the device's
    compute-unit count (1023 tiles on 256 units: 2046 partial blocks of 8 KiB and their maxima and sums, more than the
    16 MiB array).  The VX_FA_* variables move those thresholds and are read once per process: with any of them set the
    test has no shape to offer."""
    import ctypes as C
    import os
    import torch
    moved = [n for n in ("VX_FA_WAVES_PER_CU", "VX_FA_MAX_SPLITS", "VX_FA_MIN_CHUNK") if os.environ.get(n)]
    if moved:
        pytest.skip(f"{moved} change how many key ranges a call is cut into")
    lib = gpu.lib()
    cus = C.c_int(0)
    assert lib.vx_device_info(0, None, 0, None, None, C.byref(cus)) == 0
    D, L = 128, 512
    tiles = 4 * cus.value - 1
    need = 2 * tiles * 16 * (D + 2) * 4
    say(f"no-alloc attention: oversized request ({tiles} tiles in two key ranges on {cus.value} compute units: {need} bytes)")
    if need <= 16 * 1024 * 1024:
        pytest.skip(f"no decode shape of head size {D} exceeds the fixed array on a device with {cus.value} compute units")
    B, Hkv = tiles, 1
    q = torch.zeros((B, Hkv, 1, D), device="cuda")
    k = torch.zeros((B, Hkv, L, D), dtype=torch.float16, device="cuda")
    out = torch.full((B, 1, Hkv, D), 7.0, device="cuda")
    rc = lib.vx_flash_attn_ext_static(gpu.desc(q), gpu.desc(k), gpu.desc(k), None, None, gpu.desc(out), 0.1, 0.0, 0.0,
                                      torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert rc == 2, rc  # VX_ERR_UNSUPPORTED
    assert b"fixed scratch" in lib.vx_last_error()
    assert float(out.min()) == 7.0  # untouched
    got = gpu.flash_attn_ext(q, k, k, None, 0.1)  # the allocating call takes it
    assert float(got.abs().max()) == 0.0
