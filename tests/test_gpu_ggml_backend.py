"""The drop-in boundary on the GPU: the ggml backend plugin (libggml-gfx950.so) driven by the
REFERENCE's own ggml -- its registry loader, allocator, buffer/stream vtables and its own
any-backend-vs-CPU operator test (ggml/tests/test-backend-ops.cpp) -- all built from the
reference checkout into oracle/_ref.  Skipped where oracle/_ref was not prebuilt."""
import ctypes as C
import os
import re
import subprocess
import sys

import numpy as np
import pytest

import reflib
from reflib import nmse, rng

pytestmark = pytest.mark.gpu

OPS = ["RMS_NORM", "ROPE", "SOFT_MAX", "FLASH_ATTN_EXT", "MUL_MAT",
       # the glue of a decoder layer
       "ADD", "SUB", "MUL", "DIV", "ADD1", "SCALE", "CPY", "CONT", "DUP", "CONCAT", "SUM", "SILU", "SWIGLU",
       # the ops around the stacks: masks, token embeddings, the timestep embedding, FSQ's rounding
       "ARANGE", "REPEAT", "GET_ROWS", "SIN", "COS", "SQR", "SQRT", "LOG", "ROUND", "FLOOR", "CEIL", "TRUNC",
       "STEP", "ABS", "EXP", "TANH"]


def plugin_path(pkg):
    if not os.path.exists(pkg.PLUGIN_PATH):
        pytest.skip("libggml-gfx950.so was not prebuilt (needs the reference's ggml headers)")
    return pkg.PLUGIN_PATH


@pytest.mark.parametrize("op", OPS)
def test_ggml_test_backend_ops(gpu, ref, op):
    """ggml's own op test: every case of `op` the backend claims must pass against ggml-cpu."""
    exe = os.path.join(reflib.ref_dir(), "test-backend-ops")
    if not os.path.exists(exe):
        pytest.skip("test-backend-ops was not prebuilt")
    env = dict(os.environ, GGML_BACKEND_PATH=plugin_path(gpu))
    print(f"test-backend-ops test -b GFX950_0 -o {op}", flush=True)
    p = subprocess.run([exe, "test", "-b", "GFX950_0", "-o", op], env=env, capture_output=True, text=True, timeout=600)
    out = p.stdout + p.stderr
    m = re.search(r"(\d+)/(\d+) tests passed", out)
    assert m, out[-2000:]
    passed, total = int(m.group(1)), int(m.group(2))
    print(f"   {passed}/{total} supported cases passed, {out.count('not supported')} not claimed", flush=True)
    assert p.returncode == 0 and passed == total and total > 0, out[-3000:]


def test_plugin_through_ggml_vtables(gpu, ref):
    """Load the plugin through ggml's registry in this process, run each claimed op on device
    GFX950_0 via ggml_backend_alloc_ctx_tensors / tensor_set / graph_compute / tensor_get and
    compare with the same graph on ggml-cpu."""
    assert ref.rh_load_plugin(plugin_path(gpu).encode()) == 0
    names = [ref.rh_device_name(i).decode() for i in range(ref.rh_device_count())]
    print("devices:", names, flush=True)
    assert "GFX950_0" in names and "CPU" in names

    def both(fn):
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        a = fn()
        assert ref.rh_use_device(b"GFX950_0", 0, 0) == 0
        b = fn()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return a, b

    x = rng("plug", "x").standard_normal((4, 1024)).astype(np.float32)
    a, b = both(lambda: reflib.ref_rms_norm(x, 1e-5))
    assert np.abs(a - b).max() <= 1e-6

    xr = rng("plug", "r").standard_normal((1, 5, 16, 64)).astype(np.float32)
    pos = np.arange(100, 105, dtype=np.int32)
    ff = (1 + rng("plug", "ff").random(32)).astype(np.float32)
    a, b = both(lambda: reflib.ref_rope(xr, pos, ff, 64, 2))
    assert np.abs(a - b).max() <= 2e-5

    # attention on the permuted / cache views attention_forward builds
    T, maxlen = 33, 64
    qb = rng("plug", "q").standard_normal((1, T, 16, 64)).astype(np.float32)
    q = qb.transpose(0, 2, 1, 3)
    ck = rng("plug", "k").standard_normal((1, 2, maxlen, 64)).astype(np.float32)
    cv = rng("plug", "v").standard_normal((1, 2, maxlen, 64)).astype(np.float32)
    mask = reflib.causal_mask(T, T)
    a, b = both(lambda: reflib.ref_fa(q, ck[:, :, :T], cv[:, :, :T], mask))
    print("   attention vs ggml-cpu max-abs", np.abs(a - b).max(), flush=True)
    assert np.abs(a - b).max() <= 2e-3

    w = (rng("plug", "w").standard_normal((256, 1024)) * 0.02).astype(np.float32)
    wq = reflib.quantize_q8_0(w)
    xx = rng("plug", "xx").standard_normal((3, 1024)).astype(np.float32)
    a, b = both(lambda: reflib.ref_mul_mat(wq, xx, 1024))
    print("   Q8_0 mul_mat vs ggml-cpu nmse", nmse(a, b), flush=True)
    assert nmse(a, b) <= 5e-4
