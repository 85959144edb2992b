#!/usr/bin/env python3
"""Writes tests/golden/ggml_cpu_golden.npz: outputs of the REFERENCE's own ggml-cpu (built from
the reference checkout into oracle/_ref by oracle/Makefile) on small seeded inputs, one entry
per operator of the hot path.  Inputs are regenerated from the seeds by the tests; only the
outputs (and Q8_0 bytes) are stored.  Run here, where the reference checkout is; the fixture
is what lets the oracle be checked on machines that have neither the checkout nor oracle/_ref.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import reflib  # noqa: E402
from reflib import rng  # noqa: E402


def inputs():
    """Seeded inputs shared by this script and tests/test_oracle.py."""
    d = {}
    d["rms_x"] = rng("g", "rms").standard_normal((3, 1024)).astype(np.float32)
    d["rope_x"] = rng("g", "rope").standard_normal((1, 6, 4, 64)).astype(np.float32)
    d["rope_pos"] = np.array([0, 1, 17, 255, 4095, 8191], np.int32)
    d["rope_ff"] = (1.0 + rng("g", "ff").random(32)).astype(np.float32)
    d["sm_x"] = rng("g", "sm").standard_normal((1, 4, 3, 50)).astype(np.float32)
    d["sm_mask"] = rng("g", "smm").standard_normal((1, 1, 3, 50)).astype(np.float16)
    d["w"] = (rng("g", "w").standard_normal((48, 256)) * 0.02).astype(np.float32)
    d["x"] = rng("g", "x").standard_normal((5, 256)).astype(np.float32)
    d["q_pre"] = rng("g", "q1").standard_normal((1, 16, 70, 64)).astype(np.float32)
    d["k_pre"] = rng("g", "k1").standard_normal((1, 2, 70, 64)).astype(np.float16)
    d["v_pre"] = rng("g", "v1").standard_normal((1, 2, 70, 64)).astype(np.float16)
    d["q_dec"] = rng("g", "q2").standard_normal((1, 16, 1, 64)).astype(np.float32)
    d["k_dec"] = rng("g", "k2").standard_normal((1, 2, 600, 64)).astype(np.float16)
    d["v_dec"] = rng("g", "v2").standard_normal((1, 2, 600, 64)).astype(np.float16)
    return d


def main():
    ref = reflib.load_ref()
    assert ref is not None, "oracle/_ref is not built: make -C oracle ref"
    assert ref.rh_use_device(b"CPU", 4, 0) == 0
    d = inputs()
    out = {}
    out["rms"] = reflib.ref_rms_norm(d["rms_x"], 1e-5)
    out["rope_neox"] = reflib.ref_rope(d["rope_x"], d["rope_pos"], d["rope_ff"], 64, 2)
    out["rope_normal"] = reflib.ref_rope(d["rope_x"], d["rope_pos"], None, 64, 0)
    out["soft_max"] = reflib.ref_soft_max(d["sm_x"], d["sm_mask"], 0.25, 8.0)
    import ctypes as C
    wq = np.empty((48, 256 // 32 * 34), np.uint8)
    ref.rh_quantize_q8_0(reflib.ptr(d["w"], C.c_float), wq.ctypes.data, 48, 256)
    out["w_q8_0"] = wq
    deq = np.empty((48, 256), np.float32)
    ref.rh_dequantize_q8_0(wq.ctypes.data, reflib.ptr(deq, C.c_float), 48 * 256)
    out["w_dequant"] = deq
    xq = np.empty((5, 256 // 32 * 34), np.uint8)
    for i in range(5):
        ref.rh_quantize_q8_0_cpu(reflib.ptr(d["x"][i], C.c_float), xq[i].ctypes.data, 256)
    out["x_q8_0_cpu"] = xq
    out["mul_mat_q8_0"] = reflib.ref_mul_mat(wq, d["x"], 256)
    out["mul_mat_f16"] = reflib.ref_mul_mat(d["w"].astype(np.float16), d["x"])
    mask = reflib.causal_mask(70, 70)
    out["fa_prefill_f16"] = reflib.ref_fa(d["q_pre"], d["k_pre"], d["v_pre"], mask)  # tiled path
    out["fa_decode_f32kv"] = reflib.ref_fa(d["q_dec"], d["k_dec"].astype(np.float32), d["v_dec"].astype(np.float32))
    out["fa_decode_f16kv"] = reflib.ref_fa(d["q_dec"], d["k_dec"], d["v_dec"])  # F16 accumulator
    path = os.path.join(HERE, "ggml_cpu_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
