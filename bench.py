#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

Prints ONE JSON line.  The default workload is BASELINE config 2: backbone-shaped decode
attention -- 24 layers x GQA attention (16 Q / 2 KV heads, head_dim 64), batch 2, one new
token per step, f16 KV cache of length 4096.  A step is one pass over the 24 layers (24
calls of vx_flash_attn_ext, each on its own layer's resident cache); `value` is the
algorithmic KV bytes of a step divided by its wall time, inputs already in HBM.

The same line carries, under "others", shorter measurements of the other BASELINE shapes
(other KV lengths, the batch-16 / 8192-key decode, prefill attention, LocDiT attention,
the Q8_0 projections), a `roofline` object for the dominant kernel of the headline
workload and a `cpu_baseline` object: the reference's own ggml-cpu (oracle/_ref) timed on
this machine's host cores on one layer of the same workload.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
MFMA_F16_PEAK_TFLOPS = 2500.0  # dense f16/bf16 MFMA, published

HQ, HKV, D, LAYERS = 16, 2, 64, 24

# (batch, KV length) -> HBM bytes per vx_flash_attn_ext call, measured with hardware counters
# (see --calibrate-copy); algorithmic bytes of the same call: kv_bytes(2, 4096) = 4194304
MEASURED_TRAFFIC_BYTES = {(2, 4096): 5654 * 1024}


def kv_bytes(batch, length, es=2):
    """algorithmic HBM bytes of one decode attention launch: every K and V element once"""
    return 2 * batch * HKV * length * D * es


class Timer:
    """HIP events on torch's current stream (the stream every vx_* call is enqueued on)."""

    def __init__(self):
        import torch
        self.torch = torch
        self.e0 = torch.cuda.Event(enable_timing=True)
        self.e1 = torch.cuda.Event(enable_timing=True)

    def run(self, fn, iters, warmup=3):
        for _ in range(warmup):
            fn()
        self.torch.cuda.synchronize()
        self.e0.record()
        for _ in range(iters):
            fn()
        self.e1.record()
        self.torch.cuda.synchronize()
        return self.e0.elapsed_time(self.e1) * 1e-3 / iters  # seconds per call


def graphed(fn, stream):
    """Capture fn's launches (all on `stream`) into a HIP graph; returns the replay callable.
    fn runs eagerly first so that the library's per-stream scratch exists before capture."""
    import torch
    with torch.cuda.stream(stream):
        fn()
        fn()
    stream.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=stream):
        fn()
    return g.replay


def decode_attn_setup(pkg, batch, length, layers):
    import torch
    g = torch.Generator(device="cuda").manual_seed(1234 + length)
    caches = []
    for _ in range(layers):
        k = torch.randn((batch, HKV, length, D), generator=g, device="cuda", dtype=torch.float32).half()
        v = torch.randn((batch, HKV, length, D), generator=g, device="cuda", dtype=torch.float32).half()
        caches.append((k, v))
    q = torch.randn((batch, HQ, 1, D), generator=g, device="cuda", dtype=torch.float32)
    out = torch.empty((batch, 1, HQ, D), device="cuda", dtype=torch.float32)
    lib = pkg.lib()
    qd, od = pkg.desc(q), pkg.desc(out)
    descs = [(pkg.desc(k), pkg.desc(v)) for k, v in caches]

    def step():
        for kd, vd in descs:
            rc = lib.vx_flash_attn_ext(qd, kd, vd, None, None, od, 0.125, 0.0, 0.0, torch.cuda.current_stream().cuda_stream)
            if rc:
                pkg.check(rc, "vx_flash_attn_ext")

    def one_layer():
        kd, vd = descs[0]
        rc = lib.vx_flash_attn_ext(qd, kd, vd, None, None, od, 0.125, 0.0, 0.0, torch.cuda.current_stream().cuda_stream)
        if rc:
            pkg.check(rc, "vx_flash_attn_ext")

    return step, one_layer, (q, caches, out)


def prefill_attn_setup(pkg, batch, T):
    import torch
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import reflib
    g = torch.Generator(device="cuda").manual_seed(99 + T)
    q = torch.randn((batch, HQ, T, D), generator=g, device="cuda", dtype=torch.float32)
    k = torch.randn((batch, HKV, T, D), generator=g, device="cuda", dtype=torch.float32).half()
    v = torch.randn((batch, HKV, T, D), generator=g, device="cuda", dtype=torch.float32).half()
    mask = torch.from_numpy(reflib.causal_mask(T, T)).cuda()
    out = torch.empty((batch, T, HQ, D), device="cuda", dtype=torch.float32)
    lib = pkg.lib()
    qd, kd, vd, md, od = pkg.desc(q), pkg.desc(k), pkg.desc(v), pkg.desc(mask), pkg.desc(out)

    def call():
        rc = lib.vx_flash_attn_ext(qd, kd, vd, md, None, od, 0.125, 0.0, 0.0, torch.cuda.current_stream().cuda_stream)
        if rc:
            pkg.check(rc, "vx_flash_attn_ext")

    flops = 4.0 * HQ * D * T * (T + 1) / 2 * batch  # causal-exact
    return call, flops, (q, k, v, mask, out)


def locdit_attn_setup(pkg, requests=8, branch=7, layers=4, timesteps=10):
    import torch
    import reflib
    L = 2 * branch
    pos = np.zeros(L, np.int32)
    m = np.zeros((L, L), np.uint16)
    reflib.load_oracle().orc_cfg_pair_constants(branch, reflib.ptr(pos, C.c_int32), reflib.ptr(m, C.c_uint16))
    g = torch.Generator(device="cuda").manual_seed(7)
    q = torch.randn((requests, HQ, L, D), generator=g, device="cuda")
    k = torch.randn((requests, HKV, L, D), generator=g, device="cuda")
    v = torch.randn((requests, HKV, L, D), generator=g, device="cuda")
    mask = torch.from_numpy(m.view(np.float16)).cuda()
    out = torch.empty((requests, L, HQ, D), device="cuda")
    lib = pkg.lib()
    qd, kd, vd, md, od = pkg.desc(q), pkg.desc(k), pkg.desc(v), pkg.desc(mask), pkg.desc(out)
    n_calls = layers * (timesteps - 1)  # the first Euler step is skipped under cfg-zero-star

    def solve():
        for _ in range(n_calls):
            rc = lib.vx_flash_attn_ext(qd, kd, vd, md, None, od, 0.125, 0.0, 0.0, torch.cuda.current_stream().cuda_stream)
            if rc:
                pkg.check(rc, "vx_flash_attn_ext")

    return solve, n_calls, (q, k, v, mask, out)


def q8_proj_setup(pkg, M, K, N):
    import torch
    import reflib
    w = (reflib.rng("bench", "w", M, K).standard_normal((M, K)) * 0.02).astype(np.float32)
    wq = torch.from_numpy(reflib.quantize_q8_0(w)).cuda()
    x = torch.randn((N, K), device="cuda")
    out = torch.empty((N, M), device="cuda")
    lib = pkg.lib()
    wd, xd, od = pkg.desc_q8(wq, K), pkg.desc(x), pkg.desc(out)

    def call():
        rc = lib.vx_mul_mat(wd, xd, od, pkg.ACT_FLOAT, torch.cuda.current_stream().cuda_stream)
        if rc:
            pkg.check(rc, "vx_mul_mat")

    return call, (wq, x, out)


def cpu_baseline(batch, length, threads):
    """ggml-cpu (the reference build in oracle/_ref) on one layer of the decode workload."""
    import reflib
    ref = reflib.load_ref()
    q = reflib.rng("cpu", "q").standard_normal((batch, HQ, 1, D)).astype(np.float32)
    k = reflib.rng("cpu", "k").standard_normal((batch, HKV, length, D)).astype(np.float16)
    v = reflib.rng("cpu", "v").standard_normal((batch, HKV, length, D)).astype(np.float16)
    if ref is not None:
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
        # size the sample to roughly 10 s of CPU work
        _, (mean1, _) = reflib.ref_fa(q, k, v, reps=20)
        reps = int(max(50, min(20000, 10.0 / max(mean1, 1e-6))))
        _, (mean, best) = reflib.ref_fa(q, k, v, reps=reps)
        return {"value": kv_bytes(batch, length) / mean / 1e9, "unit": "GB/s", "cores": threads, "kind": "reference",
                "sample": f"{reps} repeats of one layer's ggml_flash_attn_ext on ggml-cpu (batch {batch}, KV {length}, "
                          f"f16 K/V), mean {mean * 1e6:.1f} us, best {best * 1e6:.1f} us"}
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        reflib.oracle_fa(q, k.astype(np.float32), v.astype(np.float32))
    mean = (time.perf_counter() - t0) / reps
    return {"value": kv_bytes(batch, length) / mean / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{reps} repeats of one layer on the scalar C oracle (oracle/_ref not prebuilt)"}


def backbone_bench(pkg, timer, side, threads, with_cpu, layers=LAYERS, batch=2, prefill=512, steps=256, do_prefill=True, cpu_reps=40):
    """BASELINE config 4: the whole decoder stack with Q8_0 weights (hidden 1024, 16/2 heads, FFN 4096),
    batch 2, prefill 512 tokens then 256 decode steps.  The GPU side is the host-side mirror of the
    reference's layer_forward over the C ABI (voxcpm.cpp_amd/backbone.py, F32 KV cache as in the
    reference); a decode step is replayed from a captured HIP graph.  Four KV lengths spread over the
    256-step range are captured and each replayed steps/4 times, so the timed work is that of the
    512 -> 768 decode.  ggml-cpu runs the reference-structured graph of the same stack beside it."""
    import torch
    import reflib
    bbmod = __import__("voxcpm_cpp_amd.backbone", fromlist=["MiniCPMBackbone"])
    params = reflib.backbone_params("bench-bb", 1)   # one layer's seeded weights, placed in `layers` separate buffers
    lw = params["layers"][0]
    max_len = prefill + steps
    m = bbmod.MiniCPMBackbone(n_layer=layers, max_length=max_len, batch=batch, use_mup=True, kv_f16=False)
    for li in range(layers):
        for n in reflib.BB_WEIGHTS:
            m.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
        for n in ("input_layernorm", "post_layernorm"):
            m.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
    m.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
    m.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
    weight_bytes = layers * sum(lw[n].nbytes for n in reflib.BB_WEIGHTS)

    t_prefill = None
    t_prefill_f16 = None
    xp = None
    if do_prefill:
        xp = torch.randn((batch, prefill, 1024), device="cuda", generator=torch.Generator(device="cuda").manual_seed(7))
        mask = torch.from_numpy(reflib.causal_mask(prefill, prefill)).cuda()
        run_p, _ = m.plan(xp, prefill, 0, mask)
        t_prefill = timer.run(run_p, iters=3, warmup=1)
        # the same prefill with the F32 cache rounded to f16 on its way into the LDS-tiled attention kernel (opt-in, read per call)
        os.environ["VX_FA_F32_PREFILL"] = "1"
        t_prefill_f16 = timer.run(run_p, iters=3, warmup=1)
        del os.environ["VX_FA_F32_PREFILL"]
        timer.run(run_p, iters=1, warmup=0)  # leave the cache as the default route writes it
    else:   # long caches: decode over seeded cache contents instead of a real prefill
        gk = torch.Generator(device="cuda").manual_seed(11)
        for t in m.k_cache + m.v_cache:
            t.normal_(generator=gk)

    x1 = torch.randn((batch, 1, 1024), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    points = [prefill + (2 * i + 1) * steps // 8 for i in range(4)]
    replays, n_calls = [], 0
    for n_past in points:
        run_d, _ = m.plan(x1, 1, n_past)
        n_calls = run_d.n_calls
        replays.append((graphed(run_d, side), run_d))
    per = steps // 4
    for rp, _ in replays:
        rp()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for rp, _ in replays:
        for _ in range(per):
            rp()
    torch.cuda.synchronize()
    t_step = (time.perf_counter() - t0) / (per * 4)
    kvb = layers * 2 * batch * HKV * (prefill + steps // 2) * D * 4
    res = {"decode_steps_per_s": 1.0 / t_step, "ms_per_step": t_step * 1e3, "launches_per_step": n_calls,
           "weight_GB/s": weight_bytes / t_step / 1e9, "hbm_frac_weights_plus_kv": (weight_bytes + kvb) / t_step / 1e9 / HBM_PEAK_GBS,
           "prefill_ms": t_prefill * 1e3 if t_prefill else None, "prefill_tokens_per_s": batch * prefill / t_prefill if t_prefill else None,
           "prefill_ms_VX_FA_F32_PREFILL": t_prefill_f16 * 1e3 if t_prefill else None,
           "kv_cache": "f32 (the reference's cache type)", "launch": "captured HIP graph per step, KV lengths " + str(points)}
    del replays, m
    ref = reflib.load_ref() if with_cpu else None
    if ref is not None:
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
        params["dims"]["n_layer"] = layers
        params["layers"] = [lw] * layers
        reflib.ref_backbone_create(params, max_len, batch, use_mup=True, kv_f16=False)
        cpu_prefill = None
        if do_prefill:
            xph = xp.cpu().numpy()
            tp0 = time.perf_counter()
            reflib.ref_backbone_forward(xph, 0, reflib.causal_mask(prefill, prefill))
            cpu_prefill = time.perf_counter() - tp0
        _, (mean, best), n_nodes = reflib.ref_backbone_forward(x1.cpu().numpy(), prefill + steps // 2, None, reps=cpu_reps)
        ref.rh_bb_free()
        res["ggml_cpu"] = {"decode_steps_per_s": 1.0 / mean, "ms_per_step": mean * 1e3, "best_ms": best * 1e3, "threads": threads,
                           "graph_nodes": n_nodes, "prefill_ms": cpu_prefill * 1e3 if cpu_prefill else None,
                           "sample": f"{cpu_reps} repeats of the decode step at KV length {prefill + steps // 2}" + (", one prefill" if do_prefill else ", cache contents as left by allocation")}
        res["speedup_vs_ggml_cpu"] = mean / t_step
    return res


def locdit_stack_bench(pkg, timer, side, threads, with_cpu, requests=8, branch=7, layers=4, timesteps=10):
    """BASELINE config 3 as a whole decoder pass: LocDiT runs the MiniCPM layer stack non-causally over the CFG
    pair laid out as one 2 x 7-token sequence with a block-diagonal mask (src/locdit.cpp:400-464), no cache write;
    8 concurrent requests ride in the batch dimension.  One CFM solve is (timesteps - 1) such passes."""
    import torch
    import reflib
    bbmod = __import__("voxcpm_cpp_amd.backbone", fromlist=["MiniCPMBackbone"])
    T = 2 * branch
    pos = np.zeros(T, np.int32)
    mk = np.zeros((T, T), np.uint16)
    reflib.load_oracle().orc_cfg_pair_constants(branch, reflib.ptr(pos, C.c_int32), reflib.ptr(mk, C.c_uint16))
    params = reflib.backbone_params("bench-locdit", 1)
    lw = params["layers"][0]
    m = bbmod.MiniCPMBackbone(n_layer=layers, max_length=T, batch=requests, use_mup=False, kv_f16=False)
    for li in range(layers):
        for n in reflib.BB_WEIGHTS:
            m.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
        for n in ("input_layernorm", "post_layernorm"):
            m.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
    m.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
    m.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
    x = torch.randn((requests, T, 1024), device="cuda", generator=torch.Generator(device="cuda").manual_seed(9))
    mask = torch.from_numpy(mk.view(np.float16)).cuda()
    run, _ = m.plan(x, T, 0, mask, write_kv=False)
    s = timer.run(graphed(run, side), iters=50, warmup=5)
    res = {"us_per_decoder_pass": s * 1e6, "us_per_cfm_solve": s * (timesteps - 1) * 1e6, "launches_per_pass": run.n_calls,
           "shape": f"{layers} layers, {requests} requests x {T} tokens (CFG pair), non-causal, Q8_0 weights"}
    # one request alone (the reference's own call shape: 14 tokens, every projection on the streaming kernel)
    m1 = bbmod.MiniCPMBackbone(n_layer=layers, max_length=T, batch=1, use_mup=False, kv_f16=False)
    m1.weights, m1.norms, m1.final_norm, m1.rope_factors = m.weights, m.norms, m.final_norm, m.rope_factors
    run1, _ = m1.plan(x[:1].contiguous(), T, 0, mask, write_kv=False)
    s1 = timer.run(graphed(run1, side), iters=50, warmup=5)
    res["one_request"] = {"us_per_decoder_pass": s1 * 1e6, "launches_per_pass": run1.n_calls}
    del m, m1
    ref = reflib.load_ref() if with_cpu else None
    if ref is not None:
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
        params["dims"]["n_layer"] = layers
        params["layers"] = [lw] * layers
        reflib.ref_backbone_create(params, T, requests, use_mup=False, kv_f16=False)
        _, (mean, best), _ = reflib.ref_backbone_forward(x.cpu().numpy(), 0, mk.view(np.float16), write_kv=False, reps=40)
        ref.rh_bb_free()
        res["ggml_cpu_us_per_decoder_pass"] = mean * 1e6
        res["ggml_cpu_threads"] = threads
        res["speedup_vs_ggml_cpu"] = mean / s
    return res


def cfm_solve_bench(pkg, timer, side, threads, with_cpu, layers=4, patch=2, prefix=4, timesteps=10):
    """BASELINE config 3 as one whole UnifiedCFM solve of one request (src/unified_cfm.cpp:88-149): per Euler step the
    input projection, the assembly of the 14-token CFG-pair sequence, the 4-layer decoder pass, the output projections
    and the zero-star guidance arithmetic with the update of x -- every launch of the solve, replayed from one HIP graph.
    ggml-cpu runs the same solve as the one graph the reference builds."""
    import torch
    import reflib
    bbmod = __import__("voxcpm_cpp_amd.backbone", fromlist=["MiniCPMBackbone"])
    cfmmod = __import__("voxcpm_cpp_amd.cfm", fromlist=["LocDiTCfmSolver"])
    params = reflib.backbone_params("bench-locdit", 1)
    lw = params["layers"][0]
    cp = reflib.cfm_params("bench-cfm")
    T = 2 * (1 + prefix + patch)
    dec = bbmod.MiniCPMBackbone(n_layer=layers, max_length=T, batch=1, use_mup=False, kv_f16=False)
    for li in range(layers):
        for n in reflib.BB_WEIGHTS:
            dec.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
        for n in ("input_layernorm", "post_layernorm"):
            dec.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
    dec.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
    dec.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
    q8 = lambda w, b: (torch.from_numpy(reflib.quantize_q8_0(w)).cuda(), w.shape[1], torch.from_numpy(b).cuda())
    solver = cfmmod.LocDiTCfmSolver(dec, 64, q8(cp["in_w"], cp["in_b"]), q8(cp["cond_w"], cp["cond_b"]), q8(cp["out_w"], cp["out_b"]))
    rs = np.random.default_rng(11)
    z, mu = rs.standard_normal((patch, 64)).astype(np.float32), rs.standard_normal(1024).astype(np.float32)
    cond, table = rs.standard_normal((prefix, 64)).astype(np.float32), rs.standard_normal((timesteps, 1024)).astype(np.float32)
    t_span = np.zeros(timesteps + 1, np.float32)
    reflib.load_oracle().orc_t_span(timesteps, 1.0, reflib.ptr(t_span, C.c_float))
    run, _ = solver.plan(*(torch.from_numpy(a).cuda() for a in (z, mu, cond, table)), t_span, cfg_value=2.0)
    s = timer.run(graphed(run, side), iters=30, warmup=3)
    res = {"us_per_cfm_solve": s * 1e6, "launches_per_solve": run.n_calls, "launches_per_step": run.n_calls / (timesteps - 1),
           "shape": f"one request: {timesteps} Euler steps ({timesteps - 1} estimator passes under zero-star), {layers} layers, "
                    f"CFG pair as one {T}-token sequence, Q8_0 weights"}
    del solver, dec
    ref = reflib.load_ref() if with_cpu else None
    if ref is not None:
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
        params["dims"]["n_layer"] = layers
        params["layers"] = [lw] * layers
        reflib.ref_backbone_create(params, T, 1, use_mup=False, kv_f16=False, fused_weights=True)
        reflib.ref_cfm_create(cp)
        _, (mean, best), n_nodes = reflib.ref_cfm_solve(z, mu, cond, table, n_steps=timesteps, reps=10)
        ref.rh_cfm_free()
        ref.rh_bb_free()
        res["ggml_cpu_us_per_cfm_solve"] = mean * 1e6
        res["ggml_cpu_threads"] = threads
        res["ggml_graph_nodes"] = n_nodes
        res["speedup_vs_ggml_cpu"] = mean / s
    return res


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--length", type=int, default=4096, help="KV length of the headline decode workload")
    ap.add_argument("--no-others", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the ggml-cpu baseline")
    ap.add_argument("--eager", action="store_true", help="launch every call from Python instead of replaying a HIP graph")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 256 MiB -> 256 MiB elementwise copy kernel a few times (the known-size "
                         "launch that hardware byte counters are scaled by) and exit")
    ap.add_argument("--profile", choices=["prefill", "backbone", "cfm", "gemm"], default=None,
                    help="run only this secondary workload a few times (for rocprofv3) and print its figures")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path has no cross-GPU step); run with --gpus 1")

    import torch
    if args.calibrate_copy:
        n = 64 << 20  # float32 elements: 256 MiB read + 256 MiB written per launch
        x = torch.ones(n, device="cuda", dtype=torch.float32)
        y = torch.empty_like(x)
        for _ in range(5):
            torch.mul(x, 2.0, out=y)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy": {"kernel": "torch elementwise mul (vectorized_elementwise_kernel)",
                                             "bytes_read": 4 * n, "bytes_written": 4 * n, "launches": 5}}))
        return
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg.check(pkg.lib().vx_init(0), "vx_init")
    timer = Timer()

    if args.profile == "prefill":   # config 5 prefill attention, 16 streams x 4096 tokens
        call, flops, keep = prefill_attn_setup(pkg, 16, 4096)
        s = timer.run(call, iters=5, warmup=2)
        print(json.dumps({"profile": "cfg5_prefill_attn_T4096_B16", "us": s * 1e6, "TFLOP/s_causal_exact": flops / s / 1e12,
                          "mfma_frac": flops / s / 1e12 / MFMA_F16_PEAK_TFLOPS}))
        return
    if args.profile == "gemm":      # the prefill-sized Q8_0 projection, 4096 rows x 1024 x 16384 tokens
        M, K, N = 4096, 1024, 16384
        call, keep = q8_proj_setup(pkg, M, K, N)
        s = timer.run(call, iters=5, warmup=2)
        print(json.dumps({"profile": "q8_0_mul_mat_4096x1024x16384", "us": s * 1e6, "TFLOP/s": 2.0 * M * K * N / s / 1e12,
                          "mfma_frac": 2.0 * M * K * N / s / 1e12 / MFMA_F16_PEAK_TFLOPS, "VX_GEMM_LDS": os.environ.get("VX_GEMM_LDS", "1")}))
        return
    if args.profile == "cfm":       # config 3: whole CFM solves of one request, replayed from a HIP graph
        print(json.dumps({"profile": "cfg3_cfm_solve_one_request", **cfm_solve_bench(pkg, timer, torch.cuda.Stream(), 1, False)}))
        return
    if args.profile == "backbone":  # config 4 decode steps, eager launches so that every kernel is traced
        print(json.dumps({"profile": "cfg4_backbone_24layers_b2", **backbone_bench(pkg, timer, torch.cuda.Stream(), 1, False, steps=16)}))
        return

    # ---- headline: config 2, L = args.length -------------------------------------------
    B, L = 2, args.length
    side = torch.cuda.Stream()
    step_eager, one_layer, keep = decode_attn_setup(pkg, B, L, LAYERS)
    eager_sec = timer.run(step_eager, iters=20)
    # the 24 launches of a step replayed as one HIP graph: what a C++ host looping over graph
    # nodes achieves, without the Python call overhead of this script
    step = graphed(step_eager, side) if not args.eager else step_eager
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    sec_per_step = (time.perf_counter() - t0) / args.steps
    step_bytes = LAYERS * kv_bytes(B, L)
    value = step_bytes / sec_per_step / 1e9

    # dominant kernel: one vx_flash_attn_ext call (split-KV kernel + combine), HIP events
    launch_sec = timer.run(step, iters=200, warmup=10) / LAYERS
    achieved = kv_bytes(B, L) / launch_sec / 1e9
    # HBM bytes per call from rocprofv3 FETCH_SIZE / WRITE_SIZE (split kernel + merge kernel, scaled
    # by the same counters on a 256 MiB copy: x2.000 and x1.000), taken at the default length only
    traffic = MEASURED_TRAFFIC_BYTES.get((B, L))
    roofline = {"bound": "hbm", "kernel": "fattn_cols16_kernel<64,f16> + fattn_merge_kernel<64>", "achieved": achieved,
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                "launch_us": launch_sec * 1e6, "bytes_per_launch": kv_bytes(B, L),
                "note": "average over the 24 launches of a graph-replayed step (HIP events on the launch stream)"}
    del keep

    others = {}
    if not args.no_others:
        for L2 in (128, 512, 2048, 4096):
            st, one, keep = decode_attn_setup(pkg, 2, L2, LAYERS)
            s = timer.run(graphed(st, side), iters=50)
            others[f"cfg2_decode_attn_L{L2}"] = {"us_per_layer": s / LAYERS * 1e6,
                                                  "GB/s": LAYERS * kv_bytes(2, L2) / s / 1e9}
            del keep
        st, one, keep = decode_attn_setup(pkg, 16, 8192, LAYERS)  # 1.5 GiB of KV: no cache reuse
        s = timer.run(graphed(st, side), iters=20, warmup=3) / LAYERS
        others["cfg5_decode_attn_B16_L8192"] = {"us_per_layer": s * 1e6, "GB/s": kv_bytes(16, 8192) / s / 1e9,
                                                "hbm_frac": kv_bytes(16, 8192) / s / 1e9 / HBM_PEAK_GBS}
        del keep
        for name, b, T, it in (("cfg1_prefill_attn_T256", 1, 256, 200), ("cfg5_prefill_attn_T4096_B1", 1, 4096, 5),
                                  ("cfg5_prefill_attn_T4096_B16", 16, 4096, 3)):
            call, flops, keep = prefill_attn_setup(pkg, b, T)
            s = timer.run(call, iters=it, warmup=2)
            others[name] = {"us": s * 1e6, "TFLOP/s_causal_exact": flops / s / 1e12,
                            "mfma_frac": flops / s / 1e12 / MFMA_F16_PEAK_TFLOPS}
            del keep
        solve, n_calls, keep = locdit_attn_setup(pkg)
        s = timer.run(graphed(solve, side), iters=20)
        others["cfg3_locdit_attn_16seq_x7"] = {"us_per_cfm_solve": s * 1e6, "launches_per_solve": n_calls,
                                               "us_per_attention": s / n_calls * 1e6}
        del keep
        for name, M, K, N in (("q8_0_proj_1024x1024_n2", 1024, 1024, 2), ("q8_0_ffn_up_4096x1024_n2", 4096, 1024, 2),
                              ("q8_0_proj_1024x1024_n1024", 1024, 1024, 1024), ("q8_0_ffn_up_4096x1024_n1024", 4096, 1024, 1024),
                              ("q8_0_proj_1024x1024_n16384", 1024, 1024, 16384)):
            call, keep = q8_proj_setup(pkg, M, K, N)
            s = timer.run(call, iters=200 if N <= 1024 else 20, warmup=5)
            wbytes = M * K // 32 * 34
            others[name] = {"us": s * 1e6, "weight_GB/s": wbytes / s / 1e9, "TFLOP/s": 2.0 * M * K * N / s / 1e12}
            del keep

    threads = min(16, os.cpu_count() or 1)
    if not args.no_others:
        others["cfg4_backbone_24layers_b2"] = backbone_bench(pkg, timer, side, threads, not args.no_cpu)
        others["cfg3_locdit_stack_8req_x14"] = locdit_stack_bench(pkg, timer, side, threads, not args.no_cpu)
        others["cfg3_cfm_solve_one_request"] = cfm_solve_bench(pkg, timer, side, threads, not args.no_cpu)
        # BASELINE config 5 as a whole stack: 8 streams x CFG pair (batch 16) decoding from KV length 4096 towards 8192
        # (F32 cache as in the reference; the decode steps run over seeded cache contents)
        others["cfg5_backbone_24layers_b16_L4096"] = backbone_bench(pkg, timer, side, threads, not args.no_cpu, batch=16, prefill=4096,
                                                                    steps=256, do_prefill=False, cpu_reps=3)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(B, L, threads)

    line = {
        # BASELINE.json's metric, verbatim; `value` is its decode component on config 2 (see config.value_is),
        # the prefill TFLOP/s and backbone steps/s components are repeated under "components"
        "metric": "attn TFLOP/s (prefill) & HBM GB/s (decode) vs roofline; backbone decode steps/s",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec_per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 K/V, f32 accumulate", "data": "synthetic (seeded N(0,1))",
        "config": {"workload": f"BASELINE config 2: 24 layers x GQA decode attention, 16/2 heads, head_dim 64, "
                               f"batch 2, f16 KV length {L}",
                   "value_is": "decode attention HBM GB/s: algorithmic K/V bytes of the 24 calls of a step / wall time of the step",
                   "decode_attn_steps_per_s": 1.0 / sec_per_step,
                   "launch": "eager from Python" if args.eager else "one HIP graph replay per step",
                   "eager_python_ms_per_step": eager_sec * 1e3},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "components": {
            "decode_attn_GB/s_cfg2": value,
            "decode_attn_hbm_frac_cfg5_B16_L8192": others.get("cfg5_decode_attn_B16_L8192", {}).get("hbm_frac"),
            "prefill_attn_TFLOP/s_cfg5_T4096_B16": others.get("cfg5_prefill_attn_T4096_B16", {}).get("TFLOP/s_causal_exact"),
            "prefill_attn_mfma_frac_cfg5_T4096_B16": others.get("cfg5_prefill_attn_T4096_B16", {}).get("mfma_frac"),
            "backbone_decode_steps_per_s_cfg4": others.get("cfg4_backbone_24layers_b2", {}).get("decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg4_ggml_cpu": others.get("cfg4_backbone_24layers_b2", {}).get("ggml_cpu", {}).get("decode_steps_per_s"),
        },
        "others": others,
    }
    print(json.dumps(line, allow_nan=False))


if __name__ == "__main__":
    main()
