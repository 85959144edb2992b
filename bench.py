#!/usr/bin/env python3
"""Benchmark of the attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  The headline workload is BASELINE config 5's decode attention, the largest
single-GPU configuration: 8 synthesis streams x CFG pair (batch 16), 16 Q / 2 KV heads, head_dim 64,
one new token per step over an f16 KV cache of 8192 keys, 24 layers.  A step is one pass over the 24
layers (24 calls of vx_flash_attn_ext, each on its own layer's resident cache: 1.5 GiB of K/V per
step, so nothing is served from a cache); `value` is the algorithmic K/V bytes of a step divided by
its wall time, inputs already in HBM.

The same line carries a `roofline` object for that call (published peak, the peak a plain streaming
read reaches on this box, measured HBM traffic when a counter profile of the current kernels is on
file), a `cpu_baseline` object (the reference's own ggml-cpu, oracle/_ref, timed on this machine's
host cores on one layer of the same workload, at the box's core share and at 8 threads), and under
"others" the other BASELINE shapes: config 2's decode lengths, prefill attention, LocDiT attention
and the CFM solve, the Q8_0 projections, and the config 4 / 5 decoder stacks with F32 and f16 caches.
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


def measured_traffic(batch, length):
    """HBM bytes per vx_flash_attn_ext call from the counter profile on file for this shape (rocprofv3 FETCH_SIZE /
    WRITE_SIZE scaled by a plain copy; profiles/decode_attn_*_kernel_trace_and_counters.txt carries a line
    `traffic_bytes_per_call: N` and the commit it was taken at), or None."""
    path = os.path.join(ROOT, "profiles", f"decode_attn_B{batch}_L{length}_kernel_trace_and_counters.txt")
    try:
        text = open(path).read()
    except OSError:
        return None, None
    import re
    m = re.search(r"^traffic_bytes_per_call:\s*(\d+)", text, re.M)
    c = re.search(r"^commit:\s*(\S+)", text, re.M)
    return (int(m.group(1)) if m else None), (c.group(1) if c else None)


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

    def sustained(self, fn, iters, rounds=6):
        """Matrix-bound kernels run 15-25 % slower in the first 15-20 ms of a burst than afterwards (the clocks step up
        under load): `rounds` back-to-back rounds of `iters` calls; returns (median round, first round), seconds per call."""
        per = [self.run(fn, iters, warmup=0) for _ in range(rounds)]
        return float(np.median(per)), per[0]


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


def pinned_in_turns(pkg, timer, call, wq, rounds, iters):
    """The same product timed in turns with its weights' tiles made on every call and made once and kept (vx_weights_pin),
    so that both see the same clocks (a run of large products slows the clocks down, and they recover over seconds)."""
    turns = {"tiles_made_per_call": [], "weights_pinned": []}
    for _ in range(rounds):
        turns["tiles_made_per_call"].append(timer.run(call, iters=iters, warmup=2))
        pkg.check(pkg.lib().vx_weights_pin(wq.data_ptr(), wq.numel()), "vx_weights_pin")
        turns["weights_pinned"].append(timer.run(call, iters=iters, warmup=2))
        pkg.check(pkg.lib().vx_weights_unpin(wq.data_ptr()), "vx_weights_unpin")
    return turns


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def stats(times):
    """mean / median / p90 / best of a list of seconds, as the reference's benchmark reports them
    (benchmark/voxcpm_benchmark.cpp:623-669)."""
    t = np.sort(np.asarray(times, np.float64))
    return {"mean": float(t.mean()), "median": float(np.median(t)), "p90": float(t[min(len(t) - 1, int(np.ceil(0.9 * len(t))) - 1)]),
            "best": float(t[0]), "repeats": int(len(t))}


def cpu_baseline(batch, length, core_share):
    """ggml-cpu (the reference build in oracle/_ref) on one layer of the headline decode workload: at every core
    of this box's share and at 8 threads (the reference's own benchmark setting, README.md:504), a few seconds each."""
    import reflib
    ref = reflib.load_ref()
    q = reflib.rng("cpu", "q").standard_normal((batch, HQ, 1, D)).astype(np.float32)
    k = reflib.rng("cpu", "k").standard_normal((batch, HKV, length, D)).astype(np.float16)
    v = reflib.rng("cpu", "v").standard_normal((batch, HKV, length, D)).astype(np.float16)
    nbytes = kv_bytes(batch, length)
    if ref is None:
        t0 = time.perf_counter()
        reflib.oracle_fa(q[:1], k[:1].astype(np.float32), v[:1].astype(np.float32))
        sec = (time.perf_counter() - t0) * batch
        return {"value": nbytes / sec / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": "one stream of one layer on the scalar C oracle, scaled to the batch (oracle/_ref not prebuilt)"}
    runs = {}
    for threads in sorted({core_share, min(8, core_share)}, reverse=True):
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
        _, (mean1, _) = reflib.ref_fa(q, k, v, reps=3)
        reps = int(max(5, min(2000, 6.0 / max(mean1, 1e-6))))   # about 6 s of CPU work per setting
        reflib.ref_fa(q, k, v, reps=reps)
        st = stats(reflib.ref_last_times())
        runs[threads] = {"GB/s": nbytes / st["mean"] / 1e9, "us": {n: st[n] * 1e6 for n in ("mean", "median", "p90", "best")}, "repeats": st["repeats"]}
    assert ref.rh_use_device(b"CPU", min(8, core_share), 0) == 0
    top = runs[core_share]
    eight = runs[min(8, core_share)]
    return {"value": top["GB/s"], "unit": "GB/s", "cores": core_share, "kind": "reference", "cpu": cpu_model(),
            "value_8_threads": eight["GB/s"], "us_8_threads": eight["us"]["mean"], "us": top["us"]["mean"],
            "host_logical_cpus": os.cpu_count(),
            "sample": f"{top['repeats']} repeats of one layer's ggml_flash_attn_ext on ggml-cpu (batch {batch}, KV {length}, f16 K/V, "
                      f"{nbytes >> 20} MiB of K/V): mean {top['us']['mean']:.0f} us, median {top['us']['median']:.0f}, p90 {top['us']['p90']:.0f}; "
                      f"{core_share} threads = this box's core share for one GPU",
            "by_threads": {str(t): r for t, r in runs.items()}}


def load_stack(pkg, layers, max_len, batch, kv_f16, lw, params, use_mup=True):
    import torch
    import reflib
    bbmod = __import__("voxcpm_cpp_amd.backbone", fromlist=["MiniCPMBackbone"])
    m = bbmod.MiniCPMBackbone(n_layer=layers, max_length=max_len, batch=batch, use_mup=use_mup, kv_f16=kv_f16)
    for li in range(layers):
        for n in reflib.BB_WEIGHTS:
            m.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
        for n in ("input_layernorm", "post_layernorm"):
            m.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
    m.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
    m.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
    return m


def backbone_bench(pkg, timer, side, threads, with_cpu, layers=LAYERS, batch=2, prefill=512, steps=256, kv_f16=False,
                   cpu_reps=40, cpu_prefill=True, plugin_reps=40, f32_prefill_switch=False):
    """A whole decoder stack with Q8_0 weights (hidden 1024, 16/2 heads, FFN 4096): BASELINE config 4 (batch 2,
    prefill 512 tokens then 256 decode steps) or config 5 (batch 16, prefill 4096, decode to 8192).  The GPU side is
    the host-side mirror of the reference's layer_forward over the C ABI (voxcpm.cpp_amd/backbone.py), a decode step
    replayed from a captured HIP graph: four KV lengths spread over the decode range are captured and each replayed
    steps/4 times, so the timed work is that of the whole decode.  Beside it: the same step through the product
    boundary -- the reference-structured graph handed to the plugin's graph_compute by ggml, eager, rebuilt per call
    as the reference does -- and ggml-cpu on that graph."""
    import torch
    import reflib
    params = reflib.backbone_params("bench-bb", 1)   # one layer's seeded weights, placed in `layers` separate buffers
    lw = params["layers"][0]
    max_len = prefill + steps
    m = load_stack(pkg, layers, max_len, batch, kv_f16, lw, params)
    weight_bytes = layers * sum(lw[n].nbytes for n in reflib.BB_WEIGHTS)
    es = 2 if kv_f16 else 4

    gk = torch.Generator(device="cuda").manual_seed(11)
    for t in m.k_cache + m.v_cache:      # seeded cache contents; the prefill overwrites its part
        if kv_f16:
            t.copy_(torch.randn(t.shape, device="cuda", generator=gk).half())
        else:
            t.normal_(generator=gk)
    xp = torch.randn((batch, prefill, 1024), device="cuda", generator=torch.Generator(device="cuda").manual_seed(7))
    mask = torch.from_numpy(reflib.causal_mask(prefill, prefill)).cuda()
    run_p, _ = m.plan(xp, prefill, 0, mask)
    big = batch * prefill > 4096
    # in turns (a run of large products slows the clocks down): the weights as they are / declared constant, as the plugin declares
    # a buffer that ggml marks as weights -- the products of 1024 tokens and more then keep their weights' tiles between calls
    t_un, t_pin = [], []
    for _ in range(2):
        m.unpin_weights()
        t_un.append(timer.run(run_p, iters=1 if big else 3, warmup=1))
        m.pin_weights()
        t_pin.append(timer.run(run_p, iters=1 if big else 3, warmup=1))
    t_prefill_unpinned, t_prefill = min(t_un), min(t_pin)
    t_prefill_f16 = None
    if f32_prefill_switch:
        # the same prefill with its F32 keys and values on the hi/lo wave kernel instead of the LDS-tiled one (read per call)
        os.environ["VX_FA_F32_PREFILL"] = "0"
        t_prefill_f16 = timer.run(run_p, iters=1 if big else 3, warmup=1)
        del os.environ["VX_FA_F32_PREFILL"]
        timer.run(run_p, iters=1, warmup=0)  # leave the cache as the default route writes it
    del run_p, mask

    x1 = torch.randn((batch, 1, 1024), device="cuda", generator=torch.Generator(device="cuda").manual_seed(8))
    points = [prefill + (2 * i + 1) * steps // 8 for i in range(4)]
    replays, n_calls = [], 0
    for n_past in points:
        run_d, _ = m.plan(x1, 1, n_past)
        n_calls = run_d.n_calls
        replays.append((graphed(run_d, side), run_d))
    per = max(1, min(64, steps // 4))
    for rp, _ in replays:
        rp()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for rp, _ in replays:
        for _ in range(per):
            rp()
    torch.cuda.synchronize()
    t_step = (time.perf_counter() - t0) / (per * 4)
    kvb = layers * 2 * batch * HKV * (prefill + steps // 2) * D * es
    res = {"decode_steps_per_s": 1.0 / t_step, "ms_per_step": t_step * 1e3, "launches_per_step": n_calls,
           "weight_GB/s": weight_bytes / t_step / 1e9, "hbm_frac_weights_plus_kv": (weight_bytes + kvb) / t_step / 1e9 / HBM_PEAK_GBS,
           "prefill_ms": t_prefill * 1e3, "prefill_tokens_per_s": batch * prefill / t_prefill,
           "prefill_ms_weights_not_pinned": t_prefill_unpinned * 1e3,
           "prefill_ms_VX_FA_F32_PREFILL=0": t_prefill_f16 * 1e3 if t_prefill_f16 else None,
           "kv_cache": "f16" if kv_f16 else "f32 (the reference's cache type)",
           "launch": f"captured HIP graph per step, KV lengths {points} ({per} replays each)"}
    del replays, m, xp
    torch.cuda.empty_cache()
    ref = reflib.load_ref()
    mid = prefill + steps // 2
    params["dims"]["n_layer"] = layers
    params["layers"] = [lw] * layers
    if ref is not None and plugin_reps > 0:
        # through the product boundary: ggml hands the reference-structured graph to the plugin's graph_compute
        assert ref.rh_load_plugin(pkg.PLUGIN_PATH.encode()) == 0
        assert ref.rh_use_device(b"GFX950_0", 1, 0) == 0
        plug = C.CDLL(pkg.PLUGIN_PATH)
        reflib.ref_backbone_create(params, max_len, batch, use_mup=True, kv_f16=kv_f16)
        plug.ggml_backend_gfx950_set_graph_replay(0)   # a decode step's graph changes with the KV length: launched node group by node group
        _, _, n_nodes = reflib.ref_backbone_forward(x1.cpu().numpy(), mid, None, reps=plugin_reps)
        st = stats(reflib.ref_last_times())
        launches = plug.ggml_backend_gfx950_last_launches()
        plug.ggml_backend_gfx950_set_graph_replay(1)   # the same graph again and again (what a fixed-length step would be): recorded, then replayed
        reflib.ref_backbone_forward(x1.cpu().numpy(), mid, None, reps=plugin_reps + 3)   # three runs until the replay is in place
        st_r = stats(reflib.ref_last_times()[3:])
        # what "decode steps/s" means for a drop-in: consecutive steps, a graph built per position as the reference builds it
        # (src/voxcpm.cpp:485-513), laid out, its inputs uploaded, computed, the hidden state fetched -- wall clock of the loop
        plug.ggml_backend_gfx950_set_graph_replay(1)
        n_loop = min(256, steps)
        patch_before = plug.ggml_backend_gfx950_set_graph_patch(0)   # the default: every step launched node group by node group
        _, lp = reflib.ref_backbone_decode_loop(x1.cpu().numpy(), prefill, n_loop)
        plug.ggml_backend_gfx950_host_ns.restype = C.c_longlong
        host0 = [plug.ggml_backend_gfx950_host_ns(i) / 1e3 for i in (0, 1)]
        _, lpo = reflib.ref_backbone_decode_loop(x1.cpu().numpy(), prefill, n_loop, overlap=True)
        plug.ggml_backend_gfx950_set_graph_patch(1)   # a step as an earlier step's recording with the changed arguments set on its nodes
        n_p0 = plug.ggml_backend_gfx950_patched_replays()
        _, lp1 = reflib.ref_backbone_decode_loop(x1.cpu().numpy(), prefill, n_loop)
        n_p1 = plug.ggml_backend_gfx950_patched_replays()
        host1 = [plug.ggml_backend_gfx950_host_ns(i) / 1e3 for i in (0, 1)]
        changed = plug.ggml_backend_gfx950_last_patched()
        _, lpo1 = reflib.ref_backbone_decode_loop(x1.cpu().numpy(), prefill, n_loop, overlap=True)
        plug.ggml_backend_gfx950_set_graph_patch(patch_before)
        ref.rh_bb_free()
        consecutive = {"decode_steps_per_s": 1.0 / lp["wall"], "ms_per_step": lp["wall"] * 1e3, "graph_compute_ms": lp["graph_compute"] * 1e3,
                       "host_us_last_step_analysis_and_issue": host0,
                       "steps_as_patched_recordings_GGML_GFX950_GRAPH_PATCH=1": {
                           "decode_steps_per_s": 1.0 / lp1["wall"], "ms_per_step": lp1["wall"] * 1e3, "graph_compute_ms": lp1["graph_compute"] * 1e3,
                           "next_graph_built_under_the_running_one_decode_steps_per_s": 1.0 / lpo1["wall"],
                           "host_us_last_step_analysis_and_comparison": host1, "steps_run_this_way": n_p1 - n_p0,
                           "kernels_whose_arguments_changed_in_the_last_step": changed,
                           "how": "each step's node-by-node pass is made against a recording of an earlier step (nothing launched, differing arguments "
                                  "set with hipGraphExecKernelNodeSetParams), then one hipGraphLaunch: the host pass runs before the GPU starts"},
                       "graph_build_and_layout_ms": lp["build"] * 1e3, "steps": n_loop, "from_kv_length": prefill,
                       "nodes_at_another_address_than_the_step_before": lp["moved"],
                       "how": "the drop-in figure: every step's graph rebuilt for its position, ggml_backend_graph_compute (synchronous), "
                              "wall clock over the loop including graph construction, layout, uploads and the fetch of the hidden state",
                       "next_graph_built_under_the_running_one": {"decode_steps_per_s": 1.0 / lpo["wall"], "ms_per_step": lpo["wall"] * 1e3,
                           "how": "the same loop with graph_compute_async: the host builds the next position's graph while the device computes"}}
        res["plugin_graph_compute"] = {"decode_steps_per_s": 1.0 / st["mean"], "ms_per_step": {n: st[n] * 1e3 for n in ("mean", "median", "p90", "best")},
                                       "graph_nodes": n_nodes, "launches": launches, "kv_length": mid,
                                       "consecutive_steps": consecutive,
                                       "how": "ggml_backend_graph_compute on libggml-gfx950.so, eager, synchronised per call",
                                       "same_graph_replayed": {"decode_steps_per_s": 1.0 / st_r["mean"], "ms_per_step": {n: st_r[n] * 1e3 for n in ("mean", "median", "p90", "best")},
                                                               "how": "the identical graph computed repeatedly: the plugin records it at its third run and replays one HIP graph"}}
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
    if ref is not None and with_cpu:
        assert ref.rh_use_device(b"CPU", threads, 0) == 0
        reflib.ref_backbone_create(params, max_len, batch, use_mup=True, kv_f16=kv_f16)
        cpu_pf = None
        if cpu_prefill:
            xph = np.random.default_rng(7).standard_normal((batch, prefill, 1024)).astype(np.float32)
            tp0 = time.perf_counter()
            reflib.ref_backbone_forward(xph, 0, reflib.causal_mask(prefill, prefill))
            cpu_pf = time.perf_counter() - tp0
        if not cpu_prefill:   # no prefill (it would take minutes): the cache gets seeded values instead, one array for every layer
            kvt = np.float16 if kv_f16 else np.float32
            fill = np.random.default_rng(5).standard_normal(batch * HKV * max_len * D, dtype=np.float32).astype(kvt)
            for li in range(layers):
                for which in (0, 1):
                    assert ref.rh_bb_cache_set(li, which, fill.ctypes.data, fill.nbytes) == 0
            del fill
        _, (mean, best), n_nodes = reflib.ref_backbone_forward(x1.cpu().numpy(), mid, None, reps=cpu_reps)
        st = stats(reflib.ref_last_times())
        ref.rh_bb_free()
        res["ggml_cpu"] = {"decode_steps_per_s": 1.0 / mean, "ms_per_step": mean * 1e3, "median_ms": st["median"] * 1e3, "p90_ms": st["p90"] * 1e3,
                           "best_ms": best * 1e3, "threads": threads, "graph_nodes": n_nodes, "prefill_ms": cpu_pf * 1e3 if cpu_pf else None,
                           "sample": f"{cpu_reps} repeats of the decode step at KV length {mid}" + (", one prefill" if cpu_prefill else ", the cache filled with seeded N(0,1) values, no prefill (it would take minutes)")}
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


def cfm_requests_bench(pkg, threads, with_cpu, requests=8, layers=4, patch=2, prefix=4, timesteps=10, reps=12):
    """BASELINE config 3 at its batch: whole UnifiedCFM solves of `requests` concurrent requests (CFG pair each) as ONE
    ggml graph with the requests in ggml's batch dimension, through the plugin's graph_compute (recorded at its third
    run, replayed after) and on ggml-cpu."""
    import reflib
    ref = reflib.load_ref()
    if ref is None:
        return None
    params = reflib.backbone_params("bench-locdit", 1)
    lw = params["layers"][0]
    params["dims"]["n_layer"] = layers
    params["layers"] = [lw] * layers
    cp = reflib.cfm_params("bench-cfm")
    T = 2 * (1 + prefix + patch)
    rs = np.random.default_rng(12)
    z, mu = rs.standard_normal((requests, patch, 64)).astype(np.float32), rs.standard_normal((requests, 1024)).astype(np.float32)
    cond, table = rs.standard_normal((requests, prefix, 64)).astype(np.float32), rs.standard_normal((timesteps, 1024)).astype(np.float32)

    def run(device, n_threads, n):
        assert ref.rh_use_device(device, n_threads, 0) == 0
        try:
            reflib.ref_backbone_create(params, T, requests, use_mup=False, kv_f16=False, fused_weights=True)
            reflib.ref_cfm_create(cp)
            _, _, n_nodes = reflib.ref_cfm_solve(z, mu, cond, table, n_steps=timesteps, reps=n)
            return reflib.ref_last_times(), n_nodes
        finally:
            ref.rh_cfm_free()
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", threads, 0) == 0

    assert ref.rh_load_plugin(pkg.PLUGIN_PATH.encode()) == 0
    times, n_nodes = run(b"GFX950_0", 1, reps)
    plug = C.CDLL(pkg.PLUGIN_PATH)
    st = stats(times[3:])   # the first runs are launched group by group while the graph is being recognised
    res = {"requests": requests, "ms_per_batch_of_solves": {n: st[n] * 1e3 for n in ("mean", "median", "p90", "best")},
           "us_per_request_solve": st["mean"] / requests * 1e6, "solves_per_s": requests / st["mean"],
           "first_runs_ms": [t * 1e3 for t in times[:3]], "graph_nodes": n_nodes, "launches": plug.ggml_backend_gfx950_last_launches(),
           "how": "ONE ggml graph for all requests (batch dimension), ggml_backend_graph_compute on libggml-gfx950.so, synchronised per call; "
                  "replayed as a recorded HIP graph from the third run"}
    if with_cpu:
        ctimes, _ = run(b"CPU", threads, 3)
        cs = stats(ctimes)
        res["ggml_cpu"] = {"ms_per_batch_of_solves": cs["mean"] * 1e3, "threads": threads, "sample": "3 repeats of the same graph"}
        res["speedup_vs_ggml_cpu"] = cs["mean"] / st["mean"]
    return res


def load_peaks():
    lib = C.CDLL(os.path.join(ROOT, "voxcpm.cpp_amd", "lib", "libvx_peaks.so"))
    lib.vxp_stream_read.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_void_p]
    lib.vxp_mfma_f16.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.vxp_mfma_f16_flop.argtypes = [C.c_int, C.c_int]
    lib.vxp_mfma_f16_flop.restype = C.c_double
    lib.vxp_grid_barrier.argtypes = [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    lib.vxp_coexec.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.vxp_lds_read.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
    lib.vxp_fill_rate.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_void_p, C.c_void_p]
    return lib


def peaks_bench(timer):
    """What this box delivers on the two simplest kernels: a streaming read (1 GiB at once; and 64 MiB per launch over 24
    distinct buffers, the size and reuse pattern of the headline attention call) and a loop of independent f16 MFMAs."""
    import torch
    lib = load_peaks()
    st = lambda: torch.cuda.current_stream().cuda_stream
    sink = torch.zeros(1 << 20, dtype=torch.int32, device="cuda")
    big = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
    big.fill_(1)
    s_big = timer.run(lambda: lib.vxp_stream_read(big.data_ptr(), big.numel(), sink.data_ptr(), 0, st()), iters=20, warmup=3)
    chunk = 64 << 20
    parts = [big[i * chunk:(i + 1) * chunk] for i in range(16)] + [torch.ones(chunk, dtype=torch.uint8, device="cuda") for _ in range(8)]

    def sweep():
        for p_ in parts:
            lib.vxp_stream_read(p_.data_ptr(), chunk, sink.data_ptr(), 0, st())

    s_chunk = timer.run(sweep, iters=10, warmup=2) / len(parts)
    fsink = torch.zeros(4096 * 256, dtype=torch.float32, device="cuda")
    blocks, iters = 2048, 4096
    s_mfma, _ = timer.sustained(lambda: lib.vxp_mfma_f16(blocks, iters, fsink.data_ptr(), st()), 5)
    # a barrier across a resident grid: 1000 rounds a launch, the counter cleared by a fill kernel before each
    flags = torch.zeros(2, dtype=torch.int32, device="cuda")
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    barrier = {}
    for per_cu in (1, 2):
        for ordered in (0, 1):
            rounds = 1000

            def one():
                flags.zero_()
                rc = lib.vxp_grid_barrier(per_cu * cus, rounds, ordered, flags.data_ptr(), flags.data_ptr() + 4, st())
                assert rc == 0, rc

            empty = timer.run(lambda: flags.zero_(), iters=10, warmup=2)
            s_bar = timer.run(one, iters=5, warmup=2)
            assert int(flags[1].item()) == 0, "a work-group gave up waiting at the grid barrier"
            barrier[f"{per_cu * cus}_work_groups_{'release_acquire' if ordered else 'relaxed'}_us"] = (s_bar - empty) / rounds * 1e6
    # two instruction streams on one SIMD (waves 0-3 and 4-7 of an 8-wave work-group): alone and in pairs
    names = {1: "mfma", 2: "fma", 3: "exp"}
    coexec = {}
    it_ = 20000
    for ra, rb in ((1, 0), (2, 0), (3, 0), (1, 1), (2, 2), (3, 3), (1, 2), (1, 3), (2, 3)):
        s_co = timer.run(lambda: lib.vxp_coexec(cus, ra, rb, it_, fsink.data_ptr(), st()), iters=3, warmup=1)
        coexec[names[ra] + ("_alone" if rb == 0 else "_with_" + names[rb])] = s_co / it_ * 1e9
    coexec["unit"] = ("ns per iteration of a wave: mfma = 4 independent v_mfma_f32_32x32x16_f16 (128 cycles), fma = 32 v_fma_f32 in 8 chains, "
                      "exp = 16 v_exp_f32 + 16 v_sub_f32; a pair that ran side by side would take the longer of its two times alone")
    # LDS read rate per compute unit (16-byte reads, 8 per iteration and wave) and a compute unit's fill rate with all pulling
    lds = {}
    lit = 4000
    for waves in (4, 8, 16):
        for same in (0, 1):
            s_l = timer.run(lambda: lib.vxp_lds_read(cus, waves, lit, same, fsink.data_ptr(), st()), iters=3, warmup=1)
            lds[f"{waves}_waves_{'one_address_per_16_lanes' if same else 'lane_contiguous'}_bytes_per_ns_per_cu"] = lit * 8 * waves * 1024 / (s_l * 1e9)
    fill = {}
    per_wg = 8 << 20
    for region in (2 << 20, 16 << 20, 64 << 20):
        s_f = timer.run(lambda: lib.vxp_fill_rate(big.data_ptr(), region, per_wg, cus, sink.data_ptr(), st()), iters=3, warmup=1)
        fill[f"region_{region >> 20}MiB_GB/s_per_cu"] = per_wg / s_f / 1e9
    return {"grid_barrier": barrier, "two_streams_on_one_simd": coexec, "lds_read_16_bytes_per_lane": lds, "fill_rate_all_compute_units_pulling": fill,
            "hbm_stream_read_1GiB_GB/s": big.numel() / s_big / 1e9,
            "hbm_stream_read_64MiB_per_launch_GB/s": chunk / s_chunk / 1e9, "hbm_stream_read_64MiB_us": s_chunk * 1e6,
            "mfma_f16_TFLOP/s": lib.vxp_mfma_f16_flop(blocks, iters) / s_mfma / 1e12,
            "how": "libvx_peaks.so: 16-byte nontemporal loads, 8 in flight per lane, 8 blocks per CU; 8 independent v_mfma_f32_32x32x16_f16 per wave in a loop"}


# ---- profiles/: the rocprofv3 runs behind the committed summaries, and the summariser --------------------------------
SQ_SET_1 = "SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_WAIT_INST_ANY SQ_INSTS_VMEM_RD SQ_INSTS_VALU SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_WAVES"
SQ_SET_2 = "SQ_INSTS_SALU SQ_INSTS_LDS SQ_WAIT_ANY SQ_ACTIVE_INST_ANY SQ_INST_CYCLES_VMEM SQ_ACTIVE_INST_VALU SQ_LDS_BANK_CONFLICT GRBM_GUI_ACTIVE"
TCC_SET = "TCC_HIT_sum TCC_MISS_sum TCC_EA0_RDREQ_sum TCC_REQ_sum"
TCP_SET = "TCP_PENDING_STALL_CYCLES_sum TCP_TOTAL_CACHE_ACCESSES_sum TCP_TCC_READ_REQ_sum TCP_TCP_TA_DATA_STALL_CYCLES_sum"
# file stem, bench.py --profile name, title, counter passes (tag, counters), kernels whose counters are listed
PROFILE_RUNS = [
    ("decode_attn_B16_L8192", "decode5", "Decode attention, batch 16, 8192 keys, 2 KV heads x 8 query heads, head_dim 64, f16 K/V",
     [("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE"), ("sq1", SQ_SET_1), ("sq2", SQ_SET_2), ("tcc", TCC_SET), ("tcp", TCP_SET)], "fattn"),
    ("decode_attn_B2_L4096", "decode2", "Decode attention, batch 2, 4096 keys, 2 KV heads x 8 query heads, head_dim 64, f16 K/V",
     [("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")], "fattn"),
    ("prefill_attn_cfg5_T4096_B16", "prefill", "Prefill attention, 16 sequences x 4096 tokens, 16 query / 2 KV heads, head_dim 64 (BASELINE config 5)",
     [("sq1", SQ_SET_1), ("sq2", SQ_SET_2)], "pf_"),
    ("prefill_attn_cfg5_T4096_B1", "prefill1", "Prefill attention, one sequence of 4096 tokens, 16 query / 2 KV heads, head_dim 64",
     [("sq1", SQ_SET_1), ("sq2", SQ_SET_2)], "pf_"),
    ("mul_mat_q8_0_4096x1024x16384", "gemm", "Q8_0 MUL_MAT, 4096 rows x K 1024 x 16384 tokens (the gate/up projection of 16 x 1024 prefill tokens)",
     [("sq1", SQ_SET_1), ("sq2", SQ_SET_2), ("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")], "gemm|mm_|qt_"),
    ("backbone_decode_cfg4", "backbone", "Backbone decode step, 24 layers, batch 2, Q8_0 weights, f16 KV cache at ~520 keys (BASELINE config 4)", [], ""),
    ("backbone_decode_cfg5", "backbone16", "Backbone stack at BASELINE config 5 (batch 16, f16 KV 4096 -> 8192, prefill 16 x 4096)", [], ""),
    ("cfm_solve_cfg3", "cfm", "One UnifiedCFM solve of one request (10 Euler steps, CFG pair as one 14-token sequence, 4 LocDiT layers; BASELINE config 3)", [], ""),
    ("cfm_solve_cfg3_8_requests", "cfm8", "UnifiedCFM solves of 8 concurrent requests as one ggml graph through the plugin (BASELINE config 3 at its batch)", [], ""),
]


def profile_commands(raw):
    """The rocprofv3 runs of PROFILE_RUNS, one per line as 'name<TAB>command' (each is its own process; run them from
    /tmp with TMPDIR=/tmp, every line under a time limit of its own).  Outputs go under `raw`."""
    here = os.path.abspath(__file__)
    out = []
    for stem, prof, _, passes, _ in PROFILE_RUNS:
        out.append((f"kt_{prof}", f"rocprofv3 --kernel-trace --stats --output-format csv -d {raw}/kt_{prof} -o kt -- python3 {here} --profile {prof}"))
        for tag, counters in passes:
            out.append((f"pmc_{prof}_{tag}", f"rocprofv3 --pmc {counters} --output-format csv -d {raw}/pmc_{prof}_{tag} -o pm -- python3 {here} --profile {prof}"))
    for tag, counter in (("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")):
        out.append((f"cal_{tag}", f"rocprofv3 --pmc {counter} --output-format csv -d {raw}/cal_{tag} -o pm -- python3 {here} --calibrate-copy"))
    return out


def summarize_profiles(raw, out, commit):
    """Writes profiles/*.txt from the raw rocprofv3 output of profile_commands(): per kernel the calls and average
    duration, per counter pass the mean / min / max over dispatches, and for FETCH_SIZE / WRITE_SIZE the traffic scaled
    by what the same counter reads on a copy of known size."""
    import collections
    import csv
    import glob

    def kstats(d):
        rows = []
        for f in glob.glob(d + "/**/*kernel_stats.csv", recursive=True):
            for r in csv.DictReader(open(f)):
                rows.append((r["Name"], int(r["Calls"]), float(r["AverageNs"]), float(r["TotalDurationNs"]), float(r["Percentage"])))
        return sorted(rows, key=lambda r: -r[3])

    def counters(d):
        acc = collections.defaultdict(list)
        for f in glob.glob(d + "/**/*counter_collection.csv", recursive=True):
            for r in csv.DictReader(open(f)):
                acc[(r["Kernel_Name"], r["Counter_Name"])].append(float(r["Counter_Value"]))
        return acc

    def short(n, w=100):
        return n.replace("(anonymous namespace)::", "").replace("void ", "")[:w]

    def ours(n):
        return "at::native" not in n and "rocclr" not in n and "elementwise_kernel" not in n

    def bench_line(name):
        try:
            lines = [ln for ln in open(f"{raw}/{name}.log").read().split("\n") if ln.startswith("{")]
            return lines[-1][:2500]
        except OSError as e:
            return f"(no log: {e})"

    cal = {}
    for tag in ("fetch", "write"):
        vals = max((v for (k, c), v in counters(f"{raw}/cal_{tag}").items() if "elementwise" in k), key=len, default=None)
        if vals and len(vals) > 1:
            mean = sum(vals[1:]) / len(vals[1:])
            cal[tag] = (mean, 262144.0 / mean)
    os.makedirs(out, exist_ok=True)
    import re
    for stem, prof, title, passes, kernels in PROFILE_RUNS:
        ks = kstats(f"{raw}/kt_{prof}")
        if not ks:
            print(f"summarize: no kernel trace for {prof}, {stem} left alone", file=sys.stderr)
            continue
        cmds = dict(profile_commands("<out>"))
        here = os.path.abspath(__file__)
        with open(f"{out}/{stem}_kernel_trace{'_and_counters' if passes else ''}.txt", "w") as f:
            f.write(f"{title}\ncommit: {commit}\nOne MI355X (gfx950), rocprofv3 run from /tmp with TMPDIR=/tmp; every run is its own process.\nCommands:\n")
            for name in [f"kt_{prof}"] + [f"pmc_{prof}_{t}" for t, _ in passes] + (["cal_fetch", "cal_write"] if any(t in ("fetch", "write") for t, _ in passes) else []):
                f.write("  " + cmds[name].replace(here, "bench.py") + "\n")
            f.write(f"\nbench.py's own line of the kernel-trace run:\n  {bench_line('kt_' + prof)}\n\n")
            f.write(f"  {'kernel':100s} {'calls':>7s} {'avg us':>9s} {'total ms':>9s} {'%':>6s}\n")
            for n, c, a, t, p in [r for r in ks if ours(r[0])][:16]:
                f.write(f"  {short(n):100s} {c:7d} {a / 1e3:9.2f} {t / 1e6:9.3f} {p:6.2f}\n")
            scaled = {}
            for tag, _ in passes:
                acc = counters(f"{raw}/pmc_{prof}_{tag}")
                note = " (SQ cycle counters count in units of four cycles)" if tag.startswith("sq") else " (KiB)" if tag in cal else ""
                f.write(f"\nCounters per dispatch, pass '{tag}'{note}:\n")
                for (k, c), v in sorted(acc.items()):
                    if ours(k) and re.search(kernels, k):
                        f.write(f"  {short(k, 72):72s} {c:34s} n={len(v):5d} mean {sum(v) / len(v):15.1f} min {min(v):15.1f} max {max(v):15.1f}\n")
                        if tag in cal:
                            scaled[(tag, short(k, 72))] = sum(v) / len(v) * cal[tag][1]
            if scaled:
                f.write("\nCalibration (torch elementwise copy kernel, 262144 KiB read and 262144 KiB written per launch, first launch excluded):\n")
                for tag in ("fetch", "write"):
                    if tag in cal:
                        f.write(f"  {tag.upper()}_SIZE mean {cal[tag][0]:.1f} KiB -> factor {cal[tag][1]:.3f}\n")
                f.write("Scaled HBM traffic per dispatch (KiB):\n")
                for (tag, k), v in sorted(scaled.items()):
                    f.write(f"  {tag:6s} {k:72s} {v:12.0f}\n")
                f.write(f"traffic_bytes_per_call: {int(sum(scaled.values()) * 1024)}   (every kernel above, reads plus writes)\n")
    peaks_log = f"{raw}/peaks.log"
    if os.path.exists(peaks_log):
        with open(f"{out}/peaks_measured.txt", "w") as f:
            f.write(f"What the box delivers on the simplest kernels (libvx_peaks.so)\ncommit: {commit}\nCommand:\n  python3 bench.py --profile peaks\n\n")
            f.write(open(peaks_log).read().strip().split("\n")[-1] + "\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-others", action="store_true", help="skip the secondary workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the ggml-cpu baselines")
    ap.add_argument("--eager", action="store_true", help="launch every call from Python instead of replaying a HIP graph")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run only a plain 256 MiB -> 256 MiB elementwise copy kernel a few times (the known-size "
                         "launch that hardware byte counters are scaled by) and exit")
    ap.add_argument("--profile-commands", metavar="RAW", default=None, help="print the rocprofv3 runs behind profiles/ (name, tab, command), outputs under RAW")
    ap.add_argument("--summarize", nargs=3, metavar=("RAW", "OUT", "COMMIT"), default=None, help="write profiles/*.txt from the raw output of those runs")
    ap.add_argument("--profile", choices=["decode5", "decode2", "prefill", "prefill1", "backbone", "backbone16", "cfm", "cfm8", "gemm", "peaks"], default=None,
                    help="run only this workload a few times (for rocprofv3) and print its figures")
    args = ap.parse_args()
    if args.profile_commands:
        for name, cmd in profile_commands(args.profile_commands):
            print(f"{name}\t{cmd}")
        return
    if args.summarize:
        summarize_profiles(*args.summarize)
        return
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

    if args.profile in ("decode5", "decode2"):   # the decode attention call alone, eager, every layer's own cache
        b, L = (16, 8192) if args.profile == "decode5" else (2, 4096)
        st, one, keep = decode_attn_setup(pkg, b, L, LAYERS)
        s = timer.run(st, iters=5, warmup=2) / LAYERS
        print(json.dumps({"profile": f"decode_attn_B{b}_L{L}", "us_per_call": s * 1e6, "GB/s": kv_bytes(b, L) / s / 1e9,
                          "calls": 7 * LAYERS, "bytes_per_call": kv_bytes(b, L)}))
        return
    if args.profile == "peaks":
        print(json.dumps({"profile": "peaks", **peaks_bench(timer)}))
        return
    if args.profile in ("prefill", "prefill1"):   # config 5 prefill attention, 16 streams (or one) x 4096 tokens
        nb = 16 if args.profile == "prefill" else 1
        call, flops, keep = prefill_attn_setup(pkg, nb, 4096)
        s, s_first = timer.sustained(call, 20 if nb == 16 else 100)
        print(json.dumps({"profile": f"cfg5_prefill_attn_T4096_B{nb}", "us": s * 1e6, "TFLOP/s_causal_exact": flops / s / 1e12,
                          "mfma_frac": flops / s / 1e12 / MFMA_F16_PEAK_TFLOPS, "first_round_us": s_first * 1e6,
                          "how": "median of 6 back-to-back rounds; the first round runs while the clocks still step up"}))
        return
    if args.profile == "gemm":      # the prefill-sized Q8_0 projection, 4096 rows x 1024 x 16384 tokens
        M, K, N = 4096, 1024, 16384
        call, keep = q8_proj_setup(pkg, M, K, N)
        s = timer.run(call, iters=5, warmup=2)   # the first calls of a process: the clocks have not settled under the load yet
        # then in turns, so that both see the same clocks: the weights' tiles made on every call / made once and kept
        # (vx_weights_pin), 4 rounds of 25 calls each
        turns = pinned_in_turns(pkg, timer, call, keep[0], 4, 25)
        flops = 2.0 * M * K * N
        fig = lambda v: {"us": v * 1e6, "TFLOP/s": flops / v / 1e12, "mfma_frac": flops / v / 1e12 / MFMA_F16_PEAK_TFLOPS}
        print(json.dumps({"profile": "q8_0_mul_mat_4096x1024x16384", **fig(s), "how": "the first 5 calls of the process after 2 warm-up calls",
                          "sustained": {k: {**fig(float(np.median(v))), "rounds_us": [x * 1e6 for x in v]} for k, v in turns.items()},
                          "VX_GEMM_LDS": os.environ.get("VX_GEMM_LDS", "1")}))
        return
    if args.profile == "cfm":       # config 3: whole CFM solves of one request, replayed from a HIP graph
        print(json.dumps({"profile": "cfg3_cfm_solve_one_request", **cfm_solve_bench(pkg, timer, torch.cuda.Stream(), 1, False)}))
        return
    if args.profile == "cfm8":      # config 3 at its batch: 8 requests' solves as one graph through the plugin
        print(json.dumps({"profile": "cfg3_cfm_solve_8_requests_through_plugin", **cfm_requests_bench(pkg, 1, False)}))
        return
    if args.profile == "backbone":  # config 4 decode steps (f16 cache)
        print(json.dumps({"profile": "cfg4_backbone_24layers_b2", **backbone_bench(pkg, timer, torch.cuda.Stream(), 1, False, steps=128, kv_f16=True, plugin_reps=5)}))
        return
    if args.profile == "backbone16":  # config 5 decode steps (f16 cache)
        print(json.dumps({"profile": "cfg5_backbone_24layers_b16", **backbone_bench(pkg, timer, torch.cuda.Stream(), 1, False, batch=16, prefill=4096,
                                                                                     steps=4096, kv_f16=True, plugin_reps=3)}))
        return

    # ---- headline: config 5 decode attention, batch 16, 8192 keys, 24 layers ------------------------
    B, L = 16, 8192
    side = torch.cuda.Stream()
    step_eager, one_layer, keep = decode_attn_setup(pkg, B, L, LAYERS)
    eager_sec = timer.run(step_eager, iters=10)
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

    # dominant kernel: one vx_flash_attn_ext call (split-KV kernel + the merge of its partials), HIP events on the launch stream
    launch_sec = timer.run(step, iters=100, warmup=10) / LAYERS
    achieved = kv_bytes(B, L) / launch_sec / 1e9
    traffic, traffic_commit = measured_traffic(B, L)
    peaks = peaks_bench(timer)
    roofline = {"bound": "hbm", "kernel": "fattn_dec64_kernel + fattn_merge_kernel<64>", "achieved": achieved,
                "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                "traffic_source": (f"profiles/decode_attn_B{B}_L{L}_kernel_trace_and_counters.txt (rocprofv3 FETCH_SIZE + WRITE_SIZE scaled by a plain copy, taken at commit {traffic_commit})"
                                   if traffic else None),
                "achievable_peak": peaks["hbm_stream_read_64MiB_per_launch_GB/s"],
                "frac_of_achievable": achieved / peaks["hbm_stream_read_64MiB_per_launch_GB/s"],
                "achievable_peak_is": "a plain streaming read of 64 MiB per launch over 24 distinct buffers, measured in this run (libvx_peaks.so); "
                                      f"1 GiB in one launch: {peaks['hbm_stream_read_1GiB_GB/s']:.0f} GB/s",
                "launch_us": launch_sec * 1e6, "bytes_per_launch": kv_bytes(B, L),
                "note": "average over the 24 calls of a graph-replayed step, each two kernels (HIP events on the launch stream)"}
    del keep, step, step_eager, one_layer
    torch.cuda.empty_cache()

    others = {"peaks_measured_on_this_box": peaks}
    if not args.no_others:
        for L2 in (128, 512, 2048, 4096):
            st, one, keep = decode_attn_setup(pkg, 2, L2, LAYERS)
            s = timer.run(graphed(st, side), iters=50)
            others[f"cfg2_decode_attn_B2_L{L2}"] = {"us_per_layer": s / LAYERS * 1e6, "GB/s": LAYERS * kv_bytes(2, L2) / s / 1e9,
                                                     "hbm_frac": LAYERS * kv_bytes(2, L2) / s / 1e9 / HBM_PEAK_GBS}
            del keep, st, one
        for name, b, T, it in (("cfg1_prefill_attn_T256", 1, 256, 200), ("cfg5_prefill_attn_T4096_B1", 1, 4096, 100),
                                  ("cfg5_prefill_attn_T4096_B16", 16, 4096, 20)):
            call, flops, keep = prefill_attn_setup(pkg, b, T)
            s, s_first = timer.sustained(call, it)
            others[name] = {"us": s * 1e6, "TFLOP/s_causal_exact": flops / s / 1e12,
                            "mfma_frac": flops / s / 1e12 / MFMA_F16_PEAK_TFLOPS,
                            "frac_of_measured_mfma_loop": flops / s / 1e12 / peaks["mfma_f16_TFLOP/s"],
                            "how": f"median of 6 back-to-back rounds of {it} calls; the first round (the clocks still stepping up): "
                                   f"{s_first * 1e6:.1f} us, {flops / s_first / 1e12:.0f} TFLOP/s"}
            del keep, call
        solve, n_calls, keep = locdit_attn_setup(pkg)
        s = timer.run(graphed(solve, side), iters=20)
        others["cfg3_locdit_attn_16seq_x7"] = {"us_per_cfm_solve": s * 1e6, "launches_per_solve": n_calls,
                                               "us_per_attention": s / n_calls * 1e6}
        del keep, solve
        for name, M, K, N in (("q8_0_proj_1024x1024_n2", 1024, 1024, 2), ("q8_0_ffn_up_4096x1024_n2", 4096, 1024, 2),
                              ("q8_0_proj_1024x1024_n1024", 1024, 1024, 1024), ("q8_0_ffn_up_4096x1024_n1024", 4096, 1024, 1024),
                              ("q8_0_proj_1024x1024_n16384", 1024, 1024, 16384), ("q8_0_ffn_up_4096x1024_n16384", 4096, 1024, 16384)):
            call, keep = q8_proj_setup(pkg, M, K, N)
            if N <= 16:   # a few microseconds a call: 64 calls replayed from one HIP graph, so that the kernel is timed and not Python
                def many(call=call):
                    for _ in range(64):
                        call()
                s = timer.run(graphed(many, side), iters=50, warmup=5) / 64
            else:
                s, _ = timer.sustained(call, 200 if N <= 1024 else 20)
            wbytes = M * K // 32 * 34
            others[name] = {"us": s * 1e6, "weight_GB/s": wbytes / s / 1e9, "TFLOP/s": 2.0 * M * K * N / s / 1e12,
                            "launch": "64 calls per HIP graph replay (the same weights: they stay in cache)" if N <= 16 else "eager"}
            if N >= 16384 and M >= 4096:   # the same call in turns with the weights declared constant (vx_weights_pin: their tiles are made once)
                turns = pinned_in_turns(pkg, timer, call, keep[0], 3, 20)
                others[name]["in_turns"] = {k: {"us": float(np.median(v)) * 1e6, "TFLOP/s": 2.0 * M * K * N / float(np.median(v)) / 1e12,
                                                "rounds_us": [x * 1e6 for x in v]} for k, v in turns.items()}
            del keep, call
        torch.cuda.empty_cache()

    threads = min(16, os.cpu_count() or 1)   # a one-GPU box's share of the host
    if not args.no_others:
        cpu_on = not args.no_cpu
        # BASELINE config 4 with the reference's F32 cache and with the f16 cache BASELINE's configs name
        others["cfg4_backbone_24layers_b2"] = backbone_bench(pkg, timer, side, threads, cpu_on, f32_prefill_switch=True)
        others["cfg4_backbone_24layers_b2_f16kv"] = backbone_bench(pkg, timer, side, threads, False, kv_f16=True)
        others["cfg3_locdit_stack_8req_x14"] = locdit_stack_bench(pkg, timer, side, threads, cpu_on)
        others["cfg3_cfm_solve_one_request"] = cfm_solve_bench(pkg, timer, side, threads, cpu_on)
        others["cfg3_cfm_solve_8_requests_through_plugin"] = cfm_requests_bench(pkg, threads, cpu_on)
        # BASELINE config 5 as a whole stack: 8 streams x CFG pair (batch 16), prefill 4096 tokens, decode from 4096 to 8192
        others["cfg5_backbone_24layers_b16_f16kv"] = backbone_bench(pkg, timer, side, threads, cpu_on, batch=16, prefill=4096, steps=4096,
                                                                    kv_f16=True, cpu_reps=3, cpu_prefill=False, plugin_reps=10)
        others["cfg5_backbone_24layers_b16"] = backbone_bench(pkg, timer, side, threads, False, batch=16, prefill=4096, steps=4096,
                                                              kv_f16=False, plugin_reps=0)

    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(B, L, threads)

    def pick(name, *path):
        v = others.get(name, {})
        for k_ in path:
            v = v.get(k_, {}) if isinstance(v, dict) else {}
        return v if not isinstance(v, dict) else None

    line = {
        # BASELINE.json's metric, verbatim; `value` is its decode component on config 5 (see config.value_is),
        # the prefill TFLOP/s and backbone steps/s components are repeated under "components"
        "metric": "attn TFLOP/s (prefill) & HBM GB/s (decode) vs roofline; backbone decode steps/s",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": sec_per_step * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 K/V, f32 accumulate", "data": "synthetic (seeded N(0,1))",
        "config": {"workload": f"BASELINE config 5 decode: 24 layers x GQA decode attention, 16/2 heads, head_dim 64, "
                               f"8 streams x CFG pair (batch {B}), f16 KV length {L}",
                   "value_is": "decode attention HBM GB/s: algorithmic K/V bytes of the 24 calls of a step / wall time of the step",
                   "decode_attn_steps_per_s": 1.0 / sec_per_step,
                   "launch": "eager from Python" if args.eager else "one HIP graph replay per step",
                   "eager_python_ms_per_step": eager_sec * 1e3},
        "roofline": roofline,
        "cpu_baseline": cpu,
        "components": {
            "decode_attn_GB/s_cfg5_B16_L8192": value,
            "decode_attn_hbm_frac_cfg5_B16_L8192": value / HBM_PEAK_GBS,
            "decode_attn_GB/s_cfg2_B2_L4096": pick("cfg2_decode_attn_B2_L4096", "GB/s"),
            "prefill_attn_TFLOP/s_cfg5_T4096_B16": pick("cfg5_prefill_attn_T4096_B16", "TFLOP/s_causal_exact"),
            "prefill_attn_mfma_frac_cfg5_T4096_B16": pick("cfg5_prefill_attn_T4096_B16", "mfma_frac"),
            "prefill_attn_mfma_frac_cfg5_T4096_B1": pick("cfg5_prefill_attn_T4096_B1", "mfma_frac"),
            "backbone_decode_steps_per_s_cfg4": pick("cfg4_backbone_24layers_b2", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg4_f16kv": pick("cfg4_backbone_24layers_b2_f16kv", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg4_through_plugin": pick("cfg4_backbone_24layers_b2", "plugin_graph_compute", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg4_through_plugin_same_graph_replayed": pick("cfg4_backbone_24layers_b2", "plugin_graph_compute", "same_graph_replayed", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg4_f16kv_through_plugin_consecutive_steps": pick("cfg4_backbone_24layers_b2_f16kv", "plugin_graph_compute", "consecutive_steps", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg5_f16kv_through_plugin_consecutive_steps": pick("cfg5_backbone_24layers_b16_f16kv", "plugin_graph_compute", "consecutive_steps", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg4_ggml_cpu": pick("cfg4_backbone_24layers_b2", "ggml_cpu", "decode_steps_per_s"),
            "backbone_decode_steps_per_s_cfg5_f16kv": pick("cfg5_backbone_24layers_b16_f16kv", "decode_steps_per_s"),
            "backbone_prefill_tokens_per_s_cfg4": pick("cfg4_backbone_24layers_b2", "prefill_tokens_per_s"),
            "backbone_prefill_tokens_per_s_cfg5_f16kv": pick("cfg5_backbone_24layers_b16_f16kv", "prefill_tokens_per_s"),
            "cfm_solve_us_cfg3_one_request": pick("cfg3_cfm_solve_one_request", "us_per_cfm_solve"),
            "cfm_solves_per_s_cfg3_8_requests_through_plugin": pick("cfg3_cfm_solve_8_requests_through_plugin", "solves_per_s"),
        },
        "others": others,
    }
    print(json.dumps(line, allow_nan=False))


if __name__ == "__main__":
    main()
