"""BASELINE configurations 4 and 5 at their full sizes, against the reference's ggml-cpu (oracle/_ref).

cfg 4: the 24-layer backbone, batch 2, a 512-token prefill and then all 256 decode steps; every call runs on ggml-cpu,
       on the plugin (the reference-structured graph through ggml's graph_compute) and on the C-ABI mirror, each backend
       reading the cache it wrote itself; outputs are compared at the prefill and at KV lengths 512, 640 and 767.
cfg 5: 8 streams x CFG pair (batch 16), an f16 KV cache already holding 4096+ seeded tokens, one decode step through the
       stack; and the 16 x 4096-token prefill attention against the oracle on sampled rows.

Bars.  ggml-cpu quantises the activations of every product to int8 blocks (a step of amax/127 per block).  VX_ACT_FLOAT
rounds them to f16 instead, so the two stacks differ by ggml-cpu's own quantisation noise, which the residual stream
carries along without amplifying it: measured 2.0e-5 .. 2.5e-5 NMSE at 24 layers, the same as at 3.  VX_ACT_Q8 repeats
ggml-cpu's integer arithmetic product by product (1e-5 relative, tests/test_gpu_parity.py), but a stack of quantisers is
not continuous: a difference d in front of a quantiser of step s comes out with mean square d*s (a rounding flips with
probability d/s and then moves the value by s), so differences of one ulp in a summation order grow layer by layer to
the step itself and the stacks decorrelate to the same noise level, 2.1e-5 .. 2.4e-5 measured.  The bar is 1e-4 for both
modes (ggml's own per-operator bar in test-backend-ops is 5e-4).  The mirror runs the plugin's launches on buffers of its
own: the same kernels on the same values, bit for bit in both modes."""
import ctypes
import sys

import numpy as np
import pytest

import reflib
from reflib import nmse, rng

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def load_mirror(gpu, params, n_layer, max_len, batch, use_mup, kv_f16, act):
    import torch
    from voxcpm_cpp_amd import backbone as bb
    m = bb.MiniCPMBackbone(n_layer=n_layer, max_length=max_len, batch=batch, use_mup=use_mup, kv_f16=kv_f16, act_mode=act)
    for li, lw in enumerate(params["layers"]):
        for n in reflib.BB_WEIGHTS:
            m.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
        for n in ("input_layernorm", "post_layernorm"):
            m.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
    m.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
    m.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
    return m


@pytest.mark.parametrize("act", ["float", "q8"])
def test_backbone_cfg4_full(gpu, ref, act):
    """24 layers, batch 2, prefill 512, 256 decode steps (src/minicpm.cpp:749-846 is the loop this follows)."""
    import torch
    N_LAYER, BATCH, T0, STEPS = 24, 2, 512, 256
    MAX_LEN = T0 + STEPS
    check_at = {0: "prefill", 1: "KV 512", 129: "KV 640", 256: "KV 767"}   # call index -> label
    act_mode = gpu.ACT_Q8 if act == "q8" else gpu.ACT_FLOAT
    bar = 1e-4
    say(f"cfg 4 at full size: {N_LAYER} layers, batch {BATCH}, prefill {T0} + {STEPS} decode steps, activations {act}")
    params = reflib.backbone_params("bb4", N_LAYER)
    xs = [rng("bb4", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)]
    xs += [rng("bb4", "x", i + 1).standard_normal((BATCH, 1, 1024)).astype(np.float32) for i in range(STEPS)]
    mask0 = reflib.causal_mask(T0, T0)

    def run(device, threads):
        assert ref.rh_use_device(device, threads, 0) == 0
        reflib.ref_backbone_create(params, MAX_LEN, BATCH, use_mup=True, kv_f16=False)
        outs, n_past = {}, 0
        for i, x in enumerate(xs):
            o, _, _ = reflib.ref_backbone_forward(x, n_past, mask0 if i == 0 else None)
            if i in check_at:
                outs[i] = o
            n_past += x.shape[1]
        ref.rh_bb_free()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return outs

    say("   ggml-cpu ...")
    cpu = run(b"CPU", 16)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plugin = ctypes.CDLL(gpu.PLUGIN_PATH)
    before = plugin.ggml_backend_gfx950_set_mul_mat_act(act_mode)
    try:
        say("   plugin ...")
        plug = run(b"GFX950_0", 8)
    finally:
        plugin.ggml_backend_gfx950_set_mul_mat_act(before)
    launches = plugin.ggml_backend_gfx950_last_launches()
    say(f"   plugin: {launches} launches for the last decode step")
    assert launches == N_LAYER * 5 + 1
    for i, label in check_at.items():
        e = nmse(cpu[i], plug[i])
        say(f"   plugin vs ggml-cpu at {label}: nmse {e:.3e}")
        assert np.isfinite(plug[i]).all() and e <= bar, (label, e)

    say("   C-ABI mirror ...")
    m = load_mirror(gpu, params, N_LAYER, MAX_LEN, BATCH, True, False, act_mode)
    n_past = 0
    for i, x in enumerate(xs):
        T = x.shape[1]
        run_, got = m.plan(torch.from_numpy(x).cuda(), T, n_past, torch.from_numpy(mask0).cuda() if i == 0 else None)
        run_()
        if i in check_at:
            torch.cuda.synchronize()
            g = got.cpu().numpy()
            e = nmse(cpu[i], g)
            say(f"   mirror vs ggml-cpu at {check_at[i]}: nmse {e:.3e}")
            assert e <= bar, (check_at[i], e)
            # the mirror issues the plugin's launches on its own buffers: the same kernels on the same values
            assert np.array_equal(g, plug[i]), f"mirror and plugin differ at {check_at[i]}: nmse {nmse(plug[i], g):.3e}"
        n_past += T


@pytest.mark.parametrize("kv_f16", [True, False])
def test_backbone_cfg5_stack_step(gpu, ref, kv_f16):
    """Batch 16 (8 streams x CFG pair), a KV cache that already holds 4100 seeded tokens (f16 as BASELINE config 5 names
    it, and F32 as the reference allocates it), one decode step that appends token 4100, then a second step that reads it
    back: 4 layers, plugin and mirror against ggml-cpu."""
    import torch
    N_LAYER, BATCH, PAST, MAX_LEN = 4, 16, 4100, 4160
    say(f"cfg 5 stack: {N_LAYER} layers, batch {BATCH}, {'f16' if kv_f16 else 'F32'} KV cache holding {PAST} tokens, two decode steps")
    params = reflib.backbone_params("bb5", N_LAYER)
    xs = [rng("bb5", "x", i).standard_normal((BATCH, 1, 1024)).astype(np.float32) for i in range(2)]
    dt = np.float16 if kv_f16 else np.float32
    caches = {}
    for li in range(N_LAYER):
        for w in (0, 1):
            c = np.zeros((BATCH, 2, MAX_LEN, 64), dt)
            c[:, :, :PAST] = rng("bb5", "cache", li, w).standard_normal((BATCH, 2, PAST, 64)).astype(dt)
            caches[(li, w)] = c

    def run(device, threads):
        assert ref.rh_use_device(device, threads, 0) == 0
        reflib.ref_backbone_create(params, MAX_LEN, BATCH, use_mup=True, kv_f16=kv_f16)
        for (li, w), c in caches.items():
            assert ref.rh_bb_cache_set(li, w, c.ctypes.data, c.nbytes) == 0
        outs = [reflib.ref_backbone_forward(x, PAST + i, None)[0] for i, x in enumerate(xs)]
        slot = np.empty_like(caches[(0, 0)])
        assert ref.rh_bb_cache_get(N_LAYER - 1, 0, slot.ctypes.data, slot.nbytes) == 0
        ref.rh_bb_free()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return outs, slot

    cpu, cpu_cache = run(b"CPU", 16)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug, plug_cache = run(b"GFX950_0", 8)
    launches = ctypes.CDLL(gpu.PLUGIN_PATH).ggml_backend_gfx950_last_launches()
    say(f"   plugin: {launches} launches for the decode step")
    for i in range(2):
        e = nmse(cpu[i], plug[i])
        say(f"   plugin vs ggml-cpu, step {i}: nmse {e:.3e}")
        assert np.isfinite(plug[i]).all() and e <= 2e-4
    # the cache: the seeded past untouched, the two appended tokens close to ggml-cpu's
    assert np.array_equal(plug_cache[:, :, :PAST], caches[(N_LAYER - 1, 0)][:, :, :PAST])
    new_cpu, new_plug = cpu_cache[:, :, PAST:PAST + 2].astype(np.float32), plug_cache[:, :, PAST:PAST + 2].astype(np.float32)
    assert np.abs(new_plug).max() > 0 and nmse(new_cpu, new_plug) <= 2e-4
    assert not plug_cache[:, :, PAST + 2:].any()

    m = load_mirror(gpu, params, N_LAYER, MAX_LEN, BATCH, True, kv_f16, gpu.ACT_FLOAT)
    for li in range(N_LAYER):
        m.k_cache[li].copy_(torch.from_numpy(caches[(li, 0)]).cuda())
        m.v_cache[li].copy_(torch.from_numpy(caches[(li, 1)]).cuda())
    for i, x in enumerate(xs):
        run_, got = m.plan(torch.from_numpy(x).cuda(), 1, PAST + i, None)
        run_()
        torch.cuda.synchronize()
        g = got.cpu().numpy()
        e = nmse(cpu[i], g)
        say(f"   mirror vs ggml-cpu, step {i}: nmse {e:.3e} ({run_.n_calls} calls)")
        assert e <= 2e-4
        assert np.array_equal(g, plug[i]), f"mirror and plugin differ at step {i}: nmse {nmse(plug[i], g):.3e}"


def test_fa_cfg5_prefill_b16_t4096(gpu):
    """The 16 x 4096-token causal prefill attention of config 5 (f16 K/V) on the LDS-tiled kernel: every output finite
    and inside the convex hull of its stream's V, and sampled (stream, row) pairs against the oracle -- row r of a causal
    prefill is a decode attention over keys 0..r."""
    import torch
    B, Hq, Hkv, T, D = 16, 16, 2, 4096, 64
    say(f"cfg 5 prefill attention: B={B}, T={T}, {Hq}/{Hkv} heads, f16 K/V, causal")
    q = torch.from_numpy(rng("cfg5pf", "q").standard_normal((B, Hq, T, D)).astype(np.float32)).cuda()
    k = rng("cfg5pf", "k").standard_normal((B, Hkv, T, D)).astype(np.float16)
    v = rng("cfg5pf", "v").standard_normal((B, Hkv, T, D)).astype(np.float16)
    mask = torch.from_numpy(reflib.causal_mask(T, T)).cuda()
    out = gpu.flash_attn_ext(q, torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), mask, 0.125)   # (B, T, Hq, D)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    vf = torch.from_numpy(v.astype(np.float32)).cuda()
    vmin = torch.cummin(vf, dim=2).values   # (B, Hkv, T, D): hull of keys 0..r
    vmax = torch.cummax(vf, dim=2).values
    for h in range(Hq):
        o = out[:, :, h]                     # (B, T, D)
        assert bool((o >= vmin[:, h // 8] - 2e-3).all()) and bool((o <= vmax[:, h // 8] + 2e-3).all()), h
    gen = rng("cfg5pf", "rows")
    pairs = [(0, 0), (0, 1), (15, T - 1), (7, 63), (7, 64), (3, 2047), (3, 2048)] + \
            [(int(gen.integers(B)), int(gen.integers(T))) for _ in range(25)]
    worst = 0.0
    qh = q.cpu().numpy()
    for b, r in pairs:
        want = reflib.oracle_fa(qh[b:b + 1, :, r:r + 1], k[b:b + 1, :, :r + 1].astype(np.float32), v[b:b + 1, :, :r + 1].astype(np.float32))
        err = float(np.abs(out[b, r].cpu().numpy() - want[0, 0]).max())
        worst = max(worst, err)
        assert err <= 2e-3, (b, r, err)
    say(f"   {len(pairs)} sampled rows against the oracle: worst max-abs {worst:.3e}")


def test_backbone_cfg5_prefill_b16_t4096(gpu, ref):
    """Config 5's prefill at its full size through the plugin: 16 sequences x 4096 tokens (65536 tokens a product, the
    causal attention of test_fa_cfg5_prefill_b16_t4096 inside), f16 KV cache, two layers of the stack and the final norm.
    Against ggml-cpu on the whole output and on the cache that the call wrote, and grouped launches against every node
    as its own launch."""
    N_LAYER, BATCH, T = 2, 16, 4096
    say(f"cfg 5 prefill through the plugin: {N_LAYER} layers, {BATCH} x {T} tokens, f16 KV cache")
    params = reflib.backbone_params("bb5p", N_LAYER)
    x = rng("bb5p", "x").standard_normal((BATCH, T, 1024)).astype(np.float32)
    mask = reflib.causal_mask(T, T)

    def run(device, threads):
        assert ref.rh_use_device(device, threads, 0) == 0
        reflib.ref_backbone_create(params, T, BATCH, use_mup=True, kv_f16=True)
        try:
            out = reflib.ref_backbone_forward(x, 0, mask)[0]
            cache = np.empty((BATCH, 2, T, 64), np.float16)
            assert ref.rh_bb_cache_get(N_LAYER - 1, 1, cache.ctypes.data, cache.nbytes) == 0
        finally:
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return out, cache

    say("   ggml-cpu ...")
    cpu, cpu_cache = run(b"CPU", 16)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plugin = ctypes.CDLL(gpu.PLUGIN_PATH)
    say("   plugin ...")
    plug, plug_cache = run(b"GFX950_0", 8)
    launches = plugin.ggml_backend_gfx950_last_launches()
    e, ec = nmse(cpu, plug), nmse(cpu_cache.astype(np.float32), plug_cache.astype(np.float32))
    say(f"   plugin ({launches} launches) vs ggml-cpu: hidden states nmse {e:.3e}, last layer's V cache nmse {ec:.3e}")
    assert np.isfinite(plug).all() and e <= 1e-4 and ec <= 1e-4
    rows = np.abs(cpu - plug).reshape(BATCH * T, -1).max(axis=1) / np.abs(cpu).max()
    say(f"   worst token: {rows.max():.3e} of the largest value (token {int(rows.argmax()) % T} of sequence {int(rows.argmax()) // T})")
    assert rows.max() <= 5e-2
    before = plugin.ggml_backend_gfx950_set_fusion(0)
    try:
        plain, plain_cache = run(b"GFX950_0", 8)
    finally:
        plugin.ggml_backend_gfx950_set_fusion(before)
    plain_launches = plugin.ggml_backend_gfx950_last_launches()
    same = np.array_equal(plain, plug) and np.array_equal(plain_cache, plug_cache)
    say(f"   every node its own launch ({plain_launches} launches): bit-equal to the grouped run: {same}; nmse {nmse(plain, plug):.3e}")
    assert plain_launches > launches
    assert same, "grouped launches changed a result"


@pytest.mark.parametrize("kv_f16", [True, False])
def test_backbone_prompt_lengths_grouped_equals_node_by_node(gpu, ref, kv_f16):
    """A two-layer stack through the plugin at prompt lengths on both sides of every dispatch boundary a prompt crosses --
    the streaming kernel's token limits (16, 64, 204), the three regimes of the cache write (128 / 129 and 512 / 513
    tokens at batch 1), the LDS-tiled attention's minimum, the ROPE kernels' switch at 1024 tokens, the pre-tiled product's
    thresholds --, batch 1 to 3: with node groups on, hidden states and the written cache are bit-equal to every node run
    as its own launch, and finite.  The same for a second chunk of tokens behind cached keys."""
    say(f"plugin prefill, grouped against node by node, over prompt lengths; f16 cache {kv_f16}")
    layers = 2
    params = reflib.backbone_params("bb-lengths", layers)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plugin = ctypes.CDLL(gpu.PLUGIN_PATH)
    assert ref.rh_use_device(b"GFX950_0", 1, 0) == 0
    replay = plugin.ggml_backend_gfx950_set_graph_replay(0)
    lengths = {1: (17, 63, 64, 65, 128, 129, 204, 205, 256, 511, 512, 513, 1023, 1024, 1100, 2048, 4096),
               2: (64, 65, 128, 200, 256, 257, 512, 700, 1024, 2100),
               3: (63, 100, 171, 342, 1000, 1536)}
    try:
        for B, Ts in lengths.items():
            for T in Ts:
                reflib.ref_backbone_create(params, T + 8, B, use_mup=True, kv_f16=kv_f16)
                try:
                    x = rng("bb-lengths", B, T).standard_normal((B, T, 1024)).astype(np.float32)
                    mask = reflib.causal_mask(T, T)
                    runs = []
                    for fusion in (1, 0):
                        before = plugin.ggml_backend_gfx950_set_fusion(fusion)
                        try:
                            out = reflib.ref_backbone_forward(x, 0, mask)[0].copy()
                            cache = np.empty((B, 2, T + 8, 64), np.float16 if kv_f16 else np.float32)
                            assert ref.rh_bb_cache_get(layers - 1, 0, cache.ctypes.data, cache.nbytes) == 0
                        finally:
                            plugin.ggml_backend_gfx950_set_fusion(before)
                        runs.append((out, cache[:, :, :T].copy(), plugin.ggml_backend_gfx950_last_launches()))
                finally:
                    ref.rh_bb_free()
                (o1, c1, l1), (o0, c0, l0) = runs
                assert np.isfinite(o1).all(), (B, T)
                if (B, T) in ((1, 129), (1, 256), (1, 513), (2, 257), (3, 342)):   # and against ggml-cpu where that is quick
                    assert ref.rh_use_device(b"CPU", 16, 0) == 0
                    reflib.ref_backbone_create(params, T + 8, B, use_mup=True, kv_f16=kv_f16)
                    try:
                        cpu = reflib.ref_backbone_forward(x, 0, mask)[0].copy()
                        ccache = np.empty((B, 2, T + 8, 64), np.float16 if kv_f16 else np.float32)
                        assert ref.rh_bb_cache_get(layers - 1, 0, ccache.ctypes.data, ccache.nbytes) == 0
                    finally:
                        ref.rh_bb_free()
                        assert ref.rh_use_device(b"GFX950_0", 1, 0) == 0
                    e, ec = nmse(cpu, o1), nmse(ccache[:, :, :T].astype(np.float32), c1.astype(np.float32))
                    say(f"   batch {B}, {T} tokens ({l1} launches): nmse vs ggml-cpu {e:.3e}, last layer's K cache {ec:.3e}")
                    assert e <= 1e-4 and ec <= 1e-4, (B, T, e, ec)
                assert l1 < l0, (B, T, l1, l0)
                assert np.array_equal(o1, o0) and np.array_equal(c1, c0), f"batch {B}, {T} tokens: {l1} grouped launches differ from {l0} separate ones"
        # and a second chunk behind cached keys (the CONCAT / cast nodes of a step with a past, at prompt sizes)
        for B, T0, T in ((1, 512, 600), (2, 100, 1000), (1, 1024, 64), (1, 2048, 256), (2, 300, 300)):
            runs = []
            for fusion in (1, 0):
                reflib.ref_backbone_create(params, T0 + T + 8, B, use_mup=True, kv_f16=kv_f16)
                before = plugin.ggml_backend_gfx950_set_fusion(fusion)
                try:
                    x0 = rng("bb-lengths", B, T0, "first").standard_normal((B, T0, 1024)).astype(np.float32)
                    reflib.ref_backbone_forward(x0, 0, reflib.causal_mask(T0, T0))
                    x = rng("bb-lengths", B, T, "second").standard_normal((B, T, 1024)).astype(np.float32)
                    out = reflib.ref_backbone_forward(x, T0, reflib.causal_mask(T, T0 + T, T0))[0].copy()
                    cache = np.empty((B, 2, T0 + T + 8, 64), np.float16 if kv_f16 else np.float32)
                    assert ref.rh_bb_cache_get(layers - 1, 0, cache.ctypes.data, cache.nbytes) == 0
                finally:
                    plugin.ggml_backend_gfx950_set_fusion(before)
                    ref.rh_bb_free()
                runs.append((out, cache[:, :, :T0 + T].copy(), plugin.ggml_backend_gfx950_last_launches()))
            (o1, c1, l1), (o0, c0, l0) = runs
            assert np.isfinite(o1).all() and l1 < l0, (B, T0, T, l1, l0)
            assert np.array_equal(o1, o0) and np.array_equal(c1, c0), f"batch {B}, {T} tokens behind {T0}: {l1} grouped launches differ from {l0} separate ones"
    finally:
        plugin.ggml_backend_gfx950_set_graph_replay(replay)
        assert ref.rh_use_device(b"CPU", 8, 0) == 0


def test_mirror_prefill_one_pass_calls_grouped_unfused_and_captured(gpu):
    """A two-layer stack at 16 x 2048 tokens through the C ABI -- the size from which a layer is three one-pass calls
    (vx_norm_qkv_proj_rope with the rotations in the product's epilogue, vx_flash_attn_ext_store_proj, vx_mlp_tiled) --:
    the same bits as every node as its own call, cache included; and captured into a HIP graph, every replay (with other
    work on the stream between them) gives the eager run's bits again."""
    import torch
    from voxcpm_cpp_amd import backbone as bb
    layers, B, T = 2, 16, 2048
    say(f"C ABI mirror, {layers} layers, {B} x {T} tokens: one-pass calls against separate ones, eager and replayed")
    params = reflib.backbone_params("bb-onepass", layers)
    x = torch.from_numpy(rng("bb-onepass", "x").standard_normal((B, T, 1024)).astype(np.float32)).cuda()
    mask = torch.from_numpy(reflib.causal_mask(T, T)).cuda()
    outs, caches, calls = [], [], []
    for fuse in (True, False):
        m = bb.MiniCPMBackbone(n_layer=layers, max_length=T + 8, batch=B, use_mup=True, kv_f16=True, act_mode=gpu.ACT_FLOAT, fuse_pairs=fuse)
        for li, lw in enumerate(params["layers"]):
            for n in reflib.BB_WEIGHTS:
                m.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
            for n in ("input_layernorm", "post_layernorm"):
                m.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
        m.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
        m.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
        run, got = m.plan(x, T, 0, mask)
        run()
        torch.cuda.synchronize()
        outs.append(got.clone()); caches.append(m.k_cache[layers - 1].clone()); calls.append(run.n_calls)
        if fuse:
            fused_model, fused_run, fused_out = m, run, got
    say(f"   {calls[0]} calls against {calls[1]}")
    assert calls[0] == 3 * layers + 1
    assert bool(torch.isfinite(outs[0]).all())
    assert torch.equal(outs[0], outs[1]) and torch.equal(caches[0].view(torch.uint8), caches[1].view(torch.uint8))
    # captured and replayed (two eager runs on the capture stream first: its workspace block must exist before the capture)
    cap = torch.cuda.Stream()
    with torch.cuda.stream(cap):
        for _ in range(2):
            fused_run()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=cap):
        fused_run()
    for rep in range(3):
        fused_out.zero_()
        fused_model.k_cache[layers - 1].zero_()
        (torch.randn(1 << 20, device="cuda") * 2).sum().item()   # other work between the replays
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(fused_out, outs[0]), f"replay {rep}"
        assert torch.equal(fused_model.k_cache[layers - 1].view(torch.uint8), caches[0].view(torch.uint8)), f"replay {rep}: cache"
