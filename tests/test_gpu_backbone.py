"""The whole decoder stack (BASELINE config 4's shape, fewer layers) three ways on the same seeded
Q8_0 weights: the reference-structured ggml graph on ggml-cpu (oracle/_ref), the same graph run
entirely on the gfx950 backend plugin through ggml's own graph_compute, and the host-side
mirror in voxcpm.cpp_amd/backbone.py issuing vx_* calls through the C ABI.  Prefill, then decode
steps that read the KV cache the earlier calls appended."""
import numpy as np
import pytest

import reflib
from reflib import nmse, rng

pytestmark = pytest.mark.gpu

N_LAYER, BATCH, STEPS = 3, 2, 3


def run_reference(params, xs, device, kv_f16, use_mup, max_len):
    ref = reflib.load_ref()
    assert ref.rh_use_device(device, 8, 0) == 0
    reflib.ref_backbone_create(params, max_len, BATCH, use_mup=use_mup, kv_f16=kv_f16)
    outs, n_past = [], 0
    for x in xs:
        T = x.shape[1]
        mask = reflib.causal_mask(T, T) if T > 1 else None
        o, _, n_nodes = reflib.ref_backbone_forward(x, n_past, mask)
        outs.append(o)
        n_past += T
    ref.rh_bb_free()
    assert ref.rh_use_device(b"CPU", 8, 0) == 0
    return outs, n_nodes


# prefill 9: decode attention over a dozen keys (one wave per tile); prefill 300: more than 256 keys, the
# split + merge path with the cache write folded into the merge, as at the benchmark's KV lengths
@pytest.mark.parametrize("kv_f16,use_mup,T0", [(False, True, 9), (True, False, 9), (False, True, 300)])
def test_backbone_three_ways(gpu, ref, kv_f16, use_mup, T0):
    import torch
    from voxcpm_cpp_amd import backbone as bb
    MAX_LEN = T0 + 55
    print(f"backbone: {N_LAYER} layers, batch {BATCH}, prefill {T0} + {STEPS} decode steps, kv_f16={kv_f16} mup={use_mup}", flush=True)
    params = reflib.backbone_params("bb", N_LAYER)
    xs = [rng("bb", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)]
    xs += [rng("bb", "x", i + 1).standard_normal((BATCH, 1, 1024)).astype(np.float32) for i in range(STEPS)]

    cpu, n_nodes = run_reference(params, xs, b"CPU", kv_f16, use_mup, MAX_LEN)
    print(f"   ggml-cpu graph: {n_nodes} nodes per decode step", flush=True)

    # the same ggml graph, every node on the plugin (direct ggml_backend_graph_compute, no scheduler)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug, _ = run_reference(params, xs, b"GFX950_0", kv_f16, use_mup, MAX_LEN)
    import ctypes
    plugin_launches = ctypes.CDLL(gpu.PLUGIN_PATH).ggml_backend_gfx950_last_launches()  # of the last decode step
    print(f"   plugin: {plugin_launches} operator launches for the {n_nodes}-node decode graph", flush=True)
    for i, (a, b) in enumerate(zip(cpu, plug)):
        e = nmse(a, b)
        print(f"   plugin vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
        assert e <= 1e-4

    # the C-ABI mirror, Q8 activations (ggml-cpu's arithmetic) and float activations.  Even with
    # ggml-cpu's integer dots an activation one ulp away can round to the neighbouring int8, so the
    # stack agrees to ~1e-5 NMSE, not bit for bit; float activations sit at ggml's own 5e-4 / op bar.
    unfused = {}
    for act, bar, fuse in ((gpu.ACT_Q8, 5e-5, True), (gpu.ACT_FLOAT, 1e-4, False), (gpu.ACT_FLOAT, 1e-4, True)):
        m = bb.MiniCPMBackbone(n_layer=N_LAYER, max_length=MAX_LEN, batch=BATCH, use_mup=use_mup, kv_f16=kv_f16, act_mode=act,
                               fuse_pairs=fuse)
        for li, lw in enumerate(params["layers"]):
            for n in reflib.BB_WEIGHTS:
                m.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
            for n in ("input_layernorm", "post_layernorm"):
                m.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
        m.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
        m.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
        n_past = 0
        for i, x in enumerate(xs):
            T = x.shape[1]
            mask = torch.from_numpy(reflib.causal_mask(T, T)).cuda() if T > 1 else None
            run, got = m.plan(torch.from_numpy(x).cuda(), T, n_past, mask)
            run()
            if fuse and i == len(xs) - 1:  # the mirror issues exactly what the plugin issues for the reference's graph
                assert run.n_calls == plugin_launches, (run.n_calls, plugin_launches)   # F32 and F16 caches alike
            torch.cuda.synchronize()
            e = nmse(cpu[i], got.cpu().numpy())
            print(f"   C ABI mirror (act_mode {act}, fused pairs {fuse}) vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
            assert e <= bar
            if act == gpu.ACT_FLOAT and not fuse:
                unfused[i] = got.cpu().numpy()
            elif act == gpu.ACT_FLOAT:   # the one-launch pairs round where the separate nodes do
                assert np.array_equal(unfused[i], got.cpu().numpy()), f"fused pairs changed the result of call {i}"
            n_past += T


@pytest.mark.parametrize("kv_f16", [False, True])
@pytest.mark.parametrize("T0", [9, 300])
def test_plugin_groups_fall_back_when_memory_is_reused(gpu, ref, kv_f16, T0):
    """Graph shapes in which ggml-alloc hands the memory of a group's operand to a later node: decode steps that do
    not write the cache (the step's keys die at the CONCAT), repeated steps at one position, and the same with
    grouping switched off.  The plugin must give ggml-cpu's result in all of them, and the grouped and the
    node-by-node runs must agree bit for bit."""
    import ctypes
    import os
    import subprocess
    import sys
    max_len = T0 + 20
    params = reflib.backbone_params("bb", N_LAYER)
    xp = rng("bbf", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)
    xs = [rng("bbf", "x", i + 1).standard_normal((BATCH, 1, 1024)).astype(np.float32) for i in range(3)]

    def run(device):
        assert ref.rh_use_device(device, 8, 0) == 0
        reflib.ref_backbone_create(params, max_len, BATCH, use_mup=True, kv_f16=kv_f16)
        outs = [reflib.ref_backbone_forward(xp, 0, reflib.causal_mask(T0, T0))[0]]
        outs.append(reflib.ref_backbone_forward(xs[0], T0, None, write_kv=False)[0])     # peek: cache untouched
        outs.append(reflib.ref_backbone_forward(xs[1], T0, None, write_kv=False)[0])
        outs.append(reflib.ref_backbone_forward(xs[0], T0, None, write_kv=True)[0])      # now append
        outs.append(reflib.ref_backbone_forward(xs[2], T0 + 1, None, write_kv=False)[0])
        ref.rh_bb_free()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return outs

    cpu = run(b"CPU")
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug = run(b"GFX950_0")
    launches = ctypes.CDLL(gpu.PLUGIN_PATH).ggml_backend_gfx950_last_launches()
    print(f"backbone without cache write: kv_f16={kv_f16} T0={T0}, {launches} launches for the last step", flush=True)
    for i, (a, b) in enumerate(zip(cpu, plug)):
        e = nmse(a, b)
        print(f"   plugin vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
        assert e <= 1e-4
    assert np.array_equal(plug[1], plug[3]), "the appended step must repeat the peeked one"
    # the same calls with every node as its own launch, in a fresh process (the switch is read once)
    code = (
        "import sys, numpy as np; sys.path.insert(0, %r); sys.path.insert(0, %r)\n"
        "import reflib, __graft_entry__ as e\n"
        "from reflib import rng\n"
        "pkg = e.load_package(); ref = reflib.load_ref()\n"
        "assert ref.rh_load_plugin(pkg.PLUGIN_PATH.encode()) == 0 and ref.rh_use_device(b'GFX950_0', 8, 0) == 0\n"
        "params = reflib.backbone_params('bb', %d)\n"
        "reflib.ref_backbone_create(params, %d, %d, use_mup=True, kv_f16=%r)\n"
        "xp = rng('bbf', 'x', 0).standard_normal((%d, %d, 1024)).astype(np.float32)\n"
        "xs = [rng('bbf', 'x', i + 1).standard_normal((%d, 1, 1024)).astype(np.float32) for i in range(3)]\n"
        "o = [reflib.ref_backbone_forward(xp, 0, reflib.causal_mask(%d, %d))[0]]\n"
        "o.append(reflib.ref_backbone_forward(xs[0], %d, None, write_kv=False)[0])\n"
        "o.append(reflib.ref_backbone_forward(xs[1], %d, None, write_kv=False)[0])\n"
        "o.append(reflib.ref_backbone_forward(xs[0], %d, None, write_kv=True)[0])\n"
        "o.append(reflib.ref_backbone_forward(xs[2], %d, None, write_kv=False)[0])\n"
        "np.save(sys.argv[1], np.stack([a.reshape(-1)[:2048] for a in o[1:]]))\n"
    ) % (os.path.dirname(os.path.dirname(os.path.abspath(__file__))), os.path.dirname(os.path.abspath(__file__)), N_LAYER, max_len, BATCH,
         kv_f16, BATCH, T0, BATCH, T0, T0, T0, T0, T0, T0 + 1)
    out_path = f"/tmp/bb_nofusion_{int(kv_f16)}_{T0}.npy"
    env = dict(os.environ, GGML_GFX950_NO_FUSION="1")
    subprocess.run([sys.executable, "-c", code, out_path], check=True, env=env, timeout=200)
    plain = np.load(out_path)
    grouped = np.stack([a.reshape(-1)[:2048] for a in plug[1:]])
    assert np.array_equal(plain, grouped), "grouped launches changed a result"


@pytest.mark.parametrize("T0,causal", [(9, True), (300, True), (14, False)])
def test_plugin_on_row_fused_weight_graphs(gpu, ref, T0, causal):
    """The graph variant the reference builds for the LocDiT decoder on a GPU backend (one MUL_MAT over row-fused
    q/k/v weights with strided views, one over gate/up): plugin against ggml-cpu, the launch count of the grouped
    decode layer, and grouped against node-by-node results.  causal=False is the LocDiT call shape: the CFG pair as
    one 14-token sequence, block-diagonal mask, no cache write."""
    import ctypes
    params = reflib.backbone_params("bb", N_LAYER)
    max_len = T0 + 20
    xp = rng("bbw", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)
    xs = [rng("bbw", "x", i + 1).standard_normal((BATCH, 1, 1024)).astype(np.float32) for i in range(2)]
    if causal:
        mask0 = reflib.causal_mask(T0, T0)
    else:
        pos = np.zeros(T0, np.int32)
        mk = np.zeros((T0, T0), np.uint16)
        reflib.load_oracle().orc_cfg_pair_constants(T0 // 2, reflib.ptr(pos, ctypes.c_int32), reflib.ptr(mk, ctypes.c_uint16))
        mask0 = mk.view(np.float16)

    def run(device, fused_weights):
        assert ref.rh_use_device(device, 8, 0) == 0
        reflib.ref_backbone_create(params, max_len, BATCH, use_mup=True, kv_f16=False, fused_weights=fused_weights)
        outs = [reflib.ref_backbone_forward(xp, 0, mask0, write_kv=causal)[0]]
        if causal:
            outs.append(reflib.ref_backbone_forward(xs[0], T0, None)[0])
            outs.append(reflib.ref_backbone_forward(xs[1], T0 + 1, None)[0])
        ref.rh_bb_free()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return outs

    cpu = run(b"CPU", True)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug = run(b"GFX950_0", True)
    launches = ctypes.CDLL(gpu.PLUGIN_PATH).ggml_backend_gfx950_last_launches()
    print(f"row-fused weights, T0={T0} causal={causal}: {launches} launches for the last graph", flush=True)
    for i, (a, b) in enumerate(zip(cpu, plug)):
        e = nmse(a, b)
        print(f"   plugin vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
        assert e <= 1e-4
    # five launches per layer and the final norm, the same groups as with separate weight tensors; up to 256 keys the
    # attention takes one kernel and the cache write is a launch of its own (with more than 16 tokens the K = 4096
    # down-projection leaves the streaming kernel: its scaled residual add stays in the product's launch there too)
    per_layer = 6 if causal and T0 + 2 <= 256 else 5
    assert launches == N_LAYER * per_layer + 1, launches
    # the separate-weights graph: the same rows through the same streaming kernel while the token count is small
    # (identical results); a long prefill tiles the wider fused matrices differently
    plain = run(b"GFX950_0", False)
    for a, b in zip(plug, plain):
        if BATCH * T0 <= 32:
            assert np.array_equal(a, b)
        else:
            assert nmse(a, b) <= 1e-6


@pytest.mark.parametrize("T0", [9, 300])
def test_plugin_under_the_scheduler_with_a_cross_split_reader(gpu, ref, T0):
    """ggml_backend_sched over {plugin, CPU} on a graph that holds, per layer, an operator the plugin does not claim
    (GELU) reading the normalised hidden state in the middle of a group: the scheduler cuts the graph there, and the
    value that a group would keep to itself has to be stored for the CPU's part.  Checked against ggml-cpu running
    the same graph."""
    params = reflib.backbone_params("bb", N_LAYER)
    max_len = T0 + 20
    xp = rng("bbs", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)
    xs = [rng("bbs", "x", i + 1).standard_normal((BATCH, 1, 1024)).astype(np.float32) for i in range(2)]

    def run(device, sched):
        assert ref.rh_use_device(device, 8, 0) == 0
        ref.rh_bb_options(int(sched), 1)
        try:
            reflib.ref_backbone_create(params, max_len, BATCH, use_mup=True, kv_f16=False)
            outs, splits = [], 0
            o, _, splits = reflib.ref_backbone_forward(xp, 0, reflib.causal_mask(T0, T0))
            outs.append(o)
            for i, x in enumerate(xs):
                o, _, splits = reflib.ref_backbone_forward(x, T0 + i, None)
                outs.append(o)
            ref.rh_bb_free()
        finally:
            ref.rh_bb_options(0, 0)
            assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return outs, splits

    cpu, _ = run(b"CPU", False)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug, splits = run(b"GFX950_0", True)
    print(f"scheduler with probe, T0={T0}: {splits} splits in the decode graph", flush=True)
    assert splits > N_LAYER          # the graph really was cut around every GELU
    for i, (a, b) in enumerate(zip(cpu, plug)):
        e = nmse(a, b)
        print(f"   plugin + scheduler vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
        assert e <= 1e-4


@pytest.mark.parametrize("T0", [9, 300])
def test_plugin_runs_the_whole_forward_graph_without_a_scheduler(gpu, ref, T0):
    """VoxCPM's default is a direct graph_compute on one backend (src/backend.cpp:569), which only works when every node
    of the graph is claimed.  Here the graph also holds the reference's mask-building chain (ARANGE, CAST, REPEAT,
    SUB, ADD1, STEP, SCALE, CAST, CONT: src/minicpm.cpp:602-620) and an embedding GET_ROWS: the plugin must run it
    as it stands, and give bit for bit what it gives when the finished mask is handed in."""
    params = reflib.backbone_params("bb", N_LAYER)
    max_len = T0 + 20
    xp = rng("bbg", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)
    xs = rng("bbg", "x", 1).standard_normal((BATCH, 1, 1024)).astype(np.float32)
    mask0 = reflib.causal_mask(T0, T0)

    def run(device, whole):
        assert ref.rh_use_device(device, 8, 0) == 0
        ref.rh_bb_whole_graph(int(whole))
        try:
            reflib.ref_backbone_create(params, max_len, BATCH, use_mup=True, kv_f16=False)
            outs = [reflib.ref_backbone_forward(xp, 0, mask0)[0], reflib.ref_backbone_forward(xs, T0, None)[0]]
        finally:
            ref.rh_bb_whole_graph(0)
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return outs

    cpu = run(b"CPU", True)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    whole = run(b"GFX950_0", True)
    handed = run(b"GFX950_0", False)
    for i, (a, b, c) in enumerate(zip(cpu, whole, handed)):
        e = nmse(a, b)
        print(f"   whole graph on the plugin vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
        assert e <= 1e-4
        assert np.array_equal(b, c), i


@pytest.mark.parametrize("T", [1, 9])
def test_plugin_keeps_state_on_the_device_between_two_graphs(gpu, ref, T):
    """Two dependent stages as the reference's decode step has them (base LM step, then the residual LM step on its
    hidden state plus the step's embedding, src/voxcpm.cpp:1067-1093): with the state fetched, added on the host and
    uploaded again between the graphs, and with the state in a persistent tensor of the backend's buffer (the second
    graph begins with the ADD, nothing crosses the bus between the stages).  Same nodes, same arithmetic: bit-equal on
    ggml-cpu and on the plugin; the plugin against ggml-cpu within the stack's bar."""
    params = reflib.backbone_params("bb", N_LAYER)
    x = rng("two-stage", T).standard_normal((BATCH, T, 1024)).astype(np.float32)
    mask = reflib.causal_mask(T, T)

    def run(device):
        assert ref.rh_use_device(device, 8, 0) == 0
        try:
            reflib.ref_backbone_create(params, T + 4, BATCH, use_mup=True, kv_f16=False)
            host, host_s = reflib.ref_backbone_two_stage(x, mask, False, reps=5)
            dev_, dev_s = reflib.ref_backbone_two_stage(x, mask, True, reps=5)
        finally:
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", 8, 0) == 0
        return host, dev_, host_s, dev_s

    c_host, c_dev, _, _ = run(b"CPU")
    assert np.isfinite(c_host).all() and np.array_equal(c_host, c_dev)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    g_host, g_dev, hs, ds = run(b"GFX950_0")
    assert np.array_equal(g_host, g_dev)
    e = nmse(c_host, g_dev)
    print(f"two stages of {N_LAYER} layers, T={T}: host round trip {hs[1] * 1e6:.0f} us, state on the device {ds[1] * 1e6:.0f} us per step "
          f"(best of 5); nmse vs ggml-cpu {e:.3e}", flush=True)
    assert e <= 1e-4


def test_plugin_runs_a_cfm_solve_of_eight_requests(gpu, ref):
    """BASELINE config 3 at its batch: the CFG pair of 8 concurrent requests, whole UnifiedCFM solves (ten Euler steps,
    projections, sequence assembly, 4 decoder layers, zero-star guidance, update of x) as ONE graph with the requests in
    ggml's own batch dimension -- the decoder sees 8 x 14 tokens, the guidance sums are SUM_ROWS over each request.
    Checked three ways: the plugin against ggml-cpu on the same graph; ggml-cpu's batched graph against eight solves of
    the reference's single-request graph (the batching changes no request's arithmetic: bit-equal on the CPU); and the
    plugin's batched result against its own single-request results (each request within the product kernels' own
    difference between 14 and 112 tokens)."""
    R = 8
    params = reflib.backbone_params("locdit", 4)
    cp = reflib.cfm_params("cfm")
    z = rng("cfm8", "z").standard_normal((R, 2, 64)).astype(np.float32)
    mu = rng("cfm8", "mu").standard_normal((R, 1024)).astype(np.float32)
    cond = rng("cfm8", "cond").standard_normal((R, 4, 64)).astype(np.float32)
    table = rng("cfm8", "table").standard_normal((10, 1024)).astype(np.float32)

    def run(device, batch, reps=0):
        assert ref.rh_use_device(device, 8, 0) == 0
        try:
            reflib.ref_backbone_create(params, 32, batch, use_mup=True, kv_f16=False, fused_weights=True)
            reflib.ref_cfm_create(cp)
            if batch == R:
                return reflib.ref_cfm_solve(z, mu, cond, table, reps=reps)
            return np.stack([reflib.ref_cfm_solve(z[r], mu[r], cond[r], table)[0] for r in range(R)]), None, None
        finally:
            ref.rh_cfm_free()
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", 8, 0) == 0

    cpu8, cpu_s, n_nodes = run(b"CPU", R, reps=2)
    cpu1 = run(b"CPU", 1)[0]
    assert np.isfinite(cpu8).all() and np.abs(cpu8 - z).max() > 1e-2
    assert np.array_equal(cpu8, cpu1), np.abs(cpu8 - cpu1).max()        # batching leaves every request's arithmetic alone
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug8, plug_s, _ = run(b"GFX950_0", R, reps=6)
    import ctypes
    launches = ctypes.CDLL(gpu.PLUGIN_PATH).ggml_backend_gfx950_last_launches()
    plug1 = run(b"GFX950_0", 1)[0]
    e8, e1, e81 = nmse(cpu8, plug8), nmse(cpu1, plug1), nmse(plug1, plug8)
    print(f"CFM solve of {R} requests, 10 steps: {n_nodes} graph nodes, {launches} launches on the plugin; nmse vs ggml-cpu {e8:.3e} "
          f"(single-request graphs {e1:.3e}), batched vs single on the plugin {e81:.3e}; ggml-cpu (8 threads) {cpu_s[1] * 1e3:.2f} ms, "
          f"plugin {plug_s[1] * 1e3:.3f} ms per {R} solves", flush=True)
    assert e8 <= 1e-3 and e1 <= 1e-3 and e81 <= 1e-3


@pytest.mark.parametrize("time_table", [True, False])
def test_plugin_runs_a_whole_cfm_solve_graph(gpu, ref, time_table):
    """BASELINE config 3 as the reference builds it (src/unified_cfm.cpp:88-184 around src/locdit.cpp:401-464): ten
    Euler steps of the LocDiT estimator in ONE graph -- input projection, the CFG pair as one 14-token non-causal
    sequence through 4 decoder layers with row-fused weights, output projection of both branches, the zero-star
    guidance scale (MUL, SUM, ARANGE, DIV, REPEAT) and the update of x.  Direct graph_compute on the plugin against
    ggml-cpu, grouped launches against node-by-node ones (same bits), and the launch count of a solve.
    time_table=False: the combined time embedding of every step is computed in the graph too, as UnifiedCFM::forward does
    without a precomputed table (sinusoidal embedding -- ARANGE, SCALE, EXP, REPEAT, MUL, SIN, COS, CONCAT -- and the two
    timestep MLPs, src/locdit.cpp:186-246)."""
    import ctypes
    import subprocess
    import sys
    params = reflib.backbone_params("locdit", 4)
    cp = reflib.cfm_params("cfm")
    z = rng("cfm", "z").standard_normal((2, 64)).astype(np.float32)
    mu = rng("cfm", "mu").standard_normal(1024).astype(np.float32)
    cond = rng("cfm", "cond").standard_normal((4, 64)).astype(np.float32)
    table = rng("cfm", "table").standard_normal((10, 1024)).astype(np.float32) if time_table else None

    def run(device, reps=0):
        assert ref.rh_use_device(device, 8, 0) == 0
        try:
            reflib.ref_backbone_create(params, 32, 1, use_mup=True, kv_f16=False, fused_weights=True)
            reflib.ref_cfm_create(cp)
            return reflib.ref_cfm_solve(z, mu, cond, table, reps=reps)
        finally:
            ref.rh_cfm_free()
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", 8, 0) == 0

    cpu, cpu_s, n_nodes = run(b"CPU", reps=3)
    assert np.isfinite(cpu).all() and np.abs(cpu - z).max() > 1e-2          # the solve moved x
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug, plug_s, _ = run(b"GFX950_0", reps=5)
    launches = ctypes.CDLL(gpu.PLUGIN_PATH).ggml_backend_gfx950_last_launches()
    e = nmse(cpu, plug)
    print(f"CFM solve, 10 steps: {n_nodes} graph nodes, {launches} launches on the plugin; nmse vs ggml-cpu {e:.3e}; "
          f"ggml-cpu (8 threads) {cpu_s[1] * 1e3:.2f} ms, plugin {plug_s[1] * 1e3:.3f} ms per solve", flush=True)
    assert e <= 1e-3
    # nine estimator passes (step 1 is zero under zero-star): 4 layers x 5 launches + the final norm for the decoder,
    # at most 26 for the projections, the five CONCATs, the guidance arithmetic and the update of x (and at most 12 more
    # per step for a time embedding built in the graph)
    assert launches <= 9 * (4 * 5 + 1 + 26 + (0 if time_table else 12)) + 5 + (0 if time_table else 12), (launches, n_nodes)
    # node by node in a fresh process: the groups must not change a bit
    code = (
        "import sys, numpy as np\n"
        f"sys.path.insert(0, {repr(str(__import__('os').path.dirname(__file__)))})\n"
        "import reflib\n"
        "from reflib import rng\n"
        "ref = reflib.load_ref()\n"
        f"assert ref.rh_load_plugin({repr(gpu.PLUGIN_PATH)}.encode()) == 0\n"
        "assert ref.rh_use_device(b'GFX950_0', 0, 0) == 0\n"
        "params = reflib.backbone_params('locdit', 4); cp = reflib.cfm_params('cfm')\n"
        "z = rng('cfm', 'z').standard_normal((2, 64)).astype(np.float32)\n"
        "mu = rng('cfm', 'mu').standard_normal(1024).astype(np.float32)\n"
        "cond = rng('cfm', 'cond').standard_normal((4, 64)).astype(np.float32)\n"
        f"table = rng('cfm', 'table').standard_normal((10, 1024)).astype(np.float32) if {time_table} else None\n"
        "reflib.ref_backbone_create(params, 32, 1, use_mup=True, kv_f16=False, fused_weights=True)\n"
        "reflib.ref_cfm_create(cp)\n"
        "out = reflib.ref_cfm_solve(z, mu, cond, table)[0]\n"
        "sys.stdout.write('BITS ' + out.tobytes().hex() + '\\n')\n"
    )
    env = dict(__import__("os").environ, GGML_GFX950_NO_FUSION="1")
    p = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    bits = [l for l in p.stdout.splitlines() if l.startswith("BITS ")][0][5:]
    assert bytes.fromhex(bits) == plug.tobytes()
    if not time_table:
        return
    # the C-ABI mirror of the solve (voxcpm.cpp_amd/cfm.py): the plugin's launches issued by hand, the same bits
    import torch
    from voxcpm_cpp_amd import backbone as bb, cfm
    dec = bb.MiniCPMBackbone(n_layer=4, max_length=32, batch=1, use_mup=True, kv_f16=False)
    for li, lw in enumerate(params["layers"]):
        for n in reflib.BB_WEIGHTS:
            dec.set_weight(li, n, torch.from_numpy(lw[n]).cuda(), params["shapes"][n][1])
        for n in ("input_layernorm", "post_layernorm"):
            dec.set_norm(li, n, torch.from_numpy(lw[n]).cuda())
    dec.set_norm(-1, "norm", torch.from_numpy(params["final_norm"]).cuda())
    dec.rope_factors = torch.from_numpy(params["rope_factors"]).cuda()
    q8 = lambda w, b: (torch.from_numpy(reflib.quantize_q8_0(w)).cuda(), w.shape[1], torch.from_numpy(b).cuda())
    solver = cfm.LocDiTCfmSolver(dec, 64, q8(cp["in_w"], cp["in_b"]), q8(cp["cond_w"], cp["cond_b"]), q8(cp["out_w"], cp["out_b"]))
    t_span = np.zeros(11, np.float32)
    reflib.load_oracle().orc_t_span(10, 1.0, reflib.ptr(t_span, ctypes.c_float))
    run, x = solver.plan(*(torch.from_numpy(a).cuda() for a in (z, mu, cond, table)), t_span, cfg_value=2.0)
    run()
    torch.cuda.synchronize()
    print(f"   C ABI mirror: {run.n_calls} calls per solve", flush=True)
    assert launches - 2 <= run.n_calls <= launches, (run.n_calls, launches)   # ggml's node order splits one run of tiny nodes in two
    assert x.cpu().numpy().tobytes() == plug.tobytes()


@pytest.mark.parametrize("kv_f16", [True, False])
def test_plugin_runs_consecutive_decode_steps(gpu, ref, kv_f16):
    """A run of decode steps as the reference drives them (src/voxcpm.cpp:485-513, 1027-1128): a graph built for every
    position, laid out by one graph allocator, computed, the hidden state fetched.  72 consecutive steps behind a
    prefill of 300 tokens (so the key ranges are cut and merged, and the cut changes along the way) through the plugin:
    against ggml-cpu on the same loop, against the same steps computed one by one through rh_bb_forward (the same
    launches: bit for bit, the caches included), and with the next step's graph built while the device computes the
    current one (the same launches again).  All of that with every step launched node by node; then the same loops with
    the steps run as patched recordings (from the fourth step on a step is the recorded HIP graph of an earlier one with
    the arguments that follow from the position set on its nodes): the same bits again, the caches included."""
    import ctypes
    T0, N = 300, 72
    max_len = T0 + N + 8
    params = reflib.backbone_params("bb", N_LAYER)
    xp = rng("bbl", "x", 0).standard_normal((BATCH, T0, 1024)).astype(np.float32)
    x1 = rng("bbl", "x", 1).standard_normal((BATCH, 1, 1024)).astype(np.float32)
    cache_bytes = 64 * max_len * 2 * BATCH * (2 if kv_f16 else 4)

    def caches():
        out = []
        for layer in range(N_LAYER):
            for which in (0, 1):
                buf = np.empty(cache_bytes, np.uint8)
                assert ref.rh_bb_cache_get(layer, which, buf.ctypes.data, buf.nbytes) == 0
                out.append(buf)
        return out

    plugin = ctypes.CDLL(gpu.PLUGIN_PATH)

    def run(device, how, patch=False):
        assert ref.rh_use_device(device, 8, 0) == 0
        patch_before = plugin.ggml_backend_gfx950_set_graph_patch(int(patch))
        reflib.ref_backbone_create(params, max_len, BATCH, use_mup=True, kv_f16=kv_f16)
        try:
            reflib.ref_backbone_forward(xp, 0, reflib.causal_mask(T0, T0))
            if how == "one by one":
                for s in range(N):
                    out = reflib.ref_backbone_forward(x1, T0 + s, None)[0]
                info = None
            else:
                out, info = reflib.ref_backbone_decode_loop(x1, T0, N, overlap=(how == "overlapped"))
            return out, caches(), info
        finally:
            ref.rh_bb_free()
            plugin.ggml_backend_gfx950_set_graph_patch(patch_before)
            assert ref.rh_use_device(b"CPU", 8, 0) == 0

    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    cpu, cpu_cache, _ = run(b"CPU", "loop")
    loop, loop_cache, info = run(b"GFX950_0", "loop")
    launches = plugin.ggml_backend_gfx950_last_launches()
    print(f"consecutive decode steps, kv_f16={kv_f16}: {N} steps, {info['n_nodes']} nodes and {launches} launches a step, "
          f"{info['moved'] * 100:.0f} % of the nodes at another address than the step before", flush=True)
    assert launches == 5 * N_LAYER + 1
    e = nmse(cpu, loop)
    print(f"   last hidden state, plugin vs ggml-cpu: nmse {e:.3e}", flush=True)
    assert e <= 1e-4
    for a, b in zip(cpu_cache, loop_cache):  # what the steps appended (f16 or F32 values of O(1))
        w = np.float16 if kv_f16 else np.float32
        af, bf = a.view(w).astype(np.float32), b.view(w).astype(np.float32)
        assert nmse(af, bf) <= 2e-4 and np.abs(af - bf).max() <= 5e-2
    single, single_cache, _ = run(b"GFX950_0", "one by one")
    assert np.array_equal(loop, single), "the loop's last step differs from the step computed on its own"
    for a, b in zip(loop_cache, single_cache):
        assert np.array_equal(a, b), "cache contents differ"
    over, over_cache, _ = run(b"GFX950_0", "overlapped")
    assert np.array_equal(loop, over), "building the next graph under the running one changed a result"
    for a, b in zip(loop_cache, over_cache):
        assert np.array_equal(a, b), "cache contents differ (overlapped)"
    for how in ("loop", "overlapped", "one by one"):
        n0 = plugin.ggml_backend_gfx950_patched_replays()
        out, cache, _ = run(b"GFX950_0", how, patch=True)
        n1 = plugin.ggml_backend_gfx950_patched_replays()
        print(f"   steps as patched recordings ({how}): {n1 - n0} of {N} steps, {plugin.ggml_backend_gfx950_last_patched()} kernels' "
              f"arguments changed in the last one", flush=True)
        assert n1 - n0 >= N - 12, "the steps were not run as patched recordings"
        assert plugin.ggml_backend_gfx950_last_launches() == launches
        assert np.array_equal(loop, out), f"a patched recording gave another result than node-by-node launches ({how})"
        for a, b in zip(loop_cache, cache):
            assert np.array_equal(a, b), f"cache contents differ (patched recordings, {how})"


def test_plugin_follows_weights_rewritten_in_place(gpu, ref, monkeypatch):
    """The plugin tells the library that a buffer marked GGML_BACKEND_BUFFER_USAGE_WEIGHTS is constant, and the large
    products then keep their weights' tiles between graphs; a ggml_backend_tensor_set into such a buffer must drop what
    was derived from the bytes it writes.  A 1024-token prefill, the same again (served from the kept tiles), new weights
    uploaded into the same tensors, the prefill again: against ggml-cpu on the new weights, and bit for bit against a
    stack created with the new weights from the start."""
    import ctypes as C
    T0, layers = 1024, 2
    monkeypatch.setenv("VX_GEMM_Q8T", "2")   # (the prefill's products are smaller than what takes the pre-tiled kernel by itself)
    pa, pb = reflib.backbone_params("pin-a", layers), reflib.backbone_params("pin-b", layers)
    x = rng("pin", "x").standard_normal((1, T0, 1024)).astype(np.float32)
    mask = reflib.causal_mask(T0, T0)
    lib = gpu.lib()

    def held():
        v = [C.c_size_t() for _ in range(3)]
        gpu.check(lib.vx_weights_info(*[C.byref(a) for a in v]), "info")
        return tuple(a.value for a in v)

    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    base = held()
    assert ref.rh_use_device(b"GFX950_0", 8, 0) == 0
    try:
        reflib.ref_backbone_create(pa, T0 + 8, 1, use_mup=True, kv_f16=True)
        a1 = reflib.ref_backbone_forward(x, 0, mask)[0]
        h1 = held()
        print(f"weights buffer pinned: {h1[0] - base[0]} range, {h1[1] - base[1]} copies, {(h1[2] - base[2]) >> 20} MiB", flush=True)
        assert h1[0] == base[0] + 1 and h1[1] > base[1]
        a2 = reflib.ref_backbone_forward(x, 0, mask)[0]
        assert held() == h1 and np.array_equal(a1, a2)
        reflib.ref_backbone_upload(pb)
        assert held()[1] == base[1], "copies of rewritten weights were kept"
        b1 = reflib.ref_backbone_forward(x, 0, mask)[0]
        b2 = reflib.ref_backbone_forward(x, 0, mask)[0]
        assert np.array_equal(b1, b2) and not np.array_equal(a1, b1)
        ref.rh_bb_free()
        assert held() == base, "freeing the buffer left a pinned range or copies behind"
        reflib.ref_backbone_create(pb, T0 + 8, 1, use_mup=True, kv_f16=True)
        fresh = reflib.ref_backbone_forward(x, 0, mask)[0]
        assert np.array_equal(b1, fresh), "results after an in-place upload differ from a stack created with those weights"
    finally:
        ref.rh_bb_free()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
    reflib.ref_backbone_create(pb, T0 + 8, 1, use_mup=True, kv_f16=True)
    try:
        cpu = reflib.ref_backbone_forward(x, 0, mask)[0]
    finally:
        ref.rh_bb_free()
    e = nmse(cpu, b1)
    print(f"   prefill after the upload vs ggml-cpu: nmse {e:.3e}", flush=True)
    assert e <= 1e-4


def test_plugin_replays_a_recurring_graph(gpu, ref):
    """A graph the plugin has run twice is recorded on its third run and replayed from then on (a CFM solve has the same
    shapes and addresses on every call; the reference rebuilds and relaunches it each time, src/voxcpm.cpp:485-495).
    The replays must give what node-by-node launches give, with the host writing fresh inputs between them, with other
    graphs run in between, and a graph of another shape must never be mistaken for a recorded one."""
    import ctypes
    params = reflib.backbone_params("locdit", 4)
    cp = reflib.cfm_params("cfm")
    mu = rng("cfmr", "mu").standard_normal(1024).astype(np.float32)
    cond = rng("cfmr", "cond").standard_normal((4, 64)).astype(np.float32)
    table = rng("cfmr", "table").standard_normal((10, 1024)).astype(np.float32)
    zs = [rng("cfmr", "z", i).standard_normal((2, 64)).astype(np.float32) for i in range(3)]
    plugin = ctypes.CDLL(gpu.PLUGIN_PATH)

    def solve_all(device, replay, reps):
        assert ref.rh_use_device(device, 8, 0) == 0
        before = plugin.ggml_backend_gfx950_set_graph_replay(int(replay))
        ref.rh_out_after_reps(1)
        try:
            reflib.ref_backbone_create(params, 32, 1, use_mup=True, kv_f16=False, fused_weights=True)
            reflib.ref_cfm_create(cp)
            outs = []
            for z in zs:
                outs.append(reflib.ref_cfm_solve(z, mu, cond, table, reps=reps)[0])            # the last repeat's result
                outs.append(reflib.ref_cfm_solve(z[:1], mu, cond[:2], table, reps=0)[0])       # another shape in between
            return outs
        finally:
            ref.rh_out_after_reps(0)
            plugin.ggml_backend_gfx950_set_graph_replay(before)
            ref.rh_cfm_free()
            ref.rh_bb_free()
            assert ref.rh_use_device(b"CPU", 8, 0) == 0

    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plain = solve_all(b"GFX950_0", False, 4)
    n0 = plugin.ggml_backend_gfx950_replays()
    replayed = solve_all(b"GFX950_0", True, 4)
    n1 = plugin.ggml_backend_gfx950_replays()
    print(f"recurring CFM solve graph: {n1 - n0} of {len(zs) * 6} graph_compute calls were replays", flush=True)
    assert n1 - n0 >= len(zs) * 2          # runs 3, 4, 5 of every five identical computes at the least
    for i, (a, b) in enumerate(zip(plain, replayed)):
        assert np.array_equal(a, b), f"solve {i}: a replay differs from node-by-node launches"
    cpu = solve_all(b"CPU", False, 0)
    for i, (a, b) in enumerate(zip(cpu, replayed)):
        assert nmse(a, b) <= 1e-3, i


def test_plugin_replay_keys_on_the_activation_mode(gpu, ref):
    """A recording holds the launches of the activation mode it was made under (ggml_backend_gfx950_set_mul_mat_act): the
    same graph at the same addresses after a switch of the mode is another graph.  Four solves with float activations
    (recorded at the third, replayed at the fourth), the switch to Q8 activations, four more: they must give what Q8
    launches give without any replay, and not what the float recording holds."""
    import ctypes
    params = reflib.backbone_params("locdit", 4)
    cp = reflib.cfm_params("cfm")
    mu = rng("cfmr", "mu").standard_normal(1024).astype(np.float32)
    cond = rng("cfmr", "cond").standard_normal((4, 64)).astype(np.float32)
    table = rng("cfmr", "table").standard_normal((10, 1024)).astype(np.float32)
    z = rng("cfmr", "z", 0).standard_normal((2, 64)).astype(np.float32)
    plugin = ctypes.CDLL(gpu.PLUGIN_PATH)
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    assert ref.rh_use_device(b"GFX950_0", 8, 0) == 0
    replay_before = plugin.ggml_backend_gfx950_set_graph_replay(1)
    act_before = plugin.ggml_backend_gfx950_set_mul_mat_act(0)
    ref.rh_out_after_reps(1)
    try:
        reflib.ref_backbone_create(params, 32, 1, use_mup=True, kv_f16=False, fused_weights=True)
        reflib.ref_cfm_create(cp)
        n0 = plugin.ggml_backend_gfx950_replays()
        out_float = reflib.ref_cfm_solve(z, mu, cond, table, reps=4)[0]
        n1 = plugin.ggml_backend_gfx950_replays()
        assert n1 > n0, "the float-mode graph was never replayed: the test would prove nothing"
        plugin.ggml_backend_gfx950_set_mul_mat_act(1)
        out_q8 = reflib.ref_cfm_solve(z, mu, cond, table, reps=4)[0]
        plugin.ggml_backend_gfx950_set_graph_replay(0)
        out_q8_plain = reflib.ref_cfm_solve(z, mu, cond, table, reps=1)[0]
    finally:
        ref.rh_out_after_reps(0)
        plugin.ggml_backend_gfx950_set_mul_mat_act(act_before)
        plugin.ggml_backend_gfx950_set_graph_replay(replay_before)
        ref.rh_cfm_free()
        ref.rh_bb_free()
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
    print(f"activation mode and replay: float vs q8 max-abs {np.abs(out_float - out_q8).max():.3e}", flush=True)
    assert np.array_equal(out_q8, out_q8_plain), "a recording made under another activation mode was replayed"
    assert not np.array_equal(out_float, out_q8)


@pytest.mark.gpu
def test_plugin_on_random_graphs_of_small_operators(gpu, ref):
    """Seeded random DAGs of the exact small operators (binary operators with broadcast, SCALE, SQR, NEG, CONT, REPEAT,
    CONCAT and a view back, SUM_ROWS, SUM, DIV), allocated by ggml_gallocr -- which hands a dead tensor's memory to the next
    node at once -- and computed twice: the plugin's per-graph decisions (runs of tiny nodes in one launch, values kept in LDS
    only, CONCAT trees written from their leaves, node pairs) against ggml-cpu on the same graph.  The operators are exact,
    so the results agree bit for bit except through the order of a sum's fp64 additions."""
    import ctypes as C
    assert ref.rh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    plug = C.CDLL(gpu.PLUGIN_PATH)
    cap = 4096 * 8
    worst, fused, exact, overflowed = 0.0, 0, 0, 0
    seeds = list(range(600))
    for seed in seeds:
        outs = []
        for device in (b"CPU", b"GFX950_0"):
            assert ref.rh_use_device(device, 8, 0) == 0
            buf = np.zeros(cap, np.float32)
            n, nodes = C.c_int64(0), C.c_int(0)
            rc = ref.rh_random_graph(seed, 8 + seed % 40, buf.ctypes.data_as(C.POINTER(C.c_float)), cap, C.byref(n), C.byref(nodes))
            assert rc == 0, (seed, device, rc)
            outs.append(buf[:n.value].copy())
            if device != b"CPU":
                launches = plug.ggml_backend_gfx950_last_launches()
                fused += launches < nodes.value
        assert ref.rh_use_device(b"CPU", 8, 0) == 0
        cpu, dev_ = outs
        if not np.isfinite(cpu).all():   # a chain of squares ran out of range: the same non-finite values have to come back
            assert np.array_equal(np.isnan(cpu), np.isnan(dev_)), seed
            overflowed += 1
            continue
        err = float(np.abs(cpu - dev_).max() / max(1.0, float(np.abs(cpu).max())))
        exact += bool(np.array_equal(cpu, dev_))
        worst = max(worst, err)
        assert err <= 1e-5, (seed, err, nodes.value)
    print(f"random graphs: {len(seeds)} seeds ({overflowed} out of range), {exact} bit-equal, worst relative difference {worst:.2e}, {fused} with fewer launches than nodes", flush=True)
    assert fused >= len(seeds) // 2 and exact >= len(seeds) * 9 // 10 and overflowed <= len(seeds) // 50

