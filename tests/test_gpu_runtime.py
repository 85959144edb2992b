"""The per-stream workspace on the device: a HIP graph captured at a small shape must replay correctly after
the workspace has grown for a larger one (the block it was recorded with stays allocated at its address)."""
import sys

import numpy as np
import pytest

from reflib import rng

pytestmark = pytest.mark.gpu


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def test_captured_graph_survives_workspace_growth(gpu):
    import ctypes as C
    import torch
    lib = gpu.lib()
    side = torch.cuda.Stream()  # a fresh stream: its workspace starts empty
    B, Hq, Hkv, D = 2, 16, 2, 64

    def tensors(L, tag):
        q = torch.from_numpy(rng("wsgrow", tag, "q").standard_normal((B, Hq, 1, D)).astype(np.float32)).cuda()
        k = torch.from_numpy(rng("wsgrow", tag, "k").standard_normal((B, Hkv, L, D)).astype(np.float16)).cuda()
        v = torch.from_numpy(rng("wsgrow", tag, "v").standard_normal((B, Hkv, L, D)).astype(np.float16)).cuda()
        return q, k, v

    q1, k1, v1 = tensors(2048, "small")
    out1 = torch.zeros((B, 1, Hq, D), device="cuda")
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        say("eager small call, then capture of the same call")
        gpu.flash_attn_ext(q1, k1, v1, None, 0.125, out=out1)   # grows the workspace to its floor (1 MiB)
        side.synchronize()
        want1 = out1.clone()
        ptr, size, retired = C.c_void_p(), C.c_size_t(), C.c_int()
        gpu.check(lib.vx_workspace_info(side.cuda_stream, C.byref(ptr), C.byref(size), C.byref(retired)), "info")
        first_ptr, first_size = ptr.value, size.value
        assert first_ptr and first_size >= 1 << 20 and retired.value == 0
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            gpu.flash_attn_ext(q1, k1, v1, None, 0.125, out=out1)
        # a call that must grow the workspace is refused while the stream is capturing
        qb, kb, vb = tensors(8192, "large")
        qb = qb.repeat(32, 1, 1, 1)[:48].contiguous(); kb = kb.repeat(32, 1, 1, 1)[:48].contiguous(); vb = kb.clone()
        outb = torch.empty((48, 1, Hq, D), device="cuda")
    with torch.cuda.stream(side):
        say("larger eager call: the workspace grows")
        gpu.flash_attn_ext(qb, kb, vb, None, 0.125, out=outb)
        side.synchronize()
        gpu.check(lib.vx_workspace_info(side.cuda_stream, C.byref(ptr), C.byref(size), C.byref(retired)), "info")
        assert size.value > first_size and ptr.value != first_ptr and retired.value == 1
        # scribble over the new block's users, then replay the graph recorded with the old block
        out1.zero_()
        say("replay of the graph captured before the growth")
        graph.replay()
        side.synchronize()
        assert torch.equal(out1, want1)
        # and once more after more eager work on the grown workspace
        gpu.flash_attn_ext(qb, kb, vb, None, 0.125, out=outb)
        out1.zero_()
        graph.replay()
        side.synchronize()
        assert torch.equal(out1, want1)


def test_workspace_growth_during_capture_is_refused(gpu):
    import torch
    lib = gpu.lib()
    side = torch.cuda.Stream()
    B, Hq, Hkv, D, L = 48, 16, 2, 64, 8192   # partials beyond the 1 MiB floor
    q = torch.zeros((B, Hq, 1, D), device="cuda")
    k = torch.zeros((B, Hkv, L, D), dtype=torch.float16, device="cuda")
    out = torch.empty((B, 1, Hq, D), device="cuda")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    say("capture of a call whose workspace was not reserved")
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            rc = lib.vx_flash_attn_ext(gpu.desc(q), gpu.desc(k), gpu.desc(k), None, None, gpu.desc(out), 0.125, 0.0, 0.0,
                                       side.cuda_stream)
        assert rc == 2 and b"vx_workspace_reserve" in lib.vx_last_error()
        gpu.check(lib.vx_workspace_reserve(side.cuda_stream, 64 << 20), "reserve")
        graph2 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph2, stream=side):
            rc = lib.vx_flash_attn_ext(gpu.desc(q), gpu.desc(k), gpu.desc(k), None, None, gpu.desc(out), 0.125, 0.0, 0.0,
                                       side.cuda_stream)
        assert rc == 0
        graph2.replay()
        side.synchronize()
        assert float(out.abs().max()) == 0.0


def test_a_recording_runs_again_with_other_arguments(gpu):
    """vx_graph_patch_begin/_end: the calls of a decode step made against a recording launch nothing, the recorded graph
    then runs with their arguments.  A step with a growing key count, another query and alternating outputs, each run
    checked against the same calls made directly, with direct work between the runs; then a call sequence with another
    kernel in it, which the comparison must refuse."""
    import ctypes as C
    import torch
    lib = gpu.lib()
    side = torch.cuda.Stream()
    B, Hq, Hkv, D, cap = 2, 16, 2, 64, 1400
    g = lambda *tag: rng("patch", *tag)
    kc = torch.from_numpy(g("k").standard_normal((B, Hkv, cap, D)).astype(np.float16)).cuda()
    vc = torch.from_numpy(g("v").standard_normal((B, Hkv, cap, D)).astype(np.float16)).cuda()
    w = torch.from_numpy(g("w").standard_normal(Hq * D).astype(np.float32)).cuda()
    qs = [torch.from_numpy(g("q", i).standard_normal((B, Hq, 1, D)).astype(np.float32)).cuda() for i in range(3)]
    outs = [torch.zeros((B, 1, Hq, D), device="cuda") for _ in range(2)]
    normed = [torch.zeros((B, 1, Hq * D), device="cuda") for _ in range(2)]
    torch.cuda.synchronize()

    def step(L, i):   # attention over the first L keys, then a norm of its output
        gpu.flash_attn_ext(qs[i % 3], kc[:, :, :L], vc[:, :, :L], None, 0.125, out=outs[i % 2])
        gpu.rms_norm(outs[i % 2].view(B, 1, Hq * D), 1e-5, out=normed[i % 2])

    with torch.cuda.stream(side):
        gpu.check(lib.vx_workspace_reserve(side.cuda_stream, 8 << 20), "reserve")
        step(900, 0)
        side.synchronize()
        gpu.check(lib.vx_graph_begin(side.cuda_stream), "begin")
        step(900, 0)
        rec = C.c_void_p()
        gpu.check(lib.vx_graph_end(side.cuda_stream, C.byref(rec)), "end")
        assert rec.value and lib.vx_graph_patchable(rec) == 1
        changed = C.c_int()
        for i, L in enumerate([900, 901, 902, 1023, 1024, 1025, 1399, 64, 1]):
            say(f"recording run again for {L} keys")
            step(L, i)   # directly
            side.synchronize()
            want = (outs[i % 2].clone(), normed[i % 2].clone())
            outs[i % 2].zero_(); normed[i % 2].zero_()
            gpu.check(lib.vx_graph_patch_begin(rec), "patch_begin")
            step(L, i)   # compared with the recording: nothing runs
            side.synchronize()
            assert float(outs[i % 2].abs().max()) == 0.0, "a call made during the comparison ran"
            rc = lib.vx_graph_patch_end(rec, C.byref(changed))
            if rc == 2:  # another kernel for this key count than the recorded one: the recording is of no use for it
                say(f"   {L} keys take other kernels than the recording's")
                assert L in (64, 1)
                gpu.check(lib.vx_graph_destroy(rec), "destroy")
                gpu.check(lib.vx_graph_begin(side.cuda_stream), "begin")
                step(L, i)
                gpu.check(lib.vx_graph_end(side.cuda_stream, C.byref(rec)), "end")
                assert rec.value and lib.vx_graph_patchable(rec) == 1
            else:
                assert rc == 0 and (changed.value >= 1 or i == 0)
            gpu.check(lib.vx_graph_launch(rec, side.cuda_stream), "launch")
            side.synchronize()
            assert torch.equal(outs[i % 2], want[0]) and torch.equal(normed[i % 2], want[1]), L
        # a different sequence of calls: refused, and the thread launches normally again afterwards
        gpu.check(lib.vx_graph_patch_begin(rec), "patch_begin")
        gpu.rms_norm(outs[0].view(B, 1, Hq * D), 1e-5, out=normed[0])
        assert lib.vx_graph_patch_end(rec, C.byref(changed)) == 2
        gpu.check(lib.vx_graph_destroy(rec), "destroy")
        step(900, 0)
        side.synchronize()
        assert float(outs[0].abs().max()) > 0.0
