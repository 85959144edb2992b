"""The plugin on graphs that the REFERENCE's own code builds: a synthetic model file written with ggml's gguf API is
loaded by the reference's VoxCPMWeightStore and MiniCPMModel (compiled from its sources into oracle/_ref, driven by
oracle/vox_harness.cpp), and MiniCPMModel::forward / forward_step (src/minicpm.cpp:779-846) run on ggml-cpu and on the
plugin.  The reference selects its GPU device by registry name, so the plugin is loaded under the alias
GGML_GFX950_REG_NAME=CUDA-gfx950 -- the way an unpatched VoxCPM build reaches it -- in a process of its own (the
registry name is fixed when the plugin is first asked for it).

Checked: the plugin's results against ggml-cpu's on the same graphs; that the node groups found on the restated graphs
are found on the real ones (launches per decode step); that the restated single-sequence graph of
oracle/ref_harness.cpp gives ggml-cpu the same bits as the reference's builder does; and where the weights were put."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

import reflib
from reflib import nmse, rng

pytestmark = pytest.mark.gpu

N_LAYER, T0, STEPS = 3, 300, 3

CHILD = r"""
import json, os, sys
import numpy as np
sys.path.insert(0, sys.argv[1]); sys.path.insert(0, os.path.join(sys.argv[1], "tests"))
import reflib
from reflib import rng
import __graft_entry__ as entry
pkg = entry.load_package()
mode, gguf, prefix, out_path = sys.argv[2], sys.argv[3], sys.argv[4], sys.argv[5]
N_LAYER, T0, STEPS = (int(a) for a in sys.argv[6:9])
vox = reflib.load_vox()
if mode == "gpu":
    assert vox.vh_load_plugin(pkg.PLUGIN_PATH.encode()) == 0
    assert vox.vh_open(1, 8) == 0, vox.vh_last_error()     # BackendType::CUDA: found through the registry alias
else:
    assert vox.vh_open(0, 8) == 0, vox.vh_last_error()
assert vox.vh_minicpm_load(gguf.encode(), prefix.encode(), T0 + STEPS + 8) == 0, vox.vh_last_error()
info = {"backend": vox.vh_backend_name().decode(), "is_gpu": vox.vh_backend_is_gpu(), "weights_on_host": vox.vh_weights_on_host(),
        "weight_bytes": vox.vh_weight_bytes(), "launches": [], "nodes": [], "ms": []}
import ctypes
plugin = ctypes.CDLL(pkg.PLUGIN_PATH) if mode == "gpu" else None
xs = [rng("refg", "x", 0).standard_normal((T0, 1024)).astype(np.float32)]
xs += [rng("refg", "x", i + 1).standard_normal((1, 1024)).astype(np.float32) for i in range(STEPS)]
outs, pos = [], 0
for i, x in enumerate(xs):
    o = np.empty_like(x)
    sec = ctypes.c_double()
    rc = vox.vh_minicpm_run(x.ctypes.data, x.shape[0], -1 if i == 0 else pos, o.ctypes.data, 5 if i else 0, ctypes.byref(sec))
    assert rc == 0, vox.vh_last_error()
    outs.append(o)
    info["nodes"].append(vox.vh_last_graph_nodes())
    info["ms"].append(sec.value * 1e3)
    if plugin is not None:
        info["launches"].append(plugin.ggml_backend_gfx950_last_launches())
    pos += x.shape[0]
kc = np.empty((2, T0 + STEPS + 8, 64), np.float32)
assert vox.vh_cache_get(N_LAYER - 1, 0, kc.ctypes.data, kc.nbytes) == 0
np.savez(out_path, *outs, cache=kc)
print("INFO " + json.dumps(info))
"""


def run_child(mode, gguf, prefix, out_path, alias):
    env = dict(os.environ)
    if alias:
        env["GGML_GFX950_REG_NAME"] = alias
    p = subprocess.run([sys.executable, "-c", CHILD, reflib.ROOT, mode, gguf, prefix, out_path, str(N_LAYER), str(T0), str(STEPS)],
                       env=env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stdout[-2000:] + p.stderr[-3000:]
    info = json.loads([l for l in p.stdout.splitlines() if l.startswith("INFO ")][0][5:])
    data = np.load(out_path)
    return info, [data[f"arr_{i}"] for i in range(STEPS + 1)], data["cache"]


def test_plugin_on_graphs_built_by_the_reference(gpu, ref, tmp_path):
    if reflib.load_vox() is None:
        pytest.skip("oracle/_ref/libvox_harness.so was not prebuilt")
    params = reflib.backbone_params("refg", N_LAYER)
    gguf = str(tmp_path / "residual_lm.gguf")
    reflib.write_minicpm_gguf(gguf, params, "residual_lm", 4096, use_mup=True)
    print(f"reference-built graphs: {N_LAYER} layers, one sequence, prefill {T0} + {STEPS} decode steps; model file {os.path.getsize(gguf) >> 20} MiB", flush=True)
    ci, cpu, cpu_cache = run_child("cpu", gguf, "residual_lm", str(tmp_path / "cpu.npz"), None)
    gi, gpu_out, gpu_cache = run_child("gpu", gguf, "residual_lm", str(tmp_path / "gpu.npz"), "CUDA-gfx950")
    print(f"   ggml-cpu: backend {ci['backend']}, graph nodes {ci['nodes']}, ms {['%.2f' % m for m in ci['ms']]}", flush=True)
    print(f"   plugin:   backend {gi['backend']} (is_gpu {gi['is_gpu']}), launches {gi['launches']}, ms {['%.3f' % m for m in gi['ms']]}; "
          f"weights on host: {gi['weights_on_host']}, {gi['weight_bytes'] >> 20} MiB", flush=True)
    assert gi["is_gpu"] == 1 and gi["backend"].startswith("GFX950") and gi["weights_on_host"] == 0
    # on a backend whose weights are not in host memory mlp_forward emits one SWIGLU node for SILU + MUL (src/minicpm.cpp:729-745)
    assert [n - N_LAYER for n in ci["nodes"]] == gi["nodes"]
    for i, (a, b) in enumerate(zip(cpu, gpu_out)):
        e = nmse(a, b)
        print(f"   plugin vs ggml-cpu, call {i}: nmse {e:.3e}", flush=True)
        assert np.isfinite(b).all() and e <= 1e-4
    # the cache the reference's builder wrote through the plugin: positions 0 .. T0 + STEPS - 1, the rest untouched
    assert nmse(cpu_cache[:, :T0 + STEPS], gpu_cache[:, :T0 + STEPS]) <= 1e-4 and not gpu_cache[:, T0 + STEPS:].any()
    # the node groups of the decode step: five launches per layer and the final norm, as on the restated graphs
    assert gi["launches"][-1] == N_LAYER * 5 + 1, gi["launches"]
    # the restated single-sequence graph (oracle/ref_harness.cpp, batch 1) on ggml-cpu: the same operators in the same
    # order as the reference's builder emits, hence the same bits
    assert ref.rh_use_device(b"CPU", 8, 0) == 0
    reflib.ref_backbone_create(params, T0 + STEPS + 8, 1, use_mup=True, kv_f16=False)
    xs = [rng("refg", "x", 0).standard_normal((T0, 1024)).astype(np.float32)]
    xs += [rng("refg", "x", i + 1).standard_normal((1, 1024)).astype(np.float32) for i in range(STEPS)]
    pos = 0
    for i, x in enumerate(xs):
        o, _, n_nodes = reflib.ref_backbone_forward(x[None], pos, reflib.causal_mask(T0, T0) if i == 0 else None)
        same = np.array_equal(o[0], cpu[i])
        print(f"   restated graph on ggml-cpu, call {i}: {n_nodes} nodes, same bits as the reference's builder: {same} (nmse {nmse(cpu[i], o[0]):.2e})", flush=True)
        assert nmse(cpu[i], o[0]) <= 1e-10
        pos += x.shape[0]
    ref.rh_bb_free()


def test_weight_placement_under_the_scheduler(gpu, ref, tmp_path):
    """A model file with the stack's weights and AudioVAE weights, allocated by the plugin's placement helper (stack ->
    device buffer, audio_vae.* -> pinned host buffer) instead of the reference's one-buffer rule, and a graph with one
    weight of each kind under ggml_backend_sched over {plugin, CPU}: the projection of the stack runs on the plugin, the
    AudioVAE side (host weights, an operator the plugin does not claim) on ggml-cpu, and the result equals ggml-cpu's."""
    import ctypes
    vox = reflib.load_vox()
    if vox is None:
        pytest.skip("oracle/_ref/libvox_harness.so was not prebuilt")
    params = reflib.backbone_params("place", 1)
    g = rng("place", "vae")
    extra = [("audio_vae.encoder.fc_mu.weight", (g.standard_normal((64, 1024)) / 32).astype(np.float32)),
             ("audio_vae.encoder.fc_mu.bias", (0.1 * g.standard_normal(64)).astype(np.float32)),
             ("audio_vae.decoder.model.0.weight", g.standard_normal((7, 64)).astype(np.float32))]
    gguf = str(tmp_path / "placed.gguf")
    reflib.write_minicpm_gguf(gguf, params, "residual_lm", 4096, extra=extra)
    T = 9
    x = rng("place", "x").standard_normal((T, 1024)).astype(np.float32)
    names = (b"residual_lm.blk.0.attn_q.weight", b"audio_vae.encoder.fc_mu.weight", b"audio_vae.encoder.fc_mu.bias")

    def run(device, placement):
        out = np.zeros((T, 64), np.float32)
        flags = (ctypes.c_int64 * 5)()
        rc = vox.vh_placed_run(gguf.encode(), device, placement, *names, x.ctypes.data, T, out.ctypes.data, flags)
        assert rc == 0, vox.vh_last_error()
        return out, list(flags)

    cpu, cf = run(b"CPU", 0)
    assert vox.vh_load_plugin(gpu.PLUGIN_PATH.encode()) == 0
    placed, pf = run(b"GFX950_0", 1)
    one_buf, of = run(b"GFX950_0", 0)
    print(f"placement: splits {pf[0]}, stack weight on host {pf[1]}, audio_vae weight on host {pf[2]}, device buffer {pf[3] >> 20} MiB, "
          f"host buffer {pf[4]} bytes; one-buffer rule: splits {of[0]}, device buffer {of[3] >> 20} MiB", flush=True)
    assert pf[1] == 0 and pf[2] == 1 and pf[3] > 15 << 20 and 0 < pf[4] < 1 << 20
    assert of[1] == 0 and of[2] == 0 and of[4] == 0          # the reference's rule: everything on the device
    assert pf[0] == 2                                          # the plugin's part, then ggml-cpu's
    e = nmse(cpu, placed)
    print(f"   placed weights vs ggml-cpu: nmse {e:.3e};  one buffer vs ggml-cpu: nmse {nmse(cpu, one_buf):.3e}", flush=True)
    assert e <= 1e-4 and nmse(cpu, one_buf) <= 1e-4
