"""Host-side mirror of one UnifiedCFM solve around the LocDiT estimator, over the C ABI.

`LocDiTCfmSolver.plan` issues what `UnifiedCFM::solve_euler` (src/unified_cfm.cpp:88-149 of the reference) builds into
one ggml graph, with the launches the ggml backend plugin uses for it: per Euler step the input projection with its
bias (one call), the assembly of the CFG pair as ONE sequence of 2 * (1 + prefix + patch) tokens -- time token (+ mu
for the conditioned branch), projected condition, projected noisy patches, twice (src/locdit.cpp:401-452; one
vx_small_graph call) --, the decoder stack (`MiniCPMBackbone.plan`, non-causal, block-diagonal mask, positions
i mod branch length, no cache write), the output projection of both branches with its bias (two calls) and the
zero-star guidance arithmetic with the update of x (src/unified_cfm.cpp:30-86, 146; one vx_small_graph call).
Nothing is computed on the host.
"""
import numpy as np

from . import (NODE_ADD, NODE_ARANGE, NODE_CONCAT, NODE_DIV, NODE_MUL, NODE_REPEAT, NODE_SCALE, NODE_SUB, NODE_SUM, VxSmallNode, _stream,
               check, desc, desc_q8, lib, small_node)


class LocDiTCfmSolver:
    def __init__(self, decoder, feat, in_proj, cond_proj, out_proj):
        """decoder: a MiniCPMBackbone with batch 1 (weights loaded).  in_proj / cond_proj / out_proj: (Q8_0 rows as a uint8
        device tensor, row length K, F32 bias device tensor) -- feat -> hidden, feat -> hidden, hidden -> feat."""
        assert decoder.batch == 1
        self.dec, self.feat = decoder, feat
        self.in_proj, self.cond_proj, self.out_proj = in_proj, cond_proj, out_proj

    def plan(self, z, mu, cond, table, t_span, cfg_value=2.0, zero_star=True):
        """z (patch, feat), mu (hidden,), cond (prefix, feat), table (n_steps, hidden): F32 device tensors read at replay
        time; t_span: n_steps + 1 host floats.  Returns (run, x): run() enqueues the whole solve, x is the tensor it fills."""
        torch, L = self.dec.torch, lib()
        dev, f32 = z.device, torch.float32
        H, F = self.dec.hidden, self.feat
        patch, prefix = z.shape[0], cond.shape[0]
        n_steps = len(t_span) - 1
        Lb = 1 + prefix + patch
        T = 2 * Lb
        assert prefix >= 1 and T <= self.dec.max_length and table.shape == (n_steps, H)
        new = lambda *shape: torch.empty(shape, dtype=f32, device=dev)
        act = self.dec.act_mode
        calls, keep = [], [z, mu, cond, table]

        def call(fn, *args):
            calls.append((fn, args))

        def graph(nodes):   # a run of tiny nodes: one launch
            arr = (VxSmallNode * len(nodes))(*nodes)
            keep.append((nodes, arr))
            call(L.vx_small_graph, arr, len(nodes))

        def project(w, xin, dst):   # MUL_MAT + ADD(bias row), LocDiTModel::project_input / project_condition / out_proj
            rows, K, bias = w
            call(L.vx_mul_mat_scale_add, desc_q8(rows, K), desc(xin), desc(bias), desc(dst), 1.0, act)

        # the CFG-pair constants (LocDiTModel::ensure_cfg_pair_constants, src/locdit.cpp:63-130)
        pos = (torch.arange(T, dtype=torch.int32, device=dev) % Lb).to(torch.int32)
        branch = torch.arange(T, device=dev) >= Lb
        mask = torch.where(branch[None, :] != branch[:, None], float("-inf"), 0.0).to(torch.float16).contiguous()
        cond_p, x_proj = new(prefix, H), new(patch, H)
        comb_c, a5, a7, b5, b7, pair = new(1, H), new(1 + prefix, H), new(Lb, H), new(1 + prefix, H), new(Lb, H), new(T, H)
        vc, vu = new(patch, F), new(patch, F)
        tmp = {n: new(patch, F) for n in ("pc", "uu", "rep", "us", "diff", "cs", "dphi", "step")}
        sc = {n: new(1) for n in ("dot", "nrm", "eps", "den", "st")}
        xs = [new(patch, F) for _ in range(2)]
        keep += [pos, mask, cond_p, x_proj, comb_c, a5, a7, b5, b7, pair, vc, vu, tmp, sc, xs]
        dec_run, hidden = self.dec.plan(pair.view(1, T, H), T, 0, mask, write_kv=False, positions=pos)
        keep.append(dec_run)
        h2 = hidden.view(T, H)
        hc, hu = h2[prefix + 1:prefix + 1 + patch], h2[Lb + prefix + 1:Lb + prefix + 1 + patch]

        project(self.cond_proj, cond, cond_p)
        x = z
        f = np.float32                                   # solve_euler keeps t and dt in single precision
        t_span = [f(v) for v in t_span]
        t, dt = t_span[0], f(t_span[0] - t_span[1])
        zero_init_steps = max(1, int((n_steps + 1) * 0.04)) if n_steps > 1 else 0
        n_dec = 0
        for step in range(1, n_steps + 1):
            xn = xs[step % 2]
            if zero_star and step <= zero_init_steps:
                graph([small_node(NODE_SCALE, tmp["dphi"], x, p0=0.0, private=True), small_node(NODE_SCALE, tmp["step"], tmp["dphi"], p0=float(dt), private=True),
                       small_node(NODE_SUB, xn, x, tmp["step"])])
            else:
                project(self.in_proj, x, x_proj)
                row = table[step - 1:step]                       # the step's combined time embedding, (1, hidden)
                # (everything but the last node of a run is read inside the run only, as the plugin finds from the graph)
                graph([small_node(NODE_ADD, comb_c, row, mu.view(1, H), private=True),
                       small_node(NODE_CONCAT, a5, comb_c, cond_p, aux=1, private=True), small_node(NODE_CONCAT, a7, a5, x_proj, aux=1, private=True),
                       small_node(NODE_CONCAT, b5, row, cond_p, aux=1, private=True), small_node(NODE_CONCAT, b7, b5, x_proj, aux=1, private=True),
                       small_node(NODE_CONCAT, pair, a7, b7, aux=1)])
                calls.append((dec_run, None))
                n_dec += 1
                project(self.out_proj, hc, vc)
                project(self.out_proj, hu, vu)
                if zero_star:
                    nodes = [small_node(NODE_MUL, tmp["pc"], vc, vu, private=True), small_node(NODE_SUM, sc["dot"], tmp["pc"], private=True),
                             small_node(NODE_MUL, tmp["uu"], vu, vu, private=True), small_node(NODE_SUM, sc["nrm"], tmp["uu"], private=True),
                             small_node(NODE_ARANGE, sc["eps"], p0=1.0e-8, p1=1.0, private=True), small_node(NODE_ADD, sc["den"], sc["nrm"], sc["eps"], private=True),
                             small_node(NODE_DIV, sc["st"], sc["dot"], sc["den"], private=True), small_node(NODE_REPEAT, tmp["rep"], sc["st"], private=True),
                             small_node(NODE_MUL, tmp["us"], vu, tmp["rep"], private=True), small_node(NODE_SUB, tmp["diff"], vc, tmp["us"], private=True),
                             small_node(NODE_SCALE, tmp["cs"], tmp["diff"], p0=cfg_value, private=True), small_node(NODE_ADD, tmp["dphi"], tmp["us"], tmp["cs"], private=True)]
                else:
                    nodes = [small_node(NODE_SUB, tmp["diff"], vc, vu, private=True), small_node(NODE_SCALE, tmp["cs"], tmp["diff"], p0=cfg_value, private=True),
                             small_node(NODE_ADD, tmp["dphi"], vu, tmp["cs"], private=True)]
                nodes += [small_node(NODE_SCALE, tmp["step"], tmp["dphi"], p0=float(dt), private=True), small_node(NODE_SUB, xn, x, tmp["step"])]
                graph(nodes)
            x = xn
            t = f(t - dt)
            if step < n_steps:
                dt = f(t - t_span[step + 1])

        def run():
            st = _stream()
            for fn, args in calls:
                if args is None:
                    fn()
                    continue
                rc = fn(*args, st)
                if rc:
                    check(rc, fn.__name__)

        run._keep = keep
        run.n_calls = len(calls) - n_dec + n_dec * dec_run.n_calls
        return run, x
