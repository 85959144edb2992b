"""Host-side mirror of the reference's MiniCPM decoder stack over the C ABI.

`MiniCPMBackbone.forward` issues, operator for operator, what `MiniCPMModel::layer_forward`,
`attention_forward` and `mlp_forward` put into a ggml graph (src/minicpm.cpp:572-846 of the
reference): rms_norm * weight, separate Q/K/V projections, NEOX rope with frequency factors,
the KV append (ggml_cpy into the cache's write view, followed by the cont/sum/scale-by-zero
chain the reference uses to order the write), concat(past view, current keys), flash
attention, add1, the output projection, the muP residual scale and the SwiGLU MLP.  Every
operator is one vx_* call on device tensors; nothing is computed on the host.

Independent sequences (the CFG pair, concurrent streams) ride in the batch dimension, which is
ggml's ne[3]; with batch 1 the call sequence is the reference's graph node for node.

A `plan` is the prepared call list for one (n_tokens, n_past): descriptors and intermediates
are built once, so a plan can be replayed from a captured HIP graph.

With `fuse_pairs=True` the adjacent nodes the ggml backend plugin runs as one launch (rms_norm+mul,
scale+add, cont+sum, add+scale, and at decode size the gate/up/SwiGLU triple, projection+scale+add, the
nine-node cache write with its ordering scalar, the q/k/v projections with both rotations, rms_norm joined
to the projections behind it, and attention over cached + current keys without the two concats) are issued as the plugin issues them, so a plan
has as many launches as the plugin needs for the reference's graph; the results are bit-identical
to the unfused sequence.
"""
import math

import numpy as np

from . import (ACT_FLOAT, BIN_ADD, BIN_MUL, F16, F32, GLU_SWIGLU, _p, _stream, check, desc, desc_q8, lib)

WEIGHT_NAMES = ("q_proj", "k_proj", "v_proj", "o_proj", "gate_proj", "up_proj", "down_proj")


class MiniCPMBackbone:
    def __init__(self, n_layer=24, hidden=1024, n_heads=16, n_kv_heads=2, head_dim=64, ffn=4096, max_length=1024,
                 batch=1, eps=1e-5, use_mup=False, scale_depth=1.4, kv_f16=False, act_mode=ACT_FLOAT,
                 rope_base=10000.0, rope_original_max=32768, fuse_pairs=True):
        import torch
        self.torch = torch
        self.n_layer, self.hidden, self.n_heads, self.n_kv, self.D = n_layer, hidden, n_heads, n_kv_heads, head_dim
        self.ffn, self.max_length, self.batch, self.eps = ffn, max_length, batch, eps
        self.use_mup = use_mup
        # in single precision, as MiniCPMModel computes it (src/minicpm.cpp:276): the double-precision quotient rounds to
        # the neighbouring float for some layer counts (6, 24), and every residual update would differ in its last bit
        self.residual_scale = float(np.float32(scale_depth) / np.sqrt(np.float32(max(1, n_layer)))) if use_mup else 1.0
        self.act_mode = act_mode
        self.fuse_pairs = fuse_pairs
        self.rope_base, self.rope_original_max = rope_base, rope_original_max
        self.kv_dtype = torch.float16 if kv_f16 else torch.float32
        dev = "cuda"
        # KV cache, src/minicpm.cpp:178-187: per layer K and V [head_dim, max_length, n_kv_heads] (x batch)
        self.k_cache = [torch.zeros((batch, n_kv_heads, max_length, head_dim), dtype=self.kv_dtype, device=dev) for _ in range(n_layer)]
        self.v_cache = [torch.zeros((batch, n_kv_heads, max_length, head_dim), dtype=self.kv_dtype, device=dev) for _ in range(n_layer)]
        self.weights = [dict() for _ in range(n_layer)]   # name -> (uint8 Q8_0 rows, K)
        self._pinned = {}                                 # base address -> tensor, for the ranges given to vx_weights_pin
        self.norms = [dict() for _ in range(n_layer)]     # "input_layernorm" / "post_layernorm" -> f32 [hidden]
        self.final_norm = None
        self.rope_factors = None                          # f32 [head_dim / 2] or None

    # ---- loading --------------------------------------------------------------------------
    def set_weight(self, layer, name, q8_rows, K):
        """q8_rows: uint8 tensor (rows, K/32*34) of Q8_0 blocks, on the device."""
        self.unpin_weights()
        self.weights[layer][name] = (q8_rows, K)

    def pin_weights(self):
        """Declare the loaded weights constant (vx_weights_pin), as the reference marks its weight buffers
        (src/weight-store.cpp:86): the large products then keep their weights' tiles between calls.  The tensors must
        not be written to or released while pinned; set_weight and the destructor unpin."""
        for layer in self.weights:
            for q8_rows, _ in layer.values():
                base, size = q8_rows.data_ptr(), q8_rows.numel() * q8_rows.element_size()
                if base not in self._pinned:
                    check(lib().vx_weights_pin(base, size), "vx_weights_pin")
                    self._pinned[base] = q8_rows   # (kept alive while pinned)

    def unpin_weights(self):
        for base in list(self._pinned):
            lib().vx_weights_unpin(base)
            del self._pinned[base]

    def __del__(self):
        try:
            self.unpin_weights()
        except Exception:
            pass

    def set_norm(self, layer, name, w):
        if layer < 0:
            self.final_norm = w
        else:
            self.norms[layer][name] = w

    def clear_cache(self):
        for t in self.k_cache + self.v_cache:
            t.zero_()

    # ---- one (n_tokens, n_past) call list -----------------------------------------------------
    def plan(self, x, n_tokens, n_past, mask=None, write_kv=True, positions=None):
        """x: (batch, n_tokens, hidden) f32 device tensor, read at replay time.  Returns
        (run, out): run() enqueues the whole stack on torch's current stream; out is the
        (batch, n_tokens, hidden) result tensor it fills.  positions: int32 device tensor of n_tokens rope
        positions (default n_past .. n_past + n_tokens - 1; LocDiT's CFG pair passes i mod branch length)."""
        torch, L = self.torch, lib()
        B, T, H, Hkv, D = self.batch, n_tokens, self.n_heads, self.n_kv, self.D
        assert x.shape == (B, T, self.hidden) and x.dtype == torch.float32 and x.is_contiguous()
        assert n_past + T <= self.max_length
        dev = x.device
        f32 = torch.float32
        N = B * T

        def new(*shape, dtype=f32):
            return torch.empty(shape, dtype=dtype, device=dev)

        pos = torch.arange(n_past, n_past + T, dtype=torch.int32, device=dev) if positions is None else positions
        assert pos.dtype == torch.int32 and pos.numel() == T
        seq_len = n_past + T
        attn_factor = 1.0
        if seq_len > self.rope_original_max > 1:  # apply_rope, src/minicpm.cpp:590-594
            attn_factor = math.sqrt(1.0 + math.log(seq_len / self.rope_original_max) / math.log(self.rope_original_max))
        keep = [pos, x, mask]
        calls = []

        def call(fn, *args):
            calls.append((fn, args))

        fuse = self.fuse_pairs

        def norm(xin, w, dst):          # MiniCPMModel::rms_norm
            if fuse:
                call(L.vx_rms_norm_mul, desc(xin), desc(w), desc(dst), self.eps)
            else:
                call(L.vx_rms_norm, desc(xin), desc(dst), self.eps)
                call(L.vx_binary, BIN_MUL, desc(dst), desc(w), desc(dst))

        def project_residual(wdesc, xin, branch, res, dst):  # projection, optional muP scale, residual add
            sc = self.residual_scale if self.use_mup else 1.0
            if fuse and L.vx_supports_mul_mat_scale_add(wdesc, desc(xin), desc(res), desc(dst)):
                call(L.vx_mul_mat_scale_add, wdesc, desc(xin), desc(res), desc(dst), sc, self.act_mode)
                return
            call(L.vx_mul_mat, wdesc, desc(xin), desc(branch), self.act_mode)
            residual(res, branch, dst)

        def residual(res, branch, dst):  # optional muP scale, then the residual add
            if self.use_mup and fuse:
                call(L.vx_scale_add, desc(res), desc(branch), desc(dst), self.residual_scale)
                return
            if self.use_mup:
                call(L.vx_scale, desc(branch), desc(branch), self.residual_scale, 0.0)
            call(L.vx_binary, BIN_ADD, desc(res), desc(branch), desc(dst))

        # buffers reused by every layer (the stack is sequential)
        normed, q, k, v = new(N, self.hidden), new(N, H * D), new(N, Hkv * D), new(N, Hkv * D)
        kcont, vcont = new(B, T, Hkv, D), new(B, T, Hkv, D)   # the written slot as dense F32 (CONT, or the cast back from F16)
        sk, sv = new(1), new(1)
        sync = new(1)
        kall = new(B, Hkv, seq_len, D, dtype=self.kv_dtype) if n_past > 0 else None
        vall = new(B, Hkv, seq_len, D, dtype=self.kv_dtype) if n_past > 0 else None
        kcast = new(B, Hkv, T, D, dtype=self.kv_dtype) if (n_past > 0 and self.kv_dtype != f32) else None
        vcast = new(B, Hkv, T, D, dtype=self.kv_dtype) if (n_past > 0 and self.kv_dtype != f32) else None
        attn, attn_o = new(B, T, H, D), new(N, self.hidden)
        gate, up, act, down = new(N, self.ffn), new(N, self.ffn), new(N, self.ffn), new(N, self.hidden)
        hs = [new(N, self.hidden) for _ in range(2)]   # residual stream ping-pong
        h_mid = new(N, self.hidden)
        out = new(B, T, self.hidden)
        keep += [normed, q, k, v, kcont, vcont, sk, sv, sync, kall, vall, kcast, vcast, attn, attn_o, gate, up, act, down, h_mid, out] + hs
        # The cont/sum/scale-by-zero chain only exists to order the cache write inside a ggml graph.  It is typed
        # F32 (ggml's SCALE and ADD1 are F32 operators): with an F16 cache the written slot is read back through a
        # cast to F32 where the F32 cache has its CONT.
        chain = write_kv
        f16_cache = self.kv_dtype != f32
        scale = 1.0 / math.sqrt(D)
        ff = _p(self.rope_factors)
        cur_x = x.view(N, self.hidden)
        for li in range(self.n_layer):
            w, nrm = self.weights[li], self.norms[li]
            kc, vc = self.k_cache[li], self.v_cache[li]
            wd = {n: desc_q8(*w[n]) for n in WEIGHT_NAMES}
            # -- attention_forward
            q4, k4, v4 = q.view(B, T, H, D), k.view(B, T, Hkv, D), v.view(B, T, Hkv, D)
            rope_args = (D, 2, self.rope_original_max, self.rope_base, 1.0, 0.0, attn_factor, 32.0, 1.0)
            # (with an F16 cache the graph casts the rotated keys between the K and V projections; the plugin only groups
            # the projections when no other node runs between them, i.e. when attention reads the F32 keys in place and
            # the casts are never run -- which needs the keys alive at the attention node: a step that writes the cache)
            plain_order = n_past == 0 or not f16_cache or write_kv
            wqkv = (wd["q_proj"], wd["k_proj"], wd["v_proj"])
            nw_in = nrm["input_layernorm"]
            if fuse and plain_order and (L.vx_supports_norm_qkv_proj_rope(desc(cur_x), desc(nw_in), *wqkv, desc(q4), desc(k4), desc(v), D, 2) or
                                         L.vx_supports_norm_qkv_proj_rope_tiled(desc(cur_x), desc(nw_in), *wqkv, desc(q4), desc(k4), desc(v), D, 2, self.act_mode)):
                # rms_norm, the three projections and both rotations as one call (one launch at decode sizes; at prefill sizes the
                # norm in the activation pass, one product for the three matrices, the rotations behind it)
                call(L.vx_norm_qkv_proj_rope, desc(cur_x), desc(nw_in), self.eps, *wqkv, _p(pos), ff, desc(q4), desc(k4), desc(v),
                     *rope_args, self.act_mode)
            elif fuse and plain_order and L.vx_supports_qkv_proj_rope(*wqkv, desc(normed), desc(q4), desc(k4), desc(v), D, 2):
                norm(cur_x, nw_in, normed)
                call(L.vx_qkv_proj_rope, *wqkv, desc(normed), _p(pos), ff, desc(q4), desc(k4), desc(v), *rope_args, self.act_mode)
            else:
                norm(cur_x, nw_in, normed)
                call(L.vx_mul_mat, wd["q_proj"], desc(normed), desc(q), self.act_mode)
                call(L.vx_rope, desc(q4), _p(pos), ff, desc(q4), *rope_args)
                if fuse and plain_order and L.vx_supports_kv_proj_rope(wd["k_proj"], wd["v_proj"], desc(normed), desc(k4), desc(v), D, 2):
                    # a prompt of a few hundred tokens: k, v and k's rotation still fit one launch of the streaming kernel
                    call(L.vx_kv_proj_rope, wd["k_proj"], wd["v_proj"], desc(normed), _p(pos), ff, desc(k4), desc(v), *rope_args, self.act_mode)
                else:
                    call(L.vx_mul_mat, wd["k_proj"], desc(normed), desc(k), self.act_mode)
                    call(L.vx_rope, desc(k4), _p(pos), ff, desc(k4), *rope_args)
                    call(L.vx_mul_mat, wd["v_proj"], desc(normed), desc(v), self.act_mode)
            # from here on in the order ggml_build_forward_expand gives the reference's graph: concat, attention,
            # then the cache append with its ordering chain, then add1 (only adjacent nodes are run as one launch)
            k_all, v_all = k4.transpose(1, 2), v4.transpose(1, 2)   # ggml_permute(0, 2, 1, 3)
            stored = False
            projected = False
            if n_past > 0:
                kp, vp = kc[:, :, :n_past], vc[:, :, :n_past]
                qd = desc(q4.transpose(1, 2))
                # The plugin lets attention read the cached and the current keys where they lie (no concat, and with an
                # F16 cache no cast: the kernel rounds the F32 keys as it loads them) when the current keys are still
                # alive at the attention node.  In the reference's graph they are when the cache write, their other
                # reader, comes later: a step that writes the cache.
                alive = write_kv
                if not (fuse and alive) and kcast is not None:
                    call(L.vx_cpy, desc(k_all), desc(kcast))
                    call(L.vx_cpy, desc(v_all), desc(vcast))
                    k_all, v_all = kcast, vcast
                kw = kc[:, :, n_past:n_past + T].transpose(1, 2)   # the cache's write views, ggml [D, Hkv, T, B]
                vw = vc[:, :, n_past:n_past + T].transpose(1, 2)
                if fuse and alive and L.vx_supports_flash_attn_ext_kv2_store(qd, desc(kp), desc(k_all), desc(vp), desc(v_all), desc(mask),
                                                                             desc(k4), desc(kw), desc(v4), desc(vw), desc(attn)):
                    # attention, the cache write and its ordering scalar as one call (two kernels)
                    keep += [kw, vw]
                    call(L.vx_flash_attn_ext_kv2_store, qd, desc(kp), desc(k_all), desc(vp), desc(v_all), desc(mask), None,
                         desc(k4), desc(kw), desc(v4), desc(vw), desc(attn), scale, 0.0, 0.0, 0.0, 0.0)
                    k_all = None
                    stored = True
                elif fuse and alive and L.vx_supports_flash_attn_ext_kv2(qd, desc(kp), desc(k_all), desc(vp), desc(v_all), desc(mask), desc(attn)):
                    call(L.vx_flash_attn_ext_kv2, qd, desc(kp), desc(k_all), desc(vp), desc(v_all), desc(mask), None, desc(attn),
                         scale, 0.0, 0.0)
                    k_all = None
                else:
                    if k_all.dtype != kp.dtype:   # (a shape the two-segment kernel leaves to the tiled one)
                        call(L.vx_cpy, desc(k_all), desc(kcast))
                        call(L.vx_cpy, desc(v_all), desc(vcast))
                        k_all, v_all = kcast, vcast
                    call(L.vx_concat, desc(kp), desc(k_all), desc(kall), 1)
                    call(L.vx_concat, desc(vp), desc(v_all), desc(vall), 1)
                    k_all, v_all = kall, vall
            if k_all is not None:
                qd = desc(q4.transpose(1, 2))
                kw = kc[:, :, n_past:n_past + T].transpose(1, 2)
                vw = vc[:, :, n_past:n_past + T].transpose(1, 2)
                sc_o = self.residual_scale if self.use_mup else 1.0
                attn2 = attn.view(N, H * D)
                if write_kv and chain and fuse and L.vx_supports_flash_attn_ext_store_proj(
                        qd, desc(k_all), desc(v_all), desc(mask), desc(k4), desc(kw), desc(v4), desc(vw), desc(attn2), wd["o_proj"], desc(cur_x),
                        desc(h_mid), 0.0, self.act_mode):
                    # a large prefill: as below, and the attention's result goes to the o projection as that product's f16
                    # tiles (it is never stored); the projection applies the residual update
                    keep += [kw, vw, attn2]
                    call(L.vx_flash_attn_ext_store_proj, qd, desc(k_all), desc(v_all), desc(mask), None, desc(k4), desc(kw), desc(v4), desc(vw),
                         desc(attn2), wd["o_proj"], desc(cur_x), desc(h_mid), scale, 0.0, 0.0, 0.0, 0.0, sc_o, self.act_mode)
                    stored = True
                    projected = True
                elif write_kv and chain and fuse and L.vx_supports_flash_attn_ext_store(qd, desc(k_all), desc(v_all), desc(mask), desc(k4), desc(kw),
                                                                                      desc(v4), desc(vw), desc(attn), 0.0):
                    # a prefill: the cache write and its scalar first, the scalar added in the attention's epilogue
                    keep += [kw, vw]
                    call(L.vx_flash_attn_ext_store, qd, desc(k_all), desc(v_all), desc(mask), None, desc(k4), desc(kw), desc(v4), desc(vw),
                         desc(attn), scale, 0.0, 0.0, 0.0, 0.0)
                    stored = True
                else:
                    call(L.vx_flash_attn_ext, qd, desc(k_all), desc(v_all), desc(mask), None, desc(attn), scale, 0.0, 0.0)
            grouped = stored
            if write_kv and not stored:
                kw = kc[:, :, n_past:n_past + T].transpose(1, 2)   # ggml [D, Hkv, T, B], src/minicpm.cpp:222-236
                vw = vc[:, :, n_past:n_past + T].transpose(1, 2)
                keep += [kw, vw]
                grouped = bool(chain and fuse and L.vx_supports_kv_store_sync(desc(k4), desc(kw), desc(v4), desc(vw), desc(attn), desc(attn)))
            if stored:
                pass
            elif grouped:      # both cache writes, their sums, add, scale and add1 as one launch
                call(L.vx_kv_store_sync, desc(k4), desc(kw), desc(v4), desc(vw), desc(attn), desc(attn), 0.0, 0.0)
            elif write_kv:
                for src4, wv, cont, ssum in ((k4, kw, kcont, sk), (v4, vw, vcont, sv)):
                    call(L.vx_cpy, desc(src4), desc(wv))
                    if chain and fuse and not f16_cache:
                        call(L.vx_sum, desc(wv), desc(ssum))       # cont + sum
                    elif chain:
                        call(L.vx_cpy, desc(wv), desc(cont))
                        call(L.vx_sum, desc(cont), desc(ssum))
            if grouped:
                pass
            elif chain and fuse:
                call(L.vx_add_scale, desc(sk), desc(sv), desc(sync), 0.0, 0.0)
            elif chain:
                call(L.vx_binary, BIN_ADD, desc(sk), desc(sv), desc(sync))
                call(L.vx_scale, desc(sync), desc(sync), 0.0, 0.0)
            if chain and not grouped:
                call(L.vx_add1, desc(attn), desc(sync), desc(attn))
            if not projected:
                project_residual(wd["o_proj"], attn.view(N, H * D), attn_o, cur_x, h_mid)
            # -- mlp_forward
            nw_post = nrm["post_layernorm"]
            nxt = hs[li % 2]
            sc_res = self.residual_scale if self.use_mup else 1.0
            if fuse and L.vx_supports_mlp_tiled(desc(h_mid), desc(nw_post), wd["gate_proj"], wd["up_proj"], wd["down_proj"], desc(h_mid), desc(nxt), self.act_mode):
                # prefill sizes: the whole of mlp_forward with its residual update as one call (the tokens x ffn tensor is never stored)
                call(L.vx_mlp_tiled, desc(h_mid), desc(nw_post), self.eps, wd["gate_proj"], wd["up_proj"], wd["down_proj"], desc(h_mid), sc_res,
                     desc(nxt), self.act_mode)
                cur_x = nxt
                continue
            if fuse and (L.vx_supports_norm_mul_mat_swiglu(desc(h_mid), desc(nw_post), wd["gate_proj"], wd["up_proj"], desc(act)) or
                         L.vx_supports_norm_mul_mat_swiglu_tiled(desc(h_mid), desc(nw_post), wd["gate_proj"], wd["up_proj"], desc(act), self.act_mode)):
                # rms_norm, gate, up and SwiGLU as one launch
                call(L.vx_norm_mul_mat_swiglu, desc(h_mid), desc(nw_post), self.eps, wd["gate_proj"], wd["up_proj"], desc(act), self.act_mode)
            elif fuse and (N <= 16 or L.vx_supports_mul_mat_swiglu_tiled(wd["gate_proj"], wd["up_proj"], desc(normed), desc(act), self.act_mode)):
                # gate, up and SwiGLU as one launch (few tokens: the streaming kernel; prefill sizes: the tiled kernel's epilogue)
                norm(h_mid, nw_post, normed)
                call(L.vx_mul_mat_swiglu, wd["gate_proj"], wd["up_proj"], desc(normed), desc(act), self.act_mode)
            else:
                norm(h_mid, nw_post, normed)
                call(L.vx_mul_mat, wd["gate_proj"], desc(normed), desc(gate), self.act_mode)
                call(L.vx_mul_mat, wd["up_proj"], desc(normed), desc(up), self.act_mode)
                call(L.vx_glu, GLU_SWIGLU, desc(gate), desc(up), desc(act), 0)
            nxt = hs[li % 2]
            project_residual(wd["down_proj"], act, down, h_mid, nxt)
            cur_x = nxt
        o2 = out.view(N, self.hidden)
        norm(cur_x, self.final_norm, o2)

        def run():
            st = _stream()
            for fn, args in calls:
                rc = fn(*args, st)
                if rc:
                    check(rc, fn.__name__)

        run._keep = keep
        run.calls = calls           # (function, arguments) in launch order, for tools that time parts of a step
        run.n_calls = len(calls)
        return run, out

    def forward(self, x, n_past=0, mask=None, write_kv=True):
        """MiniCPMModel::forward / forward_step: x (batch, n_tokens, hidden) -> same shape."""
        run, out = self.plan(x.contiguous(), x.shape[1], n_past, mask, write_kv)
        run()
        return out
