/*
 * ggml-gfx950.h -- what libggml-gfx950.so exports beside ggml's own plugin entry points
 * (ggml_backend_init / ggml_backend_score).  All of it is also reachable through
 * ggml_backend_reg_get_proc_address(reg, "<name>"), the way ggml hands out backend-specific functions.
 */
#ifndef GGML_GFX950_H
#define GGML_GFX950_H

#include "ggml-backend.h"
#include "ggml.h"

#ifdef __cplusplus
extern "C" {
#endif

GGML_BACKEND_API ggml_backend_reg_t ggml_backend_gfx950_reg(void);

/* Weight placement.  The reference puts every tensor of the model file into ONE buffer of the chosen backend
 * (VoxCPMWeightStore::load_from_file, src/weight-store.cpp:58-122).  This backend claims the operators of the
 * transformer stacks only, so the weights of what stays on ggml-cpu -- the AudioVAE's convolutions and snake
 * activations, `audio_vae.*` in the reference's GGUF naming (src/audio-vae.cpp:164-303) -- belong in host memory,
 * where ggml-cpu reads them in place, and everything else (token_embd, blk.*, residual_lm.*, locenc.*, locdit.*,
 * fsq.*, stop.*, the projections between the stages) in device memory.  With the weights split like this
 * ggml_backend_sched assigns each node to the backend that holds its weight and no weight ever crosses PCIe
 * after loading. */

/* 1: device buffer; 0: pinned host buffer.  By tensor name, as the reference's converter writes them. */
GGML_BACKEND_API int ggml_backend_gfx950_weight_on_device(const char * tensor_name);

/* Allocates every not yet allocated tensor of `ctx` (a no_alloc context, e.g. from gguf_init_from_file) by that rule:
 * tensors for the device in one device buffer, the rest in one pinned host buffer of this backend (either may come
 * back NULL when no tensor asks for it).  Both buffers get GGML_BACKEND_BUFFER_USAGE_WEIGHTS.  The caller frees them.
 * Returns false when an allocation fails (nothing is left allocated then). */
GGML_BACKEND_API bool ggml_backend_gfx950_alloc_weights(struct ggml_context * ctx, ggml_backend_t backend,
                                                        ggml_backend_buffer_t * device_buffer,
                                                        ggml_backend_buffer_t * host_buffer);

/* diagnostics and switches */
GGML_BACKEND_API int ggml_backend_gfx950_last_launches(void);
GGML_BACKEND_API int ggml_backend_gfx950_set_graph_replay(int on);  /* recognise recurring graphs and replay them; returns the previous setting */
GGML_BACKEND_API int ggml_backend_gfx950_replays(void);   /* graph_compute calls served by replaying recorded launches */
/* Graphs that share their nodes' operators and types with one seen before but differ in addresses, extents or
 * parameters (the steps of a decode loop) are run as that graph's recording with the differing launch arguments set
 * first.  Off by default (the comparison pass runs on the host before the GPU gets its first launch, which costs a
 * caller that waits for every step more than the launches it saves); GGML_GFX950_GRAPH_PATCH=1 or set_graph_patch(1)
 * switches it on; the setter returns the previous setting. */
GGML_BACKEND_API int ggml_backend_gfx950_set_graph_patch(int on);
GGML_BACKEND_API int ggml_backend_gfx950_patched_replays(void);   /* how many of the replays were of that kind */
GGML_BACKEND_API int ggml_backend_gfx950_last_patched(void);      /* launches whose arguments the latest one changed */
GGML_BACKEND_API int ggml_backend_gfx950_set_mul_mat_act(int mode);
GGML_BACKEND_API int ggml_backend_gfx950_set_fusion(int on);        /* groups of nodes as one launch (default) or every node its own; returns the previous setting */
GGML_BACKEND_API long long ggml_backend_gfx950_host_ns(int which);  /* the last node-by-node graph_compute: host ns spent (0) analysing the graph, (1) issuing launches */

#ifdef __cplusplus
}
#endif
#endif
