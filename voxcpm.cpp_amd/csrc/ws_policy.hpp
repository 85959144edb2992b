// ws_policy.hpp -- growth policy of the per-stream scratch workspace.  Free of HIP calls (the allocator
// is a parameter), so the policy can be exercised on a host without a device.
//
// Rule: a block that was ever handed out is never freed or moved while its stream lives.  Kernels already
// queued on the stream, and HIP graphs captured from it, hold the block's address in their arguments; a
// replay after the workspace has grown must still find the memory it was recorded with.  Growth therefore
// allocates a new block and retires the old one; retired blocks are released when the stream is destroyed.
// Each growth at least doubles the block, so all retired blocks together are smaller than the live one.
// Growth while the stream is being captured is refused (an allocation must not be recorded into a graph):
// reserve the largest size before capturing.
#pragma once

#include <cstddef>
#include <vector>

struct vx_ws_block {
    void * ptr   = nullptr;
    size_t bytes = 0;
};

struct vx_ws_state {
    vx_ws_block              cur;
    std::vector<vx_ws_block> retired;
};

enum vx_ws_result { VX_WS_OK = 0, VX_WS_GREW = 1, VX_WS_CAPTURING = 2, VX_WS_ALLOC_FAILED = 3 };

static inline size_t vx_ws_grown_size(size_t have, size_t bytes) {
    size_t want = bytes + bytes / 4;
    if (want < 2 * have) want = 2 * have;
    if (want < ((size_t) 1 << 20)) want = (size_t) 1 << 20;
    return (want + 255) & ~(size_t) 255;
}

// alloc(bytes) returns a pointer or nullptr.  *out is the block to use on VX_WS_OK / VX_WS_GREW.
template <class Alloc>
static inline vx_ws_result vx_ws_request(vx_ws_state & s, size_t bytes, bool capturing, Alloc && alloc, void ** out) {
    if (bytes <= s.cur.bytes) {
        *out = s.cur.ptr;
        return VX_WS_OK;
    }
    if (capturing) return VX_WS_CAPTURING;
    const size_t want = vx_ws_grown_size(s.cur.bytes, bytes);
    void *       p    = alloc(want);
    if (!p) return VX_WS_ALLOC_FAILED;
    if (s.cur.ptr) s.retired.push_back(s.cur);
    s.cur.ptr   = p;
    s.cur.bytes = want;
    *out        = p;
    return VX_WS_GREW;
}

// every block of the stream, live and retired, handed to release(ptr); the state is empty afterwards
template <class Release>
static inline void vx_ws_release_all(vx_ws_state & s, Release && release) {
    if (s.cur.ptr) release(s.cur.ptr);
    for (const vx_ws_block & b : s.retired) release(b.ptr);
    s.cur = vx_ws_block{};
    s.retired.clear();
}
