// Host-only exercise of the workspace growth policy (voxcpm.cpp_amd/csrc/ws_policy.hpp) with a counting
// allocator in place of hipMalloc.  Prints "ok" or the first violated expectation; the Python test compiles
// and runs it with g++.
#include "../voxcpm.cpp_amd/csrc/ws_policy.hpp"

#include <cstdio>
#include <cstdlib>
#include <set>

#define EXPECT(c)                                              \
    do {                                                       \
        if (!(c)) {                                            \
            printf("line %d: %s\n", __LINE__, #c);             \
            return 1;                                          \
        }                                                      \
    } while (0)

int main() {
    std::set<void *> live;
    size_t           total = 0;
    bool             fail  = false;
    auto alloc = [&](size_t n) -> void * {
        if (fail) return nullptr;
        void * p = malloc(16);
        live.insert(p);
        total += n;
        return p;
    };
    vx_ws_state s;
    void *      p0 = nullptr;
    // first request: at least 1 MiB, a multiple of 256
    EXPECT(vx_ws_request(s, 1000, false, alloc, &p0) == VX_WS_GREW);
    EXPECT(s.cur.bytes == ((size_t) 1 << 20) && s.cur.ptr == p0 && s.retired.empty());
    // a smaller or equal request: same block, no allocation
    void * p1 = nullptr;
    EXPECT(vx_ws_request(s, 4096, false, alloc, &p1) == VX_WS_OK && p1 == p0);
    EXPECT(vx_ws_request(s, (size_t) 1 << 20, false, alloc, &p1) == VX_WS_OK && p1 == p0 && live.size() == 1);
    // growth during a stream capture is refused and changes nothing
    void * pc = (void *) 0x1;
    EXPECT(vx_ws_request(s, (size_t) 3 << 20, true, alloc, &pc) == VX_WS_CAPTURING);
    EXPECT(pc == (void *) 0x1 && s.cur.ptr == p0 && live.size() == 1);
    // a request that fits is fine during a capture
    EXPECT(vx_ws_request(s, 4096, true, alloc, &pc) == VX_WS_OK && pc == p0);
    // growth: a new block, the old one is retired -- still allocated, at its address
    void * p2 = nullptr;
    EXPECT(vx_ws_request(s, (size_t) 3 << 20, false, alloc, &p2) == VX_WS_GREW);
    EXPECT(p2 != p0 && s.cur.ptr == p2 && s.retired.size() == 1 && s.retired[0].ptr == p0 && live.count(p0) == 1);
    EXPECT(s.cur.bytes >= ((size_t) 3 << 20) + ((size_t) 3 << 18) && s.cur.bytes % 256 == 0);
    // a barely larger request at least doubles, so the retired blocks stay smaller than the live one
    void * p3 = nullptr;
    const size_t before = s.cur.bytes;
    EXPECT(vx_ws_request(s, before + 1, false, alloc, &p3) == VX_WS_GREW && s.cur.bytes >= 2 * before);
    size_t retired = 0;
    for (const vx_ws_block & b : s.retired) retired += b.bytes;
    EXPECT(retired < s.cur.bytes && s.retired.size() == 2);
    // an allocation failure leaves the state as it was
    fail = true;
    void * p4 = (void *) 0x2;
    EXPECT(vx_ws_request(s, s.cur.bytes * 4, false, alloc, &p4) == VX_WS_ALLOC_FAILED);
    EXPECT(p4 == (void *) 0x2 && s.cur.ptr == p3 && s.retired.size() == 2);
    fail = false;
    // destroying the stream releases every block exactly once
    size_t released = 0;
    vx_ws_release_all(s, [&](void * p) { released += live.erase(p); free(p); });
    EXPECT(released == 3 && live.empty() && s.cur.ptr == nullptr && s.cur.bytes == 0 && s.retired.empty());
    (void) total;
    printf("ok\n");
    return 0;
}
