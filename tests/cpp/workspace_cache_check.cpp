// Host-only check of the scratch-buffer bookkeeping (clblas_amd/csrc/workspace.hpp) with a
// counting allocator in place of hipMalloc / hipFree.  Prints "ok" and exits 0 on success.
#include <cstdio>
#include <cstdlib>
#include <set>

#include "workspace.hpp"

static std::set<void *> live;
static size_t live_bytes = 0, syncs = 0;
static std::map<void *, size_t> sizes;
static bool fail_big = false;

static void *t_alloc(int, size_t bytes) {
    if (fail_big && bytes > ((size_t)64 << 20)) return nullptr;
    void *p = std::malloc(16);
    live.insert(p);
    sizes[p] = bytes;
    live_bytes += bytes;
    return p;
}
static void t_release(int, void *p) {
    if (!live.count(p)) { std::puts("double free"); std::exit(1); }
    live.erase(p);
    live_bytes -= sizes[p];
    std::free(p);
}
static bool sync_ok = true;
static bool t_sync(int) { ++syncs; return sync_ok; }

#define CHECK(c) do { if (!(c)) { std::printf("FAILED line %d: %s\n", __LINE__, #c); return 1; } } while (0)

int main() {
    using namespace cba;
    WorkspaceAllocator a{t_alloc, t_release, t_sync};
    {
        WorkspaceCache c(a, 4);
        WorkspaceError err;
        const void *s1 = (const void *)0x10, *s2 = (const void *)0x20;
        // nothing exists, allocation not allowed (stream under capture)
        CHECK(c.get(0, s1, WS_GEMM, 100, false, &err) == nullptr && err == WS_CAPTURING);
        CHECK(c.stream_count() == 0 && live.empty());
        void *p = c.get(0, s1, WS_GEMM, 100, true, &err);
        CHECK(p && err == WS_OK && sizes[p] == WorkspaceCache::kMinBytes);
        CHECK(c.get(0, s1, WS_GEMM, 4096, true, &err) == p);           // reused
        CHECK(c.get(0, s1, WS_GEMM, 4096, false, &err) == p);          // fast path needs no allocation
        void *q = c.get(0, s1, WS_GEMM, (size_t)3 << 20, true, &err);  // outgrown: the old one is parked
        CHECK(q && q != p && live.count(p) && live.size() == 2);
        void *r = c.get(0, s1, WS_GEMM, ((size_t)3 << 20) + 1, true, &err);  // grows by at least half
        CHECK(r != q && sizes[r] >= sizes[q] + sizes[q] / 2);
        CHECK(c.get(0, s1, WS_TRSM, 10, true, &err) != r);             // kinds are separate buffers
        CHECK(c.get(0, s1, WS_GEMM, (size_t)1 << 40, false, &err) == nullptr && err == WS_CAPTURING);
        // create / use / release cycles do not accumulate
        const size_t before = live.size();
        for (uintptr_t i = 0; i < 1000; ++i) {
            const void *s = (const void *)(0x1000 + 16 * i);
            CHECK(c.get(0, s, WS_GEMM, (size_t)2 << 20, true, &err));
            CHECK(c.get(0, s, WS_TRMM, (size_t)5 << 20, true, &err));
            c.release_stream(0, s);
        }
        CHECK(live.size() == before && c.stream_count() == 1 && syncs == 0);
        // ... and neither do cycles without release: the least recently used stream is evicted
        for (uintptr_t i = 0; i < 1000; ++i) {
            const void *s = (const void *)(0x100000 + 16 * i);
            CHECK(c.get(0, s, WS_GEMM, (size_t)2 << 20, true, &err));
            CHECK(c.stream_count() <= 4);
        }
        CHECK(syncs > 0 && c.stream_count() == 4 && live.size() == 4);
        CHECK(c.bytes_held() == 4 * ((size_t)2 << 20));
        // another device has its own quota; a recently used stream survives
        CHECK(c.get(1, s2, WS_GEMM, 10, true, &err));
        CHECK(c.stream_count() == 5);
        const void *keep = (const void *)(0x100000 + 16 * 999);
        void *kp = c.get(0, keep, WS_GEMM, 10, false, &err);
        CHECK(kp);
        for (uintptr_t i = 0; i < 3; ++i) {
            CHECK(c.get(0, (const void *)(0x900000 + 16 * i), WS_GEMM, 10, true, &err));
            CHECK(c.get(0, keep, WS_GEMM, 10, false, &err) == kp);
        }
        // out of memory: first the margin is dropped, then the request fails cleanly
        fail_big = true;
        CHECK(c.get(0, keep, WS_TRMM, (size_t)60 << 20, true, &err));
        CHECK(c.get(0, keep, WS_TRMM, (size_t)64 << 20, true, &err));  // 1.5 x 60 MiB refused, 64 MiB fits
        CHECK(c.get(0, keep, WS_TRMM, (size_t)65 << 20, true, &err) == nullptr && err == WS_NO_MEMORY);
        fail_big = false;
        const size_t syncs_before = syncs;
        CHECK(c.release_all());
        CHECK(syncs == syncs_before + 2);  // once per device that held buffers
        CHECK(live.empty() && live_bytes == 0 && c.stream_count() == 0);
    }
    {
        // outgrown buffers count in the statistics until they are freed
        WorkspaceCache c(a, 4);
        WorkspaceError err;
        const void *s1 = (const void *)0x10;
        CHECK(c.get(0, s1, WS_GEMM, (size_t)2 << 20, true, &err));
        CHECK(c.get(0, s1, WS_GEMM, (size_t)8 << 20, true, &err));
        CHECK(c.bytes_held() == ((size_t)2 << 20) + ((size_t)8 << 20) && c.allocations() == 2);
        CHECK(c.release_all() && live.empty());
    }
    {
        // leases and pins keep an entry from eviction; a failed synchronisation evicts nothing
        WorkspaceCache c(a, 2);
        WorkspaceError err;
        const void *s1 = (const void *)0x10, *s2 = (const void *)0x20, *s3 = (const void *)0x30, *s4 = (const void *)0x40;
        void *p1 = c.get(0, s1, WS_GEMM, 10, true, &err);
        CHECK(!c.lease(0, s3));                       // no entry: nothing to hold
        CHECK(c.lease(0, s1));
        void *p2 = c.get(0, s2, WS_GEMM, 10, true, &err);
        CHECK(p1 && p2);
        CHECK(c.get(0, s3, WS_GEMM, 10, true, &err));  // s1 is the oldest but leased: s2 goes
        CHECK(c.get(0, s1, WS_GEMM, 10, false, &err) == p1);
        CHECK(c.get(0, s2, WS_GEMM, 10, false, &err) == nullptr);
        c.unlease(0, s1);
        c.pin(0, s1);
        CHECK(c.pinned(0, s1) && !c.pinned(0, s3));
        CHECK(c.get(0, s4, WS_GEMM, 10, true, &err));  // s1 pinned: s3 goes
        CHECK(c.get(0, s1, WS_GEMM, 10, false, &err) == p1);
        CHECK(c.get(0, s3, WS_GEMM, 10, false, &err) == nullptr);
        sync_ok = false;
        CHECK(c.get(0, s2, WS_GEMM, 10, true, &err));  // cannot synchronise: nobody is evicted, the quota is exceeded
        CHECK(c.stream_count() == 3);
        CHECK(!c.release_all() && c.stream_count() == 3);
        sync_ok = true;
        CHECK(c.release_all() && live.empty() && c.stream_count() == 0);
    }
    std::puts("ok");
    return 0;
}
