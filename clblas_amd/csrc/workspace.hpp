// Library-owned device scratch, one set of buffers per (device, stream).
//
// The reference allocates and frees its temporaries inside every call
// (src/library/blas/xtrsm.cc:1186-1207, 1499-1500); here buffers are kept and reused in stream
// order, so a call whose buffers exist only enqueues kernels.  The bookkeeping is plain host
// code, written against an allocator interface so that it can be unit-tested without a device.
//
// Rules:
//   * A buffer that is outgrown is not freed at once - kernels already enqueued may still use
//     it - but parked in the stream's "retired" list; the replacement is at least 1.5 times as
//     large, so the retired ones add up to at most twice the current size.
//   * release_stream(device, stream) frees everything the pair owns; the caller promises that the
//     stream's work has completed (it is about to destroy the stream).
//   * At most `max_streams` streams per device keep buffers.  When one more appears, the least
//     recently used one is evicted: the allocator's sync() hook runs first (device-wide
//     synchronisation), then its buffers are freed.  A process that creates and destroys
//     streams therefore holds a bounded amount of scratch even if it never calls
//     release_stream().
//   * Nothing is allocated while `may_allocate` (asked per request) says no - that is how a
//     stream under graph capture is kept from reaching hipMalloc.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <utility>
#include <vector>

namespace cba {

struct WorkspaceAllocator {
    void *(*alloc)(int device, size_t bytes);  // nullptr on failure
    void (*release)(int device, void *ptr);
    void (*sync)(int device);                  // all work on `device` has completed when it returns
};

enum WorkspaceKind { WS_GEMM = 0, WS_TRMM = 1, WS_TRSM = 2, WS_KINDS = 3 };

enum WorkspaceError { WS_OK = 0, WS_NO_MEMORY = 1, WS_CAPTURING = 2 };

class WorkspaceCache {
public:
    explicit WorkspaceCache(const WorkspaceAllocator &a, size_t max_streams = 32) : alloc_(a), max_streams_(max_streams) {}

    // Buffer of `kind` for (device, stream), at least `bytes` long; nullptr (and *err) on failure.
    // allow_alloc == false: only an existing, large enough buffer is returned (WS_CAPTURING otherwise).
    void *get(int device, const void *stream, int kind, size_t bytes, bool allow_alloc, WorkspaceError *err) {
        std::lock_guard<std::mutex> lock(mu_);
        if (err) *err = WS_OK;
        Key key(device, stream);
        auto it = streams_.find(key);
        if (it == streams_.end()) {
            if (!allow_alloc) { if (err) *err = WS_CAPTURING; return nullptr; }
            evict_for(device);
            it = streams_.emplace(key, Entry()).first;
        }
        Entry &e = it->second;
        e.last_use = ++clock_;
        Slot &s = e.slot[kind];
        if (s.ptr && s.bytes >= bytes) return s.ptr;
        if (!allow_alloc) { if (err) *err = WS_CAPTURING; return nullptr; }
        size_t want = bytes < kMinBytes ? kMinBytes : bytes;
        if (want < s.bytes + s.bytes / 2) want = s.bytes + s.bytes / 2;
        void *p = alloc_.alloc(device, want);
        if (!p && want != bytes) {  // no room for the margin: try the size that is needed
            want = bytes;
            p = alloc_.alloc(device, want);
        }
        if (!p) { if (err) *err = WS_NO_MEMORY; return nullptr; }
        if (s.ptr) e.retired.push_back(s.ptr);
        s.ptr = p;
        s.bytes = want;
        return p;
    }

    // Frees everything (device, stream) owns.  The stream's work must have completed.
    void release_stream(int device, const void *stream) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = streams_.find(Key(device, stream));
        if (it == streams_.end()) return;
        free_entry(device, it->second);
        streams_.erase(it);
    }

    void release_all() {
        std::lock_guard<std::mutex> lock(mu_);
        for (auto &kv : streams_) free_entry(kv.first.first, kv.second);
        streams_.clear();
    }

    size_t stream_count() {
        std::lock_guard<std::mutex> lock(mu_);
        return streams_.size();
    }
    size_t bytes_held() {
        std::lock_guard<std::mutex> lock(mu_);
        size_t n = 0;
        for (auto &kv : streams_)
            for (int k = 0; k < WS_KINDS; ++k) n += kv.second.slot[k].bytes;
        return n;
    }

    static constexpr size_t kMinBytes = (size_t)1 << 20;

private:
    typedef std::pair<int, const void *> Key;
    struct Slot { void *ptr = nullptr; size_t bytes = 0; };
    struct Entry {
        Slot slot[WS_KINDS];
        std::vector<void *> retired;
        uint64_t last_use = 0;
    };

    void free_entry(int device, Entry &e) {
        for (int k = 0; k < WS_KINDS; ++k)
            if (e.slot[k].ptr) alloc_.release(device, e.slot[k].ptr);
        for (void *p : e.retired) alloc_.release(device, p);
        e = Entry();
    }

    // Makes room for one more stream on `device`.
    void evict_for(int device) {
        for (;;) {
            size_t n = 0;
            std::map<Key, Entry>::iterator oldest = streams_.end();
            for (auto it = streams_.begin(); it != streams_.end(); ++it) {
                if (it->first.first != device) continue;
                ++n;
                if (oldest == streams_.end() || it->second.last_use < oldest->second.last_use) oldest = it;
            }
            if (n < max_streams_ || oldest == streams_.end()) return;
            alloc_.sync(device);
            free_entry(device, oldest->second);
            streams_.erase(oldest);
        }
    }

    WorkspaceAllocator alloc_;
    size_t max_streams_;
    std::mutex mu_;
    std::map<Key, Entry> streams_;
    uint64_t clock_ = 0;
};

}  // namespace cba
