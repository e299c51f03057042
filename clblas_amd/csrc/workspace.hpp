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
//     stream's work has completed (the C entry point synchronises the stream first).
//   * release_all() runs the allocator's sync() hook for every device that holds buffers, then
//     frees them.
//   * At most `max_streams` streams per device keep buffers.  When one more appears, the least
//     recently used one that may go is evicted: the allocator's sync() hook runs first (device-wide
//     synchronisation; if it fails nothing is evicted), then its buffers are freed.  A process that
//     creates and destroys streams therefore holds a bounded amount of scratch even if it never
//     calls release_stream().  An entry may not go while a call holds a lease on it (lease() /
//     unlease(): the call has a pointer and may not have enqueued its kernels yet) or once it has
//     been pinned (pin(): a captured graph holds its pointers for as long as the graph lives).
//   * Nothing is allocated while `allow_alloc` (asked per request) says no - that is how a
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
    bool (*sync)(int device);                  // true: all work on `device` has completed
};

enum WorkspaceKind { WS_GEMM = 0, WS_TRMM = 1, WS_TRSM = 2, WS_KINDS = 3 };

enum WorkspaceError { WS_OK = 0, WS_NO_MEMORY = 1, WS_CAPTURING = 2 };

class WorkspaceCache {
public:
    explicit WorkspaceCache(const WorkspaceAllocator &a, size_t max_streams = 32) : alloc_(a), max_streams_(max_streams) {}

    // Buffer of `kind` for (device, stream), at least `bytes` long; nullptr (and *err) on failure.
    // allow_alloc == false: only an existing, large enough buffer is returned (WS_CAPTURING otherwise).
    // take_lease: on success the entry's lease count goes up by one (see lease()); is_pinned receives
    // whether the entry is pinned.
    void *get(int device, const void *stream, int kind, size_t bytes, bool allow_alloc, WorkspaceError *err,
              bool take_lease = false, bool *is_pinned = nullptr) {
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
        if (is_pinned) *is_pinned = e.pinned;
        if (s.ptr && s.bytes >= bytes) {
            if (take_lease) ++e.users;
            return s.ptr;
        }
        if (!allow_alloc) { if (err) *err = WS_CAPTURING; return nullptr; }
        size_t want = bytes < kMinBytes ? kMinBytes : bytes;
        if (want < s.bytes + s.bytes / 2) want = s.bytes + s.bytes / 2;
        void *p = alloc_.alloc(device, want);
        if (!p && want != bytes) {  // no room for the margin: try the size that is needed
            want = bytes;
            p = alloc_.alloc(device, want);
        }
        if (!p) { if (err) *err = WS_NO_MEMORY; return nullptr; }
        if (s.ptr) { e.retired.push_back(s.ptr); e.retired_bytes += s.bytes; }
        ++allocations_;
        s.ptr = p;
        s.bytes = want;
        if (take_lease) ++e.users;
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

    // Synchronises every device that holds buffers, then frees them all.  Buffers of a device whose
    // synchronisation fails are kept (their kernels may still be running); returns false then.
    bool release_all() {
        std::lock_guard<std::mutex> lock(mu_);
        bool all = true;
        std::map<int, bool> synced;
        for (auto it = streams_.begin(); it != streams_.end();) {
            const int device = it->first.first;
            auto s = synced.find(device);
            if (s == synced.end()) s = synced.emplace(device, alloc_.sync(device)).first;
            if (!s->second) { all = false; ++it; continue; }
            free_entry(device, it->second);
            it = streams_.erase(it);
        }
        return all;
    }

    // A call's claim on the entry of (device, stream): while any stands, the entry is not evicted.
    // lease() returns false if the pair has no entry (nothing to protect).
    bool lease(int device, const void *stream) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = streams_.find(Key(device, stream));
        if (it == streams_.end()) return false;
        ++it->second.users;
        return true;
    }
    void unlease(int device, const void *stream) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = streams_.find(Key(device, stream));
        if (it != streams_.end() && it->second.users > 0) --it->second.users;
    }
    // Keeps the entry of (device, stream) from eviction for good (until release_stream / release_all).
    void pin(int device, const void *stream) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = streams_.find(Key(device, stream));
        if (it != streams_.end()) it->second.pinned = true;
    }
    bool pinned(int device, const void *stream) {
        std::lock_guard<std::mutex> lock(mu_);
        auto it = streams_.find(Key(device, stream));
        return it != streams_.end() && it->second.pinned;
    }

    size_t stream_count() {
        std::lock_guard<std::mutex> lock(mu_);
        return streams_.size();
    }
    // Bytes of the current buffers plus those of the outgrown ones that are still parked.
    size_t bytes_held() {
        std::lock_guard<std::mutex> lock(mu_);
        size_t n = 0;
        for (auto &kv : streams_) {
            for (int k = 0; k < WS_KINDS; ++k) n += kv.second.slot[k].bytes;
            n += kv.second.retired_bytes;
        }
        return n;
    }
    // Allocations made since the cache was created.
    size_t allocations() {
        std::lock_guard<std::mutex> lock(mu_);
        return allocations_;
    }

    static constexpr size_t kMinBytes = (size_t)1 << 20;

private:
    typedef std::pair<int, const void *> Key;
    struct Slot { void *ptr = nullptr; size_t bytes = 0; };
    struct Entry {
        Slot slot[WS_KINDS];
        std::vector<void *> retired;
        size_t retired_bytes = 0;
        uint64_t last_use = 0;
        int users = 0;        // leases outstanding
        bool pinned = false;  // a captured graph holds pointers into the buffers
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
                if (it->second.users > 0 || it->second.pinned) continue;  // in use by a call / held by a graph
                if (oldest == streams_.end() || it->second.last_use < oldest->second.last_use) oldest = it;
            }
            if (n < max_streams_ || oldest == streams_.end()) return;
            if (!alloc_.sync(device)) return;  // (e.g. a stream of the device is being captured): keep everything
            free_entry(device, oldest->second);
            streams_.erase(oldest);
        }
    }

    WorkspaceAllocator alloc_;
    size_t max_streams_;
    std::mutex mu_;
    std::map<Key, Entry> streams_;
    uint64_t clock_ = 0;
    size_t allocations_ = 0;
};

}  // namespace cba
