// Resident-weight table of the HIP backend: which host ranges have a device copy, which of them a call may evict,
// and whether a missing range is worth keeping.  Host-only logic over an allocator interface, so that the policy is
// testable without a device (tests/cpp/residency_test.cpp drives it with a fake allocator that injects
// out-of-memory results).
//
// Policy, following the reference:
//  * byte-budgeted least-recently-used accounting, crates/rnb-memory/src/byte_lru.rs:32-91 (a clock, a heap of
//    (last touch, key) with stale heap entries skipped on pop);
//  * eviction candidates in least-recently-used order, never a pinned (prewarmed) entry and never an entry the
//    current call has already resolved (the reference's protected keys),
//    crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:1263-1330;
//  * admission of a missing range that does not fit without evictions only when it pays:
//    missing * (predicted reuses + 1) > missing + bytes that would have to be reloaded later
//    (evaluate_expert_bundle_admission, crates/rnb-memory/src/sparse_expert_cache.rs:221-250, strict inequality,
//    the current lookup counted as one saved transfer); otherwise the bytes are uploaded for this call only;
//  * predicted reuses = decayed frequency of earlier lookups of the same range
//    (ExpertBundleReuseHistory, sparse_expert_cache.rs:272-395: halves once per `decay_interval` unobserved epochs,
//    bounded capacity, lowest (frequency, recency, key) leaves first);
//  * when the allocator reports out of memory although the budget had room, further candidates are evicted one at
//    a time and the allocation retried until it succeeds or nothing evictable is left, in which case the first
//    out-of-memory error is returned (resident_q4k_mem_alloc_after_oom_with_bundle_eviction_retry,
//    q4k_cache.rs:1055-1079); the budget itself is never changed by a failed allocation;
//  * counters in the shape of ExpertBundleCacheStats (sparse_expert_cache.rs:383-395).
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <map>
#include <queue>
#include <string>
#include <utility>
#include <vector>

namespace rnb {

// What the table needs from the device: 0 = ok, 1 = out of memory, anything else = failure (message in *err).
struct DeviceAllocator {
    virtual ~DeviceAllocator() = default;
    virtual int alloc(size_t bytes, void **out, std::string *err) = 0;
    virtual int free(void *ptr, std::string *err) = 0;
    // untouched copy of [src, src + bytes) to the device allocation dst, complete on return
    virtual int upload(void *dst, const void *src, size_t bytes, std::string *err) = 0;
};

struct ResidencyStats {
    uint64_t lookups = 0, hits = 0, sub_range_hits = 0, misses = 0;
    uint64_t admissions = 0, evictions = 0, admitted_bytes = 0, evicted_bytes = 0;
    uint64_t h2d_bytes = 0, temp_h2d_bytes = 0, oom_retries = 0;
};

// Bounded frequency-and-recency history of lookups (sparse_expert_cache.rs:272-395).
class ReuseHistory {
  public:
    explicit ReuseHistory(size_t capacity = 4096) : capacity_(capacity), decay_interval_(capacity ? capacity : 1) {}
    // records one lookup, returns the decayed frequency before it
    uint64_t observe(std::pair<uintptr_t, size_t> key);
    size_t size() const { return entries_.size(); }
    void set_capacity(size_t capacity);

  private:
    struct Entry {
        uint64_t frequency, last_seen;
    };
    uint64_t effective(const Entry &e) const;
    void evict_lowest();
    size_t capacity_;
    uint64_t decay_interval_, epoch_ = 0;
    std::map<std::pair<uintptr_t, size_t>, Entry> entries_;
};

class ResidentTable {
  public:
    struct Entry {
        size_t len = 0;
        void *dev = nullptr;
        uint64_t fingerprint = 0;
        uint64_t last_touch = 0;
        uint64_t call = 0;    // the call that last resolved it: entries of the current call are never its victims
        bool pinned = false;  // prewarmed: never evicted, and the only kind a sub-range may resolve to
    };

    explicit ResidentTable(DeviceAllocator *alloc) : alloc_(alloc) {}

    // A smaller budget takes effect at once: least recently used unpinned entries go until the table fits (or none is left).
    void set_budget(uint64_t bytes);
    uint64_t budget() const { return budget_; }
    uint64_t resident_bytes() const { return resident_bytes_; }
    size_t entries() const { return table_.size(); }
    const ResidencyStats &stats() const { return stats_; }
    ReuseHistory &history() { return history_; }

    // A new API call starts: what it resolves from now on is protected from its own evictions.
    void begin_call() { ++call_; }
    // The call is over and the stream has drained: frees the uploads that were made for this call only.
    int end_call(std::string *err);
    bool has_call_temps() const { return !temps_.empty(); }

    // Device address of [ptr, ptr + len): an exact resident match (same address, length and fingerprint), a sub-range
    // of a pinned parent, a fresh upload that becomes resident, or an upload for this call only.  `fingerprint` is the
    // caller's cheap content hash of the range.  Returns 0, or an error code of the allocator with *err set.
    int resolve(const uint8_t *ptr, size_t len, uint64_t fingerprint, bool pin, const uint8_t **dev_out, std::string *err);
    // Device address of [ptr, ptr + len) when it is resident already (exact match or sub-range of a pinned parent);
    // false otherwise: nothing is uploaded and nothing evicted (the embedding gather then moves only the rows it needs).
    bool peek(const uint8_t *ptr, size_t len, uint64_t fingerprint, const uint8_t **dev_out);
    // Drops the entry that starts at ptr with this length; false when there is none.
    bool release(const uint8_t *ptr, size_t len, std::string *err);
    // Frees every unpinned entry (offload_non_pinned_resident_q4k, q4k_cache.rs:276-303); returns the bytes freed.
    uint64_t offload_unpinned(std::string *err);

  private:
    using Key = uintptr_t;
    bool evictable(const Entry &e) const { return !e.pinned && e.call != call_; }
    // least-recently-used evictable entries whose bytes bring resident + incoming under the budget; false when even
    // evicting all of them does not
    bool plan(uint64_t incoming, std::vector<Key> *victims, uint64_t *victim_bytes);
    bool pop_oldest_evictable(Key *key);
    void touch(Key key, Entry &e);
    int drop(Key key, std::string *err, bool count_eviction);
    int alloc_with_retry(size_t bytes, void **dev, std::string *err);

    DeviceAllocator *alloc_;
    uint64_t budget_ = ~uint64_t(0), resident_bytes_ = 0, clock_ = 0, call_ = 0;
    std::map<Key, Entry> table_;  // keyed by host base address
    // (last touch, key), oldest first; entries whose touch no longer matches the table are stale and skipped
    std::priority_queue<std::pair<uint64_t, Key>, std::vector<std::pair<uint64_t, Key>>,
                        std::greater<std::pair<uint64_t, Key>>>
        oldest_;
    std::vector<void *> temps_;
    ReuseHistory history_;
    ResidencyStats stats_;
};

}  // namespace rnb
