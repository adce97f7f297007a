// Host-only test of the resident-weight table (runnburn_amd/csrc/residency.{h,cpp}) against a fake device
// allocator: eviction order, protection of the current call's ranges and of prewarmed ones, the admission rule of
// crates/rnb-memory/src/sparse_expert_cache.rs:221-250, the out-of-memory retry ladder of
// crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:1055-1079 and the reuse history of
// sparse_expert_cache.rs:272-395.  The byte-LRU cases restate crates/rnb-memory/src/byte_lru.rs:108-135.
//   g++ -O1 -std=c++17 tests/cpp/residency_test.cpp runnburn_amd/csrc/residency.cpp -o tests/cpp/residency_test
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>

#include "../../runnburn_amd/csrc/residency.h"

using namespace rnb;

static int g_checks = 0, g_failed = 0;
#define CHECK(cond)                                                         \
    do {                                                                    \
        ++g_checks;                                                         \
        if (!(cond)) {                                                      \
            ++g_failed;                                                     \
            std::printf("FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);   \
        }                                                                   \
    } while (0)

// "device" = malloc'd host memory with a byte capacity; counts what is live
struct FakeDevice : DeviceAllocator {
    size_t capacity = ~size_t(0), used = 0, inject_oom = 0, uploads = 0, upload_bytes = 0;
    bool fail_upload = false;
    std::map<void *, size_t> live;
    ~FakeDevice() override {
        for (auto &kv : live) std::free(kv.first);  // what the table still holds when a test ends
    }
    int alloc(size_t bytes, void **out, std::string *err) override {
        if (inject_oom > 0) {
            --inject_oom;
            *err = "injected out of memory";
            return 1;
        }
        if (used + bytes > capacity) {
            *err = "out of memory: " + std::to_string(bytes);
            return 1;
        }
        *out = std::malloc(bytes ? bytes : 1);
        live[*out] = bytes;
        used += bytes;
        return 0;
    }
    int free(void *p, std::string *err) override {
        auto it = live.find(p);
        if (it == live.end()) {
            *err = "free of a pointer that is not live";
            return 2;
        }
        used -= it->second;
        live.erase(it);
        std::free(p);
        return 0;
    }
    int upload(void *dst, const void *src, size_t bytes, std::string *err) override {
        if (fail_upload) {
            *err = "upload failed";
            return 2;
        }
        if (!live.count(dst)) {
            *err = "upload into a pointer that is not live";
            return 2;
        }
        std::memcpy(dst, src, bytes);
        ++uploads;
        upload_bytes += bytes;
        return 0;
    }
    bool is_live(const void *p) const { return live.count(const_cast<void *>(p)) != 0; }
};

static uint8_t g_host[1 << 16];
static const uint8_t *H(size_t off) { return g_host + off; }

static const uint8_t *resolve_ok(ResidentTable &t, size_t off, size_t len, bool pin = false, uint64_t fp = 1) {
    const uint8_t *dev = nullptr;
    std::string err;
    const int rc = t.resolve(H(off), len, fp, pin, &dev, &err);
    CHECK(rc == 0);
    if (rc != 0) std::printf("  resolve error: %s\n", err.c_str());
    return dev;
}

static void test_hits_and_accounting() {
    FakeDevice d;
    ResidentTable t(&d);
    t.set_budget(10);
    t.begin_call();
    for (size_t i = 0; i < sizeof(g_host); i++) g_host[i] = static_cast<uint8_t>(i * 7 + 3);
    const uint8_t *a = resolve_ok(t, 0, 4);
    CHECK(std::memcmp(a, H(0), 4) == 0);  // untouched copy
    const uint8_t *b = resolve_ok(t, 100, 4);
    t.begin_call();
    CHECK(resolve_ok(t, 0, 4) == a);  // hit: same device address, no second upload
    CHECK(d.uploads == 2);
    CHECK(t.resident_bytes() == 8 && t.entries() == 2);
    CHECK(t.stats().lookups == 3 && t.stats().hits == 1 && t.stats().misses == 2 && t.stats().admissions == 2);
    // same address and length, different contents (fingerprint): uploaded again
    t.begin_call();
    const uint8_t *a2 = resolve_ok(t, 0, 4, false, 2);
    CHECK(d.uploads == 3 && t.resident_bytes() == 8);
    (void)a2;
    // same address, another length: the old entry is stale
    t.begin_call();
    resolve_ok(t, 100, 3);
    CHECK(t.resident_bytes() == 7 && t.entries() == 2 && !d.is_live(b));
    std::string err;
    CHECK(t.release(H(100), 3, &err) && t.resident_bytes() == 4);
    CHECK(!t.release(H(100), 3, &err));
    CHECK(d.used == 4);
}

static void test_admission_and_lru_order() {
    // budget 10 as in byte_lru.rs: 1 (4 bytes), 2 (4 bytes), touch 1, then 3 (5 bytes) must displace 2, the oldest
    FakeDevice d;
    ResidentTable t(&d);
    t.set_budget(10);
    t.begin_call();
    const uint8_t *k1 = resolve_ok(t, 0, 4);
    t.begin_call();
    const uint8_t *k2 = resolve_ok(t, 100, 4);
    t.begin_call();
    CHECK(resolve_ok(t, 0, 4) == k1);
    // first lookup of 3: keeping it would cost 4 bytes of later reload and save nothing yet (5 * 1 > 5 + 4 is false):
    // uploaded for this call only
    t.begin_call();
    const uint8_t *k3 = resolve_ok(t, 200, 5);
    CHECK(d.is_live(k3) && d.is_live(k2) && t.resident_bytes() == 8 && t.has_call_temps());
    CHECK(t.stats().temp_h2d_bytes == 5 && t.stats().evictions == 0);
    std::string err;
    CHECK(t.end_call(&err) == 0 && !d.is_live(k3) && !t.has_call_temps());
    // second lookup: one earlier lookup predicted, 5 * 2 > 5 + 4: admitted, and the victim is 2, not the touched 1
    t.begin_call();
    k3 = resolve_ok(t, 200, 5);
    CHECK(d.is_live(k3) && d.is_live(k1) && !d.is_live(k2));
    CHECK(t.resident_bytes() == 9 && t.stats().evictions == 1 && t.stats().evicted_bytes == 4);
    CHECK(!t.has_call_temps());
}

static void test_current_call_is_protected() {
    // a call whose three matrices exceed the budget: none of them may be freed under the call
    FakeDevice d;
    ResidentTable t(&d);
    t.set_budget(10);
    t.begin_call();
    const uint8_t *old = resolve_ok(t, 900, 3);  // an earlier call's range
    for (int round = 0; round < 3; round++) {    // also once the history predicts reuse
        t.begin_call();
        const uint8_t *gate = resolve_ok(t, 0, 6);
        const uint8_t *up = resolve_ok(t, 100, 6);
        const uint8_t *down = resolve_ok(t, 200, 6);
        CHECK(d.is_live(gate) && d.is_live(up) && d.is_live(down));
        CHECK(gate != up && up != down && gate != down);
        CHECK(std::memcmp(gate, H(0), 6) == 0 && std::memcmp(up, H(100), 6) == 0 && std::memcmp(down, H(200), 6) == 0);
        CHECK(t.resident_bytes() <= t.budget());
        std::string err;
        CHECK(t.end_call(&err) == 0);
        CHECK(t.resident_bytes() <= t.budget());
    }
    (void)old;
    CHECK(t.budget() == 10);
}

static void test_pinned_and_sub_ranges() {
    FakeDevice d;
    ResidentTable t(&d);
    t.set_budget(20);
    t.begin_call();
    const uint8_t *slab = resolve_ok(t, 0, 16, /*pin=*/true);
    t.begin_call();
    // an expert inside the prewarmed slab resolves to parent + offset without an upload
    CHECK(resolve_ok(t, 4, 8) == slab + 4 && d.uploads == 1 && t.stats().sub_range_hits == 1);
    const uint8_t *u = resolve_ok(t, 1000, 4);  // unpinned
    t.begin_call();
    // a sub-range of an UNPINNED entry is not served from it
    const uint8_t *sub = resolve_ok(t, 1001, 2);
    CHECK(sub != u + 1);
    // pressure: pinned entries are never victims, even for a range seen often
    for (int i = 0; i < 4; i++) {
        t.begin_call();
        resolve_ok(t, 2000, 12);
        std::string err;
        t.end_call(&err);
    }
    CHECK(d.is_live(slab));
    // prewarm requests are always kept (they may take the table over the budget)
    t.begin_call();
    const uint8_t *slab2 = resolve_ok(t, 3000, 16, true);
    CHECK(d.is_live(slab) && d.is_live(slab2));
    // a smaller budget evicts at once, least recently used first, never the prewarmed ranges
    t.begin_call();
    const uint8_t *v1 = resolve_ok(t, 5000, 2);
    t.begin_call();
    const uint8_t *v2 = resolve_ok(t, 5100, 2);
    t.begin_call();
    t.set_budget(t.resident_bytes() - 1);
    CHECK(!d.is_live(u) && d.is_live(v1) && d.is_live(v2) && d.is_live(slab) && d.is_live(slab2));  // u is the oldest
    std::string err;
    CHECK(t.offload_unpinned(&err) <= 20);
    CHECK(d.is_live(slab) && d.is_live(slab2) && t.entries() == 2);
}

static void test_peek_never_uploads() {
    // the embedding gather asks whether a table is resident already and moves single rows when it is not
    FakeDevice d;
    ResidentTable t(&d);
    t.set_budget(64);
    const uint8_t *dev = nullptr;
    CHECK(!t.peek(H(0), 16, 1, &dev) && d.uploads == 0 && t.entries() == 0 && t.stats().lookups == 0);
    t.begin_call();
    const uint8_t *table = resolve_ok(t, 0, 16);
    t.begin_call();
    CHECK(t.peek(H(0), 16, 1, &dev) && dev == table && d.uploads == 1 && t.stats().hits == 1);
    CHECK(!t.peek(H(0), 16, /*fingerprint=*/2, &dev));  // the host range now holds other bytes: not the resident copy
    CHECK(!t.peek(H(0), 8, 1, &dev) && !t.peek(H(4), 8, 1, &dev));  // unpinned entries serve no sub-ranges
    t.begin_call();
    const uint8_t *slab = resolve_ok(t, 100, 32, /*pin=*/true);
    CHECK(t.peek(H(108), 8, 7, &dev) && dev == slab + 8 && t.stats().sub_range_hits == 1);
    CHECK(!t.peek(H(124), 16, 7, &dev));  // runs past the end of the parent
    CHECK(d.uploads == 2 && t.entries() == 2 && t.stats().misses == 2);
    // a peek counts as a use: the peeked entry is not the next victim
    t.begin_call();
    const uint8_t *other = resolve_ok(t, 200, 8);
    t.begin_call();
    CHECK(t.peek(H(0), 16, 1, &dev));
    t.begin_call();
    t.set_budget(t.resident_bytes() - 1);  // one unpinned entry has to go: the one at 200, the older use
    CHECK(d.is_live(table) && !d.is_live(other) && t.stats().evictions == 1 && t.entries() == 2);
}

static void test_oom_ladder() {
    FakeDevice d;
    d.capacity = 12;  // the device holds less than the budget allows
    ResidentTable t(&d);
    t.set_budget(100);
    t.begin_call();
    const uint8_t *a = resolve_ok(t, 0, 5);
    t.begin_call();
    const uint8_t *b = resolve_ok(t, 100, 5);
    t.begin_call();
    const uint8_t *c = resolve_ok(t, 200, 5);  // fits the budget, not the device: the oldest range goes, then it fits
    CHECK(d.is_live(c) && d.is_live(b) && !d.is_live(a));
    CHECK(t.stats().oom_retries == 1 && t.stats().evictions == 1 && t.budget() == 100);
    // nothing evictable is left inside one call: the first out-of-memory error comes back, the table stays consistent
    t.begin_call();
    resolve_ok(t, 100, 5);
    resolve_ok(t, 200, 5);
    const uint8_t *dev = nullptr;
    std::string err;
    CHECK(t.resolve(H(300), 5, 1, false, &dev, &err) == 1 && err.find("out of memory") != std::string::npos);
    CHECK(d.is_live(b) && d.is_live(c) && t.resident_bytes() == 10 && t.budget() == 100);
    // the next call can evict them again
    t.begin_call();
    CHECK(resolve_ok(t, 300, 5) != nullptr);
    // an upload failure frees the fresh allocation
    d.fail_upload = true;
    t.begin_call();
    const size_t used = d.used;
    CHECK(t.resolve(H(400), 1, 1, false, &dev, &err) == 2 && d.used == used);
}

static void test_reuse_history() {
    ReuseHistory h(2);  // decay interval = capacity = 2 epochs
    const std::pair<uintptr_t, size_t> k1{1, 8}, k2{2, 8}, k3{3, 8};
    CHECK(h.observe(k1) == 0);
    CHECK(h.observe(k1) == 1);
    CHECK(h.observe(k1) == 2);
    CHECK(h.observe(k2) == 0);  // epoch 4
    CHECK(h.observe(k2) == 1);  // epoch 5
    CHECK(h.observe(k2) == 2);  // epoch 6
    CHECK(h.observe(k2) == 3);  // epoch 7
    CHECK(h.observe(k1) == 0);  // epoch 8: k1 (frequency 3, last seen at 3) unobserved for 4 epochs = 2 halvings: 3 >> 2
    ReuseHistory g(4);
    CHECK(g.observe(k1) == 0 && g.observe(k1) == 1 && g.observe(k1) == 2 && g.observe(k1) == 3);  // frequency 4 at epoch 4
    for (int i = 0; i < 5; i++) g.observe(k2);  // epochs 5..9
    CHECK(g.observe(k1) == 2);  // epoch 10: unobserved 5, one interval of 4 -> 4 >> 1
    // bounded: the lowest (frequency, recency) leaves
    ReuseHistory b(2);
    b.observe(k1);
    b.observe(k1);
    b.observe(k2);
    b.observe(k3);  // k2 (frequency 1, older) leaves, k1 and k3 stay
    CHECK(b.size() == 2);
    CHECK(b.observe(k2) == 0);
}

int main() {
    test_hits_and_accounting();
    test_admission_and_lru_order();
    test_current_call_is_protected();
    test_pinned_and_sub_ranges();
    test_peek_never_uploads();
    test_oom_ladder();
    test_reuse_history();
    std::printf("%d checks, %d failed\n", g_checks, g_failed);
    return g_failed == 0 ? 0 : 1;
}
