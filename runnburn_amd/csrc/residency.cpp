// Resident-weight table: accounting, eviction planning, admission and the out-of-memory retry ladder (residency.h).
#include "residency.h"

#include <algorithm>

namespace rnb {

// ---- reuse history -------------------------------------------------------------------------------

uint64_t ReuseHistory::effective(const Entry &e) const {
    const uint64_t unobserved = epoch_ - e.last_seen > 0 ? epoch_ - e.last_seen - 1 : 0;
    const uint64_t periods = unobserved / decay_interval_;
    return periods >= 64 ? 0 : e.frequency >> periods;
}

void ReuseHistory::evict_lowest() {
    auto victim = entries_.end();
    for (auto it = entries_.begin(); it != entries_.end(); ++it) {
        if (victim == entries_.end()) {
            victim = it;
            continue;
        }
        const uint64_t fa = effective(it->second), fb = effective(victim->second);
        if (fa < fb || (fa == fb && it->second.last_seen < victim->second.last_seen)) victim = it;  // key order breaks ties
    }
    if (victim != entries_.end()) entries_.erase(victim);
}

uint64_t ReuseHistory::observe(std::pair<uintptr_t, size_t> key) {
    if (epoch_ != ~uint64_t(0)) ++epoch_;
    if (capacity_ == 0) return 0;
    uint64_t prior = 0;
    auto it = entries_.find(key);
    if (it != entries_.end()) prior = effective(it->second);
    entries_[key] = Entry{prior == ~uint64_t(0) ? prior : prior + 1, epoch_};
    if (entries_.size() > capacity_) evict_lowest();
    return prior;
}

void ReuseHistory::set_capacity(size_t capacity) {
    while (entries_.size() > capacity) evict_lowest();
    capacity_ = capacity;
    decay_interval_ = capacity ? capacity : 1;
}

// ---- table ---------------------------------------------------------------------------------------

void ResidentTable::set_budget(uint64_t bytes) {
    budget_ = bytes;
    Key victim;
    std::string scratch;
    while (resident_bytes_ > budget_ && pop_oldest_evictable(&victim)) drop(victim, &scratch, true);
}

void ResidentTable::touch(Key key, Entry &e) {
    e.last_touch = ++clock_;
    e.call = call_;
    oldest_.push({e.last_touch, key});
}

int ResidentTable::drop(Key key, std::string *err, bool count_eviction) {
    auto it = table_.find(key);
    if (it == table_.end()) return 0;
    const int rc = alloc_->free(it->second.dev, err);
    resident_bytes_ -= it->second.len;
    if (count_eviction) {
        ++stats_.evictions;
        stats_.evicted_bytes += it->second.len;
    }
    table_.erase(it);
    return rc;
}

bool ResidentTable::pop_oldest_evictable(Key *key) {
    // stale heap entries are discarded; live entries that may not be evicted now are put back afterwards
    std::vector<std::pair<uint64_t, Key>> keep;
    bool found = false;
    while (!oldest_.empty()) {
        const auto top = oldest_.top();
        oldest_.pop();
        auto it = table_.find(top.second);
        if (it == table_.end() || it->second.last_touch != top.first) continue;
        if (!evictable(it->second)) {
            keep.push_back(top);
            continue;
        }
        *key = top.second;
        keep.push_back(top);  // still live until the caller drops it
        found = true;
        break;
    }
    for (const auto &k : keep) oldest_.push(k);
    return found;
}

bool ResidentTable::plan(uint64_t incoming, std::vector<Key> *victims, uint64_t *victim_bytes) {
    victims->clear();
    *victim_bytes = 0;
    if (resident_bytes_ + incoming <= budget_) return true;
    std::vector<std::pair<uint64_t, Key>> order;
    for (const auto &kv : table_)
        if (evictable(kv.second)) order.push_back({kv.second.last_touch, kv.first});
    std::sort(order.begin(), order.end());
    for (const auto &cand : order) {
        victims->push_back(cand.second);
        *victim_bytes += table_[cand.second].len;
        if (resident_bytes_ - *victim_bytes + incoming <= budget_) return true;
    }
    return false;
}

int ResidentTable::alloc_with_retry(size_t bytes, void **dev, std::string *err) {
    std::string first;
    int rc = alloc_->alloc(bytes, dev, &first);
    if (rc != 1) {
        if (rc != 0) *err = first;
        return rc;
    }
    for (;;) {
        Key victim;
        if (!pop_oldest_evictable(&victim)) {
            *err = first;  // nothing evictable is left: the first out-of-memory error stands
            return 1;
        }
        std::string scratch;
        if (int frc = drop(victim, &scratch, true); frc != 0) {
            *err = scratch;
            return frc;
        }
        ++stats_.oom_retries;
        rc = alloc_->alloc(bytes, dev, &scratch);
        if (rc == 0) return 0;
        if (rc != 1) {
            *err = scratch;
            return rc;
        }
    }
}

bool ResidentTable::peek(const uint8_t *ptr, size_t len, uint64_t fingerprint, const uint8_t **dev_out) {
    const Key key = reinterpret_cast<Key>(ptr);
    auto it = table_.find(key);
    if (it != table_.end() && it->second.len == len) {
        if (it->second.fingerprint != fingerprint) return false;
        ++stats_.lookups;
        ++stats_.hits;
        touch(key, it->second);
        *dev_out = static_cast<const uint8_t *>(it->second.dev);
        return true;
    }
    auto up = table_.upper_bound(key);
    while (up != table_.begin()) {
        --up;
        const Key base = up->first;
        if (up->second.pinned && key >= base && key + len <= base + up->second.len) {
            ++stats_.lookups;
            ++stats_.sub_range_hits;
            touch(base, up->second);
            *dev_out = static_cast<const uint8_t *>(up->second.dev) + (key - base);
            return true;
        }
    }
    return false;
}

int ResidentTable::resolve(const uint8_t *ptr, size_t len, uint64_t fingerprint, bool pin, const uint8_t **dev_out,
                           std::string *err) {
    const Key key = reinterpret_cast<Key>(ptr);
    ++stats_.lookups;
    auto it = table_.find(key);
    if (it != table_.end() && it->second.len == len) {
        if (it->second.fingerprint == fingerprint) {
            touch(key, it->second);
            it->second.pinned = it->second.pinned || pin;
            ++stats_.hits;
            *dev_out = static_cast<const uint8_t *>(it->second.dev);
            return 0;
        }
        // same address and length, different bytes: the host range was reused
        if (int rc = drop(key, err, false); rc != 0) return rc;
    } else if (!pin) {
        // sub-range of a pinned parent (crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:722-741).  Unpinned
        // entries never serve sub-ranges: their host memory may have been freed and reused.
        auto up = table_.upper_bound(key);
        while (up != table_.begin()) {
            --up;
            const Key base = up->first;
            if (up->second.pinned && key >= base && key + len <= base + up->second.len) {
                touch(base, up->second);
                ++stats_.sub_range_hits;
                *dev_out = static_cast<const uint8_t *>(up->second.dev) + (key - base);
                return 0;
            }
        }
    }
    // an entry that starts at this address with another length is stale
    if (table_.count(key))
        if (int rc = drop(key, err, false); rc != 0) return rc;

    ++stats_.misses;
    // the history knows a range by address, length AND content: host memory that was freed and holds other data now is
    // a range that has not been seen before
    const uint64_t reuses = history_.observe({key, len + static_cast<size_t>(0x9E3779B97F4A7C15ull * fingerprint)});
    std::vector<Key> victims;
    uint64_t victim_bytes = 0;
    const bool fits = plan(len, &victims, &victim_bytes);
    // without evictions a missing range is always kept; with evictions only when keeping it saves more transfers than
    // reloading the victims costs (strict); a prewarm request is the caller's decision and always kept
    const bool pays = static_cast<unsigned __int128>(len) * (reuses + 1) >
                      static_cast<unsigned __int128>(len) + victim_bytes;
    const bool admit = pin || (fits && (victims.empty() || pays));
    void *dev = nullptr;
    if (!admit) {
        // this call only: outside the budget, freed by end_call
        if (int rc = alloc_with_retry(len, &dev, err); rc != 0) return rc;
        if (int rc = alloc_->upload(dev, ptr, len, err); rc != 0) {
            std::string scratch;
            alloc_->free(dev, &scratch);
            return rc;
        }
        temps_.push_back(dev);
        stats_.temp_h2d_bytes += len;
        *dev_out = static_cast<const uint8_t *>(dev);
        return 0;
    }
    for (const Key v : victims)
        if (int rc = drop(v, err, true); rc != 0) return rc;
    if (int rc = alloc_with_retry(len, &dev, err); rc != 0) return rc;
    if (int rc = alloc_->upload(dev, ptr, len, err); rc != 0) {
        std::string scratch;
        alloc_->free(dev, &scratch);
        return rc;
    }
    Entry e;
    e.len = len;
    e.dev = dev;
    e.fingerprint = fingerprint;
    e.pinned = pin;
    table_[key] = e;
    touch(key, table_[key]);
    resident_bytes_ += len;
    ++stats_.admissions;
    stats_.admitted_bytes += len;
    stats_.h2d_bytes += len;
    *dev_out = static_cast<const uint8_t *>(dev);
    return 0;
}

int ResidentTable::end_call(std::string *err) {
    int rc = 0;
    for (void *p : temps_) {
        std::string scratch;
        if (int frc = alloc_->free(p, &scratch); frc != 0 && rc == 0) {
            rc = frc;
            *err = scratch;
        }
    }
    temps_.clear();
    return rc;
}

bool ResidentTable::release(const uint8_t *ptr, size_t len, std::string *err) {
    auto it = table_.find(reinterpret_cast<Key>(ptr));
    if (it == table_.end() || it->second.len != len) return false;
    drop(it->first, err, false);
    return true;
}

uint64_t ResidentTable::offload_unpinned(std::string *err) {
    std::vector<Key> keys;
    for (const auto &kv : table_)
        if (!kv.second.pinned) keys.push_back(kv.first);
    uint64_t freed = 0;
    for (const Key k : keys) {
        freed += table_[k].len;
        drop(k, err, true);
    }
    return freed;
}

}  // namespace rnb
