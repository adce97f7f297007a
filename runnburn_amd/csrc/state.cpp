// Device state: lazy open, scratch, pinned bounce buffers, resident weights.
#include "state.h"

#include <cstdlib>
#include <cstring>

#include "../../include/rnb_hip.h"

namespace rnb {

namespace {
thread_local std::string t_last_error;
std::mutex g_mutex;
State *g_state = nullptr;
int g_open_status = -1;  // -1 = not tried yet
std::string g_open_error;

size_t round_up(size_t v, size_t to) { return (v + to - 1) / to * to; }

// Sampled FNV-1a over (len, first/last 256 bytes, 64 strided 8-byte probes): cheap enough to run
// per call, and catches a host address that was reused for different contents.  The reference
// hashes the storage identity or the whole slice (crates/rnb-backend/cuda/src/runtime/helpers.rs:3-30).
uint64_t fingerprint(const uint8_t *p, size_t len) {
    uint64_t h = 0xcbf29ce484222325ull;
    auto mix = [&h](const uint8_t *q, size_t n) {
        for (size_t i = 0; i < n; i++) h = (h ^ q[i]) * 0x100000001b3ull;
    };
    uint64_t l = len;
    mix(reinterpret_cast<const uint8_t *>(&l), 8);
    if (len <= 1024) {
        mix(p, len);
        return h;
    }
    mix(p, 256);
    mix(p + len - 256, 256);
    const size_t stride = (len - 8) / 64;
    for (size_t i = 1; i < 64; i++) mix(p + i * stride, 8);
    return h;
}
}  // namespace

void set_last_error(const std::string &msg) { t_last_error = msg; }
const char *last_error_cstr() { return t_last_error.c_str(); }

hipError_t DeviceBuf::reserve(size_t bytes) {
    if (bytes <= cap) return hipSuccess;
    if (ptr) {
        hipError_t e = hipFree(ptr);
        ptr = nullptr;
        cap = 0;
        if (e != hipSuccess) return e;
    }
    const size_t want = round_up(bytes + bytes / 4, 4096);
    hipError_t e = hipMalloc(&ptr, want);
    if (e != hipSuccess) {
        ptr = nullptr;
        return e;
    }
    cap = want;
    return hipSuccess;
}

hipError_t PinnedBuf::reserve(size_t bytes) {
    if (bytes <= cap) return hipSuccess;
    if (ptr) {
        hipError_t e = hipHostFree(ptr);
        ptr = nullptr;
        cap = 0;
        if (e != hipSuccess) return e;
    }
    const size_t want = round_up(bytes + bytes / 4, 4096);
    hipError_t e = hipHostMalloc(&ptr, want, hipHostMallocDefault);
    if (e != hipSuccess) {
        ptr = nullptr;
        return e;
    }
    cap = want;
    return hipSuccess;
}

void State::evict_unpinned_until(uint64_t need) {
    // least-recently-used first (crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:789-823)
    while (resident_bytes + need > resident_budget) {
        auto victim = residents.end();
        for (auto it = residents.begin(); it != residents.end(); ++it)
            if (!it->second.pinned && (victim == residents.end() || it->second.epoch < victim->second.epoch)) victim = it;
        if (victim == residents.end()) return;
        (void)hipStreamSynchronize(stream);
        (void)hipFree(victim->second.dev);
        resident_bytes -= victim->second.len;
        residents.erase(victim);
    }
}

hipError_t State::resident_ptr(const uint8_t *ptr, size_t len, const uint8_t **dev_out, bool pin) {
    const uintptr_t key = reinterpret_cast<uintptr_t>(ptr);
    ++epoch;
    auto it = residents.find(key);
    if (it != residents.end() && it->second.len == len) {
        if (it->second.fingerprint == fingerprint(ptr, len)) {
            it->second.epoch = epoch;
            it->second.pinned = it->second.pinned || pin;
            *dev_out = static_cast<const uint8_t *>(it->second.dev);
            return hipSuccess;
        }
        // same address and length, different bytes: the host range was reused
        resident_bytes -= it->second.len;
        (void)hipStreamSynchronize(stream);
        (void)hipFree(it->second.dev);
        residents.erase(it);
    } else if (!pin) {
        // sub-range of a pinned parent slab (crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:722-741).
        // Unpinned entries never serve sub-ranges: their host memory may have been freed and reused.
        auto up = residents.upper_bound(key);
        while (up != residents.begin()) {
            --up;
            const uintptr_t base = up->first;
            if (up->second.pinned && key >= base && key + len <= base + up->second.len) {
                up->second.epoch = epoch;
                *dev_out = static_cast<const uint8_t *>(up->second.dev) + (key - base);
                return hipSuccess;
            }
        }
    }
    // an entry that starts at this address with another length is stale
    it = residents.find(key);
    if (it != residents.end()) {
        resident_bytes -= it->second.len;
        (void)hipStreamSynchronize(stream);
        (void)hipFree(it->second.dev);
        residents.erase(it);
    }
    evict_unpinned_until(len);
    void *dev = nullptr;
    hipError_t e = hipMalloc(&dev, round_up(len, 256) + 256);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        resident_budget = resident_bytes;  // out of memory: shrink the budget to what fits and retry once
        evict_unpinned_until(len);
        e = hipMalloc(&dev, round_up(len, 256) + 256);
        if (e != hipSuccess) return e;
    }
    e = hipMemcpyAsync(dev, ptr, len, hipMemcpyHostToDevice, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) {
        (void)hipFree(dev);
        return e;
    }
    h2d_bytes += len;
    Resident r;
    r.len = len;
    r.dev = dev;
    r.fingerprint = fingerprint(ptr, len);
    r.epoch = epoch;
    r.pinned = pin;
    residents[key] = r;
    resident_bytes += len;
    *dev_out = static_cast<const uint8_t *>(dev);
    return hipSuccess;
}

bool State::release(const uint8_t *ptr, size_t len) {
    auto it = residents.find(reinterpret_cast<uintptr_t>(ptr));
    if (it == residents.end() || it->second.len != len) return false;
    (void)hipStreamSynchronize(stream);
    (void)hipFree(it->second.dev);
    resident_bytes -= it->second.len;
    residents.erase(it);
    return true;
}

Guard::Guard() : lock(g_mutex) {
    if (g_state) {
        state = g_state;
        hipError_t e = hipSetDevice(state->device);
        if (e != hipSuccess) {
            set_last_error(std::string("hipSetDevice: ") + hipGetErrorString(e));
            status = RNB_HIP_EXECUTION_FAILED;
            state = nullptr;
        }
        return;
    }
    if (g_open_status > 0) {  // an earlier open failed; report the same thing without retrying
        set_last_error(g_open_error);
        status = g_open_status;
        return;
    }
    auto fail = [this](int st, const std::string &msg) {
        g_open_status = st;
        g_open_error = msg;
        set_last_error(msg);
        status = st;
    };
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess || count <= 0) {
        (void)hipGetLastError();
        fail(RNB_HIP_NO_DEVICE, std::string("no HIP device: hipGetDeviceCount: ") +
                                    (e != hipSuccess ? hipGetErrorString(e) : "0 devices"));
        return;
    }
    int ordinal = 0;
    if (const char *env = std::getenv("RNB_HIP_DEVICE")) ordinal = std::atoi(env);
    if (ordinal < 0 || ordinal >= count) {
        fail(RNB_HIP_NO_DEVICE, "no HIP device: RNB_HIP_DEVICE=" + std::to_string(ordinal) + " out of range, " +
                                    std::to_string(count) + " device(s)");
        return;
    }
    e = hipSetDevice(ordinal);
    if (e != hipSuccess) {
        fail(RNB_HIP_NO_DEVICE, std::string("no HIP device: hipSetDevice: ") + hipGetErrorString(e));
        return;
    }
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, ordinal);
    if (e != hipSuccess) {
        fail(RNB_HIP_NO_DEVICE, std::string("no HIP device: hipGetDeviceProperties: ") + hipGetErrorString(e));
        return;
    }
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        fail(RNB_HIP_NO_DEVICE, std::string("no HIP device: kernels are built for gfx950, device is ") + prop.gcnArchName);
        return;
    }
    State *s = new State();
    s->device = ordinal;
    s->device_name = std::string(prop.name) + " (" + prop.gcnArchName + ")";
    e = hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking);  // default priority
    if (e != hipSuccess) {
        delete s;
        fail(RNB_HIP_EXECUTION_FAILED, std::string("hipStreamCreate: ") + hipGetErrorString(e));
        return;
    }
    // resident weights may take 85% of what is free now unless RNB_HIP_RESIDENT_BUDGET_MB says otherwise
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) s->resident_budget = free_b / 100 * 85;
    if (const char *env = std::getenv("RNB_HIP_RESIDENT_BUDGET_MB")) s->resident_budget = std::strtoull(env, nullptr, 10) << 20;
    g_state = s;
    g_open_status = 0;
    state = s;
}

}  // namespace rnb
