// Device state: lazy open, scratch, pinned bounce buffers, resident weights.
#include "state.h"

#include <cstdlib>
#include <cstring>

#include "../../include/rnb_hip.h"
#include "kernels.h"

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

namespace {
thread_local std::string t_launch_failure;
}

bool allow_dynamic_lds(const void *kernel, size_t bytes, bool *done, const char *kernel_name) {
    if (*done) return true;
    const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes));
    if (e != hipSuccess) {
        (void)hipGetLastError();
        t_launch_failure = std::string(kernel_name) + ": hipFuncSetAttribute(max dynamic LDS = " + std::to_string(bytes) +
                           "): " + hipGetErrorString(e);
        return false;
    }
    *done = true;
    return true;
}

std::string take_launch_failure() {
    std::string out;
    out.swap(t_launch_failure);
    return out;
}

void set_last_error(const std::string &msg) { t_last_error = msg; }
const char *last_error_cstr() { return t_last_error.c_str(); }

hipError_t DeviceBuf::reserve(size_t bytes) {
    if (bytes <= cap) return hipSuccess;
    State *s = g_state;
    if (s != nullptr && s->capturing()) return hipErrorStreamCaptureUnsupported;
    if (ptr) {
        if (s != nullptr && s->capture_seen) {
            s->retired.push_back(ptr);  // a graph instantiated earlier may replay with this address
        } else {
            hipError_t e = hipFree(ptr);
            if (e != hipSuccess) {
                ptr = nullptr;
                cap = 0;
                return e;
            }
        }
        ptr = nullptr;
        cap = 0;
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

bool State::capturing() {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    if (st != hipStreamCaptureStatusNone) capture_seen = true;
    return st != hipStreamCaptureStatusNone;
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

namespace {
// hipMalloc / hipFree / blocking upload on the state's stream, for the resident table
class HipAllocator final : public DeviceAllocator {
  public:
    explicit HipAllocator(State *s) : s_(s) {}
    int alloc(size_t bytes, void **out, std::string *err) override {
        hipError_t e = hipMalloc(out, round_up(bytes, 256) + 256);
        if (e == hipSuccess) return 0;
        (void)hipGetLastError();
        *err = std::string("hipMalloc of ") + std::to_string(bytes) + " bytes: " + hipGetErrorString(e);
        return e == hipErrorOutOfMemory ? 1 : 2;
    }
    int free(void *ptr, std::string *err) override {
        // kernels of earlier calls may still read the range
        hipError_t e = hipStreamSynchronize(s_->stream);
        if (e == hipSuccess) e = hipFree(ptr);
        if (e == hipSuccess) return 0;
        *err = std::string("hipFree: ") + hipGetErrorString(e);
        return 2;
    }
    int upload(void *dst, const void *src, size_t bytes, std::string *err) override {
        hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, s_->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(s_->stream);
        if (e == hipSuccess) return 0;
        *err = std::string("weight upload: ") + hipGetErrorString(e);
        return 2;
    }

  private:
    State *s_;
};
}  // namespace

int State::resident_ptr(const uint8_t *ptr, size_t len, const uint8_t **dev_out, bool pin) {
    if (capturing()) {
        set_last_error("host-pointer weights cannot be resolved while the library stream is capturing");
        return RNB_HIP_INVALID_REQUEST;
    }
    std::string err;
    const int rc = table->resolve(ptr, len, fingerprint(ptr, len), pin, dev_out, &err);
    if (rc == 0) return RNB_HIP_OK;
    set_last_error(err);
    return RNB_HIP_EXECUTION_FAILED;
}

bool State::resident_peek(const uint8_t *ptr, size_t len, const uint8_t **dev_out) {
    return table->peek(ptr, len, fingerprint(ptr, len), dev_out);
}

bool State::release(const uint8_t *ptr, size_t len) {
    std::string err;
    return table->release(ptr, len, &err);
}

Guard::~Guard() {
    if (state != nullptr && state->table->has_call_temps()) {
        (void)hipStreamSynchronize(state->stream);
        std::string err;
        (void)state->table->end_call(&err);
    }
}

Guard::Guard() : lock(g_mutex) {
    if (g_state) {
        state = g_state;
        hipError_t e = hipSetDevice(state->device);
        if (e != hipSuccess) {
            set_last_error(std::string("hipSetDevice: ") + hipGetErrorString(e));
            status = RNB_HIP_EXECUTION_FAILED;
            state = nullptr;
            return;
        }
        // every entry looks at the stream once: a capture whose calls all fit the existing scratch never reaches the
        // check in DeviceBuf::reserve, and a graph instantiated from it still points into that scratch
        (void)state->capturing();
        state->table->begin_call();
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
    s->allocator.reset(new HipAllocator(s));
    s->table.reset(new ResidentTable(s->allocator.get()));
    // resident weights may take 85% of what is free now unless RNB_HIP_RESIDENT_BUDGET_MB says otherwise
    size_t free_b = 0, total_b = 0;
    if (hipMemGetInfo(&free_b, &total_b) == hipSuccess) s->table->set_budget(free_b / 100 * 85);
    if (const char *env = std::getenv("RNB_HIP_RESIDENT_BUDGET_MB")) s->table->set_budget(std::strtoull(env, nullptr, 10) << 20);
    g_state = s;
    g_open_status = 0;
    state = s;
    s->table->begin_call();
}

}  // namespace rnb
