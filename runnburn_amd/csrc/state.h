// Process-global device state of the HIP backend: one device, one stream, grow-only scratch,
// a pinned bounce buffer and the resident-weight table.  Mirrors the shape of the reference's
// CudaState (crates/rnb-backend/cuda/src/runtime/state/{init.rs,buffers.rs,q4k_cache.rs}).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <string>

namespace rnb {

void set_last_error(const std::string &msg);
const char *last_error_cstr();

// Grow-only device allocation (reference: compute_*_ptr slots, state/buffers.rs:68-310).
struct DeviceBuf {
    void *ptr = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes);
    template <typename T>
    T *as() const { return static_cast<T *>(ptr); }
};

struct PinnedBuf {
    void *ptr = nullptr;
    size_t cap = 0;
    hipError_t reserve(size_t bytes);
    template <typename T>
    T *as() const { return static_cast<T *>(ptr); }
};

struct Resident {
    size_t len = 0;
    void *dev = nullptr;
    uint64_t fingerprint = 0;
    uint64_t epoch = 0;   // last use, for least-recently-used eviction
    bool pinned = false;  // prewarmed: never evicted, and the only kind a sub-range may resolve to
};

struct TableSlot {
    PinnedBuf host;
    hipEvent_t event = nullptr;  // recorded after the slot's upload was enqueued
};

struct State {
    static constexpr int kTableRing = 8;
    int device = 0;
    hipStream_t stream = nullptr;
    std::string device_name;

    // scratch slots
    DeviceBuf x_f32;      // staged f32 activations
    DeviceBuf act_qs;     // quantised activations: int8
    DeviceBuf act_d;      // per-block scales
    DeviceBuf act_bsums;  // per-16 sums (Q8_K)
    DeviceBuf argmax_scratch;             // 257 values then 257 indices
    DeviceBuf ffn_gate, ffn_up, ffn_mid;  // dense FFN intermediates, f32 [seq][n_ff]
    DeviceBuf act_digits; // per-32 sums as two int8 digits (Q8_K, only filled for GEMM-sized batches)
    bool act_has_digits = false;
    DeviceBuf out_f32;    // staged outputs
    DeviceBuf gemm_slices;  // per-slice outputs of a GEMM whose K range was cut to fill the chip
    DeviceBuf moe_mid, moe_mid_qs, moe_mid_d, moe_mid_bsums, moe_mid_digits, moe_slot_out, moe_tables;
    PinnedBuf bounce_in, bounce_out;
    TableSlot table_ring[kTableRing];  // MoE routing tables too large for a kernel argument
    int table_ring_next = 0;

    std::map<uintptr_t, Resident> residents;  // keyed by host base address
    // what the activation scratch currently holds (set by quantize_activations)
    uint32_t act_family = 0;  // 8 = 32-wide Q8, 12 = Q8_K
    size_t act_seq = 0, act_cols = 0;

    uint64_t resident_bytes = 0;
    uint64_t resident_budget = 0;  // bytes of unpinned + pinned residents before unpinned ones are evicted
    uint64_t epoch = 0;
    uint64_t h2d_bytes = 0, d2h_bytes = 0;

    // Returns the device address of [ptr, ptr+len): an exact resident match (same address, length
    // and fingerprint), a sub-range of a pinned (prewarmed) parent, or a fresh untouched upload
    // that becomes resident.  `pin` marks the entry as prewarmed.
    hipError_t resident_ptr(const uint8_t *ptr, size_t len, const uint8_t **dev_out, bool pin = false);
    void evict_unpinned_until(uint64_t need);
    bool release(const uint8_t *ptr, size_t len);
};

// Locks the global mutex and opens the device on first use.  On failure returns a status
// (RNB_HIP_NO_DEVICE / RNB_HIP_EXECUTION_FAILED) with the message set and `state` null.
struct Guard {
    std::unique_lock<std::mutex> lock;
    State *state = nullptr;
    int status = 0;
    Guard();
};

}  // namespace rnb
