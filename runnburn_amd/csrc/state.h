// Process-global device state of the HIP backend: one device, one stream, grow-only scratch,
// a pinned bounce buffer and the resident-weight table.  Mirrors the shape of the reference's
// CudaState (crates/rnb-backend/cuda/src/runtime/state/{init.rs,buffers.rs,q4k_cache.rs}).
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "residency.h"

namespace rnb {

void set_last_error(const std::string &msg);
const char *last_error_cstr();

// Grow-only device allocation (reference: compute_*_ptr slots, state/buffers.rs:68-310).  Growing replaces the
// allocation; the old one is freed at once unless a stream capture has ever been seen on the library stream, in
// which case an instantiated graph may still hold its address and it is kept until the process ends (`retired`).
// While the stream is capturing, growth is refused: an allocation has no place inside a graph.
struct DeviceBuf {
    void *ptr = nullptr;
    size_t cap = 0;
    // hipErrorStreamCaptureUnsupported when the stream is capturing and the buffer would have to grow
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
    DeviceBuf moe_mid, moe_mid_qs, moe_mid_d, moe_mid_bsums, moe_slot_out, moe_tables;
    DeviceBuf gather_ids, gather_rows;  // embedding gather: token ids; the rows of a matrix that is not resident
    PinnedBuf bounce_in, bounce_out;
    TableSlot table_ring[kTableRing];  // MoE routing tables too large for a kernel argument
    int table_ring_next = 0;

    std::unique_ptr<DeviceAllocator> allocator;
    std::unique_ptr<ResidentTable> table;  // resident weights: (host range) -> device copy, budget, eviction, admission
    // what the activation scratch currently holds (set by quantize_activations)
    uint32_t act_family = 0;  // 8 = 32-wide Q8, 12 = Q8_K
    size_t act_seq = 0, act_cols = 0;

    uint64_t h2d_bytes = 0, d2h_bytes = 0;  // activations, outputs, tables (weights are counted by the table)
    bool capture_seen = false;              // a stream capture was observed: scratch that is replaced is retired, not freed
    std::vector<void *> retired;

    // Device address of [ptr, ptr+len) through the resident table (residency.h): an exact resident match, a sub-range
    // of a pinned (prewarmed) parent, a fresh untouched upload that becomes resident, or an upload for this call only.
    // Returns an rnb_hip_status with the message set.
    int resident_ptr(const uint8_t *ptr, size_t len, const uint8_t **dev_out, bool pin = false);
    // the device copy of [ptr, ptr+len) if there is one already (no upload); false otherwise
    bool resident_peek(const uint8_t *ptr, size_t len, const uint8_t **dev_out);
    bool release(const uint8_t *ptr, size_t len);
    // true while the library stream is capturing into a graph (also remembers that a capture happened)
    bool capturing();
};

// Locks the global mutex and opens the device on first use.  On failure returns a status
// (RNB_HIP_NO_DEVICE / RNB_HIP_EXECUTION_FAILED) with the message set and `state` null.
struct Guard {
    std::unique_lock<std::mutex> lock;
    State *state = nullptr;
    int status = 0;
    Guard();
    ~Guard();  // frees the weight uploads that were made for this call only (after the stream has drained)
};

}  // namespace rnb
