// extern "C" surface of the HIP backend (include/rnb_hip.h): validation with the reference's
// messages, staging through pinned bounce buffers, kernel sequencing on the single stream.
#include "../../include/rnb_hip.h"

#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "kernels.h"
#include "state.h"

using namespace rnb;

namespace {

struct QuantInfo {
    const char *label;
    size_t elems;
    size_t bytes;
};

bool quant_info(uint32_t quant, QuantInfo *qi) {
    switch (quant) {
    case kQ4_0: *qi = {"Q4_0", 32, kQ4_0Bytes}; return true;
    case kQ4_1: *qi = {"Q4_1", 32, kQ4_1Bytes}; return true;
    case kQ5_0: *qi = {"Q5_0", 32, kQ5_0Bytes}; return true;
    case kQ5_1: *qi = {"Q5_1", 32, kQ5_1Bytes}; return true;
    case kQ8_1: *qi = {"Q8_1", 32, kQ8_1Bytes}; return true;
    case kQ8_0: *qi = {"Q8_0", 32, kQ8_0Bytes}; return true;
    case kQ2K: *qi = {"Q2_K", 256, kQ2KBytes}; return true;
    case kQ3K: *qi = {"Q3_K", 256, kQ3KBytes}; return true;
    case kQ4K: *qi = {"Q4_K", 256, kQ4KBytes}; return true;
    case kQ5K: *qi = {"Q5_K", 256, kQ5KBytes}; return true;
    case kQ6K: *qi = {"Q6_K", 256, kQ6KBytes}; return true;
    case kIQ2XXS: *qi = {"IQ2_XXS", 256, kIQ2XXSBytes}; return true;
    case kIQ2S: *qi = {"IQ2_S", 256, kIQ2SBytes}; return true;
    case kIQ3XXS: *qi = {"IQ3_XXS", 256, kIQ3XXSBytes}; return true;
    case kIQ4XS: *qi = {"IQ4_XS", 256, kIQ4XSBytes}; return true;
    default: return false;
    }
}

// the 32-element formats take 32-wide Q8 activations, the K-quants 256-wide Q8_K
bool is_block32(uint32_t quant) {
    return quant == kQ8_0 || quant == kQ4_0 || quant == kQ4_1 || quant == kQ5_0 || quant == kQ5_1 || quant == kQ8_1;
}

int fail(int status, const std::string &msg) {
    set_last_error(msg);
    return status;
}

int hip_fail(const char *what, hipError_t e) {
    return fail(RNB_HIP_EXECUTION_FAILED, std::string(what) + ": " + hipGetErrorString(e));
}

#define HIP_TRY(expr)                                      \
    do {                                                   \
        hipError_t _e = (expr);                            \
        if (_e != hipSuccess) return hip_fail(#expr, _e);  \
    } while (0)

// Minimum tokens for which the MFMA GEMMs replace the vector-unit kernels.  Below it a batch runs the GEMV kernels that
// keep two to four tokens in registers per pass over the matrix (a pass per group of four tokens: time grows with every
// token), while a GEMM's 32-token tile costs the same from 1 to 32.  Measured crossovers (us, GEMV groups vs GEMM):
// Q4_K 14336 x 4096 (33 MB) 4 tokens 14.7 vs 17.7, 5 tokens 18.2 vs 17.5; Q5_K likewise 16.1 vs 20.3, 20.8 vs 20.0; Q6_K
// 14336 x 4096 6 tokens 23.2 vs 25.6, 7 tokens 25.9 vs 25.5 (4096 x 14336: 27.7 vs 28.6, 31.0 vs 28.7); Q2_K / Q3_K 6 tokens
// 18.1 / 21.9 vs 21.0 / 23.1, 7 tokens 22.8 / 24.9 vs 21.0 / 23.0; Q8_0 4096 x 4096 6 tokens 13.8 vs 17.1, 7 tokens 17.0
// vs 17.3 (14336 x 4096: 28.7 vs 33.2, 32.9 vs 33.1); Q4_0 14336 x 4096 8 tokens 22.5 vs 25.8, 12 tokens 29.7 vs 26.0.
// Matrices that take the chunked GEMV (rows of 9 - 16 super-blocks, 48 MB and more): Q6_K 128256 x 4096 4 tokens 107 vs
// 122, 5 tokens 163 vs 121; Q4_K / Q5_K 65536 x 4096 3 tokens 43.6 / 49.6, 4 tokens 54.5 / 60.1 vs 42.0 / 46.2.  Small
// ones: Q4_K 4096 x 4096 (9 MB) 6 tokens 11.6 vs 13.0 (the staged multi-token kernel; GEMM 11.9 from 8), 7 tokens 13.7;
// Q6_K 4096 x 4096 (14 MB) 8 tokens 14.9 vs 16.2, 12 tokens 19.7 vs 16.3; Q4_K 2048 x 2048 (2.4 MB) 16 tokens 9.0 vs 10.0.
constexpr size_t kGemmTinyBytes = size_t(4) << 20, kGemmSmallBytes = size_t(16) << 20, kGemmChunkBytes = size_t(48) << 20;
size_t gemm_min_seq(uint32_t quant, size_t rows, size_t cols) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return 8;
    const size_t per_row = cols / qi.elems, bytes = rows * per_row * qi.bytes;
    if (bytes < kGemmTinyBytes) return 17;
    const bool chunked = bytes >= kGemmChunkBytes && qi.elems == 256 && per_row > 8 && per_row <= 16;
    switch (quant) {
    case kQ4K:
    case kQ5K: return chunked ? 4 : (bytes < kGemmSmallBytes ? 7 : 5);
    case kQ6K: return chunked ? 5 : (bytes < kGemmSmallBytes ? 9 : 7);
    case kQ2K:
    case kQ3K: return chunked ? 4 : 7;
    case kQ8_0:
    case kQ8_1: return 7;
    default: return 9;  // Q4_0, Q4_1, Q5_0, Q5_1
    }
}
// The Q8_K quantiser adds the per-32 sums as two digits (the Q4_K / Q5_K GEMMs' mins term) from this many tokens on.
constexpr size_t kDigitsMinSeq = 4;  // the smallest value gemm_min_seq returns
// Minimum tokens for which the importance-quant formats take their matrix-core GEMM instead of the GEMV that dots a
// decoded block against up to four tokens (14336 x 4096, 4 tokens: 20.8 - 22.9 us against 21.8 - 25.8; 5 tokens: 29 - 35
// against 21.5 - 25.7).
constexpr size_t kIqGemmMinSeq = 5;
// Minimum tokens for which the grouped MoE GEMMs on the matrix cores are considered.
constexpr size_t kMoeMfmaMinTokens = 16;
// Minimum number of 256 x 64 tiles for which the Q4_K ping-pong GEMM replaces the smaller-tile kernel.
constexpr uint64_t kGemmBigTilesMin = 32;

// After enqueuing kernels: a launcher that could not configure its kernel (and therefore did not launch) left the
// reason; otherwise whatever the runtime recorded.
int check_launches() {
    const std::string pending = take_launch_failure();
    if (!pending.empty()) return fail(RNB_HIP_EXECUTION_FAILED, pending);
    HIP_TRY(hipGetLastError());
    return RNB_HIP_OK;
}

// Growing a scratch buffer: refused with a message while the library stream is capturing into a graph.
int reserve_fail(hipError_t e) {
    if (e == hipErrorStreamCaptureUnsupported)
        return fail(RNB_HIP_INVALID_REQUEST,
                    "scratch would have to grow while the library stream is capturing: run this shape once before the "
                    "capture, or use rnb_hip_gemv_dev_noalloc");
    return hip_fail("scratch allocation", e);
}
#define RESERVE_TRY(buf, bytes)                                \
    do {                                                       \
        hipError_t _e = (buf).reserve(bytes);                  \
        if (_e != hipSuccess) return reserve_fail(_e);         \
    } while (0)

// A fixed span of device memory that a call carves its scratch from instead of the state's grow-only buffers: the
// entry point that must not allocate passes one over its static array.
struct Arena {
    uint8_t *base = nullptr;
    size_t cap = 0, used = 0;
    const char *who = "";
};

// `bytes` of scratch: from the arena when there is one (256-byte aligned pieces, an error when it is full), else the
// state's buffer `slot`, grown if needed.
int take_scratch(DeviceBuf &slot, Arena *arena, size_t bytes, void **out) {
    if (arena) {
        const size_t at = (arena->used + 255) / 256 * 256;
        if (at + bytes > arena->cap)
            return fail(RNB_HIP_INVALID_REQUEST, std::string(arena->who) + " needs more than the " +
                                                     std::to_string(arena->cap) + " bytes of static scratch (" +
                                                     std::to_string(at + bytes) + " so far)");
        *out = arena->base + at;
        arena->used = at + bytes;
        return RNB_HIP_OK;
    }
    RESERVE_TRY(slot, bytes);
    *out = slot.ptr;
    return RNB_HIP_OK;
}

#define SCRATCH_TRY(slot, bytes, type, var)                                                         \
    type *var = nullptr;                                                                            \
    do {                                                                                            \
        void *_p = nullptr;                                                                         \
        if (int _st = take_scratch(slot, arena, bytes, &_p); _st != RNB_HIP_OK) return _st;         \
        var = static_cast<type *>(_p);                                                              \
    } while (0)

// Quantise seq*cols f32 values on the device into activation scratch (the state's, which then remembers what it holds,
// or the arena's).
// words that the quantiser's launch copies into device memory on the side (the MoE routing tables of a batch)
struct WordCopy {
    const uint32_t *src = nullptr;  // device memory or pinned host memory
    uint32_t *dst = nullptr;
    uint32_t n_words = 0;
};

int quantize_activations(State &s, uint32_t quant, const float *x_dev, size_t seq, size_t cols, ActView *view,
                         Arena *arena = nullptr, const WordCopy *copy = nullptr) {
    const size_t n = seq * cols;
    SCRATCH_TRY(s.act_qs, n, int8_t, qs);
    bool has_digits = false;
    if (is_block32(quant)) {
        SCRATCH_TRY(s.act_d, n / 32 * sizeof(float), float, d);
        launch_quantize_q8(x_dev, n / 32, qs, d, s.stream);
        *view = {qs, d, nullptr};
    } else {
        SCRATCH_TRY(s.act_d, n / 256 * sizeof(float), float, d);
        SCRATCH_TRY(s.act_bsums, n / 256 * 16 * sizeof(int16_t), int16_t, bsums);
        has_digits = seq >= kDigitsMinSeq;
        uint8_t *digits = nullptr;
        if (has_digits) {
            SCRATCH_TRY(s.act_digits, n / 256 * 16, uint8_t, dg);
            digits = dg;
        }
        if (copy != nullptr && copy->n_words != 0)
            launch_quantize_q8k_copy(x_dev, n / 256, qs, d, bsums, digits, copy->src, copy->n_words, copy->dst, s.stream);
        else
            launch_quantize_q8k(x_dev, n / 256, qs, d, bsums, digits, s.stream);
        *view = {qs, d, bsums, digits};
    }
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    if (!arena) {
        s.act_has_digits = has_digits;
        s.act_family = is_block32(quant) ? kQ8_0 : kQ4K;
        s.act_seq = seq;
        s.act_cols = cols;
    }
    return RNB_HIP_OK;
}

// what the state's activation scratch holds, as the kernels take it
ActView state_act_view(const State &s, uint32_t quant) {
    const bool b32 = is_block32(quant);
    return ActView{s.act_qs.as<int8_t>(), s.act_d.as<float>(), b32 ? nullptr : s.act_bsums.as<int16_t>(),
                   !b32 && s.act_has_digits ? s.act_digits.as<uint8_t>() : nullptr};
}

int run_matmul_quantized_dev(State &s, uint32_t quant, const uint8_t *w_dev, size_t rows, size_t cols, size_t seq,
                             float *out_dev, const ActView &act, Arena *arena = nullptr);

int run_matmul_dev(State &s, uint32_t quant, const uint8_t *w_dev, size_t rows, size_t cols, const float *x_dev,
                   size_t seq, float *out_dev, Arena *arena = nullptr) {
    // one token against rows of at most 64 super-blocks: the GEMV's workgroups quantise the token themselves
    if (seq == 1 && !is_block32(quant) && gemv_kquant_f32_supported(quant, static_cast<uint32_t>(cols / 256), x_dev, w_dev) &&
        gemv_kquant_f32_pays(quant, static_cast<uint32_t>(rows), static_cast<uint32_t>(cols / 256))) {
        launch_gemv_kquant_f32(w_dev, quant, x_dev, out_dev, static_cast<uint32_t>(rows), static_cast<uint32_t>(cols / 256),
                               1, s.stream);
        if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
        return RNB_HIP_OK;
    }
    if (seq == 1 && is_block32(quant) && gemv_block32_f32_supported(static_cast<uint32_t>(rows), static_cast<uint32_t>(cols / 32), x_dev)) {
        launch_gemv_block32_f32(w_dev, quant, x_dev, out_dev, static_cast<uint32_t>(rows), static_cast<uint32_t>(cols / 32), 1,
                                s.stream);
        if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
        return RNB_HIP_OK;
    }
    ActView act;
    int st = quantize_activations(s, quant, x_dev, seq, cols, &act, arena);
    if (st != RNB_HIP_OK) return st;
    return run_matmul_quantized_dev(s, quant, w_dev, rows, cols, seq, out_dev, act, arena);
}

int run_matmul_quantized_dev(State &s, uint32_t quant, const uint8_t *w_dev, size_t rows, size_t cols, size_t seq,
                             float *out_dev, const ActView &act, Arena *arena) {
    const uint32_t r = static_cast<uint32_t>(rows), q = static_cast<uint32_t>(seq);
    const uint32_t nb = static_cast<uint32_t>(cols / 256);
    const size_t min_gemm_seq = gemm_min_seq(quant, rows, cols);
    // workspace of the GEMMs that cut K into slices on small grids (null: none needed)
    auto slice_floats = [&](size_t floats, float **ws) -> int {
        *ws = nullptr;
        if (floats == 0) return RNB_HIP_OK;
        SCRATCH_TRY(s.gemm_slices, floats * sizeof(float), float, p);
        *ws = p;
        return RNB_HIP_OK;
    };
    auto slice_ws = [&](uint32_t k_steps, float **ws) -> int {
        return slice_floats(gemm_blocks_slice_floats(quant, r, k_steps, q), ws);
    };
    float *ws = nullptr;
    if (is_iq_quant(quant)) {
        // importance quants: the matrix-core GEMM for batches, else the GEMV (a pass per group of up to four tokens)
        if (seq >= kIqGemmMinSeq) {
            if (int st = slice_floats(gemm_iq_slice_floats(r, nb, q), &ws); st != RNB_HIP_OK) return st;
            launch_gemm_iq_mfma(w_dev, quant, act, out_dev, ws, r, nb, q, s.stream);
        } else {
            launch_gemv_iq(w_dev, quant, act, out_dev, r, nb, q, s.stream);
        }
    } else if (quant == kQ4K) {
        // the GEMM fills LDS with 16-byte loads: weights at other alignments take the vector kernels
        // gemm_q4k.hip's 256-row x 64-token workgroups (K cut into slices up to 128 tiles) win from 32 tiles on when the
        // token tile is more than half full; below that the 128 x 32 kernel of gemm_blocks.hip, sliced as well, does
        // (4096 x 4096 x 64 tokens, 16 tiles: 11.7 vs 14.8 us; 14336 x 4096 x 32: 18.1 vs 20.6 us; 14336 x 4096 x 64,
        // 56 tiles: 28.3 vs 24.0 us; 4096 x 14336 x 128, 32 tiles: 43.2 vs 32.9 us)
        const uint64_t big_tiles = static_cast<uint64_t>((rows + 255) / 256) * ((seq + 63) / 64);
        if (seq >= min_gemm_seq && act.digits != nullptr && (big_tiles < kGemmBigTilesMin || seq <= 32)) {
            if (int st = slice_ws(nb, &ws); st != RNB_HIP_OK) return st;
            launch_gemm_q4k_small(w_dev, act, out_dev, ws, r, nb, q, s.stream);
        } else if (seq >= min_gemm_seq && act.digits != nullptr && reinterpret_cast<uintptr_t>(w_dev) % 16 == 0) {
            if (int st = slice_floats(gemm_q4k_slice_floats(r, nb, q), &ws); st != RNB_HIP_OK) return st;
            launch_gemm_q4k_mfma(w_dev, act, out_dev, ws, r, nb, q, s.stream);
        } else {
            launch_gemv_q4k(w_dev, act, out_dev, r, nb, q, s.stream);
        }
    } else if (quant == kQ2K || quant == kQ3K) {
        if (seq >= min_gemm_seq) {
            if (int st = slice_ws(nb, &ws); st != RNB_HIP_OK) return st;
            launch_gemm_q23k_mfma(w_dev, quant, act, out_dev, ws, r, nb, q, s.stream);
        } else {
            launch_gemv_q2k_q3k(w_dev, quant, act, out_dev, r, nb, q, s.stream);
        }
    } else if (quant == kQ5K) {
        if (seq >= min_gemm_seq && act.digits != nullptr) {
            if (int st = slice_ws(nb, &ws); st != RNB_HIP_OK) return st;
            launch_gemm_q5k_mfma(w_dev, act, out_dev, ws, r, nb, q, s.stream);
        } else {
            launch_gemv_q5k(w_dev, act, out_dev, r, nb, q, s.stream);
        }
    } else if (quant == kQ6K) {
        if (seq >= min_gemm_seq) {
            if (int st = slice_ws(nb, &ws); st != RNB_HIP_OK) return st;
            launch_gemm_q6k_mfma(w_dev, act, out_dev, ws, r, nb, q, s.stream);
        } else {
            launch_gemv_q6k(w_dev, act, out_dev, r, nb, q, s.stream);
        }
    } else if (seq >= min_gemm_seq && gemm_q8_mfma_supported(quant, static_cast<uint32_t>(cols / 32))) {
        const uint32_t nb32 = static_cast<uint32_t>(cols / 32);
        if (int st = slice_ws((nb32 + 7) / 8, &ws); st != RNB_HIP_OK) return st;
        launch_gemm_q8_mfma(w_dev, quant, act, out_dev, ws, r, nb32, q, s.stream);
    } else {
        launch_gemv_block32(w_dev, quant, act, out_dev, r, static_cast<uint32_t>(cols / 32), q, s.stream);
    }
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    return RNB_HIP_OK;
}

// Validation order and messages: crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:183-206 (gemv),
// :340-358 (gemv_into), :2283-2307 (batch), :1983-2009 / :2030-2057 (Q8_0).
int validate_matmul(const QuantInfo &qi, size_t w_len, size_t rows, size_t cols, size_t x_len, size_t out_len,
                    bool batch, size_t *seq_out) {
    const std::string label = qi.label;
    if (cols == 0 || cols % qi.elems != 0)
        return fail(RNB_HIP_INVALID_REQUEST,
                    label + " cols must be divisible by " + std::to_string(qi.elems) + ", got " + std::to_string(cols));
    size_t seq = 1;
    if (batch) {
        if (x_len % cols != 0)
            return fail(RNB_HIP_INVALID_REQUEST, label + " batch input length " + std::to_string(x_len) +
                                                     " is not divisible by cols " + std::to_string(cols));
        seq = x_len / cols;
    }
    const size_t row_bytes = cols / qi.elems * qi.bytes;
    if (w_len != rows * row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, label + " weight byte mismatch: got " + std::to_string(w_len) +
                                                 ", expected " + std::to_string(rows * row_bytes));
    if (!batch && x_len != cols && out_len >= rows)
        return fail(RNB_HIP_INVALID_REQUEST, label + " input length mismatch: got " + std::to_string(x_len) +
                                                 ", expected " + std::to_string(cols));
    if (!batch && (x_len != cols || out_len < rows))
        return fail(RNB_HIP_INVALID_REQUEST, label + " shape mismatch: input=" + std::to_string(x_len) +
                                                 " output=" + std::to_string(out_len) + " expected input=" +
                                                 std::to_string(cols) + " output>=" + std::to_string(rows));
    if (batch && out_len < seq * rows)
        return fail(RNB_HIP_INVALID_REQUEST, label + " shape mismatch: input=" + std::to_string(x_len) +
                                                 " output=" + std::to_string(out_len) + " expected output>=" +
                                                 std::to_string(seq * rows));
    if (rows > 0x7fffffffu || cols > 0x7fffffffu || seq > 65535u)  // the kernels index with 32 bits
        return fail(RNB_HIP_INVALID_REQUEST, label + " shape out of range: rows=" + std::to_string(rows) + " cols=" +
                                                 std::to_string(cols) + " seq_len=" + std::to_string(seq));
    *seq_out = seq;
    return RNB_HIP_OK;
}

int matmul_host(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                size_t x_len, float *out, size_t out_len, bool batch) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    size_t seq = 0;
    int st = validate_matmul(qi, w_len, rows, cols, x_len, out_len, batch, &seq);
    if (st != RNB_HIP_OK) return st;
    if ((w_len && !w) || (x_len && !x) || (out_len && !out))
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " null pointer argument");
    if (rows == 0 || seq == 0) return RNB_HIP_OK;

    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *w_dev = nullptr;
    if (int rs = s.resident_ptr(w, w_len, &w_dev); rs != RNB_HIP_OK) return rs;
    const size_t in_bytes = seq * cols * sizeof(float), out_bytes = seq * rows * sizeof(float);
    RESERVE_TRY(s.bounce_in, in_bytes);
    RESERVE_TRY(s.bounce_out, out_bytes);
    HIP_TRY(s.x_f32.reserve(in_bytes));
    HIP_TRY(s.out_f32.reserve(out_bytes));
    std::memcpy(s.bounce_in.ptr, x, in_bytes);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, in_bytes, hipMemcpyHostToDevice, s.stream));
    s.h2d_bytes += in_bytes;
    st = run_matmul_dev(s, quant, w_dev, rows, cols, s.x_f32.as<float>(), seq, s.out_f32.as<float>());
    if (st != RNB_HIP_OK) return st;
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, s.out_f32.ptr, out_bytes, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += out_bytes;
    std::memcpy(out, s.bounce_out.ptr, out_bytes);
    return RNB_HIP_OK;
}

// One token that already lives on the device (a norm's output, say) against host-resident weights, result to the host:
// q4k_gemv_with_device_input / q6k_gemv_with_device_input, crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:242-330
// (checks and texts: cols, weight bytes, output size, in that order).
int matmul_device_input(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x_dev,
                        float *out, size_t out_len) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    const std::string label = qi.label;
    if (cols % qi.elems != 0)
        return fail(RNB_HIP_INVALID_REQUEST,
                    label + " cols must be divisible by " + std::to_string(qi.elems) + ", got " + std::to_string(cols));
    const size_t row_bytes = cols / qi.elems * qi.bytes;
    if (w_len != rows * row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, label + " weight byte mismatch: got " + std::to_string(w_len) + ", expected " +
                                                 std::to_string(rows * row_bytes));
    if (out_len < rows)
        return fail(RNB_HIP_INVALID_REQUEST,
                    label + " output too small: got " + std::to_string(out_len) + ", expected >= " + std::to_string(rows));
    if ((w_len && !w) || (out_len && !out)) return fail(RNB_HIP_INVALID_REQUEST, label + " null pointer argument");
    if (rows == 0) return RNB_HIP_OK;
    if (cols == 0 || !x_dev || (reinterpret_cast<uintptr_t>(x_dev) & 15u))
        return fail(RNB_HIP_INVALID_REQUEST, label + " device input must be a 16-byte aligned device pointer to cols floats");
    if (rows > 0x7fffffffu || cols > 0x7fffffffu)
        return fail(RNB_HIP_INVALID_REQUEST, label + " shape out of range: rows=" + std::to_string(rows) + " cols=" + std::to_string(cols));
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *w_dev = nullptr;
    if (int rs = s.resident_ptr(w, w_len, &w_dev); rs != RNB_HIP_OK) return rs;
    const size_t out_bytes = rows * sizeof(float);
    RESERVE_TRY(s.bounce_out, out_bytes);
    HIP_TRY(s.out_f32.reserve(out_bytes));
    if (int st = run_matmul_dev(s, quant, w_dev, rows, cols, x_dev, 1, s.out_f32.as<float>()); st != RNB_HIP_OK) return st;
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, s.out_f32.ptr, out_bytes, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += out_bytes;
    std::memcpy(out, s.bounce_out.ptr, out_bytes);
    return RNB_HIP_OK;
}

// ---- dense gated FFN --------------------------------------------------------------------------
// out[s] = W_down . Q(act(W_gate . Q8_K(x_s)) * (W_up . Q8_K(x_s))), act = SiLU or GELU: the composition the reference
// runs per token on the CPU (gate/up GEMV, fused_silu_mul / fused_gelu_mul, down GEMV).  Gate and up are Q4_K; down is Q4_K, Q5_K, Q6_K, Q8_0 or Q5_1.

// Validation order and messages: crates/rnb-backend/cuda/src/runtime/dense.rs:1712-1765.
int validate_dense_ffn(size_t gate_len, size_t up_len, size_t down_len, uint32_t down_quant, size_t n_ff, size_t n_embd,
                       size_t seq, size_t x_len, bool batch_entry, bool gelu = false) {
    const std::string name = gelu ? "dense GELU FFN" : "dense SiLU FFN";
    if (batch_entry && seq <= 1)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch requires seq_len > 1, got " + std::to_string(seq));
    if (x_len != seq * n_embd)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch input length mismatch: got " + std::to_string(x_len) +
                                                 ", expected " + std::to_string(seq * n_embd));
    const size_t down_block = (down_quant == 7 || down_quant == 8) ? 32 : 256;
    if (n_embd % 256 != 0 || n_ff % down_block != 0)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch dims must align to gate/down blocks, got n_ff=" +
                                                 std::to_string(n_ff) + " down_block=" + std::to_string(down_block) +
                                                 " n_embd=" + std::to_string(n_embd));
    size_t down_row_bytes = 0;
    switch (down_quant) {
        case 7: down_row_bytes = n_ff / 32 * 24; break;
        case 8: down_row_bytes = n_ff / 32 * 34; break;
        case 12: down_row_bytes = n_ff / 256 * 144; break;
        case 13: down_row_bytes = n_ff / 256 * 176; break;
        case 14: down_row_bytes = n_ff / 256 * 210; break;
        default:
            return fail(RNB_HIP_INVALID_REQUEST,
                        "unsupported " + name + " batch down quant code " + std::to_string(down_quant));
    }
    const size_t gate_bytes = n_ff * (n_embd / 256) * 144;
    if (gate_len != gate_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch gate byte mismatch: got " + std::to_string(gate_len) +
                                                 ", expected " + std::to_string(gate_bytes));
    if (up_len != gate_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch up byte mismatch: got " + std::to_string(up_len) +
                                                 ", expected " + std::to_string(gate_bytes));
    if (down_len != n_embd * down_row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch down byte mismatch: got " + std::to_string(down_len) +
                                                 ", expected " + std::to_string(n_embd * down_row_bytes));
    if (n_ff > 0x7fffffffu || n_embd > 0x7fffffffu || seq > 65535u)
        return fail(RNB_HIP_INVALID_REQUEST, name + " shape out of range");
    return RNB_HIP_OK;
}

int run_dense_ffn_dev(State &s, const uint8_t *gate_dev, const uint8_t *up_dev, const uint8_t *down_dev,
                      uint32_t down_quant, size_t n_ff, size_t n_embd, size_t seq, const float *x_dev, float *out_dev,
                      bool gelu = false) {
    const size_t nb_in = n_embd / 256, mid_bytes = seq * n_ff * sizeof(float);
    RESERVE_TRY(s.ffn_mid, mid_bytes);
    const bool aligned = (reinterpret_cast<uintptr_t>(gate_dev) | reinterpret_cast<uintptr_t>(up_dev)) % 16 == 0;
    // the paired gate/up GEMV (a pass over both matrices per group of up to four tokens) against two GEMMs and the
    // gated quantiser, measured on 14336 x 4096 with a Q6_K down projection: 4 tokens 44.1 vs 47.6 us for the whole
    // layer, 6 tokens 56.1 vs 59.6, 7 tokens 62.3 vs 58.7 (11008 x 4096: 8 tokens 52.6 vs 55.1)
    const size_t pair_max = n_ff * nb_in * kQ4KBytes >= kGemmSmallBytes ? 7 : 9;
    const bool small = seq < pair_max && aligned && gemv_q4k_gate_up_supported(static_cast<uint32_t>(nb_in));
    ActView act;
    int st = RNB_HIP_OK;
    if (small && seq == 1 && reinterpret_cast<uintptr_t>(x_dev) % 16 == 0) {
        // one token: one launch quantises it (per workgroup, in LDS) and makes act(gate) * up; with more tokens the
        // repeated quantisation costs more than the launch it saves (measured)
        launch_gemv_q4k_gate_up_f32(gate_dev, up_dev, x_dev, s.ffn_mid.as<float>(), static_cast<uint32_t>(n_ff),
                                    static_cast<uint32_t>(nb_in), static_cast<uint32_t>(seq), gelu, s.stream);
        if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
        return run_matmul_dev(s, down_quant, down_dev, n_embd, n_ff, s.ffn_mid.as<float>(), seq, out_dev);
    }
    st = quantize_activations(s, kQ4K, x_dev, seq, n_embd, &act);
    if (st != RNB_HIP_OK) return st;
    if (small) {
        launch_gemv_q4k_gate_up(gate_dev, up_dev, act, s.ffn_mid.as<float>(), static_cast<uint32_t>(n_ff),
                                static_cast<uint32_t>(nb_in), static_cast<uint32_t>(seq), gelu, s.stream);
    } else {
        RESERVE_TRY(s.ffn_gate, mid_bytes);
        RESERVE_TRY(s.ffn_up, mid_bytes);
        st = run_matmul_quantized_dev(s, kQ4K, gate_dev, n_ff, n_embd, seq, s.ffn_gate.as<float>(), act);
        if (st != RNB_HIP_OK) return st;
        st = run_matmul_quantized_dev(s, kQ4K, up_dev, n_ff, n_embd, seq, s.ffn_up.as<float>(), act);
        if (st != RNB_HIP_OK) return st;
        if (!is_block32(down_quant)) {
            // K-quant down projection: act(gate) * up is quantised to Q8_K as it is made, no f32 intermediate in memory
            const size_t n = seq * n_ff;
            RESERVE_TRY(s.act_qs, n);
            RESERVE_TRY(s.act_d, n / 256 * sizeof(float));
            RESERVE_TRY(s.act_bsums, n / 256 * 16 * sizeof(int16_t));
            // the scratch is about to be overwritten: it describes nothing until the launch is known to have gone out
            s.act_seq = 0;
            const bool want_digits = seq >= kDigitsMinSeq;
            if (want_digits) RESERVE_TRY(s.act_digits, n / 256 * 16);
            launch_quantize_q8k_gated(s.ffn_gate.as<float>(), s.ffn_up.as<float>(), n / 256, gelu, s.act_qs.as<int8_t>(),
                                      s.act_d.as<float>(), s.act_bsums.as<int16_t>(),
                                      want_digits ? s.act_digits.as<uint8_t>() : nullptr, s.stream);
            if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
            s.act_has_digits = want_digits;
            s.act_family = kQ4K;
            s.act_seq = seq;
            s.act_cols = n_ff;
            return run_matmul_quantized_dev(s, down_quant, down_dev, n_embd, n_ff, seq, out_dev,
                                            state_act_view(s, down_quant));
        }
        launch_act_mul(s.ffn_gate.as<float>(), s.ffn_up.as<float>(), s.ffn_mid.as<float>(), seq * n_ff, gelu, s.stream);
    }
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    // the intermediate is re-quantised in the form the down projection's rows take, then the down matmul runs
    return run_matmul_dev(s, down_quant, down_dev, n_embd, n_ff, s.ffn_mid.as<float>(), seq, out_dev);
}

// ---- MoE ------------------------------------------------------------------------------------

struct MoeShape {
    size_t per_gate, per_down, n_expert, nb_in, nb_mid;
};

// Messages: crates/rnb-backend/cuda/src/runtime/helpers.rs:1570-1600 (selected-base shape) and
// :2747-2800 (full-layer token batch).
// The shared expert of a call (the extra slot of the reference's decode call, fanout.rs:804-812, id n_expert): present
// when all three tensors are given, each with one expert's length.
struct SharedLens {
    bool any = false, all = false;
    size_t gate = 0, up = 0, down = 0;
};

int validate_moe(size_t gate_len, size_t up_len, size_t down_len, const SharedLens &shared, const uint32_t *expert_ids,
                 const uint32_t *token_ids, size_t n_slots, size_t token_count, uint32_t down_quant, size_t n_ff,
                 size_t n_embd, size_t x_len, size_t out_len, MoeShape *shape) {
    if (x_len != token_count * n_embd)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer input length mismatch: got " + std::to_string(x_len) +
                                                 ", expected " + std::to_string(token_count * n_embd));
    if (n_embd == 0 || n_ff == 0 || n_embd % 256 != 0 || n_ff % 256 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer dims must be divisible by 256, got n_ff=" +
                                                 std::to_string(n_ff) + " n_embd=" + std::to_string(n_embd));
    for (size_t i = 0; i < n_slots; i++)
        if (token_ids[i] >= token_count)
            return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer token id out of range");
    size_t down_block;
    switch (down_quant) {
    case kQ4K: down_block = kQ4KBytes; break;
    case kQ5K: down_block = kQ5KBytes; break;
    case kQ6K: down_block = kQ6KBytes; break;
    default:
        return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported Qwen35 HIP down quant code " + std::to_string(down_quant));
    }
    MoeShape sh;
    sh.nb_in = n_embd / 256;
    sh.nb_mid = n_ff / 256;
    sh.per_gate = n_ff * sh.nb_in * kQ4KBytes;
    sh.per_down = n_embd * sh.nb_mid * down_block;
    if (gate_len % sh.per_gate != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 selected-base gate length is not expert-aligned: len=" +
                                                 std::to_string(gate_len) + " per_expert=" + std::to_string(sh.per_gate));
    sh.n_expert = gate_len / sh.per_gate;
    if (up_len != sh.n_expert * sh.per_gate)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 selected-base up length mismatch: len=" + std::to_string(up_len) +
                                                 " expected=" + std::to_string(sh.n_expert * sh.per_gate));
    if (down_len != sh.n_expert * sh.per_down)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 selected-base down length mismatch: len=" +
                                                 std::to_string(down_len) + " expected=" +
                                                 std::to_string(sh.n_expert * sh.per_down));
    if (shared.any && !shared.all)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 shared expert needs its gate, up and down tensors together");
    if (shared.all && (shared.gate != sh.per_gate || shared.up != sh.per_gate || shared.down != sh.per_down))
        return fail(RNB_HIP_INVALID_REQUEST,
                    "Qwen35 shared expert length mismatch: gate=" + std::to_string(shared.gate) + " up=" +
                        std::to_string(shared.up) + " down=" + std::to_string(shared.down) + " expected gate=up=" +
                        std::to_string(sh.per_gate) + " down=" + std::to_string(sh.per_down));
    // id n_expert names the shared expert when the call carries one
    const size_t id_limit = sh.n_expert + (shared.all ? 1 : 0);
    for (size_t i = 0; i < n_slots; i++)
        if (expert_ids[i] >= id_limit)
            return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 selected-base expert id out of range: id=" +
                                                     std::to_string(expert_ids[i]) + " n_expert=" +
                                                     std::to_string(sh.n_expert));
    if (out_len < token_count * n_embd)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer output length mismatch: got " +
                                                 std::to_string(out_len) + ", expected >= " +
                                                 std::to_string(token_count * n_embd));
    if (n_slots > 0x0fffffffu || token_count > 0x0fffffffu)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer slot count out of range");
    if (n_ff > 0x00ffffffu || n_embd > 0x00ffffffu)  // the kernels index with 32 bits
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer dims out of range");
    *shape = sh;
    return RNB_HIP_OK;
}

// Up to this many slots (the reference's decode calls pass at most 32, fanout.rs:776-790) the down projection runs
// token-major with the reduce fused in; beyond it expert-major, so that an expert is read once for all its tokens.
constexpr size_t kMoeTokenMajorSlots = 32;

// Device-side sequence for the gathered expert path.  x_dev [token_count][n_embd], out_dev likewise.
int run_moe_dev(State &s, const uint8_t *gate_dev, const uint8_t *up_dev, const uint8_t *down_dev, const MoeShared &shared,
                const MoeShape &sh, const uint32_t *expert_ids, const float *route, const uint32_t *token_ids,
                size_t n_slots, size_t token_count, uint32_t down_quant, size_t n_ff, size_t n_embd,
                const float *x_dev, float *out_dev) {
    if (token_count == 0) return RNB_HIP_OK;
    if (token_count <= kMoeDecodeMaxTokens && n_slots <= kMoeDecodeMaxSlots) {
        // decode and small batches: no host-side sort by expert and no table image, two launches
        MoeDecodeTable table = {};
        table.n_slots = static_cast<uint32_t>(n_slots);
        table.n_tokens = static_cast<uint32_t>(token_count);
        size_t max_per_token = 0;
        for (size_t i = 0; i < n_slots; i++) table.tok_off[token_ids[i] + 1]++;  // token ids are validated
        for (size_t t = 0; t < token_count; t++) {
            max_per_token = std::max<size_t>(max_per_token, table.tok_off[t + 1]);
            table.tok_off[t + 1] += table.tok_off[t];
        }
        if (moe_decode_supported(token_count, n_slots, max_per_token, sh.nb_in, sh.nb_mid, x_dev, down_quant, down_dev, shared.down)) {
            uint32_t fill[kMoeDecodeMaxTokens] = {};
            for (size_t i = 0; i < n_slots; i++) {  // token by token, list order kept inside a token
                const uint32_t t = token_ids[i], at = table.tok_off[t] + fill[t]++;
                table.expert[at] = expert_ids[i];
                table.route[at] = route[i];
                table.token[at] = t;
            }
            RESERVE_TRY(s.moe_mid, n_slots * n_ff * sizeof(float));
            launch_moe_decode(gate_dev, up_dev, down_dev, shared, down_quant, table, x_dev, s.moe_mid.as<float>(), out_dev,
                              static_cast<uint32_t>(n_ff), static_cast<uint32_t>(n_embd), static_cast<uint32_t>(sh.nb_in),
                              static_cast<uint32_t>(sh.nb_mid), s.stream);
            if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
            return RNB_HIP_OK;
        }
    }
    // slots are grouped by expert, keeping slot order inside a group
    std::vector<uint32_t> order(n_slots);
    for (size_t i = 0; i < n_slots; i++) order[i] = static_cast<uint32_t>(i);
    std::stable_sort(order.begin(), order.end(),
                     [expert_ids](uint32_t a, uint32_t b) { return expert_ids[a] < expert_ids[b]; });
    std::vector<uint32_t> grp_expert, grp_start;
    for (size_t p = 0; p < n_slots; p++) {
        if (p == 0 || expert_ids[order[p]] != expert_ids[order[p - 1]]) {
            grp_expert.push_back(expert_ids[order[p]]);
            grp_start.push_back(static_cast<uint32_t>(p));
        }
    }
    grp_start.push_back(static_cast<uint32_t>(n_slots));
    const size_t n_groups = grp_expert.size();
    // one table image: route[n] | tok_offsets[T+1] | tok_slots[n] | sorted_slot[n] | sorted_token[n] | grp_expert[G] |
    // grp_start[G+1] | slot_expert[n]
    const size_t table_words = 5 * n_slots + (token_count + 1) + n_groups + (n_groups + 1);
    // Batches with at least 1.8 slots per routed expert on average: the expert GEMMs run on the matrix cores (a
    // 32-token tile costs the same whatever its number of live tokens, the integer-dot kernels cost per token; measured
    // on 128 experts x top-8: 16 / 20 / 24 tokens 71.9 / 84.2 / 93.9 us on the integer-dot kernels, 79.0 / 85.7 / 88.2
    // on the matrix cores; the ratio is 1.6 / 1.8 / 1.9 there) and need the quantiser's digits
    // (its gate/up rows arrive as 16-byte LDS-direct loads: other alignments take the vector kernels)
    // (and the Q6_K down rows as dword-aligned pieces: an even base address and whole 128-row tiles)
    const bool aligned16 = ((reinterpret_cast<uintptr_t>(gate_dev) | reinterpret_cast<uintptr_t>(up_dev) |
                             reinterpret_cast<uintptr_t>(down_dev) | reinterpret_cast<uintptr_t>(shared.gate) |
                             reinterpret_cast<uintptr_t>(shared.up) | reinterpret_cast<uintptr_t>(shared.down)) & 15u) == 0;
    const bool mfma = token_count >= kMoeMfmaMinTokens && 10 * n_slots >= 18 * n_groups && aligned16 && n_embd % 128 == 0 &&
                      moe_mfma_supported(static_cast<uint32_t>(sh.nb_in), static_cast<uint32_t>(sh.nb_mid), down_quant);
    const bool inline_tables = !mfma && table_words <= kMoeInlineWords;  // decode-sized: rides in a kernel argument
    MoeInlineTables inl;
    uint32_t *h = inl.words;
    TableSlot *ring_slot = nullptr;
    if (!inline_tables) {
        if (s.capturing())
            return fail(RNB_HIP_INVALID_REQUEST,
                        "Qwen35 full-layer routing tables of this size are uploaded from host memory and cannot be captured "
                        "into a graph (one token with at most 16 slots, or tables of at most 240 words, can)");
        // larger tables go through one of a ring of pinned buffers, so that a call never waits for the
        // previous call's upload to drain
        ring_slot = &s.table_ring[s.table_ring_next];
        s.table_ring_next = (s.table_ring_next + 1) % State::kTableRing;
        if (ring_slot->event == nullptr)
            HIP_TRY(hipEventCreateWithFlags(&ring_slot->event, hipEventDisableTiming));
        else
            HIP_TRY(hipEventSynchronize(ring_slot->event));
        RESERVE_TRY(ring_slot->host, table_words * 4);
        h = ring_slot->host.as<uint32_t>();
    }
    RESERVE_TRY(s.moe_tables, table_words * 4);
    float *h_route = reinterpret_cast<float *>(h);
    uint32_t *h_off = h + n_slots, *h_list = h_off + token_count + 1;
    uint32_t *h_sslot = h_list + n_slots, *h_stok = h_sslot + n_slots;
    uint32_t *h_gexp = h_stok + n_slots, *h_gstart = h_gexp + n_groups, *h_sexp = h_gstart + n_groups + 1;
    if (n_slots) std::memcpy(h_route, route, n_slots * 4);
    if (n_slots) std::memcpy(h_sexp, expert_ids, n_slots * 4);
    std::vector<uint32_t> counts(token_count + 1, 0);
    for (size_t i = 0; i < n_slots; i++) counts[token_ids[i] + 1]++;
    for (size_t t = 0; t < token_count; t++) counts[t + 1] += counts[t];
    std::memcpy(h_off, counts.data(), (token_count + 1) * 4);
    for (size_t i = 0; i < n_slots; i++) h_list[counts[token_ids[i]]++] = static_cast<uint32_t>(i);  // slot order kept
    for (size_t p = 0; p < n_slots; p++) {
        h_sslot[p] = order[p];
        h_stok[p] = token_ids[order[p]];
    }
    if (n_groups) std::memcpy(h_gexp, grp_expert.data(), n_groups * 4);
    std::memcpy(h_gstart, grp_start.data(), (n_groups + 1) * 4);
    uint32_t *d = s.moe_tables.as<uint32_t>();
    const float *d_route = reinterpret_cast<const float *>(d);
    const uint32_t *d_off = d + n_slots, *d_list = d_off + token_count + 1;
    uint32_t max_group = 0;
    for (size_t g = 0; g < n_groups; g++) max_group = std::max(max_group, grp_start[g + 1] - grp_start[g]);
    const MoeGroups groups{d_list + 3 * n_slots, d_list + 3 * n_slots + n_groups, d_list + n_slots, d_list + 2 * n_slots,
                           static_cast<uint32_t>(n_groups), max_group};

    ActView act;
    if (inline_tables) {
        // quantise x and drop the tables into device memory with the same launch
        const size_t nq = token_count * n_embd;
        RESERVE_TRY(s.act_qs, nq);
        RESERVE_TRY(s.act_d, nq / 256 * sizeof(float));
        RESERVE_TRY(s.act_bsums, nq / 256 * 16 * sizeof(int16_t));
        launch_quantize_q8k_with_tables(x_dev, nq / 256, s.act_qs.as<int8_t>(), s.act_d.as<float>(),
                                        s.act_bsums.as<int16_t>(), inl, static_cast<uint32_t>(table_words), d, s.stream);
        if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
        act = {s.act_qs.as<int8_t>(), s.act_d.as<float>(), s.act_bsums.as<int16_t>()};
        s.act_family = kQ4K;
        s.act_has_digits = false;
        s.act_seq = token_count;
        s.act_cols = n_embd;
    } else {
        // the quantiser's launch reads the tables from the pinned buffer and leaves them in device memory (no copy command)
        const WordCopy tables{h, d, static_cast<uint32_t>(table_words)};
        int st = quantize_activations(s, kQ4K, x_dev, token_count, n_embd, &act, nullptr, &tables);
        if (st != RNB_HIP_OK) return st;
        HIP_TRY(hipEventRecord(ring_slot->event, s.stream));  // the pinned buffer is free again once that launch is done
        s.h2d_bytes += table_words * 4;
    }
    if (n_slots == 0) {  // nothing routed: the reduce kernel alone writes the zero rows
        launch_moe_reduce(nullptr, d_off, d_list, out_dev, static_cast<uint32_t>(token_count),
                          static_cast<uint32_t>(n_embd), s.stream);
        if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
        return RNB_HIP_OK;
    }
    RESERVE_TRY(s.moe_mid, n_slots * n_ff * sizeof(float));
    RESERVE_TRY(s.moe_slot_out, n_slots * n_embd * sizeof(float));
    if (mfma && act.digits != nullptr) {
        // prefill: grouped GEMMs on the matrix cores; the down kernel quantises the intermediate as it stages it
        launch_moe_gate_up_mfma(gate_dev, up_dev, shared, act, groups, s.moe_mid.as<float>(), static_cast<uint32_t>(n_ff),
                                static_cast<uint32_t>(sh.nb_in), s.stream);
        launch_moe_down_mfma(down_dev, shared, down_quant, s.moe_mid.as<float>(), groups, d_route, s.moe_slot_out.as<float>(),
                             static_cast<uint32_t>(n_embd), static_cast<uint32_t>(sh.nb_mid), s.stream);
        launch_moe_reduce(s.moe_slot_out.as<float>(), d_off, d_list, out_dev, static_cast<uint32_t>(token_count),
                          static_cast<uint32_t>(n_embd), s.stream);
        if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
        return RNB_HIP_OK;
    }
    RESERVE_TRY(s.moe_mid_qs, n_slots * n_ff);
    RESERVE_TRY(s.moe_mid_d, n_slots * sh.nb_mid * sizeof(float));
    RESERVE_TRY(s.moe_mid_bsums, n_slots * sh.nb_mid * 16 * sizeof(int16_t));
    launch_moe_gate_up(gate_dev, up_dev, shared, act, groups, s.moe_mid.as<float>(), static_cast<uint32_t>(n_ff),
                       static_cast<uint32_t>(sh.nb_in), s.stream);
    const bool token_major = n_slots <= kMoeTokenMajorSlots && sh.nb_mid <= 16;
    // expert-major with short intermediates: the down kernel quantises the rows it stages, one launch fewer
    const bool down_quantises = !token_major && moe_down_quantises(static_cast<uint32_t>(sh.nb_mid));
    if (!down_quantises)
        launch_quantize_q8k(s.moe_mid.as<float>(), n_slots * sh.nb_mid, s.moe_mid_qs.as<int8_t>(), s.moe_mid_d.as<float>(),
                            s.moe_mid_bsums.as<int16_t>(), nullptr, s.stream);
    ActView mid{s.moe_mid_qs.as<int8_t>(), s.moe_mid_d.as<float>(), s.moe_mid_bsums.as<int16_t>()};
    if (token_major) {
        // decode: few slots, every expert is read by one token anyway; one launch does down, route and the ordered sum
        const uint32_t *d_sexp = d_list + 3 * n_slots + n_groups + (n_groups + 1);
        launch_moe_down_token(down_dev, shared, down_quant, mid, d_off, d_list, d_sexp, d_route, out_dev,
                              static_cast<uint32_t>(token_count), static_cast<uint32_t>(n_embd),
                              static_cast<uint32_t>(sh.nb_mid), s.stream);
    } else {
        launch_moe_down(down_dev, shared, down_quant, mid, down_quantises ? s.moe_mid.as<float>() : nullptr, groups, d_route,
                        s.moe_slot_out.as<float>(),
                        static_cast<uint32_t>(n_embd), static_cast<uint32_t>(sh.nb_mid), s.stream);
        launch_moe_reduce(s.moe_slot_out.as<float>(), d_off, d_list, out_dev, static_cast<uint32_t>(token_count),
                          static_cast<uint32_t>(n_embd), s.stream);
    }
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    return RNB_HIP_OK;
}

int static_scratch_ptr(State &s, uint8_t **out);

}  // namespace

extern "C" {

int rnb_hip_backend_kind(void) { return 6; }

int rnb_hip_backend_supports(int op) { return (op == RNB_OP_MATMUL || op == RNB_OP_MOE) ? 1 : 0; }

int rnb_hip_backend_supports_quant(int op, uint32_t quant) {
    if (op == RNB_OP_MATMUL) return (is_block32(quant) || (quant >= kQ2K && quant <= kQ6K) || is_iq_quant(quant)) ? 1 : 0;
    if (op == RNB_OP_MOE) return (quant == kQ4K || quant == kQ5K || quant == kQ6K) ? 1 : 0;
    return 0;
}

int rnb_hip_init(void) {
    Guard g;
    if (!g.state) return g.status;
    uint8_t *unused = nullptr;  // the no-allocation entry point's scratch address is looked up here, once per device
    return static_scratch_ptr(*g.state, &unused);
}

const char *rnb_hip_last_error(void) { return last_error_cstr(); }

int rnb_hip_device_name(char *buf, size_t buf_len) {
    Guard g;
    if (!g.state) return g.status;
    if (!buf || buf_len == 0) return fail(RNB_HIP_INVALID_REQUEST, "device_name: empty buffer");
    std::strncpy(buf, g.state->device_name.c_str(), buf_len - 1);
    buf[buf_len - 1] = 0;
    return RNB_HIP_OK;
}

int rnb_hip_sync(void) {
    Guard g;
    if (!g.state) return g.status;
    HIP_TRY(hipStreamSynchronize(g.state->stream));
    return RNB_HIP_OK;
}

int rnb_hip_transfer_counters(uint64_t *h2d_bytes, uint64_t *d2h_bytes) {
    Guard g;
    if (!g.state) return g.status;
    const ResidencyStats &rs = g.state->table->stats();
    if (h2d_bytes) *h2d_bytes = g.state->h2d_bytes + rs.h2d_bytes + rs.temp_h2d_bytes;
    if (d2h_bytes) *d2h_bytes = g.state->d2h_bytes;
    return RNB_HIP_OK;
}

void *rnb_hip_stream(void) {
    Guard g;
    return g.state ? static_cast<void *>(g.state->stream) : nullptr;
}

int rnb_hip_prewarm(const uint8_t *const *ptrs, const size_t *lens, size_t n) {
    Guard g;
    if (!g.state) return g.status;
    for (size_t i = 0; i < n; i++) {
        if (!ptrs[i] || lens[i] == 0) continue;
        const uint8_t *dev = nullptr;
        if (int rs = g.state->resident_ptr(ptrs[i], lens[i], &dev, /*pin=*/true); rs != RNB_HIP_OK) return rs;
    }
    return RNB_HIP_OK;
}

int rnb_hip_release(const uint8_t *ptr, size_t len) {
    Guard g;
    if (!g.state) return g.status;
    if (g.state->capturing())
        return fail(RNB_HIP_INVALID_REQUEST, "release frees device memory and cannot run while the library stream is capturing");
    if (!g.state->release(ptr, len)) return fail(RNB_HIP_INVALID_REQUEST, "release: range is not resident");
    return RNB_HIP_OK;
}

int rnb_hip_resident_bytes(uint64_t *bytes, uint64_t *entries) {
    Guard g;
    if (!g.state) return g.status;
    if (bytes) *bytes = g.state->table->resident_bytes();
    if (entries) *entries = g.state->table->entries();
    return RNB_HIP_OK;
}

int rnb_hip_calib_read(const void *dev, size_t bytes, int non_temporal) {
    if (!dev || (reinterpret_cast<uintptr_t>(dev) & 15u)) return fail(RNB_HIP_INVALID_REQUEST, "calibration read needs a 16-byte aligned device pointer");
    Guard g;
    if (!g.state) return g.status;
    RESERVE_TRY(g.state->argmax_scratch, 257 * 8);
    launch_calib_read(dev, bytes, non_temporal != 0, g.state->argmax_scratch.as<uint32_t>(), g.state->stream);
    return check_launches();
}

int rnb_hip_calib_mfma_i8(uint32_t iters, uint32_t workgroups, uint64_t *ops) {
    Guard g;
    if (!g.state) return g.status;
    RESERVE_TRY(g.state->argmax_scratch, 257 * 8);
    const uint64_t n = launch_calib_mfma_i8(iters, workgroups, g.state->argmax_scratch.as<int>(), g.state->stream);
    if (ops) *ops = n;
    return check_launches();
}

int rnb_hip_residency_stats(uint64_t *out, size_t n) {
    Guard g;
    if (!g.state) return g.status;
    const ResidencyStats &rs = g.state->table->stats();
    const uint64_t v[12] = {rs.lookups, rs.hits, rs.sub_range_hits, rs.misses, rs.admissions, rs.evictions,
                            rs.admitted_bytes, rs.evicted_bytes, rs.h2d_bytes, rs.temp_h2d_bytes, rs.oom_retries,
                            g.state->table->budget()};
    for (size_t i = 0; i < n && i < 12; i++) out[i] = v[i];
    return RNB_HIP_OK;
}

int rnb_hip_set_resident_budget(uint64_t bytes) {
    Guard g;
    if (!g.state) return g.status;
    if (g.state->capturing())
        return fail(RNB_HIP_INVALID_REQUEST, "set_resident_budget frees device memory and cannot run while the library stream is capturing");
    g.state->table->set_budget(bytes);
    return RNB_HIP_OK;
}

int rnb_hip_offload_unpinned(uint64_t *freed_bytes) {
    Guard g;
    if (!g.state) return g.status;
    if (g.state->capturing())
        return fail(RNB_HIP_INVALID_REQUEST, "offload_unpinned frees device memory and cannot run while the library stream is capturing");
    std::string err;
    const uint64_t freed = g.state->table->offload_unpinned(&err);
    if (freed_bytes) *freed_bytes = freed;
    if (!err.empty()) return fail(RNB_HIP_EXECUTION_FAILED, err);
    return RNB_HIP_OK;
}

int rnb_hip_quantize_q8k(const float *x, size_t n, void *out_blocks, size_t out_bytes) {
    if (n % 256 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_K input length must be divisible by 256, got " + std::to_string(n));
    const size_t nb = n / 256;
    if (out_bytes < nb * 292)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_K output byte mismatch: got " + std::to_string(out_bytes) +
                                                 ", expected " + std::to_string(nb * 292));
    if (nb == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    RESERVE_TRY(s.bounce_in, n * 4);
    HIP_TRY(s.x_f32.reserve(n * 4));
    std::memcpy(s.bounce_in.ptr, x, n * 4);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, n * 4, hipMemcpyHostToDevice, s.stream));
    ActView act;
    int st = quantize_activations(s, kQ4K, s.x_f32.as<float>(), 1, n, &act);
    if (st != RNB_HIP_OK) return st;
    const size_t qs_b = n, d_b = nb * 4, bs_b = nb * 32;
    RESERVE_TRY(s.bounce_out, qs_b + d_b + bs_b);
    uint8_t *h = s.bounce_out.as<uint8_t>();
    HIP_TRY(hipMemcpyAsync(h, act.qs, qs_b, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipMemcpyAsync(h + qs_b, act.d, d_b, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipMemcpyAsync(h + qs_b + d_b, act.bsums, bs_b, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.h2d_bytes += n * 4;
    s.d2h_bytes += qs_b + d_b + bs_b;
    // repack the device structure-of-arrays into the reference's 292-byte repr(C) block
    uint8_t *o = static_cast<uint8_t *>(out_blocks);
    for (size_t b = 0; b < nb; b++) {
        std::memcpy(o + b * 292, h + qs_b + b * 4, 4);
        std::memcpy(o + b * 292 + 4, h + b * 256, 256);
        std::memcpy(o + b * 292 + 260, h + qs_b + d_b + b * 32, 32);
    }
    return RNB_HIP_OK;
}

int rnb_hip_quantize_q8(const float *x, size_t n, void *out_blocks, size_t out_bytes) {
    if (n % 32 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8 input length must be divisible by 32, got " + std::to_string(n));
    const size_t nb = n / 32;
    if (out_bytes < nb * 36)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8 output byte mismatch: got " + std::to_string(out_bytes) +
                                                 ", expected " + std::to_string(nb * 36));
    if (nb == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    RESERVE_TRY(s.bounce_in, n * 4);
    HIP_TRY(s.x_f32.reserve(n * 4 + 1024));
    std::memcpy(s.bounce_in.ptr, x, n * 4);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, n * 4, hipMemcpyHostToDevice, s.stream));
    ActView act;
    int st = quantize_activations(s, kQ8_0, s.x_f32.as<float>(), 1, n, &act);
    if (st != RNB_HIP_OK) return st;
    RESERVE_TRY(s.bounce_out, n + nb * 4);
    uint8_t *h = s.bounce_out.as<uint8_t>();
    HIP_TRY(hipMemcpyAsync(h, act.qs, n, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipMemcpyAsync(h + n, act.d, nb * 4, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.h2d_bytes += n * 4;
    s.d2h_bytes += n + nb * 4;
    uint8_t *o = static_cast<uint8_t *>(out_blocks);
    for (size_t b = 0; b < nb; b++) {
        std::memcpy(o + b * 36, h + n + b * 4, 4);
        std::memcpy(o + b * 36 + 4, h + b * 32, 32);
    }
    return RNB_HIP_OK;
}

int rnb_hip_q4k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                     float *out, size_t out_len) {
    return matmul_host(kQ4K, w, w_len, rows, cols, x, x_len, out, out_len, false);
}
int rnb_hip_q4k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                           float *out, size_t out_len) {
    return matmul_host(kQ4K, w, w_len, rows, cols, x, x_len, out, out_len, true);
}
#define RNB_BLOCK32_ENTRY(name, quant)                                                                                \
    int rnb_hip_##name##_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,  \
                              float *out, size_t out_len) {                                                            \
        return matmul_host(quant, w, w_len, rows, cols, x, x_len, out, out_len, false);                                \
    }                                                                                                                  \
    int rnb_hip_##name##_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,          \
                                    size_t x_len, float *out, size_t out_len) {                                        \
        return matmul_host(quant, w, w_len, rows, cols, x, x_len, out, out_len, true);                                 \
    }
RNB_BLOCK32_ENTRY(q4_0, kQ4_0)
RNB_BLOCK32_ENTRY(q4_1, kQ4_1)
RNB_BLOCK32_ENTRY(q5_0, kQ5_0)
RNB_BLOCK32_ENTRY(q5_1, kQ5_1)
RNB_BLOCK32_ENTRY(q8_1, kQ8_1)
#undef RNB_BLOCK32_ENTRY

int rnb_hip_q2k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                     float *out, size_t out_len) {
    return matmul_host(kQ2K, w, w_len, rows, cols, x, x_len, out, out_len, false);
}
int rnb_hip_q2k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                           float *out, size_t out_len) {
    return matmul_host(kQ2K, w, w_len, rows, cols, x, x_len, out, out_len, true);
}
int rnb_hip_q3k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                     float *out, size_t out_len) {
    return matmul_host(kQ3K, w, w_len, rows, cols, x, x_len, out, out_len, false);
}
int rnb_hip_q3k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                           float *out, size_t out_len) {
    return matmul_host(kQ3K, w, w_len, rows, cols, x, x_len, out, out_len, true);
}
#define RNB_IQ_ENTRY(name, quant)                                                                                   \
    int rnb_hip_##name##_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,  \
                              float *out, size_t out_len) {                                                          \
        return matmul_host(quant, w, w_len, rows, cols, x, x_len, out, out_len, false);                              \
    }                                                                                                                \
    int rnb_hip_##name##_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,          \
                                    size_t x_len, float *out, size_t out_len) {                                      \
        return matmul_host(quant, w, w_len, rows, cols, x, x_len, out, out_len, true);                               \
    }
RNB_IQ_ENTRY(iq2_xxs, kIQ2XXS)
RNB_IQ_ENTRY(iq2_s, kIQ2S)
RNB_IQ_ENTRY(iq3_xxs, kIQ3XXS)
RNB_IQ_ENTRY(iq4_xs, kIQ4XS)
#undef RNB_IQ_ENTRY

int rnb_hip_q4k_gemv_with_device_input(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x_dev,
                                       float *out, size_t out_len) {
    return matmul_device_input(kQ4K, w, w_len, rows, cols, x_dev, out, out_len);
}
int rnb_hip_q6k_gemv_with_device_input(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x_dev,
                                       float *out, size_t out_len) {
    return matmul_device_input(kQ6K, w, w_len, rows, cols, x_dev, out, out_len);
}

int rnb_hip_q5k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                     float *out, size_t out_len) {
    return matmul_host(kQ5K, w, w_len, rows, cols, x, x_len, out, out_len, false);
}
int rnb_hip_q5k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                           float *out, size_t out_len) {
    return matmul_host(kQ5K, w, w_len, rows, cols, x, x_len, out, out_len, true);
}
int rnb_hip_q6k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                     float *out, size_t out_len) {
    return matmul_host(kQ6K, w, w_len, rows, cols, x, x_len, out, out_len, false);
}
int rnb_hip_q6k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                           float *out, size_t out_len) {
    return matmul_host(kQ6K, w, w_len, rows, cols, x, x_len, out, out_len, true);
}
int rnb_hip_q8_0_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                      float *out, size_t out_len) {
    return matmul_host(kQ8_0, w, w_len, rows, cols, x, x_len, out, out_len, false);
}
int rnb_hip_q8_0_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                            float *out, size_t out_len) {
    return matmul_host(kQ8_0, w, w_len, rows, cols, x, x_len, out, out_len, true);
}

// q8_0_head_gemv_batch, crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:824-882 (checks and texts in its order):
// head h has its own rows_per_head rows, token t's input for it is x[(t * head_count + h) * cols ..], out is
// [token][head_count * rows_per_head].  Every (token, head) group is the Q8_0 GEMV on that head's rows.
int rnb_hip_q8_0_head_gemv_batch(const uint8_t *w, size_t w_len, size_t head_count, size_t rows_per_head, size_t cols,
                                 size_t token_count, const float *x, size_t x_len, float *out, size_t out_len) {
    if (head_count == 0 || rows_per_head == 0 || token_count == 0)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch dimensions must be non-zero: heads=" + std::to_string(head_count) +
                                                 " rows_per_head=" + std::to_string(rows_per_head) +
                                                 " tokens=" + std::to_string(token_count));
    if (cols == 0 || cols % 32 != 0)
        return fail(RNB_HIP_INVALID_REQUEST,
                    "Q8_0 head batch cols must be non-zero and divisible by 32, got " + std::to_string(cols));
    const size_t nb32 = cols / 32;
    size_t rows = 0, blocks = 0, expected_w = 0;
    if (__builtin_mul_overflow(head_count, rows_per_head, &rows) || __builtin_mul_overflow(rows, nb32, &blocks) ||
        __builtin_mul_overflow(blocks, size_t(34), &expected_w))
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch weight byte size overflow");
    if (w_len != expected_w)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch weight byte mismatch: got " + std::to_string(w_len) +
                                                 ", expected " + std::to_string(expected_w));
    size_t vecs = 0, expected_x = 0;
    if (__builtin_mul_overflow(token_count, head_count, &vecs) || __builtin_mul_overflow(vecs, cols, &expected_x))
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch input length overflow");
    if (x_len != expected_x)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch input length mismatch: got " + std::to_string(x_len) +
                                                 ", expected " + std::to_string(expected_x));
    size_t n_out = 0;
    if (__builtin_mul_overflow(token_count, rows, &n_out) || out_len < n_out)
        return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch output too small: got " + std::to_string(out_len) +
                                                 ", expected >= " + std::to_string(token_count) + " x " + std::to_string(rows));
    if (!w || !x || !out) return fail(RNB_HIP_INVALID_REQUEST, "Q8_0 head batch null pointer argument");
    if (!gemv_q8_0_heads_supported(static_cast<uint32_t>(nb32 > 0xffffffffu ? 0xffffffffu : nb32)) || head_count > 65535 ||
        rows_per_head > 0x7fffffffu || token_count > 262140u)
        return fail(RNB_HIP_UNSUPPORTED_OP, "Q8_0 head batch shape not supported: cols=" + std::to_string(cols) + " heads=" +
                                                std::to_string(head_count) + " tokens=" + std::to_string(token_count) +
                                                " (cols <= 4096, heads <= 65535, tokens <= 262140)");
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *w_dev = nullptr;
    if (int rs = s.resident_ptr(w, w_len, &w_dev); rs != RNB_HIP_OK) return rs;
    const size_t in_bytes = expected_x * sizeof(float), out_bytes = n_out * sizeof(float);
    RESERVE_TRY(s.bounce_in, in_bytes);
    RESERVE_TRY(s.bounce_out, out_bytes);
    HIP_TRY(s.x_f32.reserve(in_bytes));
    HIP_TRY(s.out_f32.reserve(out_bytes));
    std::memcpy(s.bounce_in.ptr, x, in_bytes);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, in_bytes, hipMemcpyHostToDevice, s.stream));
    s.h2d_bytes += in_bytes;
    ActView act;
    // every (token, head) vector is quantised as a row of its own: token_count * head_count rows of cols
    if (int st = quantize_activations(s, kQ8_0, s.x_f32.as<float>(), vecs, cols, &act); st != RNB_HIP_OK) return st;
    launch_gemv_q8_0_heads(w_dev, act, s.out_f32.as<float>(), static_cast<uint32_t>(head_count),
                           static_cast<uint32_t>(rows_per_head), static_cast<uint32_t>(nb32), static_cast<uint32_t>(token_count),
                           s.stream);
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, s.out_f32.ptr, out_bytes, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += out_bytes;
    std::memcpy(out, s.bounce_out.ptr, out_bytes);
    return RNB_HIP_OK;
}

int rnb_hip_moe_sparse_experts_by_token(const uint8_t *gate_all, size_t gate_len, const uint8_t *up_all,
                                        size_t up_len, const uint8_t *down_all, size_t down_len,
                                        const uint8_t *shared_gate, size_t shared_gate_len, const uint8_t *shared_up,
                                        size_t shared_up_len, const uint8_t *shared_down, size_t shared_down_len,
                                        const uint32_t *expert_ids, const float *route_weights,
                                        const uint32_t *token_ids, size_t n_slots, size_t token_count,
                                        uint32_t down_quant, size_t n_ff, size_t n_embd, const float *x, size_t x_len,
                                        float *out, size_t out_len) {
    MoeShape sh;
    SharedLens sl;
    sl.any = shared_gate != nullptr || shared_up != nullptr || shared_down != nullptr;
    sl.all = shared_gate != nullptr && shared_up != nullptr && shared_down != nullptr;
    sl.gate = shared_gate_len, sl.up = shared_up_len, sl.down = shared_down_len;
    int st = validate_moe(gate_len, up_len, down_len, sl, expert_ids, token_ids, n_slots, token_count, down_quant, n_ff,
                          n_embd, x_len, out_len, &sh);
    if (st != RNB_HIP_OK) return st;
    if (token_count == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *gate_dev = nullptr, *up_dev = nullptr, *down_dev = nullptr;
    if (int rs = s.resident_ptr(gate_all, gate_len, &gate_dev); rs != RNB_HIP_OK) return rs;
    if (int rs = s.resident_ptr(up_all, up_len, &up_dev); rs != RNB_HIP_OK) return rs;
    if (int rs = s.resident_ptr(down_all, down_len, &down_dev); rs != RNB_HIP_OK) return rs;
    MoeShared shared;
    if (sl.all) {
        if (int rs = s.resident_ptr(shared_gate, shared_gate_len, &shared.gate); rs != RNB_HIP_OK) return rs;
        if (int rs = s.resident_ptr(shared_up, shared_up_len, &shared.up); rs != RNB_HIP_OK) return rs;
        if (int rs = s.resident_ptr(shared_down, shared_down_len, &shared.down); rs != RNB_HIP_OK) return rs;
        shared.n_routed = static_cast<uint32_t>(sh.n_expert);
    }
    const size_t io_bytes = token_count * n_embd * sizeof(float);
    RESERVE_TRY(s.bounce_in, io_bytes);
    RESERVE_TRY(s.bounce_out, io_bytes);
    HIP_TRY(s.x_f32.reserve(io_bytes));
    HIP_TRY(s.out_f32.reserve(io_bytes));
    std::memcpy(s.bounce_in.ptr, x, io_bytes);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, io_bytes, hipMemcpyHostToDevice, s.stream));
    s.h2d_bytes += io_bytes;
    st = run_moe_dev(s, gate_dev, up_dev, down_dev, shared, sh, expert_ids, route_weights, token_ids, n_slots, token_count,
                     down_quant, n_ff, n_embd, s.x_f32.as<float>(), s.out_f32.as<float>());
    if (st != RNB_HIP_OK) return st;
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, s.out_f32.ptr, io_bytes, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += io_bytes;
    std::memcpy(out, s.bounce_out.ptr, io_bytes);
    return RNB_HIP_OK;
}

// ---- device-resident variants ------------------------------------------------------------------

void *rnb_hip_dev_alloc(size_t bytes) {
    Guard g;
    if (!g.state) return nullptr;
    void *p = nullptr;
    hipError_t e = hipMalloc(&p, bytes ? bytes : 1);
    if (e != hipSuccess) {
        hip_fail("hipMalloc", e);
        return nullptr;
    }
    return p;
}

int rnb_hip_dev_free(void *ptr) {
    Guard g;
    if (!g.state) return g.status;
    HIP_TRY(hipStreamSynchronize(g.state->stream));
    HIP_TRY(hipFree(ptr));
    return RNB_HIP_OK;
}

int rnb_hip_dev_upload(void *dst_dev, const void *src_host, size_t bytes) {
    Guard g;
    if (!g.state) return g.status;
    HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, g.state->stream));
    HIP_TRY(hipStreamSynchronize(g.state->stream));
    g.state->h2d_bytes += bytes;
    return RNB_HIP_OK;
}

int rnb_hip_dev_download(void *dst_host, const void *src_dev, size_t bytes) {
    Guard g;
    if (!g.state) return g.status;
    HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, g.state->stream));
    HIP_TRY(hipStreamSynchronize(g.state->stream));
    g.state->d2h_bytes += bytes;
    return RNB_HIP_OK;
}

}  // extern "C"

namespace {

// LM-head GEMV with the arg-max taken on the device.  The same three checks and texts as the format's plain GEMV
// (crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:2176-2193 for Q6_K, :739-756 for Q8_0).
int gemv_argmax_host(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                     size_t x_len, uint32_t *index_out, float *value_out) {
    QuantInfo qi;
    quant_info(quant, &qi);
    const std::string label = qi.label;
    size_t seq = 0;
    int st = validate_matmul(qi, w_len, rows, cols, x_len, rows, false, &seq);
    if (st != RNB_HIP_OK) return st;
    if (!w || !x || !index_out || !value_out) return fail(RNB_HIP_INVALID_REQUEST, label + " null pointer argument");
    if (rows == 0) return fail(RNB_HIP_INVALID_REQUEST, label + " argmax needs at least one row");
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *w_dev = nullptr;
    if (int rs = s.resident_ptr(w, w_len, &w_dev); rs != RNB_HIP_OK) return rs;
    const size_t in_bytes = cols * sizeof(float);
    RESERVE_TRY(s.bounce_in, in_bytes);
    RESERVE_TRY(s.bounce_out, 16);
    HIP_TRY(s.x_f32.reserve(in_bytes));
    HIP_TRY(s.out_f32.reserve(rows * sizeof(float)));
    RESERVE_TRY(s.argmax_scratch, 257 * 8);
    std::memcpy(s.bounce_in.ptr, x, in_bytes);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, in_bytes, hipMemcpyHostToDevice, s.stream));
    s.h2d_bytes += in_bytes;
    st = run_matmul_dev(s, quant, w_dev, rows, cols, s.x_f32.as<float>(), 1, s.out_f32.as<float>());
    if (st != RNB_HIP_OK) return st;
    float *vals = s.argmax_scratch.as<float>();
    uint32_t *idxs = reinterpret_cast<uint32_t *>(vals + 257);
    launch_argmax(s.out_f32.as<float>(), static_cast<uint32_t>(rows), vals, idxs, vals + 256, idxs + 256, s.stream);
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    // only the winner crosses the bus: 8 bytes instead of rows * 4
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, vals + 256, 4, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipMemcpyAsync(static_cast<uint8_t *>(s.bounce_out.ptr) + 4, idxs + 256, 4, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += 8;
    std::memcpy(value_out, s.bounce_out.ptr, 4);
    std::memcpy(index_out, static_cast<uint8_t *>(s.bounce_out.ptr) + 4, 4);
    return RNB_HIP_OK;
}

}  // namespace

extern "C" {

int rnb_hip_q6k_gemv_argmax(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                            uint32_t *index_out, float *value_out) {
    return gemv_argmax_host(kQ6K, w, w_len, rows, cols, x, x_len, index_out, value_out);
}

int rnb_hip_q8_0_gemv_argmax(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                             uint32_t *index_out, float *value_out) {
    return gemv_argmax_host(kQ8_0, w, w_len, rows, cols, x, x_len, index_out, value_out);
}

// q8_0_gemv_argmax_q8dot, quant_api.rs:770-805: the variant whose name says that the input is quantised to Q8 and dotted in
// integers, which is what the entry above does as well
int rnb_hip_q8_0_gemv_argmax_q8dot(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                                   uint32_t *index_out, float *value_out) {
    return gemv_argmax_host(kQ8_0, w, w_len, rows, cols, x, x_len, index_out, value_out);
}

int rnb_hip_dense_q4k_attention_qkv(const uint8_t *q_w, size_t q_len, const uint8_t *k_w, size_t k_len, const uint8_t *v_w,
                                    size_t v_len, size_t q_rows, size_t kv_rows, size_t n_embd, const float *x, size_t x_len,
                                    float *q, size_t q_cap, float *k, size_t k_cap, float *v, size_t v_cap) {
    // validation order and texts: crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:928-968
    if (x_len != n_embd)
        return fail(RNB_HIP_INVALID_REQUEST,
                    "dense QKV input length mismatch: got " + std::to_string(x_len) + ", expected " + std::to_string(n_embd));
    if (n_embd % 256 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV cols must be divisible by 256, got " + std::to_string(n_embd));
    if (q_cap < q_rows || k_cap < kv_rows || v_cap < kv_rows)
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV output length mismatch: q=" + std::to_string(q_cap) + " k=" +
                                                 std::to_string(k_cap) + " v=" + std::to_string(v_cap) + " expected q>=" +
                                                 std::to_string(q_rows) + " k/v>=" + std::to_string(kv_rows));
    const size_t row_bytes = n_embd / 256 * kQ4KBytes;
    if (q_len != q_rows * row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV q byte mismatch: got " + std::to_string(q_len) + ", expected " +
                                                 std::to_string(q_rows * row_bytes));
    if (k_len != kv_rows * row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV k byte mismatch: got " + std::to_string(k_len) + ", expected " +
                                                 std::to_string(kv_rows * row_bytes));
    if (v_len != kv_rows * row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV v byte mismatch: got " + std::to_string(v_len) + ", expected " +
                                                 std::to_string(kv_rows * row_bytes));
    if (q_rows > 0x3fffffffu || kv_rows > 0x1fffffffu || n_embd > 0x7fffffffu)
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV shape out of range");
    if ((q_len && !q_w) || (k_len && !k_w) || (v_len && !v_w) || (x_len && !x) || (q_rows && !q) || (kv_rows && (!k || !v)))
        return fail(RNB_HIP_INVALID_REQUEST, "dense QKV null pointer argument");
    const size_t total = q_rows + 2 * kv_rows;
    if (total == 0 || n_embd == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *w_dev[3] = {nullptr, nullptr, nullptr};
    if (q_len) if (int rs = s.resident_ptr(q_w, q_len, &w_dev[0]); rs != RNB_HIP_OK) return rs;
    if (k_len) if (int rs = s.resident_ptr(k_w, k_len, &w_dev[1]); rs != RNB_HIP_OK) return rs;
    if (v_len) if (int rs = s.resident_ptr(v_w, v_len, &w_dev[2]); rs != RNB_HIP_OK) return rs;
    const size_t in_bytes = n_embd * sizeof(float), out_bytes = total * sizeof(float);
    RESERVE_TRY(s.bounce_in, in_bytes);
    RESERVE_TRY(s.bounce_out, out_bytes);
    HIP_TRY(s.x_f32.reserve(in_bytes));
    HIP_TRY(s.out_f32.reserve(out_bytes));
    std::memcpy(s.bounce_in.ptr, x, in_bytes);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, in_bytes, hipMemcpyHostToDevice, s.stream));
    s.h2d_bytes += in_bytes;
    const uint32_t rows[3] = {static_cast<uint32_t>(q_rows), static_cast<uint32_t>(kv_rows), static_cast<uint32_t>(kv_rows)};
    if (n_embd / 256 <= 16) {  // the workgroups quantise the token themselves: one launch for the three projections
        launch_gemv_q4k_multi_f32(w_dev, rows, s.x_f32.as<float>(), s.out_f32.as<float>(), static_cast<uint32_t>(n_embd / 256),
                                  s.stream);
    } else {
        ActView act;
        int st = quantize_activations(s, kQ4K, s.x_f32.as<float>(), 1, n_embd, &act);  // once for the three projections
        if (st != RNB_HIP_OK) return st;
        launch_gemv_q4k_multi(w_dev, rows, act, s.out_f32.as<float>(), static_cast<uint32_t>(n_embd / 256), s.stream);
    }
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, s.out_f32.ptr, out_bytes, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += out_bytes;
    const float *res = static_cast<const float *>(s.bounce_out.ptr);
    std::memcpy(q, res, q_rows * sizeof(float));
    std::memcpy(k, res + q_rows, kv_rows * sizeof(float));
    std::memcpy(v, res + q_rows + kv_rows, kv_rows * sizeof(float));
    return RNB_HIP_OK;
}

}  // extern "C"

namespace {

// host-pointer gated FFN after validation: residency, staging, the device sequence, the copy back
int dense_ffn_host(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len, const uint8_t *down,
                   size_t down_len, uint32_t down_quant, size_t n_ff, size_t n_embd, size_t seq_len, const float *x,
                   float *out, size_t out_len, bool gelu) {
    const std::string name = gelu ? "dense GELU FFN" : "dense SiLU FFN";
    if (out_len < seq_len * n_embd)
        return fail(RNB_HIP_INVALID_REQUEST, name + " batch output length mismatch: got " + std::to_string(out_len) +
                                                 ", expected at least " + std::to_string(seq_len * n_embd));
    if (!gate || !up || !down || !x || !out) return fail(RNB_HIP_INVALID_REQUEST, name + " null pointer argument");
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint8_t *gate_dev = nullptr, *up_dev = nullptr, *down_dev = nullptr;
    if (int rs = s.resident_ptr(gate, gate_len, &gate_dev); rs != RNB_HIP_OK) return rs;
    if (int rs = s.resident_ptr(up, up_len, &up_dev); rs != RNB_HIP_OK) return rs;
    if (int rs = s.resident_ptr(down, down_len, &down_dev); rs != RNB_HIP_OK) return rs;
    const size_t io_bytes = seq_len * n_embd * sizeof(float);
    RESERVE_TRY(s.bounce_in, io_bytes);
    RESERVE_TRY(s.bounce_out, io_bytes);
    HIP_TRY(s.x_f32.reserve(io_bytes));
    HIP_TRY(s.out_f32.reserve(io_bytes));
    std::memcpy(s.bounce_in.ptr, x, io_bytes);
    HIP_TRY(hipMemcpyAsync(s.x_f32.ptr, s.bounce_in.ptr, io_bytes, hipMemcpyHostToDevice, s.stream));
    s.h2d_bytes += io_bytes;
    int st = run_dense_ffn_dev(s, gate_dev, up_dev, down_dev, down_quant, n_ff, n_embd, seq_len, s.x_f32.as<float>(),
                               s.out_f32.as<float>(), gelu);
    if (st != RNB_HIP_OK) return st;
    HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, s.out_f32.ptr, io_bytes, hipMemcpyDeviceToHost, s.stream));
    HIP_TRY(hipStreamSynchronize(s.stream));
    s.d2h_bytes += io_bytes;
    std::memcpy(out, s.bounce_out.ptr, io_bytes);
    return RNB_HIP_OK;
}

}  // namespace

extern "C" {

int rnb_hip_dense_q4k_silu_ffn_batch(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len,
                                     const uint8_t *down, size_t down_len, uint32_t down_quant, size_t n_ff,
                                     size_t n_embd, size_t seq_len, const float *x, size_t x_len, float *out,
                                     size_t out_len) {
    int st = validate_dense_ffn(gate_len, up_len, down_len, down_quant, n_ff, n_embd, seq_len, x_len, true);
    if (st != RNB_HIP_OK) return st;
    return dense_ffn_host(gate, gate_len, up, up_len, down, down_len, down_quant, n_ff, n_embd, seq_len, x, out, out_len,
                          false);
}

int rnb_hip_dense_q4k_gelu_ffn_batch(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len,
                                     const uint8_t *down, size_t down_len, uint32_t down_quant, size_t n_ff,
                                     size_t n_embd, size_t seq_len, const float *x, size_t x_len, float *out,
                                     size_t out_len) {
    int st = validate_dense_ffn(gate_len, up_len, down_len, down_quant, n_ff, n_embd, seq_len, x_len, true, true);
    if (st != RNB_HIP_OK) return st;
    return dense_ffn_host(gate, gate_len, up, up_len, down, down_len, down_quant, n_ff, n_embd, seq_len, x, out, out_len,
                          true);
}

int rnb_hip_dense_q4k_gelu_ffn(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len, const uint8_t *down,
                               size_t down_len, uint32_t down_quant, size_t n_ff, size_t n_embd, const float *x,
                               size_t x_len, float *out, size_t out_len) {
    // validation order and texts: crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:191-232
    if (x_len != n_embd)
        return fail(RNB_HIP_INVALID_REQUEST, "dense GELU FFN input length mismatch: got " + std::to_string(x_len) +
                                                 ", expected " + std::to_string(n_embd));
    if (n_embd % 256 != 0 || n_ff % 256 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "dense GELU FFN dims must be divisible by 256, got n_ff=" +
                                                 std::to_string(n_ff) + " n_embd=" + std::to_string(n_embd));
    size_t down_row_bytes = 0;
    switch (down_quant) {
        case 12: down_row_bytes = n_ff / 256 * 144; break;
        case 13: down_row_bytes = n_ff / 256 * 176; break;
        case 14: down_row_bytes = n_ff / 256 * 210; break;
        default:
            return fail(RNB_HIP_INVALID_REQUEST, "unsupported dense GELU FFN down quant code " + std::to_string(down_quant));
    }
    const size_t gate_bytes = n_ff * (n_embd / 256) * 144;
    if (gate_len != gate_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, "dense GELU FFN gate byte mismatch: got " + std::to_string(gate_len) +
                                                 ", expected " + std::to_string(gate_bytes));
    if (up_len != gate_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, "dense GELU FFN up byte mismatch: got " + std::to_string(up_len) +
                                                 ", expected " + std::to_string(gate_bytes));
    if (down_len != n_embd * down_row_bytes)
        return fail(RNB_HIP_INVALID_REQUEST, "dense GELU FFN down byte mismatch: got " + std::to_string(down_len) +
                                                 ", expected " + std::to_string(n_embd * down_row_bytes));
    if (n_ff > 0x7fffffffu || n_embd > 0x7fffffffu) return fail(RNB_HIP_INVALID_REQUEST, "dense GELU FFN shape out of range");
    if (n_embd == 0) return RNB_HIP_OK;
    return dense_ffn_host(gate, gate_len, up, up_len, down, down_len, down_quant, n_ff, n_embd, 1, x, out, out_len, true);
}

int rnb_hip_dense_q4k_silu_ffn_dev(const void *gate_dev, const void *up_dev, const void *down_dev, uint32_t down_quant,
                                   size_t n_ff, size_t n_embd, size_t seq_len, const float *x_dev, float *out_dev) {
    const size_t gate_bytes = n_embd % 256 == 0 ? n_ff * (n_embd / 256) * 144 : 0;
    size_t down_bytes = 0;
    switch (down_quant) {
        case 8: down_bytes = n_ff % 32 == 0 ? n_embd * (n_ff / 32) * 34 : 0; break;
        case 12: down_bytes = n_ff % 256 == 0 ? n_embd * (n_ff / 256) * 144 : 0; break;
        case 14: down_bytes = n_ff % 256 == 0 ? n_embd * (n_ff / 256) * 210 : 0; break;
        case 7: down_bytes = n_ff % 32 == 0 ? n_embd * (n_ff / 32) * 24 : 0; break;
        case 13: down_bytes = n_ff % 256 == 0 ? n_embd * (n_ff / 256) * 176 : 0; break;
        default: break;
    }
    int st = validate_dense_ffn(gate_bytes, gate_bytes, down_bytes, down_quant, n_ff, n_embd, seq_len, seq_len * n_embd,
                                false);
    if (st != RNB_HIP_OK) return st;
    if (!gate_dev || !up_dev || !down_dev || !x_dev || !out_dev)
        return fail(RNB_HIP_INVALID_REQUEST, "dense SiLU FFN null device pointer");
    if ((reinterpret_cast<uintptr_t>(gate_dev) | reinterpret_cast<uintptr_t>(up_dev) |
         reinterpret_cast<uintptr_t>(down_dev) | reinterpret_cast<uintptr_t>(x_dev)) & 15u)
        return fail(RNB_HIP_INVALID_REQUEST, "dense SiLU FFN device pointers must be 16-byte aligned");
    if (seq_len == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    return run_dense_ffn_dev(*g.state, static_cast<const uint8_t *>(gate_dev), static_cast<const uint8_t *>(up_dev),
                             static_cast<const uint8_t *>(down_dev), down_quant, n_ff, n_embd, seq_len, x_dev, out_dev);
}

int rnb_hip_gemv_dev(uint32_t quant, const void *w_dev, size_t rows, size_t cols, const float *x_dev, size_t seq_len,
                     float *out_dev) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    if (cols == 0 || cols % qi.elems != 0)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " cols must be divisible by " +
                                                 std::to_string(qi.elems) + ", got " + std::to_string(cols));
    if (!w_dev || !x_dev || !out_dev) return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " null device pointer");
    if ((reinterpret_cast<uintptr_t>(w_dev) | reinterpret_cast<uintptr_t>(x_dev)) & 15u)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " device pointers must be 16-byte aligned");
    if (rows > 0x7fffffffu || cols > 0x7fffffffu || seq_len > 65535u)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " shape out of range");
    if (rows == 0 || seq_len == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    return run_matmul_dev(*g.state, quant, static_cast<const uint8_t *>(w_dev), rows, cols, x_dev, seq_len, out_dev);
}

}  // extern "C"

namespace {

// device address of the no-allocation entry point's scratch array on the state's device (the Guard has made it current)
int static_scratch_ptr(State &s, uint8_t **out) {
    void *p = nullptr;
    const hipError_t e = static_scratch_address(s.device, &p);
    if (e != hipSuccess) return hip_fail("static scratch: hipGetSymbolAddress", e);
    if (p == nullptr) return fail(RNB_HIP_EXECUTION_FAILED, "static scratch: no address for device " + std::to_string(s.device));
    *out = static_cast<uint8_t *>(p);
    return RNB_HIP_OK;
}

// argument checks shared by rnb_hip_gemv_dev and rnb_hip_gemv_dev_noalloc
int validate_gemv_dev(uint32_t quant, const void *w_dev, size_t rows, size_t cols, const float *x_dev, size_t seq_len,
                      const float *out_dev) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    if (cols == 0 || cols % qi.elems != 0)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " cols must be divisible by " +
                                                 std::to_string(qi.elems) + ", got " + std::to_string(cols));
    if (!w_dev || !x_dev || !out_dev) return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " null device pointer");
    if ((reinterpret_cast<uintptr_t>(w_dev) | reinterpret_cast<uintptr_t>(x_dev)) & 15u)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " device pointers must be 16-byte aligned");
    if (rows > 0x7fffffffu || cols > 0x7fffffffu || seq_len > 65535u)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " shape out of range");
    return RNB_HIP_OK;
}

}  // namespace

extern "C" {

size_t rnb_hip_gemv_dev_noalloc_scratch_bytes(void) { return kStaticScratchBytes; }

int rnb_hip_gemv_dev_noalloc(uint32_t quant, const void *w_dev, size_t rows, size_t cols, const float *x_dev,
                             size_t seq_len, float *out_dev) {
    int st = validate_gemv_dev(quant, w_dev, rows, cols, x_dev, seq_len, out_dev);
    if (st != RNB_HIP_OK) return st;
    if (rows == 0 || seq_len == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    Arena arena;
    arena.cap = kStaticScratchBytes;
    arena.who = "rnb_hip_gemv_dev_noalloc";
    st = static_scratch_ptr(*g.state, &arena.base);
    if (st != RNB_HIP_OK) return st;
    return run_matmul_dev(*g.state, quant, static_cast<const uint8_t *>(w_dev), rows, cols, x_dev, seq_len, out_dev, &arena);
}

}  // extern "C"

namespace {

// shared by the three norm entry points: checks, activation scratch for the Q8_K output, launch
int rms_norm_dev(const char *what, const float *input, const float *post_weight, float post_eps, int post_unit,
                 float *residual, const float *weight, float eps, int unit, size_t seq_len, size_t hidden, float *out_f32,
                 bool quantize) {
    const std::string name = what;
    if (hidden == 0 || hidden % 256 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, name + " hidden size must be divisible by 256, got " + std::to_string(hidden));
    if (!input || !weight || (residual && !post_weight) || (!quantize && !out_f32))
        return fail(RNB_HIP_INVALID_REQUEST, name + " null device pointer");
    if ((reinterpret_cast<uintptr_t>(input) | reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(residual) |
         reinterpret_cast<uintptr_t>(post_weight) | reinterpret_cast<uintptr_t>(out_f32)) & 15u)
        return fail(RNB_HIP_INVALID_REQUEST, name + " device pointers must be 16-byte aligned");
    if (hidden > 0x00ffffffu || seq_len > 65535u) return fail(RNB_HIP_INVALID_REQUEST, name + " shape out of range");
    if (seq_len == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    int8_t *qs = nullptr;
    float *d = nullptr;
    int16_t *bsums = nullptr;
    uint8_t *digits = nullptr;
    if (quantize) {
        const size_t n = seq_len * hidden;
        s.act_seq = 0;  // the scratch describes nothing until the launch below is known to have gone out
        RESERVE_TRY(s.act_qs, n);
        RESERVE_TRY(s.act_d, n / 256 * sizeof(float));
        RESERVE_TRY(s.act_bsums, n / 256 * 16 * sizeof(int16_t));
        if (seq_len >= kDigitsMinSeq) {
            RESERVE_TRY(s.act_digits, n / 256 * 16);
            digits = s.act_digits.as<uint8_t>();
        }
        qs = s.act_qs.as<int8_t>();
        d = s.act_d.as<float>();
        bsums = s.act_bsums.as<int16_t>();
    }
    launch_rms_norm(input, post_weight, post_eps, post_unit != 0, residual, weight, eps, unit != 0,
                    static_cast<uint32_t>(seq_len), static_cast<uint32_t>(hidden / 256), out_f32, qs, d, bsums, digits, s.stream);
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    if (quantize) {
        s.act_has_digits = digits != nullptr;
        s.act_family = kQ4K;
        s.act_seq = seq_len;
        s.act_cols = hidden;
    }
    return RNB_HIP_OK;
}

}  // namespace

extern "C" {

int rnb_hip_rms_norm_dev(const float *x_dev, const float *weight_dev, float eps, int unit_offset, size_t seq_len,
                         size_t hidden, float *out_dev) {
    return rms_norm_dev("RMS norm", x_dev, nullptr, 0.0f, 0, nullptr, weight_dev, eps, unit_offset, seq_len, hidden, out_dev,
                        false);
}

int rnb_hip_rms_norm_quantize_dev(const float *x_dev, const float *weight_dev, float eps, int unit_offset, size_t seq_len,
                                  size_t hidden, float *out_dev) {
    return rms_norm_dev("RMS norm + Q8_K", x_dev, nullptr, 0.0f, 0, nullptr, weight_dev, eps, unit_offset, seq_len, hidden,
                        out_dev, true);
}

int rnb_hip_rms_norm_add_rms_norm_quantize_dev(const float *input_dev, const float *post_weight_dev, float post_eps,
                                               int post_unit_offset, float *residual_dev, const float *pre_weight_dev,
                                               float pre_eps, int pre_unit_offset, size_t seq_len, size_t hidden,
                                               float *out_dev) {
    if (!residual_dev) return fail(RNB_HIP_INVALID_REQUEST, "RMS norm + add + RMS norm + Q8_K null device pointer");
    return rms_norm_dev("RMS norm + add + RMS norm + Q8_K", input_dev, post_weight_dev, post_eps, post_unit_offset,
                        residual_dev, pre_weight_dev, pre_eps, pre_unit_offset, seq_len, hidden, out_dev, true);
}

int rnb_hip_moe_route_topk_dev(const float *logits_dev, size_t token_count, size_t n_expert, size_t k, uint32_t *idx_dev,
                               float *weights_dev) {
    if (!logits_dev || !idx_dev || !weights_dev) return fail(RNB_HIP_INVALID_REQUEST, "router null device pointer");
    if (n_expert > 0xffffu || k > 0xffffu || token_count > 0x00ffffffu ||
        !route_topk_supported(static_cast<uint32_t>(n_expert), static_cast<uint32_t>(k)))
        return fail(RNB_HIP_INVALID_REQUEST, "router supports 1..512 experts and top-1..32, got n_expert=" +
                                                 std::to_string(n_expert) + " k=" + std::to_string(k));
    if (token_count == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    launch_route_topk(logits_dev, static_cast<uint32_t>(token_count), static_cast<uint32_t>(n_expert), static_cast<uint32_t>(k),
                      idx_dev, weights_dev, g.state->stream);
    return check_launches();
}

int rnb_hip_quantize_dev(uint32_t quant, const float *x_dev, size_t seq_len, size_t cols) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    if (cols == 0 || cols % qi.elems != 0)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " cols must be divisible by " +
                                                 std::to_string(qi.elems) + ", got " + std::to_string(cols));
    if (!x_dev || (reinterpret_cast<uintptr_t>(x_dev) & 15u))
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " input must be a 16-byte aligned device pointer");
    if (cols > 0x7fffffffu || seq_len > 65535u)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " shape out of range");
    if (seq_len == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    ActView act;
    return quantize_activations(*g.state, quant, x_dev, seq_len, cols, &act);
}

int rnb_hip_gemv_quantized_dev(uint32_t quant, const void *w_dev, size_t rows, size_t cols, size_t seq_len,
                               float *out_dev) {
    QuantInfo qi;
    if (!quant_info(quant, &qi)) return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    if (!w_dev || !out_dev || (reinterpret_cast<uintptr_t>(w_dev) & 15u))
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " weights must be a 16-byte aligned device pointer");
    if (rows > 0x7fffffffu || seq_len > 65535u)
        return fail(RNB_HIP_INVALID_REQUEST, std::string(qi.label) + " shape out of range");
    if (rows == 0 || seq_len == 0) return RNB_HIP_OK;
    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    const uint32_t family = is_block32(quant) ? kQ8_0 : kQ4K;
    if (s.act_family != family || s.act_seq != seq_len || s.act_cols != cols)
        return fail(RNB_HIP_INVALID_REQUEST,
                    std::string(qi.label) + " activation scratch holds seq_len=" + std::to_string(s.act_seq) + " cols=" +
                        std::to_string(s.act_cols) + " family=" + std::to_string(s.act_family) + ", requested seq_len=" +
                        std::to_string(seq_len) + " cols=" + std::to_string(cols));
    return run_matmul_quantized_dev(s, quant, static_cast<const uint8_t *>(w_dev), rows, cols, seq_len, out_dev,
                                    state_act_view(s, quant));
}

int rnb_hip_moe_sparse_experts_by_token_dev(const void *gate_dev, const void *up_dev, const void *down_dev,
                                            size_t n_expert, const void *shared_gate_dev, const void *shared_up_dev,
                                            const void *shared_down_dev, const uint32_t *expert_ids, const float *route_weights,
                                            const uint32_t *token_ids, size_t n_slots, size_t token_count,
                                            uint32_t down_quant, size_t n_ff, size_t n_embd, const float *x_dev,
                                            float *out_dev) {
    if (n_embd == 0 || n_ff == 0 || n_embd % 256 != 0 || n_ff % 256 != 0)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer dims must be divisible by 256, got n_ff=" +
                                                 std::to_string(n_ff) + " n_embd=" + std::to_string(n_embd));
    QuantInfo down_qi;
    if ((down_quant != kQ4K && down_quant != kQ5K && down_quant != kQ6K) || !quant_info(down_quant, &down_qi))
        return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported Qwen35 HIP down quant code " + std::to_string(down_quant));
    const size_t down_block = down_qi.bytes;
    MoeShape sh;
    sh.nb_in = n_embd / 256;
    sh.nb_mid = n_ff / 256;
    sh.per_gate = n_ff * sh.nb_in * kQ4KBytes;
    sh.per_down = n_embd * sh.nb_mid * down_block;
    sh.n_expert = n_expert;
    MoeShape checked;
    SharedLens sl;
    sl.any = shared_gate_dev != nullptr || shared_up_dev != nullptr || shared_down_dev != nullptr;
    sl.all = shared_gate_dev != nullptr && shared_up_dev != nullptr && shared_down_dev != nullptr;
    sl.gate = sl.up = sh.per_gate, sl.down = sh.per_down;  // device tensors carry no length: one expert each
    MoeShared shared;
    if (sl.all) {
        shared.gate = static_cast<const uint8_t *>(shared_gate_dev);
        shared.up = static_cast<const uint8_t *>(shared_up_dev);
        shared.down = static_cast<const uint8_t *>(shared_down_dev);
        shared.n_routed = static_cast<uint32_t>(n_expert);
    }
    int st = validate_moe(n_expert * sh.per_gate, n_expert * sh.per_gate, n_expert * sh.per_down, sl, expert_ids, token_ids,
                          n_slots, token_count, down_quant, n_ff, n_embd, token_count * n_embd, token_count * n_embd,
                          &checked);
    if (st != RNB_HIP_OK) return st;
    if (!gate_dev || !up_dev || !down_dev || !x_dev || !out_dev)
        return fail(RNB_HIP_INVALID_REQUEST, "Qwen35 full-layer null device pointer");
    Guard g;
    if (!g.state) return g.status;
    return run_moe_dev(*g.state, static_cast<const uint8_t *>(gate_dev), static_cast<const uint8_t *>(up_dev),
                       static_cast<const uint8_t *>(down_dev), shared, sh, expert_ids, route_weights, token_ids, n_slots,
                       token_count, down_quant, n_ff, n_embd, x_dev, out_dev);
}

}  // extern "C"

namespace {

// The formats of the embedding gather with the names the reference prints (`{quant:?}` of its QuantFormat) and its
// table of elements and bytes per block: crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:1834-1853.
struct EmbedFormat {
    const char *name;
    size_t elems, bytes;
};
bool embed_format(uint32_t quant, EmbedFormat *f) {
    switch (quant) {
    case kF32: *f = {"F32", 32, 128}; return true;
    case kF16: *f = {"F16", 32, 64}; return true;
    case kBF16: *f = {"BF16", 32, 64}; return true;
    case kQ4_0: *f = {"Q40", 32, kQ4_0Bytes}; return true;
    case kQ4_1: *f = {"Q41", 32, kQ4_1Bytes}; return true;
    case kQ5_0: *f = {"Q50", 32, kQ5_0Bytes}; return true;
    case kQ5_1: *f = {"Q51", 32, kQ5_1Bytes}; return true;
    case kQ8_0: *f = {"Q80", 32, kQ8_0Bytes}; return true;
    case kQ8_1: *f = {"Q81", 32, kQ8_1Bytes}; return true;
    case kQ2K: *f = {"Q2K", 256, kQ2KBytes}; return true;
    case kQ3K: *f = {"Q3K", 256, kQ3KBytes}; return true;
    case kQ4K: *f = {"Q4K", 256, kQ4KBytes}; return true;
    case kQ5K: *f = {"Q5K", 256, kQ5KBytes}; return true;
    case kQ6K: *f = {"Q6K", 256, kQ6KBytes}; return true;
    case kIQ2XXS: *f = {"IQ2XXS", 256, kIQ2XXSBytes}; return true;
    case kIQ2S: *f = {"IQ2S", 256, kIQ2SBytes}; return true;
    case kIQ3XXS: *f = {"IQ3XXS", 256, kIQ3XXSBytes}; return true;
    case kIQ4XS: *f = {"IQ4XS", 256, kIQ4XSBytes}; return true;
    default: return false;
    }
}

// quant_embedding_gather (quant_api.rs:1827-1975): checks and texts in the reference's order (cols, empty id list, id
// range, weight bytes).  A matrix that is resident already (prewarmed, or uploaded by an earlier call) is read where
// it is; otherwise only the rows the ids name travel, one per id, and the kernel reads them in order (the
// reference's compact_embedding_rows).  Output to the host (out_host) or to device memory (out_dev), never both.
int embedding_gather(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols, const uint32_t *token_ids,
                     size_t n_tokens, float *out_host, size_t out_len, float *out_dev) {
    EmbedFormat f;
    if (!embed_format(quant, &f) || !embed_gather_supported(quant))
        return fail(RNB_HIP_UNSUPPORTED_OP, "unsupported quant id " + std::to_string(quant));
    const std::string name = f.name;
    if (cols == 0 || cols % f.elems != 0)
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding cols must be non-zero and divisible by " +
                                                 std::to_string(f.elems) + ", got " + std::to_string(cols));
    if (n_tokens == 0) return RNB_HIP_OK;
    if (!token_ids) return fail(RNB_HIP_INVALID_REQUEST, name + " embedding null pointer argument");
    for (size_t i = 0; i < n_tokens; i++)
        if (token_ids[i] >= rows)
            return fail(RNB_HIP_INVALID_REQUEST, name + " embedding token id " + std::to_string(token_ids[i]) +
                                                     " is out of range for " + std::to_string(rows) + " rows");
    const size_t blocks_per_row = cols / f.elems;
    size_t row_bytes = 0, expected = 0, out_need = 0;
    if (__builtin_mul_overflow(blocks_per_row, f.bytes, &row_bytes) || __builtin_mul_overflow(rows, row_bytes, &expected))
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding weight byte size overflow");
    if (w_len != expected)
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding weight byte mismatch: got " + std::to_string(w_len) +
                                                 ", expected " + std::to_string(expected));
    if (__builtin_mul_overflow(n_tokens, cols, &out_need) || out_need > (~size_t(0)) / sizeof(float))
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding output length overflow");
    if (out_host != nullptr && out_len < out_need)
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding output too small: got " + std::to_string(out_len) +
                                                 ", expected >= " + std::to_string(out_need));
    if (!w || (out_host == nullptr && out_dev == nullptr))
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding null pointer argument");
    if (out_dev != nullptr && (reinterpret_cast<uintptr_t>(out_dev) & 15u))
        return fail(RNB_HIP_INVALID_REQUEST, name + " embedding output must be a 16-byte aligned device pointer");
    if (cols > 0x7fffffffu) return fail(RNB_HIP_INVALID_REQUEST, name + " embedding shape out of range");

    Guard g;
    if (!g.state) return g.status;
    State &s = *g.state;
    if (s.capturing())
        return fail(RNB_HIP_INVALID_REQUEST, "host-pointer weights cannot be resolved while the library stream is capturing");
    const size_t ids_bytes = n_tokens * sizeof(uint32_t), out_bytes = out_need * sizeof(float);
    const uint8_t *w_dev = nullptr;
    const uint32_t *ids_dev = nullptr;
    if (s.resident_peek(w, w_len, &w_dev)) {
        RESERVE_TRY(s.bounce_in, ids_bytes);
        HIP_TRY(s.gather_ids.reserve(ids_bytes));
        std::memcpy(s.bounce_in.ptr, token_ids, ids_bytes);
        HIP_TRY(hipMemcpyAsync(s.gather_ids.ptr, s.bounce_in.ptr, ids_bytes, hipMemcpyHostToDevice, s.stream));
        s.h2d_bytes += ids_bytes;
        ids_dev = s.gather_ids.as<uint32_t>();
    } else {
        size_t compact_bytes = 0;
        if (__builtin_mul_overflow(n_tokens, row_bytes, &compact_bytes))
            return fail(RNB_HIP_INVALID_REQUEST, name + " embedding row byte size overflow");
        RESERVE_TRY(s.bounce_in, compact_bytes);
        HIP_TRY(s.gather_rows.reserve(compact_bytes));
        uint8_t *stage = static_cast<uint8_t *>(s.bounce_in.ptr);
        for (size_t i = 0; i < n_tokens; i++) std::memcpy(stage + i * row_bytes, w + token_ids[i] * row_bytes, row_bytes);
        HIP_TRY(hipMemcpyAsync(s.gather_rows.ptr, stage, compact_bytes, hipMemcpyHostToDevice, s.stream));
        s.h2d_bytes += compact_bytes;
        w_dev = s.gather_rows.as<uint8_t>();
    }
    float *dst = out_dev;
    if (dst == nullptr) {
        HIP_TRY(s.out_f32.reserve(out_bytes));
        dst = s.out_f32.as<float>();
    }
    for (size_t t0 = 0; t0 < n_tokens; t0 += 65535) {  // grid.y carries the token
        const uint32_t n = static_cast<uint32_t>(std::min<size_t>(65535, n_tokens - t0));
        launch_embed_gather(quant, ids_dev ? w_dev : w_dev + t0 * row_bytes, row_bytes, ids_dev ? ids_dev + t0 : nullptr, n,
                            static_cast<uint32_t>(cols), dst + t0 * cols, s.stream);
    }
    if (int ls = check_launches(); ls != RNB_HIP_OK) return ls;
    if (out_host != nullptr) {
        RESERVE_TRY(s.bounce_out, out_bytes);
        HIP_TRY(hipMemcpyAsync(s.bounce_out.ptr, dst, out_bytes, hipMemcpyDeviceToHost, s.stream));
        HIP_TRY(hipStreamSynchronize(s.stream));
        s.d2h_bytes += out_bytes;
        std::memcpy(out_host, s.bounce_out.ptr, out_bytes);
    } else {
        // the ids (or rows) went through the shared pinned buffer: the next call may refill it, so the copy must be done
        HIP_TRY(hipStreamSynchronize(s.stream));
    }
    return RNB_HIP_OK;
}

}  // namespace

extern "C" {

int rnb_hip_quant_embedding_gather(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                                   const uint32_t *token_ids, size_t n_tokens, float *out, size_t out_len) {
    return embedding_gather(quant, w, w_len, rows, cols, token_ids, n_tokens, out, out_len, nullptr);
}

int rnb_hip_quant_embedding_gather_dev(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                                       const uint32_t *token_ids, size_t n_tokens, float *out_dev) {
    return embedding_gather(quant, w, w_len, rows, cols, token_ids, n_tokens, nullptr, 0, out_dev);
}

}  // extern "C"
