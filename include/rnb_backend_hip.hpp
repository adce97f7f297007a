// rnb_backend_hip.hpp -- C++ host-side mirror of the reference's operator interface over the C ABI
// in rnb_hip.h.  The reference's host code is Rust; with no Rust toolchain available this header
// restates, name for name, the free functions a `rnb-backend-hip` crate would export:
//
//   q4k_gemv / q4k_gemv_into / q4k_gemv_batch   crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:183-238, 2283-2319
//   q4_0 / q4_1 / q5_0 / q5_1 _gemv (+ _batch)  quant_api.rs:374-496
//   q8_1_gemv (+ _batch)                         quant_api.rs:507-541
//   iq2_xxs / iq2_s / iq3_xxs / iq4_xs _gemv (+ _batch)  quant_api.rs:543-722
//   q2k_gemv / q3k_gemv (+ _batch)              quant_api.rs:73-181
//   q5k_gemv / q5k_gemv_into / q5k_gemv_batch   quant_api.rs:2207-2281, 3957-3993
//   q6k_gemv / q6k_gemv_into / q6k_gemv_batch   quant_api.rs:2071-2168, 3919-3955
//   q8_0_gemv / q8_0_gemv_batch                 quant_api.rs:498-505, 807-822
//   q8_0_head_gemv_batch                        quant_api.rs:824-882
//   q6k_gemv_argmax / q8_0_gemv_argmax          quant_api.rs:2170-2204, 733-768
//   qwen35_sparse_experts_selected_base_by_token  api/qwen_moe_api.rs:2529-2541
//   dense_q4k_silu_ffn_batch                    api/dense_api.rs:297-337
//   dense_q4k_gelu_ffn / dense_q4k_gelu_ffn_batch  api/dense_api.rs:182-293
//   dense_q4k_attention_qkv                     api/dense_api.rs:916-985
//   GgufFile                                    crates/rnb-loader/src/gguf/parser.rs:16-24, 247-407
//   HipBackend                                  crates/rnb-backend/api/src/lib.rs:1281-1285 (trait Backend)
//
// `Result<T, String>` becomes rnb_hip::Result<T>: either a value or the reference's error message.
#pragma once

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

#include "rnb_hip.h"

namespace rnb_hip {

template <typename T>
struct Result {
    bool ok = false;
    T value{};
    int status = RNB_HIP_OK;  // rnb_hip_status
    std::string error;
    explicit operator bool() const { return ok; }
};

struct Unit {};

template <typename T>
inline Result<T> make_err(int status) {
    Result<T> r;
    r.status = status;
    r.error = rnb_hip_last_error();
    return r;
}
template <typename T>
inline Result<T> make_ok(T v) {
    Result<T> r;
    r.ok = true;
    r.value = std::move(v);
    return r;
}

// borrowed byte / float ranges (the reference's &[u8] / &[f32])
struct Bytes {
    const uint8_t *ptr;
    size_t len;
};
struct Floats {
    const float *ptr;
    size_t len;
};

using MatmulFn = int (*)(const uint8_t *, size_t, size_t, size_t, const float *, size_t, float *, size_t);

inline Result<std::vector<float>> gemv_impl(MatmulFn fn, Bytes w, size_t rows, size_t cols, Floats x, size_t out_n) {
    std::vector<float> out(out_n);
    const int st = fn(w.ptr, w.len, rows, cols, x.ptr, x.len, out.data(), out.size());
    if (st != RNB_HIP_OK) return make_err<std::vector<float>>(st);
    return make_ok(std::move(out));
}
inline Result<Unit> gemv_into_impl(MatmulFn fn, Bytes w, size_t rows, size_t cols, Floats x, float *out, size_t out_len) {
    const int st = fn(w.ptr, w.len, rows, cols, x.ptr, x.len, out, out_len);
    if (st != RNB_HIP_OK) return make_err<Unit>(st);
    return make_ok(Unit{});
}
inline size_t batch_seq(Floats x, size_t cols) { return (cols != 0 && x.len % cols == 0) ? x.len / cols : 0; }

inline Result<std::vector<float>> q4k_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q4k_gemv, weights, rows, cols, input, rows);
}
inline Result<Unit> q4k_gemv_into(Bytes weights, size_t rows, size_t cols, Floats input, float *output, size_t output_len) {
    return gemv_into_impl(rnb_hip_q4k_gemv, weights, rows, cols, input, output, output_len);
}
inline Result<std::vector<float>> q4k_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q4k_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);
}
// dense_q4k_attention_qkv(q_weights, k_weights, v_weights, q_rows, kv_rows, n_embd, input, q, k, v), api/dense_api.rs:916-985
inline Result<Unit> dense_q4k_attention_qkv(Bytes q_weights, Bytes k_weights, Bytes v_weights, size_t q_rows, size_t kv_rows,
                                            size_t n_embd, Floats input, float *q, size_t q_len, float *k, size_t k_len,
                                            float *v, size_t v_len) {
    const int st = rnb_hip_dense_q4k_attention_qkv(q_weights.ptr, q_weights.len, k_weights.ptr, k_weights.len, v_weights.ptr,
                                                   v_weights.len, q_rows, kv_rows, n_embd, input.ptr, input.len, q, q_len, k,
                                                   k_len, v, v_len);
    if (st != RNB_HIP_OK) return make_err<Unit>(st);
    return make_ok(Unit{});
}
// q6k_gemv_argmax / q8_0_gemv_argmax -> (row index, value), quant_api.rs:2170-2204, 733-768
inline Result<std::pair<uint32_t, float>> q6k_gemv_argmax(Bytes weights, size_t rows, size_t cols, Floats input) {
    std::pair<uint32_t, float> best{0, 0.0f};
    const int st = rnb_hip_q6k_gemv_argmax(weights.ptr, weights.len, rows, cols, input.ptr, input.len, &best.first, &best.second);
    if (st != RNB_HIP_OK) return make_err<std::pair<uint32_t, float>>(st);
    return make_ok(best);
}
inline Result<std::pair<uint32_t, float>> q8_0_gemv_argmax(Bytes weights, size_t rows, size_t cols, Floats input) {
    std::pair<uint32_t, float> best{0, 0.0f};
    const int st = rnb_hip_q8_0_gemv_argmax(weights.ptr, weights.len, rows, cols, input.ptr, input.len, &best.first, &best.second);
    if (st != RNB_HIP_OK) return make_err<std::pair<uint32_t, float>>(st);
    return make_ok(best);
}
// q8_0_gemv_argmax_q8dot, quant_api.rs:770-805
inline Result<std::pair<uint32_t, float>> q8_0_gemv_argmax_q8dot(Bytes weights, size_t rows, size_t cols, Floats input) {
    std::pair<uint32_t, float> best{0, 0.0f};
    const int st = rnb_hip_q8_0_gemv_argmax_q8dot(weights.ptr, weights.len, rows, cols, input.ptr, input.len, &best.first, &best.second);
    if (st != RNB_HIP_OK) return make_err<std::pair<uint32_t, float>>(st);
    return make_ok(best);
}
#define RNB_HIP_BLOCK32_MIRROR(name)                                                                               \
    inline Result<std::vector<float>> name##_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {         \
        return gemv_impl(rnb_hip_##name##_gemv, weights, rows, cols, input, rows);                                 \
    }                                                                                                              \
    inline Result<std::vector<float>> name##_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {   \
        return gemv_impl(rnb_hip_##name##_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);  \
    }
RNB_HIP_BLOCK32_MIRROR(q4_0)
RNB_HIP_BLOCK32_MIRROR(q4_1)
RNB_HIP_BLOCK32_MIRROR(q5_0)
RNB_HIP_BLOCK32_MIRROR(q5_1)
RNB_HIP_BLOCK32_MIRROR(q8_1)
// iq2_xxs_gemv / iq2_s_gemv / iq3_xxs_gemv / iq4_xs_gemv (+ _batch), quant_api.rs:543-722: the same shape of function
RNB_HIP_BLOCK32_MIRROR(iq2_xxs)
RNB_HIP_BLOCK32_MIRROR(iq2_s)
RNB_HIP_BLOCK32_MIRROR(iq3_xxs)
RNB_HIP_BLOCK32_MIRROR(iq4_xs)
#undef RNB_HIP_BLOCK32_MIRROR
// quant_embedding_gather(quant, weights, rows, cols, token_ids), quant_api.rs:1827-1975; `quant` is the ggml type id
// (RNB_GGML_*), the reference's QuantFormat value
inline Result<std::vector<float>> quant_embedding_gather(uint32_t quant, Bytes weights, size_t rows, size_t cols,
                                                         const std::vector<uint32_t> &token_ids) {
    std::vector<float> out(token_ids.size() * cols);
    const int st = rnb_hip_quant_embedding_gather(quant, weights.ptr, weights.len, rows, cols, token_ids.data(),
                                                  token_ids.size(), out.data(), out.size());
    if (st != RNB_HIP_OK) return make_err<std::vector<float>>(st);
    return make_ok(std::move(out));
}
inline Result<std::vector<float>> q2k_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q2k_gemv, weights, rows, cols, input, rows);
}
inline Result<std::vector<float>> q2k_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q2k_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);
}
inline Result<std::vector<float>> q3k_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q3k_gemv, weights, rows, cols, input, rows);
}
inline Result<std::vector<float>> q3k_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q3k_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);
}
inline Result<std::vector<float>> q5k_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q5k_gemv, weights, rows, cols, input, rows);
}
inline Result<Unit> q5k_gemv_into(Bytes weights, size_t rows, size_t cols, Floats input, float *output, size_t output_len) {
    return gemv_into_impl(rnb_hip_q5k_gemv, weights, rows, cols, input, output, output_len);
}
inline Result<std::vector<float>> q5k_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q5k_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);
}
inline Result<std::vector<float>> q6k_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q6k_gemv, weights, rows, cols, input, rows);
}
inline Result<Unit> q6k_gemv_into(Bytes weights, size_t rows, size_t cols, Floats input, float *output, size_t output_len) {
    return gemv_into_impl(rnb_hip_q6k_gemv, weights, rows, cols, input, output, output_len);
}
inline Result<std::vector<float>> q6k_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q6k_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);
}
inline Result<std::vector<float>> q8_0_gemv(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q8_0_gemv, weights, rows, cols, input, rows);
}
inline Result<std::vector<float>> q8_0_gemv_batch(Bytes weights, size_t rows, size_t cols, Floats input) {
    return gemv_impl(rnb_hip_q8_0_gemv_batch, weights, rows, cols, input, batch_seq(input, cols) * rows);
}
// q8_0_head_gemv_batch(weights, head_count, rows_per_head, cols, token_count, input), quant_api.rs:824-882
inline Result<std::vector<float>> q8_0_head_gemv_batch(Bytes weights, size_t head_count, size_t rows_per_head, size_t cols,
                                                       size_t token_count, Floats input) {
    std::vector<float> out(token_count * head_count * rows_per_head);
    const int st = rnb_hip_q8_0_head_gemv_batch(weights.ptr, weights.len, head_count, rows_per_head, cols, token_count,
                                                input.ptr, input.len, out.data(), out.size());
    if (st != RNB_HIP_OK) return make_err<std::vector<float>>(st);
    return make_ok(std::move(out));
}

// prewarm_q4k_weights(&[&[u8]]), quant_api.rs:952
inline Result<Unit> prewarm_weights(const std::vector<Bytes> &ranges) {
    std::vector<const uint8_t *> ptrs;
    std::vector<size_t> lens;
    for (const Bytes &b : ranges) {
        ptrs.push_back(b.ptr);
        lens.push_back(b.len);
    }
    const int st = rnb_hip_prewarm(ptrs.data(), lens.data(), ptrs.size());
    if (st != RNB_HIP_OK) return make_err<Unit>(st);
    return make_ok(Unit{});
}

inline Result<std::vector<float>> qwen35_sparse_experts_selected_base_by_token(
    Bytes gate_all, Bytes up_all, Bytes down_all, const std::vector<uint32_t> &expert_ids,
    const std::vector<float> &route_weights, const std::vector<uint32_t> &token_ids, size_t token_count,
    uint32_t down_quant, size_t n_ff, size_t n_embd, Floats input, Bytes shared_gate = Bytes{}, Bytes shared_up = Bytes{},
    Bytes shared_down = Bytes{}) {
    // shared_*: the shared expert (slot id n_expert with the shared gate's scalar as its weight, the extra slot of the
    // decode call in crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:804-812); empty = none
    if (route_weights.size() != expert_ids.size() || token_ids.size() != expert_ids.size()) {
        Result<std::vector<float>> r;
        r.status = RNB_HIP_INVALID_REQUEST;
        r.error = "Qwen35 full-layer token-batch length mismatch: expert=" + std::to_string(expert_ids.size()) +
                  " route=" + std::to_string(route_weights.size()) + " token=" + std::to_string(token_ids.size());
        return r;
    }
    std::vector<float> out(token_count * n_embd);
    const int st = rnb_hip_moe_sparse_experts_by_token(
        gate_all.ptr, gate_all.len, up_all.ptr, up_all.len, down_all.ptr, down_all.len, shared_gate.ptr, shared_gate.len,
        shared_up.ptr, shared_up.len, shared_down.ptr, shared_down.len, expert_ids.data(),
        route_weights.data(), token_ids.data(), expert_ids.size(), token_count, down_quant, n_ff, n_embd, input.ptr,
        input.len, out.data(), out.size());
    if (st != RNB_HIP_OK) return make_err<std::vector<float>>(st);
    return make_ok(std::move(out));
}

// dense_q4k_silu_ffn_batch, crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:297-337
inline Result<std::vector<float>> dense_q4k_silu_ffn_batch(Bytes gate_weights, Bytes up_weights, Bytes down_weights,
                                                           uint32_t down_quant, size_t n_ff, size_t n_embd,
                                                           size_t seq_len, Floats input) {
    std::vector<float> out(seq_len * n_embd);
    const int st = rnb_hip_dense_q4k_silu_ffn_batch(gate_weights.ptr, gate_weights.len, up_weights.ptr, up_weights.len,
                                                    down_weights.ptr, down_weights.len, down_quant, n_ff, n_embd, seq_len,
                                                    input.ptr, input.len, out.data(), out.size());
    return st == RNB_HIP_OK ? make_ok(std::move(out)) : make_err<std::vector<float>>(st);
}
inline Result<std::vector<float>> dense_q4k_gelu_ffn_batch(Bytes gate_weights, Bytes up_weights, Bytes down_weights,
                                                           uint32_t down_quant, size_t n_ff, size_t n_embd,
                                                           size_t seq_len, Floats input) {
    std::vector<float> out(seq_len * n_embd);
    const int st = rnb_hip_dense_q4k_gelu_ffn_batch(gate_weights.ptr, gate_weights.len, up_weights.ptr, up_weights.len,
                                                    down_weights.ptr, down_weights.len, down_quant, n_ff, n_embd, seq_len,
                                                    input.ptr, input.len, out.data(), out.size());
    return st == RNB_HIP_OK ? make_ok(std::move(out)) : make_err<std::vector<float>>(st);
}
inline Result<std::vector<float>> dense_q4k_gelu_ffn(Bytes gate_weights, Bytes up_weights, Bytes down_weights, uint32_t down_quant,
                                                    size_t n_ff, size_t n_embd, Floats input) {
    std::vector<float> out(n_embd);
    const int st = rnb_hip_dense_q4k_gelu_ffn(gate_weights.ptr, gate_weights.len, up_weights.ptr, up_weights.len,
                                              down_weights.ptr, down_weights.len, down_quant, n_ff, n_embd, input.ptr,
                                              input.len, out.data(), out.size());
    if (st != RNB_HIP_OK) return make_err<std::vector<float>>(st);
    return make_ok(std::move(out));
}

// trait Backend { kind, capabilities, execute }, crates/rnb-backend/api/src/lib.rs:1281-1285
struct BackendCapabilities {
    bool matmul, attention, gdn, moe, sampler;
};
class HipBackend {
  public:
    int kind() const { return rnb_hip_backend_kind(); }
    BackendCapabilities capabilities() const {
        return {rnb_hip_backend_supports(RNB_OP_MATMUL) != 0, rnb_hip_backend_supports(RNB_OP_ATTENTION) != 0,
                rnb_hip_backend_supports(RNB_OP_GDN) != 0, rnb_hip_backend_supports(RNB_OP_MOE) != 0,
                rnb_hip_backend_supports(RNB_OP_SAMPLER) != 0};
    }
    // Like CudaBackend::execute (crates/rnb-backend/cuda/src/lib.rs:193-195): requests are not executed through
    // the trait; the operator functions above do the work.
    Result<Unit> execute(int /*op*/) const {
        Result<Unit> r;
        r.status = RNB_HIP_UNSUPPORTED_OP;
        r.error = "HipBackend::execute: requests are served by the operator functions";
        return r;
    }
};

// GGUFFile (crates/rnb-loader/src/gguf/parser.rs:16-24) over the C ABI: the handle owns the file mapping, tensors are
// views into it.  `open` = parse + map_tensors (crates/rnb-loader/src/convert.rs:99-178).
struct GgufTensorView {
    std::string name;
    std::vector<uint64_t> shape;  // row-major
    uint32_t ggml_type = 0;
    uint64_t file_offset = 0;
    Bytes bytes{nullptr, 0};      // the tensor's block bytes inside the mapping
    size_t index = 0;
};

class GgufFile {
  public:
    GgufFile() = default;
    GgufFile(const GgufFile &) = delete;
    GgufFile &operator=(const GgufFile &) = delete;
    GgufFile(GgufFile &&o) noexcept : h_(o.h_) { o.h_ = nullptr; }
    GgufFile &operator=(GgufFile &&o) noexcept {
        if (this != &o) {
            rnb_hip_gguf_close(h_);
            h_ = o.h_;
            o.h_ = nullptr;
        }
        return *this;
    }
    ~GgufFile() { rnb_hip_gguf_close(h_); }

    static Result<GgufFile> open(const std::string &path) {
        Result<GgufFile> r;
        r.status = rnb_hip_gguf_open(path.c_str(), &r.value.h_);
        return finish(std::move(r));
    }
    static Result<GgufFile> parse(Bytes data) {  // borrows `data`
        Result<GgufFile> r;
        r.status = rnb_hip_gguf_parse(data.ptr, data.len, &r.value.h_);
        return finish(std::move(r));
    }
    uint32_t version() const { return rnb_hip_gguf_version(h_); }
    uint64_t alignment() const { return rnb_hip_gguf_alignment(h_); }
    uint64_t data_start() const { return rnb_hip_gguf_data_start(h_); }
    size_t tensor_count() const { return rnb_hip_gguf_tensor_count(h_); }
    Result<GgufTensorView> tensor(size_t index) const {
        rnb_hip_gguf_tensor t;
        const int st = rnb_hip_gguf_tensor_at(h_, index, &t);
        if (st != RNB_HIP_OK) return make_err<GgufTensorView>(st);
        GgufTensorView v;
        v.name = t.name;
        v.shape.assign(t.shape, t.shape + t.n_dims);
        v.ggml_type = t.ggml_type;
        v.file_offset = t.file_offset;
        v.bytes = Bytes{t.data, t.data != nullptr ? static_cast<size_t>(t.n_bytes) : 0};
        v.index = index;
        return make_ok(std::move(v));
    }
    Result<GgufTensorView> tensor(const std::string &name) const {
        for (size_t i = 0, n = tensor_count(); i < n; i++) {
            Result<GgufTensorView> r = tensor(i);
            if (r && r.value.name == name) return r;
        }
        Result<GgufTensorView> r;
        r.status = RNB_HIP_INVALID_REQUEST;
        r.error = "missing tensor: " + name;
        return r;
    }
    std::string metadata_str(const std::string &key) const {
        const char *s = rnb_hip_gguf_metadata_str(h_, key.c_str());
        return s != nullptr ? s : "";
    }
    Result<uint64_t> metadata_u64(const std::string &key) const {
        uint64_t v = 0;
        const int st = rnb_hip_gguf_metadata_u64(h_, key.c_str(), &v);
        return st == RNB_HIP_OK ? make_ok(v) : make_err<uint64_t>(st);
    }
    // untouched upload of one tensor, pinned in the resident table
    Result<Unit> prewarm(size_t index) const {
        const int st = rnb_hip_gguf_prewarm_tensor(h_, index);
        return st == RNB_HIP_OK ? make_ok(Unit{}) : make_err<Unit>(st);
    }

  private:
    static Result<GgufFile> finish(Result<GgufFile> r) {
        r.ok = r.status == RNB_HIP_OK;
        if (!r.ok) r.error = rnb_hip_last_error();
        return r;
    }
    rnb_hip_gguf *h_ = nullptr;
};

}  // namespace rnb_hip
