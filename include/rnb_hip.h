/*
 * rnb_hip.h -- C ABI of the MI355X (gfx950) backend for runNburn's quantized matmul path.
 *
 * Every entry point states the reference interface it replaces (paths relative to the
 * reference checkout).  The ABI uses plain pointers and sizes only; all functions return an
 * rnb_hip_status and leave a message retrievable with rnb_hip_last_error() (thread-local).
 *
 * Semantics are those of the reference's rnb-cpu crate: activations are quantised on the
 * device to Q8_K (256-wide, crates/rnb-cpu/src/gemm/activation_q8.rs:149-173) for the K-quant
 * weights (Q2_K ... Q6_K) and to the 32-wide f32-scale Q8 block (:14-32) for the 32-element formats; weight blocks are
 * consumed exactly as stored in GGUF (18 ... 34 / 84 / 110 / 144 / 176 / 210 bytes, no repack, no requantisation).
 *
 * Threading model (crates/rnb-backend/cuda/src/runtime.rs:9): one process-global state behind
 * a mutex, opened lazily on first use, one device, one stream.  Host-pointer entry points
 * block until the result is in the caller's buffer.  `_dev` entry points only enqueue on the
 * library stream (rnb_hip_stream()) and return.
 */
#ifndef RNB_HIP_H
#define RNB_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Error classes of crates/rnb-backend/api/src/lib.rs:55-108 (BackendErrorKind) plus NO_DEVICE so
 * that callers can skip like crates/rnb-backend/cuda/src/runtime/tests.rs:22831-22834. */
typedef enum {
    RNB_HIP_OK = 0,
    RNB_HIP_INVALID_REQUEST = 1,
    RNB_HIP_UNSUPPORTED_OP = 2,
    RNB_HIP_EXECUTION_FAILED = 3,
    RNB_HIP_NO_DEVICE = 4
} rnb_hip_status;

/* ggml type ids, crates/rnb-loader/src/gguf/types.rs:5-41 */
#define RNB_GGML_Q4_0 2u
#define RNB_GGML_Q4_1 3u
#define RNB_GGML_Q5_0 6u
#define RNB_GGML_Q5_1 7u
#define RNB_GGML_Q8_1 9u
#define RNB_GGML_Q8_0 8u
#define RNB_GGML_Q2_K 10u
#define RNB_GGML_Q3_K 11u
#define RNB_GGML_Q4_K 12u
#define RNB_GGML_Q5_K 13u
#define RNB_GGML_Q6_K 14u
#define RNB_GGML_IQ2_XXS 16u
#define RNB_GGML_IQ3_XXS 18u
#define RNB_GGML_IQ2_S 22u
#define RNB_GGML_IQ4_XS 23u
/* float formats: embedding tables only (rnb_hip_quant_embedding_gather) */
#define RNB_GGML_F32 0u
#define RNB_GGML_F16 1u
#define RNB_GGML_BF16 30u

/* BackendOp, crates/rnb-backend/api/src/lib.rs:12-18 */
#define RNB_OP_MATMUL 0
#define RNB_OP_ATTENTION 1
#define RNB_OP_GDN 2
#define RNB_OP_MOE 3
#define RNB_OP_SAMPLER 4

/* ---- trait facade: crates/rnb-backend/api/src/lib.rs:1281-1285 (trait Backend) ------------ */
/* kind(): the reference's BackendKind (:2-9) has no HIP variant; this returns the ordinal a new
 * `Hip` variant appended to that enum would take (6). */
int rnb_hip_backend_kind(void);
/* capabilities(): 1 when `op` (RNB_OP_*) executes on this backend, else 0. */
int rnb_hip_backend_supports(int op);
/* 1 when (op, ggml quant id) is supported: MatMul x {Q4_0,Q4_1,Q5_0,Q5_1,Q8_0,Q8_1,Q2_K..Q6_K,IQ2_XXS,IQ2_S,IQ3_XXS,IQ4_XS}; MoE x gate/up Q4_K with
 * down Q4_K|Q5_K|Q6_K (pass the down quant). */
int rnb_hip_backend_supports_quant(int op, uint32_t quant);

/* ---- lifecycle / diagnostics -------------------------------------------------------------- */
/* CudaState::open (crates/rnb-backend/cuda/src/runtime/state/init.rs:75-118): opens device
 * RNB_HIP_DEVICE (default 0) lazily; explicit call returns RNB_HIP_NO_DEVICE when none opens. */
int rnb_hip_init(void);
const char *rnb_hip_last_error(void);
int rnb_hip_device_name(char *buf, size_t buf_len);
/* cuStreamSynchronize at the end of every reference call (runtime/gemv.rs:285-295) */
int rnb_hip_sync(void);
/* DeviceTransferCounters, crates/rnb-backend/api/src/lib.rs:213-242 */
int rnb_hip_transfer_counters(uint64_t *h2d_bytes, uint64_t *d2h_bytes);
/* the library's only stream, as a hipStream_t */
void *rnb_hip_stream(void);

/* ---- calibration for the benchmark's roofline lines (no counterpart in the reference) ------------
 * rnb_hip_calib_read enqueues a kernel that only reads `bytes` of device memory (16-byte loads, optionally
 * non-temporal); rnb_hip_calib_mfma_i8 one that only issues v_mfma_i32_32x32x32_i8 (`workgroups` x 8 waves x 4 chains x
 * `iters`) and reports the integer operations it performs.  Both run on the library stream and do not synchronise. */
int rnb_hip_calib_read(const void *dev, size_t bytes, int non_temporal);
int rnb_hip_calib_mfma_i8(uint32_t iters, uint32_t workgroups, uint64_t *ops);

/* ---- weight residency: crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:399-405,757-851 */
/* prewarm_q4k_weights (api/quant_api.rs:952): upload host ranges untouched and keep them
 * resident, keyed by (pointer, length, sampled fingerprint).  Sub-ranges of a resident range
 * resolve to parent + offset (q4k_cache.rs:722-741). */
int rnb_hip_prewarm(const uint8_t *const *ptrs, const size_t *lens, size_t n);
/* drop a resident range (call before unmapping the host bytes) */
int rnb_hip_release(const uint8_t *ptr, size_t len);
int rnb_hip_resident_bytes(uint64_t *bytes, uint64_t *entries);
/* Residency policy (crates/rnb-memory/src/byte_lru.rs:32-91, sparse_expert_cache.rs:221-250 and :272-395,
 * crates/rnb-backend/cuda/src/runtime/state/q4k_cache.rs:1055-1079, :1263-1459): host ranges that are not prewarmed
 * stay resident least-recently-used inside a byte budget (85 % of the HBM free at open, RNB_HIP_RESIDENT_BUDGET_MB, or
 * rnb_hip_set_resident_budget).  A missing range that fits only by evicting others is kept when
 * bytes * (decayed earlier lookups + 1) > bytes + evicted bytes, else uploaded for that call alone; a call never
 * evicts what it has itself resolved, nor prewarmed ranges; on a device out-of-memory further ranges are evicted and
 * the allocation retried.
 * rnb_hip_residency_stats fills up to 12 counters, the fields of ExpertBundleCacheStats (sparse_expert_cache.rs:383-395)
 * as they apply here: lookups, hits, sub-range hits, misses, admissions, evictions, admitted bytes, evicted bytes,
 * resident h2d bytes, per-call (temporary) h2d bytes, out-of-memory retries, and the budget in bytes. */
int rnb_hip_residency_stats(uint64_t *out, size_t n);
int rnb_hip_set_resident_budget(uint64_t bytes);
/* offload_non_pinned_resident_q4k, q4k_cache.rs:276-303: frees every range that is not prewarmed */
int rnb_hip_offload_unpinned(uint64_t *freed_bytes);

/* ---- activation quantisers (bit-exact contract) --------------------------------------------- */
/* quantize_input_q8k, crates/rnb-cpu/src/gemm/activation_q8.rs:109-139: n floats (n % 256 == 0)
 * -> n/256 blocks of {f32 d; i8 qs[256]; i16 bsums[16]} = 292 bytes each, computed on the device. */
int rnb_hip_quantize_q8k(const float *x, size_t n, void *out_blocks, size_t out_bytes);
/* quantize_input_q8, activation_q8.rs:14-32: n floats (n % 32 == 0) -> n/32 blocks of
 * {f32 d; i8 qs[32]} = 36 bytes each. */
int rnb_hip_quantize_q8(const float *x, size_t n, void *out_blocks, size_t out_bytes);

/* ---- operator surface, host in / host out ------------------------------------------------- */
/* q4k_gemv / q4k_gemv_into, crates/rnb-backend/cuda/src/runtime/api/quant_api.rs:183-238,340-365:
 * out[row] = Q4_K row . Q8_K(x);  x_len == cols, out_len >= rows. */
int rnb_hip_q4k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                     size_t x_len, float *out, size_t out_len);
/* q4k_gemv_batch, quant_api.rs:2283-2319: seq_len = x_len / cols, out[s*rows + row],
 * out_len >= seq_len*rows.  seq_len >= 4 (matrices of 16 MB and more) or >= 8 takes the int8-MFMA GEMM. */
int rnb_hip_q4k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                           const float *x, size_t x_len, float *out, size_t out_len);
/* q4_0_gemv, q4_1_gemv, q5_0_gemv, q5_1_gemv and their batch forms, quant_api.rs:374-496 (checks and texts of
 * q5_basic_gemv(_batch), :1983-2075): 18 / 20 / 22 / 24-byte blocks of 32 x the 32-wide Q8 activation, the integer
 * dots of crates/rnb-cpu/src/gemm/neon_dot.rs:83-214 and neon_quant.rs:88-158 */
int rnb_hip_q4_0_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                      size_t x_len, float *out, size_t out_len);
int rnb_hip_q4_0_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                            const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_q4_1_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                      size_t x_len, float *out, size_t out_len);
int rnb_hip_q4_1_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                            const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_q5_0_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                      size_t x_len, float *out, size_t out_len);
int rnb_hip_q5_0_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                            const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_q5_1_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                      size_t x_len, float *out, size_t out_len);
int rnb_hip_q5_1_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                            const float *x, size_t x_len, float *out, size_t out_len);
/* q8_1_gemv / q8_1_gemv_batch, quant_api.rs:507-541 (checks and texts of quant_block_gemv(_batch), :1680-1775):
 * 36-byte blocks {f16 d, f16 s, i8 qs[32]} x the 32-wide Q8 activation; the stored sum s is not read
 * (crates/rnb-cpu/src/gemm/neon_quant.rs:236-253) */
int rnb_hip_q8_1_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                      size_t x_len, float *out, size_t out_len);
int rnb_hip_q8_1_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                            const float *x, size_t x_len, float *out, size_t out_len);
/* q2k_gemv / q3k_gemv and their batch forms, quant_api.rs:73-181 (same three checks and texts): Q2_K (84-byte) and
 * Q3_K (110-byte) rows x Q8_K(x), the block dots of crates/rnb-cpu/src/gemm/avx2_dot.rs:169-375 */
int rnb_hip_q2k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                     size_t x_len, float *out, size_t out_len);
int rnb_hip_q2k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                           const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_q3k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                     size_t x_len, float *out, size_t out_len);
int rnb_hip_q3k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                           const float *x, size_t x_len, float *out, size_t out_len);
/* q4k_gemv_with_device_input / q6k_gemv_with_device_input, quant_api.rs:242-330: one token that already lives on the
 * device (x_dev: cols floats, 16-byte aligned, e.g. the output of rnb_hip_rms_norm_dev) against host-resident weights,
 * result to the host.  Checks and texts in the reference's order: cols, weight bytes, "<fmt> output too small: got {},
 * expected >= {rows}". */
int rnb_hip_q4k_gemv_with_device_input(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                                       const float *x_dev, float *out, size_t out_len);
int rnb_hip_q6k_gemv_with_device_input(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                                       const float *x_dev, float *out, size_t out_len);
/* quant_embedding_gather, quant_api.rs:1827-1975: out[t][cols] = row token_ids[t] of a rows x cols matrix in any of the
 * block formats above or f32 / f16 / bf16 (quant = ggml type id), dequantised to f32 with the float operations of the
 * reference's dequantisers in their order (crates/rnb-cpu/src/quantize/dequant.rs, iq.rs), so the values are theirs bit
 * for bit.  Checks and texts in the reference's order, with its names for the formats (Q4K, Q80, IQ2XXS, ...):
 * "<fmt> embedding cols must be non-zero and divisible by {32|256}, got {}", an empty id list returns at once,
 * "<fmt> embedding token id {} is out of range for {} rows", "<fmt> embedding weight byte mismatch: got {}, expected {}".
 * A matrix that is resident already (rnb_hip_prewarm or an earlier matmul) is read in place; otherwise only the rows
 * named by the ids are uploaded, for this call.  out_len >= n_tokens * cols. */
int rnb_hip_quant_embedding_gather(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                                   const uint32_t *token_ids, size_t n_tokens, float *out, size_t out_len);
/* the same with the result left on the device (out_dev: n_tokens * cols floats, 16-byte aligned; the call returns when
 * the rows are there), where
 * rnb_hip_rms_norm_dev picks it up: launch_quant_embedding_gather_with_weights_dev,
 * crates/rnb-backend/cuda/src/runtime/state/launchers.rs:4062 */
int rnb_hip_quant_embedding_gather_dev(uint32_t quant, const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                                       const uint32_t *token_ids, size_t n_tokens, float *out_dev);
/* iq2_xxs_gemv / iq2_s_gemv / iq3_xxs_gemv / iq4_xs_gemv and their batch forms, quant_api.rs:543-722 (same checks and
 * texts): importance-quant rows (66 / 82 / 98 / 136-byte blocks of 256 elements) x Q8_K(x), the block dots of
 * crates/rnb-cpu/src/gemm/neon_quant.rs:273-411 over the layouts of crates/rnb-cpu/src/quantize/iq.rs:23-116.  Batches
 * of five tokens and more run on the matrix cores (the same integer group sums, one f32 update per block); smaller
 * ones on the GEMV, a decoded block dotted against up to four tokens per pass. */
int rnb_hip_iq2_xxs_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                         size_t x_len, float *out, size_t out_len);
int rnb_hip_iq2_xxs_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                               const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_iq2_s_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                       size_t x_len, float *out, size_t out_len);
int rnb_hip_iq2_s_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                             const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_iq3_xxs_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                         size_t x_len, float *out, size_t out_len);
int rnb_hip_iq3_xxs_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                               const float *x, size_t x_len, float *out, size_t out_len);
int rnb_hip_iq4_xs_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                        size_t x_len, float *out, size_t out_len);
int rnb_hip_iq4_xs_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                              const float *x, size_t x_len, float *out, size_t out_len);
/* q5k_gemv / q5k_gemv_into, quant_api.rs:2207-2281: Q5_K rows (176-byte blocks) x Q8_K(x), the block dot of
 * crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800 */
int rnb_hip_q5k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                     size_t x_len, float *out, size_t out_len);
/* q5k_gemv_batch, quant_api.rs:3957-3993 */
int rnb_hip_q5k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                           const float *x, size_t x_len, float *out, size_t out_len);
/* q6k_gemv / q6k_gemv_into, quant_api.rs:2071-2168 */
int rnb_hip_q6k_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                     size_t x_len, float *out, size_t out_len);
/* q6k_gemv_batch, quant_api.rs:3919-3955 */
int rnb_hip_q6k_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                           const float *x, size_t x_len, float *out, size_t out_len);
/* q8_0_gemv, quant_api.rs:498-505 (validation in q5_basic_gemv :1983-2028); semantics are the
 * Q8 x Q8_0 integer dot of crates/rnb-cpu/src/gemm/neon_dot.rs:376-436 */
int rnb_hip_q8_0_gemv(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x,
                      size_t x_len, float *out, size_t out_len);
/* q8_0_gemv_batch, quant_api.rs:807-822 */
int rnb_hip_q8_0_gemv_batch(const uint8_t *w, size_t w_len, size_t rows, size_t cols,
                            const float *x, size_t x_len, float *out, size_t out_len);
/* q8_0_head_gemv_batch(weights, head_count, rows_per_head, cols, token_count, input) -> Vec<f32>, quant_api.rs:824-882
 * (the per-head projections of the GLM MLA path, crates/rnb-llm/src/engine/models/glm_dsa.rs:95-122): weights
 * [head_count][rows_per_head][cols / 32 blocks of 34 bytes], x [token_count][head_count][cols], out
 * [token_count][head_count * rows_per_head].  Every (token, head) group is the Q8_0 GEMV of that head's rows on that
 * vector (Q8 x Q8_0 integer dots, the bits of rnb_hip_q8_0_gemv on the head's sub-matrix); cols <= 4096. */
int rnb_hip_q8_0_head_gemv_batch(const uint8_t *w, size_t w_len, size_t head_count, size_t rows_per_head, size_t cols,
                                 size_t token_count, const float *x, size_t x_len, float *out, size_t out_len);

/* qwen35_sparse_experts_selected_base_by_token, crates/rnb-backend/cuda/src/runtime/api/
 * qwen_moe_api.rs:2529-2541 (validation: runtime/helpers.rs:1496-1600, 2747-2800): whole-layer
 * expert tensors + per-slot (expert id, route weight, token id).  Gate/up are Q4_K
 * [n_expert][n_ff][n_embd]; down is [n_expert][n_embd][n_ff] in `down_quant` (12 = Q4_K,
 * 13 = Q5_K, 14 = Q6_K).  out[token][n_embd] = sum over that token's slots, in slot order, of
 * route * W_down[e] . Q8_K(silu(W_gate[e] . Q8_K(x)) * (W_up[e] . Q8_K(x))).
 * The shared expert: the reference's decode call appends it to the slot list as expert id n_expert
 * with the shared gate's scalar as its route weight and its three tensors beside the routed ones
 * (crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:804-812; the id form is
 * qwen_moe_decode_sparse_experts_id_into, crates/rnb-llm/src/engine/backend_runtime/qwen_moe.rs:
 * 2807-2825).  shared_gate / shared_up / shared_down are those tensors, one expert's bytes each in
 * the routed experts' formats (the reference's condition, fanout.rs:790-803), or all three NULL;
 * with them a slot may carry expert id n_expert, without them that id is out of range. */
int rnb_hip_moe_sparse_experts_by_token(const uint8_t *gate_all, size_t gate_len,
                                        const uint8_t *up_all, size_t up_len,
                                        const uint8_t *down_all, size_t down_len,
                                        const uint8_t *shared_gate, size_t shared_gate_len,
                                        const uint8_t *shared_up, size_t shared_up_len,
                                        const uint8_t *shared_down, size_t shared_down_len,
                                        const uint32_t *expert_ids, const float *route_weights,
                                        const uint32_t *token_ids, size_t n_slots,
                                        size_t token_count, uint32_t down_quant, size_t n_ff,
                                        size_t n_embd, const float *x, size_t x_len, float *out,
                                        size_t out_len);

/* ---- device-resident variants --------------------------------------------------------------
 * The reference's device-input entry points (quant_api.rs:242-330 take `input_dev: u64`) keep
 * activations on the device between operators.  These take device pointers for weights, input
 * and output, enqueue on the library stream and return without synchronising. */
void *rnb_hip_dev_alloc(size_t bytes);
int rnb_hip_dev_free(void *ptr);
int rnb_hip_dev_upload(void *dst_dev, const void *src_host, size_t bytes);
int rnb_hip_dev_download(void *dst_host, const void *src_dev, size_t bytes);
/* quant: RNB_GGML_*; x_dev [seq_len][cols] f32 (16-byte aligned); out_dev [seq_len][rows] f32 */
int rnb_hip_gemv_dev(uint32_t quant, const void *w_dev, size_t rows, size_t cols,
                     const float *x_dev, size_t seq_len, float *out_dev);
/* rnb_hip_gemv_dev for callers that cannot allocate (code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc).  No counterpart in the reference.  Same arguments, arithmetic and results as
 * rnb_hip_gemv_dev, but the quantised activations and the K-slice partial sums live in a fixed array inside the
 * library's code object (rnb_hip_gemv_dev_noalloc_scratch_bytes() bytes per GPU, held until the process ends) instead
 * of the grow-only scratch, so the call never allocates or frees device memory.  Shapes that need more scratch than
 * that are rejected with RNB_HIP_INVALID_REQUEST (about 1.32 bytes per activation element, seq_len * cols, plus
 * slices * seq_len * rows * 4 for the small-grid GEMMs).  The array keeps the previous call's contents and every call
 * on a GPU shares it: calls that overlap on one GPU race, and it does not feed rnb_hip_gemv_quantized_dev. */
size_t rnb_hip_gemv_dev_noalloc_scratch_bytes(void);
int rnb_hip_gemv_dev_noalloc(uint32_t quant, const void *w_dev, size_t rows, size_t cols,
                             const float *x_dev, size_t seq_len, float *out_dev);
/* The two halves of rnb_hip_gemv_dev, for callers that feed several weight matrices from one
 * activation (the reference quantises once for gate+up / QKV: rnb_quantize_q8_1_by_32 followed by
 * rnb_q4k_gate_up_gemv_* in crates/rnb-backend/cuda/cuda/kernels/quant_gemv.cuh:700-1267).
 * rnb_hip_quantize_dev fills the library's activation scratch from x_dev [seq_len][cols];
 * rnb_hip_gemv_quantized_dev multiplies a weight matrix with whatever the scratch holds and must
 * be given the same quant family (32-element formats -> 32-wide Q8, K-quants -> Q8_K), cols and seq_len. */
int rnb_hip_quantize_dev(uint32_t quant, const float *x_dev, size_t seq_len, size_t cols);
int rnb_hip_gemv_quantized_dev(uint32_t quant, const void *w_dev, size_t rows, size_t cols,
                               size_t seq_len, float *out_dev);
/* RMS norm in front of the GEMVs, device-resident.  Arithmetic of crates/rnb-cpu/src/kernels/norm.rs:140-225: mean square
 * in f64 and out = (x / rms) * weight (rms_norm_into, the default path); with unit_offset != 0 the mean square in f32 and
 * out = (x / rms) * (1 + weight) (rms_norm_unit_offset_into).  x_dev [seq_len][hidden], hidden % 256 == 0.
 * rnb_hip_rms_norm_dev replaces rnb_rms_norm_f32 (crates/rnb-backend/cuda/cuda/kernels/quant_batch_and_ops.cuh:4031).
 * rnb_hip_rms_norm_quantize_dev also leaves Q8_K(out) in the library's activation scratch, exactly what
 * rnb_hip_quantize_dev would make of `out`, so that rnb_hip_gemv_quantized_dev (K-quant weights, cols == hidden) follows
 * without a quantiser launch; out_dev may be null when only the quantised form is wanted. */
int rnb_hip_rms_norm_dev(const float *x_dev, const float *weight_dev, float eps, int unit_offset, size_t seq_len,
                         size_t hidden, float *out_dev);
int rnb_hip_rms_norm_quantize_dev(const float *x_dev, const float *weight_dev, float eps, int unit_offset, size_t seq_len,
                                  size_t hidden, float *out_dev);
/* rnb_rms_norm_add_then_rms_norm_q8_1_f32 (quant_batch_and_ops.cuh:4275) with rnb-cpu's arithmetic and Q8_K output:
 * residual += norm(input, post_weight, post_eps); out = norm(residual, pre_weight, pre_eps); Q8_K(out) -> activation
 * scratch.  residual_dev is updated in place; out_dev may be null. */
int rnb_hip_rms_norm_add_rms_norm_quantize_dev(const float *input_dev, const float *post_weight_dev, float post_eps,
                                               int post_unit_offset, float *residual_dev, const float *pre_weight_dev,
                                               float pre_eps, int pre_unit_offset, size_t seq_len, size_t hidden,
                                               float *out_dev);
/* rnb_moe_route_topk_f32 (quant_batch_and_ops.cuh) with the selection rule of
 * crates/rnb-llm/src/engine/models/shared_expert_moe/routing.rs:18-64: per token the k largest logits (ties to the lower
 * expert id, NaN never selected), softmax over the selected logits, rank order.  logits_dev [token_count][n_expert];
 * idx_dev / weights_dev [token_count][min(k, n_expert)]; n_expert <= 512, k <= 32. */
int rnb_hip_moe_route_topk_dev(const float *logits_dev, size_t token_count, size_t n_expert, size_t k, uint32_t *idx_dev,
                               float *weights_dev);
/* device-resident form of rnb_hip_moe_sparse_experts_by_token: weights, x and out on the device;
 * the slot arrays stay on the host (the caller routes on the host, as the reference does).  The
 * shared expert's tensors (one expert each, on the device) or three NULLs. */
int rnb_hip_moe_sparse_experts_by_token_dev(const void *gate_dev, const void *up_dev,
                                            const void *down_dev, size_t n_expert,
                                            const void *shared_gate_dev, const void *shared_up_dev,
                                            const void *shared_down_dev,
                                            const uint32_t *expert_ids,
                                            const float *route_weights, const uint32_t *token_ids,
                                            size_t n_slots, size_t token_count,
                                            uint32_t down_quant, size_t n_ff, size_t n_embd,
                                            const float *x_dev, float *out_dev);

/* q6k_gemv_argmax(weights, rows, cols, input) -> (u32, f32), quant_api.rs:2170-2204: the LM-head GEMV with the
 * arg-max taken on the device (larger value wins, ties go to the lower row, as in
 * crates/rnb-backend/cuda/cuda/kernels/quant_batch_and_ops.cuh:3286-3328); 8 bytes come back instead of rows*4. */
int rnb_hip_q6k_gemv_argmax(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                            uint32_t *index_out, float *value_out);
/* q8_0_gemv_argmax, quant_api.rs:733-768: the same for a Q8_0 head (Q8 x Q8_0 integer dot) */
int rnb_hip_q8_0_gemv_argmax(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                             uint32_t *index_out, float *value_out);
/* q8_0_gemv_argmax_q8dot, quant_api.rs:770-805 (Q8 x Q8_0 integer dots by name): the same computation as the entry above */
int rnb_hip_q8_0_gemv_argmax_q8dot(const uint8_t *w, size_t w_len, size_t rows, size_t cols, const float *x, size_t x_len,
                                   uint32_t *index_out, float *value_out);

/* dense_q4k_attention_qkv(q_weights, k_weights, v_weights, q_rows, kv_rows, n_embd, input, q, k, v),
 * crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:916-985 (validation order and texts :928-968): the three Q4_K
 * projections of one decode token.  x is quantised once and the rows of the three matrices run as ONE launch;
 * q[0..q_rows), k[0..kv_rows), v[0..kv_rows) are written (capacities may be larger). */
int rnb_hip_dense_q4k_attention_qkv(const uint8_t *q_w, size_t q_len, const uint8_t *k_w, size_t k_len,
                                    const uint8_t *v_w, size_t v_len, size_t q_rows, size_t kv_rows,
                                    size_t n_embd, const float *x, size_t x_len, float *q, size_t q_cap,
                                    float *k, size_t k_cap, float *v, size_t v_cap);

/* ---- dense SwiGLU FFN: the GEMV's neighbours fused into one call -------------------------------
 * dense_q4k_silu_ffn_batch(gate, up, down, down_quant, n_ff, n_embd, seq_len, input) -> Vec<f32>,
 * crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:297-337; validation order and texts from
 * crates/rnb-backend/cuda/src/runtime/dense.rs:1712-1765 (seq_len > 1 required, as there).
 * out[s] = W_down . Q(silu(W_gate . Q8_K(x_s)) * (W_up . Q8_K(x_s))): gate/up are Q4_K [n_ff][n_embd],
 * down is [n_embd][n_ff] in Q4_K (12), Q5_K (13), Q6_K (14), Q8_0 (8) or Q5_1 (7), the reference's five codes.  Intermediates never leave the device. */
int rnb_hip_dense_q4k_silu_ffn_batch(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len,
                                     const uint8_t *down, size_t down_len, uint32_t down_quant, size_t n_ff,
                                     size_t n_embd, size_t seq_len, const float *x, size_t x_len, float *out,
                                     size_t out_len);
/* dense_q4k_gelu_ffn_batch, dense_api.rs:256-293: the same with the tanh form of GELU between the halves
 * (crates/rnb-cpu/src/kernels/activation.rs:91-98); validation shared with the SiLU form (dense.rs:1712-1765, texts
 * say "GELU") */
int rnb_hip_dense_q4k_gelu_ffn_batch(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len,
                                     const uint8_t *down, size_t down_len, uint32_t down_quant, size_t n_ff,
                                     size_t n_embd, size_t seq_len, const float *x, size_t x_len, float *out,
                                     size_t out_len);
/* dense_q4k_gelu_ffn(gate, up, down, down_quant, n_ff, n_embd, input) -> Vec<f32>, dense_api.rs:182-254: one token;
 * down in Q4_K, Q5_K or Q6_K (validation order and texts :191-232) */
int rnb_hip_dense_q4k_gelu_ffn(const uint8_t *gate, size_t gate_len, const uint8_t *up, size_t up_len,
                               const uint8_t *down, size_t down_len, uint32_t down_quant, size_t n_ff,
                               size_t n_embd, const float *x, size_t x_len, float *out, size_t out_len);
/* device-resident form (the reference's dev-input chain, dense.rs:2189-2219); also accepts one token */
int rnb_hip_dense_q4k_silu_ffn_dev(const void *gate_dev, const void *up_dev, const void *down_dev,
                                   uint32_t down_quant, size_t n_ff, size_t n_embd, size_t seq_len,
                                   const float *x_dev, float *out_dev);

/* ---- GGUF container: header, tensor table, untouched upload -------------------------------------
 * The reader side of the path: crates/rnb-loader/src/gguf/parser.rs:247-407 (GGUFFile::parse; same
 * limits, checks and message texts, reported through rnb_hip_last_error() with the Display strings of
 * crates/rnb-loader/src/error.rs:4-16), crates/rnb-loader/src/gguf/types.rs:5-41 (ggml type ids),
 * crates/rnb-loader/src/convert.rs:23-83 (tensor byte sizes) and :99-178 (map_tensors: every tensor
 * inside the file).  Tensor payloads are never copied or transformed on the host: `data` points into
 * the mapping, and rnb_hip_gguf_prewarm_tensor uploads exactly those bytes. */
typedef struct rnb_hip_gguf rnb_hip_gguf;
typedef struct rnb_hip_gguf_tensor {
    const char *name;      /* owned by the rnb_hip_gguf */
    uint32_t n_dims;       /* 0..4 */
    uint64_t shape[4];     /* row-major (outermost first): the file stores innermost first, parser.rs:356-357 */
    uint32_t ggml_type;    /* ggml type id: 2/3/6/7/8/9 = Q4_0/Q4_1/Q5_0/Q5_1/Q8_0/Q8_1, 10..14 = Q2_K..Q6_K, 0 = F32, ... */
    uint64_t offset;       /* relative to the data section, as stored */
    uint64_t file_offset;  /* data_start + offset */
    uint64_t n_bytes;      /* elements / block elements * block bytes; 0 if the shape is not block-aligned */
    const uint8_t *data;   /* mapping + file_offset, or NULL if the tensor does not lie inside the file */
} rnb_hip_gguf_tensor;

/* mmap + parse + map_tensors checks; the handle owns the mapping until rnb_hip_gguf_close.
 * Split models (crates/rnb-loader/src/gguf/sharded.rs:22-105, load_mapped_gguf): when the file's
 * metadata carries `split.count`, `path` may name any shard `<prefix>-<index>-of-<count>.gguf`; every
 * shard is mapped and checked (split.no / split.count / split.tensors.count agree with the selected
 * file and with the name, :107-158 and :181-236), the handle lists all tensors in shard order with
 * `file_offset` and `data` relative to the tensor's own shard, a name in two shards and a total that
 * differs from split.tensors.count are refused (:62-104), and the metadata is shard zero's.  Failures
 * read `parse error at offset 0: invalid split GGUF: ...` with the reference's texts. */
int rnb_hip_gguf_open(const char *path, rnb_hip_gguf **out);
/* GGUFFile::parse over caller-owned bytes (borrowed for the handle's lifetime); payload bounds are
 * not checked here, exactly as in the reference: call rnb_hip_gguf_map_tensors for that */
int rnb_hip_gguf_parse(const uint8_t *data, size_t len, rnb_hip_gguf **out);
int rnb_hip_gguf_map_tensors(const rnb_hip_gguf *g);
void rnb_hip_gguf_close(rnb_hip_gguf *g);
uint32_t rnb_hip_gguf_version(const rnb_hip_gguf *g);
uint64_t rnb_hip_gguf_alignment(const rnb_hip_gguf *g);   /* general.alignment, default 32 */
uint64_t rnb_hip_gguf_data_start(const rnb_hip_gguf *g);  /* header end rounded up to the alignment */
size_t rnb_hip_gguf_tensor_count(const rnb_hip_gguf *g);
int rnb_hip_gguf_tensor_at(const rnb_hip_gguf *g, size_t index, rnb_hip_gguf_tensor *out);
int rnb_hip_gguf_find_tensor(const rnb_hip_gguf *g, const char *name, rnb_hip_gguf_tensor *out);
/* checked_tensor_size, convert.rs:28-43 (shape row-major) */
int rnb_hip_gguf_tensor_size(const uint64_t *shape, uint32_t n_dims, uint32_t ggml_type, uint64_t *bytes);
/* metadata in file order; value type ids 0..12 as in the GGUF specification (8 = string, 9 = array);
 * rnb_hip_gguf_metadata_type returns -1 for an absent key */
size_t rnb_hip_gguf_metadata_count(const rnb_hip_gguf *g);
const char *rnb_hip_gguf_metadata_key(const rnb_hip_gguf *g, size_t index);
int rnb_hip_gguf_metadata_type(const rnb_hip_gguf *g, const char *key);
int rnb_hip_gguf_metadata_u64(const rnb_hip_gguf *g, const char *key, uint64_t *out); /* any non-negative integer, bool */
int rnb_hip_gguf_metadata_i64(const rnb_hip_gguf *g, const char *key, int64_t *out);
int rnb_hip_gguf_metadata_f64(const rnb_hip_gguf *g, const char *key, double *out);   /* F32 or F64 */
const char *rnb_hip_gguf_metadata_str(const rnb_hip_gguf *g, const char *key);        /* NULL unless a string */
int rnb_hip_gguf_metadata_array(const rnb_hip_gguf *g, const char *key, uint32_t *elem_type, uint64_t *count);
const char *rnb_hip_gguf_metadata_array_str(const rnb_hip_gguf *g, const char *key, uint64_t index);
int rnb_hip_gguf_metadata_array_f64(const rnb_hip_gguf *g, const char *key, uint64_t index, double *out);
/* uploads the tensor's bytes as stored (no requantisation, no repack) and pins them in the resident
 * table (rnb_hip_prewarm): operator calls that pass `data`, or a sub-range of it such as one expert
 * of a stacked [n_expert, rows, cols] tensor, then run from the device copy */
int rnb_hip_gguf_prewarm_tensor(const rnb_hip_gguf *g, size_t index);

#ifdef __cplusplus
}
#endif
#endif
