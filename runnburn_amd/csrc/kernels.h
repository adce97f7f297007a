// Kernel launchers of the gfx950 quantized-matmul backend (internal; the public surface is
// include/rnb_hip.h).  All launchers only enqueue on `stream`.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include <string>

namespace rnb {

constexpr uint32_t kQ4_0 = 2, kQ4_1 = 3, kQ5_0 = 6, kQ5_1 = 7, kQ8_0 = 8, kQ8_1 = 9, kQ2K = 10, kQ3K = 11, kQ4K = 12, kQ5K = 13, kQ6K = 14;  // ggml type ids
constexpr uint32_t kF32 = 0, kF16 = 1, kBF16 = 30;  // float formats (embedding tables only)
constexpr uint32_t kIQ2XXS = 16, kIQ3XXS = 18, kIQ2S = 22, kIQ4XS = 23;  // importance quants (256-element blocks, Q8_K activations)
constexpr size_t kIQ2XXSBytes = 66, kIQ3XXSBytes = 98, kIQ2SBytes = 82, kIQ4XSBytes = 136;
constexpr size_t kQ4_0Bytes = 18, kQ4_1Bytes = 20, kQ5_0Bytes = 22, kQ5_1Bytes = 24, kQ8_0Bytes = 34, kQ8_1Bytes = 36, kQ2KBytes = 84, kQ3KBytes = 110, kQ4KBytes = 144, kQ5KBytes = 176, kQ6KBytes = 210;

// Device layout of quantised activations (structure of arrays, one set per call):
//   Q8_K:  qs    int8  [seq][K]          (16-byte aligned rows, K % 256 == 0)
//          d     f32   [seq][K/256]
//          bsums int16 [seq][K/256][16]  (sums of 16 consecutive qs)
//          digits u8   [seq][K/256][16]  (optional; bsum32[k] = bsums[2k] + bsums[2k+1] = b0[k] + 64*b1[k]
//                                         as int8 digits: b0[0..8) in 0..63, then b1[0..8) in -64..63)
//   Q8:    qs    int8  [seq][K]
//          d     f32   [seq][K/32]
struct ActView {
    const int8_t *qs;
    const float *d;
    const int16_t *bsums;  // null for the 32-wide Q8 form
    const uint8_t *digits = nullptr;
};

// x: f32, 16-byte aligned, n_blocks*256 values
// digits may be null
void launch_quantize_q8k(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums, uint8_t *digits,
                         hipStream_t stream);
// the same launch also copies n_words 32-bit words from words_src (device memory or pinned host memory) to words_dst
void launch_quantize_q8k_copy(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums, uint8_t *digits,
                              const uint32_t *words_src, uint32_t n_words, uint32_t *words_dst, hipStream_t stream);
// x: f32, 16-byte aligned, n_blocks*32 values; n_blocks % 8 == 0 not required
void launch_quantize_q8(const float *x, size_t n_blocks, int8_t *qs, float *d, hipStream_t stream);

// out[s*rows + row] for s < seq; weights row-major packed blocks, base 16-byte aligned
void launch_gemv_q4k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb,
                     uint32_t seq, hipStream_t stream);
void launch_gemv_q5k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb,
                     uint32_t seq, hipStream_t stream);
// IQ2_XXS / IQ2_S / IQ3_XXS / IQ4_XS rows (2-byte aligned blocks) against Q8_K activations, a grid row per group of up
// to four tokens
bool is_iq_quant(uint32_t quant);
void launch_gemv_iq(const uint8_t *w, uint32_t quant, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                    hipStream_t stream);
// Embedding gather: out[t][cols] = dequantised row ids[t] (row t when ids is null) of a matrix in any of the block formats
// or f32 / f16 / bf16; values bit-identical to the reference's dequantisers.  n_tokens <= 65535, cols % 32 (256) == 0.
bool embed_gather_supported(uint32_t quant);
void launch_embed_gather(uint32_t quant, const uint8_t *w, size_t row_bytes, const uint32_t *ids, uint32_t n_tokens,
                         uint32_t cols, float *out, hipStream_t stream);
void launch_embed_gather_iq(uint32_t quant, const uint8_t *w, size_t row_bytes, const uint32_t *ids, uint32_t n_tokens,
                            uint32_t cols, float *out, hipStream_t stream);
// the same formats for batches, on the matrix cores; slice_out: workspace of gemm_iq_slice_floats(rows, nb, seq) floats (or
// null: no K slices)
size_t gemm_iq_slice_floats(uint32_t rows, uint32_t nb, uint32_t seq);
void launch_gemm_iq_mfma(const uint8_t *w, uint32_t quant, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                         uint32_t seq, hipStream_t stream);
// Q2_K / Q3_K rows (84 / 110-byte blocks at 4- / 2-byte alignment); quant is kQ2K or kQ3K
void launch_gemv_q2k_q3k(const uint8_t *w, uint32_t quant, ActView act, float *out, uint32_t rows, uint32_t nb,
                         uint32_t seq, hipStream_t stream);
// 32-element formats straight from an f32 token (the workgroup quantises it to 32-wide Q8 in LDS): rows of at most
// 128 blocks, x 16-byte aligned; same output contract as launch_gemv_block32
bool gemv_block32_f32_supported(uint32_t rows, uint32_t nb32, const void *x);  // false below the size where it pays
void launch_gemv_block32_f32(const uint8_t *w, uint32_t quant, const float *x, float *out, uint32_t rows, uint32_t nb32,
                             uint32_t seq, hipStream_t stream);
// the f32-token forms of launch_gemv_q4k_gate_up and launch_gemv_q4k_multi (rows of at most 16 super-blocks, x 16-byte
// aligned; weights 16-byte aligned as for the quantised forms)
void launch_gemv_q4k_gate_up_f32(const uint8_t *wg, const uint8_t *wu, const float *x, float *mid, uint32_t rows,
                                 uint32_t nb, uint32_t seq, bool gelu, hipStream_t stream);
void launch_gemv_q4k_multi_f32(const uint8_t *const w[3], const uint32_t rows[3], const float *x, float *out, uint32_t nb,
                               hipStream_t stream);
// K-quant GEMV straight from f32 tokens (the workgroup quantises its token to Q8_K in LDS): rows of at most 64
// super-blocks (beyond 16 a workgroup of sixteen waves works as split-K teams of two to four waves; its Q6_K form wants
// the matrix at an even address), x 16-byte aligned; same output contract and the same bits as launch_gemv_q4k on the
// stand-alone quantiser's output
bool gemv_kquant_f32_supported(uint32_t quant, uint32_t nb, const void *x, const void *w);
// false for matrices so large that quantising with a launch of its own and running the chunked GEMV is faster
bool gemv_kquant_f32_pays(uint32_t quant, uint32_t rows, uint32_t nb);
void launch_gemv_kquant_f32(const uint8_t *w, uint32_t quant, const float *x, float *out, uint32_t rows, uint32_t nb,
                            uint32_t seq, hipStream_t stream);
void launch_gemv_q6k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb,
                     uint32_t seq, hipStream_t stream);
void launch_gemv_q8_0(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb32,
                      uint32_t seq, hipStream_t stream);
// Per-head Q8_0 projections (q8_0_head_gemv_batch): weights [heads][rows_per_head][nb32 blocks of 34 bytes], 32-wide Q8
// activations [tokens][heads][nb32 * 32], out [tokens][heads * rows_per_head]; rows of at most 128 blocks; grid.z = heads
// (at most 65535), every (token, head) row group has the bits of launch_gemv_q8_0 on that head's rows
bool gemv_q8_0_heads_supported(uint32_t nb32);
void launch_gemv_q8_0_heads(const uint8_t *w, ActView act, float *out, uint32_t heads, uint32_t rows_per_head, uint32_t nb32,
                            uint32_t tokens, hipStream_t stream);
// any 32-element format (kQ4_0, kQ4_1, kQ5_0, kQ5_1, kQ8_0, kQ8_1) against 32-wide Q8 activations
void launch_gemv_block32(const uint8_t *w, uint32_t quant, ActView act, float *out, uint32_t rows, uint32_t nb32,
                         uint32_t seq, hipStream_t stream);

// gated-FFN front half, rows of at most 16 super-blocks: mid[s*rows + r] = act(Wg[r] . a_s) * (Wu[r] . a_s),
// act = SiLU or (gelu) the tanh form of GELU
bool gemv_q4k_gate_up_supported(uint32_t nb);
void launch_gemv_q4k_gate_up(const uint8_t *wg, const uint8_t *wu, ActView act, float *mid, uint32_t rows, uint32_t nb,
                             uint32_t seq, bool gelu, hipStream_t stream);
// up to three Q4_K matrices of nb super-blocks per row against one activation (token 0 of `act`), one launch;
// out = [rows[0] results | rows[1] results | rows[2] results]
void launch_gemv_q4k_multi(const uint8_t *const w[3], const uint32_t rows[3], ActView act, float *out, uint32_t nb,
                           hipStream_t stream);
// arg-max of `len` f32 (ties to the lower index); scratch_* hold 256 entries each, the result lands in out_*[0]
void launch_argmax(const float *values, uint32_t len, float *scratch_values, uint32_t *scratch_indices, float *out_value,
                   uint32_t *out_index, hipStream_t stream);
// out[i] = act(gate[i]) * up[i]
void launch_act_mul(const float *gate, const float *up, float *out, size_t n, bool gelu, hipStream_t stream);

// Q6_K / Q5_K x Q8_K and 32-element formats (Q8_0, Q8_1, Q4_0, Q4_1, Q5_0, Q5_1) x Q8 GEMMs on int8 MFMA (scale groups applied on the vector units); same contracts as
// launch_gemv_q6k / launch_gemv_block32, intended for seq >= 16.  Small grids are cut into K slices that are summed by
// a second kernel: slice_out is the workspace for that, gemm_blocks_slice_floats(quant, rows, k_steps, seq) floats
// (k_steps = 256-element steps per row: blocks, or ceil(32-element blocks / 8)); when that is 0, or slice_out is null,
// the kernel writes out directly.
size_t gemm_blocks_slice_floats(uint32_t quant, uint32_t rows, uint32_t k_steps, uint32_t seq);
void launch_gemm_q6k_mfma(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                          uint32_t seq, hipStream_t stream);
// Q5_K needs act.digits (the quantiser writes them for 16+ tokens)
void launch_gemm_q5k_mfma(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                          uint32_t seq, hipStream_t stream);
// Q4_K through the same kernel (scales on the vector units): for shapes that give gemm_q4k.hip's 256 x 64 tiles too few
// workgroups to fill the chip
void launch_gemm_q4k_small(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                           uint32_t seq, hipStream_t stream);
// Q2_K / Q3_K (needs act.bsums, which the Q8_K quantiser always writes)
void launch_gemm_q23k_mfma(const uint8_t *w, uint32_t quant, ActView act, float *out, float *slice_out, uint32_t rows,
                           uint32_t nb, uint32_t seq, hipStream_t stream);
bool gemm_q8_mfma_supported(uint32_t quant, uint32_t nb32);
void launch_gemm_q8_mfma(const uint8_t *w, uint32_t quant, ActView act, float *out, float *slice_out, uint32_t rows,
                         uint32_t nb32, uint32_t seq, hipStream_t stream);
// Q4_K x Q8_K GEMM on int8 MFMA; same contract as launch_gemv_q4k, intended for seq >= 16
// Up to 128 tiles the K range is cut into slices (workspace: gemm_q4k_slice_floats floats, as for the kernels above)
size_t gemm_q4k_slice_floats(uint32_t rows, uint32_t nb, uint32_t seq);
void launch_gemm_q4k_mfma(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                          uint32_t seq, hipStream_t stream);
// out[i] = parts[0][i] + parts[1][i] + ... in that order (n floats per slice)
void launch_sum_slices(const float *parts, float *out, size_t n, uint32_t slices, hipStream_t stream);

// ---- gathered sparse-MoE ------------------------------------------------------------------
// Slots grouped by expert (device arrays).  Group i covers sorted positions [start[i], start[i+1]);
// sorted_slot[p] is the caller's slot index at sorted position p, sorted_token[p] its token.
struct MoeGroups {
    const uint32_t *expert;        // [n_groups]
    const uint32_t *start;         // [n_groups + 1]
    const uint32_t *sorted_slot;   // [n_slots]
    const uint32_t *sorted_token;  // [n_slots]
    uint32_t n_groups;
    uint32_t max_group = 32;       // slots of the largest group (host-side knowledge: sizes the matrix-core kernels' LDS)
};
// Q8_K of act(gate[i]) * up[i] (SiLU, or the tanh form of GELU): the gated FFN's intermediate quantised as it is made
void launch_quantize_q8k_gated(const float *gate, const float *up, size_t n_blocks, bool gelu, int8_t *qs, float *d,
                               int16_t *bsums, uint8_t *digits, hipStream_t stream);
// Decode-sized routing tables travel as a kernel argument instead of a host-to-device copy: the
// activation quantiser's launch also writes them to their device buffer.
constexpr uint32_t kMoeInlineWords = 240;  // 960 bytes of kernel argument
struct MoeInlineTables {
    uint32_t words[kMoeInlineWords];
};
void launch_quantize_q8k_with_tables(const float *x, size_t n_blocks, int8_t *qs, float *d, int16_t *bsums,
                                     const MoeInlineTables &tables, uint32_t n_words, uint32_t *tables_dev,
                                     hipStream_t stream);
// The shared expert of a call: the reference's decode call appends it to the slot list as expert id n_expert with the
// shared gate's scalar as its route weight (crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:804-812);
// its three matrices have the routed experts' shapes and formats but live in allocations of their own.  Slots whose
// expert id is >= n_routed read these; without a shared expert the pointers are null and n_routed is UINT32_MAX.
struct MoeShared {
    const uint8_t *gate = nullptr, *up = nullptr, *down = nullptr;
    uint32_t n_routed = 0xffffffffu;
};
// mid[slot][n_ff] = silu(Wg[e] . h_tok) * (Wu[e] . h_tok); act = Q8_K(x) per token
void launch_moe_gate_up(const uint8_t *gate_all, const uint8_t *up_all, const MoeShared &shared, ActView act, MoeGroups groups,
                        float *mid, uint32_t n_ff, uint32_t nb_in, hipStream_t stream);
// slot_out[slot][n_embd] = route[slot] * (Wd[e] . Q8_K(mid[slot])); mid_act is indexed by slot; with mid_f32
// ([slot][nb_mid * 256], non-null) the workgroups quantise the rows they stage themselves and mid_act is not read
bool moe_down_quantises(uint32_t nb_mid);  // whether that pays (short intermediates)
void launch_moe_down(const uint8_t *down_all, const MoeShared &shared, uint32_t down_quant, ActView mid_act,
                     const float *mid_f32, MoeGroups groups, const float *slot_route, float *slot_out, uint32_t n_embd, uint32_t nb_mid, hipStream_t stream);
// the same two steps on the matrix cores for batches (act / mid_act carry digits, except a Q6_K down's mid_act):
// 32-token tiles per expert group, see moe_mfma.hip
bool moe_mfma_supported(uint32_t nb_in, uint32_t nb_mid, uint32_t down_quant);  // the tiles' LDS images fit
void launch_moe_gate_up_mfma(const uint8_t *gate_all, const uint8_t *up_all, const MoeShared &shared, ActView act,
                             MoeGroups groups, float *mid, uint32_t n_ff, uint32_t nb_in, hipStream_t stream);
void launch_moe_down_mfma(const uint8_t *down_all, const MoeShared &shared, uint32_t down_quant, const float *mid, MoeGroups groups,
                          const float *slot_route, float *slot_out, uint32_t n_embd, uint32_t nb_mid, hipStream_t stream);
// down + route weight + ordered per-token sum in one launch (rows of at most 16 super-blocks); slot_expert [n_slots]
void launch_moe_down_token(const uint8_t *down_all, const MoeShared &shared, uint32_t down_quant, ActView mid_act, const uint32_t *tok_offsets,
                           const uint32_t *tok_slots, const uint32_t *slot_expert, const float *slot_route, float *out,
                           uint32_t token_count, uint32_t n_embd, uint32_t nb_mid, hipStream_t stream);
// A few tokens (decode and small batches: at most 8 tokens and 64 slots, at most 16 slots per token): the whole expert
// step in two launches, the routing table as a kernel argument.  Slots are listed token by token, in list order inside a
// token (tok_off[t] .. tok_off[t + 1]); x f32 [n_tokens][n_embd] 16-byte aligned, mid scratch [n_slots][n_ff], out
// [n_tokens][n_embd]; the same bits as the general sequence
constexpr uint32_t kMoeDecodeMaxSlots = 64, kMoeDecodeMaxTokens = 8, kMoeDecodeMaxPerToken = 16;
struct MoeDecodeTable {
    uint32_t n_slots, n_tokens;
    uint32_t expert[kMoeDecodeMaxSlots];
    float route[kMoeDecodeMaxSlots];
    uint32_t token[kMoeDecodeMaxSlots];
    uint32_t tok_off[kMoeDecodeMaxTokens + 1];
};
// max_per_token: the largest number of slots any one token has
bool moe_decode_supported(size_t n_tokens, size_t n_slots, size_t max_per_token, size_t nb_in, size_t nb_mid, const void *x,
                          uint32_t down_quant, const void *down, const void *down_shared);
void launch_moe_decode(const uint8_t *gate_all, const uint8_t *up_all, const uint8_t *down_all, const MoeShared &shared,
                       uint32_t down_quant,
                       const MoeDecodeTable &table, const float *x, float *mid, float *out, uint32_t n_ff, uint32_t n_embd,
                       uint32_t nb_in, uint32_t nb_mid, hipStream_t stream);
// out[token][n_embd] = sum of slot_out over the token's slots, in list order;
// tok_offsets [token_count+1], tok_slots [n_slots] (CSR built by the host)
void launch_moe_reduce(const float *slot_out, const uint32_t *tok_offsets, const uint32_t *tok_slots,
                       float *out, uint32_t token_count, uint32_t n_embd, hipStream_t stream);

// ---- RMS norm (+ residual add) with optional Q8_K output, router (norm_route.hip) ------------------------------------
// Rows of nb * 256 floats, one workgroup each.  residual != null: residual += norm(input, post_weight, post_eps) first and
// the normalised row is the new residual; else it is input.  out_f32 and (qs, d, bsums[, digits]) are optional outputs.
void launch_rms_norm(const float *input, const float *post_weight, float post_eps, bool post_unit, float *residual,
                     const float *weight, float eps, bool unit, uint32_t seq, uint32_t nb, float *out_f32, int8_t *qs,
                     float *d, int16_t *bsums, uint8_t *digits, hipStream_t stream);
// top-k of each token's logits (ties to the lower id), softmax over the selected ones, rank order: idx_out / w_out
// [tokens][min(k, n_expert)]
bool route_topk_supported(uint32_t n_expert, uint32_t k);
void launch_route_topk(const float *logits, uint32_t tokens, uint32_t n_expert, uint32_t k, uint32_t *idx_out, float *w_out,
                       hipStream_t stream);

// ---- calibration (calib.hip): a read-only stream over `bytes` of device memory, and int8 matrix instructions only ----
void launch_calib_read(const void *dev, size_t bytes, bool non_temporal, uint32_t *sink, hipStream_t stream);
// returns the integer operations the launch performs (2 per multiply-add)
uint64_t launch_calib_mfma_i8(uint32_t iters, uint32_t workgroups, int *sink, hipStream_t stream);

// ---- launch configuration failures ------------------------------------------------------------------
// Raises `kernel`'s dynamic LDS limit to `bytes` (above the default 64 KB) once: `*done` is set only when the runtime
// accepted it, so a failure is tried again by the next launch.  On failure the launcher must not launch; the reason is
// kept for the API layer, which reports it instead of an unrelated launch error (take_launch_failure).
bool allow_dynamic_lds(const void *kernel, size_t bytes, bool *done, const char *kernel_name);
// the pending failure text of this thread, cleared by the call; empty when there is none
std::string take_launch_failure();

// ---- scratch that is part of the code object (static_scratch.hip) ---------------------------------
// Device address of the library's fixed scratch array on `device` (which must be current): looked up once per device.
constexpr size_t kStaticScratchBytes = size_t(8) << 20;
hipError_t static_scratch_address(int device, void **out);

}  // namespace rnb
