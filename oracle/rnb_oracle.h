/*
 * rnb_oracle.h -- CPU restatement of runNburn's rnb-cpu quantized-matmul arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker that the HIP kernels are
 * compared against and the CPU baseline that is timed beside them.  It is never linked
 * into, loaded by, or called from the shipped library (runnburn_amd/librnb_hip.so).
 *
 * Every function cites the reference source (paths relative to the reference checkout)
 * whose arithmetic it restates.  The reference is a Rust workspace and no Rust toolchain
 * exists here, so the oracle is pinned against the known-answer vectors in the
 * reference's own unit tests and against independent mathematical checks (see
 * tests/test_oracle_*.py).
 *
 * Pin status per function is listed in rnb_oracle.c's header comment.
 */
#ifndef RNB_ORACLE_H
#define RNB_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RNBO_QK_K 256
#define RNBO_Q8_0_BLOCK_BYTES 34
#define RNBO_Q4_0_BLOCK_BYTES 18
#define RNBO_Q4_1_BLOCK_BYTES 20
#define RNBO_Q5_0_BLOCK_BYTES 22
#define RNBO_Q5_1_BLOCK_BYTES 24
#define RNBO_Q8_1_BLOCK_BYTES 36
#define RNBO_Q2_K_BLOCK_BYTES 84
#define RNBO_Q3_K_BLOCK_BYTES 110
#define RNBO_Q4_K_BLOCK_BYTES 144
#define RNBO_Q5_K_BLOCK_BYTES 176
#define RNBO_Q6_K_BLOCK_BYTES 210
/* importance quants (ggml type ids 16, 22, 18, 23), crates/rnb-cpu/src/quantize/iq.rs:23-116 */
#define RNBO_IQ2_XXS_BLOCK_BYTES 66
#define RNBO_IQ2_S_BLOCK_BYTES 82
#define RNBO_IQ3_XXS_BLOCK_BYTES 98
#define RNBO_IQ4_XS_BLOCK_BYTES 136

/* Q8_K activation block, crates/rnb-cpu/src/gemm/activation_q8.rs:66-72 (repr(C), 292 B). */
typedef struct {
    float d;
    int8_t qs[256];
    int16_t bsums[16];
} rnbo_q8k_block;

/* 32-wide activation block, crates/rnb-cpu/src/gemm/activation_q8.rs:7-10 (36 B). */
typedef struct {
    float d;
    int8_t qs[32];
} rnbo_q8_block;

/* ---- scalar helpers ------------------------------------------------------------ */
float rnbo_f16_to_f32(uint16_t bits);
uint16_t rnbo_f32_to_f16(float value);
void rnbo_get_scale_min_k4(int j, const uint8_t *q12, uint8_t *sc, uint8_t *mn);
int rnbo_nearest_int(float fval);

/* ---- dequantisers (element order of the formats) -------------------------------- */
void rnbo_dequantize_q8_0(const uint8_t *blocks, size_t n_blocks, float *out);
/* quant: 2 = Q4_0, 3 = Q4_1, 6 = Q5_0, 7 = Q5_1 (32-element blocks); non-zero return: unknown id */
int rnbo_dequantize_legacy(uint32_t quant, const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_q2_k(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_q3_k(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_q4_k(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_q5_k(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_q6_k(const uint8_t *blocks, size_t n_blocks, float *out);

/* ---- activation quantisers (bit-exact contract) --------------------------------- */
void rnbo_quantize_q8k(const float *x, size_t n, rnbo_q8k_block *out);
void rnbo_quantize_q8(const float *x, size_t n, rnbo_q8_block *out);

/* ---- row dots ------------------------------------------------------------------- */
float rnbo_dot_legacy_q8(uint32_t quant, const uint8_t *row, const rnbo_q8_block *act, size_t n_blocks);
double rnbo_dot_legacy_q8_f64(uint32_t quant, const uint8_t *row, const rnbo_q8_block *act, size_t n_blocks);
float rnbo_dot_q2k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_q3k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_q4k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_q5k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_q6k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_q8_0_q8(const uint8_t *row, const rnbo_q8_block *act, size_t n_blocks);
float rnbo_dot_q8_0_f32(const uint8_t *row, const float *x, size_t n_blocks);
/* f64-accumulated "gold" forms of the same integer arithmetic */
double rnbo_dot_q2k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
double rnbo_dot_q3k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
double rnbo_dot_q4k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
double rnbo_dot_q5k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
double rnbo_dot_q6k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
double rnbo_dot_q8_0_q8_f64(const uint8_t *row, const rnbo_q8_block *act, size_t n_blocks);

/* ---- importance quants (rnb_oracle_iq.c) ------------------------------------------ */
void rnbo_dequantize_iq2_xxs(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_iq2_s(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_iq3_xxs(const uint8_t *blocks, size_t n_blocks, float *out);
void rnbo_dequantize_iq4_xs(const uint8_t *blocks, size_t n_blocks, float *out);
float rnbo_dot_iq2_xxs_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_iq2_s_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_iq3_xxs_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_iq4_xs_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_iq_q8k(uint32_t quant, const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
double rnbo_dot_iq_q8k_f64(uint32_t quant, const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
size_t rnbo_iq_grid(int which, uint64_t *out);
void rnbo_make_iq_row(uint32_t quant, size_t n_blocks, uint64_t seed, float sigma, uint8_t *out);

/* ---- GEMV / GEMM drivers: out[s*rows + row], x is [seq_len][cols] --------------- */
/* quant: 2 = Q4_0, 3 = Q4_1, 6 = Q5_0, 7 = Q5_1, 8 = Q8_0 (all against 32-wide Q8 activations), 10 = Q2_K, 11 = Q3_K, 12 = Q4_K, 13 = Q5_K, 14 = Q6_K (ggml type ids).  */
int rnbo_gemv(uint32_t quant, const uint8_t *w, size_t rows, size_t cols, const float *x,
              size_t seq_len, float *out, int n_threads);
int rnbo_gemv_f64(uint32_t quant, const uint8_t *w, size_t rows, size_t cols, const float *x,
                  size_t seq_len, double *out, int n_threads);
/* x86 default for Q8_0: f32 activations, no activation quantisation. */
int rnbo_gemv_q8_0_f32act(const uint8_t *w, size_t rows, size_t cols, const float *x,
                          size_t seq_len, float *out, int n_threads);

/* ---- MoE ------------------------------------------------------------------------ */
void rnbo_silu_mul_inplace(float *gate, const float *up, size_t n);
void rnbo_gelu_mul_inplace(float *gate, const float *up, size_t n);
size_t rnbo_route_topk(const float *logits, size_t n_expert, size_t k, uint32_t *idx_out,
                       float *weights_out);
int rnbo_moe_sparse_experts_by_token(const uint8_t *gate_all, const uint8_t *up_all,
                                     const uint8_t *down_all, size_t n_expert,
                                     const uint32_t *expert_ids, const float *route,
                                     const uint32_t *token_ids, size_t n_slots, size_t token_count,
                                     uint32_t down_quant, size_t n_ff, size_t n_embd,
                                     const float *x, float *out, int n_threads);

/* ---- input generation (not on the GPU path) ------------------------------------- */
int rnbo_quantize_row_legacy(uint32_t quant, const float *x, size_t n, uint8_t *out);
void rnbo_quantize_row_q2_k(const float *x, size_t n, uint8_t *out);
void rnbo_quantize_row_q3_k(const float *x, size_t n, uint8_t *out);
void rnbo_quantize_row_q4_k(const float *x, size_t n, uint8_t *out);
void rnbo_quantize_row_q5_k(const float *x, size_t n, uint8_t *out);
void rnbo_quantize_row_q6_k(const float *x, size_t n, uint8_t *out);
void rnbo_quantize_row_q8_0(const float *x, size_t n, uint8_t *out);
void rnbo_fill_normal(float *out, size_t n, uint64_t seed, float sigma);
/* rows x cols fp32 N(0, sigma) from `seed`, quantised row by row; multi-threaded.    */
int rnbo_make_weights(uint32_t quant, size_t rows, size_t cols, uint64_t seed, float sigma,
                      uint8_t *out, int n_threads);

/* ---- x86 production-order restatement (AVX2+FMA), used as the timed CPU baseline - */
int rnbo_have_avx2(void);
float rnbo_dot_q4k_q8k_avx2(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
float rnbo_dot_q6k_q8k_avx2(const uint8_t *row, const rnbo_q8k_block *act, size_t n_blocks);
int rnbo_gemv_avx2(uint32_t quant, const uint8_t *w, size_t rows, size_t cols, const float *x,
                   size_t seq_len, float *out, int n_threads);
/* rnbo_moe_sparse_experts_by_token over the AVX2 dots (Q5_K down keeps the scalar dot);
 * returns 3 on a machine without AVX2+FMA.                                            */
int rnbo_moe_sparse_experts_by_token_avx2(const uint8_t *gate_all, const uint8_t *up_all,
                                          const uint8_t *down_all, size_t n_expert,
                                          const uint32_t *expert_ids, const float *route,
                                          const uint32_t *token_ids, size_t n_slots,
                                          size_t token_count, uint32_t down_quant, size_t n_ff,
                                          size_t n_embd, const float *x, float *out, int n_threads);

#ifdef __cplusplus
}
#endif
#endif
