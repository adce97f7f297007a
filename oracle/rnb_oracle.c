/*
 * rnb_oracle.c -- scalar, integer-exact CPU restatement of rnb-cpu's quantized matmul path.
 *
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the timed CPU baseline.
 * Nothing shipped links or loads this file.
 *
 * Reference paths are relative to the reference checkout (crates/...).  The reference is
 * Rust and cannot be built here (no cargo/rustc), so each function is pinned without it:
 *
 *   function                    pinned by (tests/test_oracle_*.py)
 *   --------------------------  ------------------------------------------------------------
 *   f16 <-> f32                 all 65536 bit patterns vs numpy.float16 (IEEE binary16)
 *   get_scale_min_k4            hand-decoded vector from the reference's CUDA tests + brute force
 *   dequantize_*                brute-force numpy restatement of the public GGUF layouts + round
 *                               trips through independent numpy packers
 *   quantize_q8k                the reference's exact vectors (activation_q8.rs:179-217)
 *   quantize_q8                 closed-form cases + numpy restatement (formula is 6 lines)
 *   dot_q4k_q8k                 reference closed forms 0 / 0 / 2560.0 (tile_q4k.rs:2019-2151),
 *                               f64 numpy dequant(W) . dequant(Q8K(x)) identity
 *   dequantize_q4_0 .. _q5_1    one-hot placement of every nibble and high bit + independent numpy statements
 *   dot_q4_0/_q4_1/_q5_0/_q5_1  hand-built vectors (offset 8 / 16, min term against the activation sum, high bits),
 *   (x Q8)                      f64 numpy dequant identity
 *   dequantize_q2_k/_q3_k       the reference's own vectors (dequant.rs:898-927, 1009-1019: zero blocks, qs[1] = 3 ->
 *                               out[1] = 3) + one-hot placement of every field + independent numpy statements
 *   dot_q2k_q8k, dot_q3k_q8k    hand-built vectors per sub-block scale / min / high bit, f64 numpy dequant
 *                               identity (the reference's AVX2 kernels are checked the same way, loosely:
 *                               avx2_dot.rs tests)
 *   dot_q5k_q8k                 one-hot fifth-bit vectors (each qh bit moves exactly the element the
 *                               reference's tile_q5k.rs:944-976 statement names), f64 numpy dequant
 *                               identity, reduction to dot_q4k_q8k when qh == 0
 *   dot_q6k_q8k                 f64 numpy dequant identity; bsums identity (avx2_dot.rs:824,880)
 *   dot_q8_0_*                  reference vector 528.0 (quant_gemv.rs:1448-1464), numpy identity
 *   Q8_1 dequant / dot          the reference holds no known-answer test for Q8_1: hand-built bytes (every
 *                               element position, the stored sum ignored), closed form on constant vectors,
 *                               f64 numpy dequant identity
 *   gemv drivers                seq-major layout vector (quant_gemv.rs:1448-1464)
 *   gelu_mul_inplace            reference vector (activation.rs:166-173: gate [1, -1], up [2, 3] -> 1.6824, -0.4764)
 *                               + f64 numpy statement of the tanh form
 *   route_topk                  reference vectors (routing.rs:272-318)
 *   moe_sparse_experts_by_token f32-dequant statement of the reference's CUDA test oracle
 *                               (cuda tests.rs:29561-29584) to activation-quant noise; composition
 *                               of already-pinned pieces
 *   quantize_row_q4_k           PARITY UNPINNED at byte level (needs the Rust original); only the
 *                               reference's round-trip property (quant.rs:766-798) is checked.
 *                               Input generation only -- GPU and oracle consume identical bytes.
 *   quantize_row_q5_k           as quantize_row_q4_k: byte parity UNPINNED, the reference's round-trip
 *                               property (quant.rs:732-764) is checked.  Input generation only.
 *   quantize_row_q2_k           restates quant.rs:44-160; byte parity UNPINNED (cannot run the original), the
 *                               reference's round-trip bound (cosine >= 0.90) is checked.  Input generation only.
 *   quantize_row_q3_k           not in the reference (plain symmetric fit).  Input generation only.
 *   quantize_row_q4_0 .. _q5_1, _q8_1  not in the reference (ggml reference semantics).  Input generation only.
 *   quantize_row_q6_k/_q8_0     not in the reference at all (ggml reference semantics); round
 *                               trip through the pinned dequantisers.  Input generation only.
 *   IQ2_XXS / IQ2_S / IQ3_XXS / IQ4_XS  dequantisers and Q8_K dots live in rnb_oracle_iq.c (pins listed there: the
 *                               reference's FNV-1a known answers, iq.rs:258-334); rms_norm is numpy, in oracle.py
 *                               (pinned on the reference's vectors, norm.rs tests)
 */
#include "rnb_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ================================================================================ */
/* f16: the reference uses the `half` crate (IEEE binary16, RNE on from_f32).        */
/* ================================================================================ */

float rnbo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int shift = 0;
            while ((man & 0x400u) == 0) {
                man <<= 1;
                shift++;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

uint16_t rnbo_f32_to_f16(float value) {
    uint32_t x;
    memcpy(&x, &value, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t exp = (x >> 23) & 0xffu;
    uint32_t man = x & 0x7fffffu;
    if (exp == 255) { /* inf / nan */
        if (man == 0) return (uint16_t)(sign | 0x7c00u);
        return (uint16_t)(sign | 0x7c00u | 0x200u | (man >> 13));
    }
    int e = (int)exp - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign; /* underflow -> signed zero */
        man |= 0x800000u;
        int shift = 14 - e; /* 14..24 */
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++; /* may carry into exponent */
    return (uint16_t)(sign | half);
}

static inline float rd_f16(const uint8_t *p) {
    return rnbo_f16_to_f32((uint16_t)(p[0] | ((uint16_t)p[1] << 8)));
}

static inline void wr_f16(uint8_t *p, float v) {
    uint16_t h = rnbo_f32_to_f16(v);
    p[0] = (uint8_t)(h & 0xff);
    p[1] = (uint8_t)(h >> 8);
}

/* crates/rnb-cpu/src/quantize/quant.rs:591-599 (get_scale_min_k4) */
void rnbo_get_scale_min_k4(int j, const uint8_t *q, uint8_t *sc, uint8_t *mn) {
    if (j < 4) {
        *sc = q[j] & 63;
        *mn = q[j + 4] & 63;
    } else {
        *sc = (uint8_t)((q[j + 4] & 0x0f) | ((q[j - 4] >> 6) << 4));
        *mn = (uint8_t)((q[j + 4] >> 4) | ((q[j] >> 6) << 4));
    }
}

/* crates/rnb-cpu/src/quantize/quant.rs:173-178 (nearest_int) */
int rnbo_nearest_int(float fval) {
    float val = fval + 12582912.0f;
    uint32_t bits;
    memcpy(&bits, &val, 4);
    return (int)(bits & 0x007fffffu) - 0x00400000;
}

/* ================================================================================ */
/* Dequantisers                                                                      */
/* ================================================================================ */

/* crates/rnb-cpu/src/quantize/dequant.rs:55-60 */
void rnbo_dequantize_q8_0(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_Q8_0_BLOCK_BYTES;
        float d = rd_f16(blk);
        for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)blk[2 + i] * d;
    }
}

/* The 32-element formats with 4- or 5-bit codes: crates/rnb-cpu/src/quantize/dequant.rs:7-53.
 *   Q4_0 {f16 d, qs[16]}                 (code - 8) * d        Q4_1 {f16 d, f16 m, qs[16]}          code * d + m
 *   Q5_0 {f16 d, qh[4], qs[16]}          (code - 16) * d       Q5_1 {f16 d, f16 m, qh[4], qs[16]}   code * d + m
 * Element i < 16 is the low nibble of qs[i], element 16 + i the high nibble; the fifth bit of element e is bit e of
 * the little-endian 32-bit qh.
 *   Q8_1 {f16 d, f16 s, i8 qs[32]}       code * d  (whole-byte codes; s = d * sum(qs) is stored for other back ends and
 *                                        not used: crates/rnb-cpu/src/gemm/quant_gemv.rs:210-216, neon_quant.rs:236-253) */
typedef struct {
    int bytes, qs_off, qh_off, has_min, offset; /* qh_off < 0: no fifth bit */
    int byte_codes;                             /* codes are the 32 signed bytes at qs_off */
} legacy_fmt;

static int legacy_format(uint32_t quant, legacy_fmt *f) {
    switch (quant) {
    case 2: *f = (legacy_fmt){RNBO_Q4_0_BLOCK_BYTES, 2, -1, 0, 8, 0}; return 1;
    case 3: *f = (legacy_fmt){RNBO_Q4_1_BLOCK_BYTES, 4, -1, 1, 0, 0}; return 1;
    case 6: *f = (legacy_fmt){RNBO_Q5_0_BLOCK_BYTES, 6, 2, 0, 16, 0}; return 1;
    case 7: *f = (legacy_fmt){RNBO_Q5_1_BLOCK_BYTES, 8, 4, 1, 0, 0}; return 1;
    case 9: *f = (legacy_fmt){RNBO_Q8_1_BLOCK_BYTES, 4, -1, 0, 0, 1}; return 1;
    default: return 0;
    }
}

static inline int legacy_code(const legacy_fmt *f, const uint8_t *blk, int e) {
    if (f->byte_codes) return (int)(int8_t)blk[f->qs_off + e];
    int nib = e < 16 ? (blk[f->qs_off + e] & 0x0f) : (blk[f->qs_off + e - 16] >> 4);
    if (f->qh_off >= 0) {
        uint32_t qh = (uint32_t)blk[f->qh_off] | ((uint32_t)blk[f->qh_off + 1] << 8) |
                      ((uint32_t)blk[f->qh_off + 2] << 16) | ((uint32_t)blk[f->qh_off + 3] << 24);
        nib |= (int)((qh >> e) & 1u) << 4;
    }
    return nib;
}

int rnbo_dequantize_legacy(uint32_t quant, const uint8_t *blocks, size_t n_blocks, float *out) {
    legacy_fmt f;
    if (!legacy_format(quant, &f)) return 1;
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * (size_t)f.bytes;
        float d = rd_f16(blk), m = f.has_min ? rd_f16(blk + 2) : 0.0f;
        for (int e = 0; e < 32; e++) {
            int code = legacy_code(&f, blk, e);
            out[b * 32 + e] = f.has_min ? (float)code * d + m : ((float)code - (float)f.offset) * d;
        }
    }
    return 0;
}

/* crates/rnb-cpu/src/quantize/dequant.rs:66-86.  Block = {u8 scales[16] (scale | min << 4), u8 qs[64], f16 d,
 * f16 dmin}; sub-block j (16 elements) lives in half j/8, bytes 16*(j%2).. of that half's 32, bit pair (j%8)/2. */
void rnbo_dequantize_q2_k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_Q2_K_BLOCK_BYTES;
        const uint8_t *qs = blk + 16;
        float d = rd_f16(blk + 80), dmin = rd_f16(blk + 82);
        float *y = out + b * 256;
        for (int j = 0; j < 16; j++) {
            float scale = d * (float)(blk[j] & 0x0f);
            float min = dmin * (float)(blk[j] >> 4);
            int q_base = (j / 8) * 32 + (j % 2) * 16, shift = ((j % 8) / 2) * 2;
            for (int l = 0; l < 16; l++) {
                float q = (float)((qs[q_base + l] >> shift) & 3);
                y[16 * j + l] = q * scale - min;
            }
        }
    }
}

/* The sixteen 6-bit scales of a Q3_K block: crates/rnb-cpu/src/quantize/dequant.rs:240-263.  Scale k keeps its
 * low four bits in nibble k/8 of byte k%8 and its high two in bit pair k/4 of byte 8 + k%4. */
static void q3k_scales(const uint8_t *sb, int8_t *scales) {
    for (int k = 0; k < 16; k++) {
        int lo = (k < 8) ? (sb[k] & 0x0f) : (sb[k - 8] >> 4);
        int hi = (sb[8 + (k % 4)] >> (2 * (k / 4))) & 3;
        scales[k] = (int8_t)(lo | (hi << 4));
    }
}

/* crates/rnb-cpu/src/quantize/dequant.rs:237-297.  Block = {u8 hmask[32], u8 qs[64], u8 scales[12], f16 d}; the
 * value is the 2-bit field minus 4 unless its hmask bit is set; qs is laid out as for Q2_K and the 32-element
 * group g = 4*half + bit-pair uses bit g of hmask[l]. */
void rnbo_dequantize_q3_k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_Q3_K_BLOCK_BYTES;
        const uint8_t *hm = blk, *q = blk + 32;
        float d_all = rd_f16(blk + 108);
        int8_t scales[16];
        q3k_scales(blk + 96, scales);
        float *y = out + b * 256;
        int is = 0;
        uint8_t m = 1;
        for (int n = 0; n < 2; n++) {
            for (int shift = 0; shift < 8; shift += 2) {
                for (int h = 0; h < 2; h++) {
                    float dl = d_all * ((float)scales[is++] - 32.0f);
                    for (int l = 0; l < 16; l++) {
                        int qv = (q[32 * n + 16 * h + l] >> shift) & 3;
                        int hv = (hm[16 * h + l] & m) ? 0 : 4;
                        *y++ = dl * (float)(qv - hv);
                    }
                }
                m = (uint8_t)(m << 1);
            }
        }
    }
}

/* crates/rnb-cpu/src/quantize/dequant.rs:353-381 */
void rnbo_dequantize_q4_k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_Q4_K_BLOCK_BYTES;
        float d = rd_f16(blk);
        float dmin = rd_f16(blk + 2);
        const uint8_t *q = blk + 16;
        float *y = out + b * 256;
        for (int g = 0; g < 4; g++) {
            uint8_t sc1, mn1, sc2, mn2;
            rnbo_get_scale_min_k4(2 * g, blk + 4, &sc1, &mn1);
            rnbo_get_scale_min_k4(2 * g + 1, blk + 4, &sc2, &mn2);
            float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
            float d2 = d * (float)sc2, m2 = dmin * (float)mn2;
            for (int l = 0; l < 32; l++) y[64 * g + l] = d1 * (float)(q[32 * g + l] & 0x0f) - m1;
            for (int l = 0; l < 32; l++) y[64 * g + 32 + l] = d2 * (float)(q[32 * g + l] >> 4) - m2;
        }
    }
}

/* crates/rnb-cpu/src/quantize/dequant.rs:735-770: Q4_K's walk with a fifth bit per element, bit 2g of
 * qh[l] for the low-nibble half of group g and bit 2g+1 for the high-nibble half. */
void rnbo_dequantize_q5_k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_Q5_K_BLOCK_BYTES;
        float d = rd_f16(blk);
        float dmin = rd_f16(blk + 2);
        const uint8_t *qh = blk + 16, *ql = blk + 48;
        float *y = out + b * 256;
        uint8_t u1 = 1, u2 = 2;
        for (int g = 0; g < 4; g++) {
            uint8_t sc1, mn1, sc2, mn2;
            rnbo_get_scale_min_k4(2 * g, blk + 4, &sc1, &mn1);
            rnbo_get_scale_min_k4(2 * g + 1, blk + 4, &sc2, &mn2);
            float d1 = d * (float)sc1, m1 = dmin * (float)mn1;
            float d2 = d * (float)sc2, m2 = dmin * (float)mn2;
            for (int l = 0; l < 32; l++) {
                uint8_t v = (uint8_t)((ql[32 * g + l] & 0x0f) + ((qh[l] & u1) ? 16 : 0));
                y[64 * g + l] = d1 * (float)v - m1;
            }
            for (int l = 0; l < 32; l++) {
                uint8_t v = (uint8_t)((ql[32 * g + l] >> 4) + ((qh[l] & u2) ? 16 : 0));
                y[64 * g + 32 + l] = d2 * (float)v - m2;
            }
            u1 = (uint8_t)(u1 << 2);
            u2 = (uint8_t)(u2 << 2);
        }
    }
}

/* crates/rnb-cpu/src/quantize/dequant.rs:780-807 */
void rnbo_dequantize_q6_k(const uint8_t *blocks, size_t n_blocks, float *out) {
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_Q6_K_BLOCK_BYTES;
        const uint8_t *ql = blk, *qh = blk + 128;
        const int8_t *sc = (const int8_t *)(blk + 192);
        float d = rd_f16(blk + 208);
        float *y = out + b * 256;
        for (int n = 0; n < 2; n++) {
            for (int l = 0; l < 32; l++) {
                int is = l / 16;
                uint8_t h = qh[32 * n + l];
                int q1 = (ql[64 * n + l] & 0x0f) | ((h & 3) << 4);
                int q2 = (ql[64 * n + l + 32] & 0x0f) | (((h >> 2) & 3) << 4);
                int q3 = (ql[64 * n + l] >> 4) | (((h >> 4) & 3) << 4);
                int q4 = (ql[64 * n + l + 32] >> 4) | (((h >> 6) & 3) << 4);
                y[128 * n + l] = d * (float)sc[8 * n + is] * (float)(q1 - 32);
                y[128 * n + l + 32] = d * (float)sc[8 * n + is + 2] * (float)(q2 - 32);
                y[128 * n + l + 64] = d * (float)sc[8 * n + is + 4] * (float)(q3 - 32);
                y[128 * n + l + 96] = d * (float)sc[8 * n + is + 6] * (float)(q4 - 32);
            }
        }
    }
}

/* ================================================================================ */
/* Activation quantisers                                                             */
/* ================================================================================ */

/* Rust's `f32 as i32`: NaN -> 0, out-of-range values saturate (the C conversion is undefined for both) */
static inline int32_t f32_as_i32(float v) {
    if (v != v) return 0;
    if (v >= 2147483648.0f) return INT32_MAX;
    if (v <= -2147483648.0f) return INT32_MIN;
    return (int32_t)v;
}

/* crates/rnb-cpu/src/gemm/activation_q8.rs:149-173 (quantize_q8k_block_ggml) */
static void quantize_q8k_block(const float *x, rnbo_q8k_block *blk) {
    float amax = 0.0f, max_val = 0.0f;
    for (int i = 0; i < 256; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) { /* strict: first occurrence wins */
            amax = ax;
            max_val = x[i];
        }
    }
    memset(blk, 0, sizeof(*blk));
    if (amax == 0.0f) return;
    volatile float iscale = -127.0f / max_val;
    volatile float d = 1.0f / iscale;
    blk->d = d;
    for (int i = 0; i < 256; i++) {
        volatile float prod = iscale * x[i];
        int v = f32_as_i32(rintf(prod)); /* round half to even (default rounding mode), then `as i32` */
        if (v > 127) v = 127;     /* upper clamp only */
        int8_t q = (int8_t)v;
        blk->qs[i] = q;
        blk->bsums[i / 16] = (int16_t)(blk->bsums[i / 16] + q);
    }
}

/* crates/rnb-cpu/src/gemm/activation_q8.rs:109-139 */
void rnbo_quantize_q8k(const float *x, size_t n, rnbo_q8k_block *out) {
    size_t nb = n / 256;
    for (size_t b = 0; b < nb; b++) quantize_q8k_block(x + b * 256, out + b);
}

/* crates/rnb-cpu/src/gemm/activation_q8.rs:14-52 (quantize_input_q8) */
void rnbo_quantize_q8(const float *x, size_t n, rnbo_q8_block *out) {
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; b++) {
        const float *c = x + b * 32;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            float ax = fabsf(c[i]);
            /* f32::max ignores a NaN operand, as this comparison does */
            if (ax > amax) amax = ax;
        }
        volatile float d = amax / 127.0f;
        volatile float id = (d != 0.0f) ? 1.0f / d : 0.0f;
        out[b].d = d;
        for (int i = 0; i < 32; i++) {
            volatile float prod = c[i] * id;
            float r = roundf(prod); /* half away from zero */
            if (r < -128.0f) r = -128.0f;
            if (r > 127.0f) r = 127.0f;
            out[b].qs[i] = (int8_t)f32_as_i32(r); /* NaN.clamp(..) stays NaN, `as i8` makes it 0 */
        }
    }
}

static inline int bsum32(const rnbo_q8k_block *a, int k) { /* activation_q8.rs:80-82 */
    return (int16_t)(a->bsums[2 * k] + a->bsums[2 * k + 1]);
}

/* ================================================================================ */
/* Row dots                                                                          */
/* ================================================================================ */

/* integer part of one Q4_K block: crates/rnb-cpu/src/gemm/neon_dot.rs:884-916 */
static inline void q4k_block_ints(const uint8_t *blk, const rnbo_q8k_block *a, int32_t *sumi_out,
                                  int32_t *summ_out) {
    const uint8_t *qs = blk + 16;
    int32_t sumi = 0, summ = 0;
    for (int g = 0; g < 4; g++) {
        uint8_t sc0, mn0, sc1, mn1;
        rnbo_get_scale_min_k4(2 * g, blk + 4, &sc0, &mn0);
        rnbo_get_scale_min_k4(2 * g + 1, blk + 4, &sc1, &mn1);
        int32_t i0 = 0, i1 = 0;
        for (int l = 0; l < 32; l++) {
            i0 += (int32_t)(qs[32 * g + l] & 0x0f) * (int32_t)a->qs[64 * g + l];
            i1 += (int32_t)(qs[32 * g + l] >> 4) * (int32_t)a->qs[64 * g + 32 + l];
        }
        sumi += (int32_t)sc0 * i0 + (int32_t)sc1 * i1;
        summ += (int32_t)mn0 * bsum32(a, 2 * g) + (int32_t)mn1 * bsum32(a, 2 * g + 1);
    }
    *sumi_out = sumi;
    *summ_out = summ;
}

/* crates/rnb-cpu/src/gemm/neon_dot.rs:884-916 (dot_q4_k_q8k_scalar);
 * same block formula as the test oracle crates/rnb-cpu/src/gemm/tile_q4k.rs:1749-1800 */
float rnbo_dot_q4k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q4_K_BLOCK_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        int32_t sumi, summ;
        q4k_block_ints(blk, &act[b], &sumi, &summ);
        volatile float t0 = d * (float)sumi;
        volatile float t1 = dmin * (float)summ;
        volatile float t2 = t0 - t1;
        volatile float t3 = act[b].d * t2;
        acc += t3;
    }
    return acc;
}

double rnbo_dot_q4k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q4_K_BLOCK_BYTES;
        double d = rd_f16(blk), dmin = rd_f16(blk + 2);
        int32_t sumi, summ;
        q4k_block_ints(blk, &act[b], &sumi, &summ);
        acc += (double)act[b].d * (d * (double)sumi - dmin * (double)summ);
    }
    return acc;
}

/* integer parts of one Q2_K block: crates/rnb-cpu/src/gemm/avx2_dot.rs:169-242 (sub-block scales times 16-element
 * dots; mins times the Q8_K block's 16-element sums) */
static inline void q2k_block_ints(const uint8_t *blk, const rnbo_q8k_block *a, int32_t *sumi_out,
                                  int32_t *summ_out) {
    const uint8_t *qs = blk + 16;
    int32_t sumi = 0, summ = 0;
    for (int j = 0; j < 16; j++) {
        int q_base = (j / 8) * 32 + (j % 2) * 16, shift = ((j % 8) / 2) * 2;
        int32_t p = 0;
        for (int l = 0; l < 16; l++) p += (int32_t)((qs[q_base + l] >> shift) & 3) * (int32_t)a->qs[16 * j + l];
        sumi += (int32_t)(blk[j] & 0x0f) * p;
        summ += (int32_t)(blk[j] >> 4) * (int32_t)a->bsums[j];
    }
    *sumi_out = sumi;
    *summ_out = summ;
}

/* crates/rnb-cpu/src/gemm/avx2_dot.rs:169-242 (dot_q2k_q8k_avx2): per block acc += (-d_x * dmin) * summ, then
 * acc += (d_x * d) * sumi.  The reference keeps eight f32 lanes and adds them at the end; this form adds in block
 * order -- the difference is f32 summation order only. */
float rnbo_dot_q2k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q2_K_BLOCK_BYTES;
        int32_t sumi, summ;
        q2k_block_ints(blk, &act[b], &sumi, &summ);
        volatile float d = act[b].d * rd_f16(blk + 80);
        volatile float dmin = act[b].d * rd_f16(blk + 82);
        volatile float t1 = dmin * (float)summ;
        volatile float t0 = d * (float)sumi;
        acc -= t1;
        acc += t0;
    }
    return acc;
}

double rnbo_dot_q2k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q2_K_BLOCK_BYTES;
        int32_t sumi, summ;
        q2k_block_ints(blk, &act[b], &sumi, &summ);
        acc += (double)act[b].d * ((double)rd_f16(blk + 80) * (double)sumi - (double)rd_f16(blk + 82) * (double)summ);
    }
    return acc;
}

/* integer part of one Q3_K block: crates/rnb-cpu/src/gemm/avx2_dot.rs:247-375 */
static inline int32_t q3k_block_int(const uint8_t *blk, const rnbo_q8k_block *a) {
    const uint8_t *hm = blk, *q = blk + 32;
    int8_t scales[16];
    q3k_scales(blk + 96, scales);
    int32_t sumi = 0;
    for (int j = 0; j < 16; j++) {
        int n = j / 8, pair = (j % 8) / 2, h = j % 2;
        uint8_t m = (uint8_t)(1u << (4 * n + pair));
        int32_t p = 0;
        for (int l = 0; l < 16; l++) {
            int qv = (q[32 * n + 16 * h + l] >> (2 * pair)) & 3;
            int hv = (hm[16 * h + l] & m) ? 0 : 4;
            p += (int32_t)(qv - hv) * (int32_t)a->qs[16 * j + l];
        }
        sumi += ((int32_t)scales[j] - 32) * p;
    }
    return sumi;
}

/* crates/rnb-cpu/src/gemm/avx2_dot.rs:247-375 (dot_q3k_q8k_avx2): acc += (d_x * d) * sumi per block */
float rnbo_dot_q3k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q3_K_BLOCK_BYTES;
        int32_t sumi = q3k_block_int(blk, &act[b]);
        volatile float d = act[b].d * rd_f16(blk + 108);
        volatile float t = d * (float)sumi;
        acc += t;
    }
    return acc;
}

double rnbo_dot_q3k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q3_K_BLOCK_BYTES;
        acc += (double)act[b].d * (double)rd_f16(blk + 108) * (double)q3k_block_int(blk, &act[b]);
    }
    return acc;
}

/* integer part of one Q5_K block: crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800 */
static inline void q5k_block_ints(const uint8_t *blk, const rnbo_q8k_block *a, int32_t *sumi_out,
                                  int32_t *summ_out) {
    const uint8_t *qh = blk + 16, *qs = blk + 48;
    int32_t sumi = 0, summ = 0;
    for (int g = 0; g < 4; g++) {
        uint8_t sc0, mn0, sc1, mn1;
        rnbo_get_scale_min_k4(2 * g, blk + 4, &sc0, &mn0);
        rnbo_get_scale_min_k4(2 * g + 1, blk + 4, &sc1, &mn1);
        const uint8_t u1 = (uint8_t)(1u << (2 * g)), u2 = (uint8_t)(2u << (2 * g));
        int32_t i0 = 0, i1 = 0;
        for (int l = 0; l < 32; l++) {
            int32_t w0 = (int32_t)(qs[32 * g + l] & 0x0f) + ((qh[l] & u1) ? 16 : 0);
            int32_t w1 = (int32_t)(qs[32 * g + l] >> 4) + ((qh[l] & u2) ? 16 : 0);
            i0 += w0 * (int32_t)a->qs[64 * g + l];
            i1 += w1 * (int32_t)a->qs[64 * g + 32 + l];
        }
        sumi += (int32_t)sc0 * i0 + (int32_t)sc1 * i1;
        summ += (int32_t)mn0 * bsum32(a, 2 * g) + (int32_t)mn1 * bsum32(a, 2 * g + 1);
    }
    *sumi_out = sumi;
    *summ_out = summ;
}

/* crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800 (dot_q5_k_q8k_scalar); the same per-block formula as the
 * test oracle crates/rnb-cpu/src/gemm/tile_q5k.rs:979-1036 (q5k_q8k_exact_ref) */
float rnbo_dot_q5k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q5_K_BLOCK_BYTES;
        float d = rd_f16(blk), dmin = rd_f16(blk + 2);
        int32_t sumi, summ;
        q5k_block_ints(blk, &act[b], &sumi, &summ);
        volatile float t0 = d * (float)sumi;
        volatile float t1 = dmin * (float)summ;
        volatile float t2 = t0 - t1;
        volatile float t3 = act[b].d * t2;
        acc += t3;
    }
    return acc;
}

double rnbo_dot_q5k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q5_K_BLOCK_BYTES;
        double d = rd_f16(blk), dmin = rd_f16(blk + 2);
        int32_t sumi, summ;
        q5k_block_ints(blk, &act[b], &sumi, &summ);
        acc += (double)act[b].d * (d * (double)sumi - dmin * (double)summ);
    }
    return acc;
}

/* integer part of one Q6_K block: crates/rnb-cpu/src/gemm/neon_dot.rs:2240-2288 */
static inline int32_t q6k_block_int(const uint8_t *blk, const rnbo_q8k_block *a) {
    const uint8_t *ql = blk, *qh = blk + 128;
    const int8_t *s = (const int8_t *)(blk + 192);
    int32_t sumi = 0;
    for (int n = 0; n < 2; n++) {
        for (int l = 0; l < 32; l++) {
            int is = l / 16;
            uint8_t h = qh[32 * n + l];
            int q1 = ((ql[64 * n + l] & 0x0f) | ((h & 3) << 4)) - 32;
            int q2 = ((ql[64 * n + l + 32] & 0x0f) | (((h >> 2) & 3) << 4)) - 32;
            int q3 = ((ql[64 * n + l] >> 4) | (((h >> 4) & 3) << 4)) - 32;
            int q4 = ((ql[64 * n + l + 32] >> 4) | (((h >> 6) & 3) << 4)) - 32;
            sumi += (int32_t)s[8 * n + is] * q1 * (int32_t)a->qs[128 * n + l];
            sumi += (int32_t)s[8 * n + is + 2] * q2 * (int32_t)a->qs[128 * n + l + 32];
            sumi += (int32_t)s[8 * n + is + 4] * q3 * (int32_t)a->qs[128 * n + l + 64];
            sumi += (int32_t)s[8 * n + is + 6] * q4 * (int32_t)a->qs[128 * n + l + 96];
        }
    }
    return sumi;
}

/* crates/rnb-cpu/src/gemm/neon_dot.rs:2240-2288 (dot_q6_k_q8k_scalar) */
float rnbo_dot_q6k_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q6_K_BLOCK_BYTES;
        float d = rd_f16(blk + 208);
        int32_t sumi = q6k_block_int(blk, &act[b]);
        volatile float t0 = d * act[b].d;
        volatile float t1 = t0 * (float)sumi;
        acc += t1;
    }
    return acc;
}

double rnbo_dot_q6k_q8k_f64(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q6_K_BLOCK_BYTES;
        double d = rd_f16(blk + 208);
        acc += d * (double)act[b].d * (double)q6k_block_int(blk, &act[b]);
    }
    return acc;
}

/* crates/rnb-cpu/src/gemm/neon_dot.rs:376-436 (dot_q8_0_q8_neon): per block
 * acc += (f16(d_w) * d_x) * (f32)sum_i w_i*x_i, integer sum exact.  The NEON code keeps two
 * f32 accumulators (even/odd blocks) and adds them at the end; this scalar form adds in
 * block order -- the difference is f32 add order only. */
float rnbo_dot_q8_0_q8(const uint8_t *row, const rnbo_q8_block *act, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q8_0_BLOCK_BYTES;
        float d = rd_f16(blk);
        int32_t p = 0;
        for (int i = 0; i < 32; i++) p += (int32_t)(int8_t)blk[2 + i] * (int32_t)act[b].qs[i];
        volatile float s = d * act[b].d;
        volatile float t = (float)p * s;
        acc += t;
    }
    return acc;
}

double rnbo_dot_q8_0_q8_f64(const uint8_t *row, const rnbo_q8_block *act, size_t nb) {
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q8_0_BLOCK_BYTES;
        double d = rd_f16(blk);
        int32_t p = 0;
        for (int i = 0; i < 32; i++) p += (int32_t)(int8_t)blk[2 + i] * (int32_t)act[b].qs[i];
        acc += d * (double)act[b].d * (double)p;
    }
    return acc;
}

/* Q4_0 / Q5_0 x Q8: crates/rnb-cpu/src/gemm/neon_dot.rs:83-137, 163-214: acc += (f32)sum((code - offset) * q) *
 * (d * d_x).  Q4_1 / Q5_1 x Q8: crates/rnb-cpu/src/gemm/neon_quant.rs:88-158: acc += d_x * (d * (f32)sum(code * q) +
 * m * (f32)sum(q)).  Integer sums exact; the two-accumulator NEON forms differ by f32 add order only. */
static inline void legacy_block_ints(const legacy_fmt *f, const uint8_t *blk, const rnbo_q8_block *a, int32_t *dot,
                                     int32_t *sum) {
    int32_t p = 0, sq = 0;
    for (int e = 0; e < 32; e++) {
        p += (int32_t)(legacy_code(f, blk, e) - f->offset) * (int32_t)a->qs[e];
        sq += (int32_t)a->qs[e];
    }
    *dot = p;
    *sum = sq;
}

float rnbo_dot_legacy_q8(uint32_t quant, const uint8_t *row, const rnbo_q8_block *act, size_t nb) {
    legacy_fmt f;
    if (!legacy_format(quant, &f)) return NAN;
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * (size_t)f.bytes;
        int32_t p, sq;
        legacy_block_ints(&f, blk, &act[b], &p, &sq);
        float d = rd_f16(blk);
        if (f.has_min) {
            volatile float t0 = d * (float)p;
            volatile float t1 = rd_f16(blk + 2) * (float)sq;
            volatile float t2 = t0 + t1;
            volatile float t3 = act[b].d * t2;
            acc += t3;
        } else {
            volatile float sc = d * act[b].d;
            volatile float t = (float)p * sc;
            acc += t;
        }
    }
    return acc;
}

double rnbo_dot_legacy_q8_f64(uint32_t quant, const uint8_t *row, const rnbo_q8_block *act, size_t nb) {
    legacy_fmt f;
    if (!legacy_format(quant, &f)) return NAN;
    double acc = 0.0;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * (size_t)f.bytes;
        int32_t p, sq;
        legacy_block_ints(&f, blk, &act[b], &p, &sq);
        double m = f.has_min ? (double)rd_f16(blk + 2) : 0.0;
        acc += (double)act[b].d * ((double)rd_f16(blk) * (double)p + m * (double)sq);
    }
    return acc;
}

/* crates/rnb-cpu/src/gemm/quant_gemv.rs:127-141 (dot_q8_0_row): f32 activations */
float rnbo_dot_q8_0_f32(const uint8_t *row, const float *x, size_t nb) {
    float acc = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_Q8_0_BLOCK_BYTES;
        float d = rd_f16(blk);
        float block_sum = 0.0f;
        for (int i = 0; i < 32; i++) {
            volatile float p = (float)(int8_t)blk[2 + i] * x[b * 32 + i];
            block_sum += p;
        }
        volatile float t = d * block_sum;
        acc += t;
    }
    return acc;
}

/* ================================================================================ */
/* Drivers: crates/rnb-cpu/src/gemm/quant_gemv.rs:360-536, 1104-1196                 */
/* each token quantised once; rows independent; out[s*rows + row]                    */
/* ================================================================================ */

static size_t block_bytes_of(uint32_t quant, size_t *elems) {
    switch (quant) {
    case 2: *elems = 32; return RNBO_Q4_0_BLOCK_BYTES;
    case 3: *elems = 32; return RNBO_Q4_1_BLOCK_BYTES;
    case 6: *elems = 32; return RNBO_Q5_0_BLOCK_BYTES;
    case 7: *elems = 32; return RNBO_Q5_1_BLOCK_BYTES;
    case 8: *elems = 32; return RNBO_Q8_0_BLOCK_BYTES;
    case 9: *elems = 32; return RNBO_Q8_1_BLOCK_BYTES;
    case 10: *elems = 256; return RNBO_Q2_K_BLOCK_BYTES;
    case 11: *elems = 256; return RNBO_Q3_K_BLOCK_BYTES;
    case 12: *elems = 256; return RNBO_Q4_K_BLOCK_BYTES;
    case 13: *elems = 256; return RNBO_Q5_K_BLOCK_BYTES;
    case 14: *elems = 256; return RNBO_Q6_K_BLOCK_BYTES;
    case 16: *elems = 256; return RNBO_IQ2_XXS_BLOCK_BYTES;
    case 18: *elems = 256; return RNBO_IQ3_XXS_BLOCK_BYTES;
    case 22: *elems = 256; return RNBO_IQ2_S_BLOCK_BYTES;
    case 23: *elems = 256; return RNBO_IQ4_XS_BLOCK_BYTES;
    default: *elems = 0; return 0;
    }
}

static float kquant_dot(uint32_t quant, const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    switch (quant) {
    case 10: return rnbo_dot_q2k_q8k(row, act, nb);
    case 11: return rnbo_dot_q3k_q8k(row, act, nb);
    case 12: return rnbo_dot_q4k_q8k(row, act, nb);
    case 13: return rnbo_dot_q5k_q8k(row, act, nb);
    case 16: case 18: case 22: case 23: return rnbo_dot_iq_q8k(quant, row, act, nb);
    default: return rnbo_dot_q6k_q8k(row, act, nb);
    }
}

static double kquant_dot_f64(uint32_t quant, const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    switch (quant) {
    case 10: return rnbo_dot_q2k_q8k_f64(row, act, nb);
    case 11: return rnbo_dot_q3k_q8k_f64(row, act, nb);
    case 12: return rnbo_dot_q4k_q8k_f64(row, act, nb);
    case 13: return rnbo_dot_q5k_q8k_f64(row, act, nb);
    case 16: case 18: case 22: case 23: return rnbo_dot_iq_q8k_f64(quant, row, act, nb);
    default: return rnbo_dot_q6k_q8k_f64(row, act, nb);
    }
}

static int resolve_threads(int n_threads) {
#ifdef _OPENMP
    if (n_threads <= 0) n_threads = omp_get_max_threads();
#else
    n_threads = 1;
#endif
    return n_threads < 1 ? 1 : n_threads;
}

int rnbo_gemv(uint32_t quant, const uint8_t *w, size_t rows, size_t cols, const float *x,
              size_t seq_len, float *out, int n_threads) {
    size_t elems;
    size_t bb = block_bytes_of(quant, &elems);
    if (bb == 0 || cols % elems != 0) return 1;
    size_t nb = cols / elems, row_bytes = nb * bb;
    n_threads = resolve_threads(n_threads);
    if (elems == 32) {
        rnbo_q8_block *act = (rnbo_q8_block *)malloc(sizeof(rnbo_q8_block) * nb * seq_len);
        if (!act) return 2;
        for (size_t s = 0; s < seq_len; s++) rnbo_quantize_q8(x + s * cols, cols, act + s * nb);
#pragma omp parallel for schedule(static) num_threads(n_threads)
        for (long r = 0; r < (long)rows; r++)
            for (size_t s = 0; s < seq_len; s++)
                out[s * rows + r] = quant == 8 ? rnbo_dot_q8_0_q8(w + r * row_bytes, act + s * nb, nb)
                                               : rnbo_dot_legacy_q8(quant, w + r * row_bytes, act + s * nb, nb);
        free(act);
        return 0;
    }
    rnbo_q8k_block *act = (rnbo_q8k_block *)malloc(sizeof(rnbo_q8k_block) * nb * seq_len);
    if (!act) return 2;
    for (size_t s = 0; s < seq_len; s++) rnbo_quantize_q8k(x + s * cols, cols, act + s * nb);
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long r = 0; r < (long)rows; r++)
        for (size_t s = 0; s < seq_len; s++)
            out[s * rows + r] = kquant_dot(quant, w + r * row_bytes, act + s * nb, nb);
    free(act);
    return 0;
}

int rnbo_gemv_f64(uint32_t quant, const uint8_t *w, size_t rows, size_t cols, const float *x,
                  size_t seq_len, double *out, int n_threads) {
    size_t elems;
    size_t bb = block_bytes_of(quant, &elems);
    if (bb == 0 || cols % elems != 0) return 1;
    size_t nb = cols / elems, row_bytes = nb * bb;
    n_threads = resolve_threads(n_threads);
    if (elems == 32) {
        rnbo_q8_block *act = (rnbo_q8_block *)malloc(sizeof(rnbo_q8_block) * nb * seq_len);
        if (!act) return 2;
        for (size_t s = 0; s < seq_len; s++) rnbo_quantize_q8(x + s * cols, cols, act + s * nb);
#pragma omp parallel for schedule(static) num_threads(n_threads)
        for (long r = 0; r < (long)rows; r++)
            for (size_t s = 0; s < seq_len; s++)
                out[s * rows + r] = quant == 8 ? rnbo_dot_q8_0_q8_f64(w + r * row_bytes, act + s * nb, nb)
                                               : rnbo_dot_legacy_q8_f64(quant, w + r * row_bytes, act + s * nb, nb);
        free(act);
        return 0;
    }
    rnbo_q8k_block *act = (rnbo_q8k_block *)malloc(sizeof(rnbo_q8k_block) * nb * seq_len);
    if (!act) return 2;
    for (size_t s = 0; s < seq_len; s++) rnbo_quantize_q8k(x + s * cols, cols, act + s * nb);
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long r = 0; r < (long)rows; r++)
        for (size_t s = 0; s < seq_len; s++)
            out[s * rows + r] = kquant_dot_f64(quant, w + r * row_bytes, act + s * nb, nb);
    free(act);
    return 0;
}

/* crates/rnb-cpu/src/gemm/quant_gemv.rs:360-401 (gemv_q8_0, the x86 default) */
int rnbo_gemv_q8_0_f32act(const uint8_t *w, size_t rows, size_t cols, const float *x,
                          size_t seq_len, float *out, int n_threads) {
    if (cols % 32 != 0) return 1;
    size_t nb = cols / 32, row_bytes = nb * RNBO_Q8_0_BLOCK_BYTES;
    n_threads = resolve_threads(n_threads);
#pragma omp parallel for schedule(static) num_threads(n_threads)
    for (long r = 0; r < (long)rows; r++)
        for (size_t s = 0; s < seq_len; s++)
            out[s * rows + r] = rnbo_dot_q8_0_f32(w + r * row_bytes, x + s * cols, nb);
    return 0;
}

/* ================================================================================ */
/* MoE                                                                               */
/* ================================================================================ */

/* crates/rnb-cpu/src/kernels/activation.rs:73-89 (fused_silu_mul_inplace) */
void rnbo_silu_mul_inplace(float *gate, const float *up, size_t n) {
    for (size_t i = 0; i < n; i++) {
        float g = gate[i];
        volatile float e = expf(-g);
        volatile float den = 1.0f + e;
        volatile float s = g / den;
        volatile float r = s * up[i];
        gate[i] = r;
    }
}

/* crates/rnb-cpu/src/kernels/activation.rs:91-98 (fused_gelu_mul_inplace): tanh form,
 * 0.5 * g * (1 + tanh(sqrt(2/pi) * (g + 0.044715 * g^3))) * up, every step rounded to f32 */
void rnbo_gelu_mul_inplace(float *gate, const float *up, size_t n) {
    const float sqrt_2_over_pi = sqrtf(2.0f / 3.14159265358979323846f);
    for (size_t i = 0; i < n; i++) {
        float g = gate[i];
        volatile float g2 = g * g;
        volatile float g3 = g2 * g;
        volatile float c = 0.044715f * g3;
        volatile float inner = g + c;
        volatile float arg = sqrt_2_over_pi * inner;
        volatile float t = tanhf(arg);
        volatile float one = 1.0f + t;
        volatile float half = 0.5f * g;
        volatile float act = half * one;
        volatile float r = act * up[i];
        gate[i] = r;
    }
}

/* crates/rnb-llm/src/engine/models/shared_expert_moe/routing.rs:18-64
 * (qwen35_select_topk_logits_bounded): insertion into a sorted list, ties -> lower id,
 * softmax over the selected logits, output sorted by logit descending. */
size_t rnbo_route_topk(const float *logits, size_t n_expert, size_t k, uint32_t *idx_out,
                       float *weights_out) {
    size_t sel = k < n_expert ? k : n_expert;
    if (sel == 0) return 0;
    if (sel > 32) sel = 32;
    float best_vals[32];
    size_t best_ids[32];
    for (size_t i = 0; i < 32; i++) {
        best_vals[i] = -INFINITY;
        best_ids[i] = (size_t)-1;
    }
    for (size_t e = 0; e < n_expert; e++) {
        float v = logits[e];
        for (size_t rank = 0; rank < sel; rank++) {
            if (v > best_vals[rank] || (v == best_vals[rank] && e < best_ids[rank])) {
                for (size_t sh = sel - 1; sh > rank; sh--) {
                    best_vals[sh] = best_vals[sh - 1];
                    best_ids[sh] = best_ids[sh - 1];
                }
                best_vals[rank] = v;
                best_ids[rank] = e;
                break;
            }
        }
    }
    float mx = best_vals[0], sum = 0.0f;
    for (size_t r = 0; r < sel; r++) {
        float wv = expf(best_vals[r] - mx);
        idx_out[r] = (uint32_t)best_ids[r];
        weights_out[r] = wv;
        sum += wv;
    }
    if (sum != 0.0f)
        for (size_t r = 0; r < sel; r++) weights_out[r] /= sum;
    return sel;
}

/* One slot: crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:260-327
 * (compute_expert_host_from_slices): gate/up GEMV on Q8_K(h), SiLU*up, down GEMV on the
 * re-quantised intermediate, scale by the route weight.  Gate/up are Q4_K; down is
 * Q4_K (12), Q5_K (13) or Q6_K (14).  `h_q8k` is the token's already-quantised activation. */
typedef float (*moe_dot_fn)(const uint8_t *row, const rnbo_q8k_block *act, size_t nb);

static void moe_slot(const uint8_t *gate, const uint8_t *up, const uint8_t *down,
                     uint32_t down_quant, size_t n_ff, size_t n_embd, const rnbo_q8k_block *h_q8k,
                     float route_weight, float *gate_out, float *up_out, rnbo_q8k_block *mid_q8k,
                     float *expert_out, moe_dot_fn gate_dot, moe_dot_fn down_dot) {
    size_t nb_in = n_embd / 256, nb_mid = n_ff / 256;
    size_t gate_row = nb_in * RNBO_Q4_K_BLOCK_BYTES;
    for (size_t r = 0; r < n_ff; r++) {
        gate_out[r] = gate_dot(gate + r * gate_row, h_q8k, nb_in);
        up_out[r] = gate_dot(up + r * gate_row, h_q8k, nb_in);
    }
    rnbo_silu_mul_inplace(gate_out, up_out, n_ff);
    rnbo_quantize_q8k(gate_out, n_ff, mid_q8k);
    size_t elems;
    size_t down_row = nb_mid * block_bytes_of(down_quant, &elems);
    for (size_t r = 0; r < n_embd; r++) {
        float o = down_dot ? down_dot(down + r * down_row, mid_q8k, nb_mid)
                           : kquant_dot(down_quant, down + r * down_row, mid_q8k, nb_mid);
        volatile float scaled = o * route_weight; /* fanout.rs:306-308 */
        expert_out[r] = scaled;
    }
}

/* Whole-layer tensors + per-slot (expert, token, weight): the `selected_base_by_token` form of
 * crates/rnb-backend/cuda/src/runtime/api/qwen_moe_api.rs:2529-2541.  Per token the scaled
 * expert outputs are added in slot order (decode: crates/rnb-llm/.../moe_view.rs:416-426;
 * batched: .../prefill_cpu.rs:167-194 adds in rank order, which is slot order when the caller
 * lists a token's slots by rank). */
static int moe_by_token(const uint8_t *gate_all, const uint8_t *up_all, const uint8_t *down_all,
                        size_t n_expert, const uint32_t *expert_ids, const float *route,
                        const uint32_t *token_ids, size_t n_slots, size_t token_count,
                        uint32_t down_quant, size_t n_ff, size_t n_embd, const float *x, float *out,
                        int n_threads, moe_dot_fn gate_dot, moe_dot_fn down_dot) {
    if (n_ff % 256 != 0 || n_embd % 256 != 0) return 1;
    if (down_quant != 12 && down_quant != 13 && down_quant != 14) return 1;
    for (size_t s = 0; s < n_slots; s++)
        if (expert_ids[s] >= n_expert || token_ids[s] >= token_count) return 1;
    size_t nb_in = n_embd / 256, nb_mid = n_ff / 256;
    size_t per_gate = n_ff * nb_in * RNBO_Q4_K_BLOCK_BYTES;
    size_t down_elems;
    size_t per_down = n_embd * nb_mid * block_bytes_of(down_quant, &down_elems);
    n_threads = resolve_threads(n_threads);

    rnbo_q8k_block *h_q8k = (rnbo_q8k_block *)malloc(sizeof(rnbo_q8k_block) * nb_in * token_count);
    float *slot_out = (float *)malloc(sizeof(float) * n_embd * (n_slots ? n_slots : 1));
    if (!h_q8k || !slot_out) {
        free(h_q8k);
        free(slot_out);
        return 2;
    }
    for (size_t t = 0; t < token_count; t++)
        rnbo_quantize_q8k(x + t * n_embd, n_embd, h_q8k + t * nb_in);

#pragma omp parallel num_threads(n_threads)
    {
        float *gate_out = (float *)malloc(sizeof(float) * n_ff);
        float *up_out = (float *)malloc(sizeof(float) * n_ff);
        rnbo_q8k_block *mid = (rnbo_q8k_block *)malloc(sizeof(rnbo_q8k_block) * nb_mid);
#pragma omp for schedule(dynamic, 1)
        for (long s = 0; s < (long)n_slots; s++) {
            size_t e = expert_ids[s];
            moe_slot(gate_all + e * per_gate, up_all + e * per_gate, down_all + e * per_down,
                     down_quant, n_ff, n_embd, h_q8k + (size_t)token_ids[s] * nb_in, route[s],
                     gate_out, up_out, mid, slot_out + (size_t)s * n_embd, gate_dot, down_dot);
        }
        free(gate_out);
        free(up_out);
        free(mid);
    }
    memset(out, 0, sizeof(float) * token_count * n_embd);
    for (size_t s = 0; s < n_slots; s++) {
        float *dst = out + (size_t)token_ids[s] * n_embd;
        const float *src = slot_out + s * n_embd;
        for (size_t i = 0; i < n_embd; i++) dst[i] += src[i];
    }
    free(h_q8k);
    free(slot_out);
    return 0;
}

int rnbo_moe_sparse_experts_by_token(const uint8_t *gate_all, const uint8_t *up_all,
                                     const uint8_t *down_all, size_t n_expert,
                                     const uint32_t *expert_ids, const float *route,
                                     const uint32_t *token_ids, size_t n_slots, size_t token_count,
                                     uint32_t down_quant, size_t n_ff, size_t n_embd,
                                     const float *x, float *out, int n_threads) {
    return moe_by_token(gate_all, up_all, down_all, n_expert, expert_ids, route, token_ids, n_slots,
                        token_count, down_quant, n_ff, n_embd, x, out, n_threads, rnbo_dot_q4k_q8k, NULL);
}

/* The same call over the AVX2+FMA block dots (Q4_K gate/up; Q6_K down, the other down formats keep
 * the scalar dot): what rnb-cpu runs on x86_64, timed as the CPU baseline of the MoE configurations.
 * Integer sums are the scalar form's; the f32 accumulation order inside a row differs, so an
 * intermediate on a rounding tie can re-quantise to the neighbouring int8. */
int rnbo_moe_sparse_experts_by_token_avx2(const uint8_t *gate_all, const uint8_t *up_all,
                                          const uint8_t *down_all, size_t n_expert,
                                          const uint32_t *expert_ids, const float *route,
                                          const uint32_t *token_ids, size_t n_slots,
                                          size_t token_count, uint32_t down_quant, size_t n_ff,
                                          size_t n_embd, const float *x, float *out, int n_threads) {
    if (!rnbo_have_avx2()) return 3;
    return moe_by_token(gate_all, up_all, down_all, n_expert, expert_ids, route, token_ids, n_slots,
                        token_count, down_quant, n_ff, n_embd, x, out, n_threads, rnbo_dot_q4k_q8k_avx2,
                        down_quant == 12 ? rnbo_dot_q4k_q8k_avx2
                                         : (down_quant == 14 ? rnbo_dot_q6k_q8k_avx2 : NULL));
}

/* ================================================================================ */
/* Input generation                                                                  */
/* ================================================================================ */

/* crates/rnb-cpu/src/quantize/quant.rs:189-280 (make_qkx2_quants), use_mad = false */
static float make_qkx2_quants(int n, int nmax, const float *x, const float *weights, uint8_t *L,
                              float *the_min, uint8_t *Laux, float rmin, float rdelta, int nstep) {
    float min = x[0], max = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; i++) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0.0f) min = 0.0f;
    if (max == min) {
        for (int i = 0; i < n; i++) L[i] = 0;
        *the_min = -min;
        return 0.0f;
    }
    float iscale = (float)nmax / (max - min);
    float scale = 1.0f / iscale;
    float best_error = 0.0f;
    for (int i = 0; i < n; i++) {
        int l = rnbo_nearest_int(iscale * (x[i] - min));
        l = l < 0 ? 0 : (l > nmax ? nmax : l);
        L[i] = (uint8_t)l;
        float diff = scale * (float)l + min - x[i];
        diff = diff * diff;
        best_error += weights[i] * diff;
    }
    if (nstep < 1) {
        *the_min = -min;
        return scale;
    }
    for (int is = 0; is <= nstep; is++) {
        iscale = (rmin + rdelta * (float)is + (float)nmax) / (max - min);
        float sum_l = 0.0f, sum_l2 = 0.0f, sum_xl = 0.0f;
        for (int i = 0; i < n; i++) {
            int l = rnbo_nearest_int(iscale * (x[i] - min));
            l = l < 0 ? 0 : (l > nmax ? nmax : l);
            Laux[i] = (uint8_t)l;
            float w = weights[i];
            sum_l += w * (float)l;
            sum_l2 += w * (float)l * (float)l;
            sum_xl += w * (float)l * x[i];
        }
        float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0.0f) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0.0f) {
                this_min = 0.0f;
                this_scale = sum_xl / sum_l2;
            }
            float cur_error = 0.0f;
            for (int i = 0; i < n; i++) {
                float diff = this_scale * (float)Laux[i] + this_min - x[i];
                diff = diff * diff;
                cur_error += weights[i] * diff;
            }
            if (cur_error < best_error) {
                memcpy(L, Laux, (size_t)n);
                best_error = cur_error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

/* Shared front half of the Q4_K and Q5_K quantisers (crates/rnb-cpu/src/quantize/quant.rs:312-378 and
 * :456-545, which differ only in nmax = 15 / 31): per-sub-block fit, 6-bit packing of the sub-block
 * scales and mins into `ys`, f16 super-block scales into hdr[0..4), then the element codes L re-derived
 * from the rounded scales. */
static void kquant_min_codes(const float *x, int nmax, uint8_t *hdr, uint8_t *ys, uint8_t *L) {
    uint8_t Laux[32];
    float mins[8], scales[8], weights[32];
    float max_scale = 0.0f, max_min = 0.0f;
    for (int j = 0; j < 8; j++) {
        const float *xs = x + 32 * j;
        float sum_x2 = 0.0f;
        for (int l = 0; l < 32; l++) sum_x2 += xs[l] * xs[l];
        float av_x = sqrtf(sum_x2 / 32.0f);
        for (int l = 0; l < 32; l++) weights[l] = av_x + fabsf(xs[l]);
        float sub_min = 0.0f;
        float s = make_qkx2_quants(32, nmax, xs, weights, L + 32 * j, &sub_min, Laux, -0.5f, 0.1f, 15);
        scales[j] = s;
        mins[j] = sub_min;
        if (s > max_scale) max_scale = s;
        if (sub_min > max_min) max_min = sub_min;
    }
    float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
    float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
    memset(ys, 0, 12);
    for (int j = 0; j < 8; j++) {
        int ls = rnbo_nearest_int(inv_scale * scales[j]);
        int lm = rnbo_nearest_int(inv_min * mins[j]);
        ls = ls < 0 ? 0 : (ls > 63 ? 63 : ls);
        lm = lm < 0 ? 0 : (lm > 63 ? 63 : lm);
        if (j < 4) {
            ys[j] = (uint8_t)ls;
            ys[j + 4] = (uint8_t)lm;
        } else {
            ys[j + 4] = (uint8_t)((ls & 0x0f) | ((lm & 0x0f) << 4));
            ys[j - 4] |= (uint8_t)((ls >> 4) << 6);
            ys[j] |= (uint8_t)((lm >> 4) << 6);
        }
    }
    wr_f16(hdr, max_scale / 63.0f);
    wr_f16(hdr + 2, max_min / 63.0f);
    float d_round = rd_f16(hdr), dmin_round = rd_f16(hdr + 2);
    for (int j = 0; j < 8; j++) {
        uint8_t sc, mn;
        rnbo_get_scale_min_k4(j, ys, &sc, &mn);
        float d_sub = d_round * (float)sc;
        if (d_sub == 0.0f) continue;
        float dm_sub = dmin_round * (float)mn;
        for (int ii = 0; ii < 32; ii++) {
            int l = rnbo_nearest_int((x[32 * j + ii] + dm_sub) / d_sub);
            L[32 * j + ii] = (uint8_t)(l < 0 ? 0 : (l > nmax ? nmax : l));
        }
    }
}

/* crates/rnb-cpu/src/quantize/quant.rs:289-413 (quantize_row_q4_k).
 * Byte parity with the Rust original is UNPINNED (cannot run it); input generation only. */
void rnbo_quantize_row_q4_k(const float *input, size_t n, uint8_t *output) {
    size_t nb = n / 256;
    uint8_t L[256], ys[12];
    for (size_t i = 0; i < nb; i++) {
        uint8_t *out = output + i * RNBO_Q4_K_BLOCK_BYTES;
        kquant_min_codes(input + i * 256, 15, out, ys, L);
        memcpy(out + 4, ys, 12);
        uint8_t *qs = out + 16;
        for (int g = 0; g < 4; g++)
            for (int j = 0; j < 32; j++)
                qs[32 * g + j] = (uint8_t)((L[64 * g + j] & 0x0f) | ((L[64 * g + j + 32] & 0x0f) << 4));
    }
}

/* crates/rnb-cpu/src/quantize/quant.rs:433-585 (quantize_row_q5_k): 5-bit codes, the low four bits in
 * qs as for Q4_K, the fifth in qh (bit 2g for the first half of group g, bit 2g+1 for the second).
 * Byte parity with the Rust original is UNPINNED (cannot run it); input generation only. */
void rnbo_quantize_row_q5_k(const float *input, size_t n, uint8_t *output) {
    size_t nb = n / 256;
    uint8_t L[256], ys[12];
    for (size_t i = 0; i < nb; i++) {
        uint8_t *out = output + i * RNBO_Q5_K_BLOCK_BYTES;
        kquant_min_codes(input + i * 256, 31, out, ys, L);
        memcpy(out + 4, ys, 12);
        uint8_t *qh = out + 16, *qs = out + 48;
        memset(qh, 0, 32);
        for (int g = 0; g < 4; g++) {
            for (int j = 0; j < 32; j++) {
                int l1 = L[64 * g + j], l2 = L[64 * g + j + 32];
                if (l1 > 15) {
                    l1 -= 16;
                    qh[j] |= (uint8_t)(1u << (2 * g));
                }
                if (l2 > 15) {
                    l2 -= 16;
                    qh[j] |= (uint8_t)(2u << (2 * g));
                }
                qs[32 * g + j] = (uint8_t)(l1 | (l2 << 4));
            }
        }
    }
}

/* crates/rnb-cpu/src/quantize/quant.rs:44-160 (quantize_row_q2_k): min/max fit per 16 elements, 4-bit scale and min
 * codes against d = max scale / 15 and dmin = max min / 15.  Byte parity with the Rust original is UNPINNED
 * (cannot run it); input generation only. */
void rnbo_quantize_row_q2_k(const float *input, size_t n, uint8_t *output) {
    const float eps = 1e-10f;
    for (size_t sb = 0; sb < n / 256; sb++) {
        const float *x = input + sb * 256;
        uint8_t *out = output + sb * RNBO_Q2_K_BLOCK_BYTES;
        float sub_scale[16], sub_min[16];
        uint8_t q[256];
        memset(q, 0, sizeof q);
        for (int j = 0; j < 16; j++) {
            const float *xs = x + 16 * j;
            float lo = xs[0], hi = xs[0];
            for (int l = 1; l < 16; l++) {
                if (xs[l] < lo) lo = xs[l];
                if (xs[l] > hi) hi = xs[l];
            }
            float base = lo <= 0.0f ? lo : 0.0f;
            float range = hi - base;
            sub_scale[j] = range > eps ? range / 3.0f : 0.0f;
            sub_min[j] = -base;
            if (sub_scale[j] > eps)
                for (int l = 0; l < 16; l++) {
                    float r = roundf((xs[l] - base) / sub_scale[j]);
                    q[16 * j + l] = (uint8_t)(r < 0.0f ? 0.0f : (r > 3.0f ? 3.0f : r));
                }
        }
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 16; j++) {
            if (sub_scale[j] > max_scale) max_scale = sub_scale[j];
            if (sub_min[j] > max_min) max_min = sub_min[j];
        }
        float d = max_scale > eps ? max_scale / 15.0f : 0.0f, dmin = max_min > eps ? max_min / 15.0f : 0.0f;
        for (int j = 0; j < 16; j++) {
            float sc = d > eps ? roundf(sub_scale[j] / d) : 0.0f, mn = dmin > eps ? roundf(sub_min[j] / dmin) : 0.0f;
            sc = sc < 0.0f ? 0.0f : (sc > 15.0f ? 15.0f : sc);
            mn = mn < 0.0f ? 0.0f : (mn > 15.0f ? 15.0f : mn);
            out[j] = (uint8_t)(((uint8_t)mn << 4) | ((uint8_t)sc & 0x0f));
        }
        memset(out + 16, 0, 64);
        for (int i = 0; i < 256; i++)
            out[16 + (i / 128) * 32 + i % 32] |= (uint8_t)((q[i] & 3) << (((i % 128) / 32) * 2));
        wr_f16(out + 80, d);
        wr_f16(out + 82, dmin);
    }
}

/* Q3_K generator: NOT in the reference repository.  Symmetric fit per 16 elements (scale = max |x| / 4), 6-bit scale
 * codes 32 + round(scale / d) against d = max scale / 31, values round(x / (d * code)) in -4..3. */
void rnbo_quantize_row_q3_k(const float *input, size_t n, uint8_t *output) {
    for (size_t sb = 0; sb < n / 256; sb++) {
        const float *x = input + sb * 256;
        uint8_t *out = output + sb * RNBO_Q3_K_BLOCK_BYTES;
        float sub_scale[16], max_scale = 0.0f;
        for (int j = 0; j < 16; j++) {
            float amax = 0.0f;
            for (int l = 0; l < 16; l++) amax = fmaxf(amax, fabsf(x[16 * j + l]));
            sub_scale[j] = amax / 4.0f;
            max_scale = fmaxf(max_scale, sub_scale[j]);
        }
        memset(out, 0, RNBO_Q3_K_BLOCK_BYTES);
        wr_f16(out + 108, max_scale / 31.0f);
        float d = rd_f16(out + 108);
        for (int j = 0; j < 16; j++) {
            int code = d > 0.0f ? (int)roundf(sub_scale[j] / d) : 0;
            code = code < 0 ? 0 : (code > 31 ? 31 : code);
            int stored = code + 32; /* 6 bits: low four in byte j%8 (nibble j/8), high two in byte 8 + j%4 */
            if (j < 8)
                out[96 + j] |= (uint8_t)(stored & 0x0f);
            else
                out[96 + j - 8] |= (uint8_t)((stored & 0x0f) << 4);
            out[96 + 8 + (j % 4)] |= (uint8_t)(((stored >> 4) & 3) << (2 * (j / 4)));
            float step = d * (float)code;
            int n_half = j / 8, pair = (j % 8) / 2, h = j % 2;
            for (int l = 0; l < 16; l++) {
                int v = step > 0.0f ? (int)roundf(x[16 * j + l] / step) : 0;
                v = v < -4 ? -4 : (v > 3 ? 3 : v);
                int u = v + 4; /* 0..7: low two bits in qs, the third bit set in hmask */
                out[32 + 32 * n_half + 16 * h + l] |= (uint8_t)((u & 3) << (2 * pair));
                if (u & 4) out[16 * h + l] |= (uint8_t)(1u << (4 * n_half + pair));
            }
        }
    }
}

/* Symmetric fit used by the Q6_K generator (ggml reference `make_qx_quants`, rmse_type 1,
 * no external quant weights: w = x^2).  NOT in the reference repository. */
static float make_qx_quants(int n, int nmax, const float *x, int8_t *L) {
    float max = 0.0f, amax = 0.0f;
    for (int i = 0; i < n; i++) {
        float ax = fabsf(x[i]);
        if (ax > amax) {
            amax = ax;
            max = x[i];
        }
    }
    if (amax < 1e-30f) {
        for (int i = 0; i < n; i++) L[i] = 0;
        return 0.0f;
    }
    float iscale = -(float)nmax / max;
    float sumlx = 0.0f, suml2 = 0.0f;
    for (int i = 0; i < n; i++) {
        int l = rnbo_nearest_int(iscale * x[i]);
        l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
        L[i] = (int8_t)(l + nmax);
        float w = x[i] * x[i];
        sumlx += w * x[i] * (float)l;
        suml2 += w * (float)l * (float)l;
    }
    float scale = suml2 != 0.0f ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; is++) {
        if (is == 0) continue;
        iscale = -((float)nmax + 0.1f * (float)is) / max;
        sumlx = 0.0f;
        suml2 = 0.0f;
        for (int i = 0; i < n; i++) {
            int l = rnbo_nearest_int(iscale * x[i]);
            l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
            float w = x[i] * x[i];
            sumlx += w * x[i] * (float)l;
            suml2 += w * (float)l * (float)l;
        }
        if (suml2 > 0.0f && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; i++) {
                int l = rnbo_nearest_int(iscale * x[i]);
                l = l < -nmax ? -nmax : (l > nmax - 1 ? nmax - 1 : l);
                L[i] = (int8_t)(l + nmax);
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

/* Q6_K weight generator: ggml reference semantics (quantize_row_q6_K_ref); the reference
 * repository has no Q6_K weight quantiser.  Layout is the inverse of
 * crates/rnb-cpu/src/quantize/dequant.rs:780-807. */
void rnbo_quantize_row_q6_k(const float *input, size_t n, uint8_t *output) {
    size_t nb = n / 256;
    int8_t L[256];
    float scales[16];
    for (size_t i = 0; i < nb; i++) {
        const float *x = input + i * 256;
        uint8_t *out = output + i * RNBO_Q6_K_BLOCK_BYTES;
        float max_scale = 0.0f, max_abs_scale = 0.0f;
        for (int ib = 0; ib < 16; ib++) {
            float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
            scales[ib] = scale;
            float abs_scale = fabsf(scale);
            if (abs_scale > max_abs_scale) {
                max_abs_scale = abs_scale;
                max_scale = scale;
            }
        }
        memset(out, 0, RNBO_Q6_K_BLOCK_BYTES);
        if (max_abs_scale < 1e-30f) continue;
        float iscale = -128.0f / max_scale;
        wr_f16(out + 208, 1.0f / iscale);
        float d = rd_f16(out + 208);
        int8_t *sc = (int8_t *)(out + 192);
        for (int ib = 0; ib < 16; ib++) {
            int v = rnbo_nearest_int(iscale * scales[ib]);
            sc[ib] = (int8_t)(v > 127 ? 127 : v);
        }
        for (int j = 0; j < 16; j++) {
            float dd = d * (float)sc[j];
            if (dd == 0.0f) continue;
            for (int ii = 0; ii < 16; ii++) {
                int l = rnbo_nearest_int(x[16 * j + ii] / dd);
                l = l < -32 ? -32 : (l > 31 ? 31 : l);
                L[16 * j + ii] = (int8_t)(l + 32);
            }
        }
        uint8_t *ql = out, *qh = out + 128;
        for (int h = 0; h < 2; h++) {
            for (int l = 0; l < 32; l++) {
                uint8_t q1 = (uint8_t)L[128 * h + l], q2 = (uint8_t)L[128 * h + l + 32];
                uint8_t q3 = (uint8_t)L[128 * h + l + 64], q4 = (uint8_t)L[128 * h + l + 96];
                ql[64 * h + l] = (uint8_t)((q1 & 0x0f) | ((q3 & 0x0f) << 4));
                ql[64 * h + l + 32] = (uint8_t)((q2 & 0x0f) | ((q4 & 0x0f) << 4));
                qh[32 * h + l] =
                    (uint8_t)((q1 >> 4) | ((q2 >> 4) << 2) | ((q3 >> 4) << 4) | ((q4 >> 4) << 6));
            }
        }
    }
}

/* Generators for the 4- and 5-bit 32-element formats: ggml reference semantics (quantize_row_q4_0_ref and
 * siblings: d = signed max / -2^(bits-1) for the _0 formats, (max - min) / (2^bits - 1) with m = min for the _1
 * formats); the reference repository has none.  Input generation only. */
int rnbo_quantize_row_legacy(uint32_t quant, const float *input, size_t n, uint8_t *output) {
    legacy_fmt f;
    if (!legacy_format(quant, &f)) return 1;
    const int top = f.qh_off >= 0 ? 31 : 15;
    for (size_t b = 0; b < n / 32; b++) {
        const float *x = input + b * 32;
        uint8_t *out = output + b * (size_t)f.bytes;
        memset(out, 0, (size_t)f.bytes);
        if (f.byte_codes) { /* Q8_1, ggml reference semantics: d = amax / 127, q = round(x / d), s = d * sum(q) */
            float amax = 0.0f;
            for (int i = 0; i < 32; i++)
                if (fabsf(x[i]) > amax) amax = fabsf(x[i]);
            float d = amax / 127.0f, id = d != 0.0f ? 1.0f / d : 0.0f;
            int sum = 0;
            for (int i = 0; i < 32; i++) {
                int q = (int)roundf(x[i] * id);
                out[f.qs_off + i] = (uint8_t)(int8_t)q;
                sum += q;
            }
            wr_f16(out, d);
            wr_f16(out + 2, d * (float)sum);
            continue;
        }
        float d, base;
        if (f.has_min) {
            float lo = x[0], hi = x[0];
            for (int i = 1; i < 32; i++) {
                if (x[i] < lo) lo = x[i];
                if (x[i] > hi) hi = x[i];
            }
            d = (hi - lo) / (float)top;
            base = lo;
            wr_f16(out + 2, lo);
        } else {
            float amax = 0.0f, vmax = 0.0f;
            for (int i = 0; i < 32; i++)
                if (fabsf(x[i]) > amax) {
                    amax = fabsf(x[i]);
                    vmax = x[i];
                }
            d = vmax / -(float)f.offset;
            base = 0.0f;
        }
        wr_f16(out, d);
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        uint32_t qh = 0;
        for (int e = 0; e < 32; e++) {
            float v = f.has_min ? (x[e] - base) * id + 0.5f : x[e] * id + (float)f.offset + 0.5f;
            int code = (int)v;
            code = code < 0 ? 0 : (code > top ? top : code);
            if (e < 16)
                out[f.qs_off + e] |= (uint8_t)(code & 0x0f);
            else
                out[f.qs_off + e - 16] |= (uint8_t)((code & 0x0f) << 4);
            qh |= (uint32_t)((code >> 4) & 1) << e;
        }
        if (f.qh_off >= 0)
            for (int k = 0; k < 4; k++) out[f.qh_off + k] = (uint8_t)(qh >> (8 * k));
    }
    return 0;
}

/* Q8_0 weight generator: ggml reference semantics (quantize_row_q8_0_ref); the reference
 * repository has no Q8_0 weight quantiser. */
void rnbo_quantize_row_q8_0(const float *input, size_t n, uint8_t *output) {
    size_t nb = n / 32;
    for (size_t b = 0; b < nb; b++) {
        const float *x = input + b * 32;
        uint8_t *out = output + b * RNBO_Q8_0_BLOCK_BYTES;
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) {
            float ax = fabsf(x[i]);
            if (ax > amax) amax = ax;
        }
        float d = amax / 127.0f;
        float id = d != 0.0f ? 1.0f / d : 0.0f;
        wr_f16(out, d);
        for (int i = 0; i < 32; i++) out[2 + i] = (uint8_t)(int8_t)roundf(x[i] * id);
    }
}

/* Counter-based generator: element i of stream `seed` is a pure function of (seed, i), so
 * any slice can be regenerated independently and in parallel.  SplitMix64 finaliser ->
 * two 24-bit uniforms -> Box-Muller in f64 -> f32. */
static inline uint64_t splitmix64(uint64_t z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

static inline float normal_at(uint64_t seed, uint64_t i, float sigma) {
    uint64_t r = splitmix64(seed * 0xd1342543de82ef95ull + i);
    double u1 = ((double)((r >> 40) & 0xffffff) + 1.0) / 16777217.0; /* (0,1) */
    double u2 = (double)((r >> 16) & 0xffffff) / 16777216.0;         /* [0,1) */
    double z = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
    return (float)(z * (double)sigma);
}

void rnbo_fill_normal(float *out, size_t n, uint64_t seed, float sigma) {
    for (size_t i = 0; i < n; i++) out[i] = normal_at(seed, i, sigma);
}

int rnbo_make_weights(uint32_t quant, size_t rows, size_t cols, uint64_t seed, float sigma,
                      uint8_t *out, int n_threads) {
    size_t elems;
    size_t bb = block_bytes_of(quant, &elems);
    if (bb == 0 || cols % elems != 0) return 1;
    size_t row_bytes = cols / elems * bb;
    n_threads = resolve_threads(n_threads);
#pragma omp parallel num_threads(n_threads)
    {
        float *row = (float *)malloc(sizeof(float) * cols);
#pragma omp for schedule(static)
        for (long r = 0; r < (long)rows; r++) {
            for (size_t c = 0; c < cols; c++) row[c] = normal_at(seed, (uint64_t)r * cols + c, sigma);
            uint8_t *dst = out + (size_t)r * row_bytes;
            if (quant == 16 || quant == 18 || quant == 22 || quant == 23)
                rnbo_make_iq_row(quant, cols / 256, seed * 1000003ull + (uint64_t)r, sigma, dst);
            else if (quant == 2 || quant == 3 || quant == 6 || quant == 7 || quant == 9)
                rnbo_quantize_row_legacy(quant, row, cols, dst);
            else if (quant == 10)
                rnbo_quantize_row_q2_k(row, cols, dst);
            else if (quant == 11)
                rnbo_quantize_row_q3_k(row, cols, dst);
            else if (quant == 12)
                rnbo_quantize_row_q4_k(row, cols, dst);
            else if (quant == 13)
                rnbo_quantize_row_q5_k(row, cols, dst);
            else if (quant == 14)
                rnbo_quantize_row_q6_k(row, cols, dst);
            else
                rnbo_quantize_row_q8_0(row, cols, dst);
        }
        free(row);
    }
    return 0;
}
