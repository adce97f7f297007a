/*
 * rnb_oracle_iq.c -- CPU restatement of the reference's importance-quant formats (IQ2_XXS, IQ2_S, IQ3_XXS, IQ4_XS):
 * dequantisers and the dot products against Q8_K activations.
 *
 * TEST INFRASTRUCTURE ONLY, like rnb_oracle.c: the checker for the HIP kernels.  Nothing shipped links or loads it.
 *
 *   function                  follows                                            pinned by (tests/test_oracle_pins.py)
 *   ------------------------  -------------------------------------------------  -------------------------------------------
 *   dequantize_iq2_xxs        crates/rnb-cpu/src/quantize/iq.rs:23-44            the reference's known answers: FNV-1a hash of
 *   dequantize_iq2_s          iq.rs:46-72                                        the decoded deterministic block (iq.rs:258-
 *   dequantize_iq3_xxs        iq.rs:74-95                                        334) and zero codes -> all ones (iq.rs:281-
 *   dequantize_iq4_xs         iq.rs:97-116                                       299; IQ4_XS: closed form on a constant block)
 *   dot_iq*_q8k               crates/rnb-cpu/src/gemm/neon_quant.rs:273-411      f64 numpy identity dequant(W) . dequant(Q8_K(x))
 *                                                                                and hand-built one-block vectors
 *
 * The codebooks are ggml's (the reference lists them in crates/rnb-core/src/quant_codebooks.rs).  Here they are kept in a
 * packed form, one 16-bit word per grid entry (iq_grids.inc): every byte of an IQ2 grid entry is one of {8, 25, 43}
 * (two bits per byte, eight bytes), every byte of an IQ3_XXS entry is 4 + 8 c, 62 for c = 7 (three bits per byte, four
 * bytes).  The sign table is i | parity(i) << 7.  The hashes above cover every grid entry the deterministic blocks
 * touch; tests/test_oracle_pins.py also checks the alphabets and that all entries are distinct.
 */
#include "rnb_oracle.h"

#include <string.h>

#include "iq_grids.inc"

static uint64_t g_iq2xxs[256], g_iq2s[1024];
static uint32_t g_iq3xxs[256];
static int g_ready;

static uint64_t expand2(uint16_t w) {
    static const uint8_t alphabet[3] = {8, 25, 43};
    uint64_t v = 0;
    for (int j = 0; j < 8; j++) v |= (uint64_t)alphabet[(w >> (2 * j)) & 3] << (8 * j);
    return v;
}

static uint32_t expand3(uint16_t w) {
    uint32_t v = 0;
    for (int j = 0; j < 4; j++) {
        uint32_t c = (w >> (3 * j)) & 7;
        v |= (c == 7 ? 62u : 4u + 8u * c) << (8 * j);
    }
    return v;
}

static void ready(void) {
    if (g_ready) return;
    for (int i = 0; i < 256; i++) g_iq2xxs[i] = expand2(kIq2xxsPacked[i]);
    for (int i = 0; i < 1024; i++) g_iq2s[i] = expand2(kIq2sPacked[i]);
    for (int i = 0; i < 256; i++) g_iq3xxs[i] = expand3(kIq3xxsPacked[i]);
    g_ready = 1;
}

/* test access to the expanded tables: which = 0 IQ2_XXS (256 x u64), 1 IQ2_S (1024 x u64), 2 IQ3_XXS (256 x u32 widened) */
size_t rnbo_iq_grid(int which, uint64_t *out) {
    ready();
    if (which == 0) { memcpy(out, g_iq2xxs, sizeof g_iq2xxs); return 256; }
    if (which == 1) { memcpy(out, g_iq2s, sizeof g_iq2s); return 1024; }
    for (int i = 0; i < 256; i++) out[i] = g_iq3xxs[i];
    return 256;
}

static inline uint8_t ksigns(uint32_t i) { /* KSIGNS_IQ2XS[i]: seven sign bits and their parity */
    i &= 127;
    return (uint8_t)(i | ((uint32_t)__builtin_parity(i) << 7));
}

static inline uint32_t rd_u32(const uint8_t *p) {
    return (uint32_t)p[0] | (uint32_t)p[1] << 8 | (uint32_t)p[2] << 16 | (uint32_t)p[3] << 24;
}

static inline float rd_half(const uint8_t *p) { return rnbo_f16_to_f32((uint16_t)(p[0] | p[1] << 8)); }

/* the 32 signed codes of group `ib32` of a block, as the dots and the dequantisers both see them */
static void iq2xxs_codes(const uint8_t *blk, int ib32, int8_t *q, uint32_t *scale4) {
    const uint8_t *packed = blk + 2 + 8 * ib32;
    uint32_t ss = rd_u32(packed + 4);
    for (int l = 0; l < 4; l++) {
        uint64_t grid = g_iq2xxs[packed[l]];
        uint8_t s = ksigns(ss >> (7 * l));
        for (int j = 0; j < 8; j++) {
            int v = (int)((grid >> (8 * j)) & 0xff);
            q[8 * l + j] = (int8_t)((s >> j) & 1 ? -v : v);
        }
    }
    *scale4 = ss >> 28;
}

static void iq2s_codes(const uint8_t *blk, int ib32, int8_t *q, uint32_t *scale_lo, uint32_t *scale_hi) {
    const uint8_t *qs = blk + 2, *qh = blk + 66, *scales = blk + 74, *signs = qs + 32;
    for (int l = 0; l < 4; l++) {
        uint32_t high = ((uint32_t)qh[ib32] << (8 - 2 * l)) & 0x300;
        uint64_t grid = g_iq2s[qs[4 * ib32 + l] | high];
        uint8_t s = signs[4 * ib32 + l];
        for (int j = 0; j < 8; j++) {
            int v = (int)((grid >> (8 * j)) & 0xff);
            q[8 * l + j] = (int8_t)((s >> j) & 1 ? -v : v);
        }
    }
    *scale_lo = scales[ib32] & 0x0f;
    *scale_hi = scales[ib32] >> 4;
}

static void iq3xxs_codes(const uint8_t *blk, int ib32, int8_t *q, uint32_t *scale4) {
    const uint8_t *qs = blk + 2;
    uint32_t packed = rd_u32(blk + 66 + 4 * ib32);
    for (int l = 0; l < 4; l++) {
        uint8_t s = ksigns(packed >> (7 * l));
        uint32_t g1 = g_iq3xxs[qs[8 * ib32 + 2 * l]], g2 = g_iq3xxs[qs[8 * ib32 + 2 * l + 1]];
        for (int j = 0; j < 4; j++) {
            int v1 = (int)((g1 >> (8 * j)) & 0xff), v2 = (int)((g2 >> (8 * j)) & 0xff);
            q[8 * l + j] = (int8_t)((s >> j) & 1 ? -v1 : v1);
            q[8 * l + j + 4] = (int8_t)((s >> (j + 4)) & 1 ? -v2 : v2);
        }
    }
    *scale4 = packed >> 28;
}

static const int8_t kvalues_iq4nl[16] = {-127, -104, -83, -65, -49, -35, -22, -10, 1, 13, 25, 38, 53, 69, 89, 113};

static void iq4xs_codes(const uint8_t *blk, int ib, int8_t *q, int *scale) {
    uint32_t scales_h = (uint32_t)blk[2] | (uint32_t)blk[3] << 8;
    const uint8_t *scales_l = blk + 4, *qs = blk + 8 + 16 * ib;
    uint32_t low = (scales_l[ib / 2] >> (4 * (ib % 2))) & 0x0f, high = ((scales_h >> (2 * ib)) & 3) << 4;
    *scale = (int)(low | high) - 32;
    for (int j = 0; j < 16; j++) {
        q[j] = kvalues_iq4nl[qs[j] & 0x0f];
        q[j + 16] = kvalues_iq4nl[qs[j] >> 4];
    }
}

/* ---- dequantisers: crates/rnb-cpu/src/quantize/iq.rs -------------------------------------------- */

void rnbo_dequantize_iq2_xxs(const uint8_t *blocks, size_t n_blocks, float *out) { /* iq.rs:23-44 */
    ready();
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_IQ2_XXS_BLOCK_BYTES;
        float d = rd_half(blk);
        for (int ib = 0; ib < 8; ib++) {
            int8_t q[32];
            uint32_t s4;
            iq2xxs_codes(blk, ib, q, &s4);
            volatile float t = d * (0.5f + (float)s4);
            float db = t * 0.25f;
            /* iq.rs:39 multiplies db * grid * sign in that order; the sign is +-1, so the bits equal db * (signed code) */
            for (int j = 0; j < 32; j++) out[b * 256 + 32 * ib + j] = db * (float)q[j];
        }
    }
}

void rnbo_dequantize_iq2_s(const uint8_t *blocks, size_t n_blocks, float *out) { /* iq.rs:46-72 */
    ready();
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_IQ2_S_BLOCK_BYTES;
        float d = rd_half(blk);
        for (int ib = 0; ib < 8; ib++) {
            int8_t q[32];
            uint32_t lo, hi;
            iq2s_codes(blk, ib, q, &lo, &hi);
            for (int l = 0; l < 4; l++) {
                volatile float t = d * (0.5f + (float)(l < 2 ? lo : hi));
                float db = t * 0.25f;
                for (int j = 0; j < 8; j++) out[b * 256 + 32 * ib + 8 * l + j] = db * (float)q[8 * l + j];
            }
        }
    }
}

void rnbo_dequantize_iq3_xxs(const uint8_t *blocks, size_t n_blocks, float *out) { /* iq.rs:74-95 */
    ready();
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_IQ3_XXS_BLOCK_BYTES;
        float d = rd_half(blk);
        for (int ib = 0; ib < 8; ib++) {
            int8_t q[32];
            uint32_t s4;
            iq3xxs_codes(blk, ib, q, &s4);
            volatile float t = d * (0.5f + (float)s4);
            float db = t * 0.5f;
            for (int j = 0; j < 32; j++) out[b * 256 + 32 * ib + j] = db * (float)q[j];
        }
    }
}

void rnbo_dequantize_iq4_xs(const uint8_t *blocks, size_t n_blocks, float *out) { /* iq.rs:97-116 */
    for (size_t b = 0; b < n_blocks; b++) {
        const uint8_t *blk = blocks + b * RNBO_IQ4_XS_BLOCK_BYTES;
        float d = rd_half(blk);
        for (int ib = 0; ib < 8; ib++) {
            int8_t q[32];
            int scale;
            iq4xs_codes(blk, ib, q, &scale);
            float dl = d * ((float)(scale + 32) - 32.0f);
            for (int j = 0; j < 32; j++) out[b * 256 + 32 * ib + j] = dl * (float)q[j];
        }
    }
}

/* ---- dots against Q8_K: crates/rnb-cpu/src/gemm/neon_quant.rs:273-411 --------------------------------- */

static inline int32_t dot_i8(const int8_t *a, const int8_t *b, int n) {
    int32_t s = 0;
    for (int i = 0; i < n; i++) s += (int32_t)a[i] * (int32_t)b[i];
    return s;
}

/* neon_quant.rs:273-298: block_sum is f32, (0.5 + scale) * dot per group of 32 */
float rnbo_dot_iq2_xxs_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    ready();
    float sum = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_IQ2_XXS_BLOCK_BYTES;
        float block_sum = 0.0f;
        for (int g = 0; g < 8; g++) {
            int8_t q[32];
            uint32_t s4;
            iq2xxs_codes(blk, g, q, &s4);
            volatile float t = (0.5f + (float)s4) * (float)dot_i8(q, act[b].qs + 32 * g, 32);
            block_sum += t;
        }
        volatile float t0 = rd_half(blk) * act[b].d;
        volatile float t1 = t0 * 0.25f;
        volatile float t2 = t1 * block_sum;
        sum += t2;
    }
    return sum;
}

/* neon_quant.rs:300-330: integer block sum, (1 + 2 scale) per half group, 0.125 */
float rnbo_dot_iq2_s_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    ready();
    float sum = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_IQ2_S_BLOCK_BYTES;
        int32_t block_sum = 0;
        for (int g = 0; g < 8; g++) {
            int8_t q[32];
            uint32_t lo, hi;
            iq2s_codes(blk, g, q, &lo, &hi);
            block_sum += dot_i8(q, act[b].qs + 32 * g, 16) * (int32_t)(1 + 2 * lo);
            block_sum += dot_i8(q + 16, act[b].qs + 32 * g + 16, 16) * (int32_t)(1 + 2 * hi);
        }
        volatile float t0 = rd_half(blk) * act[b].d;
        volatile float t1 = t0 * 0.125f;
        volatile float t2 = t1 * (float)block_sum;
        sum += t2;
    }
    return sum;
}

/* neon_quant.rs:337-374 */
float rnbo_dot_iq3_xxs_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    ready();
    float sum = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_IQ3_XXS_BLOCK_BYTES;
        float block_sum = 0.0f;
        for (int g = 0; g < 8; g++) {
            int8_t q[32];
            uint32_t s4;
            iq3xxs_codes(blk, g, q, &s4);
            volatile float t = (0.5f + (float)s4) * (float)dot_i8(q, act[b].qs + 32 * g, 32);
            block_sum += t;
        }
        volatile float t0 = rd_half(blk) * act[b].d;
        volatile float t1 = t0 * 0.5f;
        volatile float t2 = t1 * block_sum;
        sum += t2;
    }
    return sum;
}

/* neon_quant.rs:376-411 */
float rnbo_dot_iq4_xs_q8k(const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    float sum = 0.0f;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *blk = row + b * RNBO_IQ4_XS_BLOCK_BYTES;
        int32_t block_sum = 0;
        for (int ib = 0; ib < 8; ib++) {
            int8_t q[32];
            int scale;
            iq4xs_codes(blk, ib, q, &scale);
            block_sum += dot_i8(q, act[b].qs + 32 * ib, 32) * scale;
        }
        volatile float t0 = rd_half(blk) * act[b].d;
        volatile float t1 = t0 * (float)block_sum;
        sum += t1;
    }
    return sum;
}

/* f64 gold forms: the same integers, every float step in double */
double rnbo_dot_iq_q8k_f64(uint32_t quant, const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    ready();
    double sum = 0.0;
    for (size_t b = 0; b < nb; b++) {
        double bs = 0.0;
        const uint8_t *blk;
        int8_t q[32];
        uint32_t s4, lo, hi;
        int sc;
        switch (quant) {
        case 16:
            blk = row + b * RNBO_IQ2_XXS_BLOCK_BYTES;
            for (int g = 0; g < 8; g++) {
                iq2xxs_codes(blk, g, q, &s4);
                bs += (0.5 + (double)s4) * (double)dot_i8(q, act[b].qs + 32 * g, 32);
            }
            sum += (double)rd_half(blk) * (double)act[b].d * 0.25 * bs;
            break;
        case 22:
            blk = row + b * RNBO_IQ2_S_BLOCK_BYTES;
            for (int g = 0; g < 8; g++) {
                iq2s_codes(blk, g, q, &lo, &hi);
                bs += (double)dot_i8(q, act[b].qs + 32 * g, 16) * (1.0 + 2.0 * lo);
                bs += (double)dot_i8(q + 16, act[b].qs + 32 * g + 16, 16) * (1.0 + 2.0 * hi);
            }
            sum += (double)rd_half(blk) * (double)act[b].d * 0.125 * bs;
            break;
        case 18:
            blk = row + b * RNBO_IQ3_XXS_BLOCK_BYTES;
            for (int g = 0; g < 8; g++) {
                iq3xxs_codes(blk, g, q, &s4);
                bs += (0.5 + (double)s4) * (double)dot_i8(q, act[b].qs + 32 * g, 32);
            }
            sum += (double)rd_half(blk) * (double)act[b].d * 0.5 * bs;
            break;
        default:
            blk = row + b * RNBO_IQ4_XS_BLOCK_BYTES;
            for (int g = 0; g < 8; g++) {
                iq4xs_codes(blk, g, q, &sc);
                bs += (double)dot_i8(q, act[b].qs + 32 * g, 32) * (double)sc;
            }
            sum += (double)rd_half(blk) * (double)act[b].d * bs;
            break;
        }
    }
    return sum;
}

float rnbo_dot_iq_q8k(uint32_t quant, const uint8_t *row, const rnbo_q8k_block *act, size_t nb) {
    switch (quant) {
    case 16: return rnbo_dot_iq2_xxs_q8k(row, act, nb);
    case 22: return rnbo_dot_iq2_s_q8k(row, act, nb);
    case 18: return rnbo_dot_iq3_xxs_q8k(row, act, nb);
    default: return rnbo_dot_iq4_xs_q8k(row, act, nb);
    }
}

/* Input generation only: a block of any bytes is a valid IQ block (every index is in its table); the scale d is set to
 * a small finite half so that the values have the magnitude of quantised N(0, sigma) weights. */
void rnbo_make_iq_row(uint32_t quant, size_t n_blocks, uint64_t seed, float sigma, uint8_t *out) {
    size_t bb = quant == 16 ? RNBO_IQ2_XXS_BLOCK_BYTES : quant == 22 ? RNBO_IQ2_S_BLOCK_BYTES
              : quant == 18 ? RNBO_IQ3_XXS_BLOCK_BYTES : RNBO_IQ4_XS_BLOCK_BYTES;
    /* typical code magnitude x typical sub-scale, so that d * that ~ sigma */
    float unit = quant == 16 ? 25.0f * 8.0f * 0.25f : quant == 22 ? 25.0f * 8.0f * 0.25f
               : quant == 18 ? 30.0f * 8.0f * 0.5f : 50.0f * 16.0f;
    uint64_t z = seed * 0x9e3779b97f4a7c15ull + 0x1234567ull;
    for (size_t b = 0; b < n_blocks; b++) {
        uint8_t *blk = out + b * bb;
        for (size_t i = 0; i < bb; i++) {
            z += 0x9e3779b97f4a7c15ull;
            uint64_t x = z;
            x = (x ^ (x >> 30)) * 0xbf58476d1ce4e5b9ull;
            x = (x ^ (x >> 27)) * 0x94d049bb133111ebull;
            x ^= x >> 31;
            blk[i] = (uint8_t)(x >> 24);
        }
        float d = sigma / unit * (0.5f + (float)(blk[0] & 63) / 64.0f);
        if (blk[1] & 1) d = -d; /* negative block scales are legal */
        uint16_t h = rnbo_f32_to_f16(d);
        blk[0] = (uint8_t)(h & 0xff);
        blk[1] = (uint8_t)(h >> 8);
    }
}
