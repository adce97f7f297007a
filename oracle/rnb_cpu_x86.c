/*
 * rnb_cpu_x86.c -- AVX2+FMA restatement of rnb-cpu's x86_64 production dot kernels, used as
 * the timed CPU baseline beside the GPU numbers.
 *
 * TEST INFRASTRUCTURE ONLY (see rnb_oracle.h).  Follows the lane structure of
 * crates/rnb-cpu/src/gemm/avx2_dot.rs:622-696 (Q4_K x Q8_K) and :801-885 (Q6_K x Q8_K):
 * eight i32 lanes of per-block integer sums are converted and FMA-accumulated into eight
 * f32 lanes with the per-block scale, the Q4_K mins term goes through four f32 lanes, and
 * horizontal sums happen once per row.  Rows are split over threads in contiguous chunks of
 * ceil(rows / n_threads) for one token, and parallel over rows with an inner token loop for
 * batches (crates/rnb-cpu/src/gemm/quant_gemv.rs:1104-1196).
 *
 * Integer sums are identical to the scalar oracle; only the f32 accumulation order differs.
 */
#include "rnb_oracle.h"

#include <immintrin.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int rnbo_have_avx2(void) {
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma");
}

static inline float hsum8(__m256 v) {
    __m128 r = _mm_add_ps(_mm256_extractf128_ps(v, 1), _mm256_castps256_ps128(v));
    r = _mm_add_ps(r, _mm_movehl_ps(r, r));
    r = _mm_add_ss(r, _mm_movehdup_ps(r));
    return _mm_cvtss_f32(r);
}

static inline uint32_t load_u32(const uint8_t *p) {
    uint32_t v;
    memcpy(&v, p, 4);
    return v;
}

static inline float load_f16(const uint8_t *p) {
    uint16_t h;
    memcpy(&h, p, 2);
    return rnbo_f16_to_f32(h);
}

/* byte-pair broadcast: 16-bit element `k` of a 128-bit vector replicated over 256 bits */
static inline __m256i bcast_i16(__m128i v16, int k) {
    const __m128i idx = _mm_set1_epi16((short)((2 * k) | ((2 * k + 1) << 8)));
    __m128i r = _mm_shuffle_epi8(v16, idx);
    return _mm256_set_m128i(r, r);
}

__attribute__((target("avx2,fma"))) float rnbo_dot_q4k_q8k_avx2(const uint8_t *row,
                                                                 const rnbo_q8k_block *y,
                                                                 size_t nb) {
    const __m256i low4 = _mm256_set1_epi8(0x0f);
    __m256 acc = _mm256_setzero_ps();
    __m128 acc_m = _mm_setzero_ps();
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = row + i * RNBO_Q4_K_BLOCK_BYTES;
        const float d = y[i].d * load_f16(blk);
        const float dmin = -y[i].d * load_f16(blk + 2);

        /* 6-bit unpack on three dwords: u[0..1] = 8 scales, u[2..3] = 8 mins */
        uint32_t u0 = load_u32(blk + 4), u1 = load_u32(blk + 8), u2 = load_u32(blk + 12);
        uint32_t sc_lo = u0 & 0x3f3f3f3fu;
        uint32_t sc_hi = (u2 & 0x0f0f0f0fu) | (((u0 >> 6) & 0x03030303u) << 4);
        uint32_t mn_lo = u1 & 0x3f3f3f3fu;
        uint32_t mn_hi = ((u2 >> 4) & 0x0f0f0f0fu) | (((u1 >> 6) & 0x03030303u) << 4);
        __m256i sm16 = _mm256_cvtepu8_epi16(
            _mm_set_epi32((int)mn_hi, (int)mn_lo, (int)sc_hi, (int)sc_lo));
        __m128i sc16 = _mm256_castsi256_si128(sm16);
        __m128i mn16 = _mm256_extracti128_si256(sm16, 1);

        __m256i bs = _mm256_loadu_si256((const __m256i *)y[i].bsums);
        __m128i bs32 = _mm_hadd_epi16(_mm256_castsi256_si128(bs), _mm256_extracti128_si256(bs, 1));
        __m128i mprod = _mm_madd_epi16(mn16, bs32);
        acc_m = _mm_fmadd_ps(_mm_set1_ps(dmin), _mm_cvtepi32_ps(mprod), acc_m);

        __m256i sumi = _mm256_setzero_si256();
        const uint8_t *q4 = blk + 16;
        const int8_t *q8 = y[i].qs;
        for (int g = 0; g < 4; g++) {
            __m256i bits = _mm256_loadu_si256((const __m256i *)(q4 + 32 * g));
            __m256i lo = _mm256_and_si256(bits, low4);
            __m256i hi = _mm256_and_si256(_mm256_srli_epi16(bits, 4), low4);
            __m256i a_lo = _mm256_loadu_si256((const __m256i *)(q8 + 64 * g));
            __m256i a_hi = _mm256_loadu_si256((const __m256i *)(q8 + 64 * g + 32));
            __m256i p_lo = _mm256_madd_epi16(bcast_i16(sc16, 2 * g), _mm256_maddubs_epi16(lo, a_lo));
            __m256i p_hi =
                _mm256_madd_epi16(bcast_i16(sc16, 2 * g + 1), _mm256_maddubs_epi16(hi, a_hi));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p_lo, p_hi));
        }
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    __m128 m = _mm_add_ps(acc_m, _mm_movehl_ps(acc_m, acc_m));
    m = _mm_add_ss(m, _mm_movehdup_ps(m));
    return hsum8(acc) + _mm_cvtss_f32(m);
}

/* scale k (i8) of the 16 Q6_K sub-block scales, sign-extended and replicated as i16 over the
 * 8 lanes that hold sub-block k's pair sums: lanes 0-7 -> scale 2j, lanes 8-15 -> scale 2j+1 */
static inline __m256i q6_scale_pair(__m128i scales8, int pair) {
    const __m128i idx = _mm_set_epi8((char)(2 * pair + 1), (char)(2 * pair + 1), (char)(2 * pair + 1),
                                     (char)(2 * pair + 1), (char)(2 * pair + 1), (char)(2 * pair + 1),
                                     (char)(2 * pair + 1), (char)(2 * pair + 1), (char)(2 * pair),
                                     (char)(2 * pair), (char)(2 * pair), (char)(2 * pair),
                                     (char)(2 * pair), (char)(2 * pair), (char)(2 * pair),
                                     (char)(2 * pair));
    return _mm256_cvtepi8_epi16(_mm_shuffle_epi8(scales8, idx));
}

__attribute__((target("avx2,fma"))) float rnbo_dot_q6k_q8k_avx2(const uint8_t *row,
                                                                 const rnbo_q8k_block *y,
                                                                 size_t nb) {
    const __m256i m03 = _mm256_set1_epi8(0x03), m0f = _mm256_set1_epi8(0x0f);
    const __m256i m0c = _mm256_set1_epi8(0x0c), m30 = _mm256_set1_epi8(0x30);
    const __m256i mc0 = _mm256_set1_epi8((char)0xc0);
    __m256 acc = _mm256_setzero_ps();
    for (size_t i = 0; i < nb; i++) {
        const uint8_t *blk = row + i * RNBO_Q6_K_BLOCK_BYTES;
        const float d = y[i].d * load_f16(blk + 208);
        __m128i scales8 = _mm_loadu_si128((const __m128i *)(blk + 192));
        __m256i bs = _mm256_loadu_si256((const __m256i *)y[i].bsums);
        /* 32 * sum_sb scale[sb] * bsum[sb], pairwise in 8 i32 lanes */
        __m256i bias = _mm256_slli_epi32(_mm256_madd_epi16(bs, _mm256_cvtepi8_epi16(scales8)), 5);

        __m256i sumi = _mm256_setzero_si256();
        const int8_t *q8 = y[i].qs;
        for (int n = 0; n < 2; n++) {
            __m256i l1 = _mm256_loadu_si256((const __m256i *)(blk + 64 * n));
            __m256i l2 = _mm256_loadu_si256((const __m256i *)(blk + 64 * n + 32));
            __m256i h = _mm256_loadu_si256((const __m256i *)(blk + 128 + 32 * n));
            __m256i h0 = _mm256_slli_epi16(_mm256_and_si256(h, m03), 4);
            __m256i h1 = _mm256_slli_epi16(_mm256_and_si256(h, m0c), 2);
            __m256i h2 = _mm256_and_si256(h, m30);
            __m256i h3 = _mm256_srli_epi16(_mm256_and_si256(h, mc0), 2);
            __m256i u0 = _mm256_or_si256(_mm256_and_si256(l1, m0f), h0);
            __m256i u1 = _mm256_or_si256(_mm256_and_si256(l2, m0f), h1);
            __m256i u2 = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(l1, 4), m0f), h2);
            __m256i u3 = _mm256_or_si256(_mm256_and_si256(_mm256_srli_epi16(l2, 4), m0f), h3);
            __m256i p0 = _mm256_maddubs_epi16(u0, _mm256_loadu_si256((const __m256i *)(q8 + 128 * n)));
            __m256i p1 =
                _mm256_maddubs_epi16(u1, _mm256_loadu_si256((const __m256i *)(q8 + 128 * n + 32)));
            __m256i p2 =
                _mm256_maddubs_epi16(u2, _mm256_loadu_si256((const __m256i *)(q8 + 128 * n + 64)));
            __m256i p3 =
                _mm256_maddubs_epi16(u3, _mm256_loadu_si256((const __m256i *)(q8 + 128 * n + 96)));
            p0 = _mm256_madd_epi16(q6_scale_pair(scales8, 4 * n + 0), p0);
            p1 = _mm256_madd_epi16(q6_scale_pair(scales8, 4 * n + 1), p1);
            p2 = _mm256_madd_epi16(q6_scale_pair(scales8, 4 * n + 2), p2);
            p3 = _mm256_madd_epi16(q6_scale_pair(scales8, 4 * n + 3), p3);
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p0, p1));
            sumi = _mm256_add_epi32(sumi, _mm256_add_epi32(p2, p3));
        }
        sumi = _mm256_sub_epi32(sumi, bias);
        acc = _mm256_fmadd_ps(_mm256_set1_ps(d), _mm256_cvtepi32_ps(sumi), acc);
    }
    return hsum8(acc);
}

static int threads_or_default(int n_threads) {
#ifdef _OPENMP
    if (n_threads <= 0) n_threads = omp_get_max_threads();
#else
    n_threads = 1;
#endif
    return n_threads < 1 ? 1 : n_threads;
}

/* crates/rnb-cpu/src/gemm/quant_gemv.rs:1104-1196 (gemv_quantized_avx2) for Q4_K / Q6_K, and
 * :360-401 (gemv_q8_0, f32 activations) for Q8_0 -- what an x86 host runs by default. */
int rnbo_gemv_avx2(uint32_t quant, const uint8_t *w, size_t rows, size_t cols, const float *x,
                   size_t seq_len, float *out, int n_threads) {
    if (!rnbo_have_avx2()) return 3;
    n_threads = threads_or_default(n_threads);
    if (quant == 8) return rnbo_gemv_q8_0_f32act(w, rows, cols, x, seq_len, out, n_threads);
    if ((quant != 12 && quant != 14) || cols % 256 != 0) return 1;
    size_t nb = cols / 256;
    size_t row_bytes = nb * (quant == 12 ? RNBO_Q4_K_BLOCK_BYTES : RNBO_Q6_K_BLOCK_BYTES);
    rnbo_q8k_block *act = (rnbo_q8k_block *)malloc(sizeof(rnbo_q8k_block) * nb * seq_len);
    if (!act) return 2;
    for (size_t s = 0; s < seq_len; s++) rnbo_quantize_q8k(x + s * cols, cols, act + s * nb);
    if (seq_len == 1) {
        size_t chunk = rows <= 64 ? rows : (rows + (size_t)n_threads - 1) / (size_t)n_threads;
        if (chunk == 0) chunk = 1;
        long n_chunks = (long)((rows + chunk - 1) / chunk);
#pragma omp parallel for schedule(static, 1) num_threads(n_threads)
        for (long c = 0; c < n_chunks; c++) {
            size_t start = (size_t)c * chunk, end = start + chunk < rows ? start + chunk : rows;
            for (size_t r = start; r < end; r++)
                out[r] = quant == 12 ? rnbo_dot_q4k_q8k_avx2(w + r * row_bytes, act, nb)
                                     : rnbo_dot_q6k_q8k_avx2(w + r * row_bytes, act, nb);
        }
    } else {
        float *row_major = (float *)malloc(sizeof(float) * rows * seq_len);
        if (!row_major) {
            free(act);
            return 2;
        }
#pragma omp parallel for schedule(dynamic, 16) num_threads(n_threads)
        for (long r = 0; r < (long)rows; r++)
            for (size_t s = 0; s < seq_len; s++)
                row_major[(size_t)r * seq_len + s] =
                    quant == 12 ? rnbo_dot_q4k_q8k_avx2(w + (size_t)r * row_bytes, act + s * nb, nb)
                                : rnbo_dot_q6k_q8k_avx2(w + (size_t)r * row_bytes, act + s * nb, nb);
        for (size_t r = 0; r < rows; r++)
            for (size_t s = 0; s < seq_len; s++) out[s * rows + r] = row_major[r * seq_len + s];
        free(row_major);
    }
    free(act);
    return 0;
}
