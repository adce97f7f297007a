// Prefill GEMM for the formats whose scales do not fold onto an int8 operand: Q6_K (int8 scale per 16 elements), Q5_K
// (6-bit scale per 32 five-bit codes: scale times code needs 11 bits), Q2_K / Q3_K (sixteen sub-blocks like Q6_K) and
// the 32-element formats Q8_0 / Q8_1 / Q4_0 / Q4_1 / Q5_0 / Q5_1 (f16 scale per 32 elements).  out[seq][rows], same
// contract as the GEMVs.  Small grids are cut along K into slices whose outputs a second kernel adds in slice order.
//
// The matrix cores do the integer part of one scale group per instruction and the vector units apply the group's scale
// to the 16 results a lane holds:
//   Q6_K   v_mfma_i32_32x32x16_i8 per 16-element sub-block: I_sb = sum (q - 32) * a  (exact), tot += sc[r][sb] * I_sb
//          in 24-bit integer multiplies, and once per super-block out += (d[r] * d_x[s]) * float(tot): the arithmetic of
//          crates/rnb-cpu/src/gemm/neon_dot.rs:2240-2288 (dot_q6_k_q8k_scalar).
//   Q5_K   v_mfma_i32_32x32x32_i8 per 32-element sub-block, tot += sc * I_sb, the mins through two K=16 instructions on
//          the quantiser's digits, out += d_x * (d * float(tot) - dmin * float(S)) per super-block.
//   Q8_0   v_mfma_i32_32x32x32_i8 per 32-element block: out += (d[r][b] * d_x[s][b]) * float(I_b),
//   Q8_1   crates/rnb-cpu/src/gemm/neon_dot.rs:376-436, neon_quant.rs:236-253.
//   Q4_0 Q4_1 Q5_0 Q5_1   the same with the block's nibbles (and fifth bits) made into signed bytes when consumed; the
//          d n + m formats add (m * d_x) * sum(a) from a second instruction against a row of ones.
//   Q2_K Q3_K   Q6_K's scheme; Q2_K's mins term through two K=16 instructions over the sub-block sums' digits:
//          crates/rnb-cpu/src/gemm/avx2_dot.rs:169-242 (Q2_K), :247-375 (Q3_K).
// That is 16 (Q6_K) or 48 (Q8) vector instructions per matrix instruction, so these kernels are bound by the vector
// port, not the matrix pipe; at 512 tokens they measured 9 to 17 times faster than GEMV passes over the tokens on the
// vector units' integer dots.
//
// Tiling: workgroup = 4 waves = 128 weight rows x kTT*32 tokens; a wave owns 32 rows and all the workgroup's tokens.
// MFMA "M" = token, "N" = weight row: a lane's 16 results belong to ONE row (lane % 32), so that row's scales are
// per-lane scalars; both operands take their K bytes per lane from the same K positions (8 or 16 times lane / 32 + j),
// so the contraction does not depend on how the hardware orders K inside the instruction.  Weights go from global
// memory straight to the registers of the lane that owns the row (one scale group ahead of use is the next
// super-block / block pair, requested before the current one is multiplied); the quantised activations of the
// workgroup's tokens are staged in LDS, double-buffered, one barrier per step.
#include "device_utils.h"
#include "kernels.h"
#include <algorithm>

#include "mfma_blocks.h"

namespace rnb {

namespace {

template <int kTT, int kLive>
__global__ void __launch_bounds__(kGbThreads, 2)
    gemm_q6k_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                         float *__restrict__ out, uint32_t rows, uint32_t nb, uint32_t seq, uint32_t nb_slice) {
    constexpr int kToks = 32 * kTT;
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][kToks * kGbStride64];
    __shared__ __attribute__((aligned(16))) uint8_t s_w[kGbWaves][32 * kQ6StripStride];
    __shared__ __attribute__((aligned(16))) float s_dx[2][kToks];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t row = blockIdx.x * kGbRows + wave * 32 + lrow;
    const uint32_t tok0 = blockIdx.y * kToks, last_tok = seq - 1;
    const uint8_t *wrow = w + static_cast<size_t>(min(row, rows - 1)) * nb * kQ6KBytes;

    float accf[kTT][16];
    int tot[kTT][16];
#pragma unroll
    for (int t = 0; t < kTT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            accf[t][i] = 0.0f;
            tot[t][i] = 0;
        }
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    // the wave's 32 rows come in by whole cache lines and reach their lanes through the wave's strip of LDS
    const uint32_t wrow0 = min(blockIdx.x * kGbRows + wave * 32, rows - 1);
    const uint8_t *wbase = w + static_cast<size_t>(wrow0) * nb * kQ6KBytes;
    uint8_t *strip = s_w[wave];
    RowRoute<kQ6Pieces> rt;
    route_setup<kQ6Pieces, kQ6StripStride>(rt, rows - wrow0, static_cast<size_t>(nb) * kQ6KBytes, lane);

    // K slice of this workgroup (blockIdx.z): blocks b0 .. b1, its sums go to the slice's own copy of the output
    const uint32_t b0 = blockIdx.z * nb_slice, b1 = min(nb, b0 + nb_slice);
    out += static_cast<size_t>(blockIdx.z) * seq * rows;

    Stage<kToks> st;
    stage_load<kToks>(st, aq, ad, tok0, last_tok, nb, b0, tid);
    route_load(rt, wbase + static_cast<size_t>(b0) * kQ6KBytes);
    Q6Row cur;
    cur.d = ld_f16(wrow + static_cast<size_t>(b0) * kQ6KBytes + 208);
    route_store(rt, strip, lane);
    q6_row_from_strip(cur, strip + lrow * kQ6StripStride, khalf);
    stage_store<kToks>(st, s_a[0], s_dx[0], tid);
    __syncthreads();

    for (uint32_t b = b0; b < b1; b++) {
        const int buf = (b - b0) & 1;
        const uint32_t bn = b + 1 < b1 ? b + 1 : b;  // the last step reloads its own block, unused
        stage_load<kToks>(st, aq, ad, tok0, last_tok, nb, bn, tid);
        route_load(rt, wbase + static_cast<size_t>(bn) * kQ6KBytes);
        const float d_next = ld_f16(wrow + static_cast<size_t>(bn) * kQ6KBytes + 208);
        const float d_cur = cur.d;
        const uint8_t *abase = s_a[buf] + lrow * kGbStride64 + 8 * khalf;

        // One 16-element sub-block: operand from the packed row, one matrix instruction per token tile, the sub-block's
        // scale applied to the 16 results.  The token tiles' instructions are issued together and their results
        // scaled afterwards, so the second tile's instruction runs while the first tile's results are scaled.  The
        // empty asm and the scheduling barrier keep the sub-blocks in order: left alone the compiler turns each
        // result's sixteen additions into a tree and keeps all 256 products alive.
        long aop_cur[kTT], aop_nxt[kTT];  // the tokens' operands are read from LDS one sub-block ahead of their use
#pragma unroll
        for (int t = 0; t < kTT; t++) aop_cur[t] = *reinterpret_cast<const long *>(abase + 32 * t * kGbStride64);
#define RNB_Q6_SCALE(ACC, SC)                                                                                          \
    {                                                                                                                  \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                              \
            _Pragma("unroll") for (int i = 0; i < kLive; i++) {                                                        \
                tot[t][i] += mul24(ACC[t][i], SC); /* |I_sb| <= 16 * 32 * 127 */                                       \
                asm volatile("" : "+v"(tot[t][i])); /* no re-association of the sixteen sums into a tree */            \
            }                                                                                                          \
        }                                                                                                              \
    }
#define RNB_Q6_SUB_BLOCK(SB)                                                                                           \
    {                                                                                                                  \
        const long bop = q6_operand<SB>(cur);                                                                          \
        const int sc = q6_scale<SB>(cur);                                                                              \
        _Pragma("unroll") for (int t = 0; t < kTT; t++)                                                                \
            aop_nxt[t] = *reinterpret_cast<const long *>(abase + 32 * t * kGbStride64 + 16 * ((SB) < 15 ? (SB) + 1 : 15)); \
        if constexpr (kTT == 1) {                                                                                      \
            /* one token tile: the instruction of this sub-block is issued before the previous sub-block's results */  \
            /* are scaled (two result sets in turn, all sixteen registers of a set the instruction's until then) */    \
            if constexpr (((SB) & 1) == 0) {                                                                           \
                acc_a[0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop_cur[0], bop, zero16, 0, 0, 0);                    \
                sc_a = sc;                                                                                             \
                asm volatile("" : "+v"(acc_a[0])); /* pins the instruction in front of the fence */                   \
                __builtin_amdgcn_sched_barrier(0);                                                                     \
                if constexpr ((SB) > 0) {                                                                              \
                    RNB_Q6_SCALE(acc_b, sc_b)                                                                          \
                    asm volatile("" ::"v"(acc_b[0]));                                                                  \
                }                                                                                                      \
            } else {                                                                                                   \
                acc_b[0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop_cur[0], bop, zero16, 0, 0, 0);                    \
                sc_b = sc;                                                                                             \
                asm volatile("" : "+v"(acc_b[0]));                                                                     \
                __builtin_amdgcn_sched_barrier(0);                                                                     \
                RNB_Q6_SCALE(acc_a, sc_a)                                                                              \
                asm volatile("" ::"v"(acc_a[0]));                                                                      \
            }                                                                                                          \
            if constexpr ((SB) == 15) {                                                                                \
                __builtin_amdgcn_sched_barrier(0);                                                                     \
                RNB_Q6_SCALE(acc_b, sc_b)                                                                              \
            }                                                                                                          \
        } else {                                                                                                       \
            v16i acc[kTT];                                                                                             \
            _Pragma("unroll") for (int t = 0; t < kTT; t++)                                                            \
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop_cur[t], bop, zero16, 0, 0, 0);                      \
            RNB_Q6_SCALE(acc, sc)                                                                                      \
        }                                                                                                              \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) aop_cur[t] = aop_nxt[t];                                       \
        __builtin_amdgcn_sched_barrier(0);                                                                             \
    }
        [[maybe_unused]] v16i acc_a[1], acc_b[1];  // the one-tile form's two result sets
        [[maybe_unused]] int sc_a = 0, sc_b = 0;
        RNB_Q6_SUB_BLOCK(0)
        RNB_Q6_SUB_BLOCK(1)
        RNB_Q6_SUB_BLOCK(2)
        RNB_Q6_SUB_BLOCK(3)
        RNB_Q6_SUB_BLOCK(4)
        RNB_Q6_SUB_BLOCK(5)
        RNB_Q6_SUB_BLOCK(6)
        RNB_Q6_SUB_BLOCK(7)
        RNB_Q6_SUB_BLOCK(8)
        RNB_Q6_SUB_BLOCK(9)
        RNB_Q6_SUB_BLOCK(10)
        RNB_Q6_SUB_BLOCK(11)
        RNB_Q6_SUB_BLOCK(12)
        RNB_Q6_SUB_BLOCK(13)
        RNB_Q6_SUB_BLOCK(14)
        RNB_Q6_SUB_BLOCK(15)
#undef RNB_Q6_SCALE
#undef RNB_Q6_SUB_BLOCK

        // out += (d * d_x) * float(sum): result i of a tile is token 8 * (i / 4) + 4 * khalf + i % 4
#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int j = 0; j < kLive / 4; j++) {
                const float4 dx4 = reinterpret_cast<const float4 *>(s_dx[buf])[8 * t + 2 * j + khalf];
                const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = 4 * j + i;
                    accf[t][r] += (d_cur * dx[i]) * static_cast<float>(tot[t][r]);
                    tot[t][r] = 0;
                }
            }
        stage_store<kToks>(st, s_a[buf ^ 1], s_dx[buf ^ 1], tid);
        route_store(rt, strip, lane);
        q6_row_from_strip(cur, strip + lrow * kQ6StripStride, khalf);
        cur.d = d_next;
        __syncthreads();
    }

    if (row < rows) {
#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int r = 0; r < kLive; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row] = accf[t][r];
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Q2_K {u8 scales[16] (scale | min << 4), u8 qs[64], f16 d, f16 dmin} (84 bytes) and Q3_K {u8 hmask[32], u8 qs[64],
// u8 scales[12], f16 d} (110 bytes): sixteen 16-element sub-blocks like Q6_K, so the same scheme: one K=16 matrix
// instruction per sub-block and the sub-block's scale on its 16 results.  Byte 32n + l of qs holds elements
// 128n + 32j + l in bit pair j; sub-block 8n + 2j + l/16 is elements 16 sb .. + 16, of which the lane of K-half k takes
// l%16 = 8k .. + 8.  Q3_K: code | hbit << 2 (bit 4n + j of hmask[l]) minus 4 in packed bytes, scale = 6-bit code - 32.
// Q2_K: unsigned codes, 4-bit scales; its mins term sum_sb mn_sb * bsum16_sb is itself a K=16 contraction over the
// sub-blocks: the activations' 16-element sums are staged as two int8 digits (bsum = lo + 64 hi, lo = bsum & 63) and
// two more matrix instructions per block and token tile deliver it in the result layout.
// ---------------------------------------------------------------------------------------------
struct Q23Row {
    uint2 qs[2][2];  // [n][l / 16]: the lane's 8 bytes
    uint2 hm[2];     // [l / 16] (Q3_K)
    uint4 sc;        // Q2_K: scales[16]; Q3_K: scales[12] in x, y, z
    float d, dmin;
};

template <bool kThree>
__device__ __forceinline__ Q23Row q23_load_row(const uint8_t *__restrict__ blk, int khalf) {
    Q23Row r;
    constexpr int kQsOff = kThree ? 32 : 16;
#pragma unroll
    for (int n = 0; n < 2; n++)
#pragma unroll
        for (int h = 0; h < 2; h++) r.qs[n][h] = ld_u2_a2(blk + kQsOff + 32 * n + 16 * h + 8 * khalf);
    if constexpr (kThree) {
#pragma unroll
        for (int h = 0; h < 2; h++) r.hm[h] = ld_u2_a2(blk + 16 * h + 8 * khalf);
        const uint2 s01 = ld_u2_a2(blk + 96);
        r.sc = make_uint4(s01.x, s01.y, ld_u32_a2(blk + 104), 0);
        r.d = ld_f16(blk + 108);
        r.dmin = 0.0f;
    } else {
        r.hm[0] = r.hm[1] = make_uint2(0, 0);
        r.sc = ld_u4_a2(blk);
        const uint32_t dd = ld_u32_a2(blk + 80);
        r.d = f16_bits_to_f32(dd);
        r.dmin = f16_bits_to_f32(dd >> 16);
    }
    return r;
}

template <int kSb, bool kThree>
__device__ __forceinline__ long q23_operand(const Q23Row &r) {
    constexpr int g = kSb >> 1, n = g >> 2, j = g & 3, h = kSb & 1;
    uint32_t v0 = (r.qs[n][h].x >> (2 * j)) & 0x03030303u, v1 = (r.qs[n][h].y >> (2 * j)) & 0x03030303u;
    if constexpr (kThree) {
        v0 |= ((r.hm[h].x >> g) & 0x01010101u) << 2;
        v1 |= ((r.hm[h].y >> g) & 0x01010101u) << 2;
        v0 = (v0 + 0x7c7c7c7cu) ^ 0x80808080u;  // v - 4 per byte: v + 0x7c never carries, flipping bit 7 finishes it
        v1 = (v1 + 0x7c7c7c7cu) ^ 0x80808080u;
    }
    return static_cast<long>(static_cast<unsigned long>(v0) | (static_cast<unsigned long>(v1) << 32));
}

template <int kSb, bool kThree>
__device__ __forceinline__ int q23_scale(const Q23Row &r) {
    const uint32_t w[4] = {r.sc.x, r.sc.y, r.sc.z, r.sc.w};
    if constexpr (kThree) {
        // code k: low nibble = nibble k / 8 of byte k % 8, high two bits = bit pair k / 4 of byte 8 + k % 4
        const uint32_t lo = (w[(kSb & 7) >> 2] >> (8 * (kSb & 3) + 4 * (kSb >> 3))) & 15u;
        const uint32_t hi = (w[2] >> (8 * (kSb & 3) + 2 * (kSb >> 2))) & 3u;
        return static_cast<int>(lo | (hi << 4)) - 32;
    } else {
        return static_cast<int>((w[kSb >> 2] >> (8 * (kSb & 3))) & 15u);
    }
}

template <int kTT, bool kThree, int kLive>
__global__ void __launch_bounds__(kGbThreads, 2)
    gemm_q23k_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                          const int16_t *__restrict__ abs16, float *__restrict__ out, uint32_t rows, uint32_t nb,
                          uint32_t seq, uint32_t nb_slice) {
    constexpr int kToks = 32 * kTT;
    constexpr int kBlockBytes = kThree ? kQ3KBytes : kQ2KBytes;
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][kToks * kGbStride64];
    __shared__ __attribute__((aligned(16))) float s_dx[2][kToks];
    __shared__ __attribute__((aligned(16))) uint4 s_bd[2][kToks][2];  // Q2_K: digits lo, hi of the 16 sub-block sums
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t row = blockIdx.x * kGbRows + wave * 32 + lrow;
    const uint32_t tok0 = blockIdx.y * kToks, last_tok = seq - 1;
    const uint8_t *wrow = w + static_cast<size_t>(min(row, rows - 1)) * nb * kBlockBytes;

    float accf[kTT][16];
    int tot[kTT][16];
#pragma unroll
    for (int t = 0; t < kTT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            accf[t][i] = 0.0f;
            tot[t][i] = 0;
        }
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    Stage<kToks> st;
    uint4 bd_lo = make_uint4(0, 0, 0, 0), bd_hi = make_uint4(0, 0, 0, 0);
    auto stage_load2 = [&](uint32_t b) {
        stage_load<kToks>(st, aq, ad, tok0, last_tok, nb, b, tid);
        if constexpr (!kThree) {
            if (tid < kToks) {
                const int16_t *bs = abs16 + (static_cast<size_t>(min(tok0 + tid, last_tok)) * nb + b) * 16;
                const uint4 s0 = *reinterpret_cast<const uint4 *>(bs), s1 = *reinterpret_cast<const uint4 *>(bs + 8);
                const uint32_t pr[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};  // two sums per dword
                uint32_t lo[4] = {0, 0, 0, 0}, hi[4] = {0, 0, 0, 0};
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const int v = static_cast<int16_t>(pr[i >> 1] >> (16 * (i & 1)));
                    lo[i >> 2] |= static_cast<uint32_t>(v & 63) << (8 * (i & 3));
                    hi[i >> 2] |= (static_cast<uint32_t>(v >> 6) & 0xffu) << (8 * (i & 3));  // |sum| <= 2048: -32 .. 31
                }
                bd_lo = make_uint4(lo[0], lo[1], lo[2], lo[3]);
                bd_hi = make_uint4(hi[0], hi[1], hi[2], hi[3]);
            }
        }
    };
    auto stage_store2 = [&](int buf) {
        stage_store<kToks>(st, s_a[buf], s_dx[buf], tid);
        if constexpr (!kThree) {
            if (tid < kToks) {
                s_bd[buf][tid][0] = bd_lo;
                s_bd[buf][tid][1] = bd_hi;
            }
        }
    };

    // K slice of this workgroup (blockIdx.z): blocks b0 .. b1, its sums go to the slice's own copy of the output
    const uint32_t b0 = blockIdx.z * nb_slice, b1 = min(nb, b0 + nb_slice);
    out += static_cast<size_t>(blockIdx.z) * seq * rows;
    stage_load2(b0);
    Q23Row cur = q23_load_row<kThree>(wrow + static_cast<size_t>(b0) * kBlockBytes, khalf);
    stage_store2(0);
    __syncthreads();

    for (uint32_t b = b0; b < b1; b++) {
        const int buf = (b - b0) & 1;
        const uint32_t bn = b + 1 < b1 ? b + 1 : b;  // the last step reloads its own block, unused
        stage_load2(bn);
        const Q23Row nxt = q23_load_row<kThree>(wrow + static_cast<size_t>(bn) * kBlockBytes, khalf);
        const uint8_t *abase = s_a[buf] + lrow * kGbStride64 + 8 * khalf;

        // as in the Q6_K kernel: the empty asm and the scheduling barrier keep the sixteen sub-blocks a chain
#define RNB_Q23_SCALE(ACC, SC)                                                                                         \
    {                                                                                                                  \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                              \
            _Pragma("unroll") for (int i = 0; i < kLive; i++) {                                                        \
                tot[t][i] += mul24(ACC[t][i], SC); /* |I_sb| <= 16 * 4 * 127 */                                        \
                asm volatile("" : "+v"(tot[t][i]));                                                                    \
            }                                                                                                          \
        }                                                                                                              \
    }
#define RNB_Q23_SUB_BLOCK(SB)                                                                                          \
    {                                                                                                                  \
        const long bop = q23_operand<SB, kThree>(cur);                                                                 \
        const int sc = q23_scale<SB, kThree>(cur);                                                                     \
        if constexpr (kTT == 1) {                                                                                      \
            /* one token tile: this sub-block's instruction before the previous sub-block's scaling, see the Q6_K */   \
            /* kernel */                                                                                               \
            const long aop = *reinterpret_cast<const long *>(abase + 16 * SB);                                         \
            if constexpr (((SB) & 1) == 0) {                                                                           \
                acc_a[0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop, bop, zero16, 0, 0, 0);                           \
                sc_a = sc;                                                                                             \
                asm volatile("" : "+v"(acc_a[0]));                                                                     \
                __builtin_amdgcn_sched_barrier(0);                                                                     \
                if constexpr ((SB) > 0) {                                                                              \
                    RNB_Q23_SCALE(acc_b, sc_b)                                                                         \
                    asm volatile("" ::"v"(acc_b[0]));                                                                  \
                }                                                                                                      \
            } else {                                                                                                   \
                acc_b[0] = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop, bop, zero16, 0, 0, 0);                           \
                sc_b = sc;                                                                                             \
                asm volatile("" : "+v"(acc_b[0]));                                                                     \
                __builtin_amdgcn_sched_barrier(0);                                                                     \
                RNB_Q23_SCALE(acc_a, sc_a)                                                                             \
                asm volatile("" ::"v"(acc_a[0]));                                                                      \
            }                                                                                                          \
            if constexpr ((SB) == 15) {                                                                                \
                __builtin_amdgcn_sched_barrier(0);                                                                     \
                RNB_Q23_SCALE(acc_b, sc_b)                                                                             \
            }                                                                                                          \
        } else {                                                                                                       \
            v16i acc[kTT]; /* the tiles' instructions first, then their results: see the Q6_K kernel */                \
            _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                          \
                const long aop = *reinterpret_cast<const long *>(abase + 32 * t * kGbStride64 + 16 * SB);              \
                acc[t] = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop, bop, zero16, 0, 0, 0);                             \
            }                                                                                                          \
            RNB_Q23_SCALE(acc, sc)                                                                                     \
        }                                                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                                             \
    }
        [[maybe_unused]] v16i acc_a[1], acc_b[1];  // the one-tile form's two result sets
        [[maybe_unused]] int sc_a = 0, sc_b = 0;
        RNB_Q23_SUB_BLOCK(0)
        RNB_Q23_SUB_BLOCK(1)
        RNB_Q23_SUB_BLOCK(2)
        RNB_Q23_SUB_BLOCK(3)
        RNB_Q23_SUB_BLOCK(4)
        RNB_Q23_SUB_BLOCK(5)
        RNB_Q23_SUB_BLOCK(6)
        RNB_Q23_SUB_BLOCK(7)
        RNB_Q23_SUB_BLOCK(8)
        RNB_Q23_SUB_BLOCK(9)
        RNB_Q23_SUB_BLOCK(10)
        RNB_Q23_SUB_BLOCK(11)
        RNB_Q23_SUB_BLOCK(12)
        RNB_Q23_SUB_BLOCK(13)
        RNB_Q23_SUB_BLOCK(14)
        RNB_Q23_SUB_BLOCK(15)
#undef RNB_Q23_SUB_BLOCK
#undef RNB_Q23_SCALE

        // Q2_K mins: K slot i of the lane's K-half is sub-block 8 khalf + i on both sides
        const uint32_t mn0 = ((khalf ? cur.sc.z : cur.sc.x) >> 4) & 0x0f0f0f0fu, mn1 = ((khalf ? cur.sc.w : cur.sc.y) >> 4) & 0x0f0f0f0fu;
        const long mnop = static_cast<long>(static_cast<unsigned long>(mn0) | (static_cast<unsigned long>(mn1) << 32));
#pragma unroll
        for (int t = 0; t < kTT; t++) {
            v16i mins = zero16;
            if constexpr (!kThree) {
                const uint8_t *dg = reinterpret_cast<const uint8_t *>(&s_bd[buf][32 * t + lrow][0]) + 8 * khalf;
                const long lo = *reinterpret_cast<const long *>(dg), hi = *reinterpret_cast<const long *>(dg + 16);
                const v16i c0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(lo, mnop, zero16, 0, 0, 0);
                const v16i c1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(hi, mnop, zero16, 0, 0, 0);
#pragma unroll
                for (int i = 0; i < kLive; i++) mins[i] = c0[i] + 64 * c1[i];
            }
#pragma unroll
            for (int j = 0; j < kLive / 4; j++) {
                const float4 dx4 = reinterpret_cast<const float4 *>(s_dx[buf])[8 * t + 2 * j + khalf];
                const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = 4 * j + i;
                    accf[t][r] += (cur.d * dx[i]) * static_cast<float>(tot[t][r]);
                    if constexpr (!kThree) accf[t][r] -= (cur.dmin * dx[i]) * static_cast<float>(mins[r]);
                    tot[t][r] = 0;
                }
            }
        }
        stage_store2(buf ^ 1);
        cur = nxt;
        __syncthreads();
    }

    if (row < rows) {
#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int r = 0; r < kLive; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row] = accf[t][r];
            }
    }
}

// ---------------------------------------------------------------------------------------------
// Q5_K: block = {f16 d, f16 dmin, scales[12] (eight 6-bit scales and mins), qh[32], qs[128]}, 176 bytes.  Element
// 64g + 32h + l = nibble h of qs[32g + l] | bit (2g + h) of qh[l] << 4 (0..31), sub-block 2g + h.  One K=32 matrix
// instruction per sub-block, tot += sc * I_sb; the mins term S = sum mn * bsum32 rides on the matrix cores through the
// quantiser's digits (bsum32 = b0 + 64 * b1): two K=16 instructions with eight live K slots per token tile.
// Per super-block out += d_x * (d * float(tot) - dmin * float(S)): crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800.
// ---------------------------------------------------------------------------------------------
template <int kTT, bool kFifth, int kLive>
__global__ void __launch_bounds__(kGbThreads, 2)
    gemm_q45k_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                         const uint8_t *__restrict__ adig, float *__restrict__ out, uint32_t rows, uint32_t nb,
                         uint32_t seq, uint32_t nb_slice) {
    constexpr int kToks = 32 * kTT;
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][kToks * kGbStride128];
    __shared__ __attribute__((aligned(16))) float s_dx[2][kToks];
    __shared__ __attribute__((aligned(16))) uint4 s_dig[2][kToks];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t row = blockIdx.x * kGbRows + wave * 32 + lrow;
    const uint32_t tok0 = blockIdx.y * kToks, last_tok = seq - 1;
    constexpr size_t kBlockBytes = kFifth ? kQ5KBytes : kQ4KBytes;
    const uint8_t *wrow = w + static_cast<size_t>(min(row, rows - 1)) * nb * kBlockBytes;

    float accf[kTT][16];
    int tot[kTT][16];
#pragma unroll
    for (int t = 0; t < kTT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) {
            accf[t][i] = 0.0f;
            tot[t][i] = 0;
        }
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    Stage<kToks> st;
    uint4 sdig = make_uint4(0, 0, 0, 0);
    auto stage_load5 = [&](uint32_t b) {
        stage_load<kToks>(st, aq, ad, tok0, last_tok, nb, b, tid);
        if (tid < kToks)
            sdig = *reinterpret_cast<const uint4 *>(adig + (static_cast<size_t>(min(tok0 + tid, last_tok)) * nb + b) * 16);
    };
    auto stage_store5 = [&](int buf) {
#pragma unroll
        for (int i = 0; i < Stage<kToks>::kChunks; i++) {
            const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;
            *reinterpret_cast<uint2 *>(s_a[buf] + (c >> 5) * kGbStride128 + (c & 31) * 8) = st.v[i];
        }
        if (tid < kToks) {
            s_dx[buf][tid] = st.dx;
            s_dig[buf][tid] = sdig;
        }
    };
    // K slice of this workgroup (blockIdx.z): blocks b0 .. b1, its sums go to the slice's own copy of the output
    const uint32_t b0 = blockIdx.z * nb_slice, b1 = min(nb, b0 + nb_slice);
    out += static_cast<size_t>(blockIdx.z) * seq * rows;
    stage_load5(b0);
    Q5Row cur = q45_load_row<kFifth>(wrow + static_cast<size_t>(b0) * kBlockBytes, khalf);
    stage_store5(0);
    __syncthreads();

    for (uint32_t b = b0; b < b1; b++) {
        const int buf = (b - b0) & 1;
        const uint32_t bn = b + 1 < b1 ? b + 1 : b;  // the last step reloads its own block, unused
        stage_load5(bn);
        const Q5Row nxt = q45_load_row<kFifth>(wrow + static_cast<size_t>(bn) * kBlockBytes, khalf);
        const uint8_t *abase = s_a[buf] + lrow * kGbStride128 + 16 * khalf;
        const Q4KScales sc8 = unpack_q4k_scales(cur.hdr.y, cur.hdr.z, cur.hdr.w);

        if constexpr (kFifth) {
#define RNB_Q5_SUB_BLOCK(SB)                                                                                           \
    {                                                                                                                  \
        const v4i bop = q45_operand<SB, kFifth>(cur);                                                                  \
        const int sc = byte_of(sc8.sc_lo, sc8.sc_hi, SB);                                                              \
        v16i acc[kTT]; /* the tiles' instructions first, then their results: see the Q6_K kernel */                    \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                              \
            const v4i aop = *reinterpret_cast<const v4i *>(abase + 32 * t * kGbStride128 + 32 * (SB));                 \
            acc[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bop, zero16, 0, 0, 0);                                 \
        }                                                                                                              \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                              \
            _Pragma("unroll") for (int i = 0; i < kLive; i++) {                                                        \
                tot[t][i] += mul24(acc[t][i], sc); /* |I_sb| <= 32 * 31 * 127 */                                       \
                asm volatile("" : "+v"(tot[t][i])); /* no re-association of the eight sums into a tree */              \
            }                                                                                                          \
        }                                                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                                             \
    }
            RNB_Q5_SUB_BLOCK(0)
            RNB_Q5_SUB_BLOCK(1)
            RNB_Q5_SUB_BLOCK(2)
            RNB_Q5_SUB_BLOCK(3)
            RNB_Q5_SUB_BLOCK(4)
            RNB_Q5_SUB_BLOCK(5)
            RNB_Q5_SUB_BLOCK(6)
            RNB_Q5_SUB_BLOCK(7)
#undef RNB_Q5_SUB_BLOCK
        } else {
            // Q4_K: the 6-bit scale is folded into the weight operand as in gemm_q4k.hip (sc = lo + 8 * hi, lo * nib and
            // hi * nib <= 105 are int8 values made with one packed 16-bit multiply per four weights), two accumulator
            // chains over the whole super-block and I = I_lo + 8 * I_hi: no multiply-add per result and sub-block
            const uint32_t dlo[2] = {sc8.sc_lo & 0x07070707u, sc8.sc_hi & 0x07070707u};
            const uint32_t dhi[2] = {(sc8.sc_lo >> 3) & 0x07070707u, (sc8.sc_hi >> 3) & 0x07070707u};
            v16i acc_lo[kTT], acc_hi[kTT];
#define RNB_Q4_SUB_BLOCK(SB)                                                                                           \
    {                                                                                                                  \
        const v4i nib = q45_operand<SB, false>(cur);                                                                   \
        constexpr uint32_t sel = 0x0c000c00u | (((SB) & 3) << 16) | ((SB) & 3);                                        \
        const uint32_t slo = __builtin_amdgcn_perm(0u, dlo[(SB) >> 2], sel);                                           \
        const uint32_t shi = __builtin_amdgcn_perm(0u, dhi[(SB) >> 2], sel);                                           \
        const v4i wlo = {pk_scale(nib[0], slo), pk_scale(nib[1], slo), pk_scale(nib[2], slo), pk_scale(nib[3], slo)};  \
        const v4i whi = {pk_scale(nib[0], shi), pk_scale(nib[1], shi), pk_scale(nib[2], shi), pk_scale(nib[3], shi)};  \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                              \
            const v4i aop = *reinterpret_cast<const v4i *>(abase + 32 * t * kGbStride128 + 32 * (SB));                 \
            acc_lo[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, wlo, (SB) == 0 ? zero16 : acc_lo[t], 0, 0, 0);      \
            acc_hi[t] = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, whi, (SB) == 0 ? zero16 : acc_hi[t], 0, 0, 0);      \
        }                                                                                                              \
    }
            RNB_Q4_SUB_BLOCK(0)
            RNB_Q4_SUB_BLOCK(1)
            RNB_Q4_SUB_BLOCK(2)
            RNB_Q4_SUB_BLOCK(3)
            RNB_Q4_SUB_BLOCK(4)
            RNB_Q4_SUB_BLOCK(5)
            RNB_Q4_SUB_BLOCK(6)
            RNB_Q4_SUB_BLOCK(7)
#undef RNB_Q4_SUB_BLOCK
#pragma unroll
            for (int t = 0; t < kTT; t++)
#pragma unroll
                for (int i = 0; i < kLive; i++) tot[t][i] = acc_lo[t][i] + 8 * acc_hi[t][i];
        }

        // mins: K slots 0..7 of the lower K-half carry the eight mins (weights) and the eight digits (tokens)
        const float d = f16_bits_to_f32(cur.hdr.x), dmin = f16_bits_to_f32(cur.hdr.x >> 16);
        const long mnop = khalf == 0 ? static_cast<long>(static_cast<unsigned long>(sc8.mn_lo) |
                                                         (static_cast<unsigned long>(sc8.mn_hi) << 32))
                                     : 0L;
#pragma unroll
        for (int t = 0; t < kTT; t++) {
            const uint4 dig = s_dig[buf][32 * t + lrow];
            const long op0 = khalf == 0 ? static_cast<long>(static_cast<unsigned long>(dig.x) | (static_cast<unsigned long>(dig.y) << 32)) : 0L;
            const long op1 = khalf == 0 ? static_cast<long>(static_cast<unsigned long>(dig.z) | (static_cast<unsigned long>(dig.w) << 32)) : 0L;
            const v16i c0 = __builtin_amdgcn_mfma_i32_32x32x16_i8(op0, mnop, zero16, 0, 0, 0);
            const v16i c1 = __builtin_amdgcn_mfma_i32_32x32x16_i8(op1, mnop, zero16, 0, 0, 0);
#pragma unroll
            for (int j = 0; j < kLive / 4; j++) {
                const float4 dx4 = reinterpret_cast<const float4 *>(s_dx[buf])[8 * t + 2 * j + khalf];
                const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = 4 * j + i;
                    const int smin = c0[r] + 64 * c1[r];
                    accf[t][r] += dx[i] * (d * static_cast<float>(tot[t][r]) - dmin * static_cast<float>(smin));
                    tot[t][r] = 0;
                }
            }
        }
        stage_store5(buf ^ 1);
        cur = nxt;
        __syncthreads();
    }

    if (row < rows) {
#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int r = 0; r < kLive; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row] = accf[t][r];
            }
    }
}

// ---------------------------------------------------------------------------------------------
// The 32-element formats against 32-wide Q8 activations (one f32 scale per 32 elements): Q8_0 {f16 d, i8 qs[32]} (34
// bytes), Q8_1 {f16 d, f16 s, i8 qs[32]} (36), and the nibble formats Q4_0 {d, 16 bytes} (18; element j < 16 = low nibble
// of byte j, j + 16 the high one; value d (n - 8)), Q4_1 {d, m, 16 bytes} (20; d n + m), Q5_0 {d, u32 qh, 16 bytes} (22;
// fifth bit of element j = bit j of qh; d (n - 16)), Q5_1 {d, m, qh, 16 bytes} (24; d n + m).  A step covers 8 blocks
// = 256 elements, staged exactly like a Q8_K block.  The K-half of a lane is elements 16 khalf .. + 16 of a block: for
// the nibble formats the low (khalf 0) or high nibbles of the same 16 bytes.
// ---------------------------------------------------------------------------------------------
template <uint32_t kFmt>
struct B32 {
    static constexpr bool kNibbles = kFmt == kQ4_0 || kFmt == kQ4_1 || kFmt == kQ5_0 || kFmt == kQ5_1;
    static constexpr bool kFifth = kFmt == kQ5_0 || kFmt == kQ5_1;
    static constexpr bool kMin = kFmt == kQ4_1 || kFmt == kQ5_1;  // value = d * code + m
    static constexpr int kBytes = kFmt == kQ8_0 ? 34 : kFmt == kQ8_1 ? 36 : kFmt == kQ4_0 ? 18 : kFmt == kQ4_1 ? 20 : kFmt == kQ5_0 ? 22 : 24;
    static constexpr int kQhOff = kMin ? 4 : 2;
    static constexpr int kQsOff = kFmt == kQ8_0 ? 2 : kFmt == kQ8_1 ? 4 : kBytes - 16;
};

struct Q8Blocks {
    uint4 q[8];       // Q8: the lane's 16 codes (K-half) of each of the 8 blocks; nibble formats: the block's 16 bytes
    uint32_t qh[8];   // fifth bits (Q5_0, Q5_1)
    float d[8], m[8];
};

template <uint32_t kFmt>
__device__ __forceinline__ Q8Blocks q8_load_blocks(const uint8_t *__restrict__ rowp, uint32_t blk0, uint32_t nb32, int khalf) {
    Q8Blocks r;
#pragma unroll
    for (int k = 0; k < 8; k++) {
        const uint32_t b = min(blk0 + k, nb32 - 1);  // a partial last step repeats the last block; its results are dropped
        const uint8_t *blk = rowp + static_cast<size_t>(b) * B32<kFmt>::kBytes;
        r.q[k] = ld_u4_a2(blk + B32<kFmt>::kQsOff + (B32<kFmt>::kNibbles ? 0 : 16 * khalf));
        r.d[k] = ld_f16(blk);
        r.qh[k] = 0;
        r.m[k] = 0.0f;
        if constexpr (B32<kFmt>::kFifth) r.qh[k] = ld_u32_a2(blk + B32<kFmt>::kQhOff);
        if constexpr (B32<kFmt>::kMin) r.m[k] = ld_f16(blk + 2);
    }
    return r;
}

// the lane's 16 codes of a block as signed bytes: Q8 as stored; nibbles split by K-half, fifth bits spread with one
// multiply per four (bit j of a 4-bit group to bit 8 j), the symmetric formats' offset (8, 16) taken in packed bytes
template <uint32_t kFmt>
__device__ __forceinline__ v4i b32_operand(uint4 q, uint32_t qh, int khalf) {
    uint32_t v[4] = {q.x, q.y, q.z, q.w};
    if constexpr (B32<kFmt>::kNibbles) {
        const uint32_t bits = khalf ? qh >> 16 : qh & 0xffffu;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = khalf ? (v[i] >> 4) & 0x0f0f0f0fu : v[i] & 0x0f0f0f0fu;
            if constexpr (B32<kFmt>::kFifth) v[i] |= ((((bits >> (4 * i)) & 0xfu) * 0x00204081u) & 0x01010101u) << 4;
            if constexpr (kFmt == kQ4_0) v[i] = (v[i] + 0x78787878u) ^ 0x80808080u;  // n - 8 per byte, no carries
            if constexpr (kFmt == kQ5_0) v[i] = (v[i] + 0x70707070u) ^ 0x80808080u;  // n - 16
        }
    }
    return v4i{static_cast<int>(v[0]), static_cast<int>(v[1]), static_cast<int>(v[2]), static_cast<int>(v[3])};
}

// Route of a wave's 32 rows of one step (8 blocks) to the lanes that own them, by whole cache lines (see RowRoute):
// lane takes the 16-byte half j % 2 of block j / 2 (j = lane % 16) of rows lane / 16 + 4 i, and the scale of block
// lane % 8 of rows lane / 8 + 8 i.  In the strip a row is its 256 codes (rows kGbStride128 bytes apart), followed by
// the 32 rows' scales (8 f16 each).  Only for rows whose block count is a multiple of 8, where every step is whole.
constexpr int kQ8StripBytes = 32 * kGbStride128 + 32 * 16;

struct Q8Route {
    uint32_t qoff[8], doff[4];  // byte offsets from the wave's first row (rows past the end: the last row)
    uint4 q[8];
    uint16_t d[4];
};

template <int kBlockBytes, int kQsOff>
__device__ __forceinline__ void q8_route_setup(Q8Route &rt, uint32_t rows_left, size_t row_bytes, int lane) {
#pragma unroll
    for (int i = 0; i < 8; i++)
        rt.qoff[i] = static_cast<uint32_t>(min(static_cast<uint32_t>(lane >> 4) + 4 * i, rows_left - 1) * row_bytes) +
                     ((lane & 15) >> 1) * kBlockBytes + kQsOff + 16 * (lane & 1);
#pragma unroll
    for (int i = 0; i < 4; i++)
        rt.doff[i] = static_cast<uint32_t>(min(static_cast<uint32_t>(lane >> 3) + 8 * i, rows_left - 1) * row_bytes) +
                     (lane & 7) * kBlockBytes;
}

__device__ __forceinline__ void q8_route_load(Q8Route &rt, const uint8_t *__restrict__ base) {
#pragma unroll
    for (int i = 0; i < 8; i++) rt.q[i] = ld_u4_a2(base + rt.qoff[i]);
#pragma unroll
    for (int i = 0; i < 4; i++) rt.d[i] = *reinterpret_cast<const uint16_t *>(base + rt.doff[i]);
}

__device__ __forceinline__ void q8_route_store(const Q8Route &rt, uint8_t *strip, int lane) {
#pragma unroll
    for (int i = 0; i < 8; i++)
        *reinterpret_cast<uint4 *>(strip + ((lane >> 4) + 4 * i) * kGbStride128 + 16 * (lane & 15)) = rt.q[i];
#pragma unroll
    for (int i = 0; i < 4; i++)
        *reinterpret_cast<uint16_t *>(strip + 32 * kGbStride128 + ((lane >> 3) + 8 * i) * 16 + 2 * (lane & 7)) = rt.d[i];
}

__device__ __forceinline__ Q8Blocks q8_blocks_from_strip(const uint8_t *strip, int lrow, int khalf) {
    Q8Blocks r;
#pragma unroll
    for (int k = 0; k < 8; k++)
        r.q[k] = *reinterpret_cast<const uint4 *>(strip + lrow * kGbStride128 + 32 * k + 16 * khalf);
    const uint4 d8 = *reinterpret_cast<const uint4 *>(strip + 32 * kGbStride128 + lrow * 16);
    const uint32_t dw[4] = {d8.x, d8.y, d8.z, d8.w};
#pragma unroll
    for (int k = 0; k < 8; k++) r.d[k] = f16_bits_to_f32(dw[k >> 1] >> (16 * (k & 1)));
    return r;
}

// The same route for the nibble formats, whose block has one 16-byte piece (the nibbles; both K-halves read it) and a
// header of two to eight bytes: lane takes block lane % 8 of rows lane / 8 + 8 i.  In the strip a row is its eight pieces
// (144 bytes apart: conflict-free 128-bit reads) and, after the 32 rows, eight pairs {d | m << 16, qh} per row.  The strip is no
// larger than the Q8 one, so both share the LDS layout.
struct N4Route {
    uint32_t off[4];  // byte offset of the lane's block from the wave's first row (rows past the end: the last row)
    uint4 q[4];
    uint32_t dm[4], qh[4];
};
constexpr int kN4RowStride = 144;
static_assert(32 * kN4RowStride + 32 * 64 <= kQ8StripBytes, "the nibble strip fits the Q8 strip");

template <uint32_t kFmt>
__device__ __forceinline__ void n4_route_setup(N4Route &rt, uint32_t rows_left, size_t row_bytes, int lane) {
#pragma unroll
    for (int i = 0; i < 4; i++)
        rt.off[i] = static_cast<uint32_t>(min(static_cast<uint32_t>(lane >> 3) + 8 * i, rows_left - 1) * row_bytes) +
                    (lane & 7) * B32<kFmt>::kBytes;
}

template <uint32_t kFmt>
__device__ __forceinline__ void n4_route_load(N4Route &rt, const uint8_t *__restrict__ base) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        rt.q[i] = ld_u4_a2(base + rt.off[i] + B32<kFmt>::kQsOff);
        if constexpr (B32<kFmt>::kMin)
            rt.dm[i] = ld_u32_a2(base + rt.off[i]);
        else
            rt.dm[i] = *reinterpret_cast<const uint16_t *>(base + rt.off[i]);
        rt.qh[i] = 0;
        if constexpr (B32<kFmt>::kFifth) rt.qh[i] = ld_u32_a2(base + rt.off[i] + B32<kFmt>::kQhOff);
    }
}

__device__ __forceinline__ void n4_route_store(const N4Route &rt, uint8_t *strip, int lane) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int r = (lane >> 3) + 8 * i;
        *reinterpret_cast<uint4 *>(strip + r * kN4RowStride + 16 * (lane & 7)) = rt.q[i];
        *reinterpret_cast<uint2 *>(strip + 32 * kN4RowStride + r * 64 + 8 * (lane & 7)) = make_uint2(rt.dm[i], rt.qh[i]);
    }
}

__device__ __forceinline__ Q8Blocks n4_blocks_from_strip(const uint8_t *strip, int lrow) {
    Q8Blocks r;
#pragma unroll
    for (int k = 0; k < 8; k++) r.q[k] = *reinterpret_cast<const uint4 *>(strip + lrow * kN4RowStride + 16 * k);
#pragma unroll
    for (int p = 0; p < 4; p++) {  // two blocks' {d | m << 16, qh} per 128-bit read
        const uint4 h = *reinterpret_cast<const uint4 *>(strip + 32 * kN4RowStride + lrow * 64 + 16 * p);
        r.d[2 * p] = f16_bits_to_f32(h.x);
        r.m[2 * p] = f16_bits_to_f32(h.x >> 16);
        r.qh[2 * p] = h.y;
        r.d[2 * p + 1] = f16_bits_to_f32(h.z);
        r.m[2 * p + 1] = f16_bits_to_f32(h.z >> 16);
        r.qh[2 * p + 1] = h.w;
    }
    return r;
}

template <int kTT>
constexpr size_t q8_lds_bytes(bool routed) {
    return 2 * (32 * kTT) * kGbStride128 + 2 * 8 * (32 * kTT) * sizeof(float) + (routed ? kGbWaves * kQ8StripBytes : 0);
}

template <int kTT, uint32_t kFmt, bool kRouted, int kLive>
__global__ void __launch_bounds__(kGbThreads, 2)
    gemm_q8_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                        float *__restrict__ out, uint32_t rows, uint32_t nb32, uint32_t seq, uint32_t steps_slice) {
    constexpr int kToks = 32 * kTT;
    constexpr int kDxPerThread = kToks * 8 / kGbThreads;  // 1 (32 tokens) or 2 (64 tokens)
    constexpr int kBlockBytes = B32<kFmt>::kBytes, kQsOff = B32<kFmt>::kQsOff;
    extern __shared__ __attribute__((aligned(16))) uint8_t s_dyn[];
    uint8_t(*s_a)[kToks * kGbStride128] = reinterpret_cast<uint8_t(*)[kToks * kGbStride128]>(s_dyn);
    float(*s_dx)[8][kToks] = reinterpret_cast<float(*)[8][kToks]>(s_dyn + 2 * kToks * kGbStride128);  // [block][token]
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t row = blockIdx.x * kGbRows + wave * 32 + lrow;
    const uint32_t tok0 = blockIdx.y * kToks, last_tok = seq - 1;
    const uint8_t *wrow = w + static_cast<size_t>(min(row, rows - 1)) * nb32 * kBlockBytes;
    // K slice of this workgroup (blockIdx.z): steps s0 .. s1, its sums go to the slice's own copy of the output
    const uint32_t s0 = blockIdx.z * steps_slice, s1 = min((nb32 + 7) / 8, s0 + steps_slice);
    out += static_cast<size_t>(blockIdx.z) * seq * rows;
    const size_t tok_bytes = static_cast<size_t>(nb32) * 32;

    float accf[kTT][16];
#pragma unroll
    for (int t = 0; t < kTT; t++)
#pragma unroll
        for (int i = 0; i < 16; i++) accf[t][i] = 0.0f;
    const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

    uint2 sv[kToks * 32 / kGbThreads];
    float sdx[kDxPerThread];
    auto stage_load8 = [&](uint32_t step) {
#pragma unroll
        for (int i = 0; i < kToks * 32 / kGbThreads; i++) {
            const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;
            const uint32_t t = min(tok0 + (c >> 5), last_tok);
            // 8-byte chunk (c & 31) of the step; chunks past the end of the row re-read the row's last 8 bytes
            const size_t off = min(static_cast<size_t>(step) * 256 + (c & 31) * 8, tok_bytes - 8);
            sv[i] = *reinterpret_cast<const uint2 *>(aq + static_cast<size_t>(t) * tok_bytes + off);
        }
#pragma unroll
        for (int i = 0; i < kDxPerThread; i++) {
            const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;  // c = block-in-step * kToks + token
            const uint32_t t = min(tok0 + c % kToks, last_tok);
            const uint32_t blk = min(step * 8 + c / kToks, nb32 - 1);
            sdx[i] = ad[static_cast<size_t>(t) * nb32 + blk];
        }
    };
    auto stage_store8 = [&](int buf) {
#pragma unroll
        for (int i = 0; i < kToks * 32 / kGbThreads; i++) {
            const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;
            *reinterpret_cast<uint2 *>(s_a[buf] + (c >> 5) * kGbStride128 + (c & 31) * 8) = sv[i];
        }
#pragma unroll
        for (int i = 0; i < kDxPerThread; i++) {
            const uint32_t c = static_cast<uint32_t>(tid) + i * kGbThreads;
            s_dx[buf][c / kToks][c % kToks] = sdx[i];
        }
    };

    const uint32_t wrow0 = min(blockIdx.x * kGbRows + wave * 32, rows - 1);
    const uint8_t *wbase = w + static_cast<size_t>(wrow0) * nb32 * kBlockBytes;
    uint8_t *strip = s_dyn + q8_lds_bytes<kTT>(false) + wave * kQ8StripBytes;
    Q8Route rt;
    N4Route nrt;
    Q8Blocks cur, nxt;
    stage_load8(s0);
    if constexpr (kRouted) {
        if constexpr (B32<kFmt>::kNibbles) {
            n4_route_setup<kFmt>(nrt, rows - wrow0, static_cast<size_t>(nb32) * kBlockBytes, lane);
            n4_route_load<kFmt>(nrt, wbase + static_cast<size_t>(s0) * 8 * kBlockBytes);
            n4_route_store(nrt, strip, lane);
            cur = n4_blocks_from_strip(strip, lrow);
        } else {
            q8_route_setup<kBlockBytes, kQsOff>(rt, rows - wrow0, static_cast<size_t>(nb32) * kBlockBytes, lane);
            q8_route_load(rt, wbase + static_cast<size_t>(s0) * 8 * kBlockBytes);
            q8_route_store(rt, strip, lane);
            cur = q8_blocks_from_strip(strip, lrow, khalf);
        }
    } else {
        cur = q8_load_blocks<kFmt>(wrow, s0 * 8, nb32, khalf);
    }
    stage_store8(0);
    __syncthreads();

    for (uint32_t step = s0; step < s1; step++) {
        const int buf = (step - s0) & 1;
        const uint32_t sn = step + 1 < s1 ? step + 1 : step;
        stage_load8(sn);
        if constexpr (kRouted)
            if constexpr (B32<kFmt>::kNibbles)
                n4_route_load<kFmt>(nrt, wbase + static_cast<size_t>(sn) * 8 * kBlockBytes);
            else
                q8_route_load(rt, wbase + static_cast<size_t>(sn) * 8 * kBlockBytes);
        else
            nxt = q8_load_blocks<kFmt>(wrow, sn * 8, nb32, khalf);
        const uint8_t *abase = s_a[buf] + lrow * kGbStride128 + 16 * khalf;
        const uint32_t live = min(8u, nb32 - step * 8);  // blocks of this step that exist (workgroup-uniform)
#pragma unroll
        for (int k = 0; k < 8; k++) {
            if (static_cast<uint32_t>(k) < live) {
                const v4i bop = b32_operand<kFmt>(cur.q[k], cur.qh[k], khalf);
#pragma unroll
                for (int t = 0; t < kTT; t++) {
                    const v4i aop = *reinterpret_cast<const v4i *>(abase + 32 * t * kGbStride128 + 32 * k);
                    const v16i acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, bop, zero16, 0, 0, 0);
                    v16i sum = zero16;  // d n + m formats: the block's sum of activations, from a row of ones
                    if constexpr (B32<kFmt>::kMin) {
                        const v4i ones = {0x01010101, 0x01010101, 0x01010101, 0x01010101};
                        sum = __builtin_amdgcn_mfma_i32_32x32x32_i8(aop, ones, zero16, 0, 0, 0);
                    }
#pragma unroll
                    for (int j = 0; j < kLive / 4; j++) {
                        const float4 dx4 = reinterpret_cast<const float4 *>(s_dx[buf][k])[8 * t + 2 * j + khalf];
                        const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                        for (int i = 0; i < 4; i++) {
                            accf[t][4 * j + i] += (cur.d[k] * dx[i]) * static_cast<float>(acc[4 * j + i]);
                            if constexpr (B32<kFmt>::kMin)
                                accf[t][4 * j + i] += (cur.m[k] * dx[i]) * static_cast<float>(sum[4 * j + i]);
                        }
                    }
                }
            }
        }
        stage_store8(buf ^ 1);
        if constexpr (kRouted) {
            if constexpr (B32<kFmt>::kNibbles) {
                n4_route_store(nrt, strip, lane);
                cur = n4_blocks_from_strip(strip, lrow);
            } else {
                q8_route_store(rt, strip, lane);
                cur = q8_blocks_from_strip(strip, lrow, khalf);
            }
        } else {
            cur = nxt;
        }
        __syncthreads();
    }

    if (row < rows) {
#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int r = 0; r < kLive; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row] = accf[t][r];
            }
    }
}

}  // namespace

// 64-token workgroups halve the weight re-reads, 32-token ones double the number of workgroups: the wider tile only when
// it still leaves about two workgroups per compute unit (Q6_K 4096 x 4096 x 64: 76 -> 52 us; Q5_K 4096 x 14336 x 512:
// 153 -> 138 us)
static bool wide_tiles(uint32_t row_tiles, uint32_t seq) {
    return seq > 32 && static_cast<uint64_t>(row_tiles) * ((seq + 63) / 64) >= 512;
}

// ---------------------------------------------------------------------------------------------
// K slices.  A grid of rows / 128 x tokens / 32 workgroups leaves most of the 256 compute units idle when both are
// small (a 4096-row projection of 64 tokens: 64 workgroups, each walking the whole row): then the blocks of a row are
// dealt out to blockIdx.z, every slice writes its own copy of the output and a second small kernel adds the copies in
// slice order, so the result does not depend on which slice finishes first.
// ---------------------------------------------------------------------------------------------
constexpr uint32_t kSliceTargetWgs = 512;  // slices are added until the grid has this many workgroups
constexpr uint32_t kSliceMax = 16;

// measured on 4096 x 4096 and 4096 x 14336 at 16 .. 256 tokens: up to 5x faster where the unsliced grid has at most 128
// workgroups; at 256 workgroups only Q6_K and Q8 (the slowest per block) still gain, hence split_at_256; a slice keeps
// four 256-element steps, two on the smallest grids
static uint32_t k_slices(uint64_t wgs, uint32_t k_steps, bool split_at_256) {
    if (wgs > 256 || (wgs == 256 && !split_at_256)) return 1;
    const uint64_t want = (kSliceTargetWgs + wgs - 1) / wgs;
    const uint32_t min_steps = wgs <= 32 ? 2 : 4;
    return static_cast<uint32_t>(std::max<uint64_t>(1, std::min<uint64_t>({want, k_steps / min_steps, kSliceMax})));
}

static uint64_t tile_grid(uint32_t rows, uint32_t seq, bool wide) {
    return static_cast<uint64_t>((rows + kGbRows - 1) / kGbRows) * (wide ? (seq + 63) / 64 : (seq + 31) / 32);
}

namespace {
__global__ void __launch_bounds__(256) sum_slices_kernel(const float *__restrict__ parts, float *__restrict__ out, size_t n,
                                                         uint32_t slices) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= n) return;
    float acc = parts[i];
    for (uint32_t z = 1; z < slices; z++) acc += parts[z * n + i];
    out[i] = acc;
}
}  // namespace

void launch_sum_slices(const float *parts, float *out, size_t n, uint32_t slices, hipStream_t stream) {
    hipLaunchKernelGGL(sum_slices_kernel, dim3(static_cast<uint32_t>((n + 255) / 256)), dim3(256), 0, stream, parts, out, n,
                       slices);
}

static bool is_b32(uint32_t quant) {
    return quant == kQ8_0 || quant == kQ8_1 || quant == kQ4_0 || quant == kQ4_1 || quant == kQ5_0 || quant == kQ5_1;
}

// Q6_K spends the most vector work per tile, and the 64-token form saves the most of it: it also wins where its
// workgroups fill the 256 compute units just once (4096 rows x 512 tokens x 14336: 164 vs 189 us; with 224 or 320
// workgroups the 32-token form is level or ahead)
static bool q6_wide_tiles(uint32_t row_tiles, uint32_t seq) {
    const uint64_t tiles = static_cast<uint64_t>(row_tiles) * ((seq + 63) / 64);
    return seq > 32 && (tiles >= 512 || (tiles > 224 && tiles <= 256));
}

size_t gemm_blocks_slice_floats(uint32_t quant, uint32_t rows, uint32_t k_steps, uint32_t seq) {
    if (rows == 0 || seq == 0 || k_steps == 0) return 0;
    const uint32_t row_tiles = (rows + kGbRows - 1) / kGbRows;
    const bool wide = is_b32(quant) ? seq > 32
                      : quant == kQ6K                    ? q6_wide_tiles(row_tiles, seq)
                                                         : wide_tiles(row_tiles, seq);
    const uint32_t slices = k_slices(tile_grid(rows, seq, wide), k_steps, quant != kQ4K && quant != kQ5K);  // as the launchers
    return slices > 1 ? static_cast<size_t>(slices) * seq * rows : 0;
}

// A batch of at most 8 / 16 tokens fills only the first 4 / 8 of the sixteen results a lane holds per 32-token tile
// (result r is token 8 (r / 4) + 4 khalf + r % 4): the kernels are instantiated for 4, 8 and 16 live results and apply
// scales, float updates and stores to those only.
#define RNB_BY_LIVE_TOKENS(SEQ, LAUNCH) \
    do {                                \
        if ((SEQ) <= 8)                 \
            LAUNCH(4);                  \
        else if ((SEQ) <= 16)           \
            LAUNCH(8);                  \
        else                            \
            LAUNCH(16);                 \
    } while (0)

void launch_gemm_q6k_mfma(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                          uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    const uint32_t row_tiles = (rows + kGbRows - 1) / kGbRows;
    const bool wide = q6_wide_tiles(row_tiles, seq);
    const uint32_t slices = slice_out ? k_slices(tile_grid(rows, seq, wide), nb, true) : 1;
    const uint32_t nb_slice = (nb + slices - 1) / slices, nz = (nb + nb_slice - 1) / nb_slice;
    float *dst = nz > 1 ? slice_out : out;
    if (wide) {
        const dim3 grid(row_tiles, (seq + 63) / 64, nz);
        hipLaunchKernelGGL((gemm_q6k_mfma_kernel<2, 16>), grid, dim3(kGbThreads), 0, stream, w, act.qs, act.d, dst, rows, nb,
                           seq, nb_slice);
    } else {
        const dim3 grid(row_tiles, (seq + 31) / 32, nz);
#define RNB_LAUNCH_Q6(LIVE)                                                                                            \
    hipLaunchKernelGGL((gemm_q6k_mfma_kernel<1, LIVE>), grid, dim3(kGbThreads), 0, stream, w, act.qs, act.d, dst, rows, nb, \
                       seq, nb_slice)
        RNB_BY_LIVE_TOKENS(seq, RNB_LAUNCH_Q6);
#undef RNB_LAUNCH_Q6
    }
    if (nz > 1) launch_sum_slices(slice_out, out, static_cast<size_t>(seq) * rows, nz, stream);
}

void launch_gemm_q23k_mfma(const uint8_t *w, uint32_t quant, ActView act, float *out, float *slice_out, uint32_t rows,
                           uint32_t nb, uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    const uint32_t row_tiles = (rows + kGbRows - 1) / kGbRows;
    const bool wide = wide_tiles(row_tiles, seq);
    const uint32_t slices = slice_out ? k_slices(tile_grid(rows, seq, wide), nb, true) : 1;
    const uint32_t nb_slice = (nb + slices - 1) / slices, nz = (nb + nb_slice - 1) / nb_slice;
    float *dst = nz > 1 ? slice_out : out;
    const dim3 grid(row_tiles, wide ? (seq + 63) / 64 : (seq + 31) / 32, nz), block(kGbThreads);
#define RNB_LAUNCH_Q23(TT, THREE, LIVE)                                                                                \
    hipLaunchKernelGGL((gemm_q23k_mfma_kernel<TT, THREE, LIVE>), grid, block, 0, stream, w, act.qs, act.d, act.bsums, dst, \
                       rows, nb, seq, nb_slice)
#define RNB_LAUNCH_Q3_LIVE(LIVE) RNB_LAUNCH_Q23(1, true, LIVE)
#define RNB_LAUNCH_Q2_LIVE(LIVE) RNB_LAUNCH_Q23(1, false, LIVE)
    if (quant == kQ3K) {
        if (wide)
            RNB_LAUNCH_Q23(2, true, 16);
        else
            RNB_BY_LIVE_TOKENS(seq, RNB_LAUNCH_Q3_LIVE);
    } else {
        if (wide)
            RNB_LAUNCH_Q23(2, false, 16);
        else
            RNB_BY_LIVE_TOKENS(seq, RNB_LAUNCH_Q2_LIVE);
    }
#undef RNB_LAUNCH_Q2_LIVE
#undef RNB_LAUNCH_Q3_LIVE
#undef RNB_LAUNCH_Q23
    if (nz > 1) launch_sum_slices(slice_out, out, static_cast<size_t>(seq) * rows, nz, stream);
}

template <bool kFifth>
static void launch_gemm_q45k(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                             uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    const uint32_t row_tiles = (rows + kGbRows - 1) / kGbRows;
    const bool wide = wide_tiles(row_tiles, seq);
    const uint32_t slices = slice_out ? k_slices(tile_grid(rows, seq, wide), nb, false) : 1;
    const uint32_t nb_slice = (nb + slices - 1) / slices, nz = (nb + nb_slice - 1) / nb_slice;
    float *dst = nz > 1 ? slice_out : out;
    if (wide) {
        const dim3 grid(row_tiles, (seq + 63) / 64, nz);
        hipLaunchKernelGGL((gemm_q45k_mfma_kernel<2, kFifth, 16>), grid, dim3(kGbThreads), 0, stream, w, act.qs, act.d,
                           act.digits, dst, rows, nb, seq, nb_slice);
    } else {
        const dim3 grid(row_tiles, (seq + 31) / 32, nz);
#define RNB_LAUNCH_Q45(LIVE)                                                                                           \
    hipLaunchKernelGGL((gemm_q45k_mfma_kernel<1, kFifth, LIVE>), grid, dim3(kGbThreads), 0, stream, w, act.qs, act.d,  \
                       act.digits, dst, rows, nb, seq, nb_slice)
        RNB_BY_LIVE_TOKENS(seq, RNB_LAUNCH_Q45);
#undef RNB_LAUNCH_Q45
    }
    if (nz > 1) launch_sum_slices(slice_out, out, static_cast<size_t>(seq) * rows, nz, stream);
}

void launch_gemm_q5k_mfma(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                          uint32_t seq, hipStream_t stream) {
    launch_gemm_q45k<true>(w, act, out, slice_out, rows, nb, seq, stream);
}

void launch_gemm_q4k_small(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                           uint32_t seq, hipStream_t stream) {
    launch_gemm_q45k<false>(w, act, out, slice_out, rows, nb, seq, stream);
}

bool gemm_q8_mfma_supported(uint32_t quant, uint32_t nb32) { return is_b32(quant) && nb32 >= 1; }

void launch_gemm_q8_mfma(const uint8_t *w, uint32_t quant, ActView act, float *out, float *slice_out, uint32_t rows,
                         uint32_t nb32, uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb32 == 0) return;
    const uint32_t row_tiles = (rows + kGbRows - 1) / kGbRows;
    const bool wide = seq > 32;  // measured: the 64-token tile wins here even on a small grid (4096 x 4096 x 512: 100 vs 123 us)
    const uint32_t steps = (nb32 + 7) / 8;
    const uint32_t slices = slice_out ? k_slices(tile_grid(rows, seq, wide), steps, true) : 1;
    const uint32_t steps_slice = (steps + slices - 1) / slices, nz = (steps + steps_slice - 1) / steps_slice;
    float *dst = nz > 1 ? slice_out : out;
    const dim3 grid(row_tiles, wide ? (seq + 63) / 64 : 1, nz), block(kGbThreads);
    // the strip routes: whole steps only (a partial step's pieces would leave the last row)
    const bool routed = nb32 % 8 == 0;
#define RNB_LAUNCH_Q8R(TT, FMT, R, LIVE)                                                                               \
    {                                                                                                                  \
        constexpr size_t lds = q8_lds_bytes<TT>(R);                                                                    \
        static bool configured = false; /* above the default 64 KB of dynamic LDS in the routed 64-token form */       \
        if (!allow_dynamic_lds(reinterpret_cast<const void *>(gemm_q8_mfma_kernel<TT, FMT, R, LIVE>), lds, &configured, \
                               "gemm_q8_mfma_kernel"))                                                                 \
            return;                                                                                                    \
        hipLaunchKernelGGL((gemm_q8_mfma_kernel<TT, FMT, R, LIVE>), grid, block, lds, stream, w, act.qs, act.d, dst,   \
                           rows, nb32, seq, steps_slice);                                                              \
    }
#define RNB_LAUNCH_Q8N(FMT, R) /* one 32-token tile: by the number of live results */                                  \
    {                                                                                                                  \
        if (seq <= 8) RNB_LAUNCH_Q8R(1, FMT, R, 4)                                                                     \
        else if (seq <= 16) RNB_LAUNCH_Q8R(1, FMT, R, 8)                                                               \
        else RNB_LAUNCH_Q8R(1, FMT, R, 16)                                                                             \
    }
#define RNB_LAUNCH_Q8(FMT, ROUTABLE)                                                                                   \
    if constexpr (ROUTABLE) {                                                                                          \
        if (routed && wide) RNB_LAUNCH_Q8R(2, FMT, true, 16)                                                           \
        else if (routed) RNB_LAUNCH_Q8N(FMT, true)                                                                     \
        else if (wide) RNB_LAUNCH_Q8R(2, FMT, false, 16)                                                               \
        else RNB_LAUNCH_Q8N(FMT, false)                                                                                \
    } else {                                                                                                           \
        if (wide) RNB_LAUNCH_Q8R(2, FMT, false, 16)                                                                    \
        else RNB_LAUNCH_Q8N(FMT, false)                                                                                \
    }
    switch (quant) {
    case kQ8_0: RNB_LAUNCH_Q8(kQ8_0, true) break;
    case kQ8_1: RNB_LAUNCH_Q8(kQ8_1, true) break;
    case kQ4_0: RNB_LAUNCH_Q8(kQ4_0, true) break;
    case kQ4_1: RNB_LAUNCH_Q8(kQ4_1, true) break;
    case kQ5_0: RNB_LAUNCH_Q8(kQ5_0, true) break;
    default: RNB_LAUNCH_Q8(kQ5_1, true) break;
    }
#undef RNB_LAUNCH_Q8N
#undef RNB_LAUNCH_Q8R
#undef RNB_LAUNCH_Q8
    if (nz > 1) launch_sum_slices(slice_out, out, static_cast<size_t>(seq) * rows, nz, stream);
}

}  // namespace rnb
