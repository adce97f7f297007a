// Decode GEMV kernels: one packed GGUF row x one quantised activation vector -> one f32.
//
//  Q2_K x Q8_K : crates/rnb-cpu/src/gemm/avx2_dot.rs:169-242   (dot_q2k_q8k_avx2)
//  Q3_K x Q8_K : crates/rnb-cpu/src/gemm/avx2_dot.rs:247-375   (dot_q3k_q8k_avx2)
//  Q4_K x Q8_K : crates/rnb-cpu/src/gemm/neon_dot.rs:884-916   (dot_q4_k_q8k_scalar)
//  Q5_K x Q8_K : crates/rnb-cpu/src/gemm/neon_dot.rs:1742-1800 (dot_q5_k_q8k_scalar)
//  Q6_K x Q8_K : crates/rnb-cpu/src/gemm/neon_dot.rs:2240-2288 (dot_q6_k_q8k_scalar)
//  Q8_0 x Q8   : crates/rnb-cpu/src/gemm/neon_dot.rs:376-436   (dot_q8_0_q8_neon); Q4_0, Q4_1, Q5_0, Q5_1 x Q8 below
//  driver      : crates/rnb-cpu/src/gemm/quant_gemv.rs:403-536, out[s*rows + row]
//
// These kernels are HBM-bound: every weight byte is fetched once with 16-byte loads.  Four lanes own
// a 256-element super-block, so a wave64 pass covers 16 super-blocks: one 4096-wide row, or two /
// four shorter rows side by side (kRowsPerWave).  About 4096 waves are launched in total (16 per CU)
// and each walks several rows, so the quantised activation of a lane's K-slice is loaded into
// registers once per wave instead of once per row.  Integer sums per lane are exact
// (v_dot4_i32_i8); the per-block f32 scale is applied once per lane and the partial sums are added
// across lanes on the DPP path, so results differ from the scalar reference only by f32 summation order.

#include "act_quant.h"
#include "block_dots.h"
#include "device_utils.h"
#include "kernels.h"
#include <cstdlib>

namespace rnb {

namespace {

constexpr int kWavesPerWg = 4;
constexpr uint32_t kTargetWaves = 4096;  // total waves per launch: enough loads in flight, short tail
// Matrices from this size on take gemv_kquant_chunks_kernel (measured crossover on Q4_K rows of 16 super-blocks: 33 MB
// 7.5 us either way, 66 MB 12.4 against 13.0 us, 132 MB 22.1 against 24.1 us).
constexpr uint64_t kGemvChunkMinBytes = uint64_t(48) << 20;

// ---------------------------------------------------------------------------------------------
// K-quant GEMV (Q2_K ... Q6_K share the structure; only the block functions differ)
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant, int kRowsPerWave>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_kquant_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                       const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                       uint32_t row_groups) {
    using Q = KQuant<kQuant>;
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    constexpr uint32_t kBlocksPerPass = kLanesPerRow / 4;
    constexpr size_t kBlockBytes = Q::kBytes;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const uint32_t tok = blockIdx.y;
    const size_t abase = static_cast<size_t>(tok) * nb;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;

    if (nb <= kBlocksPerPass) {
        // the whole row fits one pass: this lane's activation slice stays in registers for every row
        const bool has_block = bslot < nb;
        const size_t ab = abase + (has_block ? bslot : 0);
        const typename Q::Act a = Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
        for (uint32_t grp = wave_global; grp < row_groups; grp += n_waves) {
            const uint32_t row = grp * kRowsPerWave + rsel;
            float acc = 0.0f;
            if (has_block && row < rows) {
                const uint8_t *blk = w + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(bslot) * kBlockBytes;
                acc = kquant_partial<kQuant>(Q::load_block(blk, g), a, g);
            }
            acc = seg_sum<kLanesPerRow>(acc);
            if (sub == kLanesPerRow - 1 && row < rows) out[static_cast<size_t>(tok) * rows + row] = acc;
        }
    } else {
        for (uint32_t grp = wave_global; grp < row_groups; grp += n_waves) {
            const uint32_t row = grp * kRowsPerWave + rsel;
            float acc = 0.0f;
            if (row < rows) {
                const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
                for (uint32_t b = bslot; b < nb; b += kBlocksPerPass) {
                    const uint8_t *blk = rowp + static_cast<size_t>(b) * kBlockBytes;
                    const size_t ab = abase + b;
                    acc += kquant_partial<kQuant>(Q::load_block(blk, g),
                                                  Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g), g);
                }
            }
            acc = seg_sum<kLanesPerRow>(acc);
            if (sub == kLanesPerRow - 1 && row < rows) out[static_cast<size_t>(tok) * rows + row] = acc;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Two to four tokens per pass over the matrix (small decode batches, rows of at most 16 super-blocks): the lane keeps
// the activation slices of kTokens tokens in registers, every weight block is fetched and unpacked once and dotted
// against each of them.  Per token the arithmetic and the cross-lane sum are those of gemv_kquant_kernel: same bits.
// grid.y = token groups; the last group may hold fewer tokens (its spare slots repeat the last token and are not stored).
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant, int kRowsPerWave, int kTokens>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_kquant_tokens_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                              const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                              uint32_t row_groups, uint32_t seq) {
    using Q = KQuant<kQuant>;
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    constexpr size_t kBlockBytes = Q::kBytes;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const uint32_t tok0 = blockIdx.y * kTokens;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    const bool has_block = bslot < nb;
    typename Q::Act a[kTokens];
#pragma unroll
    for (int t = 0; t < kTokens; t++) {
        const uint32_t tok = tok0 + t < seq ? tok0 + t : seq - 1;
        const size_t ab = static_cast<size_t>(tok) * nb + (has_block ? bslot : 0);
        a[t] = Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
    }
    for (uint32_t grp = wave_global; grp < row_groups; grp += n_waves) {
        const uint32_t row = grp * kRowsPerWave + rsel;
        const bool live = has_block && row < rows;
        const uint8_t *blk = w + (live ? static_cast<size_t>(row) * row_bytes + static_cast<size_t>(bslot) * kBlockBytes : 0);
        const typename Q::Prep p = Q::prepare(Q::load_block(blk, g), g);  // rows >= 1 and nb >= 1: offset 0 is readable
#pragma unroll
        for (int t = 0; t < kTokens; t++) {
            float acc = live ? Q::dot(p, a[t]) : 0.0f;
            acc = seg_sum<kLanesPerRow>(acc);
            if (sub == kLanesPerRow - 1 && row < rows && tok0 + t < seq) out[static_cast<size_t>(tok0 + t) * rows + row] = acc;
        }
    }
}

// ---------------------------------------------------------------------------------------------
// The same GEMV for matrices far larger than what the chip holds in flight (rows of 9 to 16 super-blocks): every wave
// takes kRows CONSECUTIVE rows, requests all of them at once and retires; with one wave per chunk the hardware
// dispatcher keeps the CUs supplied with fresh waves, so the window of outstanding requests sweeps the matrix in
// address order.  Measured on 264 MB of Q4_K: 41.5 us against 46.4 us for the grid-stride kernel above (80 % against
// 71 % of 8 TB/s); on 33 MB the two are equal, so the launcher keeps the kernel above for small matrices.
// The per-row arithmetic and the cross-lane sum are those of gemv_kquant_kernel: same bits.
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant, int kRows>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_kquant_chunks_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                              const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                              uint32_t n_chunks) {
    using Q = KQuant<kQuant>;
    const int lane = threadIdx.x & (kWave - 1);
    const int g = lane & 3;
    const uint32_t bslot = lane >> 2;
    const bool has_block = bslot < nb;
    const uint32_t tok = blockIdx.y;
    const size_t row_bytes = static_cast<size_t>(nb) * Q::kBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    const size_t ab = static_cast<size_t>(tok) * nb + (has_block ? bslot : 0);
    const typename Q::Act a = Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
    for (uint32_t c = wave_global; c < n_chunks; c += n_waves) {
        typename Q::Regs r[kRows];
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            const uint32_t row = c * kRows + k;
            const bool ok = has_block && row < rows;  // rows >= 1 and nb >= 1: offset 0 is readable
            r[k] = Q::load_block(w + (ok ? static_cast<size_t>(row) * row_bytes + static_cast<size_t>(bslot) * Q::kBytes : 0), g);
        }
        float v = 0.0f;
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            const uint32_t row = c * kRows + k;
            float acc = (has_block && row < rows) ? kquant_partial<kQuant>(r[k], a, g) : 0.0f;
            acc = seg_sum<kWave>(acc);
            // lane 63 - k keeps row k's sum, so that one store instruction writes the chunk
            const float t = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, acc), kWave - 1));
            v = (lane == kWave - 1 - k) ? t : v;
        }
        const uint32_t row = c * kRows + (kWave - 1 - lane);
        if (lane >= kWave - kRows && row < rows) out[static_cast<size_t>(tok) * rows + row] = v;
    }
}

// The chunked GEMV for two to four tokens per pass over the matrix (per token the arithmetic of
// gemv_kquant_chunks_kernel: same bits); grid.y = token groups.
template <uint32_t kQuant, int kRows, int kTokens>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_kquant_chunks_tokens_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                     const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                                     uint32_t n_chunks, uint32_t seq) {
    using Q = KQuant<kQuant>;
    const int lane = threadIdx.x & (kWave - 1);
    const int g = lane & 3;
    const uint32_t bslot = lane >> 2;
    const bool has_block = bslot < nb;
    const uint32_t tok0 = blockIdx.y * kTokens;
    const size_t row_bytes = static_cast<size_t>(nb) * Q::kBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    typename Q::Act a[kTokens];
#pragma unroll
    for (int t = 0; t < kTokens; t++) {
        const uint32_t tok = tok0 + t < seq ? tok0 + t : seq - 1;
        const size_t ab = static_cast<size_t>(tok) * nb + (has_block ? bslot : 0);
        a[t] = Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
    }
    for (uint32_t c = wave_global; c < n_chunks; c += n_waves) {
        typename Q::Regs r[kRows];
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            const uint32_t row = c * kRows + k;
            const bool ok = has_block && row < rows;  // rows >= 1 and nb >= 1: offset 0 is readable
            r[k] = Q::load_block(w + (ok ? static_cast<size_t>(row) * row_bytes + static_cast<size_t>(bslot) * Q::kBytes : 0), g);
        }
#pragma unroll
        for (int k = 0; k < kRows; k++) {
            const uint32_t row = c * kRows + k;
            const typename Q::Prep p = Q::prepare(r[k], g);
#pragma unroll
            for (int t = 0; t < kTokens; t++) {
                float acc = (has_block && row < rows) ? Q::dot(p, a[t]) : 0.0f;
                acc = seg_sum<kWave>(acc);
                if (lane == kWave - 1 && row < rows && tok0 + t < seq) out[static_cast<size_t>(tok0 + t) * rows + row] = acc;
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// K-quant GEMV of ONE f32 token: the workgroup quantises the token to Q8_K itself into LDS (the same wave-level
// quantiser as the stand-alone kernel, so the same bits), then runs the row loop of gemv_kquant_kernel against it.
// Rows of at most 16 super-blocks.  Each lane requests its first rows' weight blocks before the quantisation starts,
// so the weight stream is already in flight while the activation is prepared; the separate quantise launch and the
// gap behind it disappear from a decode step.
// ---------------------------------------------------------------------------------------------
constexpr int kFusedWaves = 8;   // waves per workgroup: each quantises 16 / 8 = 2 blocks of the token
constexpr int kDepth = 1;        // rows requested ahead of the one being reduced (two, with three register sets: 8.16 against 7.99 us)
constexpr uint32_t kFusedTargetWaves = 4096;  // 3584, 4784 and 7168 (whole rows per wave for 14336 rows) measured slower
// Waves of a one-launch decode kernel for `groups` row groups: one per group up to kFusedTargetWaves, except where two
// groups per wave make 1536 - 2048 waves, i.e. one workgroup per compute unit or a little less: then half as many
// workgroups quantise the token and they run in a single round (Q8_0 4096 x 4096 5.65 -> 5.18 us per step, 3072 rows
// 5.20 -> 4.90; Q6_K 4096 x 4096 5.63 -> 5.33, 8192 x 2048 5.40 -> 4.84; Q4_K within 2 % either way; two groups per wave
// on 2048 or 5120 rows of Q8_0, 128 or 320 workgroups, lose 15 %, hence the window).
static uint32_t fused_waves(uint32_t groups) {
    const uint32_t half = (groups + 1) / 2;
    if (half >= 1536 && half <= 2048) return half;
    return groups < kFusedTargetWaves ? groups : kFusedTargetWaves;
}
template <uint32_t kQuant, int kRowsPerWave>
__global__ void __launch_bounds__(kWave *kFusedWaves)
    gemv_kquant_f32_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out,
                           uint32_t rows, uint32_t nb, uint32_t row_groups) {
    using Q = KQuant<kQuant>;
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    constexpr size_t kBlockBytes = Q::kBytes;
    __shared__ __attribute__((aligned(16))) int8_t s_qs[16 * 256];
    __shared__ float s_d[16];
    __shared__ __attribute__((aligned(16))) int16_t s_bsums[16 * 16];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const bool has_block = bslot < nb;
    const uint32_t tok = blockIdx.y;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint32_t n_waves = gridDim.x * kFusedWaves;
    uint32_t grp = blockIdx.x * kFusedWaves + wave;
    uint32_t row = grp * kRowsPerWave + rsel;
    // the activation is requested first: loads return in order, and the quantiser must not wait for weights
    TokenSpans<kFusedWaves> xv;
    token_load<kFusedWaves>(x + static_cast<size_t>(tok) * nb * 256, nb, wave, lane, xv);
    // kDepth rows in flight per lane segment, the first ones requested before the quantisation starts
    typename Q::Regs regs[kDepth];
    bool live[kDepth];
    auto fetch = [&](uint32_t group, bool *ok) {
        const uint32_t r = group * kRowsPerWave + rsel;
        *ok = has_block && group < row_groups && r < rows;
        const size_t off = *ok ? static_cast<size_t>(r) * row_bytes + static_cast<size_t>(bslot) * kBlockBytes : 0;
        return Q::load_block(w + off, g);  // rows >= 1 and nb >= 1: offset 0 is readable
    };
#pragma unroll
    for (int i = 0; i < kDepth; i++) regs[i] = fetch(grp + i * n_waves, &live[i]);

    token_quantize<kFusedWaves>(xv, nb, wave, lane, s_qs, s_d, s_bsums);
    __syncthreads();
    const uint32_t ab = has_block ? bslot : 0;
    const typename Q::Act a = Q::load_act(s_qs + ab * 256, s_d[ab], s_bsums + ab * 16, g);

    auto reduce = [&](const typename Q::Regs &r, bool ok) {
        row = grp * kRowsPerWave + rsel;
        float acc = ok ? kquant_partial<kQuant>(r, a, g) : 0.0f;
        acc = seg_sum<kLanesPerRow>(acc);
        if (sub == kLanesPerRow - 1 && row < rows) out[static_cast<size_t>(tok) * rows + row] = acc;
    };
    // The register sets take turns: handing the look-ahead row's registers over to "the current row" at the end of an
    // iteration would be a copy, and a copy waits for the loads it copies, so that no request would be in flight while
    // a wave waits
    if constexpr (kDepth == 1) {
        typename Q::Regs other;
        bool other_live;
        while (grp < row_groups) {
            other = fetch(grp + n_waves, &other_live);
            reduce(regs[0], live[0]);
            grp += n_waves;
            if (grp >= row_groups) break;
            regs[0] = fetch(grp + n_waves, &live[0]);
            reduce(other, other_live);
            grp += n_waves;
        }
    } else {
        static_assert(kDepth <= 2, "register sets of the row loop");
        typename Q::Regs third;
        bool third_live;
        while (grp < row_groups) {
            third = fetch(grp + 2 * n_waves, &third_live);
            reduce(regs[0], live[0]);
            grp += n_waves;
            if (grp >= row_groups) break;
            regs[0] = fetch(grp + 2 * n_waves, &live[0]);
            reduce(regs[kDepth - 1], live[kDepth - 1]);
            grp += n_waves;
            if (grp >= row_groups) break;
            regs[kDepth - 1] = fetch(grp + 2 * n_waves, &live[kDepth - 1]);
            reduce(third, third_live);
            grp += n_waves;
        }
    }
}

template <uint32_t kQuant, int kRowsPerWave>
void launch_kquant_f32(const uint8_t *w, const float *x, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                       hipStream_t stream) {
    const uint32_t row_groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
    const uint32_t waves = fused_waves(row_groups);
    const dim3 grid((waves + kFusedWaves - 1) / kFusedWaves, seq, 1);
    hipLaunchKernelGGL((gemv_kquant_f32_kernel<kQuant, kRowsPerWave>), grid, dim3(kWave * kFusedWaves), 0, stream, w, x, out,
                       rows, nb, row_groups);
}

template <uint32_t kQuant>
void launch_kquant_f32_any(const uint8_t *w, const float *x, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                           hipStream_t stream) {
    if (nb <= 4)
        launch_kquant_f32<kQuant, 4>(w, x, out, rows, nb, seq, stream);
    else if (nb <= 8)
        launch_kquant_f32<kQuant, 2>(w, x, out, rows, nb, seq, stream);
    else
        launch_kquant_f32<kQuant, 1>(w, x, out, rows, nb, seq, stream);
}

// ---------------------------------------------------------------------------------------------
// Gated-FFN front half for decode-sized batches: mid[s][r] = act(Wg[r] . a_s) * (Wu[r] . a_s) with one launch (act = SiLU or GELU).  Same lane
// mapping as gemv_kquant_kernel (rows of at most 16 super-blocks); a wave fetches row r of BOTH matrices against the
// one activation slice it holds, so the activation is loaded once and gate/up never travel through memory.
// ---------------------------------------------------------------------------------------------
template <int kRowsPerWave, bool kGelu, int kTokens>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_q4k_gate_up_kernel(const uint8_t *__restrict__ wg, const uint8_t *__restrict__ wu,
                            const int8_t *__restrict__ aq, const float *__restrict__ ad, const int16_t *__restrict__ abs,
                            float *__restrict__ mid, uint32_t rows, uint32_t nb, uint32_t row_groups, uint32_t seq) {
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const bool has_block = bslot < nb;
    const uint32_t tok0 = blockIdx.y * kTokens;  // a group of kTokens tokens per pass over the two matrices
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    Q4KAct a4[kTokens];
#pragma unroll
    for (int t = 0; t < kTokens; t++) {
        const uint32_t tok = tok0 + t < seq ? tok0 + t : seq - 1;  // the last group's spare slots repeat the last token
        const size_t ab = static_cast<size_t>(tok) * nb + (has_block ? bslot : 0);
        a4[t] = q4k_load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
    }
    for (uint32_t grp = wave_global; grp < row_groups; grp += n_waves) {
        const uint32_t row = grp * kRowsPerWave + rsel;
        const bool live = has_block && row < rows;
        const size_t off = live ? static_cast<size_t>(row) * row_bytes + static_cast<size_t>(bslot) * kQ4KBytes : 0;
        const Q4KPrep pg = q4k_prepare(q4k_load_block(wg + off, g), g), pu = q4k_prepare(q4k_load_block(wu + off, g), g);
#pragma unroll
        for (int t = 0; t < kTokens; t++) {
            float gs = live ? q4k_dot(pg, a4[t]) : 0.0f, us = live ? q4k_dot(pu, a4[t]) : 0.0f;
            gs = seg_sum<kLanesPerRow>(gs);
            us = seg_sum<kLanesPerRow>(us);
            if (sub == kLanesPerRow - 1 && row < rows && tok0 + t < seq)
                mid[static_cast<size_t>(tok0 + t) * rows + row] = act_mul<kGelu>(gs, us);
        }
    }
}

template <int kRowsPerWave>
void launch_gate_up(const uint8_t *wg, const uint8_t *wu, ActView act, float *mid, uint32_t rows, uint32_t nb,
                    uint32_t seq, bool gelu, hipStream_t stream) {
    const uint32_t row_groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
    const uint32_t waves = row_groups < kTargetWaves ? row_groups : kTargetWaves;
    // groups of equal size, at most four tokens each
    const auto [groups, per] = token_groups(seq);
    const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, groups, 1);
#define RNB_LAUNCH_GU(GELU, T)                                                                                              \
    hipLaunchKernelGGL((gemv_q4k_gate_up_kernel<kRowsPerWave, GELU, T>), grid, dim3(kWave * kWavesPerWg), 0, stream, wg, wu, \
                       act.qs, act.d, act.bsums, mid, rows, nb, row_groups, seq)
#define RNB_LAUNCH_GU_T(GELU)      \
    do {                           \
        if (per == 1)              \
            RNB_LAUNCH_GU(GELU, 1); \
        else if (per == 2)         \
            RNB_LAUNCH_GU(GELU, 2); \
        else if (per == 3)         \
            RNB_LAUNCH_GU(GELU, 3); \
        else                       \
            RNB_LAUNCH_GU(GELU, 4); \
    } while (0)
    if (gelu)
        RNB_LAUNCH_GU_T(true);
    else
        RNB_LAUNCH_GU_T(false);
#undef RNB_LAUNCH_GU_T
#undef RNB_LAUNCH_GU
}

// The same front half straight from f32 tokens: the workgroup quantises token blockIdx.y to Q8_K in LDS as
// gemv_kquant_f32_kernel does, with the first rows of both matrices already requested.
template <int kRowsPerWave, bool kGelu>
__global__ void __launch_bounds__(kWave *kFusedWaves)
    gemv_q4k_gate_up_f32_kernel(const uint8_t *__restrict__ wg, const uint8_t *__restrict__ wu, const float *__restrict__ x,
                                float *__restrict__ mid, uint32_t rows, uint32_t nb, uint32_t row_groups) {
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    __shared__ __attribute__((aligned(16))) int8_t s_qs[16 * 256];
    __shared__ float s_d[16];
    __shared__ __attribute__((aligned(16))) int16_t s_bsums[16 * 16];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const bool has_block = bslot < nb;
    const uint32_t tok = blockIdx.y;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    const uint32_t n_waves = gridDim.x * kFusedWaves;
    uint32_t grp = blockIdx.x * kFusedWaves + wave;
    TokenSpans<kFusedWaves> xv;
    token_load<kFusedWaves>(x + static_cast<size_t>(tok) * nb * 256, nb, wave, lane, xv);
    auto offset_of = [&](uint32_t group, bool *ok) {
        const uint32_t r = group * kRowsPerWave + rsel;
        *ok = has_block && group < row_groups && r < rows;
        return *ok ? static_cast<size_t>(r) * row_bytes + static_cast<size_t>(bslot) * kQ4KBytes : 0;  // 0 is readable
    };
    bool live, next_live;
    size_t off = offset_of(grp, &live);
    Q4KRegs rg = q4k_load_block(wg + off, g), ru = q4k_load_block(wu + off, g);
    off = offset_of(grp + n_waves, &next_live);
    Q4KRegs ng = q4k_load_block(wg + off, g), nu = q4k_load_block(wu + off, g);

    token_quantize<kFusedWaves>(xv, nb, wave, lane, s_qs, s_d, s_bsums);
    __syncthreads();
    const uint32_t ab = has_block ? bslot : 0;
    const Q4KAct a4 = q4k_load_act(s_qs + ab * 256, s_d[ab], s_bsums + ab * 16, g);

    // Three register sets take turns as current, next and far row group: handing a set's registers on by copy would
    // wait for the loads it copies at the end of every iteration, with nothing in flight meanwhile.  One step requests
    // the group two ahead into the free set and reduces the current one.
    Q4KRegs fg, fu;
    bool far_live;
    auto step = [&](const Q4KRegs &cg, const Q4KRegs &cu, bool clive, Q4KRegs &tg, Q4KRegs &tu, bool &tlive) {
        const uint32_t row = grp * kRowsPerWave + rsel;
        const size_t o = offset_of(grp + 2 * n_waves, &tlive);
        tg = q4k_load_block(wg + o, g);
        tu = q4k_load_block(wu + o, g);
        float gs = clive ? q4k_partial(cg, a4, g) : 0.0f;
        float us = clive ? q4k_partial(cu, a4, g) : 0.0f;
        gs = seg_sum<kLanesPerRow>(gs);
        us = seg_sum<kLanesPerRow>(us);
        if (sub == kLanesPerRow - 1 && row < rows) mid[static_cast<size_t>(tok) * rows + row] = act_mul<kGelu>(gs, us);
        grp += n_waves;
    };
    while (grp < row_groups) {
        step(rg, ru, live, fg, fu, far_live);
        if (grp >= row_groups) break;
        step(ng, nu, next_live, rg, ru, live);
        if (grp >= row_groups) break;
        step(fg, fu, far_live, ng, nu, next_live);
    }
}

template <int kRowsPerWave>
void launch_gate_up_f32(const uint8_t *wg, const uint8_t *wu, const float *x, float *mid, uint32_t rows, uint32_t nb,
                        uint32_t seq, bool gelu, hipStream_t stream) {
    const uint32_t row_groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
    const uint32_t waves = row_groups < kFusedTargetWaves ? row_groups : kFusedTargetWaves;
    const dim3 grid((waves + kFusedWaves - 1) / kFusedWaves, seq, 1);
    if (gelu)
        hipLaunchKernelGGL((gemv_q4k_gate_up_f32_kernel<kRowsPerWave, true>), grid, dim3(kWave * kFusedWaves), 0, stream, wg,
                           wu, x, mid, rows, nb, row_groups);
    else
        hipLaunchKernelGGL((gemv_q4k_gate_up_f32_kernel<kRowsPerWave, false>), grid, dim3(kWave * kFusedWaves), 0, stream, wg,
                           wu, x, mid, rows, nb, row_groups);
}

// ---------------------------------------------------------------------------------------------
// Several Q4_K matrices against ONE quantised activation in one launch (the Q, K and V projections of a decode step:
// crates/rnb-backend/cuda/src/runtime/api/dense_api.rs:916-985): the rows of the matrices are numbered through, a
// lane segment finds its row's matrix by comparing against the running row counts, results go to one contiguous
// vector [rows of matrix 0 | rows of matrix 1 | rows of matrix 2].
// ---------------------------------------------------------------------------------------------
struct MultiMat {
    const uint8_t *w[3];
    uint32_t end[3];  // running row counts: rows of matrices 0..i
};

template <int kRowsPerWave>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_q4k_multi_kernel(MultiMat mats, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                          const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t nb, uint32_t row_groups) {
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    constexpr uint32_t kBlocksPerPass = kLanesPerRow / 4;
    const int lane = threadIdx.x & (kWave - 1);
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    const uint32_t rows = mats.end[2];
    for (uint32_t grp = wave_global; grp < row_groups; grp += n_waves) {
        const uint32_t row = grp * kRowsPerWave + rsel;
        float acc = 0.0f;
        if (row < rows) {
            const int m = row < mats.end[0] ? 0 : (row < mats.end[1] ? 1 : 2);
            const uint32_t local = row - (m == 0 ? 0u : mats.end[m - 1]);
            const uint8_t *rowp = mats.w[m] + static_cast<size_t>(local) * row_bytes;
            for (uint32_t b = bslot; b < nb; b += kBlocksPerPass) {
                const uint8_t *blk = rowp + static_cast<size_t>(b) * kQ4KBytes;
                acc += q4k_partial(q4k_load_block(blk, g), q4k_load_act(aq + static_cast<size_t>(b) * 256, ad[b], abs + b * 16, g), g);
            }
        }
        acc = seg_sum<kLanesPerRow>(acc);
        if (sub == kLanesPerRow - 1 && row < rows) out[row] = acc;
    }
}

template <int kRowsPerWave>
void launch_multi(const MultiMat &mats, ActView act, float *out, uint32_t nb, hipStream_t stream) {
    const uint32_t rows = mats.end[2];
    const uint32_t row_groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
    const uint32_t waves = row_groups < kTargetWaves ? row_groups : kTargetWaves;
    const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, 1, 1);
    hipLaunchKernelGGL((gemv_q4k_multi_kernel<kRowsPerWave>), grid, dim3(kWave * kWavesPerWg), 0, stream, mats, act.qs, act.d,
                       act.bsums, out, nb, row_groups);
}

// The same straight from the f32 token (rows of at most 16 super-blocks): quantised by the workgroup in LDS.
template <int kRowsPerWave>
__global__ void __launch_bounds__(kWave *kFusedWaves)
    gemv_q4k_multi_f32_kernel(MultiMat mats, const float *__restrict__ x, float *__restrict__ out, uint32_t nb,
                              uint32_t row_groups) {
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    __shared__ __attribute__((aligned(16))) int8_t s_qs[16 * 256];
    __shared__ float s_d[16];
    __shared__ __attribute__((aligned(16))) int16_t s_bsums[16 * 16];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const bool has_block = bslot < nb;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    const uint32_t n_waves = gridDim.x * kFusedWaves;
    const uint32_t rows = mats.end[2];
    uint32_t grp = blockIdx.x * kFusedWaves + wave;
    TokenSpans<kFusedWaves> xv;
    token_load<kFusedWaves>(x, nb, wave, lane, xv);
    auto fetch = [&](uint32_t group, bool *ok) {
        const uint32_t r = group * kRowsPerWave + rsel;
        *ok = has_block && group < row_groups && r < rows;
        const int m = r < mats.end[0] ? 0 : (r < mats.end[1] ? 1 : 2);
        const uint32_t local = r - (m == 0 ? 0u : mats.end[m - 1]);
        // a dead lane reads the first block of the first matrix that has rows
        const uint8_t *blk = *ok ? mats.w[m] + static_cast<size_t>(local) * row_bytes + static_cast<size_t>(bslot) * kQ4KBytes
                                 : mats.w[mats.end[0] > 0 ? 0 : (mats.end[1] > mats.end[0] ? 1 : 2)];
        return q4k_load_block(blk, g);
    };
    bool live, next_live;
    Q4KRegs cur = fetch(grp, &live);
    Q4KRegs nxt = fetch(grp + n_waves, &next_live);

    token_quantize<kFusedWaves>(xv, nb, wave, lane, s_qs, s_d, s_bsums);
    __syncthreads();
    const uint32_t ab = has_block ? bslot : 0;
    const Q4KAct a4 = q4k_load_act(s_qs + ab * 256, s_d[ab], s_bsums + ab * 16, g);

    // three register sets in turn (see gemv_q4k_gate_up_f32_kernel): no copies, so no wait for the rows in flight
    Q4KRegs far;
    bool far_live;
    auto step = [&](const Q4KRegs &c, bool clive, Q4KRegs &t, bool &tlive) {
        const uint32_t row = grp * kRowsPerWave + rsel;
        t = fetch(grp + 2 * n_waves, &tlive);
        float acc = clive ? q4k_partial(c, a4, g) : 0.0f;
        acc = seg_sum<kLanesPerRow>(acc);
        if (sub == kLanesPerRow - 1 && row < rows) out[row] = acc;
        grp += n_waves;
    };
    while (grp < row_groups) {
        step(cur, live, far, far_live);
        if (grp >= row_groups) break;
        step(nxt, next_live, cur, live);
        if (grp >= row_groups) break;
        step(far, far_live, nxt, next_live);
    }
}

template <int kRowsPerWave>
void launch_multi_f32(const MultiMat &mats, const float *x, float *out, uint32_t nb, hipStream_t stream) {
    const uint32_t rows = mats.end[2];
    const uint32_t row_groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
    const uint32_t waves = row_groups < kFusedTargetWaves ? row_groups : kFusedTargetWaves;
    const dim3 grid((waves + kFusedWaves - 1) / kFusedWaves, 1, 1);
    hipLaunchKernelGGL((gemv_q4k_multi_f32_kernel<kRowsPerWave>), grid, dim3(kWave * kFusedWaves), 0, stream, mats, x, out, nb,
                       row_groups);
}

template <bool kGelu>
__global__ void __launch_bounds__(256) act_mul_kernel(const float *__restrict__ gate, const float *__restrict__ up,
                                                     float *__restrict__ out, size_t n) {
    for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        out[i] = act_mul<kGelu>(gate[i], up[i]);
}

// ---------------------------------------------------------------------------------------------
// Long rows (more than 16 super-blocks): the K dimension is split across the waves of a workgroup, wave j
// owning super-blocks [16j, 16j+16) of every row, so each lane's activation slice is loaded once and stays
// in registers; the per-wave partial sums of kSplitRows consecutive rows meet in LDS and are added in
// wave order.  A step's blocks are requested at its start and reduced at once: requesting the next step's blocks
// ahead (before or after the barrier) measured 9 - 13 % slower, as did more rows per step.
// ---------------------------------------------------------------------------------------------
constexpr int kSplitRows = 1;  // rows per workgroup and step: 1 / 2 / 4 / 8 measured 11.6 / 12.8 / 13.5 / 33 us on 4096 x 14336 Q6_K
constexpr uint32_t kSplitMaxWaves = 16;  // rows of up to 256 super-blocks

// kDefer: the waves do not meet after every row; the partial sums of up to kSplitBatch of the workgroup's rows wait in
// LDS for one barrier (same additions in the same order, so the same bits).  It pays for two and four waves per workgroup
// (4096 x 14336 Q6_K 11.4 -> 10.7 us, 5120 x 13824 13.4 -> 12.4, 16384 x 6144 18.2 -> 17.0, Q4_K 4096 x 14336 8.4 -> 8.1)
// and costs for three, five and seven (4096 x 11008 9.8 -> 10.1, 4096 x 20480 16.2 -> 17.2, 8192 x 28672 39.4 -> 41.9):
// the launcher chooses.  One row requested ahead on top of it is slower again (10.7 -> 12.7 us).
constexpr int kSplitBatch = 8;

template <uint32_t kQuant, bool kDefer>
__global__ void __launch_bounds__(kWave *kSplitMaxWaves)
    gemv_kquant_splitk_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                              const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                              uint32_t row_chunks) {
    using Q = KQuant<kQuant>;
    using Regs = typename Q::Regs;
    constexpr size_t kBlockBytes = Q::kBytes;
    __shared__ float s_part[kDefer ? kSplitBatch : 2][kSplitRows][kSplitMaxWaves];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6, n_slices = blockDim.x >> 6;
    const int g = lane & 3;
    const uint32_t b = wave * 16 + (lane >> 2);
    const bool has_block = b < nb;
    const uint32_t tok = blockIdx.y;
    const size_t ab = static_cast<size_t>(tok) * nb + (has_block ? b : 0);
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const typename Q::Act a = Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
    if constexpr (kDefer) {
        static_assert(kSplitRows == 1, "one row per step");
        for (uint32_t chunk0 = blockIdx.x; chunk0 < row_chunks; chunk0 += kSplitBatch * gridDim.x) {
            uint32_t n = 0;
            for (uint32_t chunk = chunk0; chunk < row_chunks && n < kSplitBatch; chunk += gridDim.x, n++) {
                Regs r = Regs{};  // idle lanes keep zeros
                if (has_block) r = Q::load_block(w + static_cast<size_t>(chunk) * row_bytes + static_cast<size_t>(b) * kBlockBytes, g);
                float acc = kquant_partial<kQuant>(r, a, g);
                acc = seg_sum<kWave>(has_block ? acc : 0.0f);
                if (lane == kWave - 1) s_part[n][0][wave] = acc;
            }
            __syncthreads();
            if (threadIdx.x < n) {
                float sum = 0.0f;
                for (uint32_t j = 0; j < n_slices; j++) sum += s_part[threadIdx.x][0][j];
                out[static_cast<size_t>(tok) * rows + chunk0 + threadIdx.x * gridDim.x] = sum;
            }
            __syncthreads();  // the sums are read before the next batch overwrites them
        }
        return;
    }
    uint32_t parity = 0;
    for (uint32_t chunk = blockIdx.x; chunk < row_chunks; chunk += gridDim.x, parity ^= 1) {
        const uint32_t row0 = chunk * kSplitRows;
        Regs r[kSplitRows];
#pragma unroll
        for (int i = 0; i < kSplitRows; i++) {
            r[i] = Regs{};  // idle lanes and rows past the end keep zeros
            if (has_block && row0 + i < rows) {
                const uint8_t *blk = w + static_cast<size_t>(row0 + i) * row_bytes + static_cast<size_t>(b) * kBlockBytes;
                r[i] = Q::load_block(blk, g);
            }
        }
#pragma unroll
        for (int i = 0; i < kSplitRows; i++) {
            float acc = kquant_partial<kQuant>(r[i], a, g);
            acc = seg_sum<kWave>(has_block ? acc : 0.0f);
            if (lane == kWave - 1) s_part[parity][i][wave] = acc;
        }
        __syncthreads();  // the other parity's buffer is reused only after the next barrier
        if (threadIdx.x < kSplitRows && row0 + threadIdx.x < rows) {
            float sum = 0.0f;
            for (uint32_t j = 0; j < n_slices; j++) sum += s_part[parity][threadIdx.x][j];
            out[static_cast<size_t>(tok) * rows + row0 + threadIdx.x] = sum;
        }
    }
}

// The split-K GEMV for two to four tokens per pass over the matrix: each wave keeps its K slice of kTokens tokens in
// registers and dots every fetched block against all of them; one barrier per row, partial sums added in wave order
// (per token the same sums in the same order as gemv_kquant_splitk_kernel: same bits).  grid.y = token groups.
template <uint32_t kQuant, int kTokens>
__global__ void __launch_bounds__(kWave *kSplitMaxWaves)
    gemv_kquant_splitk_tokens_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                     const int16_t *__restrict__ abs, float *__restrict__ out, uint32_t rows, uint32_t nb,
                                     uint32_t seq) {
    using Q = KQuant<kQuant>;
    using Regs = typename Q::Regs;
    constexpr size_t kBlockBytes = Q::kBytes;
    __shared__ float s_part[2][kTokens][kSplitMaxWaves];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6, n_slices = blockDim.x >> 6;
    const int g = lane & 3;
    const uint32_t b = wave * 16 + (lane >> 2);
    const bool has_block = b < nb;
    const uint32_t tok0 = blockIdx.y * kTokens;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    typename Q::Act a[kTokens];
#pragma unroll
    for (int t = 0; t < kTokens; t++) {
        const uint32_t tok = tok0 + t < seq ? tok0 + t : seq - 1;
        const size_t ab = static_cast<size_t>(tok) * nb + (has_block ? b : 0);
        a[t] = Q::load_act(aq + ab * 256, ad[ab], abs + ab * 16, g);
    }
    uint32_t parity = 0;
    for (uint32_t row = blockIdx.x; row < rows; row += gridDim.x, parity ^= 1) {
        Regs r = Regs{};  // idle lanes keep zeros
        if (has_block) r = Q::load_block(w + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b) * kBlockBytes, g);
        const typename Q::Prep p = Q::prepare(r, g);
#pragma unroll
        for (int t = 0; t < kTokens; t++) {
            float acc = Q::dot(p, a[t]);
            acc = seg_sum<kWave>(has_block ? acc : 0.0f);
            if (lane == kWave - 1) s_part[parity][t][wave] = acc;
        }
        __syncthreads();  // the other parity's buffer is reused only after the next barrier
        if (threadIdx.x < kTokens && tok0 + threadIdx.x < seq) {
            float sum = 0.0f;
            for (uint32_t j = 0; j < n_slices; j++) sum += s_part[parity][threadIdx.x][j];
            out[static_cast<size_t>(tok0 + threadIdx.x) * rows + row] = sum;
        }
    }
}

template <uint32_t kQuant>
void launch_kquant_splitk(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                          hipStream_t stream) {
    const uint32_t n_slices = (nb + 15) / 16;
    const uint32_t row_chunks = (rows + kSplitRows - 1) / kSplitRows;
    const uint32_t want = kTargetWaves / n_slices;  // workgroups for about kTargetWaves waves
    if (seq >= 2) {  // several tokens per pass over the matrix, in groups of equal size (at most four)
        const auto [groups, per] = token_groups(seq);
        const dim3 tgrid(rows < want ? rows : want, groups, 1);
#define RNB_LAUNCH_TOKENS(T)                                                                                                  \
    hipLaunchKernelGGL((gemv_kquant_splitk_tokens_kernel<kQuant, T>), tgrid, dim3(kWave * n_slices), 0, stream, w, act.qs, act.d, \
                       act.bsums, out, rows, nb, seq)
        if (per == 2)
            RNB_LAUNCH_TOKENS(2);
        else if (per == 3)
            RNB_LAUNCH_TOKENS(3);
        else
            RNB_LAUNCH_TOKENS(4);
#undef RNB_LAUNCH_TOKENS
        return;
    }
    const dim3 grid(row_chunks < want ? row_chunks : want, seq, 1);
    if (n_slices == 2 || n_slices == 4)
        hipLaunchKernelGGL((gemv_kquant_splitk_kernel<kQuant, true>), grid, dim3(kWave * n_slices), 0, stream, w, act.qs, act.d,
                           act.bsums, out, rows, nb, row_chunks);
    else
        hipLaunchKernelGGL((gemv_kquant_splitk_kernel<kQuant, false>), grid, dim3(kWave * n_slices), 0, stream, w, act.qs, act.d,
                           act.bsums, out, rows, nb, row_chunks);
}

// ---------------------------------------------------------------------------------------------
// Split-K GEMV of ONE f32 token in one launch, rows of 17 to 64 super-blocks: a workgroup of 16 waves quantises the whole
// token to Q8_K in its LDS (kSlices blocks per wave, the wave-level quantiser of the stand-alone kernel, so the same bits),
// then works as `teams` split-K teams of kSlices waves, each team on rows of its own; the partial sums of up to
// kSplitBatch rows per team wait for one barrier and are added in slice order, as in gemv_kquant_splitk_kernel (the same
// bits).  The teams of a launch are as many as the split-K kernel has workgroups, so the weight stream looks the same;
// the token is read once per 16 waves, and the quantiser's launch and the gap behind it go.
//
// Two register sets take turns over ALL of a wave's rows: the first is requested before the token is quantised, the
// second right behind the quantisation (in front of the barrier), and each again as soon as its row is reduced, also
// across the batches' barriers.  Steps measured against quantiser + split-K GEMV in two launches (us): 4096 x 14336 Q6_K
// 11.2 vs 13.3, Q4_K 9.3 vs 10.8, 4096 x 11008 Q4_K 8.2 vs 10.1, 8192 x 8192 Q4_K 8.45 vs 10.9, Q6_K 11.9 vs 14.1,
// 13824 x 5120 Q4_K 9.8 vs 12.3, 28672 x 8192 Q4_K 23.8 vs 25.7.  What it took, in the order found:
//  * a loop that waited for every row before requesting the next lost to the two launches from three slices on
//    (4096 x 11008 16.0 vs 12.0 us); with the next row of a batch requested ahead: 9.15;
//  * that loop started its two sets anew after the early rows and after every batch, with nothing in flight in between,
//    and needed TWO early rows with four slices to win (13.0 us on 4096 x 14336 Q6_K; three spill); as one pipeline over
//    all rows ONE early row is best everywhere (11.2 us; two: 12.5; none: 12.9);
//  * requests that only some paths make (the last rows, a second set when there is a second pass) cost every path a full
//    wait, because the compiler's wait counts follow the issue order of the worst path: the steady-state loop requests
//    unconditionally, and the last one to three rows are code of their own;
//  * the Q6_K loader without its odd-address path (load_block_even; the launcher sends such matrices to the two
//    launches): with it the compiler merged both paths into single-dword loads and grouped them again as 1 + 3 dwords
//    for one piece, copied into place (and waited for) where the set is assigned, i.e. in front of the barrier.
// The slice count is a template parameter: with two slices the blocks past the end of the token are quantised as
// zeros rather than branched around, which lets the compiler interleave the two chains of max, division and rounding
// (Q6_K 5120 x 5120 8.84 -> 8.45 us); with three or four that loses 1.5 % and the branches stay.
// ---------------------------------------------------------------------------------------------
constexpr int kWideWaves = 16;
constexpr uint32_t kWideMaxBlocks = 64;
template <uint32_t kQuant, uint32_t kSlices>
__global__ void __launch_bounds__(kWave *kWideWaves)
    gemv_kquant_wide_f32_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out,
                                uint32_t rows, uint32_t nb) {
    using Q = KQuant<kQuant>;
    using Regs = typename Q::Regs;
    constexpr size_t kBlockBytes = Q::kBytes;
    constexpr uint32_t n_slices = kSlices, teams = kWideWaves / kSlices;
    constexpr uint32_t kBlocks = kSlices * 16;  // LDS image of the token: blocks past nb are quantised zeros
    __shared__ __attribute__((aligned(16))) int8_t s_qs[kBlocks * 256];
    __shared__ float s_d[kBlocks];
    __shared__ __attribute__((aligned(16))) int16_t s_bsums[kBlocks * 16];
    __shared__ float s_part[kSplitBatch][kWideWaves];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t team = wave / n_slices, slice = wave - team * n_slices;
    const int g = lane & 3;
    const uint32_t b = slice * 16 + (lane >> 2);
    const bool has_block = team < teams && b < nb;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint32_t stride = gridDim.x * teams;          // rows per pass of the whole launch
    const uint32_t first = blockIdx.x * teams;          // this workgroup's first row of pass 0
    const uint32_t n_pass = (rows + stride - 1) / stride;
    // the token is requested first: loads return in order, and the quantiser must not wait for weights
    float4 xv[kSlices];
#pragma unroll
    for (uint32_t i = 0; i < kSlices; i++) {
        const uint32_t blk = wave + i * kWideWaves;
        xv[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (blk < nb) xv[i] = reinterpret_cast<const float4 *>(x + static_cast<size_t>(blk) * 256)[lane];
    }
    // (idle lanes and rows past the end read a valid block; their sums are masked out below)
    const size_t lane_off = static_cast<size_t>(has_block ? b : 0) * kBlockBytes;
    auto row_of = [&](uint32_t pass) { return pass * stride + first + team; };
    auto fetch = [&](uint32_t pass) {
        const uint32_t row = row_of(pass);
        return Q::load_block_even(w + static_cast<size_t>(row < rows ? row : 0) * row_bytes + lane_off, g);
    };
    // two register sets in turn (a copy from a "next" set to a "current" one would wait for the loads it copies)
    Regs s0 = fetch(0), s1;
    // with two slices every wave quantises both of its blocks, whether they exist or not (zeros past nb)
#pragma unroll
    for (uint32_t i = 0; i < kSlices; i++) {
        const uint32_t blk = wave + i * kWideWaves;
        if (kSlices == 2 || blk < nb) q8k_quantize_vals(xv[i], lane, s_qs + blk * 256, s_d + blk, s_bsums + blk * 16);
    }
    // (with a single pass the second set fetches the first row again: a request that only some launches make would
    // cost all of them a full wait in front of the first row, see below)
    s1 = fetch(1 < n_pass ? 1 : 0);
    __syncthreads();
    const uint32_t ab = has_block ? b : 0;
    const typename Q::Act a = Q::load_act(s_qs + ab * 256, s_d[ab], s_bsums + ab * 16, g);
    auto partial = [&](const Regs &r, uint32_t pass) {
        float acc = kquant_partial<kQuant>(r, a, g);
        acc = seg_sum<kWave>(has_block && row_of(pass) < rows ? acc : 0.0f);
        if (lane == kWave - 1) s_part[pass % kSplitBatch][wave] = acc;
    };
    // the batch that ends with pass `last`: slice sums added in slice order, one thread per row
    auto flush = [&](uint32_t last) {
        __syncthreads();
        const uint32_t p0 = last - last % kSplitBatch, n = last - p0 + 1;
        if (threadIdx.x < n * teams) {
            const uint32_t k = threadIdx.x / teams, tm = threadIdx.x - k * teams;
            const uint32_t row = (p0 + k) * stride + first + tm;
            if (row < rows) {
                float sum = 0.0f;
                for (uint32_t j = 0; j < n_slices; j++) sum += s_part[k][tm * n_slices + j];
                out[row] = sum;
            }
        }
        __syncthreads();  // the sums are read before the next batch overwrites them
    };
    static_assert(kSplitBatch % 2 == 0, "a batch ends behind the second register set");
    // While both sets have a row left to request, the requests are unconditional: the waits the compiler places count
    // requests in issue order, and a request that only one path makes costs every path a full wait.
    uint32_t pass = 0;
    for (; pass + 3 < n_pass; pass += 2) {
        partial(s0, pass);
        s0 = fetch(pass + 2);
        partial(s1, pass + 1);
        s1 = fetch(pass + 3);
        if ((pass + 1) % kSplitBatch == kSplitBatch - 1) flush(pass + 1);
    }
    // one to three passes are left: s0 holds the first of them, s1 the second
    if (n_pass - pass == 3) {
        partial(s0, pass);
        s0 = fetch(pass + 2);
        partial(s1, pass + 1);
        if ((pass + 1) % kSplitBatch == kSplitBatch - 1) flush(pass + 1);
        partial(s0, pass + 2);
    } else {
        partial(s0, pass);
        if (n_pass - pass == 2) partial(s1, pass + 1);
    }
    flush(n_pass - 1);
}

template <uint32_t kQuant>
void launch_kquant_wide_f32(const uint8_t *w, const float *x, float *out, uint32_t rows, uint32_t nb, hipStream_t stream) {
    const uint32_t n_slices = (nb + 15) / 16;
    const uint32_t teams = kWideWaves / n_slices;
    // one workgroup of sixteen waves per compute unit's share of kTargetWaves
    const uint32_t want = kTargetWaves / kWideWaves;
    const uint32_t all = (rows + teams - 1) / teams;
    const dim3 grid(all < want ? all : want), block(kWave * kWideWaves);
#define RNB_LAUNCH_WIDE(S) \
    hipLaunchKernelGGL((gemv_kquant_wide_f32_kernel<kQuant, S>), grid, block, 0, stream, w, x, out, rows, nb)
    if (n_slices == 2)
        RNB_LAUNCH_WIDE(2);
    else if (n_slices == 3)
        RNB_LAUNCH_WIDE(3);
    else
        RNB_LAUNCH_WIDE(4);
#undef RNB_LAUNCH_WIDE
}

template <uint32_t kQuant, int kRowsPerWave>
void launch_kquant(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                   hipStream_t stream) {
    const uint32_t row_groups = (rows + kRowsPerWave - 1) / kRowsPerWave;
    const uint32_t waves = row_groups < kTargetWaves ? row_groups : kTargetWaves;
    // several tokens per pass over the matrix, in groups of equal size (at most four); rows longer than one wave pass
    // (only reached beyond the K-split kernel's 256 super-blocks) keep one pass per token
    if (seq >= 2 && nb <= static_cast<uint32_t>(kWave / kRowsPerWave / 4)) {
        const auto [groups, per] = token_groups(seq);
        const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, groups, 1);
#define RNB_LAUNCH_TOKENS(T)                                                                                                 \
    hipLaunchKernelGGL((gemv_kquant_tokens_kernel<kQuant, kRowsPerWave, T>), grid, dim3(kWave * kWavesPerWg), 0, stream, w, \
                       act.qs, act.d, act.bsums, out, rows, nb, row_groups, seq)
        if (per == 2)
            RNB_LAUNCH_TOKENS(2);
        else if (per == 3)
            RNB_LAUNCH_TOKENS(3);
        else
            RNB_LAUNCH_TOKENS(4);
#undef RNB_LAUNCH_TOKENS
        return;
    }
    const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, seq, 1);
    hipLaunchKernelGGL((gemv_kquant_kernel<kQuant, kRowsPerWave>), grid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs,
                       act.d, act.bsums, out, rows, nb, row_groups);
}

// one wave per chunk of kRows rows (at most kChunkMaxWaves waves; beyond that the waves loop)
constexpr uint32_t kChunkMaxWaves = 1u << 20;
template <uint32_t kQuant, int kRows>
void launch_kquant_chunks(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                          hipStream_t stream) {
    const uint32_t n_chunks = (rows + kRows - 1) / kRows;
    const uint32_t waves = n_chunks < kChunkMaxWaves ? n_chunks : kChunkMaxWaves;
    if (seq >= 2) {  // several tokens per pass over the matrix, in groups of equal size (at most four)
        const auto [groups, per] = token_groups(seq);
        const dim3 tgrid((waves + kWavesPerWg - 1) / kWavesPerWg, groups, 1);
#define RNB_LAUNCH_TOKENS(T)                                                                                                  \
    hipLaunchKernelGGL((gemv_kquant_chunks_tokens_kernel<kQuant, kRows, T>), tgrid, dim3(kWave * kWavesPerWg), 0, stream, w,  \
                       act.qs, act.d, act.bsums, out, rows, nb, n_chunks, seq)
        if (per == 2)
            RNB_LAUNCH_TOKENS(2);
        else if (per == 3)
            RNB_LAUNCH_TOKENS(3);
        else
            RNB_LAUNCH_TOKENS(4);
#undef RNB_LAUNCH_TOKENS
        return;
    }
    const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, seq, 1);
    hipLaunchKernelGGL((gemv_kquant_chunks_kernel<kQuant, kRows>), grid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs,
                       act.d, act.bsums, out, rows, nb, n_chunks);
}

template <uint32_t kQuant>
void launch_kquant_any(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                       hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    if (nb > 8 && nb <= 16 && static_cast<uint64_t>(rows) * nb * KQuant<kQuant>::kBytes >= kGemvChunkMinBytes) {
        // Q6_K measured best with four rows per wave (431 MB: 71.7 against 77.0 us with two), Q4_K with two
        if (kQuant == kQ6K)
            launch_kquant_chunks<kQuant, 4>(w, act, out, rows, nb, seq, stream);
        else
            launch_kquant_chunks<kQuant, 2>(w, act, out, rows, nb, seq, stream);
    } else if (nb > 16 && nb <= 16 * kSplitMaxWaves)
        launch_kquant_splitk<kQuant>(w, act, out, rows, nb, seq, stream);
    else if (nb <= 4)
        launch_kquant<kQuant, 4>(w, act, out, rows, nb, seq, stream);
    else if (nb <= 8)
        launch_kquant<kQuant, 2>(w, act, out, rows, nb, seq, stream);
    else
        launch_kquant<kQuant, 1>(w, act, out, rows, nb, seq, stream);
}

// ---------------------------------------------------------------------------------------------
// The 32-element formats against 32-wide Q8 activations, one lane per block (blocks are 2-byte aligned: 16-byte loads
// at 2-byte alignment).  Rows of up to 128 blocks (K <= 4096) keep the lane's two activation blocks in registers.
//   Q8_0 {f16 d, i8 qs[32]}                 (d * d_x) * sum(w * q)                   neon_dot.rs:376-436
//   Q4_0 {f16 d, qs[16]}                    (d * d_x) * sum((code - 8) * q)          neon_dot.rs:83-137
//   Q5_0 {f16 d, u32 qh, qs[16]}            (d * d_x) * sum((code - 16) * q)         neon_dot.rs:163-214
//   Q4_1 {f16 d, f16 m, qs[16]}             d_x * (d * sum(code * q) + m * sum(q))   neon_quant.rs:88-108
//   Q5_1 {f16 d, f16 m, u32 qh, qs[16]}     likewise                                 neon_quant.rs:130-158
//   Q8_1 {f16 d, f16 s, i8 qs[32]}          (d * d_x) * sum(w * q), s is not read      neon_quant.rs:236-253
// (all under crates/rnb-cpu/src/gemm/).  Element i < 16 is the low nibble of qs[i], element 16 + i the high nibble; the
// fifth bit of element e is bit e of qh.  (code - offset) is applied as dot(code, q) - offset * sum(q).
// ---------------------------------------------------------------------------------------------
struct Q8Act {
    uint4 a0, a1;
    float dx;
    int sum;  // of the 32 activations (unused by Q8_0)
};

template <bool kWithSum>
__device__ __forceinline__ Q8Act q8_load_act(const int8_t *__restrict__ aq_blk, float dx) {
    Q8Act a;
    a.a0 = *reinterpret_cast<const uint4 *>(aq_blk);
    a.a1 = *reinterpret_cast<const uint4 *>(aq_blk + 16);
    a.dx = dx;
    a.sum = 0;
    if constexpr (kWithSum) {
        int s = 0;
        s = dot4(0x01010101u, a.a0.x, s);
        s = dot4(0x01010101u, a.a0.y, s);
        s = dot4(0x01010101u, a.a0.z, s);
        s = dot4(0x01010101u, a.a0.w, s);
        s = dot4(0x01010101u, a.a1.x, s);
        s = dot4(0x01010101u, a.a1.y, s);
        s = dot4(0x01010101u, a.a1.z, s);
        s = dot4(0x01010101u, a.a1.w, s);
        a.sum = s;
    }
    return a;
}

struct Block32Layout {
    int bytes, qs, qh, offset;  // block size, offsets of qs and qh (qh < 0: no fifth bit), code offset
    bool min;                   // f16 m follows d
};
template <uint32_t kQuant>
constexpr Block32Layout block32_layout() {
    switch (kQuant) {
    case kQ4_0: return {static_cast<int>(kQ4_0Bytes), 2, -1, 8, false};
    case kQ4_1: return {static_cast<int>(kQ4_1Bytes), 4, -1, 0, true};
    case kQ5_0: return {static_cast<int>(kQ5_0Bytes), 6, 2, 16, false};
    case kQ5_1: return {static_cast<int>(kQ5_1Bytes), 8, 4, 0, true};
    case kQ8_1: return {static_cast<int>(kQ8_1Bytes), 4, -1, 0, false};
    default: return {static_cast<int>(kQ8_0Bytes), 2, -1, 0, false};
    }
}

// four bits -> bit 4 of four bytes (bit j of x lands in byte j)
__device__ __forceinline__ uint32_t spread_fifth_bits(uint32_t x) {
    return ((__umul24(x & 15u, 0x00204081u)) & 0x01010101u) << 4;
}

// one weight block in registers: loads and arithmetic are separate calls so that a kernel can request a block early
struct Block32Regs {
    uint4 q0, q1;  // Q8_0: the 32 codes; others: q0 = the 16 bytes of nibbles
    uint32_t qh;
    float d, m;
};
template <uint32_t kQuant>
__device__ __forceinline__ Block32Regs block32_load(const uint8_t *__restrict__ blk) {
    constexpr Block32Layout F = block32_layout<kQuant>();
    Block32Regs r;
    r.d = ld_f16(blk);
    r.m = 0.0f;
    r.qh = 0;
    r.q1 = make_uint4(0, 0, 0, 0);
    if constexpr (kQuant == kQ8_0 || kQuant == kQ8_1) {  // whole-byte codes
        r.q0 = ld_u4_a2(blk + F.qs);
        r.q1 = ld_u4_a2(blk + F.qs + 16);
    } else {
        r.q0 = ld_u4_a2(blk + F.qs);
        if constexpr (F.qh >= 0) r.qh = ld_u32_a2(blk + F.qh);
        if constexpr (F.min) r.m = ld_f16(blk + 2);
    }
    return r;
}
// Blocks of 18, 22 and 34 bytes (Q4_0, Q5_0, Q8_0) start on 2 mod 4 every other time, and a 16-byte load whose address
// is not a multiple of 4 runs at about two thirds of the rate of one that is (measured on 4096 x 4096: Q8_0 6.2 us
// against 5.3 us for the 36-byte Q8_1 blocks, which carry more bytes).  Two consecutive blocks are 36, 44 or 68 bytes:
// a pair that starts on a 4-byte boundary is fetched as whole dwords and the first block's fields, which sit two
// bytes into their dwords, are put together with funnel shifts; the second block's fields are dwords as loaded.
template <uint32_t kQuant>
constexpr bool block32_pairs() {
    return kQuant == kQ8_0 || kQuant == kQ4_0 || kQuant == kQ5_0;
}
__device__ __forceinline__ uint32_t mid32(uint32_t hi, uint32_t lo) { return __builtin_amdgcn_alignbit(hi, lo, 16); }
template <uint32_t kQuant>
__device__ __forceinline__ void block32_load_pair(const uint8_t *__restrict__ pair, Block32Regs &a, Block32Regs &b) {
    static_assert(block32_pairs<kQuant>(), "formats whose blocks are 2 mod 4 bytes");
    a.m = b.m = 0.0f;
    a.qh = b.qh = 0;
    a.q1 = b.q1 = make_uint4(0, 0, 0, 0);
    const uint4 d0 = *reinterpret_cast<const uint4_a4 *>(pair), d1 = *reinterpret_cast<const uint4_a4 *>(pair + 16);
    if constexpr (kQuant == kQ8_0) {  // {d, 32 codes} {d, 32 codes}: dwords 0..16
        const uint4 d2 = *reinterpret_cast<const uint4_a4 *>(pair + 32), d3 = *reinterpret_cast<const uint4_a4 *>(pair + 48);
        const uint32_t d4 = *reinterpret_cast<const uint32_t *>(pair + 64);
        a.d = f16_bits_to_f32(d0.x);
        a.q0 = make_uint4(mid32(d0.y, d0.x), mid32(d0.z, d0.y), mid32(d0.w, d0.z), mid32(d1.x, d0.w));
        a.q1 = make_uint4(mid32(d1.y, d1.x), mid32(d1.z, d1.y), mid32(d1.w, d1.z), mid32(d2.x, d1.w));
        b.d = f16_bits_to_f32(d2.x >> 16);
        b.q0 = make_uint4(d2.y, d2.z, d2.w, d3.x);
        b.q1 = make_uint4(d3.y, d3.z, d3.w, d4);
    } else if constexpr (kQuant == kQ4_0) {  // {d, 16 bytes of nibbles} twice: dwords 0..8
        const uint32_t d2 = *reinterpret_cast<const uint32_t *>(pair + 32);
        a.d = f16_bits_to_f32(d0.x);
        a.q0 = make_uint4(mid32(d0.y, d0.x), mid32(d0.z, d0.y), mid32(d0.w, d0.z), mid32(d1.x, d0.w));
        b.d = f16_bits_to_f32(d1.x >> 16);
        b.q0 = make_uint4(d1.y, d1.z, d1.w, d2);
    } else {  // Q5_0 {d, qh, 16 bytes of nibbles} twice: dwords 0..10
        const uint2 d2 = *reinterpret_cast<const uint2_a4 *>(pair + 32);
        const uint32_t d3 = *reinterpret_cast<const uint32_t *>(pair + 40);
        a.d = f16_bits_to_f32(d0.x);
        a.qh = mid32(d0.y, d0.x);
        a.q0 = make_uint4(mid32(d0.z, d0.y), mid32(d0.w, d0.z), mid32(d1.x, d0.w), mid32(d1.y, d1.x));
        b.d = f16_bits_to_f32(d1.y >> 16);
        b.qh = d1.z;
        b.q0 = make_uint4(d1.w, d2.x, d2.y, d3);
    }
}
template <uint32_t kQuant>
__device__ __forceinline__ float block32_dot(const Block32Regs &r, const Q8Act &a) {
    constexpr Block32Layout F = block32_layout<kQuant>();
    if constexpr (kQuant == kQ8_0 || kQuant == kQ8_1) {
        int p = 0;
        p = dot4(r.q0.x, a.a0.x, p);
        p = dot4(r.q0.y, a.a0.y, p);
        p = dot4(r.q0.z, a.a0.z, p);
        p = dot4(r.q0.w, a.a0.w, p);
        p = dot4(r.q1.x, a.a1.x, p);
        p = dot4(r.q1.y, a.a1.y, p);
        p = dot4(r.q1.z, a.a1.z, p);
        p = dot4(r.q1.w, a.a1.w, p);
        return (r.d * a.dx) * static_cast<float>(p);
    } else {
        const uint4 qs = r.q0;
        uint4 lo = make_uint4(qs.x & 0x0f0f0f0fu, qs.y & 0x0f0f0f0fu, qs.z & 0x0f0f0f0fu, qs.w & 0x0f0f0f0fu);
        uint4 hi = make_uint4((qs.x >> 4) & 0x0f0f0f0fu, (qs.y >> 4) & 0x0f0f0f0fu, (qs.z >> 4) & 0x0f0f0f0fu,
                              (qs.w >> 4) & 0x0f0f0f0fu);
        if constexpr (F.qh >= 0) {
            const uint32_t qh = r.qh;
            lo.x |= spread_fifth_bits(qh);
            lo.y |= spread_fifth_bits(qh >> 4);
            lo.z |= spread_fifth_bits(qh >> 8);
            lo.w |= spread_fifth_bits(qh >> 12);
            hi.x |= spread_fifth_bits(qh >> 16);
            hi.y |= spread_fifth_bits(qh >> 20);
            hi.z |= spread_fifth_bits(qh >> 24);
            hi.w |= spread_fifth_bits(qh >> 28);
        }
        int p = 0;
        p = dot4(lo.x, a.a0.x, p);
        p = dot4(lo.y, a.a0.y, p);
        p = dot4(lo.z, a.a0.z, p);
        p = dot4(lo.w, a.a0.w, p);
        p = dot4(hi.x, a.a1.x, p);
        p = dot4(hi.y, a.a1.y, p);
        p = dot4(hi.z, a.a1.z, p);
        p = dot4(hi.w, a.a1.w, p);
        if constexpr (F.min) {
            return a.dx * (r.d * static_cast<float>(p) + r.m * static_cast<float>(a.sum));
        } else {
            return (r.d * a.dx) * static_cast<float>(p - F.offset * a.sum);
        }
    }
}
template <uint32_t kQuant>
__device__ __forceinline__ float block32_partial(const uint8_t *__restrict__ blk, const Q8Act &a) {
    return block32_dot<kQuant>(block32_load<kQuant>(blk), a);
}

// kPaired (an even number of blocks per row, formats of block32_pairs): a lane takes blocks 2 l and 2 l + 1 of the row
// through block32_load_pair instead of blocks l and l + 64.
template <uint32_t kQuant, bool kPaired>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_block32_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                        float *__restrict__ out, uint32_t rows, uint32_t nb32) {
    constexpr size_t kBlockBytes = block32_layout<kQuant>().bytes;
    constexpr bool kSum = kQuant != kQ8_0 && kQuant != kQ8_1;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t tok = blockIdx.y;
    const size_t abase = static_cast<size_t>(tok) * nb32;
    const size_t row_bytes = static_cast<size_t>(nb32) * kBlockBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    if constexpr (kPaired) {
        const uint32_t n_pairs = nb32 / 2;
        if (n_pairs <= kWave) {
            const bool has = static_cast<uint32_t>(lane) < n_pairs;
            const uint32_t b0 = has ? 2 * lane : 0;
            const Q8Act a0 = q8_load_act<kSum>(aq + (abase + b0) * 32, ad[abase + b0]);
            const Q8Act a1 = q8_load_act<kSum>(aq + (abase + b0 + 1) * 32, ad[abase + b0 + 1]);
            for (uint32_t row = wave_global; row < rows; row += n_waves) {
                float acc = 0.0f;
                if (has) {
                    Block32Regs c0, c1;
                    block32_load_pair<kQuant>(w + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b0) * kBlockBytes, c0, c1);
                    acc = block32_dot<kQuant>(c0, a0) + block32_dot<kQuant>(c1, a1);
                }
                acc = seg_sum<kWave>(acc);
                if (lane == kWave - 1) out[static_cast<size_t>(tok) * rows + row] = acc;
            }
        } else {
            for (uint32_t row = wave_global; row < rows; row += n_waves) {
                const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
                float acc = 0.0f;
                for (uint32_t b = 2 * lane; b < nb32; b += 2 * kWave) {
                    Block32Regs c0, c1;
                    block32_load_pair<kQuant>(rowp + static_cast<size_t>(b) * kBlockBytes, c0, c1);
                    acc += block32_dot<kQuant>(c0, q8_load_act<kSum>(aq + (abase + b) * 32, ad[abase + b]));
                    acc += block32_dot<kQuant>(c1, q8_load_act<kSum>(aq + (abase + b + 1) * 32, ad[abase + b + 1]));
                }
                acc = seg_sum<kWave>(acc);
                if (lane == kWave - 1) out[static_cast<size_t>(tok) * rows + row] = acc;
            }
        }
        return;
    }
    if (nb32 <= 2 * kWave) {
        const uint32_t b0 = lane, b1 = lane + kWave;
        const bool has0 = b0 < nb32, has1 = b1 < nb32;
        const Q8Act a0 = q8_load_act<kSum>(aq + (abase + (has0 ? b0 : 0)) * 32, ad[abase + (has0 ? b0 : 0)]);
        const Q8Act a1 = q8_load_act<kSum>(aq + (abase + (has1 ? b1 : 0)) * 32, ad[abase + (has1 ? b1 : 0)]);
        for (uint32_t row = wave_global; row < rows; row += n_waves) {
            const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
            float acc = 0.0f;
            if (has0) acc = block32_partial<kQuant>(rowp + static_cast<size_t>(b0) * kBlockBytes, a0);
            if (has1) acc += block32_partial<kQuant>(rowp + static_cast<size_t>(b1) * kBlockBytes, a1);
            acc = seg_sum<kWave>(acc);
            if (lane == kWave - 1) out[static_cast<size_t>(tok) * rows + row] = acc;
        }
    } else {
        for (uint32_t row = wave_global; row < rows; row += n_waves) {
            const uint8_t *rowp = w + static_cast<size_t>(row) * row_bytes;
            float acc = 0.0f;
            for (uint32_t b = lane; b < nb32; b += kWave)
                acc += block32_partial<kQuant>(rowp + static_cast<size_t>(b) * kBlockBytes,
                                               q8_load_act<kSum>(aq + (abase + b) * 32, ad[abase + b]));
            acc = seg_sum<kWave>(acc);
            if (lane == kWave - 1) out[static_cast<size_t>(tok) * rows + row] = acc;
        }
    }
}

// Two to four tokens per pass over the matrix, rows of at most 128 blocks (the register-resident branches of
// gemv_block32_kernel): a lane keeps its two activation blocks of kTokens tokens and dots each fetched weight block
// against all of them; per token the same expression as the one-token kernel (same bits).  grid.y = token groups.
// grid.z = heads (1 for a plain matrix): head z has its own `rows` rows of weights, reads activation row tok * heads + z
// and writes out[tok][z * rows + row], the per-head projections of q8_0_head_gemv_batch.
// kRows rows side by side in a wave (1, 4 or 16; a row's blocks must fit its 64 / kRows lanes): short rows, as the per-head
// projections have, would leave most of a wave idle otherwise; a row's sum keeps the bits of the one-row-per-wave form.
template <uint32_t kQuant, bool kPaired, int kTokens, int kRows = 1>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    gemv_block32_tokens_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                               float *__restrict__ out, uint32_t rows, uint32_t nb32, uint32_t seq) {
    constexpr size_t kBlockBytes = block32_layout<kQuant>().bytes;
    constexpr bool kSum = kQuant != kQ8_0 && kQuant != kQ8_1;
    const int lane = threadIdx.x & (kWave - 1);
    constexpr int kLanesPerRow = kWave / kRows;
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const uint32_t tok0 = blockIdx.y * kTokens, heads = gridDim.z, head = blockIdx.z;
    const size_t row_bytes = static_cast<size_t>(nb32) * kBlockBytes;
    const uint32_t wave_global = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t n_waves = gridDim.x * kWavesPerWg;
    const uint32_t b0 = kPaired ? 2 * sub : sub, b1 = kPaired ? 2 * sub + 1 : sub + kLanesPerRow;
    const bool has0 = b0 < nb32, has1 = b1 < nb32;  // kPaired: nb32 is even, a pair is there or not as a whole
    Q8Act a0[kTokens], a1[kTokens];
#pragma unroll
    for (int t = 0; t < kTokens; t++) {
        const uint32_t tok = tok0 + t < seq ? tok0 + t : seq - 1;
        const size_t abase = (static_cast<size_t>(tok) * heads + head) * nb32;
        a0[t] = q8_load_act<kSum>(aq + (abase + (has0 ? b0 : 0)) * 32, ad[abase + (has0 ? b0 : 0)]);
        a1[t] = q8_load_act<kSum>(aq + (abase + (has1 ? b1 : 0)) * 32, ad[abase + (has1 ? b1 : 0)]);
    }
    for (uint32_t grp = wave_global; grp * kRows < rows; grp += n_waves) {
        const uint32_t row = grp * kRows + rsel;
        const bool live0 = has0 && row < rows, live1 = has1 && row < rows;
        const uint8_t *rowp = w + (static_cast<size_t>(head) * rows + (row < rows ? row : 0)) * row_bytes;
        Block32Regs c0 = Block32Regs{}, c1 = Block32Regs{};
        if constexpr (kPaired) {
            if (live0) block32_load_pair<kQuant>(rowp + static_cast<size_t>(b0) * kBlockBytes, c0, c1);
        } else {
            if (live0) c0 = block32_load<kQuant>(rowp + static_cast<size_t>(b0) * kBlockBytes);
            if (live1) c1 = block32_load<kQuant>(rowp + static_cast<size_t>(b1) * kBlockBytes);
        }
#pragma unroll
        for (int t = 0; t < kTokens; t++) {
            float acc = 0.0f;
            if constexpr (kPaired) {
                if (live0) acc = block32_dot<kQuant>(c0, a0[t]) + block32_dot<kQuant>(c1, a1[t]);
            } else {
                if (live0) acc = block32_dot<kQuant>(c0, a0[t]);
                if (live1) acc += block32_dot<kQuant>(c1, a1[t]);
            }
            acc = seg_sum<kLanesPerRow>(acc);
            if (sub == kLanesPerRow - 1 && row < rows && tok0 + t < seq)
                out[(static_cast<size_t>(tok0 + t) * heads + head) * rows + row] = acc;
        }
    }
}

template <uint32_t kQuant>
void launch_block32(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb32, uint32_t seq,
                    hipStream_t stream) {
    const uint32_t waves = rows < kTargetWaves ? rows : kTargetWaves;
    if (seq >= 2 && nb32 <= 2 * kWave) {  // several tokens per pass over the matrix, in groups of equal size (at most four)
        const auto [groups, per] = token_groups(seq);
        const dim3 tgrid((waves + kWavesPerWg - 1) / kWavesPerWg, groups, 1);
        bool paired = false;
        if constexpr (block32_pairs<kQuant>()) paired = nb32 % 2 == 0 && reinterpret_cast<uintptr_t>(w) % 4 == 0;
#define RNB_LAUNCH_TOKENS(P, T)                                                                                              \
    hipLaunchKernelGGL((gemv_block32_tokens_kernel<kQuant, P, T>), tgrid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs, \
                       act.d, out, rows, nb32, seq)
#define RNB_LAUNCH_TOKENS_P(P)    \
    do {                          \
        if (per == 2)             \
            RNB_LAUNCH_TOKENS(P, 2); \
        else if (per == 3)        \
            RNB_LAUNCH_TOKENS(P, 3); \
        else                      \
            RNB_LAUNCH_TOKENS(P, 4); \
    } while (0)
        if constexpr (block32_pairs<kQuant>()) {
            if (paired) {
                RNB_LAUNCH_TOKENS_P(true);
                return;
            }
        }
        RNB_LAUNCH_TOKENS_P(false);
#undef RNB_LAUNCH_TOKENS_P
#undef RNB_LAUNCH_TOKENS
        return;
    }
    const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, seq, 1);
    if constexpr (block32_pairs<kQuant>()) {
        if (nb32 % 2 == 0 && reinterpret_cast<uintptr_t>(w) % 4 == 0) {  // every pair of every row starts on a 4-byte boundary
            hipLaunchKernelGGL((gemv_block32_kernel<kQuant, true>), grid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs, act.d,
                               out, rows, nb32);
            return;
        }
    }
    hipLaunchKernelGGL((gemv_block32_kernel<kQuant, false>), grid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs, act.d, out,
                       rows, nb32);
}

// Per-head Q8_0 projections of a token batch: weights [heads][rows_per_head][nb32 blocks], activations (32-wide Q8)
// [tokens][heads][nb32], out [tokens][heads * rows_per_head]; rows of at most 128 blocks.
void launch_heads_q8_0(const uint8_t *w, ActView act, float *out, uint32_t heads, uint32_t rows_per_head, uint32_t nb32,
                       uint32_t tokens, hipStream_t stream) {
    const bool paired = nb32 % 2 == 0 && reinterpret_cast<uintptr_t>(w) % 4 == 0;
    // rows per wave: as many as the row's blocks (two per lane when paired) leave room for
    const uint32_t lanes = paired ? nb32 / 2 : nb32;
    const uint32_t rpw = lanes <= 4 ? 16 : (lanes <= 16 ? 4 : 1);
    const uint32_t row_groups = (rows_per_head + rpw - 1) / rpw;
    const uint32_t waves = row_groups < kTargetWaves ? row_groups : kTargetWaves;
    const auto [groups, per] = token_groups(tokens);
    const dim3 grid((waves + kWavesPerWg - 1) / kWavesPerWg, groups, heads);
#define RNB_LAUNCH_HEADS(P, T, R)                                                                                             \
    hipLaunchKernelGGL((gemv_block32_tokens_kernel<kQ8_0, P, T, R>), grid, dim3(kWave * kWavesPerWg), 0, stream, w, act.qs, \
                       act.d, out, rows_per_head, nb32, tokens)
#define RNB_LAUNCH_HEADS_T(P, R)      \
    do {                              \
        if (per == 1)                 \
            RNB_LAUNCH_HEADS(P, 1, R); \
        else if (per == 2)            \
            RNB_LAUNCH_HEADS(P, 2, R); \
        else if (per == 3)            \
            RNB_LAUNCH_HEADS(P, 3, R); \
        else                          \
            RNB_LAUNCH_HEADS(P, 4, R); \
    } while (0)
#define RNB_LAUNCH_HEADS_R(P)         \
    do {                              \
        if (rpw == 16)                \
            RNB_LAUNCH_HEADS_T(P, 16); \
        else if (rpw == 4)            \
            RNB_LAUNCH_HEADS_T(P, 4);  \
        else                          \
            RNB_LAUNCH_HEADS_T(P, 1);  \
    } while (0)
    if (paired)
        RNB_LAUNCH_HEADS_R(true);
    else
        RNB_LAUNCH_HEADS_R(false);
#undef RNB_LAUNCH_HEADS_R
#undef RNB_LAUNCH_HEADS_T
#undef RNB_LAUNCH_HEADS
}

// One f32 token against rows of at most 128 blocks: the workgroup quantises the token to 32-wide Q8 in LDS itself
// (the wave-level quantiser of quantize_q8_kernel, so the same bits), as gemv_kquant_f32_kernel does for Q8_K; each
// lane's first row blocks are requested before the quantisation (a second row in flight measured slower here).
template <uint32_t kQuant, bool kPaired>
__global__ void __launch_bounds__(kWave *kFusedWaves)
    gemv_block32_f32_kernel(const uint8_t *__restrict__ w, const float *__restrict__ x, float *__restrict__ out, uint32_t rows,
                            uint32_t nb32) {
    constexpr size_t kBlockBytes = block32_layout<kQuant>().bytes;
    constexpr bool kSum = kQuant != kQ8_0 && kQuant != kQ8_1;
    constexpr int kSpans = 16 / kFusedWaves;
    __shared__ __attribute__((aligned(16))) int8_t s_qs[128 * 32];
    __shared__ float s_d[128];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t tok = blockIdx.y;
    const float *x_tok = x + static_cast<size_t>(tok) * nb32 * 32;
    const size_t row_bytes = static_cast<size_t>(nb32) * kBlockBytes;
    const uint32_t n_waves = gridDim.x * kFusedWaves;
    uint32_t row = blockIdx.x * kFusedWaves + wave;
    // kPaired (see gemv_block32_kernel): blocks 2 l and 2 l + 1, fetched as one aligned pair
    const uint32_t b0 = kPaired ? 2 * lane : lane, b1 = kPaired ? 2 * lane + 1 : lane + kWave;
    const bool has0 = b0 < nb32, has1 = b1 < nb32;
    // the token first (span = 256 elements = 8 blocks; the last span may be partial), then the first rows' blocks
    float4 xv[kSpans];
    int live[kSpans];
#pragma unroll
    for (int i = 0; i < kSpans; i++) {
        const uint32_t span = wave + i * kFusedWaves;
        const int left = static_cast<int>(nb32) - static_cast<int>(span) * 8;
        live[i] = left < 0 ? 0 : (left > 8 ? 8 : left);
        xv[i] = q8_load_span(x_tok + static_cast<size_t>(span) * 256, lane, live[i]);
    }
    auto fetch = [&](uint32_t r, bool has, uint32_t b) {
        const size_t off = (has && r < rows) ? static_cast<size_t>(r) * row_bytes + static_cast<size_t>(b) * kBlockBytes : 0;
        return block32_load<kQuant>(w + off);  // rows >= 1 and nb32 >= 1: offset 0 is readable
    };
    Block32Regs c0, c1;
    auto fetch_row = [&](uint32_t r) {
        if constexpr (kPaired) {  // nb32 is even: a pair is there or not as a whole
            const size_t off = (has0 && r < rows) ? static_cast<size_t>(r) * row_bytes + static_cast<size_t>(b0) * kBlockBytes : 0;
            block32_load_pair<kQuant>(w + off, c0, c1);  // offset 0 holds a whole pair
        } else {
            c0 = fetch(r, has0, b0);
            c1 = fetch(r, has1, b1);
        }
    };
    fetch_row(row);
#pragma unroll
    for (int i = 0; i < kSpans; i++) {
        const uint32_t span = wave + i * kFusedWaves;
        q8_quantize_vals(xv[i], lane, live[i], s_qs + span * 256, s_d + span * 8);
    }
    __syncthreads();
    const Q8Act a0 = q8_load_act<kSum>(s_qs + (has0 ? b0 : 0) * 32, s_d[has0 ? b0 : 0]);
    const Q8Act a1 = q8_load_act<kSum>(s_qs + (has1 ? b1 : 0) * 32, s_d[has1 ? b1 : 0]);
    for (; row < rows; row += n_waves) {
        float acc = 0.0f;
        if (has0) acc = block32_dot<kQuant>(c0, a0);
        if (has1) acc += block32_dot<kQuant>(c1, a1);
        acc = seg_sum<kWave>(acc);
        if (lane == kWave - 1) out[static_cast<size_t>(tok) * rows + row] = acc;
        fetch_row(row + n_waves);
    }
}

template <uint32_t kQuant>
void launch_block32_f32(const uint8_t *w, const float *x, float *out, uint32_t rows, uint32_t nb32, uint32_t seq,
                        hipStream_t stream) {
    const uint32_t waves = fused_waves(rows);
    const dim3 grid((waves + kFusedWaves - 1) / kFusedWaves, seq, 1);
    if constexpr (block32_pairs<kQuant>()) {
        if (nb32 % 2 == 0 && reinterpret_cast<uintptr_t>(w) % 4 == 0) {
            hipLaunchKernelGGL((gemv_block32_f32_kernel<kQuant, true>), grid, dim3(kWave * kFusedWaves), 0, stream, w, x, out, rows,
                               nb32);
            return;
        }
    }
    hipLaunchKernelGGL((gemv_block32_f32_kernel<kQuant, false>), grid, dim3(kWave * kFusedWaves), 0, stream, w, x, out, rows, nb32);
}

}  // namespace

void launch_gemv_q4k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                     hipStream_t stream) {
    launch_kquant_any<kQ4K>(w, act, out, rows, nb, seq, stream);
}

void launch_gemv_q5k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                     hipStream_t stream) {
    launch_kquant_any<kQ5K>(w, act, out, rows, nb, seq, stream);
}

void launch_gemv_q2k_q3k(const uint8_t *w, uint32_t quant, ActView act, float *out, uint32_t rows, uint32_t nb,
                         uint32_t seq, hipStream_t stream) {
    if (quant == kQ2K)
        launch_kquant_any<kQ2K>(w, act, out, rows, nb, seq, stream);
    else
        launch_kquant_any<kQ3K>(w, act, out, rows, nb, seq, stream);
}

void launch_gemv_q6k(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                     hipStream_t stream) {
    launch_kquant_any<kQ6K>(w, act, out, rows, nb, seq, stream);
}

bool gemv_kquant_f32_supported(uint32_t quant, uint32_t nb, const void *x, const void *w) {
    const bool kq = quant == kQ2K || quant == kQ3K || quant == kQ4K || quant == kQ5K || quant == kQ6K;
    // the sixteen-wave kernel fetches Q6_K blocks without the odd-address path
    if (quant == kQ6K && nb > 16 && reinterpret_cast<uintptr_t>(w) % 2 != 0) return false;
    return kq && nb >= 1 && nb <= kWideMaxBlocks && reinterpret_cast<uintptr_t>(x) % 16 == 0;
}

bool gemv_kquant_f32_pays(uint32_t quant, uint32_t rows, uint32_t nb) {
    // From about 300 MB on, the separate quantiser launch costs less than what the chunked kernel gains over the
    // one-launch kernel, whose workgroups loop (steps measured back to back: 264 MB of Q4_K 49.5 us in one launch against
    // 51.1 in two, 431 MB of Q6_K 83.1 against 79.0).  The chunked kernel with the quantiser in front (one chunk per wave,
    // one barrier per workgroup of 4, 8 or 16 waves) was tried: 431 MB of Q6_K 81 / 86 / 94 us, 264 MB of Q4_K 71 / 56 us;
    // so was the one-launch kernel looping over chunks of consecutive rows (1, 2 or 4 rows, with and without the next
    // chunk requested ahead): 79.5 - 82.4 us and 47.2 - 50.0 us, inside the spread between boxes of what is here.
    size_t bytes = 0;
    switch (quant) {
    case kQ2K: bytes = kQ2KBytes; break;
    case kQ3K: bytes = kQ3KBytes; break;
    case kQ4K: bytes = kQ4KBytes; break;
    case kQ5K: bytes = kQ5KBytes; break;
    default: bytes = kQ6KBytes; break;
    }
    return nb <= 8 || static_cast<uint64_t>(rows) * nb * bytes < (uint64_t(300) << 20);
}

void launch_gemv_kquant_f32(const uint8_t *w, uint32_t quant, const float *x, float *out, uint32_t rows, uint32_t nb,
                            uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    if (nb > 16) {  // rows of 17 to 64 super-blocks: one token per launch
        for (uint32_t t = 0; t < seq; t++) {
            const float *xt = x + static_cast<size_t>(t) * nb * 256;
            float *ot = out + static_cast<size_t>(t) * rows;
            switch (quant) {
            case kQ2K: launch_kquant_wide_f32<kQ2K>(w, xt, ot, rows, nb, stream); break;
            case kQ3K: launch_kquant_wide_f32<kQ3K>(w, xt, ot, rows, nb, stream); break;
            case kQ4K: launch_kquant_wide_f32<kQ4K>(w, xt, ot, rows, nb, stream); break;
            case kQ5K: launch_kquant_wide_f32<kQ5K>(w, xt, ot, rows, nb, stream); break;
            default: launch_kquant_wide_f32<kQ6K>(w, xt, ot, rows, nb, stream); break;
            }
        }
        return;
    }
    switch (quant) {
    case kQ2K: launch_kquant_f32_any<kQ2K>(w, x, out, rows, nb, seq, stream); break;
    case kQ3K: launch_kquant_f32_any<kQ3K>(w, x, out, rows, nb, seq, stream); break;
    case kQ4K: launch_kquant_f32_any<kQ4K>(w, x, out, rows, nb, seq, stream); break;
    case kQ5K: launch_kquant_f32_any<kQ5K>(w, x, out, rows, nb, seq, stream); break;
    default: launch_kquant_f32_any<kQ6K>(w, x, out, rows, nb, seq, stream); break;
    }
}

bool gemv_q8_0_heads_supported(uint32_t nb32) { return nb32 >= 1 && nb32 <= 2 * kWave; }

void launch_gemv_q8_0_heads(const uint8_t *w, ActView act, float *out, uint32_t heads, uint32_t rows_per_head, uint32_t nb32,
                            uint32_t tokens, hipStream_t stream) {
    if (heads == 0 || rows_per_head == 0 || tokens == 0) return;
    launch_heads_q8_0(w, act, out, heads, rows_per_head, nb32, tokens, stream);
}

bool gemv_q4k_gate_up_supported(uint32_t nb) { return nb >= 1 && nb <= 16; }

void launch_gemv_q4k_gate_up(const uint8_t *wg, const uint8_t *wu, ActView act, float *mid, uint32_t rows, uint32_t nb,
                             uint32_t seq, bool gelu, hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    if (nb <= 4)
        launch_gate_up<4>(wg, wu, act, mid, rows, nb, seq, gelu, stream);
    else if (nb <= 8)
        launch_gate_up<2>(wg, wu, act, mid, rows, nb, seq, gelu, stream);
    else
        launch_gate_up<1>(wg, wu, act, mid, rows, nb, seq, gelu, stream);
}

void launch_gemv_q4k_gate_up_f32(const uint8_t *wg, const uint8_t *wu, const float *x, float *mid, uint32_t rows,
                                 uint32_t nb, uint32_t seq, bool gelu, hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    if (nb <= 4)
        launch_gate_up_f32<4>(wg, wu, x, mid, rows, nb, seq, gelu, stream);
    else if (nb <= 8)
        launch_gate_up_f32<2>(wg, wu, x, mid, rows, nb, seq, gelu, stream);
    else
        launch_gate_up_f32<1>(wg, wu, x, mid, rows, nb, seq, gelu, stream);
}

void launch_gemv_q4k_multi_f32(const uint8_t *const w[3], const uint32_t rows[3], const float *x, float *out, uint32_t nb,
                               hipStream_t stream) {
    MultiMat mats;
    uint32_t total = 0;
    for (int i = 0; i < 3; i++) {
        mats.w[i] = w[i];
        total += rows[i];
        mats.end[i] = total;
    }
    if (total == 0) return;
    if (nb <= 4)
        launch_multi_f32<4>(mats, x, out, nb, stream);
    else if (nb <= 8)
        launch_multi_f32<2>(mats, x, out, nb, stream);
    else
        launch_multi_f32<1>(mats, x, out, nb, stream);
}

void launch_gemv_q4k_multi(const uint8_t *const w[3], const uint32_t rows[3], ActView act, float *out, uint32_t nb,
                           hipStream_t stream) {
    MultiMat mats;
    uint32_t total = 0;
    for (int i = 0; i < 3; i++) {
        mats.w[i] = w[i];
        total += rows[i];
        mats.end[i] = total;
    }
    if (total == 0) return;
    if (nb <= 4)
        launch_multi<4>(mats, act, out, nb, stream);
    else if (nb <= 8)
        launch_multi<2>(mats, act, out, nb, stream);
    else
        launch_multi<1>(mats, act, out, nb, stream);
}

void launch_act_mul(const float *gate, const float *up, float *out, size_t n, bool gelu, hipStream_t stream) {
    if (n == 0) return;
    const size_t blocks = (n + 255) / 256;
    const dim3 grid(static_cast<unsigned>(blocks < 4096 ? blocks : 4096));
    if (gelu)
        hipLaunchKernelGGL(act_mul_kernel<true>, grid, dim3(256), 0, stream, gate, up, out, n);
    else
        hipLaunchKernelGGL(act_mul_kernel<false>, grid, dim3(256), 0, stream, gate, up, out, n);
}

void launch_gemv_q8_0(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb32, uint32_t seq,
                      hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    launch_block32<kQ8_0>(w, act, out, rows, nb32, seq, stream);
}

void launch_gemv_block32(const uint8_t *w, uint32_t quant, ActView act, float *out, uint32_t rows, uint32_t nb32,
                         uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    switch (quant) {
    case kQ4_0: launch_block32<kQ4_0>(w, act, out, rows, nb32, seq, stream); break;
    case kQ4_1: launch_block32<kQ4_1>(w, act, out, rows, nb32, seq, stream); break;
    case kQ5_0: launch_block32<kQ5_0>(w, act, out, rows, nb32, seq, stream); break;
    case kQ5_1: launch_block32<kQ5_1>(w, act, out, rows, nb32, seq, stream); break;
    case kQ8_1: launch_block32<kQ8_1>(w, act, out, rows, nb32, seq, stream); break;
    default: launch_block32<kQ8_0>(w, act, out, rows, nb32, seq, stream); break;
    }
}

bool gemv_block32_f32_supported(uint32_t rows, uint32_t nb32, const void *x) {
    // measured: the saved launch outweighs the per-workgroup quantisation from about 4096 x 2048 upwards
    return nb32 >= 1 && nb32 <= 128 && static_cast<uint64_t>(rows) * nb32 >= (1u << 18) &&
           reinterpret_cast<uintptr_t>(x) % 16 == 0;
}

void launch_gemv_block32_f32(const uint8_t *w, uint32_t quant, const float *x, float *out, uint32_t rows, uint32_t nb32,
                             uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0) return;
    switch (quant) {
    case kQ4_0: launch_block32_f32<kQ4_0>(w, x, out, rows, nb32, seq, stream); break;
    case kQ4_1: launch_block32_f32<kQ4_1>(w, x, out, rows, nb32, seq, stream); break;
    case kQ5_0: launch_block32_f32<kQ5_0>(w, x, out, rows, nb32, seq, stream); break;
    case kQ5_1: launch_block32_f32<kQ5_1>(w, x, out, rows, nb32, seq, stream); break;
    case kQ8_1: launch_block32_f32<kQ8_1>(w, x, out, rows, nb32, seq, stream); break;
    default: launch_block32_f32<kQ8_0>(w, x, out, rows, nb32, seq, stream); break;
    }
}

}  // namespace rnb
