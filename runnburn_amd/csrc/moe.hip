// Gathered sparse-MoE expert path (Qwen3-MoE style): per routed slot (token, expert, weight)
//   mid   = silu(W_gate[e] . Q8_K(h)) * (W_up[e] . Q8_K(h))      Q4_K rows, K = n_embd
//   o     = route * (W_down[e] . Q8_K(mid))                       Q4_K | Q6_K rows, K = n_ff
//   out[token] = sum of o over the token's slots in slot order
// following crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:260-327
// (compute_expert_host_from_slices), crates/rnb-cpu/src/kernels/activation.rs:73-89
// (fused_silu_mul_inplace) and .../shared_expert_moe/prefill_cpu.rs:167-194 (ordered reduce).
//
// Expert weights are never copied: an expert is base + e * bytes_per_expert, the slicing of
// fanout.rs:4-22.  Slots are grouped by expert (the expert-major order of prefill_cpu.rs:113-146):
// a workgroup owns a tile of rows of ONE expert, stages the quantised activations of that expert's
// tokens in LDS, then every wave keeps a row's packed blocks in registers and walks the tokens, so
// an expert's weights are streamed from HBM once however many tokens were routed to it.  A decode
// call (one token) is the same kernel with one token per group.
#include "act_quant.h"
#include "block_dots.h"
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

constexpr int kWavesPerWg = 4;
constexpr int kMaxChunkTokens = 8;  // tokens staged in LDS at a time

// LDS staging of `nt` quantised activation rows: qs [nt][nb][272] | d [nt][nb] | bsums [nt][nb*16].  A block's 256
// int8 take a 272-byte slot: the lanes of a wave read 16-byte pieces of different blocks, and a 256-byte stride
// would put them all on the same banks.
constexpr uint32_t kStageBlk = 272;
struct Staged {
    const int8_t *qs;
    const float *d;
    const int16_t *bsums;
};

__host__ __device__ __forceinline__ size_t stage_d_offset(uint32_t tmax, uint32_t nb) {
    return static_cast<size_t>(tmax) * nb * kStageBlk;
}
__host__ __device__ __forceinline__ size_t stage_bsums_offset(uint32_t tmax, uint32_t nb) {
    return stage_d_offset(tmax, nb) + ((static_cast<size_t>(tmax) * nb * 4 + 15) & ~static_cast<size_t>(15));
}
__host__ __device__ __forceinline__ size_t stage_bytes(uint32_t tmax, uint32_t nb) {
    return stage_bsums_offset(tmax, nb) + static_cast<size_t>(tmax) * nb * 32;
}

__device__ __forceinline__ Staged stage_layout(uint8_t *lds, uint32_t tmax, uint32_t nb) {
    Staged s;
    s.qs = reinterpret_cast<const int8_t *>(lds);
    s.d = reinterpret_cast<const float *>(lds + stage_d_offset(tmax, nb));
    s.bsums = reinterpret_cast<const int16_t *>(lds + stage_bsums_offset(tmax, nb));
    return s;
}

// copies activation row `src_row` (global, SoA) into staging slot t
__device__ __forceinline__ void stage_row(uint8_t *lds, uint32_t tmax, uint32_t nb, uint32_t t, size_t src_row,
                                          const int8_t *__restrict__ aq, const float *__restrict__ ad,
                                          const int16_t *__restrict__ abs) {
    uint8_t *dq = lds + static_cast<size_t>(t) * nb * kStageBlk;
    const uint4 *sq = reinterpret_cast<const uint4 *>(aq + src_row * nb * 256);
    for (uint32_t i = threadIdx.x; i < nb * 16; i += blockDim.x)
        *reinterpret_cast<uint4 *>(dq + (i >> 4) * kStageBlk + (i & 15) * 16) = sq[i];
    float *dd = reinterpret_cast<float *>(lds + stage_d_offset(tmax, nb)) + static_cast<size_t>(t) * nb;
    for (uint32_t i = threadIdx.x; i < nb; i += blockDim.x) dd[i] = ad[src_row * nb + i];
    uint4 *db = reinterpret_cast<uint4 *>(lds + stage_bsums_offset(tmax, nb)) + static_cast<size_t>(t) * nb * 2;
    const uint4 *sb = reinterpret_cast<const uint4 *>(abs + src_row * nb * 16);
    for (uint32_t i = threadIdx.x; i < nb * 2; i += blockDim.x) db[i] = sb[i];
}

// quantises f32 row `src` (nb blocks of 256) into staging slot t: the stand-alone quantiser's wave routine, a wave per
// block (the same bits); must be called by the whole workgroup
__device__ __forceinline__ void stage_row_f32(uint8_t *lds, uint32_t tmax, uint32_t nb, uint32_t t, const float *__restrict__ src) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6, n_waves = blockDim.x >> 6;
    int8_t *dq = reinterpret_cast<int8_t *>(lds) + static_cast<size_t>(t) * nb * kStageBlk;
    float *dd = reinterpret_cast<float *>(lds + stage_d_offset(tmax, nb)) + static_cast<size_t>(t) * nb;
    int16_t *db = reinterpret_cast<int16_t *>(lds + stage_bsums_offset(tmax, nb)) + static_cast<size_t>(t) * nb * 16;
    for (uint32_t b = wave; b < nb; b += n_waves)
        q8k_quantize_span(src + static_cast<size_t>(b) * 256, lane, dq + static_cast<size_t>(b) * kStageBlk, dd + b, db + b * 16);
}

// ---------------------------------------------------------------------------------------------
// gate + up + SiLU*up.  Grid (row tiles, expert groups).  kRowsPerWave rows side by side per wave.
// ---------------------------------------------------------------------------------------------
template <int kRowsPerWave>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    moe_gate_up_kernel(const uint8_t *__restrict__ gate_all, const uint8_t *__restrict__ up_all,
                       const uint8_t *__restrict__ gate_shared, const uint8_t *__restrict__ up_shared, uint32_t n_routed,
                       const int8_t *__restrict__ aq, const float *__restrict__ ad, const int16_t *__restrict__ abs,
                       const uint32_t *__restrict__ grp_expert, const uint32_t *__restrict__ grp_start,
                       const uint32_t *__restrict__ sorted_slot, const uint32_t *__restrict__ sorted_token,
                       float *__restrict__ mid, uint32_t n_ff, uint32_t nb, uint32_t iters, uint32_t tmax) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    constexpr uint32_t kBlocksPerPass = kLanesPerRow / 4;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const uint32_t grp = blockIdx.y;
    const uint32_t expert = grp_expert[grp], start = grp_start[grp], count = grp_start[grp + 1] - start;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    const uint8_t *gate_e = expert_base(gate_all, gate_shared, n_routed, expert, n_ff * row_bytes);
    const uint8_t *up_e = expert_base(up_all, up_shared, n_routed, expert, n_ff * row_bytes);
    const uint32_t rows_per_wg = kWavesPerWg * kRowsPerWave * iters;
    const Staged st = stage_layout(lds, tmax, nb);
    float2 *xch = reinterpret_cast<float2 *>(lds + stage_bytes(tmax, nb)) + wave * (kMaxChunkTokens * kRowsPerWave);

    for (uint32_t c0 = 0; c0 < count; c0 += tmax) {
        const uint32_t nt = min(tmax, count - c0);
        if (c0) __syncthreads();
        for (uint32_t t = 0; t < nt; t++) stage_row(lds, tmax, nb, t, sorted_token[start + c0 + t], aq, ad, abs);
        __syncthreads();
        for (uint32_t it = 0; it < iters; it++) {
            const uint32_t row0_it = blockIdx.x * rows_per_wg + (it * kWavesPerWg + wave) * kRowsPerWave;
            const uint32_t row = row0_it + rsel;
            const bool row_ok = row < n_ff;
            float gacc[kMaxChunkTokens], uacc[kMaxChunkTokens];
#pragma unroll
            for (int t = 0; t < kMaxChunkTokens; t++) gacc[t] = uacc[t] = 0.0f;
            for (uint32_t b = bslot; b < nb; b += kBlocksPerPass) {
                if (!row_ok) break;
                const size_t off = static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b) * kQ4KBytes;
                const Q4KPrep gp = q4k_prepare(q4k_load_block(gate_e + off, g), g);
                const Q4KPrep up = q4k_prepare(q4k_load_block(up_e + off, g), g);
#pragma unroll
                for (int t = 0; t < kMaxChunkTokens; t++) {
                    if (static_cast<uint32_t>(t) < nt) {
                        const size_t ab = static_cast<size_t>(t) * nb + b;
                        const Q4KAct a = q4k_load_act(st.qs + ab * kStageBlk, st.d[ab], st.bsums + ab * 16, g);
                        gacc[t] += q4k_dot(gp, a);
                        uacc[t] += q4k_dot(up, a);
                    }
                }
            }
            // The row sums land in the last lane of each row segment.  SiLU on them lane by lane would spend a full
            // instruction stream per token on one or two useful lanes, so the (gate, up) pairs of all staged tokens go
            // through a per-wave LDS slot and lane t * kRowsPerWave + r finishes token t of row r: one SiLU pass per
            // row iteration.  LDS operations of one wave complete in order; the fence only pins the compiler's order.
#pragma unroll
            for (int t = 0; t < kMaxChunkTokens; t++) {
                if (static_cast<uint32_t>(t) < nt) {  // nt is workgroup-uniform
                    const float gs = seg_sum<kLanesPerRow>(gacc[t]);
                    const float us = seg_sum<kLanesPerRow>(uacc[t]);
                    if (sub == kLanesPerRow - 1) xch[t * kRowsPerWave + rsel] = make_float2(gs, us);
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            if (static_cast<uint32_t>(lane) < nt * kRowsPerWave) {
                const uint32_t t = lane / kRowsPerWave;
                const uint32_t r2 = row0_it + lane % kRowsPerWave;
                const float2 v = xch[lane];
                if (r2 < n_ff) {
                    // crates/rnb-cpu/src/kernels/activation.rs:73-89: (g / (1 + exp(-g))) * up
                    const float e = expf(-v.x);
                    mid[static_cast<size_t>(sorted_slot[start + c0 + t]) * n_ff + r2] = (v.x / (1.0f + e)) * v.y;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
        }
    }
}

// ---------------------------------------------------------------------------------------------
// down projection of the re-quantised intermediate, scaled by the route weight.
// ---------------------------------------------------------------------------------------------
// kFromF32: the intermediates come as f32 rows (mid_f32[slot][nb * 256]) and are quantised while they are staged
template <uint32_t kQuant, int kRowsPerWave, bool kFromF32>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    moe_down_kernel(const uint8_t *__restrict__ down_all, const uint8_t *__restrict__ down_shared, uint32_t n_routed,
                    const int8_t *__restrict__ mq, const float *__restrict__ md,
                    const int16_t *__restrict__ mbs, const float *__restrict__ mid_f32,
                    const uint32_t *__restrict__ grp_expert,
                    const uint32_t *__restrict__ grp_start, const uint32_t *__restrict__ sorted_slot,
                    const float *__restrict__ slot_route, float *__restrict__ slot_out, uint32_t n_embd, uint32_t nb,
                    uint32_t iters, uint32_t tmax) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    constexpr int kLanesPerRow = kWave / kRowsPerWave;
    constexpr uint32_t kBlocksPerPass = kLanesPerRow / 4;
    using Q = KQuant<kQuant>;
    constexpr size_t kBlockBytes = Q::kBytes;
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
    const int sub = lane & (kLanesPerRow - 1);
    const uint32_t rsel = lane / kLanesPerRow;
    const int g = sub & 3;
    const uint32_t bslot = sub >> 2;
    const uint32_t grp = blockIdx.y;
    const uint32_t expert = grp_expert[grp], start = grp_start[grp], count = grp_start[grp + 1] - start;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint8_t *down_e = expert_base(down_all, down_shared, n_routed, expert, n_embd * row_bytes);
    const uint32_t rows_per_wg = kWavesPerWg * kRowsPerWave * iters;
    const Staged st = stage_layout(lds, tmax, nb);

    for (uint32_t c0 = 0; c0 < count; c0 += tmax) {
        const uint32_t nt = min(tmax, count - c0);
        if (c0) __syncthreads();
        for (uint32_t t = 0; t < nt; t++) {
            const uint32_t slot = sorted_slot[start + c0 + t];
            if constexpr (kFromF32)
                stage_row_f32(lds, tmax, nb, t, mid_f32 + static_cast<size_t>(slot) * nb * 256);
            else
                stage_row(lds, tmax, nb, t, slot, mq, md, mbs);
        }
        __syncthreads();
        for (uint32_t it = 0; it < iters; it++) {
            const uint32_t row = blockIdx.x * rows_per_wg + (it * kWavesPerWg + wave) * kRowsPerWave + rsel;
            const bool row_ok = row < n_embd;
            float acc[kMaxChunkTokens];
#pragma unroll
            for (int t = 0; t < kMaxChunkTokens; t++) acc[t] = 0.0f;
            for (uint32_t b = bslot; b < nb; b += kBlocksPerPass) {
                if (!row_ok) break;
                const uint8_t *blk = down_e + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b) * kBlockBytes;
                const typename Q::Prep p = Q::prepare(Q::load_block(blk, g), g);
#pragma unroll
                for (int t = 0; t < kMaxChunkTokens; t++) {
                    if (static_cast<uint32_t>(t) < nt) {
                        const size_t ab = static_cast<size_t>(t) * nb + b;
                        acc[t] += Q::dot(p, Q::load_act(st.qs + ab * kStageBlk, st.d[ab], st.bsums + ab * 16, g));
                    }
                }
            }
#pragma unroll
            for (int t = 0; t < kMaxChunkTokens; t++) {
                if (static_cast<uint32_t>(t) < nt) {
                    const float s = seg_sum<kLanesPerRow>(acc[t]);
                    if (sub == kLanesPerRow - 1 && row_ok) {
                        const uint32_t slot = sorted_slot[start + c0 + t];
                        slot_out[static_cast<size_t>(slot) * n_embd + row] = s * slot_route[slot];  // fanout.rs:306-308
                    }
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Decode-sized calls: down projection, route weight and the per-token ordered sum in one launch, no slot_out round
// trip.  A wave owns ONE output row of one token; its lanes are split into 64/L groups of L = 4 * (blocks a group can
// hold) lanes, each group dotting that row of a different slot's expert against that slot's quantised intermediate.
// The groups' sums (last lane of each group) are then added in list order, so the result is the same sequence of f32
// additions as moe_down_kernel followed by moe_reduce_kernel.
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant, int kGroups>
__global__ void __launch_bounds__(kWave *kWavesPerWg)
    moe_down_token_kernel(const uint8_t *__restrict__ down_all, const uint8_t *__restrict__ down_shared, uint32_t n_routed,
                          const int8_t *__restrict__ mq,
                          const float *__restrict__ md, const int16_t *__restrict__ mbs,
                          const uint32_t *__restrict__ tok_offsets, const uint32_t *__restrict__ tok_slots,
                          const uint32_t *__restrict__ slot_expert, const float *__restrict__ slot_route,
                          float *__restrict__ out, uint32_t n_embd, uint32_t nb) {
    constexpr int kLanes = kWave / kGroups;  // lanes per (slot, row) pair
    using Q = KQuant<kQuant>;
    constexpr size_t kBlockBytes = Q::kBytes;
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kWavesPerWg + (threadIdx.x >> 6);
    const uint32_t tok = blockIdx.y;
    if (row >= n_embd) return;  // wave-uniform
    const int sub = lane & (kLanes - 1);
    const uint32_t grp = lane / kLanes;
    const int g = sub & 3;
    const uint32_t b = sub >> 2;
    const bool has_block = b < nb;
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    const uint32_t begin = tok_offsets[tok], end = tok_offsets[tok + 1];
    float acc = 0.0f;
    for (uint32_t k0 = begin; k0 < end; k0 += kGroups) {
        const uint32_t k = k0 + grp;
        float o = 0.0f;
        if (k < end && has_block) {
            const uint32_t slot = tok_slots[k];
            const uint8_t *blk = expert_base(down_all, down_shared, n_routed, slot_expert[slot], n_embd * row_bytes) +
                                 static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b) * kBlockBytes;
            const size_t ab = static_cast<size_t>(slot) * nb + b;
            o = kquant_partial<kQuant>(Q::load_block(blk, g), Q::load_act(mq + ab * 256, md[ab], mbs + ab * 16, g), g);
        }
        o = seg_sum<kLanes>(o);
        if (k < end) o *= slot_route[tok_slots[k]];  // fanout.rs:306-308; only the group's last lane is read below
#pragma unroll
        for (int j = 0; j < kGroups; j++) {
            const float v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, o), j * kLanes + kLanes - 1));
            if (k0 + j < end) acc += v;  // wave-uniform
        }
    }
    if (lane == 0) out[static_cast<size_t>(tok) * n_embd + row] = acc;
}

// ---------------------------------------------------------------------------------------------
// A few tokens (decode, small batches): two launches for the whole expert step, the routing table riding in the kernel
// arguments, slots listed token by token.
//   moe_decode_gate_up_kernel   grid (row groups / 8, slots): the workgroup quantises its slot's token to Q8_K in LDS (as
//                               gemv_kquant_f32_kernel does), every wave makes one group of rows of its slot's expert
//   moe_decode_down_kernel      grid (rows / 8, tokens): the workgroup quantises its token's slots' intermediates
//                               (slots * nb_mid <= 64 blocks) in LDS, then moe_down_token_kernel's row scheme: down,
//                               route weight, ordered sum; two register sets in turn over the wave's (row, slot group)
//                               steps (four tokens of 8 slots on 128 experts 24.0 -> 23.0 us per call)
// Same quantiser, dots and order of additions as the general path, so the same bits.  An expert that several tokens
// chose is read once per slot here (the second time mostly from the L2), which is what bounds the batch this pays for.
// ---------------------------------------------------------------------------------------------
constexpr int kDecodeWaves = 8;

// kOne: a call of one token (token index 0 for every slot, the whole list is the token's): no table look-ups in front of
// the first loads
template <int kRowsPerWave, bool kOne>
__global__ void __launch_bounds__(kWave *kDecodeWaves)
    moe_decode_gate_up_kernel(const uint8_t *__restrict__ gate_all, const uint8_t *__restrict__ up_all,
                              const uint8_t *__restrict__ gate_shared, const uint8_t *__restrict__ up_shared,
                              uint32_t n_routed, const float *__restrict__ x, const MoeDecodeTable table, float *__restrict__ mid,
                              uint32_t n_ff, uint32_t nb) {
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
    const uint32_t slot = blockIdx.y;
    const uint32_t row = (blockIdx.x * kDecodeWaves + wave) * kRowsPerWave + rsel;
    const bool live = bslot < nb && row < n_ff;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    TokenSpans<kDecodeWaves> xv;
    token_load<kDecodeWaves>(x + (kOne ? 0 : static_cast<size_t>(table.token[slot]) * nb * 256), nb, wave, lane, xv);
    // dead lanes read the expert's first block
    const size_t off = live ? static_cast<size_t>(row) * row_bytes + static_cast<size_t>(bslot) * kQ4KBytes : 0;
    const uint32_t expert = table.expert[slot];
    const Q4KRegs rg = q4k_load_block(expert_base(gate_all, gate_shared, n_routed, expert, n_ff * row_bytes) + off, g),
                  ru = q4k_load_block(expert_base(up_all, up_shared, n_routed, expert, n_ff * row_bytes) + off, g);
    token_quantize<kDecodeWaves>(xv, nb, wave, lane, s_qs, s_d, s_bsums);
    __syncthreads();
    const uint32_t ab = bslot < nb ? bslot : 0;
    const Q4KAct a = q4k_load_act(s_qs + ab * 256, s_d[ab], s_bsums + ab * 16, g);
    float gs = 0.0f, us = 0.0f;
    if (live) {
        gs = q4k_dot(q4k_prepare(rg, g), a);
        us = q4k_dot(q4k_prepare(ru, g), a);
    }
    gs = seg_sum<kLanesPerRow>(gs);
    us = seg_sum<kLanesPerRow>(us);
    // crates/rnb-cpu/src/kernels/activation.rs:73-89
    if (sub == kLanesPerRow - 1 && row < n_ff) mid[static_cast<size_t>(slot) * n_ff + row] = act_mul<false>(gs, us);
}

// kRows: output rows per wave, one after the other against the same quantised intermediates.  A workgroup's set-up (its
// token's intermediates read and quantised: 24 KB and 24 blocks for eight slots of 768) is repeated by every workgroup
// of the token, so calls of several tokens, whose grids are large anyway, take more rows per workgroup.
template <uint32_t kQuant, int kGroups, bool kOne, int kRows>
__global__ void __launch_bounds__(kWave *kDecodeWaves)
    moe_decode_down_kernel(const uint8_t *__restrict__ down_all, const uint8_t *__restrict__ down_shared, uint32_t n_routed,
                           const float *__restrict__ mid, const MoeDecodeTable table,
                           float *__restrict__ out, uint32_t n_embd, uint32_t nb) {
    constexpr int kLanes = kWave / kGroups;  // lanes per (slot, row) pair
    constexpr int kSpans = 64 / kDecodeWaves;
    using Q = KQuant<kQuant>;
    constexpr size_t kBlockBytes = Q::kBytes;
    __shared__ __attribute__((aligned(16))) int8_t s_qs[64 * 256];
    __shared__ float s_d[64];
    __shared__ __attribute__((aligned(16))) int16_t s_bsums[64 * 16];
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t row0 = (blockIdx.x * kDecodeWaves + wave) * kRows;
    const int sub = lane & (kLanes - 1);
    const uint32_t grp = lane / kLanes;
    const int g = sub & 3;
    const uint32_t b = sub >> 2;
    const uint32_t tok = blockIdx.y;
    const uint32_t first = kOne ? 0 : table.tok_off[tok];
    const uint32_t n_slots = kOne ? table.n_slots : table.tok_off[tok + 1] - first, n_blocks = n_slots * nb;
    mid += static_cast<size_t>(first) * nb * 256;  // this token's slots: k below counts from `first`
    const size_t row_bytes = static_cast<size_t>(nb) * kBlockBytes;
    // the intermediates first, then the weights of the first row's first kGroups slots, then the quantisation
    float4 mv[kSpans];
#pragma unroll
    for (int i = 0; i < kSpans; i++) {
        const uint32_t blk = wave + i * kDecodeWaves;
        mv[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (blk < n_blocks) mv[i] = reinterpret_cast<const float4 *>(mid + static_cast<size_t>(blk) * 256)[lane];
    }
    // The token's expert ids and route weights go to LDS once: the table is a kernel argument, and a look-up by a lane's
    // slot is a vector load from it that the compiler waits for together with every other load of the wave (the next
    // slots' weights were only requested once the current ones had arrived, and each route weight cost a round trip).
    // (Wave-uniform scalar look-ups with a select per lane instead of this copy measured slower.)
    __shared__ uint32_t s_expert[kMoeDecodeMaxPerToken];
    __shared__ float s_route[kMoeDecodeMaxPerToken];
    // (every thread reads an entry, together with the first two steps' expert ids below and in front of the first weight
    // request: one wait for all table reads; the copy itself is written behind that request)
    const uint32_t stage_at = first + (threadIdx.x < n_slots ? threadIdx.x : 0);
    const uint32_t stage = stage_at < kMoeDecodeMaxSlots ? stage_at : 0;  // a last token without slots: first = the slot count
    const uint32_t stage_expert = table.expert[stage];
    const float stage_route = table.route[stage];
    // slot k of row `row`; past the token's slots the walk goes on with the next row's first slots
    auto fetch_of = [&](uint32_t row, uint32_t k, uint32_t expert, bool *ok) {
        *ok = b < nb && row < n_embd && k < n_slots;
        const uint8_t *blk = down_all;  // dead lanes read the first block of the tensor
        if (*ok)
            blk = expert_base(down_all, down_shared, n_routed, expert, n_embd * row_bytes) +
                  static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b) * kBlockBytes;
        return Q::load_block_even(blk, g);  // the launcher has checked the tensors' addresses
    };
    if (n_slots == 0) {  // workgroup-uniform: a token without slots gets zero rows
        if (lane == 0) {
            for (int r = 0; r < kRows; r++)
                if (row0 + r < n_embd) out[static_cast<size_t>(tok) * n_embd + row0 + r] = 0.0f;
        }
        return;
    }
    // The wave's work is a sequence of steps, one group of kGroups slots of one row each, rows in order.  Two register
    // sets take turns over the steps, each requested again as soon as its step is reduced (handing a look-ahead set
    // over to "the current one" would be a copy, and a copy waits for the loads it copies).  The first two steps read
    // their expert ids from the table itself, both before the first weight request (a look-up behind it would wait
    // for the weights too); the later ones read the LDS copy.
    const uint32_t n_groups = (n_slots + kGroups - 1) / kGroups, total = kRows * n_groups;
    const uint32_t k1 = n_groups > 1 ? kGroups + grp : grp;                           // step 1: the row's second group,
    const uint32_t row1 = n_groups > 1 ? row0 : (kRows > 1 ? row0 + 1 : n_embd);      // or the next row's first one
    const uint32_t e0 = table.expert[first + (grp < n_slots ? grp : 0)], e1 = table.expert[first + (k1 < n_slots ? k1 : 0)];
    bool ok0, ok1;
    typename Q::Regs s0 = fetch_of(row0, grp, e0, &ok0), s1;
    if (threadIdx.x < n_slots) {
        s_expert[threadIdx.x] = stage_expert;
        s_route[threadIdx.x] = stage_route;
    }
#pragma unroll
    for (int i = 0; i < kSpans; i++) {
        const uint32_t blk = wave + i * kDecodeWaves;
        if (blk < n_blocks) q8k_quantize_vals(mv[i], lane, s_qs + blk * 256, s_d + blk, s_bsums + blk * 16);
    }
    s1 = fetch_of(row1, k1, e1, &ok1);
    __syncthreads();
    // the request cursor stands at step 2, the reduce cursor at step 0 (row index and first slot of the group)
    uint32_t fr = 0, fk0 = 0, cr = 0, ck0 = 0;
    auto advance = [&](uint32_t &r, uint32_t &k0) {
        k0 += kGroups;
        if (k0 >= n_slots) {
            k0 = 0;
            r++;
        }
    };
    advance(fr, fk0);
    advance(fr, fk0);
    auto fetch_next = [&](bool *ok) {  // past the last step: dead lanes' block
        const uint32_t k = fk0 + grp;
        const typename Q::Regs r = fetch_of(fr < static_cast<uint32_t>(kRows) ? row0 + fr : n_embd, k, s_expert[k < n_slots ? k : 0], ok);
        advance(fr, fk0);
        return r;
    };
    float acc = 0.0f;
    auto reduce = [&](const typename Q::Regs &regs, bool ok) {
        const uint32_t k = ck0 + grp;
        float o = 0.0f;
        if (ok) {
            const uint32_t ab = k * nb + b;
            o = kquant_partial<kQuant>(regs, Q::load_act(s_qs + ab * 256, s_d[ab], s_bsums + ab * 16, g), g);
        }
        o = seg_sum<kLanes>(o);
        if (k < n_slots) o *= s_route[k];  // fanout.rs:306-308; only the group's last lane is read below
#pragma unroll
        for (int j = 0; j < kGroups; j++) {
            const float v = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, o), j * kLanes + kLanes - 1));
            if (ck0 + j < n_slots) acc += v;  // wave-uniform
        }
        if (ck0 + kGroups >= n_slots) {  // the row's last group
            if (lane == 0 && row0 + cr < n_embd) out[static_cast<size_t>(tok) * n_embd + row0 + cr] = acc;
            acc = 0.0f;
        }
        advance(cr, ck0);
    };
    // while both sets have a step left to request the requests are unconditional (the compiler's wait counts follow the
    // issue order of the worst path); the last one to three steps are code of their own
    uint32_t s = 0;
    for (; s + 3 < total; s += 2) {
        reduce(s0, ok0);
        s0 = fetch_next(&ok0);
        reduce(s1, ok1);
        s1 = fetch_next(&ok1);
    }
    if (total - s == 3) {
        reduce(s0, ok0);
        s0 = fetch_next(&ok0);
        reduce(s1, ok1);
        reduce(s0, ok0);
    } else {
        reduce(s0, ok0);
        if (total - s == 2) reduce(s1, ok1);
    }
}

// out[token] = sum of its slots' rows in list (= rank) order.  A thread owns four consecutive columns (n_embd is a
// multiple of 256) and requests the rows of up to eight slots before the first addition: the additions keep the list
// order, the loads no longer wait for one another.
__global__ void __launch_bounds__(256)
    moe_reduce_kernel(const float *__restrict__ slot_out, const uint32_t *__restrict__ tok_offsets,
                      const uint32_t *__restrict__ tok_slots, float *__restrict__ out, uint32_t n_embd) {
    const uint32_t tok = blockIdx.y;
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i >= n_embd) return;
    const uint32_t begin = tok_offsets[tok], end = tok_offsets[tok + 1];
    float4 acc = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (uint32_t k0 = begin; k0 < end; k0 += 8) {
        float4 v[8];
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const uint32_t k = min(k0 + j, end - 1);
            v[j] = *reinterpret_cast<const float4 *>(slot_out + static_cast<size_t>(tok_slots[k]) * n_embd + i);
        }
#pragma unroll
        for (int j = 0; j < 8; j++) {
            if (k0 + j < end) {
                acc.x += v[j].x;
                acc.y += v[j].y;
                acc.z += v[j].z;
                acc.w += v[j].w;
            }
        }
    }
    *reinterpret_cast<float4 *>(out + static_cast<size_t>(tok) * n_embd + i) = acc;
}

struct TilePlan {
    uint32_t iters, tmax, tiles;
    size_t lds_bytes;
};

// rows per workgroup = 4 waves * rows_per_wave * iters; keep >= ~2048 workgroups in flight when the
// problem allows it, and at most 48 KiB of staged activations
TilePlan plan_tiles(uint32_t rows, uint32_t nb, uint32_t n_groups, int rows_per_wave) {
    TilePlan p;
    const uint32_t per_pass = kWavesPerWg * static_cast<uint32_t>(rows_per_wave);
    const uint64_t passes_total = static_cast<uint64_t>((rows + per_pass - 1) / per_pass) * n_groups;
    uint32_t iters = static_cast<uint32_t>(passes_total / 2048);
    p.iters = iters < 1 ? 1 : (iters > 8 ? 8 : iters);
    const size_t per_token = static_cast<size_t>(nb) * (kStageBlk + 36);
    uint32_t tmax = static_cast<uint32_t>((48 * 1024) / per_token);
    p.tmax = tmax < 1 ? 1 : (tmax > kMaxChunkTokens ? kMaxChunkTokens : tmax);
    p.lds_bytes = stage_bytes(p.tmax, nb);
    p.tiles = (rows + per_pass * p.iters - 1) / (per_pass * p.iters);
    return p;
}

int rows_per_wave_for(uint32_t nb) { return nb <= 4 ? 4 : (nb <= 8 ? 2 : 1); }

// LAUNCH(format id, rows or slots per wave) for a run-time K-quant id (Q4_K, Q5_K or Q6_K; callers have
// validated it) and a run-time 4 / 2 / 1 split
#define RNB_DISPATCH_KQUANT_R(Q, rpw, LAUNCH) \
    do {                                      \
        if ((rpw) == 4)                       \
            LAUNCH(Q, 4);                     \
        else if ((rpw) == 2)                  \
            LAUNCH(Q, 2);                     \
        else                                  \
            LAUNCH(Q, 1);                     \
    } while (0)
#define RNB_DISPATCH_KQUANT(quant, rpw, LAUNCH)          \
    do {                                                 \
        if ((quant) == kQ6K)                             \
            RNB_DISPATCH_KQUANT_R(kQ6K, rpw, LAUNCH);    \
        else if ((quant) == kQ5K)                        \
            RNB_DISPATCH_KQUANT_R(kQ5K, rpw, LAUNCH);    \
        else                                             \
            RNB_DISPATCH_KQUANT_R(kQ4K, rpw, LAUNCH);    \
    } while (0)

}  // namespace

void launch_moe_gate_up(const uint8_t *gate_all, const uint8_t *up_all, const MoeShared &shared, ActView act, MoeGroups groups,
                        float *mid, uint32_t n_ff, uint32_t nb_in, hipStream_t stream) {
    if (groups.n_groups == 0) return;
    const int rpw = rows_per_wave_for(nb_in);
    const TilePlan p = plan_tiles(n_ff, nb_in, groups.n_groups, rpw);
    const dim3 grid(p.tiles, groups.n_groups, 1), block(kWave * kWavesPerWg);
    // staged activations, then one (gate, up) exchange slot per wave, staged token and row
    const size_t lds_bytes = p.lds_bytes + kWavesPerWg * kMaxChunkTokens * 4 * sizeof(float2);
#define RNB_LAUNCH_GU(R)                                                                                             \
    hipLaunchKernelGGL(moe_gate_up_kernel<R>, grid, block, lds_bytes, stream, gate_all, up_all, shared.gate, shared.up, \
                       shared.n_routed, act.qs, act.d, act.bsums, groups.expert, groups.start, groups.sorted_slot, groups.sorted_token, mid, n_ff,   \
                       nb_in, p.iters, p.tmax)
    if (rpw == 4)
        RNB_LAUNCH_GU(4);
    else if (rpw == 2)
        RNB_LAUNCH_GU(2);
    else
        RNB_LAUNCH_GU(1);
#undef RNB_LAUNCH_GU
}

// every workgroup of an expert group repeats the quantisation of the group's rows: worth it for short intermediates
bool moe_down_quantises(uint32_t nb_mid) { return nb_mid <= 8; }

void launch_moe_down(const uint8_t *down_all, const MoeShared &shared, uint32_t down_quant, ActView mid_act,
                     const float *mid_f32, MoeGroups groups, const float *slot_route, float *slot_out, uint32_t n_embd, uint32_t nb_mid, hipStream_t stream) {
    if (groups.n_groups == 0) return;
    const int rpw = rows_per_wave_for(nb_mid);
    const TilePlan p = plan_tiles(n_embd, nb_mid, groups.n_groups, rpw);
    const dim3 grid(p.tiles, groups.n_groups, 1), block(kWave * kWavesPerWg);
#define RNB_LAUNCH_DOWN(Q, R)                                                                                             \
    hipLaunchKernelGGL((moe_down_kernel<Q, R, false>), grid, block, p.lds_bytes, stream, down_all, shared.down,           \
                       shared.n_routed, mid_act.qs, mid_act.d, mid_act.bsums, nullptr, groups.expert, groups.start, groups.sorted_slot, slot_route, slot_out,     \
                       n_embd, nb_mid, p.iters, p.tmax)
#define RNB_LAUNCH_DOWN_F32(Q, R)                                                                                         \
    hipLaunchKernelGGL((moe_down_kernel<Q, R, true>), grid, block, p.lds_bytes, stream, down_all, shared.down,            \
                       shared.n_routed, nullptr, nullptr, nullptr, mid_f32, groups.expert, groups.start, groups.sorted_slot, slot_route, slot_out, n_embd,   \
                       nb_mid, p.iters, p.tmax)
    if (mid_f32 != nullptr)
        RNB_DISPATCH_KQUANT(down_quant, rpw, RNB_LAUNCH_DOWN_F32);
    else
        RNB_DISPATCH_KQUANT(down_quant, rpw, RNB_LAUNCH_DOWN);
#undef RNB_LAUNCH_DOWN_F32
#undef RNB_LAUNCH_DOWN
}

void launch_moe_down_token(const uint8_t *down_all, const MoeShared &shared, uint32_t down_quant, ActView mid_act, const uint32_t *tok_offsets,
                           const uint32_t *tok_slots, const uint32_t *slot_expert, const float *slot_route, float *out,
                           uint32_t token_count, uint32_t n_embd, uint32_t nb_mid, hipStream_t stream) {
    if (token_count == 0) return;
    const dim3 grid((n_embd + kWavesPerWg - 1) / kWavesPerWg, token_count, 1), block(kWave * kWavesPerWg);
#define RNB_LAUNCH_DT(Q, G)                                                                                           \
    hipLaunchKernelGGL((moe_down_token_kernel<Q, G>), grid, block, 0, stream, down_all, shared.down, shared.n_routed, \
                       mid_act.qs, mid_act.d, mid_act.bsums, tok_offsets, tok_slots, slot_expert, slot_route, out, n_embd, nb_mid)
    RNB_DISPATCH_KQUANT(down_quant, rows_per_wave_for(nb_mid), RNB_LAUNCH_DT);
#undef RNB_LAUNCH_DT
}

bool moe_decode_supported(size_t n_tokens, size_t n_slots, size_t max_per_token, size_t nb_in, size_t nb_mid, const void *x,
                          uint32_t down_quant, const void *down, const void *down_shared) {
    // the down kernel fetches Q6_K blocks without the odd-address path
    if (down_quant == kQ6K && ((reinterpret_cast<uintptr_t>(down) | reinterpret_cast<uintptr_t>(down_shared)) & 1u) != 0) return false;
    return n_tokens >= 1 && n_tokens <= kMoeDecodeMaxTokens && n_slots >= 1 && n_slots <= kMoeDecodeMaxSlots &&
           max_per_token <= kMoeDecodeMaxPerToken && nb_in >= 1 && nb_in <= 16 && nb_mid >= 1 && nb_mid <= 16 &&
           max_per_token * nb_mid <= 64 && reinterpret_cast<uintptr_t>(x) % 16 == 0;
}

void launch_moe_decode(const uint8_t *gate_all, const uint8_t *up_all, const uint8_t *down_all, const MoeShared &shared,
                       uint32_t down_quant, const MoeDecodeTable &table, const float *x, float *mid, float *out, uint32_t n_ff, uint32_t n_embd,
                       uint32_t nb_in, uint32_t nb_mid, hipStream_t stream) {
    const dim3 block(kWave * kDecodeWaves);
    {
        const int rpw = rows_per_wave_for(nb_in);
        const uint32_t row_groups = (n_ff + rpw - 1) / rpw;
        const dim3 grid((row_groups + kDecodeWaves - 1) / kDecodeWaves, table.n_slots, 1);
#define RNB_LAUNCH_DGU1(Q, R)                                                                                      \
    hipLaunchKernelGGL((moe_decode_gate_up_kernel<R, true>), grid, block, 0, stream, gate_all, up_all, shared.gate, \
                       shared.up, shared.n_routed, x, table, mid, n_ff, nb_in)
#define RNB_LAUNCH_DGU(Q, R)                                                                                        \
    hipLaunchKernelGGL((moe_decode_gate_up_kernel<R, false>), grid, block, 0, stream, gate_all, up_all, shared.gate, \
                       shared.up, shared.n_routed, x, table, mid, n_ff, nb_in)
        if (table.n_tokens == 1)
            RNB_DISPATCH_KQUANT_R(kQ4K, rpw, RNB_LAUNCH_DGU1);
        else
            RNB_DISPATCH_KQUANT_R(kQ4K, rpw, RNB_LAUNCH_DGU);
#undef RNB_LAUNCH_DGU
#undef RNB_LAUNCH_DGU1
    }
    // one token: a row per wave; several tokens: kMultiRows rows per wave
    constexpr int kMultiRows = 2;  // 128 experts x top-8, four tokens: 1 / 2 / 4 rows 15.5 / 14.2 / 15.7 us
    const uint32_t rows_per_wg = kDecodeWaves * (table.n_tokens == 1 ? 1 : kMultiRows);
    const dim3 grid((n_embd + rows_per_wg - 1) / rows_per_wg, table.n_tokens, 1);
#define RNB_LAUNCH_DD1(Q, G)                                                                                     \
    hipLaunchKernelGGL((moe_decode_down_kernel<Q, G, true, 1>), grid, block, 0, stream, down_all, shared.down,    \
                       shared.n_routed, mid, table, out, n_embd, nb_mid)
#define RNB_LAUNCH_DD(Q, G)                                                                                       \
    hipLaunchKernelGGL((moe_decode_down_kernel<Q, G, false, kMultiRows>), grid, block, 0, stream, down_all,       \
                       shared.down, shared.n_routed, mid, table, out, n_embd, nb_mid)
    if (table.n_tokens == 1)
        RNB_DISPATCH_KQUANT(down_quant, rows_per_wave_for(nb_mid), RNB_LAUNCH_DD1);
    else
        RNB_DISPATCH_KQUANT(down_quant, rows_per_wave_for(nb_mid), RNB_LAUNCH_DD);
#undef RNB_LAUNCH_DD
#undef RNB_LAUNCH_DD1
}

void launch_moe_reduce(const float *slot_out, const uint32_t *tok_offsets, const uint32_t *tok_slots, float *out,
                       uint32_t token_count, uint32_t n_embd, hipStream_t stream) {
    if (token_count == 0) return;
    dim3 grid((n_embd / 4 + 255) / 256, token_count, 1);
    hipLaunchKernelGGL(moe_reduce_kernel, grid, dim3(256), 0, stream, slot_out, tok_offsets, tok_slots, out, n_embd);
}

}  // namespace rnb
