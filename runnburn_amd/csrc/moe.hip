// Gathered sparse-MoE expert path (Qwen3-MoE style): per routed slot (token, expert, weight)
//   mid   = silu(W_gate[e] . Q8_K(h)) * (W_up[e] . Q8_K(h))      Q4_K rows, K = n_embd
//   o     = route * (W_down[e] . Q8_K(mid))                       Q4_K | Q6_K rows, K = n_ff
//   out[token] = sum of o over the token's slots in slot order
// following crates/rnb-llm/src/engine/models/shared_expert_moe/moe_view/fanout.rs:260-327
// (compute_expert_host_from_slices), crates/rnb-cpu/src/kernels/activation.rs:73-89
// (fused_silu_mul_inplace) and .../shared_expert_moe/prefill_cpu.rs:167-194 (ordered reduce).
// Expert weights are never copied: a slot addresses its expert as base + e * bytes_per_expert,
// the slicing of fanout.rs:4-22.
#include "block_dots.h"
#include "device_utils.h"
#include "kernels.h"

namespace rnb {

namespace {

constexpr int kRowsPerWg = 4;

__global__ void __launch_bounds__(kWave *kRowsPerWg)
    moe_gate_up_kernel(const uint8_t *__restrict__ gate_all, const uint8_t *__restrict__ up_all,
                       const int8_t *__restrict__ aq, const float *__restrict__ ad, const int16_t *__restrict__ abs,
                       const uint32_t *__restrict__ slot_expert, const uint32_t *__restrict__ slot_token,
                       float *__restrict__ mid, uint32_t n_ff, uint32_t nb) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
    const uint32_t slot = blockIdx.y;
    if (row >= n_ff) return;
    const size_t row_bytes = static_cast<size_t>(nb) * kQ4KBytes;
    const size_t off = (static_cast<size_t>(slot_expert[slot]) * n_ff + row) * row_bytes;
    const size_t abase = static_cast<size_t>(slot_token[slot]) * nb;
    const int c = lane & 7;
    float gacc = 0.0f, uacc = 0.0f;
    for (uint32_t b = lane >> 3; b < nb; b += 8) {
        const size_t boff = off + static_cast<size_t>(b) * kQ4KBytes;
        const int8_t *a = aq + (abase + b) * 256;
        const int16_t *bs = abs + (abase + b) * 16;
        const float dx = ad[abase + b];
        gacc += q4k_block_partial(gate_all + boff, a, dx, bs, c);
        uacc += q4k_block_partial(up_all + boff, a, dx, bs, c);
    }
    gacc = wave_sum(gacc);
    uacc = wave_sum(uacc);
    if (lane == 0) {
        // crates/rnb-cpu/src/kernels/activation.rs:73-89: (g / (1 + exp(-g))) * up
        const float e = expf(-gacc);
        mid[static_cast<size_t>(slot) * n_ff + row] = (gacc / (1.0f + e)) * uacc;
    }
}

template <bool kDownQ6>
__global__ void __launch_bounds__(kWave *kRowsPerWg)
    moe_down_kernel(const uint8_t *__restrict__ down_all, const int8_t *__restrict__ mq, const float *__restrict__ md,
                    const int16_t *__restrict__ mbs, const uint32_t *__restrict__ slot_expert,
                    const float *__restrict__ slot_route, float *__restrict__ slot_out, uint32_t n_embd, uint32_t nb) {
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t row = blockIdx.x * kRowsPerWg + (threadIdx.x >> 6);
    const uint32_t slot = blockIdx.y;
    if (row >= n_embd) return;
    const size_t blk_bytes = kDownQ6 ? kQ6KBytes : kQ4KBytes;
    const size_t row_bytes = static_cast<size_t>(nb) * blk_bytes;
    const uint8_t *rowp = down_all + (static_cast<size_t>(slot_expert[slot]) * n_embd + row) * row_bytes;
    const size_t abase = static_cast<size_t>(slot) * nb;
    const int sub = lane & 7;
    float acc = 0.0f;
    for (uint32_t b = lane >> 3; b < nb; b += 8) {
        if (kDownQ6)
            acc += q6k_block_partial(rowp + static_cast<size_t>(b) * blk_bytes, mq + (abase + b) * 256, md[abase + b], sub);
        else
            acc += q4k_block_partial(rowp + static_cast<size_t>(b) * blk_bytes, mq + (abase + b) * 256, md[abase + b],
                               mbs + (abase + b) * 16, sub);
    }
    acc = wave_sum(acc);
    if (lane == 0) slot_out[static_cast<size_t>(slot) * n_embd + row] = acc * slot_route[slot];  // fanout.rs:306-308
}

__global__ void __launch_bounds__(256)
    moe_reduce_kernel(const float *__restrict__ slot_out, const uint32_t *__restrict__ tok_offsets,
                      const uint32_t *__restrict__ tok_slots, float *__restrict__ out, uint32_t n_embd) {
    const uint32_t tok = blockIdx.y;
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_embd) return;
    const uint32_t begin = tok_offsets[tok], end = tok_offsets[tok + 1];
    float acc = 0.0f;
    for (uint32_t k = begin; k < end; k++) acc += slot_out[static_cast<size_t>(tok_slots[k]) * n_embd + i];
    out[static_cast<size_t>(tok) * n_embd + i] = acc;
}

}  // namespace

void launch_moe_gate_up(const uint8_t *gate_all, const uint8_t *up_all, ActView act, MoeSlots slots, float *mid,
                        uint32_t n_ff, uint32_t nb_in, hipStream_t stream) {
    if (slots.n_slots == 0) return;
    dim3 grid((n_ff + kRowsPerWg - 1) / kRowsPerWg, slots.n_slots, 1);
    hipLaunchKernelGGL(moe_gate_up_kernel, grid, dim3(kWave * kRowsPerWg), 0, stream, gate_all, up_all, act.qs, act.d,
                       act.bsums, slots.expert, slots.token, mid, n_ff, nb_in);
}

void launch_moe_down(const uint8_t *down_all, uint32_t down_quant, ActView mid_act, MoeSlots slots, float *slot_out,
                     uint32_t n_embd, uint32_t nb_mid, hipStream_t stream) {
    if (slots.n_slots == 0) return;
    dim3 grid((n_embd + kRowsPerWg - 1) / kRowsPerWg, slots.n_slots, 1);
    if (down_quant == kQ6K)
        hipLaunchKernelGGL(moe_down_kernel<true>, grid, dim3(kWave * kRowsPerWg), 0, stream, down_all, mid_act.qs,
                           mid_act.d, mid_act.bsums, slots.expert, slots.route, slot_out, n_embd, nb_mid);
    else
        hipLaunchKernelGGL(moe_down_kernel<false>, grid, dim3(kWave * kRowsPerWg), 0, stream, down_all, mid_act.qs,
                           mid_act.d, mid_act.bsums, slots.expert, slots.route, slot_out, n_embd, nb_mid);
}

void launch_moe_reduce(const float *slot_out, const uint32_t *tok_offsets, const uint32_t *tok_slots, float *out,
                       uint32_t token_count, uint32_t n_embd, hipStream_t stream) {
    if (token_count == 0) return;
    dim3 grid((n_embd + 255) / 256, token_count, 1);
    hipLaunchKernelGGL(moe_reduce_kernel, grid, dim3(256), 0, stream, slot_out, tok_offsets, tok_slots, out, n_embd);
}

}  // namespace rnb
