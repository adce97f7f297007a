// Wave-level activation quantisers, bit-exact with rnb-cpu: one wave64
// quantises one 256-element span (one Q8_K block, or eight 32-wide Q8 blocks); each lane owns four
// consecutive elements.  Single IEEE multiplies and correctly rounded divisions only
// (-ffp-contract=off), see quantize_act.hip.
//
//  Q8_K: crates/rnb-cpu/src/gemm/activation_q8.rs:149-173 (quantize_q8k_block_ggml)
//  Q8  : crates/rnb-cpu/src/gemm/activation_q8.rs:14-32   (quantize_input_q8)
#pragma once

#include "device_utils.h"

namespace rnb {

// Quantises x_blk[0..256) to one Q8_K block: qs (256 int8, 16-byte aligned), *d_out, bsums (16 int16).
// Must be called by all 64 lanes of the wave.
// `v` = this lane's four consecutive elements (x_blk[4*lane .. 4*lane+4)), already loaded.
// `digits` (optional, 16 bytes) receives the 32-element sums split as b0 + 64*b1: b0[0..8) then b1[0..8).
__device__ __forceinline__ void q8k_quantize_vals(const float4 v, int lane, int8_t *qs, float *d_out, int16_t *bsums,
                                                  uint8_t *digits = nullptr) {
    const float e[4] = {v.x, v.y, v.z, v.w};
    // max |x| of the span: per lane, then across the wave on the DPP path (lane 63 ends up with the maximum)
    const float ax[4] = {fabsf(e[0]), fabsf(e[1]), fabsf(e[2]), fabsf(e[3])};
    float lmax = fmaxf(fmaxf(ax[0], ax[1]), fmaxf(ax[2], ax[3]));
    lmax = dpp_max<0xB1, 0xf>(lmax);   // quad_perm [1,0,3,2]
    lmax = dpp_max<0x4E, 0xf>(lmax);   // quad_perm [2,3,0,1]
    lmax = dpp_max<0x141, 0xf>(lmax);  // row_half_mirror
    lmax = dpp_max<0x140, 0xf>(lmax);  // row_mirror
    lmax = dpp_max<0x142, 0xa>(lmax);  // row_bcast15
    lmax = dpp_max<0x143, 0xc>(lmax);  // row_bcast31
    const float amax = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, lmax), 63));
    // the element that attains it first in index order: lowest lane with a match, lowest element inside that lane
    const bool hit[4] = {ax[0] == amax, ax[1] == amax, ax[2] == amax, ax[3] == amax};
    const unsigned long long lanes = __builtin_amdgcn_ballot_w64(hit[0] || hit[1] || hit[2] || hit[3]);
    // amax is one of the |x| unless every comparison failed (a block of NaNs: the reference's `ax > amax` is never
    // true either, it keeps amax = 0 and writes d = 0 with all-zero codes)
    const int first_lane = lanes != 0 ? __builtin_ctzll(lanes) : 0;
    const float mine = hit[0] ? e[0] : hit[1] ? e[1] : hit[2] ? e[2] : e[3];
    const float max_val = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), first_lane));
    float iscale = 0.0f, d = 0.0f;
    if (lanes != 0 && amax != 0.0f) {
        iscale = -127.0f / max_val;
        d = 1.0f / iscale;
    }
    int part = 0;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float prod = iscale * e[i];
        int r = __float2int_rn(prod);  // round half to even
        r = r > 127 ? 127 : r;         // upper clamp only
        const int q = static_cast<int>(static_cast<int8_t>(r));
        part += q;
        packed |= (static_cast<uint32_t>(q) & 0xffu) << (8 * i);
    }
    reinterpret_cast<uint32_t *>(qs)[lane] = packed;
    // 4 lanes = 16 consecutive elements: two quad permutes leave the sum in every lane of the quad
    int sum16 = part + __builtin_amdgcn_update_dpp(0, part, 0xB1, 0xf, 0xf, false);
    sum16 += __builtin_amdgcn_update_dpp(0, sum16, 0x4E, 0xf, 0xf, false);
    if ((lane & 3) == 0) bsums[lane >> 2] = static_cast<int16_t>(sum16);
    if (lane == 0) *d_out = d;
    if (digits != nullptr) {  // wave-uniform
        const int sum32 = sum16 + __shfl_xor(sum16, 4, kWave);       // every lane of an 8-lane group
        const int mine = __shfl(sum32, 8 * (lane & 7), kWave);       // lanes 0..15: sum of sub-block lane % 8
        if (lane < 16) digits[lane] = static_cast<uint8_t>(lane < 8 ? (mine & 63) : (mine >> 6));
    }
}

__device__ __forceinline__ void q8k_quantize_span(const float *__restrict__ x_blk, int lane, int8_t *qs, float *d_out,
                                                  int16_t *bsums, uint8_t *digits = nullptr) {
    q8k_quantize_vals(reinterpret_cast<const float4 *>(x_blk)[lane], lane, qs, d_out, bsums, digits);
}

// A workgroup of kWaves waves quantises one token of at most 16 Q8_K blocks into its LDS (qs[nb][256], d[nb],
// bsums[nb][16]): wave `wave` takes blocks wave, wave + kWaves, ...  The loads are a call of their own so that a
// kernel can request the token before its first weights and quantise after them.
template <int kWaves>
struct TokenSpans {
    float4 v[16 / kWaves];
};
template <int kWaves>
__device__ __forceinline__ void token_load(const float *__restrict__ x_tok, uint32_t nb, uint32_t wave, int lane,
                                           TokenSpans<kWaves> &xv) {
#pragma unroll
    for (int i = 0; i < 16 / kWaves; i++) {
        const uint32_t blk = wave + i * kWaves;
        xv.v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (blk < nb) xv.v[i] = reinterpret_cast<const float4 *>(x_tok + static_cast<size_t>(blk) * 256)[lane];
    }
}
template <int kWaves>
__device__ __forceinline__ void token_quantize(const TokenSpans<kWaves> &xv, uint32_t nb, uint32_t wave, int lane,
                                               int8_t *s_qs, float *s_d, int16_t *s_bsums) {
#pragma unroll
    for (int i = 0; i < 16 / kWaves; i++) {
        const uint32_t blk = wave + i * kWaves;
        if (blk < nb) q8k_quantize_vals(xv.v[i], lane, s_qs + blk * 256, s_d + blk, s_bsums + blk * 16);
    }
}

// Quantises x_span[0..256) to eight 32-wide Q8 blocks (8 lanes per block); lanes whose block index
// (lane / 8) is >= live_blocks neither read nor write.
__device__ __forceinline__ float4 q8_load_span(const float *__restrict__ x_span, int lane, int live_blocks) {
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if ((lane >> 3) < live_blocks) v = reinterpret_cast<const float4 *>(x_span)[lane];
    return v;
}

__device__ __forceinline__ void q8_quantize_vals(const float4 v, int lane, int live_blocks, int8_t *qs, float *d_out) {
    const bool live = (lane >> 3) < live_blocks;
    const float e[4] = {v.x, v.y, v.z, v.w};
    float amax = fmaxf(fmaxf(fabsf(e[0]), fabsf(e[1])), fmaxf(fabsf(e[2]), fabsf(e[3])));
#pragma unroll
    for (int off = 4; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, kWave));
    amax = fmaxf(amax, 0.0f);  // a block of NaNs: the reference's fold starts from 0.0 and f32::max ignores NaN
    const float d = amax / 127.0f;
    const float id = (d != 0.0f) ? 1.0f / d : 0.0f;
    uint32_t packed = 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const float prod = e[i] * id;
        float r = roundf(prod);  // half away from zero
        r = fminf(fmaxf(r, -128.0f), 127.0f);
        r = prod != prod ? 0.0f : r;  // NaN (a NaN input, or inf * 0): the reference's NaN.clamp(..) as i8 is 0
        packed |= (static_cast<uint32_t>(static_cast<int>(r)) & 0xffu) << (8 * i);
    }
    if (live) {
        reinterpret_cast<uint32_t *>(qs)[lane] = packed;
        if ((lane & 7) == 0) d_out[lane >> 3] = d;
    }
}

__device__ __forceinline__ void q8_quantize_span(const float *__restrict__ x_span, int lane, int live_blocks, int8_t *qs,
                                                 float *d_out) {
    q8_quantize_vals(q8_load_span(x_span, lane, live_blocks), lane, live_blocks, qs, d_out);
}

}  // namespace rnb
