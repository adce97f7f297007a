// GEMV of the importance-quant formats against Q8_K activations: IQ2_XXS (66-byte blocks), IQ2_S (82), IQ3_XXS (98) and
// IQ4_XS (136), 256 elements a block, every block 2-byte aligned.  The arithmetic is the reference's Q8_K form
// (crates/rnb-cpu/src/gemm/neon_quant.rs:273-411; element layouts crates/rnb-cpu/src/quantize/iq.rs:23-116): exact
// int8 dot products per 32-element group, the group scale, then d * d_x per block in f32.
//   IQ2_XXS  group = 4 grid indices + u32 {4 x 7 sign bits | scale << 28}; value = +-grid byte; d d_x / 4 * sum (0.5 + s) dot
//   IQ2_S    group = 4 low index bytes (+ 2 high bits each in qh), 4 sign bytes, scale nibbles per 16;  d d_x / 8 * sum (1 + 2 s) dot
//   IQ3_XXS  group = 8 grid indices (4 bytes each) + u32 as IQ2_XXS;                                    d d_x / 2 * sum (0.5 + s) dot
//   IQ4_XS   group = 16 bytes of nibbles through the 16-entry table, 6-bit scale - 32;                  d d_x * sum s dot
// Lane mapping as for the K-quants: four lanes per block, lane g owning groups 2g and 2g + 1 (64 consecutive elements),
// sixteen blocks per wave and pass; one wave per row, the lanes' partial sums added on the DPP path.
// The grids are ggml's codebooks, kept packed (a 16-bit word per entry: every byte of an IQ2 entry is one of 8, 25, 43,
// every byte of an IQ3_XXS entry is 4 + 8 c, 62 for c = 7) and expanded at compile time into device tables, which every
// workgroup copies into LDS once (the look-ups are gathers: 14336 x 4096 IQ2_XXS 13.7 -> 9.6 us, IQ3_XXS 19.6 -> 11.2 us
// against tables read through the vector cache); a sign index of seven bits stands for those bits and their parity.
#include <algorithm>

#include "embed_gather.h"
#include "kernels.h"
#include "mfma_blocks.h"

namespace rnb {

namespace {

#include "iq_grids_packed.inc"

struct Grid64x256 { uint64_t v[256]; };
struct Grid64x1024 { uint64_t v[1024]; };
struct Grid32x256 { uint32_t v[256]; };

constexpr uint64_t expand2(uint16_t w) {
    uint64_t v = 0;
    for (int j = 0; j < 8; j++) {
        const uint32_t c = (w >> (2 * j)) & 3;
        v |= static_cast<uint64_t>(c == 0 ? 8 : (c == 1 ? 25 : 43)) << (8 * j);
    }
    return v;
}
constexpr uint32_t expand3(uint16_t w) {
    uint32_t v = 0;
    for (int j = 0; j < 4; j++) {
        const uint32_t c = (w >> (3 * j)) & 7;
        v |= (c == 7 ? 62u : 4u + 8u * c) << (8 * j);
    }
    return v;
}
constexpr Grid64x256 make_iq2xxs() {
    Grid64x256 t{};
    for (int i = 0; i < 256; i++) t.v[i] = expand2(kIq2xxsPacked[i]);
    return t;
}
constexpr Grid64x1024 make_iq2s() {
    Grid64x1024 t{};
    for (int i = 0; i < 1024; i++) t.v[i] = expand2(kIq2sPacked[i]);
    return t;
}
constexpr Grid32x256 make_iq3xxs() {
    Grid32x256 t{};
    for (int i = 0; i < 256; i++) t.v[i] = expand3(kIq3xxsPacked[i]);
    return t;
}
__device__ const Grid64x256 g_iq2xxs = make_iq2xxs();
__device__ const Grid64x1024 g_iq2s = make_iq2s();
__device__ const Grid32x256 g_iq3xxs = make_iq3xxs();

// four bytes of a grid entry with the signs of four bits applied: byte j negated when bit j of `bits` is set (the bytes
// are positive and below 128, so v ^ 0xff plus one never carries into the next byte)
__device__ __forceinline__ uint32_t apply_signs4(uint32_t v, uint32_t bits) {
    const uint32_t m01 = ((bits & 15u) * 0x00204081u) & 0x01010101u;  // bit j -> byte j
    const uint32_t mask = (m01 << 8) - m01;
    return (v ^ mask) + m01;
}
// seven sign bits and their parity
__device__ __forceinline__ uint32_t sign_byte(uint32_t seven) {
    seven &= 127u;
    return seven | ((__builtin_popcount(seven) & 1u) << 7);
}

// the lane's 64 activations: groups 2g and 2g + 1
struct IqAct {
    uint4 a[4];
    float dx;
};
__device__ __forceinline__ IqAct iq_load_act(const int8_t *aq_blk, float dx, int g) {
    IqAct r;
#pragma unroll
    for (int i = 0; i < 4; i++) r.a[i] = *reinterpret_cast<const uint4 *>(aq_blk + 64 * g + 16 * i);
    r.dx = dx;
    return r;
}
__device__ __forceinline__ int dot8(uint32_t lo, uint32_t hi, const uint4 &a, int half, int acc) {
    return half == 0 ? dot4(hi, a.y, dot4(lo, a.x, acc)) : dot4(hi, a.w, dot4(lo, a.z, acc));
}

template <uint32_t kQuant>
struct Iq;

template <>
struct Iq<kIQ2XXS> {
    static constexpr size_t kBytes = kIQ2XXSBytes;
    static constexpr int kTableBytes = 2048;
    static __device__ __forceinline__ const void *table() { return g_iq2xxs.v; }
    // kT tokens against one decoded block: res[t] = this lane's part of token t's dot (per token the one-token arithmetic)
    template <int kT>
    static __device__ __forceinline__ void partial(const uint8_t *blk, const IqAct (&act)[kT], int g, const void *tab,
                                                   float (&res)[kT]) {
        const uint64_t *grid_tab = static_cast<const uint64_t *>(tab);
        const uint4 raw = ld_u4_a2(blk + 2 + 16 * g);  // two groups: {indices, scales and signs} each
        const uint32_t idx[2] = {raw.x, raw.z}, ss[2] = {raw.y, raw.w};
        float fsum[kT];
#pragma unroll
        for (int t = 0; t < kT; t++) fsum[t] = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int isum[kT];
#pragma unroll
            for (int t = 0; t < kT; t++) isum[t] = 0;
#pragma unroll
            for (int l = 0; l < 4; l++) {
                const uint64_t grid = grid_tab[(idx[h] >> (8 * l)) & 0xffu];
                const uint32_t s = sign_byte(ss[h] >> (7 * l));
                const uint32_t lo = apply_signs4(static_cast<uint32_t>(grid), s);
                const uint32_t hi = apply_signs4(static_cast<uint32_t>(grid >> 32), s >> 4);
#pragma unroll
                for (int t = 0; t < kT; t++) isum[t] = dot8(lo, hi, act[t].a[2 * h + (l >> 1)], l & 1, isum[t]);
            }
#pragma unroll
            for (int t = 0; t < kT; t++) fsum[t] += (0.5f + static_cast<float>(ss[h] >> 28)) * static_cast<float>(isum[t]);
        }
        const float d = ld_f16(blk);
#pragma unroll
        for (int t = 0; t < kT; t++) res[t] = d * act[t].dx * 0.25f * fsum[t];
    }
};

template <>
struct Iq<kIQ2S> {
    static constexpr size_t kBytes = kIQ2SBytes;
    static constexpr int kTableBytes = 8192;
    static __device__ __forceinline__ const void *table() { return g_iq2s.v; }
    template <int kT>
    static __device__ __forceinline__ void partial(const uint8_t *blk, const IqAct (&act)[kT], int g, const void *tab,
                                                   float (&res)[kT]) {
        const uint64_t *grid_tab = static_cast<const uint64_t *>(tab);
        const uint2 lowb = ld_u2_a2(blk + 2 + 8 * g), signb = ld_u2_a2(blk + 34 + 8 * g);
        const uint32_t qh2 = *reinterpret_cast<const unsigned short *>(blk + 66 + 2 * g);
        const uint32_t sc2 = *reinterpret_cast<const unsigned short *>(blk + 74 + 2 * g);
        const uint32_t low[2] = {lowb.x, lowb.y}, sg[2] = {signb.x, signb.y};
        int isum[kT];
#pragma unroll
        for (int t = 0; t < kT; t++) isum[t] = 0;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t qh = (qh2 >> (8 * h)) & 0xffu, sc = (sc2 >> (8 * h)) & 0xffu;
            int half_sum[kT][2];
#pragma unroll
            for (int t = 0; t < kT; t++) half_sum[t][0] = half_sum[t][1] = 0;
#pragma unroll
            for (int l = 0; l < 4; l++) {
                const uint32_t index = ((low[h] >> (8 * l)) & 0xffu) | ((qh << (8 - 2 * l)) & 0x300u);
                const uint64_t grid = grid_tab[index];
                const uint32_t s = (sg[h] >> (8 * l)) & 0xffu;
                const uint32_t lo = apply_signs4(static_cast<uint32_t>(grid), s);
                const uint32_t hi = apply_signs4(static_cast<uint32_t>(grid >> 32), s >> 4);
#pragma unroll
                for (int t = 0; t < kT; t++)
                    half_sum[t][l >> 1] = dot8(lo, hi, act[t].a[2 * h + (l >> 1)], l & 1, half_sum[t][l >> 1]);
            }
#pragma unroll
            for (int t = 0; t < kT; t++)
                isum[t] += half_sum[t][0] * static_cast<int>(1 + 2 * (sc & 15u)) + half_sum[t][1] * static_cast<int>(1 + 2 * (sc >> 4));
        }
        const float d = ld_f16(blk);
#pragma unroll
        for (int t = 0; t < kT; t++) res[t] = d * act[t].dx * 0.125f * static_cast<float>(isum[t]);
    }
};

template <>
struct Iq<kIQ3XXS> {
    static constexpr size_t kBytes = kIQ3XXSBytes;
    static constexpr int kTableBytes = 1024;
    static __device__ __forceinline__ const void *table() { return g_iq3xxs.v; }
    template <int kT>
    static __device__ __forceinline__ void partial(const uint8_t *blk, const IqAct (&act)[kT], int g, const void *tab,
                                                   float (&res)[kT]) {
        const uint32_t *grid_tab = static_cast<const uint32_t *>(tab);
        const uint4 idx = ld_u4_a2(blk + 2 + 16 * g);  // eight indices per group, two groups
        const uint2 ssb = ld_u2_a2(blk + 66 + 8 * g);
        const uint32_t iw[4] = {idx.x, idx.y, idx.z, idx.w}, ss[2] = {ssb.x, ssb.y};
        float fsum[kT];
#pragma unroll
        for (int t = 0; t < kT; t++) fsum[t] = 0.0f;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            int isum[kT];
#pragma unroll
            for (int t = 0; t < kT; t++) isum[t] = 0;
#pragma unroll
            for (int l = 0; l < 4; l++) {
                const uint32_t pair = iw[2 * h + (l >> 1)] >> (16 * (l & 1));  // indices 2l and 2l + 1 of the group
                const uint32_t s = sign_byte(ss[h] >> (7 * l));
                const uint32_t lo = apply_signs4(grid_tab[pair & 0xffu], s);
                const uint32_t hi = apply_signs4(grid_tab[(pair >> 8) & 0xffu], s >> 4);
#pragma unroll
                for (int t = 0; t < kT; t++) isum[t] = dot8(lo, hi, act[t].a[2 * h + (l >> 1)], l & 1, isum[t]);
            }
#pragma unroll
            for (int t = 0; t < kT; t++) fsum[t] += (0.5f + static_cast<float>(ss[h] >> 28)) * static_cast<float>(isum[t]);
        }
        const float d = ld_f16(blk);
#pragma unroll
        for (int t = 0; t < kT; t++) res[t] = d * act[t].dx * 0.5f * fsum[t];
    }
};

// four table values for four indices 0..15, one per byte
__device__ __forceinline__ uint32_t iq4nl_lookup(uint32_t idx4) {
    // -127 -104 -83 -65 | -49 -35 -22 -10 | 1 13 25 38 | 53 69 89 113 as bytes, little-endian words
    constexpr uint32_t t0 = 0xbfad9881u, t1 = 0xf6eaddcfu, t2 = 0x26190d01u, t3 = 0x71594535u;
    const uint32_t low3 = idx4 & 0x07070707u;
    const uint32_t below = __builtin_amdgcn_perm(t1, t0, low3), above = __builtin_amdgcn_perm(t3, t2, low3);
    const uint32_t m01 = (idx4 >> 3) & 0x01010101u, mask = (m01 << 8) - m01;
    return (below & ~mask) | (above & mask);
}

template <>
struct Iq<kIQ4XS> {
    static constexpr size_t kBytes = kIQ4XSBytes;
    static constexpr int kTableBytes = 0;
    static __device__ __forceinline__ const void *table() { return nullptr; }
    template <int kT>
    static __device__ __forceinline__ void partial(const uint8_t *blk, const IqAct (&act)[kT], int g, const void *,
                                                   float (&res)[kT]) {
        const uint2 hdr = ld_u2_a2(blk);  // f16 d | scales_h << 16, then scales_l
        const uint4 q0 = ld_u4_a2(blk + 8 + 32 * g), q1 = ld_u4_a2(blk + 24 + 32 * g);
        const uint32_t scales_h = hdr.x >> 16;
        const uint32_t both = (hdr.y >> (8 * g)) & 0xffu;  // scales_l[g]: groups 2g (low nibble) and 2g + 1
        const int s0 = static_cast<int>((both & 15u) | (((scales_h >> (4 * g)) & 3u) << 4)) - 32;
        const int s1 = static_cast<int>((both >> 4) | (((scales_h >> (4 * g + 2)) & 3u) << 4)) - 32;
        const uint32_t w0[4] = {q0.x, q0.y, q0.z, q0.w}, w1[4] = {q1.x, q1.y, q1.z, q1.w};
        int d0[kT], d1[kT];
#pragma unroll
        for (int t = 0; t < kT; t++) d0[t] = d1[t] = 0;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            // byte j of the group: element j (low nibble) and element 16 + j (high nibble)
            const uint32_t c00 = iq4nl_lookup(w0[i] & 0x0f0f0f0fu), c01 = iq4nl_lookup((w0[i] >> 4) & 0x0f0f0f0fu);
            const uint32_t c10 = iq4nl_lookup(w1[i] & 0x0f0f0f0fu), c11 = iq4nl_lookup((w1[i] >> 4) & 0x0f0f0f0fu);
#pragma unroll
            for (int t = 0; t < kT; t++) {
                const uint32_t a0[4] = {act[t].a[0].x, act[t].a[0].y, act[t].a[0].z, act[t].a[0].w};
                const uint32_t a1[4] = {act[t].a[1].x, act[t].a[1].y, act[t].a[1].z, act[t].a[1].w};
                const uint32_t a2[4] = {act[t].a[2].x, act[t].a[2].y, act[t].a[2].z, act[t].a[2].w};
                const uint32_t a3[4] = {act[t].a[3].x, act[t].a[3].y, act[t].a[3].z, act[t].a[3].w};
                d0[t] = dot4(c00, a0[i], d0[t]);
                d0[t] = dot4(c01, a1[i], d0[t]);
                d1[t] = dot4(c10, a2[i], d1[t]);
                d1[t] = dot4(c11, a3[i], d1[t]);
            }
        }
        const float d = f16_bits_to_f32(hdr.x);
#pragma unroll
        for (int t = 0; t < kT; t++) res[t] = d * act[t].dx * static_cast<float>(d0[t] * s0 + d1[t] * s1);
    }
};

// ---- dequantisers of the embedding gather (crates/rnb-cpu/src/quantize/iq.rs:23-116): the group scale first,
// d * (0.5 + s) * 0.25 (IQ3_XXS: * 0.5) or d * (s - 32), then times the signed code -------------------------------
__device__ __forceinline__ uint32_t ld_u32_le(const uint8_t *p) {
    return static_cast<uint32_t>(p[0]) | (static_cast<uint32_t>(p[1]) << 8) | (static_cast<uint32_t>(p[2]) << 16) |
           (static_cast<uint32_t>(p[3]) << 24);
}
// eight bytes of a grid entry, byte j negated when bit j of `signs` is set
__device__ __forceinline__ void signed_codes8(uint64_t grid, uint32_t signs, float db, float (&y)[8]) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int v = static_cast<int>((grid >> (8 * j)) & 0xffu);
        y[j] = db * static_cast<float>((signs >> j) & 1u ? -v : v);
    }
}
struct DqIQ2XXS {  // {f16 d, 8 x {u8 index[4], u32 signs and scale}}
    static constexpr uint32_t kElems = 256, kBytes = kIQ2XXSBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int ib = o >> 2, l = o & 3;
        const uint8_t *packed = blk + 2 + 8 * ib;
        const uint32_t ss = ld_u32_le(packed + 4);
        const float t = ld_f16(blk) * (0.5f + static_cast<float>(ss >> 28));
        signed_codes8(g_iq2xxs.v[packed[l]], sign_byte(ss >> (7 * l)), t * 0.25f, y);
    }
};
struct DqIQ2S {  // {f16 d, u8 index_low[32], u8 signs[32], u8 qh[8], u8 scales[8]}
    static constexpr uint32_t kElems = 256, kBytes = kIQ2SBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int ib = o >> 2, l = o & 3;
        const uint32_t high = (static_cast<uint32_t>(blk[66 + ib]) << (8 - 2 * l)) & 0x300u;
        const uint32_t sc = l < 2 ? (blk[74 + ib] & 0x0fu) : (blk[74 + ib] >> 4);
        const float t = ld_f16(blk) * (0.5f + static_cast<float>(sc));
        signed_codes8(g_iq2s.v[blk[2 + 4 * ib + l] | high], blk[34 + 4 * ib + l], t * 0.25f, y);
    }
};
struct DqIQ3XXS {  // {f16 d, u8 index[64], 8 x u32 signs and scale}
    static constexpr uint32_t kElems = 256, kBytes = kIQ3XXSBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int ib = o >> 2, l = o & 3;
        const uint32_t packed = ld_u32_le(blk + 66 + 4 * ib);
        const float t = ld_f16(blk) * (0.5f + static_cast<float>(packed >> 28));
        const uint64_t grid = static_cast<uint64_t>(g_iq3xxs.v[blk[2 + 8 * ib + 2 * l]]) |
                              (static_cast<uint64_t>(g_iq3xxs.v[blk[2 + 8 * ib + 2 * l + 1]]) << 32);
        signed_codes8(grid, sign_byte(packed >> (7 * l)), t * 0.5f, y);
    }
};
struct DqIQ4XS {  // {f16 d, u16 scales_h, u8 scales_l[4], u8 qs[128]}: byte j of a group = elements j and 16 + j
    static constexpr uint32_t kElems = 256, kBytes = kIQ4XSBytes;
    static __device__ __forceinline__ void octet(const uint8_t *blk, int o, float (&y)[8]) {
        const int ib = o >> 2, m = o & 3;
        const uint32_t scales_h = blk[2] | (static_cast<uint32_t>(blk[3]) << 8);
        const uint32_t low = (blk[4 + ib / 2] >> (4 * (ib % 2))) & 0x0fu, high = ((scales_h >> (2 * ib)) & 3u) << 4;
        const float dl = ld_f16(blk) * (static_cast<float>(low | high) - 32.0f);
        const uint8_t *qs = blk + 8 + 16 * ib + 8 * (m & 1);
        const uint32_t w0 = ld_u32_le(qs) >> (4 * (m >> 1)), w1 = ld_u32_le(qs + 4) >> (4 * (m >> 1));
        const uint32_t c0 = iq4nl_lookup(w0 & 0x0f0f0f0fu), c1 = iq4nl_lookup(w1 & 0x0f0f0f0fu);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            y[j] = dl * static_cast<float>(static_cast<int8_t>((c0 >> (8 * j)) & 0xffu));
            y[4 + j] = dl * static_cast<float>(static_cast<int8_t>((c1 >> (8 * j)) & 0xffu));
        }
    }
};

constexpr int kIqWaves = 4;

// kTokens tokens per pass over the matrix (grid.y = token groups; the last group's spare slots repeat the last token and
// are not stored): a block's codes are looked up and signed once and dotted against every token of the group, which is
// most of the work of these formats; per token the one-token arithmetic, so the same bits.
template <uint32_t kQuant, int kTokens>
__global__ void __launch_bounds__(kWave *kIqWaves)
    gemv_iq_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                   float *__restrict__ out, uint32_t rows, uint32_t nb, uint32_t seq) {
    // the format's grid goes to LDS once per workgroup: the look-ups are gathers, which LDS serves faster than the vector cache
    __shared__ __attribute__((aligned(16))) uint8_t s_table[Iq<kQuant>::kTableBytes > 0 ? Iq<kQuant>::kTableBytes : 16];
    if constexpr (Iq<kQuant>::kTableBytes > 0) {
        const uint4 *src = static_cast<const uint4 *>(Iq<kQuant>::table());
        for (int i = threadIdx.x; i < Iq<kQuant>::kTableBytes / 16; i += kWave * kIqWaves) reinterpret_cast<uint4 *>(s_table)[i] = src[i];
        __syncthreads();
    }
    const int lane = threadIdx.x & (kWave - 1);
    const uint32_t wave = threadIdx.x >> 6;
    const int g = lane & 3;
    const uint32_t tok0 = blockIdx.y * kTokens;
    const size_t row_bytes = static_cast<size_t>(nb) * Iq<kQuant>::kBytes;
    const uint32_t n_waves = gridDim.x * kIqWaves;
    for (uint32_t row = blockIdx.x * kIqWaves + wave; row < rows; row += n_waves) {
        float acc[kTokens];
#pragma unroll
        for (int t = 0; t < kTokens; t++) acc[t] = 0.0f;
        for (uint32_t b = lane >> 2; b < nb; b += 16) {
            IqAct act[kTokens];
#pragma unroll
            for (int t = 0; t < kTokens; t++) {
                const uint32_t tok = tok0 + t < seq ? tok0 + t : seq - 1;
                const size_t ab = static_cast<size_t>(tok) * nb + b;
                act[t] = iq_load_act(aq + ab * 256, ad[ab], g);
            }
            float part[kTokens];
            Iq<kQuant>::template partial<kTokens>(w + static_cast<size_t>(row) * row_bytes + static_cast<size_t>(b) * Iq<kQuant>::kBytes,
                                                  act, g, s_table, part);
#pragma unroll
            for (int t = 0; t < kTokens; t++) acc[t] += part[t];
        }
#pragma unroll
        for (int t = 0; t < kTokens; t++) {
            const float sum = seg_sum<kWave>(acc[t]);
            if (lane == kWave - 1 && tok0 + t < seq) out[static_cast<size_t>(tok0 + t) * rows + row] = sum;
        }
    }
}

template <uint32_t kQuant>
void launch_iq(const uint8_t *w, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq, hipStream_t stream) {
    const uint32_t want = (rows + kIqWaves - 1) / kIqWaves;
    // groups of equal size, at most four tokens each
    const auto [groups, per] = token_groups(seq);
    const dim3 grid(want < 1024 ? want : 1024, groups, 1);  // 4096 waves; every workgroup stages the grid once
#define RNB_LAUNCH_IQ(T) \
    hipLaunchKernelGGL((gemv_iq_kernel<kQuant, T>), grid, dim3(kWave * kIqWaves), 0, stream, w, act.qs, act.d, out, rows, nb, seq)
    if (per == 1)
        RNB_LAUNCH_IQ(1);
    else if (per == 2)
        RNB_LAUNCH_IQ(2);
    else if (per == 3)
        RNB_LAUNCH_IQ(3);
    else
        RNB_LAUNCH_IQ(4);
#undef RNB_LAUNCH_IQ
}

// ---------------------------------------------------------------------------------------------
// Batches on the matrix cores: the scheme of gemm_blocks.hip's Q2_K / Q3_K kernel.  M = token, N = weight row, lane =
// (row lane % 32, K-half lane / 32); one K=16 instruction (v_mfma_i32_32x32x16_i8) per 16 elements, i.e. two per
// 32-element group, the lane supplying the eight signed codes of elements 16 sb + 8 khalf .. + 8: one grid entry
// (IQ2_XXS, IQ2_S), two four-code entries (IQ3_XXS) or eight nibbles through the 16-entry table (IQ4_XS).  The group's
// integer scale goes onto the sixteen results (tot += sc * I, 24-bit multiplies), one f32 update per block:
//   IQ2_XXS, IQ2_S  out += (d / 8) d_x sum (2 s + 1) I      IQ3_XXS  out += (d / 4) d_x sum (2 s + 1) I
//   IQ4_XS          out += d d_x sum (s - 32) I
// which are the reference's sums (crates/rnb-cpu/src/gemm/neon_quant.rs:273-411) with the halves made integers.  The
// tokens' int8 activations are staged in LDS, double-buffered, one barrier per block; the grids sit in LDS as in the
// GEMV.  Small grids cut K into slices (blockIdx.z), summed in slice order by sum_slices_kernel.
// ---------------------------------------------------------------------------------------------
template <uint32_t kQuant>
struct IqRow;

template <>
struct IqRow<kIQ2XXS> {  // 8 x {u8 index[4], u32 signs | scale << 28}
    uint32_t w[16];
    float d;
    __device__ __forceinline__ void load(const uint8_t *blk, int) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint4 v = ld_u4_a2(blk + 2 + 16 * i);
            w[4 * i] = v.x, w[4 * i + 1] = v.y, w[4 * i + 2] = v.z, w[4 * i + 3] = v.w;
        }
        d = ld_f16(blk) * 0.125f;
    }
    template <int kSb>
    __device__ __forceinline__ long operand(int khalf, const void *tab, int *scale) const {
        constexpr int ib = kSb >> 1;
        const int l = 2 * (kSb & 1) + khalf;
        const uint32_t ss = w[2 * ib + 1];
        const uint64_t grid = static_cast<const uint64_t *>(tab)[(w[2 * ib] >> (8 * l)) & 0xffu];
        const uint32_t sg = sign_byte(ss >> (7 * l));
        *scale = static_cast<int>(2 * (ss >> 28) + 1);
        return static_cast<long>(static_cast<uint64_t>(apply_signs4(static_cast<uint32_t>(grid), sg)) |
                                 (static_cast<uint64_t>(apply_signs4(static_cast<uint32_t>(grid >> 32), sg >> 4)) << 32));
    }
};

template <>
struct IqRow<kIQ2S> {  // u8 index_low[32], u8 signs[32], u8 qh[8], u8 scales[8]
    uint32_t w[20];
    float d;
    __device__ __forceinline__ void load(const uint8_t *blk, int) {
#pragma unroll
        for (int i = 0; i < 5; i++) {
            const uint4 v = ld_u4_a2(blk + 2 + 16 * i);
            w[4 * i] = v.x, w[4 * i + 1] = v.y, w[4 * i + 2] = v.z, w[4 * i + 3] = v.w;
        }
        d = ld_f16(blk) * 0.125f;
    }
    template <int kSb>
    __device__ __forceinline__ long operand(int khalf, const void *tab, int *scale) const {
        constexpr int ib = kSb >> 1;
        const int l = 2 * (kSb & 1) + khalf;
        const uint32_t qh = (w[16 + (ib >> 2)] >> (8 * (ib & 3))) & 0xffu, sc = (w[18 + (ib >> 2)] >> (8 * (ib & 3))) & 0xffu;
        const uint32_t index = ((w[ib] >> (8 * l)) & 0xffu) | ((qh << (8 - 2 * l)) & 0x300u);
        const uint64_t grid = static_cast<const uint64_t *>(tab)[index];
        const uint32_t sg = (w[8 + ib] >> (8 * l)) & 0xffu;
        *scale = static_cast<int>(2 * ((kSb & 1) ? (sc >> 4) : (sc & 15u)) + 1);
        return static_cast<long>(static_cast<uint64_t>(apply_signs4(static_cast<uint32_t>(grid), sg)) |
                                 (static_cast<uint64_t>(apply_signs4(static_cast<uint32_t>(grid >> 32), sg >> 4)) << 32));
    }
};

template <>
struct IqRow<kIQ3XXS> {  // u8 index[64], 8 x u32 signs | scale << 28
    uint32_t w[24];
    float d;
    __device__ __forceinline__ void load(const uint8_t *blk, int) {
#pragma unroll
        for (int i = 0; i < 6; i++) {
            const uint4 v = ld_u4_a2(blk + 2 + 16 * i);
            w[4 * i] = v.x, w[4 * i + 1] = v.y, w[4 * i + 2] = v.z, w[4 * i + 3] = v.w;
        }
        d = ld_f16(blk) * 0.25f;
    }
    template <int kSb>
    __device__ __forceinline__ long operand(int khalf, const void *tab, int *scale) const {
        constexpr int ib = kSb >> 1;
        const int l = 2 * (kSb & 1) + khalf;
        const uint32_t packed = w[16 + ib];
        const uint32_t pair = (khalf ? (w[2 * ib + (kSb & 1)] >> 16) : w[2 * ib + (kSb & 1)]) & 0xffffu;  // indices 2 l, 2 l + 1
        const uint32_t *grid = static_cast<const uint32_t *>(tab);
        const uint32_t sg = sign_byte(packed >> (7 * l));
        *scale = static_cast<int>(2 * (packed >> 28) + 1);
        return static_cast<long>(static_cast<uint64_t>(apply_signs4(grid[pair & 0xffu], sg)) |
                                 (static_cast<uint64_t>(apply_signs4(grid[pair >> 8], sg >> 4)) << 32));
    }
};

template <>
struct IqRow<kIQ4XS> {  // u16 scales_h, u8 scales_l[4], u8 qs[128]: byte j of a group = elements j and 16 + j
    uint32_t w[16];  // the lane's eight bytes of every group: bytes 8 khalf .. + 8
    uint32_t scales_h, scales_l;
    float d;
    __device__ __forceinline__ void load(const uint8_t *blk, int khalf) {
        const uint2 hdr = ld_u2_a2(blk);
#pragma unroll
        for (int ib = 0; ib < 8; ib++) {
            const uint2 v = ld_u2_a2(blk + 8 + 16 * ib + 8 * khalf);
            w[2 * ib] = v.x, w[2 * ib + 1] = v.y;
        }
        scales_h = hdr.x >> 16;
        scales_l = hdr.y;
        d = f16_bits_to_f32(hdr.x);
    }
    template <int kSb>
    __device__ __forceinline__ long operand(int, const void *, int *scale) const {
        constexpr int ib = kSb >> 1, h = kSb & 1;
        *scale = static_cast<int>(((scales_l >> (4 * ib)) & 15u) | (((scales_h >> (2 * ib)) & 3u) << 4)) - 32;
        return static_cast<long>(static_cast<uint64_t>(iq4nl_lookup((w[2 * ib] >> (4 * h)) & 0x0f0f0f0fu)) |
                                 (static_cast<uint64_t>(iq4nl_lookup((w[2 * ib + 1] >> (4 * h)) & 0x0f0f0f0fu)) << 32));
    }
};

template <uint32_t kQuant, int kTT>
__global__ void __launch_bounds__(kGbThreads, 2)
    gemm_iq_mfma_kernel(const uint8_t *__restrict__ w, const int8_t *__restrict__ aq, const float *__restrict__ ad,
                        float *__restrict__ out, uint32_t rows, uint32_t nb, uint32_t seq, uint32_t nb_slice) {
    constexpr int kToks = 32 * kTT;
    constexpr size_t kBlockBytes = Iq<kQuant>::kBytes;
    __shared__ __attribute__((aligned(16))) uint8_t s_a[2][kToks * kGbStride64];
    __shared__ __attribute__((aligned(16))) float s_dx[2][kToks];
    __shared__ __attribute__((aligned(16))) uint8_t s_table[Iq<kQuant>::kTableBytes > 0 ? Iq<kQuant>::kTableBytes : 16];
    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid >> 6;
    const int lrow = lane & 31, khalf = lane >> 5;
    const uint32_t row = blockIdx.x * kGbRows + wave * 32 + lrow;
    const uint32_t tok0 = blockIdx.y * kToks, last_tok = seq - 1;
    const uint8_t *wrow = w + static_cast<size_t>(min(row, rows - 1)) * nb * kBlockBytes;
    if constexpr (Iq<kQuant>::kTableBytes > 0) {
        const uint4 *src = static_cast<const uint4 *>(Iq<kQuant>::table());
        for (int i = tid; i < Iq<kQuant>::kTableBytes / 16; i += kGbThreads) reinterpret_cast<uint4 *>(s_table)[i] = src[i];
    }

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

    // K slice of this workgroup (blockIdx.z): blocks b0 .. b1, its sums go to the slice's own copy of the output
    const uint32_t b0 = blockIdx.z * nb_slice, b1 = min(nb, b0 + nb_slice);
    out += static_cast<size_t>(blockIdx.z) * seq * rows;
    Stage<kToks> st;
    stage_load<kToks>(st, aq, ad, tok0, last_tok, nb, b0, tid);
    IqRow<kQuant> cur;
    cur.load(wrow + static_cast<size_t>(b0) * kBlockBytes, khalf);
    stage_store<kToks>(st, s_a[0], s_dx[0], tid);
    __syncthreads();  // also: the table is in place

    for (uint32_t b = b0; b < b1; b++) {
        const int buf = (b - b0) & 1;
        const uint32_t bn = b + 1 < b1 ? b + 1 : b;  // the last step reloads its own block, unused
        stage_load<kToks>(st, aq, ad, tok0, last_tok, nb, bn, tid);
        IqRow<kQuant> nxt;
        nxt.load(wrow + static_cast<size_t>(bn) * kBlockBytes, khalf);
        const uint8_t *abase = s_a[buf] + lrow * kGbStride64 + 8 * khalf;

        // the empty asm and the scheduling barrier keep the sixteen sub-blocks a chain (a tree keeps 256 products alive)
#define RNB_IQ_SUB_BLOCK(SB)                                                                                           \
    {                                                                                                                  \
        int sc;                                                                                                        \
        const long bop = cur.template operand<SB>(khalf, s_table, &sc);                                                \
        _Pragma("unroll") for (int t = 0; t < kTT; t++) {                                                              \
            const long aop = *reinterpret_cast<const long *>(abase + 32 * t * kGbStride64 + 16 * SB);                  \
            const v16i acc = __builtin_amdgcn_mfma_i32_32x32x16_i8(aop, bop, zero16, 0, 0, 0);                         \
            _Pragma("unroll") for (int i = 0; i < 16; i++) {                                                           \
                tot[t][i] += mul24(acc[i], sc); /* |I| <= 16 * 127 * 127 */                                            \
                asm volatile("" : "+v"(tot[t][i]));                                                                    \
            }                                                                                                          \
        }                                                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                                             \
    }
        RNB_IQ_SUB_BLOCK(0)
        RNB_IQ_SUB_BLOCK(1)
        RNB_IQ_SUB_BLOCK(2)
        RNB_IQ_SUB_BLOCK(3)
        RNB_IQ_SUB_BLOCK(4)
        RNB_IQ_SUB_BLOCK(5)
        RNB_IQ_SUB_BLOCK(6)
        RNB_IQ_SUB_BLOCK(7)
        RNB_IQ_SUB_BLOCK(8)
        RNB_IQ_SUB_BLOCK(9)
        RNB_IQ_SUB_BLOCK(10)
        RNB_IQ_SUB_BLOCK(11)
        RNB_IQ_SUB_BLOCK(12)
        RNB_IQ_SUB_BLOCK(13)
        RNB_IQ_SUB_BLOCK(14)
        RNB_IQ_SUB_BLOCK(15)
#undef RNB_IQ_SUB_BLOCK

#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const float4 dx4 = reinterpret_cast<const float4 *>(s_dx[buf])[8 * t + 2 * j + khalf];
                const float dx[4] = {dx4.x, dx4.y, dx4.z, dx4.w};
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int r = 4 * j + i;
                    accf[t][r] += (cur.d * dx[i]) * static_cast<float>(tot[t][r]);
                    tot[t][r] = 0;
                }
            }
        stage_store<kToks>(st, s_a[buf ^ 1], s_dx[buf ^ 1], tid);
        cur = nxt;
        __syncthreads();
    }

    if (row < rows) {
#pragma unroll
        for (int t = 0; t < kTT; t++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t tok = tok0 + 32 * t + 8 * (r >> 2) + 4 * khalf + (r & 3);
                if (tok < seq) out[static_cast<size_t>(tok) * rows + row] = accf[t][r];
            }
    }
}

// the tiling and slicing choices, shared by the launcher and the workspace size
struct IqGemmPlan {
    bool wide;  // 64-token workgroups
    uint32_t slices;
};
IqGemmPlan iq_gemm_plan(uint32_t rows, uint32_t nb, uint32_t seq) {
    const uint64_t row_tiles = (rows + kGbRows - 1) / kGbRows;
    IqGemmPlan p;
    p.wide = seq > 32 && row_tiles * ((seq + 63) / 64) >= 512;  // the wider tile while it leaves two workgroups per compute unit
    const uint64_t wgs = row_tiles * (p.wide ? (seq + 63) / 64 : (seq + 31) / 32);
    p.slices = 1;
    if (wgs <= 256) {  // K slices until the grid has about 512 workgroups; a slice keeps four blocks, two on the smallest grids
        const uint64_t want = (512 + wgs - 1) / wgs, min_steps = wgs <= 32 ? 2 : 4;
        p.slices = static_cast<uint32_t>(std::max<uint64_t>(1, std::min<uint64_t>({want, nb / min_steps, 16})));
    }
    return p;
}

template <uint32_t kQuant>
void launch_iq_gemm(const uint8_t *w, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb, uint32_t seq,
                    hipStream_t stream) {
    const IqGemmPlan p = iq_gemm_plan(rows, nb, seq);
    const uint32_t slices = slice_out ? p.slices : 1;
    const uint32_t nb_slice = (nb + slices - 1) / slices, nz = (nb + nb_slice - 1) / nb_slice;
    float *dst = nz > 1 ? slice_out : out;
    const dim3 grid((rows + kGbRows - 1) / kGbRows, p.wide ? (seq + 63) / 64 : (seq + 31) / 32, nz), block(kGbThreads);
    if (p.wide)
        hipLaunchKernelGGL((gemm_iq_mfma_kernel<kQuant, 2>), grid, block, 0, stream, w, act.qs, act.d, dst, rows, nb, seq, nb_slice);
    else
        hipLaunchKernelGGL((gemm_iq_mfma_kernel<kQuant, 1>), grid, block, 0, stream, w, act.qs, act.d, dst, rows, nb, seq, nb_slice);
    if (nz > 1) launch_sum_slices(slice_out, out, static_cast<size_t>(seq) * rows, nz, stream);
}

}  // namespace

bool is_iq_quant(uint32_t quant) { return quant == kIQ2XXS || quant == kIQ2S || quant == kIQ3XXS || quant == kIQ4XS; }

void launch_gemv_iq(const uint8_t *w, uint32_t quant, ActView act, float *out, uint32_t rows, uint32_t nb, uint32_t seq,
                    hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    switch (quant) {
    case kIQ2XXS: launch_iq<kIQ2XXS>(w, act, out, rows, nb, seq, stream); break;
    case kIQ2S: launch_iq<kIQ2S>(w, act, out, rows, nb, seq, stream); break;
    case kIQ3XXS: launch_iq<kIQ3XXS>(w, act, out, rows, nb, seq, stream); break;
    default: launch_iq<kIQ4XS>(w, act, out, rows, nb, seq, stream); break;
    }
}

size_t gemm_iq_slice_floats(uint32_t rows, uint32_t nb, uint32_t seq) {
    if (rows == 0 || nb == 0 || seq == 0) return 0;
    const IqGemmPlan p = iq_gemm_plan(rows, nb, seq);
    return p.slices > 1 ? static_cast<size_t>(p.slices) * seq * rows : 0;
}

void launch_gemm_iq_mfma(const uint8_t *w, uint32_t quant, ActView act, float *out, float *slice_out, uint32_t rows, uint32_t nb,
                         uint32_t seq, hipStream_t stream) {
    if (rows == 0 || seq == 0 || nb == 0) return;
    switch (quant) {
    case kIQ2XXS: launch_iq_gemm<kIQ2XXS>(w, act, out, slice_out, rows, nb, seq, stream); break;
    case kIQ2S: launch_iq_gemm<kIQ2S>(w, act, out, slice_out, rows, nb, seq, stream); break;
    case kIQ3XXS: launch_iq_gemm<kIQ3XXS>(w, act, out, slice_out, rows, nb, seq, stream); break;
    default: launch_iq_gemm<kIQ4XS>(w, act, out, slice_out, rows, nb, seq, stream); break;
    }
}

void launch_embed_gather_iq(uint32_t quant, const uint8_t *w, size_t row_bytes, const uint32_t *ids, uint32_t n_tokens,
                            uint32_t cols, float *out, hipStream_t stream) {
    switch (quant) {
    case kIQ2XXS: launch_embed_gather_format<DqIQ2XXS>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kIQ2S: launch_embed_gather_format<DqIQ2S>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    case kIQ3XXS: launch_embed_gather_format<DqIQ3XXS>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    default: launch_embed_gather_format<DqIQ4XS>(w, row_bytes, ids, n_tokens, cols, out, stream); break;
    }
}

}  // namespace rnb
