// Per-lane partial dot products of one GGUF super-block against one Q8_K activation block, shared
// by the decode GEMV and the gathered-MoE kernels.  Eight lanes cooperate on a 256-element block;
// the caller adds the partials across lanes.
#pragma once

#include "device_utils.h"
#include "kernels.h"

namespace rnb {

// ---------------------------------------------------------------------------------------------
// Q4_K: block = {f16 d, f16 dmin, u8 scales[12], u8 qs[128]}.  Lane c (0..7) of a block group
// owns qs[16c .. 16c+16): group g = c/2 holds elements 64g + 16(c&1) + [0,16) in the low nibbles
// (scale 2g) and 64g + 32 + 16(c&1) + [0,16) in the high nibbles (scale 2g+1).  The mins term of
// sub-block c goes to lane c.
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ float q4k_block_partial(const uint8_t *__restrict__ blk, const int8_t *__restrict__ aq,
                                                   float dx, const int16_t *__restrict__ bs, int c) {
    const uint4 hdr = *reinterpret_cast<const uint4 *>(blk);
    const uint4 q = *reinterpret_cast<const uint4 *>(blk + 16 + 16 * c);
    const int g = c >> 1, half = c & 1;
    const uint4 a_lo = *reinterpret_cast<const uint4 *>(aq + 64 * g + 16 * half);
    const uint4 a_hi = *reinterpret_cast<const uint4 *>(aq + 64 * g + 32 + 16 * half);
    const uint32_t bs_pair = *reinterpret_cast<const uint32_t *>(bs + 2 * c);  // bsums[2c], bsums[2c+1]

    const float d = f16_bits_to_f32(hdr.x);
    const float dmin = f16_bits_to_f32(hdr.x >> 16);
    const Q4KScales s = unpack_q4k_scales(hdr.y, hdr.z, hdr.w);
    const int sc0 = byte_of(s.sc_lo, s.sc_hi, 2 * g);
    const int sc1 = byte_of(s.sc_lo, s.sc_hi, 2 * g + 1);
    const int mn = byte_of(s.mn_lo, s.mn_hi, c);

    int i0 = 0, i1 = 0;
    i0 = dot4(q.x & 0x0f0f0f0fu, a_lo.x, i0);
    i0 = dot4(q.y & 0x0f0f0f0fu, a_lo.y, i0);
    i0 = dot4(q.z & 0x0f0f0f0fu, a_lo.z, i0);
    i0 = dot4(q.w & 0x0f0f0f0fu, a_lo.w, i0);
    i1 = dot4((q.x >> 4) & 0x0f0f0f0fu, a_hi.x, i1);
    i1 = dot4((q.y >> 4) & 0x0f0f0f0fu, a_hi.y, i1);
    i1 = dot4((q.z >> 4) & 0x0f0f0f0fu, a_hi.z, i1);
    i1 = dot4((q.w >> 4) & 0x0f0f0f0fu, a_hi.w, i1);
    const int sumi = sc0 * i0 + sc1 * i1;
    const int bsum32 = static_cast<int>(static_cast<int16_t>(bs_pair & 0xffffu)) + (static_cast<int>(bs_pair) >> 16);
    const int summ = mn * bsum32;
    return dx * (d * static_cast<float>(sumi) - dmin * static_cast<float>(summ));
}

// ---------------------------------------------------------------------------------------------
// Q6_K: block = {u8 ql[128], u8 qh[64], i8 scales[16], f16 d}, 210 bytes, 2-byte aligned.
// Lane (n = half 0/1, t = 0..3) of a block group owns l = 8t .. 8t+7 of half n: 8 bytes of
// ql[64n + l], 8 of ql[64n + 32 + l], 8 of qh[32n + l] -> 32 six-bit values, four per activation
// quarter 128n + 32i + l.  (q - 32) is applied as  dot(q, a) - 32 * sum(a).
// ---------------------------------------------------------------------------------------------
__device__ __forceinline__ int sext8(uint32_t v, int shift) { return static_cast<int>(static_cast<int8_t>((v >> shift) & 0xffu)); }

__device__ __forceinline__ float q6k_block_partial(const uint8_t *__restrict__ blk, const int8_t *__restrict__ aq,
                                                   float dx, int sub) {
    const int n = sub >> 2, t = sub & 3;
    const uint2 A = ld_u2_a2(blk + 64 * n + 8 * t);
    const uint2 B = ld_u2_a2(blk + 64 * n + 32 + 8 * t);
    const uint2 H = ld_u2_a2(blk + 128 + 32 * n + 8 * t);
    const uint2 S = ld_u2_a2(blk + 192 + 8 * n);
    const float d = ld_f16(blk + 208);
    const int8_t *a = aq + 128 * n + 8 * t;
    const uint2 a0 = *reinterpret_cast<const uint2 *>(a);
    const uint2 a1 = *reinterpret_cast<const uint2 *>(a + 32);
    const uint2 a2 = *reinterpret_cast<const uint2 *>(a + 64);
    const uint2 a3 = *reinterpret_cast<const uint2 *>(a + 96);

    const int is = (t >> 1) * 8;  // l / 16 selects scale byte 0 or 1 of each pair
    const int s0 = sext8(S.x, is), s1 = sext8(S.x, is + 16), s2 = sext8(S.y, is), s3 = sext8(S.y, is + 16);

    int p0 = 0, p1 = 0, p2 = 0, p3 = 0;
#define RNB_Q6_STEP(Ak, Bk, Hk, a0k, a1k, a2k, a3k)                                   \
    {                                                                                 \
        const uint32_t u0 = ((Ak) & 0x0f0f0f0fu) | (((Hk) & 0x03030303u) << 4);       \
        const uint32_t u1 = ((Bk) & 0x0f0f0f0fu) | (((Hk) & 0x0c0c0c0cu) << 2);       \
        const uint32_t u2 = (((Ak) >> 4) & 0x0f0f0f0fu) | ((Hk) & 0x30303030u);       \
        const uint32_t u3 = (((Bk) >> 4) & 0x0f0f0f0fu) | (((Hk) & 0xc0c0c0c0u) >> 2); \
        p0 = dot4(u0, a0k, p0) - dot4(0x20202020u, a0k, 0);                           \
        p1 = dot4(u1, a1k, p1) - dot4(0x20202020u, a1k, 0);                           \
        p2 = dot4(u2, a2k, p2) - dot4(0x20202020u, a2k, 0);                           \
        p3 = dot4(u3, a3k, p3) - dot4(0x20202020u, a3k, 0);                           \
    }
    RNB_Q6_STEP(A.x, B.x, H.x, a0.x, a1.x, a2.x, a3.x)
    RNB_Q6_STEP(A.y, B.y, H.y, a0.y, a1.y, a2.y, a3.y)
#undef RNB_Q6_STEP
    const int sumi = s0 * p0 + s1 * p1 + s2 * p2 + s3 * p3;
    return (d * dx) * static_cast<float>(sumi);
}

}  // namespace rnb
